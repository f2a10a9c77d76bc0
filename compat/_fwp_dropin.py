"""Where the shim modules of this directory find the MI355X implementation.

This directory holds one module for every module path under which the reference's code imports
the fast-weight operators (``fast_weight``, ``utils.fast_fast_weight``, ``torchbeast.fast_weight``,
...).  Put it FIRST on ``sys.path`` and those import lines resolve to the HIP operators with no
edit of the reference's files::

    sys.path.insert(0, "/path/to/this/repo/compat")        # or:  python compat/run.py train.py ...

``utils`` and ``torchbeast`` have no ``__init__.py`` here, as in the reference: they are namespace
packages, so the reference's other modules of those names (``utils.performer_helper``,
``torchbeast.core`` ...) are still found in the reference's own directories, while the operator
modules, which exist in both places, are taken from the directory that comes first.
"""
import importlib
import os
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_PACKAGE = "recurrent-fwp_amd"          # not an identifier, hence importlib
_pkg = None


def package():
    global _pkg
    if _pkg is None:
        if _ROOT not in sys.path:
            sys.path.append(_ROOT)
        _pkg = importlib.import_module(_PACKAGE)
    return _pkg
