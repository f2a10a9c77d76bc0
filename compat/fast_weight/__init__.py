"""``fast_weight``: the reference's module of this name (algorithmic/fast_weight/__init__.py), served by the
MI355X implementation: delta-rule fast weight memory.  Imported as ``from fast_weight import fast_weight_delta``
(algorithmic/layers.py:7-10)."""
from _fwp_dropin import package as _package

DeltaFastWeight = _package().DeltaFastWeight
fast_weight_delta = _package().fast_weight_delta

__all__ = ["DeltaFastWeight", "fast_weight_delta"]
