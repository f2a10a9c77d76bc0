"""``utils.fast_fast_weight``: the reference's module of this name (language_modeling/src/utils/fast_fast_weight/__init__.py), served by the
MI355X implementation: delta-rule fast weight memory.  Imported as ``from utils.fast_fast_weight import fast_weight_delta``
(language_modeling/src/utils/cuda_fast_weight_layer.py:9-23)."""
from _fwp_dropin import package as _package

DeltaFastWeight = _package().DeltaFastWeight
fast_weight_delta = _package().fast_weight_delta

__all__ = ["DeltaFastWeight", "fast_weight_delta"]
