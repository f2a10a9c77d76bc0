"""``utils.fast_transformers``: the reference's module of this name (language_modeling/src/utils/fast_transformers/__init__.py), served by the
MI355X implementation: sum update rule (causal linear attention).  Imported as ``from utils.fast_transformers import fast_weight_sum``
(language_modeling/src/utils/cuda_fast_weight_layer.py:9-23)."""
from _fwp_dropin import package as _package

FastWeightSum = _package().FastWeightSum
fast_weight_sum = _package().fast_weight_sum

__all__ = ["FastWeightSum", "fast_weight_sum"]
