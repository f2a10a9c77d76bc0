"""``fast_transformers``: the reference's module of this name (algorithmic/fast_transformers/__init__.py), served by the
MI355X implementation: sum update rule (causal linear attention).  Imported as ``from fast_transformers import fast_weight_sum``
(algorithmic/layers.py:7-10)."""
from _fwp_dropin import package as _package

FastWeightSum = _package().FastWeightSum
fast_weight_sum = _package().fast_weight_sum

__all__ = ["FastWeightSum", "fast_weight_sum"]
