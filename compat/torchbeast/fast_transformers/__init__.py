"""``torchbeast.fast_transformers``: the reference's module of this name (reinforcement_learning/torchbeast/fast_transformers/__init__.py), served by the
MI355X implementation: sum update rule (causal linear attention).  Imported as ``from torchbeast.fast_transformers import fast_weight_sum``
(reinforcement_learning/torchbeast/layer.py:7-10)."""
from _fwp_dropin import package as _package

FastWeightSum = _package().FastWeightSum
fast_weight_sum = _package().fast_weight_sum

__all__ = ["FastWeightSum", "fast_weight_sum"]
