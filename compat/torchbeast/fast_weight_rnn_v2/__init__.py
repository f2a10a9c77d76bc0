"""``torchbeast.fast_weight_rnn_v2``: the reference's module of this name (reinforcement_learning/torchbeast/fast_weight_rnn_v2/__init__.py), served by the
MI355X implementation: Delta RNN v2.  Imported as ``from torchbeast.fast_weight_rnn_v2 import fast_rnn_v2``
(reinforcement_learning/torchbeast/layer.py:7-10)."""
from _fwp_dropin import package as _package

FastRNNv2 = _package().FastRNNv2
fast_rnn_v2 = _package().fast_rnn_v2

__all__ = ["FastRNNv2", "fast_rnn_v2"]
