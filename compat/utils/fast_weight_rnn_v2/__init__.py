"""``utils.fast_weight_rnn_v2``: the reference's module of this name (language_modeling/src/utils/fast_weight_rnn_v2/__init__.py), served by the
MI355X implementation: Delta RNN v2.  Imported as ``from utils.fast_weight_rnn_v2 import fast_rnn_v2``
(language_modeling/src/utils/cuda_fast_weight_layer.py:9-23)."""
from _fwp_dropin import package as _package

FastRNNv2 = _package().FastRNNv2
fast_rnn_v2 = _package().fast_rnn_v2

__all__ = ["FastRNNv2", "fast_rnn_v2"]
