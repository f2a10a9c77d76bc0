"""MI355X-native fast-weight update operators with the Python API of
IDSIA/recurrent-fwp: ``fast_weight_delta``, ``rec_update_fwm_tanh``,
``fast_rnn_v2`` and the sum-rule baseline ``fast_weight_sum`` (argument order, ``[N,H,L,D]`` shapes, returned gradients and
in/out state tensors as in the reference's ``autograd.Function``s).  The
arithmetic runs in hand-written HIP kernels for gfx950 reached through the C ABI
of ``libfwp_hip.so``; there is no other implementation behind these names.
"""
from . import _lib
from .fast_weight import DeltaFastWeight, fast_weight_delta
from .fast_transformers import FastWeightSum, fast_weight_sum
from .fast_lstm_v4 import FastLSTMv4, fast_lstm_v4
from .fast_weight_rnn_v2 import FastRNNv2, fast_rnn_v2
from .rec_update_fwm_tanh import FastWeightRecUpdateTanh, rec_update_fwm_tanh
from .layers import DeltaNetDecoderLayer, DeltaNetLayer, DeltaNetPrep, PositionalEmbedding, PositionwiseFF
from .lm import DeltaNetLM

__all__ = ["DeltaFastWeight", "fast_weight_delta", "FastWeightSum", "fast_weight_sum", "FastRNNv2", "fast_rnn_v2",
           "FastLSTMv4", "fast_lstm_v4",
           "FastWeightRecUpdateTanh", "rec_update_fwm_tanh", "DeltaNetLayer", "DeltaNetPrep",
           "DeltaNetDecoderLayer", "PositionwiseFF", "PositionalEmbedding", "DeltaNetLM"]
