"""``utils.fast_lstm_v4``: the reference's module of this name (language_modeling/src/utils/fast_lstm_v4/__init__.py), served by the
MI355X implementation: Delta LSTM v4.  Imported as ``from utils.fast_lstm_v4 import fast_lstm_v4``
(language_modeling/src/utils/cuda_fast_weight_layer.py:9-23)."""
from _fwp_dropin import package as _package

FastLSTMv4 = _package().FastLSTMv4
fast_lstm_v4 = _package().fast_lstm_v4

__all__ = ["FastLSTMv4", "fast_lstm_v4"]
