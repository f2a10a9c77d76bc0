"""``utils.fast_lstm_v2``: present so that ``from utils.fast_lstm_v2 import fast_lstm_v2`` (language_modeling/src/utils/cuda_fast_weight_layer.py:9-23) resolves.
This earlier variant of the operator (language_modeling/src/utils/fast_lstm_v2/__init__.py) is not part of the MI355X
implementation; calling it raises.  Its successor is fast_lstm_v4 (utils.fast_lstm_v4)."""


def fast_lstm_v2(*args, **kwargs):
    raise NotImplementedError("fast_lstm_v2 has no MI355X implementation; use fast_lstm_v4 (utils.fast_lstm_v4)")


class FastLSTMv2:
    apply = staticmethod(fast_lstm_v2)


__all__ = ["FastLSTMv2", "fast_lstm_v2"]
