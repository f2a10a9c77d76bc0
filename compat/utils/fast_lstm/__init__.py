"""``utils.fast_lstm``: present so that ``from utils.fast_lstm import fast_lstm`` (language_modeling/src/utils/cuda_fast_weight_layer.py:9-23) resolves.
This earlier variant of the operator (language_modeling/src/utils/fast_lstm/__init__.py) is not part of the MI355X
implementation; calling it raises.  Its successor is fast_lstm_v4 (utils.fast_lstm_v4)."""


def fast_lstm(*args, **kwargs):
    raise NotImplementedError("fast_lstm has no MI355X implementation; use fast_lstm_v4 (utils.fast_lstm_v4)")


class FastLSTM:
    apply = staticmethod(fast_lstm)


__all__ = ["FastLSTM", "fast_lstm"]
