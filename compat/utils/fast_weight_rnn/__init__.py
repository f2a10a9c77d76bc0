"""``utils.fast_weight_rnn``: present so that ``from utils.fast_weight_rnn import fast_rnn`` (language_modeling/src/utils/cuda_fast_weight_layer.py:9-23) resolves.
This earlier variant of the operator (language_modeling/src/utils/fast_weight_rnn/__init__.py) is not part of the MI355X
implementation; calling it raises.  Its successor is fast_rnn_v2 (utils.fast_weight_rnn_v2)."""


def fast_rnn(*args, **kwargs):
    raise NotImplementedError("fast_rnn has no MI355X implementation; use fast_rnn_v2 (utils.fast_weight_rnn_v2)")


class FastRNN:
    apply = staticmethod(fast_rnn)


__all__ = ["FastRNN", "fast_rnn"]
