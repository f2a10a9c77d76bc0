"""Head sizes between the ones the register kernels of the recurrent operators take (16 and 32).

Those operators read their state with a softmax over the fed-back vector, so zero padding alone would
change the result: a padded entry would take its share exp(0) of the softmax.  What makes the padded
problem equal to the narrow one is a padded softmax input of -BIG: its exponential is exactly zero, the
padded entry of the softmax is exactly zero, and every padded row and column of the state stays zero
(padded keys and values are zero).  BIG is finite and small enough that products of two such entries stay
finite, so that nothing in the backward pass turns into 0 * inf.
"""
import torch

WIDTHS = (16, 32)
BIG = 1.0e9
_pad = torch.nn.functional.pad


def padded_width(D):
    """The width a head size of D runs at, or None when it runs as it is (the kernels take it, or it is
    wider than any of them and goes to the kernels that keep the state in LDS)."""
    if D in WIDTHS:
        return None
    return next((w for w in WIDTHS if w > D), None)


def last(t, n, value=0.0):
    """t with n more entries of `value` along its last axis."""
    return _pad(t, (0, n), value=value)


def square(t, n):
    """t [..., D, D] with n more rows and columns of zeros."""
    return _pad(t, (0, n, 0, n))


def state_ok(t, shape):
    return t.shape == shape and t.is_contiguous() and t.dtype == torch.float32
