"""TEST INFRASTRUCTURE ONLY: the reference's PyTorch step loops, restated.

These are differentiable step-by-step PyTorch versions of the three operators,
taking the operators' own ``[N,H,L,*]`` tensors.  Autograd through them is the
gradient the reference's self tests compare its kernels with, and their run
time on the host is the reference's CPU path.

  delta rule           algorithmic/fast_weight/__init__.py:178-187
  Delta RNN v2         algorithmic/fast_weight_rnn_v2/__init__.py:205-217
  Recurrent Delta Net  algorithmic/rec_update_fwm_tanh/__init__.py:263-302
  sum rule             algorithmic/fast_transformers/__init__.py:145-152
  Delta LSTM v4        language_modeling/src/utils/fast_lstm_v4/__init__.py:397-432

The state is kept as ``W[N,H,E,M]`` (the operators' layout) instead of the
reference loop's transposed ``[N*H,M,E]``; the arithmetic per step is the same.
"""
import torch


def _read(W, x):
    """W^T x : [N,H,E,M],[N,H,E] -> [N,H,M]."""
    return torch.matmul(x.unsqueeze(-2), W).squeeze(-2)


def _write(W, k, v, beta):
    """One delta-rule write; returns the new state."""
    v_old = _read(W, k)
    u = beta * (v - v_old)
    return W + k.unsqueeze(-1) * u.unsqueeze(-2)


def delta_loop(q, k, v, beta, W0):
    """-> (out[N,H,L,M], W_L)."""
    W = W0
    outs = []
    for t in range(q.shape[2]):
        W = _write(W, k[:, :, t], v[:, :, t], beta[:, :, t])
        outs.append(_read(W, q[:, :, t]))
    return torch.stack(outs, dim=2), W


def sum_loop(q, k, v, W0):
    """Sum update rule (algorithmic/fast_transformers/__init__.py:149-152). -> (out, W_L)."""
    W = W0
    outs = []
    for t in range(q.shape[2]):
        W = W + k[:, :, t].unsqueeze(-1) * v[:, :, t].unsqueeze(-2)
        outs.append(_read(W, q[:, :, t]))
    return torch.stack(outs, dim=2), W


def rnn_v2_loop(z, k, v, W0, beta, h0):
    """Argument order of the reference op. -> (out[N,H,L,D], W_L, h_L[N,H,1,D])."""
    W = W0
    h = h0[:, :, 0]
    outs = []
    for t in range(z.shape[2]):
        s = torch.softmax(h, dim=-1)
        W = _write(W, k[:, :, t], v[:, :, t], beta[:, :, t])
        h = _read(W, s) + z[:, :, t]
        outs.append(h)
    return torch.stack(outs, dim=2), W, h.unsqueeze(2)


def lstm_v4_loop(zi, ki, vi, bi, Wi, zu, ku, vu, bu, Wu, zo, ko, vo, bo, Wo, h0, c0):
    """Argument order of the reference op. -> (out, cell_out, (W_i, W_u, W_o), h_L, c_L)."""
    h, c = h0[:, :, 0], c0[:, :, 0]
    outs, cells = [], []
    for t in range(zi.shape[2]):
        Wi = _write(Wi, ki[:, :, t], vi[:, :, t], bi[:, :, t])
        Wu = _write(Wu, ku[:, :, t], vu[:, :, t], bu[:, :, t])
        Wo = _write(Wo, ko[:, :, t], vo[:, :, t], bo[:, :, t])
        s = torch.softmax(h, dim=-1)
        gate_i = torch.sigmoid(_read(Wi, s) + zi[:, :, t])
        upd = _read(Wu, s) + zu[:, :, t]
        gate_o = torch.sigmoid(_read(Wo, s) + zo[:, :, t])
        c = gate_i * upd + (1.0 - gate_i) * c
        h = c * gate_o
        outs.append(h)
        cells.append(c)
    return torch.stack(outs, dim=2), torch.stack(cells, dim=2), (Wi, Wu, Wo), h.unsqueeze(2), c.unsqueeze(2)


def rec_update_loop(qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0):
    """-> (out[N,H,L,D], W_L, h_L[N,H,1,D]); R_* [1,H,D,D], r_b [1,H,1,D]."""
    W = W0
    h = h0[:, :, 0]
    Rq, Rk, Rv, rb = R_q[0], R_k[0], R_v[0], r_b[0, :, 0]
    outs = []
    for t in range(qx.shape[2]):
        y = torch.tanh(h)                                   # [N,H,D]
        yr = y.unsqueeze(-2)                                # [N,H,1,D]
        q = torch.softmax(qx[:, :, t] + torch.matmul(yr, Rq).squeeze(-2), dim=-1)
        k = torch.softmax(kx[:, :, t] + torch.matmul(yr, Rk).squeeze(-2), dim=-1)
        v = vx[:, :, t] + torch.matmul(yr, Rv).squeeze(-2)
        b = torch.sigmoid(bx[:, :, t] + (y * rb).sum(-1, keepdim=True))
        W = _write(W, k, v, b)
        h = _read(W, q)
        outs.append(h)
    return torch.stack(outs, dim=2), W, h.unsqueeze(2)


def grads(loop, inputs, diff_idx, grad_out):
    """Run ``loop(*inputs)`` with ``requires_grad`` on inputs[diff_idx] and
    return (out, [grads...]) for upstream gradient ``grad_out`` on the output."""
    xs = [x.detach().clone() for x in inputs]
    for i in diff_idx:
        xs[i].requires_grad_(True)
    out = loop(*xs)[0]
    out.backward(grad_out)
    return out.detach(), [xs[i].grad for i in diff_idx]
