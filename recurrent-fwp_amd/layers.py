"""The caller of ``fast_weight_delta`` in language modelling: the Delta-Net layer and the
feed-forward block that follows it, with the module and parameter names of the reference
(language_modeling/src/utils/cuda_fast_weight_layer.py:57-188, utils/model_utils.py:15-67)
so a reference state_dict loads unchanged.  The fast-weight operator and, on the GPU, the
elementwise lines in front of it are HIP kernels; the rest is stock PyTorch.  A caller may pass
another operator (tests do, to compare against a step-by-step loop); the layer then also takes
the stock-PyTorch form of those lines.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib
from .fast_weight import fast_weight_delta


class PositionalEmbedding(nn.Module):
    """Sinusoidal embedding of a position sequence: ``[sin | cos]`` halves, shape
    ``[len, 1, demb]`` (or ``[len, bsz, demb]``).  utils/model_utils.py:15-31."""

    def __init__(self, demb):
        super().__init__()
        self.demb = demb
        self.register_buffer("inv_freq", 10000.0 ** (-torch.arange(0.0, demb, 2.0) / demb))

    def forward(self, pos_seq, bsz=None):
        phase = pos_seq[:, None] * self.inv_freq[None, :]
        emb = torch.cat((phase.sin(), phase.cos()), dim=-1).unsqueeze(1)
        return emb if bsz is None else emb.expand(-1, bsz, -1)


class PositionwiseFF(nn.Module):
    """Linear-ReLU-Linear with residual and LayerNorm (after, or before when
    ``pre_lnorm``).  utils/model_utils.py:34-67.  The reference's ReLU works in place; on a
    ``[len, bsz, d_inner]`` input that is a view of the projection's 2-D result, and autograd then
    rebuilds the base tensor in backward (three copies and a clone of the widest activation per
    layer, 4 % of the language model's step): not in place here."""

    def __init__(self, d_model, d_inner, dropout, pre_lnorm=False):
        super().__init__()
        self.d_model, self.d_inner, self.dropout, self.pre_lnorm = d_model, d_inner, dropout, pre_lnorm
        self.CoreNet = nn.Sequential(
            nn.Linear(d_model, d_inner), nn.ReLU(), nn.Dropout(dropout),
            nn.Linear(d_inner, d_model), nn.Dropout(dropout))
        self.layer_norm = nn.LayerNorm(d_model)

    def forward(self, inp):
        if self.pre_lnorm:
            return inp + self.CoreNet(self.layer_norm(inp))
        return self.layer_norm(inp + self.CoreNet(inp))


def sum_normalised_elu(x):
    """``phi(x) = (elu(x) + 1) / sum_D(elu(x) + 1)``: positive features that sum to one
    (cuda_fast_weight_layer.py:118-123)."""
    x = F.elu(x) + 1.0
    return x / x.sum(-1, keepdim=True)


class DeltaNetPrep(torch.autograd.Function):
    """``q, k, v, beta = DeltaNetPrep.apply(qkvb, n_head, d_head[, q_scale])``: the lines between the layer's
    projection and the operator (cuda_fast_weight_layer.py:108-125) as one HIP kernel each way.
    ``qkvb`` is the contiguous ``[len, bsz, n_head * (3 d_head + 1)]`` projection; the results are
    contiguous ``[bsz, n_head, len, .]``: q, k through :func:`sum_normalised_elu`, v copied, beta
    through a sigmoid.  ``q_scale`` multiplies q: the operator's output is linear in q, so the
    ``1/sqrt(d_head)`` the layer applies to that output (:155-157) can ride here for free."""

    @staticmethod
    def supported(qkvb, d_head):
        return (qkvb.is_cuda and qkvb.dtype == torch.float32 and qkvb.is_contiguous()
                and d_head in (16, 32, 64))

    @staticmethod
    def forward(ctx, qkvb, n_head, d_head, q_scale=1.0):
        _lib.require_device(qkvb)
        T, B, _ = qkvb.shape
        H, D = n_head, d_head
        f32 = dict(device=qkvb.device, dtype=torch.float32)
        q, k, v = (torch.empty((B, H, T, D), **f32) for _ in range(3))
        beta = torch.empty((B, H, T, 1), **f32)
        with _lib.on_device(qkvb):
            rc = _lib.lib().fwp_deltanet_prep_fwd(qkvb.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                                  beta.data_ptr(), T, B, H, D, float(q_scale),
                                                  _lib.stream_of(qkvb))
        _lib.check(rc, "fwp_deltanet_prep_fwd")
        ctx.save_for_backward(qkvb)
        ctx.dims = (T, B, H, D, float(q_scale))
        return q, k, v, beta

    @staticmethod
    def backward(ctx, gq, gk, gv, gbeta):
        (qkvb,) = ctx.saved_tensors
        T, B, H, D, q_scale = ctx.dims
        gq, gk, gv, gbeta = (g.contiguous() for g in (gq, gk, gv, gbeta))
        gqkvb = torch.empty_like(qkvb)
        with _lib.on_device(qkvb):
            rc = _lib.lib().fwp_deltanet_prep_bwd(qkvb.data_ptr(), gq.data_ptr(), gk.data_ptr(), gv.data_ptr(),
                                                  gbeta.data_ptr(), gqkvb.data_ptr(), T, B, H, D, q_scale,
                                                  _lib.stream_of(qkvb))
        _lib.check(rc, "fwp_deltanet_prep_bwd")
        return gqkvb, None, None, None


class DeltaNetLayer(nn.Module):
    """Delta-rule linear-Transformer layer (the reference's
    ``CudaFastWeightLinearTransformerLayer`` with its default
    ``skip_attn_normalization=True``).

    ``h`` is ``[len, bsz, d_model]``.  One projection gives q, k, v and a scalar
    write strength per head; q and k go through :func:`sum_normalised_elu`, beta
    through a sigmoid, and the fast weight memory ``W[bsz, n_head, D, D]`` (zero, or
    ``mems[0]`` when a segment's state is carried over) is updated step by step by
    ``fast_weight_delta``.  The read-out is scaled by ``1/sqrt(D)``, projected, and
    added to the input with LayerNorm.  With ``carry_over_fast_weight`` the call
    returns ``(output, (W_final, None))``.
    """

    def __init__(self, n_head, d_model, d_head, dropout=0.0, dropatt=0.0, pre_lnorm=False,
                 layer_id=None, num_layer=None, fast_weight_op=None):
        super().__init__()
        self.n_head, self.d_model, self.d_head, self.dropout = n_head, d_model, d_head, dropout
        self.layer_id, self.num_layer = layer_id, num_layer
        self.qkvb_net = nn.Linear(d_model, n_head * (3 * d_head + 1), bias=False)
        self.drop = nn.Dropout(dropout)
        self.dropatt = nn.Dropout(dropatt)
        self.o_net = nn.Linear(n_head * d_head, d_model, bias=False)
        self.layer_norm = nn.LayerNorm(d_model)
        self.scale = 1.0 / d_head ** 0.5
        self.pre_lnorm = pre_lnorm
        self.fast_weight_op = fast_weight_op or fast_weight_delta

    def forward(self, h, attn_mask=None, mems=None, carry_over_fast_weight=False):
        slen, bsz, _ = h.shape
        H, D = self.n_head, self.d_head
        x = self.layer_norm(h) if self.pre_lnorm else h
        # The reference's pre-LN branch adds the normalised input back (it rebinds h, :100-104).
        residual = x

        qkvb = self.qkvb_net(x)
        hip_op = self.fast_weight_op is fast_weight_delta
        fused = hip_op and DeltaNetPrep.supported(qkvb, D)
        if fused:
            # one fused kernel each way; q carries the 1/sqrt(D) of the read-out (the operator is
            # linear in q), and the operator writes [len, bsz, H, D] storage: no pass over its output
            q, k, v, beta = DeltaNetPrep.apply(qkvb, H, D, self.scale)
        else:
            qkvb = qkvb.view(slen, bsz, H, 3 * D + 1)
            q, k, v, beta = (t.permute(1, 2, 0, 3) for t in qkvb.split((D, D, D, 1), dim=-1))
            q, k, beta = sum_normalised_elu(q), sum_normalised_elu(k), torch.sigmoid(beta)

        if hip_op and q.dtype != torch.float32:
            # half or bf16 activations (autocast): the operator and its state are fp32, as the
            # reference's kernel and its torch.zeros state are
            q, k, v, beta = q.float(), k.float(), v.float(), beta.float()
        if mems is None:
            W = torch.zeros(bsz, H, D, D, device=h.device, dtype=torch.float32 if hip_op else q.dtype)
        else:
            if not carry_over_fast_weight:
                raise ValueError("mems are only meaningful with carry_over_fast_weight=True")
            # The last batch of an epoch may be smaller than the carried state.  The
            # operator overwrites its state argument, so it gets storage of its own.
            W = mems[0][:bsz].clone()

        if fused:
            out = fast_weight_delta(q, k, v, beta, W, True)          # [bsz, H, slen, D] over [slen, bsz, H, D] storage
            out = out.permute(2, 0, 1, 3).reshape(slen, bsz, H * D)  # a view
        else:
            out = self.fast_weight_op(q, k, v, beta, W)              # [bsz, H, slen, D]
            out = (self.scale * out).permute(2, 0, 1, 3).reshape(slen, bsz, H * D).to(x.dtype)
        out = residual + self.drop(self.o_net(out))
        if not self.pre_lnorm:
            out = self.layer_norm(out)
        if carry_over_fast_weight:
            return out, (W.detach(), None)
        return out


class DeltaNetDecoderLayer(nn.Module):
    """Delta-Net layer followed by the feed-forward block (``DecoderLayer`` with
    ``attn_type=24``, model_main.py:703-775); sub-module names ``dec_attn`` and
    ``pos_ff`` as there."""

    def __init__(self, n_head, d_model, d_head, d_inner, dropout=0.0, dropatt=0.0, pre_lnorm=False,
                 layer_id=None, num_layer=None, fast_weight_op=None):
        super().__init__()
        self.dec_attn = DeltaNetLayer(n_head, d_model, d_head, dropout, dropatt, pre_lnorm,
                                      layer_id, num_layer, fast_weight_op)
        self.pos_ff = PositionwiseFF(d_model, d_inner, dropout, pre_lnorm)

    def forward(self, dec_inp, dec_attn_mask=None, mems=None, carry_over_fast_weight=False):
        out = self.dec_attn(dec_inp, attn_mask=dec_attn_mask, mems=mems,
                            carry_over_fast_weight=carry_over_fast_weight)
        if carry_over_fast_weight:
            out, new_mem = out
            return self.pos_ff(out), new_mem
        return self.pos_ff(out)
