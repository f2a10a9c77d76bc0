"""Minimal Delta-Net language model: the part of the reference's ``MemTransformerLM`` that
the Delta-Net configuration uses (language_modeling/src/model_main.py:1178-1207, absolute
positions :1267-1303, loss :1333-1361): scaled word embedding + sinusoidal positions,
a stack of Delta-Net decoder layers, tied softmax with per-token negative log-likelihood.
No adaptive softmax, no attention memory: the fast weights are the only state carried
from one segment to the next.  Parameter names follow the reference
(``word_emb.emb_layers.0.weight``, ``layers.N.dec_attn.qkvb_net.weight``,
``crit.out_layers.0.bias`` ...).
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from .layers import DeltaNetDecoderLayer, PositionalEmbedding


class _WordEmbedding(nn.Module):
    """One embedding table, output scaled by sqrt(d_model) (AdaptiveEmbedding with
    ``div_val=1`` and no cut-offs, model_main.py:836-898)."""

    def __init__(self, n_token, d_model):
        super().__init__()
        self.emb_scale = d_model ** 0.5
        self.emb_layers = nn.ModuleList([nn.Embedding(n_token, d_model)])

    def forward(self, inp):
        return self.emb_layers[0](inp) * self.emb_scale


class _TiedSoftmaxLoss(nn.Module):
    """Per-token negative log-likelihood under ``softmax(hidden @ E^T + b)``
    (ProjectedAdaptiveLogSoftmax without clusters)."""

    def __init__(self, n_token, d_model):
        super().__init__()
        self.out_layers = nn.ModuleList([nn.Linear(d_model, n_token)])

    def forward(self, hidden, target):
        return F.cross_entropy(self.out_layers[0](hidden), target, reduction="none")


class DeltaNetLM(nn.Module):
    """``forward(data, target, *mems, carry_over_fast_weight=False)`` with ``data`` and
    ``target`` of shape ``[len, bsz]`` (int64) returns ``[loss]`` or, when the fast
    weights are carried, ``[loss, mem_0, ..., mem_{n_layer-1}]``; ``loss`` is
    ``[len, bsz]`` and each ``mem_i`` is the pair ``(W[bsz,H,D,D], None)`` the layers take.
    """

    def __init__(self, n_token, n_layer, n_head, d_model, d_head, d_inner, dropout=0.0,
                 dropatt=0.0, pre_lnorm=False, tie_weight=True, clamp_len=-1, init_std=0.02,
                 fast_weight_op=None):
        super().__init__()
        self.n_token, self.n_layer, self.d_model, self.clamp_len = n_token, n_layer, d_model, clamp_len
        self.word_emb = _WordEmbedding(n_token, d_model)
        self.pos_emb = PositionalEmbedding(d_model)
        self.drop = nn.Dropout(dropout)
        self.layers = nn.ModuleList([
            DeltaNetDecoderLayer(n_head, d_model, d_head, d_inner, dropout, dropatt, pre_lnorm,
                                 layer_id=i, num_layer=n_layer, fast_weight_op=fast_weight_op)
            for i in range(n_layer)])
        self.crit = _TiedSoftmaxLoss(n_token, d_model)
        self.reset_parameters(init_std)
        if tie_weight:
            self.crit.out_layers[0].weight = self.word_emb.emb_layers[0].weight

    def reset_parameters(self, std):
        """N(0, std) weights, zero biases, LayerNorm gains N(1, std) (train.py:378-432)."""
        for m in self.modules():
            if isinstance(m, (nn.Linear, nn.Embedding)):
                nn.init.normal_(m.weight, 0.0, std)
                if getattr(m, "bias", None) is not None:
                    nn.init.zeros_(m.bias)
            elif isinstance(m, nn.LayerNorm):
                nn.init.normal_(m.weight, 1.0, std)
                nn.init.zeros_(m.bias)

    def hidden(self, data, mems=None, carry_over_fast_weight=False):
        qlen = data.shape[0]
        emb = self.word_emb(data)
        # Positions count down to zero at the newest token (model_main.py:1273-1280).
        pos_seq = torch.arange(qlen - 1, -1, -1.0, device=emb.device, dtype=emb.dtype)
        if self.clamp_len > 0:
            pos_seq.clamp_(max=self.clamp_len)
        out = self.drop(emb + self.pos_emb(pos_seq))
        new_mems = []
        for i, layer in enumerate(self.layers):
            out = layer(out, mems=None if mems is None else mems[i],
                        carry_over_fast_weight=carry_over_fast_weight)
            if carry_over_fast_weight:
                out, mem = out
                new_mems.append(mem)
        return self.drop(out), (new_mems if carry_over_fast_weight else None)

    def forward(self, data, target, *mems, carry_over_fast_weight=False):
        hid, new_mems = self.hidden(data, mems or None, carry_over_fast_weight)
        tgt_len = target.shape[0]
        hid = hid[-tgt_len:]
        loss = self.crit(hid.reshape(-1, hid.shape[-1]), target.reshape(-1)).view(tgt_len, -1)
        return [loss] if new_mems is None else [loss] + new_mems
