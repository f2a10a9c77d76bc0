"""Delta-Net layer and minimal language model (the callers of ``fast_weight_delta``).

CPU part: the layer's plumbing (projection split, feature map, head layout, scaling,
residual + LayerNorm, carried state) with the step-by-step float64 loop as operator,
against a per-(batch, head) numpy restatement built on the C oracle, plus causality and
segment splitting.  GPU part: the same modules with the HIP operator against themselves
with the loop operator: outputs, losses and every parameter gradient.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle.torch_loop import delta_loop

ATOL, RTOL = 1e-4, 1e-3


def loop_op(q, k, v, beta, W):
    """The operator contract (state updated in place) on the differentiable loop."""
    out, W_end = delta_loop(q, k, v, beta, W.clone())
    W.copy_(W_end.detach())
    return out


def layer_numpy(layer, h, W0=None):
    """[len, bsz, d_model] -> (output, W_end), one (batch, head) sequence at a time."""
    p = {k: v.detach().double().numpy() for k, v in layer.state_dict().items()}
    T, B, dm = h.shape
    H, D = layer.n_head, layer.d_head
    x = h
    if layer.pre_lnorm:
        x = layer_norm_numpy(h, p["layer_norm.weight"], p["layer_norm.bias"])
    proj = x @ p["qkvb_net.weight"].T                       # [T, B, H*(3D+1)]
    read = np.zeros((T, B, H * D))
    W_end = np.zeros((B, H, D, D))
    for b in range(B):
        for hd in range(H):
            blk = proj[:, b, hd * (3 * D + 1):(hd + 1) * (3 * D + 1)]
            q, k, v, beta = blk[:, :D], blk[:, D:2 * D], blk[:, 2 * D:3 * D], blk[:, 3 * D:]
            phi = lambda a: np.where(a > 0, a + 1.0, np.exp(np.minimum(a, 0.0)))
            q, k = phi(q), phi(k)
            q, k = q / q.sum(-1, keepdims=True), k / k.sum(-1, keepdims=True)
            beta = 1.0 / (1.0 + np.exp(-beta))
            w0 = np.zeros((1, 1, D, D)) if W0 is None else W0[b:b + 1, hd:hd + 1]
            out, w = oracle.delta_fwd(q[None, None], k[None, None], v[None, None], beta[None, None], w0)
            read[:, b, hd * D:(hd + 1) * D] = out[0, 0] / np.sqrt(D)
            W_end[b, hd] = w[0, 0]
    y = x + read @ p["o_net.weight"].T
    if not layer.pre_lnorm:
        y = layer_norm_numpy(y, p["layer_norm.weight"], p["layer_norm.bias"])
    return y, W_end


def layer_norm_numpy(x, g, b, eps=1e-5):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * g + b


@pytest.fixture(scope="module")
def pkg(fwp):
    return fwp


def make_layer(pkg, pre_lnorm, seed=0, H=2, D=4, dm=12, op=loop_op):
    torch.manual_seed(seed)
    layer = pkg.DeltaNetLayer(H, dm, D, dropout=0.0, pre_lnorm=pre_lnorm, layer_id=0, num_layer=1,
                              fast_weight_op=op).double()
    with torch.no_grad():
        for prm in layer.parameters():
            prm.normal_(0.0, 0.5)
    return layer


@pytest.mark.parametrize("pre_lnorm", [False, True])
def test_layer_matches_numpy_restatement(pkg, pre_lnorm):
    layer = make_layer(pkg, pre_lnorm)
    h = torch.randn(9, 3, 12, dtype=torch.float64)
    W0 = torch.randn(3, 2, 4, 4, dtype=torch.float64) * 0.3
    got = layer(h)
    want, _ = layer_numpy(layer, h.numpy())
    assert np.abs(got.detach().numpy() - want).max() < 1e-10
    got, (W_end, k_acc) = layer(h, mems=(W0.clone(), None), carry_over_fast_weight=True)
    want, W_want = layer_numpy(layer, h.numpy(), W0.numpy())
    assert k_acc is None
    assert np.abs(got.detach().numpy() - want).max() < 1e-10
    assert np.abs(W_end.numpy() - W_want).max() < 1e-10
    assert not W_end.requires_grad


def test_layer_is_causal_and_splits_into_segments(pkg):
    layer = make_layer(pkg, False, seed=1)
    h = torch.randn(10, 2, 12, dtype=torch.float64)
    whole = layer(h)
    h2 = h.clone()
    h2[6:] += 1.0
    assert torch.equal(layer(h2)[:6], whole[:6])            # later inputs cannot reach back
    first, mem = layer(h[:4], carry_over_fast_weight=True)
    second, mem2 = layer(h[4:], mems=mem, carry_over_fast_weight=True)
    assert torch.allclose(torch.cat((first, second)), whole, atol=1e-12)
    # a smaller last batch takes the leading rows of the carried state
    part, _ = layer(h[4:, :1], mems=mem, carry_over_fast_weight=True)
    assert torch.allclose(part, whole[4:, :1], atol=1e-12)
    with pytest.raises(ValueError):
        layer(h, mems=mem)


def test_positional_embedding_and_ff(pkg):
    pe = pkg.PositionalEmbedding(8)
    pos = torch.arange(4, -1, -1.0)
    e = pe(pos)
    assert e.shape == (5, 1, 8)
    assert torch.allclose(e[-1, 0], torch.tensor([0.0] * 4 + [1.0] * 4))      # position 0
    assert torch.allclose(e[0, 0, 0], torch.sin(torch.tensor(4.0)))
    assert torch.allclose(e[0, 0, 5], torch.cos(torch.tensor(4.0 / 10000 ** 0.25)))
    assert pe(pos, bsz=3).shape == (5, 3, 8)
    torch.manual_seed(0)
    x = torch.randn(3, 2, 8)
    for pre in (False, True):
        ff = pkg.PositionwiseFF(8, 16, 0.0, pre_lnorm=pre)
        core = ff.CoreNet
        want = (x + core(ff.layer_norm(x))) if pre else ff.layer_norm(x + core(x))
        assert torch.allclose(ff(x), want)


def make_lm(pkg, op, device="cpu", dtype=torch.float64, **kw):
    cfg = dict(n_token=50, n_layer=2, n_head=2, d_model=16, d_head=4, d_inner=24)
    cfg.update(kw)
    torch.manual_seed(3)
    return pkg.DeltaNetLM(fast_weight_op=op, init_std=0.3, **cfg).to(device=device, dtype=dtype)


def test_lm_loss_shape_tying_and_carry_over(pkg):
    lm = make_lm(pkg, loop_op)
    assert lm.crit.out_layers[0].weight is lm.word_emb.emb_layers[0].weight
    names = set(lm.state_dict())
    assert {"word_emb.emb_layers.0.weight", "layers.1.dec_attn.qkvb_net.weight",
            "layers.0.pos_ff.CoreNet.3.bias", "crit.out_layers.0.bias"} <= names
    g = torch.Generator().manual_seed(0)
    data = torch.randint(0, 50, (12, 3), generator=g)
    target = torch.randint(0, 50, (12, 3), generator=g)
    (loss,) = lm(data, target)
    assert loss.shape == (12, 3)
    # per-token NLL of a softmax: exp(-loss) is a probability, and it is the right one
    hid, _ = lm.hidden(data)
    logp = torch.log_softmax(hid @ lm.word_emb.emb_layers[0].weight.T + lm.crit.out_layers[0].bias, -1)
    assert torch.allclose(loss, -logp.gather(-1, target.unsqueeze(-1)).squeeze(-1), atol=1e-10)
    # Carrying the fast weights joins segments exactly, except that positions restart.
    out = lm(data[:5], target[:5], carry_over_fast_weight=True)
    assert len(out) == 1 + lm.n_layer and out[1][0].shape == (3, 2, 4, 4) and out[1][1] is None
    out2 = lm(data[5:], target[5:], *out[1:], carry_over_fast_weight=True)
    assert out2[0].shape == (7, 3)
    loss.mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in lm.parameters())


# ------------------------------------------------------------------ GPU: HIP op in situ

def close(name, got, want):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    err = (got - want).abs()
    assert bool((err <= ATOL + RTOL * want.abs()).all()), f"{name}: max abs err {err.max():.3e}"


@pytest.mark.gpu
@pytest.mark.parametrize("pre_lnorm,D", [(False, 16), (True, 32), (False, 8)])
def test_gpu_layer_against_loop_operator(pkg, pre_lnorm, D):
    H, dm, T, B = 4, 64, 150, 3
    torch.manual_seed(0)
    ours = pkg.DeltaNetLayer(H, dm, D, pre_lnorm=pre_lnorm, layer_id=0, num_layer=1).cuda()
    ref = pkg.DeltaNetLayer(H, dm, D, pre_lnorm=pre_lnorm, layer_id=0, num_layer=1,
                            fast_weight_op=loop_op).double()
    with torch.no_grad():
        for prm in ours.parameters():
            prm.normal_(0.0, 0.3)
    ref.load_state_dict(ours.state_dict())
    h = torch.randn(T, B, dm, device="cuda", requires_grad=True)
    h_ref = h.detach().double().cpu().requires_grad_(True)
    W0 = torch.randn(B, H, D, D, device="cuda") * 0.2
    g = torch.randn(T, B, dm, device="cuda")
    out, (W_end, _) = ours(h, mems=(W0, None), carry_over_fast_weight=True)
    out_ref, (W_ref, _) = ref(h_ref, mems=(W0.double().cpu(), None), carry_over_fast_weight=True)
    close("out", out, out_ref)
    close("W_end", W_end, W_ref)
    out.backward(g)
    out_ref.backward(g.double().cpu())
    close("grad_h", h.grad, h_ref.grad)
    for (name, a), (_, b) in zip(ours.named_parameters(), ref.named_parameters()):
        scale = b.grad.abs().max()
        err = (a.grad.double().cpu() - b.grad).abs().max()
        assert err <= 1e-4 * max(1.0, float(scale)), f"grad {name}: {err:.3e} (scale {scale:.3e})"


@pytest.mark.gpu
def test_gpu_lm_against_loop_operator(pkg):
    kw = dict(n_token=211, n_layer=3, n_head=4, d_model=64, d_head=16, d_inner=96)
    ours = make_lm(pkg, None, device="cuda", dtype=torch.float32, **kw)
    ref = make_lm(pkg, loop_op, **kw)
    ref.load_state_dict({k: v.double().cpu() for k, v in ours.state_dict().items()})
    g = torch.Generator().manual_seed(1)
    data = torch.randint(0, 211, (96, 4), generator=g)
    target = torch.randint(0, 211, (96, 4), generator=g)
    (loss,) = ours(data.cuda(), target.cuda())
    (loss_ref,) = ref(data, target)
    close("loss", loss, loss_ref)
    loss.mean().backward()
    loss_ref.mean().backward()
    for (name, a), (_, b) in zip(ours.named_parameters(), ref.named_parameters()):
        scale = float(b.grad.abs().max())
        err = float((a.grad.double().cpu() - b.grad).abs().max())
        assert err <= 2e-4 * max(scale, 1e-3) + 1e-7, f"grad {name}: {err:.3e} (scale {scale:.3e})"


@pytest.mark.gpu
def test_gpu_lm_at_benchmark_size_against_loop_operator(pkg):
    """The 16-layer language model of the benchmark (d_model 256, 8 heads of 32, FFN 1024, vocabulary
    32768, 32 sequences of 1024 tokens drawn from Zipf(1.1), initialisation N(0, 0.02)): fp32 with the HIP
    operator against float64 with the step loop as operator, same weights and tokens.  Per-token
    losses within 1e-4 + 1e-3 |want|; every parameter gradient within 1e-3 of its largest entry."""
    cfg = dict(n_token=32768, n_layer=16, n_head=8, d_model=256, d_head=32, d_inner=1024)
    B, T = 32, 1024
    torch.manual_seed(5)
    ours = pkg.DeltaNetLM(init_std=0.02, **cfg).cuda()
    ref = pkg.DeltaNetLM(fast_weight_op=loop_op, init_std=0.02, **cfg).to(device="cuda", dtype=torch.float64)
    ref.load_state_dict({k: v.double() for k, v in ours.state_dict().items()})
    p = np.arange(1, cfg["n_token"] + 1, dtype=np.float64) ** -1.1
    cdf = np.cumsum(p / p.sum())
    toks = np.minimum(np.searchsorted(cdf, np.random.default_rng(0).random((T + 1, B))), cfg["n_token"] - 1)
    toks = torch.from_numpy(toks.astype(np.int64)).cuda()
    data, target = toks[:-1], toks[1:]
    (loss,) = ours(data, target)
    loss.mean().backward()
    (loss_ref,) = ref(data, target)
    loss_ref.mean().backward()
    torch.cuda.synchronize()
    err = (loss.detach().double() - loss_ref.detach()).abs()
    print(f"\nLM at benchmark size: mean loss {float(loss_ref.detach().mean()):.4f}, per-token loss max abs err "
          f"{float(err.max()):.3e}", flush=True)
    assert bool((err <= ATOL + RTOL * loss_ref.detach().abs()).all()), f"loss: max abs err {float(err.max()):.3e}"
    worst = 0.0
    for (name, a), (_, b) in zip(ours.named_parameters(), ref.named_parameters()):
        scale = float(b.grad.abs().max())
        e = float((a.grad.double() - b.grad).abs().max())
        worst = max(worst, e / max(scale, 1e-30))
        assert e <= 1e-3 * scale + 1e-9, f"grad {name}: {e:.3e} (scale {scale:.3e})"
    print(f"parameter gradients: worst error relative to the tensor's largest entry {worst:.3e}", flush=True)


@pytest.mark.gpu
@pytest.mark.parametrize("scale", [1.0, 0.25])
@pytest.mark.parametrize("D", [16, 32, 64])
def test_gpu_fused_pre_step_against_the_pytorch_lines(pkg, D, scale):
    from importlib import import_module
    layers = import_module(pkg.__name__ + ".layers")
    T, B, H = 37, 3, 5
    torch.manual_seed(D)
    qkvb = (torch.randn(T, B, H * (3 * D + 1), device="cuda") * 2).requires_grad_(True)
    ref_in = qkvb.detach().double().requires_grad_(True)
    got = pkg.DeltaNetPrep.apply(qkvb, H, D, scale)
    x = ref_in.view(T, B, H, 3 * D + 1)
    q, k, v, beta = (t.permute(1, 2, 0, 3) for t in x.split((D, D, D, 1), dim=-1))
    want = (scale * layers.sum_normalised_elu(q), layers.sum_normalised_elu(k), v, torch.sigmoid(beta))
    gs = [torch.randn_like(w) for w in want]
    for name, a, b in zip("q k v beta".split(), got, want):
        assert a.is_contiguous() and a.shape == b.shape
        close(name, a, b)
    torch.autograd.backward(got, [g.float().cuda() for g in gs])
    torch.autograd.backward(want, gs)
    close("grad_qkvb", qkvb.grad, ref_in.grad)
