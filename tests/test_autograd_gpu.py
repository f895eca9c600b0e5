"""Gradients through the layer and stack MODULES (the reference trains through
layers/mvpa.py:280-337 and models/mvpformer.py:132-147): the HIP path - library GEMMs with GEMM
backward passes, FlashMVPA with the mvpa_backward kernels, RMSNorm - against reverse-mode
differentiation of the CPU oracle on the same bf16-rounded weights, in float64.
Tolerances are this build's statement for bf16 arithmetic: relative L2 error of every gradient
<= 3e-2 (fp32 layer: <= 2e-4)."""
import math

import pytest
import torch

from layers import MVPFormerGQAAttention, MVPFormerGQAFlashAttention
from models.fftencoder import WaveEncoder
from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead
from oracle import mvpa_oracle as O

pytestmark = pytest.mark.gpu


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def _config(**kw):
    base = dict(n_positions=16, n_channels=40, n_embd=128, n_layer=2, n_head=2, n_inner=256,
                n_head_kv=1, resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)
    base.update(kw)
    return MVPFormerConfig(**base)


def _oracle_layer_grads(layer, hidden, pos, chan, g_out, dtype=torch.float64, **flags):
    names = ["q_attn.weight", "c_attn.weight", "position_net.weight", "channel_net.weight",
             "c_proj.weight", "attn_bias"]
    w = {n: layer.state_dict()[n].detach().cpu().to(dtype).requires_grad_(True) for n in names}
    x = hidden.detach().cpu().to(dtype).requires_grad_(True)
    p = pos.detach().cpu().to(dtype).requires_grad_(True)
    c = chan.detach().cpu().to(dtype).requires_grad_(True)
    out = O.attention_layer_forward(x, p, c, w, layer.num_heads, layer.num_kv_heads, **flags)
    (out * g_out.cpu().to(dtype)).sum().backward()
    grads = {n: t.grad for n, t in w.items()}
    grads.update(hidden=x.grad, pos=p.grad, chan=c.grad)
    return out.detach(), grads


@pytest.mark.parametrize("cls,dims", [
    (MVPFormerGQAFlashAttention, dict(n_embd=128, n_head=2, n_head_kv=1, T=13, C=33)),      # Dh 64: matrix-core backward
    (MVPFormerGQAAttention, dict(n_embd=128, n_head=2, n_head_kv=2, T=12, C=20)),
    (MVPFormerGQAFlashAttention, dict(n_embd=64, n_head=4, n_head_kv=2, T=14, C=5)),        # Dh 16: row-per-lane backward
], ids=["flash-dh64", "masked-dh64", "flash-dh16"])
def test_layer_gradients_bf16(cls, dims):
    torch.manual_seed(5)
    T, C = dims.pop("T"), dims.pop("C")
    cfg = _config(**dims)
    layer = cls(cfg, layer_idx=0).to(device="cuda", dtype=torch.bfloat16).train()
    with torch.no_grad():
        for prm in layer.parameters():
            prm.mul_(4.0)                      # away from the tiny init: every path carries signal
    E = cfg.n_embd
    hidden = torch.randn(2, T, C, E, device="cuda").to(torch.bfloat16).requires_grad_(True)
    pos = (torch.randn(1, T, E, device="cuda") * 0.5).to(torch.bfloat16).requires_grad_(True)
    chan = (torch.randn(1, C, E, device="cuda") * 0.5).to(torch.bfloat16).requires_grad_(True)
    g_out = torch.randn(2, T, C, E, device="cuda").to(torch.bfloat16)
    out = layer(hidden, pos, chan)[0]
    assert out.requires_grad
    (out.float() * g_out.float()).sum().backward()
    ref_out, ref = _oracle_layer_grads(layer, hidden, pos, chan, g_out)
    assert _rel(out.detach(), ref_out) <= 1e-2
    got = {n: p.grad for n, p in layer.named_parameters()}
    got.update(hidden=hidden.grad, pos=pos.grad, chan=chan.grad)
    for n, r in ref.items():
        assert got[n] is not None, n
        err = _rel(got[n], r)
        assert err <= 3e-2, f"{n}: rel-L2 {err:.3e}"


def test_layer_gradients_fp32_with_channel_mask():
    """fp32 tensors (row-per-lane kernels, torch's fp32 GEMM) with an additive key mask that
    marks absent channels: gradients to 2e-4, and exactly zero into the absent channels' keys."""
    torch.manual_seed(6)
    cfg = _config(n_embd=64, n_head=4, n_head_kv=2)
    T, C, E = 9, 6, 64
    layer = MVPFormerGQAAttention(cfg, layer_idx=0).to(device="cuda").train()
    with torch.no_grad():
        for prm in layer.parameters():
            prm.mul_(4.0)
    hidden = torch.randn(2, T, C, E, device="cuda", requires_grad=True)
    pos = (torch.randn(1, T, E, device="cuda") * 0.5).requires_grad_(True)
    chan = (torch.randn(1, C, E, device="cuda") * 0.5).requires_grad_(True)
    valid = torch.tensor([[1, 1, 0, 1, 1, 0], [1, 0, 1, 1, 1, 1]], dtype=torch.bool, device="cuda")
    m = valid[:, None, :].expand(2, T, C).reshape(2, T * C).float()
    am = ((1.0 - m) * torch.finfo(torch.float32).min)[:, None, None, :]
    g_out = torch.randn(2, T, C, E, device="cuda")
    out = layer(hidden, pos, chan, attention_mask=am)[0]
    (out * g_out).sum().backward()
    ref_out, ref = _oracle_layer_grads(layer, hidden, pos, chan, g_out,
                                       attention_mask=am.cpu().double())
    assert (out.detach().cpu().double() - ref_out).abs().max().item() <= 2e-5
    got = {n: p.grad for n, p in layer.named_parameters()}
    got.update(hidden=hidden.grad, pos=pos.grad, chan=chan.grad)
    for n, r in ref.items():
        err = _rel(got[n], r)
        assert err <= 2e-4, f"{n}: rel-L2 {err:.3e}"


def test_eval_forward_stays_on_the_fused_path():
    """eval() mode on an input without a graph: no autograd graph is built even with grad mode
    on, and the result is the inference path's bit for bit."""
    torch.manual_seed(7)
    cfg = _config()
    layer = MVPFormerGQAFlashAttention(cfg, layer_idx=0).to(device="cuda", dtype=torch.bfloat16).eval()
    hidden = torch.randn(1, 6, 33, 128, device="cuda").to(torch.bfloat16)
    pos = torch.randn(1, 6, 128, device="cuda").to(torch.bfloat16)
    chan = torch.randn(1, 33, 128, device="cuda").to(torch.bfloat16)
    a = layer(hidden, pos, chan)[0]
    with torch.no_grad():
        b = layer(hidden, pos, chan)[0]
    assert not a.requires_grad and torch.equal(a, b)
    # an input that carries a graph switches the differentiable path on, also in eval() mode
    c = layer(hidden.clone().requires_grad_(True), pos, chan)[0]
    assert c.requires_grad
    assert (c.detach().float() - a.float()).abs().max().item() <= 2e-2
    # dropout needs the differentiable path: train() mode under no_grad has none
    layer.train()
    layer.attn_dropout.p = 0.1
    with torch.no_grad(), pytest.raises(NotImplementedError):
        layer(hidden, pos, chan)
    # the masked layer's dropout acts on the [B,H,N,N] weights, which are never formed
    masked = MVPFormerGQAAttention(cfg, layer_idx=0).to(device="cuda", dtype=torch.bfloat16).train()
    masked.attn_dropout.p = 0.1
    with pytest.raises(NotImplementedError):
        masked(hidden, pos, chan)


def _keep_masks(T, C, drop_t, drop_c):
    tk = torch.ones(T, dtype=torch.bool)
    ck = torch.ones(C, dtype=torch.bool)
    tk[list(drop_t)] = False
    ck[list(drop_c)] = False
    return tk, ck


def test_attention_dropout_is_the_reference_kernels():
    """attentions/attn.py:1052-1059, 222-227: whole key steps and channels are dropped, AFTER the
    soft-max sum, the rest divided by 1 - p.  With v = 1 the output of a query is therefore its
    kept probability mass / (1 - p) - below 1 / (1 - p) wherever a visible key was dropped (a
    dropout that masked keys before the soft-max would give exactly 1 / (1 - p)) - and equals the
    oracle's attention on the indicator of the kept keys; with random v output and gradients
    equal the oracle's on values scaled key by key."""
    import math
    from attentions import flashmvpa
    from mvpa_hip.synthetic import make_mvpa_inputs
    B, C, T, H, Hkv, Dh, p = 2, 12, 9, 2, 1, 32, 0.25
    inp = make_mvpa_inputs(B=B, C=C, T=T, H=H, Hkv=Hkv, Dh=Dh, seed=3, qkv_unit=True)
    tk, ck = _keep_masks(T, C, drop_t=(2, 7), drop_c=(0, 5, 11))
    keep = torch.zeros(T * C, dtype=torch.float64)
    for t in range(T):
        for c in range(C):
            keep[t * C + c] = 1.0 if (tk[t] and ck[c]) else 0.0
    d = inp.to("cuda", torch.float32)

    def run(v, **kw):
        return flashmvpa(d.q, d.u.view(1, Hkv, 1, Dh), d.vb.view(1, Hkv, 1, Dh), d.z.view(1, Hkv, 1, Dh), d.k,
                         d.k_time.view(1, Hkv, T, Dh), d.k_chan.view(1, Hkv, C, Dh), v, True,
                         1.0 / math.sqrt(Dh), window_size=10, **kw)
    ones = torch.ones_like(d.v)
    got = run(ones, p_drop=p, time_keep=tk.cuda(), chan_keep=ck.cuda()).double().cpu()
    args64 = [t.double() for t in (inp.q, inp.k)]
    tabs64 = [t.double() for t in (inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan)]
    mass = O.mvpa_direct(args64[0], args64[1], keep[None, None, :, None].expand(B, Hkv, T * C, Dh).contiguous(),
                         *tabs64, window=10)
    assert (got - mass / (1 - p)).abs().max().item() <= 1e-5
    rows_with_a_dropped_key = got[:, :, 3 * C:, 0]                 # from time step 3 on, step 2 is visible
    assert (rows_with_a_dropped_key < 1 / (1 - p) - 1e-4).all()
    # random values, output and every gradient
    leaves = {n: getattr(d, n).clone().requires_grad_(True) for n in ("q", "k", "v")}
    out = flashmvpa(leaves["q"], d.u.view(1, Hkv, 1, Dh), d.vb.view(1, Hkv, 1, Dh), d.z.view(1, Hkv, 1, Dh),
                    leaves["k"], d.k_time.view(1, Hkv, T, Dh), d.k_chan.view(1, Hkv, C, Dh), leaves["v"], True,
                    1.0 / math.sqrt(Dh), window_size=10, p_drop=p, time_keep=tk.cuda(), chan_keep=ck.cuda())
    g_out = torch.randn(out.shape, device="cuda", generator=torch.Generator("cuda").manual_seed(1))
    out.backward(g_out)
    ref_leaves = {n: getattr(inp, n).double().clone().requires_grad_(True) for n in ("q", "k", "v")}
    ref = O.mvpa_direct(ref_leaves["q"], ref_leaves["k"], ref_leaves["v"] * (keep / (1 - p))[None, None, :, None],
                        *tabs64, window=10)
    (ref * g_out.double().cpu()).sum().backward()
    assert (out.detach().double().cpu() - ref.detach()).abs().max().item() <= 1e-5
    for n in ("q", "k", "v"):
        err = (leaves[n].grad.double().cpu() - ref_leaves[n].grad).abs().max().item()
        assert err <= 2e-5 + 1e-4 * ref_leaves[n].grad.abs().max().item(), (n, err)
    assert leaves["v"].grad[:, :, keep == 0].abs().max().item() == 0.0     # dropped keys: no value gradient


def test_attention_dropout_masks_are_drawn_as_the_reference_draws_them():
    """Channels first, then time steps, `torch.rand(n) > 1 - sqrt(1 - p)` on the device from the
    generator given (attentions/attn.py:1052-1059): the same generator state gives the same masks
    as those two calls, and the keep rate per key is 1 - p."""
    from attentions.attn import dropout_key_scale
    T, C, p = 64, 128, 0.19
    g = torch.Generator("cuda").manual_seed(123)
    scale = dropout_key_scale(p, T, C, torch.device("cuda"), g)
    g2 = torch.Generator("cuda").manual_seed(123)
    per_dim = 1 - (1 - p) ** 0.5
    chan = torch.rand(C, device="cuda", generator=g2) > per_dim
    time = torch.rand(T, device="cuda", generator=g2) > per_dim
    want = (time[:, None] & chan[None, :]).reshape(-1).float() / (1 - p)
    assert torch.equal(scale, want)
    rate = torch.stack([(dropout_key_scale(p, T, C, torch.device("cuda"), g) > 0).float().mean() for _ in range(200)]).mean().item()
    assert abs(rate - (1 - p)) <= 0.02, rate


def test_layer_and_stack_train_with_the_shipped_dropout_rates():
    """train() mode with resid_pdrop = embd_pdrop = attn_pdrop = 0.1 (the reference's defaults,
    models/mvpformer.py:43): the flash layer and the stack run forward and backward, the draw
    follows torch's generator (same seed, same result; another seed, another result), eval() is
    untouched, and every parameter receives a finite gradient."""
    torch.manual_seed(11)
    cfg = _config(resid_pdrop=0.1, embd_pdrop=0.1, attn_pdrop=0.1)
    layer = MVPFormerGQAFlashAttention(cfg, layer_idx=0).to(device="cuda", dtype=torch.bfloat16)
    hidden = torch.randn(2, 9, 33, 128, device="cuda").to(torch.bfloat16)
    pos = torch.randn(1, 9, 128, device="cuda").to(torch.bfloat16)
    chan = torch.randn(1, 33, 128, device="cuda").to(torch.bfloat16)
    ref = layer.eval()(hidden, pos, chan)[0]
    layer.train()
    torch.manual_seed(1)
    a = layer(hidden, pos, chan)[0]
    torch.manual_seed(1)
    b = layer(hidden, pos, chan)[0]
    torch.manual_seed(2)
    c = layer(hidden, pos, chan)[0]
    assert torch.equal(a, b) and not torch.equal(a, c) and not torch.equal(a.detach(), ref)
    assert torch.equal(layer.eval()(hidden, pos, chan)[0], ref)
    L, B, T, C = 64, 2, 7, 33
    model = HMVPFormer(cfg, WaveEncoder(L, cfg.n_embd), MVPFormerHead(cfg.n_embd, cfg.n_embd))
    model = model.to(device="cuda", dtype=torch.bfloat16).train()
    x = torch.randn(B, T, C, L, device="cuda")
    out = model.predict_next_segment(x)
    y = out[0] if isinstance(out, (tuple, list)) else out
    y.float().pow(2).mean().backward()
    used = [n for n, prm in model.named_parameters() if prm.grad is not None]
    assert len(used) >= 10
    for n, prm in model.named_parameters():
        if prm.grad is not None:
            assert torch.isfinite(prm.grad).all(), n


def test_stack_gradients_bf16():
    """Encoder -> two parallel blocks -> final norm in train() mode: the gradient of a scalar of
    the last hidden state with respect to EVERY parameter that the forward uses, against the
    oracle stack in float64 on the same bf16-rounded weights."""
    torch.manual_seed(8)
    cfg = _config()
    L, B, T, C = 64, 2, 7, 33
    model = HMVPFormer(cfg, WaveEncoder(L, cfg.n_embd), MVPFormerHead(cfg.n_embd, cfg.n_embd))
    model = model.to(device="cuda", dtype=torch.bfloat16).train()
    with torch.no_grad():
        for n, prm in model.named_parameters():
            if "ln" in n:
                prm.add_(0.2 * torch.randn_like(prm))
            elif prm.dim() == 2 or "attn_bias" in n:
                prm.mul_(3.0)
    x = torch.randn(B, T, C, L, device="cuda")
    g_out = torch.randn(B, T, C, cfg.n_embd, device="cuda").to(torch.bfloat16)
    out, emb = model._common_forward(x)
    assert out.requires_grad and emb.requires_grad
    (out.float() * g_out.float()).sum().backward()

    params = {k: v.detach().cpu().double().requires_grad_(True) for k, v in model.state_dict().items()
              if v.dtype.is_floating_point and v.dim() > 0 and "time_bias" not in k}
    ref_out, _ = O.mvpformer_forward(x.cpu().double(), params, dict(n_layer=2, n_head=2, n_head_kv=1))
    (ref_out * g_out.cpu().double()).sum().backward()
    assert _rel(out.detach(), ref_out.detach()) <= 2e-2
    checked = 0
    for n, prm in model.named_parameters():
        r = params[n].grad if n in params else None
        if r is None or r.abs().max() == 0:
            # parameters the forward does not touch: ln_2 (models/mvpformer.py:104-147), the head,
            # the seizure embeddings
            assert prm.grad is None or prm.grad.abs().max().item() == 0, n
            continue
        if "embedding" in n:          # only the first T / C rows are used: the rest get zero
            rows = T if "positional" in n else C
            assert prm.grad[rows:].abs().max().item() == 0
        err = _rel(prm.grad, r)
        assert err <= 3e-2, f"{n}: rel-L2 {err:.3e}"
        checked += 1
    assert checked >= 2 * 9 + 5        # every weight of both blocks, norms, embeddings, encoder


def test_generative_score_is_differentiable_in_train_mode():
    """predict_next_segment (models/mvpformer.py:749-764) in train() mode gives a score with a
    graph that reaches the head, the blocks and the encoder's projection."""
    torch.manual_seed(9)
    cfg = _config()
    model = HMVPFormer(cfg, WaveEncoder(64, cfg.n_embd), MVPFormerHead(cfg.n_embd, cfg.n_embd))
    model = model.to(device="cuda", dtype=torch.bfloat16).train()
    x = torch.randn(1, 6, 33, 64, device="cuda")
    score = model.predict_next_segment(x)
    assert score.shape == (1, 5, 33) and score.requires_grad
    (-score.mean()).backward()
    for n in ("head.head.weight", "encoder.proj.weight", "mvpformer.h.0.attn.c_attn.weight",
              "mvpformer.h.1.mlp.down_proj.weight", "mvpformer.h.0.attn.attn_bias"):
        g = dict(model.named_parameters())[n].grad
        assert g is not None and torch.isfinite(g.float()).all() and g.abs().max().item() > 0, n
    model.eval()
    with torch.no_grad():
        s2 = model.predict_next_segment(x)
    assert (s2.float() - score.detach().float()).abs().max().item() <= 3e-2
