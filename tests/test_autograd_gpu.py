"""Gradients through the layer and stack MODULES (the reference trains through
layers/mvpa.py:280-337 and models/mvpformer.py:132-147): the HIP path - library GEMMs with GEMM
backward passes, FlashMVPA with the mvpa_backward kernels, RMSNorm - against reverse-mode
differentiation of the CPU oracle on the same bf16-rounded weights, in float64.
Tolerances are this build's statement for bf16 arithmetic: relative L2 error of every gradient
<= 3e-2 (fp32 layer: <= 2e-4)."""
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
    layer.train()
    layer.attn_dropout.p = 0.1
    with pytest.raises(NotImplementedError):
        layer(hidden, pos, chan)


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
