"""GPU checks of the attention layers and of the MVPFormer stack against the CPU oracle."""
from types import SimpleNamespace

import pytest
import torch

from layers import MVPFormerGQAAttention, MVPFormerGQAFlashAttention
from mvpa_hip.synthetic import make_ieeg
from oracle import mvpa_oracle as O

pytestmark = pytest.mark.gpu


def _cfg(**kw):
    base = dict(max_position_embeddings=32, hidden_size=128, num_attention_heads=4, n_head_kv=2,
                n_inner=256, global_att=True, scale_attn_weights=True,
                scale_attn_by_inverse_layer_idx=False, reorder_and_upcast_attn=False,
                lora=False, attn_pdrop=0.1, resid_pdrop=0.1)
    base.update(kw)
    return SimpleNamespace(**base)


def _layer_io(T=14, C=6, E=128, B=2, seed=0):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(B, T, C, E, generator=g)
    pos = torch.randn(1, T, E, generator=g) * 0.5
    chan = torch.randn(1, C, E, generator=g) * 0.5
    return h, pos, chan


def _oracle_layer(layer, h, pos, chan, heads, kv, **kw):
    w = {k: v.detach().float().cpu() for k, v in layer.state_dict().items()}
    return O.attention_layer_forward(h, pos, chan, w, heads, kv, **kw)


def test_layer_fp32_matches_oracle():
    """MVPFormerGQAAttention in fp32 (generic kernel + BLAS projections), with the additive
    attention_mask the model builds from a 0/1 mask."""
    torch.manual_seed(0)
    layer = MVPFormerGQAAttention(_cfg(), layer_idx=0).eval()
    for p in layer.parameters():
        p.data.mul_(4.0)            # lift the logits off zero so masks and biases matter
    h, pos, chan = _layer_io()
    B, T, C, _ = h.shape
    keep = (torch.rand(B, T * C, generator=torch.Generator().manual_seed(1)) > 0.2).float()
    am = ((1.0 - keep) * torch.finfo(torch.float32).min)[:, None, None, :]
    ref = _oracle_layer(layer, h, pos, chan, 4, 2, attention_mask=am)
    lg = layer.cuda()
    out, present = lg(h.cuda(), pos.cuda(), chan.cuda(), attention_mask=am.cuda())
    assert present is None
    assert (out.cpu() - ref).abs().max().item() <= 2e-4
    out2 = lg(h.cuda(), pos.cuda(), chan.cuda(), attention_mask=am.cuda(), use_cache=True)
    assert out2[1][0].shape == (B, 2, T, C, 32)
    with pytest.raises(NotImplementedError):
        lg(h.cuda(), pos.cuda(), chan.cuda(), output_attentions=True)
    # a mask that is constant over time is recognised as channel validity (same result)
    keep_c = torch.tensor([[1, 1, 0, 1, 1, 0], [0, 1, 1, 1, 1, 1]], dtype=torch.float32)
    am2 = ((1.0 - keep_c[:, None, :].expand(B, T, C).reshape(B, T * C)) * torch.finfo(torch.float32).min)[:, None, None, :]
    assert lg._as_channel_validity(am2.cuda(), B, T, C) is not None
    assert lg._as_channel_validity(am.cuda(), B, T, C) is None
    ref2 = _oracle_layer(layer.cpu(), h, pos, chan, 4, 2, attention_mask=am2)
    out3 = layer.cuda()(h.cuda(), pos.cuda(), chan.cuda(), attention_mask=am2.cuda())[0]
    assert (out3.cpu() - ref2).abs().max().item() <= 2e-4


def test_flash_layer_bf16_matches_oracle_and_ignores_mask():
    torch.manual_seed(1)
    layer = MVPFormerGQAFlashAttention(_cfg(lora=True, lora_rank=8, lora_alpha=16, lora_dropout=0,
                                            lora_merge=True), layer_idx=0).eval()
    for p in layer.parameters():
        p.data.mul_(3.0)
    layer.c_attn.lora_B.data.normal_(0, 0.05)          # make the adapter path matter
    layer = layer.to(torch.bfloat16)
    h, pos, chan = _layer_io(T=20, C=40, seed=3)
    hb, pb, cb = h.bfloat16(), pos.bfloat16(), chan.bfloat16()
    w = {k: v.detach().float() for k, v in layer.state_dict().items()}
    w["q_attn.weight"] = layer.q_attn.effective_weight().detach().float()
    w["c_attn.weight"] = layer.c_attn.effective_weight().detach().float()
    ref = O.attention_layer_forward(hb.float(), pb.float(), cb.float(), w, 4, 2)
    lg = layer.cuda()
    out = lg(hb.cuda(), pb.cuda(), cb.cuda(), attention_mask=torch.full((2, 1, 1, 800), -1e30).cuda())
    assert len(out) == 2 and out[1] is None
    o = out[0].float().cpu()
    rel = ((o - ref).norm() / ref.norm()).item()
    assert rel <= 2e-2, rel
    out3 = lg(hb.cuda(), pb.cuda(), cb.cuda(), output_attentions=True)
    assert len(out3) == 3 and out3[2] is None


def test_mvpformer_forward_matches_oracle():
    """Encoder -> two parallel blocks -> final norm -> head, bf16 on the GPU against the fp32
    oracle stack on the same (bf16-rounded) parameters."""
    from models.fftencoder import WaveEncoder
    from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead
    torch.manual_seed(2)
    cfg = MVPFormerConfig(n_positions=16, n_channels=16, n_embd=128, n_layer=2, n_head=4,
                          n_head_kv=2, n_inner=256)
    model = HMVPFormer(cfg, WaveEncoder(512, 128), MVPFormerHead(128, 128)).to(torch.bfloat16).eval()
    for name, p in model.named_parameters():
        if "attn" in name or "embedding" in name:
            p.data.mul_(3.0)
    sd = model.state_dict()
    assert "mvpformer.h.1.attn.c_attn.weight" in sd and "mvpformer.h.0.ln_2.weight" in sd
    assert "mvpformer.h.0.mlp.gate_proj.weight" in sd and "encoder.proj.weight" in sd
    assert "head.head.weight" in sd and "seizure_embeddings" in sd and sd["encoder.proj.weight"].shape == (128, 550)
    x = make_ieeg(2, 8, 6, 512, seed=5)
    params = {k: v.float() for k, v in sd.items()}
    ref, ref_emb = O.mvpformer_forward(x, params, dict(n_layer=2, n_head=4, n_head_kv=2))
    out, emb = model.cuda()._common_forward(x.cuda())
    rel_e = ((emb.float().cpu() - ref_emb).norm() / ref_emb.norm()).item()
    rel_o = ((out.float().cpu() - ref).norm() / ref.norm()).item()
    assert rel_e <= 1e-2, rel_e
    assert rel_o <= 3e-2, rel_o
    score = model.predict_next_segment(x.cuda())
    assert score.shape == (2, 5, 8) and torch.isfinite(score).all()


def test_mvpformer_s_dims_match_oracle_stack():
    """MVPFormer-S as shipped (configs/mvpformer_s_generative.yaml:49-71: E768 L12 H12 Hkv4 Dh64
    n_inner 1728, LoRA adapters on and made non-zero), B1 C64 T16 segments of 512 samples: all
    twelve blocks in bf16 on the GPU against the fp32 oracle stack on the same parameters."""
    from models.configs import MVPFORMER_S
    from models.fftencoder import WaveEncoder
    from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead
    torch.manual_seed(4)
    cfg = MVPFormerConfig(**MVPFORMER_S)
    model = HMVPFormer(cfg, WaveEncoder(512, cfg.n_embd), MVPFormerHead(cfg.n_embd, cfg.n_embd)).to(torch.bfloat16).eval()
    for name, p in model.named_parameters():
        if "lora_B" in name:
            p.data.normal_(0, 0.02)
        elif "attn" in name or "embedding" in name:
            p.data.mul_(2.0)
    x = make_ieeg(1, 64, 16, 512, seed=11)
    params = {k: v.float() for k, v in model.state_dict().items()}
    for i, blk in enumerate(model.mvpformer.h):                   # the oracle takes merged weights
        for lin in ("q_attn", "c_attn"):
            params[f"mvpformer.h.{i}.attn.{lin}.weight"] = getattr(blk.attn, lin).effective_weight().detach().float()
    ref, ref_emb = O.mvpformer_forward(x, params, dict(n_layer=12, n_head=12, n_head_kv=4))
    out, emb = model.cuda()._common_forward(x.cuda())
    rel_e = ((emb.float().cpu() - ref_emb).norm() / ref_emb.norm()).item()
    rel_o = ((out.float().cpu() - ref).norm() / ref.norm()).item()
    print(f"MVPFormer-S dims, 12 blocks: rel-L2 embeddings {rel_e:.3e}, output {rel_o:.3e}")
    assert rel_e <= 1e-2, rel_e
    assert rel_o <= 3e-2, rel_o


def test_mvpformer_s_full_size_properties():
    """The benchmark's MVPFormer-S window (B4 C64 T64 segments of 512 samples) at full size,
    through properties that need no oracle: finite scores, and time-causality of the whole stack,
    bit for bit - changing the last k segments leaves the hidden states of every earlier segment
    untouched."""
    from bench_model import build_mvpformer_s
    model = build_mvpformer_s(512)
    x = make_ieeg(4, 64, 64, 512, seed=0).cuda()
    out, _ = model._common_forward(x)
    assert out.shape == (4, 64, 64, 768) and torch.isfinite(out.float()).all()
    score = model.predict_next_segment(x)
    assert score.shape == (4, 63, 64) and torch.isfinite(score).all()
    x2 = x.clone()
    x2[:, -9:] = x2[:, -9:].flip(-1) * 1.5
    out2, _ = model._common_forward(x2)
    # the last time step keeps the content term for every key, earlier steps only inside the
    # window, but no step ever sees a later one
    assert torch.equal(out2[:, :-9], out[:, :-9])
    assert not torch.equal(out2[:, -9:], out[:, -9:])


@pytest.mark.parametrize("flash", [True, False], ids=["flash", "masked"])
def test_block_with_fused_products_matches_the_separate_ones(flash, monkeypatch):
    """A parallel block at 640 rows: the path that forms q/kv + gate/up in one launch and the block's
    tail (c_proj + down + residual) as one product, against the same block with every product on
    its own (the path of small inputs), with an attention mask (honoured by the masked class only)
    and use_cache: hidden states to bf16 rounding of the different summation order, presents equal."""
    import mvpa_hip
    from models.mvpformer import MVPFormerBlock, MVPFormerConfig
    torch.manual_seed(7)
    cfg = MVPFormerConfig(n_positions=16, n_channels=64, n_embd=128, n_layer=1, n_head=4, n_head_kv=2, n_inner=320)
    blk = MVPFormerBlock(cfg, layer_idx=0, flash=flash).to(device="cuda", dtype=torch.bfloat16).eval()
    for p in blk.parameters():
        p.data.normal_(0, 0.05)
    blk.ln_1.weight.data.fill_(1.0)
    B, T, C, E = 1, 16, 40, 128
    x = torch.randn(B, T, C, E, device="cuda").bfloat16()
    pos = (torch.randn(1, T, E, device="cuda") * 0.3).bfloat16()
    chan = (torch.randn(1, C, E, device="cuda") * 0.3).bfloat16()
    valid = torch.ones(B, T, C, device="cuda")
    valid[:, :, 5] = 0
    valid[:, :, 33:] = 0
    mask = ((1.0 - valid.view(B, -1)) * torch.finfo(torch.bfloat16).min)[:, None, None, :].to(torch.bfloat16)

    def run():
        with torch.no_grad():
            (h, present), normed = blk.forward_fused(x, None, blk.ln_2, pos, chan, attention_mask=mask, use_cache=True)
        return h, present, normed

    assert mvpa_hip.linear_residual_supported(B * T * C, E + 320) and mvpa_hip.linear_dual_supported(B * T * C, E)
    h1, p1, n1 = run()
    monkeypatch.setattr(mvpa_hip, "linear_residual_supported", lambda *a: False)
    h0, p0, n0 = run()
    assert torch.equal(p1[0], p0[0]) and torch.equal(p1[1], p0[1])
    live = valid.bool()[..., None]
    err = ((h1.float() - h0.float()) * live).abs().max().item()
    assert err <= 2 ** -6 * h0.float().abs().max().item(), err
    assert ((n1.float() - n0.float()) * live).abs().max().item() <= 5e-2
    if not flash:           # the mask reaches the kernel: an absent channel's keys change nothing
        x2 = x.clone()
        x2[:, :, 33:] += 1.0
        monkeypatch.undo()
        with torch.no_grad():
            (h2, _), _ = blk.forward_fused(x2, None, blk.ln_2, pos, chan, attention_mask=mask, use_cache=True)
        assert torch.equal(h2[:, :, :5], h1[:, :, :5])


@pytest.mark.parametrize("flash", [True, False], ids=["flash", "masked"])
def test_block_with_the_norm_inside_the_products(flash):
    """forward_norm_fused (ln_1 applied in the epilogue of the q/kv + gate/up launch, row
    statistics written by the tail product) against forward_fused (norm kernel, then the same
    products) on 640 rows: hidden states to bf16 rounding, and the statistics that come out equal
    the sums of squares of the rows that were written."""
    import mvpa_hip
    from models.mvpformer import MVPFormerBlock, MVPFormerConfig
    torch.manual_seed(11)
    cfg = MVPFormerConfig(n_positions=16, n_channels=64, n_embd=128, n_layer=1, n_head=4, n_head_kv=2, n_inner=320)
    blk = MVPFormerBlock(cfg, layer_idx=0, flash=flash).to(device="cuda", dtype=torch.bfloat16).eval()
    for p in blk.parameters():
        p.data.normal_(0, 0.05)
    blk.ln_1.weight.data.copy_(1.0 + 0.3 * torch.randn(128))
    B, T, C, E = 1, 16, 40, 128
    x = (torch.randn(B, T, C, E, device="cuda") * 2.0).bfloat16()
    pos = (torch.randn(1, T, E, device="cuda") * 0.3).bfloat16()
    chan = (torch.randn(1, C, E, device="cuda") * 0.3).bfloat16()
    valid = torch.ones(B, T, C, device="cuda")
    valid[:, :, 7] = 0
    mask = ((1.0 - valid.view(B, -1)) * torch.finfo(torch.bfloat16).min)[:, None, None, :].to(torch.bfloat16)
    assert blk.norm_fused_supported(B * T * C)
    with torch.no_grad():
        (h0, p0), _ = blk.forward_fused(x, None, None, pos, chan, attention_mask=mask, use_cache=True)
        ss_in = mvpa_hip.row_sumsq(x.view(-1, E))
        assert torch.allclose(ss_in[:, 0], x.view(-1, E).float().pow(2).sum(-1), rtol=1e-5)
        (h1, p1), ss = blk.forward_norm_fused(x, ss_in, pos, chan, attention_mask=mask, use_cache=True)
    live = valid.bool()[..., None]
    scale = h0.float().abs().max().item()
    assert ((h1.float() - h0.float()) * live).abs().max().item() <= 2 ** -6 * scale
    assert ((p1[0].float() - p0[0].float()).abs().max().item() <= 2 ** -6 * p0[0].float().abs().max().item())
    assert ss.shape == (B * T * C, mvpa_hip.load_library().mvpa_linear_sumsq_parts(B * T * C, E))
    assert torch.allclose(ss.sum(-1), h1.view(-1, E).float().pow(2).sum(-1), rtol=1e-5)
    # the statistics split over two parts per row give the same block
    with torch.no_grad():
        half = ss_in / 2
        (h2, _), _ = blk.forward_norm_fused(x, torch.cat([half, half], 1).contiguous(), pos, chan,
                                            attention_mask=mask, use_cache=True)
    assert torch.equal(h2, h1)


def test_stack_with_the_norms_inside_the_products_matches_the_norm_kernels(monkeypatch):
    """The stack forward takes the norm-fused blocks where the shapes allow; against the same
    stack with that path switched off: last hidden state to bf16 rounding."""
    import mvpa_hip
    from models.mvpformer import MVPFormerConfig, MVPFormerModel
    torch.manual_seed(12)
    cfg = MVPFormerConfig(n_positions=16, n_channels=64, n_embd=128, n_layer=3, n_head=2, n_head_kv=1, n_inner=320)
    model = MVPFormerModel(cfg).to(device="cuda", dtype=torch.bfloat16).eval()
    for n, p in model.named_parameters():
        if "ln" in n:
            p.data.copy_(1.0 + 0.2 * torch.randn_like(p))
        else:
            p.data.mul_(3.0)
    x = torch.randn(1, 16, 40, 128, device="cuda").bfloat16()
    calls = []
    orig = mvpa_hip.row_sumsq
    monkeypatch.setattr(mvpa_hip, "row_sumsq", lambda t: (calls.append(1), orig(t))[1])
    with torch.no_grad():
        a = model(inputs_embeds=x)
    assert calls, "the norm-fused path did not run"
    monkeypatch.setattr(mvpa_hip, "linear_norm_fused_supported", lambda *args: False)
    with torch.no_grad():
        b = model(inputs_embeds=x)
    assert (a.float() - b.float()).abs().max().item() <= 3e-2 * b.float().abs().max().item()
    assert ((a.float() - b.float()).norm() / b.float().norm()).item() <= 1e-2


def test_base_classification_bf16_then_fp8():
    """Base-size dims (E2048 H16 Hkv8 Dh128 n_inner5632, C=128) cut to two layers and 12 segments:
    binary-head logits in bf16 and with fp8 QK^T against the fp32 oracle stack.  Tolerances are
    this build's statement: logits within 3e-2 (bf16) and 8e-2 (fp8) of the fp32 reference in
    units of the logit spread (measured on this single window with doubled attention weights, i.e.
    unit-variance content logits: bf16 3.5e-3, fp8 5e-2 .. 6.4e-2 depending on where the other
    roundings of the forward fall)."""
    from models.configs import MVPFORMER_BASE
    from models.fftencoder import WaveEncoder
    from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead
    dims = dict(MVPFORMER_BASE, n_layer=2)
    x = make_ieeg(1, 128, 12, 512, seed=7)
    logits = {}
    for fp8 in (False, True):
        torch.manual_seed(3)
        cfg = MVPFormerConfig(**dims, fp8_qk=fp8)
        model = HMVPFormer(cfg, WaveEncoder(512, cfg.n_embd), MVPFormerHead(cfg.n_embd, 2)).to(torch.bfloat16).eval()
        for name, p in model.named_parameters():
            if "attn" in name or "embedding" in name:
                p.data.mul_(2.0)
        if not fp8:
            params = {k: v.float() for k, v in model.state_dict().items()}
            h, _ = O.mvpformer_forward(x, params, dict(n_layer=2, n_head=16, n_head_kv=8))
            ref = torch.nn.functional.linear(h[:, -1].mean(dim=1), params["head.head.weight"])
        logits[fp8] = model.cuda().classify(x.cuda()).float().cpu()
    spread = ref.abs().max().item() + 1e-6
    e16 = (logits[False] - ref).abs().max().item() / spread
    e8 = (logits[True] - ref).abs().max().item() / spread
    print(f"base-size logits: ref {ref.flatten().tolist()}, bf16 err {e16:.3e}, fp8 err {e8:.3e} (relative to spread)")
    assert e16 <= 3e-2 and e8 <= 8e-2


def test_base_classification_full_size_properties():
    """The base-size classification forward at the benchmark's full size (B1 C128 T512 segments of
    512 samples, 24 layers, Dh 128), through properties that need no oracle: finite logits,
    time-causality of the whole stack bit for bit, and the bf16 / fp8-QK^T logit gap inside the
    stated 6e-2 of the logit spread."""
    from models.configs import MVPFORMER_BASE
    from models.fftencoder import WaveEncoder
    from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead
    T, C = 512, 128
    x = make_ieeg(1, C, T, 512, seed=7).cuda()
    x2 = x.clone()
    x2[:, -40:] = x2[:, -40:].flip(-1) * 1.5
    logits = {}
    for fp8 in (False, True):
        torch.manual_seed(3)
        cfg = MVPFormerConfig(**dict(MVPFORMER_BASE, n_positions=T), fp8_qk=fp8)
        model = HMVPFormer(cfg, WaveEncoder(512, cfg.n_embd), MVPFormerHead(cfg.n_embd, 2))
        model = model.to(device="cuda", dtype=torch.bfloat16).eval()
        assert len(model.mvpformer.h) == 24
        out, _ = model._common_forward(x)
        assert out.shape == (1, T, C, 2048) and torch.isfinite(out.float()).all()
        logits[fp8] = model.classify(x).float().cpu()
        assert logits[fp8].shape == (1, 2) and torch.isfinite(logits[fp8]).all()
        if not fp8:
            out2, _ = model._common_forward(x2)
            assert torch.equal(out2[:, :-40], out[:, :-40])
            assert not torch.equal(out2[:, -40:], out[:, -40:])
            del out2
        del model, out
        torch.cuda.empty_cache()
    spread = logits[False].abs().max().item() + 1e-6
    gap = (logits[True] - logits[False]).abs().max().item() / spread
    print(f"base model, full size: logits {logits[False].flatten().tolist()}, fp8 gap {gap:.3e} of the spread")
    assert gap <= 6e-2


@pytest.mark.parametrize("flash", [True, False], ids=["flash", "masked"])
def test_layer_incremental_step_matches_full_forward(flash):
    """use_cache / layer_past: the layer run on T-1 time steps with use_cache, then on the last
    step alone with layer_past, gives the last step of the layer run on all T steps, to bf16
    rounding (the one-step projections go through the K-split GEMM, which sums in another order)."""
    from layers import MVPFormerGQAAttention, MVPFormerGQAFlashAttention
    from models.mvpformer import MVPFormerConfig
    torch.manual_seed(5)
    cfg = MVPFormerConfig(n_embd=256, n_head=4, n_head_kv=2, n_layer=1, n_positions=16, n_channels=24)
    cls = MVPFormerGQAFlashAttention if flash else MVPFormerGQAAttention
    layer = cls(cfg, layer_idx=0).to("cuda", torch.bfloat16).eval()
    B, T, C, E = 2, 11, 24, 256
    x = torch.randn(B, T, C, E, device="cuda").bfloat16()
    pos = torch.randn(1, T, E, device="cuda").bfloat16() * 0.02
    chan = torch.randn(1, C, E, device="cuda").bfloat16() * 0.02
    full = layer(x, pos, chan)[0]
    # the first T-1 steps see the last T-1 rows of the relative-time table: positions 1 .. T-1
    _, present = layer(x[:, :T - 1], pos[:, 1:], chan, use_cache=True)[:2]
    assert present[0].shape == (B, 2, T - 1, C, 64)
    step, present2 = layer(x[:, T - 1:], pos, chan, layer_past=present, use_cache=True)[:2]
    assert step.shape == (B, 1, C, E) and present2[0].shape == (B, 2, T, C, 64)
    err = (step[:, 0].float() - full[:, T - 1].float()).abs().max().item()
    assert err <= 2 ** -7 * full[:, T - 1].float().abs().max().item(), err


def _small_harness():
    from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead
    from models.fftencoder import WaveEncoder
    torch.manual_seed(9)
    cfg = MVPFormerConfig(n_embd=256, n_head=4, n_head_kv=2, n_layer=3, n_positions=12, n_channels=20,
                          n_inner=512)
    enc = WaveEncoder(size_input=512, size_output=256)
    model = HMVPFormer(cfg, enc, MVPFormerHead(256, 2)).to("cuda", torch.bfloat16).eval()
    return model, cfg


def test_stream_of_segments_matches_full_forward():
    """classify_step feeds a stream one segment at a time (encoder on the new segment, one decoding
    step per block against in-place caches).  At every step the hidden state equals the last step
    of the full forward over the segments so far with the position rows ending at max_steps, and at
    step max_steps the logits are classify() on the whole window (bf16 tolerance: the key runs of a
    decoding step are merged through bf16 partial outputs)."""
    model, cfg = _small_harness()
    B, T, C = 2, cfg.n_positions, 20
    batch = torch.randn(B, T, C, 512, device="cuda")
    past, logits = None, None
    for t in range(T):
        logits, past = model.classify_step(batch[:, t], past)
        embeds = model.encoder(batch[:, :t + 1].reshape(B * (t + 1) * C, 512)).view(B, t + 1, C, -1)
        full = model.mvpformer(inputs_embeds=embeds, position_end=T)
        head = model.head(full[:, -1].float().mean(dim=1).to(full.dtype))
        spread = head.float().abs().max().item() + 1e-3
        assert (logits.float() - head.float()).abs().max().item() <= 3e-2 * spread, t
    assert all(c.length == T for c in past)
    ref = model.classify(batch)
    assert (logits.float() - ref.float()).abs().max().item() <= 3e-2 * (ref.float().abs().max().item() + 1e-3)


def test_stream_differs_from_the_window_forward_once_the_window_bites():
    """Streams longer than 12 segments: with ONE block a streamed step still equals the last step
    of the full forward (a decoding step and the last row of the window both keep the content term
    for every key); with two or more blocks it does not - the cached keys and values of older steps
    were produced while those steps were the newest ones, with full content attention, whereas the
    window forward zeroes their content term beyond 10 steps.  The deviation is measured here so
    that the documentation's statement rests on a number."""
    from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead
    from models.fftencoder import WaveEncoder
    B, T, C = 2, 24, 12
    batch = torch.randn(B, T, C, 512, device="cuda", generator=torch.Generator("cuda").manual_seed(3))
    dev = {}
    for n_layer in (1, 3):
        torch.manual_seed(21)
        cfg = MVPFormerConfig(n_embd=256, n_head=4, n_head_kv=2, n_layer=n_layer, n_positions=T,
                              n_channels=C, n_inner=512)
        model = HMVPFormer(cfg, WaveEncoder(512, 256), MVPFormerHead(256, 2)).to("cuda", torch.bfloat16).eval()
        for name, p in model.named_parameters():
            if "attn" in name or "embedding" in name:
                p.data.mul_(3.0)                 # content logits wide enough for the window to matter
        past = None
        for t in range(T):
            logits, past = model.classify_step(batch[:, t], past)
        ref = model.classify(batch)
        dev[n_layer] = ((logits.float() - ref.float()).abs().max() / (ref.float().abs().max() + 1e-3)).item()
    print(f"stream vs window forward at T=24: 1 block {dev[1]:.3e}, 3 blocks {dev[3]:.3e} (relative to the logit spread)")
    assert dev[1] <= 3e-2
    assert dev[3] > 3e-2          # not the same function: far outside bf16 rounding


def test_stream_slides_past_the_window():
    """Past max_steps segments the oldest step leaves the caches; the buffers wrap without the
    live steps changing, and the result stays finite and close to the full forward over the last
    max_steps segments (not equal: cached hidden states of the window's first steps still carry
    what they saw of segments that have since left)."""
    from layers import MvpaKVCache
    model, cfg = _small_harness()
    B, T, C = 1, cfg.n_positions, 20
    n_seg = 3 * T + 1
    batch = torch.randn(B, n_seg, C, 512, device="cuda")
    past = None
    for t in range(n_seg):
        logits, past = model.classify_step(batch[:, t], past)
    assert all(c.length == T and c.start + c.length <= c.capacity for c in past)
    assert torch.isfinite(logits.float()).all()
    # the cache itself: appending past capacity keeps exactly the last max_steps steps, in order
    cache = MvpaKVCache(1, 1, 2, 8, max_steps=5, dtype=torch.float32, device="cuda", slack=2)
    for i in range(23):
        k, v = cache.append(torch.full((1, 1, 2, 8), float(i), device="cuda"), torch.full((1, 1, 2, 8), -float(i), device="cuda"))
        want = torch.arange(max(0, i - 4), i + 1, device="cuda", dtype=torch.float32)
        assert torch.equal(k[0, 0, :, 0, 0], want) and torch.equal(v[0, 0, :, 0, 0], -want)


def test_model_use_cache_returns_presents_like_the_reference():
    """use_cache on the stack: one (k, v) pair per block, [B,Hkv,T,C,Dh]; feeding them back with one
    more time step equals the full forward's last step when both end at the same position row."""
    model, cfg = _small_harness()
    B, T, C = 2, 7, 20
    x = torch.randn(B, T, C, 256, device="cuda").bfloat16()
    full = model.mvpformer(inputs_embeds=x, position_end=T)
    out, presents = model.mvpformer(inputs_embeds=x[:, :T - 1], use_cache=True, position_end=T)
    assert len(presents) == cfg.n_layer and presents[0][0].shape == (B, 2, T - 1, C, 64)
    step, presents2 = model.mvpformer(inputs_embeds=x[:, T - 1:], past_key_values=presents, position_end=T)
    assert presents2[0][0].shape == (B, 2, T, C, 64)
    err = (step[:, 0].float() - full[:, T - 1].float()).abs().max().item()
    assert err <= 3e-2 * full.float().abs().max().item(), err


def test_graph_replayed_stream_step_matches_eager_steps():
    """capture_stream: once the window is full, one classify_step on ring caches is captured into a
    HIP graph; every replay (with eager work of the same model between replays) gives the logits
    of the eager classify_step on the in-place caches, to bf16 rounding - the ring visits the key
    steps in another order."""
    model, cfg = _small_harness()
    B, T, C = 2, cfg.n_positions, 20
    n_more = 2 * T + 3                                   # the ring wraps more than twice
    batch = torch.randn(B, T + n_more, C, 512, device="cuda")
    past = None
    for t in range(T):
        _, past = model.classify_step(batch[:, t], past)
    step = model.capture_stream(past, batch[:, 0])
    for t in range(T, T + n_more):
        want, past = model.classify_step(batch[:, t], past)          # eager, in-place caches
        model.classify(batch[:, t - T + 1:t + 1])                    # unrelated eager work in between
        got = step(batch[:, t])
        spread = want.float().abs().max().item() + 1e-3
        assert (got.float() - want.float()).abs().max().item() <= 3e-2 * spread, t


def test_streamed_next_segment_scores_match_the_window_forward():
    """predict_step over a stream of max_steps segments gives, call by call, the columns of
    predict_next_segment on the whole window (bf16 tolerance)."""
    from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead
    from models.fftencoder import WaveEncoder
    torch.manual_seed(11)
    cfg = MVPFormerConfig(n_embd=256, n_head=4, n_head_kv=2, n_layer=2, n_positions=9, n_channels=12, n_inner=512)
    model = HMVPFormer(cfg, WaveEncoder(size_input=512, size_output=256), MVPFormerHead(256, 256)).to("cuda", torch.bfloat16).eval()
    B, T, C = 2, cfg.n_positions, 12
    batch = torch.randn(B, T, C, 512, device="cuda")
    want = model.predict_next_segment(batch)                     # [B, T-1, C]
    past, cols = None, []
    for t in range(T):
        sim, pred, past = model.predict_step(batch[:, t], past)
        assert pred.shape == (B, C, 256)
        assert (sim is None) == (t == 0)
        if sim is not None:
            cols.append(sim)
    got = torch.stack(cols, dim=1)
    # the full forward of t+1 segments predicts from rows that END at row T of the position table
    # only when t+1 == T; earlier columns see the same relative rows through position_end, so all
    # columns agree
    assert (got - want).abs().max().item() <= 3e-2


def test_graph_replayed_prediction_stream_matches_eager_steps():
    """capture_stream(predict=True): replays of predict_step on ring caches give the similarity
    and the forecast of the eager predict_step, call after call (bf16 tolerance)."""
    from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead
    from models.fftencoder import WaveEncoder
    torch.manual_seed(13)
    cfg = MVPFormerConfig(n_embd=256, n_head=4, n_head_kv=2, n_layer=2, n_positions=9, n_channels=12, n_inner=512)
    model = HMVPFormer(cfg, WaveEncoder(size_input=512, size_output=256), MVPFormerHead(256, 256)).to("cuda", torch.bfloat16).eval()
    B, T, C = 2, cfg.n_positions, 12
    batch = torch.randn(B, 3 * T, C, 512, device="cuda")
    past = None
    for t in range(T):
        _, _, past = model.predict_step(batch[:, t], past)
    step = model.capture_stream(past, batch[:, 0], predict=True)
    for t in range(T, 3 * T):
        sim_e, pred_e, past = model.predict_step(batch[:, t], past)
        sim_g, pred_g = step(batch[:, t])
        assert (sim_g - sim_e).abs().max().item() <= 3e-2, t
        assert (pred_g.float() - pred_e.float()).abs().max().item() <= 3e-2 * (pred_e.float().abs().max().item() + 1e-3), t
