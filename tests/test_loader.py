"""Checkpoint loading of the inference harness (models/mvpformer.py:470-485, 845-904): a state
dict written out under the reference's own key names and shapes - spelled here by hand from the
reference's module tree, not read off this build's modules - must load strict=True, and the
classification harness's missing/unknown-key policy must hold."""
import pytest
import torch


DIMS = dict(n_positions=14, n_channels=10, n_embd=64, n_layer=2, n_head=4, n_head_kv=2, n_inner=96,
            lora=True, lora_rank=4, lora_alpha=16)
SEG = 128


def reference_state_dict(dims=DIMS, seg=SEG, head_out=2, seed=0, std=0.05):
    """Keys of HMVPFormer.state_dict() in the reference: MVPFormerModel (models/mvpformer.py:155-177:
    h.N.{ln_1, attn, ln_2, mlp}, ln_f, positional_embedding, channel_embedding), the attention
    layer's parameters and persistent buffers (layers/mvpa.py:17-23, 43-84; the adapter library
    adds lora_A [r, in] and lora_B [out_slice, r] to q_attn and to the value half of c_attn), the
    gated MLP (gate/up/down_proj), WaveEncoder (models/fftencoder.py:67-68: ln, proj),
    MVPFormerHead (models/mvpformer.py:979-984: head.head) and seizure_embeddings (:438-445)."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *shape: torch.randn(*shape, generator=g) * std      # noqa: E731
    E, P, L, r = dims["n_embd"], dims["n_positions"], dims["n_layer"], dims["lora_rank"]
    kv = E // dims["n_head"] * dims["n_head_kv"]
    inner = dims["n_inner"]
    n, dwt = seg, 0
    import math
    sizes = []
    for _ in range(int(math.floor(math.log2(seg / 7)))):
        n = (n + 7) // 2
        sizes.append(n)
    dwt = sum(sizes) + sizes[-1]
    sd = {}
    for i in range(L):
        pre = f"mvpformer.h.{i}."
        sd[pre + "ln_1.weight"] = 1 + rn(E)
        sd[pre + "attn.time_bias"] = torch.tril(torch.ones(P, P, dtype=torch.bool)).view(1, 1, P, P)
        sd[pre + "attn.masked_bias"] = torch.tensor(-1e4)
        sd[pre + "attn.q_attn.weight"] = rn(E, E)
        sd[pre + "attn.c_attn.weight"] = rn(2 * kv, E)
        if dims.get("lora"):
            sd[pre + "attn.q_attn.lora_A"] = rn(r, E)
            sd[pre + "attn.q_attn.lora_B"] = rn(E, r)
            sd[pre + "attn.c_attn.lora_A"] = rn(r, E)
            sd[pre + "attn.c_attn.lora_B"] = rn(kv, r)
        sd[pre + "attn.position_net.weight"] = rn(kv, E)
        sd[pre + "attn.channel_net.weight"] = rn(kv, E)
        sd[pre + "attn.c_proj.weight"] = rn(E, E)
        sd[pre + "attn.attn_bias"] = rn(3 * kv)
        sd[pre + "ln_2.weight"] = torch.ones(E)
        sd[pre + "mlp.gate_proj.weight"] = rn(inner, E)
        sd[pre + "mlp.up_proj.weight"] = rn(inner, E)
        sd[pre + "mlp.down_proj.weight"] = rn(E, inner)
    sd["mvpformer.ln_f.weight"] = 1 + rn(E)
    sd["mvpformer.positional_embedding.weight"] = rn(P, E)
    sd["mvpformer.channel_embedding.weight"] = rn(dims["n_channels"], E)
    sd["encoder.ln.weight"] = 1 + rn(dwt)
    sd["encoder.proj.weight"] = rn(E, dwt)
    sd["head.head.weight"] = rn(head_out, E)
    sd["seizure_embeddings"] = rn(3, seg)
    return sd


def _model(cls_name="HMVPFormer", head_out=2, **over):
    import models.mvpformer as M
    from models.fftencoder import WaveEncoder
    dims = dict(DIMS, **over)
    cfg = M.MVPFormerConfig(**dims)
    cls = getattr(M, cls_name)
    return cls(cfg, WaveEncoder(SEG, cfg.n_embd), M.MVPFormerHead(cfg.n_embd, head_out))


def test_reference_state_dict_loads_strict():
    sd = reference_state_dict()
    model = _model()
    assert sorted(model.state_dict().keys()) == sorted(sd.keys())
    for k, v in model.state_dict().items():
        assert v.shape == sd[k].shape, k
    model.load_reference_state_dicts(sd)
    got = model.state_dict()
    for k, v in sd.items():
        if k == "encoder.ln.weight":                      # reset on load, models/mvpformer.py:483
            assert torch.equal(got[k], torch.ones_like(v))
        else:
            assert torch.equal(got[k], v), k
    # strict: a missing or an unknown key is an error
    bad = dict(sd)
    del bad["mvpformer.h.1.attn.c_attn.lora_B"]
    with pytest.raises(RuntimeError):
        _model().load_reference_state_dicts(bad)
    bad = dict(sd, extra=torch.zeros(1))
    with pytest.raises(RuntimeError):
        _model().load_reference_state_dicts(bad)


def test_base_model_path_argument(tmp_path):
    """base_model= names a file that is read with torch.load(weights_only=True) at construction
    (models/mvpformer.py:470-479); a path that does not exist loads nothing."""
    sd = reference_state_dict(seed=3)
    path = tmp_path / "base.pt"
    torch.save(sd, path)
    import models.mvpformer as M
    from models.fftencoder import WaveEncoder
    cfg = M.MVPFormerConfig(**DIMS)
    model = M.HMVPFormer(cfg, WaveEncoder(SEG, cfg.n_embd), M.MVPFormerHead(cfg.n_embd, 2), base_model=str(path))
    assert torch.equal(model.state_dict()["mvpformer.h.0.attn.attn_bias"], sd["mvpformer.h.0.attn.attn_bias"])
    M.HMVPFormer(cfg, WaveEncoder(SEG, cfg.n_embd), M.MVPFormerHead(cfg.n_embd, 2),
                 base_model=str(tmp_path / "absent.pt"))


def test_classification_checkpoint_policy():
    base = reference_state_dict(head_out=DIMS["n_embd"], seed=1)      # generative base: E -> E head
    for k in [k for k in base if "lora" in k]:
        del base[k]                                                    # pre-trained without adapters
    model = _model("ClassificationHMVPFormer")
    fresh_head = model.head.head.weight.clone()
    model.load_reference_state_dicts(base)
    assert torch.equal(model.head.head.weight, fresh_head)             # head of another shape: dropped
    assert torch.equal(model.mvpformer.h[1].attn.c_proj.weight, base["mvpformer.h.1.attn.c_proj.weight"])
    # a base that lacks a frozen weight is refused; so is one with an unknown key
    bad = dict(base)
    del bad["mvpformer.h.0.mlp.up_proj.weight"]
    with pytest.raises(AttributeError, match="missing from the base model"):
        _model("ClassificationHMVPFormer").load_reference_state_dicts(bad)
    with pytest.raises(AttributeError, match="unknown in the base model"):
        _model("ClassificationHMVPFormer").load_reference_state_dicts(dict(base, stray=torch.zeros(2)))
    # head state dict: head + adapters, class_loss.weight tolerated
    full = reference_state_dict(seed=2)
    head_sd = {k: v for k, v in full.items() if "lora" in k or k.startswith("head.")}
    head_sd["class_loss.weight"] = torch.ones(2)
    model.load_reference_state_dicts(None, head_sd)
    assert torch.equal(model.head.head.weight, full["head.head.weight"])
    assert torch.equal(model.mvpformer.h[0].attn.q_attn.lora_B, full["mvpformer.h.0.attn.q_attn.lora_B"])
    partial = {k: v for k, v in head_sd.items() if "q_attn.lora_A" not in k}
    with pytest.raises(AttributeError, match="missing from the head model"):
        _model("ClassificationHMVPFormer").load_reference_state_dicts(None, partial)
    with pytest.raises(AttributeError, match="unknown in the model"):
        _model("ClassificationHMVPFormer").load_reference_state_dicts(None, dict(head_sd, other=torch.zeros(1)))
    # without adapters every base key is needed
    plain = reference_state_dict(dims=dict(DIMS, lora=False), seed=4)
    m2 = _model("ClassificationHMVPFormer", lora=False)
    m2.load_reference_state_dicts(plain)
    del plain["mvpformer.ln_f.weight"]
    with pytest.raises(AttributeError, match="missing from the base model"):
        _model("ClassificationHMVPFormer", lora=False).load_reference_state_dicts(plain)


@pytest.mark.gpu
def test_loaded_model_forward_matches_oracle_stack():
    """A model that got its weights from a reference-shaped state dict computes what the oracle
    stack computes from that same state dict (adapters merged as W + alpha/r * B A)."""
    from mvpa_hip.synthetic import make_ieeg
    from oracle import mvpa_oracle as O
    sd = reference_state_dict(seed=7, std=0.08)
    sd = {k: (v.bfloat16().float() if v.is_floating_point() else v) for k, v in sd.items()}
    model = _model().load_reference_state_dicts(sd).to("cuda", torch.bfloat16).eval()
    x = make_ieeg(2, 10, 14, SEG, seed=3)
    params = dict(sd)
    params["encoder.ln.weight"] = torch.ones_like(sd["encoder.ln.weight"])
    r, alpha = DIMS["lora_rank"], DIMS["lora_alpha"]
    kv = DIMS["n_embd"] // DIMS["n_head"] * DIMS["n_head_kv"]
    for i in range(DIMS["n_layer"]):
        pre = f"mvpformer.h.{i}.attn."
        params[pre + "q_attn.weight"] = sd[pre + "q_attn.weight"] + (alpha / r) * sd[pre + "q_attn.lora_B"] @ sd[pre + "q_attn.lora_A"]
        w = sd[pre + "c_attn.weight"].clone()
        w[kv:] += (alpha / r) * sd[pre + "c_attn.lora_B"] @ sd[pre + "c_attn.lora_A"]    # value half only
        params[pre + "c_attn.weight"] = w
    ref, _ = O.mvpformer_forward(x, params, dict(n_layer=DIMS["n_layer"], n_head=4, n_head_kv=2))
    out, _ = model._common_forward(x.cuda())
    rel = ((out.float().cpu() - ref).norm() / ref.norm()).item()
    assert rel <= 3e-2, rel
