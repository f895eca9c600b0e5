"""Pins the layer-, encoder- and stack-level functions of the CPU oracle (oracle/mvpa_oracle.py)
without the GPU, each against a statement that shares no code with it: library routines
(torch.nn.functional.rms_norm, torch.nn.RMSNorm, torch.nn.Linear, torch.nn.Embedding,
transformers' LlamaMLP) and explicit index sums (einsum over named head/time/channel axes, the
float64 brute-force operator).  A swapped K/V half of c_attn, a wrong permute in split/merge
heads, eps outside the root, ln_2 applied before the MLP, or a sequential instead of a parallel
block each fail at least one test here."""
import math

import pytest
import torch

from oracle import mvpa_oracle as O

F = torch.nn.functional


def _gen(seed):
    return torch.Generator().manual_seed(seed)


# --------------------------------------------------------------------------------------
# rmsnorm  (models/mvpformer.py:108, 133; models/fftencoder.py:66, 93)
# --------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 0.0)])
def test_rmsnorm_matches_library(dtype, tol):
    """O.rmsnorm == torch.nn.functional.rms_norm == torch.nn.RMSNorm (eps 1e-5 INSIDE the root,
    mean over the last axis, weight applied after the normalisation).  bf16: the library computes
    in fp32 and rounds once, as the reference's fused RMSNorm does; compared after one more
    rounding step of slack (0 or 1 ulp)."""
    g = _gen(3)
    x = (torch.randn(7, 5, 96, generator=g) * 3.0 + 0.5).to(dtype)
    w = (1.0 + 0.3 * torch.randn(96, generator=g)).to(dtype)
    got = O.rmsnorm(x, w, 1e-5)
    assert got.dtype == dtype
    want = F.rms_norm(x.float(), (96,), w.float(), 1e-5)
    mod = torch.nn.RMSNorm(96, eps=1e-5)
    with torch.no_grad():
        mod.weight.copy_(w.float())
        want2 = mod(x.float())
    assert torch.allclose(want, want2, atol=1e-6)
    if dtype == torch.float32:
        assert (got - want).abs().max().item() <= tol
    else:
        # one bf16 ulp at most (the oracle rounds the fp32 result once)
        assert (got.float() - want).abs().max().item() <= want.abs().max().item() * 2 ** -8
    # eps matters and sits inside the root: a tiny-norm row must come out as x / sqrt(eps)
    tiny = torch.full((1, 96), 1e-6)
    assert torch.allclose(O.rmsnorm(tiny, torch.ones(96), 1e-5), tiny / math.sqrt(1e-12 + 1e-5), rtol=1e-5)


# --------------------------------------------------------------------------------------
# split_heads / merge_heads / attention_layer_forward  (layers/mvpa.py:161-171, 280-337)
# --------------------------------------------------------------------------------------

def test_split_and_merge_heads_by_explicit_index():
    """split_heads puts feature h*Dh + d of token (b, t, c) at [b, h, t, c, d]
    (layers/mvpa.py:161-166); merge_heads is its inverse (layers/mvpa.py:168-171)."""
    B, T, C, H, Dh = 2, 3, 4, 5, 6
    x = torch.arange(B * T * C * H * Dh, dtype=torch.float32).view(B, T, C, H * Dh)
    y = O.split_heads(x, H, Dh)
    assert y.shape == (B, H, T, C, Dh)
    for (b, h, t, c, d) in [(0, 0, 0, 0, 0), (1, 4, 2, 3, 5), (0, 2, 1, 3, 4), (1, 0, 2, 0, 1)]:
        assert y[b, h, t, c, d].item() == x[b, t, c, h * Dh + d].item()
    assert torch.equal(O.merge_heads(y, H, Dh), x)


def _layer_weights(E, kvE, g, std=0.3):
    mk = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * std  # noqa: E731
    return {"q_attn.weight": mk(E, E), "c_attn.weight": mk(2 * kvE, E),
            "position_net.weight": mk(kvE, E), "channel_net.weight": mk(kvE, E),
            "c_proj.weight": mk(E, E), "attn_bias": mk(3 * kvE)}


def _layer_by_einsum(hidden, pos, chan, w, H, Hkv, *, window=10, chan_valid=None):
    """MVPFormerGQAAttention.forward (layers/mvpa.py:280-337) written without split/merge helpers:
    every projection is an einsum into explicitly named (head, dim) axes, the attention operator
    is the float64 brute force over tokens n = t*C + c, and the output projection contracts
    (head, dim) against c_proj's input axis h*Dh + d."""
    B, T, C, E = hidden.shape
    Dh = E // H
    kvE = Hkv * Dh
    wq = w["q_attn.weight"].view(H, Dh, E)
    wk = w["c_attn.weight"][:kvE].view(Hkv, Dh, E)          # first half of c_attn is K (:309)
    wv = w["c_attn.weight"][kvE:].view(Hkv, Dh, E)          # second half is V
    q = torch.einsum("btce,hde->bhtcd", hidden, wq).reshape(B, H, T * C, Dh)
    k = torch.einsum("btce,gde->bgtcd", hidden, wk).reshape(B, Hkv, T * C, Dh)
    v = torch.einsum("btce,gde->bgtcd", hidden, wv).reshape(B, Hkv, T * C, Dh)
    k_time = torch.einsum("te,gde->gtd", pos[0], w["position_net.weight"].view(Hkv, Dh, E))
    k_chan = torch.einsum("ce,gde->gcd", chan[0], w["channel_net.weight"].view(Hkv, Dh, E))
    u, vb, z = [w["attn_bias"][i * kvE:(i + 1) * kvE].view(Hkv, Dh) for i in range(3)]  # :185-187
    o = O.mvpa_bruteforce(q, k, v, u, vb, z, k_time, k_chan, window=window, chan_valid=chan_valid)
    o = o.view(B, H, T, C, Dh)
    return torch.einsum("bhtcd,ehd->btce", o, w["c_proj.weight"].view(E, H, Dh))


@pytest.mark.parametrize("H,Hkv,T,C,window", [(4, 2, 5, 3, 10), (2, 2, 13, 2, 3), (6, 2, 4, 4, 10)])
def test_attention_layer_forward_matches_einsum_statement(H, Hkv, T, C, window):
    """O.attention_layer_forward against the einsum + brute-force statement (float64, <= 1e-10).
    V is drawn from a different distribution than K through a c_attn whose halves differ in
    scale, so a swapped split fails; H != T != C so a wrong permute changes the shape or the
    values."""
    g = _gen(11 * H + T)
    B, Dh = 2, 4
    E = H * Dh
    w = _layer_weights(E, Hkv * Dh, g)
    w["c_attn.weight"][Hkv * Dh:] *= 3.0
    hidden = torch.randn(B, T, C, E, generator=g, dtype=torch.float64)
    pos = torch.randn(1, T, E, generator=g, dtype=torch.float64)
    chan = torch.randn(1, C, E, generator=g, dtype=torch.float64)
    got = O.attention_layer_forward(hidden, pos, chan, w, H, Hkv, window=window)
    want = _layer_by_einsum(hidden, pos, chan, w, H, Hkv, window=window)
    assert got.shape == want.shape == (B, T, C, E)
    assert (got - want).abs().max().item() <= 1e-10
    # the swapped split is a different function (the test has teeth)
    sw = dict(w)
    kvE = Hkv * Dh
    sw["c_attn.weight"] = torch.cat([w["c_attn.weight"][kvE:], w["c_attn.weight"][:kvE]])
    assert (O.attention_layer_forward(hidden, pos, chan, sw, H, Hkv, window=window) - want).abs().max().item() > 1e-3


def test_attention_layer_forward_with_additive_mask():
    """The additive key mask of models/mvpformer.py:262-268, (1 - m) * finfo.min over [B,1,1,N],
    is the channel-validity mask when m[b, t*C + c] = valid[b, c]: the layer must then equal the
    einsum statement with those keys left out."""
    g = _gen(5)
    B, H, Hkv, T, C, Dh = 2, 4, 2, 4, 5, 4
    E = H * Dh
    w = _layer_weights(E, Hkv * Dh, g)
    hidden = torch.randn(B, T, C, E, generator=g, dtype=torch.float64)
    pos = torch.randn(1, T, E, generator=g, dtype=torch.float64)
    chan = torch.randn(1, C, E, generator=g, dtype=torch.float64)
    valid = torch.tensor([[1, 0, 1, 1, 0], [1, 1, 1, 0, 1]], dtype=torch.bool)
    m = valid[:, None, :].expand(B, T, C).reshape(B, T * C).double()
    am = (1.0 - m)[:, None, None, :] * torch.finfo(torch.float64).min
    got = O.attention_layer_forward(hidden, pos, chan, w, H, Hkv, attention_mask=am)
    want = _layer_by_einsum(hidden, pos, chan, w, H, Hkv, chan_valid=valid)
    assert (got - want).abs().max().item() <= 1e-10


# --------------------------------------------------------------------------------------
# wave_encoder_forward  (models/fftencoder.py:80-97)
# --------------------------------------------------------------------------------------

def _wavedec_pad_conv(x):
    """ptwt.wavedec(x, db4, mode="periodic") by its published algorithm with torch's pad and
    conv1d (circular pad 6 left, 6 + n % 2 right; stride-2 cross-correlation with the flipped
    decomposition filters; floor(log2(n / 7)) levels; [cA_L, cD_L .. cD_1])."""
    lo = torch.tensor(O.DB4_DEC_LO, dtype=x.dtype).flip(0)
    hi = torch.tensor(O.DB4_DEC_HI, dtype=x.dtype).flip(0)
    filt = torch.stack([lo, hi])[:, None, :]
    a = x[:, None, :]
    details = []
    for _ in range(int(math.floor(math.log2(x.shape[-1] / 7)))):
        n = a.shape[-1]
        res = F.conv1d(F.pad(a, (6, 6 + n % 2), mode="circular"), filt, stride=2)
        a, d = res[:, :1], res[:, 1]
        details.append(d)
    return torch.cat([a[:, 0]] + details[::-1], dim=-1)


class _EncoderByModules(torch.nn.Module):
    """WaveEncoder as the reference wires it (models/fftencoder.py:66-67, 90-97): coefficients,
    RMSNorm(dwt_size, eps 1e-5), cast to the input dtype, bias-free Linear."""

    def __init__(self, size_input, size_output):
        super().__init__()
        dwt = sum(O.dwt_sizes(size_input))
        self.ln = torch.nn.RMSNorm(dwt, eps=1e-5)
        self.proj = torch.nn.Linear(dwt, size_output, bias=False)

    def forward(self, x):
        return self.proj(self.ln(_wavedec_pad_conv(x.float())).type(x.dtype))


@pytest.mark.parametrize("L", [512, 97])
def test_wave_encoder_forward_matches_module_composition(L):
    torch.manual_seed(L)
    enc = _EncoderByModules(L, 24)
    with torch.no_grad():
        enc.ln.weight.copy_(1.0 + 0.2 * torch.randn_like(enc.ln.weight))
        x = torch.randn(6, L)
        want = enc(x)
        got = O.wave_encoder_forward(x, enc.ln.weight, enc.proj.weight)
    assert got.shape == want.shape == (6, 24)
    assert (got - want).abs().max().item() <= 2e-5


# --------------------------------------------------------------------------------------
# the MLP lines and the whole stack  (models/mvpformer.py:104-152, 246-283, 380, 596-607)
# --------------------------------------------------------------------------------------

def _llama_mlp(E, inner):
    from transformers.models.llama.configuration_llama import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaMLP
    cfg = LlamaConfig(hidden_size=E, intermediate_size=inner, hidden_act="silu", mlp_bias=False,
                      pretraining_tp=1, num_attention_heads=1, num_key_value_heads=1)
    return LlamaMLP(cfg)


class _AttnByModules(torch.nn.Module):
    """The attention layer as bias-free torch.nn.Linear modules around the einsum-free torch
    operator: q/k/v in [B, heads, N, Dh] by reshape-then-transpose of the token axis (a different
    route from the oracle's 5-D permute), scored by the closed-form operator O.mvpa_direct (pinned
    on its own in tests/test_oracle.py)."""

    def __init__(self, E, H, Hkv):
        super().__init__()
        self.H, self.Hkv, self.Dh = H, Hkv, E // H
        kvE = Hkv * self.Dh
        self.q_attn = torch.nn.Linear(E, E, bias=False)
        self.c_attn = torch.nn.Linear(E, 2 * kvE, bias=False)
        self.position_net = torch.nn.Linear(E, kvE, bias=False)
        self.channel_net = torch.nn.Linear(E, kvE, bias=False)
        self.c_proj = torch.nn.Linear(E, E, bias=False)
        self.attn_bias = torch.nn.Parameter(torch.zeros(3 * kvE))

    def forward(self, x, pos, chan, chan_valid=None):
        B, T, C, E = x.shape
        H, Hkv, Dh = self.H, self.Hkv, self.Dh
        tok = x.reshape(B, T * C, E)
        q = self.q_attn(tok).reshape(B, T * C, H, Dh).transpose(1, 2)
        kv = self.c_attn(tok)
        k = kv[..., :Hkv * Dh].reshape(B, T * C, Hkv, Dh).transpose(1, 2)
        v = kv[..., Hkv * Dh:].reshape(B, T * C, Hkv, Dh).transpose(1, 2)
        kt = self.position_net(pos[0]).reshape(T, Hkv, Dh).transpose(0, 1)
        kc = self.channel_net(chan[0]).reshape(C, Hkv, Dh).transpose(0, 1)
        u, vb, z = self.attn_bias.reshape(3, Hkv, Dh)
        o = O.mvpa_direct(q, k, v, u, vb, z, kt, kc, chan_valid=chan_valid, dtype=x.dtype)
        return self.c_proj(o.transpose(1, 2).reshape(B, T, C, E))


class _StackByModules(torch.nn.Module):
    """Encoder -> embeddings -> parallel blocks -> ln_f out of library modules, wired as the
    reference states it: both branches of a block read ln_1(x), ln_2 exists and is never applied
    (models/mvpformer.py:104-147), positions and channels are the first T / C rows of the two
    embedding tables (:246-261, 282-283), ln_f closes the stack (:380)."""

    def __init__(self, cfg, L):
        super().__init__()
        E = cfg["n_embd"]
        self.encoder = _EncoderByModules(L, E)
        self.positional_embedding = torch.nn.Embedding(cfg["n_positions"], E)
        self.channel_embedding = torch.nn.Embedding(cfg["n_channels"], E)
        self.h = torch.nn.ModuleList()
        for _ in range(cfg["n_layer"]):
            blk = torch.nn.Module()
            blk.ln_1 = torch.nn.RMSNorm(E, eps=cfg["layer_norm_epsilon"])
            blk.ln_2 = torch.nn.RMSNorm(E, eps=cfg["layer_norm_epsilon"])
            blk.attn = _AttnByModules(E, cfg["n_head"], cfg["n_head_kv"])
            blk.mlp = _llama_mlp(E, cfg["n_inner"])
            self.h.append(blk)
        self.ln_f = torch.nn.RMSNorm(E, eps=cfg["layer_norm_epsilon"])

    def forward(self, x, chan_valid=None):
        B, T, C, L = x.shape
        embeds = self.encoder(x.reshape(B * T * C, L)).view(B, T, C, -1)
        pos = self.positional_embedding(torch.arange(T))[None]
        chan = self.channel_embedding(torch.arange(C))[None]
        h = embeds
        for blk in self.h:
            residual = h
            hn = blk.ln_1(h)
            h = residual + blk.mlp(hn) + blk.attn(hn, pos, chan, chan_valid)
        return self.ln_f(h), embeds


def _oracle_params(model):
    """The module composition's weights under the reference's state-dict names."""
    p = {"encoder.ln.weight": model.encoder.ln.weight, "encoder.proj.weight": model.encoder.proj.weight,
         "mvpformer.positional_embedding.weight": model.positional_embedding.weight,
         "mvpformer.channel_embedding.weight": model.channel_embedding.weight,
         "mvpformer.ln_f.weight": model.ln_f.weight}
    for i, blk in enumerate(model.h):
        pre = f"mvpformer.h.{i}."
        p[pre + "ln_1.weight"] = blk.ln_1.weight
        p[pre + "ln_2.weight"] = blk.ln_2.weight
        for n in ("q_attn", "c_attn", "position_net", "channel_net", "c_proj"):
            p[pre + f"attn.{n}.weight"] = getattr(blk.attn, n).weight
        p[pre + "attn.attn_bias"] = blk.attn.attn_bias
        for n in ("gate_proj", "up_proj", "down_proj"):
            p[pre + f"mlp.{n}.weight"] = getattr(blk.mlp, n).weight
    return {k: v.detach() for k, v in p.items()}


def test_mlp_lines_match_llama_mlp():
    """The three MLP lines of O.mvpformer_forward are transformers' LlamaMLP with mlp_bias=False
    (models/mvpformer.py:114, 146): a stack with the attention output projection zeroed and
    ln_f = identity weights leaves rmsnorm(x + mlp(ln_1(x)))."""
    torch.manual_seed(0)
    E, inner = 16, 40
    mlp = _llama_mlp(E, inner).double()
    x = torch.randn(3, 5, E, dtype=torch.float64)
    with torch.no_grad():
        want = mlp(x)
    lin = F.linear
    got = lin(F.silu(lin(x, mlp.gate_proj.weight)) * lin(x, mlp.up_proj.weight), mlp.down_proj.weight)
    assert torch.allclose(got, want, atol=1e-12)        # the formula the oracle's three lines spell
    # and through the oracle itself: one block whose attention branch is switched off
    cfg = dict(n_embd=E, n_inner=inner, n_layer=1, n_head=4, n_head_kv=2, n_positions=8,
               n_channels=8, layer_norm_epsilon=1e-5)
    model = _StackByModules(cfg, 64).double()
    with torch.no_grad():
        model.h[0].attn.c_proj.weight.zero_()
        model.h[0].mlp.load_state_dict(mlp.state_dict())
        xs = torch.randn(1, 3, 2, 64, dtype=torch.float64)
        out, emb = O.mvpformer_forward(xs, _oracle_params(model), cfg)
        hn = F.rms_norm(emb, (E,), model.h[0].ln_1.weight, 1e-5)
        want = F.rms_norm(emb + mlp(hn), (E,), model.ln_f.weight, 1e-5)
    assert (out - want).abs().max().item() <= 2e-6      # the oracle's norms compute in fp32


@pytest.mark.parametrize("masked", [False, True])
def test_mvpformer_forward_matches_module_composition(masked):
    """O.mvpformer_forward == the composition of library modules (float64 weights, <= 1e-8 on
    unit-scale outputs).  Norm weights, ln_2 included, are drawn away from 1 so that a misplaced
    or extra norm shows; embedding tables are longer than T and C so that the row slices matter."""
    torch.manual_seed(7)
    cfg = dict(n_embd=24, n_inner=40, n_layer=3, n_head=6, n_head_kv=2, n_positions=9,
               n_channels=7, layer_norm_epsilon=1e-5)
    B, T, C, L = 2, 6, 4, 97
    model = _StackByModules(cfg, L).double()
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("ln.weight") or ".ln_" in name or name.startswith("ln_f"):
                p.copy_(1.0 + 0.3 * torch.randn_like(p))
            elif "attn_bias" in name:
                p.copy_(0.2 * torch.randn_like(p))
            elif p.dim() == 2:
                p.copy_(torch.randn_like(p) * (1.5 / math.sqrt(p.shape[1])))
        x = torch.randn(B, T, C, L, dtype=torch.float64)
        valid = torch.tensor([[1, 1, 0, 1], [0, 1, 1, 1]], dtype=torch.bool) if masked else None
        want, want_emb = model(x, valid)
        am = None
        if masked:     # models/mvpformer.py:262-268 takes a 0/1 mask over the B x (T*C) tokens
            am = valid[:, None, :].expand(B, T, C).reshape(B, T * C).double()
        got, got_emb = O.mvpformer_forward(x, _oracle_params(model), cfg, attention_mask=am)
    assert got.shape == want.shape == (B, T, C, cfg["n_embd"])
    assert (got_emb - want_emb).abs().max().item() <= 1e-5      # DWT runs in fp32 in both
    # the oracle's norms and DWT compute in fp32, the module composition's norms in float64
    assert (got - want).abs().max().item() <= 2e-4
    # teeth: a sequential block (MLP reading ln_2(x + attn)) is a different function
    with torch.no_grad():
        h = want_emb
        pos = model.positional_embedding(torch.arange(T))[None]
        chan = model.channel_embedding(torch.arange(C))[None]
        for blk in model.h:
            a = h + blk.attn(blk.ln_1(h), pos, chan, valid)
            h = a + blk.mlp(blk.ln_2(a))
        seq = model.ln_f(h)
    assert (seq - want).abs().max().item() > 1e-2
