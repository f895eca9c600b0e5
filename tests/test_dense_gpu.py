"""GPU checks of the dense ops behind the C ABI (linear, RMSNorm, residual add, db4 DWT)."""
import pytest
import torch

import mvpa_hip
from oracle import mvpa_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 200, 72), (1000, 768, 550), (64, 2304, 768), (17, 33, 8),
                                   (2048, 768, 768), (1024, 1280, 768), (600, 130, 72), (4100, 2048, 552),
                                   (16384, 768, 1728),
                                   # tile rows a multiple of 32: the XCD-aware tile order, with ragged N and a K tail
                                   (8192, 1000, 200), (16384, 520, 72),
                                   # K a multiple of 64: the 64-wide two-stage kernel, ragged rows and columns, two k-blocks only
                                   (600, 130, 128), (1000, 200, 192), (5000, 333, 256), (513, 257, 1024),
                                   # at most 128 rows: the K-split kernel of a decoding step
                                   (64, 1280, 768), (64, 768, 1728), (33, 130, 550), (1, 768, 768), (20, 100, 72),
                                   (32, 2048, 5632), (128, 2048, 2048), (100, 3072, 2048), (65, 96, 24)])
def test_linear_bf16(M, N, K):
    g = torch.Generator().manual_seed(M + N + K)
    ldk = (K + 7) // 8 * 8
    x = torch.zeros(M, ldk).bfloat16()
    w = torch.zeros(N, ldk).bfloat16()
    x[:, :K] = torch.randn(M, K, generator=g).bfloat16()
    w[:, :K] = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    # poison the padding: it must not be read as data
    xg, wg = x.cuda(), w.cuda()
    y = mvpa_hip.linear(xg[:, :K], wg[:, :K]).float().cpu()
    ref = x[:, :K].double() @ w[:, :K].double().T
    # fp32 accumulation, one bf16 rounding at the end: rel error <= 2^-8
    assert (y.double() - ref).abs().max().item() <= 2 ** -8 * ref.abs().max().item() + 1e-6


@pytest.mark.parametrize("M,N,K", [(200, 96, 64), (1024, 1728, 768), (700, 200, 136), (4096, 64, 768),
                                   (64, 1728, 768), (20, 70, 136), (40, 33, 552), (7, 5632, 2048), (128, 5632, 2048), (97, 40, 72),
                                   (8192, 300, 136),       # the XCD-aware tile order
                                   (700, 200, 128), (2100, 70, 320)])   # the 64-wide two-stage kernel, ragged
def test_linear_gated(M, N, K):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(2 * N, K, generator=g) * 0.2).bfloat16()
    y = mvpa_hip.linear(x.cuda(), w.cuda(), gated=True).float().cpu()
    gate = x.double() @ w[:N].double().T
    up = x.double() @ w[N:].double().T
    ref = torch.nn.functional.silu(gate) * up
    assert (y.double() - ref).abs().max().item() <= 2 ** -7 * ref.abs().max().item() + 1e-5


@pytest.mark.parametrize("M,N,K", [(1024, 768, 2496), (16384, 768, 2496), (600, 130, 96), (4096, 2048, 7680),
                                   (2000, 200, 160), (8192, 520, 256)])
def test_linear_with_residual_in_the_epilogue(M, N, K):
    """y = x w^T + r against float64 (fp32 accumulation, the product rounded to bf16, the sum with r
    rounded once more: 2^-8 of the product's range + 2^-8 of the sum's), with the operands as
    column slices of wider buffers (row pitches that are not the row lengths) and r odd-pitched."""
    g = torch.Generator().manual_seed(M + N + K)
    xw = torch.randn(M, K + 64, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    rw = torch.randn(M, N + 3, generator=g).bfloat16()
    xg, rg = xw.cuda(), rw.cuda()
    y = mvpa_hip.linear(xg[:, 32:32 + K], w.cuda(), residual=rg[:, :N]).float().cpu()
    prod = xw[:, 32:32 + K].double() @ w.double().T
    ref = prod + rw[:, :N].double()
    tol = 2 ** -8 * prod.abs().max().item() + 2 ** -8 * ref.abs().max().item() + 1e-6
    assert (y.double() - ref).abs().max().item() <= tol
    # into a view of a wider output, in place over the residual
    wide = torch.zeros(M, N + 40, dtype=torch.bfloat16, device="cuda")
    wide[:, 8:8 + N] = rg[:, :N]
    mvpa_hip.linear(xg[:, 32:32 + K], w.cuda(), residual=wide[:, 8:8 + N], out=wide[:, 8:8 + N])
    assert torch.equal(wide[:, 8:8 + N].float().cpu(), y)
    assert wide[:, :8].abs().max().item() == 0 and wide[:, 8 + N:].abs().max().item() == 0


def test_linear_with_residual_refuses_small_shapes():
    x = torch.zeros(64, 768, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(768, 768, dtype=torch.bfloat16, device="cuda")
    assert not mvpa_hip.linear_residual_supported(64, 768)
    with pytest.raises(mvpa_hip.MvpaError):
        mvpa_hip.linear(x, w, residual=x)


@pytest.mark.parametrize("B,T,C,E", [(4, 64, 64, 768), (1, 2, 3, 8), (2, 5, 7, 1032), (3, 1, 4, 64)])
def test_cosine_similarity_of_consecutive_steps(B, T, C, E):
    """The generative score in one kernel against torch.cosine_similarity on the fp32 values."""
    g = torch.Generator().manual_seed(B * T + C)
    a = torch.randn(B, T, C, E, generator=g).bfloat16()
    b = (torch.randn(B, T, C, E, generator=g) * 3).bfloat16()
    b[0, 0, 0] = 0                                   # a zero row: eps keeps it finite
    out = mvpa_hip.cosine_similarity_steps(a.cuda(), b.cuda()).cpu()
    assert out.shape == (B, T - 1, C) and out.dtype == torch.float32
    if T > 1:
        ref = torch.cosine_similarity(a[:, 1:].double(), b[:, :-1].double(), dim=-1)
        assert torch.isfinite(out).all()
        assert (out.double() - ref).abs().max().item() <= 2e-6


@pytest.mark.parametrize("M,N0,N1,K", [(16384, 1280, 1728, 768), (1024, 520, 300, 128), (600, 192, 64, 192),
                                       (4096, 4096, 5632, 2048)])
def test_two_products_of_one_launch_equal_the_separate_ones(M, N0, N1, K):
    """mvpa_linear_bf16_dual against the two single launches, bit for bit (same kernels' tiles),
    with the gated output a column slice of a wider buffer."""
    g = torch.Generator().manual_seed(M + N0 + N1 + K)
    x = torch.randn(M, K, generator=g).bfloat16().cuda()
    w0 = (torch.randn(N0, K, generator=g) * 0.05).bfloat16().cuda()
    w1 = (torch.randn(2 * N1, K, generator=g) * 0.05).bfloat16().cuda()
    wide = torch.full((M, N1 + 72), 3.0, dtype=torch.bfloat16, device="cuda")
    y0, y1 = mvpa_hip.linear_dual(x, w0, w1, out_gated=wide[:, 8:8 + N1])
    assert torch.equal(y0, mvpa_hip.linear(x, w0))
    assert torch.equal(y1, mvpa_hip.linear(x, w1, gated=True))
    assert (wide[:, :8] == 3.0).all() and (wide[:, 8 + N1:] == 3.0).all()


def test_two_products_of_one_launch_refuse_small_shapes():
    x = torch.zeros(64, 768, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(768, 768, dtype=torch.bfloat16, device="cuda")
    assert not mvpa_hip.linear_dual_supported(64, 768) and not mvpa_hip.linear_dual_supported(1024, 96)
    with pytest.raises(mvpa_hip.MvpaError):
        mvpa_hip.linear_dual(x, w, w)


def test_linear_into_a_column_slice():
    """The gated product written into a column slice of a wider buffer (the block's tail operand)."""
    g = torch.Generator().manual_seed(9)
    x = torch.randn(1024, 768, generator=g).bfloat16().cuda()
    w = (torch.randn(2 * 1728, 768, generator=g) * 0.05).bfloat16().cuda()
    ref = mvpa_hip.linear(x, w, gated=True)
    both = torch.full((1024, 768 + 1728), 7.0, dtype=torch.bfloat16, device="cuda")
    mvpa_hip.linear(x, w, gated=True, out=both[:, 768:])
    assert torch.equal(both[:, 768:], ref) and (both[:, :768] == 7.0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(dtype):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(37, 550, generator=g).to(dtype)
    w = torch.rand(550, generator=g) + 0.5
    y = mvpa_hip.rmsnorm(x.cuda(), w.cuda(), 1e-5).float().cpu()
    ref = O.rmsnorm(x.float(), w, 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (y - ref).abs().max().item() <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols", [(37, 768), (5, 552), (130, 1536)])
def test_rmsnorm_row_vector_path(dtype, rows, cols):
    """Row lengths that are multiples of 8 take the one-wave-per-row kernel."""
    g = torch.Generator().manual_seed(rows)
    x = torch.randn(rows, cols, generator=g).to(dtype)
    w = torch.rand(cols, generator=g) + 0.5
    y = mvpa_hip.rmsnorm(x.cuda(), w.cuda(), 1e-5).float().cpu()
    ref = O.rmsnorm(x.float(), w, 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (y - ref).abs().max().item() <= tol


@pytest.mark.parametrize("rows,cols", [(37, 768), (3, 8), (129, 2048), (6, 1000), (5, 4096), (9, 1032)])
def test_add3_rmsnorm_equals_separate_kernels(rows, cols):
    """The fused residual-sum + norm is bit-identical to add3 followed by rmsnorm, and both
    agree with the fp32 statement of the two operations."""
    g = torch.Generator().manual_seed(cols)
    a, b, c = (torch.randn(rows, cols, generator=g).bfloat16().cuda() for _ in range(3))
    w = (torch.rand(cols, generator=g) + 0.5).cuda()
    total, normed = mvpa_hip.add3_rmsnorm(a, b, c, w, 1e-5)
    total2 = mvpa_hip.add3(a, b, c)
    normed2 = mvpa_hip.rmsnorm(total2, w, 1e-5)
    assert torch.equal(total, total2) and torch.equal(normed, normed2)
    ref_sum = (a.float() + b.float() + c.float()).bfloat16()
    assert torch.equal(total, ref_sum)
    ref = O.rmsnorm(ref_sum.float().cpu(), w.cpu(), 1e-5)
    assert (normed.float().cpu() - ref).abs().max().item() <= 2e-2


def test_add3():
    g = torch.Generator().manual_seed(2)
    a, b, c = (torch.randn(5, 1000, generator=g).bfloat16() for _ in range(3))
    y = mvpa_hip.add3(a.cuda(), b.cuda(), c.cuda()).cpu()
    assert torch.equal(y, (a.float() + b.float() + c.float()).bfloat16())


@pytest.mark.parametrize("L", [512, 2560, 100, 333, 12000])     # 12000: more than 64 KiB of LDS per row pair
def test_wavedec_db4(L):
    g = torch.Generator().manual_seed(L)
    x = torch.randn(9, L, generator=g)
    y = mvpa_hip.wavedec_db4(x.cuda()).cpu()
    ref = O.wavedec_db4_periodic(x)
    assert y.shape == ref.shape
    assert (y - ref).abs().max().item() <= 2e-5


def test_ring_append_writes_the_slot_the_device_counter_names():
    """mvpa_ring_append_bf16: keys and values of one step, given as strided views of a fused
    projection output, land in slot head[0] of both rings; everything else stays."""
    B, Hkv, C, Dh, steps = 2, 3, 5, 16, 7
    row = 4 * Dh + 2 * Hkv * Dh
    qkv = torch.randn(B, C, row, device="cuda").bfloat16()
    k_new = qkv[:, :, 4 * Dh:4 * Dh + Hkv * Dh].view(B, C, Hkv, Dh).permute(0, 2, 1, 3)
    v_new = qkv[:, :, 4 * Dh + Hkv * Dh:].view(B, C, Hkv, Dh).permute(0, 2, 1, 3)
    k_ring = torch.randn(B, Hkv, steps, C, Dh, device="cuda").bfloat16()
    v_ring = torch.randn(B, Hkv, steps, C, Dh, device="cuda").bfloat16()
    k0, v0 = k_ring.clone(), v_ring.clone()
    head = torch.tensor([4], dtype=torch.int32, device="cuda")
    mvpa_hip.ring_append(k_new, v_new, k_ring, v_ring, head)
    k0[:, :, 4], v0[:, :, 4] = k_new, v_new
    assert torch.equal(k_ring, k0) and torch.equal(v_ring, v0)


@pytest.mark.parametrize("M,N,K,gated", [(128, 2048, 2048, False), (128, 4096, 2048, False), (100, 2048, 5632, False),
                                         (128, 5632, 2048, True), (65, 96, 24, False), (33, 130, 550, False),
                                         (7, 70, 136, True), (128, 33, 300, True), (1, 64, 256, False)])
def test_linear_split_k_pair(M, N, K, gated):
    """mvpa_linear_bf16_splitk (K slices of 256 on separate workgroups, fp32 partial tiles through a
    workspace, second kernel sums and applies the epilogue) against float64, and against the
    one-kernel path to fp32 summation order."""
    g = torch.Generator().manual_seed(M * 7 + N + K)
    ldk = (K + 7) // 8 * 8
    x = torch.zeros(M, ldk).bfloat16()
    w = torch.zeros((2 if gated else 1) * N, ldk).bfloat16()
    x[:, :K] = torch.randn(M, K, generator=g).bfloat16()
    w[:, :K] = (torch.randn(w.shape[0], K, generator=g) * 0.05).bfloat16()
    xg, wg = x.cuda(), w.cuda()
    y = mvpa_hip.linear(xg[:, :K], wg[:, :K], gated=gated, split_k=True).float().cpu()
    y1 = mvpa_hip.linear(xg[:, :K], wg[:, :K], gated=gated, split_k=False).float().cpu()
    if gated:
        ref = torch.nn.functional.silu(x[:, :K].double() @ w[:N, :K].double().T) * (x[:, :K].double() @ w[N:, :K].double().T)
    else:
        ref = x[:, :K].double() @ w[:, :K].double().T
    tol = (2 ** -7 if gated else 2 ** -8) * ref.abs().max().item() + 1e-5
    assert (y.double() - ref).abs().max().item() <= tol
    assert (y - y1).abs().max().item() <= 2 * tol


@pytest.mark.parametrize("M,N,K", [(256, 128, 128), (70, 33, 50), (1, 5, 3), (513, 96, 129)])
def test_linear_f32_matches_float64_product(M, N, K):
    """The fp32 product of the fp32 layer path (fp32 MFMA, fp32 accumulation) against a float64
    matrix product: max-abs error <= 1e-5 on unit-scale operands, any M, N, K, row-pitched x."""
    torch.manual_seed(M + N)
    xw = torch.randn(M, K + 3, device="cuda")
    x = xw[:, :K]                                   # a row-pitched view
    w = torch.randn(N, K, device="cuda") / K ** 0.5
    y = mvpa_hip.linear_f32(x, w)
    ref = (x.double() @ w.double().t())
    assert y.shape == (M, N) and (y.double() - ref).abs().max().item() <= 1e-5
    y3 = mvpa_hip.linear_f32(x.reshape(1, M, K), w)
    assert y3.shape == (1, M, N) and torch.equal(y3[0], y)
