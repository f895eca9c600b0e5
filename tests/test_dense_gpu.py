"""GPU checks of the dense ops behind the C ABI (linear, RMSNorm, residual add, db4 DWT)."""
import pytest
import torch

import mvpa_hip
from oracle import mvpa_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 200, 72), (1000, 768, 550), (64, 2304, 768), (17, 33, 8),
                                   (2048, 768, 768), (1024, 1280, 768), (600, 130, 72), (4100, 2048, 552),
                                   (16384, 768, 1728)])
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


@pytest.mark.parametrize("M,N,K", [(200, 96, 64), (1024, 1728, 768), (700, 200, 136), (4096, 64, 768)])
def test_linear_gated(M, N, K):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(2 * N, K, generator=g) * 0.2).bfloat16()
    y = mvpa_hip.linear(x.cuda(), w.cuda(), gated=True).float().cpu()
    gate = x.double() @ w[:N].double().T
    up = x.double() @ w[N:].double().T
    ref = torch.nn.functional.silu(gate) * up
    assert (y.double() - ref).abs().max().item() <= 2 ** -7 * ref.abs().max().item() + 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(dtype):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(37, 550, generator=g).to(dtype)
    w = torch.rand(550, generator=g) + 0.5
    y = mvpa_hip.rmsnorm(x.cuda(), w.cuda(), 1e-5).float().cpu()
    ref = O.rmsnorm(x.float(), w, 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (y - ref).abs().max().item() <= tol


def test_add3():
    g = torch.Generator().manual_seed(2)
    a, b, c = (torch.randn(5, 1000, generator=g).bfloat16() for _ in range(3))
    y = mvpa_hip.add3(a.cuda(), b.cuda(), c.cuda()).cpu()
    assert torch.equal(y, (a.float() + b.float() + c.float()).bfloat16())


@pytest.mark.parametrize("L", [512, 2560, 100])
def test_wavedec_db4(L):
    g = torch.Generator().manual_seed(L)
    x = torch.randn(9, L, generator=g)
    y = mvpa_hip.wavedec_db4(x.cuda()).cpu()
    ref = O.wavedec_db4_periodic(x)
    assert y.shape == ref.shape
    assert (y - ref).abs().max().item() <= 2e-5
