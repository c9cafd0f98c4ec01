"""GPU parity of the fused channel-last MLP kernel (fc1 -> GELU -> fc2 -> + residual) against the unfused torch
operators the reference uses (classification/models/vmamba.py:1116-1131, :1229) and against float64 math.

Tolerance: the 16-bit bound (2e-2): both paths round fc1, GELU and fc2 outputs to the tensor type, but accumulate in
different orders; against float64 the error is a few 16-bit roundings."""
import pytest
import torch
import torch.nn.functional as F

from vmamba_amd import _lib
from vmamba_amd.mlp import mlp_fused_hip
from vmamba_amd.vssm import Mlp

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make(seed, M, C, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, C, generator=g).to(dtype)
    res = torch.randn(M, C, generator=g).to(dtype)
    w1 = (torch.randn(4 * C, C, generator=g) * C ** -0.5).to(dtype)
    b1 = (torch.randn(4 * C, generator=g) * 0.5).to(dtype)
    w2 = (torch.randn(C, 4 * C, generator=g) * (4 * C) ** -0.5).to(dtype)
    b2 = (torch.randn(C, generator=g) * 0.5).to(dtype)
    return x, w1, b1, w2, b2, res


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("M,C", [(256, 96), (128, 192), (1000, 96), (77, 192), (1, 96), (64 * 3136, 96), (16 * 784, 192)])
def test_mlp_fused_matches_unfused_operators(M, C, dtype):
    print("CASE mlp", M, C, dtype, flush=True)
    x, w1, b1, w2, b2, res = [t.to(DEV) for t in make(M + C, M, C, dtype)]
    got = mlp_fused_hip(x, w1, b1, w2, b2, res)
    torch.cuda.synchronize()
    want = res + F.linear(F.gelu(F.linear(x, w1, b1)), w2, b2)                   # the reference's operator sequence
    exact = (res.double() + F.linear(F.gelu(F.linear(x.double(), w1.double(), b1.double())), w2.double(), b2.double()))
    assert got.shape == x.shape and got.dtype == dtype
    tol = 2e-2 if dtype == torch.bfloat16 else 4e-3
    scale = exact.abs().max().item()
    assert (got.double() - exact).abs().max().item() <= tol * scale
    assert (got.double() - want.double()).abs().max().item() <= tol * scale
    # the kernel is at least as close to exact math as the unfused 16-bit pipeline is (mean error)
    assert (got.double() - exact).abs().mean().item() <= 1.5 * (want.double() - exact).abs().mean().item() + 1e-6
    # optional arguments
    got2 = mlp_fused_hip(x, w1, None, w2, None, None)
    want2 = F.linear(F.gelu(F.linear(x, w1)), w2)
    assert (got2.double() - want2.double()).abs().max().item() <= tol * scale
    # the block's second LayerNorm in front (vmamba.py:1229): x -> x + mlp(norm2(x))
    g = torch.Generator().manual_seed(M)
    gamma = (1.0 + 0.2 * torch.randn(C, generator=g)).to(dtype).to(DEV)
    beta = (0.2 * torch.randn(C, generator=g)).to(dtype).to(DEV)
    xs = (x * 1.5 + 0.3).to(dtype)
    got3 = mlp_fused_hip(xs, w1, b1, w2, b2, xs, gamma, beta, 1e-6)
    want3 = xs + F.linear(F.gelu(F.linear(F.layer_norm(xs, (C,), gamma, beta, 1e-6), w1, b1)), w2, b2)
    d = lambda t: t.double()
    exact3 = d(xs) + F.linear(F.gelu(F.linear(F.layer_norm(d(xs), (C,), d(gamma), d(beta), 1e-6), d(w1), d(b1))), d(w2), d(b2))
    scale3 = exact3.abs().max().item()
    assert (d(got3) - exact3).abs().max().item() <= tol * scale3
    assert (d(got3) - d(want3)).abs().max().item() <= tol * scale3
    assert (d(got3) - exact3).abs().mean().item() <= 1.5 * (d(want3) - exact3).abs().mean().item() + 1e-6


def test_mlp_module_uses_the_kernel_and_falls_back_by_shape():
    torch.manual_seed(0)
    for C, fused in ((96, True), (192, True), (384, False)):
        m = Mlp(C, 4 * C, channel_first=False).to(DEV).bfloat16().eval()
        x = torch.randn(2, 5, 7, C, device=DEV).bfloat16()
        r = torch.randn_like(x)
        norm = torch.nn.LayerNorm(C).to(DEV).bfloat16()
        with torch.no_grad():
            norm.weight.uniform_(0.8, 1.2); norm.bias.uniform_(-0.2, 0.2)
            got = m(x, residual=r)
            want = r + m.fc2(m.act(m.fc1(x)))
            got_n = m(x, residual=x, pre_norm=norm)
            want_n = x + m.fc2(m.act(m.fc1(norm(x))))
        assert got.shape == x.shape
        assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=2e-2)
        assert torch.allclose(got_n.float(), want_n.float(), rtol=2e-2, atol=2e-2)
    # under autograd the torch operators run, and gradients flow
    m = Mlp(96, 384, channel_first=False).to(DEV).bfloat16().train()
    x = torch.randn(3, 96, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    m(x, residual=x).float().sum().backward()
    assert x.grad is not None and m.fc1.weight.grad is not None


def test_mlp_fused_rejections():
    x, w1, b1, w2, b2, res = [t.to(DEV) for t in make(1, 8, 96, torch.bfloat16)]
    with pytest.raises(ValueError):
        mlp_fused_hip(x, w1[:10], b1, w2, b2, res)
    with pytest.raises(TypeError):
        mlp_fused_hip(x.float(), w1.float(), None, w2.float(), None, None)
    with pytest.raises(NotImplementedError):
        mlp_fused_hip(x.cpu(), w1.cpu(), None, w2.cpu(), None, None)
    L = _lib.lib()
    assert L.ss2d_mlp_fused(x.data_ptr(), None, None, 1e-5, w1.data_ptr(), None, w2.data_ptr(), None, None, x.data_ptr(), 8, 100,
                            _lib.SS2D_BF16, None) == _lib.SS2D_ENOTSUP
    assert L.ss2d_mlp_fused(None, None, None, 1e-5, None, None, None, None, None, None, 8, 96, _lib.SS2D_BF16, None) == _lib.SS2D_EINVAL
    assert L.ss2d_mlp_fused(x.data_ptr(), None, b2.data_ptr(), 1e-5, w1.data_ptr(), None, w2.data_ptr(), None, None, x.data_ptr(), 8, 96,
                            _lib.SS2D_BF16, None) == _lib.SS2D_EINVAL          # LayerNorm bias without weight
    assert mlp_fused_hip(x[:0], w1, b1, w2, b2, res[:0]).shape == (0, 96)
