"""GPU parity of the narrow channel-last projection kernel (LayerNorm -> Linear -> + residual in one pass) against the
separate torch operators the reference uses (classification/models/vmamba.py:1225-1228, :648-650, :662) and against
float64 math.  Tolerance: the 16-bit bound of this package (2e-2 bf16, 4e-3 fp16, of the output scale): both paths
round the LayerNorm output, the projection output and the sum to the tensor type; accumulation orders differ."""
import pytest
import torch
import torch.nn.functional as F

from vmamba_amd import _lib
from vmamba_amd.linear import linear_cl_hip, linear_fusable

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make(seed, M, K, N, dtype):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(M, K, generator=g) * 1.5 + 0.3).to(dtype)
    res = torch.randn(M, N, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * K ** -0.5).to(dtype)
    b = (torch.randn(N, generator=g) * 0.5).to(dtype)
    gamma = (1.0 + 0.2 * torch.randn(K, generator=g)).to(dtype)
    beta = (0.2 * torch.randn(K, generator=g)).to(dtype)
    return x, res, w, b, gamma, beta


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("M,K", [(1, 96), (77, 96), (256, 96), (1000, 96), (16 * 3136, 96), (128 * 3136, 96)])
def test_linear_cl_matches_separate_operators(M, K, dtype):
    print("CASE linear_cl", M, K, dtype, flush=True)
    N = K
    x, res, w, b, gamma, beta = [t.to(DEV) for t in make(M, M, K, N, dtype)]
    tol = 2e-2 if dtype == torch.bfloat16 else 4e-3
    d = lambda t: t.double()
    for use_ln, use_bias, use_res in ((True, False, False), (False, False, True), (True, True, True), (False, True, False)):
        got = linear_cl_hip(x, w, b if use_bias else None, res if use_res else None,
                            gamma if use_ln else None, beta if use_ln else None, 1e-5)
        torch.cuda.synchronize()
        h = F.layer_norm(x, (K,), gamma, beta, 1e-5) if use_ln else x
        want = F.linear(h, w, b if use_bias else None)
        want = want + res if use_res else want
        he = F.layer_norm(d(x), (K,), d(gamma), d(beta), 1e-5) if use_ln else d(x)
        exact = F.linear(he, d(w), d(b) if use_bias else None) + (d(res) if use_res else 0.0)
        scale = exact.abs().max().item()
        assert got.shape == want.shape and got.dtype == dtype
        assert (d(got) - exact).abs().max().item() <= tol * scale, (use_ln, use_bias, use_res)
        assert (d(got) - d(want)).abs().max().item() <= tol * scale, (use_ln, use_bias, use_res)
        assert (d(got) - exact).abs().mean().item() <= 1.5 * (d(want) - exact).abs().mean().item() + 1e-6


def test_linear_cl_layer_norm_without_bias_and_shapes():
    x, res, w, b, gamma, beta = [t.to(DEV) for t in make(3, 2 * 5 * 7, 96, 96, torch.bfloat16)]
    x4 = x.view(2, 5, 7, 96)
    got = linear_cl_hip(x4, w, None, None, gamma, None, 1e-6)
    want = F.linear(F.layer_norm(x4, (96,), gamma, None, 1e-6), w)
    assert got.shape == (2, 5, 7, 96)
    assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=2e-2)
    assert linear_cl_hip(x4[:0], w).shape == (0, 5, 7, 96)


def test_linear_cl_rejections():
    x, res, w, b, gamma, beta = [t.to(DEV) for t in make(1, 8, 96, 96, torch.bfloat16)]
    assert linear_fusable(x, w) and not linear_fusable(x.float(), w.float()) and not linear_fusable(x.cpu(), w.cpu())
    with pytest.raises(ValueError):
        linear_cl_hip(x, w[:, :10])
    with pytest.raises(TypeError):
        linear_cl_hip(x.float(), w.float())
    with pytest.raises(NotImplementedError):
        linear_cl_hip(x.cpu(), w.cpu())
    with pytest.raises(ValueError):
        linear_cl_hip(x, w, residual=res[:4])
    L = _lib.lib()
    args = lambda K, N, dt: (x.data_ptr(), None, None, 1e-5, w.data_ptr(), None, None, x.data_ptr(), 8, K, N, dt, None)
    assert L.ss2d_linear_cl(*args(192, 192, _lib.SS2D_BF16)) == _lib.SS2D_ENOTSUP
    assert L.ss2d_linear_cl(*args(96, 192, _lib.SS2D_BF16)) == _lib.SS2D_ENOTSUP
    assert L.ss2d_linear_cl(*args(96, 96, _lib.SS2D_F32)) == _lib.SS2D_ENOTSUP
    assert L.ss2d_linear_cl(None, None, None, 1e-5, None, None, None, None, 8, 96, 96, _lib.SS2D_BF16, None) == _lib.SS2D_EINVAL
    assert L.ss2d_linear_cl(x.data_ptr(), None, gamma.data_ptr(), 1e-5, w.data_ptr(), None, None, x.data_ptr(), 8, 96, 96,
                            _lib.SS2D_BF16, None) == _lib.SS2D_EINVAL          # LayerNorm bias without weight


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("B,L", [(1, 32), (3, 64), (2, 3136), (5, 96)])
@pytest.mark.parametrize("with_residual", [False, True])
def test_linear_cf_ln_matches_out_norm_then_out_proj(B, L, dtype, with_residual):
    """out_norm over the channels of the fp32 channel-first map (fp32 statistics, result rounded to the 16-bit type), then
    the projection (+ bias, rounded) and the residual add (rounded): the separate operators on the CPU in fp32."""
    from vmamba_amd.linear import linear_cf_ln_hip
    print("CASE linear_cf_ln", B, L, dtype, with_residual, flush=True)
    K = N = 96
    g = torch.Generator().manual_seed(B * 7 + L)
    y = torch.randn(B, K, L, generator=g) * 2 + 0.3
    gamma, beta = (torch.randn(K, generator=g) * 0.3 + 1).to(dtype), (torch.randn(K, generator=g) * 0.3).to(dtype)
    w, bias = (torch.randn(N, K, generator=g) * K ** -0.5).to(dtype), (torch.randn(N, generator=g) * 0.1).to(dtype)
    res = torch.randn(B, L, N, generator=g).to(dtype) if with_residual else None
    r = lambda t: t.to(dtype).float()
    normed = r(torch.nn.functional.layer_norm(y.permute(0, 2, 1), (K,), gamma.float(), beta.float(), 1e-5))
    want = r(normed @ w.float().t() + bias.float())
    if with_residual:
        want = r(want + res.float())
    dev = lambda t: None if t is None else t.to(DEV)
    got = linear_cf_ln_hip(dev(y), dev(gamma), dev(beta), 1e-5, dev(w), dev(bias), dev(res))
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == (B, L, N)
    assert torch.allclose(got.cpu().float(), want, rtol=2e-2, atol=2e-2)


def test_linear_cf_ln_rejections():
    from vmamba_amd.linear import linear_cf_ln_fusable, linear_cf_ln_hip
    w = torch.zeros(96, 96, device=DEV, dtype=torch.bfloat16)
    assert linear_cf_ln_fusable(96, w, 64) and not linear_cf_ln_fusable(96, w, 49) and not linear_cf_ln_fusable(96, w.float(), 64)
    with pytest.raises(_lib.Ss2dError) as e:
        linear_cf_ln_hip(torch.zeros(1, 96, 49, device=DEV), w[0], None, 1e-5, w)                       # L % 32 != 0
    assert e.value.code == _lib.SS2D_ENOTSUP
    with pytest.raises(TypeError):
        linear_cf_ln_hip(torch.zeros(1, 96, 64, device=DEV, dtype=torch.bfloat16), w[0], None, 1e-5, w)  # the map must be fp32
    with pytest.raises(ValueError):
        linear_cf_ln_hip(torch.zeros(1, 96, 64, device=DEV), None, None, 1e-5, w)
    assert linear_cf_ln_hip(torch.zeros(0, 96, 64, device=DEV), w[0], None, 1e-5, w).shape == (0, 64, 96)
