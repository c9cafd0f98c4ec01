"""GPU parity of the classifier's global average pool (ss2d_mean_pool_cl through the C ABI) against the float64 mean of
the same 16-bit values on the CPU: the kernel sums in fp32 and rounds once, so the bound is half a unit in the last
place of the output type plus the fp32 summation error."""
import pytest
import torch

from vmamba_amd import _lib
from vmamba_amd.pool import GlobalAvgPool2d, mean_pool_cl_hip, mean_pool_fusable

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("B,L,C", [(128, 49, 768), (1, 1, 8), (3, 7, 264), (2, 1024, 96), (5, 50, 1000), (4, 196, 384)])
def test_mean_pool_matches_float64_mean(B, L, C, dtype):
    print("CASE mean_pool", B, L, C, dtype, flush=True)
    g = torch.Generator().manual_seed(B + L + C)
    x = (torch.randn(B, L, C, generator=g) * 2 + 0.5).to(dtype)
    got = mean_pool_cl_hip(x.to(DEV))
    torch.cuda.synchronize()
    assert got.shape == (B, C) and got.dtype == dtype
    want64 = x.double().mean(1)
    ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    err = (got.cpu().double() - want64).abs()
    assert (err <= 0.5001 * ulp * want64.abs().clamp_min(2.0 ** -14) * 2 + 1e-6).all(), err.max().item()
    # and the library's mean of the same values (its fp32 summation order differs: equal up to one rounding step)
    lib = x.float().mean(1).to(dtype).float()
    assert torch.allclose(got.cpu().float(), lib, rtol=2 * ulp, atol=1e-6)


def test_mean_pool_is_exact_on_constant_maps():
    x = torch.full((2, 49, 16), 3.0, dtype=torch.bfloat16, device=DEV)      # 49 * 3 / 49 in fp32 rounds to 3
    assert torch.equal(mean_pool_cl_hip(x), torch.full((2, 16), 3.0, dtype=torch.bfloat16, device=DEV))


def test_module_pools_channel_last_and_falls_back_to_the_library_otherwise():
    pool = GlobalAvgPool2d()
    x = torch.randn(2, 7, 7, 24, device=DEV).bfloat16()
    y = pool(x.permute(0, 3, 1, 2))                                         # (B, C, H, W) view of channel-last memory
    assert y.shape == (2, 24, 1, 1)
    assert torch.allclose(y.float().flatten(1), x.float().mean((1, 2)), rtol=1e-2, atol=1e-3)
    xc = torch.randn(2, 24, 7, 7, device=DEV).bfloat16()                    # channel-first memory: the library's kernel
    assert not mean_pool_fusable(xc)
    assert torch.allclose(pool(xc).float(), xc.float().mean((2, 3), keepdim=True), rtol=1e-2, atol=1e-3)
    assert not mean_pool_fusable(x.float().permute(0, 3, 1, 2))


def test_mean_pool_rejections():
    L = _lib.lib()
    x = torch.zeros(2, 4, 12, device=DEV, dtype=torch.bfloat16)
    y = torch.zeros(2, 12, device=DEV, dtype=torch.bfloat16)
    assert L.ss2d_mean_pool_cl(x.data_ptr(), y.data_ptr(), 2, 4, 12, _lib.SS2D_BF16, None) == _lib.SS2D_ENOTSUP   # C % 8
    assert L.ss2d_mean_pool_cl(x.data_ptr(), y.data_ptr(), 2, 4, 16, _lib.SS2D_F32, None) == _lib.SS2D_ENOTSUP
    assert L.ss2d_mean_pool_cl(x.data_ptr(), y.data_ptr(), 2, 0, 16, _lib.SS2D_BF16, None) == _lib.SS2D_EINVAL
    assert L.ss2d_mean_pool_cl(None, y.data_ptr(), 2, 4, 16, _lib.SS2D_BF16, None) == _lib.SS2D_EINVAL
    assert L.ss2d_mean_pool_cl(None, None, 0, 4, 16, _lib.SS2D_BF16, None) == _lib.SS2D_OK
    with pytest.raises(TypeError):
        mean_pool_cl_hip(torch.zeros(2, 4, 16, device=DEV))
