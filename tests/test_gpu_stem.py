"""GPU parity of the fused first patch-embedding layer (conv 3x3 stride 2 -> LayerNorm -> GELU in one kernel, through
the C ABI) against the fp32 CPU composition of the three torch operators on the same 16-bit operands.

The kernel rounds to the 16-bit type where the separate operators would (convolution output, LayerNorm output, GELU
output), so the bound is a few roundings of the output type: 2e-2 absolute on values of order one."""
import pytest
import torch
import torch.nn.functional as F

from vmamba_amd import _lib
from vmamba_amd.stem import stem_conv_ln_gelu_hip

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def reference(x, w, b, g, beta, eps, dtype):
    r = lambda t: t.to(dtype).float()                         # the roundings of the separate operators
    y = r(F.conv2d(x.float(), w.float(), None if b is None else b.float(), stride=2, padding=1)).permute(0, 2, 3, 1)
    y = r(F.layer_norm(y, (w.shape[0],), None if g is None else g.float(), None if beta is None else beta.float(), eps))
    return r(F.gelu(y))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("B,H,W,C", [(2, 224, 224, 48), (1, 64, 64, 64), (3, 31, 45, 48), (2, 8, 8, 48), (1, 1, 1, 48), (1, 17, 2, 64),
                                     (1, 130, 72, 48)])
@pytest.mark.parametrize("channels_last_weight", [False, True])
def test_stem_matches_conv_layernorm_gelu(B, H, W, C, dtype, channels_last_weight):
    print("CASE stem", B, H, W, C, dtype, channels_last_weight, flush=True)
    g = torch.Generator().manual_seed(B * 100 + H + W + C)
    x = torch.randn(B, 3, H, W, generator=g).to(dtype)
    w = (torch.randn(C, 3, 3, 3, generator=g) * 0.3).to(dtype)
    b = (torch.randn(C, generator=g) * 0.2).to(dtype)
    gamma, beta = (torch.randn(C, generator=g) * 0.3 + 1).to(dtype), (torch.randn(C, generator=g) * 0.3).to(dtype)
    want = reference(x, w, b, gamma, beta, 1e-5, dtype)
    wd = w.to(DEV)
    if channels_last_weight:
        wd = wd.contiguous(memory_format=torch.channels_last)
    got = stem_conv_ln_gelu_hip(x.to(DEV), wd, b.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5)
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == want.shape == (B, (H - 1) // 2 + 1, (W - 1) // 2 + 1, C)
    err = (got.cpu().float() - want).abs().max().item()
    assert err <= 2e-2, f"max err {err}"


def test_stem_without_affine_parameters_and_rejections():
    bf = dict(device=DEV, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(3)
    x, w = torch.randn(2, 3, 16, 16, generator=g).bfloat16(), (torch.randn(48, 3, 3, 3, generator=g) * 0.3).bfloat16()
    got = stem_conv_ln_gelu_hip(x.to(DEV), w.to(DEV), None, None, None, 1e-6)
    assert (got.cpu().float() - reference(x, w, None, None, None, 1e-6, torch.bfloat16)).abs().max().item() <= 2e-2
    with pytest.raises(_lib.Ss2dError) as e:
        stem_conv_ln_gelu_hip(torch.zeros(1, 3, 8, 8, **bf), torch.zeros(40, 3, 3, 3, **bf), None, None, None)     # width 40
    assert e.value.code == _lib.SS2D_ENOTSUP
    with pytest.raises(RuntimeError):
        stem_conv_ln_gelu_hip(torch.zeros(1, 3, 8, 8, device=DEV), torch.zeros(48, 3, 3, 3, device=DEV), None, None, None)   # fp32
    with pytest.raises(ValueError):
        stem_conv_ln_gelu_hip(torch.zeros(1, 4, 8, 8, **bf), torch.zeros(48, 4, 3, 3, **bf), None, None, None)
    with pytest.raises(NotImplementedError):
        stem_conv_ln_gelu_hip(torch.zeros(1, 3, 8, 8).bfloat16(), torch.zeros(48, 3, 3, 3).bfloat16(), None, None, None)
    assert stem_conv_ln_gelu_hip(torch.zeros(0, 3, 8, 8, **bf), torch.zeros(48, 3, 3, 3, **bf), None, None, None).shape == (0, 4, 4, 48)
