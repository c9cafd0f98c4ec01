"""GPU parity of the fused depthwise-conv + SiLU kernel against torch's CPU conv2d + silu (the calls the
reference makes, classification/models/vmamba.py:654-658).  fp32: rtol/atol 1e-5; 16-bit: two units in the last
place (the conv result and the SiLU result are each rounded once, and nine-term sums may round differently)."""
import pytest
import torch

from oracle import torch_ref
from vmamba_amd.conv import dwconv3x3_silu_hip

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SHAPES = [(2, 96, 56, 56), (3, 192, 28, 28), (2, 384, 14, 14), (2, 768, 7, 7), (1, 8, 3, 3), (2, 40, 9, 13), (1, 96, 1, 1),
          (2, 12, 5, 6), (1, 7, 4, 4), (1, 32, 1, 70), (1, 16, 2, 200), (1, 64, 20, 128),
          # channel tiles of 64 / 32 with row tiles and a short last one, rows of 16- and 8-byte pieces, odd whole images,
          # a map too tall for one tile whose rows take no 8-byte stores (the older row-tile kernel), the widest rows
          (2, 64, 30, 56), (1, 32, 37, 28), (2, 128, 5, 9), (1, 64, 100, 14), (1, 32, 3, 120), (1, 160, 9, 12), (3, 64, 8, 8),
          # tiles of at most 32 positions with several channel groups (the rotation of the output rows wraps)
          (3, 40, 4, 2), (2, 24, 4, 4), (1, 48, 5, 6), (2, 16, 3, 3), (1, 72, 2, 9),
          # wide images in column tiles of 8 / 4 / 5 / 4 segments (and 17 segments, which no tile width divides)
          (1, 32, 20, 256), (2, 64, 9, 128), (1, 32, 33, 200), (1, 64, 5, 192), (1, 96, 16, 136)]


def _tol(dtype):
    return {torch.float32: dict(rtol=1e-5, atol=1e-5), torch.bfloat16: dict(rtol=2 ** -6, atol=2 ** -6),
            torch.float16: dict(rtol=2 ** -9, atol=2 ** -9)}[dtype]


@pytest.mark.parametrize("B,D,H,W", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("channel_last", [False, True])
@pytest.mark.parametrize("has_bias,silu", [(False, True), (True, True), (True, False)])
def test_dwconv_silu(B, D, H, W, dtype, channel_last, has_bias, silu):
    print("CASE dwconv", B, D, H, W, dtype, channel_last, has_bias, silu, flush=True)
    g = torch.Generator().manual_seed(51)
    x = torch.randn(B, D, H, W, generator=g).to(dtype)
    w = (torch.randn(D, 1, 3, 3, generator=g) * 0.3).to(dtype)
    b = torch.randn(D, generator=g).to(dtype) if has_bias else None
    xin = x.permute(0, 2, 3, 1).contiguous() if channel_last else x
    want = torch_ref.dwconv3x3_silu(xin.float(), w.float(), None if b is None else b.float(), channel_last, apply_silu=False)
    want = want.to(dtype)                                   # conv result rounded to the tensor dtype ...
    if silu:
        want = torch.nn.functional.silu(want.float()).to(dtype)   # ... then SiLU, rounded again
    got = dwconv3x3_silu_hip(xin.to(DEV), w.to(DEV), None if b is None else b.to(DEV), channel_last, silu).cpu()
    assert got.shape == (B, D, H, W) and got.dtype == dtype
    assert torch.allclose(got.float(), want.float(), **_tol(dtype))


def test_dwconv_identity_and_errors():
    x = torch.randn(2, 16, 6, 7, generator=torch.Generator().manual_seed(52)).bfloat16().to(DEV)
    ident = torch.zeros(16, 1, 3, 3, device=DEV, dtype=torch.bfloat16)
    ident[:, 0, 1, 1] = 1.0
    assert torch.equal(dwconv3x3_silu_hip(x, ident, None, False, False), x)
    assert torch.equal(dwconv3x3_silu_hip(x.permute(0, 2, 3, 1).contiguous(), ident, None, True, False), x)
    with pytest.raises(ValueError):
        dwconv3x3_silu_hip(x, torch.zeros(16, 1, 5, 5, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        dwconv3x3_silu_hip(x.cpu(), ident.cpu())
    assert dwconv3x3_silu_hip(x[:0], ident).shape == (0, 16, 6, 7)
