"""GPU parity of CrossScan / CrossMerge in every layout and mode (channel-first / channel-last on either side,
one-by-one, scans 0 / 1 / 2) through the C ABI against the CPU oracle.  Bit-exact: the scan is a permutation, and
the merge's additions are rounded in the oracle's order."""
import itertools

import pytest
import torch

from oracle import torch_ref
import vmamba_amd as va
from vmamba_amd import _lib
from vmamba_amd.csm import cross_merge_flex_hip

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

MODES = list(itertools.product([True, False], [True, False], [False, True], [0, 1, 2]))
SHAPES = [(2, 3, 5, 7), (1, 8, 14, 14), (2, 96, 7, 7), (1, 2, 1, 9), (1, 1, 33, 2), (2, 5, 8, 16)]


def _x_shape(B, C, H, W, icf, obo):
    if icf:
        return (B, 4, C, H, W) if obo else (B, C, H, W)
    return (B, H, W, 4, C) if obo else (B, H, W, C)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.uint8, torch.float64], ids=str)
@pytest.mark.parametrize("icf,ocf,obo,scans", MODES)
def test_cross_scan_every_mode_bit_exact(icf, ocf, obo, scans, dtype):
    print("CASE scan-flex", icf, ocf, obo, scans, dtype, flush=True)
    for (B, C, H, W) in SHAPES:
        g = torch.Generator().manual_seed(B + C + H + W)
        x = (torch.randn(_x_shape(B, C, H, W, icf, obo), generator=g) * 40).to(dtype)
        want = torch_ref.cross_scan_flex(x, icf, ocf, obo, scans)
        got = va.cross_scan_fn(x.to(DEV), icf, ocf, obo, scans)
        torch.cuda.synchronize()
        assert got.shape == want.shape and torch.equal(got.cpu(), want), (B, C, H, W)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("icf,ocf,obo,scans", MODES)
def test_cross_merge_every_mode_bit_exact(icf, ocf, obo, scans, dtype):
    print("CASE merge-flex", icf, ocf, obo, scans, dtype, flush=True)
    for (B, C, H, W) in SHAPES:
        g = torch.Generator().manual_seed(B * 7 + C + H + W)
        y = torch.randn((B, 4, C, H, W) if ocf else (B, H, W, 4, C), generator=g).to(dtype)
        want = torch_ref.cross_merge_flex(y, icf, ocf, obo, scans)
        got = va.cross_merge_fn(y.to(DEV), icf, ocf, obo, scans)
        torch.cuda.synchronize()
        assert got.shape == want.shape and got.dtype == dtype
        if scans == 1 and not obo and dtype == torch.float32:
            # a four-term fp32 reduction: the library's order of additions is not specified
            assert torch.allclose(got.cpu(), want, rtol=3e-7, atol=1e-7), (B, C, H, W)
        else:
            assert torch.equal(got.cpu(), want), (B, C, H, W)


@pytest.mark.parametrize("x_cl,obo,scans", [(0, 0, 0), (1, 0, 0), (0, 1, 0), (1, 1, 0), (0, 0, 2), (1, 0, 1), (1, 1, 2)])
def test_staged_mixed_layout_scan_equals_the_route_kernel(x_cl, obo, scans):
    """ss2d_cross_scan_flex_ws (transpose into the workspace + same-layout kernel) against ss2d_cross_scan_flex (one
    gather) through the C ABI: the same permutation, bit for bit; a workspace larger than needed is fine."""
    print("CASE scan-flex-ws", x_cl, obo, scans, flush=True)
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    for (B, C, H, W) in [(2, 96, 14, 14), (3, 5, 7, 9), (1, 130, 5, 13)]:
        K = 4 if obo else 1
        x = torch.randint(-30000, 30000, (B * K * C * H * W,), dtype=torch.int16, device=DEV)
        want = torch.empty(B * 4 * C * H * W, dtype=torch.int16, device=DEV)
        got = torch.full_like(want, 7)
        ws = torch.empty(x.numel() + 64, dtype=torch.int16, device=DEV)
        y_cl = 1 - x_cl
        assert L.ss2d_cross_scan_flex(x.data_ptr(), want.data_ptr(), B, C, H, W, 2, x_cl, y_cl, obo, scans, stream) == 0
        assert L.ss2d_cross_scan_flex_ws(x.data_ptr(), got.data_ptr(), B, C, H, W, 2, x_cl, y_cl, obo, scans, ws.data_ptr(),
                                         ws.numel() * 2, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), (B, C, H, W)
    # same layout on both sides: the workspace is not needed
    x = torch.randint(-9, 9, (2 * 3 * 4 * 5,), dtype=torch.int16, device=DEV)
    a, b = torch.empty(2 * 4 * 3 * 20, dtype=torch.int16, device=DEV), torch.empty(2 * 4 * 3 * 20, dtype=torch.int16, device=DEV)
    assert L.ss2d_cross_scan_flex(x.data_ptr(), a.data_ptr(), 2, 3, 4, 5, 2, 1, 1, 0, 0, stream) == 0
    assert L.ss2d_cross_scan_flex_ws(x.data_ptr(), b.data_ptr(), 2, 3, 4, 5, 2, 1, 1, 0, 0, None, 0, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(a, b)


@pytest.mark.parametrize("B,R,S", [(2, 96, 3136), (3, 64, 64), (1, 72, 200), (2, 8, 8), (1, 136, 24), (2, 96, 49), (1, 5, 7), (2, 100, 36)])
@pytest.mark.parametrize("dtype", [torch.int16, torch.int32, torch.int8, torch.int64])
def test_transpose_bcl_is_a_transpose(B, R, S, dtype):
    """(B, R, S) -> (B, S, R): extents that take the 16-byte kernel (multiples of a vector, with short last tiles) and
    extents that take the element-wise one, every element size, bit for bit against torch."""
    from vmamba_amd.csm import transpose_bcl_hip
    info = torch.iinfo(dtype)
    x = torch.randint(max(info.min, -2 ** 31), min(info.max, 2 ** 31 - 1), (B, R, S), dtype=dtype, device=DEV)
    assert torch.equal(transpose_bcl_hip(x), x.transpose(1, 2).contiguous())


def test_cross_merge_flex_left_to_right_order():
    y = torch.randn(2, 7, 5, 4, 6, generator=torch.Generator().manual_seed(1)).bfloat16()
    want = torch_ref.cross_merge_flex(y, False, False, False, 0, left_to_right=True)
    got = cross_merge_flex_hip(y.to(DEV), False, False, False, 0, order=_lib.MERGE_LEFT_TO_RIGHT)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("icf,ocf,obo,scans", MODES)
def test_flex_modes_round_trip_and_autograd(icf, ocf, obo, scans):
    """merge(scan(x)) = 4x (one-by-one: x) exactly on small integers; the backward of each operator is the other."""
    B, C, H, W = 2, 3, 4, 5
    x = torch.randint(-8, 8, _x_shape(B, C, H, W, icf, obo), generator=torch.Generator().manual_seed(2)).float().to(DEV)
    x.requires_grad_(True)
    y = va.cross_scan_fn(x, icf, ocf, obo, scans)
    y5 = y.view(B, 4, C, H, W) if ocf else y.view(B, H, W, 4, C)
    back = va.cross_merge_fn(y5, icf, ocf, obo, scans)
    assert torch.equal(back.reshape(x.shape), x.detach() * (1 if obo else 4))
    gy = torch.randint(-8, 8, y.shape, generator=torch.Generator().manual_seed(3)).float().to(DEV)
    (gx,) = torch.autograd.grad(y, x, gy)
    want = va.cross_merge_fn((gy.view(B, 4, C, H, W) if ocf else gy.view(B, H, W, 4, C)), icf, ocf, obo, scans)
    assert torch.equal(gx, want.reshape(x.shape))
    # <scan(x), gy> = <x, merge(gy)>
    assert (y.detach() * gy).sum().item() == (x.detach() * gx).sum().item()


def test_flex_rejections():
    with pytest.raises(NotImplementedError):
        va.cross_scan_fn(torch.zeros(1, 2, 3, 3, device=DEV), scans=3)
    with pytest.raises(ValueError):
        va.cross_scan_fn(torch.zeros(1, 2, 3, 3, device=DEV), one_by_one=True, in_channel_first=False)
    with pytest.raises(ValueError):
        va.cross_merge_fn(torch.zeros(1, 3, 2, 3, 3, device=DEV), in_channel_first=False)
    assert va.cross_scan_fn(torch.zeros(0, 3, 3, 2, device=DEV), in_channel_first=False, out_channel_first=False).shape == (0, 9, 4, 2)
    L = _lib.lib()
    assert L.ss2d_cross_scan_flex(None, None, 1, 1, 1, 1, 2, 2, 0, 0, 0, None) == _lib.SS2D_EINVAL
    assert L.ss2d_cross_scan_flex(None, None, 1, 1, 1, 1, 2, 0, 0, 0, 3, None) == _lib.SS2D_EINVAL
    assert L.ss2d_cross_merge_flex(None, None, 1, 1, 1, 1, 7, 0, 0, 0, 0, 0, None) == _lib.SS2D_EINVAL
