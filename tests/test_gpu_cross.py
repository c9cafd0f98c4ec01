"""GPU parity of CrossScan / CrossMerge against the CPU oracle: bit-exact (torch.equal)."""
import json
import os

import pytest
import torch

from oracle import ss2d_oracle as orc
from oracle import torch_ref
import vmamba_amd as va
from vmamba_amd import _lib
from vmamba_amd.csm import cross_merge_hip, cross_scan_hip

pytestmark = pytest.mark.gpu

DEV = "cuda:0"

# (B, C, H, W): SS2D stage shapes, the reference's odd shapes (csm_triton.py:524, 670), degenerate
# strips, maps that need the tiled kernels (large H*W) and partial tiles.
SHAPES = [
    (1, 1, 1, 1), (2, 3, 3, 5), (3, 5, 7, 7), (2, 9, 14, 14), (2, 6, 28, 28), (2, 96, 56, 56),
    (3, 5, 56, 57), (2, 7, 57, 58), (130, 3, 1, 1), (2, 3, 1, 37), (2, 3, 41, 1),
    (1, 2, 200, 130), (1, 3, 128, 128), (1, 1, 256, 256), (1, 2, 65, 300),
    # odd maps with an even channel count (16-bit elements then travel as pairs across map boundaries): one group, several
    # groups with a short last one, single positions
    (2, 6, 7, 7), (3, 10, 5, 9), (1, 2, 1, 1), (2, 4, 3, 3), (2, 170, 7, 7), (1, 86, 7, 7), (2, 768, 7, 7),
    # ... and with a multiple of 8 channels (16-byte vectors across map boundaries): one group, a short last group, maps of
    # more than 256 positions, several groups of 8
    (2, 8, 7, 7), (1, 96, 7, 7), (3, 16, 5, 9), (2, 8, 3, 3), (1, 8, 17, 17), (1, 24, 17, 17), (2, 104, 7, 7),
]


def _announce(*what):
    print("CASE", *what, flush=True)


@pytest.fixture(scope="module")
def kat(golden_dir):
    with open(os.path.join(golden_dir, "cross_scan_kat.json")) as f:
        return json.load(f)


def test_known_answers_on_gpu(kat):
    for case in kat["scan"]:
        H, W = case["H"], case["W"]
        _announce("kat", H, W)
        x = torch.tensor(case["x"], dtype=torch.float32, device=DEV).view(1, 1, H, W)
        y = va.cross_scan_fn(x)
        assert y.view(4, -1).cpu().tolist() == [[float(v) for v in row] for row in case["y"]]
        assert va.cross_merge_fn(y.view(1, 4, 1, H, W)).view(-1).cpu().tolist() == [float(v) for v in case["merged"]]
    m = kat["merge"]
    ys = torch.tensor(m["ys"], dtype=torch.float32, device=DEV).view(1, 4, 1, m["H"], m["W"])
    assert va.cross_merge_fn(ys).view(-1).cpu().tolist() == [float(v) for v in m["out"]]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.int64, torch.uint8])
def test_cross_scan_bit_exact(shape, dtype):
    _announce("cross_scan", shape, dtype)
    g = torch.Generator().manual_seed(11)
    if dtype.is_floating_point:
        x = torch.randn(shape, generator=g).to(dtype)
    else:
        x = torch.randint(0, 255, shape, generator=g).to(dtype)
    want = orc.cross_scan(x)
    got = cross_scan_hip(x.to(DEV))
    torch.cuda.synchronize()
    assert got.shape == want.shape and got.dtype == want.dtype
    assert torch.equal(got.cpu().view(torch.uint8), want.view(torch.uint8))


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("order", [_lib.MERGE_PAIRWISE, _lib.MERGE_LEFT_TO_RIGHT])
def test_cross_merge_bit_exact(shape, dtype, order):
    _announce("cross_merge", shape, dtype, order)
    B, C, H, W = shape
    g = torch.Generator().manual_seed(12)
    ys = torch.randn((B, 4, C, H, W), generator=g).to(dtype)
    if dtype == torch.float16:   # the C oracle has no f16; the torch restatement rounds the same way
        want = torch_ref.cross_merge(ys) if order == 0 else torch_ref.cross_merge_left_to_right(ys)
    else:
        want = orc.cross_merge(ys, order=order)
    got = cross_merge_hip(ys.to(DEV), order=order)
    torch.cuda.synchronize()
    assert got.shape == want.shape and got.dtype == want.dtype
    assert torch.equal(got.cpu(), want)


def test_merge_add_order_on_gpu():
    y = torch.zeros(1, 4, 1, 1, 1)
    y[0, 0], y[0, 1], y[0, 2], y[0, 3] = 1.0, 2.0 ** -24, -1.0, 2.0 ** -24
    assert cross_merge_hip(y.to(DEV)).item() == 2.0 ** -23
    assert cross_merge_hip(y.to(DEV), order=_lib.MERGE_LEFT_TO_RIGHT).item() == 2.0 ** -24
    yb = torch.zeros(1, 4, 1, 1, 1, dtype=torch.bfloat16)
    yb[0, 0], yb[0, 1], yb[0, 2], yb[0, 3] = 1.0, 2.0 ** -9, -1.0, 2.0 ** -9
    assert cross_merge_hip(yb.to(DEV)).item() == 2.0 ** -8
    assert cross_merge_hip(yb.to(DEV), order=_lib.MERGE_LEFT_TO_RIGHT).item() == 2.0 ** -9


def test_empty_inputs():
    assert va.cross_scan_fn(torch.zeros(0, 3, 4, 4, device=DEV)).shape == (0, 4, 3, 16)
    assert va.cross_scan_fn(torch.zeros(2, 0, 4, 4, device=DEV)).shape == (2, 4, 0, 16)
    assert va.cross_merge_fn(torch.zeros(0, 4, 3, 4, 4, device=DEV)).shape == (0, 3, 16)


def test_non_contiguous_input_is_made_contiguous():
    g = torch.Generator().manual_seed(13)
    x = torch.randn(2, 14, 14, 6, generator=g)
    got = va.cross_scan_fn(x.to(DEV).permute(0, 3, 1, 2))          # channel-last storage, channel-first view
    assert torch.equal(got.cpu(), orc.cross_scan(x.permute(0, 3, 1, 2).contiguous()))


def test_autograd_is_the_adjoint():
    g = torch.Generator().manual_seed(14)
    x = torch.randint(-4, 4, (2, 3, 5, 6), generator=g).float().to(DEV).requires_grad_()
    gy = torch.randint(-4, 4, (2, 4, 3, 30), generator=g).float().to(DEV)
    va.cross_scan_fn(x).backward(gy)
    assert torch.equal(x.grad.cpu(), orc.cross_merge(gy.cpu().view(2, 4, 3, 5, 6)).view(2, 3, 5, 6))
    ys = torch.randint(-4, 4, (2, 4, 3, 5, 6), generator=g).float().to(DEV).requires_grad_()
    go = torch.randint(-4, 4, (2, 3, 30), generator=g).float().to(DEV)
    va.cross_merge_fn(ys).backward(go)
    assert torch.equal(ys.grad.cpu(), orc.cross_scan(go.cpu().view(2, 3, 5, 6)).view(2, 4, 3, 5, 6))


@pytest.mark.parametrize("shape,dtype", [((128, 96, 56, 56), torch.bfloat16), ((128, 192, 28, 28), torch.bfloat16),
                                         ((128, 384, 14, 14), torch.bfloat16), ((128, 768, 7, 7), torch.bfloat16),
                                         ((4, 96, 256, 256), torch.bfloat16), ((64, 96, 56, 56), torch.float32)])
def test_full_size_properties(shape, dtype):
    """At benchmark sizes: merge(scan(x)) == 4x exactly, every direction is the stated permutation of x
    (checked through library flips/transposes on the GPU), and one image matches the oracle."""
    _announce("full", shape, dtype)
    B, C, H, W = shape
    g = torch.Generator(device=DEV).manual_seed(15)
    x = torch.randn(shape, generator=g, device=DEV).to(dtype)
    y = va.cross_scan_fn(x)
    L = H * W
    assert torch.equal(y[:, 0], x.view(B, C, L))
    assert torch.equal(y[:, 1], x.transpose(2, 3).reshape(B, C, L))
    assert torch.equal(y[:, 2], x.view(B, C, L).flip(-1))
    assert torch.equal(y[:, 3], x.transpose(2, 3).reshape(B, C, L).flip(-1))
    back = va.cross_merge_fn(y.view(B, 4, C, H, W))
    assert torch.equal(back.view(shape).float(), 4 * x.float())
    b = B - 1
    assert torch.equal(y[b:b + 1].cpu(), orc.cross_scan(x[b:b + 1].cpu()))
    if dtype in (torch.float32, torch.bfloat16):
        ys = torch.randn((1, 4, C, H, W), generator=g, device=DEV).to(dtype)
        assert torch.equal(va.cross_merge_fn(ys).cpu(), orc.cross_merge(ys.cpu()))
