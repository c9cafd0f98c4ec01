"""GPU parity of the LayerNorm kernels against torch's CPU layer_norm (the call the reference makes,
classification/models/vmamba.py:52-57).  fp32 output: rtol/atol 1e-4 (rsqrt and summation order differ in the
last bits); 16-bit output: one unit in the last place of the 16-bit type (rtol 2^-7 bf16, 2^-10 f16)."""
import pytest
import torch

from oracle import torch_ref
from vmamba_amd import _lib
from vmamba_amd.norm import (LayerNorm, LayerNorm2d, add_layer_norm_fusable, add_layer_norm_hip, bias_layer_norm_fusable,
                             bias_layer_norm_hip, layer_norm_cf_hip,
                             layer_norm_hip)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tol(dtype):
    return {torch.float32: dict(rtol=1e-4, atol=1e-4), torch.bfloat16: dict(rtol=2 ** -7, atol=2 ** -7),
            torch.float16: dict(rtol=2 ** -10, atol=2 ** -10)}[dtype]


def _dev(t):
    return None if t is None else t.to(DEV)


ROWS = [(1, 8), (3, 48), (401, 96), (77, 192), (50, 384), (33, 768), (9, 1024), (5, 1032), (4, 2048), (7, 100), (6, 3), (2, 1), (300, 16)]
TRIPLES = [(torch.float32, torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16, torch.bfloat16),
           (torch.float32, torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32, torch.bfloat16),
           (torch.bfloat16, torch.float32, torch.bfloat16), (torch.float16, torch.float16, torch.float16)]


@pytest.mark.parametrize("rows,C", ROWS)
@pytest.mark.parametrize("in_dt,w_dt,out_dt", TRIPLES)
def test_layer_norm_rows(rows, C, in_dt, w_dt, out_dt):
    print("CASE ln-rows", rows, C, in_dt, w_dt, out_dt, flush=True)
    g = torch.Generator().manual_seed(41)
    x = (torch.randn(rows, C, generator=g) * 2 + 0.5).to(in_dt)
    w, b = (torch.randn(C, generator=g) + 1).to(w_dt), torch.randn(C, generator=g).to(w_dt)
    want = torch_ref.layer_norm_rows(x, w, b, 1e-5, out_dt)
    got = layer_norm_hip(_dev(x), _dev(w), _dev(b), 1e-5, out_dtype=out_dt).cpu()
    assert got.dtype == want.dtype and got.shape == want.shape
    assert torch.allclose(got.float(), want.float(), **_tol(out_dt))


@pytest.mark.parametrize("rows,C", [(1, 8), (401, 96), (77, 192), (128 * 196, 384), (33, 768), (9, 1024)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_add_layer_norm_is_the_add_then_the_norm(rows, C, dt):
    """sum bit-identical to the separate add (one rounding to the tensor type); the norm as the rows kernel's."""
    print("CASE add-ln", rows, C, dt, flush=True)
    g = torch.Generator().manual_seed(rows + C)
    x = (torch.randn(rows, C, generator=g) * 2 + 0.5).to(dt)
    r = torch.randn(rows, C, generator=g).to(dt)
    w, b = (torch.randn(C, generator=g) + 1).to(dt), torch.randn(C, generator=g).to(dt)
    total, normed = add_layer_norm_hip(_dev(x), _dev(r), _dev(w), _dev(b), 1e-6)
    want_total = x + r
    assert torch.equal(total.cpu(), want_total)
    want = torch_ref.layer_norm_rows(want_total, w, b, 1e-6, dt)
    assert torch.allclose(normed.cpu().float(), want.float(), **_tol(dt))
    assert torch.equal(normed, layer_norm_hip(total, _dev(w), _dev(b), 1e-6))


def test_add_layer_norm_rejections():
    x = torch.randn(4, 100, device=DEV).bfloat16()          # C % 8 != 0: no fused kernel
    assert not add_layer_norm_fusable(x, x)
    with pytest.raises(_lib.Ss2dError):
        add_layer_norm_hip(x, x, None, None)
    with pytest.raises(ValueError):
        add_layer_norm_hip(x, x[:2], None, None)
    with pytest.raises(NotImplementedError):
        add_layer_norm_hip(x.cpu(), x.cpu(), None, None)
    assert _lib.lib().ss2d_add_layer_norm(x.data_ptr(), None, None, None, x.data_ptr(), x.data_ptr(), 4, 96, 1e-5, 1, 1, 1, None) == _lib.SS2D_EINVAL


@pytest.mark.parametrize("rows,C", [(3, 8), (500, 48), (401, 96), (77, 192), (50, 384), (33, 768), (9, 1024)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_bias_layer_norm_is_the_add_then_the_norm(rows, C, dt):
    """LayerNorm(x + per-channel bias) in one kernel: bit-identical to the rows kernel applied to the separately added
    (and rounded) sum, and within tolerance of the torch reference."""
    print("CASE bias-ln", rows, C, dt, flush=True)
    g = torch.Generator().manual_seed(7 * rows + C)
    x = (torch.randn(rows, C, generator=g) * 2 + 0.5).to(dt)
    pb = torch.randn(C, generator=g).to(dt)
    w, b = (torch.randn(C, generator=g) + 1).to(dt), torch.randn(C, generator=g).to(dt)
    got = bias_layer_norm_hip(_dev(x), _dev(pb), _dev(w), _dev(b), 1e-6)
    total = x + pb
    assert torch.equal(got, layer_norm_hip(_dev(total), _dev(w), _dev(b), 1e-6))
    assert torch.allclose(got.cpu().float(), torch_ref.layer_norm_rows(total, w, b, 1e-6, dt).float(), **_tol(dt))


def test_bias_layer_norm_rejections():
    x = torch.randn(4, 100, device=DEV).bfloat16()          # C % 8 != 0: no fused kernel
    assert not bias_layer_norm_fusable(x.dtype, 100) and bias_layer_norm_fusable(x.dtype, 96)
    with pytest.raises(_lib.Ss2dError):
        bias_layer_norm_hip(x, x[0], None, None)
    with pytest.raises(ValueError):
        bias_layer_norm_hip(x, x[0, :50], None, None)
    with pytest.raises(NotImplementedError):
        bias_layer_norm_hip(x.cpu(), x[0].cpu(), None, None)
    assert _lib.lib().ss2d_bias_layer_norm(x.data_ptr(), None, None, None, x.data_ptr(), 4, 96, 1e-5, 1, 1, 1, None) == _lib.SS2D_EINVAL


def test_layer_norm_rows_without_affine_and_known_answers():
    x = torch.randn(10, 96, generator=torch.Generator().manual_seed(42))
    got = layer_norm_hip(_dev(x), None, None).cpu()
    assert torch.allclose(got, torch_ref.layer_norm_rows(x, None, None), rtol=1e-4, atol=1e-4)
    assert torch.allclose(got.mean(-1), torch.zeros(10), atol=1e-5) and torch.allclose(got.var(-1, unbiased=False), torch.ones(10), atol=1e-3)
    const = layer_norm_hip(torch.full((2, 16), 3.0, device=DEV), torch.ones(16, device=DEV), torch.full((16,), 0.25, device=DEV))
    assert torch.equal(const.cpu(), torch.full((2, 16), 0.25))
    assert layer_norm_hip(torch.zeros(0, 8, device=DEV), None, None).shape == (0, 8)


# B, C, H, W
CF = [(2, 96, 56, 56), (2, 48, 5, 7), (3, 192, 28, 28), (2, 384, 14, 14), (2, 768, 7, 7), (1, 1000, 3, 3), (2, 7, 9, 4), (1, 96, 1, 1),
      (1, 1300, 3, 5), (1, 97, 8, 9), (2, 200, 3, 70), (1, 500, 6, 6), (2, 768, 6, 6), (3, 40, 2, 2), (1, 136, 4, 9),
      # short images, one workgroup per image or per share of one: odd maps (rows that are not 16-byte aligned), a last
      # lane group that holds fewer channels, maps of two and of one position, shares of unequal size
      (3, 40, 5, 5), (2, 24, 3, 3), (2, 16, 1, 2), (2, 100, 4, 4), (5, 104, 13, 4), (2, 8, 1, 1), (3, 72, 31, 1), (2, 20, 3, 3),
      (2, 384, 10, 10), (1, 192, 31, 33),
      # few channels on many positions: a workgroup with fewer threads than positions
      (1, 16, 6, 12), (2, 8, 8, 8), (1, 24, 9, 20), (3, 8, 16, 16),
      # rows wider than the register variants hold: the LDS-tile kernel with 8 and with 4 positions per workgroup (the
      # 2048 inner channels of the widest reference model; a tile beyond 64 KB of LDS)
      (2, 1600, 3, 3), (2, 2048, 7, 7), (1, 4000, 2, 5)]


@pytest.mark.parametrize("B,C,H,W", CF)
@pytest.mark.parametrize("in_dt,w_dt,out_dt", [(torch.float32, torch.float32, torch.float32),
                                               (torch.float32, torch.bfloat16, torch.bfloat16),
                                               (torch.bfloat16, torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("out_cl", [False, True])
def test_layer_norm_channel_first(B, C, H, W, in_dt, w_dt, out_dt, out_cl):
    print("CASE ln-cf", B, C, H, W, in_dt, w_dt, out_dt, out_cl, flush=True)
    g = torch.Generator().manual_seed(43)
    x = (torch.randn(B, C, H, W, generator=g) * 2 - 0.3).to(in_dt)
    w, b = (torch.randn(C, generator=g) + 1).to(w_dt), torch.randn(C, generator=g).to(w_dt)
    want = torch_ref.layer_norm_cf(x, w, b, 1e-5, out_cl, out_dt)
    got = layer_norm_cf_hip(_dev(x), _dev(w), _dev(b), 1e-5, out_channel_last=out_cl, out_dtype=out_dt).cpu()
    assert got.dtype == want.dtype and got.shape == want.shape
    assert torch.allclose(got.float(), want.float(), **_tol(out_dt))


@pytest.mark.parametrize("B,C,H,W", [(128, 192, 28, 28), (128, 384, 14, 14), (128, 768, 7, 7), (64, 384, 14, 14), (300, 768, 7, 7)])
def test_layer_norm_channel_first_benchmark_batches(B, C, H, W):
    """The out_norm shapes of the 224 x 224 model at the benchmark's batch (the split of an image over workgroups
    depends on the batch): fp32 scan output in, bf16 channel-last rows out, every image against the oracle."""
    print("CASE ln-cf-batch", B, C, H, W, flush=True)
    g = torch.Generator().manual_seed(44)
    x = torch.randn(B, C, H, W, generator=g) * 1.5 + 0.2
    w, b = (torch.randn(C, generator=g) + 1).bfloat16(), torch.randn(C, generator=g).bfloat16()
    want = torch_ref.layer_norm_cf(x, w, b, 1e-5, True, torch.bfloat16)
    got = layer_norm_cf_hip(_dev(x), _dev(w), _dev(b), 1e-5, out_channel_last=True, out_dtype=torch.bfloat16).cpu()
    assert got.shape == want.shape and torch.allclose(got.float(), want.float(), **_tol(torch.bfloat16))
    got_cf = layer_norm_cf_hip(_dev(x), _dev(w), _dev(b), 1e-5, out_channel_last=False, out_dtype=torch.bfloat16).cpu()
    assert torch.equal(got_cf.permute(0, 2, 3, 1), got)


@pytest.mark.parametrize("B,C,H,W", [(3, 384, 14, 14), (2, 768, 7, 7), (2, 96, 56, 56), (2, 40, 5, 5)])
@pytest.mark.parametrize("out_cl", [False, True])
def test_layer_norm_channel_first_without_affine_and_views(B, C, H, W, out_cl):
    """No weight / no bias on every channel-first kernel, zero-size batches, and a non-contiguous input (made
    contiguous by the wrapper): per-position mean 0 and variance 1 besides the oracle."""
    g = torch.Generator().manual_seed(45)
    x = torch.randn(B, C, H, W, generator=g) * 3 + 1
    got = layer_norm_cf_hip(_dev(x), None, None, 1e-5, out_channel_last=out_cl).cpu()
    want = torch_ref.layer_norm_cf(x, None, None, 1e-5, out_cl, torch.float32)
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-4)
    axis = -1 if out_cl else 1
    assert torch.allclose(got.mean(axis), torch.zeros(()), atol=1e-5) and torch.allclose(got.var(axis, unbiased=False), torch.ones(()), atol=1e-3)
    w = torch.randn(C, generator=g)
    only_w = layer_norm_cf_hip(_dev(x), _dev(w), None, 1e-5, out_channel_last=out_cl).cpu()
    assert torch.allclose(only_w, torch_ref.layer_norm_cf(x, w, None, 1e-5, out_cl, torch.float32), rtol=1e-4, atol=1e-4)
    xt = x.transpose(2, 3)                                   # a view: (B, C, W, H), not contiguous
    got_t = layer_norm_cf_hip(_dev(xt), None, None, 1e-5, out_channel_last=out_cl).cpu()
    assert torch.allclose(got_t, torch_ref.layer_norm_cf(xt.contiguous(), None, None, 1e-5, out_cl, torch.float32), rtol=1e-4, atol=1e-4)
    assert layer_norm_cf_hip(_dev(x[:0]), None, None, out_channel_last=out_cl).numel() == 0


def test_modules_share_state_dict_with_torch():
    ln, ref = LayerNorm(24).to(DEV), torch.nn.LayerNorm(24)
    ref.weight.data.normal_(); ref.bias.data.normal_()
    ln.load_state_dict(ref.state_dict())
    x = torch.randn(3, 5, 24)
    assert torch.allclose(ln(x.to(DEV)).cpu(), ref(x), rtol=1e-4, atol=1e-4)
    ln2 = LayerNorm2d(24).to(DEV)
    ln2.load_state_dict(ref.state_dict())
    x2 = torch.randn(2, 24, 4, 6)
    assert torch.allclose(ln2(x2.to(DEV)).cpu(), ref(x2.permute(0, 2, 3, 1)).permute(0, 3, 1, 2), rtol=1e-4, atol=1e-4)
    with pytest.raises(NotImplementedError):
        ln.cpu()(x)


@pytest.mark.parametrize("rows,C", [(128 * 3136, 96), (128 * 49, 768)])
def test_layer_norm_full_size_properties(rows, C):
    """Stage shapes at batch 128: per-row mean 0 / variance 1 without affine, invariance to a per-row shift by a
    power of two... and a slice against the oracle."""
    print("CASE ln-full", rows, C, flush=True)
    g = torch.Generator(device=DEV).manual_seed(44)
    x = torch.randn(rows, C, generator=g, device=DEV).bfloat16()
    y = layer_norm_hip(x, None, None, out_dtype=torch.float32) if False else layer_norm_hip(x.float(), None, None)
    assert torch.allclose(y.mean(-1), torch.zeros(rows, device=DEV), atol=1e-5)
    assert torch.allclose(y.var(-1, unbiased=False), torch.ones(rows, device=DEV), atol=1e-3)
    yb = layer_norm_hip(x, None, None)
    sl = slice(rows - 300, rows)
    assert torch.allclose(yb[sl].float().cpu(), torch_ref.layer_norm_rows(x[sl].cpu(), None, None).float(), rtol=2 ** -7, atol=2 ** -7)
