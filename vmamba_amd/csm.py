"""CrossScan / CrossMerge operator API, mirroring classification/models/csm_triton.py:501-517.

``cross_scan_fn`` and ``cross_merge_fn`` keep the reference's signatures.  The combination the
SS2D core uses -- channel-first in and out, not one-by-one, ``scans=0`` (vmamba.py:603, 632) --
runs on the HIP kernels in libss2d_hip.so through the C ABI, and so does the one-by-one CrossScan
(forward only).  Other layouts / scan modes raise NotImplementedError; CPU tensors raise as well:
this package has no CPU path.

Both operators are each other's adjoint (csm_triton.py:208-225, 249-273), so autograd is
supported with the same two kernels.
"""
import torch

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.SS2D_F32, torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(t, what):
    if not t.is_cuda:
        raise NotImplementedError(f"{what}: vmamba_amd runs on the GPU only (got a {t.device.type} tensor)")


def _require_default_mode(what, in_channel_first, out_channel_first, one_by_one, scans, force_torch, allow_1b1=False):
    if force_torch:
        raise NotImplementedError(f"{what}: force_torch=True asks for the PyTorch implementation, which this package does not ship")
    if not (in_channel_first and out_channel_first and (allow_1b1 or not one_by_one) and scans == 0):
        raise NotImplementedError(
            f"{what}: only in_channel_first=True, out_channel_first=True, one_by_one=False, scans=0 has a HIP kernel "
            f"(got {in_channel_first}, {out_channel_first}, {one_by_one}, {scans})")


def cross_scan_hip(x):
    """x (B,C,H,W) -> (B,4,C,H*W), any 1/2/4/8-byte dtype, bit-exact permutation."""
    _require_gpu(x, "cross_scan")
    if x.dim() != 4:
        raise ValueError(f"cross_scan expects (B,C,H,W), got {tuple(x.shape)}")
    x = x.contiguous()
    B, C, H, W = x.shape
    y = x.new_empty((B, 4, C, H * W))
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_cross_scan(x.data_ptr(), y.data_ptr(), B, C, H, W, x.element_size(), _stream(x))
    _lib.check(rc, "ss2d_cross_scan")
    return y


def cross_scan_1b1_hip(x, out=None):
    """One-by-one CrossScan: x (B,4,C,H,W) -> (B,4,C,H*W), direction slice k in its own scan order.

    ``out``, if given, is any view of shape (B,4,C,H*W) whose last stride is 1 (e.g. a permuted
    (4,C,B,L) buffer): the kernel writes through its batch / direction / channel strides."""
    _require_gpu(x, "cross_scan (one_by_one)")
    if x.dim() != 5 or x.shape[1] != 4:
        raise ValueError(f"one-by-one cross_scan expects (B,4,C,H,W), got {tuple(x.shape)}")
    x = x.contiguous()
    B, K, C, H, W = x.shape
    if out is None:
        out = x.new_empty((B, 4, C, H * W))
    if tuple(out.shape) != (B, 4, C, H * W) or out.dtype != x.dtype or out.device != x.device:
        raise ValueError(f"out must be a {(B, 4, C, H * W)} {x.dtype} tensor on {x.device}")
    if out.numel() and H * W > 1 and out.stride(3) != 1:
        raise ValueError("out must be contiguous in its last dimension")
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_cross_scan_1b1(x.data_ptr(), out.data_ptr(), B, C, H, W, x.element_size(), out.stride(0),
                                            out.stride(1), out.stride(2), _stream(x))
    _lib.check(rc, "ss2d_cross_scan_1b1")
    return out


def cross_merge_hip(ys, order=_lib.MERGE_PAIRWISE):
    """ys (B,4,C,H,W) -> (B,C,H*W); adds rounded to ys.dtype in the order of cross_merge_fwd."""
    _require_gpu(ys, "cross_merge")
    if ys.dim() != 5 or ys.shape[1] != 4:
        raise ValueError(f"cross_merge expects (B,4,C,H,W), got {tuple(ys.shape)}")
    if ys.dtype not in _DTYPE_CODE:
        raise TypeError(f"cross_merge: unsupported dtype {ys.dtype}")
    ys = ys.contiguous()
    B, K, C, H, W = ys.shape
    out = ys.new_empty((B, C, H * W))
    with torch.cuda.device(ys.device):
        rc = _lib.lib().ss2d_cross_merge(ys.data_ptr(), out.data_ptr(), B, C, H, W, _DTYPE_CODE[ys.dtype], order, _stream(ys))
    _lib.check(rc, "ss2d_cross_merge")
    return out


class CrossScanHip(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.shape = x.shape
        return cross_scan_hip(x)

    @staticmethod
    def backward(ctx, grad_y):
        B, C, H, W = ctx.shape
        return cross_merge_hip(grad_y.reshape(B, 4, C, H, W)).view(B, C, H, W)


class CrossMergeHip(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ys):
        ctx.shape = ys.shape
        return cross_merge_hip(ys)

    @staticmethod
    def backward(ctx, grad_out):
        B, K, C, H, W = ctx.shape
        return cross_scan_hip(grad_out.reshape(B, C, H, W)).view(B, 4, C, H, W)


class CrossScan1b1Hip(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        return cross_scan_1b1_hip(x)

    @staticmethod
    def backward(ctx, grad_y):
        raise NotImplementedError("one-by-one cross_scan: forward only (its adjoint, the one-by-one merge, has no HIP kernel)")


def cross_scan_fn(x, in_channel_first=True, out_channel_first=True, one_by_one=False, scans=0, force_torch=False):
    # x: (B, C, H, W) -> y: (B, 4, C, L);  one_by_one: x (B, 4, C, H, W)
    _require_default_mode("cross_scan_fn", in_channel_first, out_channel_first, one_by_one, scans, force_torch, allow_1b1=True)
    return CrossScan1b1Hip.apply(x) if one_by_one else CrossScanHip.apply(x)


def cross_merge_fn(y, in_channel_first=True, out_channel_first=True, one_by_one=False, scans=0, force_torch=False):
    # y: (B, 4, C, H, W) -> (B, C, L)
    _require_default_mode("cross_merge_fn", in_channel_first, out_channel_first, one_by_one, scans, force_torch)
    return CrossMergeHip.apply(y)
