"""CrossScan / CrossMerge operator API, mirroring classification/models/csm_triton.py:501-517.

``cross_scan_fn`` and ``cross_merge_fn`` keep the reference's signatures and serve every layout and
mode of the reference (channel-first / channel-last on either side, one-by-one, ``scans`` 0/1/2)
on the HIP kernels in libss2d_hip.so through the C ABI: the combination the SS2D core uses --
channel-first in and out, not one-by-one, ``scans=0`` (vmamba.py:603, 632) -- and the
channel-first one-by-one scan on tiled kernels, everything else on the generic "flex" kernels.
``force_torch=True`` and CPU tensors raise: this package has no PyTorch or CPU path.

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


def _require_hip(what, scans, force_torch):
    if force_torch:
        raise NotImplementedError(f"{what}: force_torch=True asks for the PyTorch implementation, which this package does not ship")
    if scans not in (0, 1, 2):
        raise NotImplementedError(f"{what}: scans must be 0 (cross), 1 (unidirectional) or 2 (bidirectional), got {scans}")


def _flex_dims(t, channel_first, one_by_one, what):
    """(B, C, H, W) of an x-side / merge-input tensor: (B,[4,]C,H,W) or (B,H,W,[4,]C)."""
    want = 5 if one_by_one else 4
    if t.dim() != want or (one_by_one and t.shape[1 if channel_first else 3] != 4):
        raise ValueError(f"{what}: expected a {'(B,4,C,H,W)' if channel_first else '(B,H,W,4,C)'} tensor"
                         f"{'' if one_by_one else ' without the direction axis'}, got {tuple(t.shape)}")
    if channel_first:
        return t.shape[0], t.shape[-3], t.shape[-2], t.shape[-1]
    return t.shape[0], t.shape[-1], t.shape[1], t.shape[2]


def transpose_bcl_hip(x):
    """(B, R, S) -> (B, S, R) contiguous (ss2d_transpose_bcl)."""
    x = x.contiguous()
    B, R, S = x.shape
    y = x.new_empty((B, S, R))
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_transpose_bcl(x.data_ptr(), y.data_ptr(), B, R, S, x.element_size(), _stream(x))
    _lib.check(rc, "ss2d_transpose_bcl")
    return y


def cross_scan_flex_hip(x, in_channel_first=True, out_channel_first=True, one_by_one=False, scans=0):
    """Any layout / mode of CrossScan; bit-exact for any 1/2/4/8-byte dtype.  Mixed layouts go through
    ss2d_cross_scan_flex_ws, which first brings x (the small side) to the layout of y with one tiled transpose into a
    staging buffer allocated here, then runs the same-layout kernel."""
    _require_gpu(x, "cross_scan")
    B, C, H, W = _flex_dims(x, in_channel_first, one_by_one, "cross_scan")
    x = x.contiguous()
    if in_channel_first != out_channel_first and x.numel():
        y = x.new_empty((B, 4, C, H * W) if out_channel_first else (B, H * W, 4, C))
        staging = torch.empty_like(x)          # one copy of x in the layout of y
        with torch.cuda.device(x.device):
            rc = _lib.lib().ss2d_cross_scan_flex_ws(x.data_ptr(), y.data_ptr(), B, C, H, W, x.element_size(),
                                                    0 if in_channel_first else 1, 0 if out_channel_first else 1,
                                                    1 if one_by_one else 0, scans, staging.data_ptr(),
                                                    staging.numel() * staging.element_size(), _stream(x))
        _lib.check(rc, "ss2d_cross_scan_flex_ws")
        return y
    y = x.new_empty((B, 4, C, H * W) if out_channel_first else (B, H * W, 4, C))
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_cross_scan_flex(x.data_ptr(), y.data_ptr(), B, C, H, W, x.element_size(),
                                             0 if in_channel_first else 1, 0 if out_channel_first else 1,
                                             1 if one_by_one else 0, scans, _stream(x))
    _lib.check(rc, "ss2d_cross_scan_flex")
    return y


def cross_merge_flex_hip(y, in_channel_first=True, out_channel_first=True, one_by_one=False, scans=0,
                         order=_lib.MERGE_PAIRWISE):
    """Any layout / mode of CrossMerge (ss2d_cross_merge_flex): y (B,4,C,H,W) | (B,H,W,4,C) ->
    (B,[4,]C,L) | (B,L,[4,]C)."""
    _require_gpu(y, "cross_merge")
    B, C, H, W = _flex_dims(y, out_channel_first, True, "cross_merge")
    if y.dtype not in _DTYPE_CODE:
        raise TypeError(f"cross_merge: unsupported dtype {y.dtype}")
    y = y.contiguous()
    L = H * W
    if in_channel_first != out_channel_first and y.numel():
        # mixed layouts: merge in the layout of y, then bring the (small) result to the other layout
        x = cross_merge_flex_hip(y, out_channel_first, out_channel_first, one_by_one, scans, order)
        K = 4 if one_by_one else 1
        if out_channel_first:     # (B, K*C, L) -> (B, L, K*C)
            return transpose_bcl_hip(x.view(B, K * C, L)).view((B, L, 4, C) if one_by_one else (B, L, C))
        return transpose_bcl_hip(x.view(B, L, K * C)).view((B, 4, C, L) if one_by_one else (B, C, L))
    if in_channel_first and out_channel_first and (not one_by_one) and scans == 0:
        return cross_merge_hip(y, order)
    if one_by_one:
        x = y.new_empty((B, 4, C, L) if in_channel_first else (B, L, 4, C))
    else:
        x = y.new_empty((B, C, L) if in_channel_first else (B, L, C))
    with torch.cuda.device(y.device):
        rc = _lib.lib().ss2d_cross_merge_flex(y.data_ptr(), x.data_ptr(), B, C, H, W, _DTYPE_CODE[y.dtype],
                                              0 if in_channel_first else 1, 0 if out_channel_first else 1,
                                              1 if one_by_one else 0, scans, order, _stream(y))
    _lib.check(rc, "ss2d_cross_merge_flex")
    return x


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


class CrossScanFlexHip(torch.autograd.Function):
    """Any mode; the two operators are each other's adjoint for every mode (csm_triton.py:208-225, 249-273)."""
    @staticmethod
    def forward(ctx, x, in_channel_first, out_channel_first, one_by_one, scans):
        ctx.mode = (in_channel_first, out_channel_first, one_by_one, scans)
        ctx.dims = _flex_dims(x, in_channel_first, one_by_one, "cross_scan")
        if in_channel_first and out_channel_first and one_by_one and scans == 0:
            return cross_scan_1b1_hip(x)
        return cross_scan_flex_hip(x, in_channel_first, out_channel_first, one_by_one, scans)

    @staticmethod
    def backward(ctx, grad_y):
        icf, ocf, obo, scans = ctx.mode
        B, C, H, W = ctx.dims
        g = grad_y.reshape(B, 4, C, H, W) if ocf else grad_y.reshape(B, H, W, 4, C)
        gx = cross_merge_flex_hip(g, icf, ocf, obo, scans)
        if obo:
            gx = gx.view(B, 4, C, H, W) if icf else gx.view(B, H, W, 4, C)
        else:
            gx = gx.view(B, C, H, W) if icf else gx.view(B, H, W, C)
        return gx, None, None, None, None


class CrossMergeFlexHip(torch.autograd.Function):
    @staticmethod
    def forward(ctx, y, in_channel_first, out_channel_first, one_by_one, scans):
        ctx.mode = (in_channel_first, out_channel_first, one_by_one, scans)
        ctx.dims = _flex_dims(y, out_channel_first, True, "cross_merge")
        return cross_merge_flex_hip(y, in_channel_first, out_channel_first, one_by_one, scans)

    @staticmethod
    def backward(ctx, grad_x):
        icf, ocf, obo, scans = ctx.mode
        B, C, H, W = ctx.dims
        if obo:
            g = grad_x.reshape(B, 4, C, H, W) if icf else grad_x.reshape(B, H, W, 4, C)
        else:
            g = grad_x.reshape(B, C, H, W) if icf else grad_x.reshape(B, H, W, C)
        gy = cross_scan_flex_hip(g, icf, ocf, obo, scans)
        return (gy.view(B, 4, C, H, W) if ocf else gy.view(B, H, W, 4, C)), None, None, None, None


def cross_scan_fn(x, in_channel_first=True, out_channel_first=True, one_by_one=False, scans=0, force_torch=False):
    # x: (B, C, H, W) | (B, H, W, C) | (B, 4, C, H, W) | (B, H, W, 4, C)
    # y: (B, 4, C, L) | (B, L, 4, C)
    # scans: 0: cross scan; 1 unidirectional; 2: bidirectional;
    _require_hip("cross_scan_fn", scans, force_torch)
    if in_channel_first and out_channel_first and (not one_by_one) and scans == 0:
        return CrossScanHip.apply(x)
    return CrossScanFlexHip.apply(x, in_channel_first, out_channel_first, one_by_one, scans)


def cross_merge_fn(y, in_channel_first=True, out_channel_first=True, one_by_one=False, scans=0, force_torch=False):
    # y: (B, 4, C, H, W) | (B, H, W, 4, C)
    # x: (B, C, H * W) | (B, H * W, C) | (B, 4, C, H * W) | (B, H * W, 4, C)
    _require_hip("cross_merge_fn", scans, force_torch)
    if in_channel_first and out_channel_first and (not one_by_one) and scans == 0:
        return CrossMergeHip.apply(y)
    return CrossMergeFlexHip.apply(y, in_channel_first, out_channel_first, one_by_one, scans)
