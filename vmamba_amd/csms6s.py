"""Selective-scan operator API, mirroring classification/models/csms6s.py:71-126.

``selective_scan_fn(u, delta, A, B, C, D, delta_bias, delta_softplus, oflex, backend)`` keeps
the reference's positional signature.  The forward runs the HIP scan in libss2d_hip.so; there
is no torch or CPU implementation here, so ``backend="torch"`` and CPU tensors raise.  The
argument checks are those of selective_scan_fwd / selective_scan_bwd
(kernels/selective_scan/csrc/selective_scan/cusoflex/selective_scan_oflex.cpp:152-204, 244-300) and fail
with RuntimeError as the reference's TORCH_CHECKs do.  The backward runs on the HIP kernel as well, so the
operator trains.
"""
import torch

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.SS2D_F32, torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}
MAX_DSTATE = 256


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _scan_params(u, delta, A, B, C, D, delta_bias, delta_softplus, out, x):
    """struct ss2d_scan_params for these tensors (shapes and dtypes already checked)."""
    p = _lib.ScanParams()
    p.batch, p.dim, p.seqlen = u.shape
    p.dstate, p.n_groups, p.delta_dim = A.size(1), B.size(1), delta.size(1)
    p.in_dtype, p.out_dtype = _DTYPE_CODE[u.dtype], _DTYPE_CODE[out.dtype]
    p.delta_softplus = int(bool(delta_softplus))
    p.u, p.delta, p.A, p.B, p.C = u.data_ptr(), delta.data_ptr(), A.data_ptr(), B.data_ptr(), C.data_ptr()
    p.D = D.data_ptr() if D is not None else None
    p.delta_bias = delta_bias.data_ptr() if delta_bias is not None else None
    p.out = out.data_ptr()
    p.x = x.data_ptr() if x is not None else None
    p.u_batch_stride, p.u_d_stride = u.stride(0), u.stride(1)
    p.delta_batch_stride, p.delta_d_stride = delta.stride(0), delta.stride(1)
    p.A_d_stride, p.A_dstate_stride = A.stride(0), A.stride(1)
    p.B_batch_stride, p.B_group_stride, p.B_dstate_stride = B.stride(0), B.stride(1), B.stride(2)
    p.C_batch_stride, p.C_group_stride, p.C_dstate_stride = C.stride(0), C.stride(1), C.stride(2)
    p.out_batch_stride, p.out_d_stride = out.stride(0), out.stride(1)
    return p


def scan_kernel_name(u, delta, A, B, C, out, x=None):
    """Which kernel of the library serves these (already allocated) tensors: one of _lib.SCAN_KERNEL_NAMES.  Nothing
    is launched (ss2d_selective_scan_kernel)."""
    rc = _lib.lib().ss2d_selective_scan_kernel(_scan_params(u, delta, A, B, C, None, None, True, out, x))
    _lib.check(min(rc, 0), "ss2d_selective_scan_kernel")
    return _lib.SCAN_KERNEL_NAMES[rc]


def selective_scan_fwd(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False, nrows=1, out_float=True,
                       want_x=True):
    """Python twin of ``selective_scan_cuda_oflex.fwd``: returns [out, x].

    out (batch, dim, L) is fp32 when ``out_float`` else u.dtype; x (batch, dim, n_chunks, 2N)
    holds the chunk-end states (None when ``want_x`` is False).  ``nrows`` is accepted and
    ignored, as in the reference (selective_scan_oflex.cpp:224-226).
    """
    _check(u.dtype in _DTYPE_CODE, f"selective_scan_fwd not implemented for input type '{u.dtype}'")
    _check(A.dtype == torch.float32, "A must be float32")
    _check(delta.dtype == u.dtype and B.dtype == u.dtype and C.dtype == u.dtype, "delta, B, C must have u's dtype")
    for name, t in (("u", u), ("delta", delta), ("A", A), ("B", B), ("C", C)):
        _check(t.is_cuda, f"{name} must be a GPU tensor: vmamba_amd has no CPU path")
    _check(u.dim() == 3 and delta.dim() == 3 and A.dim() == 2 and B.dim() == 4 and C.dim() == 4, "bad tensor ranks")
    _check(u.stride(-1) == 1 or u.size(-1) == 1, "u must be contiguous in its last dimension")
    _check(delta.stride(-1) == 1 or delta.size(-1) == 1, "delta must be contiguous in its last dimension")
    batch, dim, seqlen = u.shape
    dstate, n_groups, delta_dim = A.size(1), B.size(1), delta.size(1)
    _check(dim % n_groups == 0, "dims should be dividable by n_groups")
    _check(dim % delta_dim == 0, "dims should be dividable by delta_dim")
    _check(dstate <= MAX_DSTATE, "selective_scan only supports state dimension <= 256")
    _check(tuple(delta.shape) == (batch, delta_dim, seqlen), "delta must have shape (batch_size, delta_dim, seqlen)")
    _check(tuple(A.shape) == (dim, dstate), "A must have shape (dim, dstate)")
    _check(tuple(B.shape) == (batch, n_groups, dstate, seqlen), "B must have shape (batch_size, n_groups, dstate, seqlen)")
    _check(tuple(C.shape) == (batch, n_groups, dstate, seqlen), "C must have shape (batch_size, n_groups, dstate, seqlen)")
    _check(B.stride(-1) == 1 or B.size(-1) == 1, "B must be contiguous in its last dimension")
    _check(C.stride(-1) == 1 or C.size(-1) == 1, "C must be contiguous in its last dimension")
    if D is not None:
        _check(D.dtype == torch.float32 and D.is_cuda, "D must be a float32 GPU tensor")
        _check(tuple(D.shape) == (dim,), "D must have shape (dim)")
        D = D.contiguous()
    if delta_bias is not None:
        _check(delta_bias.dtype == torch.float32 and delta_bias.is_cuda, "delta_bias must be a float32 GPU tensor")
        _check(tuple(delta_bias.shape) == (delta_dim,), "delta_bias must have shape (delta_dim)")
        delta_bias = delta_bias.contiguous()

    n_chunks = (seqlen + _lib.SCAN_CHUNK - 1) // _lib.SCAN_CHUNK
    out = torch.empty((batch, dim, seqlen), device=u.device, dtype=torch.float32 if out_float else u.dtype)
    x = torch.empty((batch, dim, n_chunks, dstate * 2), device=u.device, dtype=torch.float32) if want_x else None

    p = _scan_params(u, delta, A, B, C, D, delta_bias, delta_softplus, out, x)
    with torch.cuda.device(u.device):
        rc = _lib.lib().ss2d_selective_scan_fwd(p, torch.cuda.current_stream(u.device).cuda_stream)
    _lib.check(rc, "ss2d_selective_scan_fwd")
    return [out, x]


def selective_scan_from_map(x, delta, A, B, C, D=None, delta_bias=None, delta_softplus=True, out_float=True):
    """``selective_scan_fwd(cross_scan_fn(x).view(batch, 4 * D, L), delta, ...)[0]`` without the four scan-ordered copies:
    x (batch, D, H, W) is read through CrossScan's routes inside the scan kernel (its transpose is made here, one small
    pass).  Inference only; several states per channel (ss2d_selective_scan_fwd_maps).  Raises Ss2dError with status
    SS2D_ENOTSUP for shapes that kernel does not take: the caller then runs cross_scan_fn and selective_scan_fn."""
    from .csm import transpose_bcl_hip
    _check(x.is_cuda and x.dim() == 4 and x.dtype in _DTYPE_CODE, "x must be a (batch, D, H, W) GPU tensor of a supported dtype")
    _check(A.dtype == torch.float32, "A must be float32")
    _check(delta.dtype == x.dtype and B.dtype == x.dtype and C.dtype == x.dtype, "delta, B, C must have x's dtype")
    batch, Dm, H, W = x.shape
    L, dim = H * W, 4 * Dm
    dstate = A.size(1)
    _check(tuple(delta.shape) == (batch, dim, L) and tuple(A.shape) == (dim, dstate), "delta must be (batch, 4 D, L) and A (4 D, dstate)")
    _check(tuple(B.shape) == (batch, 4, dstate, L) and tuple(C.shape) == (batch, 4, dstate, L), "B and C must be (batch, 4, dstate, L)")
    for name, t in (("delta", delta), ("B", B), ("C", C)):
        _check(t.is_cuda and (t.stride(-1) == 1 or t.size(-1) == 1), f"{name} must be a GPU tensor contiguous in its last dimension")
    if D is not None:
        _check(D.dtype == torch.float32 and D.is_cuda and tuple(D.shape) == (dim,), "D must be a float32 GPU tensor of shape (4 D)")
        D = D.contiguous()
    if delta_bias is not None:
        _check(delta_bias.dtype == torch.float32 and delta_bias.is_cuda and tuple(delta_bias.shape) == (dim,),
               "delta_bias must be a float32 GPU tensor of shape (4 D)")
        delta_bias = delta_bias.contiguous()
    x = x.contiguous()
    x_t = transpose_bcl_hip(x.view(batch * Dm, H, W))                       # every map as W x H
    out = torch.empty((batch, dim, L), device=x.device, dtype=torch.float32 if out_float else x.dtype)
    p = _scan_params(out, delta, A, B, C, D, delta_bias, delta_softplus, out, None)     # shapes of the scan; u set below
    p.in_dtype = _DTYPE_CODE[x.dtype]
    p.u = x.data_ptr()
    p.u_batch_stride, p.u_d_stride = Dm * L, L
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_selective_scan_fwd_maps(p, x_t.data_ptr(), torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_selective_scan_fwd_maps")
    return out


def selective_scan_bwd(u, delta, A, B, C, D, delta_bias, dout, x=None, delta_softplus=False, nrows=1):
    """Python twin of ``selective_scan_cuda_oflex.bwd``: returns [du, ddelta, dA, dB, dC, dD, ddelta_bias]
    (selective_scan_oflex.cpp:233-355).  ``x`` (the forward's chunk states) and ``nrows`` are accepted and unused:
    the kernel recomputes the states it needs."""
    _check(u.dtype in _DTYPE_CODE, f"selective_scan_bwd not implemented for input type '{u.dtype}'")
    _check(A.dtype == torch.float32, "A must be float32")
    _check(dout.dtype in (u.dtype, torch.float32), "dout must have u's dtype or be float32")
    _check(delta.dtype == u.dtype and B.dtype == u.dtype and C.dtype == u.dtype, "delta, B, C must have u's dtype")
    for name, t in (("u", u), ("delta", delta), ("A", A), ("B", B), ("C", C), ("dout", dout)):
        _check(t.is_cuda, f"{name} must be a GPU tensor: vmamba_amd has no CPU path")
    for name, t in (("u", u), ("delta", delta), ("dout", dout), ("B", B), ("C", C)):
        _check(t.stride(-1) == 1 or t.size(-1) == 1, f"{name} must be contiguous in its last dimension")
    batch, dim, seqlen = u.shape
    dstate, n_groups, delta_dim = A.size(1), B.size(1), delta.size(1)
    _check(dim % n_groups == 0, "dims should be dividable by n_groups")
    _check(dim % delta_dim == 0, "dims should be dividable by delta_dim")
    _check(dstate <= MAX_DSTATE, "selective_scan only supports state dimension <= 256")
    _check(tuple(delta.shape) == (batch, delta_dim, seqlen), "delta must have shape (batch_size, delta_dim, seqlen)")
    _check(tuple(A.shape) == (dim, dstate), "A must have shape (dim, dstate)")
    _check(tuple(B.shape) == (batch, n_groups, dstate, seqlen), "B must have shape (batch_size, n_groups, dstate, seqlen)")
    _check(tuple(C.shape) == (batch, n_groups, dstate, seqlen), "C must have shape (batch_size, n_groups, dstate, seqlen)")
    _check(tuple(dout.shape) == (batch, dim, seqlen), "dout must have shape (batch_size, dim, seqlen)")
    if D is not None:
        _check(D.dtype == torch.float32 and D.is_cuda and tuple(D.shape) == (dim,), "D must be a float32 GPU tensor of shape (dim)")
        D = D.contiguous()
    if delta_bias is not None:
        _check(delta_bias.dtype == torch.float32 and delta_bias.is_cuda and tuple(delta_bias.shape) == (delta_dim,),
               "delta_bias must be a float32 GPU tensor of shape (delta_dim)")
        delta_bias = delta_bias.contiguous()

    dev = u.device
    du = torch.empty((batch, dim, seqlen), device=dev, dtype=u.dtype)
    ddelta = torch.empty((batch, dim, seqlen), device=dev, dtype=u.dtype)
    dA = torch.zeros((dim, dstate), device=dev, dtype=torch.float32)
    dB = torch.zeros((batch, n_groups, dstate, seqlen), device=dev, dtype=torch.float32)
    dC = torch.zeros((batch, n_groups, dstate, seqlen), device=dev, dtype=torch.float32)
    dD = torch.zeros((dim,), device=dev, dtype=torch.float32) if D is not None else None
    dbias = torch.zeros((dim,), device=dev, dtype=torch.float32) if delta_bias is not None else None

    p = _lib.ScanBwdParams()
    p.batch, p.dim, p.seqlen, p.dstate, p.n_groups, p.delta_dim = batch, dim, seqlen, dstate, n_groups, delta_dim
    p.in_dtype, p.dout_dtype = _DTYPE_CODE[u.dtype], _DTYPE_CODE[dout.dtype]
    p.delta_softplus = int(bool(delta_softplus))
    p.u, p.delta, p.A, p.B, p.C, p.dout = (u.data_ptr(), delta.data_ptr(), A.data_ptr(), B.data_ptr(), C.data_ptr(),
                                           dout.data_ptr())
    p.D = D.data_ptr() if D is not None else None
    p.delta_bias = delta_bias.data_ptr() if delta_bias is not None else None
    p.du, p.ddelta, p.dA, p.dB, p.dC = du.data_ptr(), ddelta.data_ptr(), dA.data_ptr(), dB.data_ptr(), dC.data_ptr()
    p.dD = dD.data_ptr() if dD is not None else None
    p.ddelta_bias = dbias.data_ptr() if dbias is not None else None
    p.u_batch_stride, p.u_d_stride = u.stride(0), u.stride(1)
    p.delta_batch_stride, p.delta_d_stride = delta.stride(0), delta.stride(1)
    p.A_d_stride, p.A_dstate_stride = A.stride(0), A.stride(1)
    p.B_batch_stride, p.B_group_stride, p.B_dstate_stride = B.stride(0), B.stride(1), B.stride(2)
    p.C_batch_stride, p.C_group_stride, p.C_dstate_stride = C.stride(0), C.stride(1), C.stride(2)
    p.dout_batch_stride, p.dout_d_stride = dout.stride(0), dout.stride(1)
    if u.numel():
        with torch.cuda.device(dev):
            rc = _lib.lib().ss2d_selective_scan_bwd(p, torch.cuda.current_stream(dev).cuda_stream)
        _lib.check(rc, "ss2d_selective_scan_bwd")
    if delta_dim != dim:        # channels sharing a delta row (selective_scan_oflex.cpp:347-352)
        ddelta = ddelta.view(batch, delta_dim, dim // delta_dim, seqlen).sum(2)
        if dbias is not None:
            dbias = dbias.view(delta_dim, dim // delta_dim).sum(1)
    return [du, ddelta, dA, dB.to(B.dtype), dC.to(C.dtype), dD, dbias]


class SelectiveScanHip(torch.autograd.Function):
    """Counterpart of SelectiveScanCuda (csms6s.py:71-109)."""

    @staticmethod
    def forward(ctx, u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False, oflex=True, backend=None):
        ctx.delta_softplus = delta_softplus
        out, _ = selective_scan_fwd(u, delta, A, B, C, D, delta_bias, delta_softplus, 1, oflex, want_x=False)
        ctx.save_for_backward(u, delta, A, B, C, D, delta_bias)
        return out

    @staticmethod
    def backward(ctx, dout, *args):
        u, delta, A, B, C, D, delta_bias = ctx.saved_tensors
        if dout.stride(-1) != 1:
            dout = dout.contiguous()
        du, ddelta, dA, dB, dC, dD, ddelta_bias = selective_scan_bwd(u, delta, A, B, C, D, delta_bias, dout, None,
                                                                     ctx.delta_softplus, 1)
        return du, ddelta, dA, dB, dC, dD, ddelta_bias, None, None, None


def selective_scan_fn(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=True, oflex=True, backend=None):
    # u, delta: (B, K*C, L); A: (K*C, N); B, C: (B, K, N, L); D, delta_bias: (K*C)
    if backend not in (None, "oflex"):
        raise NotImplementedError(f"selective_scan_fn: backend={backend!r} is not available; this package ships the HIP 'oflex' forward only")
    return SelectiveScanHip.apply(u, delta, A, B, C, D, delta_bias, delta_softplus, oflex, backend)
