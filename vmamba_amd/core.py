"""Fused SS2D core operator: CrossScan -> selective scan -> CrossMerge in one HIP kernel (d_state = 1).

Stands in for the three operator calls of SS2Dv2.forward_corev2 (classification/models/vmamba.py:604,
625-633, 638) when the model has one state per channel; the projections between them remain the caller's.
"""
import math

import torch

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.SS2D_F32, torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _lds_extent(n, es):
    """Elements an LDS array of n logical elements takes: one spare 4-byte word per 32 words, rounded to 8 elements."""
    idx = n + (n >> 5) if es == 4 else n + ((n >> 6) << 1)
    return (idx + 8) & ~7


def core_fits(H, W, dtype):
    """True when the fused core takes an H x W image of this dtype: at least 8 positions, and either the LDS arrays
    of one image (two fp32 merge planes, two copies of the x map plus a block of 8 zeros each) within the 160 KiB of a CU --
    the single kernel, maps of up to ~13 000 positions -- or 16-bit maps whose sides are multiples of 8, which the tiled two-pass kernels take at any size."""
    if dtype not in _DTYPE_CODE:
        return False
    L = H * W
    es = 4 if dtype == torch.float32 else 2
    if _fits_single_kernel(L, es):
        return True
    return es == 2 and ((H % 8 == 0 and W % 8 == 0) or padded_map_size(H, W, dtype) is not None)


def _fits_single_kernel(L, es):
    maps = _lds_extent(((L + 7) & ~7) + 8, es)
    return L >= 8 and 2 * _lds_extent(L, 4) * 4 + 2 * maps * es <= 160 * 1024 - 256


def padded_map_size(H, W, dtype):
    """(H', W') >= (H, W) in which a caller should embed an H x W map for the fused core, or None when the map is fine
    as it is (or padding would not pay).  16-bit maps only.  The core's vector paths want a number of positions that is
    a multiple of 8 and, for the 4 x 4 tiles of its staging and merge, sides that are multiples of 4 (so: multiples of
    4, whose product is a multiple of 16); maps beyond the single kernel's LDS arrays go to the tiled kernels, which want
    multiples of 8.  Without them the core walks the map element by element at a third to a quarter of the rate, which a
    padded area of up to 1.5 times the map's beats."""
    if dtype not in (torch.bfloat16, torch.float16):
        return None
    L = H * W
    if H == W == 7:                      # has a kernel of its own (one map row per lane)
        return None
    if _fits_single_kernel(L, 2):
        if math.gcd(L, 8) >= 4:
            return None
        H4, W4 = (H + 3) & ~3, (W + 3) & ~3
        if _fits_single_kernel(H4 * W4, 2):
            return (H4, W4) if H4 * W4 <= 1.5 * L else None
    if H % 8 == 0 and W % 8 == 0:
        return None
    H8, W8 = (H + 7) & ~7, (W + 7) & ~7
    return (H8, W8) if H8 * W8 <= 1.5 * L else None


def core_mask_pads_hip(delta, H, W, Hp, Wp):
    """delta (4, D, B, Hp*Wp) view of the padded map's steps: -inf at the scan positions that fall on the rows >= H and the
    columns >= W, in every direction's order (ss2d_core_mask_pads).  In place."""
    _check(delta.is_cuda and delta.dim() == 4 and delta.shape[0] == 4 and delta.shape[3] == Hp * Wp, "delta must be (4, D, B, Hp*Wp) on the GPU")
    _check(delta.dtype in _DTYPE_CODE and (delta.stride(3) == 1 or delta.shape[3] == 1), "delta must be contiguous along the map")
    with torch.cuda.device(delta.device):
        rc = _lib.lib().ss2d_core_mask_pads(delta.data_ptr(), delta.shape[2], delta.shape[1], H, W, Hp, Wp, delta.stride(0),
                                            delta.stride(1), delta.stride(2), _DTYPE_CODE[delta.dtype],
                                            torch.cuda.current_stream(delta.device).cuda_stream)
    _lib.check(rc, "ss2d_core_mask_pads")
    return delta


def embed_maps_hip(src, dst_rows, dst_cols):
    """src (n_maps, rows, cols), contiguous, 2- or 4-byte elements -> (n_maps, dst_rows, dst_cols): the maps zero-padded at
    the bottom / right or cropped there, in one pass (ss2d_core_embed_maps)."""
    _check(src.is_cuda and src.dim() == 3 and src.is_contiguous(), "embed_maps: a contiguous (n_maps, rows, cols) GPU tensor")
    _check(src.element_size() in (2, 4), "embed_maps: 2- or 4-byte elements")
    n, rows, cols = src.shape
    dst = src.new_empty((n, dst_rows, dst_cols))
    if dst.numel() == 0:
        return dst
    if src.numel() == 0:
        return dst.zero_()
    with torch.cuda.device(src.device):
        rc = _lib.lib().ss2d_core_embed_maps(src.data_ptr(), dst.data_ptr(), n, rows, cols, dst_rows, dst_cols, src.element_size(),
                                             torch.cuda.current_stream(src.device).cuda_stream)
    _lib.check(rc, "ss2d_core_embed_maps")
    return dst


def ss2d_core_hip(x, delta, Bs, Cs, As, Ds=None, delta_bias=None, delta_softplus=True, out=None):
    """x (B,D,H,W); delta (4,D,B,L) view; Bs, Cs (4,B,L) views (last stride 1), all of x.dtype and already in the
    scan order of their direction; As, Ds, delta_bias (4*D) fp32.  Returns the merged y (B,D,L) fp32 (written into
    ``out`` when given: a contiguous fp32 tensor of that shape).

    Raises Ss2dError with status SS2D_ENOTSUP when the shape has no fused kernel (an image too large for the LDS
    planes that the tiled kernels do not take either: fp32, sides not multiples of 8, unaligned rows): callers fall
    back to the three separate operators.
    """
    _check(x.is_cuda, "ss2d_core: vmamba_amd runs on the GPU only")
    _check(x.dim() == 4, "x must be (B, D, H, W)")
    _check(x.dtype in _DTYPE_CODE, f"ss2d_core not implemented for input type '{x.dtype}'")
    B, D, H, W = x.shape
    L = H * W
    for name, t in (("delta", delta), ("B", Bs), ("C", Cs)):
        _check(t.is_cuda and t.dtype == x.dtype, f"{name} must be a GPU tensor of x's dtype")
        _check(t.stride(-1) == 1 or t.size(-1) == 1, f"{name} must be contiguous in its last dimension")
    _check(tuple(delta.shape) == (4, D, B, L), "delta must have shape (4, dim, batch, L)")
    _check(tuple(Bs.shape) == (4, B, L) and tuple(Cs.shape) == (4, B, L), "B and C must have shape (4, batch, L)")
    _check(As.dtype == torch.float32 and As.is_cuda and As.numel() == 4 * D, "A must be (4*dim) float32 (one state)")
    As = As.contiguous()
    if Ds is not None:
        _check(Ds.dtype == torch.float32 and Ds.is_cuda and tuple(Ds.shape) == (4 * D,), "D must be (4*dim) float32")
        Ds = Ds.contiguous()
    if delta_bias is not None:
        _check(delta_bias.dtype == torch.float32 and delta_bias.is_cuda and tuple(delta_bias.shape) == (4 * D,),
               "delta_bias must be (4*dim) float32")
        delta_bias = delta_bias.contiguous()
    x = x.contiguous()
    if out is None:
        y = torch.empty((B, D, L), device=x.device, dtype=torch.float32)
    else:
        _check(out.is_cuda and out.dtype == torch.float32 and tuple(out.shape) == (B, D, L) and out.is_contiguous(),
               "out must be a contiguous float32 GPU tensor of shape (batch, dim, L)")
        y = out
    p = _lib.CoreParams()
    p.batch, p.dim, p.height, p.width = B, D, H, W
    p.in_dtype = _DTYPE_CODE[x.dtype]
    p.delta_softplus = 1 if delta_softplus else 0
    p.x, p.delta, p.A, p.B, p.C = x.data_ptr(), delta.data_ptr(), As.data_ptr(), Bs.data_ptr(), Cs.data_ptr()
    p.D = Ds.data_ptr() if Ds is not None else None
    p.delta_bias = delta_bias.data_ptr() if delta_bias is not None else None
    p.y = y.data_ptr()
    p.delta_dir_stride, p.delta_dim_stride, p.delta_batch_stride = delta.stride(0), delta.stride(1), delta.stride(2)
    p.B_dir_stride, p.B_batch_stride = Bs.stride(0), Bs.stride(1)
    p.C_dir_stride, p.C_batch_stride = Cs.stride(0), Cs.stride(1)
    with torch.cuda.device(x.device):
        # maps too large for the single kernel are walked in tiles, twice, through scratch memory of the size the library asks for
        need = _lib.lib().ss2d_core_workspace_bytes(p)
        _lib.check(min(need, 0), "ss2d_core_workspace_bytes")
        stream = torch.cuda.current_stream(x.device).cuda_stream
        if need > 0:
            workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
            rc = _lib.lib().ss2d_core_fwd_ws(p, workspace.data_ptr(), need, stream)
        else:
            rc = _lib.lib().ss2d_core_fwd(p, stream)
    _lib.check(rc, "ss2d_core_fwd")
    return y


DT_PROJ_MAX_RANK = 48


def dt_proj_hip(x, weight, mask=None, fill=0.0):
    """delta[k] = weight[k] @ x[k]: x (K, R, N) with contiguous rows (any direction / rank strides), weight (K, D, R),
    both bf16 or fp16 -> (K, D, N) of the same dtype, on the matrix cores (ss2d_dt_proj).  With ``mask`` -- (K, N) int16,
    0 or -1 -- every channel's delta at the positions marked -1 is ``fill`` instead (ss2d_dt_proj_masked)."""
    _check(x.is_cuda and weight.is_cuda, "dt_proj: vmamba_amd runs on the GPU only")
    _check(x.dim() == 3 and weight.dim() == 3 and x.shape[0] == weight.shape[0] and x.shape[1] == weight.shape[2],
           "dt_proj expects x (K, R, N) and weight (K, D, R)")
    _check(x.dtype == weight.dtype and x.dtype in (torch.bfloat16, torch.float16), "dt_proj: bf16 or fp16 tensors")
    _check(x.stride(2) == 1 or x.size(2) == 1, "x must be contiguous in its last dimension")
    K, R, N = x.shape
    D = weight.shape[1]
    if mask is not None:
        _check(mask.is_cuda and mask.device == x.device and mask.dtype == torch.int16 and tuple(mask.shape) == (K, N)
               and mask.is_contiguous(), "dt_proj: mask must be a contiguous (K, N) int16 tensor on x's device")
    weight = weight.contiguous()
    out = torch.empty((K, D, N), device=x.device, dtype=x.dtype)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_dt_proj_masked(x.data_ptr(), weight.data_ptr(), None if mask is None else mask.data_ptr(), float(fill),
                                            out.data_ptr(), K, D, R, N, x.stride(0), x.stride(1), _DTYPE_CODE[x.dtype],
                                            torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_dt_proj")
    return out
