"""Narrow channel-last projection on the HIP kernel ss2d_linear_cl: out = [LayerNorm](x) W^T + bias + residual.

Stands in, in a channel-last VSS block of width 96, for norm + in_proj and for out_proj + the residual add
(classification/models/vmamba.py:1225-1228, :648-650, :662) at inference in bf16 / fp16; other widths, fp32 and
training stay on the PyTorch-ROCm operators.
"""
import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}
FUSED_SHAPES = ((96, 96),)            # (in_features, out_features)


def linear_fusable(x, weight):
    """True when ss2d_linear_cl takes this call."""
    return (x.is_cuda and x.dtype in _DTYPE_CODE and weight.dtype == x.dtype and weight.dim() == 2
            and (x.shape[-1], weight.shape[0]) in FUSED_SHAPES and weight.shape[1] == x.shape[-1])


def linear_cl_hip(x, weight, bias=None, residual=None, ln_weight=None, ln_bias=None, eps=1e-5):
    """x (..., K) channel-last, weight (N, K); returns [layer_norm(x)] @ weight.T + bias + residual, shape (..., N)."""
    if not x.is_cuda:
        raise NotImplementedError("linear_cl_hip: vmamba_amd runs on the GPU only")
    if x.dtype not in _DTYPE_CODE:
        raise TypeError(f"linear_cl_hip: unsupported dtype {x.dtype}")
    K = x.shape[-1]
    if weight.dim() != 2 or weight.shape[1] != K:
        raise ValueError(f"linear_cl_hip: weight must be (N, {K}), got {tuple(weight.shape)}")
    N = weight.shape[0]
    x = x.contiguous()
    out = torch.empty(x.shape[:-1] + (N,), device=x.device, dtype=x.dtype)
    if residual is not None and (residual.shape != out.shape or residual.dtype != x.dtype):
        raise ValueError("linear_cl_hip: residual must have the shape and dtype of the result")
    small = [None if t is None else t.to(x.dtype).contiguous() for t in (ln_weight, ln_bias, bias)]
    keep = [weight.contiguous(), None if residual is None else residual.contiguous()]
    ptr = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_linear_cl(x.data_ptr(), ptr(small[0]), ptr(small[1]), float(eps), keep[0].data_ptr(), ptr(small[2]),
                                       ptr(keep[1]), out.data_ptr(), x.numel() // K, K, N, _DTYPE_CODE[x.dtype],
                                       torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_linear_cl")
    return out


def linear_cf_ln_fusable(K, weight, L):
    """True when ss2d_linear_cf_ln takes an fp32 channel-first map (B, K, L) with this 16-bit GPU weight (N, K)."""
    return (weight.is_cuda and weight.dtype in _DTYPE_CODE and weight.dim() == 2 and weight.shape[1] == K
            and (K, weight.shape[0]) in FUSED_SHAPES and L % 32 == 0)


def linear_cf_ln_hip(y, ln_weight, ln_bias, eps, weight, bias=None, residual=None):
    """y (B, K, L) fp32 channel-first (the merged output of the SS2D core), weight (N, K) bf16 / fp16: returns
    layer_norm(y over K, computed in fp32, rounded to the weight's dtype) @ weight.T + bias + residual as the
    channel-last tensor (B, L, N) -- out_norm and out_proj of the block (vmamba.py:641-646, :662) in one kernel."""
    if not y.is_cuda:
        raise NotImplementedError("linear_cf_ln_hip: vmamba_amd runs on the GPU only")
    if y.dtype != torch.float32 or y.dim() != 3 or weight.dtype not in _DTYPE_CODE:
        raise TypeError("linear_cf_ln_hip: y must be (B, K, L) float32 and the weight bf16 or fp16")
    B, K, L = y.shape
    if weight.dim() != 2 or weight.shape[1] != K:
        raise ValueError(f"linear_cf_ln_hip: weight must be (N, {K}), got {tuple(weight.shape)}")
    N, dt = weight.shape[0], weight.dtype
    y = y.contiguous()
    out = torch.empty((B, L, N), device=y.device, dtype=dt)
    if residual is not None and (residual.numel() != out.numel() or residual.dtype != dt):
        raise ValueError("linear_cf_ln_hip: residual must have the size and dtype of the result")
    small = [None if t is None else t.to(dt).contiguous() for t in (ln_weight, ln_bias, bias)]
    if small[0] is None:
        raise ValueError("linear_cf_ln_hip: the LayerNorm weight is required")
    keep = [weight.contiguous(), None if residual is None else residual.contiguous()]
    ptr = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(y.device):
        rc = _lib.lib().ss2d_linear_cf_ln(y.data_ptr(), ptr(small[0]), ptr(small[1]), float(eps), keep[0].data_ptr(), ptr(small[2]),
                                          ptr(keep[1]), out.data_ptr(), B, L, K, N, _DTYPE_CODE[dt],
                                          torch.cuda.current_stream(y.device).cuda_stream)
    _lib.check(rc, "ss2d_linear_cf_ln")
    return out
