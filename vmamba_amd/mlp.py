"""Fused channel-last MLP (fc1 -> GELU -> fc2 -> + residual) on the HIP kernel ss2d_mlp_fused.

Stands in for Mlp.forward and the residual add of a VSS block (classification/models/vmamba.py:1116-1131, :1229) when the
layer is narrow enough (C = 96, 192: the stages whose MLP is bound by the hidden tensor's trips to HBM), the tensors are
bf16 / fp16 and autograd is off; wider layers, fp32 and training stay on the PyTorch-ROCm operators.
"""
import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}
FUSED_WIDTHS = (96, 192)


def mlp_fusable(x, fc1, fc2):
    """True when ss2d_mlp_fused takes this call."""
    C = x.shape[-1]
    return (x.is_cuda and x.dtype in _DTYPE_CODE and C in FUSED_WIDTHS and tuple(fc1.weight.shape) == (4 * C, C)
            and tuple(fc2.weight.shape) == (C, 4 * C) and fc1.weight.dtype == x.dtype and fc2.weight.dtype == x.dtype)


def mlp_fused_hip(x, w1, b1, w2, b2, residual=None, ln_weight=None, ln_bias=None, eps=1e-5):
    """x (..., C) channel-last; returns residual + fc2(gelu(fc1(h))) with the shape of x, where h = x or, when ln_weight
    is given, layer_norm(x) over the channels."""
    if not x.is_cuda:
        raise NotImplementedError("mlp_fused_hip: vmamba_amd runs on the GPU only")
    if x.dtype not in _DTYPE_CODE:
        raise TypeError(f"mlp_fused_hip: unsupported dtype {x.dtype}")
    C = x.shape[-1]
    x = x.contiguous()
    w1, w2 = w1.contiguous(), w2.contiguous()
    if tuple(w1.shape) != (4 * C, C) or tuple(w2.shape) != (C, 4 * C):
        raise ValueError(f"mlp_fused_hip: expected fc1 (4C, C) and fc2 (C, 4C) weights, got {tuple(w1.shape)}, {tuple(w2.shape)}")
    if residual is not None:
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise ValueError("mlp_fused_hip: residual must have the shape and dtype of x")
        residual = residual.contiguous()
    out = torch.empty_like(x)
    ptr = lambda t: None if t is None else t.contiguous().data_ptr()
    keep = [None if t is None else t.to(x.dtype).contiguous() for t in (b1, b2, ln_weight, ln_bias)]
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_mlp_fused(x.data_ptr(), ptr(keep[2]), ptr(keep[3]), float(eps), w1.data_ptr(), ptr(keep[0]),
                                       w2.data_ptr(), ptr(keep[1]), ptr(residual),
                                       out.data_ptr(), x.numel() // C, C, _DTYPE_CODE[x.dtype],
                                       torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_mlp_fused")
    return out
