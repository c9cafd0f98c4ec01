"""Channel LayerNorm on the HIP kernels of libss2d_hip.so (ss2d_layer_norm / ss2d_layer_norm_cf).

``LayerNorm`` is nn.LayerNorm for (..., C) activations, ``LayerNorm2d`` the reference's channel-first
variant (classification/models/vmamba.py:52-57).  Same parameters (``weight``, ``bias``, ``eps``) as the
torch modules, so state_dicts are interchangeable.  GPU tensors only: there is no CPU path here.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.SS2D_F32, torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}


def _params(weight, bias):
    if weight is not None and bias is not None and weight.dtype != bias.dtype:
        bias = bias.to(weight.dtype)
    wdt = weight.dtype if weight is not None else (bias.dtype if bias is not None else torch.float32)
    return (weight.contiguous() if weight is not None else None, bias.contiguous() if bias is not None else None, wdt)


def layer_norm_hip(x, weight, bias, eps=1e-5, out_dtype=None):
    """LayerNorm over the last axis of a contiguous GPU tensor."""
    if not x.is_cuda:
        raise NotImplementedError("layer_norm_hip: vmamba_amd runs on the GPU only")
    x = x.contiguous()
    C = x.shape[-1]
    weight, bias, wdt = _params(weight, bias)
    y = torch.empty(x.shape, device=x.device, dtype=out_dtype or x.dtype)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_layer_norm(x.data_ptr(), weight.data_ptr() if weight is not None else None,
                                        bias.data_ptr() if bias is not None else None, y.data_ptr(),
                                        x.numel() // max(C, 1), C, eps, _DTYPE_CODE[x.dtype], _DTYPE_CODE[wdt],
                                        _DTYPE_CODE[y.dtype], torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_layer_norm")
    return y


def add_layer_norm_fusable(x, residual):
    """True when ss2d_add_layer_norm takes these rows (vectorisable: C % 8 == 0, C <= 1024)."""
    C = x.shape[-1]
    return (x.is_cuda and x.dtype in _DTYPE_CODE and residual.dtype == x.dtype and residual.shape == x.shape
            and C % 8 == 0 and C <= 1024)


def add_layer_norm_hip(x, residual, weight, bias, eps=1e-5):
    """(x + residual, LayerNorm(x + residual)) over the last axis in one pass; the sum is rounded to x.dtype first, as
    the separate add would leave it."""
    if not x.is_cuda:
        raise NotImplementedError("add_layer_norm_hip: vmamba_amd runs on the GPU only")
    if residual.shape != x.shape or residual.dtype != x.dtype:
        raise ValueError("add_layer_norm_hip: residual must have the shape and dtype of x")
    x, residual = x.contiguous(), residual.contiguous()
    C = x.shape[-1]
    weight, bias, wdt = _params(weight, bias)
    total, y = torch.empty_like(x), torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_add_layer_norm(x.data_ptr(), residual.data_ptr(), weight.data_ptr() if weight is not None else None,
                                            bias.data_ptr() if bias is not None else None, total.data_ptr(), y.data_ptr(),
                                            x.numel() // max(C, 1), C, eps, _DTYPE_CODE[x.dtype], _DTYPE_CODE[wdt],
                                            _DTYPE_CODE[y.dtype], torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_add_layer_norm")
    return total, y


def bias_layer_norm_fusable(dtype, C):
    """True when ss2d_bias_layer_norm takes rows of C channels of this dtype (vectorisable: C % 8 == 0, C <= 1024)."""
    return dtype in _DTYPE_CODE and C % 8 == 0 and C <= 1024


def bias_layer_norm_hip(x, pre_bias, weight, bias, eps=1e-5):
    """LayerNorm(x + pre_bias) over the last axis in one pass, pre_bias one value per channel; the sum is rounded to
    x.dtype first, as the separate add would leave it."""
    if not x.is_cuda:
        raise NotImplementedError("bias_layer_norm_hip: vmamba_amd runs on the GPU only")
    C = x.shape[-1]
    if pre_bias.shape != (C,):
        raise ValueError("bias_layer_norm_hip: pre_bias must hold one value per channel")
    x = x.contiguous()
    weight, bias, wdt = _params(weight, bias)
    pre_bias = pre_bias.to(wdt).contiguous()
    y = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_bias_layer_norm(x.data_ptr(), pre_bias.data_ptr(), weight.data_ptr() if weight is not None else None,
                                             bias.data_ptr() if bias is not None else None, y.data_ptr(),
                                             x.numel() // max(C, 1), C, eps, _DTYPE_CODE[x.dtype], _DTYPE_CODE[wdt],
                                             _DTYPE_CODE[y.dtype], torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_bias_layer_norm")
    return y


def layer_norm_cf_hip(x, weight, bias, eps=1e-5, out_channel_last=False, out_dtype=None):
    """LayerNorm over axis 1 of a channel-first (B, C, *spatial) GPU tensor.

    Returns (B, *spatial, C) when ``out_channel_last`` else (B, C, *spatial)."""
    if not x.is_cuda:
        raise NotImplementedError("layer_norm_cf_hip: vmamba_amd runs on the GPU only")
    x = x.contiguous()
    B, C = x.shape[0], x.shape[1]
    spatial = tuple(x.shape[2:])
    L = 1
    for s in spatial:
        L *= s
    weight, bias, wdt = _params(weight, bias)
    shape = (B, *spatial, C) if out_channel_last else (B, C, *spatial)
    y = torch.empty(shape, device=x.device, dtype=out_dtype or x.dtype)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_layer_norm_cf(x.data_ptr(), weight.data_ptr() if weight is not None else None,
                                           bias.data_ptr() if bias is not None else None, y.data_ptr(), B, C, L, eps,
                                           _DTYPE_CODE[x.dtype], _DTYPE_CODE[wdt], _DTYPE_CODE[y.dtype],
                                           int(bool(out_channel_last)), torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_layer_norm_cf")
    return y


def needs_grad(*tensors):
    """True when autograd has to see this call: the HIP LayerNorm / conv kernels are inference kernels, so modules
    route such calls to the differentiable torch operators the reference itself uses."""
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def _gpu_only(x, what):
    if not x.is_cuda:
        raise NotImplementedError(f"{what}: vmamba_amd runs on the GPU only (got a {x.device.type} tensor)")


class LayerNorm(nn.LayerNorm):
    def forward(self, x):
        _gpu_only(x, "LayerNorm")
        if needs_grad(x, self.weight, self.bias):
            return F.layer_norm(x, self.normalized_shape, self.weight, self.bias, self.eps)
        return layer_norm_hip(x, self.weight, self.bias, self.eps)


class LayerNorm2d(nn.LayerNorm):
    def forward(self, x):
        _gpu_only(x, "LayerNorm2d")
        if needs_grad(x, self.weight, self.bias):          # vmamba.py:52-57
            return F.layer_norm(x.permute(0, 2, 3, 1), self.normalized_shape, self.weight, self.bias, self.eps).permute(0, 3, 1, 2)
        return layer_norm_cf_hip(x, self.weight, self.bias, self.eps, out_channel_last=False)
