"""First layer of the patch embedding as one HIP kernel (ss2d_stem_conv_ln_gelu): Conv2d(3, C, 3, stride 2, padding 1)
-> LayerNorm(C) -> GELU on channel-last activations (classification/models/vmamba.py:1403-1411)."""
import ctypes

import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}
STEM_WIDTHS = (48, 64)


def stem_fusable(x, conv, norm, act):
    """True when the kernel serves this conv / norm / activation triple on x."""
    return (x.is_cuda and x.dim() == 4 and x.dtype in _DTYPE_CODE and conv.in_channels == 3 and x.shape[1] == 3
            and conv.out_channels in STEM_WIDTHS and tuple(conv.kernel_size) == (3, 3) and tuple(conv.stride) == (2, 2)
            and tuple(conv.padding) == (1, 1) and tuple(conv.dilation) == (1, 1) and conv.groups == 1
            and conv.padding_mode == "zeros" and conv.weight.dtype == x.dtype
            and tuple(norm.normalized_shape) == (conv.out_channels,) and norm.elementwise_affine
            and norm.weight.dtype == x.dtype and getattr(act, "approximate", "none") == "none")


def stem_conv_ln_gelu_hip(x, weight, bias, ln_weight, ln_bias, eps=1e-5):
    """GELU(LayerNorm(conv2d(x, weight, bias, stride 2, padding 1))) for x (B, 3, H, W): returns the channel-last
    activation (B, Ho, Wo, C).  The weight is read through its strides (contiguous or channels-last)."""
    if not x.is_cuda:
        raise NotImplementedError("stem_conv_ln_gelu: vmamba_amd runs on the GPU only")
    if x.dim() != 4 or x.shape[1] != 3 or weight.dim() != 4 or tuple(weight.shape[1:]) != (3, 3, 3):
        raise ValueError("stem_conv_ln_gelu expects x (B, 3, H, W) and weight (C, 3, 3, 3)")
    if x.dtype not in _DTYPE_CODE or weight.dtype != x.dtype:
        raise RuntimeError("stem_conv_ln_gelu: bf16 or fp16 tensors")
    x = x.contiguous()
    B, _, H, W = x.shape
    C = weight.shape[0]
    cast = lambda t: None if t is None else t.to(x.dtype).contiguous()
    bias, ln_weight, ln_bias = cast(bias), cast(ln_weight), cast(ln_bias)
    ptr = lambda t: None if t is None else t.data_ptr()
    y = torch.empty((B, (H - 1) // 2 + 1, (W - 1) // 2 + 1, C), device=x.device, dtype=x.dtype)
    strides = (ctypes.c_int64 * 4)(*weight.stride())
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_stem_conv_ln_gelu(x.data_ptr(), weight.data_ptr(), strides, ptr(bias), ptr(ln_weight), ptr(ln_bias),
                                               eps, y.data_ptr(), B, H, W, C, _DTYPE_CODE[x.dtype],
                                               torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_stem_conv_ln_gelu")
    return y
