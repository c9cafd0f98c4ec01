"""Depthwise 3x3 convolution + SiLU in front of the SS2D core, on the HIP kernel ss2d_dwconv3x3_silu.

Mirrors the three lines of SS2Dv2.forwardv2 (classification/models/vmamba.py:654-658): bring the in_proj
output to channel-first, depthwise conv2d, SiLU -- as one kernel that reads either layout and always writes
(B, D, H, W).  GPU tensors only.
"""
import torch

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.SS2D_F32, torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}


def dwconv3x3_silu_hip(x, weight, bias=None, in_channel_last=False, apply_silu=True):
    """x (B,H,W,D) if in_channel_last else (B,D,H,W); weight (D,1,3,3); returns (B,D,H,W)."""
    if not x.is_cuda:
        raise NotImplementedError("dwconv3x3_silu_hip: vmamba_amd runs on the GPU only")
    if x.dim() != 4 or weight.dim() != 4 or tuple(weight.shape[1:]) != (1, 3, 3):
        raise ValueError(f"dwconv3x3_silu_hip: expected a 4-D input and a (D,1,3,3) weight, got {tuple(x.shape)}, {tuple(weight.shape)}")
    if x.dtype not in _DTYPE_CODE:
        raise TypeError(f"dwconv3x3_silu_hip: unsupported dtype {x.dtype}")
    x = x.contiguous()
    if in_channel_last:
        B, H, W, D = x.shape
    else:
        B, D, H, W = x.shape
    if weight.shape[0] != D:
        raise ValueError("dwconv3x3_silu_hip: weight channels do not match the input")
    weight = weight.to(x.dtype).contiguous()
    bias = bias.to(x.dtype).contiguous() if bias is not None else None
    y = torch.empty((B, D, H, W), device=x.device, dtype=x.dtype)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_dwconv3x3_silu(x.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None,
                                            y.data_ptr(), B, D, H, W, _DTYPE_CODE[x.dtype], int(bool(in_channel_last)),
                                            int(bool(apply_silu)), torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_dwconv3x3_silu")
    return y
