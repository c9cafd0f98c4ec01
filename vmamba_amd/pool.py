"""Global average pool of the classifier head as one HIP kernel (ss2d_mean_pool_cl): AdaptiveAvgPool2d(1) on a
channel-last activation (classification/models/vmamba.py:1357-1363)."""
import torch
import torch.nn as nn

from . import _lib
from .norm import needs_grad

_DTYPE_CODE = {torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}


def mean_pool_fusable(x):
    """True for a 16-bit GPU tensor (B, C, H, W) whose memory is channel-last (B, H, W, C), C a multiple of 8."""
    return (x.is_cuda and x.dim() == 4 and x.dtype in _DTYPE_CODE and x.shape[1] % 8 == 0 and x.numel() > 0
            and x.permute(0, 2, 3, 1).is_contiguous() and not needs_grad(x))


def mean_pool_cl_hip(x):
    """x (B, L, C) contiguous, bf16 / fp16 -> (B, C): the mean over L (fp32 sum, one rounding)."""
    if not x.is_cuda:
        raise NotImplementedError("mean_pool_cl_hip: vmamba_amd runs on the GPU only")
    if x.dim() != 3 or x.dtype not in _DTYPE_CODE:
        raise TypeError("mean_pool_cl_hip: x must be (B, L, C) bf16 or fp16")
    x = x.contiguous()
    B, L, C = x.shape
    y = torch.empty((B, C), device=x.device, dtype=x.dtype)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ss2d_mean_pool_cl(x.data_ptr(), y.data_ptr(), B, L, C, _DTYPE_CODE[x.dtype],
                                          torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "ss2d_mean_pool_cl")
    return y


class GlobalAvgPool2d(nn.AdaptiveAvgPool2d):
    """AdaptiveAvgPool2d(1); a 16-bit channel-last GPU activation in inference goes through the HIP kernel, whose result
    does not depend on scheduling (the library's reduction may meet through a counter that it clears with a memset,
    which HIP-graph replays running beside other work have been seen to get wrong)."""

    def __init__(self):
        super().__init__(1)

    def forward(self, x):
        if mean_pool_fusable(x):
            B, C, H, W = x.shape
            return mean_pool_cl_hip(x.permute(0, 2, 3, 1).reshape(B, H * W, C)).view(B, C, 1, 1)
        return super().forward(x)
