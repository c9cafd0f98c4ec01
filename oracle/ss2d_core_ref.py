"""TEST INFRASTRUCTURE ONLY -- the SS2D block and model composed from torch-on-CPU reference operators.

``RefSS2D`` is the package's SS2D block with ``forward_core`` replaced by the torch restatement
(oracle/torch_ref.py) in the order of classification/models/vmamba.py:603-646, and ``TorchLayers`` supplies
the reference's own norm layers (nn.LayerNorm; LayerNorm2d = permute, F.layer_norm, permute, vmamba.py:52-57)
instead of the package's HIP ones.  It is what model-level parity tests compare against and what the benchmark
times as the "reference torch CPU path".
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from vmamba_amd.ss2d import SS2D
from . import torch_ref


class TorchLayerNorm2d(nn.LayerNorm):
    def forward(self, x):
        y = F.layer_norm(x.permute(0, 2, 3, 1), self.normalized_shape, self.weight.to(x.dtype), self.bias.to(x.dtype), self.eps)
        return y.permute(0, 3, 1, 2)


class TorchLayers:
    LayerNorm = nn.LayerNorm
    LayerNorm2d = TorchLayerNorm2d

    @staticmethod
    def out_norm(norm, y, channel_first, dtype):
        # vmamba.py:641-646: (transpose to channel-last if the block is channel-last,) out_norm, cast
        B, D, H, W = y.shape
        if channel_first:
            return norm(y).to(dtype)
        y = y.view(B, D, H * W).transpose(1, 2).contiguous().view(B, H, W, D)
        return F.layer_norm(y, (D,), norm.weight.to(y.dtype), norm.bias.to(y.dtype), norm.eps).to(dtype)


    @staticmethod
    def conv_act(conv2d, x, channel_first):
        # vmamba.py:654-658
        if not channel_first:
            x = x.permute(0, 3, 1, 2).contiguous()
        return F.silu(conv2d(x) if conv2d is not None else x)


class RefSS2D(SS2D):
    def __init__(self, *args, **kwargs):
        kwargs.setdefault("layers", TorchLayers)
        super().__init__(*args, **kwargs)

    def forward_core(self, x):
        B, D, H, W = x.shape
        K, L = self.k_group, H * W
        xs = torch_ref.cross_scan(x)
        dts, Bs, Cs = self.project(xs.contiguous())
        ys = torch_ref.selective_scan(xs.reshape(B, K * D, L), dts, -self.A_logs.float().exp(), Bs.contiguous(),
                                      Cs.contiguous(), self.Ds.float(), self.dt_projs_bias.view(-1).float(), True)
        y = torch_ref.cross_merge(ys.view(B, K, D, H, W))
        return self.finish_core(y, B, D, H, W, x.dtype)


def reference_vmamba_tiny(channel_first=True):
    """The harness model with every custom operator replaced by its torch reference."""
    from vmamba_amd.vssm import vmamba_tiny_s1l8
    return vmamba_tiny_s1l8(channel_first=channel_first, ss2d_cls=RefSS2D, layers=TorchLayers)
