"""TEST INFRASTRUCTURE ONLY -- the SS2D block and model composed from torch-on-CPU reference operators.

``RefSS2D`` takes only the parameter set (names, shapes, initialisation) from the package's SS2D block; its
``forward`` / ``forward_core`` are restated here from classification/models/vmamba.py:603-663 on the torch
restatement of the three operators (oracle/torch_ref.py) with the projections as the reference's einsums, and ``TorchLayers`` supplies
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
    """Holds the parameters of the package's block (so state dicts are interchangeable) but computes nothing with the
    package's forward code: ``forward_core`` and ``forward`` below are written from the reference's text."""

    def __init__(self, *args, **kwargs):
        kwargs.setdefault("layers", TorchLayers)
        super().__init__(*args, **kwargs)

    def forward_core(self, x):
        # vmamba.py:603-646, the cross2d / non-cascade branch in its einsum spelling (:610-615)
        B, D, H, W = x.shape
        K, L, R, N = self.k_group, H * W, self.dt_rank, self.d_state
        xs = torch_ref.cross_scan(x)                                                         # (B, K, D, L)
        x_dbl = torch.einsum("b k d l, k c d -> b k c l", xs, self.x_proj_weight)
        dts, Bs, Cs = torch.split(x_dbl, [R, N, N], dim=2)
        dts = torch.einsum("b k r l, k d r -> b k d l", dts, self.dt_projs_weight)
        ys = torch_ref.selective_scan(xs.reshape(B, K * D, L), dts.contiguous().view(B, K * D, L),
                                      -self.A_logs.float().exp(), Bs.contiguous(), Cs.contiguous(), self.Ds.float(),
                                      self.dt_projs_bias.view(-1).float(), True)
        y = torch_ref.cross_merge(ys.view(B, K, D, H, W))                                    # (B, D, L)
        return TorchLayers.out_norm(self.out_norm, y.view(B, D, H, W), self.channel_first, x.dtype)

    def forward(self, x, residual=None, pre_norm=None, post_norm=None):
        # vmamba.py:648-663 (forwardv2), with the block's norms and residual of VSSBlock._forward (:1225-1229)
        h = x if pre_norm is None else pre_norm(x)
        h = self.in_proj(h)
        z = None
        if not self.disable_z:
            h, z = h.chunk(2, dim=(1 if self.channel_first else -1))
            z = self.act(z)
        h = TorchLayers.conv_act(self.conv2d if self.with_dconv else None, h, self.channel_first)
        y = self.forward_core(h)
        if z is not None:
            y = y * z
        out = self.out_proj(y)
        if residual is not None:
            out = residual + out
        return out if post_norm is None else (out, post_norm(out))


def reference_vmamba_tiny(channel_first=True):
    """The harness model with every custom operator replaced by its torch reference."""
    from vmamba_amd.vssm import vmamba_tiny_s1l8
    return vmamba_tiny_s1l8(channel_first=channel_first, ss2d_cls=RefSS2D, layers=TorchLayers)
