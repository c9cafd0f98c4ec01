"""VMamba-T-shaped backbone used as the throughput harness (random init, inference).

Layer order and shapes follow VSSM / VSSBlock of classification/models/vmamba.py:1153-1505 for
the ``vmamba_tiny_s1l8`` recipe (:1717-1728): patch-embed v2, downsample v3, depths 2/2/8/2, dims
96/192/384/768, d_state 1, ssm_ratio 1, forward type v05_noz, MLP ratio 4.  As in the reference the
same weights run in two activation layouts: ``channel_first=True`` ("ln2d": (B,C,H,W), 1x1 convs,
LayerNorm2d) and ``channel_first=False`` ("ln": (B,H,W,C), nn.Linear, nn.LayerNorm).  The norm
layers come from ``layers`` (default: this package's HIP LayerNorm kernels); convolutions, the projection and
MLP GEMMs and activations are stock torch; drop-path is the identity at inference.

Module names -- hence state_dict keys -- are the reference's (``patch_embed.{0,2,5,7}``,
``layers.{i}.blocks.{j}.{norm,op,norm2,mlp}``, ``layers.{i}.downsample.{1,3}``, ``classifier.{norm,head}``), and
``VSSM._load_from_state_dict`` applies the reference's renames for checkpoints written by its older training code
(vmamba.py:1531-1570), so a released VMamba checkpoint of this architecture loads with ``load_state_dict``.
"""
from collections import OrderedDict

import torch
import torch.nn as nn

from .mlp import mlp_fusable, mlp_fused_hip
from .norm import LayerNorm as HipLayerNorm
from .norm import add_layer_norm_fusable, add_layer_norm_hip, bias_layer_norm_fusable, bias_layer_norm_hip, needs_grad
from .ss2d import SS2D, HipLayers, Linear2d
from .pool import GlobalAvgPool2d
from .stem import stem_conv_ln_gelu_hip, stem_fusable


class Permute(nn.Module):
    def __init__(self, *dims):
        super().__init__()
        self.dims = dims

    def forward(self, x):
        return x.permute(*self.dims)


def _to_cl(channel_first):      # (B,C,H,W) -> block layout
    return nn.Identity() if channel_first else Permute(0, 2, 3, 1)


def _to_cf(channel_first):      # block layout -> (B,C,H,W)
    return nn.Identity() if channel_first else Permute(0, 3, 1, 2)


class ConvNormSequence(nn.Sequential):
    """The patch-embedding and downsampling stacks (vmamba.py:1403-1417, 1430-1437).  Where a Conv2d with a bias is
    followed by the permute to channel-last and this package's LayerNorm, the convolution runs without its bias and
    the LayerNorm kernel adds it on the way in (ss2d_bias_layer_norm): one pass over the activation fewer."""

    def forward(self, x):
        mods = list(self)
        i = 0
        while i < len(mods):
            conv = mods[i]
            if i + 4 < len(mods) and self._stem(x, conv, *mods[i + 1:i + 5]):
                norm = mods[i + 2]                    # conv, LayerNorm and GELU in one kernel; the result is channel-last
                x = stem_conv_ln_gelu_hip(x, conv.weight, conv.bias, norm.weight, norm.bias, norm.eps).permute(0, 3, 1, 2)
                i += 5
            elif i + 2 < len(mods) and self._fusable(x, conv, mods[i + 1], mods[i + 2]):
                norm = mods[i + 2]
                x = conv._conv_forward(x, conv.weight, None).permute(0, 2, 3, 1)
                x = bias_layer_norm_hip(x, conv.bias, norm.weight, norm.bias, norm.eps)
                i += 3
            else:
                x = conv(x)
                i += 1
        return x

    @staticmethod
    def _stem(x, conv, to_cl, norm, to_cf, act):
        return (isinstance(conv, nn.Conv2d) and isinstance(to_cl, Permute) and tuple(to_cl.dims) == (0, 2, 3, 1)
                and isinstance(norm, HipLayerNorm) and isinstance(to_cf, Permute) and tuple(to_cf.dims) == (0, 3, 1, 2)
                and isinstance(act, nn.GELU) and stem_fusable(x, conv, norm, act)
                and not needs_grad(x, conv.weight, conv.bias, norm.weight, norm.bias))

    @staticmethod
    def _fusable(x, conv, permute, norm):
        return (isinstance(conv, nn.Conv2d) and conv.bias is not None and isinstance(permute, Permute)
                and tuple(permute.dims) == (0, 2, 3, 1) and isinstance(norm, HipLayerNorm) and norm.elementwise_affine
                and x.is_cuda and x.dim() == 4 and bias_layer_norm_fusable(x.dtype, conv.out_channels)
                and not needs_grad(x, conv.weight, conv.bias, norm.weight, norm.bias))


class Mlp(nn.Module):
    def __init__(self, dim, hidden, channel_first=True, fused=True):
        super().__init__()
        self.channel_first, self.fused = channel_first, fused
        Linear = Linear2d if channel_first else nn.Linear
        self.fc1 = Linear(dim, hidden)
        self.act = nn.GELU()
        self.fc2 = Linear(hidden, dim)

    def takes_norm(self, x):
        """True when forward runs the fused kernel for x (which then takes the preceding LayerNorm as a prologue)."""
        return (self.fused and not self.channel_first and mlp_fusable(x, self.fc1, self.fc2)
                and not needs_grad(x, self.fc1.weight, self.fc2.weight, self.fc1.bias, self.fc2.bias))

    def forward(self, x, residual=None, pre_norm=None):
        """fc2(GELU(fc1(h))) (+ residual), h = x or pre_norm(x) (the block's second LayerNorm, vmamba.py:1229).
        Channel-last 16-bit inference at widths 96 / 192 runs as one HIP kernel that normalises the rows on the way
        in and keeps the hidden activations in registers; everything else on the torch operators."""
        if (self.fused and not self.channel_first and mlp_fusable(x, self.fc1, self.fc2)
                and not needs_grad(x, self.fc1.weight, self.fc2.weight, self.fc1.bias, self.fc2.bias)):
            if pre_norm is None:
                return mlp_fused_hip(x, self.fc1.weight, self.fc1.bias, self.fc2.weight, self.fc2.bias, residual)
            if (isinstance(pre_norm, nn.LayerNorm) and pre_norm.elementwise_affine
                    and not needs_grad(pre_norm.weight, pre_norm.bias)):
                return mlp_fused_hip(x, self.fc1.weight, self.fc1.bias, self.fc2.weight, self.fc2.bias, residual,
                                     pre_norm.weight, pre_norm.bias, pre_norm.eps)
        if pre_norm is not None:
            x = pre_norm(x)
        y = self.fc2(self.act(self.fc1(x)))
        return y if residual is None else residual + y


class VSSBlock(nn.Module):
    def __init__(self, dim, d_state=1, ssm_ratio=1.0, mlp_ratio=4.0, ss2d_cls=SS2D, channel_first=True, layers=HipLayers,
                 **ss2d_kwargs):
        super().__init__()
        Norm = layers.LayerNorm2d if channel_first else layers.LayerNorm
        self.norm = Norm(dim)
        self.op = ss2d_cls(d_model=dim, d_state=d_state, ssm_ratio=ssm_ratio, channel_first=channel_first, layers=layers,
                           **ss2d_kwargs)
        self.norm2 = Norm(dim)
        self.mlp = Mlp(dim, int(dim * mlp_ratio), channel_first)

    def forward(self, x):
        x, pending = self.step(x, None)
        return x if pending is None else x + pending

    def step(self, x, pending):
        """One block on the residual stream x, with ``pending`` (or None) a term the previous block has not added to x
        yet; returns (x, pending) in the same sense.  Deferring the MLP's residual add lets the next block do it
        together with its first LayerNorm in one kernel (ss2d_add_layer_norm); it is only deferred where that kernel
        exists (channel-last 16-bit inference)."""
        inp, pre = x, self.norm
        if pending is not None:
            if self._fusable_add_norm(x, pending, self.norm):
                x, inp = add_layer_norm_hip(pending, x, self.norm.weight, self.norm.bias, self.norm.eps)
                pre = None
            else:
                x = inp = x + pending
        if self.mlp.takes_norm(x):                    # the fused MLP kernel normalises its input itself
            x = self.op(inp, residual=x, pre_norm=pre)
            return self.mlp(x, residual=x, pre_norm=self.norm2), None
        x, h = self.op(inp, residual=x, pre_norm=pre, post_norm=self.norm2)
        m = self.mlp(h)
        if self._fusable_add_norm(x, m, self.norm):
            return x, m
        return x + m, None

    def _fusable_add_norm(self, x, term, norm):
        return (not self.op.channel_first and isinstance(norm, nn.LayerNorm) and norm.elementwise_affine
                and add_layer_norm_fusable(x, term) and x.dtype != torch.float32
                and not needs_grad(x, term, norm.weight, norm.bias))


class BlockSequence(nn.Sequential):
    """The blocks of one stage; threads the deferred residual term from block to block (see VSSBlock.step)."""

    def forward(self, x):
        pending = None
        for block in self:
            x, pending = block.step(x, pending)
        return x if pending is None else x + pending


class VSSM(nn.Module):
    def __init__(self, in_chans=3, num_classes=1000, depths=(2, 2, 8, 2), dims=(96, 192, 384, 768), d_state=1,
                 ssm_ratio=1.0, mlp_ratio=4.0, ss2d_cls=SS2D, channel_first=True, layers=HipLayers, **ss2d_kwargs):
        super().__init__()
        self._build_args = dict(in_chans=in_chans, num_classes=num_classes, depths=tuple(depths), dims=tuple(dims), d_state=d_state,
                                ssm_ratio=ssm_ratio, mlp_ratio=mlp_ratio, ss2d_cls=ss2d_cls, layers=layers, **ss2d_kwargs)
        cf = channel_first
        Norm = layers.LayerNorm2d if cf else layers.LayerNorm
        d0 = dims[0]
        self.patch_embed = ConvNormSequence(
            nn.Conv2d(in_chans, d0 // 2, kernel_size=3, stride=2, padding=1), _to_cl(cf), Norm(d0 // 2), _to_cf(cf),
            nn.GELU(),
            nn.Conv2d(d0 // 2, d0, kernel_size=3, stride=2, padding=1), _to_cl(cf), Norm(d0))
        stages = []
        for i, (depth, dim) in enumerate(zip(depths, dims)):
            blocks = [VSSBlock(dim, d_state, ssm_ratio, mlp_ratio, ss2d_cls, cf, layers, **ss2d_kwargs) for _ in range(depth)]
            down = (ConvNormSequence(_to_cf(cf), nn.Conv2d(dim, dims[i + 1], kernel_size=3, stride=2, padding=1), _to_cl(cf),
                                  Norm(dims[i + 1]))
                    if i + 1 < len(dims) else nn.Identity())
            stages.append(nn.Sequential(OrderedDict(blocks=BlockSequence(*blocks), downsample=down)))
        self.layers = nn.ModuleList(stages)
        self.classifier = nn.Sequential(OrderedDict(
            norm=Norm(dims[-1]), permute=_to_cf(cf), avgpool=GlobalAvgPool2d(), flatten=nn.Flatten(1),
            head=nn.Linear(dims[-1], num_classes)))
        self.apply(self._init_weights)

    # key prefixes of checkpoints from the reference's previous training code -> current names (vmamba.py:1557-1564)
    LEGACY_KEYS = (("patch_embed.proj", "patch_embed.0"), ("patch_embed.norm", "patch_embed.2"),
                   ("norm", "classifier.norm"), ("head", "classifier.head"))
    LEGACY_BLOCK_KEYS = (("ln_1", "norm"), ("self_attention", "op"))

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        def rename(src, dst):
            for key in [k for k in state_dict if k.startswith(prefix + src)]:
                state_dict[prefix + dst + key[len(prefix + src):]] = state_dict.pop(key)

        for i, stage in enumerate(self.layers):
            for j in range(len(stage.blocks)):
                for src, dst in self.LEGACY_BLOCK_KEYS:
                    rename(f"layers.{i}.blocks.{j}.{src}", f"layers.{i}.blocks.{j}.{dst}")
        for src, dst in self.LEGACY_KEYS:
            rename(src, dst)
        return super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    @staticmethod
    def _init_weights(m):
        if isinstance(m, nn.Linear):
            nn.init.trunc_normal_(m.weight, std=0.02)
            if m.bias is not None:
                nn.init.zeros_(m.bias)
        elif isinstance(m, nn.LayerNorm):
            nn.init.ones_(m.weight)
            nn.init.zeros_(m.bias)

    def forward(self, x):
        x = self.patch_embed(x)
        for layer in self.layers:
            x = layer(x)
        return self.classifier(x)

    def with_layout(self, channel_first, share_weights=False):
        """The same model (same device, dtype and mode) with its blocks in the other activation layout.  The reference's
        "ln2d" configurations build channel-first blocks (vmamba.py:1281); the two layouts compute the same function and
        share one state_dict (a Linear2d weight is a view of the nn.Linear one, vmamba.py:47-49), and the channel-last
        build is the one whose projections, MLPs and LayerNorms run on this package's fused kernels.

        The twin holds a copy of the weights, or -- ``share_weights=True`` -- the very same Parameter and buffer objects
        (every parameter has the same shape in both builds), so that loading, casting, moving or training either model
        is seen by the other."""
        twin = VSSM(channel_first=channel_first, **self._build_args)
        if not share_weights:
            twin.load_state_dict(self.state_dict())
            p = next(self.parameters())
            return twin.to(device=p.device, dtype=p.dtype).train(self.training)
        mine = dict(self.named_modules())
        for name, module in twin.named_modules():
            src = mine[name]
            for key in list(module._parameters):
                module._parameters[key] = src._parameters[key]
            for key in list(module._buffers):
                module._buffers[key] = src._buffers[key]
        return twin.train(self.training)


def vmamba_tiny_s1l8(channel_first=True, **kwargs):
    return VSSM(depths=(2, 2, 8, 2), dims=(96, 192, 384, 768), d_state=1, ssm_ratio=1.0, mlp_ratio=4.0,
                channel_first=channel_first, **kwargs)
