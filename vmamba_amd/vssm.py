"""VMamba-T-shaped backbone used as the throughput harness (random init, inference).

Layer order and shapes follow VSSM / VSSBlock of classification/models/vmamba.py:1153-1505 for
the ``vmamba_tiny_s1l8`` recipe (:1717-1728): channel-first ("ln2d"), patch-embed v2, downsample
v3, depths 2/2/8/2, dims 96/192/384/768, d_state 1, ssm_ratio 1, forward type v05_noz, MLP ratio 4.
Everything outside the SS2D core is stock torch; drop-path is the identity at inference.
"""
import torch
import torch.nn as nn

from .ss2d import SS2D, LayerNorm2d, Linear2d


class Mlp(nn.Module):
    def __init__(self, dim, hidden):
        super().__init__()
        self.fc1 = Linear2d(dim, hidden)
        self.act = nn.GELU()
        self.fc2 = Linear2d(hidden, dim)

    def forward(self, x):
        return self.fc2(self.act(self.fc1(x)))


class VSSBlock(nn.Module):
    def __init__(self, dim, d_state=1, ssm_ratio=1.0, mlp_ratio=4.0, ss2d_cls=SS2D, **ss2d_kwargs):
        super().__init__()
        self.norm = LayerNorm2d(dim)
        self.op = ss2d_cls(d_model=dim, d_state=d_state, ssm_ratio=ssm_ratio, **ss2d_kwargs)
        self.norm2 = LayerNorm2d(dim)
        self.mlp = Mlp(dim, int(dim * mlp_ratio))

    def forward(self, x):
        x = x + self.op(self.norm(x))
        return x + self.mlp(self.norm2(x))


class VSSM(nn.Module):
    def __init__(self, in_chans=3, num_classes=1000, depths=(2, 2, 8, 2), dims=(96, 192, 384, 768), d_state=1,
                 ssm_ratio=1.0, mlp_ratio=4.0, ss2d_cls=SS2D, **ss2d_kwargs):
        super().__init__()
        d0 = dims[0]
        self.patch_embed = nn.Sequential(
            nn.Conv2d(in_chans, d0 // 2, kernel_size=3, stride=2, padding=1), LayerNorm2d(d0 // 2), nn.GELU(),
            nn.Conv2d(d0 // 2, d0, kernel_size=3, stride=2, padding=1), LayerNorm2d(d0))
        layers = []
        for i, (depth, dim) in enumerate(zip(depths, dims)):
            blocks = [VSSBlock(dim, d_state, ssm_ratio, mlp_ratio, ss2d_cls, **ss2d_kwargs) for _ in range(depth)]
            down = (nn.Sequential(nn.Conv2d(dim, dims[i + 1], kernel_size=3, stride=2, padding=1), LayerNorm2d(dims[i + 1]))
                    if i + 1 < len(dims) else nn.Identity())
            layers.append(nn.Sequential(*blocks, down))
        self.layers = nn.ModuleList(layers)
        self.classifier = nn.Sequential(LayerNorm2d(dims[-1]), nn.AdaptiveAvgPool2d(1), nn.Flatten(1),
                                        nn.Linear(dims[-1], num_classes))
        self.apply(self._init_weights)

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


def vmamba_tiny_s1l8(**kwargs):
    return VSSM(depths=(2, 2, 8, 2), dims=(96, 192, 384, 768), d_state=1, ssm_ratio=1.0, mlp_ratio=4.0, **kwargs)
