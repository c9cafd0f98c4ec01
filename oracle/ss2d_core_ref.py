"""TEST INFRASTRUCTURE ONLY -- the SS2D core composed from the CPU oracle operators.

``RefSS2D`` is the package's SS2D block with ``forward_core`` replaced by the torch-on-CPU
restatement (oracle/torch_ref.py) in the order of classification/models/vmamba.py:603-646.  It
is what model-level parity tests compare against and what the benchmark times as the
"reference torch CPU path".
"""
import torch

from vmamba_amd.ss2d import SS2D
from . import torch_ref


class RefSS2D(SS2D):
    def forward_core(self, x):
        B, D, H, W = x.shape
        K, L = self.k_group, H * W
        xs = torch_ref.cross_scan(x)
        dts, Bs, Cs = self.project(xs.contiguous())
        ys = torch_ref.selective_scan(xs.reshape(B, K * D, L), dts, -self.A_logs.float().exp(), Bs.contiguous(),
                                      Cs.contiguous(), self.Ds.float(), self.dt_projs_bias.view(-1).float(), True)
        y = torch_ref.cross_merge(ys.view(B, K, D, H, W))
        return self.finish_core(y, B, D, H, W, x.dtype)
