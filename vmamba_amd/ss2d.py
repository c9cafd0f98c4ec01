"""SS2D block and its hot core, mirroring SS2Dv2 of classification/models/vmamba.py:380-664.

``SS2D.forward_core`` keeps the reference's calling convention, ``(B, D, H, W) -> (B, D, H, W)``
channel-first (vmamba.py:493-646, the non-cascade ``cross2d`` branch with ``no_einsum=True``,
``force_fp32=False``, i.e. forward types ``v05`` / ``v05_noz``):

    CrossScan -> x_proj -> split (dt, B, C) -> dt_proj -> selective scan -> CrossMerge -> out_norm

CrossScan, the selective scan and CrossMerge run on this package's HIP kernels; the two tiny
projections stay PyTorch-ROCm GEMMs.  B and C are handed to the scan as strided views of the
projection output: the kernel honours batch/group/state strides, so the reference's
``.contiguous()`` copies (vmamba.py:621-622) are not needed.

Parameter names, shapes and initialisation follow vmamba.py:165-232 and :463-479, so a
reference state_dict of this block loads as is.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from ._lib import SS2D_ENOTSUP, Ss2dError
from .core import (DT_PROJ_MAX_RANK, core_fits, core_mask_pads_hip, dt_proj_hip, embed_maps_hip, padded_map_size,
                   ss2d_core_hip)
from .csm import cross_merge_fn, cross_scan_1b1_hip, cross_scan_fn
from .csms6s import selective_scan_fn, selective_scan_from_map
from .conv import dwconv3x3_silu_hip
from .linear import linear_cf_ln_fusable, linear_cf_ln_hip, linear_cl_hip, linear_fusable
from .norm import (LayerNorm, LayerNorm2d, add_layer_norm_fusable, add_layer_norm_hip, layer_norm_cf_hip,
                   needs_grad)


class Linear2d(nn.Linear):
    """1x1 convolution stored as a Linear weight (vmamba.py:42-49)."""

    def forward(self, x):
        return F.conv2d(x, self.weight[:, :, None, None], self.bias)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        key = prefix + "weight"
        if key in state_dict:
            state_dict[key] = state_dict[key].view(self.weight.shape)
        return super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)


class HipLayers:
    """The layer classes the blocks are built from: LayerNorm on the HIP kernels of this package."""
    LayerNorm = LayerNorm
    LayerNorm2d = LayerNorm2d

    @staticmethod
    def out_norm(norm, y, channel_first, dtype):
        """out_norm of forward_core on the merged channel-first map y (B, D, H, W), returned in the block's
        layout and dtype: one kernel reads (B, D, L) and writes the normalised (B, D, L) or (B, L, D).  Under
        autograd: the reference's own torch operators (vmamba.py:641-646)."""
        if needs_grad(y, norm.weight, norm.bias):
            out = F.layer_norm(y.permute(0, 2, 3, 1), norm.normalized_shape, norm.weight, norm.bias, norm.eps)
            return (out.permute(0, 3, 1, 2) if channel_first else out).to(dtype)
        return layer_norm_cf_hip(y, norm.weight, norm.bias, norm.eps, out_channel_last=not channel_first, out_dtype=dtype)

    @staticmethod
    def conv_act(conv2d, x, channel_first):
        """Depthwise conv + SiLU on the in_proj output x ((B,D,H,W) if channel_first else (B,H,W,D)); returns the
        channel-first (B,D,H,W) input of forward_core (vmamba.py:654-658).  ``conv2d`` None means no conv."""
        fusable = conv2d is not None and conv2d.kernel_size == (3, 3) and conv2d.padding == (1, 1) and conv2d.stride == (1, 1)
        if fusable and not needs_grad(x, conv2d.weight, conv2d.bias):
            return dwconv3x3_silu_hip(x, conv2d.weight, conv2d.bias, in_channel_last=not channel_first, apply_silu=True)
        if not channel_first:
            x = x.permute(0, 3, 1, 2).contiguous()
        return F.silu(conv2d(x) if conv2d is not None else x)


def init_dt_A_D(d_state, dt_rank, d_inner, dt_scale=1.0, dt_min=0.001, dt_max=0.1, dt_init_floor=1e-4, k_group=4):
    """S4D-real A, unit D, dt bias = softplus^-1(dt), dt log-uniform in [dt_min, dt_max] (vmamba.py:165-232)."""
    std = dt_rank ** -0.5 * dt_scale
    dt_w = torch.empty(k_group, d_inner, dt_rank).uniform_(-std, std)
    dt = torch.exp(torch.rand(k_group, d_inner) * (math.log(dt_max) - math.log(dt_min)) + math.log(dt_min)).clamp(min=dt_init_floor)
    dt_b = dt + torch.log(-torch.expm1(-dt))
    A_logs = torch.log(torch.arange(1, d_state + 1, dtype=torch.float32)).repeat(k_group * d_inner, 1)
    Ds = torch.ones(k_group * d_inner)
    return nn.Parameter(A_logs), nn.Parameter(Ds), nn.Parameter(dt_w), nn.Parameter(dt_b)


_PAD_MASKS = {}            # the most recent (map size, image count) pairs
_PAD_MASKS_PINNED = {}     # those a graph capture has read: never dropped, a captured kernel holds their address


def _pad_mask(H0, W0, H, W, n_images, device):
    """(4, n_images * H*W) int16 tensor for dt_proj_hip: -1 (all bits set) at the scan positions of each direction
    (cross_scan_fwd's orders, classification/models/csm_triton.py:22-29, on the H x W map) that lie outside the map's
    top-left H0 x W0 part, 0 elsewhere; the same for every image."""
    key = (H0, W0, H, W, n_images, str(device))
    if key in _PAD_MASKS_PINNED:
        return _PAD_MASKS_PINNED[key]
    capturing = torch.device(device).type == "cuda" and torch.cuda.is_current_stream_capturing()
    mask = _PAD_MASKS.pop(key, None)
    built = mask is None
    if built:
        m = torch.zeros((H, W), dtype=torch.bool, device=device)      # built on the device: no host copy inside a capture
        m[H0:, :] = True
        m[:, W0:] = True
        rows, cols = m.flatten(), m.t().flatten()
        one = -torch.stack([rows, cols, rows.flip(0), cols.flip(0)]).to(torch.int16)
        mask = one.view(4, 1, H * W).expand(4, n_images, H * W).reshape(4, n_images * H * W)
    if capturing:
        if not built:              # (built inside the capture, its memory is the graph's own and is rewritten by every replay)
            _PAD_MASKS_PINNED[key] = mask
        return mask
    _PAD_MASKS[key] = mask                                            # (re-)inserted as the newest
    while len(_PAD_MASKS) > 8:
        _PAD_MASKS.pop(next(iter(_PAD_MASKS)))
    return mask


class SS2D(nn.Module):
    """SS2D block: in_proj -> dwconv3x3 -> SiLU -> forward_core -> (gate) -> out_proj.

    ``channel_first=True`` takes and returns (B, C, H, W) with 1x1-conv projections and LayerNorm2d
    (the reference's "ln2d" models); ``channel_first=False`` takes and returns (B, H, W, C) with nn.Linear
    and nn.LayerNorm (its "ln" models, vmamba.py:415-417, 642-643, 654-655).  The core itself always works
    channel-first.
    """

    def __init__(self, d_model=96, d_state=1, ssm_ratio=1.0, dt_rank="auto", d_conv=3, conv_bias=False, bias=False,
                 disable_z=True, dt_min=0.001, dt_max=0.1, dt_scale=1.0, dt_init_floor=1e-4, channel_first=True,
                 layers=HipLayers, fused_core=True):
        super().__init__()
        self.channel_first = channel_first
        self.fused_core = fused_core
        self.layers = layers
        Linear = Linear2d if channel_first else nn.Linear
        self.k_group = 4
        self.d_model, self.d_state = int(d_model), int(d_state)
        self.d_inner = int(ssm_ratio * d_model)
        self.dt_rank = int(math.ceil(self.d_model / 16) if dt_rank == "auto" else dt_rank)
        self.disable_z = disable_z
        self.with_dconv = d_conv > 1
        self.in_proj = Linear(self.d_model, self.d_inner if disable_z else 2 * self.d_inner, bias=bias)
        self.act = nn.SiLU()
        if self.with_dconv:
            self.conv2d = nn.Conv2d(self.d_inner, self.d_inner, kernel_size=d_conv, padding=(d_conv - 1) // 2,
                                    groups=self.d_inner, bias=conv_bias)
        x_proj = [nn.Linear(self.d_inner, self.dt_rank + 2 * self.d_state, bias=False) for _ in range(self.k_group)]
        self.x_proj_weight = nn.Parameter(torch.stack([t.weight for t in x_proj], dim=0))   # (K, R+2N, D)
        self.out_norm = layers.LayerNorm2d(self.d_inner) if channel_first else layers.LayerNorm(self.d_inner)
        self.out_proj = Linear(self.d_inner, self.d_model, bias=bias)
        self.A_logs, self.Ds, self.dt_projs_weight, self.dt_projs_bias = init_dt_A_D(
            self.d_state, self.dt_rank, self.d_inner, dt_scale, dt_min, dt_max, dt_init_floor, self.k_group)

    def _inference_constants(self, batch):
        """Tensors that depend only on the parameters (and the batch size): A = -exp(A_logs), fp32 D and dt bias
        (vmamba.py:619-623) and the projection weights repeated over the batch so each projection is ONE
        strided-batched GEMM over B*K problems.  Recomputed whenever autograd is on or a parameter changed; kept for up to
        four batch sizes.

        Under a graph capture the kernels record the addresses of these tensors.  An entry the capture reads is therefore
        moved to ``_pinned_consts``, which keeps it while the parameters stay as they are (entries for other parameter values are
        dropped when a new one is pinned), so it outlives any graph that may still be replayed; an entry
        missing during a capture is computed inside the graph (its memory then belongs to the graph and is rewritten by
        every replay) and is not kept.  Pinned entries are copies of the parameter values at capture time: whoever
        replays the graph must not do so after an in-place parameter update (ConcurrentGraphRunner.replay checks)."""
        params = (self.A_logs, self.Ds, self.dt_projs_bias, self.x_proj_weight, self.dt_projs_weight)
        key = (batch, torch.is_grad_enabled(), tuple((p._version, p.data_ptr(), p.dtype, p.device) for p in params))
        cache = self.__dict__.setdefault("_const_cache", {})
        pinned = self.__dict__.setdefault("_pinned_consts", {})
        capturing = self.A_logs.is_cuda and torch.cuda.is_current_stream_capturing()
        if key in pinned:
            return pinned[key]
        if key in cache:
            if capturing:
                # entries pinned for other parameter values belong to graphs that must not be replayed any more
                # (ConcurrentGraphRunner.replay refuses them): dropping them here keeps re-captures after weight
                # updates from piling up one set of batch-replicated weights each
                for k in [k for k in pinned if k[2] != key[2]]:
                    del pinned[k]
                pinned[key] = cache.pop(key)
                return pinned[key]
            return cache[key]
        K = self.k_group
        consts = dict(
            As=-self.A_logs.float().exp(), Ds=self.Ds.float(), dt_bias=self.dt_projs_bias.reshape(-1).float(),
            Wx_all=self.x_proj_weight.reshape(1, -1, self.d_inner).expand(batch, -1, -1).contiguous(),
            Wx=self.x_proj_weight.unsqueeze(0).expand(batch, -1, -1, -1).reshape(batch * K, -1, self.d_inner).contiguous(),
            Wdt=self.dt_projs_weight.unsqueeze(0).expand(batch, -1, -1, -1).reshape(batch * K, self.d_inner, -1).contiguous())
        if not torch.is_grad_enabled() and not capturing:
            stale = [k for k in cache if k[2] != key[2]]
            for k in stale:
                del cache[k]
            if len(cache) >= 4:
                cache.pop(next(iter(cache)))
            cache[key] = consts
        return consts

    def project(self, xs, consts=None):
        """x_proj and dt_proj (vmamba.py:605-615) as two strided-batched PyTorch-ROCm GEMMs.  xs: (B, K, D, L).

        The reference offers a grouped-conv1d and an einsum spelling of the same contraction; on this stack
        a batched matmul over the B*K (image, direction) problems is several times faster than either.
        Returns dts (B, K*D, L) and B, C as strided views (B, K, N, L) of the projection output.
        """
        B, K, D, L = xs.shape
        R, N = self.dt_rank, self.d_state
        consts = consts or self._inference_constants(B)
        x_dbl = torch.bmm(consts["Wx"], xs.view(B * K, D, L)).view(B, K, R + 2 * N, L)
        dts, Bs, Cs = torch.split(x_dbl, [R, N, N], dim=2)
        dts = torch.bmm(consts["Wdt"], dts.reshape(B * K, R, L)).view(B, K * D, L)
        return dts, Bs, Cs

    def project_from_map(self, x, consts):
        """The same dts, B, C as ``project(cross_scan(x))`` from the map x (B, D, H, W) itself: a projection is a
        per-position contraction, so x_proj is applied once to x in its natural order with the four directions' weights
        stacked, and only its small output (R + 2N rows per direction instead of D) is put into scan order, each
        direction's rows in that direction's order.  x_proj then reads the map once instead of its four copies."""
        B, D, H, W = x.shape
        K, L, R, N = self.k_group, H * W, self.dt_rank, self.d_state
        proj = torch.bmm(consts["Wx_all"], x.reshape(B, D, L)).view(B, K, R + 2 * N, H, W)
        x_dbl = cross_scan_fn(proj, in_channel_first=True, out_channel_first=True, one_by_one=True, scans=0)   # (B, K, R+2N, L)
        dts, Bs, Cs = torch.split(x_dbl, [R, N, N], dim=2)
        dts = dts.reshape(B * K, R, L)
        if dts.dtype != torch.float32 and R <= DT_PROJ_MAX_RANK and not needs_grad(dts, self.dt_projs_weight):
            dts = dt_proj_hip(dts, consts["Wdt"])                     # one (image, direction) problem per weight copy
        else:
            dts = torch.bmm(consts["Wdt"], dts)
        return dts.view(B, K * D, L), Bs, Cs

    def forward_core_fused(self, x, consts, crop=True):
        """One state per channel: the three operators as ONE kernel (ss2d_core_fwd).  Returns y (B, D, L) fp32; with
        ``crop=False`` the pair (y on the map the kernel ran on -- possibly a padded one --, that map's (H, W)).

        A projection is a per-position contraction, so x_proj is applied to x in its natural order for all four
        directions at once, and only its small output (R + 2 rows per direction instead of D) is put into scan
        order -- direction-major and batch-innermost, which makes dt_proj ONE GEMM per direction over all B*L
        positions and hands the kernel delta rows of consecutive images side by side.
        """
        B, D, H0, W0 = x.shape
        K, R = self.k_group, self.dt_rank
        C = R + 2
        # Maps the kernel would walk element by element (sides like 57 x 58, 75, 19: a number of positions that is not a
        # multiple of 4) are embedded in a slightly larger map: zeros on the added rows / columns, the projections
        # computed on the padded map, and the step of the added positions set to 0 (delta = -inf), which makes them
        # neutral elements of the scan; the result is cropped.
        padded = padded_map_size(H0, W0, x.dtype)
        if padded is not None:
            x = embed_maps_hip(x.contiguous().view(B * D, H0, W0), padded[0], padded[1]).view(B, D, padded[0], padded[1])
        H, W = x.shape[2], x.shape[3]
        L = H * W
        proj = torch.bmm(consts["Wx_all"], x.view(B, D, L))                                   # (B, K*C, L)
        # Rows of B*L positions start on 16-byte boundaries only if B*L is a multiple of the 16-byte vector: maps with
        # an odd (or 2, 4 mod 8) number of positions get room for a few images more, which nothing reads back --
        # dt_proj and the kernel's delta stream then keep their 16-byte accesses.
        vec = 16 // proj.element_size()
        unit = vec // math.gcd(L, vec)
        Bp = (B + unit - 1) // unit * unit
        # On a padded map the step of the added positions must be 0: the 16-bit dt_proj on the matrix cores writes -1e30
        # (-65504 in fp16) there instead of the projection (a mask of those positions in each direction's order), and the
        # softplus of that is exactly 0.  Otherwise ss2d_core_mask_pads writes -inf into delta afterwards, a scattered
        # pass over its rows.
        x_dbl = proj.new_empty((K, C, B, L)) if Bp == B else proj.new_zeros((K, C, Bp, L))
        cross_scan_1b1_hip(proj.view(B, K, C, H, W), out=x_dbl[:, :, :B].permute(2, 0, 1, 3))
        dts = x_dbl[:, :R].reshape(K, R, Bp * L)
        if dts.dtype != torch.float32 and R <= DT_PROJ_MAX_RANK:
            if padded is not None:
                big = -65504.0 if proj.dtype == torch.float16 else -1e30
                delta = dt_proj_hip(dts, self.dt_projs_weight, _pad_mask(H0, W0, H, W, Bp, proj.device), big).view(K, D, Bp, L)
            else:
                delta = dt_proj_hip(dts, self.dt_projs_weight).view(K, D, Bp, L)
        else:
            delta = torch.bmm(self.dt_projs_weight, dts).view(K, D, Bp, L)
            if padded is not None:
                core_mask_pads_hip(delta[:, :, :B], H0, W0, H, W)
        y = ss2d_core_hip(x, delta[:, :, :B], x_dbl[:, R, :B], x_dbl[:, R + 1, :B], consts["As"].view(-1), consts["Ds"],
                          consts["dt_bias"], True)
        if not crop:
            return y, (H, W)
        if padded is not None:
            y = embed_maps_hip(y.view(B * D, H, W), H0, W0).view(B, D, H0 * W0)
        return y

    def _fused_core_applies(self, x):
        """The fused kernel is an inference kernel for one-state models whose map fits its LDS planes; under autograd
        the three operators (each with a backward) run."""
        trains = needs_grad(x, self.x_proj_weight, self.dt_projs_weight, self.A_logs, self.Ds, self.dt_projs_bias)
        return self.d_state == 1 and self.fused_core and not trains and core_fits(x.shape[2], x.shape[3], x.dtype)

    def forward_core(self, x):
        B, D, H, W = x.shape
        K, L = self.k_group, H * W
        consts = self._inference_constants(B)
        if self._fused_core_applies(x):
            try:
                # out_norm runs on the map the kernel ran on (a padded map has rows the norm's vector paths like as
                # well) and the added rows / columns are cut off its 16-bit result, half the bytes of the fp32 map
                y, (Hp, Wp) = self.forward_core_fused(x, consts, crop=False)
                out = self.finish_core(y, B, D, Hp, Wp, x.dtype)
                if (Hp, Wp) != (H, W):
                    if self.channel_first:
                        out = embed_maps_hip(out.contiguous().view(-1, Hp, Wp), H, W).view(B, -1, H, W)
                    else:
                        Dm = out.shape[-1]
                        out = embed_maps_hip(out.contiguous().view(B, Hp, Wp * Dm), H, W * Dm).view(B, H, W, Dm)
                return out
            except Ss2dError as e:          # a shape the fused kernel has no variant for: the three operators take it
                if e.code != SS2D_ENOTSUP:
                    raise
        dts, Bs, Cs = self.project_from_map(x, consts)
        ys = None
        if self.d_state > 1 and x.is_cuda and not needs_grad(x, dts, Bs, self.A_logs, self.Ds, self.dt_projs_bias):
            # several states per channel: the scan kernel reads x through CrossScan's routes, xs is never written
            try:
                ys = selective_scan_from_map(x, dts, consts["As"], Bs, Cs, consts["Ds"], consts["dt_bias"], True, True)
            except Ss2dError as e:
                if e.code != SS2D_ENOTSUP:
                    raise
        if ys is None:
            xs = cross_scan_fn(x, in_channel_first=True, out_channel_first=True, scans=0)      # (B, 4, D, L)
            ys = selective_scan_fn(xs.view(B, K * D, L), dts, consts["As"], Bs, Cs, consts["Ds"], consts["dt_bias"],
                                   True, True)                                                 # fp32 (oflex)
        y = cross_merge_fn(ys.view(B, K, D, H, W), in_channel_first=True, out_channel_first=True, scans=0)
        return self.finish_core(y, B, D, H, W, x.dtype)

    def finish_core(self, y, B, D, H, W, dtype):
        """out_norm on the merged (B, D, L) map, in the block's layout (vmamba.py:641-646)."""
        return self.layers.out_norm(self.out_norm, y.view(B, D, H, W), self.channel_first, dtype)

    def _forward_with_post_norm(self, x, residual, pre_norm, post_norm):
        fuse = (residual is not None and not self.channel_first and isinstance(post_norm, nn.LayerNorm)
                and post_norm.elementwise_affine and add_layer_norm_fusable(residual, residual)
                and not self._narrow(residual, self.out_proj)
                and not needs_grad(residual, self.out_proj.weight, self.out_proj.bias, post_norm.weight, post_norm.bias))
        if not fuse:
            total = self.forward(x, residual, pre_norm)
            return total, post_norm(total)
        proj = self.forward(x, None, pre_norm)
        return add_layer_norm_hip(proj, residual, post_norm.weight, post_norm.bias, post_norm.eps)

    def _narrow(self, x, linear, *extra):
        """True when ss2d_linear_cl serves this projection: channel-last, 16-bit, width 96, no autograd."""
        return (not self.channel_first and isinstance(linear, nn.Linear) and not isinstance(linear, Linear2d)
                and linear_fusable(x, linear.weight) and not needs_grad(x, linear.weight, linear.bias, *extra))

    def _norm_proj_fusable(self, x, residual):
        """True when ss2d_linear_cf_ln serves out_norm + out_proj (+ residual) of this block for the conv output x."""
        L = x.shape[2] * x.shape[3]
        return (not self.channel_first and isinstance(self.out_norm, LayerNorm) and self.out_norm.elementwise_affine
                and isinstance(self.out_proj, nn.Linear) and not isinstance(self.out_proj, Linear2d)
                and self.out_proj.weight.dtype == x.dtype and self._fused_core_applies(x)
                and x.is_cuda and linear_cf_ln_fusable(self.d_inner, self.out_proj.weight, L)
                and (residual is None or residual.dtype == x.dtype)
                and not needs_grad(residual, self.out_proj.weight, self.out_proj.bias, self.out_norm.weight, self.out_norm.bias))

    def forward(self, x, residual=None, pre_norm=None, post_norm=None):
        """``pre_norm``: the block's LayerNorm, applied to x first (vmamba.py:1227); ``residual`` (same layout as x) is
        added to the result (:1228).  A channel-last block of width 96 runs norm + in_proj and out_proj + add as one
        HIP kernel each (ss2d_linear_cl); otherwise channel-last blocks without an out_proj bias fold the addition
        into the out_proj GEMM (one pass over the activation fewer than the block's separate add).

        ``post_norm``: the block's second LayerNorm (:1229).  When given, the result is the pair
        (sum, post_norm(sum)); in channel-last 16-bit inference the add and the LayerNorm are one kernel
        (ss2d_add_layer_norm) behind a plain out_proj GEMM."""
        if post_norm is not None:
            return self._forward_with_post_norm(x, residual, pre_norm, post_norm)
        if (pre_norm is not None and isinstance(pre_norm, nn.LayerNorm) and pre_norm.elementwise_affine
                and self._narrow(x, self.in_proj, pre_norm.weight, pre_norm.bias)):
            x = linear_cl_hip(x, self.in_proj.weight, self.in_proj.bias, None, pre_norm.weight, pre_norm.bias, pre_norm.eps)
        else:
            x = self.in_proj(x if pre_norm is None else pre_norm(x))
        z = None
        if not self.disable_z:
            x, z = x.chunk(2, dim=(1 if self.channel_first else -1))
            z = self.act(z)
        x = self.layers.conv_act(self.conv2d if self.with_dconv else None, x, self.channel_first)   # (B, D, H, W)
        if z is None and self._norm_proj_fusable(x, residual):
            # out_norm, out_proj and the residual add in one kernel, straight from the core's fp32 map
            B, _, H, W = x.shape
            try:
                y = self.forward_core_fused(x, self._inference_constants(B))                    # (B, D, L) fp32
            except Ss2dError as e:          # no fused variant for this shape: forward_core's three-operator path below
                if e.code != SS2D_ENOTSUP:
                    raise
                y = None
            if y is not None:
                return linear_cf_ln_hip(y, self.out_norm.weight, self.out_norm.bias, self.out_norm.eps, self.out_proj.weight,
                                        self.out_proj.bias, residual).view(B, H, W, self.d_model)
        y = self.forward_core(x)
        if z is not None:
            y = y * z
        if self._narrow(y, self.out_proj, residual):
            return linear_cl_hip(y, self.out_proj.weight, self.out_proj.bias, residual)
        if residual is None:
            return self.out_proj(y)
        if self.channel_first or self.out_proj.bias is not None:
            return residual + self.out_proj(y)
        return torch.addmm(residual.reshape(-1, self.d_model), y.reshape(-1, self.d_inner), self.out_proj.weight.t()).view(residual.shape)
