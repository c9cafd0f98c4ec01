"""TEST INFRASTRUCTURE ONLY -- torch-on-CPU restatement of the reference's Python path.

Second, independent formulation of the three operators, built from library
``transpose`` / ``flip`` / ``einsum`` the way the reference's torch fallbacks
are.  It serves two purposes: (1) it cross-checks the C oracle (two
formulations written differently must agree), (2) it is the "reference torch
CPU path" that the benchmark times on the host cores as ``cpu_baseline``.

Follows, without importing them:
  cross_scan   classification/models/csm_triton.py:22-29 and :532-541
  cross_scan_1b1  classification/models/csm_triton.py:88-99 (one-by-one, scans = 0)
  cross_merge  classification/models/csm_triton.py:56-62 and :543-551
  cross_scan_flex / cross_merge_flex  every layout / mode of csm_triton.py:22-179, stated as index gathers
                  over the routes of the flex kernel (:308-328)
  selective_scan  kernels/selective_scan/test_selective_scan.py:168-234
                  (selective_scan_ref; same arithmetic as csms6s.py:25-68 but
                  the bias add and softplus happen after the widening to fp32,
                  as in the device kernel, selective_scan_fwd_kernel_oflex.cuh:123-127)
"""
import torch
import torch.nn.functional as F


def cross_scan(x):
    B, C, H, W = x.shape
    row_major = x.reshape(B, C, H * W)
    col_major = x.transpose(2, 3).reshape(B, C, H * W)
    return torch.stack([row_major, col_major, row_major.flip(-1), col_major.flip(-1)], dim=1)


def cross_scan_1b1(x):
    """x (B,4,C,H,W): direction slice k laid out in the scan order of direction k."""
    B, K, C, H, W = x.shape
    col = lambda v: v.transpose(2, 3).reshape(B, C, H * W)
    return torch.stack([x[:, 0].reshape(B, C, H * W), col(x[:, 1]),
                        x[:, 2].reshape(B, C, H * W).flip(-1), col(x[:, 3]).flip(-1)], dim=1)


def scan_routes(H, W, scans):
    """(4, L) int64: routes[k, r] = scan position at which direction k visits row-major spatial index r."""
    L = H * W
    r = torch.arange(L)
    col = (r % W) * H + r // W
    if scans == 0:
        return torch.stack([r, col, L - 1 - r, L - 1 - col])
    if scans == 1:
        return torch.stack([r, r, r, r])
    if scans == 2:
        return torch.stack([r, r, L - 1 - r, L - 1 - r])
    raise ValueError(scans)


def cross_scan_flex(x, in_channel_first=True, out_channel_first=True, one_by_one=False, scans=0):
    """x (B,[4,]C,H,W) | (B,H,W,[4,]C) -> y (B,4,C,L) | (B,L,4,C):  y_k[route_k(r)] = x_(k)[r]."""
    if in_channel_first:
        B, C, H, W = x.shape[0], x.shape[-3], x.shape[-2], x.shape[-1]
        xs = x.reshape(B, -1, C, H * W)
    else:
        B, H, W, C = x.shape[0], x.shape[1], x.shape[2], x.shape[-1]
        xs = x.reshape(B, H * W, -1, C).permute(0, 2, 3, 1)
    xs = xs.expand(B, 4, C, H * W)
    routes = scan_routes(H, W, scans)
    y = x.new_empty((B, 4, C, H * W))
    for k in range(4):
        y[:, k, :, routes[k]] = xs[:, k]
    return y if out_channel_first else y.permute(0, 3, 1, 2).contiguous()


def cross_merge_flex(y, in_channel_first=True, out_channel_first=True, one_by_one=False, scans=0, left_to_right=False):
    """y (B,4,C,H,W) | (B,H,W,4,C) -> x (B,[4,]C,L) | (B,L,[4,]C):  x[r] = sum_k y_k[route_k(r)] (one_by_one: no sum).
    scans 0, 2: (y0 + y2) + (y1 + y3) rounded per add (or left to right); scans 1: a 4-term reduction."""
    if out_channel_first:
        B, _, C, H, W = y.shape
        ys = y.reshape(B, 4, C, H * W)
    else:
        B, H, W, _, C = y.shape
        ys = y.reshape(B, H * W, 4, C).permute(0, 2, 3, 1)
    routes = scan_routes(H, W, scans)
    g = [ys[:, k][..., routes[k]] for k in range(4)]
    if one_by_one:
        x = torch.stack(g, dim=1)                                   # (B, 4, C, L)
        return x if in_channel_first else x.permute(0, 3, 1, 2).contiguous()
    if scans == 1:
        x = torch.stack(g, dim=1).sum(1)                            # the reference's y.sum(1)
    elif left_to_right:
        x = ((g[0] + g[1]) + g[2]) + g[3]
    else:
        x = (g[0] + g[2]) + (g[1] + g[3])
    return x if in_channel_first else x.permute(0, 2, 1).contiguous()


def cross_merge(ys):
    B, K, C, H, W = ys.shape
    y = ys.reshape(B, K, C, H * W)
    both = y[:, 0:2] + y[:, 2:4].flip(-1)            # (y0 + flip y2), (y1 + flip y3)
    col = both[:, 1].reshape(B, C, W, H).transpose(2, 3).reshape(B, C, H * W)
    return both[:, 0] + col


def cross_merge_left_to_right(ys):
    """Add order of the Triton kernel, csm_triton.py:362-370: ((y0+y1')+y2')+y3'."""
    B, K, C, H, W = ys.shape
    y = ys.reshape(B, K, C, H * W)
    t = lambda v: v.reshape(B, C, W, H).transpose(2, 3).reshape(B, C, H * W)
    return ((y[:, 0] + t(y[:, 1])) + y[:, 2].flip(-1)) + t(y[:, 3].flip(-1))


def layer_norm_rows(x, weight, bias, eps=1e-5, out_dtype=None):
    """nn.LayerNorm over the last axis, statistics in fp32 (what torch does for 16-bit inputs as well)."""
    y = F.layer_norm(x.float(), (x.shape[-1],), None if weight is None else weight.float(),
                     None if bias is None else bias.float(), eps)
    return y.to(out_dtype or x.dtype)


def layer_norm_cf(x, weight, bias, eps=1e-5, out_channel_last=False, out_dtype=None):
    """LayerNorm2d (classification/models/vmamba.py:52-57): permute to channel-last, layer_norm, permute back;
    with ``out_channel_last`` the result stays channel-last, which is forward_core's out_norm step in
    channel-last models (vmamba.py:642-644)."""
    nd = x.dim()
    to_cl = (0, *range(2, nd), 1)
    y = layer_norm_rows(x.permute(*to_cl), weight, bias, eps, out_dtype)
    return y.contiguous() if out_channel_last else y.permute(0, nd - 1, *range(1, nd - 1)).contiguous()


def dwconv3x3_silu(x, weight, bias=None, in_channel_last=False, apply_silu=True):
    """vmamba.py:654-658: to channel-first, depthwise conv2d (k=3, pad=1), SiLU -- as separate torch ops in x.dtype."""
    if in_channel_last:
        x = x.permute(0, 3, 1, 2)
    y = F.conv2d(x, weight.to(x.dtype), None if bias is None else bias.to(x.dtype), padding=1, groups=x.shape[1])
    return F.silu(y) if apply_silu else y


def selective_scan(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False, out_float=True,
                   return_last_state=False):
    dtype_in = u.dtype
    batch, dim, L = u.shape
    G, N = B.shape[1], B.shape[2]
    u32, dl = u.float(), delta.float()
    if delta.shape[1] != dim:                       # delta-group broadcast, oflex.h dim_deltagroups_ratio
        rep = dim // delta.shape[1]
        dl = dl.repeat_interleave(rep, dim=1)
        if delta_bias is not None:
            delta_bias = delta_bias.repeat_interleave(rep)
    if delta_bias is not None:
        dl = dl + delta_bias.float()[None, :, None]
    if delta_softplus:
        dl = F.softplus(dl)
    Bf = B.float().repeat_interleave(dim // G, dim=1)  # (batch, dim, N, L)
    Cf = C.float().repeat_interleave(dim // G, dim=1)
    decay = torch.exp(torch.einsum("bdl,dn->bdln", dl, A.float()))
    drive = torch.einsum("bdl,bdnl,bdl->bdln", dl, Bf, u32)
    h = torch.zeros(batch, dim, N, dtype=torch.float32)
    ys = []
    for t in range(L):
        h = decay[:, :, t] * h + drive[:, :, t]
        ys.append(torch.einsum("bdn,bdn->bd", h, Cf[..., t]))
    y = torch.stack(ys, dim=2) if L > 0 else torch.zeros(batch, dim, 0)
    if D is not None:
        y = y + u32 * D.float()[None, :, None]
    out = y if out_float else y.to(dtype_in)
    return (out, h) if return_last_state else out


def selective_scan_f64(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False):
    """The same recurrence in float64, differentiable by autograd (no dtype round trips): the gradient oracle."""
    batch, dim, L = u.shape
    G, N = B.shape[1], B.shape[2]
    dl = delta
    if delta.shape[1] != dim:
        rep = dim // delta.shape[1]
        dl = dl.repeat_interleave(rep, dim=1)
        if delta_bias is not None:
            delta_bias = delta_bias.repeat_interleave(rep)
    if delta_bias is not None:
        dl = dl + delta_bias[None, :, None]
    if delta_softplus:
        dl = F.softplus(dl)
    Bf = B.repeat_interleave(dim // G, dim=1)
    Cf = C.repeat_interleave(dim // G, dim=1)
    decay = torch.exp(torch.einsum("bdl,dn->bdln", dl, A))
    drive = torch.einsum("bdl,bdnl,bdl->bdln", dl, Bf, u)
    h = torch.zeros(batch, dim, N, dtype=u.dtype)
    ys = []
    for t in range(L):
        h = decay[:, :, t] * h + drive[:, :, t]
        ys.append(torch.einsum("bdn,bdn->bd", h, Cf[..., t]))
    y = torch.stack(ys, dim=2)
    if D is not None:
        y = y + u * D[None, :, None]
    return y


def selective_scan_grads(u, delta, A, B, C, D, delta_bias, dout, delta_softplus):
    """[du, ddelta, dA, dB, dC, dD, ddelta_bias] of sum(y * dout) by float64 autograd (None where the input is None)."""
    leaves = [None if t is None else t.detach().double().requires_grad_(True) for t in (u, delta, A, B, C, D, delta_bias)]
    y = selective_scan_f64(*leaves, delta_softplus=delta_softplus)
    y.backward(dout.double())
    return [None if t is None else t.grad for t in leaves]
