"""Pins the CPU oracle (oracle/ss2d_oracle.c and oracle/torch_ref.py) without the reference.

Every check is chosen so that a plausible slip (a transposed index, a dropped flip, a wrong
add order, a missing bias, the wrong group for B/C) fails at least one of them.
"""
import json
import math
import os

import pytest
import torch

from oracle import ss2d_oracle as orc
from oracle import torch_ref


@pytest.fixture(scope="module")
def kat(golden_dir):
    with open(os.path.join(golden_dir, "cross_scan_kat.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def scan_golden(golden_dir):
    with open(os.path.join(golden_dir, "selective_scan_f64.json")) as f:
        return json.load(f)


# ---------------------------------------------------------------- cross scan
@pytest.mark.parametrize("impl", [orc.cross_scan, torch_ref.cross_scan])
def test_cross_scan_known_answers(kat, impl):
    for case in kat["scan"]:
        H, W = case["H"], case["W"]
        x = torch.tensor(case["x"], dtype=torch.float32).view(1, 1, H, W)
        y = impl(x)
        assert y.shape == (1, 4, 1, H * W)
        assert y.view(4, -1).tolist() == [[float(v) for v in row] for row in case["y"]]


@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (2, 3, 3, 5), (1, 2, 7, 7), (2, 2, 14, 14), (1, 3, 56, 57), (1, 2, 57, 58)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.int64, torch.uint8])
def test_cross_scan_brute_force_and_second_formulation(shape, dtype):
    B, C, H, W = shape
    g = torch.Generator().manual_seed(1)
    x = torch.randint(0, 250, shape, generator=g).to(dtype)
    y = orc.cross_scan(x)
    assert torch.equal(y, torch_ref.cross_scan(x))
    L = H * W
    for b in range(B):
        for c in range(C):
            for h in range(0, H, max(1, H // 5)):
                for w in range(0, W, max(1, W // 5)):
                    v = x[b, c, h, w]
                    assert y[b, 0, c, h * W + w] == v
                    assert y[b, 1, c, w * H + h] == v
                    assert y[b, 2, c, L - 1 - (h * W + w)] == v
                    assert y[b, 3, c, L - 1 - (w * H + h)] == v
    # each direction is a permutation of the map
    for k in range(4):
        assert torch.equal(y[:, k].float().sort(-1).values, x.reshape(B, C, L).float().sort(-1).values)


def test_cross_scan_1b1_pins():
    """One-by-one scan: with the same map in all four slices it IS cross_scan; and slice k only depends on
    input slice k (checked by perturbing one slice at a time)."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 3, 4, 6, generator=g)
    x4 = x.unsqueeze(1).expand(-1, 4, -1, -1, -1).contiguous()
    assert torch.equal(torch_ref.cross_scan_1b1(x4), orc.cross_scan(x))
    base = torch.randn(2, 4, 3, 4, 6, generator=g)
    y = torch_ref.cross_scan_1b1(base)
    for k in range(4):
        z = base.clone()
        z[:, k] += 1.0
        yz = torch_ref.cross_scan_1b1(z)
        for kk in range(4):
            assert torch.equal(yz[:, kk], y[:, kk]) == (kk != k)
        assert torch.equal(yz[:, k], orc.cross_scan(z[:, k])[:, k])


def _flat_offsets(B, C, H, W, x_cl, y_cl, one_by_one):
    """Flat element offsets of x[b,(k),c,r] and y[b,k,c,j], as the flex kernel computes its pointers
    (classification/models/csm_triton.py:330-384): channel-first = (B,[4,]C,L) / (B,4,C,L), channel-last =
    (B,L,[4,]C) / (B,L,4,C)."""
    L, K = H * W, (4 if one_by_one else 1)

    def xo(b, k, c, r):
        kk = k if one_by_one else 0
        return ((b * L + r) * K + kk) * C + c if x_cl else ((b * K + kk) * C + c) * L + r

    def yo(b, k, c, j):
        return ((b * L + j) * 4 + k) * C + c if y_cl else ((b * 4 + k) * C + c) * L + j
    return xo, yo


def _route(k, scans, h, w, H, W):
    """csm_triton.py:308-328: none; trans; flip; trans + flip | none x4 | none, none, flip, flip."""
    L = H * W
    if scans == 0:
        return [h * W + w, w * H + h, L - 1 - (h * W + w), L - 1 - (w * H + h)][k]
    if scans == 1:
        return h * W + w
    return h * W + w if k < 2 else L - 1 - (h * W + w)


@pytest.mark.parametrize("scans", [0, 1, 2])
@pytest.mark.parametrize("one_by_one", [False, True])
@pytest.mark.parametrize("x_cl,y_cl", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_cross_flex_against_flat_offset_loops(x_cl, y_cl, one_by_one, scans):
    """The tensor formulation against element-by-element loops over flat offsets, for every layout and mode; the
    default mode is also tied to the functions the known-answer cases pin."""
    B, C, H, W = 2, 3, 3, 4
    L, K = H * W, (4 if one_by_one else 1)
    xo, yo = _flat_offsets(B, C, H, W, x_cl, y_cl, one_by_one)
    x_flat = torch.arange(B * K * C * L, dtype=torch.float32) + 1
    shape = ((B, H, W) + ((4,) if one_by_one else ()) + (C,)) if x_cl else ((B,) + ((4,) if one_by_one else ()) + (C, H, W))
    x = x_flat.view(shape)
    want = torch.zeros(B * 4 * C * L)
    for b in range(B):
        for k in range(4):
            for c in range(C):
                for h in range(H):
                    for w in range(W):
                        want[yo(b, k, c, _route(k, scans, h, w, H, W))] = x_flat[xo(b, k, c, h * W + w)]
    got = torch_ref.cross_scan_flex(x, not x_cl, not y_cl, one_by_one, scans)
    assert got.shape == ((B, L, 4, C) if y_cl else (B, 4, C, L))
    assert torch.equal(got.reshape(-1), want)
    # merge: x[b,(k),c,r] = sum_k y[b,k,c,route_k(r)]
    y_flat = torch.arange(B * 4 * C * L, dtype=torch.float32) * 3 + 2
    y = y_flat.view((B, H, W, 4, C) if y_cl else (B, 4, C, H, W))
    wantm = torch.zeros(B * K * C * L)
    for b in range(B):
        for c in range(C):
            for h in range(H):
                for w in range(W):
                    terms = [y_flat[yo(b, k, c, _route(k, scans, h, w, H, W))] for k in range(4)]
                    if one_by_one:
                        for k in range(4):
                            wantm[xo(b, k, c, h * W + w)] = terms[k]
                    else:
                        wantm[xo(b, 0, c, h * W + w)] = sum(terms)
    gotm = torch_ref.cross_merge_flex(y, not x_cl, not y_cl, one_by_one, scans)
    assert gotm.shape == (((B, L) + ((4,) if one_by_one else ()) + (C,)) if x_cl else ((B,) + ((4,) if one_by_one else ()) + (C, L)))
    assert torch.equal(gotm.reshape(-1), wantm)            # small integers: every order of addition is exact
    if not (x_cl or y_cl or scans):
        if one_by_one:
            assert torch.equal(got, torch_ref.cross_scan_1b1(x))
        else:
            assert torch.equal(got, orc.cross_scan(x)) and torch.equal(gotm, orc.cross_merge(y))


@pytest.mark.parametrize("scans", [0, 1, 2])
def test_cross_merge_flex_rounding(scans):
    """bf16: scans 0 / 2 round every pairwise add; scans 1 is the library reduction over the four copies."""
    g = torch.Generator().manual_seed(9)
    y = (torch.randn(2, 4, 3, 5, 6, generator=g) * 3).bfloat16()
    B, K, C, H, W = y.shape
    routes = torch_ref.scan_routes(H, W, scans)
    t = [y.view(B, 4, C, -1)[:, k][..., routes[k]] for k in range(4)]
    got = torch_ref.cross_merge_flex(y, scans=scans)
    if scans == 1:
        assert torch.equal(got, y.view(B, 4, C, -1).sum(1))
    else:
        want = ((t[0].float() + t[2].float()).bfloat16().float() + (t[1].float() + t[3].float()).bfloat16().float()).bfloat16()
        assert torch.equal(got, want)
        ltr = torch_ref.cross_merge_flex(y, scans=scans, left_to_right=True)
        w2 = t[0]
        for k in (1, 2, 3):
            w2 = (w2.float() + t[k].float()).bfloat16()
        assert torch.equal(ltr, w2)


def test_cross_scan_empty():
    assert orc.cross_scan(torch.zeros(0, 3, 4, 4)).shape == (0, 4, 3, 16)
    assert orc.cross_scan(torch.zeros(2, 0, 4, 4)).shape == (2, 4, 0, 16)


# --------------------------------------------------------------- cross merge
@pytest.mark.parametrize("impl", [orc.cross_merge, torch_ref.cross_merge])
def test_cross_merge_known_answer(kat, impl):
    m = kat["merge"]
    ys = torch.tensor(m["ys"], dtype=torch.float32).view(1, 4, 1, m["H"], m["W"])
    assert impl(ys).view(-1).tolist() == [float(v) for v in m["out"]]
    for case in kat["scan"]:
        ys = torch.tensor(case["y"], dtype=torch.float32).view(1, 4, 1, case["H"], case["W"])
        assert impl(ys).view(-1).tolist() == [float(v) for v in case["merged"]]


@pytest.mark.parametrize("shape", [(2, 3, 3, 5), (1, 2, 7, 7), (1, 3, 56, 57), (1, 2, 57, 58)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_cross_merge_matches_second_formulation_bitwise(shape, dtype):
    B, C, H, W = shape
    g = torch.Generator().manual_seed(2)
    ys = torch.randn((B, 4, C, H, W), generator=g).to(dtype)
    assert torch.equal(orc.cross_merge(ys), torch_ref.cross_merge(ys))
    assert torch.equal(orc.cross_merge(ys, order=1), torch_ref.cross_merge_left_to_right(ys))


def test_cross_merge_add_order_is_observable():
    # values chosen so that fp32 rounding separates the two association orders
    y = torch.zeros(1, 4, 1, 1, 1)
    y[0, 0], y[0, 1], y[0, 2], y[0, 3] = 1.0, 2.0 ** -24, -1.0, 2.0 ** -24
    # torch order: (1 + -1) + (2^-24 + 2^-24) = 2^-23 ; left-to-right: ((1+2^-24)+-1)+2^-24 = 2^-24
    assert orc.cross_merge(y).item() == 2.0 ** -23
    assert orc.cross_merge(y, order=1).item() == 2.0 ** -24
    # bf16: each pairwise sum is rounded to bf16
    yb = torch.zeros(1, 4, 1, 1, 1, dtype=torch.bfloat16)
    yb[0, 0], yb[0, 1], yb[0, 2], yb[0, 3] = 1.0, 2.0 ** -9, -1.0, 2.0 ** -9
    assert orc.cross_merge(yb).item() == 2.0 ** -8
    assert orc.cross_merge(yb, order=1).item() == 2.0 ** -9


@pytest.mark.parametrize("shape", [(2, 3, 3, 5), (2, 4, 14, 14), (1, 2, 57, 58)])
def test_merge_of_scan_is_four_x_and_adjoint(shape):
    B, C, H, W = shape
    g = torch.Generator().manual_seed(3)
    x = torch.randn(shape, generator=g)
    for order in (0, 1):
        assert torch.equal(orc.cross_merge(orc.cross_scan(x).view(B, 4, C, H, W), order=order).view(shape), 4 * x)
    # <scan(x), y> == <x, merge(y)> (how the reference defines the backward, csm_triton.py:208-225)
    xi = torch.randint(-8, 8, shape, generator=g).float()
    yi = torch.randint(-8, 8, (B, 4, C, H, W), generator=g).float()
    lhs = (orc.cross_scan(xi).view(-1) * yi.view(-1)).sum()
    rhs = (xi.view(-1) * orc.cross_merge(yi).view(-1)).sum()
    assert lhs == rhs


# ------------------------------------------------------------ selective scan
def _t(v, dtype=torch.float32):
    return None if v is None else torch.tensor(v, dtype=dtype)


def _case_tensors(case):
    return dict(u=_t(case["u"]), delta=_t(case["delta"]), A=_t(case["A"]), B=_t(case["B"]), C=_t(case["C"]),
                D=_t(case["D"]), delta_bias=_t(case["delta_bias"]), delta_softplus=case["delta_softplus"])


@pytest.mark.parametrize("idx", range(5))
def test_scan_golden_float64_vectors(scan_golden, idx):
    case = scan_golden[idx]
    kw = _case_tensors(case)
    want = torch.tensor(case["out"], dtype=torch.float64)
    wide = orc.selective_scan(**kw, wide=True)
    assert torch.allclose(wide, want, rtol=1e-12, atol=1e-12)
    got, xst = orc.selective_scan(**kw, return_x=True)
    assert torch.allclose(got.double(), want, rtol=1e-4, atol=1e-5)
    last = torch.tensor(case["last_state"], dtype=torch.float64)
    assert torch.allclose(xst[:, :, -1, 1::2].double(), last, rtol=1e-4, atol=1e-5)
    ref, h = torch_ref.selective_scan(**kw, return_last_state=True)
    assert torch.allclose(ref.double(), want, rtol=1e-4, atol=1e-5)
    assert torch.allclose(h.double(), last, rtol=1e-4, atol=1e-5)


def _rand_inputs(seed, batch, dim, G, N, L, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    # distributions of the reference's own test, test_selective_scan.py:414-444
    A = -0.5 * torch.rand(dim, N, generator=g)
    B = torch.randn(batch, G, N, L, generator=g).to(dtype)
    C = torch.randn(batch, G, N, L, generator=g).to(dtype)
    D = torch.randn(dim, generator=g)
    bias = 0.5 * torch.rand(dim, generator=g)
    u = torch.randn(batch, dim, L, generator=g).to(dtype)
    delta = (0.5 * torch.rand(batch, dim, L, generator=g)).to(dtype)
    return u, delta, A, B, C, D, bias


@pytest.mark.parametrize("N,L", [(1, 64), (1, 300), (8, 129), (16, 40)])
@pytest.mark.parametrize("softplus", [False, True])
def test_scan_c_oracle_vs_torch_restatement(N, L, softplus):
    u, delta, A, B, C, D, bias = _rand_inputs(5, 2, 8, 2, N, L)
    a = orc.selective_scan(u, delta, A, B, C, D, bias, softplus)
    b = torch_ref.selective_scan(u, delta, A, B, C, D, bias, softplus)
    assert torch.allclose(a, b, rtol=1e-5, atol=1e-5)
    w = orc.selective_scan(u, delta, A, B, C, D, bias, softplus, wide=True)
    assert torch.allclose(a.double(), w, rtol=1e-4, atol=1e-4)


def test_scan_length_one_closed_form():
    u, delta, A, B, C, D, bias = _rand_inputs(6, 3, 4, 2, 3, 1)
    out = orc.selective_scan(u, delta, A, B, C, D, bias, True)
    dl = torch.nn.functional.softplus(delta + bias[None, :, None])
    Bf, Cf = B.repeat_interleave(2, 1), C.repeat_interleave(2, 1)
    want = (Cf * Bf).sum(2) * dl * u + D[None, :, None] * u      # y = C.B dl u + D u
    assert torch.allclose(out, want, rtol=1e-5, atol=1e-6)


def test_scan_zero_A_is_cumsum():
    u, delta, A, B, C, D, bias = _rand_inputs(7, 2, 4, 4, 1, 200)
    out = orc.selective_scan(u, delta, torch.zeros_like(A), B, C, None, None, False)
    h = torch.cumsum((delta * B[:, :, 0] * u).double(), dim=-1)
    assert torch.allclose(out.double(), h * C[:, :, 0].double(), rtol=1e-4, atol=1e-4)


def test_scan_geometric_series():
    L, dl, Av = 500, 0.05, -0.7
    one = torch.ones(1, 1, L)
    out = orc.selective_scan(one, dl * one, torch.tensor([[Av]]), one.view(1, 1, 1, L), one.view(1, 1, 1, L))
    a = math.exp(dl * Av)
    want = torch.tensor([dl * (1 - a ** (t + 1)) / (1 - a) for t in range(L)], dtype=torch.float64)
    assert torch.allclose(out.view(-1).double(), want, rtol=1e-4)


def test_scan_zero_B_is_skip_path_and_output_dtype():
    u, delta, A, B, C, D, bias = _rand_inputs(8, 2, 4, 2, 2, 50, dtype=torch.bfloat16)
    out = orc.selective_scan(u, delta, A, torch.zeros_like(B), C, D, bias, True)
    assert out.dtype == torch.float32 and torch.equal(out, u.float() * D[None, :, None])
    out_in = orc.selective_scan(u, delta, A, torch.zeros_like(B), C, D, bias, True, out_float=False)
    assert out_in.dtype == torch.bfloat16 and torch.equal(out_in, (u.float() * D[None, :, None]).bfloat16())


def test_scan_softplus_threshold_and_bias():
    # delta+bias > 20 passes through unchanged (fwd_kernel_oflex.cuh:126); softplus(0)=ln 2
    one = torch.ones(1, 1, 1)
    k = dict(A=torch.zeros(1, 1), B=one.view(1, 1, 1, 1), C=one.view(1, 1, 1, 1))
    assert orc.selective_scan(one, 20.0 * one, delta_bias=torch.tensor([5.0]), delta_softplus=True, **k).item() == 25.0
    got = orc.selective_scan(one, -3.0 * one, delta_bias=torch.tensor([3.0]), delta_softplus=True, **k).item()
    assert abs(got - math.log(2.0)) < 1e-6
    assert orc.selective_scan(one, -3.0 * one, delta_bias=torch.tensor([3.5]), delta_softplus=False, **k).item() == 0.5


def test_scan_group_broadcast_uses_floor_division():
    # channel d reads B[:, d // (dim/G)] (csms6s.py:53 == fwd_kernel_oflex.cuh:90)
    batch, dim, G, L = 1, 6, 3, 5
    u, dl = torch.ones(batch, dim, L), torch.ones(batch, dim, L)
    B = torch.arange(1, G + 1).float().view(1, G, 1, 1).expand(1, G, 1, L).contiguous()
    C = torch.ones(1, G, 1, L)
    out = orc.selective_scan(u, dl, torch.zeros(dim, 1), B, C)
    assert out[0, :, 0].tolist() == [1.0, 1.0, 2.0, 2.0, 3.0, 3.0]
    # delta groups: delta (batch, 2, L) shared by dim/2 channels each (test_selective_scan.py:446-450)
    dl2 = torch.tensor([1.0, 3.0]).view(1, 2, 1).expand(1, 2, L).contiguous()
    out = orc.selective_scan(u, dl2, torch.zeros(dim, 1), torch.ones(1, 1, 1, L), torch.ones(1, 1, 1, L))
    assert out[0, :, 0].tolist() == [1.0, 1.0, 1.0, 3.0, 3.0, 3.0]


def test_scan_chunk_states_layout():
    # x[b,d,c,2n] = running product of a since t=0, x[b,d,c,2n+1] = h at chunk end (chunks of 2048)
    L = 2048 + 700
    u, delta, A, B, C, D, bias = _rand_inputs(9, 1, 2, 1, 2, L)
    out, xst = orc.selective_scan(u, delta, A, B, C, D, bias, True, return_x=True)
    assert xst.shape == (1, 2, 2, 4)
    _, h_end = torch_ref.selective_scan(u, delta, A, B, C, D, bias, True, return_last_state=True)
    assert torch.allclose(xst[:, :, -1, 1::2], h_end, rtol=1e-4, atol=1e-5)
    _, h_mid = torch_ref.selective_scan(u[..., :2048], delta[..., :2048], A, B[..., :2048], C[..., :2048], D, bias, True,
                                        return_last_state=True)
    assert torch.allclose(xst[:, :, 0, 1::2], h_mid, rtol=1e-4, atol=1e-5)
    dl = torch.nn.functional.softplus(delta + bias[None, :, None]).double()
    aprod = torch.exp((dl.sum(-1)[..., None] * A.double()[None]))
    assert torch.allclose(xst[:, :, -1, 0::2].double(), aprod, rtol=1e-3, atol=1e-30)


def test_scan_split_invariance():
    # scanning [0,s) then [s,L) with the carried state equals one scan: the state after s steps is
    # recovered from the outputs with C=1, N=1
    L, s = 90, 37
    u, delta, A, B, C, D, bias = _rand_inputs(10, 1, 3, 1, 1, L)
    ones = torch.ones_like(C)
    h = orc.selective_scan(u, delta, A, B, ones, None, bias, True)            # h_t itself
    h2 = orc.selective_scan(u[..., s:], delta[..., s:], A, B[..., s:], ones[..., s:], None, bias, True)
    dl = torch.nn.functional.softplus(delta + bias[None, :, None])
    decay = torch.exp(torch.cumsum(dl[..., s:] * A[None, :, 0, None], -1))
    assert torch.allclose(h[..., s:], h2 + decay * h[..., s - 1:s], rtol=1e-4, atol=1e-5)


# ----------------------------------------------------------------- layer norm
def test_layer_norm_against_float64_definition():
    g = torch.Generator().manual_seed(31)
    x = torch.randn(5, 7, 24, generator=g) * 3 + 1
    w, b = torch.randn(24, generator=g), torch.randn(24, generator=g)
    xd = x.double()
    want = (xd - xd.mean(-1, keepdim=True)) / torch.sqrt(xd.var(-1, unbiased=False, keepdim=True) + 1e-5) * w.double() + b.double()
    assert torch.allclose(torch_ref.layer_norm_rows(x, w, b).double(), want, rtol=1e-5, atol=1e-5)
    # known answers: a constant row normalises to the bias; [0,1] -> -1,+1 up to eps
    assert torch.equal(torch_ref.layer_norm_rows(torch.full((1, 8), 3.0), torch.ones(8), torch.full((8,), 0.25)), torch.full((1, 8), 0.25))
    y = torch_ref.layer_norm_rows(torch.tensor([[0.0, 1.0]]), None, None, eps=0.0)
    assert torch.allclose(y, torch.tensor([[-1.0, 1.0]]))


def test_layer_norm_cf_is_permute_norm_permute():
    g = torch.Generator().manual_seed(32)
    x = torch.randn(2, 6, 3, 5, generator=g)
    w, b = torch.randn(6, generator=g), torch.randn(6, generator=g)
    cl = torch_ref.layer_norm_cf(x, w, b, out_channel_last=True)
    cf = torch_ref.layer_norm_cf(x, w, b, out_channel_last=False)
    assert cl.shape == (2, 3, 5, 6) and cf.shape == x.shape
    assert torch.equal(cl.permute(0, 3, 1, 2), cf)
    for h in range(3):
        for wi in range(5):
            assert torch.allclose(cl[1, h, wi], torch_ref.layer_norm_rows(x[1, :, h, wi][None], w, b)[0], atol=1e-6)


# ------------------------------------------------------------- depthwise conv
def test_dwconv_against_brute_force():
    g = torch.Generator().manual_seed(33)
    B, D, H, W = 2, 3, 4, 5
    x, w, b = torch.randn(B, D, H, W, generator=g), torch.randn(D, 1, 3, 3, generator=g), torch.randn(D, generator=g)
    want = torch.zeros(B, D, H, W, dtype=torch.float64)
    for bi in range(B):
        for d in range(D):
            for h in range(H):
                for wi in range(W):
                    acc = float(b[d])
                    for kh in range(3):
                        for kw in range(3):
                            hh, ww = h + kh - 1, wi + kw - 1
                            if 0 <= hh < H and 0 <= ww < W:
                                acc += float(w[d, 0, kh, kw]) * float(x[bi, d, hh, ww])
                    want[bi, d, h, wi] = acc / (1.0 + math.exp(-acc))
    got = torch_ref.dwconv3x3_silu(x, w, b)
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-6)
    got_cl = torch_ref.dwconv3x3_silu(x.permute(0, 2, 3, 1).contiguous(), w, b, in_channel_last=True)
    assert torch.allclose(got_cl, got, rtol=1e-6, atol=1e-6)
    # identity kernel (centre tap 1) without SiLU returns the input
    ident = torch.zeros(D, 1, 3, 3); ident[:, 0, 1, 1] = 1.0
    assert torch.equal(torch_ref.dwconv3x3_silu(x, ident, None, apply_silu=False), x)


def test_selective_scan_gradient_oracle_against_finite_differences():
    """The float64 restatement used as gradient oracle: equal to the fp32 one on the forward, and its autograd
    gradients equal to central finite differences (torch.autograd.gradcheck) for every input."""
    g = torch.Generator().manual_seed(77)
    batch, dim, G, N, L = 1, 4, 2, 3, 6
    u = torch.randn(batch, dim, L, generator=g, dtype=torch.float64)
    delta = 0.5 * torch.rand(batch, 2, L, generator=g, dtype=torch.float64)          # two channels per delta row
    A = -0.5 * torch.rand(dim, N, generator=g, dtype=torch.float64)
    Bm = torch.randn(batch, G, N, L, generator=g, dtype=torch.float64)
    Cm = torch.randn(batch, G, N, L, generator=g, dtype=torch.float64)
    D = torch.randn(dim, generator=g, dtype=torch.float64)
    bias = 0.5 * torch.rand(2, generator=g, dtype=torch.float64)
    for softplus in (True, False):
        y64 = torch_ref.selective_scan_f64(u, delta, A, Bm, Cm, D, bias, softplus)
        y32 = torch_ref.selective_scan(u.float(), delta.float(), A.float(), Bm.float(), Cm.float(), D.float(), bias.float(), softplus)
        assert torch.allclose(y64.float(), y32, rtol=1e-5, atol=1e-5)
        leaves = [t.clone().requires_grad_(True) for t in (u, delta, A, Bm, Cm, D, bias)]
        assert torch.autograd.gradcheck(lambda *a: torch_ref.selective_scan_f64(*a, delta_softplus=softplus), leaves,
                                        eps=1e-6, atol=1e-6, rtol=1e-5)
        dout = torch.randn(y64.shape, generator=g, dtype=torch.float64)
        grads = torch_ref.selective_scan_grads(u, delta, A, Bm, Cm, D, bias, dout, softplus)
        want = torch.autograd.grad((torch_ref.selective_scan_f64(*leaves, delta_softplus=softplus) * dout).sum(), leaves)
        for a, b in zip(grads, want):
            assert torch.equal(a, b)
