"""Writes the golden vectors under tests/golden/ from first principles.

Nothing here imports the oracle, the package or the reference: the cross-scan
vectors are the hand-checkable 4x4 and 2x3 cases (the 4x4 one is the case the
reference prints at classification/models/vmamba_checks.py:310-313), spelled
out literally; the selective-scan vectors come from a float64 pure-Python
loop over the textbook recurrence
    h_t = exp(dl_t*A) h_{t-1} + dl_t*B_t*u_t,  y_t = sum_n C_t h_t + D u_t
with inputs drawn from Python's own Mersenne twister, so a reader can rerun
this file anywhere and get the same JSON byte for byte.

Run:  python tests/golden/make_golden.py
"""
import json
import math
import os
import random

HERE = os.path.dirname(os.path.abspath(__file__))


def cross_scan_kats():
    kats = []
    # 4x4 arange map: row-major, column-major and their reversals.
    x = list(range(16))
    d0 = list(range(16))
    d1 = [0, 4, 8, 12, 1, 5, 9, 13, 2, 6, 10, 14, 3, 7, 11, 15]
    kats.append(dict(H=4, W=4, x=x, y=[d0, d1, d0[::-1], d1[::-1]],
                     merged=[4 * v for v in x]))
    # 2x3 map [[0,1,2],[3,4,5]]: column-major order reads 0,3,1,4,2,5.
    x = [0, 1, 2, 3, 4, 5]
    d0 = [0, 1, 2, 3, 4, 5]
    d1 = [0, 3, 1, 4, 2, 5]
    kats.append(dict(H=2, W=3, x=x, y=[d0, d1, d0[::-1], d1[::-1]],
                     merged=[4 * v for v in x]))
    # 3x1 and 1x3 strips: transposition is the identity on the flat order.
    for H, W in ((3, 1), (1, 3)):
        x = [7, 8, 9]
        kats.append(dict(H=H, W=W, x=x, y=[x, x, x[::-1], x[::-1]], merged=[4 * v for v in x]))
    return kats


def cross_merge_kat():
    # 2x2 maps with distinct values per direction; worked by hand:
    # out[h,w] = (y0[r] + y2[3-r]) + (y1[t] + y3[3-t]),  r=2h+w, t=2w+h
    y0, y1, y2, y3 = [1, 2, 3, 4], [10, 20, 30, 40], [100, 200, 300, 400], [1000, 2000, 3000, 4000]
    out = []
    for h in range(2):
        for w in range(2):
            r, t = 2 * h + w, 2 * w + h
            out.append((y0[r] + y2[3 - r]) + (y1[t] + y3[3 - t]))
    assert out == [4411, 2332, 3223, 1144]  # e.g. (h,w)=(0,1): r=1,t=2 -> (2+300)+(30+2000)
    return dict(H=2, W=2, ys=[y0, y1, y2, y3], out=out)


def softplus(v):
    return v if v > 20.0 else math.log1p(math.exp(v))


def scan_case(rng, batch, dim, G, N, L, delta_dim, has_D, has_bias, use_softplus):
    g = lambda: rng.gauss(0.0, 1.0)
    # values snapped to multiples of 1/64 (exact in bf16 for |v|<4) so the same JSON feeds fp32
    # and bf16 tests without an input rounding step
    snap = lambda v: round(max(-3.9, min(3.9, v)) * 64.0) / 64.0
    u = [[[snap(g()) for _ in range(L)] for _ in range(dim)] for _ in range(batch)]
    delta = [[[snap(0.5 * rng.random()) if not use_softplus else snap(g() - 2.0) for _ in range(L)]
              for _ in range(delta_dim)] for _ in range(batch)]
    A = [[-snap(0.0625 + 0.5 * rng.random()) for _ in range(N)] for _ in range(dim)]
    Bm = [[[[snap(g()) for _ in range(L)] for _ in range(N)] for _ in range(G)] for _ in range(batch)]
    Cm = [[[[snap(g()) for _ in range(L)] for _ in range(N)] for _ in range(G)] for _ in range(batch)]
    D = [snap(g()) for _ in range(dim)] if has_D else None
    bias = [snap(0.5 * rng.random()) for _ in range(delta_dim)] if has_bias else None
    out = [[[0.0] * L for _ in range(dim)] for _ in range(batch)]
    last = [[[0.0] * N for _ in range(dim)] for _ in range(batch)]
    for b in range(batch):
        for d in range(dim):
            grp, dg = d // (dim // G), d // (dim // delta_dim)
            h = [0.0] * N
            for t in range(L):
                dl = delta[b][dg][t] + (bias[dg] if bias else 0.0)
                if use_softplus:
                    dl = softplus(dl)
                y = 0.0
                for n in range(N):
                    h[n] = math.exp(dl * A[d][n]) * h[n] + dl * Bm[b][grp][n][t] * u[b][d][t]
                    y += h[n] * Cm[b][grp][n][t]
                out[b][d][t] = y + (D[d] * u[b][d][t] if D else 0.0)
            last[b][d] = h
    return dict(batch=batch, dim=dim, G=G, N=N, L=L, delta_dim=delta_dim, delta_softplus=use_softplus,
                u=u, delta=delta, A=A, B=Bm, C=Cm, D=D, delta_bias=bias, out=out, last_state=last)


def main():
    with open(os.path.join(HERE, "cross_scan_kat.json"), "w") as f:
        json.dump(dict(scan=cross_scan_kats(), merge=cross_merge_kat()), f)
    rng = random.Random(20240607)
    cases = [
        scan_case(rng, 2, 4, 4, 1, 7, 4, True, True, True),      # SS2D-like: K=4 groups, N=1
        scan_case(rng, 1, 8, 4, 1, 49, 8, True, True, True),     # 7x7 map length
        scan_case(rng, 2, 6, 2, 4, 33, 6, True, False, False),   # N=4, 2 groups, no bias/softplus
        scan_case(rng, 1, 4, 1, 16, 130, 2, False, True, True),  # N=16, delta-group broadcast, no D
        scan_case(rng, 1, 2, 2, 2, 1, 2, True, True, True),      # L=1
    ]
    with open(os.path.join(HERE, "selective_scan_f64.json"), "w") as f:
        json.dump(cases, f)
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
