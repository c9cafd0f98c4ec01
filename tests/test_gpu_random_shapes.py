"""Seeded random shapes for the kernels whose variant is chosen by shape and alignment: each family is run on a few dozen
shapes per seed against torch's own operators (fp32) or the CPU oracle, so that planner corner cases -- a last lane group
with fewer channels, a workgroup with fewer threads than positions, tiles that end inside a row or an image -- are met
without being listed one by one."""
import random

import pytest
import torch
import torch.nn.functional as F

import vmamba_amd as va
from oracle import ss2d_oracle as orc
from oracle import torch_ref
from vmamba_amd.conv import dwconv3x3_silu_hip
from vmamba_amd.core import dt_proj_hip
from vmamba_amd.csm import transpose_bcl_hip
from vmamba_amd.norm import add_layer_norm_hip, layer_norm_cf_hip, layer_norm_hip

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SEEDS = [11, 12, 13]


@pytest.mark.parametrize("seed", SEEDS)
def test_random_channel_first_layer_norm(seed):
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    for _ in range(40):
        B, C = rnd.randint(1, 5), rnd.choice([7, 8, 16, 24, 36, 40, 64, 96, 104, 192, 200, 384, 768, 1000])
        H, W = rnd.randint(1, 30), rnd.randint(1, 30)
        if C * H * W > 400000:
            H = W = 7
        in_dt = rnd.choice([torch.float32, torch.float32, torch.bfloat16])
        x = (torch.randn(B, C, H, W, device=DEV) * 2 + 0.5).to(in_dt)
        w, b = torch.randn(C, device=DEV).to(in_dt), torch.randn(C, device=DEV).to(in_dt)
        for out_cl in (False, True):
            out_dt = rnd.choice([in_dt, torch.bfloat16])
            print("CASE random ln-cf", seed, B, C, H, W, in_dt, out_dt, out_cl, flush=True)
            got = layer_norm_cf_hip(x, w, b, 1e-5, out_channel_last=out_cl, out_dtype=out_dt)
            want = F.layer_norm(x.float().permute(0, 2, 3, 1), (C,), w.float(), b.float(), 1e-5)
            want = want if out_cl else want.permute(0, 3, 1, 2)
            tol = 1e-4 if out_dt == torch.float32 else 2e-2
            assert torch.allclose(got.float(), want, rtol=tol, atol=tol), (B, C, H, W, in_dt, out_dt, out_cl)


@pytest.mark.parametrize("seed", SEEDS)
def test_random_row_layer_norm(seed):
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    for _ in range(40):
        rows, C = rnd.randint(1, 3000), rnd.choice([8, 48, 96, 97, 192, 200, 384, 768, 1000, 1024])
        in_dt, w_dt, out_dt = rnd.choice([(torch.float32,) * 3, (torch.bfloat16,) * 3, (torch.float32, torch.bfloat16, torch.bfloat16),
                                          (torch.float16,) * 3])
        print("CASE random ln-rows", seed, rows, C, in_dt, w_dt, out_dt, flush=True)
        x = torch.randn(rows, C, device=DEV).to(in_dt)
        w, b = torch.randn(C, device=DEV).to(w_dt), torch.randn(C, device=DEV).to(w_dt)
        tol = 1e-4 if out_dt == torch.float32 else 2e-2
        got = layer_norm_hip(x, w, b, out_dtype=out_dt)
        assert torch.allclose(got.float(), F.layer_norm(x.float(), (C,), w.float(), b.float(), 1e-5), rtol=tol, atol=tol), (rows, C)
        if C % 8 == 0 and in_dt == torch.bfloat16:
            r = torch.randn(rows, C, device=DEV).bfloat16()
            s, n = add_layer_norm_hip(x, r, w, b)
            sw = (x.float() + r.float()).bfloat16()
            assert torch.equal(s, sw), (rows, C)
            assert torch.allclose(n.float(), F.layer_norm(sw.float(), (C,), w.float(), b.float(), 1e-5), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("seed", SEEDS)
def test_random_depthwise_conv(seed):
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    for _ in range(40):
        D = rnd.choice([8, 16, 32, 40, 64, 96, 128, 192, 256, 384, 768])
        H, W, B = rnd.randint(1, 60), rnd.choice([1, 2, 3, 4, 7, 8, 12, 14, 16, 20, 28, 30, 56, 57, 64, 100, 120, 121, 128, 130, 136,
                                                  160, 192, 200, 256, 320]), rnd.randint(1, 3)
        if B * D * H * W > 3_000_000:
            H = max(1, 3_000_000 // (B * D * W))
        dt = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
        cl, has_bias, silu = rnd.random() < 0.8, rnd.random() < 0.5, rnd.random() < 0.7
        print("CASE random dwconv", seed, B, D, H, W, dt, cl, has_bias, silu, flush=True)
        x, w = torch.randn(B, D, H, W, device=DEV).to(dt), (torch.randn(D, 1, 3, 3, device=DEV) * 0.3).to(dt)
        b = torch.randn(D, device=DEV).to(dt) if has_bias else None
        got = dwconv3x3_silu_hip(x.permute(0, 2, 3, 1).contiguous() if cl else x, w, b, cl, silu)
        want = F.conv2d(x.float(), w.float(), None if b is None else b.float(), padding=1, groups=D).to(dt)   # rounded as stored ...
        if silu:
            want = F.silu(want.float()).to(dt)                                                                 # ... then SiLU
        tol = {torch.bfloat16: 2 ** -6, torch.float16: 2 ** -9, torch.float32: 1e-5}[dt]
        assert torch.allclose(got.float(), want.float(), rtol=tol, atol=tol), (B, D, H, W, dt, cl, has_bias, silu)


@pytest.mark.parametrize("seed", SEEDS)
def test_random_transpose_dt_proj_and_flex_round_trips(seed):
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    for _ in range(40):
        B, R, S = rnd.randint(1, 3), rnd.choice([7, 8, 16, 24, 64, 96, 100, 130, 256]), rnd.choice([8, 16, 33, 49, 64, 196, 200, 3136])
        for dt in (torch.bfloat16, torch.float32):
            t = torch.randn(B, R, S, device=DEV).to(dt)
            assert torch.equal(transpose_bcl_hip(t), t.transpose(1, 2).contiguous()), (B, R, S, dt)
        K, D, Rk = rnd.choice([1, 4]), rnd.choice([8, 32, 96, 100, 192, 384, 768]), rnd.choice([1, 3, 6, 7, 12, 24, 48])
        N, dt = rnd.choice([8, 64, 72, 245, 588, 1000, 3136]), rnd.choice([torch.bfloat16, torch.float16])
        print("CASE random dt_proj", seed, K, D, Rk, N, dt, flush=True)
        x, Wt = torch.randn(K, Rk, N, device=DEV).to(dt), (torch.randn(K, D, Rk, device=DEV) * Rk ** -0.5).to(dt)
        tol = 2 ** -7 if dt == torch.bfloat16 else 2 ** -10
        assert torch.allclose(dt_proj_hip(x, Wt).float(), torch.bmm(Wt.float(), x.float()), rtol=tol, atol=4 * tol), (K, D, Rk, N, dt)
        Bc, C, H, W = rnd.randint(1, 3), rnd.choice([3, 5, 8, 16, 96]), rnd.randint(1, 15), rnd.randint(1, 15)
        icf, ocf, obo, scans = rnd.random() < 0.5, rnd.random() < 0.5, rnd.random() < 0.3, rnd.choice([0, 1, 2])
        shape = ((Bc, 4, C, H, W) if obo else (Bc, C, H, W)) if icf else ((Bc, H, W, 4, C) if obo else (Bc, H, W, C))
        xi = torch.randint(-8, 8, shape, device=DEV).to(rnd.choice([torch.float32, torch.bfloat16]))
        y = va.cross_scan_fn(xi, icf, ocf, obo, scans)
        assert torch.equal(y.cpu().reshape(-1), torch_ref.cross_scan_flex(xi.cpu(), icf, ocf, obo, scans).reshape(-1)), (shape, icf, ocf, obo, scans)
        back = va.cross_merge_fn(y.view(Bc, 4, C, H, W) if ocf else y.view(Bc, H, W, 4, C), icf, ocf, obo, scans)
        assert torch.equal(back.reshape(xi.shape).float(), xi.float() * (1 if obo else 4)), (shape, icf, ocf, obo, scans)


def _scan_inputs(gen, batch, dim, G, N, L, dtype):
    u = torch.randn(batch, dim, L, generator=gen).to(dtype)
    delta = (torch.randn(batch, dim, L, generator=gen) * 0.5).to(dtype)
    A = -(torch.rand(dim, N, generator=gen) + 0.5)
    Bm, Cm = torch.randn(batch, G, N, L, generator=gen).to(dtype), torch.randn(batch, G, N, L, generator=gen).to(dtype)
    return u, delta, A, Bm, Cm, torch.randn(dim, generator=gen), torch.randn(dim, generator=gen) - 2.0


@pytest.mark.parametrize("seed", SEEDS)
def test_random_selective_scan(seed):
    rnd = random.Random(seed)
    gen = torch.Generator().manual_seed(seed)
    for _ in range(30):
        L = rnd.choice([7, 49, 49, 64, 100, 196, 196, 513, 1024, 2049, 3136, 4100])
        G, dpg, batch = rnd.choice([1, 2, 4]), rnd.choice([1, 2, 3, 4, 8, 16, 24, 32]), rnd.randint(1, 5)
        N = 1 if L > 2048 else rnd.choice([1, 1, 1, 2, 4, 16])
        dtype = rnd.choice([torch.float32, torch.bfloat16, torch.float16])
        print("CASE random scan", seed, batch, G * dpg, G, N, L, dtype, flush=True)
        u, delta, A, Bm, Cm, D, bias = _scan_inputs(gen, batch, G * dpg, G, N, L, dtype)
        want = orc.selective_scan(u, delta, A, Bm, Cm, D, bias, True, out_float=True)
        dev = lambda t: t.to(DEV)
        got = va.selective_scan_fn(dev(u), dev(delta), dev(A), dev(Bm), dev(Cm), dev(D), dev(bias), True)
        assert torch.allclose(got.cpu(), want, rtol=1e-3, atol=2e-4), (batch, G * dpg, G, N, L, dtype, (got.cpu() - want).abs().max().item())


@pytest.mark.parametrize("seed", SEEDS)
def test_random_cross_scan_merge_and_one_by_one(seed):
    """Plain CrossScan / CrossMerge and the one-by-one CrossScan (contiguous and through output strides), bit for bit
    against the torch restatement; some inputs start one element off the allocation's alignment."""
    from vmamba_amd.csm import cross_scan_1b1_hip
    rnd = random.Random(seed)
    for _ in range(60):
        B, C = rnd.randint(1, 4), rnd.choice([1, 2, 3, 4, 5, 8, 13, 26, 50, 96])
        H, W = rnd.randint(1, 33), rnd.randint(1, 33)
        if rnd.random() < 0.3:
            H = W = rnd.choice([7, 14, 28, 56])
        if rnd.random() < 0.1:
            H, W, C = rnd.choice([(130, 70), (64, 128), (100, 100)]) + (rnd.choice([1, 2]),)
        if C * H * W > 200000:
            C = 4
        dt = rnd.choice([torch.float32, torch.bfloat16, torch.float16, torch.uint8])
        print("CASE random cross", seed, B, C, H, W, dt, flush=True)
        x = torch.randint(0, 16, (B, C, H, W)).to(dt).to(DEV)
        if rnd.random() < 0.3 and dt != torch.uint8:
            buf = torch.zeros(x.numel() + 1, dtype=dt, device=DEV)
            buf[1:] = x.flatten()
            x = buf[1:].view(B, C, H, W)
        want = torch_ref.cross_scan(x.cpu())
        assert torch.equal(va.cross_scan_fn(x).cpu().view(want.shape), want), (B, C, H, W, dt)
        if dt in (torch.float32, torch.bfloat16):
            ys = torch.randint(-8, 8, (B, 4, C, H, W)).to(dt).to(DEV)
            wm = torch_ref.cross_merge(ys.cpu())
            assert torch.equal(va.cross_merge_fn(ys).cpu().view(wm.shape), wm), (B, C, H, W, dt)
        x4 = torch.randint(0, 16, (B, 4, C, H, W)).to(dt).to(DEV)
        w1 = torch_ref.cross_scan_1b1(x4.cpu())
        assert torch.equal(va.cross_scan_fn(x4, one_by_one=True).cpu().view(w1.shape), w1), (B, C, H, W, dt)
        buf = torch.zeros((4, C, B, H * W), dtype=dt, device=DEV)
        cross_scan_1b1_hip(x4, out=buf.permute(2, 0, 1, 3))
        assert torch.equal(buf.permute(2, 0, 1, 3).cpu().reshape(w1.shape), w1), (B, C, H, W, dt)


@pytest.mark.parametrize("seed", SEEDS)
def test_random_fused_core(seed):
    """The fused core on random map sizes (square and not, odd and even), batches and channel counts against the CPU
    oracle's composition of the three operators."""
    from test_gpu_core import make_core_inputs, oracle_core, run_core
    rnd = random.Random(seed)
    for it in range(20):
        H = rnd.choice([7, 14, 28, 56, 3, 5, 8, 12, 19, 20, 24, 32, 40])
        W = H if rnd.random() < 0.6 else rnd.choice([3, 4, 6, 9, 16, 28])
        B, D = rnd.randint(1, 50), rnd.choice([1, 2, 3, 4, 5, 8])
        if B * D * H * W > 200000:
            B = max(1, 200000 // (D * H * W))
        dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
        print("CASE random core", seed, B, D, H, W, dtype, flush=True)
        inp = make_core_inputs(100 * seed + it, B, D, H, W, dtype)
        assert torch.allclose(run_core(*inp), oracle_core(*inp), rtol=1e-3, atol=4e-4), (B, D, H, W, dtype)


@pytest.mark.parametrize("seed", SEEDS)
def test_random_models(seed):
    """Whole models of random widths, depths, state counts, layouts and image sizes (sides that are not multiples of 32
    included) against the all-torch CPU model holding the same weights."""
    from oracle.ss2d_core_ref import RefSS2D, TorchLayers
    from vmamba_amd.vssm import VSSM
    rnd = random.Random(seed)
    for it in range(4):
        d0 = rnd.choice([16, 32, 48, 96])
        cfg = dict(dims=(d0, 2 * d0, 4 * d0, 8 * d0), depths=tuple(rnd.choice([1, 1, 2]) for _ in range(4)),
                   d_state=rnd.choice([1, 1, 1, 2, 4]), ssm_ratio=rnd.choice([1.0, 1.0, 2.0]), num_classes=50)
        H = 32 * rnd.randint(1, 7) if rnd.random() < 0.6 else rnd.randint(20, 230)
        W = H if rnd.random() < 0.6 else rnd.randint(20, 230)
        B, cf = rnd.randint(1, 4), rnd.random() < 0.4
        dtype = rnd.choice([torch.float32, torch.bfloat16, torch.bfloat16])
        print("CASE random model", seed, cfg, H, W, B, cf, dtype, flush=True)
        torch.manual_seed(100 * seed + it)
        ref = VSSM(**cfg, channel_first=cf, ss2d_cls=RefSS2D, layers=TorchLayers).eval()
        if dtype != torch.float32:
            ref = ref.bfloat16().float()
        hip = VSSM(**cfg, channel_first=cf).eval()
        hip.load_state_dict(ref.state_dict())
        hip = hip.to(dtype).to(DEV)
        x = torch.randn(B, 3, H, W, generator=torch.Generator().manual_seed(it)).to(dtype)
        with torch.no_grad():
            want, got = ref(x.float()), hip(x.to(DEV)).float().cpu()
        tol = 2e-3 if dtype == torch.float32 else 3e-2
        assert (got - want).abs().max().item() <= tol * want.abs().max().item(), (cfg, H, W, B, cf, dtype)
