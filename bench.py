#!/usr/bin/env python3
"""Benchmark of the SS2D inference hot path on one MI355X.

Step     = one forward of a random-init VMamba-T (vmamba_tiny_s1l8 shape) on a synthetic
           (128, 3, 224, 224) bf16 batch already resident in HBM; the reference's throughput
           protocol (classification/main.py:346-363) with explicit warm-up / step counts.
value    = images per second of that forward.
roofline = the dominant kernel of that forward: the fused SS2D core (CrossScan + selective scan + CrossMerge in
           one launch) at stage-1 shape (benchmark config 1: B=128, D=96, 56x56, K=4, N=1, bf16 in, fp32 out),
           timed with HIP events on the launch stream; achieved = algorithmic bytes / average launch time,
           peak = 8 TB/s.  scan_roofline = the same for the stand-alone selective-scan kernel behind
           selective_scan_fn (the "scan GB/s" of the metric), which the three-operator path still uses.
cpu_baseline = the torch-on-CPU restatement of the reference path (oracle/) run through the same
           model on a bounded sample, on this box's host cores (img/s, the metric's unit).
cpu_baseline_op / parity = benchmark config 0 (the reference's CPU-runnable SS2D operator: fp32, x (2,96,56,56) ->
           CrossScan -> selective scan -> CrossMerge, seed 0) timed on the host cores with the torch restatement and
           with the C oracle, beside the GPU's time on the same bits, and the GPU's error against that CPU result.
Extra keys: ms_per_step_eager / ms_per_step_one_graph / ms_per_step_concurrent (the three launch modes of the same
           forward; `value` is the fastest validated one and `config.launch` names it), config4 (4 x 1024^2 forward),
           fp32 (the same batch-128 forward at the reference harness's precision).

One JSON line is printed on stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FP32_VECTOR_PEAK_TFLOPS = 157.3
PROFILE_SUMMARY = os.path.join(ROOT, "profiles", "ss2d_core_kernels_vmamba_t_bs128.txt")
COUNTER_SUMMARY = os.path.join(ROOT, "profiles", "ss2d_core_sq_counters_vmamba_t_bs128.txt")


def measured_issue(kernel_tag):
    """Vector-ALU occupancy of a kernel from the committed rocprofv3 SQ-counter summary: the line
        ISSUE <tag> valu_busy=<4 * SQ_ACTIVE_INST_VALU / (SIMDs * duration in cycles)> valu_per_unit=<SQ_INSTS_VALU * 64 / units>
    Returns (dict, "file: line") or (None, reason)."""
    try:
        with open(COUNTER_SUMMARY) as f:
            for n, line in enumerate(f, 1):
                parts = line.split()
                if len(parts) >= 3 and parts[0] == "ISSUE" and parts[1] == kernel_tag:
                    return {k: float(v) for k, v in (p.split("=", 1) for p in parts[2:])}, f"{os.path.relpath(COUNTER_SUMMARY, ROOT)}:{n}"
    except (OSError, ValueError) as e:
        return None, f"{type(e).__name__}: {e}"
    return None, f"no ISSUE line for {kernel_tag} in {os.path.relpath(COUNTER_SUMMARY, ROOT)}"


def measured_traffic(kernel_tag):
    """HBM bytes per launch of a kernel from the committed rocprofv3 counter summary.  Counters cannot be read from
    inside the timed process; the summary holds one line per kernel of the form
        TRAFFIC <tag> fetch_kib=<FETCH_SIZE per dispatch> write_kib=<WRITE_SIZE per dispatch> fetch_scale=<f> write_scale=<w>
    (the scales are what the same counters read for the 1 GiB calibration copy of `bench.py --kernels-only`).
    Returns (bytes, "file: line") or (None, reason)."""
    try:
        with open(PROFILE_SUMMARY) as f:
            for n, line in enumerate(f, 1):
                parts = line.split()
                if len(parts) >= 6 and parts[0] == "TRAFFIC" and parts[1] == kernel_tag:
                    kv = dict(p.split("=", 1) for p in parts[2:])
                    total = 1024.0 * (float(kv["fetch_kib"]) * float(kv["fetch_scale"]) + float(kv["write_kib"]) * float(kv["write_scale"]))
                    return total, f"{os.path.relpath(PROFILE_SUMMARY, ROOT)}:{n}"
    except (OSError, KeyError, ValueError) as e:
        return None, f"{type(e).__name__}: {e}"
    return None, f"no TRAFFIC line for {kernel_tag} in {os.path.relpath(PROFILE_SUMMARY, ROOT)}"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def scan_bytes(B, KD, L, N, K, s_in, s_out):
    """Algorithmic bytes of one scan launch: u, delta in; out; B, C rows; A, D, bias."""
    return B * KD * L * (2 * s_in + s_out) + 2 * B * K * N * L * s_in + 4 * KD * (N + 2)


def core_bytes(B, D, L, s_in, K=4):
    """Algorithmic bytes of one fused-core launch: x in, the K delta rows in, merged fp32 y out; B, C rows; A, D, bias."""
    return B * D * L * (s_in + K * s_in + 4) + 2 * B * K * L * s_in + 4 * K * D * 3


def time_op(fn, reps, warm=None):
    import torch
    # as many untimed launches as timed ones: the first few dozen launches of a kernel over freshly allocated
    # tensors read ~5 % slower than its steady state
    for _ in range(reps if warm is None else warm):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps * 1e-3      # seconds per launch


def kernel_lines(reps):
    """Per-kernel timings of the SS2D core at the four VMamba-T stage shapes (bs128, bf16 in) and at the
    benchmark config 3 / config 4 operator shapes."""
    import torch
    import vmamba_amd as va
    from vmamba_amd import oflex_ext
    from vmamba_amd.core import core_fits, dt_proj_hip, ss2d_core_hip
    from vmamba_amd.csms6s import scan_kernel_name
    ext = oflex_ext.load()
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(0)
    out = []
    shapes = dict(stage1=(128, 96, 56, 56, 1), stage2=(128, 192, 28, 28, 1), stage3=(128, 384, 14, 14, 1),
                  stage4=(128, 768, 7, 7, 1),
                  # benchmark config 3 (16 states, ssm_ratio 2) and the stage-1 shape of config 4 (1024^2 images, batch 4)
                  n16=(64, 192, 56, 56, 16), hires=(4, 96, 256, 256, 1))
    for name, (B, D, H, W, N) in shapes.items():
        K, L = 4, H * W
        x = torch.randn(B, D, H, W, device=dev, generator=g).bfloat16()
        delta = (torch.randn(B, K * D, L, device=dev, generator=g) * 0.5).bfloat16()
        Bm = torch.randn(B, K, N, L, device=dev, generator=g).bfloat16()
        Cm = torch.randn(B, K, N, L, device=dev, generator=g).bfloat16()
        A = -torch.arange(1, N + 1, device=dev, dtype=torch.float32).repeat(K * D, 1)
        Dv = torch.ones(K * D, device=dev)
        bias = torch.full((K * D,), -3.0, device=dev)
        xs = va.cross_scan_fn(x)
        u = xs.view(B, K * D, L)
        ys = va.selective_scan_fn(u, delta, A, Bm, Cm, Dv, bias, True)
        ys5 = ys.view(B, K, D, H, W)
        E = B * D * L
        t_cs = time_op(lambda: va.cross_scan_fn(x), reps)
        t_sc = time_op(lambda: va.selective_scan_fn(u, delta, A, Bm, Cm, Dv, bias, True), reps)
        # the same scan through the reference's extension interface, which always returns the chunk states too
        # (out, x = selective_scan_cuda_oflex.fwd(...), classification/models/csms6s.py:81)
        t_ext = time_op(lambda: ext.fwd(u, delta, A, Bm, Cm, Dv, bias, True, 1, True), reps)
        scan_kernel = scan_kernel_name(u, delta, A, Bm, Cm, ys, torch.empty(B, K * D, (L + 2047) // 2048, 2 * N, device=dev))
        t_cm = time_op(lambda: va.cross_merge_fn(ys5), reps)
        b_cs, b_sc, b_cm = 5 * E * 2, scan_bytes(B, K * D, L, N, K, 2, 4), 5 * E * 4
        fused = {}
        if N == 1 and core_fits(H, W, x.dtype):
            # the same work as ONE kernel; delta and B / C direction-major, batch-innermost
            delta_k = delta.view(B, K, D, L).permute(1, 2, 0, 3).contiguous()
            B_k, C_k = Bm.view(B, K, L).permute(1, 0, 2).contiguous(), Cm.view(B, K, L).permute(1, 0, 2).contiguous()
            A1 = A.view(-1)
            t_f = time_op(lambda: ss2d_core_hip(x, delta_k, B_k, C_k, A1, Dv, bias, True), reps)
            b_f = core_bytes(B, D, L, 2)
            fused = dict(core_fused_us=t_f * 1e6, core_fused_GBs=b_f / t_f / 1e9, core_fused_bytes=b_f)
            # dt_proj (rank R = D/16 -> D, per direction) on the matrix cores, writing that delta layout
            R = max(D // 16, 1)
            dts = torch.randn(K, R, B * L, device=dev, generator=g).bfloat16()
            Wdt = (torch.randn(K, D, R, device=dev, generator=g) * R ** -0.5).bfloat16()
            t_dt = time_op(lambda: dt_proj_hip(dts, Wdt), reps)
            b_dt = 2 * K * (D + R) * B * L + 2 * K * D * R
            fused.update(dt_proj_us=t_dt * 1e6, dt_proj_GBs=b_dt / t_dt / 1e9)
            del delta_k, B_k, C_k, dts, Wdt
        if N == 1 and name != "hires":
            # the two ops around the core in a block: depthwise conv + SiLU on the channel-last in_proj output, writing the
            # channel-first map (bytes: the map in and out once), and out_norm on the core's fp32 channel-first output,
            # writing the channel-last 16-bit activation (bytes: 4 in + 2 out per element)
            from vmamba_amd.conv import dwconv3x3_silu_hip
            from vmamba_amd.norm import layer_norm_cf_hip
            x_cl = x.permute(0, 2, 3, 1).contiguous()
            wconv = (torch.randn(D, 1, 3, 3, device=dev, generator=g) * 0.3).bfloat16()
            t_dw = time_op(lambda: dwconv3x3_silu_hip(x_cl, wconv, None, in_channel_last=True), reps)
            ycf = torch.randn(B, D, H, W, device=dev, generator=g)
            gam, bet = torch.ones(D, device=dev).bfloat16(), torch.zeros(D, device=dev).bfloat16()
            t_ln = time_op(lambda: layer_norm_cf_hip(ycf, gam, bet, 1e-5, out_channel_last=True, out_dtype=torch.bfloat16), reps)
            fused.update(dwconv_us=t_dw * 1e6, dwconv_GBs=E * 4 / t_dw / 1e9, layer_norm_cf_us=t_ln * 1e6,
                         layer_norm_cf_GBs=E * 6 / t_ln / 1e9)
            del x_cl, ycf, wconv
        if N > 1:
            # several states per channel: the scan is bound by vector-ALU issue, not by HBM -- its VALU occupancy and
            # instruction count per (position, state) come from the committed SQ-counter summary -- and CrossScan is
            # folded into it (the kernel reads x and its transpose through the routes): core_n = that scan + CrossMerge
            from vmamba_amd.csms6s import selective_scan_from_map
            issue, issue_src = measured_issue("scan_chan_kernel@config3")
            t_n = time_op(lambda: va.cross_merge_fn(selective_scan_from_map(x, delta, A, Bm, Cm, Dv, bias, True, True).view(B, K, D, H, W)), reps)
            # the same three steps as separate operators, also timed as one chain (a kernel that follows another kind of
            # kernel starts on a cold cache, which the per-kernel lines above do not see)
            t_3 = time_op(lambda: va.cross_merge_fn(va.selective_scan_fn(va.cross_scan_fn(x).view(B, K * D, L), delta, A, Bm, Cm, Dv, bias,
                                                                         True).view(B, K, D, H, W)), reps)
            flops = 9.0 * B * K * D * L * N + B * K * D * L          # the reference's own count, csms6s.py:139-160
            fused.update(scan_TFLOPs=flops / t_sc / 1e12, issue_frac=(issue or {}).get("valu_busy"),
                         valu_per_position_state=(issue or {}).get("valu_per_unit"), issue_source=issue_src,
                         core_n_us=t_n * 1e6, core_n_GBs=(b_cs + b_sc + b_cm) / t_n / 1e9,
                         three_operators_us=t_3 * 1e6)
        if name in ("stage1", "stage2"):
            # block-level kernels of the narrow stages (harness side): fused LayerNorm + MLP + residual, and at width 96
            # the two projections with their LayerNorm / residual.  Bytes: activations in and out once (+ residual).
            from vmamba_amd.mlp import mlp_fused_hip
            from vmamba_amd.linear import linear_cf_ln_fusable, linear_cf_ln_hip, linear_cl_hip, linear_fusable
            M = B * L
            xa = torch.randn(M, D, device=dev, generator=g).bfloat16()
            w1 = (torch.randn(4 * D, D, device=dev, generator=g) * D ** -0.5).bfloat16()
            w2 = (torch.randn(D, 4 * D, device=dev, generator=g) * (4 * D) ** -0.5).bfloat16()
            b1, b2 = torch.zeros(4 * D, device=dev).bfloat16(), torch.zeros(D, device=dev).bfloat16()
            gam, bet = torch.ones(D, device=dev).bfloat16(), torch.zeros(D, device=dev).bfloat16()
            t_m = time_op(lambda: mlp_fused_hip(xa, w1, b1, w2, b2, xa, gam, bet, 1e-5), reps)
            fused.update(mlp_fused_us=t_m * 1e6, mlp_fused_TFLOPs=16.0 * M * D * D / t_m / 1e12, mlp_fused_GBs=3 * M * D * 2 / t_m / 1e9)
            wp = (torch.randn(D, D, device=dev, generator=g) * D ** -0.5).bfloat16()
            if linear_fusable(xa, wp):
                t_i = time_op(lambda: linear_cl_hip(xa, wp, None, None, gam, bet, 1e-5), reps)
                t_o = time_op(lambda: linear_cl_hip(xa, wp, None, xa), reps)
                fused.update(ln_in_proj_us=t_i * 1e6, ln_in_proj_GBs=2 * M * D * 2 / t_i / 1e9,
                             out_proj_add_us=t_o * 1e6, out_proj_add_GBs=3 * M * D * 2 / t_o / 1e9)
                if linear_cf_ln_fusable(D, wp, H * W):
                    # out_norm + out_proj + residual straight from the core's fp32 channel-first map
                    ycf = torch.randn(B, D, H * W, device=dev, generator=g)
                    t_n = time_op(lambda: linear_cf_ln_hip(ycf, gam, bet, 1e-5, wp, None, xa), reps)
                    fused.update(norm_out_proj_add_us=t_n * 1e6, norm_out_proj_add_GBs=M * D * (4 + 2 + 2) / t_n / 1e9)
                    del ycf
            del xa, w1, w2, wp
            if name == "stage1":
                # the patch embedding's first layer (conv 3x3 stride 2 + LayerNorm + GELU in one kernel): the image
                # batch in, the (B, 112, 112, 48) activation out
                from vmamba_amd.stem import stem_conv_ln_gelu_hip
                img = torch.randn(B, 3, 4 * H, 4 * W, device=dev, generator=g).bfloat16()
                wc = (torch.randn(48, 3, 3, 3, device=dev, generator=g) * 0.2).bfloat16()
                v48 = torch.ones(48, device=dev).bfloat16()
                t_s = time_op(lambda: stem_conv_ln_gelu_hip(img, wc, v48, v48, v48, 1e-5), reps)
                b_s = img.numel() * 2 + B * (2 * H) * (2 * W) * 48 * 2
                fused.update(stem_us=t_s * 1e6, stem_GBs=b_s / t_s / 1e9)
                del img
        out.append(dict(shape=name, B=B, D=D, H=H, W=W, N=N,
                        cross_scan_us=t_cs * 1e6, cross_scan_GBs=b_cs / t_cs / 1e9,
                        scan_us=t_sc * 1e6, scan_GBs=b_sc / t_sc / 1e9, scan_kernel=scan_kernel,
                        ext_fwd_us=t_ext * 1e6, ext_fwd_GBs=b_sc / t_ext / 1e9, ext_fwd_over_fn=t_ext / t_sc,
                        cross_merge_us=t_cm * 1e6, cross_merge_GBs=b_cm / t_cm / 1e9,
                        core_GBs=(b_cs + b_sc + b_cm) / (t_cs + t_sc + t_cm) / 1e9,
                        scan_bytes=b_sc, **fused))
        if name in ("stage4", "hires"):
            # yardstick for the two kernels furthest below 0.6 of the HBM peak among the three operators: a plain elementwise
            # kernel (dst = src + 0 on 32-bit words) that moves the same number of bytes, half read, half written.  (Not
            # copy_: the runtime's copy kernel is what the profiler counters are calibrated on, at 1 GiB.)
            b_y = b_cs if name == "stage4" else b_sc
            src_y = torch.zeros(b_y // 8, dtype=torch.int32, device=dev)
            dst_y = torch.empty_like(src_y)
            t_y = time_op(lambda: torch.add(src_y, 0, out=dst_y), reps)
            key = "cross_scan" if name == "stage4" else "scan"
            out[-1].update({key + "_copy_us": t_y * 1e6, key + "_over_copy": (t_cs if name == "stage4" else t_sc) / t_y})
            del src_y, dst_y
        if name == "stage1":
            # the scan's backward at the same shape (fp32 dout, as the oflex forward hands back): algorithmic bytes =
            # u, delta, dout in; du, ddelta out; B, C in and fp32 dB, dC out once per (batch, direction)
            dout = torch.randn(B, K * D, L, device=dev, generator=g)
            t_b = time_op(lambda: va.selective_scan_bwd(u, delta, A, Bm, Cm, Dv, bias, dout, None, True, 1), max(reps // 4, 2), warm=2)
            b_b = B * K * D * L * (2 + 2 + 4 + 2 + 2) + B * K * N * L * (2 * 2 + 2 * 4)
            out[-1].update(scan_bwd_us=t_b * 1e6, scan_bwd_GBs=b_b / t_b / 1e9, scan_bwd_bytes=b_b)
            del dout
            # the other layouts / modes of the two operators (generic kernels), same shape; bytes = 5 E s as above
            flex = {}
            x_cl = x.permute(0, 2, 3, 1).contiguous()
            y_cl = ys5.permute(0, 3, 4, 1, 2).contiguous()
            for tag, (icf, ocf, scans) in dict(cl_cl_s0=(False, False, 0), cf_cl_s0=(True, False, 0),
                                               cl_cf_s0=(False, True, 0), cf_cf_s2=(True, True, 2)).items():
                xi, yi = (x if icf else x_cl), (ys5 if ocf else y_cl)
                t_s = time_op(lambda: va.cross_scan_fn(xi, icf, ocf, False, scans), reps)
                t_m = time_op(lambda: va.cross_merge_fn(yi, icf, ocf, False, scans), reps)
                flex[tag] = dict(scan_us=t_s * 1e6, scan_GBs=b_cs / t_s / 1e9, merge_us=t_m * 1e6, merge_GBs=b_cm / t_m / 1e9)
            out[-1]["flex_modes"] = flex
            del x_cl, y_cl
        log("kernels", out[-1])
        del x, delta, Bm, Cm, xs, u, ys, ys5
    return out


def odd_map_lines(reps):
    """SS2D.forward_core (projections + fused core + out_norm, inference) on maps whose sides the vector paths do not like,
    each beside a neighbouring map that they do: time per element and the ratio (57 x 58 is the reference's own check size,
    classification/models/csm_triton.py:524, 670)."""
    import torch
    from vmamba_amd.core import padded_map_size
    from vmamba_amd.ss2d import SS2D
    dev = "cuda:0"
    out = []
    for odd, aligned in (((48, 96, 57, 58), (48, 96, 56, 56)), ((8, 192, 75, 75), (8, 192, 72, 72)),
                         ((64, 384, 19, 19), (64, 384, 20, 20)), ((16, 96, 200, 334), (16, 96, 200, 336))):
        line = {}
        for tag, (B, D, H, W) in (("odd", odd), ("aligned", aligned)):
            torch.manual_seed(0)
            m = SS2D(d_model=D, d_state=1, ssm_ratio=1.0, channel_first=False).eval().bfloat16().to(dev)
            x = torch.randn(B, D, H, W, device=dev).bfloat16()
            t = time_op(lambda: m.forward_core(x), reps, warm=5)
            line[tag] = dict(shape=[B, D, H, W], us=round(t * 1e6, 1), ns_per_element=round(t * 1e9 / (B * D * H * W), 4))
            if tag == "odd":
                pad = padded_map_size(H, W, x.dtype)
                line["embedded_in"] = list(pad) if pad else None
            del m, x
        line["per_element_ratio"] = round(line["odd"]["ns_per_element"] / line["aligned"]["ns_per_element"], 3)
        out.append(line)
        log("odd_maps", line)
    return out


def host_cpu():
    """(threads to use, description).  The box gives a job a share of the host's cores and exports it as
    OMP_NUM_THREADS; more threads than that share only oversubscribe it."""
    count = os.cpu_count() or 1
    share = os.environ.get("OMP_NUM_THREADS")
    try:
        affinity = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        affinity = count
    threads = min(count, affinity, int(share)) if share and share.isdigit() and int(share) > 0 else min(count, affinity)
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return threads, dict(cpu_model=model, host_cpu_count=count, sched_affinity=affinity, omp_num_threads_env=share)


def cpu_baseline(seconds_budget=20.0):
    """Reference torch CPU path through the same model, fp32, on a bounded sample."""
    import torch
    from oracle.ss2d_core_ref import reference_vmamba_tiny
    cores, info = host_cpu()
    torch.set_num_threads(cores)
    torch.manual_seed(0)
    model = reference_vmamba_tiny().eval()
    batch = 16
    x = torch.randn(batch, 3, 224, 224)
    with torch.no_grad():
        t0 = time.perf_counter()
        model(x)
        first = time.perf_counter() - t0
        reps, spent = 0, 0.0
        while reps < 12 and spent + 2 * first < seconds_budget:
            t0 = time.perf_counter()
            model(x)
            spent += time.perf_counter() - t0
            reps += 1
    per = spent / reps if reps else first
    return dict(value=batch / per, unit="img/s", cores=cores, kind="port", **info,
                sample=f"VMamba-T forward, batch {batch} @224^2 fp32, torch CPU restatement of selective_scan_ref + "
                       f"torch CrossScan/CrossMerge, {max(reps, 1)} timed forward(s) after 1 warm-up, {per:.2f} s each")


def config0_inputs():
    """Benchmark config 0, seed 0, generated on the CPU in fp32 (the GPU gets copies of the same bits)."""
    import math
    import torch
    Bsz, Dn, H, W, K, N = 2, 96, 56, 56, 4, 1
    L = H * W
    g = torch.Generator().manual_seed(0)
    x = torch.randn(Bsz, Dn, H, W, generator=g)
    delta = torch.randn(Bsz, K * Dn, L, generator=g)
    dt = torch.exp(torch.rand(K * Dn, generator=g) * (math.log(0.1) - math.log(1e-3)) + math.log(1e-3))
    bias = dt + torch.log(-torch.expm1(-dt))
    A = -torch.exp(torch.log(torch.arange(1, N + 1, dtype=torch.float32))).repeat(K * Dn, 1)
    Bm, Cm = torch.randn(Bsz, K, N, L, generator=g), torch.randn(Bsz, K, N, L, generator=g)
    return x, delta, A, Bm, Cm, torch.ones(K * Dn), bias


def err_stats(got, want, rtol, atol):
    import torch
    diff = (got.double() - want.double()).abs()
    return dict(max_abs_err=diff.max().item(), max_rel_err=(diff / want.double().abs().clamp_min(atol / rtol)).max().item(),
                rtol=rtol, atol=atol, within_tolerance=bool(torch.allclose(got.float(), want.float(), rtol=rtol, atol=atol)))


def cpu_baseline_op(reps=3):
    """Config 0 on the host cores and on the GPU, same bits: seconds, GB/s over the same algorithmic bytes, and the GPU's
    error against the CPU result.  max_rel_err = max |gpu - cpu| / max(|cpu|, atol/rtol) (the reference tests' mixed
    tolerance, kernels/selective_scan/test_selective_scan.py:401-403, as one number: <= rtol means within tolerance)."""
    import statistics
    import torch
    import vmamba_amd as va
    from oracle import ss2d_oracle as orc
    from oracle import torch_ref
    from vmamba_amd.core import ss2d_core_hip
    cores, info = host_cpu()
    torch.set_num_threads(cores)
    x, delta, A, Bm, Cm, Dv, bias = config0_inputs()
    Bsz, Dn, H, W = x.shape
    K, L, N = 4, H * W, 1
    E = Bsz * Dn * L
    b_cs, b_sc, b_cm = 5 * E * 4, scan_bytes(Bsz, K * Dn, L, N, K, 4, 4), 5 * E * 4
    bytes_total = b_cs + b_sc + b_cm

    def torch_path():
        xs = torch_ref.cross_scan(x)
        ys = torch_ref.selective_scan(xs.reshape(Bsz, K * Dn, L), delta, A, Bm, Cm, Dv, bias, True)
        return xs, ys, torch_ref.cross_merge(ys.view(Bsz, K, Dn, H, W))

    def c_path():
        xs = orc.cross_scan(x)
        ys = orc.selective_scan(xs.view(Bsz, K * Dn, L), delta, A, Bm, Cm, Dv, bias, True)
        return xs, ys, orc.cross_merge(ys.view(Bsz, K, Dn, H, W))

    def timed(fn):
        fn()                                                    # warm-up
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            out = fn()
            ts.append(time.perf_counter() - t0)
        return statistics.median(ts), out

    with torch.no_grad():
        t_torch, (xs_t, ys_t, y_t) = timed(torch_path)
        t_c, (xs_c, ys_c, y_c) = timed(c_path)
        dev = "cuda:0"
        xd, dd, Ad, Bd, Cd, Dd, bd = (t.to(dev) for t in (x, delta, A, Bm, Cm, Dv, bias))

        def gpu_path():
            xs = va.cross_scan_fn(xd)
            ys = va.selective_scan_fn(xs.view(Bsz, K * Dn, L), dd, Ad, Bd, Cd, Dd, bd, True)
            return xs, ys, va.cross_merge_fn(ys.view(Bsz, K, Dn, H, W))

        delta_k = dd.view(Bsz, K, Dn, L).permute(1, 2, 0, 3).contiguous()
        B_k, C_k = Bd.view(Bsz, K, L).permute(1, 0, 2).contiguous(), Cd.view(Bsz, K, L).permute(1, 0, 2).contiguous()
        A1 = Ad.view(-1)
        t_gpu = time_op(gpu_path, 30)
        t_fused = time_op(lambda: ss2d_core_hip(xd, delta_k, B_k, C_k, A1, Dd, bd, True), 30)
        xs_g, ys_g, y_g = (t.cpu() for t in gpu_path())
        y_f = ss2d_core_hip(xd, delta_k, B_k, C_k, A1, Dd, bd, True).cpu()
    parity = dict(
        config="0: fp32, x (2,96,56,56) seed 0 -> CrossScan -> selective scan (softplus, N=1) -> CrossMerge",
        cpu_formulations_agree=dict(cross_scan_bit_exact=bool(torch.equal(xs_t, xs_c)), scan=err_stats(ys_c, ys_t, 1e-3, 1e-4),
                                    merged=err_stats(y_c, y_t, 1e-3, 4e-4)),
        cross_scan_bit_exact=bool(torch.equal(xs_g, xs_t)),
        scan_vs_torch_cpu=err_stats(ys_g, ys_t, 1e-3, 1e-4),
        cross_merge_bit_exact_on_gpu_scan_output=bool(torch.equal(y_g, torch_ref.cross_merge(ys_g.view(Bsz, K, Dn, H, W)))),
        three_operators_vs_torch_cpu=err_stats(y_g, y_t, 1e-3, 4e-4),
        fused_core_vs_torch_cpu=err_stats(y_f, y_t, 1e-3, 4e-4))
    base = dict(config="0", algorithmic_bytes=bytes_total, cores=cores, **info,
                torch_cpu=dict(seconds=t_torch, GBs=bytes_total / t_torch / 1e9, kind="port",
                               what=f"torch restatement of cross_scan_fwd + selective_scan_ref + cross_merge_fwd, median of {reps} after 1 warm-up"),
                c_oracle_cpu=dict(seconds=t_c, GBs=bytes_total / t_c / 1e9, kind="port",
                                  what=f"plain-C oracle (OpenMP over rows, {orc.num_threads()} threads), median of {reps} after 1 warm-up"),
                gpu_three_operators=dict(seconds=t_gpu, GBs=bytes_total / t_gpu / 1e9),
                gpu_fused_core=dict(seconds=t_fused, GBs=core_bytes(Bsz, Dn, L, 4) / t_fused / 1e9,
                                    algorithmic_bytes=core_bytes(Bsz, Dn, L, 4)),
                note="config 0 is 53 MB of traffic: on the GPU it is launch-bound (three launches of a few microseconds each)")
    return base, parity


def stage_parity(n_images=2):
    """A slice of every GPU configuration (bf16, batch 128) against the C oracle: the fused core's output for the first
    and the last ``n_images`` images of each VMamba-T stage shape."""
    import torch
    from oracle import ss2d_oracle as orc
    from vmamba_amd.core import ss2d_core_hip
    dev = "cuda:0"
    out = {}
    for name, (B, D, H, W) in dict(stage1=(128, 96, 56, 56), stage2=(128, 192, 28, 28), stage3=(128, 384, 14, 14),
                                   stage4=(128, 768, 7, 7)).items():
        L = H * W
        g = torch.Generator(device=dev).manual_seed(B + D)
        rn = lambda *s: torch.randn(*s, device=dev, generator=g)
        x, delta = rn(B, D, H, W).bfloat16(), (rn(4, D, B, L) * 0.5).bfloat16()
        Bs, Cs = rn(4, B, L).bfloat16(), rn(4, B, L).bfloat16()
        A, Dv, bias = -(0.5 + torch.rand(4 * D, device=dev, generator=g)), rn(4 * D), rn(4 * D) - 3.0
        y = ss2d_core_hip(x, delta, Bs, Cs, A, Dv, bias, True)
        worst = None
        for b0 in (0, B - n_images):
            sl = slice(b0, b0 + n_images)
            xs = orc.cross_scan(x[sl].cpu())
            ys = orc.selective_scan(xs.reshape(n_images, 4 * D, L), delta[:, :, sl].permute(2, 0, 1, 3).reshape(n_images, 4 * D, L).cpu(),
                                    A.view(-1, 1).cpu(), Bs[:, sl].permute(1, 0, 2).unsqueeze(2).cpu(), Cs[:, sl].permute(1, 0, 2).unsqueeze(2).cpu(),
                                    Dv.cpu(), bias.cpu(), True)
            want = orc.cross_merge(ys.view(n_images, 4, D, H, W))
            st = err_stats(y[sl].cpu(), want, 1e-3, 4e-4)
            if worst is None or st["max_rel_err"] > worst["max_rel_err"]:
                worst = st
        out[name] = worst
        del x, delta, Bs, Cs, y
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--batch", type=int, default=128)
    ap.add_argument("--image-size", type=int, default=224,
                    help="side of the square input images; 224 is the metric's workload, other sizes are side runs named in "
                         "config.workload (benchmark config 4: --batch 4 --image-size 1024 --sub-batches 1)")
    ap.add_argument("--kernel-reps", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--no-odd-maps", action="store_true", help="skip the forward_core lines on maps of odd sizes")
    ap.add_argument("--no-extra-forwards", action="store_true",
                    help="skip the config-4 (4 x 1024^2) and fp32 forwards reported as extra keys")
    ap.add_argument("--kernels-only", action="store_true",
                    help="skip the model: time the SS2D-core kernels at the four stage shapes plus a 1 GiB "
                         "device copy (the known-size kernel profiler counters are scaled against)")
    ap.add_argument("--eager", action="store_true",
                    help="time eager launches only.  By default three launch modes of the same forward are timed -- eager "
                         "launches, one captured HIP graph, sub-batch graphs side by side -- each graph mode only after its "
                         "replays reproduced the eager result bit for bit, and the fastest becomes `value`")
    ap.add_argument("--sub-batches", type=int, default=4,
                    help="run the batch as this many equal sub-batches, each captured into a HIP graph of its own and "
                         "replayed on its own stream, all launched together (kernels of one sub-batch fill the compute "
                         "units another leaves idle: 5.7 -> 5.2 ms); this number and half of it are tried and the faster kept; "
                         "the replays are first checked bit for bit against the eager sub-batch forwards; 1 = the whole "
                         "batch as one graph")
    ap.add_argument("--no-gemm-tuning", action="store_true",
                    help="skip PyTorch's TunableOp pass: by default the first (untimed) forward lets PyTorch-ROCm time the "
                         "hipBLASLt / rocBLAS solutions for each GEMM shape of the model and keep the fastest (~12 s)")
    ap.add_argument("--layout", choices=["channel_first", "channel_last"], default="channel_last",
                    help="activation layout of the harness outside the SS2D core (same weights, same math)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this build is the single-GPU SS2D hot path; it runs on exactly one GPU (--gpus 1).")
        sys.exit(2)

    import torch
    import vmamba_amd  # noqa: F401  (fails loudly if libss2d_hip.so is missing)
    from vmamba_amd.vssm import vmamba_tiny_s1l8

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    dev = "cuda:0"
    if args.kernels_only:
        with torch.no_grad():
            src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
            dst = torch.empty_like(src)
            t = time_op(lambda: dst.copy_(src), args.kernel_reps)
            log(f"calibration copy: 1 GiB read + 1 GiB write in {t * 1e6:.1f} us = {2 * (1 << 30) / t / 1e9:.0f} GB/s")
            del src, dst
            print(json.dumps({"kernels": kernel_lines(args.kernel_reps),
                              "odd_maps": None if args.no_odd_maps else odd_map_lines(args.kernel_reps)}))
        return
    torch.backends.cudnn.benchmark = True
    torch.manual_seed(0)
    model = vmamba_tiny_s1l8(channel_first=(args.layout == "channel_first")).to(dev).bfloat16().eval()
    if args.layout != "channel_first":
        # conv weights in channels-last memory format (same values, same state_dict): the stem / downsample convs then
        # run NHWC kernels and the permutes around them are views instead of copies
        model = model.to(memory_format=torch.channels_last)
    x = torch.randn(args.batch, 3, args.image_size, args.image_size, device=dev).bfloat16()

    def time_steps(step, warmup, steps):
        """The reference's protocol (classification/main.py:346-363): warm-up, synchronise, time `steps` launches
        between synchronisations.  Returns seconds for the `steps` launches."""
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    def capture_forward(net, inp):
        """Capture one forward into a HIP graph and check replays against the eager result (replays interleaved
        with eager work and synchronisations); returns (graph, static_output) or None if anything differs."""
        eager = net(inp).float()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                net(inp)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            out = net(inp)
        for _ in range(3):
            graph.replay()
            torch.cuda.synchronize()
            if not torch.equal(out.float(), eager):
                return None
            net(inp)                       # eager work between replays
            torch.cuda.synchronize()
        return graph, out

    tunable = None

    def tune(net, inp):
        """One untimed forward in which PyTorch's TunableOp times the library's own GEMM solutions for every GEMM shape
        it meets and keeps the fastest.  The projection / MLP GEMMs of stages 2-4 stay PyTorch-ROCm library calls."""
        if tunable is None:
            return
        tunable.tuning_enable(True)
        net(inp)
        torch.cuda.synchronize()
        tunable.tuning_enable(False)

    gemm_mode = "library-default GEMM solutions"
    sub_batches = args.sub_batches if (args.sub_batches > 1 and args.batch % args.sub_batches == 0) else 1
    modes = {}          # launch mode -> seconds for args.steps steps
    with torch.no_grad():
        model(x)
        torch.cuda.synchronize()
        log("first forward done")
        if not args.no_gemm_tuning:
            try:
                import torch.cuda.tunable as tunable_mod
                tunable_mod.enable(True)
                for setter, value in (("set_filename", "/tmp/vmamba_amd_tunableop.csv"), ("set_max_tuning_duration", 60),
                                      ("set_max_tuning_iterations", 60)):
                    if hasattr(tunable_mod, setter):
                        getattr(tunable_mod, setter)(value)
                tunable = tunable_mod
                t_tune = time.perf_counter()
                tune(model, x)
                gemm_mode = "GEMM solutions picked by PyTorch TunableOp"
                log(f"GEMM tuning forward: {time.perf_counter() - t_tune:.1f} s, {len(tunable.get_results())} shapes")
            except Exception as e:      # an optimisation of library calls, never a requirement
                log(f"TunableOp unavailable ({type(e).__name__}: {e}); library-default GEMM solutions")
                try:
                    tunable_mod.enable(False)
                except Exception:
                    pass
                tunable = None

        # ---- mode 1: eager launches, exactly the reference's loop ------------------------------------------------
        modes["eager"] = time_steps(lambda: model(x), args.warmup, args.steps)
        log(f"eager launches: {modes['eager'] / args.steps * 1e3:.2f} ms/step")

        # ---- mode 2: the forward as one captured HIP graph -------------------------------------------------------
        graph = None
        if not args.eager:
            try:
                captured = capture_forward(model, x)
                if captured is None:
                    log("graph replay did not reproduce the eager result; no one-graph figure")
                else:
                    graph = captured[0]
                    modes["one_graph"] = time_steps(graph.replay, args.warmup, args.steps)
                    log(f"one graph per forward: {modes['one_graph'] / args.steps * 1e3:.2f} ms/step")
            except Exception as e:          # capture is an optimisation of the launch path, never a requirement
                log(f"graph capture failed ({type(e).__name__}: {e})")

        # ---- mode 3: sub-batch graphs side by side ---------------------------------------------------------------
        runner = None
        if not args.eager and sub_batches > 1:
            from vmamba_amd.runner import ConcurrentGraphRunner
            for n in sorted({sub_batches, max(2, sub_batches // 2)}, reverse=True):
                if args.batch % n != 0:
                    continue
                try:
                    tune(model, x.chunk(n)[0])          # GEMM shapes of this sub-batch size
                    cand = ConcurrentGraphRunner(model, x, n)
                    replay_err = cand.max_replay_error(replays=5)
                    log(f"{n} concurrent sub-batch graphs: {cand.step_ms:.2f} ms per step; vs eager forwards over 5 replays: "
                        f"max abs difference {replay_err:g}")
                    if replay_err != 0.0:       # bit for bit, or not at all
                        log(f"{n} concurrent sub-batch graphs did not reproduce the eager result")
                    elif runner is None or cand.step_ms < runner.step_ms:
                        runner = cand
                    cand = None
                except Exception as e:          # an optimisation of the launch path, never a requirement
                    log(f"sub-batch graph capture failed ({type(e).__name__}: {e})")
            if runner is not None:
                sub_batches = len(runner.graphs)
                modes["concurrent"] = time_steps(runner.replay, args.warmup, args.steps)
                log(f"{sub_batches} sub-batch graphs side by side: {modes['concurrent'] / args.steps * 1e3:.2f} ms/step")

    launch = min(modes, key=modes.get)
    dt = modes[launch]
    launch_text = dict(eager="eager launches", one_graph="one captured HIP graph per forward",
                       concurrent=f"the batch as {sub_batches} sub-batches of {args.batch // sub_batches}, one captured HIP graph each, "
                                  f"replayed side by side (the caller's stream + {sub_batches - 1} more); replays checked bit for bit "
                                  f"against the eager sub-batch forwards before timing")[launch]
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    log(f"VMamba-T bs{args.batch}: {ms:.2f} ms/step, {value:.0f} img/s ({launch})")
    ms_of = lambda k: modes[k] / args.steps * 1e3 if k in modes else None

    # ---- benchmark config 4 and the fp32 forward (extra keys; eager launches, short runs) ---------------------------
    extra = {}
    if not args.no_extra_forwards:
        with torch.no_grad():
            try:
                runner = graph = None
                x4 = torch.randn(4, 3, 1024, 1024, device=dev).bfloat16()
                model(x4)
                tune(model, x4)
                t4 = time_steps(lambda: model(x4), 5, 10) / 10
                extra["config4"] = dict(workload="VMamba-T forward, 4 x 1024^2, bf16 (stage maps 256/128/64/32); ms_per_forward = eager "
                                                 "launches (four images leave them bound by the host's launch rate), "
                                                 "ms_per_forward_one_graph = the forward replayed as one captured HIP graph",
                                        ms_per_forward=t4 * 1e3, img_per_s=4 / t4)
                if not args.eager:
                    try:
                        captured4 = capture_forward(model, x4)
                        if captured4 is not None:
                            t4g = time_steps(captured4[0].replay, 5, 10) / 10
                            extra["config4"].update(ms_per_forward_one_graph=t4g * 1e3, img_per_s_one_graph=4 / t4g)
                        captured4 = None
                    except Exception as e:
                        log(f"config-4 graph capture failed ({type(e).__name__}: {e})")
                log("config 4:", extra["config4"])
                del x4
            except Exception as e:
                log(f"config-4 forward failed ({type(e).__name__}: {e})")
            try:
                model32 = model.float()
                x32 = x.float()
                model32(x32)
                t_tune = time.perf_counter()
                tune(model32, x32)
                log(f"fp32 GEMM tuning forward: {time.perf_counter() - t_tune:.1f} s")
                t32 = time_steps(lambda: model32(x32), 3, 10) / 10
                extra["fp32"] = dict(workload=f"VMamba-T forward, batch {args.batch} @{args.image_size}^2, fp32 activations and weights (the reference "
                                              f"harness's precision, no AMP), eager launches, {gemm_mode}",
                                     ms_per_step=t32 * 1e3, img_per_s=args.batch / t32)
                log("fp32:", extra["fp32"])
                if args.layout != "channel_first" and hasattr(model32, "with_layout"):
                    # the reference's own "ln2d" build of the model (channel-first blocks, Linear2d = 1x1 convolutions) in
                    # fp32: the configuration its published throughput figures were taken in
                    model_cf = model32.with_layout(True)
                    model_cf(x32)
                    tcf = time_steps(lambda: model_cf(x32), 2, 5) / 5
                    extra["fp32_channel_first"] = dict(
                        workload=f"VMamba-T forward, batch {args.batch} @{args.image_size}^2, fp32, channel-first blocks (the reference's "
                                 f"ln2d configuration, vmamba.py:1281), eager launches",
                        ms_per_step=tcf * 1e3, img_per_s=args.batch / tcf)
                    log("fp32 channel-first:", extra["fp32_channel_first"])
                    del model_cf
                del x32, model32
            except Exception as e:
                log(f"fp32 forward failed ({type(e).__name__}: {e})")
        torch.cuda.empty_cache()

    kernels, roofline, scan_roofline, ops_roofline, ext_fwd, odd_maps = None, None, None, None, None, None
    if not args.no_kernels:
        with torch.no_grad():
            kernels = kernel_lines(args.kernel_reps)
            odd_maps = None if args.no_odd_maps else odd_map_lines(args.kernel_reps)
        k1 = kernels[0]
        core_traffic, core_src = measured_traffic("ss2d_core_kernel@stage1")
        scan_traffic, scan_src = measured_traffic("scan_row_kernel@stage1")
        roofline = dict(bound="hbm", kernel="ss2d_core_kernel<bf16> (CrossScan+scan+CrossMerge fused) @ stage1 (B=128, D=96, 56x56, K=4)",
                        achieved=k1["core_fused_GBs"], peak=HBM_PEAK_GBS, unit="GB/s",
                        frac=k1["core_fused_GBs"] / HBM_PEAK_GBS, traffic=core_traffic, traffic_source=core_src,
                        bytes_per_launch=k1["core_fused_bytes"], us_per_launch=k1["core_fused_us"],
                        note="14 algorithmic bytes per element instead of the 62 of the three-operator path it replaces "
                             "(cross_scan + scan + cross_merge); the kernel is bound by VALU/transcendental issue, not HBM")
        scan_roofline = dict(bound="hbm", kernel="scan_row_kernel<bf16,f32,N=1> @ stage1 (B=128, KD=384, L=3136)",
                             achieved=k1["scan_GBs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=k1["scan_GBs"] / HBM_PEAK_GBS,
                             traffic=scan_traffic, traffic_source=scan_src, bytes_per_launch=k1["scan_bytes"],
                             us_per_launch=k1["scan_us"])
        # the three operators one after the other at stage-1 shape: the "SS2D scan + cross-scan/merge" of the metric
        ops_us = k1["cross_scan_us"] + k1["scan_us"] + k1["cross_merge_us"]
        ops_roofline = dict(bound="hbm", kernel="cross_scan + selective_scan + cross_merge (three launches) @ stage1",
                            achieved=k1["core_GBs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=k1["core_GBs"] / HBM_PEAK_GBS,
                            bytes_per_launch=k1["core_GBs"] * 1e9 * ops_us * 1e-6, us_per_launch=ops_us, traffic=None)
        # the scan through the reference's extension interface (it always returns the chunk states) beside selective_scan_fn
        ext_fwd = {k["shape"]: dict(kernel=k["scan_kernel"], fn_us=round(k["scan_us"], 1), ext_fwd_us=round(k["ext_fwd_us"], 1),
                                    ratio=round(k["ext_fwd_over_fn"], 3)) for k in kernels}
    cpu, cpu_op, parity = None, None, None
    if not args.no_cpu_baseline:
        cpu_op, parity = cpu_baseline_op()
        log("cpu_baseline_op", cpu_op)
        with torch.no_grad():
            parity["fused_core_bf16_bs128_vs_c_oracle"] = stage_parity()
        log("parity", parity)
        cpu = cpu_baseline()

    def compact(k):
        """One kernel line without the harness-side entries, numbers rounded: the full lines go to stderr."""
        keep = ("shape", "B", "D", "H", "W", "N", "scan_kernel", "cross_scan_us", "cross_scan_GBs", "scan_us", "scan_GBs", "ext_fwd_us",
                "cross_merge_us", "cross_merge_GBs", "core_GBs", "core_fused_us", "core_fused_GBs", "dt_proj_us", "dt_proj_GBs",
                "dwconv_us", "layer_norm_cf_us", "scan_bwd_us", "issue_frac", "valu_per_position_state", "core_n_us", "core_n_GBs",
                "three_operators_us", "cross_scan_copy_us", "cross_scan_over_copy", "scan_copy_us", "scan_over_copy")
        return {key: (round(v, 1 if key.endswith(("_us", "_GBs")) else 3) if isinstance(v, float) else v) for key, v in k.items() if key in keep}

    fp32 = extra.get("fp32") or {}
    fp32_cf = extra.get("fp32_channel_first") or {}
    c4 = extra.get("config4") or {}
    record = {
        "metric": "VMamba-T img/s @224^2 bs128 on 1xMI355X; SS2D scan HBM GB/s vs peak",
        "value": value, "unit": "img/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"launch": launch, "sub_batches": sub_batches if launch == "concurrent" else 1,
                   "workload": f"VMamba-T (vmamba_tiny_s1l8 shape, random init) forward, batch {args.batch} @{args.image_size}x{args.image_size}, "
                               f"bf16 activations/weights, fp32 scan state, {args.layout} blocks, {launch_text}, {gemm_mode}; "
                               f"SS2D core, LayerNorm, depthwise conv, patch-embedding stem, narrow-stage MLP and projections on HIP kernels",
                   # the reference's own protocol is one eager model(images) per step (classification/main.py:346-363)
                   "img_per_s_eager": args.batch / (ms_of("eager") * 1e-3) if ms_of("eager") else None,
                   "img_per_s_fp32": fp32.get("img_per_s"), "img_per_s_fp32_channel_first": fp32_cf.get("img_per_s")},
        "ms_per_step_eager": ms_of("eager"), "ms_per_step_one_graph": ms_of("one_graph"),
        "ms_per_step_concurrent": ms_of("concurrent"),
        "ms_per_step_fp32": fp32.get("ms_per_step"), "ms_per_step_fp32_channel_first": fp32_cf.get("ms_per_step"),
        "config4_ms_per_forward": c4.get("ms_per_forward"), "config4_ms_per_forward_one_graph": c4.get("ms_per_forward_one_graph"),
        "roofline": roofline, "scan_roofline": scan_roofline, "three_operator_roofline": ops_roofline,
        "ext_fwd": ext_fwd, "cpu_baseline": cpu,
    }
    # Everything else -- the workload descriptions of the extra forwards, the CPU operator leg with its parity numbers and
    # the full per-kernel lines -- goes to stderr as one JSON document, and in compact form into the record, so that the
    # record stays a line of a few KB.
    details = {**extra, "cpu_baseline_op": cpu_op, "parity": parity, "kernels": kernels}
    log("DETAILS " + json.dumps(details))
    if cpu_op is not None:
        record["cpu_baseline_op"] = dict(config=cpu_op["config"], cores=cpu_op["cores"], algorithmic_bytes=cpu_op["algorithmic_bytes"],
                                         torch_cpu_s=cpu_op["torch_cpu"]["seconds"], c_oracle_cpu_s=cpu_op["c_oracle_cpu"]["seconds"],
                                         gpu_three_operators_s=cpu_op["gpu_three_operators"]["seconds"],
                                         gpu_fused_core_s=cpu_op["gpu_fused_core"]["seconds"])
    if parity is not None:
        flat = {}
        for key, v in parity.items():
            if isinstance(v, dict) and "max_rel_err" in v:
                flat[key] = dict(max_rel_err=float(f"{v['max_rel_err']:.3g}"), ok=v["within_tolerance"])
            elif isinstance(v, dict):
                flat[key] = {k2: (dict(max_rel_err=float(f"{v2['max_rel_err']:.3g}"), ok=v2["within_tolerance"])
                                  if isinstance(v2, dict) and "max_rel_err" in v2 else v2) for k2, v2 in v.items()}
            elif isinstance(v, bool):
                flat[key] = v
        record["parity"] = flat
    if kernels is not None:
        record["kernels"] = [compact(k) for k in kernels]
    if odd_maps is not None:
        record["odd_maps"] = [dict(odd=o["odd"]["shape"], aligned=o["aligned"]["shape"], embedded_in=o["embedded_in"],
                                   odd_us=o["odd"]["us"], aligned_us=o["aligned"]["us"], per_element_ratio=o["per_element_ratio"])
                              for o in odd_maps]
    print(json.dumps(record))


if __name__ == "__main__":
    main()
