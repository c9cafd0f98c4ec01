"""Composition parity: SS2D.forward_core and the VMamba-T-shaped harness on the GPU (HIP core)
against the same modules with the torch-on-CPU reference core and identical weights."""
import copy

import pytest
import torch

from oracle.ss2d_core_ref import RefSS2D, reference_vmamba_tiny
from vmamba_amd.ss2d import SS2D
from vmamba_amd.vssm import VSSM, vmamba_tiny_s1l8

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def bf16_ulp(scale):
    """Spacing of bf16 numbers at magnitude `scale` (8 significand bits)."""
    import math
    return 2.0 ** (math.floor(math.log2(scale)) - 7)


def logit_error_report(got, want, what):
    """Per-element error of logits against the fp32 reference: in units of the bf16 spacing at the largest |logit|, and
    relative to each reference logit (floored at 5 % of the largest, random-init logits crossing zero).  Returns the
    largest error in bf16 spacings and the median relative error; prints median / p99 / max of both."""
    got, want = got.double().cpu(), want.double().cpu()
    scale = want.abs().max().item()
    err = (got - want).abs().flatten()
    rel = err / want.abs().flatten().clamp_min(0.05 * scale)
    q = lambda t, p: torch.quantile(t, p).item()
    print(f"{what}: largest |logit| {scale:.4g} (bf16 spacing {bf16_ulp(scale):.3g}); |error| in spacings: median "
          f"{q(err, 0.5) / bf16_ulp(scale):.3f} p99 {q(err, 0.99) / bf16_ulp(scale):.3f} max {err.max().item() / bf16_ulp(scale):.3f}; "
          f"relative error: median {q(rel, 0.5):.3g} p99 {q(rel, 0.99):.3g} max {rel.max().item():.3g}", flush=True)
    return err.max().item() / bf16_ulp(scale), q(rel, 0.5)


def _pair(d_model, d_state, ssm_ratio=1.0, disable_z=True, seed=0):
    torch.manual_seed(seed)
    ref = RefSS2D(d_model=d_model, d_state=d_state, ssm_ratio=ssm_ratio, disable_z=disable_z).eval()
    hip = SS2D(d_model=d_model, d_state=d_state, ssm_ratio=ssm_ratio, disable_z=disable_z).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, hip.to(DEV)


def _pair_cl(d_model, d_state, ssm_ratio=1.0, seed=0):
    torch.manual_seed(seed)
    ref = RefSS2D(d_model=d_model, d_state=d_state, ssm_ratio=ssm_ratio, channel_first=False).eval()
    hip = SS2D(d_model=d_model, d_state=d_state, ssm_ratio=ssm_ratio, channel_first=False).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, hip.to(DEV)


def test_forward_core_channel_last_output():
    """channel_first=False blocks: forward_core still takes (B,D,H,W) and returns (B,H,W,D) (vmamba.py:642-643)."""
    print("CASE core-cl", flush=True)
    ref, hip = _pair_cl(48, 1)
    x = torch.randn(2, 48, 14, 14, generator=torch.Generator().manual_seed(6))
    with torch.no_grad():
        want = ref.forward_core(x)
        got = hip.forward_core(x.to(DEV)).cpu()
    assert got.shape == want.shape == (2, 14, 14, 48)
    assert torch.allclose(got, want, rtol=1e-3, atol=1e-3)
    xb = torch.randn(2, 14, 14, 48, generator=torch.Generator().manual_seed(7))
    with torch.no_grad():
        assert torch.allclose(hip(xb.to(DEV)).cpu(), ref(xb), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("d_model,d_state,ratio,H,W", [(96, 1, 1.0, 56, 56), (32, 1, 1.0, 7, 7), (24, 16, 2.0, 14, 14),
                                                     (16, 1, 1.0, 9, 13)])
def test_forward_core_fp32(d_model, d_state, ratio, H, W):
    print("CASE core-fp32", d_model, d_state, ratio, H, W, flush=True)
    ref, hip = _pair(d_model, d_state, ratio)
    x = torch.randn(2, ref.d_inner, H, W, generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        want = ref.forward_core(x)
    for fused in (True, False):       # one fused kernel (one-state models) / the three operators
        hip.fused_core = fused
        with torch.no_grad():
            got = hip.forward_core(x.to(DEV)).cpu()
        assert got.shape == want.shape == x.shape and got.dtype == x.dtype
        assert torch.allclose(got, want, rtol=1e-3, atol=1e-3), f"fused={fused}"


def test_forward_core_bf16_activations():
    """benchmark config 1 recipe at reduced batch: bf16 activations and weights, fp32 scan state.  The GEMMs run
    in bf16 on both sides but with different accumulation orders, so the bound is the bf16 one (2e-2)."""
    print("CASE core-bf16", flush=True)
    ref, hip = _pair(96, 1)
    ref, hip = ref.bfloat16(), hip.bfloat16()
    x = torch.randn(4, 96, 56, 56, generator=torch.Generator().manual_seed(2)).bfloat16()
    with torch.no_grad():
        want = ref.forward_core(x).float()
    for fused in (True, False):
        hip.fused_core = fused
        with torch.no_grad():
            got = hip.forward_core(x.to(DEV)).float().cpu()
        assert torch.allclose(got, want, rtol=2e-2, atol=2e-2), f"fused={fused}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("channel_first", [True, False], ids=["cf", "cl"])
@pytest.mark.parametrize("d_model,B,H,W", [(96, 3, 57, 58), (32, 5, 19, 19), (192, 2, 75, 75), (128, 2, 19, 19), (48, 2, 37, 41), (768, 1, 19, 19), (1024, 1, 19, 19)])
def test_forward_core_on_maps_embedded_in_padded_ones(d_model, B, H, W, channel_first, dtype):
    """16-bit maps whose sides the vector paths do not like run the fused core on a zero-padded map (the added positions made
    neutral by the masked dt_proj, or by ss2d_core_mask_pads where the rank is beyond that kernel -- 64 here) and are cut out of its
    result: against the fp32 CPU model at the 16-bit bound, and against the three-operator path of the same module, which
    pads nothing, at a few roundings of the 16-bit output."""
    from vmamba_amd.core import padded_map_size
    print("CASE core-padded", d_model, B, H, W, channel_first, dtype, flush=True)
    torch.manual_seed(3)
    ref = RefSS2D(d_model=d_model, d_state=1, ssm_ratio=1.0, channel_first=channel_first).eval()
    hip = SS2D(d_model=d_model, d_state=1, ssm_ratio=1.0, channel_first=channel_first).eval()
    hip.load_state_dict(ref.state_dict())
    hip = hip.to(dtype).to(DEV)
    assert padded_map_size(H, W, dtype) is not None
    x = torch.randn(B, d_model, H, W, generator=torch.Generator().manual_seed(4)).to(dtype)
    with torch.no_grad():
        want = ref.forward_core(x.float())
        hip.fused_core = True
        got = hip.forward_core(x.to(DEV))
        hip.fused_core = False
        ops = hip.forward_core(x.to(DEV))
    assert got.shape == want.shape and got.dtype == dtype
    tol = 2e-2 if dtype == torch.bfloat16 else 4e-3
    assert torch.allclose(got.float().cpu(), want, rtol=tol, atol=tol)
    assert torch.allclose(got.float(), ops.float(), rtol=tol / 2, atol=tol / 2)


def test_block_with_gate_matches():
    print("CASE block-z", flush=True)
    ref, hip = _pair(24, 16, 2.0, disable_z=False)
    x = torch.randn(2, 24, 14, 14, generator=torch.Generator().manual_seed(3))
    with torch.no_grad():
        assert torch.allclose(hip(x.to(DEV)).cpu(), ref(x), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("channel_first", [True, False])
def test_vmamba_tiny_logits_match_reference_core(channel_first):
    print("CASE vssm", channel_first, flush=True)
    torch.manual_seed(4)
    ref = reference_vmamba_tiny().eval()                             # all-torch CPU model, channel-first layout
    assert sum(p.numel() for p in ref.parameters()) == 30249064      # analyze/tp.py:162
    hip = vmamba_tiny_s1l8(channel_first=channel_first).eval()
    hip.load_state_dict(ref.state_dict())
    hip = hip.to(DEV)
    x = torch.randn(2, 3, 96, 96, generator=torch.Generator().manual_seed(5))
    with torch.no_grad():
        want = ref(x)
        got = hip(x.to(DEV)).cpu()
    assert got.shape == (2, 1000)
    assert torch.allclose(got, want, rtol=2e-3, atol=2e-3)


def test_vmamba_tiny_bf16_benchmark_layout_matches_fp32_reference():
    """The benchmark's model at its own resolution: bf16, 224^2 (stage maps 56 / 28 / 14 / 7, so every stage takes the
    kernels it takes in the benchmark -- the fused core with its per-stage tile choices, LayerNorm + MLP in one kernel
    at widths 96 / 192, the narrow projections, add + LayerNorm between blocks).  Checked against the all-torch fp32
    CPU model holding the same bf16-rounded weights, and against the channel-first bf16 model, which shares the
    weights but none of the block-level kernels.  22 blocks of bf16 activations: the bound is the bf16 one (2e-2)
    on the scale of the logits."""
    print("CASE vssm-bf16-224", flush=True)
    torch.manual_seed(14)
    ref = reference_vmamba_tiny().eval().bfloat16().float()          # weights exactly representable in bf16
    x = torch.randn(2, 3, 224, 224, generator=torch.Generator().manual_seed(15)).bfloat16()
    with torch.no_grad():
        want = ref(x.float())
    scale = want.abs().max().item()
    got = {}
    for channel_first in (False, True):
        hip = vmamba_tiny_s1l8(channel_first=channel_first).eval()
        hip.load_state_dict(ref.state_dict())
        hip = hip.bfloat16().to(DEV)
        with torch.no_grad():
            got[channel_first] = hip(x.to(DEV)).float().cpu()
        err = (got[channel_first] - want).abs().max().item()
        assert got[channel_first].shape == (2, 1000)
        assert err <= 2e-2 * scale, f"channel_first={channel_first}"
        # per element: no logit further from the fp32 model than two bf16 spacings at the logits' scale (measured: 0.6),
        # half of them within 1 % of their value (measured: 0.5 %)
        worst, median_rel = logit_error_report(got[channel_first], want, f"bf16 224^2 channel_first={channel_first} vs fp32 CPU model")
        assert worst <= 2.0 and median_rel <= 1e-2, f"channel_first={channel_first}"
    assert (got[True] - got[False]).abs().max().item() <= 2e-2 * scale


def test_vmamba_tiny_bf16_1024px_batch4():
    """Benchmark config 4: the full backbone on a batch of four 1024^2 images in bf16.  Stage maps 256 / 128 / 64 / 32:
    stages 1-2 (L = 65536, 16384) take the three separate operators -- the scan splits each row over the four
    wavefronts of a workgroup and carries the state from 2048-chunk to chunk -- stages 3-4 the fused core.  One image
    is checked against the all-torch fp32 CPU model (same bf16-rounded weights), all four between the channel-last
    and the channel-first model."""
    print("CASE vssm-bf16-1024", flush=True)
    torch.manual_seed(16)
    ref = reference_vmamba_tiny().eval().bfloat16().float()
    x = torch.randn(4, 3, 1024, 1024, generator=torch.Generator().manual_seed(17)).bfloat16()
    with torch.no_grad():
        want = ref(x[3:4].float())
    scale = want.abs().max().item()
    got = {}
    for channel_first in (False, True):
        hip = vmamba_tiny_s1l8(channel_first=channel_first).eval()
        hip.load_state_dict(ref.state_dict())
        hip = hip.bfloat16().to(DEV)
        with torch.no_grad():
            got[channel_first] = hip(x.to(DEV)).float().cpu()
        del hip
        err = (got[channel_first][3:4] - want).abs().max().item()
        assert got[channel_first].shape == (4, 1000) and torch.isfinite(got[channel_first]).all()
        assert err <= 2e-2 * scale, f"channel_first={channel_first}"
        worst, median_rel = logit_error_report(got[channel_first][3:4], want, f"bf16 1024^2 channel_first={channel_first} vs fp32 CPU model")
        assert worst <= 2.0 and median_rel <= 1e-2, f"channel_first={channel_first}"
    assert (got[True] - got[False]).abs().max().item() <= 2e-2 * scale


@pytest.mark.parametrize("dims,ratio,d_state,size", [((128, 256, 512, 1024), 2.0, 1, 224), ((96, 192, 384, 768), 2.0, 1, 128),
                                                     ((64, 128, 256, 512), 1.0, 4, 96)])
def test_other_model_widths_match_reference_core(dims, ratio, d_state, size):
    """The widths of the reference's larger models (ssm_ratio 2: up to 2048 inner channels, dt ranks up to 64) and a
    several-state variant, one block per stage, bf16 channel-last: logits against the all-torch fp32 CPU model that
    holds the same bf16-rounded weights."""
    from oracle.ss2d_core_ref import TorchLayers
    print("CASE vssm-widths", dims, ratio, d_state, size, flush=True)
    torch.manual_seed(21)
    cfg = dict(depths=(1, 1, 1, 1), dims=dims, d_state=d_state, ssm_ratio=ratio, num_classes=40)
    ref = VSSM(**cfg, channel_first=True, ss2d_cls=RefSS2D, layers=TorchLayers).eval().bfloat16().float()
    hip = VSSM(**cfg, channel_first=False).eval()
    hip.load_state_dict(ref.state_dict())
    hip = hip.bfloat16().to(DEV)
    x = torch.randn(2, 3, size, size, generator=torch.Generator().manual_seed(22)).bfloat16()
    with torch.no_grad():
        want = ref(x.float())
        got = hip(x.to(DEV)).float().cpu()
    scale = want.abs().max().item()
    assert got.shape == (2, 40)
    assert (got - want).abs().max().item() <= 2e-2 * scale


def test_with_layout_twin_gives_the_same_logits():
    """A model built channel-first (what the reference's "ln2d" configurations do) and its channel-last twin: same
    logits to the bf16 bound."""
    print("CASE vssm-with-layout", flush=True)
    torch.manual_seed(31)
    cf = vmamba_tiny_s1l8(channel_first=True).eval().bfloat16().to(DEV)
    cl = cf.with_layout(False)
    assert next(cl.parameters()).device.type == "cuda" and next(cl.parameters()).dtype == torch.bfloat16
    x = torch.randn(3, 3, 224, 224, device=DEV).bfloat16()
    shared = cf.with_layout(False, share_weights=True)
    with torch.no_grad():
        a, b, c = cf(x).float(), cl(x).float(), shared(x).float()
    assert (a - b).abs().max().item() <= 2e-2 * a.abs().max().item()
    # same weights through the same kernels; not asserted bit for bit, since the library may pick another convolution
    # or GEMM solution for the second model, whose fp32 sums then round differently here and there: two bf16 spacings
    # at the logits' scale bound that (measured over three seeds: 0, 0.5 and 1 spacing)
    worst, _ = logit_error_report(c, b, "shared-weights twin vs its channel-last original")
    assert worst <= 2.0


def test_small_vssm_trains_on_the_gpu():
    """One training step: gradients of a small model on the GPU (HIP scan / cross-scan / cross-merge backward, torch
    autograd for the rest) against the all-torch CPU model with the same weights."""
    print("CASE vssm-train", flush=True)
    from oracle.ss2d_core_ref import TorchLayers
    torch.manual_seed(11)
    cfg = dict(depths=(1, 1), dims=(16, 32), num_classes=7)
    ref = VSSM(**cfg, channel_first=True, ss2d_cls=RefSS2D, layers=TorchLayers).train()
    hip = VSSM(**cfg, channel_first=False).train()
    hip.load_state_dict(ref.state_dict())
    hip = hip.to(DEV)
    x = torch.randn(2, 3, 32, 32, generator=torch.Generator().manual_seed(12))
    target = torch.tensor([1, 5])
    loss_ref = torch.nn.functional.cross_entropy(ref(x), target)
    loss_ref.backward()
    loss_hip = torch.nn.functional.cross_entropy(hip(x.to(DEV)), target.to(DEV))
    loss_hip.backward()
    assert abs(loss_hip.item() - loss_ref.item()) < 1e-3
    grads_ref = dict(ref.named_parameters())
    n = 0
    for name, p in hip.named_parameters():
        g, w = p.grad, grads_ref[name].grad
        assert g is not None and torch.isfinite(g).all(), name
        w = w.view(g.shape)                   # 1x1-conv weights of the channel-first model are the same matrices
        scale = w.abs().max().item()
        assert (g.cpu() - w).abs().max().item() <= 5e-3 * scale + 1e-6, name
        n += 1
    assert n == len(grads_ref)
