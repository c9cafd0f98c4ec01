"""CPU checks of the host-side model code (no kernels run): shapes, parameter inventory and the
projection identity the SS2D core relies on."""
import torch

from oracle.ss2d_core_ref import RefSS2D
from vmamba_amd.ss2d import SS2D
from vmamba_amd.vssm import vmamba_tiny_s1l8


def test_parameter_inventory_matches_reference_shapes():
    m = SS2D(d_model=96, d_state=1, ssm_ratio=1.0)
    K, D, R, N = 4, 96, 6, 1
    assert m.x_proj_weight.shape == (K, R + 2 * N, D)        # vmamba.py:468
    assert m.dt_projs_weight.shape == (K, D, R)              # vmamba.py:225
    assert m.dt_projs_bias.shape == (K, D)
    assert m.A_logs.shape == (K * D, N) and m.Ds.shape == (K * D,)
    assert torch.equal(m.Ds, torch.ones(K * D))
    dt = torch.nn.functional.softplus(m.dt_projs_bias)
    assert dt.min() >= 1e-3 * 0.999 and dt.max() <= 0.1 * 1.001  # dt log-uniform in [1e-3, 0.1]
    m16 = SS2D(d_model=96, d_state=16, ssm_ratio=2.0, disable_z=False)
    assert torch.allclose(m16.A_logs[5].exp(), torch.arange(1, 17).float())
    assert m16.in_proj.weight.shape == (2 * 192, 96)


def test_vmamba_tiny_parameter_count():
    assert sum(p.numel() for p in vmamba_tiny_s1l8().parameters()) == 30249064   # analyze/tp.py:162


def test_grouped_conv_equals_einsum():
    # x_proj/dt_proj as grouped conv1d == the einsum form (vmamba.py:605-608 vs :610-615)
    torch.manual_seed(0)
    m = SS2D(d_model=16, d_state=2, ssm_ratio=1.0)
    xs = torch.randn(2, 4, 16, 30)
    dts, Bs, Cs = m.project(xs)
    x_dbl = torch.einsum("bkdl,kcd->bkcl", xs, m.x_proj_weight)
    r, Bs2, Cs2 = torch.split(x_dbl, [m.dt_rank, 2, 2], dim=2)
    dts2 = torch.einsum("bkrl,kdr->bkdl", r, m.dt_projs_weight).reshape(2, -1, 30)
    assert torch.allclose(dts, dts2, atol=1e-5) and torch.allclose(Bs, Bs2, atol=1e-5) and torch.allclose(Cs, Cs2, atol=1e-5)


def test_reference_core_runs_on_cpu():
    torch.manual_seed(0)
    m = RefSS2D(d_model=8, d_state=1).eval()
    with torch.no_grad():
        y = m(torch.randn(1, 8, 5, 6))
    assert y.shape == (1, 8, 5, 6) and torch.isfinite(y).all()


def test_vssm_state_dict_uses_reference_key_names_and_loads_legacy_checkpoints():
    """State-dict keys are the reference's (classification/models/vmamba.py:1356-1363, 1402-1437, 1487-1490), and the
    key prefixes of its older training code are renamed on load (vmamba.py:1557-1564)."""
    import torch
    from oracle.ss2d_core_ref import reference_vmamba_tiny
    from vmamba_amd.vssm import VSSM

    torch.manual_seed(0)
    small = dict(depths=(1, 2), dims=(16, 32), num_classes=5)
    src = VSSM(**small, channel_first=False, layers=__import__("oracle.ss2d_core_ref", fromlist=["TorchLayers"]).TorchLayers)
    keys = set(src.state_dict().keys())
    block = {"norm.weight", "norm.bias", "op.x_proj_weight", "op.A_logs", "op.Ds", "op.dt_projs_weight", "op.dt_projs_bias",
             "op.in_proj.weight", "op.conv2d.weight", "op.out_norm.weight", "op.out_norm.bias", "op.out_proj.weight",
             "norm2.weight", "norm2.bias", "mlp.fc1.weight", "mlp.fc1.bias", "mlp.fc2.weight", "mlp.fc2.bias"}
    want = {f"patch_embed.{i}.{p}" for i in (0, 2, 5, 7) for p in ("weight", "bias")}
    want |= {f"layers.{i}.blocks.{j}.{k}" for (i, j) in ((0, 0), (1, 0), (1, 1)) for k in block}
    want |= {f"layers.0.downsample.{i}.{p}" for i in (1, 3) for p in ("weight", "bias")}
    want |= {f"classifier.{m}.{p}" for m in ("norm", "head") for p in ("weight", "bias")}
    assert keys == want
    assert len(reference_vmamba_tiny().state_dict()) == 276

    # a checkpoint written with the old names
    legacy = {}
    for k, v in src.state_dict().items():
        k = k.replace(".norm.", ".ln_1.") if ".blocks." in k and ".norm." in k and ".op." not in k else k
        k = k.replace(".op.", ".self_attention.")
        k = k.replace("patch_embed.0.", "patch_embed.proj.").replace("patch_embed.2.", "patch_embed.norm.")
        k = k.replace("classifier.norm.", "norm.").replace("classifier.head.", "head.")
        legacy[k] = v.clone()
    assert set(legacy) != keys
    dst = VSSM(**small, channel_first=False, layers=src.layers[0].blocks[0].op.layers)
    result = dst.load_state_dict(legacy, strict=True)
    assert not result.missing_keys and not result.unexpected_keys
    for (ka, a), (kb, b) in zip(src.state_dict().items(), dst.state_dict().items()):
        assert ka == kb and torch.equal(a, b)
    # channel-first models store 1x1-conv weights; a channel-last checkpoint loads into them (vmamba.py:47-49)
    cf = VSSM(**small, channel_first=True, layers=src.layers[0].blocks[0].op.layers)
    cf.load_state_dict(src.state_dict(), strict=True)
    assert torch.equal(cf.layers[0].blocks[0].mlp.fc1.weight, src.layers[0].blocks[0].mlp.fc1.weight)


def test_gelu_table_is_what_the_generator_writes_and_matches_erf():
    """The fused MLP kernel's GELU table: the committed include equals a fresh render, and its entries are
    0.5 erf(x / sqrt 2) at the bf16 grid (checked against scipy's erf, an independent implementation)."""
    import importlib.util, os, re, struct
    import numpy as np
    from scipy.special import erf
    here = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "vmamba_amd", "csrc")
    spec = importlib.util.spec_from_file_location("gen_gelu_table", os.path.join(here, "gen_gelu_table.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    text = open(os.path.join(here, "gelu_table.inc")).read()
    assert text == gen.render()
    bits = np.array([int(h, 16) for h in re.findall(r"0x([0-9a-f]{8})u", text)], dtype=np.uint32)
    assert bits.size == gen.HI_BITS - gen.LO_BITS == 2176
    vals = bits.view(np.float32).astype(np.float64)
    x = (np.arange(gen.LO_BITS, gen.HI_BITS, dtype=np.uint32) << 16).view(np.float32).astype(np.float64)
    assert x[0] == 2.0 ** -14 and x[-1] < 8.0 and x[-1] > 7.9
    want = 0.5 * erf(x / np.sqrt(2.0))
    assert np.all(np.abs(vals - want) <= 2.0 ** -24 * np.maximum(want, 1e-30) * 1.01)      # fp32 rounding of the exact value
    assert vals[-1] == 0.5 and np.all(np.diff(vals) >= 0)
    # the identity the kernel uses: gelu(x) = 0.5 x + |x| E(|x|), both signs
    for s in (1.0, -1.0):
        g = 0.5 * s * x + x * vals
        assert np.allclose(g, 0.5 * s * x * (1.0 + erf(s * x / np.sqrt(2.0))), rtol=0, atol=1e-6)


def test_inference_constants_are_kept_per_batch_size_and_follow_the_parameters():
    """A = -exp(A_logs) etc. (vmamba.py:619-623) are cached per batch size -- the sub-batches of a runner alternate with
    whole batches -- and recomputed when a parameter changes or autograd is on."""
    m = SS2D(d_model=8, d_state=1, ssm_ratio=1.0, dt_rank=2, channel_first=False)
    with torch.no_grad():
        c2, c3 = m._inference_constants(2), m._inference_constants(3)
        assert m._inference_constants(2) is c2 and m._inference_constants(3) is c3
        assert c2["Wx"].shape[0] == 2 * 4 and c3["Wx"].shape[0] == 3 * 4
        assert torch.equal(c2["As"], -m.A_logs.float().exp())
        for b in range(4, 10):                                   # the cache stays small
            m._inference_constants(b)
        assert len(m._const_cache) <= 4
        m.A_logs.add_(0.5)                                       # in-place update bumps the version: everything stale
        fresh = m._inference_constants(2)
        assert fresh is not c2 and torch.equal(fresh["As"], -m.A_logs.float().exp())
        assert all(k[0] == 2 for k in m._const_cache)
    assert m._inference_constants(2) is not m._inference_constants(2)      # under autograd nothing is kept


def test_with_layout_keeps_keys_values_and_mode():
    """VSSM.with_layout: the channel-last twin of a channel-first model holds the same state_dict (names, shapes, values)
    -- a Linear2d weight (out, in, 1, 1) and the nn.Linear weight (out, in) are one tensor viewed two ways
    (vmamba.py:47-49) -- and converts back."""
    from vmamba_amd.vssm import VSSM
    torch.manual_seed(3)
    m = VSSM(depths=(1, 1, 1, 1), dims=(16, 32, 64, 128), d_state=2, ssm_ratio=2.0, num_classes=10, channel_first=True).eval()
    twin = m.with_layout(False)
    assert not twin.training and twin.layers[0].blocks[0].op.channel_first is False
    sd, sd2 = m.state_dict(), twin.state_dict()
    assert list(sd) == list(sd2)
    for k in sd:
        assert sd[k].numel() == sd2[k].numel() and torch.equal(sd[k].reshape(-1), sd2[k].reshape(-1)), k
    back = twin.with_layout(True).state_dict()
    assert all(back[k].shape == sd[k].shape and torch.equal(back[k], sd[k]) for k in sd)
    # shared weights: the same Parameter objects under the same names; a change through one model is seen by the other
    shared = m.with_layout(False, share_weights=True)
    for (k, p), (k2, p2) in zip(m.named_parameters(), shared.named_parameters()):
        assert k == k2 and p is p2
    with torch.no_grad():
        m.classifier.head.weight.mul_(2.0)
    assert shared.classifier.head.weight is m.classifier.head.weight
    m.double()
    assert next(shared.parameters()).dtype == torch.float64
