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
