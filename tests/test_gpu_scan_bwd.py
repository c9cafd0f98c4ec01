"""GPU parity of the selective-scan backward (through the C ABI and through autograd) against float64 autograd of
the CPU restatement.  Tolerance: rtol 2e-3 plus 2e-3 of the gradient's largest magnitude for fp32 inputs (sums over
up to a few thousand positions in fp32 with hardware exp2 / log2); 16-bit inputs: 3e-2."""
import pytest
import torch

from oracle import torch_ref
import vmamba_amd as va
from vmamba_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NAMES = ["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias"]


def make(seed, batch, dim, G, N, L, dtype, delta_dim=None, softplus=True):
    g = torch.Generator().manual_seed(seed)
    delta_dim = delta_dim or dim
    A = -0.5 * torch.rand(dim, N, generator=g) - 0.05
    if softplus:
        delta = torch.randn(batch, delta_dim, L, generator=g) - 1.0
        bias = torch.randn(delta_dim, generator=g) * 0.5 - 1.0
    else:
        delta = 0.3 * torch.rand(batch, delta_dim, L, generator=g)
        bias = 0.2 * torch.rand(delta_dim, generator=g)
    B = torch.randn(batch, G, N, L, generator=g)
    C = torch.randn(batch, G, N, L, generator=g)
    u = torch.randn(batch, dim, L, generator=g)
    D = torch.randn(dim, generator=g)
    dout = torch.randn(batch, dim, L, generator=g)
    return u.to(dtype), delta.to(dtype), A, B.to(dtype), C.to(dtype), D, bias, dout


def compare(got, want, tol, what):
    for name, g, w in zip(NAMES, got, want):
        if w is None:
            assert g is None, name
            continue
        g, w = g.double().cpu(), w.double()
        assert g.shape == w.shape, (name, g.shape, w.shape)
        scale = w.abs().max().item() + 1e-12
        err = (g - w).abs().max().item()
        assert err <= tol * scale + tol * 1e-3, f"{what} {name}: max err {err} vs scale {scale}"


CASES = [
    # batch, dim, G, N, L, delta_dim, softplus
    (2, 4, 1, 1, 40, None, True),          # one short pass
    (2, 8, 4, 1, 700, None, True),         # two passes, SS2D-like grouping (2 channels per B/C row)
    (1, 4, 2, 4, 1030, None, True),        # three passes, several states
    (2, 6, 2, 3, 513, 3, True),            # delta rows shared by two channels; one element into the second pass
    (1, 4, 1, 16, 300, None, True),        # 16 states
    (2, 4, 2, 2, 600, None, False),        # no softplus
    (1, 3, 1, 1, 9, None, True),           # shorter than a lane's 8 items + 1
    (2, 32, 2, 1, 700, None, True),        # 16 channels per group: dB / dC summed per workgroup in LDS
    (1, 60, 2, 2, 300, None, True),        # 30 channels per group in two chunks of 15, two states
    (1, 27, 1, 1, 520, 9, True),           # 27 channels in chunks of 14 + 13, delta rows shared by three channels
    (1, 24, 1, 1, 3136, None, True),       # one state, 7 passes, 6 channels per wavefront (pass-major kernel)
    (2, 10, 1, 1, 100, None, False),       # the same kernel without softplus, wavefronts with 3 and 2 channels
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_scan_bwd_fp32_against_float64_autograd(case):
    batch, dim, G, N, L, delta_dim, softplus = case
    print("CASE scan-bwd", case, flush=True)
    u, delta, A, B, C, D, bias, dout = make(sum(map(int, case[:5])), batch, dim, G, N, L, torch.float32, delta_dim, softplus)
    want = torch_ref.selective_scan_grads(u, delta, A, B, C, D, bias, dout, softplus)
    dev = [t.to(DEV) for t in (u, delta, A, B, C, D, bias, dout)]
    got = va.selective_scan_bwd(*dev, None, softplus, 1)
    torch.cuda.synchronize()
    compare(got, want, 2e-3, "abi")
    # optional arguments absent
    want2 = torch_ref.selective_scan_grads(u, delta, A, B, C, None, None, dout, softplus if softplus else False)
    got2 = va.selective_scan_bwd(dev[0], dev[1], dev[2], dev[3], dev[4], None, None, dev[7], None, softplus, 1)
    compare(got2, want2, 2e-3, "no D / bias")


@pytest.mark.parametrize("dim,G", [(8, 4), (16, 1)], ids=["rows", "grouped"])
@pytest.mark.parametrize("dtype,dout_float", [(torch.bfloat16, True), (torch.bfloat16, False), (torch.float16, True)])
def test_scan_bwd_16bit_inputs(dtype, dout_float, dim, G):
    print("CASE scan-bwd-16", dtype, dout_float, dim, G, flush=True)
    u, delta, A, B, C, D, bias, dout = make(5, 2, dim, G, 1, 1200, dtype)
    dout = dout if dout_float else dout.to(dtype)
    want = torch_ref.selective_scan_grads(u.float(), delta.float(), A, B.float(), C.float(), D, bias, dout.float(), True)
    got = va.selective_scan_bwd(*[t.to(DEV) for t in (u, delta, A, B, C, D, bias, dout)], None, True, 1)
    assert got[0].dtype == dtype and got[1].dtype == dtype and got[3].dtype == dtype and got[2].dtype == torch.float32
    compare(got, want, 3e-2, "16-bit")


def test_selective_scan_fn_trains():
    """autograd through selective_scan_fn (csms6s.py:112-126): gradients reach every input."""
    print("CASE scan-autograd", flush=True)
    u, delta, A, B, C, D, bias, dout = make(9, 2, 8, 4, 1, 640, torch.float32)
    want = torch_ref.selective_scan_grads(u, delta, A, B, C, D, bias, dout, True)
    leaves = [t.to(DEV).requires_grad_(True) for t in (u, delta, A, B, C, D, bias)]
    y = va.selective_scan_fn(*leaves, True, True)
    y.backward(dout.to(DEV))
    compare([t.grad for t in leaves], want, 2e-3, "autograd")


def test_scan_bwd_rejections():
    u, delta, A, B, C, D, bias, dout = [t.to(DEV) for t in make(1, 1, 4, 1, 1, 16, torch.float32)]
    with pytest.raises(RuntimeError):
        va.selective_scan_bwd(u, delta, A, B, C, D, bias, dout[:, :2], None, True, 1)
    with pytest.raises(RuntimeError):
        va.selective_scan_bwd(u, delta, A.double(), B, C, D, bias, dout, None, True, 1)
    with pytest.raises(RuntimeError):
        va.selective_scan_bwd(u.cpu(), delta, A, B, C, D, bias, dout, None, True, 1)
    p = _lib.ScanBwdParams()
    assert _lib.lib().ss2d_selective_scan_bwd(p, None) == _lib.SS2D_EINVAL           # dstate 0
    assert _lib.lib().ss2d_selective_scan_bwd(None, None) == _lib.SS2D_EINVAL
