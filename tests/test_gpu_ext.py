"""The pybind shim `selective_scan_cuda_oflex`, called the way the reference calls it (csms6s.py:81)."""
import pytest
import torch

from oracle import ss2d_oracle as orc
from vmamba_amd import oflex_ext

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("dtype,L,N", [(torch.float32, 300, 1), (torch.bfloat16, 3136, 1), (torch.float16, 64, 16), (torch.bfloat16, 4500, 2)])
def test_fwd_matches_oracle_and_returns_chunk_states(dtype, L, N):
    print("CASE ext", dtype, L, N, flush=True)
    import selective_scan_cuda_oflex  # noqa: F401  resolved by install() in the fixture below
    g = torch.Generator().manual_seed(61)
    batch, dim, G = 2, 8, 4
    A = -0.5 * torch.rand(dim, N, generator=g)
    B, C = torch.randn(batch, G, N, L, generator=g).to(dtype), torch.randn(batch, G, N, L, generator=g).to(dtype)
    D, bias = torch.randn(dim, generator=g), 0.5 * torch.rand(dim, generator=g)
    u, delta = torch.randn(batch, dim, L, generator=g).to(dtype), (0.5 * torch.rand(batch, dim, L, generator=g)).to(dtype)
    dev = lambda t: t.to(DEV)
    out, x, *rest = selective_scan_cuda_oflex.fwd(dev(u), dev(delta), dev(A), dev(B), dev(C), dev(D), dev(bias), True, 1, True)
    want, xw = orc.selective_scan(u, delta, A, B, C, D, bias, True, return_x=True)
    assert out.dtype == torch.float32 and rest == []
    assert torch.allclose(out.cpu(), want, rtol=1e-3, atol=1e-4)
    assert x.shape == xw.shape
    last_state = x[:, :, -1, 1::2]                      # test_selective_scan.py:79
    assert torch.allclose(last_state.cpu(), xw[:, :, -1, 1::2], rtol=1e-3, atol=1e-4)
    out16, _ = selective_scan_cuda_oflex.fwd(dev(u), dev(delta), dev(A), dev(B), dev(C), None, None, False, 1, False)
    assert out16.dtype == dtype
    want16 = orc.selective_scan(u, delta, A, B, C, None, None, False, out_float=False)
    assert torch.allclose(out16.float().cpu(), want16.float(), rtol=2e-2, atol=2e-2)


@pytest.fixture(autouse=True, scope="module")
def _installed():
    oflex_ext.install()
    yield


def test_errors_are_runtime_errors():
    import selective_scan_cuda_oflex as ext
    u = torch.zeros(1, 4, 8, device=DEV)
    A = torch.zeros(4, 1, device=DEV)
    Bm = torch.zeros(1, 4, 1, 8, device=DEV)
    with pytest.raises(RuntimeError):
        ext.fwd(u, u.double(), A, Bm, Bm, None, None, True, 1, True)
    with pytest.raises(RuntimeError):
        ext.fwd(u, u, A, torch.zeros(1, 3, 1, 8, device=DEV), Bm, None, None, True, 1, True)
    with pytest.raises(RuntimeError):
        ext.fwd(u.cpu(), u.cpu(), A.cpu(), Bm.cpu(), Bm.cpu(), None, None, True, 1, True)
    with pytest.raises(RuntimeError):
        ext.bwd(u, u, A, Bm, Bm, None, None, u[:, :2], None, True, 1)           # dout shape


def test_bwd_matches_python_twin():
    """selective_scan_cuda_oflex.bwd (selective_scan_oflex.cpp:233-355) against vmamba_amd.selective_scan_bwd and
    the float64 autograd oracle, with channels sharing delta rows."""
    import selective_scan_cuda_oflex as ext
    import vmamba_amd as va
    from oracle import torch_ref
    g = torch.Generator().manual_seed(3)
    batch, dim, G, N, L, dd = 2, 8, 4, 2, 700, 4
    u = torch.randn(batch, dim, L, generator=g)
    delta = torch.randn(batch, dd, L, generator=g) - 1
    A = -0.5 * torch.rand(dim, N, generator=g) - 0.05
    Bm, Cm = torch.randn(batch, G, N, L, generator=g), torch.randn(batch, G, N, L, generator=g)
    D, bias, dout = torch.randn(dim, generator=g), torch.randn(dd, generator=g) - 1, torch.randn(batch, dim, L, generator=g)
    dev = [t.to(DEV) for t in (u, delta, A, Bm, Cm, D, bias, dout)]
    got = ext.bwd(*dev, None, True, 1)
    twin = va.selective_scan_bwd(*dev, None, True, 1)
    want = torch_ref.selective_scan_grads(u, delta, A, Bm, Cm, D, bias, dout, True)
    assert len(got) == 7
    for a, b, w in zip(got, twin, want):
        assert a.shape == b.shape == w.shape and a.dtype == b.dtype
        scale = w.abs().max().item()
        assert (a.double().cpu() - w).abs().max().item() <= 2e-3 * scale + 1e-6
        assert (a - b).abs().max().item() <= 1e-4 * scale + 1e-6            # same kernel; atomics reorder the sums
