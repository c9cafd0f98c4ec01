"""CPU-only checks of the C ABI: the library loads, exports what include/ss2d_hip.h declares,
and validates arguments before touching the GPU (no kernel is launched here)."""
import ctypes
import os
import re

import pytest

from vmamba_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "ss2d_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ss2d_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    names = _declared_functions()
    assert set(names) == set(_lib.EXPORTS), names
    L = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(L, n), n


def test_version_and_strerror():
    assert _lib.lib().ss2d_abi_version() == _lib.ABI_VERSION
    text = open(os.path.join(ROOT, "include", "ss2d_hip.h")).read()
    assert f"#define SS2D_ABI_VERSION {_lib.ABI_VERSION}" in text
    assert _lib.strerror(0) == "ok"
    assert "invalid" in _lib.strerror(_lib.SS2D_EINVAL)
    assert "unknown" in _lib.strerror(12345)


def test_struct_layout_matches_header():
    # 10 int32 + 9 pointers + 14 int64, no padding surprises
    assert ctypes.sizeof(_lib.ScanParams) == 10 * 4 + 9 * 8 + 14 * 8
    assert _lib.ScanParams.u.offset == 40 and _lib.ScanParams.u_batch_stride.offset == 40 + 72


def test_cross_scan_argument_validation():
    L = _lib.lib()
    assert L.ss2d_cross_scan(None, None, 0, 3, 4, 4, 4, None) == _lib.SS2D_OK          # empty: no-op
    assert L.ss2d_cross_scan(None, None, 2, 3, 0, 4, 2, None) == _lib.SS2D_OK
    assert L.ss2d_cross_scan(None, None, 1, 1, 1, 1, 4, None) == _lib.SS2D_EINVAL      # null pointers
    assert L.ss2d_cross_scan(None, None, 1, 1, 1, 1, 3, None) == _lib.SS2D_EINVAL      # element size
    assert L.ss2d_cross_scan(None, None, -1, 1, 1, 1, 4, None) == _lib.SS2D_EINVAL


def test_cross_merge_argument_validation():
    L = _lib.lib()
    assert L.ss2d_cross_merge(None, None, 0, 3, 4, 4, _lib.SS2D_F32, 0, None) == _lib.SS2D_OK
    assert L.ss2d_cross_merge(None, None, 1, 1, 1, 1, _lib.SS2D_F32, 0, None) == _lib.SS2D_EINVAL
    assert L.ss2d_cross_merge(None, None, 1, 1, 1, 1, 7, 0, None) == _lib.SS2D_EINVAL   # dtype
    assert L.ss2d_cross_merge(None, None, 1, 1, 1, 1, _lib.SS2D_F32, 2, None) == _lib.SS2D_EINVAL  # order


def test_cross_scan_flex_workspace_validation():
    """ss2d_cross_scan_flex_ws: argument and workspace checks happen before anything is launched."""
    L = _lib.lib()
    ws = ctypes.c_void_p(256)       # never dereferenced: every call below is refused first
    mixed = (0, 1, 0, 0)            # x channel-first, y channel-last
    assert L.ss2d_cross_scan_flex_ws(None, None, 0, 3, 4, 4, 2, *mixed, None, 0, None) == _lib.SS2D_OK       # empty
    assert L.ss2d_cross_scan_flex_ws(None, None, 1, 3, 4, 4, 3, *mixed, ws, 1 << 20, None) == _lib.SS2D_EINVAL  # element size
    assert L.ss2d_cross_scan_flex_ws(None, None, 1, 3, 4, 4, 2, 0, 2, 0, 0, ws, 1 << 20, None) == _lib.SS2D_EINVAL  # flag
    assert L.ss2d_cross_scan_flex_ws(ws, ws, 1, 3, 4, 4, 2, *mixed, None, 1 << 20, None) == _lib.SS2D_EINVAL    # no workspace
    assert L.ss2d_cross_scan_flex_ws(ws, ws, 1, 3, 4, 4, 2, *mixed, ctypes.c_void_p(260), 1 << 20, None) == _lib.SS2D_EINVAL  # alignment
    need = 1 * 3 * 16 * 2
    assert L.ss2d_cross_scan_flex_ws(ws, ws, 1, 3, 4, 4, 2, *mixed, ws, need - 1, None) == _lib.SS2D_ENOMEM
    assert L.ss2d_cross_scan_flex_ws(ws, ws, 1, 3, 4, 4, 2, 0, 1, 1, 0, ws, 4 * need - 1, None) == _lib.SS2D_ENOMEM  # one-by-one: 4 slices
    assert "workspace" in _lib.strerror(_lib.SS2D_ENOMEM)


def test_scan_argument_validation():
    L = _lib.lib()
    assert L.ss2d_selective_scan_fwd(None, None) == _lib.SS2D_EINVAL
    p = _lib.ScanParams()
    p.batch, p.dim, p.seqlen, p.dstate, p.n_groups, p.delta_dim = 0, 8, 16, 1, 4, 8
    p.in_dtype, p.out_dtype = _lib.SS2D_BF16, _lib.SS2D_F32
    assert L.ss2d_selective_scan_fwd(p, None) == _lib.SS2D_OK               # empty batch
    p.batch = 2
    assert L.ss2d_selective_scan_fwd(p, None) == _lib.SS2D_EINVAL           # null pointers
    p.dstate = 257
    assert L.ss2d_selective_scan_fwd(p, None) == _lib.SS2D_EINVAL           # dstate > 256
    p.dstate, p.n_groups = 1, 3
    assert L.ss2d_selective_scan_fwd(p, None) == _lib.SS2D_EINVAL           # dim % n_groups
    p.n_groups, p.out_dtype = 4, _lib.SS2D_F16
    assert L.ss2d_selective_scan_fwd(p, None) == _lib.SS2D_EINVAL           # out dtype neither f32 nor input


def _scan_plan(batch, dim, L, N, G, in_dtype=_lib.SS2D_BF16, with_x=True, base=1 << 20):
    """ss2d_selective_scan_kernel for dense tensors of these sizes at made-up, 256-byte aligned addresses (the query
    reads the struct only)."""
    p = _lib.ScanParams()
    p.batch, p.dim, p.seqlen, p.dstate, p.n_groups, p.delta_dim = batch, dim, L, N, G, dim
    p.in_dtype, p.out_dtype, p.delta_softplus = in_dtype, _lib.SS2D_F32, 1
    p.u, p.delta, p.A, p.B, p.C, p.out = (base * k for k in range(1, 7))
    p.x = base * 7 if with_x else None
    p.u_batch_stride, p.u_d_stride = dim * L, L
    p.delta_batch_stride, p.delta_d_stride = dim * L, L
    p.A_d_stride, p.A_dstate_stride = N, 1
    p.B_batch_stride, p.B_group_stride, p.B_dstate_stride = G * N * L, N * L, L
    p.C_batch_stride, p.C_group_stride, p.C_dstate_stride = G * N * L, N * L, L
    p.out_batch_stride, p.out_d_stride = dim * L, L
    return _lib.lib().ss2d_selective_scan_kernel(p)


def test_scan_kernel_choice_does_not_depend_on_the_chunk_state_output():
    """The reference's extension interface always asks for the chunk states `x`
    (selective_scan_oflex.cpp:207-208): every benchmark shape must reach the same kernel with and without it."""
    shapes = {  # batch, dim = 4 * d_inner, L, N -> kernel
        (128, 384, 3136, 1): _lib.SCAN_KERNEL_ROW, (128, 768, 784, 1): _lib.SCAN_KERNEL_ROW,
        (128, 1536, 196, 1): _lib.SCAN_KERNEL_SMALL, (128, 3072, 49, 1): _lib.SCAN_KERNEL_SMALL,
        (64, 768, 3136, 16): _lib.SCAN_KERNEL_CHAN, (4, 384, 65536, 1): _lib.SCAN_KERNEL_ROW4,
        (4, 768, 16384, 1): _lib.SCAN_KERNEL_ROW, (48, 384, 3306, 1): _lib.SCAN_KERNEL_FLAT,
        (16, 384, 100, 1): _lib.SCAN_KERNEL_FLAT,
    }
    for (batch, dim, L, N), kernel in shapes.items():
        for with_x in (False, True):
            assert _scan_plan(batch, dim, L, N, 4, with_x=with_x) == kernel, (batch, dim, L, N, with_x)
    assert _scan_plan(0, 384, 3136, 1, 4) == _lib.SCAN_KERNEL_NONE
    assert _scan_plan(2, 384, 3136, 1, 5) == _lib.SS2D_EINVAL
    assert _lib.lib().ss2d_selective_scan_kernel(None) == _lib.SS2D_EINVAL
    assert len(_lib.SCAN_KERNEL_NAMES) == 6


def test_host_api_rejects_cpu_tensors_and_unsupported_modes():
    import torch
    import vmamba_amd as va
    x = torch.zeros(1, 2, 3, 3)
    with pytest.raises(NotImplementedError):
        va.cross_scan_fn(x)
    with pytest.raises(NotImplementedError):
        va.cross_merge_fn(torch.zeros(1, 4, 2, 3, 3))
    with pytest.raises(NotImplementedError):
        va.cross_scan_fn(x, scans=1)
    with pytest.raises(NotImplementedError):
        va.cross_scan_fn(x, force_torch=True)
    u = torch.zeros(1, 4, 8)
    with pytest.raises(RuntimeError):
        va.selective_scan_fn(u, u, torch.zeros(4, 1), torch.zeros(1, 4, 1, 8), torch.zeros(1, 4, 1, 8))
    with pytest.raises(NotImplementedError):
        va.selective_scan_fn(u, u, torch.zeros(4, 1), torch.zeros(1, 4, 1, 8), torch.zeros(1, 4, 1, 8), backend="torch")


def test_block_level_wrappers_have_no_cpu_path():
    """The harness-side kernels (fused MLP, narrow projection, LayerNorm variants, depthwise conv, fused core) raise on
    CPU tensors instead of computing anything there, and their 'fusable' predicates are False off the GPU."""
    import torch
    from vmamba_amd.conv import dwconv3x3_silu_hip
    from vmamba_amd.core import dt_proj_hip, ss2d_core_hip
    from vmamba_amd.linear import linear_cl_hip, linear_fusable
    from vmamba_amd.mlp import mlp_fusable, mlp_fused_hip
    from vmamba_amd.norm import add_layer_norm_fusable, add_layer_norm_hip, layer_norm_cf_hip, layer_norm_hip
    x = torch.zeros(4, 96, dtype=torch.bfloat16)
    w1, w2, w = torch.zeros(384, 96, dtype=torch.bfloat16), torch.zeros(96, 384, dtype=torch.bfloat16), torch.zeros(96, 96, dtype=torch.bfloat16)
    for call in (lambda: mlp_fused_hip(x, w1, None, w2, None), lambda: linear_cl_hip(x, w), lambda: layer_norm_hip(x, None, None),
                 lambda: add_layer_norm_hip(x, x, None, None), lambda: layer_norm_cf_hip(torch.zeros(1, 8, 4), None, None),
                 lambda: dwconv3x3_silu_hip(torch.zeros(1, 4, 4, 8), torch.zeros(8, 1, 3, 3), None, in_channel_last=True)):
        with pytest.raises(NotImplementedError):
            call()
    with pytest.raises(RuntimeError):
        ss2d_core_hip(torch.zeros(1, 2, 3, 3), torch.zeros(4, 2, 1, 9), torch.zeros(4, 1, 9), torch.zeros(4, 1, 9), torch.zeros(8))
    with pytest.raises(RuntimeError):
        dt_proj_hip(torch.zeros(4, 6, 8, dtype=torch.bfloat16), torch.zeros(4, 96, 6, dtype=torch.bfloat16))
    lin1, lin2 = torch.nn.Linear(96, 384).bfloat16(), torch.nn.Linear(384, 96).bfloat16()
    assert not mlp_fusable(x, lin1, lin2) and not linear_fusable(x, w) and not add_layer_norm_fusable(x, x)


def test_torch_extension_shim_loads_and_validates_on_cpu():
    import torch
    from vmamba_amd import oflex_ext
    ext = oflex_ext.load()
    assert hasattr(ext, "fwd") and hasattr(ext, "bwd")
    z = torch.zeros(1, 4, 8)
    with pytest.raises(RuntimeError):       # CPU tensors are refused before anything touches a GPU
        ext.fwd(z, z, torch.zeros(4, 1), torch.zeros(1, 4, 1, 8), torch.zeros(1, 4, 1, 8), None, None, True, 1, True)
