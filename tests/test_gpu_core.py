"""GPU parity of the fused SS2D core (CrossScan -> selective scan -> CrossMerge in one kernel) and of the
one-by-one CrossScan, through the C ABI, against the CPU oracle's composition of the three operators.

Tolerance: the scan bound (fp32 output: rtol 1e-3) with an absolute floor of 4e-4 -- the merged value is a sum of
four scan outputs, each good to atol 1e-4.
"""
import pytest
import torch

from oracle import ss2d_oracle as orc
from oracle import torch_ref
import vmamba_amd as va
from vmamba_amd import _lib
from vmamba_amd.core import ss2d_core_hip
from vmamba_amd.csm import cross_scan_1b1_hip

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = dict(rtol=1e-3, atol=4e-4)


def _announce(*what):
    print("CASE", *what, flush=True)


def make_core_inputs(seed, B, D, H, W, dtype):
    g = torch.Generator().manual_seed(seed)
    L = H * W
    dt = torch.exp(torch.rand(4 * D, generator=g) * (torch.log(torch.tensor(0.1)) - torch.log(torch.tensor(1e-3)))
                   + torch.log(torch.tensor(1e-3)))
    bias = dt + torch.log(-torch.expm1(-dt))
    A = -(0.5 + torch.rand(4 * D, generator=g))
    Dv = torch.randn(4 * D, generator=g)
    x = torch.randn(B, D, H, W, generator=g).to(dtype)
    delta = torch.randn(4, D, B, L, generator=g).to(dtype)
    Bs = torch.randn(4, B, L, generator=g).to(dtype)
    Cs = torch.randn(4, B, L, generator=g).to(dtype)
    return x, delta, Bs, Cs, A, Dv, bias


def oracle_core(x, delta, Bs, Cs, A, Dv, bias, softplus=True):
    """cross_scan -> selective_scan (fp32 out) -> cross_merge, each the CPU oracle's."""
    B, D, H, W = x.shape
    L = H * W
    xs = orc.cross_scan(x)                                                    # (B, 4, D, L)
    ys = orc.selective_scan(xs.reshape(B, 4 * D, L), delta.permute(2, 0, 1, 3).reshape(B, 4 * D, L).contiguous(),
                            A.view(4 * D, 1), Bs.permute(1, 0, 2).unsqueeze(2).contiguous(),
                            Cs.permute(1, 0, 2).unsqueeze(2).contiguous(), Dv, bias, softplus, out_float=True)
    return orc.cross_merge(ys.view(B, 4, D, H, W))                            # (B, D, L) fp32, pairwise order


def run_core(x, delta, Bs, Cs, A, Dv, bias, softplus=True):
    dev = lambda t: None if t is None else t.to(DEV)
    y = ss2d_core_hip(dev(x), dev(delta), dev(Bs), dev(Cs), dev(A), dev(Dv), dev(bias), softplus)
    torch.cuda.synchronize()
    return y.cpu()


CORE_SHAPES = [
    (2, 3, 56, 56),      # one image per workgroup, 8-wide B/C groups
    (5, 4, 28, 28),      # several images per workgroup + a shorter last tile
    (18, 2, 14, 14),     # L % 8 == 4: an even number of images per workgroup
    (19, 1, 14, 14),     # ... and a last tile of odd length: its final 16-byte delta load runs past the tensor's end
    (5, 2, 14, 14),      # one tile whose length is not a multiple of 8
    (70, 2, 7, 7),       # odd L: many images per workgroup, element-wise B/C gathers
    (8, 2, 14, 14),      # 3 full passes + 32 positions walked one per lane
    (21, 1, 7, 7),       # 2 full passes + 5 positions
    (3, 2, 4, 4),        # rows shorter than a block of 8 (element-wise staging), 16-byte merge stores
    (2, 2, 8, 2),        # rows shorter than 4
    (2, 2, 2, 8),
    (3, 2, 7, 9),        # H != W, odd L
    (2, 2, 10, 12),      # H != W
    (9, 1, 6, 5),        # L = 30: two-element granularity handled element-wise
    (1, 1, 3, 3),        # smallest supported image
    (1, 2, 64, 48),      # L = 3072
    # 7 x 7 and 14 x 14 maps whose streams start on 16-byte boundaries take the row-per-lane kernel (16-bit inputs):
    (16, 5, 7, 7),       # two tiles of 8 maps; channels not a multiple of the 4 per workgroup
    (24, 3, 7, 7),       # three tiles, three channels (one wavefront of the workgroup has no channel)
    (40, 8, 7, 7),
    (6, 5, 14, 14),      # tiles of 4 maps, the last one half full
    (2, 1, 14, 14),      # a single, half-full tile
    (12, 4, 14, 14),
    # maps whose LDS arrays take more than a third of a CU's 160 KB (two workgroups per CU, then one): up to ~13 000 positions
    (1, 2, 80, 80),      # 78 KB
    (2, 1, 76, 76),      # sides multiples of 4 only
    (1, 2, 96, 96),      # 113 KB: one workgroup per CU
    (1, 1, 112, 112),    # 153 KB, the largest square map with sides multiples of 8
    (1, 2, 100, 128),    # 157 KB, H != W
    (1, 1, 75, 75),      # element-wise walk (an odd number of positions) at 69 KB
    (1, 1, 64, 200),     # 157 KB with fewer rows than columns
    # (above 53 KB two wavefronts per direction take alternate passes: 80 x 80 is 7 passes, 76 x 76 6, 96 x 96 9)
    (2, 2, 72, 72),      # 5 passes and 64 positions walked one per lane
    (1, 1, 32, 194),     # 6 passes and 64 positions; rows that are no multiple of 4
    (3, 1, 68, 68),      # 4 passes + a fifth of 528 positions; three images
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape", CORE_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_core_matches_oracle_composition(shape, dtype):
    from vmamba_amd.core import core_fits
    if not core_fits(shape[2], shape[3], dtype):
        pytest.skip("fp32 maps of this size are beyond the LDS arrays (and the tiled kernels take 16-bit inputs)")
    _announce("core", shape, dtype)
    args = make_core_inputs(sum(shape), *shape, dtype)
    want = oracle_core(*args)
    got = run_core(*args)
    assert got.dtype == torch.float32 and got.shape == want.shape
    err = (got - want).abs().max().item()
    assert torch.allclose(got, want, **TOL), f"max abs err {err}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("S", [7, 14, 9, 19])
@pytest.mark.parametrize("B", [1, 3, 5, 9, 11])
def test_core_small_maps_in_the_padded_batch_layout(B, S, dtype):
    """The layout SS2D.forward_core_fused hands over when batch * L is not a multiple of the 16-byte vector: delta
    (4, D, Bp, L) and the projection rows (4, R + 2, Bp, L) with room for Bp >= B images, sliced to the first B.  This is
    how the row-per-lane kernel meets a short last tile of an ODD number of 7 x 7 maps, and the general kernel a
    16-byte-aligned stream of odd maps (9 x 9, 19 x 19) that ends in the middle of a 16-byte vector: the last
    elements of such a stream must arrive although the vector that holds them reaches past the stream's extent.
    Every image against the oracle."""
    _announce("core padded batch", B, S, dtype)
    D, L, R = 5, S * S, 3
    unit = 8 // __import__("math").gcd(L, 8)
    Bp = (B + unit - 1) // unit * unit
    x, delta, Bs, Cs, A, Dv, bias = make_core_inputs(100 * B + S, B, D, S, S, dtype)
    delta_buf = torch.zeros(4, D, Bp, L, dtype=dtype)
    x_dbl = torch.zeros(4, R + 2, Bp, L, dtype=dtype)
    delta_buf[:, :, :B] = delta
    x_dbl[:, R, :B], x_dbl[:, R + 1, :B] = Bs, Cs
    want = oracle_core(x, delta, Bs, Cs, A, Dv, bias)
    dbuf, xbuf = delta_buf.to(DEV), x_dbl.to(DEV)
    dview, bview, cview = dbuf[:, :, :B], xbuf[:, R, :B], xbuf[:, R + 1, :B]
    assert dview.stride() == (D * Bp * L, Bp * L, L, 1) and bview.stride() == ((R + 2) * Bp * L, L, 1)
    got = ss2d_core_hip(x.to(DEV), dview, bview, cview, A.to(DEV), Dv.to(DEV), bias.to(DEV), True)
    torch.cuda.synchronize()
    err = (got.cpu() - want).abs().max().item()
    assert torch.allclose(got.cpu(), want, **TOL), f"max abs err {err}"
    # the last image's last positions in every direction's order are where a dropped stream element would show
    assert torch.allclose(got.cpu()[B - 1, :, -S:], want[B - 1, :, -S:], **TOL)
    assert torch.allclose(got.cpu()[B - 1, :, :S], want[B - 1, :, :S], **TOL)


@pytest.mark.parametrize("B", [1, 3, 9])
def test_core_small_maps_contiguous_streams_end_at_the_allocation(B):
    """7 x 7 maps, contiguous (4, D, B, L) streams whose last tile is short and odd and whose last element is the last
    element of the tensor: B / C rows of 8-element-aligned direction stride take the row-per-lane kernel only when
    B * L is a multiple of 8, so this runs the general kernel at odd B -- same bound, same inputs."""
    _announce("core contiguous odd batch", B)
    args = make_core_inputs(700 + B, B, 4, 7, 7, torch.bfloat16)
    want = oracle_core(*args)
    got = run_core(*args)
    assert torch.allclose(got, want, **TOL), f"max abs err {(got - want).abs().max().item()}"


# Maps that do not fit the single kernel's LDS arrays (more than ~13 000 positions): 64 x 64 tiles, walked twice with a carry
# scan in between (16-bit inputs, sides multiples of 8).  Whole tiles; edge tiles narrower / shorter than 64; a single row
# or column of tiles; maps with fewer than 64 rows; several images and channels.
TILED_SHAPES = [
    (1, 2, 128, 128), (2, 3, 144, 120), (1, 1, 64, 264), (1, 2, 256, 256), (2, 2, 8, 2048), (1, 2, 264, 64), (3, 1, 136, 120),
    (1, 1, 2000, 8),
]


def core_workspace_bytes(B, D, H, W, dtype=torch.bfloat16):
    """ss2d_core_workspace_bytes for dense, aligned tensors of these sizes (the query reads the struct only)."""
    p = _lib.CoreParams()
    p.batch, p.dim, p.height, p.width = B, D, H, W
    p.in_dtype = {torch.float32: _lib.SS2D_F32, torch.bfloat16: _lib.SS2D_BF16, torch.float16: _lib.SS2D_F16}[dtype]
    p.delta_softplus = 1
    p.x, p.delta, p.A, p.B, p.C, p.y = (4096 * k for k in range(1, 7))
    L = H * W
    p.delta_dir_stride, p.delta_dim_stride, p.delta_batch_stride = D * B * L, B * L, L
    p.B_dir_stride, p.B_batch_stride, p.C_dir_stride, p.C_batch_stride = B * L, L, B * L, L
    return _lib.lib().ss2d_core_workspace_bytes(p)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("shape", TILED_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_core_large_maps_in_tiles_match_oracle_composition(shape, dtype):
    _announce("core tiled", shape, dtype)
    assert core_workspace_bytes(*shape, dtype) > 0            # the two-pass path, not the single kernel
    args = make_core_inputs(sum(shape), *shape, dtype)
    want = oracle_core(*args)
    got = run_core(*args)
    assert got.dtype == torch.float32 and got.shape == want.shape
    # rows of up to 65536 positions: the absolute part scales with the output (the state remembers ~1 / (dt |A|) steps)
    tol = dict(rtol=1e-3, atol=max(4e-4, 2e-5 * want.abs().max().item()))
    err = (got - want).abs().max().item()
    assert torch.allclose(got, want, **tol), f"max abs err {err}"


def test_core_tiled_optional_arguments_and_workspace_contract():
    _announce("core tiled optional")
    x, delta, Bs, Cs, A, Dv, bias = make_core_inputs(77, 2, 2, 136, 128, torch.bfloat16)
    g = torch.Generator().manual_seed(3)
    delta_pos = (0.5 * torch.rand(delta.shape, generator=g)).to(delta.dtype)
    bias_pos = 0.5 * torch.rand(bias.shape, generator=g)
    for dl, dv, bi, sp in ((delta, None, bias, True), (delta, Dv, None, True), (delta_pos, Dv, bias_pos, False), (delta_pos, None, None, False)):
        want = oracle_core(x, dl, Bs, Cs, A, dv, bi, sp)
        got = run_core(x, dl, Bs, Cs, A, dv, bi, sp)
        assert torch.allclose(got, want, **TOL), f"max abs err {(got - want).abs().max().item()}"
    # the workspace contract of the C ABI: 0 for maps the single kernel takes, a refusal where neither path applies,
    # SS2D_ENOMEM for a workspace that is too small, and the plain entry point still refuses large maps
    assert core_workspace_bytes(4, 8, 56, 56) == 0
    assert core_workspace_bytes(1, 1, 112, 112) == 0                          # 153 KB of LDS: still the single kernel
    assert core_workspace_bytes(1, 1, 129, 129) == _lib.SS2D_ENOTSUP          # sides not multiples of 8
    assert core_workspace_bytes(1, 1, 128, 128, torch.float32) == _lib.SS2D_ENOTSUP
    need = core_workspace_bytes(2, 2, 136, 128)
    assert need == 4 * 2 * 2 * max(136 * 2, 128 * 3) * 12
    dev = [t.to(DEV) for t in (x, delta, Bs, Cs, A, Dv, bias)]
    y = torch.empty(2, 2, 136 * 128, device=DEV)
    p = _lib.CoreParams()
    p.batch, p.dim, p.height, p.width, p.in_dtype, p.delta_softplus = 2, 2, 136, 128, _lib.SS2D_BF16, 1
    p.x, p.delta, p.B, p.C, p.A, p.D, p.delta_bias, p.y = (t.data_ptr() for t in dev + [y])
    p.delta_dir_stride, p.delta_dim_stride, p.delta_batch_stride = dev[1].stride(0), dev[1].stride(1), dev[1].stride(2)
    p.B_dir_stride, p.B_batch_stride, p.C_dir_stride, p.C_batch_stride = dev[2].stride(0), dev[2].stride(1), dev[3].stride(0), dev[3].stride(1)
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    assert _lib.lib().ss2d_core_fwd(p, stream) == _lib.SS2D_ENOTSUP
    assert _lib.lib().ss2d_core_fwd_ws(p, ws.data_ptr(), need - 1, stream) == _lib.SS2D_ENOMEM
    assert _lib.lib().ss2d_core_fwd_ws(p, None, need, stream) == _lib.SS2D_EINVAL
    assert _lib.lib().ss2d_core_fwd_ws(p, ws.data_ptr(), need, stream) == _lib.SS2D_OK
    torch.cuda.synchronize()
    assert torch.allclose(y.cpu(), oracle_core(x, delta, Bs, Cs, A, Dv, bias), **TOL)


# (n_maps, source rows, cols, destination rows, cols): embeddings and crops through every copy variant -- rows of whole
# 16-byte vectors on both sides (channel-last crops), a destination of whole vectors with ragged rows (75 -> 80, 19 -> 20,
# crops whose total size is a multiple of the vector), 4-byte pairs (57 x 58 -> 60 x 60 with an odd number of maps), single
# elements, growth in one direction only, rows and columns at once
EMBED_CASES = [(6, 57, 58, 60, 60), (3, 57, 58, 60, 60), (8, 75, 75, 80, 80), (5, 19, 19, 20, 20), (1, 20, 20, 19, 19),
               (4, 60, 60 * 96, 57, 58 * 96), (8, 60, 60, 57, 58), (3, 60, 60, 57, 58), (1, 3, 3, 5, 5), (7, 9, 13, 12, 16),
               (2, 8, 8, 8, 16), (2, 8, 16, 16, 16), (3, 5, 8, 8, 4), (2, 1, 1, 1, 1), (1, 200, 334, 200, 336)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("case", EMBED_CASES, ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("offset", [0, 1], ids=["aligned", "shifted"])
def test_embed_maps_pads_with_zeros_and_crops(case, dtype, offset):
    """ss2d_core_embed_maps against slicing and zero-filling in torch, bit for bit; with a source that starts one element
    into its allocation as well (no 16-byte alignment)."""
    from vmamba_amd.core import embed_maps_hip
    n, sr, sc, dr, dc = case
    print("CASE embed", case, dtype, offset, flush=True)
    g = torch.Generator().manual_seed(sum(case))
    src = torch.randn((n, sr, sc), generator=g).to(dtype)
    want = torch.zeros((n, dr, dc), dtype=dtype)
    want[:, :min(sr, dr), :min(sc, dc)] = src[:, :min(sr, dr), :min(sc, dc)]
    buf = torch.empty(src.numel() + offset, dtype=dtype, device=DEV)
    dev_src = buf[offset:].view(n, sr, sc)
    dev_src.copy_(src)
    got = embed_maps_hip(dev_src, dr, dc)
    torch.cuda.synchronize()
    assert got.shape == want.shape and torch.equal(got.cpu().view(torch.uint8), want.view(torch.uint8))


def test_embed_maps_rejects_what_it_cannot_address():
    L = _lib.lib()
    x = torch.zeros(64, dtype=torch.int16, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    assert L.ss2d_core_embed_maps(x.data_ptr(), x.data_ptr(), 1, 2, 2, 2, 2, 1, stream) == _lib.SS2D_EINVAL      # 1-byte elements
    assert L.ss2d_core_embed_maps(None, x.data_ptr(), 1, 2, 2, 2, 2, 2, stream) == _lib.SS2D_EINVAL
    assert L.ss2d_core_embed_maps(x.data_ptr(), x.data_ptr(), 1 << 20, 1 << 10, 1 << 10, 1 << 10, 1 << 10, 2, stream) == _lib.SS2D_ENOTSUP
    assert L.ss2d_core_embed_maps(x.data_ptr(), x.data_ptr(), 0, 2, 2, 2, 2, 2, stream) == _lib.SS2D_OK          # nothing to do


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "f16", "f32"])
@pytest.mark.parametrize("sizes", [(57, 58, 60, 60), (19, 19, 20, 20), (9, 13, 16, 16), (75, 75, 80, 80), (8, 8, 8, 16), (5, 3, 8, 8)],
                         ids=lambda s: "x".join(map(str, s)))
def test_core_mask_pads_marks_exactly_the_added_positions(sizes, dtype):
    """ss2d_core_mask_pads: -inf at the scan positions of every direction that fall on added rows / columns, nothing else
    touched.  The expected positions come from the oracle's CrossScan applied to a 0 / 1 picture of the padded map."""
    from vmamba_amd.core import core_mask_pads_hip
    H, W, Hp, Wp = sizes
    _announce("mask pads", sizes, dtype)
    D, B = 3, 2
    g = torch.Generator().manual_seed(H * W)
    delta = torch.randn(4, D, B + 1, Hp * Wp, generator=g).to(dtype)          # a batch-padded buffer, sliced
    picture = torch.ones(1, 1, Hp, Wp)
    picture[:, :, :H, :W] = 0
    marks = orc.cross_scan(picture).view(4, Hp * Wp).bool()                   # (direction, scan position): added or not
    dev = delta.to(DEV)
    core_mask_pads_hip(dev[:, :, :B], H, W, Hp, Wp)
    torch.cuda.synchronize()
    got = dev.cpu()
    want = delta.clone()
    want[:, :, :B] = torch.where(marks[:, None, None, :], torch.tensor(float("-inf")).to(dtype), delta[:, :, :B])
    assert torch.equal(got.view(torch.int16 if dtype != torch.float32 else torch.int32),
                       want.view(torch.int16 if dtype != torch.float32 else torch.int32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("shape,padded", [((3, 2, 57, 58), (60, 60)), ((5, 3, 19, 19), (20, 20)), ((2, 2, 75, 75), (76, 76)),
                                          ((2, 1, 25, 42), (28, 44)), ((1, 2, 100, 167), (104, 168)), ((1, 2, 123, 125), (128, 128))],
                         ids=lambda v: "x".join(map(str, v)))
def test_core_on_a_padded_map_equals_the_oracle_on_the_map_itself(shape, padded, dtype):
    """The embedding SS2D.forward_core_fused uses for maps with awkward sides: x zero-padded, the streams given on the
    padded map (B, C arbitrary on the added positions, delta -inf there through ss2d_core_mask_pads), the result cropped
    -- against the oracle's composition on the ORIGINAL map with the original streams."""
    from vmamba_amd.core import core_mask_pads_hip, padded_map_size
    B, D, H, W = shape
    Hp, Wp = padded
    assert padded_map_size(H, W, dtype) == padded
    _announce("core padded map", shape, padded, dtype)
    g = torch.Generator().manual_seed(sum(shape))
    # streams on the padded map, in natural (h, w) order first: (4, rows, B, Hp, Wp); the original map's streams are the crops
    nat = lambda rows: torch.randn(4, rows, B, Hp, Wp, generator=g).to(dtype)
    delta_nat, B_nat, C_nat = nat(D), nat(1), nat(1)
    x, _, _, _, A, Dv, bias = make_core_inputs(sum(shape), B, D, H, W, dtype)

    def in_scan_order(t, h, w):          # (4, rows, B, h, w) natural -> each direction slice in its own order: (4, rows, B, h*w)
        rows = t.shape[1]
        return torch_ref.cross_scan_1b1(t.permute(2, 0, 1, 3, 4).contiguous()).permute(1, 2, 0, 3).reshape(4, rows, B, h * w).contiguous()

    crop = lambda t: t[..., :H, :W].contiguous()
    want = oracle_core(x, in_scan_order(crop(delta_nat), H, W), in_scan_order(crop(B_nat), H, W)[:, 0],
                       in_scan_order(crop(C_nat), H, W)[:, 0], A, Dv, bias)
    x_pad = torch.nn.functional.pad(x, (0, Wp - W, 0, Hp - H))
    delta_p = in_scan_order(delta_nat, Hp, Wp).to(DEV)
    core_mask_pads_hip(delta_p, H, W, Hp, Wp)
    got = ss2d_core_hip(x_pad.to(DEV), delta_p, in_scan_order(B_nat, Hp, Wp)[:, 0].to(DEV), in_scan_order(C_nat, Hp, Wp)[:, 0].to(DEV),
                        A.to(DEV), Dv.to(DEV), bias.to(DEV), True)
    torch.cuda.synchronize()
    got = got.view(B, D, Hp, Wp)[:, :, :H, :W].reshape(B, D, H * W).cpu()
    tol = dict(rtol=1e-3, atol=max(4e-4, 2e-5 * want.abs().max().item()))
    assert torch.allclose(got, want, **tol), f"max abs err {(got - want).abs().max().item()}"


def test_core_tiled_equals_three_kernels_at_config4_shapes():
    """The stage-1 and stage-2 maps of four 1024 x 1024 images (256 x 256 and 128 x 128), full size: the tiled kernels
    against this package's own cross_scan / scan / merge kernels, which the oracle pins at smaller sizes."""
    for (B, D, H, W) in ((4, 96, 256, 256), (4, 192, 128, 128)):
        _announce("core tiled vs kernels", B, D, H, W)
        x, delta, Bs, Cs, A, Dv, bias = [t.to(DEV) for t in make_core_inputs(B + D, B, D, H, W, torch.bfloat16)]
        L = H * W
        xs = va.cross_scan_fn(x)
        ys = va.selective_scan_fn(xs.view(B, 4 * D, L), delta.permute(2, 0, 1, 3).reshape(B, 4 * D, L), A.view(4 * D, 1),
                                  Bs.permute(1, 0, 2).unsqueeze(2), Cs.permute(1, 0, 2).unsqueeze(2), Dv, bias, True, True)
        want = va.cross_merge_fn(ys.view(B, 4, D, H, W))
        got = ss2d_core_hip(x, delta, Bs, Cs, A, Dv, bias, True)
        torch.cuda.synchronize()
        tol = dict(rtol=1e-3, atol=max(4e-4, 2e-5 * want.abs().max().item()))
        err = (got - want).abs().max().item()
        assert torch.allclose(got, want, **tol), f"max abs err {err}"


@pytest.mark.parametrize("softplus", [True, False])
def test_core_optional_arguments(softplus):
    _announce("core optional", softplus)
    x, delta, Bs, Cs, A, Dv, bias = make_core_inputs(11, 6, 3, 14, 14, torch.bfloat16)
    if not softplus:        # delta + bias is the step itself: keep it positive (the reference's own test ranges)
        g = torch.Generator().manual_seed(3)
        delta = (0.5 * torch.rand(delta.shape, generator=g)).to(delta.dtype)
        bias = 0.5 * torch.rand(bias.shape, generator=g)
    for dv, bi in ((None, bias), (Dv, None), (None, None)):
        want = oracle_core(x, delta, Bs, Cs, A, dv, bi, softplus)
        got = run_core(x, delta, Bs, Cs, A, dv, bi, softplus)
        assert torch.allclose(got, want, **TOL), f"max abs err {(got - want).abs().max().item()}"


def test_core_into_caller_buffer_not_16_byte_aligned():
    """The result may land anywhere a float can: the kernel then stores element by element."""
    _announce("core unaligned out")
    x, delta, Bs, Cs, A, Dv, bias = make_core_inputs(5, 3, 2, 28, 28, torch.bfloat16)
    want = oracle_core(x, delta, Bs, Cs, A, Dv, bias)
    dev = lambda t: t.to(DEV)
    buf = torch.full((want.numel() + 5,), 7.0, device=DEV)
    out = buf[1:1 + want.numel()].view(want.shape)
    assert out.data_ptr() % 16 == 4
    got = ss2d_core_hip(dev(x), dev(delta), dev(Bs), dev(Cs), dev(A), dev(Dv), dev(bias), True, out=out)
    torch.cuda.synchronize()
    assert got.data_ptr() == out.data_ptr()
    assert torch.allclose(got.cpu(), want, **TOL)
    assert buf[0].item() == 7.0 and torch.all(buf[1 + want.numel():] == 7.0)


def test_core_reference_layout_strides():
    """delta (B,4,D,L) and B/C (B,4,1,L) as the reference's projections lay them out, passed as permuted views:
    one image per workgroup, same result."""
    _announce("core strided")
    x, delta, Bs, Cs, A, Dv, bias = make_core_inputs(21, 5, 3, 28, 28, torch.bfloat16)
    want = oracle_core(x, delta, Bs, Cs, A, Dv, bias)
    dev = lambda t: t.to(DEV)
    delta_ref = dev(delta).permute(2, 0, 1, 3).contiguous()            # (B, 4, D, L)
    B_ref = dev(Bs).permute(1, 0, 2).contiguous()                     # (B, 4, L)
    C_ref = dev(Cs).permute(1, 0, 2).contiguous()
    got = ss2d_core_hip(dev(x), delta_ref.permute(1, 2, 0, 3), B_ref.permute(1, 0, 2), C_ref.permute(1, 0, 2), dev(A), dev(Dv),
                        dev(bias), True)
    torch.cuda.synchronize()
    assert torch.allclose(got.cpu(), want, **TOL)
    same = run_core(x, delta, Bs, Cs, A, Dv, bias)
    assert torch.allclose(got.cpu(), same, rtol=1e-5, atol=1e-6)      # both layouts: same arithmetic per image


def test_core_equals_three_kernels_at_model_shape():
    """Full stage shapes: the fused kernel against this package's own cross_scan / scan / merge kernels (which the
    oracle pins at smaller sizes)."""
    for (B, D, H, W) in ((16, 96, 56, 56), (16, 192, 28, 28), (32, 384, 14, 14), (128, 768, 7, 7)):
        _announce("core vs kernels", B, D, H, W)
        x, delta, Bs, Cs, A, Dv, bias = [None if t is None else t.to(DEV) for t in make_core_inputs(B + D, B, D, H, W, torch.bfloat16)]
        L = H * W
        xs = va.cross_scan_fn(x)
        ys = va.selective_scan_fn(xs.view(B, 4 * D, L), delta.permute(2, 0, 1, 3).reshape(B, 4 * D, L), A.view(4 * D, 1),
                                  Bs.permute(1, 0, 2).unsqueeze(2), Cs.permute(1, 0, 2).unsqueeze(2), Dv, bias, True, True)
        want = va.cross_merge_fn(ys.view(B, 4, D, H, W))
        got = ss2d_core_hip(x, delta, Bs, Cs, A, Dv, bias, True)
        torch.cuda.synchronize()
        err = (got - want).abs().max().item()
        assert torch.allclose(got, want, **TOL), f"max abs err {err}"


# Benchmark configurations 1 and 2 at their own batch: the fused kernel picks its tile (images per workgroup) from the
# batch -- 1 / 2 / 10 / 40 images at the four stage shapes, with a shorter last tile of 8 at the last two -- so the
# tiles the benchmark runs only exist at B = 128.  Image ranges below cover the first tile, an interior tile and the
# last (short) tile of every shape, and more than one tile where tiles are small.
BENCH_TILES = [
    ((128, 96, 56, 56), [(0, 2), (64, 66), (126, 128)]),
    ((128, 192, 28, 28), [(0, 4), (62, 66), (124, 128)]),
    ((128, 384, 14, 14), [(0, 10), (60, 70), (118, 128)]),
    ((128, 768, 7, 7), [(0, 40), (40, 80), (118, 128)]),
]


@pytest.mark.parametrize("shape,ranges", BENCH_TILES, ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else None)
def test_core_matches_oracle_at_benchmark_batch(shape, ranges):
    """bf16, B = 128: the fused kernel against the CPU oracle's composition on whole tiles of images."""
    B, D, H, W = shape
    L = H * W
    _announce("core bench-batch", shape)
    g = torch.Generator(device=DEV).manual_seed(B + D + H)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV)
    x, delta = rn(B, D, H, W).bfloat16(), rn(4, D, B, L).bfloat16()
    Bs, Cs = rn(4, B, L).bfloat16(), rn(4, B, L).bfloat16()
    _, _, _, _, A, Dv, bias = make_core_inputs(B + D, 1, D, 2, 4, torch.bfloat16)       # the per-channel constants
    got = ss2d_core_hip(x, delta, Bs, Cs, A.to(DEV), Dv.to(DEV), bias.to(DEV), True)
    torch.cuda.synchronize()
    assert got.shape == (B, D, L) and got.dtype == torch.float32
    for b0, b1 in ranges:
        want = oracle_core(x[b0:b1].cpu(), delta[:, :, b0:b1].cpu().contiguous(), Bs[:, b0:b1].cpu().contiguous(),
                           Cs[:, b0:b1].cpu().contiguous(), A, Dv, bias)
        err = (got[b0:b1].cpu() - want).abs().max().item()
        assert torch.allclose(got[b0:b1].cpu(), want, **TOL), f"images {b0}..{b1 - 1}: max abs err {err}"


def test_benchmark_config0_three_operators_and_fused_core():
    """Benchmark config 0 verbatim: fp32, x (2, 96, 56, 56) ~ N(0,1) -> CrossScan -> u (2, 384, 3136); delta_raw ~ N(0,1);
    dt log-uniform in [1e-3, 0.1], delta_bias = softplus^-1(dt); A = -exp(log 1) = -1; B, C (2, 4, 1, 3136) ~ N(0,1);
    D = 1; selective scan with softplus; CrossMerge back to (2, 96, 3136).  Both GPU paths against the CPU oracle
    (tolerances of kernels/selective_scan/test_selective_scan.py:401-403, fp32: rtol 1e-3; the permutation bit-exact,
    the merge bit-exact on the GPU's own scan output)."""
    import math
    _announce("config0")
    Bsz, Dn, H, W, K, N = 2, 96, 56, 56, 4, 1
    L = H * W
    g = torch.Generator().manual_seed(0)
    x = torch.randn(Bsz, Dn, H, W, generator=g)
    delta = torch.randn(Bsz, K * Dn, L, generator=g)
    dt = torch.exp(torch.rand(K * Dn, generator=g) * (math.log(0.1) - math.log(1e-3)) + math.log(1e-3))
    bias = dt + torch.log(-torch.expm1(-dt))
    A = -torch.exp(torch.log(torch.arange(1, N + 1, dtype=torch.float32))).repeat(K * Dn, 1)
    Bm, Cm = torch.randn(Bsz, K, N, L, generator=g), torch.randn(Bsz, K, N, L, generator=g)
    Dv = torch.ones(K * Dn)
    # CPU oracle
    xs_ref = orc.cross_scan(x)
    ys_ref = orc.selective_scan(xs_ref.view(Bsz, K * Dn, L), delta, A, Bm, Cm, Dv, bias, True)
    y_ref = orc.cross_merge(ys_ref.view(Bsz, K, Dn, H, W))
    # the torch restatement agrees with the C oracle on this very input (two formulations, one answer)
    assert torch.equal(torch_ref.cross_scan(x), xs_ref)
    # GPU: three operators
    dev = lambda t: t.to(DEV)
    xs = va.cross_scan_fn(dev(x))
    ys = va.selective_scan_fn(xs.view(Bsz, K * Dn, L), dev(delta), dev(A), dev(Bm), dev(Cm), dev(Dv), dev(bias), True)
    y = va.cross_merge_fn(ys.view(Bsz, K, Dn, H, W))
    torch.cuda.synchronize()
    assert torch.equal(xs.cpu(), xs_ref)
    assert torch.allclose(ys.cpu(), ys_ref, rtol=1e-3, atol=1e-4), f"scan max abs err {(ys.cpu() - ys_ref).abs().max().item()}"
    assert torch.equal(y.cpu(), orc.cross_merge(ys.cpu().view(Bsz, K, Dn, H, W)))
    assert torch.allclose(y.cpu(), y_ref, **TOL)
    # GPU: the fused kernel, projections handed over direction-major and batch-innermost
    delta_k = delta.view(Bsz, K, Dn, L).permute(1, 2, 0, 3).contiguous()
    B_k, C_k = Bm.view(Bsz, K, L).permute(1, 0, 2).contiguous(), Cm.view(Bsz, K, L).permute(1, 0, 2).contiguous()
    y_fused = ss2d_core_hip(dev(x), dev(delta_k), dev(B_k), dev(C_k), dev(A.view(-1)), dev(Dv), dev(bias), True)
    torch.cuda.synchronize()
    err = (y_fused.cpu() - y_ref).abs().max().item()
    assert torch.allclose(y_fused.cpu(), y_ref, **TOL), f"fused core max abs err {err}"


def test_core_rejections():
    x, delta, Bs, Cs, A, Dv, bias = [t.to(DEV) for t in make_core_inputs(1, 2, 2, 4, 4, torch.bfloat16)]
    with pytest.raises(RuntimeError):
        ss2d_core_hip(x, delta[:, :, :1], Bs, Cs, A, Dv, bias)
    with pytest.raises(RuntimeError):
        ss2d_core_hip(x, delta.float(), Bs, Cs, A, Dv, bias)
    with pytest.raises(RuntimeError):
        ss2d_core_hip(x.cpu(), delta, Bs, Cs, A, Dv, bias)
    # image too large for the LDS planes with sides the tiled kernels do not take: a clean "not supported", never a launch
    big = [t.to(DEV) for t in make_core_inputs(1, 1, 1, 129, 129, torch.bfloat16)]
    with pytest.raises(_lib.Ss2dError) as e:
        ss2d_core_hip(*big)
    assert e.value.code == _lib.SS2D_ENOTSUP
    # images shorter than one lane's 8 positions
    tiny = [t.to(DEV) for t in make_core_inputs(1, 2, 2, 2, 2, torch.bfloat16)]
    with pytest.raises(_lib.Ss2dError) as e:
        ss2d_core_hip(*tiny)
    assert e.value.code == _lib.SS2D_ENOTSUP
    assert ss2d_core_hip(*[t.to(DEV) for t in make_core_inputs(1, 0, 2, 4, 4, torch.bfloat16)]).shape == (0, 2, 16)


# ---- one-by-one CrossScan ----------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.uint8, torch.float64], ids=str)
@pytest.mark.parametrize("shape", [(2, 3, 56, 56), (3, 5, 7, 9), (1, 2, 1, 17), (2, 1, 13, 1), (1, 1, 130, 100),
                                   (2, 6, 14, 14), (3, 2, 4, 6), (2, 3, 2, 1), (1, 5, 3, 10), (2, 2, 30, 27),
                                   (1, 2, 256, 256), (2, 1, 130, 197), (1, 1, 65, 400)],      # maps walked in 64 x 64 tiles
                         ids=lambda s: "x".join(map(str, s)))
def test_cross_scan_1b1_bit_exact(shape, dtype):
    _announce("cross_scan_1b1", shape, dtype)
    B, C, H, W = shape
    g = torch.Generator().manual_seed(B * 100 + C)
    x = (torch.randn(B, 4, C, H, W, generator=g) * 50).to(dtype)
    want = torch_ref.cross_scan_1b1(x)
    got = va.cross_scan_fn(x.to(DEV), one_by_one=True)
    torch.cuda.synchronize()
    assert torch.equal(got.cpu(), want)
    # direction-major, batch-innermost destination: same values through the strides
    buf = torch.full((4, C, B, H * W), 7, dtype=dtype, device=DEV)
    out = cross_scan_1b1_hip(x.to(DEV), out=buf.permute(2, 0, 1, 3))
    torch.cuda.synchronize()
    assert out.data_ptr() == buf.data_ptr()
    assert torch.equal(buf.permute(2, 0, 1, 3).cpu(), want)


def test_cross_scan_1b1_empty_and_bad_args():
    assert va.cross_scan_fn(torch.zeros(0, 4, 3, 4, 4, device=DEV), one_by_one=True).shape == (0, 4, 3, 16)
    with pytest.raises(ValueError):
        va.cross_scan_fn(torch.zeros(2, 3, 3, 4, 4, device=DEV), one_by_one=True)
    with pytest.raises(NotImplementedError):
        va.cross_scan_fn(torch.zeros(2, 4, 3, 4, 4), one_by_one=True)


# ---- dt_proj on the matrix cores -----------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("K,D,R,N", [(4, 96, 6, 2 * 3136), (4, 192, 12, 3 * 784), (4, 384, 24, 5 * 196), (4, 768, 48, 7 * 49),
                                     (2, 40, 3, 77), (1, 100, 17, 1000), (3, 33, 8, 32), (4, 8, 40, 5)])
def test_dt_proj_matches_fp32_matmul(K, D, R, N, dtype):
    """One rounding of an fp32-accumulated sum of exact 16-bit products: against the fp32 matmul of the same
    16-bit operands the result is within one rounding of the output type (plus fp32 summation-order noise)."""
    from vmamba_amd.core import dt_proj_hip
    _announce("dt_proj", K, D, R, N, dtype)
    g = torch.Generator().manual_seed(K * 1000 + D + R)
    x = torch.randn(K, R, N, generator=g).to(dtype)
    w = (torch.randn(K, D, R, generator=g) * R ** -0.5).to(dtype)
    want = torch.bmm(w.float(), x.float())
    got = dt_proj_hip(x.to(DEV), w.to(DEV))
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == (K, D, N)
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11          # half an ulp, relative
    err = (got.cpu().float() - want).abs()
    assert bool((err <= eps * want.abs() * 1.01 + 1e-6).all()), f"max err {err.max().item()}"
    # rows taken through strides: the dts slice of a (K, C, N) projection output
    C = R + 2
    x_dbl = torch.randn(K, C, N, generator=g).to(dtype).to(DEV)
    got2 = dt_proj_hip(x_dbl[:, :R], w.to(DEV))
    want2 = torch.bmm(w.float(), x_dbl[:, :R].cpu().float())
    err2 = (got2.cpu().float() - want2).abs()
    assert bool((err2 <= eps * want2.abs() * 1.01 + 1e-6).all())


@pytest.mark.parametrize("dtype,fill", [(torch.bfloat16, -1e30), (torch.float16, -65504.0), (torch.bfloat16, 0.25)],
                         ids=["bf16", "f16", "bf16-small"])
@pytest.mark.parametrize("K,D,R,N", [(4, 96, 6, 2 * 3600), (4, 384, 24, 5 * 400), (2, 40, 3, 77), (1, 100, 17, 1001), (3, 200, 8, 36)])
def test_dt_proj_masked_positions_take_the_fill_value(K, D, R, N, dtype, fill):
    """Marked positions hold the fill value in every channel, bit for bit; the others are the plain projection, bit for bit."""
    from vmamba_amd.core import dt_proj_hip
    _announce("dt_proj-masked", K, D, R, N, dtype, fill)
    g = torch.Generator().manual_seed(K * 1000 + D + R + 1)
    x = torch.randn(K, R, N, generator=g).to(dtype).to(DEV)
    w = (torch.randn(K, D, R, generator=g) * R ** -0.5).to(dtype).to(DEV)
    marked = torch.rand(K, N, generator=g) < 0.3
    marked[:, -1] = True                                                # the last position, in an odd-length tail too
    mask = (-marked.to(torch.int16)).to(DEV)
    plain = dt_proj_hip(x, w)
    got = dt_proj_hip(x, w, mask, fill)
    torch.cuda.synchronize()
    want = torch.where(marked.to(DEV)[:, None, :], torch.tensor(fill, dtype=dtype, device=DEV), plain)
    assert got.dtype == dtype and torch.equal(got.view(torch.int16), want.view(torch.int16))
    with pytest.raises(RuntimeError):
        dt_proj_hip(x, w, mask[:, :-1].contiguous(), fill)             # wrong shape
    with pytest.raises(RuntimeError):
        dt_proj_hip(x, w, mask.to(torch.int32), fill)                  # wrong type


def test_dt_proj_rejections():
    from vmamba_amd.core import dt_proj_hip
    with pytest.raises(RuntimeError):
        dt_proj_hip(torch.zeros(4, 6, 64, device=DEV), torch.zeros(4, 96, 6, device=DEV))              # fp32: library GEMM
    with pytest.raises(_lib.Ss2dError) as e:
        dt_proj_hip(torch.zeros(1, 64, 64, device=DEV, dtype=torch.bfloat16), torch.zeros(1, 8, 64, device=DEV, dtype=torch.bfloat16))
    assert e.value.code == _lib.SS2D_ENOTSUP
    assert dt_proj_hip(torch.zeros(4, 6, 0, device=DEV, dtype=torch.bfloat16),
                       torch.zeros(4, 96, 6, device=DEV, dtype=torch.bfloat16)).shape == (4, 96, 0)
