// Selective-scan forward for SHORT rows and one state per channel: rows of 49 or 196 positions (the 7 x 7 and 14 x 14
// stages of a 224 x 224 VMamba), 16-bit u / delta / B / C, rows adjacent in memory.
//
// The flat kernel (selective_scan.hip) walks a run of such rows as one stream, 8 positions per lane, and pays for it in
// bookkeeping: rows start inside a lane's items, per-row constants are selected per group, B / C are gathered in pieces.
// Here a row of kNl * kNi positions occupies kNl lanes of a group of 8 or 16 lanes (the DPP row or half row), kNi
// consecutive positions per lane, 8 or 4 rows per wavefront:
//   * the wavefront's rows of u and delta are one contiguous block of memory: fetched with 16-byte loads, parked in LDS
//     as loaded and read back as per-lane runs; the B and C rows (one pair per tile: its rows belong to one image and
//     one group) go the same way; a wavefront walks two or four such tiles, the next one's loads in flight while one
//     is computed, and nothing is shared between wavefronts (no workgroup barrier);
//   * a lane scans its kNi items serially in registers, the lane totals are combined by a DPP scan over the DPP row of
//     16 lanes, and the state entering the lane is pushed through its items; the idle lanes behind a row's segments
//     enter that scan as the pair (0, 0), which stops anything on its way to the next group of the same DPP row;
//   * every index is a compile-time constant; the outputs go back through LDS (over the u / delta tiles) and leave as
//     16-byte stores of consecutive lanes, like the loads.
// Semantics: selective_scan_fn forward (classification/models/csms6s.py:25-68; kernel
// kernels/selective_scan/csrc/selective_scan/cusoflex/selective_scan_fwd_kernel_oflex.cuh:133-171) with d_state = 1.
#include "scan_common.h"

namespace ss2d {

// Tiles a wavefront walks, the next one's loads in flight while one is computed (more where a tile is smaller).
template <int kNl> constexpr int small_tiles() { return kNl <= 8 ? 4 : 2; }

// kX: the state at the end of every row is written too (rows are shorter than a 2048-position chunk, so that is the whole
// chunk-state output): x[row][0] = product of a over the row, x[row][1] = h at its last position.
template <typename in_t, typename out_t, int kNl, int kNi, bool kSoftplus, bool kX>
__global__ __launch_bounds__(kBlock) void scan_small_kernel(const ScanArgs p, int bc_vec, FastDiv div_dim, FastDiv div_dpg) {
    constexpr int kSmallTiles = small_tiles<kNl>();
    constexpr int kLanes = kNl <= 8 ? 8 : 16;                // lanes per row
    constexpr int kRows = kWave / kLanes;                    // rows per tile
    constexpr int kL = kNl * kNi;
    constexpr int kTileElems = kRows * kL;                   // a tile's rows, adjacent in memory
    constexpr int kTileVecs = kTileElems / 8;                // in 16-byte pieces
    constexpr int kVecsPerLane = (kTileVecs + kWave - 1) / kWave;
    constexpr int kRowPad = (kL + 7) & ~7;
    constexpr int kBcPerLane = (kL + kWave - 1) / kWave;     // element-wise B / C fetch
    static_assert(kTileElems % 8 == 0 && sizeof(in_t) == 2, "16-bit streams in whole 16-byte pieces");
    static_assert(kL % 4 != 0 || kL / 4 <= kWave, "a row in one 8-byte load per lane");
    // per wavefront: its u tile and its delta tile side by side -- together exactly the room of the fp32 output tile that
    // takes their place at the end of a tile
    __shared__ __align__(16) uint16_t s_ud[kWavesPerWg * 2 * kTileElems + kRunSlack];
    __shared__ __align__(16) uint16_t s_bc[kWavesPerWg * 2 * kRowPad + kRunSlack];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // (row indices fit 31 bits: the entry point refuses more rows)
    const int64_t row_first64 = ((int64_t)blockIdx.x * kWavesPerWg + wave) * (kSmallTiles * kRows);
    if (row_first64 >= p.rows) return;                       // whole wavefront; no workgroup barrier in this kernel
    const int row_first = (int)row_first64;
    const int g = lane / kLanes, i = lane % kLanes;
    const int ic = min(i, kNl - 1);                          // clamped: every lane addresses real memory

    uint16_t *tile_u = s_ud + wave * 2 * kTileElems, *tile_dl = tile_u + kTileElems;
    uint16_t *tile_b = s_bc + wave * 2 * kRowPad, *tile_c = tile_b + kRowPad;

    // What one tile brings in, as it arrives.  A tile's rows share image and group (host-checked: dim and dim_per_group
    // are multiples of kRows).
    struct TileLoads {
        uint4 vu[kVecsPerLane], vd[kVecsPerLane];
        uint2 vb, vc;
        uint16_t eb[kBcPerLane], ec[kBcPerLane];
        float A2, Dk, bias;
    };
    auto rows_of = [&](int row0) { return min(kRows, p.rows - row0); };
    auto fetch = [&](int row0, TileLoads &t) {
        const int nr = rows_of(row0);
        const int tile_bytes = nr * kL * 2;                  // range-checked: a short last tile reads zeros past its end
        const in_t *u_t = reinterpret_cast<const in_t *>(p.u) + (int64_t)row0 * kL;
        const in_t *dl_t = reinterpret_cast<const in_t *>(p.delta) + (int64_t)row0 * kL;
        const __amdgpu_buffer_rsrc_t ru = __builtin_amdgcn_make_buffer_rsrc(const_cast<in_t *>(u_t), 0, tile_bytes, kBufferRsrcWord3);
        const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(const_cast<in_t *>(dl_t), 0, tile_bytes, kBufferRsrcWord3);
#pragma unroll
        for (int v = 0; v < kVecsPerLane; ++v) {
            const auto tu = __builtin_amdgcn_raw_buffer_load_b128(ru, (v * kWave + lane) * 16, 0, 0);
            const auto td = __builtin_amdgcn_raw_buffer_load_b128(rd, (v * kWave + lane) * 16, 0, 0);
            t.vu[v] = make_uint4(tu[0], tu[1], tu[2], tu[3]);
            t.vd[v] = make_uint4(td[0], td[1], td[2], td[3]);
        }
        uint32_t b, d0, grp, rem;
        divmod((uint32_t)row0, div_dim, b, d0);
        divmod(d0, div_dpg, grp, rem);
        const in_t *B_row = reinterpret_cast<const in_t *>(p.B) + (int64_t)b * p.B_bs + (int64_t)grp * p.B_gs;
        const in_t *C_row = reinterpret_cast<const in_t *>(p.C) + (int64_t)b * p.C_bs + (int64_t)grp * p.C_gs;
        t.vb = make_uint2(0, 0); t.vc = make_uint2(0, 0);
        if (bc_vec) {                                        // rows on an 8-byte grid: 4 elements per lane
            if (lane < kL / 4) {
                t.vb = *reinterpret_cast<const uint2 *>(B_row + 4 * lane);
                t.vc = *reinterpret_cast<const uint2 *>(C_row + 4 * lane);
            }
        } else {
#pragma unroll
            for (int n = 0; n < kBcPerLane; ++n) {
                const int e = min(n * kWave + lane, kL - 1);
                t.eb[n] = B_row[e].bits; t.ec[n] = C_row[e].bits;
            }
        }
        const int kd = (int)d0 + min(g, nr - 1);
        t.A2 = p.A[(int64_t)kd * p.A_ds] * kLog2e;
        t.Dk = p.D ? p.D[kd] : 0.0f;
        t.bias = p.bias ? p.bias[kd] : 0.0f;
    };
    auto park = [&](const TileLoads &t) {
        if (bc_vec) {
            if (lane < kL / 4) {
                *reinterpret_cast<uint2 *>(tile_b + 4 * lane) = t.vb;
                *reinterpret_cast<uint2 *>(tile_c + 4 * lane) = t.vc;
            }
        } else {
#pragma unroll
            for (int n = 0; n < kBcPerLane; ++n) {
                const int e = n * kWave + lane;
                if (e < kL) { tile_b[e] = t.eb[n]; tile_c[e] = t.ec[n]; }
            }
        }
#pragma unroll
        for (int v = 0; v < kVecsPerLane; ++v) {
            const int vec = v * kWave + lane;
            if (vec < kTileVecs) {
                *reinterpret_cast<uint4 *>(tile_u + vec * 8) = t.vu[v];
                *reinterpret_cast<uint4 *>(tile_dl + vec * 8) = t.vd[v];
            }
        }
    };

    TileLoads cur;
    fetch(row_first, cur);
#pragma unroll
    for (int tile = 0; tile < kSmallTiles; ++tile) {
        const int row0 = row_first + tile * kRows;
        if (row0 >= p.rows) break;                           // uniform over the wavefront
        const int nr = rows_of(row0);
        const bool active = g < nr && i < kNl;
        const int gc = min(g, nr - 1);
        park(cur);
        const float A2 = cur.A2, Dk = cur.Dk, bias = cur.bias;
        wave_lds_sync();
        // the next tile's loads travel while this one is computed
        if (tile + 1 < kSmallTiles && row0 + kRows < p.rows) fetch(row0 + kRows, cur);

        // ---- this lane's run ----------------------------------------------------------------------------------------
        Run<in_t, kNi> raw, uu, Bv, Cv;
        raw.read(tile_dl, gc * kL + ic * kNi);
        uu.read(tile_u, gc * kL + ic * kNi);
        Bv.read(tile_b, ic * kNi);
        Cv.read(tile_c, ic * kNi);
        float ac[kNi], hh[kNi];
#pragma unroll
        for (int j = 0; j < kNi; ++j) {
            float dl;
            if constexpr (kSoftplus) dl = softplus_log2(fmaf(raw.item(j), kLog2e, bias * kLog2e));
            else dl = raw.item(j) + bias;
            const float a = __builtin_amdgcn_exp2f(dl * A2);
            const float bb = Bv.item(j) * (dl * uu.item(j));
            ac[j] = j == 0 ? a : ac[j - 1] * a;
            hh[j] = j == 0 ? bb : fmaf(a, hh[j - 1], bb);
        }
        // lanes that hold no segment stop the state: nothing travels from one group of lanes into the next (the first
        // lane of a DPP row has no lane below it)
        const float a_tot = active ? ac[kNi - 1] : 0.0f, h_tot = active ? hh[kNi - 1] : 0.0f;
        float a_incl = 1.0f;
        const float h_in = row_scan_state_in<false>(a_tot, h_tot, kX ? &a_incl : nullptr);
        float y[kNi];
#pragma unroll
        for (int j = 0; j < kNi; ++j) y[j] = fmaf(Cv.item(j), fmaf(ac[j], h_in, hh[j]), Dk * uu.item(j));
        if constexpr (kX) {
            // the product of the row's lane products ends up in its last lane: each step multiplies in the lane 1 / 2 / 4
            // (/ 8) below, lanes without a source and idle lanes count as 1, and with groups of 8 lanes the steps stop
            // at 4 so that a lane reaches back 7 lanes, to its own group's idle lane at most
            // (with one row per DPP row -- 16 lanes, 14 x 14 maps -- the scan above has left exactly that product in the
            // row's last lane: no idle lane sits below it)
            float pr = a_incl;
            if constexpr (kLanes != 16) {
                pr = active ? ac[kNi - 1] : 1.0f;
                pr *= dpp_move<kDppRowShr1>(1.0f, pr);
                pr *= dpp_move<kDppRowShr2>(1.0f, pr);
                pr *= dpp_move<kDppRowShr4>(1.0f, pr);
            }
            if (active && i == kNl - 1) {
                float *xo = p.x + (int64_t)(row0 + g) * 2;
                xo[0] = pr;
                xo[1] = fmaf(ac[kNi - 1], h_in, hh[kNi - 1]);
            }
        }
        if (nr == kRows && p.vec_out_ok) {
            // a full tile: park the outputs where u / delta sat (every lane has read its runs) and store the tile as it
            // lies in memory, 16 bytes per lane
            wave_lds_sync();
            out_t *ty = reinterpret_cast<out_t *>(tile_u);
            if (active) {
#pragma unroll
                for (int j = 0; j < kNi; ++j) ty[g * kL + i * kNi + j] = from_f32<out_t>(y[j]);
            }
            wave_lds_sync();
            constexpr int kOutVecs = kTileElems * (int)sizeof(out_t) / 16;
            uint4 *dst = reinterpret_cast<uint4 *>(reinterpret_cast<out_t *>(p.out) + (int64_t)row0 * kL);
            const uint4 *src = reinterpret_cast<const uint4 *>(ty);
#pragma unroll
            for (int v = 0; v < (kOutVecs + kWave - 1) / kWave; ++v) {
                const int vec = v * kWave + lane;
                // written once, read back by another kernel: streaming stores (14 x 14 maps at batch 128: 65 -> 56 us; streaming
                // LOADS of u / delta cost more than they gave, 7 x 7: 30 -> 34 us)
                if (vec < kOutVecs) store_streaming(dst + vec, src[vec]);
            }
        } else if (active) {
            out_t *yo = reinterpret_cast<out_t *>(p.out) + (int64_t)(row0 + g) * kL + i * kNi;
#pragma unroll
            for (int j = 0; j < kNi; ++j) yo[j] = from_f32<out_t>(y[j]);
        }
        wave_lds_sync();                                     // the tiles are free for the next tile's streams
    }
}

static bool small_rows_of(int L, int &rows_per_wave) {
    if (L == 196) { rows_per_wave = 4; return true; }
    if (L == 49) { rows_per_wave = 8; return true; }
    return false;
}

bool scan_small_eligible(const ScanArgs &a, int in_dtype, const void *u, const void *delta, const void *out) {
    int rpw;
    if (in_dtype != SS2D_BF16 && in_dtype != SS2D_F16) return false;
    if (a.N != 1 || a.dim_per_delta != 1 || !small_rows_of(a.L, rpw)) return false;
    const int64_t L = a.L, KD = a.dim;
    // rows adjacent in every stream; a wavefront's rows inside one image and one group
    if (a.u_ds != L || a.dl_ds != L || a.o_ds != L || a.u_bs != KD * L || a.dl_bs != KD * L || a.o_bs != KD * L) return false;
    if (KD % rpw != 0 || a.dim_per_group % rpw != 0) return false;
    auto al = [](const void *ptr, uintptr_t n) { return (reinterpret_cast<uintptr_t>(ptr) % n) == 0; };
    if (!al(u, 16) || !al(delta, 16)) return false;
    return (int64_t)a.rows * L * 2 < 0x7fffffffll;
}

template <typename in_t, typename out_t>
static int launch_small_typed(const ScanArgs &a, hipStream_t stream) {
    int rpw = 4;
    small_rows_of(a.L, rpw);
    const int tiles = a.L == 196 ? small_tiles<14>() : small_tiles<7>();
    const int64_t n_waves = ((int64_t)a.rows + rpw * tiles - 1) / (rpw * tiles);
    const int64_t n_wg = (n_waves + kWavesPerWg - 1) / kWavesPerWg;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    // B / C rows on an 8-byte grid (row length a multiple of 4): one 8-byte load per lane
    const uintptr_t bases = reinterpret_cast<uintptr_t>(a.B) | reinterpret_cast<uintptr_t>(a.C);
    ScanArgs b = a;
    b.vec_out_ok = reinterpret_cast<uintptr_t>(a.out) % 16 == 0;   // a wavefront's output tile starts on a 16-byte boundary
    const int bc_vec = a.L % 4 == 0 && bases % 8 == 0 && a.B_bs % 4 == 0 && a.B_gs % 4 == 0 && a.C_bs % 4 == 0 && a.C_gs % 4 == 0;
#define SS2D_LAUNCH_SMALL(NL, NI, SP, X)                                                                                       \
    hipLaunchKernelGGL((scan_small_kernel<in_t, out_t, NL, NI, SP, X>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream, b, bc_vec, \
                       make_fastdiv((uint32_t)a.dim), make_fastdiv((uint32_t)a.dim_per_group))
#define SS2D_LAUNCH_SMALL_L(SP, X) \
    if (a.L == 196) SS2D_LAUNCH_SMALL(14, 14, SP, X); else SS2D_LAUNCH_SMALL(7, 7, SP, X)
    if (a.x) { if (a.softplus) { SS2D_LAUNCH_SMALL_L(true, true); } else { SS2D_LAUNCH_SMALL_L(false, true); } }
    else { if (a.softplus) { SS2D_LAUNCH_SMALL_L(true, false); } else { SS2D_LAUNCH_SMALL_L(false, false); } }
#undef SS2D_LAUNCH_SMALL_L
#undef SS2D_LAUNCH_SMALL
    return launch_status();
}

int launch_scan_small(const ScanArgs &a, int in_dtype, int out_dtype, hipStream_t stream) {
    if (in_dtype == SS2D_BF16) {
        return out_dtype == SS2D_F32 ? launch_small_typed<bf16_t, float>(a, stream) : launch_small_typed<bf16_t, bf16_t>(a, stream);
    }
    return out_dtype == SS2D_F32 ? launch_small_typed<f16_t, float>(a, stream) : launch_small_typed<f16_t, f16_t>(a, stream);
}

}  // namespace ss2d
