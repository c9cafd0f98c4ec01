// Fused SS2D core (CrossScan -> selective scan -> CrossMerge, d_state = 1) for maps of ANY size: the map is cut into
// 64 x 64 tiles, and the kernel runs twice over the tiles with a small carry scan in between.
//
// The single-kernel core (ss2d_core.hip) keeps a whole map and its two merge planes in LDS, which ends at ~13 000
// positions.  A scan direction crosses a tile as 64 separate runs of 64 consecutive positions (row pieces for the
// row-major directions 0 / 2, column pieces for the column-major directions 1 / 3); given the state that ENTERS a run, the
// run is an independent piece of work.  So:
//   pass A   every workgroup takes a tile and computes, per run and direction, the run's aggregate (product of the
//            decays, state at its end from a zero start) -- the scan operator's summary of the run;            [agg]
//   carries  one workgroup per (direction, image, channel) combines the aggregates in that direction's order and leaves
//            the state entering every run;                                                                     [carry]
//   pass B   every workgroup takes its tile again, starts each run from its carry and produces the outputs.
// Both passes read x and delta once (the B / C rows are shared by the channels of an image and come from L2): 10 and 14
// bytes per element instead of the 62 of the three operators, for twice the arithmetic of the scan.
//
// Because runs are independent, the forward and the backward direction of a pair walk the SAME positions in the same
// lanes -- lane l of a pass owns 8 consecutive positions of one run; backwards it takes them in descending order and the
// lanes of the run combine in descending order -- so y_0 + y_2 (and y_1 + y_3) are summed in registers: no merge planes,
// no read-add-write, no barriers inside the scan.  The one exchange is the transposition of the column-major sums into
// row-major order, through a 64 x 64 fp32 tile in LDS.  Every wavefront does two passes of column runs, then (after the
// one barrier) two passes of row runs, which add the transposed sums and the skip term and store the result.
//
// A run of 64 positions occupies 8 lanes (half a DPP row).  The lane-local scan of 8 items is followed by a scan over
// the 8 lanes with DPP row shifts; the run's first lane (in the direction's order) takes the carry in and passes on a
// decay of zero, which also stops anything from the other run that shares its DPP row.
// Semantics: as ss2d_core_fwd (classification/models/vmamba.py:604, 625-633, 638; cross_merge_fwd's pairing,
// classification/models/csm_triton.py:56-62).
#include <type_traits>

#include "scan_common.h"

namespace ss2d {

constexpr int kTile = 64;                  // tile side (positions)
constexpr int kTilePitch = kTile + 1;      // floats per row of the transposition tile

struct TiledGeom {
    int32_t ntr, ntc;                      // tiles down and across a map
    int32_t nr02, nr13, nr_max;            // runs per (image, channel) of a row-major / column-major direction
    FastDiv div_tiles, div_ntc, div_D;
};

// Inclusive scan of (a, h) pairs over the lanes of a DPP row in three steps (reach: 7 lanes), ascending or descending;
// returns the h of the lane before this one in scan order (0 where there is none in the DPP row).  A lane whose a is 0
// cuts the chain: that is how the 8-lane runs of a 16-lane DPP row are kept apart.
template <bool kReverse>
__device__ __forceinline__ float run_scan(float a, float &h) {
    float hx = 0.0f;
#define SS2D_RUN_STEP(CTRL)                                             \
    "v_fmac_f32_dpp %1, %1, %0 " CTRL " row_mask:0xf bank_mask:0xf\n\t" \
    "v_mul_f32_dpp %0, %0, %0 " CTRL " row_mask:0xf bank_mask:0xf\n\t"  \
    "s_nop 0\n\t"
    if constexpr (!kReverse) {
        asm("s_nop 1\n\t" SS2D_RUN_STEP("row_shr:1") SS2D_RUN_STEP("row_shr:2") SS2D_RUN_STEP("row_shr:4")
            "s_nop 0\n\t"
            "v_mov_b32_dpp %2, %1 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 0"
            : "+v"(a), "+v"(h), "+v"(hx));
    } else {
        asm("s_nop 1\n\t" SS2D_RUN_STEP("row_shl:1") SS2D_RUN_STEP("row_shl:2") SS2D_RUN_STEP("row_shl:4")
            "s_nop 0\n\t"
            "v_mov_b32_dpp %2, %1 row_shl:1 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 0"
            : "+v"(a), "+v"(h), "+v"(hx));
    }
#undef SS2D_RUN_STEP
    return hx;
}

// Product of v over the 8 lanes of a run, delivered in the run's last lane in scan order.
template <bool kReverse>
__device__ __forceinline__ float run_product(float v) {
    if constexpr (!kReverse) {
        v *= dpp_move<kDppRowShr1>(1.0f, v);
        v *= dpp_move<kDppRowShr2>(1.0f, v);
        v *= dpp_move<kDppRowShr4>(1.0f, v);
    } else {
        constexpr int kShl1 = 0x101, kShl2 = 0x102, kShl4 = 0x104;
        v *= dpp_move<kShl1>(1.0f, v);
        v *= dpp_move<kShl2>(1.0f, v);
        v *= dpp_move<kShl4>(1.0f, v);
    }
    return v;
}

// What one pass of one lane brings in: delta and B (and C for the outputs) of its 8 positions for the forward and the
// backward direction of the pair, its 8 values of x, and the two carries of its run.
template <bool kCol, bool kOut>
struct TilePassLoads {
    uint4 dl[2], bq[2], cq[kOut ? 2 : 1];
    uint32_t u[kCol ? 8 : 4];              // column runs: one 16-bit value per register, as gathered
    float carry[kOut ? 2 : 1];
    int32_t run, p;                        // run index of the pair's forward direction; first stream position of the lane
    bool valid, line_ok;
};

template <typename in_t, bool kSoftplus, bool kOut>
__global__ __launch_bounds__(kBlock) void core_tiled_kernel(const CoreArgs p, const TiledGeom g, float2 *__restrict__ agg,
                                                            const float *__restrict__ carry) {
    static_assert(sizeof(in_t) == 2, "16-bit streams");
    __shared__ float s_plane[kOut ? kTile * kTilePitch : 1];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // neighbours in the grid are the channels of one tile of one image: they read the same B / C pieces, so each XCD
    // (one L2) gets a contiguous range of them
    const uint32_t wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
    uint32_t bt, d, b, tile, tr, tc;
    divmod(wg, g.div_D, bt, d);
    divmod(bt, g.div_tiles, b, tile);
    divmod(tile, g.div_ntc, tr, tc);
    const int H = p.H, W = p.W, L = p.L;
    const int h0 = (int)tr * kTile, w0 = (int)tc * kTile;
    const int seg = lane & 7, sub = lane >> 3;               // piece of the run; run of the pass
    const in_t *x_map = reinterpret_cast<const in_t *>(p.x) + ((int64_t)b * p.D + d) * L;
    const in_t *dl_bd = reinterpret_cast<const in_t *>(p.delta) + (int64_t)d * p.dl_ds + (int64_t)b * p.dl_bs;
    const in_t *B_b = reinterpret_cast<const in_t *>(p.Bm) + (int64_t)b * p.B_bs;
    const in_t *C_b = reinterpret_cast<const in_t *>(p.Cm) + (int64_t)b * p.C_bs;
    const int64_t bd = (int64_t)b * p.D + d, BD = (int64_t)p.B * p.D;
    // with softplus the step is kept in units of ln 2 (softplus_over_ln2): decay 2^(step * A) with A as given, sums in
    // units of ln 2, one multiplication by ln 2 per output
    float A2[4], bias[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        A2[k] = kSoftplus ? p.A[k * p.D + (int)d] : p.A[k * p.D + (int)d] * kLog2e;
        bias[k] = p.bias ? p.bias[k * p.D + (int)d] : 0.0f;
    }

    // ---- one pass: 8 runs of the tile (rows h0 + line, or columns w0 + line), 8 positions per lane -------------------
    auto issue = [&](auto col_tag, int pass, auto &r) {
        constexpr bool kCol = decltype(col_tag)::value;
        const int line = wave * 16 + pass * 8 + sub;
        const int n_lines = kCol ? W : H, n_along = kCol ? H : W;
        const int line_abs = (kCol ? w0 : h0) + line, along = (kCol ? h0 : w0) + 8 * seg;
        r.line_ok = line < kTile && line_abs < n_lines;
        r.valid = r.line_ok && along < n_along;
        // lanes without positions address the map's first vector and are kept out of the scan and the stores
        r.p = r.valid ? line_abs * n_along + along : 0;
        r.run = r.line_ok ? line_abs * (kCol ? g.ntr : g.ntc) + (int)(kCol ? tr : tc) : 0;
        constexpr int kf = kCol ? 1 : 0, kb = kf + 2;
        const int q = L - kItems - r.p;                          // the same 8 positions in the backward direction's order
        r.dl[0] = *reinterpret_cast<const uint4 *>(dl_bd + kf * p.dl_ks + r.p);
        r.dl[1] = *reinterpret_cast<const uint4 *>(dl_bd + kb * p.dl_ks + q);
        r.bq[0] = *reinterpret_cast<const uint4 *>(B_b + kf * p.B_ks + r.p);
        r.bq[1] = *reinterpret_cast<const uint4 *>(B_b + kb * p.B_ks + q);
        if constexpr (kOut) {
            r.cq[0] = *reinterpret_cast<const uint4 *>(C_b + kf * p.C_ks + r.p);
            r.cq[1] = *reinterpret_cast<const uint4 *>(C_b + kb * p.C_ks + q);
            r.carry[0] = carry[(kf * BD + bd) * g.nr_max + r.run];
            r.carry[1] = carry[(kb * BD + bd) * g.nr_max + r.run];
        }
        if constexpr (kCol) {
            const in_t *src = x_map + (r.valid ? along * W + line_abs : 0);
#pragma unroll
            for (int i = 0; i < kItems; ++i) r.u[i] = src[r.valid ? i * W : 0].bits;
        } else {
            const uint4 t = *reinterpret_cast<const uint4 *>(x_map + r.p);
            r.u[0] = t.x; r.u[1] = t.y; r.u[2] = t.z; r.u[3] = t.w;
        }
    };

    // One direction of a pass.  Items j = 0..7 are in the direction's order; position index i = j forwards, 7 - j
    // backwards.  kOut: acc[i] (by position) receives C * h; else the run's aggregate goes to agg.
    auto direction = [&](auto rev_tag, auto first_tag, int k, const uint4 &dl_raw, const uint4 &b_raw, const uint4 &c_raw,
                         const float (&uf)[kItems], float carry_in, bool valid, bool line_ok, int run, float (&acc)[kItems]) {
        constexpr bool kRev = decltype(rev_tag)::value, kFirstOfPair = decltype(first_tag)::value;
        const uint32_t dw[4] = {dl_raw.x, dl_raw.y, dl_raw.z, dl_raw.w}, bw[4] = {b_raw.x, b_raw.y, b_raw.z, b_raw.w};
        float ac[kItems], hh[kItems];
#pragma unroll
        for (int j = 0; j < kItems; ++j) {
            const float raw = (j & 1) ? unpack_hi<in_t>(dw[j / 2]) : unpack_lo<in_t>(dw[j / 2]);
            const float Bv = (j & 1) ? unpack_hi<in_t>(bw[j / 2]) : unpack_lo<in_t>(bw[j / 2]);
            float dl;
            if constexpr (kSoftplus) dl = softplus_over_ln2(fmaf(raw, kLog2e, bias[k] * kLog2e));
            else dl = raw + bias[k];
            const float a = __builtin_amdgcn_exp2f(dl * A2[k]);
            const float bb = Bv * (dl * uf[kRev ? kItems - 1 - j : j]);
            ac[j] = j == 0 ? a : ac[j - 1] * a;
            hh[j] = j == 0 ? bb : fmaf(a, hh[j - 1], bb);
        }
        // lanes without positions are the identity; the run's first lane takes the carry in and cuts the chain
        const float a_lane = valid ? ac[kItems - 1] : 1.0f, h_lane = valid ? hh[kItems - 1] : 0.0f;
        const bool first = kRev ? seg == 7 : seg == 0;
        const float c_in = kOut ? carry_in : 0.0f;
        float h_run = first ? fmaf(a_lane, c_in, h_lane) : h_lane;
        const float h_before = run_scan<kRev>(first ? 0.0f : a_lane, h_run);
        if constexpr (kOut) {
            const uint32_t cw[4] = {c_raw.x, c_raw.y, c_raw.z, c_raw.w};
            const float s_in = first ? c_in : h_before;
#pragma unroll
            for (int j = 0; j < kItems; ++j) {
                const int i = kRev ? kItems - 1 - j : j;
                const float Cv = (j & 1) ? unpack_hi<in_t>(cw[j / 2]) : unpack_lo<in_t>(cw[j / 2]);
                const float h = fmaf(ac[j], s_in, hh[j]);
                acc[i] = kFirstOfPair ? Cv * h : fmaf(Cv, h, acc[i]);
            }
        } else {
            const float prod = run_product<kRev>(a_lane);
            const bool last = kRev ? seg == 0 : seg == 7;
            if (last && line_ok) agg[(k * BD + bd) * g.nr_max + run] = make_float2(prod, h_run);
        }
    };

    auto compute = [&](auto col_tag, const auto &r, float (&acc)[kItems], float (&uf)[kItems]) {
        constexpr bool kCol = decltype(col_tag)::value;
        constexpr int kf = kCol ? 1 : 0, kb = kf + 2;
        if constexpr (kCol) {
#pragma unroll
            for (int i = 0; i < kItems; ++i) uf[i] = to_f32(in_t{(uint16_t)r.u[i]});
        } else {
#pragma unroll
            for (int i = 0; i < kItems; ++i) uf[i] = (i & 1) ? unpack_hi<in_t>(r.u[i / 2]) : unpack_lo<in_t>(r.u[i / 2]);
        }
        direction(std::false_type{}, std::true_type{}, kf, r.dl[0], r.bq[0], r.cq[0], uf, r.carry[0], r.valid, r.line_ok, r.run, acc);
        direction(std::true_type{}, std::false_type{}, kb, r.dl[1], r.bq[1], r.cq[kOut ? 1 : 0], uf, r.carry[kOut ? 1 : 0], r.valid,
                  r.line_ok, r.run, acc);
    };

    using ColLoads = TilePassLoads<true, kOut>;
    using RowLoads = TilePassLoads<false, kOut>;
    ColLoads c0, c1;
    RowLoads r0, r1;
    issue(std::true_type{}, 0, c0);
    issue(std::true_type{}, 1, c1);
    float acc[kItems], uf[kItems];

    // ---- column runs: directions 1 + 3; the sums go into the transposition tile, [column][row] ---------------------
    auto column_pass = [&](int pass, const ColLoads &r) {
        compute(std::true_type{}, r, acc, uf);
        if constexpr (kOut) {
            float *dst = s_plane + (wave * 16 + pass * 8 + sub) * kTilePitch + 8 * seg;
#pragma unroll
            for (int i = 0; i < kItems; ++i) dst[i] = acc[i];
        }
    };
    column_pass(0, c0);
    issue(std::false_type{}, 0, r0);
    column_pass(1, c1);
    issue(std::false_type{}, 1, r1);
    if constexpr (kOut) __syncthreads();

    // ---- row runs: directions 0 + 2, then out = (y0 + y2) + (y1 + y3) + (D0 + D1 + D2 + D3) x ----------------------
    float Dsum = 0.0f;
    if (kOut && p.Dv) Dsum = (p.Dv[d] + p.Dv[2 * p.D + (int)d]) + (p.Dv[p.D + (int)d] + p.Dv[3 * p.D + (int)d]);
    auto row_pass = [&](int pass, const RowLoads &r) {
        compute(std::false_type{}, r, acc, uf);
        if constexpr (kOut) {
            const int line = wave * 16 + pass * 8 + sub;
            const float *src = s_plane + (8 * seg) * kTilePitch + line;
            float o[kItems];
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                const float sums = acc[i] + src[i * kTilePitch];
                o[i] = kSoftplus ? fmaf(sums, kLn2, Dsum * uf[i]) : fmaf(Dsum, uf[i], sums);
            }
            if (r.valid) {
                float *yo = reinterpret_cast<float *>(p.y) + bd * L + r.p;
                *reinterpret_cast<float4 *>(yo) = make_float4(o[0], o[1], o[2], o[3]);
                *reinterpret_cast<float4 *>(yo + 4) = make_float4(o[4], o[5], o[6], o[7]);
            }
        }
    };
    row_pass(0, r0);
    row_pass(1, r1);
}

// One workgroup per (direction, image, channel): the state entering every run, in the direction's order of the runs.  A
// round covers 4 x 64 x kPer runs: wavefront w scans its quarter, the four quarters' aggregates meet in LDS, and each
// wavefront folds the ones before it into the state its quarter starts from.
__global__ __launch_bounds__(kBlock) void core_carry_kernel(const float2 *__restrict__ agg, float *__restrict__ carry, int rows,
                                                            int BD, int nr02, int nr13, int nr_max) {
    constexpr int kPer = 4;                                  // runs per lane and round
    constexpr int kRound = kWavesPerWg * kWave * kPer;       // runs per workgroup and round
    __shared__ float2 s_agg[2][kWavesPerWg];                 // double-buffered by round parity: one barrier per round
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int row = (int)blockIdx.x;                         // grid == rows
    const int k = row / BD;
    const int n = (k & 1) ? nr13 : nr02;
    const bool rev = k >= 2;
    const float2 *src = agg + (int64_t)row * nr_max;
    float *dst = carry + (int64_t)row * nr_max;
    float state = 0.0f;
    int par = 0;
    for (int j0 = 0; j0 < n; j0 += kRound, par ^= 1) {       // uniform over the workgroup: every wavefront meets the barrier
        float ac[kPer], hh[kPer];
#pragma unroll
        for (int t = 0; t < kPer; ++t) {
            const int j = j0 + (wave * kWave + lane) * kPer + t;
            float2 v = make_float2(1.0f, 0.0f);
            if (j < n) v = src[rev ? n - 1 - j : j];
            ac[t] = t == 0 ? v.x : ac[t - 1] * v.x;
            hh[t] = t == 0 ? v.y : fmaf(v.x, hh[t - 1], v.y);
        }
        float a_ex, h_ex, a_tot, h_tot;
        wave_scan_pairs(ac[kPer - 1], hh[kPer - 1], a_ex, h_ex, a_tot, h_tot);
        if (lane == 0) s_agg[par][wave] = make_float2(a_tot, h_tot);
        __syncthreads();
        float c_in = state;                                  // the state this wavefront's quarter starts from ...
#pragma unroll
        for (int w = 0; w < kWavesPerWg; ++w) {
            const float2 g = s_agg[par][w];
            if (w < wave) c_in = fmaf(g.x, c_in, g.y);
            state = fmaf(g.x, state, g.y);                   // ... and the one the next round starts from
        }
        const float s_in = fmaf(a_ex, c_in, h_ex);
#pragma unroll
        for (int t = 0; t < kPer; ++t) {
            const int j = j0 + (wave * kWave + lane) * kPer + t;
            if (j < n) dst[rev ? n - 1 - j : j] = t == 0 ? s_in : fmaf(ac[t - 1], s_in, hh[t - 1]);
        }
    }
    (void)rows;
}

static TiledGeom tiled_geometry(const CoreArgs &a) {
    TiledGeom g;
    g.ntr = (a.H + kTile - 1) / kTile;
    g.ntc = (a.W + kTile - 1) / kTile;
    g.nr02 = a.H * g.ntc;
    g.nr13 = a.W * g.ntr;
    g.nr_max = g.nr02 > g.nr13 ? g.nr02 : g.nr13;
    g.div_tiles = make_fastdiv((uint32_t)(g.ntr * g.ntc));
    g.div_ntc = make_fastdiv((uint32_t)g.ntc);
    g.div_D = make_fastdiv((uint32_t)a.D);
    return g;
}

bool core_tiled_eligible(const CoreArgs &a, int in_dtype) {
    if (in_dtype != SS2D_BF16 && in_dtype != SS2D_F16) return false;
    if (a.H % kItems != 0 || a.W % kItems != 0) return false;
    auto al = [](const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) % 16) == 0; };
    if (!al(a.x) || !al(a.delta) || !al(a.Bm) || !al(a.Cm) || !al(a.y)) return false;
    const int64_t strides[] = {a.dl_ks, a.dl_ds, a.dl_bs, a.B_ks, a.B_bs, a.C_ks, a.C_bs};
    for (int64_t s : strides)
        if (s % kItems != 0) return false;
    const TiledGeom g = tiled_geometry(a);
    const int64_t n_wg = (int64_t)a.B * a.D * g.ntr * g.ntc;
    return n_wg <= 0x7fffffff && 4 * (int64_t)a.B * a.D <= 0x7fffffff - kWavesPerWg;
}

int64_t core_tiled_workspace_bytes(const CoreArgs &a) {
    const TiledGeom g = tiled_geometry(a);
    // aggregates (two floats per run) and carries (one), for the four directions
    return 4 * (int64_t)a.B * a.D * g.nr_max * (int64_t)(sizeof(float2) + sizeof(float));
}

template <typename in_t>
static int launch_core_tiled_typed(const CoreArgs &a, void *workspace, hipStream_t stream) {
    const TiledGeom g = tiled_geometry(a);
    const int64_t rows = 4 * (int64_t)a.B * a.D;
    float2 *agg = reinterpret_cast<float2 *>(workspace);
    float *carry = reinterpret_cast<float *>(agg + rows * g.nr_max);
    const uint32_t n_wg = (uint32_t)((int64_t)a.B * a.D * g.ntr * g.ntc);
    const uint32_t carry_wg = (uint32_t)rows;                // one workgroup per (direction, image, channel)
#define SS2D_TILED_LAUNCH(SP)                                                                                                      \
    hipLaunchKernelGGL((core_tiled_kernel<in_t, SP, false>), dim3(n_wg), dim3(kBlock), 0, stream, a, g, agg, (const float *)carry); \
    hipLaunchKernelGGL(core_carry_kernel, dim3(carry_wg), dim3(kBlock), 0, stream, (const float2 *)agg, carry, (int)rows,           \
                       a.B * a.D, g.nr02, g.nr13, g.nr_max);                                                                        \
    hipLaunchKernelGGL((core_tiled_kernel<in_t, SP, true>), dim3(n_wg), dim3(kBlock), 0, stream, a, g, agg, (const float *)carry)
    if (a.softplus) { SS2D_TILED_LAUNCH(true); } else { SS2D_TILED_LAUNCH(false); }
#undef SS2D_TILED_LAUNCH
    return launch_status();
}

int launch_core_tiled(const CoreArgs &a, int in_dtype, void *workspace, hipStream_t stream) {
    return in_dtype == SS2D_BF16 ? launch_core_tiled_typed<bf16_t>(a, workspace, stream)
                                 : launch_core_tiled_typed<f16_t>(a, workspace, stream);
}

}  // namespace ss2d
