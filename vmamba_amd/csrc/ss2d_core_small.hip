// Fused SS2D core (CrossScan -> selective scan -> CrossMerge, d_state = 1) for SMALL square maps -- 7 x 7 and 14 x 14,
// the last two stages of a 224 x 224 VMamba -- with one map ROW per lane and every index fixed at compile time.
//
// The general kernel (ss2d_core.hip) walks the images of a workgroup as one stream, 8 positions per lane; on maps of
// 49 or 196 positions most of its instructions are bookkeeping: images start inside a lane's 8 items, B / C are gathered
// in groups of 1 or 4, the transposed copies of the map and of the result are built element by element.  Here
//   * a map of S x S positions occupies S lanes of a group of 8 or 16 lanes (the DPP row or half row), 4 or 8 maps per
//     wavefront, the maps of a wavefront being consecutive images of one channel (their delta / B / C rows are adjacent
//     in the batch-innermost layout, so a stream tile is fetched with one or two 16-byte loads per lane and parked in
//     LDS as loaded); the four wavefronts of a workgroup are four channels on the same images and share the B / C tiles;
//     everything a workgroup reads is requested before its arithmetic starts;
//   * for the row-major directions (0, 2) lane i owns row i, for the column-major ones (1, 3) column i: either way its
//     S positions are S consecutive stream items, which it scans serially in registers; the lane totals are combined
//     by a DPP scan over the lane group (forward for directions 0 / 1, in reverse lane order for 2 / 3), and the state
//     entering the lane is pushed through its items.  A map's first item is forced to a = 0, which stops anything
//     arriving from the neighbouring group;
//   * u comes from two register copies of the map as loaded (its row, 4-byte loads, and its column, 2-byte loads the
//     first-level cache serves); the outputs of directions 1 + 3 accumulate in registers indexed by row and go through
//     one LDS transposition (over delta tiles that are no longer needed) into row layout, those of 0 + 2 accumulate in
//     registers indexed by column, and out = (y0 + y2) + (y1 + y3) + (D0 + D1 + D2 + D3) x leaves as plain row
//     stores -- the association order of cross_merge_fwd (classification/models/csm_triton.py:61-62), the skip term,
//     the same multiple of x in all four directions, added once.
// No stream position, image boundary or LDS address is computed at run time.
#include "scan_common.h"

namespace ss2d {

constexpr int kSmallChans = kWavesPerWg;     // channels per workgroup: one per wavefront, all on the same images

// Registers are capped so that as many workgroups share a CU as its LDS tiles allow (4 for 14 x 14, 5-6 for 7 x 7).
template <typename in_t, int kS, bool kSoftplus>
__global__ __launch_bounds__(kBlock, kS <= 8 ? 5 : 4) void ss2d_core_small_kernel(const CoreArgs p, int chan_quads, FastDiv div_quads) {
    constexpr int kLanes = kS <= 8 ? 8 : 16;                 // lanes per map
    constexpr int kMaps = kWave / kLanes;                    // maps per wavefront
    constexpr int kL = kS * kS;
    constexpr int kTileElems = kMaps * kL;                   // one stream tile: the maps' rows are adjacent in memory
    constexpr int kTileVecs = kTileElems / 8;                // in 16-byte pieces (392 or 784 elements: whole pieces)
    constexpr int kVecsPerLane = (kTileVecs + kWave - 1) / kWave;
    constexpr int kBcPieces = 8 * kTileVecs;                 // B and C tiles of the four directions
    constexpr int kBcPerThread = (kBcPieces + kBlock - 1) / kBlock;
    static_assert(kTileElems % 8 == 0 && sizeof(in_t) == 2, "16-bit streams in whole 16-byte pieces");
    // Everything a workgroup reads is fetched before its arithmetic starts (one memory latency per workgroup; the
    // registers that carry the loads are free again when the per-map arrays come alive):
    //   shared by the four wavefronts (same images): the B and C tiles of the four directions   [dir][B|C][tile]
    //   per wavefront (its channel): the four delta tiles, in the order of use 1, 3, 0, 2; once directions 1 and 3 are
    //   done, the room of their two tiles holds the fp32 tile of the (y1 + y3) sums for the column -> row transposition
    __shared__ __align__(16) uint16_t s_bc[8 * kTileElems + kRunSlack];
    __shared__ __align__(16) uint16_t s_dl[kWavesPerWg * 4 * kTileElems + kRunSlack];
    static_assert(2 * kTileElems * sizeof(uint16_t) == kTileElems * sizeof(float), "the fp32 tile fits two delta tiles");

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    uint32_t bt, dq;
    divmod(blockIdx.x, div_quads, bt, dq);                   // neighbouring workgroups: other channels of the same images
    const int d_raw = (int)dq * kSmallChans + wave;
    const bool chan_ok = d_raw < p.D;                        // (a wavefront without a channel still helps to fetch B / C)
    const int d = min(d_raw, p.D - 1);
    const int b0 = (int)bt * kMaps;
    const int nb = min(kMaps, p.B - b0);
    const int g = lane / kLanes, i = lane % kLanes;
    const bool active = g < nb && i < kS;
    const int gc = min(g, nb - 1), ic = min(i, kS - 1);      // clamped: every lane addresses real memory

    uint16_t *tile_dl = s_dl + wave * 4 * kTileElems;
    float *tile_tr = reinterpret_cast<float *>(tile_dl);    // over the tiles of directions 1 and 3 (slots 0 and 1)
    constexpr int kSlot[4] = {2, 0, 3, 1};                   // direction -> slot of its delta tile

    // ---- fetch ------------------------------------------------------------------------------------------------------
    // delta: four tiles of this wavefront's channel, 16-byte buffer loads (range-checked: a short last tile reads zeros
    // past its end)
    uint4 r_dl[4][kVecsPerLane];
    {
        const in_t *dl_all = reinterpret_cast<const in_t *>(p.delta);
        // (the extent in whole 16-byte pieces: a piece that straddles the extent loses more than the bytes behind it --
        //  measured: with the exact extent the last element of a short tile of odd maps came back as zero.  What the
        //  last piece holds behind the tile is the next image's first elements or, at the tensor's end, the rest of
        //  a 16-byte block that starts inside the tensor; no lane with a map uses it)
        const int tile_bytes = (nb * kL * 2 + 15) & ~15;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const in_t *dl_k = dl_all + (int64_t)k * p.dl_ks + (int64_t)d * p.dl_ds + (int64_t)b0 * kL;
            const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<in_t *>(dl_k), 0, tile_bytes, kBufferRsrcWord3);
#pragma unroll
            for (int v = 0; v < kVecsPerLane; ++v) {
                const auto t = __builtin_amdgcn_raw_buffer_load_b128(rs, (v * kWave + lane) * 16, 0, 0);
                r_dl[k][v] = make_uint4(t[0], t[1], t[2], t[3]);
            }
        }
    }
    // B / C: the workgroup's threads share the 8 tiles; one descriptor over each tensor (its extent rounded up to whole
    // 16-byte pieces by the host, as above), the tile chosen per lane (what lies behind a short last tile is other
    // images' data or, past the tensor, zeros: never stored)
    uint4 r_bc[kBcPerThread];
    {
        const __amdgpu_buffer_rsrc_t rB = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.Bm), 0, (int)p.B_span_bytes, kBufferRsrcWord3);
        const __amdgpu_buffer_rsrc_t rC = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.Cm), 0, (int)p.C_span_bytes, kBufferRsrcWord3);
#pragma unroll
        for (int n = 0; n < kBcPerThread; ++n) {
            const int piece = n * kBlock + (int)threadIdx.x;     // [dir][B|C][piece of the tile]
            const int t = min(piece, kBcPieces - 1) / kTileVecs, v = min(piece, kBcPieces - 1) % kTileVecs;
            const int k = t >> 1;
            const uint32_t off_B = (uint32_t)(k * p.B_ks + (int64_t)b0 * kL) * 2u + (uint32_t)v * 16u;
            const uint32_t off_C = (uint32_t)(k * p.C_ks + (int64_t)b0 * kL) * 2u + (uint32_t)v * 16u;
            const auto tb = __builtin_amdgcn_raw_buffer_load_b128(rB, (int)off_B, 0, 0);
            const auto tc = __builtin_amdgcn_raw_buffer_load_b128(rC, (int)off_C, 0, 0);
            const bool is_c = (t & 1) != 0;
            r_bc[n] = make_uint4(is_c ? tc[0] : tb[0], is_c ? tc[1] : tb[1], is_c ? tc[2] : tb[2], is_c ? tc[3] : tb[3]);
        }
    }
    // the map: this lane's row and this lane's column, as loaded (16-bit; widened where used)
    Run<in_t, kS> x_row, x_col;
    {
        const in_t *map = reinterpret_cast<const in_t *>(p.x) + ((int64_t)(b0 + gc) * p.D + d) * kL;
        if constexpr (kS % 2 == 0) {
            x_row.read(reinterpret_cast<const uint16_t *>(map), ic * kS);
        } else {
            // an odd row is fetched as the kS + 1 elements that start at its first one -- for the map's last row, which
            // ends where the map ends, as those that start one element earlier, shifted into place: nothing outside
            // the map is touched
            const int back = ic == kS - 1 ? 1 : 0;
            x_row.read_from(reinterpret_cast<const uint16_t *>(map) + ic * kS - back, back);
        }
        uint16_t e[kS];
#pragma unroll
        for (int j = 0; j < kS; ++j) e[j] = map[j * kS + ic].bits;
        x_col.pack(e);
    }
    // ---- park the streams in LDS ------------------------------------------------------------------------------------
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int v = 0; v < kVecsPerLane; ++v) {
            const int vec = v * kWave + lane;
            if (vec < kTileVecs) *reinterpret_cast<uint4 *>(tile_dl + kSlot[k] * kTileElems + vec * 8) = r_dl[k][v];
        }
#pragma unroll
    for (int n = 0; n < kBcPerThread; ++n) {
        const int piece = n * kBlock + (int)threadIdx.x;
        if (piece < kBcPieces) *reinterpret_cast<uint4 *>(s_bc + piece * 8) = r_bc[n];
    }
    __syncthreads();                                         // the only workgroup barrier: B / C tiles are in place
    if (!chan_ok) return;

    float acc[kS];                                           // y1 + y3 by row of column i, then y0 + y2 by column of row i
#pragma unroll
    for (int j = 0; j < kS; ++j) acc[j] = 0.0f;

    auto direction = [&](auto dir_tag) {
        constexpr int kDir = decltype(dir_tag)::value;
        constexpr bool kRev = kDir >= 2, kCol = (kDir & 1) != 0;
        // reversed directions: stream position t' = L-1-t, so the run holding this lane's row / column is run kS-1-i,
        // met from its far end -- item j of the run is column (row) kS-1-j
        const int run = gc * kL + (kRev ? kS - 1 - ic : ic) * kS;
        Run<in_t, kS> raw, Bv, Cv;
        raw.read(tile_dl + kSlot[kDir] * kTileElems, run);
        Bv.read(s_bc + (2 * kDir) * kTileElems, run);
        Cv.read(s_bc + (2 * kDir + 1) * kTileElems, run);

        const int kd = kDir * p.D + d;
        // with softplus the step is kept in units of ln 2 (softplus_over_ln2): the decay is 2^(step * A) with A as given,
        // the sums collect y / ln 2 and the merge multiplies by ln 2 once per position
        const float A2 = kSoftplus ? p.A[kd] : p.A[kd] * kLog2e;
        const float bias = p.bias ? p.bias[kd] : 0.0f;
        const bool first = kRev ? i == kS - 1 : i == 0;      // the lane that starts the map in this direction's order
        float ac[kS], hh[kS];
#pragma unroll
        for (int j = 0; j < kS; ++j) {
            const int m = kRev ? kS - 1 - j : j;             // column (directions 0 / 2) or row (1 / 3) of item j
            const float u = kCol ? x_col.item(m) : x_row.item(m);
            float dl;
            if constexpr (kSoftplus) dl = softplus_over_ln2(fmaf(raw.item(j), kLog2e, bias * kLog2e));
            else dl = raw.item(j) + bias;
            float a = __builtin_amdgcn_exp2f(dl * A2);
            if (j == 0) a = first ? 0.0f : a;                // nothing enters a map from the lanes before it
            const float bb = Bv.item(j) * (dl * u);
            ac[j] = j == 0 ? a : ac[j - 1] * a;
            hh[j] = j == 0 ? bb : fmaf(a, hh[j - 1], bb);
        }
        // lanes that hold no row pass the state through unchanged (and keep whatever they computed out of the scan)
        const float a_tot = active ? ac[kS - 1] : 1.0f, h_tot = active ? hh[kS - 1] : 0.0f;
        const float h_in = row_scan_state_in<kRev>(a_tot, h_tot);
#pragma unroll
        for (int j = 0; j < kS; ++j) {
            const int m = kRev ? kS - 1 - j : j;
            acc[m] += Cv.item(j) * fmaf(ac[j], h_in, hh[j]);
        }
    };
    // (y1 + y3), then (y0 + y2): the first addition into a zero is exact, the second rounds once
    direction(std::integral_constant<int, 1>{});
    direction(std::integral_constant<int, 3>{});
    // bring (y1 + y3) from column layout to row layout through LDS: this lane is column i, element (row j, col i)
    wave_lds_sync();                                         // every lane has read its runs of the delta tiles 1 and 3
    if (active) {                                            // (idle lanes address the last row / map: they must not write)
#pragma unroll
        for (int j = 0; j < kS; ++j) { tile_tr[gc * kL + j * kS + ic] = acc[j]; acc[j] = 0.0f; }
    }
    direction(std::integral_constant<int, 0>{});
    direction(std::integral_constant<int, 2>{});

    // ---- merge: add the transposed sums and the skip term, store the row ---------------------------------------------
    float Dsum = 0.0f;
    if (p.Dv) Dsum = (p.Dv[d] + p.Dv[2 * p.D + d]) + (p.Dv[p.D + d] + p.Dv[3 * p.D + d]);
    wave_lds_sync();
    float out[kS];
#pragma unroll
    for (int j = 0; j < kS; ++j) {
        const float sums = acc[j] + tile_tr[gc * kL + ic * kS + j];
        out[j] = kSoftplus ? fmaf(sums, kLn2, Dsum * x_row.item(j)) : fmaf(Dsum, x_row.item(j), sums);
    }
    if (active) {
        float *yo = reinterpret_cast<float *>(p.y) + ((int64_t)(b0 + g) * p.D + d) * kL + i * kS;
        if constexpr (kS % 2 == 0) {
#pragma unroll
            for (int k = 0; k < kS / 2; ++k) reinterpret_cast<float2 *>(yo)[k] = make_float2(out[2 * k], out[2 * k + 1]);
        } else {
#pragma unroll
            for (int j = 0; j < kS; ++j) yo[j] = out[j];
        }
    }
}

bool core_small_eligible(const CoreArgs &a, int in_dtype) {
    if (in_dtype != SS2D_BF16 && in_dtype != SS2D_F16) return false;
    if (a.H != a.W || (a.H != 7 && a.H != 14)) return false;
    const int64_t L = a.L;
    // consecutive images adjacent in every stream (batch-innermost layout), all tile starts on 16-byte boundaries
    if (a.dl_bs != L || a.B_bs != L || a.C_bs != L) return false;
    auto al = [](const void *ptr, uintptr_t n) { return (reinterpret_cast<uintptr_t>(ptr) % n) == 0; };
    if (!al(a.delta, 16) || !al(a.Bm, 16) || !al(a.Cm, 16) || !al(a.x, 4) || !al(a.y, 8)) return false;
    if (a.dl_ks % 8 != 0 || a.dl_ds % 8 != 0 || a.B_ks % 8 != 0 || a.C_ks % 8 != 0) return false;
    return true;
}

template <typename in_t, int kS>
static int launch_core_small_typed(const CoreArgs &a, hipStream_t stream) {
    constexpr int kMaps = kWave / (kS <= 8 ? 8 : 16);
    const int tiles = (a.B + kMaps - 1) / kMaps;
    const int quads = (a.D + kSmallChans - 1) / kSmallChans;
    const int64_t n_wg = (int64_t)quads * tiles;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    const FastDiv dq = make_fastdiv((uint32_t)quads);
    if (a.softplus) hipLaunchKernelGGL((ss2d_core_small_kernel<in_t, kS, true>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream, a, quads, dq);
    else hipLaunchKernelGGL((ss2d_core_small_kernel<in_t, kS, false>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream, a, quads, dq);
    return launch_status();
}

int launch_core_small(const CoreArgs &a, int in_dtype, hipStream_t stream) {
    if (in_dtype == SS2D_BF16) {
        return a.H == 7 ? launch_core_small_typed<bf16_t, 7>(a, stream) : launch_core_small_typed<bf16_t, 14>(a, stream);
    }
    return a.H == 7 ? launch_core_small_typed<f16_t, 7>(a, stream) : launch_core_small_typed<f16_t, 14>(a, stream);
}

}  // namespace ss2d
