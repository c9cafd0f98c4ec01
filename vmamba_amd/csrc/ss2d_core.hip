// Fused SS2D core for one state per channel (d_state = 1, the VMamba-T/S/B setting):
//     CrossScan  ->  selective scan  ->  CrossMerge        in ONE kernel.
//
// The unfused path writes the four scan-ordered copies of x (xs), reads them back in the scan, writes the four
// scan outputs (ys) and reads them back in the merge: 62 bytes per activation element at bf16-in / fp32-out.
// Here a workgroup owns one channel d of CB images.  Its four wavefronts are the four scan directions:
//   * the CB x maps are loaded once and kept in LDS twice, in row-major order (xR) and in column-major order
//     (xT).  Direction 0 walks xR forwards, 2 walks it backwards, 1 walks xT forwards, 3 backwards: every
//     wavefront reads the u of ITS scan order with plain index arithmetic, and xs never exists;
//   * delta (from dt_proj) and the B / C rows (from x_proj) are streamed from HBM / L2 exactly as in the scan
//     kernels: 8 positions per lane, DPP wavefront scan, state carried in a register, softplus fused;
//   * each wavefront puts its outputs into an fp32 LDS plane at the position the merge wants them: plane A
//     (row-major index) collects directions 0 and 2, plane B (column-major index) directions 1 and 3.  Every
//     plane entry has exactly two writers, one forward and one backward direction; the planes start at zero and
//     both add, giving fl(y0 + y2) resp. fl(y1 + y3) -- the association order of cross_merge_fwd
//     (classification/models/csm_triton.py:61-62) -- and ys never exists.  LDS float atomics are an order of
//     magnitude slower than plain LDS traffic on this chip, so the updates are plain read-add-write sequences kept
//     apart by construction: the four wavefronts advance pass by pass, in each pass the forward directions update
//     the planes, a barrier, then the backward directions, a barrier;
//   * finally out[r] = (A[r] + B[t(r)]) + (D0 + D1 + D2 + D3) * x[r] is written once: the skip term D_k * u is the same
//     multiple of x[r] in all four directions, so it is added once here instead of once per direction and item.
// HBM traffic per element: x (s_in) + 4 delta (4 s_in) + out (s_out) = 14 bytes instead of 62.
//
// LDS banks: a lane owns 8 consecutive positions, so for a fixed item the 64 lanes touch addresses 8 apart, which
// would fold onto 4 of the 32 banks.  The fp32 planes therefore skip one 4-byte word after every 32 words
// (lds_index): lanes 0..31 of one access then fall into 32 different banks.  The maps are padded the same way only
// where they are read element by element; 16-bit maps walked in aligned blocks of 8 are read 16 bytes per lane,
// consecutive lanes consecutive addresses, and are plain arrays (map_index).
//
// Staging and merge work on 4 x 4 tiles of a map, one per thread, when H and W are multiples of 4: rows are 8-byte
// (staging) or 16-byte (merge) accesses on the row-major side, columns the same on the column-major side, and the
// transposition between them happens in registers.
//
// The CB images of a workgroup are walked as one stream per direction (restart by a = 0 at each image start, as
// in the flat scan kernel), which needs their delta rows adjacent in memory: delta is therefore taken with
// explicit (direction, channel, batch) strides and CB > 1 requires batch stride == L, i.e. the batch-innermost
// layout (K, D, B, L) that a single large dt_proj GEMM per direction produces.
#include <type_traits>

#include "scan_common.h"

namespace ss2d {

// Index of logical element a in an LDS array of kBytes-wide elements that skips one word after every 32 words.
template <int kBytes> __host__ __device__ __forceinline__ constexpr int lds_index(int a) {
    static_assert(kBytes == 2 || kBytes == 4, "16-bit or 32-bit elements");
    return kBytes == 4 ? a + (a >> 5) : a + ((a >> 6) << 1);
}
// Elements to allocate for n logical elements (a multiple of 16 bytes).
template <int kBytes> __host__ __device__ __forceinline__ constexpr int lds_extent(int n) {
    return (lds_index<kBytes>(n) + 8) & ~7;
}

// The x maps.  With 16-bit elements walked in aligned blocks of 8 (kFlat) every access of the passes is a 16-byte
// access of consecutive lanes, which needs no padding: the maps are then plain arrays.  Otherwise they skip words
// like the planes.  They carry one extra aligned block of kItems zeros behind the last image: groups past the end of
// the stream read their u there, so that u = 0 (and with it the drive term) needs no select.
template <int kBytes, bool kFlat> __host__ __device__ __forceinline__ constexpr int map_index(int a) {
    return kFlat ? a : lds_index<kBytes>(a);
}
__host__ __device__ __forceinline__ constexpr int core_zero_block(int n) { return (n + kItems - 1) & ~(kItems - 1); }
template <int kBytes, bool kFlat> __host__ __device__ __forceinline__ constexpr int core_map_extent(int n) {
    return kFlat ? core_zero_block(n) + kItems : lds_extent<kBytes>(core_zero_block(n) + kItems);
}
template <typename in_t, int kGran> constexpr bool core_flat_maps() { return sizeof(in_t) == 2 && kGran == kItems; }
// Positions per lane and pass: 8, or 16 (two blocks of 8, 1024 positions per pass; 16-bit maps walked in blocks only).
// With 16 the lane-local scan runs over 16 items and the wavefront scan, the plane bookkeeping and the loop are paid once
// per 1024 positions instead of once per 512; it needs more registers (five wavefronts per SIMD instead of six) and
// longer tiles, so the host picks it where a tile's LDS arrays keep a CU below six workgroups anyway.
template <bool kWide> constexpr int core_items() { return kWide ? 2 * kItems : kItems; }

// Wavefronts per SIMD the register allocation aims at: six for the 16-bit walks in blocks (what their LDS arrays allow;
// a few values that only live before and after the pass loop are then parked in scratch memory), four otherwise.
template <typename in_t, int kGran, bool kWide> constexpr int core_min_waves() { return sizeof(in_t) == 2 && kGran >= 4 && !kWide ? 6 : 4; }

constexpr int kCoreBurst = 2;     // passes whose delta / B / C loads are in flight per wavefront

// What one pass of one lane loads from memory, as it arrives.
template <typename in_t, int kGran, bool kWide>
struct CorePassLoads {
    static constexpr int kIt = core_items<kWide>();
    static constexpr int kGroups = kIt / kGran;
    static constexpr int kBlocks = kIt / kItems;
    static constexpr int kWords = gather_words<in_t, kGran>();
    Raw8<in_t> dl[kBlocks];
    uint32_t b[kGroups][kWords], c[kGroups][kWords];
    uint32_t img, j0;     // first element of the image (its index times L) and position in it of the lane's first item
};

// kWpd > 1: kWpd wavefronts per direction (8 or 16 in the workgroup), for maps whose LDS arrays leave a CU one or two
// workgroups -- four or eight wavefronts on a CU cannot hide the LDS round trips and barriers of the plane updates, which
// come one after the other.  The wavefronts of a direction take the passes of a ROUND of kWpd passes side by side:
// everything of a pass that does not need the incoming state -- loads, softplus, decays, the scan inside the lanes and
// across the wavefront -- then each leaves its pass's aggregate in LDS, a barrier, each folds the aggregates of the passes
// before its own into the state the round started from, and the plane updates of the whole round happen in the usual two
// phases (the passes of a round cover different positions, so the forward wavefronts do not meet each other, nor the
// backward ones).  Two barriers and two update phases per kWpd passes instead of per pass.
template <typename in_t, bool kSoftplus, int kGran, bool kVecDelta, bool kWide, int kWpd = 1>
__global__ __launch_bounds__(kWpd * kBlock, (kWpd > 1 ? 4 : core_min_waves<in_t, kGran, kWide>())) void ss2d_core_kernel(const CoreArgs p, FastDiv divL, FastDiv divW, FastDiv divD, FastDiv divTiles,
                                                           FastDiv divWt) {
    extern __shared__ __align__(16) float core_smem[];
    static_assert(kWpd == 1 || kWide, "several wavefronts per direction: the 16-positions-per-lane variant only");
    constexpr bool kPair = kWpd > 1;
    constexpr int kThreads = kWpd * kBlock;
    constexpr int kStride = kWpd;                        // passes from one pass of a wavefront to its next
    __shared__ float s_carry[4];                         // kWpd > 1: the state after the latest finished round, per direction
    __shared__ float2 s_agg[4][4];                       // ... and the aggregates of the current round's passes [direction][wavefront]
    constexpr int kEs = (int)sizeof(in_t);
    constexpr bool kFlat = core_flat_maps<in_t, kGran>();
    static_assert(!kWide || core_flat_maps<in_t, kGran>(), "16 positions per lane: 16-bit maps walked in blocks of 8 only");
    constexpr int kIt = core_items<kWide>();             // positions per lane and pass
    constexpr int kBlocks = kIt / kItems;
    constexpr int kGroups = kIt / kGran;
    constexpr int kPassLen = kWave * kIt;                // positions per pass
    // 16-bit streams with softplus: the step is kept in units of ln 2 (softplus_over_ln2), the decay is then
    // 2^(step * A) with A as given, the planes collect y / ln 2 and the merge multiplies by ln 2 once per position
    constexpr bool kBits = kSoftplus && sizeof(in_t) == 2;
    using Loads = CorePassLoads<in_t, kGran, kWide>;
    const int L = p.L, H = p.H;
    const int n_max = p.CB * L;
    const int plane_ext = lds_extent<4>(n_max), map_ext = core_map_extent<kEs, kFlat>(n_max);
    float *planeA = core_smem;                           // fl(y0 + y2), row-major index
    float *planeB = planeA + plane_ext;                  // fl(y1 + y3), column-major index
    in_t *xR = reinterpret_cast<in_t *>(planeB + plane_ext);
    in_t *xT = xR + map_ext;

    uint32_t bt, d;
    divmod(blockIdx.x, divD, bt, d);                     // neighbouring workgroups share B / C rows (same images)
    const int b0 = (int)bt * p.CB;
    const int nb = min(p.CB, p.B - b0);
    const int n_el = nb * L;

    // ---- this wavefront's direction ---------------------------------------------------------------------------
    const int lane = threadIdx.x & (kWave - 1);
    const int wave_id = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int dir = wave_id & 3, half = wave_id >> 2;    // (half is 0 without kPair)
    const int zero_block = core_zero_block(n_max);
    const in_t *xs = (dir & 1) ? xT : xR;
    float *plane = (dir & 1) ? planeB : planeA;
    const int kd = dir * p.D + (int)d;
    const in_t *dl_base = reinterpret_cast<const in_t *>(p.delta) + dir * p.dl_ks + (int64_t)d * p.dl_ds + b0 * p.dl_bs;
    const __amdgpu_buffer_rsrc_t dl_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<in_t *>(dl_base), 0, (n_el * kEs + 3) & ~3, kBufferRsrcWord3);
    const __amdgpu_buffer_rsrc_t B_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.Bm), 0, (int)p.B_span_bytes, kBufferRsrcWord3);
    const __amdgpu_buffer_rsrc_t C_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.Cm), 0, (int)p.C_span_bytes, kBufferRsrcWord3);
    const uint32_t B_soff = (uint32_t)(dir * p.B_ks + b0 * p.B_bs), C_soff = (uint32_t)(dir * p.C_ks + b0 * p.C_bs);
    const float A_log2e = kBits ? p.A[kd] : p.A[kd] * kLog2e;
    const float bias = p.bias ? p.bias[kd] : 0.0f;
    const bool reverse = dir >= 2;                       // uniform per wavefront
    const uint32_t u_sel = reverse ? 0x05040706u : 0x03020100u;
    // B / C rows of consecutive images adjacent in memory (what one x_proj GEMM per direction writes): a lane's offset
    // into them is its stream position
    const bool bc_dense = p.B_bs == L && p.C_bs == L;
    // passes of 512 or 1024 positions; a remainder of at most 64 positions is walked one position per lane instead
    const int tail_len = n_el % kPassLen;
    const bool short_tail = tail_len > 0 && tail_len <= kWave;
    const int n_pass = short_tail ? n_el / kPassLen : (n_el + kPassLen - 1) / kPassLen;

    // Image and position of this lane's first item in the pass issued next: passes are issued strictly in order, so
    // the pair just advances by 512 positions each time (no division in the loop).
    uint32_t next_img, next_j, step_img, step_j;
    divmod((uint32_t)(lane * kIt + half * kPassLen), divL, next_img, next_j);
    divmod((uint32_t)(kStride * kPassLen), divL, step_img, step_j);
    next_img *= (uint32_t)L; step_img *= (uint32_t)L;
    auto issue = [&](int pass, Loads &r) {
        const int e0 = pass * kPassLen + lane * kIt;
#pragma unroll
        for (int blk = 0; blk < kBlocks; ++blk) {
            if constexpr (kVecDelta) {
                // the stream starts 16-byte aligned (host-checked); the descriptor's range check returns 0 for the dwords
                // past its end.  What those items hold is immaterial: they follow every valid item of the stream, their u
                // is 0 and their outputs are never stored.
                const int byte_off = (e0 + blk * kItems) * kEs;
                const auto t0 = __builtin_amdgcn_raw_buffer_load_b128(dl_rsrc, byte_off, 0, 0);
                r.dl[blk].w[0] = t0[0]; r.dl[blk].w[1] = t0[1]; r.dl[blk].w[2] = t0[2]; r.dl[blk].w[3] = t0[3];
                if constexpr (kEs == 4) {
                    const auto t1 = __builtin_amdgcn_raw_buffer_load_b128(dl_rsrc, byte_off + 16, 0, 0);
                    r.dl[blk].w[4] = t1[0]; r.dl[blk].w[5] = t1[1]; r.dl[blk].w[6] = t1[2]; r.dl[blk].w[7] = t1[3];
                }
            } else {
                r.dl[blk] = load_raw<in_t, false>(dl_base, e0 + blk * kItems, n_el, delta_fill<kSoftplus>());
            }
        }
        r.img = next_img; r.j0 = next_j;
        next_img += step_img; next_j += step_j;
        if (next_j >= (uint32_t)L) { next_j -= (uint32_t)L; next_img += (uint32_t)L; }
        if (bc_dense) {                                  // uniform
#pragma unroll
            for (int gi = 0; gi < kGroups; ++gi) {
                gather_group_raw<in_t, kGran>(B_rsrc, (uint32_t)(e0 + gi * kGran), B_soff, r.b[gi]);
                gather_group_raw<in_t, kGran>(C_rsrc, (uint32_t)(e0 + gi * kGran), C_soff, r.c[gi]);
            }
            return;
        }
        uint32_t i0, rem;
        divmod(r.img, divL, i0, rem);
        const int k = kGran == kIt ? kIt : min(kIt, L - (int)r.j0);   // items before the next image starts
        const uint32_t B_a = i0 * (uint32_t)p.B_bs + r.j0, C_a = i0 * (uint32_t)p.C_bs + r.j0;   // image i0
        const uint32_t B_b = B_a + (uint32_t)p.B_bs - (uint32_t)(r.j0 + k), C_b = C_a + (uint32_t)p.C_bs - (uint32_t)(r.j0 + k);
#pragma unroll
        for (int gi = 0; gi < kGroups; ++gi) {
            const bool in_a = kGran == kIt ? true : gi * kGran < k;
            // image i0: position j0 + gi*kGran; image i0 + 1: position gi*kGran - k
            gather_group_raw<in_t, kGran>(B_rsrc, (in_a ? B_a : B_b) + gi * kGran, B_soff, r.b[gi]);
            gather_group_raw<in_t, kGran>(C_rsrc, (in_a ? C_a : C_b) + gi * kGran, C_soff, r.c[gi]);
        }
    };

    // the first passes' loads fly while the maps are staged
    Loads regs[kCoreBurst];
#pragma unroll
    for (int q = 0; q < kCoreBurst; ++q)
        if (kStride * q + half < n_pass) issue(kStride * q + half, regs[q]);

    // ---- stage: copy the maps into xR / xT ------------------------------------------------------------------------
    const in_t *xin = reinterpret_cast<const in_t *>(p.x);
    auto stage_elements = [&]() {
        constexpr int kChunk = 8;
        for (int base = 0; base < n_el; base += kChunk * kThreads) {
            in_t v[kChunk];
            uint32_t ii[kChunk], rr[kChunk];
#pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const int idx = base + u * kThreads + (int)threadIdx.x;
                divmod((uint32_t)min(idx, n_el - 1), divL, ii[u], rr[u]);
                v[u] = xin[((size_t)(b0 + ii[u]) * p.D + d) * L + rr[u]];
            }
#pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const int idx = base + u * kThreads + (int)threadIdx.x;
                if (idx < n_el) {
                    uint32_t h, w;
                    divmod(rr[u], divW, h, w);
                    xR[map_index<kEs, kFlat>(idx)] = v[u];
                    xT[map_index<kEs, kFlat>((int)(ii[u] * L + w * H + h))] = v[u];
                }
            }
        }
    };
    // Plain 16-bit maps, H and W multiples of 4, x 8-byte aligned (host-checked): one 4 x 4 tile of a map per thread.
    // Its four rows go into the row-major map as they are; its four columns are put together from the rows' dwords
    // with byte permutes and go into the column-major map, 8 bytes at a time.
    auto stage_tiles = [&]() {
        const int n_tiles = nb * (int)divTiles.d;        // tiles per image: (H / 4) * (W / 4)
        for (int q = threadIdx.x; q < n_tiles; q += kThreads) {
            uint32_t img, rest, hb, wb;
            divmod((uint32_t)q, divTiles, img, rest);
            divmod(rest, divWt, hb, wb);
            const int in_img = (int)hb * 4 * p.W + (int)wb * 4;
            const in_t *src = xin + ((size_t)(b0 + img) * p.D + d) * L + in_img;
            uint2 row[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) row[k] = *reinterpret_cast<const uint2 *>(src + k * p.W);
            in_t *dr = xR + (int)img * L + in_img;
            in_t *dt = xT + (int)img * L + (int)wb * 4 * H + (int)hb * 4;
#pragma unroll
            for (int k = 0; k < 4; ++k) *reinterpret_cast<uint2 *>(dr + k * p.W) = row[k];
            // column c: (row0[c], row1[c]) and (row2[c], row3[c]); element c of a row is half c % 2 of its dword c / 2
            const uint32_t r0[2] = {row[0].x, row[0].y}, r1[2] = {row[1].x, row[1].y};
            const uint32_t r2[2] = {row[2].x, row[2].y}, r3[2] = {row[3].x, row[3].y};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t sel = c % 2 ? 0x07060302u : 0x05040100u;    // (low source . half, high source . half)
                uint2 col;
                col.x = __builtin_amdgcn_perm(r1[c / 2], r0[c / 2], sel);
                col.y = __builtin_amdgcn_perm(r3[c / 2], r2[c / 2], sel);
                *reinterpret_cast<uint2 *>(dt + c * H) = col;
            }
        }
    };
    if constexpr (kFlat) {
        if (p.stage_tiles) stage_tiles();
        else stage_elements();
    } else {
        stage_elements();
    }
    // the merge planes start at zero (every entry is then updated by plain read-add-write, 0 + y being exact), and so
    // does the block behind the maps
    {
        float4 *planes4 = reinterpret_cast<float4 *>(planeA);
        for (int i = threadIdx.x; i < 2 * plane_ext / 4; i += kThreads) planes4[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if constexpr (kPair) {
            if (threadIdx.x < 4) s_carry[threadIdx.x] = 0.0f;
        }
        if (threadIdx.x < 2 * kItems) {
            in_t *m = threadIdx.x < kItems ? xR : xT;
            m[map_index<kEs, kFlat>(core_zero_block(n_max) + (int)(threadIdx.x % kItems))] = in_t{};
        }
    }
    __syncthreads();

    // ---- scan: 8 positions per lane per pass, loads kCoreBurst passes ahead ---------------------------------------
    // Where one group of kGran consecutive positions (never split between images) sits in the LDS arrays.
    struct GroupSlot {
        int plane_idx;     // index into the plane of the group's lowest logical index
        bool valid;        // inside the stream
    };

    // One pass: the states h of its items in yv (scan order) and the plane slots of its groups; the plane update
    // multiplies by C as it adds.  The skip term D * u is the same multiple of x[r] in all four directions and is added
    // once, in the merge.
    // kDefer (kPair): stops before the incoming state is needed -- yv receives the lane's running products, hv its states
    // from a zero start, ex the wavefront scan's (a_ex, h_ex, a_tot, h_tot) -- and apply_carry finishes the pass.
    struct WaveScan { float a_ex, h_ex, a_tot, h_tot; };
    auto compute = [&](bool reverse, int pass, const Loads &r, float &h_carry, float (&yv)[kIt], GroupSlot (&slot)[kGroups], auto defer_tag,
                       float (&hv)[kIt], WaveScan &ex) {
        constexpr bool kDefer = decltype(defer_tag)::value;
        const int e0 = pass * kPassLen + lane * kIt;
        const int j0 = (int)r.j0;
        const int k = kGran == kIt ? kIt : min(kIt, L - j0);
        const int img_base = (int)r.img;
        float dl[kIt], Bv[kIt], uv[kIt];
#pragma unroll
        for (int blk = 0; blk < kBlocks; ++blk) {
            float raw8[kItems], bias8[kItems], dl8[kItems];
            unpack_raw<in_t>(r.dl[blk], raw8);
            if constexpr (kBits) {
#pragma unroll
                for (int i = 0; i < kItems; ++i) dl8[i] = softplus_over_ln2(fmaf(raw8[i], kLog2e, bias * kLog2e));
            } else {
#pragma unroll
                for (int i = 0; i < kItems; ++i) bias8[i] = bias;
                delta_transform<kSoftplus>(raw8, bias8, dl8);
            }
#pragma unroll
            for (int i = 0; i < kItems; ++i) dl[blk * kItems + i] = dl8[i];
        }
        bool first[kGroups];
#pragma unroll
        for (int gi = 0; gi < kGroups; ++gi) {
            const bool in_a = kGran == kIt ? true : gi * kGran < k;
            const int jg = in_a ? j0 + gi * kGran : gi * kGran - k;          // position of the group in its image
            const int img_off = in_a ? img_base : img_base + L;              // img * L
            first[gi] = jg == 0;
            float bg[kGran];
            unpack_group<in_t, kGran>(r.b[gi], bg);
#pragma unroll
            for (int i = 0; i < kGran; ++i) Bv[gi * kGran + i] = bg[i];
            // The group's kGran logical indices in this direction's order are consecutive and kGran-aligned (L and
            // every group start are multiples of kGran): forwards they are the stream positions e0 + gi*kGran + t,
            // backwards img*L + L-1 - (jg + t), i.e. the block starting at img*L + L - jg - kGran read downwards.
            const bool valid = e0 + gi * kGran < n_el;
            int base = reverse ? img_off + L - jg - kGran : e0 + gi * kGran;
            base = valid ? base : zero_block;                                // past the end: u = 0
            slot[gi].valid = valid;
            slot[gi].plane_idx = lds_index<4>(base);
            const in_t *src = xs + map_index<kEs, kFlat>(base);              // no pad word inside an aligned block
            if constexpr (kFlat) {
                // one 16-byte read; backwards the four dwords are taken in the opposite order with their halves
                // exchanged, one byte permute each (the selector is uniform over the wavefront)
                const uint4 t = *reinterpret_cast<const uint4 *>(src);
                const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
                for (int jw = 0; jw < 4; ++jw) {
                    const uint32_t o = __builtin_amdgcn_perm(w[3 - jw], w[jw], u_sel);
                    uv[gi * kGran + 2 * jw] = to_f32(in_t{(uint16_t)(o & 0xffffu)});
                    uv[gi * kGran + 2 * jw + 1] = to_f32(in_t{(uint16_t)(o >> 16)});
                }
            } else {
                float um[kGran];
#pragma unroll
                for (int c = 0; c < kGran; ++c) um[c] = to_f32(src[c]);
#pragma unroll
                for (int t = 0; t < kGran; ++t) uv[gi * kGran + t] = reverse ? um[kGran - 1 - t] : um[t];
            }
        }
        float ac[kIt], hh[kIt];
#pragma unroll
        for (int i = 0; i < kIt; ++i) {
            // past the end of the stream delta was filled so that dl = 0 (softplus) or is zeroed here; u is 0 there and
            // B finite (the buffer load returns 0 out of range), so the pair is the identity (1, 0)
            if constexpr (!kSoftplus) dl[i] = slot[i / kGran].valid ? dl[i] : 0.0f;
            float a = __builtin_amdgcn_exp2f(dl[i] * A_log2e);
            if (i % kGran == 0) a = first[i / kGran] ? 0.0f : a;
            const float bb = Bv[i] * (dl[i] * uv[i]);
            ac[i] = i == 0 ? a : ac[i - 1] * a;
            hh[i] = i == 0 ? bb : fmaf(a, hh[i - 1], bb);
        }
        float a_ex, h_ex, a_tot, h_tot;
        wave_scan_pairs(ac[kIt - 1], hh[kIt - 1], a_ex, h_ex, a_tot, h_tot);
        if constexpr (kDefer) {
            ex.a_ex = a_ex; ex.h_ex = h_ex; ex.a_tot = a_tot; ex.h_tot = h_tot;
#pragma unroll
            for (int i = 0; i < kIt; ++i) { yv[i] = ac[i]; hv[i] = hh[i]; }
        } else {
            const float s_in = fmaf(a_ex, h_carry, h_ex);
            h_carry = fmaf(a_tot, h_carry, h_tot);
#pragma unroll
            for (int i = 0; i < kIt; ++i) yv[i] = fmaf(ac[i], s_in, hh[i]);
        }
    };
    // the rest of a deferred pass: the state that enters the round folded with the aggregates of the round's earlier passes;
    // returns the state after this pass
    auto apply_carry = [&](float (&yv)[kIt], const float (&hv)[kIt], const WaveScan &ex) {
        float h_carry = s_carry[dir];
#pragma unroll
        for (int w = 0; w < kWpd - 1; ++w) {
            const float2 g = s_agg[dir][w];
            if (w < half) h_carry = fmaf(g.x, h_carry, g.y);
        }
        const float s_in = fmaf(ex.a_ex, h_carry, ex.h_ex);
#pragma unroll
        for (int i = 0; i < kIt; ++i) yv[i] = fmaf(yv[i], s_in, hv[i]);
        return fmaf(ex.a_tot, h_carry, ex.h_tot);
    };

    // Plane update of one pass: every entry is reached once by the forward and once by the backward direction of its
    // plane; each adds its C * h to the zero-initialised entry with one fused multiply-add, so the entry ends as the
    // sum of the two outputs whatever the order (the first addition, into a zero, is the rounded product itself).  Only
    // when the two meet in the same pass could the read-add-write sequences overlap: the barrier between the two halves
    // of a pass keeps them apart.  C is widened here, from the registers it arrived in.
    auto update_plane = [&](bool reverse, const Loads &r, const float (&hv)[kIt], const GroupSlot (&slot)[kGroups]) {
#pragma unroll
        for (int gi = 0; gi < kGroups; ++gi) {
            if (slot[gi].valid) {
                float *dst = plane + slot[gi].plane_idx;
                float old[kGran], cg[kGran];
#pragma unroll
                for (int c = 0; c < kGran; ++c) old[c] = dst[c];
                unpack_group<in_t, kGran>(r.c[gi], cg);
#pragma unroll
                for (int c = 0; c < kGran; ++c) {
                    const int it = reverse ? kGran - 1 - c : c;
                    dst[c] = fmaf(cg[it], hv[gi * kGran + it], old[c]);
                }
            }
        }
    };

    // The short last pass: lane l holds stream position kPassLen * n_pass + l.  Same arithmetic and the same two-barrier
    // plane update as a full pass, one item per lane.
    auto short_pass = [&](bool reverse, float h_carry, bool active) {
        const int e = n_pass * kPassLen + lane;
        const bool valid = active && e < n_el;
        uint32_t i, jj;
        divmod((uint32_t)min(e, n_el - 1), divL, i, jj);
        const int base = reverse ? (int)(i * L) + L - 1 - (int)jj : e;      // this direction's index of the position
        float raw = 0.0f, Bv = 0.0f, Cv = 0.0f, u = 0.0f;
        if (valid) {
            raw = to_f32(dl_base[e]);
            Bv = gather_elem<in_t>(B_rsrc, B_soff + i * (uint32_t)p.B_bs + jj);
            Cv = gather_elem<in_t>(C_rsrc, C_soff + i * (uint32_t)p.C_bs + jj);
            u = to_f32(xs[map_index<kEs, kFlat>(base)]);
        }
        float dl;
        if constexpr (kBits) dl = softplus_over_ln2(fmaf(raw, kLog2e, bias * kLog2e));
        else dl = kSoftplus ? softplus_log2(fmaf(raw, kLog2e, bias * kLog2e)) : raw + bias;
        dl = valid ? dl : 0.0f;
        float a = __builtin_amdgcn_exp2f(dl * A_log2e);
        a = (valid && jj == 0) ? 0.0f : a;                                   // an image starts: the state restarts
        const float b = Bv * (dl * u);
        float a_ex, h_ex, a_tot, h_tot;
        wave_scan_pairs(a, b, a_ex, h_ex, a_tot, h_tot);
        const float h = fmaf(a, fmaf(a_ex, h_carry, h_ex), b);
        float *dst = plane + lds_index<4>(base);
        if (!reverse && valid) *dst = fmaf(Cv, h, *dst);
        __syncthreads();
        if (reverse && valid) *dst = fmaf(Cv, h, *dst);
        __syncthreads();
    };

    if constexpr (!kPair) {
        float h_carry = 0.0f;
        for (int pass0 = 0; pass0 < n_pass; pass0 += kCoreBurst) {
#pragma unroll
            for (int q = 0; q < kCoreBurst; ++q) {
                const int pass = pass0 + q;
                if (pass < n_pass) {                 // uniform over the workgroup: every wavefront meets every barrier
                    float yv[kIt];
                    GroupSlot slot[kGroups];
                    WaveScan unused;
                    compute(reverse, pass, regs[q], h_carry, yv, slot, std::false_type{}, yv, unused);
                    if (!reverse) update_plane(false, regs[q], yv, slot);
                    __syncthreads();
                    if (reverse) update_plane(true, regs[q], yv, slot);
                    __syncthreads();
                    if (pass + kCoreBurst < n_pass) issue(pass + kCoreBurst, regs[q]);
                }
            }
        }
        if (short_tail) short_pass(reverse, h_carry, true);
    } else {
        // rounds of kWpd passes: pass kWpd * round + w belongs to wavefront w of each direction
        const int n_round = (n_pass + kWpd - 1) / kWpd;
        for (int r0 = 0; r0 < n_round; r0 += kCoreBurst) {
#pragma unroll
            for (int q = 0; q < kCoreBurst; ++q) {
                const int round = r0 + q;
                if (round < n_round) {               // uniform over the workgroup
                    const int pass = kWpd * round + half;
                    const bool active = pass < n_pass;                          // uniform over the wavefront
                    const bool last = pass == min(kWpd * round + kWpd, n_pass) - 1;   // the round's last pass: its owner hands on the state
                    float yv[kIt], hv[kIt];
                    GroupSlot slot[kGroups];
                    WaveScan ex;
                    float unused = 0.0f;
                    if (active) {
                        compute(reverse, pass, regs[q], unused, yv, slot, std::true_type{}, hv, ex);
                        if (lane == 0 && half < kWpd - 1) s_agg[dir][half] = make_float2(ex.a_tot, ex.h_tot);
                    }
                    __syncthreads();                 // aggregates of this round, state and plane updates of the round before
                    float h_out = 0.0f;
                    if (active) h_out = apply_carry(yv, hv, ex);
                    if (active && !reverse) update_plane(false, regs[q], yv, slot);
                    __syncthreads();
                    if (active && reverse) update_plane(true, regs[q], yv, slot);
                    if (last && lane == 0) s_carry[dir] = h_out;               // (everyone has read the old one before the barrier above)
                    if (active && pass + kWpd * kCoreBurst < n_pass) issue(pass + kWpd * kCoreBurst, regs[q]);
                }
            }
        }
        __syncthreads();                             // the last state and the last plane updates are in place
        if (short_tail) short_pass(reverse, s_carry[dir], half == 0);
    }

    // ---- merge: out[r] = (A[r] + B[t(r)]) + (D0 + D1 + D2 + D3) * x[r] ---------------------------------------------
    float Dsum = 0.0f;
    if (p.Dv) Dsum = (p.Dv[d] + p.Dv[2 * p.D + (int)d]) + (p.Dv[p.D + (int)d] + p.Dv[3 * p.D + (int)d]);
    float *yo = reinterpret_cast<float *>(p.y);
    // (sum of the two planes, x) -> output: the planes hold y / ln 2 when the step was kept in units of ln 2
    auto finish = [&](float planes, float xv) {
        if constexpr (kBits) return fmaf(planes, kLn2, Dsum * xv);
        else return fmaf(Dsum, xv, planes);
    };
    if (p.tile_merge) {
        // H and W multiples of 4, y 16-byte aligned (host-checked): one 4 x 4 tile of a map per thread.  Its rows are
        // four consecutive entries of plane A each, its columns four consecutive entries of plane B each -- the
        // transposition is a renaming of registers -- and every row leaves as one 16-byte store.
        const int n_tiles = nb * (int)divTiles.d;
        for (int q = threadIdx.x; q < n_tiles; q += kThreads) {
            uint32_t img, rest, hb, wb;
            divmod((uint32_t)q, divTiles, img, rest);
            divmod(rest, divWt, hb, wb);
            const int in_img = (int)hb * 4 * p.W + (int)wb * 4;
            const int r0 = (int)img * L + in_img;
            const int t0 = (int)img * L + (int)wb * 4 * H + (int)hb * 4;
            float a[4][4], b[4][4], x[4][4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float *pa = planeA + lds_index<4>(r0 + k * p.W);      // no pad word inside an aligned group of 4
                const float *pb = planeB + lds_index<4>(t0 + k * H);
                const in_t *px = xR + map_index<kEs, kFlat>(r0 + k * p.W);
#pragma unroll
                for (int c = 0; c < 4; ++c) { a[k][c] = pa[c]; b[k][c] = pb[c]; x[k][c] = to_f32(px[c]); }
            }
            float *dst = yo + ((size_t)(b0 + img) * p.D + d) * L + in_img;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                *reinterpret_cast<float4 *>(dst + k * p.W) =
                    make_float4(finish(a[k][0] + b[0][k], x[k][0]), finish(a[k][1] + b[1][k], x[k][1]),
                                finish(a[k][2] + b[2][k], x[k][2]), finish(a[k][3] + b[3][k], x[k][3]));
        }
        return;
    }
    if (kGran >= 4 && p.vec_out && p.W >= 4) {
        // four consecutive positions per lane (L is a multiple of kGran, so they share an image and, with W >= 4, span
        // at most two rows): one 16-byte store
        const int n_quad = n_el / 4;
        for (int base = 0; base < n_quad; base += 2 * kThreads) {
            float4 v[2];
            size_t off[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int idx = 4 * min(base + u * kThreads + (int)threadIdx.x, n_quad - 1);
                uint32_t i, r, h, w;
                divmod((uint32_t)idx, divL, i, r);
                divmod(r, divW, h, w);
                const float *pa = planeA + lds_index<4>(idx);               // no pad word inside an aligned group of 4
                const in_t *px = xR + map_index<kEs, kFlat>(idx);
                const int n_first = p.W - (int)w;
                const int t0 = (int)(i * L + w * H + h), t1 = (int)(i * L + h + 1) - n_first * H;
                float o[4];
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    o[c] = finish(pa[c] + planeB[lds_index<4>((c < n_first ? t0 : t1) + c * H)], to_f32(px[c]));
                v[u] = make_float4(o[0], o[1], o[2], o[3]);
                off[u] = ((size_t)(b0 + i) * p.D + d) * L + r;
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
                if (base + u * kThreads + (int)threadIdx.x < n_quad) *reinterpret_cast<float4 *>(yo + off[u]) = v[u];
        }
        return;
    }
    for (int base = 0; base < n_el; base += 4 * kThreads) {
        float v[4];
        size_t off[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int idx = min(base + u * kThreads + (int)threadIdx.x, n_el - 1);
            uint32_t i, r, h, w;
            divmod((uint32_t)idx, divL, i, r);
            divmod(r, divW, h, w);
            v[u] = finish(planeA[lds_index<4>(idx)] + planeB[lds_index<4>((int)(i * L + w * H + h))],
                          to_f32(xR[map_index<kEs, kFlat>(idx)]));
            off[u] = ((size_t)(b0 + i) * p.D + d) * L + r;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (base + u * kThreads + (int)threadIdx.x < n_el) yo[off[u]] = v[u];
    }
}

// What a workgroup may have of the 160 KB of LDS of a CU: all of it.  Maps of up to ~13 000 positions then run as ONE
// workgroup per CU (four wavefronts), which still beats walking them twice in tiles (80 x 80 x 192 channels x 8 images: 59 us
// against 145; 112 x 112 x 96 x 64: 644 against 695).  The launch passes the size as dynamic shared memory and does NOT
// raise hipFuncAttributeMaxDynamicSharedMemorySize first: this runtime does not need it, and with the attribute set every
// launch of that instantiation, small maps included, ran as if it held the maximum.
constexpr size_t kCoreMaxLds = 160 * 1024 - 256;      // (the kernel has 144 bytes of static LDS besides the arrays)
constexpr size_t kCorePairLds = 53 * 1024;            // above a third of a CU's LDS: at most two workgroups per CU
constexpr size_t kCoreQuadLds = 80 * 1024;            // above half: one
constexpr size_t kCoreSixPerCu = 26 * 1024;     // a sixth of the 160 KB of LDS of a CU: the kernel's registers allow six wavefronts per SIMD

static int core_gcd(int64_t a, int64_t b) { while (b) { const int64_t t = a % b; a = b; b = t; } return (int)(a < 0 ? -a : a); }

// LDS bytes of a tile of n positions: two fp32 planes and two maps.
template <typename in_t> static size_t lds_bytes_of(int64_t n64, bool flat) {
    const int n = (int)n64;
    const int map_ext = flat ? core_map_extent<(int)sizeof(in_t), true>(n) : core_map_extent<(int)sizeof(in_t), false>(n);
    return 2 * (size_t)lds_extent<4>(n) * sizeof(float) + 2 * (size_t)map_ext * sizeof(in_t);
}

// Granularity of the B / C gathers and of the walk: the largest of 8, 4, 1 positions that divides L and every B / C
// stride and for which the B / C bases are aligned.
template <typename in_t>
static int64_t core_granularity(const CoreArgs &a) {
    int64_t g = core_gcd(a.L, kItems);
    const int64_t strides[] = {a.B_ks, a.B_bs, a.C_ks, a.C_bs};
    for (int64_t s : strides) g = core_gcd(g, s == 0 ? g : s);
    const uintptr_t bases = reinterpret_cast<uintptr_t>(a.Bm) | reinterpret_cast<uintptr_t>(a.Cm);
    while (g > 1 && (bases % (uintptr_t)(g * sizeof(in_t))) != 0) g /= 2;
    return g == 2 ? 1 : g;
}

// True when one image of this problem fits the LDS arrays of ss2d_core_kernel.
template <typename in_t>
static bool core_fits_lds(const CoreArgs &a) {
    const bool flat = sizeof(in_t) == 2 && core_granularity<in_t>(a) == kItems;
    return lds_bytes_of<in_t>(a.L, flat) <= kCoreMaxLds;
}

template <typename in_t>
static int launch_core(CoreArgs a, hipStream_t stream) {
    const int64_t L = a.L;
    const int64_t g = core_granularity<in_t>(a);
    const bool flat = sizeof(in_t) == 2 && g == kItems;       // core_flat_maps
    // 16 positions per lane and pass where one image alone takes more LDS than a sixth of a CU (the tile cannot be
    // shortened, six workgroups per CU are out of reach anyway); else 8, with tiles that let six workgroups share a CU
    const bool wide = flat && a.dl_bs == L && lds_bytes_of<in_t>(L, true) > kCoreSixPerCu;
    const int64_t pass_len = wide ? 2 * kPass : kPass;         // core_items * 64
    const size_t lds_cap = wide ? 40 * 1024 : kCoreSixPerCu;
    // Images per workgroup.  A workgroup walks its CB images as one stream in passes of 512 positions, so the last
    // pass of a tile is partly empty (a remainder of up to 64 positions costs little, see short_pass); CB is chosen to
    // minimise the passes of the whole batch among the tile sizes whose LDS arrays still let six workgroups share a
    // CU (~2200 positions; measured: more resident workgroups beat longer tiles).  A workgroup's first delta row sits
    // on a 16-byte boundary when CB*L is a multiple of 8 elements.
    auto lds_bytes = [&](int64_t cb) { return lds_bytes_of<in_t>(cb * L, flat); };
    const int64_t align_rows = 8 / core_gcd(L, 8);
    auto passes = [&](int64_t images) {                       // cost of a tile in tenths of a full pass
        const int64_t n = images * L, rem = n % pass_len;
        return 10 * (n / pass_len) + (rem == 0 ? 0 : rem <= kWave ? 3 : 10);
    };
    int64_t CB = 1;
    if (a.dl_bs == L) {                                       // adjacent delta rows need the batch-innermost layout
        int64_t best = -1;
        for (int64_t cb = align_rows; cb < a.B && lds_bytes(cb) <= lds_cap; cb += align_rows) {
            const int64_t cost = (a.B / cb) * passes(cb) + passes(a.B % cb);
            if (best < 0 || cost <= best) { best = cost; CB = cb; }
        }
        if (lds_bytes(a.B) <= lds_cap && (best < 0 || passes(a.B) <= best)) CB = a.B;   // a single tile starts at image 0
    }
    const size_t smem = lds_bytes(CB);
    if (smem > kCoreMaxLds) return SS2D_ENOTSUP;
    a.CB = (int)CB;
    // 16-byte loads of the delta stream need every (direction, channel, first image of a workgroup) start aligned;
    // otherwise the kernel loads element-wise
    const int64_t vec = 16 / (int64_t)sizeof(in_t);
    a.vec_ok = (reinterpret_cast<uintptr_t>(a.delta) % 16 == 0) && a.dl_ks % vec == 0 && a.dl_ds % vec == 0 &&
               (CB >= a.B || (CB * a.dl_bs) % vec == 0);
    a.vec_out = reinterpret_cast<uintptr_t>(a.y) % 16 == 0;   // 16-byte stores of the result (rows are multiples of 4 then)
    // 4 x 4 tiles of a map per thread for the staging of 16-bit maps (8-byte loads) and for the merge (16-byte stores)
    const bool tiled = a.H % 4 == 0 && a.W % 4 == 0;
    a.stage_tiles = flat && tiled && reinterpret_cast<uintptr_t>(a.x) % 8 == 0;
    a.tile_merge = tiled && a.vec_out;
    const int64_t tiles = (a.B + CB - 1) / CB;
    const int64_t n_wg = tiles * a.D;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    const FastDiv dL = make_fastdiv((uint32_t)L), dW = make_fastdiv((uint32_t)a.W), dD = make_fastdiv((uint32_t)a.D);
    const FastDiv dT = make_fastdiv((uint32_t)(tiled ? (a.H / 4) * (a.W / 4) : 1)), dWt = make_fastdiv((uint32_t)(tiled ? a.W / 4 : 1));
    // several wavefronts per direction where the arrays leave a CU two workgroups (two each) or one (four)
    const int wpd = !(wide && smem > kCorePairLds) ? 1 : smem > kCoreQuadLds ? 4 : 2;
#define SS2D_CORE_LAUNCH_W(SP, G, V, W16)                                                                                         \
    hipLaunchKernelGGL((ss2d_core_kernel<in_t, SP, G, V, W16>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, a, dL, dW, dD, dT, dWt)
#define SS2D_CORE_LAUNCH_P(SP, G, V, WPD)                                                                                         \
    hipLaunchKernelGGL((ss2d_core_kernel<in_t, SP, G, V, true, WPD>), dim3((uint32_t)n_wg), dim3(WPD * kBlock), smem, stream, a, dL, dW, dD, dT, dWt)
#define SS2D_CORE_LAUNCH(SP, G)                                                                                                     \
    do {                                                                                                                            \
        if constexpr (G == kItems && sizeof(in_t) == 2) {                                                                          \
            if (wpd == 4) { if (a.vec_ok) SS2D_CORE_LAUNCH_P(SP, G, true, 4); else SS2D_CORE_LAUNCH_P(SP, G, false, 4); break; }  \
            if (wpd == 2) { if (a.vec_ok) SS2D_CORE_LAUNCH_P(SP, G, true, 2); else SS2D_CORE_LAUNCH_P(SP, G, false, 2); break; }  \
            if (wide) { if (a.vec_ok) SS2D_CORE_LAUNCH_W(SP, G, true, true); else SS2D_CORE_LAUNCH_W(SP, G, false, true); break; } \
        }                                                                                                                           \
        if (a.vec_ok) SS2D_CORE_LAUNCH_W(SP, G, true, false); else SS2D_CORE_LAUNCH_W(SP, G, false, false);                         \
    } while (0)
    if (a.softplus) {
        if (g == 8) SS2D_CORE_LAUNCH(true, 8); else if (g == 4) SS2D_CORE_LAUNCH(true, 4); else SS2D_CORE_LAUNCH(true, 1);
    } else {
        if (g == 8) SS2D_CORE_LAUNCH(false, 8); else if (g == 4) SS2D_CORE_LAUNCH(false, 4); else SS2D_CORE_LAUNCH(false, 1);
    }
#undef SS2D_CORE_LAUNCH_W
#undef SS2D_CORE_LAUNCH_P
#undef SS2D_CORE_LAUNCH
    return launch_status();
}

}  // namespace ss2d

namespace ss2d {

// Validation shared by the core's entry points.  Returns SS2D_OK with `a` filled, 1 for an empty problem, or a negative status.
static int core_args(const ss2d_core_params *q, CoreArgs &a) {
    if (!q) return SS2D_EINVAL;
    if (q->batch < 0 || q->dim < 0 || q->height < 0 || q->width < 0) return SS2D_EINVAL;
    if (q->in_dtype != SS2D_F32 && q->in_dtype != SS2D_BF16 && q->in_dtype != SS2D_F16) return SS2D_EINVAL;
    if (q->batch == 0 || q->dim == 0 || q->height == 0 || q->width == 0) return 1;
    if (!q->x || !q->delta || !q->A || !q->B || !q->C || !q->y) return SS2D_EINVAL;
    const int64_t L = (int64_t)q->height * q->width;
    if (L < kItems || L > 0x0fffffff) return SS2D_ENOTSUP;
    if (q->delta_batch_stride < 0 || q->delta_dir_stride < 0 || q->delta_dim_stride < 0 || q->B_dir_stride < 0 ||
        q->B_batch_stride < 0 || q->C_dir_stride < 0 || q->C_batch_stride < 0) return SS2D_EINVAL;
    a.x = q->x; a.delta = q->delta; a.Bm = q->B; a.Cm = q->C;
    a.A = (const float *)q->A; a.Dv = (const float *)q->D; a.bias = (const float *)q->delta_bias;
    a.y = q->y;
    a.B = q->batch; a.D = q->dim; a.H = q->height; a.W = q->width; a.L = (int32_t)L;
    a.softplus = q->delta_softplus;
    a.dl_ks = q->delta_dir_stride; a.dl_ds = q->delta_dim_stride; a.dl_bs = q->delta_batch_stride;
    a.B_ks = q->B_dir_stride; a.B_bs = q->B_batch_stride; a.C_ks = q->C_dir_stride; a.C_bs = q->C_batch_stride;
    const int64_t eb = q->in_dtype == SS2D_F32 ? 4 : 2;
    // extents in whole 16-byte pieces: a vector load that straddles the extent loses more than the bytes behind it, and
    // rows of odd length end in the middle of a piece (the rest of that piece lies in the same 16-byte block of memory)
    const int64_t B_span = ((3 * a.B_ks + (int64_t)(a.B - 1) * a.B_bs + L) * eb + 15) & ~(int64_t)15;
    const int64_t C_span = ((3 * a.C_ks + (int64_t)(a.B - 1) * a.C_bs + L) * eb + 15) & ~(int64_t)15;
    if (B_span >= 0x7fffffffll || C_span >= 0x7fffffffll) return SS2D_ENOTSUP;
    a.B_span_bytes = (uint32_t)B_span; a.C_span_bytes = (uint32_t)C_span;
    a.CB = 1; a.vec_ok = 0; a.vec_out = 0; a.stage_tiles = 0; a.tile_merge = 0;
    return SS2D_OK;
}

// True when the single-kernel core (whole maps in LDS) takes this problem.
static bool core_single_kernel(const CoreArgs &a, int in_dtype) {
    if (core_small_eligible(a, in_dtype)) return true;
    return in_dtype == SS2D_F32 ? core_fits_lds<float>(a) : core_fits_lds<bf16_t>(a);
}

static int core_launch_single(const CoreArgs &a, int in_dtype, hipStream_t s) {
    // 7 x 7 and 14 x 14 maps in the batch-innermost layout: one map row per lane, everything in registers
    if (core_small_eligible(a, in_dtype)) return launch_core_small(a, in_dtype, s);
    if (in_dtype == SS2D_F32) return launch_core<float>(a, s);
    if (in_dtype == SS2D_BF16) return launch_core<bf16_t>(a, s);
    return launch_core<f16_t>(a, s);
}

}  // namespace ss2d

extern "C" int ss2d_core_fwd(const ss2d_core_params *q, void *stream) {
    using namespace ss2d;
    CoreArgs a;
    const int rc = core_args(q, a);
    if (rc != SS2D_OK) return rc > 0 ? SS2D_OK : rc;
    return core_launch_single(a, q->in_dtype, (hipStream_t)stream);
}

extern "C" int64_t ss2d_core_workspace_bytes(const ss2d_core_params *q) {
    using namespace ss2d;
    CoreArgs a;
    const int rc = core_args(q, a);
    if (rc != SS2D_OK) return rc > 0 ? 0 : rc;
    if (core_single_kernel(a, q->in_dtype)) return 0;
    if (!core_tiled_eligible(a, q->in_dtype)) return SS2D_ENOTSUP;
    return core_tiled_workspace_bytes(a);
}

extern "C" int ss2d_core_fwd_ws(const ss2d_core_params *q, void *workspace, int64_t workspace_bytes, void *stream) {
    using namespace ss2d;
    CoreArgs a;
    const int rc = core_args(q, a);
    if (rc != SS2D_OK) return rc > 0 ? SS2D_OK : rc;
    hipStream_t s = (hipStream_t)stream;
    if (core_single_kernel(a, q->in_dtype)) return core_launch_single(a, q->in_dtype, s);
    if (!core_tiled_eligible(a, q->in_dtype)) return SS2D_ENOTSUP;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) % 16) != 0) return SS2D_EINVAL;
    if (workspace_bytes < core_tiled_workspace_bytes(a)) return SS2D_ENOMEM;
    return launch_core_tiled(a, q->in_dtype, workspace, s);
}

// ---- CrossScan, one-by-one --------------------------------------------------------------
// Each of the four direction slices of x (B,4,C,H,W) is laid out in ITS scan order (cross_scan1b1_fwd,
// classification/models/csm_triton.py:88-131, scans = 0).  One workgroup per (b, k, c) map; the transposing
// directions go through an LDS copy of the map with an odd row pitch.
namespace ss2d {

template <typename T>
__global__ __launch_bounds__(kBlock) void cross_scan_1b1_kernel(const T *__restrict__ x, T *__restrict__ y, int H, int W,
                                                                int Wp, int use_lds, int64_t y_bs, int64_t y_ks,
                                                                int64_t y_cs, FastDiv divC, FastDiv divW, FastDiv divH) {
    extern __shared__ __align__(16) unsigned char map_smem[];
    T *tile = reinterpret_cast<T *>(map_smem);
    uint32_t bk, c;
    divmod(blockIdx.x, divC, bk, c);
    const uint32_t b = bk / 4, k = bk % 4;
    const int L = H * W;
    const T *src = x + (size_t)blockIdx.x * L;
    T *dst = y + (int64_t)b * y_bs + (int64_t)k * y_ks + (int64_t)c * y_cs;
    if ((k & 1u) == 0) {
        for (int j = threadIdx.x; j < L; j += kBlock) dst[j] = src[k == 0 ? j : L - 1 - j];
        return;
    }
    if (use_lds) {
        for (int r = threadIdx.x; r < L; r += kBlock) {
            uint32_t h, w;
            divmod((uint32_t)r, divW, h, w);
            tile[h * Wp + w] = src[r];
        }
        __syncthreads();
    }
    for (int j = threadIdx.x; j < L; j += kBlock) {
        uint32_t w, h;
        divmod((uint32_t)(k == 1 ? j : L - 1 - j), divH, w, h);
        dst[j] = use_lds ? tile[h * Wp + w] : src[h * W + w];
    }
}

// Large maps: one workgroup per 64 x 64 tile of a map.  Rows are read along W; the row-major directions store them as
// they are (forwards or mirrored), the column-major ones read the tile back down its columns from LDS (pitch 65) and
// store along H, so both sides of every direction are contiguous per wavefront.
constexpr int k1b1Tile = 64;
template <typename T>
__global__ __launch_bounds__(kBlock) void cross_scan_1b1_tile_kernel(const T *__restrict__ x, T *__restrict__ y, int H, int W,
                                                                     int tiles_h, int tiles_w, int64_t y_bs, int64_t y_ks,
                                                                     int64_t y_cs, FastDiv divC) {
    __shared__ T tile[k1b1Tile * (k1b1Tile + 1)];
    const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    uint32_t wg = blockIdx.x;
    const uint32_t tw = wg % (uint32_t)tiles_w; wg /= (uint32_t)tiles_w;
    const uint32_t th = wg % (uint32_t)tiles_h; wg /= (uint32_t)tiles_h;      // wg: the map (b, k, c)
    uint32_t bk, c;
    divmod(wg, divC, bk, c);
    const uint32_t b = bk / 4, k = bk % 4;
    const size_t L = (size_t)H * W;
    const T *src = x + (size_t)wg * L;
    T *dst = y + (int64_t)b * y_bs + (int64_t)k * y_ks + (int64_t)c * y_cs;
    const uint32_t h0 = th * k1b1Tile, w0 = tw * k1b1Tile;
    const bool column_major = (k & 1u) != 0, mirrored = k >= 2;
    for (uint32_t rr = wave; rr < (uint32_t)k1b1Tile; rr += kBlock / kWave) {
        const uint32_t h = h0 + rr, w = w0 + lane;
        if (h < (uint32_t)H && w < (uint32_t)W) {
            const size_t r = (size_t)h * W + w;
            const T v = src[r];
            if (column_major) tile[rr * (k1b1Tile + 1) + lane] = v;
            else dst[mirrored ? L - 1 - r : r] = v;
        }
    }
    if (!column_major) return;                 // uniform over the workgroup
    __syncthreads();
    for (uint32_t cc = wave; cc < (uint32_t)k1b1Tile; cc += kBlock / kWave) {
        const uint32_t w = w0 + cc, h = h0 + lane;
        if (h < (uint32_t)H && w < (uint32_t)W) {
            const size_t t = (size_t)w * H + h;
            dst[mirrored ? L - 1 - t : t] = tile[lane * (k1b1Tile + 1) + cc];
        }
    }
}

// Short maps (L <= 1024): one WAVEFRONT per map, four maps per workgroup, each with a private LDS tile -- a whole
// workgroup per 49- or 196-element map leaves most of its lanes idle and the launch is then bound by workgroup count.
template <typename T>
__global__ __launch_bounds__(kBlock) void cross_scan_1b1_wave_kernel(const T *__restrict__ x, T *__restrict__ y, int H, int W,
                                                                     int Wp, int64_t n_maps, int64_t y_bs, int64_t y_ks,
                                                                     int64_t y_cs, FastDiv divC, FastDiv divW, FastDiv divH) {
    extern __shared__ __align__(16) unsigned char map_smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int64_t map = (int64_t)blockIdx.x * (kBlock / kWave) + wave;
    if (map >= n_maps) return;                 // whole wavefront leaves; no workgroup barrier in this kernel
    T *tile = reinterpret_cast<T *>(map_smem) + (size_t)wave * H * Wp;
    uint32_t bk, c;
    divmod((uint32_t)map, divC, bk, c);
    const uint32_t b = bk / 4, k = bk % 4;
    const int L = H * W;
    const T *src = x + (size_t)map * L;
    T *dst = y + (int64_t)b * y_bs + (int64_t)k * y_ks + (int64_t)c * y_cs;
    if ((k & 1u) == 0) {
        for (int j = lane; j < L; j += kWave) dst[j] = src[k == 0 ? j : L - 1 - j];
        return;
    }
    for (int r = lane; r < L; r += kWave) {
        uint32_t h, w;
        divmod((uint32_t)r, divW, h, w);
        tile[h * Wp + w] = src[r];
    }
    wave_lds_sync();
    for (int j = lane; j < L; j += kWave) {
        uint32_t w, h;
        divmod((uint32_t)(k == 1 ? j : L - 1 - j), divH, w, h);
        dst[j] = tile[h * Wp + w];
    }
}

// One workgroup per map, 16-bit maps with an even number of positions on 4-byte boundaries: two positions per lane and
// memory instruction (see the wavefront variant below).
__global__ __launch_bounds__(kBlock) void cross_scan_1b1_pairs_kernel(const uint16_t *__restrict__ x, uint16_t *__restrict__ y, int H,
                                                                      int W, int Wp, int64_t y_bs, int64_t y_ks, int64_t y_cs,
                                                                      FastDiv divC, FastDiv divW, FastDiv divH) {
    extern __shared__ __align__(16) unsigned char map_smem[];
    uint16_t *tile = reinterpret_cast<uint16_t *>(map_smem);
    uint32_t bk, c;
    divmod(blockIdx.x, divC, bk, c);
    const uint32_t b = bk / 4, k = bk % 4;
    const int L = H * W, P = L / 2;
    const uint32_t *src = reinterpret_cast<const uint32_t *>(x + (size_t)blockIdx.x * L);
    uint32_t *dst = reinterpret_cast<uint32_t *>(y + (int64_t)b * y_bs + (int64_t)k * y_ks + (int64_t)c * y_cs);
    if ((k & 1u) == 0) {
        for (int q = threadIdx.x; q < P; q += kBlock) {
            const uint32_t v = src[k == 0 ? q : P - 1 - q];
            dst[q] = k == 0 ? v : (v >> 16) | (v << 16);
        }
        return;
    }
    for (int q = threadIdx.x; q < P; q += kBlock) {
        const uint32_t v = src[q];
        uint32_t h, w;
        divmod((uint32_t)(2 * q), divW, h, w);
        tile[h * Wp + w] = (uint16_t)(v & 0xffffu);
        if (++w == (uint32_t)W) { w = 0; ++h; }
        tile[h * Wp + w] = (uint16_t)(v >> 16);
    }
    __syncthreads();
    for (int q = threadIdx.x; q < P; q += kBlock) {
        uint32_t e[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int j = 2 * q + i;
            uint32_t w, h;
            divmod((uint32_t)(k == 1 ? j : L - 1 - j), divH, w, h);
            e[i] = tile[h * Wp + w];
        }
        dst[q] = e[0] | (e[1] << 16);
    }
}

// The same for 16-bit maps with an even number of positions whose rows start on 4-byte boundaries on both sides: two
// positions per lane and memory instruction (the reversed routes swap the halves; the transposing routes pick the two
// elements from the LDS copy).
__global__ __launch_bounds__(kBlock) void cross_scan_1b1_wave_pairs_kernel(const uint16_t *__restrict__ x, uint16_t *__restrict__ y,
                                                                           int H, int W, int Wp, int64_t n_maps, int64_t y_bs,
                                                                           int64_t y_ks, int64_t y_cs, FastDiv divC, FastDiv divW,
                                                                           FastDiv divH) {
    extern __shared__ __align__(16) unsigned char map_smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int64_t map = (int64_t)blockIdx.x * (kBlock / kWave) + wave;
    if (map >= n_maps) return;                 // whole wavefront leaves; no workgroup barrier in this kernel
    uint16_t *tile = reinterpret_cast<uint16_t *>(map_smem) + (size_t)wave * H * Wp;
    uint32_t bk, c;
    divmod((uint32_t)map, divC, bk, c);
    const uint32_t b = bk / 4, k = bk % 4;
    const int L = H * W, P = L / 2;
    const uint32_t *src = reinterpret_cast<const uint32_t *>(x + (size_t)map * L);
    uint32_t *dst = reinterpret_cast<uint32_t *>(y + (int64_t)b * y_bs + (int64_t)k * y_ks + (int64_t)c * y_cs);
    if ((k & 1u) == 0) {
        for (int q = lane; q < P; q += kWave) {
            const uint32_t v = src[k == 0 ? q : P - 1 - q];
            dst[q] = k == 0 ? v : (v >> 16) | (v << 16);
        }
        return;
    }
    for (int q = lane; q < P; q += kWave) {
        const uint32_t v = src[q];
        uint32_t h, w;
        divmod((uint32_t)(2 * q), divW, h, w);
        tile[h * Wp + w] = (uint16_t)(v & 0xffffu);
        if (++w == (uint32_t)W) { w = 0; ++h; }
        tile[h * Wp + w] = (uint16_t)(v >> 16);
    }
    wave_lds_sync();
    for (int q = lane; q < P; q += kWave) {
        uint32_t e[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int j = 2 * q + i;
            uint32_t w, h;
            divmod((uint32_t)(k == 1 ? j : L - 1 - j), divH, w, h);
            e[i] = tile[h * Wp + w];
        }
        dst[q] = e[0] | (e[1] << 16);
    }
}

template <typename T>
static int launch_cross_scan_1b1(const void *x, void *y, int B, int C, int H, int W, int64_t y_bs, int64_t y_ks, int64_t y_cs,
                                 hipStream_t stream) {
    const int64_t n_wg = (int64_t)B * 4 * C;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    const int Wp = W | 1;
    size_t smem = (size_t)H * Wp * sizeof(T);
    if ((int64_t)H * W <= 1024 && smem * (kBlock / kWave) <= 48 * 1024) {
        const int64_t n = (n_wg + kBlock / kWave - 1) / (kBlock / kWave);
        if constexpr (sizeof(T) == 2) {
            const bool even = ((int64_t)H * W) % 2 == 0 && y_bs % 2 == 0 && y_ks % 2 == 0 && y_cs % 2 == 0 &&
                              (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) % 4 == 0;
            if (even) {
                hipLaunchKernelGGL(cross_scan_1b1_wave_pairs_kernel, dim3((uint32_t)n), dim3(kBlock), smem * (kBlock / kWave), stream,
                                   (const uint16_t *)x, (uint16_t *)y, H, W, Wp, n_wg, y_bs, y_ks, y_cs, make_fastdiv((uint32_t)C),
                                   make_fastdiv((uint32_t)W), make_fastdiv((uint32_t)H));
                return launch_status();
            }
        }
        hipLaunchKernelGGL((cross_scan_1b1_wave_kernel<T>), dim3((uint32_t)n), dim3(kBlock), smem * (kBlock / kWave), stream, (const T *)x,
                           (T *)y, H, W, Wp, n_wg, y_bs, y_ks, y_cs, make_fastdiv((uint32_t)C), make_fastdiv((uint32_t)W),
                           make_fastdiv((uint32_t)H));
        return launch_status();
    }
    // maps too large for one workgroup's LDS, or few large maps (a workgroup per map would leave most of the chip idle)
    const bool by_tiles = smem > 48 * 1024 || ((int64_t)H * W >= 8192 && n_wg < 2048);
    const int use_lds = !by_tiles;
    if constexpr (sizeof(T) == 2) {
        const bool even = ((int64_t)H * W) % 2 == 0 && y_bs % 2 == 0 && y_ks % 2 == 0 && y_cs % 2 == 0 &&
                          (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) % 4 == 0;
        if (even && use_lds) {
            hipLaunchKernelGGL(cross_scan_1b1_pairs_kernel, dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, (const uint16_t *)x,
                               (uint16_t *)y, H, W, Wp, y_bs, y_ks, y_cs, make_fastdiv((uint32_t)C), make_fastdiv((uint32_t)W),
                               make_fastdiv((uint32_t)H));
            return launch_status();
        }
    }
    if (!use_lds) {
        const int tiles_h = (H + k1b1Tile - 1) / k1b1Tile, tiles_w = (W + k1b1Tile - 1) / k1b1Tile;
        const int64_t n_tiles = n_wg * tiles_h * tiles_w;
        if (n_tiles <= 0x7fffffff) {
            hipLaunchKernelGGL((cross_scan_1b1_tile_kernel<T>), dim3((uint32_t)n_tiles), dim3(kBlock), 0, stream, (const T *)x, (T *)y,
                               H, W, tiles_h, tiles_w, y_bs, y_ks, y_cs, make_fastdiv((uint32_t)C));
            return launch_status();
        }
        smem = 0;
    }
    hipLaunchKernelGGL((cross_scan_1b1_kernel<T>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, (const T *)x, (T *)y, H, W, Wp,
                       use_lds, y_bs, y_ks, y_cs, make_fastdiv((uint32_t)C), make_fastdiv((uint32_t)W), make_fastdiv((uint32_t)H));
    return launch_status();
}

}  // namespace ss2d

extern "C" int ss2d_cross_scan_1b1(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int64_t y_batch_stride,
                                   int64_t y_dir_stride, int64_t y_chan_stride, void *stream) {
    using namespace ss2d;
    if (B < 0 || C < 0 || H < 0 || W < 0) return SS2D_EINVAL;
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return SS2D_EINVAL;
    if (B == 0 || C == 0 || H == 0 || W == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    if ((int64_t)H * W > 0x3fffffff) return SS2D_ENOTSUP;
    if (y_batch_stride < 0 || y_dir_stride < 0 || y_chan_stride < 0) return SS2D_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    switch (elem_bytes) {
        case 1: return launch_cross_scan_1b1<uint8_t>(x, y, B, C, H, W, y_batch_stride, y_dir_stride, y_chan_stride, s);
        case 2: return launch_cross_scan_1b1<uint16_t>(x, y, B, C, H, W, y_batch_stride, y_dir_stride, y_chan_stride, s);
        case 4: return launch_cross_scan_1b1<uint32_t>(x, y, B, C, H, W, y_batch_stride, y_dir_stride, y_chan_stride, s);
        default: return launch_cross_scan_1b1<uint64_t>(x, y, B, C, H, W, y_batch_stride, y_dir_stride, y_chan_stride, s);
    }
}
