// Selective-scan forward for several states per channel (d_state 4 / 8 / 16 / 32): one CHANNEL per lane, walked
// serially along the sequence.
//
// With N states the work per position is N recurrences  h_n = a_n h_n + B_n du,  y += C_n h_n.  The wavefront-scan
// kernels (selective_scan.hip) pay a 64-lane DPP scan per (512 positions, state) and fetch B / C per lane.  Here the
// 64 lanes of a wavefront are 64 channels of one (image, group): all of them meet the same B_n,t and C_n,t, so these
// are wave-uniform values that ride in scalar registers (the loads below have uniform addresses), the recurrence is a
// plain serial chain per lane -- multiply, exp2, multiply, two fused multiply-adds per (position, state) -- and no
// scan, no carry logic and no per-lane B / C traffic remain.
//
// Parallelism: a workgroup owns 64 channels; its four wavefronts split the STATES (N/4 each), so each keeps N/4
// independent chains in flight, and their partial sums over n meet in LDS.  Per step of 32 positions:
//   stage    thread (row r = tid/4, quarter q) loads 2 x 4 positions of u and delta of channel r (the next step's loads
//            are issued before this step's arithmetic), computes dl = softplus(delta + bias), du = dl u and the skip
//            term D u, and writes dl / du into LDS tiles [channel][position] -- the transposition that lets global
//            accesses run along the sequence while the compute phase reads along channels;
//   compute  twice 16 positions: every lane reads its channel's dl / du (16-byte LDS reads), runs its wavefront's
//            states over them and leaves 16 partial outputs in LDS;
//   combine  thread (r, q) adds the four partials and the skip term for 4 positions and stores them (16 bytes of fp32).
#include "scan_common.h"

namespace ss2d {

constexpr int kChanTile = 32;                     // positions staged per step
constexpr int kChanSub = 16;                      // positions per compute / combine round
constexpr int kChanTilePitch = kChanTile + 4;     // floats; + 4 spreads the 16-byte reads of 8 lanes over all banks
constexpr int kChanSubPitch = kChanSub + 4;
constexpr int kChanBlock = 64;                    // channels per workgroup

// The B and C values of one state for one round of 16 positions, as loaded: two halves of 8 positions, each at a
// wave-uniform, 16-byte aligned address.  The addresses are uniform and the memory is read-only for the kernel, so these
// are scalar loads and the widening to fp32 is scalar ALU work.
template <typename in_t> struct UniRaw {
    static constexpr int kVecs = (int)sizeof(in_t);      // 16-byte pieces per 16 elements
    uint4 b[kVecs], c[kVecs];
};

template <typename in_t>
__device__ __forceinline__ void load_uniform(const in_t *__restrict__ Brow, const in_t *__restrict__ Crow, int half0, int half1,
                                             UniRaw<in_t> &r) {
    constexpr int kHalfVecs = UniRaw<in_t>::kVecs / 2;  // 1 (16-bit) or 2 (fp32) pieces per 8 elements
    constexpr int kPer = 16 / (int)sizeof(in_t);
#pragma unroll
    for (int v = 0; v < kHalfVecs; ++v) {
        r.b[v] = *reinterpret_cast<const uint4 *>(Brow + half0 + v * kPer);
        r.b[kHalfVecs + v] = *reinterpret_cast<const uint4 *>(Brow + half1 + v * kPer);
        r.c[v] = *reinterpret_cast<const uint4 *>(Crow + half0 + v * kPer);
        r.c[kHalfVecs + v] = *reinterpret_cast<const uint4 *>(Crow + half1 + v * kPer);
    }
}

// Makes the compiler wait here until every dword of r has arrived (it places its wait before the first use of a loaded
// register, and scalar loads complete out of order, so that wait is for all outstanding ones): put in front of the
// NEXT set of requests, it keeps them out of the wait for this set.
template <typename in_t>
__device__ __forceinline__ void arrived(const UniRaw<in_t> &r) {
#pragma unroll
    for (int v = 0; v < UniRaw<in_t>::kVecs; ++v)
        asm volatile("" ::"s"(r.b[v].x), "s"(r.b[v].y), "s"(r.b[v].z), "s"(r.b[v].w), "s"(r.c[v].x), "s"(r.c[v].y), "s"(r.c[v].z),
                     "s"(r.c[v].w));
}

template <typename in_t>
__device__ __forceinline__ void widen16(const uint4 (&w)[UniRaw<in_t>::kVecs], float (&v)[16]) {
    if constexpr (sizeof(in_t) == 2) {
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const uint32_t ww[4] = {w[k].x, w[k].y, w[k].z, w[k].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[8 * k + 2 * i] = to_f32(in_t{(uint16_t)(ww[i] & 0xffffu)});
                v[8 * k + 2 * i + 1] = to_f32(in_t{(uint16_t)(ww[i] >> 16)});
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            v[4 * k] = bits_to_f32(w[k].x); v[4 * k + 1] = bits_to_f32(w[k].y);
            v[4 * k + 2] = bits_to_f32(w[k].z); v[4 * k + 3] = bits_to_f32(w[k].w);
        }
    }
}

// Four consecutive elements of a row as loaded (8 bytes of 16-bit values or 16 bytes of fp32).
template <typename in_t> struct Raw4 { uint32_t w[sizeof(in_t)]; };

template <typename in_t>
__device__ __forceinline__ Raw4<in_t> load_raw4(const in_t *__restrict__ row, int pos, int L, float fill) {
    Raw4<in_t> r;
    if constexpr (sizeof(in_t) == 2) {
        const uint32_t f2 = (uint32_t)from_f32<in_t>(fill).bits * 0x10001u;
        uint2 v = make_uint2(f2, f2);
        if (pos < L) v = *reinterpret_cast<const uint2 *>(row + pos);
        r.w[0] = v.x; r.w[1] = v.y;
    } else {
        const uint32_t f = f32_to_bits(fill);
        uint4 v = make_uint4(f, f, f, f);
        if (pos < L) v = *reinterpret_cast<const uint4 *>(row + pos);
        r.w[0] = v.x; r.w[1] = v.y; r.w[2] = v.z; r.w[3] = v.w;
    }
    return r;
}

template <typename in_t>
__device__ __forceinline__ void unpack_raw4(const Raw4<in_t> &r, float (&v)[4]) {
    if constexpr (sizeof(in_t) == 2) {
        v[0] = to_f32(in_t{(uint16_t)(r.w[0] & 0xffffu)}); v[1] = to_f32(in_t{(uint16_t)(r.w[0] >> 16)});
        v[2] = to_f32(in_t{(uint16_t)(r.w[1] & 0xffffu)}); v[3] = to_f32(in_t{(uint16_t)(r.w[1] >> 16)});
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = bits_to_f32(r.w[i]);
    }
}

template <typename out_t>
__device__ __forceinline__ void store4(out_t *__restrict__ dst, const float (&v)[4]) {
    if constexpr (sizeof(out_t) == 4) {
        *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
        *reinterpret_cast<uint2 *>(dst) = make_uint2(pack2_from_f32<out_t>(v[0], v[1]), pack2_from_f32<out_t>(v[2], v[3]));
    }
}

struct ChanGeom {
    int32_t n_cb;            // channel blocks of 64 per group
    FastDiv div_cb, div_groups;
};

// kX: the chunk-end states are written as well -- x[row][chunk][2n] = product of a_n since the row's start,
// x[..][2n + 1] = h_n, after every 2048 positions and at the row's end.  h is what the lane holds; the product is
// exp2(A_n log2e * sum dl), and the sum is per CHANNEL, not per state: each of the four wavefronts adds up a quarter of
// every round's positions for its lane's channel (one LDS read, four adds per 16 positions) and the quarters meet in LDS
// when a chunk ends.
//
// kMaps: CrossScan folded in.  u is not the (batch, 4 D, L) tensor of the four scan-ordered copies but the map itself,
// x (batch, D, L), plus its transpose xt (batch, D, L: every H x W map stored as W x H): direction k = the channel's
// group reads x (k = 0, 2) or xt (k = 1, 3), forwards (k < 2) or backwards -- position t of the scan is element t or
// L - 1 - t of that row (cross_scan_fwd, classification/models/csm_triton.py:22-29).  A thread's four positions are then
// the four elements that END at L - 1 - t, taken in reverse.
template <typename in_t>
__device__ __forceinline__ Raw4<in_t> reverse4(const Raw4<in_t> &r) {
    Raw4<in_t> o;
    if constexpr (sizeof(in_t) == 2) {
        o.w[0] = __builtin_amdgcn_alignbit(r.w[1], r.w[1], 16);      // halves of a dword exchanged
        o.w[1] = __builtin_amdgcn_alignbit(r.w[0], r.w[0], 16);
    } else {
        o.w[0] = r.w[3]; o.w[1] = r.w[2]; o.w[2] = r.w[1]; o.w[3] = r.w[0];
    }
    return o;
}

template <typename in_t, typename out_t, int kSpw, bool kSoftplus, bool kX, bool kMaps = false>
__global__ __launch_bounds__(kBlock) void scan_chan_kernel(const in_t *__restrict__ u_all, const in_t *__restrict__ dl_all,
                                                           const in_t *__restrict__ B_all, const in_t *__restrict__ C_all,
                                                           const float *__restrict__ A_all, out_t *__restrict__ o_all,
                                                           const ScanArgs p, const ChanGeom geo,
                                                           const in_t *__restrict__ ut_all = nullptr) {
    __shared__ __align__(16) float s_dl[kChanBlock * kChanTilePitch];
    __shared__ __align__(16) float s_du[kChanBlock * kChanTilePitch];
    __shared__ __align__(16) float s_y[kWavesPerWg * kChanBlock * kChanSubPitch];
    __shared__ float s_sum[kX ? kWavesPerWg * kChanBlock : 1];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    // neighbouring workgroups are the channel blocks of one (image, group) and read the same B / C rows: keep them
    // on one XCD (one L2)
    const uint32_t wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
    uint32_t bg, cb, b, grp;
    divmod(wg, geo.div_cb, bg, cb);
    divmod(bg, geo.div_groups, b, grp);
    const int L = p.L, dpg = p.dim_per_group;

    // ---- staging / combine role: row r, quarter q -----------------------------------------------------------------
    const int r = tid >> 2, q = tid & 3;
    const int cs = (int)cb * kChanBlock + r;
    const bool row_ok = cs < dpg;
    const int ds = (int)grp * dpg + min(cs, dpg - 1);
    const int dgs = ds / p.dim_per_delta;
    const in_t *u_row = u_all + (int64_t)b * p.u_bs + (int64_t)ds * p.u_ds;
    bool u_rev = false;                                     // kMaps: uniform over the workgroup (one group = one direction)
    if constexpr (kMaps) {
        const int Dm = p.dim >> 2, k = ds / Dm;
        u_row = ((k & 1) ? ut_all : u_all) + (int64_t)b * p.u_bs + (int64_t)(ds - k * Dm) * p.u_ds;
        u_rev = k >= 2;
    }
    // four positions of u from position pos of the scan on, as they lie in memory: backwards these are the four elements
    // that end at L - 1 - pos, and they are put in scan order where they are widened (in_scan_order) -- not here, which
    // would make the wavefront wait for a load it has just issued for the NEXT step
    auto load_u = [&](int pos) {
        if constexpr (kMaps) {
            if (u_rev) return load_raw4<in_t>(u_row, pos < L ? L - 4 - pos : L, L, 0.0f);
        }
        return load_raw4<in_t>(u_row, pos, L, 0.0f);
    };
    auto in_scan_order = [&](const Raw4<in_t> &r) {
        if constexpr (kMaps) {
            if (u_rev) return reverse4<in_t>(r);
        }
        return r;
    };
    const in_t *dl_row = dl_all + (int64_t)b * p.dl_bs + (int64_t)dgs * p.dl_ds;
    out_t *o_row = o_all + (int64_t)b * p.o_bs + (int64_t)ds * p.o_ds;
    const float bias_s = p.bias ? p.bias[dgs] : 0.0f;
    const float D_s = p.D ? p.D[ds] : 0.0f;
    float *st_dl = s_dl + r * kChanTilePitch + 4 * q;
    float *st_du = s_du + r * kChanTilePitch + 4 * q;

    // ---- compute role: channel = lane, states wave*kSpw .. + kSpw ---------------------------------------------------
    const int dc = (int)grp * dpg + min((int)cb * kChanBlock + lane, dpg - 1);
    float A2[kSpw], h[kSpw];
#pragma unroll
    for (int j = 0; j < kSpw; ++j) {
        A2[j] = A_all[(int64_t)dc * p.A_ds + (int64_t)(wave * kSpw + j) * p.A_ns] * kLog2e;
        h[j] = 0.0f;
    }
    const in_t *B_wave = B_all + (int64_t)b * p.B_bs + (int64_t)grp * p.B_gs + (int64_t)(wave * kSpw) * p.B_ns;
    const in_t *C_wave = C_all + (int64_t)b * p.C_bs + (int64_t)grp * p.C_gs + (int64_t)(wave * kSpw) * p.C_ns;
    const float *my_dl = s_dl + lane * kChanTilePitch, *my_du = s_du + lane * kChanTilePitch;
    float *my_y = s_y + (wave * kChanBlock + lane) * kChanSubPitch;
    const float *sum_y = s_y + r * kChanSubPitch + 4 * q;
    float dl_sum = 0.0f;                                    // kX: this wavefront's quarter of the channel's sum of dl
    const bool chan_ok = (int)cb * kChanBlock + lane < dpg;
    float *x_lane = kX ? p.x + ((int64_t)b * p.dim + dc) * p.n_chunks * 2 * p.N + 2 * (wave * kSpw) : nullptr;

    constexpr float kFill = delta_fill<kSoftplus>();
    Raw4<in_t> ru[2], rd[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        ru[s] = load_u(s * kChanSub + 4 * q);
        rd[s] = load_raw4<in_t>(dl_row, s * kChanSub + 4 * q, L, kFill);
    }
    // B / C of the (round, state) processed next are always one step ahead in scalar registers: requested before the
    // arithmetic of the current state starts, they have arrived when it ends.  Rows are multiples of 8 positions, so
    // the second half of a round lies entirely inside or entirely outside the row; outside, the first half is read
    // again (du is 0 there, nothing of it is stored), and a round past the row's end reads the row's start.
    UniRaw<in_t> next_bc;
    load_uniform<in_t>(B_wave, C_wave, 0, 8 < L ? 8 : 0, next_bc);

    for (int t0 = 0; t0 < L; t0 += kChanTile) {
        // ---- stage: dl, du into LDS; the skip term stays with this thread for the combine ---------------------------
        float skip[2][4];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            float uv[4], raw[4], dl[4], du[4];
            unpack_raw4<in_t>(in_scan_order(ru[s]), uv);
            unpack_raw4<in_t>(rd[s], raw);
            const bool in_row = t0 + s * kChanSub + 4 * q < L;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if constexpr (kSoftplus) dl[i] = softplus_log2(fmaf(raw[i], kLog2e, bias_s * kLog2e));   // fill -inf: 0
                else dl[i] = in_row ? raw[i] + bias_s : 0.0f;
                du[i] = dl[i] * uv[i];
                skip[s][i] = D_s * uv[i];
            }
            *reinterpret_cast<float4 *>(st_dl + s * kChanSub) = make_float4(dl[0], dl[1], dl[2], dl[3]);
            *reinterpret_cast<float4 *>(st_du + s * kChanSub) = make_float4(du[0], du[1], du[2], du[3]);
        }
        // the next step's inputs travel while this step computes
        if (t0 + kChanTile < L) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                ru[s] = load_u(t0 + kChanTile + s * kChanSub + 4 * q);
                rd[s] = load_raw4<in_t>(dl_row, t0 + kChanTile + s * kChanSub + 4 * q, L, kFill);
            }
        }
        __syncthreads();                                    // dl / du of this step are in place

#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int ps = t0 + s * kChanSub;
            if (ps < L) {                                   // uniform over the workgroup
                // ---- compute: 16 positions, this wavefront's states -------------------------------------------------
                float dl[kChanSub], du[kChanSub], y[kChanSub];
#pragma unroll
                for (int v = 0; v < kChanSub / 4; ++v) {
                    const float4 a4 = *reinterpret_cast<const float4 *>(my_dl + s * kChanSub + 4 * v);
                    const float4 b4 = *reinterpret_cast<const float4 *>(my_du + s * kChanSub + 4 * v);
                    dl[4 * v] = a4.x; dl[4 * v + 1] = a4.y; dl[4 * v + 2] = a4.z; dl[4 * v + 3] = a4.w;
                    du[4 * v] = b4.x; du[4 * v + 1] = b4.y; du[4 * v + 2] = b4.z; du[4 * v + 3] = b4.w;
                }
#pragma unroll
                for (int i = 0; i < kChanSub; ++i) y[i] = 0.0f;
                if constexpr (kX) {
                    const float4 q4 = *reinterpret_cast<const float4 *>(my_dl + s * kChanSub + 4 * wave);
                    dl_sum += (q4.x + q4.y) + (q4.z + q4.w);  // (dl is 0 past the row's end)
                }
                // the LDS reads above have landed before the first scalar request below is made (one wait covers both
                // kinds of traffic, so a request issued earlier would be waited for at once)
                asm volatile("" ::"v"(dl[0]), "v"(dl[4]), "v"(dl[8]), "v"(dl[12]), "v"(du[0]), "v"(du[4]), "v"(du[8]), "v"(du[12]));
#pragma unroll
                for (int j = 0; j < kSpw; ++j) {
                    const UniRaw<in_t> cur_bc = next_bc;
                    arrived<in_t>(cur_bc);
                    {
                        // what comes next: the following state of this round, or the first state of the next round
                        const int jn = j + 1 < kSpw ? j + 1 : 0;
                        int pn = j + 1 < kSpw ? ps : ps + kChanSub;
                        pn = pn < L ? pn : 0;
                        const int pn1 = pn + 8 < L ? pn + 8 : pn;
                        load_uniform<in_t>(B_wave + (int64_t)jn * p.B_ns, C_wave + (int64_t)jn * p.C_ns, pn, pn1, next_bc);
                    }
                    __builtin_amdgcn_sched_barrier(0);      // the requests above are issued before the arithmetic below
                    float Bv[kChanSub], Cv[kChanSub];
                    widen16<in_t>(cur_bc.b, Bv);
                    widen16<in_t>(cur_bc.c, Cv);
                    float a[kChanSub];
#pragma unroll
                    for (int i = 0; i < kChanSub; ++i) a[i] = __builtin_amdgcn_exp2f(dl[i] * A2[j]);
                    float hj = h[j];
#pragma unroll
                    for (int i = 0; i < kChanSub; ++i) {
                        hj = fmaf(a[i], hj, Bv[i] * du[i]);
                        y[i] = fmaf(Cv[i], hj, y[i]);
                    }
                    h[j] = hj;
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int v = 0; v < kChanSub / 4; ++v)
                    *reinterpret_cast<float4 *>(my_y + 4 * v) = make_float4(y[4 * v], y[4 * v + 1], y[4 * v + 2], y[4 * v + 3]);
            }
            __syncthreads();                                // the four partial sums of this round are in place
            if (ps < L) {
                // ---- combine: 4 positions of row r ---------------------------------------------------------------
                float acc[4] = {skip[s][0], skip[s][1], skip[s][2], skip[s][3]};
#pragma unroll
                for (int w = 0; w < kWavesPerWg; ++w) {
                    const float4 part = *reinterpret_cast<const float4 *>(sum_y + w * kChanBlock * kChanSubPitch);
                    acc[0] += part.x; acc[1] += part.y; acc[2] += part.z; acc[3] += part.w;
                }
                if (row_ok && ps + 4 * q < L) store4<out_t>(o_row + ps + 4 * q, acc);
            }
            if (s == 0) __syncthreads();                    // partials read before the next round overwrites them
            // (after the second round the barrier at the top of the next step does this: its staging writes touch
            //  dl / du only, which every wavefront has finished reading by then)
        }
        if constexpr (kX) {
            const int t_end = t0 + kChanTile;
            if (t_end % SS2D_SCAN_CHUNK == 0 || t_end >= L) {   // uniform over the workgroup; at least 64 steps apart
                s_sum[wave * kChanBlock + lane] = dl_sum;
                __syncthreads();
                const float total = (s_sum[lane] + s_sum[kChanBlock + lane]) + (s_sum[2 * kChanBlock + lane] + s_sum[3 * kChanBlock + lane]);
                if (chan_ok) {
                    float *xo = x_lane + (int64_t)((min(t_end, L) - 1) / SS2D_SCAN_CHUNK) * 2 * p.N;
#pragma unroll
                    for (int j = 0; j < kSpw; ++j) {
                        xo[2 * j] = __builtin_amdgcn_exp2f(A2[j] * total);
                        xo[2 * j + 1] = h[j];
                    }
                }
            }
        }
    }
}

bool scan_chan_eligible(const ScanArgs &a) {
    // N/4 states per wavefront; rows in whole 8-position vectors; at least half a wavefront of channels per group
    return (a.N == 4 || a.N == 8 || a.N == 16 || a.N == 32) && a.L % 8 == 0 && a.dim_per_group >= 32;
}

template <typename in_t, typename out_t>
static int launch_chan_typed(const ScanArgs &a, const void *xt, hipStream_t stream) {
    ChanGeom geo;
    geo.n_cb = (a.dim_per_group + kChanBlock - 1) / kChanBlock;
    const int groups = a.dim / a.dim_per_group;
    geo.div_cb = make_fastdiv((uint32_t)geo.n_cb);
    geo.div_groups = make_fastdiv((uint32_t)groups);
    const int64_t n_wg = (int64_t)a.batch * groups * geo.n_cb;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
#define SS2D_LAUNCH_CHAN(SPW, SP, X, M)                                                                                    \
    hipLaunchKernelGGL((scan_chan_kernel<in_t, out_t, SPW, SP, X, M>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream,       \
                       (const in_t *)a.u, (const in_t *)a.delta, (const in_t *)a.B, (const in_t *)a.C, a.A, (out_t *)a.out, a, geo, \
                       (const in_t *)xt)
#define SS2D_LAUNCH_CHAN_N(SP, X, M)                            \
    switch (a.N) {                                              \
        case 4: SS2D_LAUNCH_CHAN(1, SP, X, M); break;           \
        case 8: SS2D_LAUNCH_CHAN(2, SP, X, M); break;           \
        case 16: SS2D_LAUNCH_CHAN(4, SP, X, M); break;          \
        default: SS2D_LAUNCH_CHAN(8, SP, X, M); break;          \
    }
#define SS2D_LAUNCH_CHAN_X(SP, M) \
    if (a.x) { SS2D_LAUNCH_CHAN_N(SP, true, M) } else { SS2D_LAUNCH_CHAN_N(SP, false, M) }
    if (xt) {
        if (a.softplus) { SS2D_LAUNCH_CHAN_X(true, true) } else { SS2D_LAUNCH_CHAN_X(false, true) }
    } else {
        if (a.softplus) { SS2D_LAUNCH_CHAN_X(true, false) } else { SS2D_LAUNCH_CHAN_X(false, false) }
    }
#undef SS2D_LAUNCH_CHAN_X
#undef SS2D_LAUNCH_CHAN_N
#undef SS2D_LAUNCH_CHAN
    return launch_status();
}

int launch_scan_chan(const ScanArgs &a, int in_dtype, int out_dtype, hipStream_t stream, const void *xt) {
    if (in_dtype == SS2D_F32) return launch_chan_typed<float, float>(a, xt, stream);
    if (in_dtype == SS2D_BF16) {
        return out_dtype == SS2D_F32 ? launch_chan_typed<bf16_t, float>(a, xt, stream) : launch_chan_typed<bf16_t, bf16_t>(a, xt, stream);
    }
    return out_dtype == SS2D_F32 ? launch_chan_typed<f16_t, float>(a, xt, stream) : launch_chan_typed<f16_t, f16_t>(a, xt, stream);
}

}  // namespace ss2d
