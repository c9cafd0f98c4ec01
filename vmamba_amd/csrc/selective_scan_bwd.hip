// Selective-scan backward for gfx950: the adjoint of selective_scan.hip's recurrence, one wavefront per
// (batch, channel) row, 512 positions per pass.
//
//   forward     dl_t = softplus(delta_t + bias);  a_t = exp(dl_t A_n);  h_t = a_t h_t-1 + dl_t B_t u_t;
//               y_t = sum_n C_n,t h_n,t + D u_t
//   backward    g_t = C_t dy_t + a_t+1 g_t+1                      (adjoint state, a reverse-time scan)
//               d dl_t = sum_n g_t (h_t-1 a_t A_n + B_t u_t)       d delta_t = d dl_t * sigmoid(delta_t + bias)
//               du_t   = dy_t D + sum_n g_t dl_t B_t               dB_n,t += g_t dl_t u_t     dC_n,t += dy_t h_t
//               dA_n  += sum_t g_t h_t-1 a_t dl_t                  dD += sum_t dy_t u_t       dbias += sum_t d delta_t
//
// A row is swept twice.  The first sweep runs the forward recurrence and keeps only the state entering every pass
// (one float per pass and state, in LDS).  The second sweep walks the passes backwards: it recomputes a, b and h
// inside the pass from that entering state (so no state per position is ever stored), runs the reverse scan of
// g with the same wavefront-scan machinery on lane-reversed data, and emits the gradients.  dB and dC are shared
// by all channels of a group and dA / dD / dbias by all batches, so they are accumulated with fp32 hardware
// atomics into zero-initialised buffers; du and d delta are written once per element.
#include <type_traits>

#include "scan_common.h"

namespace ss2d {

struct ScanBwdArgs {
    const void *u, *delta, *B, *C, *dout;
    const float *A, *D, *bias;
    void *du, *ddelta;
    float *dA, *dB, *dC, *dD, *dbias;
    int32_t batch, dim, L, N, dim_per_group, dim_per_delta, softplus, vec_ok, rows, n_pass;
    int64_t u_bs, u_ds, dl_bs, dl_ds, A_ds, A_ns, B_bs, B_gs, B_ns, C_bs, C_gs, C_ns, do_bs, do_ds;
    int64_t g_bs, g_gs, g_ns;      // strides of dB / dC (contiguous (batch, groups, N, L))
};

__device__ __forceinline__ float lane_reverse(float v, int lane) { return __shfl(v, kWave - 1 - lane, kWave); }

// One (batch, channel) row by one wavefront.  `h_in` is the wavefront's LDS scratch ((n_pass + 2) * N floats).
// kGroupAcc: dB / dC contributions go into the workgroup's LDS accumulators accB / accC ([N][L], shared by the
// channels of one group that the workgroup walks) instead of straight to memory.
template <typename in_t, typename dy_t, bool kSoftplus, bool kGroupAcc>
__device__ __forceinline__ void scan_bwd_row(const ScanBwdArgs &p, int b, int d, float *h_in, float *accB, float *accC) {
    const int lane = threadIdx.x & (kWave - 1);
    const int N = p.N, L = p.L, P = p.n_pass;
    float *g_carry = h_in + (size_t)P * N, *a_next = g_carry + N;
    const int grp = d / p.dim_per_group, dg = d / p.dim_per_delta;
    const in_t *u_row = reinterpret_cast<const in_t *>(p.u) + b * p.u_bs + d * p.u_ds;
    const in_t *dl_row = reinterpret_cast<const in_t *>(p.delta) + b * p.dl_bs + dg * p.dl_ds;
    const in_t *B_row = reinterpret_cast<const in_t *>(p.B) + b * p.B_bs + grp * p.B_gs;
    const in_t *C_row = reinterpret_cast<const in_t *>(p.C) + b * p.C_bs + grp * p.C_gs;
    const dy_t *dy_row = reinterpret_cast<const dy_t *>(p.dout) + b * p.do_bs + d * p.do_ds;
    in_t *du_row = reinterpret_cast<in_t *>(p.du) + ((size_t)b * p.dim + d) * L;
    in_t *dd_row = reinterpret_cast<in_t *>(p.ddelta) + ((size_t)b * p.dim + d) * L;
    float *dB_row = p.dB + b * p.g_bs + grp * p.g_gs, *dC_row = p.dC + b * p.g_bs + grp * p.g_gs;
    const float *A_row = p.A + d * p.A_ds;
    const float Dv = p.D ? p.D[d] : 0.0f;
    const float bias = p.bias ? p.bias[dg] : 0.0f;
    const bool vec = p.vec_ok != 0;

    auto load8 = [&](const auto *rowp, int pos, float (&v)[kItems], float fill) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(rowp)>>;
        if (vec) load_items<T, true>(rowp, pos, L, v, fill);
        else load_items<T, false>(rowp, pos, L, v, fill);
    };
    // dl (bias + softplus applied) and u of one pass; positions past the end give dl = 0, u = 0
    auto load_dl_u = [&](int pos, float (&dl)[kItems], float (&uv)[kItems], float (&z)[kItems]) {
        float raw[kItems], bias_items[kItems];
        load8(dl_row, pos, raw, delta_fill<kSoftplus>());
        load8(u_row, pos, uv, 0.0f);
#pragma unroll
        for (int i = 0; i < kItems; ++i) { bias_items[i] = bias; z[i] = raw[i] + bias; }
        delta_transform<kSoftplus>(raw, bias_items, dl);
        if constexpr (!kSoftplus) {
#pragma unroll
            for (int i = 0; i < kItems; ++i) dl[i] = pos + i < L ? dl[i] : 0.0f;
        }
    };

    // ---- sweep 1: the state entering every pass ---------------------------------------------------------------------
    for (int n = lane; n < N; n += kWave) { h_in[n] = 0.0f; g_carry[n] = 0.0f; a_next[n] = 1.0f; }
    for (int pass = 0; pass + 1 < P; ++pass) {
        const int pos = pass * kPass + lane * kItems;
        float dl[kItems], uv[kItems], z[kItems];
        load_dl_u(pos, dl, uv, z);
        for (int n = 0; n < N; ++n) {
            float Bv[kItems];
            load8(B_row + n * p.B_ns, pos, Bv, 0.0f);
            const float A_log2e = A_row[n * p.A_ns] * kLog2e;
            float ac = 1.0f, hh = 0.0f;
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                const float a = __builtin_amdgcn_exp2f(dl[i] * A_log2e);
                ac *= a;
                hh = fmaf(a, hh, Bv[i] * (dl[i] * uv[i]));
            }
            float a_ex, h_ex, a_tot, h_tot;
            wave_scan_pairs(ac, hh, a_ex, h_ex, a_tot, h_tot);
            const float carry = h_in[pass * N + n];
            if (lane == 0) h_in[(pass + 1) * N + n] = fmaf(a_tot, carry, h_tot);
        }
    }

    // ---- sweep 2: passes in reverse ------------------------------------------------------------------------------------
    float dD_acc = 0.0f, dbias_acc = 0.0f;
    for (int pass = P - 1; pass >= 0; --pass) {
        const int pos = pass * kPass + lane * kItems;
        float dl[kItems], uv[kItems], z[kItems], dy[kItems];
        load_dl_u(pos, dl, uv, z);
        load8(dy_row, pos, dy, 0.0f);
        float d_dl[kItems], du[kItems];
#pragma unroll
        for (int i = 0; i < kItems; ++i) { d_dl[i] = 0.0f; du[i] = dy[i] * Dv; dD_acc = fmaf(dy[i], uv[i], dD_acc); }

        for (int n = 0; n < N; ++n) {
            float Bv[kItems], Cv[kItems];
            load8(B_row + n * p.B_ns, pos, Bv, 0.0f);
            load8(C_row + n * p.C_ns, pos, Cv, 0.0f);
            const float An = A_row[n * p.A_ns];
            const float A_log2e = An * kLog2e;
            // forward inside the pass: a, and h at every position from the state entering the pass
            float a[kItems], ac[kItems], hh[kItems];
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                a[i] = __builtin_amdgcn_exp2f(dl[i] * A_log2e);
                const float bb = Bv[i] * (dl[i] * uv[i]);
                ac[i] = i == 0 ? a[i] : ac[i - 1] * a[i];
                hh[i] = i == 0 ? bb : fmaf(a[i], hh[i - 1], bb);
            }
            float a_ex, h_ex, a_tot, h_tot;
            wave_scan_pairs(ac[kItems - 1], hh[kItems - 1], a_ex, h_ex, a_tot, h_tot);
            const float s_in = fmaf(a_ex, h_in[pass * N + n], h_ex);       // h just before this lane's first item
            float h[kItems];
#pragma unroll
            for (int i = 0; i < kItems; ++i) h[i] = fmaf(ac[i], s_in, hh[i]);

            // reverse scan: g_t = C_t dy_t + a_t+1 g_t+1.  a_t+1 of a lane's last item is the next lane's first a
            // (for the last lane: the first a of the pass after this one).
            float a_up = dpp_move<kDppWaveShl1>(0.0f, a[0]);
            const float a_after = a_next[n];
            a_up = lane == kWave - 1 ? a_after : a_up;
            float m[kItems], gl[kItems];
#pragma unroll
            for (int i = kItems - 1; i >= 0; --i) {
                const float sh = i == kItems - 1 ? a_up : a[i + 1];
                const float c = Cv[i] * dy[i];
                m[i] = i == kItems - 1 ? sh : sh * m[i + 1];
                gl[i] = i == kItems - 1 ? c : fmaf(sh, gl[i + 1], c);
            }
            // suffix over lanes = prefix over reversed lanes: with G the g just after a lane's last item,
            // g_first(lane) = gl[0] + m[0] * G(lane),  G(lane) = g_first(lane + 1)
            float me, ge, mt, gt;
            wave_scan_pairs(lane_reverse(m[0], lane), lane_reverse(gl[0], lane), me, ge, mt, gt);
            const float gc = g_carry[n];
            const float G = lane_reverse(fmaf(me, gc, ge), lane);
            if (lane == 0) { g_carry[n] = fmaf(mt, gc, gt); a_next[n] = a[0]; }

            float dA_acc = 0.0f;
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                const float g = fmaf(m[i], G, gl[i]);
                const float h_prev = i == 0 ? s_in : h[i - 1];
                const float da_a = g * h_prev * a[i];                       // dL/da_t * a_t
                d_dl[i] = fmaf(da_a, An, fmaf(g, Bv[i] * uv[i], d_dl[i]));
                dA_acc = fmaf(da_a, dl[i], dA_acc);
                du[i] = fmaf(g, dl[i] * Bv[i], du[i]);
                if (pos + i < L) {
                    if constexpr (kGroupAcc) {
                        __hip_atomic_fetch_add(accB + n * L + pos + i, g * dl[i] * uv[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        __hip_atomic_fetch_add(accC + n * L + pos + i, dy[i] * h[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    } else {
                        unsafeAtomicAdd(dB_row + n * p.g_ns + pos + i, g * dl[i] * uv[i]);
                        unsafeAtomicAdd(dC_row + n * p.g_ns + pos + i, dy[i] * h[i]);
                    }
                }
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) dA_acc += __shfl_xor(dA_acc, off, kWave);
            if (lane == 0) unsafeAtomicAdd(p.dA + d * N + n, dA_acc);
        }

        float dd[kItems];
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            if constexpr (kSoftplus) {
                // softplus'(z) = sigmoid(z); beyond the threshold the forward is the identity
                const float sg = z[i] > kSoftplusThreshold ? 1.0f : 1.0f / (1.0f + __expf(-z[i]));
                dd[i] = d_dl[i] * sg;
            } else {
                dd[i] = d_dl[i];
            }
            dd[i] = pos + i < L ? dd[i] : 0.0f;
            dbias_acc += dd[i];
        }
        if (vec) { store_items<in_t, true>(du_row, pos, L, du); store_items<in_t, true>(dd_row, pos, L, dd); }
        else { store_items<in_t, false>(du_row, pos, L, du); store_items<in_t, false>(dd_row, pos, L, dd); }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        dD_acc += __shfl_xor(dD_acc, off, kWave);
        dbias_acc += __shfl_xor(dbias_acc, off, kWave);
    }
    if (lane == 0) {
        if (p.dD) unsafeAtomicAdd(p.dD + d, dD_acc);
        if (p.dbias) unsafeAtomicAdd(p.dbias + d, dbias_acc);
    }
}

// One wavefront per row, 4 rows per workgroup; dB / dC straight to memory with atomics (any N, any L).
template <typename in_t, typename dy_t, bool kSoftplus>
__global__ __launch_bounds__(kBlock) void scan_bwd_kernel(const ScanBwdArgs p) {
    extern __shared__ __align__(16) float bwd_smem[];      // per wavefront: h_in [n_pass][N], g carry [N], a_next [N]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int row = (int)(blockIdx.x * kWavesPerWg) + wave;
    if (row >= p.rows) return;           // whole wavefront leaves; no workgroup barrier in this kernel
    scan_bwd_row<in_t, dy_t, kSoftplus, false>(p, row / p.dim, row % p.dim, bwd_smem + (size_t)wave * (p.n_pass + 2) * p.N,
                                               nullptr, nullptr);
}

// A workgroup walks `chunk` channels of ONE (batch, group): their dB / dC contributions -- the same N x L entries
// for every channel -- are summed in LDS and reach memory once per workgroup (one atomic per entry per `chunk`
// channels instead of one per channel).  Used when the N x L accumulators fit LDS.
template <typename in_t, typename dy_t, bool kSoftplus>
__global__ __launch_bounds__(kBlock) void scan_bwd_group_kernel(const ScanBwdArgs p, int chunk, int chunks_per_group, int n_groups) {
    extern __shared__ __align__(16) float bwd_smem[];      // accB [N][L], accC [N][L], then the per-wavefront scratch
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int NL = p.N * p.L;
    float *accB = bwd_smem, *accC = bwd_smem + NL;
    float *scratch = accC + NL + (size_t)wave * (p.n_pass + 2) * p.N;
    uint32_t wg = blockIdx.x;
    const int ck = (int)(wg % chunks_per_group); wg /= chunks_per_group;
    const int grp = (int)(wg % n_groups);
    const int b = (int)(wg / n_groups);
    for (int i = threadIdx.x; i < 2 * NL; i += kBlock) bwd_smem[i] = 0.0f;
    __syncthreads();
    const int d_end = min((ck + 1) * chunk, p.dim_per_group);
    for (int c = ck * chunk + wave; c < d_end; c += kWavesPerWg)
        scan_bwd_row<in_t, dy_t, kSoftplus, true>(p, b, grp * p.dim_per_group + c, scratch, accB, accC);
    __syncthreads();
    float *dB_row = p.dB + b * p.g_bs + grp * p.g_gs, *dC_row = p.dC + b * p.g_bs + grp * p.g_gs;
    for (int i = threadIdx.x; i < NL; i += kBlock) {
        unsafeAtomicAdd(dB_row + i, accB[i]);
        unsafeAtomicAdd(dC_row + i, accC[i]);
    }
}

// The same for ONE state per channel (the VMamba setting), pass-major: a wavefront walks its channels of the group
// inside every pass, so the B / C items of the pass are loaded once for all of them and the channels' dB / dC
// contributions are summed in registers first -- one LDS atomic per entry per wavefront and pass instead of one per
// channel (LDS float atomics cost about ten plain LDS accesses here).  Per-channel state between passes (the state
// entering each pass, the adjoint carry, the next pass's first a, the row sums) lives in a few floats of LDS per channel.
template <typename in_t, typename dy_t, bool kSoftplus>
__global__ __launch_bounds__(kBlock) void scan_bwd_group1_kernel(const ScanBwdArgs p, int chunk, int chunks_per_group, int n_groups) {
    extern __shared__ __align__(16) float bwd_smem[];      // accB [L], accC [L], then the per-wavefront scratch
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int L = p.L, P = p.n_pass;
    float *accB = bwd_smem, *accC = bwd_smem + L;
    const int nc_max = (chunk + kWavesPerWg - 1) / kWavesPerWg;
    float *h_in = accC + L + (size_t)wave * nc_max * (P + 5);        // [nc_max][P]: state entering each pass
    float *g_carry = h_in + nc_max * P, *a_next = g_carry + nc_max;  // [nc_max] each
    float *dA_s = a_next + nc_max, *dD_s = dA_s + nc_max, *db_s = dD_s + nc_max;
    uint32_t wg = blockIdx.x;
    const int ck = (int)(wg % chunks_per_group); wg /= chunks_per_group;
    const int grp = (int)(wg % n_groups);
    const int b = (int)(wg / n_groups);
    for (int i = threadIdx.x; i < 2 * L; i += kBlock) bwd_smem[i] = 0.0f;
    for (int i = lane; i < nc_max; i += kWave) {
        h_in[i * P] = 0.0f; g_carry[i] = 0.0f; a_next[i] = 1.0f; dA_s[i] = 0.0f; dD_s[i] = 0.0f; db_s[i] = 0.0f;
    }
    __syncthreads();

    const int c_first = ck * chunk + wave, c_end = min((ck + 1) * chunk, p.dim_per_group);
    const int nc = c_first < c_end ? (c_end - c_first + kWavesPerWg - 1) / kWavesPerWg : 0;
    const in_t *B_row = reinterpret_cast<const in_t *>(p.B) + b * p.B_bs + grp * p.B_gs;
    const in_t *C_row = reinterpret_cast<const in_t *>(p.C) + b * p.C_bs + grp * p.C_gs;
    const bool vec = p.vec_ok != 0;
    auto load8 = [&](const auto *rowp, int pos, float (&v)[kItems], float fill) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(rowp)>>;
        if (vec) load_items<T, true>(rowp, pos, L, v, fill);
        else load_items<T, false>(rowp, pos, L, v, fill);
    };
    struct Row {
        const in_t *u, *dl;
        const dy_t *dy;
        in_t *du, *dd;
        float A_log2e, An, Dv, bias;
        int d;
    };
    auto row_of = [&](int i) {
        Row r;
        r.d = grp * p.dim_per_group + c_first + i * kWavesPerWg;
        const int dg = r.d / p.dim_per_delta;
        r.u = reinterpret_cast<const in_t *>(p.u) + b * p.u_bs + r.d * p.u_ds;
        r.dl = reinterpret_cast<const in_t *>(p.delta) + b * p.dl_bs + dg * p.dl_ds;
        r.dy = reinterpret_cast<const dy_t *>(p.dout) + b * p.do_bs + r.d * p.do_ds;
        r.du = reinterpret_cast<in_t *>(p.du) + ((size_t)b * p.dim + r.d) * L;
        r.dd = reinterpret_cast<in_t *>(p.ddelta) + ((size_t)b * p.dim + r.d) * L;
        r.An = p.A[r.d * p.A_ds];
        r.A_log2e = r.An * kLog2e;
        r.Dv = p.D ? p.D[r.d] : 0.0f;
        r.bias = p.bias ? p.bias[dg] : 0.0f;
        return r;
    };
    auto load_dl_u = [&](const Row &r, int pos, float (&dl)[kItems], float (&uv)[kItems], float (&z)[kItems]) {
        float raw[kItems], bias_items[kItems];
        load8(r.dl, pos, raw, delta_fill<kSoftplus>());
        load8(r.u, pos, uv, 0.0f);
#pragma unroll
        for (int i = 0; i < kItems; ++i) { bias_items[i] = r.bias; z[i] = raw[i] + r.bias; }
        delta_transform<kSoftplus>(raw, bias_items, dl);
        if constexpr (!kSoftplus) {
#pragma unroll
            for (int i = 0; i < kItems; ++i) dl[i] = pos + i < L ? dl[i] : 0.0f;
        }
    };

    // ---- sweep 1: the state entering every pass, for every channel of this wavefront -------------------------------
    for (int pass = 0; pass + 1 < P; ++pass) {
        const int pos = pass * kPass + lane * kItems;
        float Bv[kItems];
        load8(B_row, pos, Bv, 0.0f);
        for (int ci = 0; ci < nc; ++ci) {
            const Row r = row_of(ci);
            float dl[kItems], uv[kItems], z[kItems];
            load_dl_u(r, pos, dl, uv, z);
            float ac = 1.0f, hh = 0.0f;
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                const float a = __builtin_amdgcn_exp2f(dl[i] * r.A_log2e);
                ac *= a;
                hh = fmaf(a, hh, Bv[i] * (dl[i] * uv[i]));
            }
            float a_ex, h_ex, a_tot, h_tot;
            wave_scan_pairs(ac, hh, a_ex, h_ex, a_tot, h_tot);
            const float carry = h_in[ci * P + pass];
            if (lane == 0) h_in[ci * P + pass + 1] = fmaf(a_tot, carry, h_tot);
        }
    }

    // ---- sweep 2: passes in reverse, channels inside ------------------------------------------------------------------
    for (int pass = P - 1; pass >= 0; --pass) {
        const int pos = pass * kPass + lane * kItems;
        float Bv[kItems], Cv[kItems], sumB[kItems], sumC[kItems];
        load8(B_row, pos, Bv, 0.0f);
        load8(C_row, pos, Cv, 0.0f);
#pragma unroll
        for (int i = 0; i < kItems; ++i) { sumB[i] = 0.0f; sumC[i] = 0.0f; }
        for (int ci = 0; ci < nc; ++ci) {
            const Row r = row_of(ci);
            float dl[kItems], uv[kItems], z[kItems], dy[kItems];
            load_dl_u(r, pos, dl, uv, z);
            load8(r.dy, pos, dy, 0.0f);
            // forward inside the pass: a, and h at every position from the state entering the pass
            float a[kItems], ac[kItems], hh[kItems];
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                a[i] = __builtin_amdgcn_exp2f(dl[i] * r.A_log2e);
                const float bb = Bv[i] * (dl[i] * uv[i]);
                ac[i] = i == 0 ? a[i] : ac[i - 1] * a[i];
                hh[i] = i == 0 ? bb : fmaf(a[i], hh[i - 1], bb);
            }
            float a_ex, h_ex, a_tot, h_tot;
            wave_scan_pairs(ac[kItems - 1], hh[kItems - 1], a_ex, h_ex, a_tot, h_tot);
            const float s_in = fmaf(a_ex, h_in[ci * P + pass], h_ex);       // h just before this lane's first item
            // reverse scan: g_t = C_t dy_t + a_t+1 g_t+1 (see scan_bwd_row)
            float a_up = dpp_move<kDppWaveShl1>(0.0f, a[0]);
            const float a_after = a_next[ci];
            a_up = lane == kWave - 1 ? a_after : a_up;
            float m[kItems], gl[kItems];
#pragma unroll
            for (int i = kItems - 1; i >= 0; --i) {
                const float sh = i == kItems - 1 ? a_up : a[i + 1];
                const float c = Cv[i] * dy[i];
                m[i] = i == kItems - 1 ? sh : sh * m[i + 1];
                gl[i] = i == kItems - 1 ? c : fmaf(sh, gl[i + 1], c);
            }
            float me, ge, mt, gt;
            wave_scan_pairs(lane_reverse(m[0], lane), lane_reverse(gl[0], lane), me, ge, mt, gt);
            const float gc = g_carry[ci];
            const float G = lane_reverse(fmaf(me, gc, ge), lane);
            if (lane == 0) { g_carry[ci] = fmaf(mt, gc, gt); a_next[ci] = a[0]; }

            float dA_acc = 0.0f, dD_acc = 0.0f, db_acc = 0.0f, du[kItems], dd[kItems];
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                const float g = fmaf(m[i], G, gl[i]);
                const float h = fmaf(ac[i], s_in, hh[i]);
                const float h_prev = i == 0 ? s_in : fmaf(ac[i - 1], s_in, hh[i - 1]);
                const float da_a = g * h_prev * a[i];                       // dL/da_t * a_t
                const float d_dl = fmaf(da_a, r.An, g * (Bv[i] * uv[i]));
                dA_acc = fmaf(da_a, dl[i], dA_acc);
                dD_acc = fmaf(dy[i], uv[i], dD_acc);
                du[i] = fmaf(g, dl[i] * Bv[i], dy[i] * r.Dv);
                sumB[i] = fmaf(g, dl[i] * uv[i], sumB[i]);
                sumC[i] = fmaf(dy[i], h, sumC[i]);
                if constexpr (kSoftplus) {
                    const float sg = z[i] > kSoftplusThreshold ? 1.0f : 1.0f / (1.0f + __expf(-z[i]));
                    dd[i] = d_dl * sg;
                } else {
                    dd[i] = d_dl;
                }
                dd[i] = pos + i < L ? dd[i] : 0.0f;
                db_acc += dd[i];
            }
            if (vec) { store_items<in_t, true>(r.du, pos, L, du); store_items<in_t, true>(r.dd, pos, L, dd); }
            else { store_items<in_t, false>(r.du, pos, L, du); store_items<in_t, false>(r.dd, pos, L, dd); }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                dA_acc += __shfl_xor(dA_acc, off, kWave);
                dD_acc += __shfl_xor(dD_acc, off, kWave);
                db_acc += __shfl_xor(db_acc, off, kWave);
            }
            if (lane == 0) { dA_s[ci] += dA_acc; dD_s[ci] += dD_acc; db_s[ci] += db_acc; }
        }
#pragma unroll
        for (int i = 0; i < kItems; ++i)
            if (pos + i < L && nc > 0) {
                __hip_atomic_fetch_add(accB + pos + i, sumB[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(accC + pos + i, sumC[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
    }
    for (int ci = lane; ci < nc; ci += kWave) {
        const int d = grp * p.dim_per_group + c_first + ci * kWavesPerWg;
        unsafeAtomicAdd(p.dA + d, dA_s[ci]);
        if (p.dD) unsafeAtomicAdd(p.dD + d, dD_s[ci]);
        if (p.dbias) unsafeAtomicAdd(p.dbias + d, db_s[ci]);
    }
    __syncthreads();
    float *dB_row = p.dB + b * p.g_bs + grp * p.g_gs, *dC_row = p.dC + b * p.g_bs + grp * p.g_gs;
    for (int i = threadIdx.x; i < L; i += kBlock) {
        unsafeAtomicAdd(dB_row + i, accB[i]);
        unsafeAtomicAdd(dC_row + i, accC[i]);
    }
}

}  // namespace ss2d

extern "C" int ss2d_selective_scan_bwd(const ss2d_scan_bwd_params *q, void *stream) {
    using namespace ss2d;
    if (!q) return SS2D_EINVAL;
    if (q->batch < 0 || q->dim < 0 || q->seqlen < 0) return SS2D_EINVAL;
    if (q->dstate <= 0 || q->dstate > 256 || q->n_groups <= 0 || q->delta_dim <= 0) return SS2D_EINVAL;
    if (q->in_dtype != SS2D_F32 && q->in_dtype != SS2D_BF16 && q->in_dtype != SS2D_F16) return SS2D_EINVAL;
    if (q->dout_dtype != SS2D_F32 && q->dout_dtype != q->in_dtype) return SS2D_EINVAL;
    if (q->dim % q->n_groups != 0 || q->dim % q->delta_dim != 0) return SS2D_EINVAL;
    if (q->batch == 0 || q->dim == 0 || q->seqlen == 0) return SS2D_OK;
    if (!q->u || !q->delta || !q->A || !q->B || !q->C || !q->dout || !q->du || !q->ddelta || !q->dA || !q->dB || !q->dC)
        return SS2D_EINVAL;
    if ((q->D == nullptr) != (q->dD == nullptr)) return SS2D_EINVAL;
    if ((q->delta_bias == nullptr) != (q->ddelta_bias == nullptr)) return SS2D_EINVAL;
    if ((int64_t)q->batch * q->dim > 0x7fffffff - kWavesPerWg) return SS2D_ENOTSUP;

    ScanBwdArgs a;
    a.u = q->u; a.delta = q->delta; a.B = q->B; a.C = q->C; a.dout = q->dout;
    a.A = (const float *)q->A; a.D = (const float *)q->D; a.bias = (const float *)q->delta_bias;
    a.du = q->du; a.ddelta = q->ddelta;
    a.dA = (float *)q->dA; a.dB = (float *)q->dB; a.dC = (float *)q->dC; a.dD = (float *)q->dD; a.dbias = (float *)q->ddelta_bias;
    a.batch = q->batch; a.dim = q->dim; a.L = q->seqlen; a.N = q->dstate;
    a.dim_per_group = q->dim / q->n_groups;
    a.dim_per_delta = q->dim / q->delta_dim;
    a.softplus = q->delta_softplus;
    a.rows = q->batch * q->dim;
    a.n_pass = (q->seqlen + kPass - 1) / kPass;
    a.u_bs = q->u_batch_stride; a.u_ds = q->u_d_stride;
    a.dl_bs = q->delta_batch_stride; a.dl_ds = q->delta_d_stride;
    a.A_ds = q->A_d_stride; a.A_ns = q->A_dstate_stride;
    a.B_bs = q->B_batch_stride; a.B_gs = q->B_group_stride; a.B_ns = q->B_dstate_stride;
    a.C_bs = q->C_batch_stride; a.C_gs = q->C_group_stride; a.C_ns = q->C_dstate_stride;
    a.do_bs = q->dout_batch_stride; a.do_ds = q->dout_d_stride;
    a.g_ns = q->seqlen; a.g_gs = (int64_t)q->dstate * q->seqlen; a.g_bs = (int64_t)q->n_groups * a.g_gs;
    const size_t smem = (size_t)kWavesPerWg * (a.n_pass + 2) * a.N * sizeof(float);
    if (smem > 48 * 1024) return SS2D_ENOTSUP;        // very long rows x many states: the per-pass states do not fit LDS

    auto al16 = [](const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; };
    const int64_t in_vec = q->in_dtype == SS2D_F32 ? 4 : 8, dy_vec = q->dout_dtype == SS2D_F32 ? 4 : 8;
    bool vec = al16(q->u) && al16(q->delta) && al16(q->B) && al16(q->C) && al16(q->dout) && al16(q->du) && al16(q->ddelta);
    vec = vec && q->seqlen % in_vec == 0 && q->seqlen % dy_vec == 0;
    const int64_t in_strides[] = {a.u_bs, a.u_ds, a.dl_bs, a.dl_ds, a.B_bs, a.B_gs, a.B_ns, a.C_bs, a.C_gs, a.C_ns};
    for (int64_t s : in_strides) vec = vec && (s % in_vec == 0);
    vec = vec && a.do_bs % dy_vec == 0 && a.do_ds % dy_vec == 0;
    a.vec_ok = vec ? 1 : 0;

    hipStream_t s = (hipStream_t)stream;
    // group kernel: N x L accumulators for dB and dC in LDS
    const size_t acc_bytes = 2 * (size_t)a.N * a.L * sizeof(float);
    if (acc_bytes + smem <= 56 * 1024 && a.dim_per_group >= 2 * kWavesPerWg) {
        int chunk = a.dim_per_group < 24 ? a.dim_per_group : 24;            // channels per workgroup
        const int cpg = (a.dim_per_group + chunk - 1) / chunk;
        chunk = (a.dim_per_group + cpg - 1) / cpg;                           // even split
        const int64_t n = (int64_t)q->batch * q->n_groups * cpg;
        if (n <= 0x7fffffff) {
            const uint32_t n_wg_g = (uint32_t)n;
            const size_t smem_g = acc_bytes + smem;
            if (a.N == 1) {
                // one state: the pass-major kernel (channels inside the pass, dB / dC summed in registers first)
                const int nc_max = (chunk + kWavesPerWg - 1) / kWavesPerWg;
                const size_t smem_1 = acc_bytes + (size_t)kWavesPerWg * nc_max * (a.n_pass + 5) * sizeof(float);
#define SS2D_BWD_GROUP1(IN, DY)                                                                                                 \
    do {                                                                                                                        \
        if (a.softplus) hipLaunchKernelGGL((scan_bwd_group1_kernel<IN, DY, true>), dim3(n_wg_g), dim3(kBlock), smem_1, s, a, chunk, cpg, q->n_groups); \
        else hipLaunchKernelGGL((scan_bwd_group1_kernel<IN, DY, false>), dim3(n_wg_g), dim3(kBlock), smem_1, s, a, chunk, cpg, q->n_groups);          \
    } while (0)
                if (q->in_dtype == SS2D_F32) SS2D_BWD_GROUP1(float, float);
                else if (q->in_dtype == SS2D_BF16) { if (q->dout_dtype == SS2D_F32) SS2D_BWD_GROUP1(bf16_t, float); else SS2D_BWD_GROUP1(bf16_t, bf16_t); }
                else { if (q->dout_dtype == SS2D_F32) SS2D_BWD_GROUP1(f16_t, float); else SS2D_BWD_GROUP1(f16_t, f16_t); }
#undef SS2D_BWD_GROUP1
                return launch_status();
            }
#define SS2D_BWD_GROUP(IN, DY)                                                                                                  \
    do {                                                                                                                        \
        if (a.softplus) hipLaunchKernelGGL((scan_bwd_group_kernel<IN, DY, true>), dim3(n_wg_g), dim3(kBlock), smem_g, s, a, chunk, cpg, q->n_groups); \
        else hipLaunchKernelGGL((scan_bwd_group_kernel<IN, DY, false>), dim3(n_wg_g), dim3(kBlock), smem_g, s, a, chunk, cpg, q->n_groups);          \
    } while (0)
            if (q->in_dtype == SS2D_F32) SS2D_BWD_GROUP(float, float);
            else if (q->in_dtype == SS2D_BF16) { if (q->dout_dtype == SS2D_F32) SS2D_BWD_GROUP(bf16_t, float); else SS2D_BWD_GROUP(bf16_t, bf16_t); }
            else { if (q->dout_dtype == SS2D_F32) SS2D_BWD_GROUP(f16_t, float); else SS2D_BWD_GROUP(f16_t, f16_t); }
#undef SS2D_BWD_GROUP
            return launch_status();
        }
    }
    const uint32_t n_wg = (uint32_t)((a.rows + kWavesPerWg - 1) / kWavesPerWg);
#define SS2D_BWD_LAUNCH(IN, DY)                                                                                         \
    do {                                                                                                                \
        if (a.softplus) hipLaunchKernelGGL((scan_bwd_kernel<IN, DY, true>), dim3(n_wg), dim3(kBlock), smem, s, a);      \
        else hipLaunchKernelGGL((scan_bwd_kernel<IN, DY, false>), dim3(n_wg), dim3(kBlock), smem, s, a);                \
    } while (0)
    if (q->in_dtype == SS2D_F32) SS2D_BWD_LAUNCH(float, float);
    else if (q->in_dtype == SS2D_BF16) { if (q->dout_dtype == SS2D_F32) SS2D_BWD_LAUNCH(bf16_t, float); else SS2D_BWD_LAUNCH(bf16_t, bf16_t); }
    else { if (q->dout_dtype == SS2D_F32) SS2D_BWD_LAUNCH(f16_t, float); else SS2D_BWD_LAUNCH(f16_t, f16_t); }
#undef SS2D_BWD_LAUNCH
    return launch_status();
}
