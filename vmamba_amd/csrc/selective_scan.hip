// Selective-scan forward for gfx950: a chunked linear-recurrence scan written for 64-lane
// wavefronts.
//
//   dl_t  = softplus(delta_t + bias)                     (fused into the load)
//   h_n,t = exp(dl_t A_n) h_n,t-1 + dl_t B_n,t u_t       (fp32 state)
//   y_t   = sum_n C_n,t h_n,t + D u_t
//
// The recurrence is the scan of pairs (a,b) under (a1,b1) o (a0,b0) = (a1 a0, a1 b0 + b1).
// A wavefront covers 512 consecutive positions per pass: every lane scans its 8 consecutive
// items in registers, the 64 lane totals are scanned with DPP row shifts / row broadcasts (no
// LDS, no barrier), and the running state is carried from pass to pass in a register.
//
//   row kernel   one wavefront per (batch, channel) row, 4 rows per workgroup.
//   row4 kernel  long rows with few of them: the 4 wavefronts of a workgroup split each
//                2048-position chunk of one row and exchange their totals through LDS.
//
// I/O is 16-byte vectors per lane whenever pointers, strides and the row length allow
// (kVec); otherwise element-wise with bounds checks.  Positions past the end of a row are fed
// as dl = 0, u = 0, i.e. the identity pair (1, 0), so the state at the end of the last pass is
// the state at the last real position.
#include "scan_common.h"

namespace ss2d {

constexpr int kScanTailMax = 2;     // the short-tail row kernel takes up to this many 64-position tail passes

// ---- one wavefront per row ------------------------------------------------------------
// kN == 1: the single state lives in registers and inputs are fetched in bursts.
// kN == 0: any dstate; the per-wave states (running product, h) live in LDS, 2*dstate floats per wave: they
//          are wave-uniform, and keeping 3*dstate of them in vector registers (tried for dstate 16) spills.
template <typename in_t, typename out_t, int kN, bool kVec, bool kSoftplus, bool kShortTail = false>
__global__ __launch_bounds__(kBlock) void scan_row_kernel(const ScanArgs p) {
    static_assert(!kShortTail || (kN == 1 && kVec), "the short tail belongs to the one-state vector kernel");
    extern __shared__ __align__(16) float dyn_state[];   // kN == 0 only: [wave][N][2]
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // With several states the B/C rows (shared by dim/n_groups channels) are worth keeping in one XCD's L2, so
    // each XCD gets a contiguous range of rows.  With one state they are 1 % of the traffic and the hardware's
    // round-robin order, which keeps all active rows in one moving window of memory, measured faster.
    const uint32_t wg = kN == 1 ? blockIdx.x : xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int row = (int)(wg * kWavesPerWg) + wave;
    if (row >= p.rows) return;           // whole wavefront leaves; this kernel has no barrier

    const int N = kN > 0 ? kN : p.N;
    const int b = row / p.dim, d = row - b * p.dim;
    const int grp = d / p.dim_per_group, dg = d / p.dim_per_delta;
    const in_t *u_row = reinterpret_cast<const in_t *>(p.u) + b * p.u_bs + d * p.u_ds;
    const in_t *dl_row = reinterpret_cast<const in_t *>(p.delta) + b * p.dl_bs + dg * p.dl_ds;
    const in_t *B_row = reinterpret_cast<const in_t *>(p.B) + b * p.B_bs + grp * p.B_gs;
    const in_t *C_row = reinterpret_cast<const in_t *>(p.C) + b * p.C_bs + grp * p.C_gs;
    out_t *o_row = reinterpret_cast<out_t *>(p.out) + b * p.o_bs + d * p.o_ds;
    const float *A_row = p.A + d * p.A_ds;
    float *x_row = p.x ? p.x + (size_t)row * p.n_chunks * 2 * N : nullptr;
    const float Dv = p.D ? p.D[d] : 0.0f;
    const float bias = p.bias ? p.bias[dg] : 0.0f;
    const int L = p.L;
    // multi-state vector path: B / C through buffer descriptors (the host checked the extents fit 31 bits)
    const __amdgpu_buffer_rsrc_t B_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.B), 0, (int)p.B_span_bytes, kBufferRsrcWord3);
    const __amdgpu_buffer_rsrc_t C_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.C), 0, (int)p.C_span_bytes, kBufferRsrcWord3);
    const uint32_t B_soff = (uint32_t)(b * p.B_bs + grp * p.B_gs), C_soff = (uint32_t)(b * p.C_bs + grp * p.C_gs);
    const bool use_buffers = kVec && p.B_span_bytes != 0;

    float h_reg[kN > 0 ? kN : 1], ap_reg[kN > 0 ? kN : 1], A_reg[kN > 0 ? kN : 1];
    float *st = dyn_state + (size_t)wave * 2 * N;
    if constexpr (kN > 0) {
#pragma unroll
        for (int n = 0; n < kN; ++n) { h_reg[n] = 0.0f; ap_reg[n] = 1.0f; A_reg[n] = A_row[n * p.A_ns] * kLog2e; }
    } else {
        for (int n = lane; n < N; n += kWave) { st[2 * n] = 1.0f; st[2 * n + 1] = 0.0f; }
    }

    // u and delta are read once: streaming loads (B and C, shared by the channels of a group, stay ordinary ones).  With
    // the streaming stores of the outputs: stage-1 scan 236 -> 222 us, CrossScan + scan + CrossMerge 466 -> 415.
    // Burst loads: with a single state the inputs of kBurst consecutive passes (u, delta, B, C: 4 x 1 KB each per
    // wavefront and pass) are requested together before any of them is processed.  A row is then fetched in two
    // or three long runs instead of seven short visits, which the memory system serves measurably faster, and
    // each wavefront keeps several KB in flight.
    constexpr bool kBurstBC = kN == 1;
    constexpr int kBurst = kN == 1 ? 4 : 1;
    // kShortTail (chosen by the host when a row ends with at most kScanTailMax * 64 positions past its last full pass;
    // 56 x 56 maps: 6 passes + 64): those positions are walked one per lane -- about a fifth of the cost of a full
    // pass each -- instead of as an eighth-full pass of 8 per lane.  It is an instantiation of its own because the
    // extra code costs the register that lets five wavefronts share a SIMD, which the other row lengths keep.
    const int tail = L % kPass;
    const bool short_tail = kShortTail;
    const int n_pass = short_tail ? L / kPass : (L + kPass - 1) / kPass;
    const int L_body = short_tail ? n_pass * kPass : L;              // what the 8-per-lane passes cover
    constexpr bool kTiledStore = kVec && sizeof(out_t) == 4;     // fp32 out as whole 1 KB runs (store_pass_f32)
    __shared__ __align__(16) float y_tile[kTiledStore ? kWavesPerWg : 1][kTiledStore ? kPass : 4];
    const __amdgpu_buffer_rsrc_t o_buf = row_buffer(o_row, kTiledStore ? L_body : 0);
    for (int pass0 = 0; pass0 < n_pass; pass0 += kBurst) {
        Raw8<in_t> u_burst[kBurst], dl_burst[kBurst], B_burst[kBurst], C_burst[kBurst];
#pragma unroll
        for (int s = 0; s < kBurst; ++s) {
            const int pos_s = (pass0 + s) * kPass + lane * kItems;
            u_burst[s] = load_raw<in_t, kVec, true>(u_row, pos_s, L_body);
            dl_burst[s] = load_raw<in_t, kVec, true>(dl_row, pos_s, L_body, delta_fill<kSoftplus>());
            if constexpr (kBurstBC) {
                B_burst[s] = load_raw<in_t, kVec>(B_row, pos_s, L_body);
                C_burst[s] = load_raw<in_t, kVec>(C_row, pos_s, L_body);
            }
        }
#pragma unroll
        for (int s = 0; s < kBurst; ++s) {
        const int pass = pass0 + s;
        if (pass >= n_pass) break;
        const int pos = pass * kPass + lane * kItems;
        const Raw8<in_t> u_raw = u_burst[s], dl_raw = dl_burst[s];
        Raw8<in_t> B_raw, C_raw;
        if constexpr (kBurstBC) { B_raw = B_burst[s]; C_raw = C_burst[s]; }
        float dl[kItems], du[kItems], y[kItems];
        prepare_delta_u<in_t, kSoftplus>(u_raw, dl_raw, L_body - pos, bias, Dv, dl, du, y);
        const bool chunk_end = x_row && ((pass + 1) % kPassesPerChunk == 0 || (pass == n_pass - 1 && !short_tail));
        float *x_out = chunk_end ? x_row + (size_t)(pass / kPassesPerChunk) * 2 * N : nullptr;

        if constexpr (kN > 0) {
#pragma unroll
            for (int n = 0; n < kN; ++n) {
                float Bv[kItems], Cv[kItems], a_tot, h_tot;
                if constexpr (kBurstBC) {
                    unpack_raw<in_t>(B_raw, Bv);
                    unpack_raw<in_t>(C_raw, Cv);
                } else {
                    load_items<in_t, kVec>(B_row + n * p.B_ns, pos, L, Bv);
                    load_items<in_t, kVec>(C_row + n * p.C_ns, pos, L, Cv);
                }
                scan_state_pass(dl, du, Bv, Cv, A_reg[n], h_reg[n], y, a_tot, h_tot);
                h_reg[n] = fmaf(a_tot, h_reg[n], h_tot);
                ap_reg[n] *= a_tot;
                if (chunk_end && lane == 0) { x_out[2 * n] = ap_reg[n]; x_out[2 * n + 1] = h_reg[n]; }
            }
        } else {
            for (int n = 0; n < N; ++n) {
                float Bv[kItems], Cv[kItems], a_tot, h_tot;
                if (use_buffers) {
                    // the row / state part of the address is a wave-uniform scalar offset, the lane part (the position)
                    // one 32-bit register shared by all 2N loads of the pass; unconditional (a lane past the end
                    // re-reads the row's last vector; its du is 0, so the values are never used)
                    // (each 16-byte half is clamped on its own: rows of fp32 may end on a multiple of 4)
                    constexpr int kHalf = 16 / (int)sizeof(in_t) >= kItems ? kItems : 16 / (int)sizeof(in_t);
#pragma unroll
                    for (int hv = 0; hv < kItems / kHalf; ++hv) {
                        const int pos_ld = min(pos + hv * kHalf, L - kHalf);
                        float bh[kHalf], ch[kHalf];
                        gather_group<in_t, kHalf>(B_rsrc, (uint32_t)pos_ld, B_soff + (uint32_t)n * (uint32_t)p.B_ns, bh);
                        gather_group<in_t, kHalf>(C_rsrc, (uint32_t)pos_ld, C_soff + (uint32_t)n * (uint32_t)p.C_ns, ch);
#pragma unroll
                        for (int i = 0; i < kHalf; ++i) { Bv[hv * kHalf + i] = bh[i]; Cv[hv * kHalf + i] = ch[i]; }
                    }
                } else {
                    load_items<in_t, kVec>(B_row + n * p.B_ns, pos, L, Bv);
                    load_items<in_t, kVec>(C_row + n * p.C_ns, pos, L, Cv);
                }
                const float ap = st[2 * n], h0 = st[2 * n + 1];
                scan_state_pass(dl, du, Bv, Cv, A_row[n * p.A_ns] * kLog2e, h0, y, a_tot, h_tot);
                const float h1 = fmaf(a_tot, h0, h_tot), ap1 = ap * a_tot;
                if (lane == 0) {
                    st[2 * n] = ap1; st[2 * n + 1] = h1;
                    if (chunk_end) { x_out[2 * n] = ap1; x_out[2 * n + 1] = h1; }
                }
            }
        }
        if constexpr (kVec && sizeof(out_t) == 4) store_pass_f32(y_tile[wave], o_buf, pass * kPass, lane, y);
        else store_items<out_t, kVec>(o_row, pos, L_body, y);
        }
    }
    if constexpr (kShortTail) {
        if (short_tail) {
#pragma unroll
            for (int t = 0; t < kScanTailMax; ++t) {
                if (t * kWave >= tail) break;
                const int tp = L_body + t * kWave + lane;
                const bool ok = tp < L;
                const int tq = ok ? tp : L - 1;
                const float tu = ok ? to_f32(u_row[tq]) : 0.0f;                  // u = 0 and dl = 0: the identity pair
                const float tdl = ok ? to_f32(dl_row[tq]) : delta_fill<kSoftplus>();
                const float tB = to_f32(B_row[tq]), tC = to_f32(C_row[tq]);
                float dl;
                if constexpr (kSoftplus) dl = softplus_log2(fmaf(tdl, kLog2e, bias * kLog2e));
                else dl = ok ? tdl + bias : 0.0f;
                const float a = __builtin_amdgcn_exp2f(dl * A_reg[0]);
                const float bb = tB * (dl * tu);
                float a_ex, h_ex, a_tot, h_tot;
                wave_scan_pairs(a, bb, a_ex, h_ex, a_tot, h_tot);
                const float hv = fmaf(a, fmaf(a_ex, h_reg[0], h_ex), bb);
                if (ok) o_row[tp] = from_f32<out_t>(fmaf(tC, hv, Dv * tu));
                h_reg[0] = fmaf(a_tot, h_reg[0], h_tot);
                ap_reg[0] *= a_tot;
            }
            // the tail belongs to the chunk of pass n_pass: it ends that chunk (and the row)
            if (x_row && lane == 0) {
                float *x_out = x_row + (size_t)(n_pass / kPassesPerChunk) * 2 * N;
                x_out[0] = ap_reg[0]; x_out[1] = h_reg[0];
            }
        }
    }
}

// ---- many short rows per wavefront ------------------------------------------------------------
// Rows shorter than a pass would leave most lanes idle in the row kernel.  Here a wavefront
// walks a contiguous run of `rows_per_wave` rows as ONE stream of positions (u, delta and out
// are dense, so consecutive rows are adjacent in memory and the 16-byte lane vectors stay
// aligned because rows_per_wave is a multiple of 8).  The recurrence restarts at every row
// simply by forcing a = 0 at a row's first position: the pair (0, b) discards whatever state
// arrives from the previous row.
//
// kGran = gcd(L, 8) (further reduced by what the B/C strides and alignment allow) is the
// granularity at which rows can change inside a lane's 8 items: the items form 8/kGran groups
// that each lie in one row, so the per-row constants (A, D, bias, the B/C row) are selected per
// group, not per item, and B/C are gathered kGran elements at a time through buffer
// descriptors (their rows are shared by dim/n_groups channels and stay in L1/L2).  A lane
// touches at most two rows (L >= 8); with kGran == 8 exactly one.
//
// kX: the chunk-end states are written too.  h at a chunk's (or row's) last position is what the scan yields there.  The
// product of a since the row's start is a second recurrence on the SAME multipliers: with a forced to 0 at a row's
// first position, g_t = a_t g_(t-1) + c_t with c = the true a at that first position and 0 elsewhere gives
// g_t = a_start ... a_t, so it rides through the lane-local and the wavefront scan beside h (wave_scan_pairs2).  Chunk
// and row ends fall on group boundaries (rows start at multiples of kGran in the stream, chunks at multiples of 8).
template <typename in_t, typename out_t, int kN, bool kSoftplus, int kGran, bool kX>
__global__ __launch_bounds__(kBlock) void scan_flat_kernel(const ScanArgs p, int rows_per_wave, FastDiv divL,
                                                           FastDiv divDim, FastDiv divDpg) {
    constexpr int kGroups = kItems / kGran;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int64_t r0 = ((int64_t)wg * kWavesPerWg + wave) * rows_per_wave;
    if (r0 >= p.rows) return;
    const int L = p.L;
    const int n_rows = (int)min((int64_t)rows_per_wave, (int64_t)p.rows - r0);
    const int n_el = n_rows * L;
    const in_t *u_base = reinterpret_cast<const in_t *>(p.u) + r0 * L;
    const in_t *dl_base = reinterpret_cast<const in_t *>(p.delta) + r0 * L;
    // 32-bit byte offsets per lane, no 64-bit address math, hardware range checking (past the extent reads 0)
    const __amdgpu_buffer_rsrc_t B_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.B), 0, (int)p.B_span_bytes, kBufferRsrcWord3);
    const __amdgpu_buffer_rsrc_t C_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.C), 0, (int)p.C_span_bytes, kBufferRsrcWord3);
    out_t *o_base = reinterpret_cast<out_t *>(p.out) + r0 * L;
    // fp32 out leaves as whole 1 KB runs (store_pass_f32); the descriptor drops what lies past the run's last element
    __shared__ __align__(16) float y_tile[sizeof(out_t) == 4 ? kWavesPerWg : 1][sizeof(out_t) == 4 ? kPass : 4];
    const __amdgpu_buffer_rsrc_t o_buf = row_buffer(o_base, sizeof(out_t) == 4 ? n_el : 0);

    float h_reg[kN], g_reg[kX ? kN : 1];
#pragma unroll
    for (int n = 0; n < kN; ++n) h_reg[n] = 0.0f;
#pragma unroll
    for (int n = 0; n < (kX ? kN : 1); ++n) g_reg[n] = 0.0f;

    const int n_pass = (n_el + kPass - 1) / kPass;
    for (int pass = 0; pass < n_pass; ++pass) {
        const int e0 = pass * kPass + lane * kItems;
        const bool full = e0 + kItems <= n_el;
        constexpr float kFill = delta_fill<kSoftplus>();
        float uv[kItems], raw[kItems], dl[kItems];
        if (full) {
            load_items<in_t, true>(u_base, e0, n_el, uv);
            load_items<in_t, true>(dl_base, e0, n_el, raw, kFill);
        } else {
            load_items<in_t, false>(u_base, e0, n_el, uv);
            load_items<in_t, false>(dl_base, e0, n_el, raw, kFill);
        }

        // the (at most) two rows this lane touches: items [0,k) lie in row a, [k,8) in row b
        uint32_t rl, l0;
        divmod((uint32_t)min(e0, n_el - 1), divL, rl, l0);
        const int k = kGran == kItems ? kItems : min(kItems, L - (int)l0);
        float A_a[kN], A_b[kN], D_a, D_b, bias_a, bias_b;
        uint32_t Boff_a, Boff_b, Coff_a, Coff_b;      // element offsets; the host checked they fit 32 bits
        {
            const uint32_t row_a = (uint32_t)r0 + rl;
            uint32_t b, d, grp, rem;
            divmod(row_a, divDim, b, d);
            divmod(d, divDpg, grp, rem);
#pragma unroll
            for (int n = 0; n < kN; ++n) A_a[n] = p.A[d * p.A_ds + n * p.A_ns] * kLog2e;
            D_a = p.D ? p.D[d] : 0.0f;
            bias_a = p.bias ? p.bias[d] : 0.0f;
            Boff_a = b * (uint32_t)p.B_bs + grp * (uint32_t)p.B_gs;
            Coff_a = b * (uint32_t)p.C_bs + grp * (uint32_t)p.C_gs;
            if constexpr (kGran != kItems) {
                const uint32_t row_b = min(row_a + 1u, (uint32_t)p.rows - 1u);
                divmod(row_b, divDim, b, d);
                divmod(d, divDpg, grp, rem);
#pragma unroll
                for (int n = 0; n < kN; ++n) A_b[n] = p.A[d * p.A_ds + n * p.A_ns] * kLog2e;
                D_b = p.D ? p.D[d] : 0.0f;
                bias_b = p.bias ? p.bias[d] : 0.0f;
                Boff_b = b * (uint32_t)p.B_bs + grp * (uint32_t)p.B_gs;
                Coff_b = b * (uint32_t)p.C_bs + grp * (uint32_t)p.C_gs;
            } else {
#pragma unroll
                for (int n = 0; n < kN; ++n) A_b[n] = A_a[n];
                D_b = D_a; bias_b = bias_a; Boff_b = Boff_a; Coff_b = Coff_a;
            }
        }

        // Every group's (row, position) is a real run of kGran elements of B / C even for items past the end of
        // this wavefront's run (row b is clamped, positions stay below L), so the gathers need no guard.
        float du[kItems], y[kItems], bias_items[kItems];
        bool in_a[kGroups], first[kGroups];
        uint32_t boff[kGroups], coff[kGroups];
        float *x_end[kX ? kGroups : 1];       // kX: where the group's last item puts its state (null: not a chunk end)
#pragma unroll
        for (int gi = 0; gi < kGroups; ++gi) {
            in_a[gi] = kGran == kItems ? true : gi * kGran < k;
            const uint32_t li = in_a[gi] ? l0 + gi * kGran : (uint32_t)(gi * kGran - k);
            first[gi] = li == 0;
            if constexpr (kX) {
                const uint32_t l_end = li + kGran;
                const bool ends = e0 + gi * kGran < n_el && (l_end == (uint32_t)L || l_end % SS2D_SCAN_CHUNK == 0);
                const int64_t row = r0 + rl + (in_a[gi] ? 0 : 1);
                x_end[gi] = ends ? p.x + (row * p.n_chunks + (l_end - 1) / SS2D_SCAN_CHUNK) * 2 * kN : nullptr;
            }
            boff[gi] = (in_a[gi] ? Boff_a : Boff_b) + li;
            coff[gi] = (in_a[gi] ? Coff_a : Coff_b) + li;
#pragma unroll
            for (int i = 0; i < kGran; ++i) bias_items[gi * kGran + i] = in_a[gi] ? bias_a : bias_b;
        }
        delta_transform<kSoftplus>(raw, bias_items, dl);
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            if constexpr (!kSoftplus) dl[i] = (e0 + i < n_el) ? dl[i] : 0.0f;
            du[i] = dl[i] * uv[i];                       // u is 0 past the end of the run
            y[i] = (in_a[i / kGran] ? D_a : D_b) * uv[i];
        }

#pragma unroll
        for (int n = 0; n < kN; ++n) {
            float Bv[kItems], Cv[kItems];
#pragma unroll
            for (int gi = 0; gi < kGroups; ++gi) {
                float bg[kGran], cg[kGran];
                gather_group<in_t, kGran>(B_rsrc, boff[gi], (uint32_t)n * (uint32_t)p.B_ns, bg);
                gather_group<in_t, kGran>(C_rsrc, coff[gi], (uint32_t)n * (uint32_t)p.C_ns, cg);
#pragma unroll
                for (int i = 0; i < kGran; ++i) { Bv[gi * kGran + i] = bg[i]; Cv[gi * kGran + i] = cg[i]; }
            }
            float ac[kItems], hh[kItems], gg[kX ? kItems : 1];
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                const int gi = i / kGran;
                float a = __builtin_amdgcn_exp2f(dl[i] * (in_a[gi] ? A_a[n] : A_b[n]));
                float c = 0.0f;
                if (i % kGran == 0) {
                    if constexpr (kX) c = first[gi] ? a : 0.0f;
                    a = first[gi] ? 0.0f : a;
                }
                // past the end of the run the gathered B belongs to some other row: keep it out
                const float bb = (e0 + i < n_el) ? Bv[i] * du[i] : 0.0f;
                ac[i] = i == 0 ? a : ac[i - 1] * a;
                hh[i] = i == 0 ? bb : fmaf(a, hh[i - 1], bb);
                if constexpr (kX) gg[i] = i == 0 ? c : (i % kGran == 0 ? fmaf(a, gg[i - 1], c) : a * gg[i - 1]);
            }
            float a_ex, h_ex, a_tot, h_tot, s_in;
            if constexpr (kX) {
                float g_ex, g_tot;
                wave_scan_pairs2(ac[kItems - 1], hh[kItems - 1], gg[kItems - 1], a_ex, h_ex, g_ex, a_tot, h_tot, g_tot);
                s_in = fmaf(a_ex, h_reg[n], h_ex);
                const float g_in = fmaf(a_ex, g_reg[n], g_ex);
#pragma unroll
                for (int gi = 0; gi < kGroups; ++gi) {
                    const int ie = gi * kGran + kGran - 1;
                    if (x_end[gi]) {
                        x_end[gi][2 * n] = fmaf(ac[ie], g_in, gg[ie]);
                        x_end[gi][2 * n + 1] = fmaf(ac[ie], s_in, hh[ie]);
                    }
                }
                g_reg[n] = fmaf(a_tot, g_reg[n], g_tot);
            } else {
                wave_scan_pairs(ac[kItems - 1], hh[kItems - 1], a_ex, h_ex, a_tot, h_tot);
                s_in = fmaf(a_ex, h_reg[n], h_ex);
            }
#pragma unroll
            for (int i = 0; i < kItems; ++i) y[i] = fmaf(Cv[i], fmaf(ac[i], s_in, hh[i]), y[i]);
            h_reg[n] = fmaf(a_tot, h_reg[n], h_tot);
        }
        if constexpr (sizeof(out_t) == 4) store_pass_f32(y_tile[wave], o_buf, pass * kPass, lane, y);
        else if (full) store_items<out_t, true>(o_base, e0, n_el, y);
        else store_items<out_t, false>(o_base, e0, n_el, y);
    }
}

// ---- four wavefronts per row -------------------------------------------------------------
// Workgroup = one row.  Per 2048-position chunk wave w takes positions [w*512, w*512+512).
// LDS: agg[2][N][4] pass totals (double-buffered by chunk parity), state[2][N] chunk-start
// state (running a-product, h).  One barrier per (chunk, state).
template <typename in_t, typename out_t, bool kVec, bool kSoftplus>
__global__ __launch_bounds__(kBlock) void scan_row4_kernel(const ScanArgs p) {
    extern __shared__ __align__(16) float smem[];
    const int N = p.N;
    float2 *agg = reinterpret_cast<float2 *>(smem);                  // [2][N][4]
    float2 *state = agg + 2 * N * kWavesPerWg;                       // [2][N]
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int row = (int)xcd_contiguous_id(blockIdx.x, gridDim.x);   // grid == rows exactly

    const int b = row / p.dim, d = row - b * p.dim;
    const int grp = d / p.dim_per_group, dg = d / p.dim_per_delta;
    const in_t *u_row = reinterpret_cast<const in_t *>(p.u) + b * p.u_bs + d * p.u_ds;
    const in_t *dl_row = reinterpret_cast<const in_t *>(p.delta) + b * p.dl_bs + dg * p.dl_ds;
    const in_t *B_row = reinterpret_cast<const in_t *>(p.B) + b * p.B_bs + grp * p.B_gs;
    const in_t *C_row = reinterpret_cast<const in_t *>(p.C) + b * p.C_bs + grp * p.C_gs;
    out_t *o_row = reinterpret_cast<out_t *>(p.out) + b * p.o_bs + d * p.o_ds;
    const float *A_row = p.A + d * p.A_ds;
    float *x_row = p.x ? p.x + (size_t)row * p.n_chunks * 2 * N : nullptr;
    const float Dv = p.D ? p.D[d] : 0.0f;
    const float bias = p.bias ? p.bias[dg] : 0.0f;
    const int L = p.L;

    constexpr bool kTiledStore = kVec && sizeof(out_t) == 4;     // fp32 out as whole 1 KB runs (store_pass_f32)
    __shared__ __align__(16) float y_tile[kTiledStore ? kWavesPerWg : 1][kTiledStore ? kPass : 4];
    const __amdgpu_buffer_rsrc_t o_buf = row_buffer(o_row, kTiledStore ? L : 0);
    const int n_chunks = (L + SS2D_SCAN_CHUNK - 1) / SS2D_SCAN_CHUNK;
    // the next chunk's u / delta (and B / C of the first state) are requested before this chunk's arithmetic and its
    // barriers: a wavefront always has a chunk of loads in flight (positions past the row's end come back as the fill)
    const int pos_first = wave * kPass + lane * kItems;
    Raw8<in_t> u_nx = load_raw<in_t, kVec, true>(u_row, pos_first, L);
    Raw8<in_t> dl_nx = load_raw<in_t, kVec, true>(dl_row, pos_first, L, delta_fill<kSoftplus>());
    Raw8<in_t> B_nx = load_raw<in_t, kVec>(B_row, pos_first, L), C_nx = load_raw<in_t, kVec>(C_row, pos_first, L);
    for (int chunk = 0; chunk < n_chunks; ++chunk) {
        const int par = chunk & 1;
        const int pos = chunk * SS2D_SCAN_CHUNK + pos_first;
        const Raw8<in_t> u_raw = u_nx, dl_raw = dl_nx, B_raw = B_nx, C_raw = C_nx;
        if (chunk + 1 < n_chunks) {
            const int pos_nx = pos + SS2D_SCAN_CHUNK;
            u_nx = load_raw<in_t, kVec, true>(u_row, pos_nx, L);
            dl_nx = load_raw<in_t, kVec, true>(dl_row, pos_nx, L, delta_fill<kSoftplus>());
            B_nx = load_raw<in_t, kVec>(B_row, pos_nx, L);
            C_nx = load_raw<in_t, kVec>(C_row, pos_nx, L);
        }
        float dl[kItems], du[kItems], y[kItems];
        prepare_delta_u<in_t, kSoftplus>(u_raw, dl_raw, L - pos, bias, Dv, dl, du, y);
        for (int n = 0; n < N; ++n) {
            float Bv[kItems], Cv[kItems];
            if (n == 0) {
                unpack_raw<in_t>(B_raw, Bv);
                unpack_raw<in_t>(C_raw, Cv);
            } else {
                load_items<in_t, kVec>(B_row + n * p.B_ns, pos, L, Bv);
                load_items<in_t, kVec>(C_row + n * p.C_ns, pos, L, Cv);
            }
            const float A_log2e = A_row[n * p.A_ns] * kLog2e;
            float ac[kItems], hh[kItems];
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                const float a = __builtin_amdgcn_exp2f(dl[i] * A_log2e);
                const float bb = Bv[i] * du[i];
                ac[i] = i == 0 ? a : ac[i - 1] * a;
                hh[i] = i == 0 ? bb : fmaf(a, hh[i - 1], bb);
            }
            float a_ex, h_ex, a_tot, h_tot;
            wave_scan_pairs(ac[kItems - 1], hh[kItems - 1], a_ex, h_ex, a_tot, h_tot);
            float2 *agg_n = agg + ((size_t)par * N + n) * kWavesPerWg;
            if (lane == 0) agg_n[wave] = make_float2(a_tot, h_tot);
            __syncthreads();
            const float2 st = chunk == 0 ? make_float2(1.0f, 0.0f) : state[par * N + n];
            float cin = st.y, aprod = st.x;
#pragma unroll
            for (int j = 0; j < kWavesPerWg; ++j) {
                const float2 g = agg_n[j];
                if (j < wave) cin = fmaf(g.x, cin, g.y);
                aprod *= g.x;
            }
            const float s_in = fmaf(a_ex, cin, h_ex);
#pragma unroll
            for (int i = 0; i < kItems; ++i) y[i] = fmaf(Cv[i], fmaf(ac[i], s_in, hh[i]), y[i]);
            if (wave == kWavesPerWg - 1 && lane == 0) {
                const float h_end = fmaf(a_tot, cin, h_tot);
                state[(par ^ 1) * N + n] = make_float2(aprod, h_end);
                if (x_row) {
                    x_row[(size_t)chunk * 2 * N + 2 * n] = aprod;
                    x_row[(size_t)chunk * 2 * N + 2 * n + 1] = h_end;
                }
            }
        }
        if constexpr (kTiledStore) store_pass_f32(y_tile[wave], o_buf, chunk * SS2D_SCAN_CHUNK + wave * kPass, lane, y);
        else store_items<out_t, kVec>(o_row, pos, L, y);
    }
}

// ---- four wavefronts per row, one state, 16-byte vectors: the chunks' loads in a ring ----------------------------------
// The same split of a row, with u, delta, B, C and out addressed through buffer descriptors: every load and store is
// unconditional (the hardware drops what lies past the row's end) and every chunk is the same instruction stream, so
// the memory counter -- loads and stores retire in issue order -- can be waited on exactly.  A chunk waits for ITS four
// loads while those of the next kRing - 1 chunks and the stores of the last ones are in flight, and re-issues its
// registers for the chunk kRing ahead when it is done with them.  (With loads under per-lane conditions the compiler
// has to wait for everything outstanding, the stores of the chunk before included, ahead of each chunk.)
template <typename in_t, typename out_t, bool kSoftplus>
__global__ __launch_bounds__(kBlock, 6) void scan_row4_ring_kernel(const ScanArgs p) {
    constexpr int kRing = 2;      // three chunks deep measured the same and leaves a SIMD four wavefronts instead of six
    __shared__ float2 agg[2][kWavesPerWg];                           // pass totals, by chunk parity
    __shared__ float2 state[2];                                      // (running a-product, h) entering a chunk
    constexpr bool kTiledStore = sizeof(out_t) == 4;
    __shared__ __align__(16) float y_tile[kTiledStore ? kWavesPerWg : 1][kTiledStore ? kPass : 4];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int row = (int)xcd_contiguous_id(blockIdx.x, gridDim.x);   // grid == rows exactly

    const int b = row / p.dim, d = row - b * p.dim;
    const int grp = d / p.dim_per_group, dg = d / p.dim_per_delta;
    const int L = p.L;
    const __amdgpu_buffer_rsrc_t u_buf = row_buffer(reinterpret_cast<const in_t *>(p.u) + b * p.u_bs + d * p.u_ds, L),
                                 dl_buf = row_buffer(reinterpret_cast<const in_t *>(p.delta) + b * p.dl_bs + dg * p.dl_ds, L),
                                 B_buf = row_buffer(reinterpret_cast<const in_t *>(p.B) + b * p.B_bs + grp * p.B_gs, L),
                                 C_buf = row_buffer(reinterpret_cast<const in_t *>(p.C) + b * p.C_bs + grp * p.C_gs, L),
                                 o_buf = row_buffer(reinterpret_cast<out_t *>(p.out) + b * p.o_bs + d * p.o_ds, L);
    float *x_row = p.x ? p.x + (size_t)row * p.n_chunks * 2 : nullptr;
    const float A_log2e = p.A[d * p.A_ds] * kLog2e;
    const float Dv = p.D ? p.D[d] : 0.0f;
    const float bias = p.bias ? p.bias[dg] : 0.0f;

    const int n_chunks = (L + SS2D_SCAN_CHUNK - 1) / SS2D_SCAN_CHUNK;
    const int pos_first = wave * kPass + lane * kItems;
    struct ChunkLoads { Raw8<in_t> u, dl, B, C; };
    ChunkLoads ring[kRing];
    auto issue = [&](int chunk, ChunkLoads &r) {                     // a chunk beyond the row reads nothing
        const int pos = chunk * SS2D_SCAN_CHUNK + pos_first;
        r.u = load_raw_buffer<in_t, true>(u_buf, pos);
        r.dl = load_raw_buffer<in_t, true>(dl_buf, pos);
        r.B = load_raw_buffer<in_t>(B_buf, pos);
        r.C = load_raw_buffer<in_t>(C_buf, pos);
    };
#pragma unroll
    for (int s = 0; s < kRing; ++s) {
        issue(s, ring[s]);
        __builtin_amdgcn_sched_barrier(0);       // in chunk order, as the loop issues them: the waits count on it
    }
    auto do_chunk = [&](int chunk, const ChunkLoads &r) {
        const int par = chunk & 1;
        const int pos = chunk * SS2D_SCAN_CHUNK + pos_first;
        float dl[kItems], du[kItems], y[kItems], Bv[kItems], Cv[kItems];
        prepare_delta_u<in_t, kSoftplus>(r.u, r.dl, kItems, bias, Dv, dl, du, y);
        unpack_raw<in_t>(r.B, Bv);
        unpack_raw<in_t>(r.C, Cv);
        if (chunk == n_chunks - 1) {
            // lanes past the row's end were fed zeros: u = 0 already makes their b term 0; their step must be 0 too
            // (a = 1), or the state the row ends with would go on decaying
#pragma unroll
            for (int i = 0; i < kItems; ++i) dl[i] = pos + i < L ? dl[i] : 0.0f;   // (fp32 rows may end mid-lane)
        }
        float ac[kItems], hh[kItems];
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            const float a = __builtin_amdgcn_exp2f(dl[i] * A_log2e);
            const float bb = Bv[i] * du[i];
            ac[i] = i == 0 ? a : ac[i - 1] * a;
            hh[i] = i == 0 ? bb : fmaf(a, hh[i - 1], bb);
        }
        float a_ex, h_ex, a_tot, h_tot;
        wave_scan_pairs(ac[kItems - 1], hh[kItems - 1], a_ex, h_ex, a_tot, h_tot);
        if (lane == 0) agg[par][wave] = make_float2(a_tot, h_tot);
        __syncthreads();
        const float2 st = chunk == 0 ? make_float2(1.0f, 0.0f) : state[par];
        float cin = st.y, aprod = st.x;
#pragma unroll
        for (int j = 0; j < kWavesPerWg; ++j) {
            const float2 g = agg[par][j];
            if (j < wave) cin = fmaf(g.x, cin, g.y);
            aprod *= g.x;
        }
        const float s_in = fmaf(a_ex, cin, h_ex);
#pragma unroll
        for (int i = 0; i < kItems; ++i) y[i] = fmaf(Cv[i], fmaf(ac[i], s_in, hh[i]), y[i]);
        if (wave == kWavesPerWg - 1 && lane == 0) {
            const float h_end = fmaf(a_tot, cin, h_tot);
            state[par ^ 1] = make_float2(aprod, h_end);
            if (x_row) { x_row[(size_t)chunk * 2] = aprod; x_row[(size_t)chunk * 2 + 1] = h_end; }
        }
        if constexpr (kTiledStore) store_pass_f32(y_tile[wave], o_buf, chunk * SS2D_SCAN_CHUNK + wave * kPass, lane, y);
        else store_items_buffer<out_t>(o_buf, pos, y);
    };
    // whole turns of the ring, then the last, partial turn as straight code (a `break` inside the turn would be one more
    // way into the loop header, from a state with fresh loads outstanding, and the waits there would have to allow for it)
    int c0 = 0;
    for (; c0 + kRing <= n_chunks; c0 += kRing) {
#pragma unroll
        for (int s = 0; s < kRing; ++s) {
            do_chunk(c0 + s, ring[s]);
            issue(c0 + s + kRing, ring[s]);
        }
    }
#pragma unroll
    for (int s = 0; s < kRing - 1; ++s)
        if (c0 + s < n_chunks) do_chunk(c0 + s, ring[s]);
}

// ---- host side -----------------------------------------------------------------------------
static bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

constexpr int kFlatTargetElems = 4096;   // positions a wavefront of the flat kernel walks

// Largest element offset the flat kernel forms into B or C (it indexes them with 32-bit offsets).
static int64_t span_elems(const ScanArgs &a, int64_t bs, int64_t gs, int64_t ns) {
    const int64_t groups = a.dim / a.dim_per_group;
    return (int64_t)(a.batch - 1) * bs + (groups - 1) * gs + (int64_t)(a.N - 1) * ns + a.L;
}
static bool span_fits_u32(const ScanArgs &a, int64_t elem_bytes) {
    const int64_t lim = 0x7fffffffll;   // byte extents are handed to the buffer descriptor as a positive int
    return a.B_bs >= 0 && a.B_gs >= 0 && a.B_ns >= 0 && a.C_bs >= 0 && a.C_gs >= 0 && a.C_ns >= 0 &&
           span_elems(a, a.B_bs, a.B_gs, a.B_ns) * elem_bytes < lim && span_elems(a, a.C_bs, a.C_gs, a.C_ns) * elem_bytes < lim;
}

// The flat kernel needs dense u / delta / out (rows adjacent in memory, base 16-byte aligned), one delta row
// per channel, rows of at least one lane vector, and dstate 1 or 16.
static bool flat_eligible(const ScanArgs &a, const ss2d_scan_params *q) {
    const int64_t L = a.L, KD = a.dim;
    // rows of four passes and more only where the row kernel would fall back to element-wise accesses (the caller
    // checks that) and there are rows enough to fill the chip eight to a wavefront (measured, unaligned bf16 rows of
    // 5625 positions: 27 264 rows 515 us against 1112, 6144 rows 191 against 241, 3072 rows 153 against 114)
    const bool length_ok = L < 4 * kPass || (L <= (1 << 24) && a.N == 1 && a.rows >= 6144);
    return L >= kItems && length_ok && (a.N == 1 || a.N == 16) && q->delta_dim == q->dim &&
           a.u_ds == L && a.dl_ds == L && a.o_ds == L && a.u_bs == KD * L && a.dl_bs == KD * L && a.o_bs == KD * L &&
           aligned16(q->u) && aligned16(q->delta) && aligned16(q->out) &&
           span_fits_u32(a, q->in_dtype == SS2D_F32 ? 4 : 2);
}

static int gcd_i64(int64_t a, int64_t b) { while (b) { const int64_t t = a % b; a = b; b = t; } return (int)(a < 0 ? -a : a); }

// Largest granularity (1, 2, 4 or 8 elements) at which the flat kernel may treat rows and gather B / C: it must
// divide L (rows change only at multiples of it) and every B / C stride, and the B / C bases must be aligned to it.
static int flat_granularity(const ScanArgs &a, int64_t elem_bytes) {
    int64_t g = gcd_i64(a.L, kItems);
    const int64_t strides[] = {a.B_bs, a.B_gs, a.B_ns, a.C_bs, a.C_gs, a.C_ns};
    for (int64_t s : strides) g = gcd_i64(g, s == 0 ? g : s);
    const uintptr_t bases = reinterpret_cast<uintptr_t>(a.B) | reinterpret_cast<uintptr_t>(a.C);
    while (g > 1 && (bases % (uintptr_t)(g * elem_bytes)) != 0) g /= 2;
    return (int)g;
}

template <typename in_t, typename out_t>
static int launch_flat(const ScanArgs &a_in, hipStream_t stream) {
    ScanArgs a = a_in;
    a.B_span_bytes = (uint32_t)(span_elems(a, a.B_bs, a.B_gs, a.B_ns) * (int64_t)sizeof(in_t));
    a.C_span_bytes = (uint32_t)(span_elems(a, a.C_bs, a.C_gs, a.C_ns) * (int64_t)sizeof(in_t));
    int rows_per_wave = 8 * (int)((kFlatTargetElems + 8 * (int64_t)a.L - 1) / (8 * (int64_t)a.L));
    const int64_t n_waves = ((int64_t)a.rows + rows_per_wave - 1) / rows_per_wave;
    const uint32_t n_wg = (uint32_t)((n_waves + kWavesPerWg - 1) / kWavesPerWg);
    const FastDiv dL = make_fastdiv((uint32_t)a.L), dDim = make_fastdiv((uint32_t)a.dim),
                  dDpg = make_fastdiv((uint32_t)a.dim_per_group);
    const int gran = flat_granularity(a, (int64_t)sizeof(in_t));
#define SS2D_LAUNCH_FLAT(N, SP, G, X) \
    hipLaunchKernelGGL((scan_flat_kernel<in_t, out_t, N, SP, G, X>), dim3(n_wg), dim3(kBlock), 0, stream, a, rows_per_wave, dL, dDim, dDpg)
#define SS2D_LAUNCH_FLAT_G(N, SP, X)                                \
    switch (gran) {                                                  \
        case 8: SS2D_LAUNCH_FLAT(N, SP, 8, X); break;                \
        case 4: SS2D_LAUNCH_FLAT(N, SP, 4, X); break;                \
        case 2: SS2D_LAUNCH_FLAT(N, SP, 2, X); break;                \
        default: SS2D_LAUNCH_FLAT(N, SP, 1, X); break;               \
    }
#define SS2D_LAUNCH_FLAT_X(N, SP) \
    if (a.x) { SS2D_LAUNCH_FLAT_G(N, SP, true) } else { SS2D_LAUNCH_FLAT_G(N, SP, false) }
    if (a.N == 1) {
        if (a.softplus) { SS2D_LAUNCH_FLAT_X(1, true) } else { SS2D_LAUNCH_FLAT_X(1, false) }
    } else {
        if (a.softplus) { SS2D_LAUNCH_FLAT_X(16, true) } else { SS2D_LAUNCH_FLAT_X(16, false) }
    }
#undef SS2D_LAUNCH_FLAT_X
#undef SS2D_LAUNCH_FLAT_G
#undef SS2D_LAUNCH_FLAT
    return launch_status();
}

template <typename in_t, typename out_t, bool kVec>
static int launch_scan(const ScanArgs &a, bool split_rows, hipStream_t stream) {
    if (split_rows) {
        if constexpr (kVec) {
            if (a.N == 1) {
                // one state, vector I/O: the ring kernel (256^2 maps at batch 4: 170 -> 165 us)
                if (a.softplus) hipLaunchKernelGGL((scan_row4_ring_kernel<in_t, out_t, true>), dim3((uint32_t)a.rows), dim3(kBlock), 0, stream, a);
                else hipLaunchKernelGGL((scan_row4_ring_kernel<in_t, out_t, false>), dim3((uint32_t)a.rows), dim3(kBlock), 0, stream, a);
                return launch_status();
            }
        }
        const size_t smem = (size_t)(2 * a.N * kWavesPerWg + 2 * a.N) * sizeof(float2);
        if (a.softplus) {
            hipLaunchKernelGGL((scan_row4_kernel<in_t, out_t, kVec, true>), dim3((uint32_t)a.rows), dim3(kBlock), smem, stream, a);
        } else {
            hipLaunchKernelGGL((scan_row4_kernel<in_t, out_t, kVec, false>), dim3((uint32_t)a.rows), dim3(kBlock), smem, stream, a);
        }
        return launch_status();
    }
    const uint32_t n_wg = (uint32_t)((a.rows + kWavesPerWg - 1) / kWavesPerWg);
#define SS2D_LAUNCH_ROW(N, SP, SMEM) \
    hipLaunchKernelGGL((scan_row_kernel<in_t, out_t, N, kVec, SP>), dim3(n_wg), dim3(kBlock), SMEM, stream, a)
    if (a.N == 1) {
        const int tail = a.L % kPass;
        if constexpr (kVec) {
            if (tail > 0 && tail <= kScanTailMax * kWave) {
                if (a.softplus) {
                    hipLaunchKernelGGL((scan_row_kernel<in_t, out_t, 1, true, true, true>), dim3(n_wg), dim3(kBlock), 0, stream, a);
                } else {
                    hipLaunchKernelGGL((scan_row_kernel<in_t, out_t, 1, true, false, true>), dim3(n_wg), dim3(kBlock), 0, stream, a);
                }
                return launch_status();
            }
        }
        if (a.softplus) SS2D_LAUNCH_ROW(1, true, 0); else SS2D_LAUNCH_ROW(1, false, 0);
    } else {
        const size_t smem = (size_t)kWavesPerWg * 2 * a.N * sizeof(float);
        if (a.softplus) SS2D_LAUNCH_ROW(0, true, smem); else SS2D_LAUNCH_ROW(0, false, smem);
    }
#undef SS2D_LAUNCH_ROW
    return launch_status();
}

template <typename in_t, typename out_t>
static int dispatch_vec(const ScanArgs &a, bool vec, int kernel, hipStream_t stream) {
    if (kernel == SS2D_SCAN_KERNEL_FLAT) return launch_flat<in_t, out_t>(a, stream);
    const bool split_rows = kernel == SS2D_SCAN_KERNEL_ROW4;
    return vec ? launch_scan<in_t, out_t, true>(a, split_rows, stream) : launch_scan<in_t, out_t, false>(a, split_rows, stream);
}

}  // namespace ss2d

namespace ss2d {

// Validation and kernel choice shared by the launch and the query entry points.  Returns an SS2D_SCAN_KERNEL_* id
// (SS2D_SCAN_KERNEL_NONE for an empty problem) or a negative status; fills `a` and `vec` for the launch.
static int plan_scan(const ss2d_scan_params *q, ScanArgs &a, bool &vec) {
    if (!q) return SS2D_EINVAL;
    if (q->batch < 0 || q->dim < 0 || q->seqlen < 0) return SS2D_EINVAL;
    if (q->dstate <= 0 || q->dstate > 256 || q->n_groups <= 0 || q->delta_dim <= 0) return SS2D_EINVAL;
    if (q->in_dtype != SS2D_F32 && q->in_dtype != SS2D_BF16 && q->in_dtype != SS2D_F16) return SS2D_EINVAL;
    if (q->out_dtype != SS2D_F32 && q->out_dtype != q->in_dtype) return SS2D_EINVAL;
    if (q->dim % q->n_groups != 0 || q->dim % q->delta_dim != 0) return SS2D_EINVAL;
    if (q->batch == 0 || q->dim == 0 || q->seqlen == 0) return SS2D_SCAN_KERNEL_NONE;
    if (!q->u || !q->delta || !q->A || !q->B || !q->C || !q->out) return SS2D_EINVAL;
    if ((int64_t)q->batch * q->dim > 0x7fffffff - kWavesPerWg) return SS2D_ENOTSUP;

    a.u = q->u; a.delta = q->delta; a.B = q->B; a.C = q->C;
    a.A = (const float *)q->A; a.D = (const float *)q->D; a.bias = (const float *)q->delta_bias;
    a.out = q->out; a.x = (float *)q->x;
    a.batch = q->batch; a.dim = q->dim; a.L = q->seqlen; a.N = q->dstate;
    a.dim_per_group = q->dim / q->n_groups;
    a.dim_per_delta = q->dim / q->delta_dim;
    a.n_chunks = (q->seqlen + SS2D_SCAN_CHUNK - 1) / SS2D_SCAN_CHUNK;
    a.softplus = q->delta_softplus;
    a.u_bs = q->u_batch_stride; a.u_ds = q->u_d_stride;
    a.dl_bs = q->delta_batch_stride; a.dl_ds = q->delta_d_stride;
    a.A_ds = q->A_d_stride; a.A_ns = q->A_dstate_stride;
    a.B_bs = q->B_batch_stride; a.B_gs = q->B_group_stride; a.B_ns = q->B_dstate_stride;
    a.C_bs = q->C_batch_stride; a.C_gs = q->C_group_stride; a.C_ns = q->C_dstate_stride;
    a.o_bs = q->out_batch_stride; a.o_ds = q->out_d_stride;
    a.rows = q->batch * q->dim;
    a.vec_out_ok = 0;
    a.B_span_bytes = a.C_span_bytes = 0;
    const int64_t in_bytes = q->in_dtype == SS2D_F32 ? 4 : 2;
    const bool spans_fit = span_fits_u32(a, in_bytes);
    if (spans_fit) {
        a.B_span_bytes = (uint32_t)(span_elems(a, a.B_bs, a.B_gs, a.B_ns) * in_bytes);
        a.C_span_bytes = (uint32_t)(span_elems(a, a.C_bs, a.C_gs, a.C_ns) * in_bytes);
    }

    // 16-byte vector I/O needs every row start and the row length on a 16-byte grid.
    const int64_t in_vec = q->in_dtype == SS2D_F32 ? 4 : 8;
    const int64_t out_vec = q->out_dtype == SS2D_F32 ? 4 : 8;
    const int64_t in_strides[] = {a.u_bs, a.u_ds, a.dl_bs, a.dl_ds, a.B_bs, a.B_gs, a.B_ns, a.C_bs, a.C_gs, a.C_ns};
    vec = aligned16(q->u) && aligned16(q->delta) && aligned16(q->B) && aligned16(q->C) && aligned16(q->out);
    vec = vec && (q->seqlen % in_vec == 0) && (q->seqlen % out_vec == 0);
    vec = vec && q->seqlen < (1 << 29);               // the vector paths address a row with 32-bit byte offsets
    for (int64_t s : in_strides) vec = vec && (s % in_vec == 0);
    vec = vec && (a.o_bs % out_vec == 0) && (a.o_ds % out_vec == 0);

    // rows of 49 / 196 positions, one state, rows adjacent in memory: one segment of a row per lane
    if (scan_small_eligible(a, q->in_dtype, q->u, q->delta, q->out)) return SS2D_SCAN_KERNEL_SMALL;
    // several states per channel and enough channels per group to fill wavefronts: one channel per lane
    if (vec && scan_chan_eligible(a)) return SS2D_SCAN_KERNEL_CHAN;
    // A pass of the flat kernel costs about 1.4x a pass of the row kernel (measured), so the flat kernel wins
    // when the row kernel would leave more than ~30 % of its lanes idle, or cannot use vector I/O at all.
    const int64_t row_slots = ((int64_t)q->seqlen + kPass - 1) / kPass * kPass;
    if (flat_eligible(a, q) && (!vec || 10 * (int64_t)q->seqlen < 7 * row_slots)) return SS2D_SCAN_KERNEL_FLAT;
    // few long rows: every row split over the four wavefronts of a workgroup (3072 rows and more: a wavefront per row is faster)
    if (a.L > SS2D_SCAN_CHUNK && a.rows < 2048) return SS2D_SCAN_KERNEL_ROW4;
    return SS2D_SCAN_KERNEL_ROW;
}

}  // namespace ss2d

extern "C" int ss2d_selective_scan_kernel(const ss2d_scan_params *q) {
    ss2d::ScanArgs a;
    bool vec = false;
    return ss2d::plan_scan(q, a, vec);
}

extern "C" int ss2d_selective_scan_fwd_maps(const ss2d_scan_params *q, const void *x_t, void *stream) {
    using namespace ss2d;
    if (!q || !x_t) return SS2D_EINVAL;
    if (q->n_groups != 4 || q->dim % 4 != 0) return SS2D_EINVAL;
    ScanArgs a;
    bool vec = false;
    const int kernel = plan_scan(q, a, vec);
    if (kernel < 0) return kernel;
    if (kernel == SS2D_SCAN_KERNEL_NONE) return SS2D_OK;
    // only the channel-per-lane kernel reads u through the routes
    if (kernel != SS2D_SCAN_KERNEL_CHAN || !aligned16(x_t)) return SS2D_ENOTSUP;
    return launch_scan_chan(a, q->in_dtype, q->out_dtype, (hipStream_t)stream, x_t);
}

extern "C" int ss2d_selective_scan_fwd(const ss2d_scan_params *q, void *stream) {
    using namespace ss2d;
    ScanArgs a;
    bool vec = false;
    const int kernel = plan_scan(q, a, vec);
    if (kernel < 0) return kernel;
    if (kernel == SS2D_SCAN_KERNEL_NONE) return SS2D_OK;
    hipStream_t s = (hipStream_t)stream;
    if (kernel == SS2D_SCAN_KERNEL_SMALL) return launch_scan_small(a, q->in_dtype, q->out_dtype, s);
    if (kernel == SS2D_SCAN_KERNEL_CHAN) return launch_scan_chan(a, q->in_dtype, q->out_dtype, s);
    if (q->in_dtype == SS2D_F32) return dispatch_vec<float, float>(a, vec, kernel, s);
    if (q->in_dtype == SS2D_BF16) {
        return q->out_dtype == SS2D_F32 ? dispatch_vec<bf16_t, float>(a, vec, kernel, s)
                                        : dispatch_vec<bf16_t, bf16_t>(a, vec, kernel, s);
    }
    return q->out_dtype == SS2D_F32 ? dispatch_vec<f16_t, float>(a, vec, kernel, s) : dispatch_vec<f16_t, f16_t>(a, vec, kernel, s);
}

extern "C" int ss2d_abi_version(void) { return SS2D_ABI_VERSION; }

extern "C" const char *ss2d_strerror(int code) {
    switch (code) {
        case SS2D_OK: return "ok";
        case SS2D_EINVAL: return "invalid argument (shape, stride, dtype, pointer or flag)";
        case SS2D_ENOTSUP: return "request is valid but not supported by this build";
        case SS2D_ELAUNCH: return "HIP runtime refused the kernel launch";
        case SS2D_ENOMEM: return "workspace too small for this call (see the entry point's size rule)";
        default: return "unknown ss2d status";
    }
}
