// Device helpers shared by the scan kernels (selective_scan.hip, ss2d_core.hip): 8-wide loads and stores,
// buffer-descriptor gathers, the delta transform (bias + softplus) and the wavefront scan of (a, b) pairs.
#pragma once

#include "ss2d_common.h"

namespace ss2d {

constexpr int kItems = 8;                    // consecutive positions per lane per pass
constexpr int kPass = kWave * kItems;        // 512 positions per wavefront pass
constexpr int kWavesPerWg = kBlock / kWave;  // 4
constexpr int kPassesPerChunk = SS2D_SCAN_CHUNK / kPass;  // 4
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Arguments of the stand-alone scan kernels (selective_scan.hip, scan_chan.hip): the C ABI's ss2d_scan_params with
// derived fields.  Strides in elements.
struct ScanArgs {
    const void *u, *delta, *B, *C;
    const float *A, *D, *bias;
    void *out;
    float *x;
    int32_t batch, dim, L, N, dim_per_group, dim_per_delta, n_chunks, softplus;
    int64_t u_bs, u_ds, dl_bs, dl_ds, A_ds, A_ns, B_bs, B_gs, B_ns, C_bs, C_gs, C_ns, o_bs, o_ds;
    int32_t rows;
    int32_t vec_out_ok;                    // scan_small.hip: the output base is 16-byte aligned
    uint32_t B_span_bytes, C_span_bytes;   // extent of B / C reachable through the strides (buffer-descriptor kernels)
};

// scan_chan.hip: the channel-per-lane kernel for several states per channel.  True when it takes this problem
// (the caller has already established 16-byte vector I/O); launch returns an SS2D status.
bool scan_chan_eligible(const ScanArgs &a);
// xt != nullptr: a.u is the map x (batch, dim / 4, L) and xt its transpose, read through CrossScan's routes (group = direction)
int launch_scan_chan(const ScanArgs &a, int in_dtype, int out_dtype, hipStream_t stream, const void *xt = nullptr);

// Arguments of the fused core kernels (ss2d_core.hip, ss2d_core_small.hip): the C ABI's ss2d_core_params with derived
// fields.  Strides in elements.
struct CoreArgs {
    const void *x, *delta, *Bm, *Cm;
    const float *A, *Dv, *bias;
    void *y;
    int32_t B, D, H, W, L, CB, softplus, vec_ok, vec_out, stage_tiles, tile_merge;
    int64_t dl_ks, dl_ds, dl_bs;        // delta strides over direction, channel, batch (elements)
    int64_t B_ks, B_bs, C_ks, C_bs;     // B / C strides over direction and batch (elements)
    uint32_t B_span_bytes, C_span_bytes;
};

// scan_small.hip: the stand-alone scan for rows of 49 or 196 positions and one state, one segment of a row per lane.
bool scan_small_eligible(const ScanArgs &a, int in_dtype, const void *u, const void *delta, const void *out);
int launch_scan_small(const ScanArgs &a, int in_dtype, int out_dtype, hipStream_t stream);

// ss2d_core_small.hip: the row-per-lane kernel for small square maps.
bool core_small_eligible(const CoreArgs &a, int in_dtype);
int launch_core_small(const CoreArgs &a, int in_dtype, hipStream_t stream);

// ss2d_core_tiled.hip: the fused core for maps of any size (64 x 64 tiles, two passes and a carry scan; 16-bit inputs,
// map sides multiples of 8).  The workspace holds the runs' aggregates and carries.
bool core_tiled_eligible(const CoreArgs &a, int in_dtype);
int64_t core_tiled_workspace_bytes(const CoreArgs &a);
int launch_core_tiled(const CoreArgs &a, int in_dtype, void *workspace, hipStream_t stream);

// ---- 8-wide loads / stores ------------------------------------------------------------
// Eight consecutive elements of a row as they sit in registers before widening: 4 dwords for 16-bit
// types, 8 for fp32.  Keeping loads in this form lets a pass issue the NEXT pass's loads before it
// starts computing (software prefetch), which is what keeps enough bytes in flight per wavefront.
template <typename T> struct Raw8 { uint32_t w[sizeof(T) * 2]; };

// Items at positions >= L come back as `fill`.
template <typename T, bool kVec, bool kStream = false>
__device__ __forceinline__ Raw8<T> load_raw(const T *__restrict__ row, int pos, int L, float fill = 0.0f) {
    Raw8<T> r;
    // kStream: data read once (u, delta of a scan) as non-temporal loads of the vector path
    auto get = [](const T *src) {
        if constexpr (kStream) return load_streaming(reinterpret_cast<const uint4 *>(src));
        else return *reinterpret_cast<const uint4 *>(src);
    };
    if constexpr (kVec) {
        // the host guarantees 16-byte alignment and L % (16/sizeof(T)) == 0, so a vector is either
        // entirely inside the row or entirely outside
        if constexpr (sizeof(T) == 2) {
            const uint32_t fill2 = (uint32_t)from_f32<T>(fill).bits * 0x10001u;
            uint4 v = make_uint4(fill2, fill2, fill2, fill2);
            if (pos < L) v = get(row + pos);
            r.w[0] = v.x; r.w[1] = v.y; r.w[2] = v.z; r.w[3] = v.w;
        } else {
            const uint32_t f = f32_to_bits(fill);
            uint4 lo = make_uint4(f, f, f, f), hi = lo;
            if (pos < L) lo = get(row + pos);
            if (pos + 4 < L) hi = get(row + pos + 4);
            r.w[0] = lo.x; r.w[1] = lo.y; r.w[2] = lo.z; r.w[3] = lo.w;
            r.w[4] = hi.x; r.w[5] = hi.y; r.w[6] = hi.z; r.w[7] = hi.w;
        }
    } else {
        if constexpr (sizeof(T) == 2) {
            const uint32_t fb = from_f32<T>(fill).bits;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t lo = (pos + 2 * i < L) ? row[pos + 2 * i].bits : fb;
                const uint32_t hi = (pos + 2 * i + 1 < L) ? row[pos + 2 * i + 1].bits : fb;
                r.w[i] = lo | (hi << 16);
            }
        } else {
#pragma unroll
            for (int i = 0; i < kItems; ++i) r.w[i] = f32_to_bits((pos + i < L) ? row[pos + i] : fill);
        }
    }
    return r;
}

// Eight in-range, 16-byte-aligned elements, no bounds check.
template <typename T>
__device__ __forceinline__ Raw8<T> load_raw_unchecked(const T *__restrict__ row, int pos) {
    Raw8<T> r;
    const uint4 lo = *reinterpret_cast<const uint4 *>(row + pos);
    r.w[0] = lo.x; r.w[1] = lo.y; r.w[2] = lo.z; r.w[3] = lo.w;
    if constexpr (sizeof(T) == 4) {
        const uint4 hi = *reinterpret_cast<const uint4 *>(row + pos + 4);
        r.w[4] = hi.x; r.w[5] = hi.y; r.w[6] = hi.z; r.w[7] = hi.w;
    }
    return r;
}

template <typename T>
__device__ __forceinline__ void unpack_raw(const Raw8<T> &r, float (&v)[kItems]) {
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = to_f32(T{(uint16_t)(r.w[i] & 0xffffu)});
            v[2 * i + 1] = to_f32(T{(uint16_t)(r.w[i] >> 16)});
        }
    } else {
#pragma unroll
        for (int i = 0; i < kItems; ++i) v[i] = bits_to_f32(r.w[i]);
    }
}

template <typename T, bool kVec>
__device__ __forceinline__ void load_items(const T *__restrict__ row, int pos, int L, float (&v)[kItems],
                                           float fill = 0.0f) {
    unpack_raw<T>(load_raw<T, kVec>(row, pos, L, fill), v);
}

template <typename T, bool kVec>
__device__ __forceinline__ void store_items(T *__restrict__ row, int pos, int L, const float (&v)[kItems]) {
    if constexpr (kVec) {
        if constexpr (sizeof(T) == 2) {
            if (pos < L) {
                uint32_t w[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) w[i] = pack2_from_f32<T>(v[2 * i], v[2 * i + 1]);
                *reinterpret_cast<uint4 *>(row + pos) = make_uint4(w[0], w[1], w[2], w[3]);
            }
        } else {
            if (pos < L) *reinterpret_cast<float4 *>(row + pos) = make_float4(v[0], v[1], v[2], v[3]);
            if (pos + 4 < L) *reinterpret_cast<float4 *>(row + pos + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < kItems; ++i)
            if (pos + i < L) row[pos + i] = from_f32<T>(v[i]);
    }
}

constexpr int kBufferRsrcWord3 = 0x00020000;   // raw buffer, 32-bit data format (gfx9 family)

// A row of n_elems elements seen through a buffer descriptor: 32-bit byte offsets, and the hardware checks every dword
// against the row's end -- a load past it returns 0, a store past it is dropped -- so loads and stores need no branch.
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t row_buffer(const T *row, int n_elems) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(row), 0, n_elems * (int)sizeof(T), kBufferRsrcWord3);
}

// Eight elements from position `pos` of such a row (16-byte aligned: the vector paths' precondition).
template <typename T, bool kStream = false>
__device__ __forceinline__ Raw8<T> load_raw_buffer(__amdgpu_buffer_rsrc_t rsrc, int pos) {
    Raw8<T> r;
    const int byte_off = pos * (int)sizeof(T);
    constexpr int kAux = kStream ? 2 : 0;                        // the builtin's cache-policy operand: bit 1 = nt
    const auto lo = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_off, 0, kAux);
    r.w[0] = lo[0]; r.w[1] = lo[1]; r.w[2] = lo[2]; r.w[3] = lo[3];
    if constexpr (sizeof(T) == 4) {
        const auto hi = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_off + 16, 0, kAux);
        r.w[4] = hi[0]; r.w[5] = hi[1]; r.w[6] = hi[2]; r.w[7] = hi[3];
    }
    return r;
}

template <typename T>
__device__ __forceinline__ void store_items_buffer(__amdgpu_buffer_rsrc_t rsrc, int pos, const float (&v)[kItems]) {
    typedef uint32_t words4_t __attribute__((ext_vector_type(4)));
    const int byte_off = pos * (int)sizeof(T);
    if constexpr (sizeof(T) == 2) {
        words4_t w;
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = pack2_from_f32<T>(v[2 * i], v[2 * i + 1]);
        __builtin_amdgcn_raw_buffer_store_b128(w, rsrc, byte_off, 0, 0);
    } else {
        words4_t lo, hi;
#pragma unroll
        for (int i = 0; i < 4; ++i) { lo[i] = f32_to_bits(v[i]); hi[i] = f32_to_bits(v[4 + i]); }
        __builtin_amdgcn_raw_buffer_store_b128(lo, rsrc, byte_off, 0, 0);
        __builtin_amdgcn_raw_buffer_store_b128(hi, rsrc, byte_off + 16, 0, 0);
    }
}

// A pass's outputs, 8 consecutive positions per lane, stored as fp32 so that each store instruction writes 1 KB of
// consecutive addresses: at 32 bytes per lane an instruction would write every other 16 bytes of a 2 KB span, and
// memory takes the half-written lines measurably worse (one-state row scan of 56 x 56 maps, batch 128: 258 -> 232 us).
// The values go through a wavefront-private LDS tile of kPass floats (LDS serves a wavefront's accesses in order:
// no barrier), lane l then holds positions 4l .. 4l+3 and 256+4l .. 256+4l+3 of the pass.
__device__ __forceinline__ void store_pass_f32(float *tile, __amdgpu_buffer_rsrc_t rsrc, int pass_pos, int lane,
                                               const float (&v)[kItems]) {
    typedef uint32_t words4_t __attribute__((ext_vector_type(4)));
    float4 *t4 = reinterpret_cast<float4 *>(tile);
    t4[2 * lane] = make_float4(v[0], v[1], v[2], v[3]);
    t4[2 * lane + 1] = make_float4(v[4], v[5], v[6], v[7]);
    const float4 lo = t4[lane], hi = t4[kWave + lane];
    const words4_t wl = {f32_to_bits(lo.x), f32_to_bits(lo.y), f32_to_bits(lo.z), f32_to_bits(lo.w)};
    const words4_t wh = {f32_to_bits(hi.x), f32_to_bits(hi.y), f32_to_bits(hi.z), f32_to_bits(hi.w)};
    // non-temporal: the outputs are written once and read back by another kernel after hundreds of MB of other traffic
    // (stand-alone scan -2.5 .. -8 % by shape, scan + CrossMerge chains -2 .. -8 % except +2 % on 256 x 256 maps)
    constexpr int kNonTemporal = 2;      // the builtin's cache-policy operand: bit 1 = nt
    __builtin_amdgcn_raw_buffer_store_b128(wl, rsrc, (pass_pos + 4 * lane) * 4, 0, kNonTemporal);
    __builtin_amdgcn_raw_buffer_store_b128(wh, rsrc, (pass_pos + kPass / 2 + 4 * lane) * 4, 0, kNonTemporal);
}

template <typename T>
__device__ __forceinline__ float gather_elem(__amdgpu_buffer_rsrc_t rsrc, uint32_t elem_offset) {
    if constexpr (sizeof(T) == 2) {
        return to_f32(T{(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc, (int)(elem_offset * 2u), 0, 0)});
    } else {
        return bits_to_f32((uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(elem_offset * 4u), 0, 0));
    }
}

// delta -> dl for the 8 items of a lane.
//   kSoftplus: dl = softplus(x), x = raw + bias, as  max(x, 0) + log(1 + exp(-|x|))  with the two hardware
//   transcendentals in base 2: z = x * log2e, t = 2^-|z| <= 1, w = 1 + t, dl = ln2 * (max(z, 0) + log2 w) + c.
//   w = 1 + t loses the low bits of a small t; c = t - (w - 1) is exactly that loss (1 <= w <= 2), and
//   log(1 + t) = log(w) + c/w with c/w ~ c.  For x above the reference's threshold of 20 (where it returns x itself)
//   the log term is below 2.1e-9 = 1e-10 x, invisible in fp32, so no special case is needed.
//   A raw value of -inf (the fill for positions past the end of a row) gives t = 0, dl = 0: the identity pair.
//   !kSoftplus: dl = raw + bias; the caller zeroes positions past the end.
constexpr float kSoftplusThreshold = 20.0f;     // the backward's d softplus / dx is 1 above it, as in the reference

// softplus(x) for z = x * log2e
__device__ __forceinline__ float softplus_log2(float z) {
    const float t = __builtin_amdgcn_exp2f(-__builtin_fabsf(z));
    const float w = 1.0f + t;
    const float c = t - (w - 1.0f);
    return fmaf(__builtin_fmaxf(z, 0.0f), kLn2, fmaf(kLn2, __builtin_amdgcn_logf(w), c));
}

// softplus(x) / ln 2 for z = x * log2e:  max(z, 0) + log2(1 + 2^-|z|), without the compensation term of softplus_log2.
// 1 + t is rounded to fp32, which changes the result by at most 2^-24 * log2e in absolute terms: invisible unless the
// step itself is below ~1e-4, where 16-bit inputs have long lost it in their own rounding (a bf16 delta of -10 is known
// to 3 %).  For kernels whose delta arrives as bf16 / fp16 and whose time is their instruction count; results stay in
// units of ln 2 (the recurrence is linear in the step, so the factor is applied once to the output).
__device__ __forceinline__ float softplus_over_ln2(float z) {
    const float t = __builtin_amdgcn_exp2f(-__builtin_fabsf(z));
    return __builtin_fmaxf(z, 0.0f) + __builtin_amdgcn_logf(1.0f + t);
}

template <bool kSoftplus>
__device__ __forceinline__ void delta_transform(const float (&raw)[kItems], const float (&bias)[kItems],
                                                float (&dl)[kItems]) {
    if constexpr (kSoftplus) {
#pragma unroll
        for (int i = 0; i < kItems; ++i) dl[i] = softplus_log2(fmaf(raw[i], kLog2e, bias[i] * kLog2e));
    } else {
#pragma unroll
        for (int i = 0; i < kItems; ++i) dl[i] = raw[i] + bias[i];
    }
}

// Inclusive scan of (a,h) over the 64 lanes; returns this lane's EXCLUSIVE prefix in
// (a_ex,h_ex) and the wave total, uniform, in (a_tot,h_tot).  Call with all 64 lanes active.
// Each step combines a lane with the lane `shift` below it:  h += a * h_below;  a *= a_below.  The DPP operand does
// the lane movement inside the arithmetic instruction, and a lane without a source (row start, masked row) is left
// untouched by the hardware -- which is the identity (a_below = 1, h_below = 0) -- so a step is two instructions.
// The compiler does not fold its own DPP moves into these operations, hence the assembly; the s_nop are the two wait
// states a DPP read needs after a VALU write of the same register.
__device__ __forceinline__ void wave_scan_pairs(float a, float h, float &a_ex, float &h_ex, float &a_tot,
                                                float &h_tot) {
    float ax = 1.0f, hx = 0.0f;
#define SS2D_SCAN_STEP(CTRL)                                   \
    "v_fmac_f32_dpp %1, %1, %0 " CTRL " bank_mask:0xf\n\t" \
    "v_mul_f32_dpp %0, %0, %0 " CTRL " bank_mask:0xf\n\t"  \
    "s_nop 0\n\t"
    asm("s_nop 1\n\t"
                 SS2D_SCAN_STEP("row_shr:1 row_mask:0xf")
                 SS2D_SCAN_STEP("row_shr:2 row_mask:0xf")
                 SS2D_SCAN_STEP("row_shr:4 row_mask:0xf")
                 SS2D_SCAN_STEP("row_shr:8 row_mask:0xf")
                 SS2D_SCAN_STEP("row_bcast:15 row_mask:0xa")
                 SS2D_SCAN_STEP("row_bcast:31 row_mask:0xc")
                 "s_nop 0\n\t"
                 "v_mov_b32_dpp %2, %0 wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
                 "v_mov_b32_dpp %3, %1 wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1"
                 : "+v"(a), "+v"(h), "+v"(ax), "+v"(hx));
#undef SS2D_SCAN_STEP
    a_ex = ax;
    h_ex = hx;
    a_tot = read_lane(a, kWave - 1);
    h_tot = read_lane(h, kWave - 1);
}

// The same scan for two recurrences that share their multipliers: (a, h) and (a, g).  Per step one more fused
// multiply-add; the exclusive prefixes and totals of both come back.
__device__ __forceinline__ void wave_scan_pairs2(float a, float h, float g, float &a_ex, float &h_ex, float &g_ex, float &a_tot,
                                                 float &h_tot, float &g_tot) {
    float ax = 1.0f, hx = 0.0f, gx = 0.0f;
#define SS2D_SCAN_STEP2(CTRL)                                  \
    "v_fmac_f32_dpp %1, %1, %0 " CTRL " bank_mask:0xf\n\t" \
    "v_fmac_f32_dpp %2, %2, %0 " CTRL " bank_mask:0xf\n\t" \
    "v_mul_f32_dpp %0, %0, %0 " CTRL " bank_mask:0xf\n\t"  \
    "s_nop 0\n\t"
    asm("s_nop 1\n\t"
                 SS2D_SCAN_STEP2("row_shr:1 row_mask:0xf")
                 SS2D_SCAN_STEP2("row_shr:2 row_mask:0xf")
                 SS2D_SCAN_STEP2("row_shr:4 row_mask:0xf")
                 SS2D_SCAN_STEP2("row_shr:8 row_mask:0xf")
                 SS2D_SCAN_STEP2("row_bcast:15 row_mask:0xa")
                 SS2D_SCAN_STEP2("row_bcast:31 row_mask:0xc")
                 "s_nop 0\n\t"
                 "v_mov_b32_dpp %3, %0 wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
                 "v_mov_b32_dpp %4, %1 wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
                 "v_mov_b32_dpp %5, %2 wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1"
                 : "+v"(a), "+v"(h), "+v"(g), "+v"(ax), "+v"(hx), "+v"(gx));
#undef SS2D_SCAN_STEP2
    a_ex = ax;
    h_ex = hx;
    g_ex = gx;
    a_tot = read_lane(a, kWave - 1);
    h_tot = read_lane(h, kWave - 1);
    g_tot = read_lane(g, kWave - 1);
}

// One state of one pass: lane-local scan of its 8 items, wave scan of the lane totals, then
// the state entering the lane (from `carry`, the state entering the pass) is pushed through
// the items and C*h is accumulated into y.  Returns the pass totals.
__device__ __forceinline__ void scan_state_pass(const float (&dl)[kItems], const float (&du)[kItems],
                                                const float (&Bv)[kItems], const float (&Cv)[kItems], float A_log2e,
                                                float carry, float (&y)[kItems], float &a_tot, float &h_tot) {
    float ac[kItems], hh[kItems];
#pragma unroll
    for (int i = 0; i < kItems; ++i) {
        const float a = __builtin_amdgcn_exp2f(dl[i] * A_log2e);
        const float b = Bv[i] * du[i];
        ac[i] = i == 0 ? a : ac[i - 1] * a;
        hh[i] = i == 0 ? b : fmaf(a, hh[i - 1], b);
    }
    float a_ex, h_ex;
    wave_scan_pairs(ac[kItems - 1], hh[kItems - 1], a_ex, h_ex, a_tot, h_tot);
    const float s_in = fmaf(a_ex, carry, h_ex);
#pragma unroll
    for (int i = 0; i < kItems; ++i) y[i] = fmaf(Cv[i], fmaf(ac[i], s_in, hh[i]), y[i]);
}

// The fill the delta loads use past the end of a row (see delta_transform).
template <bool kSoftplus> __device__ __forceinline__ constexpr float delta_fill() {
    return kSoftplus ? -__builtin_inff() : 0.0f;
}

// Widen u and delta, apply bias/softplus, and start the output with the D*u skip term.  `n_valid` is how many
// of the 8 items lie inside the row.
template <typename in_t, bool kSoftplus>
__device__ __forceinline__ void prepare_delta_u(const Raw8<in_t> &u_raw, const Raw8<in_t> &dl_raw, int n_valid,
                                                float bias, float Dv, float (&dl)[kItems], float (&du)[kItems],
                                                float (&y)[kItems]) {
    float uv[kItems], raw[kItems], bias_items[kItems];
    unpack_raw<in_t>(u_raw, uv);
    unpack_raw<in_t>(dl_raw, raw);
#pragma unroll
    for (int i = 0; i < kItems; ++i) bias_items[i] = bias;
    delta_transform<kSoftplus>(raw, bias_items, dl);
#pragma unroll
    for (int i = 0; i < kItems; ++i) {
        if constexpr (!kSoftplus) dl[i] = (i < n_valid) ? dl[i] : 0.0f;   // identity pair past the end of the row
        du[i] = dl[i] * uv[i];                                            // u is 0 past the end
        y[i] = Dv * uv[i];
    }
}

template <typename in_t, bool kVec, bool kSoftplus>
__device__ __forceinline__ void load_delta_u(const in_t *u_row, const in_t *dl_row, int pos, int L, float bias,
                                             float Dv, float (&dl)[kItems], float (&du)[kItems], float (&y)[kItems]) {
    const Raw8<in_t> u_raw = load_raw<in_t, kVec>(u_row, pos, L);
    const Raw8<in_t> dl_raw = load_raw<in_t, kVec>(dl_row, pos, L, delta_fill<kSoftplus>());
    prepare_delta_u<in_t, kSoftplus>(u_raw, dl_raw, L - pos, bias, Dv, dl, du, y);
}

// kGran consecutive elements through a buffer descriptor (32-bit offsets, hardware range check), as loaded:
// kGran * sizeof(T) bytes in 32-bit words (a lone 16-bit element sits in the low half of its word).
template <typename T, int kGran> constexpr int gather_words() { return kGran * (int)sizeof(T) >= 4 ? kGran * (int)sizeof(T) / 4 : 1; }

template <typename T, int kGran>
__device__ __forceinline__ void gather_group_raw(__amdgpu_buffer_rsrc_t rsrc, uint32_t elem_offset, uint32_t uniform_elem_offset,
                                                 uint32_t (&w)[gather_words<T, kGran>()]) {
    // elem_offset: per lane; uniform_elem_offset: the same for the whole wavefront (rides in a scalar register)
    const int byte_off = (int)(elem_offset * (uint32_t)sizeof(T));
    const int soff = (int)(uniform_elem_offset * (uint32_t)sizeof(T));
    constexpr int kBytes = kGran * (int)sizeof(T);
    if constexpr (kBytes == 2) {
        w[0] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc, byte_off, soff, 0);
    } else if constexpr (kBytes == 4) {
        w[0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_off, soff, 0);
    } else if constexpr (kBytes == 8) {
        const auto t = __builtin_amdgcn_raw_buffer_load_b64(rsrc, byte_off, soff, 0);
        w[0] = t[0]; w[1] = t[1];
    } else if constexpr (kBytes == 16) {
        const auto t = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_off, soff, 0);
        w[0] = t[0]; w[1] = t[1]; w[2] = t[2]; w[3] = t[3];
    } else {
        static_assert(kBytes == 32, "8 fp32 elements");
        const auto t0 = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_off, soff, 0);
        const auto t1 = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_off + 16, soff, 0);
        w[0] = t0[0]; w[1] = t0[1]; w[2] = t0[2]; w[3] = t0[3]; w[4] = t1[0]; w[5] = t1[1]; w[6] = t1[2]; w[7] = t1[3];
    }
}

template <typename T, int kGran>
__device__ __forceinline__ void unpack_group(const uint32_t (&w)[gather_words<T, kGran>()], float (&v)[kGran]) {
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int i = 0; i < kGran; ++i) v[i] = to_f32(T{(uint16_t)(w[i / 2] >> (16 * (i % 2)))});
    } else {
#pragma unroll
        for (int i = 0; i < kGran; ++i) v[i] = bits_to_f32(w[i]);
    }
}

template <typename T, int kGran>
__device__ __forceinline__ void gather_group(__amdgpu_buffer_rsrc_t rsrc, uint32_t elem_offset, uint32_t uniform_elem_offset,
                                             float (&v)[kGran]) {
    uint32_t w[gather_words<T, kGran>()];
    gather_group_raw<T, kGran>(rsrc, elem_offset, uniform_elem_offset, w);
    unpack_group<T, kGran>(w, v);
}

// ---- short rows: one segment of a row per lane (ss2d_core_small.hip, scan_small.hip) --------------------------------
// Inclusive scan of (a, h) pairs over the 16-lane DPP row, in lane order or in reverse lane order; returns the
// EXCLUSIVE h (the state entering this lane; 0 for the first lane of the row).  Lanes without a source keep their value.
// a_incl (optional) receives the inclusive product of a up to this lane.
template <bool kReverse>
__device__ __forceinline__ float row_scan_state_in(float a, float h, float *a_incl = nullptr) {
    float hx = 0.0f;
#define SS2D_ROW_STEP(CTRL)                                         \
    "v_fmac_f32_dpp %1, %1, %0 " CTRL " row_mask:0xf bank_mask:0xf\n\t" \
    "v_mul_f32_dpp %0, %0, %0 " CTRL " row_mask:0xf bank_mask:0xf\n\t"  \
    "s_nop 0\n\t"
    if constexpr (!kReverse) {
        asm("s_nop 1\n\t" SS2D_ROW_STEP("row_shr:1") SS2D_ROW_STEP("row_shr:2") SS2D_ROW_STEP("row_shr:4") SS2D_ROW_STEP("row_shr:8")
            "s_nop 0\n\t"
            "v_mov_b32_dpp %2, %1 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 0"
            : "+v"(a), "+v"(h), "+v"(hx));
    } else {
        asm("s_nop 1\n\t" SS2D_ROW_STEP("row_shl:1") SS2D_ROW_STEP("row_shl:2") SS2D_ROW_STEP("row_shl:4") SS2D_ROW_STEP("row_shl:8")
            "s_nop 0\n\t"
            "v_mov_b32_dpp %2, %1 row_shl:1 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 0"
            : "+v"(a), "+v"(h), "+v"(hx));
    }
#undef SS2D_ROW_STEP
    if (a_incl) *a_incl = a;
    return hx;
}

// kS consecutive 16-bit elements of an LDS tile, packed two to a register as they sit there; item() widens element j.
// Even kS: the run starts at an even element offset (4-byte reads).  Odd kS: it may start anywhere -- the dwords that
// cover it are read and funnel-shifted into place (one more LDS element than the run is touched when it starts at an
// even offset: tiles keep a few elements of slack behind them).
template <typename in_t, int kS> struct Run {
    static constexpr int kWords = (kS + 1) / 2;
    uint32_t w[kWords];
    __device__ __forceinline__ void read(const uint16_t *tile, int elem_off) {
        if constexpr (kS % 2 == 0) {
            const uint32_t *src = reinterpret_cast<const uint32_t *>(tile + elem_off);
#pragma unroll
            for (int k = 0; k < kWords; ++k) w[k] = src[k];
        } else {
            const uint32_t *src = reinterpret_cast<const uint32_t *>(tile + (elem_off & ~1));
            const uint32_t shift = (uint32_t)(elem_off & 1) * 16u;
            uint32_t r[kWords];
#pragma unroll
            for (int k = 0; k < kWords; ++k) r[k] = src[k];
#pragma unroll
            for (int k = 0; k + 1 < kWords; ++k) w[k] = __builtin_amdgcn_alignbit(r[k + 1], r[k], shift);
            w[kWords - 1] = r[kWords - 1] >> shift;
        }
    }
    // Odd kS, global memory: the kS elements that follow the first `skip` (0 or 1) of the kS + 1 elements at src.
    // src may sit on any 2-byte boundary; every element read lies in [src, src + kS + 1).
    __device__ __forceinline__ void read_from(const uint16_t *src, int skip) {
        static_assert(kS % 2 != 0, "even runs are read in place");
        uint32_t r[kWords];
#pragma unroll
        for (int k = 0; k < kWords; ++k) __builtin_memcpy(&r[k], src + 2 * k, 4);
        const uint32_t shift = (uint32_t)skip * 16u;
#pragma unroll
        for (int k = 0; k + 1 < kWords; ++k) w[k] = __builtin_amdgcn_alignbit(r[k + 1], r[k], shift);
        w[kWords - 1] = r[kWords - 1] >> shift;
    }
    __device__ __forceinline__ void pack(const uint16_t (&e)[kS]) {
#pragma unroll
        for (int k = 0; k < kS / 2; ++k) w[k] = (uint32_t)e[2 * k] | ((uint32_t)e[2 * k + 1] << 16);
        if constexpr (kS % 2 != 0) w[kWords - 1] = e[kS - 1];
    }
    __device__ __forceinline__ float item(int j) const {
        return (j & 1) ? unpack_hi<in_t>(w[j / 2]) : unpack_lo<in_t>(w[j / 2]);
    }
};
constexpr int kRunSlack = 8;     // 16-bit elements kept free behind an LDS array whose last run may be read one element long

}  // namespace ss2d
