// LayerNorm over the channel axis for the two layouts the SS2D block meets it in.
//
//   ss2d_layer_norm        rows of C contiguous channels ((B,H,W,C) activations, nn.LayerNorm)
//   ss2d_layer_norm_cf     channel-FIRST input (B,C,L) -- the merged scan output -- normalised over C
//                          and written either channel-last (B,L,C) or channel-first (B,C,L)
//                          (LayerNorm2d = permute, layer_norm, permute; vmamba.py:52-57 and the
//                          out_norm step of forward_core, vmamba.py:641-646)
//
// y = (x - mean) * rsqrt(var + eps) * weight + bias with mean/var (biased) over the C channels,
// statistics and arithmetic in fp32 whatever the I/O types, as torch.nn.functional.layer_norm does.
// Pure HBM streaming: one read, one write.  C is small here (48..768), so a whole row lives in the
// registers of a few lanes: a power-of-two group of lanes shares a row, each lane holding 8
// consecutive channels per 16-byte (16-bit types) or 2x16-byte (fp32) load; the two reductions are
// butterfly shuffles inside the group.  Variance is computed from centred values (second pass in
// registers), not from E[x^2] - mean^2.
#include "ss2d_common.h"

namespace ss2d {

constexpr int kLnItems = 8;       // channels per lane per chunk
constexpr int kLnMaxChunks = 2;   // chunks per lane: rows up to 64 lanes * 8 * 2 = 1024 channels

template <typename T> __device__ __forceinline__ void ln_load8(const T *p, float (&v)[kLnItems]) {
    if constexpr (sizeof(T) == 2) {
        const uint4 raw = *reinterpret_cast<const uint4 *>(p);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = to_f32(T{(uint16_t)(w[i] & 0xffffu)});
            v[2 * i + 1] = to_f32(T{(uint16_t)(w[i] >> 16)});
        }
    } else {
        const float4 lo = *reinterpret_cast<const float4 *>(p), hi = *reinterpret_cast<const float4 *>(p + 4);
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    }
}
template <typename T> __device__ __forceinline__ void ln_store8(T *p, const float (&v)[kLnItems]) {
    if constexpr (sizeof(T) == 2) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = pack2_from_f32<T>(v[2 * i], v[2 * i + 1]);   // one conversion per pair
        *reinterpret_cast<uint4 *>(p) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
}

// Eight elements as loaded (one 16-byte piece for 16-bit types, two for fp32), widened when they are used.
template <typename T> struct LnRaw { uint4 a, b; };
template <typename T> __device__ __forceinline__ LnRaw<T> ln_load_raw(const T *p) {
    LnRaw<T> r;
    r.a = *reinterpret_cast<const uint4 *>(p);
    if constexpr (sizeof(T) == 4) r.b = *reinterpret_cast<const uint4 *>(p + 4);
    else r.b = r.a;
    return r;
}
template <typename T> __device__ __forceinline__ void ln_widen(const LnRaw<T> &r, float (&v)[kLnItems]) {
    if constexpr (sizeof(T) == 2) {
        const uint32_t w[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = to_f32(T{(uint16_t)(w[i] & 0xffffu)});
            v[2 * i + 1] = to_f32(T{(uint16_t)(w[i] >> 16)});
        }
    } else {
        v[0] = bits_to_f32(r.a.x); v[1] = bits_to_f32(r.a.y); v[2] = bits_to_f32(r.a.z); v[3] = bits_to_f32(r.a.w);
        v[4] = bits_to_f32(r.b.x); v[5] = bits_to_f32(r.b.y); v[6] = bits_to_f32(r.b.z); v[7] = bits_to_f32(r.b.w);
    }
}

// v[i] = (v[i] + r[i]) rounded to T and widened again -- what a separate add in the tensor's type would leave
template <typename T> __device__ __forceinline__ void ln_add_rounded(float (&v)[kLnItems], const float (&r)[kLnItems]) {
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int i = 0; i < kLnItems; i += 2) {
            const uint32_t two = pack2_from_f32<T>(v[i] + r[i], v[i + 1] + r[i + 1]);
            v[i] = unpack_lo<T>(two);
            v[i + 1] = unpack_hi<T>(two);
        }
    } else {
#pragma unroll
        for (int i = 0; i < kLnItems; ++i) v[i] = v[i] + r[i];
    }
}

// Sum over a power-of-two group of lanes, the same value in every lane of the group.  Inside a row of 16 lanes the
// partners come through the DPP operand of the add itself (lane ^ 1 and lane ^ 2 as quad permutations, then the mirror
// images inside 8 and 16 lanes: a quad meets the other quad of its half, a half the other half) -- no LDS round trip;
// wider groups finish with lane exchanges.
template <int kGroup> __device__ __forceinline__ float group_sum(float v) {
    if constexpr (kGroup >= 2) v += dpp_move<0xB1>(v, v);      // quad_perm [1,0,3,2]
    if constexpr (kGroup >= 4) v += dpp_move<0x4E>(v, v);      // quad_perm [2,3,0,1]
    if constexpr (kGroup >= 8) v += dpp_move<0x141>(v, v);     // row_half_mirror
    if constexpr (kGroup >= 16) v += dpp_move<0x140>(v, v);    // row_mirror
#pragma unroll
    for (int off = 16; off < kGroup; off <<= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// ---- rows of contiguous channels --------------------------------------------------------------
// kGroup lanes per row, kChunks 8-channel chunks per lane (chunk j of lane g covers channels
// (j*kGroup + g)*8 ..+8).  Requires C % 8 == 0 and 16-byte aligned rows (host-checked).
template <typename in_t, typename w_t, typename out_t, int kGroup, int kChunks>
__global__ __launch_bounds__(kBlock) void layer_norm_rows_kernel(const in_t *__restrict__ x, const w_t *__restrict__ weight,
                                                                 const w_t *__restrict__ bias, out_t *__restrict__ y,
                                                                 int64_t rows, int C, float eps,
                                                                 const in_t *__restrict__ residual = nullptr,
                                                                 in_t *__restrict__ sum_out = nullptr,
                                                                 const w_t *__restrict__ pre_bias = nullptr) {
    constexpr int kRowsPerBlock = kBlock / kGroup;
    const int g = threadIdx.x % kGroup;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kGroup;
    const bool row_ok = row < rows;
    const int64_t row_c = row_ok ? row : rows - 1;   // lanes without a row or a chunk load real memory and drop it
    // Everything the row needs is requested before anything is used (raw 16-byte pieces, widened later): one memory
    // latency per workgroup instead of one per chunk and operand.
    LnRaw<in_t> x_raw[kChunks], r_raw[kChunks];
    LnRaw<w_t> pb_raw[kChunks], w_raw[kChunks], b_raw[kChunks];
    bool have[kChunks];
    int c0c[kChunks];
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
        const int c0 = (j * kGroup + g) * kLnItems;
        have[j] = row_ok && c0 < C;
        c0c[j] = c0 < C ? c0 : C - kLnItems;
        x_raw[j] = ln_load_raw<in_t>(x + row_c * C + c0c[j]);
    }
    if (residual) {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) r_raw[j] = ln_load_raw<in_t>(residual + row_c * C + c0c[j]);
    }
    if (pre_bias) {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) pb_raw[j] = ln_load_raw<w_t>(pre_bias + c0c[j]);
    }
    if (weight) {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) w_raw[j] = ln_load_raw<w_t>(weight + c0c[j]);
    }
    if (bias) {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) b_raw[j] = ln_load_raw<w_t>(bias + c0c[j]);
    }

    float v[kChunks][kLnItems];
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
        ln_widen<in_t>(x_raw[j], v[j]);
        if (residual) {
            // the row is x + residual, rounded to the tensor type as the separate add would leave it
            float r[kLnItems];
            ln_widen<in_t>(r_raw[j], r);
            ln_add_rounded<in_t>(v[j], r);
            if (have[j]) ln_store8<in_t>(sum_out + row * C + c0c[j], v[j]);
        }
        if (pre_bias) {
            // the row is x + pre_bias (one value per channel), rounded as the separate add would leave it
            float pb[kLnItems];
            ln_widen<w_t>(pb_raw[j], pb);
            ln_add_rounded<in_t>(v[j], pb);
        }
#pragma unroll
        for (int i = 0; i < kLnItems; ++i) { v[j][i] = have[j] ? v[j][i] : 0.0f; s += v[j][i]; }
    }
    const float inv_c = 1.0f / (float)C;
    const float mean = group_sum<kGroup>(s) * inv_c;
    float q = 0.0f;
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
#pragma unroll
        for (int i = 0; i < kLnItems; ++i) {
            const float d = v[j][i] - mean;
            q = have[j] ? fmaf(d, d, q) : q;
        }
    }
    const float rstd = rsqrtf(group_sum<kGroup>(q) * inv_c + eps);
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
        float wv[kLnItems], bv[kLnItems], o[kLnItems];
        if (weight) ln_widen<w_t>(w_raw[j], wv);
        if (bias) ln_widen<w_t>(b_raw[j], bv);
#pragma unroll
        for (int i = 0; i < kLnItems; ++i) {
            float t = (v[j][i] - mean) * rstd;
            if (weight) t *= wv[i];
            if (bias) t += bv[i];
            o[i] = t;
        }
        if (have[j]) ln_store8<out_t>(y + row * C + c0c[j], o);
    }
}

// Any C, any alignment: one wavefront per row, channels strided over the lanes, three passes over the row
// (the second and third hit L1/L2).
template <typename in_t, typename w_t, typename out_t>
__global__ __launch_bounds__(kBlock) void layer_norm_rows_generic_kernel(const in_t *__restrict__ x,
                                                                         const w_t *__restrict__ weight,
                                                                         const w_t *__restrict__ bias, out_t *__restrict__ y,
                                                                         int64_t rows, int C, float eps) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (row >= rows) return;
    const in_t *xr = x + row * C;
    float s = 0.0f;
    for (int c = lane; c < C; c += kWave) s += to_f32(xr[c]);
    const float mean = group_sum<kWave>(s) / (float)C;
    float q = 0.0f;
    for (int c = lane; c < C; c += kWave) { const float d = to_f32(xr[c]) - mean; q = fmaf(d, d, q); }
    const float rstd = rsqrtf(group_sum<kWave>(q) / (float)C + eps);
    for (int c = lane; c < C; c += kWave) {
        float t = (to_f32(xr[c]) - mean) * rstd;
        if (weight) t *= to_f32(weight[c]);
        if (bias) t += to_f32(bias[c]);
        y[row * C + c] = from_f32<out_t>(t);
    }
}

// ---- channel-first input ------------------------------------------------------------------------
// LDS-tile variant (rows wider than the register variant below covers).
// x (B,C,L).  A workgroup takes kCfTile consecutive positions of one image and all C channels: the tile is read
// lane-contiguously along L (each channel row gives a kCfTile-element segment), parked in LDS as fp32
// [C][kCfTile+1], reduced per position (a group of 256/kCfTile lanes walks the channels of one position; the odd
// pitch keeps those column reads conflict-free), normalised in LDS, and written out lane-contiguously in the
// requested layout: channel-last (B,L,C) rows, or channel-first (B,C,L) segments.
template <typename in_t, typename w_t, typename out_t, bool kOutChannelLast, int kCfTile>
__global__ __launch_bounds__(kBlock) void layer_norm_cf_kernel(const in_t *__restrict__ x, const w_t *__restrict__ weight,
                                                               const w_t *__restrict__ bias, out_t *__restrict__ y,
                                                               int C, int L, int tiles_per_image, float eps) {
    constexpr int kCfPitch = kCfTile + 1;
    extern __shared__ __align__(16) float tile[];          // [C][kCfPitch]
    __shared__ float s_mean[kCfTile], s_rstd[kCfTile];
    const uint32_t b = blockIdx.x / tiles_per_image;
    const int l0 = (int)(blockIdx.x - b * tiles_per_image) * kCfTile;
    const int nl = min(kCfTile, L - l0);
    const in_t *xb = x + (size_t)b * C * L;

    // load: thread -> (channel c = idx / kCfTile, position p = idx % kCfTile)
    for (int idx = threadIdx.x; idx < C * kCfTile; idx += kBlock) {
        const int c = idx / kCfTile, p = idx % kCfTile;
        tile[c * kCfPitch + p] = p < nl ? to_f32(xb[(size_t)c * L + l0 + p]) : 0.0f;
    }
    __syncthreads();
    // statistics: kBlock / kCfTile = 8 lanes per position
    constexpr int kLanesPerPos = kBlock / kCfTile;
    {
        const int p = threadIdx.x / kLanesPerPos, g = threadIdx.x % kLanesPerPos;
        float s = 0.0f;
        for (int c = g; c < C; c += kLanesPerPos) s += tile[c * kCfPitch + p];
        const float mean = group_sum<kLanesPerPos>(s) / (float)C;
        float q = 0.0f;
        for (int c = g; c < C; c += kLanesPerPos) { const float d = tile[c * kCfPitch + p] - mean; q = fmaf(d, d, q); }
        const float rstd = rsqrtf(group_sum<kLanesPerPos>(q) / (float)C + eps);
        if (g == 0) { s_mean[p] = mean; s_rstd[p] = rstd; }
    }
    __syncthreads();
    if constexpr (kOutChannelLast) {
        // y (B,L,C): the tile is nl*C contiguous outputs; thread -> (p = idx / C, c = idx % C)
        out_t *yb = y + ((size_t)b * L + l0) * C;
        for (int idx = threadIdx.x; idx < nl * C; idx += kBlock) {
            const int p = idx / C, c = idx - p * C;
            float t = (tile[c * kCfPitch + p] - s_mean[p]) * s_rstd[p];
            if (weight) t *= to_f32(weight[c]);
            if (bias) t += to_f32(bias[c]);
            yb[idx] = from_f32<out_t>(t);
        }
    } else {
        out_t *yb = y + (size_t)b * C * L;
        for (int idx = threadIdx.x; idx < C * kCfTile; idx += kBlock) {
            const int c = idx / kCfTile, p = idx % kCfTile;
            if (p >= nl) continue;
            float t = (tile[c * kCfPitch + p] - s_mean[p]) * s_rstd[p];
            if (weight) t *= to_f32(weight[c]);
            if (bias) t += to_f32(bias[c]);
            yb[(size_t)c * L + l0 + p] = from_f32<out_t>(t);
        }
    }
}

// Register variant of the channel-first LayerNorm (C up to kG*kVPT channels).  Threads are laid out positions x
// groups: lane -> position (so every channel row is read as one contiguous run of kTP elements), group g holds
// channels g, g+kG, g+2kG, ... of its position in registers.  The two reductions cross the kG groups through a
// few floats of LDS.  Channel-first output goes straight back from registers (contiguous along positions);
// channel-last output is turned round through an LDS tile [position][channel] and copied out row by row.
template <typename in_t, typename w_t, typename out_t, bool kOutChannelLast, int kTP, int kG, int kVPT>
__global__ __launch_bounds__(kBlock) void layer_norm_cf_reg_kernel(const in_t *__restrict__ x, const w_t *__restrict__ weight,
                                                                   const w_t *__restrict__ bias, out_t *__restrict__ y, int C,
                                                                   int L, int tiles_per_image, int Cp, float eps) {
    static_assert(kTP * kG == kBlock, "one thread per (position, group)");
    extern __shared__ __align__(16) unsigned char ln_smem[];
    __shared__ float red[2][kG][kTP];
    const uint32_t b = blockIdx.x / tiles_per_image;
    const int l0 = (int)(blockIdx.x - b * tiles_per_image) * kTP;
    const int p = threadIdx.x % kTP, g = threadIdx.x / kTP;
    const int l = l0 + p;
    const bool valid = l < L;
    // The image sits behind a buffer descriptor and elements outside it (position past L, channel past C) are
    // pointed beyond its end, where the hardware returns 0: every load is unconditional, so the kVPT loads of a lane
    // are all in flight together (a select on the loaded value makes the compiler branch around each load and
    // wait for it).  Host-checked: C * L * sizeof(in_t) < 2 GiB.
    const in_t *xb = x + (size_t)b * C * L;
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<in_t *>(xb), 0, C * L * (int)sizeof(in_t), 0x00020000);

    float v[kVPT];
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
        const int c = g + i * kG;
        const uint32_t off = (valid && c < C) ? (uint32_t)(c * L + l) * (uint32_t)sizeof(in_t) : 0x7ffffff0u;
        if constexpr (sizeof(in_t) == 4) {
            v[i] = bits_to_f32((uint32_t)__builtin_amdgcn_raw_buffer_load_b32(x_rsrc, (int)off, 0, 0));
        } else {
            v[i] = to_f32(in_t{(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(x_rsrc, (int)off, 0, 0)});
        }
        s += v[i];
    }
    red[0][g][p] = s;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int j = 0; j < kG; ++j) tot += red[0][j][p];
    const float mean = tot / (float)C;
    float q = 0.0f;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
        const float d = v[i] - mean;
        q = (g + i * kG < C) ? fmaf(d, d, q) : q;
    }
    red[1][g][p] = q;
    __syncthreads();
    float qt = 0.0f;
#pragma unroll
    for (int j = 0; j < kG; ++j) qt += red[1][j][p];
    const float rstd = rsqrtf(qt / (float)C + eps);

    if constexpr (!kOutChannelLast) {
        out_t *yb = y + (size_t)b * C * L + l;
#pragma unroll
        for (int i = 0; i < kVPT; ++i) {
            const int c = g + i * kG;
            if (valid && c < C) {
                float t = (v[i] - mean) * rstd;
                if (weight) t *= to_f32(weight[c]);
                if (bias) t += to_f32(bias[c]);
                yb[(size_t)c * L] = from_f32<out_t>(t);
            }
        }
    } else {
        out_t *ot = reinterpret_cast<out_t *>(ln_smem);          // [kTP][Cp]
#pragma unroll
        for (int i = 0; i < kVPT; ++i) {
            const int c = g + i * kG;
            if (c < C) {
                float t = (v[i] - mean) * rstd;
                if (weight) t *= to_f32(weight[c]);
                if (bias) t += to_f32(bias[c]);
                ot[p * Cp + c] = from_f32<out_t>(t);
            }
        }
        __syncthreads();
        const int nl = min(kTP, L - l0);
        out_t *yb = y + ((size_t)b * L + l0) * C;
        if (sizeof(out_t) == 2 && (C % 2) == 0) {
            const int half = C / 2;                                // 4-byte units per row
            for (int idx = threadIdx.x; idx < nl * half; idx += kBlock) {
                const int pp = idx / half, cc = (idx - pp * half) * 2;
                *reinterpret_cast<uint32_t *>(yb + (size_t)pp * C + cc) = *reinterpret_cast<const uint32_t *>(ot + pp * Cp + cc);
            }
        } else {
            for (int idx = threadIdx.x; idx < nl * C; idx += kBlock) {
                const int pp = idx / C, cc = idx - pp * C;
                yb[(size_t)pp * C + cc] = ot[pp * Cp + cc];
            }
        }
    }
}

// Quad variant of the register kernel for channel-first input (fp32: the merged scan output feeding out_norm; 16-bit:
// LayerNorm2d on activations): a lane owns FOUR consecutive positions, so every load is 16 bytes (8 of 16-bit input;
// the address pipeline is priced per instruction, and the
// 4-byte loads of the variant above leave it the bottleneck on short images).  Threads are laid out quads x groups;
// group g holds channels g, g+kG, ... of its four positions.  Sums cross the groups of a wavefront by lane
// exchanges and the wavefronts through a few floats of LDS.
template <typename in_t, typename w_t, typename out_t, bool kOutChannelLast, int kQ, int kG, int kCPL>
__global__ __launch_bounds__(kBlock) void layer_norm_cf_quad_kernel(const in_t *__restrict__ x, const w_t *__restrict__ weight,
                                                                    const w_t *__restrict__ bias, out_t *__restrict__ y, int C,
                                                                    int L, int tiles_per_image, int Cp, float eps) {
    static_assert(kQ * kG == kBlock && kQ <= kWave, "one thread per (position quad, group)");
    constexpr int kTP = 4 * kQ;                      // positions per workgroup
    constexpr int kWaves = kBlock / kWave;
    extern __shared__ __align__(16) unsigned char lnq_smem[];
    __shared__ float red[2][kWaves][kTP];
    const uint32_t b = blockIdx.x / tiles_per_image;
    const int l0 = (int)(blockIdx.x - b * tiles_per_image) * kTP;
    const int q = threadIdx.x % kQ, g = threadIdx.x / kQ;
    const int wave = threadIdx.x / kWave;
    const int l = l0 + 4 * q;
    const bool valid = l < L;                        // L % 4 == 0 (host-checked): a quad is inside or outside
    const in_t *xb = x + (size_t)b * C * L;
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<in_t *>(xb), 0, C * L * (int)sizeof(in_t), 0x00020000);

    float v[kCPL][4];
    float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < kCPL; ++i) {
        const int c = g + i * kG;
        // outside the image: pointed past the end of the buffer, where the hardware returns 0 (loads stay unconditional)
        const uint32_t off = (valid && c < C) ? (uint32_t)(c * L + l) * (uint32_t)sizeof(in_t) : 0x7ffffff0u;
        if constexpr (sizeof(in_t) == 4) {
            const auto t = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) v[i][j] = bits_to_f32(t[j]);
        } else {
            const auto t = __builtin_amdgcn_raw_buffer_load_b64(x_rsrc, (int)off, 0, 0);
            v[i][0] = unpack_lo<in_t>(t[0]); v[i][1] = unpack_hi<in_t>(t[0]);
            v[i][2] = unpack_lo<in_t>(t[1]); v[i][3] = unpack_hi<in_t>(t[1]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) s[j] += v[i][j];
    }
    auto reduce_groups = [&](float (&acc)[4], int which) {
#pragma unroll
        for (int m = kQ; m < kWave; m *= 2)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] += __shfl_xor(acc[j], m, kWave);
        if ((threadIdx.x & (kWave - 1)) < kQ) {
#pragma unroll
            for (int j = 0; j < 4; ++j) red[which][wave][4 * q + j] = acc[j];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float t = 0.0f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) t += red[which][w][4 * q + j];
            acc[j] = t;
        }
    };
    reduce_groups(s, 0);
    float mean[4], qq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 4; ++j) mean[j] = s[j] / (float)C;
#pragma unroll
    for (int i = 0; i < kCPL; ++i) {
        const bool live = g + i * kG < C;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float d = v[i][j] - mean[j];
            qq[j] = live ? fmaf(d, d, qq[j]) : qq[j];
        }
    }
    reduce_groups(qq, 1);
    float rstd[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) rstd[j] = rsqrtf(qq[j] / (float)C + eps);

    if constexpr (!kOutChannelLast) {
        out_t *yb = y + (size_t)b * C * L + l;
#pragma unroll
        for (int i = 0; i < kCPL; ++i) {
            const int c = g + i * kG;
            if (valid && c < C) {
                const float wv = weight ? to_f32(weight[c]) : 1.0f, bv = bias ? to_f32(bias[c]) : 0.0f;
                float o[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = fmaf((v[i][j] - mean[j]) * rstd[j], wv, bv);
                out_t *dst = yb + (size_t)c * L;
                if constexpr (sizeof(out_t) == 4) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(o[0], o[1], o[2], o[3]);
                } else {
                    *reinterpret_cast<uint2 *>(dst) = make_uint2(pack2_from_f32<out_t>(o[0], o[1]), pack2_from_f32<out_t>(o[2], o[3]));
                }
            }
        }
    } else {
        out_t *ot = reinterpret_cast<out_t *>(lnq_smem);          // [kTP][Cp]
#pragma unroll
        for (int i = 0; i < kCPL; ++i) {
            const int c = g + i * kG;
            if (c < C) {
                const float wv = weight ? to_f32(weight[c]) : 1.0f, bv = bias ? to_f32(bias[c]) : 0.0f;
                float o[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = fmaf((v[i][j] - mean[j]) * rstd[j], wv, bv);
                if constexpr (sizeof(out_t) == 4) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) ot[(4 * q + j) * Cp + c] = o[j];
                } else {                                           // one conversion per pair of positions
                    uint16_t *ot16 = reinterpret_cast<uint16_t *>(ot);
#pragma unroll
                    for (int j = 0; j < 4; j += 2) {
                        const uint32_t two = pack2_from_f32<out_t>(o[j], o[j + 1]);
                        ot16[(4 * q + j) * Cp + c] = (uint16_t)(two & 0xffffu);
                        ot16[(4 * q + j + 1) * Cp + c] = (uint16_t)(two >> 16);
                    }
                }
            }
        }
        __syncthreads();
        const int nl = min(kTP, L - l0);
        out_t *yb = y + ((size_t)b * L + l0) * C;
        constexpr int kPiece = 16 / (int)sizeof(out_t);            // elements per 16-byte piece; C % kPiece == 0 (host)
        const int pieces = C / kPiece;
        for (int idx = threadIdx.x; idx < nl * pieces; idx += kBlock) {
            const int pp = idx / pieces, cc = (idx - pp * pieces) * kPiece;
            *reinterpret_cast<uint4 *>(yb + (size_t)pp * C + cc) = *reinterpret_cast<const uint4 *>(ot + pp * Cp + cc);
        }
    }
}

// Image variant for channel-first input (fp32, or 16-bit with 8-byte vectors) of SHORT images (7 x 7 ... 28 x 28 maps): the tile kernels above cut an
// image into pieces of 16 or 32 positions, i.e. 64- or 128-byte runs per channel row, and on short rows that is what
// they are bound by.  Here a workgroup of up to 1024 threads takes a whole image, or a 1/T share of its positions, and
// reads it as 16-byte vectors of ONE flat stream:
//   * kCh = 1 (L a multiple of 4): a unit is one channel row, Q = L/4 vectors; the workgroup takes Qn consecutive
//     vectors of every row;
//   * kCh = 4 (any other L, C a multiple of 4): a unit is four consecutive channel rows = L vectors that start on a
//     16-byte boundary although the rows do not; element j of vector q is (channel e / L, position e % L), e = 4q+j.
// Thread (q, g) holds vector q of units g*kU .. g*kU+kU-1; which (channel offset, position) its four elements are
// does not depend on the unit, so a lane adds its units up in registers, the partial sums of the groups meet in LDS
// (in a fixed order: results do not depend on timing), and mean and 1/std come back per position.  Variance from
// centred values, as everywhere in this file.  Channel-first output leaves as it came; channel-last output is turned
// round through an LDS tile [position][channel] whose pitch is an odd number of dwords.
constexpr int kLnImgBlock = 1024;
constexpr int kLnImgStat = 256;                      // positions per workgroup at most

template <typename in_t, typename w_t, typename out_t, bool kOutChannelLast, int kCh, int kU>
__global__ __launch_bounds__(kLnImgBlock) void layer_norm_cf_image_kernel(const in_t *__restrict__ x, const w_t *__restrict__ weight,
                                                                          const w_t *__restrict__ bias, out_t *__restrict__ y, int C,
                                                                          int L, int T, int Qn, int G, int pitch_dw, float eps) {
    static_assert(kCh == 1 || kCh == 4, "a unit is one channel row or four");
    static_assert(kU % 2 == 0, "channel pairs share a dword of the output tile");
    extern __shared__ __align__(16) unsigned char lni_smem[];
    float *red = reinterpret_cast<float *>(lni_smem);                          // [thread][4]
    float *stat = red + 4 * kLnImgBlock;                                       // [2][kLnImgStat]
    float *wb = stat + 2 * kLnImgStat;                                         // [2][C] weight, bias
    uint32_t *tile = reinterpret_cast<uint32_t *>(wb + 2 * C);                 // [position][pitch_dw]
    const int Q = kCh * L / 4, n_units = C / kCh;
    const int b = blockIdx.x / T, q0 = ((int)blockIdx.x - b * T) * Qn;
    const int Qt = min(Qn, Q - q0);
    const int t = threadIdx.x, g = t / Qn, q = t - g * Qn;
    const bool lane_on = g < G && q < Qt;
    const int Lt = kCh == 1 ? 4 * Qt : L;                                      // positions of this workgroup
    int lj[4], cc[4];                                                          // element j: position (tile-relative), channel offset
    if constexpr (kCh == 1) {
#pragma unroll
        for (int j = 0; j < 4; ++j) { lj[j] = 4 * q + j; cc[j] = 0; }
    } else {
        const int e0 = min(4 * q, kCh * L - 4);                                // idle lanes: any vector of the unit
        cc[0] = e0 / L; lj[0] = e0 - cc[0] * L;
#pragma unroll
        for (int j = 1; j < 4; ++j) {
            const bool wrap = lj[j - 1] + 1 == L;
            lj[j] = wrap ? 0 : lj[j - 1] + 1;
            cc[j] = wrap ? cc[j - 1] + 1 : cc[j - 1];
        }
    }
    const int n_valid = lane_on ? min(max(n_units - g * kU, 0), kU) : 0;       // units this lane really holds
    const in_t *xb = x + (size_t)b * C * L;
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<in_t *>(xb), 0, C * L * (int)sizeof(in_t), 0x00020000);

    float v[kU][4];
    float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int n = 0; n < kU; ++n) {
        const int unit = g * kU + n;
        // idle lanes and units past the last point past the end of the buffer, where the hardware returns 0
        // (a vector is four positions: 16 bytes of fp32 input, 8 bytes of 16-bit input)
        const uint32_t off = n < n_valid ? (uint32_t)(unit * Q + q0 + q) * (4u * (uint32_t)sizeof(in_t)) : 0x7ffffff0u;
        if constexpr (sizeof(in_t) == 4) {
            const auto r = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) v[n][j] = bits_to_f32(r[j]);
        } else {
            const auto r = __builtin_amdgcn_raw_buffer_load_b64(x_rsrc, (int)off, 0, 0);
            v[n][0] = unpack_lo<in_t>(r[0]); v[n][1] = unpack_hi<in_t>(r[0]);
            v[n][2] = unpack_lo<in_t>(r[1]); v[n][3] = unpack_hi<in_t>(r[1]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) s[j] += v[n][j];
    }
    // weight and bias wait in LDS (read after the barriers of the two reductions)
    for (int c = t; c < C; c += (int)blockDim.x) {
        wb[c] = weight ? to_f32(weight[c]) : 1.0f;
        wb[C + c] = bias ? to_f32(bias[c]) : 0.0f;
    }
    // per-position totals over groups (and, kCh = 4, over the four channel offsets), always in the same order
    auto totals = [&](const float (&acc)[4], int which, auto finish) {
        *reinterpret_cast<float4 *>(red + 4 * t) = make_float4(acc[0], acc[1], acc[2], acc[3]);
        __syncthreads();
        for (int l = t; l < Lt; l += (int)blockDim.x) {      // (a workgroup may have fewer threads than positions)
            float tot = 0.0f;
#pragma unroll 4
            for (int gg = 0; gg < G; ++gg)
#pragma unroll
                for (int c = 0; c < kCh; ++c) tot += red[gg * Qn * 4 + c * L + l];
            stat[which * kLnImgStat + l] = finish(tot);
        }
        __syncthreads();
    };
    const float inv_c = 1.0f / (float)C;
    totals(s, 0, [&](float tot) { return tot * inv_c; });
    float mean[4], qq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 4; ++j) mean[j] = stat[lj[j]];
#pragma unroll
    for (int n = 0; n < kU; ++n) {
        if (n < n_valid) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float d = v[n][j] - mean[j];
                qq[j] = fmaf(d, d, qq[j]);
            }
        }
    }
    totals(qq, 1, [&](float tot) { return rsqrtf(tot * inv_c + eps); });
    float rstd[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) rstd[j] = stat[kLnImgStat + lj[j]];

    // normalised values, in place.  A unit's weight and bias are one value (kCh = 1) or four, of which a lane's
    // four consecutive elements meet at most two neighbours.
    const int cc_lo = cc[0], cc_hi = min(cc[0] + 1, kCh - 1);
#pragma unroll
    for (int n = 0; n < kU; ++n) {
        const int unit = min(g * kU + n, n_units - 1);
        const float w_lo = wb[unit * kCh + cc_lo], b_lo = wb[C + unit * kCh + cc_lo];
        float w_hi = w_lo, b_hi = b_lo;
        if constexpr (kCh > 1) {
            w_hi = wb[unit * kCh + cc_hi];
            b_hi = wb[C + unit * kCh + cc_hi];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float wv = cc[j] == cc_lo ? w_lo : w_hi, bv = cc[j] == cc_lo ? b_lo : b_hi;
            v[n][j] = fmaf((v[n][j] - mean[j]) * rstd[j], wv, bv);
        }
    }

    if constexpr (!kOutChannelLast) {
        out_t *yb = y + (size_t)b * C * L;
#pragma unroll
        for (int n = 0; n < kU; ++n) {
            const int unit = g * kU + n;
            if (n < n_valid) {
                out_t *dst = yb + ((size_t)unit * Q + q0 + q) * 4;
                if constexpr (sizeof(out_t) == 4) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(v[n][0], v[n][1], v[n][2], v[n][3]);
                } else {
                    *reinterpret_cast<uint2 *>(dst) = make_uint2(pack2_from_f32<out_t>(v[n][0], v[n][1]), pack2_from_f32<out_t>(v[n][2], v[n][3]));
                }
            }
        }
    } else {
        // element j of unit n sits at row lj[j], column (g * kU + n) * kCh + cc[j]: per-lane bases, constant steps
        if constexpr (sizeof(out_t) == 4) {
            int base[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) base[j] = lj[j] * pitch_dw + g * kU * kCh + cc[j];
#pragma unroll
            for (int n = 0; n < kU; ++n) {
                if (n < n_valid) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) tile[base[j] + n * kCh] = __builtin_bit_cast(uint32_t, v[n][j]);
                }
            }
        } else if constexpr (kCh == 1) {
            // a lane's channels are consecutive and start on an even one: pairs go out as dwords (C is even,
            // host-checked: a pair is inside or outside)
            int base[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) base[j] = lj[j] * pitch_dw + g * (kU / 2);
#pragma unroll
            for (int n = 0; n < kU; n += 2) {
                if (n < n_valid) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) tile[base[j] + n / 2] = pack2_from_f32<out_t>(v[n][j], v[n + 1][j]);
                }
            }
        } else {
            uint16_t *tile16 = reinterpret_cast<uint16_t *>(tile);
            int base[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) base[j] = lj[j] * pitch_dw * 2 + g * kU * kCh + cc[j];
#pragma unroll
            for (int n = 0; n < kU; n += 2) {
                if (n < n_valid) {                     // the units of a lane come in pairs (C / 4 even: host-checked)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t two = pack2_from_f32<out_t>(v[n][j], v[n + 1][j]);
                        tile16[base[j] + n * kCh] = (uint16_t)(two & 0xffffu);
                        tile16[base[j] + (n + 1) * kCh] = (uint16_t)(two >> 16);
                    }
                }
            }
        }
        __syncthreads();
        // rows of C channels, 16 bytes per lane (C * sizeof(out_t) is a multiple of 16: host-checked)
        const int pieces = C * (int)sizeof(out_t) / 16;
        const int l0 = kCh == 1 ? 4 * q0 : 0;
        uint4 *yb = reinterpret_cast<uint4 *>(y + ((size_t)b * L + l0) * C);
        int r = t / pieces, pc = t - r * pieces;
        const int step_r = (int)blockDim.x / pieces, step_p = (int)blockDim.x - step_r * pieces;
        while (r < Lt) {
            const uint32_t *src = tile + r * pitch_dw + pc * 4;
            yb[(size_t)r * pieces + pc] = make_uint4(src[0], src[1], src[2], src[3]);
            r += step_r; pc += step_p;
            if (pc >= pieces) { pc -= pieces; ++r; }
        }
    }
}

// ---- host side ----------------------------------------------------------------------------------
static bool ln_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename in_t, typename w_t, typename out_t>
static int launch_ln_rows(const void *x, const void *w, const void *b, void *y, int64_t rows, int C, float eps,
                          hipStream_t stream, const void *residual = nullptr, void *sum_out = nullptr,
                          const void *pre_bias = nullptr) {
    const in_t *xp = (const in_t *)x; const w_t *wp = (const w_t *)w; const w_t *bp = (const w_t *)b; out_t *yp = (out_t *)y;
    const in_t *rp = (const in_t *)residual; in_t *sp = (in_t *)sum_out; const w_t *pp = (const w_t *)pre_bias;
    const bool fast = C % kLnItems == 0 && C <= kWave * kLnItems * kLnMaxChunks && ln_aligned16(x) && ln_aligned16(y) &&
                      (!w || ln_aligned16(w)) && (!b || ln_aligned16(b)) && ln_aligned16(residual) && ln_aligned16(sum_out) &&
                      ln_aligned16(pre_bias);
    if (!fast) {
        if (residual || pre_bias) return SS2D_ENOTSUP;          // the fused adds exist for vectorisable rows only
        const int64_t n_wg = (rows + kBlock / kWave - 1) / (kBlock / kWave);
        if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
        hipLaunchKernelGGL((layer_norm_rows_generic_kernel<in_t, w_t, out_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream,
                           xp, wp, bp, yp, rows, C, eps);
        return launch_status();
    }
    const int vecs = C / kLnItems;     // 16-byte (or 2x16-byte) vectors per row
#define SS2D_LN_LAUNCH(GROUP, CHUNKS)                                                                                    \
    {                                                                                                                    \
        const int64_t n_wg = (rows + kBlock / GROUP - 1) / (kBlock / GROUP);                                             \
        if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;                                                                      \
        hipLaunchKernelGGL((layer_norm_rows_kernel<in_t, w_t, out_t, GROUP, CHUNKS>), dim3((uint32_t)n_wg), dim3(kBlock), \
                           0, stream, xp, wp, bp, yp, rows, C, eps, rp, sp, pp);                                         \
    }
    // widths of 3 * 2^k vectors would leave a quarter of a power-of-two group idle: three chunks per lane instead
    // (C = 192: 23.7 -> 18.7 us, with the residual add 33.7 -> 28.1; C = 384: 13.1 -> 12.3 and 19.2 -> 16.6; at C = 96
    // the add variant got slower -- and the layout is chosen by width alone, so that the add variant and the plain one sum
    // in the same order and agree bit for bit -- and C = 768 did not change, so those keep the layouts below)
    if (vecs == 24) SS2D_LN_LAUNCH(8, 3)
    else if (vecs == 48) SS2D_LN_LAUNCH(16, 3)
    else if (vecs <= 4) SS2D_LN_LAUNCH(4, 1)
    else if (vecs <= 8) SS2D_LN_LAUNCH(8, 1)
    else if (vecs <= 16) SS2D_LN_LAUNCH(16, 1)
    else if (vecs <= 32) SS2D_LN_LAUNCH(32, 1)
    else if (vecs <= 64) SS2D_LN_LAUNCH(64, 1)
    else SS2D_LN_LAUNCH(64, 2)
#undef SS2D_LN_LAUNCH
    return launch_status();
}

template <typename in_t, typename w_t, typename out_t, int kCfTile>
static int launch_ln_cf_tile(const void *x, const void *w, const void *b, void *y, int B, int C, int L, float eps,
                             int out_channel_last, hipStream_t stream) {
    const int tiles = (L + kCfTile - 1) / kCfTile;
    const int64_t n_wg = (int64_t)B * tiles;
    const size_t smem = (size_t)C * (kCfTile + 1) * sizeof(float);
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    // tiles beyond the default 64 KB of dynamic LDS are requested explicitly (a CU has 160 KB)
    auto raise_limit = [&](const void *kern) {
        return smem <= 64 * 1024 ||
               hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) == hipSuccess;
    };
    if (out_channel_last) {
        auto kern = layer_norm_cf_kernel<in_t, w_t, out_t, true, kCfTile>;
        if (!raise_limit(reinterpret_cast<const void *>(kern))) return SS2D_ELAUNCH;
        hipLaunchKernelGGL(kern, dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, (const in_t *)x, (const w_t *)w, (const w_t *)b,
                           (out_t *)y, C, L, tiles, eps);
    } else {
        auto kern = layer_norm_cf_kernel<in_t, w_t, out_t, false, kCfTile>;
        if (!raise_limit(reinterpret_cast<const void *>(kern))) return SS2D_ELAUNCH;
        hipLaunchKernelGGL(kern, dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, (const in_t *)x, (const w_t *)w, (const w_t *)b,
                           (out_t *)y, C, L, tiles, eps);
    }
    return launch_status();
}

template <typename in_t, typename w_t, typename out_t, int kTP, int kG, int kVPT>
static int launch_ln_cf_reg(const void *x, const void *w, const void *b, void *y, int B, int C, int L, float eps,
                            int out_channel_last, hipStream_t stream) {
    const int tiles = (L + kTP - 1) / kTP;
    const int64_t n_wg = (int64_t)B * tiles;
    if (n_wg > 0x7fffffff || (int64_t)C * L * (int64_t)sizeof(in_t) >= 0x7ffffff0ll) return SS2D_ENOTSUP;
    // LDS pitch of the turn-round tile: lanes walk positions, so consecutive rows must land in different banks
    int Cp = sizeof(out_t) == 2 ? ((C + 1) & ~1) : (C | 1);
    if (sizeof(out_t) == 2 && (Cp / 2) % 2 == 0) Cp += 2;
    if (out_channel_last) {
        const size_t smem = (size_t)kTP * Cp * sizeof(out_t);
        hipLaunchKernelGGL((layer_norm_cf_reg_kernel<in_t, w_t, out_t, true, kTP, kG, kVPT>), dim3((uint32_t)n_wg), dim3(kBlock),
                           smem, stream, (const in_t *)x, (const w_t *)w, (const w_t *)b, (out_t *)y, C, L, tiles, Cp, eps);
    } else {
        hipLaunchKernelGGL((layer_norm_cf_reg_kernel<in_t, w_t, out_t, false, kTP, kG, kVPT>), dim3((uint32_t)n_wg), dim3(kBlock),
                           0, stream, (const in_t *)x, (const w_t *)w, (const w_t *)b, (out_t *)y, C, L, tiles, Cp, eps);
    }
    return launch_status();
}

template <typename in_t, typename w_t, typename out_t, int kQ, int kG, int kCPL>
static int launch_ln_cf_quad(const void *x, const void *w, const void *b, void *y, int B, int C, int L, float eps,
                             int out_channel_last, hipStream_t stream) {
    constexpr int kTP = 4 * kQ;
    const int tiles = (L + kTP - 1) / kTP;
    const int64_t n_wg = (int64_t)B * tiles;
    // LDS pitch of the turn-round tile: rows 16-byte aligned, and four rows apart never in the same banks
    const int piece = 16 / (int)sizeof(out_t);
    const int Cp = ((C + piece - 1) / piece) * piece + piece;
    if (out_channel_last) {
        const size_t smem = (size_t)kTP * Cp * sizeof(out_t);
        hipLaunchKernelGGL((layer_norm_cf_quad_kernel<in_t, w_t, out_t, true, kQ, kG, kCPL>), dim3((uint32_t)n_wg), dim3(kBlock), smem,
                           stream, (const in_t *)x, (const w_t *)w, (const w_t *)b, (out_t *)y, C, L, tiles, Cp, eps);
    } else {
        hipLaunchKernelGGL((layer_norm_cf_quad_kernel<in_t, w_t, out_t, false, kQ, kG, kCPL>), dim3((uint32_t)n_wg), dim3(kBlock), 0,
                           stream, (const in_t *)x, (const w_t *)w, (const w_t *)b, (out_t *)y, C, L, tiles, Cp, eps);
    }
    return launch_status();
}

// The image variant's split of an image and its launch; false when the shape is not one it covers.
struct LnImagePlan { int kch, ku, T, Qn, G, threads, pitch_dw; size_t smem; };
static bool ln_image_plan(int B, int C, int L, size_t out_size, bool out_channel_last, LnImagePlan &p) {
    if (L > 1024 || (int64_t)C * L * 4 >= 0x7ffffff0ll) return false;
    p.kch = L % 4 == 0 ? 1 : 4;
    if (C % (2 * p.kch) != 0) return false;                     // a lane's channels (kCh = 1) or units (kCh = 4) come in pairs
    if (out_channel_last && (C * out_size) % 16 != 0) return false;
    const int Q = p.kch * L / 4, n_units = C / p.kch;
    p.pitch_dw = (int)(out_size == 4 ? C : C / 2) | 1;
    if (p.kch == 4 && L < 2) return false;                     // four elements of a vector would meet more than two channels
    // The fewest workgroups per image that fit (threads, LDS), then finer splits: down to runs of 384 bytes per
    // channel row in any case (smaller tiles let two workgroups share a CU and overlap their phases), and down to
    // 192 bytes while there are fewer workgroups than CUs.
    const int t_max = p.kch == 1 ? Q : 1;
    bool found = false;
    size_t tile_cl = 0;                                        // LDS of the plan found so far if it wrote channel-last
    for (int T = 1; T <= t_max; ++T) {
        const int Qn = (Q + T - 1) / T;
        if ((Qn - 1) * T >= Q) continue;                       // an empty last share: the split of a smaller T
        // (a channel-last tile beyond half a CU's LDS keeps the CU to one workgroup, which is fine while the chip holds
        // every workgroup at once; with more workgroups than CUs split on until two fit.  The channel-first output
        // takes the same split, so that both layouts hold the same values bit for bit)
        const bool one_round = tile_cl <= 76 * 1024 || (int64_t)B * p.T <= 256;
        if (found && one_round && (Qn < 12 || (Qn < 24 && (int64_t)B * p.T >= 256))) break;
        const int positions = p.kch == 1 ? 4 * Qn : L;
        if (positions > kLnImgStat) continue;
        const size_t smem_cl = (size_t)4 * kLnImgBlock * 4 + 2 * kLnImgStat * 4 + (size_t)2 * C * 4 + (size_t)positions * p.pitch_dw * 4;
        const size_t smem = out_channel_last ? smem_cl : smem_cl - (size_t)positions * p.pitch_dw * 4;
        if (smem > 100 * 1024) continue;
        for (int ku : {8, 10}) {
            const int G = (n_units + ku - 1) / ku;
            if ((int64_t)G * Qn > kLnImgBlock) continue;
            p.ku = ku; p.T = T; p.Qn = Qn; p.G = G; p.threads = ((G * Qn + kWave - 1) / kWave) * kWave; p.smem = smem;
            tile_cl = smem_cl;
            found = true;
            break;
        }
    }
    return found;
}

template <typename in_t, typename w_t, typename out_t>
static int launch_ln_cf_image(const LnImagePlan &p, const void *x, const void *w, const void *b, void *y, int B, int C, int L,
                              float eps, int out_channel_last, hipStream_t stream) {
    const int64_t n_wg = (int64_t)B * p.T;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
#define SS2D_LN_IMAGE(CL, KCH, KU)                                                                                              \
    {                                                                                                                            \
        auto kern = layer_norm_cf_image_kernel<in_t, w_t, out_t, CL, KCH, KU>;                                                   \
        if (p.smem > 64 * 1024 &&                                                                                                \
            hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)p.smem) != hipSuccess) \
            return SS2D_ELAUNCH;                                                                                                 \
        hipLaunchKernelGGL(kern, dim3((uint32_t)n_wg), dim3(p.threads), p.smem, stream, (const in_t *)x, (const w_t *)w,         \
                           (const w_t *)b, (out_t *)y, C, L, p.T, p.Qn, p.G, p.pitch_dw, eps);                                   \
    }
    if (out_channel_last) {
        if (p.kch == 1) { if (p.ku == 8) SS2D_LN_IMAGE(true, 1, 8) else SS2D_LN_IMAGE(true, 1, 10) }
        else { if (p.ku == 8) SS2D_LN_IMAGE(true, 4, 8) else SS2D_LN_IMAGE(true, 4, 10) }
    } else {
        if (p.kch == 1) { if (p.ku == 8) SS2D_LN_IMAGE(false, 1, 8) else SS2D_LN_IMAGE(false, 1, 10) }
        else { if (p.ku == 8) SS2D_LN_IMAGE(false, 4, 8) else SS2D_LN_IMAGE(false, 4, 10) }
    }
#undef SS2D_LN_IMAGE
    return launch_status();
}

template <typename in_t, typename w_t, typename out_t>
static int launch_ln_cf(const void *x, const void *w, const void *b, void *y, int B, int C, int L, float eps,
                        int out_channel_last, hipStream_t stream) {
    {
        // short images: a whole image, or an even share of one, per workgroup
        LnImagePlan plan;
        if (L <= 1024 && ln_aligned16(x) && ln_aligned16(y) && ln_image_plan(B, C, L, sizeof(out_t), out_channel_last != 0, plan))
            return launch_ln_cf_image<in_t, w_t, out_t>(plan, x, w, b, y, B, C, L, eps, out_channel_last, stream);
    }
    {
        // quads of positions: 16-byte loads of fp32 input, 8-byte loads of 16-bit input (and 16-byte channel-last stores)
        const bool quad_ok = L % 4 == 0 && ln_aligned16(x) && (int64_t)C * L * 4 < 0x7ffffff0ll && (int64_t)B * ((L + 15) / 16) <= 0x7fffffff &&
                             (out_channel_last ? (C % (16 / (int)sizeof(out_t)) == 0 && ln_aligned16(y)) : ln_aligned16(y));
        if (quad_ok) {
            if (C <= 96) return launch_ln_cf_quad<in_t, w_t, out_t, 16, 16, 6>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
            if (C <= 192) return launch_ln_cf_quad<in_t, w_t, out_t, 16, 16, 12>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
            if (C <= 384) return launch_ln_cf_quad<in_t, w_t, out_t, 8, 32, 12>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
            if (C <= 768) return launch_ln_cf_quad<in_t, w_t, out_t, 4, 64, 12>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
        }
    }
    if (C <= 96) return launch_ln_cf_reg<in_t, w_t, out_t, 64, 4, 24>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
    if (C <= 192) return launch_ln_cf_reg<in_t, w_t, out_t, 64, 4, 48>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
    if (C <= 384) return launch_ln_cf_reg<in_t, w_t, out_t, 32, 8, 48>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
    if (C <= 768) return launch_ln_cf_reg<in_t, w_t, out_t, 16, 16, 48>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
    if (C <= 1536) return launch_ln_cf_reg<in_t, w_t, out_t, 8, 32, 48>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
    // very wide rows: the LDS-tile kernel, 8 positions per workgroup while that fits 48 KB, else 4 (up to 7800 channels
    // in 156 KB of LDS)
    if ((size_t)C * 9 * sizeof(float) <= 48 * 1024)
        return launch_ln_cf_tile<in_t, w_t, out_t, 8>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
    if ((size_t)C * 5 * sizeof(float) <= 156 * 1024)
        return launch_ln_cf_tile<in_t, w_t, out_t, 4>(x, w, b, y, B, C, L, eps, out_channel_last, stream);
    return SS2D_ENOTSUP;
}

// dtype triple dispatch: F(in, w, out)
#define SS2D_LN_DISPATCH(CALL)                                                                              \
    switch (in_dtype * 9 + w_dtype * 3 + out_dtype) {                                                        \
        case SS2D_F32 * 9 + SS2D_F32 * 3 + SS2D_F32: return CALL(float, float, float);                      \
        case SS2D_F32 * 9 + SS2D_F32 * 3 + SS2D_BF16: return CALL(float, float, bf16_t);                    \
        case SS2D_F32 * 9 + SS2D_BF16 * 3 + SS2D_BF16: return CALL(float, bf16_t, bf16_t);                  \
        case SS2D_F32 * 9 + SS2D_BF16 * 3 + SS2D_F32: return CALL(float, bf16_t, float);                    \
        case SS2D_BF16 * 9 + SS2D_BF16 * 3 + SS2D_BF16: return CALL(bf16_t, bf16_t, bf16_t);                \
        case SS2D_BF16 * 9 + SS2D_F32 * 3 + SS2D_BF16: return CALL(bf16_t, float, bf16_t);                  \
        case SS2D_F32 * 9 + SS2D_F16 * 3 + SS2D_F16: return CALL(float, f16_t, f16_t);                      \
        case SS2D_F16 * 9 + SS2D_F16 * 3 + SS2D_F16: return CALL(f16_t, f16_t, f16_t);                      \
        case SS2D_F16 * 9 + SS2D_F32 * 3 + SS2D_F16: return CALL(f16_t, float, f16_t);                      \
        default: return SS2D_ENOTSUP;                                                                        \
    }

static bool ln_dtype_ok(int d) { return d == SS2D_F32 || d == SS2D_BF16 || d == SS2D_F16; }

}  // namespace ss2d

extern "C" int ss2d_layer_norm(const void *x, const void *weight, const void *bias, void *y, int64_t rows, int C, float eps,
                               int in_dtype, int w_dtype, int out_dtype, void *stream) {
    using namespace ss2d;
    if (rows < 0 || C < 0 || !ln_dtype_ok(in_dtype) || !ln_dtype_ok(w_dtype) || !ln_dtype_ok(out_dtype)) return SS2D_EINVAL;
    if (rows == 0 || C == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    hipStream_t s = (hipStream_t)stream;
#define SS2D_CALL(I, W, O) launch_ln_rows<I, W, O>(x, weight, bias, y, rows, C, eps, s)
    SS2D_LN_DISPATCH(SS2D_CALL)
#undef SS2D_CALL
}

extern "C" int ss2d_add_layer_norm(const void *x, const void *residual, const void *weight, const void *bias, void *sum_out,
                                   void *y, int64_t rows, int C, float eps, int in_dtype, int w_dtype, int out_dtype,
                                   void *stream) {
    using namespace ss2d;
    if (rows < 0 || C < 0 || !ln_dtype_ok(in_dtype) || !ln_dtype_ok(w_dtype) || !ln_dtype_ok(out_dtype)) return SS2D_EINVAL;
    if (rows == 0 || C == 0) return SS2D_OK;
    if (!x || !residual || !sum_out || !y) return SS2D_EINVAL;
    hipStream_t s = (hipStream_t)stream;
#define SS2D_CALL(I, W, O) launch_ln_rows<I, W, O>(x, weight, bias, y, rows, C, eps, s, residual, sum_out)
    SS2D_LN_DISPATCH(SS2D_CALL)
#undef SS2D_CALL
}

extern "C" int ss2d_bias_layer_norm(const void *x, const void *pre_bias, const void *weight, const void *bias, void *y,
                                    int64_t rows, int C, float eps, int in_dtype, int w_dtype, int out_dtype, void *stream) {
    using namespace ss2d;
    if (rows < 0 || C < 0 || !ln_dtype_ok(in_dtype) || !ln_dtype_ok(w_dtype) || !ln_dtype_ok(out_dtype)) return SS2D_EINVAL;
    if (rows == 0 || C == 0) return SS2D_OK;
    if (!x || !pre_bias || !y) return SS2D_EINVAL;
    hipStream_t s = (hipStream_t)stream;
#define SS2D_CALL(I, W, O) launch_ln_rows<I, W, O>(x, weight, bias, y, rows, C, eps, s, nullptr, nullptr, pre_bias)
    SS2D_LN_DISPATCH(SS2D_CALL)
#undef SS2D_CALL
}

extern "C" int ss2d_layer_norm_cf(const void *x, const void *weight, const void *bias, void *y, int B, int C, int L, float eps,
                                  int in_dtype, int w_dtype, int out_dtype, int out_channel_last, void *stream) {
    using namespace ss2d;
    if (B < 0 || C < 0 || L < 0 || !ln_dtype_ok(in_dtype) || !ln_dtype_ok(w_dtype) || !ln_dtype_ok(out_dtype)) return SS2D_EINVAL;
    if (B == 0 || C == 0 || L == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    hipStream_t s = (hipStream_t)stream;
#define SS2D_CALL(I, W, O) launch_ln_cf<I, W, O>(x, weight, bias, y, B, C, L, eps, out_channel_last, s)
    SS2D_LN_DISPATCH(SS2D_CALL)
#undef SS2D_CALL
}
