// Device-side helpers shared by the SS2D kernels (gfx950 / CDNA4, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ss2d_hip.h"

namespace ss2d {

constexpr int kWave = 64;       // CDNA wavefront
constexpr int kBlock = 256;     // 4 waves per workgroup everywhere
constexpr int kXcds = 8;        // MI355X: 8 XCDs, workgroups are dealt to them round-robin

// ---- element types ----------------------------------------------------------
struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };

template <typename T> struct ElemTraits;
template <> struct ElemTraits<float> { static constexpr int dtype = SS2D_F32; };
template <> struct ElemTraits<bf16_t> { static constexpr int dtype = SS2D_BF16; };
template <> struct ElemTraits<f16_t> { static constexpr int dtype = SS2D_F16; };

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return bits_to_f32(((uint32_t)v.bits) << 16); }
__device__ __forceinline__ float to_f32(f16_t v) { return (float)__builtin_bit_cast(_Float16, v.bits); }

// round-to-nearest-even, NaN stays NaN (quiet)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = f32_to_bits(f);
    uint32_t r = u + 0x7fffu + ((u >> 16) & 1u);
    r = ((u & 0x7fffffffu) > 0x7f800000u) ? (u | 0x00400000u) : r;
    return (uint16_t)(r >> 16);
}

template <typename T> __device__ __forceinline__ T from_f32(float f);
template <> __device__ __forceinline__ float from_f32<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float f) { return bf16_t{f32_to_bf16_bits(f)}; }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float f) {
    return f16_t{__builtin_bit_cast(uint16_t, (_Float16)f)};
}

// two fp32 -> one dword of packed 16-bit values (low half first), round-to-nearest-even: v_cvt_pk_bf16_f32 /
// v_cvt_pk_f16_f32, the same results as from_f32 in one instruction per pair
typedef float floatx2_t __attribute__((ext_vector_type(2)));
template <typename T> __device__ __forceinline__ uint32_t pack2_from_f32(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2_from_f32<bf16_t>(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const floatx2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
template <> __device__ __forceinline__ uint32_t pack2_from_f32<f16_t>(float lo, float hi) {
    typedef _Float16 halfx2_t __attribute__((ext_vector_type(2)));
    const floatx2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, halfx2_t));
}
template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t w) { return to_f32(T{(uint16_t)(w & 0xffffu)}); }
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t w) { return to_f32(T{(uint16_t)(w >> 16)}); }
template <> __device__ __forceinline__ float unpack_hi<bf16_t>(uint32_t w) { return bits_to_f32(w & 0xffff0000u); }

// ---- division by a runtime constant -------------------------------------------
// q = n / d for n < 2^32 using one mulhi and one correction; m = floor(2^32 / d) (d >= 2) or
// the divisor 1 flagged by m == 0.
struct FastDiv {
    uint32_t d, m;
};
inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    f.m = d <= 1 ? 0u : (uint32_t)((1ull << 32) / d);
    return f;
}
__device__ __forceinline__ void divmod(uint32_t n, const FastDiv f, uint32_t &q, uint32_t &r) {
    if (f.m == 0u) { q = n; r = 0; return; }
    q = __umulhi(n, f.m);
    r = n - q * f.d;
    if (r >= f.d) { q += 1; r -= f.d; }
}

// ---- XCD-aware workgroup order ---------------------------------------------------
// Hardware deals workgroup ids round-robin over the 8 XCDs (each with its own L2).  This maps
// a hardware id to a logical id so that every XCD works on one contiguous range of logical
// workgroups: neighbours (which share B/C rows or cache lines) meet in the same L2.
__device__ __forceinline__ uint32_t xcd_contiguous_id(uint32_t hw_id, uint32_t n_wg) {
    const uint32_t per = n_wg / kXcds, rem = n_wg % kXcds;
    const uint32_t xcd = hw_id % kXcds, idx = hw_id / kXcds;
    return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

// ---- DPP lane movement --------------------------------------------------------------
// Lanes whose source is out of range (or whose row is masked off) receive `old`.
template <int kCtrl, int kRowMask = 0xF>
__device__ __forceinline__ float dpp_move(float old, float v) {
    return bits_to_f32((uint32_t)__builtin_amdgcn_update_dpp((int)f32_to_bits(old), (int)f32_to_bits(v), kCtrl,
                                                             kRowMask, 0xF, false));
}
constexpr int kDppRowShr1 = 0x111, kDppRowShr2 = 0x112, kDppRowShr4 = 0x114, kDppRowShr8 = 0x118;
constexpr int kDppRowBcast15 = 0x142, kDppRowBcast31 = 0x143, kDppWaveShr1 = 0x138, kDppWaveShl1 = 0x130;

__device__ __forceinline__ float read_lane(float v, int lane) {
    return bits_to_f32((uint32_t)__builtin_amdgcn_readlane((int)f32_to_bits(v), lane));
}

// ---- streaming accesses ---------------------------------------------------------------------------------------
// Non-temporal loads and stores for data that is read once, or written once and read back only after far more traffic
// than the caches hold: they leave the cache replacement order alone.  U: any trivially copyable type of 1, 2, 4, 8 or 16 bytes.
template <int kBytes> struct StreamWord;
template <> struct StreamWord<1> { using type = uint8_t; };
template <> struct StreamWord<2> { using type = uint16_t; };
template <> struct StreamWord<4> { using type = uint32_t; };
template <> struct StreamWord<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct StreamWord<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <typename U> __device__ __forceinline__ U load_streaming(const U *p) {
    using W = typename StreamWord<sizeof(U)>::type;
    return __builtin_bit_cast(U, __builtin_nontemporal_load(reinterpret_cast<const W *>(p)));
}
template <typename U> __device__ __forceinline__ void store_streaming(U *p, U v) {
    using W = typename StreamWord<sizeof(U)>::type;
    __builtin_nontemporal_store(__builtin_bit_cast(W, v), reinterpret_cast<W *>(p));
}

// ---- matrix cores -------------------------------------------------------------------------------------------
// v_mfma_f32_32x32x8 (bf16 / f16 operands, fp32 accumulate): D (32 x 32) += A (32 x 8) * B (8 x 32).  Lane l supplies
// A[l % 32][4*(l/32) .. +3] and B[4*(l/32) .. +3][l % 32] as two dwords of packed 16-bit values, and holds
// D[8*(v/4) + 4*(l/32) + v%4][l % 32] in accumulator v = 0..15.
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ floatx16_t mfma_32x32x8(bf16_t, const uint32_t (&a)[2], const uint32_t (&b)[2], floatx16_t c) {
    const short4_t av = {(short)(a[0] & 0xffffu), (short)(a[0] >> 16), (short)(a[1] & 0xffffu), (short)(a[1] >> 16)};
    const short4_t bv = {(short)(b[0] & 0xffffu), (short)(b[0] >> 16), (short)(b[1] & 0xffffu), (short)(b[1] >> 16)};
    return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(av, bv, c, 0, 0, 0);
}
__device__ __forceinline__ floatx16_t mfma_32x32x8(f16_t, const uint32_t (&a)[2], const uint32_t (&b)[2], floatx16_t c) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 aw = {a[0], a[1]}, bw = {b[0], b[1]};
    return __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(half4_t, aw), __builtin_bit_cast(half4_t, bw), c, 0, 0, 0);
}

// v_mfma_f32_32x32x16 (gfx950): D (32 x 32) += A (32 x 16) * B (16 x 32).  Lane l supplies A[l % 32][8*(l/32) .. +7] and
// B[8*(l/32) .. +7][l % 32] as four dwords; the accumulator layout is that of 32x32x8.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ floatx16_t mfma_32x32x16(bf16_t, u32x4_t a, u32x4_t b, floatx16_t c) {
    typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ floatx16_t mfma_32x32x16(f16_t, u32x4_t a, u32x4_t b, floatx16_t c) {
    typedef _Float16 halfx8_t __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8_t, a), __builtin_bit_cast(halfx8_t, b), c, 0, 0, 0);
}

// LDS traffic of one wavefront is ordered by program order; this keeps the compiler from moving it around when
// lanes exchange data through a wavefront-private LDS region (no workgroup barrier needed).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// LayerNorm of the 32 rows of a wavefront-private LDS tile of 16-bit values, in place: row j (pitch `pitch` elements,
// K channels) is normalised by lanes j and j + 32, each owning half of the channels; fp32 statistics with the centred
// variance, result rounded to T.  gamma / beta: K 16-bit values each in LDS (16-byte aligned).  The caller brackets
// the call with wave_lds_sync().
template <typename T, int K>
__device__ __forceinline__ void layer_norm_tile_rows(uint16_t *tile, int pitch, int lane, const uint16_t *gamma,
                                                     const uint16_t *beta, float eps) {
    constexpr int kHalf = K / 2, kVec = kHalf / 8;
    static_assert(kHalf % 8 == 0, "whole 16-byte pieces per half row");
    const int j = lane & 31, kh = lane >> 5;
    uint16_t *row = tile + j * pitch + kh * kHalf;
    float v[kHalf];
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
        const uint4 q4 = *reinterpret_cast<const uint4 *>(row + 8 * i);
        const uint32_t ww[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[8 * i + 2 * e] = unpack_lo<T>(ww[e]);
            v[8 * i + 2 * e + 1] = unpack_hi<T>(ww[e]);
            sum += v[8 * i + 2 * e] + v[8 * i + 2 * e + 1];
        }
    }
    sum += __shfl_xor(sum, 32);
    const float mean = sum * (1.0f / K);
    float sq = 0.0f;
#pragma unroll
    for (int i = 0; i < kHalf; ++i) { const float c = v[i] - mean; sq = fmaf(c, c, sq); }
    sq += __shfl_xor(sq, 32);
    const float rstd = __builtin_amdgcn_rsqf(sq * (1.0f / K) + eps);
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
        const uint4 g4 = *reinterpret_cast<const uint4 *>(gamma + kh * kHalf + 8 * i);
        const uint4 b4 = *reinterpret_cast<const uint4 *>(beta + kh * kHalf + 8 * i);
        const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, bw[4] = {b4.x, b4.y, b4.z, b4.w};
        uint32_t ow[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float lo = fmaf((v[8 * i + 2 * e] - mean) * rstd, unpack_lo<T>(gw[e]), unpack_lo<T>(bw[e]));
            const float hi = fmaf((v[8 * i + 2 * e + 1] - mean) * rstd, unpack_hi<T>(gw[e]), unpack_hi<T>(bw[e]));
            ow[e] = pack2_from_f32<T>(lo, hi);
        }
        *reinterpret_cast<uint4 *>(row + 8 * i) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
}

inline int launch_status() { return hipGetLastError() == hipSuccess ? SS2D_OK : SS2D_ELAUNCH; }

}  // namespace ss2d
