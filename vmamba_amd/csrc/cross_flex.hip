// CrossScan / CrossMerge for every layout and scan mode of the reference's "flex" kernel
// (classification/models/csm_triton.py:278-400; torch semantics :22-179):
//   x layout   channel-first (B,[4,]C,H,W)  or channel-last (B,H,W,[4,]C)
//   y layout   channel-first (B,4,C,L)      or channel-last (B,L,4,C)
//   one_by_one: x carries its own slice per direction instead of one map shared by the four
//   scans      0: the four cross-scan routes (row-major, column-major, both reversed)
//              1: four times the row-major route           2: row-major twice, reversed twice
// The combination the SS2D core uses (both channel-first, shared map, scans = 0) has its own tiled kernels
// (cross_scan.hip, cross_merge.hip); this file covers all the others with one kernel per operation: a thread per
// OUTPUT element in the output's memory order (so stores are coalesced), the source found through the route.
// Reads are coalesced whenever the route keeps the innermost dimension (every channel-last source, and the
// non-transposing routes of channel-first sources); the transposing routes of channel-first sources gather through L2.
#include <mutex>

#include "ss2d_common.h"

namespace ss2d {

struct FlexArgs {
    const void *src;
    void *dst;
    int32_t B, C, H, W, L, x_cl, y_cl, one_by_one, scans, order;
    uint32_t total;          // output elements (or channel vectors); host-checked < 2^32
    int32_t stream_out;      // CrossScan: the output exceeds the last-level cache and leaves as non-temporal stores;
                             // CrossMerge: operands beyond that cache, in 16-byte pieces, are read (and the result written) so
    FastDiv divC, divL, divW, divH;
};

// scan position of direction k for the row-major spatial index r (csm_triton.py:308-328)
__device__ __forceinline__ uint32_t flex_route(int k, int scans, uint32_t r, const FlexArgs &p) {
    const bool reversed = scans == 1 ? false : k >= 2;
    const bool transposed = scans == 0 && (k & 1);
    uint32_t j = r;
    if (transposed) {
        uint32_t h, w;
        divmod(r, p.divW, h, w);
        j = w * (uint32_t)p.H + h;
    }
    return reversed ? (uint32_t)p.L - 1 - j : j;
}
// its inverse: the row-major spatial index that direction k visits at scan position j
__device__ __forceinline__ uint32_t flex_route_inv(int k, int scans, uint32_t j, const FlexArgs &p) {
    const bool reversed = scans == 1 ? false : k >= 2;
    const bool transposed = scans == 0 && (k & 1);
    uint32_t s = reversed ? (uint32_t)p.L - 1 - j : j;
    if (transposed) {
        uint32_t w, h;
        divmod(s, p.divH, w, h);
        s = h * (uint32_t)p.W + w;
    }
    return s;
}

__device__ __forceinline__ int64_t flex_x_offset(const FlexArgs &p, uint32_t b, int k, uint32_t c, uint32_t r) {
    const int K = p.one_by_one ? 4 : 1, kk = p.one_by_one ? k : 0;
    return p.x_cl ? (((int64_t)b * p.L + r) * K + kk) * p.C + c : (((int64_t)b * K + kk) * p.C + c) * p.L + r;
}
__device__ __forceinline__ int64_t flex_y_offset(const FlexArgs &p, uint32_t b, int k, uint32_t c, uint32_t j) {
    return p.y_cl ? (((int64_t)b * p.L + j) * 4 + k) * p.C + c : (((int64_t)b * 4 + k) * p.C + c) * p.L + j;
}

// y (in its own memory order) <- x
template <typename U>
__global__ __launch_bounds__(kBlock) void cross_scan_flex_kernel(const FlexArgs p) {
    const uint32_t idx = blockIdx.x * kBlock + threadIdx.x;
    if (idx >= p.total) return;
    uint32_t b, k, c, j, q;
    if (p.y_cl) {                           // (B, L, 4, C)
        divmod(idx, p.divC, q, c);
        k = q & 3;
        divmod(q >> 2, p.divL, b, j);
    } else {                                // (B, 4, C, L)
        divmod(idx, p.divL, q, j);
        uint32_t bk;
        divmod(q, p.divC, bk, c);
        b = bk >> 2; k = bk & 3;
    }
    const uint32_t r = flex_route_inv((int)k, p.scans, j, p);
    const U v = reinterpret_cast<const U *>(p.src)[flex_x_offset(p, b, (int)k, c, r)];
    if (p.stream_out) store_streaming(reinterpret_cast<U *>(p.dst) + idx, v);       // uniform
    else reinterpret_cast<U *>(p.dst)[idx] = v;
}

// Channel-first on both sides with routes that do not transpose (scans 1 and 2): y_k is x_(k) copied or reversed
// along L, so a thread moves 16 bytes; reversed routes read the mirrored 16 bytes and swap the elements inside.
template <int kElemBytes> __device__ __forceinline__ uint4 flex_reverse16(uint4 v) {
    if constexpr (kElemBytes == 8) return make_uint4(v.z, v.w, v.x, v.y);
    uint4 r = make_uint4(v.w, v.z, v.y, v.x);
    if constexpr (kElemBytes <= 2) {
        r.x = (r.x >> 16) | (r.x << 16); r.y = (r.y >> 16) | (r.y << 16);
        r.z = (r.z >> 16) | (r.z << 16); r.w = (r.w >> 16) | (r.w << 16);
    }
    if constexpr (kElemBytes == 1) {
        r.x = ((r.x & 0x00ff00ffu) << 8) | ((r.x >> 8) & 0x00ff00ffu); r.y = ((r.y & 0x00ff00ffu) << 8) | ((r.y >> 8) & 0x00ff00ffu);
        r.z = ((r.z & 0x00ff00ffu) << 8) | ((r.z >> 8) & 0x00ff00ffu); r.w = ((r.w & 0x00ff00ffu) << 8) | ((r.w >> 8) & 0x00ff00ffu);
    }
    return r;
}

template <int kElemBytes>
__global__ __launch_bounds__(kBlock) void cross_scan_rows_vec_kernel(const FlexArgs p, uint32_t Lv, FastDiv divLv) {
    const uint32_t idx = blockIdx.x * kBlock + threadIdx.x;          // over (B, 4, C, L / vec)
    if (idx >= p.total) return;
    uint32_t q, jv, bk, c;
    divmod(idx, divLv, q, jv);
    divmod(q, p.divC, bk, c);
    const uint32_t b = bk >> 2, k = bk & 3;
    const bool reversed = p.scans == 2 && k >= 2;
    const uint32_t K = p.one_by_one ? 4 : 1, kk = p.one_by_one ? k : 0;
    const uint4 *src = reinterpret_cast<const uint4 *>(p.src) + ((size_t)(b * K + kk) * p.C + c) * Lv;
    uint4 v = src[reversed ? Lv - 1 - jv : jv];
    if (reversed) v = flex_reverse16<kElemBytes>(v);
    if (p.stream_out) store_streaming(reinterpret_cast<uint4 *>(p.dst) + idx, v);   // uniform
    else reinterpret_cast<uint4 *>(p.dst)[idx] = v;
}

template <typename T> __device__ __forceinline__ T flex_add(T a, T b) { return from_f32<T>(to_f32(a) + to_f32(b)); }

// x (in its own memory order) <- y
template <typename T> __device__ __forceinline__ T flex_combine(const T (&v)[4], int scans, int order) {
    if (scans == 1)     // the reference sums the four copies with a reduction (csm_triton.py:64, 75): fp32, one rounding
        return from_f32<T>(((to_f32(v[0]) + to_f32(v[1])) + to_f32(v[2])) + to_f32(v[3]));
    if (order == SS2D_MERGE_PAIRWISE) return flex_add(flex_add(v[0], v[2]), flex_add(v[1], v[3]));
    return flex_add(flex_add(flex_add(v[0], v[1]), v[2]), v[3]);
}

// x (in its own memory order) <- y.  kVec elements of T per thread along the channel axis (kVec > 1 only when both
// sides are channel-last; C then counts vectors).
template <typename T, int kVec>
__global__ __launch_bounds__(kBlock) void cross_merge_flex_kernel(const FlexArgs p) {
    const uint32_t idx = blockIdx.x * kBlock + threadIdx.x;
    if (idx >= p.total) return;
    uint32_t b, k = 0, c, r, q;
    if (p.x_cl) {                           // (B, L, [4,] C)
        divmod(idx, p.divC, q, c);
        if (p.one_by_one) { k = q & 3; q >>= 2; }
        divmod(q, p.divL, b, r);
    } else {                                // (B, [4,] C, L)
        divmod(idx, p.divL, q, r);
        uint32_t bk;
        divmod(q, p.divC, bk, c);
        if (p.one_by_one) { b = bk >> 2; k = bk & 3; } else { b = bk; }
    }
    struct alignas(sizeof(T) * kVec) Vec { T e[kVec]; };
    const Vec *y = reinterpret_cast<const Vec *>(p.src);
    Vec *x = reinterpret_cast<Vec *>(p.dst);
    // operands read once, result written once: streaming accesses where they pay (channel vectors of operands beyond the
    // last-level cache, stage 1 channel-last 139 -> 129 us; element-wise they cost, 144 -> 156)
    auto get = [&](const Vec *src) { return p.stream_out ? load_streaming(src) : *src; };
    auto put = [&](Vec *dst, const Vec &v) {
        if (p.stream_out) store_streaming(dst, v);
        else *dst = v;
    };
    if (p.one_by_one) {
        put(x + idx, get(y + flex_y_offset(p, b, (int)k, c, flex_route((int)k, p.scans, r, p))));
        return;
    }
    Vec v[4], out;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) v[kk] = get(y + flex_y_offset(p, b, kk, c, flex_route(kk, p.scans, r, p)));
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
        const T t[4] = {v[0].e[i], v[1].e[i], v[2].e[i], v[3].e[i]};
        out.e[i] = flex_combine(t, p.scans, p.order);
    }
    put(x + idx, out);
}

static int flex_fill(FlexArgs &a, int B, int C, int H, int W, int x_cl, int y_cl, int one_by_one, int scans) {
    if (B < 0 || C < 0 || H < 0 || W < 0) return SS2D_EINVAL;
    if ((x_cl | 1) != 1 || (y_cl | 1) != 1 || (one_by_one | 1) != 1 || scans < 0 || scans > 2) return SS2D_EINVAL;
    const int64_t L = (int64_t)H * W;
    if (L > 0x3fffffff || (int64_t)B * 4 * C > 0x7fffffff || (int64_t)B * L * 4 > 0x7fffffff) return SS2D_ENOTSUP;
    a.B = B; a.C = C; a.H = H; a.W = W; a.L = (int32_t)L;
    a.x_cl = x_cl; a.y_cl = y_cl; a.one_by_one = one_by_one; a.scans = scans; a.order = 0;
    a.divC = make_fastdiv((uint32_t)(C > 0 ? C : 1)); a.divL = make_fastdiv((uint32_t)(L > 0 ? L : 1));
    a.divW = make_fastdiv((uint32_t)(W > 0 ? W : 1)); a.divH = make_fastdiv((uint32_t)(H > 0 ? H : 1));
    a.stream_out = 0;
    return SS2D_OK;
}

}  // namespace ss2d

extern "C" int ss2d_cross_scan_flex(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int x_channel_last,
                                    int y_channel_last, int one_by_one, int scans, void *stream) {
    using namespace ss2d;
    FlexArgs a;
    const int rc = flex_fill(a, B, C, H, W, x_channel_last, y_channel_last, one_by_one, scans);
    if (rc != SS2D_OK) return rc;
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return SS2D_EINVAL;
    if (B == 0 || C == 0 || H == 0 || W == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    a.src = x; a.dst = y;
    a.stream_out = (int64_t)B * 4 * C * a.L * elem_bytes > ((int64_t)256 << 20);
    // both sides channel-last: the copy moves whole channel rows, so it is done in 16-byte pieces when they divide C
    if (x_channel_last && y_channel_last && ((int64_t)C * elem_bytes) % 16 == 0 &&
        ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0) {
        a.C = (int32_t)((int64_t)C * elem_bytes / 16);
        a.divC = make_fastdiv((uint32_t)a.C);
        elem_bytes = 16;
    }
    hipStream_t s = (hipStream_t)stream;
    // both sides channel-first, no transposing route: 16-byte pieces along L
    const int vec = 16 / elem_bytes;
    if (!x_channel_last && !y_channel_last && scans != 0 && elem_bytes < 16 && a.L % vec == 0 &&
        ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0) {
        const uint32_t Lv = (uint32_t)(a.L / vec);
        const int64_t total_v = (int64_t)B * 4 * C * Lv;
        if (total_v > 0xffffffffll) return SS2D_ENOTSUP;
        a.total = (uint32_t)total_v;
        const uint32_t n = (uint32_t)((total_v + kBlock - 1) / kBlock);
        const FastDiv dLv = make_fastdiv(Lv);
        switch (elem_bytes) {
            case 1: hipLaunchKernelGGL((cross_scan_rows_vec_kernel<1>), dim3(n), dim3(kBlock), 0, s, a, Lv, dLv); break;
            case 2: hipLaunchKernelGGL((cross_scan_rows_vec_kernel<2>), dim3(n), dim3(kBlock), 0, s, a, Lv, dLv); break;
            case 4: hipLaunchKernelGGL((cross_scan_rows_vec_kernel<4>), dim3(n), dim3(kBlock), 0, s, a, Lv, dLv); break;
            default: hipLaunchKernelGGL((cross_scan_rows_vec_kernel<8>), dim3(n), dim3(kBlock), 0, s, a, Lv, dLv); break;
        }
        return launch_status();
    }
    const int64_t total = (int64_t)B * 4 * a.C * a.L;
    if (total > 0xffffffffll) return SS2D_ENOTSUP;
    a.total = (uint32_t)total;
    const int64_t n_wg = (total + kBlock - 1) / kBlock;
    if (elem_bytes == 16) {
        hipLaunchKernelGGL((cross_scan_flex_kernel<uint4>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, a);
        return launch_status();
    }
    switch (elem_bytes) {
        case 1: hipLaunchKernelGGL((cross_scan_flex_kernel<uint8_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, a); break;
        case 2: hipLaunchKernelGGL((cross_scan_flex_kernel<uint16_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, a); break;
        case 4: hipLaunchKernelGGL((cross_scan_flex_kernel<uint32_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, a); break;
        default: hipLaunchKernelGGL((cross_scan_flex_kernel<uint64_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, a); break;
    }
    return launch_status();
}

extern "C" int ss2d_cross_merge_flex(const void *y, void *x, int B, int C, int H, int W, int dtype, int x_channel_last,
                                     int y_channel_last, int one_by_one, int scans, int order, void *stream) {
    using namespace ss2d;
    FlexArgs a;
    const int rc = flex_fill(a, B, C, H, W, x_channel_last, y_channel_last, one_by_one, scans);
    if (rc != SS2D_OK) return rc;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (order != SS2D_MERGE_PAIRWISE && order != SS2D_MERGE_LEFT_TO_RIGHT) return SS2D_EINVAL;
    if (B == 0 || C == 0 || H == 0 || W == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    a.src = y; a.dst = x; a.order = order;
    const int eb = dtype == SS2D_F32 ? 4 : 2, vec = 16 / eb;
    const bool use_vec = x_channel_last && y_channel_last && C % vec == 0 &&
                         ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
    if (use_vec) {
        a.C = C / vec;
        a.divC = make_fastdiv((uint32_t)a.C);
    }
    a.stream_out = use_vec && 4 * (int64_t)B * C * a.L * eb > ((int64_t)256 << 20);
    const int64_t total = (int64_t)B * (one_by_one ? 4 : 1) * a.C * a.L;
    if (total > 0xffffffffll) return SS2D_ENOTSUP;
    a.total = (uint32_t)total;
    const int64_t n_wg = (total + kBlock - 1) / kBlock;
    hipStream_t s = (hipStream_t)stream;
#define SS2D_FLEX_MERGE(T, V) hipLaunchKernelGGL((cross_merge_flex_kernel<T, V>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, a)
    switch (dtype) {
        case SS2D_F32: if (use_vec) SS2D_FLEX_MERGE(float, 4); else SS2D_FLEX_MERGE(float, 1); break;
        case SS2D_BF16: if (use_vec) SS2D_FLEX_MERGE(bf16_t, 8); else SS2D_FLEX_MERGE(bf16_t, 1); break;
        default: if (use_vec) SS2D_FLEX_MERGE(f16_t, 8); else SS2D_FLEX_MERGE(f16_t, 1); break;
    }
#undef SS2D_FLEX_MERGE
    return launch_status();
}

// ---- layout change (B, C, L) <-> (B, L, C) --------------------------------------------------------------------
// The mixed-layout modes are served by the host as "bring the small x-side tensor to the other layout, then run the
// same-layout kernel": this is that layout change, a batched matrix transpose through a 64 x 64 LDS tile (reads
// and writes both run along the innermost axis of their side).
namespace ss2d {

template <typename U>
__global__ __launch_bounds__(kBlock) void transpose_bcl_kernel(const U *__restrict__ src, U *__restrict__ dst, int R, int S,
                                                               int r_tiles, int s_tiles) {
    // src (B, R, S) -> dst (B, S, R)
    constexpr int kT = 64;
    __shared__ U tile[kT][kT + 1];
    uint32_t wg = blockIdx.x;
    const uint32_t st = wg % s_tiles; wg /= s_tiles;
    const uint32_t rt = wg % r_tiles;
    const uint32_t b = wg / r_tiles;
    const int r0 = (int)rt * kT, s0 = (int)st * kT;
    const int lx = threadIdx.x % kT, ly = threadIdx.x / kT;            // 64 x 4
    const U *sb = src + (size_t)b * R * S;
    U *db = dst + (size_t)b * R * S;
#pragma unroll 4
    for (int i = ly; i < kT; i += kBlock / kT) {
        const int r = r0 + i, s = s0 + lx;
        if (r < R && s < S) tile[i][lx] = sb[(size_t)r * S + s];
    }
    __syncthreads();
#pragma unroll 4
    for (int i = ly; i < kT; i += kBlock / kT) {
        const int s = s0 + i, r = r0 + lx;
        if (r < R && s < S) db[(size_t)s * R + r] = tile[lx][i];
    }
}

// The same for 2- and 4-byte elements when both extents are multiples of a 16-byte vector and the tensors are 16-byte
// aligned: 16-byte loads along S, 16-byte stores along R, the turn made by reading the LDS tile down its columns one
// element at a time (the element-wise kernel above moves 128 bytes per wavefront instruction and is bound by their
// number).  Row pitch: an odd number of dwords, so that the 8 (16) row groups of a column read fall into different banks.
template <typename U>
__global__ __launch_bounds__(kBlock) void transpose_bcl_vec_kernel(const U *__restrict__ src, U *__restrict__ dst, int R, int S,
                                                                   int r_tiles, int s_tiles) {
    constexpr int kT = 64, kVec = 16 / (int)sizeof(U), kPpr = kT / kVec;   // pieces per tile row
    constexpr int kPitchDw = sizeof(U) == 2 ? 33 : 65;                      // dwords per tile row
    __shared__ uint32_t tile[kT * kPitchDw];
    uint32_t wg = blockIdx.x;
    const uint32_t st = wg % s_tiles; wg /= s_tiles;
    const uint32_t rt = wg % r_tiles;
    const uint32_t b = wg / r_tiles;
    const int r0 = (int)rt * kT, s0 = (int)st * kT;
    const U *sb = src + (size_t)b * R * S;
    U *db = dst + (size_t)b * R * S;
#pragma unroll
    for (int p = threadIdx.x; p < kT * kPpr; p += kBlock) {
        const int i = p / kPpr, pc = p % kPpr;
        const int r = r0 + i, sp = s0 + pc * kVec;
        if (r < R && sp < S) {
            const uint4 v = *reinterpret_cast<const uint4 *>(sb + (size_t)r * S + sp);
            uint32_t *row = tile + i * kPitchDw + pc * 4;
            row[0] = v.x; row[1] = v.y; row[2] = v.z; row[3] = v.w;
        }
    }
    __syncthreads();
#pragma unroll
    for (int p = threadIdx.x; p < kT * kPpr; p += kBlock) {
        const int si = p / kPpr, rp = p % kPpr;
        const int sp = s0 + si, r = r0 + rp * kVec;
        if (sp < S && r < R) {
            uint32_t w[4];
            if constexpr (sizeof(U) == 2) {
                const uint16_t *t16 = reinterpret_cast<const uint16_t *>(tile);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t lo = t16[(rp * 8 + 2 * k) * (2 * kPitchDw) + si], hi = t16[(rp * 8 + 2 * k + 1) * (2 * kPitchDw) + si];
                    w[k] = lo | (hi << 16);
                }
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) w[k] = tile[(rp * 4 + k) * kPitchDw + si];
            }
            *reinterpret_cast<uint4 *>(db + (size_t)sp * R + r) = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
}

}  // namespace ss2d

extern "C" int ss2d_transpose_bcl(const void *x, void *y, int B, int R, int S, int elem_bytes, void *stream) {
    using namespace ss2d;
    if (B < 0 || R < 0 || S < 0) return SS2D_EINVAL;
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return SS2D_EINVAL;
    if (B == 0 || R == 0 || S == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    const int r_tiles = (R + 63) / 64, s_tiles = (S + 63) / 64;
    const int64_t n_wg = (int64_t)B * r_tiles * s_tiles;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    hipStream_t s = (hipStream_t)stream;
    const int vec = 16 / elem_bytes;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
    if ((elem_bytes == 2 || elem_bytes == 4) && R % vec == 0 && S % vec == 0 && aligned) {
        if (elem_bytes == 2) hipLaunchKernelGGL((transpose_bcl_vec_kernel<uint16_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (const uint16_t *)x, (uint16_t *)y, R, S, r_tiles, s_tiles);
        else hipLaunchKernelGGL((transpose_bcl_vec_kernel<uint32_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (const uint32_t *)x, (uint32_t *)y, R, S, r_tiles, s_tiles);
        return launch_status();
    }
    switch (elem_bytes) {
        case 1: hipLaunchKernelGGL((transpose_bcl_kernel<uint8_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (const uint8_t *)x, (uint8_t *)y, R, S, r_tiles, s_tiles); break;
        case 2: hipLaunchKernelGGL((transpose_bcl_kernel<uint16_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (const uint16_t *)x, (uint16_t *)y, R, S, r_tiles, s_tiles); break;
        case 4: hipLaunchKernelGGL((transpose_bcl_kernel<uint32_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (const uint32_t *)x, (uint32_t *)y, R, S, r_tiles, s_tiles); break;
        default: hipLaunchKernelGGL((transpose_bcl_kernel<uint64_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (const uint64_t *)x, (uint64_t *)y, R, S, r_tiles, s_tiles); break;
    }
    return launch_status();
}

// ---- mixed layouts through a staging buffer --------------------------------------------------------------------
// When x and y differ in layout the route kernel above gathers across the innermost axis of its source (through L2,
// 4-5x slower than the copy-shaped cases).  Staged instead: the x-side tensor -- the small side, a fifth of the traffic
// -- is first brought to the layout of y with the tiled transpose, then the same-layout kernel runs.  The staging buffer
// holds one copy of x and is the caller's (a workspace argument).
namespace ss2d {

// Bytes of staging a mixed-layout CrossScan needs (0 when the layouts agree); negative status on bad arguments.
static int64_t cross_scan_staging_bytes(int B, int C, int H, int W, int elem_bytes, int x_cl, int y_cl, int one_by_one, int scans) {
    FlexArgs a;
    const int rc = flex_fill(a, B, C, H, W, x_cl, y_cl, one_by_one, scans);
    if (rc != SS2D_OK) return rc;
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return SS2D_EINVAL;
    if (x_cl == y_cl) return 0;
    return (int64_t)B * (one_by_one ? 4 : 1) * C * a.L * elem_bytes;
}

// The two launches.  Every limit either launch would refuse is checked before the first, so an error leaves nothing
// enqueued.  `staging` must hold cross_scan_staging_bytes(...) bytes, 16-byte aligned.
static int cross_scan_flex_staged(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int x_cl, int y_cl,
                                  int one_by_one, int scans, void *staging, void *stream) {
    const int64_t L = (int64_t)H * W, KC = (int64_t)(one_by_one ? 4 : 1) * C;
    if (KC > 0x7fffffff || (int64_t)B * 4 * C * L > 0xffffffffll) return SS2D_ENOTSUP;
    const int64_t r = x_cl ? L : KC, sdim = x_cl ? KC : L;           // x as (B, r, sdim) -> staging (B, sdim, r)
    if ((int64_t)B * ((r + 63) / 64) * ((sdim + 63) / 64) > 0x7fffffff) return SS2D_ENOTSUP;
    int rc = ss2d_transpose_bcl(x, staging, B, (int)r, (int)sdim, elem_bytes, stream);
    if (rc != SS2D_OK) return rc;
    if (y_cl) return ss2d_cross_scan_flex(staging, y, B, C, H, W, elem_bytes, 1, 1, one_by_one, scans, stream);
    if (scans != 0) return ss2d_cross_scan_flex(staging, y, B, C, H, W, elem_bytes, 0, 0, one_by_one, scans, stream);
    if (one_by_one) return ss2d_cross_scan_1b1(staging, y, B, C, H, W, elem_bytes, 4 * (int64_t)C * L, (int64_t)C * L, L, stream);
    return ss2d_cross_scan(staging, y, B, C, H, W, elem_bytes, stream);
}

}  // namespace ss2d

extern "C" int ss2d_cross_scan_flex_ws(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int x_channel_last,
                                       int y_channel_last, int one_by_one, int scans, void *workspace, int64_t workspace_bytes,
                                       void *stream) {
    using namespace ss2d;
    const int64_t need = cross_scan_staging_bytes(B, C, H, W, elem_bytes, x_channel_last, y_channel_last, one_by_one, scans);
    if (need < 0) return (int)need;
    if (need == 0) return ss2d_cross_scan_flex(x, y, B, C, H, W, elem_bytes, x_channel_last, y_channel_last, one_by_one, scans, stream);
    if (B == 0 || C == 0 || H == 0 || W == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0) return SS2D_EINVAL;
    if (workspace_bytes < need) return SS2D_ENOMEM;
    return cross_scan_flex_staged(x, y, B, C, H, W, elem_bytes, x_channel_last, y_channel_last, one_by_one, scans, workspace, stream);
}

// ---- the same with the library's own staging: an entry point that allocates nothing ---------------------------------
// For callers that cannot allocate (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc): the
// staging buffer is a fixed array in device memory that comes with the library's code object.  Every device that runs
// this library holds its own copy at its own address until the process ends; the address is looked up once per device.
namespace ss2d {

static __device__ __align__(256) unsigned char scratch[SS2D_STATIC_STAGING_BYTES];

constexpr int kMaxDevices = 64;
static std::mutex scratch_mutex;
static void *scratch_ptr[kMaxDevices];       // device address of `scratch` on device i; host code never uses the name itself

// The current device's copy of the array.  `scratch` in host code is only a handle for the runtime's symbol table, not
// a device address: kernels and copies get the pointer resolved here.
static int static_scratch(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) { (void)hipGetLastError(); return SS2D_ELAUNCH; }
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) { (void)hipGetLastError(); return SS2D_ELAUNCH; }
        scratch_ptr[dev] = ptr;
    }
    *out = scratch_ptr[dev];
    return SS2D_OK;
}

}  // namespace ss2d

extern "C" int ss2d_cross_scan_flex_static(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int x_channel_last,
                                           int y_channel_last, int one_by_one, int scans, void *stream) {
    using namespace ss2d;
    const int64_t need = cross_scan_staging_bytes(B, C, H, W, elem_bytes, x_channel_last, y_channel_last, one_by_one, scans);
    if (need < 0) return (int)need;
    if (need == 0) return ss2d_cross_scan_flex(x, y, B, C, H, W, elem_bytes, x_channel_last, y_channel_last, one_by_one, scans, stream);
    if (B == 0 || C == 0 || H == 0 || W == 0) return SS2D_OK;
    if (need > (int64_t)SS2D_STATIC_STAGING_BYTES) return SS2D_ENOMEM;
    if (!x || !y) return SS2D_EINVAL;
    void *staging = nullptr;
    const int rc = static_scratch(&staging);
    if (rc != SS2D_OK) return rc;
    // the transpose overwrites every byte the second launch reads: nothing of an earlier call's contents survives into
    // this one, so the array needs no clearing
    return cross_scan_flex_staged(x, y, B, C, H, W, elem_bytes, x_channel_last, y_channel_last, one_by_one, scans, staging, stream);
}
