// CrossMerge (scans=0, channel-first): ys (B,4,C,L) -> out (B,C,L), the summing inverse of
// CrossScan.  With r = h*W+w (row-major) and t = w*H+h (column-major):
//   pairwise order:       out[r] = (y0[r] + y2[L-1-r]) + (y1[t] + y3[L-1-t])
//   left-to-right order:  out[r] = ((y0[r] + y1[t]) + y2[L-1-r]) + y3[L-1-t]
// Each add is rounded to the tensor dtype (fp32 adds are exact IEEE adds; bf16/f16 adds are
// done in fp32 and rounded to nearest even), so the result is bit-identical to elementwise
// torch arithmetic in the same order.
//
// HBM-bound: 4 reads + 1 write per element.  The column-major operands are read
// lane-contiguously in THEIR order, combined, and transposed through LDS (odd pitch, so the
// strided writes are conflict-free); the row-major operands and the output are then
// lane-contiguous as well.  No strided global access anywhere.
#include "ss2d_common.h"

namespace ss2d {

constexpr int kMTile = 64;
constexpr int kMTilePitch = kMTile + 1;
constexpr int kMergeLdsBytes = 32 * 1024;
constexpr int kMergeTargetElems = 4096;

template <typename T> __device__ __forceinline__ T add_rn(T a, T b) { return from_f32<T>(to_f32(a) + to_f32(b)); }

// 16-bit elements travel two to a lane (one 4-byte access) when L is even; kUnroll independent units are
// loaded before any is combined, so each thread keeps several requests in flight.
template <typename T, int kVec> struct MergePack { using type = T; };
template <> struct MergePack<bf16_t, 2> { using type = uint32_t; };
template <> struct MergePack<f16_t, 2> { using type = uint32_t; };
template <> struct MergePack<float, 4> { using type = float4; };     // fp32 maps of 4n positions: 16 bytes to a lane

template <typename T, int kVec>
__device__ __forceinline__ T unit_get(typename MergePack<T, kVec>::type p, int i) {
    if constexpr (kVec == 1) return p;
    else if constexpr (kVec == 4) return i == 0 ? p.x : i == 1 ? p.y : i == 2 ? p.z : p.w;
    else return T{(uint16_t)(p >> (16 * i))};
}
template <typename T, int kVec>
__device__ __forceinline__ typename MergePack<T, kVec>::type unit_make(const T (&v)[kVec]) {
    if constexpr (kVec == 1) return v[0];
    else if constexpr (kVec == 4) return make_float4(v[0], v[1], v[2], v[3]);
    else return (uint32_t)v[0].bits | ((uint32_t)v[1].bits << 16);
}
// element i of the unit that sits REVERSED in memory
template <typename T, int kVec>
__device__ __forceinline__ T unit_get_reversed(typename MergePack<T, kVec>::type p, int i) {
    return unit_get<T, kVec>(p, kVec - 1 - i);
}

constexpr int kMergeUnroll = 4;

// kStream: operands and result as non-temporal accesses.  Chosen by the host when the four operands are more than the
// last-level cache holds (they are read once, the result is written once: stage 1, fp32, 616 MB: 150 -> 131 us alone,
// scan + merge 373 -> 352); smaller ones are found in the cache by ordinary loads (stage 3, 154 MB: 30 us against 36).
constexpr int64_t kStreamOperandBytes = (int64_t)256 << 20;

template <typename T, int kOrder, int kVec, bool kStream>
__global__ __launch_bounds__(kBlock) void cross_merge_maps_kernel(const T *__restrict__ ys, T *__restrict__ out, int C,
                                                                  int H, int W, int G, int groups_per_image,
                                                                  FastDiv divL, FastDiv divH, FastDiv divW, int Wp) {
    using unit_t = typename MergePack<T, kVec>::type;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *lds = reinterpret_cast<T *>(smem_raw);

    const uint32_t wg = blockIdx.x;
    const uint32_t b = wg / (uint32_t)groups_per_image;
    const uint32_t c0 = (wg - b * groups_per_image) * (uint32_t)G;
    const uint32_t g = min((uint32_t)G, (uint32_t)C - c0);
    const uint32_t L = divL.d;
    const uint32_t units = g * L / kVec;           // the host guarantees L % kVec == 0
    const uint32_t Lp = (uint32_t)H * (uint32_t)Wp;
    const uint32_t lds_dir = (uint32_t)G * Lp;     // second LDS plane (left-to-right order only)

    const size_t CL = (size_t)C * L;
    const T *y0 = ys + ((size_t)b * 4 + 0) * CL + (size_t)c0 * L;
    const T *y1 = y0 + CL;
    const T *y2 = y1 + CL;
    const T *y3 = y2 + CL;
    T *o = out + ((size_t)b * C + c0) * L;

    auto get = [](const unit_t *src) {
        if constexpr (kStream) return load_streaming(src);
        else return *src;
    };
    // column-major operands -> LDS, transposed
    for (uint32_t base = threadIdx.x; base < units; base += kBlock * kMergeUnroll) {
        unit_t a[kMergeUnroll], c[kMergeUnroll];
        uint32_t mm[kMergeUnroll], tt[kMergeUnroll];
#pragma unroll
        for (int k = 0; k < kMergeUnroll; ++k) {
            const uint32_t q = base + k * kBlock;
            if (q < units) {
                divmod(q * kVec, divL, mm[k], tt[k]);
                a[k] = get(reinterpret_cast<const unit_t *>(y1) + q);
                c[k] = get(reinterpret_cast<const unit_t *>(y3 + mm[k] * L + (L - kVec - tt[k])));
            }
        }
#pragma unroll
        for (int k = 0; k < kMergeUnroll; ++k) {
            const uint32_t q = base + k * kBlock;
            if (q >= units) continue;
            uint32_t w, h;
            divmod(tt[k], divH, w, h);
#pragma unroll
            for (int i = 0; i < kVec; ++i) {
                const T ai = unit_get<T, kVec>(a[k], i), ci = unit_get_reversed<T, kVec>(c[k], i);
                const uint32_t li = mm[k] * Lp + h * Wp + w;
                if (kOrder == SS2D_MERGE_PAIRWISE) {
                    lds[li] = add_rn(ai, ci);
                } else {
                    lds[li] = ai;
                    lds[lds_dir + li] = ci;
                }
                if (++h == (uint32_t)H) { h = 0; ++w; }
            }
        }
    }
    __syncthreads();
    // row-major operands + LDS -> out
    for (uint32_t base = threadIdx.x; base < units; base += kBlock * kMergeUnroll) {
        unit_t a[kMergeUnroll], c[kMergeUnroll];
        uint32_t mm[kMergeUnroll], rr[kMergeUnroll];
#pragma unroll
        for (int k = 0; k < kMergeUnroll; ++k) {
            const uint32_t q = base + k * kBlock;
            if (q < units) {
                divmod(q * kVec, divL, mm[k], rr[k]);
                a[k] = get(reinterpret_cast<const unit_t *>(y0) + q);
                c[k] = get(reinterpret_cast<const unit_t *>(y2 + mm[k] * L + (L - kVec - rr[k])));
            }
        }
#pragma unroll
        for (int k = 0; k < kMergeUnroll; ++k) {
            const uint32_t q = base + k * kBlock;
            if (q >= units) continue;
            uint32_t h, w;
            divmod(rr[k], divW, h, w);
            T res[kVec];
#pragma unroll
            for (int i = 0; i < kVec; ++i) {
                const T ai = unit_get<T, kVec>(a[k], i), ci = unit_get_reversed<T, kVec>(c[k], i);
                const uint32_t li = mm[k] * Lp + h * Wp + w;
                if (kOrder == SS2D_MERGE_PAIRWISE) {
                    res[i] = add_rn(add_rn(ai, ci), lds[li]);
                } else {
                    res[i] = add_rn(add_rn(add_rn(ai, lds[li]), ci), lds[lds_dir + li]);
                }
                if (++w == (uint32_t)W) { w = 0; ++h; }
            }
            if constexpr (kStream) store_streaming(reinterpret_cast<unit_t *>(o) + q, unit_make<T, kVec>(res));
            else reinterpret_cast<unit_t *>(o)[q] = unit_make<T, kVec>(res);
        }
    }
}

template <typename T, int kOrder, bool kStream>
__global__ __launch_bounds__(kBlock) void cross_merge_tile_kernel(const T *__restrict__ ys, T *__restrict__ out, int C,
                                                                  int H, int W, int tiles_h, int tiles_w) {
    __shared__ T lds[(kOrder == SS2D_MERGE_PAIRWISE ? 1 : 2) * kMTile * kMTilePitch];
    constexpr uint32_t kPlane = kMTile * kMTilePitch;
    const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    uint32_t wg = blockIdx.x;
    const uint32_t tw = wg % tiles_w; wg /= tiles_w;
    const uint32_t th = wg % tiles_h; wg /= tiles_h;
    const uint32_t c = wg % C, b = wg / C;
    const uint32_t h0 = th * kMTile, w0 = tw * kMTile;
    const size_t L = (size_t)H * W, CL = (size_t)C * L;

    const T *y0 = ys + ((size_t)b * 4 + 0) * CL + (size_t)c * L;
    const T *y1 = y0 + CL;
    const T *y2 = y1 + CL;
    const T *y3 = y2 + CL;
    T *o = out + ((size_t)b * C + c) * L;

    for (uint32_t cc = wave; cc < kMTile; cc += kBlock / kWave) {
        const uint32_t w = w0 + cc, h = h0 + lane;
        if (h < (uint32_t)H && w < (uint32_t)W) {
            const size_t t = (size_t)w * H + h;
            const T a = kStream ? load_streaming(y1 + t) : y1[t];
            const T d = kStream ? load_streaming(y3 + (L - 1 - t)) : y3[L - 1 - t];
            if (kOrder == SS2D_MERGE_PAIRWISE) {
                lds[lane * kMTilePitch + cc] = add_rn(a, d);
            } else {
                lds[lane * kMTilePitch + cc] = a;
                lds[kPlane + lane * kMTilePitch + cc] = d;
            }
        }
    }
    __syncthreads();
    for (uint32_t rr = wave; rr < kMTile; rr += kBlock / kWave) {
        const uint32_t h = h0 + rr, w = w0 + lane;
        if (h < (uint32_t)H && w < (uint32_t)W) {
            const size_t r = (size_t)h * W + w;
            const T a = kStream ? load_streaming(y0 + r) : y0[r];
            const T d = kStream ? load_streaming(y2 + (L - 1 - r)) : y2[L - 1 - r];
            const uint32_t li = rr * kMTilePitch + lane;
            if (kOrder == SS2D_MERGE_PAIRWISE) {
                o[r] = add_rn(add_rn(a, d), lds[li]);
            } else {
                o[r] = add_rn(add_rn(add_rn(a, lds[li]), d), lds[kPlane + li]);
            }
        }
    }
}

template <typename T, int kOrder>
static int launch_cross_merge(const void *ys, void *out, int B, int C, int H, int W, hipStream_t stream) {
    const int64_t L = (int64_t)H * W;
    const int Wp = W | 1;
    const int planes = kOrder == SS2D_MERGE_PAIRWISE ? 1 : 2;
    const int64_t map_lds = (int64_t)planes * H * Wp * (int64_t)sizeof(T);
    const bool stream_ops = 4 * (int64_t)B * C * L * (int64_t)sizeof(T) > kStreamOperandBytes;
    if (map_lds <= kMergeLdsBytes) {
        int G = (int)((kMergeTargetElems + L - 1) / L);
        G = G < 1 ? 1 : G;
        G = G > C ? C : G;
        const int64_t cap = kMergeLdsBytes / map_lds;
        G = G > cap ? (int)cap : G;
        const int groups = (C + G - 1) / G;
        const int64_t n_wg = (int64_t)B * groups;
        if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
        bool pairs = false;
        if constexpr (sizeof(T) == 2) {
            pairs = (L % 2 == 0) && ((reinterpret_cast<uintptr_t>(ys) | reinterpret_cast<uintptr_t>(out)) % 4 == 0);
        }
        bool quads = false;
        if constexpr (sizeof(T) == 4) {
            quads = (L % 4 == 0) && ((reinterpret_cast<uintptr_t>(ys) | reinterpret_cast<uintptr_t>(out)) % 16 == 0);
        }
#define SS2D_LAUNCH_MERGE_MAPS(VEC, ST)                                                                                        \
    hipLaunchKernelGGL((cross_merge_maps_kernel<T, kOrder, VEC, ST>), dim3((uint32_t)n_wg), dim3(kBlock), (size_t)(G * map_lds), \
                       stream, (const T *)ys, (T *)out, C, H, W, G, groups, make_fastdiv((uint32_t)L), make_fastdiv((uint32_t)H), \
                       make_fastdiv((uint32_t)W), Wp)
        if (quads) {
            if constexpr (sizeof(T) == 4) {
                if (stream_ops) SS2D_LAUNCH_MERGE_MAPS(4, true); else SS2D_LAUNCH_MERGE_MAPS(4, false);
            }
        } else if (pairs) {
            if constexpr (sizeof(T) == 2) {
                if (stream_ops) SS2D_LAUNCH_MERGE_MAPS(2, true); else SS2D_LAUNCH_MERGE_MAPS(2, false);
            }
        } else {
            if (stream_ops) SS2D_LAUNCH_MERGE_MAPS(1, true); else SS2D_LAUNCH_MERGE_MAPS(1, false);
        }
#undef SS2D_LAUNCH_MERGE_MAPS
    } else {
        const int tiles_h = (H + kMTile - 1) / kMTile, tiles_w = (W + kMTile - 1) / kMTile;
        const int64_t n_wg = (int64_t)B * C * tiles_h * tiles_w;
        if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
        if (stream_ops) {
            hipLaunchKernelGGL((cross_merge_tile_kernel<T, kOrder, true>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream,
                               (const T *)ys, (T *)out, C, H, W, tiles_h, tiles_w);
        } else {
            hipLaunchKernelGGL((cross_merge_tile_kernel<T, kOrder, false>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream,
                               (const T *)ys, (T *)out, C, H, W, tiles_h, tiles_w);
        }
    }
    return launch_status();
}

template <typename T>
static int dispatch_order(const void *ys, void *out, int B, int C, int H, int W, int order, hipStream_t s) {
    return order == SS2D_MERGE_PAIRWISE ? launch_cross_merge<T, SS2D_MERGE_PAIRWISE>(ys, out, B, C, H, W, s)
                                        : launch_cross_merge<T, SS2D_MERGE_LEFT_TO_RIGHT>(ys, out, B, C, H, W, s);
}

}  // namespace ss2d

extern "C" int ss2d_cross_merge(const void *ys, void *out, int B, int C, int H, int W, int dtype, int order,
                                void *stream) {
    using namespace ss2d;
    if (B < 0 || C < 0 || H < 0 || W < 0) return SS2D_EINVAL;
    if (order != SS2D_MERGE_PAIRWISE && order != SS2D_MERGE_LEFT_TO_RIGHT) return SS2D_EINVAL;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (B == 0 || C == 0 || H == 0 || W == 0) return SS2D_OK;
    if (!ys || !out) return SS2D_EINVAL;
    if ((int64_t)H * W > 0x3fffffff) return SS2D_ENOTSUP;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case SS2D_F32: return dispatch_order<float>(ys, out, B, C, H, W, order, s);
        case SS2D_BF16: return dispatch_order<bf16_t>(ys, out, B, C, H, W, order, s);
        default: return dispatch_order<f16_t>(ys, out, B, C, H, W, order, s);
    }
}
