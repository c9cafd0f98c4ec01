// CrossScan (scans=0, channel-first): x (B,C,H,W) -> y (B,4,C,L), a pure permutation.
//
// HBM-bound: 1 read + 4 writes per element.  Directions 0/2 (row-major and its reversal) are
// written straight from the loaded registers; directions 1/3 (column-major and its reversal)
// go through an LDS transpose so that both the global read and the global writes are
// lane-contiguous.  LDS rows are padded to an odd pitch so the strided side is conflict-free.
//
// Two shapes of workgroup:
//   maps kernel  - small maps (<= kMapsLdsBytes): a workgroup takes G whole maps of one image;
//                  7x7 .. 90x90 feature maps land here.
//   tile kernel  - large maps: a workgroup takes one 64x64 tile of one map.
#include "ss2d_common.h"

namespace ss2d {

constexpr int kTile = 64;
constexpr int kTilePitch = kTile + 1;
constexpr int kMapsLdsBytes = 32 * 1024;   // per-workgroup LDS budget of the maps kernel
constexpr int kMapsTargetElems = 4096;     // elements a maps-workgroup aims to move per direction

// kVec elements travel per lane and memory instruction: 2 for 16-bit elements when L is even (a 4-byte lane
// access moves ~1.3x the bytes per second of a 2-byte one on this GPU), else 1.  kUnroll independent
// units are loaded before any is stored, so each thread keeps several requests in flight.
template <typename T, int kVec> struct PackOf { using type = T; };
template <> struct PackOf<uint16_t, 2> { using type = uint32_t; };

template <typename T, int kVec>
__device__ __forceinline__ T pack_get(typename PackOf<T, kVec>::type p, int i) {
    if constexpr (kVec == 1) return p;
    else return (T)(p >> (16 * i));
}
template <typename T, int kVec>
__device__ __forceinline__ typename PackOf<T, kVec>::type pack_reversed(typename PackOf<T, kVec>::type p) {
    if constexpr (kVec == 1) return p;
    else return (p >> 16) | (p << 16);
}

constexpr int kUnroll = 4;

// kStream: the four outputs leave as non-temporal stores.  Chosen by the host when they are more than the last-level cache
// holds (stage 1 of VMamba-T at batch 128, 308 MB: 81 -> 65 us); smaller outputs are better left where the next kernel
// finds them (154 MB: 33 us with ordinary stores, 51 with streaming ones).
constexpr int64_t kStreamOutputBytes = (int64_t)256 << 20;

template <typename T, int kVec, bool kStream>
__global__ __launch_bounds__(kBlock) void cross_scan_maps_kernel(const T *__restrict__ x, T *__restrict__ y, int C,
                                                                 int H, int W, int G, int groups_per_image,
                                                                 FastDiv divL, FastDiv divH, FastDiv divW, int Wp) {
    using pack_t = typename PackOf<T, kVec>::type;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *lds = reinterpret_cast<T *>(smem_raw);
    auto put = [](pack_t *dst, pack_t v) {
        if constexpr (kStream) store_streaming(dst, v);
        else *dst = v;
    };

    const uint32_t wg = blockIdx.x;
    const uint32_t b = wg / (uint32_t)groups_per_image;
    const uint32_t c0 = (wg - b * groups_per_image) * (uint32_t)G;
    const uint32_t g = min((uint32_t)G, (uint32_t)C - c0);
    const uint32_t L = divL.d;
    const uint32_t units = g * L / kVec;             // the host guarantees L % kVec == 0
    const uint32_t Lp = (uint32_t)H * (uint32_t)Wp;

    const size_t CL = (size_t)C * L;
    const T *xin = x + ((size_t)b * C + c0) * L;
    T *y0 = y + ((size_t)b * 4 + 0) * CL + (size_t)c0 * L;
    T *y1 = y0 + CL;
    T *y2 = y1 + CL;
    T *y3 = y2 + CL;
    const pack_t *xin_p = reinterpret_cast<const pack_t *>(xin);
    pack_t *y0_p = reinterpret_cast<pack_t *>(y0);
    pack_t *y1_p = reinterpret_cast<pack_t *>(y1);

    for (uint32_t base = threadIdx.x; base < units; base += kBlock * kUnroll) {
        pack_t v[kUnroll];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const uint32_t q = base + k * kBlock;
            if (q < units) v[k] = xin_p[q];
        }
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const uint32_t q = base + k * kBlock;
            if (q >= units) continue;
            uint32_t m, j, h, w;
            divmod(q * kVec, divL, m, j);
            divmod(j, divW, h, w);
            put(&y0_p[q], v[k]);
            put(reinterpret_cast<pack_t *>(y2 + m * L + (L - kVec - j)), pack_reversed<T, kVec>(v[k]));
#pragma unroll
            for (int i = 0; i < kVec; ++i) {
                lds[m * Lp + h * Wp + w] = pack_get<T, kVec>(v[k], i);
                if (++w == (uint32_t)W) { w = 0; ++h; }
            }
        }
    }
    __syncthreads();
    for (uint32_t base = threadIdx.x; base < units; base += kBlock * kUnroll) {
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const uint32_t q = base + k * kBlock;
            if (q >= units) continue;
            uint32_t m, t, h, w;
            divmod(q * kVec, divL, m, t);
            divmod(t, divH, w, h);          // t = w*H + h
            pack_t v;
            if constexpr (kVec == 1) {
                v = lds[m * Lp + h * Wp + w];
            } else {
                const uint32_t lo = lds[m * Lp + h * Wp + w];
                if (++h == (uint32_t)H) { h = 0; ++w; }
                const uint32_t hi = lds[m * Lp + h * Wp + w];
                v = lo | (hi << 16);
            }
            put(&y1_p[q], v);
            put(reinterpret_cast<pack_t *>(y3 + m * L + (L - kVec - t)), pack_reversed<T, kVec>(v));
        }
    }
}

// 16-bit maps with an ODD number of positions (7 x 7, 5 x 9 ...): single maps start on odd element offsets, but a group
// of an even number of maps is one block of memory that starts on a 4-byte boundary in x and in each of the four
// outputs (C even).  The block is read, kept in LDS and written as a flat stream of 4-byte pairs: output pair q of a
// direction is two consecutive scan positions (possibly the last of one map and the first of the next), each picked
// from the LDS copy through the direction's route.  Half the memory instructions of the element-wise variant.
__global__ __launch_bounds__(kBlock) void cross_scan_maps_flat_kernel(const uint16_t *__restrict__ x, uint16_t *__restrict__ y,
                                                                      int C, int H, int W, int G, int groups_per_image,
                                                                      FastDiv divL, FastDiv divH) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    uint16_t *lds = reinterpret_cast<uint16_t *>(smem_raw);      // the g maps as they lie in memory
    const uint32_t wg = blockIdx.x;
    const uint32_t b = wg / (uint32_t)groups_per_image;
    const uint32_t c0 = (wg - b * groups_per_image) * (uint32_t)G;
    const uint32_t g = min((uint32_t)G, (uint32_t)C - c0);
    const uint32_t L = divL.d, n = g * L, pairs = n / 2;         // an odd last element (odd g) is handled on its own
    const size_t CL = (size_t)C * L;
    const uint16_t *xin = x + ((size_t)b * C + c0) * L;
    uint16_t *y0 = y + ((size_t)b * 4) * CL + (size_t)c0 * L;
    const uint32_t *xin_p = reinterpret_cast<const uint32_t *>(xin);
    uint32_t *lds_p = reinterpret_cast<uint32_t *>(lds), *y0_p = reinterpret_cast<uint32_t *>(y0);
    for (uint32_t base = threadIdx.x; base < pairs; base += kBlock * kUnroll) {
        uint32_t v[kUnroll];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const uint32_t q = base + k * kBlock;
            if (q < pairs) v[k] = xin_p[q];
        }
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const uint32_t q = base + k * kBlock;
            if (q < pairs) { y0_p[q] = v[k]; lds_p[q] = v[k]; }
        }
    }
    if ((n & 1u) && threadIdx.x == 0) { const uint16_t v = xin[n - 1]; y0[n - 1] = v; lds[n - 1] = v; }
    __syncthreads();
    // source element (inside the block) of scan position t of map m, per direction
    auto src1 = [&](uint32_t m, uint32_t t) { uint32_t w, h; divmod(t, divH, w, h); return m * L + h * (uint32_t)W + w; };
    uint16_t *y1 = y0 + CL, *y2 = y1 + CL, *y3 = y2 + CL;
    for (uint32_t q = threadIdx.x; q < pairs; q += kBlock) {
        uint32_t m0, t0;
        divmod(2 * q, divL, m0, t0);
        const bool wrap = t0 + 1 == L;
        const uint32_t m1 = wrap ? m0 + 1 : m0, t1 = wrap ? 0 : t0 + 1;
        const uint32_t a1 = lds[src1(m0, t0)], b1 = lds[src1(m1, t1)];
        const uint32_t a2 = lds[m0 * L + (L - 1 - t0)], b2 = lds[m1 * L + (L - 1 - t1)];
        const uint32_t a3 = lds[src1(m0, L - 1 - t0)], b3 = lds[src1(m1, L - 1 - t1)];
        reinterpret_cast<uint32_t *>(y1)[q] = a1 | (b1 << 16);
        reinterpret_cast<uint32_t *>(y2)[q] = a2 | (b2 << 16);
        reinterpret_cast<uint32_t *>(y3)[q] = a3 | (b3 << 16);
    }
    if ((n & 1u) && threadIdx.x == 0) {
        const uint32_t m = g - 1, t = L - 1;
        y1[n - 1] = lds[src1(m, t)];
        y2[n - 1] = lds[m * L];
        y3[n - 1] = lds[src1(m, 0)];
    }
}

// The same flat stream in 16-byte vectors: with a multiple of 8 maps per workgroup (and C a multiple of 8, x and y 16-byte
// aligned) the block is a whole number of vectors on both sides.  A thread builds 8 consecutive scan positions of each
// direction: the column-major route of one map sits in a small LDS table (rt[t] = h W + w for t = w H + h), direction 3's
// source is its mirror image (L - 1 - rt[t]), direction 2's is L - 1 - t, and the walk steps over map ends by itself.  A
// quarter of the store instructions of the pair variant and a third of its index arithmetic.
__global__ __launch_bounds__(kBlock) void cross_scan_maps_flat8_kernel(const uint16_t *__restrict__ x, uint16_t *__restrict__ y,
                                                                       int C, int H, int W, int G, int groups_per_image,
                                                                       FastDiv divL, FastDiv divH) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    uint16_t *lds = reinterpret_cast<uint16_t *>(smem_raw);      // the g maps as they lie in memory
    const uint32_t L = divL.d;
    uint16_t *rt = lds + (size_t)G * L;                          // G L is a multiple of 8: the table starts 16-byte aligned
    const uint32_t wg = blockIdx.x;
    const uint32_t b = wg / (uint32_t)groups_per_image;
    const uint32_t c0 = (wg - b * groups_per_image) * (uint32_t)G;
    const uint32_t g = min((uint32_t)G, (uint32_t)C - c0);       // a multiple of 8 (C and G are)
    const uint32_t nv = g * L / 8;
    const size_t CL = (size_t)C * L;
    const uint4 *xin = reinterpret_cast<const uint4 *>(x + ((size_t)b * C + c0) * L);
    uint16_t *y0 = y + ((size_t)b * 4) * CL + (size_t)c0 * L;
    uint4 *lds4 = reinterpret_cast<uint4 *>(lds);
    uint4 *y0_4 = reinterpret_cast<uint4 *>(y0), *y1_4 = reinterpret_cast<uint4 *>(y0 + CL);
    uint4 *y2_4 = reinterpret_cast<uint4 *>(y0 + 2 * CL), *y3_4 = reinterpret_cast<uint4 *>(y0 + 3 * CL);
    for (uint32_t v = threadIdx.x; v < nv; v += kBlock) {
        const uint4 q = xin[v];
        y0_4[v] = q;
        lds4[v] = q;
    }
    if (threadIdx.x < L) {
        uint32_t w, h;
        divmod(threadIdx.x, divH, w, h);
        rt[threadIdx.x] = (uint16_t)(h * (uint32_t)W + w);
    }
    for (uint32_t t = kBlock + threadIdx.x; t < L; t += kBlock) {   // maps of more than 256 positions
        uint32_t w, h;
        divmod(t, divH, w, h);
        rt[t] = (uint16_t)(h * (uint32_t)W + w);
    }
    __syncthreads();
    for (uint32_t v = threadIdx.x; v < nv; v += kBlock) {
        uint32_t m, t;
        divmod(8 * v, divL, m, t);
        uint32_t base = m * L;
        uint32_t o1[4], o2[4], o3[4];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t s = rt[t];
            const uint32_t a1 = lds[base + s], a2 = lds[base + (L - 1 - t)], a3 = lds[base + (L - 1 - s)];
            if (i % 2 == 0) { o1[i / 2] = a1; o2[i / 2] = a2; o3[i / 2] = a3; }
            else { o1[i / 2] |= a1 << 16; o2[i / 2] |= a2 << 16; o3[i / 2] |= a3 << 16; }
            if (++t == L) { t = 0; base += L; }
        }
        y1_4[v] = make_uint4(o1[0], o1[1], o1[2], o1[3]);
        y2_4[v] = make_uint4(o2[0], o2[1], o2[2], o2[3]);
        y3_4[v] = make_uint4(o3[0], o3[1], o3[2], o3[3]);
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void cross_scan_tile_kernel(const T *__restrict__ x, T *__restrict__ y, int C,
                                                                 int H, int W, int tiles_h, int tiles_w) {
    __shared__ T lds[kTile * kTilePitch];
    const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    uint32_t wg = blockIdx.x;
    const uint32_t tw = wg % tiles_w; wg /= tiles_w;
    const uint32_t th = wg % tiles_h; wg /= tiles_h;
    const uint32_t c = wg % C, b = wg / C;
    const uint32_t h0 = th * kTile, w0 = tw * kTile;
    const size_t L = (size_t)H * W, CL = (size_t)C * L;

    const T *xm = x + ((size_t)b * C + c) * L;
    T *y0 = y + ((size_t)b * 4 + 0) * CL + (size_t)c * L;
    T *y1 = y0 + CL;
    T *y2 = y1 + CL;
    T *y3 = y2 + CL;

    for (uint32_t rr = wave; rr < kTile; rr += kBlock / kWave) {
        const uint32_t h = h0 + rr, w = w0 + lane;
        if (h < (uint32_t)H && w < (uint32_t)W) {
            const size_t r = (size_t)h * W + w;
            const T v = xm[r];
            lds[rr * kTilePitch + lane] = v;
            y0[r] = v;
            y2[L - 1 - r] = v;
        }
    }
    __syncthreads();
    for (uint32_t cc = wave; cc < kTile; cc += kBlock / kWave) {
        const uint32_t w = w0 + cc, h = h0 + lane;
        if (h < (uint32_t)H && w < (uint32_t)W) {
            const size_t t = (size_t)w * H + h;
            const T v = lds[lane * kTilePitch + cc];
            y1[t] = v;
            y3[L - 1 - t] = v;
        }
    }
}

template <typename T>
static int launch_cross_scan(const void *x, void *y, int B, int C, int H, int W, hipStream_t stream) {
    const int64_t L = (int64_t)H * W;
    const int Wp = W | 1;
    const int64_t map_lds = (int64_t)H * Wp * (int64_t)sizeof(T);
    if (map_lds <= kMapsLdsBytes) {
        int G = (int)((kMapsTargetElems + L - 1) / L);
        G = G < 1 ? 1 : G;
        G = G > C ? C : G;
        const int64_t cap = kMapsLdsBytes / map_lds;
        G = G > cap ? (int)cap : G;
        const int groups = (C + G - 1) / G;
        const int64_t n_wg = (int64_t)B * groups;
        if (n_wg > 0x7fffffff || (int64_t)G * L > 0x7fffffff) return SS2D_ENOTSUP;
        // 16-bit elements go two to a lane when every map starts on a 4-byte boundary
        bool pairs = false;
        if constexpr (sizeof(T) == 2) {
            pairs = (L % 2 == 0) && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) % 4 == 0);
        }
        if constexpr (sizeof(T) == 2) {
            // odd maps: an even number of maps per workgroup is a 4-byte aligned block on both sides
            const bool aligned4 = (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) % 4 == 0;
            // ... and a multiple of 8 maps of a multiple of 8 channels a block of whole 16-byte vectors
            const bool aligned16 = (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) % 16 == 0;
            if (L % 2 == 1 && C % 8 == 0 && aligned16 && G >= 8 && L <= 0xffff) {
                const int G8 = G & ~7;
                const int groups_8 = (C + G8 - 1) / G8;
                const int64_t n_wg_8 = (int64_t)B * groups_8;
                const size_t smem = (size_t)G8 * L * 2 + (((size_t)L * 2 + 15) & ~(size_t)15);
                if (n_wg_8 <= 0x7fffffff && smem <= 64 * 1024) {
                    hipLaunchKernelGGL(cross_scan_maps_flat8_kernel, dim3((uint32_t)n_wg_8), dim3(kBlock), smem, stream,
                                       (const uint16_t *)x, (uint16_t *)y, C, H, W, G8, groups_8, make_fastdiv((uint32_t)L),
                                       make_fastdiv((uint32_t)H));
                    return launch_status();
                }
            }
            if (L % 2 == 1 && C % 2 == 0 && aligned4 && G >= 2) {
                const int Gf = G & ~1;
                const int groups_f = (C + Gf - 1) / Gf;
                const int64_t n_wg_f = (int64_t)B * groups_f;
                if (n_wg_f <= 0x7fffffff) {
                    hipLaunchKernelGGL(cross_scan_maps_flat_kernel, dim3((uint32_t)n_wg_f), dim3(kBlock), (size_t)(Gf * L * 2 + 4), stream,
                                       (const uint16_t *)x, (uint16_t *)y, C, H, W, Gf, groups_f, make_fastdiv((uint32_t)L),
                                       make_fastdiv((uint32_t)H));
                    return launch_status();
                }
            }
        }
        const bool stream_out = 4 * (int64_t)B * C * L * (int64_t)sizeof(T) > kStreamOutputBytes;
#define SS2D_LAUNCH_MAPS(VEC, ST)                                                                                              \
    hipLaunchKernelGGL((cross_scan_maps_kernel<T, VEC, ST>), dim3((uint32_t)n_wg), dim3(kBlock), (size_t)(G * map_lds), stream, \
                       (const T *)x, (T *)y, C, H, W, G, groups, make_fastdiv((uint32_t)L), make_fastdiv((uint32_t)H),          \
                       make_fastdiv((uint32_t)W), Wp)
        if (pairs) {
            if constexpr (sizeof(T) == 2) {
                if (stream_out) SS2D_LAUNCH_MAPS(2, true); else SS2D_LAUNCH_MAPS(2, false);
            }
        } else {
            if (stream_out) SS2D_LAUNCH_MAPS(1, true); else SS2D_LAUNCH_MAPS(1, false);
        }
#undef SS2D_LAUNCH_MAPS
    } else {
        const int tiles_h = (H + kTile - 1) / kTile, tiles_w = (W + kTile - 1) / kTile;
        const int64_t n_wg = (int64_t)B * C * tiles_h * tiles_w;
        if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
        hipLaunchKernelGGL(cross_scan_tile_kernel<T>, dim3((uint32_t)n_wg), dim3(kBlock), 0, stream, (const T *)x,
                           (T *)y, C, H, W, tiles_h, tiles_w);
    }
    return launch_status();
}

}  // namespace ss2d

extern "C" int ss2d_cross_scan(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, void *stream) {
    using namespace ss2d;
    if (B < 0 || C < 0 || H < 0 || W < 0) return SS2D_EINVAL;
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return SS2D_EINVAL;
    if (B == 0 || C == 0 || H == 0 || W == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    if ((int64_t)H * W > 0x3fffffff) return SS2D_ENOTSUP;
    hipStream_t s = (hipStream_t)stream;
    switch (elem_bytes) {
        case 1: return launch_cross_scan<uint8_t>(x, y, B, C, H, W, s);
        case 2: return launch_cross_scan<uint16_t>(x, y, B, C, H, W, s);
        case 4: return launch_cross_scan<uint32_t>(x, y, B, C, H, W, s);
        default: return launch_cross_scan<uint64_t>(x, y, B, C, H, W, s);
    }
}
