// Global average pool of a channel-last map for gfx950: y[b, c] = mean over the L positions of x[b, :, c].
//
// The classifier head of the backbone pools the last stage's (B, 7, 7, 768) map (classification/models/vmamba.py:
// 1357-1363, AdaptiveAvgPool2d(1)).  The library's reduction kernel may split a reduction over several workgroups that
// meet through a counter it clears with a memset; this kernel needs neither: a workgroup owns one image and 256
// channels, eight groups of lanes each sum every eighth position of 8 channels (16-byte loads, fp32), and the eight
// partial sums meet in LDS and are added in a fixed order, so the result does not depend on scheduling.
// Result: fp32 sum times 1/L (fp32), rounded once to the tensor's type -- what mean() computes.
#include "ss2d_common.h"

namespace ss2d {

constexpr int kPoolSlices = 8;                          // position slices per workgroup
constexpr int kPoolGroups = kBlock / kPoolSlices;       // 32 groups of 8 channels = 256 channels per workgroup

template <typename T>
__global__ __launch_bounds__(kBlock) void mean_pool_cl_kernel(const T *__restrict__ x, T *__restrict__ y, int L, int C,
                                                              int ch_tiles, float inv_L) {
    __shared__ float part[kPoolSlices][kPoolGroups * 8 + 8];
    const int ct = blockIdx.x % ch_tiles, b = blockIdx.x / ch_tiles;
    const int grp = threadIdx.x % kPoolGroups, slice = threadIdx.x / kPoolGroups;
    const int c0 = (ct * kPoolGroups + grp) * 8;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    if (c0 < C) {
        const T *xb = x + (size_t)b * L * C + c0;
        // eight positions requested together (long maps would otherwise pay one memory latency per position), added
        // in position order
        constexpr int kAhead = 8;
        for (int l0 = slice; l0 < L; l0 += kAhead * kPoolSlices) {
            uint4 v[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const int l = min(l0 + u * kPoolSlices, L - 1);
                v[u] = *reinterpret_cast<const uint4 *>(xb + (size_t)l * C);
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                if (l0 + u * kPoolSlices < L) {
                    const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc[2 * i] += unpack_lo<T>(w[i]);
                        acc[2 * i + 1] += unpack_hi<T>(w[i]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[slice][grp * 8 + i] = acc[i];
    __syncthreads();
    // one lane per channel adds the eight slices in order
    const int c = ct * kPoolGroups * 8 + threadIdx.x;
    if (c < C) {
        float s = part[0][threadIdx.x];
#pragma unroll
        for (int k = 1; k < kPoolSlices; ++k) s += part[k][threadIdx.x];
        y[(size_t)b * C + c] = from_f32<T>(s * inv_L);
    }
}

}  // namespace ss2d

extern "C" int ss2d_mean_pool_cl(const void *x, void *y, int B, int L, int C, int dtype, void *stream) {
    using namespace ss2d;
    if (B < 0 || L <= 0 || C <= 0) return SS2D_EINVAL;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (B == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    if (dtype == SS2D_F32 || C % 8 != 0 || (reinterpret_cast<uintptr_t>(x) & 15u) != 0) return SS2D_ENOTSUP;
    const int ch_tiles = (C + kPoolGroups * 8 - 1) / (kPoolGroups * 8);
    const int64_t n_wg = (int64_t)B * ch_tiles;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    hipStream_t s = (hipStream_t)stream;
    const float inv_L = 1.0f / (float)L;
    if (dtype == SS2D_BF16) {
        hipLaunchKernelGGL((mean_pool_cl_kernel<bf16_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (const bf16_t *)x,
                           (bf16_t *)y, L, C, ch_tiles, inv_L);
    } else {
        hipLaunchKernelGGL((mean_pool_cl_kernel<f16_t>), dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (const f16_t *)x,
                           (f16_t *)y, L, C, ch_tiles, inv_L);
    }
    return launch_status();
}
