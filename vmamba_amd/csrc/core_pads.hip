// Maps whose sides do not suit the fused core's vector paths (57 x 58, 75 x 75, 19 x 19 ...) are embedded by the caller in a
// slightly larger map whose sides do: the added positions hold x = 0, and their step must be 0 so that they are neutral
// elements of the scan (decay exp(0 * A) = 1, drive 0 * B * u = 0: the state passes through them unchanged, exactly).  The
// core applies softplus to delta + bias, so a delta of -infinity there gives that step.  This kernel writes it: for each
// direction k, channel d and image b, delta[k, d, b, j] = -inf at the scan positions j of direction k that fall on added
// rows or columns -- direction orders as in cross_scan_fwd (classification/models/csm_triton.py:22-29) on the padded map.
#include "ss2d_common.h"

namespace ss2d {

template <typename T>
__global__ __launch_bounds__(kBlock) void core_mask_pads_kernel(T *__restrict__ delta, T fill, int D, int H, int W, int H8, int W8,
                                                                int64_t ks, int64_t ds, int64_t bs, FastDiv div_D,
                                                                FastDiv div_right, FastDiv div_W8) {
    uint32_t b, d;
    divmod(blockIdx.x, div_D, b, d);
    T *row = delta + (int64_t)d * ds + (int64_t)b * bs;
    const int right = W8 - W;                       // added columns
    const int n_right = H * right, n_all = n_right + (H8 - H) * W8;
    const int L8 = H8 * W8;
    for (int i = threadIdx.x; i < n_all; i += kBlock) {
        uint32_t h, w;
        if (i < n_right) {
            divmod((uint32_t)i, div_right, h, w);
            w += (uint32_t)W;
        } else {
            divmod((uint32_t)(i - n_right), div_W8, h, w);
            h += (uint32_t)H;
        }
        const int r = (int)(h * (uint32_t)W8 + w), t = (int)(w * (uint32_t)H8 + h);
        row[r] = fill;
        row[ks + t] = fill;
        row[2 * ks + (L8 - 1 - r)] = fill;
        row[3 * ks + (L8 - 1 - t)] = fill;
    }
}

}  // namespace ss2d

extern "C" int ss2d_core_mask_pads(void *delta, int batch, int dim, int height, int width, int padded_height, int padded_width,
                                   int64_t delta_dir_stride, int64_t delta_dim_stride, int64_t delta_batch_stride, int dtype,
                                   void *stream) {
    using namespace ss2d;
    if (batch < 0 || dim < 0 || height <= 0 || width <= 0 || padded_height < height || padded_width < width) return SS2D_EINVAL;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (delta_dir_stride < 0 || delta_dim_stride < 0 || delta_batch_stride < 0) return SS2D_EINVAL;
    if ((int64_t)padded_height * padded_width > 0x0fffffff) return SS2D_ENOTSUP;
    if (batch == 0 || dim == 0 || (padded_height == height && padded_width == width)) return SS2D_OK;
    if (!delta) return SS2D_EINVAL;
    const int64_t n_wg = (int64_t)batch * dim;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    const FastDiv dD = make_fastdiv((uint32_t)dim), dR = make_fastdiv((uint32_t)(padded_width > width ? padded_width - width : 1)),
                  dW = make_fastdiv((uint32_t)padded_width);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == SS2D_F32) {
        hipLaunchKernelGGL(core_mask_pads_kernel<uint32_t>, dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (uint32_t *)delta, 0xff800000u, dim,
                           height, width, padded_height, padded_width, delta_dir_stride, delta_dim_stride, delta_batch_stride, dD, dR, dW);
    } else {
        const uint16_t fill = dtype == SS2D_BF16 ? (uint16_t)0xff80u : (uint16_t)0xfc00u;
        hipLaunchKernelGGL(core_mask_pads_kernel<uint16_t>, dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (uint16_t *)delta, fill, dim, height,
                           width, padded_height, padded_width, delta_dir_stride, delta_dim_stride, delta_batch_stride, dD, dR, dW);
    }
    return launch_status();
}
