// Maps whose sides do not suit the fused core's vector paths (57 x 58, 75 x 75, 19 x 19 ...) are embedded by the caller in a
// slightly larger map whose sides do: the added positions hold x = 0, and their step must be 0 so that they are neutral
// elements of the scan (decay exp(0 * A) = 1, drive 0 * B * u = 0: the state passes through them unchanged, exactly).  The
// core applies softplus to delta + bias, so a delta of -infinity there gives that step.  This kernel writes it: for each
// direction k, channel d and image b, delta[k, d, b, j] = -inf at the scan positions j of direction k that fall on added
// rows or columns -- direction orders as in cross_scan_fwd (classification/models/csm_triton.py:22-29) on the padded map.
#include "ss2d_common.h"

namespace ss2d {

// One workgroup per (image, channel).  The added positions are enumerated twice, each time in the address order of a pair
// of directions: row-major for directions 0 / 2 (short runs at the row ends, then the added rows as one block) and
// column-major for 1 / 3 (short runs at the column ends, then the added columns as one block), so that consecutive
// threads write consecutive addresses wherever the runs are long.
template <typename T>
__global__ __launch_bounds__(kBlock) void core_mask_pads_kernel(T *__restrict__ delta, T fill, int D, int H, int W, int H8, int W8,
                                                                int64_t ks, int64_t ds, int64_t bs, FastDiv div_D,
                                                                FastDiv div_right, FastDiv div_W8, FastDiv div_below, FastDiv div_H8) {
    uint32_t b, d;
    divmod(blockIdx.x, div_D, b, d);
    T *row = delta + (int64_t)d * ds + (int64_t)b * bs;
    const int L8 = H8 * W8;
    const int n_all = L8 - H * W;
    // lines of `len` valid positions followed by `pitch - len` added ones (`lines` of them), then whole added lines
    auto walk = [&](T *fwd, T *bwd, int lines, int len, int pitch, const FastDiv &div_short, const FastDiv &div_pitch) {
        const int n_short = lines * (pitch - len);
        for (int i = threadIdx.x; i < n_all; i += kBlock) {
            uint32_t line, k;
            if (i < n_short) {
                divmod((uint32_t)i, div_short, line, k);
                k += (uint32_t)len;
            } else {
                divmod((uint32_t)(i - n_short), div_pitch, line, k);
                line += (uint32_t)lines;
            }
            const int j = (int)(line * (uint32_t)pitch + k);
            fwd[j] = fill;
            bwd[L8 - 1 - j] = fill;
        }
    };
    walk(row, row + 2 * ks, H, W, W8, div_right, div_W8);            // r = h W8 + w
    walk(row + ks, row + 3 * ks, W, H, H8, div_below, div_H8);      // t = w H8 + h
}

// Embeds maps in larger ones or cuts them out again: dst[m][r][c] = src[m][r][c] where the source has that row and
// column, 0 elsewhere -- n_maps maps of src_rows x src_cols resp. dst_rows x dst_cols units of sizeof(unit_t) bytes, both
// dense.  (A channel-last activation (B, H, W, D) is B maps of H rows of W * D elements.)  Fewer than 2^32 units.
template <typename unit_t>
__global__ __launch_bounds__(kBlock) void embed_units_kernel(const unit_t *__restrict__ src, unit_t *__restrict__ dst, uint32_t n_units,
                                                             int src_rows, int src_cols, FastDiv div_cols, FastDiv div_rows) {
    constexpr int kPer = 4;
    const uint32_t base = blockIdx.x * (uint32_t)(kPer * kBlock) + threadIdx.x;     // the grid covers the units exactly once
    unit_t v[kPer];
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        const uint32_t j = base + (uint32_t)(u * kBlock);
        v[u] = unit_t{};
        if (j < n_units && j >= base) {                                             // (no wrap-around at the top of the range)
            uint32_t line, c, m, r;
            divmod(j, div_cols, line, c);                                           // j = (m * dst_rows + r) * dst_cols + c
            divmod(line, div_rows, m, r);
            if (r < (uint32_t)src_rows && c < (uint32_t)src_cols) v[u] = src[((int64_t)m * src_rows + r) * src_cols + c];
        }
    }
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        const uint32_t j = base + (uint32_t)(u * kBlock);
        if (j < n_units && j >= base) dst[j] = v[u];
    }
}

// The same for rows that are no whole 16-byte vectors (75 x 75 16-bit maps into 80 x 80: source rows of 150 bytes; 19 x 19
// into 20 x 20: rows of 38 and 40 bytes): the destination is written as one flat stream of 16-byte vectors -- its total
// size is a multiple of the vector -- and each element of a vector is fetched on its own, the walk stepping over row and
// map ends by itself.
template <typename T>
__global__ __launch_bounds__(kBlock) void embed_gather_kernel(const T *__restrict__ src, T *__restrict__ dst, uint32_t n_vec, int src_rows,
                                                              int src_cols, int dst_rows, int dst_cols, FastDiv div_cols, FastDiv div_rows) {
    constexpr int kVec = 16 / (int)sizeof(T);
    struct alignas(16) Vec { T e[kVec]; };
    const uint32_t j = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    if (j >= n_vec) return;
    uint32_t line, c, m, r;
    divmod(j * (uint32_t)kVec, div_cols, line, c);
    divmod(line, div_rows, m, r);
    int64_t s_row = ((int64_t)m * src_rows + r) * src_cols;          // (read only where the source has the row)
    Vec v;
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
        v.e[i] = (r < (uint32_t)src_rows && c < (uint32_t)src_cols) ? src[s_row + c] : T{};
        if (++c == (uint32_t)dst_cols) {
            c = 0;
            if (++r == (uint32_t)dst_rows) { r = 0; ++m; }
            s_row = ((int64_t)m * src_rows + r) * src_cols;
        }
    }
    reinterpret_cast<Vec *>(dst)[j] = v;
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
                  dW = make_fastdiv((uint32_t)padded_width),
                  dB = make_fastdiv((uint32_t)(padded_height > height ? padded_height - height : 1)), dH = make_fastdiv((uint32_t)padded_height);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == SS2D_F32) {
        hipLaunchKernelGGL(core_mask_pads_kernel<uint32_t>, dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (uint32_t *)delta, 0xff800000u, dim,
                           height, width, padded_height, padded_width, delta_dir_stride, delta_dim_stride, delta_batch_stride, dD, dR, dW, dB, dH);
    } else {
        const uint16_t fill = dtype == SS2D_BF16 ? (uint16_t)0xff80u : (uint16_t)0xfc00u;
        hipLaunchKernelGGL(core_mask_pads_kernel<uint16_t>, dim3((uint32_t)n_wg), dim3(kBlock), 0, s, (uint16_t *)delta, fill, dim, height,
                           width, padded_height, padded_width, delta_dir_stride, delta_dim_stride, delta_batch_stride, dD, dR, dW, dB, dH);
    }
    return launch_status();
}

extern "C" int ss2d_core_embed_maps(const void *src, void *dst, int64_t n_maps, int src_rows, int64_t src_cols, int dst_rows,
                                    int64_t dst_cols, int elem_bytes, void *stream) {
    using namespace ss2d;
    if (n_maps < 0 || src_rows < 0 || src_cols < 0 || dst_rows < 0 || dst_cols < 0) return SS2D_EINVAL;
    if (elem_bytes != 2 && elem_bytes != 4) return SS2D_EINVAL;
    if (n_maps == 0 || dst_rows == 0 || dst_cols == 0) return SS2D_OK;
    if (!dst || !src) return SS2D_EINVAL;
    if (src_rows == 0 || src_cols == 0) return SS2D_EINVAL;                      // an empty source has no address to take
    if (src_cols > 0x7fffffff || dst_cols > 0x7fffffff) return SS2D_ENOTSUP;
    const int64_t n_elems = n_maps * (int64_t)dst_rows * dst_cols;
    if (n_elems > 0xffffffffll - 4 * kBlock || n_maps * (int64_t)src_rows * src_cols > 0xffffffffll) return SS2D_ENOTSUP;
    hipStream_t s = (hipStream_t)stream;
    const uintptr_t ps = reinterpret_cast<uintptr_t>(src), pd = reinterpret_cast<uintptr_t>(dst);
    if (ps % (uintptr_t)elem_bytes != 0 || pd % (uintptr_t)elem_bytes != 0) return SS2D_EINVAL;
    const int64_t sb = src_cols * elem_bytes, db = dst_cols * elem_bytes;      // row bytes
#define SS2D_EMBED_UNITS(UT, UB)                                                                                                   \
    do {                                                                                                                           \
        const uint32_t n_units = (uint32_t)(n_maps * (int64_t)dst_rows * (db / (UB)));                                             \
        const uint32_t grid = (n_units + 4 * kBlock - 1) / (4 * kBlock);                                                           \
        hipLaunchKernelGGL(embed_units_kernel<UT>, dim3(grid), dim3(kBlock), 0, s, (const UT *)src, (UT *)dst, n_units, src_rows,  \
                           (int)(sb / (UB)), make_fastdiv((uint32_t)(db / (UB))), make_fastdiv((uint32_t)dst_rows));               \
        return launch_status();                                                                                                    \
    } while (0)
    if (sb % 16 == 0 && db % 16 == 0 && ps % 16 == 0 && pd % 16 == 0) SS2D_EMBED_UNITS(uint4, 16);
    const int per_vec = 16 / elem_bytes;
    if (n_elems % per_vec == 0 && pd % 16 == 0) {
        const uint32_t n_vec = (uint32_t)(n_elems / per_vec);
        const uint32_t grid = (n_vec + kBlock - 1) / kBlock;
        const FastDiv dC = make_fastdiv((uint32_t)dst_cols), dR = make_fastdiv((uint32_t)dst_rows);
        if (elem_bytes == 2) {
            hipLaunchKernelGGL(embed_gather_kernel<uint16_t>, dim3(grid), dim3(kBlock), 0, s, (const uint16_t *)src, (uint16_t *)dst, n_vec,
                               src_rows, (int)src_cols, dst_rows, (int)dst_cols, dC, dR);
        } else {
            hipLaunchKernelGGL(embed_gather_kernel<uint32_t>, dim3(grid), dim3(kBlock), 0, s, (const uint32_t *)src, (uint32_t *)dst, n_vec,
                               src_rows, (int)src_cols, dst_rows, (int)dst_cols, dC, dR);
        }
        return launch_status();
    }
    if (sb % 4 == 0 && db % 4 == 0 && ps % 4 == 0 && pd % 4 == 0) SS2D_EMBED_UNITS(uint32_t, 4);
    if (elem_bytes == 4) return SS2D_EINVAL;                                     // (4-byte elements always take the branch above)
    SS2D_EMBED_UNITS(uint16_t, 2);
#undef SS2D_EMBED_UNITS
}
