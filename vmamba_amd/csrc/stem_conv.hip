// First layer of the patch embedding in one kernel (classification/models/vmamba.py:1403-1411, patch-embed v2):
//     y = GELU(LayerNorm(conv2d(x, w, b; kernel 3, stride 2, padding 1)))
//     x (B, 3, H, W) NCHW, w (Cout, 3, 3, 3), y (B, Ho, Wo, Cout) channel-last, Cout = 48 or 64, 16-bit tensors.
// As separate operators the convolution output (the largest activation of the network, 4x the input) makes three
// round trips through HBM: written by the convolution, read and written by the LayerNorm, read and written by the
// GELU.  Here the input is read once and the activation written once.
//   * A workgroup owns TR output rows of one image.  The 2*TR + 1 input rows of the 3 channels go into LDS with
//     16-byte loads, behind 8 zero columns (and followed by 8) so that the padding needs no tests.
//   * The convolution is a 27-deep contraction per position: two k-steps of v_mfma_f32_32x32x16 with the weights as
//     the A operand (rows = output channels, k = (channel, tap row, tap column), zero beyond 27) and, as the B operand,
//     the 3x3x3 patch of the lane's position gathered from the LDS tile with 2-byte reads.  fp32 accumulation.
//   * In the accumulator layout lane (position j, half kh) holds channels 8g + 4kh + t of its position, so the
//     LayerNorm is a sum over the lane's values and one exchange with lane j + 32; bias, normalisation, GELU and the
//     16-bit roundings between them (convolution output, LayerNorm output, GELU output: what the separate operators
//     leave) happen in registers, and the result is stored as 8-byte runs of 4 channels.
#include "gelu.h"

namespace ss2d {

constexpr int kStemCin = 3, kStemTaps = 27;
constexpr int kStemPad = 8;            // zero columns in front of (and behind) every input row in LDS
constexpr int kStemWPitch = 40;        // LDS pitch of a weight row (32 k-slots + 8): 16-byte rows, banks spread

struct StemArgs {
    const void *x, *w, *b, *gamma, *beta;
    void *y;
    int32_t B, H, W, Ho, Wo, TR, tiles, vec;     // TR output rows per workgroup, tiles per image, 16-byte input loads
    int64_t ws_o, ws_c, ws_h, ws_w;              // weight strides (elements)
    float eps;
};

template <typename T, int kCout>
__global__ __launch_bounds__(kBlock) void stem_conv_ln_gelu_kernel(const StemArgs p, FastDiv divWo, FastDiv divTiles) {
    static_assert(kCout == 48 || kCout == 64, "one full and one partial or full tile of 32 output channels");
    constexpr bool kTable = ElemTraits<T>::dtype == SS2D_BF16;
    constexpr int kG1 = (kCout - 32) / 8;                      // channel groups of 8 in the second tile
    constexpr int kPerLane = 16 + 4 * kG1;                     // channels a lane holds of its position
    constexpr int kWaves = kBlock / kWave;
    extern __shared__ __align__(16) uint16_t st_smem[];
    const int Wp = p.W + 2 * kStemPad, rows_in = 2 * p.TR + 1;
    const int n_in = kStemCin * rows_in * Wp;                   // followed by 8 zeros (the k-slots beyond 27 read there)
    uint16_t *in_tile = st_smem;
    uint16_t *wl = in_tile + ((n_in + 8 + 7) & ~7);             // [64][kStemWPitch], 16-byte aligned
    float *prm = reinterpret_cast<float *>(wl + 64 * kStemWPitch);   // bias, gamma, beta: [3][kCout]
    float *tbl = prm + 3 * kCout;                               // [kGeluEntries], bf16 only

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int j = lane & 31, kh = lane >> 5;
    uint32_t b, tile_idx;
    divmod(blockIdx.x, divTiles, b, tile_idx);
    const int oh0 = (int)tile_idx * p.TR;
    const int tr = min(p.TR, p.Ho - oh0);
    const int ih0 = 2 * oh0 - 1;

    // ---- input rows -> LDS ---------------------------------------------------------------------------------------
    const T *xb = reinterpret_cast<const T *>(p.x) + (size_t)b * kStemCin * p.H * p.W;
    {
        const int ppr = Wp / 8;                                 // 16-byte pieces per LDS row (W % 8 == 0 when vec)
        if (p.vec) {
            for (int idx = threadIdx.x; idx < kStemCin * rows_in * ppr; idx += kBlock) {
                const int row = idx / ppr, q = idx - row * ppr;
                const int c = row / rows_in, r = row - c * rows_in;
                const int ih = ih0 + r, iw = 8 * q - kStemPad;
                uint4 v = make_uint4(0, 0, 0, 0);
                if (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W)
                    v = *reinterpret_cast<const uint4 *>(xb + ((size_t)c * p.H + ih) * p.W + iw);
                *reinterpret_cast<uint4 *>(in_tile + row * Wp + 8 * q) = v;
            }
        } else {
            for (int idx = threadIdx.x; idx < n_in; idx += kBlock) {
                const int row = idx / Wp, col = idx - row * Wp;
                const int c = row / rows_in, r = row - c * rows_in;
                const int ih = ih0 + r, iw = col - kStemPad;
                uint16_t v = 0;
                if (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W) v = xb[((size_t)c * p.H + ih) * p.W + iw].bits;
                in_tile[idx] = v;
            }
        }
        if (threadIdx.x < 8) in_tile[n_in + threadIdx.x] = 0;
    }
    // ---- weights [o][k], k = (c, tap row, tap column), zero for o >= kCout or k >= 27; bias / gamma / beta; table --------
    {
        const T *w = reinterpret_cast<const T *>(p.w);
        for (int idx = threadIdx.x; idx < 64 * 32; idx += kBlock) {
            const int o = idx >> 5, k = idx & 31;
            uint16_t v = 0;
            if (o < kCout && k < kStemTaps) {
                const int c = k / 9, t = k - 9 * c, th = t / 3, tw = t - 3 * th;
                v = w[o * p.ws_o + c * p.ws_c + th * p.ws_h + tw * p.ws_w].bits;
            }
            wl[o * kStemWPitch + k] = v;
        }
        for (int idx = threadIdx.x; idx < kCout; idx += kBlock) {
            prm[idx] = p.b ? to_f32(reinterpret_cast<const T *>(p.b)[idx]) : 0.0f;
            prm[kCout + idx] = p.gamma ? to_f32(reinterpret_cast<const T *>(p.gamma)[idx]) : 1.0f;
            prm[2 * kCout + idx] = p.beta ? to_f32(reinterpret_cast<const T *>(p.beta)[idx]) : 0.0f;
        }
        if constexpr (kTable)
            for (int idx = threadIdx.x; idx < kGeluEntries / 4; idx += kBlock)
                reinterpret_cast<uint4 *>(tbl)[idx] = reinterpret_cast<const uint4 *>(kGeluHalfErfBits)[idx];
    }
    __syncthreads();

    // weight fragments: lane (row j of tile mt, half kh) holds W[mt*32 + j][16 s + 8 kh .. + 7]
    u32x4_t wf[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int s = 0; s < 2; ++s) wf[mt][s] = *reinterpret_cast<const u32x4_t *>(wl + (mt * 32 + j) * kStemWPitch + 16 * s + 8 * kh);
    // where k-slot e of step s sits in the tile relative to the patch's first element, or -1 beyond the 27 taps
    int koff[2][8];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int k = 16 * s + 8 * kh + e;
            const int c = k / 9, t = k - 9 * c, th = t / 3, tw = t - 3 * th;
            koff[s][e] = k < kStemTaps ? (c * rows_in + th) * Wp + tw : -1;
        }
    // this lane's channels: value i < 16 is channel 8 (i/4) + 4 kh + i%4, value 16 + i is channel 32 + 8 (i/4) + 4 kh + i%4.
    // The bias rides in as the accumulators' initial value.
    floatx16_t bias_acc[2];
    float gamma_v[kPerLane], beta_v[kPerLane];
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const int ch = (i < 16 ? 0 : 32) + 8 * ((i & 15) / 4) + 4 * kh + (i & 3);
        bias_acc[i / 16][i & 15] = ch < kCout ? prm[ch] : 0.0f;
        if (i < kPerLane) { gamma_v[i] = prm[kCout + ch]; beta_v[i] = prm[2 * kCout + ch]; }
    }

    T *y = reinterpret_cast<T *>(p.y);
    const int n_pos = tr * p.Wo;
    for (int nt = wave; nt * 32 < n_pos; nt += kWaves) {
        const int n = nt * 32 + j;
        const bool valid = n < n_pos;
        uint32_t rl, ow;
        divmod((uint32_t)(valid ? n : 0), divWo, rl, ow);
        const int base = (2 * (int)rl) * Wp + 2 * (int)ow + kStemPad - 1;        // the patch's first element (tap 0,0 of channel 0)
        floatx16_t acc[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            uint32_t e[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) e[q] = in_tile[koff[s][q] < 0 ? n_in : base + koff[s][q]];
            const u32x4_t xf = {e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) acc[mt] = mfma_32x32x16(T{}, wf[mt][s], xf, s == 0 ? bias_acc[mt] : acc[mt]);
        }
        // convolution output as stored (bias included, rounded), LayerNorm over the position's kCout channels
        float v[kPerLane];
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < kPerLane; i += 2) {
            const uint32_t w2 = pack2_from_f32<T>(i < 16 ? acc[0][i] : acc[1][i - 16], i < 16 ? acc[0][i + 1] : acc[1][i - 15]);
            v[i] = unpack_lo<T>(w2); v[i + 1] = unpack_hi<T>(w2);
            sum += v[i] + v[i + 1];
        }
        sum += __shfl_xor(sum, 32);
        const float mean = sum * (1.0f / kCout);
        float sq = 0.0f;
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) { const float d = v[i] - mean; sq = fmaf(d, d, sq); }
        sq += __shfl_xor(sq, 32);
        const float rstd = __builtin_amdgcn_rsqf(sq * (1.0f / kCout) + p.eps);
        if (valid) {
            T *dst = y + (((size_t)b * p.Ho + oh0 + rl) * p.Wo + ow) * kCout;
#pragma unroll
            for (int g = 0; g < kPerLane / 4; ++g) {
                uint32_t o[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int i = 4 * g + 2 * h;
                    const uint32_t normed = pack2_from_f32<T>(fmaf((v[i] - mean) * rstd, gamma_v[i], beta_v[i]),
                                                              fmaf((v[i + 1] - mean) * rstd, gamma_v[i + 1], beta_v[i + 1]));
                    o[h] = gelu_pair(T{}, normed, tbl);
                }
                const int ch0 = (g < 4 ? 0 : 32) + 8 * (g & 3) + 4 * kh;
                *reinterpret_cast<uint2 *>(dst + ch0) = make_uint2(o[0], o[1]);
            }
        }
    }
}

template <typename T, int kCout>
static int launch_stem(StemArgs a, hipStream_t stream) {
    // output rows per workgroup: about 900 positions, the input rows within 40 KB of LDS
    int tr = 900 / a.Wo;
    tr = tr < 1 ? 1 : (tr > a.Ho ? a.Ho : tr);
    const int Wp = a.W + 2 * kStemPad;
    while (tr > 1 && (size_t)kStemCin * (2 * tr + 1) * Wp * 2 > 40 * 1024) --tr;
    a.TR = tr;
    a.tiles = (a.Ho + tr - 1) / tr;
    const size_t smem = ((((size_t)kStemCin * (2 * tr + 1) * Wp + 8 + 7) & ~(size_t)7) + 64 * kStemWPitch) * sizeof(uint16_t) + 3 * kCout * sizeof(float) +
                        (ElemTraits<T>::dtype == SS2D_BF16 ? kGeluEntries * sizeof(float) : 0);
    if (smem > 64 * 1024) return SS2D_ENOTSUP;
    const int64_t n_wg = (int64_t)a.B * a.tiles;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    hipLaunchKernelGGL((stem_conv_ln_gelu_kernel<T, kCout>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, a,
                       make_fastdiv((uint32_t)a.Wo), make_fastdiv((uint32_t)a.tiles));
    return launch_status();
}

}  // namespace ss2d

extern "C" int ss2d_stem_conv_ln_gelu(const void *x, const void *weight, const int64_t *weight_strides, const void *bias,
                                      const void *ln_weight, const void *ln_bias, float eps, void *y, int B, int H, int W,
                                      int Cout, int dtype, void *stream) {
    using namespace ss2d;
    if (B < 0 || H < 0 || W < 0 || Cout <= 0) return SS2D_EINVAL;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (B == 0 || H == 0 || W == 0) return SS2D_OK;
    if (!x || !weight || !weight_strides || !y) return SS2D_EINVAL;
    if (dtype == SS2D_F32 || (Cout != 48 && Cout != 64)) return SS2D_ENOTSUP;          // other shapes: the library operators
    if ((int64_t)kStemCin * H * W >= 0x7fffffffll || (reinterpret_cast<uintptr_t>(y) & 7u)) return SS2D_ENOTSUP;
    StemArgs a;
    a.x = x; a.w = weight; a.b = bias; a.gamma = ln_weight; a.beta = ln_bias; a.y = y;
    a.B = B; a.H = H; a.W = W; a.Ho = (H - 1) / 2 + 1; a.Wo = (W - 1) / 2 + 1; a.TR = 1; a.tiles = 1;
    a.vec = (W % 8 == 0) && (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    a.ws_o = weight_strides[0]; a.ws_c = weight_strides[1]; a.ws_h = weight_strides[2]; a.ws_w = weight_strides[3];
    a.eps = eps;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == SS2D_BF16) return Cout == 48 ? launch_stem<bf16_t, 48>(a, s) : launch_stem<bf16_t, 64>(a, s);
    return Cout == 48 ? launch_stem<f16_t, 48>(a, s) : launch_stem<f16_t, 64>(a, s);
}
