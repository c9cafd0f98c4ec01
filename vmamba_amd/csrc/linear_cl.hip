// Narrow channel-last projection with its neighbours folded in:
//     out = [LayerNorm](x) W^T + bias + residual        x (M, K), W (N, K), 16-bit tensors, K = N = 96
// -- the in_proj of a VSS block with the block's first LayerNorm in front (classification/models/vmamba.py:1225-1227,
// :648-650) and its out_proj with the residual add behind (:662, :1228).  At K = N = 96 these GEMMs move 154 MB for
// 7.4 GFLOP: they are bound by HBM, and the library kernels picked for them reach 1.5 TB/s.  Here the whole weight
// matrix (18 KB) sits in LDS, a wavefront owns 64 positions at a time, reads them with 16-byte loads into a private
// LDS tile (normalising the rows in place when asked to), takes matrix-core fragments from there
// (D[n][position] = W x^T, v_mfma_f32_32x32x16, fp32 accumulate) and sends the result back through the tile so that
// the stores and the residual loads are 16 bytes per lane as well.
// Rounding follows the separate operators: LayerNorm output, projection output (+ bias), and the sum with the
// residual are each rounded to the tensor type.  LayerNorm statistics are fp32 with the centred variance.
#include "ss2d_common.h"

namespace ss2d {

struct LinArgs {
    const void *x, *ln_w, *ln_b, *w, *bias, *residual;
    void *out;
    int64_t M;
    float eps;
    int tiles_per_wg;
    int L;                  // kCfIn: positions per image (a multiple of 32)
};

// kCfIn: x is the fp32 channel-first map (B, K, L) -- the merged output of the SS2D core -- and the LayerNorm (the
// block's out_norm, classification/models/vmamba.py:641-646) is computed from the fp32 values, as the separate
// operator does, before its result is rounded to T and multiplied.
template <typename T, int K, int N, int kCT, bool kLN, bool kCfIn = false>
__global__ __launch_bounds__(kBlock, 2) void linear_cl_kernel(const LinArgs p) {
    static_assert(!kCfIn || (kLN && K % 8 == 0), "the channel-first input path normalises");
    constexpr int kSteps = K / 16;                  // k-steps of the contraction
    constexpr int kOG = N / 32;                     // output-channel groups
    constexpr int PK = K + 8;                       // weight row pitch (elements): 16-byte rows, banks spread
    constexpr int kMaxKN = K > N ? K : N;
    constexpr int PS = kMaxKN + 8;                  // staging pitch
    constexpr int kWaves = kBlock / kWave;
    constexpr int kRowPieces = PK / 8, kPiecesW = N * kRowPieces;     // 16-byte pieces of the padded weight array
    static_assert(kPiecesW % 32 == 0, "whole or half wavefronts of pieces");
    extern __shared__ __align__(16) uint16_t lin_smem[];
    uint16_t *wl = lin_smem;                                        // [N][PK]
    uint16_t *stage_all = wl + N * PK;                              // [kWaves][32][PS]
    uint16_t *bias_l = stage_all + kWaves * 32 * PS;                // [N]
    uint16_t *gamma_l = bias_l + N;                                 // [K]
    uint16_t *beta_l = gamma_l + K;                                 // [K]

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int j = lane & 31, kh = lane >> 5;
    uint16_t *stage = stage_all + wave * 32 * PS;
    const T *x = reinterpret_cast<const T *>(p.x);
    const T *w = reinterpret_cast<const T *>(p.w);

    // ---- weights: global -> LDS directly; the pad piece that ends every row is filled from a valid address ---------
    constexpr int kDmaIters = (kPiecesW + kBlock - 1) / kBlock;
#pragma unroll
    for (int it = 0; it < kDmaIters; ++it) {
        const int first = (it * kWaves + wave) * kWave;              // wave-uniform
        if (first + lane < kPiecesW) {
            const int piece = first + lane;
            const int n = piece / kRowPieces, q = min(piece % kRowPieces, kRowPieces - 2);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(w + n * K + 8 * q),
                                             (__attribute__((address_space(3))) void *)(wl + first * 8), 16, 0, 0);
        }
    }
    for (int i = threadIdx.x; i < N; i += kBlock) bias_l[i] = p.bias ? reinterpret_cast<const uint16_t *>(p.bias)[i] : (uint16_t)0;
    if constexpr (kLN)
        for (int i = threadIdx.x; i < K; i += kBlock) {
            gamma_l[i] = reinterpret_cast<const uint16_t *>(p.ln_w)[i];
            beta_l[i] = p.ln_b ? reinterpret_cast<const uint16_t *>(p.ln_b)[i] : (uint16_t)0;
        }
    __syncthreads();

    T *out = reinterpret_cast<T *>(p.out);
    const T *res = reinterpret_cast<const T *>(p.residual);
    constexpr int kPiecesIn = 32 * K / 8, kPiecesOut = 32 * N / 8;     // 16-byte pieces of a 32-position tile
    for (int t = 0; t < p.tiles_per_wg; ++t) {
        const int64_t pos0 = (((int64_t)blockIdx.x * p.tiles_per_wg + t) * kWaves + wave) * (kCT * 32);
        if (pos0 >= p.M) break;                                      // wave-uniform; no workgroup barrier below
        u32x4_t xf[kCT][kSteps];
#pragma unroll
        for (int ct = 0; ct < kCT; ++ct) {
            if constexpr (kCfIn) {
                // 32 positions of one image (L % 32 == 0, M % 32 == 0): lane (channel group cs = lane / 8, quad = lane % 8)
                // loads positions 4 quad .. + 3 of channels cs, cs + 8, ..., 16 bytes each
                constexpr int kCPL = K / 8;
                const int64_t tpos = pos0 + ct * 32;
                const int64_t tb = (tpos < p.M ? tpos : 0) / p.L;
                const int l0 = (int)((tpos < p.M ? tpos : 0) - tb * p.L);
                const int cs = lane >> 3, quad = lane & 7;
                const float *src = reinterpret_cast<const float *>(p.x) + ((size_t)tb * K + cs) * p.L + l0 + 4 * quad;
                float4 v[kCPL];
                float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int i = 0; i < kCPL; ++i) {
                    v[i] = *reinterpret_cast<const float4 *>(src + (size_t)(8 * i) * p.L);
                    sum[0] += v[i].x; sum[1] += v[i].y; sum[2] += v[i].z; sum[3] += v[i].w;
                }
                float mean[4], sq[4] = {0.0f, 0.0f, 0.0f, 0.0f}, rstd[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sum[e] += __shfl_xor(sum[e], 8); sum[e] += __shfl_xor(sum[e], 16); sum[e] += __shfl_xor(sum[e], 32);
                    mean[e] = sum[e] * (1.0f / K);
                }
#pragma unroll
                for (int i = 0; i < kCPL; ++i) {
                    const float d0 = v[i].x - mean[0], d1 = v[i].y - mean[1], d2 = v[i].z - mean[2], d3 = v[i].w - mean[3];
                    sq[0] = fmaf(d0, d0, sq[0]); sq[1] = fmaf(d1, d1, sq[1]); sq[2] = fmaf(d2, d2, sq[2]); sq[3] = fmaf(d3, d3, sq[3]);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sq[e] += __shfl_xor(sq[e], 8); sq[e] += __shfl_xor(sq[e], 16); sq[e] += __shfl_xor(sq[e], 32);
                    rstd[e] = __builtin_amdgcn_rsqf(sq[e] * (1.0f / K) + p.eps);
                }
#pragma unroll
                for (int i = 0; i < kCPL; ++i) {
                    const int c = cs + 8 * i;
                    const float g = to_f32(T{gamma_l[c]}), bt = to_f32(T{beta_l[c]});
                    const float in[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
                    for (int e = 0; e < 4; e += 2) {                 // one conversion per pair of positions
                        const uint32_t two = pack2_from_f32<T>(fmaf((in[e] - mean[e]) * rstd[e], g, bt),
                                                               fmaf((in[e + 1] - mean[e + 1]) * rstd[e + 1], g, bt));
                        stage[(4 * quad + e) * PS + c] = (uint16_t)(two & 0xffffu);
                        stage[(4 * quad + e + 1) * PS + c] = (uint16_t)(two >> 16);
                    }
                }
                wave_lds_sync();
            } else {
#pragma unroll
                for (int it = 0; it < kPiecesIn / kWave; ++it) {
                    const int idx = lane + it * kWave;
                    const int r = idx / (K / 8), q = idx % (K / 8);
                    int64_t pos = pos0 + ct * 32 + r;
                    pos = pos < p.M ? pos : p.M - 1;                     // rows past the end: any valid row, never stored
                    *reinterpret_cast<uint4 *>(stage + r * PS + 8 * q) = *reinterpret_cast<const uint4 *>(x + pos * K + 8 * q);
                }
                wave_lds_sync();
                if constexpr (kLN) {
                    layer_norm_tile_rows<T, K>(stage, PS, lane, gamma_l, beta_l, p.eps);
                    wave_lds_sync();
                }
            }
#pragma unroll
            for (int s = 0; s < kSteps; ++s) xf[ct][s] = *reinterpret_cast<const u32x4_t *>(stage + j * PS + 16 * s + 8 * kh);
            wave_lds_sync();
        }
#pragma unroll
        for (int ct = 0; ct < kCT; ++ct) {
#pragma unroll
            for (int og = 0; og < kOG; ++og) {
                floatx16_t acc;
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
#pragma unroll
                for (int s = 0; s < kSteps; ++s) {
                    const u32x4_t a = *reinterpret_cast<const u32x4_t *>(wl + (og * 32 + j) * PK + 16 * s + 8 * kh);
                    acc = mfma_32x32x16(T{}, a, xf[ct][s], acc);
                }
                // lane (position j, half kh) holds channels og*32 + 8g + 4kh + t in accumulator 4g + t
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int c0 = og * 32 + 8 * g + 4 * kh;
                    const uint2 bb = *reinterpret_cast<const uint2 *>(bias_l + c0);
                    *reinterpret_cast<uint2 *>(stage + j * PS + c0) =
                        make_uint2(pack2_from_f32<T>(acc[4 * g + 0] + unpack_lo<T>(bb.x), acc[4 * g + 1] + unpack_hi<T>(bb.x)),
                                   pack2_from_f32<T>(acc[4 * g + 2] + unpack_lo<T>(bb.y), acc[4 * g + 3] + unpack_hi<T>(bb.y)));
                }
            }
            wave_lds_sync();
#pragma unroll
            for (int it = 0; it < kPiecesOut / kWave; ++it) {
                const int idx = lane + it * kWave;
                const int r = idx / (N / 8), q = idx % (N / 8);
                const int64_t pos = pos0 + ct * 32 + r;
                if (pos < p.M) {
                    uint4 v = *reinterpret_cast<const uint4 *>(stage + r * PS + 8 * q);
                    if (res) {
                        const uint4 rv = *reinterpret_cast<const uint4 *>(res + pos * N + 8 * q);
                        uint32_t vw[4] = {v.x, v.y, v.z, v.w};
                        const uint32_t rw[4] = {rv.x, rv.y, rv.z, rv.w};
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            vw[e] = pack2_from_f32<T>(unpack_lo<T>(vw[e]) + unpack_lo<T>(rw[e]), unpack_hi<T>(vw[e]) + unpack_hi<T>(rw[e]));
                        v = make_uint4(vw[0], vw[1], vw[2], vw[3]);
                    }
                    *reinterpret_cast<uint4 *>(out + pos * N + 8 * q) = v;
                }
            }
            wave_lds_sync();
        }
    }
}

template <typename T, int K, int N, int kCT, bool kCfIn = false>
static int launch_linear(LinArgs a, hipStream_t stream) {
    constexpr int kMaxKN = K > N ? K : N;
    const size_t smem = (size_t)(N * (K + 8) + (kBlock / kWave) * 32 * (kMaxKN + 8) + N + 2 * K) * sizeof(uint16_t);
    const int64_t per_tile = (int64_t)(kBlock / kWave) * kCT * 32;
    const int64_t tiles = (a.M + per_tile - 1) / per_tile;
    // a workgroup loads the weights once and then walks several tiles: about as many workgroups as fit the GPU at once
    int dev = 0, n_cu = 256;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        (void)hipGetLastError();
        n_cu = 256;
    }
    const int64_t slots = (int64_t)n_cu * (int64_t)((160 * 1024) / smem);
    const int64_t per_wg = (tiles + slots - 1) / slots;
    a.tiles_per_wg = (int)(per_wg < 1 ? 1 : per_wg > 64 ? 64 : per_wg);
    const int64_t n_wg = (tiles + a.tiles_per_wg - 1) / a.tiles_per_wg;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    if (smem > 64 * 1024) {
        const void *fn = kCfIn  ? reinterpret_cast<const void *>(&linear_cl_kernel<T, K, N, kCT, true, kCfIn>)
                       : a.ln_w ? reinterpret_cast<const void *>(&linear_cl_kernel<T, K, N, kCT, true>)
                                : reinterpret_cast<const void *>(&linear_cl_kernel<T, K, N, kCT, false>);
        if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
            (void)hipGetLastError();
            return SS2D_ENOTSUP;
        }
    }
    if constexpr (kCfIn) hipLaunchKernelGGL((linear_cl_kernel<T, K, N, kCT, true, true>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, a);
    else if (a.ln_w) hipLaunchKernelGGL((linear_cl_kernel<T, K, N, kCT, true>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, a);
    else hipLaunchKernelGGL((linear_cl_kernel<T, K, N, kCT, false>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, a);
    return launch_status();
}

}  // namespace ss2d

extern "C" int ss2d_linear_cl(const void *x, const void *ln_weight, const void *ln_bias, float eps, const void *weight,
                              const void *bias, const void *residual, void *out, int64_t M, int K, int N, int dtype,
                              void *stream) {
    using namespace ss2d;
    if (M < 0 || K <= 0 || N <= 0) return SS2D_EINVAL;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (M == 0) return SS2D_OK;
    if (!x || !weight || !out) return SS2D_EINVAL;
    if (ln_bias && !ln_weight) return SS2D_EINVAL;
    // other widths, fp32: the library GEMMs (measured at K = N = 192, where the weights take 77 KB of LDS and one
    // workgroup fits a CU: 47 us with the LayerNorm against 47 us for the two separate kernels -- not kept)
    if (dtype == SS2D_F32 || K != 96 || N != 96) return SS2D_ENOTSUP;
    const void *ptrs[] = {x, ln_weight, ln_bias, weight, bias, residual, out};
    for (const void *q : ptrs)
        if (q && (reinterpret_cast<uintptr_t>(q) & 15u) != 0) return SS2D_ENOTSUP;
    LinArgs a;
    a.x = x; a.ln_w = ln_weight; a.ln_b = ln_bias; a.w = weight; a.bias = bias; a.residual = residual; a.out = out;
    a.M = M; a.eps = eps; a.tiles_per_wg = 1; a.L = 0;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == SS2D_BF16) return launch_linear<bf16_t, 96, 96, 2>(a, s);
    return launch_linear<f16_t, 96, 96, 2>(a, s);
}

extern "C" int ss2d_linear_cf_ln(const void *x, const void *ln_weight, const void *ln_bias, float eps, const void *weight,
                                 const void *bias, const void *residual, void *out, int B, int L, int K, int N, int dtype,
                                 void *stream) {
    using namespace ss2d;
    if (B < 0 || L < 0 || K <= 0 || N <= 0) return SS2D_EINVAL;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (B == 0 || L == 0) return SS2D_OK;
    if (!x || !ln_weight || !weight || !out) return SS2D_EINVAL;
    if (dtype == SS2D_F32 || K != 96 || N != 96 || L % 32 != 0) return SS2D_ENOTSUP;
    const void *ptrs[] = {x, ln_weight, ln_bias, weight, bias, residual, out};
    for (const void *q : ptrs)
        if (q && (reinterpret_cast<uintptr_t>(q) & 15u) != 0) return SS2D_ENOTSUP;
    LinArgs a;
    a.x = x; a.ln_w = ln_weight; a.ln_b = ln_bias; a.w = weight; a.bias = bias; a.residual = residual; a.out = out;
    a.M = (int64_t)B * L; a.eps = eps; a.tiles_per_wg = 1; a.L = L;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == SS2D_BF16) return launch_linear<bf16_t, 96, 96, 2, true>(a, s);
    return launch_linear<f16_t, 96, 96, 2, true>(a, s);
}
