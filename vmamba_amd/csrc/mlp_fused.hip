// Fused channel-last MLP of a VSS block (classification/models/vmamba.py:1116-1131 Mlp, :1229 the residual add):
//     out = residual + fc2(GELU(fc1(x)))          x (M, C), fc1 (4C x C) + bias, fc2 (C x 4C) + bias, 16-bit tensors
// in ONE kernel for the narrow stages (C = 96, 192), where the two library GEMMs, the GELU pass and the add are all
// bound by the (M, 4C) hidden tensor going to HBM and back three times.  Here the hidden activations never leave the
// registers:
//   * a wavefront owns 32 positions (kCT tiles of 32; measured at C = 96: one tile and three workgroups per CU beat
//     two tiles and two workgroups) and walks the hidden units in chunks of 32;
//   * GEMM 1 computes the chunk transposed, D1[hidden][position] = W1 chunk * x^T (v_mfma_f32_32x32x16, fp32
//     accumulate).  In the MFMA output layout a lane holds, for its position, hidden units 8g + 4*(lane/32) + t
//     (g, t = 0..3), accumulator 4g + t.  GEMM 2, D2[channel][position] += W2 chunk * h, contracts 16 hidden units per
//     instruction and a lane supplies 8 of them; the order of the contraction index is free as long as both operands
//     agree, so k-slot e of lane half kh in step s is DEFINED as hidden unit 16s + 8(e/4) + 4kh + e%4 -- which makes
//     accumulators 8s .. 8s+7 (after bias, GELU and rounding to 16 bits) the B fragment of step s with no data
//     movement between the two GEMMs.  The matching W2 fragment is two 8-byte runs of a row (one ds_read2_b64);
//   * the W1 / W2 chunks (2 x 6..12 KB) go from global memory straight into LDS (global_load_lds_dwordx4, no
//     registers in between), double-buffered, one barrier per chunk, the next chunk in flight during the whole of
//     the current one; x tiles come in and results go out through a wavefront-private LDS tile so that global loads and
//     stores are 16 bytes per lane along the channel axis; the residual is added on the way out.
// Rounding follows the unfused reference: fc1 output, GELU output and fc2 output are each rounded to the 16-bit type,
// then the residual add is rounded once more.  GELU is the exact (erf) form:
//   * bf16: the pre-activation is a bf16 value, so gelu(x) = 0.5 x + |x| E(|x|), E(x) = 0.5 erf(x / sqrt 2), with E read
//     from a 2176-entry fp32 table in LDS indexed by the bf16 bit pattern clamped to [2^-14, 8) (below, |x| E is under
//     1e-4 of 0.5 |x|; above, E is 0.5 to fp32 precision).  The table is generated in double precision at build time;
//   * fp16: erf from Abramowitz-Stegun 7.1.26 (absolute error 1.5e-7, far below 16-bit rounding).
#include "gelu.h"

namespace ss2d {

constexpr int kMlpChunk = 32;      // hidden units per chunk = one MFMA tile

// One global_load_lds_dwordx4: every lane fetches 16 bytes from its own address, the wavefront's 1 KB lands at
// lds_base + 16 * lane (lds_base wave-uniform).  Written as assembly so that the compiler does not order every later
// LDS read behind the outstanding load (it cannot tell the double buffers apart and waits for vmcnt(0) at the first
// LDS access after the issue, which puts the whole L2 latency on the critical path of every chunk); the waits are
// placed by hand instead: wait_loads_to_lds() before the barrier that publishes a buffer.
__device__ __forceinline__ void load_to_lds_16(const void *src, const void *lds_base) {
    const uint32_t base = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)lds_base);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void wait_loads_to_lds() { asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); }

struct MlpArgs {
    const void *x, *ln_w, *ln_b, *w1, *b1, *w2, *b2, *residual;
    void *out;
    int64_t M;
    float eps;
};

template <typename T, int C> struct MlpLayout {
    static constexpr bool kTable = ElemTraits<T>::dtype == SS2D_BF16;
    static constexpr int P1 = C + 8, P2 = kMlpChunk + 8, PS = C + 8;   // LDS row pitches (elements): rows stay 16-byte
                                                                       // aligned and 16 rows x 16 bytes cover all banks
    static constexpr int kW1Elems = kMlpChunk * P1, kW2Elems = C * P2, kBufElems = kW1Elems + kW2Elems;
    static constexpr int kStageElems = kMlpChunk * PS;                 // one 32-position tile per wavefront
    static constexpr size_t kBytes = (size_t)(2 * kBufElems + 5 * C + 2 * C) * sizeof(uint16_t) + (kTable ? kGeluEntries * sizeof(float) : 0);
};

template <typename T, int C, int kCT, bool kLN>
__global__ __launch_bounds__(kBlock, (kCT == 1 && C == 96 ? 3 : 2)) void mlp_fused_kernel(const MlpArgs p) {
    using Lay = MlpLayout<T, C>;
    constexpr int kHidden = 4 * C;
    constexpr int kChunks = kHidden / kMlpChunk;
    constexpr int kSteps1 = C / 16;                 // k-steps of GEMM 1
    constexpr int kOG = C / 32;                     // output-channel groups of GEMM 2
    constexpr int P1 = Lay::P1, P2 = Lay::P2, PS = Lay::PS;
    constexpr int kW1Elems = Lay::kW1Elems, kBufElems = Lay::kBufElems, kStageElems = Lay::kStageElems;
    constexpr int kWaves = kBlock / kWave;
    static_assert(2 * kBufElems >= kWaves * kStageElems, "the staging tiles alias the weight buffers");
    static_assert((2 * kBufElems + 5 * C) % 8 == 0 && C % 8 == 0, "LayerNorm vectors and the table start 16-byte aligned");
    extern __shared__ __align__(16) uint16_t mlp_smem[];
    uint16_t *wbuf = mlp_smem;                                      // [2][W1 chunk | W2 chunk]
    uint16_t *bias1 = mlp_smem + 2 * kBufElems;                     // [4C]
    uint16_t *bias2 = bias1 + kHidden;                              // [C]
    uint16_t *gamma_l = bias2 + C;                                  // [C] LayerNorm weight
    uint16_t *beta_l = gamma_l + C;                                 // [C] LayerNorm bias
    float *tbl = reinterpret_cast<float *>(beta_l + C);             // [kGeluEntries], bf16 only

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int j = lane & 31, kh = lane >> 5;
    uint16_t *stage = mlp_smem + wave * kStageElems;                // aliases wbuf: used before and after the chunk loop
    const T *x = reinterpret_cast<const T *>(p.x);
    const T *w1 = reinterpret_cast<const T *>(p.w1), *w2 = reinterpret_cast<const T *>(p.w2);
    const int64_t pos0 = ((int64_t)blockIdx.x * kWaves + wave) * (kCT * 32);   // first position of this wavefront

    // ---- weight chunks: global -> LDS directly (global_load_lds_dwordx4), one chunk ahead --------------------------------
    // A wavefront's load instruction writes 64 consecutive 16-byte pieces of LDS (piece = lane), each lane fetching from
    // its own global address; the buffer [W1 chunk | W2 chunk] is one run of pieces, the pad piece that ends every row
    // is filled from a valid address and never read.
    constexpr int kRow1 = P1 / 8, kRow2 = P2 / 8;                     // pieces per LDS row, pad included
    constexpr int kPieces1 = kMlpChunk * kRow1, kPiecesW = kPieces1 + C * kRow2;
    constexpr int kDmaIters = (kPiecesW + kBlock - 1) / kBlock;
    static_assert(kPiecesW % 32 == 0 && kBufElems == 8 * kPiecesW, "whole or half wavefronts of pieces");
    uint32_t w_off[kDmaIters];                                        // element offset of this lane's piece in chunk 0
    bool w_second[kDmaIters];                                         // the piece belongs to W2
#pragma unroll
    for (int it = 0; it < kDmaIters; ++it) {
        const int piece = (it * kWaves + wave) * kWave + lane;
        if (piece < kPieces1) {
            const int i = piece / kRow1, q = min(piece % kRow1, kRow1 - 2);
            w_off[it] = (uint32_t)(i * C + 8 * q); w_second[it] = false;
        } else {
            const int pp = min(piece, kPiecesW - 1) - kPieces1;
            const int o = pp / kRow2, q = min(pp % kRow2, kRow2 - 2);
            w_off[it] = (uint32_t)(o * kHidden + 8 * q); w_second[it] = true;
        }
    }
    auto fetch = [&](int chunk, int buf) {
#pragma unroll
        for (int it = 0; it < kDmaIters; ++it) {
            const int first = (it * kWaves + wave) * kWave;           // wave-uniform
            if (first + lane < kPiecesW) {
                const T *src = w_second[it] ? w2 + w_off[it] + chunk * kMlpChunk : w1 + w_off[it] + (size_t)chunk * kMlpChunk * C;
                load_to_lds_16(src, wbuf + buf * kBufElems + first * 8);
            }
        }
    };

    // ---- biases and the GELU table to LDS; x tiles -> fragments -------------------------------------------------------
    for (int i = threadIdx.x; i < kHidden; i += kBlock) bias1[i] = p.b1 ? reinterpret_cast<const uint16_t *>(p.b1)[i] : (uint16_t)0;
    for (int i = threadIdx.x; i < C; i += kBlock) bias2[i] = p.b2 ? reinterpret_cast<const uint16_t *>(p.b2)[i] : (uint16_t)0;
    if constexpr (kLN) {
        for (int i = threadIdx.x; i < C; i += kBlock) {
            gamma_l[i] = reinterpret_cast<const uint16_t *>(p.ln_w)[i];
            beta_l[i] = p.ln_b ? reinterpret_cast<const uint16_t *>(p.ln_b)[i] : (uint16_t)0;
        }
        __syncthreads();                                             // the tiles below read them
    }
    if constexpr (Lay::kTable)
        for (int i = threadIdx.x; i < kGeluEntries / 4; i += kBlock)
            reinterpret_cast<uint4 *>(tbl)[i] = reinterpret_cast<const uint4 *>(kGeluHalfErfBits)[i];
    u32x4_t xf[kCT][kSteps1];
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct) {
        constexpr int kPieces = 32 * C / 8;                          // 16-byte pieces of a 32 x C tile
#pragma unroll
        for (int it = 0; it < kPieces / kWave; ++it) {
            const int idx = lane + it * kWave;
            const int r = idx / (C / 8), q = idx % (C / 8);
            int64_t pos = pos0 + ct * 32 + r;
            pos = pos < p.M ? pos : p.M - 1;                         // rows past the end: any valid row, never stored
            *reinterpret_cast<uint4 *>(stage + r * PS + 8 * q) = *reinterpret_cast<const uint4 *>(x + pos * C + 8 * q);
        }
        wave_lds_sync();
        if constexpr (kLN) {
            layer_norm_tile_rows<T, C>(stage, PS, lane, gamma_l, beta_l, p.eps);
            wave_lds_sync();
        }
#pragma unroll
        for (int s = 0; s < kSteps1; ++s) xf[ct][s] = *reinterpret_cast<const u32x4_t *>(stage + j * PS + 16 * s + 8 * kh);
        wave_lds_sync();
    }
    __syncthreads();                                                 // staging aliases the weight buffers
    fetch(0, 0);
    wait_loads_to_lds();
    __syncthreads();

    floatx16_t acc2[kCT][kOG];
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
        for (int og = 0; og < kOG; ++og)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc2[ct][og][v] = 0.0f;

    for (int chunk = 0; chunk < kChunks; ++chunk) {
        if (chunk + 1 < kChunks) fetch(chunk + 1, (chunk + 1) & 1);
        const uint16_t *w1c = wbuf + (chunk & 1) * kBufElems, *w2c = w1c + kW1Elems;
        // GEMM 1: D1[hidden][position], one 32 x 32 tile per column tile
        floatx16_t acc1[kCT];
#pragma unroll
        for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc1[ct][v] = 0.0f;
#pragma unroll
        for (int s = 0; s < kSteps1; ++s) {
            const u32x4_t a = *reinterpret_cast<const u32x4_t *>(w1c + j * P1 + 16 * s + 8 * kh);
#pragma unroll
            for (int ct = 0; ct < kCT; ++ct) acc1[ct] = mfma_32x32x16(T{}, a, xf[ct][s], acc1[ct]);
        }
        // bias, rounding, GELU, rounding: accumulators 8s .. 8s+7 become the B fragment of GEMM 2's step s
        u32x4_t hf[kCT][2];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint2 bb = *reinterpret_cast<const uint2 *>(bias1 + chunk * kMlpChunk + 8 * g + 4 * kh);
            const float bv[4] = {unpack_lo<T>(bb.x), unpack_hi<T>(bb.x), unpack_lo<T>(bb.y), unpack_hi<T>(bb.y)};
#pragma unroll
            for (int ct = 0; ct < kCT; ++ct) {
                // fc1 output as a GEMM stores it (rounded), then GELU
                const uint32_t pre01 = pack2_from_f32<T>(acc1[ct][4 * g + 0] + bv[0], acc1[ct][4 * g + 1] + bv[1]);
                const uint32_t pre23 = pack2_from_f32<T>(acc1[ct][4 * g + 2] + bv[2], acc1[ct][4 * g + 3] + bv[3]);
                hf[ct][g >> 1][2 * (g & 1) + 0] = gelu_pair(T{}, pre01, tbl);
                hf[ct][g >> 1][2 * (g & 1) + 1] = gelu_pair(T{}, pre23, tbl);
            }
        }
        // GEMM 2: D2[channel][position] += W2[:, chunk] * h
#pragma unroll
        for (int og = 0; og < kOG; ++og)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const uint16_t *row = w2c + (og * 32 + j) * P2 + 16 * s + 4 * kh;     // units 16s+4kh.., 16s+8+4kh..
                const uint2 lo = *reinterpret_cast<const uint2 *>(row), hi = *reinterpret_cast<const uint2 *>(row + 8);
                const u32x4_t a = {lo.x, lo.y, hi.x, hi.y};
#pragma unroll
                for (int ct = 0; ct < kCT; ++ct) acc2[ct][og] = mfma_32x32x16(T{}, a, hf[ct][s], acc2[ct][og]);
            }
        wait_loads_to_lds();                                         // the next chunk, in flight since the top of this one
        __syncthreads();
    }

    // ---- out = residual + (acc2 + b2), through the wavefront's staging tile ------------------------------------------
    T *out = reinterpret_cast<T *>(p.out);
    const T *res = reinterpret_cast<const T *>(p.residual);
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct) {
#pragma unroll
        for (int og = 0; og < kOG; ++og)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int c0 = og * 32 + 8 * g + 4 * kh;             // accumulators 4g .. 4g+3: channels c0 .. c0+3
                const uint2 bb = *reinterpret_cast<const uint2 *>(bias2 + c0);
                *reinterpret_cast<uint2 *>(stage + j * PS + c0) =
                    make_uint2(pack2_from_f32<T>(acc2[ct][og][4 * g + 0] + unpack_lo<T>(bb.x), acc2[ct][og][4 * g + 1] + unpack_hi<T>(bb.x)),
                               pack2_from_f32<T>(acc2[ct][og][4 * g + 2] + unpack_lo<T>(bb.y), acc2[ct][og][4 * g + 3] + unpack_hi<T>(bb.y)));
            }
        wave_lds_sync();
        constexpr int kPieces = 32 * C / 8;
#pragma unroll
        for (int it = 0; it < kPieces / kWave; ++it) {
            const int idx = lane + it * kWave;
            const int r = idx / (C / 8), q = idx % (C / 8);
            const int64_t pos = pos0 + ct * 32 + r;
            if (pos < p.M) {
                uint4 v = *reinterpret_cast<const uint4 *>(stage + r * PS + 8 * q);
                if (res) {
                    const uint4 rv = *reinterpret_cast<const uint4 *>(res + pos * C + 8 * q);
                    uint32_t vw[4] = {v.x, v.y, v.z, v.w};
                    const uint32_t rw[4] = {rv.x, rv.y, rv.z, rv.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        vw[e] = pack2_from_f32<T>(unpack_lo<T>(vw[e]) + unpack_lo<T>(rw[e]), unpack_hi<T>(vw[e]) + unpack_hi<T>(rw[e]));
                    v = make_uint4(vw[0], vw[1], vw[2], vw[3]);
                }
                *reinterpret_cast<uint4 *>(out + pos * C + 8 * q) = v;
            }
        }
        wave_lds_sync();
    }
}

template <typename T, int C, int kCT>
static int launch_mlp(const MlpArgs &a, hipStream_t stream) {
    const size_t smem = MlpLayout<T, C>::kBytes;
    const int64_t per_wg = (int64_t)(kBlock / kWave) * kCT * 32;
    const int64_t n_wg = (a.M + per_wg - 1) / per_wg;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    if (a.ln_w) hipLaunchKernelGGL((mlp_fused_kernel<T, C, kCT, true>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, a);
    else hipLaunchKernelGGL((mlp_fused_kernel<T, C, kCT, false>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, a);
    return launch_status();
}

}  // namespace ss2d

extern "C" int ss2d_mlp_fused(const void *x, const void *ln_weight, const void *ln_bias, float eps, const void *w1,
                              const void *b1, const void *w2, const void *b2, const void *residual, void *out, int64_t M,
                              int C, int dtype, void *stream) {
    using namespace ss2d;
    if (M < 0 || C <= 0) return SS2D_EINVAL;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (M == 0) return SS2D_OK;
    if (!x || !w1 || !w2 || !out) return SS2D_EINVAL;
    if (ln_bias && !ln_weight) return SS2D_EINVAL;
    if (dtype == SS2D_F32 || (C != 96 && C != 192)) return SS2D_ENOTSUP;       // wider stages, fp32: the library GEMMs
    const void *ptrs[] = {x, ln_weight, ln_bias, w1, b1, w2, b2, residual, out};
    for (const void *q : ptrs)
        if (q && (reinterpret_cast<uintptr_t>(q) & 15u) != 0) return SS2D_ENOTSUP;
    MlpArgs a;
    a.x = x; a.ln_w = ln_weight; a.ln_b = ln_bias; a.eps = eps; a.w1 = w1; a.b1 = b1; a.w2 = w2; a.b2 = b2; a.residual = residual; a.out = out; a.M = M;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == SS2D_BF16) return C == 96 ? launch_mlp<bf16_t, 96, 1>(a, s) : launch_mlp<bf16_t, 192, 1>(a, s);
    return C == 96 ? launch_mlp<f16_t, 96, 1>(a, s) : launch_mlp<f16_t, 192, 1>(a, s);
}
