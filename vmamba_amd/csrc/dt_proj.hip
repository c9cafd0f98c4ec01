// dt_proj of the SS2D core (classification/models/vmamba.py:608-609 / :614-615): per direction k a tiny-K GEMM
//     delta[k, d, n] = sum_r W[k, d, r] * x[k, r, n],      d < D (96..768), r < R (6..48), n < N = batch * L,
// whose output is by far the largest tensor of the core (4*D values per position) while its inner dimension is
// only dt_rank.  It is bound by the HBM write of delta, and the memory pipeline prices a vector store by the
// instruction (about 16 cycles per wavefront instruction however few bytes it carries) and by the distinct lines
// it touches, so the kernel is built around full-width stores:
//   * one MFMA tile = 32 positions x 32 channels x 8 ranks (v_mfma_f32_32x32x8, bf16 or f16 operands, fp32
//     accumulate -- the arithmetic of the library GEMM it replaces: products of 16-bit values summed in fp32,
//     one rounding to the 16-bit output);
//   * a wavefront owns blocks of 64 consecutive positions.  The x rows of a block are fetched with 16-byte loads
//     into a wavefront-private LDS tile and read back as MFMA fragments; the results of two tiles (64 positions
//     x 32 channels) are parked in a second private LDS tile and written out as 16 bytes per lane, eight channels x
//     128 contiguous bytes per store instruction.  (Blocks of 128 positions -- 256-byte runs -- were slower at every
//     stage shape: the LDS tiles bound the resident wavefronts, and it is their number that hides each one's
//     load -> MFMA -> store latency.)
//   * the MFMA row index is mapped to positions through a permutation chosen so that a lane's 16 accumulators are
//     16 consecutive positions of one channel (two 16-byte LDS writes);
//   * the W fragments of up to 96 channels stay in registers for all blocks of the wavefront.
#include <string.h>

#include "ss2d_common.h"

namespace ss2d {

constexpr int kDtTile = 32;          // positions (and channels) per MFMA tile
constexpr int kDtTiles = 2;          // MFMA tiles per block
constexpr int kDtBlock = kDtTiles * kDtTile;   // positions per block
constexpr int kDtPitch = kDtBlock + 8;   // LDS row pitch in elements (144 bytes: 16-byte aligned, banks spread)
constexpr int kDtPieces = kDtBlock / 8;  // 16-byte pieces per row of a block
constexpr int kDtGroups = 3;         // channel groups of 32 per wavefront
constexpr int kDtMaxRank = 48;
constexpr uint32_t kDtOutOfRange = 0x7ffffff0u;   // byte offset beyond any buffer here (spans are checked < 2^31 - 16)

struct DtArgs {
    const void *x, *W;
    const void *mask;                    // optional (K, N) 16-bit words, 0 or 0xffff: where set, the output element is `fill`
    uint32_t fill2;                      // the fill value's 16 bits, twice
    void *out;
    int32_t K, D, R, d_chunks, blocks_per_wave, vec_ok, w_vec;
    int32_t stream_out;                  // delta larger than the last-level cache: non-temporal stores
    int64_t N, x_ks, x_rs, n_blocks, n_pos_chunks, total_waves;
    uint32_t x_span_bytes;
};

template <typename T, int kSteps>
__global__ __launch_bounds__(kBlock) void dt_proj_kernel(const DtArgs p) {
    extern __shared__ __align__(16) uint16_t dt_smem[];
    constexpr int kTiles = kDtTiles, kPieces = kDtPieces;
    constexpr int kRows = 8 * kSteps;                         // x rows held in LDS (rows >= R stay zero)
    constexpr int kWaveLds = (kRows + kDtTile) * kDtPitch;    // elements per wavefront: x tile + output tile
    const int lane = threadIdx.x & (kWave - 1);
    // readfirstlane: the wavefront index is uniform, which keeps everything derived from it in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int64_t wid = (int64_t)blockIdx.x * (kBlock / kWave) + wave;
    uint16_t *xs = dt_smem + wave * kWaveLds;                 // [kRows][kDtPitch]
    uint16_t *ob = xs + kRows * kDtPitch;                     // [32][kDtPitch]
    if (wid >= p.total_waves) return;
    const int64_t pos_chunk = wid % p.n_pos_chunks;
    const int64_t rest = wid / p.n_pos_chunks;
    const int dc = (int)(rest % p.d_chunks), k = (int)(rest / p.d_chunks);
    const int j = lane & 31, kh = lane >> 5;
    // this direction's x rows and W matrix behind buffer descriptors (32-bit byte offsets, host-checked spans)
    const T *x = reinterpret_cast<const T *>(p.x) + (int64_t)k * p.x_ks;
    const T *W = reinterpret_cast<const T *>(p.W) + (int64_t)k * p.D * p.R;
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(x), 0, (int)p.x_span_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t W_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(W), 0, p.D * p.R * 2, 0x00020000);
    T *out = reinterpret_cast<T *>(p.out) + (int64_t)k * p.D * p.N;
    const int d_base = dc * kDtGroups * kDtTile;

    // W fragments (MFMA columns = channels): lane (j, kh) holds W[d_base + 32 g + j][8 s + 4 kh .. + 3], zero outside
    // D x R.  Elements outside are pointed past the end of the buffer, where the hardware range check returns 0: the
    // loads stay unconditional and all fly together.
    uint32_t wf[kDtGroups][kSteps][2];
#pragma unroll
    for (int g = 0; g < kDtGroups; ++g) {
        const int d = d_base + g * kDtTile + j;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const int r0 = 8 * s + 4 * kh;
            if (p.w_vec) {                       // R % 4 == 0: the four ranks are one aligned 8-byte load
                const uint32_t off = (d < p.D && r0 < p.R) ? (uint32_t)(d * p.R + r0) * 2u : kDtOutOfRange;
                const auto t = __builtin_amdgcn_raw_buffer_load_b64(W_rsrc, (int)off, 0, 0);
                wf[g][s][0] = t[0];
                wf[g][s][1] = t[1];
            } else {
                uint32_t e[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t off = (d < p.D && r0 + q < p.R) ? (uint32_t)(d * p.R + r0 + q) * 2u : kDtOutOfRange;
                    e[q] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(W_rsrc, (int)off, 0, 0);
                }
                wf[g][s][0] = e[0] | (e[1] << 16);
                wf[g][s][1] = e[2] | (e[3] << 16);
            }
        }
    }
    // rows R .. kRows-1 of the x tile are never loaded: zero them once (W is zero there, but 0 * garbage may be NaN)
    for (int idx = lane; idx < (kRows - p.R) * kDtPitch; idx += kWave) xs[p.R * kDtPitch + idx] = 0;

    // MFMA row i of a tile <-> position 16*((i/4)%2) + 4*(i/8) + i%4: the 16 accumulators of lane (j, kh), rows
    // 8*(v/4) + 4*kh + v%4, are then positions 16*kh + v, v = 0..15
    const int p_in = 16 * ((j >> 2) & 1) + 4 * (j >> 3) + (j & 3);

    const int64_t block0 = pos_chunk * p.blocks_per_wave;
    const int64_t block1 = block0 + p.blocks_per_wave < p.n_blocks ? block0 + p.blocks_per_wave : p.n_blocks;
    const uint16_t *mask = p.mask ? reinterpret_cast<const uint16_t *>(p.mask) + (int64_t)k * p.N : nullptr;
    for (int64_t blk = block0; blk < block1; ++blk) {
        const int64_t n0 = blk * kDtBlock;
        // the mask words of this lane's 16-byte piece of the block (the same positions for every channel it stores)
        uint32_t mk[4] = {0u, 0u, 0u, 0u};
        if (mask) {                                                   // uniform
            const int64_t n = n0 + 8 * (lane % kPieces);
            if (p.vec_ok && n + 8 <= p.N) {
                const uint4 t = *reinterpret_cast<const uint4 *>(mask + n);
                mk[0] = t.x; mk[1] = t.y; mk[2] = t.z; mk[3] = t.w;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (n + e < p.N) mk[e / 2] |= (uint32_t)mask[n + e] << (16 * (e % 2));
            }
        }
        // ---- x rows of the block -> LDS: kPieces lanes x 16 bytes per row.  With 16-byte loads all of a lane's pieces
        // (one per 8 rows) are requested before the first is parked: one memory latency per block, not one per piece
        if (p.vec_ok) {
            uint4 v[kSteps];
#pragma unroll
            for (int it = 0; it < kSteps; ++it) {
                const int idx = lane + kWave * it, r = idx / kPieces, c = idx % kPieces;
                const int64_t n = n0 + 8 * c;
                const uint32_t off = (r < p.R && n < p.N) ? (uint32_t)(r * p.x_rs + n) * 2u : kDtOutOfRange;
                const auto t = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, 0);
                v[it] = make_uint4(t[0], t[1], t[2], t[3]);
            }
#pragma unroll
            for (int it = 0; it < kSteps; ++it) {
                const int idx = lane + kWave * it, r = idx / kPieces, c = idx % kPieces;
                if (r < p.R) *reinterpret_cast<uint4 *>(xs + r * kDtPitch + 8 * c) = v[it];
            }
        }
        for (int idx = lane; idx < (p.vec_ok ? 0 : p.R * kPieces); idx += kWave) {
            const int r = idx / kPieces, c = idx % kPieces;
            const int64_t n = n0 + 8 * c;
            uint4 v;
            if (p.vec_ok) {
                const uint32_t off = n < p.N ? (uint32_t)(r * p.x_rs + n) * 2u : kDtOutOfRange;
                const auto t = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, 0);
                v = make_uint4(t[0], t[1], t[2], t[3]);
            } else {
                uint32_t w[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t o0 = n + 2 * e < p.N ? (uint32_t)(r * p.x_rs + n + 2 * e) * 2u : kDtOutOfRange;
                    const uint32_t o1 = n + 2 * e + 1 < p.N ? (uint32_t)(r * p.x_rs + n + 2 * e + 1) * 2u : kDtOutOfRange;
                    const uint32_t lo = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(x_rsrc, (int)o0, 0, 0);
                    const uint32_t hi = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(x_rsrc, (int)o1, 0, 0);
                    w[e] = lo | (hi << 16);
                }
                v = make_uint4(w[0], w[1], w[2], w[3]);
            }
            *reinterpret_cast<uint4 *>(xs + r * kDtPitch + 8 * c) = v;
        }
        wave_lds_sync();
        // ---- x fragments of the tiles (MFMA rows = positions)
        uint32_t xf[kTiles][kSteps][2];
#pragma unroll
        for (int t = 0; t < kTiles; ++t)
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                const uint16_t *src = xs + (8 * s + 4 * kh) * kDtPitch + t * kDtTile + p_in;
                const uint32_t e0 = src[0], e1 = src[kDtPitch], e2 = src[2 * kDtPitch], e3 = src[3 * kDtPitch];
                xf[t][s][0] = e0 | (e1 << 16);
                xf[t][s][1] = e2 | (e3 << 16);
            }
#pragma unroll
        for (int g = 0; g < kDtGroups; ++g) {
            if (d_base + g * kDtTile < p.D) {                         // uniform over the wavefront
#pragma unroll
                for (int t = 0; t < kTiles; ++t) {
                    floatx16_t acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                    for (int s = 0; s < kSteps; ++s) acc = mfma_32x32x8(T{}, xf[t][s], wf[g][s], acc);
                    uint32_t w[8];
#pragma unroll
                    for (int v = 0; v < 8; ++v)
                        w[v] = pack2_from_f32<T>(acc[2 * v], acc[2 * v + 1]);
                    uint4 *dst = reinterpret_cast<uint4 *>(ob + j * kDtPitch + t * kDtTile + 16 * kh);
                    dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
                    dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
                }
                wave_lds_sync();
                // ---- 32 channels x kDtBlock positions out: lane -> (channel lane/kPieces + .., 16-byte piece lane%kPieces)
                constexpr int kChPerStore = kWave / kPieces;
#pragma unroll
                for (int it = 0; it < kDtTile / kChPerStore; ++it) {
                    const int ch = lane / kPieces + kChPerStore * it, c = lane % kPieces;
                    const int d = d_base + g * kDtTile + ch;
                    const int64_t n = n0 + 8 * c;
                    uint4 v = *reinterpret_cast<const uint4 *>(ob + ch * kDtPitch + 8 * c);
                    if (mask) {                                       // uniform
                        v.x = (v.x & ~mk[0]) | (p.fill2 & mk[0]); v.y = (v.y & ~mk[1]) | (p.fill2 & mk[1]);
                        v.z = (v.z & ~mk[2]) | (p.fill2 & mk[2]); v.w = (v.w & ~mk[3]) | (p.fill2 & mk[3]);
                    }
                    if (d < p.D) {
                        T *o = out + (int64_t)d * p.N + n;
                        if (p.vec_ok && n + 8 <= p.N) {
                            if (p.stream_out) store_streaming(reinterpret_cast<uint4 *>(o), v);     // uniform
                            else *reinterpret_cast<uint4 *>(o) = v;
                        } else {
                            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                if (n + e < p.N) o[e] = T{(uint16_t)(w[e / 2] >> (16 * (e % 2)))};
                        }
                    }
                }
                wave_lds_sync();
            }
        }
    }
}

template <typename T>
static int launch_dt_proj(DtArgs a, hipStream_t stream) {
    const int steps = (a.R + 7) / 8;
    const int64_t n_wg = (a.total_waves + (kBlock / kWave) - 1) / (kBlock / kWave);
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
#define SS2D_DT_LAUNCH(S)                                                                                          \
    hipLaunchKernelGGL((dt_proj_kernel<T, S>), dim3((uint32_t)n_wg), dim3(kBlock),                                 \
                       (size_t)(kBlock / kWave) * (8 * S + kDtTile) * kDtPitch * sizeof(uint16_t), stream, a)
    if (steps <= 1) SS2D_DT_LAUNCH(1);
    else if (steps == 2) SS2D_DT_LAUNCH(2);
    else if (steps == 3) SS2D_DT_LAUNCH(3);
    else if (steps == 4) SS2D_DT_LAUNCH(4);
    else SS2D_DT_LAUNCH(6);
#undef SS2D_DT_LAUNCH
    return launch_status();
}

}  // namespace ss2d

// The fill value as the 16 bits of the output type (round to nearest even; beyond the type's range: its infinity).
static uint32_t fill_bits16(float fill, int dtype) {
    if (dtype == SS2D_F16) {
        const _Float16 h = (_Float16)fill;
        uint16_t b;
        memcpy(&b, &h, 2);
        return b;
    }
    uint32_t u;
    memcpy(&u, &fill, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;   // NaN stays NaN
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

extern "C" int ss2d_dt_proj(const void *x, const void *weight, void *delta, int K, int D, int R, int64_t N,
                            int64_t x_dir_stride, int64_t x_rank_stride, int dtype, void *stream) {
    return ss2d_dt_proj_masked(x, weight, nullptr, 0.0f, delta, K, D, R, N, x_dir_stride, x_rank_stride, dtype, stream);
}

extern "C" int ss2d_dt_proj_masked(const void *x, const void *weight, const void *mask, float fill, void *delta, int K, int D,
                                   int R, int64_t N, int64_t x_dir_stride, int64_t x_rank_stride, int dtype, void *stream) {
    using namespace ss2d;
    if (K < 0 || D < 0 || R < 0 || N < 0 || x_dir_stride < 0 || x_rank_stride < 0) return SS2D_EINVAL;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (K == 0 || D == 0 || N == 0) return SS2D_OK;
    if (!x || !weight || !delta) return SS2D_EINVAL;
    if (dtype == SS2D_F32 || R > kDtMaxRank || R == 0) return SS2D_ENOTSUP;   // fp32 and wide ranks: the library GEMM
    DtArgs a;
    a.x = x; a.W = weight; a.out = delta;
    a.mask = mask; a.fill2 = fill_bits16(fill, dtype) * 0x10001u;
    a.K = K; a.D = D; a.R = R; a.N = N; a.x_ks = x_dir_stride; a.x_rs = x_rank_stride;
    a.d_chunks = (D + kDtGroups * kDtTile - 1) / (kDtGroups * kDtTile);
    a.n_blocks = (N + kDtBlock - 1) / kDtBlock;
    // enough wavefronts to fill the chip several times over, yet several blocks each so the W fragments are reused
    int64_t bpw = (int64_t)K * a.d_chunks * a.n_blocks / 8192;
    bpw = bpw < 1 ? 1 : (bpw > 4 ? 4 : bpw);
    a.blocks_per_wave = (int)bpw;
    a.n_pos_chunks = (a.n_blocks + bpw - 1) / bpw;
    a.total_waves = (int64_t)K * a.d_chunks * a.n_pos_chunks;
    const int64_t x_span = ((int64_t)(R - 1) * x_rank_stride + N) * 2;        // one direction's rows
    if (x_span >= 0x7ffffff0ll || (int64_t)D * R * 2 >= 0x7ffffff0ll) return SS2D_ENOTSUP;
    a.x_span_bytes = (uint32_t)x_span;
    a.w_vec = (R % 4 == 0) && (reinterpret_cast<uintptr_t>(weight) % 8 == 0);
    // 16-byte loads of x and stores of delta: rows and bases on 16-byte boundaries
    a.vec_ok = (N % 8 == 0) && (x_dir_stride % 8 == 0) && (x_rank_stride % 8 == 0) &&
               (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(delta) % 16 == 0) &&
               (reinterpret_cast<uintptr_t>(mask) % 16 == 0);
    // delta is written once and read by the next kernel: beyond what the last-level cache holds (256 MB) it leaves as
    // streaming stores (stage 1 of VMamba-T at batch 128, 308 MB: 71 -> 66 us, dt_proj + core 233 -> 224); smaller ones are
    // better left where the core finds them (154 MB: dt_proj + core 104 us against 106)
    a.stream_out = (int64_t)K * D * N * 2 > ((int64_t)256 << 20);
    hipStream_t s = (hipStream_t)stream;
    return dtype == SS2D_BF16 ? launch_dt_proj<bf16_t>(a, s) : launch_dt_proj<f16_t>(a, s);
}
