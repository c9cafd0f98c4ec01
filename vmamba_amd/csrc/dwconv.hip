// Depthwise 3x3 convolution (+ bias) + SiLU: the step in front of the SS2D core
// (classification/models/vmamba.py:654-658: permute to channel-first, conv2d(groups=d_inner, k=3, pad=1), act).
//
//   x  (B,H,W,D) channel-last (the layout in_proj = nn.Linear produces) or (B,D,H,W) channel-first
//   w  (D,1,3,3), bias (D) or NULL
//   y  (B,D,H,W) channel-first, always: what CrossScan reads
//   y = silu(round(conv(x) + bias)), products and sums in fp32; the conv result is rounded to the tensor dtype
//   before SiLU because the reference runs conv2d and SiLU as two ops.
//
// HBM-bound (one read, one write).  The channel-last variant fuses the layout change: a workgroup owns 64
// consecutive positions x 32 channels; each lane convolves 8 channels at one position from nine 16-byte
// channel-vector loads (neighbouring positions re-use the same lines out of L1/L2), parks its results in LDS and
// the tile is written back transposed, 16 bytes per lane along the position axis.
#include "ss2d_common.h"

namespace ss2d {

constexpr int kDwPos = 64;           // positions per workgroup tile
constexpr int kDwCh = 32;            // channels per workgroup tile
constexpr int kDwPitch = kDwPos + 8; // LDS row pitch in elements: keeps 16-byte alignment, spreads banks

__device__ __forceinline__ float silu_f32(float v) { return v / (1.0f + expf(-v)); }
// SiLU for results that are rounded to a 16-bit type afterwards: the two hardware transcendentals (each good to one
// fp32 ulp) instead of the library expf and an IEEE division -- a quarter of the instructions, far below 16-bit
// rounding.  exp2 overflows to +inf for very negative v, where rcp gives 0 and the product -0: SiLU's limit.
__device__ __forceinline__ float silu_fast(float v) {
    return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v * -1.4426950408889634f));
}

template <typename T> __device__ __forceinline__ void unpack8(const uint4 raw, float (&v)[8]) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = to_f32(T{(uint16_t)(w[i] & 0xffffu)});
        v[2 * i + 1] = to_f32(T{(uint16_t)(w[i] >> 16)});
    }
}

// sum += a.lo * b.lo + a.hi * b.hi for dwords of two 16-bit values, fp32 accumulation: one instruction on the packed
// data as loaded (v_dot2c_f32_bf16 / v_dot2_f32_f16) instead of two widenings and two fused multiply-adds.
__device__ __forceinline__ float dot2_acc(bf16_t, uint32_t a, uint32_t b, float sum) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), sum, false);
}
__device__ __forceinline__ float dot2_acc(f16_t, uint32_t a, uint32_t b, float sum) {
    typedef _Float16 halfx2_t __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(halfx2_t, a), __builtin_bit_cast(halfx2_t, b), sum, false);
}
// (lo half of a, lo half of b) and (hi half of a, hi half of b) as new dwords: two taps of one channel side by side
__device__ __forceinline__ uint32_t pair_lo(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x05040100u); }
__device__ __forceinline__ uint32_t pair_hi(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }

// 16-bit element types, D % 8 == 0, 16-byte aligned tensors (host-checked).
template <typename T, bool kSilu>
__global__ __launch_bounds__(kBlock) void dwconv3x3_cl2cf_kernel(const T *__restrict__ x, const T *__restrict__ weight,
                                                                 const T *__restrict__ bias, T *__restrict__ y, int D,
                                                                 int H, int W, int pos_tiles, int ch_tiles, FastDiv divW) {
    __shared__ __align__(16) uint16_t tile[kDwCh * kDwPitch];
    uint32_t wg = blockIdx.x;
    const uint32_t ct = wg % ch_tiles; wg /= ch_tiles;
    const uint32_t pt = wg % pos_tiles;
    const uint32_t b = wg / pos_tiles;
    const int L = H * W;
    const int r0 = (int)pt * kDwPos;
    const int p = threadIdx.x / 4, cv = threadIdx.x % 4;
    const int c0 = (int)ct * kDwCh + cv * 8;            // this lane's 8 channels
    const int r = r0 + p;

    if (r < L && c0 < D) {
        uint32_t h, w;
        divmod((uint32_t)r, divW, h, w);
        // 72 weights of the 8 channels: 9 consecutive 16-byte vectors
        float wt[8][9];
        {
            const uint4 *wp = reinterpret_cast<const uint4 *>(weight + (size_t)c0 * 9);
            float flat[72];
#pragma unroll
            for (int k = 0; k < 9; ++k) {
                float t8[8];
                unpack8<T>(wp[k], t8);
#pragma unroll
                for (int i = 0; i < 8; ++i) flat[k * 8 + i] = t8[i];
            }
#pragma unroll
            for (int ci = 0; ci < 8; ++ci)
#pragma unroll
                for (int t = 0; t < 9; ++t) wt[ci][t] = flat[ci * 9 + t];
        }
        float acc[8];
#pragma unroll
        for (int ci = 0; ci < 8; ++ci) acc[ci] = 0.0f;
        const T *xb = x + (size_t)b * L * D;
#pragma unroll
        for (int kh = 0; kh < 3; ++kh) {
#pragma unroll
            for (int kw = 0; kw < 3; ++kw) {
                const int hh = (int)h + kh - 1, ww = (int)w + kw - 1;
                if (hh >= 0 && hh < H && ww >= 0 && ww < W) {
                    float xv[8];
                    unpack8<T>(*reinterpret_cast<const uint4 *>(xb + ((size_t)hh * W + ww) * D + c0), xv);
#pragma unroll
                    for (int ci = 0; ci < 8; ++ci) acc[ci] = fmaf(wt[ci][kh * 3 + kw], xv[ci], acc[ci]);
                }
            }
        }
        float bv[8];
        if (bias) unpack8<T>(*reinterpret_cast<const uint4 *>(bias + c0), bv);
#pragma unroll
        for (int ci = 0; ci < 8; ++ci) {
            float v = acc[ci] + (bias ? bv[ci] : 0.0f);
            T o = from_f32<T>(v);
            if (kSilu) o = from_f32<T>(silu_fast(to_f32(o)));
            tile[(cv * 8 + ci) * kDwPitch + p] = o.bits;
        }
    }
    __syncthreads();
    // write back: lane -> (channel = tid / 8, eight consecutive positions)
    const int c = threadIdx.x / 8, chunk = threadIdx.x % 8;
    const int cg = (int)ct * kDwCh + c;
    const int rr = r0 + chunk * 8;
    if (cg < D && rr < L) {
        T *yo = y + ((size_t)b * D + cg) * L + rr;
        const uint16_t *src = tile + c * kDwPitch + chunk * 8;
        if (rr + 8 <= L && (L % 8) == 0) {
            *reinterpret_cast<uint4 *>(yo) = *reinterpret_cast<const uint4 *>(src);
        } else {
            for (int i = 0; i < 8 && rr + i < L; ++i) yo[i] = T{src[i]};
        }
    }
}

// Row-tile variant of the same operation for images up to kDwMaxW wide: a workgroup owns TH full rows x 32 channels.
// The input rows (plus one halo row above and below and one zero column either side) are copied ONCE into LDS with
// 16-byte loads -- the nine taps then come out of LDS as contiguous 16-byte reads instead of nine trips through the
// vector memory pipeline, which is what bounds the kernel above.  Results are parked channel-major in a second LDS
// tile and written as 16 bytes per lane along the row-major positions, which are contiguous in (B,D,H,W).
constexpr int kDwMaxW = 128;

template <typename T, bool kSilu>
__global__ __launch_bounds__(kBlock) void dwconv3x3_rows_kernel(const T *__restrict__ x, const T *__restrict__ weight,
                                                                const T *__restrict__ bias, T *__restrict__ y, int D,
                                                                int H, int W, int TH, int row_tiles, int ch_tiles,
                                                                int out_pitch, int flat_out, FastDiv divW, FastDiv divWp,
                                                                FastDiv divL) {
    extern __shared__ __align__(16) uint16_t dw_smem[];
    const int Wp = W + 2;
    uint16_t *in_tile = dw_smem;                                 // [TH + 2][W + 2][32]
    uint16_t *out_tile = dw_smem + (TH + 2) * Wp * kDwCh;        // [32][out_pitch]
    uint32_t wg = blockIdx.x;
    const uint32_t ct = wg % ch_tiles; wg /= ch_tiles;
    const uint32_t rt = wg % row_tiles;
    const uint32_t b = wg / row_tiles;
    const int h0 = (int)rt * TH;
    const int rows = min(TH, H - h0);
    const int c_base = (int)ct * kDwCh;
    const int cv = threadIdx.x % 4;
    const int c0 = c_base + cv * 8;                              // this lane's 8 channels, in every phase
    const int rot = flat_out ? 0 : 16;                           // rotation of the output tile's rows per channel group

    // The 72 weights of the 8 channels (9 consecutive 16-byte vectors) and the bias: requested first, so that their
    // latency passes under the tile's loads.
    const int cw = min(c0, D - 8);                               // keep the loads in range; lanes with c0 >= D store nothing
    uint32_t wraw[36];
    {
        const uint16_t *wsrc = reinterpret_cast<const uint16_t *>(weight + (size_t)cw * 9);
#pragma unroll
        for (int k = 0; k < 9; ++k) {
            const uint4 v = reinterpret_cast<const uint4 *>(wsrc)[k];
            wraw[4 * k] = v.x; wraw[4 * k + 1] = v.y; wraw[4 * k + 2] = v.z; wraw[4 * k + 3] = v.w;
        }
    }
    float bv[8];
#pragma unroll
    for (int ci = 0; ci < 8; ++ci) bv[ci] = 0.0f;
    if (bias) unpack8<T>(*reinterpret_cast<const uint4 *>(bias + cw), bv);

    // ---- input rows h0-1 .. h0+rows into LDS; outside the image (and channels >= D) zeros.  The image sits behind a
    // buffer descriptor and pieces outside it are pointed past its end, where the hardware returns 0: the loads
    // are unconditional, so a thread's six are in flight together instead of one latency after the other.
    const T *xb = x + (size_t)b * H * W * D;
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(xb), 0, H * W * D * 2, 0x00020000);
    const int n_in = (rows + 2) * Wp;
    constexpr int kLoadsInFlight = 6;
    uint32_t step_r, step_c;                                     // (row, column) of a padded-tile element advance by this per load
    divmod((uint32_t)(kBlock / 4), divWp, step_r, step_c);
    for (int e0 = threadIdx.x / 4; e0 < n_in; e0 += kLoadsInFlight * (kBlock / 4)) {
        uint4 v[kLoadsInFlight];
        uint32_t rr, cc;
        divmod((uint32_t)e0, divWp, rr, cc);
#pragma unroll
        for (int u = 0; u < kLoadsInFlight; ++u) {
            const int e = e0 + u * (kBlock / 4);
            const int h = h0 - 1 + (int)rr, w = (int)cc - 1;
            const bool inside = e < n_in && h >= 0 && h < H && w >= 0 && w < W && c0 < D;
            const uint32_t off = inside ? (uint32_t)((h * W + w) * D + c0) * 2u : 0x7ffffff0u;
            const auto t = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, 0);
            v[u] = make_uint4(t[0], t[1], t[2], t[3]);
            rr += step_r; cc += step_c;
            if (cc >= (uint32_t)Wp) { cc -= (uint32_t)Wp; rr += 1; }
        }
#pragma unroll
        for (int u = 0; u < kLoadsInFlight; ++u) {
            const int e = e0 + u * (kBlock / 4);
            if (e < n_in) *reinterpret_cast<uint4 *>(in_tile + (size_t)e * kDwCh + cv * 8) = v[u];
        }
    }
    // The weights regrouped for the dot instruction: per channel four dwords holding taps (0,1) (2,3) (4,5) (6,7);
    // tap 8 as fp32.
    uint32_t wp2[8][4];
    float w8[8];
    {
        // element e = ci * 9 + t sits in half (e & 1) of dword e / 2: a pair of taps starting at an even element IS a
        // dword of the weights as loaded, one starting at an odd element straddles two (one funnel shift)
        auto pair_at = [&](int e) -> uint32_t {
            return (e & 1) ? __builtin_amdgcn_alignbit(wraw[e / 2 + 1], wraw[e / 2], 16) : wraw[e / 2];
        };
#pragma unroll
        for (int ci = 0; ci < 8; ++ci) {
#pragma unroll
            for (int tp = 0; tp < 4; ++tp) wp2[ci][tp] = pair_at(ci * 9 + 2 * tp);
            const int e8 = ci * 9 + 8;
            w8[ci] = (e8 & 1) ? unpack_hi<T>(wraw[e8 / 2]) : unpack_lo<T>(wraw[e8 / 2]);
        }
    }
    __syncthreads();

    // ---- nine taps per output from LDS
    const int n_out = rows * W;
    for (int pidx = threadIdx.x / 4; pidx < n_out; pidx += kBlock / 4) {
        uint32_t ph, pw;
        divmod((uint32_t)pidx, divW, ph, pw);
        // Column of this position in the rows of the output tile: the rows of channel group cv are rotated by 16 * cv
        // elements, so that the four groups of a wavefront write into different banks (their rows start a multiple
        // of 32 banks apart).
        int col = pidx + rot * cv;
        col = col >= out_pitch ? col - out_pitch : col;
        // nine taps as four pairs and a single: the two taps of a pair are brought side by side per channel (one byte
        // permute per channel pair and tap pair) and multiplied-accumulated by one dot instruction per channel
        uint4 tap[9];
#pragma unroll
        for (int kh = 0; kh < 3; ++kh)
#pragma unroll
            for (int kw = 0; kw < 3; ++kw)
                tap[kh * 3 + kw] = *reinterpret_cast<const uint4 *>(in_tile + ((size_t)(ph + kh) * Wp + pw + kw) * kDwCh + cv * 8);
        // tap 8 is single: one fused multiply-add on the widened value starts each accumulator from the bias
        float acc[8];
        {
            const uint32_t a[4] = {tap[8].x, tap[8].y, tap[8].z, tap[8].w};
#pragma unroll
            for (int cp = 0; cp < 4; ++cp) {
                acc[2 * cp] = fmaf(unpack_lo<T>(a[cp]), w8[2 * cp], bv[2 * cp]);
                acc[2 * cp + 1] = fmaf(unpack_hi<T>(a[cp]), w8[2 * cp + 1], bv[2 * cp + 1]);
            }
        }
#pragma unroll
        for (int tp = 0; tp < 4; ++tp) {
            const uint32_t a[4] = {tap[2 * tp].x, tap[2 * tp].y, tap[2 * tp].z, tap[2 * tp].w};
            const uint32_t b[4] = {tap[2 * tp + 1].x, tap[2 * tp + 1].y, tap[2 * tp + 1].z, tap[2 * tp + 1].w};
#pragma unroll
            for (int cp = 0; cp < 4; ++cp) {
                acc[2 * cp] = dot2_acc(T{}, pair_lo(a[cp], b[cp]), wp2[2 * cp][tp], acc[2 * cp]);
                acc[2 * cp + 1] = dot2_acc(T{}, pair_hi(a[cp], b[cp]), wp2[2 * cp + 1][tp], acc[2 * cp + 1]);
            }
        }
#pragma unroll
        for (int ci = 0; ci < 8; ci += 2) {
            uint32_t o = pack2_from_f32<T>(acc[ci], acc[ci + 1]);                                  // conv output as stored
            if (kSilu) o = pack2_from_f32<T>(silu_fast(unpack_lo<T>(o)), silu_fast(unpack_hi<T>(o)));
            out_tile[(cv * 8 + ci) * out_pitch + col] = (uint16_t)(o & 0xffffu);
            out_tile[(cv * 8 + ci + 1) * out_pitch + col] = (uint16_t)(o >> 16);
        }
    }
    __syncthreads();

    // ---- write back: the tile's positions are contiguous per channel in (B, D, H, W)
    const int L = H * W;
    if (flat_out) {
        // A whole image per workgroup: its 32 channel rows are ONE contiguous block of y that starts on a 16-byte
        // boundary whatever L is (32 * L elements).  16 bytes per lane over the block; a piece may run from one
        // channel row into the next, so its elements are picked out of the tile one by one.
        uint4 *dst = reinterpret_cast<uint4 *>(y + ((size_t)b * D + c_base) * L);
        for (int pc = threadIdx.x; pc < kDwCh * L / 8; pc += kBlock) {
            uint32_t c, pos;
            divmod((uint32_t)pc * 8u, divL, c, pos);
            // L >= 8 (host-checked): at most one row boundary inside a piece
            const int n_first = min(8, L - (int)pos);
            const uint16_t *row0 = out_tile + c * out_pitch + pos, *row1 = out_tile + (c + 1) * out_pitch - n_first;
            uint32_t e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = (i < n_first ? row0 : row1)[i];
            dst[pc] = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
        }
        return;
    }
    const int pieces = (n_out + 7) / 8;
    const bool vec = ((h0 * W) % 8 == 0) && (L % 8 == 0);
    // a group of 8, 16 or 32 lanes per channel (the smallest that covers the tile), a lane per piece of 8 positions: no
    // division, and short tiles keep most lanes busy (tiles hold at most 256 positions)
    const int lg = pieces <= 8 ? 3 : pieces <= 16 ? 4 : 5;
    const int piece = threadIdx.x & ((1 << lg) - 1), c_first = threadIdx.x >> lg, c_step = kBlock >> lg;
    if (piece < pieces) {
        T *yo = y + ((size_t)b * D + c_base + c_first) * L + (size_t)h0 * W + piece * 8;
        const bool whole = vec && piece * 8 + 8 <= n_out;
        for (int c = c_first; c < kDwCh; c += c_step) {
            if (c_base + c < D) {
                int col = piece * 8 + 16 * (c / 8);                  // the row's rotation (see above); pieces stay whole
                col = col >= out_pitch ? col - out_pitch : col;
                const uint16_t *src = out_tile + c * out_pitch + col;
                if (whole) {
                    *reinterpret_cast<uint4 *>(yo) = *reinterpret_cast<const uint4 *>(src);
                } else {
                    for (int i = 0; i < 8 && piece * 8 + i < n_out; ++i) yo[i] = T{src[i]};
                }
            }
            yo += (size_t)c_step * L;
        }
    }
}

// Plane variant of the channel-last kernel: the layout change happens on the way INTO LDS instead of on the way out.
// A workgroup owns TH full rows x kCh channels (32 or 64, i.e. runs of 64 or 128 bytes per position).  The input rows
// (with halo) are fetched as 16-byte channel vectors, two neighbouring positions per lane, and written into one LDS plane
// per channel as dwords holding TWO NEIGHBOURING POSITIONS of that channel (one byte permute per channel and pair):
// a plane is the zero-padded image rows of one channel, [TH + 2][pitch], padded column 0 = image column -1.
// In the compute phase a lane owns one channel and segments of 8 consecutive outputs of a row.  With the taps of a
// row in dwords D_i = (p[8s + 2i], p[8s + 2i + 1]) an output needs two dot instructions per filter row and no data
// movement at all:
//   even output 2i:  (p[2i], p[2i+1]) . (k0, k1) + (p[2i+2], p[2i+3]) . (k2, 0)  = D_i . P0 + D_i+1 . P1
//   odd output 2i+1: (p[2i], p[2i+1]) . (0, k0)  + (p[2i+2], p[2i+3]) . (k1, k2) = D_i . P2 + D_i+1 . P3
// (v_dot2c_f32_bf16 / v_dot2_f32_f16, fp32 accumulation), against nine instructions per output and channel pair for
// taps that sit in different dwords.  A lane's 8 outputs are 16 contiguous bytes of the channel-first result: they
// are stored straight from registers (W a multiple of 4), or -- whole images whose rows are not 8-byte aligned --
// parked in LDS as the 64 * L (32 * L) contiguous elements they are in memory and stored 16 bytes per lane.
constexpr int kDwpMaxIt = 8;         // segments per lane at most
// Dword offset of channel plane c: planes are plane_dw apart, moved up by one where that leaves them on an even dword
// (the 8-byte reads of the compute phase).  plane_dw = 2 mod 8 for 32-channel tiles, 1 mod 8 for 64-channel tiles:
// the 4 (8) channel vectors that a wavefront writes together then land 16 (8) banks apart.
__device__ __forceinline__ int plane_at(int c, int plane_dw) { const int o = c * plane_dw; return o + (o & 1); }

template <typename T, bool kSilu, int kCh>
__global__ __launch_bounds__(kBlock) void dwconv3x3_planes_kernel(const T *__restrict__ x, const T *__restrict__ weight,
                                                                  const T *__restrict__ bias, T *__restrict__ y, int D, int H,
                                                                  int W, int TH, int row_tiles, int ch_tiles, int col_tiles,
                                                                  int TW, int pitch, int plane_dw, int nseg, int n_it,
                                                                  int flat_out, int in_channel_first, FastDiv divHalf,
                                                                  FastDiv divNseg, FastDiv divItems) {
    constexpr int kLpc = kBlock / kCh;                           // lanes per channel in the compute phase
    constexpr int kCv = kCh / 8;                                 // 16-byte channel vectors per position
    constexpr int kPer = kBlock / kCv;                           // position pairs per staging pass
    constexpr int kInFlight = 3;                                 // pairs (two loads each) a lane requests together
    extern __shared__ __align__(16) uint32_t dwp_smem[];         // [kCh][plane_dw]
    uint32_t wg = blockIdx.x;
    const uint32_t ct = wg % ch_tiles; wg /= ch_tiles;
    const uint32_t cx = wg % col_tiles; wg /= col_tiles;         // wide images: tiles of TW columns (col_tiles = 1 otherwise)
    const uint32_t rt = wg % row_tiles;
    const uint32_t b = wg / row_tiles;
    const int h0 = (int)rt * TH;
    const int rows = min(TH, H - h0);
    const int wb = (int)cx * TW;                                 // first image column of the tile
    const int c_base = (int)ct * kCh;
    const int L = H * W, half = pitch / 2;

    // compute-phase identity: channel and segment slot; its nine weights and bias, requested first
    const int cl = threadIdx.x / kLpc, slot = threadIdx.x % kLpc;
    const int c = c_base + cl;
    uint32_t wr[9];
    {
        const uint16_t *wsrc = reinterpret_cast<const uint16_t *>(weight + (size_t)c * 9);
#pragma unroll
        for (int k = 0; k < 9; ++k) wr[k] = wsrc[k];
    }
    const float bv = bias ? to_f32(bias[c]) : 0.0f;

    // ---- staging: rows h0-1 .. h0+rows of kCh channels into the planes, zeros outside the image
    if (in_channel_first) {
        // x (B, D, H, W): a plane dword is two neighbouring elements of a channel's row, starting at an odd column
        // (padded column 0 is image column -1), so the pair is put together from two 16-bit loads; consecutive lanes
        // take consecutive dwords of a plane.  kAhead dwords per lane are requested before the first is parked.
        constexpr int kAhead = 4;
        const T *xb = x + ((size_t)b * D + c_base) * H * W;
        // (planes are indexed as for a full tile of TH rows; a short last tile leaves the lanes of its missing rows idle)
        const int n_items = (rows + 2) * half, total = kCh * (TH + 2) * half;
        for (int i0 = threadIdx.x; i0 < total; i0 += kAhead * kBlock) {
            uint32_t lo[kAhead], hi[kAhead];
            int dst[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const int idx = min(i0 + u * kBlock, total - 1);
                uint32_t pc, q, rr, pp;
                divmod((uint32_t)idx, divItems, pc, q);
                divmod(q, divHalf, rr, pp);
                const int h = h0 - 1 + (int)rr, w0 = wb + 2 * (int)pp - 1, w1 = w0 + 1;
                const bool row_ok = h >= 0 && h < H && (int)q < n_items;
                const T *src = xb + ((size_t)pc * H + (row_ok ? h : 0)) * W;
                const bool ok0 = row_ok && w0 >= 0 && w0 < W, ok1 = row_ok && w1 < W;
                lo[u] = src[ok0 ? w0 : 0].bits; hi[u] = src[ok1 ? w1 : 0].bits;
                lo[u] = ok0 ? lo[u] : 0u; hi[u] = ok1 ? hi[u] : 0u;
                dst[u] = (int)q < n_items ? plane_at((int)pc, plane_dw) + (int)q : -1;
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u)
                if (i0 + u * kBlock < total && dst[u] >= 0) dwp_smem[dst[u]] = lo[u] | (hi[u] << 16);
        }
    } else {
        const int cv = threadIdx.x % kCv;
        const int c0 = c_base + cv * 8;
        const T *xb = x + (size_t)b * H * W * D;
        const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(xb), 0, H * W * D * 2, 0x00020000);
        const int n_items = (rows + 2) * half;
        uint32_t *plane0 = dwp_smem;
        for (int q0 = threadIdx.x / kCv; q0 < n_items; q0 += kInFlight * kPer) {
            uint4 va[kInFlight], vb[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                const int q = q0 + u * kPer;
                uint32_t rr, pp;
                divmod((uint32_t)q, divHalf, rr, pp);
                const int h = h0 - 1 + (int)rr, w0 = wb + 2 * (int)pp - 1, w1 = wb + 2 * (int)pp;
                const bool row_ok = q < n_items && h >= 0 && h < H;
                const uint32_t off_a = (row_ok && w0 >= 0 && w0 < W) ? (uint32_t)((h * W + w0) * D + c0) * 2u : 0x7ffffff0u;
                const uint32_t off_b = (row_ok && w1 < W) ? (uint32_t)((h * W + w1) * D + c0) * 2u : 0x7ffffff0u;
                const auto ta = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off_a, 0, 0);
                const auto tb = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off_b, 0, 0);
                va[u] = make_uint4(ta[0], ta[1], ta[2], ta[3]);
                vb[u] = make_uint4(tb[0], tb[1], tb[2], tb[3]);
            }
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                const int q = q0 + u * kPer;
                if (q < n_items) {
                    const uint32_t a[4] = {va[u].x, va[u].y, va[u].z, va[u].w}, bb[4] = {vb[u].x, vb[u].y, vb[u].z, vb[u].w};
                    uint32_t *dst = plane0 + q;                  // rr * half + pp = q
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        dst[plane_at(cv * 8 + 2 * i, plane_dw)] = pair_lo(a[i], bb[i]);
                        dst[plane_at(cv * 8 + 2 * i + 1, plane_dw)] = pair_hi(a[i], bb[i]);
                    }
                }
            }
        }
    }
    // weight pairs per filter row
    uint32_t P0[3], P1[3], P2[3], P3[3];
#pragma unroll
    for (int kr = 0; kr < 3; ++kr) {
        P0[kr] = wr[3 * kr] | (wr[3 * kr + 1] << 16);
        P1[kr] = wr[3 * kr + 2];
        P2[kr] = wr[3 * kr] << 16;
        P3[kr] = wr[3 * kr + 1] | (wr[3 * kr + 2] << 16);
    }
    __syncthreads();

    const uint32_t *plane = dwp_smem + plane_at(cl, plane_dw);
    const int n_seg = rows * nseg;
    T *yc = y + ((size_t)b * D + c) * L + (size_t)h0 * W;
    uint32_t keep[kDwpMaxIt][4];
#pragma unroll
    for (int it = 0; it < kDwpMaxIt; ++it) {
        if (it < n_it) {                                          // uniform
            const int sg = slot + kLpc * it;
            uint32_t r, seg;
            divmod((uint32_t)min(sg, n_seg - 1), divNseg, r, seg);
            float acc[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = bv;
#pragma unroll
            for (int kr = 0; kr < 3; ++kr) {
                const uint32_t *row = plane + (r + kr) * half + seg * 4;
                const uint2 d01 = *reinterpret_cast<const uint2 *>(row), d23 = *reinterpret_cast<const uint2 *>(row + 2);
                const uint32_t d[5] = {d01.x, d01.y, d23.x, d23.y, row[4]};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[2 * i] = dot2_acc(T{}, d[i], P0[kr], acc[2 * i]);
                    acc[2 * i] = dot2_acc(T{}, d[i + 1], P1[kr], acc[2 * i]);
                    acc[2 * i + 1] = dot2_acc(T{}, d[i], P2[kr], acc[2 * i + 1]);
                    acc[2 * i + 1] = dot2_acc(T{}, d[i + 1], P3[kr], acc[2 * i + 1]);
                }
            }
            uint32_t o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                o[i] = pack2_from_f32<T>(acc[2 * i], acc[2 * i + 1]);                                   // conv output as stored
                if (kSilu) o[i] = pack2_from_f32<T>(silu_fast(unpack_lo<T>(o[i])), silu_fast(unpack_hi<T>(o[i])));
            }
            if (flat_out) {
#pragma unroll
                for (int i = 0; i < 4; ++i) keep[it][i] = o[i];
            } else if (sg < n_seg) {
                T *dst = yc + r * W + wb + seg * 8;
                if (W % 8 == 0) {
                    *reinterpret_cast<uint4 *>(dst) = make_uint4(o[0], o[1], o[2], o[3]);
                } else {                                          // W % 4 == 0: 8-byte rows, a last segment of 4
                    *reinterpret_cast<uint2 *>(dst) = make_uint2(o[0], o[1]);
                    if ((int)seg * 8 + 8 <= W) *reinterpret_cast<uint2 *>(dst + 4) = make_uint2(o[2], o[3]);
                }
            }
        }
    }
    if (!flat_out) return;

    // ---- whole image: the results of the kCh channels are one contiguous block of y; park them in LDS as they lie in
    // memory (the planes are no longer needed) and store 16 bytes per lane
    __syncthreads();
    uint16_t *flat = reinterpret_cast<uint16_t *>(dwp_smem);      // [kCh][L]
#pragma unroll
    for (int it = 0; it < kDwpMaxIt; ++it) {
        const int sg = slot + kLpc * it;
        if (it < n_it && sg < n_seg) {
            uint32_t r, seg;
            divmod((uint32_t)sg, divNseg, r, seg);
            uint16_t *dst = flat + cl * L + r * W + seg * 8;
            const int nv = min(8, W - (int)seg * 8);
            if (W % 2 == 0) {                                     // every offset and count is even: whole dwords
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (2 * i < nv) reinterpret_cast<uint32_t *>(dst)[i] = keep[it][i];
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (j < nv) dst[j] = (uint16_t)((j & 1) ? keep[it][j / 2] >> 16 : keep[it][j / 2] & 0xffffu);
            }
        }
    }
    __syncthreads();
    uint4 *dst = reinterpret_cast<uint4 *>(y + ((size_t)b * D + c_base) * L);
    const uint4 *src = reinterpret_cast<const uint4 *>(flat);
    for (int pc = threadIdx.x; pc < kCh * L / 8; pc += kBlock) dst[pc] = src[pc];
}

// fp32, channel-last input: the 16-bit tap-by-tap kernel's scheme with four channels per 16-byte vector.  A workgroup
// owns 32 consecutive positions x 32 channels; a lane convolves 4 channels at one position from nine 16-byte loads
// (the eight lanes of a position read 128 contiguous bytes; neighbouring positions re-use the lines out of L1 / L2),
// parks its results in LDS and the tile leaves transposed, 16 bytes per lane along the positions.  Same arithmetic as the
// generic kernel below: taps accumulated in (kh, kw) order with fused multiply-adds, bias added last, exact SiLU.
constexpr int kDwfPos = 32, kDwfCh = 32, kDwfPitch = kDwfPos + 4;
template <bool kSilu>
__global__ __launch_bounds__(kBlock) void dwconv3x3_cl2cf_f32_kernel(const float *__restrict__ x, const float *__restrict__ weight,
                                                                     const float *__restrict__ bias, float *__restrict__ y, int D,
                                                                     int H, int W, int pos_tiles, int ch_tiles, FastDiv divW) {
    __shared__ __align__(16) float tile[kDwfCh * kDwfPitch];
    uint32_t wg = blockIdx.x;
    const uint32_t ct = wg % ch_tiles; wg /= ch_tiles;
    const uint32_t pt = wg % pos_tiles;
    const uint32_t b = wg / pos_tiles;
    const int L = H * W;
    const int r0 = (int)pt * kDwfPos;
    const int p = threadIdx.x / 8, cv = threadIdx.x % 8;
    const int c0 = (int)ct * kDwfCh + cv * 4;           // this lane's 4 channels
    const int r = r0 + p;
    if (r < L && c0 < D) {
        uint32_t h, w;
        divmod((uint32_t)r, divW, h, w);
        float wt[36];                                   // [channel][tap]: 9 consecutive 16-byte vectors
        {
            const float4 *wp = reinterpret_cast<const float4 *>(weight + (size_t)c0 * 9);
#pragma unroll
            for (int k = 0; k < 9; ++k) {
                const float4 t = wp[k];
                wt[4 * k] = t.x; wt[4 * k + 1] = t.y; wt[4 * k + 2] = t.z; wt[4 * k + 3] = t.w;
            }
        }
        const float *xb = x + (size_t)b * L * D;
        float4 tap[9];
#pragma unroll
        for (int kh = 0; kh < 3; ++kh)
#pragma unroll
            for (int kw = 0; kw < 3; ++kw) {
                const int hh = (int)h + kh - 1, ww = (int)w + kw - 1;
                const bool in = hh >= 0 && hh < H && ww >= 0 && ww < W;
                // out-of-image taps read this position's own vector (a valid address) and are left out of the sum
                const size_t off = in ? ((size_t)hh * W + ww) * D + c0 : ((size_t)h * W + w) * D + c0;
                tap[kh * 3 + kw] = *reinterpret_cast<const float4 *>(xb + off);
            }
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int kh = 0; kh < 3; ++kh)
#pragma unroll
            for (int kw = 0; kw < 3; ++kw) {
                const int hh = (int)h + kh - 1, ww = (int)w + kw - 1;
                if (hh >= 0 && hh < H && ww >= 0 && ww < W) {
                    const float xv[4] = {tap[kh * 3 + kw].x, tap[kh * 3 + kw].y, tap[kh * 3 + kw].z, tap[kh * 3 + kw].w};
#pragma unroll
                    for (int ci = 0; ci < 4; ++ci) acc[ci] = fmaf(wt[ci * 9 + kh * 3 + kw], xv[ci], acc[ci]);
                }
            }
        if (bias) {
            const float4 bv = *reinterpret_cast<const float4 *>(bias + c0);
            acc[0] += bv.x; acc[1] += bv.y; acc[2] += bv.z; acc[3] += bv.w;
        }
#pragma unroll
        for (int ci = 0; ci < 4; ++ci) tile[(cv * 4 + ci) * kDwfPitch + p] = kSilu ? silu_f32(acc[ci]) : acc[ci];
    }
    __syncthreads();
    // write back: lane -> (channel = tid / 8, four consecutive positions)
    const int c = threadIdx.x / 8, chunk = threadIdx.x % 8;
    const int cg = (int)ct * kDwfCh + c;
    const int rr = r0 + chunk * 4;
    if (cg < D && rr < L) {
        float *yo = y + ((size_t)b * D + cg) * L + rr;
        const float *src = tile + c * kDwfPitch + chunk * 4;
        if (rr + 4 <= L && (L % 4) == 0) {
            *reinterpret_cast<float4 *>(yo) = *reinterpret_cast<const float4 *>(src);
        } else {
            for (int i = 0; i < 4 && rr + i < L; ++i) yo[i] = src[i];
        }
    }
}

// fp32, channel-first input (the reference harness's own precision and layout), W a multiple of 4, 16-byte aligned maps:
// four consecutive outputs of a row per lane from three 16-byte row loads and the six neighbours either side -- a
// quarter of the load instructions of the one-output-per-lane kernel below, 16-byte stores.  Same arithmetic as that
// kernel: taps accumulated in (kh, kw) order with fused multiply-adds, bias added last, exact SiLU.
template <bool kSilu>
__global__ __launch_bounds__(kBlock) void dwconv3x3_cf_f32_kernel(const float *__restrict__ x, const float *__restrict__ weight,
                                                                  const float *__restrict__ bias, float *__restrict__ y, int D, int H,
                                                                  int W, int64_t total_quads, FastDiv divD) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;     // over (b, d, h, w / 4)
    if (idx >= total_quads) return;
    const int Wq = W / 4;
    const int64_t rows_idx = idx / Wq;                                  // (b, d, h)
    const int wq = (int)(idx - rows_idx * Wq);
    const uint32_t map = (uint32_t)(rows_idx / H);
    const int h = (int)(rows_idx - (int64_t)map * H);
    uint32_t b, d;
    divmod(map, divD, b, d);
    (void)b;
    const float *xm = x + (size_t)map * H * W;
    float wt[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) wt[t] = weight[(size_t)d * 9 + t];
    const int w0 = 4 * wq;
    float in[3][6];
    bool row_in[3];
#pragma unroll
    for (int kh = 0; kh < 3; ++kh) {
        const int hh = h + kh - 1;
        row_in[kh] = hh >= 0 && hh < H;
        const float *row = xm + (size_t)(row_in[kh] ? hh : h) * W;
        const float4 m = *reinterpret_cast<const float4 *>(row + w0);
        in[kh][0] = w0 > 0 ? row[w0 - 1] : 0.0f;
        in[kh][1] = m.x; in[kh][2] = m.y; in[kh][3] = m.z; in[kh][4] = m.w;
        in[kh][5] = w0 + 4 < W ? row[w0 + 4] : 0.0f;
    }
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int kh = 0; kh < 3; ++kh)
#pragma unroll
        for (int kw = 0; kw < 3; ++kw)
            if (row_in[kh]) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int ww = w0 + j + kw - 1;
                    if (ww >= 0 && ww < W) acc[j] = fmaf(wt[kh * 3 + kw], in[kh][j + kw], acc[j]);
                }
            }
    const float bv = bias ? bias[d] : 0.0f;
    float o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) { o[j] = acc[j] + bv; if (kSilu) o[j] = silu_f32(o[j]); }
    *reinterpret_cast<float4 *>(y + (size_t)rows_idx * W + w0) = make_float4(o[0], o[1], o[2], o[3]);
}

// Generic variant: any element type, either input layout, one output element per lane (lanes along W).
template <typename T, bool kInChannelLast, bool kSilu>
__global__ __launch_bounds__(kBlock) void dwconv3x3_generic_kernel(const T *__restrict__ x, const T *__restrict__ weight,
                                                                   const T *__restrict__ bias, T *__restrict__ y, int D, int H,
                                                                   int W, int64_t total, FastDiv divW, FastDiv divH,
                                                                   FastDiv divD) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;     // over (b, d, h, w)
    if (idx >= total) return;
    const int64_t L = (int64_t)H * W;
    const uint32_t map = (uint32_t)(idx / L);
    const uint32_t r = (uint32_t)(idx - (int64_t)map * L);
    uint32_t b, d, h, w;
    divmod(map, divD, b, d);
    divmod(r, divW, h, w);
    (void)divH;
    float acc = 0.0f;
#pragma unroll
    for (int kh = 0; kh < 3; ++kh)
#pragma unroll
        for (int kw = 0; kw < 3; ++kw) {
            const int hh = (int)h + kh - 1, ww = (int)w + kw - 1;
            if (hh >= 0 && hh < H && ww >= 0 && ww < W) {
                const size_t off = kInChannelLast ? (((size_t)b * H + hh) * W + ww) * D + d
                                                  : (((size_t)b * D + d) * H + hh) * W + ww;
                acc = fmaf(to_f32(weight[(size_t)d * 9 + kh * 3 + kw]), to_f32(x[off]), acc);
            }
        }
    if (bias) acc += to_f32(bias[d]);
    T o = from_f32<T>(acc);
    if (kSilu) o = from_f32<T>(silu_f32(to_f32(o)));
    y[idx] = o;
}

template <typename T>
static int launch_dwconv(const void *x, const void *w, const void *bias, void *y, int B, int D, int H, int W,
                         int in_channel_last, int apply_silu, hipStream_t stream) {
    const int64_t L = (int64_t)H * W;
    auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    if constexpr (sizeof(T) == 2) {
        // plane variant: channel tiles of 64 (or 32), full rows, outputs that leave as whole 8- or 16-byte pieces
        // images wider than 120 columns: column tiles of lpc, ..., 4 whole segments, if such a width divides W
        int seg_t = 0;
        if (W > 120 && W % 8 == 0)
            for (int n = kBlock / (D % 64 == 0 ? 64 : 32); n >= 4 && seg_t == 0; --n)
                if ((W / 8) % n == 0) seg_t = n;
        // (channel-first input takes the same kernel with element-wise staging: no alignment asked of x)
        if (D % 32 == 0 && (W <= 120 || seg_t > 0) && (al16(x) || !in_channel_last) && al16(y) &&
            (int64_t)H * W * D * 2 < 0x7ffffff0ll) {
            const int kch = D % 64 == 0 ? 64 : 32, lpc = kBlock / kch;
            const int TW = seg_t > 0 ? 8 * seg_t : W, col_tiles = seg_t > 0 ? W / TW : 1;
            const int nseg = (TW + 7) / 8, pitch = 8 * nseg + 4;
            int TH = (7 * lpc) / nseg;
            TH = TH > H ? H : TH;
            const int row_tiles = TH >= 1 ? (H + TH - 1) / TH : 0, ch_tiles = D / kch;
            const int flat_out = W % 4 != 0;
            const int n_it = TH >= 1 ? (TH * nseg + lpc - 1) / lpc : 0;
            int plane_dw = (TH + 2) * pitch / 2;
            const int want = kch == 64 ? 1 : 2;                    // see plane_at
            plane_dw += 1;                                         // room for the parity shift
            plane_dw += (want - plane_dw % 8 + 8) % 8;
            const size_t smem = ((size_t)kch * plane_dw + 2) * 4;
            const int64_t n_wg = (int64_t)B * row_tiles * col_tiles * ch_tiles;
            if (TH >= 1 && n_it <= kDwpMaxIt && (!flat_out || row_tiles == 1) && smem <= 64 * 1024 && n_wg <= 0x7fffffff) {
#define SS2D_DW_PLANES(SILU, KCH)                                                                                              \
    hipLaunchKernelGGL((dwconv3x3_planes_kernel<T, SILU, KCH>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, (const T *)x,  \
                       (const T *)w, (const T *)bias, (T *)y, D, H, W, TH, row_tiles, ch_tiles, col_tiles, TW, pitch, plane_dw,  \
                       nseg, n_it, flat_out, in_channel_last ? 0 : 1, make_fastdiv((uint32_t)(pitch / 2)),                     \
                       make_fastdiv((uint32_t)nseg), make_fastdiv((uint32_t)((TH + 2) * (pitch / 2))))
                if (kch == 64) { if (apply_silu) SS2D_DW_PLANES(true, 64); else SS2D_DW_PLANES(false, 64); }
                else { if (apply_silu) SS2D_DW_PLANES(true, 32); else SS2D_DW_PLANES(false, 32); }
#undef SS2D_DW_PLANES
                return launch_status();
            }
        }
        if (in_channel_last && D % 8 == 0 && W <= kDwMaxW && al16(x) && al16(w) && al16(y) && (!bias || al16(bias))) {
            // TH rows per workgroup: about 224 positions, LDS within 64 KiB
            int TH = 224 / W;
            TH = TH < 1 ? 1 : (TH > H ? H : TH);
            int out_pitch = ((TH * W + 15) / 16) * 16;                // a multiple of 16 elements: rows rotate by 16, 32, 48
            if (out_pitch < 48) out_pitch = 48;                       // ... and a rotated column wraps around at most once
            const int row_tiles = (H + TH - 1) / TH, ch_tiles = (D + kDwCh - 1) / kDwCh;
            const int64_t n_wg = (int64_t)B * row_tiles * ch_tiles;
            // whole images whose rows do not take 16-byte stores: the tile leaves as one flat block
            const int flat_out = row_tiles == 1 && D % kDwCh == 0 && L % 8 != 0 && L >= 8;
            // (its output tile is read element by element, so the rows need no 16-byte alignment: a pitch of 2 mod 16
            // elements puts the rows of the four channel groups of a wavefront 8 banks apart without any rotation)
            if (flat_out) out_pitch = (int)((L + 13) / 16) * 16 + 2;
            const size_t smem = ((size_t)(TH + 2) * (W + 2) * kDwCh + (size_t)kDwCh * out_pitch) * sizeof(uint16_t);
            if (smem <= 64 * 1024 && n_wg <= 0x7fffffff && (int64_t)H * W * D * 2 < 0x7ffffff0ll) {
                if (apply_silu) {
                    hipLaunchKernelGGL((dwconv3x3_rows_kernel<T, true>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream,
                                       (const T *)x, (const T *)w, (const T *)bias, (T *)y, D, H, W, TH, row_tiles, ch_tiles,
                                       out_pitch, flat_out, make_fastdiv((uint32_t)W), make_fastdiv((uint32_t)(W + 2)),
                                       make_fastdiv((uint32_t)L));
                } else {
                    hipLaunchKernelGGL((dwconv3x3_rows_kernel<T, false>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream,
                                       (const T *)x, (const T *)w, (const T *)bias, (T *)y, D, H, W, TH, row_tiles, ch_tiles,
                                       out_pitch, flat_out, make_fastdiv((uint32_t)W), make_fastdiv((uint32_t)(W + 2)),
                                       make_fastdiv((uint32_t)L));
                }
                return launch_status();
            }
        }
        if (in_channel_last && D % 8 == 0 && al16(x) && al16(w) && al16(y) && (!bias || al16(bias))) {
            const int pos_tiles = (int)((L + kDwPos - 1) / kDwPos), ch_tiles = (D + kDwCh - 1) / kDwCh;
            const int64_t n_wg = (int64_t)B * pos_tiles * ch_tiles;
            if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
            if (apply_silu) {
                hipLaunchKernelGGL((dwconv3x3_cl2cf_kernel<T, true>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream,
                                   (const T *)x, (const T *)w, (const T *)bias, (T *)y, D, H, W, pos_tiles, ch_tiles,
                                   make_fastdiv((uint32_t)W));
            } else {
                hipLaunchKernelGGL((dwconv3x3_cl2cf_kernel<T, false>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream,
                                   (const T *)x, (const T *)w, (const T *)bias, (T *)y, D, H, W, pos_tiles, ch_tiles,
                                   make_fastdiv((uint32_t)W));
            }
            return launch_status();
        }
    }
    if constexpr (sizeof(T) == 4) {
        if (in_channel_last && D % 4 == 0 && al16(x) && al16(w) && al16(y) && (!bias || al16(bias))) {
            const int pos_tiles = (int)((L + kDwfPos - 1) / kDwfPos), ch_tiles = (D + kDwfCh - 1) / kDwfCh;
            const int64_t n_tiles = (int64_t)B * pos_tiles * ch_tiles;
            if (n_tiles <= 0x7fffffff) {
                if (apply_silu) {
                    hipLaunchKernelGGL((dwconv3x3_cl2cf_f32_kernel<true>), dim3((uint32_t)n_tiles), dim3(kBlock), 0, stream,
                                       (const float *)x, (const float *)w, (const float *)bias, (float *)y, D, H, W, pos_tiles,
                                       ch_tiles, make_fastdiv((uint32_t)W));
                } else {
                    hipLaunchKernelGGL((dwconv3x3_cl2cf_f32_kernel<false>), dim3((uint32_t)n_tiles), dim3(kBlock), 0, stream,
                                       (const float *)x, (const float *)w, (const float *)bias, (float *)y, D, H, W, pos_tiles,
                                       ch_tiles, make_fastdiv((uint32_t)W));
                }
                return launch_status();
            }
        }
    }
    if constexpr (sizeof(T) == 4) {
        if (!in_channel_last && W % 4 == 0 && al16(x) && al16(y) && (int64_t)B * D <= 0x7fffffff) {
            const int64_t quads = (int64_t)B * D * H * (W / 4);
            const int64_t n_q = (quads + kBlock - 1) / kBlock;
            if (n_q <= 0x7fffffff) {
                if (apply_silu) {
                    hipLaunchKernelGGL((dwconv3x3_cf_f32_kernel<true>), dim3((uint32_t)n_q), dim3(kBlock), 0, stream, (const float *)x,
                                       (const float *)w, (const float *)bias, (float *)y, D, H, W, quads, make_fastdiv((uint32_t)D));
                } else {
                    hipLaunchKernelGGL((dwconv3x3_cf_f32_kernel<false>), dim3((uint32_t)n_q), dim3(kBlock), 0, stream, (const float *)x,
                                       (const float *)w, (const float *)bias, (float *)y, D, H, W, quads, make_fastdiv((uint32_t)D));
                }
                return launch_status();
            }
        }
    }
    const int64_t total = (int64_t)B * D * L;
    const int64_t n_wg = (total + kBlock - 1) / kBlock;
    if (n_wg > 0x7fffffff || (int64_t)B * D > 0x7fffffff) return SS2D_ENOTSUP;
#define SS2D_DW_GENERIC(CL, SILU)                                                                                       \
    hipLaunchKernelGGL((dwconv3x3_generic_kernel<T, CL, SILU>), dim3((uint32_t)n_wg), dim3(kBlock), 0, stream,         \
                       (const T *)x, (const T *)w, (const T *)bias, (T *)y, D, H, W, total, make_fastdiv((uint32_t)W), \
                       make_fastdiv((uint32_t)H), make_fastdiv((uint32_t)D))
    if (in_channel_last) { if (apply_silu) SS2D_DW_GENERIC(true, true); else SS2D_DW_GENERIC(true, false); }
    else { if (apply_silu) SS2D_DW_GENERIC(false, true); else SS2D_DW_GENERIC(false, false); }
#undef SS2D_DW_GENERIC
    return launch_status();
}

}  // namespace ss2d

extern "C" int ss2d_dwconv3x3_silu(const void *x, const void *weight, const void *bias, void *y, int B, int D, int H, int W,
                                   int dtype, int in_channel_last, int apply_silu, void *stream) {
    using namespace ss2d;
    if (B < 0 || D < 0 || H < 0 || W < 0) return SS2D_EINVAL;
    if (dtype != SS2D_F32 && dtype != SS2D_BF16 && dtype != SS2D_F16) return SS2D_EINVAL;
    if (B == 0 || D == 0 || H == 0 || W == 0) return SS2D_OK;
    if (!x || !weight || !y) return SS2D_EINVAL;
    if ((int64_t)H * W > 0x3fffffff) return SS2D_ENOTSUP;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case SS2D_F32: return launch_dwconv<float>(x, weight, bias, y, B, D, H, W, in_channel_last, apply_silu, s);
        case SS2D_BF16: return launch_dwconv<bf16_t>(x, weight, bias, y, B, D, H, W, in_channel_last, apply_silu, s);
        default: return launch_dwconv<f16_t>(x, weight, bias, y, B, D, H, W, in_channel_last, apply_silu, s);
    }
}
