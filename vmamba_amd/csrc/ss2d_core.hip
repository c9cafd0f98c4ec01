// Fused SS2D core for one state per channel (d_state = 1, the VMamba-T/S/B setting):
//     CrossScan  ->  selective scan  ->  CrossMerge        in ONE kernel.
//
// The unfused path writes the four scan-ordered copies of x (xs), reads them back in the scan, writes the four
// scan outputs (ys) and reads them back in the merge: 62 bytes per activation element at bf16-in / fp32-out.
// Here a workgroup owns one channel d of CB images.  Its four wavefronts are the four scan directions:
//   * the CB x maps are loaded once into LDS (odd row pitch); every wavefront reads u for ITS direction from
//     there -- row-major, column-major, or either reversed -- so xs never exists;
//   * delta (from dt_proj) and the B / C rows (from x_proj) are streamed from HBM / L2 exactly as in the scan
//     kernels: 8 positions per lane, DPP wavefront scan, state carried in a register, softplus fused;
//   * each wavefront adds its outputs into two fp32 LDS planes at the position the merge wants them: plane A
//     (row-major index) collects directions 0 and 2, plane B (column-major index, odd pitch) directions 1 and 3.
//     Each plane entry receives exactly two adds onto an initial 0, so the result is fl(y0 + y2) resp. fl(y1 + y3)
//     whatever order the LDS atomics land in -- the association order of cross_merge_fwd
//     (classification/models/csm_triton.py:61-62) -- and ys never exists;
//   * finally out[r] = A[r] + B[t(r)] is written once.
// HBM traffic per element: x (s_in) + 4 delta (4 s_in) + out (s_out) = 14 bytes instead of 62.
//
// The CB images of a workgroup are walked as one stream per direction (restart by a = 0 at each image start, as
// in the flat scan kernel), which needs their delta rows adjacent in memory: delta is therefore taken with
// explicit (direction, channel, batch) strides and CB > 1 requires batch stride == L, i.e. the batch-innermost
// layout (K, D, B, L) that a single large dt_proj GEMM per direction produces.
#include "scan_common.h"

namespace ss2d {

struct CoreArgs {
    const void *x, *delta, *Bm, *Cm;
    const float *A, *Dv, *bias;
    void *y;
    int32_t B, D, H, W, L, CB, Wp, Hp, softplus, vec_ok;
    int64_t dl_ks, dl_ds, dl_bs;        // delta strides over direction, channel, batch (elements)
    int64_t B_ks, B_bs, C_ks, C_bs;     // B / C strides over direction and batch (elements)
    uint32_t B_span_bytes, C_span_bytes;
};

// Walks the spatial position that scan position j of direction kDir reads / writes.
//   directions 0, 2: row-major index s = h*W + w  -> (q, r) = (h, w), inner extent W
//   directions 1, 3: column-major index s = w*H + h -> (q, r) = (w, h), inner extent H
//   directions 0, 1 walk s upwards from 0, directions 2, 3 downwards from L-1.
template <int kDir>
struct Walker {
    int q, r;
    __device__ __forceinline__ void init(int j, int L, FastDiv div_inner) {
        const uint32_t s = (kDir < 2) ? (uint32_t)j : (uint32_t)(L - 1 - j);
        uint32_t qq, rr;
        divmod(s, div_inner, qq, rr);
        q = (int)qq; r = (int)rr;
    }
    __device__ __forceinline__ void restart(int outer, int inner) {       // first scan position of an image
        q = (kDir < 2) ? 0 : outer - 1;
        r = (kDir < 2) ? 0 : inner - 1;
    }
    __device__ __forceinline__ void step(int inner) {
        if (kDir < 2) { ++r; const bool c = r == inner; r = c ? 0 : r; q += c ? 1 : 0; }
        else { --r; const bool c = r < 0; r = c ? inner - 1 : r; q -= c ? 1 : 0; }
    }
};

template <typename in_t, int kDir, bool kSoftplus, int kGran>
__device__ __forceinline__ void core_scan_direction(const CoreArgs &p, int d, int b0, int nb, const in_t *xmap, float *planeA,
                                                    float *planeB, FastDiv divL, FastDiv divW, FastDiv divH) {
    constexpr int kGroups = kItems / kGran;
    constexpr bool kRowMajor = (kDir % 2) == 0;
    const int lane = threadIdx.x & (kWave - 1);
    const int L = p.L, H = p.H, W = p.W, Wp = p.Wp, Hp = p.Hp;
    const int inner = kRowMajor ? W : H, outer = kRowMajor ? H : W;
    const FastDiv div_inner = kRowMajor ? divW : divH;
    const int Lp = H * Wp, WHp = W * Hp;
    const int n_el = nb * L;
    const int kd = kDir * p.D + d;
    const in_t *dl_base = reinterpret_cast<const in_t *>(p.delta) + kDir * p.dl_ks + d * p.dl_ds + b0 * p.dl_bs;
    const __amdgpu_buffer_rsrc_t B_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.Bm), 0, (int)p.B_span_bytes, kBufferRsrcWord3);
    const __amdgpu_buffer_rsrc_t C_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.Cm), 0, (int)p.C_span_bytes, kBufferRsrcWord3);
    const uint32_t B_soff = (uint32_t)(kDir * p.B_ks + b0 * p.B_bs), C_soff = (uint32_t)(kDir * p.C_ks + b0 * p.C_bs);
    const float A_log2e = p.A[kd] * kLog2e;
    const float Dv = p.Dv ? p.Dv[kd] : 0.0f;
    const float bias = p.bias ? p.bias[kd] : 0.0f;
    float *plane = kRowMajor ? planeA : planeB;
    const int plane_img = kRowMajor ? L : WHp;          // plane elements per image
    const int plane_pitch = kRowMajor ? W : Hp;

    float h_carry = 0.0f;
    const int n_pass = (n_el + kPass - 1) / kPass;
    for (int pass = 0; pass < n_pass; ++pass) {
        const int e0 = pass * kPass + lane * kItems;
        const bool full = e0 + kItems <= n_el;
        float raw[kItems];
        if (full && p.vec_ok) load_items<in_t, true>(dl_base, e0, n_el, raw, delta_fill<kSoftplus>());
        else load_items<in_t, false>(dl_base, e0, n_el, raw, delta_fill<kSoftplus>());

        uint32_t i0, j0;
        divmod((uint32_t)min(e0, n_el - 1), divL, i0, j0);
        const int k = kGran == kItems ? kItems : min(kItems, L - (int)j0);     // items before the next image starts

        // u from the LDS maps, and where each output goes in the merge planes
        Walker<kDir> wk;
        wk.init((int)j0, L, div_inner);
        int img = (int)i0;
        float uv[kItems];
        int paddr[kItems];
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            if constexpr (kGran != kItems) {
                if (i % kGran == 0) {                       // an image can only start at a group boundary
                    const bool wrap = i == k;
                    if (wrap) { wk.restart(outer, inner); }
                    img += wrap ? 1 : 0;
                }
            }
            const bool valid = e0 + i < n_el;
            const int xoff = img * Lp + (kRowMajor ? wk.q * Wp + wk.r : wk.r * Wp + wk.q);
            uv[i] = valid ? to_f32(xmap[valid ? xoff : 0]) : 0.0f;
            paddr[i] = img * plane_img + wk.q * plane_pitch + wk.r;
            wk.step(inner);
        }

        float dl[kItems], bias_items[kItems];
#pragma unroll
        for (int i = 0; i < kItems; ++i) bias_items[i] = bias;
        delta_transform<kSoftplus>(raw, bias_items, dl);

        // B, C rows of (direction, image): group gathers
        float Bv[kItems], Cv[kItems];
        bool first[kGroups];
#pragma unroll
        for (int gi = 0; gi < kGroups; ++gi) {
            const bool in_a = kGran == kItems ? true : gi * kGran < k;
            const uint32_t ig = i0 + (in_a ? 0u : 1u);
            const uint32_t jg = in_a ? j0 + gi * kGran : (uint32_t)(gi * kGran - k);
            first[gi] = jg == 0;
            float bg[kGran], cg[kGran];
            gather_group<in_t, kGran>(B_rsrc, ig * (uint32_t)p.B_bs + jg, B_soff, bg);
            gather_group<in_t, kGran>(C_rsrc, ig * (uint32_t)p.C_bs + jg, C_soff, cg);
#pragma unroll
            for (int i = 0; i < kGran; ++i) { Bv[gi * kGran + i] = bg[i]; Cv[gi * kGran + i] = cg[i]; }
        }

        float ac[kItems], hh[kItems];
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            if constexpr (!kSoftplus) dl[i] = (e0 + i < n_el) ? dl[i] : 0.0f;
            float a = __builtin_amdgcn_exp2f(dl[i] * A_log2e);
            if (i % kGran == 0) a = first[i / kGran] ? 0.0f : a;
            const float bb = (e0 + i < n_el) ? Bv[i] * (dl[i] * uv[i]) : 0.0f;
            ac[i] = i == 0 ? a : ac[i - 1] * a;
            hh[i] = i == 0 ? bb : fmaf(a, hh[i - 1], bb);
        }
        float a_ex, h_ex, a_tot, h_tot;
        wave_scan_pairs(ac[kItems - 1], hh[kItems - 1], a_ex, h_ex, a_tot, h_tot);
        const float s_in = fmaf(a_ex, h_carry, h_ex);
        h_carry = fmaf(a_tot, h_carry, h_tot);
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            const float yv = fmaf(Cv[i], fmaf(ac[i], s_in, hh[i]), Dv * uv[i]);
            if (e0 + i < n_el) __hip_atomic_fetch_add(plane + paddr[i], yv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
}

template <typename in_t, bool kSoftplus, int kGran>
__global__ __launch_bounds__(kBlock) void ss2d_core_kernel(const CoreArgs p, FastDiv divL, FastDiv divW, FastDiv divH,
                                                           FastDiv divD) {
    extern __shared__ __align__(16) float core_smem[];
    const int L = p.L, H = p.H, W = p.W;
    const int Lp = H * p.Wp, WHp = W * p.Hp;
    float *planeA = core_smem;                           // [CB][L]
    float *planeB = planeA + p.CB * L;                   // [CB][W*Hp]
    in_t *xmap = reinterpret_cast<in_t *>(planeB + p.CB * WHp);   // [CB][H*Wp]

    uint32_t bt, d;
    divmod(blockIdx.x, divD, bt, d);                     // neighbouring workgroups share B / C rows (same images)
    const int b0 = (int)bt * p.CB;
    const int nb = min(p.CB, p.B - b0);
    const int n_el = nb * L;

    for (int idx = threadIdx.x; idx < p.CB * (L + WHp); idx += kBlock) core_smem[idx] = 0.0f;
    const in_t *xin = reinterpret_cast<const in_t *>(p.x);
    for (int idx = threadIdx.x; idx < n_el; idx += kBlock) {
        uint32_t i, r, h, w;
        divmod((uint32_t)idx, divL, i, r);
        divmod(r, divW, h, w);
        xmap[i * Lp + h * p.Wp + w] = xin[((size_t)(b0 + i) * p.D + d) * L + r];
    }
    __syncthreads();

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    switch (wave) {
        case 0: core_scan_direction<in_t, 0, kSoftplus, kGran>(p, (int)d, b0, nb, xmap, planeA, planeB, divL, divW, divH); break;
        case 1: core_scan_direction<in_t, 1, kSoftplus, kGran>(p, (int)d, b0, nb, xmap, planeA, planeB, divL, divW, divH); break;
        case 2: core_scan_direction<in_t, 2, kSoftplus, kGran>(p, (int)d, b0, nb, xmap, planeA, planeB, divL, divW, divH); break;
        default: core_scan_direction<in_t, 3, kSoftplus, kGran>(p, (int)d, b0, nb, xmap, planeA, planeB, divL, divW, divH); break;
    }
    __syncthreads();

    float *yo = reinterpret_cast<float *>(p.y);
    for (int idx = threadIdx.x; idx < n_el; idx += kBlock) {
        uint32_t i, r, h, w;
        divmod((uint32_t)idx, divL, i, r);
        divmod(r, divW, h, w);
        const float v = planeA[i * L + r] + planeB[i * WHp + w * p.Hp + h];
        yo[((size_t)(b0 + i) * p.D + d) * L + r] = v;
    }
}

static int core_gcd(int64_t a, int64_t b) { while (b) { const int64_t t = a % b; a = b; b = t; } return (int)(a < 0 ? -a : a); }

template <typename in_t>
static int launch_core(CoreArgs a, hipStream_t stream) {
    const int64_t L = a.L;
    // images per workgroup: ~3072 positions per direction; a workgroup's first delta row sits on a 16-byte
    // boundary when CB*L is a multiple of 8 elements
    const int64_t align_rows = 8 / core_gcd(L, 8);
    int64_t CB = (3072 + L / 2) / L;
    CB = CB < 1 ? 1 : CB;
    CB = (CB + align_rows - 1) / align_rows * align_rows;
    if (CB >= a.B) CB = a.B;                                  // a single tile starts at image 0
    if (CB > 1 && a.dl_bs != L) CB = 1;                       // adjacent delta rows need the batch-innermost layout
    a.CB = (int)CB;
    a.Wp = a.W | 1;
    a.Hp = a.H | 1;
    const size_t smem = (size_t)CB * ((size_t)L + (size_t)a.W * a.Hp) * sizeof(float) + (size_t)CB * a.H * a.Wp * sizeof(in_t);
    if (smem > 64 * 1024) return SS2D_ENOTSUP;
    // 16-byte loads of the delta stream need every (direction, channel, first image of a workgroup) start aligned;
    // otherwise the kernel loads element-wise
    const int64_t vec = 16 / (int64_t)sizeof(in_t);
    a.vec_ok = (reinterpret_cast<uintptr_t>(a.delta) % 16 == 0) && a.dl_ks % vec == 0 && a.dl_ds % vec == 0 &&
               (CB >= a.B || (CB * a.dl_bs) % vec == 0);
    int64_t g = core_gcd(L, kItems);
    const int64_t strides[] = {a.B_ks, a.B_bs, a.C_ks, a.C_bs};
    for (int64_t s : strides) g = core_gcd(g, s == 0 ? g : s);
    const uintptr_t bases = reinterpret_cast<uintptr_t>(a.Bm) | reinterpret_cast<uintptr_t>(a.Cm);
    while (g > 1 && (bases % (uintptr_t)(g * sizeof(in_t))) != 0) g /= 2;
    if (g == 2) g = 1;
    const int64_t tiles = (a.B + CB - 1) / CB;
    const int64_t n_wg = tiles * a.D;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    const FastDiv dL = make_fastdiv((uint32_t)L), dW = make_fastdiv((uint32_t)a.W), dH = make_fastdiv((uint32_t)a.H),
                  dD = make_fastdiv((uint32_t)a.D);
#define SS2D_CORE_LAUNCH(SP, G) \
    hipLaunchKernelGGL((ss2d_core_kernel<in_t, SP, G>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, a, dL, dW, dH, dD)
    if (a.softplus) {
        if (g == 8) SS2D_CORE_LAUNCH(true, 8); else if (g == 4) SS2D_CORE_LAUNCH(true, 4); else SS2D_CORE_LAUNCH(true, 1);
    } else {
        if (g == 8) SS2D_CORE_LAUNCH(false, 8); else if (g == 4) SS2D_CORE_LAUNCH(false, 4); else SS2D_CORE_LAUNCH(false, 1);
    }
#undef SS2D_CORE_LAUNCH
    return launch_status();
}

}  // namespace ss2d

extern "C" int ss2d_core_fwd(const ss2d_core_params *q, void *stream) {
    using namespace ss2d;
    if (!q) return SS2D_EINVAL;
    if (q->batch < 0 || q->dim < 0 || q->height < 0 || q->width < 0) return SS2D_EINVAL;
    if (q->in_dtype != SS2D_F32 && q->in_dtype != SS2D_BF16 && q->in_dtype != SS2D_F16) return SS2D_EINVAL;
    if (q->batch == 0 || q->dim == 0 || q->height == 0 || q->width == 0) return SS2D_OK;
    if (!q->x || !q->delta || !q->A || !q->B || !q->C || !q->y) return SS2D_EINVAL;
    const int64_t L = (int64_t)q->height * q->width;
    if (L < kItems || L > 0x0fffffff) return SS2D_ENOTSUP;
    if (q->delta_batch_stride < 0 || q->delta_dir_stride < 0 || q->delta_dim_stride < 0 || q->B_dir_stride < 0 ||
        q->B_batch_stride < 0 || q->C_dir_stride < 0 || q->C_batch_stride < 0) return SS2D_EINVAL;

    CoreArgs a;
    a.x = q->x; a.delta = q->delta; a.Bm = q->B; a.Cm = q->C;
    a.A = (const float *)q->A; a.Dv = (const float *)q->D; a.bias = (const float *)q->delta_bias;
    a.y = q->y;
    a.B = q->batch; a.D = q->dim; a.H = q->height; a.W = q->width; a.L = (int32_t)L;
    a.softplus = q->delta_softplus;
    a.dl_ks = q->delta_dir_stride; a.dl_ds = q->delta_dim_stride; a.dl_bs = q->delta_batch_stride;
    a.B_ks = q->B_dir_stride; a.B_bs = q->B_batch_stride; a.C_ks = q->C_dir_stride; a.C_bs = q->C_batch_stride;
    const int64_t eb = q->in_dtype == SS2D_F32 ? 4 : 2;
    const int64_t B_span = (3 * a.B_ks + (int64_t)(a.B - 1) * a.B_bs + L) * eb, C_span = (3 * a.C_ks + (int64_t)(a.B - 1) * a.C_bs + L) * eb;
    if (B_span >= 0x7fffffffll || C_span >= 0x7fffffffll) return SS2D_ENOTSUP;
    a.B_span_bytes = (uint32_t)B_span; a.C_span_bytes = (uint32_t)C_span;
    a.CB = 1; a.Wp = 0; a.Hp = 0; a.vec_ok = 0;

    hipStream_t s = (hipStream_t)stream;
    if (q->in_dtype == SS2D_F32) return launch_core<float>(a, s);
    if (q->in_dtype == SS2D_BF16) return launch_core<bf16_t>(a, s);
    return launch_core<f16_t>(a, s);
}

// ---- CrossScan, one-by-one --------------------------------------------------------------
// Each of the four direction slices of x (B,4,C,H,W) is laid out in ITS scan order (cross_scan1b1_fwd,
// classification/models/csm_triton.py:88-131, scans = 0).  One workgroup per (b, k, c) map; the transposing
// directions go through an LDS copy of the map with an odd row pitch.
namespace ss2d {

template <typename T>
__global__ __launch_bounds__(kBlock) void cross_scan_1b1_kernel(const T *__restrict__ x, T *__restrict__ y, int H, int W,
                                                                int Wp, int use_lds, int64_t y_bs, int64_t y_ks,
                                                                int64_t y_cs, FastDiv divC, FastDiv divW, FastDiv divH) {
    extern __shared__ __align__(16) unsigned char map_smem[];
    T *tile = reinterpret_cast<T *>(map_smem);
    uint32_t bk, c;
    divmod(blockIdx.x, divC, bk, c);
    const uint32_t b = bk / 4, k = bk % 4;
    const int L = H * W;
    const T *src = x + (size_t)blockIdx.x * L;
    T *dst = y + (int64_t)b * y_bs + (int64_t)k * y_ks + (int64_t)c * y_cs;
    if ((k & 1u) == 0) {
        for (int j = threadIdx.x; j < L; j += kBlock) dst[j] = src[k == 0 ? j : L - 1 - j];
        return;
    }
    if (use_lds) {
        for (int r = threadIdx.x; r < L; r += kBlock) {
            uint32_t h, w;
            divmod((uint32_t)r, divW, h, w);
            tile[h * Wp + w] = src[r];
        }
        __syncthreads();
    }
    for (int j = threadIdx.x; j < L; j += kBlock) {
        uint32_t w, h;
        divmod((uint32_t)(k == 1 ? j : L - 1 - j), divH, w, h);
        dst[j] = use_lds ? tile[h * Wp + w] : src[h * W + w];
    }
}

template <typename T>
static int launch_cross_scan_1b1(const void *x, void *y, int B, int C, int H, int W, int64_t y_bs, int64_t y_ks, int64_t y_cs,
                                 hipStream_t stream) {
    const int64_t n_wg = (int64_t)B * 4 * C;
    if (n_wg > 0x7fffffff) return SS2D_ENOTSUP;
    const int Wp = W | 1;
    size_t smem = (size_t)H * Wp * sizeof(T);
    const int use_lds = smem <= 48 * 1024;
    if (!use_lds) smem = 0;
    hipLaunchKernelGGL((cross_scan_1b1_kernel<T>), dim3((uint32_t)n_wg), dim3(kBlock), smem, stream, (const T *)x, (T *)y, H, W, Wp,
                       use_lds, y_bs, y_ks, y_cs, make_fastdiv((uint32_t)C), make_fastdiv((uint32_t)W), make_fastdiv((uint32_t)H));
    return launch_status();
}

}  // namespace ss2d

extern "C" int ss2d_cross_scan_1b1(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int64_t y_batch_stride,
                                   int64_t y_dir_stride, int64_t y_chan_stride, void *stream) {
    using namespace ss2d;
    if (B < 0 || C < 0 || H < 0 || W < 0) return SS2D_EINVAL;
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return SS2D_EINVAL;
    if (B == 0 || C == 0 || H == 0 || W == 0) return SS2D_OK;
    if (!x || !y) return SS2D_EINVAL;
    if ((int64_t)H * W > 0x3fffffff) return SS2D_ENOTSUP;
    if (y_batch_stride < 0 || y_dir_stride < 0 || y_chan_stride < 0) return SS2D_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    switch (elem_bytes) {
        case 1: return launch_cross_scan_1b1<uint8_t>(x, y, B, C, H, W, y_batch_stride, y_dir_stride, y_chan_stride, s);
        case 2: return launch_cross_scan_1b1<uint16_t>(x, y, B, C, H, W, y_batch_stride, y_dir_stride, y_chan_stride, s);
        case 4: return launch_cross_scan_1b1<uint32_t>(x, y, B, C, H, W, y_batch_stride, y_dir_stride, y_chan_stride, s);
        default: return launch_cross_scan_1b1<uint64_t>(x, y, B, C, H, W, y_batch_stride, y_dir_stride, y_chan_stride, s);
    }
}
