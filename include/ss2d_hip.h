/*
 * ss2d_hip.h -- C ABI of libss2d_hip.so: the SS2D inference hot path of VMamba
 * (CrossScan -> selective-scan forward -> CrossMerge) as hand-written HIP
 * kernels for gfx950 (MI355X).
 *
 * Conventions shared by every entry point
 *   - plain pointers and sizes, no framework types; every pointer is DEVICE memory
 *     on the device that is current for the calling thread;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); work is
 *     enqueued on it and the call returns without synchronising;
 *   - nothing is allocated, freed or synchronised inside the library; outputs are
 *     caller-allocated, inputs are only read;
 *   - re-entrant: no entry point keeps state between calls, so concurrent calls on
 *     different streams are independent -- with ONE exception, ss2d_cross_scan_flex_static,
 *     whose staging buffer is a device array owned by the library (one per GPU, its address
 *     cached per device on first use): calls of it that overlap on one GPU race on that array;
 *   - the return value is SS2D_OK or a negative SS2D_E* code (errno numbering); on
 *     error nothing has been launched.  No exception crosses this boundary.
 *
 * Each entry point replaces one native piece of the reference (file:line are paths
 * inside MzeroMiko/VMamba).
 */
#ifndef SS2D_HIP_H
#define SS2D_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SS2D_ABI_VERSION 1

/* element types */
#define SS2D_F32 0
#define SS2D_BF16 1
#define SS2D_F16 2

/* status codes */
#define SS2D_OK 0
#define SS2D_EINVAL (-22)  /* bad shape, stride, pointer or flag            */
#define SS2D_ENOTSUP (-95) /* valid request this build has no kernel for    */
#define SS2D_ELAUNCH (-5)  /* the HIP runtime refused the launch            */
#define SS2D_ENOMEM (-12)  /* the workspace is smaller than the call needs  */

/* CrossMerge association orders */
#define SS2D_MERGE_PAIRWISE 0      /* (y0 + flip y2) + T(y1 + flip y3): cross_merge_fwd,
                                      classification/models/csm_triton.py:61-62           */
#define SS2D_MERGE_LEFT_TO_RIGHT 1 /* ((y0 + T y1) + flip y2) + T flip y3: the Triton
                                      kernel, classification/models/csm_triton.py:362-370 */

/* Chunk length of the `x` (chunk-end state) output of the scan:
 * kernels/selective_scan/csrc/selective_scan/cusoflex/selective_scan_oflex.cpp:206 */
#define SS2D_SCAN_CHUNK 2048

int ss2d_abi_version(void);
const char *ss2d_strerror(int code);

/*
 * CrossScan, scans=0, channel-first in and out, not one-by-one.
 * Replaces the Triton launch CrossScanTritonF.forward
 * (classification/models/csm_triton.py:405-433, kernel :278-361); semantics of
 * cross_scan_fwd (csm_triton.py:22-29).
 *   x (B,C,H,W) contiguous  ->  y (B,4,C,H*W) contiguous, same element size:
 *   y[b,0,c,h*W+w] = y[b,1,c,w*H+h] = y[b,2,c,L-1-(h*W+w)] = y[b,3,c,L-1-(w*H+h)] = x[b,c,h,w]
 * elem_bytes in {1,2,4,8}; a pure permutation, bit-exact for any payload.
 * Empty tensors (any of B,C,H,W zero) are a no-op returning SS2D_OK.
 */
int ss2d_cross_scan(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, void *stream);

/*
 * CrossMerge, scans=0, channel-first in and out, not one-by-one.
 * Replaces CrossMergeTritonF.forward (csm_triton.py:458-481, kernel :362-370);
 * default semantics and rounding order of cross_merge_fwd (csm_triton.py:56-62).
 *   ys (B,4,C,H,W) contiguous -> out (B,C,H*W) contiguous, dtype in {F32,BF16,F16};
 *   every pairwise add is rounded to `dtype` (round-to-nearest-even), in the
 *   association order selected by `order`.
 */
int ss2d_cross_merge(const void *ys, void *out, int B, int C, int H, int W, int dtype, int order,
                     void *stream);

/*
 * Selective-scan forward ("oflex" flavour: output may be fp32 whatever the input).
 * Replaces selective_scan_fwd + selective_scan_fwd_kernel
 * (kernels/selective_scan/csrc/selective_scan/cusoflex/selective_scan_oflex.cpp:143-231,
 *  .../selective_scan_fwd_kernel_oflex.cuh:67-212); the struct mirrors SSMParamsBase
 * (.../selective_scan_oflex.h:26-61).  Strides are in ELEMENTS; the innermost
 * (sequence) stride of u, delta, B, C, out is 1.
 *
 *   u      (batch, dim, seqlen)              in_dtype
 *   delta  (batch, delta_dim, seqlen)        in_dtype; dim % delta_dim == 0, channel d reads
 *                                            row d / (dim/delta_dim)
 *   A      (dim, dstate)                     fp32
 *   B, C   (batch, n_groups, dstate, seqlen) in_dtype; dim % n_groups == 0, channel d reads
 *                                            group d / (dim/n_groups)
 *   D      (dim) fp32 or NULL;  delta_bias (delta_dim) fp32 or NULL
 *   out    (batch, dim, seqlen)              out_dtype: SS2D_F32 or in_dtype
 *   x      (batch, dim, n_chunks, 2*dstate)  fp32 contiguous or NULL (skip);
 *          n_chunks = ceil(seqlen / SS2D_SCAN_CHUNK); x[..,2n] = product of a since t=0,
 *          x[..,2n+1] = h_n, both at the end of the chunk (last state = x[:,:,-1,1::2])
 *
 *   dl = delta + delta_bias;  if delta_softplus: dl = dl > 20 ? dl : log1p(exp(dl))
 *   h_n[t] = exp(dl*A[d,n]) * h_n[t-1] + dl*B[n,t]*u[t];   out[t] = sum_n C[n,t]*h_n[t] + D[d]*u[t]
 * State and arithmetic are fp32.  dstate <= 256 (selective_scan_oflex.cpp:180).
 */
typedef struct ss2d_scan_params {
    int32_t batch, dim, seqlen, dstate, n_groups, delta_dim;
    int32_t in_dtype, out_dtype;
    int32_t delta_softplus;
    int32_t reserved;
    const void *u, *delta, *A, *B, *C, *D, *delta_bias;
    void *out;
    void *x;
    int64_t u_batch_stride, u_d_stride;
    int64_t delta_batch_stride, delta_d_stride;
    int64_t A_d_stride, A_dstate_stride;
    int64_t B_batch_stride, B_group_stride, B_dstate_stride;
    int64_t C_batch_stride, C_group_stride, C_dstate_stride;
    int64_t out_batch_stride, out_d_stride;
} ss2d_scan_params;

int ss2d_selective_scan_fwd(const ss2d_scan_params *params, void *stream);

/*
 * Which kernel ss2d_selective_scan_fwd would launch for `params` (the same validation, nothing is launched):
 * one of the ids below, or a negative SS2D_E* code.  Every kernel writes `x` when it is requested, so the answer
 * does not depend on params->x.  No counterpart in the reference (its one kernel template serves every shape,
 * selective_scan_oflex.cpp:224-226); here so that a caller, a benchmark or a test can tell which code path a
 * shape takes.
 */
#define SS2D_SCAN_KERNEL_NONE 0  /* empty problem: nothing to launch                                           */
#define SS2D_SCAN_KERNEL_ROW 1   /* one wavefront per (batch, channel) row                                       */
#define SS2D_SCAN_KERNEL_ROW4 2  /* few long rows: the four wavefronts of a workgroup share a row                */
#define SS2D_SCAN_KERNEL_FLAT 3  /* short or unaligned rows walked several to a wavefront as one stream          */
#define SS2D_SCAN_KERNEL_SMALL 4 /* rows of 49 / 196 positions, one state: a segment of a row per lane           */
#define SS2D_SCAN_KERNEL_CHAN 5  /* several states per channel: one channel per lane, positions walked serially  */
int ss2d_selective_scan_kernel(const ss2d_scan_params *params);

/*
 * The same forward with CrossScan folded in, for several states per channel: params->u is not the (batch, dim, seqlen)
 * tensor of the four scan-ordered copies (cross_scan_fn's output, classification/models/vmamba.py:604, 625) but the map
 * itself, x (batch, dim / 4, seqlen) with u_batch_stride / u_d_stride its strides, and x_t (same strides) holds every
 * height x width map transposed (width x height).  n_groups must be 4 and group k is scan direction k: its channels
 * read x (k = 0, 2) or x_t (k = 1, 3), forwards (k < 2) or backwards (cross_scan_fwd, csm_triton.py:22-29).  Everything
 * else as ss2d_selective_scan_fwd.  Served by the channel-per-lane kernel only (dstate 4 / 8 / 16 / 32, seqlen a multiple
 * of 8, dim / 4 >= 32, 16-byte aligned rows): SS2D_ENOTSUP otherwise.
 */
int ss2d_selective_scan_fwd_maps(const ss2d_scan_params *params, const void *x_t, void *stream);

/*
 * Selective-scan backward.  Replaces selective_scan_bwd + selective_scan_bwd_kernel
 * (kernels/selective_scan/csrc/selective_scan/cusoflex/selective_scan_oflex.cpp:233-355,
 *  .../selective_scan_bwd_kernel_oflex.cuh); inputs as in the forward plus
 *   dout   (batch, dim, seqlen)   dout_dtype: SS2D_F32 or in_dtype (strides in elements, sequence stride 1)
 * and caller-allocated outputs
 *   du, ddelta  (batch, dim, seqlen) contiguous, in_dtype; ddelta is per CHANNEL (with delta_dim < dim the caller
 *               sums the dim/delta_dim channels of a delta row, as selective_scan_oflex.cpp:347-352 does)
 *   dA (dim, dstate), dB, dC (batch, n_groups, dstate, seqlen), dD (dim), ddelta_bias (dim): fp32, contiguous,
 *               ZERO-INITIALISED by the caller (accumulated with atomics over the rows that share them);
 *               dD / ddelta_bias NULL exactly when D / delta_bias is NULL.
 * The forward states are recomputed inside the kernel, so the forward's `x` output is not needed.
 * Returns SS2D_ENOTSUP when ceil(seqlen/512) * dstate exceeds ~3000 (per-pass states kept in LDS).
 */
typedef struct ss2d_scan_bwd_params {
    int32_t batch, dim, seqlen, dstate, n_groups, delta_dim;
    int32_t in_dtype, dout_dtype;
    int32_t delta_softplus;
    int32_t reserved;
    const void *u, *delta, *A, *B, *C, *D, *delta_bias, *dout;
    void *du, *ddelta, *dA, *dB, *dC, *dD, *ddelta_bias;
    int64_t u_batch_stride, u_d_stride;
    int64_t delta_batch_stride, delta_d_stride;
    int64_t A_d_stride, A_dstate_stride;
    int64_t B_batch_stride, B_group_stride, B_dstate_stride;
    int64_t C_batch_stride, C_group_stride, C_dstate_stride;
    int64_t dout_batch_stride, dout_d_stride;
} ss2d_scan_bwd_params;

int ss2d_selective_scan_bwd(const ss2d_scan_bwd_params *params, void *stream);

/*
 * LayerNorm over the channel axis, the step after CrossMerge (out_norm) and the block norms of the model.
 * Replaces the torch calls of LayerNorm2d.forward (classification/models/vmamba.py:52-57: permute,
 * F.layer_norm, permute) and of nn.LayerNorm on (B,H,W,C) activations, including the transposition
 * forward_core does before out_norm in channel-last models (vmamba.py:642-644).
 *   y = (x - mean) * rsqrt(var + eps) * weight + bias, mean / biased var over the C channels, fp32 statistics
 *   and arithmetic for every I/O type; weight / bias (C) may be NULL.
 * Supported (in, weight, out) dtype triples: (f32,f32,f32) (f32,f32,bf16) (f32,bf16,bf16) (f32,bf16,f32)
 * (bf16,bf16,bf16) (bf16,f32,bf16) (f32,f16,f16) (f16,f16,f16) (f16,f32,f16); others return SS2D_ENOTSUP.
 *
 * ss2d_layer_norm:    x, y (rows, C) contiguous.
 * ss2d_layer_norm_cf: x (B,C,L) contiguous, channel-first; y (B,L,C) if out_channel_last else (B,C,L).
 */
int ss2d_layer_norm(const void *x, const void *weight, const void *bias, void *y, int64_t rows, int C, float eps,
                    int in_dtype, int w_dtype, int out_dtype, void *stream);
/*
 * Residual add and LayerNorm in one pass: sum_out = x + residual (rounded to the input type, as the separate add of
 * classification/models/vmamba.py:1228 would leave it), y = LayerNorm(sum_out) (:1229 norm2).  Same dtype triples as
 * ss2d_layer_norm; rows must be vectorisable (C % 8 == 0, C <= 1024, 16-byte aligned pointers), else SS2D_ENOTSUP.
 */
int ss2d_add_layer_norm(const void *x, const void *residual, const void *weight, const void *bias, void *sum_out, void *y,
                        int64_t rows, int C, float eps, int in_dtype, int w_dtype, int out_dtype, void *stream);
/*
 * Per-channel bias add and LayerNorm in one pass: y = LayerNorm(x + pre_bias), pre_bias (C) of the weight type, the sum
 * rounded to the input type as a separate add would leave it.  Serves the convolution bias of the patch-embedding and
 * downsampling layers, each a Conv2d directly followed by a LayerNorm (classification/models/vmamba.py:1403-1417,
 * 1430-1437): the convolution then runs without its bias.  Same dtype triples and row conditions as
 * ss2d_add_layer_norm.
 */
int ss2d_bias_layer_norm(const void *x, const void *pre_bias, const void *weight, const void *bias, void *y, int64_t rows,
                         int C, float eps, int in_dtype, int w_dtype, int out_dtype, void *stream);
int ss2d_layer_norm_cf(const void *x, const void *weight, const void *bias, void *y, int B, int C, int L, float eps,
                       int in_dtype, int w_dtype, int out_dtype, int out_channel_last, void *stream);

/*
 * Depthwise 3x3 convolution (stride 1, zero padding 1) + optional bias + optional SiLU: the two ops in front of
 * forward_core in SS2Dv2.forwardv2 (classification/models/vmamba.py:654-658: permute to channel-first,
 * self.conv2d (groups = d_inner), self.act), fused with the layout change.
 *   x (B,H,W,D) if in_channel_last else (B,D,H,W); weight (D,1,3,3); bias (D) or NULL; all of `dtype`
 *   y (B,D,H,W), channel-first.  fp32 accumulation; the convolution result is rounded to `dtype` before SiLU.
 */
int ss2d_dwconv3x3_silu(const void *x, const void *weight, const void *bias, void *y, int B, int D, int H, int W,
                        int dtype, int in_channel_last, int apply_silu, void *stream);

/*
 * CrossScan, one-by-one, scans=0, channel-first: every direction slice of the input is put in ITS scan order.
 * Replaces CrossScanTriton1b1.forward / cross_scan1b1_fwd (classification/models/csm_triton.py:88-131, 400-436).
 *   x (B,4,C,H,W) contiguous -> y[b*y_batch_stride + k*y_dir_stride + c*y_chan_stride + j], j in [0, L):
 *   y[b,0,c,h*W+w] = x[b,0,c,h,w];  y[b,1,c,w*H+h] = x[b,1,c,h,w];
 *   y[b,2,c,L-1-(h*W+w)] = x[b,2,c,h,w];  y[b,3,c,L-1-(w*H+h)] = x[b,3,c,h,w]
 * Strides in elements; (4*C*L, C*L, L) is the reference's contiguous (B,4,C,L).  Other strides let the caller
 * produce e.g. the direction-major, batch-innermost (4,C,B,L) layout ss2d_core_fwd reads.  elem_bytes in {1,2,4,8}.
 */
int ss2d_cross_scan_1b1(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int64_t y_batch_stride,
                        int64_t y_dir_stride, int64_t y_chan_stride, void *stream);

/*
 * Fused SS2D core for dstate = 1: CrossScan -> selective scan (softplus, fp32 state, fp32 "oflex" output) ->
 * CrossMerge in one kernel.  Replaces the three calls of SS2Dv2.forward_corev2
 * (classification/models/vmamba.py:604, 625-633, 638: cross_scan_fn, selective_scan, cross_merge_fn) for
 * scans=0 / d_state=1; the projections between them (vmamba.py:605-615) stay the caller's GEMMs and are handed
 * over already in scan order:
 *   x      (batch, dim, height, width) contiguous, in_dtype: the conv+SiLU output; read once, never expanded
 *   delta  [k*delta_dir_stride + d*delta_dim_stride + b*delta_batch_stride + j]  in_dtype, j = scan position
 *          of direction k (dt_proj output before bias and softplus)
 *   B, C   [k*dir_stride + b*batch_stride + j]  in_dtype (x_proj's B and C rows: one state, one group per direction)
 *   A, D, delta_bias (4*dim) fp32, index k*dim + d; D and delta_bias may be NULL
 *   y      (batch, dim, height*width) contiguous fp32:
 *          y = (y_0 + flip(y_2)) + transpose(y_1 + flip(y_3)), y_k the scan output of direction k, each add
 *          rounded to fp32 -- cross_merge_fwd's order (csm_triton.py:56-62) on the oflex fp32 scan outputs.
 * Strides in elements.  The kernel walks several images per workgroup when delta_batch_stride == height*width
 * (batch-innermost layout) and falls back to one image per workgroup otherwise.  Returns SS2D_ENOTSUP when the
 * image does not fit the kernel's LDS arrays (height*width above ~13000 for 16-bit inputs, ~9700 for fp32) or has
 * fewer than 8 positions.
 */
typedef struct ss2d_core_params {
    int32_t batch, dim, height, width;
    int32_t in_dtype;
    int32_t delta_softplus;
    const void *x, *delta, *A, *B, *C, *D, *delta_bias;
    void *y;
    int64_t delta_dir_stride, delta_dim_stride, delta_batch_stride;
    int64_t B_dir_stride, B_batch_stride;
    int64_t C_dir_stride, C_batch_stride;
} ss2d_core_params;

int ss2d_core_fwd(const ss2d_core_params *params, void *stream);

/*
 * The same operator for maps of any size.  Maps that do not fit the single kernel's LDS arrays (e.g. the 256 x 256 and
 * 128 x 128 maps of a 1024 x 1024 image) are cut into 64 x 64 tiles and walked twice -- per-run aggregates, a carry scan
 * over them, then the outputs -- which needs scratch memory: ss2d_core_workspace_bytes returns how much (0 when the
 * single kernel serves the problem and no workspace is needed, SS2D_ENOTSUP when neither path does: the tiled one takes
 * 16-bit inputs, height and width multiples of 8, every stride a multiple of 8 elements and 16-byte aligned
 * pointers), and ss2d_core_fwd_ws takes that workspace (16-byte aligned device memory; SS2D_ENOMEM when it is too
 * small; contents need no initialisation and mean nothing afterwards).  The reference reaches every length with one
 * kernel by looping over 2048-position chunks (selective_scan_fwd_kernel_oflex.cuh:110-111, 156-167;
 * selective_scan_oflex.cpp:206); results as ss2d_core_fwd.
 */
int64_t ss2d_core_workspace_bytes(const ss2d_core_params *params);
int ss2d_core_fwd_ws(const ss2d_core_params *params, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Maps whose sides do not suit the core's vector paths (57 x 58 -- the reference's own check size,
 * classification/models/csm_triton.py:524, 670 -- 75 x 75, 19 x 19 ...) can be embedded by the caller in a map of
 * padded_height x padded_width >= height x width: x = 0 on the added rows / columns, the projections computed on the
 * padded map, and the step made 0 on the added positions, which makes them neutral elements of the scan (decay 1,
 * drive 0): the outputs at the original positions are those of the original map.  This call writes delta = -infinity
 * (softplus(-inf + bias) = 0) at the added positions of each direction's scan order; delta as in ss2d_core_params,
 * over the padded map; delta_softplus must be on.  No counterpart in the reference, whose kernels take any length
 * element by element.
 */
int ss2d_core_mask_pads(void *delta, int batch, int dim, int height, int width, int padded_height, int padded_width,
                        int64_t delta_dir_stride, int64_t delta_dim_stride, int64_t delta_batch_stride, int dtype, void *stream);

/*
 * The copies around such an embedding, each as one pass: dst[m][r][c] = src[m][r][c] where the source map has that row
 * and column, 0 elsewhere, for n_maps dense maps of src_rows x src_cols resp. dst_rows x dst_cols elements of 2 or 4
 * bytes.  A larger destination is the zero-padded map (what F.pad would make of x for vmamba.py:604), a smaller one the
 * crop of a result; a channel-last activation (B, H, W, D) is B maps of H rows of W * D elements.  Fewer than 2^32
 * elements on either side.  No counterpart in the reference.
 */
int ss2d_core_embed_maps(const void *src, void *dst, int64_t n_maps, int src_rows, int64_t src_cols, int dst_rows,
                         int64_t dst_cols, int elem_bytes, void *stream);

/*
 * CrossScan / CrossMerge for every layout and mode of the reference operators (cross_scan_fn / cross_merge_fn,
 * classification/models/csm_triton.py:501-517; semantics of the flex kernel :278-400 and of the torch functions
 * :22-179).  Flags are named from the scan's side, as in the reference, for both operations:
 *   x_channel_last   0: x is (B,[4,]C,H,W)      1: x is (B,H,W,[4,]C)        ("in_channel_first" negated)
 *   y_channel_last   0: y is (B,4,C,H*W)        1: y is (B,H*W,4,C)          ("out_channel_first" negated)
 *   one_by_one       x has one slice per direction (the bracketed 4) instead of one shared map
 *   scans            0: row-major, column-major, both reversed;  1: row-major four times;  2: row-major twice,
 *                    reversed twice
 * scan:   y_k[route_k(h,w)] = x_(k)[h,w]                       (a permutation / replication; any 1/2/4/8-byte type)
 * merge:  x[h,w] = sum_k y_k[route_k(h,w)]  (one_by_one: x_k[h,w] = y_k[route_k(h,w)], no sum), dtype F32/BF16/F16.
 *         Rounding: scans 0 and 2 add pairwise, (y0 + y2) + (y1 + y3), each add rounded to dtype (order = PAIRWISE,
 *         the torch functions) or left to right (order = LEFT_TO_RIGHT, the Triton kernel); scans 1 accumulates the
 *         four terms in fp32 and rounds once (a torch reduction, csm_triton.py:64).
 * The default combination (0, 0, 0, 0) is also served by the tiled kernels behind ss2d_cross_scan / ss2d_cross_merge.
 */
int ss2d_cross_scan_flex(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int x_channel_last,
                         int y_channel_last, int one_by_one, int scans, void *stream);
int ss2d_cross_merge_flex(const void *y, void *x, int B, int C, int H, int W, int dtype, int x_channel_last,
                          int y_channel_last, int one_by_one, int scans, int order, void *stream);

/*
 * ss2d_cross_scan_flex with a staging buffer for the mixed-layout modes (x channel-first and y channel-last, or the
 * reverse: the permute(...).contiguous() the reference inserts, classification/models/csm_triton.py:48-51, 116-119).
 * The x-side tensor is first transposed into `workspace` (the layout of y), then the same-layout kernel runs: two
 * copy-shaped launches instead of one gather through L2 (4-5x faster at model shapes).  Results are identical to
 * ss2d_cross_scan_flex (a permutation).  `workspace`: device memory, 16-byte aligned, at least
 * B * (one_by_one ? 4 : 1) * C * H * W * elem_bytes bytes; it is scratch (contents undefined afterwards) and must not be
 * used by other work until the call's launches have finished.  SS2D_ENOMEM when workspace_bytes is too small.  When the two
 * layouts agree the workspace is not touched (it may be NULL) and the call is ss2d_cross_scan_flex.
 */
int ss2d_cross_scan_flex_ws(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int x_channel_last,
                            int y_channel_last, int one_by_one, int scans, void *workspace, int64_t workspace_bytes,
                            void *stream);

/*
 * ss2d_cross_scan_flex_ws without the workspace argument: the staging buffer is a fixed array of
 * SS2D_STATIC_STAGING_BYTES in device memory that belongs to the library (each GPU the library runs on holds its own
 * copy until the process ends).  This entry point has no counterpart in the reference; it exists for callers that
 * cannot allocate device memory around the call -- code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It calls no hipMalloc / hipFree or any allocating routine.  Same results as
 * ss2d_cross_scan_flex.  SS2D_ENOMEM when the x-side tensor, B * (one_by_one ? 4 : 1) * C * H * W * elem_bytes bytes,
 * exceeds SS2D_STATIC_STAGING_BYTES (nothing is launched then); same-layout modes need no staging and have no limit.
 * All calls on one GPU share that GPU's array: calls whose launches can overlap on one GPU (different streams without
 * an ordering between them) race on it.  The first call on a device looks up the array's address; make that call
 * outside a graph capture.
 */
#define SS2D_STATIC_STAGING_BYTES (80 << 20)
int ss2d_cross_scan_flex_static(const void *x, void *y, int B, int C, int H, int W, int elem_bytes, int x_channel_last,
                                int y_channel_last, int one_by_one, int scans, void *stream);

/*
 * Batched transpose (B, R, S) -> (B, S, R), any 1/2/4/8-byte element: the layout change between channel-first
 * (B, C, L) and channel-last (B, L, C) activations -- the permute(...).contiguous() of cross_scan_fwd / cross_merge_fwd
 * for mixed layouts (classification/models/csm_triton.py:48-51, 80-83).  The host serves the mixed-layout modes as
 * this transpose of the small x-side tensor plus the same-layout kernel.
 */
int ss2d_transpose_bcl(const void *x, void *y, int B, int R, int S, int elem_bytes, void *stream);

/*
 * First layer of the patch embedding in one pass (classification/models/vmamba.py:1403-1411, patch-embed v2:
 * Conv2d(3, Cout, kernel 3, stride 2, padding 1) -> permute -> LayerNorm(Cout) -> permute -> GELU):
 *   y = GELU(LayerNorm(conv2d(x, weight, bias))), exact (erf) GELU, the three results rounded to dtype in turn.
 *   x (B, 3, H, W) contiguous; weight (Cout, 3, 3, 3) taken through weight_strides[4] (elements: out channel, in
 *   channel, tap row, tap column -- contiguous or channels-last weights alike); bias, ln_weight, ln_bias (Cout) or
 *   NULL; y (B, Ho, Wo, Cout) contiguous, channel-last, Ho = (H - 1)/2 + 1, Wo = (W - 1)/2 + 1.
 * dtype SS2D_BF16 or SS2D_F16 for all tensors, Cout 48 or 64; anything else returns SS2D_ENOTSUP.
 */
int ss2d_stem_conv_ln_gelu(const void *x, const void *weight, const int64_t *weight_strides, const void *bias,
                           const void *ln_weight, const void *ln_bias, float eps, void *y, int B, int H, int W, int Cout,
                           int dtype, void *stream);

/*
 * dt_proj of the SS2D core: the per-direction rank-R -> D projection between x_proj and the scan.
 * Replaces the grouped conv1d / einsum of SS2Dv2.forward_corev2 (classification/models/vmamba.py:608-609, 614-615):
 *   delta[k, d, n] = sum_r weight[k, d, r] * x[k*x_dir_stride + r*x_rank_stride + n]
 *   weight (K, D, R) contiguous; delta (K, D, N) contiguous; x rows contiguous along n (N = batch * L positions).
 * dtype SS2D_BF16 or SS2D_F16 for all three tensors; products accumulate in fp32 on the matrix cores and are
 * rounded once to dtype, as in the library GEMM.  SS2D_F32 and R > 48 return SS2D_ENOTSUP (use a library GEMM).
 */
int ss2d_dt_proj(const void *x, const void *weight, void *delta, int K, int D, int R, int64_t N, int64_t x_dir_stride,
                 int64_t x_rank_stride, int dtype, void *stream);

/*
 * The same projection with chosen positions overwritten: mask is (K, N) 16-bit words, each 0 or 0xffff, and where a word
 * is set every channel's delta at that position becomes `fill` (rounded to dtype) instead of the projection; mask == NULL
 * is ss2d_dt_proj.  For maps with awkward sides that run embedded in padded maps (SS2Dv2.forward_corev2 takes any H x W,
 * classification/models/vmamba.py:603-640): a delta of -1e30 at the pad positions is a step of exactly 0 after the
 * softplus, i.e. the identity of the recurrence, so the embedded map's states pass the pads unchanged.
 */
int ss2d_dt_proj_masked(const void *x, const void *weight, const void *mask, float fill, void *delta, int K, int D, int R,
                        int64_t N, int64_t x_dir_stride, int64_t x_rank_stride, int dtype, void *stream);

/*
 * Fused channel-last MLP of a VSS block: out = residual + fc2(GELU(fc1([LayerNorm](x)))) in one kernel, the hidden
 * activations never leaving the registers.  Replaces Mlp.forward (classification/models/vmamba.py:1116-1131: fc1, GELU
 * (erf form), fc2), the residual add of VSSBlock (:1229) and, when ln_weight is given, the block's second LayerNorm
 * (:1229 norm2) for the narrow stages.
 *   x, residual (may be NULL), out: (M, C) contiguous;  w1 (4C, C), b1 (4C) or NULL;  w2 (C, 4C), b2 (C) or NULL;
 *   ln_weight (C) or NULL = no LayerNorm, ln_bias (C) or NULL, eps;  all SS2D_BF16 or all SS2D_F16, 16-byte aligned.
 *   LayerNorm output, fc1 output, GELU output, fc2 output and the sum are each rounded to the tensor type, as the
 *   unfused operators would; LayerNorm statistics are fp32.
 * C must be 96 or 192 (wider layers are compute-bound and stay library GEMMs): anything else, and SS2D_F32,
 * returns SS2D_ENOTSUP.
 */
int ss2d_mlp_fused(const void *x, const void *ln_weight, const void *ln_bias, float eps, const void *w1, const void *b1,
                   const void *w2, const void *b2, const void *residual, void *out, int64_t M, int C, int dtype,
                   void *stream);

/*
 * Narrow channel-last projection with its neighbours folded in:  out = [LayerNorm](x) W^T + bias + residual.
 * Replaces, in a VSS block, norm + in_proj (classification/models/vmamba.py:1225-1227 ln_1, :648-650 in_proj) and
 * out_proj + the residual add (:662, :1228) where the layer is too narrow for a library GEMM to reach the HBM bound.
 *   x (M, K), residual (M, N) or NULL, out (M, N) contiguous;  weight (N, K);  bias (N) or NULL;
 *   ln_weight (K) or NULL = no LayerNorm, ln_bias (K) or NULL, eps;  all SS2D_BF16 or all SS2D_F16, 16-byte aligned.
 *   LayerNorm output, projection output and the sum are each rounded to the tensor type, as the separate operators
 *   would; statistics are fp32.
 * K = N = 96 only: anything else, and SS2D_F32, returns SS2D_ENOTSUP.
 */
int ss2d_linear_cl(const void *x, const void *ln_weight, const void *ln_bias, float eps, const void *weight,
                   const void *bias, const void *residual, void *out, int64_t M, int K, int N, int dtype, void *stream);

/*
 * The same projection fed by the SS2D core: x is the fp32 channel-first map (B, K, L) that ss2d_core_fwd (or
 * CrossMerge) leaves, the LayerNorm is the block's out_norm over the K channels of each position, computed from the
 * fp32 values and rounded to dtype as the separate operator does (classification/models/vmamba.py:641-646), and
 * out (B*L, N) = out_norm(x) weight^T + bias + residual is the block's out_proj with its residual add (:662, :1228).
 * dtype (weights, residual, out) SS2D_BF16 or SS2D_F16; K = N = 96 and L a multiple of 32, else SS2D_ENOTSUP.
 */
int ss2d_linear_cf_ln(const void *x, const void *ln_weight, const void *ln_bias, float eps, const void *weight,
                      const void *bias, const void *residual, void *out, int B, int L, int K, int N, int dtype, void *stream);

/*
 * Global average pool of a channel-last map: y (B, C) = mean over the L positions of x (B, L, C), fp32 sum times 1/L
 * rounded once to dtype -- the AdaptiveAvgPool2d(1) of the classifier head (classification/models/vmamba.py:1357-1363)
 * on the channel-last activation.  One pass, no workspace, no counters: the result does not depend on scheduling.
 * dtype SS2D_BF16 or SS2D_F16, C a multiple of 8, x 16-byte aligned; anything else returns SS2D_ENOTSUP.
 */
int ss2d_mean_pool_cl(const void *x, void *y, int B, int L, int C, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SS2D_HIP_H */
