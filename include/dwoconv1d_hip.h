/*
 * libdwoconv1d_hip.so -- C ABI of the MI355X (gfx950) depthwise oriented 1D convolution.
 *
 * This is the boundary a binding of the reference's operator module would call in place
 * of the five functions its JIT-built extension exports
 * (models/dwoconv1d/dwoconv1d_kernel.py:29-36,54-60: fprop, dgrad, wgrad, nhwc_to_nchw,
 * nchw_to_nhwc).  Plain pointers and sizes only; the library never allocates, frees or
 * retains device memory: the caller owns inputs, outputs and scratch.  Every launch is
 * asynchronous on the stream passed in (the reference launches on the current stream,
 * models/dwoconv1d/kernels/kernels.cu:25).
 *
 * First use.  The first launch of a kernel on a device queries its occupancy and sets its
 * dynamic-LDS attribute, which a stream capture does not allow.  Call dwo_init() once per
 * device (with that device current) before capturing calls into a graph; without it the set-up
 * happens lazily inside the first call of each entry point on each shape class.  Each launching
 * entry point clears the calling thread's HIP last-error state on entry, so the positive
 * status it returns always belongs to its own launches.
 *
 * Tap blobs.  `taps` arguments are device copies of a blob built by dwo_build_taps for the
 * same C and K as the call; the kernels index the blob with the call's C and K and cannot
 * verify its header, so a blob of another size leads to out-of-range reads.  The caller checks
 * the size (dwo_taps_bytes) before launching.
 *
 * Operator definition (models/dwoconv1d_reference/kernels/kernels.cpp:36-52,71-90,111-126),
 * pad = K/2, P = ceil(H/stride), Q = ceil(W/stride):
 *   dh(s) = (int)(-sinf(theta_c) * (s - pad)),  dw(s) = (int)(cosf(theta_c) * (s - pad))
 *   fprop: y[n,c,p,q]  = sum_s x[n,c,p*stride+dh(s),q*stride+dw(s)] * w[c,s]   (taps outside = 0)
 *   dgrad: dx[n,c,h,w] = sum_s dy[n,c,(h-dh(s))/stride,(w-dw(s))/stride] * w[c,s]
 *                        (only taps whose two numerators are divisible by stride and in range)
 *   wgrad: dw[c,s]     = sum_{n,p,q} x[n,c,p*stride+dh(s),q*stride+dw(s)] * dy[n,c,p,q]
 *
 * Layouts: DWO_NCHW tensors are [N,C,H,W]; DWO_NHWC tensors are [N,H,W,C].  The NHWC entry
 * points read and write NHWC directly, which replaces the reference's transpose passes
 * (models/dwoconv1d/kernels/kernels.cu:56-68, nhwc_utils.h:46-110).
 * Element types: activations x, y, dy, dx are fp32, bf16 or fp16; weights, bias, dw and db
 * are always passed as fp32 and all accumulation is fp32.  With 16-bit activations the
 * row-direction orientations of the stride-1 plane kernels multiply through a two-element dot
 * product whose operands are both in the activation type: there the weights are rounded to
 * that type first (the reference holds the weights in the activation type throughout,
 * models/dwoconv1d/kernels/kernels.cu:25); the error stays within the 16-bit tolerance.
 */
#ifndef DWOCONV1D_HIP_H
#define DWOCONV1D_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes: 0 ok, negative = argument error, positive = hipError_t of the launch */
#define DWO_OK 0
#define DWO_ERR_NULL_POINTER (-1)
#define DWO_ERR_BAD_SHAPE (-2)    /* N,C,H,W < 1 or sizes overflow int32 indexing */
#define DWO_ERR_BAD_KERNEL (-3)   /* K even, < 1 or > DWO_MAX_K */
#define DWO_ERR_BAD_STRIDE (-4)   /* stride not in {1,2,4} */
#define DWO_ERR_BAD_DTYPE (-5)
#define DWO_ERR_BAD_LAYOUT (-6)
#define DWO_ERR_SCRATCH_TOO_SMALL (-7)
#define DWO_ERR_BAD_TAPS (-8)     /* host-side tap blob does not match C,K */
#define DWO_ERR_STATIC_SCRATCH_LIMIT (-9) /* dwo_wgrad_static: partial sums exceed the static scratch */

#define DWO_MAX_K 63

#define DWO_F32 0
#define DWO_BF16 1
#define DWO_F16 2

#define DWO_NCHW 0
#define DWO_NHWC 1

/* Library version (major*10000 + minor*100 + patch). */
int dwo_version(void);

/* Human-readable text for a status returned by any entry point. */
const char *dwo_status_string(int status);

/*
 * One-time set-up of every kernel on the current device (occupancy queries, dynamic-LDS
 * attributes), so that later calls only launch kernels and can be captured into a graph.
 * Replaces nothing the reference's extension exports: there the set-up is the JIT build plus
 * the cudaFuncSetAttribute of every launcher call (models/dwoconv1d/kernels/kernels.h:520-531).
 * Idempotent and thread-safe; call once per device with that device current.
 */
int dwo_init(void);

/*
 * Host-side tap table.  Replaces the per-thread sincosf + truncation of the reference
 * kernels (models/dwoconv1d/kernels/kernels.h:240-241,285-287) with one table computed
 * on the host in fp32 exactly as kernels.cpp:37,43-44 does.  `theta_host` holds C angles
 * in radians.  The caller copies the `dwo_taps_bytes(C,K)`-byte blob to device memory and
 * passes that device pointer as `taps` below; the blob's layout is private to the library.
 */
size_t dwo_taps_bytes(int C, int K);
int dwo_build_taps(const float *theta_host, int C, int K, void *taps_host);

/* Debug/inspection helper: (dh,dw) of channel c, tap s from a host blob. */
int dwo_taps_get(const void *taps_host, int c, int s, int *dh, int *dw);

/*
 * fprop -- replaces `fprop(x, w, theta)` (models/dwoconv1d/kernels/kernels.cu:15-27) plus
 * the separate bias add of models/dwoconv1d/dwoconv1d.py:34-35 when `bias` is non-NULL.
 * x: [N,C,H,W] or [N,H,W,C] `dtype`; w: [C,K] fp32; bias: [C] fp32 or NULL;
 * y: [N,C,P,Q] or [N,P,Q,C] `dtype`.
 */
int dwo_fprop(const void *x, const float *w, const float *bias, const void *taps, void *y,
              int N, int C, int H, int W, int K, int stride, int dtype, int layout,
              void *stream);

/*
 * dgrad -- replaces `dgrad(dy, w, theta)` (models/dwoconv1d/kernels/kernels.cu:29-40).
 * dy: [N,C,P,Q] / [N,P,Q,C]; dx: [N,C,H,W] / [N,H,W,C]; H,W are the input extents.
 */
int dwo_dgrad(const void *dy, const float *w, const void *taps, void *dx,
              int N, int C, int H, int W, int K, int stride, int dtype, int layout,
              void *stream);

/*
 * wgrad -- replaces `wgrad(dy, x, theta)` (models/dwoconv1d/kernels/kernels.cu:42-54) and,
 * when `db` is non-NULL, the bias gradient `dy.sum([0,2,3])` of dwoconv1d.py:66-67.
 * Deterministic: workgroups write partial sums into `scratch` (`dwo_wgrad_scratch_bytes`
 * bytes, caller-allocated, contents undefined on entry and exit) and the partial sums of a
 * channel are added in a fixed order -- no floating-point atomics, unlike
 * models/dwoconv1d/kernels/kernels.h:504-517.  For the stride-1 plane shapes that addition
 * happens inside the same kernel (the last workgroup of a channel to finish does it, found by
 * an integer counter in device memory the library owns); otherwise, and always under stream
 * capture, a second small kernel does it.  Both give the same bits.
 * dw: [C,K] fp32 (fully overwritten); db: [C] fp32 or NULL.
 *
 * Concurrency.  Calls on one stream are ordered.  Calls on different streams may overlap as long
 * as they do not share `scratch` (or `dw`/`db`): the library's counters belong to the stream
 * (the first 64 streams that call wgrad on a device each get a set; calls on further streams,
 * on hipStreamPerThread and under capture use the second kernel instead), so no two launches
 * that can run at the same time count on the same counters.  A captured graph contains no
 * reference to library-owned memory.
 */
size_t dwo_wgrad_scratch_bytes(int N, int C, int H, int W, int K, int stride, int dtype,
                               int layout);
int dwo_wgrad(const void *dy, const void *x, const void *taps, float *dw, float *db,
              void *scratch, size_t scratch_bytes,
              int N, int C, int H, int W, int K, int stride, int dtype, int layout,
              void *stream);

/*
 * wgrad without any device allocation by caller or library -- no counterpart in the reference.
 * It is for callers that cannot allocate: code under stream capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Same results as dwo_wgrad (bit for bit: the same kernels),
 * with the partial sums kept in a DWO_STATIC_SCRATCH_BYTES array in device memory that is part
 * of the library image (one copy per GPU, held until the process ends).  Shapes whose
 * dwo_wgrad_scratch_bytes exceed it are refused with DWO_ERR_STATIC_SCRATCH_LIMIT.  Every call on a
 * GPU shares that GPU's array: calls that overlap in time on one GPU (different streams or
 * threads) race; calls on one stream are ordered.  Nothing in the array has to survive between
 * calls and nothing in it has to be cleared.
 */
#define DWO_STATIC_SCRATCH_BYTES (8u << 20)
int dwo_wgrad_static(const void *dy, const void *x, const void *taps, float *dw, float *db,
                     int N, int C, int H, int W, int K, int stride, int dtype, int layout,
                     void *stream);

/*
 * Where the partial sums of the stride-1 plane wgrad kernels are added up: in_kernel != 0 (the
 * default) inside the kernel that produced them, 0 in a second kernel.  The results are
 * bit-identical; the switch exists so that both paths can be exercised and compared.  No
 * counterpart in the reference.  Process-wide; returns the previous setting.
 */
int dwo_set_wgrad_reduction(int in_kernel);

/*
 * fprop of a pointwise-projected NHWC tensor without materialising it: y = fprop(pw(x)) with
 * pw(x)[n,h,w,c] = pw_b[c] + sum_k x[n,h,w,k] * pw_w[c,k], rounded to the activation type as the
 * separate layer's output would be.  The stem's first two layers of the reference
 * (models/convnext.py:143,177-178: pw1 = nn.Linear(3, 64) then the stride-2 oriented
 * convolution) in one pass: the 64-channel full-resolution tensor never goes to memory.
 * x is [N,H,W,Cin] with Cin in {1,2,3,4}; pw_w [C,Cin] and pw_b [C] (may be null) are fp32; C must
 * be a multiple of 4; the other arguments are those of dwo_fprop with layout DWO_NHWC.
 */
int dwo_pointwise_fprop_nhwc(const void *x, const float *pw_w, const float *pw_b, const float *w,
                             const float *bias, const void *taps, void *y, int N, int Cin, int C,
                             int H, int W, int K, int stride, int dtype, void *stream);

/*
 * Forward-only glue of a ConvNeXt-1D block, each one pass over HBM in place of the PyTorch
 * passes the reference spends around the operator (no counterpart in the reference's
 * extension; they replace models/convnext.py:306-318 -- permute + LayerNorm before the
 * pointwise layers, layer scale + permute + residual after them -- and the channels-last
 * LayerNorm + GELU of the stem, :176-190).  LayerNorm is over the channel dimension, biased
 * variance, fp32 statistics; gamma, beta and scale are fp32 [C]; C must be even.
 *
 * dwo_layernorm_nhwc:      out[r,:] = act(LN(x[r,:]) * gamma + beta) for rows of C contiguous
 *                          channels (act = exact GELU when gelu != 0), C <= 2048.
 * dwo_nchw_layernorm_nhwc: x [N,C,H,W] -> out [N,H,W,C] = LN over C * gamma + beta, C <= 1536.
 * dwo_nhwc_scale_add_nchw: y [N,H,W,C] -> out [N,C,H,W] = res + scale[c] * y; scale and res
 *                          (an [N,C,H,W] tensor) may be null.
 */
int dwo_layernorm_nhwc(const void *x, const float *gamma, const float *beta, void *out,
                       size_t rows, int C, float eps, int gelu, int dtype, void *stream);
int dwo_nchw_layernorm_nhwc(const void *x, const float *gamma, const float *beta, void *out, int N,
                            int C, int H, int W, float eps, int dtype, void *stream);
int dwo_nhwc_scale_add_nchw(const void *y, const float *scale, const void *res, void *out, int N,
                            int C, int H, int W, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DWOCONV1D_HIP_H */
