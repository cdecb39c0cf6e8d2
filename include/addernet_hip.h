/*
 * addernet_hip.h -- C ABI of libaddernet_hip.so (AdderNet convolution for gfx950).
 *
 * Plain pointers and sizes only: every pointer is a DEVICE pointer to a dense,
 * row-major fp32 array, `stream` is a hipStream_t passed as void* (NULL = the
 * default stream).  Every function returns 0 on success or a negative
 * adder_status; nothing aborts, nothing allocates, nothing synchronises.  All
 * launches are asynchronous on `stream` and safe to record into a HIP graph
 * (no memset nodes: scratch is cleared by kernels).
 *
 * The entry points replace the reference's native boundary, i.e. the four
 * pybind functions of adder_cuda/adder_cuda.cpp:88-93 and the host launchers
 * behind them (adder_cuda/adder.cu:274-465), plus the PyTorch glue the
 * reference runs around them (adder.py:22-41 im2col/col2im, adder.py:78 scaling).
 *
 * Groups, in the order they appear below.  [core] is the reference's boundary and what a port needs;
 * every [optional] group has a [core] equivalent that gives the same results in more launches, and
 * answers ADDER_ERR_UNSUPPORTED (nothing launched) where it does not apply.
 *   [core]      status / version / adder_out_dim
 *   [core]      fused NCHW path: adder_conv2d_fwd_f32, adder_conv2d_bwd_f32, adder_conv2d_bwd_workspace_bytes
 *   [optional]  ... its variants: _fwd_stats_ (BatchNorm statistics in the epilogue), _fwd_pair_stats_ (a strided
 *               1x1 layer beside a strided 3x3), adder_plain_conv2d_fwd_f32 (an ordinary convolution through the same
 *               kernel), _bwd_add_ (a second gradient added), _bf16 (bfloat16 storage), _bwd_noalloc_ (no workspace)
 *   [core]      column-matrix path: adder_col_fwd_f32 / _bwd_f32 / _gradw_f32 / _gradx_f32 (= ADDER_CONV,
 *               ADDER_BACKWARD, ADDER_CONV_WEIGHT, ADDER_CONV_INPUT), adder_col_bwd_workspace_bytes
 *   [core]      adder_grad_norm_scale_f32 (adder.py:78 on its own);  [optional] the batched form
 *   [optional]  grad_W in two stages (all layers finished together after the backward pass)
 *   [optional]  BatchNorm + residual + ReLU kernels (adder_bn_act_*)
 *   [optional]  BatchNorm backward passes folded into the adder backward kernels (adder_bn_links, *_bn_*)
 *   [optional]  the classifier head of the ResNets: average pool, matrix product, BatchNorm (adder_head_*)
 *   [optional]  the cross-entropy loss in one launch each way (adder_cross_entropy_*)
 *   [optional]  the momentum-SGD update of all parameters in one launch (adder_sgd_momentum_step_f32)
 */
#ifndef ADDERNET_HIP_H
#define ADDERNET_HIP_H

#include <stddef.h>

#if defined(__GNUC__)
#define ADDER_API __attribute__((visibility("default")))
#else
#define ADDER_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

typedef enum adder_status {
    ADDER_OK = 0,
    ADDER_ERR_NULL_POINTER = -1,   /* a required pointer is NULL                         */
    ADDER_ERR_BAD_SHAPE = -2,      /* non-positive or inconsistent dimension             */
    ADDER_ERR_TOO_LARGE = -3,      /* a tensor exceeds 2^31-1 elements                   */
    ADDER_ERR_WORKSPACE = -4,      /* workspace missing, misaligned or too small         */
    ADDER_ERR_HIP = -5,            /* a HIP call failed; see adder_last_hip_error()      */
    ADDER_ERR_ALIAS = -6,          /* an output overlaps an input                        */
    ADDER_ERR_UNSUPPORTED = -7     /* optional variant not available for these arguments */
} adder_status;

/* Text for a status code (static storage). */
ADDER_API const char *adder_strerror(int status);
/* hipGetErrorString of the last HIP failure seen by the calling thread ("" if none). */
ADDER_API const char *adder_last_hip_error(void);
/* ABI version: bumped on any signature change. */
ADDER_API int adder_abi_version(void);

/* Output extent floor((h - k + 2p)/s) + 1; replaces adder.py:26-31. Returns <=0 if invalid. */
ADDER_API int adder_out_dim(int h, int k, int pad, int stride);

/* ------------------------------------------------------------------------
 * [core] Fused NCHW path (what adder2d itself uses); the variants between here and the column-matrix path
 * are [optional].
 *   x  (N, Ci, H, W)        w  (Co, Ci, kh, kw)        y, gy (N, Co, Ho, Wo)
 * Zero padding; padded taps count as x = 0 (they add -|w| to y and -w*gy to
 * grad_w) exactly as F.unfold makes them do in adder.py:32.
 * ---------------------------------------------------------------------- */

/* y = -sum_{ci,i,j} |w - x_patch|.  Replaces adder2d_function + adder.forward
 * (adder.py:22-41, 44-60) and ADDER_CONV (adder_cuda.cpp:37-46, adder.cu:19-70,
 * 274-320) including the unfold / permute copies around it.  y is overwritten. */
ADDER_API int adder_conv2d_fwd_f32(const float *x, const float *w, float *y,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, void *stream);

/* The same forward with the statistics of the BatchNorm that follows it (resnet20.py:28-39: every adder
 * layer feeds a BatchNorm2d) collected on the way out: stats[(co * slots + s) * 2 + {0, 1}] receive partial
 * sums of y and y*y over disjoint sets of positions, in fp64; adder_bn_act_fwd_stats_f32 consumes them and
 * skips its own pass over y.  adder_conv2d_fwd_stats_slots gives `slots` for the dimensions, 0 when the
 * kernel that serves them has no such epilogue (then, and for x or y not 16-byte aligned, the _stats call
 * returns ADDER_ERR_UNSUPPORTED and the caller uses the two plain calls). */
ADDER_API int adder_conv2d_fwd_stats_slots(int N, int Ci, int H, int W, int Co, int kh, int kw,
                                           int stride, int pad, int *slots);
ADDER_API int adder_conv2d_fwd_stats_f32(const float *x, const float *w, float *y, double *stats, int stats_slots,
                                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                                         int stride, int pad, void *stream);

/* A strided 3x3 / pad 1 layer and the strided 1x1 / pad 0 layer that reads the same x beside it -- the first layer and
 * the downsample layer of a residual block that halves the map (resnet20.py:66-70, resnet50.py:84-98 build them as two
 * adder2d modules; adder_cuda.cpp:88-93 would run ADDER_CONV twice on two unfolded copies of x) -- in one launch:
 * the 1x1 layer's only tap is the centre tap of the 3x3 window, which the kernel holds in registers anyway.
 * dims describe the 3x3 layer; w_side is (Co, Ci, 1, 1); y_side and stats_side are shaped like y and stats
 * (adder_conv2d_fwd_stats_slots slots).  Rows of whole float4 groups and even H, W, 16-byte aligned tensors;
 * ADDER_ERR_UNSUPPORTED otherwise (optional: the two separate calls give the same results). */
ADDER_API int adder_conv2d_fwd_pair_stats_f32(const float *x, const float *w, const float *w_side, float *y,
                         float *y_side, double *stats, double *stats_side, int stats_slots,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, void *stream);

/* An ordinary convolution y = sum w * x (no bias) through the tiled kernel of the adder forward, for the
 * regular stem layer in front of the adder layers (resnet20.py:49 uses nn.Conv2d there): 3x3 / stride 1 /
 * pad 1 only, ADDER_ERR_UNSUPPORTED (nothing launched) elsewhere.  stats (nullable) / stats_slots as in
 * adder_conv2d_fwd_stats_f32, with the slot count of adder_conv2d_fwd_stats_slots for the same dimensions.
 * Its weight gradient: adder_conv2d_grad_w_staged_f32 with w = NULL. */
ADDER_API int adder_plain_conv2d_fwd_f32(const float *x, const float *w, float *y, double *stats, int stats_slots,
                                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                                         int stride, int pad, void *stream);

/* Bytes of scratch adder_conv2d_bwd_f32 needs for these dimensions. */
ADDER_API int adder_conv2d_bwd_workspace_bytes(int N, int Ci, int H, int W, int Co, int kh, int kw,
                                     int stride, int pad, size_t *bytes);

/* Backward of the layer.  Replaces adder.backward (adder.py:62-80), ADDER_BACKWARD
 * (adder_cuda.cpp:74-86, adder.cu:194-272, 404-465), the fold that autograd runs
 * after it and the Python-side scaling of adder.py:78.
 *   gx (N, Ci, H, W)   = fold( sum_co hardtanh(w - x) * gy )        overwritten; may be NULL
 *   gw (Co, Ci, kh, kw) = sum_{n,l} (x - w) * gy                    overwritten; may be NULL
 *   eta > 0: gw <- gw / max(||gw||_2, 1e-12) * sqrt(Co*Ci*kh*kw) * eta   (reference: eta = 0.2)
 *   eta == 0: gw is left raw.
 * ws / ws_bytes: scratch of at least adder_conv2d_bwd_workspace_bytes, 256-byte aligned. */
ADDER_API int adder_conv2d_bwd_f32(const float *gy, const float *x, const float *w,
                         float *gx, float *gw, float eta,
                         void *ws, size_t ws_bytes,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, void *stream);

/* adder_conv2d_bwd_f32 with gx = grad_X + gx_add.  Where the layer's input also feeds a residual
 * shortcut (resnet20.py:28-39, out += residual) autograd adds the shortcut's gradient to grad_X in a
 * launch of its own; here the kernel adds it on the way out.  gx_add (N, Ci, H, W) and gx must both be
 * given and must not overlap.  ADDER_ERR_UNSUPPORTED (nothing launched) where the layer's grad_X kernel
 * has no such epilogue: only the tiled 3x3 / pad 1 kernels (stride 1 or 2) do. */
ADDER_API int adder_conv2d_bwd_add_f32(const float *gy, const float *x, const float *w, const float *gx_add,
                         float *gx, float *gw, float eta,
                         void *ws, size_t ws_bytes,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, void *stream);

/* Optional reduced-storage mode: the activations and their gradients (x, y, gy, gx) are stored as bfloat16 (the
 * upper half of an fp32, rounded to nearest even on the way out) and take half the HBM traffic and half the
 * activation memory; weights and weight gradients stay fp32, every sum is accumulated as in the fp32 entry points
 * (fp32 for y and gx, fp64 for gw).  The reference computes in fp32 only (adder.cu:310-318 hard-codes
 * data<float>()), so these have no counterpart there and are never the default.  Same dimensions, semantics, eta
 * and workspace (adder_conv2d_bwd_workspace_bytes) as adder_conv2d_fwd_f32 / adder_conv2d_bwd_f32.  3x3 / pad 1
 * layers (stride 1 or 2) run on the tiled kernels, everything else on the generic ones. */
typedef unsigned short adder_bf16;
ADDER_API int adder_conv2d_fwd_bf16(const adder_bf16 *x, const float *w, adder_bf16 *y,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, void *stream);
ADDER_API int adder_conv2d_bwd_bf16(const adder_bf16 *gy, const adder_bf16 *x, const float *w,
                         adder_bf16 *gx, float *gw, float eta,
                         void *ws, size_t ws_bytes,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, void *stream);

/* adder_conv2d_bwd_f32 for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc) and have no workspace to hand over.  It has no counterpart in
 * the reference, whose backward takes every buffer from torch's allocator (adder.py:66-67).  The partial slabs
 * and norm partials live in a buffer of ADDER_NOALLOC_SCRATCH_BYTES that is part of the library's device image
 * (every GPU the library runs on holds one copy until the process ends); the call allocates and frees nothing.
 * Same arguments and results as adder_conv2d_bwd_f32 without ws / ws_bytes.  Layers whose
 * adder_conv2d_bwd_workspace_bytes exceeds ADDER_NOALLOC_SCRATCH_BYTES are refused with ADDER_ERR_WORKSPACE
 * before anything is launched (every ResNet-20 layer at batch 256 fits).  All calls on one GPU share that
 * GPU's buffer: calls that overlap in time on one GPU (different streams, or threads) race; serialise them.
 * The first call on a device looks the buffer's address up (hipGetSymbolAddress); make that call outside
 * stream capture. */
#define ADDER_NOALLOC_SCRATCH_BYTES (8u << 20)
ADDER_API int adder_conv2d_bwd_noalloc_f32(const float *gy, const float *x, const float *w,
                         float *gx, float *gw, float eta,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, void *stream);

/* ------------------------------------------------------------------------
 * [core] Column-matrix path: the literal signatures of the reference extension.
 *   Xcol (K, NL)   Wcol (Co, K)   out, gy (Co, NL)   gW (Co, K)   gX (K, NL)
 * The reference ACCUMULATES into gW / gX (atomicAdd into caller-zeroed
 * buffers, adder.cu:125,186,266-267; adder.py:66-67); so do these.
 * ---------------------------------------------------------------------- */

/* ADDER_CONV (adder_cuda.cpp:37-46; adder.cu:19-70, 274-320). out is overwritten. */
ADDER_API int adder_col_fwd_f32(const float *Xcol, const float *Wcol, float *out,
                      int K, long NL, int Co, void *stream);

/* Scratch for the three column-matrix backward entry points. */
ADDER_API int adder_col_bwd_workspace_bytes(int K, long NL, int Co, size_t *bytes);

/* ADDER_BACKWARD (adder_cuda.cpp:74-86; adder.cu:194-272, 404-465): gW += ..., gX += ... */
ADDER_API int adder_col_bwd_f32(const float *gy, const float *Xcol, const float *Wcol,
                      float *gW, float *gX, int K, long NL, int Co,
                      void *ws, size_t ws_bytes, void *stream);

/* ADDER_CONV_WEIGHT (adder_cuda.cpp:48-59; adder.cu:72-131, 322-355): gW += sum_nl (X - W) * gy */
ADDER_API int adder_col_gradw_f32(const float *gy, const float *Xcol, const float *Wcol,
                        float *gW, int K, long NL, int Co,
                        void *ws, size_t ws_bytes, void *stream);

/* ADDER_CONV_INPUT (adder_cuda.cpp:61-72; adder.cu:133-192, 357-402): gX += sum_co hardtanh(W - X) * gy.
 * Follows the arithmetic the reference states in adder_cuda/test_cuda.py:57-60, not the
 * un-parenthesised macro expansion at adder.cu:170. */
ADDER_API int adder_col_gradx_f32(const float *gy, const float *Xcol, const float *Wcol,
                        float *gX, int K, long NL, int Co, void *stream);

/* ------------------------------------------------------------------------
 * [core] Adaptive learning-rate scaling, in place (adder.py:78):
 *   g <- g / max(||g||_2, eps) * sqrt(n) * eta
 * ws must hold adder_norm_scale_workspace_bytes(n) bytes.
 * ---------------------------------------------------------------------- */
ADDER_API int adder_norm_scale_workspace_bytes(long n, size_t *bytes);
ADDER_API int adder_grad_norm_scale_f32(float *g, long n, float eta, float eps,
                              void *ws, size_t ws_bytes, void *stream);

/* The same scaling (adder.py:78) for `count` <= ADDER_NORM_BATCH_MAX tensors in two launches in all, for
 * callers that take the raw gradients of all their adder layers (adder_conv2d_bwd_f32 with eta = 0) and
 * scale them together after the backward pass.  g, n, eta are host arrays of `count` entries (device
 * pointers, element counts, eta > 0 per tensor); each tensor is scaled by its own norm.
 * ws must hold adder_norm_scale_batched_workspace_bytes(count) bytes. */
#define ADDER_NORM_BATCH_MAX 64
ADDER_API int adder_norm_scale_batched_workspace_bytes(int count, size_t *bytes);
ADDER_API int adder_grad_norm_scale_batched_f32(int count, float *const *g, const long *n, const float *eta,
                              float eps, void *ws, size_t ws_bytes, void *stream);

/* ------------------------------------------------------------------------
 * [optional] grad_W in two stages, for callers that finish the weight gradients of all their layers together after
 * the backward pass (two launches in all instead of two per layer; adder.py:62-80 has no counterpart, it
 * finishes every layer on the spot).
 *   adder_conv2d_grad_w_staged_f32: the position reduction of grad_W into partial slabs inside ws (same size
 *     as for adder_conv2d_bwd_f32), described by *stage; gw and eta are only recorded there.  ws and w must
 *     stay untouched until the stage is finished.  ADDER_ERR_UNSUPPORTED (nothing launched) for layers whose
 *     grad_W kernel has no partial slabs (kernel sizes other than 1x1 and 3x3 / pad 1).
 *     w == NULL: the stage finishes to the plain sum of x * gy, which is the weight gradient of an ordinary
 *     convolution of the same geometry (the stem of resnet20.py:49 runs through the same kernel that way).
 *   adder_grad_w_finish_f32: for each of `count` <= ADDER_GRAD_W_FINISH_MAX stages (a host array)
 *     gw = sum of the slabs - w * sum gy, then the scaling of adder.py:78 where eta > 0.  stage.gw may be
 *     redirected by the caller before this call.
 * ---------------------------------------------------------------------- */
typedef struct adder_grad_w_stage {
    const void *part;      /* partial slabs of sum x * gy   (inside the layer's workspace) */
    const void *sgpart;    /* partial sums of gy per output channel */
    const float *w;        /* the layer's weights (Co, K), or NULL (see above) */
    float *gw;             /* where the finished gradient goes (Co, K) */
    int slots, Co, K;      /* slabs, output channels, Ci * kh * kw */
    int fp64;              /* slabs are double (matrix-core kernels) or float */
    float eta;             /* 0: leave gw raw */
} adder_grad_w_stage;
#define ADDER_GRAD_W_FINISH_MAX 32
ADDER_API int adder_conv2d_grad_w_staged_f32(const float *gy, const float *x, const float *w, float *gw, float eta,
                         void *ws, size_t ws_bytes,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, adder_grad_w_stage *stage, void *stream);
ADDER_API int adder_grad_w_finish_workspace_bytes(int count, const adder_grad_w_stage *stages, size_t *bytes);
ADDER_API int adder_grad_w_finish_f32(int count, const adder_grad_w_stage *stages, void *ws, size_t ws_bytes,
                         void *stream);

/* ------------------------------------------------------------------------
 * [optional] The element-wise neighbours of every adder layer: training-mode BatchNorm2d fused with the
 * residual add and ReLU that follow it.  The reference runs these as separate PyTorch ops
 * (resnet20.py:28-39: bn -> relu, bn -> += residual -> relu); here each direction is one
 * statistics pass and one apply pass.  x, y, residual, dy, dx, dresidual are (N, C, H*W).
 *   forward : y = act(gamma * (x - mean) * rstd + beta [+ residual]),  act = ReLU if relu != 0
 *             save_mean / save_rstd (C) are written for the backward; running_mean / running_var
 *             (nullable, both or neither) are updated with `momentum` (unbiased variance);
 *             num_batches_tracked (nullable, one int64 on the device) is incremented by one.
 *   backward: dx, dgamma, dbeta; dresidual (nullable) receives the gradient of the residual input.
 *             y (the forward output) is needed only when relu != 0, and only for its sign:
 *   relu_mask (nullable, relu != 0 only): adder_bn_act_mask_words(N, C, HW) 32-bit words, one bit per
 *             element of y (bit i % 32 of word i / 32 = [y_i > 0]), written by the forward and read by the
 *             backward in place of y -- a quarter less HBM traffic in the backward.  Shapes whose planes
 *             are not whole words (H*W % 32 != 0) report 0 words and take ADDER_ERR_UNSUPPORTED for a
 *             non-null mask, as do tensors that are not 16-byte aligned.
 * ---------------------------------------------------------------------- */
ADDER_API int adder_bn_act_workspace_bytes(int N, int C, int HW, size_t *bytes);
ADDER_API int adder_bn_act_mask_words(int N, int C, int HW, size_t *words);
ADDER_API int adder_bn_act_fwd_f32(const float *x, const float *residual, const float *gamma, const float *beta,
                                   float *y, unsigned int *relu_mask, float *save_mean, float *save_rstd,
                                   float *running_mean, float *running_var, long long *num_batches_tracked,
                                   float momentum, float eps, int relu,
                                   int N, int C, int HW, void *ws, size_t ws_bytes, void *stream);
/* adder_bn_act_fwd_f32 with the statistics pass already done by the producer of x
 * (adder_conv2d_fwd_stats_f32): `stats` holds C x stats_slots pairs of partial sums; no workspace. */
ADDER_API int adder_bn_act_fwd_stats_f32(const float *x, const float *residual, const float *gamma, const float *beta,
                                         float *y, unsigned int *relu_mask, float *save_mean, float *save_rstd,
                                         float *running_mean, float *running_var, long long *num_batches_tracked,
                                         float momentum, float eps, int relu,
                                         int N, int C, int HW, const double *stats, int stats_slots, void *stream);
ADDER_API int adder_bn_act_bwd_f32(const float *dy, const float *y, const unsigned int *relu_mask,
                                   const float *x, const float *gamma,
                                   const float *save_mean, const float *save_rstd,
                                   float *dx, float *dresidual, float *dgamma, float *dbeta, int relu,
                                   int N, int C, int HW, void *ws, size_t ws_bytes, void *stream);

/* ------------------------------------------------------------------------
 * [optional] The BatchNorm backward passes folded into the adder layers' backward kernels.  No counterpart in the
 * reference, where bn -> relu and the adder layer are separate autograd nodes (resnet20.py:28-39) and the
 * BatchNorm backward is two passes of its own over every activation gradient.  In a chain
 *     ... -> adder A -> BatchNorm P -> (+ residual) -> ReLU -> adder B -> BatchNorm Q -> ...
 * the backward of B already holds what P's backward needs.  Its grad_X kernel has x = relu(...) and its own
 * result in registers, so it can write dz = (grad_X [+ gx_add]) * [x > 0], the gradient of P's output before
 * the ReLU (which is also the gradient of the residual), and P's per-channel sums of dz and dz * xhat (the
 * first pass of P's backward).  And A's grad_W kernel can form its gy = dP_input from (dz, A's output y, four
 * numbers per channel) while it stages gy into LDS (the second pass):
 *     gy = k * dz + c2 * (y - mean) - km1,   k = gamma * rstd, c2 = -k * rstd * mean(dz * xhat), km1 = k * mean(dz),
 * and leave the result in memory for A's grad_X kernel, which runs after it.  P's backward is then no pass over
 * the activation gradient at all: the four numbers come from the sums either in a tiny launch of their own
 * (adder_bn_bwd_coef_f32) or at the start of A's grad_W kernel (out_part: 1-3 us instead of a 4.6 us launch).
 *
 *   adder_bn_links: what a layer's backward is told about its two neighbours; either half may be absent (NULL).
 *     out_x, out_coef | out_part.., out_gy   the BatchNorm BEHIND the layer: out_x = the layer's output y
 *                      (N, Co, Ho, Wo); the `gy` argument is then dz, not the gradient of y; out_gy (N, Co, Ho, Wo)
 *                      receives the gradient of y from the grad_W kernel.  The coefficients: exactly one of
 *                      out_coef = 4 floats per output channel {k, c2, mean, km1} from adder_bn_bwd_coef_f32, or
 *                      out_part = the sums as the consumer's call left them in its in_part (Co, out_slots, 2)
 *                      floats, 16-byte aligned, with out_gamma / out_mean / out_rstd (Co): every workgroup of the grad_W
 *                      kernel then adds the slots of its channels itself, in fp64 and in a fixed order (all of
 *                      them arrive at the same values), and out_dgamma / out_dbeta (Co) are written by that kernel
 *                      -- one launch fewer per layer.
 *     in_x, in_mean, in_rstd, in_part, in_slots, in_relu   the BatchNorm IN FRONT of the layer, whose output
 *                      (after the residual add and, if in_relu, the ReLU) is the layer's x: in_x = that
 *                      BatchNorm's input (N, Ci, H, W), its saved mean / rstd (Ci); in_part receives
 *                      (Ci, in_slots, 2) floats (per-wave fp32 totals), in_slots = adder_conv2d_bwd_bn_slots; gx
 *                      receives dz.
 *   adder_conv2d_bwd_bn_slots: partial-sum slots per channel for in_part; 0 = this layer has no such kernels
 *     (they exist for 3x3 / pad 1 / stride 1 or 2 layers whose rows are whole groups of four floats, and for 1x1 /
 *     stride 1 layers with at least 64 input and output channels whose planes are whole groups of four floats).
 *   adder_conv2d_bwd_bn_f32: adder_conv2d_bwd_add_f32 (gx_add nullable here) with the links.  With the out_*
 *     half gw must be requested (the grad_W kernel is the one that forms gy); a caller that stages grad_W
 *     (adder_conv2d_grad_w_staged_bn_f32) calls this afterwards with gy = its out_gy and without the out_* half.
 *     ADDER_ERR_UNSUPPORTED, nothing launched, where adder_conv2d_bwd_bn_slots is 0 or a tensor is not
 *     16-byte aligned.
 *   adder_conv2d_grad_w_staged_bn_f32: adder_conv2d_grad_w_staged_f32 with the out_* half of the links
 *     (out_gy nullable).
 *   adder_bn_bwd_coef_f32: sums the slots of `part` (C, slots, 2) floats in fp64, in a fixed order, and writes coef (C, 4),
 *     dgamma and dbeta (C); count = N * H * W of the BatchNorm.
 * ---------------------------------------------------------------------- */
typedef struct adder_bn_links {
    const float *out_x;
    const float *out_coef;
    float *out_gy;
    const float *in_x;
    const float *in_mean;
    const float *in_rstd;
    float *in_part;
    int in_slots;
    int in_relu;
    /* optional, both or neither, and only for a BatchNorm whose output reached the layer through nothing but the
       ReLU (no residual added): its weight and bias (Ci).  The stride-1 kernels then take xhat = (x - beta) / gamma
       from the x they hold instead of reading in_x (which must still be given: channels with
       |gamma| < max(1, |beta|) / 64 and the stride-2 kernels read it). */
    const float *in_gamma;
    const float *in_beta;
    /* optional, both or neither, with the in_* half, for a 3x3 / stride 2 / pad 1 layer on a map of even height and
       width: the strided 1x1 / pad 0 layer that reads the same x beside this one (resnet20.py:66-70).  side_gy is
       that layer's output gradient (N, Co, Ho, Wo), side_w its weights (Co, Ci): its input gradient is added to
       grad_X inside the kernel (before the mask and the sums), as if it had been passed as gx_add. */
    const float *side_gy;
    const float *side_w;
    /* the alternative to out_coef (see above); all of them or none */
    const float *out_part;
    int out_slots;
    const float *out_gamma;
    const float *out_mean;
    const float *out_rstd;
    float *out_dgamma;
    float *out_dbeta;
} adder_bn_links;
ADDER_API int adder_conv2d_bwd_bn_slots(int N, int Ci, int H, int W, int Co, int kh, int kw, int stride, int pad,
                                        int *slots);
ADDER_API int adder_conv2d_bwd_bn_f32(const float *gy, const float *x, const float *w, const float *gx_add,
                         float *gx, float *gw, float eta,
                         void *ws, size_t ws_bytes,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, const adder_bn_links *links, void *stream);
ADDER_API int adder_conv2d_grad_w_staged_bn_f32(const float *gy, const float *x, const float *w, float *gw, float eta,
                         void *ws, size_t ws_bytes,
                         int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, const adder_bn_links *links, adder_grad_w_stage *stage, void *stream);
ADDER_API int adder_bn_bwd_coef_f32(const float *part, int slots, const float *gamma, const float *save_mean,
                                    const float *save_rstd, double count, float *coef, float *dgamma, float *dbeta,
                                    int C, void *stream);

/* ------------------------------------------------------------------------
 * [optional] The classifier head behind the last adder block (resnet20.py:55-57, 89-93 of the reference:
 * AvgPool2d over the whole map, a 1x1 convolution without bias, BatchNorm2d in training mode), two launches
 * forward and two backward where the framework's own operators take eight of 5-10 us each on N x classes values.
 *   x (N, C, HW) -> pooled (N, C) = plane means -> z (N, classes) = pooled * w^T, w (classes, C)
 *     -> y (N, classes) = gamma * (z - mean) * rstd + beta, batch statistics per class (biased variance; the running
 *     statistics, nullable, receive the unbiased one, as torch.nn.BatchNorm2d does).
 *   adder_head_supported: 1 where the kernels apply -- N >= 2, a plane of 4, 8, ... 256 positions, C a divisor of
 *     256 with N * C a multiple of four, at most 32 classes, and a batch whose pooled matrix fits the LDS (with
 *     P = 16 or 32 padded classes: N * (C + P) + max(3 * classes * (N | 1), 512 * P) floats within 144 KiB) -- else
 *     0, and the calls return ADDER_ERR_UNSUPPORTED.  x, dx and pooled 16-byte aligned.
 *   adder_head_fwd_f32: pooled, z, save_mean, save_rstd are kept for the backward.
 *   adder_head_bwd_f32: dy (N, classes) -> dgamma, dbeta, dz (N, classes: the gradient of z, scratch for the caller),
 *     dw (classes, C) = dz^T * pooled, dx (N, C, HW; nullable) = (dz * w) / HW on every position.
 * Every sum has a fixed order: results do not change from run to run.
 * ---------------------------------------------------------------------- */
ADDER_API int adder_head_supported(int N, int C, int HW, int classes);
ADDER_API int adder_head_fwd_f32(const float *x, const float *w, const float *gamma, const float *beta,
                                 float *pooled, float *z, float *y, float *save_mean, float *save_rstd,
                                 float *running_mean, float *running_var, long long *num_batches_tracked,
                                 float momentum, float eps, int N, int C, int HW, int classes, void *stream);
ADDER_API int adder_head_bwd_f32(const float *dy, const float *z, const float *pooled, const float *w,
                                 const float *gamma, const float *save_mean, const float *save_rstd,
                                 float *dz, float *dx, float *dw, float *dgamma, float *dbeta,
                                 int N, int C, int HW, int classes, void *stream);

/* ------------------------------------------------------------------------
 * [optional] The loss of the training script (main.py:66,90 of the reference: torch.nn.CrossEntropyLoss with its
 * defaults -- class indices as targets, mean over the batch) in one launch each way, for at most 32 classes
 * (ADDER_ERR_UNSUPPORTED above that).  target: N int64 class indices in [0, classes).
 *   adder_cross_entropy_fwd_f32: loss[0] = mean_n (lse[n] - logits[n, target[n]]), lse[n] = log sum_j exp(logits[n, j]),
 *     kept for the backward.  adder_cross_entropy_bwd_f32: grad_logits[n, j] =
 *     (exp(logits[n, j] - lse[n]) - [j == target[n]]) * grad_loss[0] / N, grad_loss one float in device memory.
 * ---------------------------------------------------------------------- */
ADDER_API int adder_cross_entropy_fwd_f32(const float *logits, const long long *target, float *loss, float *lse,
                                          int N, int classes, void *stream);
ADDER_API int adder_cross_entropy_bwd_f32(const float *logits, const long long *target, const float *lse,
                                          const float *grad_loss, float *grad_logits, int N, int classes,
                                          void *stream);

/* ------------------------------------------------------------------------
 * [optional] The parameter update of the training script (main.py:67 of the reference: torch.optim.SGD with
 * momentum and weight decay, no dampening, no Nesterov) for `count` <= ADDER_SGD_BATCH_MAX tensors in one launch:
 *     g' = grads[t] + weight_decay * params[t];  momentum_bufs[t] = momentum * momentum_bufs[t] + g';
 *     params[t] -= lr * momentum_bufs[t]
 * (a zero-filled buffer gives the framework's first step, buf = g').  params, grads, momentum_bufs and n are host
 * arrays of `count` device pointers / element counts.  lr_device (nullable): the learning rate as one float in
 * device memory, read by the kernel -- for callers that capture the step in a HIP graph and change the rate
 * between replays; `lr` is used when it is NULL.
 * ---------------------------------------------------------------------- */
#define ADDER_SGD_BATCH_MAX 96
ADDER_API int adder_sgd_momentum_step_f32(int count, float *const *params, const float *const *grads,
                                          float *const *momentum_bufs, const long *n, const float *lr_device,
                                          float lr, float momentum, float weight_decay, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ADDERNET_HIP_H */
