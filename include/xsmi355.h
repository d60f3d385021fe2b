/*
 * xsmi355.h -- C ABI of libxsmi355.so: the MI355X (gfx950) conv / max-pool
 * backend behind xshinnosuke's functional API.
 *
 * Conventions
 *   - Every function returns 0 on success and a non-zero code on failure; the
 *     message for the calling thread's last failure is xsmi_last_error().
 *     No C++ exception crosses this boundary.
 *   - Tensors are dense NCHW float32 in device memory.  Device pointers are the
 *     opaque values returned by xsmi_malloc.
 *   - Ops never allocate: scratch memory (packed filters, split-reduction
 *     partials) is a caller-provided workspace sized by the matching
 *     *_workspace_bytes query.  The workspace contents are dead after the call
 *     has completed on the stream.
 *   - All work is enqueued in order on one library-owned stream (xsmi_conv2d_bwd
 *     forks part of its work to a second one and joins it again before the
 *     call's successors); results are visible to the host after xsmi_sync() or
 *     a (blocking) xsmi_memcpy_d2h.  Calls are not re-entrant across threads.
 *   - Window geometry follows the reference: symmetric integer zero padding
 *     `pad`, stride (sh, sw), OH = (H + 2*pad - R)/sh + 1 (floor), no dilation,
 *     no groups.
 *
 * The reference is pure Python and has no FFI of its own; each entry point
 * below names the reference function whose arithmetic it replaces.
 */
#ifndef XSMI355_H
#define XSMI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XSMI_OK 0
#define XSMI_ERR_INVALID 1   /* bad argument (shape, pointer, workspace too small) */
#define XSMI_ERR_RUNTIME 2   /* HIP runtime failure */
#define XSMI_ERR_STATE 3     /* library not initialised */

/* flags for the conv entry points */
#define XSMI_CONV_RELU 0x1u      /* y = max(0, conv + bias)  (fused epilogue)            */
#define XSMI_CONV_BF16 0x2u      /* opt-in: operands rounded to bf16 (nearest even), fp32
                                    accumulate.  The forward (channels a multiple of 32, or at
                                    most 8) first writes a channels-last bf16 copy of x with a
                                    zero border into the workspace and multiplies from it; it
                                    takes this form when the workspace has the size that
                                    xsmi_conv2d_workspace_bytes reports, and a slower one that
                                    gathers from x directly when it only has room for the filter.
                                    The weight gradient ignores the flag.                     */
#define XSMI_CONV_WS_PACKED 0x4u /* the workspace still holds what the previous call of the same
                                    entry point with the same geometry and the same filter values
                                    left there, or what xsmi_conv2d_pack left there for this pass,
                                    geometry and filter values: the filter is not laid out again
                                    (inference loops; training steps that lay all filters out right
                                    after the optimizer step).  Ignored where no reusable layout
                                    exists.  xsmi_conv2d_bwd applies it to the data gradient.  */

#define XSMI_CONV_DW_ASYNC 0x8u  /* xsmi_conv2d_bwd only: the weight gradient stays on the library's
                                    second stream when the call returns; see xsmi_conv2d_bwd_join */

typedef struct xsmi_device_info {
    int device;
    int cu_count;
    int clock_khz;
    int lds_bytes_per_cu;
    int wavefront;
    int l2_bytes;
    uint64_t hbm_bytes;
    char name[128];
    char arch[64];
} xsmi_device_info_t;

/* ---- runtime ------------------------------------------------------------
 * Replaces the reference's array-module switch to CuPy
 * (xs/core/__global.py:9, xs/core/base.py:143-146, 167-170) and the implicit
 * host<->device copies of Tensor.to()/numpy() (xs/core/base.py:136-184, 211-217).
 */
int xsmi_init(int device);
int xsmi_is_initialized(void);
const char *xsmi_last_error(void);
int xsmi_device_info(xsmi_device_info_t *info);
/* Device memory the library itself holds on a GPU once initialised there: the exchange
 * buffers of the even-split fp32 convolution kernels (one per stream of the library) and
 * the static array of xsmi_conv2d_fwd_noalloc.  Everything else is the caller's
 * (tensors, workspaces).  No counterpart in the reference. */
size_t xsmi_scratch_bytes(void);
int xsmi_malloc(void **ptr, size_t bytes);
int xsmi_free(void *ptr);
int xsmi_memcpy_h2d(void *dst, const void *src, size_t bytes);   /* blocking */
int xsmi_memcpy_d2h(void *dst, const void *src, size_t bytes);   /* blocking */
/* Page-locked host memory and an upload from it that only enqueues on the stream: the source must
 * stay untouched until an event recorded after the call has completed.  They carry the batch
 * upload of the reference's DataLoader (xs/utils/data/dataloader.py:30-43, one fixed tensor per
 * loader refilled for every batch) without stalling the host on each copy. */
int xsmi_host_alloc(void **ptr, size_t bytes);
int xsmi_host_free(void *ptr);
int xsmi_memcpy_h2d_async(void *dst, const void *pinned_src, size_t bytes);
int xsmi_memcpy_d2d(void *dst, const void *src, size_t bytes);   /* async on the stream */
int xsmi_memset(void *dst, int byte_value, size_t bytes);        /* async on the stream (a fill kernel) */
int xsmi_sync(void);
/* Tuning switches of the kernel selection, by name: "tap_sk" (0: one tile per workgroup only, 1: even split of
 * the chunks where it pays, 3: even split wherever it applies), "sk_spin_limit" (polls before an even-split
 * workgroup gives up waiting for a partial tile; the calls that wait for the device then fail with
 * XSMI_ERR_RUNTIME), "sk_wide" (the even-split kernel's activation loads: 2: input rows staged once for the three taps of
 * a filter row where that form pays, 16-byte loads tap by tap where only those apply; 3: staged rows wherever they
 * apply; 1: 16-byte loads tap by tap; 0: one-dword loads everywhere), "pool_bwd" (workgroups per compute unit of the 3x3/2 max-pool gradient kernel whose workgroups walk
 * several pieces; 0: one piece per workgroup), "pack_lanes" (1 to 4: streams over which xsmi_conv2d_pack deals its
 * layout launches), "tap_stages", "tap_persist", "cl_halo", "cl_stem".  Each starts from the environment variable XSMI_<NAME IN CAPITALS> when that is set.
 * A caller that changes one must drop every workspace content it counted on (XSMI_CONV_WS_PACKED) and ask for
 * workspace sizes again.  No counterpart in the reference. */
int xsmi_set_option(const char *name, long value);
int xsmi_get_option(const char *name, long *value);
int xsmi_event_create(void **event);
int xsmi_event_record(void *event);                               /* on the library stream */
int xsmi_event_synchronize(void *event);                          /* host waits for the event */
int xsmi_event_elapsed_ms(void *start, void *stop, float *ms);    /* waits for `stop` */
int xsmi_event_destroy(void *event);
/* Per-op device timing: after xsmi_profiling(1) every op records one event
 * before and one after its main kernel (for conv: the MFMA kernel(s), not the
 * filter packing or the split reduction); xsmi_last_kernel_ms waits for the last
 * op and returns the time between the two. */
int xsmi_profiling(int on);
int xsmi_last_kernel_ms(float *ms);
/* plain float4 copy kernel of `bytes` bytes (multiple of 16); used to
 * calibrate HBM counters and to quote the achievable copy bandwidth. */
int xsmi_copy_kernel(void *dst, const void *src, size_t bytes);

/* ---- step graphs ----------------------------------------------------------
 * No counterpart in the reference, whose steps are NumPy calls.  A training or inference step here is a
 * few hundred short launches, and the host needs about as long to issue them as the device needs to run
 * them; a step whose launches do not change from one iteration to the next (same entry points, same
 * pointers, same sizes, same scalars) can be recorded once and re-issued with one call.
 *
 * xsmi_graph_begin() opens the recording: until xsmi_graph_end() every entry point records its launches
 * (both streams, with the fork and join of xsmi_conv2d_bwd) instead of running them, so nothing recorded has
 * happened yet when the recording ends.  Entry points that wait for the device (xsmi_sync, xsmi_memcpy_h2d,
 * xsmi_memcpy_d2h, the event calls, xsmi_last_kernel_ms) fail with XSMI_ERR_STATE while it is open, xsmi_malloc
 * stays legal, xsmi_free takes effect when it closes.  xsmi_graph_end(&graph, keep) closes it and, with
 * keep != 0, hands back an executable graph (keep == 0 discards what was recorded, e.g. after an error).
 * xsmi_graph_launch() enqueues one replay on the library stream, in order with everything else;
 * xsmi_graph_destroy() waits for the stream and releases the graph.  Every buffer the recorded launches
 * touch must stay allocated, and unused by anything that expects its contents to survive a replay, for as
 * long as the graph is replayed. */
int xsmi_graph_begin(void);
int xsmi_graph_end(void **graph, int keep);
int xsmi_graph_launch(void *graph);
int xsmi_graph_destroy(void *graph);

/* ---- convolution ---------------------------------------------------------
 * x (N,C,H,W), w (K,C,R,S), bias (K) or NULL, y (N,K,OH,OW).
 */

/* Workspace needed by the conv entry points for this geometry (the maximum
 * over fwd / bwd_data / bwd_weight / bwd and over flags). */
size_t xsmi_conv2d_workspace_bytes(int N, int C, int H, int W, int K, int R, int S,
                                   int sh, int sw, int pad);

/* The same for one pass alone (0 forward, 1 backward-data, 2 backward-weight) with the
 * given flags (XSMI_CONV_BF16 or 0): the size with which that pass's entry point picks
 * its fastest kernel.  For callers that keep one workspace per filter and pass (a filter
 * layout made ahead, XSMI_CONV_WS_PACKED): a ResNet-18 training step at N=32 then holds
 * tens of megabytes of layouts instead of a full-size workspace per filter and pass.
 * No counterpart in the reference (its conv2d allocates the im2col matrix per call,
 * xs/utils/common.py:35-46).  Returns 0 for a bad geometry or pass. */
size_t xsmi_conv2d_pass_workspace_bytes(int N, int C, int H, int W, int K, int R, int S,
                                        int sh, int sw, int pad, int pass, unsigned flags);

/* Forward: replaces conv2d (xs/nn/functional.py:405-442) incl. im2col
 * (xs/utils/common.py:35-46); with XSMI_CONV_RELU also the ReLU that
 * Conv2D.call applies (xs/layers/convolutional.py:76-77, xs/nn/td_functional.py:59-60).
 * neg_mask (N*K*OH*OW bytes) may be NULL; when given together with
 * XSMI_CONV_RELU it receives 1 where the pre-activation is < 0 and 0 elsewhere
 * (the strict mask of ReLUBackward, xs/nn/grad_fn.py:155-157). */
int xsmi_conv2d_fwd(const float *x, const float *w, const float *bias, float *y,
                    uint8_t *neg_mask,
                    int N, int C, int H, int W, int K, int R, int S,
                    int sh, int sw, int pad, unsigned flags,
                    void *workspace, size_t workspace_bytes);

/* ---- channels-last bf16 activations (inference) ----------------------------
 * An extension of the forward above for chains of layers evaluated without gradients
 * (Model.predict / evaluate, xs/nn/models.py:146-186, under bf16 conv precision): the
 * reference keeps every activation as float32 NCHW; here a tensor may instead live as
 * bf16 [N][H + 2 b][W + 2 b][C] with a zero border of b pixels ("channels-last"),
 * which is the operand layout of the bf16 MFMA kernel, so that conv -> add/ReLU ->
 * max-pool -> conv chains neither rewrite nor convert their activations.
 *
 * xsmi_conv2d_fwd_cl: conv2d (+bias, +ReLU with XSMI_CONV_RELU) with bf16 operands and
 * fp32 accumulation.  Exactly one of x (fp32 NCHW) / x_cl (channels-last, C % 32 == 0,
 * border x_border >= pad) and exactly one of y (fp32 NCHW) / y_cl (channels-last,
 * K % 8 == 0, border y_border; only the interior is written: the caller zeroes the
 * buffer once) is given.  flags: XSMI_CONV_RELU, XSMI_CONV_WS_PACKED.  Workspace:
 * xsmi_conv2d_workspace_bytes of the geometry is always enough. */
int xsmi_conv2d_fwd_cl(const float *x, const void *x_cl, int x_border, const float *w, const float *bias,
                       float *y, void *y_cl, int y_border,
                       int N, int C, int H, int W, int K, int R, int S,
                       int sh, int sw, int pad, unsigned flags,
                       void *workspace, size_t workspace_bytes);
/* out = a + b (relu = 0) or max(0, a + b) over `count` bf16 elements (a multiple of 8) of
 * equally shaped channels-last tensors, borders included: add (xs/nn/functional.py:6-21)
 * followed by relu (xs/nn/functional.py:297-313); out may be a or b. */
int xsmi_cl_add(const void *a, const void *b, void *out, size_t count, int relu);
/* max_pool2d (xs/nn/functional.py:445-491) on channels-last tensors: the input's zero
 * border (x_border >= pad) is the reference's zero-valued padding that takes part in
 * the max; writes the interior of y_cl (border y_border).  No argmax: inference only. */
int xsmi_cl_maxpool2d(const void *x_cl, int x_border, void *y_cl, int y_border,
                      int N, int C, int H, int W, int k, int sh, int sw, int pad);
/* y (fp32, N,C,H,W) = the interior of a channels-last tensor: for every consumer that
 * reads float32 NCHW. */
int xsmi_cl_to_nchw(const void *x_cl, int border, float *y, int N, int C, int H, int W);

/* The forward for callers that cannot allocate device memory or pass a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same kernels,
 * arguments and results as xsmi_conv2d_fwd (flags: XSMI_CONV_RELU, XSMI_CONV_BF16); the scratch memory is a static
 * device array of XSMI_NOALLOC_SCRATCH_BYTES (16 MiB) inside the library, one per GPU, held
 * until the process ends.  Geometries whose workspace (xsmi_conv2d_workspace_bytes of the forward alone: the
 * packed filter) exceeds it are refused with XSMI_ERR_INVALID.  All calls on a GPU share that array: calls that
 * overlap on one GPU (two host threads, two streams) race.  Calls no hipMalloc / hipFree. */
int xsmi_conv2d_fwd_noalloc(const float *x, const float *w, const float *bias, float *y,
                            uint8_t *neg_mask, int N, int C, int H, int W, int K, int R, int S,
                            int sh, int sw, int pad, unsigned flags);
#define XSMI_NOALLOC_SCRATCH_BYTES ((size_t)16 << 20)

/* Backward w.r.t. the input: dx = beta*dx + fold(dy^T . w).  Replaces the dcol
 * GEMM + col2im of Conv2DBackward (xs/nn/grad_fn.py:199-203, xs/utils/common.py:49-65).
 * beta must be 0 (overwrite) or 1 (accumulate, what the reference always does). */
int xsmi_conv2d_bwd_data(const float *dy, const float *w, float *dx,
                         int N, int C, int H, int W, int K, int R, int S,
                         int sh, int sw, int pad, float beta, unsigned flags,
                         void *workspace, size_t workspace_bytes);

/* Backward w.r.t. filter and bias: dw = beta*dw + dy . unfold(x), db = beta*db + sum(dy).
 * Replaces xs/nn/grad_fn.py:191-197.  db may be NULL.  The reduction order is
 * fixed (no float atomics): partial sums per pixel range, then one pass that adds
 * the partials in float64 in ascending range order. */
int xsmi_conv2d_bwd_weight(const float *dy, const float *x, float *dw, float *db,
                           int N, int C, int H, int W, int K, int R, int S,
                           int sh, int sw, int pad, float beta, unsigned flags,
                           void *workspace, size_t workspace_bytes);

/* Both backward passes of one layer in one call: what xsmi_conv2d_bwd_weight and
 * xsmi_conv2d_bwd_data compute, with the same results bit for bit (Conv2DBackward,
 * xs/nn/grad_fn.py:191-203, does the two one after the other).  The two share only
 * their inputs, so the weight gradient can run on a second stream of the library
 * beside the data gradient.  db may be NULL.  flags: XSMI_CONV_BF16, XSMI_CONV_DW_ASYNC,
 * XSMI_CONV_WS_PACKED (the data gradient's workspace holds the filter layout already).
 * workspace serves the data gradient, workspace_dw the weight gradient; each of
 * xsmi_conv2d_workspace_bytes() bytes is enough, and the two must not overlap.
 *
 * Without XSMI_CONV_DW_ASYNC the call is complete in stream order when it returns (the
 * library decides whether the two kernels run side by side or one after the other).
 * With it, dx is complete in stream order, but the weight gradient keeps running on the
 * second stream beside whatever is enqueued next, until xsmi_conv2d_bwd_join() (or
 * xsmi_sync(), xsmi_conv2d_bwd_weight() or a call of this function without the flag,
 * which join first).  Until then the caller must not free, write or hand to another
 * entry point: dw, db, workspace_dw (other than through further calls of this function,
 * which the second stream runs in order), and must not free or write dy and x.  A
 * backward sweep spends about as long in the memory-bound passes between two
 * convolutions as it takes to hide a good part of the weight gradients: ResNet-18 at
 * N=32, 0.4 ms of a 5.5 ms step. */
int xsmi_conv2d_bwd(const float *dy, const float *x, const float *w,
                    float *dx, float *dw, float *db,
                    int N, int C, int H, int W, int K, int R, int S,
                    int sh, int sw, int pad, float beta_dx, float beta_dw, unsigned flags,
                    void *workspace, size_t workspace_bytes,
                    void *workspace_dw, size_t workspace_dw_bytes);
/* The main stream waits for everything on the second stream (weight gradients that xsmi_conv2d_bwd
 * left there, filter layouts of xsmi_conv2d_pack); a no-op when there is nothing. */
int xsmi_conv2d_bwd_join(void);

/* Lay filters out ahead of time.  Every conv call first rewrites w into the layout its kernel reads
 * (a few microseconds of a tiny launch in front of each of the ~40 convolution passes of a ResNet-18
 * step; the reference has no counterpart, its im2col GEMM reads w as it is, xs/nn/functional.py:428).
 * This entry point runs only that step, for every job: pass 0 (xsmi_conv2d_fwd) or 1
 * (xsmi_conv2d_bwd_data / the data gradient of xsmi_conv2d_bwd) of the given fp32 geometry, all on the
 * library's second stream: ordered after everything enqueued so far, beside whatever the main stream is
 * given next.  job.packed is set to 1 when the job's workspace now holds a layout that the later call
 * accepts through XSMI_CONV_WS_PACKED (same geometry, same workspace size, w unchanged in between), and
 * to 0 when this geometry's kernel has nothing to prepare ahead (first layers, the generic kernels);
 * the later call must then not pass the flag.  The main stream has to wait for the second one
 * (xsmi_conv2d_bwd_join) before the first call that uses a prepared workspace. */
typedef struct xsmi_pack_job {
    const float *w;
    void *workspace;
    size_t workspace_bytes;
    int N, C, H, W, K, R, S, sh, sw, pad;
    int pass;
    int packed;                  /* out */
} xsmi_pack_job_t;
int xsmi_conv2d_pack(int count, xsmi_pack_job_t *jobs);

/* ---- max pooling ---------------------------------------------------------
 * x (N,C,H,W) -> y (N,C,OH,OW), square window k, zero-valued padding that takes
 * part in the max, first maximum in row-major (ky,kx) order wins.
 * idx holds ky*k+kx as uint8, stored in NCHW order (the reference keeps the same
 * values as int64 in (n,oh,ow,c) order).
 */

/* Replaces max_pool2d (xs/nn/functional.py:445-491). idx may be NULL. */
int xsmi_maxpool2d_fwd(const float *x, float *y, uint8_t *idx,
                       int N, int C, int H, int W, int k, int sh, int sw, int pad);

/* Replaces Maxpool2DBackward (xs/nn/grad_fn.py:224-235): gather formulation,
 * float64 sum over the covering windows in ascending (ky,kx) order, one rounding:
 * dx = round32(beta*dx + sum). beta is 0 or 1. */
int xsmi_maxpool2d_bwd(const float *dy, const uint8_t *idx, float *dx,
                       int N, int C, int H, int W, int k, int sh, int sw, int pad,
                       float beta);

/* ---- ReLU mask backward ----------------------------------------------------
 * dx = beta*dx + (neg_mask ? 0 : dy) over n elements.  Replaces ReLUBackward
 * (xs/nn/grad_fn.py:146-157) for the fused conv epilogue. dx may alias dy. */
int xsmi_relu_mask_bwd(const float *dy, const uint8_t *neg_mask, float *dx, size_t n, float beta);
/* The same masked gradient into two tensors in one pass: dx1 = beta1*dx1 + g, dx2 = beta2*dx2 + g with
 * g = neg_mask ? 0 : dy.  For a ReLU applied in place to a sum (a residual block's end,
 * xs/nn/grad_fn.py:146-157 followed by AddBackward, xs/nn/grad_fn.py:14-22): both addends receive it.
 * dy, dx1, dx2 16-byte aligned, neg_mask 4-byte aligned; dx1 != dx2. */
int xsmi_relu_mask_bwd2(const float *dy, const uint8_t *neg_mask, float *dx1, float beta1, float *dx2, float beta2, size_t n);

/* ---- neighbours of conv / pool in a network (device-resident tensors) --------
 * Small element-wise, normalisation and reduction kernels so that activations need not
 * leave the GPU between two convolutions.  They replace the NumPy expressions of the
 * reference's xs/nn/td_functional.py and of the named functions; all are float32 and
 * run on the library stream.  `ws` arguments are caller-provided scratch.
 */

/* y[i] += a * x[i]                       (gradient accumulation; SGD: xs/optim/sgd.py:4-9) */
int xsmi_axpy(float *y, const float *x, float a, size_t n);
/* the same for `count` tensors in one or a few launches (one SGD step over all parameters);
 * ys, xs, ns are host arrays of device pointers / element counts */
int xsmi_axpy_multi(int count, float *const *ys, const float *const *xs, const size_t *ns, float a);
/* out[i] = a[i] + b[i]                   (residual add, xs/nn/functional.py:6-21) */
int xsmi_add(const float *a, const float *b, float *out, size_t n);
/* out[i] = max(0, a[i] + b[i]): the residual add followed by the block's in-place ReLU
 * (xs/nn/functional.py:6-21 then xs/layers/activators.py:37-50) in one pass; neg_mask (or NULL)
 * receives 1 where the sum is < 0, the sign the ReLU's backward needs */
int xsmi_add_relu(const float *a, const float *b, float *out, uint8_t *neg_mask, size_t n);
/* out[i] = value */
int xsmi_fill(float *out, float value, size_t n);
/* out[i] = s * a[i] + t */
int xsmi_scale_shift(const float *a, float *out, float s, float t, size_t n);
/* y = max(0, x) (may be in place)        (xs/nn/td_functional.py:59-60) */
int xsmi_relu_fwd(const float *x, float *y, size_t n);
/* y = max(0, x) and neg_mask[i] = x[i] < 0 (for an in-place ReLU whose backward still needs the sign) */
int xsmi_relu_fwd_mask(const float *x, float *y, uint8_t *neg_mask, size_t n);
/* dx[i] = pre[i] < 0 ? 0 : dy[i]         (strict mask, xs/nn/grad_fn.py:146-157); dx may alias dy */
int xsmi_relu_bwd(const float *dy, const float *pre, float *dx, size_t n);
/* y = 1 / (1 + exp(-x)) for kind 1, tanh(x) for kind 2 (may be in place): the other two activations a layer's
 * `activation=` argument names (xs/nn/td_functional.py:63-70, xs/layers/activators.py:62-87) */
int xsmi_act_fwd(const float *x, float *y, size_t n, int kind);
/* dx = dy * y * (1 - y) for kind 1, dy * (1 - y^2) for kind 2, y being the forward's output
 * (xs/nn/grad_fn.py:161-170); dx may alias dy */
int xsmi_act_bwd(const float *dy, const float *y, float *dx, size_t n, int kind);
/* m[i] = momentum * m[i] + (1 - momentum) * cur[i]   (moving statistics, xs/nn/functional.py:700-707) */
int xsmi_lerp(float *m, const float *cur, float momentum, size_t n);

/* Batch normalisation over axis 1 of an (N, C, HW) tensor with batch statistics
 * (xs/nn/functional.py:676-707): y = gamma * xhat + beta, xhat = (x - mean) / sqrt(var + eps),
 * biased variance.  Outputs xhat (N*C*HW, or NULL to skip it), sqrtvar/mean/var (C).  ws: xsmi_bn_workspace_bytes(C). */
size_t xsmi_bn_workspace_bytes(int C);
int xsmi_bn_fwd(const float *x, const float *gamma, const float *beta, float *y, float *xhat, float *sqrtvar,
                float *mean, float *var, float *moving_mean, float *moving_var, float momentum, uint8_t *neg_mask,
                int N, int C, int HW, float eps, void *ws, size_t ws_bytes);
/* moving_mean / moving_var (both or neither): m = momentum*m + (1-momentum)*batch statistic, the update the
 * reference performs after the forward (xs/nn/functional.py:700-707), done by the normalisation kernel.
 * neg_mask (or NULL) fuses the ReLU that follows the normalisation in a residual block
 * (xs/layers/activators.py:37-50): neg_mask[i] = pre-activation < 0, y = max(pre-activation, 0). */
/* The end of a residual block as one pass: y = max(0, gamma * xhat + beta + residual), neg_mask[i] = that sum < 0, with
 * the batch statistics of x as in xsmi_bn_fwd (same outputs, same moving-statistics update, xhat never stored).  It
 * stands for xsmi_bn_fwd, xsmi_add and xsmi_relu_fwd_mask in a row (xs/nn/functional.py:676-707, xs/layers/ops.py:40-72,
 * xs/layers/activators.py:37-50) without writing and reading the normalised tensor in between; the backward is
 * xsmi_relu_mask_bwd on the sum's gradient, which then goes to xsmi_bn_bwd and to the residual branch unchanged. */
int xsmi_bn_add_relu_fwd(const float *x, const float *gamma, const float *beta, const float *residual, float *y,
                         float *sqrtvar, float *mean, float *var, float *moving_mean, float *moving_var, float momentum,
                         uint8_t *neg_mask, int N, int C, int HW, float eps, void *ws, size_t ws_bytes);
/* The head of a ResNet as two passes over the convolution's output instead of four: batch statistics, then
 * normalisation, ReLU and the 3 x 3 / stride 2 / pad 1 max-pool in one kernel.  pooled (N, C, H/2, W/2) and idx are what
 * xsmi_maxpool2d_fwd would give on the output of xsmi_bn_fwd with neg_mask (same comparisons on the same float values,
 * hence the same bits), neg_mask (N*C*H*W) and the statistics are xsmi_bn_fwd's; the normalised tensor is not stored.
 * H even, W a multiple of 4.  Stands for xs/nn/functional.py:676-707, xs/layers/activators.py:37-50 and
 * xs/nn/functional.py:445-491 in a row; the backward is xsmi_maxpool2d_bwd followed by xsmi_bn_bwd with the mask. */
int xsmi_bn_relu_maxpool_fwd(const float *x, const float *gamma, const float *beta, float *pooled, uint8_t *idx,
                             uint8_t *neg_mask, float *sqrtvar, float *mean, float *var, float *moving_mean, float *moving_var,
                             float momentum, int N, int C, int H, int W, float eps, void *ws, size_t ws_bytes);
/* Inference form with given statistics (xs/nn/functional.py:708-725); relu != 0 clips at zero. */
int xsmi_bn_infer(const float *x, const float *gamma, const float *beta, const float *mean, const float *var, float *y,
                  int N, int C, int HW, float eps, int relu);
/* The same inference normalisation folded into the convolution that precedes it (the pair
 * xs/layers/convolutional.py:69-78 then xs/nn/functional.py:708-725 collapses to one convolution):
 * w_out[k][..] = w[k][..] * gamma[k] / sqrt(var[k] + eps), b_out[k] = beta[k] + (bias[k] - mean[k]) * that scale
 * (bias may be NULL).  w is (K, per_k). */
int xsmi_bn_fold(const float *w, const float *bias, const float *gamma, const float *beta, const float *mean,
                 const float *var, float *w_out, float *b_out, int K, int per_k, float eps);
/* Backward (xs/nn/grad_fn.py:379-411): dgamma = sum(dy*xhat), dbeta = sum(dy),
 * dx = gamma / (m*sqrtvar) * (m*dy - dbeta - xhat*dgamma), m = N*HW.  All three are overwritten.
 * With neg_mask (the byte mask of a fused ReLU) dy counts as 0 where the mask is set (strict mask,
 * xs/nn/grad_fn.py:146-157).
 * mean == NULL: xhat is the normalised input that xsmi_bn_fwd stored.  mean != NULL: xsmi_bn_fwd was
 * called with xhat == NULL, the `xhat` argument is the forward's input x, and (x - mean) / sqrtvar is
 * formed again on the fly (the same float operations, hence the same bits, without the forward's
 * extra write of a tensor of x's size). */
int xsmi_bn_bwd(const float *dy, const float *xhat, const float *mean, const float *sqrtvar, const float *gamma,
                const uint8_t *neg_mask, float *dx, float *dgamma, float *dbeta, int N, int C, int HW, void *ws,
                size_t ws_bytes);

/* xsmi_maxpool2d_bwd (3 x 3, stride 2, pad 1, beta 0) followed by xsmi_bn_bwd in its mean != NULL form, without the
 * pool's input gradient ever being stored: dpooled / idx are the pool's (N, C, H/2, W/2) upstream gradient and window
 * indices, x / mean / sqrtvar / gamma / neg_mask the normalisation's, as in xsmi_bn_bwd.  The routed gradient is formed
 * where the two passes need it, with the pool kernel's own arithmetic; dx is within float32 rounding of the two
 * separate calls (the channel sums are added in another order) and reproducible.  H even, W a multiple of 4.
 * Stands for xs/nn/grad_fn.py:206-235 followed by xs/nn/grad_fn.py:379-411 (and 146-157 through neg_mask). */
int xsmi_bn_bwd_maxpool(const float *dpooled, const uint8_t *idx, const float *x, const float *mean, const float *sqrtvar,
                        const float *gamma, const uint8_t *neg_mask, float *dx, float *dgamma, float *dbeta, int N, int C,
                        int H, int W, void *ws, size_t ws_bytes);

/* Mean over k x k windows at stride (sh, sw) of an NCHW tensor, no padding: y is (N, C, (H-k)/sh+1, (W-k)/sw+1),
 * float64 sum, one rounding; and its gradient, overwritten into dx: every window hands dy / k^2 (a float32 quotient)
 * to its cells, overlapping windows add up in float64 (avg_pool2d, xs/nn/functional.py:539-583,
 * xs/nn/grad_fn.py:284-309; the reference's padded mode miscounts its output size and is not offered). */
int xsmi_avgpool_fwd(const float *x, float *y, int N, int C, int H, int W, int k, int sh, int sw);
int xsmi_avgpool_bwd(const float *dy, float *dx, int N, int C, int H, int W, int k, int sh, int sw);

/* C[M,N] = op(A) . op(B) (+ bias[N] broadcast over rows); row-major, float32.  op is a transpose when
 * trans_a / trans_b is non-zero: A is stored (K,M) resp. B is stored (N,K).
 * (Dense layer: xs/nn/functional.py:99-120, xs/nn/grad_fn.py:86-99.)
 * workspace may be NULL.  With one, a product with few output tiles and a long K is split along K over
 * up to one workgroup per compute unit (at most workspace_bytes / (4*M*N) splits, 4*M*N bytes each) and
 * the partial products are added in ascending K order by a second kernel: the result does not depend on
 * timing, only on the number of splits. */
int xsmi_gemm(const float *A, const float *B, const float *bias, float *C, int M, int N, int K, int trans_a, int trans_b,
              void *workspace, size_t workspace_bytes);
/* out[j] = sum_i a[i][j] over an (M, N) matrix */
int xsmi_colsum(const float *a, float *out, int M, int N);
/* out[0] = sum of all n elements (float64 accumulation, one workgroup) */
int xsmi_sum_all(const float *a, float *out, size_t n);

/* Softmax + negative log-likelihood over rows of an (M, N) matrix with int64 labels
 * (xs/nn/functional.py:984-1010): sm = softmax(logits), loss[0] = mean or sum of -log sm[i, label[i]].
 * `loss` must hold 1 + M floats (loss[1..M] receives the per-row terms). */
int xsmi_softmax_ce_fwd(const float *logits, const int64_t *labels, float *sm, float *loss, int M, int N, int mean);
/* dlogits = (sm - onehot(labels)) * scale * (upstream ? upstream[0] : 1)      (xs/nn/grad_fn.py:604-620)
 * upstream: the loss's own gradient as one float in device memory (or NULL), so that the caller need not
 * read it back to the host. */
int xsmi_softmax_ce_bwd(const float *sm, const int64_t *labels, const float *upstream, float *dlogits, int M, int N,
                        float scale);

#ifdef __cplusplus
}
#endif
#endif /* XSMI355_H */
