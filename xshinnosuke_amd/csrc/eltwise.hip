// Element-wise helpers of the conv path and the workspace query.
#include "xsmi_internal.h"

namespace xsmi {
size_t conv_fwd_ws_bytes(int C, int K, int R, int S);
size_t conv_bwd_data_ws_bytes(int C, int K, int R, int S, int sh, int sw);
size_t conv_bwd_weight_ws_bytes(int N, int C, int K, int R, int S, int OH, int OW);
}  // namespace xsmi

namespace {

// dx = (accumulate ? dx : 0) + (mask ? 0 : dy); four elements per thread when aligned.
__global__ void __launch_bounds__(256) relu_mask_bwd_kernel(const float *__restrict__ dy, const uint8_t *__restrict__ mask,
                                                             float *dx, size_t n, int accumulate) {
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    if (i + 4 <= n) {
        float4 g = *reinterpret_cast<const float4 *>(dy + i);
        uchar4 m = *reinterpret_cast<const uchar4 *>(mask + i);
        float4 o = make_float4(m.x ? 0.f : g.x, m.y ? 0.f : g.y, m.z ? 0.f : g.z, m.w ? 0.f : g.w);
        if (accumulate) {
            float4 d = *reinterpret_cast<const float4 *>(dx + i);
            o.x += d.x; o.y += d.y; o.z += d.z; o.w += d.w;
        }
        *reinterpret_cast<float4 *>(dx + i) = o;
    } else {
        for (; i < n; ++i) {
            float o = mask[i] ? 0.f : dy[i];
            if (accumulate) o += dx[i];
            dx[i] = o;
        }
    }
}

// the same masked gradient delivered to two tensors at once (both inputs of the addition in front of the ReLU)
__global__ void __launch_bounds__(256) relu_mask_bwd2_kernel(const float *__restrict__ dy, const uint8_t *__restrict__ mask,
                                                              float *dx1, float *dx2, size_t n, int acc1, int acc2) {
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    if (i + 4 <= n) {
        float4 g = *reinterpret_cast<const float4 *>(dy + i);
        uchar4 m = *reinterpret_cast<const uchar4 *>(mask + i);
        const float4 o = make_float4(m.x ? 0.f : g.x, m.y ? 0.f : g.y, m.z ? 0.f : g.z, m.w ? 0.f : g.w);
        float4 o1 = o, o2 = o;
        if (acc1) {
            float4 d = *reinterpret_cast<const float4 *>(dx1 + i);
            o1.x += d.x; o1.y += d.y; o1.z += d.z; o1.w += d.w;
        }
        if (acc2) {
            float4 d = *reinterpret_cast<const float4 *>(dx2 + i);
            o2.x += d.x; o2.y += d.y; o2.z += d.z; o2.w += d.w;
        }
        *reinterpret_cast<float4 *>(dx1 + i) = o1;
        *reinterpret_cast<float4 *>(dx2 + i) = o2;
    } else {
        for (; i < n; ++i) {
            const float o = mask[i] ? 0.f : dy[i];
            dx1[i] = acc1 ? dx1[i] + o : o;
            dx2[i] = acc2 ? dx2[i] + o : o;
        }
    }
}

}  // namespace

extern "C" {

size_t xsmi_conv2d_pass_workspace_bytes(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad, int pass,
                                        unsigned flags) {
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || K <= 0 || R <= 0 || S <= 0 || sh <= 0 || sw <= 0 || pad < 0) return 0;
    if (H + 2 * pad < R || W + 2 * pad < S) return 0;
    const int OH = (H + 2 * pad - R) / sh + 1, OW = (W + 2 * pad - S) / sw + 1;
    const bool bf16 = (flags & XSMI_CONV_BF16) != 0;
    auto larger = [](size_t a, size_t b) { return a > b ? a : b; };
    size_t m = 0;
    if (pass == 0) {
        m = xsmi::conv_fwd_ws_bytes(C, K, R, S);
        if (!bf16 && xsmi::stem_fwd_ok(N, C, H, W, K, R, S, sh, sw, pad))
            m = larger(m, xsmi::stem_fwd_ws_bytes(N, C, H, W, K, R, S, sh, sw, pad));
        // the even-split fp32 kernels read their own filter layout (their partial tiles live in the library)
        if (!bf16 && xsmi::sk_path_ok(C, K)) m = larger(m, xsmi::sk_fwd_ws_bytes(C, K, R, S));
        // the bf16 forward takes its fastest form when the workspace also holds a channels-last copy of x
        if (bf16 && xsmi::nhwc_fwd_ok(N, C, H, W, K, R, S, pad)) m = larger(m, xsmi::nhwc_fwd_ws_bytes(N, C, H, W, K, R, S, pad));
    } else if (pass == 1) {
        m = xsmi::conv_bwd_data_ws_bytes(C, K, R, S, sh, sw);
        if (!bf16 && xsmi::sk_bwd_data_ok(C, K, R, S, sh, sw)) m = larger(m, xsmi::sk_bwd_data_ws_bytes(C, K, R, S, sh, sw));
    } else if (pass == 2) {
        m = xsmi::conv_bwd_weight_ws_bytes(N, C, K, R, S, OH, OW);
        if (!bf16 && xsmi::stem_wgrad_ok(N, C, H, W, K, R, S, sh, sw, pad))
            m = larger(m, xsmi::stem_wgrad_ws_bytes(N, C, H, W, K, R, S, sh, sw, pad));
    }
    return m;
}

size_t xsmi_conv2d_workspace_bytes(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad) {
    size_t m = 0;
    for (int pass = 0; pass < 3; ++pass)
        for (unsigned flags : {0u, (unsigned)XSMI_CONV_BF16}) {
            const size_t e = xsmi_conv2d_pass_workspace_bytes(N, C, H, W, K, R, S, sh, sw, pad, pass, flags);
            m = m > e ? m : e;
        }
    return m;
}

int xsmi_conv2d_bwd(const float *dy, const float *x, const float *w, float *dx, float *dw, float *db, int N, int C, int H,
                    int W, int K, int R, int S, int sh, int sw, int pad, float beta_dx, float beta_dw, unsigned flags,
                    void *workspace, size_t workspace_bytes, void *workspace_dw, size_t workspace_dw_bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && H > 0 && W > 0 && K > 0 && R > 0 && S > 0 && sh > 0 && sw > 0 && pad >= 0 &&
                       H + 2 * pad >= R && W + 2 * pad >= S,
                   "xsmi_conv2d_bwd: bad geometry");
    XSMI_CHECK_ARG(dy && x && w && dx && dw, "xsmi_conv2d_bwd: null tensor pointer");
    XSMI_CHECK_ARG((beta_dx == 0.f || beta_dx == 1.f) && (beta_dw == 0.f || beta_dw == 1.f), "xsmi_conv2d_bwd: beta must be 0 or 1");
    XSMI_CHECK_ARG((flags & ~(XSMI_CONV_BF16 | XSMI_CONV_DW_ASYNC | XSMI_CONV_WS_PACKED)) == 0,
                   "xsmi_conv2d_bwd: unknown flags 0x%x", flags);
    const int OH = (H + 2 * pad - R) / sh + 1, OW = (W + 2 * pad - S) / sw + 1;
    const size_t data_need = xsmi::conv_bwd_data_ws_bytes(C, K, R, S, sh, sw);
    const size_t weight_need = xsmi::conv_bwd_weight_ws_bytes(N, C, K, R, S, OH, OW);
    XSMI_CHECK_ARG(workspace && workspace_bytes >= data_need, "xsmi_conv2d_bwd: workspace of %zu bytes needed, %zu given",
                   data_need, workspace_bytes);
    XSMI_CHECK_ARG(workspace_dw && workspace_dw_bytes >= weight_need,
                   "xsmi_conv2d_bwd: weight-gradient workspace of %zu bytes needed, %zu given", weight_need, workspace_dw_bytes);
    XSMI_CHECK_ARG((char *)workspace + workspace_bytes <= (char *)workspace_dw ||
                       (char *)workspace_dw + workspace_dw_bytes <= (char *)workspace,
                   "xsmi_conv2d_bwd: the two workspaces overlap");
    const unsigned kflags = flags & XSMI_CONV_BF16;
    // The two kernels share only their inputs.  XSMI_CONV_DW_ASYNC: the weight gradient goes to the second stream
    // and stays there; the main stream runs on (data gradient, then whatever the caller enqueues next: the
    // memory-bound passes between two convolutions of a backward sweep fit beside a matrix-bound kernel) until
    // xsmi_conv2d_bwd_join.  Without the flag the call is complete in main-stream order when it returns: where the
    // data gradient's grid (128-pixel x 64-channel tiles) leaves compute units idle the weight gradient still runs
    // beside it (6-9 % less time for both at 7x7 and 14x14 feature maps) and is joined at once; grids that fill the
    // chip alone only get in each other's way (15 % more time at 56x56) and run one after the other.
    const long long tiles = (((long long)N * H * W + 127) / 128) * xsmi::ceil_div(C, 64);
    const bool async = (flags & XSMI_CONV_DW_ASYNC) != 0;
    const bool beside = async || tiles <= xsmi::cu_count();
    int rc = beside ? xsmi::side_begin() : xsmi::side_join();    // in main-stream order: after any earlier async work
    if (rc) return rc;
    rc = xsmi_conv2d_bwd_weight(dy, x, dw, db, N, C, H, W, K, R, S, sh, sw, pad, beta_dw, kflags, workspace_dw, workspace_dw_bytes);
    if (beside) xsmi::side_end();
    if (rc == XSMI_OK)
        rc = xsmi_conv2d_bwd_data(dy, w, dx, N, C, H, W, K, R, S, sh, sw, pad, beta_dx, kflags | (flags & XSMI_CONV_WS_PACKED),
                                  workspace, workspace_bytes);
    const int rj = (beside && !async) || rc ? xsmi::side_join() : XSMI_OK;
    return rc ? rc : rj;
}

int xsmi_relu_mask_bwd(const float *dy, const uint8_t *neg_mask, float *dx, size_t n, float beta) {
    XSMI_REQUIRE_INIT();
    if (n == 0) return XSMI_OK;
    XSMI_CHECK_ARG(dy && neg_mask && dx, "xsmi_relu_mask_bwd: null pointer");
    XSMI_CHECK_ARG(beta == 0.f || beta == 1.f, "xsmi_relu_mask_bwd: beta must be 0 or 1");
    size_t threads = (n + 3) / 4;
    hipLaunchKernelGGL(relu_mask_bwd_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, xsmi::stream(), dy,
                       neg_mask, dx, n, beta == 1.f ? 1 : 0);
    XSMI_LAUNCH_CHECK("relu_mask_bwd_kernel");
    return XSMI_OK;
}

int xsmi_relu_mask_bwd2(const float *dy, const uint8_t *neg_mask, float *dx1, float beta1, float *dx2, float beta2, size_t n) {
    XSMI_REQUIRE_INIT();
    if (n == 0) return XSMI_OK;
    XSMI_CHECK_ARG(dy && neg_mask && dx1 && dx2, "xsmi_relu_mask_bwd2: null pointer");
    XSMI_CHECK_ARG(dx1 != dx2, "xsmi_relu_mask_bwd2: the two outputs must differ");
    XSMI_CHECK_ARG((beta1 == 0.f || beta1 == 1.f) && (beta2 == 0.f || beta2 == 1.f), "xsmi_relu_mask_bwd2: beta must be 0 or 1");
    XSMI_CHECK_ARG((((uintptr_t)dy | (uintptr_t)dx1 | (uintptr_t)dx2) & 15) == 0 && ((uintptr_t)neg_mask & 3) == 0,
                   "xsmi_relu_mask_bwd2: tensors must be 16-byte aligned (mask: 4)");
    size_t threads = (n + 3) / 4;
    hipLaunchKernelGGL(relu_mask_bwd2_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, xsmi::stream(), dy,
                       neg_mask, dx1, dx2, n, beta1 == 1.f ? 1 : 0, beta2 == 1.f ? 1 : 0);
    XSMI_LAUNCH_CHECK("relu_mask_bwd2_kernel");
    return XSMI_OK;
}

}  // extern "C"
