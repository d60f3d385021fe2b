// Neighbours of the bf16 convolution on channels-last bf16 activations.
//
// A channels-last tensor is bf16 [N][H + 2 b][W + 2 b][C] with a zero border of b pixels and C a multiple of 8: eight
// consecutive channels of a pixel are one 16-byte vector, which is what the bf16 convolution kernel loads as an MFMA
// operand, so a chain conv -> add/ReLU -> pool -> conv never rewrites its activations as fp32 NCHW.  All three
// kernels here move 16-byte vectors and are bound by memory bandwidth:
//   cl_add_relu   out = max(0, a + b) (or a + b) over whole buffers, borders included (0 + 0 = 0 keeps them zero)
//   cl_maxpool    k x k / stride max pooling; the zero border of the input IS the reference's zero-valued padding
//                 that takes part in the max (xs/nn/functional.py:445-491), so no bounds tests in the window loop
//   cl_to_nchw    the fp32 NCHW form of a channels-last tensor, for every consumer that does not read channels-last
#include "xsmi_internal.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__global__ void __launch_bounds__(256) cl_add_kernel(const bf16x8 *__restrict__ a, const bf16x8 *__restrict__ b,
                                                      bf16x8 *__restrict__ out, size_t vecs, int relu) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= vecs) return;
    const bf16x8 va = a[i], vb = b[i];
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float s = (float)va[e] + (float)vb[e];
        if (relu) s = s > 0.f ? s : 0.f;
        r[e] = (__bf16)s;
    }
    out[i] = r;
}

// one thread = one output pixel x eight channels; consecutive threads = consecutive channel octets, then pixels.
// K > 0: the window size at compile time, so that the K * K loads of a thread are all issued before the first
// comparison (with a run-time window each load waits for the comparison loop in front of it).
template <int K>
__global__ void __launch_bounds__(256) cl_maxpool_kernel(const bf16x8 *__restrict__ x, bf16x8 *__restrict__ y, int C8, int Wpi,
                                                          int Hpi, int off, int k_rt, int sh, int sw, int OH, int OW, int Wpo,
                                                          int Hpo, int ob, uint32_t total, xsmi::FastDiv dC8,
                                                          xsmi::FastDiv dOW, xsmi::FastDiv dOH) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= total) return;
    const uint32_t pq = xsmi::fdiv(i, dC8), c8 = i - pq * (uint32_t)C8;
    const uint32_t rq = xsmi::fdiv(pq, dOW), ox = pq - rq * (uint32_t)OW;
    const uint32_t n = xsmi::fdiv(rq, dOH), oy = rq - n * (uint32_t)OH;
    // window origin inside the padded input: (border - pad) + stride * o
    const bf16x8 *src = x + (((size_t)n * Hpi + (size_t)(off + (int)oy * sh)) * Wpi + (size_t)(off + (int)ox * sw)) * C8 + c8;
    float m[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) m[e] = -INFINITY;
    if (K > 0) {
        bf16x8 v[K > 0 ? K * K : 1];
#pragma unroll
        for (int r = 0; r < K; ++r)
#pragma unroll
            for (int s = 0; s < K; ++s) v[r * K + s] = src[((size_t)r * Wpi + s) * C8];
#pragma unroll
        for (int t = 0; t < K * K; ++t)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float f = (float)v[t][e];
                m[e] = f > m[e] ? f : m[e];
            }
    } else {
        for (int r = 0; r < k_rt; ++r)
            for (int s = 0; s < k_rt; ++s) {
                const bf16x8 v = src[((size_t)r * Wpi + s) * C8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float f = (float)v[e];
                    m[e] = f > m[e] ? f : m[e];
                }
            }
    }
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (__bf16)m[e];
    y[(((size_t)n * Hpo + oy + ob) * Wpo + ox + ob) * C8 + c8] = o;
}

// A workgroup converts one segment (at most 255 pixels) of an image row for 64 channels through an LDS tile
// [64][seg | 1] of floats: reading, eight threads cover a pixel's 64 channels (128 contiguous bytes); writing, a wave
// writes runs of one channel's row.
__global__ void __launch_bounds__(256) cl_to_nchw_kernel(const bf16x8 *__restrict__ x, float *__restrict__ y, int C, int H, int Wfull,
                                                          int b, int cgroups, int seg, int segs) {
    extern __shared__ float tile[];                   // [64][seg | 1]
    const int ldw = seg | 1;
    const int t = threadIdx.x;
    const int cg = (int)(blockIdx.x % (uint32_t)cgroups);
    const int part = (int)((blockIdx.x / (uint32_t)cgroups) % (uint32_t)segs);
    const int rowid = (int)(blockIdx.x / (uint32_t)(cgroups * segs));       // n * H + h
    const int h = rowid % H, n = rowid / H;
    const int w0 = part * seg;
    const int W = Wfull - w0 < seg ? Wfull - w0 : seg;            // pixels of this segment
    const int Wp = Wfull + 2 * b, Hp = H + 2 * b, C8 = C / 8;
    const int c0 = cg * 64;
    const int oct = t & 7;                             // octet of the 64-channel group
    const bool oct_ok = c0 + oct * 8 < C;
    const bf16x8 *row = x + (((size_t)n * Hp + h + b) * Wp + b + w0) * C8 + (c0 >> 3) + oct;
    for (int px = t >> 3; px < W; px += 32) {
        if (oct_ok) {
            const bf16x8 v = row[(size_t)px * C8];
#pragma unroll
            for (int e = 0; e < 8; ++e) tile[(oct * 8 + e) * ldw + px] = (float)v[e];
        }
    }
    __syncthreads();
    const int nch = C - c0 < 64 ? C - c0 : 64;
    float *dst = y + (((size_t)n * C + c0) * H + h) * Wfull + w0;
    for (int i = t; i < nch * W; i += 256) {
        const int c = i / W, px = i - c * W;
        dst[(size_t)c * H * Wfull + px] = tile[c * ldw + px];
    }
}

}  // namespace

int xsmi_cl_add(const void *a, const void *b, void *out, size_t count, int relu) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(a && b && out, "xsmi_cl_add: null pointer");
    XSMI_CHECK_ARG(count % 8 == 0 && (((uintptr_t)a | (uintptr_t)b | (uintptr_t)out) & 15) == 0,
                   "xsmi_cl_add: count must be a multiple of 8 and the buffers 16-byte aligned");
    const size_t vecs = count / 8;
    if (vecs == 0) return XSMI_OK;
    XSMI_CHECK_ARG((vecs + 255) / 256 < ((size_t)1 << 31), "xsmi_cl_add: too many elements");
    hipLaunchKernelGGL(cl_add_kernel, dim3((unsigned)((vecs + 255) / 256)), dim3(256), 0, xsmi::stream(), (const bf16x8 *)a,
                       (const bf16x8 *)b, (bf16x8 *)out, vecs, relu);
    XSMI_LAUNCH_CHECK("cl_add_kernel");
    return XSMI_OK;
}

int xsmi_cl_maxpool2d(const void *x_cl, int x_border, void *y_cl, int y_border, int N, int C, int H, int W, int k, int sh,
                      int sw, int pad) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(x_cl && y_cl, "xsmi_cl_maxpool2d: null pointer");
    XSMI_CHECK_ARG(N > 0 && C > 0 && C % 8 == 0 && H > 0 && W > 0, "xsmi_cl_maxpool2d: needs C %% 8 == 0 (N=%d C=%d H=%d W=%d)", N,
                   C, H, W);
    XSMI_CHECK_ARG(k >= 1 && sh >= 1 && sw >= 1 && pad >= 0 && x_border >= pad && y_border >= 0,
                   "xsmi_cl_maxpool2d: window %d stride %dx%d pad %d needs an input border >= pad (%d)", k, sh, sw, pad, x_border);
    XSMI_CHECK_ARG(H + 2 * pad >= k && W + 2 * pad >= k, "xsmi_cl_maxpool2d: window larger than the padded input");
    XSMI_CHECK_ARG((((uintptr_t)x_cl | (uintptr_t)y_cl) & 15) == 0, "xsmi_cl_maxpool2d: buffers must be 16-byte aligned");
    const int OH = (H + 2 * pad - k) / sh + 1, OW = (W + 2 * pad - k) / sw + 1;
    const int C8 = C / 8;
    const size_t total = (size_t)N * OH * OW * C8;
    XSMI_CHECK_ARG(total < ((size_t)1 << 32), "xsmi_cl_maxpool2d: too many outputs");
    const dim3 grid((unsigned)((total + 255) / 256));
#define XSMI_CL_POOL(KK)                                                                                                     \
    hipLaunchKernelGGL(cl_maxpool_kernel<KK>, grid, dim3(256), 0, xsmi::stream(), (const bf16x8 *)x_cl, (bf16x8 *)y_cl, C8,    \
                       W + 2 * x_border, H + 2 * x_border, x_border - pad, k, sh, sw, OH, OW, OW + 2 * y_border,              \
                       OH + 2 * y_border, y_border, (uint32_t)total, xsmi::make_fastdiv(C8), xsmi::make_fastdiv(OW),          \
                       xsmi::make_fastdiv(OH))
    if (k == 3) XSMI_CL_POOL(3);
    else if (k == 2) XSMI_CL_POOL(2);
    else XSMI_CL_POOL(0);
#undef XSMI_CL_POOL
    XSMI_LAUNCH_CHECK("cl_maxpool_kernel");
    return XSMI_OK;
}

int xsmi_cl_to_nchw(const void *x_cl, int border, float *y, int N, int C, int H, int W) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(x_cl && y, "xsmi_cl_to_nchw: null pointer");
    XSMI_CHECK_ARG(N > 0 && C > 0 && C % 8 == 0 && H > 0 && W > 0 && border >= 0,
                   "xsmi_cl_to_nchw: needs C %% 8 == 0 (N=%d C=%d H=%d W=%d border=%d)", N, C, H, W, border);
    XSMI_CHECK_ARG(((uintptr_t)x_cl & 15) == 0, "xsmi_cl_to_nchw: x_cl must be 16-byte aligned");
    // rows wider than 255 pixels are converted in equal segments (the tile of a segment must fit 64 KB of LDS)
    const int segs = xsmi::ceil_div(W, 255), seg = xsmi::ceil_div(W, segs);
    const size_t lds = (size_t)64 * (seg | 1) * sizeof(float);
    const int cgroups = xsmi::ceil_div(C, 64);
    const size_t blocks = (size_t)N * H * cgroups * segs;
    XSMI_CHECK_ARG(blocks < ((size_t)1 << 31), "xsmi_cl_to_nchw: too many rows");
    hipLaunchKernelGGL(cl_to_nchw_kernel, dim3((unsigned)blocks), dim3(256), lds, xsmi::stream(), (const bf16x8 *)x_cl, y, C, H, W,
                       border, cgroups, seg, segs);
    XSMI_LAUNCH_CHECK("cl_to_nchw_kernel");
    return XSMI_OK;
}
