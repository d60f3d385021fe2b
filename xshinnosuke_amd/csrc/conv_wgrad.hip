// Backward-weight (and bias) of the convolution on fp32 MFMA.
//
//     dw[k][j] += sum over pixels m = (n, oh, ow) of dy[n,k,oh,ow] * xpad[n, c, oh*sh + r - pad, ow*sw + s - pad]
//     db[k]    += sum over pixels of dy[n,k,oh,ow]                       j = (c*R + r)*S + s
//
// which is the reference's  dot(grad_reshaped, col)  and  sum(dy, axis=(0,2,3))
// (xs/nn/grad_fn.py:191-197) with the unfolded matrix formed on the fly.  The
// reduction runs over pixels, contiguous in memory for both operands, so lanes
// stream along ow.  The output is small (K x C*R*S) and the reduction long, so
// the pixel range is cut into `splits` pieces: every workgroup writes a 64x64
// partial tile for its piece and a second kernel adds the pieces in float64 in
// ascending order (deterministic; no float atomics), applies beta and rounds once.
#include "xsmi_internal.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TK = 64;     // filter rows per workgroup
constexpr int TJ = 64;     // (c,r,s) columns per workgroup
constexpr int MC = 32;     // pixels per reduction chunk
constexpr int LDW = 20;    // padded length of a 16-float LDS row
constexpr int TARGET_BLOCKS = 1024;

struct WgradParams {
    const float *dy;
    const float *x;
    float *part;       // [splits][Kp][Jp]
    float *dbpart;     // [splits][Kp] or nullptr
    uint32_t x_bytes, dy_bytes;
    int K, C, R, S, J, H, W, OH, OW, OHW, sh, sw, pad;
    int M, chunks_per_split;
    int Kp, Jp;
    xsmi::FastDiv dOHW, dOW, dRS, dS;
};

__device__ __forceinline__ float buffer_load_f32(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)byte_off, 0, 0));
}

__global__ void __launch_bounds__(256) wgrad_f32_kernel(WgradParams p) {
    __shared__ __attribute__((aligned(16))) float As[2][2][TK][LDW];
    __shared__ __attribute__((aligned(16))) float Bs[2][2][TJ][LDW];

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = t >> 6;
    const int j0 = blockIdx.x * TJ;
    const int k0 = blockIdx.y * TK;
    const int split = blockIdx.z;
    const bool want_db = p.dbpart != nullptr && blockIdx.x == 0;

    // ---- staging role: pixel mm of the chunk, rows/columns g8 + 8a ----
    const int mm = t & 31;
    const int g8 = t >> 5;
    int coff[8];     // element offset of column's (c, r-pad, s-pad) inside one image
    int drs[8];      // (r - pad) in the low half, (s - pad) in the high half
#pragma unroll
    for (int a = 0; a < 8; ++a) {
        int j = j0 + g8 + 8 * a;
        if (j < p.J) {
            uint32_t c = xsmi::fdiv((uint32_t)j, p.dRS);
            int rs = j - (int)c * (p.R * p.S);
            int r = (int)xsmi::fdiv((uint32_t)rs, p.dS);
            int s = rs - r * p.S;
            coff[a] = ((int)c * p.H + (r - p.pad)) * p.W + (s - p.pad);
            drs[a] = (int)(((uint32_t)(r - p.pad) & 0xffffu) | ((uint32_t)(s - p.pad) << 16));
        } else {
            coff[a] = 0;
            drs[a] = (int)(((uint32_t)(-30000) & 0xffffu) | ((uint32_t)(-30000) << 16));   // always out of range
        }
    }
    const int krow0 = k0 + g8;

    __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.x_bytes, 0x00020000);
    __amdgpu_buffer_rsrc_t gr = __builtin_amdgcn_make_buffer_rsrc((void *)p.dy, 0, p.dy_bytes, 0x00020000);

    const int chunk_begin = split * p.chunks_per_split;
    int nchunks = p.chunks_per_split;
    {
        int total_chunks = (p.M + MC - 1) / MC;
        if (chunk_begin + nchunks > total_chunks) nchunks = total_chunks - chunk_begin;
        if (nchunks < 0) nchunks = 0;
    }

    float an[8], bn[8];
    float dbsum[8];
#pragma unroll
    for (int a = 0; a < 8; ++a) dbsum[a] = 0.f;

    auto fetch = [&](int chunk) {
        int m = (chunk_begin + chunk) * MC + mm;
        bool live = m < p.M;
        uint32_t n = xsmi::fdiv((uint32_t)m, p.dOHW);
        int pix = m - (int)n * p.OHW;
        int oh = (int)xsmi::fdiv((uint32_t)pix, p.dOW);
        int ow = pix - oh * p.OW;
        int ihb = oh * p.sh, iwb = ow * p.sw;
        int xbase = (int)n * p.C * p.H * p.W + ihb * p.W + iwb;
        int gbase = (int)n * p.K * p.OHW + pix;
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            int krow = krow0 + 8 * a;
            bool ok = live && krow < p.K;
            uint32_t off = ok ? (uint32_t)(gbase + krow * p.OHW) * 4u : 0xffffffffu;
            an[a] = buffer_load_f32(gr, off);
        }
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            int ih = ihb + (int)(short)(drs[a] & 0xffff);
            int iw = iwb + (drs[a] >> 16);
            bool ok = live && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
            uint32_t off = ok ? (uint32_t)(xbase + coff[a]) * 4u : 0xffffffffu;
            bn[a] = buffer_load_f32(xr, off);
        }
    };
    auto stage = [&](int buf) {
        const int hh = mm >> 4, e = mm & 15;
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            As[buf][hh][g8 + 8 * a][e] = an[a];
            Bs[buf][hh][g8 + 8 * a][e] = bn[a];
        }
        if (want_db) {
#pragma unroll
            for (int a = 0; a < 8; ++a) dbsum[a] += an[a];
        }
    };

    floatx16 acc = {0};
    const int h = lane >> 5, l31 = lane & 31;
    const int wi = wave >> 1, wj = wave & 1;

    if (nchunks > 0) {
        fetch(0);
        stage(0);
    }
    __syncthreads();
    for (int c = 0; c < nchunks; ++c) {
        const int cur = c & 1;
        const bool more = c + 1 < nchunks;
        if (more) fetch(c + 1);
        const float4 *ap = reinterpret_cast<const float4 *>(&As[cur][h][wi * 32 + l31][0]);
        const float4 *bp = reinterpret_cast<const float4 *>(&Bs[cur][h][wj * 32 + l31][0]);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float4 a4 = ap[q], b4 = bp[q];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.x, b4.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.y, b4.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.z, b4.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.w, b4.w, acc, 0, 0, 0);
        }
        if (more) stage(cur ^ 1);
        __syncthreads();
    }

    // accumulator register v of lane l: row 8*(v/4) + 4*(l/32) + v%4, column l%32
    float *dst = p.part + ((size_t)split * p.Kp + k0 + wi * 32 + 4 * h) * p.Jp + j0 + wj * 32 + l31;
#pragma unroll
    for (int v = 0; v < 16; ++v) dst[(size_t)(8 * (v >> 2) + (v & 3)) * p.Jp] = acc[v];

    if (want_db) {
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            float s = dbsum[a];
            s += __shfl_xor(s, 16);
            s += __shfl_xor(s, 8);
            s += __shfl_xor(s, 4);
            s += __shfl_xor(s, 2);
            s += __shfl_xor(s, 1);
            if (mm == 0) p.dbpart[(size_t)split * p.Kp + krow0 + 8 * a] = s;
        }
    }
}

// dw[k][j] = beta*dw + sum over splits of part[split][k][j]; blocks past the last dw block do the same for
// db[k] from dbpart[split][k].  256 threads = 64 consecutive columns x 4 interleaved split groups with two
// running sums each; the groups are combined in a fixed order, all in float64 (deterministic, no atomics).
__global__ void __launch_bounds__(256) wgrad_reduce_kernel(const float *__restrict__ part, float *__restrict__ dw,
                                                            const float *__restrict__ dbpart, float *__restrict__ db,
                                                            int K, int J, int Kp, int Jp, int splits, int dw_blocks,
                                                            int accumulate) {
    __shared__ double sm[4][64];
    const int cl = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int jt = (J + 63) / 64;
    const bool bias_block = (int)blockIdx.x >= dw_blocks;      // uniform per block
    const float *src = nullptr;
    float *dst = nullptr;
    size_t stride = 0;
    if (bias_block) {
        const int k = ((int)blockIdx.x - dw_blocks) * 64 + cl;
        if (k < K) { src = dbpart + k; dst = db + k; }
        stride = (size_t)Kp;
    } else {
        const int k = (int)blockIdx.x / jt, j = ((int)blockIdx.x - k * jt) * 64 + cl;
        if (j < J) { src = part + (size_t)k * Jp + j; dst = dw + (size_t)k * J + j; }
        stride = (size_t)Kp * Jp;
    }
    double s0 = 0.0, s1 = 0.0;
    if (src) {
        int sp = g;
        for (; sp + 4 < splits; sp += 8) {
            s0 += (double)src[(size_t)sp * stride];
            s1 += (double)src[(size_t)(sp + 4) * stride];
        }
        if (sp < splits) s0 += (double)src[(size_t)sp * stride];
    }
    sm[g][cl] = s0 + s1;
    __syncthreads();
    if (g == 0 && dst) {
        double s = ((sm[0][cl] + sm[1][cl]) + sm[2][cl]) + sm[3][cl];
        if (accumulate) s += (double)*dst;
        *dst = (float)s;
    }
}

void plan_splits(int M, int K, int J, int *splits, int *chunks_per_split) {
    int tiles = xsmi::ceil_div(K, TK) * xsmi::ceil_div(J, TJ);
    int total_chunks = xsmi::ceil_div(M, MC);
    int want = xsmi::ceil_div(TARGET_BLOCKS, tiles);
    if (want < 1) want = 1;
    int cps = xsmi::ceil_div(total_chunks, want);
    if (cps < 4) cps = 4;                        // at least 128 pixels per piece
    if (cps > total_chunks) cps = total_chunks;
    *chunks_per_split = cps;
    *splits = xsmi::ceil_div(total_chunks, cps);
}

}  // namespace

namespace xsmi {
size_t conv_bwd_weight_ws_bytes(int N, int C, int K, int R, int S, int OH, int OW) {
    int splits, cps;
    plan_splits(N * OH * OW, K, C * R * S, &splits, &cps);
    size_t Kp = align_up(K, TK), Jp = align_up((size_t)C * R * S, TJ);
    size_t generic = align_up((size_t)splits * Kp * Jp * sizeof(float), 256) + align_up((size_t)splits * Kp * sizeof(float), 256);
    if (C % 64 == 0 && K % 64 == 0) {
        size_t tap = wgrad_tap_ws_bytes(N, C, K, R, S, OH, OW);
        return tap > generic ? tap : generic;
    }
    return generic;
}

int wgrad_reduce_partials(const float *part, float *dw, const float *dbpart, float *db, int K, int J, int Kp, int Jp, int splits,
                          int accumulate) {
    const int dw_blocks = K * ceil_div(J, 64);
    hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(dw_blocks + (db ? ceil_div(K, 64) : 0)), dim3(256), 0, stream(), part, dw, dbpart,
                       db, K, J, Kp, Jp, splits, dw_blocks, accumulate);
    XSMI_LAUNCH_CHECK("wgrad_reduce_kernel");
    return XSMI_OK;
}
}  // namespace xsmi

extern "C" {

int xsmi_conv2d_bwd_weight(const float *dy, const float *x, float *dw, float *db, int N, int C, int H, int W, int K,
                           int R, int S, int sh, int sw, int pad, float beta, unsigned flags, void *workspace,
                           size_t workspace_bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && H > 0 && W > 0 && K > 0, "xsmi_conv2d_bwd_weight: empty tensor");
    XSMI_CHECK_ARG(R >= 1 && S >= 1 && R <= 31 && S <= 31, "xsmi_conv2d_bwd_weight: filter %dx%d outside 1..31", R, S);
    XSMI_CHECK_ARG(sh >= 1 && sw >= 1 && pad >= 0, "xsmi_conv2d_bwd_weight: bad stride/padding");
    XSMI_CHECK_ARG(H + 2 * pad >= R && W + 2 * pad >= S, "xsmi_conv2d_bwd_weight: filter larger than the padded input");
    XSMI_CHECK_ARG(dy && x && dw, "xsmi_conv2d_bwd_weight: null tensor pointer");
    XSMI_CHECK_ARG(beta == 0.f || beta == 1.f, "xsmi_conv2d_bwd_weight: beta must be 0 or 1");
    XSMI_CHECK_ARG((flags & ~(XSMI_CONV_BF16 | XSMI_CONV_WS_PACKED)) == 0, "xsmi_conv2d_bwd_weight: unknown flags 0x%x", flags);
    // XSMI_CONV_BF16 is a permission, not a request: the weight gradient always runs on fp32 MFMA
    const int OH = (H + 2 * pad - R) / sh + 1, OW = (W + 2 * pad - S) / sw + 1;
    const double lim = 536870912.0;
    XSMI_CHECK_ARG((double)N * C * H * W < lim && (double)N * K * OH * OW < lim && (double)K * C * R * S < lim,
                   "xsmi_conv2d_bwd_weight: tensors of 2^29 elements or more are not supported");
    const size_t need = xsmi::conv_bwd_weight_ws_bytes(N, C, K, R, S, OH, OW);
    XSMI_CHECK_ARG(workspace && workspace_bytes >= need,
                   "xsmi_conv2d_bwd_weight: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    // called on the main stream while weight gradients of xsmi_conv2d_bwd are still on the second one: they may
    // add into the same dw, so they come first
    if (!xsmi::on_side_stream()) {
        int rj = xsmi::side_join();
        if (rj) return rj;
    }

    if (xsmi::stem_wgrad_ok(N, C, H, W, K, R, S, sh, sw, pad) && ((uintptr_t)dy & 15) == 0 &&
        workspace_bytes >= xsmi::stem_wgrad_ws_bytes(N, C, H, W, K, R, S, sh, sw, pad))
        return xsmi::stem_conv_bwd_weight(dy, x, dw, db, N, C, H, W, K, R, S, sh, sw, pad, OH, OW, beta == 1.f ? 1 : 0, workspace);
    if (xsmi::wgrad_tap_ok(dy, x, C, K, OH, OW))
        return xsmi::wgrad_tap(dy, x, dw, db, N, C, H, W, K, R, S, sh, sw, pad, OH, OW, beta == 1.f ? 1 : 0, workspace);

    WgradParams p;
    p.dy = dy; p.x = x;
    p.K = K; p.C = C; p.R = R; p.S = S; p.J = C * R * S; p.H = H; p.W = W; p.OH = OH; p.OW = OW; p.OHW = OH * OW;
    p.sh = sh; p.sw = sw; p.pad = pad;
    p.M = N * OH * OW;
    int splits;
    plan_splits(p.M, K, p.J, &splits, &p.chunks_per_split);
    p.Kp = (int)xsmi::align_up(K, TK);
    p.Jp = (int)xsmi::align_up(p.J, TJ);
    p.part = (float *)workspace;
    float *dbpart = (float *)((char *)workspace + xsmi::align_up((size_t)splits * p.Kp * p.Jp * sizeof(float), 256));
    p.dbpart = db ? dbpart : nullptr;
    p.x_bytes = (uint32_t)((size_t)N * C * H * W * 4);
    p.dy_bytes = (uint32_t)((size_t)N * K * OH * OW * 4);
    p.dOHW = xsmi::make_fastdiv(p.OHW); p.dOW = xsmi::make_fastdiv(OW);
    p.dRS = xsmi::make_fastdiv(R * S); p.dS = xsmi::make_fastdiv(S);

    hipStream_t st = xsmi::stream();
    dim3 grid(p.Jp / TJ, p.Kp / TK, splits);
    xsmi::prof_begin();
    hipLaunchKernelGGL(wgrad_f32_kernel, grid, dim3(256), 0, st, p);
    xsmi::prof_end();
    XSMI_LAUNCH_CHECK("wgrad_f32_kernel");
    const int acc = beta == 1.f ? 1 : 0;
    const int dw_blocks = K * xsmi::ceil_div(p.J, 64);
    hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(dw_blocks + (db ? xsmi::ceil_div(K, 64) : 0)), dim3(256), 0, st, p.part, dw,
                       dbpart, db, K, p.J, p.Kp, p.Jp, splits, dw_blocks, acc);
    XSMI_LAUNCH_CHECK("wgrad_reduce_kernel");
    return XSMI_OK;
}

}  // extern "C"
