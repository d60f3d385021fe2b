// Max-pool forward (values + first-max index) and backward (gather) kernels.
//
// Semantics (reference xs/nn/functional.py:445-491, xs/nn/grad_fn.py:224-235):
// the input is bordered with cells of value 0 that compete in the max; the
// window is scanned in row-major (ky,kx) order and a later cell replaces the
// current best only if it is strictly greater, which is np.argmax's "first
// maximum".  Backward sums, per input cell, the upstream gradient of every
// window whose recorded index points at that cell, in ascending (ky,kx) order in
// float64, and rounds once.
#include "xsmi_internal.h"
#include <stdlib.h>

namespace {

struct PoolGeom {
    int N, C, H, W, OH, OW, k, sh, sw, pad;
    xsmi::FastDiv dOW, dOH;   // forward: decompose the flat output index
    xsmi::FastDiv dW, dH;     // backward: decompose the flat input index
    xsmi::FastDiv dsh, dsw;   // backward: window range
};

// One thread per output element; lanes run along ow so that loads of one
// window row are contiguous across the wavefront.  KT > 0 unrolls the window.
template <int KT>
__global__ void __launch_bounds__(256) maxpool_fwd_generic(const float *__restrict__ x, float *__restrict__ y,
                                                            uint8_t *__restrict__ idx, PoolGeom g, uint32_t total) {
    uint32_t o = blockIdx.x * 256u + threadIdx.x;
    if (o >= total) return;
    const int k = KT > 0 ? KT : g.k;
    uint32_t t = xsmi::fdiv(o, g.dOW);
    int ow = (int)(o - t * g.OW);
    uint32_t nc = xsmi::fdiv(t, g.dOH);
    int oh = (int)(t - nc * g.OH);
    const float *plane = x + (size_t)nc * g.H * g.W;
    int ih0 = oh * g.sh - g.pad;
    int iw0 = ow * g.sw - g.pad;
    float best = 0.f;
    int where = 0;
    bool first = true;
#pragma unroll
    for (int r = 0; r < k; ++r) {
        int ih = ih0 + r;
        bool rowok = (unsigned)ih < (unsigned)g.H;
#pragma unroll
        for (int s = 0; s < k; ++s) {
            int iw = iw0 + s;
            float v = 0.f;                                   // border cell
            if (rowok && (unsigned)iw < (unsigned)g.W) v = plane[ih * g.W + iw];
            if (first || v > best) {
                best = v;
                where = r * k + s;
                first = false;
            }
        }
    }
    y[o] = best;
    if (idx) idx[o] = (uint8_t)where;
}

// 3x3 window, stride 2, pad 1, W % 4 == 0 (so OW = W/2): one thread produces two
// adjacent outputs of one row from float4 loads of columns [4j, 4j+3] of the
// three input rows; column 4j-1 comes from the previous lane (or one scalar load
// at a wavefront edge, or the zero border at j == 0).  x is fetched once per
// window row; the row shared by vertically adjacent windows is re-read from
// cache.
__global__ void __launch_bounds__(256) maxpool_fwd_3x3s2p1(const float *__restrict__ x, float *__restrict__ y,
                                                            uint8_t *__restrict__ idx, PoolGeom g,
                                                            xsmi::FastDiv dQ, uint32_t total_pairs) {
    uint32_t t = blockIdx.x * 256u + threadIdx.x;
    bool live = t < total_pairs;
    if (!live) t = total_pairs - 1;
    const int Q = g.OW >> 1;                 // output pairs per row == float4 per input row / 1
    uint32_t row = xsmi::fdiv(t, dQ);        // (nc, oh)
    int j = (int)(t - row * Q);
    uint32_t nc = xsmi::fdiv(row, g.dOH);
    int oh = (int)(row - nc * g.OH);
    const float *plane = x + (size_t)nc * g.H * g.W;
    const int lane = threadIdx.x & 63;

    float b0 = 0.f, b1 = 0.f;
    int w0 = 0, w1 = 0;
    bool first = true;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        int ih = 2 * oh - 1 + r;
        bool rowok = (unsigned)ih < (unsigned)g.H;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (rowok) v = *reinterpret_cast<const float4 *>(plane + (size_t)ih * g.W + 4 * j);
        float left = __shfl_up(v.w, 1);
        if (j == 0) left = 0.f;                                       // zero border
        else if (lane == 0) left = rowok ? plane[(size_t)ih * g.W + 4 * j - 1] : 0.f;
        // output 2j: columns 4j-1, 4j, 4j+1 ; output 2j+1: columns 4j+1, 4j+2, 4j+3
        if (first || left > b0) { b0 = left; w0 = r * 3 + 0; }
        if (v.x > b0) { b0 = v.x; w0 = r * 3 + 1; }
        if (v.y > b0) { b0 = v.y; w0 = r * 3 + 2; }
        if (first || v.y > b1) { b1 = v.y; w1 = r * 3 + 0; }
        if (v.z > b1) { b1 = v.z; w1 = r * 3 + 1; }
        if (v.w > b1) { b1 = v.w; w1 = r * 3 + 2; }
        first = false;
    }
    if (!live) return;
    size_t o = (size_t)row * g.OW + 2 * j;
    *reinterpret_cast<float2 *>(y + o) = make_float2(b0, b1);
    if (idx) *reinterpret_cast<uchar2 *>(idx + o) = make_uchar2((unsigned char)w0, (unsigned char)w1);
}

// One thread per input-gradient element.
__global__ void __launch_bounds__(256) maxpool_bwd_gather(const float *__restrict__ dy, const uint8_t *__restrict__ idx,
                                                           float *__restrict__ dx, PoolGeom g, uint32_t total, int accumulate) {
    uint32_t e = blockIdx.x * 256u + threadIdx.x;
    if (e >= total) return;
    uint32_t t = xsmi::fdiv(e, g.dW);
    int w = (int)(e - t * g.W);
    uint32_t nc = xsmi::fdiv(t, g.dH);
    int h = (int)(t - nc * g.H);
    int qh = h + g.pad, qw = w + g.pad;
    // windows oh with 0 <= qh - oh*sh < k, descending oh == ascending ky
    int oh_hi = (int)xsmi::fdiv((uint32_t)qh, g.dsh);
    int ow_hi = (int)xsmi::fdiv((uint32_t)qw, g.dsw);
    if (oh_hi > g.OH - 1) oh_hi = g.OH - 1;
    if (ow_hi > g.OW - 1) ow_hi = g.OW - 1;
    const size_t obase = (size_t)nc * g.OH * g.OW;
    double acc = 0.0;
    for (int oh = oh_hi; oh >= 0; --oh) {
        int r = qh - oh * g.sh;
        if (r >= g.k) break;
        for (int ow = ow_hi; ow >= 0; --ow) {
            int s = qw - ow * g.sw;
            if (s >= g.k) break;
            size_t o = obase + (size_t)oh * g.OW + ow;
            if ((int)idx[o] == r * g.k + s) acc += (double)dy[o];
        }
    }
    if (accumulate) acc += (double)dx[e];
    dx[e] = (float)acc;
}

// 3x3 / stride 2 / pad 1 with W % 4 == 0: one thread per four consecutive dx
// columns 4j..4j+3 of one row.  Covering windows: ow in {2j-1+1.. } i.e. columns
// qw = w+1 in [4j+1, 4j+4] are covered by ow = 2j (s = qw-4j in {1,2}),
// ow = 2j+1 (s in {0,1,2} for qw = 4j+2..4j+4) and ow = 2j+2 (s = 0 for qw = 4j+4).
__global__ void __launch_bounds__(256) maxpool_bwd_3x3s2p1(const float *__restrict__ dy, const uint8_t *__restrict__ idx,
                                                            float *__restrict__ dx, PoolGeom g, xsmi::FastDiv dQ4,
                                                            uint32_t total_quads, int accumulate) {
    uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= total_quads) return;
    const int Q4 = g.W >> 2;
    uint32_t row = xsmi::fdiv(t, dQ4);       // (nc, h)
    int j = (int)(t - row * Q4);
    uint32_t nc = xsmi::fdiv(row, g.dH);
    int h = (int)(row - nc * g.H);
    const size_t obase = (size_t)nc * g.OH * g.OW;
    const int qh = h + 1;
    double a0 = 0.0, a1 = 0.0, a2 = 0.0, a3 = 0.0;
    // ascending ky == descending oh; for one oh ascending kx == descending ow
    int oh_hi = qh >> 1;
    for (int oh = oh_hi; oh >= 0 && oh >= oh_hi - 1; --oh) {
        int r = qh - 2 * oh;
        if (r > 2 || oh >= g.OH) continue;
        const size_t ro = obase + (size_t)oh * g.OW;
        const int r3 = r * 3;
        // ow = 2j+2 (may be out of range), 2j+1, 2j
        int owc = 2 * j + 2;
        float gC = 0.f; int iC = -1;
        if (owc < g.OW) { gC = dy[ro + owc]; iC = idx[ro + owc]; }
        float2 gAB = *reinterpret_cast<const float2 *>(dy + ro + 2 * j);
        uchar2 iAB = *reinterpret_cast<const uchar2 *>(idx + ro + 2 * j);
        int iA = iAB.x, iB = iAB.y;
        // column 4j   (qw=4j+1): ow=2j s=1
        if (iA == r3 + 1) a0 += (double)gAB.x;
        // column 4j+1 (qw=4j+2): ow=2j+1 s=0 first (higher ow == lower kx), then ow=2j s=2
        if (iB == r3 + 0) a1 += (double)gAB.y;
        if (iA == r3 + 2) a1 += (double)gAB.x;
        // column 4j+2 (qw=4j+3): ow=2j+1 s=1
        if (iB == r3 + 1) a2 += (double)gAB.y;
        // column 4j+3 (qw=4j+4): ow=2j+2 s=0, then ow=2j+1 s=2
        if (iC == r3 + 0) a3 += (double)gC;
        if (iB == r3 + 2) a3 += (double)gAB.y;
    }
    float4 *out = reinterpret_cast<float4 *>(dx + (size_t)row * g.W + 4 * j);
    if (accumulate) {
        float4 old = *out;
        a0 += (double)old.x; a1 += (double)old.y; a2 += (double)old.z; a3 += (double)old.w;
    }
    *out = make_float4((float)a0, (float)a1, (float)a2, (float)a3);
}

// 3x3 / stride 2 / pad 1, W % 8 == 0, OH % RO == 0: one thread produces a 4-column x RO-row patch of outputs.
// It streams the 2*RO+1 input rows that patch needs (two 128-bit loads per row, the left neighbour column from the
// previous lane), so a row shared by vertically adjacent windows is loaded once per patch, and stores y as one
// 128-bit and idx as one 32-bit access per output row.
template <int RO>
__global__ void __launch_bounds__(256) maxpool_fwd_3x3s2p1_patch(const float *__restrict__ x, float *__restrict__ y,
                                                                  uint8_t *__restrict__ idx, PoolGeom g, xsmi::FastDiv dQ,
                                                                  xsmi::FastDiv dG, uint32_t total) {
    uint32_t t = blockIdx.x * 256u + threadIdx.x;
    const bool live = t < total;
    if (!live) t = total - 1;
    const int Q = g.OW >> 2, G = g.OH / RO;
    uint32_t rowg = xsmi::fdiv(t, dQ);       // (nc, row group)
    const int j = (int)(t - rowg * Q);
    uint32_t nc = xsmi::fdiv(rowg, dG);
    const int oh0 = ((int)(rowg - nc * G)) * RO;
    const float *plane = x + (size_t)nc * g.H * g.W;
    const int lane = threadIdx.x & 63;
    float best[RO][4];
    int where[RO][4];
    // all loads first (independent of each other), then the compare chains
    constexpr int NR = 2 * RO + 1;
    float4 va[NR], vb[NR];
    float lf[NR];
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const int ih = 2 * oh0 - 1 + i;
        va[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        vb[i] = va[i];
        lf[i] = 0.f;
        if ((unsigned)ih < (unsigned)g.H) {
            const float4 *src = reinterpret_cast<const float4 *>(plane + (size_t)ih * g.W + 8 * j);
            va[i] = src[0];
            vb[i] = src[1];
        }
    }
    if (lane == 0 && j > 0) {                     // the column left of a wavefront's first patch is not in any lane
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int ih = 2 * oh0 - 1 + i;
            if ((unsigned)ih < (unsigned)g.H) lf[i] = plane[(size_t)ih * g.W + 8 * j - 1];
        }
    }
#pragma unroll
    for (int i = 0; i <= 2 * RO; ++i) {
        const float4 v0 = va[i], v1 = vb[i];
        float left = __shfl_up(v1.w, 1);
        if (j == 0) left = 0.f;                                           // zero border
        else if (lane == 0) left = lf[i];
        const float c[9] = {left, v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
        // row i is window row 2 of output row i/2 - 1 (i even, i >= 2) and window row i%2 of output row i/2
        if ((i & 1) == 0 && i >= 2) {
            const int o = i / 2 - 1;
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int e = 0; e < 3; ++e)
                    if (c[2 * q + e] > best[o][q]) { best[o][q] = c[2 * q + e]; where[o][q] = 6 + e; }
        }
        if (i < 2 * RO) {
            const int o = i / 2, r3 = (i & 1) * 3;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if ((i & 1) == 0) { best[o][q] = c[2 * q]; where[o][q] = 0; }   // first cell of the window
                else if (c[2 * q] > best[o][q]) { best[o][q] = c[2 * q]; where[o][q] = r3; }
                if (c[2 * q + 1] > best[o][q]) { best[o][q] = c[2 * q + 1]; where[o][q] = r3 + 1; }
                if (c[2 * q + 2] > best[o][q]) { best[o][q] = c[2 * q + 2]; where[o][q] = r3 + 2; }
            }
        }
    }
    if (!live) return;
#pragma unroll
    for (int o = 0; o < RO; ++o) {
        size_t off = ((size_t)nc * g.OH + oh0 + o) * g.OW + 4 * j;
        *reinterpret_cast<float4 *>(y + off) = make_float4(best[o][0], best[o][1], best[o][2], best[o][3]);
        if (idx)
            *reinterpret_cast<uchar4 *>(idx + off) = make_uchar4((unsigned char)where[o][0], (unsigned char)where[o][1],
                                                                 (unsigned char)where[o][2], (unsigned char)where[o][3]);
    }
}

// Backward of the same geometry: one thread owns an 8-column x 2*RP-row patch of dx (rows 2a .. 2a+2RP-1) and reads
// the RP+1 output rows a .. a+RP that can route gradient into it (columns 4j .. 4j+4), each once.
// dx column 8j+2m   (even) is reached only through kx = 1 of output column 4j+m;
// dx column 8j+2m+1 (odd) through kx = 0 of output column 4j+m+1, then kx = 2 of output column 4j+m.
template <int RP>
__global__ void __launch_bounds__(256) maxpool_bwd_3x3s2p1_patch(const float *__restrict__ dy, const uint8_t *__restrict__ idx,
                                                                  float *__restrict__ dx, PoolGeom g, xsmi::FastDiv dQ8,
                                                                  xsmi::FastDiv dG, uint32_t total, int accumulate) {
    uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= total) return;
    const int Q8 = g.W >> 3, G = g.H / (2 * RP);
    uint32_t rowg = xsmi::fdiv(t, dQ8);
    const int j = (int)(t - rowg * Q8);
    uint32_t nc = xsmi::fdiv(rowg, dG);
    const int a0 = ((int)(rowg - nc * G)) * RP;
    const size_t obase = (size_t)nc * g.OH * g.OW;
    float gv[RP + 1][5];
    int iv[RP + 1][5];
#pragma unroll
    for (int q = 0; q <= RP; ++q) {
        const int oh = a0 + q;
#pragma unroll
        for (int m = 0; m < 5; ++m) { gv[q][m] = 0.f; iv[q][m] = -1; }
        if (oh < g.OH) {
            const size_t ro = obase + (size_t)oh * g.OW + 4 * j;
            float4 gg = *reinterpret_cast<const float4 *>(dy + ro);
            uchar4 ii = *reinterpret_cast<const uchar4 *>(idx + ro);
            gv[q][0] = gg.x; gv[q][1] = gg.y; gv[q][2] = gg.z; gv[q][3] = gg.w;
            iv[q][0] = ii.x; iv[q][1] = ii.y; iv[q][2] = ii.z; iv[q][3] = ii.w;
            if (4 * j + 4 < g.OW) { gv[q][4] = dy[ro + 4]; iv[q][4] = idx[ro + 4]; }
        }
    }
    auto take = [&](int q, int r, double *c) {
        const int r3 = 3 * r;
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            if (iv[q][m] == r3 + 1) c[2 * m] += (double)gv[q][m];
            if (iv[q][m + 1] == r3 + 0) c[2 * m + 1] += (double)gv[q][m + 1];
            if (iv[q][m] == r3 + 2) c[2 * m + 1] += (double)gv[q][m];
        }
    };
#pragma unroll
    for (int q = 0; q < RP; ++q) {
        const int h = 2 * (a0 + q);
        double ev[8] = {0, 0, 0, 0, 0, 0, 0, 0}, od[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        take(q, 1, ev);          // even row h: window row 1 of output row a0+q
        take(q + 1, 0, od);      // odd row h+1: window row 0 of output row a0+q+1 first (ascending ky) ...
        take(q, 2, od);          // ... then window row 2 of output row a0+q
        float4 *pe = reinterpret_cast<float4 *>(dx + ((size_t)nc * g.H + h) * g.W + 8 * j);
        float4 *po = reinterpret_cast<float4 *>(dx + ((size_t)nc * g.H + h + 1) * g.W + 8 * j);
        if (accumulate) {
            float4 a0v = pe[0], a1v = pe[1], b0v = po[0], b1v = po[1];
            ev[0] += (double)a0v.x; ev[1] += (double)a0v.y; ev[2] += (double)a0v.z; ev[3] += (double)a0v.w;
            ev[4] += (double)a1v.x; ev[5] += (double)a1v.y; ev[6] += (double)a1v.z; ev[7] += (double)a1v.w;
            od[0] += (double)b0v.x; od[1] += (double)b0v.y; od[2] += (double)b0v.z; od[3] += (double)b0v.w;
            od[4] += (double)b1v.x; od[5] += (double)b1v.y; od[6] += (double)b1v.z; od[7] += (double)b1v.w;
        }
        pe[0] = make_float4((float)ev[0], (float)ev[1], (float)ev[2], (float)ev[3]);
        pe[1] = make_float4((float)ev[4], (float)ev[5], (float)ev[6], (float)ev[7]);
        po[0] = make_float4((float)od[0], (float)od[1], (float)od[2], (float)od[3]);
        po[1] = make_float4((float)od[4], (float)od[5], (float)od[6], (float)od[7]);
    }
}

int check_geom(const char *fn, int N, int C, int H, int W, int k, int sh, int sw, int pad, PoolGeom *g) {
    XSMI_CHECK_ARG(N > 0 && C > 0 && H > 0 && W > 0, "%s: empty tensor (N=%d C=%d H=%d W=%d)", fn, N, C, H, W);
    XSMI_CHECK_ARG(k >= 1 && k <= 15, "%s: window %d outside 1..15 (index is stored in one byte)", fn, k);
    XSMI_CHECK_ARG(sh >= 1 && sw >= 1, "%s: stride must be positive", fn);
    XSMI_CHECK_ARG(pad >= 0, "%s: negative padding", fn);
    XSMI_CHECK_ARG(H + 2 * pad >= k && W + 2 * pad >= k, "%s: window %d larger than the padded input %dx%d", fn, k,
                   H + 2 * pad, W + 2 * pad);
    g->N = N; g->C = C; g->H = H; g->W = W; g->k = k; g->sh = sh; g->sw = sw; g->pad = pad;
    g->OH = (H + 2 * pad - k) / sh + 1;
    g->OW = (W + 2 * pad - k) / sw + 1;
    XSMI_CHECK_ARG((double)N * C * H * W < 2147483648.0 && (double)N * C * g->OH * g->OW < 2147483648.0,
                   "%s: tensors above 2^31 elements are not supported", fn);
    g->dOW = xsmi::make_fastdiv(g->OW); g->dOH = xsmi::make_fastdiv(g->OH);
    g->dW = xsmi::make_fastdiv(W); g->dH = xsmi::make_fastdiv(H);
    g->dsh = xsmi::make_fastdiv(sh); g->dsw = xsmi::make_fastdiv(sw);
    return XSMI_OK;
}

bool fast_3x3s2p1(const PoolGeom &g) {
    return g.k == 3 && g.sh == 2 && g.sw == 2 && g.pad == 1 && (g.W % 4) == 0 && (g.H % 2) == 0;
}

}  // namespace

extern "C" {

int xsmi_maxpool2d_fwd(const float *x, float *y, uint8_t *idx, int N, int C, int H, int W, int k, int sh, int sw,
                       int pad) {
    XSMI_REQUIRE_INIT();
    PoolGeom g;
    int rc = check_geom("xsmi_maxpool2d_fwd", N, C, H, W, k, sh, sw, pad, &g);
    if (rc) return rc;
    XSMI_CHECK_ARG(x && y, "xsmi_maxpool2d_fwd: null tensor pointer");
    uint32_t total = (uint32_t)N * C * g.OH * g.OW;
    hipStream_t st = xsmi::stream();
    xsmi::prof_begin();
    static const int pool_rows = getenv("XSMI_POOL_ROWS") ? atoi(getenv("XSMI_POOL_ROWS")) : 1;
    if (fast_3x3s2p1(g) && pool_rows >= 1 && g.W % 8 == 0 && g.OH % pool_rows == 0) {
        const int RO = pool_rows;
        uint32_t threads = total / 4 / RO;
        xsmi::FastDiv dQ = xsmi::make_fastdiv(g.OW / 4), dG = xsmi::make_fastdiv(g.OH / RO);
        dim3 grid((threads + 255) / 256);
        if (RO == 1) hipLaunchKernelGGL(maxpool_fwd_3x3s2p1_patch<1>, grid, dim3(256), 0, st, x, y, idx, g, dQ, dG, threads);
        else if (RO == 2) hipLaunchKernelGGL(maxpool_fwd_3x3s2p1_patch<2>, grid, dim3(256), 0, st, x, y, idx, g, dQ, dG, threads);
        else if (RO == 4) hipLaunchKernelGGL(maxpool_fwd_3x3s2p1_patch<4>, grid, dim3(256), 0, st, x, y, idx, g, dQ, dG, threads);
        else return xsmi::set_error("XSMI_POOL_ROWS must be 0, 1, 2 or 4"), XSMI_ERR_INVALID;
        xsmi::prof_end();
        XSMI_LAUNCH_CHECK("maxpool_fwd_3x3s2p1_patch");
        return XSMI_OK;
    }
    if (fast_3x3s2p1(g)) {
        uint32_t pairs = total / 2;
        xsmi::FastDiv dQ = xsmi::make_fastdiv(g.OW / 2);
        hipLaunchKernelGGL(maxpool_fwd_3x3s2p1, dim3((pairs + 255) / 256), dim3(256), 0, st, x, y, idx, g, dQ, pairs);
        xsmi::prof_end();
        XSMI_LAUNCH_CHECK("maxpool_fwd_3x3s2p1");
        return XSMI_OK;
    }
    dim3 grid((total + 255) / 256);
    if (k == 2)
        hipLaunchKernelGGL(maxpool_fwd_generic<2>, grid, dim3(256), 0, st, x, y, idx, g, total);
    else if (k == 3)
        hipLaunchKernelGGL(maxpool_fwd_generic<3>, grid, dim3(256), 0, st, x, y, idx, g, total);
    else
        hipLaunchKernelGGL(maxpool_fwd_generic<0>, grid, dim3(256), 0, st, x, y, idx, g, total);
    xsmi::prof_end();
    XSMI_LAUNCH_CHECK("maxpool_fwd_generic");
    return XSMI_OK;
}

int xsmi_maxpool2d_bwd(const float *dy, const uint8_t *idx, float *dx, int N, int C, int H, int W, int k, int sh,
                       int sw, int pad, float beta) {
    XSMI_REQUIRE_INIT();
    PoolGeom g;
    int rc = check_geom("xsmi_maxpool2d_bwd", N, C, H, W, k, sh, sw, pad, &g);
    if (rc) return rc;
    XSMI_CHECK_ARG(dy && idx && dx, "xsmi_maxpool2d_bwd: null tensor pointer");
    XSMI_CHECK_ARG(beta == 0.f || beta == 1.f, "xsmi_maxpool2d_bwd: beta must be 0 or 1");
    uint32_t total = (uint32_t)N * C * H * W;
    hipStream_t st = xsmi::stream();
    int acc = beta == 1.f ? 1 : 0;
    xsmi::prof_begin();
    static const int pool_rp = getenv("XSMI_POOL_RP") ? atoi(getenv("XSMI_POOL_RP")) : 1;
    if (fast_3x3s2p1(g) && pool_rp >= 1 && W % 8 == 0 && H % (2 * pool_rp) == 0) {
        const int RP = pool_rp;
        uint32_t threads = total / 8 / (2 * RP);
        xsmi::FastDiv dQ8 = xsmi::make_fastdiv(W / 8), dG = xsmi::make_fastdiv(H / (2 * RP));
        dim3 grid((threads + 255) / 256);
        if (RP == 1) hipLaunchKernelGGL(maxpool_bwd_3x3s2p1_patch<1>, grid, dim3(256), 0, st, dy, idx, dx, g, dQ8, dG, threads, acc);
        else if (RP == 2) hipLaunchKernelGGL(maxpool_bwd_3x3s2p1_patch<2>, grid, dim3(256), 0, st, dy, idx, dx, g, dQ8, dG, threads, acc);
        else return xsmi::set_error("XSMI_POOL_RP must be 0, 1 or 2"), XSMI_ERR_INVALID;
        xsmi::prof_end();
        XSMI_LAUNCH_CHECK("maxpool_bwd_3x3s2p1_patch");
        return XSMI_OK;
    }
    if (fast_3x3s2p1(g)) {
        uint32_t quads = total / 4;
        xsmi::FastDiv dQ4 = xsmi::make_fastdiv(W / 4);
        hipLaunchKernelGGL(maxpool_bwd_3x3s2p1, dim3((quads + 255) / 256), dim3(256), 0, st, dy, idx, dx, g, dQ4, quads, acc);
        xsmi::prof_end();
        XSMI_LAUNCH_CHECK("maxpool_bwd_3x3s2p1");
        return XSMI_OK;
    }
    hipLaunchKernelGGL(maxpool_bwd_gather, dim3((total + 255) / 256), dim3(256), 0, st, dy, idx, dx, g, total, acc);
    xsmi::prof_end();
    XSMI_LAUNCH_CHECK("maxpool_bwd_gather");
    return XSMI_OK;
}

}  // extern "C"
