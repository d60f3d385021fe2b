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

namespace {

typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f2v __attribute__((ext_vector_type(2)));

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
    for (int r = 0; r < k; ++r) {                            // (a compile-time k unrolls by itself)
        int ih = ih0 + r;
        bool rowok = (unsigned)ih < (unsigned)g.H;
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
// three input rows, so a wavefront's loads are contiguous.  Column 4j-1 is one
// more dword load per row (the previous lane's cache line; the zero border at
// j == 0): taking it from the previous lane's registers instead needs a
// divergent extra load at every wavefront edge, a second memory round trip that
// the whole wave waits for (measured 4 us of 33 in the backward kernel).  All
// loads are issued before the first comparison so that their latencies overlap.  x is fetched once per window row; the row shared by
// vertically adjacent windows is re-read from cache.
__global__ void __launch_bounds__(256) maxpool_fwd_3x3s2p1(const float *__restrict__ x, float *__restrict__ y,
                                                            uint8_t *__restrict__ idx, PoolGeom g,
                                                            xsmi::FastDiv dQ, uint32_t total_pairs) {
    uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= total_pairs) return;
    const int Q = g.OW >> 1;                 // output pairs per row == float4 per input row
    uint32_t row = xsmi::fdiv(t, dQ);        // (nc, oh)
    const int j = (int)(t - row * Q);
    uint32_t nc = xsmi::fdiv(row, g.dOH);
    const int oh = (int)(row - nc * g.OH);
    const float *plane = x + (size_t)nc * g.H * g.W;

    float4 v[3];
    float lf[3];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        const int ih = 2 * oh - 1 + r;
        v[r] = make_float4(0.f, 0.f, 0.f, 0.f);   // border row
        lf[r] = 0.f;
        if ((unsigned)ih < (unsigned)g.H) {
            v[r] = *reinterpret_cast<const float4 *>(plane + (size_t)ih * g.W + 4 * j);
            if (j > 0) lf[r] = plane[(size_t)ih * g.W + 4 * j - 1];
        }
    }
    float b0 = 0.f, b1 = 0.f;
    int w0 = 0, w1 = 0;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        const float left = lf[r];                                     // 0 at the border
        // output 2j: columns 4j-1, 4j, 4j+1 ; output 2j+1: columns 4j+1, 4j+2, 4j+3
        if (r == 0 || left > b0) { b0 = left; w0 = r * 3 + 0; }
        if (v[r].x > b0) { b0 = v[r].x; w0 = r * 3 + 1; }
        if (v[r].y > b0) { b0 = v[r].y; w0 = r * 3 + 2; }
        if (r == 0 || v[r].y > b1) { b1 = v[r].y; w1 = r * 3 + 0; }
        if (v[r].z > b1) { b1 = v[r].z; w1 = r * 3 + 1; }
        if (v[r].w > b1) { b1 = v[r].w; w1 = r * 3 + 2; }
    }
    size_t o = (size_t)row * g.OW + 2 * j;
    // the outputs are not read again by this kernel: non-temporal stores (measured +4 % over plain ones; non-temporal
    // loads of x lose, its rows are shared between neighbouring windows)
    f2v yv; yv.x = b0; yv.y = b1;
    __builtin_nontemporal_store(yv, reinterpret_cast<f2v *>(y + o));
    if (idx) __builtin_nontemporal_store((unsigned short)(w0 | (w1 << 8)), reinterpret_cast<unsigned short *>(idx + o));
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

// 3x3 window, stride 2, pad 1, W % 4 == 0, H % 2 == 0: one thread produces dx
// columns 4j .. 4j+3 of the two input rows 2a and 2a+1 with one float4 store per
// row, contiguous across the wavefront.  It reads output columns 2j, 2j+1 of the
// output rows a and a+1 (dy and index) and column 2j+2 with one more dword / byte
// load (nothing at the row end; see the forward kernel for why not a shuffle).
//   even row, even column: one contributor  (window row 1, kx 1)
//   even row, odd column:  two              (kx 0 of the output column to the right, kx 2 of this one)
//   odd row,  even column: two              (window row 0 of output row a+1, window row 2 of row a)
//   odd row,  odd column:  four
// The float32 sum of two float32 values equals their float64 sum rounded to
// float32, so only the four-term cells, and every cell when the previous dx is
// one more term (ACC), go through float64.
template <bool ACC>
__global__ void __launch_bounds__(256) maxpool_bwd_3x3s2p1(const float *__restrict__ dy, const uint8_t *__restrict__ idx,
                                                            float *__restrict__ dx, PoolGeom g, xsmi::FastDiv dQ4,
                                                            xsmi::FastDiv dG, uint32_t total) {
    uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= total) return;
    const int Q4 = g.W >> 2, G = g.H >> 1;
    uint32_t rowg = xsmi::fdiv(t, dQ4);      // (nc, a)
    const int j = (int)(t - rowg * Q4);
    uint32_t nc = xsmi::fdiv(rowg, dG);
    const int a = (int)(rowg - nc * G);
    const size_t obase = (size_t)nc * g.OH * g.OW;
    float gv[2][3];
    int iv[2][3];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int oh = a + q;                 // a + 1 == OH: below the last output row
        float2 gg = make_float2(0.f, 0.f);
        int i0 = -1, i1 = -1;
        float gn = 0.f;
        int in = -1;
        const size_t ro = obase + (size_t)oh * g.OW + 2 * j;
        if (oh < g.OH) {
            gg = *reinterpret_cast<const float2 *>(dy + ro);
            uchar2 ii = *reinterpret_cast<const uchar2 *>(idx + ro);
            i0 = ii.x; i1 = ii.y;
            if (2 * j + 2 < g.OW) { gn = dy[ro + 2]; in = idx[ro + 2]; }
        }
        // x + 0 turns -0 into +0 and changes nothing else: the reference's sums start at +0
        gv[q][0] = gg.x + 0.f; gv[q][1] = gg.y + 0.f; gv[q][2] = gn + 0.f;
        iv[q][0] = i0; iv[q][1] = i1; iv[q][2] = in;
    }
    const int h = 2 * a;
    float4 *pe = reinterpret_cast<float4 *>(dx + ((size_t)nc * g.H + h) * g.W + 4 * j);
    float4 *po = reinterpret_cast<float4 *>(dx + ((size_t)nc * g.H + h + 1) * g.W + 4 * j);
    float e[4], o[4];
    auto pick = [&](int q, int m, int tap) { return iv[q][m] == tap ? gv[q][m] : 0.f; };
    if (ACC) {
        const float4 ev = *pe, ov = *po;
        const float pe4[4] = {ev.x, ev.y, ev.z, ev.w}, po4[4] = {ov.x, ov.y, ov.z, ov.w};
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            e[2 * m] = (float)((double)pick(0, m, 4) + (double)pe4[2 * m]);
            e[2 * m + 1] = (float)(((double)pick(0, m + 1, 3) + (double)pick(0, m, 5)) + (double)pe4[2 * m + 1]);
            o[2 * m] = (float)(((double)pick(1, m, 1) + (double)pick(0, m, 7)) + (double)po4[2 * m]);
            o[2 * m + 1] = (float)(((((double)pick(1, m + 1, 0) + (double)pick(1, m, 2)) + (double)pick(0, m + 1, 6)) +
                                    (double)pick(0, m, 8)) + (double)po4[2 * m + 1]);
        }
    } else {
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            e[2 * m] = pick(0, m, 4);
            e[2 * m + 1] = pick(0, m + 1, 3) + pick(0, m, 5);
            o[2 * m] = pick(1, m, 1) + pick(0, m, 7);
            o[2 * m + 1] = (float)((((double)pick(1, m + 1, 0) + (double)pick(1, m, 2)) + (double)pick(0, m + 1, 6)) +
                                   (double)pick(0, m, 8));
        }
    }
    *pe = make_float4(e[0], e[1], e[2], e[3]);
    *po = make_float4(o[0], o[1], o[2], o[3]);
}

// The same gather with eight dx columns per thread (W % 8 == 0): columns 8j .. 8j+7 of the input rows 2a and 2a+1
// from output columns 4j .. 4j+3 (one 128-bit load of dy and one 32-bit load of the indices per output row) and
// column 4j+4 (a dword and a byte): half as many memory instructions per byte as the four-column form.
template <bool ACC>
__global__ void __launch_bounds__(256) maxpool_bwd_3x3s2p1_w8(const float *__restrict__ dy, const uint8_t *__restrict__ idx,
                                                               float *__restrict__ dx, PoolGeom g, xsmi::FastDiv dQ8,
                                                               xsmi::FastDiv dG, uint32_t total) {
    uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= total) return;
    const int Q8 = g.W >> 3, G = g.H >> 1;
    uint32_t rowg = xsmi::fdiv(t, dQ8);      // (nc, a)
    const int j = (int)(t - rowg * Q8);
    uint32_t nc = xsmi::fdiv(rowg, dG);
    const int a = (int)(rowg - nc * G);
    const size_t obase = (size_t)nc * g.OH * g.OW;
    float gv[2][5];
    int iv[2][5];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int oh = a + q;                 // a + 1 == OH: below the last output row
        float4 gg = make_float4(0.f, 0.f, 0.f, 0.f);
        int i0 = -1, i1 = -1, i2 = -1, i3 = -1;
        float gn = 0.f;
        int in = -1;
        const size_t ro = obase + (size_t)oh * g.OW + 4 * j;
        if (oh < g.OH) {
            gg = *reinterpret_cast<const float4 *>(dy + ro);
            const uint32_t ii = *reinterpret_cast<const uint32_t *>(idx + ro);
            i0 = ii & 255; i1 = (ii >> 8) & 255; i2 = (ii >> 16) & 255; i3 = ii >> 24;
            if (4 * j + 4 < g.OW) { gn = dy[ro + 4]; in = idx[ro + 4]; }
        }
        // x + 0 turns -0 into +0 and changes nothing else: the reference's sums start at +0
        gv[q][0] = gg.x + 0.f; gv[q][1] = gg.y + 0.f; gv[q][2] = gg.z + 0.f; gv[q][3] = gg.w + 0.f; gv[q][4] = gn + 0.f;
        iv[q][0] = i0; iv[q][1] = i1; iv[q][2] = i2; iv[q][3] = i3; iv[q][4] = in;
    }
    const int h = 2 * a;
    float4 *pe = reinterpret_cast<float4 *>(dx + ((size_t)nc * g.H + h) * g.W + 8 * j);
    float4 *po = reinterpret_cast<float4 *>(dx + ((size_t)nc * g.H + h + 1) * g.W + 8 * j);
    float e[8], o[8];
    auto pick = [&](int q, int m, int tap) { return iv[q][m] == tap ? gv[q][m] : 0.f; };
    if (ACC) {
        const float4 ev0 = pe[0], ev1 = pe[1], ov0 = po[0], ov1 = po[1];
        const float pe8[8] = {ev0.x, ev0.y, ev0.z, ev0.w, ev1.x, ev1.y, ev1.z, ev1.w};
        const float po8[8] = {ov0.x, ov0.y, ov0.z, ov0.w, ov1.x, ov1.y, ov1.z, ov1.w};
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            e[2 * m] = (float)((double)pick(0, m, 4) + (double)pe8[2 * m]);
            e[2 * m + 1] = (float)(((double)pick(0, m + 1, 3) + (double)pick(0, m, 5)) + (double)pe8[2 * m + 1]);
            o[2 * m] = (float)(((double)pick(1, m, 1) + (double)pick(0, m, 7)) + (double)po8[2 * m]);
            o[2 * m + 1] = (float)(((((double)pick(1, m + 1, 0) + (double)pick(1, m, 2)) + (double)pick(0, m + 1, 6)) +
                                    (double)pick(0, m, 8)) + (double)po8[2 * m + 1]);
        }
    } else {
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            e[2 * m] = pick(0, m, 4);
            e[2 * m + 1] = pick(0, m + 1, 3) + pick(0, m, 5);
            o[2 * m] = pick(1, m, 1) + pick(0, m, 7);
            o[2 * m + 1] = (float)((((double)pick(1, m + 1, 0) + (double)pick(1, m, 2)) + (double)pick(0, m + 1, 6)) +
                                   (double)pick(0, m, 8));
        }
    }
    pe[0] = make_float4(e[0], e[1], e[2], e[3]);
    pe[1] = make_float4(e[4], e[5], e[6], e[7]);
    po[0] = make_float4(o[0], o[1], o[2], o[3]);
    po[1] = make_float4(o[4], o[5], o[6], o[7]);
}

// The eight-column gather with the stores laid out by the workgroup instead of the thread (beta == 0 only).  In the
// kernel above a lane's two float4 of a row sit side by side, so each store instruction of a wavefront covers every
// other 16 bytes of its lines; measured on the box with the kernel's exact loads, that pattern writes 102.8 MB in
// 32 us, stores whose lanes are contiguous in 26.6 us and the same as non-temporal stores in 18.6 us.  A workgroup
// therefore takes whole row pairs (RG = 256 / (W/8) of them: a contiguous piece of dx, since planes and row pairs
// follow each other in memory), every thread puts its four float4 into the LDS image of that piece, and the image is
// written out with lane-contiguous non-temporal float4 stores.
__global__ void __launch_bounds__(256) maxpool_bwd_3x3s2p1_lds(const float *__restrict__ dy, const uint8_t *__restrict__ idx,
                                                                float *__restrict__ dx, PoolGeom g, int RG,
                                                                uint32_t total_rowg) {
    // With OH == H / 2 the row pair (nc, a) has the same linear number as the dy row (nc, a), and it needs that row
    // and the next one: the workgroup's rows_here + 1 rows of dy and idx are one contiguous piece, fetched once.
    __shared__ f4v img[1024];
    __shared__ f4v s_dy[512];                         // (RG + 1) * W/8 float4, with RG * W/8 <= 256 and W/8 <= 256
    __shared__ uint32_t s_ix[512];
    const int Q8 = g.W >> 3, G = g.H >> 1;
    const int lt = (int)threadIdx.x;
    const int lrow = lt / Q8, j = lt - lrow * Q8;
    const uint32_t rowg0 = blockIdx.x * (uint32_t)RG;
    const uint32_t rows_here = total_rowg - rowg0 < (uint32_t)RG ? total_rowg - rowg0 : (uint32_t)RG;
    {
        const uint32_t q_total = total_rowg * (uint32_t)Q8;                  // float4 (or index words) of all of dy
        const uint32_t q0 = rowg0 * (uint32_t)Q8;
        const uint32_t want = (rows_here + 1u) * (uint32_t)Q8;
        const f4v *gsrc = reinterpret_cast<const f4v *>(dy) + q0;
        const uint32_t *isrc = reinterpret_cast<const uint32_t *>(idx) + q0;
        for (uint32_t q = (uint32_t)lt; q < want; q += 256u) {
            const bool ok = q0 + q < q_total;
            s_dy[q] = ok ? gsrc[q] : f4v{0.f, 0.f, 0.f, 0.f};
            s_ix[q] = ok ? isrc[q] : 0xffffffffu;
        }
    }
    __syncthreads();
    if ((uint32_t)lrow < rows_here) {
        const uint32_t rowg = rowg0 + (uint32_t)lrow;       // (nc, a)
        const uint32_t nc = rowg / (uint32_t)G;
        const int a = (int)(rowg - nc * (uint32_t)G);
        float gv[2][5];
        int iv[2][5];
        const float *fdy = reinterpret_cast<const float *>(s_dy);
        const uint8_t *bix = reinterpret_cast<const uint8_t *>(s_ix);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int oh = a + q;                 // a + 1 == OH: below the last output row
            f4v gg = f4v{0.f, 0.f, 0.f, 0.f};
            uint32_t ii = 0xffffffffu;
            float gn = 0.f;
            int in = -1;
            const int lq = (lrow + q) * Q8 + j;
            if (oh < g.OH) {
                gg = s_dy[lq];
                ii = s_ix[lq];
                if (j + 1 < Q8) { gn = fdy[4 * lq + 4]; in = bix[4 * lq + 4]; }
            }
            // x + 0 turns -0 into +0 and changes nothing else: the reference's sums start at +0
            gv[q][0] = gg.x + 0.f; gv[q][1] = gg.y + 0.f; gv[q][2] = gg.z + 0.f; gv[q][3] = gg.w + 0.f; gv[q][4] = gn + 0.f;
            iv[q][0] = ii & 255; iv[q][1] = (ii >> 8) & 255; iv[q][2] = (ii >> 16) & 255; iv[q][3] = ii >> 24; iv[q][4] = in;
        }
        float e[8], o[8];
        auto pick = [&](int q, int m, int tap) { return iv[q][m] == tap ? gv[q][m] : 0.f; };
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            e[2 * m] = pick(0, m, 4);
            e[2 * m + 1] = pick(0, m + 1, 3) + pick(0, m, 5);
            o[2 * m] = pick(1, m, 1) + pick(0, m, 7);
            o[2 * m + 1] = (float)((((double)pick(1, m + 1, 0) + (double)pick(1, m, 2)) + (double)pick(0, m + 1, 6)) +
                                   (double)pick(0, m, 8));
        }
        f4v *row_e = img + lrow * 4 * Q8 + 2 * j;      // row 2a of the pair, then row 2a + 1
        row_e[0] = f4v{e[0], e[1], e[2], e[3]};
        row_e[1] = f4v{e[4], e[5], e[6], e[7]};
        row_e[2 * Q8] = f4v{o[0], o[1], o[2], o[3]};
        row_e[2 * Q8 + 1] = f4v{o[4], o[5], o[6], o[7]};
    }
    __syncthreads();
    const uint32_t quads = rows_here * 4u * (uint32_t)Q8;
    f4v *out = reinterpret_cast<f4v *>(dx) + (size_t)rowg0 * 4u * (uint32_t)Q8;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t q = (uint32_t)lt + 256u * k;
        if (q < quads) __builtin_nontemporal_store(img[q], out + q);
    }
}

// The same kernel with workgroups that stay: a workgroup takes the pieces p = id, id + grid, ... and has the next piece's
// rows of dy and idx copied into a second staging area (global -> LDS directly, no registers) while it gathers and
// writes out the current one.  The one-piece kernel above spends its life waiting, first for its loads and then for
// its stores (without its stores it takes 14.7 us for the 32 MB of reads of a 32 x 64 x 112 x 112 tensor's gradient,
// without its loads 18 us for the 103 MB of writes, with both 26 us); here the only wait is "at most four
// vector-memory operations outstanding" after a piece's four stores, i.e. for the loads issued before them, never for
// the stores themselves.  Two workgroups per compute unit measured best (24.8 us; three or four, or loads two pieces
// ahead: 26 to 27 us).
__global__ void __launch_bounds__(256) maxpool_bwd_3x3s2p1_stream(const float *__restrict__ dy, const uint8_t *__restrict__ idx,
                                                                   float *__restrict__ dx, PoolGeom g, int RG,
                                                                   uint32_t total_rowg, uint32_t pieces) {
    __shared__ f4v img[1024];
    __shared__ f4v s_dy[2][512];                      // (RG + 1) * W/8 float4, with RG * W/8 <= 256 and W/8 <= 256
    __shared__ uint32_t s_ix[2][512];
    const int Q8 = g.W >> 3, G = g.H >> 1;
    const int lt = (int)threadIdx.x;
    const int lane = lt & 63, wave = __builtin_amdgcn_readfirstlane(lt >> 6);
    const int lrow = lt / Q8, j = lt - lrow * Q8;
    const uint32_t q_total = total_rowg * (uint32_t)Q8;                      // float4 (or index words) of all of dy
    auto fetch = [&](uint32_t piece, int buf) {        // the piece's rows of dy and idx as they lie, zeros past the end
        const uint32_t rowg0 = piece * (uint32_t)RG;
        const uint32_t rows_here = total_rowg - rowg0 < (uint32_t)RG ? total_rowg - rowg0 : (uint32_t)RG;
        const uint32_t q0 = rowg0 * (uint32_t)Q8;
        uint32_t want = (rows_here + 1u) * (uint32_t)Q8;
        if (want > q_total - q0) want = q_total - q0;
        const xsmi::xsmi_int32x4 rd = xsmi::make_rsrc(reinterpret_cast<const f4v *>(dy) + q0, want * 16u);
        const xsmi::xsmi_int32x4 ri = xsmi::make_rsrc(reinterpret_cast<const uint32_t *>(idx) + q0, want * 4u);
        const uint32_t ld = (uint32_t)(uintptr_t)&s_dy[buf][0], li = (uint32_t)(uintptr_t)&s_ix[buf][0];
        for (uint32_t e = (uint32_t)wave; e * 64u < want; e += 4u) {        // want <= 512: e <= 7, inside the staging area
            xsmi::load_lds_b128(rd, ld + e * 1024u, (e * 64u + (uint32_t)lane) * 16u, 0u);
            xsmi::load_lds_b32(ri, li + e * 256u, (e * 64u + (uint32_t)lane) * 4u, 0u);
        }
    };
    uint32_t piece = blockIdx.x;
    if (piece >= pieces) return;
    int cur = 0;
    fetch(piece, 0);
    xsmi::wait_vmcnt<0>();
    for (; piece < pieces; piece += gridDim.x, cur ^= 1) {
        const uint32_t rowg0 = piece * (uint32_t)RG;
        const uint32_t rows_here = total_rowg - rowg0 < (uint32_t)RG ? total_rowg - rowg0 : (uint32_t)RG;
        // this wave's loads of the piece have landed (first round: waited for above; later: at the end of the last round)
        xsmi::block_barrier();                         // ... and everybody's; the other staging area and img are free
        if (piece + gridDim.x < pieces) fetch(piece + gridDim.x, cur ^ 1);
        if ((uint32_t)lrow < rows_here) {
            const uint32_t rowg = rowg0 + (uint32_t)lrow;       // (nc, a)
            const uint32_t nc = rowg / (uint32_t)G;
            const int a = (int)(rowg - nc * (uint32_t)G);
            float gv[2][5];
            int iv[2][5];
            const float *fdy = reinterpret_cast<const float *>(s_dy[cur]);
            const uint8_t *bix = reinterpret_cast<const uint8_t *>(s_ix[cur]);
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int oh = a + q;                 // a + 1 == OH: below the last output row
                f4v gg = f4v{0.f, 0.f, 0.f, 0.f};
                uint32_t ii = 0xffffffffu;
                float gn = 0.f;
                int in = -1;
                const int lq = (lrow + q) * Q8 + j;
                if (oh < g.OH) {
                    gg = s_dy[cur][lq];
                    ii = s_ix[cur][lq];
                    if (j + 1 < Q8) { gn = fdy[4 * lq + 4]; in = bix[4 * lq + 4]; }
                }
                // x + 0 turns -0 into +0 and changes nothing else: the reference's sums start at +0
                gv[q][0] = gg.x + 0.f; gv[q][1] = gg.y + 0.f; gv[q][2] = gg.z + 0.f; gv[q][3] = gg.w + 0.f; gv[q][4] = gn + 0.f;
                iv[q][0] = ii & 255; iv[q][1] = (ii >> 8) & 255; iv[q][2] = (ii >> 16) & 255; iv[q][3] = ii >> 24; iv[q][4] = in;
            }
            float e[8], o[8];
            auto pick = [&](int q, int m, int tap) { return iv[q][m] == tap ? gv[q][m] : 0.f; };
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                e[2 * m] = pick(0, m, 4);
                e[2 * m + 1] = pick(0, m + 1, 3) + pick(0, m, 5);
                o[2 * m] = pick(1, m, 1) + pick(0, m, 7);
                o[2 * m + 1] = (float)((((double)pick(1, m + 1, 0) + (double)pick(1, m, 2)) + (double)pick(0, m + 1, 6)) +
                                       (double)pick(0, m, 8));
            }
            f4v *row_e = img + lrow * 4 * Q8 + 2 * j;      // row 2a of the pair, then row 2a + 1
            row_e[0] = f4v{e[0], e[1], e[2], e[3]};
            row_e[1] = f4v{e[4], e[5], e[6], e[7]};
            row_e[2 * Q8] = f4v{o[0], o[1], o[2], o[3]};
            row_e[2 * Q8 + 1] = f4v{o[4], o[5], o[6], o[7]};
        }
        __syncthreads();
        // Always four stores per thread (those past the piece's end fall outside the buffer and are dropped), so that
        // "four outstanding" below means exactly: the next piece's loads are done.
        const uint32_t quads = rows_here * 4u * (uint32_t)Q8;
        const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(reinterpret_cast<f4v *>(dx) + (size_t)rowg0 * 4u * (uint32_t)Q8), 0, (int)(quads * 16u), 0x00020000);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t q = (uint32_t)lt + 256u * k;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(xsmi::xsmi_uint32x4, img[q]), ro, (int)(q * 16u), 0, 2 /* nt */);
        }
        asm volatile("" ::: "memory");
        xsmi::wait_vmcnt<4>();                         // all but the four stores: the next piece's loads are done
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
    if (fast_3x3s2p1(g) && (W % 8) == 0 && (((uintptr_t)dy | (uintptr_t)dx) & 15) == 0 && ((uintptr_t)idx & 3) == 0) {
        uint32_t threads = total / 16;       // eight columns of two rows each
        xsmi::FastDiv dQ8 = xsmi::make_fastdiv(W / 8), dG = xsmi::make_fastdiv(H / 2);
        dim3 grid((threads + 255) / 256);
        if (!acc && W / 8 <= 256) {
            const int RG = 256 / (W / 8);
            const uint32_t total_rowg = (uint32_t)N * C * (H / 2);
            const uint32_t pieces = (total_rowg + RG - 1) / RG;
            const long mode = xsmi::option(xsmi::OPT_POOL_BWD);
            if (mode > 0) {                               // workgroups per compute unit of the kernel whose workgroups stay
                uint32_t grid_s = (uint32_t)xsmi::cu_count() * (uint32_t)(mode > 4 ? 4 : mode);
                if (grid_s > pieces) grid_s = pieces;
                hipLaunchKernelGGL(maxpool_bwd_3x3s2p1_stream, dim3(grid_s), dim3(256), 0, st, dy, idx, dx, g, RG, total_rowg, pieces);
                xsmi::prof_end();
                XSMI_LAUNCH_CHECK("maxpool_bwd_3x3s2p1_stream");
                return XSMI_OK;
            }
            hipLaunchKernelGGL(maxpool_bwd_3x3s2p1_lds, dim3(pieces), dim3(256), 0, st, dy, idx, dx, g, RG,
                               total_rowg);
            xsmi::prof_end();
            XSMI_LAUNCH_CHECK("maxpool_bwd_3x3s2p1_lds");
            return XSMI_OK;
        }
        if (acc) hipLaunchKernelGGL(maxpool_bwd_3x3s2p1_w8<true>, grid, dim3(256), 0, st, dy, idx, dx, g, dQ8, dG, threads);
        else hipLaunchKernelGGL(maxpool_bwd_3x3s2p1_w8<false>, grid, dim3(256), 0, st, dy, idx, dx, g, dQ8, dG, threads);
        xsmi::prof_end();
        XSMI_LAUNCH_CHECK("maxpool_bwd_3x3s2p1_w8");
        return XSMI_OK;
    }
    if (fast_3x3s2p1(g)) {
        uint32_t threads = total / 8;        // four columns of two rows each
        xsmi::FastDiv dQ4 = xsmi::make_fastdiv(W / 4), dG = xsmi::make_fastdiv(H / 2);
        dim3 grid((threads + 255) / 256);
        if (acc) hipLaunchKernelGGL(maxpool_bwd_3x3s2p1<true>, grid, dim3(256), 0, st, dy, idx, dx, g, dQ4, dG, threads);
        else hipLaunchKernelGGL(maxpool_bwd_3x3s2p1<false>, grid, dim3(256), 0, st, dy, idx, dx, g, dQ4, dG, threads);
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
