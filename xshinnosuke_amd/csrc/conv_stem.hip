// Forward convolution for layers with very few input channels (a network's first layer: 3 -> 64, 7x7, stride 2),
// fp32 MFMA.
//
// With three input channels the tap-major kernels have nothing to chunk (they reduce 32 channels per tap) and the
// table-driven gather kernel spends its time on addresses.  Here the reduction index is (filter row r, channel c,
// filter column s) with s innermost and padded to 8: on a zero-bordered copy of the input, xp[n][c][ih][iw], the
// eight values (r, c, 0..7) of an output pixel are eight CONSECUTIVE floats starting at column sw * ow.  A lane of
// v_mfma_f32_32x32x2_f32 is (pixel, half h of the reduction pair), so half h takes s = 4h .. 4h+3: one lane = one
// 16-byte run, read straight from global memory into the B registers.  No LDS staging, no offset table, no
// validity test (the border is materialised; columns s >= S meet zero filter entries and are also zeroed in the
// registers, so that a non-finite value next to a window cannot leak into it).
//
// The filter (K x R*C*8 floats, 43 KB for 64 x 7 x 3 x 8) is loaded into the LDS once per workgroup, in the order
// [r*C + c][h][row][4], so an A fragment is one conflict-free 128-bit read.  A wave owns 64 rows x 32 or 64 pixels
// (2 x 1 or 2 x 2 MFMA blocks, whichever leaves the busiest SIMD fewer whole wave tiles); the four waves of a
// workgroup share only the filter, so the main loop has no barrier at all: each wave prefetches the runs of the next
// filter row while it multiplies the current one.
// Reduction length 8 * R * C instead of S * R * C: 168 / 147, i.e. 87.5 % of the issued MFMA work is useful.
#include "xsmi_internal.h"
#include <type_traits>
#include <utility>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

template <int N>
using IC = std::integral_constant<int, N>;
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, Is...>) {
    (f(IC<Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

struct StemParams {
    const float *xp;       // zero-bordered copy [N][C][Hp][Wp]
    const float *apk;      // [row tile][r*C + c][h][64 rows][4]
    const float *bias;
    float *out;
    uint8_t *mask;
    uint32_t xp_bytes;
    int M, rows;
    int Hp, Wp, sh, sw;
    int OY, OX;
    xsmi::FastDiv dOX, dOY;
    long long os_n, os_k;
    int relu;
};

// One launch prepares both operands.
// Blocks [0, pad_blocks): xp[n][c][hp][wp] = x[n][c][hp - pad][wp - pad] inside the image, 0 elsewhere (border and
// alignment slack); four columns per thread (Wp is a multiple of 4).
// Blocks [pad_blocks, ..): apk[row tile][rc = r*C + c][h][row 64][t 4] = w[row][c][r][4h + t] (0 for 4h + t >= S and
// rows >= K); absent when the caller's filter is already packed.
__global__ void __launch_bounds__(256) stem_prepare_kernel(const float *__restrict__ x, float *__restrict__ xp, int H, int W, int pad,
                                                            int Hp, int Wp4, xsmi::FastDiv dWp4, xsmi::FastDiv dHp, uint32_t quads,
                                                            uint32_t pad_blocks, const float *__restrict__ w,
                                                            float *__restrict__ apk, int K, int C, int R, int S, int pack_total) {
    if (blockIdx.x < pad_blocks) {
        const uint32_t i = blockIdx.x * 256u + threadIdx.x;
        if (i >= quads) return;
        const uint32_t q = xsmi::fdiv(i, dWp4), wq = i - q * (uint32_t)Wp4;
        const uint32_t plane = xsmi::fdiv(q, dHp), hp = q - plane * (uint32_t)Hp;
        const int ih = (int)hp - pad, iw = 4 * (int)wq - pad;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if ((unsigned)ih < (unsigned)H) {
            const float *row = x + ((size_t)plane * H + ih) * W;
            if ((unsigned)(iw + 0) < (unsigned)W) v.x = row[iw + 0];
            if ((unsigned)(iw + 1) < (unsigned)W) v.y = row[iw + 1];
            if ((unsigned)(iw + 2) < (unsigned)W) v.z = row[iw + 2];
            if ((unsigned)(iw + 3) < (unsigned)W) v.w = row[iw + 3];
        }
        reinterpret_cast<float4 *>(xp)[i] = v;
        return;
    }
    for (int i = (blockIdx.x - pad_blocks) * 256 + threadIdx.x; i < pack_total; i += (gridDim.x - pad_blocks) * 256) {
        const int tt = i & 3, rr = (i >> 2) & 63, hh = (i >> 8) & 1;
        int rest = i >> 9;
        const int rc = rest % (R * C), rt = rest / (R * C);
        const int r = rc / C, c = rc - r * C;
        const int row = rt * 64 + rr, s = 4 * hh + tt;
        apk[i] = (row < K && s < S) ? w[(((size_t)row * C + c) * R + r) * S + s] : 0.f;
    }
}

template <int RS, int C, int NJ, int WAVES>
__global__ void __launch_bounds__(64 * WAVES) stem_fwd_f32_kernel(StemParams p) {
    constexpr int R = RS, S = RS, RC = R * C;
    extern __shared__ __attribute__((aligned(16))) float sm[];   // A [RC][2][64][4], then the bias [64]
    float *s_bias = sm + RC * 512;
    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int h = lane >> 5, l31 = lane & 31;
    const int rowtile = blockIdx.y;
    const int m0 = ((int)blockIdx.x * WAVES + wave) * (32 * NJ);

    {   // the row tile's filter block and bias into the LDS
        const float4 *src = reinterpret_cast<const float4 *>(p.apk) + (size_t)rowtile * (RC * 128);
        float4 *dst = reinterpret_cast<float4 *>(sm);
        for (int i = t; i < RC * 128; i += 64 * WAVES) dst[i] = src[i];
        if (t < 64) s_bias[t] = (p.bias && rowtile * 64 + t < p.rows) ? p.bias[rowtile * 64 + t] : 0.f;
    }
    __syncthreads();
    if (m0 >= p.M) return;                               // a wave without pixels (the filter load needed its threads)

    // this lane's pixels (one per block j): byte offset of its 16-byte run for (r, c) = (0, 0)
    uint32_t voff[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        int m = m0 + 32 * j + l31;
        if (m > p.M - 1) m = p.M - 1;                     // pixels past the end read the last pixel's data; never stored
        const uint32_t q = xsmi::fdiv((uint32_t)m, p.dOX);
        const int x = m - (int)q * p.OX;
        const uint32_t n = xsmi::fdiv(q, p.dOY);
        const int y = (int)q - (int)n * p.OY;
        voff[j] = (uint32_t)((((int)n * C * p.Hp + y * p.sh) * p.Wp + x * p.sw + 4 * h) * 4);
    }
    const char *xbase = reinterpret_cast<const char *>(p.xp);
    const uint32_t row_bytes = (uint32_t)p.Wp * 4u, plane_bytes = (uint32_t)p.Hp * row_bytes;

    // Software pipeline: while the MFMAs of one (r, c) run, the A fragments of the next (r, c) are read from the LDS
    // and the runs of the NEXT filter row are requested from memory, a whole filter row of MFMAs ahead of their use.
    // The order below is a suggestion to the compiler's scheduler; pinning it with scheduling barriers measured
    // a quarter slower than the schedule the compiler picks.
    float4 b[2][C][NJ];                                  // [buffer][channel][pixel block]: s = 4h .. 4h+3
    float4 a[2][2];                                      // [buffer][row block]
    auto load_run = [&](auto buf_, auto r_, auto c_, auto j_, auto half_) {
        constexpr int bf = decltype(buf_)::value, r = decltype(r_)::value, c = decltype(c_)::value, j = decltype(j_)::value;
        // uniform row base + this lane's 32-bit offset (every run lies inside the copy, see stem_Wp)
        const char *rowp = xbase + (size_t)c * plane_bytes + (size_t)r * row_bytes;
        const float2 v = *reinterpret_cast<const float2 *>(rowp + voff[j] + 8 * decltype(half_)::value);
        if constexpr (decltype(half_)::value == 0) { b[bf][c][j].x = v.x; b[bf][c][j].y = v.y; }
        else { b[bf][c][j].z = v.x; b[bf][c][j].w = v.y; }
    };
    // columns s = 4h + t beyond the filter are zero in A; zero them in B as well (0 * inf would be NaN)
    auto clip = [&](float4 &v) {
        if (3 >= S) v.w = 0.f; else if (7 >= S && h) v.w = 0.f;
        if (2 >= S) v.z = 0.f; else if (6 >= S && h) v.z = 0.f;
        if (1 >= S) v.y = 0.f; else if (5 >= S && h) v.y = 0.f;
        if (4 >= S && h) v.x = 0.f;
    };

    floatx16 acc[2][NJ];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    const float4 *a_rd = reinterpret_cast<const float4 *>(sm) + h * 64 + l31;

    // prologue: the runs of filter row 0 and the A fragments of (0, 0)
    static_for<C>([&](auto c_) {
        static_for<NJ>([&](auto j_) { load_run(IC<0>{}, IC<0>{}, c_, j_, IC<0>{}); load_run(IC<0>{}, IC<0>{}, c_, j_, IC<1>{}); });
    });
    a[0][0] = a_rd[0];
    a[0][1] = a_rd[32];
    static_for<R>([&](auto r_) {
        constexpr int r = decltype(r_)::value;
        constexpr int bf = r & 1;
        static_for<C>([&](auto c_) { static_for<NJ>([&](auto j_) { clip(b[bf][decltype(c_)::value][decltype(j_)::value]); }); });
        static_for<C>([&](auto c_) {
            constexpr int c = decltype(c_)::value;
            constexpr int rc = r * C + c, ab = rc & 1;
            constexpr bool more = rc + 1 < RC;
            static_for<8 * NJ>([&](auto k_) {
                constexpr int k = decltype(k_)::value;
                constexpr int tt = k / (2 * NJ), i = (k / NJ) & 1, j = k % NJ;
                const float av = tt == 0 ? a[ab][i].x : tt == 1 ? a[ab][i].y : tt == 2 ? a[ab][i].z : a[ab][i].w;
                const float bv = tt == 0 ? b[bf][c][j].x : tt == 1 ? b[bf][c][j].y : tt == 2 ? b[bf][c][j].z : b[bf][c][j].w;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][j], 0, 0, 0);
                if constexpr (more && k < 2) a[ab ^ 1][k] = a_rd[(rc + 1) * 128 + 32 * k];
                // the next filter row's runs of this channel: 2 NJ loads in the slots after the A reads
                if constexpr (r + 1 < R && k >= 2 && k < 2 + 2 * NJ) {
                    constexpr int q = (k - 2);             // (pixel block, half)
                    load_run(IC<bf ^ 1>{}, IC<r + 1>{}, IC<c>{}, IC<(q >> 1)>{}, IC<(q & 1)>{});
                }
            });
        });
    });

    // accumulator register v of lane l in block (i, j): row 32 i + 8 (v / 4) + 4 (l / 32) + v % 4, pixel 32 j + l % 32
    const int rbase = rowtile * 64 + 4 * h;
    const bool all_rows = rowtile * 64 + 64 <= p.rows;   // uniform: no per-row guard needed
    // MODE 0: bias only; 1: bias + relu; 2: bias + relu + sign mask
    auto emit = [&](auto mode_, auto guard_) {
        constexpr int MODE = decltype(mode_)::value;
        constexpr bool GUARD = decltype(guard_)::value;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int m = m0 + 32 * j + l31;
            if (m >= p.M) continue;
            const uint32_t q = xsmi::fdiv((uint32_t)m, p.dOX);
            const int x = m - (int)q * p.OX;
            const uint32_t n = xsmi::fdiv(q, p.dOY);
            const int y = (int)q - (int)n * p.OY;
            // the output holds fewer than 2^31 elements (checked on the host): 32-bit lane offsets from uniform row bases
            const uint32_t lane_off = n * (uint32_t)p.os_n + (uint32_t)(y * p.OX + x) + (uint32_t)(4 * h) * (uint32_t)p.os_k;
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float4 bias4 = *reinterpret_cast<const float4 *>(&s_bias[4 * h + 32 * i + 8 * g]);
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int ro = 32 * i + 8 * g + t;
                        if (GUARD && rbase + ro >= p.rows) continue;
                        const size_t row_off = (size_t)(rowtile * 64 + ro) * (size_t)p.os_k;   // uniform
                        float val = acc[i][j][4 * g + t] + (t == 0 ? bias4.x : t == 1 ? bias4.y : t == 2 ? bias4.z : bias4.w);
                        if constexpr (MODE == 2) (p.mask + row_off)[lane_off] = val < 0.f ? 1 : 0;
                        if constexpr (MODE >= 1) val = val > 0.f ? val : 0.f;
                        (p.out + row_off)[lane_off] = val;
                    }
                }
        }
    };
    auto emit_mode = [&](auto guard_) {
        if (!p.relu) emit(IC<0>{}, guard_);
        else if (!p.mask) emit(IC<1>{}, guard_);
        else emit(IC<2>{}, guard_);
    };
    if (all_rows) emit_mode(std::false_type{});
    else emit_mode(std::true_type{});
}


// ---- weight gradient of the same layers --------------------------------------------------------------------------
// dw[k][j] = sum over pixels of dy[n][k][y][x] * xp[n][c][sh y + r][2 x + s], j = (c R + r) S + s, on the zero-bordered
// copy xp.  MFMA rows are filters (64 per workgroup row tile), columns the filter positions j (JB blocks of 32), the
// reduction runs over pixels.  Eight consecutive pixels of an output row are one unit: step t = 0..3 pairs pixel
// 8g + t (lane half 0) with pixel 8g + 4 + t (half 1), so a lane's four A values are one aligned float4 of dy and its
// four B values are xp[base + 2t]: both operands go straight from memory to registers (B as gathers of single floats
// that hit the L1: the S columns of a filter row read the same 24 floats), nothing is staged, and the waves of a
// workgroup never synchronise until the end.  Each wave takes an equal run of units; the four waves' accumulators
// are added in wave order through the LDS and the workgroup writes one partial [64][32 JB]; a second kernel adds
// the partials in float64 in ascending order.
struct StemWgradParams {
    const float *dy;       // [N][K][OH][OW]
    const float *xp;       // [N][C][Hp][Wp]
    float *part;           // [workgroups.x][K][32 JB]
    float *dbpart;         // [workgroups.x][K] or nullptr
    int K, C, R, S, J, Hp, Wp, OH, OW, sh;
    uint32_t units;        // N * OH * (OW / 8)
    xsmi::FastDiv dG8, dOH, dS, dR;
};

template <int JB>
__global__ void __launch_bounds__(256, 1) stem_wgrad_f32_kernel(StemWgradParams p) {
    extern __shared__ __attribute__((aligned(16))) float red[];       // [64][32 JB] (+ [4][64] for the bias sums)
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int kk = lane >> 5, l31 = lane & 31;
    const int rowtile = blockIdx.y;
    const int G8 = p.OW >> 3;

    constexpr int LDJ = 32 * JB;
    // this lane's column of each block: element offset of (c, r, s) inside an image of the copy
    uint32_t coloff[JB];
#pragma unroll
    for (int jb = 0; jb < JB; ++jb) {
        int j = 32 * jb + l31;
        if (j > p.J - 1) j = p.J - 1;                       // columns past the filter repeat the last one; never stored
        const uint32_t rc = xsmi::fdiv((uint32_t)j, p.dS), s_ = (uint32_t)j - rc * (uint32_t)p.S;
        const uint32_t c = xsmi::fdiv(rc, p.dR), r = rc - c * (uint32_t)p.R;
        coloff[jb] = ((c * (uint32_t)p.Hp + r) * (uint32_t)p.Wp + s_ + 8u * (uint32_t)kk);
    }
    const uint32_t nw = gridDim.x * 4u, wv = blockIdx.x * 4u + (uint32_t)wave;
    const uint32_t u0 = (uint32_t)(((uint64_t)wv * p.units) / nw), u1 = (uint32_t)(((uint64_t)(wv + 1) * p.units) / nw);
    const size_t img_in = (size_t)p.C * p.Hp * p.Wp, plane_out = (size_t)p.OH * p.OW;
    const float *dy_row = p.dy + ((size_t)rowtile * 64 + l31) * plane_out + 4 * kk;   // + n K plane + y OW + 8 g

    floatx16 acc[2][JB];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int jb = 0; jb < JB; ++jb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][jb][v] = 0.f;
    float dbs[2] = {0.f, 0.f};

    // Two register buffers: a unit's operands are requested while the previous unit multiplies (a third buffer,
    // i.e. requests two units ahead, measured slower: the loop is bound by the gathers' address work, not by latency).
    float4 a[2][2];
    float b[2][JB][4];
    auto load_unit = [&](int buf, uint32_t u) {
        const uint32_t q = xsmi::fdiv(u, p.dG8), g = u - q * (uint32_t)G8;
        const uint32_t n = xsmi::fdiv(q, p.dOH), y = q - n * (uint32_t)p.OH;
        const float *ap = dy_row + (size_t)n * p.K * plane_out + (size_t)y * p.OW + 8 * g;
        a[buf][0] = *reinterpret_cast<const float4 *>(ap);
        a[buf][1] = *reinterpret_cast<const float4 *>(ap + 32 * plane_out);
        const float *bp = p.xp + (size_t)n * img_in + (size_t)(y * (uint32_t)p.sh) * p.Wp + 16 * g;
#pragma unroll
        for (int jb = 0; jb < JB; ++jb)
#pragma unroll
            for (int e = 0; e < 4; ++e) b[buf][jb][e] = bp[coloff[jb] + 2 * e];
    };
    auto multiply = [&](int buf) {
        dbs[0] += (a[buf][0].x + a[buf][0].y) + (a[buf][0].z + a[buf][0].w);
        dbs[1] += (a[buf][1].x + a[buf][1].y) + (a[buf][1].z + a[buf][1].w);
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const float av = e == 0 ? a[buf][i].x : e == 1 ? a[buf][i].y : e == 2 ? a[buf][i].z : a[buf][i].w;
#pragma unroll
                for (int jb = 0; jb < JB; ++jb)
                    acc[i][jb] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b[buf][jb][e], acc[i][jb], 0, 0, 0);
            }
    };
    if (u0 < u1) {
        load_unit(0, u0);
        uint32_t u = u0;
        for (; u + 2 < u1; u += 2) {                        // two units per trip: the buffers alternate statically
            load_unit(1, u + 1);
            multiply(0);
            load_unit(0, u + 2);
            multiply(1);
        }
        if (u + 1 < u1) {
            load_unit(1, u + 1);
            multiply(0);
            multiply(1);
        } else {
            multiply(0);
        }
    }

    // the four waves' accumulators, added in wave order: register v of lane l in block (i, jb) is
    // row 32 i + 8 (v / 4) + 4 (l / 32) + v % 4, column 32 jb + l % 32
    float *dbred = red + 64 * LDJ;
    for (int w = 0; w < 4; ++w) {
        if (wave == w) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int jb = 0; jb < JB; ++jb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int idx = (32 * i + 8 * (v >> 2) + 4 * kk + (v & 3)) * LDJ + 32 * jb + l31;
                        red[idx] = w == 0 ? acc[i][jb][v] : red[idx] + acc[i][jb][v];
                    }
            // bias sums: the two lane halves hold different pixels of the same filter row
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const float both = dbs[i] + __shfl_xor(dbs[i], 32);
                if (kk == 0) dbred[w * 64 + 32 * i + l31] = both;
            }
        }
        __syncthreads();
    }
    float *dst = p.part + ((size_t)blockIdx.x * p.K + (size_t)rowtile * 64) * LDJ;
    for (int i = t; i < 64 * LDJ; i += 256) dst[i] = red[i];
    if (p.dbpart && t < 64)
        p.dbpart[(size_t)blockIdx.x * p.K + rowtile * 64 + t] = ((dbred[t] + dbred[64 + t]) + dbred[128 + t]) + dbred[192 + t];
}

// dw[k][j] = (accumulate ? dw : 0) + sum over the workgroups' partials, db likewise: 16 threads per output, each adds
// every 16th partial in ascending order in float64, then the 16 sums are added in a fixed order.
__global__ void __launch_bounds__(256) stem_wgrad_reduce_kernel(const float *__restrict__ part, float *__restrict__ dw,
                                                                 const float *__restrict__ dbpart, float *__restrict__ db, int K,
                                                                 int J, int LDJ, int splits, int accumulate) {
    __shared__ double sm[16][17];
    const int col = threadIdx.x & 15, grp = threadIdx.x >> 4;
    const int o = blockIdx.x * 16 + col;                    // output index: [0, K J) weights, then K biases
    const int nw = K * J;
    const float *src = nullptr;
    float *dst = nullptr;
    size_t stride = 0;
    if (o < nw) {
        const int k = o / J, j = o - k * J;
        src = part + (size_t)k * LDJ + j; stride = (size_t)K * LDJ; dst = dw + o;
    } else if (db && o < nw + K) {
        src = dbpart + (o - nw); stride = (size_t)K; dst = db + (o - nw);
    }
    double s = 0.0;
    if (src) {
        int sp = grp;
        for (; sp + 48 < splits; sp += 64) {
            const float v0 = src[(size_t)sp * stride], v1 = src[(size_t)(sp + 16) * stride];
            const float v2 = src[(size_t)(sp + 32) * stride], v3 = src[(size_t)(sp + 48) * stride];
            s += (double)v0; s += (double)v1; s += (double)v2; s += (double)v3;
        }
        for (; sp < splits; sp += 16) s += (double)src[(size_t)sp * stride];
    }
    sm[grp][col] = s;
    __syncthreads();
    if (grp == 0 && dst) {
        double tot = 0.0;
#pragma unroll
        for (int g = 0; g < 16; ++g) tot += sm[g][col];
        if (accumulate) tot += (double)*dst;
        *dst = (float)tot;
    }
}

int stem_Wp(int W, int S, int sw, int pad, int OW) {
    int need = sw * OW + 8;                              // the last pixel's run of eight; 24 floats from the last unit of eight pixels
    int wp = W + 2 * pad > need ? W + 2 * pad : need;
    return (wp + 3) & ~3;                                // runs start on 8-byte boundaries; the copy writes 16 bytes per thread
}

// 64 pixels per wave unless 32 leave the busiest SIMD less to do (every SIMD multiplies whole wave tiles)
template <int RS, int C>
void stem_launch(hipStream_t st, int rowtiles, size_t lds, const StemParams &p) {
    const long long simds = 4LL * xsmi::cu_count();
    const long long w64 = (long long)xsmi::ceil_div(p.M, 64) * rowtiles, w32 = (long long)xsmi::ceil_div(p.M, 32) * rowtiles;
    const long long cost64 = 2 * ((w64 + simds - 1) / simds), cost32 = (w32 + simds - 1) / simds;
    if (cost32 < cost64) {
        const dim3 grid((unsigned)xsmi::ceil_div(p.M, 128), (unsigned)rowtiles);
        hipLaunchKernelGGL((stem_fwd_f32_kernel<RS, C, 1, 4>), grid, dim3(256), lds, st, p);
    } else {
        const dim3 grid((unsigned)xsmi::ceil_div(p.M, 256), (unsigned)rowtiles);
        hipLaunchKernelGGL((stem_fwd_f32_kernel<RS, C, 2, 4>), grid, dim3(256), lds, st, p);
    }
}

}  // namespace

namespace xsmi {

// square filters of 3, 5 or 7 on 1 or 3 channels, horizontal stride 2 (runs start on 8-byte boundaries)
bool stem_fwd_ok(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad) {
    if (!(C == 1 || C == 3) || R != S || !(R == 3 || R == 5 || R == 7) || sw != 2 || sh < 1) return false;
    const int OW = (W + 2 * pad - S) / sw + 1;
    const size_t xp = (size_t)N * C * (H + 2 * pad) * stem_Wp(W, S, sw, pad, OW) * 4;
    const int OH = (H + 2 * pad - R) / sh + 1;
    const size_t out_elems = (size_t)N * K * OH * OW;     // the kernel forms 32-bit element offsets into the output
    return xp < ((size_t)1 << 31) && out_elems < ((size_t)1 << 31) && K >= 32;
}

size_t stem_fwd_ws_bytes(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad) {
    const int OW = (W + 2 * pad - S) / sw + 1;
    const size_t apk = align_up((size_t)ceil_div(K, 64) * R * C * 512 * sizeof(float), 256);
    const size_t xp = align_up((size_t)N * C * (H + 2 * pad) * stem_Wp(W, S, sw, pad, OW) * sizeof(float), 256);
    return apk + xp;
}

int stem_conv_fwd(const float *x, const float *w, const float *bias, float *y, uint8_t *mask, int N, int C, int H, int W,
                  int K, int R, int S, int sh, int sw, int pad, int OH, int OW, int relu, int opts, void *workspace) {
    hipStream_t st = stream();
    const int rowtiles = ceil_div(K, 64);
    const int Hp = H + 2 * pad, Wp = stem_Wp(W, S, sw, pad, OW);
    const size_t apk_bytes = align_up((size_t)rowtiles * R * C * 512 * sizeof(float), 256);
    float *apk = (float *)workspace;
    float *xp = (float *)((char *)workspace + apk_bytes);
    prof_begin();
    const uint32_t total = (uint32_t)((size_t)N * C * Hp * Wp), quads = total / 4;
    const uint32_t pad_blocks = (quads + 255) / 256;
    const int pack_total = (opts & 2) ? 0 : rowtiles * R * C * 512;
    const uint32_t pack_blocks = (uint32_t)ceil_div(pack_total, 256);
    hipLaunchKernelGGL(stem_prepare_kernel, dim3(pad_blocks + pack_blocks), dim3(256), 0, st, x, xp, H, W, pad, Hp, Wp / 4,
                       make_fastdiv(Wp / 4), make_fastdiv(Hp), quads, pad_blocks, w, apk, K, C, R, S, pack_total);
    XSMI_LAUNCH_CHECK("stem_prepare_kernel");
    StemParams p;
    p.xp = xp; p.apk = apk; p.bias = bias; p.out = y; p.mask = relu ? mask : nullptr;
    p.xp_bytes = total * 4u;
    p.M = N * OH * OW; p.rows = K;
    p.Hp = Hp; p.Wp = Wp; p.sh = sh; p.sw = sw;
    p.OY = OH; p.OX = OW; p.dOX = make_fastdiv(OW); p.dOY = make_fastdiv(OH);
    p.os_n = (long long)K * OH * OW; p.os_k = (long long)OH * OW;
    p.relu = relu;
    const size_t lds = ((size_t)R * C * 512 + 64) * sizeof(float);
    if (C == 3) {
        if (R == 7) stem_launch<7, 3>(st, rowtiles, lds, p);
        else if (R == 5) stem_launch<5, 3>(st, rowtiles, lds, p);
        else stem_launch<3, 3>(st, rowtiles, lds, p);
    } else {
        if (R == 7) stem_launch<7, 1>(st, rowtiles, lds, p);
        else if (R == 5) stem_launch<5, 1>(st, rowtiles, lds, p);
        else stem_launch<3, 1>(st, rowtiles, lds, p);
    }
    prof_end();
    XSMI_LAUNCH_CHECK("stem_fwd_f32_kernel");
    return XSMI_OK;
}


// ---- weight gradient ----
static int stem_wgrad_groups() { return cu_count(); }        // workgroups per row tile = partial sums to reduce

bool stem_wgrad_ok(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad) {
    if (C > 4 || C * R * S > 160 || R > 8 || S > 8 || sw != 2 || sh < 1 || K % 64 != 0) return false;
    const int OW = (W + 2 * pad - S) / sw + 1;
    if (OW % 8 != 0) return false;
    const size_t xp = (size_t)N * C * (H + 2 * pad) * stem_Wp(W, S, sw, pad, OW) * 4;
    return xp < ((size_t)1 << 31);
}

size_t stem_wgrad_ws_bytes(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad) {
    const int OW = (W + 2 * pad - S) / sw + 1;
    const int JB = ceil_div(C * R * S, 32);
    const size_t xp = align_up((size_t)N * C * (H + 2 * pad) * stem_Wp(W, S, sw, pad, OW) * sizeof(float), 256);
    const size_t part = align_up((size_t)stem_wgrad_groups() * K * 32 * JB * sizeof(float), 256);
    const size_t dbp = align_up((size_t)stem_wgrad_groups() * K * sizeof(float), 256);
    return xp + part + dbp;
}

template <int JB>
static void stem_wgrad_launch(hipStream_t st, dim3 grid, const StemWgradParams &p) {
    const size_t lds = ((size_t)64 * 32 * JB + 256) * sizeof(float);
    hipLaunchKernelGGL((stem_wgrad_f32_kernel<JB>), grid, dim3(256), lds, st, p);
}

int stem_conv_bwd_weight(const float *dy, const float *x, float *dw, float *db, int N, int C, int H, int W, int K, int R, int S,
                         int sh, int sw, int pad, int OH, int OW, int accumulate, void *workspace) {
    hipStream_t st = stream();
    const int Hp = H + 2 * pad, Wp = stem_Wp(W, S, sw, pad, OW);
    const int J = C * R * S, JB = ceil_div(J, 32);
    const int groups = stem_wgrad_groups();
    const size_t xp_bytes = align_up((size_t)N * C * Hp * Wp * sizeof(float), 256);
    const size_t part_bytes = align_up((size_t)groups * K * 32 * JB * sizeof(float), 256);
    float *xp = (float *)workspace;
    float *part = (float *)((char *)workspace + xp_bytes);
    float *dbpart = (float *)((char *)workspace + xp_bytes + part_bytes);
    const uint32_t quads = (uint32_t)((size_t)N * C * Hp * Wp / 4);
    const uint32_t pad_blocks = (quads + 255) / 256;
    hipLaunchKernelGGL(stem_prepare_kernel, dim3(pad_blocks), dim3(256), 0, st, x, xp, H, W, pad, Hp, Wp / 4, make_fastdiv(Wp / 4),
                       make_fastdiv(Hp), quads, pad_blocks, (const float *)nullptr, (float *)nullptr, K, C, R, S, 0);
    XSMI_LAUNCH_CHECK("stem_prepare_kernel");
    StemWgradParams p;
    p.dy = dy; p.xp = xp; p.part = part; p.dbpart = db ? dbpart : nullptr;
    p.K = K; p.C = C; p.R = R; p.S = S; p.J = J; p.Hp = Hp; p.Wp = Wp; p.OH = OH; p.OW = OW; p.sh = sh;
    p.units = (uint32_t)((size_t)N * OH * (OW / 8));
    p.dG8 = make_fastdiv(OW / 8); p.dOH = make_fastdiv(OH); p.dS = make_fastdiv(S); p.dR = make_fastdiv(R);
    const dim3 grid((unsigned)groups, (unsigned)(K / 64));
    prof_begin();
    switch (JB) {
        case 1: stem_wgrad_launch<1>(st, grid, p); break;
        case 2: stem_wgrad_launch<2>(st, grid, p); break;
        case 3: stem_wgrad_launch<3>(st, grid, p); break;
        case 4: stem_wgrad_launch<4>(st, grid, p); break;
        default: stem_wgrad_launch<5>(st, grid, p); break;
    }
    prof_end();
    XSMI_LAUNCH_CHECK("stem_wgrad_f32_kernel");
    const int outputs = K * J + (db ? K : 0);
    hipLaunchKernelGGL(stem_wgrad_reduce_kernel, dim3((unsigned)ceil_div(outputs, 16)), dim3(256), 0, st, part, dw,
                       db ? dbpart : nullptr, db, K, J, 32 * JB, groups, accumulate);
    XSMI_LAUNCH_CHECK("stem_wgrad_reduce_kernel");
    return XSMI_OK;
}

}  // namespace xsmi
