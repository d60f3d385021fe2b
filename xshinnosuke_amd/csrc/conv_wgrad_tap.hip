// Tap-major backward-weight on fp32 MFMA for layers with C % 64 == 0 and K % 64 == 0.
// When OH*OW is not a multiple of 4 (7x7 images) dy is first copied into the workspace with
// every plane padded by zeros to the next multiple of 4, which restores the 16-byte alignment
// and the whole-group validity that the 128-bit dy loads rely on.
//
// For one filter tap (r, s) the weight gradient is a plain GEMM over pixels,
//
//     dw[k][c][r][s] = sum_m dy[n, k, m] * x[n, c, (oh*sh + r - pad), (ow*sw + s - pad)]      m = (n, oh, ow)
//
// whose reduction index m is contiguous in memory for dy and (per output row) for
// x.  A workgroup owns one (tap, 64 filters, 64 channels) tile and one contiguous
// range of 32-pixel chunks; it writes its 64x64 partial to the workspace and a
// second kernel adds the ranges in a fixed order in float64 (no float atomics).
// Chunks never straddle two images.
//
// Data path: global -> LDS directly, two stages.
//   A = dy  [64 filters][32 pixels]  128-bit loads, 8 filter rows per wave-load
//   B = x   [64 channels][32 pixels] dword loads (the shifted, possibly strided
//           and border-clipped pixel needs a per-lane address), 2 channels per
//           wave-load; invalid lanes use an offset beyond the buffer, which the
//           range check turns into 0.0
// Both tiles keep the pixel axis innermost, which is what the MFMA operand layout
// wants (lane = filter/channel, registers = consecutive pixels): each lane reads
// its 16 pixels with four 128-bit LDS reads.  Rows are 128 bytes, so the 16-byte
// groups of a row are stored XOR-swizzled by (row & 7) to spread a wavefront's
// reads over all banks; since LDS-direct loads fix the LDS position of every
// lane, the swizzle is applied to the global address each lane fetches instead.
#include "xsmi_internal.h"
#include <type_traits>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TK = 64, TC = 64, MC = 32;
constexpr int STAGE_FLOATS = 4096;      // A 2048 + B 2048
constexpr int STAGES = 2;
constexpr int LOADS = 10;               // per wave and chunk: 2 dwordx4 (A) + 8 dword (B)
constexpr int TARGET_BLOCKS = 1024;

struct WgradTapParams {
    const float *dy;
    const float *x;
    float *part;        // [split][tap][K][C]
    float *dbpart;      // [split][K] or nullptr
    uint32_t x_bytes, dy_bytes;
    int N, C, K, H, W, OH, OW, OHW, R, S, sh, sw, pad;
    int OHWa;           // plane length of the dy operand as stored (OHW rounded up to a multiple of 4)
    int cpi;            // chunks per image
    int flat;           // the dy operand is a [K][N*OHW] copy and chunks run over the pixels of the whole batch
    int Mtot;           // flat: N*OHW
    xsmi::FastDiv dOHW; // flat: pixel index -> image
    int total_chunks, cps, ctiles;
    uint32_t xplane_bytes, yplane_bytes;
    xsmi::FastDiv dOW, dCT, dS;
};

// DIRECT: chunks run over the pixels of the whole batch (p.flat) and dy is read where it lies, [N][K][OHW] with OHW a
// multiple of 4 and at least MC: a lane's 16-byte piece of a filter's row never straddles two images, and its address
// is walked from chunk to chunk (MC pixels on, with a jump to the same filter's plane in the next image when the
// piece leaves its image).
template <bool DIRECT>
__global__ void __launch_bounds__(256, 4) wgrad_tap_f32_kernel(WgradTapParams p) {
    __shared__ __attribute__((aligned(16))) float smem[STAGES][STAGE_FLOATS];
    constexpr int D = STAGES - 1;

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int h = lane >> 5, l31 = lane & 31;
    const int wr = wave >> 1, wc = wave & 1;

    // logical block = (split, k tile, tap, c tile) with the tap fastest: the R*S blocks that read the
    // same dy and x pixels are neighbours in logical order and run on one XCD
    const uint32_t nbx = gridDim.x, nby = gridDim.y;
    const uint32_t logical = xsmi::xcd_contiguous_id(blockIdx.x + nbx * (blockIdx.y + nby * blockIdx.z), nbx * nby * gridDim.z);
    const uint32_t lz = logical / (nbx * nby), lxy = logical - lz * (nbx * nby);
    const uint32_t ly = lxy / nbx, lx = lxy - ly * nbx;
    const int tapidx = (int)xsmi::fdiv(lx, p.dCT);
    const int ctile = (int)lx - tapidx * p.ctiles;
    const int tr = (int)xsmi::fdiv((uint32_t)tapidx, p.dS);
    const int ts = tapidx - tr * p.S;
    const int c0 = ctile * TC, k0 = (int)ly * TK;
    const int split = (int)lz;
    const int chunk_begin = split * p.cps;
    int nchunks = p.total_chunks - chunk_begin;
    if (nchunks > p.cps) nchunks = p.cps;
    if (nchunks < 0) nchunks = 0;

    const xsmi::xsmi_int32x4 rx = xsmi::make_rsrc(p.x, p.x_bytes);
    const xsmi::xsmi_int32x4 ry = xsmi::make_rsrc(p.dy, p.dy_bytes);
    const uint32_t lds0 = (uint32_t)(uintptr_t)&smem[0][0];

    // ---- A load role: wave-load j (j = wave, wave + 4) fills rows 8j..8j+7; lane -> (row, swizzled group) ----
    const int a_row0 = 8 * wave + (lane >> 3), a_row1 = a_row0 + 32;
    const int a_q = (lane & 7) ^ (a_row0 & 7);                      // same for both rows (32 = 0 mod 8)
    const uint32_t a_v0 = (uint32_t)a_row0 * p.yplane_bytes + (uint32_t)a_q * 16u;
    const uint32_t a_v1 = (uint32_t)a_row1 * p.yplane_bytes + (uint32_t)a_q * 16u;
    // ---- B load role: wave-load j = wave + 4e fills channels 2j, 2j+1; the pixel a lane fetches is the same for all e ----
    const int b_chl = 2 * wave + (lane >> 5);                       // channel of wave-load e: b_chl + 8e
    const int b_ms = lane & 31;
    const int b_m = ((((b_ms >> 2) ^ (b_chl & 7)) << 2) | (b_ms & 3));   // pixel of the chunk this lane fetches

    // ---- issue state ----
    int in_img = 0, ci = 0;                                          // image and chunk-in-image of the next chunk to load
    {
        in_img = chunk_begin / p.cpi;
        ci = chunk_begin - in_img * p.cpi;
    }
    uint32_t ld_vb = 0, ld_sa = 0, ld_sb = 0;
    int ld_ml0 = 0;
    // DIRECT: pixel-in-image, byte offset (row a_row0) and pixels left in the batch of this lane's piece of the next chunk
    int d_pl = 0, d_addr = 0, d_left = 0;
    if constexpr (DIRECT) {
        const int m = chunk_begin * MC + 4 * a_q;
        const int img = (int)xsmi::fdiv((uint32_t)m, p.dOHW);
        d_pl = m - img * p.OHW;
        d_addr = (((img * p.K + k0 + a_row0) * p.OHW) + d_pl) * 4;
        d_left = p.Mtot - m;
    }
    int ld_tail = 0;                                                 // the chunk to load runs past the end of its image
    // The input position of this lane's pixel is walked from chunk to chunk instead of being formed by two divisions per
    // chunk (every vector instruction beside the MFMAs takes matrix-pipe time): the pixel advances by MC = q32 rows and
    // r32 columns of the output, with at most one carry.  A pixel contributes when its output row lies in
    // [ylo, ylo + ycnt) (input row inside the image, and the row exists at all: the last chunk of an image runs past its
    // end) and its column in [xlo, xlo + xcnt).  Not used when the chunks run over the whole batch (p.flat).
    const int q32 = MC / p.OW, r32 = MC - q32 * p.OW;
    const int ylo = p.pad > tr ? (p.pad - tr + p.sh - 1) / p.sh : 0;
    int yhi = (p.H - 1 + p.pad - tr) / p.sh;
    if (yhi > p.OH - 1) yhi = p.OH - 1;
    const uint32_t ycnt = yhi >= ylo ? (uint32_t)(yhi - ylo + 1) : 0u;
    const int xlo = p.pad > ts ? (p.pad - ts + p.sw - 1) / p.sw : 0;
    int xhi = (p.W - 1 + p.pad - ts) / p.sw;
    if (xhi > p.OW - 1) xhi = p.OW - 1;
    const uint32_t xcnt = xhi >= xlo ? (uint32_t)(xhi - xlo + 1) : 0u;
    const int row_bytes = p.sh * p.W * 4, col_bytes = p.sw * 4;
    const int step_bytes = q32 * row_bytes + r32 * col_bytes;        // no carry
    const int carry_bytes = step_bytes + row_bytes - p.OW * col_bytes;
    const int lane_bytes = ((tr - p.pad) * p.W + (ts - p.pad)) * 4 + b_chl * (int)p.xplane_bytes;
    int w_oh, w_ow, w_addr;                                          // of the next chunk to load
    {
        const int ml = ci * MC + b_m;
        w_oh = ml / p.OW;
        w_ow = ml - w_oh * p.OW;
        w_addr = w_oh * row_bytes + w_ow * col_bytes + lane_bytes;
    }
    auto issue_prep = [&]() {
        const int ml0 = ci * MC;
        ld_sa = (uint32_t)((in_img * p.K + k0) * p.OHWa + ml0) * 4u;
        ld_sb = (uint32_t)(in_img * p.C + c0) * p.xplane_bytes;
        // A: groups of 4 pixels are inside the (padded) plane or not as a whole; only an image's last chunk can hold any outside
        ld_ml0 = ml0;
        ld_tail = ml0 + MC > p.OHWa ? 1 : 0;
        if (p.flat) {
            // B: the shifted input position of this lane's pixel, chunks running over the pixels of the whole batch
            int ml = ml0 + b_m;
            const bool inside = ml < p.Mtot;
            const int img = (int)xsmi::fdiv((uint32_t)ml, p.dOHW);
            ml -= img * p.OHW;
            const int oh = (int)xsmi::fdiv((uint32_t)ml, p.dOW);
            const int ow = ml - oh * p.OW;
            const int ih = oh * p.sh + tr - p.pad, iw = ow * p.sw + ts - p.pad;
            const bool b_ok = inside && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
            ld_vb = b_ok ? (uint32_t)((ih * p.W + iw) * 4) + (uint32_t)(img * p.C + b_chl) * p.xplane_bytes : 0x80000000u;
            return;
        }
        const bool ok = (uint32_t)(w_oh - ylo) < ycnt && (uint32_t)(w_ow - xlo) < xcnt;
        ld_vb = ok ? (uint32_t)w_addr : 0x80000000u;
    };
    auto issue_a = [&](int j, uint32_t stage) {
        if constexpr (DIRECT) {                       // row a_row0 + 32 j: 32 planes further in the same image
            xsmi::load_lds_b128(ry, stage + (uint32_t)((wave + 4 * j) * 1024), d_left > 0 ? (uint32_t)d_addr : 0x80000000u,
                                (uint32_t)j * 32u * p.yplane_bytes);
            return;
        }
        const uint32_t v = j == 0 ? a_v0 : a_v1;
        // (a load in each branch keeps this a branch: as a select it would cost five vector instructions per chunk)
        if (ld_tail) xsmi::load_lds_b128(ry, stage + (uint32_t)((wave + 4 * j) * 1024), ld_ml0 + 4 * a_q < p.OHWa ? v : 0x80000000u, ld_sa);
        else xsmi::load_lds_b128(ry, stage + (uint32_t)((wave + 4 * j) * 1024), v, ld_sa);
    };
    auto issue_b = [&](int e, uint32_t stage) {
        xsmi::load_lds_b32(rx, stage + (uint32_t)(8192 + (wave + 4 * e) * 256), ld_vb, ld_sb + (uint32_t)(8 * e) * p.xplane_bytes);
    };
    auto issue_advance = [&]() {
        if constexpr (DIRECT) {
            d_pl += MC;
            const bool leaves = d_pl >= p.OHW;
            d_pl -= leaves ? p.OHW : 0;
            d_addr += MC * 4 + (leaves ? (p.K - 1) * (int)p.yplane_bytes : 0);
            d_left -= MC;
        }
        if (++ci == p.cpi) {
            ci = 0; ++in_img;
            w_oh = b_m / p.OW;                                       // the lane's pixel in an image's first chunk
            w_ow = b_m - w_oh * p.OW;
            w_addr = w_oh * row_bytes + w_ow * col_bytes + lane_bytes;
        } else {
            w_ow += r32;
            const bool carry = w_ow >= p.OW;
            w_ow -= carry ? p.OW : 0;
            w_oh += q32 + (carry ? 1 : 0);
            w_addr += carry ? carry_bytes : step_bytes;
        }
    };
    // chunk i of the workgroup's range lives in stage i % 2 and its fragments in register set i % 2
    auto issue_all = [&](int st) {
        const uint32_t stage = lds0 + (uint32_t)(st * STAGE_FLOATS * 4);
        issue_prep();
        issue_a(0, stage);
        issue_a(1, stage);
#pragma unroll
        for (int e = 0; e < 8; ++e) issue_b(e, stage);
        issue_advance();
    };

    // ---- fragment role ----
    const int f_arow = wr * 32 + l31, f_bch = wc * 32 + l31;
    int a_rd[4], b_rd[4];                                            // float index of this lane's four 16-byte groups
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        a_rd[g] = (f_arow * 8 + ((4 * h + g) ^ (f_arow & 7))) * 4;
        b_rd[g] = 2048 + (f_bch * 8 + ((4 * h + g) ^ (f_bch & 7))) * 4;
    }
    const int want_db = __builtin_amdgcn_readfirstlane(p.dbpart != nullptr && lx == 0 && wc == 0 ? 1 : 0);
    float dbacc = 0.f;

    floatx16 acc = {0}, acc2 = {0};
    float4 fa[2][4], fb[2][4];
#define XSMI_MFMA(ACC, AV, BV) ACC = __builtin_amdgcn_mfma_f32_32x32x2f32(AV, BV, ACC, 0, 0, 0)
#define XSMI_PIN() __builtin_amdgcn_sched_barrier(0)
    auto body = [&](auto buf_tag, auto static_tag, int it) {
        constexpr int cur = decltype(buf_tag)::value;
        constexpr int nxt = cur ^ 1;
        constexpr bool all = decltype(static_tag)::value;
        const bool has_next = all || it + 1 < nchunks;
        const bool has_load = all || it + 1 + D < nchunks;
        const float *rd_stage = smem[nxt];                               // the next chunk's stage
        const uint32_t ld_to = lds0 + (uint32_t)(cur * STAGE_FLOATS * 4);  // this chunk's stage is free after the barrier
        XSMI_MFMA(acc, fa[cur][0].x, fb[cur][0].x);
        XSMI_MFMA(acc2, fa[cur][0].y, fb[cur][0].y);
        XSMI_MFMA(acc, fa[cur][0].z, fb[cur][0].z);
        XSMI_MFMA(acc2, fa[cur][0].w, fb[cur][0].w);
        XSMI_PIN();
        if (has_next) {
            if (all || it + 1 + D <= nchunks) xsmi::wait_vmcnt<(D - 1) * LOADS>();
            else xsmi::wait_vmcnt<0>();
            xsmi::block_barrier();
        }
        XSMI_PIN();
#define XSMI_SLOT(ACC, AV, BV, STMT1, STMT2)   \
        XSMI_MFMA(ACC, AV, BV);                 \
        if (has_next) { STMT1; }                \
        if (has_load) { STMT2; }                \
        XSMI_PIN();
        XSMI_SLOT(acc, fa[cur][1].x, fb[cur][1].x, fa[nxt][0] = *reinterpret_cast<const float4 *>(rd_stage + a_rd[0]), issue_prep())
        XSMI_SLOT(acc2, fa[cur][1].y, fb[cur][1].y, fb[nxt][0] = *reinterpret_cast<const float4 *>(rd_stage + b_rd[0]), issue_a(0, ld_to))
        XSMI_SLOT(acc, fa[cur][1].z, fb[cur][1].z, fa[nxt][1] = *reinterpret_cast<const float4 *>(rd_stage + a_rd[1]), issue_a(1, ld_to))
        XSMI_SLOT(acc2, fa[cur][1].w, fb[cur][1].w, fb[nxt][1] = *reinterpret_cast<const float4 *>(rd_stage + b_rd[1]), issue_b(0, ld_to))
        XSMI_SLOT(acc, fa[cur][2].x, fb[cur][2].x, fa[nxt][2] = *reinterpret_cast<const float4 *>(rd_stage + a_rd[2]), issue_b(1, ld_to))
        XSMI_SLOT(acc2, fa[cur][2].y, fb[cur][2].y, fb[nxt][2] = *reinterpret_cast<const float4 *>(rd_stage + b_rd[2]), issue_b(2, ld_to))
        XSMI_SLOT(acc, fa[cur][2].z, fb[cur][2].z, fa[nxt][3] = *reinterpret_cast<const float4 *>(rd_stage + a_rd[3]), issue_b(3, ld_to))
        XSMI_SLOT(acc2, fa[cur][2].w, fb[cur][2].w, fb[nxt][3] = *reinterpret_cast<const float4 *>(rd_stage + b_rd[3]), issue_b(4, ld_to))
        XSMI_SLOT(acc, fa[cur][3].x, fb[cur][3].x, (void)0, issue_b(5, ld_to))
        XSMI_SLOT(acc2, fa[cur][3].y, fb[cur][3].y, (void)0, issue_b(6, ld_to))
        XSMI_SLOT(acc, fa[cur][3].z, fb[cur][3].z, (void)0, issue_b(7, ld_to))
        XSMI_SLOT(acc2, fa[cur][3].w, fb[cur][3].w, (void)0, issue_advance())
#undef XSMI_SLOT
        if (want_db) {
#pragma unroll
            for (int g = 0; g < 4; ++g) dbacc += (fa[cur][g].x + fa[cur][g].y) + (fa[cur][g].z + fa[cur][g].w);
        }
    };

    static_assert(STAGES == 2 && D == 1, "stage = chunk parity");
    if (nchunks > 0) {
        issue_all(0);
        xsmi::wait_vmcnt<0>();
        xsmi::block_barrier();
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            fa[0][g] = *reinterpret_cast<const float4 *>(smem[0] + a_rd[g]);
            fb[0][g] = *reinterpret_cast<const float4 *>(smem[0] + b_rd[g]);
        }
        if (1 < nchunks) issue_all(1);
    }
    {
        using T0 = std::integral_constant<int, 0>;
        using T1 = std::integral_constant<int, 1>;
        int it = 0;
        const int n_steady = nchunks - 1 - D;
        for (; it + 1 < n_steady; it += 2) {
            body(T0{}, std::true_type{}, it);
            body(T1{}, std::true_type{}, it + 1);
        }
        for (; it < nchunks; it += 2) {
            body(T0{}, std::false_type{}, it);
            if (it + 1 < nchunks) body(T1{}, std::false_type{}, it + 1);
        }
    }
#undef XSMI_MFMA
#undef XSMI_PIN
    acc += acc2;

    // accumulator register v of lane l: filter row 8*(v/4) + 4*(l/32) + v%4, channel column l%32
    const int taps = p.R * p.S;
    float *dst = p.part + (((size_t)split * taps + tapidx) * p.K + k0 + wr * 32 + 4 * h) * p.C + c0 + wc * 32 + l31;
#pragma unroll
    for (int v = 0; v < 16; ++v) dst[(size_t)(8 * (v >> 2) + (v & 3)) * p.C] = acc[v];

    if (want_db) {
        float other = __shfl_xor(dbacc, 32);
        if (h == 0) p.dbpart[(size_t)split * p.K + k0 + wr * 32 + l31] = dbacc + other;
    }
}

// dw[k][c][tap] = beta*dw + sum over splits (ascending, float64) of part[split][tap][k][c].
// 256 threads = 64 consecutive c x 4 interleaved split groups, combined in group order.
// Blocks past the last dw block reduce the bias partials the same way (64 filters each), so
// that db costs no launch of its own: db[k] = beta*db + sum over splits of dbpart[split][k].
__global__ void __launch_bounds__(256) wgrad_tap_reduce_kernel(const float *__restrict__ part, float *__restrict__ dw,
                                                                const float *__restrict__ dbpart, float *__restrict__ db,
                                                                int K, int C, int taps, int splits, int dw_blocks,
                                                                int accumulate) {
    __shared__ double sm[4][64];
    const int cl = threadIdx.x & 63, g = threadIdx.x >> 6;
    int b = blockIdx.x;
    const bool bias_block = b >= dw_blocks;               // uniform per block
    const float *src;
    size_t stride, o;
    float *dst;
    if (bias_block) {
        const int k = (b - dw_blocks) * 64 + cl;
        src = dbpart + k; stride = (size_t)K; dst = db; o = (size_t)k;
    } else {
        const int ctiles = C / 64;
        const int ct = b % ctiles; b /= ctiles;
        const int k = b % K;
        const int tap = b / K;
        const int c = ct * 64 + cl;
        stride = (size_t)taps * K * C;
        src = part + ((size_t)tap * K + k) * C + c;
        dst = dw; o = ((size_t)k * C + c) * taps + tap;
    }
    // group g adds the splits g, g + 4, g + 8, ... in that order; eight loads are in flight before the first add (the
    // loop is bound by memory latency: with two in flight it took 12 us for 113 splits of a 64 x 64 x 3 x 3 filter)
    double sum = 0.0;
    int sp = g;
    for (; sp + 28 < splits; sp += 32) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = src[(size_t)(sp + 4 * i) * stride];
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += (double)v[i];
    }
    for (; sp < splits; sp += 4) sum += (double)src[(size_t)sp * stride];
    sm[g][cl] = sum;
    __syncthreads();
    if (g == 0) {
        double s = ((sm[0][cl] + sm[1][cl]) + sm[2][cl]) + sm[3][cl];
        if (accumulate) s += (double)dst[o];
        dst[o] = (float)s;
    }
}

// The same reduction for large 3x3 filters (K*C >= 65536) with few splits: a thread owns one (k, c) and all nine taps,
// adds the splits in ascending order in float64 and writes nine consecutive floats of dw, so that a wavefront reads
// 256 contiguous bytes per (split, tap) and fills 2304 contiguous bytes of dw.  Bias blocks as above.
__global__ void __launch_bounds__(256) wgrad_tap_reduce9_kernel(const float *__restrict__ part, float *__restrict__ dw,
                                                                 const float *__restrict__ dbpart, float *__restrict__ db,
                                                                 int K, int C, int splits, int dw_blocks, int accumulate) {
    if ((int)blockIdx.x >= dw_blocks) {
        if (threadIdx.x >= 64) return;
        const int k = ((int)blockIdx.x - dw_blocks) * 64 + (int)threadIdx.x;
        double s = 0.0;
        for (int sp = 0; sp < splits; ++sp) s += (double)dbpart[(size_t)sp * K + k];
        if (accumulate) s += (double)db[k];
        db[k] = (float)s;
        return;
    }
    const size_t KC = (size_t)K * C;
    const bool live = (size_t)blockIdx.x * 256 + threadIdx.x < KC;
    const size_t kc = live ? (size_t)blockIdx.x * 256 + threadIdx.x : 0;      // k * C + c
    double s[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) s[t] = 0.0;
    int sp = 0;
    for (; sp + 1 < splits; sp += 2) {                 // 18 loads in flight
        const float *src = part + (size_t)sp * 9 * KC + kc;
        float v[18];
#pragma unroll
        for (int t = 0; t < 18; ++t) v[t] = src[(size_t)t * KC];
#pragma unroll
        for (int t = 0; t < 9; ++t) s[t] = (s[t] + (double)v[t]) + (double)v[9 + t];
    }
    if (sp < splits) {
        const float *src = part + (size_t)sp * 9 * KC + kc;
#pragma unroll
        for (int t = 0; t < 9; ++t) s[t] += (double)src[(size_t)t * KC];
    }
    // A thread's nine values are nine consecutive floats of dw, a workgroup's 2304 one contiguous run: they go through
    // the LDS so that every store instruction writes 256 consecutive floats (a lane storing its own nine one by one
    // touches eighteen cache lines per instruction).
    __shared__ double tile[256 * 9];                   // (float64: with `accumulate` the old value joins before the one rounding)
#pragma unroll
    for (int t = 0; t < 9; ++t) tile[threadIdx.x * 9 + t] = s[t];
    __syncthreads();
    const size_t base = (size_t)blockIdx.x * 256 * 9, limit = KC * 9;
#pragma unroll
    for (int i = 0; i < 9; ++i) {
        const size_t o = base + (size_t)i * 256 + threadIdx.x;
        if (o < limit) dw[o] = (float)(accumulate ? tile[i * 256 + threadIdx.x] + (double)dw[o] : tile[i * 256 + threadIdx.x]);
    }
}

// dst[plane][0 .. OHWa) = src[plane][0 .. OHW) followed by zeros
__global__ void __launch_bounds__(256) pad_planes_kernel(const float *__restrict__ src, float *__restrict__ dst, int OHW,
                                                          int OHWa, uint32_t total) {
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < total; i += gridDim.x * 256u) {
        const uint32_t pl = i / (uint32_t)OHWa, m = i - pl * (uint32_t)OHWa;
        dst[i] = m < (uint32_t)OHW ? src[(size_t)pl * OHW + m] : 0.f;
    }
}

// dst[k][0 .. Ma) = the pixels of filter plane k of every image, image after image (N*OHW values), then zeros:
// the reduction index of the weight gradient as one dense run per filter.
__global__ void __launch_bounds__(256) gather_filter_rows_kernel(const float *__restrict__ src, float *__restrict__ dst, int K,
                                                                 int OHW, int M, int Ma, xsmi::FastDiv dMa, xsmi::FastDiv dOHW,
                                                                 uint32_t total) {
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < total; i += gridDim.x * 256u) {
        const uint32_t k = xsmi::fdiv(i, dMa), m = i - k * (uint32_t)Ma;
        float v = 0.f;
        if (m < (uint32_t)M) {
            const uint32_t n = xsmi::fdiv(m, dOHW), pl = m - n * (uint32_t)OHW;
            v = src[((size_t)n * K + k) * OHW + pl];
        }
        dst[i] = v;
    }
}

// Small feature maps waste chunk slots when chunks may not straddle images (49 pixels fill 64 slots to 77 %, 196
// fill 224 to 88 %): they take the dense form.
bool use_flat(int OHW) { return OHW * 20 < xsmi::ceil_div(OHW, MC) * MC * 19; }

void plan(int N, int C, int K, int R, int S, int OHW, int *cpi, int *total, int *cps, int *splits) {
    if (use_flat(OHW)) {                              // one "image" holding the pixels of the whole batch
        OHW = N * OHW;
        N = 1;
    }
    const int tiles = R * S * (C / TC) * (K / TK);
    *cpi = xsmi::ceil_div(OHW, MC);
    *total = N * *cpi;
    // The number of pixel ranges is chosen by a cost model of the launch: workgroups spread evenly over the compute
    // units (four resident per CU) and the units' matrix pipes are shared by their workgroups, so the launch takes
    // about ceil(workgroups / CUs) * (chunks per range).  A few workgroups beyond a multiple of the CU count cost a
    // whole extra share (128 -> 128 at 28 x 28: 29 ranges x 36 tiles = 1044 workgroups took 88 us, 28 x 36 = 1008
    // take 74; 512 -> 512 at 7 x 7 is better off with 2 x 576 than with 1 x 576).  The CU count is the MI355X's, as a
    // constant: the workspace query must plan the same split before a device is initialised.
    constexpr int CUS = 256;
    const int want = TARGET_BLOCKS / tiles > 1 ? TARGET_BLOCKS / tiles : 1;
    long best_cost = -1;
    int best_c = 0;
    for (int sgl = want > 3 ? want - 2 : 1; sgl <= want + 2; ++sgl) {
        int c = xsmi::ceil_div(*total, sgl);
        if (c < 8) c = 8;
        // Long pixel ranges let the R*S workgroups that share a range drift apart until each fetches dy and x from
        // HBM on its own; at most 64 chunks (2048 pixels) per range keeps them within reach of one L2
        // (measured at N=256, 64->64, 56x56: 631 -> 516 us).
        if (c > 64) c = 64;
        if (c > *total) c = *total;
        const long wgs = (long)tiles * xsmi::ceil_div(*total, c);
        const long cost = ((wgs + CUS - 1) / CUS) * c;
        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_c = c; }
    }
    *cps = best_c;
    *splits = xsmi::ceil_div(*total, best_c);
}

}  // namespace

namespace xsmi {

bool wgrad_tap_ok(const float *dy, const float *x, int C, int K, int OH, int OW) {
    return C % TC == 0 && K % TK == 0 && ((uintptr_t)dy % 16) == 0 && ((uintptr_t)x % 4) == 0;
}

size_t wgrad_tap_ws_bytes(int N, int C, int K, int R, int S, int OH, int OW) {
    int cpi, total, cps, splits;
    plan(N, C, K, R, S, OH * OW, &cpi, &total, &cps, &splits);
    const int OHW = OH * OW, OHWa = (OHW + 3) & ~3;
    size_t padded = OHWa != OHW ? align_up((size_t)N * K * OHWa * sizeof(float), 256) : 0;
    if (use_flat(OHW)) padded = OHW % 4 == 0 && OHW >= MC ? 0 : align_up((size_t)K * ((N * OHW + 3) & ~3) * sizeof(float), 256);
    return align_up((size_t)splits * R * S * K * C * sizeof(float), 256) + align_up((size_t)splits * K * sizeof(float), 256) + padded;
}

int wgrad_tap(const float *dy, const float *x, float *dw, float *db, int N, int C, int H, int W, int K, int R, int S,
              int sh, int sw, int pad, int OH, int OW, int accumulate, void *workspace) {
    WgradTapParams p;
    int splits;
    plan(N, C, K, R, S, OH * OW, &p.cpi, &p.total_chunks, &p.cps, &splits);
    p.dy = dy; p.x = x;
    p.part = (float *)workspace;
    float *dbpart = (float *)((char *)workspace + align_up((size_t)splits * R * S * K * C * sizeof(float), 256));
    hipStream_t st = stream();
    int OHW = OH * OW, OHWa = (OHW + 3) & ~3;
    const bool flat = use_flat(OHW);
    p.flat = flat ? 1 : 0;
    p.Mtot = N * OHW;
    p.dOHW = make_fastdiv(OHW);
    // dy as it lies when its planes are whole 16-byte pieces and at least a chunk long
    const bool direct = flat && OHW % 4 == 0 && OHW >= MC;
    if (direct) {
        OHWa = OHW;
    } else if (flat) {
        float *dyp = (float *)((char *)dbpart + align_up((size_t)splits * K * sizeof(float), 256));
        const int Ma = (p.Mtot + 3) & ~3;
        const uint32_t total = (uint32_t)((size_t)K * Ma);
        uint32_t blocks = (total + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(gather_filter_rows_kernel, dim3(blocks), dim3(256), 0, st, dy, dyp, K, OHW, p.Mtot, Ma, make_fastdiv(Ma),
                           p.dOHW, total);
        XSMI_LAUNCH_CHECK("gather_filter_rows_kernel");
        p.dy = dyp;
        OHWa = Ma;                                   // the "plane" of the dy operand is now a filter's whole row
    } else if (OHWa != OHW) {
        float *dyp = (float *)((char *)dbpart + align_up((size_t)splits * K * sizeof(float), 256));
        const uint32_t total = (uint32_t)((size_t)N * K * OHWa);
        uint32_t blocks = (total + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(pad_planes_kernel, dim3(blocks), dim3(256), 0, st, dy, dyp, OHW, OHWa, total);
        XSMI_LAUNCH_CHECK("pad_planes_kernel");
        p.dy = dyp;
    }
    p.dbpart = db ? dbpart : nullptr;
    p.x_bytes = (uint32_t)((size_t)N * C * H * W * 4);
    p.dy_bytes = flat && !direct ? (uint32_t)((size_t)K * OHWa * 4) : (uint32_t)((size_t)N * K * OHWa * 4);
    p.N = N; p.C = C; p.K = K; p.H = H; p.W = W; p.OH = OH; p.OW = OW; p.OHW = OHW; p.OHWa = OHWa; p.R = R; p.S = S;
    p.sh = sh; p.sw = sw; p.pad = pad;
    p.ctiles = C / TC;
    p.xplane_bytes = (uint32_t)(H * W * 4); p.yplane_bytes = (uint32_t)(OHWa * 4);
    p.dOW = make_fastdiv(OW); p.dCT = make_fastdiv(p.ctiles); p.dS = make_fastdiv(S);

    dim3 grid(R * S * p.ctiles, K / TK, splits);
    prof_begin();
    if (direct) hipLaunchKernelGGL(wgrad_tap_f32_kernel<true>, grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL(wgrad_tap_f32_kernel<false>, grid, dim3(256), 0, st, p);
    prof_end();
    XSMI_LAUNCH_CHECK("wgrad_tap_f32_kernel");
    if (R * S == 9 && (size_t)K * C >= 65536 && splits <= 16) {
        const int blocks9 = (int)(((size_t)K * C + 255) / 256);
        hipLaunchKernelGGL(wgrad_tap_reduce9_kernel, dim3(blocks9 + (db ? K / 64 : 0)), dim3(256), 0, st, p.part, dw, dbpart, db,
                           K, C, splits, blocks9, accumulate);
        XSMI_LAUNCH_CHECK("wgrad_tap_reduce9_kernel");
        return XSMI_OK;
    }
    const int dw_blocks = R * S * K * p.ctiles;
    hipLaunchKernelGGL(wgrad_tap_reduce_kernel, dim3(dw_blocks + (db ? K / 64 : 0)), dim3(256), 0, st, p.part, dw, dbpart, db,
                       K, C, R * S, splits, dw_blocks, accumulate);
    XSMI_LAUNCH_CHECK("wgrad_tap_reduce_kernel");
    return XSMI_OK;
}

}  // namespace xsmi
