// Tap-major implicit-GEMM convolution (forward and backward-data) on fp32 MFMA
// for layers whose reduction-channel count is a multiple of 32.
//
// The reduction index is ordered (tap, channel) instead of the filter's own
// (channel, tap) order: for one tap (r, s) the 32 operand values a pixel needs in
// a chunk sit exactly one channel plane apart in memory and are all valid or all
// in the zero border together.  A thread therefore computes ONE byte offset and
// one validity test per tap, and the per-channel displacement rides in the
// scalar offset of the buffer load: no per-element address arithmetic, no offset
// table.  Invalid lanes use an offset beyond the buffer's size, which the
// hardware range check turns into 0.0 (the scalar offset is not part of that
// check, so valid lanes must and do stay inside the tensor).
//
// Tile: 64 rows x 64 pixels per 256-thread workgroup (2 x 2 waves of 32x32),
// chunks of 32 channels, two LDS stages.  Wave w stages channels 8w..8w+7 of the
// chunk for all 64 pixels (lane == pixel, so one load instruction covers 64
// consecutive pixels of one channel plane).  For the MFMA, lanes 0-31 consume
// channel groups 0 and 2, lanes 32-63 groups 1 and 3; each group of 8 values is
// two 128-bit LDS reads.  LDS rows are 8 floats with the two halves swapped on
// rows whose index has bit 2 set, which spreads any 8 consecutive lanes' 128-bit
// accesses over all 32 banks without padding.
#include "xsmi_internal.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TM = 64;
constexpr int BP = 64;
constexpr int KC = 32;
constexpr int STAGE_FLOATS = 4 * 64 * 8;   // one operand, one stage

struct TapParams {
    const float *in;
    const float *apk;     // [rowtile][tap*nch + cc][group 4][row 64][8]
    const float *bias;
    float *out;
    uint8_t *mask;
    uint32_t in_bytes;
    int M, rows;
    int nch;              // channel chunks per tap
    int TR, TS;           // taps
    int dy0, dx0, dstep;  // input row for tap r: y*sy + dy0 + r*dstep
    int IH, IW, sy, sx;
    int in_n_stride;      // elements
    uint32_t plane_bytes; // IH*IW*4
    int OY, OX;
    xsmi::FastDiv dOX, dOY;
    long long os_n, os_k, o_base;
    int os_y, os_x;
    int accumulate, relu;
};

__device__ __forceinline__ float buffer_load_f32(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)voff, (int)soff, 0));
}

// float offset of 128-bit half f (0/1) of LDS row `row` in group q
__device__ __forceinline__ int lds_off(int q, int row, int f) { return ((q * 64 + row) * 2 + (f ^ ((row >> 2) & 1))) * 4; }

__global__ void __launch_bounds__(256) tap_igemm_f32_kernel(TapParams p) {
    __shared__ __attribute__((aligned(16))) float As[2][STAGE_FLOATS];
    __shared__ __attribute__((aligned(16))) float Bs[2][STAGE_FLOATS];

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int m0 = blockIdx.x * BP;
    const int rowtile = blockIdx.y;

    // ---- gather role: pixel m0 + lane, channel group `wave` ----
    int iyb = 0, ixb = 0, nbase = 0;
    const bool live = m0 + lane < p.M;
    if (live) {
        uint32_t m = (uint32_t)(m0 + lane);
        uint32_t q = xsmi::fdiv(m, p.dOX);
        int x = (int)m - (int)q * p.OX;
        uint32_t n = xsmi::fdiv(q, p.dOY);
        int y = (int)q - (int)n * p.OY;
        iyb = y * p.sy + p.dy0;
        ixb = x * p.sx + p.dx0;
        nbase = (int)n * p.in_n_stride;
    }
    __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.in, 0, p.in_bytes, 0x00020000);
    const int iters = p.TR * p.TS * p.nch;
    const float4 *apk4 = reinterpret_cast<const float4 *>(p.apk) + (size_t)rowtile * iters * (TM * KC / 4) + t;

    // LDS slots this thread writes
    const int bw0 = lds_off(wave, lane, 0), bw1 = lds_off(wave, lane, 1);
    const int aw0 = lds_off(t >> 7, (t & 127) >> 1, t & 1);           // float4 #t
    const int aw1 = lds_off((t >> 7) + 2, (t & 127) >> 1, t & 1);     // float4 #t+256

    float bnext[8];
    float4 an0, an1;
    int r = 0, s = 0, cc = 0;   // position of the NEXT chunk to fetch

    auto fetch = [&](int it) {
        int iy = iyb + r * p.dstep, ix = ixb + s * p.dstep;
        bool ok = live && (unsigned)iy < (unsigned)p.IH && (unsigned)ix < (unsigned)p.IW;
        uint32_t voff = ok ? (uint32_t)((nbase + iy * p.IW + ix) * 4) : 0x80000000u;
        uint32_t soff = (uint32_t)(cc * KC + wave * 8) * p.plane_bytes;
#pragma unroll
        for (int e = 0; e < 8; ++e) bnext[e] = buffer_load_f32(rsrc, voff, soff + (uint32_t)e * p.plane_bytes);
        const float4 *ap = apk4 + (size_t)it * (TM * KC / 4);
        an0 = ap[0];
        an1 = ap[256];
        if (++cc == p.nch) {
            cc = 0;
            if (++s == p.TS) { s = 0; ++r; }
        }
    };
    auto stage = [&](int buf) {
        *reinterpret_cast<float4 *>(&Bs[buf][bw0]) = make_float4(bnext[0], bnext[1], bnext[2], bnext[3]);
        *reinterpret_cast<float4 *>(&Bs[buf][bw1]) = make_float4(bnext[4], bnext[5], bnext[6], bnext[7]);
        *reinterpret_cast<float4 *>(&As[buf][aw0]) = an0;
        *reinterpret_cast<float4 *>(&As[buf][aw1]) = an1;
    };

    floatx16 acc = {0};
    const int h = lane >> 5, l31 = lane & 31;
    const int wr = wave >> 1, wc = wave & 1;
    const int arow = wr * 32 + l31, bcol = wc * 32 + l31;
    const int ar00 = lds_off(h, arow, 0), ar01 = lds_off(h, arow, 1);
    const int ar10 = lds_off(h + 2, arow, 0), ar11 = lds_off(h + 2, arow, 1);
    const int br00 = lds_off(h, bcol, 0), br01 = lds_off(h, bcol, 1);
    const int br10 = lds_off(h + 2, bcol, 0), br11 = lds_off(h + 2, bcol, 1);

    if (iters > 0) {
        fetch(0);
        stage(0);
    }
    __syncthreads();
    for (int it = 0; it < iters; ++it) {
        const int cur = it & 1;
        const bool more = it + 1 < iters;
        if (more) fetch(it + 1);
        const float *A = As[cur], *B = Bs[cur];
        float4 a0 = *reinterpret_cast<const float4 *>(A + ar00), b0 = *reinterpret_cast<const float4 *>(B + br00);
        float4 a1 = *reinterpret_cast<const float4 *>(A + ar01), b1 = *reinterpret_cast<const float4 *>(B + br01);
        float4 a2 = *reinterpret_cast<const float4 *>(A + ar10), b2 = *reinterpret_cast<const float4 *>(B + br10);
        float4 a3 = *reinterpret_cast<const float4 *>(A + ar11), b3 = *reinterpret_cast<const float4 *>(B + br11);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.x, b0.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.y, b0.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.z, b0.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.w, b0.w, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.x, b1.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.y, b1.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.z, b1.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.w, b1.w, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a2.x, b2.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a2.y, b2.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a2.z, b2.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a2.w, b2.w, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a3.x, b3.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a3.y, b3.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a3.z, b3.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a3.w, b3.w, acc, 0, 0, 0);
        if (more) stage(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue: register v of lane l = row 8*(v/4) + 4*(l/32) + v%4, pixel l%32 ----
    const int m = m0 + wc * 32 + l31;
    if (m >= p.M) return;
    uint32_t q = xsmi::fdiv((uint32_t)m, p.dOX);
    int x = m - (int)q * p.OX;
    uint32_t n = xsmi::fdiv(q, p.dOY);
    int y = (int)q - (int)n * p.OY;
    const long long pix_off = (long long)n * p.os_n + (long long)y * p.os_y + (long long)x * p.os_x + p.o_base;
    const int rbase = rowtile * TM + wr * 32 + 4 * h;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        int row = rbase + 8 * (v >> 2) + (v & 3);
        if (row < p.rows) {
            float val = acc[v];
            if (p.bias) val += p.bias[row];
            long long o = pix_off + (long long)row * p.os_k;
            if (p.relu) {
                if (p.mask) p.mask[o] = val < 0.f ? 1 : 0;
                val = val > 0.f ? val : 0.f;
            }
            if (p.accumulate) val += p.out[o];
            p.out[o] = val;
        }
    }
}

// Packs A for the tap-major kernel.  mode 0 (forward): A[row][tap=(r,s)][ch] = w[row][ch][r][s].
// mode 1 (backward-data class): A[row=c][tap=(t,u)][ch=k] = w[k][c][r0 + sh*t][s0 + sw*u].
__global__ void __launch_bounds__(256) tap_pack_kernel(const float *__restrict__ w, float *__restrict__ apk, int mode,
                                                        int rows, int CH, int R, int S, int TR, int TS, int r0, int s0,
                                                        int sh, int sw, int rowtiles) {
    const int nch = CH / KC;
    const int iters = TR * TS * nch;
    const size_t total = (size_t)rowtiles * iters * (TM * KC);
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        int e = (int)(i & 7);
        int r64 = (int)((i >> 3) & 63);
        int q = (int)((i >> 9) & 3);
        size_t blk = i >> 11;
        int it = (int)(blk % iters);
        int rt = (int)(blk / iters);
        int cc = it % nch, tap = it / nch;
        int tr = tap / TS, ts = tap % TS;
        int ch = cc * KC + q * 8 + e;
        int row = rt * TM + r64;
        float v = 0.f;
        if (row < rows) {
            if (mode == 0)
                v = w[(((size_t)row * CH + ch) * R + tr) * S + ts];
            else
                v = w[(((size_t)ch * rows + row) * R + (r0 + sh * tr)) * S + (s0 + sw * ts)];
        }
        apk[i] = v;
    }
}

size_t tap_pack_bytes(int rows, int CH, int taps) {
    return xsmi::align_up((size_t)xsmi::ceil_div(rows, TM) * taps * (CH / KC) * TM * KC * sizeof(float), 256);
}

int launch_pack(hipStream_t st, const float *w, float *apk, int mode, int rows, int CH, int R, int S, int TR, int TS,
                int r0, int s0, int sh, int sw) {
    const int rowtiles = xsmi::ceil_div(rows, TM);
    size_t total = (size_t)rowtiles * TR * TS * (CH / KC) * TM * KC;
    if (total == 0) return XSMI_OK;
    int blocks = (int)((total + 255) / 256);
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(tap_pack_kernel, dim3(blocks), dim3(256), 0, st, w, apk, mode, rows, CH, R, S, TR, TS, r0, s0, sh,
                       sw, rowtiles);
    XSMI_LAUNCH_CHECK("tap_pack_kernel");
    return XSMI_OK;
}

}  // namespace

namespace xsmi {

bool tap_path_ok(int reduce_channels) { return reduce_channels % KC == 0; }

size_t tap_fwd_ws_bytes(int C, int K, int R, int S) { return tap_pack_bytes(K, C, R * S); }

size_t tap_bwd_data_ws_bytes(int C, int K, int R, int S, int sh, int sw) {
    size_t total = 0;
    for (int ph = 0; ph < sh; ++ph)
        for (int pw = 0; pw < sw; ++pw) total += tap_pack_bytes(C, K, ceil_div(R, sh) * ceil_div(S, sw));
    return total;
}

int tap_conv_fwd(const float *x, const float *w, const float *bias, float *y, uint8_t *mask, int N, int C, int H, int W,
                 int K, int R, int S, int sh, int sw, int pad, int OH, int OW, int relu, void *workspace) {
    hipStream_t st = stream();
    float *apk = (float *)workspace;
    int rc = launch_pack(st, w, apk, 0, K, C, R, S, R, S, 0, 0, 1, 1);
    if (rc) return rc;
    TapParams p;
    p.in = x; p.apk = apk; p.bias = bias; p.out = y; p.mask = relu ? mask : nullptr;
    p.in_bytes = (uint32_t)((size_t)N * C * H * W * 4);
    p.M = N * OH * OW; p.rows = K; p.nch = C / KC; p.TR = R; p.TS = S;
    p.dy0 = -pad; p.dx0 = -pad; p.dstep = 1;
    p.IH = H; p.IW = W; p.sy = sh; p.sx = sw;
    p.in_n_stride = C * H * W; p.plane_bytes = (uint32_t)(H * W * 4);
    p.OY = OH; p.OX = OW; p.dOX = make_fastdiv(OW); p.dOY = make_fastdiv(OH);
    p.os_n = (long long)K * OH * OW; p.os_k = (long long)OH * OW; p.o_base = 0; p.os_y = OW; p.os_x = 1;
    p.accumulate = 0; p.relu = relu;
    dim3 grid(ceil_div(p.M, BP), ceil_div(K, TM));
    prof_begin();
    hipLaunchKernelGGL(tap_igemm_f32_kernel, grid, dim3(256), 0, st, p);
    prof_end();
    XSMI_LAUNCH_CHECK("tap_igemm_f32_kernel");
    return XSMI_OK;
}

int tap_conv_bwd_data(const float *dy, const float *w, float *dx, int N, int C, int H, int W, int K, int R, int S, int sh,
                      int sw, int pad, int OH, int OW, int accumulate, void *workspace) {
    hipStream_t st = stream();
    char *ws = (char *)workspace;
    struct Plan { TapParams p; dim3 grid; };
    Plan plans[64];
    int nplans = 0;
    for (int ph = 0; ph < sh; ++ph) {
        const int OYc = ph < H ? ceil_div(H - ph, sh) : 0;
        const int r0 = (ph + pad) % sh;
        const int T = r0 < R ? ceil_div(R - r0, sh) : 0;
        const int cy = (ph + pad - r0) / sh;
        for (int pw = 0; pw < sw; ++pw) {
            const int OXc = pw < W ? ceil_div(W - pw, sw) : 0;
            if (OYc == 0 || OXc == 0) continue;
            const int s0 = (pw + pad) % sw;
            const int U = s0 < S ? ceil_div(S - s0, sw) : 0;
            const int cx = (pw + pad - s0) / sw;
            float *apk = (float *)ws;
            ws += tap_pack_bytes(C, K, T * U);
            int rc = launch_pack(st, w, apk, 1, C, K, R, S, T, U, r0, s0, sh, sw);
            if (rc) return rc;
            TapParams p;
            p.in = dy; p.apk = apk; p.bias = nullptr; p.out = dx; p.mask = nullptr;
            p.in_bytes = (uint32_t)((size_t)N * K * OH * OW * 4);
            p.M = N * OYc * OXc; p.rows = C; p.nch = K / KC; p.TR = T; p.TS = U;
            p.dy0 = cy; p.dx0 = cx; p.dstep = -1;
            p.IH = OH; p.IW = OW; p.sy = 1; p.sx = 1;
            p.in_n_stride = K * OH * OW; p.plane_bytes = (uint32_t)(OH * OW * 4);
            p.OY = OYc; p.OX = OXc; p.dOX = make_fastdiv(OXc); p.dOY = make_fastdiv(OYc);
            p.os_n = (long long)C * H * W; p.os_k = (long long)H * W; p.o_base = (long long)ph * W + pw;
            p.os_y = sh * W; p.os_x = sw;
            p.accumulate = accumulate; p.relu = 0;
            plans[nplans].p = p;
            plans[nplans].grid = dim3(ceil_div(p.M, BP), ceil_div(C, TM));
            ++nplans;
        }
    }
    prof_begin();
    for (int i = 0; i < nplans; ++i) {
        hipLaunchKernelGGL(tap_igemm_f32_kernel, plans[i].grid, dim3(256), 0, st, plans[i].p);
        XSMI_LAUNCH_CHECK("tap_igemm_f32_kernel");
    }
    prof_end();
    return XSMI_OK;
}

}  // namespace xsmi
