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
// Data path: global -> LDS directly (buffer_load ... lds), no staging registers.
// A stage holds
//     A  [8 quads][64 rows][4 floats]   (one 128-bit LDS-direct load per lane = row)
//     B  [32 channels][64 pixels]       (one dword LDS-direct load per lane = pixel)
// so each wave-level load lands as one contiguous LDS block.  STAGES stages are
// kept in flight (prefetch distance STAGES-1) and the loop waits with a vmcnt that
// leaves the younger chunks outstanding; one barrier per chunk both publishes the
// chunk that just landed and retires the stage that is about to be refilled.
//
// Tile: 64 rows x 64 pixels per 256-thread workgroup (2 x 2 waves of 32x32).  For
// the MFMA (v_mfma_f32_32x32x2_f32), lanes 0-31 take channels 0..15 of the chunk
// and lanes 32-63 channels 16..31: A comes as four 128-bit reads of consecutive
// 16-byte slots (conflict-free), B as sixteen dword reads of 32 consecutive floats.
#include "conv_store.h"
#include <stdlib.h>
#include <type_traits>

namespace {

using xsmi::floatx16;

constexpr int TM = 64;
constexpr int BP = 64;
constexpr int KC = 32;
constexpr int STAGE_FLOATS = 4096;         // A 2048 + B 2048
constexpr int LOADS_PER_CHUNK = 10;        // per wave: 8 dword (B) + 2 dwordx4 (A)
constexpr int TAP_STAGES = 2;

struct TapParams {
    const float *in;
    const float *apk;     // [rowtile][tap*nch + cc][quad 8][row 64][4]
    const float *bias;
    float *out;
    uint8_t *mask;
    uint32_t in_bytes;
    uint32_t apk_bytes;
    uint32_t out_bytes;
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
    int zfill;            // 1: the epilogue also clears the three neighbours of every stored value (see conv_store.h)
    // persistent kernel only
    uint32_t *counters;   // 8 tile counters (one per XCD), zeroed by the pack kernel
    uint32_t tiles;       // pixel tiles x row tiles
    int rowtiles;
};

// One launch can cover several parameter sets that share the row (output channel) tiling: the residue classes
// of a strided backward-data pass, each with its own pixel count, taps and packed filter.  Workgroup ids are
// concatenated class after class; first[c] is the first logical workgroup of class c.
constexpr int TAP_MAX_CLASSES = 4;
struct TapMulti {
    TapParams cls[TAP_MAX_CLASSES];
    uint32_t first[TAP_MAX_CLASSES + 1];
    int ncls;
    int rowtiles;
};

template <int STAGES>
__global__ void __launch_bounds__(256) tap_igemm_f32_kernel(TapMulti mp) {
    __shared__ __attribute__((aligned(16))) float smem[STAGES][STAGE_FLOATS];
    constexpr int D = STAGES - 1;

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    // logical block = (class, pixel tile, row tile) with the row tile fastest, contiguous per XCD: the row
    // tiles of one pixel tile and neighbouring pixel tiles (shared halo) meet in one L2
    uint32_t logical = xsmi::xcd_contiguous_id(blockIdx.x, gridDim.x);
    int ci = 0;
    while (ci + 1 < mp.ncls && logical >= mp.first[ci + 1]) ++ci;
    const TapParams &p = mp.cls[ci];
    logical -= mp.first[ci];
    const uint32_t nrt = (uint32_t)mp.rowtiles;
    const int rowtile = nrt == 1 ? 0 : (int)(logical % nrt);
    const int m0 = (int)(nrt == 1 ? logical : logical / nrt) * BP;
    // The tile's bias goes through the LDS: one coalesced load here instead of a dependent global load per
    // output element in the epilogue.  Only the forward pass has a bias, and it has at least one chunk, so a
    // barrier of the main loop lies between this store and the epilogue's reads.
    __shared__ __attribute__((aligned(16))) float s_bias[TM];
    if (p.bias && t < TM) s_bias[t] = rowtile * TM + t < p.rows ? p.bias[rowtile * TM + t] : 0.f;

    // ---- gather role: pixel m0 + lane, channels 8*wave .. 8*wave+7 of each chunk ----
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
    const xsmi::xsmi_int32x4 rin = xsmi::make_rsrc(p.in, p.in_bytes);
    const xsmi::xsmi_int32x4 rap = xsmi::make_rsrc(p.apk, p.apk_bytes);
    const uint32_t lds0 = (uint32_t)(uintptr_t)&smem[0][0];   // LDS byte address (low half of the flat address)
    const int iters = p.TR * p.TS * p.nch;
    const uint32_t a_voff = (uint32_t)((2 * wave * 64 + lane) * 16);

    // ---- issue state: position of the next chunk to load, kept in scalars ----
    int r = 0, s = 0, cc = 0;
    uint32_t ld_stage = lds0;                         // LDS byte address of the stage the next chunk goes to
    uint32_t ld_asoff = (uint32_t)rowtile * (uint32_t)iters * (uint32_t)(TM * KC * 4);
    uint32_t ld_voff = 0, ld_soff = 0;
    // per-tap part of a chunk's addresses (vector) and per-chunk part (scalar)
    auto issue_prep = [&]() {
        int iy = iyb + r * p.dstep, ix = ixb + s * p.dstep;
        bool ok = live && (unsigned)iy < (unsigned)p.IH && (unsigned)ix < (unsigned)p.IW;
        ld_voff = ok ? (uint32_t)((nbase + iy * p.IW + ix) * 4) : 0x80000000u;
        ld_soff = (uint32_t)(cc * KC + wave * 8) * p.plane_bytes;
    };
    auto issue_b = [&](int e) {                       // channel 8*wave + e of the chunk, all 64 pixels
        xsmi::load_lds_b32(rin, ld_stage + (uint32_t)((2048 + (wave * 8 + e) * 64) * 4), ld_voff,
                           ld_soff + (uint32_t)e * p.plane_bytes);
    };
    auto issue_a = [&](int qa) {                      // quad 2*wave + qa of the chunk, all 64 rows
        xsmi::load_lds_b128(rap, ld_stage + (uint32_t)((2 * wave + qa) * 1024), a_voff + (uint32_t)qa * 1024u, ld_asoff);
    };
    auto issue_advance = [&]() {
        ld_asoff += (uint32_t)(TM * KC * 4);
        ld_stage += (uint32_t)(STAGE_FLOATS * 4);
        if (ld_stage == lds0 + (uint32_t)(STAGES * STAGE_FLOATS * 4)) ld_stage = lds0;
        if (++cc == p.nch) {
            cc = 0;
            if (++s == p.TS) { s = 0; ++r; }
        }
    };
    auto issue_all = [&]() {
        issue_prep();
#pragma unroll
        for (int e = 0; e < 8; ++e) issue_b(e);
        issue_a(0);
        issue_a(1);
        issue_advance();
    };

    // Two accumulators take alternate reduction steps; they are added once at the end.
    floatx16 acc = {0}, acc2 = {0};
    const int h = lane >> 5, l31 = lane & 31;
    const int wr = wave >> 1, wc = wave & 1;
    const int a_rd = (4 * h * 64 + wr * 32 + l31) * 4;           // float index of quad 4h, this lane's row
    const int b_rd = 2048 + 16 * h * 64 + wc * 32 + l31;         // float index of channel 16h, this lane's pixel

    // Operand fragments of two consecutive chunks live in registers.  An iteration
    // is 16 MFMAs on the current fragments; after the first four it waits for the
    // next chunk and crosses the barrier, and every later MFMA is followed in
    // program order by one slice of the remaining work (one LDS fragment read of
    // the next chunk, one LDS-direct load of the chunk STAGES-1 ahead), so that work
    // issues while the matrix pipe is busy.  sched_barrier pins this order.
    float4 fa[2][4];
    float fb[2][16];
    const float *rd_stage = smem[0];                  // stage the next fragments are read from
    auto rd_advance = [&]() {
        rd_stage += STAGE_FLOATS;
        if (rd_stage == smem[0] + STAGES * STAGE_FLOATS) rd_stage = smem[0];
    };
#define XSMI_MFMA(ACC, AV, BV) ACC = __builtin_amdgcn_mfma_f32_32x32x2f32(AV, BV, ACC, 0, 0, 0)
#define XSMI_PIN() __builtin_amdgcn_sched_barrier(0)
    auto body = [&](auto buf_tag, auto static_tag, int it) {
        constexpr int cur = decltype(buf_tag)::value;
        constexpr int nxt = cur ^ 1;
        constexpr bool all = decltype(static_tag)::value;         // steady state: next chunk and next load both exist
        const bool has_next = all || it + 1 < iters;
        const bool has_load = all || it + 1 + D < iters;
        XSMI_MFMA(acc, fa[cur][0].x, fb[cur][0]);
        XSMI_MFMA(acc2, fa[cur][0].y, fb[cur][1]);
        XSMI_MFMA(acc, fa[cur][0].z, fb[cur][2]);
        XSMI_MFMA(acc2, fa[cur][0].w, fb[cur][3]);
        XSMI_PIN();
        if (has_next) {
            if (all || it + 1 + D <= iters) xsmi::wait_vmcnt<(D - 1) * LOADS_PER_CHUNK>();
            else xsmi::wait_vmcnt<0>();
            xsmi::block_barrier();
        }
        XSMI_PIN();
        XSMI_MFMA(acc, fa[cur][1].x, fb[cur][4]);
        if (has_next) fa[nxt][0] = *reinterpret_cast<const float4 *>(rd_stage + a_rd);
        if (has_load) issue_prep();
        XSMI_PIN();
        XSMI_MFMA(acc2, fa[cur][1].y, fb[cur][5]);
        if (has_next) fa[nxt][1] = *reinterpret_cast<const float4 *>(rd_stage + a_rd + 256);
        if (has_load) issue_b(0);
        XSMI_PIN();
        XSMI_MFMA(acc, fa[cur][1].z, fb[cur][6]);
        if (has_next) fa[nxt][2] = *reinterpret_cast<const float4 *>(rd_stage + a_rd + 512);
        if (has_load) issue_b(1);
        XSMI_PIN();
        XSMI_MFMA(acc2, fa[cur][1].w, fb[cur][7]);
        if (has_next) fa[nxt][3] = *reinterpret_cast<const float4 *>(rd_stage + a_rd + 768);
        if (has_load) issue_b(2);
        XSMI_PIN();
#define XSMI_SLOT(ACC, AV, J, LOADSTMT)                                      \
        XSMI_MFMA(ACC, AV, fb[cur][J]);                                      \
        if (has_next) {                                                      \
            fb[nxt][2 * (J - 8)] = rd_stage[b_rd + 64 * (2 * (J - 8))];        \
            fb[nxt][2 * (J - 8) + 1] = rd_stage[b_rd + 64 * (2 * (J - 8) + 1)]; \
        }                                                                    \
        if (has_load) { LOADSTMT; }                                          \
        XSMI_PIN();
        XSMI_SLOT(acc, fa[cur][2].x, 8, issue_b(3))
        XSMI_SLOT(acc2, fa[cur][2].y, 9, issue_b(4))
        XSMI_SLOT(acc, fa[cur][2].z, 10, issue_b(5))
        XSMI_SLOT(acc2, fa[cur][2].w, 11, issue_b(6))
        XSMI_SLOT(acc, fa[cur][3].x, 12, issue_b(7))
        XSMI_SLOT(acc2, fa[cur][3].y, 13, issue_a(0))
        XSMI_SLOT(acc, fa[cur][3].z, 14, issue_a(1))
        XSMI_SLOT(acc2, fa[cur][3].w, 15, issue_advance())
#undef XSMI_SLOT
        if (has_next) rd_advance();
    };

    // prologue: chunks 0..D-1 in flight, fragments of chunk 0 in registers, then chunk D
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (d < iters) issue_all();
    if (iters > 0) {
        if (D <= iters) xsmi::wait_vmcnt<(D - 1) * LOADS_PER_CHUNK>();
        else xsmi::wait_vmcnt<0>();
        xsmi::block_barrier();
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) fa[0][q4] = *reinterpret_cast<const float4 *>(rd_stage + a_rd + 256 * q4);
#pragma unroll
        for (int j = 0; j < 16; ++j) fb[0][j] = rd_stage[b_rd + 64 * j];
        rd_advance();
        if (D < iters) issue_all();
    }
    {
        using T0 = std::integral_constant<int, 0>;
        using T1 = std::integral_constant<int, 1>;
        int it = 0;
        const int n_steady = iters - 1 - D;           // iterations whose next chunk and next load both exist
        for (; it + 1 < n_steady; it += 2) {
            body(T0{}, std::true_type{}, it);
            body(T1{}, std::true_type{}, it + 1);
        }
        for (; it < iters; it += 2) {
            body(T0{}, std::false_type{}, it);
            if (it + 1 < iters) body(T1{}, std::false_type{}, it + 1);
        }
    }
#undef XSMI_MFMA
#undef XSMI_PIN

    acc += acc2;

    // ---- epilogue ----
    xsmi::store_block_32x32(acc, p, p.out, p.out_bytes, p.mask, p.bias ? &s_bias[0] : nullptr, p.relu, p.accumulate, rowtile * TM, TM,
                            wr * 32, m0 + wc * 32, lane, p.zfill);
}

// Persistent form of the kernel above (same tile, same loop body, 2 stages).  A launch has at most
// four workgroups per CU and every workgroup walks a sequence of tiles: the loads of a tile's first
// chunks are issued while the previous tile's last chunks multiply, and a tile's output stores
// drain while the next tile multiplies, so a CU's matrix pipes do not idle while a finished
// workgroup is replaced.  Tiles are split into eight contiguous ranges, one per XCD (workgroup
// b runs on XCD b % 8); a workgroup's first two tiles are fixed (slot, slot + P with P workgroups
// per XCD) and the rest come from its XCD's counter, fetched one tile ahead of use.  Requires an
// even chunk count >= 4 per tile and at least 8 tiles.
__global__ void __launch_bounds__(256) tap_igemm_f32_persist_kernel(TapParams p) {
    constexpr int STAGES = 2;
    __shared__ __attribute__((aligned(16))) float smem[STAGES][STAGE_FLOATS];
    __shared__ uint32_t s_next;
    __shared__ __attribute__((aligned(16))) float s_bias[2][TM];    // bias of the current tile, alternating per tile

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, P = gridDim.x >> 3;
    const uint32_t tq = p.tiles >> 3, trem = p.tiles & 7u;
    const uint32_t t_start = xcd * tq + (xcd < trem ? xcd : trem), t_count = tq + (xcd < trem ? 1u : 0u);
    const int iters = p.TR * p.TS * p.nch;

    // tile -> (first pixel, row tile); row tiles of one pixel tile are neighbours
    auto decode = [&](uint32_t local, int &m0, int &rowtile) {
        const uint32_t L = t_start + local;
        const uint32_t mt = p.rowtiles == 1 ? L : L / (uint32_t)p.rowtiles;
        rowtile = p.rowtiles == 1 ? 0 : (int)(L - mt * (uint32_t)p.rowtiles);
        m0 = (int)mt * BP;
    };
    // gather role of a lane in a tile: pixel m0 + lane
    auto lane_geom = [&](int m0, int &iyb, int &ixb, int &nbase, bool &live) {
        iyb = 0; ixb = 0; nbase = 0;
        live = m0 + lane < p.M;
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
    };

    int cur_m0, cur_rowtile, nxt_m0 = 0, nxt_rowtile = 0;
    uint32_t nxt_local = slot + P;
    bool nxt_valid = nxt_local < t_count;
    decode(slot, cur_m0, cur_rowtile);
    int iyb, ixb, nbase, iyb_n = 0, ixb_n = 0, nbase_n = 0;
    bool live, live_n = false;
    lane_geom(cur_m0, iyb, ixb, nbase, live);
    if (nxt_valid) {
        decode(nxt_local, nxt_m0, nxt_rowtile);
        lane_geom(nxt_m0, iyb_n, ixb_n, nbase_n, live_n);
    }

    const xsmi::xsmi_int32x4 rin = xsmi::make_rsrc(p.in, p.in_bytes);
    const xsmi::xsmi_int32x4 rap = xsmi::make_rsrc(p.apk, p.apk_bytes);
    const uint32_t lds0 = (uint32_t)(uintptr_t)&smem[0][0];
    const uint32_t a_voff = (uint32_t)((2 * wave * 64 + lane) * 16);
    const uint32_t a_tile_bytes = (uint32_t)iters * (uint32_t)(TM * KC * 4);

    int r = 0, s = 0, cc = 0;
    uint32_t ld_stage = lds0;
    uint32_t ld_asoff = (uint32_t)cur_rowtile * a_tile_bytes;
    uint32_t ld_voff = 0, ld_soff = 0;
    auto issue_prep = [&]() {
        int iy = iyb + r * p.dstep, ix = ixb + s * p.dstep;
        bool ok = live && (unsigned)iy < (unsigned)p.IH && (unsigned)ix < (unsigned)p.IW;
        ld_voff = ok ? (uint32_t)((nbase + iy * p.IW + ix) * 4) : 0x80000000u;
        ld_soff = (uint32_t)(cc * KC + wave * 8) * p.plane_bytes;
    };
    auto issue_b = [&](int e) {
        xsmi::load_lds_b32(rin, ld_stage + (uint32_t)((2048 + (wave * 8 + e) * 64) * 4), ld_voff,
                           ld_soff + (uint32_t)e * p.plane_bytes);
    };
    auto issue_a = [&](int qa) {
        xsmi::load_lds_b128(rap, ld_stage + (uint32_t)((2 * wave + qa) * 1024), a_voff + (uint32_t)qa * 1024u, ld_asoff);
    };
    auto issue_advance = [&]() {
        ld_asoff += (uint32_t)(TM * KC * 4);
        ld_stage += (uint32_t)(STAGE_FLOATS * 4);
        if (ld_stage == lds0 + (uint32_t)(STAGES * STAGE_FLOATS * 4)) ld_stage = lds0;
        if (++cc == p.nch) {
            cc = 0;
            if (++s == p.TS) {
                s = 0;
                if (++r == p.TR) {               // the issue side moves on to the next tile
                    r = 0;
                    iyb = iyb_n; ixb = ixb_n; nbase = nbase_n; live = live_n;
                    ld_asoff = (uint32_t)nxt_rowtile * a_tile_bytes;
                }
            }
        }
    };
    auto issue_all = [&]() {
        issue_prep();
#pragma unroll
        for (int e = 0; e < 8; ++e) issue_b(e);
        issue_a(0);
        issue_a(1);
        issue_advance();
    };

    floatx16 acc = {0}, acc2 = {0};
    const int h = lane >> 5, l31 = lane & 31;
    const int wr = wave >> 1, wc = wave & 1;
    const int a_rd = (4 * h * 64 + wr * 32 + l31) * 4;
    const int b_rd = 2048 + 16 * h * 64 + wc * 32 + l31;

    float4 fa[2][4];
    float fb[2][16];
    const float *rd_stage = smem[0];
    auto rd_advance = [&]() {
        rd_stage += STAGE_FLOATS;
        if (rd_stage == smem[0] + STAGES * STAGE_FLOATS) rd_stage = smem[0];
    };
#define XSMI_MFMA(ACC, AV, BV) ACC = __builtin_amdgcn_mfma_f32_32x32x2f32(AV, BV, ACC, 0, 0, 0)
#define XSMI_PIN() __builtin_amdgcn_sched_barrier(0)
    auto body = [&](auto buf_tag, int) {
        constexpr int cur = decltype(buf_tag)::value;
        constexpr int nxt = cur ^ 1;
        constexpr bool has_next = true, has_load = true;
        XSMI_MFMA(acc, fa[cur][0].x, fb[cur][0]);
        XSMI_MFMA(acc2, fa[cur][0].y, fb[cur][1]);
        XSMI_MFMA(acc, fa[cur][0].z, fb[cur][2]);
        XSMI_MFMA(acc2, fa[cur][0].w, fb[cur][3]);
        XSMI_PIN();
        if (has_next) {
            xsmi::wait_vmcnt<0>();
            xsmi::block_barrier();
        }
        XSMI_PIN();
        XSMI_MFMA(acc, fa[cur][1].x, fb[cur][4]);
        if (has_next) fa[nxt][0] = *reinterpret_cast<const float4 *>(rd_stage + a_rd);
        if (has_load) issue_prep();
        XSMI_PIN();
        XSMI_MFMA(acc2, fa[cur][1].y, fb[cur][5]);
        if (has_next) fa[nxt][1] = *reinterpret_cast<const float4 *>(rd_stage + a_rd + 256);
        if (has_load) issue_b(0);
        XSMI_PIN();
        XSMI_MFMA(acc, fa[cur][1].z, fb[cur][6]);
        if (has_next) fa[nxt][2] = *reinterpret_cast<const float4 *>(rd_stage + a_rd + 512);
        if (has_load) issue_b(1);
        XSMI_PIN();
        XSMI_MFMA(acc2, fa[cur][1].w, fb[cur][7]);
        if (has_next) fa[nxt][3] = *reinterpret_cast<const float4 *>(rd_stage + a_rd + 768);
        if (has_load) issue_b(2);
        XSMI_PIN();
#define XSMI_SLOT(ACC, AV, J, LOADSTMT)                                      \
        XSMI_MFMA(ACC, AV, fb[cur][J]);                                      \
        if (has_next) {                                                      \
            fb[nxt][2 * (J - 8)] = rd_stage[b_rd + 64 * (2 * (J - 8))];        \
            fb[nxt][2 * (J - 8) + 1] = rd_stage[b_rd + 64 * (2 * (J - 8) + 1)]; \
        }                                                                    \
        if (has_load) { LOADSTMT; }                                          \
        XSMI_PIN();
        XSMI_SLOT(acc, fa[cur][2].x, 8, issue_b(3))
        XSMI_SLOT(acc2, fa[cur][2].y, 9, issue_b(4))
        XSMI_SLOT(acc, fa[cur][2].z, 10, issue_b(5))
        XSMI_SLOT(acc2, fa[cur][2].w, 11, issue_b(6))
        XSMI_SLOT(acc, fa[cur][3].x, 12, issue_b(7))
        XSMI_SLOT(acc2, fa[cur][3].y, 13, issue_a(0))
        XSMI_SLOT(acc, fa[cur][3].z, 14, issue_a(1))
        XSMI_SLOT(acc2, fa[cur][3].w, 15, issue_advance())
#undef XSMI_SLOT
        if (has_next) rd_advance();
    };

    // prologue of the first tile: chunk 0 landed and in registers, chunk 1 in flight
    issue_all();
    xsmi::wait_vmcnt<0>();
    xsmi::block_barrier();
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) fa[0][q4] = *reinterpret_cast<const float4 *>(rd_stage + a_rd + 256 * q4);
#pragma unroll
    for (int j = 0; j < 16; ++j) fb[0][j] = rd_stage[b_rd + 64 * j];
    rd_advance();
    issue_all();

    using T0 = std::integral_constant<int, 0>;
    using T1 = std::integral_constant<int, 1>;
    int bias_buf = 0;
    for (;;) {
        const bool last_tile = !nxt_valid;                    // uniform over the workgroup
        // one coalesced load of the tile's bias; the chunk loop's barriers publish it before the epilogue reads
        // it, and the buffer is rewritten only two tiles later
        if (p.bias && t < TM) s_bias[bias_buf][t] = cur_rowtile * TM + t < p.rows ? p.bias[cur_rowtile * TM + t] : 0.f;
        uint32_t fetched = 0;
        if (!last_tile && t == 0) fetched = atomicAdd(p.counters + xcd, 1u);   // tile after the next one
        // Every chunk runs the full body.  In a workgroup's last tile the two chunks "after the end" are
        // loaded from a dummy tile (no live pixel: the activation loads are all out of range and touch
        // no memory; the filter loads re-read row tile 0), and their fragments are never multiplied.
        for (int it = 0; it < iters; it += 2) {
            body(T0{}, it);
            body(T1{}, it + 1);
        }
        acc += acc2;

        // ---- epilogue ----
        xsmi::store_block_32x32(acc, p, p.out, p.out_bytes, p.mask, p.bias ? &s_bias[bias_buf][0] : nullptr, p.relu, p.accumulate,
                                cur_rowtile * TM, TM, wr * 32, cur_m0 + wc * 32, lane, p.zfill);
        if (last_tile) {
            xsmi::wait_vmcnt<0>();                            // the dummy chunk's loads target this workgroup's LDS
            break;
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) { acc[v] = 0.f; acc2[v] = 0.f; }
        bias_buf ^= 1;

        // the tile fetched at the top of this iteration becomes the next one; the issue side has
        // already moved into what was the next tile and now becomes the current one
        if (t == 0) s_next = 2u * P + fetched;
        asm volatile("" ::: "memory");                        // the LDS store stays ahead of the wait below
        xsmi::wait_lgkmcnt0();
        xsmi::block_barrier();
        const uint32_t nn = __builtin_amdgcn_readfirstlane(s_next);
        cur_m0 = nxt_m0; cur_rowtile = nxt_rowtile;
        nxt_local = nn;
        nxt_valid = nn < t_count;
        if (nxt_valid) {
            decode(nxt_local, nxt_m0, nxt_rowtile);
            lane_geom(nxt_m0, iyb_n, ixb_n, nbase_n, live_n);
        } else {
            nxt_rowtile = 0; live_n = false;                  // dummy tile
        }
    }
#undef XSMI_MFMA
#undef XSMI_PIN
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

// bf16 tile kernel: operands are rounded to bf16 on their way INTO the LDS, so a stage holds bf16 in the
// layout the matrix instruction consumes and every fragment is one 128-bit LDS read.
//   tile   64*WR rows x 64*WC pixels per 256-thread workgroup, a wave owns 64 x 64 (2 x 2 blocks of 32 x 32)
//   chunk  one tap x 32 channels = two v_mfma_f32_32x32x16_bf16 steps; step u, lane half h use channel group 2u + h
//   stage  A [4 groups][ROWS][8 bf16], B [4 groups][PIX][8 bf16]; three stages
// A is packed to bf16 in exactly that layout by tap_pack_bf16_kernel and arrives by LDS-direct loads.  B is
// gathered from the fp32 tensor into registers (a thread = one pixel, 8*k consecutive channels, so every
// wave-level load is 256 contiguous bytes), converted and written with 128-bit LDS stores.  While chunk i
// multiplies, chunk i+1 is converted and stored, B of chunk i+3 is requested into the register set that frees and A
// of chunk i+2 into the stage that chunk i-1 has left.  This is the forward's fallback when the workspace has no
// room for a channels-last copy, and the bf16 backward-data kernel.
template <int WR, int WC>
__global__ void __launch_bounds__(256) tap_bf16_tile_kernel(TapMulti mp) {
    static_assert(WR * WC == 4, "four waves");
    constexpr int ROWS = 64 * WR, PIX = 64 * WC;
    constexpr int GROUPS = 256 / PIX;                 // thread groups that split a chunk's 32 channels
    constexpr int CPT = KC / GROUPS;                  // channels per thread and chunk
    constexpr int A_BYTES = ROWS * 64, B_BYTES = PIX * 64, STAGE = A_BYTES + B_BYTES;
    constexpr int NLOADS = CPT + WR;                  // vector-memory loads per thread and chunk
    __shared__ __attribute__((aligned(16))) unsigned char smem[3 * STAGE];

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    uint32_t logical = xsmi::xcd_contiguous_id(blockIdx.x, gridDim.x);
    int ci = 0;
    while (ci + 1 < mp.ncls && logical >= mp.first[ci + 1]) ++ci;
    const TapParams &p = mp.cls[ci];
    logical -= mp.first[ci];
    const uint32_t nrt = (uint32_t)mp.rowtiles;       // ROWS-row tiles
    const int rowtile = nrt == 1 ? 0 : (int)(logical % nrt);
    const int m0 = (int)(nrt == 1 ? logical : logical / nrt) * PIX;

    // ---- gather role: pixel m0 + pl, channels grp*CPT .. grp*CPT + CPT-1 of each chunk ----
    const int pl = t & (PIX - 1);
    const int grp = __builtin_amdgcn_readfirstlane(t / PIX);
    int iyb = 0, ixb = 0, nbase = 0;
    const bool live = m0 + pl < p.M;
    if (live) {
        uint32_t m = (uint32_t)(m0 + pl);
        uint32_t q = xsmi::fdiv(m, p.dOX);
        int x = (int)m - (int)q * p.OX;
        uint32_t n = xsmi::fdiv(q, p.dOY);
        int y = (int)q - (int)n * p.OY;
        iyb = y * p.sy + p.dy0;
        ixb = x * p.sx + p.dx0;
        nbase = (int)n * p.in_n_stride;
    }
    __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc((void *)p.in, 0, (int)p.in_bytes, 0x00020000);
    const xsmi::xsmi_int32x4 rap = xsmi::make_rsrc(p.apk, p.apk_bytes);
    const uint32_t lds0 = (uint32_t)(uintptr_t)&smem[0];
    const int iters = p.TR * p.TS * p.nch;
    const uint32_t a_voff = (uint32_t)((wave * WR * 64 + lane) * 16);
    // loop-invariant parameters in registers (p is indexed by class, so the compiler would re-read them)
    const int dstep = p.dstep, IH = p.IH, IW = p.IW, nch = p.nch, TS = p.TS;
    const uint32_t plane_bytes = p.plane_bytes;

    // B runs three chunks ahead of the multiply (two register sets), A two chunks ahead (three LDS stages)
    int r = 0, s = 0, cc = 0;                          // position of the next B chunk to load
    uint32_t ld_asoff = (uint32_t)rowtile * (uint32_t)iters * (uint32_t)A_BYTES;
    float breg[2][CPT];
    auto load_b = [&](auto set_tag) {
        constexpr int set = decltype(set_tag)::value;
        int iy = iyb + r * dstep, ix = ixb + s * dstep;
        bool ok = live && (unsigned)iy < (unsigned)IH && (unsigned)ix < (unsigned)IW;
        const int voff = ok ? (nbase + iy * IW + ix) * 4 : (int)0x80000000u;
        const uint32_t soff = (uint32_t)(cc * KC + grp * CPT) * plane_bytes;
#pragma unroll
        for (int e = 0; e < CPT; ++e)
            breg[set][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rin, voff, (int)(soff + (uint32_t)e * plane_bytes), 0));
        if (++cc == nch) {
            cc = 0;
            if (++s == TS) { s = 0; ++r; }
        }
    };
    auto issue_a = [&](uint32_t stage) {               // this wave's WR KB of the next chunk's packed rows
#pragma unroll
        for (int qa = 0; qa < WR; ++qa)
            xsmi::load_lds_b128(rap, lds0 + stage + (uint32_t)((wave * WR + qa) * 1024), a_voff + (uint32_t)qa * 1024u, ld_asoff);
        ld_asoff += (uint32_t)A_BYTES;
    };
    auto store_b = [&](auto set_tag, uint32_t stage) {
        constexpr int set = decltype(set_tag)::value;
#pragma unroll
        for (int j = 0; j < CPT / 8; ++j) {
            bf16x8 v;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (__bf16)breg[set][8 * j + e];
            *reinterpret_cast<bf16x8 *>(smem + stage + A_BYTES + ((grp * (CPT / 8) + j) * PIX + pl) * 16) = v;
        }
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    const int h = lane >> 5, l31 = lane & 31;
    const int wr = wave / WC, wc = wave % WC;
    const int a_rd = (h * ROWS + wr * 64 + l31) * 16;                 // byte offset of group h, row block 0
    const int b_rd = A_BYTES + (h * PIX + wc * 64 + l31) * 16;
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;

    uint32_t st_cur = 0, st_nxt = STAGE, st_nx2 = 2 * STAGE;
    // prologue: chunk 0 in the LDS, B of chunks 1 and 2 and A of chunk 1 in flight (a class without taps has
    // no chunks and writes zeros).  Loads retire in order: B0 A0 B1 A1 B2.
    if (iters > 0) {
        load_b(S0{});
        issue_a(st_cur);
        if (iters > 1) {
            load_b(S1{});
            issue_a(st_nxt);
        }
        store_b(S0{}, st_cur);
        if (iters > 2) load_b(S0{});
        constexpr int two = NLOADS + CPT < 63 ? NLOADS + CPT : 63;   // the counter holds 63 at most
        if (iters > 2) xsmi::wait_vmcnt<two>();
        else if (iters > 1) xsmi::wait_vmcnt<NLOADS>();
        else xsmi::wait_vmcnt<0>();
        xsmi::wait_lgkmcnt0();
        xsmi::block_barrier();
    }

    // iteration `it` multiplies chunk it, moves chunk it+1 (register set (it+1) % 2) into the LDS, and issues
    // B of chunk it+3 into that set and A of chunk it+2 into the stage that chunk it-1 has left
    auto body = [&](auto next_set, int it) {
        bf16x8 fa[2][2], fb[2][2];                    // [step][block]
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[u][i] = *reinterpret_cast<const bf16x8 *>(smem + st_cur + a_rd + (2 * u * ROWS + 32 * i) * 16);
                fb[u][i] = *reinterpret_cast<const bf16x8 *>(smem + st_cur + b_rd + (2 * u * PIX + 32 * i) * 16);
            }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0][i], fb[0][j], acc[i][j], 0, 0, 0);
        if (it + 1 < iters) store_b(next_set, st_nxt);
        if (it + 3 < iters) load_b(next_set);
        if (it + 2 < iters) issue_a(st_nx2);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1][i], fb[1][j], acc[i][j], 0, 0, 0);
        if (it + 1 < iters) {
            // A of chunk it+1 has landed (only this iteration's loads may still be in flight); this wave's LDS
            // stores and fragment reads are done
            if (it + 3 < iters) xsmi::wait_vmcnt<NLOADS>();
            else if (it + 2 < iters) xsmi::wait_vmcnt<WR>();
            else xsmi::wait_vmcnt<0>();
            xsmi::wait_lgkmcnt0();
            xsmi::block_barrier();
        }
        const uint32_t tmp = st_cur;
        st_cur = st_nxt; st_nxt = st_nx2; st_nx2 = tmp;
    };
    for (int it = 0; it < iters; it += 2) {
        body(S1{}, it);
        if (it + 1 < iters) body(S0{}, it + 1);
    }

    // ---- epilogue: register v of lane l in block (i, j) = row 32i + 8*(v/4) + 4*(l/32) + v%4, pixel 32j + l%32 ----
    const int rbase = rowtile * ROWS + wr * 64 + 4 * h;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int m = m0 + wc * 64 + 32 * j + l31;
        if (m >= p.M) continue;
        uint32_t q = xsmi::fdiv((uint32_t)m, p.dOX);
        int x = m - (int)q * p.OX;
        uint32_t n = xsmi::fdiv(q, p.dOY);
        int y = (int)q - (int)n * p.OY;
        const long long pix_off = (long long)n * p.os_n + (long long)y * p.os_y + (long long)x * p.os_x + p.o_base;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                int row = rbase + 32 * i + 8 * (v >> 2) + (v & 3);
                if (row < p.rows) {
                    float val = acc[i][j][v];
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
}

// ---- bf16 forward on a channels-last copy ------------------------------------------------------------
// The fastest bf16 path first rewrites the activations as bf16 [N][H + 2 pad][W + 2 pad][CP] (CP = channels
// rounded up to a multiple of 8) with a materialised zero border.  Eight consecutive channels of a pixel are
// then 16 contiguous bytes, which is exactly one lane's operand of v_mfma_f32_32x32x16_bf16, so both operands
// go global -> LDS with 128-bit LDS-direct loads: no registers, no conversion and no validity test in the
// loop, a thread's pixel offset is fixed for the whole kernel and the (tap, channel) displacement is scalar.
// A vector-memory instruction occupies the CU's address unit for 16 cycles whatever its width, so the
// per-element dword gathers of the NCHW kernels (8-32 per thread and chunk) bound them; this form needs 4-5
// loads per wave and chunk.
//
// The reduction index is a list of octets, o = tap * (CP / 8) + channel octet; a chunk is four consecutive
// octets (group g = octet 4 * chunk + g).  With CP a multiple of 32 a chunk is 32 channels of one tap; with
// CP = 8 (5 to 8 channels) it is four consecutive taps.  A stem of at most 4 channels and a filter at most 8
// wide is copied with CP = 4 instead: 16 bytes are then two horizontally adjacent pixels, an octet is two
// adjacent taps x 4 channels, and a chunk is one whole filter row (four tap pairs) -- 6 of 8 reduction slots
// carry data for RGB instead of 3 of 8.
struct NhwcParams {
    const __bf16 *xp;
    const float *apk;     // bf16 [row tile][chunk][group 4][ROWS][8]
    const float *bias;
    float *out;
    uint8_t *mask;
    uint32_t xp_bytes, apk_bytes;
    int M, rows, nchunks;
    int R, S, C8;         // filter rows, taps per filter row, octets per tap
    uint32_t pix_bytes, tap_bytes, row_bytes;   // byte steps of the copy: next pixel, next tap, next filter row
    int Hp, Wp, sy, sx;
    int OY, OX;
    xsmi::FastDiv dOX, dOY;
    long long os_n, os_k;
    int relu;
    int rowtiles;
    uint32_t tiles;       // pixel tiles x row tiles
    // channels-last bf16 output instead of `out`: [N][OY + 2 ob][OX + 2 ob][ocp], only the interior is written
    __bf16 *out_cl;
    int ob, ocp;
};

// x fp32 [N][C][H][W] -> xp bf16 [N][Hp][Wp][CP]; a workgroup converts WS pixels of one padded row through an
// LDS tile.  Reading, a wave covers 64 >> wlog channels x (1 << wlog) pixels per step (runs of consecutive
// pixels of one channel); writing, 64 >> clog pixels x (1 << clog) channel pairs (runs of consecutive channels
// of one pixel): both sides move whole contiguous runs without an integer division.
__global__ void __launch_bounds__(256) nhwc_pad_bf16_kernel(const float *__restrict__ x, __bf16 *__restrict__ xp, int C, int H,
                                                             int W, int CP, int pad, int Hp, int Wp, int WS, int nseg,
                                                             int wlog, int clog) {
    extern __shared__ float tile[];                   // [C][WS | 1]
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    // consecutive rows of an image go to the same XCD: input rows are short unaligned runs, and neighbouring rows
    // share the memory blocks their ends straddle
    const uint32_t bid = xsmi::xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int seg = (int)(bid % (uint32_t)nseg);
    const int rowid = (int)(bid / (uint32_t)nseg);    // n * Hp + hp
    const int hp = rowid % Hp, n = rowid / Hp;
    const int ih = hp - pad;
    __bf16 *row = xp + (size_t)rowid * Wp * CP;
    if (ih < 0 || ih >= H) {                          // border row: zeros
        if ((CP & 7) == 0) {                          // rows are 16-byte multiples
            uint4 *r4 = reinterpret_cast<uint4 *>(row);
            const int n16 = Wp * CP / 8;
            for (int i = seg * 256 + t; i < n16; i += nseg * 256) r4[i] = make_uint4(0, 0, 0, 0);
        } else {
            uint32_t *r1 = reinterpret_cast<uint32_t *>(row);
            const int n4 = Wp * CP / 2;
            for (int i = seg * 256 + t; i < n4; i += nseg * 256) r1[i] = 0;
        }
        return;
    }
    const int w0 = seg * WS;
    const int wn = W - w0 < WS ? W - w0 : WS;
    const int stride = WS | 1;
    const size_t HW = (size_t)H * W;
    const float *src = x + (((size_t)n * C) * H + ih) * W + w0;
    {
        const int WL = 1 << wlog, cpw = 64 >> wlog;
        const int wl0 = lane & (WL - 1), cs = lane >> wlog;
        constexpr int U = 8;                          // loads in flight per thread
        for (int wl = wl0; wl < wn; wl += WL)
            for (int c0 = wave * cpw + cs; c0 < C; c0 += 4 * cpw * U) {
                float v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int c = c0 + u * 4 * cpw;
                    v[u] = c < C ? src[(size_t)c * HW + wl] : 0.f;
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int c = c0 + u * 4 * cpw;
                    if (c < C) tile[c * stride + wl] = v[u];
                }
            }
    }
    __syncthreads();
    {
        const int CP2 = CP / 2;
        const int CL = 1 << clog, ppw = 64 >> clog;
        const int c20 = lane & (CL - 1), ps = lane >> clog;
        uint32_t *dst = reinterpret_cast<uint32_t *>(row + (size_t)(pad + w0) * CP);
#pragma unroll 4
        for (int p0 = wave * ppw; p0 < wn; p0 += 4 * ppw) {
            const int wl = p0 + ps;
            if (wl < wn)
                for (int c2 = c20; c2 < CP2; c2 += CL) {
                    const int c = 2 * c2;
                    float v0 = c < C ? tile[c * stride + wl] : 0.f;
                    float v1 = c + 1 < C ? tile[(c + 1) * stride + wl] : 0.f;
                    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
                    bf16x2 pk;
                    pk[0] = (__bf16)v0; pk[1] = (__bf16)v1;
                    dst[wl * CP2 + c2] = __builtin_bit_cast(uint32_t, pk);
                }
        }
        // left and right border pixels of the row
        uint32_t *r32 = reinterpret_cast<uint32_t *>(row);
        if (seg == 0)
            for (int i = t; i < pad * CP2; i += 256) r32[i] = 0;
        if (seg == nseg - 1)
            for (int i = t; i < pad * CP2; i += 256) r32[(size_t)(pad + W) * CP2 + i] = 0;
    }
}

// The same copy for at most 4 channels (CP = 4): a thread converts one padded pixel, reads and writes are
// both runs of consecutive pixels, no LDS.  Block b serves columns 256 * (b % nwb) .. of padded row b / nwb
// (= n * Hp + hp); the grid is one-dimensional so that the row count is not bound by the 65535 limit of grid.y.
__global__ void __launch_bounds__(256) nhwc_pad_c4_kernel(const float *__restrict__ x, __bf16 *__restrict__ xp, int C, int H,
                                                           int W, int pad, int Hp, int Wp, int nwb) {
    const int rowid = (int)(blockIdx.x / (uint32_t)nwb);
    const int wp = (int)(blockIdx.x - (uint32_t)rowid * (uint32_t)nwb) * 256 + threadIdx.x;
    if (wp >= Wp) return;
    const int hp = rowid % Hp, n = rowid / Hp;
    const int ih = hp - pad, iw = wp - pad;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (ih >= 0 && ih < H && iw >= 0 && iw < W) {
        const float *src = x + (((size_t)n * C) * H + ih) * W + iw;
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (c < C) v[c] = src[(size_t)c * H * W];
    }
    bf16x4 pk;
#pragma unroll
    for (int c = 0; c < 4; ++c) pk[c] = (__bf16)v[c];
    reinterpret_cast<uint2 *>(xp)[(size_t)rowid * Wp + wp] = __builtin_bit_cast(uint2, pk);
}

// Filters for the channels-last kernel: bf16 [row tile][chunk][ROWS][4 slots][8], the LDS image of a stage's A
// part.  Octet g of a row sits in slot g ^ ((row >> 2) & 3) (see the kernel); zero where the octet or the
// channel does not exist.
__global__ void __launch_bounds__(256) tap_pack_oct_kernel(const float *__restrict__ w, __bf16 *__restrict__ apk, int rows, int C,
                                                            int R, int S, int C8, int nchunks, int rowtiles, int ROWS, int pair) {
    const size_t total = (size_t)rowtiles * nchunks * ROWS * 32;
    const int octets = pair ? R * 4 : R * S * C8;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        int e = (int)(i & 7);
        int slot = (int)((i >> 3) & 3);
        size_t rest = i >> 5;
        int rr = (int)(rest % ROWS);
        size_t cblk = rest / ROWS;
        int it = (int)(cblk % nchunks);
        int rt = (int)(cblk / nchunks);
        int g = slot ^ ((rr >> 2) & 3);
        int o = 4 * it + g;
        int tap, ch;
        bool ok = o < octets;
        if (pair) {                                   // chunk = filter row, group = tap pair, element = (tap, channel)
            const int sx = 2 * g + (e >> 2);
            tap = it * S + sx;
            ch = e & 3;
            ok = ok && sx < S;
        } else {
            tap = o / C8;
            ch = (o - tap * C8) * 8 + e;
        }
        int row = rt * ROWS + rr;
        float v = 0.f;
        if (row < rows && ok && ch < C) v = w[((size_t)row * C + ch) * R * S + tap];
        apk[i] = (__bf16)v;
    }
}

// A workgroup walks the tiles [wg * tiles / grid, (wg + 1) * tiles / grid) as ONE stream of chunks: the loads
// run three chunks ahead of the multiply across tile boundaries and a tile's output stores drain behind the
// next tile's MFMAs.  (Stores count in vmcnt like loads; the loop's waits stay correct with stores pending,
// because loads complete in order among themselves: they just wait a little longer at a tile boundary.)  The
// host currently launches one workgroup per tile.
template <int WR, int WC, bool STEM>
__global__ void __launch_bounds__(256, WR == 2 ? 3 : 2) tap_nhwc_bf16_kernel(NhwcParams p) {
    static_assert(WR * WC == 4, "four waves");
    constexpr int ROWS = 64 * WR, PIX = 64 * WC;
    constexpr int STAGES = 3;
    constexpr int NB = PIX / 64;                      // B loads per wave and chunk (16 pixels x 64 bytes each)
    constexpr int A_BYTES = ROWS * 64, B_BYTES = PIX * 64, STAGE = A_BYTES + B_BYTES;
    constexpr int NLOADS = NB + WR;
    // A stage holds A [ROWS][64 bytes] and B [PIX][64 bytes]: the chunk's four octets of a row or pixel, octet g
    // in 16-byte slot g ^ ((index >> 2) & 3).  A fragment read (32 consecutive rows or pixels, one octet) then
    // covers 256 consecutive bytes' worth of banks with every 16 lanes (the LDS serves 256 bytes per clock), and a B load (16 consecutive pixels x 4 slots, lane = pixel * 4 +
    // slot) reads 64 contiguous bytes per pixel and lands as one contiguous KB.
    __shared__ __attribute__((aligned(16))) unsigned char smem[STAGES * STAGE];
    __shared__ float s_bias[ROWS];                    // the current tile's bias, staged once per tile

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t wg = xsmi::xcd_contiguous_id(blockIdx.x, gridDim.x);
    // tiles [tile_begin, tile_end) of the launch's p.tiles, row tile fastest
    const uint32_t tile_begin = (uint32_t)(((uint64_t)wg * p.tiles) / gridDim.x);
    const uint32_t tile_end = (uint32_t)(((uint64_t)(wg + 1) * p.tiles) / gridDim.x);
    const uint32_t nrt = (uint32_t)p.rowtiles;
    const int S = p.S, R = p.R, C8 = p.C8, Wp = p.Wp;
    const uint32_t row_bytes = p.row_bytes, tap_bytes = p.tap_bytes;
    const int iters = p.nchunks;
    const int total = (int)(tile_end - tile_begin) * iters;       // chunks of this workgroup's stream

    const xsmi::xsmi_int32x4 rin = xsmi::make_rsrc(p.xp, p.xp_bytes);
    const xsmi::xsmi_int32x4 rap = xsmi::make_rsrc(p.apk, p.apk_bytes);
    const uint32_t lds0 = (uint32_t)(uintptr_t)&smem[0];
    const uint32_t a_voff = (uint32_t)((wave * WR * 64 + lane) * 16);

    // ---- issue side: tile i_tile, chunk i_chunk; this lane's pixel and octet for each of its NB loads ----
    uint32_t i_tile = tile_begin;
    int i_chunk = 0;
    uint32_t voff[NB];                                // byte offset of the lane's pixel (+ its octet when not STEM)
    int oct[NB];                                      // the lane's octet of a chunk
    uint32_t ld_asoff = 0, ld_stage = 0;
    int r = 0, s = 0, c8 = 0;                          // chunk position when a chunk is one tap's 4 octets
    int rj[NB], sj[NB];                                // per lane: tap position when an octet is a whole tap
#pragma unroll
    for (int j = 0; j < NB; ++j) oct[j] = (lane & 3) ^ ((((wave * NB + j) * 16 + (lane >> 2)) >> 2) & 3);
    auto issue_tile = [&]() {                          // set the issue side up for tile i_tile
        const uint32_t mt = nrt == 1 ? i_tile : i_tile / nrt;
        const int rowtile = nrt == 1 ? 0 : (int)(i_tile - mt * nrt);
        const int m0 = (int)mt * PIX;
        ld_asoff = (uint32_t)rowtile * (uint32_t)iters * (uint32_t)A_BYTES;
        r = 0; s = 0; c8 = 0;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int m = m0 + (wave * NB + j) * 16 + (lane >> 2);
            voff[j] = 0x80000000u;                    // pixels beyond M read zeros
            if (m < p.M) {
                uint32_t q = xsmi::fdiv((uint32_t)m, p.dOX);
                int x = m - (int)q * p.OX;
                uint32_t n = xsmi::fdiv(q, p.dOY);
                int y = (int)q - (int)n * p.OY;
                voff[j] = (uint32_t)(((int)n * p.Hp + y * p.sy) * Wp + x * p.sx) * p.pix_bytes + (STEM ? 0u : (uint32_t)oct[j] * 16u);
            }
            if (STEM) {
                rj[j] = oct[j] / S;
                sj[j] = oct[j] - rj[j] * S;
            }
        }
    };
    auto issue = [&]() {
        // a chunk past the filter (the chunk count is rounded up to even) meets zero rows of A: re-read tap 0
        const uint32_t soff = (STEM || r >= R) ? 0u : (uint32_t)r * row_bytes + (uint32_t)s * tap_bytes + (uint32_t)c8 * 16u;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            uint32_t vo = voff[j];
            if (STEM) {
                // taps past the filter meet zero rows of A: read zeros
                vo = rj[j] < R ? vo + (uint32_t)(rj[j] * Wp + sj[j]) * 16u : 0x80000000u;
                sj[j] += 4;
                while (sj[j] >= S) { sj[j] -= S; ++rj[j]; }
            }
            xsmi::load_lds_b128(rin, lds0 + ld_stage + (uint32_t)(A_BYTES + (wave * NB + j) * 1024), vo, soff);
        }
#pragma unroll
        for (int qa = 0; qa < WR; ++qa)
            xsmi::load_lds_b128(rap, lds0 + ld_stage + (uint32_t)((wave * WR + qa) * 1024), a_voff + (uint32_t)qa * 1024u, ld_asoff);
        ld_asoff += (uint32_t)A_BYTES;
        ld_stage += (uint32_t)STAGE;
        if (ld_stage == (uint32_t)(STAGES * STAGE)) ld_stage = 0;
        if (!STEM) {
            c8 += 4;
            if (c8 == C8) {
                c8 = 0;
                if (++s == S) { s = 0; ++r; }
            }
        }
        if (++i_chunk == iters) {
            i_chunk = 0;
            if (++i_tile < tile_end) issue_tile();
        }
    };

    // ---- multiply side ----
    floatx16 acc[2][2];
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    };
    zero_acc();
    const int h = lane >> 5, l31 = lane & 31;
    const int wr = wave / WC, wc = wave % WC;
    // step u, lane half h read octet 2u + h: slot (2u) ^ xs with xs = h ^ ((l31 >> 2) & 3)
    const int xs = h ^ ((l31 >> 2) & 3);
    const int a_rd = (wr * 64 + l31) * 64;
    const int b_rd = A_BYTES + (wc * 64 + l31) * 64;
    uint32_t c_tile = tile_begin;

    // register v of lane l in block (i, j) = row 32i + 8*(v/4) + 4*(l/32) + v%4, pixel 32j + l%32
    auto epilogue = [&]() {
        const uint32_t mt = nrt == 1 ? c_tile : c_tile / nrt;
        const int rowtile = nrt == 1 ? 0 : (int)(c_tile - mt * nrt);
        const int m0 = (int)mt * PIX;
        const int rbase = rowtile * ROWS + wr * 64 + 4 * h;
        // one coalesced load of the tile's bias instead of a dependent global load per output element; the
        // barrier also keeps a faster wave's next tile from overwriting it (a workgroup-uniform branch)
        if (p.bias) {
            if (t < ROWS) s_bias[t] = rowtile * ROWS + t < p.rows ? p.bias[rowtile * ROWS + t] : 0.f;
            __syncthreads();
        }
        const int lrow = wr * 64 + 4 * h;
        if (p.out_cl) {
            // A lane holds four consecutive filters (v % 4) of a pixel: one 8-byte store of four bf16.  The two lane
            // halves and the four register groups of a block cover 32 consecutive channels, 64 contiguous bytes.
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int m = m0 + wc * 64 + 32 * j + l31;
                if (m >= p.M) continue;
                uint32_t q = xsmi::fdiv((uint32_t)m, p.dOX);
                int x = m - (int)q * p.OX;
                uint32_t n = xsmi::fdiv(q, p.dOY);
                int y = (int)q - (int)n * p.OY;
                const size_t pix = ((size_t)((int)n * (p.OY + 2 * p.ob) + y + p.ob) * (size_t)(p.OX + 2 * p.ob) + (size_t)(x + p.ob)) *
                                   (size_t)p.ocp;
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq) {
                        const int row = rbase + 32 * i + 8 * gq;
                        if (row >= p.rows) continue;                 // rows is a multiple of 4 on this path
                        float v4[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            float val = acc[i][j][4 * gq + e];
                            if (p.bias) val += s_bias[lrow + 32 * i + 8 * gq + e];
                            if (p.relu) val = val > 0.f ? val : 0.f;
                            v4[e] = val;
                        }
                        bf16x4 o4;
                        o4[0] = (__bf16)v4[0]; o4[1] = (__bf16)v4[1]; o4[2] = (__bf16)v4[2]; o4[3] = (__bf16)v4[3];
                        *reinterpret_cast<bf16x4 *>(p.out_cl + pix + row) = o4;
                    }
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int m = m0 + wc * 64 + 32 * j + l31;
            if (m >= p.M) continue;
            uint32_t q = xsmi::fdiv((uint32_t)m, p.dOX);
            int x = m - (int)q * p.OX;
            uint32_t n = xsmi::fdiv(q, p.dOY);
            int y = (int)q - (int)n * p.OY;
            const long long pix_off = (long long)n * p.os_n + (long long)y * p.OX + x;
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int row = rbase + 32 * i + 8 * (v >> 2) + (v & 3);
                    if (row < p.rows) {
                        float val = acc[i][j][v];
                        if (p.bias) val += s_bias[lrow + 32 * i + 8 * (v >> 2) + (v & 3)];
                        long long o = pix_off + (long long)row * p.os_k;
                        if (p.relu) {
                            if (p.mask) p.mask[o] = val < 0.f ? 1 : 0;
                            val = val > 0.f ? val : 0.f;
                        }
                        p.out[o] = val;
                    }
                }
        }
    };

    // Software pipeline: the fragments of chunk g+1 are read while chunk g multiplies.  An iteration issues
    // the first half of chunk g's MFMAs, then (while they execute) waits for chunk g+1, crosses the barrier,
    // refills the stage that chunk g has left with chunk g+3 and reads chunk g+1's fragments, then issues
    // the second half.  Every wave has read all of chunk g before that barrier (its fragments were complete
    // before the first half), so three stages give a prefetch distance of three chunks.
    bf16x8 fa[2][2][2], fb[2][2][2];                  // [buffer][step][block]
    uint32_t rd_stage = 0;
    auto read_frags = [&](auto buf_tag) {
        constexpr int bf = decltype(buf_tag)::value;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[bf][u][i] = *reinterpret_cast<const bf16x8 *>(smem + rd_stage + a_rd + 2048 * i + ((2 * u) ^ xs) * 16);
                fb[bf][u][i] = *reinterpret_cast<const bf16x8 *>(smem + rd_stage + b_rd + 2048 * i + ((2 * u) ^ xs) * 16);
            }
        rd_stage += (uint32_t)STAGE;
        if (rd_stage == (uint32_t)(STAGES * STAGE)) rd_stage = 0;
    };
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    auto body = [&](auto cur_tag, auto nxt_tag, int g) {
        constexpr int cur = decltype(cur_tag)::value;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[cur][0][i], fb[cur][0][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (g + 1 < total) {
            if (g + 3 <= total) xsmi::wait_vmcnt<NLOADS>();         // chunk g+2 may still be in flight
            else xsmi::wait_vmcnt<0>();
            xsmi::wait_lgkmcnt0();
            xsmi::block_barrier();
            if (g + 3 < total) issue();
            read_frags(nxt_tag);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[cur][1][i], fb[cur][1][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    if (total > 0) {
        issue_tile();
        issue();
        issue();                                       // a tile has an even number of chunks, at least two
        xsmi::wait_vmcnt<NLOADS>();
        xsmi::block_barrier();
        if (total > 2) issue();
        read_frags(B0{});
    }
    int g = 0;
    for (; c_tile < tile_end; ++c_tile) {
        for (int it = 0; it < iters; it += 2, g += 2) {
            body(B0{}, B1{}, g);
            body(B1{}, B0{}, g + 1);
        }
        epilogue();
        zero_acc();
    }
}

// Packs A for the tap-major kernel.  mode 0 (forward): A[row][tap=(r,s)][ch] = w[row][ch][r][s].
// mode 1 (backward-data class): A[row=c][tap=(t,u)][ch=k] = w[k][c][r0 + sh*t][s0 + sw*u].
// One launch lays out the filter for every class of a pass; blocks [first[j], first[j+1]) serve job j.
struct PackJob {
    float *apk;
    uint32_t *counters;
    int TR, TS, r0, s0;
};
struct PackMulti {
    PackJob job[TAP_MAX_CLASSES];
    uint32_t first[TAP_MAX_CLASSES + 1];
    int njobs;
};
__global__ void __launch_bounds__(256) tap_pack_kernel(const float *__restrict__ w, PackMulti pm, int mode, int rows, int CH,
                                                        int R, int S, int sh, int sw, int rowtiles) {
    int ji = 0;
    while (ji + 1 < pm.njobs && blockIdx.x >= pm.first[ji + 1]) ++ji;
    const PackJob &j = pm.job[ji];
    const uint32_t blk = blockIdx.x - pm.first[ji], nblk = pm.first[ji + 1] - pm.first[ji];
    if (blk == 0 && threadIdx.x < 8) j.counters[threadIdx.x] = 0;   // tile counters of the persistent kernel
    float *__restrict__ apk = j.apk;
    const int TR = j.TR, TS = j.TS, r0 = j.r0, s0 = j.s0;
    const int nch = CH / KC;
    const int iters = TR * TS * nch;
    const size_t total = (size_t)rowtiles * iters * (TM * KC);
    for (size_t i = (size_t)blk * 256 + threadIdx.x; i < total; i += (size_t)nblk * 256) {
        int e = (int)(i & 3);
        int r64 = (int)((i >> 2) & 63);
        int q = (int)((i >> 8) & 7);
        size_t cblk = i >> 11;
        int it = (int)(cblk % iters);
        int rt = (int)(cblk / iters);
        int cc = it % nch, tap = it / nch;
        int tr = tap / TS, ts = tap % TS;
        int ch = cc * KC + q * 4 + e;
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

// The 3x3 stride-1 case of the layout above with wide accesses: a thread takes one row and the four channels of one
// quad, i.e. 36 floats of w (mode 0: one contiguous run, read as nine float4; mode 1: four runs of nine), and
// stores one float4 per tap; the lanes of a wavefront are consecutive rows, so every store instruction writes 1 KB
// of one tap's block.  Twelve times fewer cache-line requests than one float per thread.
__global__ void __launch_bounds__(64) tap_pack_3x3_kernel(const float *__restrict__ w, float *__restrict__ apk,
                                                            uint32_t *__restrict__ counters, int mode, int rows, int CH,
                                                            int rowtiles) {
    if (blockIdx.x == 0 && threadIdx.x < 8) counters[threadIdx.x] = 0;   // tile counters of the persistent kernel
    const int nch = CH / KC;
    const uint32_t i = blockIdx.x * 64u + threadIdx.x;         // one wavefront per block: 64 rows of one quad
    const int r64 = (int)(i & 63), q = (int)((i >> 6) & 7);
    const uint32_t cblk = i >> 9;
    const int cc = (int)(cblk % (uint32_t)nch), rt = (int)(cblk / (uint32_t)nch);
    const int ch0 = cc * KC + q * 4, row = rt * TM + r64;
    float v[4][9];
    if (row < rows) {
        if (mode == 0) {
            const float4 *src = reinterpret_cast<const float4 *>(w + ((size_t)row * CH + ch0) * 9);
            float buf[36];
#pragma unroll
            for (int u = 0; u < 9; ++u) *reinterpret_cast<float4 *>(buf + 4 * u) = src[u];
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int t = 0; t < 9; ++t) v[e][t] = buf[e * 9 + t];
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float *src = w + ((size_t)(ch0 + e) * rows + row) * 9;
#pragma unroll
                for (int t = 0; t < 9; ++t) v[e][t] = src[t];
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int t = 0; t < 9; ++t) v[e][t] = 0.f;
    }
    float *dst = apk + ((size_t)rt * 9 * nch + cc) * (TM * KC) + q * (TM * 4) + r64 * 4;
#pragma unroll
    for (int t = 0; t < 9; ++t)
        *reinterpret_cast<float4 *>(dst + (size_t)t * nch * (TM * KC)) = make_float4(v[0][t], v[1][t], v[2][t], v[3][t]);
}

// The same filters for tap_bf16_tile_kernel: bf16, [row tile][chunk][group 4][ROWS rows][8 channels], i.e. the
// LDS image of a stage's A part per (row tile, chunk).
__global__ void __launch_bounds__(256) tap_pack_bf16_kernel(const float *__restrict__ w, PackMulti pm, int mode, int rows, int CH,
                                                             int R, int S, int sh, int sw, int rowtiles, int ROWS) {
    int ji = 0;
    while (ji + 1 < pm.njobs && blockIdx.x >= pm.first[ji + 1]) ++ji;
    const PackJob &j = pm.job[ji];
    const uint32_t blk = blockIdx.x - pm.first[ji], nblk = pm.first[ji + 1] - pm.first[ji];
    if (blk == 0 && threadIdx.x < 8) j.counters[threadIdx.x] = 0;
    __bf16 *__restrict__ apk = reinterpret_cast<__bf16 *>(j.apk);
    const int TR = j.TR, TS = j.TS, r0 = j.r0, s0 = j.s0;
    const int nch = CH / KC;
    const int iters = TR * TS * nch;
    const size_t per_block = (size_t)ROWS * KC;
    const size_t total = (size_t)rowtiles * iters * per_block;
    for (size_t i = (size_t)blk * 256 + threadIdx.x; i < total; i += (size_t)nblk * 256) {
        int e = (int)(i & 7);
        size_t rest = i >> 3;
        int rr = (int)(rest % ROWS);
        rest /= ROWS;
        int g = (int)(rest & 3);
        size_t cblk = rest >> 2;
        int it = (int)(cblk % iters);
        int rt = (int)(cblk / iters);
        int cc = it % nch, tap = it / nch;
        int tr = tap / TS, ts = tap % TS;
        int ch = cc * KC + g * 8 + e;
        int row = rt * ROWS + rr;
        float v = 0.f;
        if (row < rows) {
            if (mode == 0)
                v = w[(((size_t)row * CH + ch) * R + tr) * S + ts];
            else
                v = w[(((size_t)ch * rows + row) * R + (r0 + sh * tr)) * S + (s0 + sw * ts)];
        }
        apk[i] = (__bf16)v;
    }
}

// Rows per tile of tap_bf16_tile_kernel for a layer with `rows` output rows; 0 without the bf16 option.
int bf16_tile_rows(int opts, int rows) {
    if (!(opts & 1)) return 0;
    return rows <= 64 ? 64 : 128;
}

void launch_tap(hipStream_t st, TapMulti mp, int opts) {
    const int bf16 = opts & 1, counters_zeroed = !(opts & 2);   // the pack kernel zeroes the tile counters
    const uint32_t tiles = mp.first[mp.ncls];
    if (tiles == 0) return;
    if (bf16) {
        // tiles are 64 x 256 (one row tile) or 128 x 128; mp was built for 64 x 64
        const int trows = bf16_tile_rows(opts, mp.cls[0].rows);
        TapMulti m2 = mp;
        m2.rowtiles = xsmi::ceil_div(mp.cls[0].rows, trows);
        const int pix = trows == 64 ? 256 : 128;
        uint32_t first = 0;
        for (int c = 0; c < mp.ncls; ++c) {
            m2.first[c] = first;
            first += (uint32_t)xsmi::ceil_div(mp.cls[c].M, pix) * (uint32_t)m2.rowtiles;
        }
        m2.first[mp.ncls] = first;
        if (first == 0) return;
        if (trows == 64) hipLaunchKernelGGL((tap_bf16_tile_kernel<1, 4>), dim3(first), dim3(256), 0, st, m2);
        else hipLaunchKernelGGL((tap_bf16_tile_kernel<2, 2>), dim3(first), dim3(256), 0, st, m2);
        return;
    }
    const int stages_env = (int)xsmi::option(xsmi::OPT_TAP_STAGES), persist = (int)xsmi::option(xsmi::OPT_TAP_PERSIST);
    // With at most one tile per CU a workgroup runs alone and the two-stage pipeline waits a full load
    // latency per chunk; a third stage in flight covers it (measured 104 -> 91 us on 32x512x7x7, 3x3).
    const int stages = stages_env ? stages_env : (tiles <= (uint32_t)xsmi::cu_count() ? 3 : TAP_STAGES);
    // Measured at steady clocks: with no more tiles than resident workgroups (one tile each, no tail
    // code) the persistent kernel wins by 1-4 %; with more tiles the hardware's own workgroup
    // hand-over is as fast as the in-kernel one, and the plain kernel's dynamic dispatch balances better.
    const uint32_t resident = (uint32_t)xsmi::cu_count() * 4u;          // four workgroups per CU fit (registers)
    if (mp.ncls == 1) {
        TapParams p = mp.cls[0];
        const int iters = p.TR * p.TS * p.nch;
        if (persist && stages == 2 && iters >= 4 && (iters & 1) == 0 && tiles >= 16 &&
            (tiles <= resident || (persist > 1 && counters_zeroed))) {
            uint32_t g = tiles < resident ? tiles : resident;
            g &= ~7u;
            p.tiles = tiles;
            p.rowtiles = mp.rowtiles;
            hipLaunchKernelGGL(tap_igemm_f32_persist_kernel, dim3(g), dim3(256), 0, st, p);
            return;
        }
    }
    if (stages == 2) hipLaunchKernelGGL(tap_igemm_f32_kernel<2>, dim3(tiles), dim3(256), 0, st, mp);
    else hipLaunchKernelGGL(tap_igemm_f32_kernel<3>, dim3(tiles), dim3(256), 0, st, mp);
}

// packed filter + 256 bytes that hold the persistent kernel's eight tile counters
size_t tap_pack_bytes(int rows, int CH, int taps) {
    return xsmi::align_up((size_t)xsmi::ceil_div(rows, TM) * taps * (CH / KC) * TM * KC * sizeof(float), 256) + 256;
}
uint32_t *tap_counters(float *apk, size_t pack_bytes) { return (uint32_t *)((char *)apk + pack_bytes - 256); }

struct PackSpec { float *apk; int TR, TS, r0, s0; };

int launch_pack(hipStream_t st, const float *w, const PackSpec *specs, int nspecs, int mode, int rows, int CH, int R, int S,
                int sh, int sw, int opts) {
    const int trows = bf16_tile_rows(opts, rows);
    const int rowtiles = xsmi::ceil_div(rows, trows ? trows : TM);
    PackMulti pm;
    pm.njobs = 0;
    uint32_t blocks = 0;
    for (int i = 0; i < nspecs; ++i) {
        const PackSpec &sp = specs[i];
        size_t total = (size_t)rowtiles * sp.TR * sp.TS * (CH / KC) * (trows ? trows : TM) * KC;
        uint32_t nb = (uint32_t)((total + 255) / 256);
        if (nb > 2048) nb = 2048;
        if (nb == 0) nb = 1;                      // a class without taps still gets its counters cleared
        PackJob &j = pm.job[pm.njobs];
        j.apk = sp.apk; j.counters = tap_counters(sp.apk, tap_pack_bytes(rows, CH, sp.TR * sp.TS));
        j.TR = sp.TR; j.TS = sp.TS; j.r0 = sp.r0; j.s0 = sp.s0;
        pm.first[pm.njobs] = blocks;
        blocks += nb;
        ++pm.njobs;
    }
    if (pm.njobs == 0) return XSMI_OK;
    pm.first[pm.njobs] = blocks;
    if (!trows && nspecs == 1 && R == 3 && S == 3 && sh == 1 && sw == 1 && specs[0].TR == 3 && specs[0].TS == 3 &&
        ((uintptr_t)w & 15) == 0 && (size_t)rows * CH >= 65536) {
        // whole 3x3 filters of 2.4 MB and more (smaller ones are bound by the launch, not by the gather)
        const uint32_t nb = (uint32_t)(rowtiles * (CH / KC) * 8);
        hipLaunchKernelGGL(tap_pack_3x3_kernel, dim3(nb), dim3(64), 0, st, w, pm.job[0].apk, pm.job[0].counters, mode, rows,
                           CH, rowtiles);
        XSMI_LAUNCH_CHECK("tap_pack_3x3_kernel");
        return XSMI_OK;
    }
    if (trows)
        hipLaunchKernelGGL(tap_pack_bf16_kernel, dim3(blocks), dim3(256), 0, st, w, pm, mode, rows, CH, R, S, sh, sw, rowtiles, trows);
    else
        hipLaunchKernelGGL(tap_pack_kernel, dim3(blocks), dim3(256), 0, st, w, pm, mode, rows, CH, R, S, sh, sw, rowtiles);
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
                 int K, int R, int S, int sh, int sw, int pad, int OH, int OW, int relu, int opts, void *workspace) {
    hipStream_t st = stream();
    float *apk = (float *)workspace;
    if (!(opts & 2)) {                       // bit 1: the workspace still holds this filter's packed form
        PackSpec spec = {apk, R, S, 0, 0};
        int rc = launch_pack(st, w, &spec, 1, 0, K, C, R, S, 1, 1, opts);
        if (rc) return rc;
    }
    if (opts & 4) return XSMI_OK;            // bit 2: lay the filter out and stop
    TapParams p;
    p.in = x; p.apk = apk; p.bias = bias; p.out = y; p.mask = relu ? mask : nullptr;
    p.in_bytes = (uint32_t)((size_t)N * C * H * W * 4);
    p.out_bytes = (uint32_t)((size_t)N * K * OH * OW * 4);
    p.M = N * OH * OW; p.rows = K; p.nch = C / KC; p.TR = R; p.TS = S;
    p.dy0 = -pad; p.dx0 = -pad; p.dstep = 1;
    p.IH = H; p.IW = W; p.sy = sh; p.sx = sw;
    p.in_n_stride = C * H * W; p.plane_bytes = (uint32_t)(H * W * 4);
    p.OY = OH; p.OX = OW; p.dOX = make_fastdiv(OW); p.dOY = make_fastdiv(OH);
    p.os_n = (long long)K * OH * OW; p.os_k = (long long)OH * OW; p.o_base = 0; p.os_y = OW; p.os_x = 1;
    p.accumulate = 0; p.relu = relu; p.zfill = 0;
    p.tiles = 0; p.rowtiles = 0;
    p.apk_bytes = (uint32_t)tap_pack_bytes(K, C, R * S);
    p.counters = tap_counters(apk, tap_pack_bytes(K, C, R * S));
    TapMulti mp;
    mp.ncls = 1; mp.rowtiles = ceil_div(K, TM);
    mp.cls[0] = p;
    mp.first[0] = 0; mp.first[1] = (uint32_t)ceil_div(p.M, BP) * (uint32_t)mp.rowtiles;
    prof_begin();
    launch_tap(st, mp, opts);
    prof_end();
    XSMI_LAUNCH_CHECK("tap_igemm kernel");
    return XSMI_OK;
}

// ---- channels-last bf16 forward ----
// pair mode: at most 4 channels and a filter at most 8 wide (see the kernel's header)
static bool nhwc_pair(int C, int S) { return C <= 4 && S <= 8; }
static int nhwc_cp(int C, int S) { return nhwc_pair(C, S) ? 4 : (C + 7) / 8 * 8; }
static int nhwc_rows(int K) { return K <= 64 ? 64 : 128; }
static int nhwc_chunks(int C, int R, int S) {           // even: the kernel takes chunks in pairs
    const int octets = nhwc_pair(C, S) ? R * 4 : R * S * (nhwc_cp(C, S) / 8);
    return ceil_div(octets, 8) * 2;
}
static size_t nhwc_apk_bytes(int C, int K, int R, int S) {
    const int ROWS = nhwc_rows(K);
    return align_up((size_t)ceil_div(K, ROWS) * nhwc_chunks(C, R, S) * ROWS * 64, 256);
}
static size_t nhwc_xp_bytes(int N, int C, int H, int W, int S, int pad) {
    // one spare pixel: the last tap pair of a row may reach one pixel past the copy's end
    return align_up(((size_t)N * (H + 2 * pad) * (W + 2 * pad) + 1) * nhwc_cp(C, S) * 2, 256);
}

bool nhwc_fwd_ok(int N, int C, int H, int W, int K, int R, int S, int pad) {
    if (!(C % 32 == 0 || C <= 8)) return false;
    return nhwc_xp_bytes(N, C, H, W, S, pad) < ((size_t)1 << 31) && nhwc_apk_bytes(C, K, R, S) < ((size_t)1 << 32);
}

size_t nhwc_filter_ws_bytes(int C, int K, int R, int S) { return nhwc_apk_bytes(C, K, R, S); }

size_t nhwc_fwd_ws_bytes(int N, int C, int H, int W, int K, int R, int S, int pad) {
    return nhwc_apk_bytes(C, K, R, S) + nhwc_xp_bytes(N, C, H, W, S, pad);
}

// x_cl: the input as a channels-last bf16 tensor [N][H + 2 xb][W + 2 xb][C] with a zero border xb >= pad (C a multiple
// of 32), instead of x: no copy is made.  y_cl: the output goes to a channels-last bf16 tensor with border yb
// (K a multiple of 8; only its interior is written) instead of y.
int nhwc_conv_fwd(const float *x, const void *x_cl, int xb, const float *w, const float *bias, float *y, void *y_cl, int yb,
                  uint8_t *mask, int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad, int OH, int OW,
                  int relu, int opts, void *workspace) {
    hipStream_t st = stream();
    const bool pair = nhwc_pair(C, S);
    const int CP = nhwc_cp(C, S), C8 = pair ? 4 : CP / 8, ROWS = nhwc_rows(K);
    const int border = x_cl ? xb : pad;
    const int Hp = H + 2 * border, Wp = W + 2 * border;
    const int nchunks = nhwc_chunks(C, R, S), rowtiles = ceil_div(K, ROWS);
    __bf16 *apk = (__bf16 *)workspace;
    __bf16 *xp = (__bf16 *)((char *)workspace + nhwc_apk_bytes(C, K, R, S));
    // 3 x 3 stride-1 layers on large feature maps: the kernel that stages the input once for all nine taps
    // the first layer with channels-last output: its own kernel, filter resident in the LDS
    const bool stem_cl = pair && !x_cl && y_cl && stem_cl_ok(C, H, W, K, R, S, sh, sw, pad, OW, yb) &&
                         stem_cl_apk_bytes() <= nhwc_apk_bytes(C, K, R, S);
    const bool halo = !pair && (!y_cl || yb == 1) && halo_fwd_ok(C, H, W, K, R, S, sh, sw, pad, border) &&
                      halo_apk_bytes(C, K) <= nhwc_apk_bytes(C, K, R, S);
    if (!(opts & 2) && !halo && !stem_cl) {  // bit 1: the workspace still holds this filter's packed form
        const size_t total = (size_t)rowtiles * nchunks * ROWS * 32;
        int blocks = (int)((total + 255) / 256);
        if (blocks > 2048) blocks = 2048;
        hipLaunchKernelGGL(tap_pack_oct_kernel, dim3(blocks), dim3(256), 0, st, w, apk, K, C, R, S, C8, nchunks, rowtiles, ROWS,
                           pair ? 1 : 0);
        XSMI_LAUNCH_CHECK("tap_pack_oct_kernel");
    }
    prof_begin();
    if (x_cl) {
        // the window of output (0, 0) starts (xb - pad) rows and columns inside the border
        xp = (__bf16 *)x_cl + ((size_t)(xb - pad) * Wp + (size_t)(xb - pad)) * CP;
    } else if (CP == 4) {
        const int nwb = ceil_div(Wp, 256);
        hipLaunchKernelGGL(nhwc_pad_c4_kernel, dim3((unsigned)nwb * (unsigned)(N * Hp)), dim3(256), 0, st, x, xp, C, H,
                           W, pad, Hp, Wp, nwb);
        XSMI_LAUNCH_CHECK("nhwc_pad_c4_kernel");
    } else {
        // a workgroup converts WS pixels of one padded row through an LDS tile of C x (WS | 1) floats (<= 32 KB)
        int WS = 8192 / C - 1;
        if (WS > W) WS = W;
        if (WS < 1) WS = 1;
        const int nseg = ceil_div(W, WS);
        const size_t lds = (size_t)C * (WS | 1) * sizeof(float);
        int wlog = 0, clog = 0;
        while ((1 << wlog) < WS && wlog < 6) ++wlog;         // pixels per wave step when reading
        while ((1 << clog) < CP / 2 && clog < 6) ++clog;     // channel pairs per wave step when writing
        hipLaunchKernelGGL(nhwc_pad_bf16_kernel, dim3((unsigned)(N * Hp * nseg)), dim3(256), lds, st, x, xp, C, H, W, CP, pad, Hp,
                           Wp, WS, nseg, wlog, clog);
        XSMI_LAUNCH_CHECK("nhwc_pad_bf16_kernel");
    }
    if (stem_cl)
        return stem_cl_conv_fwd(xp, ((size_t)N * Hp * Wp + 1) * CP * 2, w, apk, bias, y_cl, N, C, H, W, K, R, S, pad, OH, OW, relu,
                                (opts & 2) != 0);
    if (halo) {
        return halo_conv_fwd(xp, (size_t)N * Hp * Wp * CP * 2, w, apk, bias, y, y_cl, mask, N, C, H, W, K, relu, (opts & 2) != 0);
    }
    NhwcParams p;
    p.xp = xp; p.apk = (const float *)apk; p.bias = bias; p.out = y; p.mask = relu ? mask : nullptr;
    p.xp_bytes = (uint32_t)((size_t)N * Hp * Wp * CP * 2);
    if (x_cl) p.xp_bytes -= (uint32_t)(((size_t)(xb - pad) * Wp + (size_t)(xb - pad)) * CP * 2);
    p.out_cl = (__bf16 *)y_cl; p.ob = yb; p.ocp = K;
    p.apk_bytes = (uint32_t)nhwc_apk_bytes(C, K, R, S);
    p.M = N * OH * OW; p.rows = K; p.nchunks = nchunks;
    p.R = R; p.S = pair ? 1 : S; p.C8 = C8; p.Hp = Hp; p.Wp = Wp; p.sy = sh; p.sx = sw;
    p.pix_bytes = (uint32_t)CP * 2u;
    p.tap_bytes = (uint32_t)CP * 2u;
    p.row_bytes = (uint32_t)Wp * (uint32_t)CP * 2u;
    p.OY = OH; p.OX = OW; p.dOX = make_fastdiv(OW); p.dOY = make_fastdiv(OH);
    p.os_n = (long long)K * OH * OW; p.os_k = (long long)OH * OW;
    p.relu = relu; p.rowtiles = rowtiles;
    const bool stem = C8 % 4 != 0;           // an octet list that does not split into whole-tap chunks (5 to 8 channels)
    p.tiles = (uint32_t)ceil_div(p.M, ROWS == 64 ? 256 : 128) * (uint32_t)rowtiles;
    // One tile per workgroup: the hardware's dispatcher balances the tail better than a static split of the
    // tiles over resident workgroups did (measured 83 against 91 us on 256x128x28x28, 3x3).
    const unsigned grid = p.tiles;
    if (ROWS == 64) {
        if (stem) hipLaunchKernelGGL((tap_nhwc_bf16_kernel<1, 4, true>), dim3(grid), dim3(256), 0, st, p);
        else hipLaunchKernelGGL((tap_nhwc_bf16_kernel<1, 4, false>), dim3(grid), dim3(256), 0, st, p);
    } else {
        if (stem) hipLaunchKernelGGL((tap_nhwc_bf16_kernel<2, 2, true>), dim3(grid), dim3(256), 0, st, p);
        else hipLaunchKernelGGL((tap_nhwc_bf16_kernel<2, 2, false>), dim3(grid), dim3(256), 0, st, p);
    }
    prof_end();
    XSMI_LAUNCH_CHECK("tap_nhwc_bf16_kernel");
    return XSMI_OK;
}

int tap_conv_bwd_data(const float *dy, const float *w, float *dx, int N, int C, int H, int W, int K, int R, int S, int sh,
                      int sw, int pad, int OH, int OW, int accumulate, int opts, void *workspace) {
    hipStream_t st = stream();
    char *ws = (char *)workspace;
    TapParams plans[64];
    PackSpec specs[64];
    int nplans = 0;
    for (int ph = 0; ph < sh; ++ph) {
        const int OYc = ph < H ? ceil_div(H - ph, sh) : 0;
        const int r0 = (ph + pad) % sh;
        const int T = r0 < R ? ceil_div(R - r0, sh) : 0;
        const int cy = (ph + pad - r0) / sh;
        for (int pw = 0; pw < sw; ++pw) {
            const int OXc = pw < W ? ceil_div(W - pw, sw) : 0;
            if (OYc == 0 || OXc == 0) continue;
            if (nplans == 64) return set_error("xsmi_conv2d_bwd_data: stride %dx%d has too many residue classes", sh, sw), XSMI_ERR_INVALID;
            const int s0 = (pw + pad) % sw;
            const int U = s0 < S ? ceil_div(S - s0, sw) : 0;
            const int cx = (pw + pad - s0) / sw;
            float *apk = (float *)ws;
            const size_t apk_bytes = tap_pack_bytes(C, K, T * U);
            ws += apk_bytes;
            specs[nplans] = PackSpec{apk, T, U, r0, s0};
            TapParams p;
            p.in = dy; p.apk = apk; p.bias = nullptr; p.out = dx; p.mask = nullptr;
            p.apk_bytes = (uint32_t)apk_bytes;
            p.counters = tap_counters(apk, apk_bytes);
            p.tiles = 0; p.rowtiles = 0;
            p.in_bytes = (uint32_t)((size_t)N * K * OH * OW * 4);
            p.out_bytes = (uint32_t)((size_t)N * C * H * W * 4);
            p.M = N * OYc * OXc; p.rows = C; p.nch = K / KC; p.TR = T; p.TS = U;
            p.dy0 = cy; p.dx0 = cx; p.dstep = -1;
            p.IH = OH; p.IW = OW; p.sy = 1; p.sx = 1;
            p.in_n_stride = K * OH * OW; p.plane_bytes = (uint32_t)(OH * OW * 4);
            p.OY = OYc; p.OX = OXc; p.dOX = make_fastdiv(OXc); p.dOY = make_fastdiv(OYc);
            p.os_n = (long long)C * H * W; p.os_k = (long long)H * W; p.o_base = (long long)ph * W + pw;
            p.os_y = sh * W; p.os_x = sw;
            p.accumulate = accumulate; p.relu = 0; p.zfill = 0;
            plans[nplans++] = p;
        }
    }
    // Residue classes no tap can reach (a stride larger than the filter: the 1 x 1 / 2 shortcuts leave three of four
    // classes empty) receive no gradient.  Accumulating, they are left alone.  Overwriting, the fp32 1 x 1 / 2 pass
    // over an even-sized tensor clears them from its own epilogue (every value is stored with its three zero
    // neighbours: one launch, every element written once); other geometries clear all of dx with one contiguous fill
    // first.  Only the classes with taps are computed, instead of tiles whose whole work is a strided store of zeros.
    {
        int kept = 0;
        for (int i = 0; i < nplans; ++i)
            if (plans[i].TR * plans[i].TS > 0) { plans[kept] = plans[i]; specs[kept] = specs[i]; ++kept; }
        if (kept < nplans) {
            const bool own_zeros = !(opts & 1) && !accumulate && kept == 1 && sh == 2 && sw == 2 && R == 1 && S == 1 &&
                                   pad == 0 && H % 2 == 0 && W % 2 == 0 && plans[0].o_base == 0;
            if (own_zeros) plans[0].zfill = 1;
            else if (!accumulate && !(opts & 4)) {
                int rc = xsmi_fill(dx, 0.f, (size_t)N * C * H * W);
                if (rc) return rc;
            }
            nplans = kept;
        }
    }
    // the residue classes of a pass run as one launch per TAP_MAX_CLASSES classes (stride 2: one launch)
    if (!(opts & 2)) {
        for (int i = 0; i < nplans; i += TAP_MAX_CLASSES) {
            const int n = nplans - i < TAP_MAX_CLASSES ? nplans - i : TAP_MAX_CLASSES;
            int rc = launch_pack(st, w, specs + i, n, 1, C, K, R, S, sh, sw, opts);
            if (rc) return rc;
        }
    }
    if (opts & 4) return XSMI_OK;            // bit 2: lay the filter out and stop
    prof_begin();
    for (int i = 0; i < nplans; i += TAP_MAX_CLASSES) {
        TapMulti mp;
        mp.ncls = nplans - i < TAP_MAX_CLASSES ? nplans - i : TAP_MAX_CLASSES;
        mp.rowtiles = ceil_div(C, TM);
        uint32_t first = 0;
        for (int c = 0; c < mp.ncls; ++c) {
            mp.cls[c] = plans[i + c];
            mp.first[c] = first;
            first += (uint32_t)ceil_div(plans[i + c].M, BP) * (uint32_t)mp.rowtiles;
        }
        mp.first[mp.ncls] = first;
        launch_tap(st, mp, opts);
        XSMI_LAUNCH_CHECK("tap_igemm kernel");
    }
    prof_end();
    return XSMI_OK;
}

}  // namespace xsmi
