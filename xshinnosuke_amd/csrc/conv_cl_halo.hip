// bf16 forward for 3 x 3, stride-1, pad-1 layers on a channels-last tensor: the input tile is staged ONCE per
// channel group with its halo, and all nine taps are multiplied from that one LDS image.
//
// The tap-major channels-last kernel (conv_tap.hip) moves, per tap and 32 channels, the whole B tile from the L2
// into the LDS again: 16-20 KB for 256 cycles of matrix work per wave, which is more than the L2 delivers, so
// that kernel runs at the L2's pace.  For a 3 x 3 filter the nine B tiles of a channel group are the same pixels
// shifted by (r, s).  Here the tile is a run of PIX consecutive positions of the zero-bordered tensor
// [N][H + 2][W + 2][C] taken as one long row of pixels: output position P needs the inputs P + (r - 1) Wp + (s - 1),
// so a run of PIX positions needs the PIX + 2 Wp + 2 pixels around it and the tap is nothing but an offset into
// that image.  Positions on the border are computed like any other and not stored (the border of the output
// stays zero): H W / ((H + 2)(W + 2)) of the work is useful, 93 % at 56 x 56, 87 % at 28 x 28, 77 % at 14 x 14 and 60 % at
// 7 x 7, which is why the host uses this kernel for feature maps of 14 x 14 and more only.
//
// LDS image of B: four planes (one per octet of the 32 channels), each [staged pixel][8 channels = 16 bytes], so a
// fragment read (32 consecutive pixels, one octet) is 512 contiguous bytes whatever the tap offset is: no bank
// conflicts and no swizzle.  The price is on the load side: a wave-load fills 64 consecutive pixels of one plane,
// 16 bytes out of each pixel's record, which the address unit serves at about half the rate of a contiguous
// kilobyte; but B is now loaded once per nine taps.  A (the filter) is packed by tap_pack_halo_kernel in exactly
// its LDS image, planes [octet][row][16 bytes], one block per (row tile, channel group, tap), and streams through
// a ring of three stages, two steps ahead.
//
// Pipeline: a step is one tap of one channel group (two MFMA k-steps of 16 channels).  While k-step 0 multiplies,
// the fragments of k-step 1 are read; while k-step 1 multiplies, the wave waits for the next step's A block (and,
// at a group's last tap, the next group's B image, which was issued over the taps before), crosses the workgroup
// barrier, refills the A stage the current step has left and reads the next step's first fragments.
#include "xsmi_internal.h"

#include <stdlib.h>
#include <type_traits>
#include <utility>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

constexpr int HALO_PIX = 256;                 // positions per tile
constexpr int HALO_PITCH = 384;               // staged pixels per plane: PIX + 2 Wp + 2 <= 384, i.e. Wp <= 63
constexpr int HALO_BLOADS = HALO_PITCH / 64;  // B wave-loads per plane and channel group

struct HaloParams {
    const __bf16 *xp;      // [N][Hp][Wp][C], zero border of one pixel
    const __bf16 *apk;     // [row tile][group][tap][octet 4][ROWS][8]
    const float *bias;
    float *out;            // fp32 [N][K][H][W], or
    uint8_t *mask;         // with out and relu: one byte per output, 1 where the pre-activation is negative
    __bf16 *out_cl;        // bf16 [N][Hp][Wp][K], interior only
    uint32_t xp_bytes, apk_bytes;
    uint32_t pixels;       // N * Hp * Wp
    uint32_t tiles;        // position tiles
    int rowtiles, groups;  // ceil(K / ROWS), C / 32
    int rows, C, Wp, Hp, H, W;
    xsmi::FastDiv dWp, dHp;
    int relu;
};

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

// WR x WC waves; a wave owns 64 rows x (PIX / WC) positions.  The grid holds as many workgroups as are resident at
// once (a multiple of the row-tile count) and workgroup w takes the work items w, w + grid, w + 2 grid, ... (item =
// position tile x row tile, row tile fastest, so a workgroup keeps its row tile) as ONE stream of steps: the next
// item's first operands are requested during the current item's last taps and an item's output stores drain behind
// the next item's MFMAs.  With one item per workgroup the first loads (about 2 us with nothing to overlap) and the
// drain of the stores cost as much as the 2-8 us of matrix work an item holds.
template <int WR, int WC>
__global__ void __launch_bounds__(256, 2) cl_halo_bf16_kernel(HaloParams p) {
    static_assert(WR * WC == 4, "four waves");
    constexpr int ROWS = 64 * WR, PIX = HALO_PIX, PIXW = PIX / WC, NBJ = PIXW / 32;
    constexpr int A_STAGE = ROWS * 64, B_STAGE = 4 * HALO_PITCH * 16;
    constexpr int NA = A_STAGE / 1024 / 4;            // A wave-loads per wave and step
    __shared__ __attribute__((aligned(16))) unsigned char s_b[2 * B_STAGE];
    __shared__ __attribute__((aligned(16))) unsigned char s_a[3 * A_STAGE];
    __shared__ __attribute__((aligned(16))) float s_bias[ROWS];

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t wg = blockIdx.x, grid = gridDim.x;
    const uint32_t nrt = (uint32_t)p.rowtiles;
    const int rowtile = (int)(wg % nrt);              // grid is a multiple of nrt
    const uint32_t tile0 = wg / nrt, tile_step = grid / nrt;
    const uint32_t items_all = p.tiles * nrt;
    const int n_items = wg < items_all ? (int)((items_all - wg + grid - 1) / grid) : 0;
    if (n_items == 0) return;
    const int Wp = p.Wp, NG = p.groups;
    const uint32_t cpb = (uint32_t)p.C * 2u;          // bytes of a pixel record
    const int total = NG * 9;                         // steps of an item

    const xsmi::xsmi_int32x4 rin = xsmi::make_rsrc(p.xp, p.xp_bytes);
    const xsmi::xsmi_int32x4 rap = xsmi::make_rsrc(p.apk, p.apk_bytes);
    const uint32_t lds_b = (uint32_t)(uintptr_t)&s_b[0];
    const uint32_t lds_a = (uint32_t)(uintptr_t)&s_a[0];

    // ---- issue side ----
    // B: wave w fills plane w (octet w of the group); load e covers staged pixels 64 e .. 64 e + 63, i.e. positions
    // tile * PIX + 64 e + lane of the bordered tensor.  Positions past the tensor's end read zeros.
    auto issue_b = [&](int e, uint32_t tile, int group, int image) {
        const uint32_t pos = tile * (uint32_t)PIX + (uint32_t)(64 * e + lane);
        const uint32_t voff = pos < p.pixels ? pos * cpb + (uint32_t)wave * 16u : 0x80000000u;
        xsmi::load_lds_b128(rin, lds_b + (uint32_t)(image * B_STAGE + (wave * HALO_PITCH + 64 * e) * 16), voff,
                            (uint32_t)group * 64u);
    };
    const uint32_t a_voff = (uint32_t)((wave * NA * 64 + lane) * 16);
    const uint32_t a_tile_off = (uint32_t)rowtile * (uint32_t)total * (uint32_t)A_STAGE;
    auto issue_a = [&](int stage_, uint32_t block_off) {          // one A block into ring stage stage_
#pragma unroll
        for (int q = 0; q < NA; ++q)
            xsmi::load_lds_b128(rap, lds_a + (uint32_t)(stage_ * A_STAGE + (wave * NA + q) * 1024), a_voff + (uint32_t)q * 1024u,
                                a_tile_off + block_off);
    };

    // ---- multiply side ----
    floatx16 acc[2][NBJ];
    const int h = lane >> 5, l31 = lane & 31;
    const int wr = wave / WC, wc = wave % WC;
    // lane half h takes octet 2 u + h of k-step u
    const int a_base = h * ROWS * 16 + (wr * 64 + l31) * 16;
    const int b_base = h * HALO_PITCH * 16 + (wc * PIXW + l31) * 16;
    bf16x8 fa[2][2], fb[2][NBJ];                      // [buffer][block]
    auto read_frags = [&](auto buf_tag, auto u_tag, int a_off, int b_off) {
        constexpr int bf = decltype(buf_tag)::value, u = decltype(u_tag)::value;
#pragma unroll
        for (int i = 0; i < 2; ++i)
            fa[bf][i] = *reinterpret_cast<const bf16x8 *>(s_a + a_off + a_base + u * 2 * ROWS * 16 + i * 512);
#pragma unroll
        for (int j = 0; j < NBJ; ++j)
            fb[bf][j] = *reinterpret_cast<const bf16x8 *>(s_b + b_off + b_base + u * 2 * HALO_PITCH * 16 + j * 512);
    };

    // register v of lane l in block (i, j): row 32 i + 8 (v / 4) + 4 (l / 32) + v % 4, position 32 j + l % 32
    const int rbase = rowtile * ROWS + wr * 64 + 4 * h;
    const int lrow = wr * 64 + 4 * h;
    const float floor_ = p.relu ? 0.f : -__builtin_inff();
    auto epilogue = [&](uint32_t tile) {
#pragma unroll
        for (int j = 0; j < NBJ; ++j) {
            // local position i is the bordered tensor's position tile * PIX + i + Wp + 1
            const uint32_t pos = tile * (uint32_t)PIX + (uint32_t)(wc * PIXW + 32 * j + l31 + Wp + 1);
            const uint32_t row_id = xsmi::fdiv(pos, p.dWp);          // n * Hp + yp
            const int xq = (int)(pos - row_id * (uint32_t)Wp);
            const uint32_t n = xsmi::fdiv(row_id, p.dHp);
            const int yq = (int)(row_id - n * (uint32_t)p.Hp);
            const bool inside = pos < p.pixels && xq >= 1 && xq <= p.W && yq >= 1 && yq <= p.H;
            if (p.out_cl) {
                // a lane holds four consecutive filters of a position: one 8-byte store each
                __bf16 *dst = p.out_cl + (size_t)pos * (size_t)p.rows;
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq) {
                        const int row = rbase + 32 * i + 8 * gq;
                        bf16x4 o4;
                        const float4 b4 = *reinterpret_cast<const float4 *>(&s_bias[lrow + 32 * i + 8 * gq]);
                        const float bv[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            float val = acc[i][j][4 * gq + e] + bv[e];
                            val = __builtin_fmaxf(val, floor_);
                            o4[e] = (__bf16)val;
                        }
                        if (inside && row < p.rows) *reinterpret_cast<bf16x4 *>(dst + row) = o4;   // rows is a multiple of 8 here
                    }
            } else if (inside) {
                const size_t o0 = ((size_t)n * p.rows * p.H + (size_t)(yq - 1)) * p.W + (size_t)(xq - 1);
                float *dst = p.out + o0;
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int row = rbase + 32 * i + 8 * (v >> 2) + (v & 3);
                        if (row >= p.rows) continue;
                        float val = acc[i][j][v];
                        if (p.bias) val += s_bias[lrow + 32 * i + 8 * (v >> 2) + (v & 3)];
                        if (p.relu) {
                            if (p.mask) p.mask[o0 + (size_t)row * p.H * p.W] = val < 0.f ? 1 : 0;
                            val = val > 0.f ? val : 0.f;
                        }
                        dst[(size_t)row * p.H * p.W] = val;
                    }
            }
        }
    };

    // prologue: the first item's first B image, A blocks 0..2
#pragma unroll
    for (int e = 0; e < HALO_BLOADS; ++e) issue_b(e, tile0, 0, 0);
    issue_a(0, 0u);
    issue_a(1, (uint32_t)A_STAGE);
    issue_a(2, 2u * (uint32_t)A_STAGE);
    if (t < ROWS) s_bias[t] = (p.bias && rowtile * ROWS + t < p.rows) ? p.bias[rowtile * ROWS + t] : 0.f;
    xsmi::wait_vmcnt<2 * NA>();
    xsmi::block_barrier();
    read_frags(IC<0>{}, IC<0>{}, 0, 0);

    // The stream is walked group by group (32 channels x 9 taps); inside a group everything that depends on the tap
    // (ring stage = tap % 3, the tap's offset into the B image, which B wave-load to request) is a compile-time
    // constant, and what depends on the group is formed once per group: the loop body has no bookkeeping of its own.
    const int groups_all = n_items * NG;
    const int wp16 = Wp * 16;
    int group = 0, image = 0;
    uint32_t tile = tile0;
    bool after_epilogue = false;
    for (int gi = 0; gi < groups_all; ++gi) {
        const bool last_group = gi + 1 == groups_all;
        const bool in_item = group + 1 < NG;
        const uint32_t next_tile = in_item ? tile : tile + tile_step;
        const int next_group = in_item ? group + 1 : 0;
        const int img_off = image * B_STAGE, next_img_off = B_STAGE - img_off;
        const uint32_t a_cur = (uint32_t)(group * 9) * (uint32_t)A_STAGE, a_next = (uint32_t)(next_group * 9) * (uint32_t)A_STAGE;
        static_for<9>([&](auto tap_c) {
            constexpr int tap = decltype(tap_c)::value, r = tap / 3, s = tap % 3;
            read_frags(IC<1>{}, IC<1>{}, (tap % 3) * A_STAGE, img_off + r * wp16 + s * 16);
            __builtin_amdgcn_sched_barrier(0);
            if (tap == 0 && group == 0) {
                // a tile's first MFMAs start from the constant zero: no pass over the accumulators between tiles
                floatx16 z;
#pragma unroll
                for (int v = 0; v < 16; ++v) z[v] = 0.f;
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < NBJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0][i], fb[0][j], z, 0, 0, 0);
            } else {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < NBJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0][i], fb[0][j], acc[i][j], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NBJ; ++j)
                acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1][0], fb[1][j], acc[0][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (tap < 8 || !last_group) {
                // The next step's A block was requested two steps ago and the block after it may still be in flight.  An
                // epilogue waits for everything requested before it issues its stores, so the two steps after it find
                // their A blocks complete and do not wait on the counter (which those stores still occupy).
                if (tap < 2) {
                    if (!after_epilogue) xsmi::wait_vmcnt<NA>();
                } else if (tap >= 7) {
                    if (last_group) xsmi::wait_vmcnt<0>(); else xsmi::wait_vmcnt<NA>();
                } else {
                    xsmi::wait_vmcnt<NA>();
                }
                xsmi::wait_lgkmcnt0();                               // this wave has read all of this step
                xsmi::block_barrier();
                // the next group's B image (of this item, or the first of the next item), one wave-load per step; the
                // other image is free since this group's first barrier
                if constexpr (tap >= 1 && tap <= HALO_BLOADS) {
                    if (!last_group) issue_b(tap - 1, next_tile, next_group, image ^ 1);
                }
                // A block of the step three ahead, into the stage this step has left
                if constexpr (tap + 3 < 9) {
                    issue_a(tap % 3, a_cur + (uint32_t)((tap + 3) * A_STAGE));
                } else {
                    if (!last_group) issue_a(tap % 3, a_next + (uint32_t)((tap + 3 - 9) * A_STAGE));
                }
                if constexpr (tap < 8) {
                    constexpr int r1 = (tap + 1) / 3, s1 = (tap + 1) % 3;
                    read_frags(IC<0>{}, IC<0>{}, ((tap + 1) % 3) * A_STAGE, img_off + r1 * wp16 + s1 * 16);
                } else {
                    read_frags(IC<0>{}, IC<0>{}, 0, next_img_off);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NBJ; ++j)
                acc[1][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1][1], fb[1][j], acc[1][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        after_epilogue = false;
        if (!in_item) {
            xsmi::wait_vmcnt<0>();                    // the two A blocks in flight have landed (see the wait above)
            epilogue(tile);
            tile += tile_step;
            group = 0;
            after_epilogue = p.out_cl != nullptr;
            if (!p.out_cl) xsmi::wait_vmcnt<0>();    // float32 output: let its many stores drain
        } else {
            ++group;
        }
        image ^= 1;
    }
}

// A in the kernel's LDS image: element ((((rt * NG + G) * 9 + tap) * 4 + o) * ROWS + row) * 8 + e
//   = w[rt * ROWS + row][32 G + 8 o + e][tap], zero for rows past K.
__global__ void __launch_bounds__(256) tap_pack_halo_kernel(const float *__restrict__ w, __bf16 *__restrict__ apk, int K, int C,
                                                             int ROWS, size_t total) {
    const int NG = C / 32;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const int e = (int)(i & 7);
        size_t rest = i >> 3;
        const int row = (int)(rest % ROWS); rest /= ROWS;
        const int o = (int)(rest & 3); rest >>= 2;
        const int tap = (int)(rest % 9); rest /= 9;
        const int G = (int)(rest % NG);
        const int rt = (int)(rest / NG);
        const int k = rt * ROWS + row, c = 32 * G + 8 * o + e;
        apk[i] = (__bf16)(k < K ? w[((size_t)k * C + c) * 9 + tap] : 0.f);
    }
}


// ---- first layer: at most 4 input channels, filter up to 7 x 8, stride 2, channels-last bf16 output ---------------
// The input is the zero-bordered bf16 copy [N][Hp][Wp][4] (8 bytes per pixel, Wp even), read as PAIRS of horizontally
// adjacent pixels: 16 bytes = two taps x 4 channels = one lane's MFMA operand.  With stride 2 the window of output
// x starts at pair x, so tap pair o of filter row r for output (y, x) is pair (2 y + r) * Wp/2 + x + o: for the 32
// consecutive outputs of an MFMA block that is 32 consecutive pairs, whatever r and o are.  A work item is two output
// rows (all of their columns, at most 128): its input is nine consecutive padded rows, one contiguous piece of memory,
// copied to the LDS as it is; the filter (R rows x 4 tap pairs x 64 filters x 16 bytes = 28 KB) stays in the LDS for the
// workgroup's whole life.  A persistent workgroup (two per CU) walks its items with the next item's rows requested
// while the current item multiplies, and needs ONE barrier per item (56 MFMAs per wave): nothing inside an item is
// produced by another wave.  The general channels-last kernel spends 21 other instructions per MFMA on this layer
// (per-lane tap bookkeeping for every load) and takes 245 us at N=256.
constexpr int STEM_ROWS_IN = 9;               // input rows of an item: 2 output rows x stride 2 + 7 - 2
constexpr int STEM_B_PAIRS = 1088;            // pixel pairs of an item's LDS image: 17 wave-loads of 64 pairs
struct StemParams {
    const __bf16 *xp;      // [N][Hp][Wp][4]
    const __bf16 *apk;     // [R][4 tap pairs][64 filters][8]
    const float *bias;
    __bf16 *out_cl;        // [N][OH + 2][OW + 2][K]
    uint32_t xp_bytes;
    int N, Hp, pitch;      // pitch = Wp / 2 pairs per padded row
    int OH, OW, K, relu;
    uint32_t items;        // N * ceil(OH / 2)
    xsmi::FastDiv dYP;     // by ceil(OH / 2)
};

template <int R>
__global__ void __launch_bounds__(256, 2) cl_stem_bf16_kernel(StemParams p) {
    constexpr int NLOADS = STEM_B_PAIRS / 64;        // B wave-loads (64 pairs each) per item, dealt round-robin to the waves
    constexpr int B_STAGE = STEM_B_PAIRS * 16;       // 9 rows x at most 115 pairs + the reach of the last block's junk columns
    constexpr int NIMG = 3;                          // images in flight: an item's rows are requested two items ahead
    __shared__ __attribute__((aligned(16))) unsigned char s_b[NIMG * B_STAGE];
    __shared__ __attribute__((aligned(16))) float s_bias[64];

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t wg = blockIdx.x, grid = gridDim.x;
    if (wg >= p.items) return;
    const int n_items = (int)((p.items - wg + grid - 1) / grid);
    const int pitch = p.pitch;
    const uint32_t ypairs = p.dYP.d;

    const xsmi::xsmi_int32x4 rin = xsmi::make_rsrc(p.xp, p.xp_bytes);
    const uint32_t lds_b = (uint32_t)(uintptr_t)&s_b[0];

    // an item's nine input rows: STEM_ROWS_IN * pitch * 16 contiguous bytes from row 2 * y0 of image n
    auto issue_b = [&](uint32_t item, int image) {
        const uint32_t n = xsmi::fdiv(item, p.dYP), yp = item - n * ypairs;
        const uint32_t base = ((n * (uint32_t)p.Hp + 2u * 2u * yp) * (uint32_t)pitch) * 16u;
        const uint32_t want = (uint32_t)(STEM_ROWS_IN * pitch) * 16u;
#pragma unroll
        for (int q0 = 0; q0 < NLOADS; q0 += 4) {
            const int q = q0 + wave;
            if (q >= NLOADS) break;
            const uint32_t off = (uint32_t)(q * 1024 + lane * 16);
            // bytes past the nine rows (or past the tensor) are junk columns' operands: zeros
            const uint32_t voff = (off < want && base + off < p.xp_bytes) ? base + off : 0x80000000u;
            xsmi::load_lds_b128(rin, lds_b + (uint32_t)(image * B_STAGE + q * 1024), voff, 0u);
        }
    };
    issue_b(wg, 0);
    if (n_items > 1) issue_b(wg + grid, 1);
    if (t < 64) s_bias[t] = (p.bias && t < p.K) ? p.bias[t] : 0.f;

    const int h = lane >> 5, l31 = lane & 31;
    const int q_row = wave >> 1, xh = wave & 1;       // this wave's output row of the pair and 64-column half
    // lane half h takes tap pair 2 u + h of k-step u
    const int b_base = ((2 * q_row) * pitch + 64 * xh + l31 + h) * 16;
    const int pitch16 = pitch * 16;
    const float floor_ = p.relu ? 0.f : -__builtin_inff();
    floatx16 acc[2][2];
    // The filter never changes: this lane's A operands of all 2 R k-steps (its row of both 32-row blocks, tap pair
    // 2 u + h of filter row r) stay in registers for the workgroup's whole life, 8 R registers, and the LDS serves
    // only the B fragments: two 128-bit reads per four MFMAs instead of four (a 64 x 64 wave tile that reads both
    // operands asks the LDS for 128 bytes per clock at full matrix rate, all it has).
    bf16x8 fa[2 * R][2];
#pragma unroll
    for (int ks = 0; ks < 2 * R; ++ks)
#pragma unroll
        for (int i = 0; i < 2; ++i)
            fa[ks][i] = *reinterpret_cast<const bf16x8 *>(p.apk + ((((ks >> 1) * 4 + 2 * (ks & 1) + h) * 64 + 32 * i + l31) * 8));
    bf16x8 fb[2][2];                                 // [buffer][block]
    auto read_frags = [&](auto buf_tag, auto ks_tag, int img_off) {
        constexpr int bf = decltype(buf_tag)::value, ks = decltype(ks_tag)::value, r = ks >> 1, u = ks & 1;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            fb[bf][j] = *reinterpret_cast<const bf16x8 *>(s_b + img_off + b_base + r * pitch16 + (32 * j + 2 * u) * 16);
    };

    if (n_items > 1) xsmi::wait_vmcnt<(NLOADS + 3) / 4>(); else xsmi::wait_vmcnt<0>();    // the filter and the first item's rows
    uint32_t item = wg;
    int image = 0;
    for (int it = 0; it < n_items; ++it, item += grid) {
        const int img_off = image * B_STAGE;
        // this item's rows have landed (waited for before the previous epilogue, or before the loop); everybody is done
        // with the other image
        __syncthreads();
        // the image two ahead is the one the previous item used: free since the barrier above
        if (it + 2 < n_items) issue_b(item + 2 * grid, image == 0 ? 2 : image - 1);
        read_frags(IC<0>{}, IC<0>{}, img_off);
        static_for<2 * R>([&](auto ks_c) {
            constexpr int ks = decltype(ks_c)::value;
            if constexpr (ks + 1 < 2 * R) read_frags(IC<(ks + 1) & 1>{}, IC<ks + 1>{}, img_off);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if constexpr (ks == 0) {
                        floatx16 z;
#pragma unroll
                        for (int v = 0; v < 16; ++v) z[v] = 0.f;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks][i], fb[ks & 1][j], z, 0, 0, 0);
                    } else {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks][i], fb[ks & 1][j], acc[i][j], 0, 0, 0);
                    }
                }
            __builtin_amdgcn_sched_barrier(0);
        });
        // The next item's rows were requested a whole item ago; waiting for them here, before this item's stores are
        // issued, keeps those stores out of the wait (they drain behind the next item's MFMAs).  Only the rows
        // requested at the top of this item (at most (NLOADS + 3) / 4 loads of this wave, a whole number less for the
        // waves that got one load fewer: the wait is then a little stricter than needed) may still be in flight.
        if (it + 2 < n_items) xsmi::wait_vmcnt<NLOADS / 4>(); else xsmi::wait_vmcnt<0>();
        // Epilogue through the LDS.  A lane holds four consecutive filters of one column, its neighbours hold columns a
        // whole 128-byte record apart: stored directly, every 8-byte store instruction touches 64 lines, and the
        // address unit needs as long for an item's 64 such stores as the matrix pipes for its MFMAs.  The item's own
        // input image is free now, and one output row (128 columns x 136 bytes: 8 bytes of padding spread the lanes'
        // 8-byte writes over all banks) fits it exactly; the row then leaves as 16-byte pieces in memory order.
        // register v of lane l in block (i, j) = filter 32 i + 8 (v / 4) + 4 (l / 32) + v % 4, column 32 j + l % 32
        const uint32_t n = xsmi::fdiv(item, p.dYP), yp = item - n * ypairs;
        constexpr int O_PITCH = 136;
        static_assert(128 * O_PITCH <= B_STAGE, "an output row fits an input image");
        unsigned char *const o_img = s_b + img_off;
        const int pieces = p.K >> 3;                   // 16-byte pieces of a column's record
        const int piece_shift = 31 - __builtin_clz(pieces);
        __syncthreads();                               // every wave has read this item's last fragments
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            if (q_row == q) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int x = 64 * xh + 32 * j + l31;
#pragma unroll
                    for (int i = 0; i < 2; ++i)
#pragma unroll
                        for (int gq = 0; gq < 4; ++gq) {
                            const int row = 32 * i + 8 * gq + 4 * h;
                            const float4 b4 = *reinterpret_cast<const float4 *>(&s_bias[row]);
                            const float bv[4] = {b4.x, b4.y, b4.z, b4.w};
                            bf16x4 o4;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                float val = acc[i][j][4 * gq + e] + bv[e];
                                val = __builtin_fmaxf(val, floor_);
                                o4[e] = (__bf16)val;
                            }
                            *reinterpret_cast<bf16x4 *>(o_img + x * O_PITCH + row * 2) = o4;
                        }
                }
            }
            __syncthreads();
            const int y = 2 * (int)yp + q;
            if (y < p.OH) {
                __bf16 *dst = p.out_cl + (((size_t)n * (size_t)(p.OH + 2) + (size_t)(y + 1)) * (size_t)(p.OW + 2) + 1) * (size_t)p.K;
                const int total = p.OW * pieces;
                for (int pc = t; pc < total; pc += 256) {
                    const int x = pc >> piece_shift, o8 = pc & (pieces - 1);     // K / 8 is a power of two (host check)
                    const uint4 v = *reinterpret_cast<const uint4 *>(o_img + x * O_PITCH + o8 * 16);
                    *reinterpret_cast<uint4 *>(dst + (size_t)pc * 8) = v;
                }
            }
            __syncthreads();                           // the image is rewritten by the other row, then by new input rows
        }
        image = image == NIMG - 1 ? 0 : image + 1;
    }
}

// A for the kernel above: element (((r * 4 + o) * 64 + k) * 8 + e) = w[k][e % 4][r][2 o + e / 4], zero past K, C or S.
__global__ void __launch_bounds__(256) tap_pack_stem_kernel(const float *__restrict__ w, __bf16 *__restrict__ apk, int K, int C,
                                                             int R, int S) {
    const int total = R * 4 * 64 * 8;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
        const int e = i & 7, k = (i >> 3) & 63, o = (i >> 9) & 3, r = i >> 11;
        const int c = e & 3, sx = 2 * o + (e >> 2);
        apk[i] = (__bf16)((k < K && c < C && sx < S) ? w[(((size_t)k * C + c) * R + r) * S + sx] : 0.f);
    }
}

}  // namespace

namespace xsmi {

// 3 x 3, stride 1, pad 1, channels a multiple of 32, a zero border of exactly one pixel, rows of at most 61 pixels,
// and feature maps large enough that the border positions are a small part of the work.
bool halo_fwd_ok(int C, int H, int W, int K, int R, int S, int sh, int sw, int pad, int border) {
    const int env = (int)xsmi::option(xsmi::OPT_CL_HALO);
    if (!env) return false;
    if (!(R == 3 && S == 3 && sh == 1 && sw == 1 && pad == 1 && border == 1)) return false;
    if (C % 32 != 0 || K % 8 != 0) return false;
    if (HALO_PIX + 2 * (W + 2) + 2 > HALO_PITCH) return false;
    return env >= 2 || (H >= 14 && W >= 14);
}

// First layer through cl_stem_bf16_kernel: at most 4 channels copied with a border of `pad` pixels (Wp even), filter
// 7 rows and at most 8 columns, stride 2 both ways, 8, 16, 32 or 64 filters, at most 128 output columns
// and an input row of at most 115 pixel pairs, channels-last output with a border of one.
bool stem_cl_ok(int C, int H, int W, int K, int R, int S, int sh, int sw, int pad, int OW, int y_border) {
    if (!xsmi::option(xsmi::OPT_CL_STEM)) return false;
    const int Wp = W + 2 * pad;
    return C <= 4 && R == 7 && S <= 8 && sh == 2 && sw == 2 && (K == 8 || K == 16 || K == 32 || K == 64) && y_border == 1 &&
           Wp % 2 == 0 &&
           OW <= 128 && (STEM_ROWS_IN - 1) * (Wp / 2) + 131 <= STEM_B_PAIRS && H + 2 * pad >= R;
}
size_t stem_cl_apk_bytes() { return 7 * 4 * 64 * 16; }

int stem_cl_conv_fwd(const void *xp, size_t xp_bytes, const float *w, void *apk, const float *bias, void *y_cl, int N, int C,
                     int H, int W, int K, int R, int S, int pad, int OH, int OW, int relu, bool packed) {
    hipStream_t st = stream();
    if (!packed) {
        hipLaunchKernelGGL(tap_pack_stem_kernel, dim3(14), dim3(256), 0, st, w, (__bf16 *)apk, K, C, R, S);
        XSMI_LAUNCH_CHECK("tap_pack_stem_kernel");
    }
    StemParams p;
    p.xp = (const __bf16 *)xp; p.apk = (const __bf16 *)apk; p.bias = bias; p.out_cl = (__bf16 *)y_cl;
    p.xp_bytes = (uint32_t)xp_bytes;
    p.N = N; p.Hp = H + 2 * pad; p.pitch = (W + 2 * pad) / 2;
    p.OH = OH; p.OW = OW; p.K = K; p.relu = relu;
    const int ypairs = ceil_div(OH, 2);
    p.items = (uint32_t)N * (uint32_t)ypairs;
    p.dYP = make_fastdiv(ypairs);
    unsigned grid = 2u * (unsigned)(cu_count() > 0 ? cu_count() : 256);
    if (grid > p.items) grid = p.items;
    hipLaunchKernelGGL(cl_stem_bf16_kernel<7>, dim3(grid), dim3(256), 0, st, p);
    prof_end();
    XSMI_LAUNCH_CHECK("cl_stem_bf16_kernel");
    return XSMI_OK;
}

size_t halo_apk_bytes(int C, int K) {
    const int ROWS = K <= 64 ? 64 : 128;
    return align_up((size_t)ceil_div(K, ROWS) * (C / 32) * 9 * ROWS * 64, 256);
}

// xp: the bordered channels-last input (border 1); apk: workspace for the packed filter (halo_apk_bytes);
// y (fp32 NCHW) or y_cl (bordered channels-last bf16, border 1) receives the result.
int halo_conv_fwd(const void *xp, size_t xp_bytes, const float *w, void *apk, const float *bias, float *y, void *y_cl,
                  uint8_t *mask, int N, int C, int H, int W, int K, int relu, bool packed) {
    hipStream_t st = stream();
    const int ROWS = K <= 64 ? 64 : 128;
    const int rowtiles = ceil_div(K, ROWS), NG = C / 32;
    const size_t apk_elems = (size_t)rowtiles * NG * 9 * ROWS * 32;
    if (!packed) {
        int blocks = (int)((apk_elems + 255) / 256);
        if (blocks > 2048) blocks = 2048;
        hipLaunchKernelGGL(tap_pack_halo_kernel, dim3(blocks), dim3(256), 0, st, w, (__bf16 *)apk, K, C, ROWS, apk_elems);
        XSMI_LAUNCH_CHECK("tap_pack_halo_kernel");
    }
    HaloParams p;
    p.xp = (const __bf16 *)xp; p.apk = (const __bf16 *)apk; p.bias = bias; p.out = y; p.out_cl = (__bf16 *)y_cl; p.mask = (relu && !y_cl) ? mask : nullptr;
    p.xp_bytes = (uint32_t)xp_bytes; p.apk_bytes = (uint32_t)(apk_elems * 2);
    p.Hp = H + 2; p.Wp = W + 2; p.H = H; p.W = W;
    p.pixels = (uint32_t)N * (uint32_t)p.Hp * (uint32_t)p.Wp;
    // local position i of tile t is position t * PIX + i + Wp + 1: the first Wp + 1 positions (border) are skipped
    const uint32_t positions = p.pixels > 2u * (uint32_t)(p.Wp + 1) ? p.pixels - 2u * (uint32_t)(p.Wp + 1) : 0u;
    p.tiles = (positions + HALO_PIX - 1) / HALO_PIX;
    p.rowtiles = rowtiles; p.groups = NG; p.rows = K; p.C = C;
    p.dWp = make_fastdiv(p.Wp); p.dHp = make_fastdiv(p.Hp);
    p.relu = relu;
    if (p.tiles == 0) return XSMI_OK;
    // as many workgroups as are resident at once (two per CU), a multiple of the row-tile count
    unsigned grid = 2u * (unsigned)(cu_count() > 0 ? cu_count() : 256);
    if (grid > p.tiles * (unsigned)rowtiles) grid = p.tiles * (unsigned)rowtiles;
    grid -= grid % (unsigned)rowtiles;
    if (grid == 0) grid = (unsigned)rowtiles;
    if (ROWS == 64) hipLaunchKernelGGL((cl_halo_bf16_kernel<1, 4>), dim3(grid), dim3(256), 0, st, p);
    else hipLaunchKernelGGL((cl_halo_bf16_kernel<2, 2>), dim3(grid), dim3(256), 0, st, p);
    prof_end();
    XSMI_LAUNCH_CHECK("cl_halo_bf16_kernel");
    return XSMI_OK;
}

}  // namespace xsmi
