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
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < NBJ; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    };
    zero_acc();
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
                            val = val > floor_ ? val : floor_;
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
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < NBJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0][i], fb[0][j], acc[i][j], 0, 0, 0);
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
            zero_acc();
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

}  // namespace

namespace xsmi {

// 3 x 3, stride 1, pad 1, channels a multiple of 32, a zero border of exactly one pixel, rows of at most 61 pixels,
// and feature maps large enough that the border positions are a small part of the work.
bool halo_fwd_ok(int C, int H, int W, int K, int R, int S, int sh, int sw, int pad, int border) {
    static int env = -1;
    if (env < 0) { const char *e = getenv("XSMI_CL_HALO"); env = e ? atoi(e) : 1; }
    if (!env) return false;
    if (!(R == 3 && S == 3 && sh == 1 && sw == 1 && pad == 1 && border == 1)) return false;
    if (C % 32 != 0 || K % 8 != 0) return false;
    if (HALO_PIX + 2 * (W + 2) + 2 > HALO_PITCH) return false;
    return env >= 2 || (H >= 14 && W >= 14);
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
