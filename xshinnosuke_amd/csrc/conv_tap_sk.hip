// Tap-major implicit-GEMM convolution (forward and backward-data), fp32 MFMA, with an even split of the launch's
// work over the resident workgroups.
//
// Same data path as conv_tap.hip (reduction index = (tap, channel); global -> LDS directly; zero border through the
// buffer range check; 64 x 64 outputs per workgroup, 32 x 32 per wave), but work is counted in chunks (one tap x 32
// channels of one tile; in the staged-row forms below one filter row x 16 channels): the launch has exactly as many workgroups as fit on
// the chip at once and workgroup g takes the contiguous range [g * U / G, (g + 1) * U / G) of the U chunks of all
// tiles, walking it as one software-pipelined stream.  Every compute unit therefore gets the same amount of matrix
// work whatever the tile count is (ResNet-18 at N=32 has 1.5 to 6.1 tiles per CU: up to a quarter of the machine
// idled in the last round of tiles).  A tile whose chunks are split between workgroups is finished by the workgroup
// that holds its first chunk: the others store their accumulators to the library's partial-tile area and raise a flag,
// the owner adds them in ascending chunk order and runs the epilogue.  The summation order is a function of the
// geometry and the grid size only: results are reproducible bit for bit, there are no float atomics.
//
// Forward progress: a workgroup waits only for workgroups with a higher logical id, and each of those stores its
// partial tile right after its first (at most one tile long) segment, before it can wait for anything itself.
// Workgroups start in id order, so whatever is resident either finishes or waits for something that has already
// started.  The wait is bounded all the same (spin_limit); when it runs out the workgroup sets the library's device
// error word and stores nothing more, and the host reports the launch as failed at its next check.
#include "conv_store.h"
#include <stdlib.h>
#include <string.h>
#include <type_traits>
#include <utility>

namespace {

using xsmi::floatx16;

constexpr int SK_MAX_CLASSES = 4;
constexpr int SK_MAX_GRID = 1024;           // upper bound of resident workgroups (flags and partial tiles are sized for it)
constexpr int SK_ROWS = 64, SK_PIX = 64, SK_KC = 32;      // outputs per workgroup, reduction channels per chunk

// One parameter set: the layer (forward) or one residue class of a strided backward-data pass.
struct SkClass {
    uint32_t apk_off;      // bytes from the common packed-filter base to this class's [rowtile][chunk][quad][row][4]
    int M, rows;
    int nch, TR, TS;       // channel chunks per tap, taps
    int dy0, dx0, dstep;   // input row for tap r: y * sy + dy0 + r * dstep
    int IH, IW, sy, sx;
    int in_n_stride;       // elements
    uint32_t plane_bytes;
    int OY, OX;
    xsmi::FastDiv dOX, dOY, dIT;
    long long os_n, os_k, o_base;
    int os_y, os_x;
    uint32_t first_unit;   // first chunk of the class in the launch's chunk numbering
    uint32_t iters;        // chunks per tile = TR * TS * nch
};

struct SkParams {
    SkClass cls[SK_MAX_CLASSES];
    uint32_t end_unit[SK_MAX_CLASSES];     // first_unit of the next class
    const float *in;
    const float *apk;
    const float *bias;
    float *out;
    uint8_t *mask;
    float *part;           // [grid][16 accumulator registers][256 threads]
    uint32_t *flags;       // [grid], zero between launches
    uint32_t *err;         // set (system scope) when a wait for a partial tile ran out
    uint32_t in_bytes, apk_bytes, out_bytes, part_bytes;
    uint32_t units;        // chunks of all tiles of all classes
    // Workgroup j of a grid of G takes the units [j * units / G, (j + 1) * units / G).  With units = upg * G + urem that
    // is j * upg + (j * urem) / G: 32-bit arithmetic with one multiply-high (j * urem < G * G), where the 64-bit
    // quotient costs the scalar unit some 250 instructions, twice when a workgroup starts and once or twice more where
    // its range ends, while every workgroup of the launch stands at its own end and the matrix pipes are idle.
    uint32_t upg, urem;
    xsmi::FastDiv dG;
    uint32_t spin_limit;   // polls of a flag before giving up; 0: every wait counts as run out (error-path tests)
    int ncls, rowtiles, accumulate, relu;
    // staged rows (one class; a unit is a filter row x 16 channels, the filter laid out per unit as three taps)
    int staged_rows;
    int out_rows;          // output rows of all images
    int run_slots;         // one-dword pieces: slots of a channel's run that a tile can need
    xsmi::FastDiv dPitch;  // by (output row length + zeros behind a row: 4, one-dword pieces: 1)
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

__device__ __forceinline__ float comp4(const float4 &v, int t) { return t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w; }

// Buffer accesses with a wave-uniform part of the address in a scalar register.  AGENT: the sc1 bit, i.e. the
// access goes past the caches that are not coherent across the chip's XCDs (partial tiles are written by one
// compute unit and read by another).
constexpr int AGENT = 16;
template <int AUX = 0>
__device__ __forceinline__ void buf_store(__amdgpu_buffer_rsrc_t r, float v, uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), r, (int)voff, (int)soff, AUX);
}
template <int AUX = 0>
__device__ __forceinline__ float buf_load(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, AUX));
}

// VEC = 1: a B wave-load is one channel x 64 pixels, any geometry.  VEC = 4 (launches of one class only): a B wave-load is four channels x 64 pixels, a lane fetching
// the 16 bytes of four consecutive pixels of one row (input walked with stride 1, rows a multiple of 4 pixels wide, taps
// that reach at most one column past a row end: the host checks) -- a quarter of the vector-memory instructions of the
// one-dword form.  A run that reaches one column past a row end is fetched as it lies, so the slot of the border
// column holds the neighbouring row's last or first value; the lane overwrites that slot with zero once the load has
// landed, between the wait for the loads and the workgroup barrier.
//
// VEC = 3 (launches of one class; 3 x 3 taps that shift the input by -1, 0, +1 columns over rows as wide as the
// output's, a multiple of four pixels and at least 20): the unit of work is one filter ROW x 16 channels.  The
// tile's input pixels of that row are staged once for the row's three taps, as one run per channel in which every
// image row is followed by four slots of zeros: a tap is then a shift of the fragment read by one slot, and the slot
// past either end of a row is a zero that the loads themselves wrote (the lanes of those slots fetch out of range).
// 16-byte loads, nothing to clear, a third of the activation traffic, one barrier per 24 MFMAs.
//
// VEC = 2: the same for rows of any width from two pixels on (14 x 14 and 7 x 7 feature maps), with one-dword pieces: a
// lane owns one slot of a run, every image row is followed by ONE slot of zeros, and a channel's run (at most 66
// slots plus one per row end inside the tile) takes two wave-loads, the second one mostly idle.
template <int VEC>
__global__ void __launch_bounds__(256, 3) tap_sk_f32_kernel(SkParams sp) {
    static_assert(VEC == 1 || VEC == 4 || VEC == 3 || VEC == 2, "B loads of one or four dwords per lane, or staged rows");
    constexpr bool ROW = VEC == 3 || VEC == 2;       // staged rows
    constexpr bool ROWD = VEC == 2;                  // ... with one-dword pieces
    constexpr int RPAD = ROWD ? 1 : 4;               // slots of zeros behind an image row = slots of a piece
    constexpr int ROWS = SK_ROWS, PIX = SK_PIX, KC = ROW ? 16 : SK_KC;
    constexpr int UTAPS = ROW ? 3 : 1;               // taps per unit of work
    constexpr int BPITCH = 128;                      // ROW: floats from one channel's run to the next (a run has 84)
    constexpr int WCn = PIX / 32;                    // waves along pixels (2 x 2 waves of 32 x 32)
    constexpr int RT = ROWS / 64, PT = PIX / 64;     // 64-row / 64-pixel blocks of the tile (units of one wave-load)
    constexpr int QUADS = KC / 4;                    // 16-byte channel groups of a chunk
    constexpr int GROUPS = KC / 8;
    // VEC = 4: a stage ends with two rows of 256 slots that take the zero writes of lanes whose run has no border column
    constexpr int SPARE_FLOATS = VEC == 4 ? 512 : 0;
    constexpr int A_FLOATS = ROWS * KC * UTAPS, B_FLOATS = ROW ? KC * BPITCH : PIX * KC;
    constexpr int STAGE_FLOATS = A_FLOATS + B_FLOATS + SPARE_FLOATS;
    constexpr int NA = UTAPS * QUADS * RT / 4;       // A wave-loads (64 rows x 16 bytes) per wave and chunk
    constexpr int NB = KC * PT / 4;                  // B wave-loads (64 pixels of one channel) per wave and chunk
    constexpr int NBW = ROWD ? 8 : ROW ? 2 : NB / VEC;   // ... as VEC-wide loads; ROW: two channels' runs per wave-load
                                                     // (one-dword pieces: half a channel's run)
    constexpr int NI = NBW + NA + 2;                 // issue items per chunk: prepare, B loads, A loads, advance
    static_assert(ROWD ? (NA == 3 && NI == 13) : ROW ? (NA == 3 && NI == 7) : (NB == 8 && NA == 2 && NI <= 12),
                  "64 x 64 tile: the issue items fit the slots of one chunk");
    __shared__ __attribute__((aligned(16))) float smem[2][STAGE_FLOATS];
    __shared__ __attribute__((aligned(16))) float s_bias[2][ROWS];
    __shared__ uint32_t s_fail;                        // a wait of this workgroup ran out: its tiles are not stored

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t G = gridDim.x;
    const uint32_t g = xsmi::xcd_contiguous_id(blockIdx.x, G);       // neighbours in chunk order share an L2
    auto range_start = [&](uint32_t j) { return j * sp.upg + xsmi::fdiv(j * sp.urem, sp.dG); };
    const uint32_t u0 = range_start(g), u1 = range_start(g + 1);
    const int rowtiles = sp.rowtiles;

    const xsmi::xsmi_int32x4 rin = xsmi::make_rsrc(sp.in, sp.in_bytes);
    const xsmi::xsmi_int32x4 rap = xsmi::make_rsrc(sp.apk, sp.apk_bytes);
    const uint32_t lds0 = (uint32_t)(uintptr_t)&smem[0][0];
    if (t == 0) s_fail = 0;                            // published by the prologue's barrier

    // ------------------------------------------------------------------ issue side
    // position of the next chunk to load: unit iu; inside a tile (r, s, cc) and the packed-filter offset
    const int pb = wave % PT;                          // pixel block (64 pixels) this wave gathers
    const int chan0 = (wave / PT) * NB;                // first of the NB channels of a chunk this wave gathers
    uint32_t iu = u0;
    uint32_t i_left = 0;                               // chunks left in the segment being issued
    int r = 0, s = 0, cc = 0;
    int i_nch = 1, i_TS = 1, i_dstep = 0, i_IH = 0, i_IW = 0;
    uint32_t i_plane = 0;
    int iyb = 0, ixb = 0, nbase = 0;
    bool live = false;
    uint32_t prep_stale = 1;                           // the pixel offset must be formed again (new segment); the uniform
                                                       // flags are integers so that they live in one scalar register each
    uint32_t ld_asoff = 0, ld_voff = 0, ld_soff = 0;
    // one-dword staged rows: the lane's second slot (lane + 64) of a run
    int iyb2 = 0, nbase2 = 0;
    bool live2 = false;
    uint32_t ld_voff2 = 0x80000000u;
    int ld_fix = 0;                                    // VEC = 4: the slot the lane clears once its run has landed (issue_prep)
    uint32_t ld_rare = 0;                              // VEC = 4, uniform: a lane of this wave has a run to move (see issue_prep)
    const int csub = VEC == 4 ? lane >> 4 : 0;         // VEC = 4: which of the wave-load's four channels the lane fetches
    const uint32_t a_lane = (uint32_t)lane * 16u;

    auto issue_segment = [&]() {                       // set up for the segment that starts at unit iu (iu < u1)
        int ci = 0;
        if constexpr (VEC != 4)
            while (ci + 1 < sp.ncls && iu >= sp.end_unit[ci]) ++ci;
        const SkClass &c = sp.cls[ci];
        const uint32_t ul = iu - c.first_unit;
        const uint32_t tile = xsmi::fdiv(ul, c.dIT);
        const uint32_t ch = ul - tile * c.iters;
        const uint32_t mt = rowtiles == 1 ? tile : tile / (uint32_t)rowtiles;
        const uint32_t rt = rowtiles == 1 ? 0u : tile - mt * (uint32_t)rowtiles;
        uint32_t n_seg = c.iters - ch;
        if (n_seg > u1 - iu) n_seg = u1 - iu;
        i_left = n_seg;
        prep_stale = 1;
        i_nch = c.nch; i_TS = ROW ? 1 : c.TS; i_dstep = c.dstep; i_IH = c.IH; i_IW = c.IW; i_plane = c.plane_bytes;
        const uint32_t tap = ch / (uint32_t)c.nch;    // ROW: the filter row
        cc = (int)(ch - tap * (uint32_t)c.nch);
        r = ROW ? (int)tap : (int)(tap / (uint32_t)c.TS);
        s = ROW ? 0 : (int)(tap - (uint32_t)r * (uint32_t)c.TS);
        ld_asoff = c.apk_off + (rt * c.iters + ch) * (uint32_t)(A_FLOATS * 4);
        iyb = 0; ixb = 0; nbase = 0;
        if constexpr (ROWD) {
            // The lane's slots are slots `lane` and `lane + 64` of a channel's run, which starts one slot before the
            // tile's first pixel; in run coordinates an image row is OX + 1 slots long, the last one a zero.
            const int m0 = (int)mt * PIX;
            const uint32_t ry0 = xsmi::fdiv((uint32_t)m0, c.dOX);
            const int pitch = c.OX + 1;
            auto place = [&](int slot, bool &lv, int &yb, int &nb) {
                const int X = m0 - (int)ry0 * c.OX - 1 + slot + pitch;          // >= 0: counted from the row before
                const uint32_t d = xsmi::fdiv((uint32_t)X, sp.dPitch);
                const int xx = X - (int)d * pitch;
                const int row = (int)ry0 + (int)d - 1;
                lv = slot < sp.run_slots && xx < c.OX && (unsigned)row < (unsigned)sp.out_rows;
                yb = 0; nb = 0;
                if (lv) {
                    const uint32_t n = xsmi::fdiv((uint32_t)row, c.dOY);
                    yb = (row - (int)n * c.OY) + c.dy0;
                    nb = (int)n * c.in_n_stride + xx;
                }
            };
            place(lane, live, iyb, nbase);
            place(lane + 64, live2, iyb2, nbase2);
            return;
        }
        if constexpr (ROW) {
            // The lane's piece is piece `lane & 31` of a channel's run: four slots of the run, which starts four slots
            // before the tile's first pixel.  In run coordinates an image row is OX + 4 slots long; a piece is either
            // four pixels of one output row (then it is fetched from the input row the tap row reaches from there, same
            // columns) or a row's trailing zeros (then the lane fetches out of range, like a row outside the image).
            const int piece = lane & 31;
            const int m0 = (int)mt * PIX;
            const uint32_t ry0 = xsmi::fdiv((uint32_t)m0, c.dOX);
            const int pitch = c.OX + 4;
            const int X = m0 - (int)ry0 * c.OX - 4 + 4 * piece + pitch;        // >= 0: counted from the row before
            const uint32_t d = xsmi::fdiv((uint32_t)X, sp.dPitch);
            const int xx = X - (int)d * pitch;
            const int row = (int)ry0 + (int)d - 1;
            live = piece < 21 && xx < c.OX && (unsigned)row < (unsigned)sp.out_rows;
            if (live) {
                const uint32_t n = xsmi::fdiv((uint32_t)row, c.dOY);
                iyb = (row - (int)n * c.OY) + c.dy0;
                nbase = (int)n * c.in_n_stride + (lane >> 5) * (int)(c.plane_bytes >> 2) + xx;
            }
            return;
        }
        const int m = VEC == 4 ? (int)mt * PIX + 4 * (lane & 15) : (int)mt * PIX + pb * 64 + lane;
        live = m < c.M;
        if (live) {
            uint32_t q = xsmi::fdiv((uint32_t)m, c.dOX);
            int x = m - (int)q * c.OX;
            uint32_t n = xsmi::fdiv(q, c.dOY);
            int y = (int)q - (int)n * c.OY;
            iyb = y * c.sy + c.dy0;
            ixb = x * c.sx + c.dx0;
            nbase = (int)n * c.in_n_stride + csub * (int)(c.plane_bytes >> 2);
        }
    };
    auto issue_prep = [&]() {
        ld_soff = (uint32_t)(cc * KC + chan0) * i_plane;
        if (cc != 0 && !prep_stale) return;            // same tap as the previous chunk: same pixel offset
        prep_stale = 0;
        const int iy = iyb + r * i_dstep, ix = ixb + s * i_dstep;
        if constexpr (ROW) {
            const bool ok = live && (unsigned)iy < (unsigned)i_IH;
            ld_voff = ok ? (uint32_t)((nbase + iy * i_IW) * 4) : 0x80000000u;
            if constexpr (ROWD) {
                const int iy2 = iyb2 + r * i_dstep;
                const bool ok2 = live2 && (unsigned)iy2 < (unsigned)i_IH;
                ld_voff2 = ok2 ? (uint32_t)((nbase2 + iy2 * i_IW) * 4) : 0x80000000u;
            }
        } else if constexpr (VEC == 4) {
            // The lane's run is columns ix .. ix + 3 of one input row; ix = -1 and ix + 3 = IW (one column past either
            // end) are the cases the host admits.  The run is fetched as it lies and the border column's slot is
            // cleared once it has landed: EVERY lane clears one slot per load then, without a test, the lanes without
            // a border column a spare slot of their own behind the stage's data.  At the very end of the tensor the
            // buffer's range check has already returned zero for the dword past it.  At its very beginning the whole
            // run would count as out of range: there the four columns inside the row are fetched and moved by one
            // place afterwards (the wave concerned takes a slower path for that tap: ld_rare).
            int off = nbase + iy * i_IW + ix;
            const int fix = ix < 0 ? 1 : (ix + 4 > i_IW ? 2 : 0);
            const bool ok = live && (unsigned)iy < (unsigned)i_IH;
            const bool moved = ok && fix == 1 && off < 0;
            if (moved) off += 1;
            ld_voff = ok ? (uint32_t)(off * 4) : 0x80000000u;
            const int run = A_FLOATS + chan0 * PIX + lane * 4;
            ld_fix = !ok || fix == 0 ? A_FLOATS + B_FLOATS + t : moved ? (run | 0x40000000) : run + (fix == 1 ? 0 : 3);
            ld_rare = (uint32_t)__builtin_amdgcn_readfirstlane(__builtin_amdgcn_ballot_w64(moved) != 0ull ? 1 : 0);
        } else {
            bool ok = live && (unsigned)iy < (unsigned)i_IH && (unsigned)ix < (unsigned)i_IW;
            ld_voff = ok ? (uint32_t)((nbase + iy * i_IW + ix) * 4) : 0x80000000u;
        }
    };
    // The LDS place of a load is a wave-uniform base (which of the chunk's channels / filter rows this wave fetches)
    // plus a constant of the unrolled loop body (stage, which of the wave's loads): the constant rides in the load
    // statement itself.
    const uint32_t lds_b = lds0 + (uint32_t)((ROW ? chan0 * BPITCH : VEC == 4 ? chan0 * PIX : chan0 * PIX + pb * 64) * 4);
    const uint32_t lds_a = lds0 + (uint32_t)(wave * NA * (ROWS / RT) * 16);
    static_assert(RT == 1, "A wave-load f of a chunk is quad f");
    auto issue_b = [&](auto e_, auto st_) {
        constexpr int e = decltype(e_)::value, st = decltype(st_)::value;
        if constexpr (ROWD)                            // channel chan0 + e / 2, slots 64 (e % 2) .. + 63 of its run
            xsmi::load_lds_b32_at<(uint32_t)((st * STAGE_FLOATS + A_FLOATS + (e / 2) * BPITCH + (e % 2) * 64) * 4)>(
                rin, lds_b, e % 2 ? ld_voff2 : ld_voff, ld_soff + (uint32_t)(e / 2) * i_plane);
        else if constexpr (ROW)                        // channels chan0 + 2 e and + 2 e + 1: 32 pieces each, 21 in use
            xsmi::load_lds_b128_at<(uint32_t)((st * STAGE_FLOATS + A_FLOATS + 2 * e * BPITCH) * 4)>(rin, lds_b, ld_voff,
                                                                                                   ld_soff + (uint32_t)(2 * e) * i_plane);
        else if constexpr (VEC == 4)                   // channels chan0 + 4 e .. + 3, the tile's 64 pixels
            xsmi::load_lds_b128_at<(uint32_t)((st * STAGE_FLOATS + A_FLOATS + 4 * e * PIX) * 4)>(rin, lds_b, ld_voff,
                                                                                                  ld_soff + (uint32_t)(4 * e) * i_plane);
        else                                           // channel chan0 + e of the chunk, this wave's 64 pixels
            xsmi::load_lds_b32_at<(uint32_t)((st * STAGE_FLOATS + A_FLOATS + e * PIX) * 4)>(rin, lds_b, ld_voff,
                                                                                             ld_soff + (uint32_t)e * i_plane);
    };
    auto issue_a = [&](auto e_, auto st_) {           // 64 rows of quad wave * NA + e
        constexpr int e = decltype(e_)::value, st = decltype(st_)::value;
        const uint32_t off = (uint32_t)((wave * NA + e) * ROWS * 16);
        xsmi::load_lds_b128_at<(uint32_t)(st * STAGE_FLOATS * 4 + e * ROWS * 16)>(rap, lds_a, a_lane + off, ld_asoff);
    };
    // VEC = 4, after the chunk's loads have landed and before the barrier that publishes them: border columns are
    // overwritten with zero, moved runs are put in place.  `stage_floats`: float offset of that stage.
    auto fix_borders = [&](int stage_floats, int fix) {
        if constexpr (VEC == 4) {
            asm volatile("" ::: "memory");
            float *stage = &smem[0][0] + stage_floats;
            if (!ld_rare) {                            // uniform
#pragma unroll
                for (int e = 0; e < NBW; ++e) stage[fix + 4 * e * PIX] = 0.f;
            } else if (fix & 0x40000000) {
#pragma unroll
                for (int e = 0; e < NBW; ++e) {
                    float4 *q4 = reinterpret_cast<float4 *>(stage + (fix & 0xffff) + 4 * e * PIX);
                    const float4 v = *q4;
                    *q4 = make_float4(0.f, v.x, v.y, v.z);
                }
            } else {
#pragma unroll
                for (int e = 0; e < NBW; ++e) stage[fix + 4 * e * PIX] = 0.f;
            }
            asm volatile("" ::: "memory");
        }
    };
    auto issue_advance = [&]() {
        if (i_left == 0) return;                       // past the end of the range: dummy chunks, nothing to advance
        ++iu;
        ld_asoff += (uint32_t)(A_FLOATS * 4);
        if (++cc == i_nch) {
            cc = 0;
            if (++s == i_TS) { s = 0; ++r; }
        }
        if (--i_left == 0) {
            if (iu < u1) {
                issue_segment();
            } else {
                // Past the range every chunk still runs the full loop body; its loads are given no live pixel
                // (they touch no memory and fill the stage with zeros) and re-read the first filter block.
                live = false; ld_asoff = 0; r = 0; s = 0; cc = 0; prep_stale = 1;
            }
        }
    };
    // the stage a chunk is loaded into follows from where the call stands in the unrolled loop (`st_`: 0 or 1)
    auto issue_item_at = [&](auto ic, auto st_) {
        constexpr int n = decltype(ic)::value;
        if constexpr (n == 0) issue_prep();
        else if constexpr (n >= 1 && n <= NBW) issue_b(IC<n - 1>{}, st_);
        else if constexpr (n > NBW && n <= NBW + NA) issue_a(IC<n - 1 - NBW>{}, st_);
        else if constexpr (n == NBW + NA + 1) issue_advance();
    };
    auto issue_all_at = [&](auto st_) { static_for<NI>([&](auto ic) { issue_item_at(ic, st_); }); };

    // ------------------------------------------------------------------ multiply side
    // two accumulators take alternate reduction steps of the wave's one
    // block and are added when a segment ends.
    constexpr int NACC = 2;
    floatx16 acc[NACC];
    auto zero_acc = [&]() {
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][v] = 0.f;
    };
    zero_acc();
    const int h = lane >> 5, l31 = lane & 31;
    const int wr = wave / WCn, wc = wave % WCn;
    // lane half h takes channels (KC/2) h .. of a chunk: quad (KC/8) h + group, channel (KC/2) h + 4 group + step
    const int a_rd = ((GROUPS * h) * ROWS + wr * 32 + l31) * 4;
    const int b_rd = A_FLOATS + (KC / 2) * h * (ROW ? BPITCH : PIX) + wc * 32 + l31;
    // ROW: where the lane's pixel lies in a channel's run depends on the tile (the run has four slots of zeros behind
    // every image row): float index of the slot one to the LEFT of the pixel, for the segment being multiplied and
    // for the tile after it (the first fragments of a unit are read while the unit before it is multiplied)
    int b_run = 0, b_run_next = 0;
    // fragments of a whole chunk, two buffers
    float4 fa[2][KC / 8];                              // [buffer][quad]
    float fb[2][KC / 2];                               // [buffer][channel]

    // compute-side cursor
    uint32_t cu = u0;
    uint32_t c_left = 0;                               // chunks left in the current segment
    int c_ci = 0, c_m0 = 0, c_rt = 0;
    uint32_t c_head = 0, c_complete = 0;               // segment holds the tile's first chunk / its last chunk
    uint32_t c_tile_end = 0;                           // unit after the tile's last chunk
    int bias_buf = 0;
    uint32_t flag_pending = 0;                         // a partial tile has been stored, its flag not raised yet
    auto compute_segment = [&]() {
        int ci = 0;
        if constexpr (VEC != 4)
            while (ci + 1 < sp.ncls && cu >= sp.end_unit[ci]) ++ci;
        const SkClass &c = sp.cls[ci];
        const uint32_t ul = cu - c.first_unit;
        const uint32_t tile = xsmi::fdiv(ul, c.dIT);
        const uint32_t ch = ul - tile * c.iters;
        const uint32_t mt = rowtiles == 1 ? tile : tile / (uint32_t)rowtiles;
        const uint32_t rt = rowtiles == 1 ? 0u : tile - mt * (uint32_t)rowtiles;
        uint32_t n_seg = c.iters - ch;
        if (n_seg > u1 - cu) n_seg = u1 - cu;
        c_left = n_seg;
        c_ci = ci; c_m0 = (int)mt * PIX; c_rt = (int)rt;
        c_head = ch == 0 ? 1u : 0u;
        c_complete = ch + n_seg == c.iters ? 1u : 0u;
        c_tile_end = cu + (c.iters - ch);
        if constexpr (ROW) {
            auto run_slot = [&](int m0) {              // pixel m0 + (wc * 32 + l31): slot RPAD + p + RPAD * (row ends before it)
                const uint32_t ry0 = xsmi::fdiv((uint32_t)m0, c.dOX);
                const int xp = m0 - (int)ry0 * c.OX + wc * 32 + l31;
                return b_rd + (RPAD - 1) + RPAD * (int)xsmi::fdiv((uint32_t)xp, c.dOX);
            };
            b_run = run_slot(c_m0);
            b_run_next = run_slot(c_rt + 1 == rowtiles ? c_m0 + PIX : c_m0);
        }
        // the tile's bias goes through the LDS (one coalesced load); the chunk loop's barriers publish it
        bias_buf ^= 1;
        if (sp.bias && c_head && t < ROWS) s_bias[bias_buf][t] = c_rt * ROWS + t < c.rows ? sp.bias[c_rt * ROWS + t] : 0.f;
    };

    // accumulator register v of lane l in block (i, j): row 32 i + 8 (v / 4) + 4 (l / 32) + v % 4, pixel 32 j + l % 32
    auto store_tile = [&]() {
        xsmi::store_block_32x32(acc[0], sp.cls[c_ci], sp.out, sp.out_bytes, sp.mask, sp.bias ? &s_bias[bias_buf][0] : nullptr,
                                sp.relu, sp.accumulate, c_rt * ROWS, ROWS, wr * 32, c_m0 + wc * 32, lane);
    };
    // the partial tile of workgroup j: register v of thread t at float (j * 16 + v) * 256 + t of the partial-tile area
    constexpr uint32_t PART_BYTES = 16 * 256 * 4;
    auto end_segment = [&]() {
        const __amdgpu_buffer_rsrc_t rpart = __builtin_amdgcn_make_buffer_rsrc((void *)sp.part, 0, (int)sp.part_bytes, 0x00020000);
        acc[0] += acc[1];
        if (!c_head) {
            // not this workgroup's tile: hand the accumulators to the workgroup that holds the tile's first chunk
#pragma unroll
            for (int v = 0; v < 16; ++v) buf_store<AGENT>(rpart, acc[0][v], (uint32_t)t * 4u, g * PART_BYTES + (uint32_t)v * 1024u);
            if (cu < u1) {
                // More chunks follow: the next chunk's body waits for all outstanding memory operations of every wave
                // (vmcnt(0), then the workgroup barrier) before it reads the next stage, which covers these stores;
                // the flag is raised after that body instead of stalling the workgroup for the write-through here.
                flag_pending = 1;
            } else {
                xsmi::wait_vmcnt<0>();                 // this thread's stores have been written through
                __syncthreads();                       // ... and everybody else's
                if (t == 0) __hip_atomic_store(sp.flags + g, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            return;
        }
        if (!c_complete) {
            // The rest of the tile was multiplied by the workgroups that follow: add their parts in chunk order.  Up to
            // three parts are fetched in one round trip (a tile of many chunks is shared by several workgroups, and
            // every one of them stands at the end of its range when the owner asks); they are added one after the
            // other, so the sum is the same as with one part at a time.
            for (uint32_t j = g + 1; j < G; j += 3) {
                if (range_start(j) >= c_tile_end) break;
                const uint32_t n = j + 1 < G && range_start(j + 1) < c_tile_end
                                       ? (j + 2 < G && range_start(j + 2) < c_tile_end ? 3u : 2u) : 1u;
                if (t == 0) {
                    // spin_limit 0: every wait counts as run out (the host's way to exercise this path)
                    for (uint32_t i = 0; i < n; ++i) {
                        uint32_t spins = 0;
                        bool there = false;
                        while (sp.spin_limit != 0u &&
                               !(there = __hip_atomic_load(sp.flags + j + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) &&
                               ++spins < sp.spin_limit)
                            __builtin_amdgcn_s_sleep(2);
                        if (!there) {
                            // Give up: the host finds the word at its next check and reports the launch as failed.
                            // Neither this tile nor any later one of the workgroup is stored, and the late partial's
                            // flag stays raised for the host to clear.
                            s_fail = 1u;
                            __hip_atomic_store(sp.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                            break;
                        }
                    }
                }
                __syncthreads();
                if (s_fail) return;
                float part[3][16];
#pragma unroll
                for (int i = 0; i < 3; ++i)
                    if ((uint32_t)i < n) {
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            part[i][v] = buf_load<AGENT>(rpart, (uint32_t)t * 4u, (j + (uint32_t)i) * PART_BYTES + (uint32_t)v * 1024u);
                    }
#pragma unroll
                for (int i = 0; i < 3; ++i)
                    if ((uint32_t)i < n) {
#pragma unroll
                        for (int v = 0; v < 16; ++v) acc[0][v] += part[i][v];
                    }
                __syncthreads();                       // everybody has read the parts before their flags are cleared
                if ((uint32_t)t < n) __hip_atomic_store(sp.flags + j + (uint32_t)t, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (s_fail) return;
        store_tile();
    };
    auto chunk_done = [&]() {
        if (flag_pending) {                            // uniform: the partial tile stored before this chunk is complete
            flag_pending = 0;
            if (t == 0) __hip_atomic_store(sp.flags + g, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        ++cu;
        if (--c_left == 0) {
            end_segment();
            zero_acc();
            if (cu < u1) compute_segment();
        }
    };

    const uint32_t total = u1 - u0;
    if (total == 0) return;
#define XSMI_PIN() __builtin_amdgcn_sched_barrier(0)
#define XSMI_MFMA(ACC, AV, BV) ACC = __builtin_amdgcn_mfma_f32_32x32x2f32(AV, BV, ACC, 0, 0, 0)
    {
        // The loop body: the fragments of two consecutive chunks live in registers.  A chunk is 16
        // MFMAs on the current fragments; after the first four it waits for the next chunk and crosses the barrier
        // (every wave then holds the current chunk in registers, so its stage is free), and every later MFMA is
        // followed by one slice of the remaining work: LDS fragment reads of the next chunk, LDS-direct loads of the
        // chunk after next.
                // Chunk 2 i of the workgroup's range lives in stage 0 and its fragments in register set 0, chunk 2 i + 1 in
        // stage 1 and set 1: everything that depends on the stage is a constant of the unrolled loop body.
        auto read_chunk = [&](auto buf_) {
            constexpr int bf = decltype(buf_)::value;
            const float *base = &smem[0][0] + bf * STAGE_FLOATS;
            const float *bsrc = base + b_rd;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) fa[bf][q4] = *reinterpret_cast<const float4 *>(base + a_rd + q4 * ROWS * 4);
#pragma unroll
            for (int jj = 0; jj < 16; ++jj) fb[bf][jj] = bsrc[jj * PIX];
        };
        auto body = [&](auto buf_) {
            constexpr int cur = decltype(buf_)::value, nxt = cur ^ 1;
            if constexpr (VEC == 4) {
                // the border columns of the chunk that has just landed are cleared first and the LDS writes complete
                // behind the chunk's first four MFMAs, not between the wait for the loads and the barrier
                xsmi::wait_vmcnt<0>();
                fix_borders(nxt * STAGE_FLOATS, ld_fix);   // the chunk that has just landed is the one issued last
                XSMI_PIN();
            }
            XSMI_MFMA(acc[0], fa[cur][0].x, fb[cur][0]);
            XSMI_MFMA(acc[1], fa[cur][0].y, fb[cur][1]);
            XSMI_MFMA(acc[0], fa[cur][0].z, fb[cur][2]);
            XSMI_MFMA(acc[1], fa[cur][0].w, fb[cur][3]);
            XSMI_PIN();
            if constexpr (VEC == 4) xsmi::wait_lgkmcnt0();
            else xsmi::wait_vmcnt<0>();
            xsmi::block_barrier();
            XSMI_PIN();
            const float *base = &smem[0][0] + nxt * STAGE_FLOATS;
            const float *bsrc = base + b_rd;
            XSMI_MFMA(acc[0], fa[cur][1].x, fb[cur][4]);
            fa[nxt][0] = *reinterpret_cast<const float4 *>(base + a_rd);
            issue_item_at(IC<0>{}, buf_);
            XSMI_PIN();
            XSMI_MFMA(acc[1], fa[cur][1].y, fb[cur][5]);
            fa[nxt][1] = *reinterpret_cast<const float4 *>(base + a_rd + ROWS * 4);
            issue_item_at(IC<1>{}, buf_);
            XSMI_PIN();
            XSMI_MFMA(acc[0], fa[cur][1].z, fb[cur][6]);
            fa[nxt][2] = *reinterpret_cast<const float4 *>(base + a_rd + 2 * ROWS * 4);
            issue_item_at(IC<2>{}, buf_);
            XSMI_PIN();
            XSMI_MFMA(acc[1], fa[cur][1].w, fb[cur][7]);
            fa[nxt][3] = *reinterpret_cast<const float4 *>(base + a_rd + 3 * ROWS * 4);
            issue_item_at(IC<3>{}, buf_);
            XSMI_PIN();
#define XSMI_SLOT(A, AV, J)                                           \
            XSMI_MFMA(acc[A], AV, fb[cur][J]);                       \
            fb[nxt][2 * (J - 8)] = bsrc[(2 * (J - 8)) * PIX];            \
            fb[nxt][2 * (J - 8) + 1] = bsrc[(2 * (J - 8) + 1) * PIX];    \
            issue_item_at(IC<J - 4>{}, buf_);                        \
            XSMI_PIN();
            XSMI_SLOT(0, fa[cur][2].x, 8)
            XSMI_SLOT(1, fa[cur][2].y, 9)
            XSMI_SLOT(0, fa[cur][2].z, 10)
            XSMI_SLOT(1, fa[cur][2].w, 11)
            XSMI_SLOT(0, fa[cur][3].x, 12)
            XSMI_SLOT(1, fa[cur][3].y, 13)
            XSMI_SLOT(0, fa[cur][3].z, 14)
            XSMI_SLOT(1, fa[cur][3].w, 15)
#undef XSMI_SLOT
        };
        // ROW: a unit is three taps of eight MFMAs each on one stage; the fragments of one TAP live in a register set,
        // tap t of a unit in stage c in set (c + t) & 1.  While a tap multiplies, the next tap's fragments are read:
        // from the same stage, and for the unit's last tap (after its first two MFMAs the next unit has landed and the
        // barrier is crossed: from then on nobody reads this stage) from the next stage, whose unit may belong to the
        // next tile (b_run_next).  The loads of the unit after next go out behind the same MFMAs.
        auto read_tap = [&](auto st_, auto tap_, auto set_, int run) {
            constexpr int st = decltype(st_)::value, tap = decltype(tap_)::value, set = decltype(set_)::value;
            const float *base = &smem[0][0] + st * STAGE_FLOATS;
#pragma unroll
            for (int i = 0; i < KC / 8; ++i)
                fa[set][i] = *reinterpret_cast<const float4 *>(base + a_rd + (tap * QUADS + i) * ROWS * 4);
#pragma unroll
            for (int k = 0; k < KC / 2; ++k) fb[set][k] = base[run + tap + k * BPITCH];
        };
        // the issue items of a unit over the six MFMAs behind the barrier: one per MFMA (one-dword pieces: two), the
        // rest with the last
        auto issue_slot = [&](auto q_, auto buf_) {
            constexpr int q = decltype(q_)::value, per = ROWD ? 2 : 1;
            static_for<per>([&](auto i) { issue_item_at(IC<q * per + decltype(i)::value>{}, buf_); });
            if constexpr (q == 5) static_for<NI - 6 * per>([&](auto i) { issue_item_at(IC<6 * per + decltype(i)::value>{}, buf_); });
        };
        auto body_row = [&](auto buf_) {
            constexpr int cur = decltype(buf_)::value, nxt = cur ^ 1;
            constexpr int s0 = cur, s1 = cur ^ 1;      // register sets of taps 0 and 2 / of tap 1
            const float *base = &smem[0][0] + cur * STAGE_FLOATS;
            // a tap's eight MFMAs with the next tap's reads from the same stage behind the first six
#define XSMI_TAP(SA, SB, TAP)                                                                                    \
            XSMI_MFMA(acc[0], fa[SA][0].x, fb[SA][0]);                                                           \
            fa[SB][0] = *reinterpret_cast<const float4 *>(base + a_rd + ((TAP) * QUADS) * ROWS * 4);             \
            XSMI_PIN();                                                                                          \
            XSMI_MFMA(acc[1], fa[SA][0].y, fb[SA][1]);                                                           \
            fa[SB][1] = *reinterpret_cast<const float4 *>(base + a_rd + ((TAP) * QUADS + 1) * ROWS * 4);         \
            XSMI_PIN();                                                                                          \
            XSMI_MFMA(acc[0], fa[SA][0].z, fb[SA][2]);                                                           \
            fb[SB][0] = base[b_run + (TAP)];                                                                     \
            fb[SB][1] = base[b_run + (TAP) + BPITCH];                                                            \
            XSMI_PIN();                                                                                          \
            XSMI_MFMA(acc[1], fa[SA][0].w, fb[SA][3]);                                                           \
            fb[SB][2] = base[b_run + (TAP) + 2 * BPITCH];                                                        \
            fb[SB][3] = base[b_run + (TAP) + 3 * BPITCH];                                                        \
            XSMI_PIN();                                                                                          \
            XSMI_MFMA(acc[0], fa[SA][1].x, fb[SA][4]);                                                           \
            fb[SB][4] = base[b_run + (TAP) + 4 * BPITCH];                                                        \
            fb[SB][5] = base[b_run + (TAP) + 5 * BPITCH];                                                        \
            XSMI_PIN();                                                                                          \
            XSMI_MFMA(acc[1], fa[SA][1].y, fb[SA][5]);                                                           \
            fb[SB][6] = base[b_run + (TAP) + 6 * BPITCH];                                                        \
            fb[SB][7] = base[b_run + (TAP) + 7 * BPITCH];                                                        \
            XSMI_PIN();                                                                                          \
            XSMI_MFMA(acc[0], fa[SA][1].z, fb[SA][6]);                                                           \
            XSMI_MFMA(acc[1], fa[SA][1].w, fb[SA][7]);                                                           \
            XSMI_PIN();
            XSMI_TAP(s0, s1, 1)
            XSMI_TAP(s1, s0, 2)
#undef XSMI_TAP
            XSMI_MFMA(acc[0], fa[s0][0].x, fb[s0][0]);
            XSMI_MFMA(acc[1], fa[s0][0].y, fb[s0][1]);
            XSMI_PIN();
            xsmi::wait_vmcnt<0>();
            xsmi::wait_lgkmcnt0();
            xsmi::block_barrier();
            XSMI_PIN();
            const float *nbase_ = &smem[0][0] + nxt * STAGE_FLOATS;
            const int run = c_left == 1 ? b_run_next : b_run;
            XSMI_MFMA(acc[0], fa[s0][0].z, fb[s0][2]);
            fa[s1][0] = *reinterpret_cast<const float4 *>(nbase_ + a_rd);
            fb[s1][0] = nbase_[run];
            fb[s1][1] = nbase_[run + BPITCH];
            issue_slot(IC<0>{}, buf_);
            XSMI_PIN();
            XSMI_MFMA(acc[1], fa[s0][0].w, fb[s0][3]);
            fa[s1][1] = *reinterpret_cast<const float4 *>(nbase_ + a_rd + ROWS * 4);
            fb[s1][2] = nbase_[run + 2 * BPITCH];
            fb[s1][3] = nbase_[run + 3 * BPITCH];
            issue_slot(IC<1>{}, buf_);
            XSMI_PIN();
            XSMI_MFMA(acc[0], fa[s0][1].x, fb[s0][4]);
            fb[s1][4] = nbase_[run + 4 * BPITCH];
            fb[s1][5] = nbase_[run + 5 * BPITCH];
            fb[s1][6] = nbase_[run + 6 * BPITCH];
            fb[s1][7] = nbase_[run + 7 * BPITCH];
            issue_slot(IC<2>{}, buf_);
            XSMI_PIN();
            XSMI_MFMA(acc[1], fa[s0][1].y, fb[s0][5]);
            issue_slot(IC<3>{}, buf_);
            XSMI_PIN();
            XSMI_MFMA(acc[0], fa[s0][1].z, fb[s0][6]);
            issue_slot(IC<4>{}, buf_);
            XSMI_PIN();
            XSMI_MFMA(acc[1], fa[s0][1].w, fb[s0][7]);
            issue_slot(IC<5>{}, buf_);
            XSMI_PIN();
        };
        // prologue: chunk 0 landed and in registers, chunk 1 in flight
        issue_segment();
        issue_all_at(IC<0>{});
        compute_segment();
        xsmi::wait_vmcnt<0>();
        fix_borders(0, ld_fix);
        xsmi::wait_lgkmcnt0();
        xsmi::block_barrier();
        if constexpr (ROW) read_tap(IC<0>{}, IC<0>{}, IC<0>{}, b_run);
        else read_chunk(IC<0>{});
        issue_all_at(IC<1>{});
        for (uint32_t k = 0; k < total; k += 2) {
            if constexpr (ROW) body_row(IC<0>{});
            else body(IC<0>{});
            chunk_done();
            if (k + 1 < total) {
                if constexpr (ROW) body_row(IC<1>{});
                else body(IC<1>{});
                chunk_done();
            }
        }
    }
#undef XSMI_MFMA
#undef XSMI_PIN
    xsmi::wait_vmcnt<0>();                             // the dummy chunks' loads target this workgroup's LDS
}

// ---- filter layout --------------------------------------------------------------------------------------------
// [rowtile][chunk = tap * nch + cc][quad KC/4][row ROWS][4 channels]: the LDS image of a stage's A part.
// mode 0 (forward): A[row][tap = (r, s)][ch] = w[row][ch][r][s].
// mode 1 (backward-data class): A[row = c][tap = (t, u)][ch = k] = w[k][c][r0 + sh t][s0 + sw u].
struct SkPackJob {
    float *apk;
    int TR, TS, r0, s0;
};
struct SkPackMulti {
    SkPackJob job[SK_MAX_CLASSES];
    uint32_t first[SK_MAX_CLASSES + 1];
    int njobs;
};
__global__ void __launch_bounds__(256) sk_pack_kernel(const float *__restrict__ w, SkPackMulti pm, int mode, int rows, int CH,
                                                       int R, int S, int sh, int sw, int rowtiles, int ROWS, int KC) {
    int ji = 0;
    while (ji + 1 < pm.njobs && blockIdx.x >= pm.first[ji + 1]) ++ji;
    const SkPackJob &j = pm.job[ji];
    const uint32_t blk = blockIdx.x - pm.first[ji], nblk = pm.first[ji + 1] - pm.first[ji];
    float *__restrict__ apk = j.apk;
    const int TR = j.TR, TS = j.TS, r0 = j.r0, s0 = j.s0;
    const int nch = CH / KC;
    const int iters = TR * TS * nch;
    const size_t total4 = (size_t)rowtiles * iters * ROWS * (KC / 4);          // float4 groups
    for (size_t i = (size_t)blk * 256 + threadIdx.x; i < total4; i += (size_t)nblk * 256) {
        const int rr = (int)(i % ROWS);
        size_t rest = i / ROWS;
        const int q = (int)(rest % (KC / 4));
        rest /= (KC / 4);
        const int it = (int)(rest % iters);
        const int rt = (int)(rest / iters);
        const int cc = it % nch, tap = it / nch;
        const int tr = tap / TS, ts = tap % TS;
        const int ch = cc * KC + q * 4;
        const int row = rt * ROWS + rr;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (row < rows) {
            const size_t cstride = mode == 0 ? (size_t)R * S : (size_t)rows * R * S;
            const float *src = mode == 0 ? w + (((size_t)row * CH + ch) * R + tr) * S + ts
                                         : w + (((size_t)ch * rows + row) * R + (r0 + sh * tr)) * S + (s0 + sw * ts);
            v = make_float4(src[0], src[cstride], src[2 * cstride], src[3 * cstride]);
        }
        reinterpret_cast<float4 *>(apk)[i] = v;
    }
}

// The 3x3, stride-1 case of sk_pack_kernel with wide accesses: a thread takes one row and one quad of channels, i.e.
// 36 floats of w (mode 0: one contiguous run, read as nine float4; mode 1: four runs of nine), and stores one float4 per
// tap; the lanes of a wavefront are consecutive rows, so a store instruction writes 1 KB of one tap's block and every
// byte of w is requested once.
// units != 0: the layout of the staged-row form, [rowtile][filter row][chunk][tap slot][quad][row][4 channels], where
// slot j holds the tap that shifts the input by j - 1 columns: filter column j (units 1: forward), 2 - j (units 2:
// backward-data, whose taps walk the other way).
__global__ void __launch_bounds__(256) sk_pack_3x3_kernel(const float *__restrict__ w, float *__restrict__ apk, int mode,
                                                           int rows, int CH, int rowtiles, int ROWS, int KC, int units) {
    const int nch = CH / KC, quads = KC / 4;
    const uint32_t total = (uint32_t)rowtiles * (uint32_t)nch * (uint32_t)quads * (uint32_t)ROWS;
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= total) return;
    const int rr = (int)(i % (uint32_t)ROWS);
    uint32_t rest = i / (uint32_t)ROWS;
    const int q = (int)(rest % (uint32_t)quads);
    rest /= (uint32_t)quads;
    const int cc = (int)(rest % (uint32_t)nch), rt = (int)(rest / (uint32_t)nch);
    const int ch0 = cc * KC + q * 4, row = rt * ROWS + rr;
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
    // float4 index ((rt * iters + tap * nch + cc) * quads + q) * ROWS + rr with iters = 9 * nch
    if (units) {
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const int tr = t / 3, ts = t % 3, slot = units == 1 ? ts : 2 - ts;
            float4 *dst = reinterpret_cast<float4 *>(apk) +
                          (((((size_t)rt * 3 + tr) * nch + cc) * 3 + slot) * quads + q) * ROWS + rr;
            *dst = make_float4(v[0][t], v[1][t], v[2][t], v[3][t]);
        }
        return;
    }
    float4 *dst = reinterpret_cast<float4 *>(apk) + (((size_t)rt * 9 * nch + cc) * quads + q) * ROWS + rr;
#pragma unroll
    for (int t = 0; t < 9; ++t) dst[(size_t)t * nch * quads * ROWS] = make_float4(v[0][t], v[1][t], v[2][t], v[3][t]);
}

struct SkShape { int rows_tile, pix_tile, kc; };
int sk_env() { return (int)xsmi::option(xsmi::OPT_TAP_SK); }
SkShape sk_shape(int) { return SkShape{SK_ROWS, SK_PIX, SK_KC}; }

size_t sk_pack_bytes(int rows, int CH, int taps, const SkShape &sh) {
    return xsmi::align_up((size_t)xsmi::ceil_div(rows, sh.rows_tile) * taps * (CH / sh.kc) * sh.rows_tile * sh.kc * sizeof(float), 256);
}
static_assert((size_t)SK_MAX_GRID * 4 <= xsmi::SK_SCRATCH_FLAG_BYTES, "one flag per workgroup");
static_assert((size_t)SK_MAX_GRID * 16 * 256 * sizeof(float) <= xsmi::SK_SCRATCH_PART_BYTES, "one partial tile per workgroup");

// resident workgroups of the kernel variant (occupancy x compute units), cached per variant
template <typename K>
int sk_resident(K kernel, int *cache, int cap) {
    if (*cache == 0) {
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, 0) != hipSuccess || per_cu < 1) per_cu = 1;
        int gsz = per_cu * xsmi::cu_count();
        if (gsz > cap) gsz = cap;
        *cache = gsz & ~7;
        if (*cache < 8) *cache = 8;
    }
    return *cache;
}

// Wide B loads: a launch of one class that walks its input with stride 1 over rows a multiple of four pixels wide,
// with taps that reach at most one column past either end of a row.
bool sk_wide_loads_ok(const SkParams &p) {
    if (xsmi::option(xsmi::OPT_SK_WIDE) == 0 || p.ncls != 1) return false;
    if ((((uintptr_t)p.in) & 3) != 0) return false;
    for (int i = 0; i < p.ncls; ++i) {
        const SkClass &c = p.cls[i];
        if (c.sx != 1 || c.OX % 4 != 0 || c.IW < 4) return false;
        for (int ts = 0; ts < c.TS; ++ts) {
            const int shift = c.dx0 + ts * c.dstep;
            if (shift < -1 || shift > c.IW - c.OX + 1) return false;
        }
    }
    return true;
}

// Staged rows (the filter must have been laid out for them): 3 x 3, stride 1, one column and one row of padding, rows
// as wide as the output's, channels in chunks of 16.  1: 16-byte pieces, for rows a multiple of four pixels and at
// least 20 wide (a tile of 64 pixels then crosses at most three row ends: 21 pieces per run); 2: one-dword pieces, for
// rows of two to eleven pixels (66 slots plus one per row end inside a tile: at most 98 of a run's 128).  The kernel
// serves wider rows in that form as well, but from 14 pixels on it is no faster than tap by tap (measured at N=32:
// 512 -> 512 at 7 x 7 65.9 -> 64.7 us, 256 -> 256 at 14 x 14 63.2 -> 63.6 us); sk_wide = 3 takes it wherever it applies.
int sk_rows_staged(int R, int S, int sh, int sw, int pad, int in_w, int out_w, int channels) {
    const long opt = xsmi::option(xsmi::OPT_SK_WIDE);
    if (opt < 2 || R != 3 || S != 3 || sh != 1 || sw != 1 || pad != 1 || in_w != out_w || channels % 16 != 0 || out_w < 2)
        return 0;
    if (out_w % 4 == 0 && out_w >= 20) return 1;
    return out_w < 12 || opt >= 3 ? 2 : 0;
}

int sk_launch(hipStream_t st, SkParams &p, const SkShape &) {
    static int res_narrow = 0, res_wide = 0, res_rows = 0;
    static int res_rows1 = 0;
    const int rows = p.staged_rows;
    const bool wide = !rows && sk_wide_loads_ok(p);
    if (rows) {
        const SkClass &c = p.cls[0];
        if (p.ncls != 1 || c.sx != 1 || c.sy != 1 || c.TS != 3 || c.dx0 + c.dstep != 0 || c.IW != c.OX || c.OX < 2 ||
            (rows == 1 && (c.OX % 4 != 0 || c.OX < 20)) || (((uintptr_t)p.in) & 3) != 0)
            return xsmi::set_error("even-split convolution: geometry not served by the staged-row form"), XSMI_ERR_INVALID;
        p.out_rows = c.M / c.OX;
        p.dPitch = xsmi::make_fastdiv(c.OX + (rows == 1 ? 4 : 1));
        p.run_slots = 66 + (c.OX - 1 + 63) / c.OX;
    }
    uint32_t gsz = (uint32_t)(rows == 1 ? sk_resident(tap_sk_f32_kernel<3>, &res_rows, SK_MAX_GRID)
                              : rows    ? sk_resident(tap_sk_f32_kernel<2>, &res_rows1, SK_MAX_GRID)
                              : wide    ? sk_resident(tap_sk_f32_kernel<4>, &res_wide, SK_MAX_GRID)
                                        : sk_resident(tap_sk_f32_kernel<1>, &res_narrow, SK_MAX_GRID));
    if (gsz > p.units) gsz = p.units;                  // every workgroup gets at least one chunk
    if (gsz == 0) return XSMI_OK;
    p.upg = p.units / gsz; p.urem = p.units % gsz; p.dG = xsmi::make_fastdiv(gsz);
    // the library's partial-tile area of this stream; a wait that ran out in an earlier launch is reported here
    // (and by every call that waits for the device) instead of starting on flags that may be stale
    int rc = xsmi::check_device_error("even-split convolution");
    if (rc) return rc;
    const xsmi::SkScratch scr = xsmi::sk_scratch();
    p.part = scr.part; p.flags = scr.flags; p.err = xsmi::device_error_word();
    p.part_bytes = (uint32_t)xsmi::SK_SCRATCH_PART_BYTES;
    const long spin = xsmi::option(xsmi::OPT_SK_SPIN_LIMIT);
    p.spin_limit = spin < 0 ? 0u : spin > 0x7fffffffL ? 0x7fffffffu : (uint32_t)spin;
    if (rows == 1) hipLaunchKernelGGL(tap_sk_f32_kernel<3>, dim3(gsz), dim3(256), 0, st, p);
    else if (rows) hipLaunchKernelGGL(tap_sk_f32_kernel<2>, dim3(gsz), dim3(256), 0, st, p);
    else if (wide) hipLaunchKernelGGL(tap_sk_f32_kernel<4>, dim3(gsz), dim3(256), 0, st, p);
    else hipLaunchKernelGGL(tap_sk_f32_kernel<1>, dim3(gsz), dim3(256), 0, st, p);
    XSMI_LAUNCH_CHECK("tap_sk_f32_kernel");
    return XSMI_OK;
}

}  // namespace

namespace xsmi {

// Usable when the reduction channels split into whole chunks of the tile shape.
bool sk_path_ok(int reduce_channels, int rows) {
    if (!sk_env()) return false;
    const SkShape s = sk_shape(rows);
    return reduce_channels % s.kc == 0 && reduce_channels % 32 == 0;
}

// Where the even split pays (measured on ResNet-18's layers at N=32 against the kernels whose workgroups take whole
// tiles): every stride-1 pass with at least four taps (+1 to +17 %: no idle compute units when there are fewer tiles
// than CUs, no mostly empty last round of tiles otherwise), and every strided backward-data pass, whose four residue
// classes of different lengths then share one balanced launch (+20 to +26 %).  Strided forwards (mixed: -13 to +5 %)
// and 1 x 1 filters (a handful of chunks per tile) stay on whole tiles, except strided forwards with fewer tiles than CUs.
bool sk_fwd_pays(int M, int rows, int R, int S, int sh, int sw) {
    if (sk_env() >= 3) return true;                    // forced, for tests and measurements
    if (R * S < 4) return false;
    if (sh == 1 && sw == 1) return true;
    // a strided forward with fewer tiles than compute units: whole tiles leave CUs idle from the start
    // (256 -> 512, 3 x 3 / 2 at 14 x 14, N=32: 200 tiles, 53.6 -> 49.6 us)
    return (long)ceil_div(M, SK_PIX) * ceil_div(rows, SK_ROWS) <= 256;        // the MI355X's CU count, as a constant: the
                                                                               // choice must not depend on whether a device is open
}
bool sk_bwd_data_pays(int M, int rows, int R, int S, int sh, int sw) {
    if (sk_env() >= 3) return true;
    if (R * S < 4) return false;
    if (sh == 1 && sw == 1) return sk_fwd_pays(M, rows, R, S, 1, 1);
    return true;
}

size_t sk_fwd_ws_bytes(int C, int K, int R, int S) {
    return sk_pack_bytes(K, C, R * S, sk_shape(K));
}

size_t sk_bwd_data_ws_bytes(int C, int K, int R, int S, int sh, int sw) {
    const SkShape s = sk_shape(C);
    size_t total = 0;
    for (int ph = 0; ph < sh; ++ph)
        for (int pw = 0; pw < sw; ++pw) total += sk_pack_bytes(C, K, ceil_div(R, sh) * ceil_div(S, sw), s);
    return total;
}

static void sk_fill_class(SkClass &c, const SkShape &shp, int rowtiles) {
    c.iters = (uint32_t)(c.TR * c.TS * c.nch);
    c.dIT = make_fastdiv(c.iters ? c.iters : 1);
    (void)shp; (void)rowtiles;
}

int sk_conv_fwd(const float *x, const float *w, const float *bias, float *y, uint8_t *mask, int N, int C, int H, int W,
                int K, int R, int S, int sh, int sw, int pad, int OH, int OW, int relu, int opts, void *workspace) {
    hipStream_t st = stream();
    const SkShape shp = sk_shape(K);
    const int rowtiles = ceil_div(K, shp.rows_tile);
    const size_t pack = sk_pack_bytes(K, C, R * S, shp);
    float *apk = (float *)workspace;
    const int staged = (((uintptr_t)w) & 15) == 0 && (((uintptr_t)x) & 3) == 0 ? sk_rows_staged(R, S, sh, sw, pad, W, OW, C) : 0;
    const int kc = staged ? 16 : shp.kc;
    if (!(opts & 2) && R == 3 && S == 3 && (((uintptr_t)w) & 15) == 0) {
        const uint32_t total = (uint32_t)rowtiles * (uint32_t)(C / kc) * (uint32_t)(kc / 4) * (uint32_t)shp.rows_tile;
        hipLaunchKernelGGL(sk_pack_3x3_kernel, dim3((total + 255) / 256), dim3(256), 0, st, w, apk, 0, K, C, rowtiles,
                           shp.rows_tile, kc, staged ? 1 : 0);
        XSMI_LAUNCH_CHECK("sk_pack_3x3_kernel");
    } else if (!(opts & 2)) {
        SkPackMulti pm;
        pm.njobs = 1;
        pm.job[0] = SkPackJob{apk, R, S, 0, 0};
        size_t total4 = pack / 16;
        uint32_t nb = (uint32_t)((total4 + 255) / 256);
        if (nb > 4096) nb = 4096;
        if (nb < 4) nb = 4;
        pm.first[0] = 0; pm.first[1] = nb;
        hipLaunchKernelGGL(sk_pack_kernel, dim3(nb), dim3(256), 0, st, w, pm, 0, K, C, R, S, 1, 1, rowtiles, shp.rows_tile,
                           shp.kc);
        XSMI_LAUNCH_CHECK("sk_pack_kernel");
    }
    if (opts & 4) return XSMI_OK;            // bit 2: lay the filter out and stop
    SkParams p;
    memset(&p, 0, sizeof(p));
    SkClass &c = p.cls[0];
    c.apk_off = 0;
    c.M = N * OH * OW; c.rows = K; c.nch = C / kc; c.TR = R; c.TS = S;
    c.dy0 = -pad; c.dx0 = -pad; c.dstep = 1;
    c.IH = H; c.IW = W; c.sy = sh; c.sx = sw;
    c.in_n_stride = C * H * W; c.plane_bytes = (uint32_t)(H * W * 4);
    c.OY = OH; c.OX = OW; c.dOX = make_fastdiv(OW); c.dOY = make_fastdiv(OH);
    c.os_n = (long long)K * OH * OW; c.os_k = (long long)OH * OW; c.o_base = 0; c.os_y = OW; c.os_x = 1;
    sk_fill_class(c, shp, rowtiles);
    if (staged) {                                      // a unit is a filter row x 16 channels
        c.iters = (uint32_t)(c.TR * c.nch);
        c.dIT = make_fastdiv(c.iters);
    }
    c.first_unit = 0;
    const uint32_t tiles = (uint32_t)ceil_div(c.M, shp.pix_tile) * (uint32_t)rowtiles;
    p.units = tiles * c.iters;
    p.end_unit[0] = p.units;
    p.in = x; p.apk = apk; p.bias = bias; p.out = y; p.mask = relu ? mask : nullptr;
    p.in_bytes = (uint32_t)((size_t)N * C * H * W * 4);
    p.out_bytes = (uint32_t)((size_t)N * K * OH * OW * 4);
    p.apk_bytes = (uint32_t)pack;
    p.ncls = 1; p.rowtiles = rowtiles; p.accumulate = 0; p.relu = relu;
    p.staged_rows = staged;
    prof_begin();
    int rc = sk_launch(st, p, shp);
    prof_end();
    return rc;
}

int sk_conv_bwd_data(const float *dy, const float *w, float *dx, int N, int C, int H, int W, int K, int R, int S, int sh,
                     int sw, int pad, int OH, int OW, int accumulate, int opts, void *workspace) {
    hipStream_t st = stream();
    const SkShape shp = sk_shape(C);
    const int rowtiles = ceil_div(C, shp.rows_tile);
    SkClass plans[SK_MAX_CLASSES];
    SkPackJob jobs[SK_MAX_CLASSES];
    int nplans = 0;
    size_t off = 0;
    for (int ph = 0; ph < sh; ++ph) {
        const int OYc = ph < H ? ceil_div(H - ph, sh) : 0;
        const int r0 = (ph + pad) % sh;
        const int T = r0 < R ? ceil_div(R - r0, sh) : 0;
        const int cy = (ph + pad - r0) / sh;
        for (int pw = 0; pw < sw; ++pw) {
            const int OXc = pw < W ? ceil_div(W - pw, sw) : 0;
            if (OYc == 0 || OXc == 0) continue;
            if (nplans == SK_MAX_CLASSES) return set_error("sk_conv_bwd_data: more than %d residue classes", SK_MAX_CLASSES), XSMI_ERR_INVALID;
            const int s0 = (pw + pad) % sw;
            const int U = s0 < S ? ceil_div(S - s0, sw) : 0;
            const int cx = (pw + pad - s0) / sw;
            SkClass c;
            memset(&c, 0, sizeof(c));
            c.apk_off = (uint32_t)off;
            jobs[nplans] = SkPackJob{(float *)((char *)workspace + off), T, U, r0, s0};
            off += sk_pack_bytes(C, K, T * U, shp);
            c.M = N * OYc * OXc; c.rows = C; c.nch = K / shp.kc; c.TR = T; c.TS = U;
            c.dy0 = cy; c.dx0 = cx; c.dstep = -1;
            c.IH = OH; c.IW = OW; c.sy = 1; c.sx = 1;
            c.in_n_stride = K * OH * OW; c.plane_bytes = (uint32_t)(OH * OW * 4);
            c.OY = OYc; c.OX = OXc; c.dOX = make_fastdiv(OXc); c.dOY = make_fastdiv(OYc);
            c.os_n = (long long)C * H * W; c.os_k = (long long)H * W; c.o_base = (long long)ph * W + pw;
            c.os_y = sh * W; c.os_x = sw;
            sk_fill_class(c, shp, rowtiles);
            plans[nplans++] = c;
        }
    }
    const size_t pack = off;
    // the pass reads dy (rows of OW pixels) and writes dx (rows of W pixels)
    const int staged = nplans == 1 && (((uintptr_t)dy) & 3) == 0 ? sk_rows_staged(R, S, sh, sw, pad, OW, W, K) : 0;
    const int kc = staged ? 16 : shp.kc;
    if (staged) {                                      // a unit is a filter row x 16 channels
        plans[0].nch = K / kc;
        plans[0].iters = (uint32_t)(plans[0].TR * plans[0].nch);
        plans[0].dIT = make_fastdiv(plans[0].iters);
    }
    if (!(opts & 2) && R == 3 && S == 3 && sh == 1 && sw == 1 && nplans == 1) {
        const uint32_t total = (uint32_t)rowtiles * (uint32_t)(K / kc) * (uint32_t)(kc / 4) * (uint32_t)shp.rows_tile;
        hipLaunchKernelGGL(sk_pack_3x3_kernel, dim3((total + 255) / 256), dim3(256), 0, st, w, jobs[0].apk, 1, C, K, rowtiles,
                           shp.rows_tile, kc, staged ? 2 : 0);
        XSMI_LAUNCH_CHECK("sk_pack_3x3_kernel");
    } else if (!(opts & 2)) {
        SkPackMulti pm;
        pm.njobs = nplans;
        uint32_t blocks = 0;
        for (int i = 0; i < nplans; ++i) {
            size_t total4 = sk_pack_bytes(C, K, plans[i].TR * plans[i].TS, shp) / 16;
            uint32_t nb = (uint32_t)((total4 + 255) / 256);
            if (nb > 2048) nb = 2048;
            if (nb < 1) nb = 1;
            pm.job[i] = jobs[i];
            pm.first[i] = blocks;
            blocks += nb;
        }
        pm.first[nplans] = blocks;
        hipLaunchKernelGGL(sk_pack_kernel, dim3(blocks), dim3(256), 0, st, w, pm, 1, C, K, R, S, sh, sw, rowtiles, shp.rows_tile,
                           shp.kc);
        XSMI_LAUNCH_CHECK("sk_pack_kernel");
    }
    if (opts & 4) return XSMI_OK;            // bit 2: lay the filter out and stop
    SkParams p;
    memset(&p, 0, sizeof(p));
    uint32_t units = 0;
    int ncls = 0;
    for (int i = 0; i < nplans; ++i) {
        SkClass c = plans[i];
        // A class without taps (a stride larger than the filter) multiplies nothing: its outputs are zero (or kept,
        // when accumulating).  It gets one all-zero chunk per tile so that the epilogue runs: not needed for the
        // layers this path serves (filter >= stride), so such geometries stay on the first-generation kernels.
        if (c.iters == 0) return set_error("sk_conv_bwd_data: residue class without taps"), XSMI_ERR_INVALID;
        c.first_unit = units;
        units += (uint32_t)ceil_div(c.M, shp.pix_tile) * (uint32_t)rowtiles * c.iters;
        p.end_unit[ncls] = units;
        p.cls[ncls++] = c;
    }
    for (int i = ncls; i < SK_MAX_CLASSES; ++i) p.end_unit[i] = units;
    p.units = units;
    p.in = dy; p.apk = (const float *)workspace; p.bias = nullptr; p.out = dx; p.mask = nullptr;
    p.in_bytes = (uint32_t)((size_t)N * K * OH * OW * 4);
    p.out_bytes = (uint32_t)((size_t)N * C * H * W * 4);
    p.apk_bytes = (uint32_t)pack;
    p.ncls = ncls; p.rowtiles = rowtiles; p.accumulate = accumulate; p.relu = 0;
    p.staged_rows = staged;
    prof_begin();
    int rc = sk_launch(st, p, shp);
    prof_end();
    return rc;
}

// backward-data geometries the second-generation kernel serves: every residue class has at least one tap
bool sk_bwd_data_ok(int C, int K, int R, int S, int sh, int sw) {
    return sk_path_ok(K, C) && sh * sw <= SK_MAX_CLASSES && R >= sh && S >= sw;
}

}  // namespace xsmi
