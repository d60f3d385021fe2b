// Epilogue shared by the fp32 tap-major kernels: a lane's 32 x 32 accumulator block goes to an NCHW tensor (or a
// strided sub-lattice of one, for the residue classes of a backward-data pass).
#pragma once
#include "xsmi_internal.h"

namespace xsmi {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t uint32x2_store __attribute__((ext_vector_type(2)));

// Register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4 and pixel l % 32 of the block whose first row is
// `row0` (a multiple of 32 inside the tile) and whose pixels are m0 .. m0 + 31 of the launch's pixel numbering.
// G: a parameter set with the fields M, rows, OX, OY, dOX, dOY, os_n, os_k, o_base, os_y, os_x.
// tile_row0: first row of the workgroup's row tile; bias_lds: the tile's bias in the LDS (indexed by row inside the
// tile) or nullptr; mask: sign mask of the pre-activation (with relu) or nullptr.
//
// Whole row tiles take the fast form: one byte offset per lane, the row's displacement in a scalar register,
// out-of-range pixels through the buffer range check, and the bias / ReLU and mask / accumulate steps as passes over
// the 16 registers, each behind one uniform branch.  Tensors hold fewer than 2^29 elements, so 32-bit byte offsets
// suffice.  A ragged last row tile tests every row.
//
// zfill (overwriting only, os_x == 2 and os_y == two tensor rows): the lattice is the (even row, even column) class of
// a stride-2 backward-data pass whose other three classes no tap reaches.  Each value is then stored together with
// its right-hand neighbour, and the same two places of the row below are cleared, so that one launch writes every
// element of the tensor once, in runs of eight bytes per pixel, and no separate fill is needed.
template <typename G>
__device__ __forceinline__ void store_block_32x32(const floatx16 &acc, const G &c, float *out, uint32_t out_bytes,
                                                  uint8_t *mask, const float *bias_lds, int relu, int accumulate,
                                                  int tile_row0, int tile_rows, int row0, int m0, int lane,
                                                  int zfill = 0) {
    const int h = lane >> 5, l31 = lane & 31;
    const int lrow = row0 + 4 * h;                     // inside the tile
    const int m = m0 + l31;
    const uint32_t q = fdiv((uint32_t)m, c.dOX);
    const int x = m - (int)q * c.OX;
    const uint32_t n = fdiv(q, c.dOY);
    const int y = (int)q - (int)n * c.OY;
    if (tile_row0 + tile_rows <= c.rows) {
        const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc((void *)out, 0, (int)out_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t rmask =
            __builtin_amdgcn_make_buffer_rsrc((void *)mask, 0, mask ? (int)(out_bytes >> 2) : 0, 0x00020000);
        const uint32_t os_k4 = (uint32_t)c.os_k * 4u;
        const uint32_t srow = (uint32_t)tile_row0 * os_k4;
        const uint32_t pix = (uint32_t)((int)n * (int)c.os_n + y * c.os_y + x * c.os_x + (int)c.o_base) * 4u + (uint32_t)lrow * os_k4;
        const uint32_t voff = m < c.M ? pix : 0x80000000u;
        auto row_off = [&](int v) { return srow + (uint32_t)(8 * (v >> 2) + (v & 3)) * os_k4; };
        floatx16 r = acc;
        if (bias_lds) {
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const float4 bz = *reinterpret_cast<const float4 *>(bias_lds + lrow + 8 * q4);
                r[4 * q4] += bz.x; r[4 * q4 + 1] += bz.y; r[4 * q4 + 2] += bz.z; r[4 * q4 + 3] += bz.w;
            }
        }
        if (relu) {
            if (mask) {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    __builtin_amdgcn_raw_buffer_store_b8((unsigned char)(r[v] < 0.f ? 1 : 0), rmask, (int)(voff >> 2), (int)(row_off(v) >> 2), 0);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) r[v] = r[v] > 0.f ? r[v] : 0.f;
        }
        if (accumulate) {
            float old[16];
#pragma unroll
            for (int v = 0; v < 16; ++v)
                old[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rout, (int)voff, (int)row_off(v), 0));
#pragma unroll
            for (int v = 0; v < 16; ++v) r[v] += old[v];
        }
        if (zfill) {
            const uint32_t below = (uint32_t)c.os_y * 2u;     // one tensor row, in bytes
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float val = r[v];
                const uint32x2_store pair = {__builtin_bit_cast(uint32_t, val), 0u}, zeros = {0u, 0u};
                __builtin_amdgcn_raw_buffer_store_b64(pair, rout, (int)voff, (int)row_off(v), 0);
                __builtin_amdgcn_raw_buffer_store_b64(zeros, rout, (int)voff, (int)(row_off(v) + below), 0);
            }
            return;
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float val = r[v];                    // (a bit_cast applied to the vector element itself reads element 0)
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, val), rout, (int)voff, (int)row_off(v), 0);
        }
        return;
    }
    if (m >= c.M) return;
    const long long pix_off = (long long)n * c.os_n + (long long)y * c.os_y + (long long)x * c.os_x + c.o_base;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int ro = lrow + 8 * (v >> 2) + (v & 3);
        if (tile_row0 + ro < c.rows) {
            float val = acc[v];
            if (bias_lds) val += bias_lds[ro];
            const long long o = pix_off + (long long)(tile_row0 + ro) * c.os_k;
            if (relu) {
                if (mask) mask[o] = val < 0.f ? 1 : 0;
                val = val > 0.f ? val : 0.f;
            }
            if (accumulate) val += out[o];
            out[o] = val;
            if (zfill) { out[o + 1] = 0.f; out[o + c.os_y / 2] = 0.f; out[o + c.os_y / 2 + 1] = 0.f; }
        }
    }
}

}  // namespace xsmi
