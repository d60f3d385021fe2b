// Internal helpers shared by the HIP translation units of libxsmi355.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/xsmi355.h"

namespace xsmi {

// Thread-local error text returned by xsmi_last_error().
void set_error(const char *fmt, ...);
// The stream ops launch on: the library's main stream, or its second stream inside a side section.
// nullptr until xsmi_init succeeded.
hipStream_t stream();
// Side section: launches between side_begin() and side_end() go to the second stream, ordered after all
// earlier main-stream work; side_join() makes the main stream wait for them (it may come much later:
// until then the main stream runs on beside them).
int side_begin();
void side_end();
int side_join();              // no-op when the second stream holds nothing the main stream has not waited for
bool side_pending();
// Inside a side section: spread independent short launches over the second stream (lane 0) and three more streams
// (lanes 1-3), which start after the same point of the main stream; side_lanes_end() makes the second stream wait
// for the others, so that side_join() covers all of them.  Launches of one lane run in order.
constexpr int SIDE_LANES = 4;
int side_lane(int lane);
int side_lanes_end();
bool on_side_stream();
bool capturing();            // a step graph is being recorded: nothing runs, nothing may wait for the device
bool ready();
int cu_count();
// Tuning switches (xsmi_set_option / environment variable / default); the order is that of the table in runtime.hip.
enum Option { OPT_TAP_SK, OPT_SK_SPIN_LIMIT, OPT_TAP_STAGES, OPT_TAP_PERSIST, OPT_CL_HALO, OPT_CL_STEM, OPT_SK_WIDE, OPT_POOL_BWD, OPT_PACK_LANES, OPT_COUNT };
long option(Option o);
// Partial tiles and flags of the even-split convolution kernels for the stream that stream() hands out; allocated
// by xsmi_init, the flags are zero between launches.
constexpr size_t SK_SCRATCH_FLAG_BYTES = 4096;                          // 1024 workgroups
constexpr size_t SK_SCRATCH_PART_BYTES = (size_t)1024 * 16 * 256 * 4;   // 1024 workgroups x one 64 x 64 tile of floats
struct SkScratch {
    uint32_t *flags;
    float *part;
};
SkScratch sk_scratch();
// Device address of the word a kernel sets (system scope) when a bounded wait ran out, and the host-side check:
// XSMI_OK, or XSMI_ERR_RUNTIME with the message set (and, outside a capture, the library reset for further use).
uint32_t *device_error_word();
int check_device_error(const char *where);
// conv_noalloc.hip: resolves the device address of the static scratch array for `device` (the current device)
int noalloc_setup(int device);
// With xsmi_profiling(1) every op brackets its main kernel(s) with two events on
// the library stream; xsmi_last_kernel_ms reads them back.
void prof_begin();
void prof_end();

#define XSMI_REQUIRE_INIT()                                              \
    do {                                                                 \
        if (!xsmi::ready()) {                                            \
            xsmi::set_error("%s: xsmi_init has not been called", __func__); \
            return XSMI_ERR_STATE;                                       \
        }                                                                \
    } while (0)

#define XSMI_CHECK_ARG(cond, ...)                  \
    do {                                           \
        if (!(cond)) {                             \
            xsmi::set_error(__VA_ARGS__);          \
            return XSMI_ERR_INVALID;               \
        }                                          \
    } while (0)

// internal flag of xsmi_conv2d_fwd / xsmi_conv2d_bwd_data (set by xsmi_conv2d_pack): lay the filter out and return
#define XSMI_CONV_PACK_ONLY 0x40000000u
// internal flag of xsmi_conv2d_fwd (set by xsmi_conv2d_fwd_noalloc): stay on the kernels whose scratch is the
// workspace alone (the even-split kernels exchange partial tiles through memory that xsmi_init allocated)
#define XSMI_CONV_WS_ONLY 0x20000000u

#define XSMI_HIP(call)                                                          \
    do {                                                                        \
        hipError_t e_ = (call);                                                 \
        if (e_ != hipSuccess) {                                                 \
            xsmi::set_error("%s failed: %s", #call, hipGetErrorString(e_));     \
            return XSMI_ERR_RUNTIME;                                            \
        }                                                                       \
    } while (0)

#define XSMI_LAUNCH_CHECK(name)                                                 \
    do {                                                                        \
        hipError_t e_ = hipGetLastError();                                      \
        if (e_ != hipSuccess) {                                                 \
            xsmi::set_error("launch of %s failed: %s", name, hipGetErrorString(e_)); \
            return XSMI_ERR_RUNTIME;                                            \
        }                                                                       \
    } while (0)

// Division of a non-negative 31-bit integer by a fixed divisor with one
// multiply-high: q = (umulhi(n, mul) + n) >> shift.
struct FastDiv {
    uint32_t mul;
    uint32_t shift;
    uint32_t d;
};

inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    uint32_t s = 0;
    while ((1ull << s) < d) ++s;
    f.shift = s;
    f.mul = (uint32_t)((((1ull << 32) * ((1ull << s) - d)) / d) + 1);
    return f;
}

__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv &f) {
    return (__umulhi(n, f.mul) + n) >> f.shift;
}

// Workgroups are handed to the 8 XCDs round-robin by linear workgroup id, and each XCD
// has its own L2.  This maps the launch's linear id to a logical id such that every XCD
// works on one contiguous range of logical ids: neighbours in logical order, which share
// operand tiles, then share an L2.  Bijective on [0, total) for any total.
__device__ __forceinline__ uint32_t xcd_contiguous_id(uint32_t lin, uint32_t total) {
    const uint32_t q = total >> 3, rem = total & 7u, xcd = lin & 7u, slot = lin >> 3;
    return xcd * q + (xcd < rem ? xcd : rem) + slot;
}

// tap-major fast path (conv_tap.hip): reduction channels must be a multiple of 32.
// opts: bit 0 = bf16 MFMA operands, bit 1 = the workspace already holds the packed filter, bit 2 = lay the filter
// out in the workspace and return (no activation pointer is touched)
bool tap_path_ok(int reduce_channels);
size_t tap_fwd_ws_bytes(int C, int K, int R, int S);
size_t tap_bwd_data_ws_bytes(int C, int K, int R, int S, int sh, int sw);
int tap_conv_fwd(const float *x, const float *w, const float *bias, float *y, uint8_t *mask, int N, int C, int H, int W,
                 int K, int R, int S, int sh, int sw, int pad, int OH, int OW, int relu, int opts, void *workspace);
int tap_conv_bwd_data(const float *dy, const float *w, float *dx, int N, int C, int H, int W, int K, int R, int S, int sh,
                      int sw, int pad, int OH, int OW, int accumulate, int opts, void *workspace);

// second-generation fp32 tap kernel (conv_tap_sk.hip): 64 x 64 outputs per wave, work split evenly over the resident
// workgroups; needs its own, larger workspace (packed filter + partial tiles)
bool sk_path_ok(int reduce_channels, int rows);
bool sk_bwd_data_ok(int C, int K, int R, int S, int sh, int sw);
bool sk_fwd_pays(int M, int rows, int R, int S, int sh, int sw);          // M = output pixels of the pass
bool sk_bwd_data_pays(int M, int rows, int R, int S, int sh, int sw);
size_t sk_fwd_ws_bytes(int C, int K, int R, int S);
size_t sk_bwd_data_ws_bytes(int C, int K, int R, int S, int sh, int sw);
int sk_conv_fwd(const float *x, const float *w, const float *bias, float *y, uint8_t *mask, int N, int C, int H, int W,
                int K, int R, int S, int sh, int sw, int pad, int OH, int OW, int relu, int opts, void *workspace);
int sk_conv_bwd_data(const float *dy, const float *w, float *dx, int N, int C, int H, int W, int K, int R, int S, int sh,
                     int sw, int pad, int OH, int OW, int accumulate, int opts, void *workspace);

// forward for very few input channels (conv_stem.hip): 1 or 3 channels, square filter of 3, 5 or 7, horizontal stride 2;
// the workspace holds the packed filter followed by a zero-bordered copy of the input
bool stem_fwd_ok(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad);
size_t stem_fwd_ws_bytes(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad);
int stem_conv_fwd(const float *x, const float *w, const float *bias, float *y, uint8_t *mask, int N, int C, int H, int W,
                  int K, int R, int S, int sh, int sw, int pad, int OH, int OW, int relu, int opts, void *workspace);

// bf16 forward on a channels-last bf16 copy of the activations (conv_tap.hip): channels a multiple of 32, or
// at most 8 (a stem); the workspace holds the packed filter followed by the copy
bool nhwc_fwd_ok(int N, int C, int H, int W, int K, int R, int S, int pad);
size_t nhwc_fwd_ws_bytes(int N, int C, int H, int W, int K, int R, int S, int pad);
size_t nhwc_filter_ws_bytes(int C, int K, int R, int S);    // the packed filter alone (input already channels-last)
// x_cl / y_cl: channels-last bf16 tensors [N][H + 2 b][W + 2 b][C] with a zero border b, used instead of x / y when given
int nhwc_conv_fwd(const float *x, const void *x_cl, int xb, const float *w, const float *bias, float *y, void *y_cl, int yb,
                  uint8_t *mask, int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad, int OH, int OW,
                  int relu, int opts, void *workspace);

// 3 x 3, stride-1, pad-1 bf16 forward that stages the bordered channels-last input once for all nine taps
// (conv_cl_halo.hip); called by nhwc_conv_fwd, shares its workspace layout (packed filter, then the copy)
bool halo_fwd_ok(int C, int H, int W, int K, int R, int S, int sh, int sw, int pad, int border);
size_t halo_apk_bytes(int C, int K);
int halo_conv_fwd(const void *xp, size_t xp_bytes, const float *w, void *apk, const float *bias, float *y, void *y_cl,
                  uint8_t *mask, int N, int C, int H, int W, int K, int relu, bool packed);

// first layer (at most 4 channels, 7-row filter, stride 2) with channels-last bf16 output (conv_cl_halo.hip); called by
// nhwc_conv_fwd after it has made the bordered 4-channel copy
bool stem_cl_ok(int C, int H, int W, int K, int R, int S, int sh, int sw, int pad, int OW, int y_border);
size_t stem_cl_apk_bytes();
int stem_cl_conv_fwd(const void *xp, size_t xp_bytes, const float *w, void *apk, const float *bias, void *y_cl, int N, int C,
                     int H, int W, int K, int R, int S, int pad, int OH, int OW, int relu, bool packed);

// weight gradient for the same few-channel layers (conv_stem.hip): horizontal stride 2, output width a multiple of 8,
// filters a multiple of 64, at most 160 filter positions; the workspace holds the copy and the workgroups' partial sums
bool stem_wgrad_ok(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad);
size_t stem_wgrad_ws_bytes(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int pad);
int stem_conv_bwd_weight(const float *dy, const float *x, float *dw, float *db, int N, int C, int H, int W, int K, int R, int S,
                         int sh, int sw, int pad, int OH, int OW, int accumulate, void *workspace);
// dw[k][j] = (accumulate ? dw : 0) + sum over splits of part[split][k][j] (float64, ascending), db likewise from
// dbpart[split][k] when given (conv_wgrad.hip)
int wgrad_reduce_partials(const float *part, float *dw, const float *dbpart, float *db, int K, int J, int Kp, int Jp, int splits,
                          int accumulate);

// tap-major backward-weight (conv_wgrad_tap.hip)
bool wgrad_tap_ok(const float *dy, const float *x, int C, int K, int OH, int OW);
size_t wgrad_tap_ws_bytes(int N, int C, int K, int R, int S, int OH, int OW);
int wgrad_tap(const float *dy, const float *x, float *dw, float *db, int N, int C, int H, int W, int K, int R, int S,
              int sh, int sw, int pad, int OH, int OW, int accumulate, void *workspace);

// ---- global -> LDS direct loads ------------------------------------------
// Written as inline asm on purpose: the compiler orders LDS reads after
// LDS-direct loads it knows about with a full vmcnt(0) wait, which would undo
// the multi-stage prefetch.  The kernels that use these helpers order the loads
// themselves (vmcnt + workgroup barrier) and contain no other instruction that
// depends on M0.
typedef int xsmi_int32x4 __attribute__((ext_vector_type(4)));
typedef unsigned xsmi_uint32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ xsmi_int32x4 make_rsrc(const void *p, uint32_t bytes) {
    uint64_t a = (uint64_t)p;
    xsmi_int32x4 r;
    r.x = (int)(uint32_t)a;
    r.y = (int)(uint32_t)((a >> 32) & 0xffff);   // stride 0: raw buffer
    r.z = (int)bytes;                           // offsets >= bytes read as 0
    r.w = 0x00020000;
    return r;
}

// One dword per lane: LDS[lds_addr + 4*lane] = buffer[voff + soff]; lds_addr and soff are wave-uniform.
__device__ __forceinline__ void load_lds_b32(xsmi_int32x4 rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
#if defined(__HIP_DEVICE_COMPILE__)
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
#endif
}

// Four dwords per lane: LDS[lds_addr + 16*lane .. +15] = buffer[voff + soff .. +15].
__device__ __forceinline__ void load_lds_b128(xsmi_int32x4 rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
#if defined(__HIP_DEVICE_COMPILE__)
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
#endif
}

// The same with the LDS address formed inside the statement as lds_base + IMM (IMM a compile-time constant): a loop
// whose loads go to a few fixed places of each stage then keeps one wave-uniform base alive instead of one address per
// load and stage.  (Addresses formed outside are loop invariants to the compiler, which keeps each in a scalar
// register of its own and, when those run out, in a lane of a vector register: the reload between two MFMAs costs a
// vector instruction and the wait states before a scalar register written by one may be used.)
template <uint32_t IMM>
__device__ __forceinline__ void load_lds_b32_at(xsmi_int32x4 rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
#if defined(__HIP_DEVICE_COMPILE__)
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("s_add_u32 m0, %0, %4\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :: "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff), "n"(IMM) : "memory", "scc");
#endif
}
template <uint32_t IMM>
__device__ __forceinline__ void load_lds_b128_at(xsmi_int32x4 rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
#if defined(__HIP_DEVICE_COMPILE__)
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("s_add_u32 m0, %0, %4\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff), "n"(IMM) : "memory", "scc");
#endif
}

// s_waitcnt that constrains only the vector-memory counter (gfx9 encoding:
// vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
#endif
}

// s_waitcnt on the LDS/scalar-memory counter only (vmcnt and expcnt left at their maxima).
__device__ __forceinline__ void wait_lgkmcnt0() {
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_s_waitcnt(15 | (3 << 14) | (7 << 4) | (0 << 8));
#endif
}

// Workgroup barrier the compiler may not move memory accesses across; it carries
// no waits of its own.
__device__ __forceinline__ void block_barrier() {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#endif
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

}  // namespace xsmi
