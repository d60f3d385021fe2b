// Internal helpers shared by the HIP translation units of libxsmi355.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/xsmi355.h"

namespace xsmi {

// Thread-local error text returned by xsmi_last_error().
void set_error(const char *fmt, ...);
// Library stream; nullptr until xsmi_init succeeded.
hipStream_t stream();
bool ready();
int cu_count();
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

// tap-major fast path (conv_tap.hip): reduction channels must be a multiple of 32
bool tap_path_ok(int reduce_channels);
size_t tap_fwd_ws_bytes(int C, int K, int R, int S);
size_t tap_bwd_data_ws_bytes(int C, int K, int R, int S, int sh, int sw);
int tap_conv_fwd(const float *x, const float *w, const float *bias, float *y, uint8_t *mask, int N, int C, int H, int W,
                 int K, int R, int S, int sh, int sw, int pad, int OH, int OW, int relu, void *workspace);
int tap_conv_bwd_data(const float *dy, const float *w, float *dx, int N, int C, int H, int W, int K, int R, int S, int sh,
                      int sw, int pad, int OH, int OW, int accumulate, void *workspace);

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

}  // namespace xsmi
