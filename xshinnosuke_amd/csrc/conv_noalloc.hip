// xsmi_conv2d_fwd_noalloc: the convolution forward for callers that can neither allocate device memory nor
// bring a workspace (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
// It runs the very kernels of xsmi_conv2d_fwd; the scratch those kernels need (the filter in the kernel's LDS
// order, the persistent kernel's tile counters) lives in a device array that is part of the library's code
// object and therefore exists, once per GPU, from the moment the library is loaded until the process ends.
#include "xsmi_internal.h"

namespace xsmi {
size_t conv_fwd_ws_bytes(int C, int K, int R, int S);
}

namespace {

// 16 MiB holds the packed filter of every fp32 ResNet-18 layer (the largest, 512 x 512 x 3 x 3, needs 9.44 MB).
constexpr size_t SCRATCH_BYTES = XSMI_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

// In host code `scratch` is only a handle for the runtime, not a device address.  The address of this GPU's copy
// of the array is looked up once, in xsmi_init with the device current; everything below uses g_scratch.
constexpr int MAX_DEVICES = 64;
void *g_scratch[MAX_DEVICES] = {nullptr};

}  // namespace

namespace xsmi {

int noalloc_setup(int device) {
    if (device < 0 || device >= MAX_DEVICES) {
        set_error("xsmi_init: device %d beyond the %d devices the static scratch table covers", device, MAX_DEVICES);
        return XSMI_ERR_INVALID;
    }
    if (g_scratch[device]) return XSMI_OK;
    void *ptr = nullptr;
    XSMI_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr || ((uintptr_t)ptr & 255) != 0) {
        set_error("xsmi_init: static scratch array resolved to %p", ptr);
        return XSMI_ERR_RUNTIME;
    }
    g_scratch[device] = ptr;
    return XSMI_OK;
}

}  // namespace xsmi

extern "C" {

int xsmi_conv2d_fwd_noalloc(const float *x, const float *w, const float *bias, float *y, uint8_t *neg_mask, int N, int C,
                            int H, int W, int K, int R, int S, int sh, int sw, int pad, unsigned flags) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && H > 0 && W > 0 && K > 0 && R > 0 && S > 0 && sh > 0 && sw > 0 && pad >= 0,
                   "xsmi_conv2d_fwd_noalloc: bad geometry");
    XSMI_CHECK_ARG((flags & ~(XSMI_CONV_RELU | XSMI_CONV_BF16)) == 0,
                   "xsmi_conv2d_fwd_noalloc: flags 0x%x (only XSMI_CONV_RELU and XSMI_CONV_BF16 apply: the scratch is "
                   "shared by all calls, so it never counts as already packed)", flags);
    const size_t need = xsmi::conv_fwd_ws_bytes(C, K, R, S);
    XSMI_CHECK_ARG(need <= SCRATCH_BYTES,
                   "xsmi_conv2d_fwd_noalloc: this filter needs %zu bytes of scratch, the static buffer holds %zu; use "
                   "xsmi_conv2d_fwd with a workspace", need, SCRATCH_BYTES);
    int device = -1;
    XSMI_HIP(hipGetDevice(&device));
    XSMI_CHECK_ARG(device >= 0 && device < MAX_DEVICES && g_scratch[device] != nullptr,
                   "xsmi_conv2d_fwd_noalloc: the current device %d is not the one xsmi_init bound", device);
    return xsmi_conv2d_fwd(x, w, bias, y, neg_mask, N, C, H, W, K, R, S, sh, sw, pad, flags | XSMI_CONV_WS_ONLY, g_scratch[device],
                           SCRATCH_BYTES);
}

}  // extern "C"
