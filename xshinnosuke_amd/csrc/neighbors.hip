// Element-wise, normalisation and reduction kernels for the ops that sit between two
// convolutions in a network (ReLU, residual add, batch norm, average pool, dense layer,
// softmax cross-entropy, SGD).  All are HBM-bound float32 passes: 128-bit accesses where
// the layout allows it, grid-stride loops, float64 for the long reductions.
#include "xsmi_internal.h"

namespace {

constexpr int BN_SPLIT = 32;     // partial reductions per channel

inline dim3 grid_for(size_t work_items, int per_block = 256, int cap_per_cu = 16) {
    size_t blocks = (work_items + per_block - 1) / per_block;
    size_t cap = (size_t)(xsmi::cu_count() > 0 ? xsmi::cu_count() : 256) * cap_per_cu;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return dim3((unsigned)blocks);
}

// Generic element-wise pass: vectorised by 4 when every pointer is 16-byte aligned.
template <typename F>
__global__ void __launch_bounds__(256) ew_kernel(size_t n, int vec, F f) {
    size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        size_t n4 = n >> 2;
        for (size_t j = i; j < n4; j += stride) f.quad(j);
        for (size_t j = (n4 << 2) + i; j < n; j += stride) f.one(j);
    } else {
        for (size_t j = i; j < n; j += stride) f.one(j);
    }
}

inline int aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

struct AxpyF {
    float *y; const float *x; float a;
    __device__ void one(size_t i) const { y[i] += a * x[i]; }
    __device__ void quad(size_t j) const {
        float4 v = reinterpret_cast<const float4 *>(x)[j];
        float4 o = reinterpret_cast<float4 *>(y)[j];
        o.x += a * v.x; o.y += a * v.y; o.z += a * v.z; o.w += a * v.w;
        reinterpret_cast<float4 *>(y)[j] = o;
    }
};
struct FillF {
    float *o; float v;
    __device__ void one(size_t i) const { o[i] = v; }
    __device__ void quad(size_t j) const { reinterpret_cast<float4 *>(o)[j] = make_float4(v, v, v, v); }
};
struct AddF {
    const float *a, *b; float *o;
    __device__ void one(size_t i) const { o[i] = a[i] + b[i]; }
    __device__ void quad(size_t j) const {
        float4 u = reinterpret_cast<const float4 *>(a)[j], v = reinterpret_cast<const float4 *>(b)[j];
        reinterpret_cast<float4 *>(o)[j] = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
    }
};
struct AddReluF {
    const float *a, *b; float *o; uint8_t *m;        // m (optional): 1 where the sum is < 0
    __device__ static float f(float t) { return t > 0.f ? t : 0.f; }
    __device__ void one(size_t i) const {
        const float t = a[i] + b[i];
        if (m) m[i] = t < 0.f ? 1 : 0;
        o[i] = f(t);
    }
    __device__ void quad(size_t j) const {
        float4 u = reinterpret_cast<const float4 *>(a)[j], v = reinterpret_cast<const float4 *>(b)[j];
        const float4 t = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
        if (m) reinterpret_cast<uchar4 *>(m)[j] = make_uchar4(t.x < 0.f, t.y < 0.f, t.z < 0.f, t.w < 0.f);
        reinterpret_cast<float4 *>(o)[j] = make_float4(f(t.x), f(t.y), f(t.z), f(t.w));
    }
};
struct ScaleF {
    const float *a; float *o; float s, t;
    __device__ void one(size_t i) const { o[i] = s * a[i] + t; }
    __device__ void quad(size_t j) const {
        float4 u = reinterpret_cast<const float4 *>(a)[j];
        reinterpret_cast<float4 *>(o)[j] = make_float4(s * u.x + t, s * u.y + t, s * u.z + t, s * u.w + t);
    }
};
struct ReluF {
    const float *x; float *y;
    __device__ void one(size_t i) const { float v = x[i]; y[i] = v > 0.f ? v : 0.f; }
    __device__ void quad(size_t j) const {
        float4 u = reinterpret_cast<const float4 *>(x)[j];
        reinterpret_cast<float4 *>(y)[j] = make_float4(u.x > 0.f ? u.x : 0.f, u.y > 0.f ? u.y : 0.f, u.z > 0.f ? u.z : 0.f,
                                                       u.w > 0.f ? u.w : 0.f);
    }
};
struct ReluMaskF {
    const float *x; float *y; uint8_t *m;
    __device__ void one(size_t i) const { float v = x[i]; m[i] = v < 0.f ? 1 : 0; y[i] = v > 0.f ? v : 0.f; }
    __device__ void quad(size_t j) const {
        float4 u = reinterpret_cast<const float4 *>(x)[j];
        reinterpret_cast<uchar4 *>(m)[j] = make_uchar4(u.x < 0.f, u.y < 0.f, u.z < 0.f, u.w < 0.f);
        reinterpret_cast<float4 *>(y)[j] = make_float4(u.x > 0.f ? u.x : 0.f, u.y > 0.f ? u.y : 0.f, u.z > 0.f ? u.z : 0.f,
                                                       u.w > 0.f ? u.w : 0.f);
    }
};
struct ReluBwdF {
    const float *dy, *pre; float *dx;
    __device__ void one(size_t i) const { dx[i] = pre[i] < 0.f ? 0.f : dy[i]; }
    __device__ void quad(size_t j) const {
        float4 g = reinterpret_cast<const float4 *>(dy)[j], p = reinterpret_cast<const float4 *>(pre)[j];
        reinterpret_cast<float4 *>(dx)[j] = make_float4(p.x < 0.f ? 0.f : g.x, p.y < 0.f ? 0.f : g.y, p.z < 0.f ? 0.f : g.z,
                                                        p.w < 0.f ? 0.f : g.w);
    }
};
// sigmoid (kind 1) and tanh (kind 2), forward and the backward written in terms of the forward's output y
struct ActF {
    const float *x; float *y; int kind;
    __device__ float f(float v) const { return kind == 1 ? 1.f / (1.f + expf(-v)) : tanhf(v); }
    __device__ void one(size_t i) const { y[i] = f(x[i]); }
    __device__ void quad(size_t j) const {
        float4 u = reinterpret_cast<const float4 *>(x)[j];
        reinterpret_cast<float4 *>(y)[j] = make_float4(f(u.x), f(u.y), f(u.z), f(u.w));
    }
};
struct ActBwdF {
    const float *dy, *y; float *dx; int kind;
    __device__ float g(float d, float o) const { return kind == 1 ? d * o * (1.f - o) : d * (1.f - o * o); }
    __device__ void one(size_t i) const { dx[i] = g(dy[i], y[i]); }
    __device__ void quad(size_t j) const {
        float4 d = reinterpret_cast<const float4 *>(dy)[j], o = reinterpret_cast<const float4 *>(y)[j];
        reinterpret_cast<float4 *>(dx)[j] = make_float4(g(d.x, o.x), g(d.y, o.y), g(d.z, o.z), g(d.w, o.w));
    }
};
struct LerpF {
    float *m; const float *c; float mom;
    __device__ void one(size_t i) const { m[i] = mom * m[i] + (1.f - mom) * c[i]; }
    __device__ void quad(size_t j) const {
        for (int e = 0; e < 4; ++e) one(4 * j + e);
    }
};

template <typename F>
int launch_ew(const char *name, size_t n, int vec, F f) {
    if (n == 0) return XSMI_OK;
    hipLaunchKernelGGL(ew_kernel<F>, grid_for(vec ? (n + 3) / 4 : n), dim3(256), 0, xsmi::stream(), n, vec, f);
    XSMI_LAUNCH_CHECK(name);
    return XSMI_OK;
}

// y_t[i] += a * x_t[i] for up to AXPY_GROUP tensors in one launch: the tensors are concatenated in units of
// 1024 elements (one workgroup each); first[t] is the first workgroup of tensor t.  The table travels in the
// kernel arguments, so no device-side pointer array has to be kept up to date.
constexpr int AXPY_GROUP = 48;
struct AxpyMulti {
    float *y[AXPY_GROUP];
    const float *x[AXPY_GROUP];
    uint32_t n[AXPY_GROUP];
    uint32_t first[AXPY_GROUP + 1];
    int count;
    float a;
};
__global__ void __launch_bounds__(256) axpy_multi_kernel(AxpyMulti m) {
    int lo = 0, hi = m.count - 1;                    // last tensor whose first workgroup is <= blockIdx.x
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (m.first[mid] <= blockIdx.x) lo = mid; else hi = mid - 1;
    }
    float *y = m.y[lo];
    const float *x = m.x[lo];
    const uint32_t n = m.n[lo];
    const uint32_t base = (blockIdx.x - m.first[lo]) * 1024u;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const uint32_t i = base + u * 256u + threadIdx.x;
        if (i < n) y[i] += m.a * x[i];
    }
}

// ---- block reductions ------------------------------------------------------
__device__ __forceinline__ double wave_sum(double v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ double block_sum(double v, double *sm) {   // 256 threads
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    return sm[0] + sm[1] + sm[2] + sm[3];
}

template <int NT>
__device__ __forceinline__ double block_sum_n(double v, double *sm) {   // NT threads, sm[NT / 64]; waves added in order
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    double r = sm[0];
#pragma unroll
    for (int w = 1; w < NT / 64; ++w) r += sm[w];
    return r;
}

// channel of flat element i of an (N, C, HW) tensor (tensors stay below 2^29 elements)
struct ChanIdx {
    xsmi::FastDiv dHW, dC;
    int C;
    __device__ __forceinline__ int operator()(uint32_t i) const {
        uint32_t q = xsmi::fdiv(i, dHW);
        return (int)(q - xsmi::fdiv(q, dC) * (uint32_t)C);
    }
};
inline ChanIdx make_chan(int C, int HW) {
    ChanIdx ci;
    ci.dHW = xsmi::make_fastdiv(HW);
    ci.dC = xsmi::make_fastdiv(C);
    ci.C = C;
    return ci;
}

// Stores of results that this kernel does not read again: non-temporal, lanes contiguous.
typedef float nt_f4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void nt_store4(float *p, float a, float b, float c, float d) {
    nt_f4 v; v.x = a; v.y = b; v.z = c; v.w = d;
    __builtin_nontemporal_store(v, reinterpret_cast<nt_f4 *>(p));
}
__device__ __forceinline__ void nt_store_mask4(uint8_t *p, unsigned a, unsigned b, unsigned c, unsigned d) {
    __builtin_nontemporal_store((uint32_t)(a | (b << 8) | (c << 16) | (d << 24)), reinterpret_cast<uint32_t *>(p));
}

// ---- batch norm --------------------------------------------------------------
// pass 1: per (channel, split) partial sums of a and a*b over the N*HW elements of the channel
// `zero` (optional, one byte per element): elements whose byte is set count as a == 0 (the gradient of a fused
// ReLU that was clipped).  A channel's elements are numbered image by image in load units (float4 when VEC:
// HW % 4 == 0, so planes are 16-byte aligned; else floats); split sp owns units [sp*per, (sp+1)*per), a fixed
// assignment, so the sums do not depend on timing.  Each thread issues four independent loads per operand
// before it adds: a block has only a few units per thread, and one load at a time would leave it waiting on
// memory latency for most of its life.
template <bool VEC>
__global__ void __launch_bounds__(256) bn_partial_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                          const uint8_t *__restrict__ zero, double *__restrict__ part,
                                                          int C, int HW, xsmi::FastDiv dU, uint32_t total, uint32_t per,
                                                          const float *__restrict__ mean, const float *__restrict__ sqrtvar) {
    constexpr int W = VEC ? 4 : 1, UNR = 4;
    __shared__ double sm[4];
    const int c = blockIdx.x, sp = blockIdx.y;
    // with `mean`, b holds the values before normalisation and (b - mean) / sqrtvar is formed here
    const float mu = mean ? mean[c] : 0.f, rs = mean ? sqrtvar[c] : 1.f;
    const uint32_t beg = (uint32_t)sp * per, end = min(total, beg + per);
    double s0 = 0.0, s1 = 0.0;
    for (uint32_t e0 = beg + threadIdx.x; e0 < end; e0 += 256 * UNR) {
        float u[UNR][W], v[UNR][W];
        unsigned char z[UNR][W];
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            const uint32_t e = e0 + 256u * k;
            const bool ok = e < end;
            const uint32_t j = xsmi::fdiv(e, dU), i = e - j * dU.d;
            const size_t off = ((size_t)j * C + c) * (size_t)HW + (size_t)i * W;
            if (VEC) {
                *reinterpret_cast<float4 *>(u[k]) = ok ? *reinterpret_cast<const float4 *>(a + off) : make_float4(0.f, 0.f, 0.f, 0.f);
                if (b) *reinterpret_cast<float4 *>(v[k]) = ok ? *reinterpret_cast<const float4 *>(b + off) : make_float4(0.f, 0.f, 0.f, 0.f);
                if (zero) *reinterpret_cast<uchar4 *>(z[k]) = ok ? *reinterpret_cast<const uchar4 *>(zero + off) : make_uchar4(0, 0, 0, 0);
            } else {
                u[k][0] = ok ? a[off] : 0.f;
                if (b) v[k][0] = ok ? b[off] : 0.f;
                if (zero) z[k][0] = ok ? zero[off] : 0;
            }
        }
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            double t0 = 0.0, t1 = 0.0;
#pragma unroll
            for (int q = 0; q < W; ++q) {
                const float uu = (zero && z[k][q]) ? 0.f : u[k][q];
                const float vv = b ? (mean ? (v[k][q] - mu) / rs : v[k][q]) : uu;
                t0 += (double)uu;
                t1 += (double)uu * (double)vv;
            }
            s0 += t0;
            s1 += t1;
        }
    }
    s0 = block_sum(s0, sm);
    s1 = block_sum(s1, sm);
    if (threadIdx.x == 0) {
        part[((size_t)c * BN_SPLIT + sp) * 2 + 0] = s0;
        part[((size_t)c * BN_SPLIT + sp) * 2 + 1] = s1;
    }
}
// Split of a channel's N*HW elements over up to BN_SPLIT blocks: at least 512 load units per block.
struct BnSplit { int nsplit; uint32_t total, per; xsmi::FastDiv dU; bool vec; };
static BnSplit bn_split(int N, int HW, bool vec) {
    BnSplit r;
    r.vec = vec;
    const uint32_t U = vec ? (uint32_t)HW >> 2 : (uint32_t)HW;
    r.total = (uint32_t)N * U;
    uint32_t s = r.total / 512;
    if (s < 1) s = 1;
    if (s > (uint32_t)BN_SPLIT) s = BN_SPLIT;
    r.per = (r.total + s - 1) / s;
    r.nsplit = (int)((r.total + r.per - 1) / r.per);
    r.dU = xsmi::make_fastdiv(U);
    return r;
}
static void launch_bn_partial(hipStream_t st, const float *a, const float *b, const uint8_t *zero, double *part, int C, int HW,
                              const BnSplit &sp, const float *mean, const float *sqrtvar) {
    if (sp.vec)
        hipLaunchKernelGGL(bn_partial_kernel<true>, dim3(C, sp.nsplit), dim3(256), 0, st, a, b, zero, part, C, HW, sp.dU,
                           sp.total, sp.per, mean, sqrtvar);
    else
        hipLaunchKernelGGL(bn_partial_kernel<false>, dim3(C, sp.nsplit), dim3(256), 0, st, a, b, zero, part, C, HW, sp.dU,
                           sp.total, sp.per, mean, sqrtvar);
}
// Sums of one channel's partials: the same fixed tree in every block of the channel, so all of them (and the one
// that stores the statistics) work with identical values.  sm: two doubles of LDS.
__device__ __forceinline__ void bn_channel_sums(const double *__restrict__ part, int c, int nsplit, double *sm, double &s0,
                                                double &s1) {
    if (threadIdx.x < 64) {
        double a = 0.0, b = 0.0;
        if ((int)threadIdx.x < nsplit) {
            a = part[((size_t)c * BN_SPLIT + threadIdx.x) * 2 + 0];
            b = part[((size_t)c * BN_SPLIT + threadIdx.x) * 2 + 1];
        }
        a = wave_sum(a);
        b = wave_sum(b);
        if (threadIdx.x == 0) { sm[0] = a; sm[1] = b; }
    }
    __syncthreads();
    s0 = sm[0];
    s1 = sm[1];
}
// pass 2 of the forward: block (c, sp) turns the channel's partial sums into mean and sqrt(var + eps) (block sp == 0
// also stores them and updates the moving statistics: m = momentum*m + (1-momentum)*cur, as xsmi_lerp computes it)
// and normalises its units of the channel, numbered as in bn_partial_kernel.  neg_mask != nullptr fuses a ReLU:
// mask = pre-activation < 0, y = max(pre-activation, 0).  residual != nullptr: a tensor of x's shape that is added to
// the normalised value before the ReLU (the end of a residual block as one pass).
struct BnFwdOut {
    float *y, *xhat, *sqrtvar, *mean, *var, *moving_mean, *moving_var;
    uint8_t *neg_mask;
    const float *residual;
};
template <bool VEC>
__global__ void __launch_bounds__(256) bn_apply_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                                        const float *__restrict__ beta, const double *__restrict__ part,
                                                        int nsplit_part, double m, float eps, float momentum, BnFwdOut o,
                                                        int C, int HW, xsmi::FastDiv dU, uint32_t total, uint32_t per) {
    constexpr int W = VEC ? 4 : 1, UNR = 4;
    __shared__ double sm[2];
    const int c = blockIdx.x, sp = blockIdx.y;
    double s0, s1;
    bn_channel_sums(part, c, nsplit_part, sm, s0, s1);
    const double mu_d = s0 / m;
    double v = s1 / m - mu_d * mu_d;
    if (v < 0.0) v = 0.0;
    const float mu = (float)mu_d, rs = (float)sqrt(v + (double)eps), g = gamma[c], bt = beta[c];
    if (sp == 0 && threadIdx.x == 0) {
        o.mean[c] = mu;
        o.var[c] = (float)v;
        o.sqrtvar[c] = rs;
        if (o.moving_mean) {
            o.moving_mean[c] = momentum * o.moving_mean[c] + (1.f - momentum) * mu;
            o.moving_var[c] = momentum * o.moving_var[c] + (1.f - momentum) * (float)v;
        }
    }
    const uint32_t beg = (uint32_t)sp * per, end = min(total, beg + per);
    for (uint32_t e0 = beg + threadIdx.x; e0 < end; e0 += 256 * UNR) {
        float xv[UNR][W], rv[UNR][W];
        size_t off[UNR];
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            const uint32_t e = e0 + 256u * k;
            const uint32_t j = xsmi::fdiv(e, dU), i = e - j * dU.d;
            off[k] = ((size_t)j * C + c) * (size_t)HW + (size_t)i * W;
#pragma unroll
            for (int q = 0; q < W; ++q) rv[k][q] = 0.f;
            if (e < end) {
                if (VEC) *reinterpret_cast<float4 *>(xv[k]) = *reinterpret_cast<const float4 *>(x + off[k]); else xv[k][0] = x[off[k]];
                if (o.residual) {
                    if (VEC) *reinterpret_cast<float4 *>(rv[k]) = *reinterpret_cast<const float4 *>(o.residual + off[k]);
                    else rv[k][0] = o.residual[off[k]];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            if (e0 + 256u * k >= end) break;
            float hv[W], yv[W];
            unsigned char mv[W];
#pragma unroll
            for (int q = 0; q < W; ++q) {
                hv[q] = (xv[k][q] - mu) / rs;
                float pre = g * hv[q] + bt;
                if (o.residual) pre += rv[k][q];
                mv[q] = pre < 0.f ? 1 : 0;
                yv[q] = (o.neg_mask && pre < 0.f) ? 0.f : pre;
            }
            if (VEC) {
                if (o.xhat) *reinterpret_cast<float4 *>(o.xhat + off[k]) = *reinterpret_cast<float4 *>(hv);
                *reinterpret_cast<float4 *>(o.y + off[k]) = *reinterpret_cast<float4 *>(yv);
                if (o.neg_mask) *reinterpret_cast<uchar4 *>(o.neg_mask + off[k]) = make_uchar4(mv[0], mv[1], mv[2], mv[3]);
            } else {
                if (o.xhat) o.xhat[off[k]] = hv[0];
                o.y[off[k]] = yv[0];
                if (o.neg_mask) o.neg_mask[off[k]] = mv[0];
            }
        }
    }
}
// Pass 2 of the forward with the ReLU and the 3 x 3 / stride 2 / pad 1 max-pool that follow it (the head of a ResNet):
// block (c, sp) forms the channel's statistics like bn_apply_kernel and then produces pooled outputs of that channel,
// two per thread and step (unit u of the channel = (image, output row, output pair)): the 3 x 5 inputs of the pair are
// normalised and clipped in registers, exactly as bn_apply_kernel would have stored them, and compared exactly as
// maxpool_fwd_3x3s2p1 compares them (first maximum in window order wins, the zero border competes).  The normalised
// tensor itself is never written; the sign mask of the pre-activation is (every input element once, by the thread whose
// pair has it in window rows 1 and 2 at columns 4j .. 4j + 3).  H even, W a multiple of 4.
typedef float bn_f2v __attribute__((ext_vector_type(2)));
__global__ void __launch_bounds__(256) bn_relu_maxpool_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                                               const float *__restrict__ beta, const double *__restrict__ part,
                                                               int nsplit_part, double m, float eps, float momentum, BnFwdOut o,
                                                               uint8_t *__restrict__ idx, int C, int H, int W,
                                                               xsmi::FastDiv dQ, xsmi::FastDiv dOHQ, uint32_t total, uint32_t per) {
    __shared__ double sm[2];
    const int c = blockIdx.x, sp = blockIdx.y;
    double s0, s1;
    bn_channel_sums(part, c, nsplit_part, sm, s0, s1);
    const double mu_d = s0 / m;
    double var = s1 / m - mu_d * mu_d;
    if (var < 0.0) var = 0.0;
    const float mu = (float)mu_d, rs = (float)sqrt(var + (double)eps), g = gamma[c], bt = beta[c];
    if (sp == 0 && threadIdx.x == 0) {
        o.mean[c] = mu;
        o.var[c] = (float)var;
        o.sqrtvar[c] = rs;
        if (o.moving_mean) {
            o.moving_mean[c] = momentum * o.moving_mean[c] + (1.f - momentum) * mu;
            o.moving_var[c] = momentum * o.moving_var[c] + (1.f - momentum) * (float)var;
        }
    }
    const int OH = H >> 1, OW = W >> 1, Q = OW >> 1;
    const uint32_t beg = (uint32_t)sp * per, end = min(total, beg + per);
    auto act = [&](float xv, unsigned char &neg) {
        const float pre = g * ((xv - mu) / rs) + bt;
        neg = pre < 0.f ? 1 : 0;
        return pre < 0.f ? 0.f : pre;
    };
    // two units per thread and step, the loads of both before the first use (a unit past the end repeats the first
    // one's loads and stores nothing)
    for (uint32_t u0 = beg + threadIdx.x; u0 < end; u0 += 512) {
        constexpr int UNR = 2;
        bool ok[UNR], have[UNR][3];
        int oh[UNR], jj[UNR];
        size_t pl[UNR];
        float4 v[UNR][3];
        float lf[UNR][3];
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            ok[k] = u0 + 256u * k < end;
            const uint32_t u = ok[k] ? u0 + 256u * k : u0;
            const uint32_t n = xsmi::fdiv(u, dOHQ), rem = u - n * dOHQ.d;
            oh[k] = (int)xsmi::fdiv(rem, dQ);
            jj[k] = (int)rem - oh[k] * Q;
            pl[k] = (size_t)n * C + c;
            const float *plane = x + pl[k] * (size_t)H * W;
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                const int ih = 2 * oh[k] - 1 + r;
                have[k][r] = (unsigned)ih < (unsigned)H;
                v[k][r] = make_float4(0.f, 0.f, 0.f, 0.f);
                lf[k][r] = 0.f;
                if (have[k][r]) {
                    v[k][r] = *reinterpret_cast<const float4 *>(plane + (size_t)ih * W + 4 * jj[k]);
                    if (jj[k] > 0) lf[k][r] = plane[(size_t)ih * W + 4 * jj[k] - 1];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            if (!ok[k]) break;
            const int j = jj[k];
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                unsigned char nl, n0, n1, n2, n3;
                if (have[k][r]) {                      // a row outside the image is the pool's zero border as it is
                    lf[k][r] = j > 0 ? act(lf[k][r], nl) : 0.f;
                    v[k][r].x = act(v[k][r].x, n0); v[k][r].y = act(v[k][r].y, n1);
                    v[k][r].z = act(v[k][r].z, n2); v[k][r].w = act(v[k][r].w, n3);
                    if (r > 0)
                        nt_store_mask4(o.neg_mask + (pl[k] * H + (2 * oh[k] - 1 + r)) * (size_t)W + 4 * j, n0, n1, n2, n3);
                }
            }
            float b0 = 0.f, b1 = 0.f;
            int w0 = 0, w1 = 0;
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                const float left = lf[k][r];
                if (r == 0 || left > b0) { b0 = left; w0 = r * 3 + 0; }
                if (v[k][r].x > b0) { b0 = v[k][r].x; w0 = r * 3 + 1; }
                if (v[k][r].y > b0) { b0 = v[k][r].y; w0 = r * 3 + 2; }
                if (r == 0 || v[k][r].y > b1) { b1 = v[k][r].y; w1 = r * 3 + 0; }
                if (v[k][r].z > b1) { b1 = v[k][r].z; w1 = r * 3 + 1; }
                if (v[k][r].w > b1) { b1 = v[k][r].w; w1 = r * 3 + 2; }
            }
            const size_t ob = (pl[k] * OH + oh[k]) * (size_t)OW + 2 * j;
            bn_f2v yv; yv.x = b0; yv.y = b1;
            __builtin_nontemporal_store(yv, reinterpret_cast<bn_f2v *>(o.y + ob));
            if (idx) __builtin_nontemporal_store((unsigned short)(w0 | (w1 << 8)), reinterpret_cast<unsigned short *>(idx + ob));
        }
    }
}
// pass 2 of the backward: block (c, sp) turns the partial sums into dbeta = sum(dy) and dgamma = sum(dy*xhat) (block
// sp == 0 stores them) and writes dx for its units of the channel.  With `mean`, xhat holds the values before
// normalisation and (xhat - mean) / sqrtvar is formed here.
template <bool VEC>
__global__ void __launch_bounds__(256) bn_bwd_apply_kernel(const float *__restrict__ dy, const float *__restrict__ xhat,
                                                            const float *__restrict__ sqrtvar, const float *__restrict__ gamma,
                                                            const double *__restrict__ part, int nsplit_part,
                                                            float *__restrict__ dgamma, float *__restrict__ dbeta,
                                                            const uint8_t *__restrict__ zero, float *__restrict__ dx, float m,
                                                            const float *__restrict__ mean, int C, int HW, xsmi::FastDiv dU,
                                                            uint32_t total, uint32_t per) {
    constexpr int W = VEC ? 4 : 1, UNR = 4;
    __shared__ double sm[2];
    const int c = blockIdx.x, sp = blockIdx.y;
    double s0, s1;
    bn_channel_sums(part, c, nsplit_part, sm, s0, s1);
    const float db = (float)s0, dg = (float)s1;
    if (sp == 0 && threadIdx.x == 0) {
        dbeta[c] = db;
        dgamma[c] = dg;
    }
    const float rs = sqrtvar[c], mu = mean ? mean[c] : 0.f, g = gamma[c], den = m * rs;
    const uint32_t beg = (uint32_t)sp * per, end = min(total, beg + per);
    for (uint32_t e0 = beg + threadIdx.x; e0 < end; e0 += 256 * UNR) {
        float gv[UNR][W], hv[UNR][W];
        unsigned char zv[UNR][W];
        size_t off[UNR];
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            const uint32_t e = e0 + 256u * k;
            const uint32_t j = xsmi::fdiv(e, dU), i = e - j * dU.d;
            off[k] = ((size_t)j * C + c) * (size_t)HW + (size_t)i * W;
            if (e < end) {
                if (VEC) {
                    *reinterpret_cast<float4 *>(gv[k]) = *reinterpret_cast<const float4 *>(dy + off[k]);
                    *reinterpret_cast<float4 *>(hv[k]) = *reinterpret_cast<const float4 *>(xhat + off[k]);
                    if (zero) *reinterpret_cast<uchar4 *>(zv[k]) = *reinterpret_cast<const uchar4 *>(zero + off[k]);
                } else {
                    gv[k][0] = dy[off[k]];
                    hv[k][0] = xhat[off[k]];
                    if (zero) zv[k][0] = zero[off[k]];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            if (e0 + 256u * k >= end) break;
            float ov[W];
#pragma unroll
            for (int q = 0; q < W; ++q) {
                const float d = (zero && zv[k][q]) ? 0.f : gv[k][q];
                const float h = mean ? (hv[k][q] - mu) / rs : hv[k][q];
                // gamma*(m*dy - sum(dy) - xhat*sum(dy*xhat)) / (m*sqrtvar); the sums carry one factor gamma in the reference
                ov[q] = g * (m * d - db - h * dg) / den;
            }
            if (VEC) *reinterpret_cast<float4 *>(dx + off[k]) = *reinterpret_cast<float4 *>(ov); else dx[off[k]] = ov[0];
        }
    }
}

// The backward of bn_relu_maxpool_kernel's chain: the gradient of the 3 x 3 / stride 2 / pad 1 max-pool is not stored
// as a tensor of the input's size and read twice, it is formed where the normalisation's two backward passes need it.
// A unit is columns 4j .. 4j + 3 of the input rows 2a and 2a + 1 of one plane: their routed gradients come from the
// pooled rows a and a + 1, columns 2j .. 2j + 2 (gradient and window index), as in maxpool_bwd_3x3s2p1: one, two, two
// and four contributors per cell, the four-term cells added in float64 (the reference's order), -0 turned into +0.
struct PoolRouted { float e[4], o[4]; };
__device__ __forceinline__ PoolRouted pool_routed_3x3s2p1(const float *__restrict__ dp, const uint8_t *__restrict__ idx,
                                                          size_t obase, int OH, int OW, int a, int j) {
    float gv[2][3];
    int iv[2][3];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int oh = a + q;                          // a + 1 == OH: below the last output row
        float2 gg = make_float2(0.f, 0.f);
        int i0 = -1, i1 = -1, in = -1;
        float gn = 0.f;
        const size_t ro = obase + (size_t)oh * OW + 2 * j;
        if (oh < OH) {
            gg = *reinterpret_cast<const float2 *>(dp + ro);
            const uchar2 ii = *reinterpret_cast<const uchar2 *>(idx + ro);
            i0 = ii.x; i1 = ii.y;
            if (2 * j + 2 < OW) { gn = dp[ro + 2]; in = idx[ro + 2]; }
        }
        gv[q][0] = gg.x + 0.f; gv[q][1] = gg.y + 0.f; gv[q][2] = gn + 0.f;
        iv[q][0] = i0; iv[q][1] = i1; iv[q][2] = in;
    }
    auto pick = [&](int q, int m, int tap) { return iv[q][m] == tap ? gv[q][m] : 0.f; };
    PoolRouted r;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        r.e[2 * m] = pick(0, m, 4);
        r.e[2 * m + 1] = pick(0, m + 1, 3) + pick(0, m, 5);
        r.o[2 * m] = pick(1, m, 1) + pick(0, m, 7);
        r.o[2 * m + 1] = (float)((((double)pick(1, m + 1, 0) + (double)pick(1, m, 2)) + (double)pick(0, m + 1, 6)) +
                                 (double)pick(0, m, 8));
    }
    return r;
}
// APPLY false: pass 1, per (channel, split) partial sums of dy and dy * xhat; true: pass 2, dx.  Units of a channel are
// numbered (image, row pair, column quad); split sp owns units [sp * per, (sp + 1) * per).
template <bool APPLY>
__global__ void __launch_bounds__(256) bn_bwd_maxpool_kernel(const float *__restrict__ dp, const uint8_t *__restrict__ idx,
                                                              const float *__restrict__ x, const float *__restrict__ mean,
                                                              const float *__restrict__ sqrtvar, const float *__restrict__ gamma,
                                                              const uint8_t *__restrict__ zero, double *__restrict__ part,
                                                              int nsplit_part, float *__restrict__ dgamma, float *__restrict__ dbeta,
                                                              float *__restrict__ dx, float m, int C, int H, int W,
                                                              xsmi::FastDiv dQ4, xsmi::FastDiv dGQ, uint32_t total, uint32_t per) {
    __shared__ double sm[4];
    const int c = blockIdx.x, sp = blockIdx.y;
    const int OH = H >> 1, OW = W >> 1, Q4 = W >> 2;
    const float mu = mean[c], rs = sqrtvar[c];
    float db = 0.f, dg = 0.f, g = 0.f, den = 1.f;
    if (APPLY) {
        double t0, t1;
        bn_channel_sums(part, c, nsplit_part, sm, t0, t1);
        db = (float)t0; dg = (float)t1;
        if (sp == 0 && threadIdx.x == 0) {
            dbeta[c] = db;
            dgamma[c] = dg;
        }
        g = gamma[c];
        den = m * rs;
    }
    const uint32_t beg = (uint32_t)sp * per, end = min(total, beg + per);
    double s0 = 0.0, s1 = 0.0;
    // two units per thread and step, all loads of both before the first use (a unit past the end repeats the first
    // one's loads and contributes nothing): one unit at a time left the kernel waiting on memory latency
    for (uint32_t u0 = beg + threadIdx.x; u0 < end; u0 += 512) {
        constexpr int UNR = 2;
        size_t off[UNR];
        bool ok[UNR];
        float4 xe[UNR], xo[UNR];
        uchar4 ze[UNR], zo[UNR];
        PoolRouted r[UNR];
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            ok[k] = u0 + 256u * k < end;
            const uint32_t u = ok[k] ? u0 + 256u * k : u0;
            const uint32_t n = xsmi::fdiv(u, dGQ), rem = u - n * dGQ.d;
            const int a = (int)xsmi::fdiv(rem, dQ4), j = (int)rem - a * Q4;
            const size_t pl = (size_t)n * C + c;
            off[k] = (pl * H + 2 * a) * (size_t)W + 4 * j;
            xe[k] = *reinterpret_cast<const float4 *>(x + off[k]);
            xo[k] = *reinterpret_cast<const float4 *>(x + off[k] + W);
            ze[k] = make_uchar4(0, 0, 0, 0); zo[k] = ze[k];
            if (zero) {
                ze[k] = *reinterpret_cast<const uchar4 *>(zero + off[k]);
                zo[k] = *reinterpret_cast<const uchar4 *>(zero + off[k] + W);
            }
            r[k] = pool_routed_3x3s2p1(dp, idx, pl * OH * (size_t)OW, OH, OW, a, j);
        }
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            const float xv[2][4] = {{xe[k].x, xe[k].y, xe[k].z, xe[k].w}, {xo[k].x, xo[k].y, xo[k].z, xo[k].w}};
            const unsigned char zv[2][4] = {{ze[k].x, ze[k].y, ze[k].z, ze[k].w}, {zo[k].x, zo[k].y, zo[k].z, zo[k].w}};
            float ov[2][4];
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                double t0 = 0.0, t1 = 0.0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float d = zv[q][i] ? 0.f : (q ? r[k].o[i] : r[k].e[i]);
                    const float h = (xv[q][i] - mu) / rs;
                    if (APPLY) {
                        ov[q][i] = g * (m * d - db - h * dg) / den;
                    } else {
                        t0 += (double)d;
                        t1 += (double)d * (double)h;
                    }
                }
                if (ok[k]) {
                    s0 += t0;
                    s1 += t1;
                }
            }
            if (APPLY && ok[k]) {
                nt_store4(dx + off[k], ov[0][0], ov[0][1], ov[0][2], ov[0][3]);
                nt_store4(dx + off[k] + W, ov[1][0], ov[1][1], ov[1][2], ov[1][3]);
            }
        }
    }
    if (!APPLY) {
        s0 = block_sum(s0, sm);
        s1 = block_sum(s1, sm);
        if (threadIdx.x == 0) {
            part[((size_t)c * BN_SPLIT + sp) * 2 + 0] = s0;
            part[((size_t)c * BN_SPLIT + sp) * 2 + 1] = s1;
        }
    }
}

// Small layers (a channel's N*HW elements fit a workgroup's registers): both passes in one kernel, one workgroup
// per channel.  The elements are read once, summed in float64 (fixed order: per thread in element order, then
// block_sum), normalised from the registers and written; a launch and a read of the tensor less than the two-kernel
// form, which matters where a launch costs as much as the data movement (14x14 and 7x7 feature maps).
constexpr int BN_SMALL_PER = 8;                       // elements per thread, kept in registers
constexpr int BN_SMALL_MAX = 1024 * BN_SMALL_PER;     // 8192 elements per channel
// Element e = thread + NT u of channel c is (image j, position i) = (e / HW, e % HW); a thread forms the pair once
// and steps it by (NT / HW, NT % HW) with one wrap, so the loop has no division.  A workgroup has 256 threads for
// channels of up to 2048 elements (7 x 7 at N=32: 1568) and 1024 threads above (14 x 14 at N=32: 6272), eight
// elements per thread either way: the loads of a channel are all in flight at once and the chains behind them short.
struct BnSmallWalk {
    uint32_t j, i, dj, di, HW;
    __device__ __forceinline__ BnSmallWalk(uint32_t e, uint32_t nt, int HW_, const xsmi::FastDiv &dHW) : HW((uint32_t)HW_) {
        j = xsmi::fdiv(e, dHW); i = e - j * HW;
        dj = xsmi::fdiv(nt, dHW); di = nt - dj * HW;
    }
    __device__ __forceinline__ size_t off(int c, int C) const { return ((size_t)j * C + c) * (size_t)HW + i; }
    __device__ __forceinline__ void step() {
        j += dj; i += di;
        if (i >= HW) { i -= HW; ++j; }
    }
};
template <int NT>
__global__ void __launch_bounds__(NT) bn_fwd_small_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                                            const float *__restrict__ beta, double m, float eps, float momentum,
                                                            BnFwdOut o, int C, int HW, xsmi::FastDiv dHW, uint32_t total) {
    constexpr int PER = BN_SMALL_PER;
    __shared__ double sm[NT / 64];
    const int c = blockIdx.x;
    float v[PER];
    uint32_t offs[PER];
    BnSmallWalk wk(threadIdx.x, NT, HW, dHW);
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const uint32_t e = threadIdx.x + (uint32_t)NT * u;
        offs[u] = (uint32_t)wk.off(c, C);             // tensors stay below 2^29 elements
        v[u] = e < total ? x[offs[u]] : 0.f;
        wk.step();
    }
    double s0 = 0.0, s1 = 0.0;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        s0 += (double)v[u];
        s1 += (double)v[u] * (double)v[u];
    }
    s0 = block_sum_n<NT>(s0, sm);
    s1 = block_sum_n<NT>(s1, sm);
    const double mu_d = s0 / m;
    double var = s1 / m - mu_d * mu_d;
    if (var < 0.0) var = 0.0;
    const float mu = (float)mu_d, rs = (float)sqrt(var + (double)eps), g = gamma[c], bt = beta[c];
    if (threadIdx.x == 0) {
        o.mean[c] = mu;
        o.var[c] = (float)var;
        o.sqrtvar[c] = rs;
        if (o.moving_mean) {
            o.moving_mean[c] = momentum * o.moving_mean[c] + (1.f - momentum) * mu;
            o.moving_var[c] = momentum * o.moving_var[c] + (1.f - momentum) * (float)var;
        }
    }
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const uint32_t e = threadIdx.x + (uint32_t)NT * u;
        if (e >= total) break;
        const size_t off = offs[u];
        const float hv = (v[u] - mu) / rs;
        float pre = g * hv + bt;
        if (o.residual) pre += o.residual[off];
        if (o.xhat) o.xhat[off] = hv;
        o.y[off] = (o.neg_mask && pre < 0.f) ? 0.f : pre;
        if (o.neg_mask) o.neg_mask[off] = pre < 0.f ? 1 : 0;
    }
}
template <int NT>
__global__ void __launch_bounds__(NT) bn_bwd_small_kernel(const float *__restrict__ dy, const float *__restrict__ xhat,
                                                            const float *__restrict__ sqrtvar, const float *__restrict__ gamma,
                                                            float *__restrict__ dgamma, float *__restrict__ dbeta,
                                                            const uint8_t *__restrict__ zero, float *__restrict__ dx, float m,
                                                            const float *__restrict__ mean, int C, int HW, xsmi::FastDiv dHW,
                                                            uint32_t total) {
    constexpr int PER = BN_SMALL_PER;
    __shared__ double sm[NT / 64];
    const int c = blockIdx.x;
    const float rs = sqrtvar[c], mu = mean ? mean[c] : 0.f, g = gamma[c], den = m * rs;
    float d[PER], h[PER];
    uint8_t z[PER];
    uint32_t offs[PER];
    BnSmallWalk wk(threadIdx.x, NT, HW, dHW);
    // all loads first (the masked gradient is selected afterwards: a load that depends on the mask would wait for it)
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const uint32_t e = threadIdx.x + (uint32_t)NT * u;
        offs[u] = (uint32_t)wk.off(c, C);
        const bool ok = e < total;
        d[u] = ok ? dy[offs[u]] : 0.f;
        h[u] = ok ? xhat[offs[u]] : 0.f;
        z[u] = (ok && zero) ? zero[offs[u]] : (uint8_t)0;
        wk.step();
    }
    double s0 = 0.0, s1 = 0.0;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const uint32_t e = threadIdx.x + (uint32_t)NT * u;
        if (z[u]) d[u] = 0.f;
        if (mean) h[u] = e < total ? (h[u] - mu) / rs : 0.f;
        s0 += (double)d[u];
        s1 += (double)d[u] * (double)h[u];
    }
    s0 = block_sum_n<NT>(s0, sm);
    s1 = block_sum_n<NT>(s1, sm);
    const float db = (float)s0, dg = (float)s1;
    if (threadIdx.x == 0) {
        dbeta[c] = db;
        dgamma[c] = dg;
    }
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const uint32_t e = threadIdx.x + (uint32_t)NT * u;
        if (e >= total) break;
        dx[offs[u]] = g * (m * d[u] - db - h[u] * dg) / den;
    }
}

template <bool VEC>
__global__ void __launch_bounds__(256) bn_infer_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                                        const float *__restrict__ beta, const float *__restrict__ mean,
                                                        const float *__restrict__ var, float *__restrict__ y, ChanIdx chan,
                                                        uint32_t total, float eps, int relu) {
    constexpr int W = VEC ? 4 : 1;
    for (uint32_t i = (blockIdx.x * 256u + threadIdx.x) * W; i < total; i += gridDim.x * 256u * W) {
        const int c = chan(i);
        const float g = gamma[c], bt = beta[c], mu = mean[c], rs = sqrtf(var[c] + eps);
        float xv[W], yv[W];
        if (VEC) *reinterpret_cast<float4 *>(xv) = *reinterpret_cast<const float4 *>(x + i); else xv[0] = x[i];
#pragma unroll
        for (int e = 0; e < W; ++e) {
            const float v = g * ((xv[e] - mu) / rs) + bt;
            yv[e] = (relu && v < 0.f) ? 0.f : v;
        }
        if (VEC) *reinterpret_cast<float4 *>(y + i) = *reinterpret_cast<float4 *>(yv); else y[i] = yv[0];
    }
}

// Folds a moving-statistics batch norm that follows a convolution into the convolution: with
// scale[k] = gamma[k] / sqrt(var[k] + eps), w_out[k][j] = w[k][j] * scale[k] and
// b_out[k] = beta[k] + (bias[k] - mean[k]) * scale[k].
__global__ void __launch_bounds__(256) bn_fold_kernel(const float *__restrict__ w, const float *__restrict__ bias,
                                                       const float *__restrict__ gamma, const float *__restrict__ beta,
                                                       const float *__restrict__ mean, const float *__restrict__ var,
                                                       float *__restrict__ w_out, float *__restrict__ b_out, int K, int per_k,
                                                       float eps) {
    const size_t total = (size_t)K * per_k;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const int k = (int)(i / per_k);
        const float scale = gamma[k] / sqrtf(var[k] + eps);
        w_out[i] = w[i] * scale;
        if (i == (size_t)k * per_k) b_out[k] = beta[k] + ((bias ? bias[k] : 0.f) - mean[k]) * scale;
    }
}

// ---- average pool over k x k blocks --------------------------------------------
__global__ void __launch_bounds__(256) avgpool_fwd_kernel(const float *__restrict__ x, float *__restrict__ y, int H, int W,
                                                           int OH, int OW, int k, int sh, int sw, size_t total) {
    for (size_t o = (size_t)blockIdx.x * 256 + threadIdx.x; o < total; o += (size_t)gridDim.x * 256) {
        int ow = (int)(o % OW);
        size_t t = o / OW;
        int oh = (int)(t % OH);
        size_t nc = t / OH;
        const float *p = x + (nc * H + (size_t)oh * sh) * W + (size_t)ow * sw;
        double s = 0.0;
        for (int r = 0; r < k; ++r)
            for (int q = 0; q < k; ++q) s += (double)p[(size_t)r * W + q];
        y[o] = (float)(s / (double)(k * k));
    }
}
// the window is the whole plane (global pooling): one wavefront per plane, lanes along the plane's contiguous elements
__global__ void __launch_bounds__(256) avgpool_plane_kernel(const float *__restrict__ x, float *__restrict__ y, int HW,
                                                             uint32_t planes) {
    const uint32_t pl = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (pl >= planes) return;
    const int lane = threadIdx.x & 63;
    const float *p = x + (size_t)pl * HW;
    double s = 0.0;
    for (int i = lane; i < HW; i += 64) s += (double)p[i];
    s = wave_sum(s);
    if (lane == 0) y[pl] = (float)(s / (double)HW);
}
__global__ void __launch_bounds__(256) avgpool_bwd_kernel(const float *__restrict__ dy, float *__restrict__ dx, int H, int W,
                                                           int OH, int OW, int k, size_t total) {
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (size_t)gridDim.x * 256) {
        int w = (int)(e % W);
        size_t t = e / W;
        int h = (int)(t % H);
        size_t nc = t / H;
        int oh = h / k, ow = w / k;
        dx[e] = (oh < OH && ow < OW) ? dy[(nc * OH + oh) * OW + ow] / (float)(k * k) : 0.f;
    }
}
// Windows that overlap or leave gaps (stride != k): an input cell gathers dy / k^2 (rounded to float32 per window, as
// the reference forms it) from every window that covers it, in ascending (ky, kx) order of its position in the window,
// in float64, rounded once: the reference's float64 col2im (xs/nn/grad_fn.py:296-307).
__global__ void __launch_bounds__(256) avgpool_bwd_strided_kernel(const float *__restrict__ dy, float *__restrict__ dx, int H,
                                                                   int W, int OH, int OW, int k, int sh, int sw, size_t total) {
    const float kk = (float)(k * k);
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (size_t)gridDim.x * 256) {
        int w = (int)(e % W);
        size_t t = e / W;
        int h = (int)(t % H);
        size_t nc = t / H;
        double s = 0.0;
        for (int ky = 0; ky < k; ++ky) {
            const int top = h - ky;
            if (top < 0 || top % sh != 0 || top / sh >= OH) continue;
            for (int kx = 0; kx < k; ++kx) {
                const int left = w - kx;
                if (left < 0 || left % sw != 0 || left / sw >= OW) continue;
                s += (double)(dy[(nc * OH + top / sh) * OW + left / sw] / kk);
            }
        }
        dx[e] = (float)s;
    }
}

// ---- small GEMM (dense layer) ----------------------------------------------------
// 32x32 output tile per 256 threads, K in chunks of 128 through LDS: the dense layer's matrices are skinny (a
// batch of 32 rows), so few workgroups run and each must keep many loads in flight; a chunk is 32 independent
// loads per thread.  Lanes always run along the contiguous axis of the operand in memory, whichever way it is
// transposed.  Each of the four waves multiplies a quarter of the chunk (32 values of k: sixteen
// v_mfma_f32_32x32x2_f32) into its own 32x32 accumulator; the four are added in wave order at the end.
constexpr int GEMM_KC = 128;
typedef float gemm_f16v __attribute__((ext_vector_type(16)));
__global__ void __launch_bounds__(256) gemm_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                    const float *__restrict__ bias, float *__restrict__ C, int M, int N,
                                                    int K, int ta, int tb, int chunks_per_split) {
    __shared__ float As[32][GEMM_KC + 1], Bs[GEMM_KC][33];
    static_assert(sizeof(As) >= 4 * 1024 * sizeof(float), "the accumulators of four waves are exchanged through As");
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, l31 = lane & 31, half = lane >> 5;
    const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    gemm_f16v acc = {0};
    // split z multiplies K range [kbeg, kend) and writes its own M x N slab of C (C is then the partial buffer)
    const int kbeg = blockIdx.z * chunks_per_split * GEMM_KC;
    const int kend = min(K, kbeg + chunks_per_split * GEMM_KC);
    C += (size_t)blockIdx.z * M * N;
    for (int k0 = kbeg; k0 < kend; k0 += GEMM_KC) {
        // all loads of the chunk first (independent, so their latencies overlap), then the LDS stores
        float ra[GEMM_KC / 8], rb[GEMM_KC / 8];
#pragma unroll
        for (int u = 0; u < GEMM_KC / 8; ++u) {
            const int i = threadIdx.x + 256 * u;
            if (ta) {                                   // A stored (K, M): lanes along m
                const int kk = i >> 5, r = i & 31;
                ra[u] = (m0 + r < M && k0 + kk < kend) ? A[(size_t)(k0 + kk) * M + m0 + r] : 0.f;
            } else {                                    // A stored (M, K): lanes along k
                const int r = i / GEMM_KC, kk = i % GEMM_KC;
                ra[u] = (m0 + r < M && k0 + kk < kend) ? A[(size_t)(m0 + r) * K + k0 + kk] : 0.f;
            }
            if (tb) {                                   // B stored (N, K): lanes along k
                const int c = i / GEMM_KC, kk = i % GEMM_KC;
                rb[u] = (n0 + c < N && k0 + kk < kend) ? B[(size_t)(n0 + c) * K + k0 + kk] : 0.f;
            } else {                                    // B stored (K, N): lanes along n
                const int kk = i >> 5, c = i & 31;
                rb[u] = (n0 + c < N && k0 + kk < kend) ? B[(size_t)(k0 + kk) * N + n0 + c] : 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < GEMM_KC / 8; ++u) {
            const int i = threadIdx.x + 256 * u;
            if (ta) As[i & 31][i >> 5] = ra[u]; else As[i / GEMM_KC][i % GEMM_KC] = ra[u];
            if (tb) Bs[i % GEMM_KC][i / GEMM_KC] = rb[u]; else Bs[i >> 5][i & 31] = rb[u];
        }
        __syncthreads();
        // operand lane l of an MFMA holds row (column) l % 32 at k = l / 32
#pragma unroll
        for (int s = 0; s < GEMM_KC / 8; ++s) {
            const int kk = wv * (GEMM_KC / 4) + 2 * s + half;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(As[l31][kk], Bs[kk][l31], acc, 0, 0, 0);
        }
        __syncthreads();
    }
    // register v of lane l holds row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32 of the tile
    float *red = &As[0][0];
#pragma unroll
    for (int v = 0; v < 16; ++v) red[wv * 1024 + v * 64 + lane] = acc[v];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = (int)threadIdx.x + 256 * i, v = e >> 6, l = e & 63;
        const float sum = ((red[e] + red[1024 + e]) + red[2048 + e]) + red[3072 + e];
        const int m = m0 + 8 * (v >> 2) + 4 * (l >> 5) + (v & 3), n = n0 + (l & 31);
        if (m < M && n < N) C[(size_t)m * N + n] = sum + (bias ? bias[n] : 0.f);
    }
}
// C = bias + the K-split partial products, added in ascending split order
__global__ void __launch_bounds__(256) gemm_reduce_kernel(const float *__restrict__ part, const float *__restrict__ bias,
                                                           float *__restrict__ C, uint32_t MN, int N, int splits) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= MN) return;
    float s = part[i];
    for (int z = 1; z < splits; ++z) s += part[(size_t)z * MN + i];
    C[i] = s + (bias ? bias[i % (uint32_t)N] : 0.f);
}

__global__ void __launch_bounds__(256) colsum_kernel(const float *__restrict__ a, float *__restrict__ out, int M, int N) {
    int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= N) return;
    double s = 0.0;
    for (int i = 0; i < M; ++i) s += (double)a[(size_t)i * N + j];
    out[j] = (float)s;
}

__global__ void __launch_bounds__(256) sum_all_kernel(const float *__restrict__ a, float *__restrict__ out, size_t n) {
    __shared__ double sm[4];
    double s = 0.0;
    for (size_t i = threadIdx.x; i < n; i += 256) s += (double)a[i];
    s = block_sum(s, sm);
    if (threadIdx.x == 0) out[0] = (float)s;
}

// ---- softmax cross-entropy: one workgroup per row --------------------------------------
// exp() in float64, once per element: a thread keeps up to SOFTMAX_KEEP of its elements' exponentials in
// registers between the sum and the division (rows of up to 256 * SOFTMAX_KEEP classes); beyond that they
// are computed again.
constexpr int SOFTMAX_KEEP = 8;
__global__ void __launch_bounds__(256) softmax_rows_kernel(const float *__restrict__ z, const int64_t *__restrict__ lab,
                                                            float *__restrict__ sm, float *__restrict__ nll, int M, int N) {
    __shared__ double red[4];
    __shared__ float redf[4];
    const int row = blockIdx.x, t = threadIdx.x;
    const float *zr = z + (size_t)row * N;
    float mx = -3.402823466e38f;
    for (int j = t; j < N; j += 256) mx = fmaxf(mx, zr[j]);
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((t & 63) == 0) redf[t >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(redf[0], redf[1]), fmaxf(redf[2], redf[3]));
    double e[SOFTMAX_KEEP];
    double s = 0.0;
#pragma unroll
    for (int u = 0; u < SOFTMAX_KEEP; ++u) {
        const int j = t + 256 * u;
        e[u] = j < N ? exp((double)(zr[j] - mx)) : 0.0;
        s += e[u];
    }
    for (int j = t + 256 * SOFTMAX_KEEP; j < N; j += 256) s += exp((double)(zr[j] - mx));
    s = block_sum(s, red);
#pragma unroll
    for (int u = 0; u < SOFTMAX_KEEP; ++u) {
        const int j = t + 256 * u;
        if (j < N) sm[(size_t)row * N + j] = (float)(e[u] / s);
    }
    for (int j = t + 256 * SOFTMAX_KEEP; j < N; j += 256) sm[(size_t)row * N + j] = (float)(exp((double)(zr[j] - mx)) / s);
    if (t == 0) {
        int64_t l = lab[row];
        double p = (l >= 0 && l < N) ? exp((double)(zr[l] - mx)) / s : 1.0;
        nll[row] = (float)(-log(p));
    }
}
__global__ void __launch_bounds__(256) nll_reduce_kernel(const float *__restrict__ nll, float *__restrict__ loss, int M,
                                                          int mean) {
    __shared__ double sm[4];
    double s = 0.0;
    for (int i = threadIdx.x; i < M; i += 256) s += (double)nll[i];
    s = block_sum(s, sm);
    if (threadIdx.x == 0) loss[0] = (float)(mean ? s / (double)M : s);
}
__global__ void __launch_bounds__(256) softmax_ce_bwd_kernel(const float *__restrict__ sm, const int64_t *__restrict__ lab,
                                                              float *__restrict__ dz, int N, size_t total, float scale,
                                                              const float *__restrict__ upstream) {
    if (upstream) scale *= upstream[0];
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        size_t row = i / N;
        int j = (int)(i - row * N);
        float v = sm[i] - (lab[row] == (int64_t)j ? 1.f : 0.f);
        dz[i] = v * scale;
    }
}

}  // namespace

extern "C" {

int xsmi_axpy(float *y, const float *x, float a, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (y && x), "xsmi_axpy: null pointer");
    return launch_ew("axpy", n, aligned16(y) && aligned16(x), AxpyF{y, x, a});
}
int xsmi_axpy_multi(int count, float *const *ys, const float *const *xs, const size_t *ns, float a) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(count >= 0 && (count == 0 || (ys && xs && ns)), "xsmi_axpy_multi: bad argument");
    for (int done = 0; done < count;) {
        AxpyMulti m;
        m.a = a;
        m.count = 0;
        uint32_t blocks = 0;
        for (; done < count && m.count < AXPY_GROUP; ++done) {
            if (ns[done] == 0) continue;
            XSMI_CHECK_ARG(ys[done] && xs[done], "xsmi_axpy_multi: null pointer in tensor %d", done);
            XSMI_CHECK_ARG(ns[done] < 4294967296.0, "xsmi_axpy_multi: tensor %d too large", done);
            m.y[m.count] = ys[done]; m.x[m.count] = xs[done]; m.n[m.count] = (uint32_t)ns[done];
            m.first[m.count] = blocks;
            blocks += (uint32_t)((ns[done] + 1023) / 1024);
            ++m.count;
        }
        if (m.count == 0) break;
        m.first[m.count] = blocks;
        hipLaunchKernelGGL(axpy_multi_kernel, dim3(blocks), dim3(256), 0, xsmi::stream(), m);
        XSMI_LAUNCH_CHECK("axpy_multi_kernel");
    }
    return XSMI_OK;
}
int xsmi_add(const float *a, const float *b, float *out, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (a && b && out), "xsmi_add: null pointer");
    return launch_ew("add", n, aligned16(a) && aligned16(b) && aligned16(out), AddF{a, b, out});
}
int xsmi_add_relu(const float *a, const float *b, float *out, uint8_t *neg_mask, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (a && b && out), "xsmi_add_relu: null pointer");
    return launch_ew("add_relu", n, aligned16(a) && aligned16(b) && aligned16(out) && (((uintptr_t)neg_mask & 3) == 0),
                     AddReluF{a, b, out, neg_mask});
}
int xsmi_fill(float *out, float value, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || out, "xsmi_fill: null pointer");
    return launch_ew("fill", n, aligned16(out), FillF{out, value});
}
int xsmi_scale_shift(const float *a, float *out, float s, float t, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (a && out), "xsmi_scale_shift: null pointer");
    return launch_ew("scale_shift", n, aligned16(a) && aligned16(out), ScaleF{a, out, s, t});
}
int xsmi_relu_fwd(const float *x, float *y, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (x && y), "xsmi_relu_fwd: null pointer");
    return launch_ew("relu_fwd", n, aligned16(x) && aligned16(y), ReluF{x, y});
}
int xsmi_relu_fwd_mask(const float *x, float *y, uint8_t *neg_mask, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (x && y && neg_mask), "xsmi_relu_fwd_mask: null pointer");
    return launch_ew("relu_fwd_mask", n, aligned16(x) && aligned16(y) && (((uintptr_t)neg_mask & 3) == 0),
                     ReluMaskF{x, y, neg_mask});
}
int xsmi_relu_bwd(const float *dy, const float *pre, float *dx, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (dy && pre && dx), "xsmi_relu_bwd: null pointer");
    return launch_ew("relu_bwd", n, aligned16(dy) && aligned16(pre) && aligned16(dx), ReluBwdF{dy, pre, dx});
}
int xsmi_act_fwd(const float *x, float *y, size_t n, int kind) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (x && y), "xsmi_act_fwd: null pointer");
    XSMI_CHECK_ARG(kind == 1 || kind == 2, "xsmi_act_fwd: kind must be 1 (sigmoid) or 2 (tanh)");
    return launch_ew("act_fwd", n, aligned16(x) && aligned16(y), ActF{x, y, kind});
}
int xsmi_act_bwd(const float *dy, const float *y, float *dx, size_t n, int kind) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (dy && y && dx), "xsmi_act_bwd: null pointer");
    XSMI_CHECK_ARG(kind == 1 || kind == 2, "xsmi_act_bwd: kind must be 1 (sigmoid) or 2 (tanh)");
    return launch_ew("act_bwd", n, aligned16(dy) && aligned16(y) && aligned16(dx), ActBwdF{dy, y, dx, kind});
}
int xsmi_lerp(float *m, const float *cur, float momentum, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(n == 0 || (m && cur), "xsmi_lerp: null pointer");
    return launch_ew("lerp", n, 0, LerpF{m, cur, momentum});
}

size_t xsmi_bn_workspace_bytes(int C) { return C > 0 ? (size_t)C * BN_SPLIT * 2 * sizeof(double) : 0; }

static int bn_fwd_impl(const float *x, const float *gamma, const float *beta, float *y, float *xhat, float *sqrtvar,
                       float *mean, float *var, float *moving_mean, float *moving_var, float momentum, uint8_t *neg_mask,
                       const float *residual, int N, int C, int HW, float eps, void *ws, size_t ws_bytes);

int xsmi_bn_fwd(const float *x, const float *gamma, const float *beta, float *y, float *xhat, float *sqrtvar, float *mean,
                float *var, float *moving_mean, float *moving_var, float momentum, uint8_t *neg_mask, int N, int C, int HW,
                float eps, void *ws, size_t ws_bytes) {
    return bn_fwd_impl(x, gamma, beta, y, xhat, sqrtvar, mean, var, moving_mean, moving_var, momentum, neg_mask, nullptr, N,
                       C, HW, eps, ws, ws_bytes);
}

int xsmi_bn_relu_maxpool_fwd(const float *x, const float *gamma, const float *beta, float *pooled, uint8_t *idx,
                             uint8_t *neg_mask, float *sqrtvar, float *mean, float *var, float *moving_mean, float *moving_var,
                             float momentum, int N, int C, int H, int W, float eps, void *ws, size_t ws_bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && H > 0 && W > 0, "xsmi_bn_relu_maxpool_fwd: empty tensor");
    XSMI_CHECK_ARG(H % 2 == 0 && W % 4 == 0, "xsmi_bn_relu_maxpool_fwd: planes of an even number of rows, a multiple of four wide");
    XSMI_CHECK_ARG((double)N * C * H * W < 536870912.0, "xsmi_bn_relu_maxpool_fwd: tensors of 2^29 elements or more are not supported");
    XSMI_CHECK_ARG(x && gamma && beta && pooled && neg_mask && sqrtvar && mean && var, "xsmi_bn_relu_maxpool_fwd: null pointer");
    XSMI_CHECK_ARG(aligned16(x) && ((uintptr_t)neg_mask & 3) == 0 && ((uintptr_t)pooled & 7) == 0 && (!idx || ((uintptr_t)idx & 1) == 0),
                   "xsmi_bn_relu_maxpool_fwd: misaligned tensor");
    XSMI_CHECK_ARG((moving_mean == nullptr) == (moving_var == nullptr), "xsmi_bn_relu_maxpool_fwd: give both moving statistics or neither");
    XSMI_CHECK_ARG(ws && ws_bytes >= xsmi_bn_workspace_bytes(C), "xsmi_bn_relu_maxpool_fwd: workspace too small");
    hipStream_t st = xsmi::stream();
    const int HW = H * W;
    double *part = (double *)ws;
    const BnSplit split = bn_split(N, HW, true);
    launch_bn_partial(st, x, nullptr, nullptr, part, C, HW, split, nullptr, nullptr);
    XSMI_LAUNCH_CHECK("bn_partial_kernel");
    const int Q = W / 4, OH = H / 2;
    const uint32_t total = (uint32_t)N * OH * Q;
    uint32_t sp = total / 2048;
    if (sp < 1) sp = 1;
    if (sp > (uint32_t)BN_SPLIT) sp = BN_SPLIT;
    const uint32_t per = (total + sp - 1) / sp;
    const int nsp = (int)((total + per - 1) / per);
    const BnFwdOut o{pooled, nullptr, sqrtvar, mean, var, moving_mean, moving_var, neg_mask, nullptr};
    hipLaunchKernelGGL(bn_relu_maxpool_kernel, dim3(C, nsp), dim3(256), 0, st, x, gamma, beta, part, split.nsplit, (double)N * HW,
                       eps, momentum, o, idx, C, H, W, xsmi::make_fastdiv(Q), xsmi::make_fastdiv(OH * Q), total, per);
    XSMI_LAUNCH_CHECK("bn_relu_maxpool_kernel");
    return XSMI_OK;
}

int xsmi_bn_add_relu_fwd(const float *x, const float *gamma, const float *beta, const float *residual, float *y,
                         float *sqrtvar, float *mean, float *var, float *moving_mean, float *moving_var, float momentum,
                         uint8_t *neg_mask, int N, int C, int HW, float eps, void *ws, size_t ws_bytes) {
    XSMI_CHECK_ARG(residual && neg_mask, "xsmi_bn_add_relu_fwd: null pointer");
    return bn_fwd_impl(x, gamma, beta, y, nullptr, sqrtvar, mean, var, moving_mean, moving_var, momentum, neg_mask, residual,
                       N, C, HW, eps, ws, ws_bytes);
}

static int bn_fwd_impl(const float *x, const float *gamma, const float *beta, float *y, float *xhat, float *sqrtvar,
                       float *mean, float *var, float *moving_mean, float *moving_var, float momentum, uint8_t *neg_mask,
                       const float *residual, int N, int C, int HW, float eps, void *ws, size_t ws_bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && HW > 0, "xsmi_bn_fwd: empty tensor");
    XSMI_CHECK_ARG((double)N * C * HW < 536870912.0, "xsmi_bn_fwd: tensors of 2^29 elements or more are not supported");
    XSMI_CHECK_ARG(x && gamma && beta && y && sqrtvar && mean && var, "xsmi_bn_fwd: null pointer");
    XSMI_CHECK_ARG((moving_mean == nullptr) == (moving_var == nullptr), "xsmi_bn_fwd: give both moving statistics or neither");
    XSMI_CHECK_ARG(ws && ws_bytes >= xsmi_bn_workspace_bytes(C), "xsmi_bn_fwd: workspace too small");
    hipStream_t st = xsmi::stream();
    if ((size_t)N * HW <= (size_t)BN_SMALL_MAX) {
        const BnFwdOut o{y, xhat, sqrtvar, mean, var, moving_mean, moving_var, neg_mask, residual};
        const uint32_t total = (uint32_t)(N * HW);
        const xsmi::FastDiv dHW = xsmi::make_fastdiv(HW);
        if (total <= 256u * BN_SMALL_PER) hipLaunchKernelGGL(bn_fwd_small_kernel<256>, dim3(C), dim3(256), 0, st, x, gamma, beta, (double)N * HW, eps, momentum, o, C, HW, dHW, total);
        else hipLaunchKernelGGL(bn_fwd_small_kernel<1024>, dim3(C), dim3(1024), 0, st, x, gamma, beta, (double)N * HW, eps, momentum, o, C, HW, dHW, total);
        XSMI_LAUNCH_CHECK("bn_fwd_small_kernel");
        return XSMI_OK;
    }
    double *part = (double *)ws;
    const BnSplit split = bn_split(N, HW, (HW & 3) == 0 && aligned16(x));
    const int nsplit = split.nsplit;
    launch_bn_partial(st, x, nullptr, nullptr, part, C, HW, split, nullptr, nullptr);
    XSMI_LAUNCH_CHECK("bn_partial_kernel");
    const BnSplit ap = bn_split(N, HW, (HW & 3) == 0 && aligned16(x) && aligned16(y) && (!xhat || aligned16(xhat)) &&
                                           (!neg_mask || ((uintptr_t)neg_mask & 3) == 0) && (!residual || aligned16(residual)));
    const BnFwdOut o{y, xhat, sqrtvar, mean, var, moving_mean, moving_var, neg_mask, residual};
    if (ap.vec)
        hipLaunchKernelGGL(bn_apply_kernel<true>, dim3(C, ap.nsplit), dim3(256), 0, st, x, gamma, beta, part, nsplit,
                           (double)N * HW, eps, momentum, o, C, HW, ap.dU, ap.total, ap.per);
    else
        hipLaunchKernelGGL(bn_apply_kernel<false>, dim3(C, ap.nsplit), dim3(256), 0, st, x, gamma, beta, part, nsplit,
                           (double)N * HW, eps, momentum, o, C, HW, ap.dU, ap.total, ap.per);
    XSMI_LAUNCH_CHECK("bn_apply_kernel");
    return XSMI_OK;
}

int xsmi_bn_infer(const float *x, const float *gamma, const float *beta, const float *mean, const float *var, float *y,
                  int N, int C, int HW, float eps, int relu) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && HW > 0, "xsmi_bn_infer: empty tensor");
    XSMI_CHECK_ARG((double)N * C * HW < 536870912.0, "xsmi_bn_infer: tensors of 2^29 elements or more are not supported");
    XSMI_CHECK_ARG(x && gamma && beta && mean && var && y, "xsmi_bn_infer: null pointer");
    size_t total = (size_t)N * C * HW;
    if ((HW & 3) == 0 && aligned16(x) && aligned16(y))
        hipLaunchKernelGGL(bn_infer_kernel<true>, grid_for(total / 4), dim3(256), 0, xsmi::stream(), x, gamma, beta, mean,
                           var, y, make_chan(C, HW), (uint32_t)total, eps, relu);
    else
        hipLaunchKernelGGL(bn_infer_kernel<false>, grid_for(total), dim3(256), 0, xsmi::stream(), x, gamma, beta, mean,
                           var, y, make_chan(C, HW), (uint32_t)total, eps, relu);
    XSMI_LAUNCH_CHECK("bn_infer_kernel");
    return XSMI_OK;
}

int xsmi_bn_fold(const float *w, const float *bias, const float *gamma, const float *beta, const float *mean,
                 const float *var, float *w_out, float *b_out, int K, int per_k, float eps) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(K > 0 && per_k > 0, "xsmi_bn_fold: empty filter");
    XSMI_CHECK_ARG(w && gamma && beta && mean && var && w_out && b_out, "xsmi_bn_fold: null pointer");
    hipLaunchKernelGGL(bn_fold_kernel, grid_for((size_t)K * per_k), dim3(256), 0, xsmi::stream(), w, bias, gamma, beta, mean,
                       var, w_out, b_out, K, per_k, eps);
    XSMI_LAUNCH_CHECK("bn_fold_kernel");
    return XSMI_OK;
}

int xsmi_bn_bwd(const float *dy, const float *xhat, const float *mean, const float *sqrtvar, const float *gamma,
                const uint8_t *neg_mask, float *dx, float *dgamma, float *dbeta, int N, int C, int HW, void *ws,
                size_t ws_bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && HW > 0, "xsmi_bn_bwd: empty tensor");
    XSMI_CHECK_ARG((double)N * C * HW < 536870912.0, "xsmi_bn_bwd: tensors of 2^29 elements or more are not supported");
    XSMI_CHECK_ARG(dy && xhat && sqrtvar && gamma && dx && dgamma && dbeta, "xsmi_bn_bwd: null pointer");
    XSMI_CHECK_ARG(ws && ws_bytes >= xsmi_bn_workspace_bytes(C), "xsmi_bn_bwd: workspace too small");
    hipStream_t st = xsmi::stream();
    if ((size_t)N * HW <= (size_t)BN_SMALL_MAX) {
        const uint32_t total = (uint32_t)(N * HW);
        const xsmi::FastDiv dHW = xsmi::make_fastdiv(HW);
        const float mf = (float)((double)N * HW);
        if (total <= 256u * BN_SMALL_PER) hipLaunchKernelGGL(bn_bwd_small_kernel<256>, dim3(C), dim3(256), 0, st, dy, xhat, sqrtvar, gamma, dgamma, dbeta, neg_mask, dx, mf, mean, C, HW, dHW, total);
        else hipLaunchKernelGGL(bn_bwd_small_kernel<1024>, dim3(C), dim3(1024), 0, st, dy, xhat, sqrtvar, gamma, dgamma, dbeta, neg_mask, dx, mf, mean, C, HW, dHW, total);
        XSMI_LAUNCH_CHECK("bn_bwd_small_kernel");
        return XSMI_OK;
    }
    double *part = (double *)ws;
    const BnSplit split = bn_split(N, HW, (HW & 3) == 0 && aligned16(dy) && aligned16(xhat) &&
                                              (!neg_mask || ((uintptr_t)neg_mask & 3) == 0));
    const int nsplit = split.nsplit;
    launch_bn_partial(st, dy, xhat, neg_mask, part, C, HW, split, mean, sqrtvar);
    XSMI_LAUNCH_CHECK("bn_partial_kernel");
    const BnSplit ap = bn_split(N, HW, split.vec && aligned16(dx));
    const float m = (float)((double)N * HW);
    if (ap.vec)
        hipLaunchKernelGGL(bn_bwd_apply_kernel<true>, dim3(C, ap.nsplit), dim3(256), 0, st, dy, xhat, sqrtvar, gamma, part,
                           nsplit, dgamma, dbeta, neg_mask, dx, m, mean, C, HW, ap.dU, ap.total, ap.per);
    else
        hipLaunchKernelGGL(bn_bwd_apply_kernel<false>, dim3(C, ap.nsplit), dim3(256), 0, st, dy, xhat, sqrtvar, gamma, part,
                           nsplit, dgamma, dbeta, neg_mask, dx, m, mean, C, HW, ap.dU, ap.total, ap.per);
    XSMI_LAUNCH_CHECK("bn_bwd_apply_kernel");
    return XSMI_OK;
}

int xsmi_bn_bwd_maxpool(const float *dpooled, const uint8_t *idx, const float *x, const float *mean, const float *sqrtvar,
                        const float *gamma, const uint8_t *neg_mask, float *dx, float *dgamma, float *dbeta, int N, int C,
                        int H, int W, void *ws, size_t ws_bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && H > 0 && W > 0, "xsmi_bn_bwd_maxpool: empty tensor");
    XSMI_CHECK_ARG(H % 2 == 0 && W % 4 == 0, "xsmi_bn_bwd_maxpool: planes of an even number of rows, a multiple of four wide");
    XSMI_CHECK_ARG((double)N * C * H * W < 536870912.0, "xsmi_bn_bwd_maxpool: tensors of 2^29 elements or more are not supported");
    XSMI_CHECK_ARG(dpooled && idx && x && mean && sqrtvar && gamma && dx && dgamma && dbeta, "xsmi_bn_bwd_maxpool: null pointer");
    XSMI_CHECK_ARG(aligned16(x) && aligned16(dx) && ((uintptr_t)dpooled & 7) == 0 && ((uintptr_t)idx & 1) == 0 &&
                       (!neg_mask || ((uintptr_t)neg_mask & 3) == 0), "xsmi_bn_bwd_maxpool: misaligned tensor");
    XSMI_CHECK_ARG(ws && ws_bytes >= xsmi_bn_workspace_bytes(C), "xsmi_bn_bwd_maxpool: workspace too small");
    hipStream_t st = xsmi::stream();
    double *part = (double *)ws;
    const int Q4 = W / 4, G = H / 2;
    const uint32_t total = (uint32_t)N * G * Q4;         // units of eight elements per channel
    uint32_t sp = total / 1024;
    if (sp < 1) sp = 1;
    if (sp > (uint32_t)BN_SPLIT) sp = BN_SPLIT;
    const uint32_t per = (total + sp - 1) / sp;
    const int nsp = (int)((total + per - 1) / per);
    const float m = (float)((double)N * H * W);
    const xsmi::FastDiv dQ4 = xsmi::make_fastdiv(Q4), dGQ = xsmi::make_fastdiv(G * Q4);
    hipLaunchKernelGGL(bn_bwd_maxpool_kernel<false>, dim3(C, nsp), dim3(256), 0, st, dpooled, idx, x, mean, sqrtvar, gamma,
                       neg_mask, part, nsp, dgamma, dbeta, dx, m, C, H, W, dQ4, dGQ, total, per);
    XSMI_LAUNCH_CHECK("bn_bwd_maxpool_kernel");
    hipLaunchKernelGGL(bn_bwd_maxpool_kernel<true>, dim3(C, nsp), dim3(256), 0, st, dpooled, idx, x, mean, sqrtvar, gamma,
                       neg_mask, part, nsp, dgamma, dbeta, dx, m, C, H, W, dQ4, dGQ, total, per);
    XSMI_LAUNCH_CHECK("bn_bwd_maxpool_kernel");
    return XSMI_OK;
}

int xsmi_avgpool_fwd(const float *x, float *y, int N, int C, int H, int W, int k, int sh, int sw) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && H > 0 && W > 0 && k >= 1 && k <= H && k <= W && sh >= 1 && sw >= 1,
                   "xsmi_avgpool_fwd: bad geometry");
    XSMI_CHECK_ARG(x && y, "xsmi_avgpool_fwd: null pointer");
    int OH = (H - k) / sh + 1, OW = (W - k) / sw + 1;
    size_t total = (size_t)N * C * OH * OW;
    if (k == H && k == W && total < 0x7fffffffu)
        hipLaunchKernelGGL(avgpool_plane_kernel, dim3((unsigned)((total + 3) / 4)), dim3(256), 0, xsmi::stream(), x, y, H * W,
                           (uint32_t)total);
    else
        hipLaunchKernelGGL(avgpool_fwd_kernel, grid_for(total), dim3(256), 0, xsmi::stream(), x, y, H, W, OH, OW, k, sh, sw, total);
    XSMI_LAUNCH_CHECK("avgpool_fwd_kernel");
    return XSMI_OK;
}

int xsmi_avgpool_bwd(const float *dy, float *dx, int N, int C, int H, int W, int k, int sh, int sw) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(N > 0 && C > 0 && H > 0 && W > 0 && k >= 1 && k <= H && k <= W && sh >= 1 && sw >= 1,
                   "xsmi_avgpool_bwd: bad geometry");
    XSMI_CHECK_ARG(dy && dx, "xsmi_avgpool_bwd: null pointer");
    int OH = (H - k) / sh + 1, OW = (W - k) / sw + 1;
    size_t total = (size_t)N * C * H * W;
    if (sh == k && sw == k)
        hipLaunchKernelGGL(avgpool_bwd_kernel, grid_for(total), dim3(256), 0, xsmi::stream(), dy, dx, H, W, OH, OW, k, total);
    else
        hipLaunchKernelGGL(avgpool_bwd_strided_kernel, grid_for(total), dim3(256), 0, xsmi::stream(), dy, dx, H, W, OH, OW, k, sh,
                           sw, total);
    XSMI_LAUNCH_CHECK("avgpool_bwd_kernel");
    return XSMI_OK;
}

int xsmi_gemm(const float *A, const float *B, const float *bias, float *C, int M, int N, int K, int trans_a, int trans_b,
              void *ws, size_t ws_bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(M > 0 && N > 0 && K > 0, "xsmi_gemm: empty matrix");
    XSMI_CHECK_ARG(A && B && C, "xsmi_gemm: null pointer");
    XSMI_CHECK_ARG((double)M * N < 2147483648.0, "xsmi_gemm: outputs of 2^31 elements or more are not supported");
    // A skinny product (a batch of 32 rows) has few 32 x 32 output tiles and a long K: with a workspace, K is
    // split over enough workgroups to occupy the chip and the partial products are added in a second pass.  A
    // workgroup spends most of a chunk waiting for its loads, so "occupy" means about four workgroups per CU
    // (256 x 1000 x 512, the ResNet-18 classifier at N=256: one workgroup per CU 56 us, four 21 us).
    const int tiles = ((N + 31) / 32) * ((M + 31) / 32), chunks = (K + GEMM_KC - 1) / GEMM_KC;
    const int want = 4 * xsmi::cu_count();
    int splits = 1;
    if (ws && chunks > 1 && tiles < want) {
        splits = (want + tiles - 1) / tiles;
        if (splits > chunks) splits = chunks;
        const size_t fit = ws_bytes / ((size_t)M * N * sizeof(float));
        if ((size_t)splits > fit) splits = (int)fit;
        if (splits < 1) splits = 1;
    }
    const int cps = (chunks + splits - 1) / splits;
    splits = (chunks + cps - 1) / cps;
    hipStream_t st = xsmi::stream();
    if (splits == 1) {
        hipLaunchKernelGGL(gemm_kernel, dim3((N + 31) / 32, (M + 31) / 32, 1), dim3(256), 0, st, A, B, bias, C, M, N, K,
                           trans_a, trans_b, chunks);
        XSMI_LAUNCH_CHECK("gemm_kernel");
        return XSMI_OK;
    }
    hipLaunchKernelGGL(gemm_kernel, dim3((N + 31) / 32, (M + 31) / 32, splits), dim3(256), 0, st, A, B,
                       (const float *)nullptr, (float *)ws, M, N, K, trans_a, trans_b, cps);
    XSMI_LAUNCH_CHECK("gemm_kernel");
    const uint32_t MN = (uint32_t)((size_t)M * N);
    hipLaunchKernelGGL(gemm_reduce_kernel, dim3((MN + 255) / 256), dim3(256), 0, st, (const float *)ws, bias, C, MN, N, splits);
    XSMI_LAUNCH_CHECK("gemm_reduce_kernel");
    return XSMI_OK;
}

int xsmi_colsum(const float *a, float *out, int M, int N) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(M > 0 && N > 0 && a && out, "xsmi_colsum: bad argument");
    hipLaunchKernelGGL(colsum_kernel, dim3((N + 255) / 256), dim3(256), 0, xsmi::stream(), a, out, M, N);
    XSMI_LAUNCH_CHECK("colsum_kernel");
    return XSMI_OK;
}

int xsmi_sum_all(const float *a, float *out, size_t n) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(a && out, "xsmi_sum_all: null pointer");
    hipLaunchKernelGGL(sum_all_kernel, dim3(1), dim3(256), 0, xsmi::stream(), a, out, n);
    XSMI_LAUNCH_CHECK("sum_all_kernel");
    return XSMI_OK;
}

int xsmi_softmax_ce_fwd(const float *logits, const int64_t *labels, float *sm, float *loss, int M, int N, int mean) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(M > 0 && N > 0 && logits && labels && sm && loss, "xsmi_softmax_ce_fwd: bad argument");
    hipStream_t st = xsmi::stream();
    // `loss` has room for 1 + M floats: loss[0] is the result, loss[1..M] the per-row terms
    hipLaunchKernelGGL(softmax_rows_kernel, dim3(M), dim3(256), 0, st, logits, labels, sm, loss + 1, M, N);
    XSMI_LAUNCH_CHECK("softmax_rows_kernel");
    hipLaunchKernelGGL(nll_reduce_kernel, dim3(1), dim3(256), 0, st, loss + 1, loss, M, mean);
    XSMI_LAUNCH_CHECK("nll_reduce_kernel");
    return XSMI_OK;
}

int xsmi_softmax_ce_bwd(const float *sm, const int64_t *labels, const float *upstream, float *dlogits, int M, int N,
                        float scale) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(M > 0 && N > 0 && sm && labels && dlogits, "xsmi_softmax_ce_bwd: bad argument");
    size_t total = (size_t)M * N;
    hipLaunchKernelGGL(softmax_ce_bwd_kernel, grid_for(total), dim3(256), 0, xsmi::stream(), sm, labels, dlogits, N, total,
                       scale, upstream);
    XSMI_LAUNCH_CHECK("softmax_ce_bwd_kernel");
    return XSMI_OK;
}

}  // extern "C"
