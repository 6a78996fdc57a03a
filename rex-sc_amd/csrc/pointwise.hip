// OR-n pointwise activation, bias/noise error injection and calibration statistics.
// All kernels are HBM-streaming: 128-bit loads/stores, grid sized to the chip, no LDS
// except for the block reduction of the calibration statistics.
//
// Scalar math follows sc_cpu.hpp:192-404 (same fmaf order); host-side dtype conventions
// follow sc_cuda_pw.cu:708-1011 (forward in fp32, backward on the fp16-rounded saved sum).
#include <hip/hip_fp16.h>

#include "profile.h"
#include "rexsc_common.h"

namespace rexsc {

// ---- scalar math -------------------------------------------------------------------------------
// exp(-x) as one v_exp_f32 on x * -log2(e), the form the reference's CUDA kernels use (__expf, sc_device.cuh:396).
// The rounding of the scaled argument costs |x| * 2^-24 relative; for the sums this path sees (0 <= x, results that
// matter for x up to a few tens) that stays below 2e-6, inside the 1e-5 the float kernels are held to.
__device__ __forceinline__ float exp_neg(float x) { return __expf(-x); }

template <int N>
__device__ __forceinline__ float orn_fwd(float x)
{
    const float e = exp_neg(x);
    if constexpr (N == 1) return 1.f - e;
    if constexpr (N == 2) { float r = fmaf(-2.f, e, 2.f); return fmaf(-x, e, r); }
    if constexpr (N == 3) {
        const float x2 = x * x;
        float r = fmaf(-3.f, e, 3.f);
        r = fmaf(-2.f * x, e, r);
        return fmaf(-0.5f * x2, e, r);
    }
    const float x2 = x * x;
    float r = fmaf(-4.f, e, 4.f);
    r = fmaf(-3.f * x, e, r);
    const float x3 = x2 * x;
    r = fmaf(-x2, e, r);
    return fmaf((-1.f / 6.f) * x3, e, r);
}

// d/dx OR_n(x) * g
template <int N>
__device__ __forceinline__ float orn_bwd(float g, float x)
{
    const float e = exp_neg(x);
    if constexpr (N == 1) return e * g;
    float r = fmaf(x, e, e);
    if constexpr (N >= 3) r = fmaf(0.5f * (x * x), e, r);
    if constexpr (N >= 4) r = fmaf((1.f / 6.f) * ((x * x) * x), e, r);
    return r * g;
}

struct Coef6 { float c[6]; };

// The six coefficients are wave-uniform: the loads become scalar loads.
__device__ __forceinline__ Coef6 load_coef(const float *__restrict__ p)
{
    Coef6 c;
#pragma unroll
    for (int i = 0; i < 6; i++) c.c[i] = p[i];
    return c;
}

__device__ __forceinline__ float bias_noise_fwd(float x, float xi, const Coef6 &b, const Coef6 &s)
{   // sc_cpu.hpp:264-284
    const float x2 = x * x;
    float xb = fmaf(b.c[1], x, b.c[0]);
    const float x3 = x2 * x;
    xb = fmaf(b.c[2], x2, xb);
    const float x4 = x3 * x;
    xb = fmaf(b.c[3], x3, xb);
    const float x5 = x4 * x;
    xb = fmaf(b.c[4], x4, xb);
    xb = fmaf(b.c[5], x5, xb);
    float xs = fmaf(s.c[1], x, s.c[0]);
    xs = fmaf(s.c[2], x2, xs);
    xs = fmaf(s.c[3], x3, xs);
    xs = fmaf(s.c[4], x4, xs);
    xs = fmaf(s.c[5], x5, xs);
    return x + xb + xs * xi;
}

// f(xp, xi1) - f(xn, xi2) for f = bias_noise_fwd with two independent N(0,1) draws has the distribution of
// (xp + poly_b(xp)) - (xn + poly_b(xn)) + sqrt(poly_s(xp)^2 + poly_s(xn)^2) * xi with ONE draw: the two noise terms
// are independent zero-mean normals and only their difference leaves the kernel (sc_cuda_pw.cu:219-373 returns
// nothing else).  Same fmaf order for the polynomials as bias_noise_fwd; with poly_s = 0 the value is the same.
__device__ __forceinline__ float bias_noise_diff(float xp, float xn, float xi, const Coef6 &b, const Coef6 &s)
{
    float det[2], var = 0.f;
    const float xv[2] = {xp, xn};
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const float x = xv[k];
        const float x2 = x * x;
        float xb = fmaf(b.c[1], x, b.c[0]);
        const float x3 = x2 * x;
        xb = fmaf(b.c[2], x2, xb);
        const float x4 = x3 * x;
        xb = fmaf(b.c[3], x3, xb);
        const float x5 = x4 * x;
        xb = fmaf(b.c[4], x4, xb);
        xb = fmaf(b.c[5], x5, xb);
        float xs = fmaf(s.c[1], x, s.c[0]);
        xs = fmaf(s.c[2], x2, xs);
        xs = fmaf(s.c[3], x3, xs);
        xs = fmaf(s.c[4], x4, xs);
        xs = fmaf(s.c[5], x5, xs);
        det[k] = x + xb;
        var = fmaf(xs, xs, var);
    }
    return (det[0] - det[1]) + __builtin_amdgcn_sqrtf(var) * xi; // v_sqrt_f32: 1 ulp, the noise scale needs no more
}

__device__ __forceinline__ float bias_bwd(float x, const Coef6 &b)
{   // sc_cpu.hpp:286-297
    const float x2 = x * x;
    float xd = fmaf(2.f * b.c[2], x, 1.f + b.c[1]);
    const float x3 = x2 * x;
    xd = fmaf(3.f * b.c[3], x2, xd);
    const float x4 = x3 * x;
    xd = fmaf(4.f * b.c[4], x3, xd);
    xd = fmaf(5.f * b.c[5], x4, xd);
    return xd;
}

template <int N>
__device__ __forceinline__ float orn_bias_bwd(float g, float x, const Coef6 &b)
{   // sc_cpu.hpp:335-404
    const float y = orn_fwd<N>(x);
    const float xd = bias_bwd(y, b) * g;
    return orn_bwd<N>(xd, x);
}

__device__ __forceinline__ float round_half(float x) { return __half2float(__float2half(x)); }

// ---- Philox4x32-10 + Box-Muller ------------------------------------------------------------------
struct U4 { uint32_t v[4]; };

__host__ __device__ inline U4 philox4x32_10(U4 ctr, uint32_t k0, uint32_t k1)
{
    const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
    for (int r = 0; r < 10; r++) {
        const uint64_t p0 = (uint64_t)M0 * ctr.v[0];
        const uint64_t p1 = (uint64_t)M1 * ctr.v[2];
        U4 n;
        n.v[0] = (uint32_t)(p1 >> 32) ^ ctr.v[1] ^ k0;
        n.v[1] = (uint32_t)p1;
        n.v[2] = (uint32_t)(p0 >> 32) ^ ctr.v[3] ^ k1;
        n.v[3] = (uint32_t)p0;
        ctr = n;
        k0 += W0; k1 += W1;
    }
    return ctr;
}

// two uniforms -> two N(0,1) draws
__device__ __forceinline__ void box_muller(uint32_t a, uint32_t b, float &z0, float &z1)
{
    const float u1 = (float)((a >> 8) + 1u) * 5.9604644775390625e-8f; // (0, 1]
    const float u2 = (float)(b >> 8) * 5.9604644775390625e-8f;        // [0, 1)
    const float r = __builtin_amdgcn_sqrtf(-2.f * __logf(u1));
    z0 = r * __builtin_amdgcn_cosf(u2); // v_cos_f32 takes revolutions
    z1 = r * __builtin_amdgcn_sinf(u2);
}

// four N(0,1) draws for vector index q of stream `which`
__device__ __forceinline__ void normal4(uint64_t seed, uint64_t q, uint32_t which, float z[4])
{
    U4 ctr; ctr.v[0] = (uint32_t)q; ctr.v[1] = (uint32_t)(q >> 32); ctr.v[2] = which; ctr.v[3] = 0;
    const U4 r = philox4x32_10(ctr, (uint32_t)seed, (uint32_t)(seed >> 32));
    box_muller(r.v[0], r.v[1], z[0], z[1]);
    box_muller(r.v[2], r.v[3], z[2], z[3]);
}

// ---- kernels ----------------------------------------------------------------------------------------
constexpr int PW_THREADS = 256;

template <int N>
__global__ __launch_bounds__(PW_THREADS) void orn_forward_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                 size_t n)
{
    const size_t nvec = n / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        const float4 v = reinterpret_cast<const float4 *>(x)[q];
        float4 r;
        r.x = orn_fwd<N>(v.x); r.y = orn_fwd<N>(v.y); r.z = orn_fwd<N>(v.z); r.w = orn_fwd<N>(v.w);
        reinterpret_cast<float4 *>(y)[q] = r;
    }
    const size_t i = nvec * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = orn_fwd<N>(x[i]);
}

template <int N>
__global__ __launch_bounds__(PW_THREADS) void orn_backward_kernel(const float *__restrict__ g,
                                                                  const float *__restrict__ x,
                                                                  float *__restrict__ gx, size_t n, int half_input)
{
    const size_t nvec = n / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        float4 v = reinterpret_cast<const float4 *>(x)[q];
        const float4 gg = reinterpret_cast<const float4 *>(g)[q];
        if (half_input) { v.x = round_half(v.x); v.y = round_half(v.y); v.z = round_half(v.z); v.w = round_half(v.w); }
        float4 r;
        r.x = orn_bwd<N>(gg.x, v.x); r.y = orn_bwd<N>(gg.y, v.y); r.z = orn_bwd<N>(gg.z, v.z); r.w = orn_bwd<N>(gg.w, v.w);
        reinterpret_cast<float4 *>(gx)[q] = r;
    }
    const size_t i = nvec * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) gx[i] = orn_bwd<N>(g[i], half_input ? round_half(x[i]) : x[i]);
}

// ONE: a single N(0,1) draw per output (bias_noise_diff); otherwise one draw per polarity, which the caller can
// have written out (noise_p / noise_n)
template <int N, bool ONE>
__global__ __launch_bounds__(PW_THREADS) void orn_bias_std_both_forward_kernel(
    const float *__restrict__ xp, const float *__restrict__ xn, const float *__restrict__ bc, const float *__restrict__ sc,
    float *__restrict__ y, size_t n, uint64_t seed, uint64_t offset, const uint64_t *__restrict__ offset_dev,
    float *__restrict__ noise_p, float *__restrict__ noise_n)
{
    if (offset_dev) offset += *offset_dev; // wave-uniform: a scalar load
    const Coef6 b = load_coef(bc), s = load_coef(sc);
    const size_t nvec = (n + 3) / 4; // the tail vector is handled element-wise below
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        float zp[4], zn[4];
        normal4(seed, offset + q, 0u, zp);
        if (ONE) {
            if (q * 4 + 3 < n) {
                const float4 a = reinterpret_cast<const float4 *>(xp)[q];
                const float4 c = reinterpret_cast<const float4 *>(xn)[q];
                float4 r;
                r.x = bias_noise_diff(orn_fwd<N>(a.x), orn_fwd<N>(c.x), zp[0], b, s);
                r.y = bias_noise_diff(orn_fwd<N>(a.y), orn_fwd<N>(c.y), zp[1], b, s);
                r.z = bias_noise_diff(orn_fwd<N>(a.z), orn_fwd<N>(c.z), zp[2], b, s);
                r.w = bias_noise_diff(orn_fwd<N>(a.w), orn_fwd<N>(c.w), zp[3], b, s);
                reinterpret_cast<float4 *>(y)[q] = r;
            } else {
                for (int j = 0; j < 4; j++) {
                    const size_t i = q * 4 + j;
                    if (i >= n) break;
                    y[i] = bias_noise_diff(orn_fwd<N>(xp[i]), orn_fwd<N>(xn[i]), zp[j], b, s);
                }
            }
            continue;
        }
        normal4(seed, offset + q, 1u, zn);
        if (q * 4 + 3 < n) {
            const float4 a = reinterpret_cast<const float4 *>(xp)[q];
            const float4 c = reinterpret_cast<const float4 *>(xn)[q];
            float4 r;
            r.x = bias_noise_fwd(orn_fwd<N>(a.x), zp[0], b, s) - bias_noise_fwd(orn_fwd<N>(c.x), zn[0], b, s);
            r.y = bias_noise_fwd(orn_fwd<N>(a.y), zp[1], b, s) - bias_noise_fwd(orn_fwd<N>(c.y), zn[1], b, s);
            r.z = bias_noise_fwd(orn_fwd<N>(a.z), zp[2], b, s) - bias_noise_fwd(orn_fwd<N>(c.z), zn[2], b, s);
            r.w = bias_noise_fwd(orn_fwd<N>(a.w), zp[3], b, s) - bias_noise_fwd(orn_fwd<N>(c.w), zn[3], b, s);
            reinterpret_cast<float4 *>(y)[q] = r;
            if (noise_p) reinterpret_cast<float4 *>(noise_p)[q] = make_float4(zp[0], zp[1], zp[2], zp[3]);
            if (noise_n) reinterpret_cast<float4 *>(noise_n)[q] = make_float4(zn[0], zn[1], zn[2], zn[3]);
        } else {
            for (int j = 0; j < 4; j++) {
                const size_t i = q * 4 + j;
                if (i >= n) break;
                y[i] = bias_noise_fwd(orn_fwd<N>(xp[i]), zp[j], b, s) - bias_noise_fwd(orn_fwd<N>(xn[i]), zn[j], b, s);
                if (noise_p) noise_p[i] = zp[j];
                if (noise_n) noise_n[i] = zn[j];
            }
        }
    }
}

template <int N>
__global__ __launch_bounds__(PW_THREADS) void orn_bias_std_both_backward_kernel(
    const float *__restrict__ g, const float *__restrict__ xp, const float *__restrict__ xn,
    const float *__restrict__ bc, float *__restrict__ gp, float *__restrict__ gn, size_t n, int half_input)
{
    const Coef6 b = load_coef(bc);
    const size_t nvec = n / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        float4 a = reinterpret_cast<const float4 *>(xp)[q];
        float4 c = reinterpret_cast<const float4 *>(xn)[q];
        const float4 gg = reinterpret_cast<const float4 *>(g)[q];
        if (half_input) {
            a.x = round_half(a.x); a.y = round_half(a.y); a.z = round_half(a.z); a.w = round_half(a.w);
            c.x = round_half(c.x); c.y = round_half(c.y); c.z = round_half(c.z); c.w = round_half(c.w);
        }
        float4 rp, rn;
        rp.x = orn_bias_bwd<N>(gg.x, a.x, b); rn.x = orn_bias_bwd<N>(-gg.x, c.x, b);
        rp.y = orn_bias_bwd<N>(gg.y, a.y, b); rn.y = orn_bias_bwd<N>(-gg.y, c.y, b);
        rp.z = orn_bias_bwd<N>(gg.z, a.z, b); rn.z = orn_bias_bwd<N>(-gg.z, c.z, b);
        rp.w = orn_bias_bwd<N>(gg.w, a.w, b); rn.w = orn_bias_bwd<N>(-gg.w, c.w, b);
        reinterpret_cast<float4 *>(gp)[q] = rp;
        reinterpret_cast<float4 *>(gn)[q] = rn;
    }
    const size_t i = nvec * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float a = half_input ? round_half(xp[i]) : xp[i];
        const float c = half_input ? round_half(xn[i]) : xn[i];
        gp[i] = orn_bias_bwd<N>(g[i], a, b);
        gn[i] = orn_bias_bwd<N>(-g[i], c, b);
    }
}

// single polarity, binary16 in and out (sc_cuda_pw.cu:375-418)
template <int N>
__global__ __launch_bounds__(PW_THREADS) void orn_bias_std_forward_f16_kernel(const __half *__restrict__ x,
                                                                              const float *__restrict__ bc,
                                                                              const float *__restrict__ sc,
                                                                              __half *__restrict__ y, size_t n,
                                                                              uint64_t seed, uint64_t offset,
                                                                              const uint64_t *__restrict__ offset_dev)
{
    if (offset_dev) offset += *offset_dev;
    const Coef6 b = load_coef(bc), s = load_coef(sc);
    const size_t nvec = (n + 3) / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        float z[4];
        normal4(seed, offset + q, 0u, z);
        for (int j = 0; j < 4; j++) {
            const size_t i = q * 4 + j;
            if (i >= n) break;
            y[i] = __float2half(bias_noise_fwd(orn_fwd<N>(__half2float(x[i])), z[j], b, s));
        }
    }
}

template <int N>
__global__ __launch_bounds__(PW_THREADS) void orn_bias_std_backward_kernel(const float *__restrict__ g,
                                                                           const float *__restrict__ x,
                                                                           const float *__restrict__ bc,
                                                                           float *__restrict__ gx, size_t n,
                                                                           int half_input)
{
    const Coef6 b = load_coef(bc);
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        gx[i] = orn_bias_bwd<N>(g[i], half_input ? round_half(x[i]) : x[i], b);
}

// ---- polarity-pair layout ------------------------------------------------------------------------
// The float surrogate of an SC layer can convolve with the positive and the negative weight parts in
// one call (2*O output channels: the O positive ones, then the O negative ones).  Its sums then lie
// in memory as [outer][2][inner] float32 -- channels-last conv output: outer = N*Ho*Wo, inner = O;
// NCHW: outer = N, inner = O*Ho*Wo; linear: outer = B, inner = O -- while the layer's result and its
// incoming gradient are [outer][inner].  These kernels read and write the pair layout in place of
// two separate tensors; inner is a multiple of 4 (whole float4 vectors), q counts float4 vectors of
// the [outer][inner] tensor and the noise stream is indexed by q exactly as in the two-tensor kernels.
__device__ __forceinline__ size_t pair_vec_offset(size_t q, unsigned inner4)
{
    const unsigned o = (unsigned)q / inner4; // the host checks that q fits 32 bits
    return (size_t)q + (size_t)o * inner4;   // = o * 2 * inner4 + (q - o * inner4)
}

// Four neighbouring elements of a float32 or binary16 tensor (16- or 8-byte access), widened to float32.
template <typename T> struct Vec4Io;
template <> struct Vec4Io<float> {
    static __device__ __forceinline__ float4 load(const float *p, size_t v) { return reinterpret_cast<const float4 *>(p)[v]; }
    static __device__ __forceinline__ void store(float *p, size_t v, float4 x) { reinterpret_cast<float4 *>(p)[v] = x; }
};
template <> struct Vec4Io<__half> {
    static __device__ __forceinline__ float4 load(const __half *p, size_t v)
    {
        const uint2 raw = reinterpret_cast<const uint2 *>(p)[v];
        const __half2 lo = *reinterpret_cast<const __half2 *>(&raw.x), hi = *reinterpret_cast<const __half2 *>(&raw.y);
        return make_float4(__low2float(lo), __high2float(lo), __low2float(hi), __high2float(hi));
    }
    static __device__ __forceinline__ void store(__half *p, size_t v, float4 x)
    {   // round to nearest even, as a tensor cast to float16 does
        const __half2 lo = __floats2half2_rn(x.x, x.y), hi = __floats2half2_rn(x.z, x.w);
        uint2 raw;
        raw.x = *reinterpret_cast<const uint32_t *>(&lo);
        raw.y = *reinterpret_cast<const uint32_t *>(&hi);
        reinterpret_cast<uint2 *>(p)[v] = raw;
    }
};

// T = float: the tensors as the float32 surrogate leaves them.  T = __half: all three tensors in binary16, as inside
// a float16 autocast region (the arithmetic stays float32; results are rounded once, on the store).
template <int N, typename T>
__global__ __launch_bounds__(PW_THREADS) void orn_pair_backward_kernel(const T *__restrict__ g, const T *__restrict__ s2,
                                                                       T *__restrict__ g2, size_t nvec,
                                                                       unsigned inner4, int half_input)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        const size_t off = pair_vec_offset(q, inner4);
        float4 a = Vec4Io<T>::load(s2, off);
        float4 c = Vec4Io<T>::load(s2, off + inner4);
        const float4 gg = Vec4Io<T>::load(g, q);
        if (half_input && sizeof(T) == 4) {
            a.x = round_half(a.x); a.y = round_half(a.y); a.z = round_half(a.z); a.w = round_half(a.w);
            c.x = round_half(c.x); c.y = round_half(c.y); c.z = round_half(c.z); c.w = round_half(c.w);
        }
        float4 rp, rn;
        rp.x = orn_bwd<N>(gg.x, a.x); rn.x = orn_bwd<N>(-gg.x, c.x);
        rp.y = orn_bwd<N>(gg.y, a.y); rn.y = orn_bwd<N>(-gg.y, c.y);
        rp.z = orn_bwd<N>(gg.z, a.z); rn.z = orn_bwd<N>(-gg.z, c.z);
        rp.w = orn_bwd<N>(gg.w, a.w); rn.w = orn_bwd<N>(-gg.w, c.w);
        Vec4Io<T>::store(g2, off, rp);
        Vec4Io<T>::store(g2, off + inner4, rn);
    }
}

template <int N>
__global__ __launch_bounds__(PW_THREADS) void orn_bias_std_pair_forward_kernel(
    const float *__restrict__ s2, const float *__restrict__ bc, const float *__restrict__ sc, float *__restrict__ y,
    size_t nvec, unsigned inner4, uint64_t seed, uint64_t offset, const uint64_t *__restrict__ offset_dev)
{
    if (offset_dev) offset += *offset_dev;
    const Coef6 b = load_coef(bc), s = load_coef(sc);
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        float z[4]; // one draw per output, the same stream the two-tensor kernel uses
        normal4(seed, offset + q, 0u, z);
        const size_t off = pair_vec_offset(q, inner4);
        const float4 a = reinterpret_cast<const float4 *>(s2)[off];
        const float4 c = reinterpret_cast<const float4 *>(s2)[off + inner4];
        float4 r;
        r.x = bias_noise_diff(orn_fwd<N>(a.x), orn_fwd<N>(c.x), z[0], b, s);
        r.y = bias_noise_diff(orn_fwd<N>(a.y), orn_fwd<N>(c.y), z[1], b, s);
        r.z = bias_noise_diff(orn_fwd<N>(a.z), orn_fwd<N>(c.z), z[2], b, s);
        r.w = bias_noise_diff(orn_fwd<N>(a.w), orn_fwd<N>(c.w), z[3], b, s);
        reinterpret_cast<float4 *>(y)[q] = r;
    }
}

template <int N>
__global__ __launch_bounds__(PW_THREADS) void orn_bias_std_pair_backward_kernel(
    const float *__restrict__ g, const float *__restrict__ s2, const float *__restrict__ bc, float *__restrict__ g2,
    size_t nvec, unsigned inner4, int half_input)
{
    const Coef6 b = load_coef(bc);
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        const size_t off = pair_vec_offset(q, inner4);
        float4 a = reinterpret_cast<const float4 *>(s2)[off];
        float4 c = reinterpret_cast<const float4 *>(s2)[off + inner4];
        const float4 gg = reinterpret_cast<const float4 *>(g)[q];
        if (half_input) {
            a.x = round_half(a.x); a.y = round_half(a.y); a.z = round_half(a.z); a.w = round_half(a.w);
            c.x = round_half(c.x); c.y = round_half(c.y); c.z = round_half(c.z); c.w = round_half(c.w);
        }
        float4 rp, rn;
        rp.x = orn_bias_bwd<N>(gg.x, a.x, b); rn.x = orn_bias_bwd<N>(-gg.x, c.x, b);
        rp.y = orn_bias_bwd<N>(gg.y, a.y, b); rn.y = orn_bias_bwd<N>(-gg.y, c.y, b);
        rp.z = orn_bias_bwd<N>(gg.z, a.z, b); rn.z = orn_bias_bwd<N>(-gg.z, c.z, b);
        rp.w = orn_bias_bwd<N>(gg.w, a.w, b); rn.w = orn_bias_bwd<N>(-gg.w, c.w, b);
        reinterpret_cast<float4 *>(g2)[off] = rp;
        reinterpret_cast<float4 *>(g2)[off + inner4] = rn;
    }
}

// SC result as the layer's float output: y = pos / L - neg / L (utils_functional.py:1181-1182, 1273-1274, 1317).
// torch divides a tensor by a Python scalar as a multiplication by the scalar's float reciprocal; so does this.
__global__ __launch_bounds__(PW_THREADS) void sc_counts_to_float_kernel(const int16_t *__restrict__ pos,
                                                                        const int16_t *__restrict__ neg,
                                                                        float *__restrict__ y, size_t n, float inv_L)
{
    const size_t nvec = n / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        const uint2 p = reinterpret_cast<const uint2 *>(pos)[q];
        const uint2 m = reinterpret_cast<const uint2 *>(neg)[q];
        float4 r;
        r.x = (float)(int16_t)(p.x & 0xffffu) * inv_L - (float)(int16_t)(m.x & 0xffffu) * inv_L;
        r.y = (float)(int16_t)(p.x >> 16) * inv_L - (float)(int16_t)(m.x >> 16) * inv_L;
        r.z = (float)(int16_t)(p.y & 0xffffu) * inv_L - (float)(int16_t)(m.y & 0xffffu) * inv_L;
        r.w = (float)(int16_t)(p.y >> 16) * inv_L - (float)(int16_t)(m.y >> 16) * inv_L;
        reinterpret_cast<float4 *>(y)[q] = r;
    }
    const size_t i = nvec * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = (float)pos[i] * inv_L - (float)neg[i] * inv_L;
}

// w2 = [clamp(w, 0, 100) ; -clamp(w, -100, 0)]  (utils_functional.py:1204-1205).  w is [O][inner] with
// inner = C*KH*KW in either memory order (src_cl: [KH*KW][C], else [C][KH*KW]); w2 is written in the
// order dst_cl names, so that a channels-last convolution gets its filters without a conversion pass.
__device__ __forceinline__ size_t weight_index(size_t i, unsigned inner, unsigned C, unsigned taps, bool from_cl, bool to_cl)
{
    // index of element i (counted in `from` order) in `to` order
    if (from_cl == to_cl) return i;
    const size_t o = i / inner;
    const unsigned r = (unsigned)(i - o * inner);
    unsigned c, t;
    if (from_cl) { t = r / C; c = r - t * C; } else { c = r / taps; t = r - c * taps; }
    return o * inner + (to_cl ? t * C + c : c * taps + t);
}

__global__ __launch_bounds__(PW_THREADS) void split_weight_kernel(const float *__restrict__ w, float *__restrict__ w2,
                                                                  size_t n, unsigned C, unsigned taps, int src_cl,
                                                                  int dst_cl)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; // in w2's order
    if (i >= n) return;
    const float v = w[weight_index(i, C * taps, C, taps, dst_cl != 0, src_cl != 0)];
    w2[i] = v != v ? v : fminf(fmaxf(v, 0.f), 100.f); // clamp keeps NaN, as torch's does
    w2[n + i] = v != v ? v : -fminf(fmaxf(v, -100.f), 0.f);
}

// Gradient of the two clamps: each passes its incoming gradient where w lies inside its closed range.
// dw is written in w's order (w_cl), dw2 is read in its own (dw2_cl).
__global__ __launch_bounds__(PW_THREADS) void merge_weight_grad_kernel(const float *__restrict__ dw2,
                                                                       const float *__restrict__ w,
                                                                       float *__restrict__ dw, size_t n, unsigned C,
                                                                       unsigned taps, int dw2_cl, int w_cl)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; // in w's order
    if (i >= n) return;
    const size_t j = weight_index(i, C * taps, C, taps, w_cl != 0, dw2_cl != 0);
    const float v = w[i];
    const float gp = (v >= 0.f && v <= 100.f) ? dw2[j] : 0.f;
    const float gn = (v >= -100.f && v <= 0.f) ? dw2[n + j] : 0.f;
    dw[i] = gp - gn;
}

// Fake quantisation of activations and weights (utils_functional.py:93-104, prune = 0):
// y = clamp(round_half_even(x * 2^prec), -(2^prec - 1), 2^prec - 1) / 2^prec; the scalings are exact.
__device__ __forceinline__ float quantize_one(float x, float scale, float inv_scale, float lim)
{
    const float r = rintf(x * scale);
    const float c = r != r ? r : fminf(fmaxf(r, 1.0f - scale), lim); // 1 - scale: +0 at prec 0, as torch's clamp bound
    return c * inv_scale;
}

__global__ __launch_bounds__(PW_THREADS) void quantize_kernel(const float *__restrict__ x, float *__restrict__ y, size_t n,
                                                             float scale, float inv_scale, float lim)
{
    const size_t nvec = n / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        const float4 v = reinterpret_cast<const float4 *>(x)[q];
        float4 r;
        r.x = quantize_one(v.x, scale, inv_scale, lim); r.y = quantize_one(v.y, scale, inv_scale, lim);
        r.z = quantize_one(v.z, scale, inv_scale, lim); r.w = quantize_one(v.w, scale, inv_scale, lim);
        reinterpret_cast<float4 *>(y)[q] = r;
    }
    const size_t i = nvec * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = quantize_one(x[i], scale, inv_scale, lim);
}

// The same on binary16 tensors: widened, quantised in float32, rounded back (exact: the results are multiples of
// 2^-prec below one).  Equal to the four float16 tensor passes for prec <= 10, where every intermediate is
// representable in binary16 or saturates the same way.
__global__ __launch_bounds__(PW_THREADS) void quantize_f16_kernel(const __half *__restrict__ x, __half *__restrict__ y, size_t n,
                                                                 float scale, float inv_scale, float lim)
{
    const size_t nvec = n / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < nvec; q += stride) {
        const float4 v = Vec4Io<__half>::load(x, q);
        float4 r;
        r.x = quantize_one(v.x, scale, inv_scale, lim); r.y = quantize_one(v.y, scale, inv_scale, lim);
        r.z = quantize_one(v.z, scale, inv_scale, lim); r.w = quantize_one(v.w, scale, inv_scale, lim);
        Vec4Io<__half>::store(y, q, r);
    }
    const size_t i = nvec * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = __float2half(quantize_one(__half2float(x[i]), scale, inv_scale, lim));
}

// Calibration statistics: per window k, count / sum / sum of squares of (a_bit - a_act) over
// the elements with lo[k] <= a_act < hi[k].  Windows may overlap.
constexpr int CAL_MAX_WIN = 64;
struct CalWindows { float lo[CAL_MAX_WIN]; float hi[CAL_MAX_WIN]; };

constexpr int CAL_E = 16; // elements a thread holds in registers while it walks the windows

__global__ __launch_bounds__(256) void calib_stats_kernel(const float *__restrict__ a_bit,
                                                          const float *__restrict__ a_act, size_t n, CalWindows w,
                                                          int n_win, double *__restrict__ stats)
{
    __shared__ double s_acc[CAL_MAX_WIN * 3];
    for (int i = threadIdx.x; i < n_win * 3; i += blockDim.x) s_acc[i] = 0.0;
    __syncthreads();
    // A thread loads CAL_E elements (coalesced across the block), then walks the windows with the
    // elements in registers: per window a few VALU operations per element, one wave reduction and
    // three LDS atomics per wave.  Sum and sum of squares are carried in double from the first term on
    // (the square of a float is exact in double), so that the variance the host forms from them as
    // s2/n - (s1/n)^2 loses nothing to the partial sums even where the bias is much larger than the spread.
    const size_t tile = (size_t)blockDim.x * CAL_E;
    for (size_t t0 = (size_t)blockIdx.x * tile; t0 < n; t0 += (size_t)gridDim.x * tile) {
        float act[CAL_E];
        double err[CAL_E];
#pragma unroll
        for (int j = 0; j < CAL_E; j++) {
            const size_t i = t0 + (size_t)j * blockDim.x + threadIdx.x;
            const bool ok = i < n;
            act[j] = ok ? a_act[i] : __builtin_nanf(""); // NaN belongs to no window
            err[j] = ok ? (double)(a_bit[i] - act[j]) : 0.0;
        }
        for (int k = 0; k < n_win; k++) {
            const float lo = w.lo[k], hi = w.hi[k];
            float c = 0.f;
            double e = 0.0, e2 = 0.0;
#pragma unroll
            for (int j = 0; j < CAL_E; j++) {
                const bool in = act[j] >= lo && act[j] < hi;
                const double x = in ? err[j] : 0.0;
                c += in ? 1.f : 0.f;
                e += x;
                e2 = fma(x, x, e2);
            }
            if (__ballot(c > 0.f) == 0) continue; // wave-uniform
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                c += __shfl_down(c, off);
                e += __shfl_down(e, off);
                e2 += __shfl_down(e2, off);
            }
            if ((threadIdx.x & 63) == 0) {
                atomicAdd(&s_acc[k * 3 + 0], (double)c);
                atomicAdd(&s_acc[k * 3 + 1], e);
                atomicAdd(&s_acc[k * 3 + 2], e2);
            }
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n_win * 3; i += blockDim.x)
        if (s_acc[i] != 0.0) atomicAdd(&stats[i], s_acc[i]);
}

__global__ void zero_f64_kernel(double *p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0;
}

// ---- host launch helpers ---------------------------------------------------------------------------
static int pw_grid(size_t work_items)
{
    size_t blocks = (work_items + PW_THREADS - 1) / PW_THREADS;
    const size_t cap = 256 * 8; // 8 blocks of 256 threads per CU
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (int)blocks;
}

#define REXSC_OR_N_SWITCH(or_n, CALL)                                      \
    switch (or_n) {                                                        \
    case 1: { constexpr int N = 1; CALL; } break;                          \
    case 2: { constexpr int N = 2; CALL; } break;                          \
    case 3: { constexpr int N = 3; CALL; } break;                          \
    case 4: { constexpr int N = 4; CALL; } break;                          \
    default: set_error("or_n must be 1..4 (got %d)", or_n); return REXSC_ERR_INVALID; \
    }

} // namespace rexsc

using namespace rexsc;

extern "C" int rexsc_orn_forward(const float *x, float *y, size_t n, int or_n, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(n == 0 || (x && y), "null pointer");
    if (n == 0) { REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n); return REXSC_OK; }
    const int grid = pw_grid((n + 3) / 4);
    ProfScope prof("orn_forward", 8.0 * n, stream);
    REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL(orn_forward_kernel<N>, dim3(grid), dim3(PW_THREADS), 0, stream, x, y, n));
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_orn_backward(const float *g, const float *x, float *gx, size_t n, int or_n, int half_input,
                                  rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(n == 0 || (g && x && gx), "null pointer");
    if (n == 0) { REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n); return REXSC_OK; }
    const int grid = pw_grid((n + 3) / 4);
    ProfScope prof("orn_backward", 12.0 * n, stream);
    REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL(orn_backward_kernel<N>, dim3(grid), dim3(PW_THREADS), 0, stream, g, x,
                                               gx, n, half_input));
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_orn_bias_std_both_forward(const float *xp, const float *xn, const float *bias_coef,
                                               const float *std_coef, float *y, size_t n, int or_n, uint64_t seed,
                                               uint64_t offset, const uint64_t *offset_dev, float *noise_p,
                                               float *noise_n, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n);
    REXSC_CHECK_ARG(bias_coef && std_coef && (n == 0 || (xp && xn && y)), "null pointer");
    if (n == 0) return REXSC_OK;
    const int grid = pw_grid((n + 3) / 4);
    ProfScope prof("orn_bias_std_both_forward", (12.0 + (noise_p ? 4.0 : 0.0) + (noise_n ? 4.0 : 0.0)) * n, stream);
    if (noise_p || noise_n) {
        REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL((orn_bias_std_both_forward_kernel<N, false>), dim3(grid), dim3(PW_THREADS), 0,
                                                   stream, xp, xn, bias_coef, std_coef, y, n, seed, offset, offset_dev,
                                                   noise_p, noise_n));
    } else {
        REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL((orn_bias_std_both_forward_kernel<N, true>), dim3(grid), dim3(PW_THREADS), 0,
                                                   stream, xp, xn, bias_coef, std_coef, y, n, seed, offset, offset_dev,
                                                   noise_p, noise_n));
    }
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_orn_bias_std_both_backward(const float *g, const float *xp, const float *xn,
                                                const float *bias_coef, float *gp, float *gn, size_t n, int or_n,
                                                int half_input, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n);
    REXSC_CHECK_ARG(bias_coef && (n == 0 || (g && xp && xn && gp && gn)), "null pointer");
    if (n == 0) return REXSC_OK;
    const int grid = pw_grid((n + 3) / 4);
    ProfScope prof("orn_bias_std_both_backward", 20.0 * n, stream);
    REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL(orn_bias_std_both_backward_kernel<N>, dim3(grid), dim3(PW_THREADS), 0,
                                               stream, g, xp, xn, bias_coef, gp, gn, n, half_input));
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_orn_bias_std_forward_f16(const uint16_t *x_half, const float *bias_coef, const float *std_coef,
                                              uint16_t *y_half, size_t n, int or_n, uint64_t seed, uint64_t offset,
                                              const uint64_t *offset_dev, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n);
    REXSC_CHECK_ARG(bias_coef && std_coef && (n == 0 || (x_half && y_half)), "null pointer");
    if (n == 0) return REXSC_OK;
    const int grid = pw_grid((n + 3) / 4);
    REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL(orn_bias_std_forward_f16_kernel<N>, dim3(grid), dim3(PW_THREADS), 0,
                                               stream, reinterpret_cast<const __half *>(x_half), bias_coef, std_coef,
                                               reinterpret_cast<__half *>(y_half), n, seed, offset, offset_dev));
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_orn_bias_std_backward(const float *g, const float *x, const float *bias_coef, float *gx,
                                           size_t n, int or_n, int half_input, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n);
    REXSC_CHECK_ARG(bias_coef && (n == 0 || (g && x && gx)), "null pointer");
    if (n == 0) return REXSC_OK;
    const int grid = pw_grid(n);
    REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL(orn_bias_std_backward_kernel<N>, dim3(grid), dim3(PW_THREADS), 0,
                                               stream, g, x, bias_coef, gx, n, half_input));
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" void rexsc_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4])
{
    U4 c;
    for (int i = 0; i < 4; i++) c.v[i] = counter[i];
    const U4 r = philox4x32_10(c, key[0], key[1]);
    for (int i = 0; i < 4; i++) out[i] = r.v[i];
}

extern "C" int rexsc_calib_stats(const float *a_bit, const float *a_act, size_t n, const float *starts_host,
                                 const float *ends_host, int n_win, double *stats, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(n_win >= 1 && n_win <= CAL_MAX_WIN, "n_win must be 1..%d (got %d)", CAL_MAX_WIN, n_win);
    REXSC_CHECK_ARG(starts_host && ends_host && stats && (n == 0 || (a_bit && a_act)), "null pointer");
    CalWindows w;
    for (int k = 0; k < n_win; k++) { w.lo[k] = starts_host[k]; w.hi[k] = ends_host[k]; }
    hipLaunchKernelGGL(zero_f64_kernel, dim3(1), dim3(256), 0, stream, stats, n_win * 3);
    REXSC_CHECK_HIP(hipGetLastError());
    if (n == 0) return REXSC_OK;
    size_t tiles = (n + 256 * CAL_E - 1) / (256 * CAL_E);
    const int grid = (int)(tiles < 4096 ? tiles : 4096);
    ProfScope prof("calib_stats", 8.0 * n, stream);
    hipLaunchKernelGGL(calib_stats_kernel, dim3(grid), dim3(256), 0, stream, a_bit, a_act, n, w, n_win, stats);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

// ---- polarity-pair entry points ----------------------------------------------------------------------
static int check_pair(size_t outer, size_t inner)
{
    REXSC_CHECK_ARG(inner % 4 == 0, "pair layout needs inner %% 4 == 0 (got %zu)", inner);
    REXSC_CHECK_ARG(outer * inner / 4 < (1ull << 32), "pair layout: tensor too large (%zu x %zu)", outer, inner);
    return REXSC_OK;
}

extern "C" int rexsc_orn_pair_backward(const float *g, const float *s2, float *g2, size_t outer, size_t inner, int or_n,
                                       int half_input, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n);
    if (int rc = check_pair(outer, inner)) return rc;
    const size_t nvec = outer * inner / 4;
    if (nvec == 0) return REXSC_OK;
    REXSC_CHECK_ARG(g && s2 && g2, "null pointer");
    const int grid = pw_grid(nvec);
    ProfScope prof("orn_pair_backward", 20.0 * outer * inner, stream);
    REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL((orn_pair_backward_kernel<N, float>), dim3(grid), dim3(PW_THREADS), 0, stream,
                                               g, s2, g2, nvec, (unsigned)(inner / 4), half_input));
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

// The same on binary16 tensors (grad_out, s2 and g2 all float16; 8-byte aligned): what the merged surrogate holds
// inside a float16 autocast region.  Equal to widening the inputs, calling rexsc_orn_pair_backward and rounding g2.
extern "C" int rexsc_orn_pair_backward_f16(const uint16_t *g, const uint16_t *s2, uint16_t *g2, size_t outer, size_t inner,
                                           int or_n, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n);
    if (int rc = check_pair(outer, inner)) return rc;
    const size_t nvec = outer * inner / 4;
    if (nvec == 0) return REXSC_OK;
    REXSC_CHECK_ARG(g && s2 && g2, "null pointer");
    REXSC_CHECK_ARG(((uintptr_t)g | (uintptr_t)s2 | (uintptr_t)g2) % 8 == 0, "float16 tensors must be 8-byte aligned");
    const int grid = pw_grid(nvec);
    ProfScope prof("orn_pair_backward", 10.0 * outer * inner, stream);
    REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL((orn_pair_backward_kernel<N, __half>), dim3(grid), dim3(PW_THREADS), 0, stream,
                                               (const __half *)g, (const __half *)s2, (__half *)g2, nvec,
                                               (unsigned)(inner / 4), 1));
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_orn_bias_std_pair_forward(const float *s2, const float *bias_coef, const float *std_coef, float *y,
                                               size_t outer, size_t inner, int or_n, uint64_t seed, uint64_t offset,
                                               const uint64_t *offset_dev, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n);
    if (int rc = check_pair(outer, inner)) return rc;
    const size_t nvec = outer * inner / 4;
    if (nvec == 0) return REXSC_OK;
    REXSC_CHECK_ARG(s2 && y && bias_coef && std_coef, "null pointer");
    const int grid = pw_grid(nvec);
    ProfScope prof("orn_bias_std_pair_forward", 12.0 * outer * inner, stream);
    REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL(orn_bias_std_pair_forward_kernel<N>, dim3(grid), dim3(PW_THREADS), 0,
                                               stream, s2, bias_coef, std_coef, y, nvec, (unsigned)(inner / 4), seed,
                                               offset, offset_dev));
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_orn_bias_std_pair_backward(const float *g, const float *s2, const float *bias_coef, float *g2,
                                                size_t outer, size_t inner, int or_n, int half_input,
                                                rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(or_n >= 1 && or_n <= 4, "or_n must be 1..4 (got %d)", or_n);
    if (int rc = check_pair(outer, inner)) return rc;
    const size_t nvec = outer * inner / 4;
    if (nvec == 0) return REXSC_OK;
    REXSC_CHECK_ARG(g && s2 && g2 && bias_coef, "null pointer");
    const int grid = pw_grid(nvec);
    ProfScope prof("orn_bias_std_pair_backward", 20.0 * outer * inner, stream);
    REXSC_OR_N_SWITCH(or_n, hipLaunchKernelGGL(orn_bias_std_pair_backward_kernel<N>, dim3(grid), dim3(PW_THREADS), 0,
                                               stream, g, s2, bias_coef, g2, nvec, (unsigned)(inner / 4), half_input));
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_sc_counts_to_float(const int16_t *pos, const int16_t *neg, float *y, size_t n, int bit_length,
                                        rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(bit_length >= 1, "bit_length must be positive (got %d)", bit_length);
    if (n == 0) return REXSC_OK;
    REXSC_CHECK_ARG(pos && neg && y, "null pointer");
    const int grid = pw_grid((n + 3) / 4);
    ProfScope prof("sc_counts_to_float", 8.0 * n, stream);
    hipLaunchKernelGGL(sc_counts_to_float_kernel, dim3(grid), dim3(PW_THREADS), 0, stream, pos, neg, y, n,
                       1.0f / (float)bit_length);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_split_weight(const float *w, float *w2, size_t out_channels, size_t in_channels, size_t taps,
                                  int w_channels_last, int w2_channels_last, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    const size_t n = out_channels * in_channels * taps;
    if (n == 0) return REXSC_OK;
    REXSC_CHECK_ARG(w && w2, "null pointer");
    REXSC_CHECK_ARG(in_channels * taps < (1ull << 32) && n < (1ull << 31) * PW_THREADS, "tensor too large");
    ProfScope prof("split_weight", 12.0 * n, stream);
    hipLaunchKernelGGL(split_weight_kernel, dim3((unsigned)((n + PW_THREADS - 1) / PW_THREADS)), dim3(PW_THREADS), 0,
                       stream, w, w2, n, (unsigned)in_channels, (unsigned)taps, w_channels_last, w2_channels_last);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_merge_weight_grad(const float *dw2, const float *w, float *dw, size_t out_channels,
                                       size_t in_channels, size_t taps, int dw2_channels_last, int w_channels_last,
                                       rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    const size_t n = out_channels * in_channels * taps;
    if (n == 0) return REXSC_OK;
    REXSC_CHECK_ARG(dw2 && w && dw, "null pointer");
    REXSC_CHECK_ARG(in_channels * taps < (1ull << 32) && n < (1ull << 31) * PW_THREADS, "tensor too large");
    ProfScope prof("merge_weight_grad", 16.0 * n, stream);
    hipLaunchKernelGGL(merge_weight_grad_kernel, dim3((unsigned)((n + PW_THREADS - 1) / PW_THREADS)), dim3(PW_THREADS),
                       0, stream, dw2, w, dw, n, (unsigned)in_channels, (unsigned)taps, dw2_channels_last,
                       w_channels_last);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_quantize_f16(const uint16_t *x, uint16_t *y, size_t n, int prec, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(prec >= 0 && prec <= 10, "prec must be 0..10 for float16 tensors (got %d)", prec);
    if (n == 0) return REXSC_OK;
    REXSC_CHECK_ARG(x && y, "null pointer");
    REXSC_CHECK_ARG(((uintptr_t)x | (uintptr_t)y) % 8 == 0, "float16 tensors must be 8-byte aligned");
    const float scale = (float)(1u << prec);
    const int grid = pw_grid((n + 3) / 4);
    ProfScope prof("quantize", 4.0 * n, stream);
    hipLaunchKernelGGL(quantize_f16_kernel, dim3(grid), dim3(PW_THREADS), 0, stream, (const __half *)x, (__half *)y, n, scale,
                       1.0f / scale, scale - 1.0f);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

extern "C" int rexsc_quantize(const float *x, float *y, size_t n, int prec, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    REXSC_CHECK_ARG(prec >= 0 && prec <= 16, "prec must be 0..16 (got %d)", prec);
    if (n == 0) return REXSC_OK;
    REXSC_CHECK_ARG(x && y, "null pointer");
    const float scale = (float)(1u << prec);
    const int grid = pw_grid((n + 3) / 4);
    ProfScope prof("quantize", 8.0 * n, stream);
    hipLaunchKernelGGL(quantize_kernel, dim3(grid), dim3(PW_THREADS), 0, stream, x, y, n, scale, 1.0f / scale,
                       scale - 1.0f);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}
