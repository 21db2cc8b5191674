// fpmath.h -- scalar arithmetic shared by every kernel of libsvox_hip.
//
// The library is compiled with -ffp-contract=off: the compiler fuses nothing on its own, and every
// fused multiply-add the kernels use is written out with fma_().  The fusions follow what nvcc's
// default contraction does to the reference's expressions (a product whose only use is an addend
// is fused; in `a*b + c*d` the left product is the fused one), so a sample position, a step length
// and therefore the sequence of leaves a ray visits are fixed functions of the inputs.
// Division and square root are the correctly rounded ones (hipcc's default for HIP).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace svox {

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_(double a, double b, double c) { return __builtin_fma(a, b, c); }

__device__ __forceinline__ float min_(float a, float b) { return __builtin_fminf(a, b); }
__device__ __forceinline__ float max_(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double min_(double a, double b) { return __builtin_fmin(a, b); }
__device__ __forceinline__ double max_(double a, double b) { return __builtin_fmax(a, b); }

__device__ __forceinline__ float floor_(float a) { return __builtin_floorf(a); }
__device__ __forceinline__ double floor_(double a) { return __builtin_floor(a); }

// Single-precision e^x standing in for the reference's expf (rt_kernel.cu:86-87, :280): Cody-Waite
// reduction by ln2 in two parts, degree-5 polynomial on [-ln2/2, ln2/2], scaling by 2^n in two
// exact steps.  At most 1 ulp from the true value on [-87, 88.72]; 0 below -87 (so no subnormal
// is ever produced), +inf above 88.7228.  Only fma/mul/add/round-to-nearest are used, so the
// result does not depend on the math library or on the machine.
__device__ __forceinline__ float expf_fixed(float x0) {
    // without branches: the polynomial runs on an argument inside the range (any, where x0 is
    // outside or NaN) and the special results are selected afterwards
    const bool low = x0 < -87.0f, high = x0 > 88.72283f, nan = !(x0 == x0);
    const float x = (low || high || nan) ? 0.0f : x0;
    const float n = __builtin_rintf(x * 1.44269504088896341f);
    float r = fma_(n, -0.693145751953125f, x);
    r = fma_(n, -1.428606765330187045e-06f, r);
    float p = 1.9875691500e-4f;
    p = fma_(p, r, 1.3981999507e-3f);
    p = fma_(p, r, 8.3334519073e-3f);
    p = fma_(p, r, 4.1665795894e-2f);
    p = fma_(p, r, 1.6666665459e-1f);
    p = fma_(p, r, 5.0000001201e-1f);
    const float z = r * r;
    float y = fma_(p, z, r);
    y = y + 1.0f;
    const int ni = (int)n;
    const int n1 = ni >> 1, n2 = ni - n1;
    const float s1 = __uint_as_float((uint32_t)(n1 + 127) << 23);
    const float s2 = __uint_as_float((uint32_t)(n2 + 127) << 23);
    const float e = (y * s1) * s2;
    return nan ? x0 : (low ? 0.0f : (high ? __builtin_inff() : e));
}

// expf applied to a scalar_t argument (the reference calls expf in double builds too)
template <typename T>
__device__ __forceinline__ T exp_sp(T x) {
    return (T)expf_fixed((float)x);
}

// _SIGMOID, rt_kernel.cu:87
template <typename T>
__device__ __forceinline__ T sigmoid_(T x) {
    return T(1) / (T(1) + exp_sp<T>(-x));
}

// _SOFTPLUS_M1, rt_kernel.cu:86: logf(1 + expf(x - 1))
template <typename T>
__device__ __forceinline__ T softplus_m1(T x) {
    return (T)__builtin_logf((float)(T(1) + exp_sp<T>(x - T(1))));
}

// _norm, rt_kernel.cu:89-93: sqrtf, i.e. a single-precision root in every build
template <typename T>
__device__ __forceinline__ T norm3(const T* d) {
    const T s = fma_(d[2], d[2], fma_(d[0], d[0], d[1] * d[1]));
    return (T)__builtin_sqrtf((float)s);
}

// _dot3, rt_kernel.cu:103-108
template <typename T>
__device__ __forceinline__ T dot3(const T* u, const T* v) {
    return fma_(u[2], v[2], fma_(u[0], v[0], u[1] * v[1]));
}

// clamp_coord, common.cuh:36-41.  The bound 1 - 1e-6 is formed in double; a float coordinate
// compares against it exactly as against its rounded value 0x3F7FFFEF.  NaN maps to the bound.
__device__ __forceinline__ float clamp01(float q) {
    return max_(0.0f, min_(__uint_as_float(0x3F7FFFEFu), q));
}
__device__ __forceinline__ double clamp01(double q) { return max_(0.0, min_(1.0 - 1e-6, q)); }

}  // namespace svox
