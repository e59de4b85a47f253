// exp and log built from IEEE-754 single-precision operations only (add, multiply, divide, fused
// multiply-add, integer bit manipulation), in a fixed order.
//
// The perplexity search stops on |H - ln(perplexity)| < epsilon, so one unit in the last place of an
// exponential can move a row's stopping point by a whole bisection step.  Library exp/log differ in
// their last bits from one implementation to the next; these do not: any machine that evaluates the same
// sequence of correctly rounded operations gets the same bits, which lets a CPU restatement follow the
// GPU's bisection path exactly.  Both are accurate to about one unit in the last place (the reference's
// __expf / __logf, src/kernels/perplexity_search.cu:32 and thrust_transform_functions.h:34, are looser).
#ifndef TSNE_HIP_DET_MATH_H_
#define TSNE_HIP_DET_MATH_H_

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstring>

namespace tsnehip {

__host__ __device__ inline float det_bits_to_float(uint32_t u) {
    float f;
    memcpy(&f, &u, sizeof(f));
    return f;
}
__host__ __device__ inline uint32_t det_float_to_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof(u));
    return u;
}

// e^x.  x = n ln2 + r with n = round(x log2 e) (formed by adding 1.5 * 2^23), |r| <= 0.347 in two steps with
// a split ln2, a degree-7 Taylor polynomial in Horner form for e^r, and the scaling by 2^n as two exact
// power-of-two factors (so the only rounding of the scaling is the one into a subnormal result).
__host__ __device__ inline float det_expf(float x) {
#pragma clang fp contract(off)
    if (x != x) return x;
    if (!(x > -104.0f)) return 0.0f;
    if (x > 88.72f) return det_bits_to_float(0x7f800000u);
    const float t = fmaf(x, 1.44269504f, 12582912.0f);
    const float n = t - 12582912.0f;
    float r = fmaf(n, -0.693145752f, x);
    r = fmaf(n, -1.42860677e-6f, r);
    float p = 1.0f / 5040.0f;
    p = fmaf(p, r, 1.0f / 720.0f);
    p = fmaf(p, r, 1.0f / 120.0f);
    p = fmaf(p, r, 1.0f / 24.0f);
    p = fmaf(p, r, 1.0f / 6.0f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    const int ni = (int)n;
    const int half = ni / 2;
    const float a = det_bits_to_float((uint32_t)(half + 127) << 23);
    const float b = det_bits_to_float((uint32_t)(ni - half + 127) << 23);
    return (p * a) * b;
}

// ln v.  v = m 2^e with m in [sqrt(1/2), sqrt(2)), f = m - 1, s = f / (2 + f), z = s^2;
// ln m = 2 atanh(s) = f - s (f - R) with R = z (2/3 + z (2/5 + z (2/7 + z (2/9 + z 2/11)))), and
// ln v = e ln2_hi + (ln m + e ln2_lo).  Subnormal arguments are scaled by 2^25 first.
__host__ __device__ inline float det_logf(float v) {
#pragma clang fp contract(off)
    if (v != v) return v;
    if (v < 0.0f) return det_bits_to_float(0x7fc00000u);
    if (v == 0.0f) return det_bits_to_float(0xff800000u);
    uint32_t bits = det_float_to_bits(v);
    if (bits == 0x7f800000u) return v;
    int e = 0;
    if (bits < 0x00800000u) {
        v = v * 33554432.0f;
        bits = det_float_to_bits(v);
        e = -25;
    }
    bits += 0x3f800000u - 0x3f3504f3u;
    e += (int)(bits >> 23) - 127;
    bits = (bits & 0x007fffffu) + 0x3f3504f3u;
    const float f = det_bits_to_float(bits) - 1.0f;
    const float s = f / (2.0f + f);
    const float z = s * s;
    float R = 2.0f / 11.0f;
    R = fmaf(R, z, 2.0f / 9.0f);
    R = fmaf(R, z, 2.0f / 7.0f);
    R = fmaf(R, z, 2.0f / 5.0f);
    R = fmaf(R, z, 2.0f / 3.0f);
    R = R * z;
    const float ef = (float)e;
    float res = fmaf(ef, 1.42860677e-6f, -(s * (f - R)));
    res = res + f;
    return fmaf(ef, 0.693145752f, res);
}

}  // namespace tsnehip

#endif  // TSNE_HIP_DET_MATH_H_
