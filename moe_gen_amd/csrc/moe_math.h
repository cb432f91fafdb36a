// Canonical fp32 exp / sigmoid of the router: a fixed sequence of IEEE operations
// (explicit fma, round-to-nearest-even, correctly rounded division) so that every
// score is a pure function of the fp32 logit, independent of libm and of compiler
// contraction.  The translation unit that includes this must be built with
// -ffp-contract=off and without fast-math.
#pragma once
#include <hip/hip_runtime.h>

namespace moe {

// exp(x): n = rne(x*log2e); r = x - n*ln2 (two-term Cody-Waite); degree-5
// polynomial (cephes expf coefficients) * r^2 + r + 1; scaled by 2^n in two
// power-of-two multiplies so a subnormal result is rounded once.
__device__ __forceinline__ float canon_expf(float x) {
    if (!(x == x)) return x;
    if (x < -104.0f) return 0.0f;
    if (x > 88.72283f) return __uint_as_float(0x7f800000u);
    float t = x * 1.44269504088896341f;
    float n = rintf(t);
    float r = fmaf(n, -0.693145751953125f, x);
    r = fmaf(n, -1.42860682030941723212e-6f, r);
    float z = r * r;
    float y = 1.9875691500e-4f;
    y = fmaf(y, r, 1.3981999507e-3f);
    y = fmaf(y, r, 8.3334519073e-3f);
    y = fmaf(y, r, 4.1665795894e-2f);
    y = fmaf(y, r, 1.6666665459e-1f);
    y = fmaf(y, r, 5.0000001201e-1f);
    y = fmaf(y, z, r);
    y = y + 1.0f;
    int ni = (int)n;
    int n1 = ni / 2, n2 = ni - n1;
    y = y * __uint_as_float((uint32_t)(n1 + 127) << 23);
    y = y * __uint_as_float((uint32_t)(n2 + 127) << 23);
    return y;
}

__device__ __forceinline__ float canon_sigmoidf(float x) { return 1.0f / (1.0f + canon_expf(-x)); }

}  // namespace moe
