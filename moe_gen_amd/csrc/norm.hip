// RMSNorm ahead of the MoE block for gfx950: the reference's post_attention_layernorm,
//   DeepseekV3RMSNorm.forward  modeling_deepseek_v3.py:125-150
//   DeepseekV2RMSNorm.forward  modeling_deepseek_v2.py:127-134
//     xf = x.float(); var = xf.pow(2).mean(-1); y = (xf * rsqrt(var + eps)).to(bf16); out = weight * y
// in one pass over the row (the reference runs five elementwise/reduction kernels and three
// host-synchronising isnan/isinf checks).  HBM bound: 2nh bytes in, 2nh bytes out.
//
// One wave per row, 16 bytes (8 bf16) per lane per step.  Summation order (shared with the CPU
// checker): lane l adds the squares of chunks l, l+64, ... in ascending order, then a xor
// butterfly 32..1; var = sum / h; rstd = 1 / sqrt(var + eps), sqrt and divide correctly rounded.
// Rows of up to 8192 elements stay in registers between the two passes (CPL = 4, 8 or 16 chunks per
// lane, all requested before the first is used); longer rows (CPL = 0) are read a second time, from
// cache.
#include "common.h"

namespace moe {
namespace {

template <int CPL>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const u32x4* __restrict__ x, const u32x4* __restrict__ w,
                                                      float eps, int n, int chunks, u32x4* __restrict__ out) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.x * 4 + wave;
    if (row >= n) return;
    const u32x4* xr = x + (size_t)row * chunks;
    constexpr bool RESIDENT = CPL > 0;
    u32x4 keep[RESIDENT ? CPL : 1];
    if (RESIDENT) {
        // unconditional loads (index clamped): the compiler then waits per chunk, not for all of them
#pragma unroll
        for (int j = 0; j < CPL; ++j) keep[j] = __builtin_nontemporal_load(&xr[min(lane + 64 * j, chunks - 1)]);
    }
    float acc = 0.0f;
    auto add_squares = [&](const u32x4 v) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = __uint_as_float(v[i] << 16), hi = __uint_as_float(v[i] & 0xffff0000u);
            acc = acc + lo * lo;
            acc = acc + hi * hi;
        }
    };
    if (RESIDENT) {
#pragma unroll
        for (int j = 0; j < CPL; ++j)
            if (lane + 64 * j < chunks) add_squares(keep[j]);
    } else {
        for (int c = lane; c < chunks; c += 64) add_squares(xr[c]);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) acc = acc + __shfl_xor(acc, m);
    const float var = acc / (float)(chunks * 8);
    // sqrt and divide correctly rounded: the plain operators are (the __fsqrt_rn intrinsic is the
    // bare v_sqrt_f32, 1 ulp, and flips a bf16 rounding of x * rstd about once in a few hundred rows)
    const float rstd = 1.0f / __builtin_sqrtf(var + eps);
    u32x4* orow = out + (size_t)row * chunks;
    auto scale = [&](const u32x4 v, const u32x4 g) {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t y = pack_bf16(__uint_as_float(v[i] << 16) * rstd, __uint_as_float(v[i] & 0xffff0000u) * rstd);
            o[i] = pack_bf16(__uint_as_float(g[i] << 16) * __uint_as_float(y << 16),
                             __uint_as_float(g[i] & 0xffff0000u) * __uint_as_float(y & 0xffff0000u));
        }
        return o;
    };
    if (RESIDENT) {
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
            const int c = lane + 64 * j;
            if (c < chunks) orow[c] = scale(keep[j], w[c]);
        }
    } else {
        for (int c = lane; c < chunks; c += 64) orow[c] = scale(xr[c], w[c]);
    }
}

}  // namespace
}  // namespace moe

extern "C" int moe_rmsnorm(const void* x, const void* weight, float eps, int32_t n_tokens, int32_t hidden, void* out,
                           void* stream) {
    using namespace moe;
    MOE_REQUIRE(n_tokens >= 0, "moe_rmsnorm: n_tokens %d < 0", n_tokens);
    if (n_tokens == 0) return MOE_OK;
    MOE_REQUIRE(x && weight && out, "moe_rmsnorm: NULL tensor pointer");
    MOE_REQUIRE(x != out, "moe_rmsnorm: out must not alias x (the row is read twice)");
    MOE_REQUIRE(hidden > 0 && hidden % 8 == 0, "moe_rmsnorm: hidden %d must be a positive multiple of 8", hidden);
    MOE_REQUIRE(eps >= 0.0f, "moe_rmsnorm: eps %g < 0", (double)eps);
    const int chunks = hidden / 8;
    const dim3 grid((unsigned)((n_tokens + 3) / 4)), block(256);
#define MOE_LAUNCH_NORM(CPL)                                                                                       \
    hipLaunchKernelGGL(rmsnorm_kernel<CPL>, grid, block, 0, as_stream(stream), static_cast<const u32x4*>(x),      \
                       static_cast<const u32x4*>(weight), eps, n_tokens, chunks, static_cast<u32x4*>(out))
    if (chunks <= 256) MOE_LAUNCH_NORM(4);
    else if (chunks <= 512) MOE_LAUNCH_NORM(8);
    else if (chunks <= 1024) MOE_LAUNCH_NORM(16);
    else MOE_LAUNCH_NORM(0);
#undef MOE_LAUNCH_NORM
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}
