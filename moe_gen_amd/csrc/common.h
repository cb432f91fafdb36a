// Shared host/device helpers of libmoe_mi355.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/moe_mi355.h"

namespace moe {

// Records the message returned by moe_last_error() for the calling thread.
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

constexpr int kWave = 64;

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(32 * sizeof(float)))) float f32x32;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// fp32 -> bf16 bits, round to nearest even (NaN stays a quiet NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ float round_to_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// Two fp32 -> packed bf16 (a in the low half) with the hardware conversion v_cvt_pk_bf16_f32: round to
// nearest even, NaN -> (bits >> 16) | 0x40, i.e. the same bits as f32_to_bf16_bits for every one of
// the 2^32 inputs (checked exhaustively on the device).
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    f32x2 f = {a, b};
    bf16x2 h = __builtin_convertvector(f, bf16x2);
    return __builtin_bit_cast(uint32_t, h);
}

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace moe

#define MOE_HIP_CHECK(expr)                                                      \
    do {                                                                         \
        hipError_t e__ = (expr);                                                 \
        if (e__ != hipSuccess) {                                                 \
            moe::set_error("%s: %s", #expr, hipGetErrorString(e__));             \
            return MOE_ERR_HIP;                                                  \
        }                                                                        \
    } while (0)

#define MOE_REQUIRE(cond, ...)                                                   \
    do {                                                                         \
        if (!(cond)) {                                                           \
            moe::set_error(__VA_ARGS__);                                         \
            return MOE_ERR_INVALID;                                              \
        }                                                                        \
    } while (0)
