// Sustained matrix-core rate of one MI355X with all operands in registers: the ceiling that the
// chip's power management leaves to any bf16 GEMM, before a single byte moves through LDS or HBM.
//
//   mfma_rate [iterations]
//
// Every wave of a one-workgroup-per-CU launch (8 waves, two per SIMD, the occupancy of the grouped
// GEMM) issues back-to-back MFMAs on 8 + 8 operand fragments that rotate from instruction to
// instruction, so no two consecutive instructions see the same inputs.  Run with random operands of
// N(0,1)-like magnitude and with all-zero operands: the gap between the two is what data-dependent
// switching power costs in clock.  Prints one line per case:  shape, operands, ms, TFLOP/s.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

#define CHECK(e)                                                                  \
    do {                                                                          \
        hipError_t err__ = (e);                                                   \
        if (err__ != hipSuccess) {                                                \
            fprintf(stderr, "%s: %s\n", #e, hipGetErrorString(err__));            \
            exit(1);                                                              \
        }                                                                         \
    } while (0)

// WIDE: v_mfma_f32_32x32x16_bf16 on 8 accumulators of 16 registers; else v_mfma_f32_16x16x32_bf16
// on 32 accumulators of 4 registers (128 accumulator registers either way, as in the GEMM).
template <bool WIDE>
__global__ __launch_bounds__(512) void mfma_loop(const bf16x8* __restrict__ src, float* __restrict__ out, int iters) {
    bf16x8 a[8], b[8];
    for (int i = 0; i < 8; ++i) {
        a[i] = src[threadIdx.x * 16 + i];
        b[i] = src[threadIdx.x * 16 + 8 + i];
    }
    float s = 0.0f;
    if (WIDE) {
        f32x16 acc[8];
        for (int i = 0; i < 8; ++i) acc[i] = f32x16{0};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + 3 * u) & 7], b[(i + u) & 7], acc[i], 0, 0, 0);
        }
        for (int i = 0; i < 8; ++i)
            for (int j = 0; j < 16; ++j) s += acc[i][j];
    } else {
        f32x4 acc[32];
        for (int i = 0; i < 32; ++i) acc[i] = f32x4{0};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    acc[i + 16 * (u & 1)] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        a[(i + 3 * u) & 7], b[(i + (i >> 3) + u) & 7], acc[i + 16 * (u & 1)], 0, 0, 0);
        }
        for (int i = 0; i < 32; ++i)
            for (int j = 0; j < 4; ++j) s += acc[i][j];
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

template <bool WIDE>
void run(const bf16x8* src, float* out, int n_cu, int iters, const char* shape, const char* operands) {
    hipLaunchKernelGGL(mfma_loop<WIDE>, dim3(n_cu), dim3(512), 0, 0, src, out, 16);
    CHECK(hipDeviceSynchronize());
    hipEvent_t t0, t1;
    CHECK(hipEventCreate(&t0));
    CHECK(hipEventCreate(&t1));
    const int reps = 10;
    CHECK(hipEventRecord(t0));
    for (int r = 0; r < reps; ++r) hipLaunchKernelGGL(mfma_loop<WIDE>, dim3(n_cu), dim3(512), 0, 0, src, out, iters);
    CHECK(hipEventRecord(t1));
    CHECK(hipEventSynchronize(t1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, t0, t1));
    ms /= reps;
    // per wave and iteration: 64 instructions of 32*32*16*2 flop, or 128 of 16*16*32*2 flop
    const double flop = (WIDE ? 64.0 * 32768 : 128.0 * 16384) * iters * 8.0 * n_cu;
    printf("%-22s %-7s %8.3f ms %8.1f TFLOP/s\n", shape, operands, ms, flop / ms / 1e9);
    fflush(stdout);
    CHECK(hipEventDestroy(t0));
    CHECK(hipEventDestroy(t1));
}

int main(int argc, char** argv) {
    const int iters = argc > 1 ? atoi(argv[1]) : 10000;
    int n_cu = 0;
    CHECK(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, 0));
    const size_t n = 512 * 16;   // fragments of 8 bf16
    std::vector<uint16_t> host(n * 8);
    bf16x8* src = nullptr;
    float* out = nullptr;
    CHECK(hipMalloc(&src, n * 16));
    CHECK(hipMalloc(&out, sizeof(float) * 512 * (size_t)n_cu));
    printf("# %d CUs, %d iterations per launch, 8 waves per CU\n", n_cu, iters);
    for (int zero = 0; zero < 2; ++zero) {
        srand(1);
        for (auto& v : host)   // random sign and mantissa, exponent 2^-7 .. 2^0
            v = zero ? 0 : (uint16_t)(((rand() & 1) << 15) | ((120 + (rand() & 7)) << 7) | (rand() & 0x7f));
        CHECK(hipMemcpy(src, host.data(), n * 16, hipMemcpyHostToDevice));
        const char* what = zero ? "zero" : "random";
        for (int rep = 0; rep < 2; ++rep) {
            run<true>(src, out, n_cu, iters, "mfma_f32_32x32x16_bf16", what);
            run<false>(src, out, n_cu, iters, "mfma_f32_16x16x32_bf16", what);
        }
    }
    CHECK(hipFree(src));
    CHECK(hipFree(out));
    return 0;
}
