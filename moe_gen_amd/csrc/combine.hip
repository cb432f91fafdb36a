// Weighted combine for gfx950: inverse permutation, weighted sum over the k slots and
// the shared-expert add in one pass over the expert outputs.
//
// Replaces the second half of moe_infer in the reference
//   V3  modeling_deepseek_v3.py:702-710:  new_x[idxs] = outs;
//        (new_x.view(n,k,h).float() * w[...,None]).sum(1).to(bf16)
//   V2  modeling_deepseek_v2.py:744-757:  same with w cast to bf16 first (bf16 products)
//   Mixtral (transformers 4.42.0): final.index_add_(0, top_x, expert_out * w) per expert
// and `y = y + self.shared_experts(identity)` (modeling_deepseek_v3.py:624-625); optionally also the
// decoder layer's `hidden_states = residual + hidden_states` that follows the block (:1365).
// The reference materialises new_x [n,k,h] (and an fp32 copy of it); here each
// output element is accumulated in a register from the k source rows.
//
// One block per token; a lane handles 8 consecutive bf16 (16 bytes) of the row, so
// every global access is a full 16-byte vector and a wave covers 1 KiB contiguous.
#include "common.h"

namespace moe {
namespace {

constexpr int MAX_K = 16;

// KB: source rows whose 16-byte chunks a lane requests back to back before it starts adding (the
// sum itself stays in slot order).  The kernel is bound by HBM latency x bytes in flight, and one
// outstanding load per lane is too few.  The block has one lane per chunk of the row where that
// fits (up to 1024 threads), so a token's loads all leave at once.  Expert outputs are read once and
// the result is not read again here: both go past the caches non-temporally (measured on 65536 x 8
// rows of 7168: 1.90 -> 1.70 ms; 32768 x 6 of 5120: 0.54 -> 0.46 ms).
template <int MODE, int KB>
__global__ __launch_bounds__(1024) void combine_kernel(const u32x4* __restrict__ y, const int32_t* __restrict__ pos,
                                                      const int32_t* __restrict__ topk_idx,
                                                      const float* __restrict__ topk_w, const u32x4* __restrict__ shared,
                                                      const u32x4* residual, int k, int chunks, u32x4* out) {
    __shared__ int s_row[MAX_K];
    __shared__ float s_w[MAX_K];
    const int t = blockIdx.x;
    if (threadIdx.x < k) {
        // position of slot j in the summation order: the slot order itself, or (Mixtral, which
        // adds expert by expert) the rank of its expert id among the k distinct ids of the token
        const int j = threadIdx.x;
        int a = j;
        if (MODE == MOE_COMBINE_BF16_SEQ) {
            const int ej = topk_idx[(size_t)t * k + j];
            a = 0;
            for (int i = 0; i < k; ++i) a += topk_idx[(size_t)t * k + i] < ej ? 1 : 0;
        }
        s_row[a] = pos[(size_t)t * k + j];
        const float w = topk_w[(size_t)t * k + j];
        s_w[a] = (MODE == MOE_COMBINE_F32) ? w : round_to_bf16(w);
    }
    __syncthreads();
    for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        u32x4 sh = {0, 0, 0, 0}, res = {0, 0, 0, 0};
        if (shared) sh = __builtin_nontemporal_load(&shared[(size_t)t * chunks + c]);
        if (residual) res = __builtin_nontemporal_load(&residual[(size_t)t * chunks + c]);   // may alias out: read before this thread writes
        for (int a0 = 0; a0 < k; a0 += KB) {
        u32x4 vb[KB];
#pragma unroll
        for (int b = 0; b < KB; ++b) {
            // past k: the last row again; a negative row (a slot whose expert id moe_dispatch found outside
            // [0, E)) is neither read nor added -- the same for every lane of the block
            const int row = s_row[min(a0 + b, k - 1)];
            vb[b] = row < 0 ? u32x4{0, 0, 0, 0} : __builtin_nontemporal_load(&y[(size_t)row * chunks + c]);
        }
#pragma unroll
        for (int b = 0; b < KB; ++b) {
            if (a0 + b >= k) break;
            if (s_row[a0 + b] < 0) continue;
            const u32x4 v = vb[b];
            const float w = s_w[a0 + b];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float lo = __uint_as_float(v[i] << 16), hi = __uint_as_float(v[i] & 0xffff0000u);
                if (MODE == MOE_COMBINE_F32) {
                    acc[2 * i] = acc[2 * i] + lo * w;
                    acc[2 * i + 1] = acc[2 * i + 1] + hi * w;
                } else {
                    acc[2 * i] = acc[2 * i] + round_to_bf16(lo * w);
                    acc[2 * i + 1] = acc[2 * i + 1] + round_to_bf16(hi * w);
                    if (MODE == MOE_COMBINE_BF16_SEQ) {
                        acc[2 * i] = round_to_bf16(acc[2 * i]);
                        acc[2 * i + 1] = round_to_bf16(acc[2 * i + 1]);
                    }
                }
            }
        }
        }
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t lo = f32_to_bf16_bits(acc[2 * i]), hi = f32_to_bf16_bits(acc[2 * i + 1]);
            if (shared) {  // bf16 + bf16 -> bf16, as torch adds two bf16 tensors
                lo = f32_to_bf16_bits(bf16_bits_to_f32(lo) + __uint_as_float(sh[i] << 16));
                hi = f32_to_bf16_bits(bf16_bits_to_f32(hi) + __uint_as_float(sh[i] & 0xffff0000u));
            }
            o[i] = lo | (hi << 16);
        }
        if (residual) {
            const u32x4 r = res;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t lo = f32_to_bf16_bits(__uint_as_float(r[i] << 16) + __uint_as_float(o[i] << 16));
                const uint32_t hi = f32_to_bf16_bits(__uint_as_float(r[i] & 0xffff0000u) + __uint_as_float(o[i] & 0xffff0000u));
                o[i] = lo | (hi << 16);
            }
        }
        __builtin_nontemporal_store(o, &out[(size_t)t * chunks + c]);
    }
}

}  // namespace
}  // namespace moe

namespace moe {
namespace {
int combine_impl(const void* y, const int32_t* pos, const int32_t* topk_idx, const float* topk_w, const void* shared,
                 const void* residual, int32_t n_tokens, int32_t top_k, int32_t hidden, int32_t mode, void* out,
                 void* stream, const char* who) {
    MOE_REQUIRE(n_tokens >= 0, "%s: n_tokens %d < 0", who, n_tokens);
    if (n_tokens == 0) return MOE_OK;
    MOE_REQUIRE(y && pos && topk_w && out, "%s: NULL tensor pointer", who);
    MOE_REQUIRE(top_k >= 1 && top_k <= MAX_K, "%s: top_k %d outside [1,%d]", who, top_k, MAX_K);
    MOE_REQUIRE(hidden > 0 && hidden % 8 == 0, "%s: hidden %d must be a positive multiple of 8", who, hidden);
    MOE_REQUIRE(mode >= MOE_COMBINE_F32 && mode <= MOE_COMBINE_BF16_SEQ, "%s: bad mode %d", who, mode);
    MOE_REQUIRE(mode != MOE_COMBINE_BF16_SEQ || topk_idx, "%s: topk_idx is required for MOE_COMBINE_BF16_SEQ", who);
    MOE_REQUIRE(out != y && out != shared, "%s: out must not alias y or shared", who);
    hipStream_t st = as_stream(stream);
    const int chunks = hidden / 8;
    // One lane per chunk (hidden <= 8192: one pass) when a token has more than two source rows; with
    // one or two rows a lane has too few loads in flight for that, and 256-thread blocks that fill
    // the CU exactly measured better (8192 x 2 rows of 6144: 0.07 vs 0.08 ms).
    const int passes = (chunks + 1023) / 1024;
    const int threads = top_k <= 2 ? 256 : (((chunks + passes - 1) / passes + 63) / 64) * 64;
    dim3 grid(n_tokens), block(threads);
    const u32x4* yv = static_cast<const u32x4*>(y);
    const u32x4* sv = static_cast<const u32x4*>(shared);
    const u32x4* rv = static_cast<const u32x4*>(residual);
    u32x4* ov = static_cast<u32x4*>(out);
#define MOE_LAUNCH_COMBINE(M, B) \
    hipLaunchKernelGGL((combine_kernel<M, B>), grid, block, 0, st, yv, pos, topk_idx, topk_w, sv, rv, top_k, chunks, ov)
#define MOE_LAUNCH_COMBINE_K(M)                          \
    do {                                                 \
        if (top_k <= 2) MOE_LAUNCH_COMBINE(M, 2);        \
        else if (top_k <= 4) MOE_LAUNCH_COMBINE(M, 4);   \
        else MOE_LAUNCH_COMBINE(M, 8);                   \
    } while (0)
    if (mode == MOE_COMBINE_F32) MOE_LAUNCH_COMBINE_K(MOE_COMBINE_F32);
    else if (mode == MOE_COMBINE_BF16_PROD) MOE_LAUNCH_COMBINE_K(MOE_COMBINE_BF16_PROD);
    else MOE_LAUNCH_COMBINE_K(MOE_COMBINE_BF16_SEQ);
#undef MOE_LAUNCH_COMBINE_K
#undef MOE_LAUNCH_COMBINE
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}
}  // namespace
}  // namespace moe

extern "C" int moe_combine(const void* y, const int32_t* pos, const int32_t* topk_idx, const float* topk_w,
                           const void* shared, int32_t n_tokens, int32_t top_k, int32_t hidden, int32_t mode,
                           void* out, void* stream) {
    return moe::combine_impl(y, pos, topk_idx, topk_w, shared, nullptr, n_tokens, top_k, hidden, mode, out, stream,
                             "moe_combine");
}

extern "C" int moe_combine_residual(const void* y, const int32_t* pos, const int32_t* topk_idx, const float* topk_w,
                                    const void* shared, const void* residual, int32_t n_tokens, int32_t top_k,
                                    int32_t hidden, int32_t mode, void* out, void* stream) {
    MOE_REQUIRE(residual || n_tokens == 0, "moe_combine_residual: NULL residual");
    return moe::combine_impl(y, pos, topk_idx, topk_w, shared, residual, n_tokens, top_k, hidden, mode, out, stream,
                             "moe_combine_residual");
}
