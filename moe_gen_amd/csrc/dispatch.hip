// Token-to-expert dispatch for gfx950: per-expert histogram, exclusive prefix sum,
// stable permutation and the row gather, all on the device (no host sync).
//
// Replaces the first half of moe_infer in the reference
// (modeling_deepseek_v3.py:630-634 and :673, identical in modeling_deepseek_v2.py:672-676,715):
//     cnts.scatter_(1, topk_ids, 1); tokens_per_expert = cnts.sum(0)
//     idxs = topk_ids.view(-1).argsort();  sorted_tokens = x[idxs // k]
// The sort is a stable counting sort: sorted row of flat entry i with expert e is
//     offsets[e] + #{i' < i : idx[i'] == e}
// which is a pure function of the index list, hence identical on every run.
//
// Three small kernels over the n*k index list (a few MB at most):
//   1. block_histogram : each block counts its 2048-entry segment per expert (LDS atomics)
//   2. scan_segments   : one wave per expert turns the per-segment counts into exclusive
//                        bases across segments and writes counts[e]
//   3. rank_scatter    : each block rebuilds offsets[] in LDS, ranks its entries with
//                        wave-level match masks and writes perm / pos (and row_map = perm / k,
//                        the token row behind each sorted row, for the GEMM's fused gather)
// and one bandwidth kernel:
//   4. gather_rows     : xs[r] = x[perm[r] / k], one wave per row, 16 bytes per lane.
#include <mutex>

#include "common.h"

namespace moe {
namespace {

constexpr int SEG_PER_WAVE = 512;   // flat entries ranked by one wave
constexpr int SEG_WAVES = 4;
constexpr int SEG = SEG_PER_WAVE * SEG_WAVES;  // entries per block
constexpr int MAX_E = 256;

__global__ void zero_i32(int32_t* a, int na, int32_t* b, int nb) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < na) a[i] = 0;
    if (i < nb) b[i] = 0;
}

__global__ __launch_bounds__(256) void block_histogram(const int32_t* __restrict__ idx, int64_t nk, int E,
                                                       int32_t* __restrict__ seg_counts) {
    __shared__ int hist[MAX_E];
    for (int e = threadIdx.x; e < E; e += 256) hist[e] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * SEG;
    for (int i = threadIdx.x; i < SEG; i += 256) {
        int64_t g = base + i;
        if (g < nk) {
            int e = idx[g];
            if ((unsigned)e < (unsigned)E) atomicAdd(&hist[e], 1);
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += 256) seg_counts[(size_t)blockIdx.x * E + e] = hist[e];
}

// one wave per expert: in-place exclusive scan of seg_counts[:, e] over segments
__global__ __launch_bounds__(256) void scan_segments(int32_t* __restrict__ seg_counts, int nseg, int E,
                                                     int32_t* __restrict__ counts) {
    const int lane = threadIdx.x & 63;
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (e >= E) return;
    int carry = 0;
    for (int b0 = 0; b0 < nseg; b0 += 64) {
        int b = b0 + lane;
        int v = b < nseg ? seg_counts[(size_t)b * E + e] : 0;
        int inc = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            int o = __shfl_up(inc, d);
            if (lane >= d) inc += o;
        }
        if (b < nseg) seg_counts[(size_t)b * E + e] = carry + inc - v;
        carry += __shfl(inc, 63);
    }
    if (lane == 0) counts[e] = carry;
}

__global__ __launch_bounds__(256) void rank_scatter(const int32_t* __restrict__ idx, int64_t nk, int E,
                                                    const int32_t* __restrict__ seg_base,
                                                    const int32_t* __restrict__ counts,
                                                    int32_t* __restrict__ offsets, int32_t* __restrict__ perm,
                                                    int32_t* __restrict__ pos, int32_t* __restrict__ row_map, int k) {
    __shared__ int off[MAX_E];                 // exclusive prefix sum of counts
    __shared__ int whist[SEG_WAVES][MAX_E];    // per-wave counts, then per-wave running cursors
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // offsets[e] = sum_{e' < e} counts[e'] : 256-wide scan by the whole block
    int cv = tid < E ? counts[tid] : 0;
    int inc = cv;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        int o = __shfl_up(inc, d);
        if (lane >= d) inc += o;
    }
    __shared__ int wtot[4];
    if (lane == 63) wtot[wave] = inc;
    for (int e = tid; e < SEG_WAVES * MAX_E; e += 256) (&whist[0][0])[e] = 0;
    __syncthreads();
    int wpre = 0;
    for (int w = 0; w < wave; ++w) wpre += wtot[w];
    off[tid] = wpre + inc - cv;
    if (blockIdx.x == 0) {
        if (tid < E) offsets[tid] = wpre + inc - cv;
        if (tid == E - 1) offsets[E] = wpre + inc;
    }

    // pass 1: counts of this wave's 512-entry slice
    const int64_t wbase = (int64_t)blockIdx.x * SEG + (int64_t)wave * SEG_PER_WAVE;
    for (int i = lane; i < SEG_PER_WAVE; i += 64) {
        int64_t g = wbase + i;
        if (g < nk) {
            int e = idx[g];
            if ((unsigned)e < (unsigned)E) atomicAdd(&whist[wave][e], 1);
        }
    }
    __syncthreads();
    // cursor of wave w for expert e = offsets[e] + base of this segment + counts of earlier waves
    if (tid < E) {
        int run = off[tid] + seg_base[(size_t)blockIdx.x * E + tid];
#pragma unroll
        for (int w = 0; w < SEG_WAVES; ++w) {
            int c = whist[w][tid];
            whist[w][tid] = run;
            run += c;
        }
    }
    __syncthreads();

    // pass 2: stable rank inside the wave slice, 64 entries at a time in index order
    int* cur = whist[wave];
    for (int i0 = 0; i0 < SEG_PER_WAVE; i0 += 64) {
        int64_t g = wbase + i0 + lane;
        const bool in_list = g < nk;
        int e = in_list ? idx[g] : 0;
        const bool ok = in_list && (unsigned)e < (unsigned)E;
        // an expert id outside [0, E) owns no sorted row: its slot gets -1, which the combine
        // skips (no row read, nothing added)
        if (in_list && !ok) pos[g] = -1;
        uint64_t peers = __ballot(ok);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            bool bit = (e >> b) & 1;
            uint64_t bal = __ballot(bit);
            peers &= bit ? bal : ~bal;
        }
        if (ok) {
            uint64_t below = peers & ((1ull << lane) - 1ull);
            int r = cur[e] + __popcll(below);
            perm[r] = (int32_t)g;
            pos[g] = r;
            if (row_map) row_map[r] = (int32_t)(g / k);
        }
        // every read of cur[] above precedes this update in the wave's LDS order
        if (ok && (peers & ((1ull << lane) - 1ull)) == 0) cur[e] += __popcll(peers);
    }
}

// The three kernels above as one workgroup of 16 waves, for index lists of up to SMALL_MAX entries (a decode or small
// prefill batch: three dependent launches of a few microseconds each cost more than their work).  Wave w owns the
// w-th slice of the list (a multiple of 64 entries): counts it, the first 256 threads turn the 16 x E counts into
// counts[], offsets[] and one cursor per (wave, expert) -- offsets[e] + entries of e in earlier slices -- and every
// wave ranks its slice as rank_scatter does.  The sorted position of an entry is the same pure function of the list.
constexpr int SMALL_WAVES = 16;
constexpr int SMALL_MAX = 12288;   // one launch of 18.6 us against three of 21.7 (16384 entries: 23.7)

__global__ __launch_bounds__(64 * SMALL_WAVES) void dispatch_small(const int32_t* __restrict__ idx, int nk, int E,
                                                                   int32_t* __restrict__ counts,
                                                                   int32_t* __restrict__ offsets,
                                                                   int32_t* __restrict__ perm, int32_t* __restrict__ pos,
                                                                   int32_t* __restrict__ row_map, int k) {
    constexpr int IT = SMALL_MAX / (SMALL_WAVES * 64);   // 64-entry steps of a wave's slice, at most
    __shared__ int whist[SMALL_WAVES][MAX_E];
    __shared__ int wtot[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int slice = (nk + SMALL_WAVES * 64 - 1) / (SMALL_WAVES * 64) * 64;
    const int wbase = wave * slice;
    // the lane's entries of the slice, all requested at once (both passes use them: a load per step would put the
    // memory latency into every step); -1 marks an entry past the list or an id outside [0, E)
    int ev[IT];
#pragma unroll
    for (int it = 0; it < IT; ++it) ev[it] = idx[min(wbase + 64 * it + lane, nk - 1)];
    for (int e = tid; e < SMALL_WAVES * MAX_E; e += 64 * SMALL_WAVES) (&whist[0][0])[e] = 0;
    __syncthreads();
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int g = wbase + 64 * it + lane;
        if (64 * it >= slice || g >= nk || (unsigned)ev[it] >= (unsigned)E) ev[it] = -1;
        if (ev[it] >= 0) atomicAdd(&whist[wave][ev[it]], 1);
    }
    __syncthreads();
    int cv = 0, inc = 0;
    if (tid < MAX_E) {                         // waves 0 .. 3, whole waves
        if (tid < E) {
#pragma unroll
            for (int w = 0; w < SMALL_WAVES; ++w) cv += whist[w][tid];
        }
        inc = cv;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int o = __shfl_up(inc, d);
            if (lane >= d) inc += o;
        }
        if (lane == 63) wtot[wave] = inc;
    }
    __syncthreads();
    if (tid < E) {
        int run = inc - cv;
        for (int w = 0; w < wave; ++w) run += wtot[w];
        counts[tid] = cv;
        offsets[tid] = run;
        if (tid == E - 1) offsets[E] = run + cv;
#pragma unroll
        for (int w = 0; w < SMALL_WAVES; ++w) {
            const int c = whist[w][tid];
            whist[w][tid] = run;
            run += c;
        }
    }
    __syncthreads();
    int* cur = whist[wave];
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        if (64 * it >= slice) break;
        const int g = wbase + 64 * it + lane;
        const int e = ev[it];
        const bool ok = e >= 0;
        if (g < nk && !ok) pos[g] = -1;        // as in rank_scatter: no sorted row, the combine skips the slot
        uint64_t peers = __ballot(ok);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const bool bit = (e >> b) & 1;
            const uint64_t bal = __ballot(bit);
            peers &= bit ? bal : ~bal;
        }
        const uint64_t below = peers & ((1ull << lane) - 1ull);
        if (ok) {
            const int r = cur[e] + __popcll(below);
            perm[r] = g;
            pos[g] = r;
            if (row_map) row_map[r] = g / k;
        }
        if (ok && below == 0) cur[e] += __popcll(peers);
    }
}

__global__ __launch_bounds__(256) void gather_rows(const u32x4* __restrict__ x, const int32_t* __restrict__ perm,
                                                   int64_t nk, int k, int chunks, u32x4* __restrict__ xs) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= nk) return;
    const int t = perm[r] / k;
    const u32x4* src = x + (size_t)t * chunks;
    u32x4* dst = xs + (size_t)r * chunks;
    for (int c = lane; c < chunks; c += 64) __builtin_nontemporal_store(src[c], dst + c);
}

}  // namespace
}  // namespace moe

extern "C" size_t moe_dispatch_workspace_bytes(int32_t n_tokens, int32_t top_k, int32_t n_experts) {
    if (n_tokens <= 0 || top_k <= 0 || n_experts <= 0) return 256;
    int64_t nk = (int64_t)n_tokens * top_k;
    int64_t nseg = (nk + moe::SEG - 1) / moe::SEG;
    return (size_t)(nseg * n_experts * 4 + 256);
}

namespace moe {
namespace {

// The launches behind both entry points; `seg` holds nseg * n_experts per-segment counts.
int dispatch_launch(const int32_t* topk_idx, int64_t nk, int32_t top_k, int32_t n_experts, int32_t* counts,
                    int32_t* offsets, int32_t* perm, int32_t* pos, int32_t* row_map, const void* x, int32_t hidden,
                    void* xs, int32_t* seg, hipStream_t st) {
    if (nk <= SMALL_MAX) {
        hipLaunchKernelGGL(dispatch_small, dim3(1), dim3(64 * SMALL_WAVES), 0, st, topk_idx, (int)nk, n_experts, counts,
                           offsets, perm, pos, row_map, top_k);
    } else {
        const int nseg = (int)((nk + SEG - 1) / SEG);
        hipLaunchKernelGGL(block_histogram, dim3(nseg), dim3(256), 0, st, topk_idx, nk, n_experts, seg);
        hipLaunchKernelGGL(scan_segments, dim3((n_experts + 3) / 4), dim3(256), 0, st, seg, nseg, n_experts, counts);
        hipLaunchKernelGGL(rank_scatter, dim3(nseg), dim3(256), 0, st, topk_idx, nk, n_experts, seg, counts, offsets,
                           perm, pos, row_map, top_k);
    }
    if (x) {
        hipLaunchKernelGGL(gather_rows, dim3((unsigned)((nk + 3) / 4)), dim3(256), 0, st,
                           static_cast<const u32x4*>(x), perm, nk, top_k, hidden / 8, static_cast<u32x4*>(xs));
    }
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}

// argument checks shared by the entry points; *nk_out = n_tokens * top_k
int dispatch_check(const char* who, const int32_t* topk_idx, int32_t n_tokens, int32_t top_k, int32_t n_experts,
                   int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* pos, const void* x, int32_t hidden,
                   void* xs, int64_t* nk_out) {
    MOE_REQUIRE(n_tokens >= 0 && top_k >= 1, "%s: bad n_tokens %d / top_k %d", who, n_tokens, top_k);
    MOE_REQUIRE(n_experts >= 1 && n_experts <= MAX_E, "%s: n_experts %d outside [1,%d]", who, n_experts, MAX_E);
    MOE_REQUIRE(counts && offsets, "%s: counts/offsets is NULL", who);
    MOE_REQUIRE((x == nullptr) == (xs == nullptr), "%s: x and xs must both be given or both be NULL", who);
    const int64_t nk = (int64_t)n_tokens * top_k;
    MOE_REQUIRE(nk < (int64_t)1 << 31, "%s: n_tokens*top_k = %lld does not fit int32", who, (long long)nk);
    if (nk > 0) {
        MOE_REQUIRE(topk_idx && perm && pos, "%s: NULL index pointer", who);
        if (x) MOE_REQUIRE(hidden > 0 && hidden % 8 == 0, "%s: hidden %d must be a positive multiple of 8", who, hidden);
    }
    *nk_out = nk;
    return MOE_OK;
}

}  // namespace
}  // namespace moe

extern "C" int moe_dispatch(const int32_t* topk_idx, int32_t n_tokens, int32_t top_k, int32_t n_experts,
                            int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* pos, int32_t* row_map,
                            const void* x, int32_t hidden, void* xs, void* workspace, size_t workspace_bytes,
                            void* stream) {
    using namespace moe;
    int64_t nk = 0;
    int rc = dispatch_check("moe_dispatch", topk_idx, n_tokens, top_k, n_experts, counts, offsets, perm, pos, x, hidden,
                            xs, &nk);
    if (rc != MOE_OK) return rc;
    hipStream_t st = as_stream(stream);
    if (nk == 0) {
        hipLaunchKernelGGL(zero_i32, dim3(2), dim3(256), 0, st, counts, n_experts, offsets, n_experts + 1);
        MOE_HIP_CHECK(hipGetLastError());
        return MOE_OK;
    }
    const size_t need = (size_t)((nk + SEG - 1) / SEG) * n_experts * 4;
    if (workspace == nullptr || workspace_bytes < need) {
        set_error("moe_dispatch: workspace %zu bytes, need %zu", workspace_bytes, need);
        return MOE_ERR_WORKSPACE;
    }
    return dispatch_launch(topk_idx, nk, top_k, n_experts, counts, offsets, perm, pos, row_map, x, hidden, xs,
                           static_cast<int32_t*>(workspace), st);
}

// ---- moe_dispatch_static: the same launches with the per-segment counts in a file-scope device
// array instead of a caller workspace, for callers that cannot allocate.
namespace moe {
namespace {

constexpr size_t STATIC_SCRATCH_INTS = MOE_DISPATCH_STATIC_SCRATCH_BYTES / sizeof(int32_t);
// One copy per GPU the library runs on, held until the process ends.  block_histogram writes
// every entry it later reads (all n_experts counts of all segments of the call), so a call needs
// nothing cleared; what an earlier call left beyond that range is never read.
static __device__ __align__(256) int32_t scratch[STATIC_SCRATCH_INTS];

constexpr int MAX_DEVICES = 64;
std::mutex scratch_mu;
int32_t* scratch_ptr[MAX_DEVICES] = {nullptr};   // device address of `scratch` on each device

// Device address of this GPU's copy of `scratch`, looked up once per device with that device
// current.  (The array's name is only a host-side handle: kernels and copies take this pointer.)
int static_scratch(int32_t** out) {
    int dev = -1;
    MOE_HIP_CHECK(hipGetDevice(&dev));
    MOE_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "moe_dispatch_static: device %d outside [0,%d)", dev, MAX_DEVICES);
    std::lock_guard<std::mutex> lk(scratch_mu);
    if (scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        MOE_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        MOE_REQUIRE(p != nullptr, "moe_dispatch_static: hipGetSymbolAddress returned NULL on device %d", dev);
        scratch_ptr[dev] = static_cast<int32_t*>(p);
    }
    *out = scratch_ptr[dev];
    return MOE_OK;
}

}  // namespace
}  // namespace moe

extern "C" int moe_dispatch_static(const int32_t* topk_idx, int32_t n_tokens, int32_t top_k, int32_t n_experts,
                                   int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* pos, int32_t* row_map,
                                   const void* x, int32_t hidden, void* xs, void* stream) {
    using namespace moe;
    int64_t nk = 0;
    int rc = dispatch_check("moe_dispatch_static", topk_idx, n_tokens, top_k, n_experts, counts, offsets, perm, pos, x,
                            hidden, xs, &nk);
    if (rc != MOE_OK) return rc;
    const size_t need = (size_t)((nk + SEG - 1) / SEG) * n_experts;
    if (need > STATIC_SCRATCH_INTS) {
        set_error("moe_dispatch_static: ceil(n_tokens*top_k / %d) * n_experts = %zu counters exceed the built-in "
                  "scratch of %zu (%zu bytes); use moe_dispatch with a workspace", SEG, need, STATIC_SCRATCH_INTS,
                  (size_t)MOE_DISPATCH_STATIC_SCRATCH_BYTES);
        return MOE_ERR_WORKSPACE;
    }
    hipStream_t st = as_stream(stream);
    if (nk == 0) {
        hipLaunchKernelGGL(zero_i32, dim3(2), dim3(256), 0, st, counts, n_experts, offsets, n_experts + 1);
        MOE_HIP_CHECK(hipGetLastError());
        return MOE_OK;
    }
    int32_t* seg = nullptr;
    rc = static_scratch(&seg);
    if (rc != MOE_OK) return rc;
    return dispatch_launch(topk_idx, nk, top_k, n_experts, counts, offsets, perm, pos, row_map, x, hidden, xs, seg, st);
}

// ---- 64-bit words from the host into device memory inside kernel arguments ----
namespace moe {
namespace {
struct WordBlock { uint64_t v[256]; };
__global__ __launch_bounds__(256) void write_words_kernel(uint64_t* __restrict__ dst, WordBlock w, int n) {
    const int i = threadIdx.x;
    if (i < n) dst[i] = w.v[i];
}
}  // namespace
}  // namespace moe

extern "C" int moe_write_words(void* dst, const uint64_t* words, int32_t n, void* stream) {
    MOE_REQUIRE(n >= 0, "moe_write_words: n %d < 0", n);
    if (n == 0) return MOE_OK;
    MOE_REQUIRE(dst && words, "moe_write_words: NULL argument");
    MOE_REQUIRE((reinterpret_cast<uintptr_t>(dst) & 7) == 0, "moe_write_words: dst is not 8-byte aligned");
    for (int32_t at = 0; at < n; at += 256) {
        moe::WordBlock w;
        const int m = n - at < 256 ? n - at : 256;
        for (int i = 0; i < m; ++i) w.v[i] = words[at + i];
        hipLaunchKernelGGL(moe::write_words_kernel, dim3(1), dim3(256), 0, moe::as_stream(stream), static_cast<uint64_t*>(dst) + at, w, m);
        MOE_HIP_CHECK(hipGetLastError());
    }
    return MOE_OK;
}
