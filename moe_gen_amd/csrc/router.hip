// Fused MoE router for gfx950: logits, scores, group-limited top-k, renormalisation
// and routed scaling in one kernel.
//
// Replaces MoEGate.forward of the reference (modeling_deepseek_v3.py:500-561,
// modeling_deepseek_v2.py:483-533) and the routing lines of transformers-4.42.0
// MixtralSparseMoeBlock.forward.
//
// Logits.  logit[t,e] = sum_k x[t,k] * W[e,k] is evaluated in fp32 in ONE fixed
// order -- acc = fma(x[k], W[k], acc) for k = 0..h-1 -- so that the selected
// expert indices are a pure function of the inputs.  The fp32 matrix core gives
// exactly that order at twice the rate of the vector ALU: v_mfma_f32_32x32x1_2b_f32
// performs one rank-1 update D = a * b^T + C per instruction, i.e. a single fused
// multiply-add per output element per k.  Operands are staged through LDS as fp32
// (bf16 -> fp32 is a 16-bit shift, exact).
//
// Selection.  After the K loop the block's logits sit in LDS; each wave then
// routes one token at a time with the 64 lanes strided over the experts
// (lane l holds experts l, l+64, l+128, l+192) and wave-level butterfly
// reductions.  Ties go to the lower expert (group) index and the slot order of
// the output is the selection order (descending score).
#include "common.h"
#include "moe_math.h"

namespace moe {
namespace {

constexpr int KC = 32;           // k elements per LDS stage
constexpr int LDK = KC + 4;      // padded fp32 row stride (144 B): conflict-free b128 reads
constexpr int MAX_EJ = 4;        // experts per lane (E <= 256)

struct ArgMax {
    float v;
    int i;
};

// max by value, equal values -> lower index; all lanes receive the result
__device__ __forceinline__ ArgMax wave_argmax(ArgMax a) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        float ov = __shfl_xor(a.v, m);
        int oi = __shfl_xor(a.i, m);
        bool take = (ov > a.v) || (ov == a.v && oi < a.i);
        a.v = take ? ov : a.v;
        a.i = take ? oi : a.i;
    }
    return a;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m));
    return v;
}

// butterfly 32,16,8,4,2,1: p[l] = p[l] + p[l^m]; fp32 addition commutes, so every
// lane ends with the same value
__device__ __forceinline__ float wave_sum_butterfly(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = v + __shfl_xor(v, m);
    return v;
}

constexpr float kNegInf = -__builtin_inff();
constexpr int kBigIdx = 0x7fffffff;

// Routes one token whose logits are in `row` (LDS, E valid entries).
__device__ void route_token(const float* row, const float* __restrict__ bias,
                            const moe_router_params& p, int32_t* __restrict__ idx_out,
                            float* __restrict__ w_out, float* __restrict__ logits_out) {
    const int lane = threadIdx.x & 63;
    const int E = p.n_experts;
    float L[MAX_EJ], s[MAX_EJ], c[MAX_EJ];
    bool valid[MAX_EJ];
#pragma unroll
    for (int j = 0; j < MAX_EJ; ++j) {
        int e = lane + 64 * j;
        valid[j] = e < E;
        L[j] = valid[j] ? row[e] : 0.0f;
        if (p.logits_bf16) L[j] = round_to_bf16(L[j]);
        if (logits_out && valid[j]) logits_out[e] = L[j];
    }
    if (p.scoring == MOE_SCORE_SIGMOID) {
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) s[j] = valid[j] ? canon_sigmoidf(L[j]) : 0.0f;
    } else {
        float m = kNegInf;
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) m = valid[j] ? fmaxf(m, L[j]) : m;
        m = wave_max(m);
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) {
            s[j] = valid[j] ? canon_expf(L[j] - m) : 0.0f;
            part = part + s[j];  // adding +0 for absent experts changes nothing
        }
        float sum = wave_sum_butterfly(part);
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) s[j] = s[j] / sum;
    }
#pragma unroll
    for (int j = 0; j < MAX_EJ; ++j) {
        c[j] = s[j];
        if (p.method == MOE_TOPK_NOAUX_TC && bias != nullptr && valid[j]) c[j] = s[j] + bias[lane + 64 * j];
    }

    float tmp[MAX_EJ];
    if (p.method == MOE_TOPK_GREEDY) {
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) tmp[j] = c[j];
    } else {
        const int G = p.n_group, per = E / G;
        int grp[MAX_EJ];
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) grp[j] = valid[j] ? (lane + 64 * j) / per : 0;
        float my_gs = kNegInf;  // lane g keeps the score of group g
        for (int g = 0; g < G; ++g) {
            ArgMax a{kNegInf, kBigIdx};
#pragma unroll
            for (int j = 0; j < MAX_EJ; ++j)
                if (valid[j] && grp[j] == g && (c[j] > a.v || a.i == kBigIdx)) a = ArgMax{c[j], lane + 64 * j};
            a = wave_argmax(a);
            float gs = a.v;
            if (p.method == MOE_TOPK_NOAUX_TC) {  // sum of the two largest of the group
                float v2 = kNegInf;
#pragma unroll
                for (int j = 0; j < MAX_EJ; ++j)
                    if (valid[j] && grp[j] == g && (lane + 64 * j) != a.i) v2 = fmaxf(v2, c[j]);
                v2 = wave_max(v2);
                gs = a.v + v2;
            }
            if (lane == g) my_gs = gs;
        }
        uint32_t keep = 0;
        bool gtaken = false;
        for (int r = 0; r < p.topk_group; ++r) {
            ArgMax a = (lane < G && !gtaken) ? ArgMax{my_gs, lane} : ArgMax{kNegInf, kBigIdx};
            a = wave_argmax(a);
            if (lane == a.i) gtaken = true;
            keep |= 1u << a.i;
        }
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j)
            tmp[j] = (valid[j] && ((keep >> grp[j]) & 1u)) ? c[j] : 0.0f;  // masked_fill(~mask, 0.0)
    }

    // top-k by repeated argmax; lane r keeps slot r
    bool taken[MAX_EJ] = {false, false, false, false};
    int my_idx = 0;
    float my_w = 0.0f;
    for (int r = 0; r < p.top_k; ++r) {
        ArgMax a{kNegInf, kBigIdx};
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j)
            if (valid[j] && !taken[j] && (a.i == kBigIdx || tmp[j] > a.v)) a = ArgMax{tmp[j], lane + 64 * j};
        a = wave_argmax(a);
        const int owner = a.i & 63, oj = a.i >> 6;
        float sv = 0.0f;
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) {
            if (lane == owner && oj == j) taken[j] = true;
            if (oj == j) sv = s[j];
        }
        sv = __shfl(sv, owner);
        // V3 gathers the unbiased score; V2 / Mixtral keep the selected value
        float wv = (p.method == MOE_TOPK_NOAUX_TC) ? sv : a.v;
        if (lane == r) {
            my_idx = a.i;
            my_w = wv;
        }
    }
    if (p.top_k > 1 && p.norm_topk_prob) {
        float sum = 0.0f;
        for (int r = 0; r < p.top_k; ++r) sum = sum + __shfl(my_w, r);
        float den = sum + p.norm_eps;
        my_w = my_w / den;
        if (p.scale_mode == MOE_SCALE_ALWAYS) my_w = my_w * p.routed_scaling_factor;
    } else if (p.scale_mode >= MOE_SCALE_IF_NOT_NORM) {
        my_w = my_w * p.routed_scaling_factor;
    }
    if (p.weights_bf16) my_w = round_to_bf16(my_w);
    if (lane < p.top_k) {
        idx_out[lane] = my_idx;
        w_out[lane] = my_w;
    }
}

// NEB: 32-expert MFMA blocks per wave (1 or 2); WE / WT: waves along experts / tokens.
template <int NEB, int WE, int WT>
__global__ __launch_bounds__(64 * WE * WT) void router_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ wg, const float* __restrict__ bias,
    moe_router_params p, int32_t* __restrict__ topk_idx, float* __restrict__ topk_w,
    float* __restrict__ logits_out) {
    constexpr int NT = 64 * WE * WT;  // threads
    constexpr int BT = 64 * WT;       // tokens per block
    constexpr int EP = 32 * NEB * WE; // padded experts per block
    constexpr int XCH = BT * (KC / 8), WCH = EP * (KC / 8);  // 16-byte chunks per stage
    constexpr int XPT = (XCH + NT - 1) / NT, WPT = (WCH + NT - 1) / NT;
    constexpr int TILE_F = (BT + EP) * LDK, LOGIT_F = BT * EP;
    constexpr int LDS_F = TILE_F > LOGIT_F ? TILE_F : LOGIT_F;
    __shared__ __attribute__((aligned(16))) float lds[LDS_F];
    float* Xs = lds;
    float* Ws = lds + BT * LDK;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int we = wave % WE, wt = wave / WE;
    const int n = p.n_tokens, h = p.hidden, E = p.n_experts;
    const int t0 = blockIdx.x * BT;

    u32x4 xr[XPT], wr[WPT];
    auto load_stage = [&](int k0) {
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            int c = tid + i * NT;
            int row = c >> 2, kk = k0 + (c & 3) * 8;
            int t = min(t0 + row, n - 1);
            xr[i] = (c < XCH && kk < h) ? *reinterpret_cast<const u32x4*>(x + (size_t)t * h + kk) : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            int c = tid + i * NT;
            int row = c >> 2, kk = k0 + (c & 3) * 8;
            int e = min(row, E - 1);
            wr[i] = (c < WCH && kk < h) ? *reinterpret_cast<const u32x4*>(wg + (size_t)e * h + kk) : u32x4{0, 0, 0, 0};
        }
    };
    auto store_chunk = [&](float* base, int c, u32x4 v) {
        float* d = base + (c >> 2) * LDK + (c & 3) * 8;
        f32x4 lo, hi;
        lo[0] = __uint_as_float(v[0] << 16); lo[1] = __uint_as_float(v[0] & 0xffff0000u);
        lo[2] = __uint_as_float(v[1] << 16); lo[3] = __uint_as_float(v[1] & 0xffff0000u);
        hi[0] = __uint_as_float(v[2] << 16); hi[1] = __uint_as_float(v[2] & 0xffff0000u);
        hi[2] = __uint_as_float(v[3] << 16); hi[3] = __uint_as_float(v[3] & 0xffff0000u);
        *reinterpret_cast<f32x4*>(d) = lo;
        *reinterpret_cast<f32x4*>(d + 4) = hi;
    };
    auto store_stage = [&]() {
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            int c = tid + i * NT;
            if (c < XCH) store_chunk(Xs, c, xr[i]);
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            int c = tid + i * NT;
            if (c < WCH) store_chunk(Ws, c, wr[i]);
        }
    };

    f32x32 acc0 = {0}, acc1 = {0};
    const float* a_row = Xs + (wt * 64 + lane) * LDK;
    const float* b0_row = Ws + (NEB == 2 ? (we * 64 + lane) : (we * 32 + (lane & 31))) * LDK;
    const float* b1_row = Ws + (we * 64 + (lane ^ 32)) * LDK;  // only read when NEB == 2

    const int nstage = (h + KC - 1) / KC;
    load_stage(0);
    for (int st = 0; st < nstage; ++st) {
        store_stage();
        __syncthreads();
        if (st + 1 < nstage) load_stage((st + 1) * KC);
#pragma unroll
        for (int k4 = 0; k4 < KC / 4; ++k4) {
            f32x4 a = *reinterpret_cast<const f32x4*>(a_row + k4 * 4);
            f32x4 b0 = *reinterpret_cast<const f32x4*>(b0_row + k4 * 4);
            f32x4 b1;
            if (NEB == 2) b1 = *reinterpret_cast<const f32x4*>(b1_row + k4 * 4);
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                acc0 = __builtin_amdgcn_mfma_f32_32x32x1f32(a[kk], b0[kk], acc0, 0, 0, 0);
                if (NEB == 2) acc1 = __builtin_amdgcn_mfma_f32_32x32x1f32(a[kk], b1[kk], acc1, 0, 0, 0);
            }
        }
        __syncthreads();
    }

    // accumulators -> LDS logits[token][expert].  In block b of the 2-block MFMA
    // result, register 16*b+i of lane l is row 8*(i/4) + 4*(l/32) + i%4, column l%32.
    float* lg = lds;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            int tl = wt * 64 + 32 * b + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
            if (NEB == 2) {
                int e0 = we * 64 + 32 * b + (lane & 31);        // acc0: A block b x B0 block b
                int e1 = we * 64 + 32 * (1 - b) + (lane & 31);  // acc1: A block b x B1 block b
                lg[tl * EP + e0] = acc0[16 * b + i];
                lg[tl * EP + e1] = acc1[16 * b + i];
            } else {
                lg[tl * EP + we * 32 + (lane & 31)] = acc0[16 * b + i];
            }
        }
    }
    __syncthreads();

    constexpr int NW = WE * WT;
    for (int tl = wave; tl < BT; tl += NW) {
        int t = t0 + tl;
        if (t >= n) break;
        route_token(lg + tl * EP, bias, p, topk_idx + (size_t)t * p.top_k, topk_w + (size_t)t * p.top_k,
                    logits_out ? logits_out + (size_t)t * E : nullptr);
    }
}

template <int NEB, int WE, int WT>
int launch(const void* x, const void* w, const float* bias, const moe_router_params& p, int32_t* idx,
           float* tw, float* lo, hipStream_t st) {
    constexpr int BT = 64 * WT;
    dim3 grid((p.n_tokens + BT - 1) / BT), block(64 * WE * WT);
    hipLaunchKernelGGL((router_kernel<NEB, WE, WT>), grid, block, 0, st, (const uint16_t*)x, (const uint16_t*)w,
                       bias, p, idx, tw, lo);
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}

}  // namespace
}  // namespace moe

extern "C" int moe_router(const void* x, const void* w_gate, const float* bias, const moe_router_params* params,
                          int32_t* topk_idx, float* topk_w, float* logits_out, void* stream) {
    using namespace moe;
    MOE_REQUIRE(params != nullptr, "moe_router: params is NULL");
    const moe_router_params& p = *params;
    MOE_REQUIRE(p.n_tokens >= 0, "moe_router: n_tokens %d < 0", p.n_tokens);
    if (p.n_tokens == 0) return MOE_OK;
    MOE_REQUIRE(x && w_gate && topk_idx && topk_w, "moe_router: NULL tensor pointer");
    MOE_REQUIRE(p.hidden > 0 && p.hidden % 8 == 0, "moe_router: hidden %d must be a positive multiple of 8", p.hidden);
    MOE_REQUIRE(p.n_experts >= 1 && p.n_experts <= 256, "moe_router: n_experts %d outside [1,256]", p.n_experts);
    MOE_REQUIRE(p.top_k >= 1 && p.top_k <= 16 && p.top_k <= p.n_experts, "moe_router: top_k %d outside [1,min(16,E)]",
                p.top_k);
    MOE_REQUIRE(p.scoring == MOE_SCORE_SOFTMAX || p.scoring == MOE_SCORE_SIGMOID,
                "moe_router: insupportable scoring function %d", p.scoring);
    MOE_REQUIRE(p.method >= MOE_TOPK_GREEDY && p.method <= MOE_TOPK_NOAUX_TC, "moe_router: insupportable TopK method %d",
                p.method);
    MOE_REQUIRE(p.scale_mode >= MOE_SCALE_NEVER && p.scale_mode <= MOE_SCALE_ALWAYS, "moe_router: bad scale_mode %d",
                p.scale_mode);
    if (p.method != MOE_TOPK_GREEDY) {
        MOE_REQUIRE(p.n_group >= 1 && p.n_group <= 32 && p.n_experts % p.n_group == 0,
                    "moe_router: n_group %d must divide n_experts %d and be <= 32", p.n_group, p.n_experts);
        MOE_REQUIRE(p.topk_group >= 1 && p.topk_group <= p.n_group, "moe_router: topk_group %d outside [1,n_group]",
                    p.topk_group);
        MOE_REQUIRE(p.method != MOE_TOPK_NOAUX_TC || p.n_experts / p.n_group >= 2,
                    "moe_router: noaux_tc needs at least 2 experts per group");
    }
    hipStream_t st = as_stream(stream);
    const int E = p.n_experts;
    if (E <= 32) return launch<1, 1, 4>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
    if (E <= 64) return launch<2, 1, 4>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
    if (E <= 128) return launch<2, 2, 2>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
    if (E <= 192) return launch<2, 3, 1>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
    return launch<2, 4, 1>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
}
