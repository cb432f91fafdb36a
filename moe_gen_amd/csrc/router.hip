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
// (bf16 -> fp32 is a 16-bit shift, exact).  For E <= 16 the 4x4x1 form of the same
// instruction is used (16 blocks of 4 tokens x 4 experts, 8 cycles): no padding to 32
// experts and an 8x shorter dependency chain per k.
//
// Selection.  After the K loop the block's logits sit in LDS; each wave then
// routes one token at a time with the 64 lanes strided over the experts
// (lane l holds experts l, l+64, l+128, l+192) and wave-level butterfly
// reductions.  Ties go to the lower expert (group) index and the slot order of
// the output is the selection order (descending score).
#include <type_traits>

#include "common.h"
#include "moe_math.h"

namespace moe {
namespace {

// Lanes of a wave work in groups of GW (64, or 16 when E <= 16): a group routes one token, its
// lanes strided over the experts (lane g of the group holds experts g, g+GW, ...).  Reductions are
// xor butterflies inside the group, so every lane of the group ends with the same value.
struct ArgMax {
    float v;
    int i;
};

// Value held by the lane's xor-M partner, without going through LDS: cross-row exchanges with
// the gfx950 lane-swap instructions, inside a 16-lane row with DPP.  M = 4 uses a rotation by 4,
// which delivers the xor-4 partner's VALUE whenever the data already agrees between lanes l and
// l^8 -- true in every butterfly below, where the step for 8 precedes the step for 4.
template <int M>
__device__ __forceinline__ int partner_bits(int x) {
    const int lane = threadIdx.x & 63;
    if constexpr (M == 32) {
        auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);   // r[0] = low half twice, r[1] = high half twice
        return (lane & 32) ? (int)r[0] : (int)r[1];
    } else if constexpr (M == 16) {
        auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);   // r[0] = even rows twice, r[1] = odd rows twice
        return (lane & 16) ? (int)r[0] : (int)r[1];
    } else if constexpr (M == 8) {
        return __builtin_amdgcn_update_dpp(x, x, 0x128, 0xf, 0xf, false);   // row_ror:8
    } else if constexpr (M == 4) {
        return __builtin_amdgcn_update_dpp(x, x, 0x124, 0xf, 0xf, false);   // row_ror:4
    } else if constexpr (M == 2) {
        return __builtin_amdgcn_update_dpp(x, x, 0x4E, 0xf, 0xf, false);    // quad_perm [2,3,0,1]
    } else {
        return __builtin_amdgcn_update_dpp(x, x, 0xB1, 0xf, 0xf, false);    // quad_perm [1,0,3,2]
    }
}
template <int M>
__device__ __forceinline__ float partner(float v) {
    return __builtin_bit_cast(float, partner_bits<M>(__builtin_bit_cast(int, v)));
}

template <int GW, int M = GW / 2, typename F>
__device__ __forceinline__ void butterfly(F&& step) {
    if constexpr (M >= 1) {
        step(std::integral_constant<int, M>{});
        butterfly<GW, M / 2>(step);
    }
}

// Order of the selections: by value with NaN above every number (as torch.topk ranks it) and all
// NaNs equal, so a NaN score is selected first, every lane of a group reaches the same decision and
// the indices written stay inside [0, E); the NaN then travels on through the weights.
__device__ __forceinline__ bool above(float a, float b) { return !(a <= b) && (b == b); }

// max by value, equal values -> lower index
template <int GW>
__device__ __forceinline__ ArgMax group_argmax(ArgMax a) {
    butterfly<GW>([&](auto m) {
        const float ov = partner<decltype(m)::value>(a.v);
        const int oi = partner_bits<decltype(m)::value>(a.i);
        const bool take = above(ov, a.v) || (!above(a.v, ov) && oi < a.i);
        a.v = take ? ov : a.v;
        a.i = take ? oi : a.i;
    });
    return a;
}

template <int GW>
__device__ __forceinline__ float group_max(float v) {
    butterfly<GW>([&](auto m) { v = fmaxf(v, partner<decltype(m)::value>(v)); });
    return v;
}

// The canonical sum over experts: 64 strided partials folded by the butterfly 32,16,8,4,2,1
// (p[l] += p[l^m]; fp32 addition commutes).  With E <= 16 (E <= 32) the partials of lanes 16..63
// (32..63) are +0, the leading steps add +0 to non-negative values, and the remaining steps are the
// 16-lane (32-lane) butterfly.
template <int GW>
__device__ __forceinline__ float group_sum_butterfly(float v) {
    butterfly<GW>([&](auto m) { v = v + partner<decltype(m)::value>(v); });
    return v;
}

constexpr float kNegInf = -__builtin_inff();
constexpr int kBigIdx = 0x7fffffff;

// Routes one token per lane group; `row` points at the group's logits (LDS, E valid entries).
// `live` is false for groups without a token (they run the same code on a valid row, store nothing).
template <int GW, int MAX_EJ>
__device__ void route_token(const float* row, const float* __restrict__ bias, const moe_router_params& p,
                            int32_t* __restrict__ idx_out, float* __restrict__ w_out,
                            float* __restrict__ logits_out, bool live) {
    // MAX_EJ: experts per lane, ceil(padded experts / GW)
    const int lane = threadIdx.x & 63, gl = lane & (GW - 1), gbase = lane - gl;
    const int E = p.n_experts;
    float L[MAX_EJ], s[MAX_EJ], c[MAX_EJ];
    bool valid[MAX_EJ];
#pragma unroll
    for (int j = 0; j < MAX_EJ; ++j) {
        int e = gl + GW * j;
        valid[j] = e < E;
        L[j] = valid[j] ? row[e] : 0.0f;
        if (p.logits_bf16) L[j] = round_to_bf16(L[j]);
        if (logits_out && valid[j] && live) logits_out[e] = L[j];
    }
    if (p.scoring == MOE_SCORE_SIGMOID) {
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) s[j] = valid[j] ? canon_sigmoidf(L[j]) : 0.0f;
    } else {
        float m = kNegInf;
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) m = valid[j] ? fmaxf(m, L[j]) : m;
        m = group_max<GW>(m);
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) {
            s[j] = valid[j] ? canon_expf(L[j] - m) : 0.0f;
            part = part + s[j];  // adding +0 for absent experts changes nothing
        }
        float sum = group_sum_butterfly<GW>(part);
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) s[j] = s[j] / sum;
    }
#pragma unroll
    for (int j = 0; j < MAX_EJ; ++j) {
        c[j] = s[j];
        if (p.method == MOE_TOPK_NOAUX_TC && bias != nullptr && valid[j]) c[j] = s[j] + bias[gl + GW * j];
    }

    float tmp[MAX_EJ];
    if (p.method == MOE_TOPK_GREEDY) {
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) tmp[j] = c[j];
    } else {
        const int G = p.n_group, per = E / G;
        int grp[MAX_EJ];
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) grp[j] = valid[j] ? (gl + GW * j) / per : 0;
        float my_gs = kNegInf;  // lane g of the group keeps the score of expert-group g
        for (int g = 0; g < G; ++g) {
            ArgMax a{kNegInf, kBigIdx};
#pragma unroll
            for (int j = 0; j < MAX_EJ; ++j)
                if (valid[j] && grp[j] == g && (above(c[j], a.v) || a.i == kBigIdx)) a = ArgMax{c[j], gl + GW * j};
            a = group_argmax<GW>(a);
            float gs = a.v;
            if (p.method == MOE_TOPK_NOAUX_TC) {  // sum of the two largest of the group
                float v2 = kNegInf;
#pragma unroll
                for (int j = 0; j < MAX_EJ; ++j)
                    if (valid[j] && grp[j] == g && (gl + GW * j) != a.i) v2 = fmaxf(v2, c[j]);
                v2 = group_max<GW>(v2);
                gs = a.v + v2;
            }
            if (gl == g) my_gs = gs;
        }
        uint32_t keep = 0;
        bool gtaken = false;
        for (int r = 0; r < p.topk_group; ++r) {
            ArgMax a = (gl < G && !gtaken) ? ArgMax{my_gs, gl} : ArgMax{kNegInf, kBigIdx};
            a = group_argmax<GW>(a);
            if (gl == a.i) gtaken = true;
            keep |= 1u << a.i;
        }
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j)
            tmp[j] = (valid[j] && ((keep >> grp[j]) & 1u)) ? c[j] : 0.0f;  // masked_fill(~mask, 0.0)
    }

    // top-k by repeated argmax; lane r of the group keeps slot r
    bool taken[MAX_EJ];
#pragma unroll
    for (int j = 0; j < MAX_EJ; ++j) taken[j] = false;
    int my_idx = 0;
    float my_w = 0.0f;
    for (int r = 0; r < p.top_k; ++r) {
        ArgMax a{kNegInf, kBigIdx};
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j)
            if (valid[j] && !taken[j] && (a.i == kBigIdx || above(tmp[j], a.v))) a = ArgMax{tmp[j], gl + GW * j};
        a = group_argmax<GW>(a);
        const int owner = a.i & (GW - 1), oj = a.i / GW;
        float sv = 0.0f;
#pragma unroll
        for (int j = 0; j < MAX_EJ; ++j) {
            if (gl == owner && oj == j) taken[j] = true;
            if (oj == j) sv = s[j];
        }
        sv = __shfl(sv, gbase + owner);
        // V3 gathers the unbiased score; V2 / Mixtral keep the selected value
        float wv = (p.method == MOE_TOPK_NOAUX_TC) ? sv : a.v;
        if (gl == r) {
            my_idx = a.i;
            my_w = wv;
        }
    }
    if (p.top_k > 1 && p.norm_topk_prob) {
        float sum = 0.0f;
        for (int r = 0; r < p.top_k; ++r) sum = sum + __shfl(my_w, gbase + r);
        float den = sum + p.norm_eps;
        my_w = my_w / den;
        if (p.scale_mode == MOE_SCALE_ALWAYS) my_w = my_w * p.routed_scaling_factor;
    } else if (p.scale_mode >= MOE_SCALE_IF_NOT_NORM) {
        my_w = my_w * p.routed_scaling_factor;
    }
    if (p.weights_bf16) my_w = round_to_bf16(my_w);
    if (live && gl < p.top_k) {
        idx_out[gl] = my_idx;
        w_out[gl] = my_w;
    }
}

// Two logit engines share the kernel:
//  SMALL == false: v_mfma_f32_32x32x1_2b_f32.  NEB: 32-expert MFMA blocks per wave (1 or 2);
//                  WE / WT: waves along experts / tokens.
//  SMALL == true : v_mfma_f32_4x4x1_16b_f32: 16 independent 4x4 blocks in 8 cycles, so nothing is
//                  padded to 32 experts and the sequential-in-k dependency chain is 8x shorter.  The
//                  blocks are TG groups of 4 tokens x 16/TG groups of 4 experts: TG = 16 is 64 tokens
//                  x 4 experts per instruction, TG = 4 is 16 x 16 (4 x 64 is router_thin_kernel's); a workgroup owns
//                  4*TG tokens.  NEB instructions per k and wave, WE waves along experts.  Used for
//                  E <= 16 (Mixtral's 8 experts) and for few tokens: a handful of workgroups cannot hide
//                  the 64-cycle latency of the 32x32 chain, and fewer tokens per workgroup spread the
//                  chains over more CUs (it reads 8x the LDS operand bytes per MAC, which is why many
//                  tokens stay on the 32x32 engine).
//  GW: lanes per token in the selection (16, 32 or 64 for E <= 16, <= 32, more).
//  NX (32x32 engine only): groups of 4 more experts that each wave adds with 4x4 instructions on the
//                  same token operand.  Both instructions cost 2 cycles per expert and k, so 160
//                  experts as 4 waves x (32 + 8) load the four SIMDs evenly (80 cycles per k each),
//                  where 5 waves x 32 put two waves on one SIMD (128 cycles, as slow as 256 experts).
// Global loads run two k-stages ahead in registers (two register sets, loop unrolled by two), which
// is what hides the load latency when only a few workgroups exist (small token counts).
// NORM: the rows of x are raw hidden states and the router reads them through the decoder layer's
//                  RMSNorm (post_attention_layernorm, modeling_deepseek_v3.py:125-150, call site :1363):
//                  a pre-pass gives every token of the workgroup its rstd (one wave per row, the
//                  summation order of rmsnorm_kernel), each staged chunk is normalised on its way to LDS,
//                  xn = bf16(w * bf16(x * rstd)), and written once to nrm.out for the expert GEMMs.  The
//                  memory pipe idles while the matrix cores run the logits, so the second read of the
//                  rows and the side output cost little next to a separate norm kernel.
struct NormArgs {
    const uint16_t* w;   // [h] bf16, NULL: no norm
    float eps;
    uint16_t* out;       // [n, h] bf16 normalised rows
};

template <bool SMALL, int TG, int NEB, int WE, int WT, int GW, int NX, bool NORM>
__global__ __launch_bounds__(64 * WE * WT) void router_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ wg, const float* __restrict__ bias,
    moe_router_params p, int32_t* __restrict__ topk_idx, float* __restrict__ topk_w,
    float* __restrict__ logits_out, NormArgs nrm) {
    constexpr int KC = SMALL ? 64 : 32;  // k elements per LDS stage
    constexpr int LDK = KC + 4;          // padded fp32 row stride: conflict-free 16-byte reads
    constexpr int NT = 64 * WE * WT;  // threads
    // SMALL: the 16 blocks of an instruction are TG groups of 4 tokens x EG groups of 4 experts
    constexpr int EG = SMALL ? 16 / TG : 1;
    constexpr int BT = SMALL ? 4 * TG * WT : 64 * WT;          // tokens per block
    constexpr int EPW = SMALL ? 4 * EG * NEB : 32 * NEB + 4 * NX;   // experts per wave
    static_assert(NX == 0 || (!SMALL && NEB == 1), "extra 4-expert groups go with one 32x32 block per wave");
    constexpr int EP = EPW * WE;                                // padded experts per block
    static_assert(!SMALL || (TG * EG == 16 && WT == 1), "4x4 engine: 16 blocks per instruction, one wave along tokens");
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

    __shared__ float s_rstd[NORM ? BT : 1];
    if (NORM) {
        // rstd of the block's tokens, one wave per row: lane l adds the squares of the 8-element chunks
        // l, l+64, ... in ascending order, xor butterfly 32..1, var = sum / h, rstd = 1 / sqrt(var + eps)
        const int chunks = h / 8;
        for (int tb = wave; tb < BT; tb += NT / 64) {
            const u32x4* row = reinterpret_cast<const u32x4*>(x + (size_t)min(t0 + tb, n - 1) * h);
            float a = 0.0f;
            for (int c0 = 0; c0 < chunks; c0 += 512) {   // 8 loads in flight per lane
                u32x4 v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = row[min(c0 + lane + 64 * j, chunks - 1)];
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (c0 + lane + 64 * j < chunks) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float lo = __uint_as_float(v[j][i] << 16), hi = __uint_as_float(v[j][i] & 0xffff0000u);
                            a = a + lo * lo;
                            a = a + hi * hi;
                        }
                    }
            }
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) a = a + __shfl_xor(a, m);
            const float var = a / (float)h;
            if (lane == 0) s_rstd[tb] = 1.0f / __builtin_sqrtf(var + nrm.eps);
        }
        __syncthreads();
    }

    u32x4 xr[2][XPT], wr[2][WPT], gr[2][NORM ? XPT : 1];
    float rstd_r[NORM ? XPT : 1];            // rstd of the token row behind this thread's i-th chunk
    if (NORM) {
#pragma unroll
        for (int i = 0; i < XPT; ++i) rstd_r[i] = s_rstd[min((tid + i * NT) / (KC / 8), BT - 1)];
    }
    // Dword q (two elements) of chunk i of a register set, normalised in place:
    // xn = bf16(w * bf16(x * rstd)), the rounding points of the reference's norm module, 12 vector
    // instructions per pair with the packed hardware conversion.  The fp32 matrix instructions run on
    // the same fp32 lanes as vector arithmetic, so this work is paid in logit time wherever it stands;
    // the pieces are spread over the MFMAs of the stage before the one that stores the set so that at
    // least no wave waits for another's.
    auto norm_piece = [&](int set, int i, int q) {
        const uint32_t xw = xr[set][i][q], gw = gr[set][i][q];
        const float r = rstd_r[i];
        const uint32_t y = pack_bf16(__uint_as_float(xw << 16) * r, __uint_as_float(xw & 0xffff0000u) * r);
        xr[set][i][q] = pack_bf16(__uint_as_float(gw << 16) * __uint_as_float(y << 16),
                                  __uint_as_float(gw & 0xffff0000u) * __uint_as_float(y & 0xffff0000u));
    };
    // Loads are unconditional (addresses clamped; chunks beyond h are zeroed when they are stored
    // to LDS, two stages later): a load under a branch makes the compiler wait for ALL outstanding
    // loads before the first LDS store of a stage, and a select right after the load makes it
    // wait at once; either would undo the two-stage prefetch.
    auto load_stage = [&](int k0, int set) {
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const int c = tid + i * NT;
            const int row = c / (KC / 8), kk = k0 + (c % (KC / 8)) * 8;
            const int t = min(t0 + row, n - 1);
            xr[set][i] = *reinterpret_cast<const u32x4*>(x + (size_t)t * h + (kk < h ? kk : 0));
            if (NORM) gr[set][i] = *reinterpret_cast<const u32x4*>(nrm.w + (kk < h ? kk : 0));
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            const int c = tid + i * NT;
            const int row = c / (KC / 8), kk = k0 + (c % (KC / 8)) * 8;
            const int e = min(row, E - 1);
            wr[set][i] = *reinterpret_cast<const u32x4*>(wg + (size_t)e * h + (kk < h ? kk : 0));
        }
    };
    auto store_chunk = [&](float* base, int c, u32x4 v) {
        float* d = base + (c / (KC / 8)) * LDK + (c % (KC / 8)) * 8;
        f32x4 lo, hi;
        lo[0] = __uint_as_float(v[0] << 16); lo[1] = __uint_as_float(v[0] & 0xffff0000u);
        lo[2] = __uint_as_float(v[1] << 16); lo[3] = __uint_as_float(v[1] & 0xffff0000u);
        hi[0] = __uint_as_float(v[2] << 16); hi[1] = __uint_as_float(v[2] & 0xffff0000u);
        hi[2] = __uint_as_float(v[3] << 16); hi[3] = __uint_as_float(v[3] & 0xffff0000u);
        *reinterpret_cast<f32x4*>(d) = lo;
        *reinterpret_cast<f32x4*>(d + 4) = hi;
    };
    auto store_stage = [&](int set, int k0) {
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            int c = tid + i * NT;
            const int kk = k0 + (c % (KC / 8)) * 8;
            const bool ok = kk < h;
            const u32x4 v = xr[set][i];               // NORM: already normalised (norm_piece)
            if (NORM && c < XCH) {
                const int row = c / (KC / 8);
                if (ok && t0 + row < n) *reinterpret_cast<u32x4*>(nrm.out + (size_t)(t0 + row) * h + kk) = v;
            }
            if (c < XCH) store_chunk(Xs, c, ok ? v : u32x4{0, 0, 0, 0});
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            int c = tid + i * NT;
            const bool ok = k0 + (c % (KC / 8)) * 8 < h;
            if (c < WCH) store_chunk(Ws, c, ok ? wr[set][i] : u32x4{0, 0, 0, 0});
        }
    };

    f32x32 acc0 = {0}, acc1 = {0};          // SMALL == false
    constexpr int N4 = SMALL ? NEB : (NX > 0 ? NX : 1);
    f32x4 acc4[N4];                         // SMALL: group j = experts 4j .. 4j+3; else the NX extra groups
#pragma unroll
    for (int j = 0; j < N4; ++j) acc4[j] = f32x4{0, 0, 0, 0};
    // 4x4 engine: lane l feeds block l/4 = (token group tg, expert group eg), row / column l%4
    const int tg = (lane >> 2) / EG, eg = (lane >> 2) % EG;
    const float* a_row = SMALL ? Xs + (4 * tg + (lane & 3)) * LDK : Xs + (wt * 64 + lane) * LDK;
    const float* b0_row = SMALL ? Ws + (we * EPW + 4 * eg + (lane & 3)) * LDK
                                : Ws + (NEB == 2 ? (we * 64 + lane) : (we * EPW + (lane & 31))) * LDK;
    const float* bx_row = Ws + (we * EPW + 32 + (lane & 3)) * LDK;   // only read when NX > 0
    const float* b1_row = Ws + (we * 64 + (lane ^ 32)) * LDK;  // only read when !SMALL && NEB == 2

    // operands of k..k+3 are read (16 bytes per lane) one step ahead of the MFMAs that use them
    constexpr int NB4 = SMALL ? NEB : 2 + NX;
    auto read_ops = [&](int k4, f32x4& a, f32x4 (&b)[NB4]) {
        a = *reinterpret_cast<const f32x4*>(a_row + k4 * 4);
        if (SMALL) {
#pragma unroll
            for (int j = 0; j < NEB; ++j) b[j] = *reinterpret_cast<const f32x4*>(b0_row + j * 4 * EG * LDK + k4 * 4);
        } else {
            b[0] = *reinterpret_cast<const f32x4*>(b0_row + k4 * 4);
            if (NEB == 2) b[1] = *reinterpret_cast<const f32x4*>(b1_row + k4 * 4);
#pragma unroll
            for (int j = 0; j < NX; ++j) b[2 + j] = *reinterpret_cast<const f32x4*>(bx_row + j * 4 * LDK + k4 * 4);
        }
    };
    constexpr int NPIECE = XPT * 4, PER_K4 = (NPIECE + KC / 4 - 1) / (KC / 4);
    auto multiply_stage = [&](int nset) {    // nset: register set of the NEXT stage, normalised on the way (NORM)
        f32x4 a[2], b[2][NB4];
        read_ops(0, a[0], b[0]);
#pragma unroll
        for (int k4 = 0; k4 < KC / 4; ++k4) {
            if (k4 + 1 < KC / 4) read_ops(k4 + 1, a[(k4 + 1) & 1], b[(k4 + 1) & 1]);
            if (NORM) {
#pragma unroll
                for (int e = k4 * PER_K4; e < (k4 + 1) * PER_K4 && e < NPIECE; ++e) norm_piece(nset, e / 4, e % 4);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                if (SMALL) {
#pragma unroll
                    for (int j = 0; j < NEB; ++j)
                        acc4[j] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[k4 & 1][kk], b[k4 & 1][j][kk], acc4[j], 0, 0, 0);
                } else {
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x1f32(a[k4 & 1][kk], b[k4 & 1][0][kk], acc0, 0, 0, 0);
                    if (NEB == 2) acc1 = __builtin_amdgcn_mfma_f32_32x32x1f32(a[k4 & 1][kk], b[k4 & 1][1][kk], acc1, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < NX; ++j)
                        acc4[j] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[k4 & 1][kk], b[k4 & 1][2 + j][kk], acc4[j], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // No load sits under a branch (the tail re-loads the last stage instead of skipping): with
    // straight-line code the compiler counts outstanding loads exactly and a stage waits only for
    // the register set it stores, not for the set that was requested one stage ago.
    const int nstage = (h + KC - 1) / KC;
    load_stage(0, 0);
    load_stage(min(1, nstage - 1) * KC, 1);
    if (NORM) {                              // the first stage has no stage before it to hide behind
#pragma unroll
        for (int e = 0; e < NPIECE; ++e) norm_piece(0, e / 4, e % 4);
    }
    auto stage = [&](int st, int set) {      // set == st & 1, a literal at both call sites
        store_stage(set, st * KC);
        __syncthreads();
        load_stage(min(st + 2, nstage - 1) * KC, set);
        multiply_stage(set ^ 1);             // (the other set holds stage st + 1, requested one stage ago)
        __syncthreads();
    };
    int st = 0;
    for (; st + 1 < nstage; st += 2) {
        stage(st, 0);
        stage(st + 1, 1);
    }
    if (st < nstage) stage(st, 0);

    // accumulators -> LDS logits[token][expert]
    float* lg = lds;
    if (SMALL) {
        // register i of lane l of instruction j: token 4*tg + i, expert 4*EG*j + 4*eg + l%4 of the wave's
#pragma unroll
        for (int j = 0; j < NEB; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) lg[(4 * tg + i) * EP + we * EPW + 4 * EG * j + 4 * eg + (lane & 3)] = acc4[j][i];
    } else {
        // in block b of the 2-block MFMA result, register 16*b+i of lane l is row
        // 8*(i/4) + 4*(l/32) + i%4, column l%32
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
                    lg[tl * EP + we * EPW + (lane & 31)] = acc0[16 * b + i];
                }
            }
        }
        // the extra groups: register i of lane l of group j is token 4*(l/4) + i, expert 32 + 4*j + l%4 of the wave's
#pragma unroll
        for (int j = 0; j < NX; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) lg[(wt * 64 + 4 * (lane >> 2) + i) * EP + we * EPW + 32 + 4 * j + (lane & 3)] = acc4[j][i];
    }
    __syncthreads();

    // selection, a lane group per token: GW = 16 lanes for E <= 16, 32 for E <= 32, else the whole wave,
    // with ceil(EP / GW) experts per lane
    // (the lane-group width is part of the canonical summation order of the softmax: it follows
    // from the expert count alone, never from the logit engine or its padding)
    constexpr int NW = WE * WT, TPW = 64 / GW;
    constexpr int EJ = (EP + GW - 1) / GW;
    for (int tb = wave * TPW; tb < BT; tb += NW * TPW) {
        if (t0 + tb >= n) break;
        const int tl = tb + (lane / GW);
        const int t = t0 + tl;
        const bool live = t < n;
        const int tr = live ? t : n - 1, tlr = live ? tl : tb;
        route_token<GW, EJ>(lg + tlr * EP, bias, p, topk_idx + (size_t)tr * p.top_k, topk_w + (size_t)tr * p.top_k,
                        logits_out ? logits_out + (size_t)tr * E : nullptr, live);
    }
}

// Third logit engine, for up to 16 experts and few tokens: one lane per (token, expert) pair on the vector
// ALU.  A chain of dependent 4x4 MFMAs advances one k in 14 cycles (measured: registers only) whatever the
// instruction's 256 outputs are used for, 26 with its operand reads, so a launch of a few thousand tokens
// takes h * 26 cycles on a handful of CUs (Mixtral-8x22B, 256 tokens: 72 us).  v_fmac_f32 is the same
// single fused multiply-add per k, the canonical order, at 9 cycles per dependent step (18 with the
// operand reads: a 16-byte LDS read costs the wave about 16 cycles of issue, whatever the read-ahead), and
// 64 pairs per wave spread a small launch over 4 to 8 times as many CUs: 51 us for the same launch.  A
// workgroup is ONE wave: 64 / EBW tokens x EBW (8 or 16, padded) experts; operands go through two LDS
// stages as fp32 (a lane reads 16 bytes of its token's row and of its expert's row per 4 k); with a single
// wave the LDS executes its accesses in program order, so the k loop needs no barrier.  The staging of
// stage st+1 (two stages ahead in registers) is spread between the multiply-adds of stage st.
template <int EBW>
__global__ __launch_bounds__(64) void router_pair_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ wg, const float* __restrict__ bias,
    moe_router_params p, int32_t* __restrict__ topk_idx, float* __restrict__ topk_w, float* __restrict__ logits_out) {
    constexpr int TBW = 64 / EBW;            // tokens per workgroup
    constexpr int KC = 128, LDK = KC + 4;    // k per stage; padded fp32 row stride: conflict-free 16-byte reads
    constexpr int ROWS = TBW + EBW;
    constexpr int CH = ROWS * (KC / 8);      // 16-byte bf16 chunks per stage
    constexpr int CPT = (CH + 63) / 64;
    __shared__ __attribute__((aligned(16))) float st0[ROWS * LDK];
    __shared__ __attribute__((aligned(16))) float st1[ROWS * LDK];
    const int lane = threadIdx.x, tl = lane / EBW, el = lane % EBW;
    const int n = p.n_tokens, h = p.hidden, E = p.n_experts;
    const int t0 = blockIdx.x * TBW;

    // chunk lane + 64 i of a stage: row (lane + 64 i) / 16 (tokens first, then experts), 8 k from (chunk % 16) * 8
    const uint16_t* src[CPT];
    int kc[CPT], dst[CPT];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = lane + 64 * i, row = min(c / (KC / 8), ROWS - 1);
        kc[i] = (c % (KC / 8)) * 8;
        src[i] = row < TBW ? x + (size_t)min(t0 + row, n - 1) * h : wg + (size_t)min(row - TBW, E - 1) * h;
        dst[i] = row * LDK + kc[i];
    }
    u32x4 r[2][CPT];
    // loads are unconditional (clamped addresses, chunks past h are zeroed on their way to LDS): a load under a
    // branch makes the compiler wait for every outstanding load at the next use
    auto load = [&](int set, int i, int k0) {
        const int k = k0 + kc[i];
        r[set][i] = *reinterpret_cast<const u32x4*>(src[i] + (k < h ? k : 0));
    };
    auto piece = [&](int i, int set, float* buf, int k0, int k0_next) {
        const u32x4 v = k0 + kc[i] < h ? r[set][i] : u32x4{0, 0, 0, 0};
        if (lane + 64 * i < CH) {
            f32x4 lo, hi;
            lo[0] = __uint_as_float(v[0] << 16); lo[1] = __uint_as_float(v[0] & 0xffff0000u);
            lo[2] = __uint_as_float(v[1] << 16); lo[3] = __uint_as_float(v[1] & 0xffff0000u);
            hi[0] = __uint_as_float(v[2] << 16); hi[1] = __uint_as_float(v[2] & 0xffff0000u);
            hi[2] = __uint_as_float(v[3] << 16); hi[3] = __uint_as_float(v[3] & 0xffff0000u);
            *reinterpret_cast<f32x4*>(buf + dst[i]) = lo;
            *reinterpret_cast<f32x4*>(buf + dst[i] + 4) = hi;
        }
        load(set, i, k0_next);
    };

    float acc = 0.0f;
    const int a_off = tl * LDK, b_off = (TBW + el) * LDK;
        constexpr int NK4 = KC / 4, AHEAD = 6;    // operand reads run AHEAD steps of 4 k in front of their multiply-adds
    auto multiply_and_stage = [&](const float* rd, float* wr, int set, int k0, int k0_next) {
        f32x4 a[NK4], b[NK4];
#pragma unroll
        for (int k4 = 0; k4 < AHEAD; ++k4) {
            a[k4] = *reinterpret_cast<const f32x4*>(rd + a_off + k4 * 4);
            b[k4] = *reinterpret_cast<const f32x4*>(rd + b_off + k4 * 4);
        }
#pragma unroll
        for (int k4 = 0; k4 < NK4; ++k4) {
            if (k4 + AHEAD < NK4) {
                a[k4 + AHEAD] = *reinterpret_cast<const f32x4*>(rd + a_off + (k4 + AHEAD) * 4);
                b[k4 + AHEAD] = *reinterpret_cast<const f32x4*>(rd + b_off + (k4 + AHEAD) * 4);
            }
#pragma unroll
            for (int i = k4 * CPT / NK4; i < (k4 + 1) * CPT / NK4; ++i) piece(i, set, wr, k0, k0_next);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)   // as volatile asm the chain stays between its operand reads (plain arithmetic
                                             // sinks to the end of the stage, and every operand of the stage is spilled)
                asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc) : "v"(a[k4][kk]), "v"(b[k4][kk]));
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int nstage = (h + KC - 1) / KC;
#pragma unroll
    for (int i = 0; i < CPT; ++i) load(0, i, 0);
#pragma unroll
    for (int i = 0; i < CPT; ++i) load(1, i, min(1, nstage - 1) * KC);
    // register set s holds stage st + 1 while stage st (parity s ^ 1) is multiplied, the other set stage st + 2
#pragma unroll
    for (int i = 0; i < CPT; ++i) piece(i, 0, st0, 0, min(2, nstage - 1) * KC);
    int st = 0;
    for (; st + 1 < nstage; st += 2) {
        multiply_and_stage(st0, st1, 1, (st + 1) * KC, min(st + 3, nstage - 1) * KC);
        multiply_and_stage(st1, st0, 0, (st + 2) * KC, min(st + 4, nstage - 1) * KC);
    }
    if (st < nstage) multiply_and_stage(st0, st1, 1, (st + 1) * KC, (nstage - 1) * KC);

    __syncthreads();                          // (one wave: orders the operand reads before the logits overwrite them)
    float* lg = st0;
    lg[tl * EBW + el] = acc;
    __syncthreads();
    // selection: 16 lanes per token, as in router_kernel for up to 16 experts
#pragma unroll
    for (int tb = 0; tb < TBW; tb += 4) {
        if (t0 + tb >= n) break;
        const int tg = tb + lane / 16, t = t0 + tg;
        const bool live = tg < TBW && t < n;
        const int tr = live ? t : min(t0 + tb, n - 1), tlr = live ? tg : tb;
        route_token<16, 1>(lg + tlr * EBW, bias, p, topk_idx + (size_t)tr * p.top_k, topk_w + (size_t)tr * p.top_k,
                           logits_out ? logits_out + (size_t)tr * E : nullptr, live);
    }
}

// Fourth logit engine, for more than 64 experts and few tokens (a decode or small prefill batch of DeepSeek-V2 /
// V3): the 4 x 64 layout of the 4x4 MFMA (4 tokens per workgroup, a wave per 64 experts, lane l of a wave the
// expert 64 wave + l) without a workgroup-wide stage.  Under router_kernel every workgroup of 4 tokens converts the
// whole gate matrix to fp32 and passes it through LDS between two barriers per 64 k: 64 KiB of LDS stores and 128 KiB
// of reads per stage, more LDS time than the 64 MFMAs of the stage take.  Here a wave works alone:
//  * the 128-byte lines of ITS 64 gate rows reach its own LDS region as bf16 by DMA (8 instructions per 64 k; chunk c
//    of row r in 16-byte slot c ^ g(r), so that the 16 lanes the LDS serves together -- rows 8i .. 8i+7 and
//    32+8i .. 39+8i -- fall on 16 different bank groups); a lane reads the 8 weights of its expert with one
//    ds_read_b128 and widens them to fp32 between the MFMAs (a shift or a mask each);
//  * the token values never touch LDS: the MFMA broadcasts the A operand of one block to all 16, so a register that
//    holds the 4 tokens' values of 16 consecutive k (one 2-byte load per lane) feeds 16 instructions;
//  * one wave's LDS reads execute in order and its DMA is ordered by vmcnt, so the k loop has no barrier.
// Each logit is the same chain of one fused multiply-add per k as in every other engine.  Per k a wave issues one
// MFMA, one conversion and an eighth of a 16-byte LDS read: 11.9 ns (DeepSeek-V3, up to 1024 tokens: 97 ... 106 us
// for h = 7168, from 165 ... 178); 9.7 ns without the conversion and 8.3 ns without the LDS read either, which is
// the MFMA chain itself.
typedef __attribute__((address_space(3))) uint8_t* lds_u8;
__device__ __forceinline__ int thin_slot(int r) { return ((r >> 1) & 3) | (((r >> 5) & 1) << 2); }

// The A operand of block B is broadcast to all 16 blocks of the instruction (cbsz = 4, abid = B), so ONE register holds
// the token values of 16 consecutive k: lanes 4b .. 4b+3 the 4 tokens at k0 + b.  The B operand of lane l is expert l
// of the wave's 64.
template <int B>
__device__ __forceinline__ f32x4 mfma_4_tokens(float a, float b, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, acc, 4, B, 0);
}

// NBUF: weight buffers per wave (3: two stages in flight, one workgroup per CU; 2: one stage in flight and at most
// 256 registers, two workgroups per CU).
template <int WE, int NBUF>
__global__ __launch_bounds__(64 * WE, NBUF == 2 ? 2 : 1) void router_thin_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ wg, const float* __restrict__ bias,
    moe_router_params p, int32_t* __restrict__ topk_idx, float* __restrict__ topk_w, float* __restrict__ logits_out) {
    constexpr int KC = 64, BT = 4, EP = 64 * WE, WBYTES = 64 * 128;
    // one array per weight buffer: a read of one then never waits for the DMA in flight into another
    __shared__ __attribute__((aligned(1024))) uint8_t wb0[WE * WBYTES];           // written by DMA only
    __shared__ __attribute__((aligned(1024))) uint8_t wb1[WE * WBYTES];
    __shared__ __attribute__((aligned(1024))) uint8_t wb2[NBUF == 3 ? WE * WBYTES : 1024];
    __shared__ __attribute__((aligned(16))) float lg[BT * EP];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = p.n_tokens, h = p.hidden, E = p.n_experts;
    const int t0 = blockIdx.x * BT;
    const int nfull = h / KC, rem8 = (h % KC) / 8, nstage = nfull + (rem8 ? 1 : 0);

    // weight DMA: instruction i brings rows 8i .. 8i+7 of the wave's 64, a lane the chunk that belongs in its slot
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void*)wg, 0, E * h * 2, 0x00020000);
    int w_voff[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = 8 * i + (lane >> 3), c = (lane & 7) ^ thin_slot(r);
        w_voff[i] = (min(64 * wave + r, E - 1) * h + c * 8) * 2;
    }
    auto dma_w = [&](uint8_t* buf, int st) {
        uint8_t* dst = buf + wave * WBYTES;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_u8)(dst + i * 1024), 16, w_voff[i], (uint32_t)(st * (KC * 2)), 0, 0);
    };
    // token values straight from memory into the broadcast layout: register g of a stage holds, in lanes
    // 4b .. 4b+3, element 16 g + b of the 4 tokens (one 2-byte load per lane and 16 k), widened when its 16 k come up
    const uint16_t* const xrow = x + (size_t)min(t0 + (lane & 3), n - 1) * h;
    uint32_t xr[2][4];
    auto load_x = [&](int set, int st) {       // (elements past h are never multiplied: any address inside the row will do)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int k = st * KC + 16 * g + (lane >> 2);
            xr[set][g] = xrow[k < h ? k : 0];
        }
    };

    f32x4 acc = {0, 0, 0, 0};                  // register i: token i, expert 64 wave + lane
    int w_roff[8];                             // chunk c of the lane's row inside a buffer
#pragma unroll
    for (int c = 0; c < 8; ++c) w_roff[c] = wave * WBYTES + lane * 128 + ((c ^ thin_slot(lane)) << 4);

    auto wf = [](const u32x4& v, int j) {      // element j of 8 bf16 as fp32
        return __uint_as_float((j & 1) ? (v[j >> 1] & 0xffff0000u) : (v[j >> 1] << 16));
    };
    // Stage st; the register set st & 1 and the buffers are literals at every call site.  The DMA of stage
    // st + NBUF - 1 leaves first, then the wait for the DMA of stage st.  Its count is the DMA instructions issued
    // since -- 8 per stage ahead -- and nothing else: the token loads sit behind the wait in program order, but the
    // compiler may place a register load on either side of it, and every one that is in the window only makes the
    // wait stricter (the oldest operations in the window are token loads of a stage ago, long complete).
    auto stage = [&](int st, int set, const uint8_t* wb, uint8_t* wb_refill, int nch) {
        uint32_t xs[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) xs[g] = xr[set][g];
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the reads of stage st - 1, a stage old, before their buffer is refilled
        dma_w(wb_refill, min(st + NBUF - 1, nstage - 1));
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NBUF - 1) * 8) : "memory");
        load_x(set, min(st + 2, nstage - 1));            // (tokens of stage st + 2 into the set that held stage st)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if (2 * g >= nch) break;
            const u32x4 w0 = *reinterpret_cast<const u32x4*>(wb + w_roff[2 * g]);
            const u32x4 w1 = *reinterpret_cast<const u32x4*>(wb + w_roff[2 * g + 1]);
            const float xa = __uint_as_float(xs[g] << 16);
#define MOE_THIN_K(B) \
    if (2 * g + ((B) >> 3) < nch) acc = mfma_4_tokens<B>(xa, wf((B) < 8 ? w0 : w1, (B) & 7), acc);
            MOE_THIN_K(0) MOE_THIN_K(1) MOE_THIN_K(2) MOE_THIN_K(3) MOE_THIN_K(4) MOE_THIN_K(5) MOE_THIN_K(6) MOE_THIN_K(7)
            MOE_THIN_K(8) MOE_THIN_K(9) MOE_THIN_K(10) MOE_THIN_K(11) MOE_THIN_K(12) MOE_THIN_K(13) MOE_THIN_K(14) MOE_THIN_K(15)
#undef MOE_THIN_K
        }
    };

    int st = 0;
    if constexpr (NBUF == 2) {
        load_x(0, 0);
        load_x(1, min(1, nstage - 1));
        dma_w(wb0, 0);
        for (; st + 2 <= nfull; st += 2) {
            stage(st, 0, wb0, wb1, 8);
            stage(st + 1, 1, wb1, wb0, 8);
        }
        const int left = nfull - st;
        if (left > 0) stage(st, 0, wb0, wb1, 8);
        if (rem8) {
            if (left == 0) stage(st, 0, wb0, wb1, rem8);
            else stage(st + 1, 1, wb1, wb0, rem8);
        }
    } else {
        load_x(0, 0);
        load_x(1, min(1, nstage - 1));
        dma_w(wb0, 0);
        dma_w(wb1, min(1, nstage - 1));
        for (; st + 6 <= nfull; st += 6) {
            stage(st, 0, wb0, wb2, 8);
            stage(st + 1, 1, wb1, wb0, 8);
            stage(st + 2, 0, wb2, wb1, 8);
            stage(st + 3, 1, wb0, wb2, 8);
            stage(st + 4, 0, wb1, wb0, 8);
            stage(st + 5, 1, wb2, wb1, 8);
        }
        // up to 5 whole stages and one of fewer than 64 k are left; stage st + i has the literals of i
        const int left = nfull - st;
        if (left > 0) stage(st, 0, wb0, wb2, 8);
        if (left > 1) stage(st + 1, 1, wb1, wb0, 8);
        if (left > 2) stage(st + 2, 0, wb2, wb1, 8);
        if (left > 3) stage(st + 3, 1, wb0, wb2, 8);
        if (left > 4) stage(st + 4, 0, wb1, wb0, 8);
        if (rem8) {
            if (left == 0) stage(st, 0, wb0, wb2, rem8);
            else if (left == 1) stage(st + 1, 1, wb1, wb0, rem8);
            else if (left == 2) stage(st + 2, 0, wb2, wb1, rem8);
            else if (left == 3) stage(st + 3, 1, wb0, wb2, rem8);
            else if (left == 4) stage(st + 4, 0, wb1, wb0, rem8);
            else stage(st + 5, 1, wb2, wb1, rem8);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // no DMA may land in LDS after the workgroup has gone

#pragma unroll
    for (int i = 0; i < 4; ++i) lg[i * EP + 64 * wave + lane] = acc[i];
    __syncthreads();
    for (int tb = wave; tb < BT; tb += WE) {
        if (t0 + tb >= n) break;
        const int t = t0 + tb;
        route_token<64, WE>(lg + tb * EP, bias, p, topk_idx + (size_t)t * p.top_k, topk_w + (size_t)t * p.top_k,
                            logits_out ? logits_out + (size_t)t * E : nullptr, true);
    }
}

template <int WE, int NBUF>
int launch_thin_as(const void* x, const void* w, const float* bias, const moe_router_params& p, int32_t* idx, float* tw,
                   float* lo, hipStream_t st) {
    hipLaunchKernelGGL((router_thin_kernel<WE, NBUF>), dim3((p.n_tokens + 3) / 4), dim3(64 * WE), 0, st,
                       (const uint16_t*)x, (const uint16_t*)w, bias, p, idx, tw, lo);
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}
// Which calls the engine above serves.  In registers a 4x4x1 MFMA issues every 8.6 cycles, every 15.5 when it
// depends on the one before; in this kernel a second, independent chain per wave (8 tokens per workgroup) still took
// 1.75 times as long as one, and two workgroups per CU take 1.5 times as long as one, so once every CU has two
// workgroups the engines with more tokens per instruction win.  Up to 1024 tokens: one workgroup per CU, three
// buffers.  Up to 2048 tokens and above 128 experts: two workgroups per CU, two buffers.  Measured (us,
// router_kernel -> this; h = 7168 / 5120):
//   256 experts:  64 ... 1024 tokens 165 ... 178 -> 97 ... 106;  2048 tokens 232 -> 171;  3072: 235 against 258
//   160 experts:  1024 tokens 96 -> 78;  2048 tokens 134 -> 118;  3072: 138 against 153
//   128 experts:  1024 tokens 91 -> 77;  2048: 98 against 114
// (a 16-token form on v_mfma_f32_16x16x1_4b_f32, 32 cycles per instruction in registers, ran at 77 per k: 304 us at
// 4096 tokens of 256 experts against 248; with two workgroups per CU 410 against 474 at 8192 tokens and behind again
// from 12288: not kept)
__host__ __device__ constexpr bool thin_serves(int E, int n) { return E > 64 && (n <= 1024 || (n <= 2048 && E > 128)); }

template <int WE>
int launch_thin(const void* x, const void* w, const float* bias, const moe_router_params& p, int32_t* idx, float* tw,
                float* lo, hipStream_t st) {
    if (p.n_tokens <= 1024) return launch_thin_as<WE, 3>(x, w, bias, p, idx, tw, lo, st);
    return launch_thin_as<WE, 2>(x, w, bias, p, idx, tw, lo, st);
}

template <int EBW>
int launch_pairs(const void* x, const void* w, const float* bias, const moe_router_params& p, int32_t* idx, float* tw,
                 float* lo, hipStream_t st) {
    constexpr int TBW = 64 / EBW;
    hipLaunchKernelGGL((router_pair_kernel<EBW>), dim3((p.n_tokens + TBW - 1) / TBW), dim3(64), 0, st, (const uint16_t*)x,
                       (const uint16_t*)w, bias, p, idx, tw, lo);
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}

template <bool SMALL, int TG, int NEB, int WE, int WT, int GW, int NX = 0>
int launch(const void* x, const void* w, const float* bias, const moe_router_params& p, int32_t* idx,
           float* tw, float* lo, const NormArgs& nrm, hipStream_t st) {
    constexpr int BT = SMALL ? 4 * TG * WT : 64 * WT;
    dim3 grid((p.n_tokens + BT - 1) / BT), block(64 * WE * WT);
    if (nrm.w)
        hipLaunchKernelGGL((router_kernel<SMALL, TG, NEB, WE, WT, GW, NX, true>), grid, block, 0, st, (const uint16_t*)x,
                           (const uint16_t*)w, bias, p, idx, tw, lo, nrm);
    else
        hipLaunchKernelGGL((router_kernel<SMALL, TG, NEB, WE, WT, GW, NX, false>), grid, block, 0, st, (const uint16_t*)x,
                           (const uint16_t*)w, bias, p, idx, tw, lo, nrm);
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}

}  // namespace
}  // namespace moe

namespace moe {
namespace {
int route(const void* x, const void* w_gate, const float* bias, const moe_router_params* params, int32_t* topk_idx,
          float* topk_w, float* logits_out, const NormArgs& nrm, void* stream);
}
}  // namespace moe

extern "C" int moe_router(const void* x, const void* w_gate, const float* bias, const moe_router_params* params,
                          int32_t* topk_idx, float* topk_w, float* logits_out, void* stream) {
    return moe::route(x, w_gate, bias, params, topk_idx, topk_w, logits_out, moe::NormArgs{nullptr, 0.0f, nullptr}, stream);
}

extern "C" int moe_router_rmsnorm(const void* x, const void* norm_weight, float eps, const void* w_gate,
                                  const float* bias, const moe_router_params* params, void* x_norm,
                                  int32_t* topk_idx, float* topk_w, float* logits_out, void* stream) {
    using namespace moe;
    if (params != nullptr && params->n_tokens == 0) return MOE_OK;
    MOE_REQUIRE(norm_weight && x_norm, "moe_router_rmsnorm: NULL norm weight or output");
    MOE_REQUIRE(x_norm != x, "moe_router_rmsnorm: x_norm must not alias x (rows are read twice)");
    MOE_REQUIRE(eps >= 0.0f, "moe_router_rmsnorm: eps %g < 0", (double)eps);
    if (params != nullptr && (params->n_experts <= 32 ||
                              thin_serves(params->n_experts, params->n_tokens))) {
        // Few experts: a launch is short chains of small MFMAs on few waves, with nothing to hide the
        // per-workgroup pre-pass behind (Mixtral-8x7B, 16384 tokens: 0.149 ms fused against 0.088 +
        // 0.045 ms).  Few tokens and many experts: the engine whose waves run without a common stage has no
        // place for the pre-pass either.  The norm kernel followed by the plain router gives the same bits.
        int rc = moe_rmsnorm(x, norm_weight, eps, params->n_tokens, params->hidden, x_norm, stream);
        if (rc != MOE_OK) return rc;
        return route(x_norm, w_gate, bias, params, topk_idx, topk_w, logits_out, NormArgs{nullptr, 0.0f, nullptr}, stream);
    }
    return route(x, w_gate, bias, params, topk_idx, topk_w, logits_out,
                 NormArgs{static_cast<const uint16_t*>(norm_weight), eps, static_cast<uint16_t*>(x_norm)}, stream);
}

namespace moe {
namespace {
int route(const void* x, const void* w_gate, const float* bias, const moe_router_params* params, int32_t* topk_idx,
          float* topk_w, float* logits_out, const NormArgs& nrm, void* stream) {
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
    const int E = p.n_experts, n = p.n_tokens;
#define MOE_ROUTE(SMALL, TG, NEB, WE, WT, GW) \
    return launch<SMALL, TG, NEB, WE, WT, GW>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, nrm, st)
    // The 4x4 engine's 16 blocks per instruction are laid out as 64 tokens x 4 experts, 16 x 16 or
    // 4 x 64: the fewer tokens a launch has, the fewer go to a workgroup, so that the sequential-in-k
    // chains run on as many CUs as possible; many tokens take the 32x32 engine (an eighth of the LDS
    // operand bytes per MAC).  The switch points are measured ones (ms, h = 2048 / 5120 / 7168):
    //   64 experts    4096 tokens: 16x16 0.040, 64x4 0.097;  24576: 0.122, 0.148;  32768: 0.157, 0.153;
    //                 131072: 64x4 0.45, 32x32 0.43
    //   8 experts    32768 tokens: 16x16 0.093, 64x4 0.104;  65536: 0.174, 0.144
    //   160 experts   1024 tokens: 16x16 0.131, 64x4 0.335;  8192: 16x16 0.250, 32x32 0.468;  12288: 0.374, 0.479
    //   256 experts   1024 tokens: 16x16 0.231, 64x4 0.583;  8192: 16x16 0.519, 32x32 0.657;  12288: 0.775, 0.683
    //   (4 x 64, the layout for the fewest tokens, is router_thin_kernel's: see thin_serves)
    // up to 16 experts and few tokens: a lane per (token, expert) pair
    // measured (us, h = 4096; pairs / 4x4 engine): 8 experts 256 tokens 35 / 50, 8192: 42 / 53, 16384: 58 / 61,
    // 32768: 122 / 89; 16 experts 4096 tokens: 41 / 50, 8192: 81 / 53
    if (E <= 8 && n <= 8192 && !nrm.w) return launch_pairs<8>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
    if (E <= 16 && n <= 4096 && !nrm.w) return launch_pairs<16>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
    if (thin_serves(E, n) && !nrm.w) {          // 4 or 8 tokens per workgroup, a wave alone per 64 experts
        if (E <= 128) return launch_thin<2>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
        if (E <= 192) return launch_thin<3>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
        return launch_thin<4>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, st);
    }
    if (E <= 64) {
        if (n <= (E <= 32 ? 32768 : 24576)) {   // 16 tokens per workgroup, 16 experts per wave
            if (E <= 16) MOE_ROUTE(true, 4, 1, 1, 1, 16);
            if (E <= 32) MOE_ROUTE(true, 4, 1, 2, 1, 32);
            if (E <= 48) MOE_ROUTE(true, 4, 1, 3, 1, 64);
            MOE_ROUTE(true, 4, 1, 4, 1, 64);
        }
        if (E <= 4) MOE_ROUTE(true, 16, 1, 1, 1, 16);   // 64 tokens per workgroup, 4 .. 16 experts per wave
        if (E <= 8) MOE_ROUTE(true, 16, 2, 1, 1, 16);
        if (E <= 16) MOE_ROUTE(true, 16, 4, 1, 1, 16);
        if (n <= 65536) {
            if (E <= 32) MOE_ROUTE(true, 16, 4, 2, 1, 32);
            if (E <= 48) MOE_ROUTE(true, 16, 4, 3, 1, 64);
            MOE_ROUTE(true, 16, 4, 4, 1, 64);
        }
        if (E <= 32) MOE_ROUTE(false, 16, 1, 1, 4, 32);
        MOE_ROUTE(false, 16, 1, 2, 2, 64);
    }
    if (n <= 8192) {                            // 16 tokens per workgroup, 16 experts per wave
        if (E <= 96) MOE_ROUTE(true, 4, 1, 6, 1, 64);
        if (E <= 128) MOE_ROUTE(true, 4, 1, 8, 1, 64);
        if (E <= 160) MOE_ROUTE(true, 4, 1, 10, 1, 64);
        if (E <= 192) MOE_ROUTE(true, 4, 1, 12, 1, 64);
        MOE_ROUTE(true, 4, 1, 16, 1, 64);
    }
    // many tokens, more than 64 experts: one wave per 32 experts (one MFMA per k and wave, no padding
    // beyond the next multiple of 32) measured 10-25 % faster than half as many waves with two MFMAs each
#define MOE_ROUTE_X(WE, NX) \
    return launch<false, 16, 1, WE, 1, 64, NX>(x, w_gate, bias, p, topk_idx, topk_w, logits_out, nrm, st)
    if (E <= 96) MOE_ROUTE(false, 16, 1, 3, 1, 64);
    if (E <= 128) MOE_ROUTE(false, 16, 1, 4, 1, 64);
    // Between 4 and 8 waves' worth of experts: 4 waves x (32 + 4 NX) keep the four SIMDs evenly loaded,
    // where 5, 6 or 7 waves of 32 put two waves on one SIMD and run as slowly as 8.  Measured, 32768
    // tokens, h = 5120 (ms): 144 experts 0.72 -> 0.56, 160: 0.77 -> 0.67 (131072 tokens: 2.93 -> 2.11),
    // 176: 0.77 -> 0.64, 192: 0.77 -> 0.68, 208: 0.79 -> 0.74; from 209 on the 8 (7) waves are as fast.
    if (E <= 144) MOE_ROUTE_X(4, 1);
    if (E <= 160) MOE_ROUTE_X(4, 2);
    if (E <= 176) MOE_ROUTE_X(4, 3);
    if (E <= 192) MOE_ROUTE_X(4, 4);
    if (E <= 208) MOE_ROUTE_X(4, 5);
    if (E <= 224) MOE_ROUTE(false, 16, 1, 7, 1, 64);
    MOE_ROUTE(false, 16, 1, 8, 1, 64);
#undef MOE_ROUTE_X
#undef MOE_ROUTE
}
}  // namespace
}  // namespace moe
