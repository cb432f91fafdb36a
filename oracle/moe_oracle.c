/*
 * moe_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A scalar CPU restatement of the MoE-layer arithmetic of EfficientMoE/MoE-Gen,
 * used only as the checker in tests/, in __graft_entry__.smoke() and in the
 * cpu_baseline leg of bench.py.  Nothing under moe_gen_amd/ may call it.
 *
 * Each function cites the reference text it follows (paths relative to the
 * reference checkout).  Where the reference leaves behaviour to the library
 * (slot order of topk(sorted=False), tie order of a non-stable argsort, the
 * summation order of a float reduction) this file fixes ONE legal behaviour,
 * the "canonical" one:
 *   - logits: fp32, acc = fma(x[k], w[k], acc) for k = 0 .. h-1, acc0 = +0
 *     (products of two bf16 values are exact in fp32, so fused and unfused
 *     multiply-add agree; only the order matters);
 *   - reductions over experts: 64 strided partial sums (lane = e mod 64,
 *     ascending e within a lane) folded by a xor butterfly 32,16,8,4,2,1;
 *   - top-k: descending value, equal values -> lower index first; the slot
 *     order of the output is that selection order;
 *   - permutation: stable counting sort of the flat (token*k + slot) list by
 *     expert id.
 *
 * Parity status of every function here: pinned (see tests/test_oracle_*.py:
 * closed forms, brute force, stock torch/numpy library routines).  The Mixtral
 * rules (orc_router with logits_bf16/weights_bf16 and combine mode 2) follow
 * transformers==4.42.0, modeling_mixtral.py, which is not vendored in the
 * reference tree: they are pinned against the stock-torch restatement of the
 * published algorithm and against the MixtralSparseMoeBlock of the transformers
 * release that is installed (a later one), except for the one rule that is
 * specific to 4.42.0 -- routing weights rounded to bf16 before the product --
 * which is "parity unpinned": it rests on the published source text alone.
 *
 * Build: gcc -O2 -fPIC -shared -ffp-contract=off -fno-fast-math (see Makefile).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* bf16 / fp8 scalar conversions                                       */
/* ------------------------------------------------------------------ */

static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

float orc_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

/* round-to-nearest-even, NaN kept quiet: what torch's .to(bfloat16) does */
uint16_t orc_f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* OCP fp8 e4m3fn (torch.float8_e4m3fn; deepseekv3_initializer.py:832):
 * 1 sign, 4 exponent (bias 7), 3 mantissa; no infinity; S.1111.111 is NaN;
 * largest finite 448; subnormals m/8 * 2^-6. */
float orc_fp8_e4m3fn_to_f32(uint8_t v) {
    int sign = v >> 7, e = (v >> 3) & 15, m = v & 7;
    float r;
    if (e == 15 && m == 7) return bits_f32(0x7fc00000u);
    if (e == 0) r = ldexpf((float)m, -9);          /* m/8 * 2^-6 */
    else        r = ldexpf((float)(8 + m), e - 10); /* (1+m/8) * 2^(e-7) */
    return sign ? -r : r;
}

/* fp32 -> e4m3fn, round-to-nearest-even; anything that rounds beyond 448 (and
 * NaN) becomes the NaN pattern, as torch's conversion does (no saturation). */
uint8_t orc_f32_to_fp8_e4m3fn(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    float a = fabsf(f);
    if (!(a == a)) return sign | 0x7f;
    if (a >= 480.0f) return sign | 0x7f;
    /* quantum: 2^-9 below 2^-6, else 2^(floor(log2 a) - 3) */
    int ex;
    (void)frexpf(a, &ex);            /* a = fr * 2^ex, fr in [0.5,1) */
    int q = (a < ldexpf(1.0f, -6)) ? -9 : (ex - 1 - 3);
    float scaled = ldexpf(a, -q);    /* exact */
    float r = nearbyintf(scaled);    /* RNE under the default rounding mode */
    float val = ldexpf(r, q);
    if (val > 448.0f) return sign | 0x7f;
    if (val == 0.0f) return sign;
    if (val < ldexpf(1.0f, -6)) return sign | (uint8_t)ldexpf(val, 9);
    int e2;
    float fr = frexpf(val, &e2);     /* val = fr * 2^e2 */
    int e = e2 - 1 + 7;
    int m = (int)ldexpf(fr, 4) - 8;  /* fr*16 in [8,16) */
    return sign | (uint8_t)(e << 3) | (uint8_t)m;
}

/* Wrapper.py:109-138 deepseek_v3_dequantization:
 *   W_bf16 = bf16( f32(W_fp8) * scale[i/128, j/128] ), ragged edges trimmed. */
void orc_dequant_block(const uint8_t* q, const float* scale, int rows, int cols,
                       int block, uint16_t* out_bf16) {
    int nbc = (cols + block - 1) / block;
    for (int i = 0; i < rows; ++i)
        for (int j = 0; j < cols; ++j) {
            float v = orc_fp8_e4m3fn_to_f32(q[(size_t)i * cols + j]);
            float s = scale[(size_t)(i / block) * nbc + (j / block)];
            out_bf16[(size_t)i * cols + j] = orc_f32_to_bf16(v * s);
        }
}

/* deepseekv3_initializer.py:191-205 per_block_cast_to_fp8:
 *   amax = clamp(max|x| over the block, 1e-4); q = fp8(x * (448/amax));
 *   scale = amax/448.  x is fp32 here (the generator draws fp32). */
void orc_quant_block(const float* x, int rows, int cols, int block,
                     uint8_t* q, float* scale) {
    int nbr = (rows + block - 1) / block, nbc = (cols + block - 1) / block;
    for (int bi = 0; bi < nbr; ++bi)
        for (int bj = 0; bj < nbc; ++bj) {
            float amax = 0.0f;
            for (int i = bi * block; i < rows && i < (bi + 1) * block; ++i)
                for (int j = bj * block; j < cols && j < (bj + 1) * block; ++j) {
                    float a = fabsf(x[(size_t)i * cols + j]);
                    if (a > amax) amax = a;
                }
            if (amax < 1e-4f) amax = 1e-4f;
            float mul = 448.0f / amax;
            for (int i = bi * block; i < rows && i < (bi + 1) * block; ++i)
                for (int j = bj * block; j < cols && j < (bj + 1) * block; ++j)
                    q[(size_t)i * cols + j] =
                        orc_f32_to_fp8_e4m3fn(x[(size_t)i * cols + j] * mul);
            scale[(size_t)bi * nbc + bj] = amax / 448.0f;
        }
}

/* ------------------------------------------------------------------ */
/* canonical exp / sigmoid                                             */
/* ------------------------------------------------------------------ */

/* exp(x) in fp32: n = rne(x*log2e); r = x - n*ln2 (two-term Cody-Waite);
 * degree-5 polynomial in r times r^2, + r + 1 (cephes expf coefficients);
 * scaled by 2^n in two exact-power-of-two multiplies so that results in the
 * subnormal range round once.  Every multiply-add is an explicit fma. */
float orc_expf(float x) {
    if (!(x == x)) return x;
    if (x < -104.0f) return 0.0f;
    if (x > 88.72283f) return bits_f32(0x7f800000u);
    float t = x * 1.44269504088896341f;
    float n = nearbyintf(t);
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
    y = y * bits_f32((uint32_t)(n1 + 127) << 23);
    y = y * bits_f32((uint32_t)(n2 + 127) << 23);
    return y;
}

/* modeling_deepseek_v3.py:510 logits.sigmoid() */
float orc_sigmoidf(float x) { return 1.0f / (1.0f + orc_expf(-x)); }

/* ------------------------------------------------------------------ */
/* router                                                              */
/* ------------------------------------------------------------------ */

typedef struct {
    int32_t n_tokens, hidden, n_experts, top_k;
    int32_t n_group, topk_group;
    int32_t scoring;        /* 0 softmax, 1 sigmoid */
    int32_t method;         /* 0 greedy, 1 group_limited_greedy (group max),
                               2 noaux_tc (bias, group = sum of top-2) */
    int32_t norm_topk_prob; /* divide by the sum of the selected weights */
    int32_t scale_mode;     /* 0 never, 1 only when not normalised (V2), 2 always (V3) */
    int32_t logits_bf16;    /* round logits to bf16 before scoring (Mixtral bf16 gate) */
    int32_t weights_bf16;   /* round the final weights to bf16 (Mixtral) */
    float norm_eps;         /* 1e-20 (DeepSeek) or 0 (Mixtral) */
    float routed_scaling_factor;
} orc_router_params;

/* 64-lane strided partial sums + xor butterfly */
static float canon_sum(const float* v, int n) {
    float p[64];
    for (int l = 0; l < 64; ++l) {
        float a = 0.0f;
        for (int e = l; e < n; e += 64) a = a + v[e];
        p[l] = a;
    }
    for (int m = 32; m >= 1; m >>= 1) {
        float q[64];
        for (int l = 0; l < 64; ++l) q[l] = p[l] + p[l ^ m];
        memcpy(p, q, sizeof p);
    }
    return p[0];
}

/* Order of every selection: by value, NaN above all numbers (the rank torch.topk gives it) and
 * all NaNs equal.  The reference leaves NaN handling to the library; fixing this rule keeps the
 * indices of a row with a NaN score well defined (inside [0, E), no duplicates) while the NaN
 * itself travels on through the weights into the output, as it does in the reference. */
static int above(float a, float b) { return !(a <= b) && (b == b); }

/* argmax with "equal -> lower index"; entries with taken[e] != 0 are skipped */
static int argmax_skip(const float* v, const uint8_t* taken, int n) {
    int best = -1;
    for (int e = 0; e < n; ++e) {
        if (taken[e]) continue;
        if (best < 0 || above(v[e], v[best])) best = e;
    }
    return best;
}

/* Logits only: F.linear(x.float(), W.float()) (modeling_deepseek_v3.py:504-508,
 * modeling_deepseek_v2.py:487-492) in the canonical order. */
void orc_logits(const uint16_t* x, const uint16_t* w, int n, int h, int E, float* out) {
    for (int t = 0; t < n; ++t)
        for (int e = 0; e < E; ++e) {
            const uint16_t* xr = x + (size_t)t * h;
            const uint16_t* wr = w + (size_t)e * h;
            float acc = 0.0f;
            for (int k = 0; k < h; ++k)
                acc = fmaf(orc_bf16_to_f32(xr[k]), orc_bf16_to_f32(wr[k]), acc);
            out[(size_t)t * E + e] = acc;
        }
}

/* Selection and weights for one token from its fp32 logits.
 * V3: modeling_deepseek_v3.py:509-561.  V2: modeling_deepseek_v2.py:493-533.
 * Mixtral: MixtralSparseMoeBlock.forward of transformers 4.42.0. */
static int route_one(const float* logit_in, const float* bias, const orc_router_params* p,
                     int32_t* idx, float* wout, float* logits_out, float* scores_out) {
    const int E = p->n_experts, k = p->top_k;
    float L[1024], s[1024], c[1024], tmp[1024];
    uint8_t taken[1024];
    if (E > 1024 || k > E) return -1;
    for (int e = 0; e < E; ++e) {
        L[e] = logit_in[e];
        if (p->logits_bf16) L[e] = orc_bf16_to_f32(orc_f32_to_bf16(L[e]));
        if (logits_out) logits_out[e] = L[e];
    }
    if (p->scoring == 1) {
        for (int e = 0; e < E; ++e) s[e] = orc_sigmoidf(L[e]);
    } else {
        float m = L[0];
        for (int e = 1; e < E; ++e) if (L[e] > m) m = L[e];
        for (int e = 0; e < E; ++e) s[e] = orc_expf(L[e] - m);
        float sum = canon_sum(s, E);
        for (int e = 0; e < E; ++e) s[e] = s[e] / sum;
    }
    if (scores_out) memcpy(scores_out, s, sizeof(float) * E);
    for (int e = 0; e < E; ++e) c[e] = (p->method == 2 && bias) ? s[e] + bias[e] : s[e];

    if (p->method == 0) {
        memcpy(tmp, c, sizeof(float) * E);
    } else {
        const int G = p->n_group, Kg = p->topk_group;
        if (G <= 0 || E % G || Kg > G || G > 64) return -2;
        const int per = E / G;
        float gs[64];
        uint8_t gtaken[64], keep[64];
        for (int g = 0; g < G; ++g) {
            const float* cg = c + g * per;
            if (p->method == 1) {                 /* max of the group */
                float m = cg[0];
                for (int i = 1; i < per; ++i) if (above(cg[i], m)) m = cg[i];
                gs[g] = m;
            } else {                              /* sum of the two largest */
                if (per < 2) return -3;
                uint8_t tk[1024];
                memset(tk, 0, per);
                int a = argmax_skip(cg, tk, per); tk[a] = 1;
                int b = argmax_skip(cg, tk, per);
                gs[g] = cg[a] + cg[b];
            }
        }
        memset(gtaken, 0, sizeof gtaken);
        memset(keep, 0, sizeof keep);
        for (int j = 0; j < Kg; ++j) {
            int g = argmax_skip(gs, gtaken, G);
            gtaken[g] = 1; keep[g] = 1;
        }
        /* masked_fill(~mask, 0.0): masked experts compete with the value 0.0 */
        for (int e = 0; e < E; ++e) tmp[e] = keep[e / per] ? c[e] : 0.0f;
    }

    memset(taken, 0, E);
    for (int j = 0; j < k; ++j) {
        int e = argmax_skip(tmp, taken, E);
        taken[e] = 1;
        idx[j] = e;
        /* V3 gathers the unbiased score (:547); V2 and Mixtral keep the
         * selected value itself, which is 0.0 for a masked expert */
        wout[j] = (p->method == 2) ? s[e] : tmp[e];
    }
    if (k > 1 && p->norm_topk_prob) {
        float sum = 0.0f;
        for (int j = 0; j < k; ++j) sum = sum + wout[j];
        float den = sum + p->norm_eps;
        for (int j = 0; j < k; ++j) wout[j] = wout[j] / den;
        if (p->scale_mode == 2)
            for (int j = 0; j < k; ++j) wout[j] = wout[j] * p->routed_scaling_factor;
    } else {
        if (p->scale_mode >= 1)
            for (int j = 0; j < k; ++j) wout[j] = wout[j] * p->routed_scaling_factor;
    }
    if (p->weights_bf16)
        for (int j = 0; j < k; ++j) wout[j] = orc_bf16_to_f32(orc_f32_to_bf16(wout[j]));
    return 0;
}

/* Full router.  logits_out / scores_out may be NULL ([n,E] fp32 otherwise). */
int orc_router(const uint16_t* x, const uint16_t* w, const float* bias,
               const orc_router_params* p, int32_t* idx, float* wout,
               float* logits_out, float* scores_out) {
    const int n = p->n_tokens, h = p->hidden, E = p->n_experts, k = p->top_k;
    float* L = (float*)malloc(sizeof(float) * (size_t)E);
    if (!L) return -9;
    int rc = 0;
    for (int t = 0; t < n && rc == 0; ++t) {
        orc_logits(x + (size_t)t * h, w, 1, h, E, L);
        rc = route_one(L, bias, p, idx + (size_t)t * k, wout + (size_t)t * k,
                       logits_out ? logits_out + (size_t)t * E : NULL,
                       scores_out ? scores_out + (size_t)t * E : NULL);
    }
    free(L);
    return rc;
}

/* Same, from precomputed fp32 logits [n,E] (used for forced-tie fixtures). */
int orc_router_from_logits(const float* logits, const float* bias,
                           const orc_router_params* p, int32_t* idx, float* wout,
                           float* scores_out) {
    const int n = p->n_tokens, E = p->n_experts, k = p->top_k;
    for (int t = 0; t < n; ++t) {
        int rc = route_one(logits + (size_t)t * E, bias, p, idx + (size_t)t * k,
                           wout + (size_t)t * k, NULL,
                           scores_out ? scores_out + (size_t)t * E : NULL);
        if (rc) return rc;
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* dispatch: modeling_deepseek_v3.py:630-634 (== modeling_deepseek_v2.py:672-676) */
/* ------------------------------------------------------------------ */

/* counts[e] = #{flat i : idx[i] == e}; offsets = exclusive prefix sum (E+1);
 * perm[r] = flat index sitting at sorted row r (stable);  pos[i] = r. */
int orc_dispatch(const int32_t* idx, int n, int k, int E, int32_t* counts,
                 int32_t* offsets, int32_t* perm, int32_t* pos) {
    const int64_t nk = (int64_t)n * k;
    memset(counts, 0, sizeof(int32_t) * (size_t)E);
    for (int64_t i = 0; i < nk; ++i) {
        if (idx[i] < 0 || idx[i] >= E) return -1;
        counts[idx[i]]++;
    }
    offsets[0] = 0;
    for (int e = 0; e < E; ++e) offsets[e + 1] = offsets[e] + counts[e];
    int32_t* cur = (int32_t*)malloc(sizeof(int32_t) * (size_t)E);
    if (!cur) return -9;
    memcpy(cur, offsets, sizeof(int32_t) * (size_t)E);
    for (int64_t i = 0; i < nk; ++i) {
        int32_t r = cur[idx[i]]++;
        perm[r] = (int32_t)i;
        pos[i] = r;
    }
    free(cur);
    return 0;
}

/* sorted_tokens = x[idxs // k]  (modeling_deepseek_v3.py:634) */
void orc_gather_rows(const uint16_t* x, const int32_t* perm, int64_t nk, int k, int h,
                     uint16_t* xs) {
    for (int64_t r = 0; r < nk; ++r)
        memcpy(xs + (size_t)r * h, x + (size_t)(perm[r] / k) * h, sizeof(uint16_t) * (size_t)h);
}

/* ------------------------------------------------------------------ */
/* combine                                                             */
/* ------------------------------------------------------------------ */

/* ys: expert outputs in sorted-row order [n*k, h] bf16; pos[t*k+j] = row of
 * slot j of token t; w [n,k] fp32; shared: optional [n,h] bf16.
 * mode 0 (V3, modeling_deepseek_v3.py:702-710): fp32 products, fp32 sum over
 *         slots in slot order, one rounding to bf16.
 * mode 1 (V2, modeling_deepseek_v2.py:744-757): weight rounded to bf16, each
 *         product rounded to bf16, sum with an fp32 accumulator, rounded once.
 * mode 2 (Mixtral 4.42.0): bf16 accumulator updated expert by expert in
 *         ascending expert id: acc = bf16(acc + bf16(y * bf16(w))).
 * then, if shared != NULL: out = bf16(f32(out) + f32(shared))  (:624-625). */
int orc_combine(const uint16_t* ys, const int32_t* pos, const int32_t* idx, const float* w,
                const uint16_t* shared, int n, int k, int h, int mode, uint16_t* out) {
    if (k > 64) return -1;
    for (int t = 0; t < n; ++t) {
        int order[64];
        for (int j = 0; j < k; ++j) order[j] = j;
        if (mode == 2) { /* ascending expert id (insertion sort, ids distinct) */
            for (int a = 1; a < k; ++a) {
                int j = order[a], b = a - 1;
                while (b >= 0 && idx[(size_t)t * k + order[b]] > idx[(size_t)t * k + j]) {
                    order[b + 1] = order[b]; --b;
                }
                order[b + 1] = j;
            }
        }
        for (int c = 0; c < h; ++c) {
            float acc = 0.0f;
            for (int a = 0; a < k; ++a) {
                int j = order[a];
                float y = orc_bf16_to_f32(ys[(size_t)pos[(size_t)t * k + j] * h + c]);
                float wj = w[(size_t)t * k + j];
                if (mode == 0) {
                    acc = acc + y * wj;
                } else {
                    float wb = orc_bf16_to_f32(orc_f32_to_bf16(wj));
                    float pr = orc_bf16_to_f32(orc_f32_to_bf16(y * wb));
                    acc = acc + pr;
                    if (mode == 2) acc = orc_bf16_to_f32(orc_f32_to_bf16(acc));
                }
            }
            uint16_t o = orc_f32_to_bf16(acc);
            if (shared)
                o = orc_f32_to_bf16(orc_bf16_to_f32(o) + orc_bf16_to_f32(shared[(size_t)t * h + c]));
            out[(size_t)t * h + c] = o;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* the step either side of the block                                   */
/* ------------------------------------------------------------------ */

/* post_attention_layernorm: DeepseekV3RMSNorm.forward (modeling_deepseek_v3.py:125-150),
 * DeepseekV2RMSNorm.forward (modeling_deepseek_v2.py:127-134):
 *   xf = f32(x); var = mean(xf^2); y = bf16(xf * rsqrt(var + eps)); out = bf16(w * y)
 * torch leaves the summation order of the mean and the accuracy of rsqrt to the
 * backend; canonical choice here: squares summed in 64 strided partials over
 * 8-element chunks (lane = chunk mod 64, ascending inside a lane), xor butterfly,
 * var = sum / h, rstd = 1 / sqrt(var + eps) with correctly rounded sqrt and divide. */
void orc_rmsnorm(const uint16_t* x, const uint16_t* w, float eps, int n, int h, uint16_t* out) {
    const int chunks = h / 8;
    for (int t = 0; t < n; ++t) {
        const uint16_t* xr = x + (size_t)t * h;
        float p[64];
        for (int l = 0; l < 64; ++l) {
            float a = 0.0f;
            for (int c = l; c < chunks; c += 64)
                for (int i = 0; i < 8; ++i) {
                    float f = orc_bf16_to_f32(xr[c * 8 + i]);
                    a = a + f * f;
                }
            p[l] = a;
        }
        for (int m = 32; m >= 1; m >>= 1) {
            float q[64];
            for (int l = 0; l < 64; ++l) q[l] = p[l] + p[l ^ m];
            memcpy(p, q, sizeof p);
        }
        const float var = p[0] / (float)h;
        const float rstd = 1.0f / sqrtf(var + eps);
        for (int c = 0; c < h; ++c) {
            float y = orc_bf16_to_f32(orc_f32_to_bf16(orc_bf16_to_f32(xr[c]) * rstd));
            out[(size_t)t * h + c] = orc_f32_to_bf16(orc_bf16_to_f32(w[c]) * y);
        }
    }
}

/* hidden_states = residual + hidden_states (modeling_deepseek_v3.py:1365): bf16 + bf16 -> bf16 */
void orc_add_residual(const uint16_t* a, const uint16_t* residual, int64_t n, uint16_t* out) {
    for (int64_t i = 0; i < n; ++i)
        out[i] = orc_f32_to_bf16(orc_bf16_to_f32(a[i]) + orc_bf16_to_f32(residual[i]));
}

/* ------------------------------------------------------------------ */
/* bulk conversions for the numpy side                                 */
/* ------------------------------------------------------------------ */

void orc_f32_to_bf16_n(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(in[i]);
}
void orc_bf16_to_f32_n(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_bf16_to_f32(in[i]);
}
void orc_expf_n(const float* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_expf(in[i]);
}
void orc_sigmoidf_n(const float* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_sigmoidf(in[i]);
}
