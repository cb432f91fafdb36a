/*
 * moe_mi355.h -- C ABI of libmoe_mi355.so: the MoE-layer hot path of MoE-Gen
 * (router -> dispatch -> grouped SwiGLU experts -> weighted combine, plus
 * expert-weight staging) as hand-written HIP kernels for one MI355X (gfx950).
 *
 * Conventions
 *   - every pointer marked "device" is HBM memory owned by the caller; the
 *     library allocates nothing inside the compute entry points;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *     all work is enqueued on it and the call returns without synchronising;
 *   - return value 0 on success, a negative moe_status otherwise; the message
 *     of the last failure on the calling thread is moe_last_error();
 *   - bf16 tensors are raw 16-bit patterns, fp8 tensors are OCP e4m3fn bytes
 *     (torch.float8_e4m3fn), both row-major with the last dimension contiguous.
 *
 * Reference paths are relative to the EfficientMoE/MoE-Gen checkout.
 */
#ifndef MOE_MI355_H
#define MOE_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum moe_status {
    MOE_OK = 0,
    MOE_ERR_INVALID = -1,    /* bad argument / unsupported shape */
    MOE_ERR_WORKSPACE = -2,  /* workspace too small */
    MOE_ERR_HIP = -3,        /* a HIP runtime call failed */
    MOE_ERR_STATE = -4       /* stager used out of protocol */
} moe_status;

/* Message of the most recent failure on this thread ("" if none). */
const char* moe_last_error(void);

/* Library version string. */
const char* moe_version(void);

/* ---------------------------------------------------------------- router */

enum { MOE_SCORE_SOFTMAX = 0, MOE_SCORE_SIGMOID = 1 };
enum { MOE_TOPK_GREEDY = 0, MOE_TOPK_GROUP_LIMITED_GREEDY = 1, MOE_TOPK_NOAUX_TC = 2 };
enum { MOE_SCALE_NEVER = 0, MOE_SCALE_IF_NOT_NORM = 1, MOE_SCALE_ALWAYS = 2 };

typedef struct moe_router_params {
    int32_t n_tokens;        /* n */
    int32_t hidden;          /* h, multiple of 8 */
    int32_t n_experts;       /* E <= 256 */
    int32_t top_k;           /* k <= 16, k <= E */
    int32_t n_group;         /* G (1 for greedy); E % G == 0, G <= 32 */
    int32_t topk_group;      /* groups kept */
    int32_t scoring;         /* MOE_SCORE_* */
    int32_t method;          /* MOE_TOPK_* */
    int32_t norm_topk_prob;  /* renormalise the k weights to sum 1 (only if k > 1) */
    int32_t scale_mode;      /* MOE_SCALE_* : V2 scales only when not normalising
                                (modeling_deepseek_v2.py:529-533), V3 always
                                (modeling_deepseek_v3.py:554-559) */
    int32_t logits_bf16;     /* round logits to bf16 before scoring (Mixtral's bf16 gate) */
    int32_t weights_bf16;    /* round the final weights to bf16 values (Mixtral) */
    float norm_eps;          /* added to the sum before dividing: 1e-20 DeepSeek, 0 Mixtral */
    float routed_scaling_factor;
} moe_router_params;

/*
 * Fused router: replaces MoEGate.forward (modeling_deepseek_v3.py:500-561,
 * modeling_deepseek_v2.py:483-533) and the routing lines of
 * MixtralSparseMoeBlock.forward (transformers 4.42.0).  One kernel computes the
 * fp32 logits x @ W^T, the scores (softmax, or sigmoid + e_score_correction_bias),
 * the group-limited selection, top-k (descending score, ties to the lower expert
 * index), renormalisation and routed scaling.
 *   x          device bf16 [n, h]
 *   w_gate     device bf16 [E, h]
 *   bias       device fp32 [E] (e_score_correction_bias) or NULL
 *   topk_idx   device int32 [n, k]   out
 *   topk_w     device fp32 [n, k]    out
 *   logits_out device fp32 [n, E]    out, may be NULL
 */
int moe_router(const void* x, const void* w_gate, const float* bias,
               const moe_router_params* params, int32_t* topk_idx, float* topk_w,
               float* logits_out, void* stream);

/* -------------------------------------------------------------- dispatch */

/*
 * Replaces the first half of moe_infer (modeling_deepseek_v3.py:630-634,673 ==
 * modeling_deepseek_v2.py:672-676,715): per-expert histogram, exclusive prefix
 * sum and the stable sort of the flat (token*k + slot) list by expert id, then
 * (optionally) the row gather sorted_tokens = x[idxs // k].  No host sync.
 *   topk_idx  device int32 [n, k]
 *   counts    device int32 [E]      out  tokens per expert
 *   offsets   device int32 [E+1]    out  exclusive prefix sum of counts
 *   perm      device int32 [n*k]    out  perm[r] = flat index at sorted row r
 *   pos       device int32 [n*k]    out  pos[flat] = sorted row (inverse of perm)
 *   row_map   device int32 [n*k]    out  row_map[r] = perm[r] / k, the token behind sorted row r
 *                                        (what the grouped GEMM's fused gather reads); may be NULL
 *   x         device bf16 [n, h]         may be NULL together with xs
 *   xs        device bf16 [n*k, h]  out  gathered rows, may be NULL
 *   workspace device, at least moe_dispatch_workspace_bytes(n, k, E) bytes
 * An id outside [0, E) is not counted and owns no sorted row; its pos entry is -1, which
 * moe_combine skips (the reference would raise an index error on such an id).
 * Limits: 1 <= E <= 256 (the histogram of a block lives in LDS), n * k < 2^31; MOE_ERR_INVALID otherwise.
 */
size_t moe_dispatch_workspace_bytes(int32_t n_tokens, int32_t top_k, int32_t n_experts);
int moe_dispatch(const int32_t* topk_idx, int32_t n_tokens, int32_t top_k, int32_t n_experts,
                 int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* pos, int32_t* row_map,
                 const void* x, int32_t hidden, void* xs,
                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * moe_dispatch without a workspace and without any allocation.  No counterpart in the reference:
 * it exists for callers that cannot allocate device memory at the call -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid it.  The per-segment counters live in a
 * device array built into the library (MOE_DISPATCH_STATIC_SCRATCH_BYTES on every GPU the
 * library runs on, for the life of the process), which bounds the size of a call:
 *     ceil(n_tokens * top_k / 2048) * n_experts * 4  <=  MOE_DISPATCH_STATIC_SCRATCH_BYTES
 * (e.g. 2 097 152 routed entries with 256 experts, four times the DeepSeek-V3 workload at
 * 65 536 tokens); larger calls fail with MOE_ERR_WORKSPACE and belong to moe_dispatch.  Same
 * kernels, same results as moe_dispatch.  All calls on one GPU share the array: calls that
 * overlap on one GPU (two streams, two threads) race; calls on one stream do not.
 * The first call on a device looks the array's address up (hipGetSymbolAddress): make that
 * call eagerly, once per device, before capturing a graph that contains further calls.
 */
#define MOE_DISPATCH_STATIC_SCRATCH_BYTES (1u << 20)
int moe_dispatch_static(const int32_t* topk_idx, int32_t n_tokens, int32_t top_k, int32_t n_experts,
                        int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* pos, int32_t* row_map,
                        const void* x, int32_t hidden, void* xs, void* stream);

/* ----------------------------------------------------- grouped SwiGLU GEMM */

/*
 * Replaces the expert loop of moe_infer (modeling_deepseek_v3.py:675-691) with
 * Expert_Wrapper.forward (Wrapper.py:470-530) and DeepseekV3MLP.forward
 * (:463-467; V2 :449-453; Mixtral w2(silu(w1 x) * w3 x)) for ALL experts in two
 * launches: for expert e and its rows r in [offsets[e], offsets[e+1])
 *     a[r] = bf16( bf16(silu(bf16(x_r Wg_e^T))) * bf16(x_r Wu_e^T) )
 *     y[r] = bf16( a[r] Wd_e^T )
 * on bf16 MFMA with fp32 accumulation.
 *   x         device bf16: rows of the sorted token matrix [n_rows, h]; or, when
 *             row_map != NULL, the unsorted matrix, row r being x[row_map[r]]
 *   x_rows    rows of x (>= 1).  It bounds the gather: a row_map entry outside [0, x_rows) stands for a
 *             row of zeros (where rows are fetched through a buffer descriptor with 32-bit offsets -- the
 *             persistent kernel, below -- an entry whose byte offset wraps 32 bits reads some row of x
 *             instead), never memory outside x.  Without row_map it only has to cover the rows the
 *             call reads
 *   row_map   device int32 [n_rows] or NULL
 *   w_gate/w_up/w_down   device arrays of E device pointers: Wg_e, Wu_e bf16
 *             [I, h]; Wd_e bf16 [h, I]  (nn.Linear [out, in] layout)
 *   offsets   device int32 [E+1] (as written by moe_dispatch).  Rows are absolute indices into
 *             act / y / row_map, so a call may cover a sub-range [a, b) of a layer's experts by
 *             passing offsets + a, the pointer arrays + a and E = b - a (weights handed out in
 *             waves by a pool smaller than the layer); n_rows must then be at least
 *             offsets[b] - offsets[a], the rows inside the range
 *   act       device bf16 [n_rows, I]  scratch for a
 *   y         device bf16 [n_rows, h]  out
 *   workspace reserved: the kernels find their tiles from offsets[] on the device and need no
 *             scratch; NULL / 0 is accepted (moe_grouped_workspace_bytes reports the reserve)
 *   phases    MOE_PHASE_GATE_UP (writes act), MOE_PHASE_DOWN (reads act, writes y) or
 *             MOE_PHASE_BOTH; the two launches can be issued (and timed) separately
 * Requires h % 64 == 0 and I % 64 == 0, 1 <= E <= 1024.  Two kernels share a call: experts that fit one tile of
 * up to 192 rows run one workgroup per tile, at a tile height chosen per expert on the device in steps of 16 rows
 * (bf16 weights: also experts of 257 to 384 rows, as two such tiles);
 * larger experts run on 256-row tiles of persistent workgroups (with fp8 weights: their full 256-row tiles, and the
 * rows these leave over as one tile of the first kind if they are at most 192).  The persistent workgroups,
 * one per CU, take whole rounds of tiles; a last, partial round is cut into 128-row halves and runs with the first
 * kind when that shortens the two launches (alone: if it is at most half the CUs' worth of tiles).  Below a mean of 128 rows per expert (n_rows / E), with K not a multiple of
 * 128, with more than 512 experts or with 4 GiB or more of gathered x, the one-workgroup-per-tile kernel serves the
 * call alone (larger experts cut into 128-row tiles).  An output row's bits depend on the row and its expert's
 * weights, never on the row's place among its expert's rows, on any expert's count or on the kernel that computes
 * it.  With bf16 weights that holds across calls too.  With fp8 weights a call that the one-workgroup-per-tile kernel
 * serves alone adds a row's products in another order than a call that launches both kernels (other starting stages
 * of its k loops, and another order within a stage for experts of up to 64 rows), and a row's last bit may differ
 * between the two kinds of call.
 */
enum { MOE_PHASE_GATE_UP = 1, MOE_PHASE_DOWN = 2, MOE_PHASE_BOTH = 3 };
size_t moe_grouped_workspace_bytes(int32_t n_rows, int32_t n_experts);
int moe_grouped_swiglu_bf16(const void* x, int32_t x_rows, const int32_t* row_map,
                            const void* const* w_gate, const void* const* w_up,
                            const void* const* w_down, const int32_t* offsets,
                            int32_t n_rows, int32_t n_experts, int32_t hidden, int32_t inter,
                            void* act, void* y, int32_t phases, void* workspace,
                            size_t workspace_bytes, void* stream);

/*
 * W8A16 variant: weights are fp8 e4m3fn with one fp32 scale per 128x128 block;
 * each weight element is dequantised in registers as bf16(f32(q) * scale)
 * (deepseek_v3_dequantization, Wrapper.py:109-138) before it reaches the MFMA.
 *   s_gate/s_up  device arrays of E pointers to fp32 [ceil(I/128), ceil(h/128)]
 *   s_down       device array  of E pointers to fp32 [ceil(h/128), ceil(I/128)]
 * Requires h % 128 == 0 and I % 128 == 0.
 */
int moe_grouped_swiglu_w8a16(const void* x, int32_t x_rows, const int32_t* row_map,
                             const void* const* w_gate, const void* const* w_up,
                             const void* const* w_down,
                             const float* const* s_gate, const float* const* s_up,
                             const float* const* s_down, const int32_t* offsets,
                             int32_t n_rows, int32_t n_experts, int32_t hidden, int32_t inter,
                             void* act, void* y, int32_t phases, void* workspace,
                             size_t workspace_bytes, void* stream);

/*
 * Write n 64-bit words (device pointers of a wave of experts, say) into device memory at dst, from host memory
 * that may be reused as soon as the call returns: the words travel inside kernel arguments, 256 per launch, on
 * `stream`, not through the copy engine.  For the per-expert pointer arrays of the two entry points above when
 * the experts' addresses change from call to call (Expert_Wrapper.get_weights hands out a pool slot per call,
 * Wrapper.py:496-500, deepseekv3_initializer.py:1259-1266): the table needs no pinned staging buffer whose reuse
 * would have to wait for a copy, and it does not queue on the copy engine behind the weight copies that the
 * stager keeps in flight there.  Allocates nothing.
 */
int moe_write_words(void* dst, const uint64_t* words, int32_t n, void* stream);

/*
 * Stand-alone block dequantisation (Wrapper.py:109-138), used by tests and by
 * callers that want a bf16 copy:  out = bf16(f32(q) * scale[i/128, j/128]).
 *   q device fp8 [rows, cols]; scale device fp32 [ceil(rows/128), ceil(cols/128)];
 *   out device bf16 [rows, cols].
 */
int moe_dequant_fp8_block128(const void* q, const float* scale, int32_t rows, int32_t cols,
                             void* out, void* stream);

/* --------------------------------------------------------------- combine */

enum {
    MOE_COMBINE_F32 = 0,       /* V3: fp32 products and sum, one rounding (modeling_deepseek_v3.py:702-710) */
    MOE_COMBINE_BF16_PROD = 1, /* V2: bf16 weight, bf16 products, fp32-accumulated sum (modeling_deepseek_v2.py:744-757) */
    MOE_COMBINE_BF16_SEQ = 2   /* Mixtral: bf16 accumulator, experts in ascending id (index_add_) */
};

/*
 * Replaces the second half of moe_infer (inverse permutation + weighted sum over
 * the k slots) and the shared-expert add (modeling_deepseek_v3.py:624-625):
 *     out[t] = sum_j w[t,j] * y[pos[t*k+j]]   (+ shared[t])
 *   y        device bf16 [n*k, h]   expert outputs in sorted-row order
 *   pos      device int32 [n*k]     a negative entry contributes nothing (no row of y is read for it)
 *   topk_idx device int32 [n, k]    (needed by MOE_COMBINE_BF16_SEQ only; else may be NULL)
 *   topk_w   device fp32 [n, k]
 *   shared   device bf16 [n, h] or NULL
 *   out      device bf16 [n, h]
 */
int moe_combine(const void* y, const int32_t* pos, const int32_t* topk_idx, const float* topk_w,
                const void* shared, int32_t n_tokens, int32_t top_k, int32_t hidden,
                int32_t mode, void* out, void* stream);

/* ------------------------------------------------- the step either side of the block */

/*
 * post_attention_layernorm, the op that produces the block's input
 * (DeepseekV3RMSNorm.forward, modeling_deepseek_v3.py:125-150; V2 :127-134; call site :1363):
 *     out = bf16( weight * bf16( f32(x) * rsqrt(mean(f32(x)^2) + eps) ) )
 * in one kernel.  x, out device bf16 [n, h] (out != x); weight device bf16 [h]; h % 8 == 0.
 */
int moe_rmsnorm(const void* x, const void* weight, float eps, int32_t n_tokens, int32_t hidden,
                void* out, void* stream);

/*
 * moe_router reading its tokens THROUGH post_attention_layernorm (modeling_deepseek_v3.py:1361-1364:
 * hidden_states = self.post_attention_layernorm(hidden_states); self.mlp(hidden_states) -> the gate's
 * F.linear at :504-508): x holds the raw hidden states, each workgroup first computes the rstd of
 * its tokens (moe_rmsnorm's summation order), normalises every chunk on its way to the matrix
 * cores, xn = bf16(weight * bf16(f32(x) * rstd)), and writes the normalised rows once to x_norm
 * for the expert GEMMs.  Results (x_norm, indices, weights, logits) are bit-identical to
 * moe_rmsnorm followed by moe_router (with 32 experts or fewer, and with more than 64 experts and a
 * small batch -- up to 1024 tokens, 2048 above 128 experts --, where the fused form does not pay,
 * the call is those two launches).
 *   x           device bf16 [n, h]  raw hidden states
 *   norm_weight device bf16 [h]
 *   x_norm      device bf16 [n, h]  out (must not alias x)
 * Other arguments as moe_router.
 */
int moe_router_rmsnorm(const void* x, const void* norm_weight, float eps, const void* w_gate,
                       const float* bias, const moe_router_params* params, void* x_norm,
                       int32_t* topk_idx, float* topk_w, float* logits_out, void* stream);

/*
 * moe_combine followed by the decoder layer's residual add
 * (hidden_states = residual + hidden_states, modeling_deepseek_v3.py:1365) in the same pass:
 *     out[t] = bf16( f32(residual[t]) + f32(<moe_combine result>[t]) )
 *   residual device bf16 [n, h]; may be the same buffer as out (in-place update of the
 *   residual stream).  Other arguments as moe_combine.
 */
int moe_combine_residual(const void* y, const int32_t* pos, const int32_t* topk_idx,
                         const float* topk_w, const void* shared, const void* residual,
                         int32_t n_tokens, int32_t top_k, int32_t hidden, int32_t mode,
                         void* out, void* stream);

/* ------------------------------------------------- expert-weight staging */

/*
 * Slot pool + cyclic prefetch of whole expert modules from pinned host memory
 * into HBM slots on a private copy stream.  Replaces, for the weights half,
 * HtoD_Engine::HtoD_Worker (core/HtoD_Engine/HtoD_Engine.cpp:201-268),
 * GPU_Weight_Buffer::{acquireEmptyBuffer, get_weights, releaseBuffer,
 * weights_copy_complete, clear_expert_buffer, resize_buffer, reset_prefill_buffer}
 * (core/GPU_Weight_Buffer/GPU_Weight_Buffer.cpp:103-379) and
 * Weights_Storage::get_module_weights_storage (core/Weights_Storage/Weights_Storage.cpp:80).
 * The reference hands slots over through a host condition variable after a
 * stream synchronise; here hand-off is by events: acquire() makes the caller's
 * compute stream wait for the copy, release() makes the next copy into the slot
 * wait for the compute stream.  The host never blocks.
 *
 * A "module type" is a family of modules sharing one slot shape (the reference's
 * "routed_expert", "shared_expert").  Modules are copied in the cyclic order in
 * which they were added, routing-agnostically, whenever a slot of their type is
 * free -- the policy of the reference's worker loop.  A module that is still resident when
 * its turn comes keeps its place in the cycle and the next non-resident one is copied (the
 * reference would copy it a second time); in the reference's order of use this never happens.
 */
typedef struct moe_stager moe_stager;

enum { MOE_STAGE_CYCLIC = 0,       /* copy every module of the type in registration order (the reference's policy) */
       MOE_STAGE_ON_DEMAND = 1     /* copy only what moe_stage_fetch / moe_stage_acquire name */ };

enum { MOE_STAGE_DEVICE = 0,       /* slots are device memory, copies use hipMemcpyAsync */
       MOE_STAGE_HOST_MEMCPY = 1   /* slots are host memory, copies use memcpy: host-only tests */ };

/* n_types module types; slot_bytes[t] bytes per slot; n_slots[t] slots;
 * slot_mem[t] points to n_slots[t]*slot_bytes[t] bytes owned by the caller. */
int moe_stage_create(moe_stager** out, int32_t n_types, const size_t* slot_bytes,
                     const int32_t* n_slots, void* const* slot_mem, int32_t backend);
/* Register a module: n_tensors source ranges (pinned host pointers) copied back
 * to back into the slot at dst_offsets.  Returns the module id (>= 0). */
int moe_stage_add_module(moe_stager* s, int32_t type, int32_t n_tensors,
                         const void* const* src, const size_t* bytes, const size_t* dst_offsets);
/*
 * Sources in ORDINARY (pageable) host memory.  Weights_Storage::Init maps the reference's POSIX shm weight
 * segment once and views it (core/Weights_Storage/Weights_Storage.cpp:52-78, core/Parameter_Server/posix_shm.cpp:36-92),
 * registering the mapping with the GPU runtime; this library never registers existing memory.  Instead of a second,
 * pinned copy of the whole model, modules registered with moe_stage_add_module_pageable (or
 * moe_stage_add_module_from_segment) travel through a ring of n_chunks pinned chunks of chunk_bytes each, allocated
 * here: a worker thread copies a piece into the next chunk with n_threads host threads and enqueues the
 * hipMemcpyAsync out of it, refilling a chunk once its previous transfer has completed.  Pinned memory held:
 * n_chunks * chunk_bytes.  moe_stage_acquire of such a module blocks the calling host thread until the worker has
 * enqueued the module's transfers (as the reference's get_weights waits for its copy worker); the stream hand-off
 * by events is unchanged.  Call once, before the first copy of a pageable module.
 */
int moe_stage_set_bounce(moe_stager* s, int32_t n_chunks, size_t chunk_bytes, int32_t n_threads);
int moe_stage_add_module_pageable(moe_stager* s, int32_t type, int32_t n_tensors,
                                  const void* const* src, const size_t* bytes, const size_t* dst_offsets);
/* Issue copies for the next modules of every type while free slots exist
 * (one turn of the reference's worker loop per free slot).  Returns the number
 * of modules whose copy was enqueued. */
int moe_stage_pump(moe_stager* s);
/* get_weights: make `stream` wait until module `id` is resident; *slot receives
 * its slot index.  If the module is not yet scheduled, pumps until it is; fails
 * with MOE_ERR_STATE if no slot can become free (all slots held). */
int moe_stage_acquire(moe_stager* s, int32_t id, void* stream, int32_t* slot);
/* free_weights_buffer: the slot may be overwritten once `stream` has finished what it was given before this call.
 * The event that says so is recorded on `stream` by the next call that copies into a released slot, one event for
 * all slots released on that stream since the last such call (so `stream` must still exist then; moe_stage_sync
 * records what is pending, for a caller that is about to destroy a stream); a copy enqueued
 * behind a wait that is still pending costs the copy stream about 0.2 ms, and ten experts released and refilled
 * one by one paid it ten times.  The release that leaves the caller holding no module refills the freed slots at
 * once (the reference's worker refills a slot as soon as it is free, HtoD_Engine.cpp:201-268); while other modules
 * stay held the refill happens at the next moe_stage_acquire / moe_stage_fetch / moe_stage_pump. */
int moe_stage_release(moe_stager* s, int32_t id, void* stream);
/* Copy policy of a module type.  MOE_STAGE_ON_DEMAND turns the cyclic prefetch of that type
 * off: the reference copies every expert of every layer whether or not a token was routed to
 * it (HtoD_Engine.cpp:201-268 walks the whole queue); with the per-expert token counts of
 * moe_dispatch on the host, a caller can stage only the experts that will run. */
int moe_stage_set_policy(moe_stager* s, int32_t type, int32_t policy);
/* Enqueue the copies of modules ids[0..n) that are not resident, in the given order (callers
 * list the busiest experts first so the grouped kernel's first tiles have their weights
 * earliest).  Fails with MOE_ERR_STATE when a module finds no free slot of its type;
 * *n_enqueued (optional) receives the number of copies issued. */
int moe_stage_fetch(moe_stager* s, const int32_t* ids, int32_t n, int32_t* n_enqueued);
/* Whether module `id` currently occupies a slot (copied or copy in flight). */
int moe_stage_resident(moe_stager* s, int32_t id);
/* Low-level form of the phase verbs below: set the number of usable slots of a type within
 * the memory given at creation.  reset != 0 also drops residency of the type and rewinds its
 * cyclic queue; it fails with MOE_ERR_STATE while a module of the type is acquired and not
 * released (its kernels may still be queued). */
int moe_stage_set_active_slots(moe_stager* s, int32_t type, int32_t n_active, int32_t reset);

/*
 * The reference's remaining verbs on the pool (core/MoE_Gen_Binding.cpp:45-65).  Modules are
 * named by tag instead of by string: moe_stage_tag_module(id, L, e) stands for the key
 * "routed_expert_{L}_{e}" (e >= 0) or "shared_expert_{L}" (e == -1) of Wrapper.py:457-468.
 */
/* model_config.model_type ("deepseek_v2", "deepseek_v3", anything else), num_hidden_layers and
 * num_local_experts, which clear_expert_buffer's previous-layer rule reads
 * (GPU_Weight_Buffer.cpp:279-300). */
int moe_stage_set_model(moe_stager* s, const char* model_type, int32_t num_hidden_layers,
                        int32_t num_local_experts);
int moe_stage_tag_module(moe_stager* s, int32_t id, int32_t layer_idx, int32_t expert_idx);
/* clear_expert_buffer (GPU_Weight_Buffer::clear_expert_buffer, GPU_Weight_Buffer.cpp:261-308):
 * release the slots of resident routed experts < expert_idx of layer_idx and of every routed
 * expert of the previous layer -- experts that were prefetched and then skipped because no
 * token was routed to them.  "Previous" is layer_idx - 1, except that layers 0-1 (deepseek_v2)
 * or 0-3 (deepseek_v3) take the last layer.  The next copy into a released slot waits for
 * `stream`.  Returns the number of modules released (>= 0) or a negative status. */
int moe_stage_clear_expert_buffer(moe_stager* s, int32_t layer_idx, int32_t expert_idx, void* stream);
/* Slots of a type in the prefill and in the decoding phase
 * (GPU_Buffer_Config.num_prefill_module_buffer / num_decoding_module_buffer,
 * deepseekv3_initializer.py:912-927); 1 <= n_prefill <= n_decoding <= slots given at creation.
 * Takes effect at once for the current phase. */
int moe_stage_set_phase_slots(moe_stager* s, int32_t type, int32_t n_prefill, int32_t n_decoding);
/* set_phase (MoE_Gen::set_phase, core/MoE_Gen.cpp:128-134): "decoding" grows every pool to its
 * decoding size (resize_buffer, GPU_Weight_Buffer.cpp:103-142); "prefill" only records the phase. */
int moe_stage_set_phase(moe_stager* s, const char* phase);
/* reset_prefill_buffer (GPU_Weight_Buffer.cpp:310-379): every pool back to its prefill size with
 * all residency dropped.  Drains the copy stream (host wait); MOE_ERR_STATE while a module is
 * acquired and not released. */
int moe_stage_reset_prefill_buffer(moe_stager* s);
/* reset_weight_copy_queue (HtoD_Engine.cpp:295-311): every cyclic queue back to registration order. */
int moe_stage_reset_weight_copy_queue(moe_stager* s);
/* Counters: copies issued, bytes issued. */
int moe_stage_stats(moe_stager* s, int64_t* n_copies, int64_t* n_bytes);
/* Host-blocking drain of the copy stream (teardown, tests). */
int moe_stage_sync(moe_stager* s);
int moe_stage_destroy(moe_stager* s);

/* ------------------------------------------------- weight arena index (wire format) */

/*
 * Where each module's tensors lie inside one contiguous host arena: the reference's
 * map module_key -> tensor_key -> tensor_meta{offset, tensor_shape, byte_size}
 * (core/Parameter_Server/Parameter_Server.h:48-59) and its length-prefixed serialisation
 * (compute_serialized_size / serialize_map_to_buffer / deserialize_map_from_buffer,
 * core/Parameter_Server/posix_shm.cpp:167-357), byte-compatible on the wire:
 *   u64 n_modules { u64 len, key, u64 n_tensors { u64 len, key, i64 offset, i64 byte_size,
 *   u64 ndim, i64 shape[ndim] } }      (native endian, no padding)
 * Parse errors carry the reference's "Buffer overflow (reading ...)" messages.
 */
typedef struct moe_arena_index moe_arena_index;

int moe_arena_index_create(moe_arena_index** out);
int moe_arena_index_destroy(moe_arena_index* ix);
/* Insert or overwrite one tensor entry; modules and tensors keep insertion order. */
int moe_arena_index_add(moe_arena_index* ix, const char* module_key, const char* tensor_key,
                        int64_t offset, int64_t byte_size, const int64_t* shape, int32_t ndim);
/* deserialize_map_from_buffer (posix_shm.cpp:270-357). */
int moe_arena_index_parse(const void* buf, size_t bytes, moe_arena_index** out);
/* compute_serialized_size (posix_shm.cpp:167-190). */
size_t moe_arena_index_wire_size(const moe_arena_index* ix);
/* serialize_map_to_buffer (posix_shm.cpp:196-268); capacity must be >= the wire size. */
int moe_arena_index_serialize(const moe_arena_index* ix, void* buf, size_t capacity);
int32_t moe_arena_index_n_modules(const moe_arena_index* ix);
/* Key and tensor count of module i; pointers stay valid until the index changes. */
int moe_arena_index_module(const moe_arena_index* ix, int32_t i, const char** key, int32_t* n_tensors);
/* Position of a module key, or -1. */
int moe_arena_index_find(const moe_arena_index* ix, const char* module_key);
int moe_arena_index_tensor(const moe_arena_index* ix, int32_t i, int32_t j, const char** key,
                           int64_t* offset, int64_t* byte_size, int32_t* ndim, const int64_t** shape);
/*
 * Register module `module_key` with a stager, its tensors read from arena_base + offset
 * (Weights_Storage::Init, core/Weights_Storage/Weights_Storage.cpp:52-77; a missing key fails
 * with "Module key not found in storage" as :80-87 does).  tensor_keys[i] is copied to
 * dst_offsets[i] of the slot.  The arena must be pinned host memory that was ALLOCATED pinned;
 * this library never registers existing memory.  Returns the module id (>= 0).
 */
int moe_stage_add_module_from_arena(moe_stager* s, int32_t type, const moe_arena_index* ix,
                                    const char* module_key, const void* arena_base,
                                    size_t arena_bytes, int32_t n_tensors,
                                    const char* const* tensor_keys, const size_t* dst_offsets);
/*
 * The same for a segment in ordinary (pageable) host memory -- the mapped shm weight segment itself, not a pinned
 * copy of it (Weights_Storage.cpp:52-78, posix_shm.cpp:36-92): the module's copies go through the stager's bounce
 * ring (moe_stage_set_bounce), so the host holds the model once.
 */
int moe_stage_add_module_from_segment(moe_stager* s, int32_t type, const moe_arena_index* ix,
                                      const char* module_key, const void* segment_base,
                                      size_t segment_bytes, int32_t n_tensors,
                                      const char* const* tensor_keys, const size_t* dst_offsets);

#ifdef __cplusplus
}
#endif
#endif /* MOE_MI355_H */
