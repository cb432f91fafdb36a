// Grouped SwiGLU expert GEMMs for gfx950 on bf16 MFMA, with a W8A16 variant that
// dequantises fp8-e4m3fn weights (one fp32 scale per 128x128 block) in registers on the
// way from HBM to LDS.
//
// Replaces the expert loop of moe_infer (modeling_deepseek_v3.py:675-691), the body of
// Expert_Wrapper.forward (Wrapper.py:470-530: fetch, dequantise, run the MLP in chunks,
// synchronise) and DeepseekV3MLP.forward (:463-467) for all experts with two launches:
//   launch 1 (SWIGLU): act = bf16( bf16(silu(bf16(X Wg^T))) * bf16(X Wu^T) )
//   launch 2         : Y   = bf16( act Wd^T )
// Rounding points are those of the reference's bf16 nn.Linear / SiLU / mul modules; the
// dequantisation is deepseek_v3_dequantization (Wrapper.py:109-138) element for element:
// w = bf16(f32(q) * scale[i/128, j/128]).
//
// Work decomposition.  Sorted rows of expert e are [offsets[e], offsets[e+1]).  Each
// expert is cut into M tiles (the last one partial); an M tile times an N tile of the
// weight matrix is one unit of work.  Every workgroup rebuilds the (tiny) M-tile prefix
// over experts in LDS from offsets[], so a launch needs neither a host sync nor a tile table.
// Two kernels, and a call usually launches both (launch_mt): every expert goes by its own count, which both
// kernels read from offsets[]; each builds the prefix over its own share of the tiles.
//  * grouped_gemm_persistent_kernel (experts above one small tile; with fp8 weights the full 256-row
//    tiles of every expert): 256-row tiles, one
//    workgroup per CU, groups of 32 consecutive tiles go round-robin to the XCDs (workgroup
//    ids are dealt to the 8 XCDs one by one by the hardware; the tiles of a group share their
//    A and B panels through that XCD's L2), and a workgroup's k pipeline runs on from one of
//    its tiles into the next.
//  * grouped_gemm_kernel (experts of up to 192 rows, and with fp8 weights what an expert's full 256-row tiles
//    leave over if that is at most 192 rows; work that mostly streams weights): one
//    workgroup per tile, grid = upper bound on the tile count, surplus workgroups exit at once;
//    the tile height (16 ... 192 rows in steps of 16) follows the expert, groups of 4 tiles go round-robin
//    to the XCDs.  Its tiles run through the weight streamers (stream16_tile, stream8x_tile, stream8w_tile, stream8_tile):
//    weights AND token rows reach LDS by DMA, three weight buffers, one barrier per stage.
//
// Workgroup = 8 waves, two per SIMD.  v_mfma_f32_16x16x32_bf16 throughout: on real (non-zero) data this
// chip is power-limited under MFMA load; the 16x16x32 shape moves a third less accumulator data per flop
// than 32x32x16 and sustains ~13 % more (1.95 vs 1.73 PFLOP/s in a registers-only loop with random
// operands), which is worth ~6 % here.  The persistent kernel's waves are 2 along M x 4 along N, 8 x 4 MFMA
// tiles each (128x64 outputs, 128 fp32 accumulators).  K advances 64 at a time through two LDS stages; rows
// are 128 bytes with a 16-byte-chunk XOR swizzle so that both the 16-byte stores and the 16-byte MFMA
// operand reads are bank-conflict free.  Token rows and bf16 weights come into LDS by DMA
// (buffer_load ... lds); fp8 weights of the persistent kernel go through registers, converted on the way,
// two k-stages ahead, every wave interleaving its share of that with its MFMAs, one piece per group of
// MFMAs, between the one barrier per k-stage.  gemm_tile, the register-staged body of the other kernel,
// remains for calls that gather from 4 GiB of rows or more (the DMA paths address them with 32 bits).
//
// The MFMA is issued with the WEIGHT fragment as srcA and the TOKEN fragment as srcB, so
// a lane ends up holding 4 consecutive output columns of one token row per accumulator;
// the epilogue transposes them through LDS into 16-byte-per-lane row-contiguous stores.

#include <type_traits>

#include "common.h"

namespace moe {
namespace {

constexpr int BK = 64;           // k per stage (bf16 elements); 128 bytes per LDS row
constexpr int ROW_B = 128;       // bytes per LDS row
constexpr int BN_ROWS = 256;     // weight rows per workgroup (128 gate + 128 up when SWIGLU)
constexpr int MAX_E = 1024;
constexpr int PAIR_LO = 257, PAIR_HI = 384;   // bf16: rows of an expert that runs as two tiles of the 192-row body

__device__ __forceinline__ float bf16r(float a) { return __uint_as_float(pack_bf16(a, 0.0f) << 16); }

// 16 fp8 bytes -> 16 bf16 (two 16-byte chunks): bf16(f32(q) * s)
__device__ __forceinline__ void dequant16(u32x4 q, float s, u32x4& lo, u32x4& hi) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(q[i], false);
        f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8(q[i], true);
        uint32_t p0 = pack_bf16(a[0] * s, a[1] * s), p1 = pack_bf16(b[0] * s, b[1] * s);
        if (i < 2) { lo[2 * i] = p0; lo[2 * i + 1] = p1; }
        else       { hi[2 * (i - 2)] = p0; hi[2 * (i - 2) + 1] = p1; }
    }
}

struct GemmArgs {
    const uint16_t* a;          // activations, row stride K
    const int32_t* row_map;     // optional: sorted row -> row of a
    size_t a_bytes;             // size of a when rows are gathered through row_map
    int a_rows;                 // rows of a when rows are gathered through row_map
    const void* const* b0;      // per-expert weight matrix [N, K] (gate when SWIGLU, else down)
    const void* const* b1;      // per-expert up matrix [N, K] (SWIGLU only)
    const float* const* s0;     // per-expert block scales of b0 (W8 only)
    const float* const* s1;     // per-expert block scales of b1 (W8, SWIGLU only)
    const int32_t* offsets;     // [E+1]
    uint16_t* c;                // output, row stride N, sorted-row order
    int E, K, N;
    int n_tiles_n;              // ceil(N / (SWIGLU ? 128 : 256))
    int cold_max;               // experts of up to this many rows belong to the one-workgroup-per-tile kernel, the
                                // others to the persistent kernel (0: all to the latter, INT_MAX: all to the former)
    int rem_split;              // 1: the rule applies to what an expert's full 256-row tiles leave over (count % 256)
                                // instead of to its count: the persistent kernel takes the full tiles, and the
                                // last, ragged one only if it holds more than cold_max rows
    int pair_rows;              // 1: experts of PAIR_LO .. PAIR_HI rows also belong to the one-workgroup-per-tile kernel
    int tail_cus;               // > 0: the persistent kernel runs whole rounds of this many tiles (one per CU); what
                                // is left goes to the other kernel as 128-row half tiles if that pays (tail_tiles)
};

// LDS rows are 128 bytes = 8 chunks of 16 bytes; chunk c of row r is stored at chunk c ^ swz(r).
// swz makes any 8 consecutive rows hit 8 different chunks (32 banks x 4 B = one 128-byte row per
// cycle) AND any 16 consecutive rows hit 16 different (row parity, chunk) slots (64 banks =
// two rows per cycle), so 16-byte operand reads by 32 consecutive rows never collide.
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// Stage at which a tile of N tile n_tile starts its walk over k.  Workgroups that run side by side mostly differ in
// their N tile; started at the same stage, their requests in flight would share the low address bits (rows of the weight
// matrices are K elements apart) and crowd the same memory channels: with the start spread over the stages a launch
// that streams weights gains about a tenth (Mixtral-8x22B shapes, 8 experts x 16 ... 120 rows: 6.1 -> 6.8, 5.4 -> 6.1
// TB/s; 128 / 160 / 192 rows next to the persistent kernel: gate/up 0.63 / 0.64 / 0.66 -> 0.55 / 0.58 / 0.62 ms).
// bf16 weights: every path of both kernels uses this rule, so which kernel or tile computes a row does not change the
// order its products are added in (the persistent kernel itself runs within 0.5 % either way).  fp8 weights (a scale
// per 128 k: pairs of stages stay together): only in calls that the one-workgroup-per-tile kernel serves alone; the
// persistent kernel loses 1.6 % of the DeepSeek-V3 step to a rotated walk, so calls that launch it start every tile
// at stage 0, in both kernels.
template <bool W8>
__device__ __forceinline__ int k_rotation(int n_tile, int nk) { return (W8 ? 2 * n_tile : n_tile) % nk; }

// global-address-space views: expert pointers come out of a pointer table in memory, and
// without the address space the compiler must emit flat loads, whose completion is tracked
// by the same counter as the LDS reads of the MFMA operands
typedef const __attribute__((address_space(1))) u32x4* gptr_u32x4;
typedef const __attribute__((address_space(1))) float* gptr_f32;
typedef const __attribute__((address_space(1))) int32_t* gptr_i32;
typedef __attribute__((address_space(3))) uint8_t* lds_u8;
typedef const __attribute__((address_space(4))) float* cptr_f32;   // constant address space: uniform addresses become scalar loads

__device__ __forceinline__ u32x4 gload16(const void* p) { return *(gptr_u32x4)(uintptr_t)p; }
// Weights under the one-workgroup-per-tile kernel are streamed: a tile of them is used by one workgroup (two
// or more for an expert above 256 rows) and never again in the launch, so those loads are non-temporal
// (Mixtral-8x22B, 256 tokens: down projection 0.325 -> 0.302 ms).  In the persistent kernel the panels are
// shared through L2 and stay plain.
template <bool STREAM>
__device__ __forceinline__ u32x4 gload16_w(const void* p) {
    return STREAM ? __builtin_nontemporal_load((gptr_u32x4)(uintptr_t)p) : *(gptr_u32x4)(uintptr_t)p;
}
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ const uint8_t* uni_ptr(const void* p) {
    uint64_t u = (uint64_t)(uintptr_t)p;
    uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u), hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return reinterpret_cast<const uint8_t*>((uintptr_t)(((uint64_t)hi << 32) | lo));
}


// ---- pieces shared by the one-workgroup-per-tile kernel and the persistent kernel ----

// Position of the expert's `local`-th tile.  Inside an expert, tiles are visited in groups of about
// GM consecutive M tiles (the expert's M tiles split as evenly as possible); within a group the M
// tile varies fastest.  The ~32 workgroups an XCD runs at once then cover ~GM M tiles x 32/GM N
// tiles and share those panels through the XCD's L2: an A panel is fetched once per 32/GM N tiles
// and a B panel once per group.  GM = 4 (4 x 8 tiles) balances the two re-fetch factors; measured on
// 64 experts x 2048 rows (7168 -> 2048, fp8) it fetches 7.0 GiB against 8.75 GiB for GM = 8 or 16.
__device__ __forceinline__ void tile_in_expert(int local, int mt_e, int n_tiles_n, int& m_tile, int& n_tile) {
    constexpr int GM = 4;
    const int ng = max(1, (mt_e + GM / 2) / GM);
    const int base = mt_e / ng, extra = mt_e - base * ng;      // `extra` groups hold base+1 tiles
    const int big = (base + 1) * n_tiles_n, cut = extra * big;
    int gm, m0, rem;
    if (local < cut) {
        const int gi = local / big;
        rem = local - gi * big; gm = base + 1; m0 = gi * (base + 1);
    } else {
        const int l2 = local - cut, sz = base * n_tiles_n, gi = l2 / sz;
        rem = l2 - gi * sz; gm = base; m0 = extra * (base + 1) + gi * base;
    }
    n_tile = rem / gm;
    m_tile = m0 + (rem - n_tile * gm);
}

// 8 fp8 weights (two dwords) -> 8 bf16: bf16(f32(q) * s), the reference's dequantisation
__device__ __forceinline__ u32x4 dequant8(uint32_t q0, uint32_t q1, float sc) {
    const f32x2 c0 = __builtin_amdgcn_cvt_pk_f32_fp8(q0, false), c1 = __builtin_amdgcn_cvt_pk_f32_fp8(q0, true);
    const f32x2 c2 = __builtin_amdgcn_cvt_pk_f32_fp8(q1, false), c3 = __builtin_amdgcn_cvt_pk_f32_fp8(q1, true);
    return u32x4{pack_bf16(c0[0] * sc, c0[1] * sc), pack_bf16(c1[0] * sc, c1[1] * sc),
                 pack_bf16(c2[0] * sc, c2[1] * sc), pack_bf16(c3[0] * sc, c3[1] * sc)};
}

// Epilogue values of one lane for one pair of accumulators: 4 consecutive output columns of one row.
// SWIGLU: act = bf16(bf16(silu(bf16(g))) * bf16(u)), the rounding points of the reference's bf16
// Linear / SiLU / mul modules (silu through the hardware exp and reciprocal); else bf16(acc).
template <bool SWIGLU>
__device__ __forceinline__ u32x2 epilogue_pack(const f32x4& a, const f32x4& up) {
    if (SWIGLU) {
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float gv = bf16r(a[i]);
            const float uv = bf16r(up[i]);
            const float sg = bf16r(gv * __builtin_amdgcn_rcpf(1.0f + __expf(-gv)));
            o[i] = sg * uv;
        }
        return u32x2{pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3])};
    }
    return u32x2{pack_bf16(a[0], a[1]), pack_bf16(a[2], a[3])};
}

// Exclusive scan of the experts' M-tile counts, tiles_of(count), by the whole workgroup: s_pref[e] = number of
// M tiles in front of expert e (the caller adds s_pref[E] if it needs it).  Returns the total; the thread that
// handled expert tid in the LAST pass keeps that expert's prefix, tile count and row range in `mine`
// (experts beyond NT take further passes), and per_expert(e, first_row, end_row) runs once per expert.
struct ExpertOfThread { int start, mt, o0, o1; };
template <int NT, typename T, typename F>
__device__ __forceinline__ int mtile_prefix_scan(const GemmArgs& g, int tid, int* s_pref, int* s_wtot,
                                                 ExpertOfThread& mine, T tiles_of, F per_expert) {
    const int lane = tid & 63, wave = tid >> 6;
    int run = 0;
    mine = ExpertOfThread{0, 0, 0, 0};
    for (int e0 = 0; e0 < g.E; e0 += NT) {
        const int e = e0 + tid;
        int mt = 0;
        if (e < g.E) {
            mine.o0 = g.offsets[e];
            mine.o1 = g.offsets[e + 1];
            mt = tiles_of(mine.o1 - mine.o0);
            per_expert(e, mine.o0, mine.o1);
        }
        int inc = mt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            int o = __shfl_up(inc, d);
            if (lane >= d) inc += o;
        }
        if (lane == 63) s_wtot[wave] = inc;
        __syncthreads();
        int pre = run, tot = 0;
#pragma unroll
        for (int w = 0; w < NT / 64; ++w) {
            if (w < wave) pre += s_wtot[w];
            tot += s_wtot[w];
        }
        mine.start = pre + inc - mt;
        mine.mt = mt;
        if (e < g.E) s_pref[e] = mine.start;
        run += tot;
        if (g.E > NT) __syncthreads();   // s_wtot is rewritten by the next pass
    }
    return run;
}

// LDS row offsets of a wave's MFMA operand fragments (v_mfma_f32_16x16x32_bf16): fragment row = base + lane%16,
// bases multiples of 16.  Tokens: the wave's 32*MT rows; weights: TN fragments of 16 rows, for SWIGLU the first
// half from the gate rows (0..127 of the tile) and the second half from the matching up rows (128..255).
template <int MT, int TN, bool SWIGLU>
__device__ __forceinline__ void fragment_rows(int wm, int wn, int frow, uint32_t (&tok_off)[2 * MT], uint32_t (&w_off)[TN]) {
#pragma unroll
    for (int mi = 0; mi < 2 * MT; ++mi) tok_off[mi] = (uint32_t)((wm * 32 * MT + 16 * mi + frow) * ROW_B);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int r = SWIGLU ? ((j < TN / 2 ? 0 : 128) + wn * (8 * TN) + 16 * (j % (TN / 2))) : (wn * (16 * TN) + 16 * j);
        w_off[j] = (uint32_t)((r + frow) * ROW_B);
    }
}

// Epilogue of one wave.  acc[mi][j][i]: token row = 16*mi + lane%16 of the wave's M range; output column
// = 16*j + 4*(lane/16) + i of the wave's N range, i.e. a lane holds 4 consecutive columns (8 bytes) of one row per
// accumulator.  Storing those directly would issue 8-byte writes to 16 different rows per instruction; instead
// the wave transposes its outputs RPW rows at a time through `ep` (its own RPW * row-bytes of idle LDS) and writes
// 16 bytes per lane, whole 64/128-byte row segments per 4/8 lanes.  `out` points at the wave's first row and
// column, rows_here rows of it are valid and cols_here columns (a ragged last N tile).
template <int MT, int TN, bool SWIGLU, int RPW, bool STREAM>
__device__ __forceinline__ void store_wave_outputs(const f32x4 (&acc)[2 * MT][TN], uint8_t* ep, int lane, uint16_t* out,
                                                   int N, int rows_here, int cols_here) {
    constexpr int CW = SWIGLU ? 8 * TN : 16 * TN;    // output columns of a wave
    constexpr int RBW = CW * 2;                      // bytes per output row of a wave
    constexpr int CPR = RBW / 16;                    // 16-byte chunks per row (4 or 8)
    constexpr int KSH = CPR == 8 ? 0 : 1;            // swizzle key = (row >> KSH) & (CPR-1)
    constexpr int RPP = 64 / CPR;                    // rows per read-back instruction
    const int frow = lane & 15, fquad = lane >> 4, rr = lane / CPR, cc = lane % CPR;
#pragma unroll
    for (int pass = 0; pass < 32 * MT / RPW; ++pass) {
#pragma unroll
        for (int ml = 0; ml < RPW / 16; ++ml) {
            const int mi = pass * (RPW / 16) + ml;
            const int r = 16 * ml + frow;
            uint8_t* erow = ep + r * RBW + (fquad & 1) * 8;
            const int key = (r >> KSH) & (CPR - 1);
#pragma unroll
            for (int jj = 0; jj < (SWIGLU ? TN / 2 : TN); ++jj) {
                const u32x2 pk = epilogue_pack<SWIGLU>(acc[mi][jj], acc[mi][SWIGLU ? jj + TN / 2 : jj]);
                *reinterpret_cast<u32x2*>(erow + (((2 * jj + (fquad >> 1)) ^ key) << 4)) = pk;
            }
        }
#pragma unroll
        for (int ps = 0; ps < RPW / RPP; ++ps) {
            const int r = rr + RPP * ps;
            const u32x4 v = *reinterpret_cast<const u32x4*>(ep + r * RBW + ((cc ^ ((r >> KSH) & (CPR - 1))) << 4));
            if (pass * RPW + r < rows_here && cc * 8 < cols_here) {
                u32x4* dst = reinterpret_cast<u32x4*>(out + (size_t)(pass * RPW + r) * N + cc * 8);
                // whole 128-byte lines per 8 lanes can be written non-temporally (the pipeline's next load waits also
                // cover these stores); half lines per wave stay plain stores, so that L2 merges the halves
                if (STREAM) __builtin_nontemporal_store(v, dst); else *dst = v;
            }
        }
    }
}

// One tile of the one-workgroup-per-tile kernel: rows [row0, min(row0 + 64 MT, row_end)) of expert e times N tile n_tile.
// MT: 32-row units per wave along M (tile rows BM = 64*MT, 2 waves along M)
// WN: waves along N; 4 -> 8 waves of up to 128x64 outputs, two per SIMD; every wave interleaves
//     its share of the load / dequantise / LDS-store work with its MFMAs, a piece per MFMA group
// smem0 / smem1: the two LDS stages (two separate arrays: stores into one stage and reads from the other provably
//     do not alias, which lets the scheduler move them past each other)
// STREAM: no other tile reads these weights (the expert has one M tile): non-temporal loads
// One LDS stage of gemm_tile: token rows, weight rows and the start of the region that the epilogue may transpose
// through (the two parts are one array in the bf16 kernel and separate arrays in the fp8 kernel, whose weight
// streamers write them by DMA)
struct Stage {
    uint8_t *a, *b, *ep;
};

template <int MT, int WN, bool SWIGLU, bool W8, bool STREAM>
__device__ __forceinline__ void gemm_tile(const GemmArgs& g, Stage st0, Stage st1, int e, int row0, int row_end,
                                          int n_tile) {
    constexpr int NT = 128 * WN;                // threads
    constexpr int BM = 64 * MT;                 // rows per workgroup
    constexpr int RA = NT / 8;                  // A rows covered by one pass of the workgroup
    constexpr int NA = BM / RA;                 // 16-byte A chunks per thread per stage
    constexpr int RB = NT / 8;                  // B rows per pass of the workgroup (8 lanes per 128-byte row)
    constexpr int NB = BN_ROWS / RB;            // 16-byte global B chunks per thread per stage (fp8: per pair of stages)
    constexpr int NBLK = SWIGLU ? 128 : 256;    // output columns per workgroup
    constexpr int NJ = 8 / WN;                  // 32-row units of the weight tile per wave
    static_assert(MT <= 3 && NA >= 1 && NB == 4, "tile/thread mismatch");

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = (wave >> 1) % WN;
    const int n0 = n_tile * NBLK;
    const int K = g.K, N = g.N;
    const int nk = K / BK;
    // (fp8 weights under tiles below 256 rows are fetched 128 k at a time, see PAIR8 below: k_rotation keeps their
    // pairs of stages together)
    constexpr bool PAIR8 = W8;
    const int rot = (W8 && g.cold_max != 0x7fffffff) ? 0 : k_rotation<W8>(n_tile, nk);
    auto stage_at = [&](int kt) { const int kp = kt + rot; return kp >= nk ? kp - nk : kp; };

    // ---- per-thread load coordinates ----
    const int lrow = tid >> 3, lchunk = tid & 7;          // bf16 tiles: row tid/8 (+RA i), chunk tid%8
    int a_src[NA];
    bool a_ok[NA];                                        // a row_map entry outside x stands for a row of zeros
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        int r = min(row0 + lrow + RA * i, row_end - 1);
        a_src[i] = g.row_map ? ((gptr_i32)(uintptr_t)g.row_map)[r] : r;
        a_ok[i] = !g.row_map || (unsigned)a_src[i] < (unsigned)g.a_rows;
        if (!a_ok[i]) a_src[i] = 0;
    }
    const uint32_t a_lds = (uint32_t)(lrow * ROW_B + ((lchunk ^ swz(lrow)) << 4));

    const uint8_t* bmat0 = uni_ptr(g.b0[e]);
    const uint8_t* bmat1 = SWIGLU ? uni_ptr(g.b1[e]) : bmat0;
    gptr_f32 sc0 = W8 ? (gptr_f32)(uintptr_t)uni_ptr(g.s0[e]) : nullptr;
    gptr_f32 sc1 = (W8 && SWIGLU) ? (gptr_f32)(uintptr_t)uni_ptr(g.s1[e]) : sc0;
    // weight rows: thread (row tid/8 + 64 i of the tile, 16-byte chunk tid%8 of a 128-byte piece of the row: one
    // k-stage of bf16 weights, a pair of k-stages of fp8 weights)
    const int brow = tid >> 3, bcol_b = (tid & 7) << 4;
    int b_n[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        int r = brow + RB * i;                            // row inside the 256-row B tile
        int n = SWIGLU ? (n0 + (r & 127)) : (n0 + r);
        b_n[i] = min(n, N - 1);
    }
    const uint32_t b_lds = (uint32_t)(brow * ROW_B + (((tid & 7) ^ swz(brow)) << 4));   // (bf16 weights)
    // block-scale rows (W8): first / second 128 rows of the B tile
    int srow0 = 0, srow1 = 0;
    const int KB = K >> 7;
    if (W8) {
        if (SWIGLU) { srow0 = (n0 >> 7) * KB; srow1 = srow0; }
        else        { srow0 = (n0 >> 7) * KB; srow1 = min((n0 >> 7) + 1, (N >> 7) - 1) * KB; }
    }

    // PF register sets: global loads run PF tiles ahead of the LDS stores.  One set when the
    // workgroup is compute bound (BM = 256, which has no registers to spare); two for the smaller
    // tiles, which mostly stream weights (decode) and where bytes in flight per CU are what
    // limits the HBM rate.
    constexpr int PF = (MT <= 2) ? 2 : 1;
    u32x4 ra[PF][NA], rb[PF][NB];

    // PAIR8.  A 64-k stage of fp8 weights is 64 bytes of a row, half a cache line: fetched stage by stage, every
    // row costs two half-line requests, and a CU can only keep so many requests in flight whatever their size
    // (DeepSeek-V3 shapes, 8 rows per expert: 3.6 TB/s of weights against 5-6.5 with bf16 weights).  So the
    // weights of TWO stages are requested together, 8 lanes x 16 bytes = one whole line per row: thread (row
    // tid/8 + 64 i, i < 4; 16-byte chunk c = tid%8) gets 16 weights of stage c/4 of the pair.  Lanes c and c^4
    // then swap their second 8 bytes, after which every lane holds 8 weights of either stage (one 16-byte LDS
    // store each, the unit of work of a data item): chunk 2 (c%4) + (c/4 ^ stage) of the stage's LDS row.  Two
    // register sets of pairs; a set is refilled while the second stage of its pair is stored, three
    // iterations before it is needed again.
    const int pq = tid & 3, phb = (tid >> 2) & 1;
    u32x4 rp[2][4];
    float rps[2][2];
    uint32_t p_lds[2];
#pragma unroll
    for (int st = 0; st < 2; ++st) p_lds[st] = (uint32_t)(brow * ROW_B + (((2 * pq + (phb ^ st)) ^ swz(brow)) << 4));
    const int npair = nk >> 1, prot = rot >> 1;
    auto pair_load = [&](int pr_pipe, int ps, int i) {      // chunk i of pair pr_pipe (pipeline order) into set ps
        const bool past = pr_pipe >= npair;                  // nobody reads it: not from the weights
        int pr = min(pr_pipe, npair - 1) + prot;
        pr = pr >= npair ? pr - npair : pr;
        const uint8_t* m = (SWIGLU && i >= 2) ? bmat1 : bmat0;
        rp[ps][i] = gload16_w<STREAM>(past ? (const uint8_t*)g.a : m + (size_t)b_n[i] * K + (size_t)pr * 128 + bcol_b);
        if (i == 1) rps[ps][0] = sc0[srow0 + pr];
        if (i == 3) rps[ps][1] = sc1[srow1 + pr];
    };
    auto pair_swap = [&](int ps, int i) {                    // lanes c and c^4 swap dwords 2, 3
        const u32x4 own = rp[ps][i];
        u32x4 o;
        // first stage of the pair: c < 4 keeps its dwords 0, 1; c >= 4 takes dwords 2, 3 of lane c-4 (row_shr:4, banks 1, 3)
        o[0] = (uint32_t)__builtin_amdgcn_update_dpp((int)own[0], (int)own[2], 0x114, 0xf, 0xa, false);
        o[1] = (uint32_t)__builtin_amdgcn_update_dpp((int)own[1], (int)own[3], 0x114, 0xf, 0xa, false);
        // second stage: c >= 4 keeps its dwords 0, 1; c < 4 takes dwords 2, 3 of lane c+4 (row_shl:4, banks 0, 2)
        o[2] = (uint32_t)__builtin_amdgcn_update_dpp((int)own[0], (int)own[2], 0x104, 0xf, 0x5, false);
        o[3] = (uint32_t)__builtin_amdgcn_update_dpp((int)own[1], (int)own[3], 0x104, 0xf, 0x5, false);
        rp[ps][i] = o;
    };
    auto pair_store = [&](uint8_t* Bs, int ps, int i, int st) {   // the 8 weights of stage st of the pair -> LDS
        const u32x4 o = dequant8(rp[ps][i][2 * st], rp[ps][i][2 * st + 1], rps[ps][i >> 1]);
        *reinterpret_cast<u32x4*>(Bs + p_lds[st] + i * RB * ROW_B) = o;
    };
    auto gload = [&](int kt_pipe, int set) {
        const int kt = stage_at(kt_pipe);
        const size_t kofs = (size_t)kt * BK;
#pragma unroll
        for (int i = 0; i < NA; ++i) ra[set][i] = gload16(g.a + (size_t)a_src[i] * K + kofs + lchunk * 8);
        if (PAIR8) return;
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const uint8_t* m = (SWIGLU && i >= NB / 2) ? bmat1 : bmat0;  // rows >= 128 of the B tile are the up matrix
            rb[set][i] = gload16_w<STREAM>(m + ((size_t)b_n[i] * K + kofs) * 2 + bcol_b);
        }
    };
    auto lds_store = [&](Stage S, int set) {
        uint8_t *As = S.a, *Bs = S.b;
#pragma unroll
        for (int i = 0; i < NA; ++i) *reinterpret_cast<u32x4*>(As + a_lds + i * RA * ROW_B) = a_ok[i] ? ra[set][i] : u32x4{0, 0, 0, 0};
        if (PAIR8) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pair_swap(0, i);
                pair_store(Bs, 0, i, 0);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NB; ++i) *reinterpret_cast<u32x4*>(Bs + b_lds + i * RB * ROW_B) = rb[set][i];
        }
    };

    // ---- MFMA operand coordinates (v_mfma_f32_16x16x32_bf16) ----
    // fragment row = base + lane%16 (bases are multiples of 16); logical chunk = 4*s + lane/16 for
    // the 32-wide k-step s of the stage: lane l supplies k = 8*(l/16) .. +7 of row l%16
    const int frow = lane & 15, fquad = lane >> 4, fkey = swz(frow);
    // The LDS serves a 16-byte read 8 + 8 lanes at a time (lanes 8i.. together with 32+8i..):
    // such a pair of lane groups must read neighbouring chunks of the same rows, which is what the
    // swizzle keeps conflict-free, so lane group q takes chunk 0,2,1,3 of the k-step instead of q
    // (with q the counter SQ_LDS_BANK_CONFLICT reads 22 % of the busy cycles, with this order
    // 0.3 %).  Both operands use the same order, and a dot product does not care in which order
    // k is walked.
    const int fchunk = ((fquad & 1) << 1) | (fquad >> 1);
    constexpr int TM = 2 * MT, TN = 2 * NJ;       // 16-row token tiles / 16-row weight tiles per wave
    uint32_t tok_off[TM], w_off[TN];
    fragment_rows<MT, TN, SWIGLU>(wm, wn, frow, tok_off, w_off);

    f32x4 acc[TM][TN];
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[mi][j] = f32x4{0};

    // A stage is multiplied in NU sub-phases: k-step s (32 wide) x token part q (TQ tiles), each
    // TQ x TN MFMAs.  Weight fragments are double-buffered by k-step; token parts ping-pong between
    // two small buffers.  Slot v of an iteration issues the MFMAs of sub-phase v-2 (the last two
    // sub-phases of a stage run in the first two slots of the next iteration, across the workgroup
    // barrier) and then requests the fragments of sub-phase v, whose buffer those MFMAs just freed.
    constexpr int TQ = MT == 3 ? 3 : (MT >= 2) ? MT / 2 : 1;    // token tiles per part (the parts per k-step, 2 MT / TQ, must divide the 4 weight tiles)
    constexpr int NP = TM / TQ;                   // parts per k-step
    constexpr int NU = 2 * NP;                    // sub-phases per stage
    bf16x8 wfr[2][TN], tq[2][TQ];
    // 16-row token groups of this wave that hold rows of the expert (the same for every lane of the wave).  With
    // few rows per expert most groups are empty: a wave whose last group is empty runs the loop in its
    // `part` form, which skips the fragment reads and MFMAs of empty groups behind wave-uniform branches
    // (Mixtral-8x22B, 64 rows per expert under 128-row tiles: gate/up 0.61 -> 0.55 ms; DeepSeek-V3 shapes, 8 rows
    // per expert, fp8: 4.3 -> 5.0 TB/s of weights).  Full waves keep the branch-free form: the branches cost the
    // exact operand waits (128 rows per expert: down projection 0.27 -> 0.30 ms with them).
    bool live[TM];
#pragma unroll
    for (int mi = 0; mi < TM; ++mi) live[mi] = wm * 32 * MT + 16 * mi < row_end - row0;
    auto read_w1 = [&](Stage S, int s, int j, auto part) __attribute__((always_inline)) {
        if (decltype(part)::value && !live[0]) return;
        const uint8_t* Bs = S.b;
        const uint32_t coff = (uint32_t)(((4 * s + fchunk) ^ fkey) << 4);
        wfr[s][j] = *reinterpret_cast<const bf16x8*>(Bs + w_off[j] + coff);
    };
    auto read_tq = [&](Stage S, int u, auto part) __attribute__((always_inline)) {
        const uint8_t* As = S.a;
        const int s = u / NP, q = u % NP;
        const uint32_t coff = (uint32_t)(((4 * s + fchunk) ^ fkey) << 4);
#pragma unroll
        for (int i = 0; i < TQ; ++i)
            if (!decltype(part)::value || live[q * TQ + i])
                tq[u & 1][i] = *reinterpret_cast<const bf16x8*>(As + tok_off[q * TQ + i] + coff);
    };
    auto mfma_sub = [&](int u, auto part) __attribute__((always_inline)) {
        const int s = u / NP, q = u % NP;
#pragma unroll
        for (int i = 0; i < TQ; ++i)
            if (!decltype(part)::value || live[q * TQ + i])
#pragma unroll
            for (int jx = 0; jx < TN; ++jx) {
                // snake order over the weight fragments: every instruction differs from the one before in
                // ONE operand (fewer input toggles per MFMA on a power-limited chip; +0.4 % measured)
                const int j = ((i + u) & 1) ? TN - 1 - jx : jx;
                acc[q * TQ + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wfr[s][j], tq[u & 1][i], acc[q * TQ + i][j], 0, 0, 0);
            }
    };
    // ---- main loop ----
    // On entry to iteration kt: LDS stage kt&1 holds tile kt and the registers hold tiles kt+1 ..
    // kt+PF (possibly still in flight).  The iteration moves tile kt+1 into the other LDS stage,
    // refills that register set with tile kt+1+PF and multiplies tile kt.
    gload(0, 0);
    if (PAIR8) {
#pragma unroll
        for (int i = 0; i < 4; ++i) pair_load(0, 0, i);
#pragma unroll
        for (int i = 0; i < 4; ++i) pair_load(1, 1, i);
    }
    lds_store(st0, 0);
    // No load or store of the pipeline sits under a branch or in a region that only some waves
    // execute (past the end the last tile is loaded again and stored where nobody reads it): with
    // straight-line code the compiler counts the outstanding loads exactly, so a store waits only
    // for the chunk it stores.  Under a branch it must assume the load may never have been issued
    // and waits for ALL outstanding loads, which serialises the whole pipeline.
#pragma unroll
    for (int d = 0; d < PF; ++d) gload(min(1 + d, nk - 1), d);
    __syncthreads();
    // One data item = one LDS store's worth of this thread's staged chunks (a 16-byte token chunk,
    // a 16-byte bf16 weight chunk, or half of a 16-byte fp8 weight chunk -> 8 bf16): store it to the
    // other stage and, once a chunk's last item is stored, refill its registers with the chunk of
    // tile kt+1+PF.  The items are spread over the iteration, one per group of MFMAs, so LDS, the
    // vector-memory pipe and the matrix core see a steady mix instead of bursts; with exact load
    // waits each item stalls only until its own chunk (requested PF iterations earlier) is there.
    constexpr int NI = NA + NB;
    // par = kt & 1 and ps, the register set of the pair that stage kt+1 belongs to, are literals at the call sites
    auto data_item = [&](int i, Stage S, int kt, int set, int par, int ps) __attribute__((always_inline)) {
        uint8_t *As = S.a, *Bs = S.b;
        const int kn = stage_at(min(kt + 1 + PF, nk - 1));
        const size_t kofs = (size_t)kn * BK;
        // past the end nobody reads what is loaded: streamed weights would come from HBM once more
        // (PF + 1 stages per tile), so those loads take the first 16 bytes of the activations instead
        const bool past = kt + 1 + PF >= nk;
        if (i < NA) {
            *reinterpret_cast<u32x4*>(As + a_lds + i * RA * ROW_B) = a_ok[i] ? ra[set][i] : u32x4{0, 0, 0, 0};
            ra[set][i] = gload16(g.a + (size_t)a_src[i] * K + kofs + lchunk * 8);
        } else if (PAIR8) {
            const int b = i - NA;
            if (par) {                      // stage kt+1 opens a pair
                pair_swap(ps, b);
                pair_store(Bs, ps, b, 0);
            } else {                        // it closes one: the set is free for the pair after the next
                pair_store(Bs, ps, b, 1);
                pair_load((kt >> 1) + 2, ps, b);
            }
        } else {
            const int b = i - NA;
            const uint8_t* m = (SWIGLU && b >= NB / 2) ? bmat1 : bmat0;
            *reinterpret_cast<u32x4*>(Bs + b_lds + b * RB * ROW_B) = rb[set][b];
            rb[set][b] = gload16_w<STREAM>(past ? (const uint8_t*)g.a : m + ((size_t)b_n[b] * K + kofs) * 2 + bcol_b);
        }
    };
    constexpr int NG = NU;                        // one group of MFMAs per slot
    constexpr int WPS = TN / NP;                  // weight fragments of the second k-step read per slot
    auto iteration = [&](int kt, int set, int par, int ps, auto part) __attribute__((always_inline)) {   // par == kt & 1
        const Stage rd = par ? st1 : st0;
        const Stage wr = par ? st0 : st1;
#pragma unroll
        for (int v = 0; v < NU; ++v) {
            // group v takes items [v*NI/NG, (v+1)*NI/NG): in order, so the two halves of an fp8
            // chunk are stored before its registers are refilled
#pragma unroll
            for (int i0 = v * NI / NG; i0 < (v + 1) * NI / NG; ++i0) {
                data_item(i0, wr, kt, set, par, ps);
            }
            if (!W8) __builtin_amdgcn_sched_barrier(0);
            if (v >= 2) mfma_sub(v - 2, part);
            else if (kt > 0) mfma_sub(NU - 2 + v, part);
            read_tq(rd, v, part);
            if (v == 0) {
#pragma unroll
                for (int j = 0; j < TN; ++j) read_w1(rd, 0, j, part);
            } else if (v >= 2 && v < 2 + NP) {
#pragma unroll
                for (int j = (v - 2) * WPS; j < (v - 1) * WPS; ++j) read_w1(rd, 1, j, part);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();   // (waits for this wave's LDS reads and writes, then for the other waves)
    };
    // Unrolled by two, the stage parity is a literal and every LDS address is a register plus an
    // immediate (about 20 vector and 12 scalar instructions less per iteration; headline -2 %).  The
    // bf16 kernel with BM = 256 has no registers for the longer live ranges (it would spill) and
    // keeps the rolled loop.
    auto k_loop = [&](auto part) __attribute__((always_inline)) {
        if (PAIR8) {
            // stage kt+1 belongs to pair (kt+1)/2, whose register set alternates: by four, every index is a literal
            int kt = 0;
            for (; kt + 4 <= nk; kt += 4) {
                iteration(kt, 0, 0, 0, part);
                iteration(kt + 1, 1, 1, 1, part);
                iteration(kt + 2, 0, 0, 1, part);
                iteration(kt + 3, 1, 1, 0, part);
            }
            if (kt < nk) {                       // (an even number of stages: fp8 scales come per 128 k)
                iteration(kt, 0, 0, 0, part);
                iteration(kt + 1, 1, 1, 1, part);
            }
        } else if (W8 || PF == 2) {
            int kt = 0;
            for (; kt + 2 <= nk; kt += 2) {
                iteration(kt, 0, 0, 0, part);
                iteration(kt + 1, PF - 1, 1, 0, part);
            }
            if (kt < nk) iteration(kt, 0, 0, 0, part);
        } else {
            for (int kt = 0; kt < nk; ++kt) iteration(kt, 0, kt & 1, 0, part);
        }
        mfma_sub(NU - 2, part);
        mfma_sub(NU - 1, part);
    };
    // (both forms pass the same barriers, so the waves of a workgroup may differ in theirs)
    if (!live[TM - 1]) k_loop(std::true_type{});
    else k_loop(std::false_type{});

    // ---- epilogue ----
    // All waves passed the loop's last barrier, so no one reads the stages: each wave transposes through its own
    // slice of them.
    constexpr int CW = SWIGLU ? 8 * TN : 16 * TN;    // output columns of this wave
    uint8_t* ep = ((wave < 4) ? st0.ep : st1.ep) + (wave & 3) * (32 * MT * CW * 2);
    const int ncol0 = n0 + wn * CW;
    store_wave_outputs<MT, TN, SWIGLU, 32 * MT, false>(acc, ep, lane, g.c + (size_t)(row0 + wm * 32 * MT) * N + ncol0, N,
                                                       min(BM, row_end - row0) - wm * 32 * MT, N - ncol0);
}

// ---- fp8 weight streamer: experts of up to 64 rows in calls that the one-workgroup-per-tile kernel serves alone ----
//
// With a handful of rows per expert a launch reads every weight once (Expert_Wrapper.forward in its decoding use,
// Wrapper.py:470-530) and is bound by how fast a CU can take fp8 weights in.  Through gemm_tile a 64-k stage of 256
// weight rows costs 16 KiB of global loads into registers, the conversion, 32 KiB of LDS stores, a barrier and
// 64 KiB of fragment reads, and streams at 4-5 TB/s.  Here
//  * the workgroup's 8 waves split the tile's WEIGHT rows (32 each: a 16-row gate fragment and the matching up
//    fragment, or two fragments of the down matrix) and every wave multiplies all token rows, so a weight is
//    converted once, by the wave that feeds it to the matrix core;
//  * weights reach LDS as fp8 by DMA (buffer_load ... lds), 8 lanes x 16 bytes per row = whole 128-byte lines per
//    request, 128 k at a time, into the wave's own 4 KiB of a buffer: no staging registers, no LDS stores, half the
//    bytes, and three buffers keep two 128-k blocks in flight per CU;
//  * a lane reads 16 consecutive fp8 weights of its fragment row (one ds_read_b128), which after conversion are its
//    A operands of BOTH 32-wide k-steps of a 64-k half: lane group q holds k = 16 f(q) + 8 s + (0..7) in step s
//    (f = 0, 2, 1, 3), and the token operand reads the chunk that holds those k.  A dot product does not care in which order k is walked,
//    and the order depends on nothing but the column: a row's result does not depend on its tile or its neighbours.
// LDS layouts (the DMA lets every lane fetch what belongs at its place, so swizzles are free):
//  weights: 128-byte rows, 16-byte part c of fragment row r at part c ^ wsw(r); tokens: 256-byte rows (128 k), chunk
//  c of row r at chunk c ^ tsw(r).  The LDS serves lanes 8 i .. 8 i + 7 together with lanes 32 + 8 i .. (the same 8
//  rows, lane groups q and q + 2, whose chunks f(q) and f(q + 2) = f(q) + 1 are neighbours): with these keys their 16
//  reads fall on 16 different bank groups.  (Measured with 8 waves reading back to back: 32 cycles per wave and
//  ds_read_b128 for both layouts, 55 with lane group q on chunk q.)
__device__ __forceinline__ int wsw(int r) { return ((r >> 1) & 1) | (((r >> 2) & 1) << 2); }
__device__ __forceinline__ int tsw(int r) { return (r & 3) | ((r & 4) << 1); }

constexpr int S8_WBYTES = 32 * 1024;              // weight region of a buffer: 8 waves x 32 rows x 128 fp8
constexpr int S8_TROWS = 64;                      // token rows staged

// A buffer of the weight streamers: the weight region and the token region are separate LDS arrays, so that a read of
// one never has to wait for a DMA into the other
struct SBuf {
    uint8_t *w, *t;
};

template <int TG, bool SWIGLU>   // TG: 16-row token groups multiplied (the expert has at most 16 TG <= 64 rows)
__device__ __forceinline__ void stream8_tile(const GemmArgs& g, SBuf buf0, SBuf buf1, SBuf buf2, int e, int row0,
                                             int row_end, int n_tile) {
    constexpr int NBLK = SWIGLU ? 128 : 256;
    constexpr int NDW = 4, NDT = 2;               // DMA instructions per wave and 128-k block: weights, tokens
    // Operations that may stay in flight at the wait for a block: the DMA of the next block, NDW + NDT instructions
    // (the counter retires in issue order).  The next block's two scale loads are issued before its DMA and are
    // older still: not counting them costs at most a wait for two small loads that hit in L2, and keeps the count
    // right for the first block, which has no scale loads of a block before it behind its DMA.
    constexpr int VM_BLOCK = NDW + NDT;
    static_assert(TG >= 1 && 16 * TG <= S8_TROWS, "token rows staged");
    const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6);
    const int n0 = n_tile * NBLK;
    const int K = g.K, N = g.N;
    const int npair = K >> 7;
    // N tile t walks k from 128-k block t (mod the number of blocks), so that the requests in flight on the chip do
    // not share their low address bits (weight rows are K bytes apart); a column's order depends on its tile alone
    const int prot = n_tile % npair;

    // ---- DMA coordinates ----
    // weights, instruction i: rows 8 i + lane / 8 of the wave's 32 (fragment i / 2, fragment row 8 (i & 1) + lane / 8)
    const int lr = lane >> 3, pp = lane & 7;
    uint32_t w_voff[NDW];
    const uint8_t* bmat[2];
    gptr_f32 sc[2];
    int srow[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        bmat[j] = uni_ptr((SWIGLU && j == 1) ? g.b1[e] : g.b0[e]);
        sc[j] = (gptr_f32)(uintptr_t)uni_ptr((SWIGLU && j == 1) ? g.s1[e] : g.s0[e]);
        srow[j] = min((n0 + (SWIGLU ? 0 : 32 * wave)) >> 7, (N >> 7) - 1) * npair;
    }
#pragma unroll
    for (int i = 0; i < NDW; ++i) {
        const int fr = 8 * (i & 1) + lr;
        const int rt = SWIGLU ? 16 * wave + fr : 32 * wave + 16 * (i >> 1) + fr;      // row of the tile's N range
        w_voff[i] = (uint32_t)min(n0 + rt, N - 1) * (uint32_t)K + (uint32_t)((pp ^ wsw(fr)) << 4);
    }
    // tokens, instruction i: rows 8 wave + 4 i + lane / 16 of the 64 staged, chunk lane % 16.  Gathered rows go through
    // one descriptor over x (a row_map entry outside x reads zeros), sorted rows through one that holds the tile's rows
    // and nothing else.  Rows past the expert's last get an offset past either descriptor: zeros arrive in LDS
    // without a request to memory (nobody uses the products of those rows; the instruction still counts).
    uint32_t t_voff[NDT];
    const uint8_t* a_base = reinterpret_cast<const uint8_t*>(g.a) + (g.row_map ? (size_t)0 : (size_t)row0 * K * 2);
    const int a_records = g.row_map ? (int)(uint32_t)g.a_bytes : (row_end - row0) * K * 2;
#pragma unroll
    for (int i = 0; i < NDT; ++i) {
        const int tr = 8 * wave + 4 * i + (lane >> 4);
        const int r = min(row0 + tr, row_end - 1);
        const int src = g.row_map ? ((gptr_i32)(uintptr_t)g.row_map)[r] : r - row0;
        t_voff[i] = (uint32_t)src * (uint32_t)(K * 2) + (uint32_t)(((lane & 15) ^ tsw(tr)) << 4);
        if (row0 + tr >= row_end || (g.row_map && (unsigned)src >= (unsigned)g.a_rows)) t_voff[i] = 0xfffffff0u;
    }
    float rsc[2][2];                              // block scales of the block being multiplied / of the next one
    auto scales = [&](int p_pipe, int set) {
        int pr = min(p_pipe, npair - 1) + prot;
        pr = pr >= npair ? pr - npair : pr;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)(uintptr_t)sc[j], 0, -1, 0x00020000);
            rsc[set][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, 0, (srow[j] + pr) * 4, 0));
        }
    };
    // DMA instruction i of a block: 0 .. NDW-1 weights (read once: non-temporal, which is worth 5 % of the stream),
    // NDW .. NDW+NDT-1 tokens
    auto dma_one = [&](int p_pipe, SBuf buf, int i) __attribute__((always_inline)) {
        // past the end of k nobody reads what arrives: an empty descriptor returns zeros without touching memory,
        // and the instruction still counts
        const int live = uni(p_pipe < npair ? -1 : 0);   // (a scalar, or the descriptor ends up in vector registers)
        int pr = min(p_pipe, npair - 1) + prot;
        pr = pr >= npair ? pr - npair : pr;
        if (i < NDW) {
            const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)bmat[i >> 1], 0, live, 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_u8)(buf.w + wave * 4096 + i * 1024), 16, w_voff[i], (uint32_t)(pr * 128), 0, 2);
        } else {
            const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)a_base, 0, live & a_records, 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_u8)(buf.t + wave * 2048 + (i - NDW) * 1024), 16, t_voff[i - NDW],
                                                     (uint32_t)(pr * 256), 0, 0);
        }
    };
    auto dma = [&](int p_pipe, SBuf buf) {
#pragma unroll
        for (int i = 0; i < NDW + NDT; ++i) dma_one(p_pipe, buf, i);
    };

    const int frow = lane & 15, q = lane >> 4;
    const int fq = ((q & 1) << 1) | (q >> 1);
    const uint32_t w_rd = (uint32_t)(wave * 4096 + frow * 128), wkey = (uint32_t)wsw(frow);
    const uint32_t t_rd = (uint32_t)(frow * 256), tkey = (uint32_t)tsw(frow);   // (group bases are multiples of 16)
    f32x4 acc[TG][2];
#pragma unroll
    for (int t = 0; t < TG; ++t) { acc[t][0] = f32x4{0}; acc[t][1] = f32x4{0}; }

    // Iteration p multiplies block p out of buffer p % 3.  Before it: this wave's DMA of block p has landed (at most the
    // DMA of block p + 1 is outstanding) and its LDS reads have returned, then everybody's (a bare s_barrier: a fence
    // would make the compiler wait for ALL outstanding DMA).  After the barrier every wave has left block p - 1,
    // whose buffer takes block p + 2 (its DMA is spread over the iteration).  The scale loads come BEFORE the DMA: the
    // compiler's own wait for a scale counts everything issued after it as allowed to be in flight.
    auto iteration = [&](int p, SBuf rd, SBuf refill, int sset) __attribute__((always_inline)) {
        // (lgkmcnt: this wave's LDS reads of block p - 1 have returned -- its last matrix instructions may be scheduled
        // behind the barrier, and the buffer they read is refilled right after it)
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" :: "n"(VM_BLOCK) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        scales(p + 1, sset ^ 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            bf16x8 wa[2][2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const u32x4 raw = *reinterpret_cast<const u32x4*>(rd.w + w_rd + j * 2048 + (((4 * h + fq) ^ wkey) << 4));
                wa[j][0] = __builtin_bit_cast(bf16x8, dequant8(raw[0], raw[1], rsc[sset][j]));
                wa[j][1] = __builtin_bit_cast(bf16x8, dequant8(raw[2], raw[3], rsc[sset][j]));
            }
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
                const uint32_t coff = (uint32_t)(((8 * h + 2 * fq + s2) ^ tkey) << 4);
#pragma unroll
                for (int t = 0; t < TG; ++t) {
                    const bf16x8 tf = *reinterpret_cast<const bf16x8*>(rd.t + t_rd + t * 16 * 256 + coff);
                    acc[t][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[0][s2], tf, acc[t][0], 0, 0, 0);
                    acc[t][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[1][s2], tf, acc[t][1], 0, 0, 0);
                }
                // the refill of the freed buffer goes out between the four groups of matrix instructions (2, 2, 1, 1
                // DMA instructions): a wave that issues all six first stands in the memory pipeline's queue while its
                // matrix instructions wait behind them (3 % at 40-64 rows)
                const int st = 2 * h + s2;
                __builtin_amdgcn_sched_barrier(0);
                dma_one(p + 2, refill, st < 2 ? 2 * st : st + 2);
                if (st < 2) dma_one(p + 2, refill, 2 * st + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    scales(0, 0);
    dma(0, buf0);
    dma(1, buf1);
    int p = 0;
    for (; p + 3 <= npair; p += 3) {
        iteration(p, buf0, buf2, 0);
        iteration(p + 1, buf1, buf0, 1);
        iteration(p + 2, buf2, buf1, 0);
        // (three iterations flip the scale set: swap so that the loop body keeps literal indices)
        const float t0 = rsc[0][0], t1 = rsc[0][1];
        rsc[0][0] = rsc[1][0]; rsc[0][1] = rsc[1][1];
        rsc[1][0] = t0; rsc[1][1] = t1;
    }
    if (p < npair) {
        iteration(p, buf0, buf2, 0);
        if (p + 1 < npair) iteration(p + 1, buf1, buf0, 1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no DMA may land in LDS after the workgroup has gone

    // ---- epilogue: a lane holds 4 consecutive columns of one row per accumulator and stores them itself ----
#pragma unroll
    for (int t = 0; t < TG; ++t) {
        const int r = row0 + 16 * t + frow;
        if (r >= row_end) continue;
        if (SWIGLU) {
            const int col = n0 + 16 * wave + 4 * q;
            if (col < N) *reinterpret_cast<u32x2*>(g.c + (size_t)r * N + col) = epilogue_pack<true>(acc[t][0], acc[t][1]);
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int col = n0 + 32 * wave + 16 * j + 4 * q;
                if (col < N) *reinterpret_cast<u32x2*>(g.c + (size_t)r * N + col) = epilogue_pack<false>(acc[t][j], acc[t][j]);
            }
        }
    }
}


// ---- fp8 weight streamer in the persistent kernel's summation order: tiles of up to 128 rows ----
//
// The same division of labour as stream8_tile (8 waves x 32 weight rows, fp8 weights by DMA in whole lines, every wave
// multiplies all token rows), for tiles whose rows another kernel might have computed: what an fp8 expert's full
// 256-row tiles leave over, the halves of the persistent kernel's last tiles, and in calls that this kernel serves
// alone the experts (or 128-row slices of experts) above 64 rows.  A row's bits must then not depend on who computes
// it, so every matrix instruction gets the k values the persistent kernel gives it, in the same lanes: lane group q
// holds k = 32 s + 8 f(q) + (0..7) of k-step s, f = 0, 2, 1, 3.  Those are 8 consecutive fp8 weights, one half of a
// 16-byte part (read whole; the weights are a ninth of the LDS reads), and the 16-byte token chunk 4 s + f(q) of a
// 64-k half.  128 token rows x 128 k would not fit LDS three times over next to the weights, so token rows travel in
// halves of 64 k (128 rows x 128 bytes = 16 KiB) through three buffers of their own, one barrier per half, while the
// weights keep their three buffers of 128 k: 96 + 48 KiB.  Per half-block a wave issues 2 weight DMA instructions (of
// the block two ahead) and 2 token DMA instructions (of the half two ahead), and the wait before a half's barrier
// leaves the 4 of the half before in flight.  k starts at block 0 unless the kernel has the call to itself.
template <int TG, bool SWIGLU>   // TG: 16-row token groups multiplied (1 .. 8)
__device__ __forceinline__ void stream8x_tile(const GemmArgs& g, SBuf b0, SBuf b1, SBuf b2, int e, int row0, int row_end,
                                              int n_tile, bool rotate) {
    constexpr int NBLK = SWIGLU ? 128 : 256;
    constexpr int VM_HALF = 4;                    // DMA instructions per wave and half-block: 2 weights + 2 tokens
    static_assert(TG >= 1 && TG <= 8, "token rows staged");
    const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6);
    const int n0 = n_tile * NBLK;
    const int K = g.K, N = g.N;
    const int npair = K >> 7;
    const int prot = rotate ? n_tile % npair : 0;             // k_rotation in blocks of 128 k

    // ---- DMA coordinates ----
    // weights, instruction i (0..3): rows 8 i + lane / 8 of the wave's 32 (fragment i / 2, fragment row 8 (i & 1) + lane / 8);
    // 16-byte part c of fragment row r at part c ^ wsw(r)
    const int lr = lane >> 3, pp = lane & 7;
    uint32_t w_voff[4];
    const uint8_t* bmat[2];
    cptr_f32 sc[2];
    int srow[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        bmat[j] = uni_ptr((SWIGLU && j == 1) ? g.b1[e] : g.b0[e]);
        sc[j] = (cptr_f32)(uintptr_t)uni_ptr((SWIGLU && j == 1) ? g.s1[e] : g.s0[e]);
        srow[j] = min((n0 + (SWIGLU ? 0 : 32 * wave)) >> 7, (N >> 7) - 1) * npair;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int fr = 8 * (i & 1) + lr;
        const int rt = SWIGLU ? 16 * wave + fr : 32 * wave + 16 * (i >> 1) + fr;      // row of the tile's N range
        w_voff[i] = (uint32_t)min(n0 + rt, N - 1) * (uint32_t)K + (uint32_t)((pp ^ wsw(fr)) << 4);
    }
    // tokens, instruction i (0..1): rows 16 wave + 8 i + lane / 8 of the 128 staged, 16-byte chunk c of row r at chunk
    // c ^ swz(r) (the persistent kernel's layout of a 64-k stage).  Rows past the tile's last: zeros, no request.
    uint32_t t_voff[2];
    const uint8_t* a_base = reinterpret_cast<const uint8_t*>(g.a) + (g.row_map ? (size_t)0 : (size_t)row0 * K * 2);
    const int a_records = g.row_map ? (int)(uint32_t)g.a_bytes : (row_end - row0) * K * 2;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int tr = 16 * wave + 8 * i + lr;
        const int r = min(row0 + tr, row_end - 1);
        const int src = g.row_map ? ((gptr_i32)(uintptr_t)g.row_map)[r] : r - row0;
        t_voff[i] = (uint32_t)src * (uint32_t)(K * 2) + (uint32_t)((pp ^ swz(tr)) << 4);
        if (row0 + tr >= row_end || (g.row_map && (unsigned)src >= (unsigned)g.a_rows)) t_voff[i] = 0xfffffff0u;
    }
    float rsc[2][2];                              // block scales of the block being multiplied / of the next one
    auto scales = [&](int p_pipe, int set) {      // scalar loads (uniform addresses in the constant address space)
        int pr = min(p_pipe, npair - 1) + prot;
        pr = pr >= npair ? pr - npair : pr;
#pragma unroll
        for (int j = 0; j < 2; ++j) rsc[set][j] = sc[j][srow[j] + pr];
    };
    // weight DMA instruction i of block p_pipe (pipeline order) / token DMA instruction i of half-block hb_pipe
    auto dma_w = [&](int p_pipe, SBuf buf, int i) __attribute__((always_inline)) {
        const int live = uni(p_pipe < npair ? -1 : 0);   // past the end: an empty descriptor, zeros without a request
        int pr = min(p_pipe, npair - 1) + prot;
        pr = pr >= npair ? pr - npair : pr;
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)bmat[i >> 1], 0, live, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_u8)(buf.w + wave * 4096 + i * 1024), 16, w_voff[i], (uint32_t)(pr * 128), 0, 2);
    };
    auto dma_t = [&](int hb_pipe, SBuf buf, int i) __attribute__((always_inline)) {
        const int live = uni(hb_pipe < 2 * npair ? -1 : 0);
        const int hb = min(hb_pipe, 2 * npair - 1);
        int pr = (hb >> 1) + prot;
        pr = pr >= npair ? pr - npair : pr;
        const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)a_base, 0, live & a_records, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_u8)(buf.t + wave * 2048 + i * 1024), 16, t_voff[i],
                                                 (uint32_t)(pr * 256 + (hb & 1) * 128), 0, 0);
    };

    const int frow = lane & 15, q = lane >> 4;
    const int fq = ((q & 1) << 1) | (q >> 1);
    // weights: the 8 bytes at 32 s + 8 f(q) of the 64-byte half h of fragment row frow: 16-byte part 4 h + 2 s + f(q) / 2
    const uint32_t w_rd = (uint32_t)(wave * 4096 + frow * 128), wkey = (uint32_t)wsw(frow);
    const uint32_t t_rd = (uint32_t)(frow * 128), tkey = (uint32_t)swz(frow);   // (group bases are multiples of 16 rows)
    f32x4 acc[TG][2];
#pragma unroll
    for (int t = 0; t < TG; ++t) { acc[t][0] = f32x4{0}; acc[t][1] = f32x4{0}; }

    // Half-block H = 2 p + h multiplies half h of block p: weights out of buffer p % 3, tokens out of token buffer
    // H % 3.  Before it: this wave's DMA of its tokens (issued two halves ago) and of everything older has landed and
    // its LDS reads have returned, then everybody's (a bare s_barrier).  After the barrier every wave has left half
    // H - 1, whose token buffer takes half H + 2, and (h == 0) block p - 1, whose weight buffer takes block p + 2 over
    // the two halves of block p.
    auto half = [&](int p, int h, SBuf wb, SBuf tb, SBuf w_refill, SBuf t_refill, int sset) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" :: "n"(VM_HALF) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // every operand of the half is requested up front (2 + TG reads per k-step): the matrix instructions then run
        // behind the LDS pipeline instead of waiting out its latency one token group at a time
        u32x2 wraw[2][2];
        bf16x8 tf[2][TG];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                // (the whole 16-byte part, of which this lane group uses one half and the group two further on the
                // other: the two read the same address in the same LDS pass, a broadcast, where 8-byte reads of
                // every other half collide -- SQ_LDS_BANK_CONFLICT was three times the LDS instruction cycles)
                const u32x4 part = *reinterpret_cast<const u32x4*>(wb.w + w_rd + j * 2048 + (((4 * h + 2 * s2 + (fq >> 1)) ^ wkey) << 4));
                wraw[s2][j] = (fq & 1) ? u32x2{part[2], part[3]} : u32x2{part[0], part[1]};
            }
            const uint32_t coff = (uint32_t)(((4 * s2 + fq) ^ tkey) << 4);
#pragma unroll
            for (int t = 0; t < TG; ++t) tf[s2][t] = *reinterpret_cast<const bf16x8*>(tb.t + t_rd + t * 16 * 128 + coff);
        }
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            bf16x8 wa[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) wa[j] = __builtin_bit_cast(bf16x8, dequant8(wraw[s2][j][0], wraw[s2][j][1], rsc[sset][j]));
#pragma unroll
            for (int t = 0; t < TG; ++t) {
                acc[t][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[0], tf[s2][t], acc[t][0], 0, 0, 0);
                acc[t][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[1], tf[s2][t], acc[t][1], 0, 0, 0);
            }
            dma_w(p + 2, w_refill, 2 * h + s2);
            dma_t(2 * p + h + 2, t_refill, s2);
        }
        // (the next block's scales: scalar loads, issued where no LDS read is outstanding -- the two share a counter
        // and scalar loads return out of order, which would turn every operand wait into a full drain)
        if (h == 0) scales(p + 1, sset ^ 1);
    };
    // Prologue: blocks 0 and 1 and halves 0 and 1, the tokens of half 0 before the weights of block 1, so that the
    // first half's wait (all but the 4 youngest instructions) covers what it reads, as in the steady state.
    scales(0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(0, b0, i);
#pragma unroll
    for (int i = 0; i < 2; ++i) dma_t(0, b0, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(1, b1, i);
#pragma unroll
    for (int i = 0; i < 2; ++i) dma_t(1, b1, i);
    // Six halves = three blocks bring both rotations back to where they started: literal buffers in the loop body.
    int p = 0;
    for (; p + 3 <= npair; p += 3) {
        half(p, 0, b0, b0, b2, b2, 0);
        half(p, 1, b0, b1, b2, b0, 0);
        half(p + 1, 0, b1, b2, b0, b1, 1);
        half(p + 1, 1, b1, b0, b0, b2, 1);
        half(p + 2, 0, b2, b1, b1, b0, 0);
        half(p + 2, 1, b2, b2, b1, b1, 0);
        const float t0 = rsc[0][0], t1 = rsc[0][1];
        rsc[0][0] = rsc[1][0]; rsc[0][1] = rsc[1][1];
        rsc[1][0] = t0; rsc[1][1] = t1;
    }
    if (p < npair) {
        half(p, 0, b0, b0, b2, b2, 0);
        half(p, 1, b0, b1, b2, b0, 0);
        if (p + 1 < npair) {
            half(p + 1, 0, b1, b2, b0, b1, 1);
            half(p + 1, 1, b1, b0, b0, b2, 1);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no DMA may land in LDS after the workgroup has gone

    // ---- epilogue: a lane holds 4 consecutive columns of one row per accumulator and stores them itself ----
#pragma unroll
    for (int t = 0; t < TG; ++t) {
        const int r = row0 + 16 * t + frow;
        if (r >= row_end) continue;
        if (SWIGLU) {
            const int col = n0 + 16 * wave + 4 * q;
            if (col < N) *reinterpret_cast<u32x2*>(g.c + (size_t)r * N + col) = epilogue_pack<true>(acc[t][0], acc[t][1]);
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int col = n0 + 32 * wave + 16 * j + 4 * q;
                if (col < N) *reinterpret_cast<u32x2*>(g.c + (size_t)r * N + col) = epilogue_pack<false>(acc[t][j], acc[t][j]);
            }
        }
    }
}

// ---- fp8 weight streamer in the persistent kernel's summation order: tiles of 129 to 192 rows ----
//
// stream8x_tile for 9 to 12 groups of 16 token rows: what an fp8 expert's full 256-row tiles leave over when that is
// more than 128 rows (as a padded 256-row tile of the persistent kernel such rows cost a third to a half more matrix
// work than they hold), and experts of that size in calls that this kernel serves alone.  Same weight DMA and LDS
// layouts, the same division of labour (a weight is converted once, by the wave that multiplies it: with two sets of
// 4 waves over the token groups, as in the bf16 streamer, every weight is converted twice, and the conversion then
// takes the vector ALU as long as the products take the matrix cores -- DeepSeek-V3 at 4096 tokens 4.52 against 4.31
// ms), same k values in the same lanes.  What differs: such a tile is bound by the matrix cores, not by the weight
// stream, and 192 token rows x 64 k are 24 KiB, so there are two weight buffers, the next block requested right
// after a block's first barrier (a block of 128 k takes the matrix cores about 2 us, more than a trip to memory), and
// two token buffers, one per half of a block, each refilled right after the barrier that retires it, one half ahead
// (token rows come out of L2).
// Before a block's first half everything this wave requested must have landed (vmcnt 0); before its second half all
// but the 4 weight instructions of the next block, which were issued behind that half's token rows.
template <int TG, bool SWIGLU>   // TG: 16-row token groups multiplied (9 .. 12)
__device__ __forceinline__ void stream8w_tile(const GemmArgs& g, uint8_t* w0, uint8_t* w1, uint8_t* t0, uint8_t* t1, int e,
                                              int row0, int row_end, int n_tile, bool rotate) {
    constexpr int NBLK = SWIGLU ? 128 : 256;
    constexpr int NF = 2;                         // 16-row weight fragments per wave
    constexpr int NDT = (2 * TG + 7) / 8;         // token DMA instructions per wave and half (8 rows each)
    static_assert(TG >= 9 && TG <= 12 && NDT == 3, "token rows staged");
    const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6);
    const int n0 = n_tile * NBLK;
    const int K = g.K, N = g.N;
    const int npair = K >> 7;
    const int prot = rotate ? n_tile % npair : 0;             // k_rotation in blocks of 128 k

    // ---- DMA coordinates (weights as in stream8x_tile: wave w brings LDS rows 32 w .. 32 w + 31, fragments 2 w, 2 w + 1) ----
    const int lr = lane >> 3, pp = lane & 7;
    uint32_t w_voff[4], t_voff[NDT];
    const uint8_t* bmat[2];
    cptr_f32 sc[2];
    int srow[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        bmat[j] = uni_ptr((SWIGLU && j == 1) ? g.b1[e] : g.b0[e]);
        sc[j] = (cptr_f32)(uintptr_t)uni_ptr((SWIGLU && j == 1) ? g.s1[e] : g.s0[e]);
        srow[j] = min((n0 + (SWIGLU ? 0 : 32 * wave)) >> 7, (N >> 7) - 1) * npair;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int fr = 8 * (i & 1) + lr;
        const int rt = SWIGLU ? 16 * wave + fr : 32 * wave + 16 * (i >> 1) + fr;      // row of the tile's N range
        w_voff[i] = (uint32_t)min(n0 + rt, N - 1) * (uint32_t)K + (uint32_t)((pp ^ wsw(fr)) << 4);
    }
    const uint8_t* a_base = reinterpret_cast<const uint8_t*>(g.a) + (g.row_map ? (size_t)0 : (size_t)row0 * K * 2);
    const int a_records = g.row_map ? (int)(uint32_t)g.a_bytes : (row_end - row0) * K * 2;
#pragma unroll
    for (int i = 0; i < NDT; ++i) {               // token rows 64 i + 8 wave + lr; rows past the tile's last: zeros, no request
        const int tr = 64 * i + 8 * wave + lr;
        const int r = min(row0 + tr, row_end - 1);
        const int src = g.row_map ? ((gptr_i32)(uintptr_t)g.row_map)[r] : r - row0;
        t_voff[i] = (uint32_t)src * (uint32_t)(K * 2) + (uint32_t)((pp ^ swz(tr)) << 4);
        if (row0 + tr >= row_end || (g.row_map && (unsigned)src >= (unsigned)g.a_rows)) t_voff[i] = 0xfffffff0u;
    }
    float rsc[2][2];                              // block scales of the block being multiplied / of the next one
    auto block_of = [&](int p_pipe) { int pr = min(p_pipe, npair - 1) + prot; return pr >= npair ? pr - npair : pr; };
    auto scales = [&](int p_pipe, int set) {      // scalar loads (uniform addresses in the constant address space)
        const int pr = block_of(p_pipe);
#pragma unroll
        for (int j = 0; j < 2; ++j) rsc[set][j] = sc[j][srow[j] + pr];
    };
    auto dma_w = [&](int p_pipe, uint8_t* wb, int i) __attribute__((always_inline)) {
        const int live = uni(p_pipe < npair ? -1 : 0);   // past the end: an empty descriptor, zeros without a request
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)bmat[i >> 1], 0, live, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_u8)(wb + wave * 4096 + i * 1024), 16, w_voff[i], (uint32_t)(block_of(p_pipe) * 128), 0, 2);
    };
    auto dma_t = [&](int hb_pipe, uint8_t* tb, int i) __attribute__((always_inline)) {
        const int live = uni(hb_pipe < 2 * npair ? -1 : 0);
        const int hb = min(hb_pipe, 2 * npair - 1);
        const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)a_base, 0, live & a_records, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_u8)(tb + (64 * i + 8 * wave) * 128), 16, t_voff[i],
                                                 (uint32_t)(block_of(hb >> 1) * 256 + (hb & 1) * 128), 0, 0);
    };

    // ---- operand coordinates: a wave multiplies the two fragments it brought ----
    const int frow = lane & 15, q = lane >> 4;
    const int fq = ((q & 1) << 1) | (q >> 1);
    const uint32_t wkey = (uint32_t)wsw(frow), tkey = (uint32_t)swz(frow);
    const uint32_t w_rd = (uint32_t)(wave * 4096 + frow * 128), t_rd = (uint32_t)(frow * 128);
    f32x4 acc[TG][NF];
#pragma unroll
    for (int t = 0; t < TG; ++t)
#pragma unroll
        for (int f = 0; f < NF; ++f) acc[t][f] = f32x4{0};

    // Half h of block p: weights out of wb (block p), token rows out of tb (half 2 p + h).
    auto half = [&](int p, int h, const uint8_t* wb, const uint8_t* tb, uint8_t* w_refill, uint8_t* t_refill, int sset) __attribute__((always_inline)) {
        if (h == 0) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // every wave has left half 2 p + h - 1 (its token buffer takes half 2 p + h + 1) and, h == 0, block p - 1 (its
        // weight buffer takes block p + 1)
#pragma unroll
        for (int i = 0; i < NDT; ++i) dma_t(2 * p + h + 1, t_refill, i);
        if (h == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) dma_w(p + 1, w_refill, i);
        }
        __builtin_amdgcn_sched_barrier(0);
        u32x2 wraw[2][NF];
        bf16x8 tf[2][TG];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                // (the whole 16-byte part, of which this lane group uses one half and the group two further on the other)
                const u32x4 part = *reinterpret_cast<const u32x4*>(wb + w_rd + f * 2048 + (((4 * h + 2 * s2 + (fq >> 1)) ^ wkey) << 4));
                wraw[s2][f] = (fq & 1) ? u32x2{part[2], part[3]} : u32x2{part[0], part[1]};
            }
            const uint32_t coff = (uint32_t)(((4 * s2 + fq) ^ tkey) << 4);
#pragma unroll
            for (int t = 0; t < TG; ++t) tf[s2][t] = *reinterpret_cast<const bf16x8*>(tb + t_rd + t * 16 * 128 + coff);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            bf16x8 wa[NF];
#pragma unroll
            for (int f = 0; f < NF; ++f)
                wa[f] = __builtin_bit_cast(bf16x8, dequant8(wraw[s2][f][0], wraw[s2][f][1], rsc[sset][f]));
#pragma unroll
            for (int t = 0; t < TG; ++t)
#pragma unroll
                for (int f = 0; f < NF; ++f) acc[t][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[f], tf[s2][t], acc[t][f], 0, 0, 0);
        }
        // (the next block's scales: scalar loads, issued where no LDS read is outstanding)
        if (h == 0) scales(p + 1, sset ^ 1);
        __builtin_amdgcn_sched_barrier(0);
    };
    scales(0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(0, w0, i);
#pragma unroll
    for (int i = 0; i < NDT; ++i) dma_t(0, t0, i);
    // Two blocks bring the weight buffers and the scale sets back to where they started: literal buffers in the loop body.
    int p = 0;
    for (; p + 2 <= npair; p += 2) {
        half(p, 0, w0, t0, w1, t1, 0);
        half(p, 1, w0, t1, w1, t0, 0);
        half(p + 1, 0, w1, t0, w0, t1, 1);
        half(p + 1, 1, w1, t1, w0, t0, 1);
    }
    if (p < npair) {
        half(p, 0, w0, t0, w1, t1, 0);
        half(p, 1, w0, t1, w1, t0, 0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no DMA may land in LDS after the workgroup has gone

    // ---- epilogue: a lane holds 4 consecutive columns of one row per accumulator and stores them itself ----
#pragma unroll
    for (int t = 0; t < TG; ++t) {
        const int r = row0 + 16 * t + frow;
        if (r >= row_end) continue;
#pragma unroll
        for (int f = 0; f < (SWIGLU ? 1 : NF); ++f) {
            const int col = n0 + (SWIGLU ? 16 : 32) * wave + 16 * f + 4 * q;
            if (col < N) *reinterpret_cast<u32x2*>(g.c + (size_t)r * N + col) = epilogue_pack<SWIGLU>(acc[t][f], acc[t][SWIGLU ? 1 : f]);
        }
    }
}

template <bool SWIGLU>
__device__ __forceinline__ void stream8w(const GemmArgs& g, uint8_t* w0, uint8_t* w1, uint8_t* t0, uint8_t* t1, int e, int row0,
                                         int row_end, int n_tile, bool rotate) {
    const int rows = row_end - row0;
    if (rows <= 144) stream8w_tile<9, SWIGLU>(g, w0, w1, t0, t1, e, row0, row_end, n_tile, rotate);
    else if (rows <= 160) stream8w_tile<10, SWIGLU>(g, w0, w1, t0, t1, e, row0, row_end, n_tile, rotate);
    else if (rows <= 176) stream8w_tile<11, SWIGLU>(g, w0, w1, t0, t1, e, row0, row_end, n_tile, rotate);
    else stream8w_tile<12, SWIGLU>(g, w0, w1, t0, t1, e, row0, row_end, n_tile, rotate);
}

// M tiles of an expert with `count` rows in the one-workgroup-per-tile kernel: one tile of up to 192 rows if that
// holds them all, else tiles of 128.  The height follows the EXPERT, not the launch: a tile taller
// than its expert stages and multiplies rows that do not exist, and an expert cut into several tiles reads its
// weights once per tile and adds workgroups (the hot expert of a skewed decode batch: 9 x 128 tiles are 4.5 rounds
// of 256 CUs and cost 5).  The tiles of an expert that is cut (above 192 rows) run side by side on one XCD and take
// the weights with plain loads, so that all but the first read of a line come out of that XCD's L2.
// 256-row tiles of an expert with `count` rows in the persistent kernel's tile space
// whether an expert of `count` rows belongs to the one-workgroup-per-tile kernel (no rem_split)
__device__ __forceinline__ bool is_cold(const GemmArgs& g, int count) {
    return count <= g.cold_max || (g.pair_rows && count >= PAIR_LO && count <= PAIR_HI);
}
__device__ __forceinline__ int persistent_tiles(const GemmArgs& g, int count) {
    if (g.rem_split) return (count >> 8) + ((count & 255) > g.cold_max ? 1 : 0);
    return is_cold(g, count) ? 0 : (count + 255) >> 8;
}
// How many tiles at the end of that space the persistent kernel leaves to the other kernel.  One workgroup per CU
// walks the space in rounds of tail_cus tiles, and a last round of a few tiles costs as much as a full one while
// most CUs idle.  Cut into 128-row halves those tiles occupy twice as many CUs for about 0.7 of a tile's time
// each, and they join the other kernel's `own` tiles in its rounds.  The last round moves if that makes the two
// launches shorter, counting a round of the persistent kernel 1.0 and a round of the other 0.72: alone (own = 0)
// that is a last round of at most half the CUs; next to other work also a longer one (Mixtral-8x22B, 1024 tokens,
// down projection: 144 tiles here and 144 there are two half-empty launches in a row, 0.71 ms; as one launch of 432
// tiles 0.56).  Both kernels evaluate this on the same offsets[].
__device__ __forceinline__ int tail_tiles(const GemmArgs& g, int total, int own) {
    if (g.tail_cus <= 0) return 0;
    const int cus = g.tail_cus, tail = total % cus;
    if (tail == 0) return 0;
    const int keep = 100 * (total / cus + 1) + 72 * ((own + cus - 1) / cus);
    const int move = 100 * (total / cus) + 72 * ((own + 2 * tail + cus - 1) / cus);
    return move < keep ? tail : 0;
}

template <bool PAIR>   // whether an expert of PAIR_LO .. PAIR_HI rows is cut in the middle (bf16 weights)
__device__ __forceinline__ int tiles_of(int count) {
    constexpr int SINGLE = 192;   // rows that one tile may hold
    if (count <= SINGLE) return count > 0 ? 1 : 0;
    // bf16 weights: an expert of 257 to 384 rows is cut in the middle, into two tiles of the 192-row body that run
    // side by side on one XCD and share the weights through its L2: 320 rows are 2 x 160 rows of MFMA work, where
    // two 256-row tiles of the persistent kernel multiply 512 and three 128-row tiles read the weights three times.
    // Mixtral-8x22B shapes, 8 experts of 288 / 320 / 384 rows: gate/up 1.31 / 1.29 / 1.30 -> 1.07 / 1.13 / 1.17 ms,
    // down projection within 4 % either way; up to 256 rows one tile of the persistent kernel stays better (224
    // rows: 0.82 against 1.01 ms).
    if (PAIR && count > PAIR_LO - 1 && count <= PAIR_HI) return 2;
    return (count + 127) >> 7;
}
// rows of either tile of such a pair (the first tile holds whole 16-row groups)
__device__ __forceinline__ int half_rows(int count) { return ((count + 1) / 2 + 15) & ~15; }

// M tiles of an expert with `count` rows in the one-workgroup-per-tile kernel's own tile space
template <bool W8>
__device__ __forceinline__ int own_tiles(const GemmArgs& g, int c) {
    if (g.rem_split) c &= 255;      // the rows the persistent kernel's full tiles leave over
    return (g.rem_split ? c > g.cold_max : !is_cold(g, c)) ? 0 : tiles_of<!W8>(c);
}

// sum over the experts of f(count) (every thread gets it; two barriers)
template <int NT, typename F>
__device__ __forceinline__ int sum_over_experts(const GemmArgs& g, int tid, int* s_wtot, F f) {
    int v = 0;
    for (int e = tid; e < g.E; e += NT) v += f(g.offsets[e + 1] - g.offsets[e]);
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
    __syncthreads();                 // whoever read s_wtot before has done so
    if ((tid & 63) == 0) s_wtot[tid >> 6] = v;
    __syncthreads();
    int tot = 0;
#pragma unroll
    for (int w = 0; w < NT / 64; ++w) tot += s_wtot[w];
    return tot;
}

// ---- bf16 weight streamer in the persistent kernel's summation order: tiles of up to 192 rows ----
//
// The fp8 streamers' way of moving data for bf16 weights: weights and token rows reach LDS by DMA in the persistent
// kernel's layout of a 64-k stage (128-byte rows, chunk c of row r at c ^ swz(r)), and every matrix instruction gets
// the k values the persistent kernel gives it, in the same lanes, so a row's bits do not depend on who computes it.
// No staging registers and no LDS stores, so every operand of a stage can be requested up front.  Up to 64 rows the 8
// waves split the tile's 256 weight rows and each multiplies all token rows; above, two sets of 4 waves take half of
// the token groups each (4 + TG / 2 operand reads per k-step for 2 TG matrix instructions, where 8 x 1 waves need
// 2 + TG for as many).  Three weight buffers of 32 KiB keep two stages of weights in flight; token rows (up to
// 24 KiB per stage, out of L2) have two buffers and travel one stage ahead, issued first in a stage so that the wait
// before the next stage's barrier leaves only the 4 weight instructions behind them in flight.
// Weight row R of a stage (LDS row R, brought by wave R / 32): column n0 + R; gate and up: gate column n0 + R,
// R < 128, up column n0 + R - 128 above.  k starts at stage 0 unless the kernel has the call to itself.
template <int TG, bool SWIGLU, bool SHARED>   // TG: 16-row token groups multiplied (1 .. 12); SHARED: another tile reads these weights
__device__ __forceinline__ void stream16_tile(const GemmArgs& g, uint8_t* w0, uint8_t* w1, uint8_t* w2, uint8_t* t0, uint8_t* t1,
                                              int e, int row0, int row_end, int n_tile) {
    constexpr int NBLK = SWIGLU ? 128 : 256;
    constexpr int WM = TG >= 5 ? 2 : 1;           // sets of waves across the token groups
    constexpr int TH = (TG + WM - 1) / WM;        // token groups per wave (an odd TG: the second set's last group is padding)
    constexpr int NF = 2 * WM;                    // 16-row weight fragments per wave
    constexpr int NDW = 4;                        // weight DMA instructions per wave and stage
    constexpr int NDT = (2 * TG + 7) / 8;         // token DMA instructions per wave and stage (8 rows each; 64 rows per round of the waves)
    static_assert(TG >= 1 && TG <= 12, "token rows staged");
    const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6);
    const int wm = WM == 2 ? wave >> 2 : 0, wn = WM == 2 ? wave & 3 : wave;
    const int n0 = n_tile * NBLK;
    const int K = g.K, N = g.N;
    const int nk = K / BK;
    const int prot = k_rotation<false>(n_tile, nk);

    // ---- DMA coordinates: lane l supplies row +l/8 of an instruction's 8 rows and the 16 bytes that belong at physical chunk l%8 ----
    const int lr = lane >> 3, pp = lane & 7;
    uint32_t w_voff[NDW], t_voff[NDT];
    const uint8_t* bmat = uni_ptr((SWIGLU && wave >= 4) ? g.b1[e] : g.b0[e]);
#pragma unroll
    for (int i = 0; i < NDW; ++i) {               // LDS rows 32 wave + 8 i + lr
        const int R = 32 * wave + 8 * i + lr;
        w_voff[i] = (uint32_t)min(n0 + (SWIGLU ? R & 127 : R), N - 1) * (uint32_t)(K * 2) + (uint32_t)((pp ^ swz(R)) << 4);
    }
    const uint8_t* a_base = reinterpret_cast<const uint8_t*>(g.a) + (g.row_map ? (size_t)0 : (size_t)row0 * K * 2);
    const int a_records = g.row_map ? (int)(uint32_t)g.a_bytes : (row_end - row0) * K * 2;
#pragma unroll
    for (int i = 0; i < NDT; ++i) {               // token rows 64 i + 8 wave + lr; rows past the tile's last: zeros, no request
        const int tr = 64 * i + 8 * wave + lr;
        const int r = min(row0 + tr, row_end - 1);
        const int src = g.row_map ? ((gptr_i32)(uintptr_t)g.row_map)[r] : r - row0;
        t_voff[i] = (uint32_t)src * (uint32_t)(K * 2) + (uint32_t)((pp ^ swz(tr)) << 4);
        if (row0 + tr >= row_end || (g.row_map && (unsigned)src >= (unsigned)g.a_rows)) t_voff[i] = 0xfffffff0u;
    }
    auto stage_off = [&](int kt_pipe) {           // byte offset of pipeline stage kt_pipe in a row (the last one again past the end)
        int kt = min(kt_pipe, nk - 1) + prot;
        kt = kt >= nk ? kt - nk : kt;
        return (uint32_t)(kt * BK * 2);
    };
    auto dma_w = [&](int kt_pipe, uint8_t* wb, int i) __attribute__((always_inline)) {
        const int live = uni(kt_pipe < nk ? -1 : 0);   // past the end: an empty descriptor, zeros without a request
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)bmat, 0, live, 0x00020000);
        // (non-temporal unless a neighbour on this XCD reads the same lines and should find them in its L2)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_u8)(wb + wave * 4096 + i * 1024), 16, w_voff[i], stage_off(kt_pipe), 0, SHARED ? 0 : 2);
    };
    auto dma_t = [&](int kt_pipe, uint8_t* tb, int i) __attribute__((always_inline)) {
        const int live = uni(kt_pipe < nk ? -1 : 0);
        const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)a_base, 0, live & a_records, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_u8)(tb + (64 * i + 8 * wave) * ROW_B), 16, t_voff[i], stage_off(kt_pipe), 0, 0);
    };

    // ---- operand coordinates: fragment j of the wave is LDS rows wrow(j) .. + 15 ----
    const int frow = lane & 15, q = lane >> 4;
    const int fq = ((q & 1) << 1) | (q >> 1);
    const uint32_t fkey = (uint32_t)swz(frow);
    auto wrow = [&](int j) { return SWIGLU ? (j / WM) * 128 + 16 * WM * wn + 16 * (j % WM) : 32 * WM * wn + 16 * j; };
    const uint32_t w_rd = (uint32_t)((wrow(0) + frow) * ROW_B), t_rd = (uint32_t)((16 * TH * wm + frow) * ROW_B);
    f32x4 acc[TH][NF];
#pragma unroll
    for (int t = 0; t < TH; ++t)
#pragma unroll
        for (int j = 0; j < NF; ++j) acc[t][j] = f32x4{0};

    // Stage kt is multiplied out of weight buffer kt % 3 and token buffer kt % 2.  Before it: this wave's DMA of its
    // tokens (issued first in the stage before) and of everything older has landed, its LDS reads have returned, then
    // everybody's (a bare s_barrier).  After the barrier every wave has left stage kt - 1: its token buffer takes
    // stage kt + 1, its weight buffer stage kt + 2.
    // Every operand of the stage is requested up front (4 + TG / 2 or 2 + TG reads per k-step): the matrix instructions
    // then run behind the LDS pipeline instead of waiting out its latency one token group at a time.
    bf16x8 wa0[NF], tf0[TH], wa1[NF], tf1[TH];
    auto read_step = [&](const uint8_t* wb, const uint8_t* tb, int s, bf16x8 (&wa)[NF], bf16x8 (&tf)[TH]) __attribute__((always_inline)) {
        const uint32_t coff = (uint32_t)(((4 * s + fq) ^ fkey) << 4);
#pragma unroll
        for (int j = 0; j < NF; ++j) wa[j] = *reinterpret_cast<const bf16x8*>(wb + w_rd + (wrow(j) - wrow(0)) * ROW_B + coff);
#pragma unroll
        for (int t = 0; t < TH; ++t) tf[t] = *reinterpret_cast<const bf16x8*>(tb + t_rd + t * 16 * ROW_B + coff);
    };
    // (with 2 of the 4 instructions of the weight DMA after the first token group)
    auto mfma_step = [&](const bf16x8 (&wa)[NF], const bf16x8 (&tf)[TH], int kt_dma, uint8_t* w_refill, int i0) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < TH; ++t) {
#pragma unroll
            for (int j = 0; j < NF; ++j) acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[j], tf[t], acc[t][j], 0, 0, 0);
            if (t == 0) { dma_w(kt_dma, w_refill, i0); dma_w(kt_dma, w_refill, i0 + 1); }
        }
    };
    auto stage = [&](int kt, const uint8_t* wb, const uint8_t* tb, uint8_t* w_refill, uint8_t* t_refill) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" :: "n"(NDW) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < NDT; ++i) dma_t(kt + 1, t_refill, i);
        __builtin_amdgcn_sched_barrier(0);
        read_step(wb, tb, 0, wa0, tf0);
        read_step(wb, tb, 1, wa1, tf1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_step(wa0, tf0, kt + 2, w_refill, 0);
        mfma_step(wa1, tf1, kt + 2, w_refill, 2);
        __builtin_amdgcn_sched_barrier(0);      // (or the matrix instructions sink below the next stage's barrier, behind its reads)
    };
    // Prologue: the tokens of stage 0 between the weights of stages 0 and 1, so that the first wait (all but the 4
    // youngest instructions) covers what stage 0 reads, as in the steady state.
#pragma unroll
    for (int i = 0; i < NDW; ++i) dma_w(0, w0, i);
#pragma unroll
    for (int i = 0; i < NDT; ++i) dma_t(0, t0, i);
#pragma unroll
    for (int i = 0; i < NDW; ++i) dma_w(1, w1, i);
    // Six stages bring both rotations back to where they started: literal buffers in the loop body.
    int kt = 0;
    for (; kt + 6 <= nk; kt += 6) {
        stage(kt, w0, t0, w2, t1);
        stage(kt + 1, w1, t1, w0, t0);
        stage(kt + 2, w2, t0, w1, t1);
        stage(kt + 3, w0, t1, w2, t0);
        stage(kt + 4, w1, t0, w0, t1);
        stage(kt + 5, w2, t1, w1, t0);
    }
    if (kt < nk) stage(kt, w0, t0, w2, t1);
    if (kt + 1 < nk) stage(kt + 1, w1, t1, w0, t0);
    if (kt + 2 < nk) stage(kt + 2, w2, t0, w1, t1);
    if (kt + 3 < nk) stage(kt + 3, w0, t1, w2, t0);
    if (kt + 4 < nk) stage(kt + 4, w1, t0, w0, t1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no DMA may land in LDS after the workgroup has gone

    // ---- epilogue: a lane holds 4 consecutive columns of one row per accumulator and stores them itself ----
#pragma unroll
    for (int t = 0; t < TH; ++t) {
        const int r = row0 + 16 * (TH * wm + t) + frow;
        if (r >= row_end) continue;
#pragma unroll
        for (int j = 0; j < (SWIGLU ? WM : NF); ++j) {
            const int col = n0 + wrow(j) + 4 * q;
            if (col < N) *reinterpret_cast<u32x2*>(g.c + (size_t)r * N + col) = epilogue_pack<SWIGLU>(acc[t][j], acc[t][SWIGLU ? WM + j : j]);
        }
    }
}

template <bool SWIGLU, bool SHARED>
__device__ __forceinline__ void stream16(const GemmArgs& g, uint8_t* w0, uint8_t* w1, uint8_t* w2, uint8_t* t0, uint8_t* t1, int e,
                                         int row0, int row_end, int n_tile) {
    const int tg = (row_end - row0 + 15) >> 4;
    switch (tg) {
#define MOE_S16_CASE(n) case n: stream16_tile<n, SWIGLU, SHARED>(g, w0, w1, w2, t0, t1, e, row0, row_end, n_tile); break;
    MOE_S16_CASE(1) MOE_S16_CASE(2) MOE_S16_CASE(3) MOE_S16_CASE(4) MOE_S16_CASE(5) MOE_S16_CASE(6)
    MOE_S16_CASE(7) MOE_S16_CASE(8) MOE_S16_CASE(9) MOE_S16_CASE(10) MOE_S16_CASE(11)
#undef MOE_S16_CASE
    default: stream16_tile<12, SWIGLU, SHARED>(g, w0, w1, w2, t0, t1, e, row0, row_end, n_tile); break;
    }
}

template <bool SWIGLU>
__device__ __forceinline__ void stream8x(const GemmArgs& g, SBuf b0, SBuf b1, SBuf b2, int e, int row0, int row_end, int n_tile,
                                         bool rotate) {
    const int rows = row_end - row0;
    if (rows <= 16) stream8x_tile<1, SWIGLU>(g, b0, b1, b2, e, row0, row_end, n_tile, rotate);
    else if (rows <= 32) stream8x_tile<2, SWIGLU>(g, b0, b1, b2, e, row0, row_end, n_tile, rotate);
    else if (rows <= 48) stream8x_tile<3, SWIGLU>(g, b0, b1, b2, e, row0, row_end, n_tile, rotate);
    else if (rows <= 64) stream8x_tile<4, SWIGLU>(g, b0, b1, b2, e, row0, row_end, n_tile, rotate);
    else if (rows <= 80) stream8x_tile<5, SWIGLU>(g, b0, b1, b2, e, row0, row_end, n_tile, rotate);
    else if (rows <= 96) stream8x_tile<6, SWIGLU>(g, b0, b1, b2, e, row0, row_end, n_tile, rotate);
    else if (rows <= 112) stream8x_tile<7, SWIGLU>(g, b0, b1, b2, e, row0, row_end, n_tile, rotate);
    else stream8x_tile<8, SWIGLU>(g, b0, b1, b2, e, row0, row_end, n_tile, rotate);
}

// One workgroup per (M tile, N tile); serves what the persistent kernel does not take (few rows per expert, odd K).
template <int WN, bool SWIGLU, bool W8>
__global__ __launch_bounds__(128 * WN) void grouped_gemm_kernel(GemmArgs g) {
    constexpr int NT = 128 * WN;
    // Three weight arrays of 32 KiB and token arrays of 16 KiB (fp8 weights: three, 128 rows; the second one 24 KiB)
    // or 24 KiB (bf16: two, 192 rows) -- the buffers of the weight streamers, written by DMA, as separate objects so
    // that a read of one waits for no DMA into another; gemm_tile's two stages (up to 128 token rows + 256 weight
    // rows) are two pairs of them.  The fp8 streamer for 129 to 192 rows has two weight buffers and keeps its token
    // rows (24 KiB per half) in the third weight array and the 24 KiB token array.
    constexpr int TB = W8 ? 128 * ROW_B : 192 * ROW_B;
    __shared__ __attribute__((aligned(1024))) uint8_t lw0[S8_WBYTES];
    __shared__ __attribute__((aligned(1024))) uint8_t lw1[S8_WBYTES];
    __shared__ __attribute__((aligned(1024))) uint8_t lw2[S8_WBYTES];
    __shared__ __attribute__((aligned(1024))) uint8_t lt0[TB];
    __shared__ __attribute__((aligned(1024))) uint8_t lt1[192 * ROW_B];
    __shared__ __attribute__((aligned(1024))) uint8_t lt2[W8 ? TB : 16];
    static_assert(S8_TROWS * 256 <= 128 * ROW_B && S8_WBYTES == BN_ROWS * ROW_B, "regions of a streamer buffer");
    auto stage = [&](int i) { return Stage{i ? lt1 : lt0, i ? lw1 : lw0, i ? lw1 : lw0}; };
    const SBuf sb0{lw0, lt0}, sb1{lw1, lt1}, sb2{lw2, lt2};
    __shared__ int s_pref[MAX_E + 1];
    __shared__ int s_wtot[NT / 64];
    __shared__ int s_sel[5];
    const int tid = threadIdx.x;

    // ---- M-tile prefix over experts ----
    ExpertOfThread mine;
    const bool s8_ok = !g.row_map || g.a_bytes < (1ull << 32);   // (the weight streamer addresses gathered rows with 32-bit offsets)
    int run = mtile_prefix_scan<NT>(g, tid, s_pref, s_wtot, mine, [&](int c) { return own_tiles<W8>(g, c); }, [](int, int, int) {});
    const int total = run * g.n_tiles_n;

    // ---- XCD-aware id: groups of 4 consecutive tiles (the M tiles of one N tile first) go round-robin to the XCDs
    // (workgroup ids are dealt to the XCDs one by one).  The tiles of a multi-tile expert that read the same
    // weights then share them through one XCD's L2, and dealing small groups round keeps the XCDs even whatever
    // the number of tiles and however much one expert's tiles cost more than another's ----
    const int slot = blockIdx.x >> 3;
    int v = (((slot >> 2) << 3) + (blockIdx.x & 7)) * 4 + (slot & 3);
    // Past this kernel's own tiles: the tiles that the persistent kernel leaves at the end of ITS tile space, two
    // workgroups (128-row halves, neighbours on one XCD) per tile.  The prefix is rebuilt over that space.
    int half = -1;
    if (v >= total) {
        if (g.tail_cus <= 0 || g.E > NT) return;
        const int t = v - total;
        __syncthreads();                 // s_wtot of the first scan has been read by everyone
        run = mtile_prefix_scan<NT>(g, tid, s_pref, s_wtot, mine, [&](int c) { return persistent_tiles(g, c); }, [](int, int, int) {});
        const int total_p = run * g.n_tiles_n;
        const int tail = tail_tiles(g, total_p, total);
        if (t >= 2 * tail) return;
        v = total_p - tail + (t >> 1);
        half = t & 1;
    }
    const int q = v / g.n_tiles_n;  // global M-tile number
    // find e with prefix[e] <= q < prefix[e+1].  Up to NT experts every thread still holds its own
    // expert's prefix, tile count and row range: the one that owns q publishes them (one barrier,
    // no search, no second trip to memory for the offsets).  More experts: binary search in LDS.
    if (g.E <= NT) {
        if (tid < g.E && mine.start <= q && q < mine.start + mine.mt) {
            s_sel[0] = tid; s_sel[1] = mine.start; s_sel[2] = mine.mt; s_sel[3] = mine.o0; s_sel[4] = mine.o1;
        }
        __syncthreads();
    } else {
        if (tid == 0) s_pref[g.E] = run;
        __syncthreads();
        int lo = 0, hi = g.E;
        while (hi - lo > 1) {
            int mid = (lo + hi) >> 1;
            if (s_pref[mid] <= q) lo = mid; else hi = mid;
        }
        if (tid == 0) {
            s_sel[0] = lo; s_sel[1] = s_pref[lo]; s_sel[2] = s_pref[lo + 1] - s_pref[lo];
            s_sel[3] = g.offsets[lo]; s_sel[4] = g.offsets[lo + 1];
        }
        __syncthreads();
    }
    const int e = uni(s_sel[0]);
    const int pe = uni(s_sel[1]);
    const int mt_e = uni(s_sel[2]);
    int m_tile, n_tile;
    tile_in_expert(v - pe * g.n_tiles_n, mt_e, g.n_tiles_n, m_tile, n_tile);
    if (half >= 0) {                     // half of a 256-row tile of the persistent kernel's space
        const int r0 = uni(s_sel[3]) + m_tile * 256 + half * 128;
        const int r1 = min(uni(s_sel[4]), uni(s_sel[3]) + (m_tile + 1) * 256);
        if (r0 >= r1) return;
        if (W8 && s8_ok) stream8x<SWIGLU>(g, sb0, sb1, sb2, e, r0, r1, n_tile, false);
        else if (s8_ok) stream16<SWIGLU, true>(g, lw0, lw1, lw2, lt0, lt1, e, r0, min(r1, r0 + 128), n_tile);
        else gemm_tile<2, WN, SWIGLU, W8, false>(g, stage(0), stage(1), e, r0, r1, n_tile);
        return;
    }
    const int row_end = uni(s_sel[4]);
    const int first_row = uni(s_sel[3]) + (g.rem_split ? ((row_end - uni(s_sel[3])) & ~255) : 0);
    const bool alone = g.cold_max == 0x7fffffff;
    if (W8 && s8_ok) {
        // fp8 weights: the weight streamers.  Up to 64 rows in a call that this kernel has to itself, where no other
        // kernel's summation order has to be matched: the form that reads a lane's 16 weights at once.  Everything
        // else -- up to 192 rows; what an expert's full 256-row tiles leave over; 128-row slices of larger experts
        // when the kernel is alone -- in the persistent kernel's order.
        const int r0 = first_row + (mt_e > 1 ? m_tile * 128 : 0), r1 = mt_e > 1 ? min(row_end, r0 + 128) : row_end;
        const int rows = r1 - r0;
        if (alone && mt_e == 1 && rows <= 64) {
            if (rows <= 16) stream8_tile<1, SWIGLU>(g, sb0, sb1, sb2, e, r0, r1, n_tile);
            else if (rows <= 32) stream8_tile<2, SWIGLU>(g, sb0, sb1, sb2, e, r0, r1, n_tile);
            else if (rows <= 48) stream8_tile<3, SWIGLU>(g, sb0, sb1, sb2, e, r0, r1, n_tile);
            else stream8_tile<4, SWIGLU>(g, sb0, sb1, sb2, e, r0, r1, n_tile);
        } else if (rows > 128) {                 // (one tile of 129 to 192 rows)
            stream8w<SWIGLU>(g, lw0, lw1, lw2, lt1, e, r0, r1, n_tile, alone);
        } else {
            stream8x<SWIGLU>(g, sb0, sb1, sb2, e, r0, r1, n_tile, alone);
        }
        return;
    }
    // The rows of this workgroup: the expert's (one tile: up to 192 rows), one half of an
    // expert of PAIR_LO .. PAIR_HI rows (bf16), or a 128-row slice.
    const int rows_e = row_end - first_row;
    const bool pair = !W8 && rows_e >= PAIR_LO && rows_e <= PAIR_HI;
    const int slice = pair ? half_rows(rows_e) : 128;
    const int t0 = mt_e > 1 ? first_row + m_tile * slice : first_row, t1 = mt_e > 1 ? min(row_end, t0 + slice) : row_end;
    if (!W8 && s8_ok) {
        // bf16 weights: the weight streamer in the persistent kernel's order
        if (mt_e == 1) stream16<SWIGLU, false>(g, lw0, lw1, lw2, lt0, lt1, e, t0, t1, n_tile);
        else stream16<SWIGLU, true>(g, lw0, lw1, lw2, lt0, lt1, e, t0, t1, n_tile);
        return;
    }
    // 4 GiB of gathered rows or more: the register-staged body, which addresses them with 64-bit offsets, 128 rows
    // at a time
    if (t1 - t0 <= 64) {
        gemm_tile<1, WN, SWIGLU, W8, true>(g, stage(0), stage(1), e, t0, t1, n_tile);
    } else if (mt_e == 1) {
        gemm_tile<2, WN, SWIGLU, W8, true>(g, stage(0), stage(1), e, t0, min(t1, t0 + 128), n_tile);
        if (t1 - t0 > 128) {
            __syncthreads();
            gemm_tile<2, WN, SWIGLU, W8, true>(g, stage(0), stage(1), e, t0 + 128, t1, n_tile);
        }
    } else {
        gemm_tile<2, WN, SWIGLU, W8, false>(g, stage(0), stage(1), e, t0, min(t1, t0 + 128), n_tile);
        if (t1 - t0 > 128) {
            __syncthreads();
            gemm_tile<2, WN, SWIGLU, W8, false>(g, stage(0), stage(1), e, t0 + 128, t1, n_tile);
        }
    }
}

// lane id produced where it is used: the compiler cannot hoist it (and everything derived from it)
// out of the tile loop and keep it in registers through the k loop
__device__ __forceinline__ int fresh_lane() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

// Persistent kernel for BM = 256: one workgroup per CU walks its share of the tiles, and the software
// pipeline runs on across the tile boundary (a tile's last k-iterations already fetch the next tile's
// first stages, the epilogue goes through the idle stage, and the next tile starts with its first stage
// in LDS).  What a fresh workgroup pays per tile -- launch, tile-prefix scan, pointer chase, first fetch,
// store drain: 6-8 us against 57 us of k loop for K = 2048 -- is paid once per workgroup or overlaps
// the previous tile's work.
//
// Token rows (and bf16 weights) reach LDS by DMA: buffer_load_dwordx4 ... lds writes 64 lanes x 16 bytes
// to 1 KiB of consecutive LDS, each lane fetching the 16 bytes that belong at its position of the
// swizzled layout, so there are no staging registers, no LDS store instructions and no per-chunk load
// waits in the MFMA stream: a wave waits once per k-iteration, before the barrier, for its own DMA of the
// next stage.  fp8 weights still go through registers (they are converted on the way), two k-stages
// ahead.  Three things make this worth it (the same loads issued as global_load ... lds in one array per
// stage measured 2 % slower than register staging; this form 3-5 % faster):
//  * buffer (MUBUF) loads.  The compiler models the FLAT-encoded global_load ... lds as a possible LDS
//    access through the flat aperture and from then on waits for ALL outstanding LDS operations
//    (lgkmcnt(0)) wherever an operand fragment is needed, which serialises the fragment reads.
//  * token stages and weight stages are separate LDS arrays.  An LDS store that may alias the target of
//    an outstanding DMA gets a vmcnt(0) in front of it; the fp8 weight stores must not.
//  * stage parities are literals (the k loop is unrolled by two), so reads of one stage provably do not
//    alias the DMA into the other.
template <bool SWIGLU, bool W8>
__global__ __launch_bounds__(512) void grouped_gemm_persistent_kernel(GemmArgs g) {
    constexpr int MT = 4, WN = 4;
    constexpr int NT = 128 * WN;
    constexpr int BM = 64 * MT;
    constexpr int A_STAGE = BM * ROW_B;
    constexpr int B_STAGE = BN_ROWS * ROW_B;
    constexpr int RB = NT / 4;                  // fp8: B rows per pass (rows are 4 chunks of 16 weights)
    constexpr int NB = BN_ROWS / RB;            // fp8: 16-byte global B chunks per thread per stage (2)
    constexpr int NBLK = SWIGLU ? 128 : 256;
    constexpr int NJ = 8 / WN;
    constexpr int ND = 4;                       // DMA instructions per wave and tile half (32 rows of 128 bytes = 4 x 1 KiB)
    // four separate arrays: the DMA writes the token stages, the fp8 path writes the weight stages with
    // ordinary LDS stores; as separate objects the two provably do not alias (otherwise every LDS store
    // waits for all outstanding DMA)
    __shared__ __attribute__((aligned(1024))) uint8_t sA0[A_STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t sA1[A_STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t sB0[B_STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t sB1[B_STAGE];
    __shared__ int s_pref[MAX_E + 1];
    __shared__ int s_wtot[NT / 64];
    constexpr int PE = 512;
    __shared__ int s_off[PE + 1];
    __shared__ unsigned long long s_ptr[4][PE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_s = uni(wave);
    const int wm = wave_s & 1, wn = (wave_s >> 1) % WN;

    // M-tile prefix over experts; the experts' row offsets and matrix pointers go to LDS tables on the way
    ExpertOfThread mine;
    const int run = mtile_prefix_scan<NT>(g, tid, s_pref, s_wtot, mine, [&](int c) { return persistent_tiles(g, c); }, [&](int e, int o0, int o1) {
        s_off[e] = o0;
        if (e == g.E - 1) s_off[g.E] = o1;
        s_ptr[0][e] = (unsigned long long)(uintptr_t)g.b0[e];
        s_ptr[1][e] = SWIGLU ? (unsigned long long)(uintptr_t)g.b1[e] : 0ull;
        s_ptr[2][e] = W8 ? (unsigned long long)(uintptr_t)g.s0[e] : 0ull;
        s_ptr[3][e] = (W8 && SWIGLU) ? (unsigned long long)(uintptr_t)g.s1[e] : 0ull;
    });
    if (tid == 0) s_pref[g.E] = run;
    __syncthreads();
    // whole rounds, and the last one unless it is better off with the other kernel, whose own tiles are counted for that
    const int own = g.tail_cus > 0 ? sum_over_experts<NT>(g, tid, s_wtot, [&](int c) { return own_tiles<W8>(g, c); }) * g.n_tiles_n : 0;
    const int total = run * g.n_tiles_n - tail_tiles(g, run * g.n_tiles_n, own);
    const int xcd = blockIdx.x & 7, slots = gridDim.x >> 3;
    int slot = blockIdx.x >> 3;
    auto tile_of = [&](int sl) { return ((sl / slots) * 8 + xcd) * slots + (sl % slots); };
    if (tile_of(slot) >= total) return;
    const int K = g.K, N = g.N;
    const int KB = K >> 7;

    // Token rows come through a buffer descriptor and 32-bit byte offsets.  Gathered rows (row_map): one
    // descriptor over all of x, whose size the launcher has checked against 4 GiB, so a row_map entry
    // outside x reads zeros instead of faulting.  Sorted rows: the descriptor starts at the tile's first row.
    const uint8_t *a_base = reinterpret_cast<const uint8_t*>(g.a), *a_base_n = a_base;
    const int a_records = g.row_map ? (int)(uint32_t)g.a_bytes : -1;
    uint32_t a_voff[ND], a_voff_n[ND];          // this wave's DMA offsets of the tile being fetched / of the next one
    // bf16 weights also by DMA: descriptors of the expert's matrices and per-lane offsets
    uint32_t b_voff[ND], b_voff_n[ND];
    const uint8_t *bm_cur = nullptr, *bm_next = nullptr;   // matrix this wave's weight rows come from (gate or up / down)
    // fp8 weights through registers
    uint32_t b8_voff[NB];
    const uint8_t *b8m0 = nullptr, *b8m1 = nullptr;
    int srow0 = 0, srow1 = 0;
    gptr_f32 sc0 = nullptr, sc1 = nullptr;
    int row0 = 0, row_end = 0, n0 = 0;
    int cur_e = 0;
    // bf16 weights: k starts at another stage for every N tile (k_rotation); stage_of is the stage that pipeline step
    // kt fetches.  The rotation is adopted with the tile's DMA coordinates.
    const int nk = K / BK;
    int rot = 0, rot_n = 0;
    auto stage_of = [&](int kt, int r) { const int kp = kt + r; return kp >= nk ? kp - nk : kp; };
    auto setup = [&](int v) {
        const int l = fresh_lane();
        const int t = wave_s * 64 + l;
        const int q = v / g.n_tiles_n;
        while (uni(s_pref[cur_e + 1]) <= q) ++cur_e;
        const int e = cur_e;
        const int pe = uni(s_pref[e]);
        const int mt_e = uni(s_pref[e + 1]) - pe;
        int m_tile, n_tile;
        tile_in_expert(v - pe * g.n_tiles_n, mt_e, g.n_tiles_n, m_tile, n_tile);
        row0 = uni(s_off[e]) + m_tile * BM;
        row_end = uni(s_off[e + 1]);
        n0 = n_tile * NBLK;
        rot_n = W8 ? 0 : k_rotation<false>(n_tile, nk);
        // DMA instruction i of this wave fills rows 32*wave + 8*i .. +7 of a stage: lane l supplies row +l/8 and
        // the 16 bytes that belong at physical chunk l%8, i.e. logical chunk (l%8) ^ swz(row)
        const int lr = l >> 3, pc = l & 7;
#pragma unroll
        for (int i = 0; i < ND; ++i) {
            const int rt = 32 * wave_s + 8 * i + lr;                 // row of the tile
            const int lc = pc ^ (lr ^ (i & 1));                       // swz(rt): rt & 7 == lr, (rt >> 3) & 1 == i & 1
            const int r = min(row0 + rt, row_end - 1);
            const int src = g.row_map ? ((gptr_i32)(uintptr_t)g.row_map)[r] : r - row0;
            a_voff_n[i] = (uint32_t)src * (uint32_t)(K * 2) + (uint32_t)(lc * 16);
        }
        if (!g.row_map) a_base_n = reinterpret_cast<const uint8_t*>(g.a) + (size_t)row0 * K * 2;
        const uint8_t* bmat0 = uni_ptr(reinterpret_cast<const void*>((uintptr_t)s_ptr[0][e]));
        const uint8_t* bmat1 = SWIGLU ? uni_ptr(reinterpret_cast<const void*>((uintptr_t)s_ptr[1][e])) : bmat0;
        if (W8) {
            sc0 = (gptr_f32)(uintptr_t)uni_ptr(reinterpret_cast<const void*>((uintptr_t)s_ptr[2][e]));
            sc1 = SWIGLU ? (gptr_f32)(uintptr_t)uni_ptr(reinterpret_cast<const void*>((uintptr_t)s_ptr[3][e])) : sc0;
            const int brow = t >> 2, bcol_b = (t & 3) << 4;
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                int r = brow + RB * i;
                int n = SWIGLU ? (n0 + (r & 127)) : (n0 + r);
                b8_voff[i] = (uint32_t)min(n, N - 1) * (uint32_t)K + (uint32_t)bcol_b;
            }
            b8m0 = bmat0; b8m1 = bmat1;
            if (SWIGLU) { srow0 = (n0 >> 7) * KB; srow1 = srow0; }
            else        { srow0 = (n0 >> 7) * KB; srow1 = min((n0 >> 7) + 1, (N >> 7) - 1) * KB; }
        } else {
            // rows 32*wave .. +31 of the weight tile: waves 0-3 the first 128 rows (gate), 4-7 the second (up)
            bm_next = (SWIGLU && wave_s >= 4) ? bmat1 : bmat0;
#pragma unroll
            for (int i = 0; i < ND; ++i) {
                const int rt = 32 * wave_s + 8 * i + lr;
                const int lc = pc ^ (lr ^ (i & 1));
                const int n = SWIGLU ? (n0 + (rt & 127)) : (n0 + rt);
                b_voff_n[i] = (uint32_t)min(n, N - 1) * (uint32_t)(K * 2) + (uint32_t)(lc * 16);
            }
        }
    };
    auto adopt = [&]() {   // the next tile's DMA coordinates become the current ones
#pragma unroll
        for (int i = 0; i < ND; ++i) { a_voff[i] = a_voff_n[i]; if (!W8) b_voff[i] = b_voff_n[i]; }
        if (!W8) bm_cur = bm_next;
        a_base = a_base_n;
        rot = rot_n;
    };
    auto dma_a = [&](uint8_t* stA, int kt, int i) {
        const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)a_base, 0, a_records, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, (lds_u8)(stA + (32 * wave_s + 8 * i) * ROW_B), 16, a_voff[i],
                                                 (uint32_t)((W8 ? kt : stage_of(kt, rot)) * BK * 2), 0, 0);
    };
    auto dma_b = [&](uint8_t* stB, int kt, int i) {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)bm_cur, 0, -1, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_u8)(stB + (32 * wave_s + 8 * i) * ROW_B), 16, b_voff[i],
                                                 (uint32_t)((W8 ? kt : stage_of(kt, rot)) * BK * 2), 0, 0);
    };
    // fp8 weight path (registers): thread t owns row t/4 (+128 i), chunks 2q, 2q+1 of the bf16 row
    const int brow = tid >> 2;
    uint32_t b_lds[2];
    const bool b_swap = W8 && ((brow >> 1) & 1);
    {
        int qd = tid & 3, sw = swz(brow), first = b_swap ? 1 : 0;
        b_lds[0] = (uint32_t)(brow * ROW_B + (((2 * qd + first) ^ sw) << 4));
        b_lds[1] = (uint32_t)(brow * ROW_B + (((2 * qd + 1 - first) ^ sw) << 4));
    }
    u32x4 rb[NB];
    float rs[2];
    auto load_b8 = [&](int i, uint32_t kofs) {
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)((SWIGLU && i >= NB / 2) ? b8m1 : b8m0), 0, -1, 0x00020000);
        return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, b8_voff[i], kofs, 0));
    };
    // Block scales come through buffer loads too, although their address is the same for every lane: as loads
    // through a pointer the compiler would be free to make them scalar loads, and the hand-written vmcnt
    // immediates below count them as vector-memory operations.
    auto load_scale = [&](gptr_f32 sc, int idx) {
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)(uintptr_t)sc, 0, -1, 0x00020000);
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, 0, idx * 4, 0));
    };
    auto gload_b = [&](int kt) {
        const size_t kofs = (size_t)kt * BK;
#pragma unroll
        for (int i = 0; i < NB; ++i) rb[i] = load_b8(i, (uint32_t)kofs);
        rs[0] = load_scale(sc0, srow0 + (kt >> 1));
        rs[1] = load_scale(sc1, srow1 + (kt >> 1));
    };
    auto store_b_all = [&](uint8_t* Bs) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            u32x4 l, h;
            dequant16(rb[i], rs[i / (NB / 2)], l, h);
            *reinterpret_cast<u32x4*>(Bs + b_lds[0] + i * RB * ROW_B) = b_swap ? h : l;
            *reinterpret_cast<u32x4*>(Bs + b_lds[1] + i * RB * ROW_B) = b_swap ? l : h;
        }
    };
    auto b_item = [&](int it, uint8_t* Bs, int kn) {   // it in 0 .. 2*NB-1: half it%2 of chunk it/2
        const int b = it >> 1, half = it & 1;
        const u32x4 o = dequant8(rb[b][2 * half], rb[b][2 * half + 1], rs[b / (NB / 2)]);
        *reinterpret_cast<u32x4*>(Bs + ((half ^ (b_swap ? 1 : 0)) ? b_lds[1] : b_lds[0]) + b * RB * ROW_B) = o;
        if (half == 1) {
            rb[b] = load_b8(b, (uint32_t)(kn * BK));
            if (b / (NB / 2) == 0) rs[0] = load_scale(sc0, srow0 + (kn >> 1));
            else rs[1] = load_scale(sc1, srow1 + (kn >> 1));
        }
    };

    const int frow = lane & 15, fquad = lane >> 4, fkey = swz(frow);
    const int fchunk = ((fquad & 1) << 1) | (fquad >> 1);
    constexpr int TM = 2 * MT, TN = 2 * NJ;
    uint32_t tok_off[TM], w_off[TN];
    fragment_rows<MT, TN, SWIGLU>(wm, wn, frow, tok_off, w_off);
    f32x4 acc[TM][TN];
    constexpr int TQ = MT / 2;
    constexpr int NP = TM / TQ;
    constexpr int NU = 2 * NP;
    bf16x8 wfr[2][TN], tq[2][TQ];
    auto read_w1 = [&](const uint8_t* Bs, int s, int j) {
        const uint32_t coff = (uint32_t)(((4 * s + fchunk) ^ fkey) << 4);
        wfr[s][j] = *reinterpret_cast<const bf16x8*>(Bs + w_off[j] + coff);
    };
    auto read_tq = [&](const uint8_t* As, int u) {
        const int s = u / NP, q = u % NP;
        const uint32_t coff = (uint32_t)(((4 * s + fchunk) ^ fkey) << 4);
#pragma unroll
        for (int i = 0; i < TQ; ++i) tq[u & 1][i] = *reinterpret_cast<const bf16x8*>(As + tok_off[q * TQ + i] + coff);
    };
    auto mfma_sub = [&](int u) {
        const int s = u / NP, q = u % NP;
#pragma unroll
        for (int i = 0; i < TQ; ++i)
#pragma unroll
            for (int jx = 0; jx < TN; ++jx) {
                const int j = ((i + u) & 1) ? TN - 1 - jx : jx;
                acc[q * TQ + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wfr[s][j], tq[u & 1][i], acc[q * TQ + i][j], 0, 0, 0);
            }
    };
    constexpr int WPS = TN / NP;
    // iteration kt multiplies stage par; the DMA brings k-stage ka (of the tile whose coordinates are current) into
    // the other token stage (and weight stage, bf16); fp8 converts the weight registers (k-stage kt+1) into the other
    // weight stage and refills them with k-stage kb
    // Vector-memory operations a wave issues per k-iteration AFTER its DMA of the next stage; they may stay in flight
    // at the iteration's barrier: the fp8 weight chunks (NB buffer loads) and their two block scales (buffer loads).
    constexpr int VM_TAIL = W8 ? NB + 2 : 0;
    auto iteration = [&](int kt, int ka, int kb, int par) {
        const uint8_t* rdA = par ? sA1 : sA0; const uint8_t* rdB = par ? sB1 : sB0;
        uint8_t* wrA = par ? sA0 : sA1; uint8_t* wrB = par ? sB0 : sB1;
#pragma unroll
        for (int v = 0; v < NU; ++v) {
            if (v < ND) {
                dma_a(wrA, ka, v);
                if (!W8) dma_b(wrB, ka, v);
            } else if (W8) {
                b_item(v - ND, wrB, kb);
            }
            if (!W8) __builtin_amdgcn_sched_barrier(0);
            if (v >= 2) mfma_sub(v - 2);
            else if (kt > 0) mfma_sub(NU - 2 + v);
            read_tq(rdA, v);
            if (v == 0) {
#pragma unroll
                for (int j = 0; j < TN; ++j) read_w1(rdB, 0, j);
            } else if (v >= 2 && v < 2 + NP) {
#pragma unroll
                for (int j = (v - 2) * WPS; j < (v - 1) * WPS; ++j) read_w1(rdB, 1, j);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // this wave's DMA has landed (the younger loads are the fp8 weight chunks and scales), then everybody's
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"(VM_TAIL) : "memory");
        __syncthreads();
    };
    static_assert(NU == 8 && ND == 4 && (!W8 || NB == 2), "slot plan");
    // ---- tiles ----
    setup(tile_of(slot));
    adopt();
#pragma unroll
    for (int i = 0; i < ND; ++i) { dma_a(sA0, 0, i); if (!W8) dma_b(sB0, 0, i); }
    if (W8) {
        gload_b(0);
        store_b_all(sB0);
        gload_b(1);
    }
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(VM_TAIL) : "memory");   // (all but gload_b(1)'s NB + 2 loads)
    __syncthreads();
    constexpr int CW = SWIGLU ? 8 * TN : 16 * TN;    // output columns of this wave
    for (;;) {
        const int out_row0 = row0, out_row_end = row_end, out_n0 = n0;
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[mi][j] = f32x4{0};
        bool more = false;
        for (int kt = 0; kt + 2 <= nk - 2; kt += 2) {
            iteration(kt, kt + 1, kt + 2, 0);
            iteration(kt + 1, kt + 2, kt + 3, 1);
        }
        slot += slots;
        more = tile_of(slot) < total;
        setup(tile_of(more ? slot : slot - slots));
        iteration(nk - 2, nk - 1, more ? 0 : nk - 1, 0);
        adopt();
        iteration(nk - 1, more ? 0 : nk - 1, more ? 1 : nk - 1, 1);
        mfma_sub(NU - 2);
        mfma_sub(NU - 1);

        // epilogue: stage 0 already holds the next tile; stage 1 is idle until the next tile's first iteration writes
        // it, so each wave transposes through its 8 KiB slice of stage 1 (64 or 128 rows at a time).  The lane id is
        // produced here, so that nothing derived from it stays live through the k loop.
        const int ncol0 = out_n0 + wn * CW;
        store_wave_outputs<MT, TN, SWIGLU, 8192 / (CW * 2), !SWIGLU>(
            acc, ((wave_s < 4) ? sA1 : sB1) + (wave_s & 3) * 8192, fresh_lane(),
            g.c + (size_t)(out_row0 + wm * 32 * MT) * N + ncol0, N, min(BM, out_row_end - out_row0) - wm * 32 * MT, N - ncol0);
        if (!more) return;
        __syncthreads();
    }
}

template <int WN, bool SWIGLU, bool W8>
int launch_tiles(const GemmArgs& g, int n_rows, hipStream_t st) {
    auto kern = grouped_gemm_kernel<WN, SWIGLU, W8>;
    // sum_e tiles_of(c_e) <= sum_e (c_e / 128 + 1); with the larger experts elsewhere, one tile per expert that has rows
    const long max_mtiles = g.cold_max <= 192 ? (g.pair_rows ? 2 : 1) * (long)(g.E < n_rows ? g.E : n_rows) : (long)n_rows / 128 + g.E;
    // (+ the persistent kernel's last tiles, less than a round of them, as two half tiles each)
    const long grid = ((max_mtiles * g.n_tiles_n + 2 * g.tail_cus + 31) / 32) * 32;   // whole rounds of 8 groups of 4 tiles
    if (grid > 0x7fffffffL) {
        set_error("grouped gemm: %ld workgroups exceed the grid limit", grid);
        return MOE_ERR_INVALID;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(128 * WN), 0, st, g);
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}

// CUs of the current device (the persistent kernel runs one workgroup on each)
inline int cu_count() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
        cached[dev] = n;
    }
    return cached[dev];
}

template <bool SWIGLU, bool W8>
int launch_persistent(const GemmArgs& g, int n_rows, hipStream_t st) {
    const long max_mtiles = (long)n_rows / 256 + g.E;
    long grid = ((max_mtiles * g.n_tiles_n + 7) / 8) * 8;
    const long ncu = (cu_count() / 8) * 8;
    if (grid > ncu) grid = ncu;
    hipLaunchKernelGGL((grouped_gemm_persistent_kernel<SWIGLU, W8>), dim3((unsigned)grid), dim3(512), 0, st, g);
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}

template <bool SWIGLU, bool W8>
int launch_mt(const GemmArgs& g0, int n_rows, hipStream_t st) {
    GemmArgs g = g0;
    const long mean = g.E > 0 ? (long)n_rows / g.E : 0;
    // the persistent kernel needs an even number of k-stages for its hand-over (fp8 sizes always have
    // one), keeps per-expert tables for up to 512 experts and addresses gathered rows with 32-bit offsets
    const bool fits = !g.row_map || g.a_bytes < (1ull << 32);
    // (below a mean of 128 rows an expert above one tile is rare and is cut into 128-row tiles where it occurs)
    if (mean < 128 || !(g.K % 128 == 0 && g.E <= 512 && fits && cu_count() >= 8)) {
        g.cold_max = 0x7fffffff;
        return launch_tiles<4, SWIGLU, W8>(g, n_rows, st);
    }
    // The counts themselves live on the device; only their mean is known here.  Both kernels are launched and every
    // expert goes by its own count: what fits one tile of the one-workgroup-per-tile kernel runs there, at its own
    // height and without 256-row padding, the rest on the persistent kernel's 256-row tiles.  A launch that finds
    // nothing of its kind costs a prefix scan per workgroup.  DeepSeek-V2-Lite, 4096 tokens (64 experts of
    // 0 ... 3989 rows, 47 of them below 193, whose 256-row tiles were 49 % padding): block step 0.923 -> 0.847 ms,
    // routed gate/up 0.395 -> 0.355 ms; DeepSeek-V2-236B, 32768 tokens: 11.48 -> 11.39 ms.
    // (The two launches on two streams, so that the second fills the CUs that the persistent kernel's last round
    // leaves idle, measured the same 0.36 ms: the launches stay on the caller's stream.)
    // fp8 weights: the rule is applied to what an expert's full 256-row tiles leave over.  A ragged
    // last tile costs the persistent kernel a full tile of MFMA time; the other kernel streams the expert's weights
    // once more for it, and fp8 weights are half the bytes.  DeepSeek-V3, 65536 tokens (256 experts of 581 ... 3941
    // rows, every second one with at most 128 rows over): block step 46.3 -> 45.8 ms, routed gate/up 25.2 -> 24.8,
    // down 12.9 -> 12.7 (with up to 64 or 96 rows over 46.2 - 46.3; with all, as two 128-row tiles, 47.1).  Up to 192
    // rows over, on the streamer form for 129 to 192 rows: the headline step stays (45.95 -> 45.85), DeepSeek-V3 at
    // 3584 / 4096 / 8192 tokens 4.53 -> 3.99, 4.64 -> 4.31, 7.50 -> 7.41 ms (at 4096 tokens 109 of the 256 experts hold
    // 129 to 192 rows, which were padded 256-row tiles).  With bf16
    // weights it is break-even (Mixtral-8x7B 9.28 -> 9.23 ms, DeepSeek-V2-236B 11.34 -> 11.42) and not done.
    // (Both launches at every mean: from 1536 rows per expert a small expert is rare, but the second launch is there
    // for the persistent kernel's last round anyway.)
    g.cold_max = 192;
    g.rem_split = W8 ? 1 : 0;
    g.pair_rows = W8 ? 0 : 1;
    // Last round of the persistent kernel (tail_tiles above): Mixtral-8x22B, 8192 tokens, down projection (6.4 rounds
    // of 0.4 ms) 2.82 -> 2.66 ms, step 8.31 -> 8.13; Mixtral-8x7B 9.39 -> 9.27 ms; DeepSeek-V2-Lite 0.855 -> 0.821 ms
    // (its shared expert's 128 down tiles become 256 half tiles: 0.071 -> 0.055 ms); DeepSeek-V2-236B 11.43 -> 11.46,
    // DeepSeek-V3 46.56 -> 46.54: short rounds gain nothing, a partial round of few CUs runs at a higher clock anyway.
    g.tail_cus = (cu_count() / 8) * 8;     // the persistent launch's grid when there is a round of tiles or more
    int rc = launch_persistent<SWIGLU, W8>(g, n_rows, st);
    if (rc != MOE_OK) return rc;
    return launch_tiles<4, SWIGLU, W8>(g, n_rows, st);
}

template <bool W8>
int grouped_swiglu(const void* x, int32_t x_rows, const int32_t* row_map, const void* const* w_gate, const void* const* w_up,
                   const void* const* w_down, const float* const* s_gate, const float* const* s_up,
                   const float* const* s_down, const int32_t* offsets, int32_t n_rows, int32_t n_experts,
                   int32_t hidden, int32_t inter, void* act, void* y, int32_t phases, void* stream, const char* who) {
    MOE_REQUIRE(n_rows >= 0, "%s: n_rows %d < 0", who, n_rows);
    MOE_REQUIRE(phases >= MOE_PHASE_GATE_UP && phases <= MOE_PHASE_BOTH, "%s: bad phases %d", who, phases);
    if (n_rows == 0) return MOE_OK;
    MOE_REQUIRE(x && w_gate && w_up && w_down && offsets && act && y, "%s: NULL pointer argument", who);
    MOE_REQUIRE(x_rows >= 1, "%s: x_rows %d < 1", who, x_rows);
    MOE_REQUIRE(!W8 || (s_gate && s_up && s_down), "%s: NULL scale pointer array", who);
    MOE_REQUIRE(n_experts >= 1 && n_experts <= MAX_E, "%s: n_experts %d outside [1,%d]", who, n_experts, MAX_E);
    const int align = W8 ? 128 : 64;
    MOE_REQUIRE(hidden > 0 && hidden % align == 0, "%s: hidden %d must be a positive multiple of %d", who, hidden, align);
    MOE_REQUIRE(inter > 0 && inter % align == 0, "%s: intermediate %d must be a positive multiple of %d", who, inter,
                align);
    hipStream_t st = as_stream(stream);
    GemmArgs g1{};
    g1.a = static_cast<const uint16_t*>(x);
    g1.row_map = row_map;
    g1.a_bytes = (size_t)x_rows * (size_t)hidden * 2;
    g1.a_rows = x_rows;
    g1.b0 = w_gate; g1.b1 = w_up; g1.s0 = s_gate; g1.s1 = s_up;
    g1.offsets = offsets;
    g1.c = static_cast<uint16_t*>(act);
    g1.E = n_experts; g1.K = hidden; g1.N = inter;
    g1.n_tiles_n = (inter + 127) / 128;
    if (phases & MOE_PHASE_GATE_UP) {
        int rc = launch_mt<true, W8>(g1, n_rows, st);
        if (rc != MOE_OK) return rc;
    }
    if (!(phases & MOE_PHASE_DOWN)) return MOE_OK;
    GemmArgs g2{};
    g2.a = static_cast<const uint16_t*>(act);
    g2.row_map = nullptr;
    g2.b0 = w_down; g2.b1 = nullptr; g2.s0 = s_down; g2.s1 = nullptr;
    g2.offsets = offsets;
    g2.c = static_cast<uint16_t*>(y);
    g2.E = n_experts; g2.K = inter; g2.N = hidden;
    g2.n_tiles_n = (hidden + 255) / 256;
    return launch_mt<false, W8>(g2, n_rows, st);
}

// out = bf16(f32(q) * scale[i/128, j/128]); one thread per 16 consecutive elements of a row
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ q, const float* __restrict__ scale,
                                                      int rows, int cols, uint16_t* __restrict__ out) {
    const int chunks = (cols + 15) / 16;
    const long id = (long)blockIdx.x * 256 + threadIdx.x;
    if (id >= (long)rows * chunks) return;
    const int r = (int)(id / chunks), c0 = (int)(id % chunks) * 16;
    const int nbc = (cols + 127) / 128;
    const float s = scale[(size_t)(r >> 7) * nbc + (c0 >> 7)];  // a 16-aligned run never crosses a 128 boundary
    const size_t base = (size_t)r * cols + c0;
    if (c0 + 16 <= cols && (base & 15) == 0) {
        u32x4 l, h;
        dequant16(*reinterpret_cast<const u32x4*>(q + base), s, l, h);
        *reinterpret_cast<u32x4*>(out + base) = l;
        *reinterpret_cast<u32x4*>(out + base + 8) = h;
    } else {
        for (int j = c0; j < cols && j < c0 + 16; ++j) {
            f32x2 f = __builtin_amdgcn_cvt_pk_f32_fp8((uint32_t)q[(size_t)r * cols + j], false);
            out[(size_t)r * cols + j] = (uint16_t)(pack_bf16(f[0] * s, 0.0f) & 0xffffu);
        }
    }
}

}  // namespace
}  // namespace moe

extern "C" size_t moe_grouped_workspace_bytes(int32_t, int32_t) { return 256; }

extern "C" int moe_grouped_swiglu_bf16(const void* x, int32_t x_rows, const int32_t* row_map, const void* const* w_gate,
                                       const void* const* w_up, const void* const* w_down, const int32_t* offsets,
                                       int32_t n_rows, int32_t n_experts, int32_t hidden, int32_t inter, void* act,
                                       void* y, int32_t phases, void*, size_t, void* stream) {
    return moe::grouped_swiglu<false>(x, x_rows, row_map, w_gate, w_up, w_down, nullptr, nullptr, nullptr, offsets, n_rows,
                                      n_experts, hidden, inter, act, y, phases, stream, "moe_grouped_swiglu_bf16");
}

extern "C" int moe_grouped_swiglu_w8a16(const void* x, int32_t x_rows, const int32_t* row_map, const void* const* w_gate,
                                        const void* const* w_up, const void* const* w_down,
                                        const float* const* s_gate, const float* const* s_up,
                                        const float* const* s_down, const int32_t* offsets, int32_t n_rows,
                                        int32_t n_experts, int32_t hidden, int32_t inter, void* act, void* y,
                                        int32_t phases, void*, size_t, void* stream) {
    return moe::grouped_swiglu<true>(x, x_rows, row_map, w_gate, w_up, w_down, s_gate, s_up, s_down, offsets, n_rows,
                                     n_experts, hidden, inter, act, y, phases, stream, "moe_grouped_swiglu_w8a16");
}

extern "C" int moe_dequant_fp8_block128(const void* q, const float* scale, int32_t rows, int32_t cols, void* out,
                                        void* stream) {
    using namespace moe;
    MOE_REQUIRE(rows >= 0 && cols >= 0, "moe_dequant_fp8_block128: negative shape %d x %d", rows, cols);
    if (rows == 0 || cols == 0) return MOE_OK;
    MOE_REQUIRE(q && scale && out, "moe_dequant_fp8_block128: NULL pointer argument");
    const long chunks = (long)rows * ((cols + 15) / 16);
    hipLaunchKernelGGL(dequant_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, as_stream(stream),
                       static_cast<const uint8_t*>(q), scale, rows, cols, static_cast<uint16_t*>(out));
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}
