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
// expert is cut into M tiles of BM rows (the last one partial); an M tile times an N tile
// of the weight matrix is one workgroup.  Every workgroup rebuilds the (tiny) M-tile
// prefix over experts in LDS from offsets[], so the launch needs neither a host sync nor
// a tile table: grid = upper bound on the tile count, surplus workgroups exit at once.
// Workgroup ids are dealt round-robin to the 8 XCDs by the hardware; the id is remapped
// so that each XCD owns a contiguous range of tiles (same expert, neighbouring M/N
// tiles), which is what makes its private L2 hold the A and B panels that are re-read.
//
// Workgroup = 4 waves (2 along M, 2 along N).  Per wave MT x 4 MFMA tiles of 32x32
// (v_mfma_f32_32x32x16_bf16), i.e. up to 128x128 outputs and 256 fp32 accumulators.
// K advances 64 at a time through a double-buffered LDS stage; rows are 128 bytes with a
// 16-byte-chunk XOR swizzle (chunk ^= row & 7) so that both the 16-byte stores and the
// 16-byte MFMA operand reads are bank-conflict free.  Global loads for stage k+2 are in
// flight while stage k is multiplied.
//
// The MFMA is issued with the WEIGHT fragment as srcA and the TOKEN fragment as srcB, so
// a lane ends up holding 4 consecutive output columns of one token row per register
// quad: the epilogue packs them into one 8-byte store.
#include "common.h"

namespace moe {
namespace {

constexpr int BK = 64;           // k per stage (bf16 elements); 128 bytes per LDS row
constexpr int ROW_B = 128;       // bytes per LDS row
constexpr int BN_ROWS = 256;     // weight rows per workgroup (128 gate + 128 up when SWIGLU)
constexpr int MAX_E = 1024;

typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    f32x2 f = {a, b};
    bf16x2 h = __builtin_convertvector(f, bf16x2);  // v_cvt_pk_bf16_f32: round to nearest even
    return __builtin_bit_cast(uint32_t, h);
}
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
    const void* const* b0;      // per-expert weight matrix [N, K] (gate when SWIGLU, else down)
    const void* const* b1;      // per-expert up matrix [N, K] (SWIGLU only)
    const float* const* s0;     // per-expert block scales of b0 (W8 only)
    const float* const* s1;     // per-expert block scales of b1 (W8, SWIGLU only)
    const int32_t* offsets;     // [E+1]
    uint16_t* c;                // output, row stride N, sorted-row order
    int E, K, N;
    int n_tiles_n;              // ceil(N / (SWIGLU ? 128 : 256))
};

template <int MT, bool SWIGLU, bool W8>
__global__ __launch_bounds__(256) void grouped_gemm_kernel(GemmArgs g) {
    constexpr int BM = 64 * MT;                 // rows per workgroup
    constexpr int A_STAGE = BM * ROW_B;         // bytes
    constexpr int B_STAGE = BN_ROWS * ROW_B;
    constexpr int NA = MT * 2;                  // 16-byte A chunks per thread per stage
    constexpr int NB = W8 ? 4 : 8;              // 16-byte global B chunks per thread per stage
    constexpr int NBLK = SWIGLU ? 128 : 256;    // output columns per workgroup
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ int s_pref[MAX_E + 1];
    __shared__ int s_wtot[4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;

    // ---- M-tile prefix over experts (exclusive scan of ceil(count/BM)) ----
    int run = 0;
    for (int e0 = 0; e0 < g.E; e0 += 256) {
        int e = e0 + tid;
        int mt = 0;
        if (e < g.E) mt = (g.offsets[e + 1] - g.offsets[e] + BM - 1) / BM;
        int inc = mt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            int o = __shfl_up(inc, d);
            if (lane >= d) inc += o;
        }
        if (lane == 63) s_wtot[wave] = inc;
        __syncthreads();
        int pre = run;
        for (int w = 0; w < wave; ++w) pre += s_wtot[w];
        if (e < g.E) s_pref[e] = pre + inc - mt;
        run += s_wtot[0] + s_wtot[1] + s_wtot[2] + s_wtot[3];
        __syncthreads();
    }
    if (tid == 0) s_pref[g.E] = run;
    __syncthreads();
    const int total = run * g.n_tiles_n;

    // ---- XCD-aware id: XCD x (= blockIdx % 8) owns tiles [x*per, (x+1)*per) ----
    const int per = (total + 7) / 8;
    const int slot = blockIdx.x >> 3;
    const int v = (blockIdx.x & 7) * per + slot;
    if (slot >= per || v >= total) return;
    const int q = v / g.n_tiles_n;  // global M-tile number
    int lo = 0, hi = g.E;           // find e with s_pref[e] <= q < s_pref[e+1]
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (s_pref[mid] <= q) lo = mid; else hi = mid;
    }
    const int e = lo;
    const int mt_e = s_pref[e + 1] - s_pref[e];
    const int local = v - s_pref[e] * g.n_tiles_n;
    const int n_tile = local / mt_e, m_tile = local - n_tile * mt_e;
    const int row0 = g.offsets[e] + m_tile * BM;
    const int row_end = g.offsets[e + 1];
    const int n0 = n_tile * NBLK;
    const int K = g.K, N = g.N;

    // ---- per-thread load coordinates ----
    const int lrow = tid >> 3, lchunk = tid & 7;          // bf16 tiles: row tid/8 (+32 i), chunk tid%8
    int a_src[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        int r = min(row0 + lrow + 32 * i, row_end - 1);
        a_src[i] = g.row_map ? g.row_map[r] : r;
    }
    const uint32_t a_lds = (uint32_t)(lrow * ROW_B + ((lchunk ^ (lrow & 7)) << 4));

    const uint8_t* bmat0 = static_cast<const uint8_t*>(g.b0[e]);
    const uint8_t* bmat1 = SWIGLU ? static_cast<const uint8_t*>(g.b1[e]) : bmat0;
    const float* sc0 = W8 ? g.s0[e] : nullptr;
    const float* sc1 = (W8 && SWIGLU) ? g.s1[e] : sc0;
    constexpr int EB = W8 ? 1 : 2;                        // bytes per weight element
    const int brow = W8 ? (tid >> 2) : (tid >> 3);        // fp8 tiles: row tid/4 (+64 i), 16-byte chunk tid%4
    const int bcol_b = W8 ? ((tid & 3) << 4) : ((tid & 7) << 4);  // byte offset inside the 64-element k slab
    constexpr int BSTEP = W8 ? 64 : 32;                   // row step between a thread's B chunks
    int b_n[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        int r = brow + BSTEP * i;                         // row inside the 256-row B tile
        int n = SWIGLU ? (n0 + (r & 127)) : (n0 + r);
        b_n[i] = min(n, N - 1);
    }
    uint32_t b_lds[2];
    if (W8) {
        int qd = tid & 3, sw = brow & 7;
        b_lds[0] = (uint32_t)(brow * ROW_B + (((2 * qd) ^ sw) << 4));
        b_lds[1] = (uint32_t)(brow * ROW_B + (((2 * qd + 1) ^ sw) << 4));
    } else {
        b_lds[0] = (uint32_t)(brow * ROW_B + (((tid & 7) ^ (brow & 7)) << 4));
        b_lds[1] = 0;
    }
    // block-scale rows (W8): first / second 128 rows of the B tile
    int srow0 = 0, srow1 = 0;
    const int KB = K >> 7;
    if (W8) {
        if (SWIGLU) { srow0 = (n0 >> 7) * KB; srow1 = srow0; }
        else        { srow0 = (n0 >> 7) * KB; srow1 = min((n0 >> 7) + 1, (N >> 7) - 1) * KB; }
    }

    u32x4 ra[NA], rb[NB];
    float rs[2] = {1.0f, 1.0f};
    auto gload = [&](int kt) {
        const size_t kofs = (size_t)kt * BK;
#pragma unroll
        for (int i = 0; i < NA; ++i)
            ra[i] = *reinterpret_cast<const u32x4*>(g.a + (size_t)a_src[i] * K + kofs + lchunk * 8);
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const uint8_t* m = (SWIGLU && i >= NB / 2) ? bmat1 : bmat0;  // rows >= 128 of the B tile are the up matrix
            rb[i] = *reinterpret_cast<const u32x4*>(m + ((size_t)b_n[i] * K + kofs) * EB + bcol_b);
        }
        if (W8) {
            rs[0] = sc0[srow0 + (kt >> 1)];
            rs[1] = sc1[srow1 + (kt >> 1)];
        }
    };
    auto lds_store = [&](int stage) {
        uint8_t* As = smem + stage * (A_STAGE + B_STAGE);
        uint8_t* Bs = As + A_STAGE;
#pragma unroll
        for (int i = 0; i < NA; ++i) *reinterpret_cast<u32x4*>(As + a_lds + i * 32 * ROW_B) = ra[i];
        if (W8) {
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                u32x4 l, h;
                dequant16(rb[i], rs[i >> 1], l, h);
                *reinterpret_cast<u32x4*>(Bs + b_lds[0] + i * 64 * ROW_B) = l;
                *reinterpret_cast<u32x4*>(Bs + b_lds[1] + i * 64 * ROW_B) = h;
            }
        } else {
#pragma unroll
            for (int i = 0; i < NB; ++i) *reinterpret_cast<u32x4*>(Bs + b_lds[0] + i * 32 * ROW_B) = rb[i];
        }
    };

    // ---- MFMA operand coordinates ----
    // fragment row = base + lane%32; logical chunk = 2*s + lane/32; swizzle key = lane%8
    const int frow = lane & 31, fhalf = lane >> 5, fkey = lane & 7;
    uint32_t tok_off[MT], w_off[4];
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) tok_off[mi] = (uint32_t)((wm * 32 * MT + 32 * mi + frow) * ROW_B);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int r = SWIGLU ? ((j < 2 ? 0 : 128) + wn * 64 + 32 * (j & 1)) : (wn * 128 + 32 * j);
        w_off[j] = (uint32_t)((r + frow) * ROW_B);
    }

    f32x16 acc[MT][4];
#pragma unroll
    for (int mi = 0; mi < MT; ++mi)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[mi][j] = f32x16{0};

    auto compute = [&](int stage) {
        const uint8_t* As = smem + stage * (A_STAGE + B_STAGE);
        const uint8_t* Bs = As + A_STAGE;
#pragma unroll
        for (int s = 0; s < BK / 16; ++s) {
            const uint32_t coff = (uint32_t)(((2 * s + fhalf) ^ fkey) << 4);
            bf16x8 tf[MT], wf[4];
#pragma unroll
            for (int mi = 0; mi < MT; ++mi) tf[mi] = *reinterpret_cast<const bf16x8*>(As + tok_off[mi] + coff);
#pragma unroll
            for (int j = 0; j < 4; ++j) wf[j] = *reinterpret_cast<const bf16x8*>(Bs + w_off[j] + coff);
#pragma unroll
            for (int mi = 0; mi < MT; ++mi)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[mi][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[j], tf[mi], acc[mi][j], 0, 0, 0);
        }
    };

    // ---- main loop ----
    const int nk = K / BK;
    gload(0);
    lds_store(0);
    if (nk > 1) gload(1);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) lds_store(cur ^ 1);
        if (kt + 2 < nk) gload(kt + 2);
        compute(cur);
        __syncthreads();
    }

    // ---- epilogue ----
    // acc[mi][j][i]: token row = 32*mi + lane%32 of the wave's M range; output column
    // = tile column base + 8*(i/4) + 4*(lane/32) + i%4.
    const int rows_here = min(BM, row_end - row0);
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) {
        const int ml = wm * 32 * MT + 32 * mi + frow;
        if (ml >= rows_here) continue;
        uint16_t* crow = g.c + (size_t)(row0 + ml) * N;
        if (SWIGLU) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    const int n = n0 + wn * 64 + 32 * j + 8 * qd + 4 * fhalf;
                    float o[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float gv = bf16r(acc[mi][j][4 * qd + i]);
                        float uv = bf16r(acc[mi][j + 2][4 * qd + i]);
                        float sg = bf16r(gv * __builtin_amdgcn_rcpf(1.0f + __expf(-gv)));
                        o[i] = sg * uv;
                    }
                    if (n < N) {
                        u32x2 pk = {pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3])};
                        *reinterpret_cast<u32x2*>(crow + n) = pk;
                    }
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    const int n = n0 + wn * 128 + 32 * j + 8 * qd + 4 * fhalf;
                    if (n < N) {
                        u32x2 pk = {pack_bf16(acc[mi][j][4 * qd], acc[mi][j][4 * qd + 1]),
                                    pack_bf16(acc[mi][j][4 * qd + 2], acc[mi][j][4 * qd + 3])};
                        *reinterpret_cast<u32x2*>(crow + n) = pk;
                    }
                }
            }
        }
    }
}

template <int MT, bool SWIGLU, bool W8>
int launch_one(const GemmArgs& g, int n_rows, hipStream_t st) {
    constexpr int BM = 64 * MT;
    constexpr int LDS = 2 * (BM * ROW_B + BN_ROWS * ROW_B);
    static bool attr_set = false;
    auto kern = grouped_gemm_kernel<MT, SWIGLU, W8>;
    if (!attr_set) {
        MOE_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        attr_set = true;
    }
    const long max_mtiles = (long)n_rows / BM + g.E;  // sum_e ceil(c_e/BM) <= n_rows/BM + E
    const long grid = ((max_mtiles * g.n_tiles_n + 7) / 8) * 8;
    if (grid > 0x7fffffffL) {
        set_error("grouped gemm: %ld workgroups exceed the grid limit", grid);
        return MOE_ERR_INVALID;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), LDS, st, g);
    MOE_HIP_CHECK(hipGetLastError());
    return MOE_OK;
}

template <bool SWIGLU, bool W8>
int launch_mt(const GemmArgs& g, int n_rows, hipStream_t st) {
    const long mean = g.E > 0 ? (long)n_rows / g.E : 0;
    if (mean >= 192) return launch_one<4, SWIGLU, W8>(g, n_rows, st);
    if (mean >= 96) return launch_one<2, SWIGLU, W8>(g, n_rows, st);
    return launch_one<1, SWIGLU, W8>(g, n_rows, st);
}

template <bool W8>
int grouped_swiglu(const void* x, const int32_t* row_map, const void* const* w_gate, const void* const* w_up,
                   const void* const* w_down, const float* const* s_gate, const float* const* s_up,
                   const float* const* s_down, const int32_t* offsets, int32_t n_rows, int32_t n_experts,
                   int32_t hidden, int32_t inter, void* act, void* y, int32_t phases, void* stream, const char* who) {
    MOE_REQUIRE(n_rows >= 0, "%s: n_rows %d < 0", who, n_rows);
    MOE_REQUIRE(phases >= MOE_PHASE_GATE_UP && phases <= MOE_PHASE_BOTH, "%s: bad phases %d", who, phases);
    if (n_rows == 0) return MOE_OK;
    MOE_REQUIRE(x && w_gate && w_up && w_down && offsets && act && y, "%s: NULL pointer argument", who);
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

extern "C" int moe_grouped_swiglu_bf16(const void* x, const int32_t* row_map, const void* const* w_gate,
                                       const void* const* w_up, const void* const* w_down, const int32_t* offsets,
                                       int32_t n_rows, int32_t n_experts, int32_t hidden, int32_t inter, void* act,
                                       void* y, int32_t phases, void*, size_t, void* stream) {
    return moe::grouped_swiglu<false>(x, row_map, w_gate, w_up, w_down, nullptr, nullptr, nullptr, offsets, n_rows,
                                      n_experts, hidden, inter, act, y, phases, stream, "moe_grouped_swiglu_bf16");
}

extern "C" int moe_grouped_swiglu_w8a16(const void* x, const int32_t* row_map, const void* const* w_gate,
                                        const void* const* w_up, const void* const* w_down,
                                        const float* const* s_gate, const float* const* s_up,
                                        const float* const* s_down, const int32_t* offsets, int32_t n_rows,
                                        int32_t n_experts, int32_t hidden, int32_t inter, void* act, void* y,
                                        int32_t phases, void*, size_t, void* stream) {
    return moe::grouped_swiglu<true>(x, row_map, w_gate, w_up, w_down, s_gate, s_up, s_down, offsets, n_rows,
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
