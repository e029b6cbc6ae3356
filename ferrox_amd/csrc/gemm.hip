// Matrix products  C[m, n] = sum_k A[m, k] * W[n, k]  (weights are [out, in] as
// the checkpoint stores them; ferrox-core/src/matmul.rs:5-8) with fused epilogues,
// for plain and for expert-grouped rows.
//
//  * bfloat16: MFMA 16x16x32 tiles, float32 accumulators.
//  * float32 : FMA in float32 only (no reduced-precision matrix mode).
//
// In both, one output element is accumulated over k in ascending order with a
// single accumulator, whatever the tile shape and whatever else is in the batch,
// so a row's result does not depend on how many rows are computed with it.
//
// Grouped mode: rows are sorted by expert; expert e owns rows
// [expert_offsets[e], expert_offsets[e+1]) and the weights at W + e * w_stride.
// Dual mode: two weight matrices (gate, up) are multiplied at once and the
// epilogue stores silu(gate) * up  (ferrox-moe/src/lib.rs:655-658).
#include "common.h"
#include <type_traits>
#include <utility>

FX_DEFINE_LAST_ERROR()

enum { EPI_STORE = 0, EPI_STORE_F32 = 1, EPI_RESID = 2, EPI_GATED = 3 };

struct GemmArgs {
    const void* A;
    long lda;
    const void* W;
    long w_stride;      // elements between experts (grouped)
    long up_offset;     // elements from the gate matrix to the up matrix (dual)
    long kb_stride;     // 0: rows of W are K long.  Else W is stored [K/64][rows][64] (64 k of every row, then the
                        // next 64 k of every row, ...) and this is rows * 64, the elements between two such slabs
    const void* bias;   // [N] or null
    int bias_dtype;
    void* C;
    long ldc;
    const float* row_scale;  // [M] or null, multiplies the product before it is added (EPI_RESID)
    const int* a_rows;       // [M] or null: row of A to read for logical row m
    const int* c_rows;       // [M] or null: row of C to write for logical row m
    const int* expert_offsets;  // [E+1] or null
    const int* pair_ids;        // few rows, unsorted: expert of logical row ("pair") m, instead of expert_offsets
    int pair_div;               //   pair m reads row m / pair_div of A and writes row m of C
    int n_always, always_rows;  //   experts E .. E+n_always-1 take rows 0 .. always_rows-1 each: their tile s writes rows
    int always_from_a;          //   M + s*always_rows + t of C and reads row t of A (1) or that same row of A (0)
    int E;
    int M, N, K;
    const void* norm_w;  // skinny bf16 kernel only: A is the float32 residual stream and RMSNorm with these weights
    int norm_dtype;      //   is applied on the way in; norm_w is [K]
    float norm_eps;
    const float* row_ss; // skinny bf16 kernel only: row m of the product is scaled by rsqrt(sum(row_ss[m][0..row_ss_n)) / K + norm_eps)
    int row_ss_n;        //   (the rows of A are x * w of an RMSNorm whose scale is still to come)
    // skinny bf16 kernel, rope epilogue: C is [M, (nh + 2 nkv) * hd], queries | keys | values of token m at position
    // positions[m] of sequence token_seq[m].  Queries are rotated and stored in C; keys are rotated and stored in their
    // page, values in theirs (transposed), nothing of either in C.  Split-half pairs (i, i + rot/2), angle
    // pos * theta^(-2i/rot) (ferrox-core/src/attention.rs:20-32); the product is rounded to bfloat16 before it is
    // rotated, as when the rotation is a kernel of its own.
    const int* rope_positions;
    const int* rope_token_seq;
    const int* rope_table;
    int rope_max_blocks;
    void* rope_k_pages;     // null: nothing is written to pages (a layer that reads another's cache)
    void* rope_v_pages;
    int rope_nh, rope_nkv, rope_hd, rope_bs, rope_rot;
    const float* rope_inv_freq;       // rot/2 floats: pair i turns by (float)pos * rope_inv_freq[i]
    const float* rope_freq_factors;   // rot/2 floats or null: the angle of pair i is divided by rope_freq_factors[i]
    int stream_w;  // tiled kernel: the weights are read about once (one row tile a weight matrix): load them non-temporal
    int act;     // EPI_GATED: which activation the gate goes through (ACT_*)
    int vec_ok;  // 16-byte loads are legal for A and W
    int n_col_tiles, n_row_tiles;  // tiled kernels: the grid they decode block ids with
};

// block -> (first logical row, end of rows, expert).  Plain: tiles of TM rows.
// Grouped: expert e has ceil(rows_e / TM) tiles, in the order of the experts; a tile past the
// last one gets r0 = -1.  Every wave finds its tile by itself, 64 experts at a time: each lane
// takes one expert's bounds, a scan over the lanes gives the tiles before it, and the lane whose
// range holds the tile tells the others.  (One load's latency instead of one per expert.)
template <int TM>
__device__ __forceinline__ void locate_rows(const GemmArgs& g, int tile, int& r0, int& r_end, int& expert) {
    if (!g.expert_offsets) {
        r0 = tile * TM;
        r_end = g.M;
        expert = 0;
        if (r0 >= g.M) r0 = -1;
        return;
    }
    const int lane = threadIdx.x & 63;
    int before = 0;
    r0 = -1;
    r_end = 0;
    expert = 0;
    for (int base = 0; base < g.E; base += 64) {
        const int e = base + lane;
        const int b = e < g.E ? g.expert_offsets[e] : 0, en = e < g.E ? g.expert_offsets[e + 1] : 0;
        const int nt = (en - b + TM - 1) / TM;
        const int incl = wave_inclusive_sum(nt);
        const int first = before + incl - nt;
        const unsigned long long hit = __ballot(tile >= first && tile < first + nt);
        if (hit) {      // (the same in every lane: what the owner knows is read from its lane, no exchange)
            const int src = __builtin_amdgcn_readfirstlane(__ffsll((long long)hit) - 1);
            r0 = __builtin_amdgcn_readlane(b + (tile - first) * TM, src);
            r_end = __builtin_amdgcn_readlane(en, src);
            expert = base + src;
            return;
        }
        before += __builtin_amdgcn_readlane(incl, 63);
    }
}

// lanes (of the 64 of a wave) whose `e` equals this lane's; e < 2^bits, e < 0 matches nothing
__device__ __forceinline__ unsigned long long same_expert_lanes(int e, int bits) {
    unsigned long long m = __ballot(e >= 0);
    for (int b = 0; b < bits; ++b) {
        const unsigned long long set = __ballot((e >> b) & 1);
        m &= ((e >> b) & 1) ? set : ~set;
    }
    return e >= 0 ? m : 0ull;
}

// Up to 64 unsorted pairs: the experts that occur, in the order of their first pairs, get one tile per 16 of
// their pairs, and a tile's rows are those pairs in their order.  Every wave works this out by itself from the
// ids (a lane per pair) with ballots and counts alone: a lane that holds an expert's first pair counts the tiles
// of the first pairs in the lanes below it (an expert has one to four tiles, so four ballots), and what the tile's
// owner knows is read from its lane directly.  (A loop over the experts that occur, two exchanges between lanes
// each, cost a wave 1-2 us before its first load.)  After those tiles come the experts that every row takes
// (n_always of them, a shared expert cut into pieces), one tile each.  Returns false for a tile past the last one;
// else the expert, and for tile row lane % 16 the rows of A and C (or -1).
__device__ __forceinline__ bool locate_pairs(const GemmArgs& g, int tile, int& expert, int& a_row, int& c_row) {
    const int lane = threadIdx.x & 63, li = lane & 15;
    int e = lane < g.M ? g.pair_ids[lane] : -1;
    if (e >= g.E) e = -1;
    int bits = 0;
    while ((1 << bits) < g.E) ++bits;
    const unsigned long long same = same_expert_lanes(e, bits);
    const bool first = e >= 0 && lane == __ffsll((long long)same) - 1;
    const int my_tiles = (__popcll(same) + 15) >> 4;
    const unsigned long long below = (1ull << lane) - 1;
    int before = 0, total = 0;      // tiles of the experts whose first pair comes earlier than this lane's; of all
#pragma unroll
    for (int t = 1; t <= 4; ++t) {
        const unsigned long long f = __ballot(first && my_tiles >= t);
        before += __popcll(f & below);
        total += __popcll(f);
    }
    a_row = c_row = -1;
    if (tile >= total) {
        const int s = tile - total;
        if (s >= g.n_always) return false;
        expert = g.E + s;
        if (li < g.always_rows) {
            c_row = g.M + s * g.always_rows + li;
            a_row = g.always_from_a ? li : c_row;
        }
        return true;
    }
    const unsigned long long sel = __ballot(first && tile >= before && tile < before + my_tiles);
    const int src = __builtin_amdgcn_readfirstlane(__ffsll((long long)sel) - 1);
    expert = __builtin_amdgcn_readlane(e, src);
    const int skip = (tile - __builtin_amdgcn_readlane(before, src)) * 16;      // pairs of this expert in its earlier tiles
    unsigned long long rows = ((unsigned long long)(unsigned)__builtin_amdgcn_readlane((int)(same >> 32), src) << 32) |
                              (unsigned)__builtin_amdgcn_readlane((int)(unsigned)same, src);
    int mine = -1;                  // pair number skip + li of this expert, if it has so many
    for (int j = 0; j < skip + 16 && rows; ++j) {
        const int p = __ffsll((long long)rows) - 1;
        rows &= rows - 1;
        if (j == skip + li) mine = p;
    }
    if (mine >= 0) {
        c_row = mine;
        a_row = mine / g.pair_div;
    }
    return true;
}

// The gated epilogue stores act(gate) * up; `act` is a parameter of the call (GemmArgs::act), uniform over the
// launch, so another gated feed-forward needs no other kernel.
//   ACT_SILU       x / (1 + exp(-x))                               (ferrox-core/src/matmul.rs:268-270)
//   ACT_GELU_TANH  0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))
//   ACT_GELU       0.5 x (1 + erf(x / sqrt(2)))
//   ACT_RELU       max(x, 0)
enum { ACT_SILU = 0, ACT_GELU_TANH = 1, ACT_GELU = 2, ACT_RELU = 3, ACT_COUNT = 4 };
__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
template <int ACT>
__device__ __forceinline__ float gated_c(float gate, float up) {
    float a;
    if constexpr (ACT == ACT_GELU_TANH) a = 0.5f * gate * (1.0f + tanhf(0.7978845608028654f * (gate + 0.044715f * gate * gate * gate)));
    else if constexpr (ACT == ACT_GELU) a = 0.5f * gate * (1.0f + erff(gate * 0.7071067811865476f));
    else if constexpr (ACT == ACT_RELU) a = fmaxf(gate, 0.0f);
    else a = silu_f(gate);
    return a * up;
}
// f(the activation as a compile-time constant): an epilogue calls this once around its loops, so that the choice is
// one jump per block and not work inside the loops (left inside, the compiler works out every activation for every
// element and picks one: the tiled products of a prompt were 4-10 % slower for it)
template <typename F>
__device__ __forceinline__ void with_activation(int act, F&& f) {
    switch (act) {
        case ACT_GELU_TANH: f(std::integral_constant<int, ACT_GELU_TANH>{}); break;
        case ACT_GELU: f(std::integral_constant<int, ACT_GELU>{}); break;
        case ACT_RELU: f(std::integral_constant<int, ACT_RELU>{}); break;
        default: f(std::integral_constant<int, ACT_SILU>{}); break;
    }
}

// ===========================================================================
// bfloat16 on MFMA
// ===========================================================================
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define BK 64
#define LDS_STRIDE (BK + 8)  // bf16 elements; keeps 16-byte reads of 16 rows on distinct banks

template <bool VEC>   // VEC: K is a multiple of 8 and rows are 16-byte aligned
__device__ __forceinline__ uint4 load_chunk(const bf16* row, int k, int K) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (!row || k >= K) return v;
    if (VEC) return *(const uint4*)(row + k);
    uint16_t tmp[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) tmp[i] = (k + i < K) ? row[k + i].bits : (uint16_t)0;
    v.x = tmp[0] | ((uint32_t)tmp[1] << 16);
    v.y = tmp[2] | ((uint32_t)tmp[3] << 16);
    v.z = tmp[4] | ((uint32_t)tmp[5] << 16);
    v.w = tmp[6] | ((uint32_t)tmp[7] << 16);
    return v;
}

// TM x TN block tile (TN counts weight rows: in dual mode half of them are gate
// rows and half up rows, interleaved in groups of 16), 4 waves of WM x WN.
template <int TM, int TN, int WM, int WN, bool DUAL, int EPI, bool VEC>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(GemmArgs g) {
    constexpr int WAVES_N = TN / WN;
    static_assert((TM / WM) * WAVES_N == 4, "four waves per block");
    constexpr int MT = WM / 16, NT = WN / 16;
    constexpr int NA = (TM * 8 + 255) / 256, NB = (TN * 8 + 255) / 256;
    constexpr int OUT_TN = DUAL ? TN / 2 : TN;
    __shared__ __attribute__((aligned(16))) bf16 As[TM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) bf16 Bs[TN * LDS_STRIDE];

    // Blocks go to the 8 XCDs in turn (block b runs on XCD b % 8), each with an L2 of its own: the
    // tiles are dealt out so that an XCD works through a contiguous range of column tiles, rows
    // fastest, and the weights of those columns stay in its L2.
    const int per_xcd = (g.n_col_tiles * g.n_row_tiles + 7) / 8;
    const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (logical >= g.n_col_tiles * g.n_row_tiles) return;
    int r0, r_end, expert;
    locate_rows<TM>(g, logical % g.n_row_tiles, r0, r_end, expert);
    if (r0 < 0) return;
    const int n0 = (logical / g.n_row_tiles) * OUT_TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const bf16* Abase = (const bf16*)g.A;
    const bf16* Wbase = (const bf16*)g.W + (size_t)expert * g.w_stride;

    // the row each of this thread's chunks comes from stays the same for all k
    const bf16* a_src[NA];
    const bf16* b_src[NB];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const int c = tid + i * 256, row = c >> 3;
        a_src[i] = nullptr;
        if (c < TM * 8 && r0 + row < r_end) {
            const int m = r0 + row;
            a_src[i] = Abase + (size_t)(g.a_rows ? g.a_rows[m] : m) * g.lda;
        }
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int c = tid + i * 256, row = c >> 3;
        b_src[i] = nullptr;
        if (c < TN * 8) {
            if (DUAL) {
                const int col = n0 + (row >> 5) * 16 + (row & 15);
                if (col < g.N) b_src[i] = Wbase + (size_t)col * g.K + (((row >> 4) & 1) ? g.up_offset : 0);
            } else {
                if (n0 + row < g.N) b_src[i] = Wbase + (size_t)(n0 + row) * g.K;
            }
        }
    }

    f32x4_t acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

    // Two tiles are on their way from memory into registers while a third is multiplied out of LDS.
    uint4 a0[NA], b0[NB], a1[NA], b1[NB];
    const int kc = (tid & 7) * 8;
#define FX_FETCH(AR, BR, K0)                                                                  \
    {                                                                                         \
        _Pragma("unroll") for (int i = 0; i < NA; ++i) AR[i] = load_chunk<VEC>(a_src[i], (K0) + kc, g.K); \
        _Pragma("unroll") for (int i = 0; i < NB; ++i) BR[i] = load_chunk<VEC>(b_src[i], (K0) + kc, g.K); \
    }
#define FX_STAGE(AR, BR)                                                                      \
    {                                                                                         \
        _Pragma("unroll") for (int i = 0; i < NA; ++i) {                                      \
            const int c = tid + i * 256;                                                      \
            if (c < TM * 8) *(uint4*)(As + (c >> 3) * LDS_STRIDE + kc) = AR[i];               \
        }                                                                                     \
        _Pragma("unroll") for (int i = 0; i < NB; ++i) {                                      \
            const int c = tid + i * 256;                                                      \
            if (c < TN * 8) *(uint4*)(Bs + (c >> 3) * LDS_STRIDE + kc) = BR[i];               \
        }                                                                                     \
    }
#define FX_MULTIPLY()                                                                         \
    _Pragma("unroll") for (int ks = 0; ks < BK / 32; ++ks) {                                  \
        const int koff = ks * 32 + (lane >> 4) * 8;                                           \
        bf16x8_t af[MT], bfr[NT];                                                             \
        _Pragma("unroll") for (int i = 0; i < MT; ++i)                                        \
            af[i] = *(const bf16x8_t*)(As + (wm * WM + i * 16 + (lane & 15)) * LDS_STRIDE + koff); \
        _Pragma("unroll") for (int j = 0; j < NT; ++j)                                        \
            bfr[j] = *(const bf16x8_t*)(Bs + (wn * WN + j * 16 + (lane & 15)) * LDS_STRIDE + koff); \
        _Pragma("unroll") for (int i = 0; i < MT; ++i)                                        \
            _Pragma("unroll") for (int j = 0; j < NT; ++j)                                    \
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0); \
    }
    FX_FETCH(a0, b0, 0);
    FX_FETCH(a1, b1, BK);          // beyond K this loads zeros
    for (int k0 = 0; k0 < g.K; k0 += 2 * BK) {
        lds_barrier();  // the previous tile has been read
        FX_STAGE(a0, b0);
        lds_barrier();
        FX_FETCH(a0, b0, k0 + 2 * BK);
        FX_MULTIPLY();
        lds_barrier();
        FX_STAGE(a1, b1);           // a tile of zeros if K ends before it
        lds_barrier();
        FX_FETCH(a1, b1, k0 + 3 * BK);
        FX_MULTIPLY();
    }
#undef FX_FETCH
#undef FX_STAGE
#undef FX_MULTIPLY

    // epilogue: lane holds rows 4*(lane/16)+r, column lane%16 of each 16x16 tile
    float bias_v[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) bias_v[j] = 0.f;
    if (!DUAL && g.bias) load_strided_as_float<NT, 16>(g.bias, g.bias_dtype, n0 + wn * WN + (lane & 15), g.N, bias_v);
    if constexpr (DUAL) {
        with_activation(g.act, [&](auto ac) {
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int ml = r0 + wm * WM + i * 16 + (lane >> 4) * 4 + r;
                    if (ml >= r_end) continue;
                    const int m = g.c_rows ? g.c_rows[ml] : ml;
#pragma unroll
                    for (int j = 0; j < NT; j += 2) {
                        const int n = n0 + wn * (WN / 2) + (j / 2) * 16 + (lane & 15);
                        if (n < g.N)
                            from_float((bf16*)g.C + (size_t)m * g.ldc + n, gated_c<decltype(ac)::value>(acc[i][j][r], acc[i][j + 1][r]));
                    }
                }
        });
        return;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int ml = r0 + wm * WM + i * 16 + (lane >> 4) * 4 + r;
            if (ml >= r_end) continue;
            const int m = g.c_rows ? g.c_rows[ml] : ml;
            {
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const int n = n0 + wn * WN + j * 16 + (lane & 15);
                    if (n >= g.N) continue;
                    float v = acc[i][j][r];
                    if (g.bias) v += bias_v[j];
                    if (EPI == EPI_STORE) {
                        from_float((bf16*)g.C + (size_t)m * g.ldc + n, v);
                    } else if (EPI == EPI_STORE_F32) {
                        ((float*)g.C)[(size_t)m * g.ldc + n] = v;
                    } else {
                        if (g.row_scale) v *= g.row_scale[ml];
                        ((float*)g.C)[(size_t)m * g.ldc + n] += v;
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Many rows, K a multiple of 64: tiles of up to 256 rows x TN weight rows, eight
// waves.  K advances in steps of 64 through a ring of NS stages in LDS; tiles
// travel from global memory straight into LDS (no registers in between), NS-1
// steps ahead of their use, and one barrier per step separates the waves that
// still read a stage from the loads that refill it.  A wave-load fills 1 KB of
// LDS, 8 rows of 64 k; inside a row the eight 16-byte chunks are stored at
// chunk ^ ((row / 2) % 8), which the loading lanes achieve by choosing which
// chunk they fetch, so that the 16 rows an MFMA operand reads fall on distinct
// banks without padding.  Waves form a 2 x 4 grid: a wave owns TN/4 weight rows
// and every second block of 16 rows (so a tile with few rows, an expert's share,
// still spreads over both halves, and the two waves of a SIMD are one of each
// half); row blocks past the tile's rows are not multiplied.  The rows' ring may
// be shallower than the weights' (NSA < NS): weights come from memory and are
// read once, so more of them are kept on their way.
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(1))) const void* fx_global_ptr;
typedef __attribute__((address_space(3))) void* fx_lds_ptr;

template <int... Is, typename F>
__device__ __forceinline__ void static_for(std::integer_sequence<int, Is...>, F&& f) {
    (f(std::integral_constant<int, Is>{}), ...);
}

template <int N>
__device__ __forceinline__ void wait_loads_but() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// The K loop of one wave for NA active row blocks (blocks wm, wm+2, ... of the tile).
template <int NA, int MT, int NT, int TM, int TN, int NSA, int NSB, bool STREAM>
__device__ __forceinline__ void wide_k_loop(f32x4_t (&acc)[MT][NT], const bf16* const (&a_src)[TM / 64],
                                            const bf16* const (&b_src)[TN / 64], bf16* stages, int K, int wave,
                                            int a_off, int b_off, int sw, int kq, long kb_stride) {
    static_assert(NSA >= 2 && NSB >= NSA, "the weights' ring is at least as deep as the rows'");
    const int koff0 = (kq ^ sw) * 8, koff1 = ((4 + kq) ^ sw) * 8;
    constexpr int NLA = TM / 64, NLB = TN / 64;     // wave-loads per wave and step
    bf16* const ring_b = stages + NSA * TM * 64;
    const int nk = K >> 6;
    // past the end: a tile nobody reads, so that the counts of loads in flight stay even
    auto issue_a = [&](int kt) {
        const int k0 = min(kt, nk - 1) << 6;
        bf16* st = stages + (kt % NSA) * (TM * 64);
#pragma unroll
        for (int i = 0; i < NLA; ++i)
            __builtin_amdgcn_global_load_lds((fx_global_ptr)(a_src[i] + k0), (fx_lds_ptr)(st + (wave + 8 * i) * 512), 16, 0, 0);
    };
    auto issue_b = [&](int kt) {
        const size_t w0 = kb_stride ? (size_t)min(kt, nk - 1) * kb_stride : (size_t)(min(kt, nk - 1) << 6);
        bf16* st = ring_b + (kt % NSB) * (TN * 64);
#pragma unroll
        for (int i = 0; i < NLB; ++i) {
            // weights that nothing reads twice come with the non-temporal hint (cache policy operand 2): each
            // load takes whole 128-byte lines that need no place in the caches, and memory delivers them up to a
            // tenth faster.  A compile-time choice: as a flag tested here the tiled products of a prompt, which
            // do not stream, were 3-4 % slower.
            __builtin_amdgcn_global_load_lds((fx_global_ptr)(b_src[i] + w0), (fx_lds_ptr)(st + (wave + 8 * i) * 512), 16, 0, STREAM ? 2 : 0);
        }
    };
    // Each step issues the rows of step kt + NSA - 1, then the weights of step kt + NSB - 1.  Weights come from
    // memory and nothing reads them twice, so their ring may be deeper: more of them are on their way at a time.
#pragma unroll
    for (int p = 0; p < NSB - 1; ++p) {
        if (p >= NSB - NSA) issue_a(p - (NSB - NSA));
        issue_b(p);
    }
    for (int kt = 0; kt < nk; ++kt) {
        // this wave's part of step kt has landed: what may still be on its way are the loads of the NSA - 2
        // steps issued since the rows of step kt, and the weights issued right after those rows
        wait_loads_but<(NSA - 2) * (NLA + NLB) + (NSB > NSA ? NLB : 0)>();
        __builtin_amdgcn_s_barrier();          // ... everyone's has, and the stages of step kt-1 are free
        issue_a(kt + NSA - 1);
        issue_b(kt + NSB - 1);
        const bf16* base_a = stages + (kt % NSA) * (TM * 64);
        const bf16* base_b = ring_b + (kt % NSB) * (TN * 64);
        // 2*NA units of one operand of rows against NT operands of weights; the rows' operands are
        // read from LDS a few units ahead of the products that use them
        constexpr int U = 2 * NA, D = U > 3 ? 3 : U - 1;
        bf16x8_t bfr[2][NT], fr[U];
#pragma unroll
        for (int j = 0; j < NT; ++j) bfr[0][j] = *(const bf16x8_t*)(base_b + b_off + j * 16 * 64 + koff0);
#pragma unroll
        for (int u = 0; u < D; ++u)
            fr[u] = *(const bf16x8_t*)(base_a + a_off + (u % NA) * 32 * 64 + ((u / NA) ? koff1 : koff0));
        static_for(std::make_integer_sequence<int, U>{}, [&](auto uc) {
            constexpr int u = decltype(uc)::value;
            if constexpr (u + D < U)
                fr[u + D] = *(const bf16x8_t*)(base_a + a_off + ((u + D) % NA) * 32 * 64 + (((u + D) / NA) ? koff1 : koff0));
            if constexpr (u == 0) {
#pragma unroll
                for (int j = 0; j < NT; ++j) bfr[1][j] = *(const bf16x8_t*)(base_b + b_off + j * 16 * 64 + koff1);
            }
            __builtin_amdgcn_sched_barrier(0);      // the reads above stay ahead of the products below
#pragma unroll
            for (int j = 0; j < NT; ++j)
                acc[u % NA][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fr[u], bfr[u / NA][j], acc[u % NA][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
    }
    wait_loads_but<0>();                       // the loads past the end, before the block leaves
}

template <int TMB, int TN, int NS, bool DUAL, int EPI, int NSA = NS, bool STREAM = false>
__global__ __launch_bounds__(512) void gemm_bf16_wide_kernel(GemmArgs g) {
    constexpr int TM = TMB * 16;
    constexpr int MT = TMB / 2;            // row blocks per wave
    constexpr int NT = TN / 64;            // 16-row blocks of W per wave
    constexpr int WN = TN / 4;
    constexpr int OUT_TN = DUAL ? TN / 2 : TN;
    constexpr int NLA = TM / 64, NLB = TN / 64;   // wave-loads (8 rows each) per wave and K step
    static_assert(TM % 64 == 0 && TN % 64 == 0, "eight waves load 64 rows at a time");
    __shared__ __attribute__((aligned(1024))) bf16 stages[(NSA * TM + NS * TN) * 64];    // the rows' ring, then the weights'

    // Blocks go to the 8 XCDs in turn (block b runs on XCD b % 8), each with an L2 of its own.  Plain: an XCD
    // works through a contiguous range of the tiles in an order that keeps neighbours in rows and columns
    // together, so the operands of the tiles it has at a time stay in its L2.  Grouped: XCD x takes the row tiles x, x + 8, ... and runs through the column tiles of each, so an
    // expert's rows are fetched once and stay in its L2 while its weights, which nothing reads twice, stream by
    // (the row tiles past the last expert are empty; dealing them out in turn spreads them over the XCDs).
    int row_tile, col_tile;
    if (g.expert_offsets) {
        const int i = blockIdx.x / 8;
        row_tile = (i / g.n_col_tiles) * 8 + blockIdx.x % 8;
        col_tile = i % g.n_col_tiles;
        if (row_tile >= g.n_row_tiles) return;
    } else {
        const int per_xcd = (g.n_col_tiles * g.n_row_tiles + 7) / 8;
        const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
        if (logical >= g.n_col_tiles * g.n_row_tiles) return;
        // bands of 8 row tiles, rows fastest inside a band: the 32 tiles that an XCD works on at a time are
        // 8 rows x 4 columns, so 12 operand tiles serve 32 products
        const int band = logical / (8 * g.n_col_tiles), rem = logical % (8 * g.n_col_tiles);
        const int band_rows = min(8, g.n_row_tiles - band * 8);
        row_tile = band * 8 + rem % band_rows;
        col_tile = rem / band_rows;
    }
    int r0, r_end, expert;
    locate_rows<TM>(g, row_tile, r0, r_end, expert);
    if (r0 < 0) return;
    const int n0 = col_tile * OUT_TN;
    const int rows_here = min(TM, r_end - r0);
    const int nblk = (rows_here + 15) >> 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // waves w and w + 4 share a SIMD: one of each half of the rows, so that a tile with few rows loads the SIMDs evenly
    const int wm = wave >> 2, wn = wave & 3;
    const bf16* Wbase = (const bf16*)g.W + (size_t)expert * g.w_stride;

    // what this lane fetches in each of its wave-loads: row 8*j + lane/8 of the tile, chunk (lane%8) ^ ((row/2)%8)
    const bf16* a_src[NLA];
    const bf16* b_src[NLB];
#pragma unroll
    for (int i = 0; i < NLA; ++i) {
        const int j = wave + 8 * i, row = 8 * j + (lane >> 3);
        const int chunk = (lane & 7) ^ (4 * (j & 1) + (lane >> 4));
        const int m = r0 + min(row, rows_here - 1);          // rows past the end repeat the last one, unused
        a_src[i] = (const bf16*)g.A + (size_t)(g.a_rows ? g.a_rows[m] : m) * g.lda + chunk * 8;
    }
#pragma unroll
    for (int i = 0; i < NLB; ++i) {
        const int j = wave + 8 * i, row = 8 * j + (lane >> 3);
        const int chunk = (lane & 7) ^ (4 * (j & 1) + (lane >> 4));
        int col = DUAL ? n0 + (row >> 5) * 16 + (row & 15) : n0 + row;
        col = min(col, g.N - 1);
        const bool up = DUAL && ((row >> 4) & 1);
        b_src[i] = g.kb_stride ? Wbase + ((size_t)col + (up ? g.up_offset / g.K : 0)) * 64 + chunk * 8
                               : Wbase + (size_t)col * g.K + (up ? g.up_offset : 0) + chunk * 8;
    }

    f32x4_t acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

    const int sw = (lane & 15) >> 1, kq = lane >> 4;
    const int a_off = (wm * 16 + (lane & 15)) * 64, b_off = (wn * WN + (lane & 15)) * 64;
    const int na = (nblk - wm + 1) >> 1;         // this wave's active row blocks
#define FX_LOOP(NA) \
    wide_k_loop<NA, MT, NT, TM, TN, NSA, NS, STREAM>(acc, a_src, b_src, stages, g.K, wave, a_off, b_off, sw, kq, g.kb_stride)
    if constexpr (MT >= 4) {
        if (na > 3 * MT / 4) FX_LOOP(MT);
        else if (na > MT / 2) FX_LOOP(3 * MT / 4);
        else if (na > MT / 4) FX_LOOP(MT / 2);
        else FX_LOOP(MT / 4);
    } else {
        if (na > MT / 2) FX_LOOP(MT);
        else FX_LOOP((MT + 1) / 2);
    }
#undef FX_LOOP

    // epilogue: lane holds rows 4*(lane/16)+r, column lane%16 of each 16x16 tile
    float bias_v[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) bias_v[j] = 0.f;
    if (!DUAL && g.bias) load_strided_as_float<NT, 16>(g.bias, g.bias_dtype, n0 + wn * WN + (lane & 15), g.N, bias_v);
    // Where each of this lane's rows goes (and its scale) is fetched for all rows at once, and so are the old
    // values that a row block adds to: a load inside the loops below would be waited for before the next leaves.
    int m_of[MT][4];
    float scale_of[MT][4];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int ml = r0 + (2 * i + wm) * 16 + (lane >> 4) * 4 + r;
            const int safe = (ml < r_end && ml < r0 + TM) ? ml : r0;
            m_of[i][r] = g.c_rows ? g.c_rows[safe] : safe;
            scale_of[i][r] = (EPI == EPI_RESID && g.row_scale) ? g.row_scale[safe] : 1.f;
        }
    if constexpr (DUAL) {
        with_activation(g.act, [&](auto ac) {
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int ml = r0 + (2 * i + wm) * 16 + (lane >> 4) * 4 + r;
                    if (ml >= r_end || ml >= r0 + TM) continue;
                    const int m = m_of[i][r];
#pragma unroll
                    for (int j = 0; j < NT; j += 2) {
                        const int n = n0 + wn * (WN / 2) + (j / 2) * 16 + (lane & 15);
                        if (n < g.N)
                            from_float((bf16*)g.C + (size_t)m * g.ldc + n, gated_c<decltype(ac)::value>(acc[i][j][r], acc[i][j + 1][r]));
                    }
                }
        });
        return;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        float old[4][NT];
        if (EPI == EPI_RESID) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const int n = min(n0 + wn * WN + j * 16 + (lane & 15), g.N - 1);
                    old[r][j] = ((const float*)g.C)[(size_t)m_of[i][r] * g.ldc + n];
                }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int ml = r0 + (2 * i + wm) * 16 + (lane >> 4) * 4 + r;
            if (ml >= r_end || ml >= r0 + TM) continue;
            const int m = m_of[i][r];
            {
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const int n = n0 + wn * WN + j * 16 + (lane & 15);
                    if (n >= g.N) continue;
                    float v = acc[i][j][r];
                    if (g.bias) v += bias_v[j];
                    if (EPI == EPI_STORE) {
                        from_float((bf16*)g.C + (size_t)m * g.ldc + n, v);
                    } else if (EPI == EPI_STORE_F32) {
                        ((float*)g.C)[(size_t)m * g.ldc + n] = v;
                    } else {
                        if (g.row_scale) {
                            v *= scale_of[i][r];
                            asm volatile("" : "+v"(v));      // rounded before it is added (no fused multiply-add)
                        }
                        ((float*)g.C)[(size_t)m * g.ldc + n] = old[r][j] + v;
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Few rows (decode): the weights are streamed once from memory straight into
// MFMA operands, no LDS staging.  A block owns NW sets of 16 rows of W and up
// to 16*MT logical rows; its WAVES waves split K between them in pieces of 128
// (with few accumulators, the next piece's loads are issued before this piece's
// products) and their partial sums are added in wave order through LDS.  A
// product wants lane (i = lane%16, g = lane/16) to hold 16 bytes (k 8g..8g+7 of
// every 32) of W row n0+i; they arrive in whole 128-byte lines, two loads and an
// exchange between lanes per 64 k (see `load_lines16`).  The activations use the
// same k -> lane assignment, which is all the MFMA needs to be right.
// W is the A operand: the accumulator of lane (m = lane%16, g) holds
// C[m][n0 + 4g + r], r = 0..3.
// ---------------------------------------------------------------------------
// rsqrt(mean of squares + eps) of a row from the sum of its squares.  Division and sqrtf are the correctly
// rounded ones (the compiler's default for HIP; __fsqrt_rn is NOT: it is the approximate instruction, whose
// result the compiler refines in some kernels and not in others), so every epilogue that scales its rows
// gets the same bits.
__device__ __forceinline__ float row_rstd(float total, int K, float eps) {
    const float mean = total / (float)K;
    return 1.0f / sqrtf(mean + eps);
}

// p[0] + p[1] + ... in that order; eight loads leave together (a plain loop would wait for each in turn)
__device__ __forceinline__ float sum_in_order(const float* p, int n) {
    float total = 0.f;
    for (int b0 = 0; b0 < n; b0 += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = p[min(b0 + u, n - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (b0 + u < n) total += v[u];
    }
    return total;
}

// NORM: the rows of A are float32 and are normed on the way in, y = x * rsqrt(mean(x^2) + eps) * w
// (ferrox-core/src/matmul.rs:62-69): x * w is rounded to bfloat16 and multiplied, the sums of
// squares that the waves gather over their parts of K are added up, and the product is scaled by
// the row's rsqrt before the bias is added.
__device__ __forceinline__ void load8f(const float* p, bool ok, float* v) {
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
    if (ok) {
        a = *(const float4*)p;
        b = *(const float4*)(p + 4);
    }
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// The weights come in whole lines with the non-temporal hint (`load_lines16`, `swap_halves`).  Measured at 8
// tokens of the A2.7B sizes against 16-byte loads of half lines: the experts' gate/up product 69.1 -> 64.4 us, their
// down product 36.6 -> 32.7 us, the head 132 -> 101 us (4.7 -> 6.2 TB/s).
// NW: sets of 16 weight rows per wave; in dual mode set a is the gate (a even) or up (a odd) rows of
// column group a / 2.
template <int MT, int WAVES, int NW, bool DUAL, int EPI, bool NORM = false, bool ROPE = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_bf16_skinny_kernel(GemmArgs g) {
    static_assert(!DUAL || NW % 2 == 0, "dual mode multiplies two matrices");
    static_assert(!ROPE || (NW == 2 && !DUAL && !NORM && EPI == EPI_STORE), "the rope epilogue pairs two sets of columns");
    static_assert(!NORM || (!DUAL && EPI == EPI_STORE), "the fused norm feeds a plain product");
    __shared__ float red_ss[NORM ? WAVES : 1][MT][64];
    float ss[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) ss[mt] = 0.f;
    constexpr int NACC = MT * NW;
    constexpr int COLS = DUAL ? 8 * NW : 16 * NW;   // output columns of a block
    // K is cut into PARTS parts whose sums are added in their order: one part per wave, or, with fewer than four
    // waves, VW consecutive parts per wave with accumulators of their own, so that one, two and four waves give
    // the same bits
    constexpr int VW = WAVES < 4 ? 4 / WAVES : 1, PARTS = WAVES * VW;
    __shared__ f32x4_t red[PARTS][NACC][64];
    int r0 = 0, r_end = 0, expert = 0, pair_a = -1, pair_c = -1;
    const bool pairs = MT == 1 && g.pair_ids != nullptr;
    if (pairs) {
        if (!locate_pairs(g, blockIdx.y, expert, pair_a, pair_c)) return;
    } else {
        locate_rows<16 * MT>(g, blockIdx.y, r0, r_end, expert);
        if (r0 < 0) return;
    }
    const int n0 = blockIdx.x * COLS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, grp = lane >> 4;
    const bf16* Wbase = (const bf16*)g.W + (size_t)expert * g.w_stride;
    // rope epilogue: a block takes 16 + 16 columns of one head, (16 j .. , rot/2 + 16 j ..) while they are rotated,
    // two neighbouring sets of 16 after that
    int rope_head = 0, rope_j = 0, rope_c0 = 0, rope_c1 = 0;
    bool rope_rotated = false;
    if constexpr (ROPE) {
        const int per_head = g.rope_hd >> 5;
        rope_head = blockIdx.x / per_head;
        rope_j = blockIdx.x - rope_head * per_head;
        const bool is_v = rope_head >= g.rope_nh + g.rope_nkv;
        const int n_rot = is_v ? 0 : g.rope_rot >> 5;          // blocks of this head whose columns are rotated
        rope_rotated = rope_j < n_rot;
        rope_c0 = rope_rotated ? 16 * rope_j : (is_v ? 32 * rope_j : g.rope_rot + 32 * (rope_j - n_rot));
        rope_c1 = rope_rotated ? rope_c0 + (g.rope_rot >> 1) : rope_c0 + 16;
    }
    const bf16* wrow[NW];     // this lane's place in the set's first load, and how far behind it the second is
    int wrow_b[NW];
#pragma unroll
    for (int a = 0; a < NW; ++a) {
        const int n = ROPE ? rope_head * g.rope_hd + (a ? rope_c1 : rope_c0) + li
                           : (DUAL ? n0 + (a >> 1) * 16 + li : n0 + a * 16 + li);
        const bool up = DUAL && (a & 1);
        // whole lines per load: the lanes of a set's first load take rows li % 8, those of its second rows
        // 8 + li % 8, both k 32 (li / 8) .. of every 64; rows past the end repeat the last one, never stored
        const int nl = n - li + (li & 7);
        const int na = min(nl, g.N - 1), nb = min(nl + 8, g.N - 1);
        const size_t rs = g.kb_stride ? 64 : (size_t)g.K;
        const size_t first = g.kb_stride ? (size_t)(up ? g.up_offset / g.K : 0) * 64 : (size_t)(up ? g.up_offset : 0);
        wrow[a] = Wbase + first + (size_t)na * rs + 32 * (li >> 3);
        wrow_b[a] = (int)((nb - na) * rs);
    }
    const size_t slab = g.kb_stride ? (size_t)g.kb_stride : 64;     // element (row, k) is at row + (k / 64) * slab + k % 64
    const bf16* xrow[MT];       // NORM: float rows, kept under the same name
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = r0 + mt * 16 + li;
        const bool live = pairs ? pair_a >= 0 : m < r_end;
        const size_t off = !live ? 0 : (size_t)(pairs ? pair_a : (g.a_rows ? g.a_rows[m] : m)) * g.lda;
        // a dead row reads the first row of A instead: its products land in rows that are never stored
        xrow[mt] = NORM ? (live ? (const bf16*)((const float*)g.A + off) : nullptr) : (const bf16*)g.A + off;
    }
    f32x4_t acc[VW][MT][NW];
#pragma unroll
    for (int p = 0; p < VW; ++p)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int a = 0; a < NW; ++a) acc[p][mt][a] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

    const int n_super = (g.K + 127) / 128;
    const int per = (n_super + PARTS - 1) / PARTS;      // pieces per part
    const int s_end = min(n_super, (wave + 1) * VW * per);
    // One piece: its loads (four per set of weight rows and per row tile), then its products.  FULL: the piece
    // lies inside K, so every load is unconditional and the compiler can count the loads in flight.
    auto load_piece = [&](auto full, int sp, uint4 (&w)[NW][4], uint4 (&x)[MT][4]) {
        constexpr bool FULL = decltype(full)::value;
        const int kb = sp * 128 + grp * 8;     // load u of this lane: k = kb + 32u .. +7
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int kl = kb + 64 * h;                       // this lane's k without its half: 32 (li / 8) is in wrow
            const bool kin = FULL || kl + 32 * (li >> 3) < g.K;
            const size_t woff = (size_t)(kl >> 6) * slab + (kl & 63);
#pragma unroll
            for (int a = 0; a < NW; ++a) {
                w[a][2 * h] = kin ? load_lines16(wrow[a] + woff) : make_uint4(0, 0, 0, 0);
                w[a][2 * h + 1] = kin ? load_lines16(wrow[a] + woff + wrow_b[a]) : make_uint4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = kb + 32 * u;
            const bool kin = FULL || k < g.K;
            if constexpr (NORM) {
                float gv[8];
                if (g.norm_dtype == FX_F32) {
                    load8f((const float*)g.norm_w + k, kin, gv);
                } else {
                    const uint4 gw = kin ? *(const uint4*)((const bf16*)g.norm_w + k) : make_uint4(0, 0, 0, 0);
                    gv[0] = __uint_as_float(gw.x << 16); gv[1] = __uint_as_float(gw.x & 0xffff0000u);
                    gv[2] = __uint_as_float(gw.y << 16); gv[3] = __uint_as_float(gw.y & 0xffff0000u);
                    gv[4] = __uint_as_float(gw.z << 16); gv[5] = __uint_as_float(gw.z & 0xffff0000u);
                    gv[6] = __uint_as_float(gw.w << 16); gv[7] = __uint_as_float(gw.w & 0xffff0000u);
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    float xv[8];
                    load8f((const float*)xrow[mt] + k, kin && xrow[mt], xv);
#pragma unroll
                    for (int i = 0; i < 8; ++i) ss[mt] += xv[i] * xv[i];
                    x[mt][u] = make_uint4(pack_bf16(xv[0] * gv[0], xv[1] * gv[1]), pack_bf16(xv[2] * gv[2], xv[3] * gv[3]),
                                          pack_bf16(xv[4] * gv[4], xv[5] * gv[5]), pack_bf16(xv[6] * gv[6], xv[7] * gv[7]));
                }
            } else {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) x[mt][u] = kin ? *(const uint4*)(xrow[mt] + k) : make_uint4(0, 0, 0, 0);
            }
        }
    };
    auto multiply_into = [&](f32x4_t (&to)[MT][NW], const uint4 (&w)[NW][4], const uint4 (&x)[MT][4]) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int a = 0; a < NW; ++a) {
                // low k: own first load below lane 8 of a row of 16, the other half's second load above;
                // high k: the other half's first load below, own second load above
                const uint4 wu = (u & 1) ? swap_halves<0x3>(w[a][u], w[a][u - 1]) : swap_halves<0xC>(w[a][u], w[a][u + 1]);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    to[mt][a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, wu), __builtin_bit_cast(bf16x8_t, x[mt][u]),
                                                                        to[mt][a], 0, 0, 0);
            }
    };
    // piece sp belongs to part sp / per, the (sp / per - wave * VW)-th of this wave (the same for all its lanes)
    auto multiply_piece = [&](int sp, const uint4 (&w)[NW][4], const uint4 (&x)[MT][4]) {
        if constexpr (VW == 1) {
            multiply_into(acc[0], w, x);
        } else {
            const int p = sp / per - wave * VW;
            if (p == 0) multiply_into(acc[0], w, x);
            else if (p == 1) multiply_into(acc[1], w, x);
            else if constexpr (VW == 4) {
                if (p == 2) multiply_into(acc[2], w, x);
                else multiply_into(acc[3], w, x);
            }
        }
    };
    constexpr std::true_type whole{};
    constexpr std::false_type masked{};
    const int s_whole = min(s_end, g.K / 128);       // pieces before this one lie inside K
    int sp = wave * VW * per;
    // Few accumulators leave registers for two pieces (see the loop below).  The first piece's loads leave here,
    // and so do the old values that a block adds its product to: nothing of the epilogue waits for memory then.
    constexpr bool TWO = MT * NW <= 4 && !NORM;
    uint4 w0[TWO ? NW : 1][4], x0[TWO ? MT : 1][4];
    if constexpr (TWO && !ROPE) {
        if (sp < s_whole) load_piece(whole, sp, w0, x0);
    }
    constexpr int SETS = DUAL ? NW / 2 : NW;      // column groups of a block
    constexpr int OUTS = MT * SETS;               // accumulator tiles (dual: pairs of them) that become output tiles
    float old_first[4] = {0.f, 0.f, 0.f, 0.f}, row_scale_first = 1.f;     // of this thread's first output tile
    if constexpr (EPI == EPI_RESID) {
        if (tid < OUTS * 64) {
            const int mt = (tid >> 6) / SETS, a = (tid >> 6) % SETS;
            const int ml = pairs ? pair_c : r0 + mt * 16 + li;
            if (pairs ? ml >= 0 : ml < r_end) {
                const int m = (g.c_rows && !pairs) ? g.c_rows[ml] : ml;
                if (g.row_scale) row_scale_first = g.row_scale[ml];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    old_first[r] = ((const float*)g.C)[(size_t)m * g.ldc + min(n0 + a * 16 + grp * 4 + r, g.N - 1)];
            }
        }
    }
    // rope epilogue: what thread (lane, wave) needs for its pairs of outputs, rows 16 mt + lane % 16, column
    // 4 (lane / 16) + wave of the two sets, is fetched and worked out here, while the weights are on their way
    float rope_sn[MT], rope_cs[MT], rope_rstd[MT], rope_b0 = 0.f, rope_b1 = 0.f;
    size_t rope_page[MT];
    int rope_slot[MT];
    if constexpr (ROPE) {
        const int cc = grp * 4 + wave;
        const bool to_pages = rope_head >= g.rope_nh && g.rope_k_pages;
        // first every load that depends on nothing, then the page ids, which need position and sequence
        int row_of[MT], pos[MT], seq[MT];
        float total[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            row_of[mt] = min(r0 + 16 * mt + li, r_end - 1);
            pos[mt] = g.rope_positions[row_of[mt]];
            seq[mt] = to_pages ? g.rope_token_seq[row_of[mt]] : 0;
        }
        // (without a bias the same loads read the positions instead: a branch around them would wait for them)
        const void* bias_or = g.bias ? g.bias : (const void*)g.rope_positions;
        const int bias_dt = g.bias ? g.bias_dtype : FX_F32;
        const RawElement e0 = fetch_element(bias_or, bias_dt, g.bias ? (size_t)rope_head * g.rope_hd + rope_c0 + cc : 0);
        const RawElement e1 = fetch_element(bias_or, bias_dt, g.bias ? (size_t)rope_head * g.rope_hd + rope_c1 + cc : 0);
        // the pair's frequency from the table (columns that are not rotated read entry 0 and do not use it)
        const int p = rope_rotated ? 16 * rope_j + cc : 0;
        const float freq = g.rope_inv_freq[p];
        const float freq_div = g.rope_freq_factors ? g.rope_freq_factors[p] : 1.f;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            total[mt] = g.row_ss ? sum_in_order(g.row_ss + (size_t)row_of[mt] * g.row_ss_n, g.row_ss_n) : 0.f;
        rope_b0 = element_as_float(e0);
        rope_b1 = element_as_float(e1);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            rope_page[mt] = 0;
            rope_slot[mt] = 0;
            if (to_pages) {
                rope_page[mt] = (size_t)g.rope_table[(size_t)seq[mt] * g.rope_max_blocks + pos[mt] / g.rope_bs];
                rope_slot[mt] = pos[mt] % g.rope_bs;
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            rope_rstd[mt] = g.row_ss ? row_rstd(total[mt], g.K, g.norm_eps) : 1.f;
            rope_sn[mt] = 0.f;
            rope_cs[mt] = 1.f;
            if (rope_rotated) {
                float angle = (float)pos[mt] * freq;
                if (g.rope_freq_factors) angle = angle / freq_div;
                sincosf(angle, &rope_sn[mt], &rope_cs[mt]);
            }
        }
    }
    // Few accumulators leave registers for two pieces: the loads of the next piece are then issued before the
    // products of this one, so a wave always has a piece on its way from memory.  Each product follows the
    // loads issued after its own in straight-line code.
    if constexpr (TWO) {
        if (sp < s_whole) {
            uint4 w1[NW][4], x1[MT][4];
            // (the rotating product fetches what its epilogue needs first: behind the weights those short loads
            // would wait for them, and measured it is slower)
            if constexpr (ROPE) load_piece(whole, sp, w0, x0);
            for (; sp + 2 < s_whole; sp += 2) {
                load_piece(whole, sp + 1, w1, x1);
                multiply_piece(sp, w0, x0);
                load_piece(whole, sp + 2, w0, x0);
                multiply_piece(sp + 1, w1, x1);
            }
            if (sp + 1 < s_whole) {
                load_piece(whole, sp + 1, w1, x1);
                multiply_piece(sp, w0, x0);
                multiply_piece(sp + 1, w1, x1);
                sp += 2;
            } else {
                multiply_piece(sp, w0, x0);
                sp += 1;
            }
        }
    } else {
        for (; sp < s_whole; ++sp) {
            uint4 w[NW][4], x[MT][4];
            load_piece(whole, sp, w, x);
            multiply_piece(sp, w, x);
        }
    }
    for (; sp < s_end; ++sp) {          // the piece that K ends in
        uint4 w[NW][4], x[MT][4];
        load_piece(masked, sp, w, x);
        multiply_piece(sp, w, x);
    }
#pragma unroll
    for (int p = 0; p < VW; ++p)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int a = 0; a < NW; ++a) red[wave * VW + p][mt * NW + a][lane] = acc[p][mt][a];
    if constexpr (NORM) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) red_ss[wave][mt][lane] = ss[mt];
    }
    __syncthreads();
    if constexpr (ROPE) {
        static_assert(!ROPE || WAVES == 4, "a wave per accumulator row");
        const int L = lane, r = wave;
        const int hd = g.rope_hd, bs = g.rope_bs, cc = (L >> 4) * 4 + r;
        const int d0 = rope_c0 + cc, d1 = rope_c1 + cc;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int ml = r0 + 16 * mt + (L & 15);
            if (ml >= r_end) continue;
            f32x4_t v0 = (f32x4_t){0.f, 0.f, 0.f, 0.f}, v1 = v0;
#pragma unroll
            for (int w = 0; w < PARTS; ++w) {
                v0 += red[w][mt * NW][L];
                v1 += red[w][mt * NW + 1][L];
            }
            // product times scale is rounded before the bias is added, as in the plain epilogue (whose bias sits
            // behind a branch); the empty statement keeps the compiler from fusing the two here
            float o0 = v0[r] * rope_rstd[mt], o1 = v1[r] * rope_rstd[mt];
            asm volatile("" : "+v"(o0), "+v"(o1));
            if (g.bias) {
                o0 += rope_b0;
                o1 += rope_b1;
            }
            const float a = bf16_to_float(float_to_bf16(o0)), b = bf16_to_float(float_to_bf16(o1));
            float y0 = a, y1 = b;
            if (rope_rotated) rotate_pair(a, b, rope_cs[mt], rope_sn[mt], y0, y1);
            if (rope_head < g.rope_nh) {
                bf16* dst = (bf16*)g.C + (size_t)ml * g.ldc + (size_t)rope_head * hd;
                from_float(dst + d0, y0);
                from_float(dst + d1, y1);
            } else if (g.rope_k_pages) {
                if (rope_head < g.rope_nh + g.rope_nkv) {
                    bf16* dst = (bf16*)g.rope_k_pages + ((rope_page[mt] * g.rope_nkv + (rope_head - g.rope_nh)) * bs + rope_slot[mt]) * hd;
                    from_float(dst + d0, y0);
                    from_float(dst + d1, y1);
                } else {
                    bf16* dst = (bf16*)g.rope_v_pages + (rope_page[mt] * g.rope_nkv + (rope_head - g.rope_nh - g.rope_nkv)) * hd * bs + rope_slot[mt];
                    from_float(dst + (size_t)d0 * bs, y0);
                    from_float(dst + (size_t)d1 * bs, y1);
                }
            }
        }
        return;
    }
    for (int idx = tid; idx < OUTS * 64; idx += WAVES * 64) {
        const int t = idx >> 6, L = idx & 63;
        const int mt = t / SETS, a = t % SETS;
        f32x4_t v = (f32x4_t){0.f, 0.f, 0.f, 0.f}, v2 = v;
#pragma unroll
        for (int w = 0; w < PARTS; ++w) {
            v += red[w][mt * NW + (DUAL ? 2 * a : a)][L];
            if (DUAL) v2 += red[w][mt * NW + 2 * a + 1][L];
        }
        const int ml = pairs ? pair_c : r0 + mt * 16 + (L & 15);      // L % 16 == lane % 16
        if (pairs ? ml < 0 : ml >= r_end) continue;
        const int m = (g.c_rows && !pairs) ? g.c_rows[ml] : ml;
        float rstd = 1.f;
        float bias_v[4] = {0.f, 0.f, 0.f, 0.f};          // of columns n0 + 16 a + 4 (L / 16) + 0..3
        if (!DUAL && g.bias) load_strided_as_float<4, 1>(g.bias, g.bias_dtype, n0 + a * 16 + (L >> 4) * 4, g.N, bias_v);
        if (!NORM && g.row_ss) rstd = row_rstd(sum_in_order(g.row_ss + (size_t)m * g.row_ss_n, g.row_ss_n), g.K, g.norm_eps);
        if constexpr (NORM) {
            float total = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w)
#pragma unroll
                for (int q = 0; q < 4; ++q) total += red_ss[w][mt][(L & 15) + 16 * q];
            rstd = row_rstd(total, g.K, g.norm_eps);
        }
        // what a row block adds to, and its scale: the first tile's came in at the start, a further one's are
        // fetched together, ahead of the stores
        float old[4] = {0.f, 0.f, 0.f, 0.f}, row_scale = 1.f;
        if (EPI == EPI_RESID) {
            if (idx == tid) {
                row_scale = row_scale_first;
#pragma unroll
                for (int r = 0; r < 4; ++r) old[r] = old_first[r];
            } else {
                if (g.row_scale) row_scale = g.row_scale[ml];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    old[r] = ((const float*)g.C)[(size_t)m * g.ldc + min(n0 + a * 16 + (L >> 4) * 4 + r, g.N - 1)];
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int n = n0 + a * 16 + (L >> 4) * 4 + r;
            if (n >= g.N) continue;
            float o = v[r] * rstd;
            asm volatile("" : "+v"(o));          // the product is rounded before the bias is added (no fused multiply-add)
            if (DUAL) {
                with_activation(g.act, [&](auto ac) { from_float((bf16*)g.C + (size_t)m * g.ldc + n, gated_c<decltype(ac)::value>(o, v2[r])); });
                continue;
            }
            if (g.bias) o += bias_v[r];
            if (EPI == EPI_STORE) {
                from_float((bf16*)g.C + (size_t)m * g.ldc + n, o);
            } else if (EPI == EPI_STORE_F32) {
                ((float*)g.C)[(size_t)m * g.ldc + n] = o;
            } else {
                if (g.row_scale) {
                    o *= row_scale;
                    asm volatile("" : "+v"(o));
                }
                ((float*)g.C)[(size_t)m * g.ldc + n] = old[r] + o;
            }
        }
    }
}

// ===========================================================================
// float32 with FMA
// ===========================================================================
#define FK 16
// 64 x 64 outputs per block, 256 threads, 4 x 4 per thread.
template <bool DUAL, int EPI>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmArgs g) {
    __shared__ float As[FK][64 + 4];
    __shared__ float Bs[DUAL ? 2 : 1][FK][64 + 4];
    int r0, r_end, expert;
    locate_rows<64>(g, blockIdx.y, r0, r_end, expert);
    if (r0 < 0) return;
    const int n0 = blockIdx.x * 64;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    const float* Abase = (const float*)g.A;
    const float* Wbase = (const float*)g.W + (size_t)expert * g.w_stride;

    // loader: element idx = tid + i*256 of a 64 x 16 tile, k fastest
    const float* a_src[4];
    const float* b_src[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = (tid + i * 256) >> 4;
        a_src[i] = nullptr;
        b_src[i] = nullptr;
        if (r0 + row < r_end) {
            const int m = r0 + row;
            a_src[i] = Abase + (size_t)(g.a_rows ? g.a_rows[m] : m) * g.lda;
        }
        if (n0 + row < g.N) b_src[i] = Wbase + (size_t)(n0 + row) * g.K;
    }
    const int kk = tid & 15;

    float acc[4][4] = {}, acc2[4][4] = {};
    for (int k0 = 0; k0 < g.K; k0 += FK) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = (tid + i * 256) >> 4;
            const bool kin = k0 + kk < g.K;
            As[kk][row] = (a_src[i] && kin) ? a_src[i][k0 + kk] : 0.f;
            Bs[0][kk][row] = (b_src[i] && kin) ? b_src[i][k0 + kk] : 0.f;
            if (DUAL) Bs[DUAL ? 1 : 0][kk][row] = (b_src[i] && kin) ? b_src[i][g.up_offset + k0 + kk] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < FK; ++k) {
            float a[4], b[4], b2[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[0][k][tx * 4 + j];
            if (DUAL) {
#pragma unroll
                for (int j = 0; j < 4; ++j) b2[j] = Bs[DUAL ? 1 : 0][k][tx * 4 + j];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
                    if (DUAL) acc2[i][j] = fmaf(a[i], b2[j], acc2[i][j]);
                }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ml = r0 + ty * 4 + i;
        if (ml >= r_end) continue;
        const int m = g.c_rows ? g.c_rows[ml] : ml;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= g.N) continue;
            float v = acc[i][j];
            float* out = (float*)g.C + (size_t)m * g.ldc + n;
            if (DUAL) {
                with_activation(g.act, [&](auto ac) { *out = gated_c<decltype(ac)::value>(v, acc2[i][j]); });
            } else {
                if (g.bias) v += load_as_float(g.bias, g.bias_dtype, n);
                if (EPI == EPI_RESID) {
                    if (g.row_scale) v *= g.row_scale[ml];
                    *out += v;
                } else {
                    *out = v;
                }
            }
        }
    }
}

// ===========================================================================
// host side
// ===========================================================================
template <int TM, int TN, int WM, int WN>
static void launch_bf16(GemmArgs g, int epi, int m_tiles, hipStream_t s) {
    const bool dual = epi == EPI_GATED;
    g.n_col_tiles = ceil_div(g.N, dual ? TN / 2 : TN);
    g.n_row_tiles = m_tiles;
    dim3 grid(8 * ceil_div((long)g.n_col_tiles * g.n_row_tiles, 8));
#define FX_TILED(DUAL_, EPI_)                                                                       \
    if (g.vec_ok) gemm_bf16_kernel<TM, TN, WM, WN, DUAL_, EPI_, true><<<grid, 256, 0, s>>>(g);     \
    else gemm_bf16_kernel<TM, TN, WM, WN, DUAL_, EPI_, false><<<grid, 256, 0, s>>>(g)
    switch (epi) {
        case EPI_STORE: FX_TILED(false, EPI_STORE); break;
        case EPI_STORE_F32: FX_TILED(false, EPI_STORE_F32); break;
        case EPI_RESID: FX_TILED(false, EPI_RESID); break;
        default: FX_TILED(true, EPI_GATED); break;
    }
#undef FX_TILED
}

// Switches for tests and measurement (ferrox_amd/debug.py is their one caller): they pick, whatever the sizes,
// a kernel variant that the sizes would otherwise choose.  The product path never sets them.
static int g_skinny_nw = 0;    // "skinny_sets": 1 or 2 sets of weight rows per wave of the product for few rows (0: by the sizes)
static int g_skinny_mt = 0;    // "skinny_row_tiles": 1, 2 or 4 tiles of 16 rows per block of that product (0: by the sizes)
static int g_skinny_waves = 0; // "skinny_waves": 1, 2, 4 or 8 waves that split K in a block of that product (0: by the sizes)
static int g_few_rows = 3;     // "few_rows": sorted by expert, up to this many rows an expert go to the product for few rows (at most 64)
static int g_head_rows = 16;   // "head_rows": plain rows against very many weight rows go to the tiled kernel from more than this many on
static int g_tile64_rows = 20; // "tile64_rows": experts with up to this many rows on average take tiles of 64 rows
static int g_no_wide = 0;      // "wide": 0 sends many-row products to the register-staged tiled kernel, 1 (default) by the sizes,
static int g_plain_rows = 0;   // "plain_rows": plain rows up to this many go to the product for few rows whatever the weight rows (0: by the sizes)
static int g_stream_w = -1;    // "stream_w": 1 / 0 forces the non-temporal hint on the tiled kernel's weight loads on / off; -1: by the shape
static int g_wide_grouped = 0; // "wide_grouped": as "wide", for products whose rows are sorted by expert only
static int g_wide_force = 0;   //         256, 192, 128, 64, 12 or 4 (tiles of 64 rows) picks that tile of the LDS-tiled kernel
FX_API int fx_debug_set(const char* key, int value) {
    if (!strcmp(key, "skinny_sets")) { g_skinny_nw = value; return 0; }
    if (!strcmp(key, "skinny_row_tiles")) { g_skinny_mt = value; return 0; }
    if (!strcmp(key, "skinny_waves")) { g_skinny_waves = value; return 0; }
    if (!strcmp(key, "few_rows")) { g_few_rows = value < 0 ? 0 : (value > 64 ? 64 : value); return 0; }
    if (!strcmp(key, "tile64_rows")) { g_tile64_rows = value; return 0; }
    if (!strcmp(key, "head_rows")) { g_head_rows = value; return 0; }
    if (!strcmp(key, "wide")) { g_no_wide = !value; g_wide_force = value > 1 ? value : 0; return 0; }
    if (!strcmp(key, "wide_grouped")) { g_wide_grouped = value > 1 ? value : 0; return 0; }
    if (!strcmp(key, "stream_w")) { g_stream_w = value; return 0; }
    if (!strcmp(key, "plain_rows")) { g_plain_rows = value; return 0; }
    FX_REQUIRE(false, "gemm: no debug switch '%s' (skinny_sets, skinny_row_tiles, skinny_waves, few_rows, head_rows, tile64_rows, wide, wide_grouped, stream_w, plain_rows)", key);
    return 1;
}

template <int TMB, int TN, int NS, int NSA, bool STREAM>
static void launch_wide_as(const GemmArgs& g, int epi, dim3 grid, hipStream_t s) {
    switch (epi) {
        case EPI_STORE: gemm_bf16_wide_kernel<TMB, TN, NS, false, EPI_STORE, NSA, STREAM><<<grid, 512, 0, s>>>(g); break;
        case EPI_STORE_F32: gemm_bf16_wide_kernel<TMB, TN, NS, false, EPI_STORE_F32, NSA, STREAM><<<grid, 512, 0, s>>>(g); break;
        case EPI_RESID: gemm_bf16_wide_kernel<TMB, TN, NS, false, EPI_RESID, NSA, STREAM><<<grid, 512, 0, s>>>(g); break;
        default:
            if constexpr (TN % 128 == 0) gemm_bf16_wide_kernel<TMB, TN, NS, true, EPI_GATED, NSA, STREAM><<<grid, 512, 0, s>>>(g);
            break;
    }
}
template <int TMB, int TN, int NS, int NSA = NS>
static void launch_wide(GemmArgs g, int epi, int m_tiles, hipStream_t s) {
    g.n_col_tiles = ceil_div(g.N, epi == EPI_GATED ? TN / 2 : TN);
    g.n_row_tiles = m_tiles;
    dim3 grid(g.expert_offsets ? 8 * ceil_div(m_tiles, 8) * g.n_col_tiles : 8 * ceil_div((long)g.n_col_tiles * m_tiles, 8));
    // the streaming variant exists for the tiles that few rows take (up to 192 of them)
    if constexpr (TMB <= 12) {
        if (g.stream_w) {
            launch_wide_as<TMB, TN, NS, NSA, true>(g, epi, grid, s);
            return;
        }
    }
    launch_wide_as<TMB, TN, NS, NSA, false>(g, epi, grid, s);
}

template <int MT, int WAVES, int NW>
static void launch_skinny_cfg(const GemmArgs& g, int epi, int m_tiles, hipStream_t s) {
    dim3 grid(ceil_div(g.N, epi == EPI_GATED ? 8 * NW : 16 * NW), m_tiles);
    if constexpr (MT * NW * WAVES <= 32) {       // the partial sums of all waves fit in LDS
        if (g.norm_w) {
            gemm_bf16_skinny_kernel<MT, WAVES, NW, false, EPI_STORE, true><<<grid, WAVES * 64, 0, s>>>(g);
            return;
        }
        switch (epi) {
            case EPI_STORE: gemm_bf16_skinny_kernel<MT, WAVES, NW, false, EPI_STORE><<<grid, WAVES * 64, 0, s>>>(g); break;
            case EPI_STORE_F32: gemm_bf16_skinny_kernel<MT, WAVES, NW, false, EPI_STORE_F32><<<grid, WAVES * 64, 0, s>>>(g); break;
            case EPI_RESID: gemm_bf16_skinny_kernel<MT, WAVES, NW, false, EPI_RESID><<<grid, WAVES * 64, 0, s>>>(g); break;
            default:
                if constexpr (NW % 2 == 0) gemm_bf16_skinny_kernel<MT, WAVES, NW, true, EPI_GATED><<<grid, WAVES * 64, 0, s>>>(g);
                break;
        }
    }
}

// mt: row tiles per block (1, 2, 4); nw: 16-row weight sets per wave; waves: 4 or 8 split K (1 or 2 with one row tile).
static void launch_skinny(const GemmArgs& g, int epi, int mt, int nw, int waves, int m_tiles, hipStream_t s) {
#define FX_SK(MT_, W_, NW_) launch_skinny_cfg<MT_, W_, NW_>(g, epi, m_tiles, s)
    if (waves == 8 && mt * nw <= 4) {
        if (nw == 2) {
            if (mt == 1) FX_SK(1, 8, 2);
            else FX_SK(2, 8, 2);
        } else {
            if (mt == 1) FX_SK(1, 8, 1);
            else if (mt == 2) FX_SK(2, 8, 1);
            else FX_SK(4, 8, 1);
        }
        return;
    }
    if (waves <= 2 && mt == 1) {
        if (waves == 1) {
            if (nw == 2) FX_SK(1, 1, 2);
            else FX_SK(1, 1, 1);
        } else {
            if (nw == 2) FX_SK(1, 2, 2);
            else FX_SK(1, 2, 1);
        }
        return;
    }
    if (nw == 2) {
        if (mt == 1) FX_SK(1, 4, 2);
        else if (mt == 2) FX_SK(2, 4, 2);
        else FX_SK(4, 4, 2);
    } else {
        if (mt == 1) FX_SK(1, 4, 1);
        else if (mt == 2) FX_SK(2, 4, 1);
        else FX_SK(4, 4, 1);
    }
#undef FX_SK
}

// The q/k/v product of up to 64 tokens with the rotation and the cache write in its epilogue (see GemmArgs):
// bfloat16, C [M, (nh + 2 nkv) hd], bias [N] or null, row_ss as in fx_gemm.  head_dim and the rotary dimension
// are multiples of 32.  k_pages [pages][nkv][bs][hd] and v_pages [pages][nkv][hd][bs], or both null.
FX_API int fx_qkv_rope(void* stream, const void* A, long lda, const void* W, long kb_rows, const void* bias, int bias_dtype,
                       void* C, long ldc, int M, int K, const float* row_ss, int row_ss_n, float eps,
                       const int* positions, const int* token_seq, const int* table, int max_blocks,
                       void* k_pages, void* v_pages, int nh, int nkv, int hd, int bs, int rot, const float* inv_freq,
                       const float* freq_factors) {
    FX_REQUIRE(M >= 1 && M <= 64 && K > 0 && K % 8 == 0 && lda % 8 == 0 && lda >= K, "qkv_rope: 1..64 rows of a multiple of 8 elements");
    FX_REQUIRE(nh > 0 && nkv > 0 && hd > 0 && hd % 32 == 0 && rot >= 0 && rot <= hd && rot % 32 == 0 && bs > 0,
               "qkv_rope: head_dim %d and rotary dimension %d must be multiples of 32", hd, rot);
    const int N = (nh + 2 * nkv) * hd;
    FX_REQUIRE(ldc >= N && (((uintptr_t)A | (uintptr_t)W) % 16) == 0, "qkv_rope: output rows too short or operands not aligned");
    FX_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "qkv_rope: key and value pages must come together");
    FX_REQUIRE(positions && token_seq && (!k_pages || (table && max_blocks > 0)), "qkv_rope: positions, sequences and block table");
    FX_REQUIRE(inv_freq || rot == 0, "qkv_rope: a rotation needs the table of its %d frequencies", rot / 2);
    FX_REQUIRE(!bias || bias_dtype == FX_F32 || bias_dtype == FX_BF16, "qkv_rope: unknown bias dtype %d", bias_dtype);
    FX_REQUIRE(kb_rows == 0 || (kb_rows == N && K % 64 == 0), "qkv_rope: weights in slabs of 64 k hold all %d rows", N);
    FX_REQUIRE(!row_ss || row_ss_n >= 1, "qkv_rope: sums of squares without their count");
    GemmArgs g = {};
    g.A = A; g.lda = lda; g.W = W; g.kb_stride = kb_rows * 64; g.bias = bias; g.bias_dtype = bias_dtype;
    g.C = C; g.ldc = ldc; g.M = M; g.N = N; g.K = K; g.vec_ok = 1;
    g.row_ss = row_ss; g.row_ss_n = row_ss_n; g.norm_eps = eps;
    g.rope_positions = positions; g.rope_token_seq = token_seq; g.rope_table = table; g.rope_max_blocks = max_blocks;
    g.rope_k_pages = k_pages; g.rope_v_pages = v_pages;
    g.rope_nh = nh; g.rope_nkv = nkv; g.rope_hd = hd; g.rope_bs = bs; g.rope_rot = rot;
    g.rope_inv_freq = inv_freq ? inv_freq : (const float*)positions;      // (rot == 0: read, never used)
    g.rope_freq_factors = freq_factors;
    dim3 grid((nh + 2 * nkv) * (hd / 32), 1);
    if (M <= 16) gemm_bf16_skinny_kernel<1, 4, 2, false, EPI_STORE, false, true><<<grid, 256, 0, (hipStream_t)stream>>>(g);
    else if (M <= 32) gemm_bf16_skinny_kernel<2, 4, 2, false, EPI_STORE, false, true><<<grid, 256, 0, (hipStream_t)stream>>>(g);
    else {
        // 33..64 rows: two blocks of 32 rows a column group rather than one of 64 (a wave fetches the operands of
        // every row tile of its block itself: a decode step at 64 sequences 11.03 -> 10.94 ms; the second block
        // finds the weights in the cache); the same bits
        grid.y = 2;
        gemm_bf16_skinny_kernel<2, 4, 2, false, EPI_STORE, false, true><<<grid, 256, 0, (hipStream_t)stream>>>(g);
    }
    FX_CHECK_LAUNCH("qkv_rope");
    return 0;
}

// dtype: type of A and W.  C is: T for EPI_STORE and EPI_GATED, float32 otherwise.
// rows_hint: in grouped mode, the expected number of rows per expert (chooses the tile).
FX_API int fx_gemm(void* stream, int dtype, int epi, const void* A, long lda, const void* W, long w_stride,
                   long up_offset, const void* bias, int bias_dtype, void* C, long ldc,
                   const float* row_scale, const int* a_rows, const int* c_rows, const int* expert_offsets,
                   int E, int M, int N, int K, const void* norm_w, int norm_dtype, float norm_eps,
                   const int* pair_ids, int pair_div, int n_always, int always_rows, int always_from_a, long kb_rows,
                   const float* row_ss, int row_ss_n, int act) {
    FX_REQUIRE(dtype == FX_F32 || dtype == FX_BF16, "gemm: unknown dtype %d", dtype);
    FX_REQUIRE(epi >= EPI_STORE && epi <= EPI_GATED, "gemm: unknown epilogue %d", epi);
    FX_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    FX_REQUIRE(lda >= K && ldc >= N, "gemm: leading dimensions lda=%ld ldc=%ld too small for K=%d N=%d", lda, ldc, K, N);
    FX_REQUIRE(!(epi == EPI_GATED && bias), "gemm: the gate/up epilogue takes no bias");
    FX_REQUIRE(act >= 0 && act < ACT_COUNT, "gemm: unknown activation %d", act);
    FX_REQUIRE(!(expert_offsets || pair_ids) || E > 0, "gemm: grouped mode needs E > 0");
    FX_REQUIRE(!pair_ids || (!expert_offsets && !a_rows && !c_rows && !row_scale && !norm_w && pair_div >= 1 && M <= 64 &&
                             dtype == FX_BF16),
               "gemm: unsorted pairs are for up to 64 bfloat16 rows without other row maps");
    FX_REQUIRE(!bias || bias_dtype == FX_F32 || bias_dtype == FX_BF16, "gemm: unknown bias dtype %d", bias_dtype);
    if (M == 0) return 0;
    if (norm_w) {
        FX_REQUIRE(dtype == FX_BF16 && epi == EPI_STORE, "gemm: the fused norm feeds a bfloat16 product that is stored");
        FX_REQUIRE(norm_dtype == FX_F32 || norm_dtype == FX_BF16, "gemm: unknown norm weight dtype %d", norm_dtype);
        FX_REQUIRE((expert_offsets ? (M + E - 1) / E : M) <= 32 && K % 8 == 0 && lda % 4 == 0 && w_stride % 8 == 0 &&
                       (((uintptr_t)A | (uintptr_t)W | (uintptr_t)norm_w) % 16 == 0),
                   "gemm: the fused norm takes up to 32 rows per group, K a multiple of 8 and 16-byte aligned rows");
    }
    GemmArgs g = {};
    g.norm_w = norm_w; g.norm_dtype = norm_dtype; g.norm_eps = norm_eps;
    g.row_ss = row_ss; g.row_ss_n = row_ss_n;
    FX_REQUIRE(!row_ss || (row_ss_n >= 1 && !norm_w && !expert_offsets && !pair_ids && !a_rows && !c_rows && dtype == FX_BF16 &&
                           epi == EPI_STORE && M <= 64 && K % 8 == 0 && lda % 8 == 0 && (((uintptr_t)A | (uintptr_t)W) % 16 == 0)),
               "gemm: a row scale from sums of squares goes with a plain stored bfloat16 product of up to 64 aligned rows");
    g.A = A; g.lda = lda; g.W = W; g.w_stride = w_stride; g.up_offset = up_offset;
    g.bias = bias; g.bias_dtype = bias_dtype; g.C = C; g.ldc = ldc; g.row_scale = row_scale;
    g.a_rows = a_rows; g.c_rows = c_rows; g.expert_offsets = expert_offsets; g.E = E; g.M = M; g.N = N; g.K = K;
    g.pair_ids = pair_ids; g.pair_div = pair_div; g.act = act;
    g.kb_stride = kb_rows * 64;
    FX_REQUIRE(kb_rows >= 0 && (kb_rows == 0 || (dtype == FX_BF16 && K % 64 == 0 && ((uintptr_t)W % 16) == 0 && lda % 8 == 0 &&
                                                 ((uintptr_t)A % 16) == 0 && (up_offset % K) == 0)),
               "gemm: weights in slabs of 64 k are bfloat16 with K a multiple of 64 and aligned operands");
    g.n_always = n_always; g.always_rows = always_rows; g.always_from_a = always_from_a;
    FX_REQUIRE(n_always >= 0 && (n_always == 0 || (pair_ids && always_rows >= 1 && always_rows <= 16)),
               "gemm: experts that every row takes come with unsorted pairs and at most 16 rows");
    hipStream_t s = (hipStream_t)stream;
    const int nonempty = expert_offsets ? (E < M ? E : M) : 0;
    if (dtype == FX_F32) {
        g.vec_ok = 0;
        const int m_tiles = M / 64 + (expert_offsets ? nonempty : (M % 64 != 0));
        dim3 grid(ceil_div(N, 64), m_tiles);
        switch (epi) {
            case EPI_STORE:
            case EPI_STORE_F32: gemm_f32_kernel<false, EPI_STORE_F32><<<grid, 256, 0, s>>>(g); break;
            case EPI_RESID: gemm_f32_kernel<false, EPI_RESID><<<grid, 256, 0, s>>>(g); break;
            default: gemm_f32_kernel<true, EPI_GATED><<<grid, 256, 0, s>>>(g); break;
        }
        FX_CHECK_LAUNCH("gemm_f32");
        return 0;
    }
    g.vec_ok = norm_w != nullptr ||
               ((K % 8 == 0) && (lda % 8 == 0) && (w_stride % 8 == 0) && (up_offset % 8 == 0) &&
                (((uintptr_t)A | (uintptr_t)W) % 16 == 0));
    const long per_group = expert_offsets ? (M + E - 1) / E : M;
    const bool wide_ok = g.vec_ok && K % 64 == 0 && !g_no_wide;
    FX_REQUIRE(!pair_ids || g.vec_ok, "gemm: unsorted pairs need K a multiple of 8 and 16-byte aligned rows");
    // 17..64 plain rows against very many weight rows (the head): tiles of 128 rows stream the weights at the same
    // speed whatever the rows (151,936 weight rows: 131-136 us from 1 to 33 rows), the kernel for few rows slows
    // down with them (98 us at 1 row, 101 at 8; decode steps of 12 and 16 sequences are 20 us shorter with it, those
    // of 24 and 32 the same either way)
    const bool many_columns = g.vec_ok && !expert_offsets && !pair_ids && !norm_w && !row_ss && !g.kb_stride && M > g_head_rows && K % 64 == 0 &&
                              !g_no_wide && ceil_div(N, 128) >= 512;
    // Rows sorted by expert: the product for few rows only up to three rows an expert on average.  Its waves fetch
    // every row tile's operands themselves, so its time grows with the rows (512 tokens of the larger model, 64 rows
    // an expert: 1,107 us for the gate/up product at 2.1 TB/s), while the tiled product, whose tile of 192 rows
    // holds an expert's share, streams the weights at the same speed whatever the rows (400 us at 5.9 TB/s); decode
    // steps of 48 and 64 sequences 10.3 -> 10.0 and 12.0 -> 11.4 ms, of 17 to 64 of the larger model's sizes 8-24 %
    // less; with three rows an expert the product for few rows is still 1-2 % ahead of the tiles of 64 rows.
    // 65 to 256 plain rows against so few weight rows that the tiled kernel, whose smallest tiles are 128 x 128, would
    // run on 32 CUs or fewer (the attention's output product): its chain of K steps takes 20-25 us whatever the rows,
    // the product for few rows, 32 or 64 rows a block, streams the weights through every CU (2,048 x 2,048 weights:
    // 11 us up to 128 rows and 18 us up to 256 against 20-24 us; 3,584 x 3,584: 26-30 us up to 128 rows against 31-39;
    // with 48 tiles, the q/k/v product, the tiled kernel is ahead)
    const bool few_tiles = !expert_offsets && !pair_ids && M > 64 && M <= 256 && (long)ceil_div(N, 128) * ceil_div(M, 128) <= 32 && !g_wide_force;
    const long plain_limit = g_plain_rows > 0 ? g_plain_rows : (few_tiles ? 256 : 64);
    const long few_limit = expert_offsets ? (wide_ok ? g_few_rows : 64) : plain_limit;
    if (g.vec_ok && (per_group <= few_limit || pair_ids) && !many_columns) {
        int mt = pair_ids ? 1 : (per_group <= 16 ? 1 : (per_group <= 32 ? 2 : 4));
        if (!expert_offsets && !pair_ids && M > 64 && (long)ceil_div(N, 32) * ceil_div(M, 64) < 256) mt = 2;     // more blocks where they are few
        const bool dual = epi == EPI_GATED;
        // 33 to 64 plain rows against few weight rows (the attention's output product: 2,048): four row tiles a
        // block leave 128 blocks; a block per row tile, with two sets of weight rows, gives 256 and every block a
        // quarter of the rows' operands to fetch (13.4 -> 9.1 us at 64 rows, 11.2 -> 9.0 at 40; with 6,144 weight
        // rows the four row tiles a block stay ahead, 17.3 against 20.1 us)
        const bool spread_rows = mt == 4 && !expert_offsets && !norm_w && epi == EPI_RESID && ceil_div(N, 16) * (long)ceil_div(M, 64) < 192;
        if (spread_rows) mt = 1;
        if (g_skinny_mt && !pair_ids) mt = g_skinny_mt;
        const int m_tiles = pair_ids ? (M < E ? M : E) + M / 16 + n_always
                                     : M / (16 * mt) + (expert_offsets ? nonempty : (M % (16 * mt) != 0));
        // two sets of weight rows per wave share the activations they multiply and halve the blocks' fixed
        // work; one set when that would leave too few blocks to keep the memory busy, or when a row or two meet
        // so many weight rows that the blocks are plenty either way (measured on the sizes of the engine)
        int nw = (dual || (long)ceil_div(N, 32) * m_tiles >= 160) ? 2 : 1;
        if (!dual && (norm_w || (M <= 2 && (long)ceil_div(N, 16) * m_tiles >= 4096))) nw = 1;
        if (spread_rows) nw = 2;
        if ((g_skinny_nw == 1 && !dual) || (g_skinny_nw == 2 && !norm_w)) nw = g_skinny_nw;
        // Waves per block: four, a part of K each, for unsorted pairs too.  (Those ran with one wave that went
        // through all four parts, or two, while a wave found its tile with a loop over the experts and each such
        // search cost 1-2 us; since the search is a few ballots, four waves are ahead again: decode steps of 1, 4, 8
        // and 16 sequences 1.87, 2.80, 3.70 and 5.17 ms with one or two waves, 1.84, 2.72, 3.64 and 5.06 ms with four.)
        // The sums are the same bits with one, two and four waves.
        int waves = 4;
        if (expert_offsets && mt == 1) waves = 2;      // sorted, up to 16 rows per expert: 152 against 159 us at 64 tokens
        if (g_skinny_waves == 8 || g_skinny_waves == 4 || g_skinny_waves == 2 || g_skinny_waves == 1) waves = g_skinny_waves;
        launch_skinny(g, epi, mt, nw, waves, m_tiles, s);
        FX_CHECK_LAUNCH("gemm_bf16_skinny");
        return 0;
    }
    FX_REQUIRE(!g.kb_stride || wide_ok, "gemm: no kernel for weights in slabs of 64 k at these sizes");
    if (per_group <= 64 && !many_columns && !wide_ok) {
        const int m_tiles = M / 64 + (expert_offsets ? nonempty : (M % 64 != 0));
        launch_bf16<64, 64, 32, 32>(g, epi, m_tiles, s);
    } else if (g.vec_ok && K % 64 == 0 && !g_no_wide) {
        // the widest tile that still gives the CUs (one block each) an even share of the work
        const bool dual = epi == EPI_GATED;
        const long cus = fx_compute_units();
        const int force = expert_offsets && g_wide_grouped ? g_wide_grouped : g_wide_force;
        // weights that are read about once (an expert's rows fit one row tile on average; plain rows: one row tile)
        // are loaded with the non-temporal hint
        g.stream_w = g_stream_w >= 0 ? g_stream_w : (expert_offsets ? per_group <= 128 : M <= 128);
        auto tiles = [&](int tm, int tn) {
            return (long)ceil_div(N, dual ? tn / 2 : tn) * (M / tm + (expert_offsets ? nonempty : (M % tm != 0)));
        };
        auto score = [&](int tm, int tn, double quality) {
            const long t = tiles(tm, tn);
            // plain rows: the share of a tile's rows that exist (an expert's missing row blocks are skipped)
            const double rows = expert_offsets ? 1.0 : (double)M / (double)((long)ceil_div(M, tm) * tm);
            return quality * rows * (double)t / (double)(ceil_div(t, cus) * cus);
        };
        double s256 = score(256, 256, 1.0), s192 = dual || expert_offsets ? 0.0 : score(256, 192, 0.92), s128 = score(256, 128, 0.85),
               s64 = score(128, 128, 0.7);
        if (force) {
            s256 = force == 256; s192 = force == 192 && !dual; s128 = force == 128; s64 = 0.5 * (force == 64);
        }
        // an expert's share of up to 192 rows: the product streams the weights once and multiplies little, so it
        // is bound by how many of them are on their way; a ring of three weight tiles beside two of the rows
        // plain rows: tiles of 192 x 256 where they divide the work more evenly (2,048 rows against 11,264 weight
        // rows: 484 tiles for two rounds of the 256 CUs instead of 352 tiles of 256 x 256)
        const double s12 = expert_offsets ? 0.0 : score(192, 256, 0.92);
        // (an expert's share beyond 192 rows: tiles of 192 rows too where they leave fewer empty rows than tiles of
        // 256 do, 273 rows an expert as 2 x 192 instead of 2 x 256: the down product of a 4,096-token step 173
        // against 190 us)
        const long pad192 = ceil_div(per_group, 192) * 192L, pad256 = ceil_div(per_group, 256) * 256L;
        const bool few_rows = force ? force == 12
                                           : (expert_offsets ? (per_group <= 176 || pad192 < pad256)
                                                             : (s12 > s256 && s12 > s192 && s12 > s128 && s12 > s64));
        // an expert's share of up to 20 rows on average: a tile of 64 rows leaves LDS for a ring of four weight tiles
        // beside two of the rows (2-5 % less time than tiles of 192 rows with a ring of three, the same bits: decode
        // at 64 sequences 11.2 -> 11.0 ms, a 192-token step 6.8 -> 6.4 ms; from 25 rows on average on, steps of 384
        // tokens, more and more experts need a second tile and it falls behind)
        if (force == 4 || (!force && expert_offsets && per_group <= g_tile64_rows))
            launch_wide<4, 256, 4, 2>(g, epi, M / 64 + (expert_offsets ? nonempty : (M % 64 != 0)), s);
        else if (few_rows)
            launch_wide<12, 256, 3, 2>(g, epi, M / 192 + (expert_offsets ? nonempty : (M % 192 != 0)), s);
        else if (s192 > s256 && s192 >= s128 && s192 >= s64)
            launch_wide<16, 192, 2>(g, epi, M / 256 + (expert_offsets ? nonempty : (M % 256 != 0)), s);
        else if (s256 >= s128 && s256 >= s64)
            launch_wide<16, 256, 2>(g, epi, M / 256 + (expert_offsets ? nonempty : (M % 256 != 0)), s);
        else if (s128 >= s64)
            launch_wide<16, 128, 3>(g, epi, M / 256 + (expert_offsets ? nonempty : (M % 256 != 0)), s);
        else
            launch_wide<8, 128, 4>(g, epi, M / 128 + (expert_offsets ? nonempty : (M % 128 != 0)), s);
    } else {
        const int m_tiles = M / 128 + (expert_offsets ? nonempty : (M % 128 != 0));
        const bool dual = epi == EPI_GATED;
        // narrow outputs: tiles of 64 columns give the CUs at least two blocks each
        if (!dual && (long)ceil_div(N, 128) * m_tiles < 2L * fx_compute_units())
            launch_bf16<128, 64, 64, 32>(g, epi, m_tiles, s);
        else
            launch_bf16<128, 128, 64, 64>(g, epi, m_tiles, s);
    }
    FX_CHECK_LAUNCH("gemm_bf16");
    return 0;
}
