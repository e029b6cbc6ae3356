// Routing of tokens to experts.
//
//  fx_router_select : from float32 router logits, a gating function over all
//                   experts, the k best, optional renormalisation; and the
//                   scalar sigmoid gate of a shared expert.
//  fx_moe_align   : sorts the (token, slot) pairs by expert with a stable
//                   counting sort, so that a grouped matrix product sees each
//                   expert's rows together.
#include "common.h"

FX_DEFINE_LAST_ERROR()

#define E_MAX 1024
#define K_MAX 32
#define NEG_INFINITY_F (-INFINITY)

enum { GATE_SOFTMAX = 0, GATE_SIGMOID = 1 };

// One wave per token, four tokens per block.  Input: float32 router logits
// [T, ld] (products of the activations with the router matrix, no bias;
// ferrox-models/src/decoder.rs:2915), optionally with the shared expert's gate
// logit in column E.
//   softmax over all E with max subtraction, then the k largest probabilities,
//   weights = those probabilities, divided by their sum if `renorm`
//   (ferrox-moe/src/lib.rs:333-355).  Ties: higher probability first, then the
//   lower expert index (the rule of ferrox-metal/src/gpu.rs:686-699).
//   GATE_SIGMOID scores each expert with 1/(1+exp(-logit)) instead
//   (ferrox-moe/src/lib.rs:100-121).
//   gate_out[t] = sigmoid(logits[t, E])  (decoder.rs:2670-2672).
// The best (score, expert) of the wave in every lane: higher score first, then the lower expert.  Six exchanges
// that stay in the vector unit (pairs inside a quad, quads, halves of a row of 16 lanes by DPP moves; rows and halves
// of the wave by the lane-swapping moves of gfx950): the order is total, so the result is the one that exchanges
// through the LDS crossbar gave, and a selection of k experts no longer waits 12 k times for that crossbar.
__device__ __forceinline__ void better_of(float& best, int& bi, float ob, int oi) {
    if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bi = oi;
    }
}
template <int CTRL>
__device__ __forceinline__ void argmax_dpp_step(float& best, int& bi) {
    const float ob = __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(best), CTRL, 0xF, 0xF, true));
    const int oi = __builtin_amdgcn_update_dpp(0, bi, CTRL, 0xF, 0xF, true);
    better_of(best, bi, ob, oi);
}
__device__ __forceinline__ void wave_argmax(float& best, int& bi) {
    argmax_dpp_step<0xB1>(best, bi);      // quad_perm [1,0,3,2]
    argmax_dpp_step<0x4E>(best, bi);      // quad_perm [2,3,0,1]
    argmax_dpp_step<0x141>(best, bi);     // row_half_mirror: the quads of eight lanes
    argmax_dpp_step<0x140>(best, bi);     // row_mirror: the halves of a row
    {
        const unsigned ub = __float_as_uint(best), ui = (unsigned)bi;
        const auto a = __builtin_amdgcn_permlane16_swap(ub, ub, false, false);
        const auto b = __builtin_amdgcn_permlane16_swap(ui, ui, false, false);
        best = __uint_as_float(a[0]);
        bi = (int)b[0];
        better_of(best, bi, __uint_as_float(a[1]), (int)b[1]);
    }
    {
        const unsigned ub = __float_as_uint(best), ui = (unsigned)bi;
        const auto a = __builtin_amdgcn_permlane32_swap(ub, ub, false, false);
        const auto b = __builtin_amdgcn_permlane32_swap(ui, ui, false, false);
        best = __uint_as_float(a[0]);
        bi = (int)b[0];
        better_of(best, bi, __uint_as_float(a[1]), (int)b[1]);
    }
}

// selection for one token by one wave; `score` is E floats of LDS owned by the wave
// (`es`: distance between the logits of neighbouring experts, 1 for a row of a [T, E] matrix)
__device__ __forceinline__ void select_token(const float* __restrict__ row, float* score, int t, int E, int k, int renorm,
                                             int gating, int* __restrict__ ids, float* __restrict__ weights,
                                             float* __restrict__ gate_out, int* ids_copy, long es = 1) {
    const int lane = threadIdx.x & 63;
    if (gate_out && lane == 0) gate_out[t] = 1.0f / (1.0f + expf(-row[E * es]));
    if (E <= 64) {
        // a lane per expert: the same sums and comparisons as below (whose loops then run once), with the scores
        // in registers, so that no round waits for LDS or for the store of the round before
        const bool mine = lane < E;
        const float x = mine ? row[lane * es] : 0.f;
        float sc;
        if (gating == GATE_SOFTMAX) {
            const float mx = wave_max(mine ? x : NEG_INFINITY_F);
            const float ex = mine ? expf(x - mx) : 0.f;
            const float sum = wave_sum(ex);
            sc = ex / sum;
        } else {
            sc = 1.0f / (1.0f + expf(-x));
        }
        if (!(sc >= 0.f)) sc = 0.f;     // a NaN logit makes every score NaN: such scores count as zero, so a choice stays in range
        if (!mine) sc = -1.f;           // below every score, like the loop's start value
        float wsum = 0.f, my_w = 0.f;
        int my_id = 0;
        for (int j = 0; j < k; ++j) {
            float best = sc;
            int bi = mine ? lane : 0x7fffffff;
            wave_argmax(best, bi);
            if (lane == j) {
                my_w = best;
                my_id = bi;
            }
            if (lane == bi) sc = -2.f;  // scores are >= 0; taken out of the race
            wsum += best;
        }
        if (lane < k) {
            store_shared(ids + t * k + lane, my_id);      // (at device scope: a block of this launch may sort them)
            if (ids_copy) ids_copy[t * k + lane] = my_id;
            weights[t * k + lane] = renorm ? my_w / wsum : my_w;
        }
        return;
    }
    if (gating == GATE_SOFTMAX) {
        float mx = NEG_INFINITY_F;
        for (int e = lane; e < E; e += 64) mx = fmaxf(mx, row[e * es]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < E; e += 64) {
            const float ex = expf(row[e * es] - mx);
            score[e] = ex;
            sum += ex;
        }
        sum = wave_sum(sum);
        for (int e = lane; e < E; e += 64) score[e] = score[e] / sum;
    } else {
        for (int e = lane; e < E; e += 64) score[e] = 1.0f / (1.0f + expf(-row[e * es]));
    }
    __builtin_amdgcn_wave_barrier();
    // k rounds of "largest remaining", lower index on ties
    float wsum = 0.f;
    float my_w = 0.f;  // lane j keeps the weight of selection j
    for (int j = 0; j < k; ++j) {
        float best = -1.f;
        int bi = 0x7fffffff;
        for (int e = lane; e < E; e += 64) {
            float v = score[e];
            if (!(v >= 0.f) && v != -2.f) v = 0.f;   // NaN counts as zero (see above): some expert in range is always found
            if (v > best) {  // ascending e within a lane: the first maximum is kept
                best = v;
                bi = e;
            }
        }
        wave_argmax(best, bi);
        if (lane == j) my_w = best;
        if (lane == 0) {
            store_shared(ids + t * k + j, bi);
            if (ids_copy) ids_copy[t * k + j] = bi;
            score[bi] = -2.f;  // scores are >= 0; taken out of the race
        }
        wsum += best;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    if (lane < k) weights[t * k + lane] = renorm ? my_w / wsum : my_w;
}

__global__ __launch_bounds__(256) void router_select_kernel(const float* __restrict__ logits, long ld, long es, int T,
                                                            int E, int k, int renorm, int gating, int* __restrict__ ids,
                                                            float* __restrict__ weights, float* __restrict__ gate_out) {
    extern __shared__ float score_all[];   // 4 x E
    const int wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= T) return;
    select_token(logits + (size_t)t * ld, score_all + wave * E, t, E, k, renorm, gating, ids, weights, gate_out, nullptr, es);
}

// logits of token t and expert e stand at logits[t * ld + e * es] (either of the two may be 1)
FX_API int fx_router_select(void* stream, const float* logits, long ld, long es, int T, int E, int k, int renorm,
                            int gating, int* ids, float* weights, float* gate_out) {
    FX_REQUIRE(T >= 0, "router: bad size T=%d", T);
    FX_REQUIRE(ld >= 1 && es >= 1, "router: bad strides %ld, %ld", ld, es);
    FX_REQUIRE(E >= 1 && E <= E_MAX, "router: %d experts, this kernel takes 1..%d", E, E_MAX);
    FX_REQUIRE(k >= 1 && k <= E && k <= K_MAX, "router: top-k %d must lie in 1..min(E, %d)", k, K_MAX);
    FX_REQUIRE(T <= 1 || es > 1 || ld >= E + (gate_out ? 1 : 0), "router: logits rows of %ld hold fewer than %d columns",
               ld, E + (gate_out ? 1 : 0));
    FX_REQUIRE(gating == GATE_SOFTMAX || gating == GATE_SIGMOID, "router: unknown gating %d", gating);
    if (T == 0) return 0;
    router_select_kernel<<<(T + 3) / 4, 256, 4 * E * sizeof(float), (hipStream_t)stream>>>(logits, ld, es, T, E, k, renorm,
                                                                                         gating, ids, weights, gate_out);
    FX_CHECK_LAUNCH("router_select");
    return 0;
}

// ---------------------------------------------------------------------------
// Stable counting sort of n = T*k (token, slot) pairs by expert, one block.
//   expert_offsets[E+1] : rows of expert e are [off[e], off[e+1])
//   sorted_token[i]     : token of sorted row i
//   sorted_pair[i]      : pair t*k + j of sorted row i
//   inv[t*k + j]        : sorted row of pair (t, j)
// The pairs are taken in groups of 64, a group per wave at a time.  Inside a
// group the lanes find, with one ballot per bit of the expert id, which lanes hold
// the same expert: that gives a pair's rank among its group's pairs of that
// expert and the group's count cnt[group][expert].  Then, per expert, a scan over
// the groups (lanes = groups) turns the counts into the number of earlier pairs;
// a scan over the experts' totals gives the offsets; and every pair is placed at
// offset + earlier groups + rank.  The order inside an expert is the order of the
// pairs, whatever the number of waves.
// ---------------------------------------------------------------------------
// lanes (of the 64 of a wave) whose `e` equals this lane's; e < 2^bits, e < 0 matches nothing
__device__ __forceinline__ unsigned long long same_expert_lanes(int e, int bits) {
    unsigned long long m = __ballot(e >= 0);
    for (int b = 0; b < bits; ++b) {
        const unsigned long long set = __ballot((e >> b) & 1);
        m &= ((e >> b) & 1) ? set : ~set;
    }
    return e >= 0 ? m : 0ull;
}

// the sort itself, by one block of whole waves; `offs` (E+1 ints) and `cnt` (rows*E ints) are LDS;
// a row is `per_row` consecutive groups, rows = ceil(ceil(n/64) / per_row)
template <bool SHARED_IDS = false>       // SHARED_IDS: other blocks of this launch wrote the ids with store_shared()
__device__ __forceinline__ void align_block(const int* ids, int n, int k, int E, int per_row, int* offs, int* cnt,
                                            int* __restrict__ expert_offsets, int* __restrict__ sorted_token,
                                            int* __restrict__ sorted_pair, int* __restrict__ inv) {
    const int nt = blockDim.x, th = threadIdx.x, lane = th & 63, wave = th >> 6, n_waves = nt >> 6;
    const int G = (n + 63) >> 6, R = (G + per_row - 1) / per_row;
    int bits = 0;
    while ((1 << bits) < E) ++bits;
    for (int i = th; i < R * E; i += nt) cnt[i] = 0;
    __syncthreads();
    for (int r = wave; r < R; r += n_waves) {          // a row belongs to one wave, its groups in order
        for (int g = r * per_row; g < min(G, (r + 1) * per_row); ++g) {
            const int i = g * 64 + lane;
            int e = i < n ? (SHARED_IDS ? load_shared(ids + i) : ids[i]) : -1;
            if (e >= E) e = -1;
            const unsigned long long same = same_expert_lanes(e, bits);
            if (e >= 0 && lane == __ffsll((long long)same) - 1) cnt[r * E + e] += __popcll(same);
        }
    }
    __syncthreads();
    // per expert: counts of the rows -> pairs in earlier rows; the total goes to offs[e + 1]
    for (int e = wave; e < E; e += n_waves) {
        int carry = 0;
        for (int base = 0; base < R; base += 64) {
            const int r = base + lane;
            const int c = r < R ? cnt[r * E + e] : 0;
            const int v = wave_inclusive_sum(c);
            if (r < R) cnt[r * E + e] = carry + v - c;
            carry += __builtin_amdgcn_readlane(v, 63);
        }
        if (lane == 0) offs[e + 1] = carry;
    }
    __syncthreads();
    if (th < 64) {   // inclusive scan of the totals by the first wave, 64 experts at a time
        int carry = 0;
        if (lane == 0) offs[0] = 0;
        for (int base = 0; base < E; base += 64) {
            const int e = base + lane;
            const int v = wave_inclusive_sum(e < E ? offs[e + 1] : 0);
            if (e < E) offs[e + 1] = carry + v;
            carry += __builtin_amdgcn_readlane(v, 63);
        }
    }
    __syncthreads();
    for (int e = th; e <= E; e += nt) expert_offsets[e] = offs[e];
    for (int r = wave; r < R; r += n_waves) {
        for (int g = r * per_row; g < min(G, (r + 1) * per_row); ++g) {
            const int i = g * 64 + lane;
            int e = i < n ? (SHARED_IDS ? load_shared(ids + i) : ids[i]) : -1;
            if (e >= E) e = -1;
            const unsigned long long same = same_expert_lanes(e, bits);
            int before = 0;
            if (e >= 0) before = cnt[r * E + e];       // pairs of this expert in earlier rows and groups
            __builtin_amdgcn_wave_barrier();
            if (e >= 0) {
                const int dst = offs[e] + before + __popcll(same & ((1ull << lane) - 1ull));
                sorted_token[dst] = i / k;
                if (sorted_pair) sorted_pair[dst] = i;
                if (inv) inv[i] = dst;
                if (lane == __ffsll((long long)same) - 1) cnt[r * E + e] = before + __popcll(same);
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// groups per row such that the rows' counters fit `bytes` of LDS beside the offsets
static int align_groups_per_row(long n, int E, size_t bytes, size_t* shm) {
    const long G = (n + 63) / 64;
    long max_rows = ((long)bytes - (long)(E + 1) * 4) / ((long)E * 4);
    if (max_rows < 1) max_rows = 1;
    long per_row = (G + max_rows - 1) / max_rows;
    if (per_row < 1) per_row = 1;
    const long R = (G + per_row - 1) / per_row;
    *shm = (size_t)(E + 1) * 4 + (size_t)(R > 0 ? R : 1) * E * 4;
    return (int)per_row;
}

__device__ __forceinline__ void align_always(int n, int k, int E, int* __restrict__ expert_offsets,
                                             int* __restrict__ sorted_token, int* __restrict__ sorted_pair, int n_always) {
    const int T = n / k;
    for (int i = threadIdx.x; i < n_always * T; i += blockDim.x) {
        sorted_token[n + i] = i % T;
        if (sorted_pair) sorted_pair[n + i] = n + i;
    }
    for (int s = threadIdx.x; s < n_always; s += blockDim.x) expert_offsets[E + 1 + s] = n + (s + 1) * T;
}

// After the experts, `n_always` further ones that each of the n / k tokens takes (a shared expert cut into pieces):
// piece s owns the sorted rows n + s T .. n + (s + 1) T, row n + s T + t being token t, and its output row has the
// same number.
__global__ __launch_bounds__(1024) void moe_align_kernel(const int* __restrict__ ids, int n, int k, int E, int per_row,
                                                         int* __restrict__ expert_offsets,
                                                        int* __restrict__ sorted_token, int* __restrict__ sorted_pair,
                                                        int* __restrict__ inv, int n_always) {
    extern __shared__ int lds[];
    align_block(ids, n, k, E, per_row, lds, lds + E + 1, expert_offsets, sorted_token, sorted_pair, inv);
    align_always(n, k, E, expert_offsets, sorted_token, sorted_pair, n_always);
}

// Many pairs: the same sort by many blocks, in two launches.  First every wave counts the experts of its
// group of 64 pairs into gcnt[group][expert].  Then every block adds up, per expert, the counts of all groups
// (the offsets) and of the groups before its own (the pairs that come earlier), and its waves place their
// groups' pairs; block 0 also writes the offsets out.  The order inside an expert is the order of the pairs.
#define SORT_WAVES 4
__global__ __launch_bounds__(SORT_WAVES * 64) void moe_count_kernel(const int* __restrict__ ids, int n, int E,
                                                                    int* __restrict__ gcnt) {
    extern __shared__ int lds[];                    // SORT_WAVES rows of E counts
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = blockIdx.x * SORT_WAVES + wave;
    if (g * 64 >= n) return;
    int* row = lds + wave * E;
    int bits = 0;
    while ((1 << bits) < E) ++bits;
    for (int e = lane; e < E; e += 64) row[e] = 0;
    __builtin_amdgcn_wave_barrier();
    const int i = g * 64 + lane;
    int e = i < n ? ids[i] : -1;
    if (e >= E) e = -1;
    const unsigned long long same = same_expert_lanes(e, bits);
    if (e >= 0 && lane == __ffsll((long long)same) - 1) row[e] = __popcll(same);
    __builtin_amdgcn_wave_barrier();
    for (int x = lane; x < E; x += 64) gcnt[(size_t)g * E + x] = row[x];
}

__global__ __launch_bounds__(SORT_WAVES * 64) void moe_place_kernel(const int* __restrict__ ids, int n, int k, int E,
                                                                    const int* __restrict__ gcnt,
                                                                    int* __restrict__ expert_offsets,
                                                                    int* __restrict__ sorted_token,
                                                                    int* __restrict__ sorted_pair, int* __restrict__ inv) {
    extern __shared__ int lds[];
    int* offs = lds;                                // E + 1: first sorted row of each expert
    int* before = lds + E + 1;                      // E: pairs of the expert in groups before this block's
    int* part = before + E;                         // SORT_WAVES x 2 x E partial sums
    const int th = threadIdx.x, lane = th & 63, wave = th >> 6;
    const int G = (n + 63) >> 6, g0 = blockIdx.x * SORT_WAVES;
    int bits = 0;
    while ((1 << bits) < E) ++bits;
    // wave w adds the groups w, w + SORT_WAVES, ...: all of them, and those before g0
    for (int e = lane; e < E; e += 64) {
        int all = 0, early = 0;
        for (int gb = wave; gb < G; gb += 8 * SORT_WAVES) {       // eight counts are fetched together
            int c[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) c[u] = gcnt[(size_t)min(gb + u * SORT_WAVES, G - 1) * E + e];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int g = gb + u * SORT_WAVES;
                if (g < G) all += c[u];
                if (g < G && g < g0) early += c[u];
            }
        }
        part[(wave * 2) * E + e] = all;
        part[(wave * 2 + 1) * E + e] = early;
    }
    __syncthreads();
    for (int e = th; e < E; e += SORT_WAVES * 64) {
        int all = 0, early = 0;
#pragma unroll
        for (int w = 0; w < SORT_WAVES; ++w) {
            all += part[(w * 2) * E + e];
            early += part[(w * 2 + 1) * E + e];
        }
        offs[e + 1] = all;
        before[e] = early;
    }
    __syncthreads();
    if (th < 64) {   // inclusive scan of the totals by the first wave, 64 experts at a time
        int carry = 0;
        if (lane == 0) offs[0] = 0;
        for (int base = 0; base < E; base += 64) {
            const int e = base + lane;
            const int v = wave_inclusive_sum(e < E ? offs[e + 1] : 0);
            if (e < E) offs[e + 1] = carry + v;
            carry += __builtin_amdgcn_readlane(v, 63);
        }
    }
    __syncthreads();
    if (blockIdx.x == 0)
        for (int e = th; e <= E; e += SORT_WAVES * 64) expert_offsets[e] = offs[e];
    const int g = g0 + wave;
    if (g >= G) return;
    const int i = g * 64 + lane;
    int e = i < n ? ids[i] : -1;
    if (e >= E) e = -1;
    if (e < 0) return;                              // (ballots below are taken by the lanes that have a pair)
    int earlier = before[e];
    for (int w = 0; w < wave; ++w) earlier += gcnt[(size_t)(g0 + w) * E + e];     // this block's groups before mine
    unsigned long long same = __ballot(1);
    for (int b = 0; b < bits; ++b) {
        const unsigned long long set = __ballot((e >> b) & 1);
        same &= ((e >> b) & 1) ? set : ~set;
    }
    const int dst = offs[e] + earlier + __popcll(same & ((1ull << lane) - 1ull));
    sorted_token[dst] = i / k;
    if (sorted_pair) sorted_pair[dst] = i;
    if (inv) inv[i] = dst;
}

// few tokens: selection (a wave per token) and the sort in one block of 16 waves
__global__ __launch_bounds__(1024) void router_select_align_kernel(const float* __restrict__ logits, long ld, int T, int E,
                                                                  int k, int renorm, int gating, int* __restrict__ ids,
                                                                  float* __restrict__ weights, float* __restrict__ gate_out,
                                                                  int* __restrict__ expert_offsets,
                                                                  int* __restrict__ sorted_token,
                                                                  int* __restrict__ sorted_pair, int* __restrict__ inv) {
    extern __shared__ int lds[];
    float* score = (float*)lds;                 // 16 x E
    int* ids_s = lds + 16 * E;                  // T * k
    int* offs = ids_s + T * k;                  // E + 1
    int* cnt = offs + E + 1;                    // groups x E
    const int wave = threadIdx.x >> 6;
    if (wave < T)
        select_token(logits + (size_t)wave * ld, score + wave * E, wave, E, k, renorm, gating, ids, weights, gate_out, ids_s);
    __syncthreads();
    align_block(ids_s, T * k, k, E, 1, offs, cnt, expert_offsets, sorted_token, sorted_pair, inv);
}

// ---------------------------------------------------------------------------
// Few tokens (decode, up to 64): everything in front of the experts in one launch.
// Block (r, t): RMSNorm of row t of the float32 residual stream (same formula and
// rounding as rmsnorm_kernel; block r = 0 writes it out as bfloat16 for the
// experts), then the products of that rounded row with router rows 8r .. 8r+7,
// two rows per wave, k in a fixed order, into `logits`.  The token's block that
// finishes last selects its experts.  Nothing is sorted: with so few rows the
// expert products group the (token, slot) pairs themselves.
// ---------------------------------------------------------------------------
#define FRONT_THREADS 256
#define FRONT_WAVES (FRONT_THREADS / 64)
#define FRONT_ROWS (2 * FRONT_WAVES)   // router rows per block

__device__ __forceinline__ float dot8(uint4 w, const float* x) {
    float a = 0.f;
    a = fmaf(__uint_as_float(w.x << 16), x[0], a);
    a = fmaf(__uint_as_float(w.x & 0xffff0000u), x[1], a);
    a = fmaf(__uint_as_float(w.y << 16), x[2], a);
    a = fmaf(__uint_as_float(w.y & 0xffff0000u), x[3], a);
    a = fmaf(__uint_as_float(w.z << 16), x[4], a);
    a = fmaf(__uint_as_float(w.z & 0xffff0000u), x[5], a);
    a = fmaf(__uint_as_float(w.w << 16), x[6], a);
    a = fmaf(__uint_as_float(w.w & 0xffff0000u), x[7], a);
    return a;
}

#define FRONT_MAX_TOKENS 256
__global__ __launch_bounds__(FRONT_THREADS) void moe_front_kernel(
    const float* __restrict__ h, long ldh, const void* __restrict__ gamma, int gamma_dtype, float eps,
    bf16* __restrict__ x_out, const bf16* __restrict__ W, int H, int T, int E, int has_gate, int k, int renorm,
    int gating, float* logits, int* ids, float* __restrict__ weights, float* __restrict__ gate_out,
    unsigned* counters, int* __restrict__ expert_offsets, int* __restrict__ sorted_token, int* __restrict__ sorted_pair,
    int* __restrict__ inv, int n_always, int per_row) {
    extern __shared__ int lds[];
    __shared__ float red[FRONT_WAVES];
    float* xs = (float*)lds;            // H: the normed row as the experts will read it
    const int t = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_rows = E + has_gate, chunks = H >> 3;

    // this wave's two router rows
    const int e_a = blockIdx.x * FRONT_ROWS + wave, e_b = e_a + FRONT_WAVES;
    const bf16* wa = e_a < n_rows ? W + (size_t)e_a * H : nullptr;
    const bf16* wb = e_b < n_rows ? W + (size_t)e_b * H : nullptr;
    const float* row = h + (size_t)t * ldh;
    float acc_a = 0.f, acc_b = 0.f;

    if (H <= FRONT_THREADS * 16) {
        // Usual widths: everything this thread reads from memory (its part of the router's rows, of the
        // residual row and of the norm's weights) is asked for at once, so that the kernel waits for memory
        // once.  Elements go to threads and are summed as in rmsnorm_kernel: the same bits.
        constexpr int NC = FRONT_THREADS * 16 / 8 / 64;      // 16-byte pieces of a router row per lane
        uint4 pa[NC], pb[NC];
#pragma unroll
        for (int i = 0; i < NC; ++i) {
            const int c = lane + 64 * i;
            pa[i] = (wa && c < chunks) ? *(const uint4*)(wa + c * 8) : make_uint4(0, 0, 0, 0);
            pb[i] = (wb && c < chunks) ? *(const uint4*)(wb + c * 8) : make_uint4(0, 0, 0, 0);
        }
        float xv[16], gv[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = tid + i * FRONT_THREADS;
            xv[i] = c < H ? row[c] : 0.f;
        }
        load_strided_as_float<16, FRONT_THREADS>(gamma, gamma_dtype, tid, H, gv);
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) ss += xv[i] * xv[i];
        ss = block_sum<FRONT_WAVES>(ss, red);
        const float scale = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = tid + i * FRONT_THREADS;
            if (c < H) {
                const bf16 b = float_to_bf16(xv[i] * scale * gv[i]);
                if (blockIdx.x == 0) x_out[(size_t)t * H + c] = b;
                xs[c] = bf16_to_float(b);
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NC; ++i) {          // k in the order of the loop below
            const int c = lane + 64 * i;
            if (c < chunks) {
                acc_a += dot8(pa[i], xs + c * 8);
                acc_b += dot8(pb[i], xs + c * 8);
            }
        }
    } else {
        // their first loads leave before the norm is done
        uint4 pa = make_uint4(0, 0, 0, 0), pb = pa;
        if (lane < chunks) {
            if (wa) pa = *(const uint4*)(wa + lane * 8);
            if (wb) pb = *(const uint4*)(wb + lane * 8);
        }
        float ss = 0.f;
        for (int c = tid; c < H; c += FRONT_THREADS) {
            const float v = row[c];
            xs[c] = v;
            ss += v * v;
        }
        ss = block_sum<FRONT_WAVES>(ss, red);
        const float scale = 1.0f / sqrtf(ss / (float)H + eps);
        for (int c = tid; c < H; c += FRONT_THREADS) {
            const bf16 b = float_to_bf16(xs[c] * scale * load_as_float(gamma, gamma_dtype, c));
            if (blockIdx.x == 0) x_out[(size_t)t * H + c] = b;
            xs[c] = bf16_to_float(b);
        }
        __syncthreads();
        for (int c = lane; c < chunks; c += 64) {
            const int cn = c + 64;
            uint4 na = make_uint4(0, 0, 0, 0), nb = na;
            if (cn < chunks) {
                if (wa) na = *(const uint4*)(wa + cn * 8);
                if (wb) nb = *(const uint4*)(wb + cn * 8);
            }
            acc_a += dot8(pa, xs + c * 8);
            acc_b += dot8(pb, xs + c * 8);
            pa = na;
            pb = nb;
        }
    }
    acc_a = wave_sum(acc_a);
    acc_b = wave_sum(acc_b);
    if (lane == 0) {
        if (wa) store_shared(logits + (size_t)t * n_rows + e_a, acc_a);
        if (wb) store_shared(logits + (size_t)t * n_rows + e_b, acc_b);
    }

    if (!last_block_arrives(counters + t, gridDim.x)) return;
    if (wave == 0) {
        float* mine = (float*)lds;                  // n_rows logits, then E scores
        for (int e = lane; e < n_rows; e += 64) mine[e] = load_shared(logits + (size_t)t * n_rows + e);
        __builtin_amdgcn_wave_barrier();
        select_token(mine, mine + n_rows, t, E, k, renorm, gating, ids, weights, has_gate ? gate_out : nullptr, nullptr);
    }
    // with a place for the sorted layout: the block that selects the last token sorts all pairs by expert
    if (!expert_offsets) return;
    if (!last_block_arrives(counters + T, T)) return;
    align_block<true>(ids, T * k, k, E, per_row, lds, lds + E + 1, expert_offsets, sorted_token, sorted_pair, inv);
    align_always(T * k, k, E, expert_offsets, sorted_token, sorted_pair, n_always);
}

// Returns 2 (and launches nothing) for sizes this kernel does not take; the caller then runs the
// norm, the router product and the two routing kernels one after the other.  `logits` holds
// T x (E + has_gate) floats; `counters` are T + 1 zeroed unsigned in device memory, left at zero, that
// launches on one stream may share.  With `expert_offsets` (E + 1 + n_always ints), `sorted_token`, `sorted_pair`
// (T k + n_always T ints) and `inv` (T k, or null) the same launch also sorts the pairs by expert, as
// fx_moe_align does.
FX_API int fx_moe_front(void* stream, const float* h, long ldh, const void* gamma, int gamma_dtype, float eps,
                        void* x_out, const void* W, int H, int T, int E, int has_gate, int k, int renorm, int gating,
                        float* logits, int* ids, float* weights, float* gate_out, unsigned* counters,
                        int* expert_offsets, int* sorted_token, int* sorted_pair, int* inv, int n_always) {
    FX_REQUIRE(T >= 0 && H > 0, "moe_front: bad sizes T=%d H=%d", T, H);
    FX_REQUIRE(E >= 1 && E <= E_MAX, "router: %d experts, this kernel takes 1..%d", E, E_MAX);
    FX_REQUIRE(k >= 1 && k <= E && k <= K_MAX, "router: top-k %d must lie in 1..min(E, %d)", k, K_MAX);
    FX_REQUIRE(gating == GATE_SOFTMAX || gating == GATE_SIGMOID, "router: unknown gating %d", gating);
    FX_REQUIRE(gamma_dtype == FX_F32 || gamma_dtype == FX_BF16, "moe_front: unknown norm weight dtype %d", gamma_dtype);
    FX_REQUIRE(ldh >= H, "moe_front: rows of %ld hold fewer than %d columns", ldh, H);
    FX_REQUIRE(!has_gate || gate_out, "moe_front: a gate row needs a place for its output");
    const size_t front = (size_t)H * 4, back = (size_t)(2 * E + 1) * 4;
    size_t shm = front > back ? front : back, sort = 0;
    int per_row = 1;
    if (expert_offsets) {       // the sort's counters share the block's LDS
        FX_REQUIRE(sorted_token && n_always >= 0, "moe_front: the sorted layout needs its arrays");
        per_row = align_groups_per_row((long)T * k, E, 40 * 1024, &sort);
        if (sort > shm) shm = sort;
    }
    if (T > FRONT_MAX_TOKENS || H % 8 != 0 || ((uintptr_t)W % 16) != 0 || shm > 48 * 1024) return 2;
    if (T == 0) return 0;
    dim3 grid(ceil_div(E + has_gate, FRONT_ROWS), T);
    moe_front_kernel<<<grid, FRONT_THREADS, shm, (hipStream_t)stream>>>(h, ldh, gamma, gamma_dtype, eps, (bf16*)x_out,
                                                                        (const bf16*)W, H, T, E, has_gate, k, renorm,
                                                                        gating, logits, ids, weights, gate_out, counters,
                                                                        expert_offsets, sorted_token, sorted_pair, inv,
                                                                        n_always, per_row);
    FX_CHECK_LAUNCH("moe_front");
    return 0;
}

// gcnt: room for ceil(n / 64) * E ints (or null: one block does it all, whatever n)
FX_API int fx_moe_align(void* stream, const int* ids, int n, int k, int E, int* expert_offsets,
                        int* sorted_token, int* sorted_pair, int* inv, int* gcnt, int n_always) {
    FX_REQUIRE(n >= 0 && k > 0 && n % k == 0, "moe_align: n=%d must be a multiple of k=%d", n, k);
    FX_REQUIRE(n_always >= 0 && (n_always == 0 || n <= 2048), "moe_align: experts that every token takes are for up to 2048 pairs");
    FX_REQUIRE(E >= 1, "moe_align: E=%d", E);
    FX_REQUIRE(E <= 4096, "moe_align: %d experts are more than this kernel's 4096", E);
    if (gcnt && n > 2048 && !n_always && (size_t)(E + 1 + E + 2 * SORT_WAVES * E) * 4 <= 60 * 1024) {
        const int G = (n + 63) / 64, blocks = (G + SORT_WAVES - 1) / SORT_WAVES;
        moe_count_kernel<<<blocks, SORT_WAVES * 64, (size_t)SORT_WAVES * E * 4, (hipStream_t)stream>>>(ids, n, E, gcnt);
        FX_CHECK_LAUNCH("moe_count");
        moe_place_kernel<<<blocks, SORT_WAVES * 64, (size_t)(E + 1 + E + 2 * SORT_WAVES * E) * 4, (hipStream_t)stream>>>(
            ids, n, k, E, gcnt, expert_offsets, sorted_token, sorted_pair, inv);
        FX_CHECK_LAUNCH("moe_place");
        return 0;
    }
    size_t shm;
    const int per_row = align_groups_per_row(n, E, 60 * 1024, &shm);
    const int nt = n > 4096 ? 1024 : (n > 256 ? 512 : 256);
    moe_align_kernel<<<1, nt, shm, (hipStream_t)stream>>>(ids, n, k, E, per_row, expert_offsets, sorted_token, sorted_pair,
                                                          inv, n_always);
    FX_CHECK_LAUNCH("moe_align");
    return 0;
}

// Both steps in one launch when the batch is small enough for one block; returns 2 (and
// launches nothing) when it is not, so that the caller runs the two kernels.
FX_API int fx_router_select_align(void* stream, const float* logits, long ld, int T, int E, int k, int renorm,
                                  int gating, int* ids, float* weights, float* gate_out, int* expert_offsets,
                                  int* sorted_token, int* sorted_pair, int* inv) {
    FX_REQUIRE(T >= 0, "router: bad size T=%d", T);
    FX_REQUIRE(E >= 1 && E <= E_MAX, "router: %d experts, this kernel takes 1..%d", E, E_MAX);
    FX_REQUIRE(k >= 1 && k <= E && k <= K_MAX, "router: top-k %d must lie in 1..min(E, %d)", k, K_MAX);
    FX_REQUIRE(ld >= E + (gate_out ? 1 : 0), "router: logits rows of %ld hold fewer than %d columns", ld, E + (gate_out ? 1 : 0));
    FX_REQUIRE(gating == GATE_SOFTMAX || gating == GATE_SIGMOID, "router: unknown gating %d", gating);
    const long n = (long)T * k;
    const long groups = (n + 63) / 64;
    const size_t shm = (size_t)(16 * E + n + E + 1) * 4 + (size_t)groups * E * 4;
    if (T > 16 || shm > 48 * 1024) return 2;
    if (T == 0) return 0;
    router_select_align_kernel<<<1, 1024, shm, (hipStream_t)stream>>>(logits, ld, T, E, k, renorm, gating, ids, weights,
                                                                     gate_out, expert_offsets, sorted_token, sorted_pair, inv);
    FX_CHECK_LAUNCH("router_select_align");
    return 0;
}
