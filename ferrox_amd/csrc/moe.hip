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
// selection for one token by one wave; `score` is E floats of LDS owned by the wave
// (`es`: distance between the logits of neighbouring experts, 1 for a row of a [T, E] matrix)
__device__ __forceinline__ void select_token(const float* __restrict__ row, float* score, int t, int E, int k, int renorm,
                                             int gating, int* __restrict__ ids, float* __restrict__ weights,
                                             float* __restrict__ gate_out, int* ids_copy, long es = 1) {
    const int lane = threadIdx.x & 63;
    if (gate_out && lane == 0) gate_out[t] = 1.0f / (1.0f + expf(-row[E * es]));
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
            const float v = score[e];
            if (v > best) {  // ascending e within a lane: the first maximum is kept
                best = v;
                bi = e;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ob > best || (ob == best && oi < bi)) {
                best = ob;
                bi = oi;
            }
        }
        if (lane == j) my_w = best;
        if (lane == 0) {
            ids[t * k + j] = bi;
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
// Thread th owns the contiguous pairs [th*c, (th+1)*c) and counts them per
// expert in its own row cnt[th][.]; thread e then turns column e into running
// sums over th; a scan over the experts' totals gives the offsets; each thread
// walks its pairs again and places them.  The order inside an expert is the
// order of the pairs, whatever the number of threads.
// ---------------------------------------------------------------------------
// the sort itself, by one block; `offs` (E+1 ints) and `cnt` (rows*E uint16) are LDS
__device__ __forceinline__ void align_block(const int* ids, int n, int k, int E, int* offs, uint16_t* cnt,
                                            int* __restrict__ expert_offsets, int* __restrict__ sorted_token,
                                            int* __restrict__ sorted_pair, int* __restrict__ inv) {
    const int nt = blockDim.x, th = threadIdx.x, lane = th & 63;
    const int c = max(1, (n + nt - 1) / nt);
    const int rows = min(nt, (n + c - 1) / c);    // threads that own at least one pair
    const int b = min(n, th * c), b_end = min(n, (th + 1) * c);
    for (int i = th; i < rows * E; i += nt) cnt[i] = 0;
    __syncthreads();
    for (int i = b; i < b_end; ++i) {
        const int e = ids[i];
        if (e >= 0 && e < E) cnt[th * E + e] += 1;
    }
    __syncthreads();
    for (int e = th; e < E; e += nt) {
        int run = 0;
        for (int r = 0; r < rows; ++r) {
            const int v = cnt[r * E + e];
            cnt[r * E + e] = (uint16_t)run;
            run += v;
        }
        offs[e + 1] = run;  // total of expert e, scanned below
    }
    __syncthreads();
    if (th < 64) {   // inclusive scan of the totals by the first wave, 64 experts at a time
        int carry = 0;
        if (lane == 0) offs[0] = 0;
        for (int base = 0; base < E; base += 64) {
            const int e = base + lane;
            int v = e < E ? offs[e + 1] : 0;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int u = __shfl_up(v, o, 64);
                if (lane >= o) v += u;
            }
            if (e < E) offs[e + 1] = carry + v;
            carry += __shfl(v, 63, 64);
        }
    }
    __syncthreads();
    for (int e = th; e <= E; e += nt) expert_offsets[e] = offs[e];
    for (int i = b; i < b_end; ++i) {
        const int e = ids[i];
        if (e >= 0 && e < E) {
            const int dst = offs[e] + cnt[th * E + e];
            cnt[th * E + e] += 1;
            sorted_token[dst] = i / k;
            if (sorted_pair) sorted_pair[dst] = i;
            if (inv) inv[i] = dst;
        }
    }
}

__global__ __launch_bounds__(256) void moe_align_kernel(const int* __restrict__ ids, int n, int k, int E,
                                                        int* __restrict__ expert_offsets,
                                                        int* __restrict__ sorted_token, int* __restrict__ sorted_pair,
                                                        int* __restrict__ inv) {
    extern __shared__ int lds[];
    align_block(ids, n, k, E, lds, (uint16_t*)(lds + E + 1), expert_offsets, sorted_token, sorted_pair, inv);
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
    uint16_t* cnt = (uint16_t*)(offs + E + 1);  // rows x E
    const int wave = threadIdx.x >> 6;
    if (wave < T)
        select_token(logits + (size_t)wave * ld, score + wave * E, wave, E, k, renorm, gating, ids, weights, gate_out, ids_s);
    __syncthreads();
    align_block(ids_s, T * k, k, E, offs, cnt, expert_offsets, sorted_token, sorted_pair, inv);
}

// ---------------------------------------------------------------------------
// Few tokens (decode): everything in front of the experts in one launch.
// Block (r, t): RMSNorm of row t of the float32 residual stream (same formula and
// rounding as rmsnorm_kernel; block r = 0 writes it out as bfloat16 for the
// experts), then the products of that rounded row with router rows 8r .. 8r+7,
// two rows per wave, k in a fixed order, into `logits`.  The block that finishes
// last selects the experts of every token (a wave per token) and sorts the pairs.
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

__global__ __launch_bounds__(FRONT_THREADS) void moe_front_kernel(
    const float* __restrict__ h, long ldh, const void* __restrict__ gamma, int gamma_dtype, float eps,
    bf16* __restrict__ x_out, const bf16* __restrict__ W, int H, int T, int E, int has_gate, int k, int renorm,
    int gating, float* logits, int* ids, float* __restrict__ weights, float* __restrict__ gate_out,
    int* __restrict__ expert_offsets, int* __restrict__ sorted_token, int* __restrict__ sorted_pair,
    int* __restrict__ inv, unsigned* counter) {
    extern __shared__ int lds[];
    __shared__ float red[FRONT_WAVES];
    float* xs = (float*)lds;            // H: the normed row as the experts will read it
    const int t = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_rows = E + has_gate, chunks = H >> 3;

    // this wave's two router rows: their first loads leave before the norm is done
    const int e_a = blockIdx.x * FRONT_ROWS + wave, e_b = e_a + FRONT_WAVES;
    const bf16* wa = e_a < n_rows ? W + (size_t)e_a * H : nullptr;
    const bf16* wb = e_b < n_rows ? W + (size_t)e_b * H : nullptr;
    uint4 pa = make_uint4(0, 0, 0, 0), pb = pa;
    if (lane < chunks) {
        if (wa) pa = *(const uint4*)(wa + lane * 8);
        if (wb) pb = *(const uint4*)(wb + lane * 8);
    }

    const float* row = h + (size_t)t * ldh;
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

    float acc_a = 0.f, acc_b = 0.f;
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
    acc_a = wave_sum(acc_a);
    acc_b = wave_sum(acc_b);
    if (lane == 0) {
        if (wa) store_shared(logits + (size_t)t * n_rows + e_a, acc_a);
        if (wb) store_shared(logits + (size_t)t * n_rows + e_b, acc_b);
    }

    if (!last_block_arrives(counter, gridDim.x * gridDim.y)) return;
    const int n = T * k;
    float* score = (float*)lds;                     // FRONT_WAVES x E
    float* lrow = score + FRONT_WAVES * E;          // FRONT_WAVES x n_rows: a token's logits
    int* ids_s = (int*)(lrow + FRONT_WAVES * n_rows);   // n
    int* offs = ids_s + n;                          // E + 1
    uint16_t* cnt = (uint16_t*)(offs + E + 1);      // rows x E
    for (int tt = wave; tt < T; tt += FRONT_WAVES) {
        float* mine = lrow + wave * n_rows;
        for (int e = lane; e < n_rows; e += 64) mine[e] = load_shared(logits + (size_t)tt * n_rows + e);
        __builtin_amdgcn_wave_barrier();
        select_token(mine, score + wave * E, tt, E, k, renorm, gating, ids, weights, has_gate ? gate_out : nullptr, ids_s);
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    align_block(ids_s, n, k, E, offs, cnt, expert_offsets, sorted_token, sorted_pair, inv);
}

// Returns 2 (and launches nothing) for sizes this kernel does not take; the caller then runs the
// norm, the router product and the two routing kernels one after the other.  `logits` holds
// T x (E + has_gate) floats; `counter` is one zeroed unsigned in device memory that launches on
// one stream may share.
FX_API int fx_moe_front(void* stream, const float* h, long ldh, const void* gamma, int gamma_dtype, float eps,
                        void* x_out, const void* W, int H, int T, int E, int has_gate, int k, int renorm, int gating,
                        float* logits, int* ids, float* weights, float* gate_out, int* expert_offsets,
                        int* sorted_token, int* sorted_pair, int* inv, unsigned* counter) {
    FX_REQUIRE(T >= 0 && H > 0, "moe_front: bad sizes T=%d H=%d", T, H);
    FX_REQUIRE(E >= 1 && E <= E_MAX, "router: %d experts, this kernel takes 1..%d", E, E_MAX);
    FX_REQUIRE(k >= 1 && k <= E && k <= K_MAX, "router: top-k %d must lie in 1..min(E, %d)", k, K_MAX);
    FX_REQUIRE(gating == GATE_SOFTMAX || gating == GATE_SIGMOID, "router: unknown gating %d", gating);
    FX_REQUIRE(gamma_dtype == FX_F32 || gamma_dtype == FX_BF16, "moe_front: unknown norm weight dtype %d", gamma_dtype);
    FX_REQUIRE(ldh >= H, "moe_front: rows of %ld hold fewer than %d columns", ldh, H);
    FX_REQUIRE(!has_gate || gate_out, "moe_front: a gate row needs a place for its output");
    const long n = (long)T * k;
    const long rows = n < FRONT_THREADS ? n : FRONT_THREADS;
    const size_t front = (size_t)H * 4;
    const size_t back = (size_t)(FRONT_WAVES * (2 * E + 1) + n + E + 1) * 4 + (size_t)rows * E * 2;
    const size_t shm = front > back ? front : back;
    if (T > 16 || H % 8 != 0 || ((uintptr_t)W % 16) != 0 || shm > 48 * 1024) return 2;
    if (T == 0) return 0;
    dim3 grid(ceil_div(E + has_gate, FRONT_ROWS), T);
    moe_front_kernel<<<grid, FRONT_THREADS, shm, (hipStream_t)stream>>>(
        h, ldh, gamma, gamma_dtype, eps, (bf16*)x_out, (const bf16*)W, H, T, E, has_gate, k, renorm, gating, logits, ids,
        weights, gate_out, expert_offsets, sorted_token, sorted_pair, inv, counter);
    FX_CHECK_LAUNCH("moe_front");
    return 0;
}

FX_API int fx_moe_align(void* stream, const int* ids, int n, int k, int E, int* expert_offsets,
                        int* sorted_token, int* sorted_pair, int* inv) {
    FX_REQUIRE(n >= 0 && k > 0 && n % k == 0, "moe_align: n=%d must be a multiple of k=%d", n, k);
    FX_REQUIRE(E >= 1, "moe_align: E=%d", E);
    int nt = 256;
    while (nt > 64 && (size_t)nt * E * 2 + (E + 1) * 4 > 48 * 1024) nt >>= 1;
    const size_t shm = (size_t)nt * E * 2 + (E + 1) * 4;
    FX_REQUIRE(shm <= 48 * 1024, "moe_align: %d experts exceed this kernel's limit of about 380", E);
    FX_REQUIRE((n + nt - 1) / nt < 65536, "moe_align: %d pairs are too many for one block", n);
    moe_align_kernel<<<1, nt, shm, (hipStream_t)stream>>>(ids, n, k, E, expert_offsets, sorted_token, sorted_pair, inv);
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
    const long rows = n < 1024 ? n : 1024;
    const size_t shm = (size_t)(16 * E + n + E + 1) * 4 + (size_t)rows * E * 2;
    if (T > 16 || shm > 48 * 1024) return 2;
    if (T == 0) return 0;
    router_select_align_kernel<<<1, 1024, shm, (hipStream_t)stream>>>(logits, ld, T, E, k, renorm, gating, ids, weights,
                                                                     gate_out, expert_offsets, sorted_token, sorted_pair, inv);
    FX_CHECK_LAUNCH("router_select_align");
    return 0;
}
