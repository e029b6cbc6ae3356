// Sampling of the next token from float32 logits, one block per row.
//
// The order of operations is the reference's (ferrox-models/src/sampling.rs:93-189):
// history penalties, greedy pick when temperature <= 0, else division by the
// temperature, softmax over the vocabulary, top-k, top-p, renormalisation and an
// inverse-CDF walk in index order with a uniform draw supplied by the caller
// (the host keeps each request's xorshift64 generator, sampling.rs:66-84).
// Greedy ties go to the lowest index.
#include "common.h"

FX_DEFINE_LAST_ERROR()

#define SB 1024  // threads per block
#define SW (SB / 64)

struct ArgBest {
    float v;
    int i;
};

__device__ __forceinline__ ArgBest better(ArgBest a, ArgBest b) {
    return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

// block-wide argmax with lowest index on ties; NaN never wins. Result valid in every thread.
__device__ ArgBest block_argmax(const float* s, int V, ArgBest* red) {
    ArgBest best = {-INFINITY, 0x7fffffff};
    for (int i = threadIdx.x; i < V; i += SB) {
        const float v = s[i];
        if (v > best.v || (v == best.v && i < best.i)) best = {v, i};
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgBest other = {__shfl_xor(best.v, o, 64), __shfl_xor(best.i, o, 64)};
        best = better(best, other);
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
    __syncthreads();
    ArgBest r = red[0];
    for (int w = 1; w < SW; ++w) r = better(r, red[w]);
    if (r.i == 0x7fffffff) r.i = 0;
    return r;
}

__device__ float block_sum_f(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
    for (int w = 0; w < SW; ++w) s += red[w];
    return s;
}

__device__ int block_sum_i(int v, int* red) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    int s = 0;
    for (int w = 0; w < SW; ++w) s += red[w];
    return s;
}

// exclusive prefix over threads of a per-thread value; `total` gets the sum.
template <typename X>
__device__ X block_exclusive_scan(X v, X* red, X& total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    X inc = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const X u = __shfl_up(inc, o, 64);
        if (lane >= o) inc += u;
    }
    __syncthreads();
    if (lane == 63) red[wave] = inc;
    __syncthreads();
    X base = 0;
    total = 0;
    for (int w = 0; w < SW; ++w) {
        if (w < wave) base += red[w];
        total += red[w];
    }
    return base + inc - v;
}

struct SampleArgs {
    const float* logits;  // [R, ldl]
    long ldl;
    float* work;          // [R, V] scratch
    int V;
    const float* temperature;  // [R]
    const int* top_k;          // [R], 0 = off
    const float* top_p;        // [R], >= 1 = off
    const float* rep_penalty;  // [R], 1 = off
    const float* presence;     // [R]
    const float* frequency;    // [R]
    const float* draw;         // [R] uniform in [0, 1)
    const int* hist;           // concatenated histories, or null
    const int* hist_start;     // [R + 1]
    int* out;                  // [R]
};

// Select, among the entries of p (all >= 0), the `need` largest; zero the others.
// Equal values are kept in ascending index order.  Radix select over the float
// bit patterns (monotone for non-negative floats), 8 bits a pass.
__device__ void keep_top_count(float* p, int V, int need, int* hist_i, int* red_i) {
    uint32_t prefix = 0, mask = 0;
    int remaining = need;  // how many to take among values matching the prefix so far
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int b = threadIdx.x; b < 256; b += SB) hist_i[b] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < V; i += SB) {
            const uint32_t u = __float_as_uint(p[i]);
            if ((u & mask) == prefix) atomicAdd(&hist_i[(u >> shift) & 255], 1);
        }
        __syncthreads();
        // walk bins from the top; every thread does the same walk
        int digit = 0, above = 0;
        for (int b = 255; b >= 0; --b) {
            const int c = hist_i[b];
            if (above + c >= remaining) {
                digit = b;
                break;
            }
            above += c;
        }
        remaining -= above;
        prefix |= (uint32_t)digit << shift;
        mask |= 255u << shift;
        __syncthreads();
    }
    // prefix is the bit pattern of the need-th largest value; `remaining` of the
    // entries equal to it are kept, lowest indices first.
    const int per = (V + SB - 1) / SB;
    const int b0 = min(V, (int)threadIdx.x * per), b1 = min(V, b0 + per);
    int eq = 0;
    for (int i = b0; i < b1; ++i) eq += __float_as_uint(p[i]) == prefix;
    int total;
    int rank = block_exclusive_scan<int>(eq, red_i, total);
    for (int i = b0; i < b1; ++i) {
        const uint32_t u = __float_as_uint(p[i]);
        if (u < prefix) {
            p[i] = 0.f;
        } else if (u == prefix) {
            if (rank >= remaining) p[i] = 0.f;
            ++rank;
        }
    }
    __syncthreads();
}

// Nucleus: walk the probabilities in descending order (ascending index among
// equals) and keep the shortest prefix whose sum reaches top_p
// (sampling.rs:139-155).  Found by a radix select on the sum of the values
// above a threshold.
__device__ void keep_top_mass(float* p, int V, float top_p, float* hist_f, int* hist_i, float* red_f, int* red_i) {
    uint32_t prefix = 0, mask = 0;
    float mass_above = 0.f;  // sum of entries strictly above every value matching the prefix
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int b = threadIdx.x; b < 256; b += SB) {
            hist_f[b] = 0.f;
            hist_i[b] = 0;
        }
        __syncthreads();
        for (int i = threadIdx.x; i < V; i += SB) {
            const uint32_t u = __float_as_uint(p[i]);
            if ((u & mask) == prefix) {
                atomicAdd(&hist_f[(u >> shift) & 255], p[i]);
                atomicAdd(&hist_i[(u >> shift) & 255], 1);
            }
        }
        __syncthreads();
        int digit = 0;
        float above = 0.f;
        for (int b = 255; b >= 0; --b) {
            if (hist_i[b] == 0) continue;
            digit = b;
            if (mass_above + above + hist_f[b] >= top_p) break;
            above += hist_f[b];
        }
        mass_above += above;
        prefix |= (uint32_t)digit << shift;
        mask |= 255u << shift;
        __syncthreads();
    }
    // entries above `prefix` are kept; of those equal to it, as many as are
    // needed to reach top_p, lowest indices first
    const float tau = __uint_as_float(prefix);
    int need_eq = 1;
    {
        float cum = mass_above + tau;
        while (cum < top_p && need_eq < V && tau > 0.f) {
            cum += tau;
            ++need_eq;
        }
    }
    const int per = (V + SB - 1) / SB;
    const int b0 = min(V, (int)threadIdx.x * per), b1 = min(V, b0 + per);
    int eq = 0;
    for (int i = b0; i < b1; ++i) eq += __float_as_uint(p[i]) == prefix;
    int total;
    int rank = block_exclusive_scan<int>(eq, red_i, total);
    for (int i = b0; i < b1; ++i) {
        const uint32_t u = __float_as_uint(p[i]);
        if (u < prefix) {
            p[i] = 0.f;
        } else if (u == prefix) {
            if (rank >= need_eq) p[i] = 0.f;
            ++rank;
        }
    }
    __syncthreads();
}

__global__ __launch_bounds__(SB) void sample_kernel(SampleArgs a) {
    __shared__ ArgBest red_b[SW];
    __shared__ float red_f[SW];
    __shared__ int red_i[SW];
    __shared__ float hist_f[256];
    __shared__ int hist_i[256];
    __shared__ int found, last_pos;
    const int r = blockIdx.x, V = a.V;
    const float* logits = a.logits + (size_t)r * a.ldl;
    float* s = a.work + (size_t)r * V;
    const float temp = a.temperature ? a.temperature[r] : 0.f;

    #pragma unroll 4
    for (int i = threadIdx.x; i < V; i += SB) s[i] = logits[i];
    __syncthreads();

    // history penalties (sampling.rs:191-215): repetition once per occurrence,
    // then frequency * count + presence once per distinct token
    if (a.hist) {
        const int h0 = a.hist_start[r], h1 = a.hist_start[r + 1];
        const float rp = a.rep_penalty ? a.rep_penalty[r] : 1.f;
        const float pp = a.presence ? a.presence[r] : 0.f;
        const float fp = a.frequency ? a.frequency[r] : 0.f;
        if (h1 > h0 && (rp != 1.f || pp != 0.f || fp != 0.f)) {
            for (int i = h0 + threadIdx.x; i < h1; i += SB) {
                const int tok = a.hist[i];
                if (tok < 0 || tok >= V) continue;
                bool first = true;
                int count = 0;
                for (int j = h0; j < h1; ++j) {
                    if (a.hist[j] == tok) {
                        if (j < i) first = false;
                        ++count;
                    }
                }
                if (!first) continue;
                float v = s[tok];
                if (rp != 1.f)
                    for (int c = 0; c < count; ++c) v = v > 0.f ? v / rp : v * rp;
                if (pp != 0.f || fp != 0.f) {
                    v -= fp * (float)count;
                    v -= pp;
                }
                s[tok] = v;
            }
            __syncthreads();
        }
    }

    if (temp <= 0.f) {
        ArgBest b = block_argmax(s, V, red_b);
        if (threadIdx.x == 0) a.out[r] = b.i;
        return;
    }

    // softmax(scores / temperature)
    float mx = -INFINITY;
    #pragma unroll 4
    for (int i = threadIdx.x; i < V; i += SB) {
        const float v = s[i] / temp;
        s[i] = v;
        mx = fmaxf(mx, v);
    }
    mx = wave_max(mx);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red_f[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = red_f[0];
    for (int w = 1; w < SW; ++w) mx = fmaxf(mx, red_f[w]);
    float sum = 0.f;
    #pragma unroll 4
    for (int i = threadIdx.x; i < V; i += SB) {
        const float e = expf(s[i] - mx);
        s[i] = e;
        sum += e;
    }
    sum = block_sum_f(sum, red_f);
    #pragma unroll 4
    for (int i = threadIdx.x; i < V; i += SB) s[i] = s[i] / sum;
    __syncthreads();

    const int tk = a.top_k ? a.top_k[r] : 0;
    if (tk > 0 && tk < V) keep_top_count(s, V, tk, hist_i, red_i);
    const float tp = a.top_p ? a.top_p[r] : 1.f;
    if (tp < 1.f) keep_top_mass(s, V, tp, hist_f, hist_i, red_f, red_i);

    // renormalise and walk the cumulative sum in index order
    const int per = (V + SB - 1) / SB;
    const int b0 = min(V, (int)threadIdx.x * per), b1 = min(V, b0 + per);
    float part = 0.f;
    for (int i = b0; i < b1; ++i) part += s[i];
    float total;
    float before = block_exclusive_scan<float>(part, red_f, total);
    if (!(total > 0.f)) {  // everything filtered away: greedy on the raw logits (sampling.rs:158-162)
        ArgBest b = block_argmax(logits, V, red_b);
        if (threadIdx.x == 0) a.out[r] = b.i;
        return;
    }
    if (threadIdx.x == 0) {
        found = 0x7fffffff;
        last_pos = -1;
    }
    __syncthreads();
    const float u = a.draw[r] * total;
    float cum = before;
    int last = -1;
    bool hit = false;
    for (int i = b0; i < b1; ++i) {
        if (!(s[i] > 0.f)) continue;
        last = i;
        cum += s[i];
        if (!hit && u < cum) {
            atomicMin(&found, i);
            hit = true;
        }
    }
    if (last >= 0) atomicMax(&last_pos, last);
    __syncthreads();
    // if rounding left the draw above the last sum, the last token with p > 0 is taken
    if (threadIdx.x == 0) a.out[r] = found != 0x7fffffff ? found : max(last_pos, 0);
}

// Greedy choice without history penalties, many blocks per row: block (b, r) finds the best of
// its slice of row r (lowest index on ties, NaN never wins) and leaves it in `part`; the row's
// last block to finish picks among the slices.
#define GREEDY_THREADS 256
__global__ __launch_bounds__(GREEDY_THREADS) void greedy_kernel(const float* __restrict__ logits, long ldl, int V,
                                                                int per_block, ArgBest* part, unsigned* counters,
                                                                int* __restrict__ out) {
    __shared__ ArgBest red[GREEDY_THREADS / 64];
    const int r = blockIdx.y, nb = gridDim.x;
    const float* row = logits + (size_t)r * ldl;
    const int b0 = blockIdx.x * per_block, b1 = min(V, b0 + per_block);
    ArgBest best = {-INFINITY, 0x7fffffff};
#pragma unroll 4
    for (int i = b0 + threadIdx.x; i < b1; i += GREEDY_THREADS) {
        const float v = row[i];
        if (v > best.v) best = {v, i};       // ascending i within a thread: the first maximum is kept
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgBest other = {__shfl_xor(best.v, o, 64), __shfl_xor(best.i, o, 64)};
        best = better(best, other);
    }
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < GREEDY_THREADS / 64; ++w) best = better(best, red[w]);
        store_shared(&part[(size_t)r * nb + blockIdx.x].v, best.v);
        store_shared(&part[(size_t)r * nb + blockIdx.x].i, best.i);
    }
    if (!last_block_arrives(counters + r, nb)) return;
    if (threadIdx.x < 64) {
        ArgBest b = {-INFINITY, 0x7fffffff};
        for (int i = threadIdx.x; i < nb; i += 64) {
            const ArgBest other = {load_shared(&part[(size_t)r * nb + i].v), load_shared(&part[(size_t)r * nb + i].i)};
            b = better(b, other);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            ArgBest other = {__shfl_xor(b.v, o, 64), __shfl_xor(b.i, o, 64)};
            b = better(b, other);
        }
        if (threadIdx.x == 0) out[r] = b.i == 0x7fffffff ? 0 : b.i;
    }
}

// part: R * 64 pairs (float, int); counters: R zeroed unsigned that the kernel leaves at zero
FX_API int fx_sample_greedy(void* stream, const float* logits, long ldl, int R, int V, void* part, unsigned* counters,
                            int* out) {
    FX_REQUIRE(R >= 0 && V > 0 && ldl >= V, "sample: bad sizes R=%d V=%d ldl=%ld", R, V, ldl);
    FX_REQUIRE(part && counters && out, "sample: scratch, counters and output are required");
    if (R == 0) return 0;
    int nb = ceil_div(V, 4 * GREEDY_THREADS);       // at least four elements per thread
    if (nb > 64) nb = 64;
    const int per_block = ceil_div(V, nb);
    greedy_kernel<<<dim3(nb, R), GREEDY_THREADS, 0, (hipStream_t)stream>>>(logits, ldl, V, per_block, (ArgBest*)part,
                                                                          counters, out);
    FX_CHECK_LAUNCH("sample_greedy");
    return 0;
}

FX_API int fx_sample(void* stream, const float* logits, long ldl, float* work, int R, int V,
                     const float* temperature, const int* top_k, const float* top_p,
                     const float* rep_penalty, const float* presence, const float* frequency,
                     const float* draw, const int* hist, const int* hist_start, int* out) {
    FX_REQUIRE(R >= 0 && V > 0 && ldl >= V, "sample: bad sizes R=%d V=%d ldl=%ld", R, V, ldl);
    FX_REQUIRE(work && out, "sample: scratch and output are required");
    FX_REQUIRE(!temperature || draw, "sample: temperatures given without uniform draws");
    FX_REQUIRE(!hist || hist_start, "sample: histories given without their offsets");
    if (R == 0) return 0;
    SampleArgs a = {logits, ldl, work, V, temperature, top_k, top_p, rep_penalty, presence, frequency,
                    draw, hist, hist_start, out};
    sample_kernel<<<R, SB, 0, (hipStream_t)stream>>>(a);
    FX_CHECK_LAUNCH("sample");
    return 0;
}
