// Causal grouped-query attention over the paged cache.
//
// Every kernel reads keys from pages [page][kv_head][slot][head_dim] and values
// from transposed pages [page][kv_head][head_dim][slot], through a block table
// [n_seqs, max_blocks].  A query at position p sees key t iff t <= p and, with a
// window W > 0, p - t < W (ferrox-core/src/attention.rs:441-447, 498-513).  Head
// h reads kv head h / (n_heads / n_kv_heads) (attention.rs:432-438).  Scores,
// softmax and the output sum are float32, in the one-pass form of
// attention.rs:146-175 over tiles of 64 keys that start at multiples of 64, so a
// query's result does not depend on what else is computed with it.
#include "common.h"
#include "attention.h"

FX_DEFINE_LAST_ERROR()

#define HD_MAX 256
#define TQ 16
#define NEG_INF (-INFINITY)

struct AttnArgs {
    const void* q;       // [tokens, n_heads * head_dim]
    long ldq;
    void* out;           // same shape
    long ldo;
    const void* k_pages;
    const void* v_pages;
    const int* block_table;
    int max_blocks;
    const int* positions;  // [tokens]
    const int* item_seq;   // per work item: sequence (row of the block table)
    const int* item_tok;   // per work item: first token
    const int* item_n;     // per work item: number of queries (prefill tiles only)
    int nh, nkv, hd, bs, window;
    int bs_shift;        // log2(bs) if bs is a power of two, else -1
    int n_items;
    float scale;
    // decode only
    float* part_o;   // [items, nh, splits, hd]
    float* part_ml;  // [items, nh, splits, 2]
    int splits, chunk;
};

static inline int log2_or_minus_one(int v) {
    if (v <= 0 || (v & (v - 1))) return -1;
    int s = 0;
    while ((1 << s) < v) ++s;
    return s;
}

// block of the table and slot in its page of key t (a shift when the page size is a power of two)
__device__ __forceinline__ void page_slot(const AttnArgs& a, int t, int& blk, int& slot) {
    if (a.bs_shift >= 0) {
        blk = t >> a.bs_shift;
        slot = t & (a.bs - 1);
    } else {
        blk = t / a.bs;
        slot = t - blk * a.bs;
    }
}

// Page ids of one sequence.  A block copies the entries of the key range it will walk into LDS once
// (stage_pages), so that finding a tile's pages is an LDS read and not a round trip to memory on
// which the tile's own loads would then wait; entries outside the copy come from memory.
#define PAGE_COPY 1024
struct PageLookup {
    const int* table;    // the sequence's row of the block table
    const int* copy;     // LDS
    int first, count;    // copy[i] = table[first + i], i < count
    __device__ __forceinline__ int page(int blk) const {
        const unsigned i = (unsigned)(blk - first);
        return i < (unsigned)count ? copy[i] : table[blk];
    }
};
// every thread of the block calls this; blocks [first_blk, last_blk] of the table are wanted
__device__ __forceinline__ PageLookup stage_pages(const int* table, int* lds, int first_blk, int last_blk) {
    PageLookup pl;
    pl.table = table;
    pl.copy = lds;
    pl.first = first_blk;
    pl.count = min(PAGE_COPY, max(0, last_blk - first_blk + 1));
    for (int i = threadIdx.x; i < pl.count; i += blockDim.x) lds[i] = table[first_blk + i];
    __syncthreads();
    return pl;
}

template <typename T>
__device__ __forceinline__ const T* key_row(const AttnArgs& a, const int* bt, int kvh, int t) {
    const int page = bt[t / a.bs];
    return (const T*)a.k_pages + (((size_t)page * a.nkv + kvh) * a.bs + t % a.bs) * a.hd;
}
template <typename T>
__device__ __forceinline__ const T* value_col(const AttnArgs& a, const int* bt, int kvh, int t) {
    const int page = bt[t / a.bs];
    return (const T*)a.v_pages + ((size_t)page * a.nkv + kvh) * a.hd * a.bs + t % a.bs;  // + d * bs
}

// ---------------------------------------------------------------------------
// Any number of queries.  A work item is a block of up to 64 consecutive
// queries of one sequence; one wave per (quarter of an item = up to 16 queries,
// head); lanes are keys for the scores and head dimensions for the output.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(64) void attn_tile_kernel(AttnArgs a) {
    __shared__ float Qs[TQ][HD_MAX];
    __shared__ float Ps[TQ][64];
    const int item = blockIdx.x >> 2, sub = blockIdx.x & 3, h = blockIdx.y, lane = threadIdx.x;
    const int kvh = h / (a.nh / a.nkv);
    const int tok0 = a.item_tok[item] + TQ * sub, n = min(TQ, a.item_n[item] - TQ * sub);
    if (n <= 0) return;
    const int* bt = a.block_table + (size_t)a.item_seq[item] * a.max_blocks;
    const int hd = a.hd;

    for (int idx = lane; idx < TQ * hd; idx += 64) {
        const int i = idx / hd, d = idx % hd;
        Qs[i][d] = i < n ? to_float(((const T*)a.q)[(size_t)(tok0 + i) * a.ldq + (size_t)h * hd + d]) * a.scale : 0.f;
    }
    int pos[TQ];
#pragma unroll
    for (int i = 0; i < TQ; ++i) pos[i] = i < n ? a.positions[tok0 + i] : -1;
    const int pmin = a.positions[tok0], pmax = a.positions[tok0 + n - 1];
    const int kv_begin = a.window > 0 ? max(0, pmin - a.window + 1) : 0;
    const int kv_end = pmax + 1;

    float m[TQ], l[TQ], o[HD_MAX / 64][TQ];
#pragma unroll
    for (int i = 0; i < TQ; ++i) {
        m[i] = NEG_INF;
        l[i] = 0.f;
#pragma unroll
        for (int dd = 0; dd < HD_MAX / 64; ++dd) o[dd][i] = 0.f;
    }
    __syncthreads();

    for (int kt0 = (kv_begin / 64) * 64; kt0 < kv_end; kt0 += 64) {
        const int t = kt0 + lane;
        const bool in_range = t >= kv_begin && t < kv_end;
        float s[TQ];
#pragma unroll
        for (int i = 0; i < TQ; ++i) s[i] = 0.f;
        if (in_range) {
            const T* kr = key_row<T>(a, bt, kvh, t);
            for (int d = 0; d < hd; ++d) {
                const float kv = to_float(kr[d]);
#pragma unroll
                for (int i = 0; i < TQ; ++i) s[i] = fmaf(Qs[i][d], kv, s[i]);
            }
        }
        float al[TQ];
#pragma unroll
        for (int i = 0; i < TQ; ++i) {
            const bool vis = in_range && t <= pos[i] && (a.window <= 0 || pos[i] - t < a.window);
            const float sv = vis ? s[i] : NEG_INF;
            const float m_new = fmaxf(m[i], wave_max(sv));
            al[i] = (m_new == NEG_INF) ? 1.f : expf(m[i] - m_new);
            const float p = vis ? expf(sv - m_new) : 0.f;
            l[i] = l[i] * al[i] + wave_sum(p);
            m[i] = m_new;
            Ps[i][lane] = p;
        }
        __syncthreads();
#pragma unroll
        for (int dd = 0; dd < HD_MAX / 64; ++dd) {
            const int d = dd * 64 + lane;
            if (d < hd) {
#pragma unroll
                for (int i = 0; i < TQ; ++i) o[dd][i] *= al[i];
                const int jn = min(64, kv_end - kt0);
                for (int j = max(0, kv_begin - kt0); j < jn; ++j) {
                    const float vv = to_float(value_col<T>(a, bt, kvh, kt0 + j)[(size_t)d * a.bs]);
#pragma unroll
                    for (int i = 0; i < TQ; ++i) o[dd][i] = fmaf(Ps[i][j], vv, o[dd][i]);
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int dd = 0; dd < HD_MAX / 64; ++dd) {
        const int d = dd * 64 + lane;
        if (d < hd) {
#pragma unroll
            for (int i = 0; i < TQ; ++i)
                if (i < n)
                    from_float((T*)a.out + (size_t)(tok0 + i) * a.ldo + (size_t)h * hd + d, o[dd][i] / l[i]);
        }
    }
}

// ---------------------------------------------------------------------------
// Single queries (decode): the keys of a sequence are cut into chunks of
// `chunk` positions; one wave per (sequence, head, chunk) writes a partial
// (max, sum, output), and a second kernel merges the chunks in ascending order.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(64) void attn_decode_kernel(AttnArgs a) {
    __shared__ float Qs[HD_MAX];
    __shared__ float Ps[64];
    const int item = blockIdx.x, h = blockIdx.y, split = blockIdx.z, lane = threadIdx.x;
    const int kvh = h / (a.nh / a.nkv);
    const int tok = a.item_tok[item];
    const int* bt = a.block_table + (size_t)a.item_seq[item] * a.max_blocks;
    const int hd = a.hd;
    const int p = a.positions[tok];
    const int kv_begin = max(a.window > 0 ? max(0, p - a.window + 1) : 0, split * a.chunk);
    const int kv_end = min(p + 1, (split + 1) * a.chunk);
    float* po = a.part_o + (((size_t)item * a.nh + h) * a.splits + split) * hd;
    float* pml = a.part_ml + (((size_t)item * a.nh + h) * a.splits + split) * 2;
    if (kv_begin >= kv_end) {
        if (lane == 0) {
            pml[0] = NEG_INF;
            pml[1] = 0.f;
        }
        return;
    }
    for (int d = lane; d < hd; d += 64) Qs[d] = to_float(((const T*)a.q)[(size_t)tok * a.ldq + (size_t)h * hd + d]) * a.scale;
    __syncthreads();
    float m = NEG_INF, l = 0.f, o[HD_MAX / 64];
#pragma unroll
    for (int dd = 0; dd < HD_MAX / 64; ++dd) o[dd] = 0.f;
    for (int kt0 = (kv_begin / 64) * 64; kt0 < kv_end; kt0 += 64) {
        const int t = kt0 + lane;
        const bool vis = t >= kv_begin && t < kv_end;
        float s = 0.f;
        if (vis) {
            const T* kr = key_row<T>(a, bt, kvh, t);
            for (int d = 0; d < hd; ++d) s = fmaf(Qs[d], to_float(kr[d]), s);
        }
        const float sv = vis ? s : NEG_INF;
        const float m_new = fmaxf(m, wave_max(sv));
        const float al = expf(m - m_new);  // a tile inside [kv_begin, kv_end) always has a visible key
        const float pr = vis ? expf(sv - m_new) : 0.f;
        l = l * al + wave_sum(pr);
        m = m_new;
        Ps[lane] = pr;
        __syncthreads();
#pragma unroll
        for (int dd = 0; dd < HD_MAX / 64; ++dd) {
            const int d = dd * 64 + lane;
            if (d < hd) {
                float acc = o[dd] * al;
                const int jn = min(64, kv_end - kt0);
                for (int j = max(0, kv_begin - kt0); j < jn; ++j)
                    acc = fmaf(Ps[j], to_float(value_col<T>(a, bt, kvh, kt0 + j)[(size_t)d * a.bs]), acc);
                o[dd] = acc;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int dd = 0; dd < HD_MAX / 64; ++dd) {
        const int d = dd * 64 + lane;
        if (d < hd) po[d] = o[dd];
    }
    if (lane == 0) {
        pml[0] = m;
        pml[1] = l;
    }
}

// Merges the chunks' partial results in ascending order.  One block per (token, head): first
// the weights exp(m_s - m) / sum of all chunks (kept in LDS), then every thread sums its head
// dimensions over the chunks with several loads in flight.
template <typename T>
__global__ __launch_bounds__(128) void attn_decode_merge_kernel(AttnArgs a) {
    extern __shared__ float wsm[];   // splits weights
    __shared__ float red[2];
    const int item = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int tok = a.item_tok[item];
    const int hd = a.hd, S = a.splits;
    const float* po = a.part_o + ((size_t)item * a.nh + h) * S * hd;
    const float* pml = a.part_ml + ((size_t)item * a.nh + h) * S * 2;
    // the first chunks' outputs for this thread's first dimension leave before anything else: they need no weight
    // to be fetched, only to be used (an empty chunk wrote nothing, and what is read there is dropped below)
    constexpr int EARLY = 16;
    float early[EARLY];
#pragma unroll
    for (int s = 0; s < EARLY; ++s) early[s] = po[(size_t)min(s, S - 1) * hd + min(tid, hd - 1)];
    float m = NEG_INF;
    for (int s = tid; s < S; s += 128) m = fmaxf(m, pml[2 * s]);
    m = wave_max(m);
    if ((tid & 63) == 0) red[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(red[0], red[1]);
    for (int s = tid; s < S; s += 128) {
        const float ms = pml[2 * s];
        wsm[s] = (ms == NEG_INF) ? 0.f : expf(ms - m);
    }
    __syncthreads();
    float l = 0.f;
    for (int s = 0; s < S; ++s) l += wsm[s] * ((wsm[s] > 0.f) ? pml[2 * s + 1] : 0.f);   // ascending, the same in every thread
    for (int d = tid; d < hd; d += 128) {
        float acc = 0.f;
        int s0 = 0;
        if (d == tid) {
#pragma unroll
            for (int s = 0; s < EARLY; ++s) {
                const float w = s < S ? wsm[s] : 0.f;
                acc = (s < S) ? fmaf(w, (w > 0.f) ? early[s] : 0.f, acc) : acc;
            }
            s0 = min(S, EARLY);
        }
#pragma unroll 8
        for (int s = s0; s < S; ++s) {
            const float w = wsm[s];
            const float v = (w > 0.f) ? po[(size_t)s * hd + d] : 0.f;   // an empty chunk wrote nothing
            acc = fmaf(w, v, acc);
        }
        from_float((T*)a.out + (size_t)tok * a.ldo + (size_t)h * hd + d, acc / l);
    }
}

// ---------------------------------------------------------------------------
// bfloat16 on MFMA (head_dim and block size multiples of 16).
//
// One wave owns 16 "rows" that share one kv head: 16 consecutive queries of one
// head (prefill), or the query heads of one kv group for a single token
// (decode).  For a tile of 64 keys it computes S^T = K Q^T with K as the A
// operand, so that the accumulator of lane (row = lane%16, g = lane/16) holds 16
// scores of its own row; the softmax runs on those registers, and the same
// registers, rounded to bfloat16, are the A operand of O += P V: two 16x16x32
// MFMAs per 16 output columns, in which lane (row, g) supplies the probabilities
// of keys 16g..16g+7 and 16g+8..16g+15.  To make that work, A-row i of key block
// kb reads key 16*(i/4) + 4*kb + i%4 of the tile, and the B operand reads 16
// consecutive keys 16g..16g+15 of a transposed value row.  Keys and values come
// from memory in whole 128-byte lines with the non-temporal hint (`load_lines16`
// and `swap_halves` in common.h): 64 sequences at 2,048 keys 219 -> 171 us a layer
// (4.9 -> 6.3 TB/s), 8 sequences 36.8 -> 29.1 us, 8 at 32,768 keys 431 -> 341 us.
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define LOG2E 1.4426950408889634f
#define LN2 0.6931471805599453f

// Maximum and sum over the four lanes li, li + 16, li + 32, li + 48 that share a row, in every one of them, with the
// two lane-swapping moves of gfx950 (rows of 16 lanes pairwise, then the halves of the wave): the same values in the
// same order as two exchanges through the LDS crossbar (__shfl_xor by 16 and by 32) would give, without the LDS.
__device__ __forceinline__ float quad_max(float x) {
    const unsigned u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const unsigned v = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
    const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_sum(float x) {
    const unsigned u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const unsigned v = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// One step of the one-pass softmax on a lane's 16 raw scores sc[kb][r] of keys key0 + 4*kb + r
// (key0 = tile start + 16g), in base 2: t = score * c with c = scale * log2(e), m and l are the
// running maximum (of t) and sum of this lane's row, shared by the row's four lanes.  MASKED: only
// keys in [lo, hi] count.  Returns the factor for what was accumulated so far, and the
// probabilities rounded to bfloat16: p_lo for keys key0 .. key0+7, p_hi for key0+8 .. key0+15.
template <bool MASKED>
__device__ __forceinline__ float softmax_step(f32x4_t (&sc)[4], int key0, int lo, int hi, float c, float& m, float& l,
                                              uint4& p_lo, uint4& p_hi) {
    // the maximum is taken over the raw scores and scaled once (c > 0, and rounding keeps the order); a score's
    // exponent is then one fused multiply-add, score * c - maximum
    float mt = NEG_INF;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (MASKED) {
                const int key = key0 + 4 * kb + r;
                sc[kb][r] = (key >= lo && key <= hi) ? sc[kb][r] : NEG_INF;
            }
            mt = fmaxf(mt, sc[kb][r]);
        }
    mt = quad_max(mt) * c;
    const float m_new = fmaxf(m, mt);
    const float m_use = (m_new == NEG_INF) ? 0.f : m_new;      // a row that has seen nothing yet
    const float alpha = __builtin_amdgcn_exp2f(m - m_use);      // exp2(-inf) = 0
    float ps = 0.f;
    float p[16];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            p[4 * kb + r] = __builtin_amdgcn_exp2f(fmaf(sc[kb][r], c, -m_use));
            ps += p[4 * kb + r];
        }
    p_lo = make_uint4(pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7]));
    p_hi = make_uint4(pack_bf16(p[8], p[9]), pack_bf16(p[10], p[11]), pack_bf16(p[12], p[13]), pack_bf16(p[14], p[15]));
    ps = quad_sum(ps);
    l = l * ((m_new == NEG_INF) ? 1.f : alpha) + ps;
    m = m_new;
    return (m_new == NEG_INF) ? 1.f : alpha;
}

// O = O * factor(row) + P V for one block of 16 output columns.  The accumulator holds rows
// 4g+r, so the factors come from the lanes that own those rows; `rescale` is false when every
// row's factor is 1.
__device__ __forceinline__ f32x4_t pv_step(f32x4_t acc, bool rescale, const float (&al)[4], uint4 p_lo, uint4 p_hi,
                                           uint4 v0, uint4 v1) {
    if (rescale) {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] *= al[r];
    }
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, p_lo), __builtin_bit_cast(bf16x8_t, v0), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, p_hi), __builtin_bit_cast(bf16x8_t, v1), acc, 0, 0, 0);
    return acc;
}

// Eight consecutive keys' values (first_key ..): those outside [kv_begin, kv_end) become zeros.  Their
// probabilities are zero, but what memory holds there need not be a number.
__device__ __forceinline__ uint4 keep_keys(uint4 v, int first_key, int kv_begin, int kv_end) {
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int key = first_key + e;
        if (key < kv_begin || key >= kv_end) w[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// All ones if `ok`, else zero, as a value the compiler knows nothing about: data that is loaded and then
// ANDed with it is loaded always.  With a plain `ok ? x : 0` the compiler loads only where ok holds, behind a
// branch, and waits for that load before it goes on: a tile's loads would then leave one at a time.
__device__ __forceinline__ uint32_t opaque_mask(bool ok) {
    uint32_t m = ok ? 0xffffffffu : 0u;
    asm volatile("" : "+v"(m));
    return m;
}
__device__ __forceinline__ uint4 and_mask(uint4 x, uint32_t m) { return make_uint4(x.x & m, x.y & m, x.z & m, x.w & m); }

template <int HD>   // compile-time bound of head_dim (a.hd <= HD)
struct WaveAttn {
    static constexpr int KS = HD / 32;   // k-steps of S^T = K Q^T
    static constexpr int CB = HD / 16;   // column blocks of O
    static constexpr bool EARLY_V = HD <= 128;   // registers allow the values to be fetched before the scores
    float m, l;                          // running max and sum of this lane's row
    f32x4_t o[CB];                       // lane (j, g): O[row 4g+r][16*cb + j]
    bf16x8_t qf[KS];                     // lane (row, g): Q[row][32u + 8g ..]

    __device__ __forceinline__ void init(const bf16* qrow, int hd) {
        m = NEG_INF;
        l = 0.f;
        const int g = threadIdx.x >> 4 & 3;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) o[cb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            const int d = 32 * u + 8 * g;
            uint4 v = (qrow && d < hd) ? *(const uint4*)(qrow + d) : make_uint4(0, 0, 0, 0);
            qf[u] = __builtin_bit_cast(bf16x8_t, v);
        }
    }

    // keys [kt0, kt0 + 64); this lane's row sees key t iff lo <= t <= hi (hi < lo: row unused)
    __device__ __forceinline__ void tile(const AttnArgs& a, const PageLookup& pl, int kvh, int kt0, int kv_begin, int kv_end,
                                         int lo, int hi) {
        const int lane = threadIdx.x & 63, li = lane & 15, g = lane >> 4;
        const int l8 = li & 7, lh = li >> 3;
        const int hd = a.hd, bs = a.bs;
        // Loads are issued without branches: a key outside [kv_begin, kv_end) (its page may have been
        // given back) reads from a group of keys that is inside, and its data is replaced by zeros.
        const int safe_group = (kv_end - 1) & ~15;
        // values first, so that they arrive while the scores are computed: 16 consecutive keys
        // kt0 + 16g .. of transposed row d = 16*cb + li
        const int kg = kt0 + 16 * g;
        const bool edge = kt0 < kv_begin || kt0 + 64 > kv_end;      // some key of the tile is outside
        const bool vlive = kg < kv_end && kg + 16 > kv_begin;
        const int vkey = vlive ? kg : safe_group;
        int vblk, vslot;
        page_slot(a, vkey, vblk, vslot);
        // every page id of the tile is looked up before the first load leaves: a lookup that stands between two
        // groups of loads makes the second group wait for the first
        const int vpage = pl.page(vblk);
        int kpage[4], kslots[4];
        bool klives[4];
        constexpr int KP = KS & ~1;      // k-steps that are loaded in pairs, whole lines of eight keys at a time
        int kpage_a[4], kslots_a[4], kpage_b[4], kslots_b[4];
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            const int key0 = kt0 + 16 * (li >> 2) + 4 * kb + (li & 3);
            klives[kb] = key0 >= kv_begin && key0 < kv_end;
            int kblk;
            if (KP < KS) {
                page_slot(a, klives[kb] ? key0 : safe_group, kblk, kslots[kb]);
                kpage[kb] = pl.page(kblk);
            }
            // rows li % 8 and 8 + li % 8 of the block's 16 keys (row i is key 16 (i / 4) + 4 kb + i % 4 of the tile)
            const int key_a = kt0 + 16 * (l8 >> 2) + 4 * kb + (l8 & 3), key_b = key_a + 32;
            page_slot(a, key_a >= kv_begin && key_a < kv_end ? key_a : safe_group, kblk, kslots_a[kb]);
            kpage_a[kb] = pl.page(kblk);
            page_slot(a, key_b >= kv_begin && key_b < kv_end ? key_b : safe_group, kblk, kslots_b[kb]);
            kpage_b[kb] = pl.page(kblk);
        }
        const bf16* vbase = (const bf16*)a.v_pages + ((size_t)vpage * a.nkv + kvh) * hd * bs + vslot;
        uint4 vv[EARLY_V ? CB : 1][2];
        const uint32_t vmask = opaque_mask(vlive);
        if (EARLY_V) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                // whole lines: the first load's lanes take rows 16 cb + li % 8, the second's the eight after them, both
                // the keys 8 (li / 8) .. of the lane's 16; the halves change places before the products
                const int d1 = 16 * cb + l8, d2 = d1 + 8;
                vv[cb][0] = load_lines16(vbase + (size_t)(d1 < hd ? d1 : 0) * bs + 8 * lh);
                vv[cb][1] = load_lines16(vbase + (size_t)(d2 < hd ? d2 : 0) * bs + 8 * lh);
            }
        }
        f32x4_t sc[4];
        uint4 kf[4][KS];
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            const bf16* kra = (const bf16*)a.k_pages + (((size_t)kpage_a[kb] * a.nkv + kvh) * bs + kslots_a[kb]) * hd;
            const bf16* krb = (const bf16*)a.k_pages + (((size_t)kpage_b[kb] * a.nkv + kvh) * bs + kslots_b[kb]) * hd;
#pragma unroll
            for (int u = 0; u < KP; u += 2) {
                const int d = 32 * u + 32 * lh + 8 * g;           // the low or the high 32 of the pair's 64
                kf[kb][u] = load_lines16(kra + (d < hd ? d : 0));
                kf[kb][u + 1] = load_lines16(krb + (d < hd ? d : 0));
            }
            if (KP < KS) {
                const bf16* kr = (const bf16*)a.k_pages + (((size_t)kpage[kb] * a.nkv + kvh) * bs + kslots[kb]) * hd;
                const uint32_t kmask = opaque_mask(klives[kb]);
#pragma unroll
                for (int u = KP; u < KS; ++u) {
                    const int d = 32 * u + 8 * g;
                    const uint4 x = *(const uint4*)(kr + (d < hd ? d : 0));
                    kf[kb][u] = and_mask(x, kmask & opaque_mask(d < hd));
                }
            }
        }
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            sc[kb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
            const uint32_t kmask = opaque_mask(klives[kb]);
#pragma unroll
            for (int u = 0; u < KS; ++u) {
                uint4 ku = kf[kb][u];
                if (u < KP) {
                    // low 32: own first load below lane 8 of a row of 16, the other half's second load above;
                    // high 32: the other half's first load below, own second load above
                    ku = (u & 1) ? swap_halves<0x3>(kf[kb][u], kf[kb][u - 1]) : swap_halves<0xC>(kf[kb][u], kf[kb][u + 1]);
                    ku = and_mask(ku, kmask & opaque_mask(32 * u + 8 * g < hd));
                }
                sc[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ku), qf[u], sc[kb], 0, 0, 0);
            }
        }
        // softmax on this lane's 16 scores (keys kt0 + 16g + 4kb + r); the row's four lanes share max and sum
        uint4 p_lo, p_hi;
        const float alpha = softmax_step<true>(sc, kt0 + 16 * g, lo, hi, a.scale * LOG2E, m, l, p_lo, p_hi);
        const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;
        float al[4] = {1.f, 1.f, 1.f, 1.f};
        if (rescale) {
#pragma unroll
            for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, 4 * g + r, 64);
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            uint4 v0, v1;
            {
                uint4 t1, t2;
                if (EARLY_V) {
                    t1 = vv[cb][0];
                    t2 = vv[cb][1];
                } else {
                    const int d1 = 16 * cb + l8, d2 = d1 + 8;
                    t1 = load_lines16(vbase + (size_t)(d1 < hd ? d1 : 0) * bs + 8 * lh);
                    t2 = load_lines16(vbase + (size_t)(d2 < hd ? d2 : 0) * bs + 8 * lh);
                }
                const uint32_t ok = vmask & opaque_mask(16 * cb + li < hd);
                v0 = and_mask(swap_halves<0xC>(t1, t2), ok);
                v1 = and_mask(swap_halves<0x3>(t2, t1), ok);
            }
            if (edge) {
                v0 = keep_keys(v0, kg, kv_begin, kv_end);
                v1 = keep_keys(v1, kg + 8, kv_begin, kv_end);
            }
            o[cb] = pv_step(o[cb], rescale, al, p_lo, p_hi, v0, v1);
        }
    }
};

// prefill: item = up to 16 consecutive queries of one sequence; block = one wave = (item, head)
template <int HD>
__global__ __launch_bounds__(64) void attn_mfma_tile_kernel(AttnArgs a) {
    const int item = blockIdx.x >> 2, sub = blockIdx.x & 3, h = blockIdx.y, lane = threadIdx.x, li = lane & 15, g = lane >> 4;
    const int kvh = h / (a.nh / a.nkv);
    const int tok0 = a.item_tok[item] + 16 * sub, n = min(16, a.item_n[item] - 16 * sub);
    if (n <= 0) return;
    const int* bt = a.block_table + (size_t)a.item_seq[item] * a.max_blocks;
    const int hd = a.hd;
    const int pmin = a.positions[tok0], pmax = a.positions[tok0 + n - 1];
    const int kv_begin = a.window > 0 ? max(0, pmin - a.window + 1) : 0;
    const int kv_end = pmax + 1;
    int lo = 1, hi = 0;
    const bf16* qrow = nullptr;
    if (li < n) {
        hi = a.positions[tok0 + li];
        lo = a.window > 0 ? max(0, hi - a.window + 1) : 0;
        qrow = (const bf16*)a.q + (size_t)(tok0 + li) * a.ldq + (size_t)h * hd;
    }
    WaveAttn<HD> w;
    w.init(qrow, hd);
    const PageLookup pl = {bt, nullptr, 0, 0};
    for (int kt0 = (kv_begin / 64) * 64; kt0 < kv_end; kt0 += 64) w.tile(a, pl, kvh, kt0, kv_begin, kv_end, lo, hi);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * g + r;
        const float lr = __shfl(w.l, row, 64);
        if (row < n) {
#pragma unroll
            for (int cb = 0; cb < WaveAttn<HD>::CB; ++cb) {
                const int d = 16 * cb + li;
                if (d < hd) from_float((bf16*)a.out + (size_t)(tok0 + row) * a.ldo + (size_t)h * hd + d, w.o[cb][r] / lr);
            }
        }
    }
}

// decode, several waves per block: block = (item, kv head x group block of 16 query heads, split);
// its waves take the split's tiles of 64 keys in turn and their results are merged through LDS in
// wave order.  With one split the block writes the output itself, no second launch.
template <int HD, int MAX_THREADS>
__global__ __launch_bounds__(MAX_THREADS) void attn_mfma_decode_block_kernel(AttnArgs a) {
    extern __shared__ float wave_out[];      // [waves][rows][HD + 2]: o, then m and l
    // The grid is (heads, items, splits): blocks go to the eight XCDs in turn, so with the heads fastest every
    // item's blocks are spread over all of them, and with the splits slowest a sequence's last, shorter chunks start
    // last.  (With the items fastest and their number a multiple of eight, as a recorded step's is, an item's blocks
    // all land on one XCD, and 17 live sequences beside 7 stand-ins give one XCD three sequences and the others
    // two: 73 against 57 us.)
    const int item = blockIdx.y, split = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    const int li = lane & 15, g = lane >> 4;
    const int group = a.nh / a.nkv, gblocks = (group + 15) / 16;
    const int kvh = blockIdx.x / gblocks, hb = blockIdx.x % gblocks;
    const int tok = a.item_tok[item];
    const int* bt = a.block_table + (size_t)a.item_seq[item] * a.max_blocks;
    const int hd = a.hd;
    const int p = a.positions[tok];
    // The keys this query sees, from the tile of 64 that holds the first of them on, go to the splits in equal
    // chunks of whole tiles: a sequence shorter than the launch's bound, or a window far into a long sequence,
    // still keeps every split busy.  (a.chunk is the longest chunk any sequence of the launch can have.)
    __shared__ int page_copy[PAGE_COPY];
    int first_blk, last_blk, unused;
    PageLookup pl;
    if (a.window <= 0) {
        // the page ids that the split can need, whatever the position turns out to be, are copied before the
        // position has arrived (entries past the sequence's pages are read and never used)
        page_slot(a, (split + 1) * a.chunk - 1, last_blk, unused);
        last_blk = min(last_blk, a.max_blocks - 1);
        pl = stage_pages(bt, page_copy, max(0, last_blk - PAGE_COPY + 1), last_blk);
    }
    const int first_key = a.window > 0 ? max(0, p - a.window + 1) : 0;
    const int base = first_key & ~63;
    const int chunk = (((p + 1 - base + a.splits - 1) / a.splits) + 63) & ~63;
    const int kv_begin = max(first_key, base + split * chunk);
    const int kv_end = min(p + 1, base + (split + 1) * chunk);
    if (a.window > 0) {
        page_slot(a, min(kv_begin, p), first_blk, unused);
        page_slot(a, max(kv_end - 1, 0), last_blk, unused);
        first_blk = min(first_blk, a.max_blocks - 1);
        last_blk = min(last_blk, a.max_blocks - 1);
        pl = stage_pages(bt, page_copy, first_blk, last_blk);
    }
    const int n = min(16, group - hb * 16);        // query heads in this block
    const int h0 = kvh * group + hb * 16;
    const bool empty = kv_begin >= kv_end;
    WaveAttn<HD> w;
    const bool row_ok = li < n;
    w.init(row_ok && !empty ? (const bf16*)a.q + (size_t)tok * a.ldq + (size_t)(h0 + li) * hd : nullptr, hd);
    if (!empty) {
        const int lo = row_ok ? kv_begin : 1, hi = row_ok ? kv_end - 1 : 0;
        for (int kt0 = (kv_begin / 64) * 64 + wave * 64; kt0 < kv_end; kt0 += n_waves * 64)
            w.tile(a, pl, kvh, kt0, kv_begin, kv_end, lo, hi);
    }
    const int stride = HD + 2;
    float* mine = wave_out + (size_t)wave * n * stride;
    if (row_ok && g == 0) {
        mine[li * stride + HD] = w.m;            // base 2
        mine[li * stride + HD + 1] = w.l;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * g + r;
        if (row < n) {
#pragma unroll
            for (int cb = 0; cb < WaveAttn<HD>::CB; ++cb) mine[row * stride + 16 * cb + li] = w.o[cb][r];
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < n * hd; idx += blockDim.x) {
        const int row = idx / hd, d = idx - row * hd;
        float m = NEG_INF;
        for (int u = 0; u < n_waves; ++u) m = fmaxf(m, wave_out[((size_t)u * n + row) * stride + HD]);
        float l = 0.f, o = 0.f;
        for (int u = 0; u < n_waves; ++u) {
            const float* src = wave_out + ((size_t)u * n + row) * stride;
            const float f = src[HD] == NEG_INF ? 0.f : __builtin_amdgcn_exp2f(src[HD] - m);
            l += f * src[HD + 1];
            o += f * src[d];
        }
        const int h = h0 + row;
        if (a.splits == 1) {
            from_float((bf16*)a.out + (size_t)tok * a.ldo + (size_t)h * hd + d, o / l);
        } else {
            a.part_o[(((size_t)item * a.nh + h) * a.splits + split) * hd + d] = o;
            if (d == 0) {
                float* pml = a.part_ml + (((size_t)item * a.nh + h) * a.splits + split) * 2;
                pml[0] = m == NEG_INF ? NEG_INF : m * LN2;
                pml[1] = l;
            }
        }
    }
}

// Prefill with the keys and values of a tile shared through LDS: a block of four waves owns up
// to 64 consecutive queries of one head (16 each); per tile of 64 keys the block stages K
// (rows permuted so that the 16 keys an MFMA operand needs lie in consecutive rows) and the
// transposed V once, and every wave takes its operands from there.  While a tile is multiplied
// the next one is already on its way from memory into registers.
template <int HD>
__global__ __launch_bounds__(256) void attn_mfma_block_kernel(AttnArgs a) {
    constexpr int KS = HD / 32, CB = HD / 16;
    constexpr int KROW = HD + 8;          // bf16 elements per staged key row (16 bytes of padding)
    constexpr int VROW = 64 + 8;          // bf16 elements per staged value row
    constexpr int KCH = 64 * (HD / 8), VCH = HD * 8;      // 16-byte chunks per tile
    constexpr int NK = (KCH + 255) / 256, NV = (VCH + 255) / 256;
    __shared__ __attribute__((aligned(16))) bf16 Ks[64 * KROW];
    __shared__ __attribute__((aligned(16))) bf16 Vs[HD * VROW];
    // Blocks go to the 8 XCDs in turn, each with an L2 of its own: block b runs on XCD b % 8.  The
    // (head, item) pairs are dealt out so that an XCD works through whole heads, whose keys and
    // values then stay in its L2, and the items with the longest key range start first.
    const int per_xcd = (a.n_items * a.nh + 7) / 8;
    const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (logical >= a.n_items * a.nh) return;
    const int h = logical / a.n_items, item = a.n_items - 1 - logical % a.n_items;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, g = lane >> 4;
    const int kvh = h / (a.nh / a.nkv);
    const int tok_first = a.item_tok[item], n_all = a.item_n[item];
    const int* bt = a.block_table + (size_t)a.item_seq[item] * a.max_blocks;
    const int hd = a.hd, bs = a.bs;
    const int pmin = a.positions[tok_first], pmax = a.positions[tok_first + n_all - 1];
    const int kv_begin = a.window > 0 ? max(0, pmin - a.window + 1) : 0;
    const int kv_end = pmax + 1;
    // this wave's 16 rows
    const int tok0 = tok_first + 16 * wave, n = min(16, n_all - 16 * wave);
    int lo = 1, hi = 0;
    const bf16* qrow = nullptr;
    if (li < n) {
        hi = a.positions[tok0 + li];
        lo = a.window > 0 ? max(0, hi - a.window + 1) : 0;
        qrow = (const bf16*)a.q + (size_t)(tok0 + li) * a.ldq + (size_t)h * hd;
    }
    int w_lo = 0x7fffffff, w_hi = -1;     // keys any row of this wave can see
    int w_lo_max = 0x7fffffff, w_hi_min = -1;   // keys every row of this wave sees: [w_lo_max, w_hi_min]
    if (n > 0) {
        w_hi = a.positions[tok0 + n - 1];
        w_lo = a.window > 0 ? max(0, a.positions[tok0] - a.window + 1) : 0;
        if (n == 16) {                    // a wave with idle rows masks always
            w_hi_min = a.positions[tok0];
            w_lo_max = a.window > 0 ? max(0, w_hi - a.window + 1) : 0;
        }
    }
    const float c2 = a.scale * LOG2E;
    float m = NEG_INF, l = 0.f;
    f32x4_t o[CB];
    bf16x8_t qf[KS];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) o[cb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < KS; ++u) {
        const int d = 32 * u + 8 * g;
        uint4 v = (qrow && d < hd) ? *(const uint4*)(qrow + d) : make_uint4(0, 0, 0, 0);
        qf[u] = __builtin_bit_cast(bf16x8_t, v);
    }

    uint4 kreg_a[NK], vreg_a[NV], kreg_b[NK], vreg_b[NV];     // two tiles on their way from memory
    // Loads are issued without branches: a key outside [kv_begin, kv_end) (its page may have been
    // given back) reads from a group of keys that is inside, and its data is replaced by zeros.
    const int safe_group = (kv_end - 1) & ~15;
    __shared__ int page_copy[PAGE_COPY];
    int first_blk, last_blk, unused;
    page_slot(a, kv_begin, first_blk, unused);
    page_slot(a, kv_end - 1, last_blk, unused);
    const PageLookup pl = stage_pages(bt, page_copy, first_blk, last_blk);
    auto fetch = [&](uint4* kreg, uint4* vreg, int kt0) {
        size_t kbase[4], vbase[4];     // page and slot of each group of 16 keys of the tile (the same for all threads)
        bool live[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int key0 = kt0 + 16 * j;
            live[j] = key0 < kv_end && key0 + 16 > kv_begin;
            int blk, slot;
            page_slot(a, live[j] ? key0 : safe_group, blk, slot);
            const size_t page = pl.page(blk);
            kbase[j] = ((page * a.nkv + kvh) * bs + slot) * hd;
            vbase[j] = (page * a.nkv + kvh) * hd * bs + slot;
        }
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int c = tid + i * 256;
            if (c < KCH) {
                const int r = c / (HD / 8), d = (c % (HD / 8)) * 8;
                const int key = kt0 + r;
                const bool ok = key >= kv_begin && key < kv_end && d < hd;
                const uint4 v = *(const uint4*)((const bf16*)a.k_pages + kbase[r >> 4] + (size_t)(r & 15) * hd + (d < hd ? d : 0));
                kreg[i] = ok ? v : make_uint4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = tid + i * 256;
            if (c < VCH) {
                const int d = c >> 3, k8 = (c & 7) * 8;
                const bool ok = d < hd && live[k8 >> 4];
                uint4 v = *(const uint4*)((const bf16*)a.v_pages + vbase[k8 >> 4] + (size_t)(d < hd ? d : 0) * bs + (k8 & 15));
                if (kt0 < kv_begin || kt0 + 64 > kv_end) v = keep_keys(v, kt0 + k8, kv_begin, kv_end);
                vreg[i] = ok ? v : make_uint4(0, 0, 0, 0);
            }
        }
    };
    auto stage = [&](const uint4* kreg, const uint4* vreg) {
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int c = tid + i * 256;
            if (c < KCH) {
                const int r = c / (HD / 8), d = (c % (HD / 8)) * 8;
                const int row = ((r >> 2) & 3) * 16 + (r >> 4) * 4 + (r & 3);     // key 16a + 4kb + b -> row 16kb + 4a + b
                *(uint4*)(Ks + row * KROW + d) = kreg[i];
            }
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = tid + i * 256;
            if (c < VCH) *(uint4*)(Vs + (c >> 3) * VROW + (c & 7) * 8) = vreg[i];
        }
    };

    const int kt_first = (kv_begin / 64) * 64;
    fetch(kreg_a, vreg_a, kt_first);
    if (kt_first + 64 < kv_end) fetch(kreg_b, vreg_b, kt_first + 64);
    int parity = 0;
    for (int kt0 = kt_first; kt0 < kv_end; kt0 += 64, parity ^= 1) {
        lds_barrier();            // the previous tile has been read by every wave
        if (parity == 0) stage(kreg_a, vreg_a); else stage(kreg_b, vreg_b);
        lds_barrier();
        if (kt0 + 128 < kv_end) {  // the registers just emptied take the tile after the next
            if (parity == 0) fetch(kreg_a, vreg_a, kt0 + 128); else fetch(kreg_b, vreg_b, kt0 + 128);
        }
        if (kt0 > w_hi || kt0 + 64 <= w_lo) continue;      // nothing in this tile for this wave's rows
        f32x4_t sc[4];
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            sc[kb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < KS; ++u) {
                const bf16x8_t kf = *(const bf16x8_t*)(Ks + (kb * 16 + li) * KROW + 32 * u + 8 * g);
                sc[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[u], sc[kb], 0, 0, 0);
            }
        }
        // tiles that every row of this wave sees whole need no mask
        const bool whole = kt0 >= w_lo_max && kt0 + 63 <= w_hi_min && kt0 >= kv_begin;
        uint4 p_lo, p_hi;
        const float alpha = whole ? softmax_step<false>(sc, kt0 + 16 * g, lo, hi, c2, m, l, p_lo, p_hi)
                                  : softmax_step<true>(sc, kt0 + 16 * g, lo, hi, c2, m, l, p_lo, p_hi);
        const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;
        float al[4] = {1.f, 1.f, 1.f, 1.f};
        if (rescale) {
#pragma unroll
            for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, 4 * g + r, 64);
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const bf16* vr = Vs + (16 * cb + li) * VROW + 16 * g;
            o[cb] = pv_step(o[cb], rescale, al, p_lo, p_hi, *(const uint4*)vr, *(const uint4*)(vr + 8));
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * g + r;
        const float lr = __shfl(l, row, 64);
        if (row < n) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const int d = 16 * cb + li;
                if (d < hd) from_float((bf16*)a.out + (size_t)(tok0 + row) * a.ldo + (size_t)h * hd + d, o[cb][r] / lr);
            }
        }
    }
}

// Prefill when head_dim is exactly 64 or 128 and a page holds a multiple of 64 keys: a tile of 64
// keys then lies in one page, 64 * HD contiguous elements of keys and as many of transposed values,
// and travels from global memory straight into LDS (no registers in between, nothing to unpack),
// two stages, the next tile's loads in flight while this one is multiplied, one barrier per tile.
// A wave-load fills 1 KB: 1024 / (2 HD) key rows, or eight value rows of 64 keys.  Key row
// 16 kb + 4 a + b of LDS holds key 16 a + 4 kb + b (what the MFMA operands want, see above; four
// such keys follow each other in memory and in LDS alike), and inside a row the 16-byte chunks
// stand at chunk ^ (row % 16) for rows of 256 bytes and chunk ^ ((row / 2) % 8) for rows of 128, which the loading
// lanes achieve by choosing which chunk they fetch: the 16 rows an operand reads then fall on
// distinct banks without padding.  Keys outside [kv_begin, kv_end) come along as whatever memory
// holds: their scores are masked, and their values are zeroed in LDS before the product.
typedef __attribute__((address_space(1))) const void* fx_global_ptr;
typedef __attribute__((address_space(3))) void* fx_lds_ptr;

// W waves per block, 16 queries each: an item is up to 16 W queries.  Eight waves share every tile that the block
// brings into LDS between twice as many queries, and four of them per SIMD (two blocks on a CU) hide each other's
// waits; four waves (items of 64) are for prompt portions too short to fill the GPU with larger items.
// G = 2: two such groups of W waves share the item's queries and take its tiles of keys in turn (group 0 the even
// ones, group 1 the odd ones), each with stages, running maxima, sums and outputs of its own; group 1 hands its
// results over through LDS at the end and group 0 merges them.  An item's chain of tiles is then half as long,
// which is what bounds a prompt portion of few items over many keys.
template <int HD, int NS, int W = 4, int G = 1>
__global__ __launch_bounds__(W * G * 64, W / 2) void attn_mfma_direct_kernel(AttnArgs a) {      // two blocks on a CU, or one of two groups
    static_assert(G == 1 || (G == 2 && NS == 2), "one group, or two with two stages each");
    constexpr int KS = HD / 32, CB = HD / 16;
    constexpr int NCH = HD / 8;                 // 16-byte chunks of a key row
    constexpr int KROWS = 1024 / (2 * HD);      // key rows of a wave-load
    constexpr int NLOAD = HD / (8 * W);         // wave-loads per wave for the keys of a tile, and as many for the values
    constexpr int TILE = 2 * 64 * HD;           // elements of a stage: keys, then values
    static_assert(NS == 2 || NS == 3, "two or three stages");
    __shared__ __attribute__((aligned(1024))) bf16 tiles[G * NS * TILE];
    __shared__ int page_copy[PAGE_COPY];
    const int per_xcd = (a.n_items * a.nh + 7) / 8;
    const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (logical >= a.n_items * a.nh) return;
    // later items of a prompt see more keys: even heads run them last to first, odd heads first to last, so that
    // the blocks that come to share a CU (two fit, handed out in turn) have about the same work together
    const int h = logical / a.n_items;
    const int item = (h & 1) ? logical % a.n_items : a.n_items - 1 - logical % a.n_items;
    const int tid = G == 1 ? (int)threadIdx.x : (int)threadIdx.x % (W * 64), lane = tid & 63, wave = tid >> 6;      // within the group
    const int grp = G == 1 ? 0 : (int)threadIdx.x / (W * 64);
    const int li = lane & 15, g = lane >> 4;
    const int kvh = h / (a.nh / a.nkv);
    const int tok_first = a.item_tok[item], n_all = a.item_n[item];
    const int* bt = a.block_table + (size_t)a.item_seq[item] * a.max_blocks;
    const int bs = a.bs;
    const int pmin = a.positions[tok_first], pmax = a.positions[tok_first + n_all - 1];
    const int kv_begin = a.window > 0 ? max(0, pmin - a.window + 1) : 0;
    const int kv_end = pmax + 1;
    const int tok0 = tok_first + 16 * wave, n = min(16, n_all - 16 * wave);
    int lo = 1, hi = 0;
    const bf16* qrow = nullptr;
    if (li < n) {
        hi = a.positions[tok0 + li];
        lo = a.window > 0 ? max(0, hi - a.window + 1) : 0;
        qrow = (const bf16*)a.q + (size_t)(tok0 + li) * a.ldq + (size_t)h * HD;
    }
    int w_lo = 0x7fffffff, w_hi = -1;
    int w_lo_max = 0x7fffffff, w_hi_min = -1;
    if (n > 0) {
        w_hi = a.positions[tok0 + n - 1];
        w_lo = a.window > 0 ? max(0, a.positions[tok0] - a.window + 1) : 0;
        if (n == 16) {
            w_hi_min = a.positions[tok0];
            w_lo_max = a.window > 0 ? max(0, w_hi - a.window + 1) : 0;
        }
    }
    const float c2 = a.scale * LOG2E;
    float m = NEG_INF, l = 0.f;
    f32x4_t o[CB];
    bf16x8_t qf[KS];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) o[cb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < KS; ++u) {
        const uint4 v = qrow ? *(const uint4*)(qrow + 32 * u + 8 * g) : make_uint4(0, 0, 0, 0);
        qf[u] = __builtin_bit_cast(bf16x8_t, v);
    }
    int first_blk, last_blk, unused;
    page_slot(a, kv_begin, first_blk, unused);
    page_slot(a, kv_end - 1, last_blk, unused);
    const PageLookup pl = stage_pages(bt, page_copy, first_blk, last_blk);

    // what this lane fetches in each of its wave-loads, relative to the tile's first key / value row 0
    int k_src[NLOAD], v_src[NLOAD];
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
        const int j = wave + W * i;                          // wave-load j of HD / 8
        const int row = KROWS * j + lane / NCH;              // LDS key row 16 kb + 4 a + b
        const int key = 16 * ((row >> 2) & 3) + 4 * (row >> 4) + (row & 3);
        k_src[i] = key * HD + (((lane % NCH) ^ (NCH == 16 ? (row & 15) : ((row >> 1) & 7))) * 8);
        const int d = 8 * j + (lane >> 3);                   // value row
        v_src[i] = d * bs + (((lane & 7) ^ ((d >> 1) & 7)) * 8);
    }
    auto issue = [&](int kt0, int stage) {
        int blk, slot;
        page_slot(a, kt0, blk, slot);
        const size_t page = (size_t)__builtin_amdgcn_readfirstlane(pl.page(blk));
        const bf16* kbase = (const bf16*)a.k_pages + ((page * a.nkv + kvh) * bs + slot) * HD;
        const bf16* vbase = (const bf16*)a.v_pages + (page * a.nkv + kvh) * HD * bs + slot;
        bf16* st = tiles + (grp * NS + stage) * TILE;
#pragma unroll
        for (int i = 0; i < NLOAD; ++i)
            __builtin_amdgcn_global_load_lds((fx_global_ptr)(kbase + k_src[i]), (fx_lds_ptr)(st + (wave + W * i) * 512), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < NLOAD; ++i)
            __builtin_amdgcn_global_load_lds((fx_global_ptr)(vbase + v_src[i]),
                                             (fx_lds_ptr)(st + 64 * HD + (wave + W * i) * 512), 16, 0, 0);
    };
    // operands: key row 16 kb + li, chunk 4 u + g; value row 16 cb + li, chunks 2 g and 2 g + 1
    const int k_at = li * HD, v_at = 64 * HD + li * 64;
    const int ksw = NCH == 16 ? li : (li >> 1) & 7, vsw = (li >> 1) & 7;

    // Every wave of the block goes through the same barriers: the loop runs over rounds of G tiles, of which group
    // grp takes tile grp (a round's last tiles may not exist: that group then only keeps step).
    const int kt_first = (kv_begin / 64) * 64;
    if (kt_first + 64 * grp < kv_end) issue(kt_first + 64 * grp, 0);
    if (NS == 3 && kt_first + 64 < kv_end) issue(kt_first + 64, 1);
    int stage = 0;
    for (int round0 = kt_first; round0 < kv_end; round0 += 64 * G, stage = (stage + 1 == NS ? 0 : stage + 1)) {
        const int kt0 = round0 + 64 * grp;
        // this wave's part of the tile has landed (with three stages the next tile's loads may still fly)
        if (NS == 3 && kt0 + 64 < kv_end) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NLOAD) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();                           // ... everyone's has, and the stage read last is free
        if (kt0 + 64 * G * (NS - 1) < kv_end) issue(kt0 + 64 * G * (NS - 1), (stage + NS - 1) % NS);
        bf16* st = tiles + (grp * NS + stage) * TILE;
        // a tile at the edge: values of keys outside become zeros.  Whether any tile of the round is one is the
        // same for all waves, so all of them meet at the barrier behind the zeros.
        bool any_edge = false;
#pragma unroll
        for (int q = 0; q < G; ++q) {
            const int kq = round0 + 64 * q;
            any_edge = any_edge || (kq < kv_end && (kq < kv_begin || kq + 64 > kv_end));
        }
        if (any_edge) {
            if (kt0 < kv_end && (kt0 < kv_begin || kt0 + 64 > kv_end)) {
                for (int idx = tid; idx < HD * 64; idx += W * 64) {
                    const int d = idx >> 6, key = idx & 63;
                    if (kt0 + key < kv_begin || kt0 + key >= kv_end)
                        st[64 * HD + d * 64 + (((key >> 3) ^ ((d >> 1) & 7)) * 8) + (key & 7)].bits = 0;
                }
            }
            lds_barrier();      // the zeros are in LDS (a bare s_barrier does not wait for this wave's stores) before any wave reads values
        }
        if (kt0 >= kv_end || kt0 > w_hi || kt0 + 64 <= w_lo) continue;      // no such tile, or nothing in it for this wave's rows
        f32x4_t sc[4];
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            sc[kb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < KS; ++u) {
                const bf16x8_t kf = *(const bf16x8_t*)(st + k_at + kb * 16 * HD + (((4 * u + g) ^ ksw) * 8));
                sc[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[u], sc[kb], 0, 0, 0);
            }
        }
        const bool whole = kt0 >= w_lo_max && kt0 + 63 <= w_hi_min && kt0 >= kv_begin;
        uint4 p_lo, p_hi;
        const float alpha = whole ? softmax_step<false>(sc, kt0 + 16 * g, lo, hi, c2, m, l, p_lo, p_hi)
                                  : softmax_step<true>(sc, kt0 + 16 * g, lo, hi, c2, m, l, p_lo, p_hi);
        const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;
        float al[4] = {1.f, 1.f, 1.f, 1.f};
        if (rescale) {
#pragma unroll
            for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, 4 * g + r, 64);
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const bf16* vr = st + v_at + cb * 16 * 64;
            o[cb] = pv_step(o[cb], rescale, al, p_lo, p_hi, *(const uint4*)(vr + (((2 * g) ^ vsw) * 8)),
                            *(const uint4*)(vr + (((2 * g + 1) ^ vsw) * 8)));
        }
    }
    if constexpr (G == 2) {
        // group 1 hands over maximum, sum and outputs, lane for lane, through the LDS that the tiles no longer need
        __syncthreads();
        float* hand = (float*)tiles + (size_t)wave * ((2 + 4 * CB) * 64);
        if (grp == 1) {
            hand[lane] = m;
            hand[64 + lane] = l;
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                for (int r = 0; r < 4; ++r) hand[(2 + 4 * cb + r) * 64 + lane] = o[cb][r];
        }
        __syncthreads();
        if (grp == 1) return;
        const float m1 = hand[lane], l1 = hand[64 + lane];
        const float mn = fmaxf(m, m1), mu = (mn == NEG_INF) ? 0.f : mn;
        const float f0 = __builtin_amdgcn_exp2f(m - mu), f1 = __builtin_amdgcn_exp2f(m1 - mu);
        l = l * f0 + l1 * f1;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float a0 = __shfl(f0, 4 * g + r, 64), a1 = __shfl(f1, 4 * g + r, 64);      // of the accumulator's row 4 g + r
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) o[cb][r] = o[cb][r] * a0 + hand[(2 + 4 * cb + r) * 64 + lane] * a1;
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * g + r;
        const float lr = __shfl(l, row, 64);
        if (row < n) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
                from_float((bf16*)a.out + (size_t)(tok0 + row) * a.ldo + (size_t)h * HD + 16 * cb + li, o[cb][r] / lr);
        }
    }
}

// Switch for tests and measurement (ferrox_amd/debug.py is its one caller); the product path never sets it.
static int g_direct = 2;     // "direct_stages": 0 keeps prefill on the kernel that stages tiles through registers; 2 (default), 3: stages
static int g_groups = 0;     // "direct_groups": 1 or 2 groups of waves per block of 64 queries in that kernel (0: by the number of blocks)
FX_API int fx_debug_set(const char* key, int value) {
    if (!strcmp(key, "direct_stages")) { g_direct = value; return 0; }
    if (!strcmp(key, "direct_groups")) { g_groups = value; return 0; }
    FX_REQUIRE(false, "attention: no debug switch '%s' (direct_stages, direct_groups)", key);
    return 1;
}

static bool mfma_ok(int dtype, int hd, int bs, const void* q, long ldq, const void* k_pages, const void* v_pages) {
    return dtype == FX_BF16 && hd % 16 == 0 && bs % 16 == 0 && hd % 8 == 0 && ldq % 8 == 0 &&
           (((uintptr_t)q | (uintptr_t)k_pages | (uintptr_t)v_pages) % 16 == 0);
}

// ---------------------------------------------------------------------------
static int check_common(const char* who, int dtype, int nh, int nkv, int hd, int bs, int window, float scale) {
    // (the bfloat16 kernels take a row's maximum over the raw scores and scale it once, which is the maximum of
    // the scaled scores only under a positive scale)
    FX_REQUIRE(scale > 0.f && scale < INFINITY, "%s: the scale of the scores must be positive and finite, got %g", who, (double)scale);
    FX_REQUIRE(dtype == FX_F32 || dtype == FX_BF16, "%s: unknown dtype %d", who, dtype);
    FX_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "%s: n_heads %d must be a multiple of n_kv_heads %d", who, nh, nkv);
    FX_REQUIRE(hd > 0 && hd <= HD_MAX, "%s: head_dim %d is outside 1..%d", who, hd, HD_MAX);
    FX_REQUIRE(bs > 0, "%s: block size %d", who, bs);
    FX_REQUIRE(window >= 0, "%s: window %d", who, window);
    return 0;
}

// Items of up to 128 queries are for bfloat16 with head_dim 64 or 128 and pages of a multiple of 64 keys.
static bool wide_items_ok(int dtype, int hd, int bs) {
    return dtype == FX_BF16 && bs % 64 == 0 && (hd == 64 || hd == 128) && g_direct == 2;
}
FX_API int fx_attn_tile_queries(int dtype, int hd, int bs) { return wide_items_ok(dtype, hd, bs) ? 128 : 64; }

// Queries in blocks: item i covers item_n[i] <= tile_q consecutive tokens of one sequence; tile_q is 64, or what
// fx_attn_tile_queries gives for these sizes.
FX_API int fx_attn_tiles(void* stream, int dtype, const void* q, long ldq, void* out, long ldo,
                         const void* k_pages, const void* v_pages, const int* block_table, int max_blocks,
                         const int* positions, const int* item_seq, const int* item_tok, const int* item_n,
                         int n_items, int nh, int nkv, int hd, int bs, int window, float scale, int tile_q) {
    if (check_common("attn_tiles", dtype, nh, nkv, hd, bs, window, scale)) return 1;
    FX_REQUIRE(tile_q == 64 || (tile_q == 128 && wide_items_ok(dtype, hd, bs) && mfma_ok(dtype, hd, bs, q, ldq, k_pages, v_pages)),
               "attn_tiles: items of %d queries (64, or 128 where fx_attn_tile_queries says so)", tile_q);
    if (n_items <= 0) return 0;
    AttnArgs a = {};
    a.q = q; a.ldq = ldq; a.out = out; a.ldo = ldo; a.k_pages = k_pages; a.v_pages = v_pages;
    a.block_table = block_table; a.max_blocks = max_blocks; a.positions = positions;
    a.item_seq = item_seq; a.item_tok = item_tok; a.item_n = item_n;
    a.nh = nh; a.nkv = nkv; a.hd = hd; a.bs = bs; a.window = window; a.scale = scale;
    a.bs_shift = log2_or_minus_one(bs);
    a.n_items = n_items;
    dim3 grid(n_items * 4, nh), grid_blocks(8 * ceil_div((long)n_items * nh, 8));     // a wave per 16 queries / a block per item
    hipStream_t s = (hipStream_t)stream;
    // no more blocks than CUs: a block's chain of tiles is what takes the time, and two groups of waves halve it
    // (measured: 512-token portions at depth 8k-24k 130 and 360 us against 214 and 616 us; from 448 blocks on, one
    // group and two blocks to a CU are as fast or faster)
    const bool two_groups = g_groups ? g_groups == 2 : (long)n_items * nh <= fx_compute_units();
    if (dtype == FX_F32)
        attn_tile_kernel<float><<<grid, 64, 0, s>>>(a);
    else if (mfma_ok(dtype, hd, bs, q, ldq, k_pages, v_pages)) {
        if (tile_q == 128 && hd == 128 && two_groups) attn_mfma_direct_kernel<128, 2, 8, 2><<<grid_blocks, 1024, 0, s>>>(a);
        else if (tile_q == 128 && hd == 64 && two_groups) attn_mfma_direct_kernel<64, 2, 8, 2><<<grid_blocks, 1024, 0, s>>>(a);
        else if (tile_q == 128 && hd == 128) attn_mfma_direct_kernel<128, 2, 8><<<grid_blocks, 512, 0, s>>>(a);
        else if (tile_q == 128) attn_mfma_direct_kernel<64, 2, 8><<<grid_blocks, 512, 0, s>>>(a);
        else if (bs % 64 == 0 && hd == 128 && g_direct == 2 && two_groups) attn_mfma_direct_kernel<128, 2, 4, 2><<<grid_blocks, 512, 0, s>>>(a);
        else if (bs % 64 == 0 && hd == 64 && g_direct == 2 && two_groups) attn_mfma_direct_kernel<64, 2, 4, 2><<<grid_blocks, 512, 0, s>>>(a);
        else if (bs % 64 == 0 && hd == 128 && g_direct == 3) attn_mfma_direct_kernel<128, 3><<<grid_blocks, 256, 0, s>>>(a);
        else if (bs % 64 == 0 && hd == 128 && g_direct) attn_mfma_direct_kernel<128, 2><<<grid_blocks, 256, 0, s>>>(a);
        else if (bs % 64 == 0 && hd == 64 && g_direct) attn_mfma_direct_kernel<64, 2><<<grid_blocks, 256, 0, s>>>(a);
        else if (hd <= 32) attn_mfma_block_kernel<32><<<grid_blocks, 256, 0, s>>>(a);
        else if (hd <= 64) attn_mfma_block_kernel<64><<<grid_blocks, 256, 0, s>>>(a);
        else if (hd <= 128) attn_mfma_block_kernel<128><<<grid_blocks, 256, 0, s>>>(a);
        else attn_mfma_tile_kernel<256><<<grid, 64, 0, s>>>(a);       // too large to stage in LDS
    } else
        attn_tile_kernel<bf16><<<grid, 64, 0, s>>>(a);
    FX_CHECK_LAUNCH("attn_tiles");
    return 0;
}

// Single queries.  part_o has n_items*nh*splits*hd floats, part_ml n_items*nh*splits*2;
// splits * chunk must cover every position + 1.
static int attn_decode_launch(void* stream, int dtype, const void* q, long ldq, void* out, long ldo,
                              const void* k_pages, const void* v_pages, const int* block_table, int max_blocks,
                              const int* positions, const int* item_seq, const int* item_tok, int n_items,
                              int nh, int nkv, int hd, int bs, int window, float scale,
                              float* part_o, float* part_ml, int splits, int chunk, int waves) {
    AttnArgs a = {};
    a.q = q; a.ldq = ldq; a.out = out; a.ldo = ldo; a.k_pages = k_pages; a.v_pages = v_pages;
    a.block_table = block_table; a.max_blocks = max_blocks; a.positions = positions;
    a.item_seq = item_seq; a.item_tok = item_tok; a.item_n = nullptr;
    a.nh = nh; a.nkv = nkv; a.hd = hd; a.bs = bs; a.window = window; a.scale = scale;
    a.bs_shift = log2_or_minus_one(bs);
    a.part_o = part_o; a.part_ml = part_ml; a.splits = splits; a.chunk = chunk;
    dim3 grid(n_items, nh, splits), grid2(n_items, nh);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FX_F32) {
        attn_decode_kernel<float><<<grid, 64, 0, s>>>(a);
        attn_decode_merge_kernel<float><<<grid2, 128, splits * sizeof(float), s>>>(a);
    } else if (mfma_ok(dtype, hd, bs, q, ldq, k_pages, v_pages)) {
        const int group = nh / nkv;
        dim3 gridm(nkv * ((group + 15) / 16), n_items, splits);
        // as many waves per block (up to 8, and no more than a split has tiles) as their results fit in LDS
        const int rows = group < 16 ? group : 16;
        const int hdc = hd <= 32 ? 32 : (hd <= 64 ? 64 : (hd <= 128 ? 128 : 256));
        const int nw_max = hd <= 128 ? 8 : 4;      // the widest heads need the registers of half a block
        int nw = nw_max;
        FX_REQUIRE(waves >= 0 && waves <= nw_max, "attn_decode: %d waves per block, this head size takes up to %d", waves, nw_max);
        const long n_blocks = (long)n_items * gridm.x * splits;
        FX_REQUIRE(n_items <= 65535 && splits <= 65535, "attn_decode: %d single queries in %d chunks each are more than a launch takes", n_items, splits);
        // fewer waves per block when there are blocks enough: a chunk's tiles then divide more evenly.  Whole
        // sequences (one chunk) keep four waves a block, or get one each once the blocks number half the GPU's wave
        // slots; two waves a block are behind both (decode steps of 72, 96 and 128 sequences of 16 kv heads: 12.3,
        // 14.3 and 16.1 ms with two waves a block, 11.9, 13.5 and 15.9 with four, 11.7, 13.3 and 15.6 with one).
        const long slots = 8L * fx_compute_units();
        const int nw_min = splits > 1 ? 1 : 4;
        while (nw > 1 && ((size_t)nw * rows * (hdc + 2) * 4 > 48 * 1024 || nw * 64 >= 2 * chunk)) nw >>= 1;
        while (nw > nw_min && n_blocks * (nw / 2) >= slots) nw >>= 1;
        if (splits == 1 && 2 * n_blocks >= slots) nw = 1;
        if (waves > 0 && (size_t)waves * rows * (hdc + 2) * 4 <= 48 * 1024) nw = waves;      // the caller's choice
        const size_t shm = (size_t)nw * rows * (hdc + 2) * 4;
        if (hd <= 32) attn_mfma_decode_block_kernel<32, 512><<<gridm, nw * 64, shm, s>>>(a);
        else if (hd <= 64) attn_mfma_decode_block_kernel<64, 512><<<gridm, nw * 64, shm, s>>>(a);
        else if (hd <= 128) attn_mfma_decode_block_kernel<128, 512><<<gridm, nw * 64, shm, s>>>(a);
        else attn_mfma_decode_block_kernel<256, 256><<<gridm, nw * 64, shm, s>>>(a);
        if (splits > 1) attn_decode_merge_kernel<bf16><<<grid2, 128, splits * sizeof(float), s>>>(a);
    } else {
        attn_decode_kernel<bf16><<<grid, 64, 0, s>>>(a);
        attn_decode_merge_kernel<bf16><<<grid2, 128, splits * sizeof(float), s>>>(a);
    }
    FX_CHECK_LAUNCH("attn_decode");
    return 0;
}

static int attn_decode_check(int dtype, int nh, int nkv, int hd, int bs, int window, float scale, int splits, int chunk) {
    if (check_common("attn_decode", dtype, nh, nkv, hd, bs, window, scale)) return 1;
    FX_REQUIRE(splits > 0 && chunk > 0 && chunk % 64 == 0, "attn_decode: chunk %d must be a positive multiple of 64", chunk);
    FX_REQUIRE(splits <= 8192, "attn_decode: %d chunks are more than the merge kernel takes (8192)", splits);
    return 0;
}

FX_API int fx_attn_decode(void* stream, int dtype, const void* q, long ldq, void* out, long ldo,
                          const void* k_pages, const void* v_pages, const int* block_table, int max_blocks,
                          const int* positions, const int* item_seq, const int* item_tok, int n_items,
                          int nh, int nkv, int hd, int bs, int window, float scale,
                          float* part_o, float* part_ml, int splits, int chunk, int waves) {
    if (attn_decode_check(dtype, nh, nkv, hd, bs, window, scale, splits, chunk)) return 1;
    if (n_items <= 0) return 0;
    return attn_decode_launch(stream, dtype, q, ldq, out, ldo, k_pages, v_pages, block_table, max_blocks, positions,
                              item_seq, item_tok, n_items, nh, nkv, hd, bs, window, scale, part_o, part_ml, splits,
                              chunk, waves);
}

// ---------------------------------------------------------------------------
// fx_attn_decode_static: fx_attn_decode for callers that cannot allocate (see attention.h).  The chunks' partial
// results, which fx_attn_decode's caller brings in part_o and part_ml, live in this array instead.  Each GPU that
// the library runs on holds its own copy until the process ends.  Every call on a GPU uses that GPU's copy from its
// start: two calls that overlap on one GPU (two streams, two threads) race; calls that follow each other on one
// stream do not.  Nothing in it has to start at zero: every chunk writes its (m, l) and its outputs before the merge
// reads them, and the merge reads no chunk of another call's larger shape.
// ---------------------------------------------------------------------------
#define FX_ATTN_STATIC_FLOATS (4u << 20)       // 16 MiB: e.g. 64 queries x 16 heads x 31 chunks x (128 + 2) floats
static __device__ __align__(256) float fx_attn_scratch[FX_ATTN_STATIC_FLOATS];

#define FX_MAX_DEVICES 64
static float* g_attn_scratch_ptr[FX_MAX_DEVICES];    // per device: the address of that device's copy (null: not asked yet)

// The array's name is only a host-side stand-in; its memory on a device is found with hipGetSymbolAddress, once
// per device, with that device current.  `stream`: the stream a call is for (its device is the one whose copy is
// used; null: the current device).  While `stream` is being captured nothing is looked up: the address must be
// known by then, through fx_attn_static_init() or an earlier call on that device.
static int attn_scratch_of(hipStream_t stream, float** out) {
    int current = -1, dev = -1;
    hipError_t e = hipGetDevice(&current);
    FX_REQUIRE(e == hipSuccess, "attn_decode_static: hipGetDevice: %s", hipGetErrorString(e));
    dev = current;
    if (stream) {
        e = hipStreamGetDevice(stream, &dev);
        FX_REQUIRE(e == hipSuccess, "attn_decode_static: hipStreamGetDevice: %s", hipGetErrorString(e));
    }
    FX_REQUIRE(dev >= 0 && dev < FX_MAX_DEVICES, "attn_decode_static: device %d is beyond the %d this library keeps", dev, FX_MAX_DEVICES);
    float* p = __atomic_load_n(&g_attn_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        if (stream) {
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            e = hipStreamIsCapturing(stream, &capturing);
            FX_REQUIRE(e == hipSuccess, "attn_decode_static: hipStreamIsCapturing: %s", hipGetErrorString(e));
            FX_REQUIRE(capturing == hipStreamCaptureStatusNone,
                       "attn_decode_static: the stream is being captured and device %d's array has not been looked up yet; "
                       "call fx_attn_static_init() with that device current before the capture begins", dev);
        }
        if (dev != current) {
            e = hipSetDevice(dev);
            FX_REQUIRE(e == hipSuccess, "attn_decode_static: hipSetDevice(%d): %s", dev, hipGetErrorString(e));
        }
        void* sym = nullptr;
        e = hipGetSymbolAddress(&sym, HIP_SYMBOL(fx_attn_scratch));
        if (dev != current) (void)hipSetDevice(current);
        FX_REQUIRE(e == hipSuccess && sym, "attn_decode_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        p = (float*)sym;
        __atomic_store_n(&g_attn_scratch_ptr[dev], p, __ATOMIC_RELEASE);     // (two threads would store the same address)
    }
    *out = p;
    return 0;
}

// The array's address on the current device, looked up now (no allocation; call it once per device before calls
// that are captured into a graph).
FX_API int fx_attn_static_init(void) {
    float* p;
    return attn_scratch_of(nullptr, &p);
}

FX_API long fx_attn_static_capacity(void) { return (long)FX_ATTN_STATIC_FLOATS; }

FX_API int fx_attn_decode_static(void* stream, int dtype, const void* q, long ldq, void* out, long ldo,
                                 const void* k_pages, const void* v_pages, const int* block_table, int max_blocks,
                                 const int* positions, const int* item_seq, const int* item_tok, int n_items,
                                 int nh, int nkv, int hd, int bs, int window, float scale, int splits, int chunk, int waves) {
    if (attn_decode_check(dtype, nh, nkv, hd, bs, window, scale, splits, chunk)) return 1;
    if (n_items <= 0) return 0;
    const size_t n_o = (size_t)n_items * nh * splits * hd, n_ml = (size_t)n_items * nh * splits * 2;
    FX_REQUIRE(n_o + n_ml <= FX_ATTN_STATIC_FLOATS,
               "attn_decode_static: %d queries x %d heads x %d chunks x (%d + 2) floats = %zu are more than the %u this entry "
               "point holds; use fewer chunks or fx_attn_decode with buffers of your own",
               n_items, nh, splits, hd, n_o + n_ml, FX_ATTN_STATIC_FLOATS);
    float* scratch = nullptr;
    if (attn_scratch_of((hipStream_t)stream, &scratch)) return 1;
    return attn_decode_launch(stream, dtype, q, ldq, out, ldo, k_pages, v_pages, block_table, max_blocks, positions,
                              item_seq, item_tok, n_items, nh, nkv, hd, bs, window, scale, scratch, scratch + n_o, splits,
                              chunk, waves);
}
