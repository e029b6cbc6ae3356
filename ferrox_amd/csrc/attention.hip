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
    float scale;
    // decode only
    float* part_o;   // [items, nh, splits, hd]
    float* part_ml;  // [items, nh, splits, 2]
    int splits, chunk;
};

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
// Any number of queries: one wave per (tile of up to 16 queries of one
// sequence, head); lanes are keys for the scores and head dimensions for the
// output.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(64) void attn_tile_kernel(AttnArgs a) {
    __shared__ float Qs[TQ][HD_MAX];
    __shared__ float Ps[TQ][64];
    const int item = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int kvh = h / (a.nh / a.nkv);
    const int tok0 = a.item_tok[item], n = a.item_n[item];
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

template <typename T>
__global__ __launch_bounds__(64) void attn_decode_merge_kernel(AttnArgs a) {
    const int item = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int tok = a.item_tok[item];
    const int hd = a.hd;
    const float* po = a.part_o + ((size_t)item * a.nh + h) * a.splits * hd;
    const float* pml = a.part_ml + ((size_t)item * a.nh + h) * a.splits * 2;
    float m = NEG_INF;
    for (int s = 0; s < a.splits; ++s) m = fmaxf(m, pml[2 * s]);
    float l = 0.f;
    for (int s = 0; s < a.splits; ++s)
        if (pml[2 * s] != NEG_INF) l += pml[2 * s + 1] * expf(pml[2 * s] - m);
    for (int d = lane; d < hd; d += 64) {
        float acc = 0.f;
        for (int s = 0; s < a.splits; ++s)
            if (pml[2 * s] != NEG_INF) acc += po[(size_t)s * hd + d] * expf(pml[2 * s] - m);
        from_float((T*)a.out + (size_t)tok * a.ldo + (size_t)h * hd + d, acc / l);
    }
}

// ---------------------------------------------------------------------------
static int check_common(const char* who, int dtype, int nh, int nkv, int hd, int bs, int window) {
    FX_REQUIRE(dtype == FX_F32 || dtype == FX_BF16, "%s: unknown dtype %d", who, dtype);
    FX_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "%s: n_heads %d must be a multiple of n_kv_heads %d", who, nh, nkv);
    FX_REQUIRE(hd > 0 && hd <= HD_MAX, "%s: head_dim %d is outside 1..%d", who, hd, HD_MAX);
    FX_REQUIRE(bs > 0, "%s: block size %d", who, bs);
    FX_REQUIRE(window >= 0, "%s: window %d", who, window);
    return 0;
}

// Queries in tiles: item i covers item_n[i] <= 16 consecutive tokens of one sequence.
FX_API int fx_attn_tiles(void* stream, int dtype, const void* q, long ldq, void* out, long ldo,
                         const void* k_pages, const void* v_pages, const int* block_table, int max_blocks,
                         const int* positions, const int* item_seq, const int* item_tok, const int* item_n,
                         int n_items, int nh, int nkv, int hd, int bs, int window, float scale) {
    if (check_common("attn_tiles", dtype, nh, nkv, hd, bs, window)) return 1;
    if (n_items <= 0) return 0;
    AttnArgs a = {};
    a.q = q; a.ldq = ldq; a.out = out; a.ldo = ldo; a.k_pages = k_pages; a.v_pages = v_pages;
    a.block_table = block_table; a.max_blocks = max_blocks; a.positions = positions;
    a.item_seq = item_seq; a.item_tok = item_tok; a.item_n = item_n;
    a.nh = nh; a.nkv = nkv; a.hd = hd; a.bs = bs; a.window = window; a.scale = scale;
    dim3 grid(n_items, nh);
    if (dtype == FX_F32)
        attn_tile_kernel<float><<<grid, 64, 0, (hipStream_t)stream>>>(a);
    else
        attn_tile_kernel<bf16><<<grid, 64, 0, (hipStream_t)stream>>>(a);
    FX_CHECK_LAUNCH("attn_tiles");
    return 0;
}

// Single queries.  part_o has n_items*nh*splits*hd floats, part_ml n_items*nh*splits*2;
// splits * chunk must cover every position + 1.
FX_API int fx_attn_decode(void* stream, int dtype, const void* q, long ldq, void* out, long ldo,
                          const void* k_pages, const void* v_pages, const int* block_table, int max_blocks,
                          const int* positions, const int* item_seq, const int* item_tok, int n_items,
                          int nh, int nkv, int hd, int bs, int window, float scale,
                          float* part_o, float* part_ml, int splits, int chunk) {
    if (check_common("attn_decode", dtype, nh, nkv, hd, bs, window)) return 1;
    FX_REQUIRE(splits > 0 && chunk > 0 && chunk % 64 == 0, "attn_decode: chunk %d must be a positive multiple of 64", chunk);
    if (n_items <= 0) return 0;
    AttnArgs a = {};
    a.q = q; a.ldq = ldq; a.out = out; a.ldo = ldo; a.k_pages = k_pages; a.v_pages = v_pages;
    a.block_table = block_table; a.max_blocks = max_blocks; a.positions = positions;
    a.item_seq = item_seq; a.item_tok = item_tok; a.item_n = nullptr;
    a.nh = nh; a.nkv = nkv; a.hd = hd; a.bs = bs; a.window = window; a.scale = scale;
    a.part_o = part_o; a.part_ml = part_ml; a.splits = splits; a.chunk = chunk;
    dim3 grid(n_items, nh, splits), grid2(n_items, nh);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FX_F32) {
        attn_decode_kernel<float><<<grid, 64, 0, s>>>(a);
        attn_decode_merge_kernel<float><<<grid2, 64, 0, s>>>(a);
    } else {
        attn_decode_kernel<bf16><<<grid, 64, 0, s>>>(a);
        attn_decode_merge_kernel<bf16><<<grid2, 64, 0, s>>>(a);
    }
    FX_CHECK_LAUNCH("attn_decode");
    return 0;
}
