// Row-wise kernels: embedding gather, RMSNorm, rotary + cache write, residual
// add, casts, the weighted sum of routed expert outputs.
//
// The residual stream `h` is float32 in both precisions; normed activations and
// q/k/v are in the activation type T (float or bf16).  Statistics, angles and
// sums are computed in float32.
#include "common.h"

FX_DEFINE_LAST_ERROR()

// ---------------------------------------------------------------------------
// embedding: h[t, :] = table[ids[t], :]   (no scale; ferrox-models/src/decoder.rs:1279-1284)
// ---------------------------------------------------------------------------
template <typename W>
__global__ void embed_kernel(const W* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ h, int H, int V) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 || id >= V) {  // the host rejects such ids; never read outside the table
        for (int c = threadIdx.x; c < H; c += blockDim.x) h[(size_t)t * H + c] = __int_as_float(0x7fc00000);
        return;
    }
    const W* row = table + (size_t)id * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) h[(size_t)t * H + c] = to_float(row[c]);
}

FX_API int fx_embed(void* stream, int w_dtype, const void* table, const int* ids, float* h,
                    int T, int H, int V) {
    FX_REQUIRE(T >= 0 && H > 0 && V > 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (w_dtype == FX_F32)
        embed_kernel<float><<<T, 256, 0, s>>>((const float*)table, ids, h, H, V);
    else if (w_dtype == FX_BF16)
        embed_kernel<bf16><<<T, 256, 0, s>>>((const bf16*)table, ids, h, H, V);
    else
        return fx_fail("embed: unknown table dtype %d", w_dtype);
    FX_CHECK_LAUNCH("embed");
    return 0;
}

// ---------------------------------------------------------------------------
// RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w, multiply order x*s*w
// (ferrox-core/src/matmul.rs:62-69).  Input rows are float32 (the residual
// stream), optionally gathered through `rows`; output is T.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ h, const int* __restrict__ rows,
                                                      const void* __restrict__ w, int w_dtype,
                                                      T* __restrict__ out, int H, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float* x = h + (size_t)(rows ? rows[r] : r) * H;
    if (H <= 256 * 16) {   // the row stays in registers: one pass over memory, the weights fetched meanwhile
        float xv[16], wv[16];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = threadIdx.x + i * 256;
            xv[i] = c < H ? x[c] : 0.f;
        }
        load_strided_as_float<16, 256>(w, w_dtype, threadIdx.x, H, wv);
#pragma unroll
        for (int i = 0; i < 16; ++i) ss += xv[i] * xv[i];
        ss = block_sum<4>(ss, red);
        const float scale = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = threadIdx.x + i * 256;
            if (c < H) from_float(out + (size_t)r * H + c, xv[i] * scale * wv[i]);
        }
        return;
    }
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += 256) {
        float v = x[c];
        ss += v * v;
    }
    ss = block_sum<4>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)H + eps);
    for (int c = threadIdx.x; c < H; c += 256)
        from_float(out + (size_t)r * H + c, x[c] * scale * load_as_float(w, w_dtype, c));
}

FX_API int fx_rmsnorm(void* stream, int out_dtype, const float* h, const int* rows, const void* w,
                      int w_dtype, void* out, int R, int H, float eps) {
    FX_REQUIRE(R >= 0 && H > 0, "rmsnorm: bad sizes R=%d H=%d", R, H);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "rmsnorm: unknown weight dtype %d", w_dtype);
    if (R == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == FX_F32)
        rmsnorm_kernel<float><<<R, 256, 0, s>>>(h, rows, w, w_dtype, (float*)out, H, eps);
    else if (out_dtype == FX_BF16)
        rmsnorm_kernel<bf16><<<R, 256, 0, s>>>(h, rows, w, w_dtype, (bf16*)out, H, eps);
    else
        return fx_fail("rmsnorm: unknown output dtype %d", out_dtype);
    FX_CHECK_LAUNCH("rmsnorm");
    return 0;
}

// ---------------------------------------------------------------------------
// Rotary position encoding of q and k, and the write of k and v into the pages.
//
// Split-half pairing (i, i + rot/2), angle = (float)pos * inv_freq[i] in float32, as the reference
// multiplies them (ferrox-core/src/attention.rs:20-32); the caller brings inv_freq[i] = theta^(-2i/rot)
// as a table of rot/2 floats, so that the frequencies are the same numbers wherever they are made.
// `interleaved` pairs (2i, 2i+1) instead.
// `freq_factors` (rot/2 floats, or null): the angle of pair i is divided by freq_factors[i]
// (per-band frequency correction, attention.rs:319-333).
// rot = 0 rotates nothing.  v is never rotated.  Key pages hold
// [page][kv_head][slot][head_dim]; value pages hold the transpose
// [page][kv_head][head_dim][slot], which is what the attention kernels read.
// ---------------------------------------------------------------------------
// The first T * split blocks rotate: `split` blocks share a token, each computes the angles' sines
// and cosines once and takes its part of the heads of q (in place) and of k (into its page); few
// tokens get several blocks each, many tokens one.  The blocks after them write v: one block per (eight
// consecutive tokens, kv head), so that eight tokens that follow each other in one page go out as
// one 16-byte store per head dimension into the transposed page.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
    T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const int* __restrict__ positions, const int* __restrict__ token_seq,
    const int* __restrict__ block_table, int max_blocks, T* __restrict__ k_pages, T* __restrict__ v_pages,
    int n_tokens, int split, int nh, int nkv, int hd, int bs, int rot, int interleaved, const float* __restrict__ inv_freq, int vec8,
    const float* __restrict__ freq_factors) {
    __shared__ float cs[128], sn[128];     // rot / 2 <= 128
    const int tid = threadIdx.x;
    const int half = rot >> 1;
    if ((int)blockIdx.x < n_tokens * split) {
        const int t = blockIdx.x / split, part = blockIdx.x % split, step = 256 * split;
        const int pos = positions[t];
        for (int p = tid; p < half; p += 256) {
            float angle = (float)pos * inv_freq[p];
            if (freq_factors) angle = angle / freq_factors[p];
            sincosf(angle, &sn[p], &cs[p]);
        }
        __syncthreads();
        T* k_dst = nullptr;
        if (k_pages) {
            const int page = block_table[(size_t)token_seq[t] * max_blocks + pos / bs];
            k_dst = k_pages + ((size_t)page * nkv * bs + pos % bs) * hd;      // + kv head * bs * hd
        }
        const int heads = nh + (k_pages ? nkv : 0);
        if (vec8) {
            // bfloat16, split halves, everything a multiple of eight: eight neighbouring pairs to a thread, 16 bytes
            // per load and store
            const int h8 = half >> 3;
            for (int i = part * 256 + tid; i < heads * h8; i += step) {
                const int head = i / h8, p = (i - head * h8) * 8;
                const T* src = head < nh ? q + (size_t)t * ldq + (size_t)head * hd : k + (size_t)t * ldk + (size_t)(head - nh) * hd;
                T* dst = head < nh ? q + (size_t)t * ldq + (size_t)head * hd : k_dst + (size_t)(head - nh) * bs * hd;
                const uint4 ua = *(const uint4*)(src + p), ub = *(const uint4*)(src + p + half);
                const uint32_t wa[4] = {ua.x, ua.y, ua.z, ua.w}, wb[4] = {ub.x, ub.y, ub.z, ub.w};
                uint32_t oa[4], ob[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float y0[2], y1[2];
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh) {
                        const float a = __uint_as_float(hh ? wa[e] & 0xffff0000u : wa[e] << 16);
                        const float b = __uint_as_float(hh ? wb[e] & 0xffff0000u : wb[e] << 16);
                        rotate_pair(a, b, cs[p + 2 * e + hh], sn[p + 2 * e + hh], y0[hh], y1[hh]);
                    }
                    oa[e] = pack_bf16(y0[0], y0[1]);
                    ob[e] = pack_bf16(y1[0], y1[1]);
                }
                *(uint4*)(dst + p) = make_uint4(oa[0], oa[1], oa[2], oa[3]);
                *(uint4*)(dst + p + half) = make_uint4(ob[0], ob[1], ob[2], ob[3]);
            }
        } else {
            for (int i = part * 256 + tid; i < heads * half; i += step) {
                const int head = i / half, p = i - head * half;
                const int ia = interleaved ? 2 * p : p;
                const int ib = interleaved ? 2 * p + 1 : p + half;
                const T* src = head < nh ? q + (size_t)t * ldq + (size_t)head * hd : k + (size_t)t * ldk + (size_t)(head - nh) * hd;
                T* dst = head < nh ? q + (size_t)t * ldq + (size_t)head * hd : k_dst + (size_t)(head - nh) * bs * hd;
                const float a = to_float(src[ia]), b = to_float(src[ib]);
                float y0, y1;
                rotate_pair(a, b, cs[p], sn[p], y0, y1);
                from_float(dst + ia, y0);
                from_float(dst + ib, y1);
            }
        }
        if (k_pages && rot < hd) {         // beyond the rotated dimensions
            const int rest = hd - rot;
            for (int i = part * 256 + tid; i < nkv * rest; i += step) {
                const int kh = i / rest, d = rot + i - kh * rest;
                k_dst[(size_t)kh * bs * hd + d] = k[(size_t)t * ldk + (size_t)kh * hd + d];
            }
        }
        return;
    }
    if (!v_pages) return;
    const int b = blockIdx.x - n_tokens * split;
    const int kh = b % nkv, t0 = (b / nkv) * 8;
    const int n = min(8, n_tokens - t0);
    const int pos0 = positions[t0], seq0 = token_seq[t0];
    bool together = sizeof(T) == 2 && n == 8 && (bs & 7) == 0 && (pos0 & 7) == 0;
    for (int i = 1; together && i < 8; ++i) together = positions[t0 + i] == pos0 + i && token_seq[t0 + i] == seq0;
    if (together) {
        const int page = block_table[(size_t)seq0 * max_blocks + pos0 / bs];
        T* dst = v_pages + ((size_t)page * nkv + kh) * hd * bs + pos0 % bs;
        for (int d = tid; d < hd; d += 256) {
            uint16_t e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = *(const uint16_t*)(v + (size_t)(t0 + i) * ldv + (size_t)kh * hd + d);
            uint4 o;
            o.x = e[0] | ((uint32_t)e[1] << 16);
            o.y = e[2] | ((uint32_t)e[3] << 16);
            o.z = e[4] | ((uint32_t)e[5] << 16);
            o.w = e[6] | ((uint32_t)e[7] << 16);
            *(uint4*)(dst + (size_t)d * bs) = o;
        }
        return;
    }
    for (int idx = tid; idx < n * hd; idx += 256) {      // tokens of different pages: element by element
        const int i = idx / hd, d = idx - i * hd;
        const int t = t0 + i, pos = positions[t];
        const int page = block_table[(size_t)token_seq[t] * max_blocks + pos / bs];
        v_pages[(((size_t)page * nkv + kh) * hd + d) * bs + pos % bs] = v[(size_t)t * ldv + (size_t)kh * hd + d];
    }
}

FX_API int fx_rope_kv_write(void* stream, int dtype, void* q, int ldq, const void* k, int ldk,
                            const void* v, int ldv, const int* positions, const int* token_seq,
                            const int* block_table, int max_blocks, void* k_pages, void* v_pages,
                            int T, int nh, int nkv, int hd, int bs, int rot, int interleaved, const float* inv_freq,
                            const float* freq_factors) {
    FX_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && hd > 0 && bs > 0, "rope_kv_write: bad sizes");
    FX_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "rope_kv_write: rotary dim %d must be even and <= head_dim %d", rot, hd);
    FX_REQUIRE(rot <= 256, "rope_kv_write: rotary dim %d is more than this kernel's 256", rot);
    FX_REQUIRE(inv_freq || rot == 0, "rope_kv_write: a rotation needs the table of its %d frequencies", rot / 2);
    FX_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "rope_kv_write: key and value pages must come together");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int split = T <= 32 ? 8 : (T <= 128 ? 2 : 1);
    const long n_blocks = (long)T * split + (v_pages ? (long)((T + 7) / 8) * nkv : 0);
    FX_REQUIRE(n_blocks < (1L << 31), "rope_kv_write: too many tokens and heads for one launch");
    const unsigned blocks = (unsigned)n_blocks;
    const int vec8 = dtype == FX_BF16 && !interleaved && rot % 16 == 0 && hd % 8 == 0 && ldq % 8 == 0 && ldk % 8 == 0 &&
                     ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && (!k_pages || ((uintptr_t)k_pages % 16) == 0);
    if (dtype == FX_F32)
        rope_kv_write_kernel<float><<<blocks, 256, 0, s>>>((float*)q, ldq, (const float*)k, ldk, (const float*)v, ldv,
                                                           positions, token_seq, block_table, max_blocks,
                                                           (float*)k_pages, (float*)v_pages, T, split, nh, nkv, hd, bs, rot,
                                                           interleaved, inv_freq, 0, freq_factors);
    else if (dtype == FX_BF16)
        rope_kv_write_kernel<bf16><<<blocks, 256, 0, s>>>((bf16*)q, ldq, (const bf16*)k, ldk, (const bf16*)v, ldv,
                                                          positions, token_seq, block_table, max_blocks,
                                                          (bf16*)k_pages, (bf16*)v_pages, T, split, nh, nkv, hd, bs, rot,
                                                          interleaved, inv_freq, vec8, freq_factors);
    else
        return fx_fail("rope_kv_write: unknown dtype %d", dtype);
    FX_CHECK_LAUNCH("rope_kv_write");
    return 0;
}

// ---------------------------------------------------------------------------
// h[t, :] += y[t, :]  (float32 sum), y of either type.  Used by parts that have
// no fused epilogue of their own.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ h, const T* __restrict__ y, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) h[i] += to_float(y[i]);
}

FX_API int fx_residual_add(void* stream, int y_dtype, float* h, const void* y, long n) {
    FX_REQUIRE(n >= 0, "residual_add: bad size");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    if (y_dtype == FX_F32)
        residual_add_kernel<float><<<blocks, 256, 0, s>>>(h, (const float*)y, (size_t)n);
    else if (y_dtype == FX_BF16)
        residual_add_kernel<bf16><<<blocks, 256, 0, s>>>(h, (const bf16*)y, (size_t)n);
    else
        return fx_fail("residual_add: unknown dtype %d", y_dtype);
    FX_CHECK_LAUNCH("residual_add");
    return 0;
}

// ---------------------------------------------------------------------------
// casts between float32 and bf16
// ---------------------------------------------------------------------------
template <typename A, typename B>
__global__ void cast_kernel(const A* __restrict__ a, B* __restrict__ b, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) from_float(b + i, to_float(a[i]));
}

FX_API int fx_cast(void* stream, int src_dtype, const void* src, int dst_dtype, void* dst, long n) {
    FX_REQUIRE(n >= 0, "cast: bad size");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    if (src_dtype == FX_F32 && dst_dtype == FX_BF16)
        cast_kernel<float, bf16><<<blocks, 256, 0, s>>>((const float*)src, (bf16*)dst, (size_t)n);
    else if (src_dtype == FX_BF16 && dst_dtype == FX_F32)
        cast_kernel<bf16, float><<<blocks, 256, 0, s>>>((const bf16*)src, (float*)dst, (size_t)n);
    else
        return fx_fail("cast: unsupported pair %d -> %d", src_dtype, dst_dtype);
    FX_CHECK_LAUNCH("cast");
    return 0;
}

// ---------------------------------------------------------------------------
// Weighted sum of the routed experts' outputs into the residual stream:
//   h[t, :] += sum_j w[t, j] * y[inv[t*k + j], :]      (inv null: y[t*k + j, :])
//              + gate[t] * shared[t, :]                  (if a shared expert's output is given)
// in ascending j, the selection order (ferrox-moe/src/lib.rs:735-745).
// y is float32 [T*k, H].
// ---------------------------------------------------------------------------
// xg != nullptr: the new rows are also written as xg = round(h * norm_w) (no scale yet) with each block's sum
// of squares of its 256 columns in ss[t * gridDim.y + blockIdx.y]: the product that reads xg scales its
// rows by rsqrt(sum / H + eps), which is RMSNorm with the rounding of the norm that a product applies itself.
// VEC = 4: a thread takes four neighbouring columns with 16-byte loads (H % 4 == 0, aligned rows); a block then
// covers 1024 columns, and each of its waves one group of 256 for the sums of squares.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ h, const float* __restrict__ y,
                                                          const int* __restrict__ inv, const float* __restrict__ w,
                                                          const float* __restrict__ shared, const float* __restrict__ gate,
                                                          int H, int k, int slabs, const void* __restrict__ norm_w,
                                                          int norm_dtype, T* __restrict__ xg, float* __restrict__ ss) {
    __shared__ float red[4];
    const int t = blockIdx.x, n_tok = gridDim.x;
    const int c = (blockIdx.y * 256 + threadIdx.x) * VEC;
    auto load = [&](const float* p, float (&out)[VEC]) {
        if constexpr (VEC == 4) {
            const float4 q = *(const float4*)p;
            out[0] = q.x; out[1] = q.y; out[2] = q.z; out[3] = q.w;
        } else {
            out[0] = *p;
        }
    };
    float v[VEC], nw[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = nw[i] = 0.f;
    if (c < H) {
        // the loads of eight terms are asked for together and added in order: the sums are those of a plain loop
        float h_old[VEC], acc[VEC];
        load(h + (size_t)t * H + c, h_old);
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
        for (int j0 = 0; j0 < k; j0 += 8) {
            float wv[8], yv[8][VEC];
            int from[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = min(j0 + u, k - 1);
                from[u] = inv ? inv[t * k + j] : t * k + j;
                wv[u] = w[t * k + j];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) load(y + (size_t)from[u] * H + c, yv[u]);
            if (j0 == 0 && xg) {     // (waits for its load: after the others have left)
#pragma unroll
                for (int i = 0; i < VEC; ++i) nw[i] = load_as_float(norm_w, norm_dtype, c + i);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (j0 + u < k) {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) acc[i] = fmaf(wv[u], yv[u][i], acc[i]);
                }
        }
        if (shared) {      // routed first, then shared (lib.rs:746-750); the shared output may come as `slabs` partial sums [slab][T][H]
            float sh[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) sh[i] = 0.f;
            for (int s0 = 0; s0 < slabs; s0 += 8) {
                float sv[8][VEC];
#pragma unroll
                for (int u = 0; u < 8; ++u) load(shared + ((size_t)min(s0 + u, slabs - 1) * n_tok + t) * H + c, sv[u]);
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (s0 + u < slabs) {
#pragma unroll
                        for (int i = 0; i < VEC; ++i) sh[i] += sv[u][i];
                    }
            }
            const float gt = gate ? gate[t] : 1.f;
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = fmaf(gt, sh[i], acc[i]);
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = h_old[i] + acc[i];
        if constexpr (VEC == 4) *(float4*)(h + (size_t)t * H + c) = make_float4(v[0], v[1], v[2], v[3]);
        else h[(size_t)t * H + c] = v[0];
    }
    if (!xg) return;
    if (c < H) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) from_float(xg + (size_t)t * H + c + i, v[i] * nw[i]);
    }
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) sq = fmaf(v[i], v[i], sq);
    const int n_groups = (H + 255) / 256;
    if constexpr (VEC == 4) {
        const float total = wave_sum(sq);
        const int group = blockIdx.y * 4 + (threadIdx.x >> 6);
        if ((threadIdx.x & 63) == 0 && group < n_groups) ss[t * n_groups + group] = total;
    } else {
        const float total = block_sum<4>(sq, red);
        if (threadIdx.x == 0) ss[t * n_groups + blockIdx.y] = total;
    }
}

// norm_w != nullptr: x_out = round(h * norm_w) of the new rows, in out_dtype, and ss[t][b] = the sum of squares of
// columns [256 b, 256 b + 256) of row t.
FX_API int fx_moe_combine(void* stream, float* h, const float* y, const int* inv, const float* w,
                          const float* shared, const float* gate, int T, int H, int k, int slabs,
                          const void* norm_w, int norm_dtype, void* x_out, int out_dtype, float* ss) {
    FX_REQUIRE(T >= 0 && H > 0 && k > 0 && slabs >= 1, "moe_combine: bad sizes");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    // few rows: a thread per column spreads the row's loads over more waves, which is what counts then
    const bool vec = (long)T * H >= (1L << 18) && H % 4 == 0 && ((uintptr_t)h % 16) == 0 && ((uintptr_t)y % 16) == 0 &&
                     (!shared || ((uintptr_t)shared % 16) == 0);
    const dim3 grid(T, vec ? (H + 1023) / 1024 : (H + 255) / 256);
#define FX_COMBINE(TYPE, XOUT) \
    do { \
        if (vec) moe_combine_kernel<TYPE, 4><<<grid, 256, 0, s>>>(h, y, inv, w, shared, gate, H, k, slabs, norm_w, norm_dtype, XOUT, ss); \
        else moe_combine_kernel<TYPE, 1><<<grid, 256, 0, s>>>(h, y, inv, w, shared, gate, H, k, slabs, norm_w, norm_dtype, XOUT, ss); \
    } while (0)
    if (norm_w) {
        FX_REQUIRE(x_out && ss, "moe_combine: the rows for the norm need places to write");
        FX_REQUIRE(norm_dtype == FX_F32 || norm_dtype == FX_BF16, "moe_combine: unknown norm weight dtype %d", norm_dtype);
        FX_REQUIRE(out_dtype == FX_F32 || out_dtype == FX_BF16, "moe_combine: unknown output dtype %d", out_dtype);
        if (out_dtype == FX_F32) FX_COMBINE(float, (float*)x_out);
        else FX_COMBINE(bf16, (bf16*)x_out);
    } else {
        norm_w = nullptr;
        ss = nullptr;
        FX_COMBINE(float, (float*)nullptr);
    }
#undef FX_COMBINE
    FX_CHECK_LAUNCH("moe_combine");
    return 0;
}

// ---------------------------------------------------------------------------
// fill a buffer of 32-bit words (used instead of a memset so that callers may
// record it into a HIP graph)
// ---------------------------------------------------------------------------
__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

FX_API int fx_fill_u32(void* stream, void* p, unsigned v, long n) {
    FX_REQUIRE(n >= 0, "fill: bad size");
    if (n == 0) return 0;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    fill_u32_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((uint32_t*)p, v, (size_t)n);
    FX_CHECK_LAUNCH("fill");
    return 0;
}

// ---------------------------------------------------------------------------
// token ids that are still on the device: tokens[pairs[i][0]] = ids[pairs[i][1]].
// A step whose tokens were sampled by the step before it can be launched before the
// host has read those ids; where it holds one of them, the host wrote a stand-in.
// ---------------------------------------------------------------------------
__global__ void feed_tokens_kernel(int* tokens, const int* ids, const int* pairs, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) tokens[pairs[2 * i]] = ids[pairs[2 * i + 1]];
}

FX_API int fx_feed_tokens(void* stream, int* tokens, const int* ids, const int* pairs, int n) {
    FX_REQUIRE(n >= 0 && tokens && ids && pairs, "feed_tokens: bad arguments");
    if (n == 0) return 0;
    feed_tokens_kernel<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(tokens, ids, pairs, n);
    FX_CHECK_LAUNCH("feed_tokens");
    return 0;
}
