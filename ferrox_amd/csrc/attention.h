// Entry points of the attention library (attention.hip), as C declarations.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

// Queries in blocks: item i covers item_n[i] <= tile_q consecutive tokens of one sequence.  tile_q is 64, or 128
// where fx_attn_tile_queries says so (bfloat16, head_dim 64 or 128, pages of a multiple of 64 keys).
int fx_attn_tile_queries(int dtype, int hd, int bs);
int fx_attn_tiles(void* stream, int dtype, const void* q, long ldq, void* out, long ldo, const void* k_pages,
                  const void* v_pages, const int* block_table, int max_blocks, const int* positions, const int* item_seq,
                  const int* item_tok, const int* item_n, int n_items, int nh, int nkv, int hd, int bs, int window, float scale,
                  int tile_q);

// Single queries.  The keys are cut into `splits` chunks of `chunk` positions; the chunks' partial results go through
// part_o [n_items, nh, splits, hd] and part_ml [n_items, nh, splits, 2] (float32, brought by the caller).
int fx_attn_decode(void* stream, int dtype, const void* q, long ldq, void* out, long ldo, const void* k_pages,
                   const void* v_pages, const int* block_table, int max_blocks, const int* positions, const int* item_seq,
                   const int* item_tok, int n_items, int nh, int nkv, int hd, int bs, int window, float scale,
                   float* part_o, float* part_ml, int splits, int chunk, int waves);

// The same for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The partial results live in an array
// inside the library (one copy per GPU, 16 MiB, held until the process ends), so the call takes no buffers beside
// its inputs and its output, and neither it nor anything it calls allocates or frees.  It refuses shapes whose
// partial results, n_items * nh * splits * (hd + 2) floats, exceed fx_attn_static_capacity().  All calls on one GPU
// share that GPU's array: calls that overlap on one GPU race; calls in stream order do not.
// The array used is that of the device that `stream` belongs to (null: the current device).
// fx_attn_static_init() looks the array's address up for the current device ahead of the first call; the first
// call on a device does it otherwise, except under stream capture, where the lookup is refused with an error:
// call fx_attn_static_init() with the stream's device current before a capture that holds this call.
int fx_attn_decode_static(void* stream, int dtype, const void* q, long ldq, void* out, long ldo, const void* k_pages,
                          const void* v_pages, const int* block_table, int max_blocks, const int* positions,
                          const int* item_seq, const int* item_tok, int n_items, int nh, int nkv, int hd, int bs, int window,
                          float scale, int splits, int chunk, int waves);
int fx_attn_static_init(void);
long fx_attn_static_capacity(void);

const char* fx_last_error(void);

#ifdef __cplusplus
}
#endif
