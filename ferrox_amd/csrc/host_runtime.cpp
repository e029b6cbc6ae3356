// Host side of the cache: pages, block tables, state slots, and the packing of a
// step's batch into the one int32 buffer that is uploaded.  No GPU code here; the
// ids handed out index device slabs that the Python side owns.
//
// Layers with the same need share a group: one pool of page ids and one block
// table per request.  A group keeps all keys (window < 0) or the last `window`.
// The reference keeps an identical store per layer and never evicts
// (ferrox-core/src/cache.rs:331-488); here a windowed group gives a page back as
// soon as every later query is past it.  Rules: a page is in exactly one place
// (free list or one table); extend() gets every page it needs in every group or
// changes nothing (cache.rs:676-739); release() may be called twice
// (cache.rs:131-139); freed pages are handed out again first (LIFO).
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <unordered_map>
#include <vector>

#define FX_API extern "C" __attribute__((visibility("default")))

namespace {

struct Pool {
    int num_pages = 0;
    std::vector<int> free_list;      // back() is handed out next
    std::vector<char> is_free;
    explicit Pool(int n) : num_pages(n), is_free(n, 1) {
        free_list.reserve(n);
        for (int p = n - 1; p >= 0; --p) free_list.push_back(p);   // 0, 1, 2, ... at first
    }
    bool take(int n, std::vector<int>& out) {
        if (n > (int)free_list.size()) return false;
        for (int i = 0; i < n; ++i) {
            const int p = free_list.back();
            free_list.pop_back();
            is_free[p] = 0;
            out.push_back(p);
        }
        return true;
    }
    bool give(int p) {
        if (p < 0 || p >= num_pages || is_free[p]) return false;
        is_free[p] = 1;
        free_list.push_back(p);
        return true;
    }
};

struct Seq {
    int slot = -1;
    int length = 0;
    std::vector<std::vector<int>> tables;   // per group: page ids, -1 where a window has passed
};

struct Manager {
    int block_size;
    std::vector<int> windows;               // per group, < 0: all keys
    std::vector<Pool> pools;
    int n_slots;
    std::vector<int> free_slots;
    std::vector<char> slot_used;
    std::unordered_map<int64_t, Seq> seqs;
    std::string error;

    int blocks_for(int len) const { return (len + block_size - 1) / block_size; }
    Seq* find(int64_t req) {
        auto it = seqs.find(req);
        return it == seqs.end() ? nullptr : &it->second;
    }
};

int fail(Manager* m, const char* fmt, long a = 0, long b = 0) {
    char buf[256];
    snprintf(buf, sizeof(buf), fmt, a, b);
    m->error = buf;
    return -2;
}

}  // namespace

FX_API void* fxc_create(int n_groups, const int* windows, const int* num_pages, int block_size, int n_slots) {
    if (n_groups < 0 || block_size < 1 || n_slots < 0) return nullptr;
    Manager* m = new Manager();
    m->block_size = block_size;
    for (int g = 0; g < n_groups; ++g) {
        if (num_pages[g] < 0) {
            delete m;
            return nullptr;
        }
        m->windows.push_back(windows[g]);
        m->pools.emplace_back(num_pages[g]);
    }
    m->n_slots = n_slots;
    m->slot_used.assign(n_slots, 0);
    for (int s = n_slots - 1; s >= 0; --s) m->free_slots.push_back(s);
    return m;
}

FX_API void fxc_destroy(void* h) { delete (Manager*)h; }
FX_API const char* fxc_last_error(void* h) { return ((Manager*)h)->error.c_str(); }

// a state slot and empty block tables; -1 if no slot is free, -2 if already admitted
FX_API int fxc_admit(void* h, int64_t req) {
    Manager* m = (Manager*)h;
    if (m->find(req)) return fail(m, "request %ld is already admitted", (long)req);
    if (m->free_slots.empty()) return -1;
    Seq s;
    s.slot = m->free_slots.back();
    m->free_slots.pop_back();
    m->slot_used[s.slot] = 1;
    s.tables.resize(m->pools.size());
    m->seqs.emplace(req, std::move(s));
    return m->seqs[req].slot;
}

FX_API int fxc_contains(void* h, int64_t req) { return ((Manager*)h)->find(req) != nullptr; }

FX_API int fxc_length(void* h, int64_t req) {
    Manager* m = (Manager*)h;
    Seq* s = m->find(req);
    return s ? s->length : fail(m, "request %ld is not admitted", (long)req);
}

FX_API int fxc_slot(void* h, int64_t req) {
    Manager* m = (Manager*)h;
    Seq* s = m->find(req);
    return s ? s->slot : fail(m, "request %ld is not admitted", (long)req);
}

// pages group g would take for extend(req, new_len); -2 on error
FX_API int fxc_pages_needed(void* h, int64_t req, int new_len, int g) {
    Manager* m = (Manager*)h;
    Seq* s = m->find(req);
    if (!s) return fail(m, "request %ld is not admitted", (long)req);
    const int need = m->blocks_for(new_len) - (int)s->tables[g].size();
    return need > 0 ? need : 0;
}

// pages for positions [length, new_len) in every group, all or nothing: 1 done, 0 not enough pages
FX_API int fxc_extend(void* h, int64_t req, int new_len, int dry_run) {
    Manager* m = (Manager*)h;
    Seq* s = m->find(req);
    if (!s) return fail(m, "request %ld is not admitted", (long)req);
    if (new_len < s->length) return fail(m, "a sequence cannot shrink (request %ld to %ld)", (long)req, new_len);
    const int blocks = m->blocks_for(new_len);
    for (size_t g = 0; g < m->pools.size(); ++g) {
        const int need = blocks - (int)s->tables[g].size();
        if (need > (int)m->pools[g].free_list.size()) return 0;
    }
    if (dry_run) return 1;
    for (size_t g = 0; g < m->pools.size(); ++g) {
        const int need = blocks - (int)s->tables[g].size();
        if (need > 0) m->pools[g].take(need, s->tables[g]);
    }
    s->length = new_len;
    return 1;
}

// Give back pages that a window has passed: every query from now on stands at a position
// >= length and sees keys t with position - t < W, so t >= length - W + 1.  Returns pages freed.
FX_API int fxc_trim(void* h, int64_t req) {
    Manager* m = (Manager*)h;
    Seq* s = m->find(req);
    if (!s) return fail(m, "request %ld is not admitted", (long)req);
    int freed = 0;
    for (size_t g = 0; g < m->pools.size(); ++g) {
        if (m->windows[g] < 0) continue;
        const int first_needed = s->length - m->windows[g] + 1;
        if (first_needed <= 0) continue;
        std::vector<int>& t = s->tables[g];
        const int upto = std::min<int>(first_needed / m->block_size, (int)t.size());
        for (int b = 0; b < upto; ++b)
            if (t[b] >= 0) {
                m->pools[g].give(t[b]);
                t[b] = -1;
                ++freed;
            }
    }
    return freed;
}

// everything the request holds goes back; a second call does nothing
FX_API void fxc_release(void* h, int64_t req) {
    Manager* m = (Manager*)h;
    auto it = m->seqs.find(req);
    if (it == m->seqs.end()) return;
    Seq& s = it->second;
    for (size_t g = 0; g < m->pools.size(); ++g)
        for (int p : s.tables[g])
            if (p >= 0) m->pools[g].give(p);
    m->slot_used[s.slot] = 0;
    m->free_slots.push_back(s.slot);
    m->seqs.erase(it);
}

FX_API int fxc_n_free_pages(void* h, int g) { return (int)((Manager*)h)->pools[g].free_list.size(); }
FX_API int fxc_num_pages(void* h, int g) { return ((Manager*)h)->pools[g].num_pages; }
FX_API int fxc_n_free_slots(void* h) { return (int)((Manager*)h)->free_slots.size(); }
FX_API int fxc_n_requests(void* h) { return (int)((Manager*)h)->seqs.size(); }

// a pool or the slots alone, without requests
FX_API int fxc_pool_take(void* h, int g, int n, int* out) {
    std::vector<int> got;
    if (n < 0 || !((Manager*)h)->pools[g].take(n, got)) return 0;
    for (int i = 0; i < n; ++i) out[i] = got[i];
    return 1;
}
FX_API int fxc_pool_give(void* h, int g, int page) { return ((Manager*)h)->pools[g].give(page) ? 1 : 0; }
FX_API int fxc_slot_take(void* h) {
    Manager* m = (Manager*)h;
    if (m->free_slots.empty()) return -1;
    const int s = m->free_slots.back();
    m->free_slots.pop_back();
    m->slot_used[s] = 1;
    return s;
}
FX_API int fxc_slot_give(void* h, int s) {
    Manager* m = (Manager*)h;
    if (s < 0 || s >= m->n_slots || !m->slot_used[s]) return 0;
    m->slot_used[s] = 0;
    m->free_slots.push_back(s);
    return 1;
}

// the block table of a request in group g: writes up to `cap` ids, returns the number of blocks
FX_API int fxc_table(void* h, int64_t req, int g, int* out, int cap) {
    Manager* m = (Manager*)h;
    Seq* s = m->find(req);
    if (!s) return fail(m, "request %ld is not admitted", (long)req);
    const std::vector<int>& t = s->tables[g];
    for (int i = 0; i < (int)t.size() && i < cap; ++i) out[i] = t[i];
    return (int)t.size();
}

// 0 if every rule holds, else -2 with a message
FX_API int fxc_check(void* h) {
    Manager* m = (Manager*)h;
    for (size_t g = 0; g < m->pools.size(); ++g) {
        Pool& p = m->pools[g];
        std::vector<int> seen(p.num_pages, 0);
        for (int q : p.free_list) {
            if (q < 0 || q >= p.num_pages || !p.is_free[q]) return fail(m, "group %ld: bad entry %ld in the free list", g, q);
            if (seen[q]++) return fail(m, "group %ld: page %ld is in the free list twice", g, q);
        }
        size_t held = 0;
        for (auto& kv : m->seqs) {
            const Seq& s = kv.second;
            if ((int)s.tables[g].size() < m->blocks_for(s.length)) return fail(m, "group %ld: request %ld has too few blocks", g, (long)kv.first);
            for (int q : s.tables[g]) {
                if (q < 0) continue;
                if (q >= p.num_pages) return fail(m, "group %ld: page %ld out of range", g, q);
                if (seen[q]++) return fail(m, "group %ld: page %ld is held twice or both free and held", g, q);
                ++held;
            }
        }
        if (held + p.free_list.size() != (size_t)p.num_pages) return fail(m, "group %ld: %ld pages lost", g, (long)(p.num_pages - held - p.free_list.size()));
    }
    std::vector<int> slot_seen(m->n_slots, 0);
    for (auto& kv : m->seqs) {
        const int s = kv.second.slot;
        if (s < 0 || s >= m->n_slots || slot_seen[s]++) return fail(m, "state slot %ld is held twice", s);
    }
    if (m->seqs.size() + m->free_slots.size() != (size_t)m->n_slots) return fail(m, "state slots lost");
    return 0;
}

// Packs one step.  Entry e brings n_tok[e] tokens (concatenated in `tokens`) of request reqs[e],
// whose pages are reserved already (length = start + n_tok), and wants the places
// want[want_start[e] .. want_start[e+1]) among them.  Writes into `out` (int32):
//   tokens[T] | positions[T] | token_seq[T] | slots[n] | rows[R] | tables[groups][n][max_blocks]
// with freed table entries as 0 (they are never read).  `sizes` receives T, R, max_blocks, and per
// entry start position and length after the step go to `starts` / `lens`.  Returns the number of
// int32 written, or -2 with a message (vocab < 0: ids are not checked).  force_blocks > 0 sets the
// width of the tables (a recorded step has a fixed one) and must cover the longest sequence.
FX_API long fxc_pack_step(void* h, int n, const int64_t* reqs, const int* n_tok, const int* tokens,
                          const int* want_start, const int* want, int vocab, int force_blocks, int* out, long cap,
                          int* sizes, int* starts, int* lens) {
    Manager* m = (Manager*)h;
    long T = 0, R = want_start[n];
    int max_blocks = 1;
    for (int e = 0; e < n; ++e) {
        Seq* s = m->find(reqs[e]);
        if (!s) return fail(m, "request %ld was not admitted", (long)reqs[e]);
        if (n_tok[e] <= 0) return fail(m, "request %ld brings no tokens to this step", (long)reqs[e]);
        if (s->length < n_tok[e]) return fail(m, "request %ld: more tokens than reserved positions (%ld)", (long)reqs[e], s->length);
        for (int f = 0; f < e; ++f)
            if (reqs[f] == reqs[e]) return fail(m, "request %ld appears twice in one step", (long)reqs[e]);
        starts[e] = s->length - n_tok[e];
        lens[e] = s->length;
        T += n_tok[e];
        max_blocks = std::max(max_blocks, m->blocks_for(s->length));
    }
    if (force_blocks > 0) {
        if (force_blocks < max_blocks) return fail(m, "tables of %ld blocks cannot hold %ld", force_blocks, max_blocks);
        max_blocks = force_blocks;
    }
    const long G = (long)m->pools.size();
    const long total = 3 * T + n + R + G * n * max_blocks;
    if (total > cap) return fail(m, "step buffer of %ld words is too small for %ld", cap, total);
    int* o_tok = out;
    int* o_pos = out + T;
    int* o_seq = out + 2 * T;
    int* o_slot = out + 3 * T;
    int* o_rows = o_slot + n;
    int* o_tab = o_rows + R;
    long t = 0;
    for (int e = 0; e < n; ++e) {
        Seq* s = m->find(reqs[e]);
        o_slot[e] = s->slot;
        for (int w = want_start[e]; w < want_start[e + 1]; ++w) {
            if (want[w] < 0 || want[w] >= n_tok[e]) return fail(m, "request %ld: wanted place %ld is outside its tokens", (long)reqs[e], want[w]);
            o_rows[w] = (int)(t + want[w]);
        }
        for (int i = 0; i < n_tok[e]; ++i, ++t) {
            const int id = tokens[t];
            if (vocab >= 0 && (id < 0 || id >= vocab)) return fail(m, "token id %ld is outside the vocabulary of %ld", id, vocab);
            o_tok[t] = id;
            o_pos[t] = starts[e] + i;
            o_seq[t] = e;
        }
        for (long g = 0; g < G; ++g) {
            int* row = o_tab + (g * n + e) * max_blocks;
            const std::vector<int>& tab = s->tables[g];
            for (int b = 0; b < max_blocks; ++b) row[b] = (b < (int)tab.size() && tab[b] >= 0) ? tab[b] : 0;
        }
    }
    sizes[0] = (int)T;
    sizes[1] = (int)R;
    sizes[2] = max_blocks;
    return total;
}

// A step in which each of n requests brings one token and wants its logits, laid out for pad_to >= n sequences
// (a recorded step has a fixed number of them):
//   tokens[N] | positions[N] | token_seq[N] | slots[N] | rows[N] | tables[groups][N][max_blocks],  N = pad_to.
// Rows n .. N-1 are stand-ins that no request owns: token 0 at position 0 of a sequence of its own, whose one
// block in group g is pad_pages[g] (a page beyond the pool, which the device slabs hold for this purpose) and
// whose state slot is pad_slot; what they compute is never looked at.  `lens` receives the n lengths after the
// step.  Returns the number of int32 written, or -2 with a message.
FX_API long fxc_pack_decode(void* h, int n, const int64_t* reqs, const int* tokens, int vocab, int force_blocks,
                            int pad_to, const int* pad_pages, int pad_slot, int* out, long cap, int* lens) {
    Manager* m = (Manager*)h;
    if (pad_to < n) return fail(m, "a step of %ld sequences cannot be laid out for %ld", n, pad_to);
    int max_blocks = 1;
    for (int e = 0; e < n; ++e) {
        Seq* s = m->find(reqs[e]);
        if (!s) return fail(m, "request %ld was not admitted", (long)reqs[e]);
        if (s->length < 1) return fail(m, "request %ld: more tokens than reserved positions (%ld)", (long)reqs[e], s->length);
        for (int f = 0; f < e; ++f)
            if (reqs[f] == reqs[e]) return fail(m, "request %ld appears twice in one step", (long)reqs[e]);
        const int id = tokens[e];
        if (vocab >= 0 && (id < 0 || id >= vocab)) return fail(m, "token id %ld is outside the vocabulary of %ld", id, vocab);
        lens[e] = s->length;
        max_blocks = std::max(max_blocks, m->blocks_for(s->length));
    }
    if (force_blocks > 0) {
        if (force_blocks < max_blocks) return fail(m, "tables of %ld blocks cannot hold %ld", force_blocks, max_blocks);
        max_blocks = force_blocks;
    }
    const long N = pad_to, G = (long)m->pools.size();
    const long total = 5 * N + G * N * max_blocks;
    if (total > cap) return fail(m, "step buffer of %ld words is too small for %ld", cap, total);
    int* o_tok = out;
    int* o_pos = out + N;
    int* o_seq = out + 2 * N;
    int* o_slot = out + 3 * N;
    int* o_rows = out + 4 * N;
    int* o_tab = out + 5 * N;
    for (long e = 0; e < N; ++e) {
        Seq* s = e < n ? m->find(reqs[e]) : nullptr;
        o_tok[e] = s ? tokens[e] : 0;
        o_pos[e] = s ? s->length - 1 : 0;
        o_seq[e] = (int)e;
        o_slot[e] = s ? s->slot : pad_slot;
        o_rows[e] = (int)e;
        for (long g = 0; g < G; ++g) {
            int* row = o_tab + (g * N + e) * max_blocks;
            for (int b = 0; b < max_blocks; ++b) {
                if (s) {
                    const std::vector<int>& tab = s->tables[g];
                    row[b] = (b < (int)tab.size() && tab[b] >= 0) ? tab[b] : 0;
                } else {
                    row[b] = pad_pages[g];
                }
            }
        }
    }
    return total;
}
