// Host-side bookkeeping of the paged cache and the layout of a step's batch, in C++.
//
// The book keeps, for every page group, a pool of page ids with a free list, and for every
// live request its state slot, its cached length and one block table per group.  A windowed
// group gives a page back as soon as no later query can see any of its positions; the table
// entry becomes -1 and is never addressed again.  Taking a page that is held or giving one back
// twice is an error, never silently accepted.
// (The reference keeps one pool and one identical table per LAYER and frees only when a
// request ends: src/llaisys/kv_cache/block_kv_cache.hpp:16-96, src/llaisys/models/qwen2.cpp:832-845,
// :1066-1070.)
//
// li_book_build_batch lays out all integers of a step in one buffer (the reference builds the
// same flat arrays, src/llaisys/models/qwen2.cpp:942-957, but its tables again for every layer,
// :993-1007).
//
// Requests are named by 64-bit handles; the caller maps its own ids to them.  Functions return
// >= 0 on success and a negative code otherwise; li_book_error() gives the text of the last
// failure of that book.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

namespace {

enum { ERR_FULL = -1, ERR_UNKNOWN = -2, ERR_POOL = -3, ERR_ARG = -4, ERR_LIVE = -5, ERR_INVARIANT = -6 };

struct Pool {
    int capacity = 0;
    std::vector<int> free_list;            // alloc() pops from the end
    std::vector<char> held;
    long total_allocations = 0;
    int peak_used = 0;                     // the most pages that were ever held at one time
    std::string error;

    bool init(int n, const int* order) {
        if (n <= 0) { error = "page pool: needs at least one page, found " + std::to_string(n); return false; }
        capacity = n;
        held.assign(n, 0);
        std::vector<char> seen(n, 0);
        free_list.resize(n);
        for (int i = 0; i < n; ++i) {
            const int id = order ? order[i] : i;
            if (id < 0 || id >= n || seen[id]) {
                error = "page pool: the free-list order must be a permutation of all page ids";
                capacity = 0;
                free_list.clear();
                return false;
            }
            seen[id] = 1;
            free_list[n - 1 - i] = id;     // the first id of `order` is taken first
        }
        return true;
    }
    int free_count() const { return (int)free_list.size(); }
    int used() const { return capacity - (int)free_list.size(); }
    int alloc() {
        if (free_list.empty()) { error = "page pool: no free page"; return ERR_FULL; }
        const int p = free_list.back();
        free_list.pop_back();
        if (held[p]) { error = "page pool: page " + std::to_string(p) + " was on the free list while held"; return ERR_POOL; }
        held[p] = 1;
        ++total_allocations;
        peak_used = std::max(peak_used, used());
        return p;
    }
    int release(int p) {
        if (p < 0 || p >= capacity) { error = "page pool: page id " + std::to_string(p) + " out of range"; return ERR_POOL; }
        if (!held[p]) { error = "page pool: page " + std::to_string(p) + " freed twice"; return ERR_POOL; }
        held[p] = 0;
        free_list.push_back(p);
        return 0;
    }
};

struct Request {
    int slot = 0;
    int cached = 0;
    std::vector<std::vector<int>> tables;      // per group: logical block -> page or -1
    std::vector<int> first_live;               // per group: first block not yet given back
};

struct Book {
    int page_size = 0, max_seqs = 0;
    std::vector<int> windows;                  // per group, 0 = all keys
    std::vector<Pool> pools;
    std::vector<int> free_slots;
    std::unordered_map<int64_t, Request> requests;
    std::string error;

    int fail(int code, const std::string& msg) { error = msg; return code; }
    Request* find(int64_t h) {
        auto it = requests.find(h);
        return it == requests.end() ? nullptr : &it->second;
    }
    int first_needed_block(int g, int first_query_pos) const {      // first block a query at that position or later sees
        if (windows[g] <= 0) return 0;
        const int lo = first_query_pos - windows[g] + 1;
        return (lo > 0 ? lo : 0) / page_size;
    }
    void pages_needed(const Request* r, int n_new, int cached, int* out) const {
        const int have_cached = cached >= 0 ? cached : (r ? r->cached : 0);
        for (size_t g = 0; g < pools.size(); ++g) {
            const int nblk = (have_cached + n_new + page_size - 1) / page_size;
            const int have = r ? (int)r->tables[g].size() : 0;
            out[g] = nblk > have ? nblk - have : 0;
        }
    }
};

inline long align4(long n) { return (n + 3) / 4 * 4; }

}  // namespace

extern "C" {

// ------------------------------------------------------------------ a pool alone
void* li_pool_create(int num_pages, const int* order) {
    Pool* p = new Pool();
    p->init(num_pages, order);              // a failed init leaves capacity 0 and the text in error
    return p;
}
void li_pool_destroy(void* p) { delete (Pool*)p; }
const char* li_pool_error(void* p) { return ((Pool*)p)->error.c_str(); }
int li_pool_capacity(void* p) { return ((Pool*)p)->capacity; }
int li_pool_free(void* p) { return ((Pool*)p)->free_count(); }
long li_pool_total_allocations(void* p) { return ((Pool*)p)->total_allocations; }
int li_pool_peak_used(void* p) { return ((Pool*)p)->peak_used; }
int li_pool_alloc(void* p) { return ((Pool*)p)->alloc(); }
int li_pool_release(void* p, int page) { return ((Pool*)p)->release(page); }
int li_pool_is_held(void* p, int page) {
    Pool* q = (Pool*)p;
    return page >= 0 && page < q->capacity ? q->held[page] : 0;
}

// ------------------------------------------------------------------ the book
// windows [ngroups]; num_pages [ngroups]: every group has a pool of its own size (a windowed group
// holds a few pages a request, whatever the context); orders null or the groups' permutations of
// their page ids one after the other (num_pages[0] ids, then num_pages[1], ...)
void* li_book_create(int page_size, int max_seqs, int ngroups, const int* windows, const int* num_pages, const int* orders) {
    Book* b = new Book();
    b->page_size = page_size;
    b->max_seqs = max_seqs;
    if (page_size <= 0) { b->error = "cache: page_size must be positive"; return b; }
    if (max_seqs <= 0 || ngroups < 0) { b->error = "cache: max_seqs must be positive"; return b; }
    b->windows.assign(windows, windows + ngroups);
    b->pools.resize(ngroups);
    size_t at = 0;
    for (int g = 0; g < ngroups; ++g) {
        if (!b->pools[g].init(num_pages[g], orders ? orders + at : nullptr)) {
            b->error = b->pools[g].error;
            return b;
        }
        at += (size_t)num_pages[g];
    }
    b->free_slots.resize(max_seqs);
    for (int i = 0; i < max_seqs; ++i) b->free_slots[i] = max_seqs - 1 - i;
    return b;
}
void li_book_destroy(void* b) { delete (Book*)b; }
const char* li_book_error(void* b) { return ((Book*)b)->error.c_str(); }
void* li_book_pool(void* b, int g) { return &((Book*)b)->pools[g]; }

int li_book_has(void* vb, int64_t h) { return ((Book*)vb)->find(h) != nullptr; }
int li_book_num_live(void* vb) { return (int)((Book*)vb)->requests.size(); }
int li_book_free_slots(void* vb) { return (int)((Book*)vb)->free_slots.size(); }
void li_book_free_pages(void* vb, int* out) {
    Book* b = (Book*)vb;
    for (size_t g = 0; g < b->pools.size(); ++g) out[g] = b->pools[g].free_count();
}

// the state slot, or ERR_LIVE / ERR_FULL
int li_book_admit(void* vb, int64_t h) {
    Book* b = (Book*)vb;
    if (b->find(h)) return b->fail(ERR_LIVE, "cache: the request is already live");
    if (b->free_slots.empty())
        return b->fail(ERR_FULL, "cache: all " + std::to_string(b->max_seqs) + " state slots are taken");
    Request r;
    r.slot = b->free_slots.back();
    b->free_slots.pop_back();
    r.tables.resize(b->pools.size());
    r.first_live.assign(b->pools.size(), 0);
    b->requests.emplace(h, std::move(r));
    return b->requests[h].slot;
}
int li_book_slot(void* vb, int64_t h) {
    Book* b = (Book*)vb;
    Request* r = b->find(h);
    return r ? r->slot : b->fail(ERR_UNKNOWN, "cache: unknown request");
}
int li_book_cached(void* vb, int64_t h) {
    Book* b = (Book*)vb;
    Request* r = b->find(h);
    return r ? r->cached : b->fail(ERR_UNKNOWN, "cache: unknown request");
}
int li_book_table_len(void* vb, int64_t h, int g) {
    Book* b = (Book*)vb;
    Request* r = b->find(h);
    return r ? (int)r->tables[g].size() : b->fail(ERR_UNKNOWN, "cache: unknown request");
}
int li_book_table(void* vb, int64_t h, int g, int* out, int cap) {
    Book* b = (Book*)vb;
    Request* r = b->find(h);
    if (!r) return b->fail(ERR_UNKNOWN, "cache: unknown request");
    const int n = (int)r->tables[g].size();
    if (n > cap) return b->fail(ERR_ARG, "cache: table buffer too short");
    std::copy(r->tables[g].begin(), r->tables[g].end(), out);
    return n;
}
// pages each group must take so that n_new more tokens fit; h < 0 or unknown: a new request;
// cached >= 0 overrides the request's cached length
int li_book_pages_needed(void* vb, int64_t h, int n_new, int cached, int* out) {
    Book* b = (Book*)vb;
    b->pages_needed(h >= 0 ? b->find(h) : nullptr, n_new, cached, out);
    return 0;
}
// all the pages that positions cached .. cached + n_new - 1 need, in every group, or none (ERR_FULL)
int li_book_reserve(void* vb, int64_t h, int n_new) {
    Book* b = (Book*)vb;
    Request* r = b->find(h);
    if (!r) return b->fail(ERR_UNKNOWN, "cache: unknown request");
    std::vector<int> need(b->pools.size());
    b->pages_needed(r, n_new, -1, need.data());
    for (size_t g = 0; g < b->pools.size(); ++g)
        if (need[g] > b->pools[g].free_count())
            return b->fail(ERR_FULL, "cache: the request needs " + std::to_string(need[g]) + " more pages, " +
                                         std::to_string(b->pools[g].free_count()) + " of " +
                                         std::to_string(b->pools[g].capacity) + " are free");
    for (size_t g = 0; g < b->pools.size(); ++g)
        for (int i = 0; i < need[g]; ++i) {
            const int p = b->pools[g].alloc();
            if (p < 0) return b->fail(p, b->pools[g].error);
            r->tables[g].push_back(p);
        }
    return 0;
}
// The same for a whole batch in one call (a step's entries): pages each of the n requests must take
// for its n_new[i] more tokens, out [n * ngroups]; a handle < 0 counts as a new request.
int li_book_pages_needed_many(void* vb, int n, const int64_t* handles, const int* n_new, int* out) {
    Book* b = (Book*)vb;
    const size_t G = b->pools.size();
    for (int i = 0; i < n; ++i)
        b->pages_needed(handles[i] >= 0 ? b->find(handles[i]) : nullptr, n_new[i], -1, out + (size_t)i * G);
    return 0;
}
// All the pages that the batch needs, in every group, or none at all (ERR_FULL, nothing changed).
int li_book_reserve_many(void* vb, int n, const int64_t* handles, const int* n_new) {
    Book* b = (Book*)vb;
    const size_t G = b->pools.size();
    std::vector<int> need((size_t)n * G), total(G, 0);
    for (int i = 0; i < n; ++i) {
        Request* r = b->find(handles[i]);
        if (!r) return b->fail(ERR_UNKNOWN, "cache: unknown request");
        b->pages_needed(r, n_new[i], -1, need.data() + (size_t)i * G);
        for (size_t g = 0; g < G; ++g) total[g] += need[(size_t)i * G + g];
    }
    for (size_t g = 0; g < G; ++g)
        if (total[g] > b->pools[g].free_count())
            return b->fail(ERR_FULL, "step: the batch needs " + std::to_string(total[g]) + " more pages, " +
                                         std::to_string(b->pools[g].free_count()) + " of " +
                                         std::to_string(b->pools[g].capacity) + " are free");
    for (int i = 0; i < n; ++i) {
        Request* r = b->find(handles[i]);
        for (size_t g = 0; g < G; ++g)
            for (int k = 0; k < need[(size_t)i * G + g]; ++k) {
                const int p = b->pools[g].alloc();
                if (p < 0) return b->fail(p, b->pools[g].error);
                r->tables[g].push_back(p);
            }
    }
    return 0;
}
// The longest block table of the batch in every group, out [ngroups].
int li_book_max_table_len(void* vb, int n, const int64_t* handles, int* out) {
    Book* b = (Book*)vb;
    const size_t G = b->pools.size();
    for (size_t g = 0; g < G; ++g) out[g] = 0;
    for (int i = 0; i < n; ++i) {
        Request* r = b->find(handles[i]);
        if (!r) return b->fail(ERR_UNKNOWN, "cache: unknown request");
        for (size_t g = 0; g < G; ++g) out[g] = std::max(out[g], (int)r->tables[g].size());
    }
    return 0;
}
// Cached lengths of the batch's requests, out [n] (-1 for a request that is not live).
int li_book_cached_many(void* vb, int n, const int64_t* handles, int* out) {
    Book* b = (Book*)vb;
    for (int i = 0; i < n; ++i) {
        Request* r = handles[i] >= 0 ? b->find(handles[i]) : nullptr;
        out[i] = r ? r->cached : -1;
    }
    return 0;
}
int li_book_commit(void* vb, int64_t h, int n_new);
int li_book_commit_many(void* vb, int n, const int64_t* handles, const int* n_new) {
    for (int i = 0; i < n; ++i) {
        const int rc = li_book_commit(vb, handles[i], n_new[i]);
        if (rc < 0) return rc;
    }
    return 0;
}
// n_new tokens were written: advance, and give back the pages the window has passed
int li_book_commit(void* vb, int64_t h, int n_new) {
    Book* b = (Book*)vb;
    Request* r = b->find(h);
    if (!r) return b->fail(ERR_UNKNOWN, "cache: unknown request");
    r->cached += n_new;
    for (size_t g = 0; g < b->pools.size(); ++g) {
        if (b->windows[g] <= 0) continue;
        const int keep_from = std::min(b->first_needed_block((int)g, r->cached), (int)r->tables[g].size());
        for (int blk = r->first_live[g]; blk < keep_from; ++blk)
            if (r->tables[g][blk] >= 0) {
                const int rc = b->pools[g].release(r->tables[g][blk]);
                if (rc < 0) return b->fail(rc, b->pools[g].error);
                r->tables[g][blk] = -1;
            }
        r->first_live[g] = std::max(r->first_live[g], keep_from);
    }
    return 0;
}
// the last n tokens are forgotten (their places will be written again); the pages stay with the
// request.  Refused where a windowed group has already given back a page that a query at the new
// position would see.
int li_book_rewind(void* vb, int64_t h, int n) {
    Book* b = (Book*)vb;
    Request* r = b->find(h);
    if (!r) return b->fail(ERR_UNKNOWN, "cache: unknown request");
    if (n < 0 || n > r->cached) return b->fail(ERR_ARG, "cache: cannot forget " + std::to_string(n) + " of " +
                                                            std::to_string(r->cached) + " cached tokens");
    for (size_t g = 0; g < b->pools.size(); ++g)
        if (b->first_needed_block((int)g, r->cached - n) < r->first_live[g])
            return b->fail(ERR_ARG, "cache: a windowed group has given back pages that the earlier position still sees");
    r->cached -= n;
    return 0;
}
int li_book_release(void* vb, int64_t h) {
    Book* b = (Book*)vb;
    auto it = b->requests.find(h);
    if (it == b->requests.end()) return b->fail(ERR_UNKNOWN, "cache: unknown request");
    for (size_t g = 0; g < b->pools.size(); ++g)
        for (int p : it->second.tables[g])
            if (p >= 0) {
                const int rc = b->pools[g].release(p);
                if (rc < 0) return b->fail(rc, b->pools[g].error);
            }
    b->free_slots.push_back(it->second.slot);
    b->requests.erase(it);
    return 0;
}
// no page lost, held twice or on the free list while in a table; no slot lost or held twice
int li_book_check(void* vb) {
    Book* b = (Book*)vb;
    for (size_t g = 0; g < b->pools.size(); ++g) {
        std::vector<char> seen(b->pools[g].capacity, 0);
        int count = 0;
        for (auto& kv : b->requests)
            for (int p : kv.second.tables[g]) {
                if (p < 0) continue;
                if (p >= b->pools[g].capacity || seen[p])
                    return b->fail(ERR_INVARIANT, "page " + std::to_string(p) + " of group " + std::to_string(g) + " is held twice");
                if (!b->pools[g].held[p])
                    return b->fail(ERR_INVARIANT, "page " + std::to_string(p) + " of group " + std::to_string(g) + " is in a table but free");
                seen[p] = 1;
                ++count;
            }
        if (count != b->pools[g].used())
            return b->fail(ERR_INVARIANT, "group " + std::to_string(g) + ": " + std::to_string(b->pools[g].used()) +
                                              " pages taken, " + std::to_string(count) + " in tables");
    }
    std::vector<char> slot_seen(b->max_seqs, 0);
    for (auto& kv : b->requests) {
        const int s = kv.second.slot;
        if (s < 0 || s >= b->max_seqs || slot_seen[s]) return b->fail(ERR_INVARIANT, "state slots are held twice");
        slot_seen[s] = 1;
    }
    for (int s : b->free_slots) {
        if (s < 0 || s >= b->max_seqs || slot_seen[s]) return b->fail(ERR_INVARIANT, "state slots are free while held");
        slot_seen[s] = 1;
    }
    if ((int)(b->requests.size() + b->free_slots.size()) != b->max_seqs) return b->fail(ERR_INVARIANT, "state slots lost");
    return 0;
}

// ------------------------------------------------------------------ the batch of a step
// Lays the step's integers out in `out` (int32 words, every array starting at a multiple of 4):
//   ids[T] pos[T] seg_of_token[T] q_start[nseg] q_len[nseg] ctx_len[nseg] slots[nseg]
//   want_rows[nwant] single[T] multi[T] tiles[ntiles * 4] id_src[T]
//   then per group: block_table[nseg * width_g] slot_map[T]
// (single and multi have room for T entries; their counts are in info.)  Pages for the entries'
// tokens must have been reserved.  want_rows come as places relative to the entry: want_off[i] ..
// want_off[i + 1] index `want`.  pad_blocks (null or [ngroups]) widens the tables.
// offsets [12 + 2 * ngroups] receives where each array starts; info receives
//   {T, nwant, num_single, num_multi, num_tiles, max_q_len, max_ctx_len, max_single_ctx, widths...}.
// tile_rows > 0: the tiles array is laid out, with tiles of that many tokens (0: none; the model's
// parts say whether their kernels want it).  token_kinds != 0: the single and multi lists are.
// With out == null nothing is written but offsets, info and the return value (the words needed).
long li_book_build_batch(void* vb, int nseg, const int64_t* handles, const int* q_len, const int* ids, const int* id_src,
                         const int* want_off, const int* want, const int* pad_blocks, int tile_rows, int token_kinds,
                         int32_t* out, long out_cap, long* offsets, int* info) {
    Book* b = (Book*)vb;
    const int G = (int)b->pools.size(), P = b->page_size;
    if (nseg <= 0 || tile_rows < 0) return b->fail(ERR_ARG, "step: empty batch");
    std::vector<Request*> reqs(nseg);
    long T = 0;
    int ntiles = 0, max_q = 0, max_ctx = 0, max_single_ctx = 0, nsingle = 0;
    for (int i = 0; i < nseg; ++i) {
        reqs[i] = b->find(handles[i]);
        if (!reqs[i]) return b->fail(ERR_UNKNOWN, "step: a request of the batch is not live");
        if (q_len[i] <= 0) return b->fail(ERR_ARG, "step: a request brings no tokens");
        T += q_len[i];
        const int ctx = reqs[i]->cached + q_len[i];
        max_q = std::max(max_q, q_len[i]);
        max_ctx = std::max(max_ctx, ctx);
        if (q_len[i] == 1) { ++nsingle; max_single_ctx = std::max(max_single_ctx, ctx); }
        else if (tile_rows > 0) ntiles += (q_len[i] + tile_rows - 1) / tile_rows;
    }
    const int nwant = want_off[nseg];
    std::vector<int> widths(G);
    for (int g = 0; g < G; ++g) {
        int w = 1;
        for (int i = 0; i < nseg; ++i) w = std::max(w, (int)reqs[i]->tables[g].size());
        if (pad_blocks) w = std::max(w, pad_blocks[g]);
        widths[g] = w;
    }
    long o = 0;
    const long kinds = token_kinds ? T : 0;
    const long sizes[12] = {T, T, T, nseg, nseg, nseg, nseg, nwant, kinds, kinds, (long)ntiles * 4, T};
    for (int k = 0; k < 12; ++k) { offsets[k] = o; o += align4(sizes[k]); }
    for (int g = 0; g < G; ++g) {
        offsets[12 + 2 * g] = o; o += align4((long)nseg * widths[g]);
        offsets[13 + 2 * g] = o; o += align4(T);
    }
    info[0] = (int)T; info[1] = nwant; info[2] = nsingle; info[3] = (int)T - nsingle; info[4] = ntiles;
    info[5] = max_q; info[6] = max_ctx; info[7] = max_single_ctx;
    for (int g = 0; g < G; ++g) info[8 + g] = widths[g];
    if (!out) return std::max(o, 4L);
    if (o > out_cap) return b->fail(ERR_ARG, "step: the batch buffer is too short");
    int32_t* d_ids = out + offsets[0];
    int32_t* d_pos = out + offsets[1];
    int32_t* d_seg = out + offsets[2];
    int32_t* d_qs = out + offsets[3];
    int32_t* d_ql = out + offsets[4];
    int32_t* d_cl = out + offsets[5];
    int32_t* d_slot = out + offsets[6];
    int32_t* d_want = out + offsets[7];
    int32_t* d_single = out + offsets[8];
    int32_t* d_multi = out + offsets[9];
    int32_t* d_tiles = out + offsets[10];
    int32_t* d_src = out + offsets[11];
    std::memcpy(d_ids, ids, sizeof(int32_t) * T);
    if (id_src) std::memcpy(d_src, id_src, sizeof(int32_t) * T);
    else std::fill(d_src, d_src + T, -1);
    int t = 0, ns = 0, nm = 0, nt = 0, nw = 0;
    for (int i = 0; i < nseg; ++i) {
        const Request* r = reqs[i];
        d_qs[i] = t; d_ql[i] = q_len[i]; d_cl[i] = r->cached + q_len[i]; d_slot[i] = r->slot;
        for (int w = want_off[i]; w < want_off[i + 1]; ++w) {
            if (want[w] < 0 || want[w] >= q_len[i]) return b->fail(ERR_ARG, "step: a wanted place is outside the entry's tokens");
            d_want[nw++] = t + want[w];
        }
        if (q_len[i] > 1 && tile_rows > 0)
            for (int a = 0; a < q_len[i]; a += tile_rows) {
                d_tiles[4 * nt] = i; d_tiles[4 * nt + 1] = t + a;
                d_tiles[4 * nt + 2] = std::min(tile_rows, q_len[i] - a); d_tiles[4 * nt + 3] = 0;
                ++nt;
            }
        for (int j = 0; j < q_len[i]; ++j, ++t) {
            d_pos[t] = r->cached + j;
            d_seg[t] = i;
            if (q_len[i] == 1) { if (token_kinds) d_single[ns] = t; ++ns; }
            else { if (token_kinds) d_multi[nm] = t; ++nm; }
        }
    }
    info[2] = ns; info[3] = nm;
    for (int g = 0; g < G; ++g) {
        int32_t* tab = out + offsets[12 + 2 * g];
        int32_t* smap = out + offsets[13 + 2 * g];
        const int w = widths[g];
        std::fill(tab, tab + (long)nseg * w, -1);
        int tt = 0;
        for (int i = 0; i < nseg; ++i) {
            const std::vector<int>& src = reqs[i]->tables[g];
            std::copy(src.begin(), src.end(), tab + (long)i * w);
            for (int j = 0; j < q_len[i]; ++j, ++tt) {
                const int pos = reqs[i]->cached + j, blk = pos / P;
                const int page = blk < (int)src.size() ? src[blk] : -1;
                if (page < 0) return b->fail(ERR_INVARIANT, "step: a token of the batch has no page");
                smap[tt] = page * P + pos % P;
            }
        }
    }
    return o;
}

}  // extern "C"
