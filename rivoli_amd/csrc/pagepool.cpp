// Host-side page allocator for the paged fp8 KV cache. Contract and the reference pattern it
// follows (crates/core/src/arena.rs:132-149) are in include/rivoli_pagepool.h.
#include "rivoli_pagepool.h"

#include <cstddef>
#include <new>
#include <vector>

// No C++ exception may cross the C boundary: an allocation failure inside an entry point is
// reported as kOutOfHostMemory, and every entry point reserves what it will need BEFORE it changes
// the pool, so a failed call leaves the pool exactly as it found it.
static constexpr int kOutOfHostMemory = -1006;

struct rivoli_pagepool {
    int n_pages = 0;
    int page_tokens = 0;
    int frontier = 0;            // pages [0, frontier) have been handed out at least once
    std::vector<int> free_list;  // LIFO: back() is the most recently freed page
    struct Seq {
        bool live = false;
        int len = 0;
        std::vector<int> pages;
    };
    std::vector<Seq> seqs;
    std::vector<int> free_ids;
    int owned = 0;

    int available() const { return (int)free_list.size() + (n_pages - frontier); }
    int take_page() {
        if (!free_list.empty()) {
            int p = free_list.back();
            free_list.pop_back();
            return p;
        }
        return frontier++;
    }
    Seq* get(int id) {
        if (id < 0 || id >= (int)seqs.size() || !seqs[id].live) return nullptr;
        return &seqs[id];
    }
    const Seq* get(int id) const { return const_cast<rivoli_pagepool*>(this)->get(id); }
};

extern "C" rivoli_pagepool* rivoli_pagepool_create(int n_pages, int page_tokens) {
    if (n_pages <= 0 || page_tokens <= 0) return nullptr;
    if ((long long)n_pages * page_tokens > 0x7fffffffLL) return nullptr;  // slots must fit int
    auto* p = new (std::nothrow) rivoli_pagepool();
    if (!p) return nullptr;
    p->n_pages = n_pages;
    p->page_tokens = page_tokens;
    try {
        p->free_list.reserve((std::size_t)n_pages);  // freeing pages can then never allocate
    } catch (...) {
        delete p;
        return nullptr;
    }
    return p;
}

extern "C" void rivoli_pagepool_destroy(rivoli_pagepool* pool) { delete pool; }

extern "C" int rivoli_pagepool_seq_create(rivoli_pagepool* pool) {
    if (!pool) return -1001;
    int id;
    if (!pool->free_ids.empty()) {
        id = pool->free_ids.back();
        pool->free_ids.pop_back();
    } else {
        id = (int)pool->seqs.size();
        try {
            // room for this id on the list of freed ids too, so seq_free cannot fail
            pool->free_ids.reserve(pool->seqs.size() + 1);
            pool->seqs.emplace_back();
        } catch (...) {
            return kOutOfHostMemory;
        }
    }
    pool->seqs[id].live = true;
    pool->seqs[id].len = 0;
    pool->seqs[id].pages.clear();
    return id;
}

extern "C" int rivoli_pagepool_seq_free(rivoli_pagepool* pool, int seq) {
    if (!pool) return -1001;
    auto* s = pool->get(seq);
    if (!s) return -1001;
    int n = (int)s->pages.size();
    for (int p : s->pages) pool->free_list.push_back(p);
    pool->owned -= n;
    s->pages.clear();
    s->len = 0;
    s->live = false;
    pool->free_ids.push_back(seq);
    return n;
}

extern "C" int rivoli_pagepool_seq_extend(rivoli_pagepool* pool, int seq, int n_tokens,
                                          int* slots_out) {
    if (!pool || n_tokens < 0) return -1001;
    auto* s = pool->get(seq);
    if (!s) return -1001;
    const int pt = pool->page_tokens;
    const long long new_len = (long long)s->len + n_tokens;
    const long long blocks_needed = (new_len + pt - 1) / pt;
    const long long extra = blocks_needed - (long long)s->pages.size();
    if (extra > pool->available()) return -1005;
    try {
        s->pages.reserve((std::size_t)blocks_needed);  // all or nothing: the pushes below cannot throw
    } catch (...) {
        return kOutOfHostMemory;
    }
    for (long long i = 0; i < extra; ++i) s->pages.push_back(pool->take_page());
    pool->owned += (int)extra;
    if (slots_out) {
        for (int i = 0; i < n_tokens; ++i) {
            int t = s->len + i;
            slots_out[i] = s->pages[t / pt] * pt + t % pt;
        }
    }
    s->len = (int)new_len;
    return 0;
}

extern "C" int rivoli_pagepool_seq_len(const rivoli_pagepool* pool, int seq) {
    const auto* s = pool ? pool->get(seq) : nullptr;
    return s ? s->len : -1001;
}

extern "C" int rivoli_pagepool_seq_blocks(const rivoli_pagepool* pool, int seq) {
    const auto* s = pool ? pool->get(seq) : nullptr;
    return s ? (int)s->pages.size() : -1001;
}

extern "C" int rivoli_pagepool_block_table(const rivoli_pagepool* pool, int seq, int* out,
                                           int max_blocks) {
    const auto* s = pool ? pool->get(seq) : nullptr;
    if (!s || (max_blocks > 0 && !out)) return -1001;
    int n = (int)s->pages.size();
    for (int i = 0; i < n && i < max_blocks; ++i) out[i] = s->pages[i];
    return n;
}

extern "C" int rivoli_pagepool_pages_free(const rivoli_pagepool* pool) {
    return pool ? pool->available() : -1001;
}
extern "C" int rivoli_pagepool_pages_owned(const rivoli_pagepool* pool) {
    return pool ? pool->owned : -1001;
}
extern "C" int rivoli_pagepool_frontier(const rivoli_pagepool* pool) {
    return pool ? pool->frontier : -1001;
}
