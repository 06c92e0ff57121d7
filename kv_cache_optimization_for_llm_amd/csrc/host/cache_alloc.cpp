// Host-side allocators of the cache manager, behind a C ABI (loaded with ctypes).
//
//  * PagePool  - fixed-size pages with a LIFO free stack and per-page reference counts: the
//    paged mode.  Mirrors what the reference keeps in its KVCacheState
//    (paged_attention/src/engine.cuh:135-178; take/share/drop paged_attention/src/engine.cu:376-404;
//    the accounting invariant :456-475): a page is on the free stack xor has refcount > 0.
//  * Buddy     - binary buddy allocator over a pool of units: the contiguous (Orca-style) mode.
//    Same scheme as base/src/engine.cu:169-254: the pool is viewed as a tree over the next power
//    of two; parts past the real end are never free; frees merge buddies upward.  It also counts
//    the failures where enough units were free in total but no aligned run existed
//    (base/src/engine.cu:336-346).
//
// No GPU code here: this library builds with a plain C++ compiler.
#include <algorithm>
#include <cstdint>
#include <vector>

namespace {

struct PagePool {
    std::vector<int> free_stack;
    std::vector<int> refcount;
    long long takes = 0;  // pages handed out over the pool's life
    long long reuses = 0; // of those, pages that had been held before
    std::vector<uint8_t> ever_used;
};

struct Buddy {
    int pool_units = 0;
    int max_order = 0;
    std::vector<std::vector<int>> free_lists;
    int free_units = 0;
    int reserved_units = 0;
    long long fragmentation_failures = 0;
};

int ceil_log2(int n) {
    int order = 0;
    while ((1LL << order) < n) ++order;
    return order;
}

void buddy_init_range(Buddy &b, int start, int order) {
    if (start >= b.pool_units) return;
    const int size = 1 << order;
    if (start + size <= b.pool_units) {
        b.free_lists[order].push_back(start);
        return;
    }
    if (order == 0) return;
    buddy_init_range(b, start, order - 1);
    buddy_init_range(b, start + size / 2, order - 1);
}

} // namespace

extern "C" {

// ------------------------------------------------------------------ page pool
void *kva_pool_create(int num_pages) {
    if (num_pages <= 0) return nullptr;
    PagePool *p = new PagePool();
    p->refcount.assign(num_pages, 0);
    p->ever_used.assign(num_pages, 0);
    p->free_stack.resize(num_pages);
    // popped from the back, so page 0 goes out first
    for (int i = 0; i < num_pages; ++i) p->free_stack[i] = num_pages - 1 - i;
    return p;
}

void kva_pool_destroy(void *h) { delete static_cast<PagePool *>(h); }

int kva_pool_num_pages(void *h) { return (int)static_cast<PagePool *>(h)->refcount.size(); }
int kva_pool_free_count(void *h) { return (int)static_cast<PagePool *>(h)->free_stack.size(); }
long long kva_pool_takes(void *h) { return static_cast<PagePool *>(h)->takes; }
long long kva_pool_reuses(void *h) { return static_cast<PagePool *>(h)->reuses; }

// Takes n pages or none.  0 on success, -1 when fewer than n are free.
int kva_pool_take(void *h, int n, int *out_pages) {
    PagePool *p = static_cast<PagePool *>(h);
    if (n < 0 || (int)p->free_stack.size() < n) return -1;
    for (int i = 0; i < n; ++i) {
        const int page = p->free_stack.back();
        p->free_stack.pop_back();
        p->refcount[page] = 1;
        ++p->takes;
        if (p->ever_used[page]) ++p->reuses;
        p->ever_used[page] = 1;
        out_pages[i] = page;
    }
    return 0;
}

// One more holder of a held page.  -1 if the page is not held.
int kva_pool_share(void *h, int page) {
    PagePool *p = static_cast<PagePool *>(h);
    if (page < 0 || page >= (int)p->refcount.size() || p->refcount[page] <= 0) return -1;
    return ++p->refcount[page];
}

// Drops one reference of each page; a page whose count reaches zero returns to the free stack.
// Returns the number of pages freed, or -1 - i if pages[i] is out of range or not held (a double
// free); nothing after index i is touched in that case.
int kva_pool_drop(void *h, const int *pages, int n) {
    PagePool *p = static_cast<PagePool *>(h);
    int freed = 0;
    for (int i = 0; i < n; ++i) {
        const int page = pages[i];
        if (page < 0 || page >= (int)p->refcount.size() || p->refcount[page] <= 0) return -1 - i;
        if (--p->refcount[page] == 0) {
            p->free_stack.push_back(page);
            ++freed;
        }
    }
    return freed;
}

int kva_pool_refcount(void *h, int page) {
    PagePool *p = static_cast<PagePool *>(h);
    if (page < 0 || page >= (int)p->refcount.size()) return -1;
    return p->refcount[page];
}

// 1 if every page is on the free stack exactly once xor held, 0 otherwise.
int kva_pool_accounting_holds(void *h) {
    PagePool *p = static_cast<PagePool *>(h);
    std::vector<uint8_t> seen(p->refcount.size(), 0);
    for (int page : p->free_stack) {
        if (page < 0 || page >= (int)p->refcount.size()) return 0;
        if (p->refcount[page] != 0 || seen[page]) return 0;
        seen[page] = 1;
    }
    long long held = 0;
    for (int rc : p->refcount) {
        if (rc < 0) return 0;
        held += rc > 0;
    }
    return held + (long long)p->free_stack.size() == (long long)p->refcount.size() ? 1 : 0;
}

// ------------------------------------------------------------------ buddy allocator
void *kva_buddy_create(int pool_units) {
    if (pool_units <= 0) return nullptr;
    Buddy *b = new Buddy();
    b->pool_units = pool_units;
    b->max_order = ceil_log2(pool_units);
    b->free_lists.assign(b->max_order + 1, {});
    buddy_init_range(*b, 0, b->max_order);
    b->free_units = pool_units;
    return b;
}

void kva_buddy_destroy(void *h) { delete static_cast<Buddy *>(h); }

// Size a request of `units` really takes: the next power of two.
int kva_buddy_round(int units) { return units <= 0 ? 0 : 1 << ceil_log2(units); }

// Start of a self-aligned run of round(units) units, or -1.
int kva_buddy_alloc(void *h, int units) {
    Buddy *b = static_cast<Buddy *>(h);
    if (units <= 0) return -1;
    const int want = ceil_log2(units);
    const int size = 1 << want;
    int k = want;
    while (k <= b->max_order && b->free_lists[k].empty()) ++k;
    if (k > b->max_order) {
        if (b->free_units >= size) ++b->fragmentation_failures;
        return -1;
    }
    const int start = b->free_lists[k].back();
    b->free_lists[k].pop_back();
    while (k > want) {
        --k;
        b->free_lists[k].push_back(start + (1 << k));
    }
    b->free_units -= size;
    b->reserved_units += size;
    return start;
}

// Gives back the run that kva_buddy_alloc(units) returned at `start`.  0 ok, -1 on a bad run.
int kva_buddy_free(void *h, int start, int units) {
    Buddy *b = static_cast<Buddy *>(h);
    if (units <= 0 || start < 0) return -1;
    int order = ceil_log2(units);
    const int size = 1 << order;
    if (start % size != 0 || start + size > b->pool_units) return -1;
    // refuse a run that overlaps anything free (a double free)
    for (int o = 0; o <= b->max_order; ++o)
        for (int s : b->free_lists[o])
            if (s < start + size && start < s + (1 << o)) return -1;
    b->free_units += size;
    b->reserved_units -= size;
    while (order < b->max_order) {
        const int buddy = start ^ (1 << order);
        std::vector<int> &list = b->free_lists[order];
        auto it = std::find(list.begin(), list.end(), buddy);
        if (it == list.end()) break;
        list.erase(it);
        start = std::min(start, buddy);
        ++order;
    }
    b->free_lists[order].push_back(start);
    return 0;
}

int kva_buddy_free_units(void *h) { return static_cast<Buddy *>(h)->free_units; }
int kva_buddy_reserved_units(void *h) { return static_cast<Buddy *>(h)->reserved_units; }
int kva_buddy_pool_units(void *h) { return static_cast<Buddy *>(h)->pool_units; }
long long kva_buddy_fragmentation_failures(void *h) {
    return static_cast<Buddy *>(h)->fragmentation_failures;
}

// Writes the free runs as (start, order) pairs, sorted; returns how many there are (even if
// that is more than `cap`).
int kva_buddy_free_runs(void *h, int *out, int cap) {
    Buddy *b = static_cast<Buddy *>(h);
    std::vector<std::pair<int, int>> runs;
    for (int o = 0; o <= b->max_order; ++o)
        for (int s : b->free_lists[o]) runs.push_back({s, o});
    std::sort(runs.begin(), runs.end());
    for (int i = 0; i < (int)runs.size() && i < cap; ++i) {
        out[2 * i] = runs[i].first;
        out[2 * i + 1] = runs[i].second;
    }
    return (int)runs.size();
}

} // extern "C"
