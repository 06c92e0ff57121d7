// Host-side allocators of the cache manager, behind a C ABI (loaded with ctypes).
//
//  * PagePool  - fixed-size pages with a LIFO free stack and per-page reference counts: the
//    paged mode.  Keeps what the reference keeps in its KVCacheState
//    (paged_attention/src/engine.cuh:135-178; take/share/drop paged_attention/src/engine.cu:376-404;
//    the accounting invariant :456-475): a page is on the free stack xor has refcount > 0.
//  * Buddy     - binary buddy allocation of power-of-two, self-aligned runs of units: the
//    contiguous (Orca-style) mode, with the behaviour of base/src/engine.cu:169-254 (a pool that
//    is no power of two never hands out its missing end; freed buddies merge; failures where
//    enough units were free in total but no aligned run existed are counted, :336-346).  The
//    structure is another one: not lists of free runs per order that are searched, but one array
//    over the implicit binary tree of all possible runs, holding for every node the largest
//    order of a wholly free run inside it.  Allocation walks down from the root (always into
//    the tighter fit, so large runs stay whole), freeing finds its node by arithmetic, both fix
//    the path to the root: O(log pool) each, and a run that is not allocated (a double free) is
//    seen from one flag, not by comparing against every free run.
//
// No GPU code here: this library builds with a plain C++ compiler.
#include <algorithm>
#include <cstdint>
#include <utility>
#include <vector>

namespace {

struct PagePool {
    std::vector<int> free_stack;
    std::vector<int> refcount;
    long long takes = 0;  // pages handed out over the pool's life
    long long reuses = 0; // of those, pages that had been held before
    std::vector<uint8_t> ever_used;
};

// Ceiling of log2(n) for n >= 1.
int order_for(int n) { return n <= 1 ? 0 : 32 - __builtin_clz((unsigned)(n - 1)); }

struct Buddy {
    static constexpr int8_t NONE = -1;
    int pool_units = 0;
    int max_order = 0;      // the tree spans 1 << max_order units; those past pool_units never exist
    // Heap numbering: node 1 is the whole span; node i has children 2i and 2i + 1; the node of the
    // run (start, order) is (1 << (max_order - order)) + (start >> order).
    std::vector<int8_t> best;    // largest order of a wholly free run inside the node, or NONE
    std::vector<uint8_t> taken;  // 1: the node is handed out as one run
    int free_units = 0;
    int reserved_units = 0;
    long long fragmentation_failures = 0;

    int node_of(int start, int order) const { return (1 << (max_order - order)) + (start >> order); }

    // What a node of `order` holds, given its children: the whole run if both halves are whole.
    int8_t joined(int node, int order) const {
        const int8_t l = best[2 * node], r = best[2 * node + 1];
        return (l == order - 1 && r == order - 1) ? (int8_t)order : std::max(l, r);
    }

    void fix_upwards(int node, int order) {
        for (node >>= 1, ++order; node >= 1; node >>= 1, ++order) best[node] = joined(node, order);
    }

    void build() {
        const int span = 1 << max_order;
        best.assign(2 * (size_t)span, NONE);
        taken.assign(2 * (size_t)span, 0);
        for (int u = 0; u < pool_units; ++u) best[span + u] = 0;
        for (int order = 1; order <= max_order; ++order) {
            const int first = 1 << (max_order - order);
            for (int node = first; node < 2 * first; ++node) best[node] = joined(node, order);
        }
    }
};

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
    if (pool_units <= 0 || pool_units > (1 << 29)) return nullptr;
    Buddy *b = new Buddy();
    b->pool_units = pool_units;
    b->max_order = order_for(pool_units);
    b->build();
    b->free_units = pool_units;
    return b;
}

void kva_buddy_destroy(void *h) { delete static_cast<Buddy *>(h); }

// Size a request of `units` really takes: the next power of two.
int kva_buddy_round(int units) { return units <= 0 ? 0 : 1 << order_for(units); }

// Start of a self-aligned run of round(units) units, or -1.
int kva_buddy_alloc(void *h, int units) {
    Buddy *b = static_cast<Buddy *>(h);
    if (units <= 0) return -1;
    const int want = order_for(units);
    if (want > b->max_order || b->best[1] < want) {
        if (want <= 30 && b->free_units >= (1 << want)) ++b->fragmentation_failures;
        return -1;
    }
    int node = 1;
    for (int order = b->max_order; order > want; --order) {
        const int8_t l = b->best[2 * node], r = b->best[2 * node + 1];
        // into the half that fits more tightly; the lower addresses on a tie
        const bool left = l >= want && (r < want || l <= r);
        node = 2 * node + (left ? 0 : 1);
    }
    b->taken[node] = 1;
    b->best[node] = Buddy::NONE;
    b->fix_upwards(node, want);
    b->free_units -= 1 << want;
    b->reserved_units += 1 << want;
    return (node - (1 << (b->max_order - want))) << want;
}

// Gives back the run that kva_buddy_alloc(units) returned at `start`.  0 ok, -1 if that is not an
// allocated run (never handed out, or given back already).
int kva_buddy_free(void *h, int start, int units) {
    Buddy *b = static_cast<Buddy *>(h);
    if (units <= 0 || start < 0) return -1;
    const int order = order_for(units);
    if (order > b->max_order) return -1;
    const int size = 1 << order;
    if (start % size != 0 || start + size > b->pool_units) return -1;
    const int node = b->node_of(start, order);
    if (!b->taken[node]) return -1;
    b->taken[node] = 0;
    b->best[node] = (int8_t)order;     // everything below it has stayed as it was: wholly free
    b->fix_upwards(node, order);
    b->free_units += size;
    b->reserved_units -= size;
    return 0;
}

int kva_buddy_free_units(void *h) { return static_cast<Buddy *>(h)->free_units; }
int kva_buddy_reserved_units(void *h) { return static_cast<Buddy *>(h)->reserved_units; }
int kva_buddy_pool_units(void *h) { return static_cast<Buddy *>(h)->pool_units; }
long long kva_buddy_fragmentation_failures(void *h) {
    return static_cast<Buddy *>(h)->fragmentation_failures;
}

// Writes the free runs as (start, order) pairs in address order, each as large as it can be
// (two free buddies are one run); returns how many there are (even if more than `cap`).
int kva_buddy_free_runs(void *h, int *out, int cap) {
    Buddy *b = static_cast<Buddy *>(h);
    int count = 0;
    std::vector<std::pair<int, int>> todo{{1, b->max_order}};     // (node, order), a stack: left halves first
    while (!todo.empty()) {
        const auto [node, order] = todo.back();
        todo.pop_back();
        if (b->best[node] == Buddy::NONE) continue;
        if (b->best[node] == order) {
            if (count < cap) {
                out[2 * count] = (node - (1 << (b->max_order - order))) << order;
                out[2 * count + 1] = order;
            }
            ++count;
            continue;
        }
        todo.push_back({2 * node + 1, order - 1});
        todo.push_back({2 * node, order - 1});
    }
    return count;
}

} // extern "C"
