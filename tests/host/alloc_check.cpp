// A driver for the host allocators (csrc/host/cache_alloc.cpp) that is built with
// -fsanitize=address,undefined and run by the CPU tests: seeded random orders of requests against
// both allocators, each step checked against a plain model of what is held (a set of pages, a
// map of runs), so that an out-of-bounds index, a use after free or an overflow in the
// allocators stops the program, and a page or run that is lost, handed out twice or freed twice
// fails a check.  Prints "ok <checks>" and exits with 0, or says what failed and exits with 1.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <set>
#include <vector>

extern "C" {
void *kva_pool_create(int num_pages);
void kva_pool_destroy(void *h);
int kva_pool_free_count(void *h);
int kva_pool_take(void *h, int n, int *out_pages);
int kva_pool_share(void *h, int page);
int kva_pool_drop(void *h, const int *pages, int n);
int kva_pool_refcount(void *h, int page);
int kva_pool_accounting_holds(void *h);
void *kva_buddy_create(int pool_units);
void kva_buddy_destroy(void *h);
int kva_buddy_round(int units);
int kva_buddy_alloc(void *h, int units);
int kva_buddy_free(void *h, int start, int units);
int kva_buddy_free_units(void *h);
int kva_buddy_reserved_units(void *h);
long long kva_buddy_fragmentation_failures(void *h);
int kva_buddy_free_runs(void *h, int *out, int cap);
}

static long long checks = 0;
#define CHECK(cond, ...)                                                                   \
    do {                                                                                   \
        ++checks;                                                                          \
        if (!(cond)) {                                                                     \
            std::fprintf(stderr, "alloc_check: " __VA_ARGS__);                             \
            std::fprintf(stderr, " (%s:%d)\n", __FILE__, __LINE__);                        \
            std::exit(1);                                                                  \
        }                                                                                  \
    } while (0)

static void pool_round(unsigned seed, int pages) {
    std::mt19937 rng(seed);
    void *p = kva_pool_create(pages);
    CHECK(p != nullptr, "pool of %d pages was not created", pages);
    std::map<int, int> held;                         // page -> references
    std::vector<int> buf(pages + 4);
    for (int step = 0; step < 4000; ++step) {
        const int what = rng() % 10;
        if (what < 4) {
            const int n = rng() % 7;
            const int free_before = kva_pool_free_count(p);
            const int rc = kva_pool_take(p, n, buf.data());
            CHECK((rc == 0) == (n <= free_before), "take(%d) with %d free returned %d", n, free_before, rc);
            if (rc == 0)
                for (int i = 0; i < n; ++i) {
                    CHECK(buf[i] >= 0 && buf[i] < pages && !held.count(buf[i]), "page %d handed out twice", buf[i]);
                    held[buf[i]] = 1;
                }
        } else if (what < 8 && !held.empty()) {
            auto it = held.begin();
            std::advance(it, rng() % held.size());
            const int page = it->first;
            const int freed = kva_pool_drop(p, &page, 1);
            CHECK(freed == (it->second == 1 ? 1 : 0), "drop of page %d with %d references freed %d", page, it->second, freed);
            if (--it->second == 0) held.erase(it);
        } else if (what == 8 && !held.empty()) {
            auto it = held.begin();
            std::advance(it, rng() % held.size());
            CHECK(kva_pool_share(p, it->first) == ++it->second, "share of page %d", it->first);
        } else {
            int page = (int)(rng() % (pages + 8)) - 4;       // sometimes outside the pool
            if (!held.count(page)) {
                CHECK(kva_pool_drop(p, &page, 1) == -1, "a page that is not held (%d) could be dropped", page);
                CHECK(kva_pool_share(p, page) == -1, "a page that is not held (%d) could be shared", page);
            }
        }
        CHECK(kva_pool_free_count(p) + (int)held.size() == pages, "%d free + %zu held is not %d",
              kva_pool_free_count(p), held.size(), pages);
        if (step % 64 == 0) CHECK(kva_pool_accounting_holds(p) == 1, "page accounting does not hold");
    }
    for (auto &kv : held) CHECK(kva_pool_refcount(p, kv.first) == kv.second, "reference count of page %d", kv.first);
    kva_pool_destroy(p);
}

static void buddy_round(unsigned seed, int units) {
    std::mt19937 rng(seed);
    void *b = kva_buddy_create(units);
    CHECK(b != nullptr, "buddy pool of %d units was not created", units);
    std::vector<int> first(2 * units + 2);
    const int n_first = kva_buddy_free_runs(b, first.data(), units + 1);
    std::map<int, int> runs;                          // start -> size as asked
    std::vector<char> used(units, 0);
    for (int step = 0; step < 4000; ++step) {
        if (rng() % 5 < 3 || runs.empty()) {
            const int want = 1 + rng() % (units / 2 + 1);
            const int size = kva_buddy_round(want);
            CHECK(size >= want && size < 2 * want + 1 && (size & (size - 1)) == 0, "round(%d) = %d", want, size);
            const long long fails = kva_buddy_fragmentation_failures(b);
            const int free_before = kva_buddy_free_units(b);
            const int start = kva_buddy_alloc(b, want);
            if (start < 0) {
                CHECK(kva_buddy_fragmentation_failures(b) == fails + (free_before >= size ? 1 : 0),
                      "fragmentation counter after a refused run of %d with %d free", size, free_before);
                continue;
            }
            CHECK(start % size == 0 && start + size <= units, "run (%d, %d) is misaligned or past the pool's end %d",
                  start, size, units);
            for (int u = start; u < start + size; ++u) {
                CHECK(!used[u], "unit %d handed out twice", u);
                used[u] = 1;
            }
            runs[start] = want;
        } else {
            auto it = runs.begin();
            std::advance(it, rng() % runs.size());
            const int start = it->first, want = it->second, size = kva_buddy_round(want);
            CHECK(kva_buddy_free(b, start, want) == 0, "run (%d, %d) could not be given back", start, want);
            CHECK(kva_buddy_free(b, start, want) == -1, "run (%d, %d) could be given back twice", start, want);
            for (int u = start; u < start + size; ++u) used[u] = 0;
            runs.erase(it);
        }
        int held = 0;
        for (char c : used) held += c;
        CHECK(kva_buddy_reserved_units(b) == held && kva_buddy_free_units(b) == units - held,
              "reserved %d + free %d against %d held of %d", kva_buddy_reserved_units(b), kva_buddy_free_units(b), held, units);
        // a run that was not handed out (anywhere, any size, also outside the pool) cannot be given back
        const int s = (int)(rng() % (2 * units)) - units / 2, n = 1 + rng() % units;
        auto live = runs.find(s);
        if (live == runs.end() || kva_buddy_round(live->second) != kva_buddy_round(n))
            CHECK(kva_buddy_free(b, s, n) == -1, "run (%d, %d) was never handed out but could be given back", s, n);
    }
    kva_buddy_destroy(b);
    // every run given back: the free runs are the initial ones again
    b = kva_buddy_create(units);
    std::vector<std::pair<int, int>> got;
    for (int i = 0; i < 200; ++i) {
        const int want = 1 + rng() % 9;
        const int s = kva_buddy_alloc(b, want);
        if (s >= 0) got.push_back({s, want});
    }
    std::shuffle(got.begin(), got.end(), rng);
    for (auto &r : got) CHECK(kva_buddy_free(b, r.first, r.second) == 0, "run (%d, %d) lost", r.first, r.second);
    std::vector<int> last(2 * units + 2);
    const int n_last = kva_buddy_free_runs(b, last.data(), units + 1);
    CHECK(n_last == n_first, "%d free runs after everything was given back, %d at the start", n_last, n_first);
    for (int i = 0; i < 2 * n_first; ++i) CHECK(first[i] == last[i], "free runs differ from the initial ones");
    kva_buddy_destroy(b);
}

int main() {
    for (unsigned seed = 0; seed < 6; ++seed) {
        pool_round(seed, 1 + (seed * 37) % 90);
        buddy_round(seed, (int[]){1, 16, 100, 7, 64, 333}[seed]);
    }
    std::printf("ok %lld\n", checks);
    return 0;
}
