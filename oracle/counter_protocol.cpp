// CPU model of the counter protocol of the overlapped path, for ThreadSanitizer.
// Test infrastructure only: nothing in the product links or runs this.
//
// What is modelled (reference: src/overlap/gemm_with_signal.h:184-201 for the
// producer side, src/wait.cuh:5-9 and src/overlap_impl.cu:257-270 for the
// waiter, the per-group collective and the event join):
//   * producer threads ("workgroups") each take tiles from a shared ticket in
//     any order, write the tile's slot of the permuted buffer with plain
//     stores, then bump MM[group(slot)] with a release-ordered fetch_add;
//   * one waiter thread walks the groups in index order: it polls MM[g] until
//     it equals cSeg[g] (bounded by a spin limit, like the library's bounded
//     wait), resets it to 0, and then "consumes" the group: copies its
//     contiguous range into the staging buffer;
//   * the next call's producers start only after the waiter has finished
//     (the event join), so a counter is never bumped before it was reset.
// The model is run for several calls on the same counters.  Under
// -fsanitize=thread any missing ordering between a tile's stores and the
// consumer's loads of it shows as a data race; the program also checks the
// staging buffer, the counters (all zero after every call) and the release
// order.  With --short-count the last group's cSeg entry is one too large:
// the waiter's bounded spin must trip, report the group and leave the rest.
// With --relaxed-signal both the signal and the poll are relaxed (the ordering
// is removed on purpose): ThreadSanitizer must then report a race, which shows
// that the model can see the mistake the ordering prevents.
//
// Build and run: see tests/test_counter_protocol.py.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <thread>
#include <vector>

namespace {

struct Problem {
    int tiles;                 // T
    int tile_elems;            // BM * BN of the model (small)
    std::vector<int> cseg;     // group sizes, sum == tiles (unless --short-count)
    std::vector<int> ra;       // tile -> slot, a permutation
    std::vector<int> group_of_slot;
};

// The epilogue's linear scan (src/overlap/gemm_with_signal.h:188-193).
int scan_group(const std::vector<int>& cseg, int slot) {
    int bound = cseg[0], g = 0;
    while (bound <= slot) {
        ++g;
        bound += cseg[g];
    }
    return g;
}

struct Shared {
    std::vector<int> c;                      // permuted output buffer (plain memory)
    std::vector<int> staging;                // consumer's destination (plain memory)
    std::vector<std::atomic<int>> mm;        // group counters
    std::atomic<int> ticket{0};              // which tile a producer takes next
    explicit Shared(const Problem& p)
        : c((size_t)p.tiles * p.tile_elems, -1), staging((size_t)p.tiles * p.tile_elems, -1), mm(p.cseg.size()) {
        for (auto& m : mm) m.store(0, std::memory_order_relaxed);
    }
};

int tile_value(int call, int tile, int e) { return call * 1000003 + tile * 131 + e; }

std::memory_order g_signal_order = std::memory_order_release;
std::memory_order g_poll_order = std::memory_order_acquire;

void producer(const Problem& p, Shared& s, int call) {
    for (;;) {
        const int t = s.ticket.fetch_add(1, std::memory_order_relaxed);
        if (t >= p.tiles) return;
        const int slot = p.ra[t];
        int* dst = s.c.data() + (size_t)slot * p.tile_elems;
        for (int e = 0; e < p.tile_elems; ++e) dst[e] = tile_value(call, t, e);   // the tile's stores
        // the signal: everything above is visible before the counter moves
        s.mm[p.group_of_slot[slot]].fetch_add(1, g_signal_order);
    }
}

// Returns the number of groups released; on a spin-limit expiry stops there and reports it.
int waiter(const Problem& p, Shared& s, long spin_limit, std::vector<int>& order, int* expired_group) {
    size_t lo = 0;
    *expired_group = -1;
    for (int g = 0; g < (int)p.cseg.size(); ++g) {
        long spins = 0;
        // the acquire pairs with the producers' release: the group's tiles are visible once the count is seen
        while (s.mm[g].load(g_poll_order) != p.cseg[g]) {
            if (++spins > spin_limit) {
                *expired_group = g;
                return g;
            }
            std::this_thread::yield();
        }
        s.mm[g].store(0, std::memory_order_relaxed);   // nothing else writes it until the next call
        const size_t n = (size_t)p.cseg[g] * p.tile_elems;
        std::memcpy(s.staging.data() + lo, s.c.data() + lo, n * sizeof(int));   // the "collective" on the group's range
        order.push_back(g);
        lo += n;
    }
    return (int)p.cseg.size();
}

}  // namespace

int main(int argc, char** argv) {
    bool short_count = false;
    int calls = 5, producers = 6;
    for (int i = 1; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--short-count")) short_count = true;
        else if (!std::strcmp(argv[i], "--relaxed-signal")) g_signal_order = g_poll_order = std::memory_order_relaxed;
        else if (!std::strcmp(argv[i], "--calls") && i + 1 < argc) calls = std::atoi(argv[++i]);
        else if (!std::strcmp(argv[i], "--producers") && i + 1 < argc) producers = std::atoi(argv[++i]);
    }
    Problem p;
    p.tiles = 96;
    p.tile_elems = 64;
    p.cseg = {5, 0, 17, 32, 1, 41};          // ragged, with an empty group
    p.ra.resize(p.tiles);
    std::iota(p.ra.begin(), p.ra.end(), 0);
    unsigned seed = 12345;                   // a fixed permutation of the slots
    for (int i = p.tiles - 1; i > 0; --i) {
        seed = seed * 1664525u + 1013904223u;
        std::swap(p.ra[i], p.ra[seed % (unsigned)(i + 1)]);
    }
    p.group_of_slot.resize(p.tiles);
    for (int sl = 0; sl < p.tiles; ++sl) p.group_of_slot[sl] = scan_group(p.cseg, sl);
    if (short_count) p.cseg.back() += 1;     // one tile more than will ever arrive
    const long spin_limit = short_count ? 200000 : 2000000000L;

    Shared s(p);
    for (int call = 0; call < calls; ++call) {
        s.ticket.store(0, std::memory_order_relaxed);
        std::vector<int> order;
        int expired = -1, released = 0;
        std::thread w([&] { released = waiter(p, s, spin_limit, order, &expired); });
        std::vector<std::thread> ps;
        for (int i = 0; i < producers; ++i) ps.emplace_back(producer, std::cref(p), std::ref(s), call);
        for (auto& t : ps) t.join();
        w.join();   // the event join: the next call starts behind the waiter
        if (short_count) {
            const int last = (int)p.cseg.size() - 1;
            if (expired != last || released != last) {
                std::printf("FAIL: expected the bounded wait to expire on group %d, got expired=%d released=%d\n", last,
                            expired, released);
                return 1;
            }
            std::printf("ok: bounded wait expired on group %d after releasing %d groups\n", expired, released);
            return 0;
        }
        if (expired != -1 || released != (int)p.cseg.size()) {
            std::printf("FAIL: call %d released %d groups, expired %d\n", call, released, expired);
            return 1;
        }
        for (int g = 0; g < released; ++g)
            if (order[g] != g) {
                std::printf("FAIL: call %d released group %d at position %d\n", call, order[g], g);
                return 1;
            }
        for (auto& m : s.mm)
            if (m.load(std::memory_order_relaxed) != 0) {
                std::printf("FAIL: call %d left a counter behind\n", call);
                return 1;
            }
        for (int t = 0; t < p.tiles; ++t)
            for (int e = 0; e < p.tile_elems; ++e)
                if (s.staging[(size_t)p.ra[t] * p.tile_elems + e] != tile_value(call, t, e)) {
                    std::printf("FAIL: call %d tile %d element %d is stale or misplaced\n", call, t, e);
                    return 1;
                }
    }
    std::printf("ok: %d calls, %d producers, %zu groups, staging equals the permuted output every time\n", calls,
                producers, p.cseg.size());
    return 0;
}
