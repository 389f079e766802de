// CPU model of the turn taking of the plain simulator's scheduled launch (mms_amd/csrc/sim_mixed.hip,
// the loop "one turn per (item, segment)"), for ThreadSanitizer: wavefronts are threads, the workgroup's
// schedule words in LDS are std::atomic<uint32_t>, and everything the protocol is there to protect is
// PLAIN memory -- the clocks an item parks in device memory between two segments and its running
// counts -- so that a missing happens-before edge between the wavefront that parks and the one that
// picks up is a data race the sanitizer reports, and a wrong hand-over is a failed check.
//
// The claim loop, the memory orders and the order of operations are those of the kernel:
//   look:    relaxed loads of the words; skip finished items and items too large for this wavefront's
//            region; among the free ones take the one furthest behind (ties: the largest)
//   claim:   compare-and-swap word -> word | 1, acquire on success; then an acquire fence
//   turn:    load the parked state (segments after the first), simulate, park the state
//   release: release fence, then a release store of (segment + 1) << 1; the last segment bumps the
//            completion counter
//   nothing to claim but items in other hands: sleep, look again, leave after `spin_limit` looks
// Checked: every (item, segment) is simulated exactly once and in order, by whichever wavefront; the
// state found at pick-up is the state the previous segment parked; every item is completed and counted
// once although wavefronts may leave early; no wavefront ever takes an item larger than its region.
//
// usage: sched_model <seed> <rounds>     exit status 0 = all checks passed (ThreadSanitizer reports on stderr
// and makes the status non-zero by itself)
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <thread>
#include <vector>

namespace {

// SCHED_MODEL_BROKEN builds the same protocol with relaxed orders and no fences: the sanitizer must then
// report the hand-over as a data race (the check of the checker).
#ifdef SCHED_MODEL_BROKEN
constexpr std::memory_order kAcquire = std::memory_order_relaxed, kRelease = std::memory_order_relaxed;
inline void fence(std::memory_order) {}
#else
constexpr std::memory_order kAcquire = std::memory_order_acquire, kRelease = std::memory_order_release;
inline void fence(std::memory_order o) { std::atomic_thread_fence(o); }
#endif

constexpr int kSlots = 6;  // parked words per item (stand-ins for clocks and counters)

struct Item {
    int bytes = 0, nseg = 1;
    uint64_t parked[kSlots] = {};  // plain: protected by the protocol alone
    int next_seg = 0;              // plain: the segment that must come next
    int turns = 0;                 // plain: how often the item was simulated
};

struct Group {
    std::vector<Item> items;
    std::vector<std::atomic<uint32_t>> word;
    std::vector<int> region_bytes;  // per wavefront, -1: none
    std::atomic<int> completed{0};
    std::atomic<int> failures{0};
    std::atomic<int> go{0};  // start gate: the wavefronts of a workgroup start together
    int spin_limit = 0;
    explicit Group(size_t n) : items(n), word(n) {
        for (auto &w : word) w.store(0u, std::memory_order_relaxed);
    }
};

uint64_t state_after(int item, int seg, int slot) {  // what segment `seg` of `item` leaves in `slot`
    uint64_t x = 0x9E3779B97F4A7C15ull * (uint64_t)(item + 1) + 0xD1B54A32D192ED03ull * (uint64_t)(seg + 1) + (uint64_t)slot;
    x ^= x >> 29;
    return x * 0xBF58476D1CE4E5B9ull;
}

void wavefront(Group &g, int wv, uint32_t seed) {
    std::minstd_rand rng(seed);
    const int part_bytes = g.region_bytes[(size_t)wv];
    if (part_bytes < 0) return;  // no LDS region in this schedule: leaves at once
    const int n_items = (int)g.items.size();
    while (g.go.load(std::memory_order_acquire) == 0) {
    }
    for (int spins = 0;;) {
        int got = -1;  // -1: nothing left for this wavefront, -2: what is left is in other hands right now
        for (int tries = 0; tries < 64; ++tries) {
            int best = -1, best_bytes = -1;
            uint32_t best_word = 0xFFFFFFFFu;
            bool pending = false;
            for (int k = 0; k < n_items; ++k) {
                const uint32_t w = g.word[(size_t)k].load(std::memory_order_relaxed);
                const int sg = (int)(w >> 1), nsg = g.items[(size_t)k].nseg, bytes = g.items[(size_t)k].bytes;
                if (sg >= nsg || bytes > part_bytes) continue;
                if (w & 1u) {
                    if (sg + 1 < nsg) pending = true;
                    continue;
                }
                if (w < best_word || (w == best_word && bytes > best_bytes)) {
                    best = k;
                    best_word = w;
                    best_bytes = bytes;
                }
            }
            if (best < 0) {
                got = pending ? -2 : -1;
                break;
            }
            uint32_t expect = best_word;
            if (g.word[(size_t)best].compare_exchange_strong(expect, best_word | 1u, kAcquire, std::memory_order_relaxed)) {
                got = best;
                break;
            }
            got = -2;
        }
        if (got == -1) break;
        if (got == -2) {
            std::this_thread::yield();
            if (++spins > g.spin_limit) break;
            continue;
        }
        spins = 0;
        Item &it = g.items[(size_t)got];
        const int seg = (int)(g.word[(size_t)got].load(std::memory_order_relaxed) >> 1);
        fence(std::memory_order_acquire);
        // ---- the turn: everything below touches plain memory only
        if (it.bytes > part_bytes) g.failures.fetch_add(1);
        if (it.next_seg != seg) g.failures.fetch_add(1);
        it.next_seg = seg + 1;
        it.turns += 1;
        if (seg > 0)
            for (int s = 0; s < kSlots; ++s)
                if (it.parked[s] != state_after(got, seg - 1, s)) g.failures.fetch_add(1);
        {   // segments take different times
            volatile unsigned work = 0;
            for (unsigned i = 0, n = 200 + rng() % 3000; i < n; ++i) work = work + i;
            if (rng() % 8 == 0) std::this_thread::yield();
        }
        const bool last_seg = seg + 1 >= it.nseg;
        if (!last_seg)
            for (int s = 0; s < kSlots; ++s) it.parked[s] = state_after(got, seg, s);
        // ---- hand the item back
        fence(std::memory_order_release);
        g.word[(size_t)got].store((uint32_t)(seg + 1) << 1, kRelease);
        if (last_seg) g.completed.fetch_add(1);
    }
}

}  // namespace

int main(int argc, char **argv) {
    const uint32_t seed = argc > 1 ? (uint32_t)std::strtoul(argv[1], nullptr, 10) : 1u;
    const int rounds = argc > 2 ? std::atoi(argv[2]) : 200;
    std::mt19937 rng(seed);
    int bad = 0;
    for (int round = 0; round < rounds; ++round) {
        // a workgroup as the host plans it: items largest first, regions sized for the largest items that fit the LDS
        const int n_items = 1 + (int)(rng() % 12), max_regions = 1 + (int)(rng() % 8);
        const int cap = 160 * 1024 - 8 * 1024;
        Group g((size_t)n_items);
        for (Item &it : g.items) {
            it.bytes = 1024 * (2 + (int)(rng() % 32));
            it.nseg = 1 + (int)(rng() % 9);
        }
        std::sort(g.items.begin(), g.items.end(), [](const Item &x, const Item &y) { return x.bytes > y.bytes; });
        int used = 0;
        for (int k = 0; k < n_items && (int)g.region_bytes.size() < max_regions; ++k)
            if (used + g.items[(size_t)k].bytes <= cap) {
                g.region_bytes.push_back(g.items[(size_t)k].bytes);
                used += g.items[(size_t)k].bytes;
            }
        while ((int)g.region_bytes.size() < 8) g.region_bytes.push_back(-1);
        const int limits[] = {0, 1, 3, 1000000};
        g.spin_limit = limits[rng() % 4];
        std::vector<std::thread> pool;
        for (int wv = 0; wv < 8; ++wv) pool.emplace_back(wavefront, std::ref(g), wv, (uint32_t)rng());
        g.go.store(1, std::memory_order_release);
        for (std::thread &t : pool) t.join();
        int turns = 0, want = 0;
        for (int k = 0; k < n_items; ++k) {
            const Item &it = g.items[(size_t)k];
            turns += it.turns;
            want += it.nseg;
            if (g.word[(size_t)k].load() != (uint32_t)it.nseg << 1) ++bad;  // every item ran to its end and was handed back
            if (it.next_seg != it.nseg) ++bad;
        }
        if (turns != want || g.completed.load() != n_items || g.failures.load() != 0) ++bad;
        if (bad) {
            std::fprintf(stderr, "round %d: %d turns of %d, %d of %d items completed, %d failed checks\n", round, turns, want,
                         g.completed.load(), n_items, g.failures.load());
            return 1;
        }
    }
    std::printf("ok: %d workgroups, every item completed once, every hand-over found the parked state\n", rounds);
    return 0;
}
