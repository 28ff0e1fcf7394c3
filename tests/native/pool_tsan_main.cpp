// ThreadSanitizer driver for the allocator's policy code: several threads allocate, free, trim
// and read statistics on ONE pool over the fake backing store, the way PyTorch's threads call
// into the library.  Built with -fsanitize=thread by tests/test_races.py; any data race makes
// the sanitizer report and the process exit non-zero.
#include <atomic>
#include <cstdio>
#include <random>
#include <thread>
#include <vector>

#include "pool_harness.cpp"

int main() {
    void* h = ph_create(64ull << 30);
    ph_set_arena(h, 256ull << 20);
    ph_set_trim(h, 1ull << 30, 256ull << 20);
    std::atomic<long> bad{0};
    auto worker = [&](unsigned seed) {
        std::mt19937 rng(seed);
        std::vector<std::pair<uintptr_t, size_t>> mine;
        for (int i = 0; i < 4000; i++) {
            const unsigned pick = rng() % 100;
            if (pick < 55 || mine.empty()) {
                size_t bytes = pick % 3 == 0 ? (size_t)(8u << 20) + (rng() % 64) * (1u << 20) : 512 + rng() % (1u << 20);
                uintptr_t p = ph_alloc(h, bytes, seed % 3, 0);
                if (!p) { bad++; continue; }
                if (ph_block_bytes(h, p) < bytes) bad++;
                mine.push_back({p, bytes});
            } else if (pick < 95) {
                size_t k = rng() % mine.size();
                if (ph_free(h, mine[k].first, seed % 3) != 0) bad++;
                mine[k] = mine.back();
                mine.pop_back();
            } else if (pick < 97) {
                ph_release_unused(h);
            } else if (pick < 99) {
                uint64_t st[32];
                ph_stats(h, st, 32);
            } else {
                ph_set_trim(h, (1ull << 30) + (rng() % 4) * (256ull << 20), 256ull << 20);
            }
        }
        for (auto& b : mine) if (ph_free(h, b.first, seed % 3) != 0) bad++;
    };
    std::vector<std::thread> threads;
    for (unsigned t = 0; t < 6; t++) threads.emplace_back(worker, 1000 + t);
    for (auto& t : threads) t.join();
    uint64_t st[32];
    ph_stats(h, st, 32);
    const unsigned long long live = st[13];          // bytes_live
    ph_release_unused(h);
    std::printf("bad=%ld live=%llu backing_used=%zu\n", bad.load(), live, ph_backing_used(h));
    const int rc = (bad.load() == 0 && live == 0 && ph_backing_used(h) == 0) ? 0 : 1;
    ph_destroy(h);
    return rc;
}
