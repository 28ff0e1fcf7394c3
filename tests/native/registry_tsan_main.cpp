// ThreadSanitizer driver for the library's host-side shared state that needs no GPU: the header ->
// id registry, the tuning knobs, the configuration setters, the error slot and the run-time
// compiler's cache.  Several threads register headers, change knobs, ask for configuration blocks
// and compile, all at once, through the C ABI.  Built (library sources included) with
// -fsanitize=thread by tests/test_races.py.
#include <atomic>
#include <cstdio>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "../../include/sideaware.h"

static std::string header_text(int k) {
    return "#define KERNEL_NAME race_test_" + std::to_string(k) + "\n"
           "typedef int o0;\ntypedef int i0;\nstruct unused {};\ntypedef unused o1, o2, o3, i1, i2, i3;\n"
           "constexpr bool reverse_order = false;\nconstexpr bool input_evict[4] = {true, false, false, false};\n"
           "__device__ void elementwise_op(size_t element_idx, int sideband, o0 &out0, o1 &out1, o2 &out2, o3 &out3,\n"
           "                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) { out0 = in0 + " +
           std::to_string(k) + "; }\n";
}

int main() {
    constexpr int kThreads = 6, kShared = 40;
    std::atomic<int> bad{0};
    std::vector<std::vector<int>> ids(kThreads, std::vector<int>(kShared, -1));
    auto worker = [&](int t) {
        for (int round = 0; round < 30; round++) {
            for (int k = 0; k < kShared; k++) {
                // every thread registers the same forty headers: they must agree on the ids
                const int id = sideaware_create_kernel(header_text(k).c_str());
                if (id <= 0) bad++;
                if (ids[t][k] == -1) ids[t][k] = id;
                else if (ids[t][k] != id) bad++;
            }
            const int own = sideaware_create_kernel(header_text(1000 + t * 100 + round).c_str());
            if (own <= 0) bad++;
            sideaware_tune("stripe_bytes", 4096ll << ((t + round) % 8));
            sideaware_tune("slot_run", (t + round) % 5);
            sideaware_tune("nt_store", (t + round) % 3);             // a compiled-in knob: bumps the generation
            if (sideaware_tune_get("wg_threads") != 256) bad++;
            if (!std::strstr(sideaware_config_block(round % 16), "SA_NUM_XCD")) bad++;
            sideaware_alloc_threshold((size_t)(4 + round % 8) << 20);
            sideaware_free_mapped_thresholds((size_t)16 << 30, (size_t)2 << 30);
            sideaware_reserve_limit(0);
            (void)sideaware_release_unused();
            (void)sideaware_last_error();
            if (round % 10 == t % 10) {
                char log[4096];
                if (sideaware_compile_check(header_text(t).c_str(), round % 2, log, sizeof log) != 0) bad++;
            }
            if (round % 7 == 0) sideaware_clear_error();
        }
    };
    std::vector<std::thread> threads;
    for (int t = 0; t < kThreads; t++) threads.emplace_back(worker, t);
    for (auto& th : threads) th.join();
    for (int t = 1; t < kThreads; t++)
        for (int k = 0; k < kShared; k++)
            if (ids[t][k] != ids[0][k]) bad++;
    // a header seen before still maps to its id; an empty header is the built-in copy
    if (sideaware_create_kernel(header_text(3).c_str()) != ids[0][3] || sideaware_create_kernel("") != 0) bad++;
    std::printf("bad=%d\n", bad.load());
    return bad.load() == 0 ? 0 : 1;
}
