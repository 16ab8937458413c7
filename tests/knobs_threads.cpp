// Host-only harness for tests/test_knobs_tsan.py: the library's process-wide knobs
// (flashoverlap_amd/csrc/fo_knobs.h) written by some threads while others read them the way the
// launchers do.  Built with -fsanitize=thread; --plain-int runs the same traffic over plain ints
// (what the knobs were before they became atomics) so the test can see that the sanitizer would
// have reported it.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "../flashoverlap_amd/csrc/fo_knobs.h"

static int g_plain_store = 1, g_plain_timeout = 10000;   // --plain-int only

int main(int argc, char** argv) {
    const bool plain = argc > 1 && !strcmp(argv[1], "--plain-int");
    constexpr int kWriters = 3, kReaders = 5, kRounds = 20000;
    std::vector<std::thread> threads;
    long long seen[kReaders] = {};
    for (int w = 0; w < kWriters; ++w)
        threads.emplace_back([=] {
            for (int i = 0; i < kRounds; ++i) {
                if (plain) {
                    g_plain_store = i & 1;
                    g_plain_timeout = 1 + (i % 5000);
                } else {
                    fo::set_knob("store_mode", i & 1);
                    fo::set_knob("release_mode", (i >> 1) & 1);
                    fo::set_knob("copy_streaming_stores", i % 3);
                    fo::set_wait_timeout(1 + (i % 5000));
                }
            }
        });
    for (int r = 0; r < kReaders; ++r)
        threads.emplace_back([=, &seen] {
            long long sum = 0;
            for (int i = 0; i < kRounds; ++i) {
                if (plain) {
                    sum += g_plain_store + g_plain_timeout;
                } else {
                    const fo::Knobs& k = fo::knobs();
                    const int store = fo::knob(k.store_mode), rel = fo::knob(k.release_mode);
                    const int copy = fo::knob(k.copy_streaming_stores), ms = fo::knob(k.wait_timeout_ms);
                    if (store < 0 || store > 1 || rel < 0 || rel > 1 || copy < 0 || copy > 2 || ms < 1 || ms > 10000) {
                        printf("knob out of range: %d %d %d %d\n", store, rel, copy, ms);
                        _Exit(3);
                    }
                    sum += store + rel + copy + ms;
                }
            }
            seen[r] = sum;
        });
    for (auto& t : threads) t.join();
    // values outside a knob's range are refused and leave it alone
    if (!plain && (fo::set_knob("copy_streaming_stores", 3) || fo::set_knob("no_such_knob", 1) || fo::set_wait_timeout(0))) {
        printf("a bad setting was accepted\n");
        return 4;
    }
    long long total = 0;
    for (long long s : seen) total += s;
    printf("ok: %d writers, %d readers, %d rounds, checksum %lld\n", kWriters, kReaders, kRounds, total);
    return 0;
}
