// Process-wide settings of libfo_hip.so (fo_tune, fo_set_wait_timeout_ms).  Plain C++: any
// thread may set one while other threads are launching, so every knob is an atomic, and a
// launcher reads each knob it needs once, at the top of the launch.
#pragma once

#include <atomic>
#include <string_view>

namespace fo {

struct Knobs {
    std::atomic<int> store_mode{1};             // 0 = cached tile stores, 1 = agent-scope write-through stores (sc1)
    std::atomic<int> release_mode{1};           // 1 = write-through tile stores, acknowledged, then a relaxed atomic; 0 = release-ordered atomic
    std::atomic<int> copy_streaming_stores{2};  // consumer copies: 0 ordinary stores, 1 non-temporal, 2 chosen per launch
    std::atomic<int> wait_timeout_ms{10000};    // bound of every device-side wait
    std::atomic<int> macro_tile{0};             // 0 = chosen per shape, 128 or 256 = forced where the layout tile allows it
};

inline Knobs& knobs() {
    static Knobs k;
    return k;
}

inline int knob(const std::atomic<int>& k) { return k.load(std::memory_order_relaxed); }

// fo_tune: false for an unknown key or a value outside the knob's range.
inline bool set_knob(std::string_view key, int value) {
    Knobs& k = knobs();
    if (key == "store_mode") k.store_mode.store(value ? 1 : 0, std::memory_order_relaxed);
    else if (key == "release_mode") k.release_mode.store(value ? 1 : 0, std::memory_order_relaxed);
    else if (key == "copy_streaming_stores" && value >= 0 && value <= 2)
        k.copy_streaming_stores.store(value, std::memory_order_relaxed);
    else if (key == "macro_tile" && (value == 0 || value == 128 || value == 256))
        k.macro_tile.store(value, std::memory_order_relaxed);
    else return false;
    return true;
}

inline bool set_wait_timeout(int ms) {
    if (ms <= 0) return false;
    knobs().wait_timeout_ms.store(ms, std::memory_order_relaxed);
    return true;
}

}  // namespace fo
