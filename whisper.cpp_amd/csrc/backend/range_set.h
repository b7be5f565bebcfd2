// Address ranges of device memory that hold no value: results that a launch folded into its consumer, or stored only
// as the activation image of the product that follows.  The graph walker decides such things from the readers it can
// see in the graph it was handed; ggml's scheduler may hand a graph over in pieces (ggml_graph_view slices,
// ggml/src/ggml-backend.cpp:1252, and node ranges with an eval callback, :1398-1440), and a reader in a later piece
// would then find memory nobody wrote.  The walker records every result it leaves unwritten here, every write takes
// its bytes out again, and every read — a node's source, a download, a copy — asks first: a stale read becomes a
// failed graph (or a poisoned download) with a log line instead of a silently wrong result.
//
// Plain C++, no HIP and no ggml: the class is also compiled into the test harness, whose selftest drives it.
#pragma once

#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <vector>

struct mi355x_range_set {
    struct range { uintptr_t lo, hi; char name[48]; };     // [lo, hi)

    // `name`: the tensor, for the log line
    void add(const void * begin, size_t size, const char * name) {
        if (!size) return;
        const uintptr_t lo = (uintptr_t) begin, hi = lo + size;
        std::lock_guard<std::mutex> lock(m);
        for (range & r : ranges) if (r.lo <= lo && hi <= r.hi) return;          // already inside one
        range r; r.lo = lo; r.hi = hi;
        strncpy(r.name, name ? name : "", sizeof(r.name) - 1); r.name[sizeof(r.name) - 1] = 0;
        ranges.push_back(r);
        count.store(ranges.size(), std::memory_order_release);
    }

    // [begin, begin + size) now holds values: ranges inside it go, ranges it cuts are trimmed or split
    void written(const void * begin, size_t size) {
        if (!size || count.load(std::memory_order_acquire) == 0) return;
        const uintptr_t lo = (uintptr_t) begin, hi = lo + size;
        std::lock_guard<std::mutex> lock(m);
        const size_t n = ranges.size();
        for (size_t i = 0; i < n && i < ranges.size();) {
            range & r = ranges[i];
            if (hi <= r.lo || r.hi <= lo) { ++i; continue; }
            if (lo <= r.lo && r.hi <= hi) { ranges[i] = ranges.back(); ranges.pop_back(); continue; }   // (the swapped-in one is looked at next)
            if (r.lo < lo && hi < r.hi) {                                       // a hole in the middle: two pieces
                range tail = r; tail.lo = hi;
                r.hi = lo;
                ranges.push_back(tail);
            } else if (r.lo < lo) r.hi = lo; else r.lo = hi;
            ++i;
        }
        count.store(ranges.size(), std::memory_order_release);
    }

    // does [begin, begin + size) touch memory that holds no value?  `name` (48 bytes) receives the tensor recorded there
    bool stale(const void * begin, size_t size, char * name = nullptr) {
        if (!size || count.load(std::memory_order_acquire) == 0) return false;
        const uintptr_t lo = (uintptr_t) begin, hi = lo + size;
        std::lock_guard<std::mutex> lock(m);
        for (const range & r : ranges) if (lo < r.hi && r.lo < hi) {
            if (name) memcpy(name, r.name, sizeof(r.name));
            return true;
        }
        return false;
    }

    void clear() {
        std::lock_guard<std::mutex> lock(m);
        ranges.clear();
        count.store(0, std::memory_order_release);
    }

    size_t size() const { return count.load(std::memory_order_acquire); }

private:
    std::mutex          m;
    std::vector<range>  ranges;
    std::atomic<size_t> count{0};
};
