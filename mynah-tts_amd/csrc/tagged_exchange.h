// Values handed from one workgroup to another inside a running kernel, without fences or counters: every 32-bit value
// travels as one 64-bit word {tag << 32 | bits}, written and read with device-scope relaxed atomics (a single 8-byte
// access that bypasses the per-XCD caches), so the data is its own flag: a reader that sees the tag it expects has the
// value that was written with it.  Tags are compared for equality and change with every use of a slot.
//
// Every wait is bounded: a poll that exceeds its spin limit (or sees the abort word set) marks its Waiter dead; the
// kernel then sets the abort word and leaves, every other waiting workgroup runs into the same bound or sees the word,
// so a grid always drains.  The host reports the abort at the next synchronisation.
#pragma once

#include "device_common.h"

namespace mynah {

typedef unsigned long long u64;

__device__ __forceinline__ void put(u64 *p, unsigned tag, float v) {
    __hip_atomic_store(p, ((u64)tag << 32) | (u64)__float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u64 get(const u64 *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ unsigned tag_of(u64 v) { return (unsigned)(v >> 32); }
__device__ __forceinline__ float value_of(u64 v) { return __uint_as_float((unsigned)v); }

struct Waiter {
    unsigned limit;
    unsigned *abort_word;
    bool dead;
};

__device__ __forceinline__ bool give_up(Waiter &w, unsigned &spins) {
    ++spins;
    if (spins > w.limit) return true;
    if ((spins & 255u) == 0u && __hip_atomic_load(w.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) return true;
    return false;
}

// A poll is a request that bypasses the caches, about a microsecond there and back.  Polling one request at a time finds a
// value, on average, half a round trip after it could have; two requests in flight, checked in turn, halve that.
__device__ __forceinline__ void poll_until(const u64 *p, const unsigned tag, Waiter &w) {
    unsigned spins = 0;
    u64 first = get(p), second = get(p);
    while (tag_of(first) != tag) {
        if (give_up(w, spins)) { w.dead = true; break; }
        first = second;
        second = get(p);
    }
}

// n tagged values -> dst (LDS floats, same index), by the whole workgroup, N values per thread and batch.  Every request
// is issued whatever the index (clamped), so that none sits behind a branch.  The batch itself is the poll, and two
// batches are in flight: while one is looked at the next is already on its way, so a value is found a fraction of a
// round trip after it became visible instead of half a round trip (one batch in flight) or a whole one (poll one value,
// then request the batch).  WAIT_FIRST: poll one value of the batch before the first batch is requested -- for batches of
// tens of values, which many workgroups would otherwise request over and over while the producers are still at work.
template <int N, bool WAIT_FIRST>
__device__ __forceinline__ void fetch_tagged(const u64 *src, float *dst, const int n, const unsigned tag, Waiter &w) {
    const int tid = threadIdx.x;
    for (int base = 0; base < n; base += kThreads * N) {
        u64 v[N], next[N];
        unsigned spins = 0;
        if (WAIT_FIRST) {
            int last = base + (N - 1) * kThreads + tid;
            while (last >= n) last -= kThreads;
            if (last >= base) poll_until(src + last, tag, w);
        }
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int i = base + j * kThreads + tid;
            v[j] = get(src + (i < n ? i : n - 1));
        }
        if (!WAIT_FIRST) {
#pragma unroll
            for (int j = 0; j < N; ++j) {
                const int i = base + j * kThreads + tid;
                next[j] = get(src + (i < n ? i : n - 1));
            }
        }
        for (;;) {
            bool all = true;
#pragma unroll
            for (int j = 0; j < N; ++j) {
                const int i = base + j * kThreads + tid;
                all = all && (i >= n || tag_of(v[j]) == tag);
            }
            if (all || w.dead) break;
            if (give_up(w, spins)) { w.dead = true; break; }
#pragma unroll
            for (int j = 0; j < N; ++j) {
                const int i = base + j * kThreads + tid;
                v[j] = WAIT_FIRST ? get(src + (i < n ? i : n - 1)) : next[j];
                if (!WAIT_FIRST) next[j] = get(src + (i < n ? i : n - 1));
            }
        }
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int i = base + j * kThreads + tid;
            if (i < n) dst[i] = value_of(v[j]);
        }
    }
}

// One tagged value that is expected to be there already (it was requested ahead); polls if it is not.
__device__ __forceinline__ float settle(u64 v, const u64 *p, const unsigned tag, Waiter &w) {
    unsigned spins = 0;
    while (tag_of(v) != tag) {
        if (give_up(w, spins)) { w.dead = true; break; }
        v = get(p);
    }
    return value_of(v);
}

}  // namespace mynah
