// The work tables of the many-stream attention launches and the device code that fills them.
#pragma once

#include "kernels.h"

namespace mynah {

constexpr int kFoldUnit = 0x7fff;   // unit number of a table entry that folds instead of attending

// Work table of the PACKED builds, one entry per workgroup index of the attention grid: which (head, stream, unit) the
// workgroup takes and where that stream's cache is.  Self-attention: first the Q+K and V roles of every stream's new row,
// head-major; then, per head, the cache chunks that exist, stream by stream.  Each of the two lists is cut into eight
// contiguous ranges, one per XCD (workgroup i runs on XCD i % 8), so a head's weight slice is fetched by at most two XCDs.
// Behind the chunks that exist: one fold entry per (stream, head) when the launch folds its own partials.  Workgroups
// numbered past all of these get code -1: they are the last ones of the grid and leave after this one read.  Written once
// per pass through the layers by extra workgroups of the kernel that starts the pass (k_step_begin for a decode step; the
// local frame's begin and token-choice kernels for its sixteen passes), so the tables cost no launch of their own.
// A workgroup takes `group` consecutive chunks of its stream and head: the smallest number with which every workgroup of the
// launch is resident at once (`budget` = the chip's workgroup slots for this kernel less the other roles).  A second round
// of workgroups would start when the first ends and run its whole dependent chain again, some 5 us, for a fifth of the work.
// uniform_length >= 0: every stream's self cache holds that many rows (the slot table's own lengths are then not read: a
// kernel that advances them in the same launch can still write the next pass's tables).
__device__ inline StepItem make_item(const StepSlots &slots, int uniform_length, int batch, int heads, bool is_self, int wg, int epoch, bool with_fold,
                                     int budget) {
    // Every stream's unit count first, from places of the table known at compile time: the loops below then run on registers.
    // (Read inside the loops, a length was one dependent fetch from the kernel's arguments per iteration, two dozen in a row.)
    int units[kMaxBatch];
#pragma unroll
    for (int s = 0; s < kMaxBatch; ++s) {
        const int len = !is_self ? slots.memory_length[s] : uniform_length >= 0 ? uniform_length : slots.length[s];
        const int live = (len + kStepUnitRows - 1) / kStepUnitRows;
        units[s] = s < batch ? (is_self ? live : max(live, 1)) : 0;
    }
    const StepItem dead{nullptr, nullptr, 0, -1, 0, 0};
    // chunks per workgroup: the smallest group size with which the launch's chunk workgroups are at most `budget`
    int all_chunks = 0;
#pragma unroll
    for (int s = 0; s < kMaxBatch; ++s) all_chunks += units[s];
    const int group = max(1, (heads * all_chunks + budget - 1) / max(budget, 1));
    int chunk_items = 0;   // groups per head
#pragma unroll
    for (int s = 0; s < kMaxBatch; ++s) chunk_items += (units[s] + group - 1) / group;
    int head, b = 0, unit = 0;
    const int producers = is_self ? 2 * batch * heads : 0;
    const int producer_grid = 8 * ((producers + 7) / 8);
    if (wg < producer_grid) {
        // the new row's Q+K and V roles, head-major, before everything that waits for them
        const int per_xcd = producer_grid / 8;
        const int xcd = wg & 7, slot = wg >> 3;
        const int p = xcd * per_xcd + slot;
        if (p >= producers) return dead;
        head = p / (2 * batch);
        const int r = p - head * 2 * batch;
        b = r >> 1;
        unit = r & 1;
    } else {
        const int w2 = wg - producer_grid;
        const int items = heads * chunk_items;
        const int per_xcd = (items + 7) / 8;
        const int xcd = w2 & 7, slot = w2 >> 3;
        const int item = xcd * per_xcd + slot;
        if (w2 >= 8 * per_xcd) {
            // behind every workgroup that attends: one fold per (stream, head)
            const int f = w2 - 8 * per_xcd;
            if (!with_fold || f >= heads * batch) return dead;
            head = f / batch;
            b = f - head * batch;
            unit = kFoldUnit;
        } else {
            if (item >= items) return dead;
            head = item / chunk_items;
            const int r = item - head * chunk_items;
            int before = 0;
#pragma unroll
            for (int s = 0; s < kMaxBatch; ++s) {
                const int n = (units[s] + group - 1) / group;   // (no units beyond the batch: nothing matches there)
                if (r >= before && r < before + n) { b = s; unit = r - before + (is_self ? 2 : 0); }
                before += n;
            }
        }
    }
    StepItem it;
    it.k = is_self ? slots.self_k[b] : const_cast<float *>(slots.cross_k[b]);
    it.v = is_self ? slots.self_v[b] : const_cast<float *>(slots.cross_v[b]);
    it.length = !is_self ? slots.memory_length[b] : uniform_length >= 0 ? uniform_length : slots.length[b];
    it.code = head | (b << 8) | (unit << 16);
    it.epoch = epoch;
    it.group = group;
    return it;
}

// Entry i of the two tables laid end to end (self first); callers run it for i = 0 .. self_entries + cross_entries - 1.
__device__ inline void write_step_item(const StepItemTables &t, const StepSlots &slots, int uniform_length, int epoch, int i) {
    if (i < t.self_entries)
        t.self_items[i] = make_item(slots, uniform_length, t.batch, t.heads, true, i, epoch, t.with_fold != 0, t.self_budget);
    else if (i - t.self_entries < t.cross_entries)
        t.cross_items[i - t.self_entries] =
            make_item(slots, uniform_length, t.batch, t.cross_heads, false, i - t.self_entries, epoch, t.with_fold != 0, t.cross_budget);
}

}  // namespace mynah
