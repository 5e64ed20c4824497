// Session-memory planning for the intermediates of a data graph: live-range interval allocation.
//
// Observable behaviour equals the reference's details::allocateIntervals
// (graph/interval_memory_planner.cpp:170-215) and is pinned by the vectors of its unit tests
// (tests/graph/interval_memory_planner_tests.cpp:17-106):
//   - tensors are placed in the order (first use ascending, size descending, creation order ascending);
//   - before a tensor is placed, every placed tensor whose last use is earlier than this tensor's first use gives
//     its block back to a pool of free blocks;
//   - a tensor takes the smallest pooled block that is large enough (ties: the block released first; what is left of
//     a split block stays in the pool under the released block's age); neighbouring pooled blocks are never merged;
//   - otherwise the arena grows at its aligned end;
//   - tensors no operator touches ("unseen") are appended, each with storage of its own.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <vector>

namespace mlel::graph::details {

struct LiveInterval {
    size_t id;       // key under which the offset is reported
    uint32_t first;  // first and last execution step that touch the tensor
    uint32_t last;
    uint64_t size;   // bytes, already rounded to the alignment
    size_t order;    // creation order (tie break)
};

struct UnseenAllocation {
    size_t id;
    uint64_t size;
};

struct AllocationPlan {
    uint64_t memorySize{0};
    std::map<size_t, uint64_t> offsets;
};

AllocationPlan allocateIntervals(std::vector<LiveInterval> intervals, const std::vector<UnseenAllocation> &unseen,
                                 uint64_t alignment);

// The reference's two other planners (graph/memory_planner.cpp), selected there by VMEL_MEMORY_PLANNER.
//
// Linear (memory_planner.cpp:52-94): every tensor gets an aligned slot of its own, in the given order.
AllocationPlan allocateLinear(const std::vector<UnseenAllocation> &tensors, uint64_t alignment);

// BestFit (memory_planner.cpp:100-382): tensors are taken by size, largest first (ties: given order).  A tensor may
// share the block of an already placed tensor B when B is at least as large and every tensor already living in
// that block is in the tensor's safe-to-reuse set; among such blocks the one of the smallest B wins (ties: order of
// `safe`).  Otherwise it goes to the end of the arena, which is then rounded up to the alignment.
// `safe[i]` lists the ids that may share memory with tensor i (the relation is symmetric).
struct BestFitTensor {
    size_t id;
    uint64_t size;
    std::vector<size_t> safe;
};
AllocationPlan allocateBestFit(const std::vector<BestFitTensor> &tensors, uint64_t alignment);

}  // namespace mlel::graph::details
