#include "session_planner.hpp"

#include <algorithm>
#include <set>
#include <tuple>

namespace mlel::graph::details {

AllocationPlan allocateIntervals(std::vector<LiveInterval> intervals, const std::vector<UnseenAllocation> &unseen,
                                 const uint64_t alignment) {
    const auto alignUp = [alignment](uint64_t v) { return alignment ? (v + alignment - 1) / alignment * alignment : v; };

    std::sort(intervals.begin(), intervals.end(), [](const LiveInterval &a, const LiveInterval &b) {
        return std::make_tuple(a.first, ~a.size, a.order) < std::make_tuple(b.first, ~b.size, b.order);
    });

    // placed tensors still alive, ordered by (last use, creation order); pooled blocks ordered by (size, age)
    std::set<std::tuple<uint32_t, size_t, uint64_t, uint64_t>> alive;  // last, order, offset, size
    std::set<std::tuple<uint64_t, size_t, uint64_t>> pool;             // size, age, offset
    size_t age = 0;
    AllocationPlan plan;

    for (const LiveInterval &t : intervals) {
        while (!alive.empty() && std::get<0>(*alive.begin()) < t.first) {
            pool.emplace(std::get<3>(*alive.begin()), age++, std::get<2>(*alive.begin()));
            alive.erase(alive.begin());
        }
        uint64_t where;
        const auto fit = pool.lower_bound(std::make_tuple(t.size, size_t(0), uint64_t(0)));
        if (fit != pool.end()) {
            const auto [blockSize, blockAge, blockOffset] = *fit;
            pool.erase(fit);
            where = blockOffset;
            if (blockSize > t.size) pool.emplace(blockSize - t.size, blockAge, blockOffset + t.size);
        } else {
            where = alignUp(plan.memorySize);
            plan.memorySize = where + t.size;
        }
        plan.offsets[t.id] = where;
        alive.emplace(t.last, t.order, where, t.size);
    }
    for (const UnseenAllocation &u : unseen) {
        const uint64_t where = alignUp(plan.memorySize);
        plan.offsets[u.id] = where;
        plan.memorySize = where + u.size;
    }
    plan.memorySize = alignUp(plan.memorySize);
    return plan;
}

}  // namespace mlel::graph::details
