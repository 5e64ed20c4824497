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

AllocationPlan allocateLinear(const std::vector<UnseenAllocation> &tensors, const uint64_t alignment) {
    const auto alignUp = [alignment](uint64_t v) { return alignment ? (v + alignment - 1) / alignment * alignment : v; };
    AllocationPlan plan;
    for (const auto &t : tensors) {
        const uint64_t where = alignUp(plan.memorySize);
        plan.offsets[t.id] = where;
        plan.memorySize = alignUp(where + t.size);
    }
    return plan;
}

AllocationPlan allocateBestFit(const std::vector<BestFitTensor> &tensors, const uint64_t alignment) {
    const auto alignUp = [alignment](uint64_t v) { return alignment ? (v + alignment - 1) / alignment * alignment : v; };
    std::map<size_t, const BestFitTensor *> byId;
    for (const auto &t : tensors) byId[t.id] = &t;

    std::vector<const BestFitTensor *> order;
    for (const auto &t : tensors) order.push_back(&t);
    std::stable_sort(order.begin(), order.end(),
                     [](const BestFitTensor *a, const BestFitTensor *b) { return a->size > b->size; });

    AllocationPlan plan;
    std::map<size_t, size_t> blockOf;                // tensor id -> block index
    std::vector<std::vector<size_t>> occupants;      // per block: the tensors placed in it
    for (const BestFitTensor *t : order) {
        // alternatives: safe tensors that are large enough, the closest in size first
        std::vector<const BestFitTensor *> alternatives;
        for (const size_t other : t->safe) {
            const auto it = byId.find(other);
            if (it != byId.end() && it->second->size >= t->size) alternatives.push_back(it->second);
        }
        std::stable_sort(alternatives.begin(), alternatives.end(),
                         [](const BestFitTensor *a, const BestFitTensor *b) { return a->size < b->size; });
        const std::set<size_t> safe(t->safe.begin(), t->safe.end());
        const BestFitTensor *host = nullptr;
        for (const BestFitTensor *alt : alternatives) {
            const auto placed = blockOf.find(alt->id);
            if (placed == blockOf.end()) continue;
            const auto &living = occupants[placed->second];
            if (std::all_of(living.begin(), living.end(), [&](size_t id) { return safe.count(id) != 0; })) {
                host = alt;
                break;
            }
        }
        if (host) {
            blockOf[t->id] = blockOf[host->id];
            plan.offsets[t->id] = plan.offsets[host->id];
            plan.memorySize = std::max(plan.memorySize, plan.offsets[t->id] + t->size);
        } else {
            blockOf[t->id] = occupants.size();
            occupants.emplace_back();
            plan.offsets[t->id] = plan.memorySize;
            plan.memorySize = alignUp(std::max(plan.memorySize, plan.memorySize + t->size));
        }
        occupants[blockOf[t->id]].push_back(t->id);
    }
    return plan;
}

}  // namespace mlel::graph::details
