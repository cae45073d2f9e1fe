#include "planner.hpp"

#include <algorithm>

namespace ratchet {
namespace planner {

Plan greedy_by_size(const std::vector<Step>& steps) {
    Plan plan;
    std::unordered_map<uint64_t, size_t> step_of;
    for (size_t i = 0; i < steps.size(); i++) step_of[steps[i].id] = i;

    // allocator.rs:141-162: walk up while the producer runs in place
    auto true_source = [&](uint64_t id) {
        for (;;) {
            auto it = step_of.find(id);
            if (it == step_of.end()) return id;                       // exists already: a root of the chain
            const Step& s = steps[it->second];
            if (s.inplace < 0) return id;
            id = s.reads[(size_t)s.inplace];
        }
    };
    for (const Step& s : steps) plan.source_of[s.id] = true_source(s.id);

    // a chain is pinned when any tensor in it is
    std::unordered_map<uint64_t, bool> chain_pinned;
    for (const Step& s : steps)
        if (s.pinned) chain_pinned[plan.source_of[s.id]] = true;

    // allocator.rs:168-204: reverse walk; the first reader met is the last consumer
    std::unordered_map<uint64_t, Record> recs;
    for (size_t k = steps.size(); k-- > 0;) {
        const Step& s = steps[k];
        for (uint64_t r : s.reads) {
            const uint64_t ts = true_source(r);
            if (!step_of.count(ts)) continue;                         // not produced by this resolve
            if (!recs.count(ts)) {
                Record rec;
                rec.id = ts;
                rec.last_consumer = k;
                rec.bytes = steps[step_of[ts]].bytes;
                recs[ts] = rec;
            }
        }
        auto it = recs.find(s.id);
        if (it != recs.end()) it->second.producer = k;
    }
    std::vector<Record> order;
    for (const Step& s : steps) {                                     // execution order, then a stable sort: deterministic ties
        auto it = recs.find(s.id);
        if (it != recs.end() && !chain_pinned.count(s.id)) order.push_back(it->second);
    }
    std::stable_sort(order.begin(), order.end(), [](const Record& a, const Record& b) { return a.bytes > b.bytes; });

    // allocator.rs:216-250
    for (Record& rec : order) {
        int best = -1;
        for (int obj = 0; obj < (int)plan.object_bytes.size(); obj++) {
            bool suitable = true;
            for (const Record& other : plan.records) {
                if (other.object != obj) continue;
                const size_t max_first = std::max(rec.producer, other.producer);
                const size_t min_last = std::min(rec.last_consumer, other.last_consumer);
                if (max_first <= min_last) {
                    suitable = false;
                    break;
                }
            }
            if (suitable) best = obj;                                 // no break: the last suitable object wins, as in the reference
        }
        if (best < 0) {
            best = (int)plan.object_bytes.size();
            plan.object_bytes.push_back(rec.bytes);
            plan.object_last_use.push_back(0);
        }
        rec.object = best;
        plan.object_last_use[(size_t)best] = std::max(plan.object_last_use[(size_t)best], rec.last_consumer);
        plan.records.push_back(rec);
    }

    // allocator.rs:252-264 (leases) and the pinned / external cases
    std::unordered_map<uint64_t, int> object_of_source;
    for (const Record& r : plan.records) object_of_source[r.id] = r.object;
    for (const Step& s : steps) {
        const uint64_t ts = plan.source_of[s.id];
        if (!step_of.count(ts)) plan.object_of[s.id] = EXTERNAL;
        else if (object_of_source.count(ts)) plan.object_of[s.id] = object_of_source[ts];
        else plan.object_of[s.id] = OWN_BUFFER;                       // pinned, or read by nobody
    }
    return plan;
}

}  // namespace planner
}  // namespace ratchet
