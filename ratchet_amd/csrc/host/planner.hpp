// Activation memory planning for one resolve(): which intermediates of the graph may share a device allocation.
//
// Follows ratchet-core's BufferAllocator (crates/ratchet-core/src/gpu/buffer_allocator/allocator.rs):
//   * determine_tensor_source (:141-162): an op that runs in place works in the buffer of its first source, so a chain
//     of such ops is one allocation, owned by the chain's first tensor ("true source");
//   * calculate_usage_records (:168-204): per true source, the index of the launch that produces it and of the last
//     launch that reads it or anything leased from it;
//   * greedy_by_size (:208-271, after arXiv 2001.03288): records sorted by size, largest first; a record goes into an
//     existing shared object if none of the records already in that object is alive at the same time (intervals
//     [producer, last_consumer] that touch count as overlapping), into the last such object found, else a new object
//     of the record's size is created.
// Differences, all on the safe side: ties in size keep execution order (the reference sorts unstably out of a hash map,
// so its choice among equals varies from run to run); a tensor that something outside the graph can still see, and
// the tensor being resolved, are "pinned": they get an allocation of their own, because the caller reads them after
// the resolve (the reference hands the caller a handle to a shared object that later launches have overwritten).
// Host code only; knows nothing about devices.
#pragma once
#include <cstddef>
#include <cstdint>
#include <unordered_map>
#include <vector>

namespace ratchet {
namespace planner {

// one launch of the resolve, in execution order
struct Step {
    uint64_t id = 0;                 // the tensor it produces
    size_t bytes = 0;                // size of that tensor
    std::vector<uint64_t> reads;     // tensors whose buffers it reads (steps of this plan or tensors that exist already)
    int inplace = -1;                // index into reads of the operand whose buffer the result takes over, -1: none
    bool pinned = false;             // visible after the resolve: never shares
};

struct Record {                      // TensorUsageRecord (tensor_usage_record.rs:8-15)
    uint64_t id = 0;                 // the true source
    size_t producer = 0, last_consumer = 0, bytes = 0;
    int object = -1;                 // shared object it was put into
};

enum : int { OWN_BUFFER = -1, EXTERNAL = -2 };   // Plan::object_of values that are not shared objects

struct Plan {
    std::vector<size_t> object_bytes;                  // shared objects in creation order
    std::vector<size_t> object_last_use;               // last step index that touches each object
    std::unordered_map<uint64_t, int> object_of;       // per step id: shared object, OWN_BUFFER (pinned), or EXTERNAL
                                                       // (runs in place in a buffer that existed before the resolve)
    std::unordered_map<uint64_t, uint64_t> source_of;  // per step id: the true source whose allocation it lives in
    std::vector<Record> records;                       // in the order they were placed (largest first)
    size_t shared_bytes() const {
        size_t s = 0;
        for (size_t b : object_bytes) s += b;
        return s;
    }
};

Plan greedy_by_size(const std::vector<Step>& steps);

}  // namespace planner
}  // namespace ratchet
