// C wrappers around the C++ host mirror (declared in include/ratchet_host.h): handles, error capture, no logic.
#include <cstring>
#include <string>
#include <vector>

#include "../../../include/ratchet_host.h"
#include "ratchet.hpp"
#include "../../../include/ratchet_hip.h"

using namespace ratchet;

struct rth_device {
    Device dev;
};
struct rth_tensor {
    Tensor t;
};
struct rth_executable {
    Executable exe;
};

static thread_local std::string g_msg, g_kind;

static void capture(const std::exception& e) {
    g_msg = e.what();
    const Error* re = dynamic_cast<const Error*>(&e);
    g_kind = re ? re->kind : "Exception";
}
template <typename F> static rth_tensor* build(F f) {
    try {
        return new rth_tensor{f()};
    } catch (const std::exception& e) {
        capture(e);
        return nullptr;
    }
}
static Shape make_shape(int rank, const uint64_t* dims) {
    std::vector<size_t> d(dims, dims + (rank > 0 ? rank : 0));
    return Shape(d);
}

extern "C" {

const char* rth_last_error(void) { return g_msg.c_str(); }
const char* rth_last_error_kind(void) { return g_kind.c_str(); }

rth_device* rth_device_request(int ordinal) {
    try {
        return new rth_device{Device::request(ordinal)};
    } catch (const std::exception& e) {
        capture(e);
        return nullptr;
    }
}
void rth_device_release(rth_device* dev) { delete dev; }
int rth_pool_stats(rth_device* dev, uint64_t out[4]) {
    return rt_pool_stats(dev->dev.raw(), &out[0], &out[1], &out[2], &out[3]);
}

int rth_pool_peak(rth_device* dev, uint64_t* peak_live_bytes, int reset) { return rt_pool_peak(dev->dev.raw(), peak_live_bytes, reset); }

rth_tensor* rth_from_host(rth_device* dev, const void* data, int rank, const uint64_t* shape, int dt) {
    return build([&] { return Tensor::from_host(data, make_shape(rank, shape), (DType)dt, dev->dev); });
}
rth_tensor* rth_from_quantized(rth_device* dev, const void* data, int rank, const uint64_t* shape, int dt) {
    return build([&] { return Tensor::from_quantized(data, make_shape(rank, shape), (DType)dt, dev->dev); });
}
uint64_t rth_storage_bytes(int rank, const uint64_t* shape, int dt) { return (uint64_t)storage_bytes(make_shape(rank, shape), (DType)dt); }
rth_tensor* rth_placeholder(int rank, const uint64_t* shape, int dt) {
    return build([&] { return Tensor::placeholder(make_shape(rank, shape), (DType)dt); });
}
void rth_release(rth_tensor* t) { delete t; }
int rth_rank(const rth_tensor* t) { return (int)t->t.rank(); }
int rth_shape(const rth_tensor* t, uint64_t* dims) {
    for (size_t i = 0; i < t->t.rank(); i++) dims[i] = t->t.shape()[i];
    return 0;
}
int rth_dtype(const rth_tensor* t) { return (int)t->t.dt(); }
int rth_resolved(const rth_tensor* t) { return t->t.resolved() ? 1 : 0; }
const char* rth_op_name(const rth_tensor* t) { return t->t.op_name(); }
uint64_t rth_id(const rth_tensor* t) { return t->t.id(); }

rth_tensor* rth_binary(const rth_tensor* a, const rth_tensor* b, int op) {
    return build([&] {
        if (op < 0 || op > 3) throw Error("InvalidOp", "binary op " + std::to_string(op));
        return a->t.binary(b->t, (BinaryOp)op);
    });
}
rth_tensor* rth_unary(const rth_tensor* x, int op) {
    return build([&] {
        if (op < 0 || op > 13) throw Error("InvalidOp", "unary op " + std::to_string(op));
        return x->t.unary((UnaryOp)op);
    });
}
rth_tensor* rth_cast(const rth_tensor* x, int dst_dt) {
    return build([&] {
        if (dst_dt < 0 || dst_dt > 4) throw Error("UnsupportedDType", std::to_string(dst_dt));
        return x->t.cast((DType)dst_dt);
    });
}
rth_tensor* rth_layer_norm(const rth_tensor* x, const rth_tensor* w, const rth_tensor* b, float eps) {
    return build([&] { return x->t.layer_norm(w->t, b ? &b->t : nullptr, eps); });
}
rth_tensor* rth_rms_norm(const rth_tensor* x, const rth_tensor* w, float eps) {
    return build([&] { return x->t.rms_norm(w->t, eps); });
}
rth_tensor* rth_group_norm(const rth_tensor* x, size_t groups, const rth_tensor* w, const rth_tensor* b, float eps) {
    return build([&] { return x->t.group_norm(groups, w->t, b ? &b->t : nullptr, eps); });
}
rth_tensor* rth_softmax(const rth_tensor* x, size_t dim, int mode) {
    return build([&] { return x->t.softmax(dim, mode == 1 ? SoftmaxMode::Stable : SoftmaxMode::Reference); });
}
rth_tensor* rth_slice(const rth_tensor* x, int n, const uint64_t* starts, const uint64_t* ends) {
    return build([&] {
        std::vector<std::pair<size_t, size_t>> r;
        for (int i = 0; i < n; i++) r.push_back({(size_t)starts[i], (size_t)ends[i]});
        return x->t.slice(r);
    });
}
rth_tensor* rth_view(const rth_tensor* x, int rank, const uint64_t* shape) {
    return build([&] { return x->t.view(make_shape(rank, shape)); });
}
rth_tensor* rth_cat(const rth_tensor* const* xs, int n, size_t dim) {
    return build([&] {
        std::vector<Tensor> ts;
        for (int i = 0; i < n; i++) ts.push_back(xs[i]->t);
        return Tensor::cat(ts, dim);
    });
}
void rth_set_pattern_fusion(int on) { ratchet::set_pattern_fusion(on != 0); }
rth_tensor* rth_cache(const rth_tensor* cache, const rth_tensor* source, size_t dim, size_t offset) {
    return build([&] { return cache->t.cache(source->t, dim, offset); });
}
rth_tensor* rth_rope(const rth_tensor* x, size_t dim, float base, size_t offset) {
    return build([&] { return x->t.rope(dim, base, offset); });
}
rth_tensor* rth_index_select(const rth_tensor* x, const rth_tensor* indices, size_t dim) {
    return build([&] { return x->t.index_select(indices->t, dim); });
}
rth_tensor* rth_index_write(const rth_tensor* dst, const rth_tensor* src, int rank, const uint64_t* write_start) {
    return build([&] {
        std::vector<size_t> ws(write_start, write_start + rank);
        return dst->t.index_write(src->t, ws);
    });
}
rth_tensor* rth_permute(const rth_tensor* x, int n, const uint64_t* dims) {
    return build([&] {
        std::vector<size_t> d(dims, dims + (n > 0 ? n : 0));
        return x->t.permute(d);
    });
}
rth_tensor* rth_broadcast_to(const rth_tensor* x, int rank, const uint64_t* shape) {
    return build([&] { return x->t.broadcast_to(make_shape(rank, shape)); });
}

int rth_resolve(rth_tensor* t) {
    try {
        t->t.resolve();
        return 0;
    } catch (const std::exception& e) {
        capture(e);
        return 1;
    }
}
int rth_to_host(const rth_tensor* t, void* out) {
    try {
        t->t.to_host(out);
        return 0;
    } catch (const std::exception& e) {
        capture(e);
        return 1;
    }
}
long rth_last_resolve_launches(const rth_tensor* t) { return (long)t->t.last_resolve_launches(); }
int rth_execution_order(const rth_tensor* t, uint64_t* ids, int cap) {
    const std::vector<uint64_t> v = t->t.execution_order_ids();
    for (int i = 0; i < cap && i < (int)v.size(); i++) ids[i] = v[i];
    return (int)v.size();
}
int rth_memory_plan(const rth_tensor* t, uint64_t* object_bytes, int object_cap, int* n_objects, int64_t* entries, int entry_cap) {
    try {
        const MemoryPlan p = t->t.memory_plan();
        if (n_objects) *n_objects = (int)p.object_bytes.size();
        for (int i = 0; i < object_cap && i < (int)p.object_bytes.size(); i++) object_bytes[i] = p.object_bytes[i];
        for (int i = 0; i < entry_cap && i < (int)p.entries.size(); i++) {
            entries[4 * i + 0] = (int64_t)p.entries[i].id;
            entries[4 * i + 1] = (int64_t)p.entries[i].bytes;
            entries[4 * i + 2] = p.entries[i].object;
            entries[4 * i + 3] = (int64_t)p.entries[i].source;
        }
        return (int)p.entries.size();
    } catch (const std::exception& e) {
        capture(e);
        return -1;
    }
}

rth_executable* rth_compile(rth_tensor* t) {
    try {
        return new rth_executable{t->t.compile()};
    } catch (const std::exception& e) {
        capture(e);
        return nullptr;
    }
}
int rth_executable_dispatch(rth_executable* exe, int wait) {
    try {
        exe->exe.dispatch(wait != 0);
        return 0;
    } catch (const std::exception& e) {
        capture(e);
        return 1;
    }
}
long rth_executable_launches(const rth_executable* exe) { return (long)exe->exe.launches(); }
uint64_t rth_executable_held_bytes(const rth_executable* exe) { return (uint64_t)exe->exe.held_bytes(); }
void rth_executable_release(rth_executable* exe) { delete exe; }
int rth_update_from_host(rth_tensor* t, const void* data) {
    try {
        t->t.update_from_host(data);
        return 0;
    } catch (const std::exception& e) {
        capture(e);
        return 1;
    }
}

}  // extern "C"
