/*
 * ratchet_host.h - C view of the C++ host mirror of ratchet-core's lazy Tensor API (ratchet_amd/csrc/host/ratchet.hpp),
 * exported by libratchet_host.so.  It exists so that non-C++ callers (the Python parity tests) can drive the same graph
 * building and resolve() code path; the device work itself goes through ratchet_hip.h.
 *
 * Handles are opaque and owned by the caller: release every rth_tensor / rth_device that a call returned.
 * Builders return NULL on error; other calls return non-zero.  rth_last_error_kind() is the invariant that failed
 * (the reference's InvariantError / assert it corresponds to, e.g. "BroadcastingFailed", "DuplicateDims",
 * "DTypeMismatch"), rth_last_error() the full message; both are thread-local.
 */
#ifndef RATCHET_HOST_H
#define RATCHET_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rth_device rth_device;
typedef struct rth_tensor rth_tensor;
typedef struct rth_executable rth_executable;

const char* rth_last_error(void);
const char* rth_last_error_kind(void);

rth_device* rth_device_request(int ordinal);                          /* Device::request_device (device.rs:61-77) */
void rth_device_release(rth_device* dev);
/* {bytes handed out, bytes parked in the pool, requests served by the pool, requests passed to the driver} (rt_pool_stats) */
int rth_pool_stats(rth_device* dev, uint64_t out[4]);
int rth_pool_peak(rth_device* dev, uint64_t* peak_live_bytes, int reset);   /* rt_pool_peak of the device */

/* Tensor::from_data + to(device) (tensor.rs:553-571,874-892); dt codes as in ratchet_hip.h */
rth_tensor* rth_from_host(rth_device* dev, const void* data, int rank, const uint64_t* shape, int dt);
/* Tensor::from_quantized (tensor.rs:618-628): dt 5 = Q8_0F, 6 = Q8_0H (codes that continue ratchet_hip.h's); data is the
 * quantized buffer as the reference lays it out (quant.rs:19-49: numel signed bytes packed four to a word, padded to 256
 * bytes, then numel / 32 scales of f32 / f16, padded to 256 bytes: rth_storage_bytes in all).  Such a tensor can only be
 * the source of rth_index_select (ops/select.rs:107-111), whose result has the scales' type. */
rth_tensor* rth_from_quantized(rth_device* dev, const void* data, int rank, const uint64_t* shape, int dt);
uint64_t rth_storage_bytes(int rank, const uint64_t* shape, int dt);
/* shape-only constant without storage: graph building and its errors can be exercised without a GPU; cannot be resolved */
rth_tensor* rth_placeholder(int rank, const uint64_t* shape, int dt);
void rth_release(rth_tensor* t);
int rth_rank(const rth_tensor* t);
int rth_shape(const rth_tensor* t, uint64_t* dims /* rank entries */);
int rth_dtype(const rth_tensor* t);
int rth_resolved(const rth_tensor* t);
const char* rth_op_name(const rth_tensor* t);

/* op builders (tensor.rs:294-495): record a node, run nothing */
rth_tensor* rth_binary(const rth_tensor* a, const rth_tensor* b, int op);         /* add/sub/mul/div = 0..3 */
rth_tensor* rth_unary(const rth_tensor* x, int op);                               /* UnaryOp order, gelu = 0 */
rth_tensor* rth_cast(const rth_tensor* x, int dst_dt);
rth_tensor* rth_layer_norm(const rth_tensor* x, const rth_tensor* weight, const rth_tensor* bias /* nullable */, float eps);
rth_tensor* rth_rms_norm(const rth_tensor* x, const rth_tensor* weight, float eps);
rth_tensor* rth_group_norm(const rth_tensor* x, size_t num_groups, const rth_tensor* weight, const rth_tensor* bias, float eps);
rth_tensor* rth_softmax(const rth_tensor* x, size_t dim, int mode);
rth_tensor* rth_slice(const rth_tensor* x, int n, const uint64_t* starts, const uint64_t* ends);
rth_tensor* rth_view(const rth_tensor* x, int rank, const uint64_t* shape);
rth_tensor* rth_cat(const rth_tensor* const* xs, int n, size_t dim);
/* one-launch replacements of full() -> norm / softmax / activation -> cast(dt) at resolve(); on by default */
void rth_set_pattern_fusion(int on);
rth_tensor* rth_cache(const rth_tensor* cache, const rth_tensor* source, size_t dim, size_t offset);   /* tensor.rs:481-486 */
rth_tensor* rth_rope(const rth_tensor* x, size_t dim, float base, size_t offset);                       /* tensor.rs:392-397 */
rth_tensor* rth_index_select(const rth_tensor* x, const rth_tensor* indices, size_t dim);               /* tensor.rs:497-502 */
rth_tensor* rth_index_write(const rth_tensor* dst, const rth_tensor* src, int rank, const uint64_t* write_start);   /* tensor.rs:504-510 */
rth_tensor* rth_permute(const rth_tensor* x, int n, const uint64_t* dims);
rth_tensor* rth_broadcast_to(const rth_tensor* x, int rank, const uint64_t* shape);

int rth_resolve(rth_tensor* t);                                        /* Tensor::resolve (tensor.rs:861-863) */
int rth_to_host(const rth_tensor* t, void* out);                       /* to(&Device::CPU) (tensor.rs:957-975) */
long rth_last_resolve_launches(const rth_tensor* t);                   /* kernels launched by the last rth_resolve(t) */
int rth_execution_order(const rth_tensor* t, uint64_t* ids, int cap);  /* ids in execution order; returns the count */
/* The memory plan rth_resolve(t) would follow (BufferAllocator::greedy_by_size with in-place leasing,
 * gpu/buffer_allocator/allocator.rs:141-271), without allocating or launching anything: the sizes of the shared objects,
 * and per launch, in execution order, four values {tensor id, bytes, object, source}: object is an index into
 * object_bytes, -1 for an allocation of its own (t itself and tensors still visible outside the graph) or -2 when the
 * op runs in place in a buffer that exists already; source is the tensor whose allocation the result lives in.
 * Returns the number of launches (entries beyond entry_cap are not written), -1 on error. */
int rth_memory_plan(const rth_tensor* t, uint64_t* object_bytes, int object_cap, int* n_objects, int64_t* entries, int entry_cap);
uint64_t rth_id(const rth_tensor* t);

/* The compiled form of a graph: what the reference's Executable is to a command buffer (executable.rs:13-59), this is
 * to a HIP graph.  rth_compile resolves t (it runs the graph once) and records the same launches, on buffers assigned
 * once by the memory plan, for replay; rth_executable_dispatch replays them with one submission (fewer than eight
 * launches: call by call, which costs less than a graph launch; wait != 0: returns after completion, like rth_resolve).  Shapes, offsets and buffer addresses are fixed at compile time: new input data
 * goes into the graph's constant tensors with rth_update_from_host, results are read from t with rth_to_host.  The
 * executable keeps every buffer of the graph alive; release it with rth_executable_release.  NULL on error. */
rth_executable* rth_compile(rth_tensor* t);
int rth_executable_dispatch(rth_executable* exe, int wait);
long rth_executable_launches(const rth_executable* exe);              /* kernels per dispatch */
uint64_t rth_executable_held_bytes(const rth_executable* exe);        /* device memory of the intermediates it keeps */
void rth_executable_release(rth_executable* exe);
/* overwrite the contents of a tensor that has storage (numel * element size bytes are read from data) */
int rth_update_from_host(rth_tensor* t, const void* data);

#ifdef __cplusplus
}
#endif
#endif
