/*
 * ratchet_hip.h - C ABI of the MI355X (gfx950) device backend for ratchet-core's memory-bound tensor ops.
 *
 * This is the seam a Rust `-sys` crate binds: it takes the place of ratchet-core's wgpu storage layer, of its
 * run-time WGSL kernel generation + dispatch, and of its command-encoder execution.  All citations are paths in
 * huggingface/ratchet (crates/ratchet-core/src/...).
 *
 * Conventions
 *   - status: 0 = ok; > 0 = rt error (enum below), detected before any HIP call; < 0 = -(hipError_t).
 *   - every launch function enqueues on the device's single in-order stream and returns immediately; only
 *     rt_sync, rt_h2d, rt_d2h, rt_event_elapsed_ms block.  Steps therefore run in call order, each seeing the
 *     previous one's writes, as the reference's single compute pass does (executable.rs:33-59).
 *   - shapes are rank-4, left-padded with 1s, exactly what Shape::promote(_, 4) produces (shape.rs:92-96).
 *   - dtype codes: F32 = 0, F16 = 1 as DType::to_u32 (dtype/mod.rs:32-38); BF16 = 2, I32 = 3, U32 = 4 added.
 *   - the caller owns every device pointer; the library allocates nothing inside launch functions except scratch
 *     owned by rt_device (GroupNorm partial statistics, the f16 lookup tables).
 *   - calls on one rt_device must be serialised by the caller (the reference keeps its device behind a RwLock,
 *     gpu/device.rs:20-29).  rt_last_error() is thread-local.
 *   - results follow ratchet's CPU executor (the cpu/ directory), including its f16 rounding points.
 */
#ifndef RATCHET_HIP_H
#define RATCHET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum rt_status {
    RT_OK = 0,
    RT_ERR_NULL_POINTER = 1,   /* a required pointer argument is NULL */
    RT_ERR_DTYPE = 2,          /* dtype code not supported by this op */
    RT_ERR_OP = 3,             /* op code out of range */
    RT_ERR_SHAPE = 4,          /* shapes inconsistent (broadcast rule, concat rule, slice bounds, zero extent) */
    RT_ERR_PERM = 5,           /* permutation is not a permutation of 0..3 (InvariantError::DuplicateDims) */
    RT_ERR_SIZE = 6,           /* element count overflows what the kernels index (2^40 elements) */
    RT_ERR_ARG = 7,            /* other bad argument (n_inputs, dim, groups, mode, elem_bytes, eps) */
    RT_ERR_NULL_DEVICE = 8,    /* rt_device* is NULL */
    RT_ERR_ALIGN = 9,          /* pointer not aligned to its element size */
    RT_ERR_CAPTURE = 10        /* the call cannot run while the device is capturing a graph (or capture state is wrong) */
};

enum rt_dtype { RT_F32 = 0, RT_F16 = 1, RT_BF16 = 2, RT_I32 = 3, RT_U32 = 4 };
/* BinaryOp, ops/binary.rs:19-24 */
enum rt_binary_op { RT_ADD = 0, RT_SUB = 1, RT_MUL = 2, RT_DIV = 3 };
/* UnaryOp, ops/unary.rs:23-38 */
enum rt_unary_op {
    RT_GELU = 0, RT_TANH, RT_EXP, RT_LOG, RT_SIN, RT_COS, RT_ABS, RT_SQRT,
    RT_RELU, RT_FLOOR, RT_CEIL, RT_NEG, RT_SILU, RT_SIGMOID, RT_UNARY_COUNT
};
/* softmax arithmetic: REFERENCE reproduces cpu/softmax.rs (no max subtraction; for 16-bit types the row sum is
 * accumulated sequentially in the element type); STABLE subtracts the row maximum and accumulates in f32. */
enum rt_softmax_mode { RT_SOFTMAX_REFERENCE = 0, RT_SOFTMAX_STABLE = 1 };

typedef struct rt_device rt_device;   /* opaque: HIP device ordinal + one stream + scratch */
typedef struct rt_event rt_event;     /* opaque: a HIP event on a device's stream */

/* ---- device / storage: replaces WgpuDevice (gpu/device.rs:18-30,53-119) and GPUBuffer
 *      (storage/gpu_buffer.rs:20-94,153-158,199-218) ------------------------------------------------------- */
int rt_device_count(int* out);
int rt_device_create(int ordinal, rt_device** out);          /* Device::request_device (device.rs:61-77) */
int rt_device_destroy(rt_device* dev);
int rt_sync(rt_device* dev);                                 /* device.poll(Wait) (tensor.rs:855-856) */
const char* rt_last_error(void);                             /* message for the last non-zero status, thread-local */
const char* rt_status_name(int status);
int rt_malloc(rt_device* dev, size_t bytes, void** dptr);    /* BufferPool::get_or_create (buffer_pool.rs:68-116): sizes
                                                                are rounded up to 4 B, minimum 16 B (:82-93) */
int rt_free(rt_device* dev, void* dptr);                     /* last drop of a PooledGPUBuffer */
/* rt_malloc / rt_free sit on a per-device pool (the role of gpu/pools/buffer_pool.rs:60-112): a freed block is parked
 * and handed out again to a later request of about its size; since every kernel and copy of a device runs on its one
 * in-order stream, neither call synchronises.  rt_pool_trim returns the parked blocks to the driver (it waits for
 * queued work first); rt_pool_begin_pass is the pool's begin_pass (gpu/pools/dynamic_resource_pool.rs:140-190, called
 * by WgpuDevice::begin_pass, gpu/device.rs:275-277, at the top of every resolve, tensor.rs:800): a block that was
 * freed before the previous call and has not been handed out since goes back to the driver, so a block survives
 * one whole pass unused, as the reference's buffers do; when there is no such block the call touches neither the
 * driver nor the stream, and while the device is capturing it frees nothing; rt_pool_stats reports bytes handed out, bytes parked, and how many requests the pool served
 * (hits) or passed to hipMalloc (misses); any out pointer may be NULL. */
int rt_pool_trim(rt_device* dev);
int rt_pool_begin_pass(rt_device* dev);
int rt_pool_stats(rt_device* dev, uint64_t* live_bytes, uint64_t* parked_bytes, uint64_t* hits, uint64_t* misses);
/* the most bytes that were handed out at one time since the last reset (reset != 0 restarts the mark at what is handed
 * out now): what a graph executor checks its activation memory plan against (allocator.rs:266-271 logs the same total) */
int rt_pool_peak(rt_device* dev, uint64_t* peak_live_bytes, int reset);
int rt_memset0(rt_device* dev, void* dptr, size_t bytes);    /* GPUBuffer::zeros (gpu_buffer.rs:29-37) */
int rt_h2d(rt_device* dev, void* dptr, const void* host, size_t bytes);   /* GPUBuffer::from_bytes (:49-59), blocking */
int rt_d2h(rt_device* dev, void* host, const void* dptr, size_t bytes);   /* GPUBuffer::to_cpu (:199-218), blocking */
int rt_d2d(rt_device* dev, void* dst, const void* src, size_t bytes);     /* GPUBuffer::deep_clone (:61-94), async */

/* timing helpers for benchmarks; take the place of the wgpu timestamp-query profiler (gpu/profiler.rs:95-238) */
int rt_event_create(rt_device* dev, rt_event** out);
int rt_event_destroy(rt_event* ev);
int rt_event_record(rt_device* dev, rt_event* ev);
int rt_event_elapsed_ms(rt_event* start, rt_event* stop, float* ms);      /* waits for `stop` */

/* ---- ops: each replaces GPUOperation::compile_gpu (op.rs:280-362) + one dispatch of Executable::dispatch
 *      (executable.rs:33-59) for the op named -------------------------------------------------------------- */

/* Binary (ops/binary.rs:135-182; arithmetic cpu/binary.rs:27-32,85-88): y[i] = a[i] op b[i], equal lengths.
 * y may alias a (the reference's in-place rule, tensor.rs:823-824) or b.  dt: F32, F16, BF16. */
int rt_binary(rt_device* dev, int op, int dt, const void* a, const void* b, void* y, uint64_t numel);

/* Binary with numpy broadcasting resolved at launch instead of a materialised broadcast_to operand
 * (tensor.rs:249-280 inserts Broadcast; this fuses it).  a_shape/b_shape must each broadcast to y_shape
 * (Shape::multi_broadcast, shape.rs:118-136).  Both sides may broadcast.  y must not alias a or b unless that
 * operand already has y_shape. */
int rt_binary_bcast(rt_device* dev, int op, int dt, const void* a, const uint32_t a_shape[4], const void* b,
                    const uint32_t b_shape[4], void* y, const uint32_t y_shape[4]);

/* Unary (ops/unary.rs:234-271; formulas cpu/unary.rs:43-66).  y may alias x.  dt: F32, F16, BF16. */
int rt_unary(rt_device* dev, int op, int dt, const void* x, void* y, uint64_t numel);

/* Cast (ops/cast.rs:113-132; cpu/mod.rs:116-156).  f32<->f16, f32<->bf16 numeric (round to nearest even);
 * f32<->i32/u32 is a bit reinterpretation as in the reference; equal dtypes copy.  Never in place. */
int rt_cast(rt_device* dev, int src_dt, int dst_dt, const void* x, void* y, uint64_t numel);

/* Permute (ops/reindex/permute.rs:22-73; cpu/reindex.rs:43-72): dst_shape[i] = src_shape[perm[i]],
 * dst[idx] = src[idx scattered through perm].  elem_bytes: 2 or 4. */
int rt_permute(rt_device* dev, int elem_bytes, const void* x, void* y, const uint32_t src_shape[4],
               const uint32_t perm[4]);

/* Slice (ops/reindex/slice.rs:22-69; cpu/reindex.rs:92-129): y = x[start : start + dst_shape] in every dim. */
int rt_slice(rt_device* dev, int elem_bytes, const void* x, void* y, const uint32_t src_shape[4],
             const uint32_t start[4], const uint32_t dst_shape[4]);

/* Broadcast (ops/reindex/broadcast.rs:17-82; cpu/reindex.rs:181-222 generic_broadcast): numpy broadcast_to. */
int rt_broadcast(rt_device* dev, int elem_bytes, const void* x, void* y, const uint32_t src_shape[4],
                 const uint32_t dst_shape[4]);

/* Concat (ops/concat.rs:13-158; cpu/mod.rs:158-182): 2..8 inputs, equal shapes except along dim. */
int rt_concat(rt_device* dev, int elem_bytes, int n_inputs, const void* const* xs, const uint32_t (*shapes)[4],
              int dim, void* y);

/* Cache, the KV-cache append (ops/cache.rs:17-105, Tensor::cache tensor.rs:481-486; callers models/phi2/attn.rs:129-135,
 * models/whisper/mha.rs:72-79): dst = cat(cache[.. 0:offset ..], source) along dim, shape = cache shape with
 * dim := offset + source_shape[dim] (:139-147), and source is also written into cache at offset (cache is updated in
 * place; it must not alias dst).  The reference has no CPU implementation; its test's ground truth is that cat. */
int rt_cache(rt_device* dev, int elem_bytes, void* cache, const uint32_t cache_shape[4], const void* source,
             const uint32_t source_shape[4], int dim, uint32_t offset, void* dst);

/* IndexSelect (ops/select.rs:20-79, cpu/mod.rs:44-84; the embedding lookup of every model):
 * dst[left, i, right] = src[left, indices[i], right] along dim, i32 indices on the device.  The reference panics on an
 * index outside [0, src_shape[dim]); here such a row is filled with zeros. */
int rt_index_select(rt_device* dev, int elem_bytes, const void* src, const uint32_t src_shape[4], const int32_t* indices,
                    uint32_t n_indices, int dim, void* dst);

/* IndexSelect from a Q8_0 source (ops/select.rs:107-111,144-161; cpu/mod.rs:86-103 with quant.rs:101-130): the
 * embedding lookup of a quantized model.  `packed` and `scales` are the two segments of the reference's quantized buffer
 * (quant.rs:19-49): numel / 4 words of four signed bytes each, then, from the next multiple of 256 bytes on, numel / 32
 * scales; scale_dt RT_F32 is Q8_0F, RT_F16 is Q8_0H, and dst has that type.  dst[left, i, right] =
 * int8(src[left, indices[i], right]) * scale[group of 32 of that flat source element], one rounding.  numel must be a
 * multiple of 32 and the extents after `dim` a multiple of 4, as in the reference; rows for indices outside the source
 * are zero (the reference's kernel clamps the index, its CPU path panics). */
int rt_index_select_q8_0(rt_device* dev, int scale_dt, const uint32_t* packed, const void* scales, const uint32_t src_shape[4],
                         const int32_t* indices, uint32_t n_indices, int dim, void* dst);

/* IndexWrite (ops/index_write.rs:14-111): dst, in place, receives the src_numel elements of src as one flat run that
 * starts at the element write_start addresses (D[offset(write_start) + i] = S[i], :96-104).  A run that would leave dst
 * is rejected (the reference's kernel has no bound). */
int rt_index_write(rt_device* dev, int elem_bytes, void* dst, const uint32_t dst_shape[4], const void* src, uint64_t src_numel,
                   const uint32_t write_start[4]);

/* RoPE on [B, H, S, D] (ops/rope.rs:17-95; arithmetic of cpu/rope.rs:23-143): the first `dim` columns are rotated in
 * halves by theta[p, i] = (offset + p) * base^(-i / (dim/2)), the rest pass through.  y may be x (the reference's GPU
 * kernel is in-place only).  F16/BF16 are widened, rotated in f32 and rounded once, which is what the models'
 * x.full().rope(..).cast(dt) yields; the reference's CPU path implements F32 only. */
int rt_rope(rt_device* dev, int dt, const void* x, void* y, const uint32_t shape[4], uint32_t dim, float base, uint32_t offset);

/* Softmax over the last dimension (ops/softmax.rs:14-39,183-199; cpu/softmax.rs:22-42): rows x cols, contiguous.
 * y may alias x (the reference kernel is in-place only, ops/softmax.rs:47-49).  dt: F32, F16, BF16. */
int rt_softmax(rt_device* dev, int dt, const void* x, void* y, uint64_t rows, uint32_t cols, int mode);

/* LayerNorm over the last dimension (ops/norm/mod.rs:17-91; cpu/norm.rs:91-147); bias may be NULL.
 * eps is converted to the element type inside (T::from(eps), cpu/norm.rs:128). */
int rt_layer_norm(rt_device* dev, int dt, const void* x, const void* scale, const void* bias, void* y,
                  uint64_t rows, uint32_t cols, float eps);

/* RMSNorm over the last dimension (cpu/norm.rs:185-213). */
int rt_rms_norm(rt_device* dev, int dt, const void* x, const void* scale, void* y, uint64_t rows, uint32_t cols,
                float eps);

/* GroupNorm on [B, C, L] with per-channel scale/bias (either may be NULL): the semantics of
 * torch.nn.functional.group_norm, which is the reference test's ground truth (ops/norm/groupnorm.rs:24-31);
 * the reference's own CPU implementation is a no-op (cpu/norm.rs:215-219). */
int rt_group_norm(rt_device* dev, int dt, const void* x, const void* scale, const void* bias, void* y, uint32_t B,
                  uint32_t C, uint32_t L, uint32_t groups, float eps);

/* rt_group_norm for callers that cannot allocate (code recorded into a HIP graph, tight serving loops, harnesses that
 * forbid hipMalloc).  No counterpart in the reference.  Same arguments, same results bit for bit, but the partial
 * statistics of groups that are split over several blocks go to a fixed 256 KiB array that lives in the library's code
 * object (one copy per GPU, held until the process ends) instead of the device's growable buffer, and the call never
 * reaches hipMalloc / hipFree.  A problem whose partials do not fit (more than about 10 900 (batch, group) pairs)
 * returns RT_ERR_SIZE.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU
 * (two rt_devices with the same ordinal, or a replaying graph next to an eager call) race; calls on one rt_device are
 * ordered by its stream.  Nothing in the array has to start at zero: each launch writes every partial it reads. */
int rt_group_norm_static(rt_device* dev, int dt, const void* x, const void* scale, const void* bias, void* y, uint32_t B,
                         uint32_t C, uint32_t L, uint32_t groups, float eps);

/* scores.add(mask).softmax(last dim) in the tensors' own arithmetic (the 16-bit sum is rounded as the separate add
 * rounds it, then Softmax's contract applies), result bit-identical to rt_binary_bcast(RT_ADD) followed by rt_softmax
 * but the sum never reaches memory when the shape allows (x / y / mask on 16-byte boundaries, a mask that covers whole
 * trailing dims and repeats over the leading ones; f16 or bf16 in reference mode: rows of whole 16-byte vectors or of
 * 192 to 4095 columns of any length; f32, and the stable mode of any type: rows of whole 16-byte vectors up to 65536
 * columns).  Each mask extent is 1 or the scores' extent; y may be x.
 * Binary: ops/binary.rs:27-119 via tensor.rs:249-280; Softmax: ops/softmax.rs:17-73, cpu/softmax.rs:22-42. */
int rt_softmax_masked(rt_device* dev, int dt, const void* x, const uint32_t x_shape[4], const void* mask,
                      const uint32_t mask_shape[4], void* y, int mode);

/* ---- Replayable launch lists ---------------------------------------------------------------------------------------
 * The reference encodes every compiled op of a graph into one command buffer and submits it once
 * (Executable::dispatch, executable.rs:33-59).  The counterpart here is a HIP graph: between rt_capture_begin and
 * rt_capture_end every launch the rt_* ops would enqueue on the device's stream is recorded instead of run;
 * rt_graph_launch replays the whole list with one submission, in stream order with everything else on the device.
 * While capturing, calls that wait for the device or go to the driver for memory return RT_ERR_CAPTURE: rt_sync,
 * rt_h2d, rt_d2h, rt_pool_trim, event calls, an rt_malloc the pool cannot serve, and the first use of an op that builds
 * a lookup table or grows scratch (run the sequence once eagerly first).  A graph holds raw pointers: every buffer it
 * touches must stay allocated while the graph is in use. */
typedef struct rt_graph rt_graph;
int rt_capture_begin(rt_device* dev);
int rt_capture_end(rt_device* dev, rt_graph** out);
int rt_graph_launch(rt_device* dev, rt_graph* graph);
int rt_graph_destroy(rt_graph* graph);

/* ---- Caller patterns in one pass --------------------------------------------------------------------------------
 * The models wrap every 16-bit norm, softmax and activation in full() ... cast(dt): widen to f32, run the f32 op,
 * round back.  These entry points produce what that op sequence produces (same rounding points: 16-bit add for the
 * mask, f32 arithmetic inside, one rounding at the end) without the f32 tensors ever reaching memory.  io_dt is
 * RT_F16 or RT_BF16. */

/* x.full().layer_norm(w, b, eps).cast(dt) (kind 0) / x.full().rms_norm(w, eps).cast(dt) (kind 1): LayerNorm and
 * RMSNorm modules, crates/ratchet-nn/src/norm.rs:35-44 and :61-70.  scale/bias are f32 (Norm::check_dtypes makes them
 * match the widened input); bias may be NULL and is ignored for kind 1. */
int rt_norm_via_f32(rt_device* dev, int kind, int io_dt, const void* x, const float* scale, const float* bias, void* y,
                    uint64_t rows, uint32_t cols, float eps);

/* scores.add(mask.cast(dt)).full().softmax(3).cast(dt): crates/ratchet-models/src/phi3/attn.rs:143-153,
 * phi2/attn.rs:143-150, whisper/mha.rs:115-124.  mask may be NULL (no add); otherwise each mask extent is 1 or the
 * scores' extent.  mode as rt_softmax. */
int rt_softmax_via_f32(rt_device* dev, int io_dt, const void* x, const uint32_t x_shape[4], const void* mask,
                       const uint32_t mask_shape[4], void* y, int mode);

/* x.full().<op>().cast(dt) for any rt_unary op (activations: crates/ratchet-models/src/phi2/mlp.rs, whisper/residual_block.rs). */
int rt_unary_via_f32(rt_device* dev, int op, int io_dt, const void* x, void* y, uint64_t numel);

/* up.mul(gate.full().<op>().cast(dt)) with gate and up given as row-strided [rows, cols] views (strides in elements),
 * so the two slices of the fused projection need no copies: crates/ratchet-models/src/phi3/mlp.rs:32-38. */
int rt_gated_mul_via_f32(rt_device* dev, int op, int io_dt, const void* gate, uint64_t gate_row_stride, const void* up,
                         uint64_t up_row_stride, void* y, uint64_t rows, uint32_t cols);

#ifdef __cplusplus
}
#endif
#endif
