// C++ host mirror of ratchet-core's lazy Tensor API for the memory-bound ops, above the C ABI of libratchet_hip.so.
//
// Same names, argument meaning and error behaviour as crates/ratchet-core/src/tensor.rs: op builders validate shapes and
// dtypes and only record a node (tensor.rs:249-510), resolve() walks the graph in topological order (tensor.rs:696-740)
// and launches one kernel per node on the device's single stream (the role of resolve_gpu + Executable::dispatch,
// tensor.rs:795-859, executable.rs:33-59), reusing the first source's buffer when the op supports in-place execution and
// nothing else holds that source (tensor.rs:823-824).  Where the reference panics (assert!) or returns Err, this throws
// ratchet::Error with the same invariant name.
//
// Deliberate differences from the reference, all on paths the reference gets wrong or does not have:
//   * a binary op whose two operands both need broadcasting works (tensor.rs:266-272 only broadcasts one side);
//   * a Broadcast node consumed only by a Binary node is fused into the binary kernel instead of being materialised;
//   * softmax accepts only the last dimension (the reference's kernels silently assume it, ops/softmax.rs:259-283);
//   * a failing kernel launch fails resolve() (the reference logs a warning and skips the op, tensor.rs:826-832).
#pragma once
#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

struct rt_device;

namespace ratchet {

struct Error : std::runtime_error {
    std::string kind;       // "BroadcastingFailed", "DTypeMismatch", "DuplicateDims", "RankMismatch", "ShapeMismatch", ...
    Error(const std::string& k, const std::string& msg) : std::runtime_error(k + ": " + msg), kind(k) {}
};

// dtype/mod.rs:12-23.  Of the quantized types only Q8_0 is here, and only as the source of index_select (the embedding
// table of a quantized model, ops/select.rs:107-111): every other op rejects it.
enum class DType { F32 = 0, F16 = 1, BF16 = 2, I32 = 3, U32 = 4, Q8_0F = 5, Q8_0H = 6 };
size_t size_of(DType dt);                                     // bytes per element; 0 for a quantized type
bool is_float(DType dt);
bool is_quantized(DType dt);
DType activation_dt(DType dt);                                // dtype/mod.rs:99-107: what a quantized tensor dequantizes to
const char* as_str(DType dt);

// shape.rs: rank <= 4 on every path here
class Shape {
  public:
    Shape() {}
    Shape(std::initializer_list<size_t> d) : dims_(d) {}
    explicit Shape(std::vector<size_t> d) : dims_(std::move(d)) {}
    size_t rank() const { return dims_.size(); }
    size_t numel() const;
    size_t operator[](size_t i) const { return dims_[i]; }
    size_t& operator[](size_t i) { return dims_[i]; }
    const std::vector<size_t>& dims() const { return dims_; }
    bool is_scalar() const;                                   // shape.rs:67-69: all dims are 1
    bool operator==(const Shape& o) const { return dims_ == o.dims_; }
    bool operator!=(const Shape& o) const { return dims_ != o.dims_; }
    static Shape promote(const Shape& s, size_t rank);        // shape.rs:92-96: left-pad with 1s
    static bool multi_broadcast(const std::vector<const Shape*>& shapes, Shape* out);   // shape.rs:118-136
    std::string to_string() const;

  private:
    std::vector<size_t> dims_;
};
std::vector<ptrdiff_t> contiguous_strides(const Shape& s);    // Strides::from(&Shape), strides.rs:85-96
// bytes of a tensor's storage: numel * size_of, or for Q8_0 the two segments of dtype/blocks.rs:73-81 (numel signed
// bytes, then numel / 32 scales of the activation type, each segment rounded up to 256 bytes)
size_t storage_bytes(const Shape& shape, DType dt);

enum class BinaryOp { Add = 0, Sub, Mul, Div };
enum class UnaryOp { Gelu = 0, Tanh, Exp, Log, Sin, Cos, Abs, Sqrt, Relu, Floor, Ceil, Neg, Silu, Sigmoid };
enum class SoftmaxMode { Reference = 0, Stable = 1 };

// gpu/device.rs: one device, one stream; cloned by handle, compared by identity
class Device {
  public:
    static Device request(int ordinal = 0);                   // Device::request_device (device.rs:61-77)
    rt_device* raw() const { return inner_ ? inner_->raw : nullptr; }
    bool operator==(const Device& o) const { return inner_ == o.inner_; }
    void sync() const;

  private:
    struct Inner {
        rt_device* raw = nullptr;
        ~Inner();
    };
    std::shared_ptr<Inner> inner_;
};

// storage/gpu_buffer.rs: ref-counted device allocation, released on last drop
struct Buffer {
    Device device;
    void* ptr = nullptr;
    size_t bytes = 0;
    Buffer(const Device& d, size_t n);
    ~Buffer();
    Buffer(const Buffer&) = delete;
    Buffer& operator=(const Buffer&) = delete;
};

// resolve() replaces the models' full() -> norm / softmax / activation -> cast(dt) sequences on 16-bit tensors (and
// phi3's gated multiply) by one launch each when the intermediate tensors are visible to nobody else.  On by default.
void set_pattern_fusion(bool on);
bool pattern_fusion();

class Tensor;
struct Node;                                                  // LazyOp + operands (op.rs:14-31)

// What resolve() would allocate for the intermediates of a graph (gpu/buffer_allocator/allocator.rs:208-271, see
// planner.hpp): one entry per launch, in execution order.
struct MemoryPlan {
    struct Entry {
        uint64_t id = 0;          // the tensor the launch produces
        size_t bytes = 0;
        int object = -1;          // index into object_bytes; -1: an allocation of its own (the resolved tensor, tensors
                                  // visible outside the graph); -2: works in place in a buffer that exists already
        uint64_t source = 0;      // the tensor whose allocation it lives in (itself unless it runs in place)
    };
    std::vector<size_t> object_bytes;
    std::vector<Entry> entries;
};

// The compiled form of a graph: the reference's Executable is the ordered list of compiled ops that dispatch() encodes
// into one command buffer and submits once (executable.rs:13-59, built by resolve_gpu, tensor.rs:795-859).  Here the
// list is a HIP graph over buffers assigned once by the memory plan: dispatch() is one graph launch, whatever the number
// of kernels (a list of fewer than eight launches is re-issued call by call instead, which is cheaper than a graph
// launch: no graph building, pattern matching, planning or allocation either way).  Shapes, offsets (cache, rope, index_write) and buffer addresses are fixed at compile(); new input data
// goes into the graph's constant tensors with Tensor::update_from_host, and the output tensor's buffer is rewritten by
// every dispatch.  The executable keeps every buffer of the graph alive, intermediates included.  Like the tensors it is
// for one thread at a time (a call-by-call dispatch lends the graph's nodes their buffers for its duration).
class Executable {
  public:
    Executable() {}
    // replays all launches of the graph in order; wait = return after completion, as resolve() does (tensor.rs:855-856)
    void dispatch(bool wait = true) const;
    size_t launches() const;                                  // kernels per dispatch
    size_t held_bytes() const;                                // device memory of the intermediates this executable keeps

  private:
    struct Inner;
    std::shared_ptr<Inner> inner_;
    friend struct Resolver;
};

class Tensor {
  public:
    Tensor() {}
    // Tensor::from_data + to(device): upload `numel * size_of(dt)` bytes (tensor.rs:553-571, 874-892)
    static Tensor from_host(const void* data, const Shape& shape, DType dt, const Device& device);
    // Tensor::from_quantized (tensor.rs:618-628): `data` is the quantized buffer as quantize() lays it out (quant.rs:19-49),
    // storage_bytes(shape, dt) bytes; numel must be a multiple of 32
    static Tensor from_quantized(const void* data, const Shape& shape, DType dt, const Device& device);
    static Tensor zeros(const Shape& shape, DType dt, const Device& device);
    // A constant without storage or device: lets graph building (shape/dtype rules, errors, execution order) run on a
    // machine without a GPU.  resolve() on a graph that contains one fails.
    static Tensor placeholder(const Shape& shape, DType dt);

    const Shape& shape() const;
    DType dt() const;
    size_t rank() const { return shape().rank(); }
    size_t numel() const { return shape().numel(); }
    const Device& device() const;
    bool resolved() const;
    uint64_t id() const;
    const char* op_name() const;

    // tensor.rs:294-298
    Tensor add(const Tensor& other) const { return binary(other, BinaryOp::Add); }
    Tensor sub(const Tensor& other) const { return binary(other, BinaryOp::Sub); }
    Tensor mul(const Tensor& other) const { return binary(other, BinaryOp::Mul); }
    Tensor div(const Tensor& other) const { return binary(other, BinaryOp::Div); }
    // tensor.rs:300-313
    Tensor gelu() const { return unary(UnaryOp::Gelu); }
    Tensor tanh() const { return unary(UnaryOp::Tanh); }
    Tensor exp() const { return unary(UnaryOp::Exp); }
    Tensor log() const { return unary(UnaryOp::Log); }
    Tensor sin() const { return unary(UnaryOp::Sin); }
    Tensor cos() const { return unary(UnaryOp::Cos); }
    Tensor abs() const { return unary(UnaryOp::Abs); }
    Tensor sqrt() const { return unary(UnaryOp::Sqrt); }
    Tensor relu() const { return unary(UnaryOp::Relu); }
    Tensor floor() const { return unary(UnaryOp::Floor); }
    Tensor ceil() const { return unary(UnaryOp::Ceil); }
    Tensor neg() const { return unary(UnaryOp::Neg); }
    Tensor sigmoid() const { return unary(UnaryOp::Sigmoid); }
    Tensor silu() const { return unary(UnaryOp::Silu); }
    Tensor binary(const Tensor& other, BinaryOp op) const;
    Tensor unary(UnaryOp op) const;

    Tensor cast(DType dst) const;                             // tensor.rs:315-324: same dtype returns self
    Tensor full() const { return cast(DType::F32); }          // tensor.rs:327-329
    Tensor half() const { return cast(DType::F16); }          // tensor.rs:332-334
    Tensor group_norm(size_t num_groups, const Tensor& weight, const Tensor* bias, float eps) const;   // tensor.rs:336-348
    Tensor layer_norm(const Tensor& weight, const Tensor* bias, float eps) const;                        // tensor.rs:350-361
    Tensor rms_norm(const Tensor& weight, float eps) const;                                              // tensor.rs:363-369
    Tensor softmax(size_t dim, SoftmaxMode mode = SoftmaxMode::Reference) const;                         // tensor.rs:385-390
    Tensor slice(const std::vector<std::pair<size_t, size_t>>& ranges) const;                            // tensor.rs:426-449
    Tensor view(const Shape& shape) const;                                                               // tensor.rs:454-461
    static Tensor cat(const std::vector<Tensor>& tensors, size_t dim);                                   // tensor.rs:463-470
    Tensor permute(const std::vector<size_t>& dims) const;                                               // tensor.rs:472-479
    // self is the cache (tensor.rs:481-486): result = cat(self[.. :offset ..], source) along dim; resolve() also writes
    // source into the cache's storage at offset
    Tensor cache(const Tensor& source, size_t dim, size_t offset) const;
    Tensor broadcast_to(const Shape& shape) const;                                                       // tensor.rs:488-495
    Tensor rope(size_t dim, float base, size_t offset) const;                                            // tensor.rs:392-397
    Tensor index_select(const Tensor& indices, size_t dim) const;                                        // tensor.rs:497-502
    // self is the destination (tensor.rs:504-510): resolve() writes src into self's storage as a flat run from write_start
    Tensor index_write(const Tensor& src, const std::vector<size_t>& write_start) const;

    // tensor.rs:861-863: runs every unresolved node this tensor depends on; returns after completion
    Tensor resolve() const;
    // resolve() that also keeps the launch list: runs the graph once (so this tensor is resolved on return), then records
    // the same launches on the same buffers into an Executable.  An op is not run in place in a buffer that existed
    // before the call (a replay would apply it to its own result); cache and index_write still update their destination.
    // A tensor that is resolved already cannot be compiled (there is nothing left to record).
    Executable compile() const;
    // to(&Device::CPU) + to_vec (tensor.rs:957-975): blocking download of the resolved tensor
    void to_host(void* out) const;
    // overwrite the contents of a resolved tensor (numel * size_of(dt) bytes), e.g. an input of a compiled graph
    void update_from_host(const void* data) const;
    // number of kernel launches the last resolve() of this tensor issued (for tests)
    size_t last_resolve_launches() const;

    // the memory plan resolve() would follow; works on placeholder graphs (nothing is allocated or launched)
    MemoryPlan memory_plan() const;

    // unit-test hook for the topological order (tensor.rs:696-740): ids in execution order
    std::vector<uint64_t> execution_order_ids() const;

  private:
    explicit Tensor(std::shared_ptr<Node> n) : node_(std::move(n)) {}
    std::shared_ptr<Node> node_;
    friend struct Node;
    friend struct Resolver;
};

}  // namespace ratchet
