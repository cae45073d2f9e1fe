// Implementation of the C++ host mirror (see ratchet.hpp).  Host code only: it talks to the GPU through the C ABI of
// libratchet_hip.so and contains no arithmetic on tensor data.
#include "ratchet.hpp"
#include "planner.hpp"

#include <algorithm>
#include <atomic>
#include <sstream>
#include <unordered_map>
#include <unordered_set>

#include "../../../include/ratchet_hip.h"

namespace ratchet {

// ------------------------------------------------------------------------------------------------------------ basics
size_t size_of(DType dt) { return is_quantized(dt) ? 0 : (dt == DType::F16 || dt == DType::BF16) ? 2 : 4; }
bool is_float(DType dt) { return dt == DType::F32 || dt == DType::F16 || dt == DType::BF16; }
bool is_quantized(DType dt) { return dt == DType::Q8_0F || dt == DType::Q8_0H; }
DType activation_dt(DType dt) { return dt == DType::Q8_0F ? DType::F32 : dt == DType::Q8_0H ? DType::F16 : dt; }
static size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
size_t storage_bytes(const Shape& shape, DType dt) {
    const size_t n = shape.numel();
    if (!is_quantized(dt)) return n * size_of(dt);
    return align256(n) + align256(n / 32 * size_of(activation_dt(dt)));
}
const char* as_str(DType dt) {
    switch (dt) {
        case DType::F32: return "F32";
        case DType::F16: return "F16";
        case DType::BF16: return "BF16";
        case DType::I32: return "I32";
        case DType::Q8_0F: return "Q8_0F";
        case DType::Q8_0H: return "Q8_0H";
        default: return "U32";
    }
}

size_t Shape::numel() const {
    size_t n = 1;
    for (size_t d : dims_) n *= d;
    return n;
}
bool Shape::is_scalar() const {
    return std::all_of(dims_.begin(), dims_.end(), [](size_t d) { return d == 1; });
}
Shape Shape::promote(const Shape& s, size_t rank) {
    std::vector<size_t> d(s.dims_);
    while (d.size() < rank) d.insert(d.begin(), 1);
    return Shape(d);
}
bool Shape::multi_broadcast(const std::vector<const Shape*>& shapes, Shape* out) {
    size_t max_rank = 0;
    for (const Shape* s : shapes) max_rank = std::max(max_rank, s->rank());
    std::vector<size_t> dims(max_rank, 1);
    for (size_t i = 0; i < max_rank; i++) {
        size_t cur = 1;
        for (const Shape* s : shapes) {
            const size_t len = s->rank();
            const size_t d = i < len ? (*s)[len - i - 1] : 1;
            if (d != 1) {
                if (cur != 1 && d != cur) return false;
                cur = d;
            }
        }
        dims[max_rank - 1 - i] = cur;
    }
    *out = Shape(dims);
    return true;
}
std::string Shape::to_string() const {
    std::ostringstream o;
    o << "[";
    for (size_t i = 0; i < dims_.size(); i++) o << (i ? "," : "") << dims_[i];
    o << "]";
    return o.str();
}
std::vector<ptrdiff_t> contiguous_strides(const Shape& s) {
    std::vector<ptrdiff_t> st(s.rank());
    ptrdiff_t acc = 1;
    for (size_t i = s.rank(); i-- > 0;) {
        st[i] = acc;
        acc *= (ptrdiff_t)s[i];
    }
    return st;
}

static void check_rt(int status, const char* what) {
    if (status != 0) throw Error(status < 0 ? "DeviceError" : rt_status_name(status), std::string(what) + ": " + rt_last_error());
}

// ------------------------------------------------------------------------------------------------------------ device
Device::Inner::~Inner() {
    if (raw) rt_device_destroy(raw);
}
Device Device::request(int ordinal) {
    Device d;
    d.inner_ = std::make_shared<Inner>();
    check_rt(rt_device_create(ordinal, &d.inner_->raw), "rt_device_create");
    return d;
}
void Device::sync() const { check_rt(rt_sync(raw()), "rt_sync"); }

Buffer::Buffer(const Device& d, size_t n) : device(d), bytes(n) { check_rt(rt_malloc(d.raw(), n, &ptr), "rt_malloc"); }
Buffer::~Buffer() {
    if (ptr) rt_free(device.raw(), ptr);
}

// ------------------------------------------------------------------------------------------------------------ graph
enum class Kind { Const, Binary, Unary, Cast, Permute, Slice, Broadcast, Concat, Cache, RoPE, IndexSelect, IndexWrite, Softmax, LayerNorm, RMSNorm, GroupNorm, View };

struct Node {
    uint64_t id = 0;
    Kind kind = Kind::Const;
    Shape shape;
    DType dt = DType::F32;
    Device device;
    std::vector<Tensor> srcs;                 // Operation::srcs(), in bind order
    BinaryOp bop = BinaryOp::Add;
    UnaryOp uop = UnaryOp::Gelu;
    std::vector<size_t> dims;                 // permute dims
    std::vector<std::pair<size_t, size_t>> ranges;
    size_t dim = 0;                           // concat / softmax
    size_t groups = 0;
    float eps = 0.0f;
    bool has_bias = false;
    SoftmaxMode mode = SoftmaxMode::Reference;
    std::shared_ptr<Buffer> storage;          // Some(..) once resolved
    size_t last_launches = 0;

    static Node* of(const Tensor& t) { return t.node_.get(); }
    static long holders(const Tensor& t) { return t.node_.use_count(); }
    static Tensor wrap(std::shared_ptr<Node> n) { return Tensor(std::move(n)); }
};

static std::atomic<uint64_t> g_next_id{1};

static std::shared_ptr<Node> new_node(Kind k, const Shape& shape, DType dt, const Device& dev) {
    auto n = std::make_shared<Node>();
    n->id = g_next_id++;
    n->kind = k;
    n->shape = shape;
    n->dt = dt;
    n->device = dev;
    return n;
}

static void require_same_device(const Tensor& a, const Tensor& b) {
    if (!(a.device() == b.device())) throw Error("DeviceMismatch", "operands live on different devices");
}
// every op but index_select computes on plain element types
static void require_plain(const Tensor& t, const char* who) {
    if (is_quantized(t.dt())) throw Error("UnsupportedDType", std::string(who) + " on a quantized tensor (" + as_str(t.dt()) + ")");
}
static void require_rank4(const Shape& s, const char* who) {
    if (s.rank() == 0 || s.rank() > 4) throw Error("RankMismatch", std::string(who) + ": rank " + std::to_string(s.rank()) + " (1..4 supported)");
}

const Shape& Tensor::shape() const { return node_->shape; }
DType Tensor::dt() const { return node_->dt; }
const Device& Tensor::device() const { return node_->device; }
bool Tensor::resolved() const { return node_ && node_->storage != nullptr; }
uint64_t Tensor::id() const { return node_->id; }
size_t Tensor::last_resolve_launches() const { return node_->last_launches; }
const char* Tensor::op_name() const {
    switch (node_->kind) {
        case Kind::Const: return "Const";
        case Kind::Binary: {
            static const char* n[] = {"Add", "Sub", "Mul", "Div"};
            return n[(int)node_->bop];
        }
        case Kind::Unary: {
            static const char* n[] = {"Gelu", "Tanh", "Exp", "Log", "Sin", "Cos", "Abs", "Sqrt", "Relu", "Floor", "Ceil", "Neg", "Silu", "Sigmoid"};
            return n[(int)node_->uop];
        }
        case Kind::Cast: return "Cast";
        case Kind::Permute: return "Permute";
        case Kind::Slice: return "Slice";
        case Kind::Broadcast: return "Broadcast";
        case Kind::Concat: return "Concat";
        case Kind::Cache: return "Cache";
        case Kind::RoPE: return "RoPE";
        case Kind::IndexSelect: return "IndexSelect";
        case Kind::IndexWrite: return "IndexWrite";
        case Kind::Softmax: return "Softmax";
        case Kind::View: return "View";
        default: return "Norm";
    }
}

Tensor Tensor::from_quantized(const void* data, const Shape& shape, DType dt, const Device& device) {
    require_rank4(shape, "from_quantized");
    if (!is_quantized(dt)) throw Error("UnsupportedDType", std::string("from_quantized takes a quantized type, got ") + as_str(dt));
    if (shape.numel() % 32 != 0) throw Error("ShapeMismatch", "a Q8_0 tensor holds whole groups of 32 elements (quant.rs:20-21)");
    auto n = new_node(Kind::Const, shape, dt, device);
    const size_t bytes = storage_bytes(shape, dt);
    n->storage = std::make_shared<Buffer>(device, bytes);
    check_rt(rt_h2d(device.raw(), n->storage->ptr, data, bytes), "rt_h2d");
    return Tensor(n);
}

Tensor Tensor::from_host(const void* data, const Shape& shape, DType dt, const Device& device) {
    require_rank4(shape, "from_host");
    if (is_quantized(dt)) throw Error("UnsupportedDType", "quantized data comes in through from_quantized");
    auto n = new_node(Kind::Const, shape, dt, device);
    const size_t bytes = shape.numel() * size_of(dt);
    n->storage = std::make_shared<Buffer>(device, bytes);
    check_rt(rt_h2d(device.raw(), n->storage->ptr, data, bytes), "rt_h2d");
    return Tensor(n);
}
Tensor Tensor::zeros(const Shape& shape, DType dt, const Device& device) {
    require_rank4(shape, "zeros");
    if (is_quantized(dt)) throw Error("UnsupportedDType", as_str(dt));
    auto n = new_node(Kind::Const, shape, dt, device);
    const size_t bytes = shape.numel() * size_of(dt);
    n->storage = std::make_shared<Buffer>(device, bytes);
    check_rt(rt_memset0(device.raw(), n->storage->ptr, bytes), "rt_memset0");
    return Tensor(n);
}

Tensor Tensor::placeholder(const Shape& shape, DType dt) {
    require_rank4(shape, "placeholder");
    return Tensor(new_node(Kind::Const, shape, dt, Device()));
}

// impl_binary_op! (tensor.rs:249-280) + Binary guards (ops/binary.rs:135-145)
Tensor Tensor::binary(const Tensor& other, BinaryOp op) const {
    require_same_device(*this, other);
    if (dt() != other.dt()) throw Error("DTypeMismatch", std::string("expected ") + as_str(dt()) + ", got " + as_str(other.dt()));
    if (!is_float(dt())) throw Error("UnsupportedDType", as_str(dt()));
    Shape out;
    if (!Shape::multi_broadcast({&shape(), &other.shape()}, &out))
        throw Error("BroadcastingFailed", shape().to_string() + " vs " + other.shape().to_string());
    Tensor lhs = *this, rhs = other;
    if (lhs.shape() != out) lhs = lhs.broadcast_to(out);       // the reference stops after the first one that needs it
    if (rhs.shape() != out) rhs = rhs.broadcast_to(out);
    auto n = new_node(Kind::Binary, out, dt(), device());
    n->bop = op;
    n->srcs = {lhs, rhs};
    return Tensor(n);
}

Tensor Tensor::unary(UnaryOp op) const {
    if (!is_float(dt())) throw Error("UnsupportedDType", as_str(dt()));
    auto n = new_node(Kind::Unary, shape(), dt(), device());
    n->uop = op;
    n->srcs = {*this};
    return Tensor(n);
}

Tensor Tensor::cast(DType dst) const {
    if (dt() == dst) return *this;
    const DType s = dt();
    const bool numeric = (s == DType::F32 && (dst == DType::F16 || dst == DType::BF16)) ||
                         ((s == DType::F16 || s == DType::BF16) && dst == DType::F32);
    const bool reinterpret = (s == DType::F32 && (dst == DType::I32 || dst == DType::U32)) ||
                             ((s == DType::I32 || s == DType::U32) && dst == DType::F32);
    if (!numeric && !reinterpret) throw Error("UnsupportedCast", std::string(as_str(s)) + " -> " + as_str(dst));   // unimplemented!() in cpu_cast
    auto n = new_node(Kind::Cast, shape(), dst, device());
    n->srcs = {*this};
    return Tensor(n);
}

static void check_norm_operands(const Tensor& x, const Tensor& w, const Tensor* b, size_t expect) {
    if (x.rank() < 2) throw Error("RankMismatch", "norm input needs rank >= 2");            // NormOp::check_shapes
    if (!is_float(x.dt())) throw Error("UnsupportedDType", as_str(x.dt()));
    if (w.dt() != x.dt()) throw Error("DTypeMismatch", std::string("expected ") + as_str(x.dt()) + ", got " + as_str(w.dt()));
    if (b && b->dt() != x.dt()) throw Error("DTypeMismatch", std::string("expected ") + as_str(x.dt()) + ", got " + as_str(b->dt()));
    if (w.numel() != expect || (b && b->numel() != expect))
        throw Error("ShapeMismatch", "scale/bias must hold " + std::to_string(expect) + " elements");
}

Tensor Tensor::layer_norm(const Tensor& weight, const Tensor* bias, float eps) const {
    check_norm_operands(*this, weight, bias, shape()[rank() - 1]);
    auto n = new_node(Kind::LayerNorm, shape(), dt(), device());
    n->eps = eps;
    n->has_bias = bias != nullptr;
    n->srcs = {*this, weight};
    if (bias) n->srcs.push_back(*bias);
    return Tensor(n);
}
Tensor Tensor::rms_norm(const Tensor& weight, float eps) const {
    check_norm_operands(*this, weight, nullptr, shape()[rank() - 1]);
    auto n = new_node(Kind::RMSNorm, shape(), dt(), device());
    n->eps = eps;
    n->srcs = {*this, weight};
    return Tensor(n);
}
Tensor Tensor::group_norm(size_t num_groups, const Tensor& weight, const Tensor* bias, float eps) const {
    if (rank() < 2) throw Error("RankMismatch", "group_norm input needs rank >= 2");
    const size_t C = shape()[1];
    if (num_groups == 0 || C % num_groups != 0)
        throw Error("InvalidGroups", std::to_string(C) + " channels do not split into " + std::to_string(num_groups) + " groups");
    check_norm_operands(*this, weight, bias, C);
    auto n = new_node(Kind::GroupNorm, shape(), dt(), device());
    n->eps = eps;
    n->groups = num_groups;
    n->has_bias = bias != nullptr;
    n->srcs = {*this, weight};
    if (bias) n->srcs.push_back(*bias);
    return Tensor(n);
}

Tensor Tensor::softmax(size_t dim, SoftmaxMode mode) const {
    if (rank() < 2) throw Error("RankMismatch", "softmax input needs rank >= 2");            // Softmax::check_shapes
    if (dim >= rank()) throw Error("DimOutOfRange", "softmax dim " + std::to_string(dim));
    if (!is_float(dt())) throw Error("UnsupportedDType", as_str(dt()));
    if (dim != rank() - 1) throw Error("UnsupportedSoftmaxDim", "only the last dimension is implemented (as in the reference's kernels)");
    auto n = new_node(Kind::Softmax, shape(), dt(), device());
    n->dim = dim;
    n->mode = mode;
    n->srcs = {*this};
    return Tensor(n);
}

Tensor Tensor::slice(const std::vector<std::pair<size_t, size_t>>& ranges) const {
    require_plain(*this, "slice");
    if (ranges.size() != rank()) throw Error("RankMismatch", "slice needs one range per dimension");
    std::vector<size_t> out;
    for (size_t i = 0; i < ranges.size(); i++) {
        const auto& r = ranges[i];
        if (r.first > r.second || r.second > shape()[i])                                      // Slice::check_shapes
            throw Error("SliceOutOfBounds", "dim " + std::to_string(i) + ": " + std::to_string(r.first) + ".." + std::to_string(r.second));
        if (r.first == r.second) throw Error("EmptySlice", "dim " + std::to_string(i));   // cpu/reindex.rs:103-105 asserts start < end
        out.push_back(r.second - r.first);
    }
    auto n = new_node(Kind::Slice, Shape(out), dt(), device());
    n->ranges = ranges;
    n->srcs = {*this};
    return Tensor(n);
}

Tensor Tensor::view(const Shape& shape_) const {
    require_plain(*this, "view");
    if (shape_.rank() != rank()) throw Error("RankMismatch", "view keeps the rank (View::check_shapes)");
    if (shape_.numel() != numel()) throw Error("ShapeMismatch", "view keeps the element count");
    auto n = new_node(Kind::View, shape_, dt(), device());
    n->srcs = {*this};
    n->storage = node_->storage;               // Tensor::shallow shares the storage when it already exists
    return Tensor(n);
}

Tensor Tensor::cat(const std::vector<Tensor>& tensors, size_t dim) {
    if (tensors.size() < 2 || tensors.size() > 8) throw Error("ConcatArity", std::to_string(tensors.size()) + " inputs (2..8 supported)");
    const Tensor& first = tensors[0];
    require_rank4(first.shape(), "cat");
    require_plain(first, "cat");
    if (dim >= first.rank()) throw Error("DimOutOfRange", "cat dim " + std::to_string(dim));
    size_t stacked = 0;
    for (const Tensor& t : tensors) {
        require_same_device(first, t);
        if (t.dt() != first.dt()) throw Error("DTypeMismatch", std::string("expected ") + as_str(first.dt()) + ", got " + as_str(t.dt()));
        if (t.rank() != first.rank()) throw Error("RankMismatch", "cat inputs must have one rank");
        for (size_t a = 0; a < first.rank(); a++)
            if (a != dim && t.shape()[a] != first.shape()[a]) throw Error("ConcatShapeMismatch", t.shape().to_string() + " vs " + first.shape().to_string());
        stacked += t.shape()[dim];
    }
    Shape out = first.shape();
    out[dim] = stacked;
    auto n = new_node(Kind::Concat, out, first.dt(), first.device());
    n->dim = dim;
    n->srcs = tensors;
    return Tensor(n);
}

// Cache guards: ops/cache.rs:124-133
Tensor Tensor::cache(const Tensor& source, size_t dim, size_t offset) const {
    require_same_device(*this, source);
    require_plain(*this, "cache");
    if (rank() < 3 || rank() > 4) throw Error("RankMismatch", "cache needs rank 3 or 4");
    if (source.rank() != rank()) throw Error("RankMismatch", "cache and source must have one rank");
    if (dt() != source.dt()) throw Error("DTypeMismatch", std::string("expected ") + as_str(dt()) + ", got " + as_str(source.dt()));
    if (dim >= rank()) throw Error("DimOutOfRange", "cache dim " + std::to_string(dim));
    for (size_t a = 0; a < rank(); a++)
        if (a != dim && source.shape()[a] != shape()[a]) throw Error("ShapeMismatch", source.shape().to_string() + " vs " + shape().to_string());
    if (offset > shape()[dim] || offset + source.shape()[dim] > shape()[dim])
        throw Error("CacheOverflow", "offset " + std::to_string(offset) + " + " + std::to_string(source.shape()[dim]) + " rows exceed " +
                                         std::to_string(shape()[dim]));
    Shape out = shape();
    out[dim] = offset + source.shape()[dim];
    auto n = new_node(Kind::Cache, out, dt(), device());
    n->dim = dim;
    n->groups = offset;                        // reuses the integer slot: the write offset
    n->srcs = {*this, source};
    return Tensor(n);
}

// RoPE guards: ops/rope.rs:52-66
Tensor Tensor::rope(size_t dim, float base, size_t offset) const {
    if (rank() != 4) throw Error("RankMismatch", "rope needs rank 4, got " + std::to_string(rank()));
    if (shape()[3] < dim) throw Error("ShapeMismatch", "rope dim " + std::to_string(dim) + " exceeds head dim " + std::to_string(shape()[3]));
    if (dim == 0 || dim % 8 != 0) throw Error("ShapeMismatch", "rope dim " + std::to_string(dim) + " is not a multiple of 8");
    if (!is_float(dt())) throw Error("UnsupportedDType", as_str(dt()));
    auto n = new_node(Kind::RoPE, shape(), dt(), device());
    n->dim = dim;
    n->groups = offset;                        // integer slot: the position offset
    n->eps = base;                             // float slot: the frequency base
    n->srcs = {*this};
    return Tensor(n);
}

// IndexSelect guards: ops/select.rs:67-79 (rank-2 source, rank-1 I32 indices) and compute_view :48-60
Tensor Tensor::index_select(const Tensor& indices, size_t dim) const {
    require_same_device(*this, indices);
    if (rank() != 2) throw Error("RankMismatch", "index_select source must have rank 2, got " + std::to_string(rank()));
    if (indices.rank() != 1) throw Error("RankMismatch", "index_select indices must have rank 1, got " + std::to_string(indices.rank()));
    if (indices.dt() != DType::I32) throw Error("DTypeMismatch", std::string("expected I32, got ") + as_str(indices.dt()));
    if (dim >= rank()) throw Error("DimOutOfRange", "index_select dim " + std::to_string(dim));
    // a Q8_0 table: whole words of four elements along the row, as the reference's kernel reads them (ops/select.rs:144-161)
    if (is_quantized(dt()) && (dim != 0 || shape()[1] % 4 != 0))
        throw Error("ShapeMismatch", "index_select from a quantized table takes rows (dim 0) of a multiple of 4 columns");
    Shape out = shape();
    out[dim] = indices.shape()[0];
    auto n = new_node(Kind::IndexSelect, out, activation_dt(dt()), device());      // compute_view, ops/select.rs:48-60
    n->dim = dim;
    n->srcs = {*this, indices};
    return Tensor(n);
}

// IndexWrite has no guards in the reference (ops/index_write.rs:29-33); the run it writes must stay inside dst
Tensor Tensor::index_write(const Tensor& src, const std::vector<size_t>& write_start) const {
    require_same_device(*this, src);
    require_plain(*this, "index_write");
    require_rank4(shape(), "index_write");
    if (dt() != src.dt()) throw Error("DTypeMismatch", std::string("expected ") + as_str(dt()) + ", got " + as_str(src.dt()));
    if (write_start.size() != rank()) throw Error("RankMismatch", "write_start must have one entry per dimension");
    size_t off = 0;
    for (size_t i = 0; i < rank(); i++) {
        if (write_start[i] >= shape()[i]) throw Error("IndexOutOfBounds", "write_start[" + std::to_string(i) + "] = " + std::to_string(write_start[i]));
        off = off * shape()[i] + write_start[i];
    }
    if (off + src.numel() > numel()) throw Error("IndexOutOfBounds", "the written run leaves the destination");
    auto n = new_node(Kind::IndexWrite, shape(), dt(), device());
    n->dims = write_start;
    n->srcs = {*this, src};
    return Tensor(n);
}

Tensor Tensor::permute(const std::vector<size_t>& dims) const {
    require_plain(*this, "permute");
    if (dims.size() != rank()) throw Error("RankMismatch", "permute needs one index per dimension");    // Permute::check_shapes
    std::vector<bool> seen(rank(), false);
    std::vector<size_t> out(rank());
    for (size_t i = 0; i < dims.size(); i++) {
        if (dims[i] >= rank()) throw Error("DimOutOfRange", "permute index " + std::to_string(dims[i]));
        if (seen[dims[i]]) throw Error("DuplicateDims", "permute indices repeat");                       // InvariantError::DuplicateDims
        seen[dims[i]] = true;
        out[i] = shape()[dims[i]];
    }
    auto n = new_node(Kind::Permute, Shape(out), dt(), device());
    n->dims = dims;
    n->srcs = {*this};
    return Tensor(n);
}

Tensor Tensor::broadcast_to(const Shape& to) const {
    require_plain(*this, "broadcast_to");
    require_rank4(to, "broadcast_to");
    if (rank() > to.rank())
        throw Error("InvalidBroadcast", "source has more dimensions than the target: " + shape().to_string() + " -> " + to.to_string());
    for (size_t i = 0; i < rank(); i++) {                                                           // Broadcast::check_shapes
        const size_t s = shape()[rank() - 1 - i], d = to[to.rank() - 1 - i];
        if (s != 1 && s != d) throw Error("InvalidBroadcast", std::to_string(s) + " cannot be broadcast to " + std::to_string(d));
    }
    auto n = new_node(Kind::Broadcast, to, dt(), device());
    n->srcs = {*this};
    return Tensor(n);
}

// ------------------------------------------------------------------------------------------------------------ resolve
static void shape4(const Shape& s, uint32_t out[4]) {
    const Shape p = Shape::promote(s, 4);
    for (int i = 0; i < 4; i++) out[i] = (uint32_t)p[i];
}

// iterative post-order DFS over srcs, sources that have sources of their own first (tensor.rs:696-740)
static std::vector<Node*> execution_order(Node* root) {
    std::unordered_set<uint64_t> done, pending;
    std::vector<Node*> order;
    std::vector<std::pair<Node*, size_t>> stack{{root, 0}};
    while (!stack.empty()) {
        auto [cur, idx] = stack.back();
        stack.pop_back();
        if (idx == cur->srcs.size()) {
            done.insert(cur->id);
            pending.erase(cur->id);
            order.push_back(cur);
            continue;
        }
        std::vector<Node*> all;
        for (const Tensor& s : cur->srcs)
            if (!Node::of(s)->srcs.empty()) all.push_back(Node::of(s));
        for (const Tensor& s : cur->srcs)
            if (Node::of(s)->srcs.empty()) all.push_back(Node::of(s));
        Node* pre = all[idx];
        if (done.count(pre->id)) {
            stack.push_back({cur, idx + 1});
        } else if (pending.count(pre->id)) {
            throw Error("CycleDetected", "cycle through tensor " + std::to_string(pre->id));
        } else {
            pending.insert(pre->id);
            stack.push_back({cur, idx});
            stack.push_back({pre, 0});
        }
    }
    return order;
}

std::vector<uint64_t> Tensor::execution_order_ids() const {
    std::vector<uint64_t> ids;
    for (Node* n : execution_order(node_.get())) ids.push_back(n->id);
    return ids;
}

static std::atomic<bool> g_fuse_patterns{true};
void set_pattern_fusion(bool on) { g_fuse_patterns = on; }
bool pattern_fusion() { return g_fuse_patterns; }

// One-pass replacements for the op sequences the models always emit around 16-bit tensors (full() ... cast(dt)).
// The graph the user built is unchanged; resolve() runs one launch at the sequence's last node and never materialises
// the interior nodes, which must be unresolved and held by nobody but their single consumer.
struct FusedPlan {
    enum What { NormVia32, SoftmaxVia32, UnaryVia32, GatedMul, SoftmaxMasked } what;
    Node* x = nullptr;            // 16-bit input (gate for GatedMul)
    Node* aux = nullptr;          // norm node (scale / bias / eps / kind), softmax node (mode), unary node (op)
    Node* mask = nullptr;         // SoftmaxVia32: tensor added to x before the softmax (nullptr: none)
    Node* up = nullptr;           // GatedMul: the multiplied operand
    uint64_t x_off = 0, up_off = 0, x_stride = 0, up_stride = 0;   // GatedMul views, in elements
};

// Everything resolve() decides before the first launch: which nodes run, which are folded into a neighbour, what
// each launch reads, and the memory plan.
struct PreparedGraph {
    std::vector<Node*> order;                                  // needed nodes, execution order
    std::unordered_set<Node*> skip;
    std::unordered_map<Node*, FusedPlan> fused;
    std::vector<planner::Step> steps;                          // one per launch
    std::vector<Node*> step_node;
    std::vector<std::vector<Node*>> step_reads;                // the nodes behind Step::reads
    std::unordered_map<Node*, size_t> step_of;
    std::vector<std::vector<Node*>> release_at;                // per index into order: nodes whose storage handle is dropped after it
    planner::Plan plan;
};

struct Executable::Inner {
    Device device;
    rt_graph* graph = nullptr;                // the recorded launches; null for a short list, which is re-issued call by call
    size_t launches = 0;
    size_t held = 0;
    PreparedGraph prepared;                   // the launch list and what each launch reads
    std::vector<std::shared_ptr<Buffer>> storage;   // per entry of prepared.order: the buffer the node had after the first run
    std::shared_ptr<Node> root;               // keeps the graph's nodes, and with them its constants' storage
    ~Inner() {
        if (graph) rt_graph_destroy(graph);
    }
};

struct Resolver {
    typedef PreparedGraph Prepared;
    // a Broadcast node nobody else holds, not yet materialised, feeding a Binary: fused into the binary kernel
    static bool fusable_broadcast(const Tensor& operand) {
        Node* b = Node::of(operand);
        return b->kind == Kind::Broadcast && !b->storage && Node::holders(operand) == 1;
    }
    // an interior node of a pattern: not yet computed and invisible to everybody but its consumer
    static bool interior(const Tensor& t, Kind k) {
        Node* n = Node::of(t);
        return n->kind == k && !n->storage && Node::holders(t) == 1;
    }
    static bool is16(DType d) { return d == DType::F16 || d == DType::BF16; }

    // `n` is a Cast f32 -> 16-bit whose source chain is <16-bit x>.full().<op>(): fills plan, lists the interior nodes
    static bool match_via32(Node* n, FusedPlan& plan, std::vector<Node*>& inner) {
        if (n->kind != Kind::Cast || !is16(n->dt) || n->storage) return false;
        const Tensor& opT = n->srcs[0];
        Node* op = Node::of(opT);
        if (op->dt != DType::F32 || op->storage || Node::holders(opT) != 1) return false;
        if (op->kind != Kind::LayerNorm && op->kind != Kind::RMSNorm && op->kind != Kind::Softmax && op->kind != Kind::Unary) return false;
        if (!interior(op->srcs[0], Kind::Cast)) return false;
        Node* widen = Node::of(op->srcs[0]);
        Node* x = Node::of(widen->srcs[0]);
        if (x->dt != n->dt) return false;                          // full() of a 16-bit tensor, cast back to the same type
        plan.x = x;
        plan.aux = op;
        inner = {op, widen};
        if (op->kind == Kind::Unary) {
            plan.what = FusedPlan::UnaryVia32;
            return true;
        }
        if (op->kind == Kind::LayerNorm || op->kind == Kind::RMSNorm) {
            plan.what = FusedPlan::NormVia32;
            return true;
        }
        if (op->dim != op->shape.rank() - 1) return false;
        plan.what = FusedPlan::SoftmaxVia32;
        // scores.add(mask): a Binary add nobody else sees, scores at full shape, the mask broadcast (or already full)
        if (interior(widen->srcs[0], Kind::Binary) && x->bop == BinaryOp::Add) {
            Node* scores = Node::of(x->srcs[0]);
            const Tensor& mT = x->srcs[1];
            Node* m = Node::of(mT);
            if (scores->shape == x->shape && !(scores->kind == Kind::Broadcast && !scores->storage)) {
                if (fusable_broadcast(mT)) {
                    inner.push_back(x);
                    inner.push_back(m);
                    plan.mask = Node::of(m->srcs[0]);
                    plan.x = scores;
                } else if (m->kind != Kind::Broadcast || m->storage) {
                    inner.push_back(x);
                    plan.mask = m;
                    plan.x = scores;
                }
            }
        }
        return true;
    }

    // scores.add(mask).softmax(last dim) in one type: the add is absorbed when nobody else sees the sum
    static bool match_masked_softmax(Node* n, FusedPlan& plan, std::vector<Node*>& inner) {
        if (n->kind != Kind::Softmax || n->storage || n->dim != n->shape.rank() - 1) return false;
        if (!interior(n->srcs[0], Kind::Binary)) return false;
        Node* add = Node::of(n->srcs[0]);
        if (add->bop != BinaryOp::Add) return false;
        Node* scores = Node::of(add->srcs[0]);
        const Tensor& mT = add->srcs[1];
        Node* m = Node::of(mT);
        if (scores->shape != add->shape || (scores->kind == Kind::Broadcast && !scores->storage)) return false;
        plan.what = FusedPlan::SoftmaxMasked;
        plan.aux = n;
        plan.x = scores;
        inner = {add};
        if (fusable_broadcast(mT)) {
            inner.push_back(m);
            plan.mask = Node::of(m->srcs[0]);
        } else if (m->kind != Kind::Broadcast || m->storage) {
            plan.mask = m;
        } else {
            return false;
        }
        return true;
    }

    // a Slice that only narrows the last dim, not yet materialised and seen by its consumer alone: a row-strided view
    static bool last_dim_view(const Tensor& t, Node*& base, uint64_t& off, uint64_t& stride) {
        Node* n = Node::of(t);
        if (n->kind != Kind::Slice || n->storage || Node::holders(t) != 1) return false;
        Node* src = Node::of(n->srcs[0]);
        const size_t r = src->shape.rank();
        if (n->ranges.size() != r) return false;
        for (size_t i = 0; i + 1 < r; i++)
            if (n->ranges[i].first != 0 || n->ranges[i].second != src->shape[i]) return false;
        base = src;
        off = n->ranges[r - 1].first;
        stride = src->shape[r - 1];
        return true;
    }

    // up.mul(gate.full().<op>().cast(dt)), either operand order
    static bool match_gated(Node* n, FusedPlan& plan, std::vector<Node*>& inner) {
        if (n->kind != Kind::Binary || n->bop != BinaryOp::Mul || !is16(n->dt) || n->storage) return false;
        for (int side = 0; side < 2; side++) {
            const Tensor& actT = n->srcs[side ^ 1];
            const Tensor& upT = n->srcs[side];
            if (!interior(actT, Kind::Cast)) continue;
            FusedPlan act;
            std::vector<Node*> act_inner;
            if (!match_via32(Node::of(actT), act, act_inner) || act.what != FusedPlan::UnaryVia32) continue;
            Node* up = Node::of(upT);
            if (up->shape != n->shape || (up->kind == Kind::Broadcast && !up->storage)) continue;
            plan.what = FusedPlan::GatedMul;
            plan.aux = act.aux;
            plan.x = act.x;
            plan.up = up;
            inner = act_inner;
            inner.push_back(Node::of(actT));
            const uint64_t cols = n->shape[n->shape.rank() - 1];
            plan.x_stride = plan.up_stride = cols;
            // the gate's slice hangs off the widening cast, the other operand's off the multiply
            Node* widen = act_inner[1];
            Node* base = nullptr;
            uint64_t off = 0, stride = 0;
            if (last_dim_view(widen->srcs[0], base, off, stride)) {
                inner.push_back(plan.x);
                plan.x = base;
                plan.x_off = off;
                plan.x_stride = stride;
            }
            if (last_dim_view(upT, base, off, stride)) {
                inner.push_back(plan.up);
                plan.up = base;
                plan.up_off = off;
                plan.up_stride = stride;
            }
            return true;
        }
        return false;
    }

    static void run_fused(Node* n, const FusedPlan& plan, size_t& launches) {
        rt_device* dev = n->device.raw();
        const int dt = (int)n->dt;
        if (!n->storage) n->storage = std::make_shared<Buffer>(n->device, n->shape.numel() * size_of(n->dt));
        const size_t cols = n->shape[n->shape.rank() - 1];
        const uint64_t rows = n->shape.numel() / cols;
        switch (plan.what) {
            case FusedPlan::NormVia32: {
                Node* op = plan.aux;
                const bool layer = op->kind == Kind::LayerNorm;
                const float* scale = static_cast<const float*>(Node::of(op->srcs[1])->storage->ptr);
                const float* bias = (layer && op->has_bias) ? static_cast<const float*>(Node::of(op->srcs[2])->storage->ptr) : nullptr;
                check_rt(rt_norm_via_f32(dev, layer ? 0 : 1, dt, plan.x->storage->ptr, scale, bias, n->storage->ptr, rows, (uint32_t)cols, op->eps),
                         "rt_norm_via_f32");
                break;
            }
            case FusedPlan::SoftmaxVia32: {
                uint32_t xs[4], ms[4];
                shape4(n->shape, xs);
                if (plan.mask) shape4(plan.mask->shape, ms);
                check_rt(rt_softmax_via_f32(dev, dt, plan.x->storage->ptr, xs, plan.mask ? plan.mask->storage->ptr : nullptr, plan.mask ? ms : nullptr,
                                            n->storage->ptr, (int)plan.aux->mode),
                         "rt_softmax_via_f32");
                break;
            }
            case FusedPlan::SoftmaxMasked: {
                uint32_t xs[4], ms[4];
                shape4(n->shape, xs);
                shape4(plan.mask->shape, ms);
                check_rt(rt_softmax_masked(dev, dt, plan.x->storage->ptr, xs, plan.mask->storage->ptr, ms, n->storage->ptr, (int)n->mode),
                         "rt_softmax_masked");
                break;
            }
            case FusedPlan::UnaryVia32:
                check_rt(rt_unary_via_f32(dev, (int)plan.aux->uop, dt, plan.x->storage->ptr, n->storage->ptr, n->shape.numel()), "rt_unary_via_f32");
                break;
            case FusedPlan::GatedMul: {
                const size_t eb = size_of(n->dt);
                const char* gate = static_cast<const char*>(plan.x->storage->ptr) + plan.x_off * eb;
                const char* up = static_cast<const char*>(plan.up->storage->ptr) + plan.up_off * eb;
                check_rt(rt_gated_mul_via_f32(dev, (int)plan.aux->uop, dt, gate, plan.x_stride, up, plan.up_stride, n->storage->ptr, rows, (uint32_t)cols),
                         "rt_gated_mul_via_f32");
                break;
            }
        }
        launches++;
    }

    static void run(Node* n, size_t& launches) {
        rt_device* dev = n->device.raw();
        const int dt = (int)n->dt;
        auto src = [&](size_t i) -> Node* { return Node::of(n->srcs[i]); };
        // resolve() has given the node its output buffer already (the source's own when the op runs in place, a shared
        // object of the memory plan, or an allocation of its own)
        auto out_buffer = [&]() {
            if (!n->storage) n->storage = std::make_shared<Buffer>(n->device, n->shape.numel() * size_of(n->dt));
        };
        auto take_src0_if_unshared = [&]() { return (bool)n->storage; };
        switch (n->kind) {
            case Kind::Const: throw Error("Unresolved", "constant tensor " + std::to_string(n->id) + " has no storage (placeholder)");
            case Kind::View: n->storage = src(0)->storage; return;
            case Kind::Binary: {
                const bool fa = fusable_broadcast(n->srcs[0]), fb = fusable_broadcast(n->srcs[1]);
                Node* a = fa ? Node::of(src(0)->srcs[0]) : src(0);
                Node* b = fb ? Node::of(src(1)->srcs[0]) : src(1);
                if (fa || fb) {
                    uint32_t as[4], bs[4], ys[4];
                    shape4(a->shape, as);
                    shape4(b->shape, bs);
                    shape4(n->shape, ys);
                    out_buffer();
                    check_rt(rt_binary_bcast(dev, (int)n->bop, dt, a->storage->ptr, as, b->storage->ptr, bs, n->storage->ptr, ys), "rt_binary_bcast");
                } else {
                    if (!take_src0_if_unshared()) out_buffer();
                    check_rt(rt_binary(dev, (int)n->bop, dt, a->storage->ptr, b->storage->ptr, n->storage->ptr, n->shape.numel()), "rt_binary");
                }
                launches++;
                return;
            }
            case Kind::Unary:
                if (!take_src0_if_unshared()) out_buffer();
                check_rt(rt_unary(dev, (int)n->uop, dt, src(0)->storage->ptr, n->storage->ptr, n->shape.numel()), "rt_unary");
                launches++;
                return;
            case Kind::Softmax: {
                if (!take_src0_if_unshared()) out_buffer();
                const size_t cols = n->shape[n->shape.rank() - 1];
                check_rt(rt_softmax(dev, dt, src(0)->storage->ptr, n->storage->ptr, n->shape.numel() / cols, (uint32_t)cols, (int)n->mode),
                         "rt_softmax");
                launches++;
                return;
            }
            case Kind::Cast:
                out_buffer();                                  // Cast::supports_inplace() is false (ops/cast.rs:128-131)
                check_rt(rt_cast(dev, (int)src(0)->dt, dt, src(0)->storage->ptr, n->storage->ptr, n->shape.numel()), "rt_cast");
                launches++;
                return;
            case Kind::Permute: {
                uint32_t ss[4], perm[4];
                shape4(src(0)->shape, ss);
                const size_t pad = 4 - n->dims.size();         // Permute::promote (ops/reindex/permute.rs:29-38)
                for (size_t i = 0; i < pad; i++) perm[i] = (uint32_t)i;
                for (size_t i = 0; i < n->dims.size(); i++) perm[pad + i] = (uint32_t)(n->dims[i] + pad);
                out_buffer();
                check_rt(rt_permute(dev, (int)size_of(n->dt), src(0)->storage->ptr, n->storage->ptr, ss, perm), "rt_permute");
                launches++;
                return;
            }
            case Kind::Slice: {
                uint32_t ss[4], st[4] = {0, 0, 0, 0}, ds[4];
                shape4(src(0)->shape, ss);
                shape4(n->shape, ds);
                const size_t pad = 4 - n->ranges.size();
                for (size_t i = 0; i < n->ranges.size(); i++) st[pad + i] = (uint32_t)n->ranges[i].first;
                out_buffer();
                check_rt(rt_slice(dev, (int)size_of(n->dt), src(0)->storage->ptr, n->storage->ptr, ss, st, ds), "rt_slice");
                launches++;
                return;
            }
            case Kind::Broadcast: {
                uint32_t ss[4], ds[4];
                shape4(src(0)->shape, ss);
                shape4(n->shape, ds);
                out_buffer();
                check_rt(rt_broadcast(dev, (int)size_of(n->dt), src(0)->storage->ptr, n->storage->ptr, ss, ds), "rt_broadcast");
                launches++;
                return;
            }
            case Kind::Concat: {
                const void* ptrs[8];
                uint32_t shapes[8][4];
                for (size_t i = 0; i < n->srcs.size(); i++) {
                    ptrs[i] = src(i)->storage->ptr;
                    shape4(src(i)->shape, shapes[i]);
                }
                out_buffer();
                check_rt(rt_concat(dev, (int)size_of(n->dt), (int)n->srcs.size(), ptrs, shapes, (int)(n->dim + 4 - n->shape.rank()), n->storage->ptr),
                         "rt_concat");
                launches++;
                return;
            }
            case Kind::Cache: {
                uint32_t cs[4], ss[4];
                shape4(src(0)->shape, cs);
                shape4(src(1)->shape, ss);
                out_buffer();                                  // Cache::supports_inplace() is false (ops/cache.rs:150-152)
                check_rt(rt_cache(dev, (int)size_of(n->dt), src(0)->storage->ptr, cs, src(1)->storage->ptr, ss,
                                  (int)(n->dim + 4 - n->shape.rank()), (uint32_t)n->groups, n->storage->ptr),
                         "rt_cache");
                launches++;
                return;
            }
            case Kind::RoPE: {
                uint32_t xs[4];
                shape4(n->shape, xs);
                if (!take_src0_if_unshared()) out_buffer();    // RoPE::supports_inplace() (ops/rope.rs:80-82)
                check_rt(rt_rope(dev, dt, src(0)->storage->ptr, n->storage->ptr, xs, (uint32_t)n->dim, n->eps, (uint32_t)n->groups), "rt_rope");
                launches++;
                return;
            }
            case Kind::IndexSelect: {
                uint32_t ss[4];
                shape4(src(0)->shape, ss);
                out_buffer();
                if (is_quantized(src(0)->dt)) {
                    const char* base = static_cast<const char*>(src(0)->storage->ptr);
                    check_rt(rt_index_select_q8_0(dev, dt, reinterpret_cast<const uint32_t*>(base), base + align256(src(0)->shape.numel()), ss,
                                                  static_cast<const int32_t*>(src(1)->storage->ptr), (uint32_t)src(1)->shape[0],
                                                  (int)(n->dim + 4 - n->shape.rank()), n->storage->ptr),
                             "rt_index_select_q8_0");
                    launches++;
                    return;
                }
                check_rt(rt_index_select(dev, (int)size_of(n->dt), src(0)->storage->ptr, ss, static_cast<const int32_t*>(src(1)->storage->ptr),
                                         (uint32_t)src(1)->shape[0], (int)(n->dim + 4 - n->shape.rank()), n->storage->ptr),
                         "rt_index_select");
                launches++;
                return;
            }
            case Kind::IndexWrite: {
                uint32_t ds[4], ws[4] = {0, 0, 0, 0};
                shape4(n->shape, ds);
                const size_t pad = 4 - n->dims.size();
                for (size_t i = 0; i < n->dims.size(); i++) ws[pad + i] = (uint32_t)n->dims[i];
                n->storage = src(0)->storage;                  // the destination's buffer is the result (ops/index_write.rs:40-50)
                check_rt(rt_index_write(dev, (int)size_of(n->dt), n->storage->ptr, ds, src(1)->storage->ptr, src(1)->shape.numel(), ws),
                         "rt_index_write");
                launches++;
                return;
            }
            case Kind::LayerNorm:
            case Kind::RMSNorm: {
                const size_t cols = n->shape[n->shape.rank() - 1];
                out_buffer();
                if (n->kind == Kind::LayerNorm)
                    check_rt(rt_layer_norm(dev, dt, src(0)->storage->ptr, src(1)->storage->ptr, n->has_bias ? src(2)->storage->ptr : nullptr,
                                           n->storage->ptr, n->shape.numel() / cols, (uint32_t)cols, n->eps),
                             "rt_layer_norm");
                else
                    check_rt(rt_rms_norm(dev, dt, src(0)->storage->ptr, src(1)->storage->ptr, n->storage->ptr, n->shape.numel() / cols,
                                         (uint32_t)cols, n->eps),
                             "rt_rms_norm");
                launches++;
                return;
            }
            case Kind::GroupNorm: {
                const size_t B = n->shape[0], C = n->shape[1];
                out_buffer();
                check_rt(rt_group_norm(dev, dt, src(0)->storage->ptr, src(1)->storage->ptr, n->has_bias ? src(2)->storage->ptr : nullptr,
                                       n->storage->ptr, (uint32_t)B, (uint32_t)C, (uint32_t)(n->shape.numel() / (B * C)), (uint32_t)n->groups, n->eps),
                         "rt_group_norm");
                launches++;
                return;
            }
        }
    }

    // the node whose buffer is read when `t` is an operand: through views (which alias their source)
    static Node* base_of(Node* n) {
        while (n->kind == Kind::View && !n->storage) n = Node::of(n->srcs[0]);
        return n;
    }

    // for_replay: the launches will run more than once (Executable), so nothing may work in place in a buffer that holds
    // an input of the graph
    static Prepared prepare(Node* root, bool for_replay = false) {
        Prepared P;
        const std::vector<Node*> full_order = execution_order(root);
        // only what the root still needs: nothing below a tensor that already has its storage (tensor.rs:783 skips those;
        // their own inputs may have given their buffers back, see below)
        std::unordered_set<Node*> needed;
        {
            std::vector<Node*> todo{root};
            while (!todo.empty()) {
                Node* n = todo.back();
                todo.pop_back();
                if (!needed.insert(n).second || n->storage) continue;
                for (const Tensor& s : n->srcs) todo.push_back(Node::of(s));
            }
        }
        std::vector<Node*>& order = P.order;
        for (Node* n : full_order)
            if (needed.count(n)) order.push_back(n);
        std::unordered_set<Node*>& skip = P.skip;
        // caller patterns, consumers first so that the longest sequence wins (the gated multiply contains a unary one)
        std::unordered_map<Node*, FusedPlan>& fused = P.fused;
        if (g_fuse_patterns) {
            for (auto it = order.rbegin(); it != order.rend(); ++it) {
                Node* n = *it;
                if (n->storage || skip.count(n)) continue;
                FusedPlan plan;
                std::vector<Node*> inner;
                if (match_gated(n, plan, inner) || match_via32(n, plan, inner) || match_masked_softmax(n, plan, inner)) {
                    fused.emplace(n, plan);
                    for (Node* i : inner) skip.insert(i);
                }
            }
        }
        // broadcasts that their (single) binary consumer will absorb are not materialised
        for (Node* n : order)
            if (n->kind == Kind::Binary && !n->storage && !skip.count(n) && !fused.count(n))
                for (const Tensor& s : n->srcs)
                    if (fusable_broadcast(s)) skip.insert(Node::of(s));

        // Liveness: an intermediate that nobody outside this graph can see drops its handle on its buffer right after the
        // last launch that reads it.  Launches run in stream order, which makes the hand-over safe without waiting.
        std::unordered_map<Node*, size_t> index_of, edges, last_use;
        std::unordered_map<Node*, Node*> consumer;                 // of a skipped node: the one node that absorbs it
        for (size_t i = 0; i < order.size(); i++) index_of[order[i]] = i;
        for (Node* n : order) {
            if (n->storage) continue;                              // a resolved node reads nothing
            for (const Tensor& s : n->srcs) {
                edges[Node::of(s)]++;
                consumer[Node::of(s)] = n;
            }
        }
        auto exec_index = [&](Node* n) {
            while (skip.count(n)) n = consumer.at(n);
            return index_of.at(n);
        };
        P.release_at.resize(order.size());
        for (Node* n : order) {
            if (n->storage) continue;
            for (const Tensor& s : n->srcs) {
                Node* src = Node::of(s);
                const size_t at = exec_index(n);
                auto it = last_use.find(src);
                if (it == last_use.end() || it->second < at) last_use[src] = at;
            }
        }
        // every holder of the node is an edge of this graph: no user handle, no other graph.  A view aliases its source's
        // buffer, so a source is only hidden when every view of it is hidden too (a view kept by the caller, or the root
        // being a view, keeps the buffer below it visible); consumers come after their sources in `order`, so the walk
        // goes backwards and a view's own answer is known before its source asks.
        std::unordered_map<Node*, const Tensor*> handle_of;        // (a pointer: a copy would be one more holder)
        std::unordered_map<Node*, std::vector<Node*>> views_of;
        for (Node* n : order) {
            if (n->storage) continue;
            for (const Tensor& s : n->srcs) {
                handle_of.emplace(Node::of(s), &s);
                if (n->kind == Kind::View) views_of[Node::of(s)].push_back(n);
            }
        }
        std::unordered_set<Node*> hidden_nodes;
        for (auto it = order.rbegin(); it != order.rend(); ++it) {
            Node* src = *it;
            auto h = handle_of.find(src);
            if (h == handle_of.end()) continue;                    // nobody in this graph reads it
            bool hidden = src != root && !src->srcs.empty() && (size_t)Node::holders(*h->second) == edges[src];
            if (hidden) {
                auto v = views_of.find(src);
                if (v != views_of.end())
                    for (Node* view : v->second) hidden = hidden && hidden_nodes.count(view);
            }
            if (!hidden) continue;
            hidden_nodes.insert(src);
            if (last_use.count(src)) {
                P.release_at[last_use[src]].push_back(src);
                last_use.erase(src);
            }
        }

        // The launches and what each reads, for the memory plan (gpu/buffer_allocator/allocator.rs:141-271).
        auto launches_here = [&](Node* n) { return !n->storage && !skip.count(n) && n->kind != Kind::View && !n->srcs.empty(); };
        std::unordered_set<Node*> in_input;                        // results that live in a buffer which existed before this graph
        for (Node* n : order) {
            if (!launches_here(n)) continue;
            planner::Step st;
            st.id = n->id;
            st.bytes = n->shape.numel() * size_of(n->dt);
            st.pinned = !hidden_nodes.count(n);
            std::vector<Node*> reads;
            std::vector<Node*> todo;
            for (auto it = n->srcs.rbegin(); it != n->srcs.rend(); ++it) todo.push_back(Node::of(*it));
            while (!todo.empty()) {                                // operands in bind order, through folded-away nodes and views
                Node* m = todo.back();
                todo.pop_back();
                if (!m->storage && (skip.count(m) || m->kind == Kind::View)) {
                    for (auto it = m->srcs.rbegin(); it != m->srcs.rend(); ++it) todo.push_back(Node::of(*it));
                    continue;
                }
                if (std::find(reads.begin(), reads.end(), m) == reads.end()) reads.push_back(m);
            }
            // tensor.rs:823-824: supports_inplace() && Arc::strong_count(srcs[0]) == 1 (here also: same size, and nobody
            // else shares a buffer that exists already); IndexWrite's result is its destination (ops/index_write.rs:40-50)
            if (!fused.count(n)) {
                const Tensor& s0T = n->srcs[0];
                Node* s0 = Node::of(s0T);
                bool in_place = false;
                if (n->kind == Kind::IndexWrite) {
                    in_place = true;
                } else if (n->kind == Kind::Unary || n->kind == Kind::Softmax || n->kind == Kind::RoPE ||
                           (n->kind == Kind::Binary && !fusable_broadcast(n->srcs[0]) && !fusable_broadcast(n->srcs[1]))) {
                    in_place = Node::holders(s0T) == 1 && s0->shape == n->shape && s0->dt == n->dt && s0->kind != Kind::View &&
                               (s0->storage ? s0->storage.use_count() == 1 : true);
                    if (for_replay && (s0->storage || in_input.count(s0))) in_place = false;
                }
                if (in_place) {
                    st.inplace = (int)(std::find(reads.begin(), reads.end(), base_of(s0)) - reads.begin());
                    if (base_of(s0)->storage || in_input.count(base_of(s0))) in_input.insert(n);
                }
            }
            for (Node* r : reads) st.reads.push_back(r->id);
            P.step_of[n] = P.steps.size();
            P.steps.push_back(st);
            P.step_node.push_back(n);
            P.step_reads.push_back(reads);
        }
        P.plan = planner::greedy_by_size(P.steps);
        return P;
    }

    static void resolve(Node* root) {
        size_t launches = 0;
        Prepared P = prepare(root);
        bool pass_begun = false;
        // shared objects come from the device's pool when their first tenant is produced and go back after their last reader
        std::vector<std::shared_ptr<Buffer>> objects(P.plan.object_bytes.size());
        for (size_t i = 0; i < P.order.size(); i++) {
            Node* n = P.order[i];
            auto st = P.step_of.find(n);
            if (st != P.step_of.end()) {
                const planner::Step& step = P.steps[st->second];
                const int obj = P.plan.object_of.at(n->id);
                if (!pass_begun) {
                    // a resolve is a pass of the storage pool, as in resolve_gpu (tensor.rs:800): blocks that nobody took
                    // during the last one go back to the driver before this one allocates
                    check_rt(rt_pool_begin_pass(n->device.raw()), "rt_pool_begin_pass");
                    pass_begun = true;
                }
                if (step.inplace >= 0) {
                    n->storage = P.step_reads[st->second][(size_t)step.inplace]->storage;
                } else if (obj >= 0) {
                    if (!objects[(size_t)obj]) objects[(size_t)obj] = std::make_shared<Buffer>(n->device, P.plan.object_bytes[(size_t)obj]);
                    n->storage = objects[(size_t)obj];
                } else {
                    n->storage = std::make_shared<Buffer>(n->device, step.bytes);
                }
                auto f = P.fused.find(n);
                if (f != P.fused.end()) run_fused(n, f->second, launches);
                else run(n, launches);
                for (size_t o = 0; o < objects.size(); o++)
                    if (objects[o] && P.plan.object_last_use[o] == st->second) objects[o].reset();
            } else if (!n->storage && !P.skip.count(n)) {
                run(n, launches);                                  // a view (no launch) or a constant without storage (throws)
            }
            for (Node* dead : P.release_at[i]) dead->storage.reset();
        }
        check_rt(rt_sync(root->device.raw()), "rt_sync");      // resolve returns after completion (tensor.rs:855-856)
        root->last_launches = launches;
    }

    // Issues the launches of a compiled graph once more on the buffers of its first run: the nodes get their buffers back
    // for the duration of the call (hidden intermediates drop theirs after resolve, the executable keeps them).
    static void replay(Executable::Inner& in) {
        const Prepared& P = in.prepared;
        std::vector<size_t> lent;
        for (size_t i = 0; i < P.order.size(); i++)
            if (!P.order[i]->storage && in.storage[i]) {
                P.order[i]->storage = in.storage[i];
                lent.push_back(i);
            }
        auto give_back = [&] {
            for (size_t i : lent) P.order[i]->storage.reset();
        };
        try {
            size_t launches = 0;
            for (Node* n : P.order) {
                if (!P.step_of.count(n)) continue;
                auto f = P.fused.find(n);
                if (f != P.fused.end()) run_fused(n, f->second, launches);
                else run(n, launches);
            }
        } catch (...) {
            give_back();
            throw;
        }
        give_back();
    }

    // A shorter launch list is re-issued call by call: measured on this stack, a graph launch costs 32-35 us up to its
    // completion whatever it holds, a list of n small kernels issued one by one about 10 + 3 n us.
    static constexpr size_t GRAPH_MIN_LAUNCHES = 8;

    // resolve() that keeps its buffers and its launch list.  The first run is a plain one (it also builds the lookup
    // tables and grows the scratch the kernels want, which a capture cannot); a list of GRAPH_MIN_LAUNCHES or more is then
    // issued again on the same buffers while the device's stream is capturing.  Every buffer is assigned before the first
    // launch and none is handed back between launches: the plan's shared objects are safe to share because a replay
    // keeps the launch order.
    static Executable compile(const std::shared_ptr<Node>& root_ref) {
        Node* root = root_ref.get();
        auto inner = std::make_shared<Executable::Inner>();
        inner->prepared = prepare(root, true);
        const Prepared& P = inner->prepared;
        for (Node* n : P.order)
            if (n->srcs.empty() && !n->storage)
                throw Error("Unresolved", "constant tensor " + std::to_string(n->id) + " has no storage (placeholder)");
        inner->device = root->device;
        inner->root = root_ref;
        check_rt(rt_pool_begin_pass(root->device.raw()), "rt_pool_begin_pass");
        std::vector<std::shared_ptr<Buffer>> objects(P.plan.object_bytes.size());
        for (size_t o = 0; o < objects.size(); o++) {
            objects[o] = std::make_shared<Buffer>(root->device, P.plan.object_bytes[o]);
            inner->held += P.plan.object_bytes[o];
        }
        rt_device* dev = root->device.raw();
        size_t launches = 0;
        for (Node* n : P.order) {
            auto st = P.step_of.find(n);
            if (st != P.step_of.end()) {
                const planner::Step& step = P.steps[st->second];
                const int obj = P.plan.object_of.at(n->id);
                if (step.inplace >= 0) {
                    n->storage = P.step_reads[st->second][(size_t)step.inplace]->storage;
                } else if (obj >= 0) {
                    n->storage = objects[(size_t)obj];
                } else {
                    n->storage = std::make_shared<Buffer>(n->device, step.bytes);
                    inner->held += step.bytes;
                }
                auto f = P.fused.find(n);
                if (f != P.fused.end()) run_fused(n, f->second, launches);
                else run(n, launches);
            } else if (!n->storage && !P.skip.count(n)) {
                run(n, launches);                                  // a view (no launch)
            }
        }
        check_rt(rt_sync(dev), "rt_sync");
        inner->launches = launches;
        root->last_launches = launches;
        // the executable now owns what the launches touch; the nodes look as they do after resolve()
        for (Node* n : P.order) inner->storage.push_back(n->storage);
        for (const std::vector<Node*>& dead_list : P.release_at)
            for (Node* dead : dead_list) dead->storage.reset();
        if (launches >= GRAPH_MIN_LAUNCHES) {
            check_rt(rt_capture_begin(dev), "rt_capture_begin");
            try {
                replay(*inner);
            } catch (...) {                                        // leave the device usable: close the capture, drop what it recorded
                rt_graph* g = nullptr;
                if (rt_capture_end(dev, &g) == RT_OK && g) rt_graph_destroy(g);
                throw;
            }
            check_rt(rt_capture_end(dev, &inner->graph), "rt_capture_end");
        }
        Executable exe;
        exe.inner_ = inner;
        return exe;
    }
};

void Executable::dispatch(bool wait) const {
    if (!inner_) throw Error("NullExecutable", "dispatch on an empty executable");
    if (inner_->graph) check_rt(rt_graph_launch(inner_->device.raw(), inner_->graph), "rt_graph_launch");
    else if (inner_->launches) Resolver::replay(*inner_);
    if (wait) check_rt(rt_sync(inner_->device.raw()), "rt_sync");
}
size_t Executable::launches() const { return inner_ ? inner_->launches : 0; }
size_t Executable::held_bytes() const { return inner_ ? inner_->held : 0; }

Executable Tensor::compile() const {
    if (!node_) throw Error("NullTensor", "compile on an empty tensor");
    // a tensor that has its storage already has nothing left to run: an executable of it would replay nothing
    if (node_->storage && !node_->srcs.empty()) throw Error("AlreadyResolved", "compile() wants a tensor that has not been resolved yet");
    return Resolver::compile(node_);
}

void Tensor::update_from_host(const void* data) const {
    if (!resolved()) throw Error("Unresolved", "update_from_host needs a tensor that has storage");
    check_rt(rt_h2d(node_->device.raw(), node_->storage->ptr, data, storage_bytes(shape(), dt())), "rt_h2d");
}

MemoryPlan Tensor::memory_plan() const {
    if (!node_) throw Error("NullTensor", "memory_plan on an empty tensor");
    Resolver::Prepared P = Resolver::prepare(node_.get());
    MemoryPlan out;
    out.object_bytes = P.plan.object_bytes;
    for (size_t i = 0; i < P.steps.size(); i++) {
        MemoryPlan::Entry e;
        e.id = P.steps[i].id;
        e.bytes = P.steps[i].bytes;
        e.object = P.plan.object_of.at(e.id);
        e.source = P.plan.source_of.at(e.id);
        out.entries.push_back(e);
    }
    return out;
}

Tensor Tensor::resolve() const {
    if (!node_) throw Error("NullTensor", "resolve on an empty tensor");
    Resolver::resolve(node_.get());
    return *this;
}

void Tensor::to_host(void* out) const {
    if (!resolved()) throw Error("Unresolved", "to_host needs a resolved tensor (call resolve() first)");
    check_rt(rt_d2h(node_->device.raw(), out, node_->storage->ptr, storage_bytes(shape(), dt())), "rt_d2h");
}

}  // namespace ratchet
