// Internal definitions shared by the HIP translation units of libratchet_hip.so (gfx950 only).
#ifndef RT_INTERNAL_H
#define RT_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/ratchet_hip.h"
#include "../../include/ratchet_hip_debug.h"

constexpr size_t RT_SM_ROW_SUMS = 1u << 19;
constexpr size_t RT_SM_MASK_TILES = 1u << 18;   // 512-column tiles of a mask that the streaming softmax can classify per launch
constexpr size_t RT_SM_TILES_HEAD = 16;         // entries in front of them that always read "load this tile"
// An operand that repeats over the leading dims of the output (an [S, T] mask under B * H heads) is re-read once per
// repeat.  Hardware block b runs on XCD b % 8, so in the plain block order each of the eight L2s (4 MiB) sees one eighth
// of that operand and keeps it between the repeats as long as the whole operand is under about 28 MiB; from there on the
// kernels that re-read such an operand order their blocks so that all repeats of a slab run back to back on one XCD.
// Below, that order loses to the plain one (it hops between the repeats every few hundred KiB): scores + mask on
// [1,32,2560,2560] f16 135 against 156 us, [4,32,1024,1024] 87 against 100; above, it is what keeps the re-reads in
// L2 at all ([1,32,4096,4096] 338 against 440 us, [1,8,6144,6144] 206 against 244).
constexpr uint64_t RT_XCD_ORDER_MIN_BYTES = 28ull << 20;

struct rt_device {
    int ordinal;
    hipStream_t stream;
    int num_cus;
    double wall_clock_hz;   // rate of the device's constant-frequency wall clock (s_memrealtime), 100 MHz on this chip
    uint32_t debug_softmax_pace;   // test hook (rt_debug_softmax_pace): replaces the computed pace of the streaming softmax, 0 = none
    // GroupNorm partial statistics: {mean, m2, count} triples, one per (group, split)
    float* gn_scratch;
    size_t gn_scratch_bytes;
    // this device's copy of the fixed partial-statistics array behind rt_group_norm_static (rt_norm.hip), resolved at create
    float* gn_static_ptr;
    // 65536-entry 16-bit -> 16-bit lookup tables, built on first use by the exact kernels ([0] = f16, [1] = bf16)
    uint16_t* unary_lut[2][RT_UNARY_COUNT];
    // the same for "widen to f32, f32 op, round once" (the full -> op -> cast caller pattern)
    uint16_t* unary_lut_via32[2][RT_UNARY_COUNT];
    int lut_attr_set;
    int gated_attr_set[2];
    unsigned gn_lds_attr_set;
    unsigned np_attr_set;   // 16-bit norm instantiations (LDS-resident rows) whose dynamic-LDS limit has been raised on this device
    uint64_t sp_attr_set;   // streaming softmax instantiations whose dynamic-LDS limit has been raised on this device
    uint64_t sp_ragged_attr_set;   // the same for the ragged-row variants
    uint32_t sp_pair_attr_set;     // the same for the variants that take one mask row for two heads
    unsigned ry_attr_set;          // the same for the one-wave-per-row softmax (rt_softmax_replay.hip)
    uint16_t rp_resident[2][9];    // wave-per-row RMSNorm: blocks of an instantiation ([f16, bf16][vectors per lane]) that one CU holds; 0 = not asked yet
    // row sums of one launch of the streaming softmax's ragged-row variant (RT_SM_ROW_SUMS 16-bit values, allocated with the device)
    uint16_t* sm_row_sums;
    // one word per 512-column tile of the mask of a masked streaming softmax (behind the row sums, in the same allocation): the
    // tile's value twice when all its elements are equal, 0xffffffff when the tile has to be loaded; the first RT_SM_TILES_HEAD
    // words always hold 0xffffffff
    uint32_t* sm_mask_tiles;
    // caching allocator behind rt_malloc / rt_free (defined in rt_device.hip)
    struct rt_pool* pool;
    int capturing;          // between rt_capture_begin and rt_capture_end
};

struct rt_event {
    hipEvent_t ev;
    int ordinal;
};

// error reporting (thread-local message)
int rt_fail(int status, const char* fmt, ...);
int rt_fail_hip(hipError_t e, const char* what);

#define RT_HIP(call)                                         \
    do {                                                     \
        hipError_t _e = (call);                              \
        if (_e != hipSuccess) return rt_fail_hip(_e, #call); \
    } while (0)

#define RT_REQUIRE(cond, status, ...)                          \
    do {                                                       \
        if (!(cond)) return rt_fail((status), __VA_ARGS__);    \
    } while (0)

// Calls that wait for the device or ask the driver for memory cannot be recorded into a graph.
#define RT_NO_CAPTURE(dev, who)                                                                                        \
    do {                                                                                                               \
        if ((dev)->capturing) return rt_fail(RT_ERR_CAPTURE, "%s cannot run while the device is capturing a graph", who); \
    } while (0)

// Returns rt_fail_hip(...) if the launch that was just enqueued was rejected.
#define RT_CHECK_LAUNCH(name)                                   \
    do {                                                        \
        hipError_t _e = hipGetLastError();                      \
        if (_e != hipSuccess) return rt_fail_hip(_e, name);     \
    } while (0)

static inline bool rt_is_float_dt(int dt) { return dt == RT_F32 || dt == RT_F16 || dt == RT_BF16; }
static inline int rt_dt_bytes(int dt) {
    switch (dt) {
        case RT_F32: case RT_I32: case RT_U32: return 4;
        case RT_F16: case RT_BF16: return 2;
        default: return 0;
    }
}
static inline bool rt_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// native clang vectors: arrays of these stay in registers (arrays of HIP's uint4 class type can end up in LDS scratch)
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

// Streaming accesses for data that is touched once: the non-temporal hint keeps it from displacing cache lines and,
// measured on MI355X with a 1 GiB copy, lifts a kernel from 5.7-6.2 TB/s to 6.5 TB/s.  Operands that are re-read
// (broadcast rows, tables, a second pass over the same tile) keep ordinary loads.
template <typename V> __device__ __forceinline__ V ld_stream(const V* p) { return __builtin_nontemporal_load(p); }
template <typename V> __device__ __forceinline__ void st_stream(V* p, V v) { __builtin_nontemporal_store(v, p); }

// the kernels index elements with 64-bit integers but grid sizes are 32-bit; 2^40 elements is far beyond 288 GB
static const uint64_t RT_MAX_NUMEL = 1ull << 40;

// Makes dev's ordinal current.  Every entry point calls it first.
int rt_enter(rt_device* dev);

// rt_norm.hip: resolves the device-side address of the fixed GroupNorm scratch array for the current device
int rt_norm_device_init(rt_device* dev);

// Device pointer to the 65536-entry table out[bits(x)] = bits(op(x)) for a 16-bit type (type_index 0 = f16, 1 = bf16),
// built on first use by running the exact unary kernel over all bit patterns (blocks until the table is ready).
int rt_unary_table(rt_device* dev, int type_index, int op, const uint16_t** out);

// The streaming 16-bit softmax (rt_softmax_stream_f16.hip / rt_softmax_stream_bf16.hip).  mask == nullptr: plain softmax;
// otherwise the mask has `period` rows of `cols` columns and repeats every `period` rows of x.  Returns RT_OK with
// *done = false when the shape does not fit the kernel (the caller then takes another path).
int rt_softmax_stream_f16(rt_device* dev, const void* x, const void* mask, uint64_t period, void* y, uint64_t rows, uint32_t cols, bool* done);
int rt_softmax_stream_bf16(rt_device* dev, const void* x, const void* mask, uint64_t period, void* y, uint64_t rows, uint32_t cols, bool* done);

// The f16 reference softmax for a few long rows, one wave per row (rt_softmax_replay.hip); arguments as above
int rt_softmax_replay_f16(rt_device* dev, const void* x, const void* mask, uint64_t period, void* y, uint64_t rows, uint32_t cols, bool* done);

// ---------------------------------------------------------------------------------------------------------
// u32 division by a launch-time constant: q = (n * m) >> (32 + s), exact for all n < 2^32 (round-up method)
// ---------------------------------------------------------------------------------------------------------
struct FastDiv {
    uint32_t d;   // divisor
    uint32_t m;   // magic multiplier
    uint32_t s;   // post shift
    uint32_t add; // 1: use the (n + hi) / 2 correction path
};
static inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    if (d == 1) { f.m = 0; f.s = 0; f.add = 2; return f; }   // add == 2: identity
    uint32_t l = 0;
    while ((1ull << l) < d) l++;                              // l = ceil(log2 d)
    const uint64_t m = ((1ull << 32) * ((1ull << l) - d)) / d + 1;
    f.m = (uint32_t)m;
    f.s = l - 1;
    f.add = 1;
    return f;
}
#ifdef __HIPCC__
__device__ __forceinline__ uint32_t fd_div(uint32_t n, const FastDiv& f) {
    if (f.add == 2) return n;
    const uint32_t t = __umulhi(n, f.m);
    return (t + ((n - t) >> 1)) >> f.s;
}
__device__ __forceinline__ void fd_divmod(uint32_t n, const FastDiv& f, uint32_t& q, uint32_t& r) {
    q = fd_div(n, f);
    r = n - q * f.d;
}
#endif

#endif
