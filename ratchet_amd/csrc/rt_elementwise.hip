// Elementwise kernels: binary (contiguous and broadcast-fused), unary, cast.
//
// All of them are streaming kernels bounded by HBM bandwidth: every lane moves 16 bytes per access (dwordx4) with the
// non-temporal hint, and a 256-thread block covers one 4 KiB slab per operand.  Measured on MI355X (1 GiB copy) that
// shape reaches 6.5 TB/s; blocks that cover 8-16 KiB reach 6.1-6.2 TB/s and the same without the hint 5.7 TB/s.
// Arithmetic follows rt_arith.h.
#include <type_traits>

#include "rt_arith.h"
#include "rt_internal.h"
#include "rt_pace.h"

namespace {

constexpr int BLOCK = 256;
constexpr int UNROLL = 1;
// below this many elements the table fill (128 KiB per CU) costs more than computing
constexpr uint64_t RT_LUT_MIN_NUMEL = 1u << 21;

// ------------------------------------------------------------------------------------------------ binary, contiguous
template <typename T, int OP>
__global__ void __launch_bounds__(BLOCK) binary_vec_kernel(const T* __restrict__ a, const T* __restrict__ b, T* y,
                                                           uint64_t numel) {
    constexpr int VE = 16 / sizeof(T);
    const uint64_t nvec = numel / VE;
    const v4u* av = reinterpret_cast<const v4u*>(a);
    const v4u* bv = reinterpret_cast<const v4u*>(b);
    v4u* yv = reinterpret_cast<v4u*>(y);
    const uint64_t base = (uint64_t)blockIdx.x * (BLOCK * UNROLL) + threadIdx.x;
    Vec16<T> ra[UNROLL], rb[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const uint64_t i = base + (uint64_t)k * BLOCK;
        if (i < nvec) {
            ra[k].u = ld_stream(av + i);
            rb[k].u = ld_stream(bv + i);
        }
    }
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const uint64_t i = base + (uint64_t)k * BLOCK;
        if (i < nvec) {
            Vec16<T> r;
#pragma unroll
            for (int e = 0; e < VE; e++) r.e[e] = ar_binary<OP, T>(ra[k].e[e], rb[k].e[e]);
            st_stream(yv + i, r.u);
        }
    }
    if (blockIdx.x == 0) {                              // the numel % VE trailing elements
        const uint64_t i = nvec * VE + threadIdx.x;
        if (i < numel) y[i] = ar_binary<OP, T>(a[i], b[i]);
    }
}

// fallback for pointers that are not 16-byte aligned
template <typename T, int OP>
__global__ void __launch_bounds__(BLOCK) binary_scalar_kernel(const T* a, const T* b, T* y, uint64_t numel) {
    const uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < numel) y[i] = ar_binary<OP, T>(a[i], b[i]);
}

// ------------------------------------------------------------------------------------------------ binary, broadcast
// y_shape = [d0, d1, d2, d3]; a/b strides in elements, 0 on broadcast dims.  One thread per VE consecutive outputs of
// the last dimension; an operand whose last-dim stride is 0 is loaded once and splatted.  The output and the
// full-size operand are streamed in plain linear order; the broadcast operand (a bias row, an [S,S] mask under 32
// heads) is re-read through L2 / Infinity Cache.  Measured on MI355X this beats a kernel that keeps the broadcast
// operand in registers and hops between heads (5.4 vs 4.6 TB/s on [1,32,4096,4096] + [4096,4096]): HBM prefers
// one long stream per block to 32 interleaved ones.
struct BcastArgs {
    FastDiv cv;        // column vectors per row = d3 / VE
    FastDiv d2, d1;
    uint32_t as[4], bs[4];
    uint32_t nvec;     // total vectors
    // XCD-aware block order for a large operand repeated over the leading dims (an [S,S] mask under H heads): hardware
    // block b runs on XCD b % 8, so the `reps` blocks that need the same 4 KiB slab of that operand are given to one
    // XCD back to back and its L2 fetches the slab once.  An XCD walks 2^chunk_log2 of its slabs per repeat before it
    // moves to the next repeat (measured on [1,32,4096,4096] + [4096,4096]: 64 slabs 363 us, 4 slabs 366 us, 1 slab
    // 376 us, 16 slabs 416 us, identity order 404 us; with one vector per thread, where a slab is 4 KiB: 128 slabs
    // 342 us, 256 slabs 349 us, 512 slabs 356 us, 64 slabs 382 us, 32 slabs 422 us, 1024 slabs 445 us: 512 KiB of the
    // repeated operand per XCD either way).  slabs == 0: identity order.
    FastDiv reps;
    uint32_t slabs;    // blocks per repeat
    uint32_t chunk_log2;
};

constexpr int BC_UNROLL = 2;
constexpr uint64_t BC_ONE_FROM_VECS = 1ull << 26;
constexpr uint32_t XCDS = 8;

// ONCE: bit 0 / bit 1 set when a / b has no broadcast dim, so each of its elements is read exactly once and its loads
// carry the non-temporal hint.  (A compile-time choice: with `once ? ld_stream(q) : *q` on a run-time flag the compiler
// merges the two loads into one ordinary load, and a 1 GiB operand then floods L2 and the memory-side cache.)
template <typename T, int OP, int VE, int ONCE, int U = BC_UNROLL>
__global__ void __launch_bounds__(BLOCK) binary_bcast_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                             T* __restrict__ y, BcastArgs p) {
    uint32_t blk = blockIdx.x;
    if (p.slabs) {
        uint32_t rep, chunk;
        const uint32_t idx = blk / XCDS;
        fd_divmod(idx >> p.chunk_log2, p.reps, chunk, rep);
        blk = rep * p.slabs + ((chunk << p.chunk_log2) + (idx & ((1u << p.chunk_log2) - 1))) * XCDS + (blk % XCDS);
    }
    const uint32_t base = blk * (BLOCK * U) + threadIdx.x;
    if (U == 1 && base >= p.nvec) return;
    // every load of the thread's U vectors is issued before the first store
    T ra[U][VE], rb[U][VE];
#pragma unroll
    for (int k = 0; k < U; k++) {
        const uint32_t v = base + k * BLOCK;
        if (v >= p.nvec) break;
        uint32_t row, col, i0, i1, i2, t;
        fd_divmod(v, p.cv, row, col);
        fd_divmod(row, p.d2, t, i2);
        fd_divmod(t, p.d1, i0, i1);
        const uint64_t ao = (uint64_t)i0 * p.as[0] + (uint64_t)i1 * p.as[1] + (uint64_t)i2 * p.as[2] +
                            (uint64_t)col * VE * p.as[3];
        const uint64_t bo = (uint64_t)i0 * p.bs[0] + (uint64_t)i1 * p.bs[1] + (uint64_t)i2 * p.bs[2] +
                            (uint64_t)col * VE * p.bs[3];
        if (VE > 1 && p.as[3] == 1) {
            Vec16<T> t16;
            const v4u* q = reinterpret_cast<const v4u*>(a + ao);
            t16.u = (ONCE & 1) ? ld_stream(q) : *q;
#pragma unroll
            for (int e = 0; e < VE; e++) ra[k][e] = t16.e[e];
        } else if (p.as[3] == 0) {
            const T one = a[ao];                                  // broadcast along the last dim: one load, splatted
#pragma unroll
            for (int e = 0; e < VE; e++) ra[k][e] = one;
        } else {
#pragma unroll
            for (int e = 0; e < VE; e++) ra[k][e] = a[ao + (uint64_t)e * p.as[3]];
        }
        if (VE > 1 && p.bs[3] == 1) {
            Vec16<T> t16;
            const v4u* q = reinterpret_cast<const v4u*>(b + bo);
            t16.u = (ONCE & 2) ? ld_stream(q) : *q;
#pragma unroll
            for (int e = 0; e < VE; e++) rb[k][e] = t16.e[e];
        } else if (p.bs[3] == 0) {
            const T one = b[bo];                                  // broadcast along the last dim: one load, splatted
#pragma unroll
            for (int e = 0; e < VE; e++) rb[k][e] = one;
        } else {
#pragma unroll
            for (int e = 0; e < VE; e++) rb[k][e] = b[bo + (uint64_t)e * p.bs[3]];
        }
    }
#pragma unroll
    for (int k = 0; k < U; k++) {
        const uint32_t v = base + k * BLOCK;
        if (v >= p.nvec) break;
        const uint64_t yo = (uint64_t)v * VE;
        if (VE > 1) {
            Vec16<T> t16;
#pragma unroll
            for (int e = 0; e < VE; e++) t16.e[e] = ar_binary<OP, T>(ra[k][e], rb[k][e]);
            // U == 1: the compiler drops the non-temporal hint of the builtin when the kernel has a single store (and the
            // lines an ordinary 1 GiB store leaves in the caches cost the kernels behind it more than this one gains)
            if (U == 1) asm volatile("global_store_dwordx4 %0, %1, off nt" ::"v"(reinterpret_cast<v4u*>(y + yo)), "v"(t16.u) : "memory");
            else st_stream(reinterpret_cast<v4u*>(y + yo), t16.u);
        } else {
            y[yo] = ar_binary<OP, T>(ra[k][0], rb[k][0]);
        }
    }
}

// Rows that are not whole vectors (a last dim of 1001), one operand of y's own shape and the other broadcast: the output
// and the full operand are taken as flat arrays in 16-byte vectors, whatever the row length, and only the broadcast
// operand is read element by element (it is the small one and stays in the caches).  A_FULL: a is the full operand.
// [4,4096,1001] + [1001] in f16: 33 -> 20 us against the element-wise kernel, + [4,4096,1]: 33 -> 14 us; f32: 5.2 TB/s.
template <typename T, int OP, bool A_FULL>
__global__ void __launch_bounds__(BLOCK) binary_flat_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ y, BcastArgs p,
                                                            uint64_t numel) {
    constexpr int VE = 16 / sizeof(T);
    const T* full = A_FULL ? a : b;
    const T* part = A_FULL ? b : a;
    const uint32_t* ps = A_FULL ? p.bs : p.as;
    const uint64_t v = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    const uint64_t f0 = v * VE;
    if (f0 >= numel) return;
    // position of the vector's first element; p.cv divides by the whole last dim here
    uint32_t row, col, i0, i1, i2, t;
    fd_divmod((uint32_t)f0, p.cv, row, col);
    fd_divmod(row, p.d2, t, i2);
    fd_divmod(t, p.d1, i0, i1);
    uint64_t off = (uint64_t)i0 * ps[0] + (uint64_t)i1 * ps[1] + (uint64_t)i2 * ps[2] + (uint64_t)col * ps[3];
    const uint32_t d3 = p.cv.d;
    T pv[VE];
#pragma unroll
    for (int e = 0; e < VE; e++) {
        pv[e] = part[f0 + e < numel ? off : 0];              // (nothing is read past the tensor's last element)
        off += ps[3];
        if (++col == d3 && e + 1 < VE) {                     // the next element starts a row
            col = 0;
            fd_divmod((uint32_t)f0 + e + 1, p.cv, row, t);
            fd_divmod(row, p.d2, t, i2);
            fd_divmod(t, p.d1, i0, i1);
            off = (uint64_t)i0 * ps[0] + (uint64_t)i1 * ps[1] + (uint64_t)i2 * ps[2];
        }
    }
    if (f0 + VE <= numel) {
        Vec16<T> fv, out;
        fv.u = ld_stream(reinterpret_cast<const v4u*>(full + f0));
#pragma unroll
        for (int e = 0; e < VE; e++) out.e[e] = A_FULL ? ar_binary<OP, T>(fv.e[e], pv[e]) : ar_binary<OP, T>(pv[e], fv.e[e]);
        st_stream(reinterpret_cast<v4u*>(y + f0), out.u);
    } else {
        for (int e = 0; e < VE && f0 + e < numel; e++)       // the tensor's last, partial vector
            y[f0 + e] = A_FULL ? ar_binary<OP, T>(full[f0 + e], pv[e]) : ar_binary<OP, T>(pv[e], full[f0 + e]);
    }
}

// ------------------------------------------------------------------------------------------------ unary
// VIA32: the caller pattern x.full().<op>().cast(dt) on a 16-bit tensor in one pass: widen, the f32 op, one rounding
template <typename T, int OP, bool VIA32> __device__ __forceinline__ T apply_unary(T v, const uint64_t* tab = rt_exp2f_tab) {
    if (VIA32) return Ar<T>::conv(ar_unary<OP, float>(Ar<T>::widen(v), tab));
    return ar_unary<OP, T>(v, tab);
}

template <typename T, int OP, bool VIA32>
__global__ void __launch_bounds__(BLOCK) unary_vec_kernel(const T* __restrict__ x, T* y, uint64_t numel) {
    constexpr int VE = 16 / sizeof(T);
    const uint64_t nvec = numel / VE;
    const v4u* xv = reinterpret_cast<const v4u*>(x);
    v4u* yv = reinterpret_cast<v4u*>(y);
    const uint64_t base = (uint64_t)blockIdx.x * (BLOCK * UNROLL) + threadIdx.x;
    Vec16<T> rx[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const uint64_t i = base + (uint64_t)k * BLOCK;
        if (i < nvec) rx[k].u = ld_stream(xv + i);
    }
    // exp, SiLU and sigmoid look 2^(i/32) up once per element, log its (1/c, log c): from a copy of the table in LDS
    constexpr bool TAB = ar_unary_uses_exp(OP) || ar_unary_uses_log(OP);
    __shared__ uint64_t exp_tab[TAB ? 32 : 1];
    const uint64_t* tab = rt_exp2f_tab;
    if (TAB) {
        if (threadIdx.x < 32)
            exp_tab[threadIdx.x] = ar_unary_uses_log(OP) ? __builtin_bit_cast(uint64_t, rt_logf_tab[threadIdx.x]) : rt_exp2f_tab[threadIdx.x];
        __syncthreads();
        tab = exp_tab;
    }
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const uint64_t i = base + (uint64_t)k * BLOCK;
        if (i < nvec) {
            Vec16<T> r;
#pragma unroll
            for (int e = 0; e < VE; e++) r.e[e] = apply_unary<T, OP, VIA32>(rx[k].e[e], tab);
            st_stream(yv + i, r.u);
        }
    }
    if (blockIdx.x == 0) {
        const uint64_t i = nvec * VE + threadIdx.x;
        if (i < numel) y[i] = apply_unary<T, OP, VIA32>(x[i], tab);
    }
}

template <typename T, int OP, bool VIA32>
__global__ void __launch_bounds__(BLOCK) unary_scalar_kernel(const T* x, T* y, uint64_t numel) {
    const uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < numel) y[i] = apply_unary<T, OP, VIA32>(x[i]);
}

// ------------------------------------------------------------------------------------------------ unary via lookup table
// A 16-bit type has only 65536 values, so any unary op on it is a 128 KiB table.  The table is produced once per
// (device, op, type) by the exact kernel above applied to all 65536 bit patterns, which makes the lookup bit-identical
// to computing.  Each block copies the table into LDS (gfx950 has 160 KiB per CU) and then streams its share of the
// tensor: 16-byte loads, eight ds_read_u16 lookups per load, 16-byte stores.  The transcendental ops (fdlibm tanh, the
// double-precision exp, two divisions for GELU/SiLU) cost 5-10x the HBM time when computed per element; the lookup
// costs less than the memory traffic.
constexpr int LUT_BLOCK = 1024;
constexpr int LUT_UNROLL = 1;                      // vectors per thread and tile
constexpr int LUT_DEPTH = 3;                       // tiles of loads in flight
constexpr int LUT_TILE = LUT_BLOCK * LUT_UNROLL;   // vectors per tile
constexpr size_t LUT_BYTES = 65536 * sizeof(uint16_t);

__global__ void iota16_kernel(uint16_t* p) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < 65536) p[i] = (uint16_t)i;
}

// one 32-bit word = two elements through the table
__device__ __forceinline__ uint32_t lut_pair(const uint16_t* lut, uint32_t w) {
    const uint32_t lo = lut[w & 0xffffu];
    const uint32_t hi = lut[w >> 16];
    return lo | (hi << 16);
}

// The tensor is cut into tiles of LUT_BLOCK * U vectors; block b takes tiles b, b + gridDim.x, ...  The loads of a block's
// next D tiles are in flight (a ring in registers) during the lookups of the current one, and those of its first D tiles
// during the table copy, so the HBM reads run underneath the LDS phases instead of after them: with every wave of the
// chip released by the same barrier, a loop that loads, looks up and stores in turn alternates between a memory-bound
// and an LDS-bound phase and pays for both.  One vector per thread and tile (16 KiB tiles, three in flight) measured
// best inside the benchmark step: GELU on 84 MB 20.4 -> 18.3 us, SiLU on 134 MB 27.6 -> 25.0 us against 64 KiB tiles
// with one in flight (depths 2 to 5 are level; 32 and 64 KiB tiles at any depth gain on the first only).
// Large tensors: every wave holds its steps to a period (rt_pace.h); the blocks start out of phase.  pace == 0: unpaced.
// On 16-bit GELU: 1 GiB 205 -> 173 us (a copy: 163), 512 MiB 100 -> 90 (83), 256 MiB 50 -> 49; on 128 MiB and below the
// kernel is over before a pace can help and loses 2 us to it, so the unary launcher paces from 32 steps per block on.  The
// gated multiply (three streams, 48 KiB a step): [32768,8192] 271 -> 252 us (a copy of as many bytes: 247), [16384,11008]
// 181 -> 172 (167), [16384,8192] 133.5 -> 129.6, but [8192,8192], 32 steps, 66.5 -> 69.2: paced from 64 steps on.
struct LutPace {
    uint32_t pace;           // ticks of the wall clock between two steps of a block
    uint32_t phase_fx;       // pace / grid in 16.16 fixed point
};
constexpr uint32_t LUT_PACE_MIN_STEPS = 32, GATED_PACE_MIN_STEPS = 64;
struct LutClock {
    uint32_t t_step = 0, t_last = 0, t_avg = 0, t_slow = 0;
    __device__ __forceinline__ explicit LutClock(const LutPace& pc) {
        if (pc.pace) {
            t_avg = pc.pace;
            t_slow = pc.pace + pc.pace / 5;
            t_last = __builtin_amdgcn_readfirstlane(rt_pace_clock());
            t_step = t_last - pc.pace + ((blockIdx.x * pc.phase_fx) >> 16);
            t_last -= pc.pace;
        }
    }
    __device__ __forceinline__ void step(const LutPace& pc) {
        if (pc.pace) rt_pace_step(t_step, t_last, t_avg, pc.pace, t_slow);
    }
};
static LutPace lut_pace_for(const rt_device* dev, uint64_t blocks, uint64_t steps_per_block, uint32_t min_steps, double bytes_per_step) {
    LutPace pc = {0, 0};
    if (blocks == (uint64_t)dev->num_cus && steps_per_block >= min_steps) {
        pc.pace = (uint32_t)(bytes_per_step * (double)blocks / RT_PACE_BYTES_PER_S * dev->wall_clock_hz + 0.5);
        pc.phase_fx = pc.pace > 0xffffu ? 0 : (pc.pace << 16) / (uint32_t)blocks;
    }
    return pc;
}

template <int U, int D>
__global__ void __launch_bounds__(LUT_BLOCK) unary_lut_kernel(const uint16_t* __restrict__ table, const uint16_t* __restrict__ x,
                                                                   uint16_t* y, uint64_t numel, LutPace pc) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
    constexpr int TILE = LUT_BLOCK * U;
    const uint64_t nvec = numel / 8;
    const uint64_t tiles = nvec / TILE;
    const v4u* xv = reinterpret_cast<const v4u*>(x);
    v4u* yv = reinterpret_cast<v4u*>(y);
    uint64_t t = blockIdx.x;
    v4u ring[D][U];
#pragma unroll
    for (int d = 0; d < D; d++) {
        const uint64_t td = t + (uint64_t)d * gridDim.x;
        if (td < tiles) {
#pragma unroll
            for (int k = 0; k < U; k++) ring[d][k] = ld_stream(xv + td * TILE + k * LUT_BLOCK + threadIdx.x);
        }
    }
    {
        const v4u* src = reinterpret_cast<const v4u*>(table);
        v4u* dst = reinterpret_cast<v4u*>(lut);
#pragma unroll
        for (int i = 0; i < (int)(LUT_BYTES / 16 / LUT_BLOCK); i++) dst[i * LUT_BLOCK + threadIdx.x] = src[i * LUT_BLOCK + threadIdx.x];
    }
    __syncthreads();
    LutClock clk(pc);
    while (t < tiles) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (t >= tiles) break;
            clk.step(pc);
            v4u cur[U];
#pragma unroll
            for (int k = 0; k < U; k++) cur[k] = ring[d][k];
            const uint64_t tn = t + (uint64_t)D * gridDim.x;
            if (tn < tiles) {
#pragma unroll
                for (int k = 0; k < U; k++) ring[d][k] = ld_stream(xv + tn * TILE + k * LUT_BLOCK + threadIdx.x);
            }
#pragma unroll
            for (int k = 0; k < U; k++) {
                v4u out;
#pragma unroll
                for (int w = 0; w < 4; w++) out[w] = lut_pair(lut, cur[k][w]);
                st_stream(yv + t * TILE + k * LUT_BLOCK + threadIdx.x, out);
            }
            t += gridDim.x;
        }
    }
    if (blockIdx.x == tiles % gridDim.x) {
        for (uint64_t i = tiles * TILE + threadIdx.x; i < nvec; i += LUT_BLOCK) {
            const v4u in = ld_stream(xv + i);
            v4u out;
#pragma unroll
            for (int w = 0; w < 4; w++) out[w] = lut_pair(lut, in[w]);
            st_stream(yv + i, out);
        }
        const uint64_t i = nvec * 8 + threadIdx.x;
        if (i < numel) y[i] = lut[x[i]];
    }
}

// ------------------------------------------------------------------------------------------------ gated multiply
// y[r, c] = up[r, c] * act(gate[r, c]) with act = cast(op(full(gate))), the feed-forward gate of phi3
// (ratchet-models/src/phi3/mlp.rs:32-38: up.mul(gate.full().silu().cast(dt)) on the two halves of one projection).
// gate and up are row-strided views, so the two slices are never materialised.  act comes from the same kind of LDS
// table as unary_lut_kernel (built by the exact kernels for "widen, f32 op, round"); the product is the type's own.
struct GatedArgs {
    FastDiv cv;              // vectors (or elements, scalar kernel) per row
    uint64_t gs, us;         // row strides of gate and up, in elements
    uint64_t nvec;           // rows * vectors per row
};

// Like unary_lut_kernel: one vector of gate and one of up per thread and step, the loads of the next LUT_DEPTH steps in
// flight during the lookups of the current one and those of the first steps during the table copy.
template <typename T, bool PACED>
__global__ void __launch_bounds__(LUT_BLOCK) gated_lut_kernel(const uint16_t* __restrict__ table, const T* __restrict__ gate,
                                                              const T* __restrict__ up, T* __restrict__ y, GatedArgs p, LutPace pc) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
    const uint64_t stride = (uint64_t)gridDim.x * LUT_BLOCK;
    uint64_t v = (uint64_t)blockIdx.x * LUT_BLOCK + threadIdx.x;
    v4u rg[LUT_DEPTH], ru[LUT_DEPTH];
    auto fetch = [&](uint64_t at, v4u& g, v4u& u) {
        uint32_t row, c;
        fd_divmod((uint32_t)at, p.cv, row, c);
        g = ld_stream(reinterpret_cast<const v4u*>(gate + (uint64_t)row * p.gs) + c);
        u = ld_stream(reinterpret_cast<const v4u*>(up + (uint64_t)row * p.us) + c);
    };
#pragma unroll
    for (int d = 0; d < LUT_DEPTH; d++)
        if (v + d * stride < p.nvec) fetch(v + d * stride, rg[d], ru[d]);
    {
        const v4u* src = reinterpret_cast<const v4u*>(table);
        v4u* dst = reinterpret_cast<v4u*>(lut);
#pragma unroll
        for (int i = 0; i < (int)(LUT_BYTES / 16 / LUT_BLOCK); i++) dst[i * LUT_BLOCK + threadIdx.x] = src[i * LUT_BLOCK + threadIdx.x];
    }
    __syncthreads();
    if constexpr (!PACED) {
        while (v < p.nvec) {
#pragma unroll
            for (int d = 0; d < LUT_DEPTH; d++) {
                if (v >= p.nvec) break;
                Vec16<T> g, u, o;
                g.u = rg[d];
                u.u = ru[d];
                const uint64_t vn = v + LUT_DEPTH * stride;
                if (vn < p.nvec) fetch(vn, rg[d], ru[d]);
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const uint32_t lo = lut[g.u[w] & 0xffffu];
                    const uint32_t hi = lut[g.u[w] >> 16];
                    g.u[w] = lo | (hi << 16);
                }
#pragma unroll
                for (int e = 0; e < 8; e++) o.e[e] = Ar<T>::mul(u.e[e], g.e[e]);
                st_stream(reinterpret_cast<v4u*>(y) + v, o.u);
                v += stride;
            }
        }
        return;
    }
    LutClock clk(pc);
    // paced: the loop runs on the index of the wave's first lane, which is the same for the whole wave (the clock lives in
    // scalar registers); only the wave that holds the tensor's end has lanes without an element
    uint64_t v0 = (uint64_t)blockIdx.x * LUT_BLOCK + __builtin_amdgcn_readfirstlane(threadIdx.x & ~63u);
    while (v0 < p.nvec) {
#pragma unroll
        for (int d = 0; d < LUT_DEPTH; d++) {
            if (v0 >= p.nvec) break;
            clk.step(pc);
            if (v < p.nvec) {
                Vec16<T> g, u, o;
                g.u = rg[d];
                u.u = ru[d];
                const uint64_t vn = v + LUT_DEPTH * stride;
                if (vn < p.nvec) fetch(vn, rg[d], ru[d]);
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const uint32_t lo = lut[g.u[w] & 0xffffu];
                    const uint32_t hi = lut[g.u[w] >> 16];
                    g.u[w] = lo | (hi << 16);
                }
#pragma unroll
                for (int e = 0; e < 8; e++) o.e[e] = Ar<T>::mul(u.e[e], g.e[e]);
                st_stream(reinterpret_cast<v4u*>(y) + v, o.u);
            }
            v += stride;
            v0 += stride;
        }
    }
}

// mid-size tensors: the table read where it lies (see unary_table_gather_kernel), one vector per thread
template <typename T>
__global__ void __launch_bounds__(BLOCK) gated_gather_kernel(const uint16_t* __restrict__ table, const T* __restrict__ gate,
                                                             const T* __restrict__ up, T* __restrict__ y, GatedArgs p) {
    const uint64_t v = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (v >= p.nvec) return;
    uint32_t row, c;
    fd_divmod((uint32_t)v, p.cv, row, c);
    Vec16<T> g, u, o;
    g.u = ld_stream(reinterpret_cast<const v4u*>(gate + (uint64_t)row * p.gs) + c);
    u.u = ld_stream(reinterpret_cast<const v4u*>(up + (uint64_t)row * p.us) + c);
#pragma unroll
    for (int w = 0; w < 4; w++) g.u[w] = (uint32_t)table[g.u[w] & 0xffffu] | ((uint32_t)table[g.u[w] >> 16] << 16);
#pragma unroll
    for (int e = 0; e < 8; e++) o.e[e] = Ar<T>::mul(u.e[e], g.e[e]);
    st_stream(reinterpret_cast<v4u*>(y) + v, o.u);
}

// any size / alignment: one element per thread, computed directly
template <typename T, int OP>
__global__ void __launch_bounds__(BLOCK) gated_scalar_kernel(const T* __restrict__ gate, const T* __restrict__ up, T* __restrict__ y,
                                                             GatedArgs p) {
    const uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i >= p.nvec) return;
    uint32_t row, c;
    fd_divmod((uint32_t)i, p.cv, row, c);
    const T act = apply_unary<T, OP, true>(gate[(uint64_t)row * p.gs + c]);
    y[i] = Ar<T>::mul(up[(uint64_t)row * p.us + c], act);
}

// ------------------------------------------------------------------------------------------------ cast
template <typename S, typename D> __device__ __forceinline__ D cast_one(S v);
template <> __device__ __forceinline__ half_t cast_one<float, half_t>(float v) { return (half_t)v; }
template <> __device__ __forceinline__ float cast_one<half_t, float>(half_t v) { return (float)v; }
template <> __device__ __forceinline__ bf16_t cast_one<float, bf16_t>(float v) { return Ar<bf16_t>::conv(v); }
template <> __device__ __forceinline__ float cast_one<bf16_t, float>(bf16_t v) { return Ar<bf16_t>::widen(v); }

// Four elements per thread and access: 8 bytes on the 2-byte side, 16 bytes on the 4-byte side, so that every load
// and every store instruction of a wave covers one contiguous run (512 B / 1 KiB).  (Eight elements per thread make the
// 4-byte side two 16-byte accesses 32 bytes apart per lane: each instruction then touches half of every 32 bytes, and
// the kernel ran at 4.6 TB/s where this layout reaches 6.)
// Accesses per thread: four up to CAST_ONE_FROM elements (31 MB of traffic: 5.3 us against 6.1 us with one), one beyond
// (a wave that stores once and ends leaves HBM a more even stream than one that stores four times: 1.6 GB of traffic
// f16 -> f32 272 -> 235 us = 6.9 TB/s, f32 -> f16 262 -> 246 us).
constexpr uint64_t CAST_ONE_FROM = 1ull << 23;
template <int BYTES> struct CastVec;
template <> struct CastVec<8> { typedef v2u type; };
template <> struct CastVec<16> { typedef v4u type; };

template <typename S, typename D, int CAST_UNROLL>
__global__ void __launch_bounds__(BLOCK) cast_vec_kernel(const S* __restrict__ x, D* __restrict__ y, uint64_t numel) {
    constexpr int PER = 4;
    typedef typename CastVec<PER * sizeof(S)>::type SV;
    typedef typename CastVec<PER * sizeof(D)>::type DV;
    const uint64_t ngrp = numel / PER;
    const uint64_t base = (uint64_t)blockIdx.x * (BLOCK * CAST_UNROLL) + threadIdx.x;
    SV raw[CAST_UNROLL];
#pragma unroll
    for (int k = 0; k < CAST_UNROLL; k++) {
        const uint64_t g = base + (uint64_t)k * BLOCK;
        if (g < ngrp) raw[k] = ld_stream(reinterpret_cast<const SV*>(x) + g);
    }
#pragma unroll
    for (int k = 0; k < CAST_UNROLL; k++) {
        const uint64_t g = base + (uint64_t)k * BLOCK;
        if (g < ngrp) {
            S in[PER];
            D out[PER];
            __builtin_memcpy(in, &raw[k], sizeof(in));
#pragma unroll
            for (int e = 0; e < PER; e++) out[e] = cast_one<S, D>(in[e]);
            DV o;
            __builtin_memcpy(&o, out, sizeof(out));
            st_stream(reinterpret_cast<DV*>(y) + g, o);
        }
    }
    if (blockIdx.x == 0) {
        const uint64_t i = ngrp * PER + threadIdx.x;
        if (i < numel) y[i] = cast_one<S, D>(x[i]);
    }
}

template <typename S, typename D>
__global__ void __launch_bounds__(BLOCK) cast_scalar_kernel(const S* x, D* y, uint64_t numel) {
    const uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < numel) y[i] = cast_one<S, D>(x[i]);
}

// plain copy (same-dtype cast, f32 <-> i32/u32 reinterpretation)
__global__ void __launch_bounds__(BLOCK) copy_vec_kernel(const unsigned char* __restrict__ x, unsigned char* __restrict__ y,
                                                         uint64_t bytes) {
    const uint64_t nvec = bytes / 16;
    const v4u* xv = reinterpret_cast<const v4u*>(x);
    v4u* yv = reinterpret_cast<v4u*>(y);
    const uint64_t base = (uint64_t)blockIdx.x * (BLOCK * UNROLL) + threadIdx.x;
    v4u r[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const uint64_t i = base + (uint64_t)k * BLOCK;
        if (i < nvec) r[k] = ld_stream(xv + i);
    }
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const uint64_t i = base + (uint64_t)k * BLOCK;
        if (i < nvec) st_stream(yv + i, r[k]);
    }
    if (blockIdx.x == 0) {
        const uint64_t i = nvec * 16 + threadIdx.x;
        if (i < bytes) y[i] = x[i];
    }
}
__global__ void __launch_bounds__(BLOCK) copy_bytes_kernel(const unsigned char* x, unsigned char* y, uint64_t bytes) {
    const uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < bytes) y[i] = x[i];
}

// ------------------------------------------------------------------------------------------------ launch helpers
inline unsigned blocks_for(uint64_t items, uint64_t per_block) {
    const uint64_t b = (items + per_block - 1) / per_block;
    return (unsigned)(b ? b : 1);
}

template <typename T, int OP>
int launch_binary(rt_device* dev, const void* a, const void* b, void* y, uint64_t numel) {
    const bool vec = rt_aligned(a, 16) && rt_aligned(b, 16) && rt_aligned(y, 16);
    if (vec) {
        constexpr int VE = 16 / sizeof(T);
        hipLaunchKernelGGL((binary_vec_kernel<T, OP>), dim3(blocks_for(numel / VE, BLOCK * UNROLL)), dim3(BLOCK), 0,
                           dev->stream, (const T*)a, (const T*)b, (T*)y, numel);
    } else {
        hipLaunchKernelGGL((binary_scalar_kernel<T, OP>), dim3(blocks_for(numel, BLOCK)), dim3(BLOCK), 0, dev->stream,
                           (const T*)a, (const T*)b, (T*)y, numel);
    }
    RT_CHECK_LAUNCH("binary kernel");
    return RT_OK;
}

template <typename T>
int dispatch_binary(rt_device* dev, int op, const void* a, const void* b, void* y, uint64_t numel) {
    switch (op) {
        case RT_ADD: return launch_binary<T, RT_ADD>(dev, a, b, y, numel);
        case RT_SUB: return launch_binary<T, RT_SUB>(dev, a, b, y, numel);
        case RT_MUL: return launch_binary<T, RT_MUL>(dev, a, b, y, numel);
        default: return launch_binary<T, RT_DIV>(dev, a, b, y, numel);
    }
}

template <typename T, int OP, bool VIA32>
int launch_unary(rt_device* dev, const void* x, void* y, uint64_t numel) {
    const bool vec = rt_aligned(x, 16) && rt_aligned(y, 16);
    if (vec) {
        constexpr int VE = 16 / sizeof(T);
        hipLaunchKernelGGL((unary_vec_kernel<T, OP, VIA32>), dim3(blocks_for(numel / VE, BLOCK * UNROLL)), dim3(BLOCK), 0,
                           dev->stream, (const T*)x, (T*)y, numel);
    } else {
        hipLaunchKernelGGL((unary_scalar_kernel<T, OP, VIA32>), dim3(blocks_for(numel, BLOCK)), dim3(BLOCK), 0, dev->stream,
                           (const T*)x, (T*)y, numel);
    }
    RT_CHECK_LAUNCH("unary kernel");
    return RT_OK;
}

template <typename T, bool VIA32 = false> int dispatch_unary(rt_device* dev, int op, const void* x, void* y, uint64_t numel) {
    switch (op) {
#define RT_CASE(OPC) case OPC: return launch_unary<T, OPC, VIA32>(dev, x, y, numel);
        RT_CASE(RT_GELU) RT_CASE(RT_TANH) RT_CASE(RT_EXP) RT_CASE(RT_LOG) RT_CASE(RT_SIN) RT_CASE(RT_COS)
        RT_CASE(RT_ABS) RT_CASE(RT_SQRT) RT_CASE(RT_RELU) RT_CASE(RT_FLOOR) RT_CASE(RT_CEIL) RT_CASE(RT_NEG)
        RT_CASE(RT_SILU) RT_CASE(RT_SIGMOID)
#undef RT_CASE
        default: return rt_fail(RT_ERR_OP, "rt_unary: op %d out of range", op);
    }
}

// ops worth a table: everything with a libm call or a division in it
inline bool lut_worthwhile(int op) {
    switch (op) {
        case RT_GELU: case RT_TANH: case RT_EXP: case RT_LOG: case RT_SIN: case RT_COS: case RT_SQRT: case RT_SILU: case RT_SIGMOID:
            return true;
        default: return false;
    }
}

template <typename T, bool VIA32 = false> int build_unary_table(rt_device* dev, int ti, int op) {
    uint16_t*& slot = VIA32 ? dev->unary_lut_via32[ti][op] : dev->unary_lut[ti][op];
    if (slot) return RT_OK;
    RT_NO_CAPTURE(dev, "building a lookup table (first use of this op and type on the device)");
    uint16_t* table = nullptr;
    uint16_t* iota = nullptr;
    RT_HIP(hipMalloc((void**)&table, LUT_BYTES));
    hipError_t e = hipMalloc((void**)&iota, LUT_BYTES);
    if (e != hipSuccess) {
        (void)hipFree(table);
        return rt_fail_hip(e, "hipMalloc(lut)");
    }
    hipLaunchKernelGGL(iota16_kernel, dim3(65536 / 256), dim3(256), 0, dev->stream, iota);
    int rc = dispatch_unary<T, VIA32>(dev, op, iota, table, 65536);   // the exact kernel defines the table
    hipError_t es = hipStreamSynchronize(dev->stream);
    (void)hipFree(iota);
    if (rc != RT_OK || es != hipSuccess) {
        (void)hipFree(table);
        return rc != RT_OK ? rc : rt_fail_hip(es, "building the unary lookup table");
    }
    slot = table;
    return RT_OK;
}

template <typename T, bool VIA32 = false> int unary_via_lut(rt_device* dev, int op, const void* x, void* y, uint64_t numel) {
    const int ti = std::is_same<T, bf16_t>::value ? 1 : 0;
    int rc = build_unary_table<T, VIA32>(dev, ti, op);
    if (rc) return rc;
    if (!dev->lut_attr_set) {
        RT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(unary_lut_kernel<LUT_UNROLL, LUT_DEPTH>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)LUT_BYTES));
        dev->lut_attr_set = 1;
    }
    uint64_t blocks = (numel / 8 + LUT_TILE - 1) / LUT_TILE;
    if (blocks > (uint64_t)dev->num_cus) blocks = dev->num_cus;          // one resident block per CU (128 KiB of LDS each)
    if (blocks < 1) blocks = 1;
    const LutPace pc = lut_pace_for(dev, blocks, numel / 8 / LUT_TILE / blocks, LUT_PACE_MIN_STEPS, (double)LUT_TILE * 16 * 2);
    hipLaunchKernelGGL((unary_lut_kernel<LUT_UNROLL, LUT_DEPTH>), dim3((unsigned)blocks), dim3(LUT_BLOCK), LUT_BYTES, dev->stream,
                       (const uint16_t*)(VIA32 ? dev->unary_lut_via32[ti][op] : dev->unary_lut[ti][op]), (const uint16_t*)x,
                       (uint16_t*)y, numel, pc);
    RT_CHECK_LAUNCH("unary_lut_kernel");
    return RT_OK;
}

// Below the size where a per-block copy of the table into LDS pays (one 128 KiB load per block), the same table is read
// where it lies: the 128 KiB stay in L2 (and largely in the CUs' L1) and every element is one 2-byte load.  For the heavy
// ops this is still far cheaper than computing: gelu on [64, 10240] f16 took 11.8 us computed, of which most is the
// dependent chain of one thread's eight exact tanh evaluations.
__global__ void __launch_bounds__(BLOCK) unary_table_gather_kernel(const uint16_t* __restrict__ table, const uint16_t* x, uint16_t* y,
                                                                   uint64_t numel) {
    const uint64_t nvec = numel / 8;
    const uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < nvec) {
        const v4u in = ld_stream(reinterpret_cast<const v4u*>(x) + i);
        v4u out;
#pragma unroll
        for (int w = 0; w < 4; w++) out[w] = (uint32_t)table[in[w] & 0xffffu] | ((uint32_t)table[in[w] >> 16] << 16);
        st_stream(reinterpret_cast<v4u*>(y) + i, out);
    }
    if (blockIdx.x == 0) {
        const uint64_t j = nvec * 8 + threadIdx.x;
        if (j < numel) y[j] = table[x[j]];
    }
}

constexpr uint64_t RT_GATHER_MIN_NUMEL = 2048;

template <typename T, bool VIA32 = false> int unary_via_table_gather(rt_device* dev, int op, const void* x, void* y, uint64_t numel) {
    const int ti = std::is_same<T, bf16_t>::value ? 1 : 0;
    int rc = build_unary_table<T, VIA32>(dev, ti, op);
    if (rc) return rc;
    hipLaunchKernelGGL(unary_table_gather_kernel, dim3(blocks_for(numel / 8 ? numel / 8 : 1, BLOCK)), dim3(BLOCK), 0, dev->stream,
                       (const uint16_t*)(VIA32 ? dev->unary_lut_via32[ti][op] : dev->unary_lut[ti][op]), (const uint16_t*)x, (uint16_t*)y,
                       numel);
    RT_CHECK_LAUNCH("unary_table_gather_kernel");
    return RT_OK;
}

template <typename T>
int launch_gated(rt_device* dev, int op, const void* gate, uint64_t gs, const void* up, uint64_t us, void* y, uint64_t rows, uint32_t cols) {
    const int ti = std::is_same<T, bf16_t>::value ? 1 : 0;
    const uint64_t numel = rows * cols;
    GatedArgs p;
    p.gs = gs;
    p.us = us;
    const bool vec = cols % 8 == 0 && gs % 8 == 0 && us % 8 == 0 && rt_aligned(gate, 16) && rt_aligned(up, 16) && rt_aligned(y, 16);
    // (while a graph is being captured a table that does not exist yet cannot be built: the computing kernel below gives
    // the same bits)
    if (vec && numel >= RT_LUT_MIN_NUMEL && (!dev->capturing || dev->unary_lut_via32[ti][op])) {
        int rc = build_unary_table<T, true>(dev, ti, op);
        if (rc) return rc;
        if (!dev->gated_attr_set[ti]) {
            RT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gated_lut_kernel<T, false>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)LUT_BYTES));
            RT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gated_lut_kernel<T, true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)LUT_BYTES));
            dev->gated_attr_set[ti] = 1;
        }
        p.cv = make_fastdiv(cols / 8);
        p.nvec = numel / 8;
        uint64_t blocks = (p.nvec + LUT_BLOCK - 1) / LUT_BLOCK;
        if (blocks > (uint64_t)dev->num_cus) blocks = dev->num_cus;
        const LutPace pc = lut_pace_for(dev, blocks, p.nvec / LUT_BLOCK / blocks, GATED_PACE_MIN_STEPS, (double)LUT_BLOCK * 16 * 3);
        if (pc.pace) {
            hipLaunchKernelGGL((gated_lut_kernel<T, true>), dim3((unsigned)blocks), dim3(LUT_BLOCK), LUT_BYTES, dev->stream,
                               (const uint16_t*)dev->unary_lut_via32[ti][op], (const T*)gate, (const T*)up, (T*)y, p, pc);
        } else {
            hipLaunchKernelGGL((gated_lut_kernel<T, false>), dim3((unsigned)blocks), dim3(LUT_BLOCK), LUT_BYTES, dev->stream,
                               (const uint16_t*)dev->unary_lut_via32[ti][op], (const T*)gate, (const T*)up, (T*)y, p, pc);
        }
        RT_CHECK_LAUNCH("gated_lut_kernel");
        return RT_OK;
    }
    if (vec && numel >= RT_GATHER_MIN_NUMEL && lut_worthwhile(op) && (!dev->capturing || dev->unary_lut_via32[ti][op])) {
        int rc = build_unary_table<T, true>(dev, ti, op);
        if (rc) return rc;
        p.cv = make_fastdiv(cols / 8);
        p.nvec = numel / 8;
        hipLaunchKernelGGL((gated_gather_kernel<T>), dim3(blocks_for(p.nvec, BLOCK)), dim3(BLOCK), 0, dev->stream,
                           (const uint16_t*)dev->unary_lut_via32[ti][op], (const T*)gate, (const T*)up, (T*)y, p);
        RT_CHECK_LAUNCH("gated_gather_kernel");
        return RT_OK;
    }
    p.cv = make_fastdiv(cols);
    p.nvec = numel;
    const dim3 grid(blocks_for(numel, BLOCK)), block(BLOCK);
    switch (op) {
#define RT_CASE(OPC) case OPC: hipLaunchKernelGGL((gated_scalar_kernel<T, OPC>), grid, block, 0, dev->stream, (const T*)gate, (const T*)up, (T*)y, p); break;
        RT_CASE(RT_GELU) RT_CASE(RT_TANH) RT_CASE(RT_EXP) RT_CASE(RT_LOG) RT_CASE(RT_SIN) RT_CASE(RT_COS)
        RT_CASE(RT_ABS) RT_CASE(RT_SQRT) RT_CASE(RT_RELU) RT_CASE(RT_FLOOR) RT_CASE(RT_CEIL) RT_CASE(RT_NEG)
        RT_CASE(RT_SILU) RT_CASE(RT_SIGMOID)
#undef RT_CASE
        default: return rt_fail(RT_ERR_OP, "rt_gated_mul_via_f32: op %d out of range", op);
    }
    RT_CHECK_LAUNCH("gated_scalar_kernel");
    return RT_OK;
}

template <typename S, typename D> int launch_cast(rt_device* dev, const void* x, void* y, uint64_t numel) {
    if (rt_aligned(x, 16) && rt_aligned(y, 16)) {
        if (numel >= CAST_ONE_FROM)
            hipLaunchKernelGGL((cast_vec_kernel<S, D, 1>), dim3(blocks_for(numel / 4, BLOCK)), dim3(BLOCK), 0, dev->stream, (const S*)x,
                               (D*)y, numel);
        else
            hipLaunchKernelGGL((cast_vec_kernel<S, D, 4>), dim3(blocks_for(numel / 4, BLOCK * 4)), dim3(BLOCK), 0, dev->stream, (const S*)x,
                               (D*)y, numel);
    } else {
        hipLaunchKernelGGL((cast_scalar_kernel<S, D>), dim3(blocks_for(numel, BLOCK)), dim3(BLOCK), 0, dev->stream,
                           (const S*)x, (D*)y, numel);
    }
    RT_CHECK_LAUNCH("cast kernel");
    return RT_OK;
}

int launch_copy(rt_device* dev, const void* x, void* y, uint64_t bytes) {
    if (rt_aligned(x, 16) && rt_aligned(y, 16)) {
        hipLaunchKernelGGL(copy_vec_kernel, dim3(blocks_for(bytes / 16, BLOCK * UNROLL)), dim3(BLOCK), 0, dev->stream,
                           (const unsigned char*)x, (unsigned char*)y, bytes);
    } else {
        hipLaunchKernelGGL(copy_bytes_kernel, dim3(blocks_for(bytes, BLOCK)), dim3(BLOCK), 0, dev->stream,
                           (const unsigned char*)x, (unsigned char*)y, bytes);
    }
    RT_CHECK_LAUNCH("copy kernel");
    return RT_OK;
}

// strides (in elements) of an operand of shape s broadcast against y: 0 where the operand's extent is 1
inline void bcast_strides(const uint32_t s[4], uint32_t out[4]) {
    uint64_t st = 1;
    for (int i = 3; i >= 0; i--) {
        out[i] = (s[i] == 1) ? 0u : (uint32_t)st;
        st *= s[i];
    }
}

template <typename T, int OP>
int launch_bcast(rt_device* dev, const void* a, const uint32_t a_shape[4], const void* b, const uint32_t b_shape[4], void* y,
                 const uint32_t y_shape[4], uint64_t y_numel) {
    constexpr int VEMAX = 16 / sizeof(T);
    BcastArgs p;
    bcast_strides(a_shape, p.as);
    bcast_strides(b_shape, p.bs);
    // vector width: the last dim must split into whole vectors, every vector-loaded operand must keep 16-byte alignment
    int ve = VEMAX;
    auto operand_ok = [&](const void* ptr, const uint32_t st[4]) {
        if (st[3] == 0) return true;                               // splat: scalar loads
        if (!rt_aligned(ptr, 16)) return false;
        for (int i = 0; i < 3; i++)
            if (st[i] % VEMAX != 0) return false;
        return true;
    };
    if (y_shape[3] % VEMAX != 0 || !rt_aligned(y, 16) || !operand_ok(a, p.as) || !operand_ok(b, p.bs)) ve = 1;
    const uint64_t nvec = y_numel / ve;
    RT_REQUIRE(nvec <= 0xffffffffull - (uint64_t)BLOCK * BC_UNROLL, RT_ERR_SIZE,
               "rt_binary_bcast: %llu output vectors exceed the 32-bit index space", (unsigned long long)nvec);
    p.cv = make_fastdiv(y_shape[3] / ve);
    p.d2 = make_fastdiv(y_shape[2]);
    p.d1 = make_fastdiv(y_shape[1]);
    p.nvec = (uint32_t)nvec;
    bool a_once = true, b_once = true;                             // read exactly once (no broadcast dim): streamed past the caches
    for (int i = 0; i < 4; i++) {
        if (a_shape[i] != y_shape[i]) a_once = false;
        if (b_shape[i] != y_shape[i]) b_once = false;
    }
    // one access per thread for a full-size operand of 1 GiB or more plus a broadcast one (measured on the [1,32,4096,4096]
    // scores + [4096,4096] mask inside the benchmark step: 343-345 us against 346-351 us with two); below that, and for
    // the other operand patterns, the two are level
    if (ve == 1 && VEMAX > 1 && a_once != b_once && rt_aligned(y, 16) && rt_aligned(a_once ? a : b, 16) && y_numel <= 0xfffffff0ull) {
        // rows that are not whole vectors, one operand of y's shape: flat vectors for it and for y
        p.cv = make_fastdiv(y_shape[3]);
        const unsigned fblocks = blocks_for((y_numel + VEMAX - 1) / VEMAX, BLOCK);
        if (a_once) hipLaunchKernelGGL((binary_flat_kernel<T, OP, true>), dim3(fblocks), dim3(BLOCK), 0, dev->stream, (const T*)a, (const T*)b, (T*)y, p, y_numel);
        else hipLaunchKernelGGL((binary_flat_kernel<T, OP, false>), dim3(fblocks), dim3(BLOCK), 0, dev->stream, (const T*)a, (const T*)b, (T*)y, p, y_numel);
        RT_CHECK_LAUNCH("binary_flat_kernel");
        return RT_OK;
    }
    const int unroll = (a_once != b_once && ve == VEMAX && nvec >= BC_ONE_FROM_VECS) ? 1 : BC_UNROLL;
    const unsigned blocks = blocks_for(nvec, BLOCK * unroll);
    // one operand full-size, the other equal to y's trailing dims and repeated over the leading ones, too large for
    // the eight L2s to keep between the repeats in the plain order (RT_XCD_ORDER_MIN_BYTES) and made of whole groups of 8 slabs
    p.slabs = 0;
    p.chunk_log2 = 0;
    p.reps = make_fastdiv(1);
    if (a_once != b_once) {
        const uint32_t* rs = a_once ? b_shape : a_shape;
        int lead = 0;
        while (lead < 4 && rs[lead] == 1) lead++;
        bool prefix = lead > 0 && lead < 4;
        uint64_t reps = 1, inner = 1;
        for (int i = 0; i < 4; i++) {
            if (i < lead) reps *= y_shape[i];
            else {
                inner *= y_shape[i];
                if (rs[i] != y_shape[i]) prefix = false;
            }
        }
        const uint64_t per_block = (uint64_t)BLOCK * unroll * ve;
        if (prefix && reps > 1 && inner * sizeof(T) >= RT_XCD_ORDER_MIN_BYTES && inner % (per_block * XCDS) == 0) {
            p.reps = make_fastdiv((uint32_t)reps);
            p.slabs = (uint32_t)(inner / per_block);
            const uint32_t per_xcd = p.slabs / XCDS;
            p.chunk_log2 = per_xcd % 64 == 0 ? 6 : per_xcd % 4 == 0 ? 2 : 0;
            if (unroll == 1 && per_xcd % 128 == 0) p.chunk_log2 = 7;
        }
    }
#define RT_BCAST1(VEC, ONCE) \
    hipLaunchKernelGGL((binary_bcast_kernel<T, OP, VEC, ONCE, 1>), dim3(blocks), dim3(BLOCK), 0, dev->stream, (const T*)a, (const T*)b, (T*)y, p)
#define RT_BCAST(VEC, ONCE) \
    hipLaunchKernelGGL((binary_bcast_kernel<T, OP, VEC, ONCE>), dim3(blocks), dim3(BLOCK), 0, dev->stream, (const T*)a, (const T*)b, (T*)y, p)
    if (ve != VEMAX) RT_BCAST(1, 0);                              // scalar accesses
    else if (a_once && b_once) RT_BCAST(VEMAX, 3);
    else if (a_once && unroll == 1) RT_BCAST1(VEMAX, 1);
    else if (b_once && unroll == 1) RT_BCAST1(VEMAX, 2);
    else if (a_once) RT_BCAST(VEMAX, 1);
    else if (b_once) RT_BCAST(VEMAX, 2);
    else RT_BCAST(VEMAX, 0);
#undef RT_BCAST
    RT_CHECK_LAUNCH("binary_bcast_kernel");
    return RT_OK;
}

template <typename T>
int dispatch_bcast(rt_device* dev, int op, const void* a, const uint32_t as[4], const void* b, const uint32_t bs[4], void* y,
                   const uint32_t ys[4], uint64_t n) {
    switch (op) {
        case RT_ADD: return launch_bcast<T, RT_ADD>(dev, a, as, b, bs, y, ys, n);
        case RT_SUB: return launch_bcast<T, RT_SUB>(dev, a, as, b, bs, y, ys, n);
        case RT_MUL: return launch_bcast<T, RT_MUL>(dev, a, as, b, bs, y, ys, n);
        default: return launch_bcast<T, RT_DIV>(dev, a, as, b, bs, y, ys, n);
    }
}

}  // namespace

int rt_unary_table(rt_device* dev, int type_index, int op, const uint16_t** out) {
    int rc = type_index == 1 ? build_unary_table<bf16_t>(dev, 1, op) : build_unary_table<half_t>(dev, 0, op);
    if (rc) return rc;
    *out = dev->unary_lut[type_index == 1 ? 1 : 0][op];
    return RT_OK;
}

extern "C" {

int rt_binary(rt_device* dev, int op, int dt, const void* a, const void* b, void* y, uint64_t numel) {
    RT_REQUIRE(op >= RT_ADD && op <= RT_DIV, RT_ERR_OP, "rt_binary: op %d out of range", op);
    RT_REQUIRE(rt_is_float_dt(dt), RT_ERR_DTYPE, "rt_binary: dtype %d is not F32/F16/BF16", dt);
    RT_REQUIRE(numel <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_binary: numel %llu too large", (unsigned long long)numel);
    if (numel == 0) return dev ? RT_OK : rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(a && b && y, RT_ERR_NULL_POINTER, "rt_binary: NULL operand");
    const size_t eb = (size_t)rt_dt_bytes(dt);
    RT_REQUIRE(rt_aligned(a, eb) && rt_aligned(b, eb) && rt_aligned(y, eb), RT_ERR_ALIGN, "rt_binary: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    switch (dt) {
        case RT_F32: return dispatch_binary<float>(dev, op, a, b, y, numel);
        case RT_F16: return dispatch_binary<half_t>(dev, op, a, b, y, numel);
        default: return dispatch_binary<bf16_t>(dev, op, a, b, y, numel);
    }
}

int rt_binary_bcast(rt_device* dev, int op, int dt, const void* a, const uint32_t a_shape[4], const void* b,
                    const uint32_t b_shape[4], void* y, const uint32_t y_shape[4]) {
    RT_REQUIRE(op >= RT_ADD && op <= RT_DIV, RT_ERR_OP, "rt_binary_bcast: op %d out of range", op);
    RT_REQUIRE(rt_is_float_dt(dt), RT_ERR_DTYPE, "rt_binary_bcast: dtype %d is not F32/F16/BF16", dt);
    RT_REQUIRE(a_shape && b_shape && y_shape, RT_ERR_NULL_POINTER, "rt_binary_bcast: NULL shape");
    uint64_t n = 1;
    for (int i = 0; i < 4; i++) {
        RT_REQUIRE(a_shape[i] > 0 && b_shape[i] > 0 && y_shape[i] > 0, RT_ERR_SHAPE, "rt_binary_bcast: zero extent in dim %d", i);
        // Shape::multi_broadcast (shape.rs:118-136): each operand extent is 1 or the output extent
        RT_REQUIRE((a_shape[i] == 1 || a_shape[i] == y_shape[i]) && (b_shape[i] == 1 || b_shape[i] == y_shape[i]) &&
                       (y_shape[i] == (a_shape[i] > b_shape[i] ? a_shape[i] : b_shape[i])),
                   RT_ERR_SHAPE, "rt_binary_bcast: dim %d: %u and %u do not broadcast to %u", i, a_shape[i], b_shape[i],
                   y_shape[i]);
        n *= y_shape[i];
        RT_REQUIRE(n <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_binary_bcast: output too large");
    }
    RT_REQUIRE(a && b && y, RT_ERR_NULL_POINTER, "rt_binary_bcast: NULL operand");
    const size_t eb = (size_t)rt_dt_bytes(dt);
    RT_REQUIRE(rt_aligned(a, eb) && rt_aligned(b, eb) && rt_aligned(y, eb), RT_ERR_ALIGN,
               "rt_binary_bcast: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    bool same = true;
    for (int i = 0; i < 4; i++) same = same && a_shape[i] == y_shape[i] && b_shape[i] == y_shape[i];
    if (same) return rt_binary(dev, op, dt, a, b, y, n);
    switch (dt) {
        case RT_F32: return dispatch_bcast<float>(dev, op, a, a_shape, b, b_shape, y, y_shape, n);
        case RT_F16: return dispatch_bcast<half_t>(dev, op, a, a_shape, b, b_shape, y, y_shape, n);
        default: return dispatch_bcast<bf16_t>(dev, op, a, a_shape, b, b_shape, y, y_shape, n);
    }
}

int rt_unary(rt_device* dev, int op, int dt, const void* x, void* y, uint64_t numel) {
    RT_REQUIRE(op >= 0 && op < RT_UNARY_COUNT, RT_ERR_OP, "rt_unary: op %d out of range", op);
    RT_REQUIRE(rt_is_float_dt(dt), RT_ERR_DTYPE, "rt_unary: dtype %d is not F32/F16/BF16", dt);
    RT_REQUIRE(numel <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_unary: numel %llu too large", (unsigned long long)numel);
    if (numel == 0) return dev ? RT_OK : rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(x && y, RT_ERR_NULL_POINTER, "rt_unary: NULL operand");
    const size_t eb = (size_t)rt_dt_bytes(dt);
    RT_REQUIRE(rt_aligned(x, eb) && rt_aligned(y, eb), RT_ERR_ALIGN, "rt_unary: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    // large 16-bit tensors: table lookup (bit-identical to computing, see unary_lut_kernel); while a graph is being
    // captured only if the table exists already (building it synchronises), otherwise the computing kernel runs
    const bool have_table = dt != RT_F32 && (!dev->capturing || dev->unary_lut[dt == RT_BF16 ? 1 : 0][op]);
    const bool lut = have_table && numel >= RT_LUT_MIN_NUMEL && lut_worthwhile(op) && rt_aligned(x, 16) && rt_aligned(y, 16);
    // in between: the table read in place
    const bool gather = dt != RT_F32 && !lut && numel >= RT_GATHER_MIN_NUMEL && lut_worthwhile(op) && rt_aligned(x, 16) && rt_aligned(y, 16) &&
                        (!dev->capturing || dev->unary_lut[dt == RT_BF16 ? 1 : 0][op]);
    switch (dt) {
        case RT_F32: return dispatch_unary<float>(dev, op, x, y, numel);
        case RT_F16:
            return lut ? unary_via_lut<half_t>(dev, op, x, y, numel)
                       : gather ? unary_via_table_gather<half_t>(dev, op, x, y, numel) : dispatch_unary<half_t>(dev, op, x, y, numel);
        default:
            return lut ? unary_via_lut<bf16_t>(dev, op, x, y, numel)
                       : gather ? unary_via_table_gather<bf16_t>(dev, op, x, y, numel) : dispatch_unary<bf16_t>(dev, op, x, y, numel);
    }
}

int rt_unary_via_f32(rt_device* dev, int op, int io_dt, const void* x, void* y, uint64_t numel) {
    RT_REQUIRE(op >= 0 && op < RT_UNARY_COUNT, RT_ERR_OP, "rt_unary_via_f32: op %d out of range", op);
    RT_REQUIRE(io_dt == RT_F16 || io_dt == RT_BF16, RT_ERR_DTYPE, "rt_unary_via_f32: dtype %d is not F16/BF16", io_dt);
    RT_REQUIRE(numel <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_unary_via_f32: numel %llu too large", (unsigned long long)numel);
    if (numel == 0) return dev ? RT_OK : rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(x && y, RT_ERR_NULL_POINTER, "rt_unary_via_f32: NULL operand");
    RT_REQUIRE(rt_aligned(x, 2) && rt_aligned(y, 2), RT_ERR_ALIGN, "rt_unary_via_f32: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    const bool have_table = !dev->capturing || dev->unary_lut_via32[io_dt == RT_BF16 ? 1 : 0][op];
    const bool lut = have_table && numel >= RT_LUT_MIN_NUMEL && lut_worthwhile(op) && rt_aligned(x, 16) && rt_aligned(y, 16);
    const bool gather = !lut && have_table && numel >= RT_GATHER_MIN_NUMEL && lut_worthwhile(op) && rt_aligned(x, 16) && rt_aligned(y, 16);
    if (io_dt == RT_F16)
        return lut ? unary_via_lut<half_t, true>(dev, op, x, y, numel)
                   : gather ? unary_via_table_gather<half_t, true>(dev, op, x, y, numel) : dispatch_unary<half_t, true>(dev, op, x, y, numel);
    return lut ? unary_via_lut<bf16_t, true>(dev, op, x, y, numel)
               : gather ? unary_via_table_gather<bf16_t, true>(dev, op, x, y, numel) : dispatch_unary<bf16_t, true>(dev, op, x, y, numel);
}

int rt_gated_mul_via_f32(rt_device* dev, int op, int io_dt, const void* gate, uint64_t gate_row_stride, const void* up,
                         uint64_t up_row_stride, void* y, uint64_t rows, uint32_t cols) {
    RT_REQUIRE(op >= 0 && op < RT_UNARY_COUNT, RT_ERR_OP, "rt_gated_mul_via_f32: op %d out of range", op);
    RT_REQUIRE(io_dt == RT_F16 || io_dt == RT_BF16, RT_ERR_DTYPE, "rt_gated_mul_via_f32: dtype %d is not F16/BF16", io_dt);
    RT_REQUIRE(cols > 0 || rows == 0, RT_ERR_SHAPE, "rt_gated_mul_via_f32: cols is 0");
    RT_REQUIRE(gate_row_stride >= cols && up_row_stride >= cols, RT_ERR_SHAPE, "rt_gated_mul_via_f32: a row stride is shorter than a row");
    RT_REQUIRE(rows <= RT_MAX_NUMEL && rows * (uint64_t)cols <= 0xffffffffull && rows * gate_row_stride <= RT_MAX_NUMEL &&
                   rows * up_row_stride <= RT_MAX_NUMEL,
               RT_ERR_SIZE, "rt_gated_mul_via_f32: tensor too large");
    if (rows == 0) return dev ? RT_OK : rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(gate && up && y, RT_ERR_NULL_POINTER, "rt_gated_mul_via_f32: NULL operand");
    RT_REQUIRE(rt_aligned(gate, 2) && rt_aligned(up, 2) && rt_aligned(y, 2), RT_ERR_ALIGN, "rt_gated_mul_via_f32: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (io_dt == RT_F16) return launch_gated<half_t>(dev, op, gate, gate_row_stride, up, up_row_stride, y, rows, cols);
    return launch_gated<bf16_t>(dev, op, gate, gate_row_stride, up, up_row_stride, y, rows, cols);
}

int rt_cast(rt_device* dev, int src_dt, int dst_dt, const void* x, void* y, uint64_t numel) {
    const int sb = rt_dt_bytes(src_dt), db = rt_dt_bytes(dst_dt);
    RT_REQUIRE(sb && db, RT_ERR_DTYPE, "rt_cast: unknown dtype %d -> %d", src_dt, dst_dt);
    // the conversions cpu_cast implements (cpu/mod.rs:131-153); anything else is unimplemented!() there
    const bool numeric = (src_dt == RT_F32 && (dst_dt == RT_F16 || dst_dt == RT_BF16)) ||
                         ((src_dt == RT_F16 || src_dt == RT_BF16) && dst_dt == RT_F32);
    const bool reinterpret = (src_dt == RT_F32 && (dst_dt == RT_I32 || dst_dt == RT_U32)) ||
                             ((src_dt == RT_I32 || src_dt == RT_U32) && dst_dt == RT_F32);
    RT_REQUIRE(numeric || reinterpret || src_dt == dst_dt, RT_ERR_DTYPE, "rt_cast: %d -> %d is not a supported cast", src_dt,
               dst_dt);
    RT_REQUIRE(numel <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_cast: numel %llu too large", (unsigned long long)numel);
    if (numel == 0) return dev ? RT_OK : rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(x && y, RT_ERR_NULL_POINTER, "rt_cast: NULL operand");
    RT_REQUIRE(rt_aligned(x, (size_t)sb) && rt_aligned(y, (size_t)db), RT_ERR_ALIGN, "rt_cast: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (!numeric) return (x == y) ? RT_OK : launch_copy(dev, x, y, numel * (uint64_t)sb);
    if (src_dt == RT_F32 && dst_dt == RT_F16) return launch_cast<float, half_t>(dev, x, y, numel);
    if (src_dt == RT_F32 && dst_dt == RT_BF16) return launch_cast<float, bf16_t>(dev, x, y, numel);
    if (src_dt == RT_F16) return launch_cast<half_t, float>(dev, x, y, numel);
    return launch_cast<bf16_t, float>(dev, x, y, numel);
}

}  // extern "C"
