// RoPE (rotary position embedding) on [B, H, S, D].
//
// Arithmetic contract = crates/ratchet-core/src/cpu/rope.rs:23-143 (f32; the reference's CPU path implements nothing else):
//     inv_freq[i] = exp((-(i as f32) * ln(base)) / half)             half = dim / 2
//     theta[p, i] = ((offset + p) as f32) * inv_freq[i]
//     y[.., p, i]        = x1 * cos(theta) - x2 * sin(theta)          x1 = x[.., p, i], x2 = x[.., p, half + i]
//     y[.., p, half + i] = x1 * sin(theta) + x2 * cos(theta)          (products rounded separately, no fused multiply-add)
//     y[.., p, j]        = x[.., p, j]  for j >= dim
// ln(base) is taken on the host with the C library's logf, which is what the reference's f32::ln resolves to; exp is the
// bit-exact restatement in rt_math.h; sin / cos are evaluated in double and rounded once.  16-bit tensors are widened,
// rotated in f32 and rounded once: what the models' x.full().rope(..).cast(dt) sequence produces
// (ratchet-models/src/phi3/attn.rs:118-133).
//
// theta depends on (p, i) only, so one thread owns a (p, i) pair, computes sin / cos once and walks the batch * heads
// rows that share it; blockIdx.y splits those rows when S * half alone would not fill the chip (decode steps).
#include <math.h>

#include "rt_arith.h"
#include "rt_internal.h"

namespace {

constexpr int BLOCK = 256;

struct RopeArgs {
    FastDiv per_row;         // work items per position: half rotated pairs + (D - dim) pass-through columns
    uint32_t S, D, half, dim, offset;
    uint32_t nbh, bh_chunk;  // batch * heads, rows of them per blockIdx.y
    uint32_t n_items;        // S * per_row
    float ln_base;
};

template <typename T>
__global__ void __launch_bounds__(BLOCK) rope_kernel(const T* x, T* y, RopeArgs a) {
    const uint32_t item = blockIdx.x * BLOCK + threadIdx.x;
    if (item >= a.n_items) return;
    uint32_t p, j;
    fd_divmod(item, a.per_row, p, j);
    const uint32_t bh0 = blockIdx.y * a.bh_chunk;
    const uint32_t bh1 = (bh0 + a.bh_chunk < a.nbh) ? bh0 + a.bh_chunk : a.nbh;
    if (j < a.half) {
        const float neg_i = -(float)j;
        const float inv = rt_expf(neg_i * a.ln_base / (float)a.half);
        const float theta = (float)(a.offset + p) * inv;
        const float sn = rt_sinf(theta), cs = rt_cosf(theta);
        for (uint32_t bh = bh0; bh < bh1; bh++) {
            const uint64_t base = ((uint64_t)bh * a.S + p) * a.D;
            const float x1 = Ar<T>::widen(x[base + j]), x2 = Ar<T>::widen(x[base + a.half + j]);
            const float r1 = x1 * cs - x2 * sn;
            const float r2 = x1 * sn + x2 * cs;
            y[base + j] = Ar<T>::conv(r1);
            y[base + a.half + j] = Ar<T>::conv(r2);
        }
    } else if (x != y) {
        const uint32_t col = a.dim + (j - a.half);
        for (uint32_t bh = bh0; bh < bh1; bh++) {
            const uint64_t at = ((uint64_t)bh * a.S + p) * a.D + col;
            y[at] = x[at];
        }
    }
}

// The same work in 16-byte vectors, for head layouts whose rotated half, rotated width and head dim are whole aligned
// vectors (every model: 32/80, 96/96, 128/128 columns).  A rotary block owns BLOCK / VE items, an item being (position,
// vector of VE frequencies): first every thread computes one (position, frequency) sin / cos pair into LDS (the double
// precision sin and cos are the long pole: one pair per thread, not VE), then thread (item, sub) rotates the item's two
// vectors in rows sub, sub + VE, ... of the block's share of batch * heads.  Blocks past the rotary ones copy the
// pass-through vectors the same way.
struct RopeVecArgs {
    FastDiv hv_div, pv_div;  // rotated vectors per half row; pass-through vectors per row
    uint32_t S, half, offset;
    uint32_t hv, pv, row_v;  // vectors: per half, pass-through, per row
    uint32_t nbh, bh_chunk;
    uint32_t rot_items, pass_items, rot_blocks;
    float ln_base;
};

template <typename T>
__global__ void __launch_bounds__(BLOCK) rope_vec_kernel(const T* x, T* y, RopeVecArgs a) {
    constexpr int VE = 16 / sizeof(T), ITEMS = BLOCK / VE;
    __shared__ float s_sn[BLOCK], s_cs[BLOCK];
    const uint32_t bh0 = blockIdx.y * a.bh_chunk;
    const uint32_t bh1 = (bh0 + a.bh_chunk < a.nbh) ? bh0 + a.bh_chunk : a.nbh;
    const v4u* xv = reinterpret_cast<const v4u*>(x);
    v4u* yv = reinterpret_cast<v4u*>(y);
    const uint32_t it = threadIdx.x % ITEMS, sub = threadIdx.x / ITEMS;
    const uint64_t row_stride = (uint64_t)a.S * a.row_v;
    if (blockIdx.x < a.rot_blocks) {
        {
            const uint32_t item = blockIdx.x * ITEMS + threadIdx.x / VE, e = threadIdx.x % VE;
            if (item < a.rot_items) {
                uint32_t p, slot;
                fd_divmod(item, a.hv_div, p, slot);
                const float neg_i = -(float)(slot * VE + e);
                const float inv = rt_expf(neg_i * a.ln_base / (float)a.half);
                const float theta = (float)(a.offset + p) * inv;
                s_sn[threadIdx.x] = rt_sinf(theta);
                s_cs[threadIdx.x] = rt_cosf(theta);
            }
        }
        __syncthreads();
        const uint32_t item = blockIdx.x * ITEMS + it;
        if (item >= a.rot_items) return;
        uint32_t p, slot;
        fd_divmod(item, a.hv_div, p, slot);
        float sn[VE], cs[VE];
#pragma unroll
        for (int e = 0; e < VE; e++) {
            sn[e] = s_sn[it * VE + e];
            cs[e] = s_cs[it * VE + e];
        }
        auto rotate = [&](Vec16<T>& lo, Vec16<T>& hi) {
#pragma unroll
            for (int e = 0; e < VE; e++) {
                const float x1 = Ar<T>::widen(lo.e[e]), x2 = Ar<T>::widen(hi.e[e]);
                const float r1 = x1 * cs[e] - x2 * sn[e];
                const float r2 = x1 * sn[e] + x2 * cs[e];
                lo.e[e] = Ar<T>::conv(r1);
                hi.e[e] = Ar<T>::conv(r2);
            }
        };
        const uint64_t at_p = (uint64_t)p * a.row_v + slot;
        for (uint32_t bh = bh0 + sub; bh < bh1; bh += 2 * VE) {     // two rows per trip, all four loads before the first store
            const uint64_t at0 = (uint64_t)bh * row_stride + at_p;
            const bool two = bh + VE < bh1;
            const uint64_t at1 = two ? at0 + (uint64_t)VE * row_stride : at0;
            Vec16<T> lo0, hi0, lo1, hi1;
            lo0.u = ld_stream(xv + at0);
            hi0.u = ld_stream(xv + at0 + a.hv);
            lo1.u = ld_stream(xv + at1);
            hi1.u = ld_stream(xv + at1 + a.hv);
            rotate(lo0, hi0);
            st_stream(yv + at0, lo0.u);
            st_stream(yv + at0 + a.hv, hi0.u);
            if (two) {
                rotate(lo1, hi1);
                st_stream(yv + at1, lo1.u);
                st_stream(yv + at1 + a.hv, hi1.u);
            }
        }
    } else {
        const uint32_t item = (blockIdx.x - a.rot_blocks) * ITEMS + it;
        if (item >= a.pass_items) return;
        uint32_t p, slot;
        fd_divmod(item, a.pv_div, p, slot);
        const uint64_t at_p = (uint64_t)p * a.row_v + 2 * a.hv + slot;
        for (uint32_t bh = bh0 + sub; bh < bh1; bh += 2 * VE) {
            const uint64_t at0 = (uint64_t)bh * row_stride + at_p;
            const bool two = bh + VE < bh1;
            const uint64_t at1 = two ? at0 + (uint64_t)VE * row_stride : at0;
            const v4u v0 = ld_stream(xv + at0), v1 = ld_stream(xv + at1);
            st_stream(yv + at0, v0);
            if (two) st_stream(yv + at1, v1);
        }
    }
}

// The vector kernel with every global access in whole contiguous runs.  A block owns PB consecutive positions and, in each
// (batch, head) row of its share, the one run of nv = PB * D / VE vectors they occupy: thread (row of the trip, vector of
// the run) loads its vector, the vectors of the rotated upper half pass through LDS to the thread that holds their
// partner, which rotates both, and every thread stores the vector it loaded to where it came from in y.  PB is small
// enough for one sin / cos pair per thread (PB * half <= 256).  rope_vec_kernel, whose waves take one vector slot of many
// positions, touches 32 to 96 bytes of every line per instruction, and fetches a line again when the next instruction
// comes for the rest of it (FETCH_SIZE 2.0 x the tensor on [4,32,2048,80] f16, rotary width 32).
constexpr int RS_U = 4;      // rows of the trip a thread holds
constexpr int RS_INV = 64;
struct RopeStageArgs {
    FastDiv rowv_div;        // vectors per position
    uint32_t S, half, offset, hv, row_v, active_v, PB, nv, rpt;   // active_v: vectors per position that move (all, or 2 * hv in place)
    uint32_t nbh, bh_chunk;
    float ln_base;
    float inv[RS_INV];       // inv_freq[i] for half <= RS_INV, from the host's expf (the value rt_expf returns)
};

template <typename T>
__global__ void __launch_bounds__(BLOCK) rope_stage_kernel(const T* x, T* y, RopeStageArgs a) {
    constexpr int VE = 16 / sizeof(T);
    __shared__ v4u stage[RS_U][BLOCK];
    __shared__ float s_sn[BLOCK], s_cs[BLOCK];
    const uint32_t p0 = blockIdx.x * a.PB;
    const uint32_t npos = (a.S - p0 < a.PB) ? a.S - p0 : a.PB;
    for (uint32_t idx = threadIdx.x; idx < npos * a.half; idx += BLOCK) {      // one per thread (PB * half <= 256)
        const uint32_t pl = idx / a.half, i = idx - pl * a.half;
        const float neg_i = -(float)i;
        const float inv = a.half <= (uint32_t)RS_INV ? a.inv[i] : rt_expf(neg_i * a.ln_base / (float)a.half);
        const float theta = (float)(a.offset + p0 + pl) * inv;
        s_sn[idx] = rt_sinf(theta);
        s_cs[idx] = rt_cosf(theta);
    }
    __syncthreads();
    const uint32_t jr = threadIdx.x / a.nv, w = threadIdx.x - jr * a.nv;      // row of the trip, vector of the run
    uint32_t pl, slot;
    fd_divmod(w, a.rowv_div, pl, slot);
    const bool mine = jr < a.rpt && pl < npos && slot < a.active_v;
    const bool rot = mine && slot < a.hv, upper = mine && slot >= a.hv && slot < 2 * a.hv;
    float sn[VE], cs[VE];
#pragma unroll
    for (int e = 0; e < VE; e++) {
        sn[e] = rot ? s_sn[pl * a.half + slot * VE + e] : 0.0f;
        cs[e] = rot ? s_cs[pl * a.half + slot * VE + e] : 0.0f;
    }
    const uint32_t bh0 = blockIdx.y * a.bh_chunk;
    const uint32_t bh1 = (bh0 + a.bh_chunk < a.nbh) ? bh0 + a.bh_chunk : a.nbh;
    const v4u* xv = reinterpret_cast<const v4u*>(x);
    v4u* yv = reinterpret_cast<v4u*>(y);
    const uint64_t row_stride = (uint64_t)a.S * a.row_v;
    // a thread without a vector of its own loads the block's first one instead (the loads below carry no condition, so the
    // four of a trip are in flight together and stay in registers) and stores nothing
    const uint64_t at_w = (uint64_t)p0 * a.row_v + (mine ? w : 0);
    for (uint32_t b = bh0; b < bh1; b += RS_U * a.rpt) {
        v4u r[RS_U];
#pragma unroll
        for (int u = 0; u < RS_U; u++) {
            const uint32_t bh = b + u * a.rpt + (mine ? jr : 0);
            r[u] = xv[(uint64_t)(bh < bh1 ? bh : bh1 - 1) * row_stride + at_w];     // cached loads: neighbouring runs share their edge lines
        }
        if (upper) {
#pragma unroll
            for (int u = 0; u < RS_U; u++) stage[u][threadIdx.x] = r[u];
        }
        __syncthreads();
        if (rot) {
#pragma unroll
            for (int u = 0; u < RS_U; u++) {
                Vec16<T> lo, hi;
                lo.u = r[u];
                hi.u = stage[u][threadIdx.x + a.hv];
#pragma unroll
                for (int e = 0; e < VE; e++) {
                    const float x1 = Ar<T>::widen(lo.e[e]), x2 = Ar<T>::widen(hi.e[e]);
                    const float r1 = x1 * cs[e] - x2 * sn[e];
                    const float r2 = x1 * sn[e] + x2 * cs[e];
                    lo.e[e] = Ar<T>::conv(r1);
                    hi.e[e] = Ar<T>::conv(r2);
                }
                r[u] = lo.u;
                stage[u][threadIdx.x + a.hv] = hi.u;
            }
        }
        __syncthreads();
        if (upper) {
#pragma unroll
            for (int u = 0; u < RS_U; u++) r[u] = stage[u][threadIdx.x];
        }
        if (mine) {
#pragma unroll
            for (int u = 0; u < RS_U; u++) {
                const uint32_t bh = b + u * a.rpt + jr;
                if (bh < bh1) st_stream(yv + (uint64_t)bh * row_stride + at_w, r[u]);
            }
        }
        // (the next trip writes stage[.][own index] only after this thread has read it, and reads a partner's entry only
        // behind the next barrier)
    }
}

template <typename T> int launch_rope_stage(rt_device* dev, const void* x, void* y, const uint32_t shape[4], uint32_t dim, uint32_t offset, float ln_base) {
    constexpr uint32_t VE = 16 / sizeof(T);
    RopeStageArgs a;
    a.S = shape[2];
    a.half = dim / 2;
    a.offset = offset;
    a.hv = a.half / VE;
    a.row_v = shape[3] / VE;
    a.active_v = (x == y) ? 2 * a.hv : a.row_v;              // in place: the pass-through columns stay where they are
    a.rowv_div = make_fastdiv(a.row_v);
    a.nbh = shape[0] * shape[1];
    a.ln_base = ln_base;
    for (uint32_t i = 0; i < (uint32_t)RS_INV; i++) a.inv[i] = i < a.half ? expf(-(float)i * ln_base / (float)a.half) : 0.0f;
    // positions per block: at most one sin / cos pair per thread (two cost the small tensors more than longer runs gain:
    // [1,32,2048,80] f16 6.9 -> 8.3 us); runs of whole 128-byte lines first (neighbouring blocks then share no line), then the
    // run that (times the rows of a trip) fills the block best
    uint32_t pb_max = BLOCK / a.half;
    if (pb_max > BLOCK / a.row_v) pb_max = BLOCK / a.row_v;
    if (pb_max > a.S) pb_max = a.S;
    if (pb_max < 1) pb_max = 1;
    uint32_t best = 1, best_score = 0;
    for (uint32_t pb = 1; pb <= pb_max; pb++) {
        const uint32_t nv = pb * a.row_v, fill = (BLOCK / nv) * nv;
        const uint32_t score = ((nv * 16) % 128 == 0 ? 1024 : 0) + fill;
        if (score >= best_score) {
            best_score = score;
            best = pb;
        }
    }
    a.PB = best;
    a.nv = a.PB * a.row_v;
    a.rpt = BLOCK / a.nv;
    const uint64_t blocks_x = ((uint64_t)a.S + a.PB - 1) / a.PB;
    RT_REQUIRE(blocks_x <= 0x7fffffffull, RT_ERR_SIZE, "rt_rope: seq_len too large");
    // batch * heads is split over blockIdx.y until about four blocks per CU exist, but not below one trip per block
    uint64_t chunks = ((uint64_t)dev->num_cus * 4 + blocks_x - 1) / blocks_x;
    const uint64_t per_trip = (uint64_t)RS_U * a.rpt;
    const uint64_t max_chunks = (a.nbh + per_trip - 1) / per_trip;
    if (chunks > max_chunks) chunks = max_chunks;
    if (chunks > 65535) chunks = 65535;
    if (chunks < 1) chunks = 1;
    a.bh_chunk = (uint32_t)((a.nbh + chunks - 1) / chunks);
    chunks = (a.nbh + a.bh_chunk - 1) / a.bh_chunk;
    hipLaunchKernelGGL((rope_stage_kernel<T>), dim3((unsigned)blocks_x, (unsigned)chunks), dim3(BLOCK), 0, dev->stream, (const T*)x, (T*)y, a);
    RT_CHECK_LAUNCH("rope_stage_kernel");
    return RT_OK;
}

template <typename T> int launch_rope_vec(rt_device* dev, const void* x, void* y, const uint32_t shape[4], uint32_t dim, uint32_t offset, float ln_base) {
    constexpr uint32_t VE = 16 / sizeof(T), ITEMS = BLOCK / VE;
    RopeVecArgs a;
    a.S = shape[2];
    a.half = dim / 2;
    a.offset = offset;
    a.hv = a.half / VE;
    a.pv = (shape[3] - dim) / VE;
    a.row_v = shape[3] / VE;
    a.nbh = shape[0] * shape[1];
    a.ln_base = ln_base;
    a.hv_div = make_fastdiv(a.hv);
    a.pv_div = make_fastdiv(a.pv ? a.pv : 1);
    const uint64_t rot_items = (uint64_t)a.S * a.hv, pass_items = (x == y) ? 0 : (uint64_t)a.S * a.pv;   // in place: nothing to copy
    RT_REQUIRE(rot_items + pass_items <= 0x7fffffffull, RT_ERR_SIZE, "rt_rope: seq_len * head_dim too large");
    a.rot_items = (uint32_t)rot_items;
    a.pass_items = (uint32_t)pass_items;
    a.rot_blocks = (uint32_t)((rot_items + ITEMS - 1) / ITEMS);
    const uint64_t blocks_x = a.rot_blocks + (pass_items + ITEMS - 1) / ITEMS;
    // batch * heads is split over blockIdx.y until about four blocks per CU exist, but not below one row per sub-thread
    uint64_t chunks = ((uint64_t)dev->num_cus * 4 + blocks_x - 1) / blocks_x;
    const uint64_t max_chunks = (a.nbh + VE - 1) / VE;
    if (chunks > max_chunks) chunks = max_chunks;
    if (chunks > 65535) chunks = 65535;
    if (chunks < 1) chunks = 1;
    a.bh_chunk = (uint32_t)((a.nbh + chunks - 1) / chunks);
    chunks = (a.nbh + a.bh_chunk - 1) / a.bh_chunk;
    hipLaunchKernelGGL((rope_vec_kernel<T>), dim3((unsigned)blocks_x, (unsigned)chunks), dim3(BLOCK), 0, dev->stream, (const T*)x, (T*)y, a);
    RT_CHECK_LAUNCH("rope_vec_kernel");
    return RT_OK;
}

template <typename T> int launch_rope(rt_device* dev, const void* x, void* y, const RopeArgs& a, unsigned chunks) {
    const dim3 grid((a.n_items + BLOCK - 1) / BLOCK, chunks);
    hipLaunchKernelGGL((rope_kernel<T>), grid, dim3(BLOCK), 0, dev->stream, (const T*)x, (T*)y, a);
    RT_CHECK_LAUNCH("rope_kernel");
    return RT_OK;
}

}  // namespace

extern "C" int rt_rope(rt_device* dev, int dt, const void* x, void* y, const uint32_t shape[4], uint32_t dim, float base, uint32_t offset) {
    RT_REQUIRE(rt_is_float_dt(dt), RT_ERR_DTYPE, "rt_rope: dtype %d is not F32/F16/BF16", dt);       // RoPE::check_dtypes
    RT_REQUIRE(shape, RT_ERR_NULL_POINTER, "rt_rope: NULL shape");
    uint64_t n = 1;
    for (int i = 0; i < 4; i++) {
        RT_REQUIRE(shape[i] > 0, RT_ERR_SHAPE, "rt_rope: zero extent in dim %d", i);
        n *= shape[i];
    }
    // RoPE::check_shapes (ops/rope.rs:52-58): shape[3] >= dim, dim % 8 == 0
    RT_REQUIRE(dim > 0 && dim % 8 == 0 && dim <= shape[3], RT_ERR_SHAPE, "rt_rope: dim %u must be a positive multiple of 8 and <= %u", dim,
               shape[3]);
    RT_REQUIRE(base > 0.0f && base == base && base < __builtin_huge_valf(), RT_ERR_ARG, "rt_rope: base must be positive and finite");
    RT_REQUIRE(n <= RT_MAX_NUMEL && (uint64_t)shape[0] * shape[1] <= 0xffffffffull, RT_ERR_SIZE, "rt_rope: tensor too large");
    RT_REQUIRE((uint64_t)offset + shape[2] <= 0xffffffffull, RT_ERR_SIZE, "rt_rope: offset + seq_len overflows");
    RT_REQUIRE(x && y, RT_ERR_NULL_POINTER, "rt_rope: NULL operand");
    const size_t eb = (size_t)rt_dt_bytes(dt);
    RT_REQUIRE(rt_aligned(x, eb) && rt_aligned(y, eb), RT_ERR_ALIGN, "rt_rope: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    RopeArgs a;
    a.S = shape[2];
    a.D = shape[3];
    a.dim = dim;
    a.half = dim / 2;
    a.offset = offset;
    a.nbh = shape[0] * shape[1];
    const uint32_t ve = 16u / (uint32_t)eb;
    if ((dim / 2) % ve == 0 && shape[3] % ve == 0 && rt_aligned(x, 16) && rt_aligned(y, 16)) {
        // rows that are not whole 256-byte units (head dims 64 to 96 in 16 bits, 80 in f32): the kernel whose accesses are
        // whole contiguous runs ([4,32,2048,80] f16, rotary width 32: 42.6 -> 22.1 us, [1,32,2048,80] 10.5 -> 7.0 us,
        // [4,32,4096,96] f16 61.4 -> 40.0 us, [4,32,4096,64] f16 30.1 -> 26.2 us; on rows of 256 and 512 bytes the slot
        // kernel's pieces are whole lines already and it is 2-8 % faster: [4,32,4096,128] f16 47.5 against 48.5 us)
        if (dim / 2 <= (uint32_t)BLOCK && shape[3] / ve <= (uint32_t)BLOCK && ((uint64_t)shape[3] * eb) % 256 != 0) {
            switch (dt) {
                case RT_F32: return launch_rope_stage<float>(dev, x, y, shape, dim, offset, logf(base));
                case RT_F16: return launch_rope_stage<half_t>(dev, x, y, shape, dim, offset, logf(base));
                default: return launch_rope_stage<bf16_t>(dev, x, y, shape, dim, offset, logf(base));
            }
        }
        switch (dt) {
            case RT_F32: return launch_rope_vec<float>(dev, x, y, shape, dim, offset, logf(base));
            case RT_F16: return launch_rope_vec<half_t>(dev, x, y, shape, dim, offset, logf(base));
            default: return launch_rope_vec<bf16_t>(dev, x, y, shape, dim, offset, logf(base));
        }
    }
    const uint32_t per_row = a.half + (a.D - dim);
    a.per_row = make_fastdiv(per_row);
    const uint64_t items = (uint64_t)a.S * per_row;
    RT_REQUIRE(items <= 0x7fffffffull, RT_ERR_SIZE, "rt_rope: seq_len * head_dim too large");
    a.n_items = (uint32_t)items;
    a.ln_base = logf(base);
    // at least ~64K threads in flight when the tensor has that much work
    uint64_t chunks = (65536 + items - 1) / items;
    if (chunks > a.nbh) chunks = a.nbh;
    if (chunks < 1) chunks = 1;
    a.bh_chunk = (uint32_t)((a.nbh + chunks - 1) / chunks);
    chunks = (a.nbh + a.bh_chunk - 1) / a.bh_chunk;
    switch (dt) {
        case RT_F32: return launch_rope<float>(dev, x, y, a, (unsigned)chunks);
        case RT_F16: return launch_rope<half_t>(dev, x, y, a, (unsigned)chunks);
        default: return launch_rope<bf16_t>(dev, x, y, a, (unsigned)chunks);
    }
}
