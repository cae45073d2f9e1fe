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
