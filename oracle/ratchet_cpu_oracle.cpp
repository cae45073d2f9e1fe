// TEST INFRASTRUCTURE ONLY (see ratchet_cpu_oracle.h): C entry points; picks the F16C build of the kernels when the
// host CPU has the instructions, the portable build otherwise.
#include "ratchet_cpu_oracle.h"
#include <cmath>
#include <cstdint>
#include "orc_table.h"

int g_orc_f16_sum_sequential = 0;
int g_orc_reference_copies = 1;

static int g_use_hw = -1;
static const OrcTable& table() {
    if (g_use_hw < 0) g_use_hw = __builtin_cpu_supports("f16c") ? 1 : 0;
    return g_use_hw ? orc_hw::kTable : orc_soft::kTable;
}

extern "C" {
int orc_binary(int op, int dt, const void* a, const void* b, void* y, size_t n) { return table().binary(op, dt, a, b, y, n); }
int orc_unary(int op, int dt, const void* x, void* y, size_t n) { return table().unary(op, dt, x, y, n); }
int orc_cast(int s, int d, const void* x, void* y, size_t n) { return table().cast(s, d, x, y, n); }
int orc_permute(int eb, const void* x, void* y, int rank, const uint64_t* shape, const uint32_t* dims) {
    return table().permute(eb, x, y, rank, shape, dims);
}
int orc_slice(int eb, const void* x, void* y, int rank, const uint64_t* shape, const uint64_t* start, const uint64_t* stop) {
    return table().slice(eb, x, y, rank, shape, start, stop);
}
int orc_broadcast(int eb, const void* x, void* y, int sr, const uint64_t* ss, int dr, const uint64_t* ds, int np) {
    return table().broadcast(eb, x, y, sr, ss, dr, ds, np);
}
int orc_concat(int eb, int n, const void* const* xs, int rank, const uint64_t* shapes, int dim, void* y) {
    return table().concat(eb, n, xs, rank, shapes, dim, y);
}
int orc_cache(int eb, void* cache, int rank, const uint64_t* cs, const void* source, const uint64_t* ss, int dim, uint64_t offset,
              void* dst) {
    return table().cache(eb, cache, rank, cs, source, ss, dim, offset, dst);
}
int orc_rope(int dt, const void* x, void* y, const uint64_t* shape, uint64_t dim, float base, uint64_t offset) {
    return table().rope(dt, x, y, shape, dim, base, offset);
}
int orc_index_select(int eb, const void* src, int rank, const uint64_t* ss, const int32_t* indices, uint64_t n, int dim, void* dst) {
    return table().index_select(eb, src, rank, ss, indices, n, dim, dst);
}
int orc_index_write(int eb, void* dst, int rank, const uint64_t* ds, const void* src, uint64_t n, const uint64_t* write_start) {
    return table().index_write(eb, dst, rank, ds, src, n, write_start);
}
int orc_softmax(int dt, const void* x, void* y, size_t rows, size_t cols) { return table().softmax(dt, x, y, rows, cols); }
int orc_layer_norm(int dt, const void* x, const void* s, const void* b, void* y, size_t rows, size_t cols, float eps,
                   size_t shape0) {
    return table().layer_norm(dt, x, s, b, y, rows, cols, eps, shape0);
}
int orc_rms_norm(int dt, const void* x, const void* s, void* y, size_t rows, size_t cols, float eps, size_t shape0) {
    return table().rms_norm(dt, x, s, y, rows, cols, eps, shape0);
}
int orc_group_norm(int dt, const void* x, const void* s, const void* b, void* y, size_t B, size_t C, size_t L, size_t G,
                   float eps) {
    return table().group_norm(dt, x, s, b, y, B, C, L, G, eps);
}
// ---- Q8_0 (quant.rs:19-49, 101-130).  f16 arithmetic = widen, operate in f32, round to nearest even (crate `half`).
static inline float q8_round_to(int fp_dt, float v) { return fp_dt == 1 ? table().f16_to_f32(table().f32_to_f16(v)) : v; }
// Rust's `as i32` on a float: truncation toward zero, saturating, NaN -> 0
static inline int32_t q8_as_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}
int orc_q8_0_quantize(int fp_dt, const void* x_in, uint64_t numel, uint32_t* words, void* scales) {
    if ((fp_dt != 0 && fp_dt != 1) || numel % 32 != 0) return 1;
    const float* xf = static_cast<const float*>(x_in);
    const uint16_t* xh = static_cast<const uint16_t*>(x_in);
    auto at = [&](uint64_t i) -> float { return fp_dt == 1 ? table().f16_to_f32(xh[i]) : xf[i]; };
    float d = 0.0f;
    for (uint64_t i = 0; i < numel; i += 4) {
        if (i % 32 == 0) {
            float m = 0.0f;                                                    // fold(0, |acc, x| acc.max(x.abs()))
            for (uint64_t k = i; k < i + 32; k++) {
                const float a = std::fabs(at(k));
                if (a == a && a > m) m = a;                                    // Float::max ignores a NaN operand
            }
            d = q8_round_to(fp_dt, m / 127.0f);
            if (fp_dt == 1) static_cast<uint16_t*>(scales)[i / 32] = table().f32_to_f16(d);
            else static_cast<float*>(scales)[i / 32] = d;
        }
        int32_t packed = 0;
        for (int j = 0; j < 4; j++) {
            const float q = q8_round_to(fp_dt, at(i + j) / d);                 // (matrix[i + j] / d)
            packed |= (q8_as_i32(std::round(q)) & 0xFF) << (j * 8);            // .round().as_() & MASK, << j * LSHIFT
        }
        words[i / 4] = (uint32_t)packed;
    }
    return 0;
}
int orc_q8_0_dequantize(int fp_dt, const uint32_t* words, const void* scales, uint64_t numel, void* y) {
    if ((fp_dt != 0 && fp_dt != 1) || numel % 32 != 0) return 1;
    for (uint64_t i = 0; i < numel; i += 4) {
        const float absmax = fp_dt == 1 ? table().f16_to_f32(static_cast<const uint16_t*>(scales)[i / 32]) : static_cast<const float*>(scales)[i / 32];
        const int32_t packed = (int32_t)words[i / 4];
        for (int j = 0; j < 4; j++) {
            // FP::from_i32((packed << (LSHIFT * (PACK_SIZE - j - 1))) >> RSHIFT) * absmax: the arithmetic shift sign-extends byte j
            const int32_t q = (int32_t)((uint32_t)packed << (8 * (3 - j))) >> 24;
            const float v = q8_round_to(fp_dt, (float)q * absmax);
            if (fp_dt == 1) static_cast<uint16_t*>(y)[i + j] = table().f32_to_f16(v);
            else static_cast<float*>(y)[i + j] = v;
        }
    }
    return 0;
}
void orc_set_reference_copies(int on) { g_orc_reference_copies = on ? 1 : 0; }
void orc_set_f16_sum_mode(int seq) { g_orc_f16_sum_sequential = seq ? 1 : 0; }
void orc_set_hw_f16(int on) { g_use_hw = (on && __builtin_cpu_supports("f16c")) ? 1 : 0; }
int orc_has_hw_f16(void) { return __builtin_cpu_supports("f16c") ? 1 : 0; }
uint16_t orc_f32_to_f16(float f) { return table().f32_to_f16(f); }
float orc_f16_to_f32(uint16_t h) { return table().f16_to_f32(h); }
uint16_t orc_f32_to_bf16(float f) { return table().f32_to_bf16(f); }
float orc_bf16_to_f32(uint16_t h) { return table().bf16_to_f32(h); }
size_t orc_count_not_close(int dt, const void* a, const void* b, size_t n, double atol, double rtol, double* mx) {
    return table().count_not_close(dt, a, b, n, atol, rtol, mx);
}
}
