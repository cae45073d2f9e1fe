// Host check of the kernels' libm-level routines: ratchet_amd/csrc/rt_libm.h compiled as plain C++ (the very text the
// kernels compile for the GPU) against this machine's C library, which is what the reference's f32::tanh / f32::exp / f32::ln / f32::sin / f32::cos
// resolve to (crates/ratchet-core/src/cpu/unary.rs:46-65, cpu/softmax.rs:30).  Bit equality is required (any NaN equals
// any NaN).  Inputs: every `stride`-th float bit pattern over the whole 2^32 range (stride 1 = exhaustive), every value
// that a 16-bit input can widen to, and the breakpoints of the algorithms.  Build: g++ -O2 -ffp-contract=off.
// Usage: device_math_check [stride]   -> prints "tanhf <n> expm1f <n> expf <n> logf <n> sinf <n> cosf <n> f2bf <n> checked <m>", exit code 0 iff all n are 0.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#define RT_FN static inline
#define RT_TABLE static const
#include "rt_libm.h"

static inline bool same(float a, float b) { return f2u(a) == f2u(b) || (a != a && b != b); }

// round to nearest even, NaN quieted with the payload's top bits kept: half::bf16::from_f32
static inline uint16_t bf16_reference(float f) {
    const uint32_t x = f2u(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
    const uint32_t lower = x & 0xffffu, keep = x >> 16;
    if (lower > 0x8000u || (lower == 0x8000u && (keep & 1u))) return (uint16_t)(keep + 1);
    return (uint16_t)keep;
}

struct Counts {
    unsigned long long tanh_bad = 0, expm1_bad = 0, exp_bad = 0, log_bad = 0, sin_bad = 0, cos_bad = 0, bf_bad = 0, checked = 0;
    void one(uint32_t bits) {
        const float x = u2f(bits);
        if (!same(rt_tanhf(x), tanhf(x))) tanh_bad++;
        if (!same(rt_expm1f(x), expm1f(x))) expm1_bad++;
        if (!same(rt_expf(x), expf(x))) exp_bad++;
        if (!same(rt_logf(x), logf(x))) log_bad++;
        if (!same(rt_sinf(x), sinf(x))) sin_bad++;
        if (!same(rt_cosf(x), cosf(x))) cos_bad++;
        if (f2bf(x) != bf16_reference(x)) bf_bad++;
        checked++;
    }
};

int main(int argc, char** argv) {
    const unsigned long long stride = argc > 1 ? strtoull(argv[1], nullptr, 10) : 1021;
    Counts c;
    for (unsigned long long u = 0; u < (1ull << 32); u += stride) c.one((uint32_t)u);
    // everything an f16 or bf16 input widens to
    for (uint32_t h = 0; h < 65536; h++) {
        c.one(h << 16);                                                          // bf16
        const uint32_t sign = (h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u;
        uint32_t bits;
        if (e == 31) bits = sign | 0x7f800000u | (m << 13);
        else if (e) bits = sign | ((e + 112u) << 23) | (m << 13);
        else if (m) { float f = (float)m * 5.9604644775390625e-08f; bits = f2u(f) | sign; }
        else bits = sign;
        c.one(bits);                                                             // f16
    }
    // breakpoints of the algorithms, with their neighbours
    const uint32_t marks[] = {0x00000000u, 0x24000000u, 0x33000000u, 0x3eb17218u, 0x3f800000u, 0x3F851592u, 0x4195b844u, 0x41b00000u,
                              0x42b00000u, 0x42b17218u, 0x42cff1b5u, 0x7f800000u, 0x7fc00000u, 0x00800000u, 0x007fffffu, 0x3f000000u};
    for (uint32_t mk : marks)
        for (int d = -64; d <= 64; d++) {
            c.one(mk + (uint32_t)d);
            c.one((mk + (uint32_t)d) ^ 0x80000000u);
        }
    printf("tanhf %llu expm1f %llu expf %llu logf %llu sinf %llu cosf %llu f2bf %llu checked %llu\n", c.tanh_bad, c.expm1_bad, c.exp_bad, c.log_bad, c.sin_bad,
           c.cos_bad, c.bf_bad, c.checked);
    return (c.tanh_bad | c.expm1_bad | c.exp_bad | c.log_bad | c.sin_bad | c.cos_bad | c.bf_bad) ? 1 : 0;
}
