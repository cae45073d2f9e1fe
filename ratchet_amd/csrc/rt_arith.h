// Per-element-type arithmetic policies for the kernels.  Ar<T> gives every kernel the rounding points of ratchet's CPU
// executor, which is generic Rust over f32 / half::f16 / half::bf16 (crates/ratchet-core/src/cpu/*.rs): for the 16-bit
// types every operator and every libm call is "widen to f32, operate, round to nearest even".
//   f16: + - * use the native v_*_f16 instructions (IEEE, correctly rounded, identical to going through f32);
//        / and sqrt go through correctly rounded f32 (24 >= 2*11+2 bits, so the second rounding is innocuous).
//   bf16: everything through f32.
// Compile with -ffp-contract=off.
#ifndef RT_ARITH_H
#define RT_ARITH_H

#include "../../include/ratchet_hip.h"
#include "rt_internal.h"
#include "rt_math.h"

struct bf16_t {
    uint16_t b;
};

template <typename T> struct Ar;

template <> struct Ar<float> {
    typedef float T;
    static constexpr int BYTES = 4;
    static __device__ __forceinline__ T conv(float f) { return f; }
    static __device__ __forceinline__ float widen(T a) { return a; }
    static __device__ __forceinline__ T add(T a, T b) { return a + b; }
    static __device__ __forceinline__ T sub(T a, T b) { return a - b; }
    static __device__ __forceinline__ T mul(T a, T b) { return a * b; }
    static __device__ __forceinline__ T div(T a, T b) { return a / b; }
    static __device__ __forceinline__ T neg(T a) { return u2f(f2u(a) ^ 0x80000000u); }
    static __device__ __forceinline__ T abs(T a) { return u2f(f2u(a) & 0x7fffffffu); }
    // f32::max(x, 0.0): NaN gives 0.0; -0.0 is kept (x86 lowering of maxnum keeps the first operand on equality)
    static __device__ __forceinline__ T relu(T a) { return (a != a) ? 0.0f : ((0.0f > a) ? 0.0f : a); }
};

template <> struct Ar<half_t> {
    typedef half_t T;
    static constexpr int BYTES = 2;
    static __device__ __forceinline__ T conv(float f) { return (half_t)f; }
    static __device__ __forceinline__ float widen(T a) { return (float)a; }
    static __device__ __forceinline__ T add(T a, T b) { return a + b; }
    static __device__ __forceinline__ T sub(T a, T b) { return a - b; }
    static __device__ __forceinline__ T mul(T a, T b) { return a * b; }
    static __device__ __forceinline__ T div(T a, T b) { return (half_t)((float)a / (float)b); }
    static __device__ __forceinline__ T neg(T a) { return bits_h((uint16_t)(h_bits(a) ^ 0x8000u)); }
    static __device__ __forceinline__ T abs(T a) { return bits_h((uint16_t)(h_bits(a) & 0x7fffu)); }
    // half's max keeps a NaN input (`if other > self && !other.is_nan() { other } else { self }`)
    static __device__ __forceinline__ T relu(T a) { return (0.0f > (float)a) ? (half_t)0.0f : a; }
};

template <> struct Ar<bf16_t> {
    typedef bf16_t T;
    static constexpr int BYTES = 2;
    // The chip's own conversion (round to nearest even, NaN quieted), one instruction, written as an instruction: through
    // `(__bf16)f` this compiler fails to select code for it in some kernels ("cannot select v2f32 = bitcast" in the
    // f32-routed unary kernel).  The second operand's half of the result is not used.  On the bit pattern the same
    // rounding is six instructions, and the 16-bit norms spend four conversions on every element.
    static __device__ __forceinline__ T conv(float f) {
        uint32_t r;
        asm("v_cvt_pk_bf16_f32 %0, %1, 0" : "=v"(r) : "v"(f));
        T out;
        out.b = (uint16_t)r;
        return out;
    }
    static __device__ __forceinline__ float widen(T a) { return bf2f(a.b); }
    static __device__ __forceinline__ T add(T a, T b) { return conv(widen(a) + widen(b)); }
    static __device__ __forceinline__ T sub(T a, T b) { return conv(widen(a) - widen(b)); }
    static __device__ __forceinline__ T mul(T a, T b) { return conv(widen(a) * widen(b)); }
    static __device__ __forceinline__ T div(T a, T b) { return conv(widen(a) / widen(b)); }
    static __device__ __forceinline__ T neg(T a) { T r; r.b = (uint16_t)(a.b ^ 0x8000u); return r; }
    static __device__ __forceinline__ T abs(T a) { T r; r.b = (uint16_t)(a.b & 0x7fffu); return r; }
    static __device__ __forceinline__ T relu(T a) { return (0.0f > widen(a)) ? conv(0.0f) : a; }
};

// libm-style calls: always through f32 (num_traits::Float on the half types widens)
template <typename T> __device__ __forceinline__ T ar_tanh(T a) { return Ar<T>::conv(rt_tanhf(Ar<T>::widen(a))); }
// (tab: the table of rt_expf_tab, where a kernel has staged a copy of it)
template <typename T> __device__ __forceinline__ T ar_exp(T a, const uint64_t* tab = rt_exp2f_tab) { return Ar<T>::conv(rt_expf_tab(Ar<T>::widen(a), tab)); }
// (tab: the 32 words of rt_logf_tab, wherever the caller keeps them)
template <typename T> __device__ __forceinline__ T ar_log(T a, const uint64_t* tab = nullptr) {
    return Ar<T>::conv(tab ? rt_logf_tab_at(Ar<T>::widen(a), reinterpret_cast<const double*>(tab)) : rt_logf(Ar<T>::widen(a)));
}
template <typename T> __device__ __forceinline__ T ar_sin(T a) { return Ar<T>::conv(rt_sinf(Ar<T>::widen(a))); }
template <typename T> __device__ __forceinline__ T ar_cos(T a) { return Ar<T>::conv(rt_cosf(Ar<T>::widen(a))); }
template <typename T> __device__ __forceinline__ T ar_sqrt(T a) { return Ar<T>::conv(__builtin_sqrtf(Ar<T>::widen(a))); }
template <typename T> __device__ __forceinline__ T ar_floor(T a) { return Ar<T>::conv(floorf(Ar<T>::widen(a))); }
template <typename T> __device__ __forceinline__ T ar_ceil(T a) { return Ar<T>::conv(ceilf(Ar<T>::widen(a))); }

// cpu/unary.rs:46-51: conv(0.5) * x * (conv(1.0) + tanh(conv(0.797_884_6) * x * (conv(1.0) + conv(0.044715) * x * x)))
template <typename T> __device__ __forceinline__ T ar_gelu(T x) {
    typedef Ar<T> A;
    const T inner = A::add(A::conv(1.0f), A::mul(A::mul(A::conv(0.044715f), x), x));
    const T arg = A::mul(A::mul(A::conv(0.7978846f), x), inner);
    const T t = ar_tanh<T>(arg);
    return A::mul(A::mul(A::conv(0.5f), x), A::add(A::conv(1.0f), t));
}
// cpu/unary.rs:64: x / (1 + exp(-x))
template <typename T> __device__ __forceinline__ T ar_silu(T x, const uint64_t* tab = rt_exp2f_tab) {
    typedef Ar<T> A;
    return A::div(x, A::add(A::conv(1.0f), ar_exp<T>(A::neg(x), tab)));
}
// cpu/unary.rs:65: 1 / (1 + exp(-x))
template <typename T> __device__ __forceinline__ T ar_sigmoid(T x, const uint64_t* tab = rt_exp2f_tab) {
    typedef Ar<T> A;
    return A::div(A::conv(1.0f), A::add(A::conv(1.0f), ar_exp<T>(A::neg(x), tab)));
}

constexpr bool ar_unary_uses_exp(int op) { return op == RT_EXP || op == RT_SILU || op == RT_SIGMOID; }
constexpr bool ar_unary_uses_log(int op) { return op == RT_LOG; }
template <int OP, typename T> __device__ __forceinline__ T ar_unary(T x, const uint64_t* tab = rt_exp2f_tab) {
    if (OP == RT_GELU) return ar_gelu<T>(x);
    if (OP == RT_TANH) return ar_tanh<T>(x);
    if (OP == RT_EXP) return ar_exp<T>(x, tab);
    if (OP == RT_LOG) return ar_log<T>(x, tab == rt_exp2f_tab ? nullptr : tab);
    if (OP == RT_SIN) return ar_sin<T>(x);
    if (OP == RT_COS) return ar_cos<T>(x);
    if (OP == RT_ABS) return Ar<T>::abs(x);
    if (OP == RT_SQRT) return ar_sqrt<T>(x);
    if (OP == RT_RELU) return Ar<T>::relu(x);
    if (OP == RT_FLOOR) return ar_floor<T>(x);
    if (OP == RT_CEIL) return ar_ceil<T>(x);
    if (OP == RT_NEG) return Ar<T>::neg(x);
    if (OP == RT_SILU) return ar_silu<T>(x, tab);
    return ar_sigmoid<T>(x, tab);
}

template <int OP, typename T> __device__ __forceinline__ T ar_binary(T a, T b) {
    if (OP == RT_ADD) return Ar<T>::add(a, b);
    if (OP == RT_SUB) return Ar<T>::sub(a, b);
    if (OP == RT_MUL) return Ar<T>::mul(a, b);
    return Ar<T>::div(a, b);
}

// 16-byte register vector viewed as elements of T
template <typename T> union Vec16 {
    v4u u;
    T e[16 / sizeof(T)];
    __device__ __forceinline__ Vec16() {}
};

#endif
