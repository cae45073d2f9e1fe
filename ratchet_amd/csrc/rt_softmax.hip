// Softmax over the last dimension.
//
// Arithmetic contract (REFERENCE mode) = crates/ratchet-core/src/cpu/softmax.rs:22-42: e_j = exp(x_j) with no max
// subtraction, stored in the element type; sum accumulated over j ascending in the element type; y_j = e_j / sum.
//   f32: the row lives in registers (one wave64 per row, 16-byte loads), one exp per element, the sum is a wave
//        butterfly instead of a sequential fold (differs from the reference by float rounding order only), one
//        IEEE division per element.  HBM traffic: one read, one write.
//   f16/bf16: the sequential 16-bit accumulation is order dependent (terms below half an ulp of the running sum
//        vanish), so it is replayed exactly: a block stages tiles of exp values through LDS and one lane per row walks
//        its row left to right with v_add_f16; the second pass recomputes the same exp values and divides.
// STABLE mode subtracts the row maximum and accumulates in f32 for every type.
#include "rt_arith.h"
#include "rt_internal.h"

namespace {

constexpr int WAVE = 64;
constexpr int BLOCK = 256;
constexpr int WAVES = BLOCK / WAVE;

template <typename T> __device__ __forceinline__ float stable_exp(float v) { return expf(v); }

// ------------------------------------------------------------------------------------------------------------------
// wave-per-row, row held in registers.  Requires cols % VE == 0, 16-byte aligned rows, cols / VE <= 64 * NV.
// MODE 0: reference arithmetic for f32 (exp, tree sum, divide).  MODE 1: stable (max subtraction, f32 accumulate) for
// any T; results are rounded to T once.
// ------------------------------------------------------------------------------------------------------------------
template <typename T, int NV, int MODE>
__global__ void __launch_bounds__(BLOCK) softmax_wave_kernel(const T* __restrict__ x, T* __restrict__ y, uint64_t rows,
                                                             uint32_t cols) {
    constexpr int VE = 16 / sizeof(T);
    const uint64_t row = (uint64_t)blockIdx.x * WAVES + (threadIdx.x / WAVE);
    if (row >= rows) return;
    const int lane = threadIdx.x & (WAVE - 1);
    const uint32_t nvec = cols / VE;
    const uint4* xr = reinterpret_cast<const uint4*>(x + row * cols);
    uint4* yr = reinterpret_cast<uint4*>(y + row * cols);
    Vec16<T> v[NV];
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * WAVE;
        if (i < nvec) v[k].u = xr[i];
    }
    float e[NV][VE];
    if (MODE == 1) {
        float m = -__builtin_huge_valf();
#pragma unroll
        for (int k = 0; k < NV; k++)
            if (lane + k * WAVE < nvec)
#pragma unroll
                for (int q = 0; q < VE; q++) m = fmaxf(m, Ar<T>::widen(v[k].e[q]));
        m = wave_max(m);
        if (m == -__builtin_huge_valf()) m = 0.0f;           // fully masked row: exp(-inf - 0) = 0, 0/0 = NaN as torch does
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; k++)
            if (lane + k * WAVE < nvec)
#pragma unroll
                for (int q = 0; q < VE; q++) {
                    e[k][q] = expf(Ar<T>::widen(v[k].e[q]) - m);
                    s += e[k][q];
                }
        s = wave_sum(s);
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = lane + k * WAVE;
            if (i < nvec) {
                Vec16<T> o;
#pragma unroll
                for (int q = 0; q < VE; q++) o.e[q] = Ar<T>::conv(e[k][q] / s);
                yr[i] = o.u;
            }
        }
    } else {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; k++)
            if (lane + k * WAVE < nvec)
#pragma unroll
                for (int q = 0; q < VE; q++) {
                    e[k][q] = rt_expf(Ar<T>::widen(v[k].e[q]));
                    s += e[k][q];
                }
        s = wave_sum(s);
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = lane + k * WAVE;
            if (i < nvec) {
                Vec16<T> o;
#pragma unroll
                for (int q = 0; q < VE; q++) o.e[q] = Ar<T>::conv(e[k][q] / s);
                yr[i] = o.u;
            }
        }
    }
}

// any cols, any alignment: one block per row, scalar accesses, row re-read from memory (cache) between passes
template <typename T, int MODE>
__global__ void __launch_bounds__(BLOCK) softmax_generic_kernel(const T* __restrict__ x, T* __restrict__ y, uint64_t rows,
                                                                uint32_t cols) {
    __shared__ float red[WAVES];
    __shared__ float bcast;
    const uint64_t row = blockIdx.x;
    const T* xr = x + row * cols;
    T* yr = y + row * cols;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    float m = 0.0f;
    if (MODE == 1) {
        float lm = -__builtin_huge_valf();
        for (uint32_t j = threadIdx.x; j < cols; j += BLOCK) lm = fmaxf(lm, Ar<T>::widen(xr[j]));
        lm = wave_max(lm);
        if (lane == 0) red[wave] = lm;
        __syncthreads();
        if (threadIdx.x == 0) {
            float t = red[0];
            for (int w = 1; w < WAVES; w++) t = fmaxf(t, red[w]);
            bcast = (t == -__builtin_huge_valf()) ? 0.0f : t;
        }
        __syncthreads();
        m = bcast;
        __syncthreads();
    }
    float s = 0.0f;
    for (uint32_t j = threadIdx.x; j < cols; j += BLOCK)
        s += (MODE == 1) ? expf(Ar<T>::widen(xr[j]) - m) : rt_expf(Ar<T>::widen(xr[j]));
    s = wave_sum(s);
    if (lane == 0) red[wave] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = red[0];
        for (int w = 1; w < WAVES; w++) t += red[w];
        bcast = t;
    }
    __syncthreads();
    s = bcast;
    for (uint32_t j = threadIdx.x; j < cols; j += BLOCK) {
        const float ev = (MODE == 1) ? expf(Ar<T>::widen(xr[j]) - m) : rt_expf(Ar<T>::widen(xr[j]));
        yr[j] = Ar<T>::conv(ev / s);
    }
}

// ------------------------------------------------------------------------------------------------------------------
// 16-bit reference arithmetic: exact replay of the sequential accumulation.
// A block owns RB consecutive rows.  Pass A walks the columns in tiles of TC: all threads load 16-byte vectors
// (coalesced), compute e = T(exp(x)) and park it in LDS; then lane r of wave 0 adds tile[r][0..TC) to its running
// T-typed sum, left to right.  Pass B re-reads x, recomputes the same e and writes T(e / sum).
// ------------------------------------------------------------------------------------------------------------------
template <typename T, int RB, int TC, bool VEC>
__global__ void __launch_bounds__(BLOCK) softmax_seq16_kernel(const T* __restrict__ x, T* __restrict__ y, uint64_t rows,
                                                              uint32_t cols) {
    constexpr int VE = VEC ? 8 : 1;
    constexpr int PAD = 8;                                   // keeps 16-byte alignment of LDS rows
    constexpr int TV = TC / VE;                              // vectors per tile row
    __shared__ __attribute__((aligned(16))) T tile[RB][TC + PAD];
    __shared__ T sums[RB];
    const uint64_t row0 = (uint64_t)blockIdx.x * RB;
    const uint32_t nrows = (rows - row0 < (uint64_t)RB) ? (uint32_t)(rows - row0) : (uint32_t)RB;
    T run = Ar<T>::conv(0.0f);

    for (uint32_t c0 = 0; c0 < cols; c0 += TC) {
        const uint32_t ncol = (cols - c0 < (uint32_t)TC) ? cols - c0 : (uint32_t)TC;
        for (uint32_t idx = threadIdx.x; idx < (uint32_t)RB * TV; idx += BLOCK) {
            const uint32_t r = idx / TV, cv = idx % TV;
            const uint32_t col = cv * VE;
            if (r < nrows && col < ncol) {
                const T* src = x + (row0 + r) * cols + c0 + col;
                if (VEC) {
                    Vec16<T> in, out;
                    in.u = *reinterpret_cast<const uint4*>(src);
#pragma unroll
                    for (int q = 0; q < 8; q++) out.e[q] = ar_exp<T>(in.e[q]);
                    *reinterpret_cast<uint4*>(&tile[r][col]) = out.u;
                } else {
                    tile[r][col] = ar_exp<T>(*src);
                }
            }
        }
        __syncthreads();
        if (threadIdx.x < nrows) {
            const T* trow = tile[threadIdx.x];
            if (VEC) {
                // ncol is a multiple of 8 here (cols % 8 == 0 and TC % 8 == 0)
                for (uint32_t j = 0; j < ncol; j += 8) {
                    Vec16<T> t;
                    t.u = *reinterpret_cast<const uint4*>(trow + j);
#pragma unroll
                    for (int q = 0; q < 8; q++) run = Ar<T>::add(run, t.e[q]);
                }
            } else {
                for (uint32_t j = 0; j < ncol; j++) run = Ar<T>::add(run, trow[j]);
            }
        }
        __syncthreads();
    }
    if (threadIdx.x < nrows) sums[threadIdx.x] = run;
    __syncthreads();

    const uint32_t cvec = cols / VE;
    for (uint32_t r = 0; r < nrows; r++) {
        const T sum = sums[r];
        const T* src = x + (row0 + r) * cols;
        T* dst = y + (row0 + r) * cols;
        for (uint32_t cv = threadIdx.x; cv < cvec; cv += BLOCK) {
            if (VEC) {
                Vec16<T> in, out;
                in.u = reinterpret_cast<const uint4*>(src)[cv];
#pragma unroll
                for (int q = 0; q < 8; q++) out.e[q] = Ar<T>::div(ar_exp<T>(in.e[q]), sum);
                reinterpret_cast<uint4*>(dst)[cv] = out.u;
            } else {
                dst[cv] = Ar<T>::div(ar_exp<T>(src[cv]), sum);
            }
        }
    }
}

template <typename T, int MODE> int launch_wave(rt_device* dev, const void* x, void* y, uint64_t rows, uint32_t cols) {
    constexpr int VE = 16 / sizeof(T);
    const uint32_t nvec = cols / VE;
    const uint32_t nv = (nvec + WAVE - 1) / WAVE;
    const uint64_t blocks = (rows + WAVES - 1) / WAVES;
    RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax: too many rows");
    const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_SM(NVC) hipLaunchKernelGGL((softmax_wave_kernel<T, NVC, MODE>), grid, block, 0, dev->stream, (const T*)x, (T*)y, rows, cols)
    if (nv <= 1) RT_SM(1);
    else if (nv <= 2) RT_SM(2);
    else if (nv <= 3) RT_SM(3);
    else if (nv <= 4) RT_SM(4);
    else if (nv <= 6) RT_SM(6);
    else RT_SM(8);
#undef RT_SM
    RT_CHECK_LAUNCH("softmax_wave_kernel");
    return RT_OK;
}

template <typename T, int MODE> int launch_f32_style(rt_device* dev, const void* x, void* y, uint64_t rows, uint32_t cols) {
    constexpr int VE = 16 / sizeof(T);
    const bool vec_ok = (cols % VE == 0) && rt_aligned(x, 16) && rt_aligned(y, 16) && (cols / VE) <= (uint32_t)(WAVE * 8);
    if (vec_ok) return launch_wave<T, MODE>(dev, x, y, rows, cols);
    RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax: too many rows");
    hipLaunchKernelGGL((softmax_generic_kernel<T, MODE>), dim3((unsigned)rows), dim3(BLOCK), 0, dev->stream, (const T*)x, (T*)y, rows,
                       cols);
    RT_CHECK_LAUNCH("softmax_generic_kernel");
    return RT_OK;
}

template <typename T> int launch_seq16(rt_device* dev, const void* x, void* y, uint64_t rows, uint32_t cols) {
    constexpr int RB = 64, TC = 128;
    const uint64_t blocks = (rows + RB - 1) / RB;
    RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax: too many rows");
    const bool vec_ok = (cols % 8 == 0) && rt_aligned(x, 16) && rt_aligned(y, 16);
    if (vec_ok) {
        hipLaunchKernelGGL((softmax_seq16_kernel<T, RB, TC, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, dev->stream, (const T*)x,
                           (T*)y, rows, cols);
    } else {
        hipLaunchKernelGGL((softmax_seq16_kernel<T, RB, TC, false>), dim3((unsigned)blocks), dim3(BLOCK), 0, dev->stream, (const T*)x,
                           (T*)y, rows, cols);
    }
    RT_CHECK_LAUNCH("softmax_seq16_kernel");
    return RT_OK;
}

}  // namespace

extern "C" int rt_softmax(rt_device* dev, int dt, const void* x, void* y, uint64_t rows, uint32_t cols, int mode) {
    RT_REQUIRE(rt_is_float_dt(dt), RT_ERR_DTYPE, "rt_softmax: dtype %d is not F32/F16/BF16", dt);   // Softmax::check_dtypes
    RT_REQUIRE(mode == RT_SOFTMAX_REFERENCE || mode == RT_SOFTMAX_STABLE, RT_ERR_ARG, "rt_softmax: unknown mode %d", mode);
    RT_REQUIRE(cols > 0, RT_ERR_SHAPE, "rt_softmax: cols is 0");
    RT_REQUIRE(rows <= RT_MAX_NUMEL / cols, RT_ERR_SIZE, "rt_softmax: tensor too large");
    if (rows == 0) return dev ? RT_OK : rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(x && y, RT_ERR_NULL_POINTER, "rt_softmax: NULL operand");
    const size_t eb = (size_t)rt_dt_bytes(dt);
    RT_REQUIRE(rt_aligned(x, eb) && rt_aligned(y, eb), RT_ERR_ALIGN, "rt_softmax: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (mode == RT_SOFTMAX_STABLE) {
        switch (dt) {
            case RT_F32: return launch_f32_style<float, 1>(dev, x, y, rows, cols);
            case RT_F16: return launch_f32_style<half_t, 1>(dev, x, y, rows, cols);
            default: return launch_f32_style<bf16_t, 1>(dev, x, y, rows, cols);
        }
    }
    switch (dt) {
        case RT_F32: return launch_f32_style<float, 0>(dev, x, y, rows, cols);
        case RT_F16: return launch_seq16<half_t>(dev, x, y, rows, cols);
        default: return launch_seq16<bf16_t>(dev, x, y, rows, cols);
    }
}
