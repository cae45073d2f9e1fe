// LayerNorm, RMSNorm (one wave64 per row, row held in registers, 16-byte loads, butterfly reductions) and GroupNorm
// (split statistics + apply, two launches).
//
// Arithmetic contract for LayerNorm / RMSNorm = crates/ratchet-core/src/cpu/norm.rs:91-147,185-213, in the element type T
// with one rounding per operation:
//     mu   = sum(x) / T(N)                 (sum::<T>: f32 accumulation; for 16-bit T rounded to T once)
//     x2   = sum(x*x) / T(N)               (each square rounded to T first)
//     var  = x2 - mu*mu                    (E[x^2] - mu^2, not a two-pass variance)
//     r    = T(1) / sqrt(var + T(eps))
//     y    = ((x - mu) * r) * scale + bias
// f32 rows: one wave64 per row, the row stays in registers, the additions form a butterfly tree instead of the
//   reference's sequential fold; that changes the sums by float rounding only (far inside the 1e-5 bar).
// 16-bit rows: the two sums are rounded to the 16-bit type before they are used (sum(x*x) ~ N has an ulp of 1-2 there),
//   so a different f32 summation order can flip that rounding and move a whole row by an ulp of r, more than 1e-3
//   allows.  These kernels therefore replay the reference's order exactly: tiles of x and T(x*x) are staged through LDS
//   as f32 and one lane per (row, sum) walks its row left to right with v_add_f32.  The walk is latency bound
//   (one dependent add per element), so many small row groups run side by side.
// GroupNorm follows torch.nn.functional.group_norm, the ground truth of the reference's own test
// (ops/norm/groupnorm.rs:24-31): statistics in f32 (Chan-combined partial mean/M2), f32 arithmetic, one final rounding.
#include <type_traits>

#include "rt_arith.h"
#include "rt_internal.h"

namespace {

constexpr int WAVE = 64;
constexpr int BLOCK = 256;
constexpr int WAVES = BLOCK / WAVE;

enum { NORM_LAYER = 0, NORM_RMS = 1 };

// Partial statistics for rt_group_norm_static, the entry point that allocates nothing: a fixed array in the code object,
// one copy per GPU.  In host code the array's name is only a stand-in; rt_norm_device_init asks the runtime where the
// current device's copy lies and every launch is given that pointer.
constexpr size_t GN_STATIC_SCRATCH_BYTES = 256 * 1024;
static __device__ __align__(256) unsigned char gn_static_scratch[GN_STATIC_SCRATCH_BYTES];
constexpr int NORM_WIDE_BLOCK = 1024;                   // threads per row for f32 rows that do not fit 256 threads' registers

// per-row statistics in T arithmetic, given f32 sums
template <typename T> struct RowStats {
    T mu, r;
};
template <typename T, int KIND> __device__ __forceinline__ RowStats<T> finish_stats(float sum_x, float sum_sq, uint32_t cols, float eps) {
    typedef Ar<T> A;
    RowStats<T> st;
    const T n = A::conv((float)cols);                       // T::from(step as f32)
    const T x2 = A::div(A::conv(sum_sq), n);
    T var;
    if (KIND == NORM_LAYER) {
        st.mu = A::div(A::conv(sum_x), n);
        var = A::sub(x2, A::mul(st.mu, st.mu));
    } else {
        st.mu = A::conv(0.0f);
        var = x2;
    }
    const T t = A::add(var, A::conv(eps));
    st.r = A::div(A::conv(1.0f), ar_sqrt<T>(t));
    return st;
}

template <typename T, int KIND> __device__ __forceinline__ T norm_one(T x, const RowStats<T>& st, T scale, T bias, bool has_bias) {
    typedef Ar<T> A;
    T v = (KIND == NORM_LAYER) ? A::sub(x, st.mu) : x;
    v = A::mul(v, st.r);
    v = A::mul(v, scale);
    if (KIND == NORM_LAYER && has_bias) v = A::add(v, bias);
    return v;
}

// x and y 16-byte aligned, at most LANES * NV vectors per row.  Rows of whole vectors (scale and bias 16-byte aligned as
// well), or SPAN: rows of any length over the aligned vectors that cover them.  A row then starts `shift` elements into
// its first vector; span elements outside the row belong to the neighbouring rows, stay out of the sums and are not
// written (the row's two ragged vectors are stored element by element), and scale / bias are read by column.  An
// aligned vector that holds one byte of the tensor lies in a mapped page, so the loads are safe at the tensor's ends too.
template <typename T, int NV, int KIND, int LANES, bool SPAN>
__global__ void __launch_bounds__(LANES > BLOCK ? LANES : BLOCK) norm_wave_kernel(const T* x, const T* __restrict__ scale,
                                                                                  const T* __restrict__ bias, T* y, uint64_t rows,
                                                                                  uint32_t cols, float eps) {
    constexpr int VE = 16 / sizeof(T);
    constexpr int THREADS = LANES > BLOCK ? LANES : BLOCK;   // rows beyond 2048 vectors: one 1024-thread block per row
    const uint64_t row = (uint64_t)blockIdx.x * (THREADS / LANES) + (threadIdx.x / LANES);
    if (row >= rows) return;
    const int lane = threadIdx.x & (LANES - 1);
    const uint64_t first = row * cols;
    const uint32_t shift = SPAN ? (uint32_t)(first & (VE - 1)) : 0;
    const uint32_t nvec = SPAN ? (shift + cols + VE - 1) / VE : cols / VE;
    const v4u* xr = reinterpret_cast<const v4u*>(x) + first / VE;
    v4u* yr = reinterpret_cast<v4u*>(y) + first / VE;
    auto inside = [&](uint32_t i, int q) -> bool { return !SPAN || i * VE + (uint32_t)q - shift < cols; };
    Vec16<T> v[NV];
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nvec) v[k].u = ld_stream(xr + i);
    }
    float sx = 0.0f, sq = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++)
        if (lane + k * LANES < nvec)
#pragma unroll
            for (int q = 0; q < VE; q++)
                if (inside(lane + k * LANES, q)) {
                    const T e = v[k].e[q];
                    if (KIND == NORM_LAYER) sx += Ar<T>::widen(e);
                    sq += Ar<T>::widen(Ar<T>::mul(e, e));
                }
    if (KIND == NORM_LAYER) sx = row_sum<LANES>(sx);
    sq = row_sum<LANES>(sq);
    const RowStats<T> st = finish_stats<T, KIND>(sx, sq, cols, eps);
    const v4u* sv = reinterpret_cast<const v4u*>(scale);
    const v4u* bv = reinterpret_cast<const v4u*>(bias);
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nvec) {
            Vec16<T> s, b, o;
            if (!SPAN) {
                s.u = sv[i];
                if (KIND == NORM_LAYER && bias) b.u = bv[i];
#pragma unroll
                for (int q = 0; q < VE; q++) o.e[q] = norm_one<T, KIND>(v[k].e[q], st, s.e[q], b.e[q], bias != nullptr);
                st_stream(yr + i, o.u);
            } else if (inside(i, 0) && inside(i, VE - 1)) {
                // a vector inside the row: its scale / bias elements are 16 contiguous bytes at element alignment
                const uint32_t c0 = i * VE - shift;
                __builtin_memcpy(&s.u, scale + c0, 16);
                if (KIND == NORM_LAYER && bias) __builtin_memcpy(&b.u, bias + c0, 16);
#pragma unroll
                for (int q = 0; q < VE; q++) o.e[q] = norm_one<T, KIND>(v[k].e[q], st, s.e[q], b.e[q], bias != nullptr);
                st_stream(yr + i, o.u);
            } else {
                T* yrow = y + first;
#pragma unroll
                for (int q = 0; q < VE; q++) {
                    const uint32_t c = i * VE + (uint32_t)q - shift;
                    if (c < cols) {
                        const T bq = (KIND == NORM_LAYER && bias) ? bias[c] : Ar<T>::conv(0.0f);
                        yrow[c] = norm_one<T, KIND>(v[k].e[q], st, scale[c], bq, bias != nullptr);
                    }
                }
            }
        }
    }
}

// any cols / alignment: one block per row, scalar accesses, the row is re-read from cache for the second pass
template <typename T, int KIND>
__global__ void __launch_bounds__(BLOCK) norm_generic_kernel(const T* __restrict__ x, const T* __restrict__ scale,
                                                             const T* __restrict__ bias, T* __restrict__ y, uint64_t rows, uint32_t cols,
                                                             float eps) {
    __shared__ float red[2][WAVES];
    const uint64_t row = blockIdx.x;
    const T* xr = x + row * cols;
    T* yr = y + row * cols;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    float sx = 0.0f, sq = 0.0f;
    for (uint32_t j = threadIdx.x; j < cols; j += BLOCK) {
        const T e = xr[j];
        sx += Ar<T>::widen(e);
        sq += Ar<T>::widen(Ar<T>::mul(e, e));
    }
    sx = wave_sum(sx);
    sq = wave_sum(sq);
    if (lane == 0) { red[0][wave] = sx; red[1][wave] = sq; }
    __syncthreads();
    sx = red[0][0]; sq = red[1][0];
    for (int w = 1; w < WAVES; w++) { sx += red[0][w]; sq += red[1][w]; }
    const RowStats<T> st = finish_stats<T, KIND>(sx, sq, cols, eps);
    for (uint32_t j = threadIdx.x; j < cols; j += BLOCK) {
        const T b = (KIND == NORM_LAYER && bias) ? bias[j] : Ar<T>::conv(0.0f);
        yr[j] = norm_one<T, KIND>(xr[j], st, scale[j], b, bias != nullptr);
    }
}

// ------------------------------------------------------------------------------------------------------------------
// The caller pattern of ratchet-nn (src/norm.rs:35-44, 61-70): x.full().layer_norm(w, b, eps).cast(src_dt) on a
// 16-bit x with f32 weights, in one pass: the row is widened into registers, the f32 norm arithmetic above is applied
// (butterfly sums) and the result is rounded once.  4 bytes of traffic per element instead of the 16 of the three
// separate ops, and no sequential chain: the f32 sums need no replay because the parity bar after the cast is the
// 16-bit one.
// ------------------------------------------------------------------------------------------------------------------
template <typename T, int NV, int KIND, int LANES>
__global__ void __launch_bounds__(BLOCK) norm_via32_wave_kernel(const T* __restrict__ x, const float* __restrict__ scale,
                                                                const float* __restrict__ bias, T* __restrict__ y, uint64_t rows,
                                                                uint32_t cols, float eps) {
    const uint64_t row = (uint64_t)blockIdx.x * (BLOCK / LANES) + (threadIdx.x / LANES);
    if (row >= rows) return;
    const int lane = threadIdx.x & (LANES - 1);
    const uint32_t nvec = cols / 8;
    const v4u* xr = reinterpret_cast<const v4u*>(x + row * cols);
    v4u* yr = reinterpret_cast<v4u*>(y + row * cols);
    Vec16<T> v[NV];
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nvec) v[k].u = ld_stream(xr + i);
    }
    float sx = 0.0f, sq = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++)
        if (lane + k * LANES < nvec)
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const float e = Ar<T>::widen(v[k].e[q]);
                if (KIND == NORM_LAYER) sx += e;
                sq += e * e;
            }
    if (KIND == NORM_LAYER) sx = row_sum<LANES>(sx);
    sq = row_sum<LANES>(sq);
    const RowStats<float> st = finish_stats<float, KIND>(sx, sq, cols, eps);
    const float4* sv = reinterpret_cast<const float4*>(scale);
    const float4* bv = reinterpret_cast<const float4*>(bias);
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nvec) {
            float s[8], b[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            *reinterpret_cast<float4*>(s) = sv[2 * i];
            *reinterpret_cast<float4*>(s + 4) = sv[2 * i + 1];
            if (KIND == NORM_LAYER && bias) {
                *reinterpret_cast<float4*>(b) = bv[2 * i];
                *reinterpret_cast<float4*>(b + 4) = bv[2 * i + 1];
            }
            Vec16<T> o;
#pragma unroll
            for (int q = 0; q < 8; q++)
                o.e[q] = Ar<T>::conv(norm_one<float, KIND>(Ar<T>::widen(v[k].e[q]), st, s[q], b[q], bias != nullptr));
            st_stream(yr + i, o.u);
        }
    }
}

// RW rows per wave (or per block, LANES == BLOCK): the f32 weights are twice the bytes of a 16-bit row (four times with a
// bias), and every row fetches them again, behind its reduction, where only the other waves hide the wait
// ([16384,4096] LayerNorm 52.8 us; without the weight loads 46.1 us; a copy of the same bytes 42.9 us).  With RW rows in
// registers the weights of a vector are loaded once and applied RW times.  The launcher says where that pays.
template <typename T, int NV, int KIND, int LANES, int RW>
__global__ void __launch_bounds__(BLOCK) norm_via32_rows_kernel(const T* __restrict__ x, const float* __restrict__ scale,
                                                                const float* __restrict__ bias, T* __restrict__ y, uint64_t rows,
                                                                uint32_t cols, float eps) {
    const uint64_t row0 = ((uint64_t)blockIdx.x * (BLOCK / LANES) + (threadIdx.x / LANES)) * RW;
    if (row0 >= rows) return;
    const int lane = threadIdx.x & (LANES - 1);
    const uint32_t nvec = cols / 8;
    Vec16<T> v[RW][NV];
#pragma unroll
    for (int r = 0; r < RW; r++) {
        // a row past the end reads the last row once more (its result is not stored): no branch around the loads
        const uint64_t row = row0 + r < rows ? row0 + r : rows - 1;
        const v4u* xr = reinterpret_cast<const v4u*>(x + row * cols);
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = lane + k * LANES;
            if (i < nvec) v[r][k].u = ld_stream(xr + i);
        }
    }
    RowStats<float> st[RW];
#pragma unroll
    for (int r = 0; r < RW; r++) {
        float sx = 0.0f, sq = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; k++)
            if (lane + k * LANES < nvec)
#pragma unroll
                for (int q = 0; q < 8; q++) {
                    const float e = Ar<T>::widen(v[r][k].e[q]);
                    if (KIND == NORM_LAYER) sx += e;
                    sq += e * e;
                }
        if (KIND == NORM_LAYER) sx = row_sum<LANES>(sx);
        sq = row_sum<LANES>(sq);
        st[r] = finish_stats<float, KIND>(sx, sq, cols, eps);
    }
    const float4* sv = reinterpret_cast<const float4*>(scale);
    const float4* bv = reinterpret_cast<const float4*>(bias);
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nvec) {
            float s[8], b[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            *reinterpret_cast<float4*>(s) = sv[2 * i];
            *reinterpret_cast<float4*>(s + 4) = sv[2 * i + 1];
            if (KIND == NORM_LAYER && bias) {
                *reinterpret_cast<float4*>(b) = bv[2 * i];
                *reinterpret_cast<float4*>(b + 4) = bv[2 * i + 1];
            }
#pragma unroll
            for (int r = 0; r < RW; r++) {
                if (row0 + r >= rows) break;
                Vec16<T> o;
#pragma unroll
                for (int q = 0; q < 8; q++)
                    o.e[q] = Ar<T>::conv(norm_one<float, KIND>(Ar<T>::widen(v[r][k].e[q]), st[r], s[q], b[q], bias != nullptr));
                st_stream(reinterpret_cast<v4u*>(y + (row0 + r) * cols) + i, o.u);
            }
        }
    }
}

// any cols / alignment: one block per row, scalar accesses, the row is re-read from cache for the second pass
template <typename T, int KIND>
__global__ void __launch_bounds__(BLOCK) norm_via32_generic_kernel(const T* __restrict__ x, const float* __restrict__ scale,
                                                                   const float* __restrict__ bias, T* __restrict__ y, uint64_t rows,
                                                                   uint32_t cols, float eps) {
    __shared__ float red[2][WAVES];
    const uint64_t row = blockIdx.x;
    const T* xr = x + row * cols;
    T* yr = y + row * cols;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    float sx = 0.0f, sq = 0.0f;
    for (uint32_t j = threadIdx.x; j < cols; j += BLOCK) {
        const float e = Ar<T>::widen(xr[j]);
        sx += e;
        sq += e * e;
    }
    sx = wave_sum(sx);
    sq = wave_sum(sq);
    if (lane == 0) { red[0][wave] = sx; red[1][wave] = sq; }
    __syncthreads();
    sx = red[0][0]; sq = red[1][0];
    for (int w = 1; w < WAVES; w++) { sx += red[0][w]; sq += red[1][w]; }
    const RowStats<float> st = finish_stats<float, KIND>(sx, sq, cols, eps);
    for (uint32_t j = threadIdx.x; j < cols; j += BLOCK) {
        const float b = (KIND == NORM_LAYER && bias) ? bias[j] : 0.0f;
        yr[j] = Ar<T>::conv(norm_one<float, KIND>(Ar<T>::widen(xr[j]), st, scale[j], b, bias != nullptr));
    }
}

// ------------------------------------------------------------------------------------------------------------------
// 16-bit LayerNorm / RMSNorm with the reference's sequential f32 accumulation.
// A block owns RB consecutive rows.  Pass A: per column tile, all threads load 16-byte vectors, widen x and T(x*x) to
// f32 and park them in LDS; lanes [0, RB) then add the squares of "their" row left to right, lanes [RB, 2RB) the values
// (LayerNorm only).  Pass B re-reads x (from cache: the block touched it moments ago), normalises and stores.
// ------------------------------------------------------------------------------------------------------------------
template <typename T, int RB, int KIND, bool VEC>
__global__ void __launch_bounds__(BLOCK) norm_seq16_kernel(const T* __restrict__ x, const T* __restrict__ scale,
                                                           const T* __restrict__ bias, T* __restrict__ y, uint64_t rows, uint32_t cols,
                                                           float eps) {
    constexpr int TC = 128;
    constexpr int PAD = 4;
    constexpr int VE = VEC ? 8 : 1;
    constexpr int TV = TC / VE;
    constexpr int NSUM = (KIND == NORM_LAYER) ? 2 : 1;
    __shared__ __attribute__((aligned(16))) float tile[NSUM][RB][TC + PAD];      // [0] = squares, [1] = values
    __shared__ float sums[NSUM][RB];
    __shared__ T s_mu[RB], s_r[RB];
    const uint64_t row0 = (uint64_t)blockIdx.x * RB;
    const uint32_t nrows = (rows - row0 < (uint64_t)RB) ? (uint32_t)(rows - row0) : (uint32_t)RB;
    const uint32_t wrow = threadIdx.x % RB, wsum = threadIdx.x / RB;                // walker role of this thread
    const bool walker = (threadIdx.x < NSUM * RB) && (wrow < nrows);
    float run = 0.0f;

    for (uint32_t c0 = 0; c0 < cols; c0 += TC) {
        const uint32_t ncol = (cols - c0 < (uint32_t)TC) ? cols - c0 : (uint32_t)TC;
        for (uint32_t idx = threadIdx.x; idx < (uint32_t)RB * TV; idx += BLOCK) {
            const uint32_t r = idx / TV, col = (idx % TV) * VE;
            if (r < nrows && col < ncol) {
                const T* src = x + (row0 + r) * cols + c0 + col;
                if (VEC) {
                    Vec16<T> in;
                    in.u = *reinterpret_cast<const v4u*>(src);
                    float sq[8], xv[8];
#pragma unroll
                    for (int q = 0; q < 8; q++) {
                        sq[q] = Ar<T>::widen(Ar<T>::mul(in.e[q], in.e[q]));
                        xv[q] = Ar<T>::widen(in.e[q]);
                    }
                    float4* d0 = reinterpret_cast<float4*>(&tile[0][r][col]);
                    d0[0] = make_float4(sq[0], sq[1], sq[2], sq[3]);
                    d0[1] = make_float4(sq[4], sq[5], sq[6], sq[7]);
                    if (KIND == NORM_LAYER) {
                        float4* d1 = reinterpret_cast<float4*>(&tile[NSUM - 1][r][col]);
                        d1[0] = make_float4(xv[0], xv[1], xv[2], xv[3]);
                        d1[1] = make_float4(xv[4], xv[5], xv[6], xv[7]);
                    }
                } else {
                    const T e = *src;
                    tile[0][r][col] = Ar<T>::widen(Ar<T>::mul(e, e));
                    if (KIND == NORM_LAYER) tile[NSUM - 1][r][col] = Ar<T>::widen(e);
                }
            }
        }
        __syncthreads();
        if (walker) {
            const float* trow = tile[wsum][wrow];
            uint32_t j = 0;
            for (; j + 4 <= ncol; j += 4) {
                const float4 t = *reinterpret_cast<const float4*>(trow + j);
                run += t.x;
                run += t.y;
                run += t.z;
                run += t.w;
            }
            for (; j < ncol; j++) run += trow[j];
        }
        __syncthreads();
    }
    if (walker) sums[wsum][wrow] = run;
    __syncthreads();
    if (threadIdx.x < nrows) {
        const RowStats<T> st = finish_stats<T, KIND>(KIND == NORM_LAYER ? sums[NSUM - 1][threadIdx.x] : 0.0f, sums[0][threadIdx.x],
                                                     cols, eps);
        s_mu[threadIdx.x] = st.mu;
        s_r[threadIdx.x] = st.r;
    }
    __syncthreads();

    const uint32_t cvec = cols / VE;
    for (uint32_t r = 0; r < nrows; r++) {
        RowStats<T> st;
        st.mu = s_mu[r];
        st.r = s_r[r];
        const T* src = x + (row0 + r) * cols;
        T* dst = y + (row0 + r) * cols;
        for (uint32_t cv = threadIdx.x; cv < cvec; cv += BLOCK) {
            if (VEC) {
                Vec16<T> in, sc, bi, out;
                in.u = reinterpret_cast<const v4u*>(src)[cv];
                sc.u = reinterpret_cast<const v4u*>(scale)[cv];
                if (KIND == NORM_LAYER && bias) bi.u = reinterpret_cast<const v4u*>(bias)[cv];
#pragma unroll
                for (int q = 0; q < 8; q++) out.e[q] = norm_one<T, KIND>(in.e[q], st, sc.e[q], bi.e[q], bias != nullptr);
                st_stream(reinterpret_cast<v4u*>(dst) + cv, out.u);
            } else {
                const T b = (KIND == NORM_LAYER && bias) ? bias[cv] : Ar<T>::conv(0.0f);
                dst[cv] = norm_one<T, KIND>(src[cv], st, scale[cv], b, bias != nullptr);
            }
        }
    }
}

// Pipelined form of the kernel above for the common case (cols % 8 == 0, 16-byte aligned operands).
// 8 rows per 320-thread block, 256-column tiles.  Wave 0 does nothing but walk (8 lanes for RMSNorm, 16 for LayerNorm)
// and raises its issue priority; the four loader waves fetch one 16-byte vector per thread per tile two tiles ahead,
// widen x and T(x*x) to f32 and park them in double-buffered LDS tiles; one barrier per tile.  The kernel runs at the
// speed of the walk.  A dependent v_add_f32 takes 4.9 cycles (2.0 ns) on this chip, but the walker also has to issue its
// own LDS reads, one per four values of an f32 tile, which brings a column to about 3 ns.  For f16 the tiles therefore
// hold the 16-bit values themselves (x, and T(x*x), which is an f16 value too): one LDS read per eight values, and the
// chain adds them with v_fma_mix_f32 (1.0 * f16 operand + running f32 sum: the same sum, the widening is part of the
// instruction).  bf16 has no such instruction and keeps the f32 tiles.
// KEEP (launches whose blocks are all resident at once, rows of at most NP_KEEP_MAX_COLS columns): the walk of every row
// of the tensor then ends at the same moment and nothing can hide what comes after it, so the output pass must be
// nothing but stores: each loader thread also parks the raw vectors it loaded in dynamic LDS, scale and bias are staged
// there once at the start, and after the statistics the block reads LDS, normalises and streams the result out,
// instead of fetching x a second time through a loop of dependent load / store pairs.
constexpr int NP_BLOCK = 320;
constexpr uint32_t NP_KEEP_MAX_COLS = 4096;
constexpr size_t NP_KEEP_BYTES_PER_TILE = 256 * 16 + 2 * 32 * 16;   // the block's x vectors, one scale and one bias vector per column group
typedef _Float16 np_h8 __attribute__((ext_vector_type(8)));
// run += the 32 f16 values packed in four vectors, left to right: each add is 1.0 * widen(f16) + run in one instruction
// with one rounding, which is the f32 sum of the widened values.  One asm statement for the whole run of adds: between
// separate statements the compiler, which cannot see into them, puts wait states that cost more than the adds.
#define NP_MIX_LO(N) "v_fma_mix_f32 %0, %" #N ", %17, %0 op_sel_hi:[1,0,0]\n"
#define NP_MIX_HI(N) "v_fma_mix_f32 %0, %" #N ", %17, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n"
#define NP_MIX(N) NP_MIX_LO(N) NP_MIX_HI(N)
__device__ __forceinline__ void np_add_f16x32(float& run, const v4u& a, const v4u& b, const v4u& c, const v4u& d) {
    const float one = 1.0f;
    asm(NP_MIX(1) NP_MIX(2) NP_MIX(3) NP_MIX(4) NP_MIX(5) NP_MIX(6) NP_MIX(7) NP_MIX(8) NP_MIX(9) NP_MIX(10) NP_MIX(11) NP_MIX(12)
        NP_MIX(13) NP_MIX(14) NP_MIX(15) NP_MIX(16)
        : "+v"(run)
        : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3]), "v"(c[0]), "v"(c[1]), "v"(c[2]), "v"(c[3]),
          "v"(d[0]), "v"(d[1]), "v"(d[2]), "v"(d[3]), "s"(one));
}
#undef NP_MIX
#undef NP_MIX_HI
#undef NP_MIX_LO
template <typename T, int KIND, bool KEEP>
__global__ void __launch_bounds__(NP_BLOCK) norm_pipe16_kernel(const T* __restrict__ x, const T* __restrict__ scale,
                                                               const T* __restrict__ bias, T* __restrict__ y, uint64_t rows, uint32_t cols,
                                                               float eps) {
    constexpr int RB = 8, TC = 256, PAD = 4, PAD16 = 8;
    constexpr int NSUM = (KIND == NORM_LAYER) ? 2 : 1;
    constexpr bool H16 = std::is_same<T, half_t>::value;                         // 16-bit tiles and the fma_mix chain
    // [.][0] = squares, [.][1] = values: f32, or the f16 bit patterns
    __shared__ __attribute__((aligned(16))) unsigned char tile_raw[H16 ? 2 * NSUM * RB * (TC + PAD16) * 2 : 2 * NSUM * RB * (TC + PAD) * 4];
    float (*tile)[NSUM][RB][TC + PAD] = reinterpret_cast<float (*)[NSUM][RB][TC + PAD]>(tile_raw);
    uint16_t (*tile16)[NSUM][RB][TC + PAD16] = reinterpret_cast<uint16_t (*)[NSUM][RB][TC + PAD16]>(tile_raw);
    __shared__ float sums[NSUM][RB];
    __shared__ T s_mu[RB], s_r[RB];
    extern __shared__ __attribute__((aligned(16))) v4u np_keep[];               // KEEP: [ntiles][256] x, [ntiles][32] scale, [ntiles][32] bias
    const uint64_t row0 = (uint64_t)blockIdx.x * RB;
    const uint32_t nrows = (rows - row0 < (uint64_t)RB) ? (uint32_t)(rows - row0) : (uint32_t)RB;
    const uint32_t ntiles = (cols + TC - 1) / TC;

    if (threadIdx.x < 64) {
        // ---------------------------------------------------------------- wave 0: the sequential sums
        __builtin_amdgcn_s_setprio(3);
        const uint32_t wrow = threadIdx.x % RB, wsum = (threadIdx.x / RB) % NSUM;   // lanes beyond NSUM*RB shadow and never publish
        const bool publish = (threadIdx.x < NSUM * RB) && (wrow < nrows);
        float run = 0.0f;
        if constexpr (H16) {
            // The barrier that says "tile t + 1 is in LDS" is taken before the last 32 adds of tile t, whose operands are in
            // registers by then (the loaders may overwrite tile t after it): the first LDS reads of the next tile are in
            // flight during those adds, so the chain never waits for LDS at a tile's start.
            __syncthreads();                                                    // tile 0 is in LDS
            v4u cur[4], nxt[4];
            {
                const v4u* first = reinterpret_cast<const v4u*>(tile16[0][wsum][wrow]);
#pragma unroll
                for (int k = 0; k < 4; k++) cur[k] = first[k];
            }
            for (uint32_t t = 0; t < ntiles; t++) {
                const v4u* trow16 = reinterpret_cast<const v4u*>(tile16[t & 1][wsum][wrow]);
                const v4u* trow16n = reinterpret_cast<const v4u*>(tile16[(t + 1) & 1][wsum][wrow]);
#pragma unroll
                for (int c = 0; c < TC / 32; c++) {
                    if (c + 1 < TC / 32) {
#pragma unroll
                        for (int k = 0; k < 4; k++) nxt[k] = trow16[(c + 1) * 4 + k];
                    } else if (t + 1 < ntiles) {
                        __syncthreads();                                        // tile t + 1 is in LDS
#pragma unroll
                        for (int k = 0; k < 4; k++) nxt[k] = trow16n[k];
                    }
                    np_add_f16x32(run, cur[0], cur[1], cur[2], cur[3]);
#pragma unroll
                    for (int k = 0; k < 4; k++) cur[k] = nxt[k];
                }
            }
        }
        for (uint32_t t = 0; !H16 && t < ntiles; t++) {
            __syncthreads();                                                    // tile t is in LDS
            // fixed trip count (tiles are zero padded): LDS reads of the next 32 values are issued before the 32 dependent
            // adds of the current ones
            const float4* trow = reinterpret_cast<const float4*>(tile[t & 1][wsum][wrow]);
            float4 cur[8], nxt[8];
#pragma unroll
            for (int k = 0; k < 8; k++) cur[k] = trow[k];
#pragma unroll
            for (int c = 0; c < TC / 32; c++) {
                if (c + 1 < TC / 32) {
#pragma unroll
                    for (int k = 0; k < 8; k++) nxt[k] = trow[(c + 1) * 8 + k];
                }
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    run += cur[k].x; run += cur[k].y; run += cur[k].z; run += cur[k].w;
                }
#pragma unroll
                for (int k = 0; k < 8; k++) cur[k] = nxt[k];
            }
        }
        if (publish) sums[wsum][wrow] = run;
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();                                                        // sums published
        if (threadIdx.x < nrows) {
            const RowStats<T> st = finish_stats<T, KIND>(KIND == NORM_LAYER ? sums[NSUM - 1][threadIdx.x] : 0.0f, sums[0][threadIdx.x],
                                                         cols, eps);
            s_mu[threadIdx.x] = st.mu;
            s_r[threadIdx.x] = st.r;
        }
        __syncthreads();                                                        // row statistics published
        return;
    }

    // -------------------------------------------------------------------- waves 1..4: loads, widening, second pass
    const uint32_t lt = threadIdx.x - 64;
    const uint32_t r = lt >> 5, cv = lt & 31;                                   // row, vector within the tile
    const bool rvalid = r < nrows;
    const T* xrow = x + (row0 + (rvalid ? r : 0)) * cols;
    v4u pre0 = {0, 0, 0, 0}, pre1 = {0, 0, 0, 0};
    v4u* keep_x = np_keep;
    v4u* keep_scale = np_keep + ntiles * 256;
    v4u* keep_bias = keep_scale + ntiles * 32;

    auto issue = [&](uint32_t t, v4u& dst) {
        const uint32_t col = t * TC + cv * 8;
        if (rvalid && t < ntiles && col < cols) dst = *reinterpret_cast<const v4u*>(xrow + col);
    };
    auto step = [&](uint32_t t, v4u& reg) {
        const uint32_t buf = t & 1;
        const uint32_t col = t * TC + cv * 8;
        if (H16 && rvalid) {
            v4u sqv = {0, 0, 0, 0}, xvv = {0, 0, 0, 0};                         // past the end of the row: +0.0 terms
            if (col < cols) {
                xvv = __builtin_bit_cast(v4u, reg);
                if (KEEP) keep_x[t * 256 + lt] = xvv;                           // read back by this same thread after the walk
                const np_h8 h = __builtin_bit_cast(np_h8, xvv);
                sqv = __builtin_bit_cast(v4u, h * h);                           // T(x*x): eight f16 products, each rounded once
            }
            *reinterpret_cast<v4u*>(&tile16[buf][0][r][cv * 8]) = sqv;
            if (KIND == NORM_LAYER) *reinterpret_cast<v4u*>(&tile16[buf][NSUM - 1][r][cv * 8]) = xvv;
        } else if (rvalid) {
            float sq[8], xv[8];
            if (col < cols) {
                Vec16<T> in;
                in.u = __builtin_bit_cast(v4u, reg);
                if (KEEP) keep_x[t * 256 + lt] = in.u;                          // read back by this same thread after the walk
#pragma unroll
                for (int q = 0; q < 8; q++) {
                    sq[q] = Ar<T>::widen(Ar<T>::mul(in.e[q], in.e[q]));
                    xv[q] = Ar<T>::widen(in.e[q]);
                }
            } else {
                // past the end of the row: +0.0 terms leave the running sums unchanged, so the walk needs no tail logic
#pragma unroll
                for (int q = 0; q < 8; q++) sq[q] = xv[q] = 0.0f;
            }
            float4* d0 = reinterpret_cast<float4*>(&tile[buf][0][r][cv * 8]);
            d0[0] = make_float4(sq[0], sq[1], sq[2], sq[3]);
            d0[1] = make_float4(sq[4], sq[5], sq[6], sq[7]);
            if (KIND == NORM_LAYER) {
                float4* d1 = reinterpret_cast<float4*>(&tile[buf][NSUM - 1][r][cv * 8]);
                d1[0] = make_float4(xv[0], xv[1], xv[2], xv[3]);
                d1[1] = make_float4(xv[4], xv[5], xv[6], xv[7]);
            }
        }
        issue(t + 2, reg);
        __syncthreads();
    };

    issue(0, pre0);
    issue(1, pre1);
    if (KEEP) {
        // scale and bias, once per block, in flight together with the first two tiles; the barriers of the walk make
        // them visible long before the output pass
        for (uint32_t c = lt; c < cols / 8; c += 256) {
            keep_scale[c] = reinterpret_cast<const v4u*>(scale)[c];
            if (KIND == NORM_LAYER && bias) keep_bias[c] = reinterpret_cast<const v4u*>(bias)[c];
        }
    }
    for (uint32_t t = 0; t < ntiles; t += 2) {
        step(t, pre0);
        if (t + 1 < ntiles) step(t + 1, pre1);
    }
    __syncthreads();                                                            // sums published (wave 0 finishes the stats)
    __syncthreads();                                                            // row statistics published
    if (!rvalid) return;
    RowStats<T> st;
    st.mu = s_mu[r];
    st.r = s_r[r];
    T* yrow = y + (row0 + r) * cols;
    const uint32_t cvec = cols / 8;
    if (KEEP) {
#pragma unroll 2
        for (uint32_t c = cv, t = 0; c < cvec; c += 32, t++) {
            Vec16<T> in, sc, bi, out;
            in.u = keep_x[t * 256 + lt];
            sc.u = keep_scale[c];
            if (KIND == NORM_LAYER && bias) bi.u = keep_bias[c];
#pragma unroll
            for (int q = 0; q < 8; q++) out.e[q] = norm_one<T, KIND>(in.e[q], st, sc.e[q], bi.e[q], bias != nullptr);
            st_stream(reinterpret_cast<v4u*>(yrow) + c, out.u);
        }
        return;
    }
    // four vectors of the row at a time, their loads issued together ([16384,4096] f16: 75.1 -> 70.4 us, RMSNorm 69.1 -> 64.0)
    constexpr int OB = 4;
    for (uint32_t c0 = cv; c0 < cvec; c0 += 32 * OB) {
        Vec16<T> in[OB], sc[OB], bi[OB];
#pragma unroll
        for (int k = 0; k < OB; k++) {
            const uint32_t c = c0 + 32 * k;
            if (c < cvec) {
                in[k].u = ld_stream(reinterpret_cast<const v4u*>(xrow) + c);
                sc[k].u = reinterpret_cast<const v4u*>(scale)[c];
                if (KIND == NORM_LAYER && bias) bi[k].u = reinterpret_cast<const v4u*>(bias)[c];
            }
        }
#pragma unroll
        for (int k = 0; k < OB; k++) {
            const uint32_t c = c0 + 32 * k;
            if (c < cvec) {
                Vec16<T> out;
#pragma unroll
                for (int q = 0; q < 8; q++) out.e[q] = norm_one<T, KIND>(in[k].e[q], st, sc[k].e[q], bi[k].e[q], bias != nullptr);
                st_stream(reinterpret_cast<v4u*>(yrow) + c, out.u);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------------------------
// GroupNorm.  x is [B, C, L] contiguous, so group (b, g) is one contiguous run of glen = (C/G)*L elements.
// stats kernel: grid (B*G, splits); block s of a group reduces elements [s*chunk, min((s+1)*chunk, glen)) to
//               (mean, M2, count) with a two-pass local variance (second pass re-reads the slice from cache).
// apply kernel: same grid; every block combines the group's partials (Chan et al.), then normalises its slice:
//               y = (x - mean) * rstd * w[c] + b[c], f32 arithmetic, rounded to T once.
// ------------------------------------------------------------------------------------------------------------------
// VE = elements per access: 16 / sizeof(T) on the vector path (slices, groups and base pointers are multiples of it), 1 otherwise
template <typename T, int VE>
__global__ void __launch_bounds__(BLOCK) gn_stats_kernel(const T* __restrict__ x, float* __restrict__ part, uint32_t glen,
                                                         uint32_t chunk, uint32_t splits) {
    __shared__ float red[WAVES];
    __shared__ float bc;
    const uint32_t s = blockIdx.y, grp = blockIdx.x;
    const T* xs = x + (uint64_t)grp * glen;
    const uint32_t c0 = s * chunk;
    const uint32_t c1 = (c0 + chunk < glen) ? c0 + chunk : glen;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    float acc = 0.0f;
    for (uint32_t i = c0 + threadIdx.x * VE; i < c1; i += BLOCK * VE) {
        if (VE > 1) {
            Vec16<T> v;
            v.u = *reinterpret_cast<const v4u*>(xs + i);
#pragma unroll
            for (int q = 0; q < VE; q++) acc += Ar<T>::widen(v.e[q]);
        } else {
            acc += Ar<T>::widen(xs[i]);
        }
    }
    acc = wave_sum(acc);
    if (lane == 0) red[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.0f;
        for (int w = 0; w < WAVES; w++) t += red[w];
        bc = t / (float)(c1 - c0);
    }
    __syncthreads();
    const float mean = bc;
    float m2 = 0.0f;
    for (uint32_t i = c0 + threadIdx.x * VE; i < c1; i += BLOCK * VE) {     // second pass: the slice is in cache
        if (VE > 1) {
            Vec16<T> v;
            v.u = *reinterpret_cast<const v4u*>(xs + i);
#pragma unroll
            for (int q = 0; q < VE; q++) {
                const float d = Ar<T>::widen(v.e[q]) - mean;
                m2 += d * d;
            }
        } else {
            const float d = Ar<T>::widen(xs[i]) - mean;
            m2 += d * d;
        }
    }
    m2 = wave_sum(m2);
    __syncthreads();
    if (lane == 0) red[wave] = m2;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.0f;
        for (int w = 0; w < WAVES; w++) t += red[w];
        float* o = part + ((uint64_t)grp * splits + s) * 3;
        o[0] = mean;
        o[1] = t;
        o[2] = (float)(c1 - c0);
    }
}

// The same partials from a slice that the block's registers hold (NV vectors a thread): the slice is read once, with all
// its loads in flight together, and the second pass runs on registers ([16,256,4096] f32, slices of 32 KiB: 49.7 -> 33.8 us for the two launches).
template <typename T, int NV>
__global__ void __launch_bounds__(BLOCK) gn_stats_reg_kernel(const T* __restrict__ x, float* __restrict__ part, uint32_t glen,
                                                             uint32_t chunk, uint32_t splits) {
    constexpr int VE = 16 / sizeof(T);
    __shared__ float red[WAVES];
    const uint32_t s = blockIdx.y, grp = blockIdx.x;
    const uint32_t c0 = s * chunk;
    const uint32_t c1 = (c0 + chunk < glen) ? c0 + chunk : glen;
    const v4u* xs = reinterpret_cast<const v4u*>(x + (uint64_t)grp * glen + c0);
    const uint32_t nvec = (c1 - c0) / VE;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    Vec16<T> v[NV];
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = threadIdx.x + k * BLOCK;
        v[k].u = v4u{0u, 0u, 0u, 0u};
        if (i < nvec) v[k].u = xs[i];
    }
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
#pragma unroll
        for (int q = 0; q < VE; q++) acc += Ar<T>::widen(v[k].e[q]);             // vectors past the slice hold zeros
    }
    acc = wave_sum(acc);
    if (lane == 0) red[wave] = acc;
    __syncthreads();
    float t = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; w++) t += red[w];
    const float mean = t / (float)(c1 - c0);
    float m2 = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
        if (threadIdx.x + k * BLOCK < nvec) {
#pragma unroll
            for (int q = 0; q < VE; q++) {
                const float d = Ar<T>::widen(v[k].e[q]) - mean;
                m2 += d * d;
            }
        }
    }
    m2 = wave_sum(m2);
    __syncthreads();
    if (lane == 0) red[wave] = m2;
    __syncthreads();
    if (threadIdx.x == 0) {
        float u = 0.0f;
        for (int w = 0; w < WAVES; w++) u += red[w];
        float* o = part + ((uint64_t)grp * splits + s) * 3;
        o[0] = mean;
        o[1] = u;
        o[2] = (float)(c1 - c0);
    }
}

// y = (x - mean) * rstd * w[c] + b[c] for the VE elements of one vector that starts at element e0 of its group, whose first
// channel is cbase.  With L a multiple of VE the vector lies in one channel; otherwise the channel is stepped element by
// element (a vector of [.., 1500] f16 rows crosses into the next channel, with L < VE into several).
template <typename T>
__device__ __forceinline__ v4u gn_affine_vec(const Vec16<T>& v, uint32_t e0, uint32_t cbase, FastDiv L, const T* __restrict__ scale,
                                             const T* __restrict__ bias, float mean, float rstd) {
    constexpr int VE = 16 / sizeof(T);
    Vec16<T> o;
    const uint32_t ch = fd_div(e0, L);
    uint32_t c = cbase + ch;
    if (L.d % VE == 0) {
        const float w = scale ? Ar<T>::widen(scale[c]) : 1.0f;
        const float b = bias ? Ar<T>::widen(bias[c]) : 0.0f;
#pragma unroll
        for (int q = 0; q < VE; q++) {
            const float t = (Ar<T>::widen(v.e[q]) - mean) * rstd;
            o.e[q] = Ar<T>::conv(t * w + b);
        }
    } else {
        uint32_t r = e0 - ch * L.d;
#pragma unroll
        for (int q = 0; q < VE; q++) {
            const float w = scale ? Ar<T>::widen(scale[c]) : 1.0f;
            const float b = bias ? Ar<T>::widen(bias[c]) : 0.0f;
            const float t = (Ar<T>::widen(v.e[q]) - mean) * rstd;
            o.e[q] = Ar<T>::conv(t * w + b);
            if (++r == L.d) {
                r = 0;
                c++;
            }
        }
    }
    return o.u;
}

// Combines the partials of one group (Chan et al.) in double, by the first wave of the block: lane k takes partial k (the
// launcher keeps splits <= 64 here), then a tree over the wave, in the same order in every block of the group.
__device__ __forceinline__ void gn_combine_wave(const float* __restrict__ p, uint32_t splits, float eps, float& s_mean, float& s_rstd) {
    if (threadIdx.x >= WAVE) return;
    double n = 0.0, mean = 0.0, m2 = 0.0;
    if (threadIdx.x < splits) {
        mean = (double)p[3 * threadIdx.x];
        m2 = (double)p[3 * threadIdx.x + 1];
        n = (double)p[3 * threadIdx.x + 2];
    }
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        const double nb = __shfl_down(n, off), mb = __shfl_down(mean, off), m2b = __shfl_down(m2, off);
        if (nb != 0.0) {
            const double nt = n + nb;
            const double delta = mb - mean;
            mean += delta * (nb / nt);
            m2 += m2b + delta * delta * (n * nb / nt);
            n = nt;
        }
    }
    if (threadIdx.x == 0) {
        s_mean = (float)mean;
        s_rstd = (float)(1.0 / sqrt(m2 / n + (double)eps));
    }
}

template <typename T, int VE>
__global__ void __launch_bounds__(BLOCK) gn_apply_kernel(const T* __restrict__ x, const T* __restrict__ scale,
                                                         const T* __restrict__ bias, T* __restrict__ y,
                                                         const float* __restrict__ part, uint32_t glen, uint32_t chunk, uint32_t splits,
                                                         uint32_t cpg, uint32_t groups, FastDiv L, float eps) {
    __shared__ float s_mean, s_rstd;
    const uint32_t s = blockIdx.y, grp = blockIdx.x;
    gn_combine_wave(part + (uint64_t)grp * splits * 3, splits, eps, s_mean, s_rstd);
    __syncthreads();
    const float meanf = s_mean, rstd = s_rstd;
    const uint32_t g = grp % groups;
    const T* xs = x + (uint64_t)grp * glen;
    T* ys = y + (uint64_t)grp * glen;
    const uint32_t c0 = s * chunk;
    const uint32_t c1 = (c0 + chunk < glen) ? c0 + chunk : glen;
    for (uint32_t i = c0 + threadIdx.x * VE; i < c1; i += BLOCK * VE) {
        if (VE > 1) {
            Vec16<T> v;
            v.u = *reinterpret_cast<const v4u*>(xs + i);
            st_stream(reinterpret_cast<v4u*>(ys + i), gn_affine_vec<T>(v, i, g * cpg, L, scale, bias, meanf, rstd));
        } else {
            const uint32_t c = g * cpg + fd_div(i, L);
            const float w = scale ? Ar<T>::widen(scale[c]) : 1.0f;
            const float b = bias ? Ar<T>::widen(bias[c]) : 0.0f;
            const float t = (Ar<T>::widen(xs[i]) - meanf) * rstd;
            ys[i] = Ar<T>::conv(t * w + b);
        }
    }
}

// gn_apply_kernel for slices of up to NV vectors a thread: all loads of the slice are in flight before the first is used
template <typename T, int NV>
__global__ void __launch_bounds__(BLOCK) gn_apply_reg_kernel(const T* __restrict__ x, const T* __restrict__ scale,
                                                             const T* __restrict__ bias, T* __restrict__ y,
                                                             const float* __restrict__ part, uint32_t glen, uint32_t chunk,
                                                             uint32_t splits, uint32_t cpg, uint32_t groups, FastDiv L, float eps) {
    constexpr int VE = 16 / sizeof(T);
    __shared__ float s_mean, s_rstd;
    const uint32_t s = blockIdx.y, grp = blockIdx.x;
    const uint32_t c0 = s * chunk;
    const uint32_t c1 = (c0 + chunk < glen) ? c0 + chunk : glen;
    const v4u* xs = reinterpret_cast<const v4u*>(x + (uint64_t)grp * glen + c0);
    v4u* ys = reinterpret_cast<v4u*>(y + (uint64_t)grp * glen + c0);
    const uint32_t nvec = (c1 - c0) / VE;
    Vec16<T> v[NV];
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = threadIdx.x + k * BLOCK;
        v[k].u = v4u{0u, 0u, 0u, 0u};
        if (i < nvec) v[k].u = ld_stream(xs + i);
    }
    gn_combine_wave(part + (uint64_t)grp * splits * 3, splits, eps, s_mean, s_rstd);
    __syncthreads();
    const float meanf = s_mean, rstd = s_rstd;
    const uint32_t g = grp % groups;
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = threadIdx.x + k * BLOCK;
        if (i < nvec) {
            st_stream(ys + i, gn_affine_vec<T>(v[k], c0 + i * VE, g * cpg, L, scale, bias, meanf, rstd));
        }
    }
}

template <typename T, int KIND, bool SPAN>
int launch_norm_wave(rt_device* dev, const void* x, const void* scale, const void* bias, void* y, uint64_t rows, uint32_t cols, float eps);

template <typename T, int KIND>
int launch_norm(rt_device* dev, const void* x, const void* scale, const void* bias, void* y, uint64_t rows, uint32_t cols, float eps) {
    constexpr int VE = 16 / sizeof(T);
    const bool io_aligned = rt_aligned(x, 16) && rt_aligned(y, 16);
    constexpr uint32_t MAX_VEC = NORM_WIDE_BLOCK * 16;       // 65536 f32 columns
    if (io_aligned && cols % VE == 0 && rt_aligned(scale, 16) && (!bias || rt_aligned(bias, 16)) && cols / VE <= MAX_VEC)
        return launch_norm_wave<T, KIND, false>(dev, x, scale, bias, y, rows, cols, eps);
    // rows that are not whole vectors (or scale / bias off their alignment): over the aligned vectors that cover each row
    if (io_aligned && (cols + 2 * VE - 2) / VE <= MAX_VEC)
        return launch_norm_wave<T, KIND, true>(dev, x, scale, bias, y, rows, cols, eps);
    RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "norm: too many rows");
    hipLaunchKernelGGL((norm_generic_kernel<T, KIND>), dim3((unsigned)rows), dim3(BLOCK), 0, dev->stream, (const T*)x, (const T*)scale,
                       (const T*)bias, (T*)y, rows, cols, eps);
    RT_CHECK_LAUNCH("norm_generic_kernel");
    return RT_OK;
}

template <typename T, int KIND, bool SPAN>
int launch_norm_wave(rt_device* dev, const void* x, const void* scale, const void* bias, void* y, uint64_t rows, uint32_t cols, float eps) {
    constexpr int VE = 16 / sizeof(T);
    const uint32_t nvec = SPAN ? (cols + 2 * VE - 2) / VE : cols / VE;       // SPAN: the most vectors a row can touch
    if (nvec <= 32) {
        // rows of at most 32 vectors: a group of 2..32 lanes per row (one vector each), so that a wave carries 2..32 rows
        // and as many bytes as with long rows
        const uint32_t lanes = nvec <= 2 ? 2 : nvec <= 4 ? 4 : nvec <= 8 ? 8 : nvec <= 16 ? 16 : 32;
        const uint64_t blocks = (rows + BLOCK / lanes - 1) / (BLOCK / lanes);
        RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "norm: too many rows");
        const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_NARROW(L) hipLaunchKernelGGL((norm_wave_kernel<T, 1, KIND, L, SPAN>), grid, block, 0, dev->stream, (const T*)x, (const T*)scale, (const T*)bias, (T*)y, rows, cols, eps)
        if (lanes == 2) RT_NARROW(2);
        else if (lanes == 4) RT_NARROW(4);
        else if (lanes == 8) RT_NARROW(8);
        else if (lanes == 16) RT_NARROW(16);
        else RT_NARROW(32);
#undef RT_NARROW
        RT_CHECK_LAUNCH("norm_wave_kernel");
        return RT_OK;
    }
    if (nvec <= (uint32_t)(WAVE * 8)) {
        const uint32_t nv = (nvec + WAVE - 1) / WAVE;
        const uint64_t blocks = (rows + WAVES - 1) / WAVES;
        RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "norm: too many rows");
        const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_NORM(NVC)                                                                                                                 \
    hipLaunchKernelGGL((norm_wave_kernel<T, NVC, KIND, WAVE, SPAN>), grid, block, 0, dev->stream, (const T*)x, (const T*)scale, (const T*)bias, \
                       (T*)y, rows, cols, eps)
        if (nv <= 1) RT_NORM(1);
        else if (nv <= 2) RT_NORM(2);
        else if (nv <= 3) RT_NORM(3);
        else if (nv <= 4) RT_NORM(4);
        else if (nv <= 5) RT_NORM(5);
        else if (nv <= 6) RT_NORM(6);
        else RT_NORM(8);
#undef RT_NORM
        RT_CHECK_LAUNCH("norm_wave_kernel");
        return RT_OK;
    }
    RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "norm: too many rows");
    if (nvec <= (uint32_t)(BLOCK * 8)) {                     // longer rows: the 256 threads of a block share one row
        const uint32_t nv = (nvec + BLOCK - 1) / BLOCK;
        const dim3 grid((unsigned)rows), block(BLOCK);
#define RT_NORM(NVC)                                                                                                                  \
    hipLaunchKernelGGL((norm_wave_kernel<T, NVC, KIND, BLOCK, SPAN>), grid, block, 0, dev->stream, (const T*)x, (const T*)scale, (const T*)bias, \
                       (T*)y, rows, cols, eps)
        if (nv <= 3) RT_NORM(3);
        else if (nv <= 4) RT_NORM(4);
        else if (nv <= 6) RT_NORM(6);
        else RT_NORM(8);
#undef RT_NORM
    } else {                                                 // up to 65536 f32 columns (the caller has checked): 1024 threads share one row
        const uint32_t nv = (nvec + NORM_WIDE_BLOCK - 1) / NORM_WIDE_BLOCK;
        const dim3 grid((unsigned)rows), block(NORM_WIDE_BLOCK);
#define RT_NORM(NVC)                                                                                                                  \
    hipLaunchKernelGGL((norm_wave_kernel<T, NVC, KIND, NORM_WIDE_BLOCK, SPAN>), grid, block, 0, dev->stream, (const T*)x, (const T*)scale, \
                       (const T*)bias, (T*)y, rows, cols, eps)
        if (nv <= 4) RT_NORM(4);
        else if (nv <= 8) RT_NORM(8);
        else if (nv <= 13) RT_NORM(13);
        else RT_NORM(16);
#undef RT_NORM
    }
    RT_CHECK_LAUNCH("norm_wave_kernel");
    return RT_OK;
}

// 16-bit reference arithmetic, many rows of at most 128 columns (whole aligned vectors): one lane per row.  A block's
// 256 rows are one contiguous run that passes through LDS with coalesced 16-byte accesses (row pitch 16 bytes more than
// the row, so neighbouring lanes' LDS accesses fall into different banks); the sequential f32 sums are short chains
// inside the lane.  (The tile walker above carries 8 rows per block however short they are: a million rows of 8 columns
// took it 479 us.)
template <typename T, int KIND, int NV>
__global__ void __launch_bounds__(BLOCK) norm16_lane_kernel(const T* x, const T* __restrict__ scale, const T* __restrict__ bias, T* y,
                                                            uint64_t rows, float eps) {
    __shared__ v4u stage[BLOCK * (NV + 1)];
    const uint64_t row0 = (uint64_t)blockIdx.x * BLOCK;
    const uint32_t nrows = rows - row0 < (uint64_t)BLOCK ? (uint32_t)(rows - row0) : (uint32_t)BLOCK;
    const v4u* xb = reinterpret_cast<const v4u*>(x) + row0 * NV;
    v4u* yb = reinterpret_cast<v4u*>(y) + row0 * NV;
    const uint32_t nvec = nrows * NV;
    for (uint32_t i = threadIdx.x; i < nvec; i += BLOCK) stage[(i / NV) * (NV + 1) + i % NV] = ld_stream(xb + i);
    __syncthreads();
    if (threadIdx.x < nrows) {
        v4u* mine = stage + threadIdx.x * (NV + 1);
        Vec16<T> v[NV];
#pragma unroll
        for (int k = 0; k < NV; k++) v[k].u = mine[k];
        float sx = 0.0f, sq = 0.0f;                          // the reference's order: element 0 first
#pragma unroll
        for (int k = 0; k < NV; k++)
#pragma unroll
            for (int q = 0; q < 8; q++) {
                sq += Ar<T>::widen(Ar<T>::mul(v[k].e[q], v[k].e[q]));
                if (KIND == NORM_LAYER) sx += Ar<T>::widen(v[k].e[q]);
            }
        const RowStats<T> st = finish_stats<T, KIND>(sx, sq, NV * 8, eps);
#pragma unroll
        for (int k = 0; k < NV; k++) {
            Vec16<T> sc, bi;
            sc.u = reinterpret_cast<const v4u*>(scale)[k];
            if (KIND == NORM_LAYER && bias) bi.u = reinterpret_cast<const v4u*>(bias)[k];
#pragma unroll
            for (int q = 0; q < 8; q++) v[k].e[q] = norm_one<T, KIND>(v[k].e[q], st, sc.e[q], bi.e[q], bias != nullptr);
            mine[k] = v[k].u;
        }
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < nvec; i += BLOCK) st_stream(yb + i, stage[(i / NV) * (NV + 1) + i % NV]);
}

// ------------------------------------------------------------------------------------------------------------------
// RMSNorm in the 16-bit types, one wave per row, with the reference's row sum replayed exactly but not sequentially.
//
// The reference adds T(x*x) left to right in f32 (cpu/norm.rs:72-89, half's Sum): s <- fl(s + a_j), a_j >= 0.  While s
// stays inside one binade, [2^e, 2^(e+1)), s is 2^e + k * ulp with an integer k, and what one add does to k depends on s
// only through the parity of k (round to nearest even: the parity decides ties).  A run of adds that stays inside the
// binade is therefore a function k -> k + c[k & 1] of two constants, and such functions compose.  Both constants come
// out of the floating-point adder itself: the run is added up twice, from 2^e and from 2^e + ulp, and c[p] is the
// distance the p-th sum has moved, read off the bit patterns.
//
// Lane i of the wave owns the contiguous run of 8 * V elements i * 8V .. (the row is turned through LDS so that it does).
//   1. approximate sums of the runs and their prefix over the lanes say in which binade each run starts and ends;
//   2. a lane whose run starts and ends in one binade, with a margin for what the approximation can be off by, is
//      `clean`: its two sums give its pair (c[0], c[1]);
//   3. a segmented scan composes the pairs of neighbouring clean lanes;
//   4. the lanes that are not clean (the first, those in which the sum crosses a power of two: about seven per row,
//      and any lane the margins do not clear) are taken in order: the composed function of the clean stretch before
//      such a lane is applied to the running value t, then every lane adds its own run to t left to right and the
//      result of the lane in question is kept.
// Nothing rests on the approximation: before a pair is applied, t must lie in the binade the pair was made for, and
// the result must still lie in it; if either fails the row is done again with every lane treated as not clean, which
// is the plain left-to-right sum, 64 runs one after the other.  bf16 takes the same path with widened operands.
// ------------------------------------------------------------------------------------------------------------------
constexpr int RP_BLOCK = 256;                                // four rows per block; the waves never meet
template <typename T> struct RpChain;
template <> struct RpChain<half_t> {
    // a <- fl(a + h) and b <- fl(b + h) for the eight halves of a vector, left to right: 1.0 * widen(h) + sum in one
    // instruction with one rounding
#define RP_MIX2(N)                                                              \
    "v_fma_mix_f32 %0, %" #N ", %6, %0 op_sel_hi:[1,0,0]\n"                      \
    "v_fma_mix_f32 %1, %" #N ", %6, %1 op_sel_hi:[1,0,0]\n"                      \
    "v_fma_mix_f32 %0, %" #N ", %6, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n"       \
    "v_fma_mix_f32 %1, %" #N ", %6, %1 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n"
    static __device__ __forceinline__ void add2(float& a, float& b, const v4u& v) {
        const float one = 1.0f;
        asm(RP_MIX2(2) RP_MIX2(3) RP_MIX2(4) RP_MIX2(5) : "+v"(a), "+v"(b) : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "s"(one));
    }
#undef RP_MIX2
#define RP_MIX1(N)                                                              \
    "v_fma_mix_f32 %0, %" #N ", %5, %0 op_sel_hi:[1,0,0]\n"                      \
    "v_fma_mix_f32 %0, %" #N ", %5, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n"
    static __device__ __forceinline__ void add1(float& a, const v4u& v) {
        const float one = 1.0f;
        asm(RP_MIX1(1) RP_MIX1(2) RP_MIX1(3) RP_MIX1(4) : "+v"(a) : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "s"(one));
    }
#undef RP_MIX1
    // the sum of the eight halves added to acc, in any order and with any rounding: only the binade is taken from it
    // (v_dot2_f32_f16 with a pair of ones; written as instructions: through the builtin this compiler fed all four the
    // vector's first word)
    static __device__ __forceinline__ float rough(const v4u& v, float acc) {
        const uint32_t ones = 0x3c003c00u;
        asm("v_dot2_f32_f16 %0, %1, %5, %0\n"
            "v_dot2_f32_f16 %0, %2, %5, %0\n"
            "v_dot2_f32_f16 %0, %3, %5, %0\n"
            "v_dot2_f32_f16 %0, %4, %5, %0\n"
            : "+v"(acc)
            : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(ones));
        return acc;
    }
    static __device__ __forceinline__ v4u square(const v4u& x) {                 // T(x*x): eight f16 products, each rounded once
        const np_h8 h = __builtin_bit_cast(np_h8, x);
        return __builtin_bit_cast(v4u, h * h);
    }
};
template <> struct RpChain<bf16_t> {
    static __device__ __forceinline__ void add2(float& a, float& b, const v4u& v) {
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float lo = u2f(v[w] << 16), hi = u2f(v[w] & 0xffff0000u);
            a += lo; b += lo; a += hi; b += hi;
        }
    }
    static __device__ __forceinline__ void add1(float& a, const v4u& v) {
#pragma unroll
        for (int w = 0; w < 4; w++) {
            a += u2f(v[w] << 16);
            a += u2f(v[w] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ float rough(const v4u& v, float acc) {
#pragma unroll
        for (int w = 0; w < 4; w++) acc += u2f(v[w] << 16) + u2f(v[w] & 0xffff0000u);
        return acc;
    }
    static __device__ __forceinline__ v4u square(const v4u& x) {
        Vec16<bf16_t> in, out;
        in.u = x;
#pragma unroll
        for (int q = 0; q < 8; q++) out.e[q] = Ar<bf16_t>::mul(in.e[q], in.e[q]);
        return out.u;
    }
};

template <typename T, int V>
__global__ void __launch_bounds__(RP_BLOCK) rms16_par_kernel(const T* __restrict__ x, const T* __restrict__ scale, T* __restrict__ y, uint64_t rows,
                                                             uint32_t cols, float eps) {
    typedef RpChain<T> C;
    extern __shared__ __attribute__((aligned(16))) v4u rp_lds[];             // [4 waves][V * 64] vectors of squares
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint64_t first = (uint64_t)blockIdx.x * (RP_BLOCK / 64) + wave, stride = (uint64_t)gridDim.x * (RP_BLOCK / 64);
    if (first >= rows) return;                                               // a whole wave; the block never synchronises
    v4u* mine = rp_lds + wave * (V * 64);
    const uint32_t nvec = cols / 8;
    // the row as it lies in memory: vector j * 64 + lane (zeros past its end: +0 terms change no sum).  A wave takes rows
    // first, first + stride, ...; the loads of the next one are in flight while it works on this one (past the last
    // row they fetch the last row once more, so that no branch stands between the loads and what waits for them)
    auto fetch = [&](uint64_t r, v4u (&dst)[V]) {
        const v4u* src = reinterpret_cast<const v4u*>(x + r * cols);
#pragma unroll
        for (int j = 0; j < V; j++) {
            const uint32_t i = j * 64 + lane;
            dst[j] = v4u{0, 0, 0, 0};
            if (i < nvec) dst[j] = ld_stream(src + i);
        }
    };
    v4u ahead[V];
    fetch(first, ahead);
    for (uint64_t row = first; row < rows; row += stride) {
    v4u xr[V];
#pragma unroll
    for (int j = 0; j < V; j++) xr[j] = ahead[j];
    fetch(row + stride < rows ? row + stride : rows - 1, ahead);
    v4u* yrow = reinterpret_cast<v4u*>(y + row * cols);
#pragma unroll
    for (int j = 0; j < V; j++) mine[j * 64 + lane] = C::square(xr[j]);
    // turned: lane i holds the run of vectors i * V .. i * V + V - 1.  The wave wrote them itself and LDS keeps a wave's
    // order, but other lanes wrote what this lane reads: the fence keeps the compiler from moving a read above a write
    // that, seen from one lane alone, goes to another address.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    v4u run[V];
#pragma unroll
    for (int v = 0; v < V; v++) run[v] = mine[lane * V + v];

    // 1. approximate sum of the run, inclusive prefix over the lanes
    float rough = 0.0f;
#pragma unroll
    for (int v = 0; v < V; v++) rough = C::rough(run[v], rough);
    float upto = rough;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float t = __shfl_up(upto, o, 64);
        if (lane >= (uint32_t)o) upto += t;
    }
    float before = __shfl_up(upto, 1, 64);
    if (lane == 0) before = 0.0f;
    // 2. clean: the run starts and ends in the binade of `before`, even if both figures are off by 2^-10 of themselves
    const uint32_t e = (f2u(before) >> 23) & 0xffu;
    const uint32_t base = e << 23;                                           // bit pattern of 2^e
    bool clean = lane != 0 && e >= 1 && e < 254 && ((f2u(before * (1.0f - 0x1p-10f)) >> 23) & 0xffu) == e &&
                 ((f2u(upto * (1.0f + 0x1p-10f)) >> 23) & 0xffu) == e;
    float s0 = u2f(base), s1 = u2f(base + 1);
#pragma unroll
    for (int v = 0; v < V; v++) C::add2(s0, s1, run[v]);
    uint32_t c0 = f2u(s0) - base, c1 = f2u(s1) - (base + 1);
    clean = clean && c0 < (1u << 23) && c1 + 1 < (1u << 23);                 // both sums stayed in the binade
    // the pairs of a stretch of clean lanes are composed as counts of one and the same ulp: a clean lane behind a clean
    // lane of another binade (which the margins make all but impossible) starts over as a lane that is not clean
    {
        const uint32_t pbase = __shfl_up(base, 1, 64);
        const uint32_t pclean = __shfl_up((uint32_t)clean, 1, 64);
        if (lane != 0 && pclean && pbase != base) clean = false;
    }
    if (!clean) c0 = c1 = 0;

    // 3. segmented scan: (c0, c1) of lane i becomes the composition of the clean lanes from the start of its stretch up to
    // i; a lane that is not clean, and the lane behind one, start a stretch.  left then right: p -> l[p] + r[(p + l[p]) & 1]
    const uint64_t dirty_mask = __builtin_amdgcn_ballot_w64(!clean);
    uint32_t head = (uint32_t)((dirty_mask >> lane) & 1u) | (lane ? (uint32_t)((dirty_mask >> (lane - 1)) & 1u) : 1u);
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t l0 = __shfl_up(c0, o, 64), l1 = __shfl_up(c1, o, 64), lh = __shfl_up(head, o, 64);
        if (lane >= (uint32_t)o && !head) {
            const uint32_t n0 = l0 + ((l0 & 1u) ? c1 : c0);
            const uint32_t n1 = l1 + (((l1 + 1u) & 1u) ? c1 : c0);
            c0 = n0;
            c1 = n1;
            head = lh;
        }
    }

    // 4. the lanes that are not clean, in order, with the clean stretches between them
    uint32_t tb = 0;                                                         // bit pattern of the running sum, the same in every lane
    uint64_t todo = dirty_mask;
    bool redo = false;
    for (;;) {
        int prev = -1;
        bool failed = false;
        // applies the composed pair of lane `last` (the end of a clean stretch) to the running sum
        auto stretch = [&](int last) {
            const uint32_t f0 = __builtin_amdgcn_readlane(c0, last), f1 = __builtin_amdgcn_readlane(c1, last);
            const uint32_t eb = __builtin_amdgcn_readlane(base, last);
            const uint32_t k = tb - eb;                                      // t = 2^e + k ulp, if t lies in that binade
            const uint32_t k2 = k + ((k & 1u) ? f1 : f0);
            if ((tb & 0x7f800000u) != eb || k2 >= (1u << 23)) failed = true;
            tb = eb + k2;
        };
        while (todo) {
            const int d = __builtin_ctzll(todo);
            todo &= todo - 1;
            if (!redo && d - 1 > prev) stretch(d - 1);
            float t = u2f(tb);
#pragma unroll
            for (int v = 0; v < V; v++) C::add1(t, run[v]);
            tb = __builtin_amdgcn_readlane(f2u(t), d);
            prev = d;
        }
        if (!redo && prev < 63) stretch(63);
        if (!failed || redo) break;
        redo = true;                                                         // the plain sum: every lane's run, one after the other
        todo = ~0ull;
        tb = 0;
    }

    const RowStats<T> st = finish_stats<T, NORM_RMS>(0.0f, u2f(tb), cols, eps);
#pragma unroll
    for (int j = 0; j < V; j++) {
        const uint32_t i = j * 64 + lane;
        if (i < nvec) {
            Vec16<T> in, sc, out;
            in.u = xr[j];
            sc.u = reinterpret_cast<const v4u*>(scale)[i];
#pragma unroll
            for (int q = 0; q < 8; q++) out.e[q] = norm_one<T, NORM_RMS>(in.e[q], st, sc.e[q], sc.e[q], false);
            st_stream(yrow + i, out.u);
        }
    }
    // the next row's squares go to the same LDS buffer: every lane has read its run by now (the run is in registers)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

template <typename T>
int launch_rms16_par(rt_device* dev, const void* x, const void* scale, void* y, uint64_t rows, uint32_t cols, float eps) {
    // as many blocks as the chip holds at one time (what the runtime says for the instantiation's registers and LDS,
    // asked once per device), each wave taking every grid-th row
    const uint32_t v = (cols + 511) / 512;
    constexpr int TI = std::is_same<T, half_t>::value ? 0 : 1;
    uint64_t blocks = (rows + RP_BLOCK / 64 - 1) / (RP_BLOCK / 64);
#define RT_RP(VC)                                                                                                                    \
    case VC:                                                                                                                         \
        if (!dev->rp_resident[TI][VC]) {                                                                                             \
            int per_cu = 0;                                                                                                          \
            RT_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, rms16_par_kernel<T, VC>, RP_BLOCK,                          \
                                                                (size_t)(RP_BLOCK / 64) * VC * 64 * 16));                            \
            dev->rp_resident[TI][VC] = (uint16_t)(per_cu < 1 ? 1 : per_cu);                                                          \
        }                                                                                                                            \
        if (blocks > (uint64_t)dev->rp_resident[TI][VC] * dev->num_cus) blocks = (uint64_t)dev->rp_resident[TI][VC] * dev->num_cus;  \
        hipLaunchKernelGGL((rms16_par_kernel<T, VC>), dim3((unsigned)blocks), dim3(RP_BLOCK), (size_t)(RP_BLOCK / 64) * VC * 64 * 16, \
                           dev->stream, (const T*)x, (const T*)scale, (T*)y, rows, cols, eps);                                       \
        break
    switch (v) {
        RT_RP(1); RT_RP(2); RT_RP(3); RT_RP(4); RT_RP(5); RT_RP(6); RT_RP(7); RT_RP(8);
        default: return rt_fail(RT_ERR_ARG, "norm: internal: %u columns in the wave-per-row RMSNorm", cols);
    }
#undef RT_RP
    RT_CHECK_LAUNCH("rms16_par_kernel");
    return RT_OK;
}

template <typename T, int KIND>
int launch_norm16_lane(rt_device* dev, const void* x, const void* scale, const void* bias, void* y, uint64_t rows, uint32_t cols, float eps) {
    const uint64_t blocks = (rows + BLOCK - 1) / BLOCK;
    RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "norm: too many rows");
#define RT_LANE(NV)                                                                                                              \
    case NV:                                                                                                                     \
        hipLaunchKernelGGL((norm16_lane_kernel<T, KIND, NV>), dim3((unsigned)blocks), dim3(BLOCK), 0, dev->stream, (const T*)x, \
                           (const T*)scale, (const T*)bias, (T*)y, rows, eps);                                                   \
        break
    switch (cols / 8) {
        RT_LANE(1); RT_LANE(2); RT_LANE(3); RT_LANE(4); RT_LANE(5); RT_LANE(6); RT_LANE(7); RT_LANE(8);
        RT_LANE(9); RT_LANE(10); RT_LANE(11); RT_LANE(12); RT_LANE(13); RT_LANE(14); RT_LANE(15); RT_LANE(16);
        default: return rt_fail(RT_ERR_ARG, "norm: internal: %u columns in the one-lane-per-row kernel", cols);
    }
#undef RT_LANE
    RT_CHECK_LAUNCH("norm16_lane_kernel");
    return RT_OK;
}

template <typename T, int KIND, int RB>
int launch_norm16_rb(rt_device* dev, const void* x, const void* scale, const void* bias, void* y, uint64_t rows, uint32_t cols, float eps) {
    const uint64_t blocks = (rows + RB - 1) / RB;
    RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "norm: too many rows");
    const bool vec_ok = (cols % 8 == 0) && rt_aligned(x, 16) && rt_aligned(y, 16) && rt_aligned(scale, 16) && (!bias || rt_aligned(bias, 16));
    if (vec_ok) {
        hipLaunchKernelGGL((norm_seq16_kernel<T, RB, KIND, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, dev->stream, (const T*)x,
                           (const T*)scale, (const T*)bias, (T*)y, rows, cols, eps);
    } else {
        hipLaunchKernelGGL((norm_seq16_kernel<T, RB, KIND, false>), dim3((unsigned)blocks), dim3(BLOCK), 0, dev->stream, (const T*)x,
                           (const T*)scale, (const T*)bias, (T*)y, rows, cols, eps);
    }
    RT_CHECK_LAUNCH("norm_seq16_kernel");
    return RT_OK;
}

// the row walk is latency bound, so prefer many small row groups until the chip is covered a few times over
template <typename T, int KIND>
int launch_norm16(rt_device* dev, const void* x, const void* scale, const void* bias, void* y, uint64_t rows, uint32_t cols, float eps) {
    const bool vec_ok = (cols % 8 == 0) && rt_aligned(x, 16) && rt_aligned(y, 16) && rt_aligned(scale, 16) && (!bias || rt_aligned(bias, 16));
    if (vec_ok && cols <= 128 && rows >= 16384) return launch_norm16_lane<T, KIND>(dev, x, scale, bias, y, rows, cols, eps);
    // RMSNorm rows of 256 to 4096 columns, as many of them as the walk below takes in one round (8 rows a block, two
    // blocks a CU): the row sum replayed by a whole wave per row.  That kernel issues about twice the instructions of
    // the walk and a row takes a wave about 2.5 us, so it pays where the walk's latency is what the launch costs
    // ([4096,3072] f16: 12.5 against 14.2 us, [2048,2560] 8.8 against 10.6, [1024,4096] 9.2 against 14.5) and loses
    // where rows come in several rounds ([8192,3072] 25.5 against 22.1 us, [65536,512] 43 against 25).
    if (vec_ok && KIND == NORM_RMS && cols >= 256 && cols <= 4096 && rows <= 16ull * (uint64_t)dev->num_cus)
        return launch_rms16_par<T>(dev, x, scale, y, rows, cols, eps);
    if (vec_ok) {
        const uint64_t blocks = (rows + 7) / 8;
        RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "norm: too many rows");
        // all blocks resident at once (the latency-bound case): the output pass comes from LDS
        const uint32_t ntiles = (cols + 255) / 256;
        const size_t keep_bytes = (size_t)ntiles * NP_KEEP_BYTES_PER_TILE;
        const size_t static_bytes = (KIND == NORM_LAYER ? 2 : 1) * 2 * 8 * (std::is_same<T, half_t>::value ? 264 * 2 : 260 * sizeof(float)) + 256;
        const size_t per_cu = (160 * 1024) / (static_bytes + keep_bytes);
        if (cols <= NP_KEEP_MAX_COLS && blocks <= (uint64_t)dev->num_cus * per_cu) {
            const int ti = (std::is_same<T, half_t>::value ? 0 : 2) + (KIND == NORM_LAYER ? 0 : 1);
            if (!(dev->np_attr_set & (1u << ti))) {
                RT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(norm_pipe16_kernel<T, KIND, true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)((NP_KEEP_MAX_COLS / 256) * NP_KEEP_BYTES_PER_TILE)));
                dev->np_attr_set |= 1u << ti;
            }
            hipLaunchKernelGGL((norm_pipe16_kernel<T, KIND, true>), dim3((unsigned)blocks), dim3(NP_BLOCK), keep_bytes, dev->stream, (const T*)x,
                               (const T*)scale, (const T*)bias, (T*)y, rows, cols, eps);
        } else {
            hipLaunchKernelGGL((norm_pipe16_kernel<T, KIND, false>), dim3((unsigned)blocks), dim3(NP_BLOCK), 0, dev->stream, (const T*)x,
                               (const T*)scale, (const T*)bias, (T*)y, rows, cols, eps);
        }
        RT_CHECK_LAUNCH("norm_pipe16_kernel");
        return RT_OK;
    }
    const uint64_t want_blocks = (uint64_t)dev->num_cus * 4;
    if (rows / 32 >= want_blocks) return launch_norm16_rb<T, KIND, 32>(dev, x, scale, bias, y, rows, cols, eps);
    if (rows / 16 >= want_blocks) return launch_norm16_rb<T, KIND, 16>(dev, x, scale, bias, y, rows, cols, eps);
    return launch_norm16_rb<T, KIND, 8>(dev, x, scale, bias, y, rows, cols, eps);
}

int norm_entry(rt_device* dev, int kind, int dt, const void* x, const void* scale, const void* bias, void* y, uint64_t rows,
               uint32_t cols, float eps, const char* who) {
    RT_REQUIRE(rt_is_float_dt(dt), RT_ERR_DTYPE, "%s: dtype %d is not F32/F16/BF16", who, dt);
    RT_REQUIRE(cols > 0, RT_ERR_SHAPE, "%s: cols is 0", who);
    RT_REQUIRE(rows <= RT_MAX_NUMEL / cols, RT_ERR_SIZE, "%s: tensor too large", who);
    RT_REQUIRE(eps == eps, RT_ERR_ARG, "%s: eps is NaN", who);
    if (rows == 0) return dev ? RT_OK : rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(x && scale && y, RT_ERR_NULL_POINTER, "%s: NULL operand", who);
    const size_t eb = (size_t)rt_dt_bytes(dt);
    RT_REQUIRE(rt_aligned(x, eb) && rt_aligned(y, eb) && rt_aligned(scale, eb) && (!bias || rt_aligned(bias, eb)), RT_ERR_ALIGN,
               "%s: misaligned pointer", who);
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (kind == NORM_LAYER) {
        switch (dt) {
            case RT_F32: return launch_norm<float, NORM_LAYER>(dev, x, scale, bias, y, rows, cols, eps);
            case RT_F16: return launch_norm16<half_t, NORM_LAYER>(dev, x, scale, bias, y, rows, cols, eps);
            default: return launch_norm16<bf16_t, NORM_LAYER>(dev, x, scale, bias, y, rows, cols, eps);
        }
    }
    switch (dt) {
        case RT_F32: return launch_norm<float, NORM_RMS>(dev, x, scale, nullptr, y, rows, cols, eps);
        case RT_F16: return launch_norm16<half_t, NORM_RMS>(dev, x, scale, nullptr, y, rows, cols, eps);
        default: return launch_norm16<bf16_t, NORM_RMS>(dev, x, scale, nullptr, y, rows, cols, eps);
    }
}

// Few, small groups (the latency-bound case: 32 groups of 96 KB in the reference's Whisper-style shape): one launch, one
// 1024-thread block per (batch, group), the group staged in LDS once, then mean, squared deviations and the output all
// come from LDS.  Same definitions as the two-kernel path (mean, then the variance about that mean, f32 arithmetic).
constexpr int GN_LDS_BLOCK = 1024;
constexpr size_t GN_LDS_MAX_BYTES = 144 * 1024;
constexpr size_t GN_REG_MAX_BYTES = 16 * 1024 * 16;           // what gn_reg_kernel holds without spilling: 16 vectors in each of 1024 threads

template <typename T>
__global__ void __launch_bounds__(GN_LDS_BLOCK) gn_lds_kernel(const T* __restrict__ x, const T* __restrict__ scale, const T* __restrict__ bias,
                                                              T* __restrict__ y, uint32_t glen, uint32_t cpg, uint32_t groups, FastDiv L,
                                                              float eps) {
    constexpr int VE = 16 / sizeof(T);
    extern __shared__ __attribute__((aligned(16))) unsigned char gn_smem[];
    v4u* stage = reinterpret_cast<v4u*>(gn_smem);
    const uint32_t grp = blockIdx.x, g = grp % groups;
    const v4u* xs = reinterpret_cast<const v4u*>(x + (uint64_t)grp * glen);
    v4u* ys = reinterpret_cast<v4u*>(y + (uint64_t)grp * glen);
    const uint32_t nvec = glen / VE;
    float acc = 0.0f;
    for (uint32_t i0 = threadIdx.x; i0 < nvec; i0 += GN_LDS_BLOCK * 8) {    // eight loads in flight per thread
        Vec16<T> v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint32_t i = i0 + k * GN_LDS_BLOCK;
            if (i < nvec) v[k].u = ld_stream(xs + i);
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint32_t i = i0 + k * GN_LDS_BLOCK;
            if (i < nvec) {
                stage[i] = v[k].u;
#pragma unroll
                for (int q = 0; q < VE; q++) acc += Ar<T>::widen(v[k].e[q]);
            }
        }
    }
    const float mean = row_sum<GN_LDS_BLOCK>(acc) / (float)glen;
    float m2 = 0.0f;
    for (uint32_t i = threadIdx.x; i < nvec; i += GN_LDS_BLOCK) {           // a thread re-reads what it wrote itself
        Vec16<T> v;
        v.u = stage[i];
#pragma unroll
        for (int q = 0; q < VE; q++) {
            const float d = Ar<T>::widen(v.e[q]) - mean;
            m2 += d * d;
        }
    }
    const float var = row_sum<GN_LDS_BLOCK>(m2) / (float)glen;
    const float rstd = 1.0f / __builtin_sqrtf(var + eps);
    for (uint32_t i = threadIdx.x; i < nvec; i += GN_LDS_BLOCK) {
        Vec16<T> v;
        v.u = stage[i];
        st_stream(ys + i, gn_affine_vec<T>(v, i * VE, g * cpg, L, scale, bias, mean, rstd));
    }
}

// The group in the registers of 1024-thread blocks (thread t holds vectors t, t + 1024, ...; NV of them), for groups too
// large for the LDS of gn_lds_kernel (one block per group) and for small problems of few groups (32 groups of 96 KB on 256
// CUs): there `slices` blocks per group, all in one launch and without any wait between blocks.  Every block of a group
// loads the WHOLE group and reduces it to the same mean and variance in the same order, so the blocks of a group agree
// bit for bit without exchanging anything; each then normalises and stores only its own run of nvec / slices vectors.
// The repeated reads of a group hit the L2 of the XCD its blocks share (see the block -> (group, slice) map in
// launch_gn), so HBM still sees the group once.  Same definitions as gn_lds_kernel.
template <typename T, int NV>
__global__ void __launch_bounds__(GN_LDS_BLOCK) gn_reg_kernel(const T* __restrict__ x, const T* __restrict__ scale, const T* __restrict__ bias,
                                                              T* __restrict__ y, uint32_t glen, uint32_t cpg, uint32_t groups, FastDiv L,
                                                              float eps, uint32_t slices, uint32_t per_xcd) {
    constexpr int VE = 16 / sizeof(T);
    // blocks are handed to the 8 XCDs round robin: pair index p runs over the (group, slice) pairs of one XCD first
    const uint32_t p = per_xcd ? (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3) : blockIdx.x;
    const uint32_t grp = p / slices, slice = p - grp * slices, g = grp % groups;
    const v4u* xs = reinterpret_cast<const v4u*>(x + (uint64_t)grp * glen);
    v4u* ys = reinterpret_cast<v4u*>(y + (uint64_t)grp * glen);
    const uint32_t nvec = glen / VE;
    Vec16<T> v[NV];
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = threadIdx.x + k * GN_LDS_BLOCK;
        v[k].u = v4u{0u, 0u, 0u, 0u};
        if (i < nvec) v[k].u = xs[i];
    }
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
#pragma unroll
        for (int q = 0; q < VE; q++) acc += Ar<T>::widen(v[k].e[q]);         // vectors past the group hold zeros
    }
    const float mean = row_sum<GN_LDS_BLOCK>(acc) / (float)glen;
    // the group stays in registers as it was loaded.  With 16 vectors a thread the widened values of one pass must not be kept
    // for the next (the compiler otherwise keeps them and spills); with fewer it may keep what fits (32 groups of 93 KiB f16,
    // 6 vectors a thread: 8.3 us when every pass widens again, 6.3 us when not)
    auto forget = [&]() {
        if (NV < 16) return;
#pragma unroll
        for (int k = 0; k < NV; k++) asm volatile("" : "+v"(v[k].u[0]), "+v"(v[k].u[1]), "+v"(v[k].u[2]), "+v"(v[k].u[3]));
    };
    forget();
    float m2 = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
        if (threadIdx.x + k * GN_LDS_BLOCK < nvec) {
#pragma unroll
            for (int q = 0; q < VE; q++) {
                const float d = Ar<T>::widen(v[k].e[q]) - mean;
                m2 += d * d;
            }
        }
    }
    const float var = row_sum<GN_LDS_BLOCK>(m2) / (float)glen;
    forget();
    const float rstd = 1.0f / __builtin_sqrtf(var + eps);
    const uint32_t lo = (uint32_t)(((uint64_t)nvec * slice) / slices), hi = (uint32_t)(((uint64_t)nvec * (slice + 1)) / slices);
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = threadIdx.x + k * GN_LDS_BLOCK;
        if (i >= lo && i < hi) {
            st_stream(ys + i, gn_affine_vec<T>(v[k], i * VE, g * cpg, L, scale, bias, mean, rstd));
        }
    }
}

// Many slices per group (few, very large groups): the partials of a group are combined once, by one block, into a
// single (mean, M2, count) triple that the apply kernel then reads as if the group had one slice.
__global__ void __launch_bounds__(BLOCK) gn_combine_kernel(const float* __restrict__ part, float* __restrict__ out, uint32_t splits) {
    __shared__ double s_n[BLOCK], s_mean[BLOCK], s_m2[BLOCK];
    const float* p = part + (uint64_t)blockIdx.x * splits * 3;
    double n = 0.0, mean = 0.0, m2 = 0.0;
    auto merge = [&](double nb, double mb, double m2b) {                       // Chan et al.
        if (nb == 0.0) return;
        const double nt = n + nb;
        const double delta = mb - mean;
        mean += delta * (nb / nt);
        m2 += m2b + delta * delta * (n * nb / nt);
        n = nt;
    };
    for (uint32_t k = threadIdx.x; k < splits; k += BLOCK) merge((double)p[3 * k + 2], (double)p[3 * k], (double)p[3 * k + 1]);
    s_n[threadIdx.x] = n;
    s_mean[threadIdx.x] = mean;
    s_m2[threadIdx.x] = m2;
    __syncthreads();
    for (int off = BLOCK / 2; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) {
            merge(s_n[threadIdx.x + off], s_mean[threadIdx.x + off], s_m2[threadIdx.x + off]);
            s_n[threadIdx.x] = n;
            s_mean[threadIdx.x] = mean;
            s_m2[threadIdx.x] = m2;
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        float* o = out + (uint64_t)blockIdx.x * 3;
        o[0] = (float)mean;
        o[1] = (float)m2;
        o[2] = (float)n;
    }
}

// fixed_scratch == nullptr: partial statistics go to the device's own buffer, grown from the driver when a problem needs
// more; otherwise to fixed_scratch (GN_STATIC_SCRATCH_BYTES), and a problem that needs more is refused.
template <typename T>
int launch_gn(rt_device* dev, const void* x, const void* scale, const void* bias, void* y, uint32_t bg, uint32_t glen, uint32_t cpg,
              uint32_t groups, uint32_t L, float eps, float* fixed_scratch) {
    // enough blocks to cover the chip, slices of at least 2048 elements; beyond 64 slices per group the partials are
    // combined by a launch of their own instead of by every apply block
    constexpr uint32_t FUSED_COMBINE_MAX = 64;
    static_assert(FUSED_COMBINE_MAX <= WAVE, "gn_apply_kernel combines one partial per lane of a wave");
    uint32_t splits = (2048 + bg - 1) / bg;
    const uint32_t max_splits = (glen + 2047) / 2048;
    if (splits > max_splits) splits = max_splits;
    if (splits > 2048) splits = 2048;
    if (splits < 1) splits = 1;
    constexpr int VEMAX = 16 / sizeof(T);
    const bool vec = (glen % VEMAX == 0) && rt_aligned(x, 16) && rt_aligned(y, 16);    // every group starts on a vector boundary
    // Which path, for vector-aligned groups (measured on 256 CUs; the two or three launches below spread any problem over the
    // whole chip in small blocks, the one-launch kernels read HBM once but run 1024-thread blocks that hold whole groups):
    //   few groups (at most half as many as CUs) of up to 9 vectors a thread (144 KiB; 12 vectors, 192 KiB, in f32):
    //        gn_reg_kernel, several blocks per group (32 groups of 93 KiB f16 6.3 us against 6.9 for the launches, 96 groups
    //        7.5 against 10.2 for gn_lds_kernel, 128 groups of 187 KiB f32 12.0 against 13.0 with one block per group).  16-bit
    //        groups beyond 9 vectors a thread widen to more registers than a thread has: 64 groups of 160 KiB f16 13.3 us
    //        against 9.6 for the launches
    //   up to 144 KiB, more groups than that (and at most eight times as many as CUs): gn_lds_kernel
    //        (93 KiB f16 x 256 groups 12.1 us against 15.2 for the launches, 64 KiB x 1024 28.4 against 34.4; gn_reg_kernel
    //        on these is within 8 % either way, except 47 KiB f16 x 2048: 53.6 against 42.3)
    //   f32 groups of 144 to 192 KiB, at least half as many groups as CUs, and of up to 256 KiB (16 vectors a thread; 20 and
    //        24 spill), at least as many groups as CUs: gn_reg_kernel, one block per group (187 KiB x 256 groups 20.0 us
    //        against 25.3 for the launches, 256 KiB x 256 27.3 against 32.9, x 1024 107 against 125; 256 KiB x 128: 16.5
    //        against 16.4).  In 16 bits the launches are as fast or faster on these (160 KiB x 128 groups 13.3 us against
    //        16.9, 256 KiB x 512 64.2 against 65.8)
    //   everything else: the launches below
    const size_t gbytes = (size_t)glen * sizeof(T);
    const uint32_t cus = (uint32_t)dev->num_cus;
    const uint32_t nv_group = (glen / VEMAX + GN_LDS_BLOCK - 1) / GN_LDS_BLOCK;          // vectors a thread of gn_reg_kernel would hold
    const bool reg_few = 2u * bg <= cus && (nv_group <= 9 || (sizeof(T) == 4 && nv_group <= 12));
    const bool reg_large = sizeof(T) == 4 && gbytes > GN_LDS_MAX_BYTES && bg <= 8u * cus &&
                           ((gbytes <= GN_REG_MAX_BYTES * 3 / 4 && 2u * bg >= cus) || (gbytes <= GN_REG_MAX_BYTES && bg >= cus));
    if (vec && (reg_few || reg_large)) {
        uint32_t slices = reg_few && bg <= cus ? cus / bg : 1;
        if (slices > 32) slices = 32;
        const uint32_t nvec = glen / VEMAX;
        if (slices > nvec) slices = nvec;
        const uint32_t blocks = bg * slices;
        // with a block count that the 8 XCDs share evenly, block b (on XCD b % 8) takes pair (b % 8) * blocks / 8 + b / 8, which
        // puts the slices of a group on one XCD (all of them when bg is a multiple of 8)
        const uint32_t per_xcd = (slices > 1 && blocks % 8 == 0) ? blocks / 8 : 0;
        const uint32_t nv = (nvec + GN_LDS_BLOCK - 1) / GN_LDS_BLOCK;
        const dim3 grid(blocks), block(GN_LDS_BLOCK);
#define RT_GN_REG(NVC)                                                                                                                      \
    hipLaunchKernelGGL((gn_reg_kernel<T, NVC>), grid, block, 0, dev->stream, (const T*)x, (const T*)scale, (const T*)bias, (T*)y, glen, cpg, \
                       groups, make_fastdiv(L), eps, slices, per_xcd)
        if (nv <= 1) RT_GN_REG(1);
        else if (nv <= 2) RT_GN_REG(2);
        else if (nv <= 4) RT_GN_REG(4);
        else if (nv <= 6) RT_GN_REG(6);
        else if (nv <= 9) RT_GN_REG(9);
        else if (nv <= 12) RT_GN_REG(12);
        else RT_GN_REG(16);
#undef RT_GN_REG
        RT_CHECK_LAUNCH("gn_reg_kernel");
        return RT_OK;
    }
    if (vec && gbytes <= GN_LDS_MAX_BYTES && 8u * bg >= 3u * cus && bg <= 8u * cus) {
        const int ti = sizeof(T) == 4 ? 0 : (std::is_same<T, half_t>::value ? 1 : 2);
        if (!(dev->gn_lds_attr_set & (1u << ti))) {
            RT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gn_lds_kernel<T>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)GN_LDS_MAX_BYTES));
            dev->gn_lds_attr_set |= 1u << ti;
        }
        hipLaunchKernelGGL((gn_lds_kernel<T>), dim3(bg), dim3(GN_LDS_BLOCK), (size_t)glen * sizeof(T), dev->stream, (const T*)x, (const T*)scale,
                           (const T*)bias, (T*)y, glen, cpg, groups, make_fastdiv(L), eps);
        RT_CHECK_LAUNCH("gn_lds_kernel");
        return RT_OK;
    }
    // slices of at most 32 KiB stay in the registers of their 256-thread block (8 vectors a thread), in the stats launch and
    // in the apply launch: more, smaller slices when the rule above leaves them larger
    constexpr uint32_t GN_SLICE_REG_VEC = 8;
    constexpr uint32_t slice_reg_elems = GN_SLICE_REG_VEC * BLOCK * VEMAX;
    if (vec) {
        const uint32_t want = (glen + slice_reg_elems - 1) / slice_reg_elems;
        // (only while the partials still fit the fixed buffer of rt_group_norm_static: both entry points slice alike)
        if (want > splits && want <= 2048 && ((size_t)bg * want + bg) * 3 * sizeof(float) <= GN_STATIC_SCRATCH_BYTES) splits = want;
    }
    uint32_t chunk = (glen + splits - 1) / splits;
    if (vec) chunk = (chunk + VEMAX - 1) / VEMAX * VEMAX;                               // slices start on vector boundaries
    splits = (glen + chunk - 1) / chunk;
    const bool slice_reg = vec && chunk <= slice_reg_elems;
    const uint32_t slice_nv = slice_reg ? (chunk / VEMAX + BLOCK - 1) / BLOCK : 0;
    const size_t need = ((size_t)bg * splits + bg) * 3 * sizeof(float);           // partials, then one combined triple per group
    if (fixed_scratch) {
        RT_REQUIRE(need <= GN_STATIC_SCRATCH_BYTES, RT_ERR_SIZE,
                   "rt_group_norm_static: %u (batch, group) pairs in %u slices need %zu bytes of partial statistics, the fixed buffer holds %zu",
                   bg, splits, need, GN_STATIC_SCRATCH_BYTES);
    } else if (need > dev->gn_scratch_bytes) {
        RT_NO_CAPTURE(dev, "growing the GroupNorm scratch");
        RT_HIP(hipStreamSynchronize(dev->stream));
        RT_HIP(hipFree(dev->gn_scratch));
        dev->gn_scratch = nullptr;
        dev->gn_scratch_bytes = 0;
        RT_HIP(hipMalloc((void**)&dev->gn_scratch, need));
        dev->gn_scratch_bytes = need;
    }
    const dim3 grid(bg, splits), block(BLOCK);
    const bool separate = splits > FUSED_COMBINE_MAX;
    float* const part = fixed_scratch ? fixed_scratch : dev->gn_scratch;
    const float* stats = separate ? part + (size_t)bg * splits * 3 : part;
    const uint32_t stat_splits = separate ? 1 : splits;
#define RT_GN_STATS(NVC) \
    hipLaunchKernelGGL((gn_stats_reg_kernel<T, NVC>), grid, block, 0, dev->stream, (const T*)x, part, glen, chunk, splits)
    if (slice_reg && slice_nv <= 1) RT_GN_STATS(1);
    else if (slice_reg && slice_nv <= 2) RT_GN_STATS(2);
    else if (slice_reg && slice_nv <= 4) RT_GN_STATS(4);
    else if (slice_reg) RT_GN_STATS(8);
    else if (vec) hipLaunchKernelGGL((gn_stats_kernel<T, VEMAX>), grid, block, 0, dev->stream, (const T*)x, part, glen, chunk, splits);
    else hipLaunchKernelGGL((gn_stats_kernel<T, 1>), grid, block, 0, dev->stream, (const T*)x, part, glen, chunk, splits);
#undef RT_GN_STATS
    RT_CHECK_LAUNCH("gn_stats_kernel");
    if (separate) {
        hipLaunchKernelGGL(gn_combine_kernel, dim3(bg), block, 0, dev->stream, (const float*)part,
                           part + (size_t)bg * splits * 3, splits);
        RT_CHECK_LAUNCH("gn_combine_kernel");
    }
#define RT_GN_APPLY(NVC)                                                                                                                   \
    hipLaunchKernelGGL((gn_apply_reg_kernel<T, NVC>), grid, block, 0, dev->stream, (const T*)x, (const T*)scale, (const T*)bias, (T*)y, stats, \
                       glen, chunk, stat_splits, cpg, groups, make_fastdiv(L), eps)
    if (slice_reg && slice_nv <= 1) RT_GN_APPLY(1);
    else if (slice_reg && slice_nv <= 2) RT_GN_APPLY(2);
    else if (slice_reg && slice_nv <= 4) RT_GN_APPLY(4);
    else if (slice_reg) RT_GN_APPLY(8);
#undef RT_GN_APPLY
    else if (vec) {
        hipLaunchKernelGGL((gn_apply_kernel<T, VEMAX>), grid, block, 0, dev->stream, (const T*)x, (const T*)scale, (const T*)bias, (T*)y, stats,
                           glen, chunk, stat_splits, cpg, groups, make_fastdiv(L), eps);
    } else {
        hipLaunchKernelGGL((gn_apply_kernel<T, 1>), grid, block, 0, dev->stream, (const T*)x, (const T*)scale, (const T*)bias, (T*)y, stats,
                           glen, chunk, stat_splits, cpg, groups, make_fastdiv(L), eps);
    }
    RT_CHECK_LAUNCH("gn_apply_kernel");
    return RT_OK;
}

template <typename T, int KIND>
int launch_norm_via32(rt_device* dev, const void* x, const float* scale, const float* bias, void* y, uint64_t rows, uint32_t cols, float eps) {
    const uint32_t nvec = cols / 8;
    const bool vec_ok = (cols % 8 == 0) && rt_aligned(x, 16) && rt_aligned(y, 16) && rt_aligned(scale, 16) && (!bias || rt_aligned(bias, 16)) &&
                        nvec <= (uint32_t)(BLOCK * 8);
    if (vec_ok && nvec <= 32) {
        // rows of at most 32 vectors: a group of 2..32 lanes per row (one vector each), so that a wave carries 2..32 rows
        // and as many bytes as with long rows
        const uint32_t lanes = nvec <= 2 ? 2 : nvec <= 4 ? 4 : nvec <= 8 ? 8 : nvec <= 16 ? 16 : 32;
        const uint64_t blocks = (rows + BLOCK / lanes - 1) / (BLOCK / lanes);
        RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_norm_via_f32: too many rows");
        const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_NARROW(L) hipLaunchKernelGGL((norm_via32_wave_kernel<T, 1, KIND, L>), grid, block, 0, dev->stream, (const T*)x, scale, bias, (T*)y, rows, cols, eps)
        if (lanes == 2) RT_NARROW(2);
        else if (lanes == 4) RT_NARROW(4);
        else if (lanes == 8) RT_NARROW(8);
        else if (lanes == 16) RT_NARROW(16);
        else RT_NARROW(32);
#undef RT_NARROW
        RT_CHECK_LAUNCH("norm_via32_wave_kernel");
        return RT_OK;
    }
    if (vec_ok && nvec <= (uint32_t)(WAVE * 8)) {
        const uint32_t nv = (nvec + WAVE - 1) / WAVE;
        // LayerNorm over 16384 rows or more: a wave takes two rows and loads the weights once for both (measured against one
        // row a wave: [32768,2048] 49.5 against 51.8 us, [16384,3072] 39.2 against 41.9, [65536,512] 25.2 against 27.1; with fewer
        // rows the chip is not covered often enough for the fatter waves, [8192,4096] 30.5 against 28.8; four rows a wave
        // win on some shapes and lose on others; RMSNorm, with half the weights, gains nothing at any size)
        const int rw = KIND == NORM_LAYER && rows >= (uint64_t)dev->num_cus * 64 ? 2 : 1;
        const uint64_t blocks = ((rows + rw - 1) / rw + WAVES - 1) / WAVES;
        RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_norm_via_f32: too many rows");
        const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_NV(NVC, RWC) hipLaunchKernelGGL((norm_via32_rows_kernel<T, NVC, KIND, WAVE, RWC>), grid, block, 0, dev->stream, (const T*)x, scale, bias, (T*)y, rows, cols, eps)
#define RT_NV1(NVC) hipLaunchKernelGGL((norm_via32_wave_kernel<T, NVC, KIND, WAVE>), grid, block, 0, dev->stream, (const T*)x, scale, bias, (T*)y, rows, cols, eps)
#define RT_NV_RW2(NVC)               \
    do {                             \
        if (rw == 2) RT_NV(NVC, 2);  \
        else RT_NV1(NVC);            \
    } while (0)
        if (nv <= 1) RT_NV_RW2(1);
        else if (nv <= 2) RT_NV_RW2(2);
        else if (nv <= 4) RT_NV_RW2(4);
        else if (nv <= 6) RT_NV_RW2(6);
        else RT_NV_RW2(8);
#undef RT_NV_RW2
#undef RT_NV1
#undef RT_NV
        RT_CHECK_LAUNCH("norm_via32_wave_kernel");
        return RT_OK;
    }
    if (vec_ok) {
        const uint32_t nv = (nvec + BLOCK - 1) / BLOCK;
        RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "rt_norm_via_f32: too many rows");
        // LayerNorm over 2048 rows or more: a block takes two rows and loads the weights once for both ([2048,8192] 12.7 against
        // 17.2 us, [8192,5120] 35.5 against 38.5, [16384,8192] 99 against 115; RMSNorm gains nothing)
        const int rw = KIND == NORM_LAYER && rows >= (uint64_t)dev->num_cus * 8 ? 2 : 1;
        const dim3 grid((unsigned)((rows + rw - 1) / rw)), block(BLOCK);
#define RT_NV(NVC, RWC) hipLaunchKernelGGL((norm_via32_rows_kernel<T, NVC, KIND, BLOCK, RWC>), grid, block, 0, dev->stream, (const T*)x, scale, bias, (T*)y, rows, cols, eps)
#define RT_NV1(NVC) hipLaunchKernelGGL((norm_via32_wave_kernel<T, NVC, KIND, BLOCK>), grid, block, 0, dev->stream, (const T*)x, scale, bias, (T*)y, rows, cols, eps)
#define RT_NV_RW2(NVC)               \
    do {                             \
        if (rw == 2) RT_NV(NVC, 2);  \
        else RT_NV1(NVC);            \
    } while (0)
        if (nv <= 3) RT_NV_RW2(3);
        else if (nv <= 4) RT_NV_RW2(4);
        else if (nv <= 6) RT_NV_RW2(6);
        else RT_NV_RW2(8);
#undef RT_NV_RW2
#undef RT_NV1
#undef RT_NV
        RT_CHECK_LAUNCH("norm_via32_wave_kernel");
        return RT_OK;
    }
    RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "rt_norm_via_f32: too many rows");
    hipLaunchKernelGGL((norm_via32_generic_kernel<T, KIND>), dim3((unsigned)rows), dim3(BLOCK), 0, dev->stream, (const T*)x, scale, bias,
                       (T*)y, rows, cols, eps);
    RT_CHECK_LAUNCH("norm_via32_generic_kernel");
    return RT_OK;
}

}  // namespace

// Called by rt_device_create with the new device current: looks up where THIS device's copy of gn_static_scratch lies.
int rt_norm_device_init(rt_device* dev) {
    void* p = nullptr;
    RT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(gn_static_scratch)));
    dev->gn_static_ptr = static_cast<float*>(p);
    return RT_OK;
}

extern "C" {

int rt_norm_via_f32(rt_device* dev, int kind, int io_dt, const void* x, const float* scale, const float* bias, void* y, uint64_t rows,
                    uint32_t cols, float eps) {
    RT_REQUIRE(kind == NORM_LAYER || kind == NORM_RMS, RT_ERR_ARG, "rt_norm_via_f32: kind %d is not 0 (layer) or 1 (rms)", kind);
    RT_REQUIRE(io_dt == RT_F16 || io_dt == RT_BF16, RT_ERR_DTYPE, "rt_norm_via_f32: dtype %d is not F16/BF16", io_dt);
    RT_REQUIRE(cols > 0, RT_ERR_SHAPE, "rt_norm_via_f32: cols is 0");
    RT_REQUIRE(rows <= RT_MAX_NUMEL / cols, RT_ERR_SIZE, "rt_norm_via_f32: tensor too large");
    RT_REQUIRE(eps == eps, RT_ERR_ARG, "rt_norm_via_f32: eps is NaN");
    if (rows == 0) return dev ? RT_OK : rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(x && scale && y, RT_ERR_NULL_POINTER, "rt_norm_via_f32: NULL operand");
    RT_REQUIRE(rt_aligned(x, 2) && rt_aligned(y, 2) && rt_aligned(scale, 4) && (!bias || rt_aligned(bias, 4)), RT_ERR_ALIGN,
               "rt_norm_via_f32: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (kind == NORM_RMS) bias = nullptr;
    if (io_dt == RT_F16)
        return kind == NORM_LAYER ? launch_norm_via32<half_t, NORM_LAYER>(dev, x, scale, bias, y, rows, cols, eps)
                                  : launch_norm_via32<half_t, NORM_RMS>(dev, x, scale, bias, y, rows, cols, eps);
    return kind == NORM_LAYER ? launch_norm_via32<bf16_t, NORM_LAYER>(dev, x, scale, bias, y, rows, cols, eps)
                              : launch_norm_via32<bf16_t, NORM_RMS>(dev, x, scale, bias, y, rows, cols, eps);
}

int rt_layer_norm(rt_device* dev, int dt, const void* x, const void* scale, const void* bias, void* y, uint64_t rows, uint32_t cols,
                  float eps) {
    return norm_entry(dev, NORM_LAYER, dt, x, scale, bias, y, rows, cols, eps, "rt_layer_norm");
}

int rt_rms_norm(rt_device* dev, int dt, const void* x, const void* scale, void* y, uint64_t rows, uint32_t cols, float eps) {
    return norm_entry(dev, NORM_RMS, dt, x, scale, nullptr, y, rows, cols, eps, "rt_rms_norm");
}

static int group_norm_entry(rt_device* dev, int dt, const void* x, const void* scale, const void* bias, void* y, uint32_t B, uint32_t C,
                            uint32_t L, uint32_t groups, float eps, bool fixed) {
    RT_REQUIRE(rt_is_float_dt(dt), RT_ERR_DTYPE, "rt_group_norm: dtype %d is not F32/F16/BF16", dt);
    RT_REQUIRE(B > 0 && C > 0 && L > 0, RT_ERR_SHAPE, "rt_group_norm: zero extent");
    RT_REQUIRE(groups > 0 && C % groups == 0, RT_ERR_ARG, "rt_group_norm: %u channels do not split into %u groups", C, groups);
    RT_REQUIRE(eps == eps, RT_ERR_ARG, "rt_group_norm: eps is NaN");
    const uint64_t glen = (uint64_t)(C / groups) * L;
    RT_REQUIRE(glen <= 0x7fffffffull && (uint64_t)B * groups <= 0x7fffffffull, RT_ERR_SIZE, "rt_group_norm: group too large");
    RT_REQUIRE(x && y, RT_ERR_NULL_POINTER, "rt_group_norm: NULL operand");
    const size_t eb = (size_t)rt_dt_bytes(dt);
    RT_REQUIRE(rt_aligned(x, eb) && rt_aligned(y, eb) && (!scale || rt_aligned(scale, eb)) && (!bias || rt_aligned(bias, eb)),
               RT_ERR_ALIGN, "rt_group_norm: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    const uint32_t bg = B * groups;
    float* fixed_scratch = nullptr;
    if (fixed) {
        fixed_scratch = dev->gn_static_ptr;
        RT_REQUIRE(fixed_scratch, RT_ERR_ARG, "rt_group_norm_static: the device's fixed scratch buffer was not resolved at rt_device_create");
    }
    switch (dt) {
        case RT_F32: return launch_gn<float>(dev, x, scale, bias, y, bg, (uint32_t)glen, C / groups, groups, L, eps, fixed_scratch);
        case RT_F16: return launch_gn<half_t>(dev, x, scale, bias, y, bg, (uint32_t)glen, C / groups, groups, L, eps, fixed_scratch);
        default: return launch_gn<bf16_t>(dev, x, scale, bias, y, bg, (uint32_t)glen, C / groups, groups, L, eps, fixed_scratch);
    }
}

int rt_group_norm(rt_device* dev, int dt, const void* x, const void* scale, const void* bias, void* y, uint32_t B, uint32_t C, uint32_t L,
                  uint32_t groups, float eps) {
    return group_norm_entry(dev, dt, x, scale, bias, y, B, C, L, groups, eps, false);
}

int rt_group_norm_static(rt_device* dev, int dt, const void* x, const void* scale, const void* bias, void* y, uint32_t B, uint32_t C,
                         uint32_t L, uint32_t groups, float eps) {
    return group_norm_entry(dev, dt, x, scale, bias, y, B, C, L, groups, eps, true);
}

}  // extern "C"
