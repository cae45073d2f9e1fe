// Softmax over the last dimension.
//
// Arithmetic contract (REFERENCE mode) = crates/ratchet-core/src/cpu/softmax.rs:22-42: e_j = exp(x_j) with no max
// subtraction, stored in the element type; sum accumulated over j ascending in the element type; y_j = e_j / sum.
//   f32: the row lives in registers (one wave64 per row, 16-byte loads), one exp per element (v_exp_f32 on
//        x * log2 e, see ref_exp_f32; the 1e-5 bar leaves room for that), the sum is a wave butterfly instead of a sequential fold
//        (differs from the reference by float rounding order only), one IEEE division per element.
//        HBM traffic: one read, one write.
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

// e^v of the f32 reference mode in the register-resident kernel: one v_exp_f32 (1 ulp) on v * log2(e).  The rounding of
// that product, half an ulp of |v| * 1.44, is the error: 3.3e-7 relative for |v| < 11, 6.6e-7 below 22, 2.6e-6 at the
// overflow threshold (bar: 1e-5).  -inf gives 0, +inf and anything from 88.73 up give inf, NaN stays NaN, as with expf;
// the library expf costs about four times the instructions, which at 27 M elements is most of the memory time.
// v_exp_f32 returns 0 where the result would be subnormal (v below about -87.3), where expf and the reference's CPU code
// return the subnormal: a row whose entries all lie there would sum to 0 and come out as 0 / 0.  Below 2^-126 the
// exponent is therefore raised by 64 before the instruction and the result scaled back by 2^-64, which is exact but for
// the one rounding into the subnormal grid that expf has too.
__device__ __forceinline__ float ref_exp_f32(float v) {
    const float p = v * 1.44269504088896341f;
    const bool tiny = p < -126.0f;
    const float e = __builtin_amdgcn_exp2f(p + (tiny ? 64.0f : 0.0f));
    return e * (tiny ? 0x1p-64f : 1.0f);
}

constexpr int WIDE_BLOCK = 1024;                        // threads per row for rows that do not fit 256 threads' registers

// ------------------------------------------------------------------------------------------------------------------
// Row held in registers by the LANES threads that share it: a wave64 (four rows per block) for rows of up to 512
// vectors, the whole 256-thread block for rows of up to 2048 vectors (8192 f32 / 16384 16-bit columns), a 1024-thread
// block for rows of up to 16384 vectors (65536 f32 columns: vocabulary-sized rows).
// Requires 16-byte aligned x and y and at most LANES * NV vectors per row; rows of whole vectors, or (SPAN) any length.
// MODE 0: reference arithmetic for f32 (exp, tree sum, divide).  MODE 1: stable (max subtraction, f32 accumulate) for
// any T; results are rounded to T once.
// ------------------------------------------------------------------------------------------------------------------
template <typename T, int NV, int MODE, int LANES, bool SPAN>
__global__ void __launch_bounds__(LANES > BLOCK ? LANES : BLOCK) softmax_wave_kernel(const T* x, T* y, uint64_t rows, uint32_t cols,
                                                                                       const T* mask, uint64_t period) {
    constexpr int VE = 16 / sizeof(T);
    constexpr int THREADS = LANES > BLOCK ? LANES : BLOCK;   // rows beyond 2048 vectors: one 1024-thread block per row
    const uint64_t row = (uint64_t)blockIdx.x * (THREADS / LANES) + (threadIdx.x / LANES);
    if (row >= rows) return;
    const int lane = threadIdx.x & (LANES - 1);
    // SPAN (rows that are not whole aligned vectors; x and y 16-byte aligned): the row is handled over the aligned vectors
    // that cover it.  It starts `shift` elements into the first one; span elements outside the row belong to the
    // neighbouring rows, are left out of the sums and are not written (the row's two ragged vectors are stored element
    // by element).  An aligned vector that holds one byte of the tensor lies in a mapped page, so the loads are safe
    // at the tensor's ends too.
    const uint64_t first = row * cols;
    const uint32_t shift = SPAN ? (uint32_t)(first & (VE - 1)) : 0;
    const uint32_t nvec = SPAN ? (shift + cols + VE - 1) / VE : cols / VE;
    const v4u* xr = reinterpret_cast<const v4u*>(x) + first / VE;
    v4u* yr = reinterpret_cast<v4u*>(y) + first / VE;
    // column of element q of vector i, valid when below cols (elements before the row wrap around)
    auto inside = [&](uint32_t i, int q) -> bool { return !SPAN || i * VE + (uint32_t)q - shift < cols; };
    Vec16<T> v[NV];
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nvec) v[k].u = ld_stream(xr + i);
    }
    // mask (rows of whole vectors only): row r of x takes mask row r % period, added in T as the separate add would, so
    // that the result has the bits of add-then-softmax.  Plain loads: a mask row is read once per leading index.
    if (!SPAN && mask) {
        const v4u* mr = reinterpret_cast<const v4u*>(mask) + (row % period) * nvec;
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = lane + k * LANES;
            if (i < nvec) {
                Vec16<T> mv;
                mv.u = mr[i];
#pragma unroll
                for (int q = 0; q < VE; q++) v[k].e[q] = Ar<T>::add(v[k].e[q], mv.e[q]);
            }
        }
    }
    float e[NV][VE];
    float m = 0.0f;
    if (MODE == 1) {
        m = -__builtin_huge_valf();
#pragma unroll
        for (int k = 0; k < NV; k++)
            if (lane + k * LANES < nvec)
#pragma unroll
                for (int q = 0; q < VE; q++)
                    if (inside(lane + k * LANES, q)) m = fmaxf(m, Ar<T>::widen(v[k].e[q]));
        m = row_max<LANES>(m);
        if (m == -__builtin_huge_valf()) m = 0.0f;           // fully masked row: exp(-inf - 0) = 0, 0/0 = NaN as torch does
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++)
        if (lane + k * LANES < nvec)
#pragma unroll
            for (int q = 0; q < VE; q++) {
                e[k][q] = 0.0f;
                if (inside(lane + k * LANES, q)) {
                    e[k][q] = (MODE == 1) ? expf(Ar<T>::widen(v[k].e[q]) - m) : ref_exp_f32(Ar<T>::widen(v[k].e[q]));
                    s += e[k][q];
                }
            }
    s = row_sum<LANES>(s);
    // MODE 0: e / s as e * (1/s) with one correctly rounded reciprocal per row and a Newton step per element.
    // A zero, subnormal, inf or NaN sum keeps the division so that 0/0, x/inf and inf/inf come out as the reference's do.
    const bool plain = MODE == 0 && (s >= 1.17549435e-38f) && (s < __builtin_huge_valf());
    const float rs = 1.0f / s;
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nvec) {
            Vec16<T> o;
#pragma unroll
            for (int q = 0; q < VE; q++) {
                const float p0 = e[k][q] * rs;               // one Newton step on e * (1/s): the correctly rounded quotient for normal sums
                o.e[q] = Ar<T>::conv(plain ? __builtin_fmaf(__builtin_fmaf(-s, p0, e[k][q]), rs, p0) : e[k][q] / s);
            }
            if (!SPAN || (inside(i, 0) && inside(i, VE - 1))) {
                st_stream(yr + i, o.u);
            } else {
                T* yrow = y + first;
#pragma unroll
                for (int q = 0; q < VE; q++)
                    if (inside(i, q)) yrow[i * VE + (uint32_t)q - shift] = o.e[q];
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
        s += (MODE == 1) ? expf(Ar<T>::widen(xr[j]) - m) : expf(Ar<T>::widen(xr[j]));
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
        const float ev = (MODE == 1) ? expf(Ar<T>::widen(xr[j]) - m) : expf(Ar<T>::widen(xr[j]));
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
                    in.u = *reinterpret_cast<const v4u*>(src);
#pragma unroll
                    for (int q = 0; q < 8; q++) out.e[q] = ar_exp<T>(in.e[q]);
                    *reinterpret_cast<v4u*>(&tile[r][col]) = out.u;
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
                    t.u = *reinterpret_cast<const v4u*>(trow + j);
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

    // the block's rows are one contiguous run of nrows * cols elements: all threads sweep it, whatever the row length
    const uint32_t cvec = cols / VE;
    const T* src = x + row0 * cols;
    T* dst = y + row0 * cols;
    for (uint64_t i = threadIdx.x; i < (uint64_t)nrows * cvec; i += BLOCK) {
        const T sum = sums[i / cvec];
        if (VEC) {
            Vec16<T> in, out;
            in.u = reinterpret_cast<const v4u*>(src)[i];
#pragma unroll
            for (int q = 0; q < 8; q++) out.e[q] = Ar<T>::div(ar_exp<T>(in.e[q]), sum);
            st_stream(reinterpret_cast<v4u*>(dst) + i, out.u);
        } else {
            dst[i] = Ar<T>::div(ar_exp<T>(src[i]), sum);
        }
    }
}

// ------------------------------------------------------------------------------------------------------------------
// 16-bit reference arithmetic, rows of at most 128 columns (whole aligned vectors): one lane per row.  A block's 256
// rows are one contiguous run: it goes to LDS with coalesced 16-byte loads, each lane takes its own row from there
// (row pitch 16 bytes more than the row, so the 16-byte LDS accesses of neighbouring lanes fall into different banks),
// computes exp, the sequential sum (a short chain inside the lane, 64 rows advancing per wave) and the quotients in
// registers, and the results leave through LDS the same way.  x moves once in and y once out whatever the number of
// rows.  (The streaming kernel below spends a 512-column step on every 30 rows however short they are: a million rows
// of 8 columns took it 282 us, the two-pass kernel 110 us.)
// ------------------------------------------------------------------------------------------------------------------
template <typename T, int NV>
__global__ void __launch_bounds__(BLOCK) softmax16_lane_kernel(const T* x, T* y, uint64_t rows) {
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
        T sum = Ar<T>::conv(0.0f);
#pragma unroll
        for (int k = 0; k < NV; k++)
#pragma unroll
            for (int q = 0; q < 8; q++) {
                v[k].e[q] = ar_exp<T>(v[k].e[q]);
                sum = Ar<T>::add(sum, v[k].e[q]);
            }
#pragma unroll
        for (int k = 0; k < NV; k++) {
#pragma unroll
            for (int q = 0; q < 8; q++) v[k].e[q] = Ar<T>::div(v[k].e[q], sum);
            mine[k] = v[k].u;
        }
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < nvec; i += BLOCK) st_stream(yb + i, stage[(i / NV) * (NV + 1) + i % NV]);
}

constexpr uint32_t LANE_MAX_COLS = 128;

template <typename T> int launch_lane16(rt_device* dev, const void* x, void* y, uint64_t rows, uint32_t cols) {
    const uint64_t blocks = (rows + BLOCK - 1) / BLOCK;
    RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax: too many rows");
#define RT_LANE(NV)                                                                                                              \
    case NV:                                                                                                                     \
        hipLaunchKernelGGL((softmax16_lane_kernel<T, NV>), dim3((unsigned)blocks), dim3(BLOCK), 0, dev->stream, (const T*)x, (T*)y, rows); \
        break
    switch (cols / 8) {
        RT_LANE(1); RT_LANE(2); RT_LANE(3); RT_LANE(4); RT_LANE(5); RT_LANE(6); RT_LANE(7); RT_LANE(8);
        RT_LANE(9); RT_LANE(10); RT_LANE(11); RT_LANE(12); RT_LANE(13); RT_LANE(14); RT_LANE(15); RT_LANE(16);
        default: return rt_fail(RT_ERR_ARG, "rt_softmax: internal: %u columns in the one-lane-per-row kernel", cols);
    }
#undef RT_LANE
    RT_CHECK_LAUNCH("softmax16_lane_kernel");
    return RT_OK;
}

constexpr uint32_t RAGGED_STREAM_MIN_COLS = 192;   // shorter ragged rows: the two-pass tile walker is faster than the streaming variant

// ------------------------------------------------------------------------------------------------------------------
// The attention caller pattern (ratchet-models/src/phi3/attn.rs:148-153, phi2/attn.rs:143-150, whisper/mha.rs:115-124):
//     w = scores.add(mask.cast(dt)).full().softmax(3).cast(dt)
// on 16-bit scores in one pass: the mask (broadcast over batch / heads, optional) is added in the 16-bit type as the
// separate add would, the sum is widened, the f32 softmax above is applied in registers and the result rounded once.
// 4 bytes of HBM traffic per element against 26 for the four separate ops (6 + 6 + 8 + 6).
// A mask too large for the L2s to keep between the heads is read in the block order of binary_bcast_kernel (all heads of a
// mask slab back to back on one XCD): [1,32,4096,4096] 329 us against 392 us in the plain order; smaller masks take the
// plain order, which is faster there ([1,32,2560,2560] 141 against 164 us, [1,32,1536,1536] 52 against 62 us).
// ------------------------------------------------------------------------------------------------------------------
struct MaskArgs {
    FastDiv d2, d1;          // x extents of dims 2 and 1 (rows = d0 * d1 * d2)
    uint32_t ms[3];          // mask row strides in elements over dims 0..2 (0 where the mask extent is 1)
    uint32_t mlast;          // 1: the mask has a full last dim, 0: one value per row
    uint32_t mvec;           // the mask starts on a 16-byte boundary (the span kernel may read it in aligned vectors)
    // Block order of the kernels with whole rows per block (four with a wave per row, one with a block per row) for a
    // large mask that repeats over the leading dims (an [S, T] mask under B * H heads): hardware block b runs on XCD
    // b % 8, so the `reps` blocks that need the same mask rows go to one XCD back to back and its L2 fetches them once;
    // an XCD takes a chunk of its row blocks (64 when they divide, else 4, else 1) per repeat before it moves to the
    // next repeat (as in the broadcast add, rt_elementwise.hip).  period (mask rows, a multiple of 32) == 0: plain order.
    FastDiv reps;
    uint32_t period;
};

template <typename T> __device__ __forceinline__ uint64_t mask_row_offset(uint64_t row, const MaskArgs& p) {
    uint32_t t, i2, i1, i0;
    fd_divmod((uint32_t)row, p.d2, t, i2);
    fd_divmod(t, p.d1, i0, i1);
    return (uint64_t)i0 * p.ms[0] + (uint64_t)i1 * p.ms[1] + (uint64_t)i2 * p.ms[2];
}

// exp for the one-pass kernels: the hardware's 2^x on x * log2(e).  Its result is within a few f32 ulps of exp(x) for
// the 16-bit inputs these kernels see (|x| <= 65504 rounds the product by at most 2^-24 relative, i.e. an absolute
// 6e-6 in the exponent at |x| = 88), far inside the 1e-3 bar that applies after the final rounding to 16 bits; the
// library expf the f32 softmax uses costs about four times as many instructions.
__device__ __forceinline__ float via32_exp(float v) { return __builtin_amdgcn_exp2f(v * 1.44269504088896341f); }

template <typename T, int NV, int MODE, bool MASK, int LANES>
__global__ void __launch_bounds__(BLOCK) softmax_via32_wave_kernel(const T* __restrict__ x, const T* __restrict__ mask,
                                                                   T* __restrict__ y, uint64_t rows, uint32_t cols, MaskArgs p) {
    uint32_t blk = blockIdx.x;
    if (MASK && (LANES == WAVE || LANES == BLOCK) && p.period) {
        const uint32_t slabs = p.period / (BLOCK / LANES);               // blocks per repeat, a multiple of 8
        const uint32_t per_xcd = slabs >> 3;
        const uint32_t cl = per_xcd % 64 == 0 ? 6 : per_xcd % 4 == 0 ? 2 : 0;
        uint32_t rep, chunk;
        const uint32_t idx = blk >> 3;
        fd_divmod(idx >> cl, p.reps, chunk, rep);
        blk = rep * slabs + ((chunk << cl) + (idx & ((1u << cl) - 1))) * 8u + (blk & 7u);
    }
    const uint64_t row = (uint64_t)blk * (BLOCK / LANES) + (threadIdx.x / LANES);
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
    if (MASK) {
        const T* mr = mask + mask_row_offset<T>(row, p);
        if (p.mlast) {
            const v4u* mv = reinterpret_cast<const v4u*>(mr);
#pragma unroll
            for (int k = 0; k < NV; k++) {
                const uint32_t i = lane + k * LANES;
                if (i < nvec) {
                    Vec16<T> m;
                    m.u = mv[i];
#pragma unroll
                    for (int q = 0; q < 8; q++) v[k].e[q] = Ar<T>::add(v[k].e[q], m.e[q]);
                }
            }
        } else {
            const T m = mr[0];
#pragma unroll
            for (int k = 0; k < NV; k++)
#pragma unroll
                for (int q = 0; q < 8; q++) v[k].e[q] = Ar<T>::add(v[k].e[q], m);
        }
    }
    float e[NV][8];
    float m = 0.0f;
    if (MODE == 1) {
        m = -__builtin_huge_valf();
#pragma unroll
        for (int k = 0; k < NV; k++)
            if (lane + k * LANES < nvec)
#pragma unroll
                for (int q = 0; q < 8; q++) m = fmaxf(m, Ar<T>::widen(v[k].e[q]));
        m = row_max<LANES>(m);
        if (m == -__builtin_huge_valf()) m = 0.0f;
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++)
        if (lane + k * LANES < nvec)
#pragma unroll
            for (int q = 0; q < 8; q++) {
                e[k][q] = via32_exp(Ar<T>::widen(v[k].e[q]) - m);
                s += e[k][q];
            }
    s = row_sum<LANES>(s);
    const bool plain = (s >= 1.17549435e-38f) && (s < __builtin_huge_valf());
    const float rs = 1.0f / s;
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nvec) {
            Vec16<T> o;
#pragma unroll
            for (int q = 0; q < 8; q++) o.e[q] = Ar<T>::conv(plain ? e[k][q] * rs : e[k][q] / s);
            st_stream(yr + i, o.u);
        }
    }
}

// Rows that are not whole aligned vectors (a prompt of 1001 tokens: [B, H, 1001, 1001] scores): the same kernel over the
// span of aligned 16-byte vectors that covers the row.  Row r starts `shift` = (r * cols) % 8 elements into its first
// vector; elements of the span outside the row belong to the neighbouring rows, are ignored on the way in and are not
// written on the way out (the two ragged vectors of a row are stored element by element).  An aligned vector that
// holds one byte of the tensor lies in a mapped page, so the loads are safe at the tensor's ends too.  The mask row has
// an alignment of its own and is read one element at a time (cache hits).  x and y themselves must be 16-byte aligned.
template <typename T, int NV, int MODE, bool MASK, int LANES>
__global__ void __launch_bounds__(BLOCK) softmax_via32_span_kernel(const T* x, const T* __restrict__ mask, T* y, uint64_t rows,
                                                                   uint32_t cols, MaskArgs p) {
    const uint64_t row = (uint64_t)blockIdx.x * (BLOCK / LANES) + (threadIdx.x / LANES);
    if (row >= rows) return;
    const int lane = threadIdx.x & (LANES - 1);
    const uint64_t first = row * cols;
    const uint32_t shift = (uint32_t)(first & 7);
    const uint32_t nspan = (shift + cols + 7) >> 3;
    const v4u* xv = reinterpret_cast<const v4u*>(x) + (first >> 3);
    v4u* yv = reinterpret_cast<v4u*>(y) + (first >> 3);
    T* yrow = y + first;
    Vec16<T> v[NV];
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nspan) v[k].u = ld_stream(xv + i);
    }
    // column of element q of span vector i: i * 8 + q - shift, valid when below cols (elements before the row wrap around)
    auto column = [&](uint32_t i, int q) -> uint32_t { return i * 8 + (uint32_t)q - shift; };
    if (MASK) {
        const uint64_t mfirst = mask_row_offset<T>(row, p);
        const T* mr = mask + mfirst;
        if (p.mlast && p.mvec) {
            // The mask element of span element (i, q) sits at mask element mfirst - shift + i * 8 + q: the eight of a span
            // vector straddle two aligned mask vectors, d elements into the first (d is the same for the whole row).
            const int64_t base = (int64_t)mfirst - (int64_t)shift;
            const int64_t a0 = base >> 3;                    // floor: -1 when the row starts the mask and shift > 0
            const uint32_t d = (uint32_t)(base - a0 * 8);
            const int64_t mend = (int64_t)mfirst + cols;     // one past the row's last mask element
            const v4u* mv = reinterpret_cast<const v4u*>(mask);
#pragma unroll
            for (int k = 0; k < NV; k++) {
                const uint32_t i = lane + k * LANES;
                const int64_t a = a0 + i;
                v4u lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
                if (a >= 0 && a * 8 < mend) lo = mv[a];      // also the lane after the span: its vector may end the row's mask
                // the second vector is the first one of the next lane; the last lane of a wave loads its own
                const bool own = LANES != 64 || lane == 63;
                if (LANES == 64) {
#pragma unroll
                    for (int w = 0; w < 4; w++) hi[w] = __shfl_down(lo[w], 1, 64);
                }
                if (own) {
                    hi = v4u{0, 0, 0, 0};
                    if (d != 0 && i < nspan && (a + 1) * 8 < mend) hi = mv[a + 1];
                }
                if (i < nspan) {
                    const uint32_t cat[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    Vec16<T> mk;
                    switch (d >> 1) {                        // uniform over the wave: a branch, not a select per lane
#define RT_PICK(O)                                                                                                              \
    _Pragma("unroll") for (int w = 0; w < 4; w++)                                                                              \
        mk.u[w] = (d & 1) ? __builtin_amdgcn_alignbyte(cat[w + O + 1 < 8 ? w + O + 1 : 7], cat[w + O], 2) : cat[w + O];
                        case 0: RT_PICK(0) break;
                        case 1: RT_PICK(1) break;
                        case 2: RT_PICK(2) break;
                        default: RT_PICK(3) break;
#undef RT_PICK
                    }
#pragma unroll
                    for (int q = 0; q < 8; q++)
                        if (column(i, q) < cols) v[k].e[q] = Ar<T>::add(v[k].e[q], mk.e[q]);
                }
            }
        } else {
#pragma unroll
            for (int k = 0; k < NV; k++) {
                const uint32_t i = lane + k * LANES;
                if (i < nspan)
#pragma unroll
                    for (int q = 0; q < 8; q++) {
                        const uint32_t c = column(i, q);
                        if (c < cols) v[k].e[q] = Ar<T>::add(v[k].e[q], mr[p.mlast ? c : 0]);
                    }
            }
        }
    }
    float e[NV][8];
    float m = 0.0f;
    if (MODE == 1) {
        m = -__builtin_huge_valf();
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = lane + k * LANES;
            if (i < nspan)
#pragma unroll
                for (int q = 0; q < 8; q++)
                    if (column(i, q) < cols) m = fmaxf(m, Ar<T>::widen(v[k].e[q]));
        }
        m = row_max<LANES>(m);
        if (m == -__builtin_huge_valf()) m = 0.0f;
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
#pragma unroll
        for (int q = 0; q < 8; q++) {
            e[k][q] = 0.0f;
            if (i < nspan && column(i, q) < cols) {
                e[k][q] = via32_exp(Ar<T>::widen(v[k].e[q]) - m);
                s += e[k][q];
            }
        }
    }
    s = row_sum<LANES>(s);
    const bool plain = (s >= 1.17549435e-38f) && (s < __builtin_huge_valf());
    const float rs = 1.0f / s;
#pragma unroll
    for (int k = 0; k < NV; k++) {
        const uint32_t i = lane + k * LANES;
        if (i < nspan) {
            Vec16<T> o;
#pragma unroll
            for (int q = 0; q < 8; q++) o.e[q] = Ar<T>::conv(plain ? e[k][q] * rs : e[k][q] / s);
            if (column(i, 0) < cols && column(i, 7) < cols) {
                st_stream(yv + i, o.u);
            } else {
#pragma unroll
                for (int q = 0; q < 8; q++) {
                    const uint32_t c = column(i, q);
                    if (c < cols) yrow[c] = o.e[q];
                }
            }
        }
    }
}

// any cols / alignment: one block per row, scalar accesses, the row re-read from cache between passes
template <typename T, int MODE, bool MASK>
__global__ void __launch_bounds__(BLOCK) softmax_via32_generic_kernel(const T* __restrict__ x, const T* __restrict__ mask,
                                                                      T* __restrict__ y, uint64_t rows, uint32_t cols, MaskArgs p) {
    __shared__ float red[WAVES];
    __shared__ float bcast;
    const uint64_t row = blockIdx.x;
    const T* xr = x + row * cols;
    T* yr = y + row * cols;
    const T* mr = MASK ? mask + mask_row_offset<T>(row, p) : nullptr;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    auto elem = [&](uint32_t j) -> float {
        T v = xr[j];
        if (MASK) v = Ar<T>::add(v, mr[p.mlast ? j : 0]);
        return Ar<T>::widen(v);
    };
    float m = 0.0f;
    if (MODE == 1) {
        float lm = -__builtin_huge_valf();
        for (uint32_t j = threadIdx.x; j < cols; j += BLOCK) lm = fmaxf(lm, elem(j));
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
    for (uint32_t j = threadIdx.x; j < cols; j += BLOCK) s += expf(elem(j) - m);
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
    for (uint32_t j = threadIdx.x; j < cols; j += BLOCK) yr[j] = Ar<T>::conv(expf(elem(j) - m) / s);
}

template <typename T, int MODE, bool SPAN>
int launch_wave(rt_device* dev, const void* x, void* y, uint64_t rows, uint32_t cols, const void* mask = nullptr, uint64_t period = 1) {
    constexpr int VE = 16 / sizeof(T);
    const uint32_t nvec = SPAN ? (cols + 2 * VE - 2) / VE : cols / VE;       // SPAN: the most vectors a row can touch
    if (nvec <= 32) {
        // rows of at most 32 vectors: a group of 2..32 lanes per row (one vector each), so that a wave carries 2..32 rows
        // and as many bytes as with long rows
        const uint32_t lanes = nvec <= 2 ? 2 : nvec <= 4 ? 4 : nvec <= 8 ? 8 : nvec <= 16 ? 16 : 32;
        const uint64_t blocks = (rows + BLOCK / lanes - 1) / (BLOCK / lanes);
        RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax: too many rows");
        const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_NARROW(L) hipLaunchKernelGGL((softmax_wave_kernel<T, 1, MODE, L, SPAN>), grid, block, 0, dev->stream, (const T*)x, (T*)y, rows, cols, (const T*)mask, period)
        if (lanes == 2) RT_NARROW(2);
        else if (lanes == 4) RT_NARROW(4);
        else if (lanes == 8) RT_NARROW(8);
        else if (lanes == 16) RT_NARROW(16);
        else RT_NARROW(32);
#undef RT_NARROW
        RT_CHECK_LAUNCH("softmax_wave_kernel");
        return RT_OK;
    }
    // One wave per row up to 320 vectors (five loads per lane) in reference mode; beyond that the block shares the row,
    // so that a thread has two or three loads and stores of its own: a kernel tends to move more bytes per second the
    // fewer accesses each thread issues before it ends.  Measured cold, wave / block per row: [1,6,1500,1500] f32 (375
    // vectors) 23.2 / 21.7 us (21.8 / 20.0 by the profiler inside the benchmark step), [8192,2048] f32 25.3 / 24.7 us;
    // [4096,1280] f32 (320 vectors) 8.2 / 10.4 us the other way, and the stable mode on 16-bit rows loses with the block
    // ([65536,2560] f16 145 / 173 us), so it keeps the wave up to 512 vectors.
    constexpr uint32_t WAVE_ROW_MAX = MODE == 0 ? WAVE * 5 : WAVE * 8;
    if (nvec <= WAVE_ROW_MAX) {
        const uint32_t nv = (nvec + WAVE - 1) / WAVE;
        const uint64_t blocks = (rows + WAVES - 1) / WAVES;
        RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax: too many rows");
        const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_SM(NVC) hipLaunchKernelGGL((softmax_wave_kernel<T, NVC, MODE, WAVE, SPAN>), grid, block, 0, dev->stream, (const T*)x, (T*)y, rows, cols, (const T*)mask, period)
        if (nv <= 1) RT_SM(1);
        else if (nv <= 2) RT_SM(2);
        else if (nv <= 3) RT_SM(3);
        else if (nv <= 4) RT_SM(4);
        else if (nv <= 6) RT_SM(6);
        else RT_SM(8);
#undef RT_SM
    } else if (nvec <= (uint32_t)(BLOCK * 8)) {
        const uint32_t nv = (nvec + BLOCK - 1) / BLOCK;
        RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax: too many rows");
        const dim3 grid((unsigned)rows), block(BLOCK);
#define RT_SM(NVC) hipLaunchKernelGGL((softmax_wave_kernel<T, NVC, MODE, BLOCK, SPAN>), grid, block, 0, dev->stream, (const T*)x, (T*)y, rows, cols, (const T*)mask, period)
        if (nv <= 3) RT_SM(3);
        else if (nv <= 4) RT_SM(4);
        else if (nv <= 6) RT_SM(6);
        else RT_SM(8);
#undef RT_SM
    } else {
        const uint32_t nv = (nvec + WIDE_BLOCK - 1) / WIDE_BLOCK;
        RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax: too many rows");
        const dim3 grid((unsigned)rows), block(WIDE_BLOCK);
#define RT_SM(NVC) hipLaunchKernelGGL((softmax_wave_kernel<T, NVC, MODE, WIDE_BLOCK, SPAN>), grid, block, 0, dev->stream, (const T*)x, (T*)y, rows, cols, (const T*)mask, period)
        if (nv <= 4) RT_SM(4);
        else if (nv <= 8) RT_SM(8);
        else if constexpr (sizeof(T) == 4) {                 // (16-bit rows hold 8 values per vector: 8 vectors are the registers' limit)
            if (nv <= 13) RT_SM(13);
            else RT_SM(16);
        }
#undef RT_SM
    }
    RT_CHECK_LAUNCH("softmax_wave_kernel");
    return RT_OK;
}

template <typename T, int MODE> int launch_f32_style(rt_device* dev, const void* x, void* y, uint64_t rows, uint32_t cols) {
    constexpr int VE = 16 / sizeof(T);
    const bool aligned = rt_aligned(x, 16) && rt_aligned(y, 16);
    constexpr uint32_t MAX_VEC = WIDE_BLOCK * (sizeof(T) == 4 ? 16 : 8);     // 65536 columns
    if (aligned && cols % VE == 0 && cols / VE <= MAX_VEC) return launch_wave<T, MODE, false>(dev, x, y, rows, cols);
    // rows that are not whole vectors: over the aligned vectors that cover each row
    if (aligned && (cols + 2 * VE - 2) / VE <= MAX_VEC) return launch_wave<T, MODE, true>(dev, x, y, rows, cols);
    RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax: too many rows");
    hipLaunchKernelGGL((softmax_generic_kernel<T, MODE>), dim3((unsigned)rows), dim3(BLOCK), 0, dev->stream, (const T*)x, (T*)y, rows,
                       cols);
    RT_CHECK_LAUNCH("softmax_generic_kernel");
    return RT_OK;
}

// (rows that are not whole aligned vectors only: everything else streams.  Eight rows per block: a thousand rows of
// 1001 columns are 125 blocks, not 16)
template <typename T> int launch_seq16(rt_device* dev, const void* x, void* y, uint64_t rows, uint32_t cols) {
    constexpr int RB = 8, TC = 512;
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

template <typename T, int MODE, bool MASK>
int launch_via32(rt_device* dev, const void* x, const void* mask, void* y, uint64_t rows, uint32_t cols, const MaskArgs& p, bool mask_vec_ok) {
    const uint32_t nvec = cols / 8;
    const bool vec_ok = (cols % 8 == 0) && rt_aligned(x, 16) && rt_aligned(y, 16) && nvec <= (uint32_t)(BLOCK * 8) && (!MASK || mask_vec_ok);
    if (vec_ok && nvec <= 32) {
        // rows of at most 32 vectors: a group of 2..32 lanes per row (one vector each), so that a wave carries 2..32 rows
        // and as many bytes as with long rows
        const uint32_t lanes = nvec <= 2 ? 2 : nvec <= 4 ? 4 : nvec <= 8 ? 8 : nvec <= 16 ? 16 : 32;
        const uint64_t blocks = (rows + BLOCK / lanes - 1) / (BLOCK / lanes);
        RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax_via_f32: too many rows");
        const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_NARROW(L) hipLaunchKernelGGL((softmax_via32_wave_kernel<T, 1, MODE, MASK, L>), grid, block, 0, dev->stream, (const T*)x, (const T*)mask, (T*)y, rows, cols, p)
        if (lanes == 2) RT_NARROW(2);
        else if (lanes == 4) RT_NARROW(4);
        else if (lanes == 8) RT_NARROW(8);
        else if (lanes == 16) RT_NARROW(16);
        else RT_NARROW(32);
#undef RT_NARROW
        RT_CHECK_LAUNCH("softmax_via32_wave_kernel");
        return RT_OK;
    }
    // (beyond 320 vectors the block shares the row in reference mode, as in launch_wave: [32768,4096] f16 90.3 -> 85.1 us,
    // with a [4096,4096] mask under 32 heads 365 -> 346 us)
    if (vec_ok && nvec <= (uint32_t)(MODE == 0 ? WAVE * 5 : WAVE * 8)) {
        const uint32_t nv = (nvec + WAVE - 1) / WAVE;
        const uint64_t blocks = (rows + WAVES - 1) / WAVES;
        RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax_via_f32: too many rows");
        const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_SV(NVC)                                                                                                                 \
    hipLaunchKernelGGL((softmax_via32_wave_kernel<T, NVC, MODE, MASK, WAVE>), grid, block, 0, dev->stream, (const T*)x, (const T*)mask, \
                       (T*)y, rows, cols, p)
        if (nv <= 1) RT_SV(1);
        else if (nv <= 2) RT_SV(2);
        else if (nv <= 4) RT_SV(4);
        else if (nv <= 6) RT_SV(6);
        else RT_SV(8);
#undef RT_SV
        RT_CHECK_LAUNCH("softmax_via32_wave_kernel");
        return RT_OK;
    }
    if (vec_ok) {                                            // rows of up to 16384 columns: the block shares the row
        const uint32_t nv = (nvec + BLOCK - 1) / BLOCK;
        RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax_via_f32: too many rows");
        const dim3 grid((unsigned)rows), block(BLOCK);
#define RT_SV(NVC)                                                                                                                  \
    hipLaunchKernelGGL((softmax_via32_wave_kernel<T, NVC, MODE, MASK, BLOCK>), grid, block, 0, dev->stream, (const T*)x, (const T*)mask, \
                       (T*)y, rows, cols, p)
        if (nv <= 3) RT_SV(3);
        else if (nv <= 4) RT_SV(4);
        else if (nv <= 6) RT_SV(6);
        else RT_SV(8);
#undef RT_SV
        RT_CHECK_LAUNCH("softmax_via32_wave_kernel");
        return RT_OK;
    }
    // rows that are not whole aligned vectors, in tensors that start on a vector boundary: the span kernel
    const uint32_t span = (cols + 14) / 8;                   // vectors a row can touch at most
    if (rt_aligned(x, 16) && rt_aligned(y, 16) && span <= (uint32_t)(BLOCK * 8)) {
        if (span <= (uint32_t)(WAVE * 8)) {
            const uint32_t nv = (span + WAVE - 1) / WAVE;
            const uint64_t blocks = (rows + WAVES - 1) / WAVES;
            RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax_via_f32: too many rows");
            const dim3 grid((unsigned)blocks), block(BLOCK);
#define RT_SV(NVC)                                                                                                                 \
    hipLaunchKernelGGL((softmax_via32_span_kernel<T, NVC, MODE, MASK, WAVE>), grid, block, 0, dev->stream, (const T*)x, (const T*)mask, \
                       (T*)y, rows, cols, p)
            if (nv <= 1) RT_SV(1);
            else if (nv <= 2) RT_SV(2);
            else if (nv <= 4) RT_SV(4);
            else if (nv <= 6) RT_SV(6);
            else RT_SV(8);
#undef RT_SV
        } else {
            const uint32_t nv = (span + BLOCK - 1) / BLOCK;
            RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax_via_f32: too many rows");
            const dim3 grid((unsigned)rows), block(BLOCK);
#define RT_SV(NVC)                                                                                                                  \
    hipLaunchKernelGGL((softmax_via32_span_kernel<T, NVC, MODE, MASK, BLOCK>), grid, block, 0, dev->stream, (const T*)x, (const T*)mask, \
                       (T*)y, rows, cols, p)
            if (nv <= 3) RT_SV(3);
            else if (nv <= 4) RT_SV(4);
            else if (nv <= 6) RT_SV(6);
            else RT_SV(8);
#undef RT_SV
        }
        RT_CHECK_LAUNCH("softmax_via32_span_kernel");
        return RT_OK;
    }
    RT_REQUIRE(rows <= 0x7fffffffull, RT_ERR_SIZE, "rt_softmax_via_f32: too many rows");
    hipLaunchKernelGGL((softmax_via32_generic_kernel<T, MODE, MASK>), dim3((unsigned)rows), dim3(BLOCK), 0, dev->stream, (const T*)x,
                       (const T*)mask, (T*)y, rows, cols, p);
    RT_CHECK_LAUNCH("softmax_via32_generic_kernel");
    return RT_OK;
}

template <typename T>
int dispatch_via32(rt_device* dev, const void* x, const void* mask, void* y, uint64_t rows, uint32_t cols, const MaskArgs& p, bool mask_vec_ok,
                   int mode) {
    if (mask) {
        return mode == RT_SOFTMAX_STABLE ? launch_via32<T, 1, true>(dev, x, mask, y, rows, cols, p, mask_vec_ok)
                                         : launch_via32<T, 0, true>(dev, x, mask, y, rows, cols, p, mask_vec_ok);
    }
    return mode == RT_SOFTMAX_STABLE ? launch_via32<T, 1, false>(dev, x, mask, y, rows, cols, p, mask_vec_ok)
                                     : launch_via32<T, 0, false>(dev, x, mask, y, rows, cols, p, mask_vec_ok);
}

}  // namespace

extern "C" int rt_softmax_via_f32(rt_device* dev, int io_dt, const void* x, const uint32_t x_shape[4], const void* mask,
                                  const uint32_t mask_shape[4], void* y, int mode) {
    RT_REQUIRE(io_dt == RT_F16 || io_dt == RT_BF16, RT_ERR_DTYPE, "rt_softmax_via_f32: dtype %d is not F16/BF16", io_dt);
    RT_REQUIRE(mode == RT_SOFTMAX_REFERENCE || mode == RT_SOFTMAX_STABLE, RT_ERR_ARG, "rt_softmax_via_f32: unknown mode %d", mode);
    RT_REQUIRE(x_shape && (!mask || mask_shape), RT_ERR_NULL_POINTER, "rt_softmax_via_f32: NULL shape");
    uint64_t n = 1;
    for (int i = 0; i < 4; i++) {
        RT_REQUIRE(x_shape[i] > 0, RT_ERR_SHAPE, "rt_softmax_via_f32: zero extent in dim %d", i);
        // the add's broadcast rule with the scores as the larger side (Shape::multi_broadcast, shape.rs:118-136)
        if (mask)
            RT_REQUIRE(mask_shape[i] == 1 || mask_shape[i] == x_shape[i], RT_ERR_SHAPE,
                       "rt_softmax_via_f32: mask dim %d: %u does not broadcast to %u", i, mask_shape[i], x_shape[i]);
        n *= x_shape[i];
        RT_REQUIRE(n <= 0xffffffffull * 8, RT_ERR_SIZE, "rt_softmax_via_f32: tensor too large");
    }
    const uint32_t cols = x_shape[3];
    const uint64_t rows = n / cols;
    RT_REQUIRE(rows <= 0xffffffffull, RT_ERR_SIZE, "rt_softmax_via_f32: too many rows");
    RT_REQUIRE(x && y, RT_ERR_NULL_POINTER, "rt_softmax_via_f32: NULL operand");
    RT_REQUIRE(rt_aligned(x, 2) && rt_aligned(y, 2) && (!mask || rt_aligned(mask, 2)), RT_ERR_ALIGN, "rt_softmax_via_f32: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    MaskArgs p;
    p.d2 = make_fastdiv(x_shape[2]);
    p.d1 = make_fastdiv(x_shape[1]);
    p.ms[0] = p.ms[1] = p.ms[2] = 0;
    p.mlast = 0;
    p.mvec = mask && rt_aligned(mask, 16) ? 1u : 0u;
    p.reps = make_fastdiv(1);
    p.period = 0;
    bool mask_vec_ok = true;
    if (mask) {
        uint64_t st = 1;
        p.mlast = mask_shape[3] != 1 || cols == 1;
        st = mask_shape[3];
        for (int i = 2; i >= 0; i--) {
            RT_REQUIRE(st <= 0xffffffffull, RT_ERR_SIZE, "rt_softmax_via_f32: mask too large");
            p.ms[i] = mask_shape[i] == 1 ? 0u : (uint32_t)st;
            st *= mask_shape[i];
        }
        mask_vec_ok = !p.mlast || (rt_aligned(mask, 16) && cols % 8 == 0);
        // a mask of whole trailing dims, too large for the L2s to keep between its repeats in the plain order
        // (RT_XCD_ORDER_MIN_BYTES), repeated over the leading dims, whose period is whole groups of eight 4-row blocks: the
        // XCD-aware block order (the kernels with whole rows per block)
        int lead = 0;
        while (lead < 3 && mask_shape[lead] == 1) lead++;
        bool whole = p.mlast && lead > 0;
        uint64_t period = 1, reps = 1;
        for (int i = 0; i < 3; i++) {
            if (i < lead) reps *= x_shape[i];
            else {
                period *= x_shape[i];
                if (mask_shape[i] != x_shape[i]) whole = false;
            }
        }
        if (whole && reps > 1 && reps <= 0xffffffffull && period * cols * 2 >= RT_XCD_ORDER_MIN_BYTES && period % (WAVES * 8) == 0 &&
            rows <= 0x7fffffffull) {
            p.reps = make_fastdiv((uint32_t)reps);
            p.period = (uint32_t)period;
        }
    }
    if (io_dt == RT_F16) return dispatch_via32<half_t>(dev, x, mask, y, rows, cols, p, mask_vec_ok, mode);
    return dispatch_via32<bf16_t>(dev, x, mask, y, rows, cols, p, mask_vec_ok, mode);
}

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
        default: {
            // 16-bit types, rows that are whole aligned vectors: one pass; up to 128 columns (and enough rows to fill the chip) a lane per row, up to 4096
            // columns streamed with the row held in registers, longer ones parked in y (also small problems: the per-block table load costs about 5 us, the two-pass walker
            // more); everything else takes the two-pass tile walker
            // (rows that are not whole vectors stream over their covering vectors, with a second small launch for the
            // shared ones: measured faster than the tile walker from about 200 columns, 12.7 against 34.5 us on [4096, 1001])
            if (rt_aligned(x, 16) && rt_aligned(y, 16) && (cols % 8 == 0 || cols >= RAGGED_STREAM_MIN_COLS)) {
                if (cols % 8 == 0 && cols <= LANE_MAX_COLS && rows >= 32768) return dt == RT_F16 ? launch_lane16<half_t>(dev, x, y, rows, cols) : launch_lane16<bf16_t>(dev, x, y, rows, cols);
                bool done = false;
                if (dt == RT_F16) {                          // a few long rows (a decode step): one wave per row
                    rc = rt_softmax_replay_f16(dev, x, nullptr, 0, y, rows, cols, &done);
                    if (rc || done) return rc;
                }
                rc = dt == RT_F16 ? rt_softmax_stream_f16(dev, x, nullptr, 0, y, rows, cols, &done)
                                  : rt_softmax_stream_bf16(dev, x, nullptr, 0, y, rows, cols, &done);
                if (rc || done) return rc;
            }
            return dt == RT_F16 ? launch_seq16<half_t>(dev, x, y, rows, cols) : launch_seq16<bf16_t>(dev, x, y, rows, cols);
        }
    }
}

extern "C" int rt_softmax_masked(rt_device* dev, int dt, const void* x, const uint32_t x_shape[4], const void* mask,
                                 const uint32_t mask_shape[4], void* y, int mode) {
    RT_REQUIRE(rt_is_float_dt(dt), RT_ERR_DTYPE, "rt_softmax_masked: dtype %d is not F32/F16/BF16", dt);
    RT_REQUIRE(mode == RT_SOFTMAX_REFERENCE || mode == RT_SOFTMAX_STABLE, RT_ERR_ARG, "rt_softmax_masked: unknown mode %d", mode);
    RT_REQUIRE(x_shape && mask_shape, RT_ERR_NULL_POINTER, "rt_softmax_masked: NULL shape");
    uint64_t n = 1;
    for (int i = 0; i < 4; i++) {
        RT_REQUIRE(x_shape[i] > 0, RT_ERR_SHAPE, "rt_softmax_masked: zero extent in dim %d", i);
        // the add's broadcast rule with the scores as the larger side (Shape::multi_broadcast, shape.rs:118-136)
        RT_REQUIRE(mask_shape[i] == 1 || mask_shape[i] == x_shape[i], RT_ERR_SHAPE, "rt_softmax_masked: mask dim %d: %u does not broadcast to %u",
                   i, mask_shape[i], x_shape[i]);
        n *= x_shape[i];
        RT_REQUIRE(n <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_softmax_masked: tensor too large");
    }
    RT_REQUIRE(x && mask && y, RT_ERR_NULL_POINTER, "rt_softmax_masked: NULL operand");
    const size_t eb = (size_t)rt_dt_bytes(dt);
    RT_REQUIRE(rt_aligned(x, eb) && rt_aligned(y, eb) && rt_aligned(mask, eb), RT_ERR_ALIGN, "rt_softmax_masked: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    const uint32_t cols = x_shape[3];
    const uint64_t rows = n / cols;
    // one pass: 16-bit types, reference arithmetic, a mask that covers whole trailing dims and repeats over the leading ones
    int lead = 0;
    while (lead < 3 && mask_shape[lead] == 1) lead++;
    bool whole = mask_shape[3] == cols;
    uint64_t period = 1;
    for (int i = lead; i < 3; i++) {
        if (mask_shape[i] != x_shape[i]) whole = false;
        period *= x_shape[i];
    }
    // (rows that are not whole vectors: from RAGGED_STREAM_MIN_COLS columns, like the plain softmax)
    if (dt != RT_F32 && mode == RT_SOFTMAX_REFERENCE && whole && (cols % 8 == 0 || cols >= RAGGED_STREAM_MIN_COLS) && rt_aligned(x, 16) &&
        rt_aligned(y, 16) && rt_aligned(mask, 16)) {
        bool done = false;
        if (dt == RT_F16) {
            rc = rt_softmax_replay_f16(dev, x, mask, period, y, rows, cols, &done);
            if (rc || done) return rc;
        }
        rc = dt == RT_F16 ? rt_softmax_stream_f16(dev, x, mask, period, y, rows, cols, &done)
                          : rt_softmax_stream_bf16(dev, x, mask, period, y, rows, cols, &done);
        if (rc || done) return rc;
    }
    // f32, and the stable mode of any type: the row-in-registers kernel adds the mask as it loads (rows of whole vectors)
    if ((dt == RT_F32 || mode == RT_SOFTMAX_STABLE) && whole && rt_aligned(x, 16) && rt_aligned(y, 16) && rt_aligned(mask, 16)) {
        const uint32_t ve = 16 / (uint32_t)eb;
        const uint32_t max_vec = (uint32_t)WIDE_BLOCK * (eb == 4 ? 16 : 8);
        if (cols % ve == 0 && cols / ve <= max_vec) {
            if (mode == RT_SOFTMAX_STABLE) {
                switch (dt) {
                    case RT_F32: return launch_wave<float, 1, false>(dev, x, y, rows, cols, mask, period);
                    case RT_F16: return launch_wave<half_t, 1, false>(dev, x, y, rows, cols, mask, period);
                    default: return launch_wave<bf16_t, 1, false>(dev, x, y, rows, cols, mask, period);
                }
            }
            return launch_wave<float, 0, false>(dev, x, y, rows, cols, mask, period);
        }
    }
    // otherwise the two ops, the sum parked in y
    rc = rt_binary_bcast(dev, RT_ADD, dt, x, x_shape, mask, mask_shape, y, x_shape);
    if (rc) return rc;
    return rt_softmax(dev, dt, y, y, rows, cols, mode);
}
