// The f16 reference softmax for a few long rows (a decode step's [B * H, T] scores): one wave64 per row, the sequential
// 16-bit row sum reproduced bit for bit without walking the row.
//
// The reference (crates/ratchet-core/src/cpu/softmax.rs:22-42) adds e_j = f16(exp(x_j)) >= 0 left to right in f16:
// s <- fl16(s + e_j).  While s stays inside one binade, [2^e, 2^(e+1)), it is 2^e + k * ulp with an integer k < 1024, and
// what one add does to k depends on s only through the parity of k (round to nearest even: the parity decides ties).  A
// run of adds that stays inside the binade is therefore a function k -> k + c[k & 1] of two constants, and such functions
// compose.  Both constants come out of the adder itself: the run is added up twice, from 2^e and from 2^e + ulp (the two
// halves of one packed add), and c[p] is the distance the p-th sum has moved, read off the bit patterns.
//
// Lane i of the wave owns the contiguous run of 8 * V elements i * 8V ..:
//   1. f32 sums of the runs and their prefix over the lanes bound the running sum at the start of each run from above.
//      The f16 sum can lag behind the true one by binades (terms below half an ulp vanish), so
//   2. every lane adds its run up from the lower end of that binade and of the two below it: a pair (c[0], c[1]) per
//      binade, if both sums stay inside;
//   3. the lanes are then taken in order with the running sum t, whose bits are exact at every point: if lane i has a
//      pair for the binade t lies in, and t + c[parity] still lies in it (the sum never decreases, so every sum in
//      between does too), that is t after the run; otherwise (the first lane, a run in which the sum crosses a power
//      of two, a lag of more than two binades) every lane adds its own run to t left to right and lane i's result is
//      kept.  A row on which no pair applies costs the plain walk, 64 runs in sequence.
// (Composing the pairs of neighbouring lanes with a scan, as the 16-bit RMSNorm does for its f32 sum, does not pay here:
// the f16 sum lags the guess, so the stretches of equal guesses and the stretches the sum really spends in a binade are
// shifted against each other, and every composite ends in the lane where the sum leaves the binade.)
// The exp values come from the 65536-entry table of the exact f16 exp, which every block copies into LDS first (128 KiB:
// looked up in global memory, each 2-byte read moves a cache line into the CU, and a row of 8192 columns took 26 us for
// that alone); y = e / sum as the streaming kernel computes it.  A mask row is added in f16 as the separate add rounds it.
#include "rt_arith.h"
#include "rt_internal.h"

namespace {

constexpr int RY_BLOCK = 256;                                // four rows per block; the waves never meet
constexpr int RY_G = 2;                                      // lanes per step of the ordered pass
constexpr int RY_K = 3;                                      // binades a lane prepares for
constexpr uint32_t RY_NO_PAIR = 0x7fff7fffu;                 // in place of a pair: added to any f16 bit pattern, either half leaves the binade
typedef _Float16 ry_h2 __attribute__((ext_vector_type(2)));
typedef _Float16 ry_h8 __attribute__((ext_vector_type(8)));
typedef float ry_f2 __attribute__((ext_vector_type(2)));

// ab.lo <- fl16(ab.lo + h), ab.hi <- fl16(ab.hi + h) for the eight halves h of v, left to right: two sums in one register
#define RY_LINK(N)                                                          \
    "v_pk_add_f16 %0, %0, %" #N " op_sel:[0,0] op_sel_hi:[1,0]\n"            \
    "v_pk_add_f16 %0, %0, %" #N " op_sel:[0,1] op_sel_hi:[1,1]\n"
__device__ __forceinline__ void ry_chain(uint32_t& ab, const v4u& v) {
    asm(RY_LINK(1) RY_LINK(2) RY_LINK(3) RY_LINK(4) : "+v"(ab) : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]));
}
#undef RY_LINK

// the f32 sum of the eight halves added to acc, in any order: only a guess at the binade is taken from it
__device__ __forceinline__ float ry_rough(const v4u& v, float acc) {
    const uint32_t ones = 0x3c003c00u;
    asm("v_dot2_f32_f16 %0, %1, %5, %0\n"
        "v_dot2_f32_f16 %0, %2, %5, %0\n"
        "v_dot2_f32_f16 %0, %3, %5, %0\n"
        "v_dot2_f32_f16 %0, %4, %5, %0\n"
        : "+v"(acc)
        : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(ones));
    return acc;
}

__device__ __forceinline__ uint32_t ry_round_pair(float q0, float q1) {
    const ry_f2 q = {q0, q1};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(q, ry_h2));
}

// eight quotients e / s rounded to f16.  fast (s normal and finite): e * (1/s) with one fma correction, which is the
// correctly rounded f32 quotient there; otherwise the IEEE division, so that 0/0, x/inf and inf/inf come out as the
// reference's do.
__device__ __forceinline__ v4u ry_quotients(const v4u& ev, float s, float rinv, bool fast) {
    v4u out;
    if (fast) {
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float e0 = (float)bits_h((uint16_t)(ev[w] & 0xffffu)), e1 = (float)bits_h((uint16_t)(ev[w] >> 16));
            const float a0 = e0 * rinv, a1 = e1 * rinv;
            const float m0 = __builtin_fmaf(-s, a0, e0), m1 = __builtin_fmaf(-s, a1, e1);
            float q0 = __builtin_fmaf(m0, rinv, a0);
            float q1 = __builtin_fmaf(m1, rinv, a1);
            // the f32 quotient and its conversion stay apart: fused into one mixed-precision fma the pair would round
            // subnormal f16 results differently
            asm volatile("" : "+v"(q0), "+v"(q1));
            out[w] = ry_round_pair(q0, q1);
        }
    } else {
#pragma unroll
        for (int w = 0; w < 4; w++)
            out[w] = ry_round_pair((float)bits_h((uint16_t)(ev[w] & 0xffffu)) / s, (float)bits_h((uint16_t)(ev[w] >> 16)) / s);
    }
    return out;
}

constexpr size_t RY_LUT_BYTES = 65536 * 2;

// x, y (and mask) on 16-byte boundaries, cols a multiple of 8 and at most 512 * V.  Row r takes mask row r % period.
// A block takes rows_per_block rows (1 or 2), one per wave; the waves without a row help to copy the table and leave.
template <int V, bool MASK>
__global__ void __launch_bounds__(RY_BLOCK) softmax16_replay_kernel(const uint16_t* __restrict__ table, const half_t* __restrict__ x,
                                                                    const half_t* __restrict__ mask, uint64_t period, half_t* __restrict__ y,
                                                                    uint64_t rows, uint32_t cols, uint32_t rows_per_block) {
    extern __shared__ __attribute__((aligned(16))) uint16_t ry_lut[];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint64_t my_row = (uint64_t)blockIdx.x * rows_per_block + wave;
    const bool has_row = wave < rows_per_block && my_row < rows;
    const uint64_t row = has_row ? my_row : 0;                               // (the loads of a wave without a row go to row 0)
    const uint32_t nvec = cols / 8;
    const v4u* src = reinterpret_cast<const v4u*>(x + row * cols);
    const v4u* msk = MASK ? reinterpret_cast<const v4u*>(mask + (row % period) * cols) : nullptr;
    v4u* dst = reinterpret_cast<v4u*>(y + row * cols);
    // the lane's run: vectors lane * V .. lane * V + V - 1.  Loads and lookups are unconditional, from the row's last
    // vector where the run lies past its end, and such vectors become zeros afterwards (+0 terms change no sum)
    v4u run[V];
#pragma unroll
    for (int v = 0; v < V; v++) {
        const uint32_t i = lane * V + v;
        run[v] = ld_stream(src + (i < nvec ? i : nvec - 1));
    }
    v4u mrun[MASK ? V : 1];
    if (MASK) {
#pragma unroll
        for (int v = 0; v < V; v++) {
            const uint32_t i = lane * V + v;
            mrun[v] = msk[i < nvec ? i : nvec - 1];
        }
    }
    // table -> LDS, behind the row's loads
    {
        const v4u* tsrc = reinterpret_cast<const v4u*>(table);
        v4u* tdst = reinterpret_cast<v4u*>(ry_lut);
#pragma unroll 8
        for (uint32_t i = 0; i < RY_LUT_BYTES / 16 / RY_BLOCK; i++) tdst[i * RY_BLOCK + threadIdx.x] = tsrc[i * RY_BLOCK + threadIdx.x];
    }
    __syncthreads();
    if (!has_row) return;                                                    // a whole wave; no barrier follows
    if (MASK) {
#pragma unroll
        for (int v = 0; v < V; v++) run[v] = __builtin_bit_cast(v4u, __builtin_bit_cast(ry_h8, run[v]) + __builtin_bit_cast(ry_h8, mrun[v]));
    }
#pragma unroll
    for (int v = 0; v < V; v++) {
#pragma unroll
        for (int w = 0; w < 4; w++) run[v][w] = (uint32_t)ry_lut[run[v][w] & 0xffffu] | ((uint32_t)ry_lut[run[v][w] >> 16] << 16);
    }
#pragma unroll
    for (int v = 0; v < V; v++)
        if (lane * V + v >= nvec) run[v] = v4u{0u, 0u, 0u, 0u};

    // 1. f32 sum of the run, exclusive prefix over the lanes: the running f16 sum at the start of the run is at most that
    // (but for roundings upwards, hence the margin), and often a few binades below it
    float rough = 0.0f;
#pragma unroll
    for (int v = 0; v < V; v++) rough = ry_rough(run[v], rough);
    float upto = rough;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float t = __shfl_up(upto, o, 64);
        if (lane >= (uint32_t)o) upto += t;
    }
    float before = __shfl_up(upto, 1, 64);
    if (lane == 0) before = 0.0f;
    // 2. the run's two sums from the lower end of RY_K binades: the guessed one and the ones below it.  pair[k]: c[0] in
    // the low half, c[1] in the high half; RY_NO_PAIR when the binade is not a normal one or a sum left it (inf and NaN
    // lie beyond every binade)
    const uint32_t e32 = (f2u(before * (1.0f + 0x1p-6f)) >> 23) & 0xffu;
    const int etop = (int)e32 - 112;                                         // f16 exponent field of the guess
    uint32_t pair[RY_K];
#pragma unroll
    for (int k = 0; k < RY_K; k++) {
        const int e = etop - k;
        const bool normal = e >= 1 && e <= 30;
        const uint32_t base = (uint32_t)(normal ? e : 15) << 10;             // bit pattern of 2^e in f16
        uint32_t ab = base | ((base + 1u) << 16);
#pragma unroll
        for (int v = 0; v < V; v++) ry_chain(ab, run[v]);
        const uint32_t c0 = (ab & 0xffffu) - base, c1 = (ab >> 16) - (base + 1u);
        pair[k] = (normal && c0 < 1024u && c1 + 1u < 1024u) ? (c0 | (c1 << 16)) : RY_NO_PAIR;
    }

    // 3. the lanes in order.  tb: bit pattern of the running sum, the same in every lane and exact at every point.  A
    // lane's pair for the binade tb lies in is used when it exists and the result stays in the binade (the sum never
    // decreases, so every sum in between does too); otherwise every lane adds its own run to tb left to right and the
    // result of the lane whose turn it is, is kept.
    // c[0] in bits 0-9, c[1] in bits 10-19, the guessed exponent field from bit 20 (127, which no f16 has, without a pair)
    const uint32_t packed = pair[0] != RY_NO_PAIR ? ((pair[0] & 0x3ffu) | ((pair[0] >> 16) << 10) | ((uint32_t)etop << 20)) : (127u << 20);
    uint32_t tb = 0;
    // one lane, d its packed word: its pair for the binade tb lies in, else its run for real
    auto one_lane = [&](int i, uint32_t d) {
        const int k = (int)(d >> 20) - (int)(tb >> 10);                      // exponent field of tb; 31 for inf and NaN
        if (k >= 0 && k <= 2) {
            uint32_t c0 = d & 0x3ffu, c1 = (d >> 10) & 0x3ffu;
            if (k != 0) {
                const uint32_t p = k == 1 ? __builtin_amdgcn_readlane(pair[1], i) : __builtin_amdgcn_readlane(pair[2], i);
                c0 = p & 0xffffu;
                c1 = p >> 16;
            }
            const uint32_t next = tb + ((tb & 1u) ? c1 : c0);
            if (((next ^ tb) & 0xfc00u) == 0) {
                tb = next;
                return;
            }
        }
        uint32_t t = tb;
#pragma unroll
        for (int v = 0; v < V; v++) ry_chain(t, run[v]);
        tb = __builtin_amdgcn_readlane(t, i) & 0xffffu;
    };
    // RY_G lanes at a time without a branch in between, for the usual case that each has a pair for the guessed binade
    // itself and the sum stays in it; a lane's guess and pair travel to the scalar unit as one word, fetched while the
    // group before is decided.  (By the device's clock, on [32, 2048]: table and loads 1.4 us, lookups 1.0 us, the pairs
    // 0.7 us, this pass 4 us, of which the groups that fall back to one_lane are more than half, quotients and stores
    // 0.6 us.)
    uint32_t dn[RY_G];
#pragma unroll
    for (int j = 0; j < RY_G; j++) dn[j] = __builtin_amdgcn_readlane(packed, j);
#pragma nounroll
    for (int i = 0; i < 64; i += RY_G) {
        uint32_t d[RY_G];
        const int nx = i + RY_G < 64 ? i + RY_G : 64 - RY_G;
#pragma unroll
        for (int j = 0; j < RY_G; j++) {
            d[j] = dn[j];
            dn[j] = __builtin_amdgcn_readlane(packed, nx + j);
        }
        uint32_t t = tb, bad = 0;
#pragma unroll
        for (int j = 0; j < RY_G; j++) {
            const uint32_t c = (t & 1u) ? ((d[j] >> 10) & 0x3ffu) : (d[j] & 0x3ffu);       // the low bit of t is the parity of k
            const uint32_t next = t + c;
            bad |= ((t >> 10) ^ (d[j] >> 20)) | ((next ^ t) & 0xfc00u);      // not the guessed binade (or no pair for it), or the sum leaves it
            t = next;
        }
        if (bad == 0) {
            tb = t;
            continue;
        }
#pragma unroll
        for (int j = 0; j < RY_G; j++) one_lane(i + j, d[j]);
    }

    const float s = (float)bits_h((uint16_t)tb);
    const bool fast = (s >= 6.103515625e-05f) && (s < __builtin_huge_valf());
    const float rinv = fast ? 1.0f / s : 0.0f;
#pragma unroll
    for (int v = 0; v < V; v++) {
        const uint32_t i = lane * V + v;
        if (i < nvec) st_stream(dst + i, ry_quotients(run[v], s, rinv, fast));
    }
}

}  // namespace

// Few long rows of whole vectors in f16: at most two rows per CU (one wave each, so that no wave waits for another),
// 2048 to 8192 columns.  Measured against the streaming kernel, whose walker lane takes a row's 512-column steps one
// after the other: [32, 2048] 13.3 -> 9.4 us, [32, 4096] 22.6 -> 12.0 us, [32, 8192] 48.6 -> 20 us, [256, 2048]
// 13.5 -> 10.4 us, [256, 4096] 22.9 -> 14.3 us; rows of 1024 columns lose (8.8 -> 10 us: the ordered pass costs 4 us
// whatever the row length), and from four rows per CU the streaming kernel's overlap wins.
// Returns RT_OK with *done = false when the shape does not fit.
int rt_softmax_replay_f16(rt_device* dev, const void* x, const void* mask, uint64_t period, void* y, uint64_t rows, uint32_t cols, bool* done) {
    *done = false;
    constexpr uint32_t MAX_RPB = 2;
    if (cols % 8 != 0 || cols < 2048 || cols > 8192 || rows == 0 || rows > (uint64_t)MAX_RPB * (uint64_t)dev->num_cus) return RT_OK;
    if (!rt_aligned(x, 16) || !rt_aligned(y, 16) || (mask && !rt_aligned(mask, 16))) return RT_OK;
    // the exp table is built on first use, which synchronises: not while a graph is being captured
    if (dev->capturing && !dev->unary_lut[0][RT_EXP]) return RT_OK;
    const uint16_t* table = nullptr;
    int rc = rt_unary_table(dev, 0, RT_EXP, &table);
    if (rc) return rc;
    if (!mask) period = 1;
    // as few rows per block as keep the blocks within one per CU: every block copies the table, a row per CU runs alone
    const uint32_t rpb = (uint32_t)((rows + dev->num_cus - 1) / dev->num_cus);
    const dim3 grid((unsigned)((rows + rpb - 1) / rpb)), block(RY_BLOCK);
#define RT_RY1(VC, M, BIT)                                                                                                        \
    do {                                                                                                                          \
        if (!(dev->ry_attr_set & (1u << (BIT)))) {           /* the LDS opt-in is per function and per device */                  \
            RT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(softmax16_replay_kernel<VC, M>),                             \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)RY_LUT_BYTES));                           \
            dev->ry_attr_set |= 1u << (BIT);                                                                                      \
        }                                                                                                                         \
        hipLaunchKernelGGL((softmax16_replay_kernel<VC, M>), grid, block, RY_LUT_BYTES, dev->stream, table, (const half_t*)x,     \
                           (const half_t*)mask, period, (half_t*)y, rows, cols, rpb);                                             \
    } while (0)
#define RT_RY(VC, BIT)                                                                                                            \
    do {                                                                                                                          \
        if (mask) RT_RY1(VC, true, 2 * (BIT) + 1);                                                                                \
        else RT_RY1(VC, false, 2 * (BIT));                                                                                        \
    } while (0)
    const uint32_t v = (cols / 8 + 63) / 64;                 // vectors per lane
    if (v <= 2) RT_RY(2, 0);
    else if (v <= 4) RT_RY(4, 1);
    else if (v <= 8) RT_RY(8, 2);
    else RT_RY(16, 3);
#undef RT_RY
#undef RT_RY1
    RT_CHECK_LAUNCH("softmax16_replay_kernel");
    *done = true;
    return RT_OK;
}
