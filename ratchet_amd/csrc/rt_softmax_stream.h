// The streaming 16-bit softmax (f16 / bf16 reference arithmetic in one pass over HBM), its launcher and the second launch
// of its ragged-row variant.  Included by one translation unit per element type (rt_softmax_stream_f16.hip,
// rt_softmax_stream_bf16.hip): the kernel has some sixty instantiations per type, and the two compile side by side.
#ifndef RT_SOFTMAX_STREAM_H
#define RT_SOFTMAX_STREAM_H

#include "rt_arith.h"
#include "rt_internal.h"
#include "rt_pace.h"

namespace {

constexpr int BLOCK = 256;

// ------------------------------------------------------------------------------------------------------------------
// 16-bit reference arithmetic (f16, bf16), single pass over HBM (cols % 8 == 0, 16-byte aligned; the description is of
// the variant for rows of at most 4096 columns, whose differences from the long-row variant are stated at the kernel).
//
// One 1024-thread block per CU walks over groups of 30 rows.  Wave 0 does nothing but the sequential sums; loader wave
// w = 1..15 owns rows w-1 and w+14 of the group: in step t its 64 lanes cover the 1 KiB at columns t*512 .. t*512+511 of
// each of the two rows (one fully contiguous 1 KiB per load instruction), and keep the exp values in registers
// (NSTEP * 8 VGPRs) until the row sum is known, so x is read once and y written once.
//   exp: a 16-bit type has 65536 values; the whole exact exp table (128 KiB) sits in LDS next to the 31 KiB tile
//        (162 400 of the CU's 163 840 bytes), so exp is one ds_read_u16 per element with the bit pattern as the index:
//        no range clamping, no NaN special case.
//   sum: per 512-column step the exp values also go to an LDS tile; lanes 0..29 of wave 0 each walk one row of the
//        tile left to right with dependent v_add_f16 (3 ns each on this chip with the LDS reads the wave issues in
//        between, 1.5 us per step; bf16: v_add_f32 and v_cvt_pk_bf16_f32 into the high half of a word, two dependent
//        instructions and one that moves the operand into place, 5 ns).  The tile is single
//        buffered with two barriers per step: the loaders look up step t+1 into registers and divide / store the
//        previous group's step t while wave 0 walks step t, and only the short LDS write of the tile sits between the
//        barriers with wave 0 idle.  A step is 30 KiB in and 30 KiB out of HBM per CU, about 2 us at a CU's share of
//        8 TB/s, so the walk stays hidden; wave 0 is kept free of any other work and raises its issue priority.
//   divide: the outputs of group g are produced while group g+1 streams in: y = e / sum with the quotient computed as
//        q0 = e * (1/sum) plus one fma correction, which is the correctly rounded f16 quotient for normal finite sums
//        (checked against IEEE division over operand pairs on the GPU); other sums, and bf16, take the IEEE path.
//   mask: with MASK, a second operand (one [P, cols] block shared by every period of P rows, e.g. an [S, T] attention
//        mask under B * H heads) is added to x in the 16-bit type as the vectors arrive: scores.add(mask).softmax() without the sum
//        ever reaching memory, bit-identical to the two separate ops.
// Global loads run SP_PF steps ahead across group boundaries, so the pipeline never drains.
// ------------------------------------------------------------------------------------------------------------------
constexpr int SP_BLOCK = 1024;
constexpr int SP_ROWS = 30;                  // 15 loader waves x 2 rows each; wave 0 only walks
constexpr int SP_HALF = SP_ROWS / 2;
constexpr int SP_TC = 512;                   // columns per step: 64 lanes x 8 halves
constexpr int SP_PAD = 8;
constexpr int SP_PF = 2;                     // steps loaded ahead
constexpr int SP_MAX_STEPS = 8;              // rows of up to 4096 columns
constexpr size_t SP_LUT_BYTES = 65536 * sizeof(uint16_t);
constexpr size_t SP_TILE_BYTES = SP_ROWS * (SP_TC + SP_PAD) * sizeof(uint16_t);
constexpr size_t SP_SMEM_BYTES = SP_LUT_BYTES + SP_TILE_BYTES + 2 * 32 * sizeof(uint16_t);      // 162 400 of the CU's 163 840 bytes

typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 h16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// exp of two packed f16 bit patterns: two lookups in the full 65536-entry table (NaN, inf and the saturated ends included)
__device__ __forceinline__ uint32_t sp_exp_pair(const uint16_t* lut, uint32_t p) {
    return (uint32_t)lut[p & 0xffffu] | ((uint32_t)lut[p >> 16] << 16);
}

// Which 30-row groups a block works on.  Rows come in `reps` periods of P rows (P = all rows when nothing repeats; P = the
// rows one mask covers when a mask is added, e.g. S rows per head for an [S, T] mask under B * H heads); a period holds
// GP = ceil(P / 30) groups, none of which straddles two periods.  Item w = block + i * grid -> (rep, group) = (w / GP, w % GP):
// the blocks running at one time work on one contiguous window of x.  (An order that put all heads of one mask slab on one
// XCD, as the broadcast add does, was measured slower here, 461 against 441 us on [1,32,4096,4096]: thirty-two streams
// 32 MiB apart collide in the memory channels, and the mask re-reads it saves are served by the Infinity Cache anyway.
// Orders in between, where the 32 blocks of an XCD work on the same 32 / h groups of h periods at one time so that the
// mask rows they share stay in that XCD's L2, change nothing for h = 1, 2 and lose for h = 4 (+1 %), 8 (+9 %), 32 (+4 %).)
struct SpSched {
    uint32_t P, GP, reps;
    uint32_t R;              // rows per group actually used (<= SP_ROWS): chosen so that the groups fill whole rounds of the grid
    uint32_t nsteps;         // 512-column steps per row, rounded up to an even number (used by the long-row variant)
    FastDiv gp_div;
    FastDiv pm_div;          // rows of the mask: row (rep * P + r) of x takes mask row (rep * P + r) % PM.  PM == P unless the
    uint32_t PM;             // mask is only a few rows tall, where groups that stop at every period would be nearly empty
    uint32_t tile_stride;    // words per mask row in the table of tile classes (the steps of a row); 0: no table, every tile is loaded
    uint32_t item_reps;      // periods in units of items: reps, or ceil(reps / 2) when a loader wave's two rows are one row of two periods
    uint32_t pace;           // shortest time between two steps of a block, in ticks of the device's wall clock (100 MHz); 0: unpaced
    uint32_t phase_fx;       // pace / grid in 16.16 fixed point: block b takes its steps b * pace / grid ticks after block 0
};

__device__ __forceinline__ uint32_t sp_item_count(const SpSched& s, uint32_t b, uint32_t G) {
    const uint32_t total = s.GP * s.item_reps;
    return b < total ? (total - b + G - 1) / G : 0;
}
__device__ __forceinline__ void sp_item(const SpSched& s, uint32_t b, uint32_t G, uint32_t it, uint32_t& rep, uint32_t& pg) {
    fd_divmod(b + it * G, s.gp_div, rep, pg);
}

// What differs between the two 16-bit types: the walker's running sum and how a packed pair is divided by the row sum.
template <typename T> struct SpType;
template <> struct SpType<half_t> {
    typedef half_t Run;
    static __device__ __forceinline__ Run zero() { return (half_t)0.0f; }
    static __device__ __forceinline__ void add_pair(Run& run, uint32_t w) {        // two dependent v_add_f16
        run = run + bits_h((uint16_t)(w & 0xffffu));
        run = run + bits_h((uint16_t)(w >> 16));
    }
    static __device__ __forceinline__ uint16_t run_bits(Run run) { return h_bits(run); }
    static __device__ __forceinline__ float widen_bits(uint32_t b) { return (float)bits_h((uint16_t)b); }
    static __device__ __forceinline__ uint32_t round_pair(float q0, float q1) {
        const f32x2 q = {q0, q1};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(q, h16x2));
    }
    static __device__ __forceinline__ v4u add_vec(const v4u& a, const v4u& b) {    // eight f16 sums, rounded as the separate add does
        return __builtin_bit_cast(v4u, __builtin_bit_cast(h16x8, a) + __builtin_bit_cast(h16x8, b));
    }
    static constexpr bool SHORT_DIVISION = true;
    static constexpr bool CHUNK_ASM = false;                                      // the walker adds pair by pair
    static constexpr uint32_t NEG_INF_PAIR = 0xfc00fc00u;                         // two -inf
};
template <> struct SpType<bf16_t> {
    typedef float Run;                                                            // always a bf16 value, held widened
    static __device__ __forceinline__ Run zero() { return 0.0f; }
    // two f32 values rounded to bf16 (nearest even) and packed, low half first: one instruction on this chip
    static __device__ __forceinline__ uint32_t cvt_pk(float lo, float hi) {
        uint32_t r;
        asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
        return r;
    }
    // bf16(a + b), held widened: converting into the high half of a word whose low half is bf16(0) = 0 gives the f32
    // form of the rounded sum directly, so a link of the walker's chain is two dependent instructions
    static __device__ __forceinline__ float add_round(float a, float b) {
        const float s = a + b;
        uint32_t r;
        asm("v_cvt_pk_bf16_f32 %0, 0, %1" : "=v"(r) : "v"(s));
        return u2f(r);
    }
    static __device__ __forceinline__ void add_pair(Run& run, uint32_t w) {
        run = add_round(run, u2f(w << 16));
        run = add_round(run, u2f(w & 0xffff0000u));
    }
    // sixteen values, left to right, as one asm statement (between separate statements the compiler, which cannot see
    // into them, puts wait states): per value the operand is moved to the top of a word, added, and the sum rounded
#define SP_BF_LINK(N)                                                                                               \
    "v_lshlrev_b32 %1, 16, %" #N "\n v_add_f32 %0, %0, %1\n v_cvt_pk_bf16_f32 %0, 0, %0\n"                           \
    "v_and_b32 %1, 0xffff0000, %" #N "\n v_add_f32 %0, %0, %1\n v_cvt_pk_bf16_f32 %0, 0, %0\n"
    static __device__ __forceinline__ void add_chunk(Run& run, const v4u& c0, const v4u& c1) {
        uint32_t t;
        asm(SP_BF_LINK(2) SP_BF_LINK(3) SP_BF_LINK(4) SP_BF_LINK(5) SP_BF_LINK(6) SP_BF_LINK(7) SP_BF_LINK(8) SP_BF_LINK(9)
            : "+v"(run), "=&v"(t)
            : "v"(c0[0]), "v"(c0[1]), "v"(c0[2]), "v"(c0[3]), "v"(c1[0]), "v"(c1[1]), "v"(c1[2]), "v"(c1[3]));
    }
#undef SP_BF_LINK
    static __device__ __forceinline__ uint16_t run_bits(Run run) { return (uint16_t)(f2u(run) >> 16); }
    static __device__ __forceinline__ float widen_bits(uint32_t b) { return u2f(b << 16); }
    static __device__ __forceinline__ uint32_t round_pair(float q0, float q1) { return cvt_pk(q0, q1); }
    static __device__ __forceinline__ v4u add_vec(const v4u& a, const v4u& b) {
        v4u r;
#pragma unroll
        for (int w = 0; w < 4; w++)
            r[w] = cvt_pk(u2f(a[w] << 16) + u2f(b[w] << 16), u2f(a[w] & 0xffff0000u) + u2f(b[w] & 0xffff0000u));
        return r;
    }
    static constexpr uint32_t NEG_INF_PAIR = 0xff80ff80u;
    static constexpr bool SHORT_DIVISION = false;                                 // the quotient's range is f32's: always the IEEE division
    static constexpr bool CHUNK_ASM = true;                                       // the walker adds sixteen values per asm statement (add_chunk)
};

// NSTEP > 0: rows of up to NSTEP * 512 columns, exp values parked in registers.  NSTEP == 0: longer rows; the exp values
// are parked in y instead and read back (by the thread that wrote them) when the row sum is known: 4 bytes of traffic per
// element and byte of the type instead of 2, any row length.
//
// RAGGED (rows that are not whole aligned vectors, e.g. 1001 columns; x and y 16-byte aligned, no mask, parked variant):
// every row is handled over the span of aligned 16-byte vectors that covers it.  Row r starts `sh` = (r * cols * 2) % 16
// bytes into its first vector; span elements outside the row belong to the neighbouring rows: they are zeroed after the
// table lookup (adding +0 leaves the running sum as it is), and a vector that is not entirely inside its row is not
// stored.  Wave 0 also writes each row's sum to `row_sums`; the elements of those ragged vectors (at most 14 per row) are
// finished by softmax16_edges_kernel from x, the table and that sum.  An aligned vector that holds one byte of the tensor
// lies in a mapped page, so the loads are safe at the tensor's ends too.  A row's span can be one vector longer than
// NSTEP steps hold (2047 columns starting 14 bytes into a vector): wave 0 reads that vector itself and adds it last.
template <typename T, int NSTEP, bool FULL, int MASK, bool RAGGED = false>
__global__ void __launch_bounds__(SP_BLOCK) softmax16_stream_kernel(const uint16_t* __restrict__ table, const T* x, const T* mask, T* y,
                                                                    uint64_t rows, uint32_t cols, SpSched sch, uint16_t* row_sums,
                                                                    const uint32_t* __restrict__ tiles) {
    typedef SpType<T> ST;
    constexpr bool PARK = NSTEP > 0;
    // The plain variant and the paired masked one hold their steps to a pace (see launch_stream16).  The paired one does
    // not get faster by it where the output lies well relative to the input in physical memory (372 against 374 us on
    // [1,32,4096,4096]), but it no longer loses 13 us where it does not: unpaced, its time depends on one bit of the
    // memory channel hash in which the two buffers' pages agree or differ.  The unpaired masked variant loses at every
    // pace tried and the ragged ones take longer per step than the pace by themselves, so for them it is compiled out.
    constexpr bool PACED = MASK != 1 && !RAGGED;
    // MASK == 2: the two rows of a loader wave are the same row of two neighbouring periods (two heads under one [S, T]
    // mask), so one mask vector serves both and the register of the second holds the mask of the step after next
    constexpr bool PAIR = MASK == 2;
    static_assert(!RAGGED || (PARK && !FULL), "the ragged variant parks in registers and has no full-step shortcut");
    static_assert(!PAIR || (PARK && !RAGGED && NSTEP % 2 == 0), "the paired variant parks in registers and alternates two mask slots");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint16_t* lut = reinterpret_cast<uint16_t*>(smem);
    uint16_t (*tile)[SP_TC + SP_PAD] = reinterpret_cast<uint16_t (*)[SP_TC + SP_PAD]>(smem + SP_LUT_BYTES);
    uint16_t (*sums)[32] = reinterpret_cast<uint16_t (*)[32]>(smem + SP_LUT_BYTES + SP_TILE_BYTES);

    // table -> LDS
    {
        const v4u* src = reinterpret_cast<const v4u*>(table);
        v4u* dst = reinterpret_cast<v4u*>(lut);
#pragma unroll
        for (uint32_t i = 0; i < SP_LUT_BYTES / 16 / SP_BLOCK; i++) dst[i * SP_BLOCK + threadIdx.x] = src[i * SP_BLOCK + threadIdx.x];
    }
    const uint32_t n_items = sp_item_count(sch, blockIdx.x, gridDim.x);
    const uint32_t nsteps = PARK ? (uint32_t)NSTEP : sch.nsteps;
    __syncthreads();                                         // table visible

    // Every wave passes the same barriers: two per step (A: the walk of the previous tile is over, the tile may be
    // overwritten; B: the new tile is complete) and one after the block's last group.
    if (threadIdx.x < 64) {
        // ------------------------------------------------------------------ wave 0: the walk, nothing else
        __builtin_amdgcn_s_setprio(3);
        const uint32_t lane = threadIdx.x;
        const uint32_t wr = lane < SP_ROWS ? lane : 0;       // lanes 30..63 shadow row 0 and never publish
        const v4u* trow = reinterpret_cast<const v4u*>(tile[wr]);
        typename ST::Run run = ST::zero();
        uint32_t gpar = 0;
        // the blocks take their steps out of phase with each other: block b starts b / grid of a step late
        uint32_t t_step = 0, t_last = 0, t_avg = sch.pace, t_slow = sch.pace + sch.pace / 5;
        if constexpr (PACED) {
            t_last = __builtin_amdgcn_readfirstlane(rt_pace_clock());
            t_step = t_last - sch.pace + ((blockIdx.x * sch.phase_fx) >> 16);
            t_last -= sch.pace;
        }
        for (uint32_t it = 0; it < n_items; it++) {
            // RAGGED: a row that starts sh bytes into its first vector can reach up to 14 bytes past its last step.  That
            // one vector is fetched here, at the start of the group, and added after the group's last step.
            uint32_t my_row = 0, tail_end = 0;               // tail_end: bytes of the row inside the extra vector, 0 = none
            bool my_ok = false;
            v4u tailv = {0, 0, 0, 0}, tailm = {0, 0, 0, 0};
            if (RAGGED) {
                uint32_t rep, pg;
                sp_item(sch, blockIdx.x, gridDim.x, it, rep, pg);
                const uint32_t prow = pg * sch.R + lane;
                my_ok = lane < sch.R && prow < sch.P;
                my_row = rep * sch.P + prow;
                const uint32_t off = my_row * (cols * 2);
                const uint32_t end = (off & 15u) + cols * 2; // one past the row's last byte, in span coordinates
                if (my_ok && end > nsteps * (SP_TC * 2)) {
                    tail_end = end - nsteps * (SP_TC * 2);
                    tailv = *reinterpret_cast<const v4u*>(reinterpret_cast<const char*>(x) + (off & ~15u) + nsteps * (SP_TC * 2));
                    if (MASK) {                              // its mask elements, one by one (the mask row has its own alignment)
                        uint32_t q, mrow;
                        fd_divmod(my_row, sch.pm_div, q, mrow);
                        const uint16_t* mp = reinterpret_cast<const uint16_t*>(mask) + (uint64_t)mrow * cols + (nsteps * (SP_TC * 2) - (off & 15u)) / 2;
#pragma unroll
                        for (int e = 0; e < 7; e++)
                            if ((uint32_t)(2 * e) < tail_end) tailm[e >> 1] |= (uint32_t)mp[e] << (16 * (e & 1));
                    }
                }
            }
#pragma unroll 1
            for (uint32_t t = 0; t < nsteps; t++) {
                if (PACED && sch.pace) rt_pace_step(t_step, t_last, t_avg, sch.pace, t_slow);   // the walker is the block's clock
                __syncthreads();                             // A
                __syncthreads();                             // B: tile t is in LDS
                // 16 values per chunk; the LDS reads of the next chunk are in flight during the 16 dependent adds
                v4u c0 = trow[0], c1 = trow[1];
#pragma unroll
                for (int c = 0; c < SP_TC / 16; c++) {
                    v4u n0 = c0, n1 = c1;
                    if (c + 1 < SP_TC / 16) {
                        n0 = trow[(c + 1) * 2];
                        n1 = trow[(c + 1) * 2 + 1];
                    }
                    if constexpr (ST::CHUNK_ASM) {
                        ST::add_chunk(run, c0, c1);
                    } else {
#pragma unroll
                        for (int w = 0; w < 4; w++) ST::add_pair(run, c0[w]);
#pragma unroll
                        for (int w = 0; w < 4; w++) ST::add_pair(run, c1[w]);
                    }
                    c0 = n0;
                    c1 = n1;
                }
            }
            if (RAGGED && tail_end) {
                if (MASK) tailv = ST::add_vec(tailv, tailm);
#pragma unroll
                for (int w = 0; w < 4; w++) {                // elements past the row's end count as +0
                    const uint32_t keep = ((uint32_t)(4 * w) < tail_end ? 0xffffu : 0u) | ((uint32_t)(4 * w + 2) < tail_end ? 0xffff0000u : 0u);
                    ST::add_pair(run, sp_exp_pair(lut, tailv[w]) & keep);
                }
            }
            if (lane < SP_ROWS) sums[gpar][lane] = ST::run_bits(run);
            if (RAGGED && my_ok) row_sums[my_row] = ST::run_bits(run);
            run = ST::zero();
            gpar ^= 1;
        }
        __syncthreads();                                     // after the last group: its sums are published
        return;
    }

    // ---------------------------------------------------------------------- waves 1..15: load, exp, park, divide, store
    // Global accesses are raw buffer loads / stores: an access whose target does not exist (rows past the end, columns
    // past a short row, the store of "the previous group" during the first one) gets an offset outside the buffer and
    // the hardware drops it.  That keeps the loop free of branches around memory instructions, so the compiler can
    // count exactly how many of them may stay in flight at each wait (with branches it waits for all of them, the
    // store issued a moment ago included, and the prefetch distance collapses).
    const uint32_t lt = threadIdx.x - 64;                    // 0..959
    const uint32_t rr = __builtin_amdgcn_readfirstlane(lt >> 6);   // rows rr and rr + 15 of the group: the same for the whole wave
    const uint32_t ccol = (lt & 63) * 8;                     // column of this thread's vectors inside a step
    const uint32_t row_bytes = cols * 2;
    // the launcher keeps this below 2^31; the ragged variant's last vector may reach past the tensor's last element
    const uint32_t nbytes = RAGGED ? (uint32_t)((rows * row_bytes + 15) & ~15ull) : (uint32_t)(rows * row_bytes);
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(x), 0, nbytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(y, 0, nbytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rm =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(MASK ? mask : x), 0,
                                          MASK ? (RAGGED ? (sch.PM * row_bytes + 15) & ~15u : sch.PM * row_bytes) : nbytes, 0x00020000);
    constexpr uint32_t OOB = 0x80000000u;                    // >= nbytes, and stays so after adding a column offset
    const uint32_t G = gridDim.x;

    // Row offsets are the same for all lanes of a wave, so they live in scalar registers (the vector registers are all
    // needed for data): byte offset of rows rr / rr + 15 of item `it` in x / y, or OOB, and the difference between that
    // and the row's offset in the mask (for a row that does not exist the mask offset is arbitrary, which is harmless:
    // the load is range checked, and what is computed from it is never stored).
    // (RAGGED: xo is the offset of the row's first span vector and mdiff carries sh, the row's start inside that vector)
    // (RAGGED with MASK: mq is the mask byte that lines up with the row's span origin, mask row offset minus sh; it is only
    // element aligned, and negative for the mask's first row when sh > 0)
    // With a mask, register-parked rows of whole vectors: the classes of the NSTEP tiles of each of the wave's mask rows
    // (one row when paired), in scalar registers (see mask_tiles_kernel)
    constexpr bool TILES = MASK && PARK && !RAGGED;
    constexpr int NCLS = TILES ? NSTEP : 1, NCROW = PAIR ? 1 : 2;
    auto item_tiles = [&](uint32_t it, uint32_t (&cw)[NCROW][NCLS]) {
        if constexpr (TILES) {
            if (sch.tile_stride == 0) {                      // no table for this launch: every tile is loaded
#pragma unroll
                for (int h = 0; h < NCROW; h++)
#pragma unroll
                    for (int t = 0; t < NCLS; t++) cw[h][t] = 0xffffffffu;
                return;
            }
            uint32_t rep, pg;
            sp_item(sch, blockIdx.x, G, it, rep, pg);
#pragma unroll
            for (int h = 0; h < NCROW; h++) {
                const uint32_t r = PAIR ? rr : rr + h * SP_HALF;
                const uint32_t prow = pg * sch.R + r;
                const bool ok = it < n_items && r < sch.R && prow < sch.P && sch.tile_stride != 0;
                uint32_t q, mrow;
                fd_divmod((PAIR ? rep * 2 : rep) * sch.P + prow, sch.pm_div, q, mrow);
                const uint32_t base = __builtin_amdgcn_readfirstlane(ok ? (uint32_t)RT_SM_TILES_HEAD + mrow * sch.tile_stride : 0u);
#pragma unroll
                for (int t = 0; t < NCLS; t++) cw[h][t] = __builtin_amdgcn_readfirstlane(tiles[base + t]);
            }
        }
    };
    auto item_off = [&](uint32_t it, uint32_t (&xo)[2], uint32_t (&mdiff)[2], uint32_t (&mq)[2]) {
        uint32_t rep, pg;
        sp_item(sch, blockIdx.x, G, it, rep, pg);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t r = PAIR ? rr : rr + h * SP_HALF;
            const uint32_t prow = pg * sch.R + r;            // row inside the period
            const uint32_t per = PAIR ? rep * 2 + h : rep;
            const bool ok = it < n_items && r < sch.R && prow < sch.P && per < sch.reps;
            const uint32_t row = per * sch.P + prow;
            mq[h] = 0;
            if (RAGGED) {
                xo[h] = __builtin_amdgcn_readfirstlane(ok ? (row * row_bytes) & ~15u : OOB);
                mdiff[h] = __builtin_amdgcn_readfirstlane((row * row_bytes) & 15u);
                if (MASK) {
                    uint32_t q, mrow;
                    fd_divmod(row, sch.pm_div, q, mrow);
                    mq[h] = __builtin_amdgcn_readfirstlane(mrow * row_bytes - ((row * row_bytes) & 15u));
                }
                continue;
            }
            xo[h] = __builtin_amdgcn_readfirstlane(ok ? row * row_bytes : OOB);
            if (MASK) {
                uint32_t q, mrow;
                fd_divmod(row, sch.pm_div, q, mrow);
                mdiff[h] = __builtin_amdgcn_readfirstlane((row - mrow) * row_bytes);
            } else {
                mdiff[h] = 0;
            }
        }
    };
    const uint32_t cbyte = ccol * 2;
    auto past_end = [&](uint32_t t) -> bool { return !(PARK && FULL) && t * SP_TC + ccol >= cols; };
    auto step_off = [&](uint32_t row_off, uint32_t t) -> uint32_t {   // per-lane offset of this thread's vector in step t of a row
        if (past_end(t)) return OOB;
        return row_off + t * (SP_TC * 2) + cbyte;
    };
    // RAGGED: the same in span coordinates.  The vector at span byte p holds row bytes [sh, sh + row_bytes) ∩ [p, p + 16).
    auto span_load_off = [&](uint32_t row_off, uint32_t sh, uint32_t t) -> uint32_t {
        const uint32_t p = t * (SP_TC * 2) + cbyte;
        return p >= sh + row_bytes ? OOB : row_off + p;
    };
    auto span_store_off = [&](uint32_t row_off, uint32_t sh, uint32_t t) -> uint32_t {     // only vectors entirely inside the row
        const uint32_t p = t * (SP_TC * 2) + cbyte;
        return (p >= sh && p + 16 <= sh + row_bytes) ? row_off + p : OOB;
    };
    auto ld_off = [&](uint32_t row_off, uint32_t sh, uint32_t t) -> uint32_t { return RAGGED ? span_load_off(row_off, sh, t) : step_off(row_off, t); };
    auto st_off = [&](uint32_t row_off, uint32_t sh, uint32_t t) -> uint32_t { return RAGGED ? span_store_off(row_off, sh, t) : step_off(row_off, t); };
    // RAGGED with MASK: the sixteen mask bytes for the vector at span byte p start at mask byte mq + p, which is only
    // element aligned: they straddle the aligned mask vectors at (mq & ~15) + p and 16 bytes on, (mq & 15) bytes into the
    // first.  A lane loads the first; the second is its right neighbour's first (one wave shift), except for lane 63,
    // which loads its own.  An offset before the mask's start wraps to a huge one and is dropped like any other.
    auto mask_lo_off = [&](uint32_t mq, uint32_t sh, uint32_t t) -> uint32_t {
        const uint32_t p = t * (SP_TC * 2) + cbyte;
        return p >= sh + row_bytes + 16 ? OOB : (mq & ~15u) + p;      // also the lane after the row's last vector: it feeds its left neighbour
    };
    auto mask_hi_off = [&](uint32_t mq, uint32_t sh, uint32_t t) -> uint32_t {
        const uint32_t p = t * (SP_TC * 2) + cbyte;
        return (cbyte != 63 * 16 || p >= sh + row_bytes) ? OOB : (mq & ~15u) + p + 16;
    };
    auto mask_funnel = [&](const v4u& lo, const v4u& hi_own, uint32_t mq) -> v4u {
        const uint32_t d = mq & 15u;                         // the same for the whole wave: branches, not selects
        uint32_t cat[8];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            cat[w] = lo[w];
            // lane i takes lane i + 1's value; lane 63 keeps the vector it loaded itself
            cat[w + 4] = (uint32_t)__builtin_amdgcn_update_dpp((int)hi_own[w], (int)lo[w], 0x130, 0xf, 0xf, false);
        }
        v4u out;
        switch (d >> 2) {
#define RT_PICK(O)                                                                                                              \
    _Pragma("unroll") for (int w = 0; w < 4; w++)                                                                              \
        out[w] = (d & 2) ? __builtin_amdgcn_alignbyte(cat[w + O + 1 < 8 ? w + O + 1 : 7], cat[w + O], 2) : cat[w + O];
            case 0: RT_PICK(0) break;
            case 1: RT_PICK(1) break;
            case 2: RT_PICK(2) break;
            default: RT_PICK(3) break;
#undef RT_PICK
        }
        return out;
    };
    auto load_x = [&](uint32_t off) -> v4u { return __builtin_amdgcn_raw_buffer_load_b128(rx, off, 0, 2); };   // 2: non-temporal
    auto load_m = [&](uint32_t off) -> v4u { return __builtin_amdgcn_raw_buffer_load_b128(rm, off, 0, 0); };   // re-read by other heads
    // A mask tile whose elements are all equal is not loaded (the offset goes outside the buffer, which costs no memory
    // access and returns zeros) and its value is put in place of those zeros when the vector is used; cw is the tile's
    // class word
    constexpr uint32_t TILE_MIXED = 0xffffffffu;
    auto load_m_tile = [&](uint32_t off, uint32_t cw) -> v4u {
        const uint32_t skip = __builtin_amdgcn_readfirstlane(cw != TILE_MIXED ? OOB : 0u);
        return load_m(off | skip);
    };
    auto tile_value = [&](const v4u& loaded, uint32_t cw) -> v4u {
        const uint32_t fill = __builtin_amdgcn_readfirstlane(cw != TILE_MIXED ? cw : 0u);
        return v4u{loaded[0] | fill, loaded[1] | fill, loaded[2] | fill, loaded[3] | fill};
    };
    auto load_y = [&](uint32_t off) -> v4u { return __builtin_amdgcn_raw_buffer_load_b128(ry, off, 0, 0); };
    auto store_y = [&](const v4u& v, uint32_t off) { __builtin_amdgcn_raw_buffer_store_b128(v, ry, off, 0, 2); };      // results: non-temporal
    auto store_park = [&](const v4u& v, uint32_t off) { __builtin_amdgcn_raw_buffer_store_b128(v, ry, off, 0, 0); };   // read back soon

    // sum of the previous group's rows, reciprocal, and whether the short division applies: wave-uniform as well
    float s_prev[2] = {1.0f, 1.0f}, rinv_prev[2] = {1.0f, 1.0f};
    bool fast_prev[2] = {true, true};

    auto quotients = [&](const v4u& ev, int h) -> v4u {      // e / sum of the previous group
        v4u out;
        const float s = s_prev[h], rinv = rinv_prev[h];
        if (ST::SHORT_DIVISION && fast_prev[h]) {
#pragma unroll
            for (int w = 0; w < 4; w++) {
                // v_fma_mix_f32 reads the f16 halves of ev[w] directly: a = e * r (+0), rem = e - s * a; no separate conversions
                float a0, a1, m0, m1;
                asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(a0) : "v"(ev[w]), "s"(rinv));
                asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(a1) : "v"(ev[w]), "s"(rinv));
                asm("v_fma_mix_f32 %0, -%1, %2, %3 op_sel_hi:[0,0,1]" : "=v"(m0) : "s"(s), "v"(a0), "v"(ev[w]));
                asm("v_fma_mix_f32 %0, -%1, %2, %3 op_sel:[0,0,1] op_sel_hi:[0,0,1]" : "=v"(m1) : "s"(s), "v"(a1), "v"(ev[w]));
                float q0 = __builtin_fmaf(m0, rinv, a0);
                float q1 = __builtin_fmaf(m1, rinv, a1);
                // keep the f32 quotient and its conversion apart: fused into v_fma_mixlo_f16 the pair rounds
                // subnormal f16 results differently from fma-then-convert
                asm volatile("" : "+v"(q0), "+v"(q1));
                out[w] = ST::round_pair(q0, q1);
            }
        } else {
#pragma unroll
            for (int w = 0; w < 4; w++) out[w] = ST::round_pair(ST::widen_bits(ev[w] & 0xffffu) / s, ST::widen_bits(ev[w] >> 16) / s);
        }
        return out;
    };
    auto read_prev_sum = [&](uint32_t par) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t sb = __builtin_amdgcn_readfirstlane((uint32_t)sums[par][rr + h * SP_HALF]);
            const float s = ST::widen_bits(sb);
            s_prev[h] = s;
            // normal, finite, not tiny: the reciprocal-plus-correction quotient is exact there
            fast_prev[h] = (s >= 6.103515625e-05f) && (s < __builtin_huge_valf());
            rinv_prev[h] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, fast_prev[h] ? 1.0f / s : 0.0f)));
        }
    };
    // exp of the vector that arrived, in place (zeros past the row end: adding +0 is a no-op; rows past the tensor's end
    // read zeros and their sums are never used)
    // A wave whose 512 values of this step are all -inf (the part of a row that a causal mask covers) takes exp(-inf) for
    // all of them without the eight table reads per lane; the test is wave-wide, so the branch is a scalar one.
    const uint32_t exp_ninf = __builtin_amdgcn_readfirstlane((uint32_t)lut[ST::NEG_INF_PAIR & 0xffffu] * 0x10001u);
    auto exp_in_place = [&](v4u& in, const v4u& m, uint32_t t, uint32_t sh) {
        if (MASK) in = ST::add_vec(in, m);                   // scores + mask in the 16-bit type, as the separate add would round it
        const bool mine = ((in[0] ^ ST::NEG_INF_PAIR) | (in[1] ^ ST::NEG_INF_PAIR) | (in[2] ^ ST::NEG_INF_PAIR) | (in[3] ^ ST::NEG_INF_PAIR)) == 0;
        if (__builtin_amdgcn_ballot_w64(!mine) == 0) {
            in = v4u{exp_ninf, exp_ninf, exp_ninf, exp_ninf};
        } else {
#pragma unroll
            for (int w = 0; w < 4; w++) in[w] = sp_exp_pair(lut, in[w]);
        }
        if (RAGGED ? t * (SP_TC * 2) + cbyte >= sh + row_bytes : past_end(t)) in = v4u{0, 0, 0, 0};
    };
    // RAGGED: the neighbours' elements in a row's first and last vector are zeroed in the tile, after the vector has been
    // written there (on the LDS copy, so that the data registers of the main path stay untouched: masking them in a branch
    // cost 50 vector registers).  Which step and lane hold those two vectors is the same for the whole wave (sh lives in a
    // scalar register), so every test below is a scalar branch except the one that picks the lane, and the zeros go out
    // as at most three aligned writes of 8, 4 and 2 bytes.
    auto zero_outside = [&](uint32_t t, uint32_t sh, uint32_t trow_idx) {
        unsigned char* trb = reinterpret_cast<unsigned char*>(&tile[trow_idx][0]);
        if (t == 0 && sh != 0 && cbyte == 0) {               // bytes [0, sh) of the span belong to the row before
            if (sh & 8) *reinterpret_cast<uint64_t*>(trb) = 0;
            if (sh & 4) *reinterpret_cast<uint32_t*>(trb + (sh & 8)) = 0;
            if (sh & 2) *reinterpret_cast<uint16_t*>(trb + (sh & 12)) = 0;
        }
        const uint32_t end = sh + row_bytes, pe = end & ~15u;        // the vector at span byte pe holds the row's end
        if ((end & 15u) != 0 && t == pe / (SP_TC * 2) && cbyte == (pe & (SP_TC * 2 - 1))) {
            uint32_t at = (pe & (SP_TC * 2 - 1)) + (end & 15u);      // bytes [at, next vector) belong to the row after
            if (at & 2) {
                *reinterpret_cast<uint16_t*>(trb + at) = 0;
                at += 2;
            }
            if (at & 4) {
                *reinterpret_cast<uint32_t*>(trb + at) = 0;
                at += 4;
            }
            if (at & 8) *reinterpret_cast<uint64_t*>(trb + at) = 0;
        }
    };

    uint32_t cur[2], nxt[2], prev[2] = {OOB, OOB}, pcur[2], pnxt[2], pprev[2] = {0, 0}, mcur[2], mnxt[2];
    uint32_t ccur[NCROW][NCLS], cnxt[NCROW][NCLS];
    item_off(0, cur, pcur, mcur);
    item_off(1, nxt, pnxt, mnxt);
    item_tiles(0, ccur);
    item_tiles(1, cnxt);
    uint32_t gpar = 0;

    if constexpr (PARK) {
        // steps of x in flight per thread: two, or the whole row when the step count is odd (the slot of step t is t % PF in
        // every group, so PF has to divide the step count)
        constexpr int PF = NSTEP % SP_PF == 0 ? SP_PF : NSTEP;
        static_assert(NSTEP % PF == 0 && PF <= 5, "prefetch slots must tile the steps of a row");
        v4u e[NSTEP][2];                                     // exp values of the group in flight, 8 halves per vector
        v4u pre[PF][2], mpre[2];                             // x: PF steps in flight; mask: one (L2 hits: a short distance is enough)
        v4u mhi[2];                                          // RAGGED: lane 63's second mask vector
#pragma unroll
        for (int t = 0; t < NSTEP; t++) e[t][0] = e[t][1] = v4u{0, 0, 0, 0};
        // The pending memory operations at the top of the group loop are the same on entry as after a group (two loads, two
        // stores, two loads, two stores: the stores here go nowhere), so the compiler can count them there too.
#pragma unroll
        for (int k = 0; k < PF; k++) {
#pragma unroll
            for (int h = 0; h < 2; h++) pre[k][h] = load_x(ld_off(cur[h], pcur[h], k));
#pragma unroll
            for (int h = 0; h < 2; h++) store_y(v4u{0, 0, 0, 0}, OOB);
        }
        if (MASK && !RAGGED) {                               // PAIR: the mask of steps 0 and 1 (NSTEP is even, so 1 exists)
#pragma unroll
            for (int h = 0; h < 2; h++)
                mpre[h] = PAIR ? load_m_tile(step_off(cur[0] - pcur[0], h), ccur[0][TILES ? h : 0])
                               : load_m_tile(step_off(cur[h] - pcur[h], 0), ccur[PAIR ? 0 : h][0]);
        }
        if (MASK && RAGGED) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                mpre[h] = load_m(mask_lo_off(mcur[h], pcur[h], 0));
                mhi[h] = load_m(mask_hi_off(mcur[h], pcur[h], 0));
            }
        }

        for (uint32_t it = 0; it < n_items; it++) {
#pragma unroll
            for (int t = 0; t < NSTEP; t++) {
#pragma unroll
                for (int h = 0; h < 2; h++)
                    exp_in_place(pre[t % PF][h],
                                 (MASK && RAGGED) ? mask_funnel(mpre[h], mhi[h], mcur[h])
                                 : PAIR           ? tile_value(mpre[t % 2], ccur[0][TILES ? t : 0])
                                 : TILES          ? tile_value(mpre[h], ccur[PAIR ? 0 : h][TILES ? t : 0])
                                                  : mpre[h],
                                 t, pcur[h]);
                __syncthreads();                             // A: wave 0 has left the previous tile
                *reinterpret_cast<v4u*>(&tile[rr][ccol]) = pre[t % PF][0];
                *reinterpret_cast<v4u*>(&tile[rr + SP_HALF][ccol]) = pre[t % PF][1];
                if (RAGGED) {
                    zero_outside(t, pcur[0], rr);
                    zero_outside(t, pcur[1], rr + SP_HALF);
                }
                // the registers are free again: next loads, PF steps ahead, possibly in the block's next group
                // (loads return in order: the mask of the next step goes first, so that waiting for it does not wait for x
                // of the step after)
                if (MASK && !RAGGED && !PAIR) {
#pragma unroll
                    for (int h = 0; h < 2; h++)
                        mpre[h] = (t + 1 < NSTEP) ? load_m_tile(step_off(cur[h] - pcur[h], t + 1), ccur[PAIR ? 0 : h][TILES && t + 1 < NSTEP ? t + 1 : 0])
                                                  : load_m_tile(step_off(nxt[h] - pnxt[h], 0), cnxt[PAIR ? 0 : h][0]);
                }
                if (PAIR)                                    // this step's slot is free: the mask of two steps ahead
                    mpre[t % 2] = (t + 2 < NSTEP) ? load_m_tile(step_off(cur[0] - pcur[0], t + 2), ccur[0][PAIR && t + 2 < NSTEP ? t + 2 : 0])
                                                  : load_m_tile(step_off(nxt[0] - pnxt[0], t + 2 - NSTEP), cnxt[0][PAIR && t + 2 >= NSTEP ? t + 2 - NSTEP : 0]);
                if (MASK && RAGGED) {
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        mpre[h] = (t + 1 < NSTEP) ? load_m(mask_lo_off(mcur[h], pcur[h], t + 1)) : load_m(mask_lo_off(mnxt[h], pnxt[h], 0));
                        mhi[h] = (t + 1 < NSTEP) ? load_m(mask_hi_off(mcur[h], pcur[h], t + 1)) : load_m(mask_hi_off(mnxt[h], pnxt[h], 0));
                    }
                }
#pragma unroll
                for (int h = 0; h < 2; h++)
                    pre[t % PF][h] = (t + PF < NSTEP) ? load_x(ld_off(cur[h], pcur[h], t + PF)) : load_x(ld_off(nxt[h], pnxt[h], t + PF - NSTEP));
                __syncthreads();                             // B: parked for the walk
                if (t == 0) read_prev_sum(gpar ^ 1);         // published by wave 0 before it reached barrier A
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    store_y(quotients(e[t][h], h), st_off(prev[h], pprev[h], t));   // first group: prev is OOB, the store is dropped
                    // this group's values come back from the tile, which stays intact until the next barrier A
                    e[t][h] = *reinterpret_cast<const v4u*>(&tile[rr + h * SP_HALF][ccol]);
                }
            }
#pragma unroll
            for (int h = 0; h < 2; h++) {
                prev[h] = cur[h];
                cur[h] = nxt[h];
            }
#pragma unroll
            for (int h = 0; h < 2; h++) {
                pprev[h] = pcur[h];
                pcur[h] = pnxt[h];
                mcur[h] = mnxt[h];
            }
            item_off(it + 2, nxt, pnxt, mnxt);
#pragma unroll
            for (int h = 0; h < NCROW; h++)
#pragma unroll
                for (int t = 0; t < NCLS; t++) ccur[h][t] = cnxt[h][t];
            item_tiles(it + 2, cnxt);
            gpar ^= 1;
        }
        // drain: outputs of the block's last group
        __syncthreads();
        read_prev_sum(gpar ^ 1);
#pragma unroll
        for (int t = 0; t < NSTEP; t++)
#pragma unroll
            for (int h = 0; h < 2; h++) store_y(quotients(e[t][h], h), st_off(prev[h], pprev[h], t));
    } else {
        // One flat loop over the steps of all groups, two steps per trip (nsteps is even; a step past the row end moves
        // nothing).  Per step and row: exp values to the tile and to y, x of two steps ahead, the previous group's exp
        // values of this step (loaded two steps ago from y, where this thread put them a group ago) divided and stored,
        // and the load of those of two steps ahead.  The prologue issues the same sequence with targets that do not exist.
        v4u pre[2][2], qpre[2][2], mpre[2];
#pragma unroll
        for (int k = 0; k < 2; k++) {
#pragma unroll
            for (int h = 0; h < 2; h++) store_park(v4u{0, 0, 0, 0}, OOB);
            if (MASK) {
#pragma unroll
                for (int h = 0; h < 2; h++) mpre[h] = load_m(step_off(cur[h] - pcur[h], 0));
            }
#pragma unroll
            for (int h = 0; h < 2; h++) pre[k][h] = load_x(step_off(cur[h], k));
#pragma unroll
            for (int h = 0; h < 2; h++) store_y(v4u{0, 0, 0, 0}, OOB);
#pragma unroll
            for (int h = 0; h < 2; h++) qpre[k][h] = load_y(OOB);
        }
        uint32_t t0 = 0;                                     // first step of the trip within its group
        const uint32_t trips = n_items * (nsteps / 2);
        for (uint32_t trip = 0; trip < trips; trip++) {
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const uint32_t t = t0 + k;
#pragma unroll
                for (int h = 0; h < 2; h++) exp_in_place(pre[k][h], mpre[h], t, 0);
                __syncthreads();                             // A
                *reinterpret_cast<v4u*>(&tile[rr][ccol]) = pre[k][0];
                *reinterpret_cast<v4u*>(&tile[rr + SP_HALF][ccol]) = pre[k][1];
#pragma unroll
                for (int h = 0; h < 2; h++) store_park(pre[k][h], step_off(cur[h], t));      // parked in y (kept in cache: read back soon)
                const bool wrap = t + 2 >= nsteps;           // two steps ahead is in the block's next group
                const uint32_t ta = wrap ? t + 2 - nsteps : t + 2;
                if (MASK) {
                    const bool w1 = t + 1 >= nsteps;
#pragma unroll
                    for (int h = 0; h < 2; h++) mpre[h] = load_m(step_off(w1 ? nxt[h] - pnxt[h] : cur[h] - pcur[h], w1 ? 0 : t + 1));
                }
#pragma unroll
                for (int h = 0; h < 2; h++) pre[k][h] = load_x(step_off(wrap ? nxt[h] : cur[h], ta));
                __syncthreads();                             // B
                if (t == 0) read_prev_sum(gpar ^ 1);
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    store_y(quotients(qpre[k][h], h), step_off(prev[h], t));
                    qpre[k][h] = load_y(step_off(wrap ? cur[h] : prev[h], ta));
                }
            }
            t0 += 2;
            if (t0 >= nsteps) {                              // next group
                t0 = 0;
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    prev[h] = cur[h];
                    cur[h] = nxt[h];
                }
                pcur[0] = pnxt[0];
                pcur[1] = pnxt[1];
                item_off(trip / (nsteps / 2) + 2, nxt, pnxt, mnxt);
                gpar ^= 1;
            }
        }
        // drain: the last group's parked values (steps 0 and 1 are already here; the values of the last steps were stored
        // a moment ago, so everything this wave has in flight completes first)
        __syncthreads();
        __builtin_amdgcn_s_waitcnt(0);
        read_prev_sum(gpar ^ 1);
        for (uint32_t t = 0; t < nsteps; t += 2) {
#pragma unroll
            for (int k = 0; k < 2; k++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    store_y(quotients(qpre[k][h], h), step_off(prev[h], t + k));
                    qpre[k][h] = load_y(step_off(prev[h], t + k + 2 < nsteps ? t + k + 2 : 0xffffu));
                }
        }
    }
}

// The ragged-row variant's second launch: the elements of a row's first and last span vectors when those vectors are
// shared with a neighbouring row (at most 7 + 7 per row), from x (plus the mask), the exp table and the row sum the streaming kernel
// left in row_sums.  Sixteen threads per row: 0..7 the elements of the first span vector, 8..15 those of the last.
// The quotient is the IEEE division the streaming kernel's short division reproduces.
template <typename T>
__global__ void __launch_bounds__(BLOCK) softmax16_edges_kernel(const uint16_t* __restrict__ table, const T* x, const T* __restrict__ mask,
                                                                uint32_t mask_rows, T* y, const uint16_t* __restrict__ row_sums,
                                                                uint64_t rows, uint32_t cols) {
    const uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    const uint64_t row = gid >> 4;
    if (row >= rows) return;
    const uint32_t j = (uint32_t)gid & 7u;
    const bool tail = (gid & 8u) != 0;
    const uint64_t first = row * cols;
    const uint32_t shift = (uint32_t)(first & 7);
    const uint32_t last_vec = (shift + cols - 1) >> 3;       // index of the row's last span vector
    const bool first_whole = shift == 0 && cols >= 8;
    const bool last_whole = ((shift + cols) & 7) == 0 && (last_vec > 0 || shift == 0);
    if (tail ? (last_vec == 0 || last_whole) : first_whole) return;
    const uint32_t e = (tail ? last_vec * 8 : 0) + j;        // element of the span
    if (e < shift || e - shift >= cols) return;
    const uint64_t at = first + (e - shift);
    T xv = x[at];
    if (mask) xv = Ar<T>::add(xv, mask[(row % mask_rows) * cols + (e - shift)]);     // row r takes mask row r % mask_rows
    const uint16_t xb = __builtin_bit_cast(uint16_t, xv);
    const T ev = __builtin_bit_cast(T, table[xb]);
    y[at] = Ar<T>::div(ev, __builtin_bit_cast(T, row_sums[row]));
}

// The class of every 512-column tile of a mask, for the masked variants of the streaming kernel that park in registers:
// a tile whose elements all have the same bits v gets the word v | v << 16 (what the kernel puts in place of the loads it
// then leaves out: under a causal mask seven tiles of eight hold nothing but 0 or nothing but -inf), any other tile, and
// a tile of 0xffff, gets 0xffffffff.  cols % 8 == 0; a row's last tile may be short.  A wave takes MT_PER_WAVE tiles with
// all their loads in flight at once.
constexpr int MT_PER_WAVE = 8;
template <typename T>
__global__ void __launch_bounds__(BLOCK) mask_tiles_kernel(const T* __restrict__ mask, uint32_t mask_rows, uint32_t cols, uint32_t nt,
                                                           uint32_t* __restrict__ tiles) {
    const uint32_t wave = blockIdx.x * (BLOCK / 64) + threadIdx.x / 64;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t ntiles = mask_rows * nt;
    const uint16_t* m16 = reinterpret_cast<const uint16_t*>(mask);
    v4u v[MT_PER_WAVE];
    bool have[MT_PER_WAVE];
#pragma unroll
    for (int k = 0; k < MT_PER_WAVE; k++) {
        const uint32_t tile = wave * MT_PER_WAVE + k;
        const uint32_t row = tile / nt, t = tile - row * nt;
        const uint32_t col = t * SP_TC + lane * 8;
        have[k] = tile < ntiles && col < cols;
        v[k] = v4u{0, 0, 0, 0};
        if (have[k]) v[k] = *reinterpret_cast<const v4u*>(m16 + (uint64_t)row * cols + col);
    }
#pragma unroll
    for (int k = 0; k < MT_PER_WAVE; k++) {
        const uint32_t tile = wave * MT_PER_WAVE + k;
        if (tile >= ntiles) break;                           // the same for the whole wave
        const uint32_t first = (__builtin_amdgcn_readfirstlane(v[k][0]) & 0xffffu) * 0x10001u;     // lane 0 holds the tile's first element
        const bool same = !have[k] || ((v[k][0] ^ first) | (v[k][1] ^ first) | (v[k][2] ^ first) | (v[k][3] ^ first)) == 0;
        const bool uniform = __builtin_amdgcn_ballot_w64(!same) == 0 && first != 0xffffffffu;
        if (lane == 0) tiles[RT_SM_TILES_HEAD + tile] = uniform ? first : 0xffffffffu;
    }
}

// mask == nullptr: plain softmax.  Otherwise the mask has `period` rows of `cols` columns and repeats every `period`
// rows of x (rows % period == 0).  Returns RT_OK with *done = false when the shape does not fit this kernel.
template <typename T>
int launch_stream16(rt_device* dev, const void* x, const void* mask, uint64_t period, void* y, uint64_t rows, uint32_t cols, bool* done) {
    *done = false;
    constexpr int TI = sizeof(typename SpType<T>::Run) == 4 ? 1 : 0;         // table and attribute index: 0 f16, 1 bf16
    const uint64_t row_bytes = (uint64_t)cols * 2;
    if (!mask) period = rows;
    const bool ragged = cols % 8 != 0;                       // rows over their covering aligned vectors, finished by the edges kernel
    // with a mask: in one launch only, and a mask on a 16-byte boundary
    if (ragged && mask && (!rt_aligned(mask, 16) || rows * row_bytes > 0x7fffffe0ull || rows > RT_SM_ROW_SUMS)) return RT_OK;
    // the kernel addresses a launch with 32-bit byte offsets below 2^31: larger tensors go in chunks of whole periods
    // (whole 30-row groups when nothing repeats)
    uint64_t chunk_rows;
    if (mask) {
        if (period * row_bytes > 0x7fffffffull) return RT_OK;
        chunk_rows = (0x7fffffffull / (period * row_bytes)) * period;
    } else if (ragged) {
        // a chunk's row sums must fit the device's buffer, and every chunk must start on a 16-byte boundary (8 rows do)
        uint64_t max_rows = 0x7fffffe0ull / row_bytes;
        if (max_rows > RT_SM_ROW_SUMS) max_rows = RT_SM_ROW_SUMS;
        chunk_rows = rows <= max_rows ? rows : max_rows / 120 * 120;
        if (chunk_rows == 0) return RT_OK;
    } else {
        chunk_rows = (0x7fffffffull / row_bytes) / SP_ROWS * SP_ROWS;
        if (chunk_rows == 0) return RT_OK;
    }
    // the exp table is built on first use, which synchronises: while a graph is being captured a missing table sends the
    // caller to the two-pass kernel instead (same bits)
    if (dev->capturing && !dev->unary_lut[TI][RT_EXP]) return RT_OK;
    const uint16_t* table = nullptr;
    int rc = rt_unary_table(dev, TI, RT_EXP, &table);
    if (rc) return rc;
    const uint32_t nt = (cols + SP_TC - 1) / SP_TC;
    if (ragged && nt > SP_MAX_STEPS) return RT_OK;           // (a ragged row's one vector past its last step is the walker's)
    const bool full = !ragged && cols % SP_TC == 0 && nt != 7 && nt <= 8;
#define RT_SP(NS, F, M)                                                                                                              \
    do {                                                                                                                             \
        const uint64_t bit = 1ull << (TI * 32 + (NS == 0 ? 4 : NS == 1 ? 0 : NS == 2 ? 1 : NS == 4 ? 2 : NS == 6 ? 5 : NS == 3 ? 6 : NS == 5 ? 7 : 3) * 4 + (F ? 2 : 0) + (M ? 1 : 0)); \
        if (!(dev->sp_attr_set & bit)) {               /* the LDS opt-in is per function and per device */                           \
            RT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(softmax16_stream_kernel<T, NS, F, M>),                          \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)SP_SMEM_BYTES));                             \
            dev->sp_attr_set |= bit;                                                                                                 \
        }                                                                                                                            \
        hipLaunchKernelGGL((softmax16_stream_kernel<T, NS, F, M>), dim3(blocks), dim3(SP_BLOCK), SP_SMEM_BYTES, dev->stream, table,  \
                           xc, (const T*)mask, yc, n, cols, sch, (uint16_t*)nullptr, (const uint32_t*)dev->sm_mask_tiles);          \
    } while (0)
#define RT_SP_PAIR(NS, F)                                                                                                            \
    do {                                                                                                                             \
        const uint32_t bit = 1u << (TI * 8 + (NS / 2 - 1) * 2 + (F ? 1 : 0));                                                        \
        if (!(dev->sp_pair_attr_set & bit)) {                                                                                        \
            RT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(softmax16_stream_kernel<T, NS, F, 2>),                          \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)SP_SMEM_BYTES));                             \
            dev->sp_pair_attr_set |= bit;                                                                                            \
        }                                                                                                                            \
        hipLaunchKernelGGL((softmax16_stream_kernel<T, NS, F, 2>), dim3(blocks), dim3(SP_BLOCK), SP_SMEM_BYTES, dev->stream, table,  \
                           xc, (const T*)mask, yc, n, cols, sch, (uint16_t*)nullptr, (const uint32_t*)dev->sm_mask_tiles);          \
    } while (0)
#define RT_SP_PAIR_NS(F)                                    \
    do {                                                    \
        if (nt <= 2) RT_SP_PAIR(2, F);                      \
        else if (nt <= 4) RT_SP_PAIR(4, F);                 \
        else if (nt <= 6) RT_SP_PAIR(6, F);                 \
        else RT_SP_PAIR(8, F);                              \
    } while (0)
#define RT_SP_RAGGED(NS, M)                                                                                                          \
    do {                                                                                                                             \
        const uint64_t bit = 1ull << ((M ? 16 : 0) + TI * 8 + (NS == 1 ? 0 : NS == 2 ? 1 : NS == 4 ? 2 : NS == 6 ? 4 : NS == 3 ? 5 : NS == 5 ? 6 : 3)); \
        if (!(dev->sp_ragged_attr_set & bit)) {                                                                                      \
            RT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(softmax16_stream_kernel<T, NS, false, M, true>),                \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)SP_SMEM_BYTES));                             \
            dev->sp_ragged_attr_set |= bit;                                                                                              \
        }                                                                                                                            \
        hipLaunchKernelGGL((softmax16_stream_kernel<T, NS, false, M, true>), dim3(blocks), dim3(SP_BLOCK), SP_SMEM_BYTES,            \
                           dev->stream, table, xc, (const T*)mask, yc, n, cols, sch, dev->sm_row_sums, (const uint32_t*)nullptr);                              \
    } while (0)
#define RT_SP_RAGGED_NS(M)                                  \
    do {                                                    \
        if (nt <= 1) RT_SP_RAGGED(1, M);                    \
        else if (nt <= 2) RT_SP_RAGGED(2, M);               \
        else if (nt <= 3) RT_SP_RAGGED(3, M);               \
        else if (nt <= 4) RT_SP_RAGGED(4, M);               \
        else if (nt <= 5) RT_SP_RAGGED(5, M);               \
        else if (nt <= 6) RT_SP_RAGGED(6, M);               \
        else RT_SP_RAGGED(8, M);                            \
    } while (0)
#define RT_SP_NS(F, M)                                      \
    do {                                                    \
        if (nt <= 1) RT_SP(1, F, M);                        \
        else if (nt <= 2) RT_SP(2, F, M);                   \
        else if (nt <= 3) RT_SP(3, F, M);                   \
        else if (nt <= 4) RT_SP(4, F, M);                   \
        else if (nt <= 5) RT_SP(5, F, M);                   \
        else if (nt <= 6) RT_SP(6, F, M);                   \
        else RT_SP(8, F, M);                                \
    } while (0)
    for (uint64_t row0 = 0; row0 < rows; row0 += chunk_rows) {
        const uint64_t n = rows - row0 < chunk_rows ? rows - row0 : chunk_rows;
        const T* xc = (const T*)x + row0 * cols;
        T* yc = (T*)y + row0 * cols;
        SpSched sch;
        // a mask of few rows (a [1, T] padding mask, a short prefill): groups run across its periods
        sch.PM = (uint32_t)(mask ? period : n);
        sch.pm_div = make_fastdiv(sch.PM);
        sch.P = (uint32_t)(mask && period >= 8 * SP_ROWS ? period : n);
        sch.reps = (uint32_t)(n / sch.P);
        sch.nsteps = (nt + 1) & ~1u;
        // one mask row for two heads: rows of an even number of steps under a mask that repeats every P rows
        const bool pair = mask && !ragged && nt <= SP_MAX_STEPS && (nt % 2 == 0 || nt == 7) && sch.PM == sch.P && sch.reps >= 2;
        sch.item_reps = pair ? (sch.reps + 1) / 2 : sch.reps;
        const uint32_t rmax = pair ? SP_HALF : SP_ROWS, rmul = pair ? 2 : 1;
        // rows per group: every block runs ceil(groups / grid) rounds of 8-or-fewer steps whatever the group holds, so
        // 4370 groups of 30 rows on 256 CUs cost 18 rounds where 17.07 are needed; 27-row groups make 19 full rounds.
        // A step takes the longer of the walk (1.5 us whatever the group holds) and the group's memory time (2 KiB per
        // row at a CU's share of the bandwidth: about 0.09 us per row), so a round costs max(R + 1, 18) in units of a
        // row's memory time; pick the size with the cheapest total, the smallest such size on a tie.  Few rows (a decode
        // step's [B * H, T] scores) spread over the CUs the same way: 32 rows run as 32 one-row groups.
        // With a mask that repeats every P rows, group pg of every period reads the same mask rows.  Item w runs on block
        // w % grid, and blocks go to the eight XCDs in turn, so those groups land on 8 / gcd(GP % 8, 8) different XCDs, each
        // of which pulls the mask rows into its own L2.  Among the sizes within 5 % of the cheapest, the one that keeps a
        // mask group on the fewest XCDs is taken ([1,16,4096,4096] with a causal mask: 27 rows, 152 groups a period, 211 us;
        // the cheapest size by the count alone, 26 rows and 158 groups, 224 us; 114 against 121 us on [1,32,2048,2048]).
        {
            auto cost_of = [&](uint32_t R) -> uint64_t {
                const uint64_t groups = (uint64_t)((sch.P + R - 1) / R) * sch.item_reps;
                const uint64_t rounds = (groups + dev->num_cus - 1) / dev->num_cus;
                return rounds * (R * rmul + 1 > 18 ? R * rmul + 1 : 18);
            };
            uint64_t best = ~0ull;
            sch.R = rmax;
            for (uint32_t R = rmax; R >= 1; R--) {
                const uint64_t cost = cost_of(R);
                if (cost <= best) {
                    best = cost;
                    sch.R = R;
                }
            }
            if (mask && sch.reps > 1 && !pair) {
                auto xcds_of = [&](uint32_t R) -> uint32_t {
                    const uint32_t g = ((sch.P + R - 1) / R) % 8;
                    return g == 0 ? 1 : (g % 4 == 0) ? 2 : (g % 2 == 0) ? 4 : 8;
                };
                uint32_t pick = sch.R, pick_x = xcds_of(sch.R);
                uint64_t pick_cost = best;
                for (uint32_t R = SP_ROWS; R >= 1; R--) {
                    const uint64_t cost = cost_of(R);
                    if (cost * 20 > best * 21) continue;
                    const uint32_t xc = xcds_of(R);
                    if (xc < pick_x || (xc == pick_x && cost < pick_cost)) {
                        pick = R;
                        pick_x = xc;
                        pick_cost = cost;
                    }
                }
                sch.R = pick;
            }
        }
        sch.GP = (sch.P + sch.R - 1) / sch.R;
        sch.pace = sch.phase_fx = 0;                         // set below, once the grid is known
        sch.gp_div = make_fastdiv(sch.GP);
        const uint64_t items = (uint64_t)sch.GP * sch.item_reps;
        RT_REQUIRE(items <= 0xffffffffull, RT_ERR_SIZE, "rt_softmax: too many row groups");
        const unsigned blocks = (unsigned)(items < (uint64_t)dev->num_cus ? items : (uint64_t)dev->num_cus);   // one resident block per CU
        // Pacing.  Left to itself the kernel offers HBM more requests than it sustains, and what it then gets is less than
        // what it gets when it asks for slightly less: 366 us unpaced against 345-350 us on [1,32,4096,4096] in the
        // benchmark step (a plain persistent copy loop shows the same: 5.9 TB/s unpaced, 6.4 TB/s with a sleep of the
        // right length per iteration, and a write-only loop 4.4 against 6.6 TB/s).  So the walker holds the block's
        // steps to the period at which all blocks together move RT_PACE_BYTES_PER_S, by the device's wall clock, and the
        // blocks start out of phase (sp_pace_step).  A pace that is too fast gives the unpaced behaviour back (7.0e12:
        // 359 us), one that is too slow costs in proportion (6.4e12: 355 us).  Paced are, on a grid that fills the
        // chip, the plain variant and the masked one that takes one mask row per pair of heads (at the same rate: 6.4e12
        // costs that one 3 us, 6.8e12 and 7.0e12 leave 5 us of its dependence on where the buffers lie).
        if (blocks == dev->num_cus && !ragged && (!mask || pair)) {
            const double rate = RT_PACE_BYTES_PER_S;
            const double group_bytes = (double)sch.R * rmul * cols * 2 * (nt > SP_MAX_STEPS ? 4 : 2);     // in and out (long rows: parked and read back)
            const double steps = nt > SP_MAX_STEPS ? sch.nsteps : nt == 7 ? 8 : nt;          // the steps the kernel variant takes per group
            sch.pace = (uint32_t)(group_bytes / steps * blocks / rate * dev->wall_clock_hz + 0.5);
            if (dev->debug_softmax_pace) sch.pace = dev->debug_softmax_pace;
            sch.phase_fx = sch.pace > 0xffffu ? 0 : (sch.pace << 16) / blocks;
        }
        // the classes of the mask's tiles, for the variants that use them (a table of at most RT_SM_MASK_TILES words).  Only
        // for a mask of 16 MiB or more: a smaller one stays in the L2s between its repeats, loading all of it costs
        // nothing that could be measured ([1,32,2048,2048] and [1,32,2560,2560]: 111 and 188 us either way), and the
        // pass over the mask is a launch of 3 us ([8,32,512,512] 71 -> 68 us, a decode step's [1,32,1,4096] 29 -> 26 us).
        sch.tile_stride = 0;
        if (mask && !ragged && nt <= SP_MAX_STEPS && (uint64_t)sch.PM * nt <= RT_SM_MASK_TILES && rt_aligned(mask, 16) &&
            (uint64_t)sch.PM * cols * sizeof(T) >= (16ull << 20)) {
            const uint32_t ntiles = sch.PM * nt;
            const uint32_t per_block = (BLOCK / 64) * MT_PER_WAVE;
            hipLaunchKernelGGL((mask_tiles_kernel<T>), dim3((ntiles + per_block - 1) / per_block), dim3(BLOCK), 0, dev->stream, (const T*)mask,
                               sch.PM, cols, nt, dev->sm_mask_tiles);
            RT_CHECK_LAUNCH("mask_tiles_kernel");
            sch.tile_stride = nt;
        }
        if (ragged) {
            if (mask) RT_SP_RAGGED_NS(true);
            else RT_SP_RAGGED_NS(false);
            RT_CHECK_LAUNCH("softmax16_stream_kernel");
            const uint64_t eblocks = (n * 16 + BLOCK - 1) / BLOCK;
            hipLaunchKernelGGL((softmax16_edges_kernel<T>), dim3((unsigned)eblocks), dim3(BLOCK), 0, dev->stream, table, xc, (const T*)mask,
                               sch.PM, yc, (const uint16_t*)dev->sm_row_sums, n, cols);
            RT_CHECK_LAUNCH("softmax16_edges_kernel");
            continue;
        }
        if (nt > SP_MAX_STEPS) {                         // long rows: exp values parked in y
            if (mask) RT_SP(0, false, true);
            else RT_SP(0, false, false);
        } else if (pair) {
            if (full) RT_SP_PAIR_NS(true);
            else RT_SP_PAIR_NS(false);
        } else if (mask) {
            if (full) RT_SP_NS(true, true);
            else RT_SP_NS(false, true);
        } else {
            if (full) RT_SP_NS(true, false);
            else RT_SP_NS(false, false);
        }
        RT_CHECK_LAUNCH("softmax16_stream_kernel");
    }
#undef RT_SP_NS
#undef RT_SP_PAIR_NS
#undef RT_SP_PAIR
#undef RT_SP_RAGGED_NS
#undef RT_SP_RAGGED
#undef RT_SP
    *done = true;
    return RT_OK;
}

}  // namespace

#endif
