// Pacing of persistent kernels.  A loop that streams through HBM from one resident block per CU offers memory more requests
// than it sustains, and what it then gets is less than what it gets when it asks for slightly less (a plain persistent
// copy loop: 5.9 TB/s left to itself, 6.4 TB/s with a wait of the right length per iteration; a write-only loop 4.4
// against 6.6 TB/s).  The kernels that are built that way because they keep a 128 KiB table in LDS (the streaming
// softmax, the table-lookup activations) therefore hold their steps to a period by the device's wall clock.
#ifndef RT_PACE_H
#define RT_PACE_H
#include <stdint.h>

// what a paced kernel asks of HBM, all blocks together (measured optimum 6.6-6.7e12 on the streaming softmax; the
// table-lookup activations on 1 GiB: 6.2e12 182 us, 6.65e12 173 us, 7.0e12 184 us, unpaced 205 us)
constexpr double RT_PACE_BYTES_PER_S = 6.65e12;

// the 100 MHz wall clock (low 32 bits), read as one opaque block so that it does not take part in the scheduling of the
// code around it
__device__ __forceinline__ uint32_t rt_pace_clock() {
    uint64_t t;
    asm volatile("s_memrealtime %0\n s_waitcnt lgkmcnt(0)" : "=s"(t) :: "memory");
    return (uint32_t)t;
}

// The block's schedule: a step may not start before `pace` ticks of the wall clock have passed since the one before
// was allowed to (t_step): a wave that arrives early waits, and a late one goes on at once and the schedule starts
// again from its arrival, so that a step which was late is not followed by a burst (it is the bursts that overload
// HBM).  Inputs whose steps are longer than the pace for reasons of their own (dense scores: the table lookups collide
// in the LDS banks) must not be held at all, because their short steps would be delayed and their long ones not made up
// for: the wave keeps a running average of the time between its steps (`avg`, a quarter of each new value), and while
// that is above 1.2 paces it only keeps time.  A wait ends after 4096 looks at the clock at the latest (a step is a few
// hundred ticks, a look takes several), so the kernel finishes whatever the clock does.  Everything is in scalar registers and in one asm statement: written as
// C++ the loop changed the register allocation and instruction order of the whole kernel, loader waves included.
__device__ __forceinline__ void rt_pace_step(uint32_t& t_step, uint32_t& t_last, uint32_t& avg, uint32_t pace, uint32_t slow) {
    asm volatile(
        "s_memrealtime s[96:97]\n"
        "s_waitcnt lgkmcnt(0)\n"
        "s_sub_u32 s98, s96, %1\n"              // time since the previous step
        "s_mov_b32 %1, s96\n"
        "s_sub_u32 s98, s98, %2\n"
        "s_ashr_i32 s98, s98, 2\n"
        "s_add_u32 %2, %2, s98\n"               // avg += (dt - avg) / 4
        "s_cmp_ge_i32 %2, %4\n"
        "s_cbranch_scc1 2f\n"                   // steps are slow by themselves: only keep time
        "s_sub_u32 s98, s96, %0\n"              // ticks since the last permitted start
        "s_cmp_ge_i32 s98, %3\n"
        "s_cbranch_scc1 2f\n"                   // late or on time
        "s_movk_i32 s99, 0x1000\n"
        "1:\n"
        "s_sleep 1\n"                           // early: wait for the step's time
        "s_memrealtime s[96:97]\n"
        "s_waitcnt lgkmcnt(0)\n"
        "s_sub_u32 s99, s99, 1\n"
        "s_cmp_eq_u32 s99, 0\n"
        "s_cbranch_scc1 2f\n"                   // 4096 looks at a clock that does not get there: stop waiting for it
        "s_sub_u32 s98, s96, %0\n"
        "s_cmp_ge_i32 s98, %3\n"
        "s_cbranch_scc0 1b\n"
        "s_add_u32 %0, %0, %3\n"                // started exactly on schedule
        "s_mov_b32 %1, s96\n"
        "s_branch 3f\n"
        "2:\n"
        "s_mov_b32 %0, s96\n"                   // the schedule starts again from this arrival
        "3:\n"
        : "+s"(t_step), "+s"(t_last), "+s"(avg)
        : "s"(pace), "s"(slow)
        : "s96", "s97", "s98", "s99", "scc", "memory");
}

#endif
