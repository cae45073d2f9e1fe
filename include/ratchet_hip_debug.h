/*
 * ratchet_hip_debug.h - test hooks of libratchet_hip.so.  Not part of the seam a `-sys` crate binds (that is ratchet_hip.h):
 * nothing here has a counterpart in ratchet, and a product build has no reason to call any of it.  The library exports
 * them so that its own tests can reach two things that do not happen on demand: a failing HIP call, and a device clock
 * that never reaches the time a kernel waits for.
 */
#ifndef RATCHET_HIP_DEBUG_H
#define RATCHET_HIP_DEBUG_H

#include "ratchet_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Test hook, no counterpart in the reference: maps a HIP error code the way every entry point maps a failed HIP call
 * (status = -code, rt_last_error() = "<what>: <hipGetErrorString> (<hipGetErrorName>)", the runtime's sticky error
 * cleared), so that the mapping can be checked without a failing GPU.  hip_error 0 returns RT_OK and leaves the message. */
int rt_debug_hip_status(int hip_error, const char* what);
/* Test hook, no counterpart in the reference: the streaming 16-bit softmax holds its blocks to a pace by the device's
 * wall clock; `ticks` (of that clock, < 2^30) replaces the pace the launcher computes, 0 restores it.  With a pace far
 * beyond what a step takes every wait runs into its own bound (4096 looks at the clock) and the kernel must still
 * finish with the same results: that is what the test checks, with every wave leaving the kernel normally. */
int rt_debug_softmax_pace(rt_device* dev, uint32_t ticks);

#ifdef __cplusplus
}
#endif

#endif
