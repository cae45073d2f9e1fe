/*
 * TEST INFRASTRUCTURE ONLY - CPU restatement of ratchet-core's CPU executor for the
 * memory-bound tensor ops (binary, unary, cast, reindex, concat, softmax, norms, cache, rope, index ops, Q8_0 gather).
 *
 * Nothing in the shipped library links, loads or calls this file.  It exists so the
 * parity tests, the smoke check and the benchmark's CPU leg have an independent answer
 * to compare the HIP kernels with.
 *
 * Every function follows one reference function (cited at its definition in the .cpp).
 * The reference is generic Rust over f32 / half::f16 / half::bf16; for the 16-bit types every
 * arithmetic operator and every libm call is "widen to f32, operate, round to nearest
 * even" - that is what the `half` crate (^2.3.1, the version the reference pins in its
 * workspace Cargo.toml) does - and this file keeps exactly those rounding points.
 *
 * Pinning status (what checks each function besides this restatement):
 *   binary, cast, reindex, concat ........ numpy / IEEE-754 closed forms, bit-exact
 *   unary f32 ............................ torch / float64 evaluation at the reference's tolerances
 *   unary f16 ............................ exhaustive (65536 inputs) against a numpy float16 model
 *   softmax, layer_norm, rms_norm ........ torch at the reference's own tolerances + invariants; the f16 and bf16 paths
 *                                          bit for bit against step-wise numpy models (float16 / bit-rounded bfloat16
 *                                          arithmetic, left-to-right float32 sums, libm expf), with variants that drop a
 *                                          rounding point or reorder a step shown to disagree
 *   unary bf16 (gelu, silu, sigmoid, exp, tanh)  all 65536 inputs, bit for bit, against the same kind of model
 *   group_norm ........................... torch F.group_norm (the reference CPU path is a no-op)
 *   cache, index_select, index_write ..... numpy concatenate / take / flat assignment and the reference's own test cases
 *   rope ................................. float64 closed form of the half-rotation RoPE (what the reference's mlx ground
 *                                          truth computes), rotation invariants, offset additivity
 *   q8_0 quantize / dequantize ........... hand-made words, a numpy byte-view model, the reference's reflexivity check
 *   PARITY UNPINNED: the accumulation type of `Sum for f16` inside `mean` (assumed: f32
 *   accumulation, one rounding; switchable with orc_set_f16_sum_mode) - the `half` crate is
 *   not present in the reference tree and no reference test exercises the f16 CPU path.
 *   PARITY UNPINNED: sign of relu(-0.0) and of the sum of an all -0.0 row (toolchain dependent).
 */
#ifndef RATCHET_CPU_ORACLE_H
#define RATCHET_CPU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes: F32 = 0 and F16 = 1 follow DType::to_u32 (crates/ratchet-core/src/dtype/mod.rs:32-38) */
enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2, ORC_I32 = 3, ORC_U32 = 4 };
/* BinaryOp order: crates/ratchet-core/src/ops/binary.rs:19-24 */
enum { ORC_ADD = 0, ORC_SUB = 1, ORC_MUL = 2, ORC_DIV = 3 };
/* UnaryOp order: crates/ratchet-core/src/ops/unary.rs:23-38 */
enum {
    ORC_GELU = 0, ORC_TANH, ORC_EXP, ORC_LOG, ORC_SIN, ORC_COS, ORC_ABS, ORC_SQRT,
    ORC_RELU, ORC_FLOOR, ORC_CEIL, ORC_NEG, ORC_SILU, ORC_SIGMOID, ORC_UNARY_COUNT
};

/* 0 = ok, 1 = bad argument / unsupported */
int orc_binary(int op, int dt, const void* a, const void* b, void* y, size_t numel);
int orc_unary(int op, int dt, const void* x, void* y, size_t numel);
int orc_cast(int src_dt, int dst_dt, const void* x, void* y, size_t numel);

/* shapes are given at their own rank (1..4); the functions promote to rank 4 themselves */
int orc_permute(int elem_bytes, const void* x, void* y, int rank, const uint64_t* src_shape, const uint32_t* dims);
int orc_slice(int elem_bytes, const void* x, void* y, int rank, const uint64_t* src_shape,
              const uint64_t* start, const uint64_t* stop);
/* numpy_semantics = 0 reproduces the reference's vector special case, 1 is numpy.broadcast_to */
int orc_broadcast(int elem_bytes, const void* x, void* y, int src_rank, const uint64_t* src_shape,
                  int dst_rank, const uint64_t* dst_shape, int numpy_semantics);
int orc_concat(int elem_bytes, int n_inputs, const void* const* xs, int rank, const uint64_t* shapes /* n*rank */,
               int dim, void* y);

/* KV-cache append (crates/ratchet-core/src/ops/cache.rs:64-105; the reference has no CPU implementation, its test uses cat as
 * ground truth): dst = cat(cache[.. :offset ..], source) along dim, and source is also written into cache at offset. */
int orc_cache(int elem_bytes, void* cache, int rank, const uint64_t* cache_shape, const void* source, const uint64_t* source_shape,
              int dim, uint64_t offset, void* dst);

/* RoPE on [B, H, S, D] (crates/ratchet-core/src/cpu/rope.rs:7-143): F32 only, as in the reference; returns 1 for other dtypes */
int orc_rope(int dt, const void* x, void* y, const uint64_t* shape4, uint64_t dim, float base, uint64_t offset);
/* IndexSelect (cpu/mod.rs:44-84) and IndexWrite (ops/index_write.rs:96-104); an out-of-range index / run is an error */
int orc_index_select(int elem_bytes, const void* src, int rank, const uint64_t* src_shape, const int32_t* indices, uint64_t n_indices,
                     int dim, void* dst);
int orc_index_write(int elem_bytes, void* dst, int rank, const uint64_t* dst_shape, const void* src, uint64_t src_numel,
                    const uint64_t* write_start);

/* Q8_0 quantized buffers (crates/ratchet-core/src/quant.rs:19-49 quantize_inner, :101-130 dequantize_inner, with
 * PACK_SIZE 4, GROUP_SIZE 32, SF 127 from dtype/blocks.rs:180-199).  fp_dt 0 = Q8_0F (f32 scales), 1 = Q8_0H (f16 scales,
 * every operation rounded to f16).  numel must be a multiple of 32.  words: numel / 4, scales: numel / 32 (the reference
 * stores them in one buffer, the scales from the next multiple of 256 bytes after the words on).
 * A quantized IndexSelect is dequantize followed by orc_index_select, as cpu/mod.rs:86-103 does it. */
int orc_q8_0_quantize(int fp_dt, const void* x, uint64_t numel, uint32_t* words, void* scales);
int orc_q8_0_dequantize(int fp_dt, const uint32_t* words, const void* scales, uint64_t numel, void* y);

int orc_softmax(int dt, const void* x, void* y, size_t rows, size_t cols);
/* shape0 = size of the input's first dimension: the reference broadcasts scale/bias with a
 * vector special case that depends on it (pass 1 to get the mathematically intended result) */
int orc_layer_norm(int dt, const void* x, const void* scale, const void* bias /* nullable */, void* y,
                   size_t rows, size_t cols, float eps, size_t shape0);
int orc_rms_norm(int dt, const void* x, const void* scale, void* y, size_t rows, size_t cols, float eps,
                 size_t shape0);
int orc_group_norm(int dt, const void* x, const void* scale /* nullable */, const void* bias /* nullable */, void* y,
                   size_t B, size_t C, size_t L, size_t groups, float eps);

/* 1 (default): every op also performs the reference's input to_vec copies and its result copy;
 * 0: arithmetic loops only.  Affects timing, never results. */
void orc_set_reference_copies(int on);
/* 0 (default): Sum for f16 accumulates in f32 and rounds once; 1: accumulates in f16 */
void orc_set_f16_sum_mode(int sequential_f16);
/* 1 = hardware F16C conversions, 0 = portable bit-twiddling ones (bit-identical; see tests) */
void orc_set_hw_f16(int on);
int orc_has_hw_f16(void);

/* scalar conversion helpers exported for tests */
uint16_t orc_f32_to_f16(float f);
float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);
float orc_bf16_to_f32(uint16_t h);

/* all_close rule of the reference (crates/ratchet-core/src/tensor.rs:1039-1043): counts elements with
 * !(both NaN || same-signed inf || |a-b| <= atol + rtol*|b|); also returns max abs diff */
size_t orc_count_not_close(int dt, const void* a, const void* b, size_t numel, double atol, double rtol,
                           double* max_abs_diff);

#ifdef __cplusplus
}
#endif
#endif
