/*
 * cigemm_probe.h -- measurement aids of the MI355X (gfx950) quantization-GEMM library.
 *
 * Nothing here has a counterpart in the reference, and nothing here is part of the drop-in
 * boundary (that is cigemm.h).  These entry points live in a library of their own,
 * libcigemm_probe.so, which the benchmark and the probe tests load beside libcigemm.so; they
 * take a handle created by cigemmCreate() and use its stream and workspace.  They exist so
 * that the benchmark can say, from the same run, what the chip sustains and where the time of
 * one launch of the product kernel goes.
 */
#ifndef CIGEMM_PROBE_H_
#define CIGEMM_PROBE_H_

#include "cigemm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Launches a register-resident matrix-core loop (no memory traffic inside the loop) on every
 * compute unit of the handle's device, on the handle's stream: kind 0 = bf16 32x32x16,
 * 1 = fp16 32x32x16, 2 = int8 32x32x32, 3 = bf16 16x16x32, 4 = fp16 16x16x32,
 * 5 = int8 16x16x64, 6 = fp32 32x32x2; random_bits 0 = constant operands, 1 = pseudo-random
 * operand bits (sustained clocks depend on the data); `iters` loop trips of 12 instructions
 * per wave.  *ops_per_launch receives 2.M.N.K summed over all instructions, for the caller to
 * divide by the time it measures. */
CIGEMM_API cigemmStatus_t cigemm_probe_mfma(cigemmHandle_t handle, int kind, int random_bits,
                                            int iters, int64_t* ops_per_launch);

/* What the other instructions of the tile kernel's main loop cost in matrix-core issue time.
 * Launches `workgroups` workgroups (1 .. number of compute units) of four waves, one per
 * SIMD, each looping `iters` times over one "stage": 32 bf16 32x32x16 matrix instructions on
 * 16 accumulator tiles (1024 issue cycles when nothing else delays them), with, spread evenly
 * between them and pinned in place like the product kernel's schedule,
 *   n_dma        global_load_lds_dwordx4 instructions (0, 2, 4 or 8; the product issues 8 per
 *                wave and stage on average) from a buffer that stays in the L2 into LDS that
 *                nothing reads,
 *   n_lds_reads  LDS fragment reads (0 or 24: 8 of 16 bytes and 16 transposing 8-byte ones,
 *                the product's count per stage), whose results feed the next stage's matrix
 *                instructions,
 *   barrier      0 / 1 workgroup barriers per stage (the product has one),
 *   placement    where the DMA instructions sit among the 32 slots between one barrier and the
 *                next (a slot = one matrix instruction; 0..15 the k-step after the barrier):
 *                0 = the first n_dma slots after the barrier, every wave alike; 1 = every second
 *                slot; 2 = every second slot, waves 1 and 3 on the odd ones; 3 = every fourth
 *                slot over both k-steps; 4 = the same, wave w one slot after wave w - 1; 5, 6 =
 *                back to back, wave w four / eight slots after wave w - 1; 7 = every second
 *                slot, wave w eight slots after wave w - 1 (1..7 need n_dma 8, n_lds_reads 24),
 *   mfma         1 = as described; 0 = the same loop without its matrix instructions (their
 *                slots stay empty; the fragments are consumed by one vector instruction each):
 *                what the stage's memory instructions take by themselves (placement 0 or 1,
 *                n_dma 0 or 8),
 *   src_kib_per_wave  bytes of DMA source a wave walks through, 8 KiB per stage, round and
 *                round: 8 = the same lines every stage (vector-L1 hits), 32 and more = lines
 *                the L1 no longer holds (served by the L2, as the product's are).
 * Synchronises the stream.  result[0..3] receive: shader cycles per stage, averaged over the
 * waves; the slowest wave's; the shader clock (GHz) held meanwhile; microseconds per launch
 * from the first wave's start to the last wave's end. */
CIGEMM_API cigemmStatus_t cigemm_probe_issue_cost(cigemmHandle_t handle, int n_dma,
                                                  int n_lds_reads, int barrier, int placement,
                                                  int mfma, int src_kib_per_wave, int workgroups,
                                                  int iters, double* result);

/* Runs ONE launch of the 256-row, four-wave LDS-tiled matrix-core kernel (the product kernel
 * with four timestamps added per workgroup) on the handle's stream, waits for it, and reduces
 * the stamps: kind 0 = bf16 (A, B, C as in cigemm_gemm_bf16), 1 = int8 K x N operands, int32
 * out (as cigemm_gemm_i8_i32 with CIGEMM_B_KN); 2 and 3 = the same two on the
 * two-workgroups-per-unit form of the kernel (128-row tiles; "stage" then means a stage of
 * such a tile, 512 matrix-core issue cycles instead of 1024); 4 = fp16 (as cigemm_gemm_f16);
 * 5 = int8 with N x K weights on 192-row tiles, int32 out (as cigemm_gemm_i8_i32 with
 * CIGEMM_B_NK; the form the quantized linear-layer shape runs on: 768 issue cycles per stage).
 * kind + 16 (kinds 0, 1 and 4 only): the same launch with every workgroup computing output
 * tile (0, 0) -- all read the same two operand panels, which stay in every L2, and store the same
 * values to the same place -- i.e. what the launch takes when no operand read leaves the L2 (C
 * then holds the right values in its first tile only).
 * Same shape and alignment conditions as the tile kernel, N % 8 == 0.
 * phases[0..7] receive, averaged over the workgroups: microseconds from workgroup start to the
 * first stage in registers; of the main loop; of the epilogue until its stores are
 * acknowledged; microseconds from the first workgroup's start to the last one's end; shader
 * cycles per 64-byte stage of k in the main loop; shader clock (GHz) held in the main loop
 * (0 when the main loop is shorter than one tick of the wall clock); microseconds from the
 * first workgroup entering its epilogue to the last one's end; number of workgroups;
 * phases[8..11]: main-loop shader clock (GHz) of the slowest and of the fastest of the chip's
 * compute dies (XCDs: each holds its own clock, and every die gets the same number of
 * workgroups); microseconds from the first workgroup's start to the end of a compute unit's last
 * workgroup, averaged over the units (the launch itself, phases[3], ends with the slowest unit);
 * number of compute units that ran a workgroup.  `phases` must hold 12 doubles.
 * Synchronises the stream; meant for profiling runs, not for the hot path. */
CIGEMM_API cigemmStatus_t cigemm_probe_tile_phases(cigemmHandle_t handle, int kind, int64_t M,
                                                   int64_t N, int64_t K, const void* A,
                                                   int64_t lda, const void* B, int64_t ldb,
                                                   void* C, int64_t ldc, double* phases);

/* The GEMMs of cigemm.h on the two-workgroups-per-unit form of the tile kernel: 128 x 256
 * tiles, four waves of 64 x 128, 80 KiB of LDS, two workgroups resident per compute unit and
 * half a tile out of phase.  K x N operands only.  Same arguments, shape conditions and
 * results (bit for bit on int8 and on exact-arithmetic 16-bit inputs) as cigemm_gemm_bf16 /
 * _f16 / _i8_i32 / _i8_dequant on the tile kernel.  The library itself never chooses this
 * form: it fills more matrix-core issue slots and runs slower under the chip's power limit. */
CIGEMM_API cigemmStatus_t cigemm_probe_gemm_bf16_paired(cigemmHandle_t handle, int64_t M,
                                                        int64_t N, int64_t K, const uint16_t* A,
                                                        int64_t lda, const uint16_t* B,
                                                        int64_t ldb, uint16_t* C, int64_t ldc);
CIGEMM_API cigemmStatus_t cigemm_probe_gemm_f16_paired(cigemmHandle_t handle, int64_t M,
                                                       int64_t N, int64_t K, const uint16_t* A,
                                                       int64_t lda, const uint16_t* B,
                                                       int64_t ldb, uint16_t* C, int64_t ldc);
CIGEMM_API cigemmStatus_t cigemm_probe_gemm_i8_i32_paired(cigemmHandle_t handle, int64_t M,
                                                          int64_t N, int64_t K, const int8_t* A,
                                                          int64_t lda, const int8_t* B,
                                                          int64_t ldb, int32_t* C, int64_t ldc);
CIGEMM_API cigemmStatus_t cigemm_probe_gemm_i8_dequant_paired(
    cigemmHandle_t handle, int64_t M, int64_t N, int64_t K, const int8_t* A, int64_t lda,
    const int8_t* B, int64_t ldb, const float* scaleA, cigemmScaleMode_t scaleA_mode,
    const float* scaleB, cigemmScaleMode_t scaleB_mode, void* out, cigemmOutType_t out_type,
    int64_t ldo, int32_t* acc_out, int64_t ldacc);

/* Test aid for the recovery of a handle whose split-K call was cut short: overwrites the first
 * `count` arrival counters and the first `count` exchange words of the handle's workspace with
 * `value` (a synchronous copy on the handle's stream), as an aborted kernel would leave them,
 * and, when `mark_dirty` is non-zero, records on the handle what a failed launch records, so
 * that the next GEMM call clears them first.  With mark_dirty = 0 the caller is expected to
 * call cigemmResetWorkspace(). */
CIGEMM_API cigemmStatus_t cigemm_probe_dirty_workspace(cigemmHandle_t handle, int count,
                                                       uint32_t value, int mark_dirty);

/* Planner evidence: imposes the tile kernel's plan on the handle's following GEMM calls (those
 * the tile kernel serves): output tiles of `tile_rows` rows (64, 128, 192 or 256) over
 * `k_ranges` ranges of K (1 = unsplit; rounded to ranges of an even number of 64-byte stages;
 * run unsplit when the handle's workspace cannot hold the partial sums).  tile_rows = 0 hands
 * the choice back to the library.  cigemmGetLastPlan() reports what ran.  Results are those of
 * the library's own plan up to the order of the K ranges' floating-point sum. */
CIGEMM_API cigemmStatus_t cigemm_probe_force_tile_plan(cigemmHandle_t handle, int tile_rows,
                                                       int k_ranges);

#ifdef __cplusplus
}
#endif
#endif /* CIGEMM_PROBE_H_ */
