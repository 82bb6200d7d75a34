/* kapy_probe.h - measurement-only entry points of libkapy_probe.so (gfx950), beside libkapy_hip.so and not part of it.
 *
 * Nothing here is needed to run a kapy program: these kernels exist so that the rates of the product's kernels can be read
 * against what the device sustains, and so that a test can bind the exported MFMA operand layouts to the hardware.  The
 * benchmark and the tests load this library; the product library does not.  The reference emits code and never runs it, so
 * there is no interface of it to cite beyond the instructions it names (MatmulOpToLLVM.cpp:269-311,
 * LdGlobalOpToLLVM.cpp:60-145).  Status codes, element types and impl_way values are kapy_hip.h's; a failing call leaves its
 * message with the product library (its kapy_last_error).  All pointers are device pointers unless said otherwise; stream is a hipStream_t. */
#ifndef KAPY_PROBE_H
#define KAPY_PROBE_H

#include "kapy_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Runs ONE matrix instruction of `impl_way` (16..19) on one wavefront, registers in and out, through the same
 * instruction wrapper the matmul kernels multiply with: lhs_regs / rhs_regs hold, for lane 0..63 back to back, the
 * lane's kpack operand elements (kapy_matmul_layouts which = 0 / 1 say which elements those are), acc_regs gets each
 * lane's m*n/64 fp32 accumulator registers (which = 2, or 3 with exchanged != 0).  The counterpart of the coordinate ->
 * loop-iv tables of MatmulOpToLLVM.cpp:94-123 made observable: a test scatters a tile by the layouts, calls this and
 * gathers the product by the layouts, which fails if they do not describe the hardware.  Device pointers. */
int kapy_mfma_probe(int32_t impl_way, int32_t lhs_dtype, int32_t rhs_dtype, int32_t exchanged, const void *lhs_regs, const void *rhs_regs,
                    float *acc_regs, void *stream);

/* What the device sustains, so that a kernel's rate can be read against a reproducible ceiling as well as against the
 * data-sheet peak (the reference emits code and never runs it; nothing there to cite beyond the instructions it names,
 * MatmulOpToLLVM.cpp:269-311, LdGlobalOpToLLVM.cpp:60-145).
 * kapy_probe_mfma: every CU runs `iterations` rounds of independent matrix instructions of `impl_way` (16..19) with the
 * register blocking of the tiled matmul and no memory traffic.  operands: 128 KiB of device memory holding operand
 * values of `dtype` (the power drawn, and so the clock held, depends on them); sink: one float per lane (workgroups *
 * 256); ticks (may be NULL): per workgroup {shader clock at start, at end, 100 MHz timer at start, at end}.  Reports
 * the workgroups launched and the flops of the launch. */
int kapy_probe_mfma(int32_t impl_way, int32_t dtype, const void *operands, int32_t iterations, float *sink, uint64_t *ticks, int32_t *workgroups,
                    int64_t *flops, void *stream);
/* kapy_probe_copy: dst <- src, `bytes` (a multiple of 16) moved 16 bytes per lane with 1, 2, 4, 8 or 16 vectors per lane in
 * flight, ordinary or non-temporal loads / stores, in one pass (persistent_per_cu = 0) or by that many persistent
 * workgroups per CU striding over the buffers.  ticks as above (4 values per workgroup; may be NULL). */
int kapy_probe_copy(const void *src, void *dst, int64_t bytes, int32_t vectors_per_lane, int32_t nt_load, int32_t nt_store, int32_t persistent_per_cu,
                    uint64_t *ticks, int32_t *workgroups, void *stream);
/* kapy_probe_read: the same stream without the stores.  Every lane folds what it reads (`bytes` of src, 16 bytes per lane
 * and load, 1 .. 16 loads in flight, ordinary or non-temporal, one pass or persistent) into a word that is never written in
 * practice (sink: one word per workgroup, at least 65536 * 16 / vectors_per_lane words for one pass over 256 MiB): the
 * ceiling of a kernel that streams a large operand and writes little. */
int kapy_probe_read(const void *src, int64_t bytes, int32_t vectors_per_lane, int32_t nt_load, int32_t persistent_per_cu, uint32_t *sink, int32_t *workgroups,
                    void *stream);

/* kapy_probe_copy_runs: dst <- src for a [rows][row_bytes] matrix, moved in pieces of run_bytes (256, 512, 1024, 2048 or 4096)
 * contiguous bytes: a workgroup owns 32 KiB / run_bytes rows of one run each.  What run length alone costs: a transposing
 * kernel reads and writes runs as long as its tile is wide. */
int kapy_probe_copy_runs(const void *src, void *dst, int64_t rows, int64_t row_bytes, int32_t run_bytes, void *stream);
/* kapy_probe_issue: what a wave can issue beside its matrix instructions.  One wave per SIMD (the tiled matmul's occupancy)
 * runs `iterations` tiles of independent matrix instructions of `impl_way` (KAPY_MFMA_16X16X32_16B: 128 per tile, or
 * KAPY_MFMA_16X16X128_F8: 64 per tile - 2048 matrix-pipe clocks either way) with, behind every instruction, filler 0: nothing;
 * 1: `count` (1, 2, 3, 4, 6, 8) scalar instructions; 2: `count` (1 .. 4) vector ALU instructions; 3: the reads and loads of
 * the tiled matmul's steady-state loop (32 LDS reads of 16 bytes per lane and 16 LDS-direct loads of 1 KiB per wave and
 * tile, from `src`: 8 windows of 2 MiB, one per XCD, that stay in the L2s); 4: that loop with the rhs kept off the LDS (16 LDS
 * reads and 8 LDS-direct loads for the lhs, the wave's 16 rhs fragments as 16-byte loads into registers).  sink: one float per lane (workgroups * 256,
 * never written in practice).  Outputs: the workgroups launched and the flops of the launch. */
int kapy_probe_issue(int32_t impl_way, int32_t filler, int32_t count, const void *src, int32_t iterations, float *sink, int32_t *workgroups, int64_t *flops,
                     void *stream);
/* kapy_probe_l2_read: every workgroup (workgroups_per_cu per CU, 256 lanes) reads the window of `src` that belongs to its XCD
 * (src holds 8 windows of window_bytes, one per XCD; a window of a few MiB stays in that XCD's L2) `iterations` x 32 KiB, 16
 * bytes per lane and instruction, as LDS-direct loads (to_lds = 1, the form the tiled matmul kernels use) or into registers.
 * Outputs: the workgroups launched and the bytes the launch reads.  sink: one word per workgroup (never written in practice). */
int kapy_probe_l2_read(const void *src, int64_t window_bytes, int32_t iterations, int32_t workgroups_per_cu, int32_t to_lds, uint32_t *sink,
                       int32_t *workgroups, int64_t *bytes_read, void *stream);

/* A copy with the access footprint of the 16-bit tile transpose (a workgroup moves 128 rows x 256 bytes of a [rows][row_bytes]
 * matrix, one wave instruction touches four 256-byte pieces of four rows), untransposed, directly or through an LDS tile and
 * a barrier: what that footprint and that detour cost against kapy_probe_copy. */
int kapy_probe_copy_tiled(const void *src, void *dst, int64_t rows, int64_t row_bytes, int32_t through_lds, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* KAPY_PROBE_H */
