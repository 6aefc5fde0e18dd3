/*
 * Test hooks of libmxfp8_gfx950.so.  NOT part of the ABI in mxfp8.h: nothing in the product path
 * calls them, their meaning may change with the kernels, and they are process-wide (a test sets
 * one, runs, and sets it back).  mx_debug_set_prof and the kernel instances it switches to exist
 * only in a library built with -DMX_TIMING_BUILD; the product build leaves them out.
 */
#ifndef MXFP8_DEBUG_H_
#define MXFP8_DEBUG_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 0: pick the dense GEMM kernel by shape (default); 1 / 2: the one-tile-per-workgroup kernel with
 * 256x256 / 128x128 tiles for every shape; 3: the persistent kernel for every shape it can take,
 * however few tiles there are. */
void mx_debug_force_kernel(int which);

/* > 0: number of persistent workgroups of the persistent kernel, rounded up to a multiple of 8
 * (also lowers how many tiles one grouped launch covers); 0: one per CU (default). */
void mx_debug_set_grid(int workgroups);

/* -DMX_TIMING_BUILD only.  Device buffer of 256 * 4 * 8 uint64 that the timing build of the persistent kernel fills with
 * per-wave cycle counts {copy wait, barriers, step body, epilogue, ...}; NULL switches the timing
 * build off (default). */
void mx_debug_set_prof(void* device_buffer);

/* HBM yardsticks for bench.py: the plainest streaming kernels (16 bytes per lane, nontemporal),
 * kind 0 = copy `bytes` from src to dst, 1 = read `bytes` of src (dst: 16 bytes that are never
 * written for ordinary data), 2 = write `bytes` to dst, 3 = read `bytes` of src and write
 * `bytes` / 2 to dst (the read : write mix of a one-direction cast).  bytes % 16 == 0, 16-byte aligned.
 * Returns an mx_status_t. */
int mx_debug_stream(int kind, const void* src, void* dst, int64_t bytes, void* stream);

/* Matrix-pipe yardstick for bench.py: `workgroups` x 4 waves run `iters` rounds of independent
 * scaled fp8 MFMAs on operands that stay in registers (shape 32: 16 x v_mfma_scale_f32_32x32x64
 * per round, shape 16: 64 x v_mfma_scale_f32_16x16x128; 2 * 32 * 32 * 64 * 16 flop per wave and
 * round either way), no LDS or memory traffic in the loop.  `operands`: 16 * 256 * 32 bytes of e4m3
 * codes (32-byte aligned), `out`: workgroups * 256 floats.  Shapes 1601 / 1604 / 1608 run the
 * 16x16x128 form in a fixed order in which 1 / 4 / 8 MFMAs in a row share an operand fragment
 * (1604 is the order of the GEMM kernel's K loop).  Returns an mx_status_t. */
int mx_debug_mfma_only(int shape, const void* operands, void* out, int workgroups, int iters, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MXFP8_DEBUG_H_ */
