/*
 * relax_amd_wq_testing.h — hooks for tests and measurement.  Not part of the drop-in
 * boundary: nothing in the reference calls these, and a deployment need not ship them.
 *
 * (1) Work-split overrides, exported by librelax_amd_wq.so.  Every entry point of
 *     relax_amd_wq.h chooses its kernel and launch shape from the problem size; the parity tests
 *     use these to run EVERY work split of a kernel on every shape.  An override belongs to the
 *     calling thread (thread-local state): set it, call the entry point, reset it to 0; other
 *     threads keep the automatic choice.
 * (2) Calibration kernels, in a library of their own (librelax_amd_wq_calibrate.so): the measured
 *     ceilings reported next to the vendor peaks (methodology precedent in the reference: the
 *     cache-flush protocol of src/runtime/profiling.cc:879-895).
 */
#ifndef RELAX_AMD_WQ_TESTING_H_
#define RELAX_AMD_WQ_TESTING_H_

#include <stdint.h>

#include "relax_amd_wq.h"

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* Tile configuration of the MFMA GEMMs (format A and B): 1..4 the register-staged kernel
 * (256x256, 128x256, 64x128, 128x128), 11..18 the LDS-staged kernel; 0 = from the shape. */
void wq_debug_set_gemm_config(int cfg);
/* Split the tiles of the last, partly filled round into row slices (default 1). */
void wq_debug_set_gemm_tail_split(int on);
/* Decode GEMV: rows per wavefront (1, 2, 4) and scale groups per lane; 0 = from the shape.  Format B: column
 * groups per wavefront (1, 2) at one row; a value other than 0 also keeps one or two rows of a narrow matrix
 * on the streaming kernel, which the dispatch otherwise hands to the small-batch kernel. */
void wq_debug_set_gemv_config(int rows, int gpl);
/* Format B decode GEMV: wavefronts that share a column group and split K between them (1, 2, 4, 8); 0 = from
 * the shape (int4 at one row of a narrow matrix; otherwise 1). */
void wq_debug_set_intb_gemv_k_split(int ways);
/* Decode GEMV: persistent workgroups per CU; 0 = from the shape. */
void wq_debug_set_gemv_blocks_per_cu(int n);
/* Small-batch kernel: wavefronts side by side (1, 2, 4, 8), ring slots, and which kernel
 * (waves 1: ring, 2: activations in registers); 0 = from the shape. */
void wq_debug_set_skinny_config(int nw, int stages, int waves);
/* How a list of 2 .. 32 activation rows was planned: the number of equal groups of workgroups that run
 * different linears side by side, or 0 if the linears of the (short) list share the 8 XCDs in sets sized by
 * their cost; -1 for a list of one activation row. */
int wq_debug_gemv_list_groups(const wq_gemv_list_t* list);

/* ---- librelax_amd_wq_calibrate.so ---- */
/* Issues `iters` x 8 independent v_mfma_f32_32x32x16_f16 per wavefront, four wavefronts
 * per CU, no memory traffic.  scratch: device memory of >= 4 bytes x 256 x number of CUs.
 * *flops receives the floating-point operations of one launch. */
int wq_calibrate_mfma_f16(void* scratch, int64_t scratch_bytes, int iters, double* flops,
                          wq_stream_t stream);
/* Streams `bytes` of device memory through the CUs with 16-byte loads and no store
 * (scratch: 4 bytes of device memory, practically never written). */
int wq_calibrate_read(const void* src, int64_t bytes, void* scratch, wq_stream_t stream);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* RELAX_AMD_WQ_TESTING_H_ */
