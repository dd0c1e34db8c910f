/*
 * relax_amd_vm.h — a destination-passing instruction-list executor for the
 * PackedFuncs of this library: the part of the Relax VM that the weight-only
 * quantized linear path runs under.
 *
 * What it stands in for in the reference:
 *   - VirtualMachineImpl::RunInstrCall (src/runtime/relax_vm/vm.cc:691-775): each
 *     instruction names a PackedFunc and passes registers (tensors) and immediates
 *     with the TVM calling convention, inputs first, outputs last;
 *   - StaticPlanBlockMemory (python/tvm/relax/pipeline.py:90; src/relax/transform/
 *     static_plan_block_memory.cc): intermediate tensors get storage from one
 *     workspace, reused when live ranges do not overlap;
 *   - RewriteCUDAGraph (python/tvm/relax/pipeline.py:91): the whole instruction list
 *     is captured once into a HIP graph and replayed.
 * It executes nothing but PackedFuncs of this library (looked up by their dotted
 * global name or C symbol) and never allocates device memory: the caller supplies
 * the workspace.
 *
 * All functions return 0 or a negative WQ_E* code with wq_last_error() set, except
 * where noted.  A program is used from one thread at a time.
 */
#ifndef RELAX_AMD_VM_H_
#define RELAX_AMD_VM_H_

#include <stdint.h>

#include "relax_amd_tvm_abi.h"
#include "relax_amd_wq.h"

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

typedef struct wq_program wq_program_t;

wq_program_t* wq_program_create(void);
void wq_program_destroy(wq_program_t* p);

/* Declares a tensor register and returns its index (>= 0), or a negative code.
 * dtype as in DLDataType (code, bits; lanes = 1), device_type kDLROCM (10) or kDLCPU (1).
 * External tensors (weights, inputs, results the caller wants to keep) carry their
 * own storage; planned tensors get theirs from the workspace (alloc_tensor in the
 * reference, src/relax/transform/call_tir_rewrite.cc:88-96). */
int wq_program_add_external(wq_program_t* p, int dtype_code, int dtype_bits, int ndim,
                            const int64_t* shape, void* data, int device_type);
int wq_program_add_planned(wq_program_t* p, int dtype_code, int dtype_bits, int ndim,
                           const int64_t* shape);
/* Points an external register at other storage of the same shape (next batch of inputs).
 * A captured graph keeps the addresses it was captured with, so the graph is dropped here:
 * wq_program_replay fails ("nothing captured") until wq_program_capture is called again. */
int wq_program_rebind(wq_program_t* p, int reg, void* data);

/* Appends `func(args...)`.  kinds[i] = 1: args[i] is a tensor register, passed as an
 * NDArray handle (type code 13) as the VM does; kinds[i] = 0: args[i] is an integer
 * immediate (type code 0); kinds[i] = 2: a null handle (type code 4) for an optional tensor
 * that is absent.  Argument order is the PackedFunc's: inputs, then outputs. */
int wq_program_add_call(wq_program_t* p, const char* func, int num_args, const int64_t* args,
                        const int* kinds);

/* Assigns workspace offsets to the planned tensors from their live ranges (first to
 * last instruction that names them); tensors whose ranges do not overlap share
 * storage.  Returns the workspace size in bytes (>= 0) or a negative code. */
int64_t wq_program_plan(wq_program_t* p);
/* Sum of the sizes of all planned tensors, i.e. the workspace without reuse (for reports). */
int64_t wq_program_unplanned_bytes(const wq_program_t* p);
/* base: device memory of at least wq_program_plan() bytes, 256-byte aligned. */
int wq_program_set_workspace(wq_program_t* p, void* base, int64_t bytes);

/* Runs every instruction in order on `stream`, without synchronising. */
int wq_program_run(wq_program_t* p, wq_stream_t stream);
/* Runs once eagerly (so that one-time kernel set-up happens outside the capture), then
 * captures one run on `stream` (which must not be the null stream) into a HIP graph. */
int wq_program_capture(wq_program_t* p, wq_stream_t stream);
/* Launches the captured graph on `stream`. */
int wq_program_replay(wq_program_t* p, wq_stream_t stream);

int wq_program_num_instructions(const wq_program_t* p);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* RELAX_AMD_VM_H_ */
