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

/* Fused decode linears.  A run of consecutive relax_amd.q4f16_1_matmul[_bias[_residual]]
 * instructions with the same number M <= 32 of rows of x (the decode step of a stack of quantized
 * linears; K % 256 == 0 where M > 1) is executed as ONE launch of the list kernel if it is long
 * enough for that to be the faster way: 2 instructions at M <= 4, 8 at M <= 8, 16 at M <= 16, 8 beyond
 * (a short list with several rows of x cannot spread the loads of the activations over small groups
 * of workgroups).  A run of relax_amd.autogptq_matmul instructions with one row of x and a group size of
 * 32 << t (t = 0 .. 6), with or without a row order, is fused the same way from 2 instructions on
 * (wq_gptq_gemv_list_create; a gather workspace argument is then not used); the two kinds do not share a run.
 * The list kernel is wq_q4g32_gemv_list_* of relax_amd_wq.h; one kernel per
 * instruction is what the reference's VM does with the generated kernels
 * of python/tvm/dlight/gpu/gemv.py.  Inside such a run, independent linears are moved between a
 * producer and its consumer (results are unchanged: every true, anti and output dependence
 * between the instructions is kept), and the planned tensors of the run do not share storage.
 * The descriptor tables live in the workspace (wq_program_plan accounts for them) and are
 * uploaded by the first wq_program_run / wq_program_capture after the plan or a rebind.
 * Option "fuse_decode" (default 1) switches this off; set it before wq_program_plan.
 * Option "spin_limit_us": the longest a fused run's wait for a producer linear may last, in microseconds
 * (default: 2 s, the lists' own; wq_q4g32_gemv_list_set_spin_limit); drops a captured graph. */
int wq_program_set_option(wq_program_t* p, const char* name, int value);
/* Number of runs that are executed fused (after the first run or capture). */
int wq_program_num_fused_groups(const wq_program_t* p);
/* A run that could not be built as a list (operands that alias in a way the list kernel cannot order) is
 * executed instruction by instruction, which is always valid; this returns what the list kernel said about
 * run `group` (numbered as found by wq_program_plan, 0 ..), or "" for a run that is fused or unknown. */
const char* wq_program_unfused_reason(const wq_program_t* p, int group);
/* The order in which run `group` walks its instructions: writes up to `capacity` instruction
 * indices to `order` and returns how many the run holds. */
int wq_program_fused_order(const wq_program_t* p, int group, int* order, int capacity);
/* Synchronises `stream` and reports a device-side wait of a fused run that hit its spin limit
 * (see wq_q4g32_gemv_list_status). */
int wq_program_status(wq_program_t* p, wq_stream_t stream);
/* The same check without synchronising (see wq_q4g32_gemv_list_poll): enqueues asynchronous copies of the
 * error words of the fused runs, one per run in program order, into host_words[0 .. capacity) (pinned host
 * memory of the caller) and returns the number of fused runs (>= 0; words beyond `capacity` are not copied),
 * or a negative code.  All words zero once the stream has passed: no wait has run out. */
int wq_program_poll(wq_program_t* p, int* host_words, int capacity, wq_stream_t stream);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* RELAX_AMD_VM_H_ */
