// Definitions shared by the two kernels that run a list of format-A linears in one launch
// (q4g32_gemv_list.hip: one activation row; q4g32_batch_list.hip: 2 .. 32 rows): the descriptor
// table, the device-side completion counters, and the host object behind wq_gemv_list_t.
#ifndef RELAX_AMD_CSRC_GEMV_LIST_COMMON_H_
#define RELAX_AMD_CSRC_GEMV_LIST_COMMON_H_

#include <vector>

#include "wq_device.h"
#include "wq_host.h"

namespace wq {

struct GemvListDesc {  // 128 bytes, device memory
  const char* W;       // uint32 [N, K/8]
  const char* S;       // fp16   [N, K/32]
  const half_t* x;     // fp16   [M, K]   (M: a property of the list, 1 .. 32)
  const half_t* bias;  // fp16   [N] or null
  const half_t* residual;  // fp16 [M, N] or null
  half_t* y;           // fp16   [M, N]
  int32_t N;
  int32_t q;           // row groups / workgroups  (a row group is 2^gs consecutive rows)
  uint32_t g_dep;      // bits 0..15: K / 32; bits 16..30: 1 + the linear of this list that writes x (0: none);
                       // bit 31: a later linear reads y
  uint16_t rem;        // row groups % workgroups
  uint16_t off;        // rotation: workgroup b owns the row groups local * workgroups + ((b - off) mod workgroups)
  // words 16 ..: the batch kernels only.  A linear is run by ONE group of workgroups: those with
  // b mod 2^gmod_log2 == gidx (member c = b >> gmod_log2 of workgroups >> gmod_log2), or, with gmod_log2 = 0x80,
  // those whose XCD (b mod 8) is in the mask gidx (members counted in order of b); q, rem and off
  // then count within the group.
  uint8_t gmod_log2, gidx;
  uint8_t rows;  // rows of x and y of this entry (the M of the launch)
  // words 17 ..: the one-row kernel only.
  uint8_t ts;          // log2 of the rows a compute wavefront takes at a time (0 .. gs)
  uint32_t x_off;      // LDS byte offset of the linear's activations (the workgroup's LDS is dealt as a ring)
  int32_t free_after;  // ... which may be written once this many linears of the list have been flushed
  uint8_t szl;         // lists of AutoGPTQ layers: log2 of (group size / 32); S then holds (scale, zero point + 1) pairs
  uint8_t pad0[3];
  const int32_t* perm; // ... and the row order of the layer, int32 [K], or null: position k' of a row of W multiplies x[perm[k']]
  uint8_t pad[40];
};
static_assert(sizeof(GemvListDesc) == 128, "descriptor layout");
constexpr uint32_t kSignal = 1u << 31;  // a later linear reads y

typedef const GemvListDesc __attribute__((address_space(4)))* gemv_desc_ptr;  // scalar loads

// xp[k'] = x[perm[k']], k' < K: the activations of an AutoGPTQ layer with a row order whose x comes from outside the list
struct GatherJob {
  const half_t* x;
  const int32_t* perm;
  half_t* xp;
  int64_t K;
};
static_assert(sizeof(GatherJob) == 32, "job layout");

constexpr int kCounterStride = 16;   // ints between two counters (64 bytes: one cache line each)
constexpr int kCountersPerLinear = 8;
constexpr int kBufferFlags = 0x00020000;  // buffer resource word 3: 32-bit data format, no swizzle
constexpr int kDeviceScope = 16;          // cache policy bit sc1: the access is coherent over the whole device

// error word: 1 + the linear a consumer waited for in vain, or kBatchInternalWait + a code: a hand-over
// inside a workgroup of the batch kernel that did not come
constexpr int kBatchInternalWait = 1 << 20;

// sync layout (ints): [lin][8] counters at stride kCounterStride, then `finished`, then `error`
__host__ __device__ inline int sync_counter_index(int lin, int k) { return (lin * kCountersPerLinear + k) * kCounterStride; }
__host__ __device__ inline int sync_finished_index(int nlin) { return sync_counter_index(nlin, 0); }
__host__ __device__ inline int sync_error_index(int nlin) { return sync_counter_index(nlin, 1); }
__host__ __device__ inline int sync_ints(int nlin) { return sync_counter_index(nlin, 2); }

__device__ __forceinline__ void lds_done_then_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

__device__ __forceinline__ void lds_spin_until(const int* flag, int target) {
  while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < target) __builtin_amdgcn_s_sleep(1);
  asm volatile("" ::: "memory");  // LDS is served in order: what was written before the flag is visible now
}

}  // namespace wq

struct wq_gemv_list {
  std::vector<wq::GemvListDesc> descs;
  int n = 0;
  void* table = nullptr;  // device: descriptors
  int* sync = nullptr;    // device: counters
  int blocks = 0, threads = 0;
  size_t lds = 0;
  int xbuf_bytes = 0, ybuf_floats = 0;
  int ybuf0 = 0;  // LDS byte offset of the row-sum buffers (one-row kernel)
  int late = 0, deps = 0;
  int nb = 2;
  int gs = 2;  // log2 of the rows per row group: 4 consecutive rows (8 KiB at K = 4096) per workgroup at a time
  long long spin_limit = 200000000;  // 2 s of the 100 MHz wall clock
  void* gather_table = nullptr;  // device: jobs of the gather kernel that runs in front of an AutoGPTQ list (GatherJob[gather_jobs])
  int gather_jobs = 0, gather_blocks = 0;
  bool zp = false;         // AutoGPTQ layers: a (scale, zero point + 1) pair per group instead of a scale per 32 columns
  int M = 1;               // activation rows of the launch; > 1: the batch kernel (q4g32_batch_list.hip) and the fields below
  int batch_u = 0;         // chunks per tile and wavefront (4: M <= 16; 2: beyond)
  int batch_groups = 1;    // groups of workgroups that run different linears side by side (0: sets of XCDs per linear)
  int batch_nxb = 0;       // panels of activations in LDS
  int batch_ring = 0;      // items the compute wavefronts may spread over (slots of scales and of partial sums)
  int batch_acc_tiles = 0; // tiles whose sums LDS keeps between the panels of a linear: a chunk of the workgroup's tiles
  bool batch_chunked = false;  // some linear is walked in several chunks
  bool batch_rows = false;     // more than 16 rows: the kernel whose wavefronts own rows of W (q4g32_batch_rows_kernel)
};

namespace wq {

constexpr size_t kListAlign = 256;

inline size_t list_table_bytes(int n) { return ((size_t)n * sizeof(GemvListDesc) + kListAlign - 1) / kListAlign * kListAlign; }


// q4g32_batch_list.hip: launch shape and LDS plan of a list with 2 .. 32 activation rows (fills
// l->blocks, threads, lds, batch_*; the descriptors' q / rem / off), and its launch
int batch_list_plan(wq_gemv_list* l);
int batch_list_launch(wq_gemv_list* l, hipStream_t stream);

}  // namespace wq
#endif  // RELAX_AMD_CSRC_GEMV_LIST_COMMON_H_
