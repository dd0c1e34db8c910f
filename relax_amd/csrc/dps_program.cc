// Destination-passing instruction-list executor: the slice of the Relax VM that the
// quantized linear path runs under (RunInstrCall, src/runtime/relax_vm/vm.cc:691-775),
// with a static memory plan in the manner of StaticPlanBlockMemory and whole-program
// HIP graph capture in the manner of RewriteCUDAGraph (python/tvm/relax/pipeline.py:90-91).
#include <algorithm>
#include <cstring>
#include <deque>
#include <string>
#include <vector>

#include "../../include/relax_amd_tvm.h"
#include "../../include/relax_amd_vm.h"
#include "wq_host.h"

namespace wq {
// tvm_packed.cc: the stream PackedFunc calls enqueue on, for the calling thread
void set_stream_override(bool on, void* stream);
WqTVMBackendPackedCFunc find_packed_function(const char* name);
}  // namespace wq

namespace {

constexpr int64_t kAlign = 256;

struct Reg {
  DLTensor dl;
  std::vector<int64_t> shape;
  int64_t bytes = 0;
  bool planned = false;
  int64_t offset = -1;     // planned: workspace offset
  int first = -1, last = -1;  // live range in instruction indices
};

struct Instr {
  std::string name;
  WqTVMBackendPackedCFunc fn;
  std::vector<TVMValue> vals;
  std::vector<int> codes;
  std::vector<int> regs;  // register per argument, -1 for an immediate
};

}  // namespace

struct wq_program {
  std::deque<Reg> regs;  // deque: DLTensor addresses stay valid as registers are added
  std::vector<Instr> instrs;
  bool planned = false;
  int64_t workspace_bytes = 0;
  void* workspace = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

static void drop_graph(wq_program* p) {
  if (p->exec) (void)hipGraphExecDestroy(p->exec);
  if (p->graph) (void)hipGraphDestroy(p->graph);
  p->exec = nullptr;
  p->graph = nullptr;
}

static int add_reg(wq_program* p, const char* who, int code, int bits, int ndim, const int64_t* shape,
                   void* data, int device_type, bool planned) {
  WQ_REQUIRE(p, "%s: null program", who);
  WQ_REQUIRE(ndim >= 0 && ndim <= 8 && (ndim == 0 || shape), "%s: bad rank %d", who, ndim);
  WQ_REQUIRE(bits == 8 || bits == 16 || bits == 32 || bits == 64, "%s: unsupported dtype bits %d", who, bits);
  WQ_REQUIRE(code >= 0 && code <= 2, "%s: unsupported dtype code %d", who, code);
  WQ_REQUIRE(device_type == kDLROCM || device_type == kDLCPU, "%s: unsupported device type %d", who, device_type);
  p->regs.emplace_back();
  Reg& r = p->regs.back();
  int64_t numel = 1;
  for (int i = 0; i < ndim; ++i) {
    if (shape[i] < 0) {
      p->regs.pop_back();
      return wq::fail(WQ_EINVAL, "%s: negative extent", who);
    }
    r.shape.push_back(shape[i]);
    numel *= shape[i];
  }
  r.bytes = numel * (bits / 8);
  r.planned = planned;
  std::memset(&r.dl, 0, sizeof(r.dl));
  r.dl.data = data;
  r.dl.device.device_type = (DLDeviceType)device_type;
  r.dl.device.device_id = 0;
  r.dl.ndim = ndim;
  r.dl.dtype.code = (uint8_t)code;
  r.dl.dtype.bits = (uint8_t)bits;
  r.dl.dtype.lanes = 1;
  r.dl.shape = r.shape.data();
  r.dl.strides = nullptr;
  r.dl.byte_offset = 0;
  p->planned = false;
  return (int)p->regs.size() - 1;
}

extern "C" wq_program_t* wq_program_create(void) { return new wq_program(); }

extern "C" void wq_program_destroy(wq_program_t* p) {
  if (!p) return;
  drop_graph(p);
  delete p;
}

extern "C" int wq_program_add_external(wq_program_t* p, int dtype_code, int dtype_bits, int ndim,
                                       const int64_t* shape, void* data, int device_type) {
  return add_reg(p, "wq_program_add_external", dtype_code, dtype_bits, ndim, shape, data, device_type, false);
}

extern "C" int wq_program_add_planned(wq_program_t* p, int dtype_code, int dtype_bits, int ndim,
                                      const int64_t* shape) {
  return add_reg(p, "wq_program_add_planned", dtype_code, dtype_bits, ndim, shape, nullptr, kDLROCM, true);
}

extern "C" int wq_program_rebind(wq_program_t* p, int reg, void* data) {
  WQ_REQUIRE(p && reg >= 0 && reg < (int)p->regs.size(), "wq_program_rebind: no such register %d", reg);
  WQ_REQUIRE(!p->regs[reg].planned, "wq_program_rebind: register %d is planned storage", reg);
  p->regs[reg].dl.data = data;
  drop_graph(p);  // a captured graph holds the old address: replay must fail until captured again
  return WQ_OK;
}

extern "C" int wq_program_add_call(wq_program_t* p, const char* func, int num_args, const int64_t* args,
                                   const int* kinds) {
  WQ_REQUIRE(p && func, "wq_program_add_call: null argument");
  WQ_REQUIRE(num_args >= 0 && (num_args == 0 || (args && kinds)), "wq_program_add_call: bad argument list");
  Instr in;
  in.name = func;
  in.fn = wq::find_packed_function(func);
  WQ_REQUIRE(in.fn, "wq_program_add_call: no PackedFunc named '%s' in this library", func);
  for (int i = 0; i < num_args; ++i) {
    TVMValue v;
    v.v_int64 = 0;
    if (kinds[i] == 1) {
      WQ_REQUIRE(args[i] >= 0 && args[i] < (int64_t)p->regs.size(),
                 "wq_program_add_call(%s): argument %d names register %lld, which does not exist", func, i,
                 (long long)args[i]);
      v.v_handle = &p->regs[(size_t)args[i]].dl;
      in.codes.push_back(kTVMNDArrayHandle);
      in.regs.push_back((int)args[i]);
    } else if (kinds[i] == 2) {  // an absent optional tensor
      v.v_handle = nullptr;
      in.codes.push_back(kTVMNullptr);
      in.regs.push_back(-1);
    } else {
      WQ_REQUIRE(kinds[i] == 0, "wq_program_add_call(%s): kinds[%d] must be 0, 1 or 2", func, i);
      v.v_int64 = args[i];
      in.codes.push_back(kTVMArgInt);
      in.regs.push_back(-1);
    }
    in.vals.push_back(v);
  }
  const int idx = (int)p->instrs.size();
  for (int r : in.regs)
    if (r >= 0) {
      Reg& reg = p->regs[r];
      if (reg.first < 0) reg.first = idx;
      reg.last = idx;
    }
  p->instrs.push_back(std::move(in));
  p->planned = false;
  drop_graph(p);
  return WQ_OK;
}

// Greedy interval colouring in order of first use: a tensor takes the smallest free
// block that holds it, else the lowest fresh offset.  A block becomes free after the
// last instruction that names its tensor; an instruction's outputs never share with
// its own inputs, because both are live at that instruction.
extern "C" int64_t wq_program_plan(wq_program_t* p) {
  WQ_REQUIRE(p, "wq_program_plan: null program");
  struct Block {
    int64_t offset, size;
    int free_after;  // instruction index after which the block is free
  };
  std::vector<Block> blocks;
  std::vector<int> order;
  for (int i = 0; i < (int)p->regs.size(); ++i)
    if (p->regs[i].planned && p->regs[i].first >= 0) order.push_back(i);
  std::stable_sort(order.begin(), order.end(),
                   [&](int a, int b) { return p->regs[a].first < p->regs[b].first; });
  int64_t top = 0;
  for (int ri : order) {
    Reg& r = p->regs[ri];
    const int64_t need = (r.bytes + kAlign - 1) / kAlign * kAlign;
    int best = -1;
    for (int b = 0; b < (int)blocks.size(); ++b)
      if (blocks[b].free_after < r.first && blocks[b].size >= need &&
          (best < 0 || blocks[b].size < blocks[best].size))
        best = b;
    if (best >= 0) {
      r.offset = blocks[best].offset;
      blocks[best].free_after = r.last;
    } else {
      r.offset = top;
      blocks.push_back({top, need, r.last});
      top += need;
    }
  }
  p->workspace_bytes = top;
  p->planned = true;
  p->workspace = nullptr;
  drop_graph(p);
  return top;
}

extern "C" int64_t wq_program_unplanned_bytes(const wq_program_t* p) {
  if (!p) return 0;
  int64_t s = 0;
  for (const Reg& r : p->regs)
    if (r.planned && r.first >= 0) s += (r.bytes + kAlign - 1) / kAlign * kAlign;
  return s;
}

extern "C" int wq_program_set_workspace(wq_program_t* p, void* base, int64_t bytes) {
  WQ_REQUIRE(p, "wq_program_set_workspace: null program");
  WQ_REQUIRE(p->planned, "wq_program_set_workspace: call wq_program_plan first");
  WQ_REQUIRE(bytes >= p->workspace_bytes, "wq_program_set_workspace: %lld bytes given, %lld needed",
             (long long)bytes, (long long)p->workspace_bytes);
  WQ_REQUIRE(p->workspace_bytes == 0 || (base && (reinterpret_cast<uintptr_t>(base) & (kAlign - 1)) == 0),
             "wq_program_set_workspace: base must be non-null and 256-byte aligned");
  for (Reg& r : p->regs)
    if (r.planned && r.first >= 0) r.dl.data = static_cast<char*>(base) + r.offset;
  p->workspace = base;
  drop_graph(p);
  return WQ_OK;
}

static int check_ready(wq_program* p, const char* who) {
  WQ_REQUIRE(p, "%s: null program", who);
  for (const Reg& r : p->regs)
    if (r.first >= 0 && r.bytes > 0 && !r.dl.data)
      return wq::fail(WQ_EINVAL, "%s: a tensor has no storage (%s)", who,
                      r.planned ? "plan the program and set the workspace" : "external tensor bound to null");
  return WQ_OK;
}

static int run_all(wq_program* p, hipStream_t stream) {
  wq::set_stream_override(true, stream);
  int rc = WQ_OK;
  for (size_t i = 0; i < p->instrs.size(); ++i) {
    Instr& in = p->instrs[i];
    TVMValue rv;
    rv.v_handle = nullptr;
    int rcode = kTVMNullptr;
    if (in.fn(in.vals.data(), in.codes.data(), (int)in.vals.size(), &rv, &rcode, nullptr) != 0) {
      // keep the callee's message, say where it happened
      std::string msg = wq_last_error();
      rc = wq::fail(WQ_EINVAL, "instruction %zu (%s): %s", i, in.name.c_str(), msg.c_str());
      break;
    }
  }
  wq::set_stream_override(false, nullptr);
  return rc;
}

extern "C" int wq_program_run(wq_program_t* p, wq_stream_t stream) {
  if (int rc = check_ready(p, "wq_program_run")) return rc;
  return run_all(p, (hipStream_t)stream);
}

extern "C" int wq_program_capture(wq_program_t* p, wq_stream_t stream_) {
  if (int rc = check_ready(p, "wq_program_capture")) return rc;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(stream != nullptr, "wq_program_capture: the null stream cannot be captured");
  drop_graph(p);
  if (int rc = run_all(p, stream)) return rc;
  WQ_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
  const int rc = run_all(p, stream);
  hipGraph_t g = nullptr;
  const hipError_t e = hipStreamEndCapture(stream, &g);
  if (rc) {
    if (g) (void)hipGraphDestroy(g);
    return rc;
  }
  if (e != hipSuccess) return wq::fail(WQ_EDEVICE, "hipStreamEndCapture failed: %s", hipGetErrorString(e));
  p->graph = g;
  WQ_HIP(hipGraphInstantiate(&p->exec, p->graph, nullptr, nullptr, 0));
  return WQ_OK;
}

extern "C" int wq_program_replay(wq_program_t* p, wq_stream_t stream) {
  WQ_REQUIRE(p && p->exec, "wq_program_replay: nothing captured (call wq_program_capture)");
  WQ_HIP(hipGraphLaunch(p->exec, (hipStream_t)stream));
  return WQ_OK;
}

extern "C" int wq_program_num_instructions(const wq_program_t* p) { return p ? (int)p->instrs.size() : 0; }
