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

// A run of consecutive decode linears (relax_amd.q4f16_1_matmul*, a few rows of x each, or
// relax_amd.autogptq_matmul with one row) that is executed as ONE launch of the list kernel
// (wq_q4g32_gemv_list_* / wq_gptq_gemv_list_create).
struct FusedGroup {
  int first = 0, last = 0;     // instruction indices, inclusive
  int64_t ws_bytes = 0;        // bytes of workspace of the list (wq_q4g32_gemv_list_workspace_bytes, or the AutoGPTQ size)
  std::vector<int> order;      // the order the list kernel walks them in
  int64_t ws_offset = 0;       // the list's descriptor table and counters inside the workspace
  wq_gemv_list_t* list = nullptr;
  bool failed = false;         // the list could not be built (aliasing operands): run one by one
  std::string why;             // ... and what wq_q4g32_gemv_list_create said
};

// What a q4f16_1_matmul* or autogptq_matmul instruction reads and writes, if it qualifies for a fused group.
struct DecodeLinear {
  int W, S, x, bias, residual, y;  // registers; bias / residual -1 when absent
  int64_t N, K;
  int64_t M;  // rows of x: 1 .. WQ_GEMV_LIST_MAX_M
  bool gptq = false;  // a prepared AutoGPTQ layer: S is SZ [N, G, 2], perm its row order (-1: none)
  int perm = -1;
  int64_t G = 0;
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
  bool fuse_decode = true;
  long long spin_limit_ticks = -1;  // of the fused runs' waits, in ticks of the 100 MHz wall clock; < 0: the lists' default
  std::vector<FusedGroup> groups;
  bool lists_stale = true;  // a register moved: the lists must be rebuilt before the next run
};

static void drop_lists(wq_program* p) {
  for (FusedGroup& g : p->groups) {
    if (g.list) wq_q4g32_gemv_list_destroy(g.list);
    g.list = nullptr;
    g.failed = false;
    g.why.clear();
  }
  p->lists_stale = true;
}

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
  drop_lists(p);
  delete p;
}

extern "C" int wq_program_set_option(wq_program_t* p, const char* name, int value) {
  WQ_REQUIRE(p && name, "wq_program_set_option: null argument");
  if (std::string(name) == "fuse_decode") {
    p->fuse_decode = value != 0;
    p->planned = false;  // the memory plan depends on it
    drop_graph(p);
    drop_lists(p);
    p->groups.clear();
    return WQ_OK;
  }
  if (std::string(name) == "spin_limit_us") {
    WQ_REQUIRE(value >= 0, "wq_program_set_option: spin_limit_us must not be negative");
    p->spin_limit_ticks = (long long)value * 100;
    for (FusedGroup& g : p->groups)
      if (g.list) (void)wq_q4g32_gemv_list_set_spin_limit(g.list, p->spin_limit_ticks);
    drop_graph(p);  // a captured launch carries the old limit as a kernel argument
    return WQ_OK;
  }
  return wq::fail(WQ_EINVAL, "wq_program_set_option: unknown option '%s'", name);
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
  drop_lists(p);  // and so do the descriptor tables of fused groups: rebuilt before the next run
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

// ---- fused groups of decode linears ----------------------------------------------------------
static bool as_decode_linear(const wq_program* p, const Instr& in, DecodeLinear* out) {
  static const char* const names[3][2] = {{"relax_amd.q4f16_1_matmul", "relax_amd_q4f16_1_matmul"},
                                          {"relax_amd.q4f16_1_matmul_bias", "relax_amd_q4f16_1_matmul_bias"},
                                          {"relax_amd.q4f16_1_matmul_bias_residual", "relax_amd_q4f16_1_matmul_bias_residual"}};
  int kind = -1;
  for (int k = 0; k < 3; ++k)
    if (in.name == names[k][0] || in.name == names[k][1]) kind = k;
  for (size_t i = 0; i < in.regs.size(); ++i)
    if (in.regs[i] < 0 && !(in.codes[i] == kTVMNullptr)) return false;
  auto numel = [&](int r) {
    int64_t n = 1;
    for (int64_t e : p->regs[r].shape) n *= e;
    return n;
  };
  auto is = [&](int r, int code, int bits) {
    const DLTensor& t = p->regs[r].dl;
    return t.dtype.code == code && t.dtype.bits == bits && t.device.device_type == kDLROCM;
  };
  if (in.name == "relax_amd.autogptq_matmul" || in.name == "relax_amd_autogptq_matmul") {
    // (W_nk, SZ, perm | null, x, residual | null, out [, workspace]); one row of x, group size 32 << t
    if (in.regs.size() != 6 && in.regs.size() != 7) return false;
    DecodeLinear d{in.regs[0], in.regs[1], in.regs[3], -1, in.regs[4], in.regs[5], 0, 0, 1};
    d.gptq = true;
    d.perm = in.regs[2];
    if (d.W < 0 || d.S < 0 || d.x < 0 || d.y < 0) return false;
    const Reg &W = p->regs[d.W], &SZ = p->regs[d.S];
    if (!is(d.W, kDLUInt, 32) || !is(d.S, kDLFloat, 16) || !is(d.x, kDLFloat, 16) || !is(d.y, kDLFloat, 16)) return false;
    if (W.shape.size() != 2 || SZ.shape.size() != 3 || SZ.shape[2] != 2 || SZ.shape[0] != W.shape[0]) return false;
    d.N = W.shape[0];
    d.K = W.shape[1] * 8;
    d.G = SZ.shape[1];
    if (d.N <= 0 || d.K <= 0 || d.K > WQ_GEMV_LIST_MAX_K || d.G <= 0 || d.K % d.G != 0) return false;
    bool size_ok = false;
    for (int t = 0; t <= 6; ++t) size_ok = size_ok || d.K / d.G == (32ll << t);
    if (!size_ok) return false;
    if (numel(d.x) != d.K || numel(d.y) != d.N) return false;
    if (d.perm >= 0 && (!is(d.perm, kDLInt, 32) || numel(d.perm) != d.K)) return false;
    if (d.residual >= 0 && (!is(d.residual, kDLFloat, 16) || numel(d.residual) != d.N)) return false;
    *out = d;
    return true;
  }
  if (kind < 0 || (int)in.regs.size() != 4 + kind) return false;
  DecodeLinear d{in.regs[0], in.regs[1], in.regs[2], kind >= 1 ? in.regs[3] : -1, kind >= 2 ? in.regs[4] : -1,
                 in.regs[3 + kind], 0, 0, 0};
  if (d.W < 0 || d.S < 0 || d.x < 0 || d.y < 0 || (kind >= 1 && d.bias < 0) || (kind >= 2 && d.residual < 0)) return false;
  const Reg &W = p->regs[d.W], &S = p->regs[d.S];
  if (!is(d.W, kDLUInt, 32) || !is(d.S, kDLFloat, 16) || !is(d.x, kDLFloat, 16) || !is(d.y, kDLFloat, 16)) return false;
  if (W.shape.size() != 2 || S.shape.size() != 2) return false;
  d.N = W.shape[0];
  d.K = W.shape[1] * 8;
  if (d.N <= 0 || d.K <= 0 || d.K > WQ_GEMV_LIST_MAX_K || S.shape[0] != d.N || S.shape[1] * 32 != d.K) return false;
  // one row of x (the decode case) or a few (a small decode batch, which the list kernel takes for K % 256 == 0)
  if (p->regs[d.x].shape.empty() || p->regs[d.x].shape.back() != d.K) return false;
  d.M = numel(d.x) / d.K;
  if (d.M < 1 || d.M > WQ_GEMV_LIST_MAX_M || (d.M > 1 && d.K % 256 != 0)) return false;
  if (p->regs[d.y].shape.empty() || p->regs[d.y].shape.back() != d.N || numel(d.y) != d.M * d.N) return false;
  if (d.bias >= 0 && (!is(d.bias, kDLFloat, 16) || numel(d.bias) != d.N)) return false;
  if (d.residual >= 0 && (!is(d.residual, kDLFloat, 16) || numel(d.residual) != d.M * d.N)) return false;
  *out = d;
  return true;
}

// Order of the linears of one group.  The list kernel overlaps a linear with its successors
// except where one reads what another wrote: that costs a device-side wait of several
// microseconds unless enough other work lies between the two.  So independent linears are moved
// between a producer and its consumer.  Of the first kWindow linears not yet placed (program
// order), those whose predecessors are all placed compete.  A consumer (its x comes from the
// group) may go once its producer lies at least kNear places back, and consumers and the other
// linears take turns as far as possible: the activations of a consumer are slow to fetch (a wait,
// then loads that bypass the caches), so a run of consumers would queue up behind each other.
static std::vector<int> schedule_group(const std::vector<DecodeLinear>& lin) {
  // measured on the 32-layer Llama-2-7B stack: (4, 8) 0.70 ms, (6, 12) 0.66 ms, (12, 24) 0.65 ms per step
  constexpr int kWindow = 12, kNear = 6;
  const int n = (int)lin.size();
  std::vector<int> order, placed_at(n, -1);
  std::vector<char> done(n, 0);
  auto reads = [&](const DecodeLinear& d, int reg) {
    return reg >= 0 && (d.W == reg || d.S == reg || d.x == reg || d.bias == reg || d.residual == reg);
  };
  bool last_was_consumer = true;  // start with the others
  while ((int)order.size() < n) {
    int first_free_consumer = -1, first_other = -1, closest_consumer = -1, closest_dist = -1, seen = 0;
    for (int i = 0; i < n && seen < kWindow; ++i) {
      if (done[i]) continue;
      ++seen;
      // every earlier linear that i depends on (it wrote what i reads or writes, or read what i writes)
      bool ready = true;
      int nearest = -1;  // position of the most recent producer
      for (int j = 0; j < i && ready; ++j) {
        const bool raw = reads(lin[i], lin[j].y);
        const bool waw = lin[i].y == lin[j].y;
        const bool war = reads(lin[j], lin[i].y);
        if (!(raw || waw || war)) continue;
        if (!done[j]) ready = false;
        else if (raw) nearest = std::max(nearest, placed_at[j]);
      }
      if (!ready) continue;
      if (nearest < 0) {
        if (first_other < 0) first_other = i;
      } else {
        const int dist = (int)order.size() - nearest;
        if (dist >= kNear && first_free_consumer < 0) first_free_consumer = i;
        if (dist > closest_dist) {
          closest_dist = dist;
          closest_consumer = i;
        }
      }
    }
    int best;
    if (first_free_consumer >= 0 && (!last_was_consumer || first_other < 0)) best = first_free_consumer;
    else if (first_other >= 0) best = first_other;
    else if (first_free_consumer >= 0) best = first_free_consumer;
    else best = closest_consumer;  // nothing else can go: the consumer whose producer lies furthest back
    last_was_consumer = best != first_other;
    done[best] = 1;  // the first unplaced linear is always ready, so one of the candidates exists
    placed_at[best] = (int)order.size();
    order.push_back(best);
  }
  return order;
}

// Shortest run worth one launch of the list kernel, by rows of x.  With several rows every workgroup of a
// linear's group loads all of that linear's activations, which a long list spreads over many small groups and a
// short one cannot (its linears share the 8 XCDs in proportion to their cost instead).  Llama-2-7B linears,
// us per decoder layer (4 linears), list against call by call:
//   M = 8:  one layer 41.5 / 44.4, two 40.2 / 44.3, four 37.0 / 44.5
//   M = 16: one layer 62.4 / 52.0, two 61.8 / 51.8, four 39.2 / 51.9
//   M = 32: one layer 111 / 70.6, two 73.8 / 70.7, four 44.2 / 70.7
// At M <= 4 the list wins from the first layer on (30 against 42 us).
static size_t min_fused_run(int64_t M) { return M <= 4 ? 2 : M <= 8 ? 4 : M <= 16 ? 16 : 12; }

static void find_groups(wq_program* p) {
  drop_lists(p);
  p->groups.clear();
  if (!p->fuse_decode) return;
  const int n = (int)p->instrs.size();
  for (int i = 0; i < n;) {
    std::vector<DecodeLinear> lin;
    DecodeLinear d;
    int j = i;
    while (j < n && (int)lin.size() < WQ_GEMV_LIST_MAX && as_decode_linear(p, p->instrs[j], &d) &&
           (lin.empty() || (d.M == lin[0].M && d.gptq == lin[0].gptq))) {  // one list, one batch size, one weight format
      // The list kernel orders a linear behind ONE earlier linear, through its x.  A bias or a residual that an
      // earlier linear of the run writes (the residual stream: down_proj adds what o_proj produced) is refused
      // by wq_q4g32_gemv_list_create: the run ends in front of such an instruction, which starts the next one.
      bool from_run = false;
      for (const DecodeLinear& e : lin)
        if ((d.bias >= 0 && d.bias == e.y) || (d.residual >= 0 && d.residual == e.y)) from_run = true;
      if (from_run) break;
      lin.push_back(d);
      ++j;
    }
    if (!lin.empty() && lin.size() >= min_fused_run(lin[0].M)) {
      FusedGroup g;
      g.first = i;
      g.last = j - 1;
      for (int k : schedule_group(lin)) g.order.push_back(i + k);
      p->groups.push_back(std::move(g));
    }
    i = std::max(j, i + 1);
  }
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
  // A fused group runs its linears concurrently and in an order of its own: every tensor it
  // touches is live over the whole group, so that none of them shares storage with another.
  find_groups(p);
  std::vector<int> lo(p->regs.size()), hi(p->regs.size());
  for (size_t i = 0; i < p->regs.size(); ++i) {
    lo[i] = p->regs[i].first;
    hi[i] = p->regs[i].last;
  }
  for (const FusedGroup& g : p->groups)
    for (int k = g.first; k <= g.last; ++k)
      for (int r : p->instrs[k].regs)
        if (r >= 0) {
          lo[r] = std::min(lo[r], g.first);
          hi[r] = std::max(hi[r], g.last);
        }
  for (int i = 0; i < (int)p->regs.size(); ++i)
    if (p->regs[i].planned && p->regs[i].first >= 0) order.push_back(i);
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return lo[a] < lo[b]; });
  int64_t top = 0;
  for (int ri : order) {
    Reg& r = p->regs[ri];
    const int r_first = lo[ri], r_last = hi[ri];
    const int64_t need = (r.bytes + kAlign - 1) / kAlign * kAlign;
    int best = -1;
    for (int b = 0; b < (int)blocks.size(); ++b)
      if (blocks[b].free_after < r_first && blocks[b].size >= need &&
          (best < 0 || blocks[b].size < blocks[best].size))
        best = b;
    if (best >= 0) {
      r.offset = blocks[best].offset;
      blocks[best].free_after = r_last;
    } else {
      r.offset = top;
      blocks.push_back({top, need, r_last});
      top += need;
    }
  }
  // descriptor tables and counters of the fused groups
  for (FusedGroup& g : p->groups) {
    g.ws_offset = top;
    int64_t need = (int64_t)wq_q4g32_gemv_list_workspace_bytes(g.last - g.first + 1);
    // AutoGPTQ layers with a row order: room for their gathered activations (sizes only: the addresses come later)
    static const int32_t kHasRowOrder = 0;  // (only whether a layer has a row order counts for the size)
    std::vector<wq_gptq_gemv_desc> shapes;
    for (int k = g.first; k <= g.last; ++k) {
      DecodeLinear d;
      if (as_decode_linear(p, p->instrs[k], &d) && d.gptq)
        shapes.push_back({nullptr, nullptr, d.perm >= 0 ? &kHasRowOrder : nullptr, nullptr, nullptr,
                          nullptr, nullptr, d.N, d.K, d.G});
    }
    if (!shapes.empty()) need = (int64_t)wq_gptq_gemv_list_workspace_bytes(shapes.data(), (int)shapes.size());
    g.ws_bytes = need;
    top += (need + kAlign - 1) / kAlign * kAlign;
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
  drop_lists(p);
  return WQ_OK;
}

static int check_ready(wq_program* p, const char* who) {
  WQ_REQUIRE(p, "%s: null program", who);
  // the descriptor tables and counters of the fused runs live in the workspace, also when every tensor is external
  if (!p->groups.empty() && !p->workspace)
    return wq::fail(WQ_EINVAL, "%s: the program has fused runs: plan it and set the workspace (%lld bytes)", who,
                    (long long)p->workspace_bytes);
  for (const Reg& r : p->regs)
    if (r.first >= 0 && r.bytes > 0 && !r.dl.data)
      return wq::fail(WQ_EINVAL, "%s: a tensor has no storage (%s)", who,
                      r.planned ? "plan the program and set the workspace" : "external tensor bound to null");
  return WQ_OK;
}

// Builds the list of every fused group from the registers' current addresses (load-time work:
// uploads the descriptor tables and synchronises the stream).
static int build_lists(wq_program* p, hipStream_t stream) {
  for (FusedGroup& g : p->groups) {
    if (g.list || g.failed) continue;
    std::vector<wq_q4g32_gemv_desc> descs;
    std::vector<wq_gptq_gemv_desc> gptq_descs;
    int64_t rows = 1;
    for (int k : g.order) {
      DecodeLinear d;
      if (!as_decode_linear(p, p->instrs[k], &d)) return wq::fail(WQ_EINVAL, "instruction %d no longer qualifies for its fused group", k);
      auto ptr = [&](int r) { return r < 0 ? nullptr : static_cast<char*>(p->regs[r].dl.data) + p->regs[r].dl.byte_offset; };
      if (d.gptq)
        gptq_descs.push_back({(const uint32_t*)ptr(d.W), (const uint16_t*)ptr(d.S), (const int32_t*)ptr(d.perm),
                              (const uint16_t*)ptr(d.x), nullptr, (const uint16_t*)ptr(d.residual), (uint16_t*)ptr(d.y),
                              d.N, d.K, d.G});
      else
        descs.push_back({(const uint32_t*)ptr(d.W), (const uint16_t*)ptr(d.S), (const uint16_t*)ptr(d.x),
                         (const uint16_t*)ptr(d.bias), (const uint16_t*)ptr(d.residual), (uint16_t*)ptr(d.y), d.N, d.K});
      rows = d.M;
    }
    char* ws = static_cast<char*>(p->workspace) + g.ws_offset;
    const int count = (int)(descs.size() + gptq_descs.size());
    g.list = !gptq_descs.empty()
                 ? wq_gptq_gemv_list_create(gptq_descs.data(), count, ws, (size_t)g.ws_bytes, stream)
                 : wq_q4g32_gemv_list_create_batched(descs.data(), count, (int)rows, ws,
                                                     wq_q4g32_gemv_list_workspace_bytes(count), stream);
    // operands that alias in a way the list kernel cannot order (or pointers it cannot take): the
    // group runs instruction by instruction, which is always valid
    if (!g.list) {
      g.failed = true;
      g.why = wq_last_error();
    } else if (p->spin_limit_ticks >= 0) (void)wq_q4g32_gemv_list_set_spin_limit(g.list, p->spin_limit_ticks);
  }
  p->lists_stale = false;
  return WQ_OK;
}

static int run_instruction(wq_program* p, size_t i) {
  Instr& in = p->instrs[i];
  TVMValue rv;
  rv.v_handle = nullptr;
  int rcode = kTVMNullptr;
  if (in.fn(in.vals.data(), in.codes.data(), (int)in.vals.size(), &rv, &rcode, nullptr) != 0) {
    // keep the callee's message, say where it happened
    std::string msg = wq_last_error();
    return wq::fail(WQ_EINVAL, "instruction %zu (%s): %s", i, in.name.c_str(), msg.c_str());
  }
  return WQ_OK;
}

static int run_all(wq_program* p, hipStream_t stream) {
  wq::set_stream_override(true, stream);
  int rc = WQ_OK;
  size_t gi = 0;
  for (size_t i = 0; i < p->instrs.size() && rc == WQ_OK;) {
    while (gi < p->groups.size() && (size_t)p->groups[gi].last < i) ++gi;
    if (gi < p->groups.size() && (size_t)p->groups[gi].first == i && p->groups[gi].list) {
      FusedGroup& g = p->groups[gi];
      if (wq_q4g32_gemv_list_run(g.list, stream) != WQ_OK) {
        std::string msg = wq_last_error();
        rc = wq::fail(WQ_EDEVICE, "instructions %d..%d (fused decode linears): %s", g.first, g.last, msg.c_str());
      }
      i = (size_t)g.last + 1;
      continue;
    }
    rc = run_instruction(p, i);
    ++i;
  }
  wq::set_stream_override(false, nullptr);
  return rc;
}

extern "C" int wq_program_run(wq_program_t* p, wq_stream_t stream) {
  if (int rc = check_ready(p, "wq_program_run")) return rc;
  if (int rc = build_lists(p, (hipStream_t)stream)) return rc;
  return run_all(p, (hipStream_t)stream);
}

extern "C" int wq_program_capture(wq_program_t* p, wq_stream_t stream_) {
  if (int rc = check_ready(p, "wq_program_capture")) return rc;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(stream != nullptr, "wq_program_capture: the null stream cannot be captured");
  drop_graph(p);
  if (int rc = build_lists(p, stream)) return rc;
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

extern "C" int wq_program_num_fused_groups(const wq_program_t* p) {
  if (!p) return 0;
  int n = 0;
  for (const FusedGroup& g : p->groups) n += g.list != nullptr;
  return n;
}

extern "C" const char* wq_program_unfused_reason(const wq_program_t* p, int group) {
  if (!p || group < 0 || group >= (int)p->groups.size()) return "";
  return p->groups[group].why.c_str();
}

extern "C" int wq_program_fused_order(const wq_program_t* p, int group, int* order, int capacity) {
  WQ_REQUIRE(p && group >= 0 && group < (int)p->groups.size(), "wq_program_fused_order: no such group");
  const FusedGroup& g = p->groups[group];
  for (int i = 0; i < (int)g.order.size() && i < capacity; ++i) order[i] = g.order[i];
  return (int)g.order.size();
}

extern "C" int wq_program_poll(wq_program_t* p, int* host_words, int capacity, wq_stream_t stream) {
  WQ_REQUIRE(p && (host_words || capacity == 0) && capacity >= 0, "wq_program_poll: bad argument");
  int n = 0;
  for (FusedGroup& g : p->groups) {
    if (!g.list) continue;
    if (n < capacity)
      if (int rc = wq_q4g32_gemv_list_poll(g.list, host_words + n, stream)) return rc;
    ++n;
  }
  return n;
}

extern "C" int wq_program_status(wq_program_t* p, wq_stream_t stream) {
  WQ_REQUIRE(p, "wq_program_status: null program");
  for (FusedGroup& g : p->groups)
    if (g.list)
      if (int rc = wq_q4g32_gemv_list_status(g.list, stream)) return rc;
  WQ_HIP(hipStreamSynchronize((hipStream_t)stream));
  return WQ_OK;
}
