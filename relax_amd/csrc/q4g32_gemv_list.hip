// A list of format-A (q4f16_1) decode linears, M = 1 each, in ONE launch.
//
// Why.  One decode linear reads 9 .. 50 MB; as a kernel of its own it lasts 4 .. 11 us, of which
// about 2.7 us are launch gap, ramp-up and drain.  A decoder layer is a list of such linears, so the
// list is executed by one grid of persistent workgroups that walks it: the weight stream of the
// next linear is already in flight while the current one finishes, and a linear that reads what an
// earlier one wrote waits on a device-side counter instead of a kernel boundary.
//
// Workgroup = NC compute wavefronts + 2 x wavefronts + 1 y wavefront, one workgroup per CU.
//   * Work is dealt in ROW GROUPS (2^gs consecutive rows of one linear).  The row groups of a
//     workgroup, over all linears in list order, form one sequence; a compute wavefront takes the
//     next one through an LDS counter whenever it has issued the last chunk of its group, so the NC
//     wavefronts stay balanced whatever the row lengths, and a wavefront only ever looks at the
//     linears in which it works.  A row is streamed in chunks of 64 scale groups (2048 k, 1 KiB of
//     codes: one 16-byte load and one scale per lane).  The chunks of all rows of a wavefront form
//     one stream that runs through a ring of D register slots: the loads of chunk f + D are issued
//     when chunk f has been consumed, also across rows, groups and linears.  Arithmetic per chunk as
//     in the single-linear kernel (q4_gemv.h): 1 shift + 4 v_and_or + 4 v_dot2 per 8 weights, zero
//     point and scale applied once per group.  Row sums go to LDS, not to memory.
//   * What bounds the kernel is the number of instructions a SIMD can issue (its waves never wait for
//     memory), the SCALAR ones first: so a chunk costs two scalars of state, everything per row is a
//     handful of additions, and the arithmetic of a row group (where it is, which linear) is paid once
//     per group.
//   * The service wavefronts do everything irregular, each at its own pace, up to NB (2..8) linears
//     ahead of or behind the compute wavefronts; LDS words (ListFlags) hand the NB buffer slots over.
//     An x wavefront waits for a producer linear (bounded spin), loads the activations of a coming
//     linear, rearranges them to the pairing of the unpack, computes the zero-point constants and
//     writes both to LDS.  The y wavefront takes the finished row sums of a linear from LDS (once
//     the compute wavefronts have counted all of the workgroup's rows of it), applies bias / cast /
//     residual, stores y, and signals completion.  They run at raised priority: they are the
//     youngest wavefronts of their SIMDs and would otherwise be starved by the compute wavefronts.
//
// Dependencies.  Linear i may read the y of an earlier linear `dep` of the same list.  Each
// workgroup adds 1 to one of 8 counters of linear `dep` once its stores of y (device scope, written
// through) have completed; the x wavefront of a consumer spins until the 8 counters sum to the number
// of workgroups and then reads x with device-scope loads (no cache is written back or invalidated:
// a release / acquire fence pair at agent scope costs about 10 us per linear here), for at most `spin_limit` ticks of the 100 MHz wall clock: after that it raises the
// error word, stops waiting for anything and lets every wavefront run to the end (results are then
// undefined, the host reads the error word).  The grid is sized so that all workgroups are resident
// at once; the bounded wait is what keeps a launch that is not (another kernel holding CUs) from
// hanging.  The waits on LDS words inside a workgroup are not bounded: every party is a wavefront of
// the same resident workgroup, and an x wavefront that has given up on a producer still stages (then
// meaningless) activations, so each of those waits ends.
// The last workgroup to finish clears the counters for the next launch.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <vector>

#include "../../include/relax_amd_wq_testing.h"
#include "gemv_list_common.h"
#include "tuning.h"
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

// LDS bytes per chunk of x: 4 blocks of 64 x 16 bytes (word ch of the chunk's group g at ch * 1024 + g * 16),
// then the 64 zero-point constants, one float per 16 bytes (so that one address register serves all five reads)
constexpr int kChunkBytes = 4096 + 1024;

// ---- where a workgroup's row groups are: its groups of all linears, in list order, form one sequence of
// ---- positions 0, 1, 2, ...; a cursor maps a position to (linear, local group).  Forward only.
struct GroupCursor {
  int lin;          // current linear (nlin: past the end)
  int base;         // position of its first group
  int R;            // positions of it that belong to this workgroup
  int rb;           // (b - off) mod workgroups: row group = local group * workgroups + rb
  int N;            // rows of the linear
  int ts;           // log2 of the rows of a position (a position is a whole row group or a part of one)
  int xoff;         // LDS offset of the linear's activations
  int C;            // chunks per row
  int row_w, row_s; // bytes per row of W and S
  int szl;          // ZP: log2 of the 32-column groups that share one (scale, zero point) pair
  const char* W;
  const char* S;
};

template <bool ZP>
__device__ __forceinline__ void group_cursor_load(GroupCursor& cu, gemv_desc_ptr descs, int nlin, int b, int nwg, int gs) {
  if (cu.lin >= nlin) {
    cu.R = 0x7fffffff;  // every position from here on is "past the end"
    return;
  }
  // (W, S: words 0..3; N, q, g_dep, rem | off << 16: 12..15)
  typedef const uint32_t __attribute__((address_space(4)))* words_ptr;
  const words_ptr p = (words_ptr)(descs + cu.lin);
  constexpr int kWords = ZP ? 20 : 19;
  uint32_t w[kWords];
#pragma unroll
  for (int i = 0; i < kWords; ++i) w[i] = p[i];  // (16: groups of the batch kernel, ts; 17: x_off; 19: szl)
  const int G = (int)(w[14] & 0xffffu);
  int rb = b - (int)(w[15] >> 16);
  if (rb < 0) rb += nwg;
  cu.rb = rb;
  cu.N = (int)w[12];
  cu.ts = (int)(w[16] >> 24);
  cu.xoff = (int)w[17];
  cu.R = ((int)w[13] + (rb < (int)(w[15] & 0xffffu) ? 1 : 0)) << (gs - cu.ts);
  cu.C = (G + 63) >> 6;
  cu.row_w = G << 4;
  if constexpr (ZP) {
    cu.szl = (int)(w[19] & 0xffu);
    cu.row_s = (G >> cu.szl) << 2;  // a pair of fp16 per group
  } else {
    cu.szl = 0;
    cu.row_s = G << 1;
  }
  cu.W = reinterpret_cast<const char*>(((uint64_t)w[1] << 32) | w[0]);
  cu.S = reinterpret_cast<const char*>(((uint64_t)w[3] << 32) | w[2]);
}

// LDS words that hand the buffers over inside a workgroup:
//   x_ready[slot]  = j + 1 once the activations of linear j are staged              (written by an x wavefront)
//   done[slot]     += 1 by a compute wavefront for every row sum it has written; the y wavefront clears it
//   flushed        = j + 1 once the row sums of linears 0..j have been stored to y   (written by the y wavefront);
//                    the buffers of linear j are free from then on (every row of it has been consumed)
// with slot = linear mod kYSlots.  The activations themselves live in a ring of LDS that the host deals out
// (GemvListDesc::x_off, free_after): a long row takes more of it than a short one.
constexpr int kYSlots = 16;  // linears in flight at most (flags and row-sum buffers: linear mod kYSlots)
struct ListFlags {
  int x_ready[kYSlots];
  int done[kYSlots];
  int flushed;
  int next_pos;  // the next position of the workgroup's sequence that nobody has taken
  int next_x;    // the next linear whose activations no x wavefront has taken
  int pad[13];
};

// ZP: the linears are prepared AutoGPTQ layers.  S holds a (scale, zero point + 1) pair of fp16 per column and
// group of 32 << szl columns; a lane loads the 4 bytes of its group's pair instead of a scale, and the constant
// that starts a group's sum becomes -(1024 A + 64 B) - zp (A + B) from the two sums the x wavefronts leave in LDS
// (A, B: the activations under the codes that are unpacked as 1024 + q and as 1024 + 16 q).
template <int NC, int XW, int D, bool ZP>
__global__ __launch_bounds__(64 * (NC + XW + 1)) void q4g32_gemv_list_kernel(const GemvListDesc* __restrict__ descs_,
                                                                        int nlin, int* __restrict__ sync,
                                                                        long long spin_limit, int ybuf0,
                                                                        int ybuf_floats, int gs, int use_sync) {
  extern __shared__ uint4_t smem[];
  const gemv_desc_ptr descs = (gemv_desc_ptr)descs_;
  char* lds = reinterpret_cast<char*>(smem);
  // flags, then the ring of activations, then (at byte ybuf0) kYSlots buffers of ybuf_floats row sums
  ListFlags* flags = reinterpret_cast<ListFlags*>(lds);
  float* ybuf = reinterpret_cast<float*>(lds + ybuf0);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nwg = gridDim.x;

  if (wave < NC) {
    // =========================== compute wavefront ===========================
    // The ring.  Its loads are written in assembly and waited for by hand.  Every turn of a slot issues
    // exactly two loads (16 bytes of codes and one scale per lane), also when the list has run out
    // (then from an empty buffer: nothing is fetched), and no other path of a compute wavefront
    // issues a vector memory operation: loads retire in order, so "at most 2 (D - 1) outstanding"
    // says that the oldest slot has landed.  (Left to the compiler, the wait of the first slot of the
    // unrolled loop comes out as "all but one".)  The loads are buffer loads over ONE ROW (base = the
    // row, size = its bytes): lanes beyond the end of a row whose K is not a multiple of 2048 receive
    // zeros for codes and scale, and the x wavefronts zero the activations of those groups, so a
    // partial last chunk needs no code of its own.
    const int b = blockIdx.x;
    const uint32_t lane16 = lane * 16;
    if (tid < (int)(sizeof(ListFlags) / sizeof(int))) reinterpret_cast<int*>(flags)[tid] = 0;
    lds_done_then_barrier();  // LDS starts undefined: the flags are cleared before anyone looks

    // slot state, two scalars.  meta: LDS offset of the chunk's activations (a multiple of 16) + the chunks of the row
    // that follow this one (0: the row ends here) + kFirst (the group's first chunk: are the activations there?) or
    // kDead (the list has run out).  yl: LDS offset of the row's sum | linear << 18.
    constexpr int kFirst = 1 << 24, kDead = 1 << 25;
    uint4_t rw[D];
    uint32_t rs[D];
    int slot_meta[D];
    int slot_yl[D];

    // the position counter: one lane adds.  The statement waits for its own answer: the compiler takes the
    // output of an asm statement as there when the statement ends (it may copy it at once).
    auto take_position = [&]() {
      int p = 0;
      if (lane == 0) {
        int one = 1;
        asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                     : "=v"(p)
                     : "v"((uint32_t)(uintptr_t)&flags->next_pos), "v"(one)
                     : "memory");
      }
      return __builtin_amdgcn_readfirstlane(p);
    };

    // issue side
    GroupCursor ic;
    ic.lin = 0;
    ic.base = 0;
    group_cursor_load<ZP>(ic, descs, nlin, b, nwg, gs);
    int i_rows = 0;       // rows of the group still to start
    int i_left = 0;       // chunks of the row still to issue
    int i_off = 0;        // byte offset of the next chunk in the row of codes
    int i_soff = 0;       // ... and in the row of scales
    int i_x = 0;          // LDS offset of the next chunk's activations
    int i_x0 = 0;         // ... of the row's first chunk
    int i_yl = 0;         // slot_yl of the row
    int i_first = 0;      // kFirst until the group's first chunk has been issued
    int i_sinc = 128;     // bytes of a row of S per chunk (64 scales; ZP: 64 >> szl pairs)
    uint32_t s_lane = lane16 >> 3;  // this lane's byte offset in a chunk's piece of S
    // buffer resources of the row: base address, size in bytes, flags (an empty one: every lane reads zero, no memory access)
    auto row_rsrc = [](const char* p, int bytes) {
      const uint64_t a = reinterpret_cast<uint64_t>(p);
      return uint4_t{(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, (uint32_t)bytes, (uint32_t)kBufferFlags};
    };
    uint4_t i_w = row_rsrc(nullptr, 0), i_s = row_rsrc(nullptr, 0);
    auto next_group = [&]() {
      int pos;
      uint32_t lp, row;
      while (true) {
        pos = take_position();
        while (ic.lin < nlin && pos >= ic.base + ic.R) {
          ic.base += ic.R;
          ++ic.lin;
          group_cursor_load<ZP>(ic, descs, nlin, b, nwg, gs);
        }
        if (ic.lin >= nlin) {  // the list has run out: the slots drain
          i_left = -1;
          i_w = row_rsrc(nullptr, 0);
          i_s = i_w;
          return;
        }
        // position -> (row group of this workgroup, part of it) -> first row; N < 2^30: 32 bits hold it
        lp = (uint32_t)(pos - ic.base) << ic.ts;  // first row of the position among the workgroup's rows of the linear
        row = (((lp >> gs) * (uint32_t)nwg + (uint32_t)ic.rb) << gs) + (lp & ((1u << gs) - 1));
        if ((int)row < ic.N) break;  // (else a part of the linear's last row group that lies beyond its last row)
      }
      i_rows = min(1 << ic.ts, ic.N - (int)row) - 1;
      const uint64_t woff = (uint64_t)row * (uint32_t)ic.row_w;  // a row of scales is an eighth of a row of codes
      i_w = row_rsrc(ic.W + woff, ic.row_w);
      if constexpr (ZP) {
        i_s = row_rsrc(ic.S + (uint64_t)row * (uint32_t)ic.row_s, ic.row_s);
        i_sinc = 256 >> ic.szl;
        s_lane = ((uint32_t)lane >> ic.szl) << 2;
      } else {
        i_s = row_rsrc(ic.S + (woff >> 3), ic.row_s);
      }
      i_left = ic.C;
      i_off = i_soff = 0;
      i_x = i_x0 = ic.xoff;
      i_yl = (ybuf0 + ((ic.lin & (kYSlots - 1)) * ybuf_floats + (int)lp) * 4) | (ic.lin << 18);
      i_first = kFirst;
    };
    auto next_row = [&]() {  // the row behind the one just issued
      --i_rows;
      uint64_t a = ((uint64_t)i_w.y << 32 | i_w.x) + (uint32_t)ic.row_w;
      i_w.x = (uint32_t)a;
      i_w.y = (uint32_t)(a >> 32);
      a = ((uint64_t)i_s.y << 32 | i_s.x) + (uint32_t)ic.row_s;
      i_s.x = (uint32_t)a;
      i_s.y = (uint32_t)(a >> 32);
      i_left = ic.C;
      i_off = i_soff = 0;
      i_x = i_x0;
      i_yl += 4;
    };

    auto issue = [&](uint4_t& w, uint32_t& s, int& meta, int& yl) {
      if (i_left == 0) {
        if (i_rows > 0) next_row();
        else next_group();
      }
      if constexpr (ZP)
        asm volatile(
            "buffer_load_dwordx4 %0, %2, %3, %4 offen nt\n\t"
            "buffer_load_dword %1, %5, %6, %7 offen nt"
            : "=&v"(w), "=&v"(s)
            : "v"(lane16), "s"(i_w), "s"(i_off), "v"(s_lane), "s"(i_s), "s"(i_soff));
      else
        asm volatile(
            "buffer_load_dwordx4 %0, %2, %3, %4 offen nt\n\t"
            "buffer_load_ushort %1, %5, %6, %7 offen nt"
            : "=&v"(w), "=&v"(s)
            : "v"(lane16), "s"(i_w), "s"(i_off), "v"(lane16 >> 3), "s"(i_s), "s"(i_soff));
      if (i_left < 0) {
        meta = kDead;
        return;
      }
      --i_left;
      meta = (i_x + i_left) | i_first;
      yl = i_yl;
      i_first = 0;
      i_off += 1024;
      i_soff += ZP ? i_sinc : 128;
      i_x += kChunkBytes;
    };

    // `magic` (0x6400 in both halves, OR-ed under every code) doubles as the token that orders the
    // reads of a ring slot behind the wait for it: the wait is an asm statement that "modifies"
    // magic, and every instruction that reads a ring register is an asm statement that takes magic as
    // an operand.  The ring registers themselves appear in no other statement, so nothing can read
    // or copy them between their load and their wait (the build checks this in the generated code).
    uint32_t magic = 0x64006400u;
    float acc = 0.0f;
    auto ring_shr8 = [&](uint32_t word) {
      uint32_t r;
      asm("v_lshrrev_b32 %0, 8, %1 ; %2" : "=v"(r) : "v"(word), "v"(magic));
      return r;
    };
    auto ring_shr16 = [&](uint32_t word) {
      uint32_t r;
      asm("v_lshrrev_b32 %0, 16, %1 ; %2" : "=v"(r) : "v"(word), "v"(magic));
      return r;
    };
    auto ring_scale = [&](uint32_t s16) {
      float r;
      asm("v_cvt_f32_f16 %0, %1 ; %2" : "=v"(r) : "v"(s16), "v"(magic));
      return r;
    };
    auto consume = [&](const uint4_t& w4, const uint32_t& s16, int meta, int yl) {
      if (meta & kFirst) {  // the first chunk of a group: the activations of its linear must be staged
        const int lin = yl >> 18;
        lds_spin_until(&flags->x_ready[lin & (kYSlots - 1)], lin + 1);
      }
      const char* xb = lds + (meta & 0xfffff0) + lane16;
      uint4_t xv[4];
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) xv[ch] = *reinterpret_cast<const uint4_t*>(xb + ch * 1024);
      float grp, zsum = 0.0f;
      if constexpr (ZP) {
        const float2 cz = *reinterpret_cast<const float2*>(xb + 4096);
        grp = cz.x;
        zsum = cz.y;
      } else {
        grp = *reinterpret_cast<const float*>(xb + 4096);
      }
      // every slot is always in flight (the drained ones with loads that fetch nothing): this one is the oldest
      asm volatile("s_waitcnt vmcnt(%1)" : "+v"(magic) : "n"(2 * (D - 1)));
      if constexpr (ZP) grp = fmaf((float)as_half((uint16_t)ring_shr16(s16)), zsum, grp);
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) {
        const uint32_t word = ch == 0 ? w4.x : ch == 1 ? w4.y : ch == 2 ? w4.z : w4.w;
        const uint32_t w8 = ring_shr8(word);
        const half2_t t0 = as_half2(and_or(word, 0x000F000Fu, magic));  // 1024 + (q0, q4)
        const half2_t t1 = as_half2(and_or(word, 0x00F000F0u, magic));  // 1024 + 16*(q1, q5)
        const half2_t t2 = as_half2(and_or(w8, 0x000F000Fu, magic));    // 1024 + (q2, q6)
        const half2_t t3 = as_half2(and_or(w8, 0x00F000F0u, magic));    // 1024 + 16*(q3, q7)
        grp = dot2(t0, as_half2(xv[ch].x), grp);
        grp = dot2(t1, as_half2(xv[ch].y), grp);
        grp = dot2(t2, as_half2(xv[ch].z), grp);
        grp = dot2(t3, as_half2(xv[ch].w), grp);
      }
      acc = fmaf(ring_scale(s16), grp, acc);
      if ((meta & 15) == 0) {  // the row ends here
        const float tot = wave_sum_to_lane63(acc);
        if (lane == 63) {
          *reinterpret_cast<float*>(lds + (yl & 0x3ffff)) = tot;
          // LDS is served in order: whoever sees the count sees the sum.  (Written out: the compiler's
          // own lowering of a one-lane atomic elects a lane and counts the others first.)
          const uint32_t done_at = (uint32_t)(uintptr_t)&flags->done[0] + (((uint32_t)yl >> 18) & (kYSlots - 1)) * 4;
          int one = 1;
          asm volatile("ds_add_u32 %0, %1" ::"v"(done_at), "v"(one) : "memory");
        }
        acc = 0.0f;
      }
    };

#pragma unroll
    for (int s = 0; s < D; ++s) issue(rw[s], rs[s], slot_meta[s], slot_yl[s]);
    bool live = true;
    while (live) {
#pragma unroll
      for (int s = 0; s < D; ++s) {
        if (slot_meta[s] & kDead) {  // the slots behind it are dead too
          live = false;
          break;
        }
        consume(rw[s], rs[s], slot_meta[s], slot_yl[s]);
        issue(rw[s], rs[s], slot_meta[s], slot_yl[s]);
      }
    }
    // the drained slots still have their (empty) loads in flight: they must have landed before the
    // ring's registers are used for something else (there is nothing else: the wavefront ends here)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }

  lds_done_then_barrier();  // the flags are cleared
  // The service wavefronts are the youngest of their SIMDs, and the arbiter serves the oldest first: at equal
  // priority the compute wavefronts, which never run out of instructions, starve them, and then wait for them.
  __builtin_amdgcn_s_setprio(3);
  bool aborted = false;

  if (wave < NC + XW) {
    // ====================== x wavefronts: activations -> LDS ======================
    // until every workgroup has signalled linear `dep`, or the spin limit passes
    auto wait_for = [&](int dep) {
      if (aborted) return;
      const long long t0 = wall_clock64();
      while (true) {
        // read-modify-write (+ 0): performed where the counter lives, never served from a stale cache line
        int v = 0;
        if (lane < kCountersPerLinear)
          v = __hip_atomic_fetch_add(sync + sync_counter_index(dep, lane), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v += __shfl_xor(v, 1, 64);
        v += __shfl_xor(v, 2, 64);
        v += __shfl_xor(v, 4, 64);
        if (__builtin_amdgcn_readfirstlane(v) >= nwg) break;
        if (wall_clock64() - t0 > spin_limit) {
          aborted = true;
          if (lane == 0)
            __hip_atomic_store(sync + sync_error_index(nlin), dep + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(4);
      }
      // whatever this XCD's L2 still holds of an earlier content of x (the addresses are reused
      // from launch to launch) must not serve the loads that follow
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    };

    // without zero points the constant 7 is folded here: 1024 + 7 and 64 + 7
    const half2_t k1031 = {(half_t)(ZP ? 1024.0f : 1031.0f), (half_t)(ZP ? 1024.0f : 1031.0f)};
    const half2_t k71 = {(half_t)(ZP ? 64.0f : 71.0f), (half_t)(ZP ? 64.0f : 71.0f)};
    const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
    const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
    while (true) {
      // whichever x wavefront is free takes the next linear, so that one slow wait does not hold up
      // the activations of the linears behind it
      int j = 0;
      if (lane == 0) j = __hip_atomic_fetch_add(&flags->next_x, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      j = __builtin_amdgcn_readfirstlane(j);
      if (j >= nlin) break;
      // everything this wavefront needs of the descriptor, fetched in one round trip before the wait below (a
      // second batch of scalar loads behind the wait costs every linear of the list half a microsecond: the
      // 4-linear step 21.1 -> 24.1 us)
      const int free_after = descs[j].free_after;
      const uint32_t g_dep = descs[j].g_dep;
      const half_t* const x_src = descs[j].x;
      const uint32_t x_off = descs[j].x_off;
      const int d_off = (int)descs[j].off, d_q = descs[j].q, d_rem = (int)descs[j].rem;
      const int32_t* perm = nullptr;
      if constexpr (ZP) perm = descs[j].perm;
      asm volatile("" ::"s"(free_after), "s"(g_dep), "s"(x_src), "s"(x_off), "s"(d_off), "s"(d_q), "s"(d_rem), "s"(perm));
      // its part of the ring (and its flags and row-sum buffer) is free once the linears that used them
      // before have been flushed: all their rows have been consumed by then
      lds_spin_until(&flags->flushed, free_after);
      // A linear of which this workgroup has no row is not staged.  (It must not be: the y wavefront declares such
      // a linear flushed at once, so a later linear may already be given the same part of the ring while this
      // wavefront still waits for a producer or writes: two consecutive rows of more than 40 KB, or a wait for a
      // producer that outlasts the staging of the linears behind it, then left a mixture of two linears'
      // activations there.)
      int rb = (int)blockIdx.x - d_off;
      if (rb < 0) rb += nwg;
      const bool has_rows = d_q + (rb < d_rem ? 1 : 0) > 0;
      const int dep = (int)((g_dep >> 16) & 0x7fffu) - 1;
      if (dep >= 0 && has_rows) wait_for(dep);
      const int K = (int)(g_dep & 0xffffu) << 5;
      // an x that other workgroups of this launch have written is read with device-scope loads
      // (sc1), which see what device-scope stores followed by the counter update have published,
      // without invalidating any cache; an x from outside the list with ordinary loads
      const __amdgpu_buffer_rsrc_t xr =
          __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x_src), 0, K * 2, kBufferFlags);
      char* xb = lds + x_off;
      // 16-byte words of 8 activations, up to the end of the last chunk (beyond K the buffer loads return zeros);
      // none without rows (the same path, so that the loop keeps its shape: a `continue` above made the compiler
      // spill this wavefront's 64 load registers)
      const int nwords = has_rows ? (((K >> 5) + 63) & ~63) << 2 : 0;
      // one 16-byte word of 8 activations (natural order) -> the pairing of the unpack and the group constants, to LDS
      auto stage = [&](int wi, const uint4_t& w8) {
        const uint32_t in[4] = {w8.x, w8.y, w8.z, w8.w};
        uint32_t o[4];
        pair_i_i4(in, o);  // o[i] = (x_i, x_{i+4})
        float c = dot2(as_half2(o[0]), k1031, 0.0f);
        c = dot2(as_half2(o[1]), k71, c);
        c = dot2(as_half2(o[2]), k1031, c);
        c = dot2(as_half2(o[3]), k71, c);
        c += dpp_shift<0xb1, 0xf>(c);  // the 4 words of a group sit in 4 adjacent lanes
        c += dpp_shift<0x4e, 0xf>(c);
        const int grp = wi >> 2, ch = wi & 3;
        char* cb = xb + (grp >> 6) * kChunkBytes;
        *reinterpret_cast<uint4_t*>(cb + ch * 1024 + (grp & 63) * 16) =
            uint4_t{o[0], as_u32(as_half2(o[1]) * sixteenth), o[2], as_u32(as_half2(o[3]) * sixteenth)};
        if constexpr (ZP) {  // the zero point multiplies the plain sum of the group's activations
          float t = dot2(as_half2(o[0]), ones, 0.0f);
          t = dot2(as_half2(o[1]), ones, t);
          t = dot2(as_half2(o[2]), ones, t);
          t = dot2(as_half2(o[3]), ones, t);
          t += dpp_shift<0xb1, 0xf>(t);
          t += dpp_shift<0x4e, 0xf>(t);
          if (ch == 0) *reinterpret_cast<float2*>(cb + 4096 + (grp & 63) * 16) = float2{-c, -t};
        } else {
          if (ch == 0) *reinterpret_cast<float*>(cb + 4096 + (grp & 63) * 16) = -c;
        }
      };
      if (ZP && perm != nullptr) {
        // a layer with a row order: position k' takes x[perm[k']]; positions beyond K (the rest of the last chunk)
        // are zeros.  Per round of 4 words a lane: the order (2 x 16 bytes per word), then 8 two-byte loads per
        // word: two round trips.  (8 words a round, or the next round's order requested ahead, need more
        // registers than the kernel's budget of 128 leaves: the compiler spilled 31 .. 158 of them.)
        const __amdgpu_buffer_rsrc_t pr =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t*>(perm), 0, K * 4, kBufferFlags);
        constexpr int UP = 4;
        uint4_t pa[UP], pb[UP];
        auto load_order = [&](int base) {
#pragma unroll
          for (int u = 0; u < UP; ++u) {
            const int wi = base + u * 64 + lane;
            pa[u] = __builtin_amdgcn_raw_buffer_load_b128(pr, wi * 32, 0, 0);  // (beyond K: zeros)
            pb[u] = __builtin_amdgcn_raw_buffer_load_b128(pr, wi * 32 + 16, 0, 0);
          }
        };
        for (int base = 0; base < nwords; base += 64 * UP) {
          load_order(base);
          half2_t h[UP][4];
#pragma unroll
          for (int u = 0; u < UP; ++u) {
            const uint32_t idx[8] = {pa[u].x, pa[u].y, pa[u].z, pa[u].w, pb[u].x, pb[u].y, pb[u].z, pb[u].w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const uint16_t bits = dep >= 0 ? (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(xr, (int)(idx[e] * 2u), 0, kDeviceScope)
                                             : (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(xr, (int)(idx[e] * 2u), 0, 0);
              if (e & 1) h[u][e >> 1].y = as_half(bits);
              else h[u][e >> 1].x = as_half(bits);
            }
          }
#pragma unroll
          for (int u = 0; u < UP; ++u) {
            const int wi = base + u * 64 + lane;
            if (wi < nwords) {  // a quad of lanes (one group) is in or out together
              const bool in_row = wi * 8 < K;
              const uint4_t w8 = {in_row ? as_u32(h[u][0]) : 0u, in_row ? as_u32(h[u][1]) : 0u,
                                  in_row ? as_u32(h[u][2]) : 0u, in_row ? as_u32(h[u][3]) : 0u};
              stage(wi, w8);
            }
          }
        }
      } else {
      constexpr int U = 16;       // loads in flight per lane: one round trip per 16 KiB of x
      for (int base = 0; base < nwords; base += 64 * U) {
        uint4_t v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int wi = base + u * 64 + lane;
          if (wi < nwords)
            v[u] = dep >= 0 ? __builtin_amdgcn_raw_buffer_load_b128(xr, wi * 16, 0, kDeviceScope)
                            : __builtin_amdgcn_raw_buffer_load_b128(xr, wi * 16, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int wi = base + u * 64 + lane;
          if (wi < nwords) stage(wi, v[u]);  // a quad of lanes (one group) is in or out together
        }
      }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (lane == 0) __hip_atomic_store(&flags->x_ready[j & (kYSlots - 1)], j + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    return;
  }

  // ================== y wavefront: row sums -> y, completion signals ==================
  for (int j = 0; j < nlin; ++j) {
    const half_t* bias = descs[j].bias;
    const half_t* residual = descs[j].residual;
    const int yslot = j & (kYSlots - 1);
    const float* yb = ybuf + yslot * ybuf_floats;
    int rb = (int)blockIdx.x - (int)descs[j].off;
    if (rb < 0) rb += nwg;
    const int N = descs[j].N;
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(descs[j].y, 0, N * 2, kBufferFlags);
    const int groups = descs[j].q + (rb < (int)descs[j].rem ? 1 : 0);
    const int R = groups << gs;  // places of this workgroup's rows in the buffer (those of a partial last group beyond N stay empty)
    // rows of this workgroup: all its groups are whole except the linear's last one
    const int last_row = (((groups - 1) * nwg + rb) << gs);
    const int rows = groups == 0 ? 0 : R - max(0, last_row + (1 << gs) - N);
    lds_spin_until(&flags->done[yslot], rows);
    for (int idx = lane; idx < R; idx += 64) {
      const int64_t n = ((((int64_t)(idx >> gs)) * nwg + rb) << gs) + (idx & ((1 << gs) - 1));
      if (n < N) {
        float v = yb[idx];
        if (bias) v += (float)bias[n];
        half_t h = (half_t)v;
        if (residual) h = h + residual[n];
        // device-scope store: written through, so that a counter update after it publishes it
        __builtin_amdgcn_raw_buffer_store_b16(as_u16(h), yr, (int)n * 2, 0, kDeviceScope);
      }
    }
    // the row sums are in registers or stored: the slots may be written again
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (lane == 0) {
      __hip_atomic_store(&flags->done[yslot], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_store(&flags->flushed, j + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    if (descs[j].g_dep & kSignal) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores of this workgroup have been written through
      if (lane == 0)
        __hip_atomic_fetch_add(sync + sync_counter_index(j, blockIdx.x & (kCountersPerLinear - 1)), 1,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (!use_sync) return;
  // the last workgroup to get here clears the counters for the next launch (every wait of this
  // workgroup lies behind it: its last row sums could only be stored after all its activations were staged)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this workgroup's own counter updates have arrived: none may land on a cleared counter
  int last = 0;
  if (lane == 0)
    last = __hip_atomic_fetch_add(sync + sync_finished_index(nlin), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
           nwg - 1;
  if (__builtin_amdgcn_readfirstlane(last)) {
    for (int i = lane; i < nlin * kCountersPerLinear; i += 64)
      __hip_atomic_store(sync + i * kCounterStride, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (lane == 0)
      __hip_atomic_store(sync + sync_finished_index(nlin), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Gathers in front of a list of AutoGPTQ layers: job blockIdx.y, 256 positions per workgroup.
__global__ __launch_bounds__(256) void gptq_list_gather_kernel(const GatherJob* __restrict__ jobs) {
  const GatherJob j = jobs[blockIdx.y];
  for (int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x; k < j.K; k += (int64_t)gridDim.x * 256) {
    const uint32_t src = (uint32_t)j.perm[k];
    j.xp[k] = src < (uint32_t)j.K ? j.x[src] : (half_t)0.0f;
  }
}

}  // namespace wq

namespace wq {
// ------------------------------------------------------------------ host side
struct GemvListConfig {
  int nc, depth, blocks_per_cu;
};

static bool ranges_overlap(const void* a, size_t na, const void* b, size_t nb) {
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
  return a && b && na && nb && a0 < b0 + nb && b0 < a0 + na;
}

}  // namespace wq

namespace wq {

constexpr int kListNC = 13;    // compute wavefronts per workgroup
constexpr int kListXW = 2;     // wavefronts that stage activations
constexpr int kListDepth = 4;  // ring slots (KiB of codes in flight) per compute wavefront: 52 KiB per CU
                               // (2, 3, 4 and 6 slots measure the same within 2 %)
}  // namespace wq

extern "C" size_t wq_q4g32_gemv_list_workspace_bytes(int n) {
  if (n <= 0) return 0;
  return wq::list_table_bytes(n) + (size_t)wq::sync_ints(n) * sizeof(int);
}

// room for the gathered activations of every layer with a row order (whether its x turns out to come from the list
// or not is only known from the addresses) and for the jobs of the gather kernel
extern "C" size_t wq_gptq_gemv_list_workspace_bytes(const wq_gptq_gemv_desc* d, int n) {
  if (!d || n <= 0) return 0;
  size_t extra = wq::kListAlign * (((size_t)n * sizeof(wq::GatherJob) + wq::kListAlign - 1) / wq::kListAlign);
  bool any = false;
  for (int i = 0; i < n; ++i)
    if (d[i].perm && d[i].K > 0) {
      any = true;
      extra += ((size_t)d[i].K * 2 + wq::kListAlign - 1) / wq::kListAlign * wq::kListAlign;
    }
  return wq_q4g32_gemv_list_workspace_bytes(n) + (any ? extra : 0);
}

extern "C" void wq_q4g32_gemv_list_destroy(wq_gemv_list_t* l) { delete l; }

extern "C" wq_gemv_list_t* wq_q4g32_gemv_list_create(const wq_q4g32_gemv_desc* d, int n, void* workspace,
                                                     size_t workspace_bytes, wq_stream_t stream) {
  return wq_q4g32_gemv_list_create_batched(d, n, 1, workspace, workspace_bytes, stream);
}

namespace wq {
// szl == nullptr: format A.  Else the linears are prepared AutoGPTQ layers: d[i].S is SZ and szl[i] the log2 of
// the 32-column groups per (scale, zero point) pair.
static wq_gemv_list_t* gemv_list_create(const char* who, const wq_q4g32_gemv_desc* d, const uint8_t* szl,
                                        const int32_t* const* perm, int n, int M, void* workspace, size_t workspace_bytes,
                                        hipStream_t stream);
}  // namespace wq

extern "C" wq_gemv_list_t* wq_q4g32_gemv_list_create_batched(const wq_q4g32_gemv_desc* d, int n, int M, void* workspace,
                                                             size_t workspace_bytes, wq_stream_t stream) {
  return wq::gemv_list_create("wq_q4g32_gemv_list_create", d, nullptr, nullptr, n, M, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" wq_gemv_list_t* wq_gptq_gemv_list_create(const wq_gptq_gemv_desc* d, int n, void* workspace,
                                                    size_t workspace_bytes, wq_stream_t stream) {
  using namespace wq;
#define bad(code, ...) ((void)fail(code, __VA_ARGS__), (wq_gemv_list_t*)nullptr)
  if (!d || n <= 0 || n > WQ_GEMV_LIST_MAX)
    return bad(WQ_EINVAL, "wq_gptq_gemv_list_create: need 1 .. %d linears, got %d", WQ_GEMV_LIST_MAX, n);
  std::vector<wq_q4g32_gemv_desc> e(n);
  std::vector<uint8_t> szl(n);
  std::vector<const int32_t*> perm(n);
  for (int i = 0; i < n; ++i) {
    const wq_gptq_gemv_desc& s = d[i];
    // a pair serves 32 << szl columns of a row; a chunk of 64 x 32 columns must hold whole pairs' worth of lanes
    int lg = -1;
    if (s.K > 0 && s.G > 0 && s.K % s.G == 0)
      for (int t = 0; t <= 6; ++t)
        if (s.K / s.G == (32ll << t)) lg = t;
    if (lg < 0)
      return bad(WQ_EUNSUPPORTED, "wq_gptq_gemv_list_create: linear %d: K=%lld G=%lld (the group size K / G must be 32, 64, ... or 2048)",
                 i, (long long)s.K, (long long)s.G);
    if (!s.SZ || (reinterpret_cast<uintptr_t>(s.SZ) & 3))
      return bad(WQ_EINVAL, "wq_gptq_gemv_list_create: linear %d: SZ must be 4-byte aligned", i);
    e[i] = wq_q4g32_gemv_desc{s.W_nk, s.SZ, s.x, s.bias, s.residual, s.y, s.N, s.K};
    szl[i] = (uint8_t)lg;
    if (s.perm && !aligned16(s.perm))
      return bad(WQ_EINVAL, "wq_gptq_gemv_list_create: linear %d: perm must be 16-byte aligned", i);
    perm[i] = s.perm;
  }
  return gemv_list_create("wq_gptq_gemv_list_create", e.data(), szl.data(), perm.data(), n, 1, workspace, workspace_bytes,
                          (hipStream_t)stream);
#undef bad
}

static wq_gemv_list_t* wq::gemv_list_create(const char* who, const wq_q4g32_gemv_desc* d, const uint8_t* szl,
                                            const int32_t* const* perm, int n, int M, void* workspace,
                                            size_t workspace_bytes, hipStream_t stream) {
#define bad(code, ...) ((void)fail(code, __VA_ARGS__), (wq_gemv_list_t*)nullptr)
  if (M < 1 || M > WQ_GEMV_LIST_MAX_M)
    return bad(WQ_EUNSUPPORTED, "%s: 1 .. %d rows of activations, got %d", who, WQ_GEMV_LIST_MAX_M, M);
  if (!d || n <= 0 || n > WQ_GEMV_LIST_MAX) return bad(WQ_EINVAL, "%s: need 1 .. %d linears, got %d", who, WQ_GEMV_LIST_MAX, n);
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & (kListAlign - 1)) ||
      workspace_bytes < wq_q4g32_gemv_list_workspace_bytes(n))
    return bad(WQ_EINVAL, "%s: workspace must be 256-byte aligned device memory of %zu bytes", who,
               wq_q4g32_gemv_list_workspace_bytes(n));
  std::vector<wq_q4g32_gemv_desc> e;
  std::vector<int> rows;
  for (int i = 0; i < n; ++i) {
    const wq_q4g32_gemv_desc& s = d[i];
    if (s.N <= 0 || s.K <= 0 || s.K % 32 != 0 || s.K > WQ_GEMV_LIST_MAX_K || s.N >= (1ll << 30))
      return bad(WQ_EINVAL, "%s: linear %d: N=%lld K=%lld (K must be a positive multiple of 32, at most %d)", who,
                 i, (long long)s.N, (long long)s.K, WQ_GEMV_LIST_MAX_K);
    if (!s.W || !s.S || !s.x || !s.y) return bad(WQ_EINVAL, "%s: linear %d: null pointer", who, i);
    if (!aligned16(s.W) || !aligned16(s.x))
      return bad(WQ_EINVAL, "%s: linear %d: W and x must be 16-byte aligned", who, i);
    // several rows: the scales travel in 16-byte pieces of 8, and rows of x and y are addressed with 32-bit offsets
    if (M > 1 && (s.K % 256 != 0 || !aligned16(s.S) || (int64_t)M * s.N >= (1ll << 30) || s.K / 32 > 0xffff))
      return bad(WQ_EUNSUPPORTED, "%s: linear %d: with %d rows of activations K=%lld must be a multiple of 256, S 16-byte aligned and M * N < 2^30", who, i, M, (long long)s.K);
    e.push_back(s);
    rows.push_back(M);
  }
  const int ne = (int)e.size();
  std::unique_ptr<wq_gemv_list> l(new wq_gemv_list());
  l->n = ne;
  l->M = M;
  l->zp = szl != nullptr;
  l->descs.resize(ne);
  int cmax = 1;
  for (int i = 0; i < ne; ++i) {
    const wq_q4g32_gemv_desc& s = e[i];
    GemvListDesc& g = l->descs[i];
    g.W = reinterpret_cast<const char*>(s.W);
    g.S = reinterpret_cast<const char*>(s.S);
    g.x = reinterpret_cast<const half_t*>(s.x);
    g.bias = reinterpret_cast<const half_t*>(s.bias);
    g.residual = reinterpret_cast<const half_t*>(s.residual);
    g.y = reinterpret_cast<half_t*>(s.y);
    g.N = (int32_t)s.N;
    g.q = 0;  // q, rem, off: once the grid is known
    g.g_dep = (uint32_t)(s.K / 32);
    g.rem = 0;
    g.off = 0;
    g.rows = (uint8_t)rows[i];
    g.szl = szl ? szl[i] : 0;
    g.perm = perm ? perm[i] : nullptr;
    cmax = std::max(cmax, (int)((s.K / 32 + 63) / 64));
  }
  // Who reads what an earlier linear of the list wrote.  Writing over something an earlier linear
  // still reads or wrote is refused: workgroups are not synchronised except through `dep`.
  for (int i = 0; i < ne; ++i) {
    const wq_q4g32_gemv_desc& a = e[i];
    const size_t ya = (size_t)a.N * 2 * rows[i], xa = (size_t)a.K * 2 * rows[i];
    for (int j = i - 1; j >= 0; --j) {
      const wq_q4g32_gemv_desc& b = e[j];
      const size_t yb = (size_t)b.N * 2 * rows[j], xb = (size_t)b.K * 2 * rows[j];
      if (ranges_overlap(a.x, xa, b.y, yb)) {
        // one producer per linear: the consumer waits for a single counter set
        if (((l->descs[i].g_dep >> 16) & 0x7fffu) != 0)
          return bad(WQ_EUNSUPPORTED, "%s: the activations of linear %d are written by more than one linear of the list (%d and %d)", who,
                     i, j, (int)((l->descs[i].g_dep >> 16) & 0x7fffu) - 1);
        l->descs[i].g_dep |= (uint32_t)(j + 1) << 16;
      }
      if (ranges_overlap(a.residual, ya, b.y, yb) || ranges_overlap(a.bias, (size_t)a.N * 2, b.y, yb))
        return bad(WQ_EUNSUPPORTED, "%s: linear %d takes its bias or residual from linear %d of the same list", who, i, j);
      if (ranges_overlap(a.y, ya, b.y, yb) || ranges_overlap(a.y, ya, b.x, xb) ||
          ranges_overlap(a.y, ya, b.residual, yb) || ranges_overlap(a.y, ya, b.bias, (size_t)b.N * 2))
        return bad(WQ_EUNSUPPORTED, "%s: the output of linear %d overlaps an operand of linear %d", who, i, j);
    }
    if (ranges_overlap(a.y, ya, a.x, xa))
      return bad(WQ_EINVAL, "%s: linear %d: y overlaps x", who, i);
    const int dep = (int)((l->descs[i].g_dep >> 16) & 0x7fffu) - 1;
    if (dep >= 0) {
      l->descs[dep].g_dep |= kSignal;
      ++l->deps;
      if (dep == i - 1) ++l->late;
    }
  }
  if (M > 1) {
    if (batch_list_plan(l.get()) != WQ_OK) return nullptr;
  } else {
  // launch shape: one workgroup of 16 wavefronts per CU.  Workgroup b owns the rows
  // n = local * workgroups + ((b - off) mod workgroups); `off` continues the round-robin where the
  // previous linear ended, so that the remainders of all linears spread over the workgroups.
  l->threads = 64 * (kListNC + kListXW + 1);
  l->blocks = std::min(cu_count(), 32768);
  int64_t turns = 1;
  int64_t off = 0;
  for (int i = 0; i < ne; ++i) {
    GemvListDesc& g = l->descs[i];
    const int64_t groups = (e[i].N + (1 << l->gs) - 1) >> l->gs;
    g.q = (int32_t)(groups / l->blocks);
    g.rem = (uint16_t)(groups % l->blocks);
    g.off = (uint16_t)off;
    off = (off + groups) % l->blocks;
    turns = std::max<int64_t>(turns, ((groups + l->blocks - 1) / l->blocks) << l->gs);
  }
  l->ybuf_floats = (int)((turns + 63) / 64 * 64);
  // LDS: flags, the ring of activations, kYSlots buffers of row sums.  A linear takes as much of the ring as its
  // row is long, from where its predecessor ends (from the start again if it does not fit before the end), and
  // may be staged once every earlier linear whose part overlaps its own has been flushed, and the linear that
  // used its flags and row-sum buffer before (kYSlots back).
  const size_t ysums = (size_t)kYSlots * l->ybuf_floats * sizeof(float);
  const size_t lds_budget = 150 * 1024;
  if (sizeof(ListFlags) + ysums + (size_t)cmax * kChunkBytes > lds_budget)
    return bad(WQ_EUNSUPPORTED, "%s: the activations and row sums do not fit the LDS", who);
  const int ring0 = (int)sizeof(ListFlags), ring1 = (int)(lds_budget - ysums);
  l->ybuf0 = ring1;
  l->lds = lds_budget;
  {
    int at = ring0;
    std::vector<int> lo(ne), hi(ne);
    for (int i = 0; i < ne; ++i) {
      const int size = (int)((e[i].K / 32 + 63) / 64) * kChunkBytes;
      if (at + size > ring1) at = ring0;
      lo[i] = at;
      hi[i] = at + size;
      at += size;
      int after = std::max(0, i - kYSlots + 1);
      for (int j = i - 1; j >= 0 && j + 1 > after; --j)
        if (lo[j] < hi[i] && lo[i] < hi[j]) after = j + 1;
      l->descs[i].x_off = (uint32_t)lo[i];
      l->descs[i].free_after = after;
    }
  }
  // rows a compute wavefront takes at a time: whole row groups where a workgroup has many rows of the linear
  // (what a position costs beyond its chunks is paid once), pairs where it has few, single rows at the end of the
  // list (the launch ends when the last wavefront does).  Measured on the four Llama-2-7B shapes: whole groups
  // for the 4096-row linears as well cost the 32-layer stack 4 %, single rows everywhere cost the 4-linear
  // step 4 %.
  {
    double tail = 0;  // weights behind the linear: about 2 us of the machine's stream are "the end of the list"
    for (int i = ne - 1; i >= 0; --i) {
      const int64_t per_wg = e[i].N / l->blocks;
      int ts = per_wg >= 32 ? l->gs : per_wg >= 8 ? std::min(1, l->gs) : 0;
      if (tail < 32e6) ts = 0;
      tail += (double)e[i].N * e[i].K;
      l->descs[i].ts = (uint8_t)ts;
    }
  }
  const void* kern = l->zp ? reinterpret_cast<const void*>(q4g32_gemv_list_kernel<kListNC, kListXW, kListDepth, true>)
                           : reinterpret_cast<const void*>(q4g32_gemv_list_kernel<kListNC, kListXW, kListDepth, false>);
  static DynamicLdsLimit limit[2];  // several lists share a kernel: its limit only ever grows
  if (l->lds > 48 * 1024 && limit[l->zp ? 1 : 0].ensure(kern, (int)l->lds) != hipSuccess)
    return bad(WQ_EDEVICE, "%s: hipFuncSetAttribute failed", who);
  int resident = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, kern, l->threads, l->lds) != hipSuccess || resident < 1)
    return bad(WQ_EDEVICE, "%s: the workgroup does not fit a CU (%zu bytes of LDS)", who, l->lds);
  }
  // Layers with a row order whose x comes from outside the list: if the workspace has room
  // (wq_gptq_gemv_list_workspace_bytes), a small kernel in front of the list gathers their activations and the list
  // reads the gathered copy like any other x; the others (and all of them in a workspace of the plain size) gather
  // while they stage, which costs the step about 3 us per layer.
  std::vector<GatherJob> jobs;
  if (perm) {
    char* const base = static_cast<char*>(workspace);
    size_t at = wq_q4g32_gemv_list_workspace_bytes(ne);
    const size_t jobs_bytes = ((size_t)ne * sizeof(GatherJob) + kListAlign - 1) / kListAlign * kListAlign;
    char* const job_table = base + at;
    at += jobs_bytes;
    int64_t kmax = 0;
    for (int i = 0; i < ne && at <= workspace_bytes; ++i) {
      GemvListDesc& g = l->descs[i];
      if (!g.perm || ((g.g_dep >> 16) & 0x7fffu) != 0) continue;
      const size_t need = ((size_t)e[i].K * 2 + kListAlign - 1) / kListAlign * kListAlign;
      if (at + need > workspace_bytes) break;
      jobs.push_back(GatherJob{g.x, g.perm, reinterpret_cast<half_t*>(base + at), e[i].K});
      g.x = reinterpret_cast<const half_t*>(base + at);
      g.perm = nullptr;
      at += need;
      kmax = std::max(kmax, e[i].K);
    }
    if (!jobs.empty()) {
      l->gather_table = job_table;
      l->gather_jobs = (int)jobs.size();
      l->gather_blocks = (int)std::min<int64_t>((kmax + 255) / 256, 64);
      if (hipMemcpyAsync(job_table, jobs.data(), jobs.size() * sizeof(GatherJob), hipMemcpyHostToDevice, stream) != hipSuccess)
        return bad(WQ_EDEVICE, "%s: could not upload the gather jobs", who);
    }
  }
  l->table = workspace;
  l->sync = reinterpret_cast<int*>(static_cast<char*>(workspace) + list_table_bytes(ne));
  if (hipMemcpyAsync(l->table, l->descs.data(), (size_t)ne * sizeof(GemvListDesc), hipMemcpyHostToDevice, stream) != hipSuccess ||
      hipMemsetAsync(l->sync, 0, (size_t)sync_ints(ne) * sizeof(int), stream) != hipSuccess ||
      hipStreamSynchronize(stream) != hipSuccess)
    return bad(WQ_EDEVICE, "%s: could not upload the descriptor table", who);
  return l.release();
#undef bad
}

extern "C" int wq_q4g32_gemv_list_run(wq_gemv_list_t* l, wq_stream_t stream) {
  using namespace wq;
  WQ_REQUIRE(l && l->table, "wq_q4g32_gemv_list_run: null list");
  if (l->M > 1) return batch_list_launch(l, (hipStream_t)stream);
  if (l->zp) {
    if (l->gather_jobs > 0)
      WQ_LAUNCH("wq_q4g32_gemv_list_run", gptq_list_gather_kernel, dim3((unsigned)l->gather_blocks, (unsigned)l->gather_jobs),
                dim3(256), 0, (hipStream_t)stream, (const GatherJob*)l->gather_table);
    WQ_LAUNCH("wq_q4g32_gemv_list_run", (q4g32_gemv_list_kernel<kListNC, kListXW, kListDepth, true>), dim3((unsigned)l->blocks),
              dim3((unsigned)l->threads), l->lds, (hipStream_t)stream, (const GemvListDesc*)l->table, l->n, l->sync,
              l->spin_limit, l->ybuf0, l->ybuf_floats, l->gs, l->deps > 0 ? 1 : 0);
    return WQ_OK;
  }
  WQ_LAUNCH("wq_q4g32_gemv_list_run", (q4g32_gemv_list_kernel<kListNC, kListXW, kListDepth, false>), dim3((unsigned)l->blocks),
            dim3((unsigned)l->threads), l->lds, (hipStream_t)stream, (const GemvListDesc*)l->table, l->n, l->sync,
            l->spin_limit, l->ybuf0, l->ybuf_floats, l->gs, l->deps > 0 ? 1 : 0);
  return WQ_OK;
}

extern "C" int wq_q4g32_gemv_list_status(wq_gemv_list_t* l, wq_stream_t stream) {
  using namespace wq;
  WQ_REQUIRE(l && l->table, "wq_q4g32_gemv_list_status: null list");
  int err = 0;
  int* p = l->sync + sync_error_index(l->n);
  WQ_HIP(hipMemcpyAsync(&err, p, sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream));
  WQ_HIP(hipStreamSynchronize((hipStream_t)stream));
  if (err == 0) return WQ_OK;
  // the counters may be mid-count after an abandoned wait: start clean
  WQ_HIP(hipMemsetAsync(l->sync, 0, (size_t)sync_ints(l->n) * sizeof(int), (hipStream_t)stream));
  WQ_HIP(hipStreamSynchronize((hipStream_t)stream));
  if (err > kBatchInternalWait)
    return fail(WQ_EDEVICE, "wq_q4g32_gemv_list: a hand-over inside a workgroup (kind %d) timed out; results of that launch are undefined",
                err - kBatchInternalWait);
  return fail(WQ_EDEVICE,
              "wq_q4g32_gemv_list: a wait for linear %d timed out (the grid was not resident at once?); "
              "results of that launch are undefined",
              err - 1);
}

extern "C" int wq_q4g32_gemv_list_poll(wq_gemv_list_t* l, int* host_word, wq_stream_t stream) {
  using namespace wq;
  WQ_REQUIRE(l && l->table && host_word, "wq_q4g32_gemv_list_poll: null argument");
  // no synchronisation and no allocation: the word arrives when the stream gets here
  WQ_HIP(hipMemcpyAsync(host_word, l->sync + sync_error_index(l->n), sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream));
  return WQ_OK;
}

extern "C" int wq_q4g32_gemv_list_info(const wq_gemv_list_t* l, int* dependencies, int* adjacent) {
  using namespace wq;
  WQ_REQUIRE(l, "wq_q4g32_gemv_list_info: null list");
  if (dependencies) *dependencies = l->deps;
  if (adjacent) *adjacent = l->late;
  return WQ_OK;
}

extern "C" int wq_debug_gemv_list_groups(const wq_gemv_list_t* l) { return l && l->M > 1 ? l->batch_groups : -1; }

extern "C" int wq_q4g32_gemv_list_set_spin_limit(wq_gemv_list_t* l, long long ticks) {
  using namespace wq;
  WQ_REQUIRE(l && ticks >= 0, "wq_q4g32_gemv_list_set_spin_limit: bad argument");
  l->spin_limit = ticks;
  return WQ_OK;
}

