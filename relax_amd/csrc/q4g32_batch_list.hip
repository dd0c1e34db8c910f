// A list of format-A (q4f16_1) linears with 2 .. 32 activation rows each, in ONE launch.
//
// The counterpart of q4g32_gemv_list.hip for a small batch: the same persistent grid (one workgroup
// per CU walks the list, device-side counters order dependent linears), but the products are done by
// the matrix cores so that all M rows share one pass over the weights, and the weights go from
// memory straight into the registers that feed them.
//
// Two kernels: up to 16 rows of activations the one described here (q4g32_batch_list_kernel), beyond that
// q4g32_batch_rows_kernel further down, which shares the unpack, the lane exchange and the staging of activations.
//
// Work.  The unit is a TILE of rows of W times a PANEL of K: 16 rows x 4096 k for M <= 8, 32 rows x 2048 k for
// M <= 16 (an item is 32 KiB of codes: what a workgroup spends per item on hand-overs does not depend on its
// size).  A linear is run by one GROUP of
// workgroups (see batch_assign_groups), its tiles dealt to them round-robin, with a rotation that continues
// from linear to linear.  Inside a workgroup the 8 compute wavefronts split a tile: 16 rows x an eighth of the
// panel each, or, with tiles of 32 rows, wavefronts 0 .. 3 a quarter of the panel of rows 0 .. 15 each and
// wavefronts 4 .. 7 of rows 16 .. 31.  A wavefront's share is U = 4 chunks; a chunk is
// one 16-byte load per lane: lane (i, kq) takes scale group 4u + kq of row i, the 32 codes that the four
// v_mfma_f32_16x16x32_f16 of the chunk consume as A operands (one dword, 8 codes, each).  (The template
// parameter R, sets of 16 activation rows per unpacked A operand, is 1 in every instantiation.)
// Unpacking is exact: OR the code into 0x6400 (1024 + q, or 1024 + 16 q), subtract 1031 (1136),
// multiply by the scale, all in packed fp16: 13 VALU instructions per 8 weights and lane, whatever M.
// The B operands (the activations of the wavefront's K slice, in the k order of the unpack, the
// 16 q positions pre-divided by 16) live in registers for the whole panel.
//
// The other four wavefronts keep everything irregular away from that loop, through LDS:
//   * 2 x wavefronts wait for a producer linear (bounded spin), load a panel of activations,
//     rearrange it and leave it in one of 1 or 2 LDS buffers (under load a round trip to L2 takes several
//     microseconds); the compute wavefronts copy their slice into registers when they reach the panel,
//     which frees the buffer at once, so even one buffer keeps the next panel ready in time.  The two take
//     whole panels by turns: while one waits for a producer the other already fetches the panel after it
//     (sharing every panel between them instead was slower at every M).
//   * the scale wavefront streams the tile's scales (per row up to 256 contiguous bytes: fetched per
//     lane they cost more than the codes) into a ring of LDS slots, a few tiles ahead.
//   * the y wavefront adds the 8 partial sums of a tile (4 per 16 rows of a 32-row tile) in a fixed order, keeps the
//     sum in LDS while further panels of the same rows follow, and at the last panel applies bias / cast / residual,
//     stores y with device-scope stores and signals the linear's completion counter.
// A linear of several panels whose kept sums would not fit the LDS is walked in CHUNKS of its tiles (all
// panels of a chunk, then the next chunk; template parameter CH): the activations are then loaded once
// per chunk, which the host weighs against fewer, larger groups when it plans the list.
// Codes in flight per CU: 8 wavefronts x (NT - 1) tiles x U KiB.
#include <algorithm>
#include <cmath>
#include <vector>

#include "gemv_list_common.h"
#include "tuning.h"

namespace wq {

constexpr int kBW = 8;     // compute wavefronts: K slices of a panel
constexpr int kBXW = 2;    // wavefronts that stage activations
constexpr int kBRing = 4;  // LDS slots of scales and of partial sums: how far the compute wavefronts may spread
constexpr int kBNT = 3;    // tile buffers per compute wavefront (NT - 1 tiles of loads in flight)
constexpr int kBThreads = 64 * (kBW + kBXW + 2);

// LDS words that hand the buffers over inside a workgroup (items = (linear, panel, tile) in the
// order the workgroup walks them; panels counted over all linears)
constexpr int kBMaxXBuf = 4;  // room in the flags; the host uses 1 or 2
struct BatchFlags {
  int x_ready[kBMaxXBuf];  // [panel mod buffers] = panel + 1 once that panel's activations are staged
  int x_taken[kBMaxXBuf];  // [panel mod buffers] += 1 by each compute wavefront that has copied the panel
                           // (per buffer: with two buffers a wavefront may be a panel ahead of another)
  int s_ready;       // items whose scales are staged
  int y_done;        // items whose partial sums have been added up
  int abort;         // a wait of this workgroup ran into the spin limit: nobody waits any more
  int pad;
  int done[kBRing];  // += 1 by each compute wavefront per item finished, by slot (item mod ring)
};
static_assert(sizeof(BatchFlags) == 64, "flags layout");

// Waits inside a workgroup are bounded like the waits between workgroups: a hand-over that never comes
// (a defect, or a wavefront that died) ends as an error word and a launch that finishes, not as a hang.
struct BatchWait {
  BatchFlags* flags;
  int* error;  // the list's error word
  long long limit;
  __device__ __forceinline__ void until(const int* flag, int target, int code) const {
    if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= target) {
      asm volatile("" ::: "memory");
      return;
    }
    const long long t0 = wall_clock64();
    while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < target) {
      if (__hip_atomic_load(&flags->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) break;
      if (wall_clock64() - t0 > limit) {
        __hip_atomic_store(&flags->abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        __hip_atomic_store(error, kBatchInternalWait + code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    asm volatile("" ::: "memory");  // LDS is served in order: what was written before the flag is visible now
  }
};

// TW = 1: a tile is 16 rows of W and the 8 compute wavefronts split the panel 8 ways along K.  TW = 2: a tile is
// 32 rows, wavefronts 0 .. 3 split the panel 4 ways for its rows 0 .. 15, wavefronts 4 .. 7 for rows 16 .. 31 (half
// as many hand-overs per byte of weights, twice the activations in a wavefront's registers).
// R: sets of 16 activation rows every wavefront holds.
__host__ __device__ constexpr int batch_k_ways(int TW) { return kBW / TW; }
__host__ __device__ constexpr int batch_panel_groups(int U, int TW) { return batch_k_ways(TW) * 4 * U; }
__host__ __device__ constexpr int batch_scale_row_bytes(int U, int TW) { return batch_panel_groups(U, TW) * 2 + 16; }  // + 16: rows on different banks
__host__ __device__ constexpr int batch_scale_slot_bytes(int U, int TW) { return 16 * TW * batch_scale_row_bytes(U, TW); }
__host__ __device__ constexpr int batch_partial_slot_bytes(int R) { return kBW * R * 1024; }  // per wavefront R sets of 16 activation rows
__host__ __device__ constexpr int batch_kept_bytes(int R, int TW) { return TW * R * 1024; }   // sums of a tile kept between panels

// ---- the walk of a workgroup over its items.  All fields are wavefront-uniform.
struct ItemCursor {
  int lin;           // current linear (nlin: past the end)
  int panel, lt;     // panel of K, local tile (tile = lt * ncu + rb)
  int lt0, ltend;    // the current chunk of local tiles: a linear of several panels is walked chunk by chunk, all
                     // panels of a chunk before the next chunk, so that LDS holds the sums of one chunk only
  int csize;         // tiles per chunk of this linear
  int T, P;          // tiles of this workgroup in the linear (> 0), panels
  int ncu, rb;       // workgroups in the linear's group; (member - off) mod ncu
  int N, G, row_w;   // rows, scale groups per row, bytes per row of W
  const char* W;
  const char* S;
};

// word 16 of a descriptor: gmod_log2 | gidx << 8 | rows << 16 (read as one word: a scalar load; single
// bytes would come through a vector load and end up in vector registers)
// Which workgroups run a linear (bits 0 .. 15 of that word), in two forms:
//   * gmod_log2 = g < 0x80: the workgroups with b mod 2^g == gidx (for g = 3 one XCD: workgroup b runs on XCD
//     b mod 8, so the activations stay in that XCD's L2);
//   * gmod_log2 = 0x80: gidx is a MASK of XCDs, the group is every workgroup whose b mod 8 is in the mask.  This is
//     what a short list uses: its few linears share the 8 XCDs in proportion to their bytes.
// A member's index counts the members in order of b.
struct GroupOf {
  bool member;
  int index, size;
};
__device__ __forceinline__ int group_size(uint32_t grp, int nwg) {
  if (grp & 0x80u) return (nwg >> 3) * __builtin_popcount((grp >> 8) & 0xffu);
  return nwg >> (grp & 0x7fu);
}
__device__ __forceinline__ GroupOf group_of(uint32_t grp, int b, int nwg) {
  GroupOf r;
  if (grp & 0x80u) {
    const uint32_t mask = (grp >> 8) & 0xffu;
    const int pc = __builtin_popcount(mask);
    r.member = (mask >> (b & 7)) & 1u;
    r.index = (b >> 3) * pc + __builtin_popcount(mask & ((1u << (b & 7)) - 1u));
    r.size = (nwg >> 3) * pc;
  } else {
    const int gl = (int)(grp & 0x7fu);
    r.member = (b & ((1 << gl) - 1)) == (int)((grp >> 8) & 0xffu);
    r.index = b >> gl;
    r.size = nwg >> gl;
  }
  return r;
}

__device__ __forceinline__ uint32_t desc_group_word(gemv_desc_ptr descs, int lin) {
  typedef const uint32_t __attribute__((address_space(4)))* words_ptr;
  return ((words_ptr)(descs + lin))[16];
}

// positions the cursor on the first linear >= c.lin in which this workgroup holds a tile
template <int PG, bool CH>
__device__ __forceinline__ void item_seek(ItemCursor& c, gemv_desc_ptr descs, int nlin, int b, int nwg, int chunk) {
  typedef const uint32_t __attribute__((address_space(4)))* words_ptr;
  while (c.lin < nlin) {
    const words_ptr p = (words_ptr)(descs + c.lin);
    const uint32_t grp = p[16];
    const GroupOf go = group_of(grp, b, nwg);
    if (go.member) {  // this workgroup's group runs the linear
      uint32_t w[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) w[i] = p[i];
      const int ncu = go.size;
      int rb = go.index - (int)(w[15] >> 16);
      if (rb < 0) rb += ncu;
      const int T = (int)w[13] + (rb < (int)(w[15] & 0xffffu) ? 1 : 0);
      if (T > 0) {
        const int G = (int)(w[14] & 0xffffu);
        c.T = T;
        c.rb = rb;
        c.ncu = ncu;
        c.G = G;
        c.P = (G + PG - 1) / PG;
        c.N = (int)w[12];
        c.row_w = G << 4;
        c.W = reinterpret_cast<const char*>(((uint64_t)w[1] << 32) | w[0]);
        c.S = reinterpret_cast<const char*>(((uint64_t)w[3] << 32) | w[2]);
        c.panel = 0;
        c.lt = 0;
        if constexpr (CH) {
          c.lt0 = 0;
          // chunks of equal size, at most `chunk` tiles (one panel: no sums are kept, one chunk)
          c.csize = T;
          if (c.P > 1 && T > chunk) {
            const int nch = (T + chunk - 1) / chunk;
            c.csize = (T + nch - 1) / nch;
          }
          c.ltend = c.csize;
        }
        return;
      }
    }
    ++c.lin;
  }
}

template <int PG, bool CH>
__device__ __forceinline__ void item_next_panel(ItemCursor& c, gemv_desc_ptr descs, int nlin, int b, int nwg, int chunk) {
  if constexpr (CH) {
    if (++c.panel == c.P) {
      c.panel = 0;
      c.lt0 = c.ltend;
      if (c.lt0 >= c.T) {
        ++c.lin;
        item_seek<PG, CH>(c, descs, nlin, b, nwg, chunk);
        return;
      }
      c.ltend = min(c.T, c.lt0 + c.csize);
    }
    c.lt = c.lt0;
  } else {
    c.lt = 0;
    if (++c.panel == c.P) {
      ++c.lin;
      item_seek<PG, CH>(c, descs, nlin, b, nwg, chunk);
    }
  }
}

template <int PG, bool CH>
__device__ __forceinline__ void item_next(ItemCursor& c, gemv_desc_ptr descs, int nlin, int b, int nwg, int chunk) {
  if (++c.lt == (CH ? c.ltend : c.T)) item_next_panel<PG, CH>(c, descs, nlin, b, nwg, chunk);
}

template <int U, int R, int TW, bool CH>
__global__ __launch_bounds__(kBThreads) void q4g32_batch_list_kernel(const GemvListDesc* __restrict__ descs_, int nlin,
                                                                     int* __restrict__ sync, long long spin_limit,
                                                                     int M, int nxb, int ring, int chunk, int use_sync) {
  constexpr int PG = batch_panel_groups(U, TW);  // scale groups per panel
  constexpr int KW = batch_k_ways(TW);          // wavefronts that share a panel along K
  constexpr int NT = kBNT;
  constexpr int SROW = batch_scale_row_bytes(U, TW), SSLOT = batch_scale_slot_bytes(U, TW);
  extern __shared__ uint4_t smem[];
  const gemv_desc_ptr descs = (gemv_desc_ptr)descs_;
  char* lds = reinterpret_cast<char*>(smem);
  // flags | nxb panels of activations, M x PG x 64 bytes each | `ring` scale slots | `ring` partial-sum slots |
  // sums kept between panels.  `ring` (2 or 4) is how many items the compute wavefronts may spread over.
  BatchFlags* flags = reinterpret_cast<BatchFlags*>(lds);
  char* const xbuf = lds + sizeof(BatchFlags);
  const int xbuf_bytes = M * (PG * 64);
  char* const sbuf = xbuf + nxb * xbuf_bytes;
  char* const pbuf = sbuf + ring * SSLOT;
  char* const abuf = pbuf + ring * batch_partial_slot_bytes(R);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nwg = gridDim.x;
  const int b = blockIdx.x;
  const BatchWait wait{flags, sync + sync_error_index(nlin), spin_limit > 0 ? spin_limit : 1000000};

  if (tid < (int)(sizeof(BatchFlags) / sizeof(int))) reinterpret_cast<int*>(flags)[tid] = 0;
  lds_done_then_barrier();  // LDS starts undefined: the flags are cleared before anyone looks

  if (wave < kBW) {
    // =========================== compute wavefront ===========================
    const int i = lane & 15, kq = lane >> 4;
    const int ks = wave & (KW - 1), rt = wave / KW;  // K slice of the panel; which 16 rows of the tile
    // The tile buffers are loaded in assembly and waited for by hand (loads retire in order and a
    // compute wavefront issues no other vector memory operation).  `magic` (0x6400 in both halves,
    // OR-ed under every code) doubles as the token that orders the reads of a buffer behind the wait
    // for it: the wait "modifies" magic, every first read of a buffer register takes magic as an
    // operand, and the registers appear in no other statement (checked in the generated code at
    // build time).
    uint4_t tb[NT][U];
    uint32_t magic = 0x64006400u;
    int ahead = 0;  // items issued and not yet consumed
    ItemCursor ic, cc;
    ic.lin = 0;
    item_seek<PG, CH>(ic, descs, nlin, b, nwg, chunk);
    cc = ic;
    int k = 0;    // items consumed
    int pk = -1;  // panels taken
    half8_t xb[R][U][4];
    const int gi0 = ks * (4 * U) + kq;  // the lane's scale group within the panel, chunk 0

    auto issue = [&](uint4_t (&buf)[U]) {
      if (ic.lin >= nlin) return;
      const int n0 = min(((ic.lt * ic.ncu + ic.rb) * TW + rt) << 4, ic.N - 1);  // (the second 16 rows of the last tile may lie past N)
      const int rows = min(16, ic.N - n0);                // >= 1
      const int pg = min(PG, ic.G - ic.panel * PG);       // scale groups of this panel (the last may be short)
      const char* base = ic.W + (int64_t)n0 * ic.row_w + ic.panel * (PG * 16);
      // rows past N repeat the last row (never stored); groups past K repeat the last group (their
      // activations and scales are staged as zeros)
      if constexpr (U >= 2) {
        // Whole 128-byte lines: the two loads of a pair of chunks take 8 rows each, lane (i, kq) the 16 bytes of
        // group 4 (i / 8) + kq of row i mod 8 (+ 8 for the second load), so a row contributes 128 contiguous
        // bytes to an instruction instead of 64 (measured on a 1 GiB stream with the full unpack + MFMA work:
        // 7.1 against 5.7 TB/s).  consume() puts the halves back where the MFMA wants them.
        const uint32_t roff_lo = __umul24((uint32_t)min(i & 7, rows - 1), (uint32_t)ic.row_w);
        const uint32_t roff_hi = __umul24((uint32_t)min(8 + (i & 7), rows - 1), (uint32_t)ic.row_w);
        const int gpair = ks * (4 * U) + (i >> 3) * 4 + kq;
#pragma unroll
        for (int u = 0; u < U; u += 2) {
          const uint32_t goff = (uint32_t)min(gpair + 4 * u, pg - 1) * 16u;
          asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=&v"(buf[u]) : "v"(roff_lo + goff), "s"(base));
          asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=&v"(buf[u + 1]) : "v"(roff_hi + goff), "s"(base));
        }
      } else {
        const uint32_t roff = __umul24((uint32_t)min(i, rows - 1), (uint32_t)ic.row_w);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t voff = roff + (uint32_t)min(gi0 + 4 * u, pg - 1) * 16u;
          asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=&v"(buf[u]) : "v"(voff), "s"(base));
        }
      }
      ++ahead;
      item_next<PG, CH>(ic, descs, nlin, b, nwg, chunk);
    };

    const half2_t k1031 = {(half_t)-1031.0f, (half_t)-1031.0f};
    const half2_t k1136 = {(half_t)-1136.0f, (half_t)-1136.0f};
    auto ring_shr8 = [&](uint32_t word) {
      uint32_t r;
      asm("v_lshrrev_b32 %0, 8, %1 ; %2" : "=v"(r) : "v"(word), "v"(magic));
      return r;
    };
    // (t + c) * s: two roundings, as the format defines.  Plain C++ on purpose: the products are the MFMA's A operand, and
    // the compiler only keeps the wait states between a VALU result and the MFMA that reads it for instructions
    // it has issued itself (written as inline assembly, v_pk_mul_f16 two instructions in front of the MFMA was
    // read before it had been written: the weights came out unscaled)
    auto unpack = [&](uint32_t t, half2_t c, half2_t s2) { return as_u32((as_half2(t) + c) * s2); };

    auto consume = [&](uint4_t (&buf)[U]) {
      if (cc.lt == (CH ? cc.lt0 : 0)) {
        // a new panel: its activations are staged (or will be); this wavefront's K slice goes to registers
        ++pk;
        const int xslot = pk % nxb;
        wait.until(&flags->x_ready[xslot], pk + 1, 1);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const char* xs = xbuf + xslot * xbuf_bytes + (ks * U * 16 * M + kq * M + min(i + 16 * r, M - 1)) * 16;
#pragma unroll
          for (int u = 0; u < U; ++u)
#pragma unroll
            for (int d = 0; d < 4; ++d) xb[r][u][d] = *reinterpret_cast<const half8_t*>(xs + ((u * 4 + d) * 4 * M) * 16);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) __hip_atomic_fetch_add(&flags->x_taken[xslot], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      wait.until(&flags->s_ready, k + 1, 2);
      const int slot = k & (ring - 1);
      const char* sb = sbuf + slot * SSLOT + (rt * 16 + i) * SROW + gi0 * 2;
      float4_t acc0[R], acc1[R];
#pragma unroll
      for (int r = 0; r < R; ++r) acc0[r] = acc1[r] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
      uint32_t cw[2][4];  // the chunks of a pair after the exchange
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const half_t sh = *reinterpret_cast<const half_t*>(sb + u * 8);
        const half2_t s16 = {sh, sh};
        if constexpr (U >= 2) {
          if ((u & 1) == 0) {
            // both loads of the pair have landed; lanes 8 .. 15 of every 16 take their half of chunk u from the second
            // load 8 lanes below, lanes 0 .. 7 their half of chunk u + 1 from the first load 8 lanes above (row_ror:8
            // turns a row of 16 lanes by 8).
            if (ahead == NT) asm volatile("s_waitcnt vmcnt(%1)" : "+v"(magic) : "n"((NT - 1) * U + (U - 2 - u)));
            else asm volatile("s_waitcnt vmcnt(0)" : "+v"(magic));
            // every ring register is first copied by a statement that depends on the wait (a cross-lane move with the
            // identity pattern: not an instruction the compiler would put there by itself), the exchange is the compiler's
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              const uint32_t lo_in = d == 0 ? buf[u].x : d == 1 ? buf[u].y : d == 2 ? buf[u].z : buf[u].w;
              const uint32_t hi_in = d == 0 ? buf[u | 1].x : d == 1 ? buf[u | 1].y : d == 2 ? buf[u | 1].z : buf[u | 1].w;
              uint32_t lo, hi;
              // (the s_nop: a DPP instruction must not read a register a VALU instruction wrote in the two cycles before it,
              // and the compiler does not count inline assembly as one)
              asm("v_mov_b32_dpp %0, %2 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xf\n\t"
                  "v_mov_b32_dpp %1, %3 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xf\n\t"
                  "s_nop 1 ; %4"
                  : "=&v"(lo), "=&v"(hi)
                  : "v"(lo_in), "v"(hi_in), "v"(magic));
              cw[0][d] = (uint32_t)__builtin_amdgcn_update_dpp((int)lo, (int)hi, 0x128 /* row_ror:8 */, 0xf, 0xc, false);
              cw[1][d] = (uint32_t)__builtin_amdgcn_update_dpp((int)hi, (int)lo, 0x128, 0xf, 0x3, false);
            }
          }
        } else {
          if (ahead == NT) asm volatile("s_waitcnt vmcnt(%1)" : "+v"(magic) : "n"((NT - 1) * U + (U - 1 - u)));
          else asm volatile("s_waitcnt vmcnt(0)" : "+v"(magic));
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          uint32_t word, w8;
          if constexpr (U >= 2) {
            word = cw[u & 1][d];
            w8 = word >> 8;
          } else {
            word = d == 0 ? buf[u].x : d == 1 ? buf[u].y : d == 2 ? buf[u].z : buf[u].w;
            w8 = ring_shr8(word);
          }
          const uint32_t a0 = unpack(and_or(word, 0x000F000Fu, magic), k1031, s16);  // (q0, q4)
          const uint32_t a1 = unpack(and_or(word, 0x00F000F0u, magic), k1136, s16);  // 16 (q1, q5)
          const uint32_t a2 = unpack(and_or(w8, 0x000F000Fu, magic), k1031, s16);    // (q2, q6)
          const uint32_t a3 = unpack(and_or(w8, 0x00F000F0u, magic), k1136, s16);    // 16 (q3, q7)
          const half8_t aop = __builtin_bit_cast(half8_t, uint4_t{a0, a1, a2, a3});
#pragma unroll
          for (int r = 0; r < R; ++r) {
            if (d & 1) acc1[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop, xb[r][u][d], acc1[r], 0, 0, 0);
            else acc0[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop, xb[r][u][d], acc0[r], 0, 0, 0);
          }
        }
      }
      --ahead;
      if (k >= ring) wait.until(&flags->y_done, k - ring + 1, 3);
#pragma unroll
      for (int r = 0; r < R; ++r)
        *reinterpret_cast<float4_t*>(pbuf + ((slot * kBW + wave) * R + r) * 1024 + lane * 16) = acc0[r] + acc1[r];
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (lane == 0) __hip_atomic_fetch_add(&flags->done[slot], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      ++k;
      item_next<PG, CH>(cc, descs, nlin, b, nwg, chunk);
    };

#pragma unroll
    for (int t = 0; t < NT - 1; ++t) issue(tb[t]);
    while (cc.lin < nlin) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        issue(tb[(t + NT - 1) % NT]);
        if (cc.lin < nlin) consume(tb[t]);
      }
    }
    return;
  }

  bool aborted = false;

  if (wave < kBW + kBXW) {
    // ====================== x wavefronts: a panel of activations -> LDS ======================
    const int xw = wave - kBW;
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
        if (__builtin_amdgcn_readfirstlane(v) >= group_size(desc_group_word(descs, dep), nwg)) break;  // every member of its group
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

    const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
    constexpr int PPR = PG * 4;  // 16-byte pieces (8 activations) per row and panel; a power of two
    constexpr int UX = 32;       // loads in flight per lane: one round trip for a panel of 8 rows x 2048 k
    ItemCursor xc;
    xc.lin = 0;
    item_seek<PG, CH>(xc, descs, nlin, b, nwg, chunk);
    // the x wavefronts take whole panels by turns (panel pk belongs to wavefront pk mod kBXW) and run up
    // to nxb panels ahead of the compute wavefronts: under load a round trip to L2 takes several microseconds
    int pk = 0;
    int confirmed = -1;  // the latest producer linear this wavefront has seen complete
    while (xc.lin < nlin) {
      if (pk % kBXW == xw) {
        const int xslot = pk % nxb;
        // the buffer is free once every compute wavefront has copied the panel that used it before
        if (pk >= nxb) wait.until(&flags->x_taken[xslot], kBW * (pk / nxb), 4);
        const int j = xc.lin;
        const int dep = (int)((descs[j].g_dep >> 16) & 0x7fffu) - 1;
        if (dep >= 0 && dep != confirmed) {
          wait_for(dep);
          confirmed = dep;
        }
        const int K = xc.G << 5;
        const int K8 = K >> 3;
        const int xrows = (int)((desc_group_word(descs, j) >> 16) & 0xffu);
        // an x that other workgroups of this launch have written is read with device-scope loads (sc1)
        const __amdgpu_buffer_rsrc_t xr =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(descs[j].x), 0, xrows * K * 2, kBufferFlags);
        char* const xdst = xbuf + xslot * xbuf_bytes;
        const int total = M * PPR;
        for (int base = 0; base < total; base += 64 * UX) {
          uint4_t v[UX];
#pragma unroll
          for (int t = 0; t < UX; ++t) {
            const int idx = base + t * 64 + lane;
            const int row = idx / PPR, o = idx & (PPR - 1);
            const int go = xc.panel * PPR + o;  // the piece's place in the row
            v[t] = uint4_t{0, 0, 0, 0};
            const int src = min(row, xrows - 1);  // rows past the entry's repeat its last row (never stored)
            if (idx < total && go < K8)
              v[t] = dep >= 0 ? __builtin_amdgcn_raw_buffer_load_b128(xr, (src * K8 + go) * 16, 0, kDeviceScope)
                              : __builtin_amdgcn_raw_buffer_load_b128(xr, (src * K8 + go) * 16, 0, 0);
          }
#pragma unroll
          for (int t = 0; t < UX; ++t) {
            const int idx = base + t * 64 + lane;
            if (idx < total) {
              const int row = idx / PPR, o = idx & (PPR - 1);
              const uint32_t in[4] = {v[t].x, v[t].y, v[t].z, v[t].w};
              uint32_t p[4];
              pair_i_i4(in, p);  // p[e] = (x_e, x_{e+4})
              // piece o: scale group g = o / 4, dword d = o % 4 of it; the group belongs to wavefront
              // g / 4U, chunk (g / 4) % U, lane quarter g % 4
              const int g = o >> 2, d = o & 3;
              const int cw = g / (4 * U), cu = (g >> 2) & (U - 1), ckq = g & 3;
              char* dst = xdst + ((((cw * U + cu) * 4 + d) * 4 + ckq) * M + row) * 16;
              *reinterpret_cast<uint4_t*>(dst) =
                  uint4_t{p[0], as_u32(as_half2(p[1]) * sixteenth), p[2], as_u32(as_half2(p[3]) * sixteenth)};
            }
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) __hip_atomic_store(&flags->x_ready[xslot], pk + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      ++pk;
      item_next_panel<PG, CH>(xc, descs, nlin, b, nwg, chunk);
    }
    return;
  }

  if (wave == kBW + kBXW) {
    // ====================== scale wavefront: the scales of a tile -> LDS ======================
    constexpr int PD = 6;            // items in flight in registers (a round trip under load is several items long)
    constexpr int PPR = PG / 8;      // 16-byte pieces (8 scales) per row and panel
    constexpr int LP = 16 * TW * PPR / 64;  // pieces per lane and item
    uint4_t sv[PD][LP];
    ItemCursor ic, cc;
    ic.lin = 0;
    item_seek<PG, CH>(ic, descs, nlin, b, nwg, chunk);
    cc = ic;
    int k = 0;
    auto issue = [&](uint4_t (&buf)[LP]) {
      if (ic.lin >= nlin) return;
      const int n0 = (ic.lt * ic.ncu + ic.rb) * (16 * TW);
      const int pg = min(PG, ic.G - ic.panel * PG);
      const char* base = ic.S + ic.panel * (PG * 2);
#pragma unroll
      for (int t = 0; t < LP; ++t) {
        const int idx = t * 64 + lane;
        const int r = idx / PPR, pc = idx % PPR;
        buf[t] = uint4_t{0, 0, 0, 0};  // groups past K: a zero scale
        if (pc * 8 < pg)
          buf[t] = __builtin_nontemporal_load(
              reinterpret_cast<const uint4_t*>(base + (int64_t)min(n0 + r, ic.N - 1) * (ic.G * 2) + pc * 16));
      }
      item_next<PG, CH>(ic, descs, nlin, b, nwg, chunk);
    };
    auto consume = [&](uint4_t (&buf)[LP]) {
      const int slot = k & (ring - 1);
      // the slot is free once every compute wavefront has finished the item that used it before
      if (k >= ring) wait.until(&flags->done[slot], kBW * (k / ring), 5);
#pragma unroll
      for (int t = 0; t < LP; ++t) {
        const int idx = t * 64 + lane;
        const int r = idx / PPR, pc = idx % PPR;
        *reinterpret_cast<uint4_t*>(sbuf + slot * SSLOT + r * SROW + pc * 16) = buf[t];
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      ++k;
      if (lane == 0) __hip_atomic_store(&flags->s_ready, k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      item_next<PG, CH>(cc, descs, nlin, b, nwg, chunk);
    };
#pragma unroll
    for (int t = 0; t < PD - 1; ++t) issue(sv[t]);
    while (cc.lin < nlin) {
#pragma unroll
      for (int t = 0; t < PD; ++t) {
        issue(sv[(t + PD - 1) % PD]);
        if (cc.lin < nlin) consume(sv[t]);
      }
    }
    return;
  }

  // ================== y wavefront: partial sums -> y, completion signals ==================
  {
    const int j16 = lane & 15, rq = lane >> 4;
    int k = 0;
    for (int lin = 0; lin < nlin; ++lin) {
      const uint32_t g_dep = descs[lin].g_dep;
      const uint32_t grp = desc_group_word(descs, lin);
      const GroupOf go = group_of(grp, b, nwg);
      if (!go.member) continue;  // another group's linear
      const int ncu = go.size;
      int rb = go.index - (int)descs[lin].off;
      if (rb < 0) rb += ncu;
      const int T = descs[lin].q + (rb < (int)descs[lin].rem ? 1 : 0);
      const int N = descs[lin].N;
      const int P = ((int)(g_dep & 0xffffu) + PG - 1) / PG;
      int csize = T;
      if (CH && P > 1 && T > chunk) {
        const int nch = (T + chunk - 1) / chunk;
        csize = (T + nch - 1) / nch;
      }
      const half_t* bias = descs[lin].bias;
      const half_t* residual = descs[lin].residual;
      const int yrows = (int)((grp >> 16) & 0xffu);
      const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(descs[lin].y, 0, yrows * N * 2, kBufferFlags);
      // the four outputs of a lane are adjacent in a row of y: one 8-byte store where the addresses allow it
      // (a store instruction waits its turn behind the weight loads of the whole workgroup)
      const bool wide = (N & 3) == 0 && (((uintptr_t)descs[lin].y | (uintptr_t)bias | (uintptr_t)residual) & 7) == 0;
      for (int lt0 = 0; lt0 < T; lt0 += csize) {
        const int ltend = min(T, lt0 + csize);
        for (int panel = 0; panel < P; ++panel) {
          for (int lt = lt0; lt < ltend; ++lt, ++k) {
            const int slot = k & (ring - 1);
            wait.until(&flags->done[slot], kBW * (k / ring + 1), 6);
            // sum[t][r]: rows 16 t .. of the tile, activation rows 16 r ..; the K slices in a fixed order
            const char* pb = pbuf + slot * batch_partial_slot_bytes(R) + lane * 16;
            float4_t sum[TW][R];
#pragma unroll
            for (int t = 0; t < TW; ++t)
#pragma unroll
              for (int r = 0; r < R; ++r) {
                sum[t][r] = *reinterpret_cast<const float4_t*>(pb + ((t * KW) * R + r) * 1024);
#pragma unroll
                for (int w = 1; w < KW; ++w) sum[t][r] += *reinterpret_cast<const float4_t*>(pb + ((t * KW + w) * R + r) * 1024);
              }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (lane == 0) __hip_atomic_store(&flags->y_done, k + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (P > 1) {
              float4_t* keep = reinterpret_cast<float4_t*>(abuf + (lt - lt0) * batch_kept_bytes(R, TW) + lane * 16);
              if (panel > 0) {
#pragma unroll
                for (int t = 0; t < TW; ++t)
#pragma unroll
                  for (int r = 0; r < R; ++r) sum[t][r] += keep[(t * R + r) * 64];
              }
              if (panel < P - 1) {
#pragma unroll
                for (int t = 0; t < TW; ++t)
#pragma unroll
                  for (int r = 0; r < R; ++r) keep[(t * R + r) * 64] = sum[t][r];
                continue;
              }
            }
#pragma unroll
            for (int t = 0; t < TW; ++t) {
              // lane (j, rq) holds rows n0 + 4 rq .. + 3 of activation rows j, j + 16
              const int n0 = (((lt * ncu + rb) * TW + t) << 4) + 4 * rq;
#pragma unroll
              for (int r = 0; r < R; ++r) {
                const int j = j16 + 16 * r;
                if (j < yrows && wide) {
                  if (n0 < N) {
                    float4_t v = sum[t][r];
                    if (bias) {
                      const half4_t bv = *reinterpret_cast<const half4_t*>(bias + n0);
#pragma unroll
                      for (int e = 0; e < 4; ++e) v[e] += (float)bv[e];
                    }
                    half4_t h = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                    if (residual) h = h + *reinterpret_cast<const half4_t*>(residual + (int64_t)j * N + n0);
                    // device-scope store: written through, so that a counter update after it publishes it
                    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uint2_t, h), yr, (j * N + n0) * 2, 0, kDeviceScope);
                  }
                } else if (j < yrows) {
#pragma unroll
                  for (int e = 0; e < 4; ++e) {
                    const int n = n0 + e;
                    if (n < N) {
                      float v = sum[t][r][e];
                      if (bias) v += (float)bias[n];
                      half_t h = (half_t)v;
                      if (residual) h = h + residual[(int64_t)j * N + n];
                      __builtin_amdgcn_raw_buffer_store_b16(as_u16(h), yr, (j * N + n) * 2, 0, kDeviceScope);
                    }
                  }
                }
              }
            }
          }
        }
      }
      if (g_dep & kSignal) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores of this workgroup have been written through
        if (lane == 0)
          __hip_atomic_fetch_add(sync + sync_counter_index(lin, b & (kCountersPerLinear - 1)), 1, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (!use_sync) return;
    // the last workgroup to get here clears the counters for the next launch (its own counter updates
    // have arrived by then: nothing of this launch may land on a cleared counter)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
}

// ====================================================================================================
// More than 16 activation rows: the wavefront that owns rows of W keeps their sums.
//
// With 17 .. 32 rows of activations a panel of 1024 k fills 64 KiB of LDS, the kernel above then hands over
// items of 16 KiB, and what an item costs in hand-overs (partial sums through LDS, the y wavefront's
// epilogue, the sums kept between panels) is paid four times per 4096 k.  Here nothing is handed over but the
// operands: a compute wavefront owns up to TR = 4 ROW TILES (16 rows each) of W for ALL of K, its accumulators
// (TR x R x 4 registers) stay in registers from the first panel to the last, and it writes its own outputs.
// The 8 compute wavefronts of a workgroup walk the panels of activations together (a PASS of the workgroup:
// up to 8 x 64 rows; the activations are loaded once per pass, which is why TR is as large as the registers
// allow: 167 of the 168 that 11 wavefronts leave each other).
//   * The activations of a panel (512 k: M x 1 KiB) lie in LDS in B-operand order; every compute wavefront
//     reads the operand of a (step, dword) pair once and uses it for its TR row tiles (LDS reads: 2 bytes per
//     byte of codes).  Two x wavefronts stage panels by turns into `nxb` buffers; a buffer is free again when
//     all 8 compute wavefronts have left it.
//   * One scale wavefront stages the scales of the rows of a pass, 1024 k (64 bytes per row) at a time, into
//     2 buffers.
//   * The unit of the weight stream is a PAIR of chunks of a wavefront's rows: 256 k, per row tile two loads of
//     8 rows x 128 bytes (whole lines; a lane exchange puts the halves where the MFMA wants them), 2 TR loads
//     in all, waited for by hand.  A pair is first exchanged into registers of its own and its ring slot
//     refilled at once, so two pairs (32 KiB per wavefront) are in flight while one is multiplied.  The loads
//     are buffer loads on the wavefront's rows of the pass: rows past them (a short last pass, the end of W)
//     read zeros without touching memory and are never stored; a wavefront without rows in a pass loads from
//     an empty buffer and only takes part in the hand-overs.
//   * A linear's completion counter is raised by the last of the 8 compute wavefronts to have its stores
//     written through.
// What bounds it (cycle counters around the phases of a compute wavefront, an instrumented copy): not memory.  A
// compute wavefront waits for its weights 1 % of the time; 43 .. 58 % goes into unpacking and multiplying a pair
// (about 1100 instructions, 6 .. 8 cycles each with two such wavefronts per SIMD), 13 .. 19 % into the lane
// exchange and the refill, and the wavefronts that share a SIMD with an older one are slower, so the older ones
// wait for them at the hand-over of the panels (35 % of their time).  Measured and not kept: B operands and
// scales requested from LDS one step ahead (no change), the refill spread over the multiplication (no change),
// a raised priority for the service wavefronts (M = 17 slower), 12 compute wavefronts of 48 rows (128 registers:
// 5 % slower), branches around the row tiles a short pass does not have (5 % slower: the unrolled code no longer
// interleaves).  The activations of every pass (M x K x 2 bytes per 512 rows: 22 % of the codes at M = 32)
// cost what their bytes cost: the stack step grows by 4.5 us per row of activations.
constexpr int kRW = 8;      // compute wavefronts
constexpr int kRXW = 2;     // wavefronts that stage activations
constexpr int kRThreads = 64 * (kRW + kRXW + 1);
constexpr int kRPairGroups = 8;   // scale groups per pair of chunks (256 k)
constexpr int kRPG = 16;          // scale groups per panel of activations
constexpr int kRSPG = 32;         // scale groups per panel of scales
constexpr int kRSRow = kRSPG * 2 + 16;  // LDS bytes per row of a panel of scales (+ 16: the 16 rows of a row tile on different banks)
constexpr int kRMaxXBuf = 4;

struct RowsFlags {
  int x_ready[kRMaxXBuf];  // [panel mod buffers] = panel + 1 once staged (panels counted over the whole launch)
  int x_taken[kRMaxXBuf];  // += 1 by each compute wavefront that has left the panel
  int s_ready[2], s_taken[2];  // the same for the panels of scales
  int lin_done[8];         // [linear mod 8] += 1 by each compute wavefront whose stores of the linear are written through
                           // (a wavefront is at most `nxb` <= 4 panels, hence linears, ahead of another)
  int exited;              // compute wavefronts that have finished the list
  int abort;               // a wait of this workgroup ran into the spin limit: nobody waits any more
  int pad[10];
};
static_assert(sizeof(RowsFlags) == 128, "flags layout");

struct RowsWait {
  int* abort;
  int* error;
  long long limit;
  __device__ __forceinline__ void until(const int* flag, int target, int code) const {
    if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= target) {
      asm volatile("" ::: "memory");
      return;
    }
    const long long t0 = wall_clock64();
    while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < target) {
      if (__hip_atomic_load(abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) break;
      if (wall_clock64() - t0 > limit) {
        __hip_atomic_store(abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        __hip_atomic_store(error, kBatchInternalWait + code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    asm volatile("" ::: "memory");
  }
};

// The walk of a workgroup over (linear, pass, pair of chunks).  All fields are wavefront-uniform.  A workgroup's
// share of a linear is a run of consecutive ROW TILES (16 rows); a pass takes up to 8 TR of them, `tr` per
// wavefront: TR while there are that many, and in the last pass as few as cover what is left with all 8
// wavefronts (three wave tiles of 64 rows left over: 6 wavefronts with 32 rows each, half the time).
struct RowsCursor {
  int lin;         // nlin: past the end
  int q, Q;        // pair of chunks within K
  int pos, left;   // first row tile of the pass; row tiles of the workgroup from there on (> 0)
  int tr;          // row tiles per wavefront in this pass (1 .. TR)
  int N, G, row_w;
  const char* W;
  const char* S;
  // row tiles of wavefront w in this pass, and the first of them
  __device__ __forceinline__ int tiles_of(int w, int TR) const { return max(0, min(tr, min(left, kRW * TR) - w * tr)); }
  __device__ __forceinline__ int first_of(int w) const { return pos + w * tr; }
};

template <int TR>
__device__ __forceinline__ void rows_begin_pass(RowsCursor& c) {
  c.q = 0;
  c.tr = (min(c.left, kRW * TR) + kRW - 1) / kRW;
}

// positions the cursor on the first linear >= c.lin in which this workgroup holds a row tile.  SIGNAL (the
// cursor that the first compute wavefront consumes with): a linear of this workgroup's group in which it
// holds none is signalled as complete on the way.
template <int TR, bool SIGNAL>
__device__ __forceinline__ void rows_seek(RowsCursor& c, gemv_desc_ptr descs, int nlin, int b, int nwg, int* sync, int lane) {
  typedef const uint32_t __attribute__((address_space(4)))* words_ptr;
  while (c.lin < nlin) {
    const words_ptr p = (words_ptr)(descs + c.lin);
    const uint32_t grp = p[16];
    const GroupOf go = group_of(grp, b, nwg);
    if (go.member) {  // this workgroup's group runs the linear
      const int ncu = go.size;
      const uint32_t w15 = p[15];
      int rb = go.index - (int)(w15 >> 16);
      if (rb < 0) rb += ncu;
      const int q = (int)p[13], rem = (int)(w15 & 0xffffu);
      const int cnt = q + (rb < rem ? 1 : 0);
      if (cnt > 0) {
        const uint32_t w14 = p[14];
        const int G = (int)(w14 & 0xffffu);
        c.left = cnt;
        c.pos = rb * q + min(rb, rem);
        c.G = G;
        c.Q = G / kRPairGroups;
        c.N = (int)p[12];
        c.row_w = G << 4;
        c.W = reinterpret_cast<const char*>(((uint64_t)p[1] << 32) | p[0]);
        c.S = reinterpret_cast<const char*>(((uint64_t)p[3] << 32) | p[2]);
        rows_begin_pass<TR>(c);
        return;
      }
      if (SIGNAL && (p[14] & kSignal) && lane == 0)
        __hip_atomic_fetch_add(sync + sync_counter_index(c.lin, b & (kCountersPerLinear - 1)), 1, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }
    ++c.lin;
  }
}

template <int TR, bool SIGNAL>
__device__ __forceinline__ void rows_advance(RowsCursor& c, int step, gemv_desc_ptr descs, int nlin, int b, int nwg, int* sync, int lane) {
  c.q += step;
  if (c.q < c.Q) return;
  const int took = min(c.left, kRW * TR);
  c.pos += took;
  c.left -= took;
  if (c.left > 0) {
    rows_begin_pass<TR>(c);
    return;
  }
  ++c.lin;
  rows_seek<TR, SIGNAL>(c, descs, nlin, b, nwg, sync, lane);
}

template <int TR, int R>
__global__ __launch_bounds__(kRThreads) void q4g32_batch_rows_kernel(const GemvListDesc* __restrict__ descs_, int nlin,
                                                                     int* __restrict__ sync, long long spin_limit,
                                                                     int M, int nxb, int use_sync) {
  constexpr int TROWS = 16 * TR;                 // rows of a wave tile
  constexpr int SBUF = kRW * TROWS * kRSRow;     // bytes of a buffer of scales
  extern __shared__ uint4_t smem[];
  const gemv_desc_ptr descs = (gemv_desc_ptr)descs_;
  char* lds = reinterpret_cast<char*>(smem);
  // flags | nxb panels of activations, M x 1 KiB each | 2 panels of scales
  RowsFlags* flags = reinterpret_cast<RowsFlags*>(lds);
  char* const xbuf = lds + sizeof(RowsFlags);
  const int xbuf_bytes = M * (kRPG * 64);
  char* const sbuf = xbuf + nxb * xbuf_bytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nwg = gridDim.x;
  const int b = blockIdx.x;
  const RowsWait wait{&flags->abort, sync + sync_error_index(nlin), spin_limit > 0 ? spin_limit : 1000000};

  if (tid < (int)(sizeof(RowsFlags) / sizeof(int))) reinterpret_cast<int*>(flags)[tid] = 0;
  lds_done_then_barrier();

  if (wave < kRW) {
    // =========================== compute wavefront ===========================
    const int i = lane & 15, kq = lane >> 4;
    constexpr int NT = 2;        // ring slots: both in flight while a pair is multiplied (out of registers of its own)
    constexpr int LPI = 2 * TR;  // loads per pair
    // The ring is loaded in assembly and waited for by hand, as in the kernel above: `magic` orders the first
    // read of every ring register behind the wait.
    uint4_t tb[NT][TR][2];
    uint32_t magic = 0x64006400u;
    int ahead = 0;
    RowsCursor ic, cc;
    ic.lin = 0;
    rows_seek<TR, false>(ic, descs, nlin, b, nwg, sync, lane);
    cc.lin = 0;
    if (wave == 0) rows_seek<TR, true>(cc, descs, nlin, b, nwg, sync, lane);
    else rows_seek<TR, false>(cc, descs, nlin, b, nwg, sync, lane);

    // the buffer of this wavefront's rows in the pass the cursor is in: rows past it read zeros
    auto tile_rsrc = [&](const RowsCursor& c) {
      const int nt = c.tiles_of(wave, TR);
      const int row0 = c.first_of(wave) * 16;
      const int rows = nt > 0 ? min(nt * 16, c.N - row0) : 0;
      const uint64_t a = reinterpret_cast<uint64_t>(c.W + (int64_t)(nt > 0 ? row0 : 0) * c.row_w);
      return uint4_t{(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, (uint32_t)(rows * c.row_w), (uint32_t)kBufferFlags};
    };

    uint4_t i_rsrc = uint4_t{0, 0, 0, (uint32_t)kBufferFlags};
    uint32_t i_voff = 0;
    auto issue = [&](uint4_t (&buf)[TR][2]) {
      if (ic.lin >= nlin) return;
      if (ic.q == 0) {
        i_rsrc = tile_rsrc(ic);
        // lane (i, kq): row i mod 8 of the half tile, scale group 4 (i / 8) + kq of the pair
        i_voff = __umul24((uint32_t)(i & 7), (uint32_t)ic.row_w) + (uint32_t)(((i >> 3) * 4 + kq) * 16);
      }
      const uint32_t rw8 = (uint32_t)ic.row_w * 8u;
      uint32_t soff = (uint32_t)ic.q * (kRPairGroups * 16);
#pragma unroll
      for (int t = 0; t < TR; ++t) {
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen nt" : "=&v"(buf[t][0]) : "v"(i_voff), "s"(i_rsrc), "s"(soff));
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen nt" : "=&v"(buf[t][1]) : "v"(i_voff), "s"(i_rsrc), "s"(soff + rw8));
        soff += 2 * rw8;
      }
      ++ahead;
      rows_advance<TR, false>(ic, 1, descs, nlin, b, nwg, sync, lane);
    };

    const half2_t k1031 = {(half_t)-1031.0f, (half_t)-1031.0f};
    const half2_t k1136 = {(half_t)-1136.0f, (half_t)-1136.0f};
    auto unpack = [&](uint32_t t, half2_t c, half2_t s2) { return as_u32((as_half2(t) + c) * s2); };

    float4_t acc[TR][R];
    int pk = -1, sk = -1;  // panels of activations / of scales taken (counted over the launch)
    int c_tr = 0;    // row tiles of this wavefront in the pass being multiplied
    int c_row0 = 0;

    auto epilogue = [&]() {
      const int lin = cc.lin;
      const int j16 = lane & 15, rq = lane >> 4;
      const half_t* bias = descs[lin].bias;
      const half_t* residual = descs[lin].residual;
      const int N = cc.N;
      const int yrows = (int)((desc_group_word(descs, lin) >> 16) & 0xffu);
      const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(descs[lin].y, 0, yrows * N * 2, kBufferFlags);
      const bool wide = (N & 3) == 0 && (((uintptr_t)descs[lin].y | (uintptr_t)bias | (uintptr_t)residual) & 7) == 0;
#pragma unroll
      for (int t = 0; t < TR; ++t) {
        if (t >= c_tr) break;
        // lane (j, rq) holds rows n0 .. n0 + 3 of activation rows j, j + 16
        const int n0 = c_row0 + 16 * t + 4 * rq;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int j = j16 + 16 * r;
          if (j < yrows && wide) {
            if (n0 < N) {
              float4_t v = acc[t][r];
              if (bias) {
                const half4_t bv = *reinterpret_cast<const half4_t*>(bias + n0);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += (float)bv[e];
              }
              half4_t h = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
              if (residual) h = h + *reinterpret_cast<const half4_t*>(residual + (int64_t)j * N + n0);
              // device-scope store: written through, so that a counter update after it publishes it
              __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uint2_t, h), yr, (j * N + n0) * 2, 0, kDeviceScope);
            }
          } else if (j < yrows) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int n = n0 + e;
              if (n < N) {
                float v = acc[t][r][e];
                if (bias) v += (float)bias[n];
                half_t h = (half_t)v;
                if (residual) h = h + residual[(int64_t)j * N + n];
                __builtin_amdgcn_raw_buffer_store_b16(as_u16(h), yr, (j * N + n) * 2, 0, kDeviceScope);
              }
            }
          }
        }
      }
    };

    auto consume = [&](uint4_t (&buf)[TR][2]) {
      if (cc.q == 0) {
        c_tr = cc.tiles_of(wave, TR);
        c_row0 = cc.first_of(wave) * 16;
#pragma unroll
        for (int t = 0; t < TR; ++t)
#pragma unroll
          for (int r = 0; r < R; ++r) acc[t][r] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
      }
      if ((cc.q & 1) == 0) {
        ++pk;
        wait.until(&flags->x_ready[pk % nxb], pk + 1, 1);
      }
      if ((cc.q & 3) == 0) {
        ++sk;
        wait.until(&flags->s_ready[sk & 1], sk + 1, 2);
      }
      if (ahead == NT) asm volatile("s_waitcnt vmcnt(%1)" : "+v"(magic) : "n"((NT - 1) * LPI));
      else asm volatile("s_waitcnt vmcnt(0)" : "+v"(magic));
      // Both loads of every row tile have landed.  The chunks of the pair, put where the MFMA wants them: lanes 8 .. 15
      // of every 16 take their half of chunk 0 from the second load 8 lanes below (row_ror:8 turns a row of 16 lanes
      // by 8), lanes 0 .. 7 their half of chunk 1 from the first load 8 lanes above.  The statements depend on the wait
      // through `magic`; they are volatile so that they stay in front of the loads that refill the slot.
      uint32_t cw[TR][2][4];
#pragma unroll
      for (int t = 0; t < TR; ++t)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t lo_in = d == 0 ? buf[t][0].x : d == 1 ? buf[t][0].y : d == 2 ? buf[t][0].z : buf[t][0].w;
          const uint32_t hi_in = d == 0 ? buf[t][1].x : d == 1 ? buf[t][1].y : d == 2 ? buf[t][1].z : buf[t][1].w;
          asm volatile("v_mov_b32_dpp %0, %2 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xf\n\t"
                       "v_mov_b32_dpp %1, %3 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xf\n\t"
                       "v_mov_b32_dpp %0, %3 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                       "v_mov_b32_dpp %1, %2 row_ror:8 row_mask:0xf bank_mask:0x3 ; %4"
                       : "=&v"(cw[t][0][d]), "=&v"(cw[t][1][d])
                       : "v"(lo_in), "v"(hi_in), "v"(magic));
        }
      // the slot is free: the pair after the next one goes into it, so that two pairs are in flight while this one
      // is multiplied
      --ahead;
      issue(buf);
      if (c_tr > 0) {
        const char* const xs = xbuf + (pk % nxb) * xbuf_bytes + (kq * M + min(i, M - 1)) * 16;
        const int xr1 = (min(i + 16, M - 1) - min(i, M - 1)) * 16;  // second set of 16 activation rows
        const char* const ss = sbuf + (sk & 1) * SBUF + (wave * TROWS + i) * kRSRow + ((cc.q & 3) * kRPairGroups + kq) * 2;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          half2_t s16[TR];
#pragma unroll
          for (int t = 0; t < TR; ++t) {
            const half_t sh = *reinterpret_cast<const half_t*>(ss + t * 16 * kRSRow + u * 8);
            s16[t] = half2_t{sh, sh};
          }
          const int step = (cc.q & 1) * 2 + u;  // 128 k each within the panel
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            half8_t xb[R];
#pragma unroll
            for (int r = 0; r < R; ++r)
              xb[r] = *reinterpret_cast<const half8_t*>(xs + ((step * 4 + d) * 4 * M) * 16 + r * xr1);
#pragma unroll
            for (int t = 0; t < TR; ++t) {
              const uint32_t word = cw[t][u][d];  // (row tiles past the wavefront's share of a short pass: zeros)
              const uint32_t w8 = word >> 8;
              const uint32_t a0 = unpack(and_or(word, 0x000F000Fu, magic), k1031, s16[t]);  // (q0, q4)
              const uint32_t a1 = unpack(and_or(word, 0x00F000F0u, magic), k1136, s16[t]);  // 16 (q1, q5)
              const uint32_t a2 = unpack(and_or(w8, 0x000F000Fu, magic), k1031, s16[t]);    // (q2, q6)
              const uint32_t a3 = unpack(and_or(w8, 0x00F000F0u, magic), k1136, s16[t]);    // 16 (q3, q7)
              const half8_t aop = __builtin_bit_cast(half8_t, uint4_t{a0, a1, a2, a3});
#pragma unroll
              for (int r = 0; r < R; ++r) acc[t][r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop, xb[r], acc[t][r], 0, 0, 0);
            }
          }
        }
      }
      const bool last = cc.q == cc.Q - 1;
      if ((cc.q & 1) == 1 || last) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wavefront's reads of the panel have returned
        if (lane == 0) __hip_atomic_fetch_add(&flags->x_taken[pk % nxb], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (((cc.q & 3) == 3 || last) && lane == 0)
          __hip_atomic_fetch_add(&flags->s_taken[sk & 1], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      if (last) {
        if (c_tr > 0) epilogue();
        if (cc.left <= kRW * TR && (descs[cc.lin].g_dep & kSignal)) {
          // the linear is complete once the stores of all 8 compute wavefronts are written through
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          int old = 0;
          int* const cnt = &flags->lin_done[cc.lin & 7];
          if (lane == 0) old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          if (__builtin_amdgcn_readfirstlane(old) == kRW - 1 && lane == 0) {
            __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __hip_atomic_fetch_add(sync + sync_counter_index(cc.lin, b & (kCountersPerLinear - 1)), 1, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      }
      if (wave == 0) rows_advance<TR, true>(cc, 1, descs, nlin, b, nwg, sync, lane);
      else rows_advance<TR, false>(cc, 1, descs, nlin, b, nwg, sync, lane);
    };

#pragma unroll
    for (int t = 0; t < NT; ++t) issue(tb[t]);
    while (cc.lin < nlin) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (cc.lin < nlin) consume(tb[t]);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing of the ring (or of the signals) is in flight any more
    if (!use_sync) return;
    // the last compute wavefront of the last workgroup to get here clears the counters for the next launch
    int old = 0;
    if (lane == 0) old = __hip_atomic_fetch_add(&flags->exited, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (__builtin_amdgcn_readfirstlane(old) != kRW - 1) return;
    int lastwg = 0;
    if (lane == 0)
      lastwg = __hip_atomic_fetch_add(sync + sync_finished_index(nlin), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nwg - 1;
    if (__builtin_amdgcn_readfirstlane(lastwg)) {
      for (int k = lane; k < nlin * kCountersPerLinear; k += 64)
        __hip_atomic_store(sync + k * kCounterStride, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (lane == 0)
        __hip_atomic_store(sync + sync_finished_index(nlin), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return;
  }

  if (wave < kRW + kRXW) {
    // ====================== x wavefronts: a panel of activations -> LDS ======================
    const int xw = wave - kRW;
    bool aborted = false;
    auto wait_for = [&](int dep) {
      if (aborted) return;
      const long long t0 = wall_clock64();
      while (true) {
        int v = 0;
        if (lane < kCountersPerLinear)
          v = __hip_atomic_fetch_add(sync + sync_counter_index(dep, lane), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v += __shfl_xor(v, 1, 64);
        v += __shfl_xor(v, 2, 64);
        v += __shfl_xor(v, 4, 64);
        if (__builtin_amdgcn_readfirstlane(v) >= group_size(desc_group_word(descs, dep), nwg)) break;  // every member of its group
        if (wall_clock64() - t0 > spin_limit) {
          aborted = true;
          if (lane == 0)
            __hip_atomic_store(sync + sync_error_index(nlin), dep + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(4);
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    };
    const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
    constexpr int PPR = kRPG * 4;  // 16-byte pieces (8 activations) per row and panel
    constexpr int UX = 32;         // loads in flight per lane: a whole panel of 32 rows
    RowsCursor xc;
    xc.lin = 0;
    rows_seek<TR, false>(xc, descs, nlin, b, nwg, sync, lane);
    int pk = 0;
    int confirmed = -1;
    while (xc.lin < nlin) {
      if (pk % kRXW == xw) {
        const int xslot = pk % nxb;
        if (pk >= nxb) wait.until(&flags->x_taken[xslot], kRW * (pk / nxb), 4);
        const int j = xc.lin;
        const int dep = (int)((descs[j].g_dep >> 16) & 0x7fffu) - 1;
        if (dep >= 0 && dep != confirmed) {
          wait_for(dep);
          confirmed = dep;
        }
        const int K8 = xc.G << 2;
        const int xrows = (int)((desc_group_word(descs, j) >> 16) & 0xffu);
        const __amdgpu_buffer_rsrc_t xr =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(descs[j].x), 0, xrows * K8 * 16, kBufferFlags);
        char* const xdst = xbuf + xslot * xbuf_bytes;
        const int p0 = xc.q * (kRPairGroups * 4);  // the panel's first piece within a row
        const int total = M * PPR;
        for (int base = 0; base < total; base += 64 * UX) {
          uint4_t v[UX];
#pragma unroll
          for (int t = 0; t < UX; ++t) {
            const int idx = base + t * 64 + lane;
            const int row = idx / PPR, o = idx & (PPR - 1);
            const int go = p0 + o;
            v[t] = uint4_t{0, 0, 0, 0};
            const int src = min(row, xrows - 1);
            if (idx < total && go < K8)
              v[t] = dep >= 0 ? __builtin_amdgcn_raw_buffer_load_b128(xr, (src * K8 + go) * 16, 0, kDeviceScope)
                              : __builtin_amdgcn_raw_buffer_load_b128(xr, (src * K8 + go) * 16, 0, 0);
          }
#pragma unroll
          for (int t = 0; t < UX; ++t) {
            const int idx = base + t * 64 + lane;
            if (idx < total) {
              const int row = idx / PPR, o = idx & (PPR - 1);
              const uint32_t in[4] = {v[t].x, v[t].y, v[t].z, v[t].w};
              uint32_t p[4];
              pair_i_i4(in, p);  // p[e] = (x_e, x_{e+4})
              // piece o: scale group g = o / 4 of the panel, dword d = o % 4 of it; step g / 4, lane quarter g % 4
              const int g = o >> 2, d = o & 3;
              char* dst = xdst + ((((g >> 2) * 4 + d) * 4 + (g & 3)) * M + row) * 16;
              *reinterpret_cast<uint4_t*>(dst) =
                  uint4_t{p[0], as_u32(as_half2(p[1]) * sixteenth), p[2], as_u32(as_half2(p[3]) * sixteenth)};
            }
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) __hip_atomic_store(&flags->x_ready[xslot], pk + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      ++pk;
      rows_advance<TR, false>(xc, kRPG / kRPairGroups, descs, nlin, b, nwg, sync, lane);
    }
    return;
  }

  // ====================== scale wavefront: the scales of a pass, 1024 k at a time -> LDS ======================
  {
    constexpr int PPR = kRSPG / 8;              // 16-byte pieces (8 scales) per row and panel
    constexpr int LP = kRW * TROWS * PPR / 64;  // pieces per lane and panel
    RowsCursor sc;
    sc.lin = 0;
    rows_seek<TR, false>(sc, descs, nlin, b, nwg, sync, lane);
    int sk = 0;
    while (sc.lin < nlin) {
      const int sslot = sk & 1;
      const int g0 = sc.q * kRPairGroups;  // first scale group of the panel
      const __amdgpu_buffer_rsrc_t sr = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<char*>(sc.S), 0, (int)min((int64_t)sc.N * sc.G * 2, (int64_t)0x7fffffff), kBufferFlags);
      uint4_t v[LP];
#pragma unroll
      for (int t = 0; t < LP; ++t) {
        const int idx = t * 64 + lane;
        const int rr = idx / PPR, pc = idx % PPR;
        const int w = rr / TROWS, r = rr % TROWS;
        const int row = sc.first_of(w) * 16 + r;
        v[t] = uint4_t{0, 0, 0, 0};  // rows past the wavefront's or past N, groups past K: a zero scale
        if (r < sc.tiles_of(w, TR) * 16 && row < sc.N && g0 + pc * 8 < sc.G)
          v[t] = __builtin_amdgcn_raw_buffer_load_b128(sr, (row * sc.G + g0 + pc * 8) * 2, 0, 0);
      }
      // the buffer is free once every compute wavefront has left the panel that used it before
      if (sk >= 2) wait.until(&flags->s_taken[sslot], kRW * (sk / 2), 5);
#pragma unroll
      for (int t = 0; t < LP; ++t) {
        const int idx = t * 64 + lane;
        const int rr = idx / PPR, pc = idx % PPR;
        *reinterpret_cast<uint4_t*>(sbuf + sslot * SBUF + rr * kRSRow + pc * 16) = v[t];
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      ++sk;
      if (lane == 0) __hip_atomic_store(&flags->s_ready[sslot], sk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      rows_advance<TR, false>(sc, kRSPG / kRPairGroups, descs, nlin, b, nwg, sync, lane);
    }
  }
}

// ------------------------------------------------------------------ host side
// the kernel a list of M activation rows runs: chunks per wavefront and tile, sets of 16 activation rows, tile rows / 16
struct BatchShape {
  int U, R, TW;
};
static BatchShape batch_shape(int M) {
  if (M <= 8) return {4, 1, 1};   // tiles of 16 rows, panels of 4096 k (tiles of 32 rows x 2048 k: the same time at M = 8, slower at M = 4)
  return {4, 1, 2};               // 32 rows, 2048 k (16 rows x 2048 k, chunks of 2: 0.90 instead of 0.81 ms for the Llama-2-7B stack)
}                                 // (more than 16 rows: q4g32_batch_rows_kernel)

static size_t batch_lds_bytes(BatchShape s, int M, int nxb, int ring, int acc_tiles) {
  return sizeof(BatchFlags) + (size_t)nxb * M * batch_panel_groups(s.U, s.TW) * 64 + (size_t)ring * batch_scale_slot_bytes(s.U, s.TW) +
         (size_t)ring * batch_partial_slot_bytes(s.R) + (size_t)acc_tiles * batch_kept_bytes(s.R, s.TW);
}

// Which group of workgroups runs which linear.  Every workgroup needs all M x K activations of a linear
// it takes part in, and those bytes cost what weight bytes cost (they pass the same memory pipeline of the
// CU): with 256 workgroups on a 4096-row linear that is twice the weights at M = 8.  So a list is run by 2^g
// groups side by side, each linear by one group (group = workgroup index mod 2^g, which is one XCD for
// g = 3: the activations then stay in that XCD's L2): a workgroup sees 1 / 2^g of the linears and 2^g times
// as many rows of each.  Linears go, in list order, to the group that can start them first (a consumer
// not before its producer has ended), with the duration of a linear estimated from the bytes a workgroup
// moves for it; g is the best of 0 .. 4 by that estimate (32-layer Llama-2-7B stack, M = 8: 1.25 ms with one
// group, 0.89 ms with 8, 0.85 ms with 16).
struct BatchGroupPlan {
  std::vector<int> group;
  double makespan = 0.0;
};

// chunks a workgroup with `tiles` tiles of a linear walks them in (each chunk loads every panel of activations again)
static int batch_chunks(int tiles, int panels, int chunk) { return panels > 1 && tiles > chunk ? (tiles + chunk - 1) / chunk : 1; }

// bytes through one workgroup of a group of `ncu` for linear i: its tiles' codes and scales, and all activations
// once per chunk
static double batch_linear_cost(const wq_gemv_list* l, int i, int ncu, BatchShape s, int chunk) {
  const GemvListDesc& g = l->descs[i];
  const int G = (int)(g.g_dep & 0xffffu);
  const double K = (double)G * 32.0;
  const int trows = 16 * s.TW;
  const double tiles = (double)((((int64_t)g.N + trows - 1) / trows + ncu - 1) / ncu);  // of one workgroup
  const int panels = (G + batch_panel_groups(s.U, s.TW) - 1) / batch_panel_groups(s.U, s.TW);
  return tiles * trows * K * (0.5 + 1.0 / 16.0) + batch_chunks((int)tiles, panels, chunk) * l->M * K * 2.0 + 4096.0;
}

// A SHORT list has too few linears for equal groups to be both many (so that few workgroups load a linear's
// activations) and busy.  Its linears share the 8 XCDs instead, level by level: the linears of a dependency
// level (level = 1 + the level of the producer) run side by side, each on a set of XCDs in proportion to what
// it costs, every set at least one XCD; levels follow each other.  cost(i, workgroups of the group) as above.
struct MaskPlan {
  bool ok = false;
  std::vector<uint8_t> mask;  // XCDs of linear i
  double makespan = 0.0;
};
template <class Cost>
static MaskPlan plan_xcd_masks(const wq_gemv_list* l, Cost cost) {
  MaskPlan plan;
  if (l->blocks % 8 != 0 || l->n > 64) return plan;
  const int per_xcd = l->blocks / 8;
  std::vector<int> level(l->n, 0);
  int levels = 0;
  for (int i = 0; i < l->n; ++i) {
    const int dep = (int)((l->descs[i].g_dep >> 16) & 0x7fffu) - 1;
    level[i] = dep >= 0 ? level[dep] + 1 : 0;
    levels = std::max(levels, level[i] + 1);
  }
  plan.mask.assign(l->n, 0);
  for (int lv = 0; lv < levels; ++lv) {
    std::vector<int> who;
    for (int i = 0; i < l->n; ++i)
      if (level[i] == lv) who.push_back(i);
    if (who.size() > 8) return plan;  // a long list: equal groups
    std::vector<int> k(who.size(), 1);
    for (int left = 8 - (int)who.size(); left > 0; --left) {  // one more XCD to whoever takes longest
      size_t worst = 0;
      for (size_t a = 1; a < who.size(); ++a)
        if (cost(who[a], per_xcd * k[a]) > cost(who[worst], per_xcd * k[worst])) worst = a;
      ++k[worst];
    }
    double t = 0.0;
    int next = 0;
    for (size_t a = 0; a < who.size(); ++a) {
      plan.mask[who[a]] = (uint8_t)(((1u << k[a]) - 1u) << next);
      next += k[a];
      t = std::max(t, cost(who[a], per_xcd * k[a]));
    }
    plan.makespan += t;
  }
  plan.ok = true;
  return plan;
}

static BatchGroupPlan batch_assign_groups(const wq_gemv_list* l, int gl, BatchShape s, int chunk) {
  const int groups = 1 << gl, ncu = l->blocks >> gl;
  BatchGroupPlan plan;
  plan.group.resize(l->n);
  std::vector<double> free_at(groups, 0.0), end(l->n, 0.0);
  for (int i = 0; i < l->n; ++i) {
    const GemvListDesc& g = l->descs[i];
    const double dur = batch_linear_cost(l, i, ncu, s, chunk);
    const int dep = (int)((g.g_dep >> 16) & 0x7fffu) - 1;
    const double ready = dep >= 0 ? end[dep] : 0.0;
    int best = 0;
    for (int c = 1; c < groups; ++c) {
      const double sb = std::max(free_at[best], ready), sc = std::max(free_at[c], ready);
      if (sc < sb || (sc == sb && free_at[c] > free_at[best])) best = c;  // earliest start, then least idle time
    }
    plan.group[i] = best;
    end[i] = std::max(free_at[best], ready) + dur;
    free_at[best] = end[i];
  }
  for (double f : free_at) plan.makespan = std::max(plan.makespan, f);
  return plan;
}

// the kernel that walks the tiles of a linear in chunks carries more loop state: only where a list needs it
typedef void (*batch_kernel_t)(const GemvListDesc*, int, int*, long long, int, int, int, int, int);
static int batch_kernel_index(BatchShape s) { return s.TW == 2 ? 1 : 0; }
static batch_kernel_t batch_kernel(BatchShape s, bool chunked) {
  switch (batch_kernel_index(s)) {
    case 1: return chunked ? q4g32_batch_list_kernel<4, 1, 2, true> : q4g32_batch_list_kernel<4, 1, 2, false>;
    default: return chunked ? q4g32_batch_list_kernel<4, 1, 1, true> : q4g32_batch_list_kernel<4, 1, 1, false>;
  }
}

// ---- lists of more than 16 activation rows: q4g32_batch_rows_kernel
constexpr int kRowsTR = 4;  // row tiles of a wave tile: 64 rows
static size_t rows_lds_bytes(int M, int nxb) {
  return sizeof(RowsFlags) + (size_t)nxb * M * kRPG * 64 + 2 * (size_t)kRW * 16 * kRowsTR * kRSRow;
}

// as batch_assign_groups, with the duration of a linear from the passes a workgroup makes over its wave tiles
// (every pass loads all activations; a pass of fewer than 8 wave tiles takes as long as a full one)
// pass by pass: all activations, and the time of 8 wavefronts x TR row tiles however few rows the pass holds (a
// wavefront unpacks and multiplies TR row tiles per pair either way; measured on the 32-layer Llama-2-7B stack,
// M = 32: 16 groups, where the 4096-row linears make one pass of 32 rows per wavefront, 1.19 ms; 32 groups 0.945 ms)
static double rows_linear_cost(const wq_gemv_list* l, int i, int ncu) {
  const GemvListDesc& g = l->descs[i];
  const double K = (double)(g.g_dep & 0xffffu) * 32.0;
  const int64_t tiles = ((int64_t)g.N + 15) / 16;   // row tiles
  const int64_t left = (tiles + ncu - 1) / ncu;      // of the workgroup with most
  const double passes = (double)((left + kRW * kRowsTR - 1) / (kRW * kRowsTR));
  return 4096.0 + passes * (kRW * kRowsTR * 16.0 * K * (0.5 + 1.0 / 16.0) + l->M * K * 2.0);
}

static BatchGroupPlan rows_assign_groups(const wq_gemv_list* l, int gl) {
  const int groups = 1 << gl, ncu = l->blocks >> gl;
  BatchGroupPlan plan;
  plan.group.resize(l->n);
  std::vector<double> free_at(groups, 0.0), end(l->n, 0.0);
  for (int i = 0; i < l->n; ++i) {
    const GemvListDesc& g = l->descs[i];
    const double dur = rows_linear_cost(l, i, ncu);
    const int dep = (int)((g.g_dep >> 16) & 0x7fffu) - 1;
    const double ready = dep >= 0 ? end[dep] : 0.0;
    int best = 0;
    for (int c = 1; c < groups; ++c) {
      const double sb = std::max(free_at[best], ready), sc = std::max(free_at[c], ready);
      if (sc < sb || (sc == sb && free_at[c] > free_at[best])) best = c;
    }
    plan.group[i] = best;
    end[i] = std::max(free_at[best], ready) + dur;
    free_at[best] = end[i];
  }
  for (double f : free_at) plan.makespan = std::max(plan.makespan, f);
  return plan;
}

static int rows_list_plan(wq_gemv_list* l) {
  for (int i = 0; i < l->n; ++i)  // the scales are addressed with 32-bit offsets
    if ((int64_t)l->descs[i].N * (l->descs[i].g_dep & 0xffffu) * 2 >= (1ll << 31))
      return fail(WQ_EUNSUPPORTED, "wq_q4g32_gemv_list_create: linear %d: with more than 16 rows of activations the scales must stay below 2 GiB", i);
  l->batch_rows = true;
  l->batch_u = 2;
  l->threads = kRThreads;
  l->blocks = std::min(cu_count(), 32768);
  const size_t budget = 160 * 1024;
  int nxb = kRMaxXBuf;
  while (nxb > 1 && rows_lds_bytes(l->M, nxb) > budget) --nxb;
  if (rows_lds_bytes(l->M, nxb) > budget)
    return fail(WQ_EUNSUPPORTED, "wq_q4g32_gemv_list_create: %d rows of activations do not fit the LDS", l->M);
  int best_gl = -1;
  BatchGroupPlan best;
  for (int gl = 0; gl <= 6; ++gl) {
    if (l->blocks % (1 << gl) != 0 || (l->blocks >> gl) < 1) break;
    BatchGroupPlan p = rows_assign_groups(l, gl);
    if (best_gl < 0 || p.makespan < best.makespan * 0.98) {
      best_gl = gl;
      best = std::move(p);
    }
  }
  int groups = 1 << best_gl;
  const MaskPlan mp = plan_xcd_masks(l, [&](int i, int ncu) { return rows_linear_cost(l, i, ncu); });
  if (mp.ok && mp.makespan < best.makespan * 0.98) {
    for (int i = 0; i < l->n; ++i) {
      GemvListDesc& g = l->descs[i];
      const int ncu = (l->blocks / 8) * __builtin_popcount(mp.mask[i]);
      const int64_t tiles = ((int64_t)g.N + 15) / 16;  // row tiles
      g.q = (int32_t)(tiles / ncu);
      g.rem = (uint16_t)(tiles % ncu);
      g.off = 0;
      g.gmod_log2 = 0x80;
      g.gidx = mp.mask[i];
    }
    groups = 0;  // (sets of XCDs)
  } else {
    const int ncu = l->blocks >> best_gl;
    std::vector<int64_t> off(groups, 0);
    for (int i = 0; i < l->n; ++i) {
      GemvListDesc& g = l->descs[i];
      const int c = best.group[i];
      const int64_t tiles = ((int64_t)g.N + 15) / 16;  // row tiles
      g.q = (int32_t)(tiles / ncu);
      g.rem = (uint16_t)(tiles % ncu);
      g.off = (uint16_t)off[c];
      off[c] = (off[c] + tiles) % ncu;
      g.gmod_log2 = (uint8_t)best_gl;
      g.gidx = (uint8_t)c;
    }
  }
  l->batch_groups = groups;
  l->batch_nxb = nxb;
  l->batch_ring = 2;
  l->batch_acc_tiles = 0;
  l->batch_chunked = false;
  l->lds = rows_lds_bytes(l->M, nxb);
  const void* kern = reinterpret_cast<const void*>(q4g32_batch_rows_kernel<kRowsTR, 2>);
  static DynamicLdsLimit limit;
  if (limit.ensure(kern, (int)l->lds) != hipSuccess)
    return fail(WQ_EDEVICE, "wq_q4g32_gemv_list_create: hipFuncSetAttribute failed");
  int resident = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, kern, l->threads, l->lds) != hipSuccess || resident < 1)
    return fail(WQ_EDEVICE, "wq_q4g32_gemv_list_create: the workgroup does not fit a CU (%zu bytes of LDS)", l->lds);
  return WQ_OK;
}

int batch_list_plan(wq_gemv_list* l) {
  if (l->M > 16) return rows_list_plan(l);
  const BatchShape s = batch_shape(l->M);
  const int U = s.U;
  const int trows = 16 * s.TW;
  l->batch_u = U;
  l->threads = kBThreads;
  l->blocks = std::min(cu_count(), 32768);
  const size_t budget = 160 * 1024;
  int best_gl = -1;
  BatchGroupPlan best;
  int best_acc = 0;
  bool best_chunked = false;
  for (int gl = 0; gl <= 4; ++gl) {
    if (l->blocks % (1 << gl) != 0 || (l->blocks >> gl) < 1) break;
    const int ncu = l->blocks >> gl;
    int acc_tiles = 0;  // most tiles a workgroup holds of a linear that spans several panels
    for (int i = 0; i < l->n; ++i) {
      const GemvListDesc& g = l->descs[i];
      const int64_t tiles = ((int64_t)g.N + trows - 1) / trows;
      if ((int)(g.g_dep & 0xffffu) > batch_panel_groups(s.U, s.TW)) acc_tiles = std::max<int>(acc_tiles, (int)((tiles + ncu - 1) / ncu));
    }
    // the sums kept between panels must fit beside one panel of activations and a ring of 2: else the tiles of
    // a linear are walked in chunks of what fits, at the price of loading the activations once per chunk
    const size_t base = batch_lds_bytes(s, l->M, 1, 2, 0);
    if (base + 4 * batch_kept_bytes(s.R, s.TW) > budget) continue;
    const int fit = (int)((budget - base) / (size_t)batch_kept_bytes(s.R, s.TW));
    const int chunk = std::min(acc_tiles, fit);
    BatchGroupPlan p = batch_assign_groups(l, gl, s, std::max(chunk, 1));
    if (best_gl < 0 || p.makespan < best.makespan * 0.98) {
      best_gl = gl;
      best = std::move(p);
      best_acc = chunk;
      best_chunked = chunk < acc_tiles;
    }
  }
  if (best_gl < 0)
    return fail(WQ_EUNSUPPORTED, "wq_q4g32_gemv_list_create: %d rows of activations do not fit the LDS", l->M);
  int groups = 1 << best_gl;
  // a short list: sets of XCDs in proportion to the linears' cost (plan_xcd_masks), if the estimate says so
  const size_t mbase = batch_lds_bytes(s, l->M, 1, 2, 0);
  const int mfit = (int)((budget - mbase) / (size_t)batch_kept_bytes(s.R, s.TW));
  const MaskPlan mp = plan_xcd_masks(l, [&](int i, int ncu) { return batch_linear_cost(l, i, ncu, s, std::max(mfit, 1)); });
  if (mp.ok && mp.makespan < best.makespan * 0.98) {
    int acc_tiles = 0;
    for (int i = 0; i < l->n; ++i) {
      GemvListDesc& g = l->descs[i];
      const int ncu = (l->blocks / 8) * __builtin_popcount(mp.mask[i]);
      const int64_t tiles = ((int64_t)g.N + trows - 1) / trows;
      if ((int)(g.g_dep & 0xffffu) > batch_panel_groups(s.U, s.TW)) acc_tiles = std::max<int>(acc_tiles, (int)((tiles + ncu - 1) / ncu));
      g.q = (int32_t)(tiles / ncu);
      g.rem = (uint16_t)(tiles % ncu);
      g.off = 0;
      g.gmod_log2 = 0x80;
      g.gidx = mp.mask[i];
    }
    best_acc = std::min(acc_tiles, mfit);
    best_chunked = best_acc < acc_tiles;
    groups = 0;  // (sets of XCDs)
  } else {
    const int ncu = l->blocks >> best_gl;
    std::vector<int64_t> off(groups, 0);
    for (int i = 0; i < l->n; ++i) {
      GemvListDesc& g = l->descs[i];
      const int c = best.group[i];
      const int64_t tiles = ((int64_t)g.N + trows - 1) / trows;
      g.q = (int32_t)(tiles / ncu);
      g.rem = (uint16_t)(tiles % ncu);
      g.off = (uint16_t)off[c];
      off[c] = (off[c] + tiles) % ncu;
      g.gmod_log2 = (uint8_t)best_gl;
      g.gidx = (uint8_t)c;
    }
  }
  l->batch_groups = groups;
  l->batch_acc_tiles = best_acc;
  l->batch_chunked = best_chunked;
  // a ring of 4 items and up to 2 panels of activations in LDS if they fit, else a ring of 2
  l->batch_ring = 4;
  l->batch_nxb = batch_lds_bytes(s, l->M, 2, 4, best_acc) <= budget ? 2 : batch_lds_bytes(s, l->M, 1, 4, best_acc) <= budget ? 1 : 0;
  if (!l->batch_nxb) {
    l->batch_ring = 2;
    l->batch_nxb = batch_lds_bytes(s, l->M, 2, 2, best_acc) <= budget ? 2 : 1;
  }
  l->lds = batch_lds_bytes(s, l->M, l->batch_nxb, l->batch_ring, best_acc);
  const void* kern = reinterpret_cast<const void*>(batch_kernel(s, best_chunked));
  // several lists share a kernel: the limit only ever grows
  static DynamicLdsLimit limits[2][2];
  if (limits[batch_kernel_index(s)][best_chunked ? 1 : 0].ensure(kern, (int)l->lds) != hipSuccess)
    return fail(WQ_EDEVICE, "wq_q4g32_gemv_list_create: hipFuncSetAttribute failed");
  int resident = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, kern, l->threads, l->lds) != hipSuccess || resident < 1)
    return fail(WQ_EDEVICE, "wq_q4g32_gemv_list_create: the workgroup does not fit a CU (%zu bytes of LDS)", l->lds);
  return WQ_OK;
}

int batch_list_launch(wq_gemv_list* l, hipStream_t stream) {
  const GemvListDesc* table = (const GemvListDesc*)l->table;
  const int use_sync = l->deps > 0 ? 1 : 0;
  if (l->batch_rows) {
    WQ_LAUNCH("wq_q4g32_gemv_list_run", (q4g32_batch_rows_kernel<kRowsTR, 2>), dim3((unsigned)l->blocks), dim3((unsigned)l->threads), l->lds,
              stream, table, l->n, l->sync, l->spin_limit, l->M, l->batch_nxb, use_sync);
    return WQ_OK;
  }
  // chunk: at least 1 (a list without a linear of several panels keeps no sums)
  WQ_LAUNCH("wq_q4g32_gemv_list_run", batch_kernel(batch_shape(l->M), l->batch_chunked), dim3((unsigned)l->blocks), dim3((unsigned)l->threads), l->lds,
            stream, table, l->n, l->sync, l->spin_limit, l->M, l->batch_nxb, l->batch_ring, std::max(l->batch_acc_tiles, 1),
            use_sync);
  return WQ_OK;
}

}  // namespace wq
