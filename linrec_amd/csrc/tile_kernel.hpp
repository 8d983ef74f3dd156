// Tile kernels: rows lie along the unit-stride axis.  A workgroup of NW wavefronts scans one tile
// of NW * S * 64 slots (a slot is VEC consecutive elements, 16 bytes when VEC == 4):
//
//   lane-level   each lane composes the VEC elements of a slot serially,
//   wave-level   64-lane DPP scan of the lane aggregates, one scan per slot row, the S rows of a
//                wave chained through scalar registers,
//   group-level  one aggregate per wave exchanged through LDS,
//   grid-level   (CARRY) tiles of one row chained by decoupled look-back through a descriptor
//                array in global memory: every tile first publishes its own aggregate, then folds
//                its predecessors' aggregates back to the nearest published inclusive value.
//
// Behaviour to match: linrec/impl/cuda/linrec_pipe.cuh:8-143 (forward and fused backward),
// linrec/impl/cuda/linrec_tile.cuh:33-114 (block scan).  The reference never splits a row over
// blocks; the grid-level chain has no counterpart there.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tile_core.hpp"

namespace linrec {

// Look-back workspace: a 16-byte header, a fixed region of completion counters, then two 64-bit
// descriptor words per tile.  Everything but `seq` and `gave_up` is zero between launches.
struct alignas(16) CarryHeader {
  uint32_t seq;      // launch sequence number; descriptor flags of other launches never match
  uint32_t gave_up;  // waits that hit the poll limit (the value was then computed from the row's own data)
  uint32_t pad[2];
};
constexpr uint32_t SEQ_MASK = 0x3fffffffu;
constexpr uint32_t STATUS_AGGREGATE = 1u;  // words hold the tile's own map (a, b)
constexpr uint32_t STATUS_INCLUSIVE = 2u;  // word 1 holds the value carried out of the tile

struct TileArgs {
  const void* in0;    // forward: inputs        backward: d_outputs   (storage type T of the kernel)
  const void* coef;   // coeffs
  const void* aux;    // backward: saved outputs; unused forward
  void* out0;         // forward: outputs       backward: d_inputs
  void* out1;         // backward: d_coeffs
  long long row_stride;
  long long num_tiles;
  int seqlen;
  int tiles_per_row;
  int base_mis;       // common misalignment of all base pointers, elements (0..VEC-1)
  long long numseq;   // rows (chain kernels)
  long long row_groups; // chain kernels: G, the row distance between a workgroup's successive tiles
  int tasks;          // chain kernels: tiles (of different rows) per workgroup
  CarryHeader* ws;
  uint32_t* counters; // completion counters (all zero between launches)
  uint64_t* desc;     // descriptors, two words per tile
  long long ws_tiles; // descriptors the workspace has room for
  int spin_limit;     // polls of one look-back window before a tile gives up
#ifdef LINREC_PHASE_TIMING
  unsigned long long* timing;  // debug builds: 8 timestamps (100 MHz) per tile
#endif
};

// The sequence number of a launch, read through the caches.  The word only changes when the launch's last
// workgroup is done, by which time every workgroup has read it, and a launch starts with the caches written back
// and invalidated, so what it reads is what the launch before it left.  An agent-scope load goes to memory every
// time: thousands of tiles asking for the one address queue up there (512 x 65536 in look-back tiles of 4096
// elements takes 109 us with it and 79 us with this), and a persistent workgroup that waits for it before its
// first loads starts a memory round trip late.
__device__ __forceinline__ uint32_t load_seq_through_caches(const CarryHeader* ws) { return ws->seq; }

__device__ __forceinline__ uint64_t pack_desc(uint32_t flag, float v) {
  return (uint64_t(flag) << 32) | uint64_t(__builtin_bit_cast(uint32_t, v));
}
__device__ __forceinline__ uint64_t ld_desc(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_desc(uint64_t* p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Executed by all 64 lanes of one wave.  Returns the value carried into tile k of its row
// (k >= 1).  `desc` points at the row's first descriptor.  Each 64-bit word carries its own flag,
// so a reader never needs a fence: a word is either from this launch (flag matches) or ignored.
//
// The wait is bounded: after `spin_limit` fruitless polls the tile counts the event in the header and
// reports it (`ok` = false); the caller then computes the value from the row's own data
// (recompute_entry), so neither a wave that never exits nor a wrong result can come of it.
__device__ __forceinline__ float look_back(const uint64_t* desc, int k, uint32_t seq, int lane,
                                           int spin_limit, CarryHeader* hdr, bool& ok) {
  ok = true;
  Affine acc = {1.0f, 0.0f};  // composition of the tiles already folded (nearest ones)
  int pred = k - 1;           // lane 0 inspects `pred`, lane i inspects pred - i
  int polls = 0;
  for (;;) {
    const int idx = pred - lane;
    uint32_t status = STATUS_INCLUSIVE;  // before the row start: nothing is carried in
    float a = 0.0f, b = 0.0f;
    if (idx >= 0) {
      // both words in one round trip; each is valid on its own (it carries its own flag)
      const uint64_t w1 = ld_desc(desc + 2 * (long long)idx + 1);
      const uint64_t w0 = ld_desc(desc + 2 * (long long)idx);
      const uint32_t f1 = uint32_t(w1 >> 32);
      status = ((f1 >> 2) == seq) ? (f1 & 3u) : 0u;
      b = __builtin_bit_cast(float, uint32_t(w1));
      if (status == STATUS_AGGREGATE) {
        const uint32_t f0 = uint32_t(w0 >> 32);
        if (f0 == ((seq << 2) | STATUS_AGGREGATE)) {
          a = __builtin_bit_cast(float, uint32_t(w0));
        } else {
          status = 0u;  // first word not visible yet
        }
      }
    }
    const uint64_t incl_mask = __ballot(status == STATUS_INCLUSIVE);
    const uint64_t wait_mask = __ballot(status == 0u);
    const int first_incl = incl_mask ? __builtin_ctzll(incl_mask) : 64;
    const uint64_t below = first_incl >= 64 ? ~0ull : ((1ull << first_incl) - 1ull);
    if (wait_mask & below) {
      if (++polls > spin_limit) {
        if (lane == 0) __hip_atomic_fetch_add(&hdr->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ok = false;
        return 0.0f;
      }
      __builtin_amdgcn_s_sleep(1);
      continue;  // a needed predecessor has not published yet: poll the same window again
    }
    polls = 0;
    // Fold lanes n..0 (farthest first).  An inclusive value acts as the constant map (0, value).
    const int n = first_incl >= 64 ? 63 : first_incl;
    Affine win = {read_lane(a, n), read_lane(b, n)};
    for (int i = n - 1; i >= 0; --i) win = compose(win, {read_lane(a, i), read_lane(b, i)});
    acc = compose(win, acc);
    if (first_incl < 64) return acc.b;
    pred -= 64;
  }
}

// Completion count of a CARRY launch.  Each tile calls this once, after it has published its
// inclusive value and so will not touch the header or any descriptor again.  The count is kept as
// a tree with fan-in 32 (a single counter would serialise one atomic per tile on one address): the
// last arrival of a group resets the group's counter and moves one level up.  The last arrival at
// the root is the last tile of the launch; it advances `seq`, which invalidates every descriptor
// for the next launch without clearing anything.
//
// The first (leaf) increment is issued early and its result consumed at the end of the kernel, so
// the atomic's round trip overlaps with the tile's stores.
__device__ __forceinline__ uint32_t signal_tile_done_begin(const TileArgs& p, long long tile) {
  if (p.num_tiles <= 1) return 0u;
  return __hip_atomic_fetch_add(&p.counters[tile >> 5], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void signal_tile_done_end(const TileArgs& p, long long tile, uint32_t seq,
                                                     uint32_t leaf_count) {
  uint32_t* level = p.counters;
  long long n = p.num_tiles;
  long long idx = tile;
  uint32_t d = leaf_count;
  bool leaf = true;
  while (n > 1) {
    const long long groups = (n + 31) >> 5;
    const long long g = idx >> 5;
    const long long rest = n - (g << 5);
    const uint32_t group_size = rest < 32 ? uint32_t(rest) : 32u;
    if (!leaf) d = __hip_atomic_fetch_add(&level[g], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    leaf = false;
    if (d + 1u != group_size) return;
    __hip_atomic_store(&level[g], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    level += groups;
    n = groups;
    idx = g;
  }
  const uint32_t next_seq = (seq + 1u) & SEQ_MASK;
  if (next_seq == 0u) {
    // Sequence numbers start over: wipe flags that an equally numbered launch left long ago.
    for (long long i = 0; i < 2 * p.ws_tiles; ++i) st_desc(p.desc + i, 0ull);
  }
  __hip_atomic_store(&p.ws->seq, next_seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T, int NW, int S, int VEC, int MODE, bool DESC, bool CARRY>
__global__ __launch_bounds__(64 * NW) void tile_kernel(TileArgs p) {
  constexpr int WAVE_SLOTS = S * 64;
  constexpr int TILE_SLOTS = NW * WAVE_SLOTS;
  __shared__ float sh_a[NW];
  __shared__ float sh_b[NW];
  __shared__ float sh_carry;

  const int lane = threadIdx.x & 63;
  const int wave = NW == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  // Tiles are numbered row-major in launch order.  A tile only ever waits for tiles with a
  // smaller number; workgroups start in increasing order, so whatever a running tile waits for
  // is itself running or finished (and the wait is bounded in any case, see look_back).
  const long long tile = blockIdx.x;
  const long long row = CARRY ? tile / p.tiles_per_row : tile;
  const int k = CARRY ? int(tile - row * p.tiles_per_row) : 0;
  uint32_t seq = 0;
  uint32_t leaf_count = 0;  // lane 0 of wave 0: result of its completion-count increment
  if constexpr (CARRY) {
    if (wave == 0) seq = load_seq_through_caches(p.ws);
  }

#ifdef LINREC_PHASE_TIMING
#define LINREC_STAMP(i) do { if (p.timing && threadIdx.x == 0) p.timing[tile * 8 + (i)] = wall_clock64(); } while (0)
#else
#define LINREC_STAMP(i) do { } while (0)
#endif
  LINREC_STAMP(0);
  const long long row_off = row * p.row_stride;
  const RowView rv = make_row_view<VEC>(p.base_mis, row_off, p.seqlen);
  const RowPtrs<T> q = make_row_ptrs<T, MODE>(p.in0, p.coef, p.aux, p.out0, p.out1, row_off, rv.lo);

  const int u_wave = k * TILE_SLOTS + wave * WAVE_SLOTS;  // first scan-order slot of this wave
  const bool interior = slots_interior<VEC, DESC>(u_wave, WAVE_SLOTS, rv);  // wave-uniform
  const bool row_start = k == 0 && wave == 0;

  TileData<S, VEC, MODE> d;
  if (interior) {
    tile_load<S, VEC, MODE, DESC, true>(d, q, rv, u_wave, lane, row_start);
  } else {
    tile_load<S, VEC, MODE, DESC, false>(d, q, rv, u_wave, lane, row_start);
  }
  TileScan<S, VEC> r;
  tile_scan<S, VEC, MODE>(d, r);
  LINREC_STAMP(1);

  // Group-level: exchange wave aggregates; grid-level: look-back.
  bool has_entry = false;  // a value enters this wave (wave-uniform)
  float entry = 0.0f;
  if constexpr (NW > 1 || CARRY) {
    if (lane == 0) {
      sh_a[wave] = r.total.a;
      sh_b[wave] = r.total.b;
    }
    __syncthreads();
    LINREC_STAMP(2);
    Affine before, total;  // the waves in front of this one, and all of them
    wave_prefixes<NW>(sh_a, sh_b, wave, lane, before, total);
    float tile_in = 0.0f;
    if constexpr (CARRY) {
      uint64_t* desc = p.desc + 2 * (row * p.tiles_per_row);
      if (wave == 0) {
        float carry_in = 0.0f;
        if (k == 0) {
          if (lane == 0) st_desc(desc + 1, pack_desc((seq << 2) | STATUS_INCLUSIVE, total.b));
        } else {
          if (lane == 0) {
            st_desc(desc + 2 * k, pack_desc((seq << 2) | STATUS_AGGREGATE, total.a));
            st_desc(desc + 2 * k + 1, pack_desc((seq << 2) | STATUS_AGGREGATE, total.b));
          }
          LINREC_STAMP(3);
          bool ok;
          carry_in = look_back(desc, k, seq, lane, p.spin_limit, p.ws, ok);
          if (!ok) carry_in = recompute_entry<VEC, MODE, DESC>(q, rv, k * TILE_SLOTS, lane);
          LINREC_STAMP(4);
          if (lane == 0)
            st_desc(desc + 2 * k + 1,
                    pack_desc((seq << 2) | STATUS_INCLUSIVE, fmaf(carry_in, total.a, total.b)));
        }
        if (lane == 0) {
          sh_carry = carry_in;
          leaf_count = signal_tile_done_begin(p, tile);
        }
      }
      __syncthreads();
      LINREC_STAMP(5);
      tile_in = sh_carry;
    }
    if (CARRY && k > 0) {
      has_entry = true;
      entry = wave == 0 ? tile_in : fmaf(tile_in, before.a, before.b);
    } else if (wave > 0) {
      has_entry = true;
      entry = before.b;
    }
  }

  if (interior) {
    tile_apply_store<S, VEC, MODE, DESC, true>(d, r, q, rv, u_wave, lane, has_entry, entry);
  } else {
    tile_apply_store<S, VEC, MODE, DESC, false>(d, r, q, rv, u_wave, lane, has_entry, entry);
  }

  LINREC_STAMP(6);
  if constexpr (CARRY) {
    if (threadIdx.x == 0) signal_tile_done_end(p, tile, seq, leaf_count);
  }
  LINREC_STAMP(7);
}

}  // namespace linrec
