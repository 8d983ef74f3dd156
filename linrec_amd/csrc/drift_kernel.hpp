// Drift kernels: the sweep kernels' launch shape (teams of M workgroups, one tile of a row each, that go
// on from row to row so that the whole launch reads one contiguous stretch of the tensors at any moment)
// with the exchange between team mates taken off the critical path: a tile that has been scanned is kept
// in registers and stored TWO steps later, while the next tiles are being scanned; by then the value that
// enters it has arrived without anybody having waited for it.
//
// Why the launch shape matters: the memory system spreads addresses over channels and banks by hashing
// address bits up to about bit 22.  One workgroup per row (stream_kernel.hpp) keeps rows-many reading
// positions a row length apart, all at the same offset inside their rows, so the bits that number the
// tile inside the row are the same for every access in flight: measured with a memory-only kernel, 2
// streams in and 1 out run at 5.5 TB/s with bits 15-17 constant among the accesses in flight against
// 6.5-6.6 TB/s for a dense window.  A dense window needs several tiles of one row in flight at once, hence
// workgroups that share rows, hence an exchange; what a sweep kernel loses by waiting for it in every
// step, these kernels keep.
//
// Restrictions as for the sweep kernels: 16-byte aligned bases, a row stride that keeps every row
// aligned, rows of a whole number K of tiles with M dividing K.  Every workgroup of the launch has to
// be resident at once (the planner sees to that); every wait is bounded all the same, and a wave whose
// wait runs out computes the value it needs from the row's own data.
//
// No counterpart in the reference (linrec/impl/cuda/linrec_pipe.cuh keeps a row in one block).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "team_kernel.hpp"  // gather_maps, TileArgs, descriptors, completion count

namespace linrec {

// The walk.  Wave 0 publishes the map of tile n after the barrier of step n and, at the top of step n, asks
// for the maps that enter tile n-2 (published by the team mates a whole step ago, so they are there),
// ahead of its own loads; the words arrive while tile n is scanned, and the value entering tile n-2 is in
// LDS by the barrier of step n.  Nothing waits for a round trip to another workgroup.
//
// The loop is unrolled three steps deep so that the three tiles in the works (being scanned, and stored
// one and two steps from now) and the tiles of loaded data change roles without a register being copied.
// PF: tiles of loads in flight ahead of the scan (1 or 2); WPE: waves per SIMD the compiler is to allow for.
template <typename T, int NW, int S, int VEC, int MODE, bool DESC, int PF, int WPE = 1>
__global__ __launch_bounds__(64 * NW, WPE) void drift_kernel(TileArgs p) {
  static_assert(PF == 1 || PF == 2, "one or two tiles of loads ahead of the scan");
  constexpr int WAVE_SLOTS = S * 64;
  constexpr int TILE_SLOTS = NW * WAVE_SLOTS;
  __shared__ float sh_a[2][NW];
  __shared__ float sh_b[2][NW];
  __shared__ float sh_carry[4];  // steps alternate between [0] and [1]; [2] and [3] are the last two tiles'

  const int lane = threadIdx.x & 63;
  const int wave = NW == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int M = p.tasks;          // team size, divides K
  const int K = p.tiles_per_row;  // every row is exactly K full tiles
  const int teams = int(p.row_groups);  // the grid is teams * M workgroups
  const int team = int(blockIdx.x) / M;
  const int j = int(blockIdx.x) - team * M;
  const int per_row = K / M;  // tiles of one row this walker takes: j, j + M, ...
  const long long my_rows = team < p.numseq ? (p.numseq - team + teams - 1) / teams : 0;
  const int items = int(my_rows * per_row);

  uint32_t seq = 0;
  if (wave == 0) seq = __hip_atomic_load(&p.ws->seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const RowView rv = make_row_view<VEC>(0, 0, p.seqlen);

  struct Item {
    int row;
    int t;
  };
  // the walk: tiles j, j + M, ... of row `team`, then of row team + teams, ...
  Item cursor = {team, j};
  auto next_item = [&]() {
    const Item it = cursor;
    cursor.t += M;
    if (cursor.t >= K) {
      cursor.t = j;
      cursor.row += teams;
    }
    return it;
  };
  auto ptrs_of = [&](int row) {
    return make_row_ptrs<T, MODE>(p.in0, p.coef, p.aux, p.out0, p.out1, (long long)row * p.row_stride, 0);
  };

  // A tile that has been scanned and not stored yet.
  struct Pending {
    TileData<S, VEC, MODE> d;  // (what the store still needs of it: the saved outputs, backward)
    TileScan<S, VEC> r;
    Affine before;  // the waves in front of this one
    Affine total;   // wave 0: the whole tile's map
    Item it;
  };
  TileData<S, VEC, MODE> D[3];  // tile n lies in D[n % 3]
  Item DI[3];
  Pending P[3];                 // and becomes P[n % 3]

  float own_out = 0.0f;  // wave 0: value that left this walker's previous tile of the current row

  // wave 0: the words of the maps in front of tile `it` (lane i: tile t-1-i), asked for ahead of time
  auto ask = [&](const Item& it, uint64_t& w0, uint64_t& w1) {
    const int t = it.t;
    const int need = t < M - 1 ? t : M - 1;
    w0 = 0;
    w1 = 0;
    if (lane < need) {
      const uint64_t* desc = p.desc + 2 * ((long long)it.row * K);
      const long long idx = t - 1 - lane;
      w0 = ld_desc(desc + 2 * idx);
      w1 = ld_desc(desc + 2 * idx + 1);
    }
  };
  // wave 0: the value entering pending tile `q`, from the words asked for (or by polling, or, when that
  // runs out, from the row's own data)
  auto resolve = [&](const Pending& q, uint64_t w0, uint64_t w1) -> float {
    const int t = q.it.t;
    const int need = t < M - 1 ? t : M - 1;
    float carry_in = 0.0f;
    if (t > 0) {
      Affine acc = {1.0f, 0.0f};
      bool ok = true;
      if (need > 0) {
        const uint32_t want = (seq << 2) | STATUS_AGGREGATE;
        const bool mine = lane >= need || (uint32_t(w0 >> 32) == want && uint32_t(w1 >> 32) == want);
        if (__ballot(!mine) == 0) {
          // lane i holds the map of tile t-1-i: fold them oldest first, towards lane 0
          float a[1] = {lane < need ? __builtin_bit_cast(float, uint32_t(w0)) : 1.0f};
          float b[1] = {lane < need ? __builtin_bit_cast(float, uint32_t(w1)) : 0.0f};
          // (inside each row of 16 lanes by DPP, which leaves a row's composition in its lane 0; then the
          // up to four rows, the highest lanes first)
          scan_step<DPP_ROW_SHL1, 0xf>(a, b);
          scan_step<DPP_ROW_SHL2, 0xf>(a, b);
          scan_step<DPP_ROW_SHL4, 0xf>(a, b);
          scan_step<DPP_ROW_SHL8, 0xf>(a, b);
          acc = {read_lane(a[0], 0), read_lane(b[0], 0)};
          if (need > 16) {
            Affine far = {read_lane(a[0], 16), read_lane(b[0], 16)};
            if (need > 32) far = compose({read_lane(a[0], 32), read_lane(b[0], 32)}, far);
            if (need > 48) far = compose({read_lane(a[0], 48), read_lane(b[0], 48)}, far);
            acc = compose(far, acc);
          }
        } else {
          ok = gather_maps(p.desc + 2 * ((long long)q.it.row * K), t, need, seq, lane, p.spin_limit, acc);
        }
      }
      if (!ok) {
        if (lane == 0) __hip_atomic_fetch_add(&p.ws->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        carry_in = recompute_entry<VEC, MODE, DESC>(ptrs_of(q.it.row), rv, t * TILE_SLOTS, lane);
      } else if (t < M) {
        carry_in = acc.b;  // the maps reach back to the row start
      } else {
        carry_in = need > 0 ? fmaf(own_out, acc.a, acc.b) : own_out;
      }
    }
    own_out = t == 0 ? q.total.b : fmaf(carry_in, q.total.a, q.total.b);
    return carry_in;
  };
  auto store_pending = [&](const Pending& q, float tile_in) {
    const int t = q.it.t;
    bool has_entry = false;
    float entry = 0.0f;
    if (t > 0) {
      has_entry = true;
      entry = wave == 0 ? tile_in : fmaf(tile_in, q.before.a, q.before.b);
    } else if (wave > 0) {
      has_entry = true;
      entry = q.before.b;
    }
    tile_apply_store<S, VEC, MODE, DESC, true>(q.d, q.r, ptrs_of(q.it.row), rv, t * TILE_SLOTS + wave * WAVE_SLOTS, lane,
                                               has_entry, entry);
  };
  auto load_next = [&](TileData<S, VEC, MODE>& d, Item& it) {
    it = next_item();
    tile_load<S, VEC, MODE, DESC, true>(d, ptrs_of(it.row), rv, it.t * TILE_SLOTS + wave * WAVE_SLOTS, lane, false);
  };

  // Step n, n % 3 == PH: tile n lies in D[PH]; P[(PH + 1) % 3] is tile n-2, stored in this step.
  auto step = [&]<int PH>(std::integral_constant<int, PH>, int n, bool prefetch) {
    constexpr int OLD = (PH + 1) % 3, LD = (PH + PF) % 3;
    __builtin_amdgcn_sched_barrier(0);  // (nothing of this step moves up into the one before)
    uint64_t w0 = 0, w1 = 0;
    if (wave == 0 && n >= 2) ask(P[OLD].it, w0, w1);
    __builtin_amdgcn_sched_barrier(0);
    if (prefetch) load_next(D[LD], DI[LD]);
    TileData<S, VEC, MODE>& d = D[PH];
    const Item it = DI[PH];
    if constexpr (MODE == MODE_FWD) {
      if (it.t == 0 && wave == 0 && lane == 0) d.cs[0][0] = 0.0f;  // the row's first coefficient takes no part
    }
    Pending& now = P[PH];
    tile_scan<S, VEC, MODE>(d, now.r);
    const int par = n & 1;
    if (lane == 0) {
      sh_a[par][wave] = now.r.total.a;
      sh_b[par][wave] = now.r.total.b;
    }
    if (wave == 0 && n >= 2) {
      const float cin = resolve(P[OLD], w0, w1);
      if (lane == 0) sh_carry[par] = cin;
    }
    __syncthreads();
    wave_prefixes<NW>(sh_a[par], sh_b[par], wave, lane, now.before, now.total);
    if (wave == 0) {
      if (lane == 0 && it.t + 1 < K) {
        uint64_t* desc = p.desc + 2 * ((long long)it.row * K);
        st_desc(desc + 2 * (long long)it.t, pack_desc((seq << 2) | STATUS_AGGREGATE, now.total.a));
        st_desc(desc + 2 * (long long)it.t + 1, pack_desc((seq << 2) | STATUS_AGGREGATE, now.total.b));
      }
    }
    if (n >= 2) store_pending(P[OLD], sh_carry[par]);
    if constexpr (MODE == MODE_BWD) now.d = d;
    now.it = it;
  };
  // The last tile lies in P[A] and the one before it in P[(A + 2) % 3]: nothing left to overlap with, so
  // both are asked for at once, and one barrier serves both.
  auto finish = [&]<int A>(std::integral_constant<int, A>) {
    constexpr int PREV = (A + 2) % 3;
    if (wave == 0) {
      uint64_t w0 = 0, w1 = 0, v0 = 0, v1 = 0;
      if (items >= 2) ask(P[PREV].it, w0, w1);
      ask(P[A].it, v0, v1);  // (published moments ago: if the words are not there yet, resolve polls for them)
      if (items >= 2) {
        const float cin = resolve(P[PREV], w0, w1);
        if (lane == 0) sh_carry[2] = cin;
      }
      const float cin = resolve(P[A], v0, v1);
      if (lane == 0) sh_carry[3] = cin;
    }
    __syncthreads();
    if (items >= 2) store_pending(P[PREV], sh_carry[2]);
    store_pending(P[A], sh_carry[3]);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;

  if (items > 0) {
    load_next(D[0], DI[0]);
    if (PF == 2 && items > 1) load_next(D[1], DI[1]);
    int n = 0;
    // every step of this loop has a tile to load ahead
    while (n + PF + 2 < items) {
      step(I0{}, n, true);
      step(I1{}, n + 1, true);
      step(I2{}, n + 2, true);
      n += 3;
    }
    // at most PF + 2 steps are left, the first at n % 3 == 0
    if (n < items) { step(I0{}, n, n + PF < items); ++n; }
    if (n < items) { step(I1{}, n, n + PF < items); ++n; }
    if (n < items) { step(I2{}, n, n + PF < items); ++n; }
    if (n < items) { step(I0{}, n, false); ++n; }
    switch ((items - 1) % 3) {
      case 0: finish(I0{}); break;
      case 1: finish(I1{}); break;
      default: finish(I2{}); break;
    }
  }

  if (threadIdx.x == 0) {
    const uint32_t leaf_count = signal_tile_done_begin(p, blockIdx.x);
    signal_tile_done_end(p, blockIdx.x, seq, leaf_count);
  }
}

}  // namespace linrec
