// Sweep kernels: teams of M workgroups as in team_kernel.hpp, but a team goes on to further rows
// (team g takes rows g, g + G, g + 2G, ... for G teams), and the launch is shaped so that at any
// moment the G * M workgroups read one contiguous stretch of the tensors: with M equal to the tiles
// of a row, step s of the walk covers rows s*G .. s*G + G - 1 completely.  One workgroup per row
// (stream_kernel.hpp) keeps rows-many reading positions a whole row length apart instead, which
// the memory system serves about a tenth slower.
//
// Restricted to the layouts whose every tile is a full one: 16-byte aligned bases, a row stride
// that keeps every row aligned, and a row length that is a whole number K of tiles with M
// dividing K.  Everything else is served by the stream and team kernels.
//
// The carry between the tiles of a row is the team kernel's: a walker publishes the map of each of
// its tiles, and folds the maps of the up to M-1 tiles between its previous tile of the row and
// this one.  Nobody waits for somebody who is waiting; every wait is bounded all the same.
//
// No counterpart in the reference (linrec/impl/cuda/linrec_pipe.cuh keeps a row in one block).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "team_kernel.hpp"  // gather_maps, TileArgs, descriptors, completion count

namespace linrec {

template <typename T, int NW, int S, int VEC, int MODE, bool DESC>
__global__ __launch_bounds__(64 * NW) void sweep_kernel(TileArgs p) {
  constexpr int WAVE_SLOTS = S * 64;
  constexpr int TILE_SLOTS = NW * WAVE_SLOTS;
  __shared__ float sh_a[2][NW];
  __shared__ float sh_b[2][NW];
  __shared__ float sh_carry[2];

  const int lane = threadIdx.x & 63;
  const int wave = NW == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int M = p.tasks;          // team size, divides K
  const int K = p.tiles_per_row;  // every row is exactly K full tiles
  const long long wg = blockIdx.x;
  const long long teams = p.row_groups;  // the grid is teams * M workgroups
  const long long team = wg / M;
  const int j = int(wg - team * M);
  const int per_row = K / M;  // tiles of one row this walker takes: j, j + M, ...
  const long long my_rows = team < p.numseq ? (p.numseq - team + teams - 1) / teams : 0;
  const long long items = my_rows * per_row;

  uint32_t seq = 0;
  uint32_t leaf_count = 0;
  if (wave == 0) seq = load_seq_through_caches(p.ws);

  // all rows look alike: aligned, seqlen / VEC full slots
  const RowView rv = make_row_view<VEC>(0, 0, p.seqlen);

  struct Item {
    long long row;
    int t;
  };
  auto item_of = [&](long long n) {
    const long long r = n / per_row;
    return Item{team + r * teams, j + int(n - r * per_row) * M};
  };
  auto ptrs_of = [&](long long row) {
    return make_row_ptrs<T, MODE>(p.in0, p.coef, p.aux, p.out0, p.out1, row * p.row_stride, 0);
  };

  float own_out = 0.0f;  // value that left this walker's previous tile of the current row

  auto finish = [&](long long n, const Item& it, const RowPtrs<T>& q, TileData<S, VEC, MODE> d, bool last) {
    const int t = it.t;
    const int u_wave = t * TILE_SLOTS + wave * WAVE_SLOTS;
    if constexpr (MODE == MODE_FWD) {
      // the coefficient of the row's first element in scan order takes no part
      if (t == 0 && wave == 0 && lane == 0) d.cs[0][0] = 0.0f;
    }
    TileScan<S, VEC> r;
    tile_scan<S, VEC, MODE>(d, r);
    const int par = int(n & 1);
    if (lane == 0) {
      sh_a[par][wave] = r.total.a;
      sh_b[par][wave] = r.total.b;
    }
    __syncthreads();
    Affine before, total;
    wave_prefixes<NW>(sh_a[par], sh_b[par], wave, lane, before, total);
    if (wave == 0) {
      uint64_t* desc = p.desc + 2 * (it.row * K);
      if (lane == 0 && t + 1 < K) {
        st_desc(desc + 2 * (long long)t, pack_desc((seq << 2) | STATUS_AGGREGATE, total.a));
        st_desc(desc + 2 * (long long)t + 1, pack_desc((seq << 2) | STATUS_AGGREGATE, total.b));
      }
      const int need = t < M - 1 ? t : M - 1;
      float carry_in = 0.0f;
      if (t > 0) {
        Affine acc = {1.0f, 0.0f};
        bool ok = true;
        if (need > 0) ok = gather_maps(desc, t, need, seq, lane, p.spin_limit, acc);
        if (!ok) {
          // the wait ran out: the value entering the tile from the row's own data instead
          if (lane == 0) __hip_atomic_fetch_add(&p.ws->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          carry_in = recompute_entry<VEC, MODE, DESC>(q, rv, t * TILE_SLOTS, lane);
        } else if (t < M) {
          carry_in = acc.b;  // the maps reach back to the row start
        } else {
          carry_in = need > 0 ? fmaf(own_out, acc.a, acc.b) : own_out;
        }
      }
      own_out = t == 0 ? total.b : fmaf(carry_in, total.a, total.b);
      if (lane == 0) {
        sh_carry[par] = carry_in;
        if (last) leaf_count = signal_tile_done_begin(p, wg);
      }
    }
    __syncthreads();
    const float tile_in = sh_carry[par];
    bool has_entry = false;
    float entry = 0.0f;
    if (t > 0) {
      has_entry = true;
      entry = wave == 0 ? tile_in : fmaf(tile_in, before.a, before.b);
    } else if (wave > 0) {
      has_entry = true;
      entry = before.b;
    }
    tile_apply_store<S, VEC, MODE, DESC, true>(d, r, q, rv, u_wave, lane, has_entry, entry);
  };

  if (items > 0) {
    Item it = item_of(0);
    RowPtrs<T> q = ptrs_of(it.row);
    TileData<S, VEC, MODE> cur;
    tile_load<S, VEC, MODE, DESC, true>(cur, q, rv, it.t * TILE_SLOTS + wave * WAVE_SLOTS, lane, false);
    for (long long n = 0; n + 1 < items; ++n) {
      const Item it2 = item_of(n + 1);
      const RowPtrs<T> q2 = ptrs_of(it2.row);
      TileData<S, VEC, MODE> nxt;
      tile_load<S, VEC, MODE, DESC, true>(nxt, q2, rv, it2.t * TILE_SLOTS + wave * WAVE_SLOTS, lane, false);
      finish(n, it, q, cur, false);
      cur = nxt;
      it = it2;
      q = q2;
    }
    finish(items - 1, it, q, cur, true);
  }

  if (items == 0 && threadIdx.x == 0) leaf_count = signal_tile_done_begin(p, wg);
  if (threadIdx.x == 0) signal_tile_done_end(p, wg, seq, leaf_count);
}

}  // namespace linrec
