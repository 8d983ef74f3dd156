// Team kernels: M workgroups share one row.  Workgroup j of the team walks tiles j, j+M, j+2M, ...
// of the row in scan order with the next of its tiles prefetched, exactly like a stream kernel, and
// the M walkers advance side by side, so M consecutive tiles of the row are in flight at any time.
//
// Carry: a tile needs the value leaving tile t-1.  The walker already knows the value that left its
// own previous tile t-M (a register); the M-1 tiles in between belong to its team mates, each of
// which publishes the tile's own map (a, b) in a descriptor as soon as the tile is scanned.  So
//   carry_in(t) = carry_out(t-M) . map(t-M+1) . ... . map(t-1)
// needs only maps, never a team mate's running value: nobody waits for somebody who is waiting.
// M = 1 degenerates to the stream kernel, M = tiles per row to one tile per workgroup.
//
// Liveness: a walker waits only for maps of smaller tiles, each published by a team mate right
// after a local scan.  Team mates have consecutive workgroup numbers and start together; the one
// team that may be split by the residency limit gets its missing members as soon as any other,
// complete team retires.  Every wait is bounded all the same (see look_back in tile_kernel.hpp).
//
// No counterpart in the reference (linrec/impl/cuda/linrec_pipe.cuh keeps a row in one block).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "tile_core.hpp"
#include "tile_kernel.hpp"  // TileArgs, descriptors, completion count

namespace linrec {

// All 64 lanes of one wave.  Folds the maps of tiles t-need .. t-1 (need <= 63), oldest first.
// Returns false after `spin_limit` fruitless polls.
__device__ __forceinline__ bool gather_maps(const uint64_t* desc, int t, int need, uint32_t seq, int lane,
                                            int spin_limit, Affine& acc) {
  float a = 1.0f, b = 0.0f;
  for (int polls = 0;; ++polls) {
    bool ok = true;
    if (lane < need) {
      const long long idx = t - 1 - lane;
      const uint64_t w0 = ld_desc(desc + 2 * idx);
      const uint64_t w1 = ld_desc(desc + 2 * idx + 1);
      const uint32_t want = (seq << 2) | STATUS_AGGREGATE;
      ok = uint32_t(w0 >> 32) == want && uint32_t(w1 >> 32) == want;
      a = __builtin_bit_cast(float, uint32_t(w0));
      b = __builtin_bit_cast(float, uint32_t(w1));
    }
    if (__ballot(!ok) == 0) break;
    if (polls >= spin_limit) return false;
    __builtin_amdgcn_s_sleep(1);
  }
  acc = {read_lane(a, need - 1), read_lane(b, need - 1)};
  for (int i = need - 2; i >= 0; --i) acc = compose(acc, {read_lane(a, i), read_lane(b, i)});
  return true;
}

template <typename T, int NW, int S, int VEC, int MODE, bool DESC>
__global__ __launch_bounds__(64 * NW) void team_kernel(TileArgs p) {
  constexpr int WAVE_SLOTS = S * 64;
  constexpr int TILE_SLOTS = NW * WAVE_SLOTS;
  __shared__ float sh_a[2][NW];
  __shared__ float sh_b[2][NW];
  __shared__ float sh_carry[2];

  const int lane = threadIdx.x & 63;
  const int wave = NW == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int M = p.tasks;            // team size
  const int K = p.tiles_per_row;    // tiles every row is cut into (host-side upper bound)
  const long long wg = blockIdx.x;
  const long long row = wg / M;
  const int j = int(wg - row * M);
  const int n_own = j < K ? (K - j + M - 1) / M : 0;

  uint32_t seq = 0;
  uint32_t leaf_count = 0;
  if (wave == 0) seq = load_seq_through_caches(p.ws);

  const long long row_off = row * p.row_stride;
  const RowView rv = make_row_view<VEC>(p.base_mis, row_off, p.seqlen);
  const RowPtrs<T> q = make_row_ptrs<T, MODE>(p.in0, p.coef, p.aux, p.out0, p.out1, row_off, rv.lo);
  uint64_t* desc = p.desc + 2 * (row * K);

  // Tiles [t_lo, t_hi) of the row are interior (every slot full) for the whole workgroup; among
  // this walker's tiles j + i*M those are i in [i_lo, i_hi).
  int i_lo, i_hi;
  {
    const int s_f0 = (rv.lo + VEC - 1) / VEC, s_f1 = rv.hi / VEC;
    const int u_f0 = DESC ? rv.nslots - s_f1 : s_f0;
    const int u_f1 = DESC ? rv.nslots - s_f0 : s_f1;
    const int t_lo = (u_f0 + TILE_SLOTS - 1) / TILE_SLOTS;
    const int t_hi = u_f1 / TILE_SLOTS;
    i_lo = t_lo <= j ? 0 : (t_lo - j + M - 1) / M;
    i_hi = t_hi <= j ? 0 : (t_hi - j + M - 1) / M;
    if (i_lo > n_own) i_lo = n_own;
    if (i_hi > n_own) i_hi = n_own;
    if (i_hi < i_lo) i_hi = i_lo;
  }

  float own_out = 0.0f;  // value that left this walker's previous tile

  // Everything after the loads of tile t: scan, exchange inside the workgroup and the team, apply, store.
  auto finish = [&](int t, const TileData<S, VEC, MODE>& d, auto interior_tag, bool last) {
    constexpr bool INTERIOR = decltype(interior_tag)::value;
    const int u_wave = t * TILE_SLOTS + wave * WAVE_SLOTS;
    TileScan<S, VEC> r;
    tile_scan<S, VEC, MODE>(d, r);
    const int par = (t / M) & 1;
    if (lane == 0) {
      sh_a[par][wave] = r.total.a;
      sh_b[par][wave] = r.total.b;
    }
    __syncthreads();
    Affine before, total;
    wave_prefixes<NW>(sh_a[par], sh_b[par], wave, lane, before, total);
    if (wave == 0) {
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
    tile_apply_store<S, VEC, MODE, DESC, INTERIOR>(d, r, q, rv, u_wave, lane, has_entry, entry);
  };
  using True = std::integral_constant<bool, true>;
  using False = std::integral_constant<bool, false>;

  auto edge_tile = [&](int i) {
    const int t = j + i * M;
    TileData<S, VEC, MODE> d;
    tile_load<S, VEC, MODE, DESC, false>(d, q, rv, t * TILE_SLOTS + wave * WAVE_SLOTS, lane, t == 0 && wave == 0);
    finish(t, d, False{}, i + 1 == n_own);
  };

  for (int i = 0; i < i_lo; ++i) edge_tile(i);
  if (i_lo < i_hi) {
    TileData<S, VEC, MODE> cur;
    {
      const int t = j + i_lo * M;
      tile_load<S, VEC, MODE, DESC, true>(cur, q, rv, t * TILE_SLOTS + wave * WAVE_SLOTS, lane, t == 0 && wave == 0);
    }
    for (int i = i_lo; i + 1 < i_hi; ++i) {
      TileData<S, VEC, MODE> nxt;
      tile_load<S, VEC, MODE, DESC, true>(nxt, q, rv, (j + (i + 1) * M) * TILE_SLOTS + wave * WAVE_SLOTS, lane, false);
      finish(j + i * M, cur, True{}, false);
      cur = nxt;
    }
    finish(j + (i_hi - 1) * M, cur, True{}, i_hi == n_own);
  }
  for (int i = i_hi; i < n_own; ++i) edge_tile(i);

  if (n_own == 0 && threadIdx.x == 0) leaf_count = signal_tile_done_begin(p, wg);
  if (threadIdx.x == 0) signal_tile_done_end(p, wg, seq, leaf_count);
}

}  // namespace linrec
