// Chain kernels: long rows split into tiles that are chained by decoupled look-back (as in the
// CARRY tile kernels), with each workgroup working through several tiles that belong to
// DIFFERENT rows: workgroup (g, k) scans tile k of rows g, g + G, g + 2G, ...  While it waits for
// the predecessors of its current tile to publish, the loads of its next tile are already in
// flight, so the wait costs no memory bandwidth.
//
// Why different rows: a workgroup may only ever wait for workgroups that were started before it
// (workgroups start in increasing order; a later one may not be resident yet).  Tile k of any row
// depends on tiles 0..k-1 of that row, which belong to workgroups (g, 0..k-1): smaller numbers,
// for every row the workgroup visits.  Successive tiles of ONE row, by contrast, could not be
// pipelined inside one workgroup without serialising the row.
//
// No counterpart in the reference, which never splits a row (linrec/impl/cuda/linrec_pipe.cuh:14-22).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tile_core.hpp"
#include "tile_kernel.hpp"  // TileArgs, descriptors, look_back, completion count

namespace linrec {

template <typename T, int NW, int S, int VEC, int MODE, bool DESC>
__global__ __launch_bounds__(64 * NW) void chain_kernel(TileArgs p) {
  constexpr int WAVE_SLOTS = S * 64;
  constexpr int TILE_SLOTS = NW * WAVE_SLOTS;
  __shared__ float sh_a[NW];
  __shared__ float sh_b[NW];
  __shared__ float sh_carry;

  const int lane = threadIdx.x & 63;
  const int wave = NW == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long long wg = blockIdx.x;
  const long long group = wg / p.tiles_per_row;  // g
  const int k = int(wg - group * p.tiles_per_row);
  // rows g, g + G, ... below numseq
  const long long G = p.row_groups;
  const int ntasks = int((p.numseq - group + G - 1) / G) < p.tasks ? int((p.numseq - group + G - 1) / G) : p.tasks;

  uint32_t seq = 0;
  uint32_t leaf_count = 0;
  if (wave == 0) seq = load_seq_through_caches(p.ws);

  const int u_wave = k * TILE_SLOTS + wave * WAVE_SLOTS;
  const bool row_start = k == 0 && wave == 0;

  struct Task {
    RowView rv;
    RowPtrs<T> q;
    long long row;
    bool interior;
  };
  auto make_task = [&](int i) {
    Task t;
    t.row = group + (long long)i * G;
    const long long row_off = t.row * p.row_stride;
    t.rv = make_row_view<VEC>(p.base_mis, row_off, p.seqlen);
    t.q = make_row_ptrs<T, MODE>(p.in0, p.coef, p.aux, p.out0, p.out1, row_off, t.rv.lo);
    t.interior = slots_interior<VEC, DESC>(u_wave, WAVE_SLOTS, t.rv);
    return t;
  };
  auto load_task = [&](const Task& t, TileData<S, VEC, MODE>& d) {
    if (t.interior) {
      tile_load<S, VEC, MODE, DESC, true>(d, t.q, t.rv, u_wave, lane, row_start);
    } else {
      tile_load<S, VEC, MODE, DESC, false>(d, t.q, t.rv, u_wave, lane, row_start);
    }
  };
  // Everything after the loads of one tile: scan, exchange, look-back, apply, store.
  auto finish_task = [&](const Task& t, const TileData<S, VEC, MODE>& d, bool last) {
    TileScan<S, VEC> r;
    tile_scan<S, VEC, MODE>(d, r);
    if (lane == 0) {
      sh_a[wave] = r.total.a;
      sh_b[wave] = r.total.b;
    }
    __syncthreads();
    Affine before, total;
    wave_prefixes<NW>(sh_a, sh_b, wave, lane, before, total);
    if (wave == 0) {
      uint64_t* desc = p.desc + 2 * (t.row * p.tiles_per_row);
      float carry_in = 0.0f;
      if (k == 0) {
        if (lane == 0) st_desc(desc + 1, pack_desc((seq << 2) | STATUS_INCLUSIVE, total.b));
      } else {
        if (lane == 0) {
          st_desc(desc + 2 * k, pack_desc((seq << 2) | STATUS_AGGREGATE, total.a));
          st_desc(desc + 2 * k + 1, pack_desc((seq << 2) | STATUS_AGGREGATE, total.b));
        }
        bool ok;
        carry_in = look_back(desc, k, seq, lane, p.spin_limit, p.ws, ok);
        if (!ok) carry_in = recompute_entry<VEC, MODE, DESC>(t.q, t.rv, k * TILE_SLOTS, lane);
        if (lane == 0)
          st_desc(desc + 2 * k + 1, pack_desc((seq << 2) | STATUS_INCLUSIVE, fmaf(carry_in, total.a, total.b)));
      }
      if (lane == 0) {
        sh_carry = carry_in;
        if (last) leaf_count = signal_tile_done_begin(p, wg);
      }
    }
    __syncthreads();
    const float tile_in = sh_carry;
    bool has_entry = false;
    float entry = 0.0f;
    if (k > 0) {
      has_entry = true;
      entry = wave == 0 ? tile_in : fmaf(tile_in, before.a, before.b);
    } else if (wave > 0) {
      has_entry = true;
      entry = before.b;
    }
    if (t.interior) {
      tile_apply_store<S, VEC, MODE, DESC, true>(d, r, t.q, t.rv, u_wave, lane, has_entry, entry);
    } else {
      tile_apply_store<S, VEC, MODE, DESC, false>(d, r, t.q, t.rv, u_wave, lane, has_entry, entry);
    }
  };

  Task cur_t = make_task(0);
  TileData<S, VEC, MODE> cur;
  load_task(cur_t, cur);
  for (int i = 0; i + 1 < ntasks; ++i) {
    const Task nxt_t = make_task(i + 1);
    TileData<S, VEC, MODE> nxt;
    load_task(nxt_t, nxt);  // in flight while this tile waits for its predecessors
    finish_task(cur_t, cur, false);
    cur_t = nxt_t;
    cur = nxt;
  }
  finish_task(cur_t, cur, true);

  if (threadIdx.x == 0) signal_tile_done_end(p, wg, seq, leaf_count);
}

}  // namespace linrec
