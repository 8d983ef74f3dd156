// Stream kernels: one workgroup walks a whole row tile by tile in scan order, carrying the running
// value in a register, with the next tile's loads in flight while the current tile is scanned and
// stored.  No workgroup ever waits for another one, so this is the kernel of choice when there are
// at least about as many rows as the chip has room for workgroups.
//
// The role of linrec_pipe_fwd_kernel / linrec_pipe_bwd_kernel in the reference
// (linrec/impl/cuda/linrec_pipe.cuh:8-143), which also keeps a row inside one block; the tile
// scan, the register double buffer and the addressing differ.
//
// Structure of a row: tiles [0, t_lo) and [t_hi, ntiles) touch a row end and take the predicated
// path without prefetch; the tiles in between are interior for every wave of the workgroup and run
// the pipelined loop, whose body is straight-line code so that the wait before scanning tile t
// leaves the loads of tile t+1 outstanding.
#pragma once
#include <hip/hip_runtime.h>

#include "tile_core.hpp"
#include "tile_kernel.hpp"  // TileArgs

namespace linrec {

template <typename T, int NW, int S, int VEC, int MODE, bool DESC>
__global__ __launch_bounds__(64 * NW) void stream_kernel(TileArgs p) {
  constexpr int WAVE_SLOTS = S * 64;
  constexpr int TILE_SLOTS = NW * WAVE_SLOTS;
  __shared__ float sh_a[2][NW];
  __shared__ float sh_b[2][NW];

  const int lane = threadIdx.x & 63;
  const int wave = NW == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long long row = blockIdx.x;
  const long long row_off = row * p.row_stride;
  const RowView rv = make_row_view<VEC>(p.base_mis, row_off, p.seqlen);
  const RowPtrs<T> q = make_row_ptrs<T, MODE>(p.in0, p.coef, p.aux, p.out0, p.out1, row_off, rv.lo);

  const int ntiles = (rv.nslots + TILE_SLOTS - 1) / TILE_SLOTS;
  // Interior tiles (every slot a full slot, for the whole workgroup) form one contiguous range
  // [t_lo, t_hi): full slots are s in [ceil(lo/VEC), floor(hi/VEC)) in memory order.
  int t_lo, t_hi;
  {
    const int s_f0 = (rv.lo + VEC - 1) / VEC, s_f1 = rv.hi / VEC;
    const int u_f0 = DESC ? rv.nslots - s_f1 : s_f0;  // the same range in scan order
    const int u_f1 = DESC ? rv.nslots - s_f0 : s_f1;
    t_lo = (u_f0 + TILE_SLOTS - 1) / TILE_SLOTS;
    t_hi = u_f1 / TILE_SLOTS;
    if (t_lo > ntiles) t_lo = ntiles;
    if (t_hi < t_lo) t_hi = t_lo;
  }

  float carry = 0.0f;      // value leaving the previous tile
  bool has_carry = false;  // false only before the first tile

#ifdef LINREC_PHASE_TIMING
  // debug builds: per row, 100 MHz wall clock at the start, after tiles 0 / 3 / 5 and at the end,
  // plus the hardware ids of the workgroup's first wave
#define LINREC_ROW_STAMP(i, v) do { if (p.timing && threadIdx.x == 0) p.timing[row * 8 + (i)] = (v); } while (0)
  LINREC_ROW_STAMP(0, wall_clock64());
  LINREC_ROW_STAMP(2, (unsigned long long)__builtin_amdgcn_s_getreg((31 << 11) | 4));   // HW_ID
  LINREC_ROW_STAMP(3, (unsigned long long)__builtin_amdgcn_s_getreg((31 << 11) | 20));  // XCC_ID
#else
#define LINREC_ROW_STAMP(i, v) do { } while (0)
#endif

  // A tile with ragged or missing slots, already in registers (loaded through the predicated path).
  auto edge_finish = [&](int t, const TileData<S, VEC, MODE>& d) {
    const int u_wave = t * TILE_SLOTS + wave * WAVE_SLOTS;
    TileScan<S, VEC> r;
    tile_scan<S, VEC, MODE>(d, r);
    const int par = t & 1;
    if (lane == 0) {
      sh_a[par][wave] = r.total.a;
      sh_b[par][wave] = r.total.b;
    }
    __syncthreads();
    Affine before, total;
    wave_prefixes<NW>(sh_a[par], sh_b[par], wave, lane, before, total);
    bool has_entry = false;
    float entry = 0.0f;
    if (has_carry) {
      has_entry = true;
      entry = wave == 0 ? carry : fmaf(carry, before.a, before.b);
    } else if (wave > 0) {
      has_entry = true;
      entry = before.b;
    }
    tile_apply_store<S, VEC, MODE, DESC, false>(d, r, q, rv, u_wave, lane, has_entry, entry);
    carry = has_carry ? fmaf(carry, total.a, total.b) : total.b;
    has_carry = true;
  };
  // The same, loaded and processed on the spot.
  auto edge_tile = [&](int t) {
    TileData<S, VEC, MODE> d;
    tile_load<S, VEC, MODE, DESC, false>(d, q, rv, t * TILE_SLOTS + wave * WAVE_SLOTS, lane, t == 0 && wave == 0);
    edge_finish(t, d);
  };

  // Scan, exchange, apply and store of an interior tile already in registers.
  auto interior_tile = [&](int t, const TileData<S, VEC, MODE>& d) {
    const int u_wave = t * TILE_SLOTS + wave * WAVE_SLOTS;
    TileScan<S, VEC> r;
    tile_scan<S, VEC, MODE>(d, r);
    const int par = t & 1;
    if (lane == 0) {
      sh_a[par][wave] = r.total.a;
      sh_b[par][wave] = r.total.b;
    }
    __syncthreads();
    Affine before, total;
    wave_prefixes<NW>(sh_a[par], sh_b[par], wave, lane, before, total);
    bool has_entry = false;
    float entry = 0.0f;
    if (has_carry) {
      has_entry = true;
      entry = wave == 0 ? carry : fmaf(carry, before.a, before.b);
    } else if (wave > 0) {
      has_entry = true;
      entry = before.b;
    }
    tile_apply_store<S, VEC, MODE, DESC, true>(d, r, q, rv, u_wave, lane, has_entry, entry);
    carry = has_carry ? fmaf(carry, total.a, total.b) : total.b;
    has_carry = true;
#ifdef LINREC_PHASE_TIMING
    if (t == 0) LINREC_ROW_STAMP(4, wall_clock64());
    if (t == 3) LINREC_ROW_STAMP(5, wall_clock64());
    if (t == 5) LINREC_ROW_STAMP(6, wall_clock64());
#endif
  };

  for (int t = 0; t < t_lo; ++t) edge_tile(t);

  if (t_lo < t_hi) {
    TileData<S, VEC, MODE> cur;
    tile_load<S, VEC, MODE, DESC, true>(cur, q, rv, t_lo * TILE_SLOTS + wave * WAVE_SLOTS, lane,
                                        t_lo == 0 && wave == 0);
    for (int t = t_lo; t + 1 < t_hi; ++t) {
      TileData<S, VEC, MODE> nxt;
      tile_load<S, VEC, MODE, DESC, true>(nxt, q, rv, (t + 1) * TILE_SLOTS + wave * WAVE_SLOTS, lane, false);
      interior_tile(t, cur);
      cur = nxt;
    }
    if (t_hi < ntiles) {
      // a partial tile ends the row: its loads go out before the last interior tile is processed, so
      // that rows of two or three tiles overlap anything at all (3355 x 10000 backward: 186 -> 123 us)
      TileData<S, VEC, MODE> last;
      tile_load<S, VEC, MODE, DESC, false>(last, q, rv, t_hi * TILE_SLOTS + wave * WAVE_SLOTS, lane, false);
      interior_tile(t_hi - 1, cur);
      edge_finish(t_hi, last);
      t_hi = ntiles;  // (at most one partial tile follows the interior ones)
    } else {
      interior_tile(t_hi - 1, cur);
    }
  }

  for (int t = t_hi; t < ntiles; ++t) edge_tile(t);
  LINREC_ROW_STAMP(1, wall_clock64());
#undef LINREC_ROW_STAMP
}

}  // namespace linrec
