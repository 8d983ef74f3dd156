// Building blocks shared by the tile kernels (one tile per workgroup, optional look-back chain) and
// the stream kernels (one workgroup walks a whole row tile by tile): loading a wave's share of a
// tile into registers, the lane- and wave-level scan, and applying the entry value and storing.
//
// A tile is NW * S * 64 slots; wave w owns the S*64 consecutive slots starting at
// u_wave = tile_index * TILE_SLOTS + w * S * 64 (scan order), lane t the slots u_wave + j*64 + t,
// j = 0..S-1, so that every access of a wave covers 64 consecutive 16-byte slots.
//
// Backward uses the "multiply after" form of the gradient recurrence so that the coefficients
// need no shifted load: with w the value handed from one element to the next in scan order,
//   dx[l] = w + dy[l];   w <- dx[l] * c[l]
// which is dx[l] = dx[l+-1] * c[l+-1] + dy[l] (linrec/impl/cuda/linrec_ref.cuh:83-87) with the
// product moved to the producing side.  d_coeffs[l] = dx[l] * y[next position in this scan's
// order], 0 past the row end (linrec_ref.cuh:90-93).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "memio.hpp"
#include "scan_primitives.hpp"

// Interior accesses either use a wave-uniform base in SGPRs plus a 32-bit lane offset, or a full
// 64-bit per-lane address.  Both are kept selectable for measurements.
#ifndef LINREC_SADDR_LOAD
#define LINREC_SADDR_LOAD 1
#endif
#ifndef LINREC_LOAD_ORDER
#define LINREC_LOAD_ORDER 2  // 0: compiler's order, 1: x, c (, y) slot row by slot row, 2: all x, all c (, all y)
#endif
#ifndef LINREC_STORE_ORDER
#define LINREC_STORE_ORDER 0  // 0: forward stores each slot row as computed, backward in two batches; 1: always batches; 2: never
#endif
#ifndef LINREC_SADDR_STORE
#define LINREC_SADDR_STORE 1
#endif

namespace linrec {

constexpr int MODE_FWD = 0;
constexpr int MODE_BWD = 1;

// Aligned-row pointers of the tensors of one row (see memio.hpp for the coordinates).
template <typename T>
struct RowPtrs {
  const T* __restrict__ in0;   // forward: inputs        backward: d_outputs
  const T* __restrict__ coef;  // coeffs
  const T* __restrict__ aux;   // backward: saved outputs
  T* __restrict__ out0;        // forward: outputs       backward: d_inputs
  T* __restrict__ out1;        // backward: d_coeffs
};

// The five row pointers of row `row_off` from the untyped kernel arguments.
template <typename T, int MODE_>
__device__ __forceinline__ RowPtrs<T> make_row_ptrs(const void* in0, const void* coef, const void* aux, void* out0,
                                                    void* out1, long long row_off, int lo) {
  const long long o = row_off - lo;
  return RowPtrs<T>{static_cast<const T*>(in0) + o, static_cast<const T*>(coef) + o,
                    MODE_ == 1 ? static_cast<const T*>(aux) + o : nullptr, static_cast<T*>(out0) + o,
                    MODE_ == 1 ? static_cast<T*>(out1) + o : nullptr};
}

template <int VEC>
__device__ __forceinline__ RowView make_row_view(int base_mis, long long row_off, int seqlen) {
  RowView rv;
  rv.lo = VEC == 1 ? 0 : int((base_mis + row_off) & (VEC - 1));
  rv.hi = rv.lo + seqlen;
  rv.nslots = (rv.hi + VEC - 1) / VEC;
  return rv;
}

// All slots u_first .. u_first + count - 1 (scan order) lie fully inside the row.
template <int VEC, bool DESC>
__device__ __forceinline__ bool slots_interior(int u_first, int count, const RowView& rv) {
  const int u_last = u_first + count - 1;
  const int s_min = DESC ? rv.nslots - 1 - u_last : u_first;
  const int s_max = DESC ? rv.nslots - 1 - u_first : u_last;
  return u_last < rv.nslots && s_min * VEC >= rv.lo && (s_max + 1) * VEC <= rv.hi;
}

// A wave's share of one tile, in scan order.
template <int S, int VEC, int MODE>
struct TileData {
  float xs[S][VEC];                         // inputs / d_outputs
  float cs[S][VEC];                         // coefficients
  float ys[MODE == MODE_BWD ? S : 1][VEC];  // saved outputs (backward only)
  float y_edge;  // backward, lane 63: first element (scan order) of the slot after the wave's last
};

// INTERIOR: the caller guarantees that every slot of the wave is fully inside the row, so the
// loads are unconditional 16-byte accesses.  `row_start`: this wave holds the row's first slot.
template <int S, int VEC, int MODE, bool DESC, bool INTERIOR, typename T>
__device__ __forceinline__ void tile_load(TileData<S, VEC, MODE>& d, const RowPtrs<T>& q, const RowView& rv,
                                          int u_wave, int lane, bool row_start) {
  if constexpr (INTERIOR) {
    // Wave-uniform base (the lowest slot of the wave's share) plus a small per-lane index: the
    // compiler keeps the base in SGPRs and folds j * 64 into the instruction's offset field.
    const long long s_low = DESC ? (long long)rv.nslots - u_wave - S * 64 : (long long)u_wave;
    const T* bx = q.in0 + s_low * VEC;
    const T* bc = q.coef + s_low * VEC;
    const T* by = MODE == MODE_BWD ? q.aux + s_low * VEC : nullptr;
    const unsigned lane_idx = DESC ? 63u - unsigned(lane) : unsigned(lane);
#if LINREC_LOAD_ORDER == 2
    // all inputs, then all coefficients
#pragma unroll
    for (int j = 0; j < S; ++j) {
      const unsigned idx = (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx;
      load_slot_full<VEC, DESC>(bx, idx, d.xs[j]);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j = 0; j < S; ++j) {
      const unsigned idx = (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx;
      load_slot_full<VEC, DESC>(bc, idx, d.cs[j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (MODE == MODE_BWD) {
#pragma unroll
      for (int j = 0; j < S; ++j) {
        const unsigned idx = (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx;
        load_slot_full<VEC, DESC>(by, idx, d.ys[j]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#else
#pragma unroll
    for (int j = 0; j < S; ++j) {
      const unsigned idx = (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx;
#if LINREC_SADDR_LOAD
      load_slot_full<VEC, DESC>(bx, idx, d.xs[j]);
#if LINREC_LOAD_ORDER == 1
      __builtin_amdgcn_sched_barrier(0);
#endif
      load_slot_full<VEC, DESC>(bc, idx, d.cs[j]);
#if LINREC_LOAD_ORDER == 1
      __builtin_amdgcn_sched_barrier(0);
#endif
      if constexpr (MODE == MODE_BWD) load_slot_full<VEC, DESC>(by, idx, d.ys[j]);
#if LINREC_LOAD_ORDER == 1
      __builtin_amdgcn_sched_barrier(0);
#endif
#else
      const unsigned s = unsigned(slot_of<VEC, DESC>(u_wave + j * 64 + lane, rv));
      load_slot_full<VEC, DESC>(q.in0, s, d.xs[j]);
      load_slot_full<VEC, DESC>(q.coef, s, d.cs[j]);
      if constexpr (MODE == MODE_BWD) load_slot_full<VEC, DESC>(q.aux, s, d.ys[j]);
      (void)idx; (void)bx; (void)bc; (void)by;
#endif
    }
#endif
  } else {
#pragma unroll
    for (int j = 0; j < S; ++j) {
      const int u = u_wave + j * 64 + lane;
      load_slot<VEC, DESC>(q.in0, u, rv, 0.0f, d.xs[j]);
      load_slot<VEC, DESC>(q.coef, u, rv, 1.0f, d.cs[j]);
      if constexpr (MODE == MODE_BWD) load_slot<VEC, DESC>(q.aux, u, rv, 0.0f, d.ys[j]);
    }
  }
  d.y_edge = 0.0f;
  if constexpr (MODE == MODE_BWD) {
    if (lane == 63) {
      const int u_next = u_wave + S * 64;
      const int s_next = slot_of<VEC, DESC>(u_next, rv);
      d.y_edge = (u_next < rv.nslots) ? load_element(q.aux, vindex<VEC, DESC>(s_next, 0), rv, 0.0f) : 0.0f;
    }
  }
  if constexpr (MODE == MODE_FWD) {
    // The coefficient of the row's first element in scan order takes no part (nothing precedes it).
    if (row_start && lane == 0) {
      const int v_first = DESC ? rv.hi - 1 : rv.lo;
      const int s0 = slot_of<VEC, DESC>(0, rv);
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        if (vindex<VEC, DESC>(s0, i) == v_first) d.cs[0][i] = 0.0f;
    }
  }
}

// A wave's share of one interior tile as it arrives from memory, still in the storage type.  A kernel that keeps
// loads in flight across the steps of a software pipeline holds 16-bit data this way (half the registers of
// TileData, and nothing that would have to wait for the loads before the step that uses them).
template <typename T, int S, int VEC, int MODE>
struct TilePacked {
  using V = typename Pack<T, VEC>::type;
  V xs[S], cs[S], ys[MODE == MODE_BWD ? S : 1];
  T y_edge;
};

// The loads of tile_load<..., INTERIOR = true>, in the same order, without the conversion.
// MASKED: the row is whole slots (rv.lo == 0, its length a multiple of VEC) and ends inside this tile: a slot lies in
// the row or beyond its end, and the slots beyond it read as inputs of zero and coefficients of one.
template <int S, int VEC, int MODE, bool DESC, bool MASKED = false, typename T>
__device__ __forceinline__ void tile_load_packed(TilePacked<T, S, VEC, MODE>& d, const RowPtrs<T>& q, const RowView& rv,
                                                 int u_wave, int lane) {
  static_assert(VEC > 1, "whole slots");
  using V = typename Pack<T, VEC>::type;
  // (with MASKED this may lie in front of the row: only slots of the row are read)
  const long long s_low = DESC ? (long long)rv.nslots - u_wave - S * 64 : (long long)u_wave;
  const V* bx = reinterpret_cast<const V*>(q.in0) + s_low;
  const V* bc = reinterpret_cast<const V*>(q.coef) + s_low;
  const V* by = MODE == MODE_BWD ? reinterpret_cast<const V*>(q.aux) + s_low : nullptr;
  const unsigned lane_idx = DESC ? 63u - unsigned(lane) : unsigned(lane);
  // (a slot beyond the row: the registers are set first and the load is skipped)
  auto load_or = [&](V& to, const V* from, int j, float fill) {
    if constexpr (MASKED) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) to[i] = T(fill);
      if (u_wave + j * 64 + lane < rv.nslots) to = stream_load(from);
    } else {
      to = stream_load(from);
    }
  };
#pragma unroll
  for (int j = 0; j < S; ++j) {
    load_or(d.xs[j], bx + (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx, j, 0.0f);
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int j = 0; j < S; ++j) {
    load_or(d.cs[j], bc + (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx, j, 1.0f);
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (MODE == MODE_BWD) {
#pragma unroll
    for (int j = 0; j < S; ++j) {
      load_or(d.ys[j], by + (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx, j, 0.0f);
      __builtin_amdgcn_sched_barrier(0);
    }
    d.y_edge = T(0.0f);
    if (lane == 63) {
      const int u_next = u_wave + S * 64;
      if (u_next < rv.nslots) {
        const int v = vindex<VEC, DESC>(slot_of<VEC, DESC>(u_next, rv), 0);
        if (v >= rv.lo && v < rv.hi) d.y_edge = q.aux[v];
      }
    }
  }
}

template <int S, int VEC, int MODE, bool DESC, typename T>
__device__ __forceinline__ void tile_unpack(const TilePacked<T, S, VEC, MODE>& k, TileData<S, VEC, MODE>& d) {
#pragma unroll
  for (int j = 0; j < S; ++j) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      d.xs[j][i] = float(k.xs[j][DESC ? VEC - 1 - i : i]);
      d.cs[j][i] = float(k.cs[j][DESC ? VEC - 1 - i : i]);
      if constexpr (MODE == MODE_BWD) d.ys[j][i] = float(k.ys[j][DESC ? VEC - 1 - i : i]);
    }
  }
  d.y_edge = MODE == MODE_BWD ? float(k.y_edge) : 0.0f;
}

// Result of the lane- and wave-level scan of a wave's share.
template <int S, int VEC>
struct TileScan {
  float pa[S][VEC], pb[S][VEC];  // element i of slot j = pa * P_j + pb, P_j the value entering the slot
  float ex_a[S], ex_b[S];        // P_j = ex_a * E + ex_b, E the value entering the wave
  Affine total;                  // the wave's whole map (wave-uniform)
};

template <int S, int VEC, int MODE>
__device__ __forceinline__ void tile_scan(const TileData<S, VEC, MODE>& d, TileScan<S, VEC>& r) {
  float agg_a[S], agg_b[S];
#pragma unroll
  for (int j = 0; j < S; ++j) {
    if constexpr (MODE == MODE_FWD) {
      r.pa[j][0] = d.cs[j][0];
      r.pb[j][0] = d.xs[j][0];
#pragma unroll
      for (int i = 1; i < VEC; ++i) {
        r.pa[j][i] = r.pa[j][i - 1] * d.cs[j][i];
        r.pb[j][i] = fmaf(r.pb[j][i - 1], d.cs[j][i], d.xs[j][i]);
      }
      agg_a[j] = r.pa[j][VEC - 1];
      agg_b[j] = r.pb[j][VEC - 1];
    } else {
      r.pa[j][0] = 1.0f;
      r.pb[j][0] = d.xs[j][0];
#pragma unroll
      for (int i = 1; i < VEC; ++i) {
        r.pa[j][i] = r.pa[j][i - 1] * d.cs[j][i - 1];
        r.pb[j][i] = fmaf(r.pb[j][i - 1], d.cs[j][i - 1], d.xs[j][i]);
      }
      agg_a[j] = r.pa[j][VEC - 1] * d.cs[j][VEC - 1];
      agg_b[j] = r.pb[j][VEC - 1] * d.cs[j][VEC - 1];
    }
  }
  // Wave-level: inclusive scan over lanes of each slot row, then chain the S rows.
  wave_inclusive_scan<S>(agg_a, agg_b);
  Affine run = {1.0f, 0.0f};  // composition of the slot rows before j (wave-uniform)
#pragma unroll
  for (int j = 0; j < S; ++j) {
    const Affine lane_ex = {shift_up_one_lane(agg_a[j], 1.0f), shift_up_one_lane(agg_b[j], 0.0f)};
    const Affine row_total = {read_lane(agg_a[j], 63), read_lane(agg_b[j], 63)};
    if (j == 0) {
      r.ex_a[j] = lane_ex.a;
      r.ex_b[j] = lane_ex.b;
    } else {
      const Affine e = compose(run, lane_ex);
      r.ex_a[j] = e.a;
      r.ex_b[j] = e.b;
    }
    run = j == 0 ? row_total : compose(run, row_total);
  }
  r.total = run;
}

// `entry` is the value entering the wave; has_entry == false means "nothing precedes" and is kept
// apart from entry == 0 so that 0 * inf can never poison a finite result.
template <int S, int VEC, int MODE, bool DESC, bool INTERIOR, typename T>
__device__ __forceinline__ void tile_apply_store(const TileData<S, VEC, MODE>& d, const TileScan<S, VEC>& r,
                                                 const RowPtrs<T>& q, const RowView& rv, int u_wave, int lane,
                                                 bool has_entry, float entry) {
  const long long s_low = DESC ? (long long)rv.nslots - u_wave - S * 64 : (long long)u_wave;
  T* b0 = q.out0 + s_low * VEC;
  T* b1 = MODE == MODE_BWD ? q.out1 + s_low * VEC : nullptr;
  const unsigned lane_idx = DESC ? 63u - unsigned(lane) : unsigned(lane);
  // Measured: issuing the two output streams of the backward as two batches is 1-2 % faster than
  // alternating them slot row by slot row; the forward is indifferent.
  if constexpr (INTERIOR && (LINREC_STORE_ORDER == 1 || (LINREC_STORE_ORDER == 0 && MODE == MODE_BWD))) {
    // compute every result first, then issue the stores back to back
    float r0[S][VEC], r1[MODE == MODE_BWD ? S : 1][VEC];
#pragma unroll
    for (int j = 0; j < S; ++j) {
      const float P = has_entry ? fmaf(entry, r.ex_a[j], r.ex_b[j]) : r.ex_b[j];
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        r0[j][i] = (MODE == MODE_BWD && i == 0) ? P + r.pb[j][0] : fmaf(r.pa[j][i], P, r.pb[j][i]);
      if constexpr (MODE == MODE_BWD) {
        const float for_lane63 = (j + 1 < S) ? read_lane(d.ys[(j + 1) % S][0], 0) : d.y_edge;
        const float y_next_slot = shift_down_one_lane(d.ys[j][0], for_lane63);
#pragma unroll
        for (int i = 0; i < VEC; ++i) r1[j][i] = r0[j][i] * (i + 1 < VEC ? d.ys[j][(i + 1) % VEC] : y_next_slot);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < S; ++j) {
      const unsigned idx = (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx;
      store_slot_full<VEC, DESC>(b0, idx, r0[j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (MODE == MODE_BWD) {
#pragma unroll
      for (int j = 0; j < S; ++j) {
        const unsigned idx = (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx;
        store_slot_full<VEC, DESC>(b1, idx, r1[j]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < S; ++j) {
    const float P = has_entry ? fmaf(entry, r.ex_a[j], r.ex_b[j]) : r.ex_b[j];
    float r0[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      r0[i] = (MODE == MODE_BWD && i == 0) ? P + r.pb[j][0] : fmaf(r.pa[j][i], P, r.pb[j][i]);
    const int u = u_wave + j * 64 + lane;
    const unsigned idx = (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx;
    if constexpr (INTERIOR) {
#if LINREC_SADDR_STORE
      store_slot_full<VEC, DESC>(b0, idx, r0);
#else
      store_slot_full<VEC, DESC>(q.out0, unsigned(slot_of<VEC, DESC>(u, rv)), r0);
      (void)b0;
#endif
    } else {
      store_slot<VEC, DESC>(q.out0, u, rv, r0);
    }
    if constexpr (MODE == MODE_BWD) {
      // d_coeffs needs the saved output one step further along this scan: the next element of
      // the slot, or the first element of the next slot, which lives in the next lane, for lane
      // 63 in lane 0 of the next slot row, and for the wave's last slot in y_edge.
      const float for_lane63 = (j + 1 < S) ? read_lane(d.ys[(j + 1) % S][0], 0) : d.y_edge;
      const float y_next_slot = shift_down_one_lane(d.ys[j][0], for_lane63);
      float r1[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) r1[i] = r0[i] * (i + 1 < VEC ? d.ys[j][(i + 1) % VEC] : y_next_slot);
      if constexpr (INTERIOR) {
#if LINREC_SADDR_STORE
        store_slot_full<VEC, DESC>(b1, idx, r1);
#else
        store_slot_full<VEC, DESC>(q.out1, unsigned(slot_of<VEC, DESC>(u, rv)), r1);
        (void)b1;
#endif
      } else {
        store_slot<VEC, DESC>(q.out1, u, rv, r1);
      }
    }
  }
}

// The value carried into scan-order slot `u_end` of a row (slots of VEC elements), computed by one wave
// from the row's own data.  The slow way out for a wave whose bounded wait for other workgroups'
// results ran out: correct whatever the others are doing (or not doing), so that a kernel whose
// workgroups wait for each other never has to hand out a wrong value.  It walks the row one element per
// lane and step (64 elements a step): as slow as it gets, and light on registers, which matters because
// it is compiled into kernels whose every register is spoken for.
template <int VEC, int MODE, bool DESC, typename T>
__device__ __forceinline__ float recompute_entry(const RowPtrs<T> q, const RowView rv, int u_end, int lane) {
  // the elements in front of slot u_end, as a row of its own in one-element slots
  RowView part;
  if constexpr (DESC) {
    const int first = (rv.nslots - u_end) * VEC;  // lowest virtual index that takes part
    part.lo = first < rv.lo ? rv.lo : first;
    part.hi = rv.hi;
  } else {
    const int end = u_end * VEC;  // one past the highest virtual index that takes part
    part.lo = rv.lo;
    part.hi = end > rv.hi ? rv.hi : end;
  }
  part.nslots = part.hi;
  const int count = part.hi - part.lo;
  float carry = 0.0f;
  bool has = false;
  for (int e = 0; e < count; e += 64) {
    // scan-order slot of element e: ascending, virtual index lo + e; descending, hi - 1 - e
    const int u = DESC ? e : part.lo + e;
    TileData<1, 1, MODE> d;
    tile_load<1, 1, MODE, DESC, false>(d, q, part, u, lane, false);
    if constexpr (MODE == MODE_FWD) {
      if (e == 0 && lane == 0) d.cs[0][0] = 0.0f;  // the row's first coefficient takes no part
    }
    TileScan<1, 1> r;
    tile_scan<1, 1, MODE>(d, r);
    carry = has ? fmaf(carry, r.total.a, r.total.b) : r.total.b;
    has = true;
  }
  return carry;
}

// Forward, 16-bit storage, for kernels that store a tile some steps after scanning it: the scan of a packed tile
// that leaves only each slot's map from the wave's entry value (ex_a, ex_b) and the wave's map (total).  The
// elements are scanned a second time when the tile is stored (tile_replay_store_packed), from the packed inputs,
// which take a quarter of the registers of the elements' maps (pa, pb) and the same number of operations.
// `row_first_lane`: this lane's first element is the row's first, whose coefficient takes no part.
template <int S, int VEC, bool DESC, typename T>
__device__ __forceinline__ void tile_scan_packed_fwd(const TilePacked<T, S, VEC, MODE_FWD>& k, bool row_first_lane,
                                                     TileScan<S, VEC>& r) {
  float agg_a[S], agg_b[S];
#pragma unroll
  for (int j = 0; j < S; ++j) {
    float a = float(k.cs[j][DESC ? VEC - 1 : 0]);
    float b = float(k.xs[j][DESC ? VEC - 1 : 0]);
    if (j == 0 && row_first_lane) a = 0.0f;
#pragma unroll
    for (int i = 1; i < VEC; ++i) {
      const float c = float(k.cs[j][DESC ? VEC - 1 - i : i]);
      a *= c;
      b = fmaf(b, c, float(k.xs[j][DESC ? VEC - 1 - i : i]));
    }
    agg_a[j] = a;
    agg_b[j] = b;
    __builtin_amdgcn_sched_barrier(0);  // (one slot's unpacked elements at a time)
  }
  wave_inclusive_scan<S>(agg_a, agg_b);
  Affine run = {1.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < S; ++j) {
    const Affine lane_ex = {shift_up_one_lane(agg_a[j], 1.0f), shift_up_one_lane(agg_b[j], 0.0f)};
    const Affine row_total = {read_lane(agg_a[j], 63), read_lane(agg_b[j], 63)};
    if (j == 0) {
      r.ex_a[j] = lane_ex.a;
      r.ex_b[j] = lane_ex.b;
    } else {
      const Affine e = compose(run, lane_ex);
      r.ex_a[j] = e.a;
      r.ex_b[j] = e.b;
    }
    run = j == 0 ? row_total : compose(run, row_total);
  }
  r.total = run;
}

// ... and the second scan: every lane runs the recurrence over its slots' elements from the value that enters the
// slot, rounds and packs the results as they come, and the stores go out back to back.
template <int S, int VEC, bool DESC, bool MASKED = false, typename T>
__device__ __forceinline__ void tile_replay_store_packed(const TilePacked<T, S, VEC, MODE_FWD>& k, const TileScan<S, VEC>& r,
                                                         bool row_first_lane, const RowPtrs<T>& q, const RowView& rv,
                                                         int u_wave, int lane, bool has_entry, float entry) {
  using V = typename Pack<T, VEC>::type;
  const long long s_low = DESC ? (long long)rv.nslots - u_wave - S * 64 : (long long)u_wave;
  V* b0 = reinterpret_cast<V*>(q.out0) + s_low;
  const unsigned lane_idx = DESC ? 63u - unsigned(lane) : unsigned(lane);
  V o[S];
#pragma unroll
  for (int j = 0; j < S; ++j) {
    float y = has_entry ? fmaf(entry, r.ex_a[j], r.ex_b[j]) : r.ex_b[j];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float x = float(k.xs[j][DESC ? VEC - 1 - i : i]);
      const float c = float(k.cs[j][DESC ? VEC - 1 - i : i]);
      y = (i == 0 && j == 0 && row_first_lane) ? x : fmaf(y, c, x);
      o[j][DESC ? VEC - 1 - i : i] = T(y);
    }
    __builtin_amdgcn_sched_barrier(0);  // (one slot's unpacked elements at a time)
  }
#pragma unroll
  for (int j = 0; j < S; ++j) {
    if (!MASKED || u_wave + j * 64 + lane < rv.nslots)  // (MASKED: rows of whole slots that end inside this tile)
      stream_store(o[j], b0 + (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// tile_apply_store for an interior tile of 16-bit storage whose saved outputs are still packed: the results are
// rounded and packed as they are computed, so the batch of stores holds S registers' worth per output tensor and
// not S * VEC floats.  The caller has folded each slot's map from the wave's entry value into the elements' maps
// (ex_a = 1, ex_b = 0, and pa[j][0] is a factor like the others, also in the backward).  `y_edge`: the saved output
// after the wave's last (what lane 63 needs; wave-uniform).
template <int S, int VEC, int MODE, bool DESC, bool MASKED = false, typename T>
__device__ __forceinline__ void tile_apply_store_packed(const typename Pack<T, VEC>::type* ys, float y_edge,
                                                        const TileScan<S, VEC>& r, const RowPtrs<T>& q, const RowView& rv,
                                                        int u_wave, int lane, bool has_entry, float entry) {
  using V = typename Pack<T, VEC>::type;
  const long long s_low = DESC ? (long long)rv.nslots - u_wave - S * 64 : (long long)u_wave;
  V* b0 = reinterpret_cast<V*>(q.out0) + s_low;
  V* b1 = MODE == MODE_BWD ? reinterpret_cast<V*>(q.out1) + s_low : nullptr;
  const unsigned lane_idx = DESC ? 63u - unsigned(lane) : unsigned(lane);
  V o0[S], o1[MODE == MODE_BWD ? S : 1];
#pragma unroll
  for (int j = 0; j < S; ++j) {
    const float P = has_entry ? fmaf(entry, r.ex_a[j], r.ex_b[j]) : r.ex_b[j];
    float r0[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) r0[i] = fmaf(r.pa[j][i], P, r.pb[j][i]);  // (the caller has folded the slot's map into pa, pb: also into pa[0])
    if constexpr (MODE == MODE_BWD) {
      // d_coeffs needs the saved output one step further along the scan (see tile_apply_store)
      const float first_of_next = (j + 1 < S) ? read_lane(float(ys[(j + 1) % S][DESC ? VEC - 1 : 0]), 0) : y_edge;
      const float y_next_slot = shift_down_one_lane(float(ys[j][DESC ? VEC - 1 : 0]), first_of_next);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float y_next = i + 1 < VEC ? float(ys[j][DESC ? VEC - 2 - i : i + 1]) : y_next_slot;
        o1[j][DESC ? VEC - 1 - i : i] = T(r0[i] * y_next);
      }
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) o0[j][DESC ? VEC - 1 - i : i] = T(r0[i]);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < S; ++j) {
    if (!MASKED || u_wave + j * 64 + lane < rv.nslots)  // (MASKED: rows of whole slots that end inside this tile)
      stream_store(o0[j], b0 + (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx);
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (MODE == MODE_BWD) {
#pragma unroll
    for (int j = 0; j < S; ++j) {
      if (!MASKED || u_wave + j * 64 + lane < rv.nslots)
        stream_store(o1[j], b1 + (DESC ? unsigned(S - 1 - j) : unsigned(j)) * 64u + lane_idx);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// The maps of the NW <= 16 waves of a workgroup lie in LDS.  Every wave folds them for itself by a
// four-step scan over the lanes of one DPP row (lane w: wave w's map, identity elsewhere) and takes what
// it needs out of it with v_readlane, so both results are wave-uniform scalars: the composition of the
// waves in front of `wave` (the identity for wave 0) and of all NW waves.
template <int NW>
__device__ __forceinline__ void wave_prefixes(const float* sh_a, const float* sh_b, int wave, int lane, Affine& before,
                                              Affine& total) {
  static_assert(NW <= 16, "one DPP row holds the waves' maps");
  float a[1] = {1.0f}, b[1] = {0.0f};
  if (lane < NW) {
    a[0] = sh_a[lane];
    b[0] = sh_b[lane];
  }
  if constexpr (NW > 1) scan_step<DPP_ROW_SHR1, 0xf>(a, b);
  if constexpr (NW > 2) scan_step<DPP_ROW_SHR2, 0xf>(a, b);
  if constexpr (NW > 4) scan_step<DPP_ROW_SHR4, 0xf>(a, b);
  if constexpr (NW > 8) scan_step<DPP_ROW_SHR8, 0xf>(a, b);
  total = {read_lane(a[0], NW - 1), read_lane(b[0], NW - 1)};
  // lane w-1 holds waves 0 .. w-1; for wave 0 this reads lane 63, which still holds the identity
  before = {read_lane(a[0], (wave - 1) & 63), read_lane(b[0], (wave - 1) & 63)};
}

}  // namespace linrec
