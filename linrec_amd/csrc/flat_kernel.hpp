// Flat kernels: dense tensors of short rows whose length is not a whole number of 16-byte slots.
// Seen row by row, every row of such a tensor starts at another phase of its first slot and ends
// inside its last one, and the kernels that give lanes to rows (group_kernel.hpp) fall back to
// element-sized accesses at both ends of every row.  Seen as one flat array the tensor is just a
// sequence of slots, all of them full and aligned, and the recurrence over the flat array is the
// recurrence over the rows as soon as the scan is cut at every row start (in scan order), where
// the definition uses no coefficient anyway (linrec/impl/cuda/linrec_ref.cuh:63,
// linrec/impl/python/ops.py:16-18).  The cut is a flag that travels with the affine maps (a
// segmented scan), not a multiplication by zero: nothing of a row, non-finite values included,
// reaches the next one.  A lane computes elements of two or three rows - of up to VEC rows where a row is
// shorter than a slot - and stores whole slots.
//
// A wave takes 64 * S consecutive slots (S rows of 64 slots, lanes interleaved for coalescing) and
// never talks to another wave: what enters its chunk depends on the elements back to the last
// row start only, fewer than one row, so the wave reads up to one more row of 64 slots in front of
// its chunk (the lanes that cover one row length) and scans it along; the cut inside it makes
// whatever came before irrelevant.  No LDS, no barrier, no workspace.
//
// Requirements (the planner's): unit element stride, row stride == row length, all bases 16-byte
// aligned, 2 <= row length <= 64 * VEC.
//
// The reference has no counterpart: its kernels give a block to every row
// (linrec/impl/cuda/linrec_tile.cuh:11-95).
#pragma once
#include <hip/hip_runtime.h>

#include "memio.hpp"
#include "scan_primitives.hpp"

namespace linrec {

struct FlatArgs {
  const void* in0;    // forward: inputs        backward: d_outputs   (storage type T of the kernel)
  const void* coef;
  const void* aux;    // backward: saved outputs
  void* out0;         // forward: outputs       backward: d_inputs
  void* out1;         // backward: d_coeffs
  long long total;    // elements of the tensor
  int seqlen;
  int zero_pos;       // position in the row whose coefficient is unused: 0, or seqlen - 1 for reverse
};

// One Kogge-Stone step of the segmented scan on R independent rows: a map that contains a cut
// (f != 0) takes nothing from the maps in front of it.
template <int CTRL, int ROW_MASK, int R>
__device__ __forceinline__ void cut_scan_step(float (&a)[R], float (&b)[R], float (&f)[R]) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float pa = dpp_move<CTRL, ROW_MASK>(1.0f, a[r]);
    const float pb = dpp_move<CTRL, ROW_MASK>(0.0f, b[r]);
    const float pf = dpp_move<CTRL, ROW_MASK>(0.0f, f[r]);
    b[r] = f[r] != 0.0f ? b[r] : fmaf(pb, a[r], b[r]);
    a[r] = pa * a[r];
    f[r] = fmaxf(f[r], pf);
  }
}

template <int R>
__device__ __forceinline__ void wave_inclusive_cut_scan(float (&a)[R], float (&b)[R], float (&f)[R]) {
  cut_scan_step<DPP_ROW_SHR1, 0xf>(a, b, f);
  cut_scan_step<DPP_ROW_SHR2, 0xf>(a, b, f);
  cut_scan_step<DPP_ROW_SHR4, 0xf>(a, b, f);
  cut_scan_step<DPP_ROW_SHR8, 0xf>(a, b, f);
  cut_scan_step<DPP_ROW_BCAST15, 0xa>(a, b, f);
  cut_scan_step<DPP_ROW_BCAST31, 0xc>(a, b, f);
}

// MODE_FWD = 0, MODE_BWD = 1 (same numbering as the tile kernels).
template <typename T, int VEC, int S, int MODE, bool DESC>
__global__ __launch_bounds__(256) void flat_kernel(FlatArgs p) {
  constexpr int R = S + 1;  // row 0 of the register tile is the look-behind row, rows 1 .. S the chunk
  const int lane = threadIdx.x & 63;
  const long long wave = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const long long nslots = (p.total + VEC - 1) / VEC;
  const long long u_chunk = wave * (64 * S);  // first slot of the chunk, in scan order
  if (u_chunk >= nslots) return;              // the whole wave
  const int L = p.seqlen;
  const T* in0 = static_cast<const T*>(p.in0);
  const T* coef = static_cast<const T*>(p.coef);
  const T* aux = static_cast<const T*>(p.aux);

  // lanes of the look-behind row that reach back one row length (and a slot) from the chunk start
  const int behind_lanes = (L + VEC - 1) / VEC + 1;

  // Position in its row of the first memory element of this lane's slot in row 1; the other rows
  // follow by steps of 64 slots.
  const long long u_first = u_chunk + lane;
  const long long s_first = DESC ? nslots - 1 - u_first : u_first;
  int r_slot = int((s_first * VEC) % L);
  const int step = (64 * VEC) % L;  // row position advances by this from one row of slots to the next in memory

  float xs[R][VEC], cs[R][VEC], yn[R][VEC];
  bool cut[R][VEC];  // forward: the scan starts anew at this element; backward: nothing leaves it
  bool have[R];  // the slot exists (and, for the look-behind row, is wanted)
  float y_first[R];  // backward: first saved output of the slot in scan order, for the neighbour lane
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const long long u = u_chunk + (long long)(j - 1) * 64 + lane;  // scan-order slot
    have[j] = u >= 0 && u < nslots && (j > 0 || lane >= 64 - behind_lanes);
    const long long s = DESC ? nslots - 1 - u : u;  // memory slot
    // row position of the slot's first memory element: j - 1 rows of 64 slots further along the scan
    // than row 1, which is forward in memory for ascending scans (|j - 1| * step < S * L)
    int r0 = r_slot + (DESC ? 1 - j : j - 1) * step;
#pragma unroll
    for (int k = 1; k < S; ++k)
      if (r0 >= L) r0 -= L;
#pragma unroll
    for (int k = 1; k < S; ++k)
      if (r0 < 0) r0 += L;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      xs[j][i] = 0.0f;
      cs[j][i] = 1.0f;
      yn[j][i] = 0.0f;
      cut[j][i] = false;
    }
    y_first[j] = 0.0f;
    if (have[j]) {
      float ys[VEC];
      load_slot_full<VEC, DESC>(in0 + s * VEC, 0u, xs[j]);
      load_slot_full<VEC, DESC>(coef + s * VEC, 0u, cs[j]);
      if constexpr (MODE == 1) {
        if (j > 0) load_slot_full<VEC, DESC>(aux + s * VEC, 0u, ys);
      }
      // row positions of the slot's elements in memory order (a row may be shorter than the slot)
      int rpos[VEC];
      rpos[0] = r0;
#pragma unroll
      for (int e = 1; e < VEC; ++e) rpos[e] = rpos[e - 1] + 1 == L ? 0 : rpos[e - 1] + 1;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const int e = DESC ? VEC - 1 - i : i;  // memory offset inside the slot of scan element i
        const int r = rpos[e];
        const bool beyond = s * VEC + e >= p.total;  // the tail of the tensor's last slot
        if (beyond) {
          xs[j][i] = 0.0f;
          cs[j][i] = 1.0f;
        }
        cut[j][i] = r == p.zero_pos && !beyond;
        if constexpr (MODE == 1) {
          if (j > 0) {
            if (beyond) ys[i] = 0.0f;
            // the saved output one step further along the scan belongs to the next scan element;
            // marked here where it does not exist (this element ends its row)
            yn[j][i] = (r == p.zero_pos || beyond) ? 0.0f : 1.0f;
          }
        }
      }
      if constexpr (MODE == 1) {
        if (j > 0) {
          y_first[j] = ys[0];
#pragma unroll
          for (int i = 0; i + 1 < VEC; ++i) yn[j][i] *= ys[i + 1];
        }
      }
    }
  }

  if constexpr (MODE == 1) {
    // last element of every slot: its successor is the first element of the next slot in scan order,
    // i.e. of the next lane, of lane 0 of the next row of slots, or of the slot after the chunk
    float after_chunk = 0.0f;
    {
      const long long u = u_chunk + (long long)S * 64;
      if (lane == 63 && u < nslots) {
        const long long s = DESC ? nslots - 1 - u : u;
        const long long m = s * VEC + (DESC ? VEC - 1 : 0);
        if (m < p.total) after_chunk = float(aux[m]);
      }
    }
#pragma unroll
    for (int j = 1; j < R; ++j) {
      float nxt = shift_down_one_lane(y_first[j], 0.0f);
      const float wrap = j + 1 < R ? read_lane(y_first[j + 1 < R ? j + 1 : j], 0) : after_chunk;
      if (lane == 63) nxt = wrap;
      yn[j][VEC - 1] *= nxt;
    }
  }

  // lane level: the slot's elements in scan order (see tile_scan in tile_core.hpp for the two forms);
  // cut_before[j][i]: a cut lies between the slot's entry and element i, which then takes nothing
  // from what enters the slot
  float pa[R][VEC], pb[R][VEC], agg_a[R], agg_b[R], agg_f[R];
  bool cut_before[R][VEC];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    if constexpr (MODE == 0) {
      pa[j][0] = cs[j][0];
      pb[j][0] = xs[j][0];
      cut_before[j][0] = cut[j][0];
#pragma unroll
      for (int i = 1; i < VEC; ++i) {
        pa[j][i] = pa[j][i - 1] * cs[j][i];
        pb[j][i] = cut[j][i] ? xs[j][i] : fmaf(pb[j][i - 1], cs[j][i], xs[j][i]);
        cut_before[j][i] = cut_before[j][i - 1] || cut[j][i];
      }
      agg_a[j] = pa[j][VEC - 1];
      agg_b[j] = pb[j][VEC - 1];
      agg_f[j] = cut_before[j][VEC - 1] ? 1.0f : 0.0f;
    } else {
      pa[j][0] = 1.0f;
      pb[j][0] = xs[j][0];
      cut_before[j][0] = false;
#pragma unroll
      for (int i = 1; i < VEC; ++i) {
        pa[j][i] = pa[j][i - 1] * cs[j][i - 1];
        pb[j][i] = cut[j][i - 1] ? xs[j][i] : fmaf(pb[j][i - 1], cs[j][i - 1], xs[j][i]);
        cut_before[j][i] = cut_before[j][i - 1] || cut[j][i - 1];
      }
      agg_a[j] = pa[j][VEC - 1] * cs[j][VEC - 1];
      agg_b[j] = cut[j][VEC - 1] ? 0.0f : pb[j][VEC - 1] * cs[j][VEC - 1];
      agg_f[j] = cut_before[j][VEC - 1] || cut[j][VEC - 1] ? 1.0f : 0.0f;
    }
  }

  // wave level: all rows of slots at once, then the rows chained in scan order
  wave_inclusive_cut_scan<R>(agg_a, agg_b, agg_f);
  float carry = 0.0f;  // what enters row 0 is cut off inside it
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const float ex_a = shift_up_one_lane(agg_a[j], 1.0f);
    const float ex_b = shift_up_one_lane(agg_b[j], 0.0f);
    const float ex_f = shift_up_one_lane(agg_f[j], 0.0f);
    const float enter = ex_f != 0.0f ? ex_b : fmaf(carry, ex_a, ex_b);
    carry = read_lane(agg_f[j], 63) != 0.0f ? read_lane(agg_b[j], 63)
                                            : fmaf(carry, read_lane(agg_a[j], 63), read_lane(agg_b[j], 63));
    if (j == 0) continue;  // nothing of the look-behind row is stored
    float r0[VEC], r1[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float with_entry = (MODE == 1 && i == 0) ? enter + pb[j][0] : fmaf(pa[j][i], enter, pb[j][i]);
      r0[i] = cut_before[j][i] ? pb[j][i] : with_entry;
      r1[i] = r0[i] * yn[j][i];
    }
    if (have[j]) {
      const long long u = u_chunk + (long long)(j - 1) * 64 + lane;
      const long long s = DESC ? nslots - 1 - u : u;
      if ((s + 1) * VEC <= p.total) {
        store_slot_full<VEC, DESC>(static_cast<T*>(p.out0) + s * VEC, 0u, r0);
        if constexpr (MODE == 1) store_slot_full<VEC, DESC>(static_cast<T*>(p.out1) + s * VEC, 0u, r1);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const long long m = s * VEC + (DESC ? VEC - 1 - i : i);
          if (m < p.total) {
            static_cast<T*>(p.out0)[m] = T(r0[i]);
            if constexpr (MODE == 1) static_cast<T*>(p.out1)[m] = T(r1[i]);
          }
        }
      }
    }
  }
}

}  // namespace linrec
