// Column block kernels: the scan axis is the strided one (element (r, l) at base[r + l*elem_stride],
// as in column_kernel.hpp), and the NW waves of a workgroup share the same 64*VEC adjacent rows.
// The scan axis is walked in steps of NW*U positions; within a step wave w takes the U positions
// [w*U, w*U + U) of every row, so a step of the workgroup reads NW*U coalesced lines per tensor
// where a lone wave of a column kernel reads U.  Per step:
//   1. every lane folds its U positions into the affine map value_out = a * value_in + b;
//   2. the maps go to LDS, one barrier;
//   3. every wave folds the maps of the waves before it into the value entering its own positions
//      (and all NW maps into the value entering the next step: every wave keeps that for itself,
//      so nothing has to be handed back), then walks its positions again from that value and stores.
// With fewer rows a wave is split into G groups of 64/G lanes: the groups share the same 64/G * VEC
// rows and take consecutive runs of positions, so a workgroup covers fewer rows and more of the
// scan axis per step, and the launch has G times as many workgroups.  The maps of a wave's groups
// of the two halves are composed through a half swap in the vector ALU (lanes_up_32) before the wave's
// total goes to LDS.  (Four groups of 16 lanes, 64-byte accesses, ran at half the rate.)
// One pass over the tensors (12 bytes per element forward, 20 backward), no workspace, no workgroup
// waits for another.  It serves row counts that leave the plain column kernel a wave or less per
// SIMD and that fill the chip with workgroups of NW waves: (batch, time, channels) data with a few
// thousand to a few ten thousand channels.
//
// The reference has no strided kernel: it rejects inputs whose last stride is not 1
// (linrec/impl/cuda/linrec_pipe.cu:35).
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "column_kernel.hpp"  // ColumnArgs, Lanes, ld_rows, st_rows

namespace linrec {

template <typename T, int VEC, int U, int NW, int G, int MODE, bool DESC>
__global__ __launch_bounds__(64 * NW) void colblock_kernel(ColumnArgs p) {
  static_assert(G == 1 || G == 2, "a wave is whole or split into its two halves");
  constexpr int RL = 64 / G;        // lanes of a group: RL * VEC rows per workgroup
  constexpr int STEP = NW * G * U;  // positions per step of the workgroup
  __shared__ float sh_a[2][NW][RL * VEC];
  __shared__ float sh_b[2][NW][RL * VEC];

  const T* in0 = static_cast<const T*>(p.in0);
  const T* coef = static_cast<const T*>(p.coef);
  const T* aux = static_cast<const T*>(p.aux);
  T* out0 = static_cast<T*>(p.out0);
  T* out1 = static_cast<T*>(p.out1);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = G == 1 ? 0 : lane / RL;  // this lane's group and its place in it
  const int rl = G == 1 ? lane : lane % RL;
  const int run = wave * G + grp;          // which run of U positions of a step this lane takes
  // Lanes beyond the last row read the last rows again and store nothing: they take part in every
  // barrier, and the loads of a full step stay unconditional.
  long long r0 = ((long long)blockIdx.x * RL + rl) * VEC;
  const bool active = r0 < p.numseq;
  if (!active) r0 = p.numseq - VEC;
  long long base = r0 * p.row_stride;  // VEC > 1 implies row_stride == 1 and rows that never straddle a batch
  if (p.rows_per_batch < p.numseq) {
    const long long batch = r0 / p.rows_per_batch;
    base = batch * p.batch_stride + (r0 - batch * p.rows_per_batch) * p.row_stride;
  }
  const int L = p.seqlen;
  constexpr bool NEED_Y = MODE == 1;

  Lanes<VEC> carry;  // value entering the current step: forward the previous output, backward the
                     // previous d_input times its coefficient; the same in every wave
#pragma unroll
  for (int e = 0; e < VEC; ++e) carry.v[e] = 0.0f;

  struct Batch {
    Lanes<VEC> x[U], c[U], yn[NEED_Y ? U : 1];
  };
  // FULL: all U positions n0 .. n0+U-1 exist and, for the backward, so do their successors.
  auto load_batch = [&](Batch& bt, int n0, auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = n0 + u;  // position in scan order
      const int l = DESC ? L - 1 - n : n;
      if (FULL || n < L) {
        const long long off = base + (long long)l * p.elem_stride;
        bt.x[u] = ld_rows<VEC>(in0 + off);
        bt.c[u] = ld_rows<VEC>(coef + off);
        if constexpr (NEED_Y) {
          // saved output one step further along this scan; nothing beyond the row end
          const int ln = DESC ? l - 1 : l + 1;
          if (FULL || (ln >= 0 && ln < L)) {
            bt.yn[u] = ld_rows<VEC>(aux + base + (long long)ln * p.elem_stride);
          } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) bt.yn[u].v[e] = 0.0f;
          }
        }
      }
    }
  };

  // Step k of the walk, this lane's positions n0 .. n0+U-1 already in registers.
  auto finish_step = [&](const Batch& bt, int k, int n0, auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    const int par = k & 1;
    // 1. the map of this lane's positions (the identity where the row has ended)
    Lanes<VEC> ma, mb;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      ma.v[e] = 1.0f;
      mb.v[e] = 0.0f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = n0 + u;
      if (FULL || n < L) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          if constexpr (MODE == 0) {
            // the coefficient of the first position takes no part (linrec_ref.cuh:63)
            mb.v[e] = n == 0 ? bt.x[u].v[e] : fmaf(mb.v[e], bt.c[u].v[e], bt.x[u].v[e]);
            ma.v[e] = n == 0 ? 0.0f : ma.v[e] * bt.c[u].v[e];
          } else {
            mb.v[e] = (mb.v[e] + bt.x[u].v[e]) * bt.c[u].v[e];
            ma.v[e] *= bt.c[u].v[e];
          }
        }
      }
    }
    // the two groups of a wave: the upper one's map becomes the map of both; it keeps what precedes it
    Lanes<VEC> ex_a, ex_b;
    if constexpr (G > 1) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        ex_a.v[e] = lanes_up_32(ma.v[e]);  // the lower group's map, which precedes the upper group's
        ex_b.v[e] = lanes_up_32(mb.v[e]);
        if (grp == 1) {
          mb.v[e] = fmaf(ex_b.v[e], ma.v[e], mb.v[e]);
          ma.v[e] = ex_a.v[e] * ma.v[e];
        }
      }
    }
    if (G == 1 || grp == G - 1) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        sh_a[par][wave][e * RL + rl] = ma.v[e];
        sh_b[par][wave][e * RL + rl] = mb.v[e];
      }
    }
    __syncthreads();
    // 2. what enters this lane's positions, and what enters the next step.  Before the first map
    // of a row there is nothing: its b is taken as it is, so that 0 * inf can never arise.
    // (four maps at a time: unrolled completely, the 2 * NW * VEC values read from LDS are all held in
    // registers at once, 128 of them for two rows per lane)
    Lanes<VEC> entry = carry;
#pragma unroll 4
    for (int w = 0; w < NW; ++w) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float a = sh_a[par][w][e * RL + rl], b = sh_b[par][w][e * RL + rl];
        carry.v[e] = (k == 0 && w == 0) ? b : fmaf(carry.v[e], a, b);
      }
      if (w + 1 == wave) entry = carry;
    }
    if constexpr (G > 1) {
      if (grp > 0) {
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          entry.v[e] = (k == 0 && wave == 0) ? ex_b.v[e] : fmaf(entry.v[e], ex_a.v[e], ex_b.v[e]);
      }
    }
    // 3. walk the positions again from the entering value
    Lanes<VEC> val = entry;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = n0 + u;
      const int l = DESC ? L - 1 - n : n;
      if (FULL || n < L) {
        const long long off = base + (long long)l * p.elem_stride;
        if constexpr (MODE == 0) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) val.v[e] = n == 0 ? bt.x[u].v[e] : fmaf(val.v[e], bt.c[u].v[e], bt.x[u].v[e]);
          if (active) st_rows<VEC>(out0 + off, val);
        } else {
          Lanes<VEC> dx, dc;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            dx.v[e] = val.v[e] + bt.x[u].v[e];
            dc.v[e] = dx.v[e] * bt.yn[u].v[e];
            val.v[e] = dx.v[e] * bt.c[u].v[e];
          }
          if (active) {
            st_rows<VEC>(out0 + off, dx);
            st_rows<VEC>(out1 + off, dc);
          }
        }
      }
    }
  };
  using True = std::integral_constant<bool, true>;
  using False = std::integral_constant<bool, false>;

  // Steps [0, kfull) are full for every wave (for the backward the last position's successor must
  // exist too); they run double-buffered, the next step's loads in flight while this one is
  // scanned and stored.  The one or two steps that hold the row end follow without prefetch.
  const int with_successor = NEED_Y ? L - 1 : L;
  const int kfull = with_successor / STEP;
  const int ksteps = (L + STEP - 1) / STEP;
  if (kfull > 0) {
    Batch cur;
    load_batch(cur, run * U, True{});
    for (int k = 0; k + 1 < kfull; ++k) {
      Batch nxt;
      load_batch(nxt, (k + 1) * STEP + run * U, True{});
      finish_step(cur, k, k * STEP + run * U, True{});
      cur = nxt;
    }
    finish_step(cur, kfull - 1, (kfull - 1) * STEP + run * U, True{});
  }
  for (int k = kfull; k < ksteps; ++k) {
    Batch tail;
    load_batch(tail, k * STEP + run * U, False{});
    finish_step(tail, k, k * STEP + run * U, False{});
  }
}

}  // namespace linrec
