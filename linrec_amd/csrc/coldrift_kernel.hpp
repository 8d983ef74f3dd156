// Column drift kernels: the column block kernels' workgroup (NW waves that share the same 64/G * VEC
// adjacent rows of a tensor whose scan axis is the strided one, colblock_kernel.hpp) in teams of M
// along the scan axis.  With only a few thousand rows a launch of one workgroup per block of rows
// leaves most of the chip idle; here M workgroups share a block of rows and take its steps (of
// NW * G * U positions) in turn, workgroup j the steps j, j + M, ..., so that the launch has M times
// as many workgroups and still reads every tensor once.
//
// What enters a step is what left the step before it, which another workgroup has: as in the drift
// kernels (drift_kernel.hpp) only the steps' affine maps travel between workgroups, and nobody waits
// for them.  A step is scanned into per-wave maps, its whole map (one per row) is published, and the
// step's data stays in registers; two of the workgroup's own steps later the maps of the M - 1 steps
// in between, asked for at the top of the step ahead of the prefetch loads, have long arrived: wave w
// collects the map of the w-th of them, all waves compose them after the barrier onto the value that
// left the workgroup's own previous step, walk the kept positions again from there and store.
//
// Every workgroup of the launch has to be resident at once (the planner sees to that).  Every wait
// is bounded all the same; a wave whose wait runs out notes it in LDS and the workgroup computes
// what enters the step from the rows' own data, one lane per row, sequentially.
//
// The reference has no strided kernel (linrec/impl/cuda/linrec_pipe.cu:35).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "column_kernel.hpp"  // ColumnArgs, Lanes, ld_rows, st_rows
#include "tile_kernel.hpp"    // TileArgs (workspace header, counters, descriptors), completion count

namespace linrec {

struct ColDriftArgs {
  ColumnArgs col;
  TileArgs chain;  // of it: ws, counters, desc, ws_tiles, spin_limit, num_tiles (workgroups), tasks (team size M)
};

// What a lane keeps of one position of its VEC rows from the load to the store three steps later: the values as
// loaded.  16-bit storage stays packed (two rows to a register) and is widened where it is used, so that a step of
// two rows per lane holds as many registers, and moves as many bytes, as an fp32 step of one.
template <typename T, int VEC>
struct Held {
  using V = typename Pack<T, VEC>::type;
  V q;
};
template <int VEC>
struct Held<float, VEC> {
  Lanes<VEC> q;
};
template <int VEC, typename T>
__device__ __forceinline__ Held<T, VEC> ld_held(const T* p) {
  Held<T, VEC> h;
  if constexpr (std::is_same_v<T, float>) {
    h.q = ld_rows<VEC>(p);
  } else {
    using V = typename Pack<T, VEC>::type;
    h.q = stream_load(reinterpret_cast<const V*>(p));
  }
  return h;
}
template <typename T, int VEC>
__device__ __forceinline__ Lanes<VEC> widen(const Held<T, VEC>& h) {
  if constexpr (std::is_same_v<T, float>) {
    return h.q;
  } else {
    Lanes<VEC> r;
#pragma unroll
    for (int e = 0; e < VEC; ++e) r.v[e] = float(h.q[e]);
    return r;
  }
}
// The same values as something the compiler knows nothing about: what was widened from `h` before is not what is
// widened from the result, so the packed register stays the one that lives from a step's scan to its store (the
// compiler would rather keep the widened values, two registers for one).
template <typename T, int VEC>
__device__ __forceinline__ Held<T, VEC> held_again(Held<T, VEC> h) {
  if constexpr (!std::is_same_v<T, float> && sizeof(typename Pack<T, VEC>::type) == 4) {
    uint32_t bits = __builtin_bit_cast(uint32_t, h.q);
    asm volatile("" : "+v"(bits));
    h.q = __builtin_bit_cast(typename Pack<T, VEC>::type, bits);
  }
  return h;
}
template <typename T, int VEC>
__device__ __forceinline__ Held<T, VEC> held_zero() {
  Held<T, VEC> h;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    if constexpr (std::is_same_v<T, float>) h.q.v[e] = 0.0f;
    else h.q[e] = T(0.0f);
  }
  return h;
}

template <typename T, int VEC, int U, int NW, int G, int MODE, bool DESC>
__global__ __launch_bounds__(64 * NW) void coldrift_kernel(ColDriftArgs args) {
  static_assert(G == 1 || G == 2, "a wave is whole or split into its two halves");
  const ColumnArgs& p = args.col;
  const TileArgs& ch = args.chain;
  constexpr int RL = 64 / G;        // lanes of a group
  constexpr int RPB = RL * VEC;     // rows per block of rows
  constexpr int STEP = NW * G * U;  // positions per step
  // the waves' maps of a step, kept until the step is stored: own step i in [i % 4]
  __shared__ float sh_a[4][NW][RPB];
  __shared__ float sh_b[4][NW][RPB];
  // the team mates' maps a wave has collected (wave w: the w-th step back): steps alternate between [0]
  // and [1]; [2] and [3] are the last two steps'
  __shared__ float sh_pa[4][NW][RPB];
  __shared__ float sh_pb[4][NW][RPB];
  __shared__ int sh_fail[4];  // the own step (-2, -3 for the last two) in which a wave's wait ran out

  const T* in0 = static_cast<const T*>(p.in0);
  const T* coef = static_cast<const T*>(p.coef);
  const T* aux = static_cast<const T*>(p.aux);
  T* out0 = static_cast<T*>(p.out0);
  T* out1 = static_cast<T*>(p.out1);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = G == 1 ? 0 : lane / RL;
  const int rl = G == 1 ? lane : lane % RL;
  const int run = wave * G + grp;  // which run of U positions of a step this lane takes
  const int M = ch.tasks;
  const long long block = blockIdx.x / M;  // block of rows
  const int j = int(blockIdx.x - block * M);
  long long r0 = (block * RL + rl) * VEC;
  const bool active = r0 < p.numseq;
  if (!active) r0 = p.numseq - VEC;  // lanes beyond the last row read the last rows again and store nothing
  long long base = r0 * p.row_stride;
  if (p.rows_per_batch < p.numseq) {
    const long long batch = r0 / p.rows_per_batch;
    base = batch * p.batch_stride + (r0 - batch * p.rows_per_batch) * p.row_stride;
  }
  const int L = p.seqlen;
  constexpr bool NEED_Y = MODE == 1;
  const int ksteps = (L + STEP - 1) / STEP;              // steps of the whole row
  const int own = j < ksteps ? (ksteps - j + M - 1) / M : 0;  // steps of this workgroup: j, j + M, ...
  const uint32_t seq = load_seq_through_caches(ch.ws);
  const uint32_t want = (seq << 2) | STATUS_AGGREGATE;
  if (threadIdx.x < 4) sh_fail[threadIdx.x] = -1;
  __syncthreads();
  // descriptors: step k of this block of rows, row i of the block: two words (a, b)
  uint64_t* const desc = ch.desc + 2 * (block * ksteps) * RPB;

  struct Batch {
    Held<T, VEC> x[U], c[U], yn[NEED_Y ? U : 1];
  };
  auto load_batch = [&](Batch& bt, int n0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = n0 + u;  // position in scan order
      const int l = DESC ? L - 1 - n : n;
      if (n < L) {
        const long long off = base + (long long)l * p.elem_stride;
        bt.x[u] = ld_held<VEC>(in0 + off);
        bt.c[u] = ld_held<VEC>(coef + off);
        if constexpr (NEED_Y) {
          const int ln = DESC ? l - 1 : l + 1;  // saved output one step further along this scan
          if (ln >= 0 && ln < L) {
            bt.yn[u] = ld_held<VEC>(aux + base + (long long)ln * p.elem_stride);
          } else {
            bt.yn[u] = held_zero<T, VEC>();
          }
        }
      }
    }
  };
  // Own step i lies in D[i % 4] from its loads (issued during step i - 1) to its stores (during step i + 2);
  // the walk is unrolled four steps deep so that the four change roles without a register being copied.
  struct Pending {
    Lanes<VEC> ex_a, ex_b;  // G == 2, upper group: the lower group's map
    int k;                  // the step's number in the row
  };
  Batch D[4];
  Pending P[4];
  Lanes<VEC> own_out;  // what left this workgroup's previous step (every wave keeps it)
#pragma unroll
  for (int e = 0; e < VEC; ++e) own_out.v[e] = 0.0f;

  // The maps of the steps between this workgroup's previous step and step k: wave w < need asks for step
  // k - 1 - w, lane by lane the rows of the block (the lanes of the upper group ask again for the same).
  struct Words {
    uint64_t w0[VEC], w1[VEC];
  };
  auto ask = [&](int k, Words& w) __attribute__((always_inline)) {
    const int need = k < M - 1 ? k : M - 1;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      w.w0[e] = 0;
      w.w1[e] = 0;
    }
    if (wave < need) {
      const uint64_t* d = desc + 2 * ((long long)(k - 1 - wave) * RPB + rl * VEC);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        w.w0[e] = ld_desc(d + 2 * e);
        w.w1[e] = ld_desc(d + 2 * e + 1);
      }
    }
  };
  auto collect = [&](int k, Words w, int slot, int token) __attribute__((always_inline)) {
    const int need = k < M - 1 ? k : M - 1;
    if (wave >= need) return;
    auto all_there = [&]() __attribute__((always_inline)) {
      bool have = true;
#pragma unroll
      for (int e = 0; e < VEC; ++e) have = have && uint32_t(w.w0[e] >> 32) == want && uint32_t(w.w1[e] >> 32) == want;
      return __ballot(!have) == 0;
    };
    // (the first look stands in front of the loop, where the wait covers exactly the loads older than the words;
    // at the head of a loop that asks again the compiler has to wait for every load of the wave)
    if (!all_there()) {
      for (int polls = 0;; ++polls) {
        if (polls >= ch.spin_limit) {
          if (lane == 0) {
            sh_fail[slot] = token;
            __hip_atomic_fetch_add(&ch.ws->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          return;
        }
        __builtin_amdgcn_s_sleep(1);
        ask(k, w);
        if (all_there()) break;
      }
    }
    if (G == 1 || grp == 0) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        sh_pa[slot][wave][e * RL + rl] = __builtin_bit_cast(float, uint32_t(w.w0[e]));
        sh_pb[slot][wave][e * RL + rl] = __builtin_bit_cast(float, uint32_t(w.w1[e]));
      }
    }
  };
  // What enters position n_end of this lane's rows, from the rows' own data (when a wait ran out): the
  // plain sequential walk.
  auto recompute = [&](int n_end) __attribute__((always_inline)) {
    Lanes<VEC> val;
#pragma unroll
    for (int e = 0; e < VEC; ++e) val.v[e] = 0.0f;
    for (int n = 0; n < n_end; ++n) {
      const int l = DESC ? L - 1 - n : n;
      const long long off = base + (long long)l * p.elem_stride;
      const Lanes<VEC> x = ld_rows_keep<VEC>(in0 + off), c = ld_rows_keep<VEC>(coef + off);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        if constexpr (MODE == 0) val.v[e] = n == 0 ? x.v[e] : fmaf(val.v[e], c.v[e], x.v[e]);
        else val.v[e] = (val.v[e] + x.v[e]) * c.v[e];
      }
    }
    return val;
  };

  // First half of own step i (tile in D[PH], step k of the row): the lane's map, the waves' maps to LDS.
  auto scan_step = [&]<int PH>(std::integral_constant<int, PH>, int k) __attribute__((always_inline)) {
    const Batch& bt = D[PH];
    Pending& now = P[PH];
    const int n0 = k * STEP + run * U;
    Lanes<VEC> ma, mb;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      ma.v[e] = 1.0f;
      mb.v[e] = 0.0f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = n0 + u;
      if (n < L) {
        const Lanes<VEC> x = widen(bt.x[u]), c = widen(bt.c[u]);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          if constexpr (MODE == 0) {
            // the coefficient of the first position takes no part (linrec_ref.cuh:63)
            mb.v[e] = n == 0 ? x.v[e] : fmaf(mb.v[e], c.v[e], x.v[e]);
            ma.v[e] = n == 0 ? 0.0f : ma.v[e] * c.v[e];
          } else {
            mb.v[e] = (mb.v[e] + x.v[e]) * c.v[e];
            ma.v[e] *= c.v[e];
          }
        }
      }
    }
    if constexpr (G > 1) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        now.ex_a.v[e] = lanes_up_32(ma.v[e]);  // the lower group's map, which precedes the upper group's
        now.ex_b.v[e] = lanes_up_32(mb.v[e]);
        if (grp == 1) {
          mb.v[e] = fmaf(now.ex_b.v[e], ma.v[e], mb.v[e]);
          ma.v[e] = now.ex_a.v[e] * ma.v[e];
        }
      }
    }
    if (G == 1 || grp == G - 1) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        sh_a[PH][wave][e * RL + rl] = ma.v[e];
        sh_b[PH][wave][e * RL + rl] = mb.v[e];
      }
    }
    now.k = k;
  };
  // After the barrier of own step i: wave 0 publishes the whole map of the step just scanned.
  auto publish = [&]<int PH>(std::integral_constant<int, PH>, int k) __attribute__((always_inline)) {
    if (wave != 0 || (G > 1 && grp != 0) || k + 1 >= ksteps) return;
    Lanes<VEC> ta, tb;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      ta.v[e] = sh_a[PH][0][e * RL + rl];
      tb.v[e] = sh_b[PH][0][e * RL + rl];
    }
#pragma unroll 4
    for (int w = 1; w < NW; ++w) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float a = sh_a[PH][w][e * RL + rl], b = sh_b[PH][w][e * RL + rl];
        tb.v[e] = fmaf(tb.v[e], a, b);
        ta.v[e] *= a;
      }
    }
    uint64_t* d = desc + 2 * ((long long)k * RPB + rl * VEC);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      st_desc(d + 2 * e, pack_desc(want, ta.v[e]));
      st_desc(d + 2 * e + 1, pack_desc(want, tb.v[e]));
    }
  };
  // After the barrier: pending step in P[PH] (step k of the row, its waves' maps in sh_a/sh_b[PH]) gets the
  // value that enters it, is walked again from there and stored.
  auto store_step = [&]<int PH>(std::integral_constant<int, PH>, int slot, int token) __attribute__((always_inline)) {
    const Pending& q = P[PH];
    const Batch& bt = D[PH];
    const int k = q.k;
    const int need = k < M - 1 ? k : M - 1;
    // what enters the step
    Lanes<VEC> carry = own_out;  // (zero before the workgroup's first step)
    if (sh_fail[slot] == token) {
      carry = recompute(k * STEP);
    } else {
      for (int m = need - 1; m >= 0; --m) {  // oldest first
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float a = sh_pa[slot][m][e * RL + rl], b = sh_pb[slot][m][e * RL + rl];
          // before the first map of a row there is nothing: its b is taken as it is, so that 0 * inf can never arise
          carry.v[e] = (k - 1 - m == 0) ? b : fmaf(carry.v[e], a, b);
        }
      }
    }
    // what enters this lane's positions, and what leaves the step
    Lanes<VEC> entry = carry;
#pragma unroll 4
    for (int w = 0; w < NW; ++w) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float a = sh_a[PH][w][e * RL + rl], b = sh_b[PH][w][e * RL + rl];
        carry.v[e] = (k == 0 && w == 0) ? b : fmaf(carry.v[e], a, b);
      }
      if (w + 1 == wave) entry = carry;
    }
    own_out = carry;
    if constexpr (G > 1) {
      if (grp > 0) {
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          entry.v[e] = (k == 0 && wave == 0) ? q.ex_b.v[e] : fmaf(entry.v[e], q.ex_a.v[e], q.ex_b.v[e]);
      }
    }
    Lanes<VEC> val = entry;
    const int n0 = k * STEP + run * U;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = n0 + u;
      const int l = DESC ? L - 1 - n : n;
      if (n < L) {
        const long long off = base + (long long)l * p.elem_stride;
        const Lanes<VEC> x = widen(held_again(bt.x[u])), c = widen(held_again(bt.c[u]));
        if constexpr (MODE == 0) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) val.v[e] = n == 0 ? x.v[e] : fmaf(val.v[e], c.v[e], x.v[e]);
          if (active) st_rows<VEC>(out0 + off, val);
        } else {
          const Lanes<VEC> yn = widen(held_again(bt.yn[u]));
          Lanes<VEC> dx, dc;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            dx.v[e] = val.v[e] + x.v[e];
            dc.v[e] = dx.v[e] * yn.v[e];
            val.v[e] = dx.v[e] * c.v[e];
          }
          if (active) {
            st_rows<VEC>(out0 + off, dx);
            st_rows<VEC>(out1 + off, dc);
          }
        }
      }
    }
  };

  // Own step i, i % 4 == PH: step k = j + i * M of the row lies in D[PH]; D[(PH + 2) % 4] is own step i - 2,
  // stored in this step; D[(PH + 1) % 4] takes the loads of own step i + 1.
  auto step = [&]<int PH>(std::integral_constant<int, PH> ph, int i) __attribute__((always_inline)) {
    constexpr int OLD = (PH + 2) % 4, LD = (PH + 1) % 4;
    const int k = j + i * M;
    __builtin_amdgcn_sched_barrier(0);  // (nothing of this step moves up into the one before)
    Words w;
    if (i >= 2) ask(P[OLD].k, w);
    __builtin_amdgcn_sched_barrier(0);
    if (i + 1 < own) load_batch(D[LD], (k + M) * STEP + run * U);
    scan_step(ph, k);
    const int par = i & 1;
    if (i >= 2) collect(P[OLD].k, w, par, i);
    __syncthreads();
    publish(ph, k);
    if (i >= 2) store_step(std::integral_constant<int, OLD>{}, par, i);
  };
  // The last step lies in D[A] and the one before it in D[(A + 3) % 4]: nothing left to overlap with, so
  // both are asked for at once, and one barrier serves both.
  auto finish = [&]<int A>(std::integral_constant<int, A>) __attribute__((always_inline)) {
    constexpr int PREV = (A + 3) % 4;
    Words w, v;
    if (own >= 2) ask(P[PREV].k, w);
    ask(P[A].k, v);  // (published moments ago: if the words are not there yet, collect asks again)
    if (own >= 2) collect(P[PREV].k, w, 2, -2);
    collect(P[A].k, v, 3, -3);
    __syncthreads();
    if (own >= 2) store_step(std::integral_constant<int, PREV>{}, 2, -2);
    store_step(std::integral_constant<int, A>{}, 3, -3);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;

  if (own > 0) {
    load_batch(D[0], j * STEP + run * U);
    int i = 0;
    while (i + 4 <= own) {
      step(I0{}, i);
      step(I1{}, i + 1);
      step(I2{}, i + 2);
      step(I3{}, i + 3);
      i += 4;
    }
    if (i < own) { step(I0{}, i); ++i; }
    if (i < own) { step(I1{}, i); ++i; }
    if (i < own) { step(I2{}, i); ++i; }
    switch ((own - 1) % 4) {
      case 0: finish(I0{}); break;
      case 1: finish(I1{}); break;
      case 2: finish(I2{}); break;
      default: finish(I3{}); break;
    }
  }

  if (threadIdx.x == 0) {
    const uint32_t leaf_count = signal_tile_done_begin(ch, blockIdx.x);
    signal_tile_done_end(ch, blockIdx.x, seq, leaf_count);
  }
}

}  // namespace linrec
