// Column kernels: the scan axis is the strided one.  Element (r, l) lives at
// base[r*row_stride + l*elem_stride]; one lane owns VEC adjacent rows and walks the scan axis
// sequentially, keeping U timesteps of loads in flight (VEC = 16 bytes of rows: 4 floats or 8
// halves).  With row_stride == 1 (a transposed view
// of a dense tensor) the 64 lanes of a wave touch 64*VEC consecutive floats per timestep, so every
// access is a full coalesced line and no cross-lane step is needed at all.  With arbitrary strides
// (VEC == 1) the same kernel is the slow, always-correct path, the analogue of the reference's
// one-thread-per-row kernels (linrec/impl/cuda/linrec_ref.cuh:53-94).
//
// With few rows the lanes of such a launch are too few to keep the memory system busy, so the scan
// axis is cut into segments that run side by side, in three launches (PHASE template argument):
//   1  reduce: every (lane, segment) walks its segment and leaves the affine map carry_out =
//      a * carry_in + b of the whole segment;
//   -  segment_carry_kernel: one wave per row scans the row's maps and leaves the value entering
//      every segment;
//   2  apply: the plain kernel again, on one segment, starting from that value.
// The inputs are read twice (20 bytes per element forward instead of 12, 28 instead of 20
// backward), against 36 and 60 for transposing the tensors into dense rows and back.
//
// The reference has no strided kernel: it rejects inputs whose last stride is not 1
// (linrec/impl/cuda/linrec_pipe.cu:35).
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "memio.hpp"
#include "scan_primitives.hpp"

namespace linrec {

constexpr int PHASE_WHOLE = 0, PHASE_REDUCE = 1, PHASE_APPLY = 2;

struct ColumnArgs {
  const void* in0;    // forward: inputs        backward: d_outputs   (storage type T of the kernel)
  const void* coef;
  const void* aux;    // backward: saved outputs
  void* out0;         // forward: outputs       backward: d_inputs
  void* out1;         // backward: d_coeffs
  long long row_stride;
  long long elem_stride;
  long long numseq;
  int seqlen;
  long long rows_per_batch;  // row r starts at (r / rows_per_batch) * batch_stride + (r % rows_per_batch) *
  long long batch_stride;    // row_stride; rows_per_batch >= numseq: one matrix, no batch stride
  int seg_len;   // segmented launches: scan positions per segment
  int segments;  // segmented launches: lanes are numbered segment by segment, `lanes_per_segment` each, with
  long long lanes_per_segment;  // no padding between segments: a wave may hold the end of one and the start of the next
  float* maps;   // segmented launches: a[segments][numseq], then b[segments][numseq]
};

template <int VEC>
struct Lanes {
  float v[VEC];
};

template <int VEC, typename T>
__device__ __forceinline__ Lanes<VEC> ld_rows(const T* p) {
  Lanes<VEC> r;
  load_slot_full<VEC, false>(p, 0u, r.v);
  return r;
}

// The same without the streaming hint, for data that is read again soon.
template <int VEC, typename T>
__device__ __forceinline__ Lanes<VEC> ld_rows_keep(const T* p) {
  Lanes<VEC> r;
  if constexpr (VEC > 1) {
    using V = typename Pack<T, VEC>::type;
    const V q = *reinterpret_cast<const V*>(p);
#pragma unroll
    for (int i = 0; i < VEC; ++i) r.v[i] = float(q[i]);
  } else {
    r.v[0] = float(*p);
  }
  return r;
}

template <int VEC, typename T>
__device__ __forceinline__ void st_rows(T* p, const Lanes<VEC>& r) {
  store_slot_full<VEC, false>(p, 0u, r.v);
}

// MODE_FWD = 0, MODE_BWD = 1 (same numbering as the tile kernels).
template <typename T, int VEC, int U, int MODE, bool DESC, int PHASE = PHASE_WHOLE>
__global__ __launch_bounds__(256) void column_kernel(ColumnArgs p) {
  const T* in0 = static_cast<const T*>(p.in0);
  const T* coef = static_cast<const T*>(p.coef);
  const T* aux = static_cast<const T*>(p.aux);
  T* out0 = static_cast<T*>(p.out0);
  T* out1 = static_cast<T*>(p.out1);
  long long group = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // VEC rows per lane
  int seg = 0;
  if constexpr (PHASE != PHASE_WHOLE) {
    const long long s = group / p.lanes_per_segment;
    if (s >= p.segments) return;
    seg = int(s);
    group -= s * p.lanes_per_segment;
  }
  const long long r0 = group * VEC;
  if (r0 >= p.numseq) return;
  long long base = r0 * p.row_stride;  // VEC > 1 implies row_stride == 1 and rows that never straddle a batch
  if (p.rows_per_batch < p.numseq) {
    const long long batch = r0 / p.rows_per_batch;
    base = batch * p.batch_stride + (r0 - batch * p.rows_per_batch) * p.row_stride;
  }
  const int L = p.seqlen;
  // scan positions [n_begin, n_end) of this launch's lanes
  const int n_begin = PHASE == PHASE_WHOLE ? 0 : seg * p.seg_len;
  const int n_end = PHASE == PHASE_WHOLE ? L : (L - n_begin < p.seg_len ? L : n_begin + p.seg_len);
  constexpr bool NEED_Y = MODE == 1 && PHASE != PHASE_REDUCE;

  Lanes<VEC> carry;  // forward: previous output; backward: previous d_input times its coefficient
  Lanes<VEC> prod;   // reduce phase: product of the coefficients so far
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    carry.v[e] = 0.0f;
    prod.v[e] = 1.0f;
  }
  if constexpr (PHASE == PHASE_APPLY) {
    if (seg > 0) {
      const float* entering = p.maps + ((long long)p.segments + seg) * p.numseq + r0;
#pragma unroll
      for (int e = 0; e < VEC; ++e) carry.v[e] = entering[e];
    }
  }

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
      if (FULL || n < n_end) {
        const long long off = base + (long long)l * p.elem_stride;
        if constexpr (PHASE == PHASE_REDUCE) {
          // the apply phase reads these again: no streaming hint, so that what fits stays in the
          // caches (256 x 65536: 60.3 / 81.1 us against 67.3 / 92.7 us; nothing from 2^26 elements on)
          bt.x[u] = ld_rows_keep<VEC>(in0 + off);
          bt.c[u] = ld_rows_keep<VEC>(coef + off);
        } else {
          bt.x[u] = ld_rows<VEC>(in0 + off);
          bt.c[u] = ld_rows<VEC>(coef + off);
        }
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
  auto finish_batch = [&](const Batch& bt, int n0, auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = n0 + u;
      const int l = DESC ? L - 1 - n : n;
      if (FULL || n < n_end) {
        const long long off = base + (long long)l * p.elem_stride;
        if constexpr (PHASE == PHASE_REDUCE) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            if constexpr (MODE == 0) {
              carry.v[e] = n == 0 ? bt.x[u].v[e] : fmaf(carry.v[e], bt.c[u].v[e], bt.x[u].v[e]);
              prod.v[e] = n == 0 ? 0.0f : prod.v[e] * bt.c[u].v[e];
            } else {
              carry.v[e] = (carry.v[e] + bt.x[u].v[e]) * bt.c[u].v[e];
              prod.v[e] *= bt.c[u].v[e];
            }
          }
        } else if constexpr (MODE == 0) {
#pragma unroll
          for (int e = 0; e < VEC; ++e)
            carry.v[e] = n == 0 ? bt.x[u].v[e] : fmaf(carry.v[e], bt.c[u].v[e], bt.x[u].v[e]);
          st_rows<VEC>(out0 + off, carry);
        } else {
          Lanes<VEC> dx, dc;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            dx.v[e] = carry.v[e] + bt.x[u].v[e];
            dc.v[e] = dx.v[e] * bt.yn[u].v[e];
            carry.v[e] = dx.v[e] * bt.c[u].v[e];
          }
          st_rows<VEC>(out0 + off, dx);
          st_rows<VEC>(out1 + off, dc);
        }
      }
    }
  };
  using True = std::integral_constant<bool, true>;
  using False = std::integral_constant<bool, false>;

  // Batches [0, nfull) are full (for the backward the last position's successor must exist too);
  // they run double-buffered, the next batch's loads in flight while this one is scanned and stored.
  const int with_successor = NEED_Y && n_end == L ? L - 1 : n_end;
  const int nfull = PHASE == PHASE_WHOLE ? (MODE == 1 ? (L - 1) / U : L / U)
                    : with_successor > n_begin ? (with_successor - n_begin) / U : 0;
  if (nfull > 0) {
    Batch cur;
    load_batch(cur, n_begin, True{});
    for (int k = 0; k + 1 < nfull; ++k) {
      Batch nxt;
      load_batch(nxt, n_begin + (k + 1) * U, True{});
      finish_batch(cur, n_begin + k * U, True{});
      cur = nxt;
    }
    finish_batch(cur, n_begin + (nfull - 1) * U, True{});
  }
  for (int n0 = n_begin + nfull * U; n0 < n_end; n0 += U) {
    Batch tail;
    load_batch(tail, n0, False{});
    finish_batch(tail, n0, False{});
  }
  if constexpr (PHASE == PHASE_REDUCE) {
    float* ma = p.maps + (long long)seg * p.numseq + r0;
    float* mb = p.maps + ((long long)p.segments + seg) * p.numseq + r0;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      ma[e] = prod.v[e];
      mb[e] = carry.v[e];
    }
  }
}

// Segmented launches, between reduce and apply: one wave per row turns the maps of the row's
// segments into the value entering each segment, written where the map's b was.  The segments are
// taken 1024 at a time: lane i takes the 16 segments [16 i, 16 i + 16) of the chunk, the wave scans
// the 64 lane totals, and what leaves the chunk enters the next one.
template <int UNUSED = 0>  // (a template so that every translation unit that includes this file may hold a copy)
__global__ __launch_bounds__(256) void segment_carry_kernel(float* maps, long long numseq, int segments) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= numseq) return;
  float* ma = maps + row;
  float* mb = maps + (long long)segments * numseq + row;
  float chunk_in = 0.0f;  // a row starts from nothing
  for (int first = 0; first < segments; first += 1024) {
    float a[16], b[16];
    float fa[1] = {1.0f}, fb[1] = {0.0f};
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int s = first + lane * 16 + k;
      a[k] = 1.0f;
      b[k] = 0.0f;
      if (s < segments) {
        a[k] = ma[(long long)s * numseq];
        b[k] = mb[(long long)s * numseq];
      }
      fb[0] = fmaf(fb[0], a[k], b[k]);
      fa[0] *= a[k];
    }
    wave_inclusive_scan<1>(fa, fb);
    const float ex_a = shift_up_one_lane(fa[0], 1.0f);
    const float ex_b = shift_up_one_lane(fb[0], 0.0f);
    float entering = fmaf(chunk_in, ex_a, ex_b);
    chunk_in = fmaf(chunk_in, read_lane(fa[0], 63), read_lane(fb[0], 63));
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int s = first + lane * 16 + k;
      if (s < segments) mb[(long long)s * numseq] = entering;
      entering = fmaf(entering, a[k], b[k]);
    }
  }
}

}  // namespace linrec
