// Memory-only model of a drift launch (drift_kernel.hpp): the same grid of persistent workgroups in teams, the
// same tiles in the same order, loads a number of tiles ahead and stores a number of steps late with one
// workgroup barrier per step - but no scan and no exchange between workgroups.  What it takes is what the
// memory system gives the launch shape; the difference to the scan kernel's time is what scan and exchange
// cost, and the difference to the streaming kernel of linrec_stream_mix_f32 (thousands of small workgroups in
// address order) is what the launch shape costs.  A measuring instrument, not part of any scan.
//
// No counterpart in the reference.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/linrec_hip.h"
#include "memio.hpp"

namespace {

using linrec::v4f;

struct ModelArgs {
  const v4f* src[3];
  v4f* dst[2];
  long long rows;
  int tiles_per_row, team, teams;
  unsigned long long* stamps;  // per workgroup: wall clock (100 MHz) at its start and at its end, or NULL
};

// Workgroup (team, j) takes tiles j, j + team, ... of rows team, team + teams, ...: drift_kernel's walk.
template <int NW, int S, int R, int W, int AHEAD, int LATE>
__global__ __launch_bounds__(64 * NW) void launch_model_kernel(ModelArgs a) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int team = int(blockIdx.x) / a.team, j = int(blockIdx.x) - team * a.team;
  constexpr int TILE = NW * S * 64;    // slots of a tile
  constexpr int NB = AHEAD + 1;        // tiles of loaded data
  constexpr int NA = LATE + 1;         // results waiting to be stored
  constexpr int UNROLL = NB * NA;      // (a common multiple, so that every buffer index is static)
  const int per_row = a.tiles_per_row / a.team;
  const long long my_rows = team < a.rows ? (a.rows - team + a.teams - 1) / a.teams : 0;
  const int items = int(my_rows * per_row);
  if (a.stamps && threadIdx.x == 0) a.stamps[2 * blockIdx.x] = wall_clock64();
  auto base_of = [&](int it) {
    const int r = it / per_row, q = it - r * per_row;
    const long long row = team + (long long)r * a.teams;
    return (row * a.tiles_per_row + j + (long long)q * a.team) * TILE + wave * S * 64 + lane;
  };
  v4f buf[NB][R][S], acc[NA][S];
  auto load = [&](int slot, int it) {
    const long long b = base_of(it);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int s = 0; s < S; ++s) buf[slot][r][s] = __builtin_nontemporal_load(a.src[r] + b + s * 64);
  };
  auto store = [&](int slot, int it) {
    const long long b = base_of(it);
#pragma unroll
    for (int w = 0; w < W; ++w)
#pragma unroll
      for (int s = 0; s < S; ++s) __builtin_nontemporal_store(acc[slot][s], a.dst[w] + b + s * 64);
  };
#pragma unroll
  for (int q = 0; q < AHEAD; ++q)
    if (q < items) load(q, q);
  for (int n0 = 0; n0 < items; n0 += UNROLL) {
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
      const int n = n0 + k;
      if (n < items) {
        __builtin_amdgcn_sched_barrier(0);
        if (n + AHEAD < items) load((k + AHEAD) % NB, n + AHEAD);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < S; ++s) {
          acc[k % NA][s] = buf[k % NB][0][s];
#pragma unroll
          for (int r = 1; r < R; ++r) acc[k % NA][s] += buf[k % NB][r][s];
        }
        __syncthreads();
        if (n >= LATE) store((k + NA - LATE) % NA, n - LATE);
      }
    }
  }
#pragma unroll
  for (int q = LATE - 1; q >= 0; --q) {
    const int n = items - 1 - q;
    if (n >= 0) {
#pragma unroll
      for (int z = 0; z < NA; ++z)
        if (n % NA == z) store(z, n);  // (the result of step n lies in acc[n % NA])
    }
  }
  if (a.stamps) {
    __syncthreads();
    if (threadIdx.x == 0) a.stamps[2 * blockIdx.x + 1] = wall_clock64();
  }
}

struct ModelEntry {
  int waves, slots, reads, writes, ahead, late;
  const void* fn;
};
#define MODEL(NW, S, R, W, AHEAD, LATE) {NW, S, R, W, AHEAD, LATE, (const void*)&launch_model_kernel<NW, S, R, W, AHEAD, LATE>}
// the drift kernels' geometries: forward (two streams in, one out) 16 x 2, 8 x 4 and 16 x 1, backward (three in,
// two out) 16 x 1 and 8 x 2; stores two steps late as in the kernels, or at once
const ModelEntry kModels[] = {
    MODEL(16, 2, 2, 1, 1, 2), MODEL(16, 2, 2, 1, 1, 0), MODEL(16, 2, 2, 1, 2, 2), MODEL(8, 4, 2, 1, 1, 2), MODEL(8, 4, 2, 1, 1, 0),
    MODEL(16, 1, 2, 1, 1, 2), MODEL(16, 1, 2, 1, 2, 2), MODEL(16, 1, 2, 1, 2, 0),
    MODEL(16, 1, 3, 2, 2, 2), MODEL(16, 1, 3, 2, 2, 0), MODEL(16, 1, 3, 2, 1, 2), MODEL(8, 2, 3, 2, 1, 2), MODEL(8, 2, 3, 2, 2, 2),
};

}  // namespace

extern "C" int linrec_launch_model_f32(int reads, int writes, const float* src0, const float* src1, const float* src2,
                                       float* dst0, float* dst1, int64_t numseq, int64_t seqlen, int waves, int slots,
                                       int team, int ahead, int late, unsigned long long* stamps, void* stream) {
  if (numseq <= 0 || seqlen <= 0 || team <= 0 || waves <= 0 || slots <= 0) return LINREC_E_INVALID;
  const ModelEntry* m = nullptr;
  for (const ModelEntry& e : kModels)
    if (e.waves == waves && e.slots == slots && e.reads == reads && e.writes == writes && e.ahead == ahead && e.late == late) m = &e;
  if (!m) return LINREC_E_UNSUPPORTED;
  const int64_t tile = int64_t(waves) * slots * 256;  // floats
  if (seqlen % tile != 0 || (seqlen / tile) % team != 0) return LINREC_E_UNSUPPORTED;
  if (numseq * (seqlen / tile) > 2147483647LL) return LINREC_E_TOO_LARGE;
  const float* srcs[3] = {src0, src1, src2};
  float* dsts[2] = {dst0, dst1};
  ModelArgs a{};
  for (int r = 0; r < reads; ++r) {
    if (!srcs[r] || (reinterpret_cast<uintptr_t>(srcs[r]) & 15u)) return LINREC_E_INVALID;
    a.src[r] = reinterpret_cast<const v4f*>(srcs[r]);
  }
  for (int w = 0; w < writes; ++w) {
    if (!dsts[w] || (reinterpret_cast<uintptr_t>(dsts[w]) & 15u)) return LINREC_E_INVALID;
    a.dst[w] = reinterpret_cast<v4f*>(dsts[w]);
  }
  // one workgroup per compute unit, whole teams only, as the planner sizes a drift launch
  const int64_t cus = linrec_compute_units();
  if (team > cus) return LINREC_E_UNSUPPORTED;
  int64_t teams = cus / team;
  if (teams > numseq) teams = numseq;
  a.rows = numseq;
  a.tiles_per_row = int(seqlen / tile);
  a.team = team;
  a.teams = int(teams);
  a.stamps = stamps;
  void* args[] = {&a};
  hipError_t e = hipLaunchKernel(m->fn, dim3((unsigned)(teams * team)), dim3((unsigned)(64 * waves)), args, 0,
                                 static_cast<hipStream_t>(stream));
  return e == hipSuccess ? int(hipGetLastError()) : int(e);
}
