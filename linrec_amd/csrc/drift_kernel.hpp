// Drift kernels: the sweep kernels' launch shape (teams of M workgroups, one tile of a row each, that go
// on from row to row so that the whole launch reads one contiguous stretch of the tensors at any moment)
// with the exchange between team mates taken off the critical path: a tile that has been scanned is kept
// in registers and stored TWO steps later, while the next tiles are being scanned; by then the value that
// enters it has arrived without anybody having waited for it.
//
// Why the launch shape matters: the memory system spreads addresses over channels and banks by hashing
// address bits up to about bit 22.  One workgroup per row (stream_kernel.hpp) keeps rows-many reading
// positions a row length apart, all at the same offset inside their rows, so the bits that number the
// tile inside the row are the same for every access in flight: measured with a memory-only kernel, 2
// streams in and 1 out run at 5.5 TB/s with bits 15-17 constant among the accesses in flight against
// 6.5-6.6 TB/s for a dense window.  A dense window needs several tiles of one row in flight at once, hence
// workgroups that share rows, hence an exchange; what a sweep kernel loses by waiting for it in every
// step, these kernels keep.
//
// Restrictions as for the sweep kernels: 16-byte aligned bases, a row stride that keeps every row
// aligned, rows of a whole number K of tiles with M dividing K.  Every workgroup of the launch has to
// be resident at once (the planner sees to that); every wait is bounded all the same, and a wave whose
// wait runs out computes the value it needs from the row's own data.
//
// No counterpart in the reference (linrec/impl/cuda/linrec_pipe.cuh keeps a row in one block).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "tile_kernel.hpp"  // TileArgs, descriptors, completion count

namespace linrec {

// The walk.  Wave 0 publishes the map of tile n after the barrier of step n.  At the top of step n the
// waves ask for the maps that enter tile n-2 (published by the team mates a whole step ago, so they are
// there), ahead of their own loads: wave w for the 64 tiles from 64 w + 1 tiles back on, a lane each, so a
// team has up to 64 NW members.  The words arrive while tile n is scanned; every wave composes its share
// into one map and leaves it in LDS before the barrier of step n, after which every wave composes the
// shares for itself.  Nothing waits for a round trip to another workgroup.
//
// The loop is unrolled three steps deep so that the three tiles in the works (being scanned, and stored
// one and two steps from now) and the tiles of loaded data change roles without a register being copied.
// PF: tiles of loads in flight ahead of the scan (1 or 2); WPE: waves per SIMD the compiler is to allow for;
// WIDE: teams of more than 64 are served (the forward with 16 waves of two slots has no registers for that).
// RAGGED: rows of whole slots whose last tile is a partial one (K = tiles of a row, the last one counted): that
// tile takes the loads and stores that look at every slot, the others stay as they are; the team need not divide K,
// and the walk's start moves on by K % M tiles in every row, so that neither the partial tiles nor the longer walks
// all fall to the same team mates.
template <typename T, int NW, int S, int VEC, int MODE, bool DESC, int PF, int WPE = 1, bool WIDE = true, bool RAGGED = false>
__global__ __launch_bounds__(64 * NW, WPE) void drift_kernel(TileArgs p) {
  static_assert(PF == 1 || PF == 2, "one or two tiles of loads ahead of the scan");
  static_assert(NW <= 16, "the waves' shares are composed inside a DPP row");
  constexpr int WAVE_SLOTS = S * 64;
  constexpr int TILE_SLOTS = NW * WAVE_SLOTS;
  __shared__ float sh_a[2][NW];
  __shared__ float sh_b[2][NW];
  // what the waves collected of the team mates' maps: steps alternate between [0] and [1]; [2] and [3]
  // are the last two tiles'
  __shared__ float sh_pa[4][NW];
  __shared__ float sh_pb[4][NW];
  __shared__ int sh_fail[4];     // the step (1 for the last two tiles) in which a wave's wait ran out
  __shared__ float sh_carry[4];  // then: the value computed from the row's own data instead

  const int lane = threadIdx.x & 63;
  const int wave = NW == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int M = p.tasks;          // team size; divides K unless RAGGED
  const int K = p.tiles_per_row;  // every row is exactly K full tiles
  const int teams = int(p.row_groups);  // the grid is teams * M workgroups
  const int team = int(blockIdx.x) / M;
  const int j = int(blockIdx.x) - team * M;
  const int per_row = K / M;  // tiles of one row this walker takes: j, j + M, ...
  const long long my_rows = team < p.numseq ? (p.numseq - team + teams - 1) / teams : 0;
  int items = int(my_rows * per_row);
  const int rem = K - per_row * M;  // RAGGED: the team need not divide K
  if constexpr (RAGGED) {
    // A walk that starts at tile s < M takes one tile more than K / M where s < rem.  The starts of this walker's rows
    // are j, j + rem, j + 2 rem, ... (mod M), which come to lie below rem once in every M / rem rows, evenly spaced (a
    // walker that took the longer walk several rows running would fall behind its team mates by as many steps): as
    // often as the sum passes a multiple of M.
    if (my_rows > 0) items += (j < rem ? 1 : 0) + int((j + (my_rows - 1) * rem) / M);
  }

  // (read through the scalar cache: it arrives beside the first tile's loads instead of holding them up, which an
  // agent-scope load did for a memory round trip at the start of every launch)
  const uint32_t seq = load_seq_through_caches(p.ws);
  if (threadIdx.x < 4) sh_fail[threadIdx.x] = 0;  // (every reader has passed a step's barrier first)
  const RowView rv = make_row_view<VEC>(0, 0, p.seqlen);

  struct Item {
    int row;
    int t;
  };
  // the walk: tiles j, j + M, ... of row `team`, then of row team + teams, ...
  Item cursor = {team, j};
  int turn = 0;  // RAGGED: how far the walk's start has moved on from j, K % M tiles a row
  auto next_item = [&]() {
    const Item it = cursor;
    cursor.t += M;
    if (cursor.t >= K) {
      if constexpr (RAGGED) {
        turn = turn + rem >= M ? turn + rem - M : turn + rem;
        cursor.t = j + turn >= M ? j + turn - M : j + turn;
      } else {
        cursor.t = j;
      }
      cursor.row += teams;
    }
    return it;
  };
  auto ptrs_of = [&](int row) {
    return make_row_ptrs<T, MODE>(p.in0, p.coef, p.aux, p.out0, p.out1, (long long)row * p.row_stride, 0);
  };

  // 16-bit storage: the tiles whose loads are in flight, and a pending tile's saved outputs, stay in the storage
  // type until their step comes (half the registers, and no conversion that would have to wait for the loads in
  // the step that issues them).
  constexpr bool PACKED = !std::is_same_v<T, float>;
  // ... and the forward keeps a scanned tile as its packed inputs plus each slot's map, and scans the elements a second
  // time when it stores them: a quarter of the registers of the elements' maps, which is what lets a lane hold two
  // slots of eight elements (a step then moves as many bytes as the fp32 kernels')
  constexpr bool REPLAY = PACKED && MODE == MODE_FWD;
  // With two slots to a lane even the packed inputs of three tiles are more than the registers hold: a scanned tile's
  // packed inputs wait in LDS (every lane its own 16-byte places: no conflicts, no barrier), which the kernel otherwise
  // leaves unused: two tiles of 64 KB.
  constexpr bool PARKED = REPLAY && S >= 2;
  using Packed16 = typename Pack<T, PACKED ? VEC : 4>::type;
  __shared__ Packed16 sh_park[PARKED ? 2 * NW * S * 2 * 64 : 1];
  using Loaded = std::conditional_t<PACKED, TilePacked<T, S, VEC, MODE>, TileData<S, VEC, MODE>>;
  // A tile that has been scanned and not stored yet.
  struct Pending {
    Loaded d;    // (what the store still needs of it: the saved outputs, backward)
    float edge;  // 16-bit storage, backward: the saved output after the wave's last, wave-uniform (a scalar register)
    TileScan<S, VEC> r;
    Affine before;  // the waves in front of this one
    Affine total;   // the whole tile's map
    Item it;
    int park;       // where its packed inputs wait in LDS (0 or 1)
  };
  Loaded D[3];  // tile n lies in D[n % 3]
  Item DI[3];
  Pending P[3];                 // and becomes P[n % 3]

  float own_out = 0.0f;  // value that left this walker's previous tile of the current row (wave 0; every wave in teams of more than 64)

  // This wave's share of the maps in front of tile `it`: lane i holds tile t - 1 - (64 wave + i).
  auto ask = [&](const Item& it, uint64_t& w0, uint64_t& w1) {
    const int t = it.t;
    const int need = t < M - 1 ? t : M - 1;
    const int i = 64 * wave + lane;
    w0 = 0;
    w1 = 0;
    if (i < need) {
      const uint64_t* desc = p.desc + 2 * ((long long)it.row * K);
      const long long idx = t - 1 - i;
      w0 = ld_desc(desc + 2 * idx);
      w1 = ld_desc(desc + 2 * idx + 1);
    }
  };
  // A team of at most 64: wave 0 holds all the maps and has the value entering the tile in LDS before the
  // barrier; the others only read it afterwards.  Larger teams: every wave leaves its share in LDS before
  // the barrier and composes all the shares for itself after it.
  const bool wide = WIDE && M > 64;
  // Before the barrier: the words asked for (asked for again while a team mate is more than two steps
  // behind) composed, oldest first.  A wait that runs out: wave 0 of a team of at most 64 computes the
  // value from the row's own data on the spot; in a larger team the wave notes it in LDS and the workgroup
  // does so after the barrier.
  auto collect = [&](const Pending& q, uint64_t w0, uint64_t w1, int slot, int token) {
    const Item it = q.it;
    const int t = it.t;
    const int need = t < M - 1 ? t : M - 1;
    const int mine = need - 64 * wave < 64 ? need - 64 * wave : 64;  // maps this wave holds
    if (wide ? mine <= 0 : wave != 0) return;
    Affine acc = {1.0f, 0.0f};
    bool ok = true;
    if (mine > 0) {
      const uint32_t want = (seq << 2) | STATUS_AGGREGATE;
      // The first look at the words stands in front of the loop.  Inside it the words may be the wave's newest
      // loads (the loop asks again), so at its head the compiler has to wait for every load of the wave, the
      // tile just asked for included (a step's worth of memory latency, in every step: 1.7 us of wave 0's 3.8 us
      // step on 512 x 65536 forward, with all other waves waiting at the barrier); in front of it the wait
      // covers exactly the loads older than the words.
      bool have = lane >= mine || (uint32_t(w0 >> 32) == want && uint32_t(w1 >> 32) == want);
      if (__ballot(!have) != 0) {
        for (int polls = 0;; ++polls) {
          if (polls >= p.spin_limit) {
            ok = false;
            break;
          }
          __builtin_amdgcn_s_sleep(1);
          ask(it, w0, w1);
          have = lane >= mine || (uint32_t(w0 >> 32) == want && uint32_t(w1 >> 32) == want);
          if (__ballot(!have) == 0) break;
        }
      }
      if (ok) {
        // towards lane 0: inside each row of 16 lanes by DPP, which leaves a row's composition in its lane
        // 0; then the up to four rows, the highest lanes first
        float a[1] = {lane < mine ? __builtin_bit_cast(float, uint32_t(w0)) : 1.0f};
        float b[1] = {lane < mine ? __builtin_bit_cast(float, uint32_t(w1)) : 0.0f};
        scan_step<DPP_ROW_SHL1, 0xf>(a, b);
        scan_step<DPP_ROW_SHL2, 0xf>(a, b);
        scan_step<DPP_ROW_SHL4, 0xf>(a, b);
        scan_step<DPP_ROW_SHL8, 0xf>(a, b);
        acc = {read_lane(a[0], 0), read_lane(b[0], 0)};
        if (mine > 16) {
          Affine far = {read_lane(a[0], 16), read_lane(b[0], 16)};
          if (mine > 32) far = compose({read_lane(a[0], 32), read_lane(b[0], 32)}, far);
          if (mine > 48) far = compose({read_lane(a[0], 48), read_lane(b[0], 48)}, far);
          acc = compose(far, acc);
        }
      } else if (lane == 0) {
        __hip_atomic_fetch_add(&p.ws->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (wide) {
      if (lane == 0) {
        if (ok) {
          sh_pa[slot][wave] = acc.a;
          sh_pb[slot][wave] = acc.b;
        } else {
          sh_fail[slot] = token;
        }
      }
      return;
    }
    float carry_in = 0.0f;
    if (t > 0) {
      if (!ok) carry_in = recompute_entry<VEC, MODE, DESC>(ptrs_of(it.row), rv, t * TILE_SLOTS, lane);
      else if (t < M) carry_in = acc.b;  // the maps reach back to the row start
      else carry_in = need > 0 ? fmaf(own_out, acc.a, acc.b) : own_out;
    }
    own_out = t == 0 ? q.total.b : fmaf(carry_in, q.total.a, q.total.b);
    if (lane == 0) sh_carry[slot] = carry_in;
  };
  // After the barrier: the value entering pending tile `q` (in a team of more than 64, composed by every
  // wave alike from the shares).
  auto combine = [&](const Pending& q, int slot, int token) -> float {
    if (!wide) return sh_carry[slot];
    const int t = q.it.t;
    const int need = t < M - 1 ? t : M - 1;
    float carry_in = 0.0f;
    if (t > 0) {
      if (sh_fail[slot] == token) {  // (the same for the whole workgroup)
        if (wave == 0) {
          const float c = recompute_entry<VEC, MODE, DESC>(ptrs_of(q.it.row), rv, t * TILE_SLOTS, lane);
          if (lane == 0) sh_carry[slot] = c;
        }
        __syncthreads();
        carry_in = sh_carry[slot];
      } else {
        const int shares = (need + 63) >> 6;  // wave w's share lies further back than wave w-1's
        float a[1] = {1.0f}, b[1] = {0.0f};
        if (lane < shares) {
          a[0] = sh_pa[slot][lane];
          b[0] = sh_pb[slot][lane];
        }
        if constexpr (NW > 1) scan_step<DPP_ROW_SHL1, 0xf>(a, b);
        if constexpr (NW > 2) scan_step<DPP_ROW_SHL2, 0xf>(a, b);
        if constexpr (NW > 4) scan_step<DPP_ROW_SHL4, 0xf>(a, b);
        if constexpr (NW > 8) scan_step<DPP_ROW_SHL8, 0xf>(a, b);
        const Affine acc = {read_lane(a[0], 0), read_lane(b[0], 0)};
        carry_in = t < M ? acc.b : fmaf(own_out, acc.a, acc.b);  // (up to the row start the maps reach back all the way)
      }
    }
    own_out = t == 0 ? q.total.b : fmaf(carry_in, q.total.a, q.total.b);
    if constexpr (PACKED) own_out = read_lane(own_out, 0);  // (wave-uniform: a scalar register, where vector registers are short)
    return carry_in;
  };
  auto store_pending = [&](const Pending& q, float tile_in) {
    const int t = q.it.t;
    bool has_entry = false;
    float entry = 0.0f;
    if (t > 0) {
      has_entry = true;
      entry = wave == 0 ? tile_in : fmaf(tile_in, q.before.a, q.before.b);
    } else if (wave > 0) {
      has_entry = true;
      entry = q.before.b;
    }
    if constexpr (PARKED) {
      Loaded k;
      const Packed16* from = sh_park + ((q.park * NW + wave) * S * 2) * 64 + lane;
#pragma unroll
      for (int j = 0; j < S; ++j) {
        k.xs[j] = from[(2 * j) * 64];
        k.cs[j] = from[(2 * j + 1) * 64];
      }
      tile_replay_store_packed<S, VEC, DESC, RAGGED>(k, q.r, t == 0 && wave == 0 && lane == 0, ptrs_of(q.it.row), rv,
                                                     t * TILE_SLOTS + wave * WAVE_SLOTS, lane, has_entry, entry);
    } else if constexpr (REPLAY) {
      tile_replay_store_packed<S, VEC, DESC, RAGGED>(q.d, q.r, t == 0 && wave == 0 && lane == 0, ptrs_of(q.it.row), rv,
                                                     t * TILE_SLOTS + wave * WAVE_SLOTS, lane, has_entry, entry);
    } else if constexpr (PACKED) {
      tile_apply_store_packed<S, VEC, MODE, DESC, RAGGED>(q.d.ys, q.edge, q.r, ptrs_of(q.it.row), rv,
                                                          t * TILE_SLOTS + wave * WAVE_SLOTS, lane, has_entry, entry);
    } else {
      if (RAGGED && t == K - 1)
        tile_apply_store<S, VEC, MODE, DESC, false>(q.d, q.r, ptrs_of(q.it.row), rv, t * TILE_SLOTS + wave * WAVE_SLOTS,
                                                    lane, has_entry, entry);
      else
        tile_apply_store<S, VEC, MODE, DESC, true>(q.d, q.r, ptrs_of(q.it.row), rv, t * TILE_SLOTS + wave * WAVE_SLOTS,
                                                   lane, has_entry, entry);
    }
  };
  auto load_next = [&](Loaded& d, Item& it) {
    it = next_item();
    if constexpr (PACKED)  // (16-bit storage: a slot either lies in the row or beyond its end, every tile asks)
      tile_load_packed<S, VEC, MODE, DESC, RAGGED>(d, ptrs_of(it.row), rv, it.t * TILE_SLOTS + wave * WAVE_SLOTS, lane);
    else if (RAGGED && it.t == K - 1)
      tile_load<S, VEC, MODE, DESC, false>(d, ptrs_of(it.row), rv, it.t * TILE_SLOTS + wave * WAVE_SLOTS, lane, false);
    else
      tile_load<S, VEC, MODE, DESC, true>(d, ptrs_of(it.row), rv, it.t * TILE_SLOTS + wave * WAVE_SLOTS, lane, false);
  };

  // Step n, n % 3 == PH: tile n lies in D[PH]; P[(PH + 1) % 3] is tile n-2, stored in this step.
  auto step = [&]<int PH>(std::integral_constant<int, PH>, int n, bool prefetch) {
    constexpr int OLD = (PH + 1) % 3, LD = (PH + PF) % 3;
    __builtin_amdgcn_sched_barrier(0);  // (nothing of this step moves up into the one before)
    uint64_t w0 = 0, w1 = 0;
    if (n >= 2 && (wide || wave == 0)) ask(P[OLD].it, w0, w1);
    __builtin_amdgcn_sched_barrier(0);
    if (prefetch) load_next(D[LD], DI[LD]);
    const Item it = DI[PH];
    Pending& now = P[PH];
    if constexpr (REPLAY) {
      tile_scan_packed_fwd<S, VEC, DESC>(D[PH], it.t == 0 && wave == 0 && lane == 0, now.r);
      if constexpr (!PARKED) now.d = D[PH];
    } else {
      TileData<S, VEC, MODE> unpacked;
      TileData<S, VEC, MODE>& d = [&]() -> TileData<S, VEC, MODE>& {
        if constexpr (PACKED) {
          tile_unpack<S, VEC, MODE, DESC>(D[PH], unpacked);
          return unpacked;
        } else {
          return D[PH];
        }
      }();
      if constexpr (MODE == MODE_FWD) {
        if (it.t == 0 && wave == 0 && lane == 0) d.cs[0][0] = 0.0f;  // the row's first coefficient takes no part
      }
      tile_scan<S, VEC, MODE>(d, now.r);
      if constexpr (MODE == MODE_FWD || PACKED) {
        // a slot's map from the wave's entry value to the slot's is folded into the elements' maps, which leaves
        // a pending tile two values per element and nothing per slot (16 waves have 128 registers each); nothing
        // enters a row's first wave, whose factors are therefore zero and never meet a product that overflowed
        // (the backward, whose first factor of a slot is one before the folding, only for 16-bit storage, where it
        // saves a register for each of the three tiles in the works)
        const bool nothing_enters = it.t == 0 && wave == 0;
#pragma unroll
        for (int j = 0; j < S; ++j) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            now.r.pb[j][i] = fmaf(now.r.pa[j][i], now.r.ex_b[j], now.r.pb[j][i]);
            now.r.pa[j][i] = nothing_enters ? 0.0f : now.r.pa[j][i] * now.r.ex_a[j];
          }
          now.r.ex_a[j] = 1.0f;
          now.r.ex_b[j] = 0.0f;
        }
      }
      if constexpr (MODE == MODE_BWD) {
        now.d = D[PH];
        if constexpr (PACKED) now.edge = read_lane(d.y_edge, 63);  // (only lane 63 holds it, only lane 63 uses it)
      }
    }
    const int par = n & 1;
    if (lane == 0) {
      sh_a[par][wave] = now.r.total.a;
      sh_b[par][wave] = now.r.total.b;
    }
    if (n >= 2) collect(P[OLD], w0, w1, par, n);
    __syncthreads();
    wave_prefixes<NW>(sh_a[par], sh_b[par], wave, lane, now.before, now.total);
    if (wave == 0) {
      if (lane == 0 && it.t + 1 < K) {
        uint64_t* desc = p.desc + 2 * ((long long)it.row * K);
        st_desc(desc + 2 * (long long)it.t, pack_desc((seq << 2) | STATUS_AGGREGATE, now.total.a));
        st_desc(desc + 2 * (long long)it.t + 1, pack_desc((seq << 2) | STATUS_AGGREGATE, now.total.b));
      }
    }
    if (n >= 2) {
      const float tile_in = combine(P[OLD], par, n);
      store_pending(P[OLD], tile_in);
    }
    if constexpr (PARKED) {
      // (into the place the tile just stored has left)
      now.park = n & 1;
      Packed16* to = sh_park + ((now.park * NW + wave) * S * 2) * 64 + lane;
#pragma unroll
      for (int j = 0; j < S; ++j) {
        to[(2 * j) * 64] = D[PH].xs[j];
        to[(2 * j + 1) * 64] = D[PH].cs[j];
      }
    }
    now.it = it;
  };
  // The last tile lies in P[A] and the one before it in P[(A + 2) % 3]: nothing left to overlap with, so
  // both are asked for at once, and one barrier serves both.
  auto finish = [&]<int A>(std::integral_constant<int, A>) {
    constexpr int PREV = (A + 2) % 3;
    uint64_t w0 = 0, w1 = 0, v0 = 0, v1 = 0;
    if (items >= 2 && (wide || wave == 0)) ask(P[PREV].it, w0, w1);
    if (wide || wave == 0) ask(P[A].it, v0, v1);  // (published moments ago: if the words are not there yet, collect asks again)
    if (items >= 2) collect(P[PREV], w0, w1, 2, 1);
    collect(P[A], v0, v1, 3, 1);
    __syncthreads();
    if (items >= 2) {
      const float tile_in = combine(P[PREV], 2, 1);
      store_pending(P[PREV], tile_in);
    }
    const float tile_in = combine(P[A], 3, 1);
    store_pending(P[A], tile_in);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;

  if (items > 0) {
    load_next(D[0], DI[0]);
    if (PF == 2 && items > 1) load_next(D[1], DI[1]);
    int n = 0;
    // every step of this loop has a tile to load ahead
    while (n + PF + 2 < items) {
      step(I0{}, n, true);
      step(I1{}, n + 1, true);
      step(I2{}, n + 2, true);
      n += 3;
    }
    // at most PF + 2 steps are left, the first at n % 3 == 0
    if (n < items) { step(I0{}, n, n + PF < items); ++n; }
    if (n < items) { step(I1{}, n, n + PF < items); ++n; }
    if (n < items) { step(I2{}, n, n + PF < items); ++n; }
    if (n < items) { step(I0{}, n, false); ++n; }
    switch ((items - 1) % 3) {
      case 0: finish(I0{}); break;
      case 1: finish(I1{}); break;
      default: finish(I2{}); break;
    }
  }

  if (threadIdx.x == 0) {
    const uint32_t leaf_count = signal_tile_done_begin(p, blockIdx.x);
    signal_tile_done_end(p, blockIdx.x, seq, leaf_count);
  }
}

}  // namespace linrec
