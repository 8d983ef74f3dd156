// C ABI, kernel table and launch planning of the gfx950 linear-recurrence scan library.
// Declarations and the reference interfaces they replace: include/linrec_hip.h.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

#include "../../include/linrec_hip.h"
#include "kernel_table.hpp"
#include "colblock_kernel.hpp"
#include "coldrift_kernel.hpp"
#include "column_kernel.hpp"
#include "flat_kernel.hpp"
#include "drift_kernel.hpp"
#include "group_kernel.hpp"
#include "chain_kernel.hpp"
#include "stream_kernel.hpp"
#include "sweep_kernel.hpp"
#include "team_kernel.hpp"
#include "tile_kernel.hpp"

// Scratch of linrec_fwd_noalloc, the entry point for callers that cannot allocate: every GPU the library
// runs on holds one copy of this array, at its own address, until the process ends.  In host code the
// name is only a handle for hipGetSymbolAddress (device_state() below keeps the address per device);
// kernels and copies are given that address, never the name.  It starts out zero-filled, which is the
// state a look-back workspace has to be in before its first launch, and every launch leaves it usable
// for the next (the counters end at zero, the launch counter moves on).
constexpr size_t kStaticScratchBytes = LINREC_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

using linrec::ColumnArgs;
using linrec::TileArgs;

// ---- kernel table ---------------------------------------------------------------------------
// The reference compiles 116 configurations of 4 kernels and matches a runtime tuple against them
// (linrec/impl/cuda/linrec.h:8-13, dispatch.h:53-72).  Here the table is a plain array of instantiations
// (kernel_table.hpp), compiled in groups (kernels_*.hip) and put together once when the library is loaded;
// the planner below picks one entry from the problem shape.
using linrec::KernelEntry;
const std::vector<KernelEntry> g_kernel_table = [] {
  std::vector<KernelEntry> all;
  for (const linrec::KernelGroup g : {linrec::kernels_f32_rows(), linrec::kernels_f32_walk(), linrec::kernels_f32_teams(), linrec::kernels_f32_cols(),
                                      linrec::kernels_f16_rows(), linrec::kernels_f16_cols(), linrec::kernels_bf16_rows(),
                                      linrec::kernels_bf16_cols()})
    all.insert(all.end(), g.entries, g.entries + g.count);
  return all;
}();
const KernelEntry* const kKernels = g_kernel_table.data();
const int kNumKernels = int(g_kernel_table.size());

int find_kernel(int dtype, int family, int waves, int slots, int vec, int mode, int desc, int carry) {
  for (int i = 0; i < kNumKernels; ++i) {
    const KernelEntry& k = kKernels[i];
    const bool waves_matter = family == LINREC_FAMILY_TILE || family == LINREC_FAMILY_STREAM ||
                              family == LINREC_FAMILY_TEAM || family == LINREC_FAMILY_SWEEP || family == LINREC_FAMILY_DRIFT || family == LINREC_FAMILY_GROUP ||
                              family == LINREC_FAMILY_FLAT || family == LINREC_FAMILY_COLDRIFT;
    if (k.dtype == dtype && k.family == family && k.slots == slots && k.vec == vec && k.mode == mode &&
        k.desc == desc && k.carry == carry && (!waves_matter || k.waves == waves))
      return i;
  }
  return -1;
}

// ---- the device ------------------------------------------------------------------------------
// What the planner needs to know about the device a call runs on, asked once per device (the
// reference asks through cudaDeviceGetAttribute, linrec/impl/cuda/cuhelpers.cuh:23-34, on every
// launch, linrec_pipe.cu:72-80): the number of compute units, how many workgroups of a kernel one CU
// holds, and where this device keeps its copy of the static scratch array.
constexpr int kDefaultComputeUnits = 256;  // MI355X; assumed when a plan is asked for on a host without a GPU
constexpr int kMaxDevices = 64;

struct DeviceState {
  std::once_flag once;
  int cus = 0;                  // hipDeviceAttributeMultiprocessorCount
  void* scratch_ptr = nullptr;  // this device's address of `scratch`
  int scratch_rc = -1;          // hipError_t of the hipGetSymbolAddress call that produced it
  std::mutex occupancy_mutex;
  std::vector<int8_t> occupancy;  // per kernel id: workgroups one CU holds, 0 = not asked yet
};
DeviceState g_devices[kMaxDevices];
std::atomic<int> g_cu_override{0};

// The state of the current device, set up by the first call made with that device current; nullptr if
// there is no device to ask.
DeviceState* device_state() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  DeviceState& d = g_devices[dev];
  std::call_once(d.once, [&] {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) d.cus = n;
    else (void)hipGetLastError();
    d.scratch_rc = int(hipGetSymbolAddress(&d.scratch_ptr, HIP_SYMBOL(scratch)));
    if (d.scratch_rc != 0) {
      (void)hipGetLastError();
      d.scratch_ptr = nullptr;
    }
  });
  return &d;
}

// Workgroups of kernel `id`, `block` lanes each, that one CU holds at a time; `assumed` when there is no
// device to ask (or a test has overridden the CU count).
int workgroups_per_cu(int id, int block, int assumed) {
  DeviceState* d = g_cu_override.load(std::memory_order_relaxed) > 0 ? nullptr : device_state();
  if (!d || d->cus <= 0) return assumed;
  std::lock_guard<std::mutex> lock(d->occupancy_mutex);
  if (d->occupancy.empty()) d->occupancy.assign(size_t(kNumKernels), 0);
  if (d->occupancy[id] == 0) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kKernels[id].fn, block, 0) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      n = -1;
    }
    d->occupancy[id] = int8_t(std::min(n, 127));
  }
  return d->occupancy[id] > 0 ? d->occupancy[id] : assumed;
}

int compute_units() {
  const int forced = g_cu_override.load(std::memory_order_relaxed);
  if (forced > 0) return forced;
  const DeviceState* d = device_state();
  return d && d->cus > 0 ? d->cus : kDefaultComputeUnits;
}

// ---- planning -------------------------------------------------------------------------------
struct Problem {
  int64_t numseq, seqlen, row_stride, elem_stride;
  int reverse, is_bwd;
  int base_mis;     // common misalignment of the bases in elements, or -1 if they disagree
  bool aligned16;   // every base is 16-byte aligned
  int dtype;        // LINREC_DTYPE_*
  int col_phase;    // misalignment of the bases in elements modulo a 16-byte slot (column kernels)
  // batches of matrices whose rows do not continue from one matrix into the next: row r starts at
  // (r / rows_per_batch) * batch_stride + (r % rows_per_batch) * row_stride; 0 = one matrix
  int64_t rows_per_batch = 0, batch_stride = 0;
  // Compute units of the device the call runs on.  Every row-count threshold below was measured on the
  // full part (256 CUs) and is kept as that number; at() scales it to the device in hand, since what a
  // threshold stands for is a number of workgroups or waves per CU.
  int64_t cus = 256;
  int64_t at(int64_t measured_on_256) const { return measured_on_256 * cus / 256; }
  // The most workspace the caller can give (0: any): the planner leaves out what would need more where
  // another kernel serves the problem with less.
  size_t workspace_cap = 0;
  bool batched() const { return rows_per_batch > 0 && rows_per_batch < numseq; }
};

int elem_size_of(int dtype) { return dtype == LINREC_DTYPE_F32 ? 4 : 2; }
int full_vec_of(int dtype) { return 16 / elem_size_of(dtype); }

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Stream kernels take over from tiles for rows of more than 2048 slots once there are enough rows
// to give every CU work.
constexpr int64_t kLongRowSlots = 2048;  // 8192 floats, 16384 halves

// The crossovers between the long-row kernels come from a generated table (plan_thresholds.inc, written by the
// tuning harness from timings on the device): kT_<name> below, and by name through linrec_plan_threshold.
struct PlanThreshold {
  const char* name;
  int64_t value;
};
#define LINREC_THRESHOLD(name, value) constexpr int64_t kT_##name = value;
#include "plan_thresholds.inc"
#undef LINREC_THRESHOLD
#define LINREC_THRESHOLD(name, value) {#name, value},
constexpr PlanThreshold kPlanThresholds[] = {
#include "plan_thresholds.inc"
};
#undef LINREC_THRESHOLD
constexpr int kNumPlanThresholds = int(sizeof(kPlanThresholds) / sizeof(kPlanThresholds[0]));

constexpr int64_t kStreamMinRows = kT_stream_min_rows;   // (these three on 256 CUs; scaled by Problem::at)
constexpr int64_t kSplitBelowRows = 192;  // rows of a few thousand elements are cut into look-back tiles below this
                                          // (launches of a few microseconds: the tuning sweep, which times launches from the host, cannot tell them apart)
constexpr int64_t kSweepBelowRows = 192;  // sweep kernels take 16 .. 191 rows, stream kernels 192 .. 256
// Fewer long rows: teams of workgroups per row, sized so that at most one workgroup per CU runs
// (measured at 2^24 elements, forward: 128 rows x2 38 us, 64 x4 39 us, 32 x8 40 us, 16 x16 42 us,
// 8 x32 45 us, against 46-51 us for one look-back tile per workgroup; below that, teams of at most
// 64 leave CUs idle and look-back tiles win).  A team size that overshoots 256 workgroups puts two
// on some CUs and everybody waits for those: 96 x 65540 teams of 3 25.0 / 38.5 us, teams of 2
// 22.2 / 32.2 us; 120 x 131076 teams of 3 51.8 / 77.4 us, teams of 2 41.1 / 65.9 us; above 128
// rows one workgroup per row does better than teams of 2 (160 x 65540: 32.7 / 50.2 us against
// 35.7 / 55.3 us).
// Sweep kernels: workgroups of a launch, two per CU forward; the backward kernels hold more
// registers and fit one per CU.
int64_t sweep_workgroups(const Problem& q) { return q.is_bwd ? q.cus : 2 * q.cus; }
constexpr int64_t kSweepMaxTeam = 16;
constexpr int64_t kSweepMinTiles = 4;  // tiles per row below which the exchange costs more than it brings

// Team kernels: one workgroup per CU.
int64_t team_workgroups(const Problem& q) { return q.cus; }

// Largest divisor of `tiles_per_row` that is at most `most`.
int64_t sweep_team_size(int64_t tiles_per_row, int64_t most = kSweepMaxTeam) {
  for (int64_t m = most; m > 1; --m)
    if (tiles_per_row % m == 0) return m;
  return 1;
}

// Drift kernels (fp32): the sweep launch shape without the wait for the exchange.  Measured against the
// table's previous choice, forward / backward in us: 512 x 65536 67.9 / 113.3 against 70.7 (stream) / 120.7
// (sweep); 288 x 65536 40.2 / 65.6 against 44.3 / 68.1; 1024 x 65536 132.5 / 224.8 against 138.0 / 233.0;
// 1024 x 32768 68.3 / 114.0 against 72.9 / 118.8; 2048 x 16384 69.1 / 114.4 against 70.4 / 120.2;
// 160 x 131072 44.8 / 73.8 against 47.9 / 78.5; 128 x 262144 69.4 / 116.3 against 78.7 / 119.9;
// forward only: 16 x 1048576 40.3 against 43.5, 64 x 524288 70.0 against 78.0, 32 x 1048576 72.9 against
// 81.9, 512 x 262144 260.9 against 279.1.  Fewer than 16 rows, where teams of more than 64 come in (against
// look-back tiles, or the sweep kernels from 6 rows on): 1 x 33554432 73.6 / 120.2 against 101.9 / 142.4,
// 3 x 8388608 58.2 / 91.7 against 82.4 / 112.2, 4 x 8388608 71.8 / 120.5 against 101.9 / 143.2,
// 6 x 4194304 56.0 / 91.4 against 62.0 (teams of 64) / 107.9, 8 x 4194304 71.4 / 120.0 against 73.4 (teams of
// 64) / 135.1.  Left to the others: more than 2048 rows (4096 x 65536 553 / 959 against 548 / 948), and the
// backward of 16 to 127 rows or of rows longer than 131072 (16 x 1048576 62.8 against 62.0, 32 x 1048576
// 121.1 against 121.6, 64 x 524288 118.8 against 118.4, 512 x 262144 459.7 against 450.8), where tiles of
// 16384 elements, which a drift kernel has no registers for, do as well or better.
//
// The team for rows of `tiles_per_row` tiles: the divisor of it that keeps most of the chip busy (whole
// teams only, every team the same number of rows where that is possible), the larger one of equals: the
// more of a row is in flight at once, the fewer gaps the launch's reading positions leave.  A lane of a
// wave per team mate: at most 64 a wave.
int64_t drift_team_size(const Problem& q, int64_t tiles_per_row, int waves, int64_t resident, bool any_team = false,
                        int64_t max_team = 0) {
  int64_t best = 1, best_large = 0;
  double best_busy = 0.0, best_large_busy = 0.0;
  if (max_team <= 0) max_team = int64_t(64) * waves;
  for (int64_t team = std::min<int64_t>({max_team, resident, tiles_per_row}); team >= 1; --team) {
    // (the kernels for rows with a partial last tile take teams that do not divide the tiles of a row)
    if (tiles_per_row % team != 0 && !any_team) continue;
    const int64_t teams = std::min(q.numseq, resident / team);
    const int64_t rounds = ceil_div(q.numseq, teams);
    // (a team that does not divide the tiles of a row: over the rows of a team some members take a tile more than others,
    // and the members are never all in step - 1024 x 50000, seven tiles a row, in teams of 4 113.0 / 192.4 us, in teams
    // of 7 108.0 / 174.9 us; 335 x 100000 backward, 25 tiles, in teams of 16 116.8 to 123.5 us, of 25 114.4 us)
    const int64_t most = rounds * (tiles_per_row / team) + ceil_div(rounds * (tiles_per_row % team), team);
    const double busy = double(q.numseq * team) / double(rounds * resident) *
                        (double(rounds * tiles_per_row) / double(team * most)) * (tiles_per_row % team ? 0.93 : 1.0);
    // (of such teams the larger one unless a smaller one keeps the chip 3 % busier: more of a row in flight at once)
    if (busy > best_busy * (any_team && best_busy > 0.0 ? 1.03 : 1.0) + 1e-9) {
      best = team;
      best_busy = busy;
    }
    if (team >= kSweepMinTiles && busy > best_large_busy + 1e-9) {
      best_large = team;
      best_large_busy = busy;
    }
  }
  // (a team too small to be worth the exchange only where no larger one keeps the chip nearly as busy)
  return best < kSweepMinTiles && best_large_busy >= 0.95 * best_busy ? best_large : best;
}
// Many rows with little work for each workgroup (at most four tiles of 8192 elements for each compute unit):
// filling and draining the three tiles a drift kernel has in the works costs more than the exchange it saves,
// and the sweep kernels' largest tiles, with the fewest exchanges, do best in both directions.  Forward /
// backward in us, drift against sweep with tiles of 16384 elements: 96 x 65536 18.4 / 25.9 against 16.6 / 23.4,
// 128 x 65536 20.1 / 33.2 against 19.9 / 29.4, 120 x 65536 18.9 / 32.4 against 18.6 / 27.9, 150 x 49152
// 18.1 / 33.3 against 18.4 / 25.7; 200 x 32768 18.2 / 28.5 against 15.2 / 22.3 for one workgroup per row.
bool little_work_in_many_rows(const Problem& q) {
  return q.dtype == LINREC_DTYPE_F32 && q.numseq * 4 >= q.cus && q.numseq * q.seqlen <= kT_little_work_max_tiles_per_cu * 8192 * q.cus;
}
// The largest team a drift kernel of this geometry serves: a lane of a wave per team mate, in every wave - except
// 16 waves of two slots of four fp32 elements, compiled for one collecting wave.
int64_t drift_max_team(int waves, int slots, int vec) { return waves == 16 && slots == 2 && vec == 4 ? 64 : int64_t(64) * waves; }
// 16-bit storage: tiles of 8192 elements in 16 waves (tiles in flight stay in the storage type, so a lane's eight
// elements of a slot cost what four fp32 elements do); forward only, tiles of 16384 elements in 16 waves (scanned tiles
// wait in LDS as packed inputs and are scanned again when they are stored), or of 4096 in 8 waves for one or two rows
// that are not whole tiles of 8192.  Returns 4, 2 or 1 accordingly, 0 for "not a drift case".
// The backward wins wherever the fp32 one does (bf16, us, against the table's choice before: 512 x 65536 56.9
// against 63.8 for one workgroup per row, 300 x 65536 36.3 against 44.0, 2048 x 32768 110.7 against 121.4, 1024 x
// 131072 220.7 against 246.9; 16 x 1048576 31.5 against 41.8 for one team per row, 64 x 524288 57.2 against 70.5;
// 1 x 33554432 59.7 against 83.9 for look-back tiles, 1 x 4194304 16.1 against 18.7, 24 x 262144 15.9 against 18.0;
// but 1 x 1048576 16.6 against 15.1).  The forward, whose step moves 48 KB, only where the rows are too few for one
// workgroup per row (1 x 33554432 43.4 against 61.3 us in tiles of 4096, 3 x 4194304 21.1 against 27.6 for one team
// per row, 64 x 524288 40.7 against 45.2, 96 x 262144 30.9 against 32.9, 16 x 1048576 25.2 against 25.5; rows of 32
// tiles and more up to 255 of them: 128 x 262144 39.2 against 41.1, 160 x 262144 47.9 against 51.4; but 128 x 65536
// 14.5 against 12.9, 200 x 65536 19.8 against 16.4, 512 x 65536 40.2 against 37.5, 2048 x 32768 73.9 against 68.2).
// Its tiles of 16384 elements move as much in a step as the fp32 forward's and serve any number of rows of four such
// tiles and more (against tiles of 8192 / the table's choice before: 16 x 1048576 20.4 against 24.7 / 25.3 us,
// 1 x 33554432 38.6 against 42.9, 64 x 524288 37.0 against 39.6, 300 x 65536 24.0 against 25.6 / 26.9 for one workgroup
// per row, 1024 x 131072 136.6 against 145.9 / 141.4, 512 x 65536 36.7 against 38.6 / 37.3; rows of two tiles:
// 2048 x 32768 70.9 against 67.9).
// Rows of whole slots whose last tile is a partial one (second pass, as for fp32): the forward's tiles of 16384
// elements, the backward's of 8192 in 8 waves of two slots (16 waves of one have no registers left for the slots that
// lie beyond the row's end); the rules count the full tiles.
int half_drift_slots_for(const Problem& q, int fv) {
  if (q.is_bwd && q.numseq > q.at(kT_drift_bwd_max_rows)) return 0;
  for (int pass = 0; pass < 2; ++pass)
  for (int s : {4, 2, 1}) {
    const bool ragged = pass == 1;
    if (s == 4 && q.is_bwd) continue;
    if (s == 1 && (q.is_bwd || q.numseq > 2)) continue;
    const int64_t tile = int64_t(8) * s * 64 * fv;
    if ((q.seqlen % tile != 0) != ragged) continue;
    if (ragged && (q.seqlen % fv != 0 || s != (q.is_bwd ? 2 : 4))) continue;
    const int64_t tiles_per_row = q.seqlen / tile;  // (full ones)
    if (s != 4 && !q.is_bwd && q.numseq > q.at(kT_half_drift_fwd_small_tiles_max_rows) && !(q.numseq < q.at(256) && tiles_per_row >= 32)) continue;
    const int64_t team = drift_team_size(q, tiles_per_row + ragged, s == 1 ? 8 : 16, q.cus, ragged);
    if (tiles_per_row < kSweepMinTiles || team < kSweepMinTiles) continue;
    if (q.workspace_cap && linrec_workspace_bytes_for_tiles(q.numseq * (tiles_per_row + ragged)) > q.workspace_cap) continue;
    // the teams have to fill at least half the chip, and every member gets a few tiles: the backward and a few rows'
    // forward (fewer than a quarter of the compute units) as many for each compute unit as the generated table says
    // (the forward's in tiles of 16384 elements, so twice as many of 8192), more rows forward four of them (200 x 65536
    // with three: 17.3 against 16.2 us for one workgroup per row), one or two rows two
    const int64_t per_cu = q.is_bwd ? kT_half_drift_bwd_min_tiles_per_cu
                           : q.numseq <= 2 ? (s == 1 ? 4 : 2)
                                           : (q.numseq * 4 < q.cus ? kT_half_drift_fwd_min_tiles_per_cu : 4) * (s == 4 ? 1 : 2);
    if (std::min(q.numseq, q.cus / team) * team * 2 < q.cus || q.numseq * tiles_per_row < per_cu * q.cus) continue;
    return s;
  }
  return 0;
}
// Returns the tile to use as slots per lane of 8 waves (4: 8192 fp32 elements, 2: 4096), 0 for "not a drift
// case"; which kernel serves the tile (8 waves, or 16 with half the slots) is the launch planner's business.
int drift_slots_for(const Problem& q, int fv) {
  const bool half = q.dtype != LINREC_DTYPE_F32;
  if (q.base_mis != 0 || (q.numseq > 1 && q.row_stride % fv != 0) || q.elem_stride != 1) return 0;
  if (half) return half_drift_slots_for(q, fv);
  // More than 2048 rows: the forward gains as well (us, against one workgroup per row: 4096 x 32768 266.0 against
  // 274.3, 4096 x 40960 335.3 against 360.1, 4096 x 16384 128.9 against 138.8), in the same tiles of 8192 elements as
  // fewer rows (tiles of 4096: 269.2, 340.2, 139.3).
  if (q.is_bwd && q.numseq > q.at(kT_drift_bwd_max_rows)) return 0;
  // The backward of 16 to 127 rows with little work in all stays with the sweep kernels' tiles of 16384 elements
  // (24 x 262144 25.3 against 26.3 us, 40 x 196608 27.0 against 30.8 us; but 100 x 131072 55.1 against 48.5 us,
  // 16 x 1048576 63.5 against 61.9 us, 32 x 1048576 123.1 against 118.0 us, 64 x 524288 118.3 against 116.3 us -
  // all with one tile of loads ahead; with two, 64 x 524288 takes 112.6 us, 256 x 262144 219.7 against 232.8 us and
  // 512 x 262144 453.1 against 452.3 us).
  if (q.is_bwd && q.numseq * 16 >= q.cus && q.numseq < q.at(128) &&
      q.numseq * q.seqlen < kT_drift_bwd_few_rows_min_tiles_per_cu * 8192 * q.cus)
    return 0;
  if (little_work_in_many_rows(q)) return 0;
  // Rows of whole tiles first; then rows of whole slots whose last tile is a partial one, in the forward's tiles of 8192
  // elements and the backward's of 4096 (forward / backward in us against one workgroup per row or one team per row:
  // 335 x 100000 69.8 / 114.6 against 83.4 / 142.9, 1024 x 50000 107.9 / 175.6 against 116.2 / 198.5, 100 x 250000
  // 53.7 / 88.4 against 62.8 / 100.9, 512 x 60000 64.7 / 107.5 against 68.3 / 116.7).  The rules count their full tiles.
  for (int pass = 0; pass < 2; ++pass)
  for (int s : {4, 2, 1}) {
    const bool ragged = pass == 1;
    if (half != (s == 1)) continue;
    if (q.is_bwd && s == 4) continue;  // (the backward pass holds three tensors: two slots per lane fit)
    const int64_t tile = int64_t(8) * s * 64 * fv;
    if ((q.seqlen % tile != 0) != ragged) continue;
    if (ragged && (half || q.seqlen % fv != 0 || s != (q.is_bwd ? 2 : 4))) continue;
    const int64_t tiles_per_row = q.seqlen / tile;  // (full ones)
    const int64_t team = drift_team_size(q, tiles_per_row + ragged, 8, q.cus, ragged);
    // the forward's tiles of 8192 elements: as many tiles a row as the generated table says, and from its number of
    // rows on also rows of two tiles in teams of two (us, against one workgroup per row: 2048 x 16384 66.2 against 69.3,
    // 4096 x 16384 128.9 against 138.8; but 600 x 16384 22.6 against 22.1, 1024 x 16384 34.5 against 35.0)
    const int64_t least_tiles = s != 4 ? kSweepMinTiles
                                : q.numseq >= q.at(kT_drift_fwd_two_tiles_min_rows) ? 2 : kT_drift_fwd_min_tiles_per_row;
    if (tiles_per_row < least_tiles || team < least_tiles) continue;
    // (a caller that can only give so much workspace is served by the kernels that need less)
    if (q.workspace_cap && linrec_workspace_bytes_for_tiles(q.numseq * (tiles_per_row + ragged)) > q.workspace_cap) continue;
    // fp32 rows of fewer than eight tiles of 4096 elements: one workgroup per row does as well or better
    // (forward / backward in us: 768 x 16384 27.3 / 46.3 against 32.3 / 47.5, 400 x 24576 22.6 / 36.4 against
    // 26.3 / 39.7, 1000 x 24576 52.2 / 89.3 against 55.7 / 90.3, 1536 x 16384 52.4 / 90.4 against 55.3 / 89.7,
    // 2048 x 16384 68.9 / 120.0 against 70.4 / 117.4)
    // (with 16 waves and two tiles of loads ahead the backward of 512 rows and more gains from four such tiles on:
    // 2048 x 16384 111.8 against 119.0 us, 768 x 16384 43.9 against 45.5 us)
    if (s == 2 && tiles_per_row < kT_drift_min_small_tiles_per_row && !(q.is_bwd && q.numseq >= q.at(kT_drift_bwd_short_rows_min_rows)))
      continue;
    // the teams have to fill at least half the chip, and every member gets a few tiles (1 x 4194304 in four
    // steps of 4096 elements: 16.4 / 19.8 us, what look-back tiles take)
    if (std::min(q.numseq, q.cus / team) * team * 2 < q.cus || q.numseq * tiles_per_row < (s == 4 ? 3 : 4) * q.cus) continue;
    return s;
  }
  return 0;
}

// Rows longer than a tile, every tile a full one: the sweep kernels spread any number of rows
// evenly over the chip, which one workgroup per row (stream) only does for multiples of the CU
// count and one team per row (team) only for a few row counts.  Measured forward / backward in us,
// default plan without this rule against sweep: 96 x 65536 21.6 / 32.9 against 17.0 / 24.2,
// 160 x 131072 61.7 / 91.1 against 47.8 / 77.7, 288 x 65536 50.2 / 82.3 against 43.2 / 69.8,
// 576 x 131072 172.8 / 300.1 against 161.1 / 270.0; 192 to 256 rows are stream's (36 / 60 against
// 39 / 62 at 256 x 65536).  Multiples of 256 rows: forward within 2 % either way, so stream's;
// backward the sweep kernels gain 2 to 6 % from 512 rows on (512 x 65536: 115.8 against 120.0 us;
// 1024 x 65536: 228.7 against 239.8 us; 4096 x 65536: 918 against 981 us; 1024 x 131072: 458
// against 475 us), except for rows of 16 tiles and more beyond 1024 rows, where they lose as much
// (1536 x 131072: 772 against 719 us; 2048 x 131072: 1034 against 962 us).
// Returns the slots per lane of the sweep kernel to use (tiles of 8 waves), 0 for "not a sweep
// case".  fp32 rows that are a whole number of 4096-element tiles but not of 8192-element ones take
// the smaller tile (300 x 36864: 27.3 / 44.1 us against the stream kernel's 31.6 / 54.9 us).
int sweep_slots_for(const Problem& q, int fv) {
  if (q.base_mis != 0 || (q.numseq > 1 && q.row_stride % fv != 0)) return 0;
  const bool half = q.dtype != LINREC_DTYPE_F32;
  int slots = 0;
  // (little work in many rows: teams of two or three are worth having)
  const bool little = little_work_in_many_rows(q);
  const int64_t least_tiles = little ? 2 : kSweepMinTiles;
  for (int s : {8, 4, 2}) {
    if (half && s >= 4) continue;
    // tiles of 16384 elements: the backward pass over fewer rows than the stream kernel takes (fewer
    // exchanges per byte; 16 x 1048576 backward 61.9 against 66.7 us, 64 x 524288 119 against 132 us,
    // 128 x 262144 121 against 135 us; forward the same or worse, and worse from 512 rows on), and both
    // passes where the rows are many and the work is little
    if (s == 8 && !((q.is_bwd || little) && q.numseq < q.at(kSweepBelowRows) && q.seqlen / 16384 >= least_tiles &&
                    sweep_team_size(q.seqlen / 16384) >= least_tiles))
      continue;
    if (q.seqlen % (int64_t(8) * s * 64 * fv) == 0) { slots = s; break; }
  }
  if (slots == 0) return 0;
  const int64_t tiles_per_row = q.seqlen / (int64_t(8) * slots * 64 * fv);
  const int64_t least = slots == 8 ? least_tiles : kSweepMinTiles;
  if (tiles_per_row < least || sweep_team_size(tiles_per_row) < least) return 0;
  // (a caller that can only give so much workspace is served by the kernels that need less)
  if (q.workspace_cap && linrec_workspace_bytes_for_tiles(q.numseq * tiles_per_row) > q.workspace_cap) return 0;
  // 16-bit storage: measured gains only below the stream kernel's row counts (bf16 96 x 65536
  // 12.3 / 17.6 us against 17.5 / 24.7 us for one team per row, 160 x 262144 51 / 101 us against
  // 62 / 121 us; 1000 x 131072 backward 286 us against the stream kernel's 238 us).  Their backward
  // pass is left to one team per row where teams of 256 / rows workgroups fill the chip (bf16, 2^25
  // elements: 32 rows 72 against 83 us, 48 rows 60 against 66 us, 128 rows 72 against 86 us; 96 rows,
  // teams of 2 on 192 CUs, the same; 160 rows 62 against 50 us).
  if (half && q.is_bwd && q.numseq <= q.cus / 2 && (team_workgroups(q) / q.numseq) * q.numseq >= q.at(240)) return 0;
  if (q.numseq >= (half ? 32 : 16) && q.numseq < q.at(kSweepBelowRows)) return slots;
  if (half) return 0;
  if (q.numseq > q.cus && (q.numseq % q.cus != 0 || (q.is_bwd && (tiles_per_row < 16 || q.numseq <= 4 * q.cus)))) return slots;
  return 0;
}
constexpr int64_t kTailMaxRows = 96;  // rows beyond one per CU that a second launch takes (on 256 CUs)
constexpr int64_t kGroupMaxSlots = 32;  // rows up to this many slots are packed several to a wave
constexpr int64_t kTeamMinRows = kT_team_min_rows;
// 16-bit storage, forward: teams of 64 already win from three rows on (bf16 3 x 4194304 28.0 against 40.3 us for
// look-back tiles, 4 x 8388608 55.1 against 85.6 us, 5 x 2097152 21.7 against 35.0 us); the backward from eight (6 x
// 1048584 25.1 against 19.4 us for look-back tiles, 8 rows 26.2 against 29.5 us).  Both from the generated table.
constexpr int64_t kTeamMinRowsHalfFwd = kT_half_team_fwd_min_rows;
constexpr int64_t kTeamMinRowsHalfBwd = kT_half_team_bwd_min_rows;

// Rows one lane of a column kernel takes: 8 bytes' worth (measured best on 262144 x 256: fp32 two
// rows 131 / 220 us against 132 / 236 us for four; bf16 four rows 70 / 114 us against 101 / 146 us
// for eight), fewer when the rows are too few to give every SIMD a few waves, but 4 bytes' worth at
// least (bf16 100000 x 1024: two rows 135 / 234 us, one row 152 / 264 us).
int kColumnRowsPerLane(const Problem& q) {
  int v = 8 / elem_size_of(q.dtype);
  const int least = 4 / elem_size_of(q.dtype);
  while (v > least && q.numseq / v < q.at(65536)) v >>= 1;
  return v;
}

// Strided scan axis with fewer rows than this: the scan axis is cut into segments.  The plain column
// kernels are bound by the loads a lane has in flight, not by their size, so 16-bit storage runs them
// at the element rate of fp32 and half its byte rate; the crossover sits twice as high there
// (16384 x 4096, segments against plain: fp32 224 / 343 us against 226 / 367 us, bf16 119 / 163 us
// against 232 / 382 us; 32768 x 2048: fp32 225 / 358 us against 145 / 254 us, bf16 132 / 180 us against
// 133 / 204 us).
constexpr int64_t kSegmentBelowRows = 16384;
constexpr int64_t kSegmentBelowRowsHalf = 32768;
constexpr int64_t kSegmentMinLen = 256;       // shorter scan axes are left to the plain column kernels
int64_t segment_waves(const Problem& q) { return 4 * q.cus; }  // waves a segmented launch aims for (one per SIMD)
constexpr int64_t kSegmentMaxSegments = 4096; // (the maps of a row are then 32 KiB)

size_t segment_maps_bytes(int64_t numseq, int64_t segments) { return size_t(2) * size_t(segments) * size_t(numseq) * 4; }

// Flat kernels: dense rows (no gaps between them, so the tensor is one array), every base 16-byte
// aligned, rows short enough for one row of 64 slots to look behind.
bool flat_applies(const Problem& q, int fv) {
  return q.elem_stride == 1 && q.numseq > 1 && q.row_stride == q.seqlen && q.base_mis == 0 && !q.batched() &&
         q.seqlen >= 2 && q.seqlen <= 60 * fv;
}
// Where they are chosen: up to 40 slots per row.  The look-behind row costs loads in proportion to the
// row length (2^25 elements, forward / backward: rows of 5 floats 69 / 111 us against 135 / 232 us for
// lanes that share a row, 30 floats 72 / 113 us against 132 / 192 us, 130 floats 77 / 118 us against
// 93 / 139 us for one wave per row, 239 floats 81 / 139 us against 69 / 115 us).
constexpr int64_t kFlatMaxSlots = 40;

// Column block kernels (16 waves of a workgroup share 64 lanes' rows, each wave a run of positions).
// Measured against the plain column kernel and the segmented launches on transposed matrices
// (forward / backward): fp32 16384 x 2048 69.9 / 127.3 us against 112.4 / 180.2 us, 10000 x 2048
// 51.0 / 85.5 us against 81.9 / 111.2 us, 12288 x 4096 111.0 / 191.7 us against 168.3 / 248.6 us,
// 16384 x 256 10.9 / 17.1 us against 15.3 / 26.1 us; two rows per lane beyond 16384 rows (24576 x 2048:
// 101.9 / 181.6 us against 113.9 / 199.6 us with one row and 126.9 / 236.0 us plain; 16384 x 2048
// 85.0 / 143.3 us), up to one workgroup per CU (32768 x 2048 128.7 / 220.4 us against
// 145.0 / 254.1 us; 40000 x 1024 loses: 88.8 us against 86.2 us).  Below 8192 rows the workgroups
// are too few (6144 x 4096: 80.3 / 134.5 us against 85.9 / 123.0 us for segments; 4096 x 8192
// 147 / 238 us against 110 / 148 us).  bf16, two rows per lane: 32768 x 2048 71.2 / 132.1 us against
// 131.5 / 220.0 us, 16384 x 4096 102.5 / 157.7 us against 122.7 / 168.2 us, 65536 x 1024
// 74.8 / 134.3 us against 87.8 / 135.7 us; 8192 and 100000 rows lose.
// Waves split into two groups of 32 lanes (half the rows per workgroup, twice the workgroups) up to 8192
// rows (16-bit storage: 16384), fp32: 6144 x 4096 63.8 / 107.0 us against 85.9 / 122.1 us for segments, 8192 x 16384
// 325.2 / 562.4 us against 325.4 / 630.7 us, 4096 x 8192 101.1 / 168.7 us against 110.5 / 148.7 us (so the
// backward starts at 6144 rows), 10000 x 4096 139.0 / 234.2 us against 97.7 / 168.2 us undivided.  16-bit
// storage, forward only (its backward would not fit the registers): 16384 x 4096 78.6 us against 101.8 us
// undivided, 12288 x 4096 71.4 us against 99.0 us for segments, 8192 x 4096 64.3 us against 69.3 us,
// 18432 x 2048 70 us against 54 us undivided.
constexpr int kColblockWaves = 16;
constexpr int64_t kColblockMinLen = 256;
// fp32, 15360 to 16384 rows of at least 1024 elements: two rows per lane in two groups per wave, the same 240
// to 256 workgroups as one row per lane in undivided waves with twice the bytes in flight (16384 x 2048
// 68 / 121 us against 71 / 128 us, 16384 x 4096 134 / 236 us against 145 / 254 us; 14000 x 2048 70 / 115 us
// against 66 / 114 us, 16384 x 512 16 / 34 us against 19 / 31 us).
bool colblock_full_house(const Problem& q) {
  return q.dtype == LINREC_DTYPE_F32 && q.numseq >= q.at(15360) && q.numseq <= q.at(16384) && q.seqlen >= 1024 && q.row_stride == 1 &&
         q.col_phase % 2 == 0 && q.elem_stride % 2 == 0 && q.numseq % 2 == 0 &&
         (!q.batched() || (q.rows_per_batch % 2 == 0 && q.batch_stride % 2 == 0));
}
// Lane groups per wave the planner picks for this problem, 0 if it leaves it to the other kernels.
// The form with the most workgroups that still gives every CU at most one is the one to take: one more
// than 256 workgroups costs a second round (fp32, one row per lane: 16384 x 2048 70 / 128 us, 17408 x 2048
// 103 / 173 us, where two rows per lane take 89 / 153 us; 16-bit, two groups: 16384 x 2048 forward 42 us,
// 17408 x 2048 70 us against 54 us undivided).
int colblock_groups(const Problem& q) {
  if (q.seqlen < kColblockMinLen) return 0;
  if (q.dtype != LINREC_DTYPE_F32) {
    // 16-bit storage, 4 bytes of rows per lane: two groups up to 16384 rows (256 workgroups), the
    // backward (runs of 4 positions) from 10240 rows on (8192 x 2048 62 us against 60 us for segments,
    // 12000 x 2048 68 us against 82 us, 16384 x 2048 73 us against 100 us); undivided waves beyond
    // (17408 x 2048 56 / 103 us against 72 / 124 us with two groups and 79 / 104 us for segments,
    // 32768 x 2048 70 / 123 us against 134 / 221 us for the plain kernel)
    if (q.numseq >= q.at(q.is_bwd ? 10240 : 8192) && q.numseq <= q.at(16384)) return 2;
    return q.numseq > q.at(16384) && q.numseq <= q.at(65536) ? 1 : 0;
  }
  if (q.numseq >= q.at(q.is_bwd ? 6144 : 4096) && q.numseq <= q.at(8192)) {
    // two groups of 32 floats are 128-byte accesses: lines that do not start on a 128-byte boundary cost
    // them more than the undivided wave (7000 x 2048: 55 / 102 us against 50 / 86 us; 5000 x 2048 forward
    // 39 us against 47 us all the same)
    if (q.numseq >= q.at(6144) && (q.elem_stride * 4) % 128 != 0) return 1;
    return 2;
  }
  if (colblock_full_house(q)) return 2;
  if (q.numseq > q.at(8192) && q.numseq <= q.at(32768)) return 1;
  // Beyond one workgroup per CU the second round has to be at least half full to beat the plain kernel:
  // two rows per lane, 384 to 480 workgroups (50000 x 2048 246 / 421 us against 284 / 457 us, 57344 x 2048
  // 244 / 425 us against 272 / 457 us; 40000 x 2048 210 / 359 us against 174 / 314 us, 45056 x 2048
  // 216 / 381 us against 214 / 337 us, 65536 x 2048 271 / 487 us against 281 / 452 us)
  return q.numseq >= q.at(49152) && q.numseq <= q.at(61440) ? 1 : 0;
}
// The block kernel for `vec` rows per lane with runs of `want_depth` positions, or of the compiled length
// (8, or 4 where three tensors of two rows per lane would not fit the registers) for 0; -1 if none.
int colblock_kernel_for(const Problem& q, int vec, int groups, int want_depth, int mode, int desc, int* depth) {
  for (int d : {8, 4}) {
    if (want_depth > 0 && d != want_depth) continue;
    const int id = find_kernel(q.dtype, LINREC_FAMILY_COLUMN, kColblockWaves, d, vec, mode, desc, groups);
    if (id >= 0) {
      *depth = d;
      return id;
    }
  }
  return -1;
}
// Rows per lane (`want`, or the planner's choice for 0) if the layout allows a block kernel, else 0.
int colblock_rows_per_lane(const Problem& q, int want) {
  if (q.elem_stride == 1 && q.seqlen != 1) return 0;
  if (q.seqlen > 2147483647LL - 1024) return 0;  // positions are counted in 32 bits, a step beyond the row end included
  if (q.row_stride != 1 && q.numseq != 1 && q.rows_per_batch != 1) return 0;
  int v = want > 0 ? want : q.dtype != LINREC_DTYPE_F32 ? 2 : (q.numseq > q.at(16384) || colblock_full_house(q)) ? 2 : 1;
  auto fits = [&](int w) {
    return w == 1 || (q.row_stride == 1 && q.col_phase % w == 0 && q.elem_stride % w == 0 && q.numseq % w == 0 &&
                      (!q.batched() || (q.rows_per_batch % w == 0 && q.batch_stride % w == 0)));
  };
  while (v > 1 && !fits(v)) {
    if (want > 0) return 0;
    v >>= 1;
  }
  return v;
}

// Column drift kernels: the team size for `blocks` blocks of rows of `steps` steps each, 0 if the launch
// would not be worth it: the power of two that fills the chip, every member with at least four steps.
// 16-bit storage (blocks of 128 rows, two to a lane): teams of 4 or 8, every member with at least two steps (bf16
// 4096 x 2048 in teams of 8: 18.1 / 22.7 us against 28.4 / 38.4 us for the segments).
int64_t coldrift_team(const Problem& q, int64_t blocks, int64_t steps, int64_t resident, int waves) {
  int64_t team = 1;
  if (q.dtype != LINREC_DTYPE_F32) {
    while (team * 2 <= 8 && blocks * team * 2 <= resident && steps >= 4 * team) team *= 2;
    return team >= 4 ? team : 0;
  }
  while (team * 2 <= waves && blocks * team * 2 <= resident && steps >= 8 * team) team *= 2;
  return team >= 2 && blocks * team * 2 > q.cus ? team : 0;
}
// Whether the planner gives this problem (strided scan axis) to the column drift kernels: fp32 rows next to
// each other, few enough that teams of at least 4 (backward: 2) along the scan axis are what fills the chip,
// and enough of them that the teams fill three quarters of it.  Measured forward / backward in us against
// what the table chose before (segments up to 4095 rows, column blocks from there): 4096 x 16384 157.1 / 255.5
// against 216.3 / 307.1; 2048 x 16384 83.6 / 132.0 against 107.4 / 150.4; 1024 x 32768 forward 95.6 against
// 110.4 (backward 162.1 against 154.6: left to the segments); 8192 x 4096 backward 126.8 against 142.7 (forward
// 80.5 against 78.9: left to the column blocks); 3072 x 16384 140.5 / 213.5 against 168.4 / 248.2; 2048 x 4096
// 25.5 / 36.2 against 40.8 / 54.3; 4096 x 2048 24.9 / 34.3 against 29.5 / 47.7; 512 x 65536 161.3 / 284.5
// against 112.7 / 149.9 (left to the segments).
//
// 16-bit storage, two rows to a lane (four bytes' worth, as fp32's one): the teams are twice as large for the same rows,
// so they pay where teams of 4 fill three quarters of the chip and teams of 8 seven eighths of it.  bf16, forward /
// backward in us against the table's choice before (segments; column blocks for the forward of 8192 rows): 4096 x 16384
// in teams of 8 108.3 / 156.1 against 130.9 / 164.4, 8192 x 4096 in teams of 4 52.0 / 78.5 against 63.3 / 93.3, 6144 x
// 4096 (192 workgroups) 46.3 / 68.3 against 55.9 / 73.9, 4096 x 2048 18.1 / 22.7 against 28.4 / 38.4; but 3072 x 16384
// (teams of 8 in 192 workgroups) 100.9 / 142.1 against 96.4 / 127.1, 2560 x 8192 50.8 / 71.3 against 48.2 / 64.5, and
// teams of 16 (2048 x 16384: 67.7 / 122.2 against 66.4 / 92.2; 2048 x 4096 21.9 / 31.3 against 26.9 / 36.5) or of 2
// (16384 x 4096: 96.3 / 145.6 against 79.4 / 132.8 for the column blocks) are left out.
bool coldrift_applies(const Problem& q) {
  const bool half = q.dtype != LINREC_DTYPE_F32;
  if (q.seqlen < 2048) return false;
  if (q.row_stride != 1 && q.numseq != 1 && q.rows_per_batch != 1) return false;
  const int vec = half ? 2 : 1;
  if (colblock_rows_per_lane(q, vec) != vec) return false;
  const int waves = q.is_bwd ? 8 : 16;
  const int64_t blocks = ceil_div(ceil_div(q.numseq, vec), 64);
  const int64_t steps = ceil_div(q.seqlen, 128);
  const int64_t team = coldrift_team(q, blocks, steps, q.cus, waves);
  // (a caller that can only give so much workspace is served by the kernels that need less)
  if (q.workspace_cap && linrec_workspace_bytes_for_tiles(blocks * steps * 64 * vec) > q.workspace_cap) return false;
  if (half) return team == 4 ? blocks * team * 4 >= 3 * q.cus : team == 8 && blocks * team * 8 >= 7 * q.cus;
  // Teams of 16 only where they fill seven eighths of the chip: 768 x 32768 forward 91.4 us in 192 workgroups
  // against 82.6 us for the segments, 900 x 32768 97.6 us in 240 against 117.6 us, 1024 x 32768 98.7 against
  // 109.1 us.  Teams of 2, which gain least, only where they fill it: 6144 x 4096 backward 110.6 us in 192
  // workgroups against 108.3 us for the column blocks, 8192 x 4096 127.3 against 141.0 us.  Teams of 4 and 8 from
  // 65 % on, forward / backward: 1300 x 16384 in 168 workgroups 76.4 / 116.8 us against 86.4 / 128.3 us, 3000 x 8000
  // in 188 80.5 / 132.0 us against 93.7 / 131.0 us; 2560 x 8192 in 160 70.3 / 102.4 us against 69.5 / 97.7 us,
  // 1100 x 16384 in 144 74.3 / 107.8 us against 75.7 / 109.9 us, 2200 x 16384 in 140 141.5 / 216.0 us against
  // 134.9 / 199.6 us.
  if (team < (q.is_bwd ? 2 : 4)) return false;
  if (team == 2) return blocks * team >= q.cus;
  if (team > 8) return blocks * team * 8 >= 7 * q.cus;
  return blocks * team * 20 >= 13 * q.cus;
}
// The rows a second launch serves: the last `tail_rows` rows of `q`, as a problem of their own.
Problem tail_problem(const Problem& q, int64_t tail_rows) {
  Problem t = q;
  const int64_t skipped = q.numseq - tail_rows;
  t.numseq = tail_rows;
  const int fv = full_vec_of(q.dtype);
  if (q.base_mis >= 0) {
    t.base_mis = int(((q.base_mis + skipped * q.row_stride) % fv + fv) % fv);
    t.aligned16 = t.base_mis == 0;
    t.col_phase = t.base_mis;
  }
  return t;
}

int make_plan(const Problem& q, const linrec_tuning_t* tune, linrec_plan_t* out) {
  std::memset(out, 0, sizeof(*out));
  out->kernel_id = -1;
  if (q.numseq < 0 || q.seqlen < 0) return LINREC_E_INVALID;
  if (q.seqlen > 2147483643LL) return LINREC_E_TOO_LARGE;
  if (q.numseq == 0 || q.seqlen == 0) return LINREC_OK;  // nothing to launch
  if (q.dtype < LINREC_DTYPE_F32 || q.dtype > LINREC_DTYPE_BF16) return LINREC_E_UNSUPPORTED;
  {
    // No two elements may share an address (results are written with the same strides): rows of whole
    // elements side by side, or elements of whole rows side by side.
    const int64_t es = q.elem_stride < 0 ? -q.elem_stride : q.elem_stride;
    const int64_t rs = q.row_stride < 0 ? -q.row_stride : q.row_stride;
    if (q.seqlen > 1 && es == 0) return LINREC_E_INVALID;
    if (q.numseq > 1 && !q.batched() && q.seqlen > 1 && !(rs >= es * q.seqlen || (rs > 0 && es >= rs * q.numseq)))
      return LINREC_E_INVALID;
    if (q.numseq > 1 && !q.batched() && q.seqlen == 1 && rs == 0) return LINREC_E_INVALID;
  }
  const int fv = full_vec_of(q.dtype);        // elements of a 16-byte slot
  const bool half = q.dtype != LINREC_DTYPE_F32;
  // slots a row needs when all rows start on a slot boundary, one more otherwise
  const bool rows_on_slots = q.base_mis == 0 && (q.row_stride % fv == 0 || q.numseq == 1);
  const int64_t full_slots = ceil_div(q.seqlen + (rows_on_slots ? 0 : fv - 1), fv);

  // The gradient scan runs against the forward scan.
  const int desc = (q.reverse != 0) != (q.is_bwd != 0) ? 1 : 0;
  const int mode = q.is_bwd ? linrec::MODE_BWD : linrec::MODE_FWD;

  int family = tune && tune->family != LINREC_FAMILY_AUTO ? tune->family : LINREC_FAMILY_AUTO;
  int use_colblock = 0;  // family COLUMN chosen below in its block form: lane groups per wave
  if (q.batched()) {
    // only the kernels for a strided scan axis take a batch stride
    if (q.numseq % q.rows_per_batch) return LINREC_E_INVALID;
    if (q.elem_stride == 1 && q.seqlen != 1) return LINREC_E_UNSUPPORTED;
    if (family != LINREC_FAMILY_AUTO && family != LINREC_FAMILY_COLUMN && family != LINREC_FAMILY_NAIVE &&
        family != LINREC_FAMILY_SEGMENT && family != LINREC_FAMILY_COLDRIFT)
      return LINREC_E_UNSUPPORTED;
  }
  if (family == LINREC_FAMILY_AUTO) {
    if (q.elem_stride == 1 || q.seqlen == 1) {
      family = LINREC_FAMILY_TILE;
      // Rows of at most 32 slots: several rows per wave.
      if (q.base_mis >= 0 && full_slots <= kGroupMaxSlots) family = LINREC_FAMILY_GROUP;
      // Dense short rows that are not whole slots: the tensor as one flat array of full slots.
      // (rows that fill 28 to 32 lanes of a group stay with the group kernel: 121 floats 66 / 112 us
      // against 76 / 132 us)
      if (flat_applies(q, fv) && q.seqlen % fv != 0 && q.seqlen <= kFlatMaxSlots * fv &&
          !(full_slots >= 28 && full_slots <= kGroupMaxSlots))
        family = LINREC_FAMILY_FLAT;
      // Many long rows: one workgroup per row, no workgroup ever waits for another.  Measured on
      // MI355X at 2^25 elements: 512 x 65536 forward 71 us against 84 us for the best look-back
      // tiling; with fewer than about a hundred rows the chip is not filled and look-back wins.
      if (q.base_mis >= 0 && full_slots > kLongRowSlots) {
        if (drift_slots_for(q, fv) > 0) family = LINREC_FAMILY_DRIFT;
        else if (sweep_slots_for(q, fv) > 0) family = LINREC_FAMILY_SWEEP;
        else if (q.numseq >= q.at(kStreamMinRows - 1) + 1) {
          family = LINREC_FAMILY_STREAM;
          // fp32 rows from a length on (generated table): look-back tiles of 16384 elements, which the dispatcher hands
          // to whichever compute unit is free (rows that are not whole slots, forward / backward in us against one
          // workgroup per row: 335 x 100001 74.7 / 134.7 against 91.7 / 159.0, 300 x 65541 47.3 / 81.8 against 58.5 / 98.9,
          // 4096 x 65541 522 / 975 against 613 / 1067, 8192 x 32770 534 / 1018 against 612 / 1078; but 2000 x 20001
          // 99.9 / 177.6 against 92.0 / 160.8; 16-bit storage, tiles of eight waves of four slots: 512 x 65542 58.7 / 86.8
          // against 42.0 / 73.0)
          // (rows of whole slots stay where the rules above left them; a caller that can only give so much workspace is
          // served by the kernel that needs none)
          if (!half && q.seqlen >= kT_stream_max_len && !(rows_on_slots && q.seqlen % fv == 0) &&
              !(q.workspace_cap && linrec_workspace_bytes_for_tiles(q.numseq * ceil_div(full_slots, int64_t(8) * 8 * 64)) > q.workspace_cap))
            family = LINREC_FAMILY_TILE;
        }
        else if (q.numseq >= (half ? (q.is_bwd ? kTeamMinRowsHalfBwd : kTeamMinRowsHalfFwd) : kTeamMinRows)) family = LINREC_FAMILY_TEAM;
      }
      // 16-bit storage, many rows of exactly two of the stream kernel's tiles (16384 elements): one workgroup of
      // 8 waves that walks the row beats one tile of 16 waves (bf16 2048 x 16384 34.1 / 57.0 against 36.4 / 59.7 us,
      // 3000 rows 48.2 / 82.4 against 50.4 / 85.4 us, 4096 rows 64.7 / 112.0 against 68.5 / 118.5 us, 1024 rows
      // 18.8 / 30.1 against 19.9 / 29.7 us; not rows with a ragged second tile: 2048 x 16000 40.6 / 67.2 against
      // 35.6 / 60.1 us, 2048 x 12288 33.7 / 53.8 against 29.8 / 46.2 us)
      if (half && family == LINREC_FAMILY_TILE && q.seqlen == 16384 && q.base_mis == 0 && q.elem_stride == 1 &&
          q.row_stride % fv == 0 && q.numseq >= q.at(2048))
        family = LINREC_FAMILY_STREAM;
    } else if (q.row_stride == 1 || q.numseq == 1 || q.rows_per_batch == 1) {
      family = q.numseq < q.at(half ? kSegmentBelowRowsHalf : kSegmentBelowRows) && q.seqlen >= kSegmentMinLen
                   ? LINREC_FAMILY_SEGMENT : LINREC_FAMILY_COLUMN;
      // a few thousand to a few ten thousand rows: workgroups whose waves share rows
      if (const int g = colblock_groups(q)) {
        const int v = colblock_rows_per_lane(q, 0);
        int d = 0;
        if (v > 0 && colblock_kernel_for(q, v, g, 0, mode, desc, &d) >= 0) {
          family = LINREC_FAMILY_COLUMN;
          use_colblock = g;
        }
      }
      // a few hundred to a few thousand rows: column blocks in teams along the scan axis
      if (coldrift_applies(q)) {
        family = LINREC_FAMILY_COLDRIFT;
        use_colblock = 0;
      }
    } else {
      family = LINREC_FAMILY_NAIVE;
    }
  }

  if (family == LINREC_FAMILY_FLAT) {
    if (!flat_applies(q, fv)) return LINREC_E_UNSUPPORTED;
    // rows of 64 slots per wave: two leave more waves in flight, four spread the look-behind row thinner
    const int slots = tune && tune->family == LINREC_FAMILY_FLAT && tune->slots > 0 ? tune->slots
                      : (half || q.seqlen <= 64) ? 2 : 4;
    const int id = find_kernel(q.dtype, LINREC_FAMILY_FLAT, 4, slots, fv, mode, desc, 0);
    if (id < 0) return LINREC_E_UNSUPPORTED;
    const int64_t total_slots = ceil_div(q.numseq * q.seqlen, fv);
    out->family = LINREC_FAMILY_FLAT;
    out->waves = 4; out->slots = slots; out->vec = fv; out->carry = 0;
    out->tiles_per_row = 1;
    out->tasks = 1;
    out->grid = ceil_div(ceil_div(total_slots, int64_t(64) * slots), 4);
    if (out->grid > 2147483647LL) return LINREC_E_TOO_LARGE;
    out->block = 256;
    out->kernel_id = id;
    out->workspace_bytes = 0;
    return LINREC_OK;
  }

  if (family == LINREC_FAMILY_GROUP) {
    if (q.elem_stride != 1 && q.seqlen != 1) return LINREC_E_UNSUPPORTED;
    if (q.numseq > 1 && q.row_stride < q.seqlen && q.row_stride > -q.seqlen) return LINREC_E_INVALID;
    const int64_t row_slots = full_slots;  // one more than seqlen / slot when rows start inside a slot
    if (q.base_mis < 0 || row_slots > 32) return LINREC_E_UNSUPPORTED;
    int group = 1;
    while (group < row_slots) group <<= 1;
    if (tune && tune->family == LINREC_FAMILY_GROUP && tune->tasks > 0) {
      group = tune->tasks;  // more lanes than the row needs: the spare ones idle
      if (group < row_slots || group > 32 || (group & (group - 1))) return LINREC_E_UNSUPPORTED;
    }
    const int id = find_kernel(q.dtype, LINREC_FAMILY_GROUP, 4, 1, fv, mode, desc, 0);
    if (id < 0) return LINREC_E_UNSUPPORTED;
    out->family = LINREC_FAMILY_GROUP;
    out->waves = 4; out->slots = 1; out->vec = fv; out->carry = 0;
    out->tiles_per_row = 1;
    out->tasks = group;  // lanes per row
    out->grid = ceil_div(ceil_div(q.numseq, 64 / group), 4);
    if (out->grid > 2147483647LL) return LINREC_E_TOO_LARGE;
    out->block = 256;
    out->kernel_id = id;
    out->workspace_bytes = 0;
    return LINREC_OK;
  }

  if (family == LINREC_FAMILY_STREAM) {
    if (q.elem_stride != 1 && q.seqlen != 1) return LINREC_E_UNSUPPORTED;
    if (q.numseq > 1 && q.row_stride < q.seqlen && q.row_stride > -q.seqlen) return LINREC_E_INVALID;
    if (q.base_mis < 0) return LINREC_E_UNSUPPORTED;  // needs a common 16-byte phase of all tensors
    const int waves = tune && tune->waves > 0 ? tune->waves : 8;
    // Tiles of 8192 elements; fp32 rows that are whole tiles of 16384 take those when the launch has
    // at most one workgroup per CU, which then needs more bytes in flight (256 x 32768: 16.2 / 26.5 us
    // against 19.0 / 31.1 us; 256 x 131072 backward 120.4 against 129.9 us), or when the rows are long
    // (512 x 262144: 274 / 478 us against 282 / 491 us) or many (1024 x 65536 forward: 135.5 against
    // 138.7 us; 4096 x 65536: 542 against 556 us).  512 x 65536 is the same either way.
    const bool big_tiles = !half && rows_on_slots && q.seqlen % 16384 == 0 &&
                           (q.numseq <= q.cus || q.seqlen >= 131072 || (q.numseq >= 4 * q.cus && q.seqlen >= 32768));
    // Tiles of 4096 elements for rows they pad less, and for rows of at most two of the larger tiles:
    // a partial last tile costs a whole one, and short walks overlap little (3355 x 10000: 73 / 122 us
    // against 77 / 162 us; 2500 x 14000 backward: 129 against 145 us; 1677 x 20000 backward: 126
    // against 135 us; whole tiles are the same either way).
    const bool small_tiles = !half && (ceil_div(full_slots, 1024) * 1024 < ceil_div(full_slots, 2048) * 2048 ||
                                       full_slots <= 4096);
    const int slots = tune && tune->slots > 0 ? tune->slots : half ? 2 : big_tiles ? 8 : small_tiles ? 2 : 4;  // four bring 16-bit storage nothing
    const int id = find_kernel(q.dtype, LINREC_FAMILY_STREAM, waves, slots, fv, mode, desc, 0);
    if (id < 0) return LINREC_E_UNSUPPORTED;
    if (q.numseq > 2147483647LL) return LINREC_E_TOO_LARGE;
    out->family = LINREC_FAMILY_STREAM;
    out->waves = waves; out->slots = slots; out->vec = fv; out->carry = 0;
    out->tiles_per_row = int32_t(ceil_div(full_slots, int64_t(waves) * slots * 64));
    out->tasks = 1;
    // One workgroup per row: the rows beyond one per CU run as a second round that leaves most of the
    // chip idle.  Without a tuning, up to 96 rows beyond 256 are left to a second launch planned for them
    // alone (teams of workgroups per row): 313 x 106924 95 / 148 us against 103 / 167 us, 257 x 130436
    // 94 / 159 us against 101 / 180 us.  With more rows in the last round, or more rounds, it brings
    // nothing (557 x 60164: 88 / 146 us against 91 / 149 us) or loses (389 x 86108: 87 / 147 us against
    // 83 / 139 us), because the second launch waits for the first.
    // 16-bit storage: the backward only (bf16 288 x 65536 28.3 / 43.2 us against 27.5 / 46.2 us in one launch,
    // 352 rows 33.3 / 50.5 us against 28.2 / 48.9 us).
    if (!tune && q.numseq > q.cus && q.numseq <= q.cus + q.at(kTailMaxRows) && !(half && !q.is_bwd))
      out->tail_rows = int32_t(q.numseq - q.cus);
    size_t tail_workspace = 0;
    if (out->tail_rows) {
      linrec_plan_t tail;
      if (make_plan(tail_problem(q, out->tail_rows), nullptr, &tail) == LINREC_OK) tail_workspace = size_t(tail.workspace_bytes);
      else out->tail_rows = 0;
    }
    out->grid = q.numseq - out->tail_rows;
    out->block = 64 * waves;
    out->kernel_id = id;
    out->workspace_bytes = tail_workspace;
    return LINREC_OK;
  }

  if (family == LINREC_FAMILY_SWEEP || family == LINREC_FAMILY_DRIFT) {
    const bool drift = family == LINREC_FAMILY_DRIFT;
    if (q.elem_stride != 1 && q.seqlen != 1) return LINREC_E_UNSUPPORTED;
    if (q.numseq > 1 && q.row_stride < q.seqlen && q.row_stride > -q.seqlen) return LINREC_E_INVALID;
    int waves = tune && tune->waves > 0 ? tune->waves : 8;
    const int auto_slots = tune && tune->family != LINREC_FAMILY_AUTO ? 0 : drift ? drift_slots_for(q, fv) : sweep_slots_for(q, fv);
    int slots = tune && tune->slots > 0 ? tune->slots : auto_slots > 0 ? auto_slots : (half ? (drift ? 1 : 2) : 4);
    // 16-bit drift tiles of 8192 elements: 16 waves with one slot each (also what a caller who names the family and
    // nothing else gets, where the rows are whole tiles of that size)
    if (drift && half && !(tune && (tune->waves > 0 || tune->slots > 0)) &&
        (auto_slots == 2 || (auto_slots == 0 && q.seqlen % (int64_t(16) * 64 * fv) == 0))) {
      waves = 16;
      slots = 1;
      // (the backward of rows with a partial last tile: 8 waves of two slots)
      if (q.is_bwd && q.seqlen % (int64_t(16) * 64 * fv) != 0) {
        waves = 8;
        slots = 2;
      }
    }
    // ... and its forward tiles of 16384 elements: 16 waves with two slots each
    if (drift && half && auto_slots == 4 && !(tune && (tune->waves > 0 || tune->slots > 0))) {
      waves = 16;
      slots = 2;
    }
    // fp32 drift tiles of 4096 elements (every backward, and the forward of rows that are not whole tiles of
    // 8192): 16 waves with one slot each rather than 8 waves with two.  Forward / backward in us: 512 x 65536
    // backward 116.2 against 117.4, 300 x 65536 70.7 against 71.5, 1024 x 65536 229.2 against 231.2, 16 x 1048576
    // 61.9 against 64.2, 1 x 33554432 74.6 / 119.8 against 82.1 / 125.0.
    if (drift && !half && auto_slots == 2 && !(tune && (tune->waves > 0 || tune->slots > 0))) {
      waves = 16;
      slots = 1;
    }
    // The forward's tiles of 8192 elements likewise, 16 waves of two slots rather than 8 of four, in teams of at
    // most 64 (one after the other in one process, us: 512 x 65536 67.9 against 68.5, 300 x 65536 42.3 against
    // 43.6, 1024 x 65536 132.2 against 133.8, 16 x 1048576 in teams of 128 37.6 against 38.1 - compiled without
    // the larger teams' code, which does not fit its registers, so those keep 8 waves).
    if (drift && !half && !q.is_bwd && auto_slots == 4 && !(tune && (tune->waves > 0 || tune->slots > 0)) &&
        drift_team_size(q, ceil_div(q.seqlen, int64_t(8) * 4 * 64 * fv), 8, q.cus, q.seqlen % (int64_t(8) * 4 * 64 * fv) != 0) <= 64) {
      waves = 16;
      slots = 2;
    }
    const int64_t tile_elems = int64_t(waves) * slots * 64 * fv;
    // every tile of every row has to be a full one; the drift kernels also come for rows of whole slots whose last
    // tile is a partial one (kernel-table code 2 in the carry column)
    const bool ragged = drift && q.seqlen % tile_elems != 0 && q.seqlen % fv == 0 && q.seqlen > tile_elems;
    if (q.base_mis != 0 || (q.numseq > 1 && q.row_stride % fv != 0) || (q.seqlen % tile_elems != 0 && !ragged)) return LINREC_E_UNSUPPORTED;
    const int id = find_kernel(q.dtype, family, waves, slots, fv, mode, desc, ragged ? 2 : 1);
    if (id < 0) return LINREC_E_UNSUPPORTED;
    const int block = 64 * waves;
    const int64_t tiles_per_row = ceil_div(q.seqlen, tile_elems);
    // Every workgroup of the launch has to be resident at once (a walker waits for its team mates, and a
    // workgroup that has not started yet only starts when another one ends): never more than the CUs hold.
    const int64_t resident = int64_t(workgroups_per_cu(id, block, drift || q.is_bwd ? 1 : 2)) * q.cus;
    const int64_t team = tune && tune->tasks > 0
                             ? tune->tasks
                             : drift ? drift_team_size(q, tiles_per_row, waves, resident, ragged, ragged ? drift_max_team(waves, slots, fv) : 0)
                                     : sweep_team_size(tiles_per_row, std::min<int64_t>(kSweepMaxTeam, resident));
    if (team > (drift ? drift_max_team(waves, slots, fv) : 64) || team > tiles_per_row || (tiles_per_row % team != 0 && !ragged)) return LINREC_E_UNSUPPORTED;
    int64_t teams = tune && tune->carry > 0 ? tune->carry : std::min(sweep_workgroups(q), resident) / team;
    if (teams > q.numseq) teams = q.numseq;
    if (teams < 1 || teams * team > resident) return LINREC_E_UNSUPPORTED;
    if (q.numseq * tiles_per_row > 2147483647LL) return LINREC_E_TOO_LARGE;
    out->family = family;
    out->waves = waves; out->slots = slots; out->vec = fv; out->carry = 1;
    out->tiles_per_row = int32_t(tiles_per_row);
    out->tasks = int32_t(team);
    out->grid = teams * team;
    out->block = block;
    out->kernel_id = id;
    out->workspace_bytes = linrec_workspace_bytes_for_tiles(q.numseq * tiles_per_row);
    return LINREC_OK;
  }

  if (family == LINREC_FAMILY_TEAM) {
    if (q.elem_stride != 1 && q.seqlen != 1) return LINREC_E_UNSUPPORTED;
    if (q.numseq > 1 && q.row_stride < q.seqlen && q.row_stride > -q.seqlen) return LINREC_E_INVALID;
    if (q.base_mis < 0) return LINREC_E_UNSUPPORTED;
    const int waves = tune && tune->waves > 0 ? tune->waves : 8;
    // 16-bit storage, 16 x 2^20: forward s4 25 us against s2 28 us; the backward with s4 does not
    // fit the register file
    const int slots = tune && tune->slots > 0 ? tune->slots : (half && q.is_bwd ? 2 : 4);
    const int id = find_kernel(q.dtype, LINREC_FAMILY_TEAM, waves, slots, fv, mode, desc, 1);
    if (id < 0) return LINREC_E_UNSUPPORTED;
    const int64_t tiles_per_row = ceil_div(full_slots, int64_t(waves) * slots * 64);
    int64_t team = tune && tune->tasks > 0 ? tune->tasks : team_workgroups(q) / q.numseq;
    if (team < 2 && !(tune && tune->tasks > 0)) team = 2;
    if (team > tiles_per_row) team = tiles_per_row;
    if (team > 64) team = 64;  // one wave gathers the team's maps, one lane per team mate
    // a team has to fit the chip, or its members would wait for mates that cannot start
    if (team > int64_t(workgroups_per_cu(id, 64 * waves, 1)) * q.cus) return LINREC_E_UNSUPPORTED;
    if (q.numseq * team > 2147483647LL || q.numseq * tiles_per_row > 2147483647LL) return LINREC_E_TOO_LARGE;
    out->family = LINREC_FAMILY_TEAM;
    out->waves = waves; out->slots = slots; out->vec = fv; out->carry = 1;
    out->tiles_per_row = int32_t(tiles_per_row);
    out->tasks = int32_t(team);
    out->grid = q.numseq * team;
    out->block = 64 * waves;
    out->kernel_id = id;
    out->workspace_bytes = linrec_workspace_bytes_for_tiles(q.numseq * tiles_per_row);
    return LINREC_OK;
  }

  if (family == LINREC_FAMILY_TILE) {
    if (q.elem_stride != 1 && q.seqlen != 1) return LINREC_E_UNSUPPORTED;
    if (q.numseq > 1 && q.row_stride < q.seqlen && q.row_stride > -q.seqlen) return LINREC_E_INVALID;
    const int vec = q.base_mis >= 0 ? fv : 1;
    const int64_t max_slots = vec > 1 ? full_slots : q.seqlen;
    int waves, slots, carry;
    if (vec == 1) {
      waves = 4; slots = 4;
      carry = max_slots > 4 * 4 * 64 ? 1 : 0;
    } else {
      carry = 0;
      // Few slots per lane win wherever a row still fits (measured at 2^25 elements, forward:
      // 256-element rows w1 s1 60 us, 1024 w4 s1 63 us against w1 s4 64 us, 2048 w4 s2 63 us
      // against w1 s8 65 us, 4096 w4 s4 and w8 s2 62 us, 8192 w16 s2 63 us against w4 s8 65 us); rows that
      // fill their tile only partly prefer more waves to more slots (3000 elements: w8 s2 72 / 120 us
      // against w4 s4 76 / 132 us).
      // A row that fills little more than half of such a tile leaves every other wave idle from the start;
      // fp32 rows in the lower part of a bucket take half the waves and twice the slots (516 elements:
      // w2 s2 74 / 123 us against w4 s1 86 / 131 us; 260 elements: w1 s2 72 / 137 us against w2 s1 85 / 136 us;
      // from three quarters of the tile on the wider workgroup wins: 800 elements 68 / 112 against 73 / 116 us).
      if (max_slots <= 64) { waves = 1; slots = 1; }
      else if (max_slots <= 128) { waves = 2; slots = 1; if (!half && max_slots <= 80) { waves = 1; slots = 2; } }
      else if (max_slots <= 256) { waves = 4; slots = 1; if (!half && max_slots <= 192) { waves = 2; slots = 2; } }
      else if (max_slots <= 512) { waves = 4; slots = 2; }
      else if (max_slots <= 1024) { waves = 8; slots = 2; }
      else if (max_slots <= 2048) { waves = 16; slots = 2; }
      else if (max_slots <= 4096 && !half) { waves = 16; slots = 4; }
      else { waves = 8; slots = half ? 4 : 8; carry = 1; }
      // Few rows of a few thousand elements: split them so that the whole chip has work.
      if (!carry && max_slots > 1024 && q.numseq < q.at(kSplitBelowRows)) { waves = 4; slots = half ? 2 : 4; carry = 1; }
    }
    if (tune && tune->family == LINREC_FAMILY_TILE) {
      if (tune->waves > 0) waves = tune->waves;
      if (tune->slots > 0) slots = tune->slots;
      if (tune->carry >= 0) carry = tune->carry;
      else carry = max_slots > int64_t(waves) * slots * 64 ? 1 : 0;
    }
    const int64_t tile_slots = int64_t(waves) * slots * 64;
    const int64_t tiles_per_row = ceil_div(max_slots, tile_slots);
    if (!carry && tiles_per_row > 1) return LINREC_E_UNSUPPORTED;  // row does not fit one tile
    int tasks = 1;
    if (carry && tune && tune->family == LINREC_FAMILY_TILE && tune->tasks > 1) tasks = tune->tasks;
    if (tasks > q.numseq) tasks = int(q.numseq);
    const int64_t row_groups = ceil_div(q.numseq, tasks);
    tasks = int(ceil_div(q.numseq, row_groups));
    // kernel-table code for the carry column: 0 single tile, 1 one tile per workgroup, 2 several
    const int id = find_kernel(q.dtype, LINREC_FAMILY_TILE, waves, slots, vec, mode, desc, carry ? (tasks > 1 ? 2 : 1) : 0);
    if (id < 0) return LINREC_E_UNSUPPORTED;
    const int64_t tiles = row_groups * tiles_per_row;  // workgroups
    if (q.numseq * tiles_per_row > 2147483647LL) return LINREC_E_TOO_LARGE;
    out->family = LINREC_FAMILY_TILE;
    out->waves = waves; out->slots = slots; out->vec = vec; out->carry = carry;
    out->tiles_per_row = int32_t(tiles_per_row);
    out->tasks = tasks;
    out->grid = tiles;
    out->block = 64 * waves;
    out->kernel_id = id;
    out->workspace_bytes = carry ? linrec_workspace_bytes_for_tiles(q.numseq * tiles_per_row) : 0;
    return LINREC_OK;
  }

  if (family == LINREC_FAMILY_SEGMENT) {
    if (q.elem_stride == 1 && q.seqlen != 1) return LINREC_E_UNSUPPORTED;
    const bool given = tune && tune->family == LINREC_FAMILY_SEGMENT;
    // rows per lane: 8 bytes' worth when that leaves at least a wave of lanes, fewer otherwise; fp32 from 512
    // rows on: four rows (16-byte accesses, a wave reads 1 KiB of every position), which the backward likes
    // (forward / backward in us, four rows against two at their best segment counts: 700 x 100000 278 / 409
    // against 304 / 465, 2200 x 16384 137 / 191 against 141 / 205, 3000 x 8000 91 / 122 against 96 / 134, 5000 x
    // 5000 97 / 130 against 97 / 136; 512 x 65536 114 / 157 against 112 / 154, 1024 x 32768 113 / 152 against 109 /
    // 151; 256 x 65536 62 / 84 against 60 / 83: left at two)
    int vec = given && tune->waves > 0 ? tune->waves : 8 / elem_size_of(q.dtype);
    if (!(given && tune->waves > 0)) {
      // (where segments of at least 32 positions of four rows per lane still make all the waves the launch is to have)
      if (q.dtype == LINREC_DTYPE_F32 && q.numseq / 4 >= q.at(128) && q.numseq * q.seqlen >= 4 * 32 * 64 * segment_waves(q)) vec = 4;
      while (vec > 1 && q.numseq / vec < 64) vec >>= 1;
    }
    auto rows_fit = [&](int v) {  // v adjacent rows per lane: adjacent in memory, aligned, never across a batch
      return v <= fv && q.row_stride == 1 && q.col_phase % v == 0 && q.elem_stride % v == 0 && q.numseq % v == 0 &&
             (!q.batched() || (q.rows_per_batch % v == 0 && q.batch_stride % v == 0));
    };
    while (vec > 1 && !rows_fit(vec)) {
      if (given && tune->waves > 0) return LINREC_E_UNSUPPORTED;
      vec >>= 1;
    }
    const int depth = given && tune->slots > 0 ? tune->slots : 8;
    const int id = find_kernel(q.dtype, LINREC_FAMILY_SEGMENT, 4, depth, vec, mode, desc, linrec::PHASE_APPLY);
    if (id < 0 || find_kernel(q.dtype, LINREC_FAMILY_SEGMENT, 4, depth, vec, mode, desc, linrec::PHASE_REDUCE) < 0)
      return LINREC_E_UNSUPPORTED;
    // Lanes are numbered segment by segment without padding, so few or odd row counts leave no lanes idle.
    // Never more waves than the target: the waves beyond a whole number per SIMD would run alone at the
    // end (12288 x 4096, 96 waves per segment: 10 segments 174 / 268 us, 11 segments 193 / 287 us)
    const int64_t lanes = ceil_div(q.numseq, vec);
    int64_t segments = given && tune->tasks > 0 ? tune->tasks : std::max<int64_t>(1, segment_waves(q) * 64 / lanes);
    if (segments > kSegmentMaxSegments) {
      if (given && tune->tasks > 0) return LINREC_E_UNSUPPORTED;
      segments = kSegmentMaxSegments;
    }
    // whole batches per segment, at least four of them
    int64_t seg_len = ceil_div(ceil_div(q.seqlen, segments), depth) * depth;
    if (seg_len < 4 * depth && !(given && tune->tasks > 0)) seg_len = 4 * depth;
    segments = ceil_div(q.seqlen, seg_len);
    out->family = LINREC_FAMILY_SEGMENT;
    out->waves = 4; out->slots = depth; out->vec = vec; out->carry = 0;
    out->tiles_per_row = int(segments);
    out->tasks = int(seg_len);
    out->grid = ceil_div(lanes * segments, 64);
    out->block = 64;
    out->kernel_id = id;
    // the maps live in the upper half of the workspace (the lower half is the look-back kernels')
    out->workspace_bytes = 2 * (segment_maps_bytes(q.numseq, segments) + 256);
    return LINREC_OK;
  }

  // Column drift: column blocks in teams along the scan axis (tuning: `waves` = waves per workgroup,
  // `slots` = positions per run, `carry` = rows per lane, `tasks` = team size).
  if (family == LINREC_FAMILY_COLDRIFT) {
    const bool given = tune && tune->family == LINREC_FAMILY_COLDRIFT;
    // (a lane takes four bytes' worth of rows: a wave reads 256 bytes of every position)
    const int vec = colblock_rows_per_lane(q, given && tune->carry > 0 ? tune->carry : half ? 2 : 1);
    if (vec == 0) return LINREC_E_UNSUPPORTED;
    int waves = 0, depth = 0, id = -1;
    // (waves, positions per run) in the planner's order of preference: forward 16 waves with runs of 8;
    // the backward holds three tensors of four steps, which 8 waves have the registers for in runs of 16
    // (4096 x 16384 255.5 us against 266.6 us for 16 waves with runs of 4; forward 167.2 against 157.1 us)
    const int fwd_shapes[][2] = {{16, 8}, {8, 16}};
    const int bwd_shapes[][2] = {{8, 16}, {16, 4}};
    for (const auto& wd : q.is_bwd ? bwd_shapes : fwd_shapes) {
      if (given && tune->waves > 0 && wd[0] != tune->waves) continue;
      if (given && tune->slots > 0 && wd[1] != tune->slots) continue;
      id = find_kernel(q.dtype, LINREC_FAMILY_COLDRIFT, wd[0], wd[1], vec, mode, desc, 1);
      if (id >= 0) {
        waves = wd[0];
        depth = wd[1];
        break;
      }
    }
    if (id < 0) return LINREC_E_UNSUPPORTED;
    const int64_t blocks = ceil_div(ceil_div(q.numseq, vec), 64);
    const int64_t steps = ceil_div(q.seqlen, int64_t(waves) * depth);
    // every workgroup of the launch has to be resident at once: team mates take the steps of a block of rows in turn
    const int64_t resident = int64_t(workgroups_per_cu(id, 64 * waves, 1)) * q.cus;
    const int64_t team = given && tune->tasks > 0 ? tune->tasks : coldrift_team(q, blocks, steps, resident, waves);
    // (a wave collects one team mate's map: a team has at most as many members as a workgroup has waves)
    if (team < 1 || team > waves || team > steps || blocks * team > resident) return LINREC_E_UNSUPPORTED;
    const int64_t rows_per_block = int64_t(64) * vec;
    if (blocks * steps * rows_per_block > 2147483647LL) return LINREC_E_TOO_LARGE;
    out->family = LINREC_FAMILY_COLDRIFT;
    out->waves = waves; out->slots = depth; out->vec = vec; out->carry = 1;
    out->tiles_per_row = int32_t(steps);
    out->tasks = int32_t(team);
    out->grid = blocks * team;
    out->block = 64 * waves;
    out->kernel_id = id;
    out->workspace_bytes = linrec_workspace_bytes_for_tiles(blocks * steps * rows_per_block);
    return LINREC_OK;
  }

  // Column block: the waves of a workgroup share rows (tuning: family COLUMN with carry = lane groups per
  // wave, 1, 2 or 4).
  if (family == LINREC_FAMILY_COLUMN && (use_colblock || (tune && tune->family == LINREC_FAMILY_COLUMN && tune->carry >= 1))) {
    const bool given = tune && tune->family == LINREC_FAMILY_COLUMN && tune->carry >= 1;
    const int vec = colblock_rows_per_lane(q, given && tune->waves > 0 ? tune->waves : 0);
    if (vec == 0) return LINREC_E_UNSUPPORTED;
    const int groups = given ? tune->carry : use_colblock;
    int depth = 0;
    const int id = colblock_kernel_for(q, vec, groups, given && tune->slots > 0 ? tune->slots : 0, mode, desc, &depth);
    if (id < 0) return LINREC_E_UNSUPPORTED;
    out->family = LINREC_FAMILY_COLUMN;
    out->waves = kColblockWaves; out->slots = depth; out->vec = vec; out->carry = groups;
    out->tiles_per_row = int(ceil_div(q.seqlen, int64_t(kColblockWaves) * groups * depth));
    out->tasks = 1;
    out->grid = ceil_div(ceil_div(q.numseq, vec), 64 / groups);
    if (out->grid > 2147483647LL) return LINREC_E_TOO_LARGE;
    out->block = 64 * kColblockWaves;
    out->kernel_id = id;
    out->workspace_bytes = 0;
    return LINREC_OK;
  }

  // Column / naive: one lane per row, or per 2 .. 16 bytes' worth of adjacent rows.
  if (family == LINREC_FAMILY_COLUMN && q.row_stride != 1 && q.numseq != 1 && q.rows_per_batch != 1) return LINREC_E_UNSUPPORTED;
  const bool depth_given = tune && tune->family == family && tune->slots > 0;
  const bool width_given = tune && tune->family == family && tune->waves > 0;
  const int cap = family != LINREC_FAMILY_COLUMN ? 1 : width_given ? tune->waves : kColumnRowsPerLane(q);
  // candidate access widths the layout allows: the preferred one first, then narrower, then wider
  // Timesteps in flight per lane: 8, or 16 when the launch has at most one wave per SIMD and each wave
  // has to keep more of the memory system busy (32768 x 2048: 145 / 254 us against 205 / 304 us;
  // 65536 x 1024 the same either way; 80000 x 1024: 174 / 317 us against 158 / 307 us).
  const bool deep = ceil_div(ceil_div(q.numseq, cap), 64) <= 4 * q.cus;
  int vec = 1, depth = depth_given ? tune->slots : 8, id = -1;
  for (int pass = 0; pass < 2 && id < 0; ++pass) {
    for (int v = pass == 0 ? cap : fv; v >= 1 && id < 0; v >>= 1) {
      if (pass == 1 && (v <= cap || width_given)) break;
      if (v > 1 && (family != LINREC_FAMILY_COLUMN || v > fv || q.col_phase % v || q.elem_stride % v || q.numseq % v ||
                    (q.batched() && (q.rows_per_batch % v || q.batch_stride % v))))
        continue;
      const int fam = v > 1 ? LINREC_FAMILY_COLUMN : LINREC_FAMILY_NAIVE;
      if (depth_given) {
        id = find_kernel(q.dtype, fam, 4, depth, v, mode, desc, 0);
      } else {
        for (int d : {deep ? 16 : 8, 8, 4, 16}) {
          id = find_kernel(q.dtype, fam, 4, d, v, mode, desc, 0);
          if (id >= 0) { depth = d; break; }
        }
      }
      if (id >= 0) vec = v;
    }
  }
  if (id < 0) return LINREC_E_UNSUPPORTED;
  out->family = family;
  out->waves = 4; out->slots = depth; out->vec = vec; out->carry = 0;
  out->tiles_per_row = 1;
  out->tasks = 1;
  // Workgroups of four waves when they spread evenly over the CUs, single waves otherwise: a CU
  // serves its workgroups oldest first, so the CUs that get one workgroup more than the others set
  // the time (transposed 300000 x 256: 192.6 / 323.1 us with four waves, 180.2 / 304.8 us with one;
  // 150000 x 256: 104.5 / 180.4 us against 87.7 / 158.2 us; 262144 x 256, 512 workgroups of four
  // waves: 132.5 / 223.8 us against 131.9 / 229.6 us).
  const int64_t lanes = ceil_div(q.numseq, vec);
  const int block = lanes % (256 * q.cus) == 0 ? 256 : 64;
  out->grid = ceil_div(lanes, block);
  if (out->grid > 2147483647LL) return LINREC_E_TOO_LARGE;
  out->block = block;
  out->kernel_id = id;
  out->workspace_bytes = 0;
  return LINREC_OK;
}

// Workspace = header | completion counters | descriptors.  The counter tree of T tiles needs
// sum_l ceil(T / 32^l) < T/31 + 8 words; T/16 + 64 words are reserved.
struct WorkspaceLayout {
  size_t counters_offset, desc_offset;
  int64_t tiles;  // descriptors (and tiles of one launch) the workspace has room for
};

size_t counter_bytes_for(int64_t tiles) { return ((size_t(tiles) / 16 + 64) * 4 + 15) & ~size_t(15); }

// (All of this in the lower half of the buffer; the upper half is scratch without a life beyond
// one call: the maps of the segmented column launches.  A map must never land where a later launch
// reads descriptors, whose validity is a bit pattern.)
WorkspaceLayout workspace_layout(size_t whole_bytes) {
  const size_t bytes = whole_bytes / 2;
  WorkspaceLayout lay{sizeof(linrec::CarryHeader), 0, 0};
  const size_t fixed = sizeof(linrec::CarryHeader) + 64 * 4 + 16;
  if (bytes <= fixed) return lay;
  // 16 bytes of descriptors and a quarter byte of counters per tile
  int64_t tiles = int64_t((bytes - fixed) * 4 / 65);
  while (tiles > 0 && sizeof(linrec::CarryHeader) + counter_bytes_for(tiles) + size_t(tiles) * 16 > bytes) --tiles;
  lay.tiles = tiles;
  lay.desc_offset = sizeof(linrec::CarryHeader) + counter_bytes_for(tiles);
  return lay;
}

// Polls of one look-back window before a tile gives up (about a second of waiting by default).  One value
// for the process: a wait that runs out costs time, never the result, so no caller depends on another's choice.
std::atomic<int> g_spin_limit{1 << 20};

#ifdef LINREC_PHASE_TIMING
unsigned long long* g_timing_buffer = nullptr;
#endif

// Common misalignment of a set of pointers in elements of the storage type (0 .. 16/size - 1), or
// -1 when they disagree or are not element-aligned.
int common_misalignment(const void* const* ptrs, int n, int dtype) {
  const uintptr_t es = uintptr_t(elem_size_of(dtype));
  int mis = -2;
  for (int i = 0; i < n; ++i) {
    if (reinterpret_cast<uintptr_t>(ptrs[i]) % es) return -1;
    const int m = int((reinterpret_cast<uintptr_t>(ptrs[i]) / es) % uintptr_t(full_vec_of(dtype)));
    if (mis == -2) mis = m;
    else if (mis != m) return -1;
  }
  return mis;
}

int launch(const linrec_plan_t& plan, const Problem& q, const void* in0, const void* coef,
           const void* aux, void* out0, void* out1, void* workspace, size_t workspace_bytes,
           hipStream_t stream) {
  if (plan.kernel_id < 0) return LINREC_OK;  // empty problem
  const KernelEntry& k = kKernels[plan.kernel_id];
  if (plan.family == LINREC_FAMILY_TILE || plan.family == LINREC_FAMILY_STREAM || plan.family == LINREC_FAMILY_TEAM ||
      plan.family == LINREC_FAMILY_SWEEP || plan.family == LINREC_FAMILY_DRIFT) {
    if (plan.carry) {
      if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 15u) || workspace_bytes < plan.workspace_bytes)
        return LINREC_E_WORKSPACE;
    }
    TileArgs a;
    a.in0 = in0; a.coef = coef; a.aux = aux; a.out0 = out0; a.out1 = out1;
    a.row_stride = q.row_stride;
    a.num_tiles = plan.grid;
    a.seqlen = int(q.seqlen);
    a.tiles_per_row = plan.tiles_per_row;
    a.base_mis = q.base_mis > 0 ? q.base_mis : 0;  // in elements of the storage type
    a.numseq = q.numseq;
    a.tasks = plan.tasks > 0 ? plan.tasks : 1;
    a.row_groups = plan.family == LINREC_FAMILY_TEAM ? q.numseq
                   : plan.family == LINREC_FAMILY_SWEEP || plan.family == LINREC_FAMILY_DRIFT ? plan.grid / a.tasks
                                                                                              : ceil_div(q.numseq, a.tasks);
    a.ws = static_cast<linrec::CarryHeader*>(workspace);
    a.counters = nullptr; a.desc = nullptr; a.ws_tiles = 0;
    if (plan.carry) {
      // fixed split of the workspace, a function of its size only, so that every launch on it
      // finds the counters where the previous one left them zeroed
      const WorkspaceLayout lay = workspace_layout(workspace_bytes);
      if (lay.tiles < q.numseq * plan.tiles_per_row) return LINREC_E_WORKSPACE;
      a.counters = reinterpret_cast<uint32_t*>(static_cast<char*>(workspace) + lay.counters_offset);
      a.desc = reinterpret_cast<uint64_t*>(static_cast<char*>(workspace) + lay.desc_offset);
      a.ws_tiles = lay.tiles;
    }
    a.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
    // (a plan made elsewhere, or edited: never a team the kernel was not compiled for)
    if (plan.family == LINREC_FAMILY_DRIFT && a.tasks > drift_max_team(k.waves, k.slots, k.vec)) return LINREC_E_INVALID;
#ifdef LINREC_PHASE_TIMING
    a.timing = g_timing_buffer;
#endif
    void* args[] = {&a};
    hipError_t e = hipLaunchKernel(k.fn, dim3((unsigned)plan.grid), dim3((unsigned)plan.block), args, 0, stream);
    return e == hipSuccess ? int(hipGetLastError()) : int(e);
  }
  if (plan.family == LINREC_FAMILY_FLAT) {
    linrec::FlatArgs a;
    a.in0 = in0; a.coef = coef; a.aux = aux; a.out0 = out0; a.out1 = out1;
    a.total = q.numseq * q.seqlen; a.seqlen = int(q.seqlen);
    a.zero_pos = q.reverse ? int(q.seqlen) - 1 : 0;
    void* args[] = {&a};
    hipError_t e = hipLaunchKernel(k.fn, dim3((unsigned)plan.grid), dim3((unsigned)plan.block), args, 0, stream);
    return e == hipSuccess ? int(hipGetLastError()) : int(e);
  }
  if (plan.family == LINREC_FAMILY_GROUP) {
    linrec::GroupArgs a;
    a.in0 = in0; a.coef = coef; a.aux = aux; a.out0 = out0; a.out1 = out1;
    a.row_stride = q.row_stride; a.numseq = q.numseq; a.seqlen = int(q.seqlen); a.group = plan.tasks;
    a.base_mis = q.base_mis > 0 ? q.base_mis : 0;
    void* args[] = {&a};
    hipError_t e = hipLaunchKernel(k.fn, dim3((unsigned)plan.grid), dim3((unsigned)plan.block), args, 0, stream);
    return e == hipSuccess ? int(hipGetLastError()) : int(e);
  }
  ColumnArgs a;
  a.in0 = in0; a.coef = coef; a.aux = aux; a.out0 = out0; a.out1 = out1;
  a.row_stride = q.row_stride; a.elem_stride = q.elem_stride;
  a.numseq = q.numseq; a.seqlen = int(q.seqlen);
  a.seg_len = 0; a.maps = nullptr; a.segments = 1; a.lanes_per_segment = 0;
  a.rows_per_batch = q.batched() ? q.rows_per_batch : q.numseq;
  a.batch_stride = q.batched() ? q.batch_stride : 0;
  if (plan.family == LINREC_FAMILY_COLDRIFT) {
    if (plan.block != 64 * k.waves || plan.tasks < 1 || plan.tasks > k.waves) return LINREC_E_INVALID;  // (what the kernel is compiled for)
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 15u) || workspace_bytes < plan.workspace_bytes)
      return LINREC_E_WORKSPACE;
    const WorkspaceLayout lay = workspace_layout(workspace_bytes);
    const int64_t rows_per_block = int64_t(64) * plan.vec;
    if (lay.tiles < (plan.grid / plan.tasks) * plan.tiles_per_row * rows_per_block) return LINREC_E_WORKSPACE;
    linrec::ColDriftArgs d{};
    d.col = a;
    d.chain.num_tiles = plan.grid;
    d.chain.tasks = plan.tasks;
    d.chain.ws = static_cast<linrec::CarryHeader*>(workspace);
    d.chain.counters = reinterpret_cast<uint32_t*>(static_cast<char*>(workspace) + lay.counters_offset);
    d.chain.desc = reinterpret_cast<uint64_t*>(static_cast<char*>(workspace) + lay.desc_offset);
    d.chain.ws_tiles = lay.tiles;
    d.chain.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
    void* dargs[] = {&d};
    hipError_t e = hipLaunchKernel(k.fn, dim3((unsigned)plan.grid), dim3((unsigned)plan.block), dargs, 0, stream);
    return e == hipSuccess ? int(hipGetLastError()) : int(e);
  }
  void* args[] = {&a};
  if (plan.family == LINREC_FAMILY_SEGMENT) {
    const int64_t segments = plan.tiles_per_row;
    const size_t maps_offset = (workspace_bytes / 2 + 255) & ~size_t(255);
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 15u) || workspace_bytes < plan.workspace_bytes ||
        workspace_bytes - maps_offset < segment_maps_bytes(q.numseq, segments))
      return LINREC_E_WORKSPACE;
    a.seg_len = plan.tasks;
    a.maps = reinterpret_cast<float*>(static_cast<char*>(workspace) + maps_offset);
    const int reduce_id = find_kernel(k.dtype, LINREC_FAMILY_SEGMENT, 4, k.slots, k.vec, k.mode, k.desc, linrec::PHASE_REDUCE);
    if (reduce_id < 0) return LINREC_E_UNSUPPORTED;
    a.segments = int(segments);
    a.lanes_per_segment = ceil_div(q.numseq, int64_t(k.vec));
    if (plan.grid > 2147483647LL) return LINREC_E_TOO_LARGE;
    const dim3 grid((unsigned)plan.grid), block((unsigned)plan.block);
    hipError_t e = hipLaunchKernel(kKernels[reduce_id].fn, grid, block, args, 0, stream);
    if (e != hipSuccess) return int(e);
    linrec::segment_carry_kernel<><<<dim3((unsigned)ceil_div(q.numseq, 4)), dim3(256), 0, stream>>>(a.maps, q.numseq, int(segments));
    e = hipLaunchKernel(k.fn, grid, block, args, 0, stream);
    return e == hipSuccess ? int(hipGetLastError()) : int(e);
  }
  hipError_t e = hipLaunchKernel(k.fn, dim3((unsigned)plan.grid), dim3((unsigned)plan.block), args, 0, stream);
  return e == hipSuccess ? int(hipGetLastError()) : int(e);
}

// The problem a forward call poses (misalignment of its pointers, device in hand).
Problem forward_problem(int dtype, const void* inputs, const void* coeffs, const void* outputs, int64_t numseq,
                        int64_t seqlen, int64_t row_stride, int64_t elem_stride, int64_t rows_per_batch,
                        int64_t batch_stride, int reverse) {
  const void* ptrs[] = {inputs, coeffs, outputs};
  Problem q{numseq, seqlen, row_stride, elem_stride, reverse, 0, common_misalignment(ptrs, 3, dtype), false, dtype, 0,
            rows_per_batch, batch_stride};
  q.aligned16 = q.base_mis == 0;
  q.col_phase = q.base_mis >= 0 ? q.base_mis : 1;
  q.cus = compute_units();
  return q;
}

__global__ __launch_bounds__(256) void copy_kernel(const linrec::v4f* __restrict__ src,
                                                   linrec::v4f* __restrict__ dst, long long n4) {
  // 4 slots per lane, 64-lane interleave: the access pattern of tile_kernel<4, 4, 4, ...>
  const long long base = (long long)blockIdx.x * 4096 / 4 + (threadIdx.x >> 6) * 256 + (threadIdx.x & 63);
  linrec::v4f r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
    if (base + j * 64 < n4) r[j] = __builtin_nontemporal_load(src + base + j * 64);
#pragma unroll
  for (int j = 0; j < 4; ++j)
    if (base + j * 64 < n4) __builtin_nontemporal_store(r[j], dst + base + j * 64);
}

struct MixArgs {
  const linrec::v4f* src[3];
  linrec::v4f* dst[2];
  long long n4;
  long long group0;  // first workgroup-sized block of 1024 slots this launch covers
  int hold_lo, hold_bits, index_bits;  // launch order other than ascending addresses, see mix_block
};

// The block of 1024 slots workgroup `b` of the launch takes.  With hold_bits > 0 the launch (of 2^index_bits
// blocks) goes through the blocks in an order that keeps bits [hold_lo, hold_lo + hold_bits) of the block
// index the same for as long as possible: they become the slowest-changing ones, so the blocks in flight at
// any moment all agree in them.
__device__ __forceinline__ long long mix_block(const MixArgs& a, long long b) {
  if (a.hold_bits <= 0) return a.group0 + b;
  const int above = a.index_bits - a.hold_lo - a.hold_bits;  // bits of the index above the held ones
  const long long low = b & ((1ll << a.hold_lo) - 1);
  const long long rest = b >> a.hold_lo;
  const long long held = rest >> above;
  const long long mid = rest & ((1ll << above) - 1);
  return low | (held << a.hold_lo) | (mid << (a.hold_lo + a.hold_bits));
}

// R streams in, W streams out, the access pattern of tile_kernel<4, 4, 4, ...>; the loads stay
// alive when nothing is stored because a store hangs on their (never matching) sum.
// CHECK: the block may reach past the end (only the last, partial block is launched that way; bounds
// checks on every access cost a memory-only kernel about 5 % of its rate).
template <int R, int W, bool CHECK>
__global__ __launch_bounds__(256) void mix_kernel(MixArgs a) {
  const long long base = mix_block(a, blockIdx.x) * 1024 + (threadIdx.x >> 6) * 256 + (threadIdx.x & 63);
  linrec::v4f acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = linrec::v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (!CHECK || base + j * 64 < a.n4) acc[j] += __builtin_nontemporal_load(a.src[r] + base + j * 64);
  }
  if constexpr (W > 0) {
#pragma unroll
    for (int w = 0; w < W; ++w) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (!CHECK || base + j * 64 < a.n4) __builtin_nontemporal_store(acc[j], a.dst[w] + base + j * 64);
    }
  } else {
    if (acc[0].x + acc[1].y + acc[2].z + acc[3].w == 12345.678f && a.dst[0]) a.dst[0][0] = acc[0];
  }
}

// 64 x 64 tile through LDS: both the reads and the writes run along the unit-stride axis of their
// matrix, four elements per lane where alignment and bounds allow.
template <typename E>
__global__ __launch_bounds__(256) void transpose_kernel(const E* __restrict__ src, E* __restrict__ dst, long long rows,
                                                        long long cols) {
  __shared__ E tile[64][64 + 4 / sizeof(E) + 1];
  typedef E V4 __attribute__((ext_vector_type(4)));
  const long long mat = (long long)blockIdx.z * rows * cols;
  src += mat;
  dst += mat;
  const long long c0 = (long long)blockIdx.x * 64, r0 = (long long)blockIdx.y * 64;
  const int lr = threadIdx.x >> 4, lc = (threadIdx.x & 15) * 4;
  const bool src_vec = (cols % 4 == 0) && ((reinterpret_cast<uintptr_t>(src) & (4 * sizeof(E) - 1)) == 0);
  const bool dst_vec = (rows % 4 == 0) && ((reinterpret_cast<uintptr_t>(dst) & (4 * sizeof(E) - 1)) == 0);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const long long r = r0 + lr + 16 * k, c = c0 + lc;
    if (r < rows) {
      if (src_vec && c + 3 < cols) {
        const V4 v = __builtin_nontemporal_load(reinterpret_cast<const V4*>(src + r * cols + c));
#pragma unroll
        for (int i = 0; i < 4; ++i) tile[lr + 16 * k][lc + i] = v[i];
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (c + i < cols) tile[lr + 16 * k][lc + i] = src[r * cols + c + i];
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const long long c = c0 + lr + 16 * k, r = r0 + lc;  // row c of the transpose, columns r .. r+3
    if (c < cols) {
      if (dst_vec && r + 3 < rows) {
        V4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = tile[lc + i][lr + 16 * k];
        __builtin_nontemporal_store(v, reinterpret_cast<V4*>(dst + c * rows + r));
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (r + i < rows) dst[c * rows + r + i] = tile[lc + i][lr + 16 * k];
      }
    }
  }
}

__global__ void copy_tail_kernel(const float* src, float* dst, long long from, long long n) {
  const long long i = from + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

}  // namespace

extern "C" {

int linrec_hip_abi_version(void) { return 1; }

const char* linrec_hip_error_string(int code) {
  switch (code) {
    case LINREC_OK: return "success";
    case LINREC_E_INVALID: return "linrec: invalid argument (null pointer, negative size or overlapping rows)";
    case LINREC_E_WORKSPACE: return "linrec: workspace missing, not 16-byte aligned or too small";
    case LINREC_E_UNSUPPORTED: return "linrec: no compiled kernel matches the requested tuning/layout";
    case LINREC_E_TOO_LARGE: return "linrec: problem too large (seqlen or tile count beyond 2^31)";
    case LINREC_E_SCRATCH: return "linrec: the call needs more scratch than the library's static 4 MiB array holds";
    default: return code > 0 ? hipGetErrorString(hipError_t(code)) : "linrec: unknown error";
  }
}

size_t linrec_workspace_bytes_for_tiles(int64_t max_tiles) {
  if (max_tiles <= 0) return 0;
  size_t bytes = 2 * (sizeof(linrec::CarryHeader) + counter_bytes_for(max_tiles) + size_t(max_tiles) * 16 + 64);
  while (workspace_layout(bytes).tiles < max_tiles) bytes += 128;
  return bytes;
}

int linrec_plan(int dtype, const void* any_input, int64_t numseq, int64_t seqlen, int64_t row_stride,
                int64_t elem_stride, int reverse, int is_bwd, const linrec_tuning_t* tuning,
                linrec_plan_t* plan) {
  if (!plan) return LINREC_E_INVALID;
  if (dtype < LINREC_DTYPE_F32 || dtype > LINREC_DTYPE_BF16) return LINREC_E_UNSUPPORTED;
  const void* ptrs[] = {any_input};
  Problem q{numseq, seqlen, row_stride, elem_stride, reverse, is_bwd, common_misalignment(ptrs, 1, dtype), false, dtype, 0};
  q.aligned16 = q.base_mis == 0;
  q.col_phase = q.base_mis >= 0 ? q.base_mis : 1;
  q.cus = compute_units();
  return make_plan(q, tuning, plan);
}

int linrec_plan_f32(const void* any_input, int64_t numseq, int64_t seqlen, int64_t row_stride,
                    int64_t elem_stride, int reverse, int is_bwd, const linrec_tuning_t* tuning,
                    linrec_plan_t* plan) {
  return linrec_plan(LINREC_DTYPE_F32, any_input, numseq, seqlen, row_stride, elem_stride, reverse, is_bwd, tuning, plan);
}

size_t linrec_workspace_bytes_dtype(int dtype, int64_t numseq, int64_t seqlen, int64_t row_stride,
                                    int64_t elem_stride, int align_elems, int is_bwd,
                                    const linrec_tuning_t* tuning) {
  if (dtype < LINREC_DTYPE_F32 || dtype > LINREC_DTYPE_BF16) return 0;
  const int mis = align_elems < 0 ? -1 : align_elems & (full_vec_of(dtype) - 1);
  Problem q{numseq, seqlen, row_stride, elem_stride, 0, is_bwd, mis, mis == 0, dtype, mis >= 0 ? mis : 1};
  q.cus = compute_units();
  linrec_plan_t plan;
  if (make_plan(q, tuning, &plan) != LINREC_OK) return 0;
  return size_t(plan.workspace_bytes);
}

size_t linrec_workspace_bytes(int64_t numseq, int64_t seqlen, int64_t row_stride, int64_t elem_stride,
                              int align_elems, int is_bwd, const linrec_tuning_t* tuning) {
  return linrec_workspace_bytes_dtype(LINREC_DTYPE_F32, numseq, seqlen, row_stride, elem_stride, align_elems, is_bwd, tuning);
}

namespace {

int fwd_impl(int dtype, const void* inputs, const void* coeffs, void* outputs, int64_t numseq, int64_t seqlen,
             int64_t row_stride, int64_t elem_stride, int64_t rows_per_batch, int64_t batch_stride, int reverse,
             void* workspace, size_t workspace_bytes, const linrec_tuning_t* tuning, void* stream,
             size_t workspace_cap = 0) {
  if (numseq < 0 || seqlen < 0 || rows_per_batch < 0) return LINREC_E_INVALID;
  if (dtype < LINREC_DTYPE_F32 || dtype > LINREC_DTYPE_BF16) return LINREC_E_UNSUPPORTED;
  if (numseq == 0 || seqlen == 0) return LINREC_OK;
  if (!inputs || !coeffs || !outputs) return LINREC_E_INVALID;
  Problem q = forward_problem(dtype, inputs, coeffs, outputs, numseq, seqlen, row_stride, elem_stride,
                              rows_per_batch, batch_stride, reverse);
  q.workspace_cap = workspace_cap;
  linrec_plan_t plan;
  int rc = make_plan(q, tuning, &plan);
  if (rc != LINREC_OK) return rc;
  rc = launch(plan, q, inputs, coeffs, nullptr, outputs, nullptr, workspace, workspace_bytes,
              static_cast<hipStream_t>(stream));
  if (rc != LINREC_OK || plan.tail_rows == 0) return rc;
  // the rows the first launch left out
  const Problem t = tail_problem(q, plan.tail_rows);
  const int64_t skip = (numseq - plan.tail_rows) * row_stride * elem_size_of(dtype);
  linrec_plan_t tail;
  rc = make_plan(t, nullptr, &tail);
  if (rc != LINREC_OK) return rc;
  return launch(tail, t, static_cast<const char*>(inputs) + skip, static_cast<const char*>(coeffs) + skip, nullptr,
                static_cast<char*>(outputs) + skip, nullptr, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int bwd_impl(int dtype, const void* d_outputs, const void* coeffs, const void* outputs, void* d_inputs,
             void* d_coeffs, int64_t numseq, int64_t seqlen, int64_t row_stride, int64_t elem_stride,
             int64_t rows_per_batch, int64_t batch_stride, int reverse, void* workspace, size_t workspace_bytes,
             const linrec_tuning_t* tuning, void* stream) {
  if (numseq < 0 || seqlen < 0 || rows_per_batch < 0) return LINREC_E_INVALID;
  if (dtype < LINREC_DTYPE_F32 || dtype > LINREC_DTYPE_BF16) return LINREC_E_UNSUPPORTED;
  if (numseq == 0 || seqlen == 0) return LINREC_OK;
  if (!d_outputs || !coeffs || !outputs || !d_inputs || !d_coeffs) return LINREC_E_INVALID;
  const void* ptrs[] = {d_outputs, coeffs, outputs, d_inputs, d_coeffs};
  Problem q{numseq, seqlen, row_stride, elem_stride, reverse, 1, common_misalignment(ptrs, 5, dtype), false, dtype, 0,
            rows_per_batch, batch_stride};
  q.aligned16 = q.base_mis == 0;
  q.col_phase = q.base_mis >= 0 ? q.base_mis : 1;
  q.cus = compute_units();
  linrec_plan_t plan;
  int rc = make_plan(q, tuning, &plan);
  if (rc != LINREC_OK) return rc;
  rc = launch(plan, q, d_outputs, coeffs, outputs, d_inputs, d_coeffs, workspace, workspace_bytes,
              static_cast<hipStream_t>(stream));
  if (rc != LINREC_OK || plan.tail_rows == 0) return rc;
  const Problem t = tail_problem(q, plan.tail_rows);
  const int64_t skip = (numseq - plan.tail_rows) * row_stride * elem_size_of(dtype);
  linrec_plan_t tail;
  rc = make_plan(t, nullptr, &tail);
  if (rc != LINREC_OK) return rc;
  return launch(tail, t, static_cast<const char*>(d_outputs) + skip, static_cast<const char*>(coeffs) + skip,
                static_cast<const char*>(outputs) + skip, static_cast<char*>(d_inputs) + skip,
                static_cast<char*>(d_coeffs) + skip, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

}  // namespace

int linrec_fwd(int dtype, const void* inputs, const void* coeffs, void* outputs, int64_t numseq,
               int64_t seqlen, int64_t row_stride, int64_t elem_stride, int reverse, void* workspace,
               size_t workspace_bytes, const linrec_tuning_t* tuning, void* stream) {
  return fwd_impl(dtype, inputs, coeffs, outputs, numseq, seqlen, row_stride, elem_stride, 0, 0, reverse, workspace,
                  workspace_bytes, tuning, stream);
}

namespace {

// The launch linrec_fwd_noalloc makes for `q` (q.workspace_cap set): the table's choice where the static array
// holds its workspace, else - without a tuning of the caller's - a kernel that needs less: segments of a strided
// scan axis as many as fit, or the kernels that need no workspace at all (one workgroup per row where the rows
// give a quarter of the chip work; one lane per row or group of rows on a strided scan axis).  `effective`
// receives the tuning to launch with (NULL for the table's choice).
int noalloc_plan(const Problem& q, const linrec_tuning_t* tuning, linrec_plan_t* plan, linrec_tuning_t* storage,
                 const linrec_tuning_t** effective) {
  *effective = tuning;
  const int rc = make_plan(q, tuning, plan);
  if (rc != LINREC_OK) return rc;
  if (plan->workspace_bytes <= q.workspace_cap) return LINREC_OK;
  if (tuning) return LINREC_E_SCRATCH;  // (a caller's own tuning is not second-guessed)
  auto fits = [&](const linrec_tuning_t& t) {
    *storage = t;
    return make_plan(q, storage, plan) == LINREC_OK && plan->family == t.family && plan->workspace_bytes <= q.workspace_cap;
  };
  bool found = false;
  if (q.elem_stride == 1 || q.seqlen == 1) {
    found = q.numseq * 4 >= q.cus && fits(linrec_tuning_t{LINREC_FAMILY_STREAM, 0, 0, -1, 0});
  } else {
    // (the maps of a segmented launch: two floats per row and segment, in the upper half of the workspace)
    const int64_t segments = (int64_t(q.workspace_cap / 2) - 512) / (8 * q.numseq);
    found = segments >= 2 && fits(linrec_tuning_t{LINREC_FAMILY_SEGMENT, 0, 0, -1, int32_t(std::min<int64_t>(segments, kSegmentMaxSegments))});
    found = found || fits(linrec_tuning_t{LINREC_FAMILY_COLUMN, 0, 0, -1, 0}) || fits(linrec_tuning_t{LINREC_FAMILY_NAIVE, 0, 0, -1, 0});
  }
  if (!found) return LINREC_E_SCRATCH;
  *effective = storage;
  return LINREC_OK;
}

}  // namespace

int linrec_plan_noalloc(int dtype, const void* any_input, int64_t numseq, int64_t seqlen, int64_t row_stride,
                        int64_t elem_stride, int reverse, const linrec_tuning_t* tuning, linrec_plan_t* plan) {
  if (!plan) return LINREC_E_INVALID;
  if (dtype < LINREC_DTYPE_F32 || dtype > LINREC_DTYPE_BF16) return LINREC_E_UNSUPPORTED;
  Problem q = forward_problem(dtype, any_input, any_input, any_input, numseq, seqlen, row_stride, elem_stride, 0, 0, reverse);
  q.workspace_cap = kStaticScratchBytes;
  linrec_tuning_t storage;
  const linrec_tuning_t* effective = nullptr;
  return noalloc_plan(q, tuning, plan, &storage, &effective);
}

int linrec_fwd_noalloc(int dtype, const void* inputs, const void* coeffs, void* outputs, int64_t numseq,
                       int64_t seqlen, int64_t row_stride, int64_t elem_stride, int reverse,
                       const linrec_tuning_t* tuning, void* stream) {
  if (numseq < 0 || seqlen < 0) return LINREC_E_INVALID;
  if (dtype < LINREC_DTYPE_F32 || dtype > LINREC_DTYPE_BF16) return LINREC_E_UNSUPPORTED;
  if (numseq == 0 || seqlen == 0) return LINREC_OK;
  if (!inputs || !coeffs || !outputs) return LINREC_E_INVALID;
  // What the call needs follows from its arguments alone, so a call that needs more than the static
  // array holds is turned down before anything is enqueued.
  Problem q = forward_problem(dtype, inputs, coeffs, outputs, numseq, seqlen, row_stride, elem_stride, 0, 0, reverse);
  q.workspace_cap = kStaticScratchBytes;
  linrec_plan_t plan;
  linrec_tuning_t storage;
  const int rc = noalloc_plan(q, tuning, &plan, &storage, &tuning);
  if (rc != LINREC_OK) return rc;
  if (plan.workspace_bytes == 0)
    return fwd_impl(dtype, inputs, coeffs, outputs, numseq, seqlen, row_stride, elem_stride, 0, 0, reverse, nullptr, 0,
                    tuning, stream, kStaticScratchBytes);
  DeviceState* d = device_state();
  if (!d) return int(hipErrorNoDevice);
  if (!d->scratch_ptr) return d->scratch_rc > 0 ? d->scratch_rc : int(hipErrorInvalidSymbol);
  // The array's size is always passed whole: the split into counters and descriptors depends on it.
  return fwd_impl(dtype, inputs, coeffs, outputs, numseq, seqlen, row_stride, elem_stride, 0, 0, reverse, d->scratch_ptr,
                  kStaticScratchBytes, tuning, stream, kStaticScratchBytes);
}

int linrec_noalloc_gave_up_count(void) {
  DeviceState* d = device_state();
  if (!d || !d->scratch_ptr) return -1;
  uint32_t header[4] = {0, 0, 0, 0};
  if (hipMemcpy(header, d->scratch_ptr, sizeof(header), hipMemcpyDeviceToHost) != hipSuccess) {
    (void)hipGetLastError();
    return -1;
  }
  return int(header[1] & 0x7fffffffu);
}

int linrec_bwd(int dtype, const void* d_outputs, const void* coeffs, const void* outputs, void* d_inputs,
               void* d_coeffs, int64_t numseq, int64_t seqlen, int64_t row_stride, int64_t elem_stride,
               int reverse, void* workspace, size_t workspace_bytes, const linrec_tuning_t* tuning,
               void* stream) {
  return bwd_impl(dtype, d_outputs, coeffs, outputs, d_inputs, d_coeffs, numseq, seqlen, row_stride, elem_stride, 0, 0,
                  reverse, workspace, workspace_bytes, tuning, stream);
}

int linrec_fwd_call(const linrec_call_t* c) {
  if (!c) return LINREC_E_INVALID;
  return fwd_impl(c->dtype, c->in0, c->coef, c->out0, c->numseq, c->seqlen, c->row_stride, c->elem_stride, 0, 0, c->reverse,
                  c->workspace, size_t(c->workspace_bytes), nullptr, c->stream);
}

int linrec_bwd_call(const linrec_call_t* c) {
  if (!c) return LINREC_E_INVALID;
  return bwd_impl(c->dtype, c->in0, c->coef, c->aux, c->out0, c->out1, c->numseq, c->seqlen, c->row_stride, c->elem_stride, 0,
                  0, c->reverse, c->workspace, size_t(c->workspace_bytes), nullptr, c->stream);
}

int linrec_fwd_batched(int dtype, const void* inputs, const void* coeffs, void* outputs, int64_t batches,
                       int64_t rows_per_batch, int64_t seqlen, int64_t batch_stride, int64_t row_stride,
                       int64_t elem_stride, int reverse, void* workspace, size_t workspace_bytes,
                       const linrec_tuning_t* tuning, void* stream) {
  if (batches < 0 || rows_per_batch < 0) return LINREC_E_INVALID;
  return fwd_impl(dtype, inputs, coeffs, outputs, batches * rows_per_batch, seqlen, row_stride, elem_stride,
                  rows_per_batch, batch_stride, reverse, workspace, workspace_bytes, tuning, stream);
}

int linrec_bwd_batched(int dtype, const void* d_outputs, const void* coeffs, const void* outputs, void* d_inputs,
                       void* d_coeffs, int64_t batches, int64_t rows_per_batch, int64_t seqlen, int64_t batch_stride,
                       int64_t row_stride, int64_t elem_stride, int reverse, void* workspace, size_t workspace_bytes,
                       const linrec_tuning_t* tuning, void* stream) {
  if (batches < 0 || rows_per_batch < 0) return LINREC_E_INVALID;
  return bwd_impl(dtype, d_outputs, coeffs, outputs, d_inputs, d_coeffs, batches * rows_per_batch, seqlen, row_stride,
                  elem_stride, rows_per_batch, batch_stride, reverse, workspace, workspace_bytes, tuning, stream);
}

int linrec_plan_batched(int dtype, const void* any_input, int64_t batches, int64_t rows_per_batch, int64_t seqlen,
                        int64_t batch_stride, int64_t row_stride, int64_t elem_stride, int reverse, int is_bwd,
                        const linrec_tuning_t* tuning, linrec_plan_t* plan) {
  if (!plan || batches < 0 || rows_per_batch < 0) return LINREC_E_INVALID;
  if (dtype < LINREC_DTYPE_F32 || dtype > LINREC_DTYPE_BF16) return LINREC_E_UNSUPPORTED;
  const void* ptrs[] = {any_input};
  Problem q{batches * rows_per_batch, seqlen, row_stride, elem_stride, reverse, is_bwd,
            common_misalignment(ptrs, 1, dtype), false, dtype, 0, rows_per_batch, batch_stride};
  q.aligned16 = q.base_mis == 0;
  q.col_phase = q.base_mis >= 0 ? q.base_mis : 1;
  q.cus = compute_units();
  return make_plan(q, tuning, plan);
}

int linrec_fwd_f32(const float* inputs, const float* coeffs, float* outputs, int64_t numseq,
                   int64_t seqlen, int64_t row_stride, int64_t elem_stride, int reverse,
                   void* workspace, size_t workspace_bytes, const linrec_tuning_t* tuning,
                   void* stream) {
  return linrec_fwd(LINREC_DTYPE_F32, inputs, coeffs, outputs, numseq, seqlen, row_stride, elem_stride, reverse,
                    workspace, workspace_bytes, tuning, stream);
}

int linrec_bwd_f32(const float* d_outputs, const float* coeffs, const float* outputs,
                   float* d_inputs, float* d_coeffs, int64_t numseq, int64_t seqlen,
                   int64_t row_stride, int64_t elem_stride, int reverse, void* workspace,
                   size_t workspace_bytes, const linrec_tuning_t* tuning, void* stream) {
  return linrec_bwd(LINREC_DTYPE_F32, d_outputs, coeffs, outputs, d_inputs, d_coeffs, numseq, seqlen, row_stride,
                    elem_stride, reverse, workspace, workspace_bytes, tuning, stream);
}

int linrec_set_compute_units(int cus) {
  const int old = g_cu_override.load(std::memory_order_relaxed);
  if (cus >= 0) g_cu_override.store(cus, std::memory_order_relaxed);
  return old;
}

int linrec_compute_units(void) { return compute_units(); }

int linrec_set_spin_limit(int polls) {
  if (polls > 0) return g_spin_limit.exchange(polls, std::memory_order_relaxed);
  return g_spin_limit.load(std::memory_order_relaxed);
}

#ifdef LINREC_PHASE_TIMING
// Debug builds only: device buffer of 8 x uint64 per tile that tile kernels stamp with the 100 MHz
// wall clock at their phase boundaries (NULL switches stamping off).
void linrec_debug_set_timing_buffer(unsigned long long* device_buffer) { g_timing_buffer = device_buffer; }
#endif

int linrec_plan_threshold_count(void) { return kNumPlanThresholds; }

const char* linrec_plan_threshold_name(int index) {
  return index >= 0 && index < kNumPlanThresholds ? kPlanThresholds[index].name : nullptr;
}

int64_t linrec_plan_threshold_value(int index) {
  return index >= 0 && index < kNumPlanThresholds ? kPlanThresholds[index].value : -1;
}

int linrec_kernel_count(void) { return kNumKernels; }

const char* linrec_kernel_name(int kernel_id) {
  return kernel_id >= 0 && kernel_id < kNumKernels ? kKernels[kernel_id].name : nullptr;
}

int linrec_kernel_attrs(int kernel_id, int* num_regs, int* lds_bytes, int* scratch_bytes, int* max_threads) {
  if (kernel_id < 0 || kernel_id >= kNumKernels) return LINREC_E_INVALID;
  hipFuncAttributes attr;
  hipError_t e = hipFuncGetAttributes(&attr, kKernels[kernel_id].fn);
  if (e != hipSuccess) return int(e);
  if (num_regs) *num_regs = attr.numRegs;
  if (lds_bytes) *lds_bytes = int(attr.sharedSizeBytes);
  if (scratch_bytes) *scratch_bytes = int(attr.localSizeBytes);
  if (max_threads) *max_threads = attr.maxThreadsPerBlock;
  return LINREC_OK;
}

int linrec_copy_f32(const float* src, float* dst, int64_t n, void* stream) {
  if (n < 0 || (n > 0 && (!src || !dst))) return LINREC_E_INVALID;
  if (n == 0) return LINREC_OK;
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) return LINREC_E_INVALID;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long n4 = n / 4;
  if (n4 > 0) {
    const long long grid = (n4 + 1023) / 1024;
    if (grid > 2147483647LL) return LINREC_E_TOO_LARGE;
    copy_kernel<<<dim3((unsigned)grid), dim3(256), 0, s>>>(reinterpret_cast<const linrec::v4f*>(src),
                                                           reinterpret_cast<linrec::v4f*>(dst), n4);
  }
  if (n4 * 4 < n) copy_tail_kernel<<<1, 64, 0, s>>>(src, dst, n4 * 4, n);
  return int(hipGetLastError());
}

int linrec_stream_mix_f32(int reads, int writes, const float* src0, const float* src1, const float* src2,
                          float* dst0, float* dst1, int64_t n, void* stream) {
  return linrec_stream_mix_order_f32(reads, writes, src0, src1, src2, dst0, dst1, n, 0, 0, stream);
}

int linrec_stream_mix_order_f32(int reads, int writes, const float* src0, const float* src1, const float* src2,
                                float* dst0, float* dst1, int64_t n, int hold_lo, int hold_bits, void* stream) {
  if (reads < 0 || reads > 3 || writes < 0 || writes > 2 || reads + writes == 0 || n < 0 || (n & 3)) return LINREC_E_INVALID;
  if (hold_lo < 0 || hold_bits < 0) return LINREC_E_INVALID;
  if (n == 0) return LINREC_OK;
  int index_bits = 0;
  if (hold_bits > 0) {
    // whole blocks of 4096 floats only, a power of two of them, and the held bits inside the index
    const int64_t blocks = n / 4096;
    if (n % 4096 != 0 || (blocks & (blocks - 1)) != 0) return LINREC_E_INVALID;
    while ((int64_t(1) << index_bits) < blocks) ++index_bits;
    if (hold_lo + hold_bits > index_bits) return LINREC_E_INVALID;
  }
  const float* srcs[3] = {src0, src1, src2};
  float* dsts[2] = {dst0, dst1};
  MixArgs a{};
  for (int r = 0; r < reads; ++r) {
    if (!srcs[r] || (reinterpret_cast<uintptr_t>(srcs[r]) & 15u)) return LINREC_E_INVALID;
    a.src[r] = reinterpret_cast<const linrec::v4f*>(srcs[r]);
  }
  for (int w = 0; w < writes; ++w) {
    if (!dsts[w] || (reinterpret_cast<uintptr_t>(dsts[w]) & 15u)) return LINREC_E_INVALID;
    a.dst[w] = reinterpret_cast<linrec::v4f*>(dsts[w]);
  }
  a.n4 = n / 4;
  a.hold_lo = hold_lo; a.hold_bits = hold_bits; a.index_bits = index_bits;
  const long long full = a.n4 / 1024;
  if (full > 2147483647LL) return LINREC_E_TOO_LARGE;
  const void* fn = nullptr;
  const void* fn_tail = nullptr;
#define LINREC_MIX_CASE(r, w) \
  if (reads == r && writes == w) { fn = (const void*)&mix_kernel<r, w, false>; fn_tail = (const void*)&mix_kernel<r, w, true>; }
  LINREC_MIX_CASE(1, 0) LINREC_MIX_CASE(2, 0) LINREC_MIX_CASE(3, 0) LINREC_MIX_CASE(0, 1) LINREC_MIX_CASE(0, 2)
  LINREC_MIX_CASE(1, 1) LINREC_MIX_CASE(2, 1) LINREC_MIX_CASE(3, 1) LINREC_MIX_CASE(1, 2) LINREC_MIX_CASE(2, 2)
  LINREC_MIX_CASE(3, 2)
#undef LINREC_MIX_CASE
  if (!fn) return LINREC_E_UNSUPPORTED;
  void* args[] = {&a};
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (full > 0) {
    a.group0 = 0;
    hipError_t e = hipLaunchKernel(fn, dim3((unsigned)full), dim3(256), args, 0, s);
    if (e != hipSuccess) return int(e);
  }
  if (full * 1024 < a.n4) {
    a.group0 = full;
    hipError_t e = hipLaunchKernel(fn_tail, dim3(1), dim3(256), args, 0, s);
    if (e != hipSuccess) return int(e);
  }
  return int(hipGetLastError());
}

int linrec_transpose(int elem_size, const void* src, void* dst, int64_t batch, int64_t rows, int64_t cols,
                     void* stream) {
  if (batch < 0 || rows < 0 || cols < 0 || (elem_size != 2 && elem_size != 4)) return LINREC_E_INVALID;
  if (batch == 0 || rows == 0 || cols == 0) return LINREC_OK;
  if (!src || !dst || (reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % uintptr_t(elem_size))
    return LINREC_E_INVALID;
  const int64_t gx = ceil_div(cols, 64), gy = ceil_div(rows, 64);
  if (gx > 2147483647LL || gy > 65535 || batch > 65535) return LINREC_E_TOO_LARGE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)batch);
  if (elem_size == 4) {
    transpose_kernel<uint32_t><<<grid, dim3(256), 0, s>>>(static_cast<const uint32_t*>(src), static_cast<uint32_t*>(dst), rows, cols);
  } else {
    transpose_kernel<uint16_t><<<grid, dim3(256), 0, s>>>(static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), rows, cols);
  }
  return int(hipGetLastError());
}

}  // extern "C"
