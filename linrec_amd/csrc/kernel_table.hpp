// The kernel table of the gfx950 linear-recurrence scan library: one entry per compiled kernel, in groups that
// are compiled as translation units of their own (kernels_*.hip) and put together in linrec_capi.hip.
#pragma once
#include "../../include/linrec_hip.h"
#include "tile_core.hpp"  // MODE_FWD, MODE_BWD

namespace linrec {

struct KernelEntry {
  const char* name;
  const void* fn;
  int dtype, family, waves, slots, vec, mode, desc, carry;
};

// A group of entries (one translation unit's kernels).
struct KernelGroup {
  const KernelEntry* entries;
  int count;
};
KernelGroup kernels_f32_rows();
KernelGroup kernels_f32_walk();
KernelGroup kernels_f32_teams();
KernelGroup kernels_f32_cols();
KernelGroup kernels_f16_rows();
KernelGroup kernels_f16_cols();
KernelGroup kernels_bf16_rows();
KernelGroup kernels_bf16_cols();

}  // namespace linrec

// ---- entries ----------------------------------------------------------------------------------
// One macro per kernel family; the *_ALL_DIRS forms give the four (pass, direction) instantiations of a
// geometry.  TT is the storage type, DT its LINREC_DTYPE_* code, PFX the prefix of the kernel's name; VEC is
// the number of elements of a slot (16 bytes of TT, or 1).
#define TILE_ENTRY(TT, DT, PFX, NW, S, VEC, MODE, DESC, CARRY)                                 \
  {PFX "tile_w" #NW "_s" #S "_v" #VEC "_" #MODE "_" #DESC "_" #CARRY,                          \
   (const void*)&linrec::tile_kernel<TT, NW, S, VEC, linrec::MODE, DESC != 0, CARRY != 0>, DT, \
   LINREC_FAMILY_TILE, NW, S, VEC, linrec::MODE, DESC, CARRY}
#define TILE_ALL_DIRS(TT, DT, PFX, NW, S, VEC, CARRY)                                          \
  TILE_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 0, CARRY), TILE_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 1, CARRY), \
  TILE_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 0, CARRY), TILE_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 1, CARRY)
#define CHAIN_ENTRY(TT, DT, PFX, NW, S, VEC, MODE, DESC)                                       \
  {PFX "chain_w" #NW "_s" #S "_v" #VEC "_" #MODE "_" #DESC,                                    \
   (const void*)&linrec::chain_kernel<TT, NW, S, VEC, linrec::MODE, DESC != 0>, DT, LINREC_FAMILY_TILE, \
   NW, S, VEC, linrec::MODE, DESC, 2}
#define CHAIN_ALL_DIRS(TT, DT, PFX, NW, S, VEC)                                                \
  CHAIN_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 0), CHAIN_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 1), \
  CHAIN_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 0), CHAIN_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 1)
#define TEAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE, DESC)                                        \
  {PFX "team_w" #NW "_s" #S "_" #MODE "_" #DESC,                                               \
   (const void*)&linrec::team_kernel<TT, NW, S, VEC, linrec::MODE, DESC != 0>, DT, LINREC_FAMILY_TEAM, \
   NW, S, VEC, linrec::MODE, DESC, 1}
#define TEAM_ALL_DIRS(TT, DT, PFX, NW, S, VEC)                                                 \
  TEAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 0), TEAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 1), \
  TEAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 0), TEAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 1)
#define SWEEP_ENTRY(TT, DT, PFX, NW, S, VEC, MODE, DESC)                                       \
  {PFX "sweep_w" #NW "_s" #S "_" #MODE "_" #DESC,                                              \
   (const void*)&linrec::sweep_kernel<TT, NW, S, VEC, linrec::MODE, DESC != 0>, DT, LINREC_FAMILY_SWEEP, \
   NW, S, VEC, linrec::MODE, DESC, 1}
#define SWEEP_ALL_DIRS(TT, DT, PFX, NW, S, VEC)                                                \
  SWEEP_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 0), SWEEP_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 1), \
  SWEEP_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 0), SWEEP_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 1)
// Tiles of loads in flight ahead of the scan: two in the backward with 16 waves of one slot, whose step loads
// only 48 KB (one after the other in one process, us, against 8 waves of two slots with one tile ahead, which one
// tile ahead in 16 waves had beaten by 1 to 4 %: 512 x 65536 112.4 against 117.5, 300 x 65536 68.3 against 71.2,
// 16 x 1048576 60.1 against 63.6, 1 x 33554432 111.6 against 124.5); the forward gains nothing from it.
// (16-bit storage, eight elements per slot: a second tile does not fit the backward's registers and brings the
// forward nothing: one slot bf16 512 x 65536 40.2 against 40.4 us, 16 x 1048576 25.2 against 25.0; two slots
// 512 x 65536 37.1 against 36.7, 16 x 1048576 23.3 against 20.4, 300 x 65536 22.8 against 24.0)
#define DRIFT_TILES_AHEAD(NW, S, VEC, MODE) ((NW) == 16 && (S) == 1 && (VEC) == 4 && linrec::MODE == linrec::MODE_BWD ? 2 : 1)
#define DRIFT_ENTRY(TT, DT, PFX, NW, S, VEC, MODE, DESC)                                        \
  {PFX "drift_w" #NW "_s" #S "_" #MODE "_" #DESC,                                               \
   (const void*)&linrec::drift_kernel<TT, NW, S, VEC, linrec::MODE, DESC != 0, DRIFT_TILES_AHEAD(NW, S, VEC, MODE), ((NW) > 8 ? 4 : 2), !((NW) == 16 && (S) == 2 && (VEC) == 4)>, DT, LINREC_FAMILY_DRIFT, \
   NW, S, VEC, linrec::MODE, DESC, 1}
// ... for rows of whole slots whose last tile is a partial one (`carry` column 2)
#define DRIFT_RAGGED_ENTRY(TT, DT, PFX, NW, S, VEC, MODE, DESC)                                 \
  {PFX "drift_ragged_w" #NW "_s" #S "_" #MODE "_" #DESC,                                        \
   (const void*)&linrec::drift_kernel<TT, NW, S, VEC, linrec::MODE, DESC != 0, DRIFT_TILES_AHEAD(NW, S, VEC, MODE), ((NW) > 8 ? 4 : 2), !((NW) == 16 && (S) == 2 && (VEC) == 4), true>, DT, LINREC_FAMILY_DRIFT, \
   NW, S, VEC, linrec::MODE, DESC, 2}
#define DRIFT_RAGGED_FWD_DIRS(TT, DT, PFX, NW, S, VEC)                                         \
  DRIFT_RAGGED_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 0), DRIFT_RAGGED_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 1)
#define DRIFT_RAGGED_BWD_DIRS(TT, DT, PFX, NW, S, VEC)                                         \
  DRIFT_RAGGED_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 0), DRIFT_RAGGED_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 1)
#define DRIFT_FWD_DIRS(TT, DT, PFX, NW, S, VEC)                                                \
  DRIFT_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 0), DRIFT_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 1)
#define DRIFT_BWD_DIRS(TT, DT, PFX, NW, S, VEC)                                                \
  DRIFT_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 0), DRIFT_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 1)
#define TEAM_FWD_DIRS(TT, DT, PFX, NW, S, VEC)                                                 \
  TEAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 0), TEAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 1)
#define STREAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE, DESC)                                      \
  {PFX "stream_w" #NW "_s" #S "_" #MODE "_" #DESC,                                             \
   (const void*)&linrec::stream_kernel<TT, NW, S, VEC, linrec::MODE, DESC != 0>, DT, LINREC_FAMILY_STREAM, \
   NW, S, VEC, linrec::MODE, DESC, 0}
#define STREAM_ALL_DIRS(TT, DT, PFX, NW, S, VEC)                                               \
  STREAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 0), STREAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_FWD, 1), \
  STREAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 0), STREAM_ENTRY(TT, DT, PFX, NW, S, VEC, MODE_BWD, 1)
#define GROUP_ENTRY(TT, DT, PFX, VEC, MODE, DESC)                                              \
  {PFX "group_v" #VEC "_" #MODE "_" #DESC,                                                     \
   (const void*)&linrec::group_kernel<TT, VEC, linrec::MODE, DESC != 0>, DT, LINREC_FAMILY_GROUP, 4, 1, VEC, \
   linrec::MODE, DESC, 0}
#define GROUP_ALL_DIRS(TT, DT, PFX, VEC)                                                       \
  GROUP_ENTRY(TT, DT, PFX, VEC, MODE_FWD, 0), GROUP_ENTRY(TT, DT, PFX, VEC, MODE_FWD, 1),      \
  GROUP_ENTRY(TT, DT, PFX, VEC, MODE_BWD, 0), GROUP_ENTRY(TT, DT, PFX, VEC, MODE_BWD, 1)
#define FLAT_ENTRY(TT, DT, PFX, VEC, S, MODE, DESC)                                            \
  {PFX "flat_s" #S "_" #MODE "_" #DESC,                                                        \
   (const void*)&linrec::flat_kernel<TT, VEC, S, linrec::MODE, DESC != 0>, DT, LINREC_FAMILY_FLAT, 4, S, VEC, \
   linrec::MODE, DESC, 0}
#define FLAT_ALL_DIRS(TT, DT, PFX, VEC, S)                                                     \
  FLAT_ENTRY(TT, DT, PFX, VEC, S, MODE_FWD, 0), FLAT_ENTRY(TT, DT, PFX, VEC, S, MODE_FWD, 1),  \
  FLAT_ENTRY(TT, DT, PFX, VEC, S, MODE_BWD, 0), FLAT_ENTRY(TT, DT, PFX, VEC, S, MODE_BWD, 1)
#define COLUMN_ENTRY(TT, DT, PFX, VEC, U, MODE, DESC)                                          \
  {PFX "column_v" #VEC "_u" #U "_" #MODE "_" #DESC,                                            \
   (const void*)&linrec::column_kernel<TT, VEC, U, linrec::MODE, DESC != 0>, DT,               \
   (VEC > 1 ? LINREC_FAMILY_COLUMN : LINREC_FAMILY_NAIVE), 4, U, VEC, linrec::MODE, DESC, 0}
#define COLUMN_ALL_DIRS(TT, DT, PFX, VEC, U)                                                   \
  COLUMN_ENTRY(TT, DT, PFX, VEC, U, MODE_FWD, 0), COLUMN_ENTRY(TT, DT, PFX, VEC, U, MODE_FWD, 1), \
  COLUMN_ENTRY(TT, DT, PFX, VEC, U, MODE_BWD, 0), COLUMN_ENTRY(TT, DT, PFX, VEC, U, MODE_BWD, 1)

// Column block kernels: the 16 waves of a workgroup share rows (the table's `carry` column holds the
// number of lane groups a wave is split into: 1, 2 or 4).
#define COLBLOCK_ENTRY(TT, DT, PFX, VEC, U, G, MODE, DESC)                                     \
  {PFX "colblock_v" #VEC "_u" #U "_g" #G "_" #MODE "_" #DESC,                                  \
   (const void*)&linrec::colblock_kernel<TT, VEC, U, 16, G, linrec::MODE, DESC != 0>, DT,      \
   LINREC_FAMILY_COLUMN, 16, U, VEC, linrec::MODE, DESC, G}
// Column drift kernels: column blocks in teams along the scan axis (`carry` column: lane groups per wave).
#define COLDRIFT_ENTRY(TT, DT, PFX, NW, VEC, U, MODE, DESC)                                    \
  {PFX "coldrift_w" #NW "_v" #VEC "_u" #U "_" #MODE "_" #DESC,                                 \
   (const void*)&linrec::coldrift_kernel<TT, VEC, U, NW, 1, linrec::MODE, DESC != 0>, DT,      \
   LINREC_FAMILY_COLDRIFT, NW, U, VEC, linrec::MODE, DESC, 1}
#define COLDRIFT_FWD_DIRS(TT, DT, PFX, NW, VEC, U)                                             \
  COLDRIFT_ENTRY(TT, DT, PFX, NW, VEC, U, MODE_FWD, 0), COLDRIFT_ENTRY(TT, DT, PFX, NW, VEC, U, MODE_FWD, 1)
#define COLDRIFT_BWD_DIRS(TT, DT, PFX, NW, VEC, U)                                             \
  COLDRIFT_ENTRY(TT, DT, PFX, NW, VEC, U, MODE_BWD, 0), COLDRIFT_ENTRY(TT, DT, PFX, NW, VEC, U, MODE_BWD, 1)
#define COLBLOCK_FWD_DIRS(TT, DT, PFX, VEC, U, G)                                              \
  COLBLOCK_ENTRY(TT, DT, PFX, VEC, U, G, MODE_FWD, 0), COLBLOCK_ENTRY(TT, DT, PFX, VEC, U, G, MODE_FWD, 1)
#define COLBLOCK_BWD_DIRS(TT, DT, PFX, VEC, U, G)                                              \
  COLBLOCK_ENTRY(TT, DT, PFX, VEC, U, G, MODE_BWD, 0), COLBLOCK_ENTRY(TT, DT, PFX, VEC, U, G, MODE_BWD, 1)

// Segmented column launches: the reduce and the apply phase of one geometry (the table's `carry`
// column holds the phase).
#define SEGMENT_ENTRY(TT, DT, PFX, VEC, U, MODE, DESC, PH, PHNAME)                             \
  {PFX "segment_" PHNAME "_v" #VEC "_u" #U "_" #MODE "_" #DESC,                                \
   (const void*)&linrec::column_kernel<TT, VEC, U, linrec::MODE, DESC != 0, linrec::PH>, DT,   \
   LINREC_FAMILY_SEGMENT, 4, U, VEC, linrec::MODE, DESC, linrec::PH}
#define SEGMENT_PHASES(TT, DT, PFX, VEC, U, MODE, DESC)                                        \
  SEGMENT_ENTRY(TT, DT, PFX, VEC, U, MODE, DESC, PHASE_REDUCE, "reduce"),                      \
  SEGMENT_ENTRY(TT, DT, PFX, VEC, U, MODE, DESC, PHASE_APPLY, "apply")
#define SEGMENT_ALL_DIRS(TT, DT, PFX, VEC, U)                                                  \
  SEGMENT_PHASES(TT, DT, PFX, VEC, U, MODE_FWD, 0), SEGMENT_PHASES(TT, DT, PFX, VEC, U, MODE_FWD, 1), \
  SEGMENT_PHASES(TT, DT, PFX, VEC, U, MODE_BWD, 0), SEGMENT_PHASES(TT, DT, PFX, VEC, U, MODE_BWD, 1)

#define F32 float, LINREC_DTYPE_F32, ""
#define F16 _Float16, LINREC_DTYPE_F16, "f16_"
#define BF16 __bf16, LINREC_DTYPE_BF16, "bf16_"
// indirection so that F32 / F16 / BF16 expand into three macro arguments
#define TILE_(...) TILE_ALL_DIRS(__VA_ARGS__)
#define CHAIN_(...) CHAIN_ALL_DIRS(__VA_ARGS__)
#define TEAM_(...) TEAM_ALL_DIRS(__VA_ARGS__)
#define SWEEP_(...) SWEEP_ALL_DIRS(__VA_ARGS__)
#define DRIFT_FWD_(...) DRIFT_FWD_DIRS(__VA_ARGS__)
#define DRIFT_BWD_(...) DRIFT_BWD_DIRS(__VA_ARGS__)
#define DRIFT_RAGGED_FWD_(...) DRIFT_RAGGED_FWD_DIRS(__VA_ARGS__)
#define DRIFT_RAGGED_BWD_(...) DRIFT_RAGGED_BWD_DIRS(__VA_ARGS__)
#define TEAM_FWD_(...) TEAM_FWD_DIRS(__VA_ARGS__)
#define STREAM_(...) STREAM_ALL_DIRS(__VA_ARGS__)
#define COLUMN_(...) COLUMN_ALL_DIRS(__VA_ARGS__)
#define GROUP_(...) GROUP_ALL_DIRS(__VA_ARGS__)
#define FLAT_(...) FLAT_ALL_DIRS(__VA_ARGS__)
#define SEGMENT_(...) SEGMENT_ALL_DIRS(__VA_ARGS__)
#define COLDRIFT_FWD_(...) COLDRIFT_FWD_DIRS(__VA_ARGS__)
#define COLDRIFT_BWD_(...) COLDRIFT_BWD_DIRS(__VA_ARGS__)
#define COLBLOCK_FWD_(...) COLBLOCK_FWD_DIRS(__VA_ARGS__)
#define COLBLOCK_BWD_(...) COLBLOCK_BWD_DIRS(__VA_ARGS__)

// The 16-bit storage types get the geometries the planner picks for them (their register tiles are
// twice as wide as fp32's, so two slots of eight elements per lane is the rule; the forward team
// kernel also comes with four, and the drift kernels, which keep three tiles in the works, with one).
#define HALF_ROW_KERNELS(TY)                                                                    \
  TILE_(TY, 1, 1, 8, 0), TILE_(TY, 2, 1, 8, 0), TILE_(TY, 4, 1, 8, 0), TILE_(TY, 4, 2, 8, 0),   \
  TILE_(TY, 8, 2, 8, 0), TILE_(TY, 16, 2, 8, 0), TILE_(TY, 4, 2, 8, 1), TILE_(TY, 8, 4, 8, 1),  \
  TILE_(TY, 4, 4, 1, 0), TILE_(TY, 4, 4, 1, 1), STREAM_(TY, 8, 2, 8), TEAM_(TY, 8, 2, 8),       \
  TEAM_FWD_(TY, 8, 4, 8), SWEEP_(TY, 8, 2, 8), DRIFT_FWD_(TY, 8, 1, 8),                            \
  DRIFT_FWD_(TY, 16, 1, 8), DRIFT_BWD_(TY, 16, 1, 8), DRIFT_FWD_(TY, 16, 2, 8),                     \
  DRIFT_RAGGED_FWD_(TY, 16, 2, 8), DRIFT_RAGGED_BWD_(TY, 8, 2, 8)
#define HALF_COLUMN_KERNELS(TY)                                                                 \
  GROUP_(TY, 8), FLAT_(TY, 8, 2),                                                               \
  COLUMN_(TY, 8, 4), COLUMN_(TY, 4, 8), COLUMN_(TY, 2, 8), COLUMN_(TY, 2, 16), COLUMN_(TY, 1, 8), COLUMN_(TY, 1, 16), \
  SEGMENT_(TY, 4, 8), SEGMENT_(TY, 2, 8), SEGMENT_(TY, 1, 8),                                   \
  COLBLOCK_FWD_(TY, 2, 8, 1), COLBLOCK_BWD_(TY, 2, 4, 1), COLBLOCK_FWD_(TY, 2, 8, 2), COLBLOCK_BWD_(TY, 2, 4, 2), \
  COLDRIFT_FWD_(TY, 16, 2, 8), COLDRIFT_BWD_(TY, 8, 2, 16), COLDRIFT_FWD_(TY, 8, 2, 16), COLDRIFT_BWD_(TY, 16, 2, 4)

#define LINREC_KERNEL_GROUP(NAME, ...)                                                          \
  namespace linrec {                                                                            \
  namespace {                                                                                   \
  const KernelEntry NAME##_entries[] = {__VA_ARGS__};                                           \
  }                                                                                             \
  KernelGroup NAME() { return {NAME##_entries, int(sizeof(NAME##_entries) / sizeof(NAME##_entries[0]))}; } \
  }
