/*
 * linrec_hip -- C ABI of the MI355X (gfx950) linear-recurrence scan library.
 *
 *   forward   y[first] = x[first];  y[l] = y[l -/+ 1] * c[l] + x[l]
 *   backward  dx = opposite-direction scan of dy against c shifted by one,
 *             dc[l] = dx[l] * y[l -/+ 1]  (0 at the first forward position)
 *
 * Every entry point is plain C: device pointers, sizes and strides in elements, a HIP stream
 * handle passed as void*.  No torch types cross this boundary.  All calls only enqueue work on
 * `stream` and return; none of them synchronises, allocates or frees device memory.
 *
 * Tensor layout: element (r, l) of every tensor of a call lives at base[r*row_stride +
 * l*elem_stride].  Either elem_stride == 1 (rows along the unit-stride axis; row_stride >= seqlen
 * allows padded rows) or row_stride == 1 (the scan axis is the strided one, e.g. a transposed
 * view); anything else is served by a slow one-lane-per-row kernel.
 *
 * Return value: 0 on success, a negative LINREC_E_* code for a rejected call, or a positive
 * hipError_t from the launch.
 */
#ifndef LINREC_HIP_H_
#define LINREC_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LINREC_OK 0
#define LINREC_E_INVALID (-1)     /* null pointer, negative size, overlapping strides */
#define LINREC_E_WORKSPACE (-2)   /* workspace missing, misaligned or too small for this call */
#define LINREC_E_UNSUPPORTED (-3) /* tuning override names a kernel that is not compiled in */
#define LINREC_E_TOO_LARGE (-4)   /* seqlen beyond 2^31-5 elements */
#define LINREC_E_SCRATCH (-5)     /* linrec_fwd_noalloc: the call needs more scratch than the static array holds */

/* Storage types (arithmetic is always fp32). */
#define LINREC_DTYPE_F32 0
#define LINREC_DTYPE_F16 1  /* IEEE half */
#define LINREC_DTYPE_BF16 2

/* Kernel families. */
#define LINREC_FAMILY_AUTO 0
#define LINREC_FAMILY_TILE 1   /* rows on the unit-stride axis; a tile of waves*slots*256 elements per
                                  workgroup; rows longer than a tile are chained by decoupled look-back */
#define LINREC_FAMILY_COLUMN 2 /* scan axis strided, rows on the unit-stride axis: one lane walks a row, or (block
                                  form, plan.carry = lane groups per wave) the 16 waves of a workgroup share rows and
                                  each walks a run of positions per step */
#define LINREC_FAMILY_NAIVE 3  /* any strides: one lane per row, sequential (debug / odd layouts) */
#define LINREC_FAMILY_STREAM 4 /* rows on the unit-stride axis; one workgroup walks a whole row tile by
                                  tile with the next tile's loads in flight (many long rows) */
#define LINREC_FAMILY_TEAM 5   /* like STREAM, but `tasks` workgroups walk one row side by side, each taking
                                  every tasks-th tile; they exchange per-tile maps through the workspace */
#define LINREC_FAMILY_SWEEP 6  /* teams as in TEAM, each going on to further rows, sized so that the launch
                                  reads the tensors front to back; rows of a whole number of tiles only.
                                  Tuning: `tasks` = team size, `carry` > 0 = number of teams */
#define LINREC_FAMILY_GROUP 7  /* rows of at most 32 slots (128 floats): 1 .. 32 adjacent lanes share a row, a
                                  wave takes 64 / lanes rows at once; rows must start on slot boundaries */
#define LINREC_FAMILY_SEGMENT 8 /* as COLUMN for few rows: the scan axis is cut into segments that run side by
                                  side (reduce, carry, apply: three launches).  Tuning: `waves` = rows per
                                  lane, `slots` = timesteps in flight, `tasks` = segments (at most 4096).
                                  In the plan, `tiles_per_row` = segments, `tasks` = positions per segment */
#define LINREC_FAMILY_FLAT 9    /* dense short rows (row stride == row length <= 240 floats, 16-byte aligned
                                  bases): the tensor as one flat array of full slots, the scan cut at the row
                                  starts by the unused coefficient there.  Tuning: `slots` = rows of 64 slots
                                  a wave takes (4 or 2) */

#define LINREC_FAMILY_DRIFT 10  /* the SWEEP launch shape with the exchange between team mates off the critical
                                  path: a scanned tile is kept (in registers; the 16-bit forward's tiles of two
                                  slots as packed inputs in LDS) and stored two steps late, by which time the
                                  value entering it has arrived without anybody waiting.  Tuning as SWEEP, with
                                  teams of up to 64 a wave: beyond 64 every wave collects maps.  Compiled (waves x slots):
                                  fp32 forward 8 x 4, 8 x 2, 4 x 4, 16 x 1 and 16 x 2 (the last for teams of at most
                                  64 only), fp32 backward 8 x 2 and 16 x 1; 16-bit storage (slots of eight
                                  elements) forward 16 x 2, 16 x 1 and 8 x 1, backward 16 x 1.
                                  The planner's picks are the 16-wave ones, and 8 x 4 forward for fp32 teams beyond 64.
                                  Rows must be whole tiles; rows of whole 16-byte slots may end in a partial tile
                                  (fp32 forward 16 x 2 and 8 x 4, backward 16 x 1; 16-bit storage forward 16 x 2,
                                  backward 8 x 2), and their teams need not divide the tiles of a row */

#define LINREC_FAMILY_COLDRIFT 11 /* as COLUMN in its block form for a few hundred to a few thousand rows: teams
                                   of workgroups share a block of rows and take its steps along the scan axis in
                                   turn; a step's data stays in registers and is stored two steps late, when the
                                   team mates' maps have arrived.  Tuning: `waves` = waves per workgroup (16 or 8),
                                   `slots` = positions per run, `carry` = rows per lane (fp32 one, 16-bit storage
                                   two), `tasks` = team size (at most the waves).  In the plan, `tiles_per_row` =
                                   steps of a row, `tasks` = team size */

/*
 * Per-call tuning override; NULL selects the built-in gfx950 table.
 * Replaces the keyword options of the reference's launchers
 * (linrec/impl/cuda/linrec_pipe.cu:40-48: kMaxElemsPerThread, kMaxThreadsPerBlock, memcode,
 * algocode) and its compile-time config table (linrec/impl/cuda/linrec.h:8-13).
 */
typedef struct linrec_tuning {
  int32_t family; /* LINREC_FAMILY_*; AUTO keeps the table's choice for every field below */
  int32_t waves;  /* TILE, STREAM: wavefronts per workgroup (1, 4, 8 or 16) */
  int32_t slots;  /* TILE, STREAM: 16-byte slots per lane (1, 2, 4 or 8); COLUMN: timesteps in flight per lane */
  int32_t carry;  /* TILE: -1 auto, 0 one tile must hold the row, 1 force the look-back chain.
                     COLUMN: 1 or 2 the block form (the 16 waves of a workgroup share rows, each wave
                     split into that many groups of lanes; `waves` = rows per lane, `slots` = positions per
                     run, 0 for the compiled choice) */
  int32_t tasks;  /* TILE with look-back: tiles (of different rows) one workgroup works through with
                     the next tile's loads in flight; 0 auto, 1 one tile per workgroup.
                     TEAM: workgroups per row (at most 64) */
} linrec_tuning_t;

/* What a call would launch; filled by linrec_plan_f32 (introspection for tests and tuning). */
typedef struct linrec_plan {
  int32_t family;
  int32_t waves;
  int32_t slots;
  int32_t vec;            /* elements per slot: 16 bytes' worth (4 floats, 8 halves) or 1 */
  int32_t carry;          /* 1 if tiles of a row are chained through the workspace; COLUMN: lane groups per wave
                             of the block form (1 or 2), 0 for the plain column kernels */
  int32_t tiles_per_row;  /* COLUMN block form: steps of the walk along the scan axis; SEGMENT: segments */
  int32_t tasks;          /* tiles per workgroup (look-back kernels), else 1 */
  int32_t tail_rows;      /* rows at the end of the tensor that a second launch, planned for them alone, serves
                             (0: one launch serves all rows) */
  int64_t grid;           /* workgroups */
  int32_t block;          /* lanes per workgroup */
  int32_t kernel_id;      /* index for linrec_kernel_name / linrec_kernel_attrs, -1 if none */
  uint64_t workspace_bytes; /* minimum workspace this call needs (0 if none) */
} linrec_plan_t;

/* Library identification; bumps when the ABI changes. */
int linrec_hip_abi_version(void);

/* Text for any code returned by this library (LINREC_E_* or hipError_t). */
const char* linrec_hip_error_string(int code);

/*
 * Forward scan.  Replaces linrec_pipe_fwd (linrec/impl/cuda/linrec_pipe.cu:16-92, declared at
 * linrec/impl/cuda/linrec.h:45-48), and through it linrec_tile_fwd (linrec_tile.cu:17-94) and
 * linrec_ref_fwd (linrec_ref.cu:11-50), which compute the same function.
 * `outputs` must not alias the inputs.  The first coefficient of each row in scan order is never
 * used (linrec_ref.cuh:63).
 * `workspace` may be NULL when linrec_workspace_bytes() is 0 for the call.  A workspace must be
 * 16-byte aligned, zero-filled before its first use, used by one stream at a time, and otherwise
 * left to this library: the kernels keep their launch counter in it and never need it cleared again.
 */
int linrec_fwd_f32(const float* inputs, const float* coeffs, float* outputs, int64_t numseq,
                   int64_t seqlen, int64_t row_stride, int64_t elem_stride, int reverse,
                   void* workspace, size_t workspace_bytes, const linrec_tuning_t* tuning,
                   void* stream);

/*
 * Backward.  Replaces linrec_pipe_bwd (linrec/impl/cuda/linrec_pipe.cu:96-174, linrec.h:50-55) and
 * its tile/ref siblings.  `reverse` is the flag of the forward call whose gradient is taken.
 */
int linrec_bwd_f32(const float* d_outputs, const float* coeffs, const float* outputs,
                   float* d_inputs, float* d_coeffs, int64_t numseq, int64_t seqlen,
                   int64_t row_stride, int64_t elem_stride, int reverse, void* workspace,
                   size_t workspace_bytes, const linrec_tuning_t* tuning, void* stream);

/*
 * The same two entry points for any storage type (LINREC_DTYPE_*): fp16 and bf16 tensors are read
 * and written as such, every intermediate is fp32.  Fills the gap the reference marks with
 * "TODO: dispatch" on the scalar type (linrec/impl/cuda/linrec_pipe.cu:22, linrec_tile.cu:23).
 * Strides and seqlen are in elements of the storage type; pointers must be element-aligned.
 */
int linrec_fwd(int dtype, const void* inputs, const void* coeffs, void* outputs, int64_t numseq,
               int64_t seqlen, int64_t row_stride, int64_t elem_stride, int reverse, void* workspace,
               size_t workspace_bytes, const linrec_tuning_t* tuning, void* stream);
int linrec_bwd(int dtype, const void* d_outputs, const void* coeffs, const void* outputs, void* d_inputs,
               void* d_coeffs, int64_t numseq, int64_t seqlen, int64_t row_stride, int64_t elem_stride,
               int reverse, void* workspace, size_t workspace_bytes, const linrec_tuning_t* tuning,
               void* stream);

/*
 * linrec_fwd / linrec_bwd with the arguments in one block of memory, for bindings whose cost per argument
 * counts (a ctypes call marshals every argument; on a 64 x 4096 tensor, whose kernel takes 3 us, the
 * binding then spends more time than the device).  The caller keeps a linrec_call_t per kind of call and only
 * rewrites the pointers.  Forward: in0 = inputs, out0 = outputs; backward: in0 = d_outputs, aux = outputs,
 * out0 = d_inputs, out1 = d_coeffs.  Same results and error codes as linrec_fwd / linrec_bwd with no tuning.
 * The counterpart of the reference's one pybind call per pass (linrec/impl/cuda/extension.cpp:61-67).
 */
typedef struct linrec_call {
  int32_t dtype;    /* LINREC_DTYPE_* */
  int32_t reverse;
  int64_t numseq, seqlen, row_stride, elem_stride;
  const void* in0;
  const void* coef;
  const void* aux;
  void* out0;
  void* out1;
  void* workspace;
  uint64_t workspace_bytes;
  void* stream;
} linrec_call_t;
int linrec_fwd_call(const linrec_call_t* call);
int linrec_bwd_call(const linrec_call_t* call);

/*
 * linrec_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the same call without the workspace arguments.
 * It has no counterpart in the reference, whose launcher allocates its result itself
 * (linrec/impl/cuda/linrec_pipe.cu:31).  Where the chosen kernel needs a workspace, the library's own
 * static device array of LINREC_NOALLOC_SCRATCH_BYTES serves as one; each GPU holds its copy of that
 * array from the first call on it until the process ends.  The call makes no hipMalloc / hipFree and
 * calls no allocating routine.  A problem that needs more than the array holds (about 130 000 tiles of
 * rows split over workgroups) returns LINREC_E_SCRATCH with nothing enqueued; results are identical to
 * linrec_fwd's.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU
 * (two streams, two threads) race on it and must be serialised by the caller, and the array must not
 * be mixed with linrec_fwd's caller-owned workspaces in any other way than by calling this function.
 * Where the table's kernel would need more than the array holds and no tuning is given, the call falls back
 * to a kernel that needs less: one workgroup per row (rows on the unit-stride axis, at least a quarter as many as
 * the device has compute units), or on a strided scan axis as many segments as fit, else one lane per row.
 * LINREC_E_SCRATCH is what remains for a few very long rows, or when the caller's own tuning asks for more.
 * The array keeps the previous call's contents; nothing in it needs clearing between calls (its launch
 * counter tells old descriptors from new ones, and the completion counters end every launch at zero).
 * The first call on a device looks up the array's address there (hipGetSymbolAddress); make that call
 * outside graph capture.
 */
#define LINREC_NOALLOC_SCRATCH_BYTES (4u << 20)
int linrec_fwd_noalloc(int dtype, const void* inputs, const void* coeffs, void* outputs, int64_t numseq,
                       int64_t seqlen, int64_t row_stride, int64_t elem_stride, int reverse,
                       const linrec_tuning_t* tuning, void* stream);
/* The launch linrec_fwd_noalloc would make (its fallbacks included); LINREC_E_SCRATCH where it would turn the call down. */
int linrec_plan_noalloc(int dtype, const void* any_input, int64_t numseq, int64_t seqlen, int64_t row_stride,
                        int64_t elem_stride, int reverse, const linrec_tuning_t* tuning, linrec_plan_t* plan);
/*
 * Waits for another workgroup that hit the poll limit in linrec_fwd_noalloc launches on the current device so far
 * (the second word of the static array's header; the results are right whatever the count).  Copies four words
 * from the device, so it synchronises with it; -1 before the first linrec_fwd_noalloc call on the device.
 * No counterpart in the reference.
 */
int linrec_noalloc_gave_up_count(void);

/*
 * Batches of matrices whose scan axis is the strided one, e.g. (batch, time, channels) tensors
 * scanned over time: `batches` matrices `batch_stride` elements apart, each of `rows_per_batch` rows
 * `row_stride` apart (1 for channels-last data), elements of a row `elem_stride` apart.  The rows of
 * such a tensor are not uniformly strided, so the entry points above cannot describe it.  Served by
 * the COLUMN, NAIVE and SEGMENT families; LINREC_E_UNSUPPORTED for a unit elem_stride (describe
 * those as rows: every dense batch is one matrix of batches * rows_per_batch rows).  No counterpart
 * in the reference, which takes (..., seqlen) tensors with a unit last stride only
 * (linrec/impl/cuda/linrec_pipe.cu:35) and leaves the transposes to its callers.
 */
int linrec_fwd_batched(int dtype, const void* inputs, const void* coeffs, void* outputs, int64_t batches,
                       int64_t rows_per_batch, int64_t seqlen, int64_t batch_stride, int64_t row_stride,
                       int64_t elem_stride, int reverse, void* workspace, size_t workspace_bytes,
                       const linrec_tuning_t* tuning, void* stream);
int linrec_bwd_batched(int dtype, const void* d_outputs, const void* coeffs, const void* outputs, void* d_inputs,
                       void* d_coeffs, int64_t batches, int64_t rows_per_batch, int64_t seqlen, int64_t batch_stride,
                       int64_t row_stride, int64_t elem_stride, int reverse, void* workspace, size_t workspace_bytes,
                       const linrec_tuning_t* tuning, void* stream);
/* The launch such a call would make; plan->workspace_bytes is the workspace it needs. */
int linrec_plan_batched(int dtype, const void* any_input, int64_t batches, int64_t rows_per_batch, int64_t seqlen,
                        int64_t batch_stride, int64_t row_stride, int64_t elem_stride, int reverse, int is_bwd,
                        const linrec_tuning_t* tuning, linrec_plan_t* plan);

int linrec_plan(int dtype, const void* any_input, int64_t numseq, int64_t seqlen, int64_t row_stride,
                int64_t elem_stride, int reverse, int is_bwd, const linrec_tuning_t* tuning,
                linrec_plan_t* plan);
size_t linrec_workspace_bytes_dtype(int dtype, int64_t numseq, int64_t seqlen, int64_t row_stride,
                                    int64_t elem_stride, int align_elems, int is_bwd,
                                    const linrec_tuning_t* tuning);

/*
 * Minimum workspace for a call with these arguments (0 when the chosen kernel needs none).
 * `align_elems` is the common misalignment of the tensors' base pointers in elements
 * ((address / element size) % (16 / element size); pass 0 for 16-byte aligned bases, a negative
 * value when the tensors of the call do not share one).  No counterpart in the reference, whose
 * rows are never split across blocks (linrec_pipe.cuh:14-22).
 */
size_t linrec_workspace_bytes(int64_t numseq, int64_t seqlen, int64_t row_stride,
                              int64_t elem_stride, int align_elems, int is_bwd,
                              const linrec_tuning_t* tuning);

/*
 * The first 16 bytes of a workspace are four uint32: the launch sequence number, the count of
 * waits for another workgroup that ran out, and two reserved words.  The second word is the only
 * one a caller may read (after synchronising).  A wave whose wait runs out computes what it was
 * waiting for from the row's own data, so the results of every launch are valid whatever the
 * count; non-zero only says that launches were slow because other work held part of the device.
 * The library never resets it.  Always pass the same
 * workspace_bytes for the same workspace: the split into counters and descriptors depends on it.
 * All of that lives in the lower half of the buffer; the upper half is scratch with no life beyond
 * one call (the per-segment maps of LINREC_FAMILY_SEGMENT), kept apart because a descriptor's
 * validity is a bit pattern that scratch values must never imitate.
 *
 * linrec_set_spin_limit: polls a wave spends on one wait for other workgroups' descriptors
 * before it stops waiting (process-wide; returns the previous value; polls <= 0 only queries;
 * a limit of 1 makes every such wait run out, which tests use).  No counterpart in the
 * reference.
 */
int linrec_set_spin_limit(int polls);

/*
 * The launch planner sizes grids by the number of compute units of the current device, asked once per
 * device (hipDeviceAttributeMultiprocessorCount; the reference asks on every launch,
 * linrec/impl/cuda/cuhelpers.cuh:23-34, linrec_pipe.cu:72-80), and by how many workgroups of the chosen
 * kernel a CU holds.  Without a device (a plan asked for on a host without a GPU) it assumes the full
 * part's 256.  linrec_compute_units returns the number in use.  linrec_set_compute_units overrides it
 * for the process (tests, planning for another part); 0 returns to asking the device; the previous
 * override is returned, and a negative argument only queries it.  A caller that keeps plans or workspace
 * sizes from one call to the next has to drop them when it changes the override.
 */
int linrec_compute_units(void);
int linrec_set_compute_units(int cus);

/* Size that serves every call with at most `max_tiles` tiles in one launch. */
size_t linrec_workspace_bytes_for_tiles(int64_t max_tiles);

/*
 * The launch a call would make, without making it.  Pointers are only inspected for alignment.
 * Replaces nothing callable in the reference; it exposes what dispatch<CONFIG_LIST>
 * (linrec/impl/cuda/dispatch.h:53-72) decides internally.
 */
int linrec_plan_f32(const void* any_input, int64_t numseq, int64_t seqlen, int64_t row_stride,
                    int64_t elem_stride, int reverse, int is_bwd, const linrec_tuning_t* tuning,
                    linrec_plan_t* plan);

/*
 * Kernel table introspection.  Replaces linrec_pipe_attrs / linrec_tile_attrs
 * (linrec/impl/cuda/linrec_pipe.cu:177-212, cuhelpers.cuh:36-55) and config_list / config_names
 * (linrec/impl/cuda/extension.cpp:38-39).  linrec_kernel_attrs needs a GPU; it reports
 * hipFuncGetAttributes' numRegs, sharedSizeBytes (LDS), localSizeBytes (scratch) and
 * maxThreadsPerBlock.
 */
/*
 * The planner's crossover thresholds between the long-row kernels, as compiled in from the generated
 * table csrc/plan_thresholds.inc (written by `python -m linrec_amd.tune --write-table` from timings on the
 * device).  The role of the dispatch table the reference's grid search writes (eval/tune.py:104-134);
 * reading them back lets a harness or a test check what the planner decides by.
 * name: NULL beyond the last index; value: -1 beyond the last index.
 */
int linrec_plan_threshold_count(void);
const char* linrec_plan_threshold_name(int index);
int64_t linrec_plan_threshold_value(int index);

int linrec_kernel_count(void);
const char* linrec_kernel_name(int kernel_id);
int linrec_kernel_attrs(int kernel_id, int* num_regs, int* lds_bytes, int* scratch_bytes,
                        int* max_threads);

/*
 * Plain streaming copy of n floats with the same 16-byte access pattern as the scan kernels:
 * the measured bandwidth ceiling the benchmark reports next to the scan (the reference's
 * "algocode 0" variants play this role, linrec/impl/cuda/linrec_pipe.cuh:48).
 */
int linrec_copy_f32(const float* src, float* dst, int64_t n, void* stream);

/*
 * The same for any mix of streams: `reads` (0..3) input streams of n floats are summed and the
 * sum is stored to `writes` (0..2) output streams (with writes == 0 nothing is stored).  The
 * forward scan moves two streams in and one out, the backward three in and two out: this kernel
 * with the same mix is the memory system's rate for that traffic with no scan attached.  n must be
 * a multiple of 4; pointers beyond the requested counts may be NULL.  Same role as above
 * (linrec/impl/cuda/linrec_pipe.cuh:48).
 */
int linrec_stream_mix_f32(int reads, int writes, const float* src0, const float* src1, const float* src2,
                          float* dst0, float* dst1, int64_t n, void* stream);

/*
 * The same traffic with the launch taking its 16 KiB blocks (4096 floats of every stream per workgroup) in
 * another order than ascending addresses: bits [hold_lo, hold_lo + hold_bits) of the block index (address
 * bits 14 + hold_lo and up) become the slowest-changing ones, so the blocks in flight at any moment all
 * agree in them, as the reading positions of a launch do that keeps one workgroup per row of 2^k bytes.
 * A probe of how the memory system spreads addresses: it is what tells a launch shape with gaps between
 * its reading positions from a dense one.  hold_bits == 0 is linrec_stream_mix_f32; otherwise n must be
 * a power of two of whole blocks and the held bits must lie inside the block index.  No counterpart in the
 * reference.
 */
int linrec_stream_mix_order_f32(int reads, int writes, const float* src0, const float* src1, const float* src2,
                                float* dst0, float* dst1, int64_t n, int hold_lo, int hold_bits, void* stream);

/*
 * Memory-only model of a drift launch: the same grid of persistent workgroups (one per compute unit) in teams
 * of `team`, the same tiles of waves x slots x 256 floats in the same order, loads `ahead` tiles ahead and
 * stores `late` steps late with one workgroup barrier per step - and neither a scan nor an exchange between
 * workgroups.  Every tile's `reads` input streams are added up and stored to each of the `writes` outputs.
 * What it takes is what the memory system gives that launch shape; a measuring instrument next to
 * linrec_stream_mix_f32 (the same bytes by thousands of small workgroups in address order).
 * Compiled: reads/writes 2/1 with waves x slots 16 x 2, 8 x 4, 16 x 1 and 3/2 with 16 x 1, 8 x 2; `ahead` 1 or 2,
 * `late` 0 or 2 (LINREC_E_UNSUPPORTED otherwise).  `seqlen` a whole number of tiles, their number a multiple of `team`.
 * stamps: NULL, or a device buffer of 2 x (workgroups) 64-bit words that receives every workgroup's wall clock
 * (100 MHz) at its start and at its end; workgroups = min(numseq, compute units / team) x team.
 * No counterpart in the reference.
 */
int linrec_launch_model_f32(int reads, int writes, const float* src0, const float* src1, const float* src2,
                            float* dst0, float* dst1, int64_t numseq, int64_t seqlen, int waves, int slots,
                            int team, int ahead, int late, unsigned long long* stamps, void* stream);

/*
 * Batched matrix transpose on the device: src holds `batch` dense row-major matrices of rows x cols
 * elements of `elem_size` bytes (2 or 4), dst receives the cols x rows transposes, also dense.
 * The binding uses it to bring tensors whose scan axis is the strided one (time-major data) into
 * the rows-on-the-unit-stride-axis layout the fast kernels want, and results back; the reference
 * leaves that re-layout to the caller (`.contiguous()`, linrec/impl/cuda/ops.py:96, and the
 * stride check at linrec_pipe.cu:35).
 */
int linrec_transpose(int elem_size, const void* src, void* dst, int64_t batch, int64_t rows, int64_t cols,
                     void* stream);

/*
 * Host (CPU) path for tensors in host memory, fp32 or fp64, same layout rules; synchronous.
 * Replaces the eager loop the reference binds as linrec.linrec when no GPU is present
 * (linrec/__init__.py:9-11 -> linrec/impl/python/ops.py:8-20 forward, :22-40 backward).
 * Never used for device memory.
 */
int linrec_host_fwd_f32(const float* inputs, const float* coeffs, float* outputs, int64_t numseq,
                        int64_t seqlen, int64_t row_stride, int64_t elem_stride, int reverse);
int linrec_host_fwd_f64(const double* inputs, const double* coeffs, double* outputs, int64_t numseq,
                        int64_t seqlen, int64_t row_stride, int64_t elem_stride, int reverse);
int linrec_host_bwd_f32(const float* d_outputs, const float* coeffs, const float* outputs,
                        float* d_inputs, float* d_coeffs, int64_t numseq, int64_t seqlen,
                        int64_t row_stride, int64_t elem_stride, int reverse);
int linrec_host_bwd_f64(const double* d_outputs, const double* coeffs, const double* outputs,
                        double* d_inputs, double* d_coeffs, int64_t numseq, int64_t seqlen,
                        int64_t row_stride, int64_t elem_stride, int reverse);

#ifdef __cplusplus
}
#endif
#endif /* LINREC_HIP_H_ */
