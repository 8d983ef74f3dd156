// Wavefront-level building blocks of the linear-recurrence scan for gfx950 (wave64).
//
// The recurrence v_l = v_{l-1} * c_l + x_l is a composition of affine maps v -> a*v + b.
// Composing "first" then "second" gives (a1*a2, b1*a2 + b2); the identity is (1, 0).  The
// reference states the same operator at linrec/impl/cuda/linrec_tile.cuh:52-55 and
// linrec/impl/python/ops.py:68-71; everything else in this file (DPP data movement, 64-lane
// shape) is specific to CDNA.
#pragma once
#include <hip/hip_runtime.h>

namespace linrec {

struct Affine {
  float a;  // product of coefficients
  float b;  // value produced from a zero input
};

__device__ __forceinline__ Affine compose(Affine first, Affine second) {
  return {first.a * second.a, fmaf(first.b, second.a, second.b)};
}

// v_mov_b32_dpp: lane i receives `src` of the lane selected by CTRL; lanes without a source
// (or rows masked out by ROW_MASK) keep `old`.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float old, float src) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, src),
                                         CTRL, ROW_MASK, 0xf, false));
}

constexpr int DPP_ROW_SHL1 = 0x101;  // lane i <- lane i+1 of the same 16-lane row
constexpr int DPP_ROW_SHL2 = 0x102;
constexpr int DPP_ROW_SHL4 = 0x104;
constexpr int DPP_ROW_SHL8 = 0x108;
constexpr int DPP_ROW_SHR1 = 0x111;
constexpr int DPP_ROW_SHR2 = 0x112;
constexpr int DPP_ROW_SHR4 = 0x114;
constexpr int DPP_ROW_SHR8 = 0x118;
constexpr int DPP_ROW_BCAST15 = 0x142;  // lane 15 of each 16-lane row -> the next row
constexpr int DPP_ROW_BCAST31 = 0x143;  // lane 31 -> lanes 32..63
constexpr int DPP_WAVE_SHL1 = 0x130;    // lane i <- lane i+1
constexpr int DPP_WAVE_SHR1 = 0x138;    // lane i <- lane i-1

__device__ __forceinline__ float read_lane(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// One Kogge-Stone step on N (1, 2 or 4) independent rows of pairs, two instructions a row: the multiply-add and the
// multiply read their first operand through DPP themselves (v_fmac_f32_dpp b, b', a: b += b' * a with b' the source
// lane's b; v_mul_f32_dpp a, a', a), and a lane without a source, or in a row masked out, is switched off for the
// instruction and keeps its pair - which is what composing with the identity gives.  The compiler does not fold a
// v_mov_b32_dpp into the arithmetic here (it leaves two moves that set the identity, two DPP moves, the multiply-add
// and the multiply: six instructions a row), hence the assembly.  A DPP operand must not be read within two wait
// states of the vector instruction that wrote it: the leading s_nop covers what the compiler placed in front, inside
// a block no instruction reads through DPP what the block wrote (the multiply-adds write b, the multiplies read a),
// and behind the block the compiler pads for its own DPP reads.
#define LINREC_DPP_FMAC(B, A, MODS) "v_fmac_f32_dpp " B ", " B ", " A " " MODS "\n\t"
#define LINREC_DPP_MUL(A, MODS) "v_mul_f32_dpp " A ", " A ", " A " " MODS "\n\t"
#define LINREC_DPP_STEP_ROWS(MODS)                                                                                  \
  if constexpr (N == 1) {                                                                                           \
    asm("s_nop 1\n\t" LINREC_DPP_FMAC("%0", "%1", MODS) LINREC_DPP_MUL("%1", MODS) : "+v"(b[0]), "+v"(a[0]));      \
  } else if constexpr (N == 2) {                                                                                    \
    asm("s_nop 1\n\t" LINREC_DPP_FMAC("%0", "%2", MODS) LINREC_DPP_FMAC("%1", "%3", MODS)                           \
        LINREC_DPP_MUL("%2", MODS) LINREC_DPP_MUL("%3", MODS)                                                       \
        : "+v"(b[0]), "+v"(b[1]), "+v"(a[0]), "+v"(a[1]));                                                          \
  } else {                                                                                                          \
    asm("s_nop 1\n\t" LINREC_DPP_FMAC("%0", "%4", MODS) LINREC_DPP_FMAC("%1", "%5", MODS)                           \
        LINREC_DPP_FMAC("%2", "%6", MODS) LINREC_DPP_FMAC("%3", "%7", MODS) LINREC_DPP_MUL("%4", MODS)              \
        LINREC_DPP_MUL("%5", MODS) LINREC_DPP_MUL("%6", MODS) LINREC_DPP_MUL("%7", MODS)                            \
        : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]));          \
  }
template <int CTRL, int ROW_MASK, int N>
__device__ __forceinline__ void scan_step_rows(float* a, float* b) {
  static_assert(N == 1 || N == 2 || N == 4, "rows of one block");
  static_assert(ROW_MASK == (CTRL == DPP_ROW_BCAST15 ? 0xa : CTRL == DPP_ROW_BCAST31 ? 0xc : 0xf), "row mask of the step");
  if constexpr (CTRL == DPP_ROW_SHR1) { LINREC_DPP_STEP_ROWS("row_shr:1 row_mask:0xf bank_mask:0xf") }
  else if constexpr (CTRL == DPP_ROW_SHR2) { LINREC_DPP_STEP_ROWS("row_shr:2 row_mask:0xf bank_mask:0xf") }
  else if constexpr (CTRL == DPP_ROW_SHR4) { LINREC_DPP_STEP_ROWS("row_shr:4 row_mask:0xf bank_mask:0xf") }
  else if constexpr (CTRL == DPP_ROW_SHR8) { LINREC_DPP_STEP_ROWS("row_shr:8 row_mask:0xf bank_mask:0xf") }
  else if constexpr (CTRL == DPP_ROW_SHL1) { LINREC_DPP_STEP_ROWS("row_shl:1 row_mask:0xf bank_mask:0xf") }
  else if constexpr (CTRL == DPP_ROW_SHL2) { LINREC_DPP_STEP_ROWS("row_shl:2 row_mask:0xf bank_mask:0xf") }
  else if constexpr (CTRL == DPP_ROW_SHL4) { LINREC_DPP_STEP_ROWS("row_shl:4 row_mask:0xf bank_mask:0xf") }
  else if constexpr (CTRL == DPP_ROW_SHL8) { LINREC_DPP_STEP_ROWS("row_shl:8 row_mask:0xf bank_mask:0xf") }
  else if constexpr (CTRL == DPP_ROW_BCAST15) { LINREC_DPP_STEP_ROWS("row_bcast:15 row_mask:0xa bank_mask:0xf") }
  else { static_assert(CTRL == DPP_ROW_BCAST31, "a step of the scan"); LINREC_DPP_STEP_ROWS("row_bcast:31 row_mask:0xc bank_mask:0xf") }
}
#undef LINREC_DPP_STEP_ROWS
#undef LINREC_DPP_MUL
#undef LINREC_DPP_FMAC

// One Kogge-Stone step on R independent rows of pairs: every lane with a source composes the
// source's pair in front of its own.  Lanes without a source keep theirs.
template <int CTRL, int ROW_MASK, int R>
__device__ __forceinline__ void scan_step(float (&a)[R], float (&b)[R]) {
  constexpr int N = R >= 4 ? 4 : R >= 2 ? 2 : 1;  // rows to a block
  static_assert(R % N == 0, "whole blocks");
#pragma unroll
  for (int r = 0; r < R; r += N) scan_step_rows<CTRL, ROW_MASK, N>(a + r, b + r);
}

// Inclusive scan over the 64 lanes of R independent rows of affine maps (lane 0 first).
// Four shifts inside each 16-lane DPP row, then two row broadcasts: six steps, no LDS.
template <int R>
__device__ __forceinline__ void wave_inclusive_scan(float (&a)[R], float (&b)[R]) {
  scan_step<DPP_ROW_SHR1, 0xf>(a, b);
  scan_step<DPP_ROW_SHR2, 0xf>(a, b);
  scan_step<DPP_ROW_SHR4, 0xf>(a, b);
  scan_step<DPP_ROW_SHR8, 0xf>(a, b);
  scan_step<DPP_ROW_BCAST15, 0xa>(a, b);
  scan_step<DPP_ROW_BCAST31, 0xc>(a, b);
}

// Lane i receives lane i-1's value; lane 0 receives `first`.
__device__ __forceinline__ float shift_up_one_lane(float v, float first) {
  return dpp_move<DPP_WAVE_SHR1, 0xf>(first, v);
}

// Lane i receives lane i+1's value; lane 63 receives `last`.
__device__ __forceinline__ float shift_down_one_lane(float v, float last) {
  return dpp_move<DPP_WAVE_SHL1, 0xf>(last, v);
}

// Lanes 32..63 receive the value of the lane 32 below; lanes 0..31 keep their own.  One vector-ALU
// instruction on gfx950: v_permlane32_swap exchanges the upper half of its first operand with the
// lower half of its second.
__device__ __forceinline__ float lanes_up_32(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  const auto halves = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, unsigned(halves[0]));
}

}  // namespace linrec
