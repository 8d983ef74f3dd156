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

// One Kogge-Stone step on R independent rows of pairs: every lane with a source composes the
// source's pair in front of its own.  Lanes without a source see the identity.
template <int CTRL, int ROW_MASK, int R>
__device__ __forceinline__ void scan_step(float (&a)[R], float (&b)[R]) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float pa = dpp_move<CTRL, ROW_MASK>(1.0f, a[r]);
    float pb = dpp_move<CTRL, ROW_MASK>(0.0f, b[r]);
    b[r] = fmaf(pb, a[r], b[r]);
    a[r] = pa * a[r];
  }
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
