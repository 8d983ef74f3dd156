/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the linear-recurrence path of
 * safelix/linrec, used as the checker for the HIP kernels and as the timed CPU
 * baseline.  Nothing in the shipped package may call into this file.
 *
 * What it restates (paths relative to the reference tree):
 *   forward   linrec/impl/python/ops.py:8-20      (prev = 0; y[i] = prev*c[i] + x[i])
 *             linrec/impl/cuda/linrec_ref.cuh:53-69   (y[first] = x[first], c[first] never read)
 *   backward  linrec/impl/python/ops.py:22-40     (shift, opposite-direction scan, multiply)
 *             linrec/impl/cuda/linrec_ref.cuh:71-94   (dx[last] = dy[last]; dc[first] = 0)
 *
 * The first coefficient in scan order is never read (linrec_ref.cuh:63), so a
 * non-finite value there does not reach the result.
 *
 * Parity pins (tests/test_oracle_pins.py): hand-computed integer known answers,
 * c==0, c==1 (cumsum), constant c (IIR filter), unit impulse (cumprod), linearity,
 * flip equivalence, chunk composition, row independence, and for the backward an
 * O(L^2) explicit-sum formulation differentiated by autograd plus central finite
 * differences.  Every function below is covered by at least one of those.
 *
 * Rows run in parallel (OpenMP); each row is the plain sequential loop.
 *
 * Layout: element (r, l) of a tensor lives at base[r*row_stride + l*elem_stride]
 * (strides in elements), so dense rows, padded rows and transposed views are all
 * addressed the same way.
 */
#include <omp.h>
#include <stddef.h>
#include <stdint.h>

/* Rows are independent (linrec/impl/cuda/linrec_pipe.cuh:14): the loops below run them on
 * several threads.  The timed CPU baseline states how many; everything else leaves OpenMP's default. */
int oracle_max_threads(void) { return omp_get_max_threads(); }
void oracle_set_threads(int n) { if (n > 0) omp_set_num_threads(n); }

#define DEFINE_ORACLE(T, SUFFIX)                                                              \
  /* forward: linrec_ref.cuh:63-68 (explicit first element), ops.py:16-18 */                  \
  void oracle_linrec_fwd_##SUFFIX(const T* x, const T* c, T* y, int64_t numseq,               \
                                  int64_t seqlen, int64_t row_stride, int64_t elem_stride,    \
                                  int reverse) {                                              \
    if (seqlen <= 0) return;                                                                  \
    _Pragma("omp parallel for schedule(static)")                                              \
    for (int64_t r = 0; r < numseq; ++r) {                                                    \
      const T* xr = x + r * row_stride;                                                       \
      const T* cr = c + r * row_stride;                                                       \
      T* yr = y + r * row_stride;                                                             \
      int64_t first = reverse ? seqlen - 1 : 0;                                               \
      int64_t step = reverse ? -1 : 1;                                                        \
      T prev = xr[first * elem_stride];                                                       \
      yr[first * elem_stride] = prev;                                                         \
      for (int64_t n = 1, l = first + step; n < seqlen; ++n, l += step) {                     \
        prev = prev * cr[l * elem_stride] + xr[l * elem_stride];                              \
        yr[l * elem_stride] = prev;                                                           \
      }                                                                                       \
    }                                                                                         \
  }                                                                                           \
  /* backward: linrec_ref.cuh:83-93; ops.py:33-35 (coeffs shifted against the scan,           \
     outputs shifted with it, fill 0 for d_coeffs at the first scan position) */              \
  void oracle_linrec_bwd_##SUFFIX(const T* dy, const T* c, const T* y, T* dx, T* dc,          \
                                  int64_t numseq, int64_t seqlen, int64_t row_stride,         \
                                  int64_t elem_stride, int reverse) {                         \
    if (seqlen <= 0) return;                                                                  \
    _Pragma("omp parallel for schedule(static)")                                              \
    for (int64_t r = 0; r < numseq; ++r) {                                                    \
      const T* dyr = dy + r * row_stride;                                                     \
      const T* cr = c + r * row_stride;                                                       \
      const T* yr = y + r * row_stride;                                                       \
      T* dxr = dx + r * row_stride;                                                           \
      T* dcr = dc + r * row_stride;                                                           \
      /* the gradient scan starts where the forward scan ended */                             \
      int64_t start = reverse ? 0 : seqlen - 1;                                               \
      int64_t step = reverse ? 1 : -1;                                                        \
      T g = dyr[start * elem_stride];                                                         \
      dxr[start * elem_stride] = g;                                                           \
      for (int64_t n = 1, l = start + step; n < seqlen; ++n, l += step) {                     \
        g = g * cr[(l - step) * elem_stride] + dyr[l * elem_stride];                          \
        dxr[l * elem_stride] = g;                                                             \
      }                                                                                       \
      /* d_coeffs[l] = d_inputs[l] * outputs[l -/+ 1]; zero where no predecessor exists */    \
      int64_t fwd_first = reverse ? seqlen - 1 : 0;                                           \
      for (int64_t l = 0; l < seqlen; ++l) {                                                  \
        if (l == fwd_first) {                                                                 \
          dcr[l * elem_stride] = (T)0;                                                        \
        } else {                                                                              \
          dcr[l * elem_stride] = dxr[l * elem_stride] * yr[(l + step) * elem_stride];         \
        }                                                                                     \
      }                                                                                       \
    }                                                                                         \
  }

DEFINE_ORACLE(double, f64)
DEFINE_ORACLE(float, f32)
