/*
 * CPU oracle for the RMSNorm operator of the reference (forward kernel and
 * Python backward).
 *
 * TEST INFRASTRUCTURE ONLY: linked into oracle/_build/libsmlm_oracle.so, used by
 * tests/, the smoke check and the benchmark's CPU leg; never by the package.
 *
 * What is pinned and by what (tests/test_oracle_pins.py):
 *   - forward  : numpy float64 closed form x / sqrt(mean(x^2) + eps) * w, the
 *                unit-weight / constant-row special cases (a row of equal values c
 *                normalises to c / sqrt(c^2 + eps)), and scale invariance for
 *                eps = 0.
 *   - backward : torch.autograd of the float64 composite, float64 finite
 *                differences, and the identity <dx, x> = 0 for eps = 0 (the
 *                output does not change when a row is scaled).
 *   - rounding mode of the reference's backward (its Python lines round
 *     intermediates to the 16-bit dtype): restated literally as a second mode and
 *     bounded against the exact mode.
 * Parity unpinned: the last-bit behaviour of the reference's rsqrtf (CUDA
 * intrinsic) and the order of its block reduction.
 *
 * dtype codes as in smlm_oracle.c: 0 = fp32 (no rounding), 1 = fp16, 2 = bf16.
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>

#define ORACLE_API __attribute__((visibility("default")))

void oracle_round(float* a, size_t n, int dtype); /* smlm_oracle.c */

static float rnd(float f, int dtype) {
  oracle_round(&f, 1, dtype);
  return f;
}

/*
 * Forward.  Follows rmsnorm_twoPassAlgo_e8
 * (kernel_src/csrc/rms_norm/rms_norm_cutlass.cu:81-159): the sum of squares of
 * a row in float (here in double when acc64), rms = 1 / sqrt(sum / n + eps)
 * stored as float (:116-119), out = round_dtype(float(x) * rms * float(w))
 * (:141-156: the product is formed left to right in float).
 * x, out: [rows, cols]; w: [cols]; rms_out: [rows].
 */
ORACLE_API int oracle_rms_norm_fwd(float* out, float* rms_out, const float* x, const float* w,
                                   int rows, int cols, float eps, int dtype, int acc64) {
  if (!out || !rms_out || !x || !w || rows < 0 || cols <= 0) return -1;
  for (int t = 0; t < rows; ++t) {
    const float* xr = x + (long)t * cols;
    float rms;
    if (acc64) {
      double s = 0.0;
      for (int j = 0; j < cols; ++j) s += (double)xr[j] * (double)xr[j];
      rms = (float)(1.0 / sqrt(s / cols + (double)eps));
    } else {
      float s = 0.0f;
      for (int j = 0; j < cols; ++j) s += xr[j] * xr[j];
      rms = 1.0f / sqrtf(s / cols + eps);
    }
    rms_out[t] = rms;
    for (int j = 0; j < cols; ++j) out[(long)t * cols + j] = rnd(xr[j] * rms * w[j], dtype);
  }
  return 0;
}

/*
 * Backward.  Follows rms_norm.backward
 * (src/loquetier_src/kernel_utils.py:169-176):
 *   d_weight = (x * rms * g).sum(dim=0)
 *   d_x_hat  = g * w
 *   dot_p    = (d_x_hat * x).sum(dim=1)
 *   dx       = (d_x_hat - (x * dot_p * rms^2) / n) * rms
 * literal != 0 rounds where the reference's tensor expressions round: g * w,
 * d_x_hat * x, its row sum and x * dot_p are 16-bit tensors there (both operands
 * 16-bit), everything that involves the float32 rms is float32; dx and d_weight
 * are rounded to the parameter dtype at the end (autograd casts them).
 * literal == 0 keeps every intermediate in double (the exact gradient of the
 * forward maths) and rounds only the results.
 */
ORACLE_API int oracle_rms_norm_bwd(float* dx, float* dw, const float* g, const float* x,
                                   const float* w, const float* rms, int rows, int cols, int dtype,
                                   int literal) {
  if (!dx || !dw || !g || !x || !w || !rms || rows < 0 || cols <= 0) return -1;
  double* dwacc = (double*)calloc((size_t)cols, sizeof(double));
  if (!dwacc) return -2;
  for (int t = 0; t < rows; ++t) {
    const float* xr = x + (long)t * cols;
    const float* gr = g + (long)t * cols;
    const double r = (double)rms[t];
    if (literal) {
      float dot = 0.0f; /* torch sums 16-bit tensors in float and rounds the result */
      for (int j = 0; j < cols; ++j) dot += rnd(rnd(gr[j] * w[j], dtype) * xr[j], dtype);
      dot = rnd(dot, dtype);
      for (int j = 0; j < cols; ++j) {
        const float dxh = rnd(gr[j] * w[j], dtype);
        const float xd = rnd(xr[j] * dot, dtype);
        const float v = (dxh - (xd * (rms[t] * rms[t])) / (float)cols) * rms[t];
        dx[(long)t * cols + j] = rnd(v, dtype);
        dwacc[j] += (double)((xr[j] * rms[t]) * gr[j]);
      }
    } else {
      double dot = 0.0;
      for (int j = 0; j < cols; ++j) dot += (double)gr[j] * (double)w[j] * (double)xr[j];
      for (int j = 0; j < cols; ++j) {
        const double dxh = (double)gr[j] * (double)w[j];
        dx[(long)t * cols + j] = rnd((float)((dxh - (double)xr[j] * dot * r * r / cols) * r), dtype);
        dwacc[j] += (double)xr[j] * r * (double)gr[j];
      }
    }
  }
  for (int j = 0; j < cols; ++j) dw[j] = rnd((float)dwacc[j], dtype);
  free(dwacc);
  return 0;
}
