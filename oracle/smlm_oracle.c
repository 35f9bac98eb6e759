/*
 * CPU oracle for Segmented Multi-LoRA Multiplication (SMLM).
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain scalar C, the
 * per-segment arithmetic of the reference operator so that the HIP kernels
 * can be checked against it.  Nothing in the shipped package links, loads or
 * calls it; only the test-suite, the smoke check and the benchmark's CPU
 * baseline leg do.
 *
 * What is pinned and by what (checked in tests/test_oracle_*.py):
 *   - segment routing            : closed form (row t belongs to the unique i
 *                                  with s[i] <= t < s[i+1]) and brute force
 *                                  pure-Python loops on tiny inputs; exact
 *                                  small-integer inputs make it bit-exact.
 *   - per-segment shrink/expand  : numpy float64 matmul per segment (a single
 *                                  segment reduces to one library GEMM).
 *   - 16-bit rounding helpers    : numpy / torch casts over every fp16 and
 *                                  bf16 bit pattern class (ties, subnormals,
 *                                  overflow).
 *   - backward (both layouts)    : torch.autograd of the float64 composite
 *                                  x@A.T@B.T, finite differences, and the
 *                                  homogeneity identity <dY,Y>=<dX,x>=<dA,A>
 *                                  =<dB,B>.
 *   - segment builder, partition : brute-force Python run-length encoding.
 *   - rank padding               : zero-padded rank equals true rank exactly.
 * Parity unpinned (nothing in this image can pin it): bit-for-bit agreement
 * with the accumulation order of the reference's CUTLASS grouped GEMM (the
 * CUTLASS submodule directory is empty and no NVIDIA toolchain exists), and
 * the dropout mask drawn upstream of the operator.
 *
 * Conventions: every matrix is passed as float; values are expected to be
 * representable in the I/O dtype (use oracle_round first).  dtype codes:
 * 0 = fp32 (no rounding), 1 = fp16, 2 = bf16.  acc64 != 0 accumulates dot
 * products in double (the "exact" host reference), else in float in index
 * order.  All functions return 0 on success, negative on bad arguments.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ---- 16-bit rounding (round to nearest even), value kept as float ------- */

static float round_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7f800000u) == 0x7f800000u) { /* inf / nan */
    if (u & 0x007fffffu) u |= 0x00400000u; /* quiet the nan, keep it a nan */
    u &= 0xffff0000u;
  } else {
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    u &= 0xffff0000u;
  }
  memcpy(&f, &u, 4);
  return f;
}

static float round_fp16(float f) {
  /* fp16: 1 sign, 5 exponent (bias 15), 10 mantissa. */
  if (isnan(f)) return f;
  double a = fabs((double)f);
  if (a == 0.0 || isinf(f)) return f;
  int e;
  (void)frexp(a, &e); /* a = m * 2^e, m in [0.5,1) -> exponent of a is e-1 */
  int ex = e - 1;
  if (ex < -14) ex = -14;            /* subnormal range shares one quantum */
  double q = ldexp(1.0, ex - 10);    /* spacing of fp16 numbers near a */
  double r = nearbyint(a / q) * q;   /* default rounding mode: nearest even */
  if (r > 65504.0) r = INFINITY;     /* 65520 and above round to infinity */
  return (float)(f < 0 ? -r : r);
}

static float round_dtype(float f, int dtype) {
  if (dtype == 1) return round_fp16(f);
  if (dtype == 2) return round_bf16(f);
  return f;
}

ORACLE_API void oracle_round(float* a, size_t n, int dtype) {
  for (size_t i = 0; i < n; ++i) a[i] = round_dtype(a[i], dtype);
}

/* ---- one dense product C[m,n] = sum_k A(m,k) * B(k,n) -------------------
 * element (i,k) of A is a[i*a_rs + k*a_cs]; (k,j) of B is b[k*b_rs + j*b_cs].
 * Result rounded to dtype and stored to c[i*ldc + j].                      */
static void dense(float* c, int ldc, const float* a, long a_rs, long a_cs,
                  const float* b, long b_rs, long b_cs, int m, int n, int k,
                  int dtype, int acc64) {
  /* output elements are independent: large products are shared out over the host cores; each
   * element is still one dot product in index order, so the result does not depend on it */
#pragma omp parallel for collapse(2) schedule(static) if ((double)m * n * k > 4e6)
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      float r;
      if (acc64) {
        double acc = 0.0;
        for (int p = 0; p < k; ++p)
          acc += (double)a[i * a_rs + p * a_cs] * (double)b[p * b_rs + j * b_cs];
        r = (float)acc;
      } else {
        float acc = 0.0f;
        for (int p = 0; p < k; ++p) acc += a[i * a_rs + p * a_cs] * b[p * b_rs + j * b_cs];
        r = acc;
      }
      c[(long)i * ldc + j] = round_dtype(r, dtype);
    }
}

/* ---- grouped GEMM -------------------------------------------------------
 * Follows kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:31-46
 * (problem i: m = s[i+1]-s[i], n = d_out, k = d_in, X_i = x + s[i]*k,
 * W_i = w[i], Y_i = y + s[i]*n, ld_w = w_ld) and the epilogue alpha = 1,
 * beta = 0 at :107 and :152, i.e. Y_i is OVERWRITTEN by X_i * W_i.
 * W_i is a d_in x d_out matrix; row_major: element (k,n) at w[k*w_ld + n]
 * (w_ld = d_out), otherwise column-major: w[n*w_ld + k] (w_ld = d_in), as
 * chosen at kernel_src/csrc/loquetier_ops.cc:297-303.  Rows outside every
 * segment are not touched.                                                 */
ORACLE_API int oracle_smlm_gemm(float* y, const float* x, const float* const* w,
                                const int32_t* s, int S, int d_in, int d_out,
                                int w_ld, int row_major, int dtype, int acc64) {
  if (!y || !x || !w || !s || S < 0 || d_in <= 0 || d_out <= 0) return -1;
  for (int i = 0; i < S; ++i) {
    int m = s[i + 1] - s[i];
    if (m < 0) return -1;
    if (m == 0) continue;
    const float* xi = x + (long)s[i] * d_in;
    float* yi = y + (long)s[i] * d_out;
    if (row_major)
      dense(yi, d_out, xi, d_in, 1, w[i], w_ld, 1, m, d_out, d_in, dtype, acc64);
    else
      dense(yi, d_out, xi, d_in, 1, w[i], 1, w_ld, m, d_out, d_in, dtype, acc64);
  }
  return 0;
}

/* ---- add_lora.forward ----------------------------------------------------
 * Follows src/loquetier_src/kernel_utils.py:102-120: v = empty(T, r) in the
 * I/O dtype, shrink call, expand call, both with is_row_major = False, so
 * A_i is [r, h_in] and B_i is [h_out, r].  v is rounded to the I/O dtype
 * between the two products.  y rows outside every segment are left as the
 * caller initialised them (the reference leaves torch.empty garbage).      */
ORACLE_API int oracle_add_lora_forward(float* y, float* v, const float* x,
                                       const float* const* wa, const float* const* wb,
                                       const int32_t* s, int S, int h_in, int h_out,
                                       int r, int dtype, int acc64) {
  int rc = oracle_smlm_gemm(v, x, wa, s, S, h_in, r, h_in, 0, dtype, acc64);
  if (rc) return rc;
  return oracle_smlm_gemm(y, v, wb, s, S, r, h_out, r, 0, dtype, acc64);
}

/* ---- MixedLoraLinear.forward tail ----------------------------------------
 * Follows src/loquetier_src/models/mixed_lora.py:198-217.  `y` holds the
 * base-layer output on entry.  lora = add_lora(...) in the I/O dtype; when
 * seg_scale is given (the not-pre-scaled branch, :206-216) each row of lora
 * is multiplied by its segment's scale held in the I/O dtype and rounded;
 * then result = base + lora, rounded.  Rows outside every segment keep the
 * base value (their lora term is treated as zero).                         */
ORACLE_API int oracle_mixed_lora_linear(float* y, const float* x,
                                        const float* const* wa, const float* const* wb,
                                        const int32_t* s, int S, const float* seg_scale,
                                        int h_in, int h_out, int r, int dtype, int acc64) {
  if (S <= 0) return S < 0 ? -1 : 0;
  int T = s[S];
  float* v = (float*)calloc((size_t)T * r + 1, sizeof(float));
  float* l = (float*)calloc((size_t)T * h_out + 1, sizeof(float));
  if (!v || !l) { free(v); free(l); return -2; }
  int rc = oracle_add_lora_forward(l, v, x, wa, wb, s, S, h_in, h_out, r, dtype, acc64);
  if (!rc) {
    for (int i = 0; i < S; ++i) {
      float sc = seg_scale ? round_dtype(seg_scale[i], dtype) : 1.0f;
      for (long t = s[i]; t < s[i + 1]; ++t)
        for (int j = 0; j < h_out; ++j) {
          float lv = l[t * h_out + j];
          if (seg_scale) lv = round_dtype(lv * sc, dtype);
          y[t * h_out + j] = round_dtype(y[t * h_out + j] + lv, dtype);
        }
    }
  }
  free(v); free(l);
  return rc;
}

/* ---- fused semantics the HIP library implements ---------------------------
 * y <- beta*y + scale_seg * (round(x A^T) B^T), one rounding at the end.
 * This is the build's fused epilogue (in-place accumulate into the base
 * output); it differs from oracle_mixed_lora_linear only by skipping the
 * intermediate roundings of mixed_lora.py:214-217.                         */
ORACLE_API int oracle_lora_fused(float* y, float* v, const float* x,
                                 const float* const* wa, const float* const* wb,
                                 const int32_t* s, int S, const float* seg_scale, float beta,
                                 int h_in, int h_out, int r, int dtype, int acc64) {
  int rc = oracle_smlm_gemm(v, x, wa, s, S, h_in, r, h_in, 0, dtype, acc64);
  if (rc) return rc;
  for (int i = 0; i < S; ++i) {
    float sc = seg_scale ? seg_scale[i] : 1.0f;
    for (long t = s[i]; t < s[i + 1]; ++t)
      for (int j = 0; j < h_out; ++j) {
        double acc = 0.0;
        float accf = 0.0f;
        for (int p = 0; p < r; ++p) {
          if (acc64) acc += (double)v[t * r + p] * (double)wb[i][(long)j * r + p];
          else accf += v[t * r + p] * wb[i][(long)j * r + p];
        }
        float a = acc64 ? (float)acc : accf;
        float prev = beta != 0.0f ? beta * y[t * h_out + j] : 0.0f;
        y[t * h_out + j] = round_dtype(prev + sc * a, dtype);
      }
  }
  return 0;
}

/* ---- add_lora.backward, literal (row-major weights) -----------------------
 * Follows src/loquetier_src/kernel_utils.py:128-147 line by line; those
 * lines are shape-valid only for wa [h_in, r], wb [r, h_out]:
 *   mid    = g[start:end] @ wb.T              -> [n, r]      (:141)
 *   grad_x[start:end] = mid @ wa.T            -> [n, h_in]   (:142)
 *   grad_wa = x[start:end].T @ mid            -> [h_in, r]   (:143)
 *   grad_wb = (wa.T @ x[start:end].T) @ g     -> [r, h_out]  (:144)
 * each torch matmul returning the I/O dtype.  grad_x is [T, h_in], zero
 * outside the train partitions (:136).  tp has P+1 entries.               */
ORACLE_API int oracle_add_lora_backward_rowmajor(float* grad_x, float* const* grad_wa,
                                                 float* const* grad_wb, const float* g,
                                                 const float* x, const float* const* wa,
                                                 const float* const* wb, const int32_t* tp,
                                                 int P, int T, int h_in, int h_out, int r,
                                                 int dtype, int acc64) {
  if (P < 0 || T < 0) return -1;
  memset(grad_x, 0, (size_t)T * h_in * sizeof(float));
  for (int p = 0; p < P; ++p) {
    int st = tp[p], n = tp[p + 1] - tp[p];
    if (n < 0 || tp[p + 1] > T) return -1;
    float* mid = (float*)calloc((size_t)n * r + 1, sizeof(float));
    float* xa = (float*)calloc((size_t)n * r + 1, sizeof(float));
    if (!mid || !xa) { free(mid); free(xa); return -2; }
    const float* gp = g + (long)st * h_out;
    const float* xp = x + (long)st * h_in;
    /* mid[i,j] = sum_k g[i,k] * wb[j,k] */
    dense(mid, r, gp, h_out, 1, wb[p], 1, h_out, n, r, h_out, dtype, acc64);
    /* grad_x[i,c] = sum_j mid[i,j] * wa[c,j] */
    dense(grad_x + (long)st * h_in, h_in, mid, r, 1, wa[p], 1, r, n, h_in, r, dtype, acc64);
    /* grad_wa[c,j] = sum_i x[i,c] * mid[i,j] */
    dense(grad_wa[p], r, xp, 1, h_in, mid, r, 1, h_in, r, n, dtype, acc64);
    /* xa^T[j,i] = sum_c wa[c,j] * x[i,c]; kept as xa[i,j] */
    dense(xa, r, xp, h_in, 1, wa[p], r, 1, n, r, h_in, dtype, acc64);
    /* grad_wb[j,c] = sum_i xa[i,j] * g[i,c] */
    dense(grad_wb[p], h_out, xa, 1, r, gp, h_out, 1, r, h_out, n, dtype, acc64);
    free(mid); free(xa);
  }
  return 0;
}

/* ---- add_lora.backward for the layout the forward really uses -------------
 * A_i [r, h_in], B_i [h_out, r] (is_row_major = False at
 * src/loquetier_src/kernel_utils.py:118-119).  Same structure as :128-147,
 * with the products written for this layout:
 *   dV = g B      [n, r]       dX = dV A     [n, h_in]
 *   dA = dV^T x   [r, h_in]    dB = g^T v    [h_out, r],  v = round(x A^T)
 * Partition p uses adapter part_adapter[p]; gradients of partitions that
 * share an adapter are summed in partition order (autograd sums the
 * per-occurrence gradients, src/loquetier_src/models/mixed_lora.py:201-204).
 * grad_a[a] / grad_b[a] are written for every a in [0, NA): zero when the
 * adapter has no rows.  The 16-bit rounding is applied once, to the sum.  */
ORACLE_API int oracle_add_lora_backward(float* grad_x, float* const* grad_a,
                                        float* const* grad_b, const float* g, const float* x,
                                        const float* const* a_w, const float* const* b_w,
                                        const int32_t* tp, const int32_t* part_adapter, int P,
                                        int NA, int T, int h_in, int h_out, int r, int dtype,
                                        int acc64) {
  if (P < 0 || T < 0 || NA < 0) return -1;
  memset(grad_x, 0, (size_t)T * h_in * sizeof(float));
  double* da = (double*)malloc(((size_t)r * h_in + 1) * sizeof(double));
  double* db = (double*)malloc(((size_t)r * h_out + 1) * sizeof(double));
  if (!da || !db) { free(da); free(db); return -2; }
  int rc = 0;
  for (int a = 0; a < NA && !rc; ++a) {
    memset(da, 0, (size_t)r * h_in * sizeof(double));
    memset(db, 0, (size_t)r * h_out * sizeof(double));
    for (int p = 0; p < P; ++p) {
      if (part_adapter[p] != a) continue;
      int st = tp[p], n = tp[p + 1] - tp[p];
      if (n < 0 || tp[p + 1] > T) { rc = -1; break; }
      float* dv = (float*)calloc((size_t)n * r + 1, sizeof(float));
      float* v = (float*)calloc((size_t)n * r + 1, sizeof(float));
      if (!dv || !v) { free(dv); free(v); rc = -2; break; }
      const float* gp = g + (long)st * h_out;
      const float* xp = x + (long)st * h_in;
      /* dV[i,j] = sum_c g[i,c] * B[c,j] */
      dense(dv, r, gp, h_out, 1, b_w[a], r, 1, n, r, h_out, dtype, acc64);
      /* v[i,j] = sum_c x[i,c] * A[j,c] */
      dense(v, r, xp, h_in, 1, a_w[a], 1, h_in, n, r, h_in, dtype, acc64);
      /* dX[i,c] = sum_j dV[i,j] * A[j,c] */
      dense(grad_x + (long)st * h_in, h_in, dv, r, 1, a_w[a], h_in, 1, n, h_in, r, dtype, acc64);
      for (int j = 0; j < r; ++j)
        for (int i = 0; i < n; ++i) {
          double d = dv[(long)i * r + j];
          double vv = v[(long)i * r + j];
          for (int c = 0; c < h_in; ++c) da[(long)j * h_in + c] += d * xp[(long)i * h_in + c];
          for (int c = 0; c < h_out; ++c) db[(long)c * r + j] += vv * gp[(long)i * h_out + c];
        }
      free(dv); free(v);
    }
    if (!rc) {
      for (long i = 0; i < (long)r * h_in; ++i) grad_a[a][i] = round_dtype((float)da[i], dtype);
      for (long i = 0; i < (long)r * h_out; ++i) grad_b[a][i] = round_dtype((float)db[i], dtype);
    }
  }
  free(da); free(db);
  return rc;
}

/* ---- segment builder -------------------------------------------------------
 * Follows src/loquetier_src/model_generation.py:267-281: run-length merge of
 * consecutive requests with equal lora_id; segment = cumsum([0] + lens).
 * Returns the number of segments written (<= n), or negative on error.
 * Outputs need room for n (ids, lens) and n+1 (segment) entries.          */
ORACLE_API int oracle_build_segments(const int32_t* req_lora_id, const int32_t* req_len, int n,
                                     int32_t* lora_ids, int32_t* lora_len, int32_t* segment) {
  if (n <= 0) return -1; /* the reference indexes requests[0] */
  int S = 1;
  lora_ids[0] = req_lora_id[0];
  lora_len[0] = 0;
  for (int i = 0; i < n; ++i) {
    if (lora_ids[S - 1] == req_lora_id[i]) {
      lora_len[S - 1] += req_len[i];
    } else {
      lora_ids[S] = req_lora_id[i];
      lora_len[S] = req_len[i];
      ++S;
    }
  }
  segment[0] = 0;
  for (int i = 0; i < S; ++i) segment[i + 1] = segment[i] + lora_len[i];
  return S;
}

/* ---- BatchLenInfo row layout ------------------------------------------------
 * Follows src/loquetier_src/kernel_utils.py:22-53: train_partition =
 * cumsum([0] + bsz*seqlen), tlen = its last entry, doff = tlen + sum of the
 * prefill lengths.  train_partition needs n_train+1 entries.               */
ORACLE_API int oracle_batch_len_info(const int32_t* train_bsz, const int32_t* train_seqlen,
                                     int n_train, const int32_t* prefills, int n_prefill,
                                     int32_t* train_partition, int32_t* tlen, int32_t* doff) {
  if (n_train < 0 || n_prefill < 0) return -1;
  train_partition[0] = 0;
  for (int i = 0; i < n_train; ++i)
    train_partition[i + 1] = train_partition[i] + train_bsz[i] * train_seqlen[i];
  *tlen = train_partition[n_train];
  int32_t pre = 0;
  for (int i = 0; i < n_prefill; ++i) pre += prefills[i];
  *doff = *tlen + pre;
  return 0;
}

/* ---- rank padding and scale folding -----------------------------------------
 * Follows src/loquetier_src/models/mixed_lora.py:501-521: a weight whose rank
 * dimension is smaller than the layer rank is copied into the top-left corner
 * of a zero matrix of the layer rank; `scaling` (0 = none) is multiplied in
 * before the cast to the I/O dtype.  rank_dim 0: w is [r0, cols] -> [r, cols];
 * rank_dim 1: w is [rows, r0] -> [rows, r].                                  */
ORACLE_API int oracle_prepare_weight(float* out, const float* w, int rows, int cols,
                                     int rank_dim, int rank, float scaling, int dtype) {
  int orow = rank_dim == 0 ? rank : rows;
  int ocol = rank_dim == 1 ? rank : cols;
  if (rows > orow || cols > ocol) return -1;
  memset(out, 0, (size_t)orow * ocol * sizeof(float));
  for (int i = 0; i < rows; ++i)
    for (int j = 0; j < cols; ++j) {
      float val = w[(long)i * cols + j];
      if (scaling != 0.0f) val *= scaling;
      out[(long)i * ocol + j] = round_dtype(val, dtype);
    }
  return 0;
}
