// RMSNorm forward and backward for gfx950.
//
// Forward takes the place of rmsnorm_twoPassAlgo_e8
// (kernel_src/csrc/rms_norm/rms_norm_cutlass.cu:81-159): out = x * rms * w with
// rms = 1 / sqrt(mean(x^2) + eps) per row, rms kept as float for the backward.
// The reference reads every row twice; here a row stays in registers between
// the sum of squares and the scaling, so it is read once.
//
// Backward takes the place of the tensor expressions of rms_norm.backward
// (src/loquetier_src/kernel_utils.py:169-176):
//   dot = sum_j g*w*x,  dx = (g*w - x*dot*rms^2/n) * rms,  dw = sum_rows x*rms*g
// in float throughout, one pass over x and g; dw is summed per workgroup into a
// float partial and folded by a second launch in fixed order (no atomics).
//
// Both are streaming kernels bound by HBM: 2*n bytes read + 2*n written per
// row forward, 4*n read + 2*n written backward.
#pragma once
#include "smlm_common.hpp"

namespace smlm {

constexpr int kRmsChunks = 8;                       // 512-element chunks a wave keeps in registers
constexpr int kRmsWaveCols = 512 * kRmsChunks;      // columns one wave covers
constexpr int kRmsMaxCols = 4 * kRmsWaveCols;       // four waves per row at most
constexpr int kRmsFoldRows = 16;                    // partial rows summed side by side in the fold

// Sum over the wave with DPP adds (shifts inside rows of 16 lanes, then the
// row totals); every lane returns the total.
__device__ __forceinline__ float wave_sum_f32(float x) {
#define SMLM_DPP_ADD(ctrl, rmask)                                                                      \
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), ctrl, rmask, \
                                                             0xf, false))
  SMLM_DPP_ADD(0x111, 0xf);  // row_shr:1
  SMLM_DPP_ADD(0x112, 0xf);  // row_shr:2
  SMLM_DPP_ADD(0x114, 0xf);  // row_shr:4
  SMLM_DPP_ADD(0x118, 0xf);  // row_shr:8
  SMLM_DPP_ADD(0x142, 0xa);  // row_bcast:15 into rows 1 and 3
  SMLM_DPP_ADD(0x143, 0xc);  // row_bcast:31 into rows 2 and 3
#undef SMLM_DPP_ADD
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

template <int DT>
__device__ __forceinline__ void unpack8(u32x4 v, float (&f)[8]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    f[2 * e] = Num<DT>::lo(v[e]);
    f[2 * e + 1] = Num<DT>::hi(v[e]);
  }
}

struct RmsFwdArgs {
  uint16_t* out;        // [rows, cols]
  float* rms;           // [rows]
  const uint16_t* x;    // [rows, cols]
  const uint16_t* w;    // [cols]
  int rows, cols;
  float eps;
};

// WPR waves share a row (1: cols <= 4096, 4: cols <= 16384); a workgroup of four
// waves handles 4 / WPR rows at a time and walks rows blockIdx.x * (4 / WPR),
// + gridDim.x * (4 / WPR), ...  Chunk i of wave v covers the 512 columns starting
// at (i * WPR + v) * 512, eight per lane.  When a workgroup has more than one
// turn, the next row is on its way from memory while the current one is
// reduced, scaled and stored.  (Measured: one turn per workgroup is fastest for
// the forward, four for the backward, whose per-workgroup dw partials cost
// traffic of their own.)
// x is read and the output written non-temporally: both are touched once per launch (the next
// reader of x is the backward, much later; a reader of the output that follows at once still
// finds it in the caches when it fits them).
template <int DT, int WPR, bool ONE_TURN>
__global__ __launch_bounds__(256) void rms_fwd_kernel(RmsFwdArgs a) {
  __shared__ float part[2][4];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int sub = wave % WPR;
  constexpr int kRows = 4 / WPR;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  bool ok[kRmsChunks];
  u32x4 wv[kRmsChunks], xv[kRmsChunks];
#pragma unroll
  for (int i = 0; i < kRmsChunks; ++i) {
    const int col = ((i * WPR + sub) * 64 + lane) * 8;
    ok[i] = col < a.cols;
    wv[i] = ldg16(a.w + (ok[i] ? col : 0));
  }
  auto load_row = [&](int row, u32x4 (&v)[kRmsChunks]) {
    const uint16_t* xr = a.x + (long)(row < a.rows ? row : 0) * a.cols;
#pragma unroll
    for (int i = 0; i < kRmsChunks; ++i) {
      const int col = ((i * WPR + sub) * 64 + lane) * 8;
      v[i] = ldg16_nt(xr + (ok[i] ? col : 0));
    }
  };
  const int step = (int)gridDim.x * kRows;
  int row = (int)blockIdx.x * kRows + wave / WPR;
  load_row(row, xv);
  int parity = 0;
  // WPR == 4: `row` is uniform over the workgroup, so every wave reaches the barrier
  for (; row < a.rows; row += step) {
    u32x4 xn[kRmsChunks];
    if (ONE_TURN) {
#pragma unroll
      for (int i = 0; i < kRmsChunks; ++i) xn[i] = zero;
    } else {
      // unconditional (past the last row it re-reads row 0): a branch around the loads would
      // make the wave wait for everything in flight where the paths join
      load_row(row + step, xn);
    }
    __builtin_amdgcn_sched_barrier(0);  // the next row's loads are issued before this row is used
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < kRmsChunks; ++i) {
      if (!ok[i]) xv[i] = zero;
      float f[8];
      unpack8<DT>(xv[i], f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
    }
    ss = wave_sum_f32(ss);
    if (WPR > 1) {
      if (lane == 0) part[parity][wave] = ss;
      __syncthreads();  // one barrier a row: the two halves of `part` alternate
      ss = (part[parity][0] + part[parity][1]) + (part[parity][2] + part[parity][3]);
      parity ^= 1;
    }
    const float rms = 1.0f / sqrtf(ss / (float)a.cols + a.eps);
    if (lane == 0 && sub == 0) a.rms[row] = rms;
    uint16_t* orow = a.out + (long)row * a.cols;
#pragma unroll
    for (int i = 0; i < kRmsChunks; ++i) {
      const int col = ((i * WPR + sub) * 64 + lane) * 8;
      if (!ok[i]) continue;
      float f[8], g[8];
      unpack8<DT>(xv[i], f);
      unpack8<DT>(wv[i], g);
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = pack2<DT>(f[2 * e] * rms * g[2 * e], f[2 * e + 1] * rms * g[2 * e + 1]);
      stg16_nt(orow + col, o);
    }
#pragma unroll
    for (int i = 0; i < kRmsChunks; ++i) xv[i] = xn[i];
  }
}

struct RmsBwdArgs {
  uint16_t* dx;         // [rows, cols]
  float* partial;       // [gridDim.x, cols] per-workgroup sums of x*rms*g
  const uint16_t* g;    // [rows, cols] upstream gradient
  const uint16_t* x;    // [rows, cols]
  const uint16_t* w;    // [cols]
  const float* rms;     // [rows]
  int rows, cols;
};

// A workgroup walks rows blockIdx.x, blockIdx.x + gridDim.x, ... (WPR == 4: one
// row at a time, a quarter of the columns per wave; WPR == 1: four rows at a
// time, one per wave) and keeps its share of dw in registers.
template <int DT, int WPR>
__global__ __launch_bounds__(256) void rms_bwd_kernel(RmsBwdArgs a) {
  __shared__ float part[2][4];
  __shared__ __attribute__((aligned(16))) float dwred[WPR == 1 ? 4 * (kRmsWaveCols / 2) : 4];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int sub = wave % WPR;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const float inv_n = 1.0f / (float)a.cols;

  u32x4 wv[kRmsChunks];
#pragma unroll
  for (int i = 0; i < kRmsChunks; ++i) {
    const int col = ((i * WPR + sub) * 64 + lane) * 8;
    wv[i] = col < a.cols ? ldg16(a.w + col) : zero;
  }
  float dw[kRmsChunks][8];
#pragma unroll
  for (int i = 0; i < kRmsChunks; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) dw[i][e] = 0.0f;

  constexpr int kRows = 4 / WPR;
  bool ok[kRmsChunks];
#pragma unroll
  for (int i = 0; i < kRmsChunks; ++i) ok[i] = ((i * WPR + sub) * 64 + lane) * 8 < a.cols;
  auto load_row = [&](int row, u32x4 (&xr)[kRmsChunks], u32x4 (&gr)[kRmsChunks], float& r) {
    const long off = (long)(row < a.rows ? row : 0) * a.cols;
#pragma unroll
    for (int i = 0; i < kRmsChunks; ++i) {
      const int col = ((i * WPR + sub) * 64 + lane) * 8;
      xr[i] = ldg16_nt(a.x + off + (ok[i] ? col : 0));
      gr[i] = ldg16_nt(a.g + off + (ok[i] ? col : 0));
    }
    r = a.rms[row < a.rows ? row : 0];
  };
  const int step = (int)gridDim.x * kRows;
  int row = (int)blockIdx.x * kRows + wave / WPR;
  u32x4 xv[kRmsChunks], gv[kRmsChunks];
  float rms;
  load_row(row, xv, gv, rms);
  int parity = 0;
  // WPR == 4: `row` is uniform over the workgroup, so every wave reaches the barrier
  for (; row < a.rows; row += step) {
    const long off = (long)row * a.cols;
    u32x4 xn[kRmsChunks], gn[kRmsChunks];
    float rms_n = 0.0f;
    // unconditional (past the last row it re-reads row 0): a branch around the loads would make
    // the wave wait for everything in flight where the paths join
    load_row(row + step, xn, gn, rms_n);
    __builtin_amdgcn_sched_barrier(0);  // the next row's loads are issued before this row is used
    float dot = 0.0f;
#pragma unroll
    for (int i = 0; i < kRmsChunks; ++i) {
      if (!ok[i]) xv[i] = gv[i] = zero;
      float xf[8], gf[8], wf[8];
      unpack8<DT>(xv[i], xf);
      unpack8<DT>(gv[i], gf);
      unpack8<DT>(wv[i], wf);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot += gf[e] * wf[e] * xf[e];
    }
    dot = wave_sum_f32(dot);
    if (WPR > 1) {
      if (lane == 0) part[parity][wave] = dot;
      __syncthreads();  // one barrier a row: the two halves of `part` alternate
      dot = (part[parity][0] + part[parity][1]) + (part[parity][2] + part[parity][3]);
      parity ^= 1;
    }
    const float coef = dot * rms * rms * inv_n;
#pragma unroll
    for (int i = 0; i < kRmsChunks; ++i) {
      const int col = ((i * WPR + sub) * 64 + lane) * 8;
      if (!ok[i]) continue;
      float xf[8], gf[8], wf[8];
      unpack8<DT>(xv[i], xf);
      unpack8<DT>(gv[i], gf);
      unpack8<DT>(wv[i], wf);
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        o[e] = pack2<DT>((gf[2 * e] * wf[2 * e] - xf[2 * e] * coef) * rms,
                         (gf[2 * e + 1] * wf[2 * e + 1] - xf[2 * e + 1] * coef) * rms);
      stg16_nt(a.dx + off + col, o);
#pragma unroll
      for (int e = 0; e < 8; ++e) dw[i][e] += xf[e] * rms * gf[e];
    }
#pragma unroll
    for (int i = 0; i < kRmsChunks; ++i) xv[i] = xn[i], gv[i] = gn[i];
    rms = rms_n;
  }

  float* prow = a.partial + (long)blockIdx.x * a.cols;
  if (WPR == 1) {
    // the four waves hold sums over different rows of the same columns: add them in wave
    // order through LDS, half of the columns at a time
    constexpr int kHalf = kRmsWaveCols / 2;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int i = 0; i < kRmsChunks / 2; ++i) {
        const int ci = h * (kRmsChunks / 2) + i, lc = (i * 64 + lane) * 8;
        *reinterpret_cast<f32x4*>(&dwred[wave * kHalf + lc]) = f32x4{dw[ci][0], dw[ci][1], dw[ci][2], dw[ci][3]};
        *reinterpret_cast<f32x4*>(&dwred[wave * kHalf + lc + 4]) = f32x4{dw[ci][4], dw[ci][5], dw[ci][6], dw[ci][7]};
      }
      __syncthreads();
      for (int lc = threadIdx.x * 4; lc < kHalf && h * kHalf + lc < a.cols; lc += 256 * 4) {
        f32x4 s = *reinterpret_cast<const f32x4*>(&dwred[lc]);
#pragma unroll
        for (int v = 1; v < 4; ++v) s += *reinterpret_cast<const f32x4*>(&dwred[v * kHalf + lc]);
        *(SMLM_GLOBAL f32x4*)(prow + h * kHalf + lc) = s;
      }
      __syncthreads();
    }
  } else {
#pragma unroll
    for (int i = 0; i < kRmsChunks; ++i) {
      const int col = ((i * WPR + sub) * 64 + lane) * 8;
      if (col >= a.cols) continue;
      *(SMLM_GLOBAL f32x4*)(prow + col) = f32x4{dw[i][0], dw[i][1], dw[i][2], dw[i][3]};
      *(SMLM_GLOBAL f32x4*)(prow + col + 4) = f32x4{dw[i][4], dw[i][5], dw[i][6], dw[i][7]};
    }
  }
}

// ---- rows wider than kRmsMaxCols: the row no longer fits the registers of four waves.  Plain
// two-pass kernels (the reference's own scheme, rms_norm_cutlass.cu:81-159): a workgroup per row
// walks the columns once for the reduction and once more for the output (the second pass mostly
// hits L2).  The backward keeps its share of dw in the float partial rows themselves, read and
// written once per row it handles.  Correct for any width that is a multiple of 8; not tuned.
__device__ __forceinline__ float block_sum_f32(float x, float* red4) {
  x = wave_sum_f32(x);
  __syncthreads();  // red4 is free again
  if ((threadIdx.x & 63) == 0) red4[threadIdx.x >> 6] = x;
  __syncthreads();
  return (red4[0] + red4[1]) + (red4[2] + red4[3]);
}

template <int DT>
__global__ __launch_bounds__(256) void rms_fwd_wide_kernel(RmsFwdArgs a) {
  __shared__ float red4[4];
  for (int row = blockIdx.x; row < a.rows; row += gridDim.x) {
    const uint16_t* xr = a.x + (long)row * a.cols;
    float ss = 0.0f;
    for (int col = threadIdx.x * 8; col < a.cols; col += 256 * 8) {
      float f[8];
      unpack8<DT>(ldg16(xr + col), f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
    }
    ss = block_sum_f32(ss, red4);
    const float rms = 1.0f / sqrtf(ss / (float)a.cols + a.eps);
    if (threadIdx.x == 0) a.rms[row] = rms;
    uint16_t* orow = a.out + (long)row * a.cols;
    for (int col = threadIdx.x * 8; col < a.cols; col += 256 * 8) {
      float f[8], g[8];
      unpack8<DT>(ldg16(xr + col), f);
      unpack8<DT>(ldg16(a.w + col), g);
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = pack2<DT>(f[2 * e] * rms * g[2 * e], f[2 * e + 1] * rms * g[2 * e + 1]);
      stg16_nt(orow + col, o);
    }
  }
}

template <int DT>
__global__ __launch_bounds__(256) void rms_bwd_wide_kernel(RmsBwdArgs a) {
  __shared__ float red4[4];
  const float inv_n = 1.0f / (float)a.cols;
  float* prow = a.partial + (long)blockIdx.x * a.cols;
  bool first = true;
  for (int row = blockIdx.x; row < a.rows; row += gridDim.x) {
    const long off = (long)row * a.cols;
    float dot = 0.0f;
    for (int col = threadIdx.x * 8; col < a.cols; col += 256 * 8) {
      float xf[8], gf[8], wf[8];
      unpack8<DT>(ldg16(a.x + off + col), xf);
      unpack8<DT>(ldg16(a.g + off + col), gf);
      unpack8<DT>(ldg16(a.w + col), wf);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot += gf[e] * wf[e] * xf[e];
    }
    dot = block_sum_f32(dot, red4);
    const float rms = a.rms[row], coef = dot * rms * rms * inv_n;
    for (int col = threadIdx.x * 8; col < a.cols; col += 256 * 8) {
      float xf[8], gf[8], wf[8];
      unpack8<DT>(ldg16(a.x + off + col), xf);
      unpack8<DT>(ldg16(a.g + off + col), gf);
      unpack8<DT>(ldg16(a.w + col), wf);
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        o[e] = pack2<DT>((gf[2 * e] * wf[2 * e] - xf[2 * e] * coef) * rms,
                         (gf[2 * e + 1] * wf[2 * e + 1] - xf[2 * e + 1] * coef) * rms);
      stg16_nt(a.dx + off + col, o);
      // this thread's columns of the workgroup's partial row: nobody else touches them
      f32x4 p0 = {0.f, 0.f, 0.f, 0.f}, p1 = p0;
      if (!first) p0 = ldg_f4(prow + col), p1 = ldg_f4(prow + col + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) p0[e] += xf[e] * rms * gf[e], p1[e] += xf[4 + e] * rms * gf[4 + e];
      *(SMLM_GLOBAL f32x4*)(prow + col) = p0;
      *(SMLM_GLOBAL f32x4*)(prow + col + 4) = p1;
    }
    first = false;
  }
  if (first)  // more workgroups than rows never happens (the host sizes the grid), but a partial row must not stay unwritten
    for (int col = threadIdx.x * 4; col < a.cols; col += 256 * 4) *(SMLM_GLOBAL f32x4*)(prow + col) = f32x4{0.f, 0.f, 0.f, 0.f};
}

struct RmsFoldArgs {
  uint16_t* dw;          // [cols]
  const float* partial;  // [n_part, cols]
  int n_part, cols;
};

// grid: ceil(cols / 64), block 256: thread (rg = tid / 16, c4 = tid % 16) adds
// partial rows rg, rg + 16, ... of four columns; the sixteen row groups are then
// added in order through LDS.
template <int DT>
__global__ __launch_bounds__(256) void rms_fold_kernel(RmsFoldArgs a) {
  __shared__ f32x4 red[kRmsFoldRows][16];
  const int rg = threadIdx.x >> 4, c4 = threadIdx.x & 15;
  const int col = (int)blockIdx.x * 64 + c4 * 4;
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  if (col < a.cols) {
    // eight partial rows are requested at a time; rows past the end re-read row rg and are dropped
    for (int p0 = rg; p0 < a.n_part; p0 += 8 * kRmsFoldRows) {
      f32x4 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int p = p0 + j * kRmsFoldRows;
        v[j] = ldg_f4(a.partial + (long)(p < a.n_part ? p : rg) * a.cols + col);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (p0 + j * kRmsFoldRows < a.n_part) s += v[j];
    }
  }
  red[rg][c4] = s;
  __syncthreads();
  if (rg == 0 && col < a.cols) {
    f32x4 t = red[0][c4];
#pragma unroll
    for (int v = 1; v < kRmsFoldRows; ++v) t += red[v][c4];
    u32x2 o;
    o[0] = pack2<DT>(t[0], t[1]);
    o[1] = pack2<DT>(t[2], t[3]);
    *(SMLM_GLOBAL u32x2*)(a.dw + col) = o;
  }
}

}  // namespace smlm
