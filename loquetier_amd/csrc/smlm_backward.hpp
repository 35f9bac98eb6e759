// Backward-only kernels: weight transposes and the per-adapter token
// reductions dA_a = sum_t dV[t,:]^T x[t,:], dB_a = sum_t dY[t,:]^T v[t,:].
//
// The reference computes these with one torch matmul per train partition
// (src/loquetier_src/kernel_utils.py:139-145); its C++ side has no backward
// (kernel_src/csrc/loquetier_ops.cc:321-322).
#pragma once
#include "smlm_common.hpp"

namespace smlm {

struct TransposeSet {
  const void* const* src_ptrs;  // [NA] matrices [rows, cols] row-major
  uint16_t* dst_base;           // NA matrices [cols, rows], `stride` elements apart
  const void** dst_ptrs;        // [NA] receives the address of each transposed matrix
  long stride;
  int rows, cols;
};

struct TransposeArgs {
  TransposeSet set[2];  // A [r, h_in] -> At [h_in, r] and B [h_out, r] -> Bt [r, h_out]
  int NA;
};

// 32x32 tiles through LDS; grid (tiles along the hidden dimension, tiles along the
// rank, 2*NA), block 256: x walks the columns of A and the rows of B.
__global__ __launch_bounds__(256) void transpose_kernel(TransposeArgs a) {
  __shared__ uint16_t t[32][33];
  const int which = blockIdx.z / a.NA, ad = blockIdx.z - which * a.NA;
  const TransposeSet S = a.set[which];
  const int c0 = (which == 0 ? blockIdx.x : blockIdx.y) * 32;
  const int r0 = (which == 0 ? blockIdx.y : blockIdx.x) * 32;
  if (c0 >= S.cols || r0 >= S.rows) return;  // uniform over the workgroup
  const uint16_t* src = reinterpret_cast<const uint16_t*>(S.src_ptrs[ad]);
  uint16_t* dst = S.dst_base + (long)ad * S.stride;
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) S.dst_ptrs[ad] = dst;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + ty + 8 * i, c = c0 + tx;
    t[ty + 8 * i][tx] = (r < S.rows && c < S.cols) ? src[(long)r * S.cols + c] : (uint16_t)0;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = c0 + ty + 8 * i, r = r0 + tx;
    if (r < S.rows && c < S.cols) dst[(long)c * S.rows + r] = t[tx][ty + 8 * i];
  }
}

struct WgradArgs {
  const int32_t* hdr;
  const int32_t* grp_tile;
  const int32_t* grp_id;
  const int32_t* tile_row;
  const uint16_t* q_a;   // x  [n_rows, h_in]   -> dA
  const uint16_t* q_b;   // dY [n_rows, h_out]  -> dB
  const uint16_t* pt_a;  // scale*dV by slot, transposed [r, pitch]
  const uint16_t* pt_b;  // scale*v  by slot, transposed [r, pitch]
  void* const* da_ptrs;  // [NA] -> [r, h_in]
  void* const* db_ptrs;  // [NA] -> [h_out, r]
  long pitch;
  int h_in, h_out, r, chunks_a;  // chunks_a = ceil(h_in/64): blockIdx.x below it works on dA
};

constexpr int kWgCols = 64;    // columns of x / dY per workgroup
constexpr int kWgPitch = 72;   // LDS row pitch in 16-bit elements (144 B: 16-byte aligned rows)

// grid: (ceil(h_in/64) + ceil(h_out/64), NA), block 256.  A workgroup owns 64
// columns of one adapter's dA or dB and walks all of that adapter's tiles, 32
// gathered rows (two tiles) per MFMA k step, the four waves taking k steps
// round-robin; the waves' accumulators are then summed through LDS in wave
// order.  The token dimension is the contraction, so the [token][column] block
// of x / dY is staged in LDS and read back with the token index innermost.
template <int DT, int NBJ>
__global__ __launch_bounds__(256) void wgrad_kernel(WgradArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t stage[4][32 * kWgPitch];
  __shared__ f32x4 red[4][4][kWaveSize];

  const int ad = blockIdx.y;
  const bool is_a = (int)blockIdx.x < a.chunks_a;
  const int n0 = (is_a ? blockIdx.x : blockIdx.x - a.chunks_a) * kWgCols;
  const int h = is_a ? a.h_in : a.h_out;
  const uint16_t* Q = is_a ? a.q_a : a.q_b;
  const uint16_t* PT = is_a ? a.pt_a : a.pt_b;
  // an address read from a table has no known address space; say it is global
  typedef __attribute__((address_space(1))) u32x2 global_u32x2;
  uint16_t* out = reinterpret_cast<uint16_t*>(is_a ? a.da_ptrs[ad] : a.db_ptrs[ad]);

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;

  // group of this adapter: groups are sorted by id
  const int NG = a.hdr[1];
  int lo = 0, hi = NG;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (a.grp_id[mid] < ad) lo = mid + 1; else hi = mid;
  }
  int t_beg = 0, t_end = 0;
  if (lo < NG && a.grp_id[lo] == ad) {
    t_beg = a.grp_tile[lo];
    t_end = a.grp_tile[lo + 1];
  }
  const int n_steps = (t_end - t_beg + 1) >> 1;
  const int n_iter = (n_steps + 3) >> 2;  // same trip count for all four waves

  const u32x4 zero = {0u, 0u, 0u, 0u};
  f32x4 acc[NBJ][4];
#pragma unroll
  for (int jb = 0; jb < NBJ; ++jb)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) acc[jb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  uint16_t* st = stage[wave];
  const int lrow = lane >> 3, lcol = (lane & 7) * 8;  // staging: 8 lanes cover 64 columns of a row

  for (int it = 0; it < n_iter; ++it) {
    const int step = it * 4 + wave;
    const int tile0 = t_beg + 2 * step;
    const bool live = step < n_steps;
    // stage 32 gathered rows x 64 columns
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int sl = 8 * u + lrow;  // slot 0..31 of this k step
      const int tile = tile0 + (sl >> 4);
      u32x4 val = zero;
      if (live && tile < t_end && n0 + lcol < h) {
        const int row = a.tile_row[tile * kTileRows + (sl & 15)];
        if (row >= 0) val = ldg16(Q + (long)row * h + n0 + lcol);
      }
      *reinterpret_cast<u32x4*>(st + sl * kWgPitch + lcol) = val;
    }
    // token-side operand: PT[j][slot .. slot+7] for the 8 slots of lane group g
    u32x4 pf[NBJ];
#pragma unroll
    for (int jb = 0; jb < NBJ; ++jb) {
      const int j = 16 * jb + c;
      const int tile = tile0 + (g >> 1);
      pf[jb] = (live && tile < t_end && j < a.r)
                   ? ldg16(PT + (long)j * a.pitch + (long)tile0 * kTileRows + 8 * g)
                   : zero;
    }
    __syncthreads();
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      // column-side operand: Q[slot 8g..8g+7][n0 + 16nb + c], token index innermost
      u32x4 qf;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t v0 = st[(8 * g + 2 * e) * kWgPitch + 16 * nb + c];
        const uint32_t v1 = st[(8 * g + 2 * e + 1) * kWgPitch + 16 * nb + c];
        qf[e] = v0 | (v1 << 16);
      }
#pragma unroll
      for (int jb = 0; jb < NBJ; ++jb) {
        // dA: rows = columns of x, cols = rank -> lane holds 4 consecutive x columns of rank c
        // dB: rows = rank, cols = columns of dY -> lane holds 4 consecutive ranks of column c
        acc[jb][nb] = is_a ? Num<DT>::mfma(qf, pf[jb], acc[jb][nb]) : Num<DT>::mfma(pf[jb], qf, acc[jb][nb]);
      }
    }
    __syncthreads();
  }

  // cross-wave sum in wave order, one rank block at a time, then store
  for (int jb = 0; jb < NBJ; ++jb) {
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) red[wave][nb][lane] = acc[jb][nb];
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        f32x4 s = red[0][nb][lane];
#pragma unroll
        for (int w = 1; w < 4; ++w) s += red[w][nb][lane];
        u32x2 o;
        o[0] = pack2<DT>(s[0], s[1]);
        o[1] = pack2<DT>(s[2], s[3]);
        if (is_a) {
          // D[m = x column 16nb + 4g + i][n = rank 16jb + c]
          const int j = 16 * jb + c, n = n0 + 16 * nb + 4 * g;
          if (j < a.r && n < h) *(global_u32x2*)(out + (long)j * h + n) = o;
        } else {
          // D[m = rank 16jb + 4g + i][n = dY column 16nb + c]
          const int j = 16 * jb + 4 * g, n = n0 + 16 * nb + c;
          if (j < a.r && n < h) *(global_u32x2*)(out + (long)n * a.r + j) = o;
        }
      }
    }
    __syncthreads();
  }
}

}  // namespace smlm
