// Shrink (skinny-N, long-K) and expand (skinny-K, wide-N) tile kernels.
//
// Both take the place of the CUTLASS GemmGrouped instantiations of
// kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:84-171.  One wave owns
// one 16-row plan tile and drives v_mfma_f32_16x16x32 with the tokens as the
// MFMA *columns* and the weight rows as the MFMA *rows*: each lane then ends
// up with consecutive output columns of one token, which is what a coalesced
// store of y needs.  Operand fragments are 16-byte global loads straight into
// registers (both x and the weights are contiguous along the contraction).
//
// Every output element is produced by the same sequence of MFMA steps over k
// whatever other rows share its tile, so regrouping or re-segmenting rows
// never changes a bit of any row.
#pragma once
#include "smlm_common.hpp"

namespace smlm {

constexpr int kFwdThreads = 256;
constexpr int kFwdWaves = kFwdThreads / kWaveSize;

struct TileArgs {
  const int32_t* hdr;
  const int32_t* tile_row;
  const int32_t* tile_rseg;
};

struct ShrinkArgs {
  TileArgs plan;
  const uint16_t* x;         // [T, d_in]
  const void* const* w_ptrs; // per segment, or per adapter with seg_adapter
  const int32_t* seg_adapter;
  float* partial;            // [ksplit, T, d_out] fp32 when ksplit > 1
  uint16_t* out;             // [T, d_out] when ksplit == 1
  const float* seg_scale;    // applied when ksplit == 1
  float beta;
  int T, d_in, d_out, ldw, k_per_wave, ksplit;
};

template <bool ROWMAJOR>
__device__ __forceinline__ u32x4 load_w8(const uint16_t* W, int n, int k, int ldw) {
  // eight consecutive-k elements of weight column n
  if (ROWMAJOR) return ldg_strided8(W + (long)k * ldw + n, ldw);
  return ldg16(W + (long)n * ldw + k);
}

// out = beta*old + scale*acc for four consecutive columns of one row
template <int DT>
__device__ __forceinline__ void store4(uint16_t* dst, f32x4 a, float scale, float beta) {
  u32x2 o;
  if (beta != 0.0f) {
    const u32x2 old = *reinterpret_cast<const u32x2*>(dst);
    o[0] = pack2<DT>(beta * Num<DT>::lo(old[0]) + scale * a[0], beta * Num<DT>::hi(old[0]) + scale * a[1]);
    o[1] = pack2<DT>(beta * Num<DT>::lo(old[1]) + scale * a[2], beta * Num<DT>::hi(old[1]) + scale * a[3]);
  } else {
    o[0] = pack2<DT>(scale * a[0], scale * a[1]);
    o[1] = pack2<DT>(scale * a[2], scale * a[3]);
  }
  *reinterpret_cast<u32x2*>(dst) = o;
}

// grid: (tile, k-split, 64-column block of d_out).  The four waves of a block
// take consecutive k ranges; their accumulators are summed through LDS in wave
// order and written either as an fp32 partial (ksplit > 1) or as the final
// 16-bit value.
template <int DT, int NB, int U, bool ROWMAJOR>
__global__ __launch_bounds__(kFwdThreads) void shrink_kernel(ShrinkArgs a) {
  const int tile = blockIdx.x;
  if (tile >= a.plan.hdr[0]) return;
  const int kz = blockIdx.y;
  const int n0 = blockIdx.z * 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;

  const int row = a.plan.tile_row[tile * kTileRows + c];
  const int seg0 = a.plan.tile_rseg[tile * kTileRows];
  const int ad = a.seg_adapter ? a.seg_adapter[seg0] : seg0;
  const uint16_t* W = reinterpret_cast<const uint16_t*>(a.w_ptrs[ad]);
  const uint16_t* xrow = a.x + (long)(row < 0 ? 0 : row) * a.d_in;

  const int kbeg = (kz * kFwdWaves + wave) * a.k_per_wave;
  const int kend = min(kbeg + a.k_per_wave, a.d_in);

  const u32x4 zero = {0u, 0u, 0u, 0u};
  f32x4 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll 1
  for (int k = kbeg; k < kend; k += 32 * U) {
    u32x4 xf[U], wf[NB][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k + 32 * u + 8 * g;
      const bool kin = kk < kend;
      xf[u] = (kin && row >= 0) ? ldg16(xrow + kk) : zero;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int n = n0 + 16 * nb + c;
        wf[nb][u] = (kin && n < a.d_out) ? load_w8<ROWMAJOR>(W, n, kk, a.ldw) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nb] = Num<DT>::mfma(wf[nb][u], xf[u], acc[nb]);
  }

  __shared__ f32x4 red[kFwdWaves][NB][kWaveSize];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) red[wave][nb][lane] = acc[nb];
  __syncthreads();
  if (wave != 0 || row < 0) return;

  const int rseg = a.plan.tile_rseg[tile * kTileRows + c];
  const float scale = (a.ksplit == 1 && a.seg_scale) ? a.seg_scale[rseg] : 1.0f;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    f32x4 sum = red[0][nb][lane];
#pragma unroll
    for (int w = 1; w < kFwdWaves; ++w) sum += red[w][nb][lane];
    const int n = n0 + 16 * nb + 4 * g;  // lane holds columns n .. n+3 of its token
    if (n >= a.d_out) continue;
    if (a.ksplit > 1) {
      *reinterpret_cast<f32x4*>(a.partial + ((long)kz * a.T + row) * a.d_out + n) = sum;
    } else {
      store4<DT>(a.out + (long)row * a.d_out + n, sum, scale, a.beta);
    }
  }
}

struct ReduceArgs {
  TileArgs plan;
  const float* partial;  // [ksplit, T, d_out]
  uint16_t* out;         // [T, d_out]
  const float* seg_scale;
  float beta;
  int T, d_out, ksplit;
};

// Folds the k-split partials of a standalone shrink call, in split order.
template <int DT>
__global__ __launch_bounds__(256) void reduce_kernel(ReduceArgs a) {
  const int tile = blockIdx.x;
  if (tile >= a.plan.hdr[0]) return;
  const int c = threadIdx.x >> 4, q = threadIdx.x & 15;
  const int row = a.plan.tile_row[tile * kTileRows + c];
  if (row < 0) return;
  const int rseg = a.plan.tile_rseg[tile * kTileRows + c];
  const float scale = a.seg_scale ? a.seg_scale[rseg] : 1.0f;
  for (int n = 4 * q; n < a.d_out; n += 64) {
    f32x4 sum = ldg_f4(a.partial + (long)row * a.d_out + n);
    for (int z = 1; z < a.ksplit; ++z) sum += ldg_f4(a.partial + ((long)z * a.T + row) * a.d_out + n);
    store4<DT>(a.out + (long)row * a.d_out + n, sum, scale, a.beta);
  }
}

struct ExpandArgs {
  TileArgs plan;
  uint16_t* y;               // [T, d_out]
  const uint16_t* v;         // [T, d_in] 16-bit, or null when partials are given
  const float* partial;      // [ksplit, T, d_in] fp32 partial sums of v
  const void* const* w_ptrs;
  const int32_t* seg_adapter;
  const float* seg_scale;
  uint16_t* v_out;           // optional [T, d_in]: rounded v, by row
  uint16_t* pt_a;            // optional [d_in, nt_max*16]: scale*v by tile slot, transposed
  uint16_t* pt_b;            // optional: same treatment of v2 (a second [T, d_in] matrix)
  const uint16_t* v2;
  float beta;
  int T, d_in, d_out, ldw, ksplit, nt_max;
};

// grid: (tile, block of 4*32*NQ output columns).  K (= LoRA rank) is short, so
// the token fragment is built once per 32-wide k step -- summing the shrink
// partials in split order and rounding to 16 bits, which is exactly the "v in
// the I/O dtype" of the reference -- and the weight rows stream through.
// MFMA row m of column block (q,p) is output column 32q + 8(m/4) + 4p + m%4, so
// that a lane's eight accumulators for one q are eight consecutive columns.
template <int DT, int NQ, bool ROWMAJOR>
__global__ __launch_bounds__(kFwdThreads) void expand_kernel(ExpandArgs a) {
  const int tile = blockIdx.x;
  if (tile >= a.plan.hdr[0]) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;
  const int ncol0 = (blockIdx.y * kFwdWaves + wave) * 32 * NQ;
  if (ncol0 >= a.d_out) return;

  const int row = a.plan.tile_row[tile * kTileRows + c];
  const int rseg = a.plan.tile_rseg[tile * kTileRows + c];
  const int seg0 = a.plan.tile_rseg[tile * kTileRows];
  const int ad = a.seg_adapter ? a.seg_adapter[seg0] : seg0;
  const uint16_t* W = reinterpret_cast<const uint16_t*>(a.w_ptrs[ad]);
  const float scale = (a.seg_scale && row >= 0) ? a.seg_scale[rseg] : 1.0f;

  const u32x4 zero = {0u, 0u, 0u, 0u};
  // y rows this lane will update: prefetch the old values early
  u32x4 yold[NQ];
  uint16_t* yrow = a.y + (long)(row < 0 ? 0 : row) * a.d_out + ncol0 + 8 * g;
  if (a.beta != 0.0f) {
#pragma unroll
    for (int q = 0; q < NQ; ++q)
      yold[q] = (row >= 0 && ncol0 + 32 * q + 8 * g < a.d_out) ? ldg16(yrow + 32 * q) : zero;
  }

  f32x4 acc[NQ][2];
#pragma unroll
  for (int q = 0; q < NQ; ++q) acc[q][0] = acc[q][1] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int mrow = 8 * (c >> 2) + (c & 3);  // column offset of MFMA row c inside a (q,p) block
  const bool side = (blockIdx.y == 0 && wave == 0);  // the one wave per tile that writes by-products

#pragma unroll 1
  for (int k0 = 0; k0 < a.d_in; k0 += 32) {
    const int kk = k0 + 8 * g;
    const bool kin = kk < a.d_in;
    u32x4 vf = zero;
    if (kin && row >= 0) {
      if (a.partial) {
        const float* pp = a.partial + (long)row * a.d_in + kk;
        f32x4 s0 = ldg_f4(pp), s1 = ldg_f4(pp + 4);
        for (int z = 1; z < a.ksplit; ++z) {
          const float* pz = pp + (long)z * a.T * a.d_in;
          s0 += ldg_f4(pz);
          s1 += ldg_f4(pz + 4);
        }
        vf[0] = pack2<DT>(s0[0], s0[1]);
        vf[1] = pack2<DT>(s0[2], s0[3]);
        vf[2] = pack2<DT>(s1[0], s1[1]);
        vf[3] = pack2<DT>(s1[2], s1[3]);
      } else {
        vf = ldg16(a.v + (long)row * a.d_in + kk);
      }
    }
    if (side && kin) {
      if (a.v_out && row >= 0) stg16(a.v_out + (long)row * a.d_in + kk, vf);
      if (a.pt_a) {
        // scale*v (and scale*v2) by tile slot, transposed: [k][slot]
        const long slot = (long)tile * kTileRows + c;
        const long pitch = (long)a.nt_max * kTileRows;
        u32x4 v2f = zero;
        if (a.pt_b && row >= 0) v2f = ldg16(a.v2 + (long)row * a.d_in + kk);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a.pt_a[(kk + 2 * e) * pitch + slot] = (uint16_t)Num<DT>::bits(scale * Num<DT>::lo(vf[e]));
          a.pt_a[(kk + 2 * e + 1) * pitch + slot] = (uint16_t)Num<DT>::bits(scale * Num<DT>::hi(vf[e]));
          if (a.pt_b) {
            a.pt_b[(kk + 2 * e) * pitch + slot] = (uint16_t)Num<DT>::bits(scale * Num<DT>::lo(v2f[e]));
            a.pt_b[(kk + 2 * e + 1) * pitch + slot] = (uint16_t)Num<DT>::bits(scale * Num<DT>::hi(v2f[e]));
          }
        }
      }
    }
    u32x4 wf[NQ][2];
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const int n = ncol0 + 32 * q + 4 * p + mrow;
        wf[q][p] = (kin && n < a.d_out) ? load_w8<ROWMAJOR>(W, n, kk, a.ldw) : zero;
      }
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int p = 0; p < 2; ++p) acc[q][p] = Num<DT>::mfma(wf[q][p], vf, acc[q][p]);
  }

  if (row < 0) return;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    if (ncol0 + 32 * q + 8 * g >= a.d_out) continue;
    const f32x4 lo4 = acc[q][0], hi4 = acc[q][1];
    u32x4 o;
    if (a.beta != 0.0f) {
      const u32x4 old = yold[q];
      o[0] = pack2<DT>(a.beta * Num<DT>::lo(old[0]) + scale * lo4[0], a.beta * Num<DT>::hi(old[0]) + scale * lo4[1]);
      o[1] = pack2<DT>(a.beta * Num<DT>::lo(old[1]) + scale * lo4[2], a.beta * Num<DT>::hi(old[1]) + scale * lo4[3]);
      o[2] = pack2<DT>(a.beta * Num<DT>::lo(old[2]) + scale * hi4[0], a.beta * Num<DT>::hi(old[2]) + scale * hi4[1]);
      o[3] = pack2<DT>(a.beta * Num<DT>::lo(old[3]) + scale * hi4[2], a.beta * Num<DT>::hi(old[3]) + scale * hi4[3]);
    } else {
      o[0] = pack2<DT>(scale * lo4[0], scale * lo4[1]);
      o[1] = pack2<DT>(scale * lo4[2], scale * lo4[3]);
      o[2] = pack2<DT>(scale * hi4[0], scale * hi4[1]);
      o[3] = pack2<DT>(scale * hi4[2], scale * hi4[3]);
    }
    stg16(yrow + 32 * q, o);
  }
}

}  // namespace smlm
