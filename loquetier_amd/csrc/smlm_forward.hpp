// Shrink (skinny-N, long-K) and expand (skinny-K, wide-N) tile kernels.
//
// Both take the place of the CUTLASS GemmGrouped instantiations of
// kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:84-171.  One wave owns
// up to MT 16-row plan tiles of one adapter and drives v_mfma_f32_16x16x32 with
// the tokens as the MFMA *columns* and the weight rows as the MFMA *rows*: each
// lane then ends up with consecutive output columns of one token, which is what
// a coalesced store of y needs.  Operand fragments are 16-byte global loads
// straight into registers (x and the weights are both contiguous along the
// contraction); a weight fragment is loaded once and used for all MT tiles.
//
// Every output element is produced by the same sequence of MFMA steps over k
// whatever other rows share its tile or its wave, so regrouping or
// re-segmenting rows never changes a bit of any row.
//
// Launches are one-dimensional.  Workgroups are handed to the 8 XCDs round
// robin by their linear id, and each XCD has its own L2; xcd_remap() turns the
// linear id into a work index such that each XCD walks one contiguous range of
// (column chunk | k slice, tile block) pairs: all tile blocks that read one
// slice of an adapter's weights run on the same XCD close in time, so that
// slice is fetched from HBM once instead of once per XCD.
#pragma once
#include "smlm_common.hpp"

namespace smlm {

constexpr int kFwdThreads = 256;
constexpr int kFwdWaves = kFwdThreads / kWaveSize;
constexpr int kMaxProj = 8;   // projections one launch can serve
constexpr int kNumXcd = 8;

struct TileArgs {
  const int32_t* hdr;        // 0 n_tiles, 4 n_blocks
  const int32_t* tile_row;
  const int32_t* tile_rseg;
  const int32_t* tile_wid;
  const int32_t* blk;        // (first tile << 3) | tile count, per tile block
};

__device__ __forceinline__ int xcd_remap(int linear, int total) {
  const int xcd = linear % kNumXcd, idx = linear / kNumXcd;
  const int base = total / kNumXcd, extra = total % kNumXcd;
  return xcd * base + (xcd < extra ? xcd : extra) + idx;
}

// which tiles this workgroup works on: a single tile (MT == 1) or one tile
// block of the plan (tiles of one adapter)
template <int MT>
__device__ __forceinline__ bool pick_tiles(const TileArgs& p, int tb, int* t0, int* cnt) {
  if (MT == 1) {
    if (tb >= p.hdr[0]) return false;
    *t0 = tb;
    *cnt = 1;
  } else {
    if (tb >= p.hdr[4]) return false;
    const int packed = p.blk[tb];
    *t0 = packed >> 3;
    *cnt = packed & 7;
  }
  return true;
}

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

// ------------------------------------------------------------------ shrink --
struct ShrinkProj {
  const uint16_t* x;          // [T, d_in]
  const void* const* w_ptrs;  // indexed by the plan's tile_wid
  float* partial;             // [ksplit, T, d_out] fp32 when ksplit > 1
  uint16_t* out;              // [T, d_out] when ksplit == 1
  int d_in, d_out, ldw, k_per_wave, ksplit, zblocks;
};

struct ShrinkArgs {
  TileArgs plan;
  ShrinkProj p[kMaxProj];
  const float* seg_scale;     // applied when ksplit == 1
  float beta;
  int T, nproj, gx, gy;       // gx tile blocks, gy = max over projections of ksplit*zblocks
};

// Work index -> (projection, k slice, 64-column block, tile block).  The four
// waves of a workgroup take consecutive k ranges; their accumulators are summed
// through LDS in wave order and written either as an fp32 partial (ksplit > 1)
// or as the final 16-bit value.
template <int DT, int NB, int U, int MT, bool ROWMAJOR>
__global__ __launch_bounds__(kFwdThreads) void shrink_kernel(ShrinkArgs a) {
  const int V = xcd_remap(blockIdx.x, gridDim.x);
  const int per = a.gx * a.gy;
  const int pj = V / per, rem = V - pj * per;
  const int yy = rem / a.gx, tb = rem - yy * a.gx;
  const ShrinkProj P = a.p[pj];
  const int kz = yy % P.ksplit, zb = yy / P.ksplit;
  if (zb >= P.zblocks) return;
  int t0, cnt;
  if (!pick_tiles<MT>(a.plan, tb, &t0, &cnt)) return;

  const int n0 = zb * 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;

  int row[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) row[i] = i < cnt ? a.plan.tile_row[(t0 + i) * kTileRows + c] : -1;
  const uint16_t* W = reinterpret_cast<const uint16_t*>(P.w_ptrs[a.plan.tile_wid[t0]]);

  const int kbeg = (kz * kFwdWaves + wave) * P.k_per_wave;
  const int kend = min(kbeg + P.k_per_wave, P.d_in);

  const u32x4 zero = {0u, 0u, 0u, 0u};
  f32x4 acc[MT][NB];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[i][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll 1
  for (int k = kbeg; k < kend; k += 32 * U) {
    u32x4 xf[MT][U], wf[NB][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k + 32 * u + 8 * g;
      const bool kin = kk < kend;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int n = n0 + 16 * nb + c;
        wf[nb][u] = (kin && n < P.d_out) ? load_w8<ROWMAJOR>(W, n, kk, P.ldw) : zero;
      }
#pragma unroll
      for (int i = 0; i < MT; ++i)
        xf[i][u] = (kin && row[i] >= 0) ? ldg16(P.x + (long)row[i] * P.d_in + kk) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < MT; ++i)
        if (i < cnt) {
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) acc[i][nb] = Num<DT>::mfma(wf[nb][u], xf[i][u], acc[i][nb]);
        }
  }

  // cross-wave sum, TP tiles per pass, wave j finishing tile j of the pass
  constexpr int TP = (MT * NB > 8) ? 8 / NB : MT;
  __shared__ f32x4 red[kFwdWaves][TP][NB][kWaveSize];
#pragma unroll
  for (int pass = 0; pass < MT / TP; ++pass) {
    if (pass * TP >= cnt) break;  // uniform over the workgroup
#pragma unroll
    for (int j = 0; j < TP; ++j)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) red[wave][j][nb][lane] = acc[pass * TP + j][nb];
    __syncthreads();
    const int i = pass * TP + wave;
    if (wave < TP && i < cnt) {
      const int slot = (t0 + i) * kTileRows + c;
      const int r = a.plan.tile_row[slot];
      if (r >= 0) {
        float scale = 1.0f;
        if (P.ksplit == 1 && a.seg_scale) scale = a.seg_scale[a.plan.tile_rseg[slot]];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          f32x4 sum = red[0][wave][nb][lane];
#pragma unroll
          for (int w = 1; w < kFwdWaves; ++w) sum += red[w][wave][nb][lane];
          const int n = n0 + 16 * nb + 4 * g;  // lane holds columns n .. n+3 of its token
          if (n >= P.d_out) continue;
          if (P.ksplit > 1)
            *reinterpret_cast<f32x4*>(P.partial + ((long)kz * a.T + r) * P.d_out + n) = sum;
          else
            store4<DT>(P.out + (long)r * P.d_out + n, sum, scale, a.beta);
        }
      }
    }
    __syncthreads();
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

// ------------------------------------------------------------------ expand --
struct ExpandProj {
  uint16_t* y;                // [T, d_out]
  const uint16_t* v;          // [T, d_in] 16-bit, or null when partials are given
  const float* partial;       // [ksplit, T, d_in] fp32 partial sums of v
  const void* const* w_ptrs;  // indexed by the plan's tile_wid
  uint16_t* v_out;            // optional [T, d_in]: rounded v, by row
  int d_in, d_out, ldw, ksplit;
};

struct ExpandArgs {
  TileArgs plan;
  ExpandProj p[kMaxProj];
  const float* seg_scale;
  uint16_t* pt_a;            // optional [d_in, nt_max*16]: scale*v by tile slot, transposed
  uint16_t* pt_b;            // optional: same treatment of v2 (a second [T, d_in] matrix)
  const uint16_t* v2;
  float beta;
  int T, nproj, gx, gy, nt_max;  // gx tile blocks, gy = max column chunks
};

// one 32-wide k step of the token operand: partial sums folded in split order
// and rounded to 16 bits (the reference's "v in the I/O dtype"), or 16-bit v
template <int DT>
__device__ __forceinline__ u32x4 load_v8(const ExpandProj& P, int T, int row, int kk) {
  if (P.partial) {
    const float* pp = P.partial + (long)row * P.d_in + kk;
    f32x4 s0 = ldg_f4(pp), s1 = ldg_f4(pp + 4);
    for (int z = 1; z < P.ksplit; ++z) {
      const float* pz = pp + (long)z * T * P.d_in;
      s0 += ldg_f4(pz);
      s1 += ldg_f4(pz + 4);
    }
    u32x4 r;
    r[0] = pack2<DT>(s0[0], s0[1]);
    r[1] = pack2<DT>(s0[2], s0[3]);
    r[2] = pack2<DT>(s1[0], s1[1]);
    r[3] = pack2<DT>(s1[2], s1[3]);
    return r;
  }
  return ldg16(P.v + (long)row * P.d_in + kk);
}

// Work index -> (projection, column chunk, tile block); each wave of the
// workgroup owns 32*NQ output columns.  K (= LoRA rank) is short: with KS > 0
// the weight fragments of all KS 32-wide k steps stay in registers and serve
// every tile of the block; KS == 0 is the general loop over k.
// MFMA row m of column block (q,p) is output column 32q + 8(m/4) + 4p + m%4, so
// that a lane's eight accumulators for one q are eight consecutive columns.
template <int DT, int NQ, int KS, int MT, bool ROWMAJOR>
__global__ __launch_bounds__(kFwdThreads) void expand_kernel(ExpandArgs a) {
  const int V = xcd_remap(blockIdx.x, gridDim.x);
  const int per = a.gx * a.gy;
  const int pj = V / per, rem = V - pj * per;
  const int yy = rem / a.gx, tb = rem - yy * a.gx;
  const ExpandProj P = a.p[pj];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;
  const int ncol0 = (yy * kFwdWaves + wave) * 32 * NQ;
  if (ncol0 >= P.d_out) return;
  int t0, cnt;
  if (!pick_tiles<MT>(a.plan, tb, &t0, &cnt)) return;
  const uint16_t* W = reinterpret_cast<const uint16_t*>(P.w_ptrs[a.plan.tile_wid[t0]]);

  const u32x4 zero = {0u, 0u, 0u, 0u};
  const int mrow = 8 * (c >> 2) + (c & 3);  // column offset of MFMA row c inside a (q,p) block
  const bool side = (yy == 0 && wave == 0);  // the one wave per tile that writes by-products
  constexpr int KSR = KS > 0 ? KS : 1;

  u32x4 wf[KSR][NQ][2];
  if (KS > 0) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int kk = 32 * ks + 8 * g;
#pragma unroll
      for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          const int n = ncol0 + 32 * q + 4 * p + mrow;
          wf[ks][q][p] = (kk < P.d_in && n < P.d_out) ? load_w8<ROWMAJOR>(W, n, kk, P.ldw) : zero;
        }
    }
  }

#pragma unroll
  for (int i = 0; i < MT; ++i) {
    if (i >= cnt) break;
    const int slot = (t0 + i) * kTileRows + c;
    const int row = a.plan.tile_row[slot];
    const float scale = (a.seg_scale && row >= 0) ? a.seg_scale[a.plan.tile_rseg[slot]] : 1.0f;

    // y rows this lane will update: fetch the old values early
    u32x4 yold[NQ];
    uint16_t* yrow = P.y + (long)(row < 0 ? 0 : row) * P.d_out + ncol0 + 8 * g;
    if (a.beta != 0.0f) {
#pragma unroll
      for (int q = 0; q < NQ; ++q)
        yold[q] = (row >= 0 && ncol0 + 32 * q + 8 * g < P.d_out) ? ldg16(yrow + 32 * q) : zero;
    }

    f32x4 acc[NQ][2];
#pragma unroll
    for (int q = 0; q < NQ; ++q) acc[q][0] = acc[q][1] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nks = KS > 0 ? KS : (P.d_in + 31) / 32;
#pragma unroll KSR
    for (int ks = 0; ks < nks; ++ks) {
      const int kk = 32 * ks + 8 * g;
      const bool kin = kk < P.d_in;
      const u32x4 vf = (kin && row >= 0) ? load_v8<DT>(P, a.T, row, kk) : zero;
      if (side && kin) {
        if (P.v_out && row >= 0) stg16(P.v_out + (long)row * P.d_in + kk, vf);
        if (a.pt_a) {
          // scale*v (and scale*v2) by tile slot, transposed: [k][slot]
          const long pitch = (long)a.nt_max * kTileRows;
          u32x4 v2f = zero;
          if (a.pt_b && row >= 0) v2f = ldg16(a.v2 + (long)row * P.d_in + kk);
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
      if (KS > 0) {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
          for (int p = 0; p < 2; ++p) acc[q][p] = Num<DT>::mfma(wf[ks < KSR ? ks : 0][q][p], vf, acc[q][p]);
      } else {
        u32x4 wg[NQ][2];
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
          for (int p = 0; p < 2; ++p) {
            const int n = ncol0 + 32 * q + 4 * p + mrow;
            wg[q][p] = (kin && n < P.d_out) ? load_w8<ROWMAJOR>(W, n, kk, P.ldw) : zero;
          }
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
          for (int p = 0; p < 2; ++p) acc[q][p] = Num<DT>::mfma(wg[q][p], vf, acc[q][p]);
      }
    }

    if (row < 0) continue;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      if (ncol0 + 32 * q + 8 * g >= P.d_out) continue;
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
}

}  // namespace smlm
