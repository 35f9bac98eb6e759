// Decode batches without a plan launch: a shrink whose workgroups find their own tile.
//
// A model step usually builds its tile plan once and every layer reuses it.  The first
// fused forward of a step can skip that launch: the batch's segment table and adapter ids
// go straight to the decode shrink (eight waves).  Every workgroup derives the tile it would have
// looked up -- the adapter and the (at most sixteen) rows of tile t, numbered exactly as
// the plan numbers them -- from the segment table itself, and ONE extra workgroup of the
// same launch builds the plan proper (the body of plan_small_kernel) for the expand launch
// that follows and for every later call.  This takes the place of the reference's
// per-call set-up kernel precompute_smlm_forward_args
// (kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:31-46), which also runs inside
// every call there.
//
// Adapter ids are table indices (SMLM_KEY_I32 with ids in [0, n_weights)), so grouping by
// adapter needs no sort: a histogram of rows per adapter in LDS, a scan over the adapters
// for the first tile of each, and a scan over the segments of the tile's adapter for its
// rows.  The plan orders groups by ascending id and a group's segments by index, which is
// what the two scans walk, so tile t here is tile t of the plan.
#pragma once
#include "smlm_forward.hpp"
#include "smlm_plan.hpp"

namespace smlm {

constexpr int kSelfPlanThreads = 512;   // eight waves, as the decode shrink_kernel
constexpr int kSelfPlanSegs = 512;      // most segments of the route: one per thread
constexpr int kSelfPlanWeights = 1024;  // most table entries (adapters) of the route: two per thread
constexpr int kSelfPlanWaveScan = 256;  // up to this many, every wave scans the adapters' tile counts by itself

struct SelfPlanArgs {
  ShrinkArgs sh;        // sh.plan is not read (the plan does not exist yet), except w_rank
  PlanSortArgs plan;    // what the extra workgroup builds; key_kind = SMLM_KEY_I32
  int n_weights;
  int units;            // tile bound = grid.y - 1; workgroups with blockIdx.y == units: the plan builder
};

// sixteen zero bytes for predicated-off loads (the other kernels read the plan header's)
__device__ __attribute__((aligned(16))) uint32_t self_plan_zeros[4];

struct SelfPlanScratch {
  int32_t hist[kSelfPlanWeights];   // rows per adapter
  uint64_t wtab[kSelfPlanWeights];  // this projection's weight table
  int32_t rtab[kSelfPlanWeights];   // true ranks, when given
  uint32_t tot_a[8], tot_b[8];      // wave totals of the two scans
  int32_t rows16[kTileRows], rseg16[kTileRows];
  int32_t sel[2];                   // adapter of the tile (-1: no such tile), tile's index within the adapter
};

// The sum's staging area lies behind the scratch where both fit under the plan builder's LDS
// (ranks up to 32) and over it otherwise.
template <int NB>
struct SelfPlanWork {
  static constexpr bool kOverlay =
      sizeof(SelfPlanScratch) + sizeof(f32x4) * 8 * NB * kWaveSize > sizeof(PlanSmallLdsT<kSelfPlanSegs>);
  SelfPlanScratch find;
  f32x4 red[kOverlay ? 1 : 8][NB][kWaveSize];
};
template <int NB>
union SelfPlanLds {
  PlanSmallLdsT<kSelfPlanSegs> plan;  // the plan-building workgroup
  SelfPlanWork<NB> work;              // the others: finding their tile, then the cross-wave sum
  f32x4 red[8][NB][kWaveSize];        // ... which reuses the scratch's memory when the two do not fit side by side
};

// Exclusive prefix of v over the workgroup (8 waves) with ONE barrier: every wave leaves its
// total, every thread adds the totals of the waves before its own.  `tot` must not be in use.
__device__ __forceinline__ uint32_t block_scan_excl_1(uint32_t v, uint32_t* tot, uint32_t* incl_out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t in_wave = wave_scan_incl_u32(v);
  if (lane == 63) tot[wave] = in_wave;
  __syncthreads();
  uint32_t before = 0;
#pragma unroll
  for (int w = 0; w < 7; ++w) before += w < wave ? tot[w] : 0u;
  *incl_out = before + in_wave;
  return before + in_wave - v;
}

template <int DT, int NB, int U>
__global__ __launch_bounds__(kSelfPlanThreads) void shrink_self_planned_kernel(SelfPlanArgs a) {
  static_assert(kSelfPlanSegs <= kSelfPlanThreads && kSelfPlanWeights == 2 * kSelfPlanThreads, "entries per thread");
  __shared__ SelfPlanLds<NB> sm;
  constexpr int NW = kSelfPlanThreads / kWaveSize;
  constexpr bool kOverlay = SelfPlanWork<NB>::kOverlay;
  const int tid = threadIdx.x;
  if ((int)blockIdx.y == a.units) {  // the extra row of the grid: one workgroup builds the plan
    if (blockIdx.x == 0 && blockIdx.z == 0) plan_small_body(a.plan, sm.plan);
    return;
  }
  const int pj = blockIdx.z, yy = blockIdx.x, tile = blockIdx.y;
  if (yy >= a.sh.items.row_start[pj + 1] - a.sh.items.row_start[pj]) return;
  const ShrinkProj P = a.sh.p[pj];
  const int S = a.plan.S, NA = a.n_weights;
  SelfPlanScratch& F = sm.work.find;
  const int wave = tid >> 6, lane = tid & 63;
  const int c = lane & 15, g = lane >> 4;
  const int kz = yy % P.ksplit, zb = yy / P.ksplit;
  const int n0 = zb * 64;
  const int kbeg = (kz * NW + wave) * P.k_per_wave;
  const int kend = min(kbeg + P.k_per_wave, P.d_in);
  const uint16_t* zeros = reinterpret_cast<const uint16_t*>(self_plan_zeros);

  // ---- which adapter and which rows make up tile `tile`.  Everything global is requested at
  // once; the first barrier (LDS cleared) passes while those loads are on their way.
  int key = -1, s0 = 0, len = 0;
  if (tid < S) {
    key = ((const SMLM_GLOBAL int32_t*)a.plan.key)[tid];
    s0 = ((const SMLM_GLOBAL int32_t*)a.plan.s)[tid];
    const int s1 = ((const SMLM_GLOBAL int32_t*)a.plan.s)[tid + 1];
    len = s1 > s0 ? s1 - s0 : 0;
  }
  uint64_t wp[2] = {0, 0};  // table entries 2 tid and 2 tid + 1
  int wr[2] = {0, 0};
#pragma unroll
  for (int e = 0; e < 2; ++e)
    if (2 * tid + e < NA) {
      wp[e] = ((const SMLM_GLOBAL uint64_t*)P.w_ptrs)[2 * tid + e];
      if (a.sh.plan.w_rank) wr[e] = ((const SMLM_GLOBAL int32_t*)a.sh.plan.w_rank)[2 * tid + e];
    }
  F.hist[2 * tid] = 0;
  F.hist[2 * tid + 1] = 0;
  if (tid < kTileRows) F.rows16[tid] = -1, F.rseg16[tid] = -1;
  if (tid == 0) F.sel[0] = -1;
  __syncthreads();
  const bool counted = len > 0 && key >= 0 && key < NA;  // ids outside the table own no tile here
  if (counted) atomicAdd(&F.hist[key], len);              // integer adds: the total does not depend on their order
#pragma unroll
  for (int e = 0; e < 2; ++e) F.wtab[2 * tid + e] = wp[e], F.rtab[2 * tid + e] = wr[e];
  __syncthreads();
  // first tile of every adapter (adapters in ascending order, as the plan's groups are) -> the
  // adapter that owns `tile` and the tile's index among that adapter's tiles
  int wid = -1, sub = 0;
  if (NA <= kSelfPlanWaveScan) {
    // few adapters: every wave walks the table by itself, 64 adapters a step, and needs no barrier
    uint32_t carry = 0;
    for (int a0 = 0; a0 < NA; a0 += kWaveSize) {
      const uint32_t n = a0 + lane < NA ? (uint32_t)((F.hist[a0 + lane] + kTileRows - 1) / kTileRows) : 0u;
      const uint32_t last = carry + wave_scan_incl_u32(n), first = last - n;
      const uint64_t hit = __ballot((uint32_t)tile >= first && (uint32_t)tile < last);
      if (hit) {  // uniform over the wave; at most one lane
        const int l = __builtin_ctzll(hit);
        wid = a0 + l;
        sub = tile - (int)__builtin_amdgcn_readlane((int)first, l);
        break;
      }
      carry = (uint32_t)__builtin_amdgcn_readlane((int)last, kWaveSize - 1);
    }
  } else {
    // many adapters: one scan over the workgroup, a thread holding two neighbouring adapters
    const uint32_t t0 = 2 * tid < NA ? (uint32_t)((F.hist[2 * tid] + kTileRows - 1) / kTileRows) : 0u;
    const uint32_t t1 = 2 * tid + 1 < NA ? (uint32_t)((F.hist[2 * tid + 1] + kTileRows - 1) / kTileRows) : 0u;
    uint32_t last;
    const uint32_t first = block_scan_excl_1(t0 + t1, F.tot_a, &last);
    if ((uint32_t)tile >= first && (uint32_t)tile < last) {
      const int e = (uint32_t)tile >= first + t0 ? 1 : 0;
      F.sel[0] = 2 * tid + e;
      F.sel[1] = tile - (int)(first + (e ? t0 : 0u));
    }
    __syncthreads();
    wid = F.sel[0];
    sub = F.sel[1];
  }
  if (wid < 0) return;  // past the last tile; uniform over the workgroup
  const uint16_t* W = reinterpret_cast<const uint16_t*>(F.wtab[wid]);
  int nlim = P.d_out;  // weight rows at or past it are zero padding
  if (a.sh.plan.w_rank) {
    const int r8 = (F.rtab[wid] + 7) & ~7;
    nlim = r8 < nlim ? r8 : nlim;
  }
  // the adapter is known: its weights are requested while the rows are still being found
  auto load_w = [&](int k, u32x4 (&wf)[NB][U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k + 32 * u + 8 * g;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int n = n0 + 16 * nb + c;
        wf[nb][u] = ldg16_or(W + (long)n * P.ldw + kk, kk < kend && n < nlim, zeros);
      }
    }
  };
  u32x4 wf[NB][U];
  load_w(kbeg, wf);

  // rows of the adapter in segment order: tile j of the adapter holds its rows 16j .. 16j+15
  const int q_lo = sub * kTileRows;
  const uint32_t mine = (counted && key == wid) ? (uint32_t)len : 0u;
  uint32_t hi_u;
  const int lo = (int)block_scan_excl_1(mine, F.tot_b, &hi_u);
  {
    const int hi = (int)hi_u;
    const int q0 = lo > q_lo ? lo : q_lo, q1 = hi < q_lo + kTileRows ? hi : q_lo + kTileRows;
    for (int q = q0; q < q1; ++q) {
      F.rows16[q - q_lo] = s0 + (q - lo);
      F.rseg16[q - q_lo] = tid;
    }
  }
  __syncthreads();
  const int row = F.rows16[c], rseg = F.rseg16[c];
  if (kOverlay) __syncthreads();  // every wave holds its tile: the scratch turns into the sum's staging area

  // ---- the product, as the eight-wave shrink_kernel does it
  f32x4 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int k = kbeg; k < kend; k += 32 * U) {
    u32x4 xf[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k + 32 * u + 8 * g;
      xf[u] = ldg16_or(P.x + (long)row * P.d_in + kk, kk < kend && row >= 0, zeros);
    }
    if (k != kbeg) load_w(k, wf);  // uniform over the wave (k is usually one batch)
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nb] = Num<DT>::mfma(wf[nb][u], xf[u], acc[nb]);
  }

  f32x4 (*red)[NB][kWaveSize] = kOverlay ? sm.red : sm.work.red;  // decided at compile time
  // cross-wave sum in wave order; wave 0 writes the tile
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) red[wave][nb][lane] = acc[nb];
  __syncthreads();
  if (wave == 0 && row >= 0) {
    const bool as_partial = P.ksplit > 1 || P.to_partial;
    float scale = 1.0f;
    if (!as_partial && a.sh.seg_scale) scale = a.sh.seg_scale[rseg];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      f32x4 part[NW];
#pragma unroll
      for (int w = 0; w < NW; ++w) part[w] = red[w][nb][lane];
      __builtin_amdgcn_sched_barrier(0);
      f32x4 sum = part[0];
#pragma unroll
      for (int w = 1; w < NW; ++w) sum += part[w];
      const int n = n0 + 16 * nb + 4 * g;  // lane holds columns n .. n+3 of its token
      if (n >= P.d_out) continue;
      if (as_partial)
        *(SMLM_GLOBAL f32x4*)(P.partial + ((long)kz * a.sh.T + row) * P.d_out + n) = sum;
      else
        store4<DT>(P.out + (long)row * P.d_out + n, sum, scale, a.sh.beta);
    }
  }
}

}  // namespace smlm
