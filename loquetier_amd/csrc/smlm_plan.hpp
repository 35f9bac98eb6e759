// Tile-plan construction on the device: sort segments by key, scan, fill tiles.
//
// Takes the place of precompute_smlm_forward_args
// (kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:31-46): there one
// thread per segment writes a GEMM problem; here segments that share a key are
// laid end to end (stable in segment order) and cut into 16-row tiles, so a
// tile never mixes adapters and an adapter's rows share tiles.
#pragma once
#include "smlm_common.hpp"

namespace smlm {

constexpr int kPlanThreads = 1024;
constexpr int kPlanLdsKeys = 4096;  // sorts up to this many keys stay in LDS

// Inclusive scan of one 64-bit value per thread over a 1024-thread block.
// `wave_tot` is LDS scratch of 16 entries.  Returns the inclusive prefix; the
// block total is left in wave_tot[16].
__device__ __forceinline__ uint64_t block_scan_incl(uint64_t v, uint64_t* wave_tot) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    uint64_t o = __shfl_up((unsigned long long)v, d, 64);
    if (lane >= d) v += o;
  }
  __syncthreads();  // previous users of wave_tot are done
  if (lane == 63) wave_tot[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint64_t run = 0;
    for (int w = 0; w < kPlanThreads / 64; ++w) {
      uint64_t t = wave_tot[w];
      wave_tot[w] = run;
      run += t;
    }
    wave_tot[16] = run;
  }
  __syncthreads();
  return v + wave_tot[wave];
}

// USE_LDS is a template parameter, not a run-time choice, so that the key array
// is addressed with LDS instructions: a generic pointer that may point into LDS
// makes the compiler emit flat accesses with folded immediate offsets, and a
// flat access whose base register sits just below the LDS aperture (K[p-1] at
// p = 0) is routed by the hardware on the base alone and faults.
template <bool USE_LDS>
__global__ __launch_bounds__(kPlanThreads) void plan_sort_kernel(PlanView pv,
                                                                 const int32_t* __restrict__ s,
                                                                 const void* key, int key_kind,
                                                                 int S, int N) {
  __shared__ uint64_t lds_keys[USE_LDS ? kPlanLdsKeys : 1];
  __shared__ uint64_t wave_tot[17];
  __shared__ int bad_key;
  __shared__ uint64_t carry;
  const int tid = threadIdx.x;
  uint64_t* K = USE_LDS ? lds_keys : pv.sort_keys;

  if (tid == 0) bad_key = 0;
  __syncthreads();
  if (key_kind == SMLM_KEY_PTR) {
    // A 16-byte aligned address below 2^48 packs into 44 bits; anything else
    // cannot be a sort key, so such a batch is planned segment by segment.
    const uint64_t* pk = reinterpret_cast<const uint64_t*>(key);
    for (int i = tid; i < S; i += kPlanThreads)
      if ((pk[i] >> 48) != 0 || (pk[i] & 15) != 0) bad_key = 1;
    __syncthreads();
  }
  const int kind = bad_key ? SMLM_KEY_NONE : key_kind;

  for (int i = tid; i < N; i += kPlanThreads) {
    uint64_t k;
    if (i >= S) {
      k = ~0ull;
    } else if (kind == SMLM_KEY_I32) {
      k = ((uint64_t)(uint32_t) reinterpret_cast<const int32_t*>(key)[i] << kSegBits) | (uint32_t)i;
    } else if (kind == SMLM_KEY_PTR) {
      k = ((reinterpret_cast<const uint64_t*>(key)[i] >> 4) << kSegBits) | (uint32_t)i;
    } else {
      k = ((uint64_t)i << kSegBits) | (uint32_t)i;
    }
    K[i] = k;
  }
  __syncthreads();

  if (kind != SMLM_KEY_NONE) {  // bitonic sort, ascending; ties impossible (segment index inside)
    for (int size = 2; size <= N; size <<= 1) {
      for (int stride = size >> 1; stride > 0; stride >>= 1) {
        for (int i = tid; i < (N >> 1); i += kPlanThreads) {
          const int lo = 2 * i - (i & (stride - 1));
          const int hi = lo + stride;
          const bool asc = (lo & size) == 0;
          const uint64_t a = K[lo], b = K[hi];
          if ((a > b) == asc) {
            K[lo] = b;
            K[hi] = a;
          }
        }
        __syncthreads();
      }
    }
  }

  // Pass A: gathered-row position of every sorted segment, group heads.
  if (tid == 0) carry = 0;
  __syncthreads();
  constexpr uint64_t kRowMask = (1ull << 40) - 1;
  for (int base = 0; base < S; base += kPlanThreads) {
    const int p = base + tid;
    const bool valid = p < S;
    int seg = 0, len = 0;
    uint64_t gk = 0;
    bool head = false;
    if (valid) {
      const uint64_t k = K[p];
      seg = (int)(k & (kMaxSegments - 1));
      gk = k >> kSegBits;
      len = s[seg + 1] - s[seg];
      if (len < 0) len = 0;
      head = true;
      if (p > 0) head = (K[p - 1] >> kSegBits) != gk;
    }
    const uint64_t v = (uint64_t)len | ((uint64_t)(head ? 1 : 0) << 40);
    const uint64_t incl = block_scan_incl(v, wave_tot) + carry;
    const uint64_t excl = incl - v;
    if (valid) {
      const int rows_before = (int)(excl & kRowMask);
      pv.sorted_seg[p] = seg;
      pv.rowpos[p] = rows_before;
      if (head) {
        const int G = (int)(incl >> 40) - 1;
        pv.grp_row[G] = rows_before;
        pv.grp_seg[G] = seg;
        pv.grp_id[G] = (int32_t)(uint32_t)gk;
      }
    }
    __syncthreads();
    if (tid == 0) carry += wave_tot[16];
    __syncthreads();
  }
  const int rows_total = (int)(carry & kRowMask);
  const int NG = (int)(carry >> 40);
  if (tid == 0) {
    pv.rowpos[S] = rows_total;
    pv.grp_row[NG] = rows_total;
    pv.hdr[1] = NG;
    pv.hdr[2] = rows_total;
    pv.hdr[3] = kind;
  }
  __syncthreads();

  // Pass B: tiles per group -> first tile of each group.
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < NG; base += kPlanThreads) {
    const int G = base + tid;
    uint64_t nt = 0;
    if (G < NG) nt = (uint64_t)((pv.grp_row[G + 1] - pv.grp_row[G] + kTileRows - 1) / kTileRows);
    const uint64_t incl = block_scan_incl(nt, wave_tot) + carry;
    if (G < NG) pv.grp_tile[G] = (int)(incl - nt);
    __syncthreads();
    if (tid == 0) carry += wave_tot[16];
    __syncthreads();
  }
  if (tid == 0) {
    pv.grp_tile[NG] = (int)carry;
    pv.hdr[0] = (int)carry;
  }
}

// One thread per tile slot: which row (and segment) sits there.
__global__ __launch_bounds__(256) void plan_fill_kernel(PlanView pv, const int32_t* __restrict__ s,
                                                        int S) {
  const long slot = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int tile = (int)(slot / kTileRows), c = (int)(slot % kTileRows);
  if (tile >= pv.nt_max) return;
  const int n_tiles = pv.hdr[0];
  if (tile >= n_tiles) return;
  const int NG = pv.hdr[1];
  // last group whose first tile is <= tile (empty groups share a first tile
  // with their successor, so "last" lands on the one that owns the tile)
  int lo = 0, hi = NG;  // invariant: grp_tile[lo] <= tile < grp_tile[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (pv.grp_tile[mid] <= tile) lo = mid; else hi = mid;
  }
  const int G = lo;
  const int q = pv.grp_row[G] + (tile - pv.grp_tile[G]) * kTileRows + c;
  int row = -1, rseg = -1;
  if (q < pv.grp_row[G + 1]) {
    int a = 0, b = S;  // invariant: rowpos[a] <= q < rowpos[b]
    while (b - a > 1) {
      const int mid = (a + b) >> 1;
      if (pv.rowpos[mid] <= q) a = mid; else b = mid;
    }
    rseg = pv.sorted_seg[a];
    row = s[rseg] + (q - pv.rowpos[a]);
  }
  pv.tile_row[slot] = row;
  pv.tile_rseg[slot] = rseg;
}

}  // namespace smlm
