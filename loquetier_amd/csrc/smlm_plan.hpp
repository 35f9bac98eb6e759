// Tile-plan construction on the device: sort segments by key, scan, fill tiles.
//
// Takes the place of precompute_smlm_forward_args
// (kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:31-46): there one
// thread per segment writes a GEMM problem; here segments that share a key are
// laid end to end (stable in segment order) and cut into 16-row tiles, so a
// tile never mixes adapters and an adapter's rows share tiles.
//
// Two routes: batches of up to 1024 segments are planned by ONE workgroup in
// one launch with every intermediate array in LDS (the decode regime, where a
// second launch would cost as much as the GEMM); larger batches use a sort /
// scan launch followed by a grid-wide fill launch.
#pragma once
#include "smlm_common.hpp"

namespace smlm {

constexpr int kPlanThreads = 1024;
constexpr int kPlanLdsKeys = 4096;   // two-launch route: sorts up to this many keys stay in LDS
constexpr int kPlanSmallSegs = 1024; // one-launch route: at most this many segments ...
constexpr int kPlanSmallTiles = 4096; // ... and at most this many possible tiles
constexpr int kNarrowIdBits = 21;     // ids below 2^21 and 10 bits of segment index make a 32-bit key

struct PlanSortArgs {
  PlanView pv;
  const int32_t* s;  // [S+1] segment boundaries
  const void* key;   // per-segment keys, see SMLM_KEY_*
  int key_kind, S, N;  // N = power of two >= S
  const void* key2;  // SMLM_KEY_PTR2: the second address of every segment (the first is in `key`)
};

// SMLM_KEY_PTR2 in the one-workgroup routes: segments are grouped by a PAIR of addresses.  The pair of
// segment i is replaced by the index of the first segment that has the same pair -- a small integer that
// then serves as an adapter id (it indexes the caller's per-segment tables at an entry that holds this
// group's weights), so everything built for SMLM_KEY_I32 plans applies.  ka / kb: the pairs by segment
// (LDS), first[i] receives the index; t1, t2: scratch of M int32 each (M a power of two); S <= blockDim.x.
// Two rounds of "smallest index per hash slot" (integer minima: the order of the atomics does not matter):
// a segment whose slot's winner holds its pair has found its first occurrence -- every segment with that
// pair hashes to the same slot -- and the few that lose their slot to another pair try a second hash among
// themselves; what is still open after that (two collisions in a row) is searched for directly.  Comparing
// every pair with every other instead costs S x S LDS reads and took longer than the shrink it serves.
// Contains barriers; leaves the result visible to every thread.
template <int M, typename A64, typename A32, typename T32>
__device__ __forceinline__ void first_equal_pair(A64& ka, A64& kb, A32& first, T32& t1, T32& t2, int S) {
  const int tid = threadIdx.x;
  for (int m = tid; m < M; m += blockDim.x) t1[m] = 0x7fffffff, t2[m] = 0x7fffffff;
  uint64_t a = 0, b = 0;
  uint32_t h1 = 0, h2 = 0;
  if (tid < S) {
    a = ka[tid], b = kb[tid];
    const uint64_t h = (a >> 4) * 0x9E3779B97F4A7C15ull ^ (b >> 4) * 0xC2B2AE3D27D4EB4Full;
    h1 = (uint32_t)(h >> 40) & (M - 1);
    h2 = (uint32_t)(h >> 24) & (M - 1);
  }
  __syncthreads();
  if (tid < S) atomicMin(&t1[h1], tid);
  __syncthreads();
  int found = -1;
  if (tid < S) {
    const int c = t1[h1];
    if (ka[c] == a && kb[c] == b) found = c;
    else atomicMin(&t2[h2], tid);
  }
  __syncthreads();
  bool open = false;
  if (tid < S && found < 0) {
    const int c = t2[h2];
    if (ka[c] == a && kb[c] == b) found = c;
    else open = true;
  }
  if (__ballot(open)) {  // uniform over the wave: a plain search for the lanes still open
    int best = tid;
    for (int j = 0; j < S; j += 8) {
      uint64_t ca[8], cb[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int je = j + e < S ? j + e : S - 1;
        ca[e] = ka[je], cb[e] = kb[je];
      }
#pragma unroll
      for (int e = 7; e >= 0; --e)
        if (j + e < best && ca[e] == a && cb[e] == b) best = j + e;
    }
    if (open) found = best;
  }
  if (tid < S) first[tid] = found;
  __syncthreads();
}

// Inclusive scan of a 32-bit value over the wave with DPP adds: four shifts
// inside each row of 16 lanes (a lane whose source falls outside its row adds
// zero), then lane 15 of rows 0 and 2 into rows 1 and 3, then lane 31 into rows
// 2 and 3.
__device__ __forceinline__ uint32_t wave_scan_incl_u32(uint32_t x) {
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xf, 0xf, false);  // row_shr:1
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xf, 0xf, false);  // row_shr:2
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x114, 0xf, 0xf, false);  // row_shr:4
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x118, 0xf, 0xf, false);  // row_shr:8
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x142, 0xa, 0xf, false);  // row_bcast:15
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x143, 0xc, 0xf, false);  // row_bcast:31
  return x;
}
// the two 32-bit halves of v are scanned independently (no carry between them)
__device__ __forceinline__ uint64_t wave_scan_incl_2x32(uint64_t v) {
  const uint32_t lo = wave_scan_incl_u32((uint32_t)v), hi = wave_scan_incl_u32((uint32_t)(v >> 32));
  return (uint64_t)lo | ((uint64_t)hi << 32);
}

// Inclusive scan over the block (a multiple of 64 threads, at most 1024) of two
// independent 32-bit counters packed into one 64-bit value per thread; neither
// total may reach 2^32.  `wave_tot` is LDS scratch of 17 entries.  Returns the
// inclusive prefix; the block total is left in wave_tot[16].
__device__ __forceinline__ uint64_t block_scan_incl(uint64_t v, uint64_t* wave_tot) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v = wave_scan_incl_2x32(v);
  __syncthreads();  // previous users of wave_tot are done
  if (lane == 63) wave_tot[wave] = v;
  __syncthreads();
  if (wave == 0) {  // exclusive scan of the (at most 16) wave totals, in registers
    const int nw = (int)(blockDim.x >> 6);
    const uint64_t t = lane < nw ? wave_tot[lane] : 0;
    const uint64_t run = wave_scan_incl_2x32(t);
    if (lane < nw) wave_tot[lane] = (uint64_t)((uint32_t)run - (uint32_t)t) |
                                    ((uint64_t)((uint32_t)(run >> 32) - (uint32_t)(t >> 32)) << 32);
    if (lane == nw - 1) wave_tot[16] = run;
  }
  __syncthreads();
  const uint64_t base = wave_tot[wave];
  return (uint64_t)((uint32_t)v + (uint32_t)base) | ((uint64_t)((uint32_t)(v >> 32) + (uint32_t)(base >> 32)) << 32);
}

// Sort key of segment i: group key in the high bits, segment index in the low
// kSegBits, so equal keys keep their segment order and no two keys are equal.
__device__ __forceinline__ uint64_t make_key(const void* key, int kind, int i) {
  if (kind == SMLM_KEY_I32)
    return ((uint64_t)(uint32_t) reinterpret_cast<const int32_t*>(key)[i] << kSegBits) | (uint32_t)i;
  if (kind == SMLM_KEY_PTR)
    return ((reinterpret_cast<const uint64_t*>(key)[i] >> 4) << kSegBits) | (uint32_t)i;
  return ((uint64_t)i << kSegBits) | (uint32_t)i;
}

// A 16-byte aligned address below 2^48 packs into 44 bits; anything else
// cannot be a sort key, so such a batch is planned segment by segment.
__device__ __forceinline__ int usable_kind(const void* key, int key_kind, int S, int* bad_key) {
  if (threadIdx.x == 0) *bad_key = 0;
  __syncthreads();
  if (key_kind == SMLM_KEY_PTR) {
    const uint64_t* pk = reinterpret_cast<const uint64_t*>(key);
    for (int i = threadIdx.x; i < S; i += blockDim.x)
      if ((pk[i] >> 48) != 0 || (pk[i] & 15) != 0) *bad_key = 1;
  }
  __syncthreads();
  return *bad_key ? SMLM_KEY_NONE : key_kind;
}

// Bitonic sort, ascending.  K must be addressed by the caller's own address
// space (LDS array or global pointer), never through a pointer that could be
// either: a generic pointer into LDS makes the compiler emit flat accesses
// with folded immediate offsets, and a flat access whose base register sits
// just below the LDS aperture is routed by the hardware on the base alone and
// faults.
// IN_LDS: the keys lie in LDS.  A stage of stride <= 64 then keeps every wave inside the 128 keys it already
// owns (pair i of a wave's 64 pairs lies in keys [128 w, 128 w + 128), in every pass of the loop over i), and
// a wave's LDS accesses complete in order: between two such stages the waves need not meet, which takes the
// barriers of 56 of the 66 stages of a 2048-key sort away (1075 segments: the launch 27.1 -> 25.6 us; placing every
// key by counting the keys below it instead, all lanes reading one LDS address at a time: 38.5 us).
template <bool IN_LDS = false, typename KeyArray>
__device__ __forceinline__ void bitonic_sort(KeyArray K, int N) {
  bool own = false;  // the stage before this one was one of those
  for (int size = 2; size <= N; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      const bool local = IN_LDS && stride <= kWaveSize;
      if (!(own && local)) __syncthreads();
      else {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      own = local;
      for (int i = threadIdx.x; i < (N >> 1); i += blockDim.x) {
        const int lo = 2 * i - (i & (stride - 1));
        const int hi = lo + stride;
        const bool asc = (lo & size) == 0;
        const uint64_t a = K[lo], b = K[hi];
        if ((a > b) == asc) {
          K[lo] = b;
          K[hi] = a;
        }
      }
    }
  }
  __syncthreads();
}

// last index i in [0, n) with a[i] <= q, given a[0] <= q < a[n]
template <typename Arr>
__device__ __forceinline__ int last_le(Arr a, int n, int q) {
  int lo = 0, hi = n;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a[mid] <= q) lo = mid; else hi = mid;
  }
  return lo;
}

// number of keys[j], j in [j0, j1), below `key`; eight LDS reads in flight at a time
template <typename T>
__device__ __forceinline__ int count_below(const T* keys, T key, int j0, int j1) {
  int n = 0, j = j0;
  for (; j + 8 <= j1; j += 8) {
    T k8[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) k8[e] = keys[j + e];
#pragma unroll
    for (int e = 0; e < 8; ++e) n += k8[e] < key ? 1 : 0;
  }
  for (; j < j1; ++j) n += keys[j] < key ? 1 : 0;
  return n;
}

// ---------------------------------------------------------------- one launch
// All global reads (keys, segment boundaries) are issued together up front: a
// first-touch global load costs more than everything else in this kernel, so
// nothing that was loaded is asked for again; the sorted arrays live in LDS.
// The workgroup's LDS of the one-launch route, as a struct so that another kernel can lend the
// same memory to a workgroup that builds a plan (it is only ever reached by name through a
// reference that the compiler resolves at compile time, never through a stored pointer).
template <int CAP>
struct PlanSmallLdsT {  // CAP segments, at most 4 * CAP possible tiles
  uint64_t K[CAP], K0[CAP];
  int32_t start0[CAP], len0[CAP];  // by segment
  int32_t sseg[CAP], rowpos[CAP + 1];  // by sorted position
  int32_t grow[CAP + 1], gtile[CAP + 1], gblk[CAP + 1];
  int32_t gseg[CAP], gid[CAP];
  int32_t gpos[CAP + 1];  // group -> sorted position of its first segment, [NG] = S
  uint64_t wave_tot[17];
  int bad_key, wide_key;
};
using PlanSmallLds = PlanSmallLdsT<kPlanSmallSegs>;

// the whole plan of a batch of at most CAP segments and 4 * CAP possible tiles, built by the
// calling workgroup (at least as many threads as segments, a multiple of 64)
// Several workgroups may share the work (part p of nparts): each of them sorts and scans for
// itself and writes the same small tables, and they deal the per-tile and per-block entries,
// which take the longest to write, out among themselves.
template <int CAP>
__device__ __forceinline__ void plan_small_body(const PlanSortArgs& args, PlanSmallLdsT<CAP>& L, int part = 0,
                                                int nparts = 1) {
  auto& K = L.K; auto& K0 = L.K0;
  auto& start0 = L.start0; auto& len0 = L.len0;
  auto& sseg = L.sseg; auto& rowpos = L.rowpos;
  auto& grow = L.grow; auto& gtile = L.gtile; auto& gblk = L.gblk;
  auto& gseg = L.gseg; auto& gid = L.gid; auto& gpos = L.gpos;
  auto& wave_tot = L.wave_tot;
  int& bad_key = L.bad_key; int& wide_key = L.wide_key;
  const PlanView pv = args.pv;
  const int S = args.S, tid = threadIdx.x;  // blockDim.x >= S

  uint64_t raw = 0, raw2 = 0;
  int s0 = 0, s1 = 0;
  if (tid < S) {
    if (args.key_kind == SMLM_KEY_I32) raw = (uint32_t) reinterpret_cast<const int32_t*>(args.key)[tid];
    if (args.key_kind == SMLM_KEY_PTR || args.key_kind == SMLM_KEY_PTR2) raw = reinterpret_cast<const uint64_t*>(args.key)[tid];
    if (args.key_kind == SMLM_KEY_PTR2) raw2 = reinterpret_cast<const uint64_t*>(args.key2)[tid];
    s0 = args.s[tid];
    s1 = args.s[tid + 1];
  }
  int key_kind = args.key_kind;
  if (key_kind == SMLM_KEY_PTR2) {  // pairs of addresses -> the first segment with the same pair, an id from here on
    if (tid < S) K0[tid] = raw, K[tid] = raw2;
    // (scratch: two of the group tables, CAP + 1 entries each, not in use yet)
    first_equal_pair<CAP>(K0, K, sseg, grow, gtile, S);
    if (tid < S) raw = (uint32_t)sseg[tid];
    key_kind = SMLM_KEY_I32;
    __syncthreads();  // K0, K, sseg are free again
  }
  if (tid == 0) bad_key = 0, wide_key = 0;
  __syncthreads();
  // A 16-byte aligned address below 2^48 packs into 44 bits; anything else
  // cannot be a sort key, so such a batch is planned segment by segment.
  if (key_kind == SMLM_KEY_PTR && tid < S && ((raw >> 48) != 0 || (raw & 15) != 0)) bad_key = 1;
  // adapter ids below 2^21 sort as 32-bit keys (id, segment), half the LDS traffic and compares
  if (tid < S && (key_kind != SMLM_KEY_I32 || raw >= (1u << kNarrowIdBits))) wide_key = 1;
  if (tid < S) {
    start0[tid] = s0;
    len0[tid] = s1 > s0 ? s1 - s0 : 0;
  }
  __syncthreads();
  const int kind = bad_key ? SMLM_KEY_NONE : key_kind;
  uint64_t mine = ~0ull;
  if (tid < S) {
    const uint64_t gkey = kind == SMLM_KEY_I32 ? raw : (kind == SMLM_KEY_PTR ? raw >> 4 : (uint64_t)tid);
    mine = (gkey << kSegBits) | (uint32_t)tid;
  }

  // Sort by counting: keys are distinct (segment index inside), so the sorted
  // position of a key is the number of smaller keys.  The block's threads split
  // the S x S comparisons: thread (part, i) counts the keys of its part below
  // key i and adds its count to rank[i].
  if (kind != SMLM_KEY_NONE) {
    const bool narrow = !wide_key;
    uint32_t* K32 = reinterpret_cast<uint32_t*>(K0);
    if (tid < S) {
      if (narrow) K32[tid] = ((uint32_t)raw << 10) | (uint32_t)tid; else K0[tid] = mine;
      sseg[tid] = 0;  // rank accumulator for now
    }
    __syncthreads();
    const int Sp = S <= 64 ? 64 : (S <= 128 ? 128 : (S <= 256 ? 256 : (S <= 512 ? 512 : 1024)));
    const int parts = (int)blockDim.x / Sp;  // blockDim.x is a multiple of Sp
    const int i = tid % Sp, part = tid / Sp;
    if (i < S && part < parts) {
      const int per = (((S + parts - 1) / parts) + 7) & ~7;
      const int j0 = part * per, j1 = (j0 + per < S) ? j0 + per : S;
      int rank = 0;
      if (j0 < j1) rank = narrow ? count_below<uint32_t>(K32, K32[i], j0, j1) : count_below<uint64_t>(K0, K0[i], j0, j1);
      if (rank) atomicAdd(&sseg[i], rank);  // integer adds: the total does not depend on their order
    }
    __syncthreads();
    if (tid < S) K[sseg[tid]] = mine;
  } else if (tid < S) {
    K[tid] = mine;
  }
  __syncthreads();

  // gathered-row position of every sorted segment, group heads
  constexpr uint64_t kRowMask = 0xffffffffull;  // rows in the low half, group heads in the high half
  int seg = 0, len = 0;
  uint64_t gk = 0;
  bool head = false;
  if (tid < S) {
    const uint64_t k = K[tid];
    seg = (int)(k & (kMaxSegments - 1));
    gk = k >> kSegBits;
    len = len0[seg];
    head = true;
    if (tid > 0) head = (K[tid - 1] >> kSegBits) != gk;
  }
  const uint64_t v = (uint64_t)len | ((uint64_t)(head ? 1 : 0) << 32);
  const uint64_t incl = block_scan_incl(v, wave_tot);
  const uint64_t total = wave_tot[16];
  const int rows_total = (int)(total & kRowMask), NG = (int)(total >> 32);
  if (tid < S) {
    const int rows_before = (int)((incl - v) & kRowMask);
    sseg[tid] = seg;
    rowpos[tid] = rows_before;
    pv.sorted_seg[tid] = seg;
    pv.rowpos[tid] = rows_before;
    if (head) {
      const int G = (int)(incl >> 32) - 1;
      grow[G] = rows_before;
      gseg[G] = seg;
      gid[G] = (int32_t)(uint32_t)gk;
      gpos[G] = tid;
    }
  }
  if (tid == 0) {
    rowpos[S] = rows_total;
    grow[NG] = rows_total;
    gpos[NG] = S;
    pv.rowpos[S] = rows_total;
  }
  __syncthreads();

  // tiles and tile blocks per group -> first tile / first block of each group (one scan)
  uint64_t nt = 0;
  if (tid < NG) nt = (uint64_t)((grow[tid + 1] - grow[tid] + kTileRows - 1) / kTileRows);
  const uint64_t nb = (nt + kBlkTiles - 1) / kBlkTiles;
  const uint64_t both = nt | (nb << 32);
  const uint64_t bincl = block_scan_incl(both, wave_tot);
  const int n_tiles = (int)(wave_tot[16] & 0xffffffffu), n_blocks = (int)(wave_tot[16] >> 32);
  if (tid < NG) {
    const uint64_t ex = bincl - both;
    gtile[tid] = (int)(ex & 0xffffffffu);
    gblk[tid] = (int)(ex >> 32);
    pv.grp_tile[tid] = gtile[tid];
    pv.grp_blk[tid] = gblk[tid];
    pv.grp_row[tid] = grow[tid];
    pv.grp_seg[tid] = gseg[tid];
    pv.grp_id[tid] = gid[tid];
  }
  if (tid == 0) {
    gtile[NG] = n_tiles;
    gblk[NG] = n_blocks;
    pv.grp_tile[NG] = n_tiles;
    pv.grp_blk[NG] = n_blocks;
    pv.grp_row[NG] = rows_total;
    pv.hdr[0] = n_tiles;
    pv.hdr[1] = NG;
    pv.hdr[2] = rows_total;
    pv.hdr[3] = kind;
    pv.hdr[4] = n_blocks;
    pv.hdr[5] = start0[0];  // segments lie end to end: the covered rows start at s[0]
#pragma unroll
    for (int i = 0; i < 4; ++i) pv.hdr[kHdrZeros + i] = 0;
  }
  __syncthreads();

  // tile -> group table (the sort keys' first copy is free by now)
  uint16_t* gt = reinterpret_cast<uint16_t*>(K0);
  for (int tile = tid; tile < n_tiles; tile += blockDim.x) gt[tile] = (uint16_t)last_le(gtile, NG, tile);
  __syncthreads();
  // tile blocks; entries past the last one say "no tiles" (kernels launched over an
  // upper bound of the block count stop there without reading the header)
  const int first = part * (int)blockDim.x + tid, stride = nparts * (int)blockDim.x;
  for (int b = first; b < pv.nt_max; b += stride) {
    int packed = 0;
    if (b < n_blocks) {
      const int G = last_le(gblk, NG, b);
      const int tile0 = gtile[G] + (b - gblk[G]) * kBlkTiles;
      const int left = gtile[G + 1] - tile0;
      packed = (tile0 << 3) | (left < kBlkTiles ? left : kBlkTiles);
    }
    pv.blk[b] = packed;
  }

  // fill: one thread per tile slot; tiles past the last one get weight index -1.  The group
  // of a tile comes from the table above and the segment of a row is searched among the
  // group's own segments only, which keeps the chains of dependent LDS reads short.
  for (int tile = n_tiles + first; tile < pv.nt_max; tile += stride) pv.tile_wid[tile] = -1;
  for (int slot = first; slot < n_tiles * kTileRows; slot += stride) {
    const int tile = slot / kTileRows, c = slot % kTileRows;
    const int G = gt[tile];
    const int q = grow[G] + (tile - gtile[G]) * kTileRows + c;
    int row = -1, rseg = -1;
    if (q < grow[G + 1]) {
      const int a0 = gpos[G];
      const int a = a0 + last_le(rowpos + a0, gpos[G + 1] - a0, q);
      rseg = sseg[a];
      row = start0[rseg] + (q - rowpos[a]);
    }
    pv.tile_row[slot] = row;
    pv.tile_rseg[slot] = rseg;
    if (c == 0) pv.tile_wid[tile] = (kind == SMLM_KEY_I32) ? gid[G] : gseg[G];
  }
}

__global__ __launch_bounds__(kPlanThreads) void plan_small_kernel(PlanSortArgs args) {
  __shared__ PlanSmallLds lds;
  plan_small_body(args, lds);
}

// --------------------------------------------------------------- two launches
template <bool USE_LDS>
__global__ __launch_bounds__(kPlanThreads) void plan_sort_kernel(PlanSortArgs args) {
  __shared__ uint64_t lds_keys[USE_LDS ? kPlanLdsKeys : 1];
  __shared__ uint64_t wave_tot[17];
  __shared__ int bad_key;
  __shared__ uint64_t carry;
  const PlanView pv = args.pv;
  const int32_t* __restrict__ s = args.s;
  const int S = args.S, N = args.N, tid = threadIdx.x;
  // pairs of addresses: sorted by the first address; a group also ends where the second changes (segments that
  // share the first address and differ in the second may then fall into more groups than they need, never fewer)
  const int kind = usable_kind(args.key, args.key_kind == SMLM_KEY_PTR2 ? SMLM_KEY_PTR : args.key_kind, S, &bad_key);
  const uint64_t* key2 = (args.key_kind == SMLM_KEY_PTR2 && kind == SMLM_KEY_PTR)
                             ? reinterpret_cast<const uint64_t*>(args.key2) : nullptr;

  if (USE_LDS) {
    for (int i = tid; i < N; i += kPlanThreads) lds_keys[i] = i < S ? make_key(args.key, kind, i) : ~0ull;
    __syncthreads();
    if (kind != SMLM_KEY_NONE) bitonic_sort<true>(lds_keys, N);
    for (int i = tid; i < S; i += kPlanThreads) pv.sort_keys[i] = lds_keys[i];
  } else {
    for (int i = tid; i < N; i += kPlanThreads) pv.sort_keys[i] = i < S ? make_key(args.key, kind, i) : ~0ull;
    __syncthreads();
    if (kind != SMLM_KEY_NONE) bitonic_sort(pv.sort_keys, N);
  }
  __syncthreads();
  const uint64_t* K = pv.sort_keys;  // global from here on

  // Pass A: gathered-row position of every sorted segment, group heads.
  if (tid == 0) carry = 0;
  __syncthreads();
  constexpr uint64_t kRowMask = 0xffffffffull;  // rows in the low half, group heads in the high half
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
      if (p > 0) {
        head = (K[p - 1] >> kSegBits) != gk;
        if (!head && key2) head = key2[(int)(K[p - 1] & (kMaxSegments - 1))] != key2[seg];
      }
    }
    const uint64_t v = (uint64_t)len | ((uint64_t)(head ? 1 : 0) << 32);
    const uint64_t incl = block_scan_incl(v, wave_tot) + carry;
    const uint64_t excl = incl - v;
    if (valid) {
      const int rows_before = (int)(excl & kRowMask);
      pv.sorted_seg[p] = seg;
      pv.rowpos[p] = rows_before;
      if (head) {
        const int G = (int)(incl >> 32) - 1;
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
  const int NG = (int)(carry >> 32);
  if (tid == 0) {
    pv.rowpos[S] = rows_total;
    pv.grp_row[NG] = rows_total;
    pv.hdr[1] = NG;
    pv.hdr[2] = rows_total;
    pv.hdr[3] = kind;
    pv.hdr[5] = s[0];  // segments lie end to end: the covered rows start at s[0]
#pragma unroll
    for (int i = 0; i < 4; ++i) pv.hdr[kHdrZeros + i] = 0;
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
  __syncthreads();

  // Pass C: tile blocks per group -> first block of each group.
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < NG; base += kPlanThreads) {
    const int G = base + tid;
    uint64_t nb = 0;
    if (G < NG) nb = (uint64_t)((pv.grp_tile[G + 1] - pv.grp_tile[G] + kBlkTiles - 1) / kBlkTiles);
    const uint64_t incl = block_scan_incl(nb, wave_tot) + carry;
    if (G < NG) pv.grp_blk[G] = (int)(incl - nb);
    __syncthreads();
    if (tid == 0) carry += wave_tot[16];
    __syncthreads();
  }
  if (tid == 0) {
    pv.grp_blk[NG] = (int)carry;
    pv.hdr[4] = (int)carry;
  }
}

struct PlanFillArgs {
  PlanView pv;
  const int32_t* s;
  int S;
};

// One thread per tile slot: which row (and segment) sits there.
__global__ __launch_bounds__(256) void plan_fill_kernel(PlanFillArgs args) {
  const PlanView pv = args.pv;
  const int32_t* __restrict__ s = args.s;
  const int S = args.S;
  const long slot = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int tile = (int)(slot / kTileRows), c = (int)(slot % kTileRows);
  if (tile >= pv.nt_max) return;
  const int NG = pv.hdr[1];
  if (slot < pv.nt_max) {  // the first nt_max threads also write the tile-block table
    const int b = (int)slot;
    int packed = 0;  // past the last block: "no tiles"
    if (b < pv.hdr[4]) {
      const int Gb = last_le(pv.grp_blk, NG, b);
      const int tile0 = pv.grp_tile[Gb] + (b - pv.grp_blk[Gb]) * kBlkTiles;
      const int left = pv.grp_tile[Gb + 1] - tile0;
      packed = (tile0 << 3) | (left < kBlkTiles ? left : kBlkTiles);
    }
    pv.blk[b] = packed;
  }
  if (tile >= pv.hdr[0]) {  // past the last tile: weight index -1
    if (c == 0) pv.tile_wid[tile] = -1;
    return;
  }
  // last group whose first tile is <= tile (empty groups share a first tile
  // with their successor, so "last" lands on the one that owns the tile)
  const int G = last_le(pv.grp_tile, NG, tile);
  const int q = pv.grp_row[G] + (tile - pv.grp_tile[G]) * kTileRows + c;
  int row = -1, rseg = -1;
  if (q < pv.grp_row[G + 1]) {
    const int a = last_le(pv.rowpos, S, q);
    rseg = pv.sorted_seg[a];
    row = s[rseg] + (q - pv.rowpos[a]);
  }
  pv.tile_row[slot] = row;
  pv.tile_rseg[slot] = rseg;
  if (c == 0) pv.tile_wid[tile] = (pv.hdr[3] == SMLM_KEY_I32) ? pv.grp_id[G] : pv.grp_seg[G];
}

}  // namespace smlm
