// Forward shrinks that need no plan launch: their workgroups find their own tiles.
//
// A model step usually builds its tile plan once and every layer reuses it.  The first
// fused forward of a step can skip that launch: the batch's segment table and adapter ids
// go straight to the shrink.  Every workgroup derives the unit of work it would have looked
// up -- the adapter and the rows of tile t (decode batches, eight-wave shrink) or of tile
// block b (larger batches, tile-block shrink), numbered exactly as the plan numbers them --
// from the segment table itself, and a few extra workgroups of the same launch build the plan
// proper (the body of plan_small_kernel, its table writes dealt out among them) for the
// launches that follow and for every later call.  This takes the place of the reference's per-call set-up kernel
// precompute_smlm_forward_args (kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:31-46),
// which also runs inside every call there.
//
// Adapter ids are table indices (SMLM_KEY_I32 with ids in [0, n_weights)), so grouping by
// adapter needs no sort: a histogram of rows per adapter in LDS, a scan over the adapters
// for the first unit of each, and a scan over the segments of the unit's adapter for its
// rows.  The plan orders groups by ascending id and a group's segments by index, which is
// what the two scans walk, so unit u here is unit u of the plan.
//
// The products themselves repeat shrink_kernel / shrink_block_kernel step for step (same MFMA
// sequence over k, same cross-wave sum): a call that builds its plan here and a call over the
// finished plan give the same bits, which the tests hold them to.  What differs is the order of
// the loads -- the weights are requested as soon as the adapter is known, before the rows are.
#pragma once
#include "smlm_forward.hpp"
#include "smlm_plan.hpp"

namespace smlm {

constexpr int kSelfPlanThreads = 512;   // decode route: eight waves, as the decode shrink_kernel, up to 512 segments;
constexpr int kSelfPlanSegs = 1024;     //   beyond, up to here, two such groups of waves share a workgroup (one segment per thread)
constexpr int kSelfPlanBlkSegs = 512;   // tile-block route: most segments (256 threads up to 256 segments, 512 beyond)
constexpr int kSelfPlanWeights = 1024;  // most table entries (adapters) of either route
constexpr int kSelfPlanBuilders = 8;     // workgroups of the launch that share the writing of the plan
constexpr int kSelfPlanWaveScan = 256;  // up to this many, every wave scans the adapters' unit counts by itself

struct SelfPlanArgs {
  ShrinkArgs sh;        // sh.plan is not read (the plan does not exist yet), except w_rank
  PlanSortArgs plan;    // what the extra workgroups build; key_kind = SMLM_KEY_I32
  int n_weights;
  int units;            // unit bound = grid.y - 1; workgroups with blockIdx.y == units: the plan builders
};

// sixteen zero bytes for predicated-off loads (the other kernels read the plan header's)
__device__ __attribute__((aligned(16))) uint32_t self_plan_zeros[4];

// ---- finding a unit of work (UT tiles of one adapter) without a plan ------------------------
// PAIRS: the kernels built for plans keyed by pairs of addresses (SMLM_KEY_PTR2).  They are kernels of their
// own because what they add costs the others dearly: the arrays below triple the finder's LDS, and their
// workgroups may take several units in turn (see shrink_self_planned_kernel), a loop around the whole body
// that takes the tile-block kernel from 68 to 128 registers a lane.
template <int N>
struct FindPairs {
  uint64_t ka[N], kb[N];  // the segments' pairs of addresses
  int32_t first[N];       // the first segment with the same pair: the segment's id
  int32_t slot[2][N];     // (scratch of first_equal_pair)
};
template <>
struct FindPairs<0> {};
template <int THREADS, bool PAIRS>
struct FindLds {
  int32_t hist[kSelfPlanWeights];   // rows per adapter
  uint64_t wtab[kSelfPlanWeights];  // this projection's weight table
  int32_t rtab[kSelfPlanWeights];   // true ranks, when given
  FindPairs<PAIRS ? kSelfPlanWeights : 0> pr;
  uint32_t tot_a[THREADS / kWaveSize], tot_b[THREADS / kWaveSize];  // wave totals of the two scans
  int32_t rows[kBlkTiles * kTileRows], rseg[kBlkTiles * kTileRows];
  int32_t sel[3];                   // adapter of the unit (-1: no such unit), unit's index within the adapter, units in all
};
struct FindSeg {  // the segment a thread holds
  int key, s0, len;
  bool counted;   // has rows and an adapter id inside the table
};
struct FoundUnit {
  int wid;        // adapter (table index), -1: the unit lies past the last one
  int sub;        // index of the unit among the adapter's units
  int tiles;      // tiles of the unit (1 .. UT)
  int total;      // units of the whole batch
};

// Exclusive prefix of v over the workgroup with ONE barrier: every wave leaves its total,
// every thread adds the totals of the waves before its own.  `tot` must not be in use.
template <int THREADS>
__device__ __forceinline__ uint32_t block_scan_excl_1(uint32_t v, uint32_t* tot, uint32_t* incl_out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t in_wave = wave_scan_incl_u32(v);
  if (lane == 63) tot[wave] = in_wave;
  __syncthreads();
  uint32_t before = 0;
#pragma unroll
  for (int w = 0; w < THREADS / kWaveSize - 1; ++w) before += w < wave ? tot[w] : 0u;
  *incl_out = before + in_wave;
  return before + in_wave - v;
}

// Which adapter owns unit `unit` (a unit = UT consecutive tiles of one adapter; adapters in
// ascending order, as the plan's groups are).  Everything global is requested at once; the
// first barrier (LDS cleared) passes while those loads are on their way.  THREADS >= S.
template <int THREADS, int UT, bool PAIRS>
__device__ __forceinline__ FoundUnit find_adapter(FindLds<THREADS, PAIRS>& F, const PlanSortArgs& pa,
                                                  const void* const* w_ptrs, const int32_t* w_rank, int NA,
                                                  int unit, FindSeg* seg) {
  constexpr int kEnt = kSelfPlanWeights / THREADS;  // table entries a thread holds: kEnt * tid ...
  const int tid = threadIdx.x, lane = tid & 63;
  int key = -1, s0 = 0, len = 0;
  uint64_t pair_a = 0, pair_b = 0;
  if (tid < pa.S) {
    if constexpr (PAIRS) {
      pair_a = ((const SMLM_GLOBAL uint64_t*)pa.key)[tid];
      pair_b = ((const SMLM_GLOBAL uint64_t*)pa.key2)[tid];
    } else {
      key = ((const SMLM_GLOBAL int32_t*)pa.key)[tid];
    }
    s0 = ((const SMLM_GLOBAL int32_t*)pa.s)[tid];
    const int s1 = ((const SMLM_GLOBAL int32_t*)pa.s)[tid + 1];
    len = s1 > s0 ? s1 - s0 : 0;
  }
  uint64_t wp[kEnt];
  int wr[kEnt];
#pragma unroll
  for (int e = 0; e < kEnt; ++e) {
    wp[e] = 0, wr[e] = 0;
    if (kEnt * tid + e < NA) {
      wp[e] = ((const SMLM_GLOBAL uint64_t*)w_ptrs)[kEnt * tid + e];
      if (w_rank) wr[e] = ((const SMLM_GLOBAL int32_t*)w_rank)[kEnt * tid + e];
    }
  }
#pragma unroll
  for (int e = 0; e < kEnt; ++e) F.hist[kEnt * tid + e] = 0;
  if (tid < UT * kTileRows) F.rows[tid] = -1, F.rseg[tid] = -1;
  if (tid == 0) F.sel[0] = -1;
  if constexpr (PAIRS) {
    // groups by pairs of addresses: the id of a segment is the first segment with its pair, as the plan
    // builders number them (first_equal_pair; its barriers also cover the clearing above)
    if (tid < pa.S) F.pr.ka[tid] = pair_a, F.pr.kb[tid] = pair_b;
    first_equal_pair<kSelfPlanWeights>(F.pr.ka, F.pr.kb, F.pr.first, F.pr.slot[0], F.pr.slot[1], pa.S);
    if (tid < pa.S) key = F.pr.first[tid];
  } else {
    __syncthreads();
  }
  const bool counted = len > 0 && key >= 0 && key < NA;  // ids outside the table own no unit here
  if (counted) atomicAdd(&F.hist[key], len);              // integer adds: the total does not depend on their order
#pragma unroll
  for (int e = 0; e < kEnt; ++e) F.wtab[kEnt * tid + e] = wp[e], F.rtab[kEnt * tid + e] = wr[e];
  __syncthreads();
  *seg = FindSeg{key, s0, len, counted};

  auto units_of = [&](int a) -> uint32_t {
    return a < NA ? (uint32_t)((F.hist[a] + UT * kTileRows - 1) / (UT * kTileRows)) : 0u;
  };
  FoundUnit u{-1, 0, 0, 0};
  if (NA <= kSelfPlanWaveScan) {
    // few adapters: every wave walks the table by itself, 64 adapters a step, and needs no barrier
    uint32_t carry = 0;
    for (int a0 = 0; a0 < NA; a0 += kWaveSize) {
      const uint32_t n = units_of(a0 + lane);
      const uint32_t last = carry + wave_scan_incl_u32(n), first = last - n;
      const uint64_t hit = __ballot((uint32_t)unit >= first && (uint32_t)unit < last);
      if (hit) {  // uniform over the wave; at most one lane
        const int l = __builtin_ctzll(hit);
        u.wid = a0 + l;
        u.sub = unit - (int)__builtin_amdgcn_readlane((int)first, l);
      }
      carry = (uint32_t)__builtin_amdgcn_readlane((int)last, kWaveSize - 1);
    }
    u.total = (int)carry;
  } else {
    // many adapters: one scan over the workgroup, a thread holding kEnt neighbouring adapters
    uint32_t n[kEnt], sum = 0;
#pragma unroll
    for (int e = 0; e < kEnt; ++e) n[e] = units_of(kEnt * tid + e), sum += n[e];
    uint32_t last;
    uint32_t first = block_scan_excl_1<THREADS>(sum, F.tot_a, &last);
    if (tid == THREADS - 1) F.sel[2] = (int)last;
    if ((uint32_t)unit >= first && (uint32_t)unit < last) {
#pragma unroll
      for (int e = 0; e < kEnt; ++e) {
        if ((uint32_t)unit >= first && (uint32_t)unit < first + n[e]) {
          F.sel[0] = kEnt * tid + e;
          F.sel[1] = unit - (int)first;
        }
        first += n[e];
      }
    }
    __syncthreads();
    u.wid = F.sel[0];
    u.sub = F.sel[1];
    u.total = F.sel[2];
  }
  if (u.wid >= 0) {
    const int tiles_a = (F.hist[u.wid] + kTileRows - 1) / kTileRows;
    u.tiles = tiles_a - UT * u.sub < UT ? tiles_a - UT * u.sub : UT;
  }
  return u;
}

// The rows of the unit, into F.rows / F.rseg (slot 16 w + c = row c of the unit's tile w; -1 =
// empty): the adapter's rows in segment order, of which the unit holds 16 UT sub ... + 16 UT - 1.
template <int THREADS, int UT, bool PAIRS>
__device__ __forceinline__ void find_rows(FindLds<THREADS, PAIRS>& F, const FindSeg& seg, const FoundUnit& u) {
  const int q_lo = u.sub * UT * kTileRows;
  const uint32_t mine = (seg.counted && seg.key == u.wid) ? (uint32_t)seg.len : 0u;
  uint32_t hi_u;
  const int lo = (int)block_scan_excl_1<THREADS>(mine, F.tot_b, &hi_u);
  const int hi = (int)hi_u;
  const int q0 = lo > q_lo ? lo : q_lo, q1 = hi < q_lo + UT * kTileRows ? hi : q_lo + UT * kTileRows;
  // every segment that reaches into the unit is written out by its whole wave, a lane a row (a long
  // segment fills the unit by itself: one lane writing 64 rows in turn is what this avoids)
  static_assert(UT * kTileRows <= kWaveSize, "a lane per row of the unit");
  const int lane = threadIdx.x & 63;
  uint64_t todo = __ballot(q0 < q1);
  while (todo) {  // uniform over the wave
    const int l = __builtin_ctzll(todo);
    todo &= todo - 1;
    const int b0 = __builtin_amdgcn_readlane(q0, l), b1 = __builtin_amdgcn_readlane(q1, l);
    const int r0 = __builtin_amdgcn_readlane(seg.s0 + (q0 - lo), l);
    if (b0 + lane < b1) {
      F.rows[b0 + lane - q_lo] = r0 + lane;
      F.rseg[b0 + lane - q_lo] = (int)(threadIdx.x - lane) + l;
    }
  }
  __syncthreads();
}

// ---- decode batches: the eight-wave shrink_kernel ------------------------------------------
// THREADS = 512: a workgroup is the eight waves of shrink_kernel and takes one k slice of its tile.
// THREADS = 1024 (more than 512 segments; the finder and the plan builders hold a segment per
// thread): two such groups of eight waves, which take two neighbouring k slices of the tile and sum
// each for itself -- the same sums as two workgroups of the 512-thread kind.
// The sums' staging area lies behind the finder's LDS where both fit under the plan builders'
// and over it otherwise.
template <int NB, int THREADS, bool PAIRS>
struct SelfPlanWork {
  static constexpr int kWaves = THREADS / kWaveSize;
  static constexpr bool kOverlay = sizeof(FindLds<THREADS, PAIRS>) + sizeof(f32x4) * kWaves * NB * kWaveSize >
                                   sizeof(PlanSmallLdsT<THREADS>);
  FindLds<THREADS, PAIRS> find;
  f32x4 red[kOverlay ? 1 : kWaves][NB][kWaveSize];
};
template <int NB, int THREADS, bool PAIRS>
union SelfPlanLds {
  PlanSmallLdsT<THREADS> plan;                      // the plan-building workgroups
  SelfPlanWork<NB, THREADS, PAIRS> work;            // the others: finding their tile, then the cross-wave sums
  f32x4 red[THREADS / kWaveSize][NB][kWaveSize];    // ... which reuse the finder's memory when the two do not fit side by side
};

template <int DT, int NB, int U, int THREADS, bool PAIRS = false>
__global__ __launch_bounds__(THREADS) void shrink_self_planned_kernel(SelfPlanArgs a) {
  static_assert(THREADS == kSelfPlanThreads || THREADS == 2 * kSelfPlanThreads, "one or two groups of eight waves");
  __shared__ SelfPlanLds<NB, THREADS, PAIRS> sm;
  constexpr int NW = kSelfPlanThreads / kWaveSize;  // waves that sum one k slice
  constexpr int HALVES = THREADS / kSelfPlanThreads;
  constexpr bool kOverlay = SelfPlanWork<NB, THREADS, PAIRS>::kOverlay;
  const int tid = threadIdx.x;
  if ((int)blockIdx.y == a.units) {  // the extra row of the grid: up to kSelfPlanBuilders workgroups build the plan
    const int part = (int)(blockIdx.z * gridDim.x + blockIdx.x), all = (int)(gridDim.x * gridDim.z);
    if (part < kSelfPlanBuilders) plan_small_body(a.plan, sm.plan, part, all < kSelfPlanBuilders ? all : kSelfPlanBuilders);
    return;
  }
  // grid x: (k slice, 64-column block) of the projection, k slices fastest -- in pairs when a
  // workgroup takes two (the host launches that kind only when every k split is even)
  const int pj = blockIdx.z;
  if ((int)blockIdx.x * HALVES >= a.sh.items.row_start[pj + 1] - a.sh.items.row_start[pj]) return;
  const ShrinkProj P = a.sh.p[pj];
  FindLds<THREADS, PAIRS>& F = sm.work.find;
  const int wave_all = tid >> 6, lane = tid & 63;
  const int wave = wave_all % NW;           // wave within its group of eight
  const int yy = (int)blockIdx.x * HALVES + wave_all / NW;
  const int c = lane & 15, g = lane >> 4;
  const int kz = yy % P.ksplit, zb = yy / P.ksplit;
  const int n0 = zb * 64;
  const int kbeg = (kz * NW + wave) * P.k_per_wave;
  const int kend = min(kbeg + P.k_per_wave, P.d_in);
  const uint16_t* zeros = reinterpret_cast<const uint16_t*>(self_plan_zeros);

  // PAIRS: the table has an entry per segment, and a row of workgroups for every tile the batch could have
  // (one more per table entry) would be mostly idle ones.  The launch has a row for every tile such a batch
  // usually has -- its rows in whole tiles plus a few dozen part-filled ones -- and a batch with more tiles
  // sends its workgroups round again.  The other kind has a row per possible tile and takes one turn.
  for (int tile = blockIdx.y;; tile += a.units) {
  FindSeg seg;
  const FoundUnit un =
      find_adapter<THREADS, 1, PAIRS>(F, a.plan, P.w_ptrs, a.sh.plan.w_rank, a.n_weights, tile, &seg);
  const int wid = un.wid;
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

  find_rows<THREADS, 1, PAIRS>(F, seg, un);
  const int row = F.rows[c], rseg = F.rseg[c];
  if (kOverlay) __syncthreads();  // every wave holds its tile: the finder's LDS turns into the sum's staging area

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

  // decided at compile time; every group of eight waves has its own part of the area
  f32x4 (*red)[NB][kWaveSize] = (kOverlay ? sm.red : sm.work.red) + (wave_all - wave);
  // cross-wave sum in wave order; the group's first wave writes the tile
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
  if (!PAIRS || tile + a.units >= un.total) return;  // uniform over the workgroup: no tile is left for it
  __syncthreads();                         // the sums are read: the finder takes its LDS back
  }
}

// ---- larger batches: the tile-block shrink_block_kernel ------------------------
// WKN: the weights are stored [k][n], as B is for the backward's dV = dY B.
// THREADS = 256: a workgroup is the four waves of shrink_block_kernel and takes one k slice of its
// tile block.  THREADS = 512 (more than 256 segments; finder and plan builders hold a segment per
// thread): two such groups of four waves, each with its own staging buffers, which take two
// neighbouring k slices -- the same sums as two workgroups of the 256-thread kind.  Both groups
// walk a whole slice's worth of batches (past the end of k they multiply zeros) so that they meet
// at the same barriers.
template <int NB, int U, bool WKN, int GROUPS>
struct SelfPlanBlockStage {
  static constexpr int kPitch = WKN ? 16 * NB + 8 : 32 * U + 8;
  uint16_t wlds[GROUPS][2][(WKN ? 32 * U : 16 * NB) * kPitch];
};
template <int NB, int U, bool WKN, int THREADS, bool PAIRS>
union SelfPlanBlockLds {
  PlanSmallLdsT<THREADS> plan;                                  // the plan-building workgroups
  FindLds<THREADS, PAIRS> find;                                 // the others: first while they find their tile block ...
  SelfPlanBlockStage<NB, U, WKN, THREADS / kFwdThreads> stage;  // ... then the staged weight batches
};

template <int DT, int NB, int U, bool WKN, int THREADS, bool PAIRS = false>
__global__ __launch_bounds__(THREADS) void shrink_block_self_planned_kernel(SelfPlanArgs a) {
  static_assert(THREADS == kFwdThreads || THREADS == 2 * kFwdThreads, "one or two groups of four waves");
  constexpr int GROUPS = THREADS / kFwdThreads;
  constexpr int KB = 32 * U;                 // k per batch
  constexpr int kRowsW = 16 * NB;            // weight rows (output columns) per workgroup
  constexpr int kPitch = SelfPlanBlockStage<NB, U, WKN, GROUPS>::kPitch;
  constexpr int kPieces = kRowsW * (KB / 8); // 16-byte pieces of one staged batch
  constexpr int kPer = (kPieces + kFwdThreads - 1) / kFwdThreads;
  __shared__ __attribute__((aligned(16))) SelfPlanBlockLds<NB, U, WKN, THREADS, PAIRS> sm;
  if ((int)blockIdx.y == a.units) {  // the extra row of the grid: up to kSelfPlanBuilders workgroups build the plan
    const int part = (int)(blockIdx.z * gridDim.x + blockIdx.x), all = (int)(gridDim.x * gridDim.z);
    if (part < kSelfPlanBuilders) plan_small_body(a.plan, sm.plan, part, all < kSelfPlanBuilders ? all : kSelfPlanBuilders);
    return;
  }
  // grid x: (k slice, 64-column block) of the projection, k slices fastest -- in pairs when a
  // workgroup takes two (the host launches that kind only when every k split is even)
  const int pj = blockIdx.z;
  if ((int)blockIdx.x * GROUPS >= a.sh.items.row_start[pj + 1] - a.sh.items.row_start[pj]) return;
  const ShrinkProj P = a.sh.p[pj];
  const int grp = threadIdx.x / kFwdThreads, tl = threadIdx.x % kFwdThreads;  // group of four waves, thread in it
  const int wave = tl >> 6, lane = threadIdx.x & 63;
  const int yy = (int)blockIdx.x * GROUPS + grp;
  const int c = lane & 15, g = lane >> 4;
  const uint16_t* zeros = reinterpret_cast<const uint16_t*>(self_plan_zeros);
  const int kz = yy % P.ksplit, zb = yy / P.ksplit;
  const int n0 = zb * 64;
  const int kbeg = kz * kFwdWaves * P.k_per_wave;
  const int kend = min(kbeg + kFwdWaves * P.k_per_wave, P.d_in);
  const int kstop = GROUPS > 1 ? kbeg + kFwdWaves * P.k_per_wave : kend;  // the same number of batches for both groups

  // (PAIRS: a row of workgroups for every tile block the batch usually has; the others go round again, as in
  // shrink_self_planned_kernel)
  for (int tb = blockIdx.y;; tb += a.units) {
  FindSeg seg;
  const FoundUnit un =
      find_adapter<THREADS, kBlkTiles, PAIRS>(sm.find, a.plan, P.w_ptrs, a.sh.plan.w_rank, a.n_weights, tb, &seg);
  if (un.wid < 0) return;  // past the last tile block; uniform over the workgroup
  const uint16_t* W = reinterpret_cast<const uint16_t*>(sm.find.wtab[un.wid]);
  int nlim = P.d_out;  // weight rows at or past it are zero padding
  if (a.sh.plan.w_rank) {
    const int r8 = (sm.find.rtab[un.wid] + 7) & ~7;
    nlim = r8 < nlim ? r8 : nlim;
  }
  const int ldw = WKN ? rank_ld(a.sh.plan, P.ldw, nlim) : P.ldw;  // [k][n] weights (B) have the rank contiguous
  auto load_w = [&](int kb, u32x4 (&st)[kPer]) {
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int idx = tl + j * kFwdThreads;
      if (WKN) {
        const int kl = idx / (kRowsW / 8), n8 = (idx % (kRowsW / 8)) * 8;
        st[j] = ldg16_or(W + (long)(kb + kl) * ldw + n0 + n8, idx < kPieces && n0 + n8 < nlim && kb + kl < kend,
                         zeros);
      } else {
        const int nl = idx / (KB / 8), k8 = (idx % (KB / 8)) * 8;
        st[j] = ldg16_or(W + (long)(n0 + nl) * ldw + kb + k8, idx < kPieces && n0 + nl < nlim && kb + k8 < kend,
                         zeros);
      }
    }
  };
  auto stage_w = [&](int buf, const u32x4 (&st)[kPer]) {
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int idx = tl + j * kFwdThreads;
      const int r_ = WKN ? idx / (kRowsW / 8) : idx / (KB / 8);
      const int c_ = WKN ? (idx % (kRowsW / 8)) * 8 : (idx % (KB / 8)) * 8;
      if (idx < kPieces) *reinterpret_cast<u32x4*>(&sm.stage.wlds[grp][buf][r_ * kPitch + c_]) = st[j];
    }
  };
  auto weight_frag = [&](int buf, int u, int nb) -> u32x4 {
    if (WKN) {  // as in shrink_block_kernel: four consecutive k rows of one column per transposing read
      const uint16_t* base = &sm.stage.wlds[grp][buf][(32 * u + 8 * g + (c >> 2)) * kPitch + 16 * nb + 4 * (c & 3)];
      const u32x2 q0 = lds_read_tr16(base), q1 = lds_read_tr16(base + 4 * kPitch);
      return u32x4{q0[0], q0[1], q1[0], q1[1]};
    }
    return *reinterpret_cast<const u32x4*>(&sm.stage.wlds[grp][buf][(16 * nb + c) * kPitch + 32 * u + 8 * g]);
  };
  // the adapter is known: its first weight batch is requested while the rows are still being found
  u32x4 wst[kPer];
  load_w(kbeg, wst);

  find_rows<THREADS, kBlkTiles, PAIRS>(sm.find, seg, un);
  const bool active = wave < un.tiles;
  const int row = active ? sm.find.rows[wave * kTileRows + c] : -1;
  const int rseg = active ? sm.find.rseg[wave * kTileRows + c] : -1;
  const uint16_t* xrow = P.x + (long)(row < 0 ? 0 : row) * P.d_in;
  auto load_x = [&](int kb, u32x4 (&xf)[U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = kb + 32 * u + 8 * g;
      xf[u] = ldg16_or(xrow + kk, row >= 0 && kk < kend, zeros);
    }
  };

  f32x4 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- the product, as shrink_block_kernel does it
  u32x4 xf[U];
  load_x(kbeg, xf);
  __syncthreads();  // every wave holds its rows: the finder's LDS turns into the weight staging area
  stage_w(0, wst);
  int buf = 0;
#pragma unroll 1
  for (int kb = kbeg; kb < kstop; kb += KB) {
    u32x4 xn[U], wn[kPer];
    load_x(kb + KB, xn);
    load_w(kb + KB, wn);
    __syncthreads();  // buffer `buf` is written; buffer `buf ^ 1` is no longer read
    if (active) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb] = Num<DT>::mfma(weight_frag(buf, u, nb), xf[u], acc[nb]);
      }
    }
    stage_w(buf ^ 1, wn);
    buf ^= 1;
#pragma unroll
    for (int u = 0; u < U; ++u) xf[u] = xn[u];
  }

  if (row >= 0) {
    const bool as_partial = P.ksplit > 1 || P.to_partial;
    float scale = 1.0f;
    if (!as_partial && a.sh.seg_scale) scale = a.sh.seg_scale[rseg];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const int n = n0 + 16 * nb + 4 * g;  // lane holds columns n .. n+3 of its token
      if (n >= P.d_out) continue;
      if (as_partial)
        *(SMLM_GLOBAL f32x4*)(P.partial + ((long)kz * a.sh.T + row) * P.d_out + n) = acc[nb];
      else
        store4<DT>(P.out + (long)row * P.d_out + n, acc[nb], scale, a.sh.beta);
    }
  }
  if (!PAIRS || tb + a.units >= un.total) return;  // uniform over the workgroup: no tile block is left for it
  __syncthreads();                       // the staged weights are read: the finder takes its LDS back
  }
}

}  // namespace smlm
