// C ABI of libsmlm_hip (see include/smlm.h): argument checks, workspace
// carving, launch-shape choice and kernel dispatch.  No allocation, no host
// synchronisation, no state.
#include <hip/hip_runtime.h>

#include <atomic>

#include "rms_norm.hpp"
#include "segments.hpp"
#include "smlm.h"
#include "smlm_backward.hpp"
#include "smlm_common.hpp"
#include "smlm_decode.hpp"
#include "smlm_forward.hpp"
#include "smlm_plan.hpp"

using namespace smlm;

// Scratch of smlm_gemm_static (file scope; see static_scratch below).
static __device__ __align__(256) unsigned char scratch[SMLM_STATIC_SCRATCH_BYTES];

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline int round_up(int a, int b) { return ceil_div(a, b) * b; }

// Every kernel takes one argument struct.  hipLaunchKernel hands back the
// status of this launch itself; the thread's "last error" slot is shared with
// every other HIP user in the process (torch leaves benign codes there), so it
// is neither read nor cleared here.
template <typename A>
int launch(void (*kernel)(A), dim3 grid, dim3 block, hipStream_t st, const A& a) {
  void* params[] = {const_cast<A*>(&a)};
  return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, params, 0, st) ==
                 hipSuccess
             ? SMLM_OK
             : SMLM_ERR_LAUNCH;
}

// ---- launch shapes: functions of (T, d_in, d_out) only, never of the
// segmentation, so re-segmenting a batch cannot change a bit of any row. ----
// Tiles per work item: single 16-row tiles for batches of few rows, tile blocks (up to kBlkTiles tiles of one
// adapter, their weights staged once in LDS) for larger ones.  Where the forward changes over depends on the
// rank -- the tile-block kernels save weight traffic in proportion to it.  Single tiles / tile blocks in us, one
// projection 4096 -> 4096: rank 16 at 2000 rows 18.4 / 20.8, at 3072 rows 26.0 / 24.5; rank 32 at 1024 rows
// 15.6 / 17.8, at 1536 rows 21.7 / 19.2; rank 64 at 256 rows 17.0 / 16.3, at 1000 rows 22.9 / 18.8.  A launch of
// several projections, whose workgroups fill the chip together, would change over earlier (q/k/v/o: rank 16 at
// 1024 rows 30.9 / 30.9, at 2048 rows 53.1 / 47.5; rank 32 at 384 rows 24.5 / 25.3, at 768 rows 34.6 / 30.7;
// rank 64 at 128 rows 27.6 / 24.7); the rule lies between the two and does not look at the number of
// projections, so that a launch of several gives the bits that launches of one give.
inline int tiles_per_wave(int T, int r) {
  const int from = r <= 16 ? 2048 : (r <= 32 ? 768 : (r <= 48 ? 512 : (r <= 64 ? 128 : 1024)));
  return T >= from ? kBlkTiles : 1;
}
// The backward runs on tile blocks at every size up to rank 64: its single-tile route needs transposed copies
// of the weights first (64 rows at rank 64: 25.0 / 18.8 us; 1024 rows at rank 16: 28.3 / 25.3 us).
inline int bwd_tiles_per_wave(int n_rows, int r) { return (r <= 64 || n_rows >= 1024) ? kBlkTiles : 1; }

// Upper bound of the number of work units along the tile axis.  `groups` bounds
// the number of distinct plan keys (adapters): every group ends in at most one
// partly filled tile and one partly filled tile block.
inline int tile_units_max(int T, int S, int groups, int mt) {
  const int g = (groups > 0 && groups < S) ? groups : S;
  const int nt = T / kTileRows + g + 1;  // never above the plan's own bound plan_nt_max(T, S)
  const int nb = nt / kBlkTiles + g + 2;
  return (mt == 1 || nb > nt) ? nt : nb;  // there are never more tile blocks than tiles
}

// Launches of at most this many items run one item per workgroup (direct mode); measured
// faster than the persistent walk at every size tried (up to ~130k workgroups), so the walk
// is only the fallback for batches far beyond those.
constexpr long kDirectItems = 1L << 22;
constexpr int kMaxGridY = 65535;  // tile units are the y axis of a direct launch

// persistent 1-D grid: a multiple of the XCD count, no larger than the work bound
constexpr int kMaxGrid = 2048;
inline dim3 work_grid(long bound) {
  const long cap = kMaxGrid;
  long g = bound < cap ? bound : cap;
  g = (g + kNumXcd - 1) / kNumXcd * kNumXcd;
  return dim3((unsigned)g);
}

struct ShrinkCfg {
  int NB, U, MT, NW, ksplit, k_per_wave, zblocks;
};

constexpr int kDecodeWaves = 8;  // waves of the decode shrink's workgroups ...
constexpr int kDecodeSplit = 4;  // ... and its k split over workgroups, folded by the expand kernel
constexpr int kMaxExpandFold = kMaxVsplit;  // most partials the expand kernel folds itself

// waves per shrink workgroup, one choice for all projections of a launch: small
// batches whose every projection has a long enough k use eight waves and split k in four
int shrink_waves(int mt, int nproj, const int* d_in, int d_out) {
  const int kq = 32 * (d_out > 32 ? 2 : 4);  // k per wave and load batch of the decode kernels
  bool all_long = mt == 1;
  for (int i = 0; i < nproj; ++i) all_long = all_long && d_in[i] >= 16 * kq;
  return all_long ? kDecodeWaves : kFwdWaves;
}

// solo: the product is only ever launched by itself (the backward's dV and v products) and may take the
// splits that suit a launch of one projection; the forward's projections keep one rule
// whether they are launched alone or together, so that either way gives the same bits
ShrinkCfg shrink_cfg(int T, int d_in, int d_out, int nw, bool solo, int mt) {
  ShrinkCfg c;
  c.zblocks = ceil_div(d_out, 64);
  const int cols = d_out >= 64 ? 64 : d_out;
  c.NB = cols <= 16 ? 1 : (cols <= 32 ? 2 : 4);
  c.MT = mt;
  // 32-wide k steps per load batch (the tile-block kernel stages four per batch in LDS)
  c.U = c.MT > 1 ? 4 : (c.NB == 4 ? 2 : 4);
  const int kq = 32 * c.U;
  c.NW = nw;
  const int units = ceil_div(T > 0 ? T : 1, kTileRows * c.MT);
  // k split over workgroups: enough of them to fill the chip, but every split writes and
  // re-reads an fp32 partial of the output (8*r bytes a row against 2*d_in of input), so
  // beyond 256 workgroups the split stops where the partials reach an eighth of the input.
  // Eight-wave workgroups (decode batches: few tiles) split k in four, which quadruples the
  // number of CUs at work; the expand kernel adds the four partials.
  // (A launch of one projection fills the chip twice over from 4096 rows on: 8192 rows at rank 64, h_in =
  // 4096, k in four instead of two: 27.6 -> 23.3 us; 4096 rows, h_in = 11008, in eight instead of five: 44.4
  // -> 35.6 us.  In a launch of several projections the same splits were 2-20 % slower: cfg5 180 -> 190 us.)
  int want = c.NW == kDecodeWaves ? kDecodeSplit : ceil_div(1024, units);
  const int cheap = d_in / (32 * d_out), fill = ceil_div((solo && c.MT > 1 && units >= 64) ? 512 : 256, units);
  const int cap = cheap > fill ? cheap : fill;
  if (want > cap) want = cap;
  int max_split = d_in / (c.NW * kq);
  if (max_split < 1) max_split = 1;
  if (max_split > kMaxKsplit) max_split = kMaxKsplit;
  const int ks = want < 1 ? 1 : (want > max_split ? max_split : want);
  // (the single-tile kernels' waves take a k range each: whole load batches a wave; a tile block's four
  // waves walk one slice together, which is cut to whole load batches, so its slices come out nearly equal:
  // k = 11008 in eight is seven slices of 1408 and one of 1152 instead of seven of 1536 and one of 256)
  c.k_per_wave = round_up(ceil_div(d_in, c.NW * ks), c.MT > 1 ? kq / c.NW : kq);
  c.ksplit = ceil_div(d_in, c.NW * c.k_per_wave);
  // An odd split (h_in = 14336 falls into seven slices of 2048) gives way to an even one of equal slices that
  // still fills the chip twice: 8192 rows, h_in = 14336, k in four instead of seven: rank 16 61.6 -> 53.1 us,
  // rank 64 80.0 -> 67.8 us (six, eight, ten ... fourteen slices: 56-65 and 77-87 us).
  if (solo && c.MT > 1 && c.ksplit > 1 && (c.ksplit & 1) && d_in % (c.NW * kq) == 0) {
    const int pieces = d_in / (c.NW * kq);
    for (int e = c.ksplit - 1; e >= 2; --e)
      if (e % 2 == 0 && pieces % e == 0 && units * e >= 512) {
        c.k_per_wave = pieces / e * kq;
        c.ksplit = e;
        break;
      }
  }
  return c;
}

// most k-split partials a shrink of this shape can leave behind, whichever wave count it runs with
int fwd_ksplit_bound(int T, int d_in, int d_out) {
  int most = 1;
  for (int solo = 0; solo < 2; ++solo) {
    const int a = shrink_cfg(T, d_in, d_out, kFwdWaves, solo != 0, 1).ksplit;
    const int b = shrink_cfg(T, d_in, d_out, kDecodeWaves, solo != 0, 1).ksplit;
    const int c = shrink_cfg(T, d_in, d_out, kFwdWaves, solo != 0, kBlkTiles).ksplit;
    most = a > most ? a : most;
    most = b > most ? b : most;
    most = c > most ? c : most;
  }
  return most;
}

int expand_nq(int T, int d_out) {
  (void)T;
  // 32-column blocks per wave: four (a workgroup then covers 512 columns) unless the
  // projection is narrower than that
  return d_out >= 512 ? 4 : 2;
}

TileArgs tile_args(const PlanView& pv, int n_weights) {
  TileArgs t{pv.hdr, pv.tile_row, pv.tile_rseg, pv.tile_wid, pv.blk};
  t.n_weights = n_weights;  // 0: unknown
  return t;
}

// grid of a launch: (chunk row, tile unit, projection), or (chunk row over all projections,
// tile unit) when flat, in direct mode; else the persistent one-dimensional grid
inline dim3 item_grid(const ItemSpace& sp, long items) {
  if (!sp.units_max) return work_grid(items);
  if (sp.flat) return dim3((unsigned)sp.row_start[sp.nproj], (unsigned)sp.units_max, 1u);
  int rows = 1;
  for (int i = 0; i < sp.nproj; ++i)
    if (sp.row_start[i + 1] - sp.row_start[i] > rows) rows = sp.row_start[i + 1] - sp.row_start[i];
  return dim3((unsigned)rows, (unsigned)sp.units_max, (unsigned)sp.nproj);
}

template <int DT, int NW, bool RM, bool DIRECT, bool DROP = false>
int launch_shrink_nb(int NB, dim3 grid, hipStream_t st, const ShrinkArgs& a) {
  const dim3 block(NW * kWaveSize);  // U must match shrink_cfg
  if (NB == 1) return launch(shrink_kernel<DT, 1, 4, NW, RM, DIRECT, DROP>, grid, block, st, a);
  if (NB == 2) return launch(shrink_kernel<DT, 2, 4, NW, RM, DIRECT, DROP>, grid, block, st, a);
  return launch(shrink_kernel<DT, 4, 2, NW, RM, DIRECT, DROP>, grid, block, st, a);
}

template <int DT, bool DIRECT, bool WKN, bool DROP = false>
int launch_shrink_block(int NB, dim3 grid, hipStream_t st, const ShrinkArgs& a) {
  const dim3 block(kFwdThreads);
  if (NB == 1) return launch(shrink_block_kernel<DT, 1, 4, DIRECT, WKN, DROP>, grid, block, st, a);
  if (NB == 2) return launch(shrink_block_kernel<DT, 2, 4, DIRECT, WKN, DROP>, grid, block, st, a);
  return launch(shrink_block_kernel<DT, 4, 4, DIRECT, WKN, DROP>, grid, block, st, a);
}

template <int DT, bool DIRECT>
int launch_shrink_dt(bool row_major, int NB, int MT, int NW, dim3 grid, hipStream_t st,
                     const ShrinkArgs& a) {
  if (row_major)  // the slow layout
    return launch_shrink_nb<DT, kFwdWaves, true, DIRECT>(NB, grid, st, a);
  if (a.drop.seg_p) {  // dropout of the training rows: x in the usual layout, weights [n][k]
    if (MT == 1)
      return NW == kDecodeWaves ? launch_shrink_nb<DT, kDecodeWaves, false, DIRECT, true>(NB, grid, st, a)
                                : launch_shrink_nb<DT, kFwdWaves, false, DIRECT, true>(NB, grid, st, a);
    return launch_shrink_block<DT, DIRECT, false, true>(NB, grid, st, a);
  }
  if (MT == 1)
    return NW == kDecodeWaves ? launch_shrink_nb<DT, kDecodeWaves, false, DIRECT>(NB, grid, st, a)
                              : launch_shrink_nb<DT, kFwdWaves, false, DIRECT>(NB, grid, st, a);
  return a.w_kn ? launch_shrink_block<DT, DIRECT, true>(NB, grid, st, a)
                : launch_shrink_block<DT, DIRECT, false>(NB, grid, st, a);
}

// all projections of one launch share NB / U / MT / NW (same rank, same T)
int launch_shrink(int dtype, bool row_major, const ShrinkCfg& c, int S, int groups, hipStream_t st,
                  ShrinkArgs& a) {
  const int MT = row_major ? 1 : c.MT;
  a.items.interleave = 1;
  const int units = tile_units_max(a.T, S, groups, MT);
  const long items = (long)units * a.items.row_start[a.items.nproj];
  a.items.units_max = (items <= kDirectItems && units <= kMaxGridY) ? units : 0;
  const dim3 grid = item_grid(a.items, items);
  const bool f16 = dtype == SMLM_DTYPE_F16;
  if (a.items.units_max)
    return f16 ? launch_shrink_dt<SMLM_DTYPE_F16, true>(row_major, c.NB, MT, c.NW, grid, st, a)
               : launch_shrink_dt<SMLM_DTYPE_BF16, true>(row_major, c.NB, MT, c.NW, grid, st, a);
  return f16 ? launch_shrink_dt<SMLM_DTYPE_F16, false>(row_major, c.NB, MT, c.NW, grid, st, a)
             : launch_shrink_dt<SMLM_DTYPE_BF16, false>(row_major, c.NB, MT, c.NW, grid, st, a);
}

template <int DT, int THREADS, bool PAIRS>
int launch_self_planned_nb(int NB, dim3 grid, hipStream_t st, const SelfPlanArgs& a) {
  const dim3 block(THREADS);  // U must match shrink_cfg
  if (NB == 1) return launch(shrink_self_planned_kernel<DT, 1, 4, THREADS, PAIRS>, grid, block, st, a);
  if (NB == 2) return launch(shrink_self_planned_kernel<DT, 2, 4, THREADS, PAIRS>, grid, block, st, a);
  return launch(shrink_self_planned_kernel<DT, 4, 2, THREADS, PAIRS>, grid, block, st, a);
}

template <int DT, bool WKN, int THREADS, bool PAIRS>
int launch_self_planned_block_nb(int NB, dim3 grid, hipStream_t st, const SelfPlanArgs& a) {
  const dim3 block(THREADS);  // U must match shrink_cfg
  if (NB == 1) return launch(shrink_block_self_planned_kernel<DT, 1, 4, WKN, THREADS, PAIRS>, grid, block, st, a);
  if (NB == 2) return launch(shrink_block_self_planned_kernel<DT, 2, 4, WKN, THREADS, PAIRS>, grid, block, st, a);
  return launch(shrink_block_self_planned_kernel<DT, 4, 4, WKN, THREADS, PAIRS>, grid, block, st, a);
}
template <int DT, bool WKN, bool PAIRS>
int launch_self_planned_block(int NB, int S, dim3 grid, hipStream_t st, const SelfPlanArgs& a) {
  if (S <= kFwdThreads) return launch_self_planned_block_nb<DT, WKN, kFwdThreads, PAIRS>(NB, grid, st, a);
  // more segments than the four-wave workgroup has threads: two such groups a workgroup, each
  // taking one of two neighbouring k slices (the caller has checked that the splits are even)
  grid.x = (grid.x + 1) / 2;
  return launch_self_planned_block_nb<DT, WKN, 2 * kFwdThreads, PAIRS>(NB, grid, st, a);
}

// batches this route takes: few enough segments for the plan-building workgroups of the launch
// (one segment per thread: 512 or 1024 in the decode shrink, 256 or 512 in the tile-block shrink),
// adapter ids that index a table of at most kSelfPlanWeights entries
bool self_planned_ok(int T, int S, int n_weights, int nt_max, int mt) {
  const int segs = mt > 1 ? (S <= kFwdThreads ? kFwdThreads : kSelfPlanBlkSegs)
                          : (S <= kSelfPlanThreads ? kSelfPlanThreads : kSelfPlanSegs);
  return S <= segs && nt_max <= 4 * segs && n_weights >= 1 && n_weights <= kSelfPlanWeights &&
         tile_units_max(T, S, n_weights, mt) < kMaxGridY;
}

template <int DT>
int launch_self_planned_dt(bool pairs, const ShrinkCfg& c, int S, dim3 grid, hipStream_t st, const SelfPlanArgs& sp) {
  if (c.MT == 1 && S > kSelfPlanThreads) {
    // more segments than the eight-wave workgroup has threads: workgroups of two such groups of
    // waves, each taking two neighbouring k slices (the caller has checked that the splits are even)
    grid.x = (grid.x + 1) / 2;
    return pairs ? launch_self_planned_nb<DT, 2 * kSelfPlanThreads, true>(c.NB, grid, st, sp)
                 : launch_self_planned_nb<DT, 2 * kSelfPlanThreads, false>(c.NB, grid, st, sp);
  }
  if (c.MT > 1 && sp.sh.w_kn) return launch_self_planned_block<DT, true, false>(c.NB, S, grid, st, sp);
  if (c.MT > 1)
    return pairs ? launch_self_planned_block<DT, false, true>(c.NB, S, grid, st, sp)
                 : launch_self_planned_block<DT, false, false>(c.NB, S, grid, st, sp);
  return pairs ? launch_self_planned_nb<DT, kSelfPlanThreads, true>(c.NB, grid, st, sp)
               : launch_self_planned_nb<DT, kSelfPlanThreads, false>(c.NB, grid, st, sp);
}

int launch_shrink_self_planned(int dtype, const ShrinkCfg& c, int S, int groups, const PlanSortArgs& build,
                               hipStream_t st, const ShrinkArgs& a) {
  if (c.MT == 1 && c.NW * kWaveSize != kSelfPlanThreads) return SMLM_ERR_ARG;
  if (c.MT > 1 && c.NW != kFwdWaves) return SMLM_ERR_ARG;
  SelfPlanArgs sp{};
  sp.sh = a;
  sp.plan = build;
  sp.n_weights = groups;
  // rows of workgroups: one per unit the batch can have.  Plans keyed by pairs of addresses (a table entry per
  // segment, so nearly all of those rows would find no unit) get no more than the batch's rows in whole units
  // plus 32 part-filled ones; their kernels take the units beyond that in further rounds.
  const bool pairs = build.key_kind == SMLM_KEY_PTR2;
  sp.units = tile_units_max(a.T, S, groups, c.MT);
  const int usual = a.T / (kTileRows * c.MT) + 1 + 32;
  if (pairs && sp.units > usual) sp.units = usual;
  if (pairs && a.w_kn) return SMLM_ERR_ARG;  // (no caller: the row-major products build their plan with a launch)
  int rows = 1;
  for (int i = 0; i < a.items.nproj; ++i)
    if (a.items.row_start[i + 1] - a.items.row_start[i] > rows) rows = a.items.row_start[i + 1] - a.items.row_start[i];
  dim3 grid((unsigned)rows, (unsigned)sp.units + 1u, (unsigned)a.items.nproj);
  return dtype == SMLM_DTYPE_F16 ? launch_self_planned_dt<SMLM_DTYPE_F16>(pairs, c, S, grid, st, sp)
                                 : launch_self_planned_dt<SMLM_DTYPE_BF16>(pairs, c, S, grid, st, sp);
}

int launch_reduce(int dtype, int S, int groups, hipStream_t st, ReduceArgs& a, bool side = false) {
  const int row_tiles = ceil_div(a.T, kTileRows);
  if (side) {  // by tile slot: the by-products are stored in slot order
    const int units = tile_units_max(a.T, S, groups, 1);
    const long items = (long)units * a.nproj;
    a.units_max = items <= kDirectItems ? units : 0;
    const int zero_blocks = a.zero.n ? a.zero.first[a.zero.n] : 0;
    if (zero_blocks && !a.units_max) {  // (a launch that walks its items has no workgroups to spare)
      const int rc = launch(zero_spans_kernel, dim3((unsigned)zero_blocks), dim3(256), st, a.zero);
      if (rc) return rc;
    }
    const dim3 grid = a.units_max ? dim3((unsigned)(items + zero_blocks)) : work_grid(items);
    if (dtype == SMLM_DTYPE_F16) return launch(reduce_kernel<SMLM_DTYPE_F16, true>, grid, dim3(256), st, a);
    return launch(reduce_kernel<SMLM_DTYPE_BF16, true>, grid, dim3(256), st, a);
  }
  if (!a.seg_scale && row_tiles <= kMaxGridY * 64) {  // no scale to look up: fold row by row
    const dim3 grid((unsigned)row_tiles, (unsigned)a.nproj);
    if (dtype == SMLM_DTYPE_F16) return launch(reduce_rows_kernel<SMLM_DTYPE_F16>, grid, dim3(256), st, a);
    return launch(reduce_rows_kernel<SMLM_DTYPE_BF16>, grid, dim3(256), st, a);
  }
  const int units = tile_units_max(a.T, S, groups, 1);
  const long items = (long)units * a.nproj;
  a.units_max = items <= kDirectItems ? units : 0;
  const dim3 grid = a.units_max ? dim3((unsigned)items) : work_grid(items);
  if (dtype == SMLM_DTYPE_F16) return launch(reduce_kernel<SMLM_DTYPE_F16>, grid, dim3(256), st, a);
  return launch(reduce_kernel<SMLM_DTYPE_BF16>, grid, dim3(256), st, a);
}

template <int DT, int NQ, bool DIRECT>
int launch_expand_wave(int KS, bool vfold, dim3 grid, hipStream_t st, const ExpandArgs& a) {
  const dim3 block(kFwdThreads);
  if (vfold) {
    if (KS == 1) return launch(expand_wave_kernel<DT, NQ, 1, false, DIRECT, true>, grid, block, st, a);
    if (KS == 2) return launch(expand_wave_kernel<DT, NQ, 2, false, DIRECT, true>, grid, block, st, a);
    return launch(expand_wave_kernel<DT, NQ, 0, false, DIRECT, true>, grid, block, st, a);
  }
  if (KS == 1) return launch(expand_wave_kernel<DT, NQ, 1, false, DIRECT, false>, grid, block, st, a);
  if (KS == 2) return launch(expand_wave_kernel<DT, NQ, 2, false, DIRECT, false>, grid, block, st, a);
  return launch(expand_wave_kernel<DT, NQ, 0, false, DIRECT, false>, grid, block, st, a);
}

template <int DT, bool DIRECT>
int launch_expand_dt(bool row_major, bool block, int nq, int KS, dim3 grid, hipStream_t st,
                     const ExpandArgs& a) {
  if (row_major)
    return launch(expand_wave_kernel<DT, 2, 0, true, DIRECT, false>, grid, dim3(kFwdThreads), st, a);
  if (a.drop.seg_p) {  // the backward's dX with the dropout of x undone: no fold
    const dim3 bl(kFwdThreads);
    if (block)  // launch_expand admits only [k][n] weights here
      return KS == 1 ? launch(expand_block_kernel<DT, 4, 1, DIRECT, true, true>, grid, bl, st, a)
                     : launch(expand_block_kernel<DT, 4, 2, DIRECT, true, true>, grid, bl, st, a);
    if (KS == 0)  // ranks above 64: the general loop over k
      return nq == 4 ? launch(expand_wave_kernel<DT, 4, 0, false, DIRECT, false, true>, grid, bl, st, a)
                     : launch(expand_wave_kernel<DT, 2, 0, false, DIRECT, false, true>, grid, bl, st, a);
    if (nq == 4)
      return KS == 1 ? launch(expand_wave_kernel<DT, 4, 1, false, DIRECT, false, true>, grid, bl, st, a)
                     : launch(expand_wave_kernel<DT, 4, 2, false, DIRECT, false, true>, grid, bl, st, a);
    return KS == 1 ? launch(expand_wave_kernel<DT, 2, 1, false, DIRECT, false, true>, grid, bl, st, a)
                   : launch(expand_wave_kernel<DT, 2, 2, false, DIRECT, false, true>, grid, bl, st, a);
  }
  if (block && a.w_kn)
    return KS == 1 ? launch(expand_block_kernel<DT, 4, 1, DIRECT, true>, grid, dim3(kFwdThreads), st, a)
                   : launch(expand_block_kernel<DT, 4, 2, DIRECT, true>, grid, dim3(kFwdThreads), st, a);
  if (block && nq == 8)
    return KS == 1 ? launch(expand_block_kernel<DT, 8, 1, DIRECT, false>, grid, dim3(kFwdThreads), st, a)
                   : launch(expand_block_kernel<DT, 8, 2, DIRECT, false>, grid, dim3(kFwdThreads), st, a);
  if (block)
    return KS == 1 ? launch(expand_block_kernel<DT, 4, 1, DIRECT, false>, grid, dim3(kFwdThreads), st, a)
                   : launch(expand_block_kernel<DT, 4, 2, DIRECT, false>, grid, dim3(kFwdThreads), st, a);
  const bool vfold = a.p[0].vsplit > 0;  // set for all projections of a launch or for none
  return nq == 4 ? launch_expand_wave<DT, 4, DIRECT>(KS, vfold, grid, st, a)
                 : launch_expand_wave<DT, 2, DIRECT>(KS, vfold, grid, st, a);
}

// all projections of one launch share the rank (d_in); d_out may differ
int launch_expand(int dtype, bool row_major, int nq, int MT, int S, int groups, int nproj, int max_d_in,
                  hipStream_t st, ExpandArgs& a) {
  const int KS = max_d_in <= 32 ? 1 : (max_d_in <= 64 ? 2 : 0);
  const bool block = !row_major && MT > 1 && KS > 0;  // tile blocks with the weights staged in LDS
  if (a.drop.seg_p && (row_major || a.p[0].vsplit > 0 || (block && !a.w_kn))) return SMLM_ERR_ARG;
  if (row_major) nq = 2;
  // Tile blocks: 128 columns a workgroup, or 256 where measured better (rank 64, 8192 rows: 5-13 % at every
  // width; a row stride that is a multiple of 4 KiB, e.g. h_out = 14336, from 4096 rows on at every rank:
  // the 64 rows of a tile block then meet in few HBM channels and pieces of 512 bytes spread them over
  // twice as many).  Elsewhere 256 columns lose 1-12 % (fewer workgroups a CU; h_out = 11008, the
  // backward's dX, whose weights lie [k][n]).
  if (block) {
    int wide = 0;
    for (int i = 0; i < nproj; ++i) wide = a.p[i].d_out > wide ? a.p[i].d_out : wide;
    const bool aligned = (wide * 2) % 4096 == 0;
    const bool wider = !a.w_kn && !a.drop.seg_p &&
                       ((KS == 2 && a.T >= 8192) || (aligned && wide >= 8192 && a.T >= 4096));
    nq = wider ? 8 : 4;
  }
  const int chunk = block ? 32 * nq : kFwdWaves * 32 * nq;  // columns per workgroup
  a.items.nproj = nproj;
  a.items.interleave = 0;
  a.items.row_start[0] = 0;
  // Workgroups go to the XCDs in turn (workgroup number modulo eight, whatever the XCDs' load).  With an odd
  // number of chunk rows a tile unit, the workgroups of one column chunk visit all eight XCDs from unit to
  // unit and each L2 fetches that chunk of an adapter's weights for itself: a launch of one projection gets one
  // empty row then (8192 rows at rank 64: h_out = 11136, 87 chunks of 128 columns, 83.4 -> 73.3 us; h_out =
  // 11008, 43 chunks of 256, 87.8 -> 71.7 us).  Launches of several projections are left as they are: empty
  // workgroups there can fall on the same few XCDs in every unit and leave the others with all the work
  // (measured on the shrink launch of five and six projections: up to 2.2 x slower).
  for (int i = 0; i < nproj; ++i) {
    int rows = ceil_div(a.p[i].d_out, chunk);
    if (nproj == 1 && rows > 1 && (rows & 1)) rows += 1;
    a.items.row_start[i + 1] = a.items.row_start[i] + rows;
  }
  const int units = tile_units_max(a.T, S, groups, block ? kBlkTiles : 1);
  const long items = (long)units * a.items.row_start[nproj];
  bool same_rows = true;
  for (int i = 1; i < nproj; ++i)
    same_rows = same_rows && (a.items.row_start[i + 1] - a.items.row_start[i] == a.items.row_start[1]);
  a.items.flat = same_rows ? 0 : 1;
  a.items.units_max = (items <= kDirectItems && units <= kMaxGridY) ? units : 0;
  const dim3 grid = item_grid(a.items, items);
  const bool f16 = dtype == SMLM_DTYPE_F16;
  if (a.items.units_max)
    return f16 ? launch_expand_dt<SMLM_DTYPE_F16, true>(row_major, block, nq, KS, grid, st, a)
               : launch_expand_dt<SMLM_DTYPE_BF16, true>(row_major, block, nq, KS, grid, st, a);
  return f16 ? launch_expand_dt<SMLM_DTYPE_F16, false>(row_major, block, nq, KS, grid, st, a)
             : launch_expand_dt<SMLM_DTYPE_BF16, false>(row_major, block, nq, KS, grid, st, a);
}

int check_common(int T, int S, int dtype) {
  if (T < 0 || S < 0) return SMLM_ERR_ARG;
  if (dtype != SMLM_DTYPE_F16 && dtype != SMLM_DTYPE_BF16) return SMLM_ERR_DTYPE;
  if (S >= kMaxSegments || T > (1 << 30)) return SMLM_ERR_LIMIT;
  return SMLM_OK;
}

int plan_build_impl(const PlanView& pv, const int32_t* seg_indptr, const void* seg_key,
                    int key_kind, int S, hipStream_t st, const void* seg_key2 = nullptr) {
  const int N = next_pow2(S);
  const PlanSortArgs sa{pv, seg_indptr, seg_key, key_kind, S, N, seg_key2};
  if (S <= kPlanSmallSegs && pv.nt_max <= kPlanSmallTiles)
    return launch(plan_small_kernel, dim3(1), dim3(kPlanThreads), st, sa);
  int rc = (N <= kPlanLdsKeys)
               ? launch(plan_sort_kernel<true>, dim3(1), dim3(kPlanThreads), st, sa)
               : launch(plan_sort_kernel<false>, dim3(1), dim3(kPlanThreads), st, sa);
  if (rc) return rc;
  const long slots = (long)pv.nt_max * kTileRows;
  const PlanFillArgs fa{pv, seg_indptr, S};
  return launch(plan_fill_kernel, dim3((unsigned)((slots + 255) / 256)), dim3(256), st, fa);
}

// shrink of one or more projections that share row routing and output width:
// out[i] = beta*out[i] + scale * x[i] W_i^T in 16 bits, via k-split fp32 partial
// sums folded by a second launch when the split is wider than one workgroup
// (fold = false leaves every projection's fp32 partials, one or more, for the consumer to fold)
// by-products a fold may leave behind (ReduceProj::pt_a ...)
struct SideOut {
  uint16_t* pt_a[kMaxProj];
  uint16_t* pt_b[kMaxProj];
  const uint16_t* v2[kMaxProj];
  const float* scale;
  long pitch;
  ZeroSpans zero;  // memory the fold's launch is to clear as well (n = 0: none)
};

int run_shrink(int dtype, bool row_major, const PlanView& pv, int T, int S, int groups, int nproj,
               const void* const* x, const void* const* const* w_ptrs, float* const* partial,
               void* const* out, const int* d_in, int d_out, const int* ldw, float beta,
               const float* seg_scale, int mt, hipStream_t st, bool fold = true, bool w_kn = false,
               const DropArgs* drop = nullptr, const int32_t* w_rank = nullptr, int packed = 0,
               const PlanSortArgs* build = nullptr, bool solo = false, const SideOut* side = nullptr,
               bool* side_done = nullptr) {
  if (drop && drop->seg_p && (row_major || w_kn)) return SMLM_ERR_ARG;
  if (side_done) *side_done = false;
  ShrinkArgs a{};
  if (drop) a.drop = *drop;
  a.w_kn = w_kn ? 1 : 0;
  a.plan = tile_args(pv, groups);
  a.plan.w_rank = w_rank;  // the output columns are the rank
  a.plan.packed = packed;
  a.seg_scale = seg_scale;
  a.beta = beta;
  a.T = T;
  a.items.nproj = nproj;
  a.items.row_start[0] = 0;
  ReduceArgs ra{};
  bool need_reduce = false, all_reduce = true;
  ShrinkCfg c0{};
  size_t bits_off = 0;
  const int nw = row_major ? kFwdWaves : shrink_waves(mt, nproj, d_in, d_out);
  for (int i = 0; i < nproj; ++i) {
    const ShrinkCfg c = shrink_cfg(T, d_in[i], d_out, nw, solo, mt);
    if (i == 0) c0 = c;
    ShrinkProj& P = a.p[i];
    P.x = reinterpret_cast<const uint16_t*>(x[i]);
    P.w_ptrs = w_ptrs[i];
    P.partial = partial[i];
    P.out = reinterpret_cast<uint16_t*>(out[i]);
    P.d_in = d_in[i]; P.d_out = d_out; P.ldw = ldw[i];
    P.k_per_wave = c.k_per_wave; P.ksplit = c.ksplit; P.zblocks = c.zblocks;
    P.to_partial = fold ? 0 : 1;
    if (drop && drop->bits) {  // projections' masks lie end to end
      P.drop_bits = drop->bits + bits_off;
      bits_off += (size_t)drop->rows * (d_in[i] / 8);
    }
    // (a launch of one projection with an odd number of chunk rows a tile unit gets one empty row, as the
    // expand launch does and for its reason: 8192 rows at rank 64, h_in = 11008, k split in five: 75.5 ->
    // 59.6 us; 6144 rows, h_in = 4096, in three: 27.2 -> 25.0; launches of several projections and those that
    // build their plan keep their grid)
    int rows = c.ksplit * c.zblocks;
    if (nproj == 1 && !build && rows > 1 && (rows & 1)) rows += 1;
    a.items.row_start[i + 1] = a.items.row_start[i] + rows;
    ra.p[i] = ReduceProj{partial[i], P.out, c.ksplit, side ? side->pt_a[i] : nullptr, side ? side->pt_b[i] : nullptr,
                         side ? side->v2[i] : nullptr};
    need_reduce = need_reduce || c.ksplit > 1;
    all_reduce = all_reduce && c.ksplit > 1;
  }
  // Folding the k-split partials inside the shrink launch (last-arriving workgroup, ticket
  // counters) was measured and dropped: the device-scope release/acquire it needs writes back
  // and invalidates a whole L2 per workgroup on this multi-XCD part and cost 5-10x the launch
  // it saves.
  // `build`: the plan does not exist yet -- the decode shrink whose workgroups find their
  // own tile, with one more workgroup that builds the plan (the caller has checked the limits)
  int rc = build ? launch_shrink_self_planned(dtype, c0, S, groups, *build, st, a)
                 : launch_shrink(dtype, row_major, c0, S, groups, st, a);
  if (rc || !need_reduce || !fold) return rc;
  ra.plan = a.plan;
  ra.seg_scale = seg_scale;
  ra.beta = beta;
  ra.T = T; ra.d_out = d_out; ra.nproj = nproj;
  // the by-products go with the fold when every projection is folded (else they are left to the caller)
  const bool with_side = side && all_reduce;
  if (with_side) {
    ra.side_scale = side->scale;
    ra.side_pitch = side->pitch;
    ra.zero = side->zero;
  }
  if (side_done) *side_done = with_side;
  return launch_reduce(dtype, S, groups, st, ra, with_side);
}

template <int DT>
int launch_wgrad(int nbj, bool split, dim3 grid, hipStream_t st, const WgradArgs& wa) {
  if (wa.drop.seg_p) {
    if (split) {
      if (nbj == 1) return launch(wgrad_kernel<DT, 1, 4, true>, grid, dim3(256), st, wa);
      if (nbj == 2) return launch(wgrad_kernel<DT, 2, 4, true>, grid, dim3(256), st, wa);
      return launch(wgrad_kernel<DT, 4, 4, true>, grid, dim3(256), st, wa);
    }
    if (nbj == 1) return launch(wgrad_kernel<DT, 1, 1, true>, grid, dim3(64), st, wa);
    if (nbj == 2) return launch(wgrad_kernel<DT, 2, 1, true>, grid, dim3(64), st, wa);
    return launch(wgrad_kernel<DT, 4, 1, true>, grid, dim3(64), st, wa);
  }
  if (split) {
    if (nbj == 1) return launch(wgrad_kernel<DT, 1, 4>, grid, dim3(256), st, wa);
    if (nbj == 2) return launch(wgrad_kernel<DT, 2, 4>, grid, dim3(256), st, wa);
    return launch(wgrad_kernel<DT, 4, 4>, grid, dim3(256), st, wa);
  }
  if (nbj == 1) return launch(wgrad_kernel<DT, 1, 1>, grid, dim3(64), st, wa);
  if (nbj == 2) return launch(wgrad_kernel<DT, 2, 1>, grid, dim3(64), st, wa);
  return launch(wgrad_kernel<DT, 4, 1>, grid, dim3(64), st, wa);
}

struct BwdProjLayout {
  size_t at, bt, at_ptrs, bt_ptrs, partial, dv16, v16, pt_a, pt_b, bits;
};
struct BwdLayout {
  BwdProjLayout p[kMaxProj];
  size_t total;
  long pitch;
};

// the projections' areas lie end to end, each laid out as a backward of that projection alone
BwdLayout bwd_layout(int n_proj, int n_rows, int P, int NA, const int* h_in, const int* h_out, int r) {
  BwdLayout L;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t o = off;
    off = align_up(off + bytes, 256);
    return o;
  };
  L.pitch = (long)plan_nt_max(n_rows, P) * kTileRows;
  for (int i = 0; i < n_proj; ++i) {
    BwdProjLayout& Q = L.p[i];
    const int ks_dv = fwd_ksplit_bound(n_rows, h_out[i], r), ks_v = fwd_ksplit_bound(n_rows, h_in[i], r);
    const int ks = ks_dv > ks_v ? ks_dv : ks_v;
    Q.at = take((size_t)NA * h_in[i] * r * 2);
    Q.bt = take((size_t)NA * h_out[i] * r * 2);
    Q.at_ptrs = take((size_t)NA * 8);
    Q.bt_ptrs = take((size_t)NA * 8);
    Q.partial = take((size_t)ks * n_rows * r * 4);
    Q.dv16 = take((size_t)n_rows * r * 2);
    Q.v16 = take((size_t)n_rows * r * 2);
    Q.pt_a = take((size_t)r * L.pitch * 2);
    Q.pt_b = take((size_t)r * L.pitch * 2);
    Q.bits = take((size_t)n_rows * (h_in[i] / 8));  // keep bits of x's dropout mask when the caller has none
  }
  L.total = off;
  return L;
}

// Scratch of smlm_gemm_static: part of the code object, so every device the library is loaded
// on has its own copy at its own address.  In host code the name is only a handle for
// hipGetSymbolAddress; kernels and copies get the looked-up device address.
constexpr int kMaxDevices = 64;
std::atomic<void*> scratch_addr[kMaxDevices];

// device address of `scratch` on the current device (looked up once per device), or null
void* static_scratch() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* p = scratch_addr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
    scratch_addr[dev].store(p, std::memory_order_release);  // every thread finds the same address
  }
  return p;
}

}  // namespace

extern "C" {

SMLM_API int smlm_abi_version(void) { return SMLM_ABI_VERSION; }

SMLM_API const char* smlm_strerror(int code) {
  switch (code) {
    case SMLM_OK: return "ok";
    case SMLM_ERR_ARG: return "invalid argument";
    case SMLM_ERR_DTYPE: return "No suitable kernel.";
    case SMLM_ERR_ALIGN: return "dimension not a multiple of 8 or pointer not 16-byte aligned";
    case SMLM_ERR_WORKSPACE: return "workspace too small";
    case SMLM_ERR_LAUNCH: return "kernel launch failed";
    case SMLM_ERR_LIMIT: return "size beyond the supported range";
    case SMLM_ERR_SCRATCH: return "the call needs more scratch than the library's static array holds";
    default: return "unknown error";
  }
}

SMLM_API int smlm_tmp_size(int num_problems, size_t* bytes) {
  if (num_problems < 0 || !bytes) return SMLM_ERR_ARG;
  *bytes = (size_t)64 * (size_t)num_problems;
  return SMLM_OK;
}

SMLM_API int smlm_plan_size(int T, int S, size_t* bytes) {
  if (T < 0 || S < 0 || !bytes) return SMLM_ERR_ARG;
  if (S >= kMaxSegments || T > (1 << 30)) return SMLM_ERR_LIMIT;
  *bytes = plan_carve(nullptr, T, S, nullptr);
  return SMLM_OK;
}

SMLM_API int smlm_plan_build(void* plan, size_t plan_bytes, const int32_t* seg_indptr,
                             const void* seg_key, int key_kind, int T, int S, void* stream) {
  if (T < 0 || S < 0) return SMLM_ERR_ARG;
  if (S >= kMaxSegments || T > (1 << 30)) return SMLM_ERR_LIMIT;
  if (key_kind != SMLM_KEY_NONE && key_kind != SMLM_KEY_I32 && key_kind != SMLM_KEY_PTR)
    return SMLM_ERR_ARG;
  if (S == 0) return SMLM_OK;
  if (!plan || !seg_indptr || (key_kind != SMLM_KEY_NONE && !seg_key)) return SMLM_ERR_ARG;
  if (!aligned16(plan)) return SMLM_ERR_ALIGN;
  PlanView pv;
  if (plan_carve(plan, T, S, &pv) > plan_bytes) return SMLM_ERR_WORKSPACE;
  return plan_build_impl(pv, seg_indptr, seg_key, key_kind, S, (hipStream_t)stream);
}

SMLM_API int smlm_plan_build2(void* plan, size_t plan_bytes, const int32_t* seg_indptr,
                              const void* const* seg_key_a, const void* const* seg_key_b, int T, int S,
                              void* stream) {
  if (T < 0 || S < 0) return SMLM_ERR_ARG;
  if (S >= kMaxSegments || T > (1 << 30)) return SMLM_ERR_LIMIT;
  if (S == 0) return SMLM_OK;
  if (!plan || !seg_indptr || !seg_key_a || !seg_key_b) return SMLM_ERR_ARG;
  if (!aligned16(plan)) return SMLM_ERR_ALIGN;
  PlanView pv;
  if (plan_carve(plan, T, S, &pv) > plan_bytes) return SMLM_ERR_WORKSPACE;
  return plan_build_impl(pv, seg_indptr, seg_key_a, SMLM_KEY_PTR2, S, (hipStream_t)stream, seg_key_b);
}

SMLM_API int smlm_gemm_planned_workspace_size(int T, int d_in, int d_out, size_t* bytes) {
  if (T < 0 || d_in <= 0 || d_out <= 0 || !bytes) return SMLM_ERR_ARG;
  if (T > (1 << 30)) return SMLM_ERR_LIMIT;
  size_t n = 256;
  if (d_in >= d_out) {
    const int ks = fwd_ksplit_bound(T, d_in, d_out);
    if (ks > 1) n = align_up((size_t)ks * T * d_out * 4, 256);
  }
  *bytes = n;
  return SMLM_OK;
}

SMLM_API int smlm_gemm_planned(void* y, const void* x, const void* const* w_ptrs, int n_weights,
                               const void* plan, void* workspace, size_t workspace_bytes, int T,
                               int S, int d_in, int d_out, int w_ld, int w_row_major, int dtype,
                               float beta, const float* seg_scale, void* stream) {
  int rc = check_common(T, S, dtype);
  if (rc) return rc;
  if (d_in <= 0 || d_out <= 0 || w_ld <= 0) return SMLM_ERR_ARG;
  if ((d_in & 7) || (d_out & 7) || (w_ld & 7)) return SMLM_ERR_ALIGN;
  if (w_ld < (w_row_major ? d_out : d_in)) return SMLM_ERR_ARG;
  if (T == 0 || S == 0) return SMLM_OK;
  if (!y || !x || !w_ptrs || !plan || !workspace) return SMLM_ERR_ARG;
  if (!aligned16(y) || !aligned16(x) || !aligned16(workspace) || !aligned16(plan))
    return SMLM_ERR_ALIGN;
  size_t need = 0;
  rc = smlm_gemm_planned_workspace_size(T, d_in, d_out, &need);
  if (rc) return rc;
  if (workspace_bytes < need) return SMLM_ERR_WORKSPACE;

  hipStream_t st = (hipStream_t)stream;
  PlanView pv;
  plan_carve(const_cast<void*>(plan), T, S, &pv);

  if (d_in < d_out) {  // the reference's "expand" branch (smlm_forward_cutlass.cuh:82)
    ExpandArgs a{};
    a.plan = tile_args(pv, n_weights);
    a.seg_scale = seg_scale;
    a.beta = beta;
    a.T = T; a.nt_max = pv.nt_max;
    ExpandProj& P = a.p[0];
    P.y = reinterpret_cast<uint16_t*>(y);
    P.v = reinterpret_cast<const uint16_t*>(x);
    P.w_ptrs = w_ptrs;
    P.d_in = d_in; P.d_out = d_out; P.ldw = w_ld;
    // Row-major weights (element (k, n) at w[k * w_ld + n]) are the [k][n] layout the tile-block kernels read
    // as it lies (as the backward's dX = dV A does): up to a contraction of 64 they run at every size, as
    // they do for the backward; longer ones keep the one-tile kernel's strided reads.
    if (w_row_major && d_in <= 64) {
      a.w_kn = 1;
      return launch_expand(dtype, false, expand_nq(T, d_out), kBlkTiles, S, n_weights, 1, d_in, st, a);
    }
    return launch_expand(dtype, w_row_major != 0, expand_nq(T, d_out), tiles_per_wave(T, d_in), S, n_weights,
                         1, d_in, st, a);
  }
  float* partial = reinterpret_cast<float*>(workspace);
  if (w_row_major)  // the tile-block shrink stages [k][n] weights as they lie (as the backward's dV = dY B does)
    return run_shrink(dtype, false, pv, T, S, n_weights, 1, &x, &w_ptrs, &partial, &y, &d_in, d_out, &w_ld, beta,
                      seg_scale, kBlkTiles, st, true, true);
  return run_shrink(dtype, false, pv, T, S, n_weights, 1, &x, &w_ptrs, &partial, &y, &d_in,
                    d_out, &w_ld, beta, seg_scale, tiles_per_wave(T, d_out), st);
}

SMLM_API int smlm_gemm_workspace_size(int T, int S, int d_in, int d_out, size_t* bytes) {
  if (T < 0 || S < 0 || d_in <= 0 || d_out <= 0 || !bytes) return SMLM_ERR_ARG;
  if (S >= kMaxSegments || T > (1 << 30)) return SMLM_ERR_LIMIT;
  size_t extra = 0;
  int rc = smlm_gemm_planned_workspace_size(T, d_in, d_out, &extra);
  if (rc) return rc;
  *bytes = plan_carve(nullptr, T, S, nullptr) + extra;
  return SMLM_OK;
}

SMLM_API int smlm_gemm(void* y, const void* x, const void* const* w_ptrs, const int32_t* seg_indptr,
                       void* workspace, size_t workspace_bytes, int T, int S, int d_in, int d_out,
                       int w_ld, int w_row_major, int dtype, float beta, const float* seg_scale,
                       void* stream) {
  int rc = check_common(T, S, dtype);
  if (rc) return rc;
  if (d_in <= 0 || d_out <= 0 || w_ld <= 0) return SMLM_ERR_ARG;
  if ((d_in & 7) || (d_out & 7) || (w_ld & 7)) return SMLM_ERR_ALIGN;
  if (w_ld < (w_row_major ? d_out : d_in)) return SMLM_ERR_ARG;
  if (T == 0 || S == 0) return SMLM_OK;
  if (!y || !x || !w_ptrs || !seg_indptr || !workspace) return SMLM_ERR_ARG;
  if (!aligned16(y) || !aligned16(x) || !aligned16(workspace)) return SMLM_ERR_ALIGN;
  size_t need = 0;
  rc = smlm_gemm_workspace_size(T, S, d_in, d_out, &need);
  if (rc) return rc;
  if (workspace_bytes < need) return SMLM_ERR_WORKSPACE;

  hipStream_t st = (hipStream_t)stream;
  PlanView pv;
  const size_t plan_bytes = plan_carve(workspace, T, S, &pv);
  // The plan groups the segments by their weight address.  A product that runs on the shrink kernels
  // (d_in >= d_out, weights [n][k]) over few enough segments builds it inside its own launch: every
  // workgroup numbers the addresses by their first occurrence and finds its tile itself, a few more
  // write the plan for the fold launch behind it (as the fused forward does with adapter ids).
  const int mt = tiles_per_wave(T, d_out);
  const int nw = shrink_waves(mt, 1, &d_in, d_out);
  const int ks = shrink_cfg(T, d_in, d_out, nw, false, mt).ksplit;
  const bool in_launch = d_in >= d_out && !w_row_major && self_planned_ok(T, S, S, pv.nt_max, mt) &&
                         (mt > 1 ? (S <= kFwdThreads || ks % 2 == 0)
                                 : (nw == kDecodeWaves && (S <= kSelfPlanThreads || ks % 2 == 0)));
  if (in_launch) {
    if (!aligned16(y) || !aligned16(x)) return SMLM_ERR_ALIGN;
    const PlanSortArgs build{pv, seg_indptr, w_ptrs, SMLM_KEY_PTR2, S, next_pow2(S), w_ptrs};
    float* partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + plan_bytes);
    return run_shrink(dtype, false, pv, T, S, S, 1, &x, &w_ptrs, &partial, &y, &d_in, d_out, &w_ld, beta,
                      seg_scale, mt, st, true, false, nullptr, nullptr, 0, &build);
  }
  rc = plan_build_impl(pv, seg_indptr, w_ptrs, SMLM_KEY_PTR, S, st);
  if (rc) return rc;
  return smlm_gemm_planned(y, x, w_ptrs, S, workspace, reinterpret_cast<char*>(workspace) + plan_bytes,
                           workspace_bytes - plan_bytes, T, S, d_in, d_out, w_ld, w_row_major, dtype,
                           beta, seg_scale, stream);
}

SMLM_API int smlm_gemm_static(void* y, const void* x, const void* const* w_ptrs,
                              const int32_t* seg_indptr, int T, int S, int d_in, int d_out, int w_ld,
                              int w_row_major, int dtype, float beta, const float* seg_scale,
                              void* stream) {
  int rc = check_common(T, S, dtype);
  if (rc) return rc;
  if (d_in <= 0 || d_out <= 0) return SMLM_ERR_ARG;
  size_t need = 0;
  if ((rc = smlm_gemm_workspace_size(T, S, d_in, d_out, &need))) return rc;
  if (need > SMLM_STATIC_SCRATCH_BYTES) return SMLM_ERR_SCRATCH;
  // an empty batch launches nothing (smlm_gemm validates the rest and returns): no device needed
  void* ws = (T == 0 || S == 0) ? nullptr : static_scratch();
  if (!ws && T != 0 && S != 0) return SMLM_ERR_LAUNCH;
  return smlm_gemm(y, x, w_ptrs, seg_indptr, ws, SMLM_STATIC_SCRATCH_BYTES, T, S, d_in, d_out, w_ld,
                   w_row_major, dtype, beta, seg_scale, stream);
}

SMLM_API int smlm_lora_fwd_multi_workspace_size(int n_proj, int T, const int* h_in, int r,
                                                size_t* bytes) {
  if (n_proj < 1 || n_proj > kMaxProj || T < 0 || !h_in || r <= 0 || !bytes) return SMLM_ERR_ARG;
  size_t n = 0;
  for (int i = 0; i < n_proj; ++i) {
    if (h_in[i] <= 0) return SMLM_ERR_ARG;
    const size_t rows = T > 0 ? T : 1;
    n += align_up((size_t)fwd_ksplit_bound(T, h_in[i], r) * rows * r * 4, 256) + align_up(rows * r * 2, 256);
  }
  *bytes = n;
  return SMLM_OK;
}

// the library's view of the caller's dropout descriptor; nullptr or seg_p == nullptr: none
static int drop_args(const smlm_dropout* d, DropArgs* out) {
  *out = DropArgs{};
  if (!d || !d->seg_p) return SMLM_OK;
  if (d->rows < 0) return SMLM_ERR_ARG;
  out->seg_p = d->seg_p;
  out->rows = d->rows;
  out->k0 = (uint32_t)d->seed; out->k1 = (uint32_t)(d->seed >> 32);
  out->o0 = (uint32_t)d->offset; out->o1 = (uint32_t)(d->offset >> 32);
  out->bits = reinterpret_cast<uint8_t*>(d->mask_bits);
  return SMLM_OK;
}

SMLM_API int smlm_lora_fwd_multi(int n_proj, void* const* y, const void* const* x,
                                 void* const* v_out, const void* const* const* a_ptrs,
                                 const void* const* const* b_ptrs, int n_weights, const int* h_in,
                                 const int* h_out, const void* plan, void* workspace,
                                 size_t workspace_bytes, int T, int S, int r, int dtype, float beta,
                                 const float* seg_scale, int stages, void* stream) {
  return smlm_lora_fwd_multi_ex(n_proj, y, x, v_out, a_ptrs, b_ptrs, n_weights, h_in, h_out, plan,
                                workspace, workspace_bytes, T, S, r, dtype, beta, seg_scale, stages,
                                nullptr, stream);
}

SMLM_API int smlm_lora_fwd_multi_ex(int n_proj, void* const* y, const void* const* x,
                                    void* const* v_out, const void* const* const* a_ptrs,
                                    const void* const* const* b_ptrs, int n_weights,
                                    const int* h_in, const int* h_out, const void* plan,
                                    void* workspace, size_t workspace_bytes, int T, int S, int r,
                                    int dtype, float beta, const float* seg_scale, int stages,
                                    const smlm_lora_opts* opts, void* stream) {
  int rc = check_common(T, S, dtype);
  if (rc) return rc;
  DropArgs drop;
  if ((rc = drop_args(opts ? opts->dropout : nullptr, &drop))) return rc;
  const int32_t* w_rank = opts ? opts->adapter_rank : nullptr;
  const int packed = (opts && opts->adapter_rank) ? opts->packed_ranks : 0;
  const int32_t* build_s = opts ? opts->build_seg_indptr : nullptr;
  const void* build_k = opts ? opts->build_seg_adapter : nullptr;
  const void* build_k2 = nullptr;
  int build_kind = SMLM_KEY_I32;
  if (opts && (opts->build_seg_key_a || opts->build_seg_key_b)) {  // grouped by pairs of addresses instead of ids
    if (build_k || !opts->build_seg_key_a || !opts->build_seg_key_b) return SMLM_ERR_ARG;
    build_k = opts->build_seg_key_a;
    build_k2 = opts->build_seg_key_b;
    build_kind = SMLM_KEY_PTR2;
  }
  if ((build_s != nullptr) != (build_k != nullptr)) return SMLM_ERR_ARG;
  if (build_s && !(stages & SMLM_STAGE_SHRINK)) return SMLM_ERR_ARG;  // the plan is built with the shrink
  if (n_proj < 1 || n_proj > kMaxProj || r <= 0 || !y || !x || !a_ptrs || !b_ptrs || !h_in || !h_out)
    return SMLM_ERR_ARG;
  if (stages < 1 || stages > (SMLM_STAGE_SHRINK | SMLM_STAGE_EXPAND)) return SMLM_ERR_ARG;
  if (r & 7) return SMLM_ERR_ALIGN;
  for (int i = 0; i < n_proj; ++i) {
    if (h_in[i] <= 0 || h_out[i] <= 0) return SMLM_ERR_ARG;
    if ((h_in[i] & 7) || (h_out[i] & 7)) return SMLM_ERR_ALIGN;
  }
  if (T == 0 || S == 0) return SMLM_OK;
  if (!plan || !workspace) return SMLM_ERR_ARG;
  if (!aligned16(workspace) || !aligned16(plan)) return SMLM_ERR_ALIGN;
  // A call that runs one stage only need not name what the other stage works on: a shrink-only
  // call no y, an expand-only call no x -- and an expand-only call skips the projections whose y
  // is NULL (the projections of one shrink call may be expanded one at a time, each when its y
  // is ready).
  const bool shrink_only = stages == SMLM_STAGE_SHRINK, expand_only = stages == SMLM_STAGE_EXPAND;
  for (int i = 0; i < n_proj; ++i) {
    if (!a_ptrs[i] || !b_ptrs[i]) return SMLM_ERR_ARG;
    if ((!y[i] && !shrink_only && !expand_only) || (!x[i] && !expand_only)) return SMLM_ERR_ARG;
    if (!aligned16(y[i]) || !aligned16(x[i]) || (v_out && v_out[i] && !aligned16(v_out[i])))
      return SMLM_ERR_ALIGN;
  }
  size_t need = 0;
  rc = smlm_lora_fwd_multi_workspace_size(n_proj, T, h_in, r, &need);
  if (rc) return rc;
  if (workspace_bytes < need) return SMLM_ERR_WORKSPACE;

  hipStream_t st = (hipStream_t)stream;
  PlanView pv;
  plan_carve(const_cast<void*>(plan), T, S, &pv);

  // shrink: every projection's v, rounded to 16 bits (into v_out when the caller wants it).
  // Decode batches (eight-wave shrink, one-tile expand) skip the fold launch: the expand
  // kernel adds the few partials while it loads v.
  float* partial[kMaxProj];
  void* v16[kMaxProj];
  int vsplit[kMaxProj];
  const int mt = tiles_per_wave(T, r);
  const int nw = shrink_waves(mt, n_proj, h_in, r);
  bool expand_folds = nw == kDecodeWaves && mt == 1;
  {
    char* w = reinterpret_cast<char*>(workspace);
    for (int i = 0; i < n_proj; ++i) {
      vsplit[i] = shrink_cfg(T, h_in[i], r, nw, false, mt).ksplit;
      expand_folds = expand_folds && vsplit[i] <= kMaxExpandFold;
      partial[i] = reinterpret_cast<float*>(w);
      w += align_up((size_t)fwd_ksplit_bound(T, h_in[i], r) * T * r * 4, 256);
      v16[i] = (v_out && v_out[i]) ? v_out[i] : w;
      w += align_up((size_t)T * r * 2, 256);
    }
  }
  // A plan still to be built (opts->build_*): decode batches build it inside the shrink launch,
  // every other batch with the plan launch first.
  PlanSortArgs build{pv, build_s, build_k, build_kind, S, next_pow2(S), build_k2};
  bool even_splits = true;  // (the decode route pairs k slices up beyond 512 segments)
  for (int i = 0; i < n_proj; ++i) even_splits = even_splits && (vsplit[i] % 2 == 0);
  // (both routes pair k slices up in one workgroup beyond 512 / 256 segments)
  const bool self_planned = build_s && !drop.seg_p && self_planned_ok(T, S, n_weights, pv.nt_max, mt) &&
                            (mt > 1 ? (S <= kFwdThreads || even_splits)
                                                   : (expand_folds && (S <= kSelfPlanThreads || even_splits)));
  if (build_s && !self_planned && (rc = plan_build_impl(pv, build_s, build_k, build_kind, S, st, build_k2))) return rc;
  if (stages & SMLM_STAGE_SHRINK) {
    rc = run_shrink(dtype, false, pv, T, S, n_weights, n_proj, x, a_ptrs, partial, v16, h_in, r, h_in,
                    0.0f, nullptr, mt, st, !expand_folds, false, &drop, w_rank, packed,
                    self_planned ? &build : nullptr);
    if (rc) return rc;
  }
  if (!(stages & SMLM_STAGE_EXPAND)) return SMLM_OK;

  ExpandArgs ea{};
  ea.plan = tile_args(pv, n_weights);
  ea.plan.w_rank = w_rank;
  ea.plan.packed = packed;
  ea.seg_scale = seg_scale;
  ea.beta = beta;
  ea.T = T; ea.nt_max = pv.nt_max;
  int n_exp = 0, exp_h_out = 0;  // an expand-only call launches only the projections it names a y for
  for (int i = 0; i < n_proj; ++i) {
    if (!y[i]) continue;
    ExpandProj& P = ea.p[n_exp++];
    P.y = reinterpret_cast<uint16_t*>(y[i]);
    P.v = reinterpret_cast<const uint16_t*>(v16[i]);
    P.w_ptrs = b_ptrs[i];
    P.d_in = r; P.d_out = h_out[i]; P.ldw = r;
    if (h_out[i] > exp_h_out) exp_h_out = h_out[i];
    if (expand_folds) {
      P.vpart = partial[i];
      P.vsplit = vsplit[i];
      // the rounded v exists only inside the expand kernel: it writes the caller's copy
      if (v_out && v_out[i]) P.v_out = reinterpret_cast<uint16_t*>(v_out[i]);
    }
  }
  if (n_exp == 0) return SMLM_OK;
  return launch_expand(dtype, false, expand_nq(T, exp_h_out), mt, S, n_weights, n_exp, r, st, ea);
}

SMLM_API int smlm_lora_fwd_workspace_size(int T, int S, int h_in, int h_out, int r, size_t* bytes) {
  if (S < 0 || h_out <= 0) return SMLM_ERR_ARG;
  return smlm_lora_fwd_multi_workspace_size(1, T, &h_in, r, bytes);
}

SMLM_API int smlm_lora_fwd(void* y, const void* x, void* v_out, const void* const* a_ptrs,
                           const void* const* b_ptrs, int n_weights, const void* plan, void* workspace,
                           size_t workspace_bytes, int T, int S, int h_in, int h_out, int r, int dtype,
                           float beta, const float* seg_scale, void* stream) {
  return smlm_lora_fwd_multi(1, &y, &x, v_out ? &v_out : nullptr, &a_ptrs, &b_ptrs, n_weights, &h_in,
                             &h_out, plan,
                             workspace, workspace_bytes, T, S, r, dtype, beta, seg_scale,
                             SMLM_STAGE_SHRINK | SMLM_STAGE_EXPAND, stream);
}

SMLM_API int smlm_lora_bwd_multi_workspace_size(int n_proj, int n_rows, int P, int NA, const int* h_in,
                                                const int* h_out, int r, size_t* bytes) {
  if (n_proj < 1 || n_proj > kMaxProj || n_rows < 0 || P < 0 || NA < 0 || !h_in || !h_out || r <= 0 || !bytes)
    return SMLM_ERR_ARG;
  for (int i = 0; i < n_proj; ++i)
    if (h_in[i] <= 0 || h_out[i] <= 0) return SMLM_ERR_ARG;
  *bytes = bwd_layout(n_proj, n_rows > 0 ? n_rows : 1, P, NA > 0 ? NA : 1, h_in, h_out, r).total;
  return SMLM_OK;
}

SMLM_API int smlm_lora_bwd_workspace_size(int n_rows, int P, int NA, int h_in, int h_out, int r,
                                          size_t* bytes) {
  return smlm_lora_bwd_multi_workspace_size(1, n_rows, P, NA, &h_in, &h_out, r, bytes);
}

SMLM_API int smlm_lora_bwd(void* dx, void* const* da_ptrs, void* const* db_ptrs, const void* dy,
                           const void* x, const void* v, const void* const* a_ptrs,
                           const void* const* b_ptrs, const void* plan, void* workspace,
                           size_t workspace_bytes, int n_rows, int P, int NA, int h_in, int h_out,
                           int r, int dtype, const float* part_scale, void* stream) {
  return smlm_lora_bwd_ex(dx, da_ptrs, db_ptrs, dy, x, v, a_ptrs, b_ptrs, plan, workspace,
                          workspace_bytes, n_rows, P, NA, h_in, h_out, r, dtype, part_scale, nullptr, stream);
}

SMLM_API int smlm_lora_bwd_ex(void* dx, void* const* da_ptrs, void* const* db_ptrs,
                              const void* dy, const void* x, const void* v,
                              const void* const* a_ptrs, const void* const* b_ptrs,
                              const void* plan, void* workspace, size_t workspace_bytes,
                              int n_rows, int P, int NA, int h_in, int h_out, int r, int dtype,
                              const float* part_scale, const smlm_lora_opts* opts, void* stream) {
  return smlm_lora_bwd_multi_ex(1, &dx, &da_ptrs, &db_ptrs, &dy, &x, v ? &v : nullptr, &a_ptrs, &b_ptrs, plan,
                                workspace, workspace_bytes, n_rows, P, NA, &h_in, &h_out, r, dtype, part_scale,
                                opts, stream);
}

// every projection's dV product is folded from k-split partials: the fold then writes what the weight gradients read
static bool bwd_all_folded(int n_proj, int n_rows, const int* h_out, int r) {
  const int mt = bwd_tiles_per_wave(n_rows, r);
  const int nw = shrink_waves(mt, n_proj, h_out, r);
  for (int i = 0; i < n_proj; ++i)
    if (shrink_cfg(n_rows, h_out[i], r, nw, true, mt).ksplit <= 1) return false;
  return true;
}

SMLM_API int smlm_lora_bwd_multi_ex(int n_proj, void* const* dx, void* const* const* da_ptrs,
                                    void* const* const* db_ptrs, const void* const* dy,
                                    const void* const* x, const void* const* v,
                                    const void* const* const* a_ptrs, const void* const* const* b_ptrs,
                                    const void* plan, void* workspace, size_t workspace_bytes,
                                    int n_rows, int P, int NA, const int* h_in, const int* h_out, int r,
                                    int dtype, const float* part_scale, const smlm_lora_opts* opts,
                                    void* stream) {
  int rc = check_common(n_rows, P, dtype);
  if (rc) return rc;
  DropArgs drop;
  if ((rc = drop_args(opts ? opts->dropout : nullptr, &drop))) return rc;
  const int32_t* w_rank = opts ? opts->adapter_rank : nullptr;
  const int packed = (opts && opts->adapter_rank) ? opts->packed_ranks : 0;
  const int stages = (opts && opts->bwd_stages) ? opts->bwd_stages : (SMLM_BWD_PRODUCTS | SMLM_BWD_DX | SMLM_BWD_WGRAD);
  // the other weight layout (the reference's is_row_major = True): A_a [h_in, r], B_a [r, h_out], and so are dA_a, dB_a
  const bool rm = opts && opts->w_row_major;
  const int dx_rows = opts ? opts->dx_rows : 0;
  if (dx_rows != 0 && dx_rows < n_rows) return SMLM_ERR_ARG;
  if (rm && (drop.seg_p || packed)) return SMLM_ERR_ARG;
  if (stages < 0 || stages > (SMLM_BWD_PRODUCTS | SMLM_BWD_DX | SMLM_BWD_WGRAD)) return SMLM_ERR_ARG;
  if (n_proj < 1 || n_proj > kMaxProj || NA < 0 || r <= 0 || !h_in || !h_out) return SMLM_ERR_ARG;
  if (r & 7) return SMLM_ERR_ALIGN;
  if (NA == 0 || n_rows == 0 || P == 0) return SMLM_ERR_ARG;
  if (!dx || !da_ptrs || !db_ptrs || !dy || !x || !a_ptrs || !b_ptrs || !workspace || !plan) return SMLM_ERR_ARG;
  if (!aligned16(workspace) || !aligned16(plan)) return SMLM_ERR_ALIGN;
  bool have_v = v != nullptr && v[0] != nullptr;
  for (int i = 0; i < n_proj; ++i) {
    if (h_in[i] <= 0 || h_out[i] <= 0) return SMLM_ERR_ARG;
    if ((h_in[i] & 7) || (h_out[i] & 7)) return SMLM_ERR_ALIGN;
    if (!da_ptrs[i] || !db_ptrs[i] || !a_ptrs[i] || !b_ptrs[i] || !dx[i] || !dy[i] || !x[i]) return SMLM_ERR_ARG;
    if (have_v != (v != nullptr && v[i] != nullptr)) return SMLM_ERR_ARG;  // v of every projection or of none
    if (!aligned16(dx[i]) || !aligned16(dy[i]) || !aligned16(x[i]) || (have_v && !aligned16(v[i])))
      return SMLM_ERR_ALIGN;
  }
  const BwdLayout L = bwd_layout(n_proj, n_rows, P, NA, h_in, h_out, r);
  if (workspace_bytes < L.total) return SMLM_ERR_WORKSPACE;

  hipStream_t st = (hipStream_t)stream;
  char* ws = reinterpret_cast<char*>(workspace);
  PlanView pv{};
  plan_carve(const_cast<void*>(plan), n_rows, P, &pv);

  // A plan still to be built (opts->build_*): the dV shrink builds it inside its launch when it is
  // the first launch to use it (tile-block route, v given, no dropout); else the plan launch first.
  const int32_t* build_s = opts ? opts->build_seg_indptr : nullptr;
  const int32_t* build_k = opts ? opts->build_seg_adapter : nullptr;
  if ((build_s != nullptr) != (build_k != nullptr)) return SMLM_ERR_ARG;
  if (build_s && !(stages & SMLM_BWD_PRODUCTS)) return SMLM_ERR_ARG;  // the plan is built with the first stage
  PlanSortArgs build{pv, build_s, build_k, SMLM_KEY_I32, P, next_pow2(P)};
  const int mt = bwd_tiles_per_wave(n_rows, r);
  bool even_dv = true;  // (k slices in pairs beyond 256 partitions)
  for (int i = 0; i < n_proj; ++i) even_dv = even_dv && shrink_cfg(n_rows, h_out[i], r, kFwdWaves, true, mt).ksplit % 2 == 0;
  const bool self_planned = build_s && have_v && !drop.seg_p && mt > 1 && r <= 64 &&
                            self_planned_ok(n_rows, P, NA, pv.nt_max, mt) && (P <= kFwdThreads || even_dv);
  const bool products = (stages & SMLM_BWD_PRODUCTS) != 0;
  if (build_s && !self_planned && (rc = plan_build_impl(pv, build_s, build_k, SMLM_KEY_I32, P, st))) return rc;

  // 1. The backward multiplies by B and A where the forward multiplies by A^T and B^T.  The
  // tile-block kernels read the weights as they lie in memory; ranks above 64 take the one-tile
  // expand kernel's general k loop, which reads [n][k] weights: transposed copies At [h_in, r],
  // Bt [r, h_out] made here.
  // (The row-major layout needs no copies at any rank: dV = dY B^T and dX = dV A^T read B [r, h_out] and
  // A [h_in, r] the way the forward reads A [r, h_in] and B [h_out, r], and v = x A reads A as [k][n].)
  const bool in_place = rm || (mt > 1 && r <= 64);
  if (!in_place && products) {
    for (int i = 0; i < n_proj; ++i) {
      TransposeArgs ta{};
      ta.set[0] = TransposeSet{a_ptrs[i], reinterpret_cast<uint16_t*>(ws + L.p[i].at),
                               reinterpret_cast<const void**>(ws + L.p[i].at_ptrs), (long)h_in[i] * r, r, h_in[i]};
      ta.set[1] = TransposeSet{b_ptrs[i], reinterpret_cast<uint16_t*>(ws + L.p[i].bt),
                               reinterpret_cast<const void**>(ws + L.p[i].bt_ptrs), (long)h_out[i] * r, h_out[i], r};
      ta.NA = NA;
      ta.w_rank = w_rank;
      ta.packed = packed;
      const int gx = ceil_div(h_in[i] > h_out[i] ? h_in[i] : h_out[i], 64), gy = ceil_div(r, 64);
      if ((rc = launch(transpose_kernel, dim3(gx, gy, 2 * NA), dim3(256), st, ta))) return rc;
    }
  }

  // The keep bits of x's dropout mask (projection i: the stream offset + i; the caller's bits of the
  // projections lie end to end): the forward's when the caller kept them, else made here (same stream,
  // same bits) so that the kernels below apply a stored mask either way.
  const uint8_t* bits[kMaxProj] = {};
  if (drop.seg_p) {
    size_t bits_off = 0;
    for (int i = 0; i < n_proj; ++i) {
      if (drop.bits) {
        bits[i] = drop.bits + bits_off;
        bits_off += (size_t)drop.rows * (h_in[i] / 8);
      } else {
        DropArgs di = drop;
        const uint64_t off = (((uint64_t)drop.o1 << 32) | drop.o0) + (uint32_t)i;
        di.o0 = (uint32_t)off; di.o1 = (uint32_t)(off >> 32);
        di.bits = reinterpret_cast<uint8_t*>(ws + L.p[i].bits);
        di.bits_pitch = h_in[i] / 8;
        bits[i] = di.bits;
        const DropBitsArgs ba{pv.hdr, pv.tile_row, pv.tile_rseg, di};
        if (products && (rc = launch(drop_bits_kernel, dim3((unsigned)pv.nt_max), dim3(256), st, ba))) return rc;
      }
    }
  }

  float* partial[kMaxProj];
  void* dv16[kMaxProj];
  void* v16[kMaxProj];
  const void* vv[kMaxProj];
  for (int i = 0; i < n_proj; ++i) {
    partial[i] = reinterpret_cast<float*>(ws + L.p[i].partial);
    dv16[i] = ws + L.p[i].dv16;
    v16[i] = ws + L.p[i].v16;
    vv[i] = have_v ? v[i] : v16[i];
  }

  // 2. v = round16(x A^T) unless the forward saved it
  if (!have_v && products) {
    DropArgs vdrop = drop;
    vdrop.bits = nullptr;  // the shrink kernels run the generator themselves; nothing to store here
    if (rm) {  // A [h_in, r] is [k][n]: the tile-block shrink at every size
      int a_ld[kMaxProj];
      for (int i = 0; i < n_proj; ++i) a_ld[i] = r;
      if ((rc = run_shrink(dtype, false, pv, n_rows, P, NA, n_proj, x, a_ptrs, partial, v16, h_in, r, a_ld, 0.0f,
                           nullptr, kBlkTiles, st, true, true, nullptr, w_rank, 0, nullptr, true)))
        return rc;
    } else if ((rc = run_shrink(dtype, false, pv, n_rows, P, NA, n_proj, x, a_ptrs, partial, v16, h_in, r, h_in,
                                0.0f, nullptr, mt, st, true, false, &vdrop, w_rank, 0, nullptr, true)))  // v of the dropped x, as the forward made it
      return rc;
  }

  // 3. dV = round16(dY B)
  const void* const* btp[kMaxProj];
  int b_ld[kMaxProj];
  for (int i = 0; i < n_proj; ++i) {
    btp[i] = in_place ? b_ptrs[i] : reinterpret_cast<const void* const*>(ws + L.p[i].bt_ptrs);
    b_ld[i] = (in_place && !rm) ? r : h_out[i];  // B [h_out, r] read as [k][n]; B [r, h_out] and the copies as [n][k]
  }
  // The weight gradients read s*dV and s*v by tile slot, transposed.  The fold of dV leaves them behind when there is
  // one for every projection (cheaper there than among dX's stores: cfg4-like batch dV 12.5 -> 13.5, dX 10.8 -> 8.2 us;
  // ragged 32-row partitions over six projections dV 84 -> 91, dX 90 -> 74 us); else dX's launch writes them.
  // (With them out of dX's launch, dX and the weight gradients need nothing of each other.  Issuing the weight
  // gradients on a second stream, forked after the fold and joined at the end, was measured under graph replay and
  // dropped: the two launches did not overlap to any gain and the fork and join cost 6 us.)
  SideOut side{};
  for (int i = 0; i < n_proj; ++i) {
    side.pt_a[i] = reinterpret_cast<uint16_t*>(ws + L.p[i].pt_a);
    side.pt_b[i] = reinterpret_cast<uint16_t*>(ws + L.p[i].pt_b);
    side.v2[i] = reinterpret_cast<const uint16_t*>(vv[i]);
  }
  side.scale = part_scale;
  side.pitch = L.pitch;
  // rows of dX past the backward's own (opts->dx_rows): cleared by the fold's launch when it runs in direct mode,
  // else by a launch of their own
  ZeroSpans tail{};
  if (dx_rows > n_rows) {
    for (int i = 0; i < n_proj; ++i) {
      tail.ptr[i] = reinterpret_cast<char*>(dx[i]) + (size_t)n_rows * h_in[i] * 2;
      tail.bytes[i] = (long)(dx_rows - n_rows) * h_in[i] * 2;  // (h_in is a multiple of 8: whole 16-byte pieces)
      tail.first[i + 1] = tail.first[i] + (int)((tail.bytes[i] + kZeroBlockBytes - 1) / kZeroBlockBytes);
    }
    tail.n = n_proj;
  }
  // (a function of the shapes and the option: the same in every call of a staged backward)
  const bool side_in_fold = bwd_all_folded(n_proj, n_rows, h_out, r);
  if (side_in_fold) side.zero = tail;
  else if (tail.n && products &&
           (rc = launch(zero_spans_kernel, dim3((unsigned)tail.first[tail.n]), dim3(256), st, tail)))
    return rc;
  bool side_done = false;
  if (products && (rc = run_shrink(dtype, false, pv, n_rows, P, NA, n_proj, dy, btp, partial, dv16, h_out, r, b_ld,
                                   0.0f, nullptr, mt, st, true, in_place && !rm, nullptr, w_rank, in_place ? packed : 0,
                                   self_planned ? &build : nullptr, true, side_in_fold ? &side : nullptr, &side_done)))
    return rc;  // (B in place is read at its stored rank; the transposed copies keep the full-rank strides)
  if (products && side_done != side_in_fold) return SMLM_ERR_ARG;  // (cannot happen: both follow shrink_cfg)

  // 4. dX = s dV A, and the slot-ordered transposed s*dV, s*v for step 5
  ExpandArgs ea{};
  ea.plan = tile_args(pv, NA);
  ea.plan.w_rank = w_rank;
  ea.seg_scale = part_scale;
  ea.beta = 0.0f;
  ea.T = n_rows; ea.nt_max = pv.nt_max;
  int widest = 0;
  for (int i = 0; i < n_proj; ++i) {
    ExpandProj& E = ea.p[i];
    E.y = reinterpret_cast<uint16_t*>(dx[i]);
    E.v = reinterpret_cast<const uint16_t*>(dv16[i]);
    E.w_ptrs = in_place ? a_ptrs[i] : reinterpret_cast<const void* const*>(ws + L.p[i].at_ptrs);
    E.d_in = r; E.d_out = h_in[i]; E.ldw = (in_place && !rm) ? h_in[i] : r;  // A [r, h_in] as [k][n]; A [h_in, r] as [n][k]
    E.pt_a = side_in_fold ? nullptr : side.pt_a[i];
    E.pt_b = side_in_fold ? nullptr : side.pt_b[i];
    E.v2 = side.v2[i];
    E.drop_bits = bits[i];
    E.drop_pitch = h_in[i] / 8;
    if (h_in[i] > widest) widest = h_in[i];
  }
  ea.w_kn = (in_place && !rm) ? 1 : 0;
  ea.drop = drop;  // dX is the gradient with respect to x before its dropout
  if ((stages & SMLM_BWD_DX) && (rc = launch_expand(dtype, false, expand_nq(n_rows, widest), mt, P, NA, n_proj, r, st, ea)))
    return rc;
  if (!(stages & SMLM_BWD_WGRAD)) return SMLM_OK;

  // 5. dA_a, dB_a for every adapter (zeros when it has no rows)
  WgradArgs wa{};
  wa.hdr = pv.hdr;
  wa.grp_tile = pv.grp_tile;
  wa.grp_id = pv.grp_id;
  wa.tile_row = pv.tile_row;
  wa.nproj = n_proj;
  // four waves splitting the rows of an adapter pay off when adapters have many rows each (whole backward,
  // 16 adapters at rank 16 / 64: 1024 rows each 124.7 -> 118.7 / 180.7 -> 175.3 us, 512 rows even, 256 rows
  // 43.5 -> 44.6 / 62.1 -> 67.3 us, 64 rows 25.7 -> 30.8 / 33.7 -> 46.5 us)
  const bool split = n_rows / NA >= 512;
  // one-wave workgroups take several neighbouring chunks in turn when there are chunks enough to keep the
  // chip busy anyway: about 8192 workgroups are left
  long all_chunks = 0;
  for (int i = 0; i < n_proj; ++i) all_chunks += ceil_div(h_in[i], kWgCols) + ceil_div(h_out[i], kWgCols);
  int walk = 1;
  if (!split) {
    const long want = all_chunks * NA * ceil_div(r, 64) / 8192;
    walk = want < 1 ? 1 : (want > 8 ? 8 : (int)want);
  }
  wa.walk = walk;
  int units = 0;
  for (int i = 0; i < n_proj; ++i) {
    WgradProj& Q = wa.p[i];
    Q.q_a = reinterpret_cast<const uint16_t*>(x[i]);
    Q.q_b = reinterpret_cast<const uint16_t*>(dy[i]);
    Q.pt_a = reinterpret_cast<const uint16_t*>(ws + L.p[i].pt_a);
    Q.pt_b = reinterpret_cast<const uint16_t*>(ws + L.p[i].pt_b);
    Q.da_ptrs = da_ptrs[i];
    Q.db_ptrs = db_ptrs[i];
    Q.h_in = h_in[i]; Q.h_out = h_out[i];
    if (rm) {
      // dB [r, h_out] = sum (s v)^T dY has the shape the kernel's first product writes ([rank, columns]) and
      // dA [h_in, r] = sum x^T (s dV) the shape of its second ([columns, rank]): the two change places
      Q.q_a = reinterpret_cast<const uint16_t*>(dy[i]);
      Q.q_b = reinterpret_cast<const uint16_t*>(x[i]);
      Q.pt_a = reinterpret_cast<const uint16_t*>(ws + L.p[i].pt_b);
      Q.pt_b = reinterpret_cast<const uint16_t*>(ws + L.p[i].pt_a);
      Q.da_ptrs = db_ptrs[i];
      Q.db_ptrs = da_ptrs[i];
      Q.h_in = h_out[i]; Q.h_out = h_in[i];
    }
    Q.chunks_a = ceil_div(Q.h_in, kWgCols);
    Q.units_a = ceil_div(Q.chunks_a, walk);
    Q.unit0 = units;
    Q.drop_bits = bits[i];
    Q.drop_pitch = h_in[i] / 8;
    units += Q.units_a + ceil_div(ceil_div(Q.h_out, kWgCols), walk);
  }
  wa.pitch = L.pitch;
  wa.r = r;
  wa.n_parts = P;
  wa.grp_seg = pv.grp_seg;
  wa.w_rank = w_rank;
  wa.packed = packed;
  wa.drop = drop;  // dA against the dropped x
  // ranks above 64 are covered 64 at a time along the grid's z axis
  const int nbj = r > 64 ? 4 : ceil_div(r, 16);
  // (along z: 64 ranks a workgroup, or what a dA workgroup of the launched kernel takes when that is less)
  const int z_per_64 = nbj / wgrad_nbj_a(nbj, split ? 4 : 1, drop.seg_p != nullptr);
  dim3 grid(units, NA, ceil_div(r, 64) * z_per_64);
  return dtype == SMLM_DTYPE_F16 ? launch_wgrad<SMLM_DTYPE_F16>(nbj, split, grid, st, wa)
                                 : launch_wgrad<SMLM_DTYPE_BF16>(nbj, split, grid, st, wa);
}

// workgroups of the RMSNorm backward: enough to fill the chip, each with several rows so that
// the partial sums of dw stay small next to x and g
// workgroups of the RMSNorm kernels: the forward gives every row group its own workgroup; the
// backward walks four turns per workgroup (the next rows are fetched while the current ones are
// worked on), so that its partial sums of dw stay small next to x and g
static int rms_blocks(int rows, int cols, bool backward) {
  if (cols > kRmsMaxCols) {  // wide rows: a workgroup per row; the backward's partial rows are whole rows of floats
    const int cap = backward ? 128 : (1 << 22);
    return rows < 1 ? 1 : (rows < cap ? rows : cap);
  }
  const int rows_per_step = cols <= kRmsWaveCols ? 4 : 1;
  int nb = ceil_div(rows, rows_per_step * (backward ? 4 : 1));
  const int cap = backward ? 512 : (1 << 22);
  if (nb > cap) nb = cap;
  return nb < 1 ? 1 : nb;
}
static int rms_bwd_blocks(int rows, int cols) { return rms_blocks(rows, cols, true); }

static int rms_check(int rows, int cols, int dtype) {
  if (rows < 0 || cols <= 0) return SMLM_ERR_ARG;
  if (dtype != SMLM_DTYPE_F16 && dtype != SMLM_DTYPE_BF16) return SMLM_ERR_DTYPE;
  if (cols & 7) return SMLM_ERR_ALIGN;
  if (cols > (1 << 24) || rows > (1 << 30)) return SMLM_ERR_LIMIT;
  return SMLM_OK;
}

SMLM_API int smlm_rms_norm_fwd(void* out, float* rms, const void* x, const void* w, int rows,
                               int cols, float eps, int dtype, void* stream) {
  int rc = rms_check(rows, cols, dtype);
  if (rc) return rc;
  if (rows == 0) return SMLM_OK;
  if (!out || !rms || !x || !w) return SMLM_ERR_ARG;
  if (!aligned16(out) || !aligned16(x) || !aligned16(w)) return SMLM_ERR_ALIGN;
  const RmsFwdArgs a{reinterpret_cast<uint16_t*>(out), rms, reinterpret_cast<const uint16_t*>(x),
                     reinterpret_cast<const uint16_t*>(w), rows, cols, eps};
  hipStream_t st = (hipStream_t)stream;
  const bool f16 = dtype == SMLM_DTYPE_F16;
  const int nb = rms_blocks(rows, cols, false);
  const dim3 grid((unsigned)nb);
  const int rows_per_step = cols <= kRmsWaveCols ? 4 : 1;
  const bool one_turn = (long)nb * rows_per_step >= rows;  // every workgroup sees one row group
  const dim3 bl(256);
  if (cols > kRmsMaxCols)
    return f16 ? launch(rms_fwd_wide_kernel<SMLM_DTYPE_F16>, grid, bl, st, a)
               : launch(rms_fwd_wide_kernel<SMLM_DTYPE_BF16>, grid, bl, st, a);
  if (cols <= kRmsWaveCols) {
    if (one_turn)
      return f16 ? launch(rms_fwd_kernel<SMLM_DTYPE_F16, 1, true>, grid, bl, st, a)
                 : launch(rms_fwd_kernel<SMLM_DTYPE_BF16, 1, true>, grid, bl, st, a);
    return f16 ? launch(rms_fwd_kernel<SMLM_DTYPE_F16, 1, false>, grid, bl, st, a)
               : launch(rms_fwd_kernel<SMLM_DTYPE_BF16, 1, false>, grid, bl, st, a);
  }
  if (one_turn)
    return f16 ? launch(rms_fwd_kernel<SMLM_DTYPE_F16, 4, true>, grid, bl, st, a)
               : launch(rms_fwd_kernel<SMLM_DTYPE_BF16, 4, true>, grid, bl, st, a);
  return f16 ? launch(rms_fwd_kernel<SMLM_DTYPE_F16, 4, false>, grid, bl, st, a)
             : launch(rms_fwd_kernel<SMLM_DTYPE_BF16, 4, false>, grid, bl, st, a);
}

SMLM_API int smlm_rms_norm_bwd_workspace_size(int rows, int cols, size_t* bytes) {
  if (!bytes) return SMLM_ERR_ARG;
  int rc = rms_check(rows, cols, SMLM_DTYPE_F16);
  if (rc) return rc;
  *bytes = align_up((size_t)rms_bwd_blocks(rows > 0 ? rows : 1, cols) * cols * 4, 256);
  return SMLM_OK;
}

SMLM_API int smlm_rms_norm_bwd(void* dx, void* dw, const void* g, const void* x, const void* w,
                               const float* rms, void* workspace, size_t workspace_bytes, int rows,
                               int cols, int dtype, void* stream) {
  int rc = rms_check(rows, cols, dtype);
  if (rc) return rc;
  if (!dx || !dw || !g || !x || !w || !rms || !workspace) return SMLM_ERR_ARG;
  if (!aligned16(dx) || !aligned16(dw) || !aligned16(g) || !aligned16(x) || !aligned16(w) ||
      !aligned16(workspace))
    return SMLM_ERR_ALIGN;
  if (rows == 0) return SMLM_ERR_ARG;  // dw would have nothing to sum
  const int nb = rms_bwd_blocks(rows, cols);
  if (workspace_bytes < (size_t)nb * cols * 4) return SMLM_ERR_WORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  const bool f16 = dtype == SMLM_DTYPE_F16;
  const RmsBwdArgs a{reinterpret_cast<uint16_t*>(dx), reinterpret_cast<float*>(workspace),
                     reinterpret_cast<const uint16_t*>(g), reinterpret_cast<const uint16_t*>(x),
                     reinterpret_cast<const uint16_t*>(w), rms, rows, cols};
  const dim3 grid((unsigned)nb);
  const dim3 bl(256);
  if (cols > kRmsMaxCols)
    rc = f16 ? launch(rms_bwd_wide_kernel<SMLM_DTYPE_F16>, grid, bl, st, a)
             : launch(rms_bwd_wide_kernel<SMLM_DTYPE_BF16>, grid, bl, st, a);
  else if (cols <= kRmsWaveCols)
    rc = f16 ? launch(rms_bwd_kernel<SMLM_DTYPE_F16, 1>, grid, bl, st, a)
             : launch(rms_bwd_kernel<SMLM_DTYPE_BF16, 1>, grid, bl, st, a);
  else
    rc = f16 ? launch(rms_bwd_kernel<SMLM_DTYPE_F16, 4>, grid, bl, st, a)
             : launch(rms_bwd_kernel<SMLM_DTYPE_BF16, 4>, grid, bl, st, a);
  if (rc) return rc;
  const RmsFoldArgs fa{reinterpret_cast<uint16_t*>(dw), reinterpret_cast<const float*>(workspace), nb, cols};
  const dim3 fgrid((unsigned)ceil_div(cols, 64));
  return f16 ? launch(rms_fold_kernel<SMLM_DTYPE_F16>, fgrid, dim3(256), st, fa)
             : launch(rms_fold_kernel<SMLM_DTYPE_BF16>, fgrid, dim3(256), st, fa);
}

SMLM_API int smlm_segments_build(const int32_t* req_adapter, const int32_t* req_len, int R,
                                 int32_t* seg_adapter, int32_t* seg_len, int32_t* seg_indptr,
                                 int32_t* n_seg, void* stream) {
  if (R < 0 || !seg_indptr || !n_seg) return SMLM_ERR_ARG;
  if (R > 0 && (!req_adapter || !req_len || !seg_adapter || !seg_len)) return SMLM_ERR_ARG;
  if (R > kMaxSegments) return SMLM_ERR_LIMIT;
  const SegmentsArgs a{req_adapter, req_len, seg_adapter, seg_len, seg_indptr, n_seg, R};
  return launch(segments_kernel, dim3(1), dim3(kPlanThreads), (hipStream_t)stream, a);
}

}  // extern "C"
