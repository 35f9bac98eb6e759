// Shrink (skinny-N, long-K) and expand (skinny-K, wide-N) tile kernels.
//
// Both take the place of the CUTLASS GemmGrouped instantiations of
// kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:84-171.  The unit of
// work is a 16-row plan tile of one adapter (or a tile block of up to four).
// v_mfma_f32_16x16x32 runs with the tokens as the MFMA *columns* and the weight
// rows as the MFMA *rows*, so a lane ends up with consecutive output columns of
// one token.  x fragments are 16-byte global loads straight into registers (x
// is contiguous along the contraction); weight fragments come straight from
// global memory in the one-tile kernels and from an LDS-staged chunk shared by
// the tiles of a block in the tile-block kernels.
//
// Every output element is produced by the same sequence of MFMA steps over k
// whatever other rows share its tile or its workgroup, so regrouping or
// re-segmenting rows never changes a bit of any row.
//
// The number of tiles is only known on the device (plan header).  Launches are
// sized on the host over an upper bound of it, one work item per workgroup
// ("direct" mode); items past the real count find an empty entry in the plan
// and leave.  A persistent one-dimensional walk over the exact count (one
// contiguous range of items per XCD, or plain round robin) remains as the
// fallback for batches beyond the direct grid's limits.
#pragma once
#include "dropout.hpp"
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
  const int32_t* w_rank;     // optional, indexed like the weight tables: true rank of each adapter
  int packed;                // with w_rank: the weights are STORED at their true rank (rounded up to 8),
                             //   A_a [r_a, h_in], B_a [h_out, r_a], instead of zero-padded to the launch's rank
  int n_weights;             // entries of the caller's weight tables (0: unknown): a tile whose index is not
                             //   below it is left alone, like a tile of a negative adapter id
};

// whether tile index `wid` of a plan names an entry of the caller's weight tables (negative: a segment no
// adapter serves; at or past the table length: an id the caller's tables do not hold -- never dereferenced)
__device__ __forceinline__ bool wid_ok(const TileArgs& p, int wid) {
  return wid >= 0 && (p.n_weights <= 0 || wid < p.n_weights);
}

// Adapters of different ranks live zero-padded to one rank (the reference pads every adapter
// of a layer to the layer's maximum, src/loquetier_src/models/mixed_lora.py:501-521).  With the
// true ranks at hand the padding is not read: loads at or past the rank (rounded up to the
// 8-element load width) are predicated off and read zeros, which is what the padding holds.
__device__ __forceinline__ int rank_limit(const TileArgs& p, int wid, int d) {
  if (!p.w_rank) return d;
  const int r = (uload(p.w_rank, wid) + 7) & ~7;
  return r < d ? r : d;
}
// Leading dimension of a weight matrix whose contiguous dimension is the rank (B [h_out, r], read
// by the expand and by the backward's dV product): the launch's rank for zero-padded storage, the
// adapter's own (rank_limit) for packed storage -- a rank-8 adapter beside rank-64 ones then costs
// 16 bytes a row instead of a 128-byte line.
__device__ __forceinline__ int rank_ld(const TileArgs& p, int ld, int lim) {
  return (p.w_rank && p.packed) ? lim : ld;
}

// Items [first, last) of this workgroup, visited with stride `step`.  The grid
// size is a multiple of kNumXcd.
struct WorkRange {
  int first, last, step;
};
__device__ __forceinline__ WorkRange work_range(int n_work, bool interleave) {
  if (interleave) return WorkRange{(int)blockIdx.x, n_work, (int)gridDim.x};
  const int xcd = blockIdx.x % kNumXcd, local = blockIdx.x / kNumXcd;
  const int base = n_work / kNumXcd, extra = n_work % kNumXcd;
  const int start = xcd * base + (xcd < extra ? xcd : extra);
  const int count = base + (xcd < extra ? 1 : 0);
  return WorkRange{start + local, start + count, (int)gridDim.x / kNumXcd};
}

// Items are numbered (chunk row, tile unit) with the tile unit fastest; the
// chunk rows of all projections are laid end to end (row_start[p] = first chunk
// row of projection p), so there are no empty items to skew the XCD ranges.
// units_max > 0 selects the direct mode used for small launches: one item per
// workgroup, numbered over the host's upper bound of the tile units, so the
// kernel need not wait for the plan header; units past the real count are
// marked empty in the plan (tile_wid < 0, blk == 0).
struct ItemSpace {
  int row_start[kMaxProj + 1];
  int nproj;
  int interleave;  // plain round-robin items instead of one range per XCD
  int units_max;
  int flat;        // direct mode: projections end to end along x instead of on z
};
__device__ __forceinline__ void item_decode(const ItemSpace& sp, int V, int units, int* pj, int* yy,
                                            int* tb) {
  const int cr = V / units;
  *tb = V - cr * units;
  int p = 0;
#pragma unroll
  for (int i = 1; i < kMaxProj; ++i) p += (i < sp.nproj && cr >= sp.row_start[i]) ? 1 : 0;
  *pj = p;
  *yy = cr - sp.row_start[p];
}
// DIRECT launches put the chunk rows on x and the tile units on y.  Chunk rows
// are the fast axis: the workgroups in flight at one time then cover whole
// output rows of a few tile units, which the memory system serves better than a
// few columns of all rows.  The projections are either the z axis (x then spans
// the longest projection and shorter ones leave empty workgroups, but the
// projection's arguments are known at once) or, with `flat`, laid end to end
// along x (row_start; no empty workgroups -- better when the projections differ
// much in width).  (Re-indexing the plane so that the workgroups sharing a
// weight chunk share an XCD's L2 was measured: it removes the repeated weight
// fetches and is no faster, or much slower when it spreads the rows in flight.)
template <bool DIRECT>
__device__ __forceinline__ WorkRange item_range(const ItemSpace& sp, int units) {
  if (DIRECT) return WorkRange{0, 1, 1};
  return work_range(units * sp.row_start[sp.nproj], sp.interleave != 0);
}
template <bool DIRECT>
__device__ __forceinline__ bool item_get(const ItemSpace& sp, int V, int units, int* pj, int* yy,
                                         int* tb) {
  if (DIRECT && !sp.flat) {
    *pj = blockIdx.z;
    *yy = blockIdx.x;
    *tb = blockIdx.y;
    return *yy < sp.row_start[*pj + 1] - sp.row_start[*pj];
  }
  if (DIRECT) {
    const int cr = blockIdx.x;
    int p = 0;
#pragma unroll
    for (int i = 1; i < kMaxProj; ++i) p += (i < sp.nproj && cr >= sp.row_start[i]) ? 1 : 0;
    *pj = p;
    *yy = cr - sp.row_start[p];
    *tb = blockIdx.y;
    return true;
  }
  item_decode(sp, V, units, pj, yy, tb);
  return true;
}

// number of units along the tile axis: single tiles (MT == 1) or the plan's tile
// blocks (tiles of one adapter, up to kBlkTiles each)
template <int MT>
__device__ __forceinline__ int tile_units(const TileArgs& p, int units_max) {
  if (units_max > 0) return units_max;
  return MT == 1 ? p.hdr[0] : p.hdr[4];
}
// tiles of unit tb and their weight index; cnt == 0 for a unit past the end
template <int MT>
__device__ __forceinline__ void pick_tiles(const TileArgs& p, int tb, int* t0, int* cnt, int* wid) {
  if (MT == 1) {
    *t0 = tb;
    *wid = uload(p.tile_wid, tb);
    *cnt = wid_ok(p, *wid) ? 1 : 0;
  } else {
    const int packed = uload(p.blk, tb);
    *t0 = packed >> 3;
    *cnt = packed & 7;
    *wid = *cnt ? uload(p.tile_wid, *t0) : -1;
    if (!wid_ok(p, *wid)) *cnt = 0;  // a negative adapter id (rows that no adapter serves) or one past the tables
  }
}

// eight consecutive-k elements of weight column n (zeros when !ok)
template <bool ROWMAJOR>
__device__ __forceinline__ u32x4 load_w8(const uint16_t* W, int n, int k, int ldw, bool ok,
                                         const uint16_t* zeros) {
  if (ROWMAJOR) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    return ok ? ldg_strided8(W + (long)k * ldw + n, ldw) : zero;
  }
  return ldg16_or(W + (long)n * ldw + k, ok, zeros);
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
  int to_partial;             // write the fp32 partial even when ksplit == 1 (the consumer rounds)
  uint8_t* drop_bits;         // DROP kernels, optional: [rows, d_in / 8] keep bits of this projection's mask
};

struct ShrinkArgs {
  TileArgs plan;
  ShrinkProj p[kMaxProj];
  const float* seg_scale;     // applied when ksplit == 1
  float beta;
  int T;
  ItemSpace items;            // chunk rows of projection p: ksplit*zblocks
  int w_kn;                   // tile-block kernel only: weights are stored [k][n]
  DropArgs drop;              // DROP kernels: dropout of the training rows of x
};

// Shrink for single tiles (batches of few rows).  Work item -> (projection, k
// slice, 64-column block, tile).  The NW waves of a workgroup take consecutive k
// ranges; their accumulators are summed through LDS in wave order and written
// either as an fp32 partial (k split over workgroups, or a consumer that folds)
// or as the final 16-bit value.  NW = 8 is for decode batches: few tiles, long k.
template <int DT, int NB, int U, int NW, bool ROWMAJOR, bool DIRECT, bool DROP = false>
__global__ __launch_bounds__(NW * kWaveSize) void shrink_kernel(ShrinkArgs a) {
  __shared__ f32x4 red[NW][NB][kWaveSize];
  const int units = DIRECT ? 0 : tile_units<1>(a.plan, 0);
  const WorkRange wr = item_range<DIRECT>(a.items, units);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;

  for (int V = wr.first; V < wr.last; V += wr.step) {
    int pj, yy, tile;
    if (!item_get<DIRECT>(a.items, V, units, &pj, &yy, &tile)) break;
    const ShrinkProj P = a.p[pj];
    const int kz = yy % P.ksplit, zb = yy / P.ksplit;
    if (zb >= P.zblocks) continue;  // a chunk row added to make the count even (uniform over the workgroup)
    const int wid = uload(a.plan.tile_wid, tile);
    if (!wid_ok(a.plan, wid)) continue;  // past the last tile (direct mode), or no such adapter; uniform over the workgroup
    const int n0 = zb * 64;
    const int slot = tile * kTileRows + c;
    const int row = a.plan.tile_row[slot];
    const uint16_t* W = uload_ptr(P.w_ptrs, wid);
    const int nlim = rank_limit(a.plan, wid, P.d_out);  // weight rows at or past it are zero padding
    DropRow dr{};
    DropArgs dp{};
    if (DROP) dp = drop_proj(a.drop, pj), dr = drop_row(dp, row, a.plan.tile_rseg, slot);

    const int kbeg = (kz * NW + wave) * P.k_per_wave;
    const int kend = min(kbeg + P.k_per_wave, P.d_in);
    const uint16_t* zeros = reinterpret_cast<const uint16_t*>(a.plan.hdr + kHdrZeros);

    f32x4 acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto load_batch = [&](int k, u32x4 (&xf)[U], u32x4 (&wf)[NB][U]) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int kk = k + 32 * u + 8 * g;
        const bool kin = kk < kend;
        xf[u] = ldg16_or(P.x + (long)row * P.d_in + kk, kin && row >= 0, zeros);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const int n = n0 + 16 * nb + c;
          wf[nb][u] = load_w8<ROWMAJOR>(W, n, kk, P.ldw, kin && n < nlim, zeros);
        }
      }
    };
    auto multiply = [&](int k, const u32x4 (&xf)[U], const u32x4 (&wf)[NB][U]) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int kk = k + 32 * u + 8 * g;
        const u32x4 xu = DROP ? drop8<DT>(xf[u], dp, dr, row, kk >> 3, P.drop_bits, P.d_in >> 3, zb == 0 && kk < kend) : xf[u];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb] = Num<DT>::mfma(wf[nb][u], xu, acc[nb]);
      }
    };
    {
      // two load batches in turn: one is on its way while the other is multiplied
      u32x4 xa[U], wa[NB][U], xb[U], wb[NB][U];
      load_batch(kbeg, xa, wa);
#pragma unroll 1
      for (int k = kbeg; k < kend; k += 64 * U) {
        const bool more = k + 32 * U < kend;  // uniform over the wave
        if (more) load_batch(k + 32 * U, xb, wb);
        multiply(k, xa, wa);
        if (!more) break;
        if (k + 64 * U < kend) load_batch(k + 64 * U, xa, wa);
        multiply(k + 32 * U, xb, wb);
      }
    }

    // cross-wave sum in wave order; wave 0 writes the tile
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) red[wave][nb][lane] = acc[nb];
    __syncthreads();
    if (wave == 0 && row >= 0) {
      float scale = 1.0f;
      const bool as_partial = P.ksplit > 1 || P.to_partial;
      if (!as_partial && a.seg_scale) scale = a.seg_scale[a.plan.tile_rseg[slot]];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        // all NW reads are issued before the first add waits for one (left to itself the
        // compiler keeps two in flight, and a many-wave kernel spends as long here as
        // in its k loop)
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
          *(SMLM_GLOBAL f32x4*)(P.partial + ((long)kz * a.T + row) * P.d_out + n) = sum;
        else
          store4<DT>(P.out + (long)row * P.d_out + n, sum, scale, a.beta);
      }
    }
    __syncthreads();  // red is free again (persistent walk)
  }
}

// Shrink for tile blocks (larger batches, and the backward).  Work item -> (projection, k
// slice, 64-column block, tile block) as above, but here wave w owns tile w of the block
// and all four waves walk the whole k slice together: each 32*U-wide batch of the weight
// rows is staged once in LDS (two buffers in turn, one barrier a batch) and shared by the
// four tiles, while every wave loads the x fragments of its own tile straight into
// registers one batch ahead.  The weights are read from L2 once per workgroup, not once per
// wave, and there is no cross-wave sum.
//
// WKN: the weight matrices are stored [k][n] (k rows of d_out contiguous columns, as B
// [h_out, r] is for the backward's dV = dY B) instead of [n][k]: a batch is then staged as
// it lies in memory and the MFMA operand, which wants eight consecutive k of one column,
// is read out of LDS with the transposing read.
template <int DT, int NB, int U, bool DIRECT, bool WKN, bool DROP = false>
__global__ __launch_bounds__(kFwdThreads) void shrink_block_kernel(ShrinkArgs a) {
  constexpr int KB = 32 * U;                 // k per batch
  constexpr int kRowsW = 16 * NB;            // weight rows (output columns) per workgroup
  constexpr int kPitch = WKN ? kRowsW + 8 : KB + 8;  // LDS row pitch in elements
  constexpr int kPieces = kRowsW * (KB / 8); // 16-byte pieces of one staged batch
  constexpr int kPer = (kPieces + kFwdThreads - 1) / kFwdThreads;
  __shared__ __attribute__((aligned(16))) uint16_t wlds[2][(WKN ? KB : kRowsW) * kPitch];
  const int units = DIRECT ? 0 : tile_units<kBlkTiles>(a.plan, 0);
  const WorkRange wr = item_range<DIRECT>(a.items, units);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;
  const uint16_t* zeros = reinterpret_cast<const uint16_t*>(a.plan.hdr + kHdrZeros);

  for (int V = wr.first; V < wr.last; V += wr.step) {
    int pj, yy, tb;
    if (!item_get<DIRECT>(a.items, V, units, &pj, &yy, &tb)) break;
    const ShrinkProj P = a.p[pj];
    const int kz = yy % P.ksplit, zb = yy / P.ksplit;
    if (zb >= P.zblocks) continue;  // a chunk row added to make the count even (uniform over the workgroup)
    int t0, cnt, wid;
    pick_tiles<kBlkTiles>(a.plan, tb, &t0, &cnt, &wid);
    if (cnt == 0) continue;  // uniform over the workgroup
    const int n0 = zb * 64;
    const bool active = wave < cnt;
    const int slot = (t0 + (active ? wave : 0)) * kTileRows + c;
    const int row = active ? a.plan.tile_row[slot] : -1;
    const uint16_t* W = uload_ptr(P.w_ptrs, wid);
    const int nlim = rank_limit(a.plan, wid, P.d_out);  // weight rows at or past it are zero padding
    const int ldw = WKN ? rank_ld(a.plan, P.ldw, nlim) : P.ldw;  // [k][n] weights (B) have the rank contiguous
    const int kbeg = kz * kFwdWaves * P.k_per_wave;
    const int kend = min(kbeg + kFwdWaves * P.k_per_wave, P.d_in);
    const uint16_t* xrow = P.x + (long)(row < 0 ? 0 : row) * P.d_in;
    DropRow dr{};
    DropArgs dp{};
    if (DROP) dp = drop_proj(a.drop, pj), dr = drop_row(dp, row, a.plan.tile_rseg, slot);

    auto load_x = [&](int kb, u32x4 (&xf)[U]) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int kk = kb + 32 * u + 8 * g;
        xf[u] = ldg16_or(xrow + kk, row >= 0 && kk < kend, zeros);
      }
    };
    auto load_w = [&](int kb, u32x4 (&st)[kPer]) {
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const int idx = threadIdx.x + j * kFwdThreads;
        if (WKN) {
          const int kl = idx / (kRowsW / 8), n8 = (idx % (kRowsW / 8)) * 8;
          st[j] = ldg16_or(W + (long)(kb + kl) * ldw + n0 + n8,
                           idx < kPieces && n0 + n8 < nlim && kb + kl < kend, zeros);
        } else {
          const int nl = idx / (KB / 8), k8 = (idx % (KB / 8)) * 8;
          st[j] = ldg16_or(W + (long)(n0 + nl) * ldw + kb + k8,
                           idx < kPieces && n0 + nl < nlim && kb + k8 < kend, zeros);
        }
      }
    };
    auto stage_w = [&](int buf, const u32x4 (&st)[kPer]) {
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const int idx = threadIdx.x + j * kFwdThreads;
        const int r_ = WKN ? idx / (kRowsW / 8) : idx / (KB / 8);
        const int c_ = WKN ? (idx % (kRowsW / 8)) * 8 : (idx % (KB / 8)) * 8;
        if (idx < kPieces) *reinterpret_cast<u32x4*>(&wlds[buf][r_ * kPitch + c_]) = st[j];
      }
    };
    auto weight_frag = [&](int buf, int u, int nb) -> u32x4 {
      if (WKN) {
        // lane c names k row 32u + 8g (+4) + c/4 and columns 16nb + 4(c%4) .. +3; it receives
        // column 16nb + c of four consecutive k rows per read
        const uint16_t* base = &wlds[buf][(32 * u + 8 * g + (c >> 2)) * kPitch + 16 * nb + 4 * (c & 3)];
        const u32x2 q0 = lds_read_tr16(base), q1 = lds_read_tr16(base + 4 * kPitch);
        return u32x4{q0[0], q0[1], q1[0], q1[1]};
      }
      return *reinterpret_cast<const u32x4*>(&wlds[buf][(16 * nb + c) * kPitch + 32 * u + 8 * g]);
    };

    f32x4 acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    u32x4 xf[U], wst[kPer];
    load_x(kbeg, xf);
    load_w(kbeg, wst);
    __syncthreads();  // every wave is done with both LDS buffers of the previous item
    stage_w(0, wst);
    int buf = 0;
#pragma unroll 1
    for (int kb = kbeg; kb < kend; kb += KB) {
      u32x4 xn[U], wn[kPer];
      // the next batch is requested before this one is multiplied (past the end: zeros)
      load_x(kb + KB, xn);
      load_w(kb + KB, wn);
      __syncthreads();  // buffer `buf` is written; buffer `buf ^ 1` is no longer read
      if (active) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int kk = kb + 32 * u + 8 * g;
          const u32x4 xu = DROP ? drop8<DT>(xf[u], dp, dr, row, kk >> 3, P.drop_bits, P.d_in >> 3, zb == 0 && kk < kend) : xf[u];
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) acc[nb] = Num<DT>::mfma(weight_frag(buf, u, nb), xu, acc[nb]);
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
      if (!as_partial && a.seg_scale) scale = a.seg_scale[a.plan.tile_rseg[slot]];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int n = n0 + 16 * nb + 4 * g;  // lane holds columns n .. n+3 of its token
        if (n >= P.d_out) continue;
        if (as_partial)
          *(SMLM_GLOBAL f32x4*)(P.partial + ((long)kz * a.T + row) * P.d_out + n) = acc[nb];
        else
          store4<DT>(P.out + (long)row * P.d_out + n, acc[nb], scale, a.beta);
      }
    }
  }
}

constexpr int kMaxKsplit = 16;  // upper bound of the k split over workgroups

// Spans of memory to be cleared by workgroups of 256 threads, kZeroBlockBytes each: span i takes blocks
// [first[i], first[i + 1]).
constexpr int kZeroBlockBytes = 32768;
struct ZeroSpans {
  char* ptr[kMaxProj];
  long bytes[kMaxProj];     // multiples of 16
  int first[kMaxProj + 1];
  int n;
};
__device__ __forceinline__ void zero_span_block(const ZeroSpans& z, int block) {
  int i = 0;
#pragma unroll
  for (int j = 1; j < kMaxProj; ++j) i += (j < z.n && block >= z.first[j]) ? 1 : 0;
  const long off0 = (long)(block - z.first[i]) * kZeroBlockBytes;
  const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < kZeroBlockBytes / (256 * 16); ++e) {
    const long off = off0 + ((long)e * 256 + threadIdx.x) * 16;
    if (off < z.bytes[i]) stg16(reinterpret_cast<uint16_t*>(z.ptr[i] + off), zero);
  }
}
__global__ __launch_bounds__(256) void zero_spans_kernel(ZeroSpans z) { zero_span_block(z, (int)blockIdx.x); }

struct ReduceProj {
  const float* partial;  // [ksplit, T, d_out]
  uint16_t* out;         // [T, d_out]
  int ksplit;            // 1: nothing to fold for this projection
  // SIDE folds (the backward's dV): side_scale * out by tile slot, transposed ([d_out][side_pitch]), and the
  // same treatment of v2 (a second [T, d_out] matrix) -- what the weight-gradient kernel reads
  uint16_t* pt_a;
  uint16_t* pt_b;
  const uint16_t* v2;
};

struct ReduceArgs {
  TileArgs plan;
  ReduceProj p[kMaxProj];
  const float* seg_scale;
  float beta;
  int T, d_out, nproj;
  int units_max;  // > 0: direct mode, one (projection, tile) per workgroup over this tile bound
  const float* side_scale;  // SIDE folds: per segment, or null for 1
  long side_pitch;          // SIDE folds: slots per row of pt_a / pt_b
  ZeroSpans zero;           // SIDE folds, direct mode: memory the launch's last workgroups clear (the rows of dX
                            //   past the backward's own)
};

// Folds the k-split partial sums of a shrink launch, in split order, into the
// 16-bit result (the reference's "v in the I/O dtype"): work item -> (projection,
// tile), 16 threads per row.
// SIDE: the fold of the backward's dV, which also leaves the by-products of write_side (further down)
// behind -- the rounded sums and v2, scaled, by tile slot and transposed; slots without a row get zeros.
template <int DT, bool SIDE = false>
__global__ __launch_bounds__(256) void reduce_kernel(ReduceArgs a) {
  const int units = tile_units<1>(a.plan, a.units_max);
  if (SIDE && a.units_max > 0 && (int)blockIdx.x >= units * a.nproj) {  // (uniform over the workgroup)
    zero_span_block(a.zero, (int)blockIdx.x - units * a.nproj);
    return;
  }
  const int c = threadIdx.x >> 4, q = threadIdx.x & 15;
  const int last = a.units_max > 0 ? (int)blockIdx.x + 1 : units * a.nproj;
  for (int V = blockIdx.x; V < last; V += gridDim.x) {
    const int pj = V / units, tile = V - pj * units;
    const ReduceProj P = a.p[pj];
    if (P.ksplit <= 1) continue;
    if (!wid_ok(a.plan, uload(a.plan.tile_wid, tile))) continue;  // past the last tile (direct mode), or no such adapter
    const int slot = tile * kTileRows + c;
    const int row = a.plan.tile_row[slot];
    if (!SIDE && row < 0) continue;
    const float scale = (a.seg_scale && row >= 0) ? a.seg_scale[a.plan.tile_rseg[slot]] : 1.0f;
    const float* zf = reinterpret_cast<const float*>(a.plan.hdr + kHdrZeros);
    for (int n = 4 * q; n < a.d_out; n += 64) {
      // all partials are requested before the first add waits for one; past ksplit the loads
      // read zeros (the k split never exceeds kMaxKsplit)
      f32x4 part[kMaxKsplit];
#pragma unroll
      for (int z = 0; z < kMaxKsplit; ++z)
        part[z] = ldg_f4((z < P.ksplit && row >= 0) ? P.partial + ((long)z * a.T + row) * a.d_out + n : zf);
      u32x2 second = {0u, 0u};
      if (SIDE && P.pt_b && row >= 0) second = *reinterpret_cast<const u32x2*>(P.v2 + (long)row * a.d_out + n);
      f32x4 sum = part[0];
#pragma unroll
      for (int z = 1; z < kMaxKsplit; ++z) sum += part[z];
      if (row >= 0) store4<DT>(P.out + (long)row * a.d_out + n, sum, scale, a.beta);
      if (SIDE) {
        const float ss = (a.side_scale && row >= 0) ? a.side_scale[a.plan.tile_rseg[slot]] : 1.0f;
        // (from the rounded value, as a reader of `out` would scale it)
        const u32x2 first = {pack2<DT>(scale * sum[0], scale * sum[1]), pack2<DT>(scale * sum[2], scale * sum[3])};
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          P.pt_a[(n + 2 * e) * a.side_pitch + slot] = (uint16_t)Num<DT>::bits(ss * Num<DT>::lo(first[e]));
          P.pt_a[(n + 2 * e + 1) * a.side_pitch + slot] = (uint16_t)Num<DT>::bits(ss * Num<DT>::hi(first[e]));
          if (P.pt_b) {
            P.pt_b[(n + 2 * e) * a.side_pitch + slot] = (uint16_t)Num<DT>::bits(ss * Num<DT>::lo(second[e]));
            P.pt_b[(n + 2 * e + 1) * a.side_pitch + slot] = (uint16_t)Num<DT>::bits(ss * Num<DT>::hi(second[e]));
          }
        }
      }
    }
  }
}

// The same fold without a scale, walking the rows in order instead of through the plan's
// tiles: grid (ceil(T / 16), projections), a workgroup folds 16 consecutive rows.  Nothing is
// looked up before the partials are requested; the rows that belong to a segment are the
// range [hdr[5], hdr[5] + hdr[2]) (segments lie end to end) and only those are stored.
template <int DT>
__global__ __launch_bounds__(256) void reduce_rows_kernel(ReduceArgs a) {
  const ReduceProj P = a.p[blockIdx.y];
  if (P.ksplit <= 1) return;
  const int c = threadIdx.x >> 4, q = threadIdx.x & 15;
  const int row = (int)blockIdx.x * kTileRows + c;
  const int first = uload(a.plan.hdr, 5), count = uload(a.plan.hdr, 2);
  const bool in_batch = row < a.T;
  const float* zf = reinterpret_cast<const float*>(a.plan.hdr + kHdrZeros);
  for (int n = 4 * q; n < a.d_out; n += 64) {
    f32x4 part[kMaxKsplit];
#pragma unroll
    for (int z = 0; z < kMaxKsplit; ++z)
      part[z] = ldg_f4((in_batch && z < P.ksplit) ? P.partial + ((long)z * a.T + row) * a.d_out + n : zf);
    f32x4 sum = part[0];
#pragma unroll
    for (int z = 1; z < kMaxKsplit; ++z) sum += part[z];
    if (in_batch && row >= first && row < first + count) store4<DT>(P.out + (long)row * a.d_out + n, sum, 1.0f, a.beta);
  }
}

// ------------------------------------------------------------------ expand --
struct ExpandProj {
  uint16_t* y;                // [T, d_out]
  const uint16_t* v;          // [T, d_in]
  const void* const* w_ptrs;  // indexed by the plan's tile_wid
  uint16_t* v_out;            // optional [T, d_in]: copy of v, by row
  const float* vpart;         // VFOLD wave kernels: v arrives as vsplit (1..4) fp32 k-split partials
  int vsplit;                 //   [vsplit, T, d_in], summed here in split order and rounded
  int d_in, d_out, ldw;
  uint16_t* pt_a;             // optional [d_in, nt_max*16]: scale*v by tile slot, transposed
  uint16_t* pt_b;             // optional: same treatment of v2 (a second [T, d_in] matrix)
  const uint16_t* v2;
  const uint8_t* drop_bits;   // DROP kernels: keep bits of this projection's mask, [rows, drop_pitch]
  long drop_pitch;
};

constexpr int kMaxVsplit = 4;  // most k-split partials of v the wave kernel folds itself

struct ExpandArgs {
  TileArgs plan;
  ExpandProj p[kMaxProj];
  const float* seg_scale;
  float beta;
  int T, nt_max;
  ItemSpace items;           // chunk rows of projection p: its column chunks
  int w_kn;                  // tile-block kernel only: weights are stored [k][n]
  DropArgs drop;             // DROP kernels (the backward's dX): the mask and factor applied to the stored values
                             //   (probabilities and row count; the keep bits are each projection's own)
};

// by-products one wave per tile writes while it holds the token fragment: the
// rounded v by row, and scale*v / scale*v2 by tile slot, transposed ([k][slot]),
// which the weight-gradient kernel reads with the token index innermost
template <int DT>
__device__ __forceinline__ void write_side(const ExpandArgs& a, const ExpandProj& P, int slot, int row,
                                           int kk, u32x4 vf, float scale) {
  const u32x4 zero = {0u, 0u, 0u, 0u};
  if (P.v_out && row >= 0) stg16(P.v_out + (long)row * P.d_in + kk, vf);
  if (P.pt_a) {
    const long pitch = (long)a.nt_max * kTileRows;
    u32x4 v2f = zero;
    if (P.pt_b && row >= 0) v2f = ldg16(P.v2 + (long)row * P.d_in + kk);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      P.pt_a[(kk + 2 * e) * pitch + slot] = (uint16_t)Num<DT>::bits(scale * Num<DT>::lo(vf[e]));
      P.pt_a[(kk + 2 * e + 1) * pitch + slot] = (uint16_t)Num<DT>::bits(scale * Num<DT>::hi(vf[e]));
      if (P.pt_b) {
        P.pt_b[(kk + 2 * e) * pitch + slot] = (uint16_t)Num<DT>::bits(scale * Num<DT>::lo(v2f[e]));
        P.pt_b[(kk + 2 * e + 1) * pitch + slot] = (uint16_t)Num<DT>::bits(scale * Num<DT>::hi(v2f[e]));
      }
    }
  }
}

// ---- y in full lines ------------------------------------------------------
// The MFMA leaves a tile's accumulators as 64-byte pieces per row (lane (c, g):
// row c, eight columns at 32q + 8g).  y is read and written a full 128-byte line
// per row and instruction instead: lane -> row lane/8 (+8), eight columns at
// (lane%8)*8 of a 64-column half chunk; the accumulators change layout through
// a per-wave LDS area on the way.  Measured on a read-modify-write of gathered
// rows: 4.4 TB/s with 64-byte pieces, 4.8 with full lines.
constexpr int kOPitch = 64 + 4;  // floats: staging rows 4 banks apart, conflict-free both ways

struct LineLane {
  int orow, ocol;     // lane's row (0..7, +8 for the second instruction) and column offset
  int srow[2];        // the two y rows of the lane, -1 = none
  float scale[2];
  uint16_t* yrow[2];  // &y[srow[j]][chunk column + ocol]
  DropRow drop[2];    // DROP kernels: dropout parameters of the two rows ...
  uint32_t keep[2][2];  // ... and the keep bits of their 64-column pieces [h][j]
};

// keep bits of the pieces a lane will store (DROP kernels): requested with the other loads of
// the item; rows that are not dropped read a zero byte that is never applied
template <int NQ>
__device__ __forceinline__ void load_keep_bits(LineLane& L, const DropArgs& d, const uint8_t* bits, long bits_pitch,
                                               int ncol0, int d_out, const uint16_t* zeros) {
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int h = 0; h < NQ / 2; ++h) {
      const int col = ncol0 + 64 * h + L.ocol;
      const bool ok = L.srow[j] >= 0 && L.srow[j] < d.rows && col < d_out;  // whatever the row's probability
      L.keep[h][j] = *(const SMLM_GLOBAL uint8_t*)(ok ? bits + (long)L.srow[j] * bits_pitch + (col >> 3)
                                                      : reinterpret_cast<const uint8_t*>(zeros));
    }
}

// y is read and written once per launch, so its accesses are marked non-temporal: left to the
// default policy its lines crowd the weights out of L2 and leave dirty lines behind that the next
// launch has to wait for (measured: 4-12 % of a step on the large batches, 3.5 % on the decode
// step).  A reader that follows at once is not slowed down as long as the data fits the caches
// (measured with a writer / reader pair: 2 and 8 MB read back equally fast, 32 MB 9 % slower).
template <int NQ>
__device__ __forceinline__ void load_y_lines(u32x4 (&yold)[NQ / 2][2], const LineLane& L, int ncol0, int d_out,
                                             bool read_y, const uint16_t* zeros) {
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int h = 0; h < NQ / 2; ++h)
      yold[h][j] = ldg16_or_nt(L.yrow[j] + 64 * h, read_y && L.srow[j] >= 0 && ncol0 + 64 * h + L.ocol < d_out, zeros);
}

// DROP: what is stored is the gradient with respect to x before its dropout: the value as it
// would be stored otherwise, times the row's factor where the element was kept, zero elsewhere
template <int DT, int NQ, bool DROP = false>
__device__ __forceinline__ void store_y_lines(float* stg, const f32x4 (&acc)[NQ][2], const u32x4 (&yold)[NQ / 2][2],
                                              const LineLane& L, int c, int g, int ncol0, int d_out, float beta) {
#pragma unroll
  for (int h = 0; h < NQ / 2; ++h) {
#pragma unroll
    for (int qq = 0; qq < 2; ++qq) {
      *reinterpret_cast<f32x4*>(&stg[c * kOPitch + 32 * qq + 8 * g]) = acc[2 * h + qq][0];
      *reinterpret_cast<f32x4*>(&stg[c * kOPitch + 32 * qq + 8 * g + 4]) = acc[2 * h + qq][1];
    }
    // a wave's own LDS accesses are served in order; the compiler must keep them in order too
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    f32x4 lo4[2], hi4[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      lo4[j] = *reinterpret_cast<const f32x4*>(&stg[(L.orow + 8 * j) * kOPitch + L.ocol]);
      hi4[j] = *reinterpret_cast<const f32x4*>(&stg[(L.orow + 8 * j) * kOPitch + L.ocol + 4]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if (L.srow[j] < 0 || ncol0 + 64 * h + L.ocol >= d_out) continue;
      const u32x4 old = yold[h][j];
      const float sc = L.scale[j];
      u32x4 o;
      if (beta != 0.0f) {
        o[0] = pack2<DT>(beta * Num<DT>::lo(old[0]) + sc * lo4[j][0], beta * Num<DT>::hi(old[0]) + sc * lo4[j][1]);
        o[1] = pack2<DT>(beta * Num<DT>::lo(old[1]) + sc * lo4[j][2], beta * Num<DT>::hi(old[1]) + sc * lo4[j][3]);
        o[2] = pack2<DT>(beta * Num<DT>::lo(old[2]) + sc * hi4[j][0], beta * Num<DT>::hi(old[2]) + sc * hi4[j][1]);
        o[3] = pack2<DT>(beta * Num<DT>::lo(old[3]) + sc * hi4[j][2], beta * Num<DT>::hi(old[3]) + sc * hi4[j][3]);
      } else {
        o[0] = pack2<DT>(sc * lo4[j][0], sc * lo4[j][1]);
        o[1] = pack2<DT>(sc * lo4[j][2], sc * lo4[j][3]);
        o[2] = pack2<DT>(sc * hi4[j][0], sc * hi4[j][1]);
        o[3] = pack2<DT>(sc * hi4[j][2], sc * hi4[j][3]);
      }
      if (DROP) o = drop8_bits<DT>(o, L.drop[j], L.keep[h][j]);
      stg16_nt(L.yrow[j] + 64 * h, o);
    }
  }
}

// Expand, one tile per work item (small batches, decode): work item -> (projection,
// column chunk, tile); each wave of the workgroup owns 32*NQ output columns and
// loads its weight fragments straight into registers.  K (= LoRA rank) is
// short: KS > 0 unrolls KS 32-wide k steps, KS == 0 is the general loop over k.
// MFMA row m of column block (q,p) is output column 32q + 8(m/4) + 4p + m%4, so
// that a lane's eight accumulators for one q are eight consecutive columns.
template <int DT, int NQ, int KS, bool ROWMAJOR, bool DIRECT, bool VFOLD, bool DROP = false>
__global__ __launch_bounds__(kFwdThreads) void expand_wave_kernel(ExpandArgs a) {
  __shared__ __attribute__((aligned(16))) float olds[kFwdWaves][kTileRows * kOPitch];
  const int units = DIRECT ? 0 : tile_units<1>(a.plan, 0);
  const WorkRange wr = item_range<DIRECT>(a.items, units);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;
  const int mrow = 8 * (c >> 2) + (c & 3);  // column offset of MFMA row c inside a (q,p) block
  constexpr int KSU = KS > 0 ? KS : 1;

  for (int V = wr.first; V < wr.last; V += wr.step) {
    int pj, yy, tile;
    if (!item_get<DIRECT>(a.items, V, units, &pj, &yy, &tile)) break;
    const ExpandProj P = a.p[pj];
    if (!P.y) continue;  // a projection this call leaves out (uniform over the workgroup)
    const int ncol0 = (yy * kFwdWaves + wave) * 32 * NQ;
    if (ncol0 >= P.d_out) continue;
    const int wid = uload(a.plan.tile_wid, tile);
    if (!wid_ok(a.plan, wid)) continue;  // past the last tile (direct mode), or no such adapter
    const uint16_t* W = uload_ptr(P.w_ptrs, wid);
    const int klim = rank_limit(a.plan, wid, P.d_in);  // k at or past it: zero padding of v and the weights
    const int ldw = ROWMAJOR ? P.ldw : rank_ld(a.plan, P.ldw, klim);
    const int slot = tile * kTileRows + c;
    const int row = a.plan.tile_row[slot];
    const int rseg = a.seg_scale ? a.plan.tile_rseg[slot] : -1;  // -1 on empty slots too
    const bool side = (yy == 0 && wave == 0);  // the one wave per tile that writes by-products
    const uint16_t* zeros = reinterpret_cast<const uint16_t*>(a.plan.hdr + kHdrZeros);

    // Every load of the item is issued before anything waits for one: the old values of the
    // y rows this lane will update, the weight fragments and v (predicated-off loads read
    // zeros instead of being patched afterwards, which would make the wave wait in between).
    LineLane L;
    L.orow = lane >> 3;
    L.ocol = (lane & 7) * 8;
    int sseg[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      L.srow[j] = a.plan.tile_row[tile * kTileRows + L.orow + 8 * j];
      sseg[j] = a.seg_scale ? a.plan.tile_rseg[tile * kTileRows + L.orow + 8 * j] : -1;
      L.yrow[j] = P.y + (long)(L.srow[j] < 0 ? 0 : L.srow[j]) * P.d_out + ncol0 + L.ocol;
      if (DROP) L.drop[j] = drop_row(a.drop, L.srow[j], a.plan.tile_rseg, tile * kTileRows + L.orow + 8 * j);
    }
    u32x4 yold[NQ / 2][2];
    load_y_lines<NQ>(yold, L, ncol0, P.d_out, a.beta != 0.0f, zeros);
    if (DROP) load_keep_bits<NQ>(L, a.drop, P.drop_bits, P.drop_pitch, ncol0, P.d_out, zeros);
#pragma unroll
    for (int j = 0; j < 2; ++j) L.scale[j] = sseg[j] >= 0 ? a.seg_scale[sseg[j]] : 1.0f;

    const float scale = (side && P.pt_a && rseg >= 0) ? a.seg_scale[rseg] : 1.0f;  // for the by-products

    f32x4 acc[NQ][2];
#pragma unroll
    for (int q = 0; q < NQ; ++q) acc[q][0] = acc[q][1] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nks = KS > 0 ? KS : (P.d_in + 31) / 32;
#pragma unroll KSU
    for (int ks = 0; ks < nks; ++ks) {
      const int kk = 32 * ks + 8 * g;
      const bool kin = kk < P.d_in, kreal = kk < klim;
      u32x4 wf[NQ][2];
#pragma unroll
      for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          const int n = ncol0 + 32 * q + 4 * p + mrow;
          wf[q][p] = load_w8<ROWMAJOR>(W, n, kk, ldw, kreal && n < P.d_out, zeros);
        }
      u32x4 vf;
      const bool vok = kreal && row >= 0;
      if (VFOLD) {  // fold (and round) the shrink's fp32 partial sums as its fold launch would
        const float* zf = reinterpret_cast<const float*>(zeros);
        f32x4 part[kMaxVsplit][2];
#pragma unroll
        for (int z = 0; z < kMaxVsplit; ++z) {
          const bool ok = vok && z < P.vsplit;
          const float* pz = ok ? P.vpart + ((long)z * a.T + row) * P.d_in + kk : zf;
          part[z][0] = ldg_f4(pz);
          part[z][1] = ldg_f4(ok ? pz + 4 : zf);
        }
        f32x4 s0 = part[0][0], s1 = part[0][1];
#pragma unroll
        for (int z = 1; z < kMaxVsplit; ++z) s0 += part[z][0], s1 += part[z][1];  // + 0.0 past vsplit
        vf = u32x4{pack2<DT>(s0[0], s0[1]), pack2<DT>(s0[2], s0[3]), pack2<DT>(s1[0], s1[1]),
                   pack2<DT>(s1[2], s1[3])};
      } else {
        vf = ldg16_or(P.v + (long)row * P.d_in + kk, vok, zeros);
      }
      if (side && kin) write_side<DT>(a, P, slot, row, kk, vf, scale);
#pragma unroll
      for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int p = 0; p < 2; ++p) acc[q][p] = Num<DT>::mfma(wf[q][p], vf, acc[q][p]);
    }
    store_y_lines<DT, NQ, DROP>(olds[wave], acc, yold, L, c, g, ncol0, P.d_out, a.beta);
  }
}

// Expand, one tile BLOCK per work item (prefill / fine-tuning batches): work item
// -> (projection, column chunk of 32*NQ columns, tile block).  The workgroup
// stages the chunk's weight rows in LDS once; wave w then multiplies tile w of
// the block with them, so an adapter's B chunk is read from L2 once per four
// tiles instead of once per tile.
// WKN: weights stored [k][n] (A [r, h_in] for the backward's dX = dV A): the chunk is staged
// as it lies in memory and read out of LDS with the transposing read.
template <int DT, int NQ, int KS, bool DIRECT, bool WKN, bool DROP = false>
// (five workgroups a CU instead of the four the compiler's own register budget gives: more y
// lines in flight per CU; worth 2 % on the prefill launch and 6 % on the fine-tune one)
__global__ __launch_bounds__(kFwdThreads) __attribute__((amdgpu_waves_per_eu(DIRECT ? (NQ > 4 ? 3 : 5) : 1)))
void expand_block_kernel(ExpandArgs a) {
  static_assert(NQ % 2 == 0, "the output is written 64 columns at a time");
  constexpr int kPitch = WKN ? 32 * NQ + 8 : 32 * KS + 8;  // LDS row pitch in 16-bit elements
  // the staged weights and the area the accumulators change layout in share their LDS (the
  // weights are done with when the accumulators are complete): five workgroups fit a CU at rank 64 too
  constexpr int kWBytes = (WKN ? 32 * KS : 32 * NQ) * kPitch * 2;
  constexpr int kOBytes = kFwdWaves * kTileRows * kOPitch * 4;
  __shared__ __attribute__((aligned(16))) char smem[kWBytes > kOBytes ? kWBytes : kOBytes];
  uint16_t* wlds = reinterpret_cast<uint16_t*>(smem);
  float(*olds)[kTileRows * kOPitch] = reinterpret_cast<float(*)[kTileRows * kOPitch]>(smem);
  const int units = DIRECT ? 0 : tile_units<kBlkTiles>(a.plan, 0);
  const WorkRange wr = item_range<DIRECT>(a.items, units);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;
  const int mrow = 8 * (c >> 2) + (c & 3);

  for (int V = wr.first; V < wr.last; V += wr.step) {
    int pj, yy, tb;
    if (!item_get<DIRECT>(a.items, V, units, &pj, &yy, &tb)) break;
    const ExpandProj P = a.p[pj];
    if (!P.y) continue;  // a projection this call leaves out (uniform over the workgroup)
    const int ncol0 = yy * 32 * NQ;
    if (ncol0 >= P.d_out) continue;  // a chunk row added to round the count up (uniform over the workgroup)
    const int packed = uload(a.plan.blk, tb);
    const int t0 = packed >> 3, cnt = packed & 7;
    if (cnt == 0) continue;  // past the last block (direct mode); uniform over the workgroup
    const int wid = uload(a.plan.tile_wid, t0);
    if (!wid_ok(a.plan, wid)) continue;  // a negative adapter id (rows that no adapter serves) or one past the tables
    const uint16_t* W = uload_ptr(P.w_ptrs, wid);
    const int klim = rank_limit(a.plan, wid, P.d_in);  // k at or past it: zero padding of v and the weights
    const int ldw = WKN ? P.ldw : rank_ld(a.plan, P.ldw, klim);  // [k][n] weights (A) have whole rows per rank
    const bool active = wave < cnt;
    const int tslot = (t0 + (active ? wave : 0)) * kTileRows;
    const int slot = tslot + c;
    const int row = active ? a.plan.tile_row[slot] : -1;  // row of the MFMA column this lane feeds
    LineLane L;  // rows this lane reads and writes in y
    L.orow = lane >> 3;
    L.ocol = (lane & 7) * 8;
    int sseg[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      L.srow[j] = active ? a.plan.tile_row[tslot + L.orow + 8 * j] : -1;
      sseg[j] = (a.seg_scale && active) ? a.plan.tile_rseg[tslot + L.orow + 8 * j] : -1;  // -1 on empty slots
      L.yrow[j] = P.y + (long)(L.srow[j] < 0 ? 0 : L.srow[j]) * P.d_out + ncol0 + L.ocol;
      if (DROP) L.drop[j] = drop_row(a.drop, L.srow[j], a.plan.tile_rseg, tslot + L.orow + 8 * j);
    }
    const int rseg = (P.pt_a && a.seg_scale && active) ? a.plan.tile_rseg[slot] : -1;
    const uint16_t* zeros = reinterpret_cast<const uint16_t*>(a.plan.hdr + kHdrZeros);

    // Every load of the item is issued before anything waits for one (predicated-off loads
    // read zeros instead of being patched afterwards).
    // weight chunk -> registers (written to LDS below): 32*NQ rows of 4*KS 16-byte pieces
    constexpr int kPieces = 32 * NQ * 4 * KS;
    constexpr int kPer = (kPieces + kFwdThreads - 1) / kFwdThreads;
    u32x4 stage[kPer];
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int idx = threadIdx.x + j * kFwdThreads;
      if (WKN) {
        const int kl = idx / (4 * NQ), n8 = (idx % (4 * NQ)) * 8;
        stage[j] = ldg16_or(W + (long)kl * ldw + ncol0 + n8,
                            idx < kPieces && ncol0 + n8 < P.d_out && kl < klim, zeros);
      } else {
        const int nl = idx / (4 * KS), k8 = (idx % (4 * KS)) * 8;
        stage[j] = ldg16_or(W + (long)(ncol0 + nl) * ldw + k8,
                            idx < kPieces && ncol0 + nl < P.d_out && k8 < klim, zeros);
      }
    }
    const bool read_y = a.beta != 0.0f;
    u32x4 yold[NQ / 2][2];
    load_y_lines<NQ>(yold, L, ncol0, P.d_out, read_y, zeros);
    if (DROP) load_keep_bits<NQ>(L, a.drop, P.drop_bits, P.drop_pitch, ncol0, P.d_out, zeros);
    u32x4 vf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int kk = 32 * ks + 8 * g;
      vf[ks] = ldg16_or(P.v + (long)row * P.d_in + kk, kk < klim && row >= 0, zeros);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) L.scale[j] = (sseg[j] >= 0 && L.srow[j] >= 0) ? a.seg_scale[sseg[j]] : 1.0f;
    if (yy == 0 && active) {  // by-products for the backward (v copy, transposed scaled copies)
      const float sc = (rseg >= 0 && row >= 0) ? a.seg_scale[rseg] : 1.0f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int kk = 32 * ks + 8 * g;
        if (kk < P.d_in) write_side<DT>(a, P, slot, row, kk, vf[ks], sc);
      }
    }

    __syncthreads();  // every wave is done reading the previous item's weights
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int idx = threadIdx.x + j * kFwdThreads;
      const int r_ = WKN ? idx / (4 * NQ) : idx / (4 * KS);
      const int c_ = WKN ? (idx % (4 * NQ)) * 8 : (idx % (4 * KS)) * 8;
      if (idx < kPieces) *reinterpret_cast<u32x4*>(&wlds[r_ * kPitch + c_]) = stage[j];
    }
    __syncthreads();
    f32x4 acc[NQ][2];
#pragma unroll
    for (int q = 0; q < NQ; ++q) acc[q][0] = acc[q][1] = f32x4{0.f, 0.f, 0.f, 0.f};
    // (waves without a tile multiply zeros: whole waves only, MFMA runs with every lane, and every
    // wave reaches the barrier below)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          u32x4 wf;
          if (WKN) {
            // lane c names k row 32ks + 8g (+4) + c/4 and columns 32q + 4p + 8(c%4) .. +3; it
            // receives column 32q + 4p + 8(c/4) + c%4 (its MFMA row's column) of four k rows
            const uint16_t* base = &wlds[(32 * ks + 8 * g + (c >> 2)) * kPitch + 32 * q + 4 * p + 8 * (c & 3)];
            const u32x2 q0 = lds_read_tr16(base), q1 = lds_read_tr16(base + 4 * kPitch);
            wf = u32x4{q0[0], q0[1], q1[0], q1[1]};
          } else {
            wf = *reinterpret_cast<const u32x4*>(&wlds[(32 * q + 4 * p + mrow) * kPitch + 32 * ks + 8 * g]);
          }
          acc[q][p] = Num<DT>::mfma(wf, vf[ks], acc[q][p]);
        }

    __syncthreads();  // every wave has read its weights: the area is free for the accumulators
    if (active) store_y_lines<DT, NQ, DROP>(olds[wave], acc, yold, L, c, g, ncol0, P.d_out, a.beta);
  }
}

}  // namespace smlm
