// Backward-only kernels: weight transposes and the per-adapter token
// reductions dA_a = sum_t dV[t,:]^T x[t,:], dB_a = sum_t dY[t,:]^T v[t,:].
//
// The reference computes these with one torch matmul per train partition
// (src/loquetier_src/kernel_utils.py:139-145); its C++ side has no backward
// (kernel_src/csrc/loquetier_ops.cc:321-322).
#pragma once
#include "dropout.hpp"
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
  const int32_t* w_rank;  // optional [NA] with packed: the sources are stored at their true rank (rounded up
  int packed;             //   to 8), A_a [r_a, h_in], B_a [h_out, r_a]; the copies keep the full-rank strides
};

constexpr int kTrPitch = 80;  // LDS row pitch in 16-bit elements (40 banks: see kWgPitch)

// 64x64 tiles through LDS, 16-byte global accesses on both sides: rows of the
// source tile are written to LDS as they are and read back down the columns
// with the transposing LDS read.  grid (tiles along the hidden dimension, tiles
// along the rank, 2*NA), block 256: x walks the columns of A and the rows of B.
// Rows and columns are multiples of 8.
__global__ __launch_bounds__(256) void transpose_kernel(TransposeArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t t[64 * kTrPitch];
  const int which = blockIdx.z / a.NA, ad = blockIdx.z - which * a.NA;
  TransposeSet S = a.set[which];
  if (a.w_rank && a.packed) {  // the rank is A's row count and B's column count
    const int full = which == 0 ? S.rows : S.cols;
    const int r8 = (uload(a.w_rank, ad) + 7) & ~7;
    const int ra = r8 < full ? r8 : full;
    if (which == 0) S.rows = ra; else S.cols = ra;
  }
  const int c0 = (which == 0 ? blockIdx.x : blockIdx.y) * 64;
  const int r0 = (which == 0 ? blockIdx.y : blockIdx.x) * 64;
  if (c0 >= S.cols || r0 >= S.rows) return;  // uniform over the workgroup
  const uint16_t* src = reinterpret_cast<const uint16_t*>(S.src_ptrs[ad]);
  uint16_t* dst = S.dst_base + (long)ad * S.stride;
  const int dst_pitch = a.set[which].rows;  // the copy is [cols, rows] of the full-rank shape
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) S.dst_ptrs[ad] = dst;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  // in: lane -> (row = tid / 8 (+32), 8 columns at (tid % 8) * 8)
  const int ir = threadIdx.x >> 3, ic = (threadIdx.x & 7) * 8;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = r0 + ir + 32 * h, c = c0 + ic;
    const u32x4 v = (r < S.rows && c < S.cols) ? ldg16(src + (long)r * S.cols + c) : zero;
    *reinterpret_cast<u32x4*>(&t[(ir + 32 * h) * kTrPitch + ic]) = v;
  }
  __syncthreads();
  // out: thread -> output row (source column) oc = tid / 8 (+32), 8 source rows at 8 * (tid % 8).
  // Within 16 lanes (two output rows... ) the transposing read wants lane i to name source row
  // (i / 4) and four columns at 4 * (i % 4); lane 4a+b then holds column 4*... of rows a, a+4, ...
  // so a wave covers 16 source columns x 16 source rows per read: organise the 256 threads as
  // (column block cb = tid / 64 -> 16 columns, wave-lane l): g = l / 16 picks 16 of the 64 rows.
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane >> 4, i = lane & 15;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    // rows 16g + 8h + {0..7} of the tile: two reads of four rows each; lane i = 4a+b names row
    // (base + i/4), columns 16*wave + 4*(i%4) .. +3 and receives column 16*wave + i, rows base + {0..3}
    const int rb = 16 * g + 8 * h;
    const uint16_t* p0 = &t[(rb + (i >> 2)) * kTrPitch + 16 * wave + 4 * (i & 3)];
    const u32x2 q0 = lds_read_tr16(p0), q1 = lds_read_tr16(p0 + 4 * kTrPitch);
    const int oc = c0 + 16 * wave + i, orow = r0 + rb;
    if (oc < S.cols && orow < S.rows) stg16(dst + (long)oc * dst_pitch + orow, u32x4{q0[0], q0[1], q1[0], q1[1]});
  }
}

constexpr int kWgMaxProj = 8;  // projections one weight-gradient launch can serve (as the forward's launches)

struct WgradProj {
  const uint16_t* q_a;   // x  [n_rows, h_in]   -> dA
  const uint16_t* q_b;   // dY [n_rows, h_out]  -> dB
  const uint16_t* pt_a;  // scale*dV by slot, transposed [r, pitch]
  const uint16_t* pt_b;  // scale*v  by slot, transposed [r, pitch]
  void* const* da_ptrs;  // [NA] -> [r, h_in]
  void* const* db_ptrs;  // [NA] -> [h_out, r]
  int h_in, h_out, chunks_a;  // chunks_a = ceil(h_in/64) 64-column chunks of dA (dB: ceil(h_out/64))
  int units_a;                // units (walk chunks each) of dA: the projection's first units_a units work on dA
  int unit0;                  // first unit (blockIdx.x) of this projection; the projections' units lie end to end
  const uint8_t* drop_bits;   // DROP kernels: keep bits of this projection's mask of x, [rows, drop_pitch]
  long drop_pitch;
};

struct WgradArgs {
  const int32_t* hdr;
  const int32_t* grp_tile;
  const int32_t* grp_id;
  const int32_t* tile_row;
  WgradProj p[kWgMaxProj];
  int nproj;
  int walk;                // chunks a one-wave workgroup takes in turn (NW = 1 kernels; else 1)
  long pitch;
  int r;
  int n_parts;             // partitions the plan was laid out for (>= 1): its group tables hold n_parts + 1 entries
  const int32_t* w_rank;   // optional [NA]: true rank of each adapter (rows of dV / v past it are zero padding)
  int packed;              // with w_rank: dA_a [r_a, h_in] and dB_a [h_out, r_a] are stored at the true rank
  const int32_t* grp_seg;  // DROP kernels: first segment of every group (its adapter's dropout probability)
  DropArgs drop;           // DROP kernels: dA is taken against the dropped x (probabilities and row count; the
                           //   keep bits are each projection's own)
};

constexpr int kWgCols = 64;     // columns of x / dY per workgroup
constexpr int kWgPitch = 80;    // LDS row pitch in 16-bit elements: 40 banks, so any eight
                                // consecutive rows start 8 banks apart and tile the 64 banks
constexpr int kWgSlots = 64;    // gathered rows (four tiles) per wave and loop step

// LDS row of gathered-row slot s of a step: bits 2 and 3 of s change places, so
// that the eight rows one half-wave reads together (slots 8g+4h+{0..3}, g = 0,1)
// are consecutive and the read touches every bank once.
__device__ __forceinline__ int wg_lds_row(int s) {
  return (s & ~12) | ((s & 4) << 1) | ((s & 8) >> 1);
}

// grid: (sum over the projections of their dA and dB units, NA, ceil(r/64) -- twice that for the kernel named at
// wgrad_nbj_a), block 64*NW; a unit is
// `walk` neighbouring 64-column chunks of one projection's dA or dB.  A workgroup owns the unit's columns (and
// up to 64 ranks) of one adapter's gradient and walks all of that adapter's tiles once per chunk, 64
// gathered rows (four tiles, two MFMA k steps) per wave and loop step.  With
// NW = 4 (adapters with many rows each; walk = 1) the waves take steps round-robin and
// their accumulators are summed through LDS in wave order; with NW = 1 (many
// adapters with few rows each) a lone wave does it all and more workgroups fit
// on a CU -- and it takes several chunks in turn, the first rows of the next chunk on their way while
// the last of this one are multiplied: an adapter of 32 rows is 4 KB of input per chunk, and a
// workgroup per chunk is all look-ups (64 adapters, 1152 chunks: 202 us for 590 MB).  The token
// dimension is the contraction, so a wave stages its
// [token][column] block of x / dY in its own part of LDS and reads it back
// token-innermost with the transposing LDS read; no workgroup barrier is needed
// inside the loop, and the rows of the next step are already on their way from
// memory while the current step is multiplied.
//
// DROP (dA only): the forward multiplied the dropped x, so dA = dV^T dropout(x).  The keep
// bits (one byte per eight columns, the projection's drop_bits) travel with the rows and are applied while the
// rows are staged; every row of the workgroup belongs to one adapter, whose probability is read
// once from the group's first segment.
template <int DT, int NBJ, int NW, bool IS_A, bool DROP = false>
__device__ __forceinline__ void wgrad_body(const WgradArgs& a, const WgradProj& P, int chunk_first, int n_chunks,
                                           int j0, char* smem) {
  constexpr int kWgWaves = NW;
  constexpr int kStageElems = kWgSlots * kWgPitch;
  constexpr int kRedBytes = NW > 1 ? NW * 4 * kWaveSize * 16 : 0;

  const int ad = blockIdx.y;
  // j0: first rank of this workgroup (16 * NBJ ranks per workgroup along the grid's z axis)
  constexpr bool is_a = IS_A;
  const int h = is_a ? P.h_in : P.h_out;
  const uint16_t* Q = is_a ? P.q_a : P.q_b;
  const uint16_t* PT = is_a ? P.pt_a : P.pt_b;
  uint16_t* out = reinterpret_cast<uint16_t*>(is_a ? P.da_ptrs[ad] : P.db_ptrs[ad]);

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;

  // Group of this adapter (ids are distinct and ascending).  When every adapter below this one
  // has rows too, it is group number `ad`: that entry is read together with the group count, so
  // the usual case costs one round trip; otherwise every lane looks at one group.
  const int Gs = ad < a.n_parts ? ad : a.n_parts - 1;  // (entries past the last group are allocated, not filled)
  const int NG = uload(a.hdr, 1);
  const int sid = uload(a.grp_id, Gs), st0 = uload(a.grp_tile, Gs), st1 = uload(a.grp_tile, Gs + 1);
  const int sseg0 = DROP ? uload(a.grp_seg, Gs) : -1;
  int t_beg = 0, t_end = 0, seg0 = -1;
  if (Gs < NG && sid == ad) {
    t_beg = st0;
    t_end = st1;
    seg0 = sseg0;
  } else {
    for (int base = 0; base < NG; base += kWaveSize) {
      const int G = base + lane;
      const bool hit = G < NG && a.grp_id[G] == ad;
      const unsigned long long m = __ballot(hit);
      if (m) {
        const int Gh = base + __builtin_ctzll(m);
        t_beg = uload(a.grp_tile, Gh);
        t_end = uload(a.grp_tile, Gh + 1);
        if (DROP) seg0 = uload(a.grp_seg, Gh);
        break;
      }
    }
  }
  int rlim = a.r;
  if (a.w_rank) {
    const int tr = (uload(a.w_rank, ad) + 7) & ~7;
    rlim = tr < a.r ? tr : a.r;
  }
  constexpr int kStepTiles = kWgSlots / kTileRows;
  const int n_steps = (t_end - t_beg + kStepTiles - 1) / kStepTiles;

  const uint16_t* zeros = reinterpret_cast<const uint16_t*>(a.hdr + kHdrZeros);
  uint16_t* st = reinterpret_cast<uint16_t*>(smem) + wave * kStageElems;
  // staging: load u of a lane brings 8 columns (lane & 7) of the slot whose LDS row is
  // 8u + rlow; the two rows a 16-lane group writes together are 4 apart (32 banks)
  const int q8 = lane >> 3, lcol = (lane & 7) * 8;
  const int rlow = (q8 >> 1) + 4 * (q8 & 1);
  // transposed reads: lane i of a 16-lane group names row (8g + 4h + i/4) of the k step,
  // columns 16nb + 4(i%4) .. +3
  const int tr_row = wg_lds_row(8 * g + (c >> 2));  // + 4h -> LDS row + 8h; + 32 per k step
  const int tr_col = 4 * (c & 3);

  auto load_rows = [&](int step, int32_t (&row)[8]) {
    const int tile0 = t_beg + kStepTiles * step;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int s = wg_lds_row(8 * u + rlow);  // the swap is its own inverse
      const int tile = tile0 + (s >> 4);
      row[u] = (step < n_steps && tile < t_end) ? a.tile_row[tile * kTileRows + (s & 15)] : -1;
    }
  };
  const uint8_t* zero_bytes = reinterpret_cast<const uint8_t*>(zeros);
  auto load_data = [&](const int32_t (&row)[8], int n0, u32x4 (&val)[8], uint32_t (&keep)[DROP ? 8 : 1]) {
    const bool col_ok = n0 + lcol < h;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const bool ok = row[u] >= 0 && col_ok;
      // x and dY are read here for the last time in the backward: non-temporal
      val[u] = ldg16_or_nt(Q + (long)row[u] * h + n0 + lcol, ok, zeros);
      if (DROP) {  // rows at or past drop.rows keep everything: their byte is never applied
        const bool dropped = ok && row[u] < a.drop.rows;
        keep[u] = *(const SMLM_GLOBAL uint8_t*)(dropped ? P.drop_bits + (long)row[u] * P.drop_pitch + ((n0 + lcol) >> 3)
                                                        : zero_bytes) | (dropped ? 0u : 0x100u);
      }
    }
  };
  auto load_p = [&](int step, u32x4 (&pf)[NBJ][2]) {
    const int tile0 = t_beg + kStepTiles * step;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int jb = 0; jb < NBJ; ++jb) {
        const int j = j0 + 16 * jb + c;
        const int tile = tile0 + 2 * ks + (g >> 1);
        const bool ok = step < n_steps && tile < t_end && j < rlim;
        pf[jb][ks] = ldg16_or(PT + (long)j * a.pitch + (long)tile0 * kTileRows + 32 * ks + 8 * g, ok, zeros);
      }
  };

  DropRow dr{0u, 1.0f, false};  // uniform over the workgroup; .on is set per row below
  bool drop_on = false;
  if (DROP && seg0 >= 0) {
    dr = drop_params(a.drop.seg_p[seg0]);
    drop_on = dr.on;
  }

  // the first step of the first chunk
  int32_t row_first[8], row_next[8];  // the rows of the wave's first step (every chunk starts with them), of the step ahead
  uint32_t keep[DROP ? 8 : 1];  // bit 8 set: the row is not dropped
  u32x4 val[8], pf[NBJ][2];
  load_rows(wave, row_first);
  load_data(row_first, chunk_first * kWgCols, val, keep);
  load_p(wave, pf);
  load_rows(wave + kWgWaves, row_next);

  f32x4(*red)[4][kWaveSize] = reinterpret_cast<f32x4(*)[4][kWaveSize]>(smem);
  // Store staging.  The MFMA leaves 32-byte pieces per output row; the totals go through LDS once
  // more (an area of their own behind `red`) so that every store instruction writes full
  // rows: lane -> output row lane/8 (+8), eight elements at (lane%8)*8.
  constexpr int kSPitch = 64 + 4;  // floats; conflict-free for the writes below and the reads
  float* sto = reinterpret_cast<float*>(smem + (NW > 1 ? kRedBytes : 0));
  const int orow = lane >> 3, ocol = (lane & 7) * 8;
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  auto read_and_pack = [&](int row) -> u32x4 {
    const f32x4 lo4 = *reinterpret_cast<const f32x4*>(&sto[row * kSPitch + ocol]);
    const f32x4 hi4 = *reinterpret_cast<const f32x4*>(&sto[row * kSPitch + ocol + 4]);
    return u32x4{pack2<DT>(lo4[0], lo4[1]), pack2<DT>(lo4[2], lo4[3]), pack2<DT>(hi4[0], hi4[1]),
                 pack2<DT>(hi4[2], hi4[3])};
  };

#pragma unroll 1
  for (int ci = 0; ci < n_chunks; ++ci) {
    const int n0 = (chunk_first + ci) * kWgCols;
    const bool more_chunks = ci + 1 < n_chunks;  // uniform over the workgroup
    f32x4 acc[NBJ][4];
#pragma unroll
    for (int jb = 0; jb < NBJ; ++jb)
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) acc[jb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int step = wave; step < n_steps; step += kWgWaves) {
      // the next step's rows and token-side operand start their way from memory now; after this chunk's
      // last step that is the first step of the next chunk (the rows are the same, the columns move on)
      const bool last = step + kWgWaves >= n_steps;
      const bool wrap = last && more_chunks;
      u32x4 val_next[8];
      uint32_t keep_next[DROP ? 8 : 1];
      if (wrap) load_data(row_first, n0 + kWgCols, val_next, keep_next);
      else load_data(row_next, n0, val_next, keep_next);
      load_rows(wrap ? wave + kWgWaves : step + 2 * kWgWaves, row_next);

      if (DROP && drop_on) {  // uniform over the workgroup
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          dr.on = (keep[u] & 0x100u) == 0;
          val[u] = drop8_bits<DT>(val[u], dr, keep[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) *reinterpret_cast<u32x4*>(st + (8 * u + rlow) * kWgPitch + lcol) = val[u];
      // the wave's own LDS accesses are served in order; only the compiler must not move
      // the reads above the writes
      wave_sync();
      // column-side operands: Q[slots 32ks + 8g .. +7][n0 + 16nb + c], token index innermost;
      // all sixteen reads are issued before the first multiply waits for them
      u32x4 qf[2][4];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
          const uint16_t* base = st + (32 * ks + tr_row) * kWgPitch + 16 * nb + tr_col;
          const u32x2 q0 = lds_read_tr16(base), q1 = lds_read_tr16(base + 8 * kWgPitch);
          qf[ks][nb] = u32x4{q0[0], q0[1], q1[0], q1[1]};
        }
#pragma unroll
      for (int jb = 0; jb < NBJ; ++jb) {
        // rank blocks past the adapter's own rank would multiply the zeros their operand was given: their sums
        // stay the zeros they start as (uniform over the workgroup)
        if (NBJ > 1 && j0 + 16 * jb >= rlim) continue;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int nb = 0; nb < 4; ++nb) {
            // dA: rows = columns of x, cols = rank -> lane holds 4 consecutive x columns of rank c
            // dB: rows = rank, cols = columns of dY -> lane holds 4 consecutive ranks of column c
            acc[jb][nb] = is_a ? Num<DT>::mfma(qf[ks][nb], pf[jb][ks], acc[jb][nb])
                               : Num<DT>::mfma(pf[jb][ks], qf[ks][nb], acc[jb][nb]);
          }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      // the token-side operand of the next step, into the registers the multiplies above are done with (it
      // arrives behind the rows requested before it, which the next step waits for first); a wave whose
      // only step this is keeps what it has, chunk after chunk
      if (!last) load_p(step + kWgWaves, pf);
      else if (wrap && wave + kWgWaves < n_steps) load_p(wave, pf);
#pragma unroll
      for (int u = 0; u < 8; ++u) val[u] = val_next[u];
      if (DROP) {
#pragma unroll
        for (int u = 0; u < 8; ++u) keep[u] = keep_next[u];
      }
    }
    // cross-wave sum in wave order, one rank block at a time; wave 0 ends up with the totals
    if (NW > 1) {
      __syncthreads();  // every wave is done with its staging area, which red overlays
      for (int jb = 0; jb < NBJ; ++jb) {
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) red[wave][nb][lane] = acc[jb][nb];
        __syncthreads();
        if (wave == 0) {
#pragma unroll
          for (int nb = 0; nb < 4; ++nb) {
            f32x4 part[kWgWaves];
#pragma unroll
            for (int w = 0; w < kWgWaves; ++w) part[w] = red[w][nb][lane];
            f32x4 sum = part[0];
#pragma unroll
            for (int w = 1; w < kWgWaves; ++w) sum += part[w];
            acc[jb][nb] = sum;
          }
        }
        __syncthreads();
      }
      if (wave != 0) return;  // no barrier follows (several waves never walk more than one chunk)
    }

    if (is_a) {
      // dA [r, h]: per rank block, 16 rank rows x 64 columns; lane (c, g) holds rank row c,
      // columns 16nb + 4g .. +3
#pragma unroll
      for (int jb = 0; jb < NBJ; ++jb) {
        if (NBJ > 1 && a.packed && j0 + 16 * jb >= rlim) continue;  // rows the packed gradient does not have
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) *reinterpret_cast<f32x4*>(&sto[c * kSPitch + 16 * nb + 4 * g]) = acc[jb][nb];
        wave_sync();
        u32x4 o[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) o[i] = read_and_pack(orow + 8 * i);
        wave_sync();
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int j = j0 + 16 * jb + orow + 8 * i, n = n0 + ocol;
          if (j < (a.packed ? rlim : a.r) && n < h) stg16_nt(out + (long)j * h + n, o[i]);
        }
      }
    } else {
      // dB [h, r]: per 16 columns of dY (output rows), all ranks; lane (c, g) holds output row
      // 16nb + c, ranks 16jb + 4g .. +3
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
        for (int jb = 0; jb < NBJ; ++jb) *reinterpret_cast<f32x4*>(&sto[c * kSPitch + 16 * jb + 4 * g]) = acc[jb][nb];
        wave_sync();
        u32x4 o[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) o[i] = read_and_pack(orow + 8 * i);
        wave_sync();
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int n = n0 + 16 * nb + orow + 8 * i;
          const int ldb = a.packed ? rlim : a.r;  // columns of dB as it is stored
          if (j0 + ocol < ldb && n < h) stg16_nt(out + (long)n * ldb + j0 + ocol, o[i]);
        }
      }
    }
  }
}

// rank blocks of 16 a dA workgroup takes (a dB workgroup: NBJ)
constexpr int wgrad_nbj_a(int nbj, int nw, bool drop) { return (drop && nw == 1 && nbj == 4) ? 2 : nbj; }

template <int DT, int NBJ, int NW, bool DROP = false>
// (two waves a SIMD at every rank: the one-wave kernels hide their latencies through occupancy)
__global__ __launch_bounds__(NW * kWaveSize) __attribute__((amdgpu_waves_per_eu(2))) void wgrad_kernel(WgradArgs a) {
  constexpr int kStageBytes = NW * kWgSlots * kWgPitch * 2;
  constexpr int kTailBytes = (NW > 1 ? NW * 4 * kWaveSize * 16 : 0) + 16 * (64 + 4) * 4;  // red + store staging
  __shared__ __attribute__((aligned(16))) char smem[kStageBytes > kTailBytes ? kStageBytes : kTailBytes];
  int pj = 0;
#pragma unroll
  for (int i = 1; i < kWgMaxProj; ++i) pj += (i < a.nproj && (int)blockIdx.x >= a.p[i].unit0) ? 1 : 0;
  const WgradProj& P = a.p[pj];
  const int unit = (int)blockIdx.x - P.unit0;
  const int walk = NW > 1 ? 1 : a.walk;
  // The one-wave kernel that applies dropout to 64 ranks at a time does not fit the registers of a lane
  // (200 bytes of spills, and twice the time of the kernel without dropout): its dA workgroups take 32 ranks
  // each, two along z where the others have one; dB, which no dropout touches, keeps 64.
  constexpr int NBJ_A = wgrad_nbj_a(NBJ, NW, DROP), ZA = NBJ / NBJ_A;
  if (unit < P.units_a) {  // uniform over the workgroup
    const int first = unit * walk, left = P.chunks_a - first;
    wgrad_body<DT, NBJ_A, NW, true, DROP>(a, P, first, left < walk ? left : walk, 16 * NBJ_A * (int)blockIdx.z, smem);
  } else {
    if (blockIdx.z % ZA) return;
    const int chunks_b = (P.h_out + kWgCols - 1) / kWgCols;
    const int first = (unit - P.units_a) * walk, left = chunks_b - first;
    wgrad_body<DT, NBJ, NW, false>(a, P, first, left < walk ? left : walk, 16 * NBJ * (int)(blockIdx.z / ZA), smem);
  }
}

}  // namespace smlm
