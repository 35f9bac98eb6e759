// Dropout of the training rows of x, applied where x (or dX) passes through registers.
//
// The reference drops x before the LoRA term, one nn.Dropout(p) per adapter
// (src/loquetier_src/models/mixed_lora.py:185-192): a dropped copy of every training partition
// plus a torch.cat of the whole batch, and autograd's mask multiply on the way back.  Here no
// dropped copy of x exists.  The mask is a pure function of (seed, offset, row, column): the
// shrink kernels generate it for the x fragments they load and leave its keep bits behind (one
// byte per eight columns, 1/16 of x's bytes); the backward applies those bits -- or the same bits
// made again by drop_bits_kernel -- to the x rows the weight-gradient kernel stages and to the
// dX values the expand kernel stores.
//
// Mask: the eight 16-bit pieces of philox4x32_10(counter = (row, col / 8, offset), key = seed)
// decide elements col .. col + 7 of a row; an element is dropped when its piece is below
// floor(p * 65536).  Kept elements become round(x * (1 / (1 - p))) (float product, as torch's
// dropout computes it), dropped ones +0.  Rows at or past `rows` (inference rows) and segments
// with p <= 0 pass through untouched.
#pragma once
#include "smlm_common.hpp"

namespace smlm {

struct DropArgs {
  const float* seg_p;  // [S] dropout probability of each segment's adapter; nullptr: no dropout
  int rows;            // training rows are [0, rows)
  uint32_t k0, k1;     // seed
  uint32_t o0, o1;     // offset (distinguishes layers / steps)
  uint8_t* bits;       // optional [rows, bits_pitch]: keep bits, one byte per eight columns of a row;
  long bits_pitch;     //   written by the forward's shrink, read by the backward instead of regenerating
};

// the arguments of projection pj of a launch over several projections: offset + pj
__device__ __forceinline__ DropArgs drop_proj(DropArgs d, int pj) {
  const uint64_t off = (((uint64_t)d.o1 << 32) | d.o0) + (uint32_t)pj;
  d.o0 = (uint32_t)off;
  d.o1 = (uint32_t)(off >> 32);
  return d;
}

struct DropRow {
  uint32_t thresh;  // pieces below it are dropped
  float scale;      // factor of kept elements
  bool on;
};

// threshold and factor of dropout probability p (p <= 0: off)
__device__ __forceinline__ DropRow drop_params(float p) {
  DropRow r{0u, 1.0f, false};
  if (p > 0.0f) {
    r.on = true;
    r.thresh = p >= 1.0f ? 65536u : (uint32_t)(p * 65536.0f);
    r.scale = p >= 1.0f ? 0.0f : 1.0f / (1.0f - p);
  }
  return r;
}

// the row's dropout parameters; its segment is only looked up for training rows
__device__ __forceinline__ DropRow drop_row(const DropArgs& d, int row, const int32_t* seg_of_slot, int slot) {
  if (row >= 0 && row < d.rows) return drop_params(d.seg_p[seg_of_slot[slot]]);
  return DropRow{0u, 1.0f, false};
}

__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                              uint32_t k1, uint32_t (&out)[4]) {
#pragma unroll
  for (int i = 0; i < 10; ++i) {
    if (i) {
      k0 += 0x9E3779B9u;
      k1 += 0xBB67AE85u;
    }
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
  }
  out[0] = c0, out[1] = c1, out[2] = c2, out[3] = c3;
}

// keep bits (bit e = element e is kept) of the eight elements at columns 8*colblk .. +7 of a row
__device__ __forceinline__ uint32_t drop_keep8(const DropArgs& d, uint32_t thresh, int row, int colblk) {
  uint32_t w[4];
  philox4x32_10((uint32_t)row, (uint32_t)colblk, d.o0, d.o1, d.k0, d.k1, w);
  uint32_t keep = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    keep |= ((w[e] & 0xffffu) >= thresh ? 1u << (2 * e) : 0u) | ((w[e] >> 16) >= thresh ? 2u << (2 * e) : 0u);
  return keep;
}

// kept elements times the factor (float product, rounded to the 16-bit type), dropped ones +0
template <int DT>
__device__ __forceinline__ u32x4 drop_apply8(u32x4 v, uint32_t keep, float scale) {
  u32x4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t scaled = pack2<DT>(Num<DT>::lo(v[e]) * scale, Num<DT>::hi(v[e]) * scale);
    const uint32_t m = ((0u - ((keep >> (2 * e)) & 1u)) & 0x0000ffffu) | ((0u - ((keep >> (2 * e + 1)) & 1u)) & 0xffff0000u);
    o[e] = scaled & m;
  }
  return o;
}

// Eight consecutive elements of one row (columns 8*colblk .. +7), packed two to a word.
// bits_out (may be nullptr): the row's keep bits, one byte per eight columns, are left there
// for a later pass that reads them instead of running the generator again (write != false
// selects the lanes that own the byte).
template <int DT>
__device__ __forceinline__ u32x4 drop8(u32x4 v, const DropArgs& d, const DropRow& r, int row, int colblk,
                                       uint8_t* bits_out = nullptr, long bits_pitch = 0, bool write = false) {
  if (__builtin_amdgcn_ballot_w64(r.on) == 0) return v;  // uniform over the wave
  const uint32_t keep = drop_keep8(d, r.thresh, row, colblk);
  if (bits_out && write && r.on) bits_out[(long)row * bits_pitch + colblk] = (uint8_t)keep;
  const u32x4 o = drop_apply8<DT>(v, keep, r.scale);
  return r.on ? o : v;
}

// the same from stored keep bits
template <int DT>
__device__ __forceinline__ u32x4 drop8_bits(u32x4 v, const DropRow& r, uint32_t keep) {
  if (__builtin_amdgcn_ballot_w64(r.on) == 0) return v;
  const u32x4 o = drop_apply8<DT>(v, keep, r.scale);
  return r.on ? o : v;
}

// Keep bits of every training row of a planned batch, for the kernels that apply a stored
// mask: workgroup -> tile, thread -> (row slot, column blocks slot-strided by 16).
struct DropBitsArgs {
  const int32_t* hdr;        // plan header: [0] = number of tiles
  const int32_t* tile_row;
  const int32_t* tile_rseg;
  DropArgs drop;             // bits / bits_pitch name the output
};

__global__ __launch_bounds__(256) void drop_bits_kernel(DropBitsArgs a) {
  const int tile = blockIdx.x;
  if (tile >= a.hdr[0]) return;
  const int slot = tile * kTileRows + (threadIdx.x >> 4);
  const int row = a.tile_row[slot];
  const DropRow r = drop_row(a.drop, row, a.tile_rseg, slot);
  if (!r.on) return;  // rows that are not dropped never have their byte read
  for (int cb = threadIdx.x & 15; cb < a.drop.bits_pitch; cb += 16)
    a.drop.bits[(long)row * a.drop.bits_pitch + cb] = (uint8_t)drop_keep8(a.drop, r.thresh, row, cb);
}

}  // namespace smlm
