// Shared device helpers for the SMLM kernels (gfx950 / CDNA4 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "smlm.h"

namespace smlm {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 16;     // rows of one MFMA tile = tokens per plan tile
constexpr int kBlkTiles = 4;      // a tile block = up to this many consecutive tiles of one group
constexpr int kWaveSize = 64;
constexpr int kSegBits = 20;      // segment index bits inside a sort key
constexpr int kMaxSegments = 1 << kSegBits;

// Element-type traits: one v_mfma_f32_16x16x32 step and the 16-bit <-> fp32
// conversions (round to nearest even on the way down).
template <int DT>
struct Num;

template <>
struct Num<SMLM_DTYPE_F16> {
  static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t bits(float f) {
    _Float16 h = (_Float16)f;
    return (uint32_t)__builtin_bit_cast(uint16_t, h);
  }
  static __device__ __forceinline__ float lo(uint32_t u) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(u & 0xffffu));
  }
  static __device__ __forceinline__ float hi(uint32_t u) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(u >> 16));
  }
};

template <>
struct Num<SMLM_DTYPE_BF16> {
  static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t bits(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7f800000u) == 0x7f800000u) {          // inf / nan: truncate, keep nan a nan
      if (u & 0x007fffffu) u |= 0x00400000u;
      return u >> 16;
    }
    u += 0x7fffu + ((u >> 16) & 1u);                 // round to nearest even
    return u >> 16;
  }
  static __device__ __forceinline__ float lo(uint32_t u) {
    return __builtin_bit_cast(float, u << 16);
  }
  static __device__ __forceinline__ float hi(uint32_t u) {
    return __builtin_bit_cast(float, u & 0xffff0000u);
  }
};

template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  return Num<DT>::bits(lo) | (Num<DT>::bits(hi) << 16);
}
// gfx950 rounds a pair of floats to fp16 or bf16 (nearest even) in one instruction
template <>
__device__ __forceinline__ uint32_t pack2<SMLM_DTYPE_F16>(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
}
template <>
__device__ __forceinline__ uint32_t pack2<SMLM_DTYPE_BF16>(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Global-memory accessors.  Addresses read from pointer tables carry no address
// space, and a generic pointer makes the compiler emit flat instructions; every
// pointer that reaches these helpers is device global memory, so say so.
#define SMLM_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ u32x4 ldg16(const uint16_t* p) {
  return *(const SMLM_GLOBAL u32x4*)(p);
}
__device__ __forceinline__ void stg16(uint16_t* p, u32x4 v) {
  *(SMLM_GLOBAL u32x4*)(p) = v;
}
__device__ __forceinline__ f32x4 ldg_f4(const float* p) {
  return *(const SMLM_GLOBAL f32x4*)(p);
}

// 16 bytes from p when ok, zeros otherwise, without a branch: the load always
// runs (from `safe`, any readable 16-byte aligned address, when !ok) so that
// the compiler keeps a run of such loads back to back.
__device__ __forceinline__ u32x4 ldg16_if(const uint16_t* p, bool ok, const uint16_t* safe) {
  const u32x4 v = ldg16(ok ? p : safe);
  const u32x4 zero = {0u, 0u, 0u, 0u};
  return ok ? v : zero;
}

// 16 bytes from p when ok, else from `zeros` (16 zero bytes in device memory: a
// plan header carries them).  Unlike ldg16_if nothing is done to the value after
// the load, so the wave need not wait for it before it goes on issuing loads.
__device__ __forceinline__ u32x4 ldg16_or(const uint16_t* p, bool ok, const uint16_t* zeros) {
  return ldg16(ok ? p : zeros);
}
// the same for data that is read once (activations, gradients): marked non-temporal so that it
// does not push the weights, which other workgroups read again, out of the caches
__device__ __forceinline__ u32x4 ldg16_or_nt(const uint16_t* p, bool ok, const uint16_t* zeros) {
  return __builtin_nontemporal_load((const SMLM_GLOBAL u32x4*)(ok ? p : zeros));
}
__device__ __forceinline__ u32x4 ldg16_nt(const uint16_t* p) {
  return __builtin_nontemporal_load((const SMLM_GLOBAL u32x4*)(p));
}
__device__ __forceinline__ void stg16_nt(uint16_t* p, u32x4 v) {
  __builtin_nontemporal_store(v, (SMLM_GLOBAL u32x4*)(p));
}
constexpr int kHdrZeros = 12;  // header words 12..15 are always zero

// Transposing LDS read of gfx950: within each 16 lanes, lane i names a "row" of
// four 16-bit elements M[i][0..3]; lane 4a+b receives M[a][b], M[4+a][b],
// M[8+a][b], M[12+a][b].
typedef __attribute__((__vector_size__(4 * sizeof(__fp16)))) __fp16 lds_tr_f16x4;
__device__ __forceinline__ u32x2 lds_read_tr16(const uint16_t* lds_addr) {
  typedef __attribute__((address_space(3))) lds_tr_f16x4 lds_vec;
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_vec*)lds_addr));
}

// Reads of plan tables and pointer tables at a wave-uniform index.  These are
// written by an earlier kernel and never by the kernel that reads them, so they
// may go through the scalar (constant) path: the loads then cost no vector
// memory slot and do not hold back the vector loads issued after them.
#define SMLM_CONST __attribute__((address_space(4)))
__device__ __forceinline__ int32_t uload(const int32_t* p, int i) {
  return ((const SMLM_CONST int32_t*)p)[i];
}
__device__ __forceinline__ float uload(const float* p, int i) {
  return ((const SMLM_CONST float*)p)[i];
}
__device__ __forceinline__ const uint16_t* uload_ptr(const void* const* tab, int i) {
  const uint64_t v = ((const SMLM_CONST uint64_t*)tab)[i];
  return reinterpret_cast<const uint16_t*>(v);
}

// Eight 16-bit elements with a stride (the slow gather used for the weight
// layout the reference never passes).
__device__ __forceinline__ u32x4 ldg_strided8(const uint16_t* p, long stride) {
  const SMLM_GLOBAL uint16_t* q = (const SMLM_GLOBAL uint16_t*)p;
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t a = q[(2 * i) * stride];
    uint32_t b = q[(2 * i + 1) * stride];
    r[i] = a | (b << 16);
  }
  return r;
}

// Views into a plan buffer (all int32).  Sizes are functions of (T, S) only.
struct PlanView {
  int32_t* hdr;         // [16]: 0 n_tiles, 1 n_groups, 2 rows covered, 3 key kind used, 4 n_blocks,
                        //       5 first covered row (the covered rows are [hdr[5], hdr[5] + hdr[2])),
                        //       12..15 zero (16 zero bytes for predicated-off loads to read)
  int32_t* sorted_seg;  // [S]   segment at sorted position p
  int32_t* rowpos;      // [S+1] first gathered-row index of sorted position p
  int32_t* grp_tile;    // [S+1] first tile of group G (exclusive scan), [NG] = n_tiles
  int32_t* grp_row;     // [S+1] first gathered-row index of group G, [NG] = rows covered
  int32_t* grp_seg;     // [S]   representative (first) segment of group G
  int32_t* grp_id;      // [S]   int32 key of group G (adapter id for SMLM_KEY_I32)
  int32_t* grp_blk;     // [S+1] first tile block of group G, [NG] = n_blocks
  int32_t* tile_row;    // [nt_max*16] row index of each tile slot, -1 = empty
  int32_t* tile_rseg;   // [nt_max*16] segment of each tile slot, -1 = empty
  int32_t* tile_wid;    // [nt_max] index into the caller's weight table: the int32 key for
                        //          SMLM_KEY_I32 plans, else the group's first segment
  int32_t* blk;         // [nt_max] tile block b: (first tile << 3) | number of tiles (1..4)
  uint64_t* sort_keys;  // [pow2 >= S] scratch for sorts that do not fit in LDS
  int nt_max;
};

inline int plan_nt_max(int T, int S) { return T / kTileRows + S + 1; }
inline int next_pow2(int v) {
  int n = 1;
  while (n < v) n <<= 1;
  return n;
}
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Carves the views out of `base`; returns the bytes used (base may be null to size).
inline size_t plan_carve(void* base, int T, int S, PlanView* pv) {
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t o = off;
    off = align_up(off + bytes, 256);
    return base ? reinterpret_cast<char*>(base) + o : nullptr;
  };
  const int nt_max = plan_nt_max(T, S);
  PlanView v;
  v.hdr = reinterpret_cast<int32_t*>(take(16 * 4));
  v.sorted_seg = reinterpret_cast<int32_t*>(take((size_t)(S + 1) * 4));
  v.rowpos = reinterpret_cast<int32_t*>(take((size_t)(S + 1) * 4));
  v.grp_tile = reinterpret_cast<int32_t*>(take((size_t)(S + 1) * 4));
  v.grp_row = reinterpret_cast<int32_t*>(take((size_t)(S + 1) * 4));
  v.grp_seg = reinterpret_cast<int32_t*>(take((size_t)(S + 1) * 4));
  v.grp_id = reinterpret_cast<int32_t*>(take((size_t)(S + 1) * 4));
  v.grp_blk = reinterpret_cast<int32_t*>(take((size_t)(S + 1) * 4));
  v.tile_row = reinterpret_cast<int32_t*>(take((size_t)nt_max * kTileRows * 4));
  v.tile_rseg = reinterpret_cast<int32_t*>(take((size_t)nt_max * kTileRows * 4));
  v.tile_wid = reinterpret_cast<int32_t*>(take((size_t)nt_max * 4));
  v.blk = reinterpret_cast<int32_t*>(take((size_t)nt_max * 4));
  v.sort_keys = reinterpret_cast<uint64_t*>(take((size_t)next_pow2(S > 0 ? S : 1) * 8));
  v.nt_max = nt_max;
  if (pv) *pv = v;
  return off;
}

}  // namespace smlm
