// C ABI of libsmlm_hip (see include/smlm.h): argument checks, workspace
// carving, launch-shape choice and kernel dispatch.  No allocation, no host
// synchronisation, no state.
#include <hip/hip_runtime.h>

#include "smlm.h"
#include "smlm_backward.hpp"
#include "smlm_common.hpp"
#include "smlm_forward.hpp"
#include "smlm_plan.hpp"

using namespace smlm;

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline int round_up(int a, int b) { return ceil_div(a, b) * b; }

int launch_status() { return hipGetLastError() == hipSuccess ? SMLM_OK : SMLM_ERR_LAUNCH; }

// ---- launch shapes: functions of (T, d_in, d_out) only, never of the
// segmentation, so re-segmenting a batch cannot change a bit of any row. ----
struct ShrinkCfg {
  int NB, U, ksplit, k_per_wave, zblocks;
};

ShrinkCfg shrink_cfg(int T, int d_in, int d_out) {
  ShrinkCfg c;
  c.zblocks = ceil_div(d_out, 64);
  const int cols = d_out >= 64 ? 64 : d_out;
  c.NB = cols <= 16 ? 1 : (cols <= 32 ? 2 : 4);
  c.U = c.NB == 4 ? 2 : 4;
  const int kq = 32 * c.U;
  const int tiles = ceil_div(T > 0 ? T : 1, kTileRows);
  const int want = ceil_div(1024, tiles);
  int max_split = d_in / (kFwdWaves * kq);
  if (max_split < 1) max_split = 1;
  if (max_split > 16) max_split = 16;
  int ks = want < 1 ? 1 : (want > max_split ? max_split : want);
  c.k_per_wave = round_up(ceil_div(d_in, kFwdWaves * ks), kq);
  c.ksplit = ceil_div(d_in, kFwdWaves * c.k_per_wave);
  return c;
}

int expand_nq(int T, int d_out) {
  const int tiles = ceil_div(T > 0 ? T : 1, kTileRows);
  return ((long)tiles * ceil_div(d_out, 512) >= 512) ? 4 : 2;
}

TileArgs tile_args(const PlanView& pv) { return TileArgs{pv.hdr, pv.tile_row, pv.tile_rseg}; }

template <int DT, bool RM>
void launch_shrink_dt(const ShrinkCfg& c, dim3 grid, hipStream_t st, const ShrinkArgs& a) {
  if (c.NB == 1) hipLaunchKernelGGL((shrink_kernel<DT, 1, 4, RM>), grid, dim3(kFwdThreads), 0, st, a);
  else if (c.NB == 2) hipLaunchKernelGGL((shrink_kernel<DT, 2, 4, RM>), grid, dim3(kFwdThreads), 0, st, a);
  else hipLaunchKernelGGL((shrink_kernel<DT, 4, 2, RM>), grid, dim3(kFwdThreads), 0, st, a);
}

int launch_shrink(int dtype, bool row_major, const ShrinkCfg& c, int nt_max, hipStream_t st,
                  const ShrinkArgs& a) {
  dim3 grid(nt_max, c.ksplit, c.zblocks);
  if (dtype == SMLM_DTYPE_F16) {
    if (row_major) launch_shrink_dt<SMLM_DTYPE_F16, true>(c, grid, st, a);
    else launch_shrink_dt<SMLM_DTYPE_F16, false>(c, grid, st, a);
  } else {
    if (row_major) launch_shrink_dt<SMLM_DTYPE_BF16, true>(c, grid, st, a);
    else launch_shrink_dt<SMLM_DTYPE_BF16, false>(c, grid, st, a);
  }
  return launch_status();
}

int launch_reduce(int dtype, int nt_max, hipStream_t st, const ReduceArgs& a) {
  if (dtype == SMLM_DTYPE_F16)
    hipLaunchKernelGGL((reduce_kernel<SMLM_DTYPE_F16>), dim3(nt_max), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((reduce_kernel<SMLM_DTYPE_BF16>), dim3(nt_max), dim3(256), 0, st, a);
  return launch_status();
}

template <int DT, bool RM>
void launch_expand_dt(int nq, dim3 grid, hipStream_t st, const ExpandArgs& a) {
  if (nq == 4) hipLaunchKernelGGL((expand_kernel<DT, 4, RM>), grid, dim3(kFwdThreads), 0, st, a);
  else hipLaunchKernelGGL((expand_kernel<DT, 2, RM>), grid, dim3(kFwdThreads), 0, st, a);
}

int launch_expand(int dtype, bool row_major, int nq, int nt_max, hipStream_t st,
                  const ExpandArgs& a) {
  dim3 grid(nt_max, ceil_div(a.d_out, kFwdWaves * 32 * nq));
  if (dtype == SMLM_DTYPE_F16) {
    if (row_major) launch_expand_dt<SMLM_DTYPE_F16, true>(nq, grid, st, a);
    else launch_expand_dt<SMLM_DTYPE_F16, false>(nq, grid, st, a);
  } else {
    if (row_major) launch_expand_dt<SMLM_DTYPE_BF16, true>(nq, grid, st, a);
    else launch_expand_dt<SMLM_DTYPE_BF16, false>(nq, grid, st, a);
  }
  return launch_status();
}

int check_common(int T, int S, int dtype) {
  if (T < 0 || S < 0) return SMLM_ERR_ARG;
  if (dtype != SMLM_DTYPE_F16 && dtype != SMLM_DTYPE_BF16) return SMLM_ERR_DTYPE;
  if (S >= kMaxSegments || T > (1 << 30)) return SMLM_ERR_LIMIT;
  return SMLM_OK;
}

int plan_build_impl(const PlanView& pv, const int32_t* seg_indptr, const void* seg_key,
                    int key_kind, int S, hipStream_t st) {
  const int N = next_pow2(S);
  if (N <= kPlanLdsKeys)
    hipLaunchKernelGGL(plan_sort_kernel<true>, dim3(1), dim3(kPlanThreads), 0, st, pv, seg_indptr,
                       seg_key, key_kind, S, N);
  else
    hipLaunchKernelGGL(plan_sort_kernel<false>, dim3(1), dim3(kPlanThreads), 0, st, pv, seg_indptr,
                       seg_key, key_kind, S, N);
  int rc = launch_status();
  if (rc) return rc;
  const long slots = (long)pv.nt_max * kTileRows;
  hipLaunchKernelGGL(plan_fill_kernel, dim3((unsigned)((slots + 255) / 256)), dim3(256), 0, st, pv,
                     seg_indptr, S);
  return launch_status();
}

struct BwdLayout {
  size_t at, bt, at_ptrs, bt_ptrs, partial, dv16, v16, pt_a, pt_b, total;
  long pitch;
  ShrinkCfg cfg_dv, cfg_v;
};

BwdLayout bwd_layout(int n_rows, int P, int NA, int h_in, int h_out, int r) {
  BwdLayout L;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t o = off;
    off = align_up(off + bytes, 256);
    return o;
  };
  L.cfg_dv = shrink_cfg(n_rows, h_out, r);
  L.cfg_v = shrink_cfg(n_rows, h_in, r);
  const int ks = L.cfg_dv.ksplit > L.cfg_v.ksplit ? L.cfg_dv.ksplit : L.cfg_v.ksplit;
  L.pitch = (long)plan_nt_max(n_rows, P) * kTileRows;
  L.at = take((size_t)NA * h_in * r * 2);
  L.bt = take((size_t)NA * h_out * r * 2);
  L.at_ptrs = take((size_t)NA * 8);
  L.bt_ptrs = take((size_t)NA * 8);
  L.partial = take((size_t)ks * n_rows * r * 4);
  L.dv16 = take((size_t)n_rows * r * 2);
  L.v16 = take((size_t)n_rows * r * 2);
  L.pt_a = take((size_t)r * L.pitch * 2);
  L.pt_b = take((size_t)r * L.pitch * 2);
  L.total = off;
  return L;
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

SMLM_API int smlm_plan_build(void* plan, size_t plan_bytes, const int32_t* seg_indptr, const void* seg_key,
                    int key_kind, int T, int S, void* stream) {
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

SMLM_API int smlm_gemm_workspace_size(int T, int S, int d_in, int d_out, size_t* bytes) {
  if (T < 0 || S < 0 || d_in <= 0 || d_out <= 0 || !bytes) return SMLM_ERR_ARG;
  if (S >= kMaxSegments || T > (1 << 30)) return SMLM_ERR_LIMIT;
  size_t n = plan_carve(nullptr, T, S, nullptr);
  if (d_in >= d_out) {
    const ShrinkCfg c = shrink_cfg(T, d_in, d_out);
    if (c.ksplit > 1) n += align_up((size_t)c.ksplit * T * d_out * 4, 256);
  }
  *bytes = n;
  return SMLM_OK;
}

SMLM_API int smlm_gemm(void* y, const void* x, const void* const* w_ptrs, const int32_t* seg_indptr,
              void* workspace, size_t workspace_bytes, int T, int S, int d_in, int d_out, int w_ld,
              int w_row_major, int dtype, float beta, const float* seg_scale, void* stream) {
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
  rc = plan_build_impl(pv, seg_indptr, w_ptrs, SMLM_KEY_PTR, S, st);
  if (rc) return rc;

  if (d_in < d_out) {  // the reference's "expand" branch (smlm_forward_cutlass.cuh:82)
    ExpandArgs a{};
    a.plan = tile_args(pv);
    a.y = reinterpret_cast<uint16_t*>(y);
    a.v = reinterpret_cast<const uint16_t*>(x);
    a.w_ptrs = w_ptrs;
    a.seg_scale = seg_scale;
    a.beta = beta;
    a.T = T; a.d_in = d_in; a.d_out = d_out; a.ldw = w_ld; a.ksplit = 1; a.nt_max = pv.nt_max;
    return launch_expand(dtype, w_row_major != 0, expand_nq(T, d_out), pv.nt_max, st, a);
  }
  const ShrinkCfg c = shrink_cfg(T, d_in, d_out);
  ShrinkArgs a{};
  a.plan = tile_args(pv);
  a.x = reinterpret_cast<const uint16_t*>(x);
  a.w_ptrs = w_ptrs;
  a.partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + plan_bytes);
  a.out = reinterpret_cast<uint16_t*>(y);
  a.seg_scale = seg_scale;
  a.beta = beta;
  a.T = T; a.d_in = d_in; a.d_out = d_out; a.ldw = w_ld;
  a.k_per_wave = c.k_per_wave; a.ksplit = c.ksplit;
  rc = launch_shrink(dtype, w_row_major != 0, c, pv.nt_max, st, a);
  if (rc || c.ksplit == 1) return rc;
  ReduceArgs ra{};
  ra.plan = a.plan;
  ra.partial = a.partial;
  ra.out = a.out;
  ra.seg_scale = seg_scale;
  ra.beta = beta;
  ra.T = T; ra.d_out = d_out; ra.ksplit = c.ksplit;
  return launch_reduce(dtype, pv.nt_max, st, ra);
}

SMLM_API int smlm_lora_fwd_workspace_size(int T, int S, int h_in, int h_out, int r, size_t* bytes) {
  if (T < 0 || S < 0 || h_in <= 0 || h_out <= 0 || r <= 0 || !bytes) return SMLM_ERR_ARG;
  const ShrinkCfg c = shrink_cfg(T, h_in, r);
  *bytes = align_up((size_t)c.ksplit * (T > 0 ? T : 1) * r * 4, 256);
  return SMLM_OK;
}

SMLM_API int smlm_lora_fwd(void* y, const void* x, void* v_out, const void* const* a_ptrs,
                  const void* const* b_ptrs, const int32_t* seg_adapter, const int32_t* seg_indptr,
                  const void* plan, void* workspace, size_t workspace_bytes, int T, int S, int h_in,
                  int h_out, int r, int dtype, float beta, const float* seg_scale, void* stream) {
  int rc = check_common(T, S, dtype);
  if (rc) return rc;
  if (h_in <= 0 || h_out <= 0 || r <= 0) return SMLM_ERR_ARG;
  if ((h_in & 7) || (h_out & 7) || (r & 7)) return SMLM_ERR_ALIGN;
  if (T == 0 || S == 0) return SMLM_OK;
  if (!y || !x || !a_ptrs || !b_ptrs || !seg_indptr || !plan || !workspace) return SMLM_ERR_ARG;
  if (!aligned16(y) || !aligned16(x) || !aligned16(workspace) || !aligned16(plan) ||
      (v_out && !aligned16(v_out)))
    return SMLM_ERR_ALIGN;
  size_t need = 0;
  smlm_lora_fwd_workspace_size(T, S, h_in, h_out, r, &need);
  if (workspace_bytes < need) return SMLM_ERR_WORKSPACE;

  hipStream_t st = (hipStream_t)stream;
  PlanView pv;
  plan_carve(const_cast<void*>(plan), T, S, &pv);
  const ShrinkCfg c = shrink_cfg(T, h_in, r);

  ShrinkArgs sa{};
  sa.plan = tile_args(pv);
  sa.x = reinterpret_cast<const uint16_t*>(x);
  sa.w_ptrs = a_ptrs;
  sa.seg_adapter = seg_adapter;
  sa.partial = reinterpret_cast<float*>(workspace);
  sa.out = reinterpret_cast<uint16_t*>(workspace);  // 16-bit v when ksplit == 1
  sa.beta = 0.0f;
  sa.T = T; sa.d_in = h_in; sa.d_out = r; sa.ldw = h_in;
  sa.k_per_wave = c.k_per_wave; sa.ksplit = c.ksplit;
  rc = launch_shrink(dtype, false, c, pv.nt_max, st, sa);
  if (rc) return rc;

  ExpandArgs ea{};
  ea.plan = sa.plan;
  ea.y = reinterpret_cast<uint16_t*>(y);
  if (c.ksplit > 1) ea.partial = sa.partial; else ea.v = sa.out;
  ea.w_ptrs = b_ptrs;
  ea.seg_adapter = seg_adapter;
  ea.seg_scale = seg_scale;
  ea.v_out = reinterpret_cast<uint16_t*>(v_out);
  ea.beta = beta;
  ea.T = T; ea.d_in = r; ea.d_out = h_out; ea.ldw = r; ea.ksplit = c.ksplit; ea.nt_max = pv.nt_max;
  return launch_expand(dtype, false, expand_nq(T, h_out), pv.nt_max, st, ea);
}

SMLM_API int smlm_lora_bwd_workspace_size(int n_rows, int P, int NA, int h_in, int h_out, int r,
                                 size_t* bytes) {
  if (n_rows < 0 || P < 0 || NA < 0 || h_in <= 0 || h_out <= 0 || r <= 0 || !bytes)
    return SMLM_ERR_ARG;
  *bytes = bwd_layout(n_rows > 0 ? n_rows : 1, P, NA > 0 ? NA : 1, h_in, h_out, r).total;
  return SMLM_OK;
}

SMLM_API int smlm_lora_bwd(void* dx, void* const* da_ptrs, void* const* db_ptrs, const void* dy,
                  const void* x, const void* v, const void* const* a_ptrs,
                  const void* const* b_ptrs, const int32_t* part_adapter,
                  const int32_t* part_indptr, const void* plan, void* workspace,
                  size_t workspace_bytes, int n_rows, int P, int NA, int h_in, int h_out, int r,
                  int dtype, const float* part_scale, void* stream) {
  int rc = check_common(n_rows, P, dtype);
  if (rc) return rc;
  if (NA < 0 || h_in <= 0 || h_out <= 0 || r <= 0) return SMLM_ERR_ARG;
  if ((h_in & 7) || (h_out & 7) || (r & 7)) return SMLM_ERR_ALIGN;
  if (r > 64) return SMLM_ERR_LIMIT;
  if (NA == 0 || n_rows == 0 || P == 0) return SMLM_ERR_ARG;
  if (!da_ptrs || !db_ptrs || !a_ptrs || !b_ptrs || !workspace) return SMLM_ERR_ARG;
  if (!dx || !dy || !x || !part_adapter || !part_indptr || !plan) return SMLM_ERR_ARG;
  if (!aligned16(dx) || !aligned16(dy) || !aligned16(x) || !aligned16(v) || !aligned16(workspace) ||
      !aligned16(plan))
    return SMLM_ERR_ALIGN;
  const BwdLayout L = bwd_layout(n_rows, P, NA, h_in, h_out, r);
  if (workspace_bytes < L.total) return SMLM_ERR_WORKSPACE;

  hipStream_t st = (hipStream_t)stream;
  char* ws = reinterpret_cast<char*>(workspace);
  uint16_t* at = reinterpret_cast<uint16_t*>(ws + L.at);
  uint16_t* bt = reinterpret_cast<uint16_t*>(ws + L.bt);
  const void** at_ptrs = reinterpret_cast<const void**>(ws + L.at_ptrs);
  const void** bt_ptrs = reinterpret_cast<const void**>(ws + L.bt_ptrs);
  float* partial = reinterpret_cast<float*>(ws + L.partial);
  uint16_t* dv16 = reinterpret_cast<uint16_t*>(ws + L.dv16);
  uint16_t* v16 = reinterpret_cast<uint16_t*>(ws + L.v16);
  uint16_t* pt_a = reinterpret_cast<uint16_t*>(ws + L.pt_a);
  uint16_t* pt_b = reinterpret_cast<uint16_t*>(ws + L.pt_b);

  PlanView pv{};
  plan_carve(const_cast<void*>(plan), n_rows, P, &pv);
  {

    // 1. transposed copies of the training adapters' weights: At [h_in, r], Bt [r, h_out]
    TransposeArgs ta{a_ptrs, at, at_ptrs, (long)h_in * r, r, h_in};
    hipLaunchKernelGGL(transpose_kernel, dim3(ceil_div(h_in, 32), ceil_div(r, 32), NA), dim3(256), 0,
                       st, ta);
    TransposeArgs tb{b_ptrs, bt, bt_ptrs, (long)h_out * r, h_out, r};
    hipLaunchKernelGGL(transpose_kernel, dim3(ceil_div(r, 32), ceil_div(h_out, 32), NA), dim3(256), 0,
                       st, tb);
    if ((rc = launch_status())) return rc;

    // 2. v = round16(x A^T) unless the forward saved it
    const uint16_t* vv = reinterpret_cast<const uint16_t*>(v);
    if (!vv) {
      ShrinkArgs sa{};
      sa.plan = tile_args(pv);
      sa.x = reinterpret_cast<const uint16_t*>(x);
      sa.w_ptrs = a_ptrs;
      sa.seg_adapter = part_adapter;
      sa.partial = partial;
      sa.out = v16;
      sa.T = n_rows; sa.d_in = h_in; sa.d_out = r; sa.ldw = h_in;
      sa.k_per_wave = L.cfg_v.k_per_wave; sa.ksplit = L.cfg_v.ksplit;
      if ((rc = launch_shrink(dtype, false, L.cfg_v, pv.nt_max, st, sa))) return rc;
      if (L.cfg_v.ksplit > 1) {
        ReduceArgs ra{};
        ra.plan = sa.plan; ra.partial = partial; ra.out = v16;
        ra.T = n_rows; ra.d_out = r; ra.ksplit = L.cfg_v.ksplit;
        if ((rc = launch_reduce(dtype, pv.nt_max, st, ra))) return rc;
      }
      vv = v16;
    }

    // 3. dV = dY B  (k-split partial sums, or 16-bit when not split)
    ShrinkArgs sd{};
    sd.plan = tile_args(pv);
    sd.x = reinterpret_cast<const uint16_t*>(dy);
    sd.w_ptrs = bt_ptrs;
    sd.seg_adapter = part_adapter;
    sd.partial = partial;
    sd.out = dv16;
    sd.T = n_rows; sd.d_in = h_out; sd.d_out = r; sd.ldw = h_out;
    sd.k_per_wave = L.cfg_dv.k_per_wave; sd.ksplit = L.cfg_dv.ksplit;
    if ((rc = launch_shrink(dtype, false, L.cfg_dv, pv.nt_max, st, sd))) return rc;

    // 4. dX = s dV A, and the slot-ordered transposed s*dV, s*v for step 5
    ExpandArgs ea{};
    ea.plan = sd.plan;
    ea.y = reinterpret_cast<uint16_t*>(dx);
    if (L.cfg_dv.ksplit > 1) ea.partial = partial; else ea.v = dv16;
    ea.w_ptrs = at_ptrs;
    ea.seg_adapter = part_adapter;
    ea.seg_scale = part_scale;
    ea.pt_a = pt_a;
    ea.pt_b = pt_b;
    ea.v2 = vv;
    ea.beta = 0.0f;
    ea.T = n_rows; ea.d_in = r; ea.d_out = h_in; ea.ldw = r; ea.ksplit = L.cfg_dv.ksplit;
    ea.nt_max = pv.nt_max;
    if ((rc = launch_expand(dtype, false, expand_nq(n_rows, h_in), pv.nt_max, st, ea))) return rc;
  }

  // 5. dA_a, dB_a for every adapter (zeros when it has no rows)
  WgradArgs wa{};
  wa.hdr = pv.hdr;
  wa.grp_tile = pv.grp_tile;
  wa.grp_id = pv.grp_id;
  wa.tile_row = pv.tile_row;
  wa.q_a = reinterpret_cast<const uint16_t*>(x);
  wa.q_b = reinterpret_cast<const uint16_t*>(dy);
  wa.pt_a = pt_a;
  wa.pt_b = pt_b;
  wa.da_ptrs = da_ptrs;
  wa.db_ptrs = db_ptrs;
  wa.pitch = L.pitch;
  wa.h_in = h_in; wa.h_out = h_out; wa.r = r;
  wa.chunks_a = ceil_div(h_in, kWgCols);
  dim3 grid(wa.chunks_a + ceil_div(h_out, kWgCols), NA);
  const int nbj = ceil_div(r, 16);
  if (dtype == SMLM_DTYPE_F16) {
    if (nbj == 1) hipLaunchKernelGGL((wgrad_kernel<SMLM_DTYPE_F16, 1>), grid, dim3(256), 0, st, wa);
    else if (nbj == 2) hipLaunchKernelGGL((wgrad_kernel<SMLM_DTYPE_F16, 2>), grid, dim3(256), 0, st, wa);
    else hipLaunchKernelGGL((wgrad_kernel<SMLM_DTYPE_F16, 4>), grid, dim3(256), 0, st, wa);
  } else {
    if (nbj == 1) hipLaunchKernelGGL((wgrad_kernel<SMLM_DTYPE_BF16, 1>), grid, dim3(256), 0, st, wa);
    else if (nbj == 2) hipLaunchKernelGGL((wgrad_kernel<SMLM_DTYPE_BF16, 2>), grid, dim3(256), 0, st, wa);
    else hipLaunchKernelGGL((wgrad_kernel<SMLM_DTYPE_BF16, 4>), grid, dim3(256), 0, st, wa);
  }
  return launch_status();
}

}  // extern "C"
