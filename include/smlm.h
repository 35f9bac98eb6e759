/*
 * libsmlm_hip -- Segmented Multi-LoRA Multiplication for AMD gfx950 (MI355X).
 *
 * C ABI of the shared library built from loquetier_amd/csrc/.  Plain pointers
 * and sizes only; every device pointer is an address in the memory of the GPU
 * that is current when the call is made.  Every call is asynchronous and
 * stream-ordered on `stream` (a hipStream_t passed as void*; NULL = the null
 * stream); none synchronises the host, none allocates or frees memory, none
 * keeps state between calls.  Return value: SMLM_OK or a negative SMLM_ERR_*.
 *
 * Maths (weights in the layout the reference passes, is_row_major = False):
 *   A_i [r, h_in] row-major, B_i [h_out, r] row-major,
 *   v = x A_i^T,  y = v B_i^T  for the rows of segment i,
 * rows [seg_indptr[i], seg_indptr[i+1]) forming segment i of the flat batch.
 *
 * Contract shared by all entry points (the reference's CUTLASS kernels are
 * instantiated with alignment 8, smlm_forward_cutlass.cuh:88-92,133-137):
 * 16-bit element types only (fp16 / bf16); every matrix pointer 16-byte
 * aligned; d_in, d_out, h_in, h_out, r multiples of 8; seg_indptr
 * non-decreasing with seg_indptr[0] >= 0 and seg_indptr[S] <= T.
 */
#ifndef SMLM_H_
#define SMLM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SMLM_ABI_VERSION 5

#if defined(__GNUC__)
#define SMLM_API __attribute__((visibility("default")))
#else
#define SMLM_API
#endif

/* element types (reference: DISPATCH_TORCH_DTYPE, loquetier_ops.cc:54-76) */
#define SMLM_DTYPE_F16 0
#define SMLM_DTYPE_BF16 1

/* what a plan groups segments by */
#define SMLM_KEY_NONE 0 /* every segment is its own group                    */
#define SMLM_KEY_I32 1  /* int32 adapter id per segment                      */
#define SMLM_KEY_PTR 2  /* 64-bit weight address per segment                 */
#define SMLM_KEY_PTR2 3 /* a pair of 64-bit weight addresses per segment (smlm_plan_build2) */

/* stages of the fused forward (smlm_lora_fwd_multi) */
#define SMLM_STAGE_SHRINK 1 /* v = x A^T, left in the workspace                */
#define SMLM_STAGE_EXPAND 2 /* y = beta*y + scale * v B^T from that workspace  */

/* stages of the backward (smlm_lora_opts.bwd_stages) */
#define SMLM_BWD_PRODUCTS 1 /* plan (when the call builds it), v when not given, dV = dY B  */
#define SMLM_BWD_DX 2       /* dX = s dV A (and the transposed s dV, s v the next stage reads) */
#define SMLM_BWD_WGRAD 4    /* dA_a, dB_a                                        */

#define SMLM_OK 0
#define SMLM_ERR_ARG (-1)       /* null pointer, negative size, bad enum      */
#define SMLM_ERR_DTYPE (-2)     /* "No suitable kernel." (loquetier_ops.cc:318) */
#define SMLM_ERR_ALIGN (-3)     /* dimension not a multiple of 8 / pointer not 16-byte aligned */
#define SMLM_ERR_WORKSPACE (-4) /* workspace or plan buffer too small         */
#define SMLM_ERR_LAUNCH (-5)    /* the HIP runtime refused a kernel launch    */
#define SMLM_ERR_LIMIT (-6)     /* size beyond what the kernels index         */
#define SMLM_ERR_SCRATCH (-7)   /* the call needs more scratch than the library's static array holds */

SMLM_API int smlm_abi_version(void);
SMLM_API const char* smlm_strerror(int code);

/*
 * Replaces smlm_forward_tmp_size (smlm_forward_cutlass.cuh:48-52), exported to
 * Python as smlm_forward_cutlass_tmp_size (loquetier_ops.cc:372).  The
 * reference carves seven per-problem arrays (60 bytes per problem) out of
 * `tmp`; this library keeps its per-call tables in the workspace sized by
 * smlm_gemm_workspace_size, so the value only has to be what the caller
 * allocates and passes back: 64 bytes per problem.
 */
SMLM_API int smlm_tmp_size(int num_problems, size_t* bytes);

/*
 * Tile plan.  Replaces precompute_smlm_forward_args
 * (smlm_forward_cutlass.cuh:31-46): the per-problem table the grouped GEMM
 * walks.  Here the table lists 16-row tiles; rows of segments that share a key
 * (adapter) are gathered into common tiles so each adapter's weights are read
 * once per tile column instead of once per segment.  The plan depends only on
 * (seg_indptr, keys): one plan serves every layer and projection of a batch.
 *   seg_key: NULL for SMLM_KEY_NONE, const int32_t* [S] for SMLM_KEY_I32,
 *            const void* const* [S] for SMLM_KEY_PTR (device memory).
 * The key kind also fixes how the GEMM entry points below index their weight
 * tables: a plan built with SMLM_KEY_I32 makes them read w_ptrs[key] (the
 * table has one entry per adapter -- the gather wa_ptrs[lora_ids] of
 * src/loquetier_src/models/mixed_lora.py:182 done inside the kernel); any other
 * plan makes them read w_ptrs[i] for segment i (one entry per segment).
 * Segments that share a key must share their weights.  A negative SMLM_KEY_I32 key marks a
 * segment that no adapter serves (a request without LoRA in a mixed batch): the forward entry
 * points leave its rows of y alone (its rows of v are undefined).  A key at or above the
 * n_weights the GEMM entry points are told (when they are told one: n_weights > 0) is treated
 * the same way -- the tables are never read past their end; the backward leaves the rows of such
 * a partition's dx as they were and sums nothing for it.
 */
SMLM_API int smlm_plan_size(int T, int S, size_t* bytes);
SMLM_API int smlm_plan_build(void* plan, size_t plan_bytes, const int32_t* seg_indptr,
                             const void* seg_key, int key_kind, int T, int S, void* stream);
/*
 * The plan of a batch whose segments name their weights by a PAIR of addresses (device arrays
 * of S addresses each), as the reference's add_lora.forward is handed them: wa_ptr[i] and
 * wb_ptr[i] per problem (src/loquetier_src/kernel_utils.py:115-119).  Segments are grouped
 * where BOTH addresses agree, so segments may share A and differ in B; one such plan serves
 * the shrink and the expand of the fused forward, whose tables then have one entry per segment.
 */
SMLM_API int smlm_plan_build2(void* plan, size_t plan_bytes, const int32_t* seg_indptr,
                              const void* const* seg_key_a, const void* const* seg_key_b, int T, int S,
                              void* stream);

/*
 * Grouped GEMM  Y_i = beta*Y_i + scale_i * X_i W_i  over the segments.
 * Replaces dispatch_smlm_forward_cutlass / smlm_forward<DType,Layout>
 * (loquetier_ops.cc:277-319, smlm_forward_cutlass.cuh:61-175), which computes
 * the beta = 0, scale = 1 case.  w_ptrs[i] (device array of S device
 * addresses) is a d_in x d_out matrix: element (k, n) at w[k*w_ld + n] when
 * w_row_major, else at w[n*w_ld + k].  seg_scale: NULL or float [S] (device).
 * Builds its own plan (grouped by weight address) inside `workspace`.
 * Rows outside every segment are not touched.
 */
SMLM_API int smlm_gemm_workspace_size(int T, int S, int d_in, int d_out, size_t* bytes);
SMLM_API int smlm_gemm(void* y, const void* x, const void* const* w_ptrs, const int32_t* seg_indptr,
                       void* workspace, size_t workspace_bytes, int T, int S, int d_in, int d_out,
                       int w_ld, int w_row_major, int dtype, float beta, const float* seg_scale,
                       void* stream);

/*
 * smlm_gemm for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart
 * in the reference (whose caller allocates `tmp` with torch,
 * src/loquetier_src/kernel_utils.py:113-116).  Same arguments as smlm_gemm
 * without the workspace, same kernels, same results bit for bit; the plan and the
 * k-split partial sums live in an array of SMLM_STATIC_SCRATCH_BYTES that is part
 * of the library's code object (every GPU the library runs on holds its own copy
 * until the process ends).  Returns SMLM_ERR_SCRATCH when
 * smlm_gemm_workspace_size(T, S, d_in, d_out) exceeds that size.  Calls neither
 * hipMalloc nor hipFree nor any allocating routine.  The first call on a device
 * looks the array's address up (hipGetSymbolAddress) and should be made outside a
 * capture.  All calls on one GPU share the array: calls that overlap on one GPU
 * (different streams, or different host threads without ordering) race; calls on
 * one stream are safe.  Nothing in the array has to start at zero -- every word a
 * kernel reads is written earlier in the same call -- so the contents left by an
 * earlier call never matter.
 */
#define SMLM_STATIC_SCRATCH_BYTES (8u << 20)
SMLM_API int smlm_gemm_static(void* y, const void* x, const void* const* w_ptrs,
                              const int32_t* seg_indptr, int T, int S, int d_in, int d_out, int w_ld,
                              int w_row_major, int dtype, float beta, const float* seg_scale,
                              void* stream);

/*
 * The same grouped GEMM with a plan built beforehand by smlm_plan_build for
 * (seg_indptr, T, S): nothing but the GEMM kernels is launched, so a caller
 * that issues many GEMMs over one batch (every layer and projection of a
 * model step) pays for the plan once.  n_weights is the number of entries of
 * w_ptrs (adapters for an id-keyed plan, S otherwise; 0 = unknown): the number
 * of distinct keys cannot exceed it, which bounds the launch size.  No
 * counterpart in the reference, which rebuilds its problem table inside every
 * call (smlm_forward_cutlass.cuh:76-79).
 */
SMLM_API int smlm_gemm_planned_workspace_size(int T, int d_in, int d_out, size_t* bytes);
SMLM_API int smlm_gemm_planned(void* y, const void* x, const void* const* w_ptrs, int n_weights,
                               const void* plan, void* workspace, size_t workspace_bytes, int T,
                               int S, int d_in, int d_out, int w_ld, int w_row_major, int dtype,
                               float beta, const float* seg_scale, void* stream);

/*
 * Fused LoRA forward  y = beta*y + scale_i * round16(x A^T) B^T.
 * Replaces the two kernel calls of add_lora.forward
 * (src/loquetier_src/kernel_utils.py:115-119) plus, with beta = 1 and
 * seg_scale, the scale multiply and residual add of MixedLoraLinear.forward
 * (src/loquetier_src/models/mixed_lora.py:214-217).
 *   a_ptrs / b_ptrs: device arrays of n_weights device addresses, indexed as
 *     the plan's key kind says (see smlm_plan_build); n_weights = 0 if unknown.
 *   plan: built by smlm_plan_build for the batch's (seg_indptr, T, S).
 *   v_out: NULL, or [T, r] receiving the rounded intermediate for backward.
 */
SMLM_API int smlm_lora_fwd_workspace_size(int T, int S, int h_in, int h_out, int r, size_t* bytes);
SMLM_API int smlm_lora_fwd(void* y, const void* x, void* v_out, const void* const* a_ptrs,
                           const void* const* b_ptrs, int n_weights, const void* plan, void* workspace,
                           size_t workspace_bytes, int T, int S, int h_in, int h_out, int r, int dtype,
                           float beta, const float* seg_scale, void* stream);

/*
 * The fused forward for up to 8 projections of one batch in two launches (one
 * shrink, one expand): q/k/v/o or gate/up/down of a layer share the plan, the
 * rank and the segment routing, and in the decode regime a launch costs as much
 * as the data movement of one projection.  y, x, v_out, a_ptrs, b_ptrs, h_in,
 * h_out are HOST arrays of n_proj entries (v_out may be NULL or hold NULLs);
 * projections may differ in h_in / h_out.  `stages` is SMLM_STAGE_SHRINK |
 * SMLM_STAGE_EXPAND for the whole forward; a caller may also issue the two
 * stages as separate calls with the same arguments and workspace (the expand
 * stage reads what the shrink stage left there).  A shrink-only call may pass
 * NULL for every y, an expand-only call NULL for every x; an expand-only call
 * skips the projections whose y is NULL, so the projections of one shrink call
 * (q, k, v of one input) can be expanded one at a time, each when its y is
 * ready, with the other arguments unchanged.  No counterpart in the reference,
 * which calls its kernel once per linear layer (mixed_lora.py:198-205).
 */
SMLM_API int smlm_lora_fwd_multi_workspace_size(int n_proj, int T, const int* h_in, int r,
                                                size_t* bytes);
SMLM_API int smlm_lora_fwd_multi(int n_proj, void* const* y, const void* const* x,
                                 void* const* v_out, const void* const* const* a_ptrs,
                                 const void* const* const* b_ptrs, int n_weights, const int* h_in,
                                 const int* h_out, const void* plan, void* workspace,
                                 size_t workspace_bytes, int T, int S, int r, int dtype, float beta,
                                 const float* seg_scale, int stages, void* stream);

/*
 * LoRA backward for fine-tuning rows.  Replaces add_lora.backward
 * (src/loquetier_src/kernel_utils.py:128-147; the C++ side of the reference
 * has only "// smlm backward // TODO", loquetier_ops.cc:321-322), with the
 * products written for the weight layout the forward uses:
 *   dV = s (dY B)   dX = dV A   dA_a = sum dV^T x   dB_a = sum dY^T (s v)
 * Rows [part_indptr[p], part_indptr[p+1]) of dy / x / v / dx form train
 * partition p, trained by adapter part_adapter[p] in [0, NA).  da_ptrs[a]
 * ([r, h_in]) and db_ptrs[a] ([h_out, r]) are overwritten for every a with the
 * sum over that adapter's partitions (zeros when it has none); summation order
 * is fixed, no atomics.  dx rows [0, n_rows) covered by a partition are
 * overwritten, others untouched.
 *   plan: built by smlm_plan_build(part_indptr, part_adapter, SMLM_KEY_I32,
 *         n_rows, P); it carries the partitions and their adapters.
 *   a_ptrs, b_ptrs, da_ptrs, db_ptrs: device arrays of NA device addresses.
 *   v: NULL (recomputed from x and A) or [n_rows, r].
 *   part_scale: NULL or float [P] (device), the forward's seg_scale.
 * Needs n_rows >= 1, P >= 1, NA >= 1 and r <= 64.
 */
SMLM_API int smlm_lora_bwd_workspace_size(int n_rows, int P, int NA, int h_in, int h_out, int r,
                                          size_t* bytes);
SMLM_API int smlm_lora_bwd(void* dx, void* const* da_ptrs, void* const* db_ptrs, const void* dy,
                           const void* x, const void* v, const void* const* a_ptrs,
                           const void* const* b_ptrs, const void* plan, void* workspace,
                           size_t workspace_bytes, int n_rows, int P, int NA, int h_in, int h_out,
                           int r, int dtype, const float* part_scale, void* stream);

/*
 * Dropout of the training rows of x inside the LoRA operator.  Replaces the
 * per-partition nn.Dropout calls and the torch.cat in MixedLoraLinear.forward
 * (src/loquetier_src/models/mixed_lora.py:185-192) and autograd's mask multiply
 * on the way back: no dropped copy of x and no mask are stored, the mask is
 * regenerated from (seed, offset, row, column) wherever x or dX pass through
 * registers.  Element (t, j) of a row t < rows whose segment has p > 0 is dropped
 * when 16-bit piece j % 8 of
 *   philox4x32_10(counter = (t, j / 8, offset_lo, offset_hi), key = (seed_lo, seed_hi))
 * is below floor(p * 65536); kept elements become round(x * (1 / (1 - p))).
 *   seg_p  : device float [S], the dropout probability of each segment's adapter
 *            (indexed like seg_scale: by the plan's segments); NULL = no dropout
 *   rows   : training rows are [0, rows) of the batch; later rows are never dropped
 *   seed, offset : the stream; the same pair must be passed to the forward and to
 *            the backward of one layer.  Projection i of a multi-projection call
 *            uses offset + i.
 *   mask_bits : optional device buffer for the keep bits, one byte per eight
 *            columns of a training row ([rows, h_in / 8] bytes; bit e of a byte =
 *            element 8*block + e is kept; the projections of a multi-projection call
 *            lie end to end).  The forward fills it when given (bytes of rows whose
 *            p is 0 are left alone); the backward reads it when given and otherwise
 *            regenerates the same bits into its workspace.  NULL is always valid.
 */
typedef struct smlm_dropout {
  const float* seg_p;
  int rows;
  uint64_t seed;
  uint64_t offset;
  void* mask_bits;
} smlm_dropout;

/*
 * Options of the _ex entry points; a NULL pointer or a zeroed struct changes nothing.
 *   dropout      : see smlm_dropout above.
 *   adapter_rank : device int32, indexed like the weight tables (by adapter id for
 *                  SMLM_KEY_I32 plans, by segment otherwise): the true rank of each
 *                  adapter.  The reference keeps adapters of different ranks zero-padded
 *                  to one rank r (MixedLoraModel._prepare_weight,
 *                  src/loquetier_src/models/mixed_lora.py:501-521); with the true ranks
 *                  the kernels do not read the padding (rows of A, columns of B and of v
 *                  at or past the rank rounded up to 8) and treat it as the zeros it
 *                  holds, so results equal the padded computation bit for bit.
 *   packed_ranks : non-zero (with adapter_rank): the weights are STORED at their true rank
 *                  rounded up to 8, A_a [r_a, h_in] and B_a [h_out, r_a] contiguous, instead of
 *                  zero-padded to r; the backward writes dA_a / dB_a in the same shapes.  A
 *                  rank-8 adapter beside rank-64 ones then costs 16 bytes of B per output
 *                  column instead of a 128-byte line.  Results equal the padded computation
 *                  bit for bit; v, dV and the workspace keep the launch's rank r.
 *   build_seg_indptr, build_seg_adapter (both or neither):
 *                  `plan` is a buffer of smlm_plan_size(T, S) bytes that holds NO plan yet; the
 *                  call builds the plan smlm_plan_build(plan, ..., build_seg_indptr,
 *                  build_seg_adapter, SMLM_KEY_I32, T, S) would build, writes it to `plan` (valid
 *                  for every later call on the stream) and uses it.  The reference sets its
 *                  problems up inside every call as well (precompute_smlm_forward_args,
 *                  kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:31-46,76-79).  With
 *                  n_weights <= 1024, no dropout and either a batch of few rows (the single-tile
 *                  kernels: below 2048 rows at rank <= 16, 768 at rank <= 32, 512 at rank <= 48,
 *                  128 at rank <= 64, 1024 above), S <= 1024 and every h_in >= 2048, or a
 *                  larger batch with S <= 512 and T / 16 + S < 1024, this costs no
 *                  launch: the shrink's workgroups derive their own tiles from the two arrays
 *                  while a few more workgroups of the same launch write the plan; other batches
 *                  get the plan launch first.  Adapter ids must lie below n_weights (negative:
 *                  no adapter, see the tile plan above); stages must include SMLM_STAGE_SHRINK.
 *                  smlm_lora_bwd_ex takes the pair (part_indptr, part_adapter) the same way and
 *                  builds its plan inside the dV launch when r <= 64, P <= 512,
 *                  n_rows / 16 + P < 1024, v is given and there is no dropout.
 *   build_seg_key_a, build_seg_key_b (both or neither, with build_seg_indptr, instead of
 *                  build_seg_adapter; smlm_lora_fwd_multi_ex only):
 *                  the plan to build is the one smlm_plan_build2 builds from these two arrays of S
 *                  addresses; with S <= 1024 (and the other limits above) inside the shrink launch.
 *                  The weight tables of the call have one entry per segment (n_weights = S).
 *   bwd_stages   : (backward entry points) 0 = the whole backward; else a set of SMLM_BWD_* bits: the
 *                  stages of one backward may be issued as separate calls with the same arguments,
 *                  workspace and stream, in the order PRODUCTS, DX, WGRAD (each reads what the stage
 *                  before left in the workspace) -- to time them one by one, or to put other work of
 *                  the stream between them.  A plan the call is to build is built by the PRODUCTS stage.
 *   w_row_major  : (backward entry points) non-zero: the weights are in the layout the reference calls
 *                  is_row_major = True -- A_a [h_in, r], B_a [r, h_out] row-major -- the layout its Python
 *                  backward is written for (src/loquetier_src/kernel_utils.py:139-145):
 *                    mid = dY B^T   dX = s mid A^T   dA_a = sum x^T (s mid)   dB_a = sum (s x A)^T dY
 *                  with dA_a [h_in, r] and dB_a [r, h_out] in the weights' own shapes.  Same kernels, no
 *                  copies; not together with dropout or packed_ranks.  (The forward in this layout is
 *                  smlm_gemm / smlm_gemm_planned with w_row_major = 1.)
 *   dx_rows      : (backward entry points) 0, or the number of rows every dx buffer has, >= n_rows: the call
 *                  then also sets rows [n_rows, dx_rows) of every dx to zero -- the rows of the batch that are
 *                  not trained, when dx is the gradient of the whole batch's x as autograd wants it -- at no
 *                  launch of its own where the dV product is folded (the fold's launch has the workgroups), by
 *                  one small launch otherwise.  With bwd_stages the SMLM_BWD_PRODUCTS stage does it.
 */
typedef struct smlm_lora_opts {
  const smlm_dropout* dropout;
  const int32_t* adapter_rank;
  int packed_ranks;
  int dx_rows;
  const int32_t* build_seg_indptr;
  const int32_t* build_seg_adapter;
  int bwd_stages;
  int w_row_major;
  const void* const* build_seg_key_a;
  const void* const* build_seg_key_b;
} smlm_lora_opts;

/* smlm_lora_fwd_multi with options. */
SMLM_API int smlm_lora_fwd_multi_ex(int n_proj, void* const* y, const void* const* x,
                                    void* const* v_out, const void* const* const* a_ptrs,
                                    const void* const* const* b_ptrs, int n_weights,
                                    const int* h_in, const int* h_out, const void* plan,
                                    void* workspace, size_t workspace_bytes, int T, int S, int r,
                                    int dtype, float beta, const float* seg_scale, int stages,
                                    const smlm_lora_opts* opts, void* stream);

/*
 * smlm_lora_bwd with options (NULL: identical to smlm_lora_bwd).  adapter_rank is
 * indexed by the training adapters 0..NA-1.  For a forward that ran with dropout:
 * seg_p is indexed by the backward plan's partitions and the
 * partitions of one adapter must carry the same probability; (seed, offset) are
 * the pair the forward of this projection used (offset + i for projection i of a
 * multi-projection call); rows >= n_rows.  x is the caller's x before dropout: v
 * (when not passed) and dA are taken against the regenerated dropped x, and dx is
 * the gradient with respect to x before its dropout (the mask and factor applied
 * once more, as autograd's dropout backward does after add_lora.backward).
 */
SMLM_API int smlm_lora_bwd_ex(void* dx, void* const* da_ptrs, void* const* db_ptrs,
                              const void* dy, const void* x, const void* v,
                              const void* const* a_ptrs, const void* const* b_ptrs,
                              const void* plan, void* workspace, size_t workspace_bytes,
                              int n_rows, int P, int NA, int h_in, int h_out, int r, int dtype,
                              const float* part_scale, const smlm_lora_opts* opts, void* stream);

/*
 * The backward of up to 8 projections of one batch in one set of launches (one dV product, one
 * fold, one dX product, one weight-gradient launch for all of them): the projections share the
 * partition plan, the adapters' indices, the rank and the scale, as q/k/v/o or gate/up/down of
 * a layer do.  dx, da_ptrs, db_ptrs, dy, x, v, a_ptrs, b_ptrs, h_in, h_out are HOST arrays of
 * n_proj entries, each entry what smlm_lora_bwd_ex takes for one projection; v is NULL or
 * names the saved intermediate of every projection.  Results equal n_proj calls of
 * smlm_lora_bwd_ex bit for bit (the kernels and their launch shapes per projection are the same).
 * With dropout, projection i uses the stream offset + i and the caller's keep bits of the
 * projections lie end to end, as smlm_lora_fwd_multi_ex leaves them.  No counterpart in the
 * reference, whose backward is a Python loop per layer and partition
 * (src/loquetier_src/kernel_utils.py:128-147).
 */
SMLM_API int smlm_lora_bwd_multi_workspace_size(int n_proj, int n_rows, int P, int NA, const int* h_in,
                                                const int* h_out, int r, size_t* bytes);
SMLM_API int smlm_lora_bwd_multi_ex(int n_proj, void* const* dx, void* const* const* da_ptrs,
                                    void* const* const* db_ptrs, const void* const* dy,
                                    const void* const* x, const void* const* v,
                                    const void* const* const* a_ptrs, const void* const* const* b_ptrs,
                                    const void* plan, void* workspace, size_t workspace_bytes,
                                    int n_rows, int P, int NA, const int* h_in, const int* h_out, int r,
                                    int dtype, const float* part_scale, const smlm_lora_opts* opts,
                                    void* stream);

/*
 * RMSNorm forward.  Replaces dispatch_rms_norm / rms_norm<T>
 * (kernel_src/csrc/loquetier_ops.cc:326-358,
 * kernel_src/csrc/rms_norm/rms_norm_cutlass.cu:81-186):
 *   rms[t] = 1 / sqrt(mean_j x[t,j]^2 + eps)   (float, kept for the backward)
 *   out[t,j] = x[t,j] * rms[t] * w[j]          (float arithmetic, rounded once)
 * out, x: [rows, cols] of `dtype`; w: [cols] of `dtype`; rms: float [rows].
 * cols a multiple of 8 (as in the reference).  Rows of up to 16384 columns stay in registers
 * between the reduction and the scaling (read once); wider rows take a two-pass kernel.
 */
SMLM_API int smlm_rms_norm_fwd(void* out, float* rms, const void* x, const void* w, int rows,
                               int cols, float eps, int dtype, void* stream);

/*
 * RMSNorm backward.  Replaces the tensor expressions of rms_norm.backward
 * (src/loquetier_src/kernel_utils.py:169-176), evaluated in float in one pass:
 *   dot[t] = sum_j g*w*x,  dx = (g*w - x*dot*rms^2/cols) * rms,
 *   dw[j] = sum_t x*rms*g   (summed in a fixed order, no atomics)
 * dx, g, x: [rows, cols]; w, dw: [cols]; rms: float [rows] from the forward.
 * The workspace holds the per-workgroup partial sums of dw.
 */
SMLM_API int smlm_rms_norm_bwd_workspace_size(int rows, int cols, size_t* bytes);
SMLM_API int smlm_rms_norm_bwd(void* dx, void* dw, const void* g, const void* x, const void* w,
                               const float* rms, void* workspace, size_t workspace_bytes, int rows,
                               int cols, int dtype, void* stream);

/*
 * Run-length segments of a flat batch, built on the device.  Replaces the host
 * loop of ModelGeneration.generate (src/loquetier_src/model_generation.py:267-283):
 * consecutive requests with the same adapter id merge into one segment; its
 * length is the sum of their token counts, seg_indptr the running sum from 0.
 *   req_adapter, req_len : int32 [R] on the device (negative lengths count as 0)
 *   seg_adapter, seg_len : int32 [R];  seg_indptr : int32 [R + 1];  n_seg : int32 [2]
 * The segment count stays on the device (n_seg[0]; n_seg[1] = total rows), so the
 * outputs have capacity R: entries past the last segment are empty segments
 * (indptr = total rows, length 0, the last request's adapter id).  Pass them on
 * with S = R; empty segments cost nothing in the plan.  R == 0 writes
 * seg_indptr[0] = 0 and n_seg = {0, 0}.
 */
SMLM_API int smlm_segments_build(const int32_t* req_adapter, const int32_t* req_len, int R,
                                 int32_t* seg_adapter, int32_t* seg_len, int32_t* seg_indptr,
                                 int32_t* n_seg, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SMLM_H_ */
