"""GPU parity tests: the HIP kernels, called through the C ABI (ctypes) behind
the reference's Python operator surface, against the CPU oracle on the same
seeded inputs.

Bars (BASELINE north star): segment / adapter routing bit-exact; fp16 / bf16
outputs and gradients within rtol 1e-2 / atol 1e-3 of the fp32 host reference
(the oracle accumulating in double).

Two kinds of inputs are used.  "dyadic" inputs (small multiples of powers of
two) make every product and partial sum exactly representable in fp32, so the
order of accumulation cannot matter and the HIP result must equal the oracle
BIT FOR BIT, forward and backward, at any size -- this is how the full
BASELINE sizes are checked.  Gaussian inputs are checked to the tolerance
above; where the rank-r intermediate is rounded to bf16 a different rounding
of one v element (fp32 vs double accumulation) moves a whole output row by up
to one bf16 ulp of v times |B|, so bf16 Gaussian cases check each GEMM stage
against the oracle fed with the same stage input, and bf16 gradients use the
atol stated in the test.
"""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "smlm_small.npz")
TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}


@pytest.fixture(scope="module")
def K(gpu_device):
    from loquetier_amd import _lib
    from loquetier_amd.ops import _kernels
    _lib.load()  # raises if the HIP library is not built: there is no fallback
    return _kernels


def dev_t(a, dt, dev):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dev).to(TDT[dt]).contiguous()


def to_np(t):
    return t.detach().float().cpu().numpy()


def ptrs(ts, dev):
    return torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=dev)


def dyadic(rng, shape, lim, denom):
    """Multiples of 1/denom in [-lim/denom, lim/denom]: exact in fp16 and bf16."""
    return (rng.integers(-lim, lim + 1, shape) / float(denom)).astype(np.float32)


def make_case(oracle, seed, T, seg, ids, NA, h_in, h_out, r, dt, ints=False, dy=False):
    rng = np.random.default_rng(seed)
    if ints:
        x = rng.integers(-2, 3, (T, h_in)).astype(np.float32)
        A = [rng.integers(-1, 2, (r, h_in)).astype(np.float32) for _ in range(NA)]
        B = [rng.integers(-1, 2, (h_out, r)).astype(np.float32) for _ in range(NA)]
    elif dy:
        x = dyadic(rng, (T, h_in), 16, 8)
        A = [dyadic(rng, (r, h_in), 8, 64) for _ in range(NA)]
        B = [dyadic(rng, (h_out, r), 8, 8) for _ in range(NA)]
    else:
        x = oracle.round_to(rng.standard_normal((T, h_in)), dt)
        A = [oracle.round_to(rng.standard_normal((r, h_in)) / np.sqrt(h_in), dt) for _ in range(NA)]
        B = [oracle.round_to(rng.standard_normal((h_out, r)) / np.sqrt(r), dt) for _ in range(NA)]
    return x, A, B


def close(got, want, rtol=RTOL, atol=ATOL):
    err = np.abs(got - want)
    bad = err > atol + rtol * np.abs(want)
    assert not bad.any(), f"max err {err.max():.4g}, {bad.sum()} of {bad.size} outside tolerance"


# ---------------------------------------------------------------- forward ---
FWD_CASES = [
    # name, T, seg, ids, NA, h_in, h_out, r
    ("tiny-with-empty-segment", 13, [0, 5, 5, 9, 13], [2, 0, 2, 1], 3, 64, 96, 8),
    ("one-segment", 16, [0, 16], [0], 1, 128, 128, 16),
    ("ragged", 77, [0, 1, 18, 18, 50, 51, 52, 77], [3, 1, 2, 1, 0, 3, 1], 4, 256, 320, 32),
    ("uncovered-rows", 40, [3, 10, 31], [1, 0], 2, 64, 64, 16),
    ("uncovered-rows-long-k", 75, [5, 22, 22, 60], [1, 0, 1], 2, 4096, 64, 16),  # k split and folded
    # more segments than the one-workgroup plan takes, first rows uncovered, k split and folded row by row
    ("many-segments-offset", 1600, list(range(7, 1508)), [i % 5 for i in range(1500)], 5, 2048, 64, 16),
    ("rank64", 45, [0, 20, 45], [0, 1], 2, 512, 256, 64),
    ("rank24", 33, [0, 33], [0], 1, 96, 136, 24),
    ("rank128", 45, [0, 20, 45], [0, 1], 2, 512, 256, 128),   # ranks above 64: general k loop in the expand
    ("rank72", 33, [0, 33], [0], 1, 96, 136, 72),
    ("decode", 64, list(range(65)), [i % 5 for i in range(64)], 5, 512, 512, 16),
]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", FWD_CASES, ids=[c[0] for c in FWD_CASES])
def test_reference_two_call_forward(K, oracle, gpu_device, case, dt):
    """kernel.smlm_forward_cutlass twice, exactly as add_lora.forward calls it
    (kernel_utils.py:115-119), against oracle_add_lora_forward."""
    name, T, seg, ids, NA, h_in, h_out, r = case
    x, A, B = make_case(oracle, 100, T, seg, ids, NA, h_in, h_out, r, dt)
    d = gpu_device
    xd = dev_t(x, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    wa, wb = ptrs([Ad[i] for i in ids], d), ptrs([Bd[i] for i in ids], d)
    tmp = torch.empty(K.smlm_forward_cutlass_tmp_size(len(ids)), dtype=torch.uint8, device=d)
    v = torch.full((T, r), 3.0, dtype=TDT[dt], device=d)
    y = torch.full((T, h_out), 5.0, dtype=TDT[dt], device=d)
    K.smlm_forward_cutlass(v, xd, wa, s, tmp, False)
    K.smlm_forward_cutlass(y, v, wb, s, tmp, False)
    y0 = np.full((T, h_out), 5.0, np.float32)
    yo, vo = oracle.add_lora_forward(x, [A[i] for i in ids], [B[i] for i in ids], seg, h_out, dt, y_init=y0)
    vo_full = np.full((T, r), 3.0, np.float32)
    for i in range(len(ids)):
        vo_full[seg[i]:seg[i + 1]] = vo[seg[i]:seg[i + 1]]
    close(to_np(v), vo_full)
    # expand stage against the oracle fed with the v the shrink stage produced
    y_stage = np.full((T, h_out), 5.0, np.float32)
    oracle.smlm_gemm(y_stage, to_np(v), [B[i] for i in ids], seg, False, dt)
    close(to_np(y), y_stage)
    if dt == "fp16":
        close(to_np(y), yo)  # end to end as well
    # rows outside every segment keep their old contents, bit for bit
    covered = np.zeros(T, bool)
    for i in range(len(ids)):
        covered[seg[i]:seg[i + 1]] = True
    assert np.all(to_np(y)[~covered] == 5.0) and np.all(to_np(v)[~covered] == 3.0)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", FWD_CASES, ids=[c[0] for c in FWD_CASES])
def test_fused_forward_accumulate(K, oracle, gpu_device, case, dt):
    """y += scale_seg * round(x A^T) B^T in one call, adapter-id indirection."""
    name, T, seg, ids, NA, h_in, h_out, r = case
    x, A, B = make_case(oracle, 101, T, seg, ids, NA, h_in, h_out, r, dt)
    rng = np.random.default_rng(5)
    base = oracle.round_to(rng.standard_normal((T, h_out)), dt)
    scale = (rng.integers(1, 5, len(ids)) / 2.0).astype(np.float32)
    d = gpu_device
    xd, yd = dev_t(x, dt, d), dev_t(base, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    ids_t = torch.tensor(ids, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(s, ids_t, T)
    v = torch.zeros(T, r, dtype=TDT[dt], device=d)
    K.smlm_lora_forward(yd, xd, ptrs(Ad, d), ptrs(Bd, d), plan, r,
                        seg_scale=torch.from_numpy(scale).to(d), beta=1.0, v_out=v)
    yo, vo = oracle.lora_fused(base, x, [A[i] for i in ids], [B[i] for i in ids], seg, scale, 1.0, dt)
    covered = np.zeros(T, bool)
    for i in range(len(ids)):
        covered[seg[i]:seg[i + 1]] = True
    close(to_np(v)[covered], vo[covered])
    # epilogue against the oracle fed with the kernel's own v: beta*y0 + scale*(v B^T), one rounding
    acc = np.zeros((T, h_out), np.float32)
    oracle.smlm_gemm(acc, to_np(v), [B[i] for i in ids], seg, False, "fp32")
    row_scale = np.ones(T, np.float32)
    for i in range(len(ids)):
        row_scale[seg[i]:seg[i + 1]] = scale[i]
    staged = oracle.round_to(base + row_scale[:, None] * acc, dt)
    close(to_np(yd)[covered], staged[covered])
    if dt == "fp16":
        close(to_np(yd), yo)
    assert np.array_equal(to_np(yd)[~covered], base[~covered])
    n_tiles, n_groups, rows, kind = plan.header()
    assert rows == covered.sum() and kind == 1
    assert n_groups == len(set(ids))


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_routing_bit_exact_small_integers(K, oracle, gpu_device, dt):
    """Exact inputs: a wrong adapter, row or segment edge changes bits."""
    T, h_in, h_out, r, NA = 150, 64, 96, 8, 6
    rng = np.random.default_rng(7)
    cuts = np.sort(rng.choice(np.arange(1, T), 40, replace=False))
    seg = [0] + cuts.tolist() + [T]
    seg = seg[:10] + [seg[10]] + seg[10:]           # one empty segment
    ids = rng.integers(0, NA, len(seg) - 1).tolist()
    x, A, B = make_case(oracle, 102, T, seg, ids, NA, h_in, h_out, r, dt, ints=True)
    d = gpu_device
    xd = dev_t(x, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    yo, vo = oracle.add_lora_forward(x, [A[i] for i in ids], [B[i] for i in ids], seg, h_out, dt)
    ids_t = torch.tensor(ids, dtype=torch.int32, device=d)
    for key in (None, ids_t, ptrs([Ad[i] for i in ids], d)):   # ungrouped, by id, by address
        plan = K.SegmentPlan(s, key, T)
        y = torch.zeros(T, h_out, dtype=TDT[dt], device=d)
        v = torch.zeros(T, r, dtype=TDT[dt], device=d)
        tabs = (ptrs(Ad, d), ptrs(Bd, d)) if key is ids_t else \
            (ptrs([Ad[i] for i in ids], d), ptrs([Bd[i] for i in ids], d))
        K.smlm_lora_forward(y, xd, tabs[0], tabs[1], plan, r, v_out=v)
        assert np.array_equal(to_np(v), vo)
        assert np.array_equal(to_np(y), yo)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_resegmenting_changes_no_bit(K, oracle, gpu_device, dt):
    """Same rows, same adapters per row, different segmentations and groupings:
    outputs are bit-identical (each row's reduction order is fixed)."""
    T, h_in, h_out, r, NA = 200, 1024, 768, 16, 3
    rng = np.random.default_rng(8)
    row_ad = np.repeat(rng.integers(0, NA, 20), 10)          # adapter of every row, runs of 10
    x, A, B = make_case(oracle, 103, T, None, None, NA, h_in, h_out, r, dt)
    d = gpu_device
    xd = dev_t(x, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]

    def run(seg, ids, key_kind):
        s = torch.tensor(seg, dtype=torch.int32, device=d)
        ids_t = torch.tensor(ids, dtype=torch.int32, device=d)
        plan = K.SegmentPlan(s, ids_t if key_kind else None, T)
        y = torch.zeros(T, h_out, dtype=TDT[dt], device=d)
        if key_kind:
            K.smlm_lora_forward(y, xd, ptrs(Ad, d), ptrs(Bd, d), plan, r)
        else:
            K.smlm_lora_forward(y, xd, ptrs([Ad[i] for i in ids], d), ptrs([Bd[i] for i in ids], d), plan, r)
        return y

    per_row = run(list(range(T + 1)), row_ad.tolist(), 1)                  # one segment per row
    runs10 = run(list(range(0, T + 1, 10)), row_ad[::10].tolist(), 1)      # runs of 10
    merged_seg, merged_ids = [0], []
    for t in range(T):                                                     # maximal runs
        if t == 0 or row_ad[t] != row_ad[t - 1]:
            if t:
                merged_seg.append(t)
            merged_ids.append(int(row_ad[t]))
    merged_seg.append(T)
    merged = run(merged_seg, merged_ids, 1)
    ungrouped = run(list(range(0, T + 1, 10)), row_ad[::10].tolist(), 0)
    assert torch.equal(per_row, runs10) and torch.equal(per_row, merged) and torch.equal(per_row, ungrouped)
    yo, _ = oracle.add_lora_forward(x, [A[i] for i in merged_ids], [B[i] for i in merged_ids],
                                    merged_seg, h_out, dt)
    close(to_np(per_row), yo)


@pytest.mark.parametrize("row_major", [False, True])
@pytest.mark.parametrize("shape", [(256, 128), (64, 4096), (1024, 16), (96, 96), (40, 8), (8, 40)])
def test_generic_grouped_gemm_shapes_and_layouts(K, oracle, gpu_device, shape, row_major):
    """smlm_forward_cutlass as a plain grouped GEMM: any d_in / d_out (multiples
    of 8), both weight layouts (loquetier_ops.cc:297-303)."""
    d_in, d_out = shape
    dt = "fp16"
    T, seg = 50, [0, 7, 30, 50]
    rng = np.random.default_rng(9)
    x = oracle.round_to(rng.standard_normal((T, d_in)), dt)
    W = [oracle.round_to(rng.standard_normal((d_in, d_out)) / np.sqrt(d_in), dt) for _ in range(3)]
    w_in = [w if row_major else np.ascontiguousarray(w.T) for w in W]
    d = gpu_device
    xd = dev_t(x, dt, d)
    wd = [dev_t(w, dt, d) for w in w_in]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    tmp = torch.empty(K.smlm_forward_cutlass_tmp_size(3), dtype=torch.uint8, device=d)
    y = torch.zeros(T, d_out, dtype=TDT[dt], device=d)
    K.smlm_forward_cutlass(y, xd, ptrs(wd, d), s, tmp, row_major)
    yo = np.zeros((T, d_out), np.float32)
    oracle.smlm_gemm(yo, x, w_in, seg, row_major, dt)
    close(to_np(y), yo)


def test_reference_call_with_a_tmp_that_holds_all_its_scratch(K, oracle, gpu_device):
    """A tmp of smlm_forward_cutlass_workspace_size bytes is the call's only scratch (the reference's
    ownership rule: everything through tmp, kernel_src/csrc/loquetier_ops.cc:304): same results as with the
    reference-sized tmp, and the bytes of the large tmp are the ones that get written."""
    name, T, seg, ids, NA, h_in, h_out, r = FWD_CASES[1]
    dt, d = "fp16", gpu_device
    x, A, B = make_case(oracle, 100, T, seg, ids, NA, h_in, h_out, r, dt)
    xd = dev_t(x, dt, d)
    Ad = [dev_t(a, dt, d) for a in A]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    wa = ptrs([Ad[i] for i in ids], d)
    small = torch.empty(K.smlm_forward_cutlass_tmp_size(len(ids)), dtype=torch.uint8, device=d)
    need = K.smlm_forward_cutlass_workspace_size(T, len(ids), h_in, r)
    assert need > small.numel()
    large = torch.full((need + 64,), 0xA5, dtype=torch.uint8, device=d)
    v1 = torch.full((T, r), 3.0, dtype=TDT[dt], device=d)
    v2 = torch.full((T, r), 3.0, dtype=TDT[dt], device=d)
    K.smlm_forward_cutlass(v1, xd, wa, s, small, False)
    K.smlm_forward_cutlass(v2, xd, wa, s, large, False)
    assert torch.equal(v1, v2)
    assert bool((large[:need] != 0xA5).any()) and bool((large[need:] == 0xA5).all())
    with pytest.raises(RuntimeError, match="aligned"):
        K.smlm_forward_cutlass(v2, xd, wa, s, torch.empty(need + 24, dtype=torch.uint8, device=d)[8:], False)


def test_reference_error_behaviour(K, gpu_device):
    d = gpu_device
    x32 = torch.zeros(4, 16, device=d)
    y32 = torch.zeros(4, 8, device=d)
    w = torch.zeros(1, dtype=torch.int64, device=d)
    s = torch.tensor([0, 4], dtype=torch.int32, device=d)
    tmp = torch.empty(K.smlm_forward_cutlass_tmp_size(1), dtype=torch.uint8, device=d)
    with pytest.raises(RuntimeError, match="No suitable kernel"):
        K.smlm_forward_cutlass(y32, x32, w, s, tmp, False)     # fp32: reference has no kernel either
    x = torch.zeros(4, 32, dtype=torch.float16, device=d)
    y = torch.zeros(4, 8, dtype=torch.float16, device=d)
    with pytest.raises(RuntimeError, match="contiguous"):
        K.smlm_forward_cutlass(y, x[:, ::2], w, s, tmp, False)
    with pytest.raises(RuntimeError, match="tmp"):
        K.smlm_forward_cutlass(y, x, w, s, tmp[:-1], False)
    with pytest.raises(RuntimeError, match="2D"):
        K.smlm_forward_cutlass(y[0], x, w, s, tmp, False)
    # an all-empty batch is a no-op
    s0 = torch.tensor([0, 0], dtype=torch.int32, device=d)
    y.fill_(1.0)
    K.smlm_forward_cutlass(y, x, w, s0, tmp, False)
    torch.cuda.synchronize()
    assert bool((y == 1.0).all())


@pytest.mark.parametrize("dt", ["fp32", "fp16", "bf16"])
def test_golden_fixture(K, gpu_device, dt):
    """Committed vectors (tests/golden/make_fixtures.py, numpy float64)."""
    z = np.load(GOLDEN)
    if dt == "fp32":
        pytest.skip("fp32 I/O has no kernel, as in the reference (loquetier_ops.cc:69-71)")
    from loquetier_amd.kernel_utils import add_lora
    d = gpu_device
    seg, ids, tp, tp_ad = z["seg"], z["ids"], z["tp"], z["tp_ad"]
    x = dev_t(z[f"{dt}_x"], dt, d).requires_grad_(True)
    A = [dev_t(a, dt, d).requires_grad_(True) for a in z[f"{dt}_A"]]
    B = [dev_t(b, dt, d).requires_grad_(True) for b in z[f"{dt}_B"]]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    wa, wb = ptrs([A[i] for i in ids], d), ptrs([B[i] for i in ids], d)
    weights = [w for ad in tp_ad for w in (A[ad], B[ad])]
    y = add_lora.apply((x.size(0), B[0].size(0)), x, wa, wb, s, A[0].size(0), int(tp[-1]),
                       tp.tolist(), *weights)
    close(to_np(y), z[f"{dt}_y"])
    y.backward(dev_t(z[f"{dt}_g"], dt, d))
    close(to_np(x.grad), z[f"{dt}_dx"])
    assert not to_np(x.grad)[int(tp[-1]):].any()
    close(to_np(A[2].grad), z[f"{dt}_dA"][2], atol=2e-2)
    close(to_np(B[2].grad), z[f"{dt}_dB"][2], atol=2e-2)
    assert A[0].grad is None and A[1].grad is None  # not passed as trainable


def _bwd_exact(K, oracle, d, dt, x, A, B, g, tp, part_ad, r, scale=None):
    n_rows, NA = tp[-1], len(A)
    xd, gd = dev_t(x, dt, d), dev_t(g, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    dA, dB = [torch.empty_like(a) for a in Ad], [torch.empty_like(b) for b in Bd]
    dx = torch.empty(n_rows, x.shape[1], dtype=TDT[dt], device=d)
    pi = torch.tensor(tp, dtype=torch.int32, device=d)
    pa = torch.tensor(part_ad, dtype=torch.int32, device=d)
    K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), gd, xd, None, ptrs(Ad, d), ptrs(Bd, d),
                         K.SegmentPlan(pi, pa, n_rows), r)
    gx, ga, gb = oracle.add_lora_backward(g, x, A, B, tp, part_ad, dt)
    covered = np.zeros(n_rows, bool)
    for p in range(len(part_ad)):
        covered[tp[p]:tp[p + 1]] = True
    assert np.array_equal(to_np(dx)[covered], gx[covered])
    for a in range(NA):
        assert np.array_equal(to_np(dA[a]), ga[a]), f"dA[{a}]"
        assert np.array_equal(to_np(dB[a]), gb[a]), f"dB[{a}]"


def _fwd_exact(K, oracle, d, dt, x, A, B, seg, ids, r, base, scale_val=2.0):
    T, h_out = x.shape[0], B[0].shape[0]
    xd, yd = dev_t(x, dt, d), dev_t(base, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    ids_t = torch.tensor(ids, dtype=torch.int32, device=d)
    v = torch.zeros(T, r, dtype=TDT[dt], device=d)
    sc = torch.full((len(ids),), scale_val, device=d)
    K.smlm_lora_forward(yd, xd, ptrs(Ad, d), ptrs(Bd, d), K.SegmentPlan(s, ids_t, T), r,
                        seg_scale=sc, beta=1.0, v_out=v)
    yo, vo = oracle.lora_fused(base, x, [A[i] for i in ids], [B[i] for i in ids], seg,
                               [scale_val] * len(ids), 1.0, dt)
    assert np.array_equal(to_np(v), vo), "v differs"
    assert np.array_equal(to_np(yd), yo), "y differs"
    return yd


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", FWD_CASES, ids=[c[0] for c in FWD_CASES])
def test_forward_dyadic_bit_exact(K, oracle, gpu_device, case, dt):
    """Exactly representable sums: v and y equal the oracle bit for bit."""
    name, T, seg, ids, NA, h_in, h_out, r = case
    x, A, B = make_case(oracle, 201, T, seg, ids, NA, h_in, h_out, r, dt, dy=True)
    base = dyadic(np.random.default_rng(22), (T, h_out), 16, 8)
    _fwd_exact(K, oracle, gpu_device, dt, x, A, B, seg, ids, r, base)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [
    # T, S, NA, h_in, h_out, r: the tile-block expand's launch shapes
    (4096, 37, 5, 128, 8192, 16),    # 4096 rows and a row stride of 16 KiB: 256 columns a workgroup
    (4100, 21, 3, 64, 10240, 32),    # the same at rank 32, rows past a multiple of 64
    (8192, 90, 7, 64, 768, 64),      # rank 64 at 8192 rows: 256 columns, three chunk rows rounded up to four
    (8200, 50, 6, 64, 1032, 48),     # ... and a width that ends inside a chunk (five chunk rows -> six)
    (2600, 12, 4, 64, 640, 16),      # 128 columns, five chunk rows rounded up to six
    (1100, 12, 4, 64, 1160, 64),     # 128 columns at rank 64 below 8192 rows, ragged last chunk (ten rows)
    (4100, 15, 3, 11008, 128, 64),   # k = 11008 split in five, ragged last slice: one empty chunk row
    (6200, 9, 2, 4096, 64, 64),      # ... k split in three: one empty chunk row
], ids=["r16-wide-aligned", "r32-wide-aligned", "r64-8192-rows", "r48-ragged-width", "odd-chunk-rows", "r64-short",
        "k-split-five", "k-split-three"])
def test_forward_expand_launch_shapes(K, oracle, gpu_device, shape, dt):
    """The widths, row counts and ranks at which the tile-block launches change their columns per
    workgroup, their k split or pad their grid: bit-exact against the oracle."""
    T, S, NA, h_in, h_out, r = shape
    rng = np.random.default_rng(47)
    seg = _ragged_segments(rng, T, S)
    ids = rng.integers(0, NA, S).tolist()
    x, A, B = make_case(oracle, 207, T, seg, ids, NA, h_in, h_out, r, dt, dy=True)
    base = dyadic(np.random.default_rng(23), (T, h_out), 16, 8)
    _fwd_exact(K, oracle, gpu_device, dt, x, A, B, seg, ids, r, base)


def _ragged_segments(rng, T, S):
    cuts = np.sort(rng.choice(np.arange(1, T), S - 1, replace=False))
    return [0] + cuts.tolist() + [T]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [
    # T, S, NA, h_in, h_out, r: tile blocks of four (larger batches: from 512 rows at rank 64 to 2560 at rank 16), ragged groups
    (1500, 40, 7, 512, 768, 32),
    (2600, 300, 5, 256, 264, 16),
    (1100, 3, 3, 128, 1024, 64),
    # more than 1024 segments: two-launch plan with the sort in LDS
    (3000, 1500, 37, 128, 160, 8),
    # more than 4096 segments: the sort runs in global memory
    (5000, 5000, 61, 64, 128, 8),
], ids=["blocks-ragged", "blocks-many-segs", "blocks-long", "plan-two-launch", "plan-global-sort"])
def test_forward_dyadic_bit_exact_larger(K, oracle, gpu_device, shape, dt):
    T, S, NA, h_in, h_out, r = shape
    rng = np.random.default_rng(31)
    seg = list(range(T + 1)) if S == T else _ragged_segments(rng, T, S)
    ids = rng.integers(0, NA, S).tolist()
    x, A, B = make_case(oracle, 202, T, seg, ids, NA, h_in, h_out, r, dt, dy=True)
    base = dyadic(rng, (T, h_out), 16, 8)
    _fwd_exact(K, oracle, gpu_device, dt, x, A, B, seg, ids, r, base)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [
    # T, S, NA, h_in, h_out, r: few rows and a long k -> eight-wave shrink with k split over
    # four workgroups, partial sums folded by the expand kernel
    (1, 1, 1, 4096, 512, 16),
    (17, 17, 5, 4096, 1024, 8),
    (256, 256, 32, 4096, 640, 16),
    (200, 23, 9, 11008, 512, 32),     # k not a multiple of the waves' share: ragged last batch
    (1000, 61, 7, 2048, 1536, 64),    # shortest k that takes the eight-wave route at rank 64
    (96, 10, 3, 4104, 264, 24),       # k and rank off the round sizes
    (300, 30, 4, 2040, 512, 16),      # just below the route's minimum k: four-wave shrink
], ids=["one-row", "r8", "decode-256", "k11008", "r64-k2048", "odd-sizes", "below-min-k"])
def test_forward_dyadic_bit_exact_decode_route(K, oracle, gpu_device, shape, dt):
    T, S, NA, h_in, h_out, r = shape
    rng = np.random.default_rng(41)
    seg = list(range(T + 1)) if S == T else _ragged_segments(rng, T, S)
    ids = rng.integers(0, NA, S).tolist()
    x, A, B = make_case(oracle, 203, T, seg, ids, NA, h_in, h_out, r, dt, dy=True)
    base = dyadic(rng, (T, h_out), 16, 8)
    _fwd_exact(K, oracle, gpu_device, dt, x, A, B, seg, ids, r, base)


@pytest.mark.parametrize("keyed", [True, False], ids=["distinct-ids", "no-key"])
def test_one_launch_plan_with_as_many_groups_as_segments(K, oracle, gpu_device, keyed):
    """The largest batch the one-workgroup plan takes (1024 segments) with every segment a group
    of its own -- 1024 distinct adapters, or a plan without keys: the group tables then have
    their last entry at index 1024."""
    T = S = 1024
    NA, h_in, h_out, r, dt = 1024, 64, 64, 8, "bf16"
    rng = np.random.default_rng(53)
    seg = list(range(T + 1))
    ids = rng.permutation(NA).tolist()
    x, A, B = make_case(oracle, 205, T, seg, ids, NA, h_in, h_out, r, dt, dy=True)
    base = dyadic(rng, (T, h_out), 16, 8)
    d = gpu_device
    if keyed:
        _fwd_exact(K, oracle, d, dt, x, A, B, seg, ids, r, base)
        return
    xd, yd = dev_t(x, dt, d), dev_t(base, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    plan = K.SegmentPlan(torch.tensor(seg, dtype=torch.int32, device=d), None, T)
    assert plan.header()[1] == S
    K.smlm_lora_forward(yd, xd, ptrs([Ad[i] for i in ids], d), ptrs([Bd[i] for i in ids], d), plan, r,
                        seg_scale=torch.full((S,), 2.0, device=d), beta=1.0)
    yo, _ = oracle.lora_fused(base, x, [A[i] for i in ids], [B[i] for i in ids], seg, [2.0] * S, 1.0, dt)
    assert np.array_equal(to_np(yd), yo)


def test_forward_beyond_the_direct_grid(K, oracle, gpu_device):
    """More than 65535 tile units: the launches fall back to the persistent walk over the
    plan's exact tile count (and the plan to its two-launch route).  Bit-exact on dyadic
    inputs, narrow matrices so that a million rows stay small."""
    T, S, NA, h_in, h_out, r, dt = 1_050_000, 64, 5, 64, 64, 8, "bf16"
    rng = np.random.default_rng(47)
    seg = _ragged_segments(rng, T, S)
    ids = rng.integers(0, NA, S).tolist()
    x, A, B = make_case(oracle, 204, T, seg, ids, NA, h_in, h_out, r, dt, dy=True)
    base = dyadic(rng, (T, h_out), 16, 8)
    _fwd_exact(K, oracle, gpu_device, dt, x, A, B, seg, ids, r, base)


def test_multi_projection_mixed_routes_equal_single_calls(K, oracle, gpu_device):
    """Projections of one launch with different k: all long (eight-wave route with a different
    k split each) and one short (which sends the whole launch down the four-wave route)."""
    d, dt = gpu_device, "fp16"
    T, r, NA, S = 120, 16, 5, 14
    rng = np.random.default_rng(43)
    seg = _ragged_segments(rng, T, S)
    ids = rng.integers(0, NA, S).tolist()
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(s, torch.tensor(ids, dtype=torch.int32, device=d), T)
    sc = torch.full((S,), 2.0, device=d)
    for dims in ([(4096, 512), (11008, 256), (2048, 1024)], [(4096, 512), (512, 512)]):
        projs = []
        for hi, ho in dims:
            A = [dev_t(dyadic(rng, (r, hi), 8, 64), dt, d) for _ in range(NA)]
            B = [dev_t(dyadic(rng, (ho, r), 8, 8), dt, d) for _ in range(NA)]
            projs.append(dict(x=dev_t(dyadic(rng, (T, hi), 16, 8), dt, d), a=ptrs(A, d), b=ptrs(B, d), A=A, B=B,
                              y0=dev_t(dyadic(rng, (T, ho), 16, 8), dt, d)))
        single, single_v = [], []
        for p in projs:
            y, v = p["y0"].clone(), torch.zeros(T, r, dtype=TDT[dt], device=d)
            K.smlm_lora_forward(y, p["x"], p["a"], p["b"], plan, r, seg_scale=sc, beta=1.0, v_out=v)
            single.append(y)
            single_v.append(v)
        ys = [p["y0"].clone() for p in projs]
        vs = [torch.zeros(T, r, dtype=TDT[dt], device=d) for _ in projs]
        K.smlm_lora_forward_multi(ys, [p["x"] for p in projs], [p["a"] for p in projs],
                                  [p["b"] for p in projs], plan, r, seg_scale=sc, beta=1.0, v_out=vs)
        for a, b in zip(single + single_v, ys + vs):
            assert torch.equal(a, b)
        # and without the copy of v, and as two separately issued stages
        ys2 = [p["y0"].clone() for p in projs]
        args = ([p["x"] for p in projs], [p["a"] for p in projs], [p["b"] for p in projs], plan, r)
        K.smlm_lora_forward_multi(ys2, *args, seg_scale=sc, beta=1.0, stages=1)
        K.smlm_lora_forward_multi(ys2, *args, seg_scale=sc, beta=1.0, stages=2)
        for a, b in zip(single, ys2):
            assert torch.equal(a, b)


def test_multi_projection_equals_single_calls(K, oracle, gpu_device):
    """q/k/v/o-style batched launch: bit-identical to one call per projection,
    with different widths per projection and a shared x for three of them."""
    d, dt = gpu_device, "bf16"
    T, r, NA = 300, 16, 6
    rng = np.random.default_rng(32)
    seg = _ragged_segments(rng, T, 25)
    ids = rng.integers(0, NA, 25).tolist()
    dims = [(512, 512), (512, 128), (512, 128), (384, 640)]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    ids_t = torch.tensor(ids, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(s, ids_t, T)
    sc = torch.full((25,), 0.5, device=d)
    xs_np = {512: oracle.round_to(rng.standard_normal((T, 512)), dt),
             384: oracle.round_to(rng.standard_normal((T, 384)), dt)}
    xs_dev = {k: dev_t(v, dt, d) for k, v in xs_np.items()}
    projs = []
    for hi, ho in dims:
        A = [dev_t(oracle.round_to(rng.standard_normal((r, hi)) / np.sqrt(hi), dt), dt, d) for _ in range(NA)]
        B = [dev_t(oracle.round_to(rng.standard_normal((ho, r)) / 4, dt), dt, d) for _ in range(NA)]
        y0 = dev_t(oracle.round_to(rng.standard_normal((T, ho)), dt), dt, d)
        projs.append(dict(x=xs_dev[hi], A=A, B=B, a=ptrs(A, d), b=ptrs(B, d), y0=y0))
    single, single_v = [], []
    for p in projs:
        y, v = p["y0"].clone(), torch.zeros(T, r, dtype=TDT[dt], device=d)
        K.smlm_lora_forward(y, p["x"], p["a"], p["b"], plan, r, seg_scale=sc, beta=1.0, v_out=v)
        single.append(y)
        single_v.append(v)
    ys = [p["y0"].clone() for p in projs]
    vs = [torch.zeros(T, r, dtype=TDT[dt], device=d) for _ in projs]
    K.smlm_lora_forward_multi(ys, [p["x"] for p in projs], [p["a"] for p in projs],
                              [p["b"] for p in projs], plan, r, seg_scale=sc, beta=1.0, v_out=vs)
    for a, b in zip(single + single_v, ys + vs):
        assert torch.equal(a, b)


# --------------------------------------------------------------- backward ---
BWD_CASES = [
    # name, tp, part_ad, NA, n_infer_rows, h_in, h_out, r
    ("two-parts", [0, 5, 12], [0, 1], 2, 3, 64, 96, 8),
    ("blocks", [0, 500, 520, 1300], [2, 0, 2], 3, 7, 256, 192, 16),
    ("shared-adapter", [0, 40, 70, 100], [1, 0, 1], 2, 5, 128, 256, 16),
    ("empty-part", [0, 17, 17, 50], [0, 1, 2], 3, 0, 256, 128, 32),
    ("rank64", [0, 33, 90], [0, 1], 2, 4, 192, 320, 64),
    ("long", [0, 300, 700], [1, 0], 2, 20, 512, 384, 16),
    # ranks above 64 (PEFT ranks 128 / 256 are ordinary): general k loop in the dX expand, the weight
    # gradient covers the rank 64 at a time
    ("rank128", [0, 33, 90], [0, 1], 2, 4, 192, 320, 128),
    ("rank72", [0, 50], [0], 1, 0, 128, 136, 72),
    ("rank256-blocks", [0, 600, 1100], [1, 0], 2, 3, 256, 192, 256),
    # few rows and long k: the eight-wave shrink (k split over workgroups, folded by a launch) for v and dV
    ("long-k", [0, 30, 75], [1, 0], 2, 4, 4096, 2048, 16),
    # more adapters than partitions, most of them without rows (zero gradients), ids not dense
    ("idle-adapters", [0, 40, 90], [4, 1], 6, 2, 128, 192, 16),
]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("with_v", [True, False])
@pytest.mark.parametrize("case", BWD_CASES, ids=[c[0] for c in BWD_CASES])
def test_backward_against_oracle(K, oracle, gpu_device, case, dt, with_v):
    name, tp, part_ad, NA, n_inf, h_in, h_out, r = case
    n_rows = tp[-1]
    T = n_rows + n_inf
    x, A, B = make_case(oracle, 104, T, None, None, NA, h_in, h_out, r, dt)
    rng = np.random.default_rng(11)
    g = oracle.round_to(rng.standard_normal((T, h_out)), dt)
    d = gpu_device
    xd, gd = dev_t(x, dt, d), dev_t(g, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    dA = [torch.full_like(a, 9.0) for a in Ad]
    dB = [torch.full_like(b, 9.0) for b in Bd]
    dx = torch.full((T, h_in), 9.0, dtype=TDT[dt], device=d)
    pi = torch.tensor(tp, dtype=torch.int32, device=d)
    pa = torch.tensor(part_ad, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(pi, pa, n_rows)
    v = None
    if with_v:
        _, vo = oracle.add_lora_forward(x[:n_rows], [A[a] for a in part_ad], [B[a] for a in part_ad],
                                        tp, h_out, dt)
        v = dev_t(vo, dt, d)
    K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), gd, xd, v, ptrs(Ad, d), ptrs(Bd, d), plan, r)
    gx, ga, gb = oracle.add_lora_backward(g[:n_rows], x[:n_rows], A, B, tp, part_ad, dt)
    # bf16: dV (|dV| up to ~8) is rounded to 8 bits inside the op; one element
    # rounding the other way moves a dX row by 2^-8 |dV| |A| ~ 4e-3
    close(to_np(dx)[:n_rows], gx, atol=ATOL if dt == "fp16" else 4e-3)
    assert np.all(to_np(dx)[n_rows:] == 9.0)  # rows past the partitions are the caller's
    for a in range(NA):
        # sums over up to 400 tokens of O(1) products: atol scaled to the result's size
        close(to_np(dA[a]), ga[a], atol=ATOL * max(1.0, float(np.abs(ga[a]).max())))
        close(to_np(dB[a]), gb[a], atol=ATOL * max(1.0, float(np.abs(gb[a]).max())))


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", BWD_CASES, ids=[c[0] for c in BWD_CASES])
def test_backward_dyadic_bit_exact(K, oracle, gpu_device, case, dt):
    """Exactly representable sums: dX, dA, dB equal the oracle bit for bit."""
    name, tp, part_ad, NA, n_inf, h_in, h_out, r = case
    n_rows = tp[-1]
    x, A, B = make_case(oracle, 204, n_rows, None, None, NA, h_in, h_out, r, dt, dy=True)
    g = dyadic(np.random.default_rng(21), (n_rows, h_out), 16, 8)
    _bwd_exact(K, oracle, gpu_device, dt, x, A, B, g, tp, part_ad, r)


@pytest.mark.parametrize("case", [
    # n_rows, partitions, NA, h_in, h_out, r: shapes at which the backward's products, always launched alone,
    # take the k splits of a lone projection
    (4100, 5, 3, 64, 11008, 64),     # dV over k = 11008 from 4096 rows on: split in eight instead of five
    (8200, 3, 2, 4096, 64, 64),      # v recomputed over k = 4096 at 8192 rows: split in four instead of two
    (8192, 4, 2, 64, 14336, 16),     # dV over k = 14336 = 7 x 2048: split in four instead of seven
], ids=["dv-k11008", "v-k4096-8192-rows", "dv-k14336"])
def test_backward_lone_product_splits(K, oracle, gpu_device, case):
    n_rows, P, NA, h_in, h_out, r = case
    rng = np.random.default_rng(61)
    tp = _ragged_segments(rng, n_rows, P)
    part_ad = [int(i) % NA for i in range(P)]
    x, A, B = make_case(oracle, 209, n_rows, None, None, NA, h_in, h_out, r, "bf16", dy=True)
    g = dyadic(np.random.default_rng(24), (n_rows, h_out), 16, 8)
    _bwd_exact(K, oracle, gpu_device, "bf16", x, A, B, g, tp, part_ad, r)


def test_backward_is_deterministic(K, oracle, gpu_device):
    tp, part_ad, NA, h_in, h_out, r, dt = [0, 300, 650, 1000], [0, 1, 0], 2, 512, 768, 16, "bf16"
    x, A, B = make_case(oracle, 105, tp[-1], None, None, NA, h_in, h_out, r, dt)
    g = oracle.round_to(np.random.default_rng(3).standard_normal((tp[-1], h_out)), dt)
    d = gpu_device
    xd, gd = dev_t(x, dt, d), dev_t(g, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    outs = []
    for _ in range(3):
        dA, dB = [torch.empty_like(a) for a in Ad], [torch.empty_like(b) for b in Bd]
        dx = torch.empty(tp[-1], h_in, dtype=TDT[dt], device=d)
        pi = torch.tensor(tp, dtype=torch.int32, device=d)
        pa = torch.tensor(part_ad, dtype=torch.int32, device=d)
        K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), gd, xd, None, ptrs(Ad, d), ptrs(Bd, d),
                             K.SegmentPlan(pi, pa, tp[-1]), r)
        outs.append([dx] + dA + dB)
    for o in outs[1:]:
        for a, b in zip(outs[0], o):
            assert torch.equal(a, b)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_add_lora_autograd_surface(K, oracle, gpu_device, dt):
    """add_lora.apply with the reference's positional arguments: train rows
    first, then inference rows; shared adapter passed twice."""
    from loquetier_amd.kernel_utils import add_lora
    tp, train_idx = [0, 30, 50, 90], [1, 0, 1]
    n_inf, NA, h_in, h_out, r = 12, 3, 128, 192, 16
    tl = tp[-1]
    T = tl + n_inf
    x, A, B = make_case(oracle, 106, T, None, None, NA, h_in, h_out, r, dt)
    g = oracle.round_to(np.random.default_rng(4).standard_normal((T, h_out)), dt)
    d = gpu_device
    xd = dev_t(x, dt, d).requires_grad_(True)
    Ad = [dev_t(a, dt, d).requires_grad_(True) for a in A]
    Bd = [dev_t(b, dt, d).requires_grad_(True) for b in B]
    # segments: partitions 0|1|2 (adapters 1,0,1), then inference rows on adapter 2
    seg, ids = tp + [T], train_idx + [2]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    wa, wb = ptrs([Ad[i] for i in ids], d), ptrs([Bd[i] for i in ids], d)
    weights = [w for i in train_idx for w in (Ad[i], Bd[i])]
    y = add_lora.apply((T, h_out), xd, wa, wb, s, r, tl, tp, *weights)
    yo, _ = oracle.add_lora_forward(x, [A[i] for i in ids], [B[i] for i in ids], seg, h_out, dt)
    close(to_np(y), yo)
    y.backward(dev_t(g, dt, d))
    gx, ga, gb = oracle.add_lora_backward(g[:tl], x[:tl], A, B, tp, train_idx, dt)
    close(to_np(xd.grad)[:tl], gx)
    assert not to_np(xd.grad)[tl:].any()
    for a in (0, 1):
        close(to_np(Ad[a].grad), ga[a], atol=ATOL * max(1.0, float(np.abs(ga[a]).max())))
        close(to_np(Bd[a].grad), gb[a], atol=ATOL * max(1.0, float(np.abs(gb[a]).max())))
    assert Ad[2].grad is None


@pytest.mark.parametrize("fused", [True, False])
def test_mixed_lora_linear_layer(K, oracle, gpu_device, fused):
    """MixedLoraLinear: base + scale * LoRA, trained and served rows in one batch."""
    from loquetier_amd.kernel_utils import BatchLenInfo
    from loquetier_amd.mixed_lora import MixedLoraContext, MixedLoraLinear, NamedLoraLayer
    from loquetier_amd.segments import build_segments
    dt, tdt = "bf16", torch.bfloat16
    d = gpu_device
    h_in, h_out, r, NA = 256, 384, 16, 4
    rng = np.random.default_rng(12)
    W = oracle.round_to(rng.standard_normal((h_out, h_in)) / 16, dt)
    x, A, B = make_case(oracle, 107, 0, None, None, NA, h_in, h_out, r, dt)
    # requests: train seq (1x24) on adapter 1, train (1x16) on adapter 3, prefill 9 on 0, decode x3 on 2,2,1
    req_ids, req_len = [1, 3, 0, 2, 2, 1], [24, 16, 9, 1, 1, 1]
    T = sum(req_len)
    xs = oracle.round_to(rng.standard_normal((T, h_in)), dt)
    scal = [2.0, 0.5, 1.0, 4.0]
    base = torch.nn.Linear(h_in, h_out, bias=False, device=d, dtype=tdt)
    base.weight.data.copy_(dev_t(W, dt, d))
    base.weight.requires_grad_(False)
    adapters = [NamedLoraLayer(f"a{i}", dev_t(A[i], dt, d), dev_t(B[i], dt, d), torch.nn.Identity(), scal[i])
                for i in range(NA)]
    ctx = MixedLoraContext()
    layer = MixedLoraLinear(ctx, base, adapters, r, tdt, is_scaled=False, fused=fused)
    layer.set_trainable([1, 3])
    lora_ids, lora_len, segment = build_segments(req_ids, req_len, d)
    blen = BatchLenInfo([(1, 24), (1, 16)], [9], 3, [], d)
    ctx.update(blen=blen, lora_ids=lora_ids, lora_len=lora_len, segment=segment, train_idx=[1, 3])
    xd = dev_t(xs, dt, d).requires_grad_(True)
    out = layer(xd)
    seg = segment.cpu().numpy()
    base_np = oracle.round_to(xs.astype(np.float64) @ W.T.astype(np.float64), dt)
    sc = [scal[i] for i in lora_ids]
    if fused:
        want, _ = oracle.lora_fused(base_np, xs, [A[i] for i in lora_ids], [B[i] for i in lora_ids], seg,
                                    sc, 1.0, dt)
    else:
        want = oracle.mixed_lora_linear(base_np, xs, [A[i] for i in lora_ids], [B[i] for i in lora_ids],
                                        seg, sc, dt)
    close(to_np(out), want, atol=2e-2)  # base GEMM by the BLAS library: its own rounding
    g = oracle.round_to(rng.standard_normal((T, h_out)), dt)
    out.backward(dev_t(g, dt, d))
    # gradients of the trainable adapters: scale * (unscaled oracle gradient)
    tp = [0, 24, 40]
    gx, ga, gb = oracle.add_lora_backward(g[:40], xs[:40], [A[1], A[3]], [B[1], B[3]], tp, [0, 1], "fp32")
    for k, idx in enumerate((1, 3)):
        pa = layer.get_parameter(f"lora-{idx}-A").grad
        pb = layer.get_parameter(f"lora-{idx}-B").grad
        close(to_np(pa), scal[idx] * ga[k], rtol=2e-2, atol=2e-2 * float(np.abs(ga[k]).max()) * scal[idx])
        close(to_np(pb), scal[idx] * gb[k], rtol=2e-2, atol=2e-2 * float(np.abs(gb[k]).max()) * scal[idx])
    # dX = g W (base path) + scale * LoRA dX on train rows
    want_dx = g.astype(np.float64) @ W.astype(np.float64)
    want_dx[:24] += scal[1] * gx[:24]
    want_dx[24:40] += scal[3] * gx[24:40]
    close(to_np(xd.grad), want_dx, rtol=2e-2, atol=5e-2)


# ------------------------------------------------- full sizes of BASELINE ---
def _dyadic_full(seed, T, h_in, h_out, r, NA):
    rng = np.random.default_rng(seed)
    x = dyadic(rng, (T, h_in), 16, 8)
    A = [dyadic(rng, (r, h_in), 8, 64) for _ in range(NA)]
    B = [dyadic(rng, (h_out, r), 8, 8) for _ in range(NA)]
    base = dyadic(rng, (T, h_out), 16, 8)
    return x, A, B, base


def _permutation_invariance(K, d, dt, x, A, B, seg, ids, r, y):
    """Routing at full size: reversing the order of the segments (rows moved
    with them) must reproduce every row bit for bit."""
    T = x.shape[0]
    xd = dev_t(x, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    order = list(range(len(ids)))[::-1]
    lens = [seg[i + 1] - seg[i] for i in order]
    seg2 = np.concatenate([[0], np.cumsum(lens)]).tolist()
    perm = torch.cat([torch.arange(seg[i], seg[i + 1]) for i in order]).to(d)
    y2 = torch.zeros_like(y)
    s2 = torch.tensor(seg2, dtype=torch.int32, device=d)
    ids2 = torch.tensor([ids[i] for i in order], dtype=torch.int32, device=d)
    K.smlm_lora_forward(y2, xd[perm].contiguous(), ptrs(Ad, d), ptrs(Bd, d), K.SegmentPlan(s2, ids2, T), r)
    y1 = torch.zeros_like(y)
    s1 = torch.tensor(seg, dtype=torch.int32, device=d)
    ids1 = torch.tensor(ids, dtype=torch.int32, device=d)
    K.smlm_lora_forward(y1, xd, ptrs(Ad, d), ptrs(Bd, d), K.SegmentPlan(s1, ids1, T), r)
    assert torch.equal(y2, y1[perm])


def test_full_config2_decode(K, oracle, gpu_device):
    """256 single-token segments over 32 adapters, 4096 -> 4096, r=16, fp16."""
    ids = np.random.default_rng(2).integers(0, 32, 256).tolist()
    seg = list(range(257))
    x, A, B, base = _dyadic_full(2, 256, 4096, 4096, 16, 32)
    y = _fwd_exact(K, oracle, gpu_device, "fp16", x, A, B, seg, ids, 16, base)
    _permutation_invariance(K, gpu_device, "fp16", x, A, B, seg, ids, 16, y)


@pytest.mark.parametrize("shape", [(4096, 11008), (11008, 4096)], ids=["gate_up", "down"])
def test_full_config3_mixed_prefill_decode(K, oracle, gpu_device, shape):
    """4 x 512 prefill + 64 decode rows, 16 adapters, r=32, Llama-2-7B MLP shapes, fp16."""
    seg = [0, 512, 1024, 1536, 2048] + list(range(2049, 2113))
    ids = [i % 16 for i in range(68)]
    x, A, B, base = _dyadic_full(3, 2112, shape[0], shape[1], 32, 16)
    y = _fwd_exact(K, oracle, gpu_device, "fp16", x, A, B, seg, ids, 32, base)
    _permutation_invariance(K, gpu_device, "fp16", x, A, B, seg, ids, 32, y)


def test_full_config4_finetune_and_serve(K, oracle, gpu_device):
    """4 x 1024 training rows (adapters 0-3, forward + backward) + 128 decode rows, bf16."""
    seg = [0, 1024, 2048, 3072, 4096] + list(range(4097, 4225))
    ids = [0, 1, 2, 3] + [4 + i % 32 for i in range(128)]
    x, A, B, base = _dyadic_full(4, 4224, 4096, 4096, 16, 36)
    _fwd_exact(K, oracle, gpu_device, "bf16", x, A, B, seg, ids, 16, base)
    g = dyadic(np.random.default_rng(44), (4096, 4096), 16, 8)
    _bwd_exact(K, oracle, gpu_device, "bf16", x[:4096], A[:4], B[:4], g, seg[:5], [0, 1, 2, 3], 16)


def _config5_segments():
    rng = np.random.default_rng(5)
    lens = []
    while sum(lens) < 8192:
        lens.append(int(np.clip(rng.geometric(1 / 8), 1, 2048)))
    lens[-1] -= sum(lens) - 8192
    return np.concatenate([[0], np.cumsum(lens)]).tolist()


@pytest.mark.parametrize("shape", [(4096, 4096), (4096, 1024), (4096, 14336), (14336, 4096)],
                         ids=["q", "k_v", "gate_up", "down"])
def test_full_config5_heterogeneous_ranks(K, oracle, gpu_device, shape):
    """64 adapters, true ranks cycling {8,16,32,64} zero-padded to 64 (the
    reference's realisation, mixed_lora.py:501-521), geometric segment lengths
    totalling 8192 rows, every projection shape of the Llama-3-8B layer (q 4096 -> 4096, k/v 4096 ->
    1024, gate/up 4096 -> 14336, down 14336 -> 4096), bf16; backward on the first quarter of the
    segments.  Bit for bit on exactly representable inputs."""
    seg = _config5_segments()
    S = len(seg) - 1
    ids = [i % 64 for i in range(S)]
    h_in, h_out = shape
    rng = np.random.default_rng(55)
    x = dyadic(rng, (8192, h_in), 16, 8)
    base = dyadic(rng, (8192, h_out), 16, 8)
    A, B = [], []
    for a in range(64):
        r0 = [8, 16, 32, 64][a % 4]
        A.append(oracle.prepare_weight(dyadic(rng, (r0, h_in), 8, 64), 0, 64, None, "bf16"))
        B.append(oracle.prepare_weight(dyadic(rng, (h_out, r0), 8, 8), 1, 64, None, "bf16"))
    y = _fwd_exact(K, oracle, gpu_device, "bf16", x, A, B, seg, ids, 64, base)
    _permutation_invariance(K, gpu_device, "bf16", x, A, B, seg, ids, 64, y)
    P = S // 4
    n_rows = seg[P]
    g = dyadic(rng, (n_rows, h_out), 16, 8)
    _bwd_exact(K, oracle, gpu_device, "bf16", x[:n_rows], A, B, g, seg[:P + 1], ids[:P], 64)


def test_full_config2_four_projections_one_call(K, oracle, gpu_device):
    """The decode step as the benchmark issues it: q, k, v, o (4096 -> 4096, own weights and
    inputs each) of 256 single-token segments over 32 adapters in ONE smlm_lora_forward_multi
    call, every projection against the oracle: bit for bit on exactly representable inputs, and
    to rtol 1e-2 / atol 1e-3 of the fp32 host reference on Gaussian ones (fp16)."""
    d, dt = gpu_device, "fp16"
    T, r, NA, n_proj = 256, 16, 32, 4
    ids = np.random.default_rng(2).integers(0, NA, T).tolist()
    seg = list(range(T + 1))
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(s, torch.tensor(ids, dtype=torch.int32, device=d), T)
    sc = torch.full((T,), 2.0, device=d)
    for exact in (True, False):
        cases = []
        for p in range(n_proj):
            if exact:
                x, A, B, base = _dyadic_full(20 + p, T, 4096, 4096, r, NA)
            else:
                x, A, B = make_case(oracle, 30 + p, T, seg, ids, NA, 4096, 4096, r, dt)
                base = oracle.round_to(np.random.default_rng(40 + p).standard_normal((T, 4096)), dt)
            cases.append((x, A, B, base))
        dev = [dict(x=dev_t(x, dt, d), A=[dev_t(a, dt, d) for a in A], B=[dev_t(b, dt, d) for b in B],
                    y=dev_t(base, dt, d)) for x, A, B, base in cases]
        vs = [torch.zeros(T, r, dtype=TDT[dt], device=d) for _ in range(n_proj)]
        K.smlm_lora_forward_multi([c["y"] for c in dev], [c["x"] for c in dev], [ptrs(c["A"], d) for c in dev],
                                  [ptrs(c["B"], d) for c in dev], plan, r, seg_scale=sc, beta=1.0, v_out=vs)
        for p, (x, A, B, base) in enumerate(cases):
            yo, vo = oracle.lora_fused(base, x, [A[i] for i in ids], [B[i] for i in ids], seg, [2.0] * T, 1.0, dt)
            if exact:
                assert np.array_equal(to_np(vs[p]), vo), f"v of projection {p}"
                assert np.array_equal(to_np(dev[p]["y"]), yo), f"y of projection {p}"
            else:
                close(to_np(vs[p]), vo)
                # y against the oracle fed with the kernel's own v (one fp16 step of a v element, fp32
                # against double accumulation, moves a whole row of y by more than atol)
                acc = np.zeros((T, 4096), np.float32)
                oracle.smlm_gemm(acc, to_np(vs[p]), [B[i] for i in ids], seg, False, "fp32")
                close(to_np(dev[p]["y"]), oracle.round_to(base + 2.0 * acc, dt))


@pytest.mark.parametrize("cfg", ["decode_fp16", "train_bf16"])
def test_full_size_gaussian_tolerance(K, gpu_device, cfg):
    """Gaussian inputs at full size against fp32 library GEMMs on the device,
    stage by stage (v, then y from the kernel's own v), rtol 1e-2 / atol 1e-3."""
    d = gpu_device
    if cfg == "decode_fp16":
        dt, T, r, NA = torch.float16, 256, 16, 32
        seg = list(range(257))
        ids = np.random.default_rng(2).integers(0, 32, 256).tolist()
    else:
        dt, T, r, NA = torch.bfloat16, 4224, 16, 36
        seg = [0, 1024, 2048, 3072, 4096] + list(range(4097, 4225))
        ids = [0, 1, 2, 3] + [4 + i % 32 for i in range(128)]
    gen = torch.Generator(device="cpu").manual_seed(7)
    x = torch.randn(T, 4096, generator=gen).to(d).to(dt)
    A = [(torch.randn(r, 4096, generator=gen) / 64).to(d).to(dt) for _ in range(NA)]
    B = [(torch.randn(4096, r, generator=gen) / r ** 0.5).to(d).to(dt) for _ in range(NA)]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    ids_t = torch.tensor(ids, dtype=torch.int32, device=d)
    y = torch.zeros(T, 4096, dtype=dt, device=d)
    v = torch.zeros(T, r, dtype=dt, device=d)
    K.smlm_lora_forward(y, x, ptrs(A, d), ptrs(B, d), K.SegmentPlan(s, ids_t, T), r, v_out=v)
    for i in range(len(ids)):
        a, b = seg[i], seg[i + 1]
        v_ref = x[a:b].float() @ A[ids[i]].float().t()
        y_ref = v[a:b].float() @ B[ids[i]].float().t()
        assert bool(((v[a:b].float() - v_ref).abs() <= ATOL + RTOL * v_ref.abs()).all())
        assert bool(((y[a:b].float() - y_ref).abs() <= ATOL + RTOL * y_ref.abs()).all())


def test_add_lora_segments_sharing_a_but_not_b(K, oracle, gpu_device):
    """The reference reads wa_ptr[i] and wb_ptr[i] per problem (smlm_forward_cutlass.cuh:31-46), so
    segments may share their A and differ in B (or the other way round): every segment must get
    its own pair."""
    from loquetier_amd.kernel_utils import add_lora
    d, dt = gpu_device, "fp16"
    T, h_in, h_out, r = 60, 256, 192, 16
    seg = [0, 10, 25, 26, 40, 60]
    a_of, b_of = [0, 0, 1, 0, 1], [0, 1, 1, 2, 0]      # A shared by segments 0, 1, 3; B differs
    rng = np.random.default_rng(61)
    x = dyadic(rng, (T, h_in), 16, 8)
    A = [dyadic(rng, (r, h_in), 8, 64) for _ in range(2)]
    B = [dyadic(rng, (h_out, r), 8, 8) for _ in range(3)]
    xd = dev_t(x, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    y = add_lora.apply((T, h_out), xd, ptrs([Ad[i] for i in a_of], d), ptrs([Bd[i] for i in b_of], d), s, r, 0, [0])
    yo, _ = oracle.add_lora_forward(x, [A[i] for i in a_of], [B[i] for i in b_of], seg, h_out, dt)
    assert np.array_equal(to_np(y), yo)
