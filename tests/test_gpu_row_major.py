"""The reference's other weight layout (is_row_major = True: W [d_in, d_out] row-major, i.e. A [h_in, r] and
B [r, h_out]): the forward as the generic grouped GEMM instantiates it
(kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cu:7-25) and the backward exactly as the reference's
Python writes it (src/loquetier_src/kernel_utils.py:139-145), against oracle.smlm_gemm(row_major=True)
and oracle.add_lora_backward_rowmajor."""
import numpy as np
import pytest
import torch

from test_gpu_parity import ATOL, TDT, K, _ragged_segments, close, dev_t, dyadic, ptrs, to_np  # noqa: F401

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [
    # T, S, NA, d_in, d_out
    (2300, 9, 3, 4096, 16),     # shrink over tile blocks, k split over workgroups and folded
    (2300, 9, 3, 16, 4096),     # expand over tile blocks, one k step
    (700, 40, 5, 1024, 64),     # shrink, 64 output columns
    (700, 40, 5, 64, 1024),     # expand, two k steps
    (300, 7, 2, 256, 192),      # shrink with three 64-column blocks
    (300, 7, 2, 96, 320),       # expand with a contraction above 64: the one-tile kernel's strided reads
    (5000, 300, 20, 2048, 32),  # many segments, plan in two launches
], ids=["shrink-r16", "expand-r16", "shrink-r64", "expand-r64", "shrink-wide", "expand-k96", "many-segments"])
def test_row_major_forward_dyadic_bit_exact(K, oracle, gpu_device, shape, dt):
    T, S, NA, d_in, d_out = shape
    d = gpu_device
    rng = np.random.default_rng(71)
    seg = _ragged_segments(rng, T, S)
    ids = [int(i) for i in rng.integers(0, NA, S)]
    x = dyadic(rng, (T, d_in), 16, 8)
    W = [dyadic(rng, (d_in, d_out), 8, 64) for _ in range(NA)]       # [d_in, d_out] row-major
    base = dyadic(rng, (T, d_out), 16, 8)
    scale = (rng.integers(1, 5, S) / 2.0).astype(np.float32)
    wd = [dev_t(w, dt, d) for w in W]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    # the reference's call: overwrite, no scale
    y = torch.full((T, d_out), 3.0, dtype=TDT[dt], device=d)
    tmp = torch.empty(K.smlm_forward_cutlass_tmp_size(S), dtype=torch.uint8, device=d)
    K.smlm_forward_cutlass(y, dev_t(x, dt, d), ptrs([wd[i] for i in ids], d), s, tmp, True)
    want = np.zeros((T, d_out), np.float32)
    oracle.smlm_gemm(want, x, [W[i] for i in ids], seg, True, dt)
    assert np.array_equal(to_np(y), want)
    # over a finished plan keyed by adapter id, accumulating with a per-segment scale
    y2 = dev_t(base, dt, d)
    plan = K.SegmentPlan(s, torch.tensor(ids, dtype=torch.int32, device=d), T)
    K.smlm_gemm_planned(y2, dev_t(x, dt, d), ptrs(wd, d), plan, is_row_major=True,
                        seg_scale=torch.from_numpy(scale).to(d), beta=1.0)
    acc = np.zeros((T, d_out), np.float32)
    oracle.smlm_gemm(acc, x, [W[i] for i in ids], seg, True, "fp32")   # exact: dyadic inputs
    row_scale = np.ones(T, np.float32)
    for i in range(S):
        row_scale[seg[i]:seg[i + 1]] = scale[i]
    assert np.array_equal(to_np(y2), oracle.round_to(base + row_scale[:, None] * acc, dt))


BWD = [
    # name, partition indptr, NA (one adapter per partition here: the reference returns one gradient per
    # partition), h_in, h_out, r
    ("small", [0, 5, 12, 40], 3, 64, 96, 8),
    ("blocks", [0, 500, 520, 1300], 3, 256, 192, 16),
    ("rank64", [0, 33, 90], 2, 192, 320, 64),
    ("rank128", [0, 33, 90], 2, 192, 320, 128),
    ("long-k", [0, 30, 75], 2, 4096, 2048, 16),
]


def _run_rm(K, d, dt, x, g, A, B, tp, part_ad, r, v=None, scale=None, tail=0):
    n_rows = tp[-1]
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    dA, dB = [torch.full_like(a, 5.0) for a in Ad], [torch.full_like(b, 5.0) for b in Bd]
    dx = torch.full((n_rows + tail, x.shape[1]), 5.0, dtype=TDT[dt], device=d)
    plan = K.SegmentPlan(torch.tensor(tp, dtype=torch.int32, device=d),
                         torch.tensor(part_ad, dtype=torch.int32, device=d), n_rows, defer=True)
    K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), dev_t(g, dt, d), dev_t(x, dt, d),
                         None if v is None else dev_t(v, dt, d), ptrs(Ad, d), ptrs(Bd, d), plan, r, scale,
                         is_row_major=True, zero_dx_tail=tail > 0)
    if tail:  # rows past the plan's: cleared by the call
        assert torch.count_nonzero(dx[n_rows:]) == 0
    return to_np(dx[:n_rows]), [to_np(t) for t in dA], [to_np(t) for t in dB]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", BWD, ids=[c[0] for c in BWD])
def test_row_major_backward_dyadic_bit_exact(K, oracle, gpu_device, case, dt):
    """Exactly representable sums: dX, dA [h_in, r], dB [r, h_out] equal the reference's literal lines bit for bit."""
    name, tp, NA, h_in, h_out, r = case
    rng = np.random.default_rng(81)
    n_rows = tp[-1]
    x, g = dyadic(rng, (n_rows, h_in), 16, 8), dyadic(rng, (n_rows, h_out), 16, 8)
    A = [dyadic(rng, (h_in, r), 8, 64) for _ in range(NA)]
    B = [dyadic(rng, (r, h_out), 8, 8) for _ in range(NA)]
    part_ad = list(range(len(tp) - 1))
    dx, dA, dB = _run_rm(K, gpu_device, dt, x, g, A, B, tp, part_ad, r, tail=11)
    gx, ga, gb = oracle.add_lora_backward_rowmajor(g, x, [A[a] for a in part_ad], [B[a] for a in part_ad], tp, dt)
    assert np.array_equal(dx, gx)
    for p, a in enumerate(part_ad):
        assert np.array_equal(dA[a], ga[p]), f"dA[{a}]"
        assert np.array_equal(dB[a], gb[p]), f"dB[{a}]"


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_row_major_backward_gaussian_shared_adapter_and_transposed_layout(K, oracle, gpu_device, dt):
    """Gaussian inputs, an adapter shared by two partitions (its gradients are the sums), a saved v and a
    scale: within the stated tolerance of the oracle's literal lines, and equal -- bit for bit -- to the
    PEFT-layout backward run on the transposed weights (the same products in the same order)."""
    d = gpu_device
    tp, part_ad, NA, h_in, h_out, r = [0, 300, 340, 700], [1, 0, 1], 2, 512, 384, 16
    rng = np.random.default_rng(82)
    n_rows = tp[-1]
    x = oracle.round_to(rng.standard_normal((n_rows, h_in)), dt)
    g = oracle.round_to(rng.standard_normal((n_rows, h_out)), dt)
    A = [oracle.round_to(rng.standard_normal((h_in, r)) / np.sqrt(h_in), dt) for _ in range(NA)]
    B = [oracle.round_to(rng.standard_normal((r, h_out)) / np.sqrt(r), dt) for _ in range(NA)]
    scale = torch.full((3,), 0.5, device=d)   # a power of two: the scaled results are exactly half
    dx, dA, dB = _run_rm(K, d, dt, x, g, A, B, tp, part_ad, r, scale=scale)
    gx, ga, gb = oracle.add_lora_backward_rowmajor(g, x, [A[a] for a in part_ad], [B[a] for a in part_ad], tp, dt)
    close(dx, 0.5 * gx, atol=ATOL if dt == "fp16" else 4e-3)   # bf16: one step of a mid element times |A|
    sums_a = [sum(ga[p] for p in range(3) if part_ad[p] == a) for a in range(NA)]
    sums_b = [sum(gb[p] for p in range(3) if part_ad[p] == a) for a in range(NA)]
    for a in range(NA):
        close(dA[a], 0.5 * sums_a[a], atol=ATOL * max(1.0, float(np.abs(sums_a[a]).max())))
        close(dB[a], 0.5 * sums_b[a], atol=ATOL * max(1.0, float(np.abs(sums_b[a]).max())))
    # the PEFT layout on the transposed weights
    At, Bt = [np.ascontiguousarray(a.T) for a in A], [np.ascontiguousarray(b.T) for b in B]
    Ad, Bd = [dev_t(a, dt, d) for a in At], [dev_t(b, dt, d) for b in Bt]
    pA, pB = [torch.empty_like(a) for a in Ad], [torch.empty_like(b) for b in Bd]
    pdx = torch.empty(n_rows, h_in, dtype=TDT[dt], device=d)
    plan = K.SegmentPlan(torch.tensor(tp, dtype=torch.int32, device=d),
                         torch.tensor(part_ad, dtype=torch.int32, device=d), n_rows)
    K.smlm_lora_backward(pdx, ptrs(pA, d), ptrs(pB, d), dev_t(g, dt, d), dev_t(x, dt, d), None, ptrs(Ad, d),
                         ptrs(Bd, d), plan, r, scale)
    assert np.array_equal(to_np(pdx), dx)
    for a in range(NA):
        assert np.array_equal(to_np(pA[a]).T, dA[a]) and np.array_equal(to_np(pB[a]).T, dB[a]), a


def test_row_major_backward_refuses_what_it_does_not_cover(K, oracle, gpu_device):
    d, dt = gpu_device, "fp16"
    tp, r, h = [0, 20], 8, 64
    x = torch.zeros(20, h, dtype=TDT[dt], device=d)
    A, B = [torch.zeros(h, r, dtype=TDT[dt], device=d)], [torch.zeros(r, h, dtype=TDT[dt], device=d)]
    plan = K.SegmentPlan(torch.tensor(tp, dtype=torch.int32, device=d), torch.zeros(1, dtype=torch.int32, device=d), 20)
    spec = K.DropoutSpec(torch.full((1,), 0.5, device=d), 20, 1, 0)
    with pytest.raises(RuntimeError):
        K.smlm_lora_backward(torch.empty_like(x), ptrs(A, d), ptrs(B, d), x, x, None, ptrs(A, d), ptrs(B, d), plan, r,
                             dropout=spec, is_row_major=True)
