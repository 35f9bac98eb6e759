"""Edges of the BASELINE workloads on the HIP path:

* BASELINE config 1 (one SMLM forward: 64 tokens in 4 segments of 16 on adapters 0-3, 4096 -> 4096,
  rank 16, scale 2, y zero-initialised) in fp16 and bf16 -- the reference runs it in fp32 on the CPU;
  its kernels take 16-bit types only (kernel_src/csrc/loquetier_ops.cc:69-71), so the same inputs
  rounded to the type are used;
* the end-to-end error bound of the forward at full size (the decode step's four projections in one
  call, and one projection of the prefill + decode batch), against the exact result;
* adapter ids the caller's tables do not hold.
"""
import numpy as np
import pytest
import torch

from test_gpu_error_budget import within_budget
from test_gpu_parity import ATOL, RTOL, TDT, K, close, dev_t, dyadic, make_case, ptrs, to_np  # noqa: F401

pytestmark = pytest.mark.gpu


def _cfg1_inputs(oracle, dt, exact):
    T, h, r, NA = 64, 4096, 16, 4
    seg, ids = [0, 16, 32, 48, 64], [0, 1, 2, 3]
    rng = np.random.default_rng(1)
    if exact:
        x = dyadic(rng, (T, h), 16, 8)
        A = [dyadic(rng, (r, h), 8, 64) for _ in range(NA)]
        B = [dyadic(rng, (h, r), 8, 8) for _ in range(NA)]
    else:  # x ~ N(0,1), A ~ N(0, 1/4096), B ~ N(0, 1/16), as BASELINE.json states them
        x = oracle.round_to(rng.standard_normal((T, h)), dt)
        A = [oracle.round_to(rng.standard_normal((r, h)) / 64.0, dt) for _ in range(NA)]
        B = [oracle.round_to(rng.standard_normal((h, r)) / 4.0, dt) for _ in range(NA)]
    return T, h, r, NA, seg, ids, x, A, B


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("route", ["fused", "reference-two-calls", "add_lora"])
def test_baseline_config1_dyadic_bit_exact(K, oracle, gpu_device, dt, route):
    """Exactly representable inputs: y = 0 + 2 (x A^T) B^T equals the oracle bit for bit, through the fused
    call, through the reference's two kernel calls (scale folded into B, as its tests fold it), and
    through add_lora.apply."""
    d = gpu_device
    T, h, r, NA, seg, ids, x, A, B = _cfg1_inputs(oracle, dt, exact=True)
    xd = dev_t(x, dt, d)
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    want, _ = oracle.lora_fused(np.zeros((T, h), np.float32), x, A, B, seg, [2.0] * 4, 1.0, dt)
    if route == "fused":
        Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
        y = torch.zeros(T, h, dtype=TDT[dt], device=d)
        plan = K.SegmentPlan(s, torch.tensor(ids, dtype=torch.int32, device=d), T, defer=True)
        K.smlm_lora_forward(y, xd, ptrs(Ad, d), ptrs(Bd, d), plan, r, seg_scale=torch.full((4,), 2.0, device=d),
                            beta=1.0)
    else:
        Ad, B2d = [dev_t(a, dt, d) for a in A], [dev_t(2.0 * b, dt, d) for b in B]  # (a power of two: exact)
        wa, wb = ptrs(Ad, d), ptrs(B2d, d)
        if route == "add_lora":
            from loquetier_amd.kernel_utils import add_lora
            y = add_lora.apply((T, h), xd, wa, wb, s, r, 0, [])
        else:
            y = torch.empty(T, h, dtype=TDT[dt], device=d)
            v = torch.empty(T, r, dtype=TDT[dt], device=d)
            tmp = torch.empty(K.smlm_forward_cutlass_tmp_size(4), dtype=torch.uint8, device=d)
            K.smlm_forward_cutlass(v, xd, wa, s, tmp, False)
            K.smlm_forward_cutlass(y, v, wb, s, tmp, False)
    assert np.array_equal(to_np(y), want)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_baseline_config1_gaussian(K, oracle, gpu_device, dt):
    """The inputs BASELINE.json states: the intermediate v within rtol 1e-2 / atol 1e-3 of the fp32 oracle,
    y within that tolerance of the oracle fed with the kernel's own v (one 16-bit step of a v element
    moves a whole row of y by more than atol), and y end to end within the error budget of the exact
    result: no worse than the reference's own semantics (v rounded to the I/O type)."""
    d = gpu_device
    T, h, r, NA, seg, ids, x, A, B = _cfg1_inputs(oracle, dt, exact=False)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    y = torch.zeros(T, h, dtype=TDT[dt], device=d)
    v = torch.zeros(T, r, dtype=TDT[dt], device=d)
    K.smlm_lora_forward(y, dev_t(x, dt, d), ptrs(Ad, d), ptrs(Bd, d),
                        K.SegmentPlan(s, torch.tensor(ids, dtype=torch.int32, device=d), T), r,
                        seg_scale=torch.full((4,), 2.0, device=d), beta=1.0, v_out=v)
    zero = np.zeros((T, h), np.float32)
    y16, v16 = oracle.lora_fused(zero, x, A, B, seg, [2.0] * 4, 1.0, dt)
    y64, _ = oracle.lora_fused(zero, x, A, B, seg, [2.0] * 4, 1.0, "fp32")
    close(to_np(v), v16)
    acc = np.zeros((T, h), np.float32)
    oracle.smlm_gemm(acc, to_np(v), B, seg, False, "fp32")
    close(to_np(y), oracle.round_to(2.0 * acc, dt))
    within_budget("y", to_np(y), y16, y64, dt)


def test_full_config2_end_to_end_error_budget(K, oracle, gpu_device):
    """The decode step's four projections in one call, Gaussian inputs, fp16: every projection's y, end to
    end, errs no more against the exact result than the reference's semantics do."""
    d, dt = gpu_device, "fp16"
    T, r, NA, n_proj, h = 256, 16, 32, 4, 4096
    ids = np.random.default_rng(2).integers(0, NA, T).tolist()
    seg = list(range(T + 1))
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(s, torch.tensor(ids, dtype=torch.int32, device=d), T, defer=True)
    cases, dev = [], []
    for p in range(n_proj):
        x, A, B = make_case(oracle, 30 + p, T, seg, ids, NA, h, h, r, dt)
        base = oracle.round_to(np.random.default_rng(40 + p).standard_normal((T, h)), dt)
        cases.append((x, A, B, base))
        dev.append(dict(x=dev_t(x, dt, d), A=[dev_t(a, dt, d) for a in A], B=[dev_t(b, dt, d) for b in B],
                        y=dev_t(base, dt, d)))
    K.smlm_lora_forward_multi([c["y"] for c in dev], [c["x"] for c in dev], [ptrs(c["A"], d) for c in dev],
                              [ptrs(c["B"], d) for c in dev], plan, r, seg_scale=torch.full((T,), 2.0, device=d),
                              beta=1.0)
    for p, (x, A, B, base) in enumerate(cases):
        wa, wb = [A[i] for i in ids], [B[i] for i in ids]
        y16, _ = oracle.lora_fused(base, x, wa, wb, seg, [2.0] * T, 1.0, dt)
        y64, _ = oracle.lora_fused(base, x, wa, wb, seg, [2.0] * T, 1.0, "fp32")
        within_budget(f"y of projection {p}", to_np(dev[p]["y"]), y16, y64, dt)


def test_full_config3_end_to_end_error_budget(K, oracle, gpu_device):
    """One projection (4096 -> 11008, the widest) of the prefill + decode batch at full size, Gaussian
    inputs, fp16, rank 32: y end to end within the error budget of the exact result."""
    d, dt = gpu_device, "fp16"
    r, NA, h_in, h_out = 32, 16, 4096, 11008
    seg = [0, 512, 1024, 1536, 2048] + list(range(2049, 2113))
    ids = [i % 16 for i in range(68)]
    T = seg[-1]
    x, A, B = make_case(oracle, 53, T, seg, ids, NA, h_in, h_out, r, dt)
    base = oracle.round_to(np.random.default_rng(54).standard_normal((T, h_out)), dt)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    y = dev_t(base, dt, d)
    plan = K.SegmentPlan(torch.tensor(seg, dtype=torch.int32, device=d), torch.tensor(ids, dtype=torch.int32, device=d), T)
    K.smlm_lora_forward(y, dev_t(x, dt, d), ptrs(Ad, d), ptrs(Bd, d), plan, r,
                        seg_scale=torch.full((len(ids),), 2.0, device=d), beta=1.0)
    wa, wb = [A[i] for i in ids], [B[i] for i in ids]
    y16, _ = oracle.lora_fused(base, x, wa, wb, seg, [2.0] * len(ids), 1.0, dt)
    y64, _ = oracle.lora_fused(base, x, wa, wb, seg, [2.0] * len(ids), 1.0, "fp32")
    within_budget("y", to_np(y), y16, y64, dt)


@pytest.mark.parametrize("route", ["decode", "tile-blocks"])
def test_adapter_ids_past_the_tables_are_skipped(K, oracle, gpu_device, route):
    """An adapter id at or past the length of the weight tables is treated like a negative one: its rows of y
    stay as they were and the table is not read past its end (the entries behind the tables here are
    poisoned addresses).  Forward over a finished plan and over one the call builds; backward: the rows of
    such a partition's dX stay, nothing is summed for it."""
    d, dt, r, NA = gpu_device, "bf16", 16, 3
    if route == "decode":
        T, h_in, h_out = 40, 2048, 256
        seg, ids = list(range(T + 1)), [int(i) for i in np.random.default_rng(5).integers(0, 5, T)]  # ids 3, 4: no such adapter
    else:
        T, h_in, h_out = 2200, 256, 384
        seg, ids = [0, 700, 1400, 1500, 2200], [1, 4, 0, 3]
    rng = np.random.default_rng(6)
    x, base = dyadic(rng, (T, h_in), 16, 8), dyadic(rng, (T, h_out), 16, 8)
    A = [dyadic(rng, (r, h_in), 8, 64) for _ in range(NA)]
    B = [dyadic(rng, (h_out, r), 8, 8) for _ in range(NA)]
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    poison = 0x7fff_dead_0000  # behind the tables: never to be dereferenced
    a_tab = torch.tensor([t.data_ptr() for t in Ad] + [poison] * 4, dtype=torch.int64, device=d)[:NA]
    b_tab = torch.tensor([t.data_ptr() for t in Bd] + [poison] * 4, dtype=torch.int64, device=d)[:NA]
    assert a_tab.size(0) == NA and a_tab.is_contiguous()
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    ids_t = torch.tensor(ids, dtype=torch.int32, device=d)
    served = [i for i in range(len(ids)) if ids[i] < NA]
    want = base.copy()
    for i in served:
        part, _ = oracle.lora_fused(base[seg[i]:seg[i + 1]], x[seg[i]:seg[i + 1]], [A[ids[i]]], [B[ids[i]]],
                                    [0, seg[i + 1] - seg[i]], None, 1.0, dt)
        want[seg[i]:seg[i + 1]] = part
    for defer in (False, True):
        y = dev_t(base, dt, d)
        K.smlm_lora_forward(y, dev_t(x, dt, d), a_tab, b_tab, K.SegmentPlan(s, ids_t, T, defer=defer), r, beta=1.0)
        torch.cuda.synchronize()
        assert np.array_equal(to_np(y), want), f"defer={defer}"
    # backward over the same partitions
    g = dyadic(rng, (T, h_out), 16, 8)
    dA, dB = [torch.full_like(a, 7.0) for a in Ad], [torch.full_like(b, 7.0) for b in Bd]
    da_tab = torch.tensor([t.data_ptr() for t in dA] + [poison] * 4, dtype=torch.int64, device=d)[:NA]
    db_tab = torch.tensor([t.data_ptr() for t in dB] + [poison] * 4, dtype=torch.int64, device=d)[:NA]
    dx = torch.full((T, h_in), 7.0, dtype=TDT[dt], device=d)
    K.smlm_lora_backward(dx, da_tab, db_tab, dev_t(g, dt, d), dev_t(x, dt, d), None, a_tab, b_tab,
                         K.SegmentPlan(s, ids_t, T), r)
    torch.cuda.synchronize()
    # the oracle on the served partitions only (the others contribute nothing and keep their rows of dX)
    keep = np.zeros(T, bool)
    for i in served:
        keep[seg[i]:seg[i + 1]] = True
    tp2, ad2, rows = [0], [], []
    for i in served:
        rows.append(np.arange(seg[i], seg[i + 1]))
        tp2.append(tp2[-1] + seg[i + 1] - seg[i])
        ad2.append(ids[i])
    rows = np.concatenate(rows)
    gx, ga, gb = oracle.add_lora_backward(g[rows], x[rows], A, B, tp2, ad2, dt)
    got = to_np(dx)
    assert np.array_equal(got[rows], gx) and np.all(got[~keep] == 7.0)
    for a in range(NA):
        assert np.array_equal(to_np(dA[a]), ga[a]) and np.array_equal(to_np(dB[a]), gb[a]), a
