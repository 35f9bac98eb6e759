"""Dropout of the training rows inside the operator (the reference's per-partition
nn.Dropout + torch.cat, src/loquetier_src/models/mixed_lora.py:185-192), against the
oracle: oracle.dropout_rows regenerates the same counter-based mask on the host, the
rest of the oracle then runs on the dropped x.

With p = 0.5 the factor of kept elements is 2, so dyadic inputs stay exact and the
kernels must equal the oracle bit for bit (mask position, rounding and routing all
show up as whole-element differences); Gaussian inputs with other p are checked to
the tolerance of the other parity tests."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3
TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}


@pytest.fixture(scope="module")
def K(gpu_device):
    from loquetier_amd import _lib
    from loquetier_amd.ops import _kernels
    _lib.load()
    return _kernels


def dev_t(a, dt, dev):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dev).to(TDT[dt]).contiguous()


def to_np(t):
    return t.detach().float().cpu().numpy()


def ptrs(ts, dev):
    return torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=dev)


def dyadic(rng, shape, lim, denom):
    return (rng.integers(-lim, lim + 1, shape) / float(denom)).astype(np.float32)


def close(got, want, rtol=RTOL, atol=ATOL):
    err = np.abs(got - want)
    bad = err > atol + rtol * np.abs(want)
    assert not bad.any(), f"max err {err.max():.4g}, {bad.sum()} of {bad.size} outside tolerance"


def row_probs(seg, seg_p, T, train_rows):
    rp = np.zeros(T, np.float32)
    for i, p in enumerate(seg_p):
        rp[seg[i]:seg[i + 1]] = p
    rp[train_rows:] = 0.0
    return rp


# name, T, seg, ids, NA, h_in, h_out, r, train_rows, per-adapter p
CASES = [
    # train rows share a tile with inference rows of the same adapter; one adapter without dropout
    ("small", 90, [0, 20, 41, 41, 60, 77, 90], [0, 1, 2, 0, 1, 2], 3, 256, 192, 16, 41, [0.5, 0.5, 0.0]),
    ("long-k", 70, [0, 33, 70], [1, 0], 2, 4096, 64, 16, 33, [0.5, 0.5]),          # k split and folded
    ("decode-route", 48, list(range(49)), [i % 3 for i in range(48)], 3, 512, 256, 16, 17, [0.5, 0.0, 0.5]),
    ("rank64", 150, [0, 64, 150], [0, 1], 2, 512, 128, 64, 64, [0.5, 0.5]),
    ("tile-blocks", 1500, [0, 700, 1100, 1101, 1500], [0, 1, 0, 2], 3, 512, 320, 32, 1100, [0.5, 0.5, 0.5]),
    ("uncovered", 60, [4, 30, 50], [0, 1], 2, 128, 64, 8, 30, [0.5, 0.5]),
]


def setup(K, rng, case, dt, d, dy=True):
    name, T, seg, ids, NA, h_in, h_out, r, train_rows, ad_p = case
    if dy:
        x = dyadic(rng, (T, h_in), 16, 8)
        A = [dyadic(rng, (r, h_in), 8, 64) for _ in range(NA)]
        B = [dyadic(rng, (h_out, r), 8, 8) for _ in range(NA)]
    else:
        x = rng.standard_normal((T, h_in)).astype(np.float32)
        A = [(rng.standard_normal((r, h_in)) / np.sqrt(h_in)).astype(np.float32) for _ in range(NA)]
        B = [(rng.standard_normal((h_out, r)) / np.sqrt(r)).astype(np.float32) for _ in range(NA)]
    xd = dev_t(x, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    x, A, B = to_np(xd), [to_np(a) for a in Ad], [to_np(b) for b in Bd]
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(s, torch.tensor(ids, dtype=torch.int32, device=d), T)
    seg_p = np.array([ad_p[i] for i in ids], np.float32)
    return x, A, B, xd, Ad, Bd, plan, seg_p


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_forward_dropout_exact(K, oracle, gpu_device, case, dt):
    name, T, seg, ids, NA, h_in, h_out, r, train_rows, ad_p = case
    d = gpu_device
    rng = np.random.default_rng(21)
    x, A, B, xd, Ad, Bd, plan, seg_p = setup(K, rng, case, dt, d)
    seed, offset = 0x5eed5eed5eed, (1 << 32) - 1   # the offset carries into its high word for projection 1
    spec = K.DropoutSpec(torch.from_numpy(seg_p).to(d), train_rows, seed, offset)
    y0 = dyadic(rng, (T, h_out), 8, 4)
    rp = row_probs(seg, seg_p, T, train_rows)
    # two projections sharing x: each gets its own mask (offset + i), as two modules of the reference would
    ys = [dev_t(y0, dt, d), dev_t(y0, dt, d)]
    vs = [torch.zeros(T, r, dtype=TDT[dt], device=d) for _ in range(2)]
    ta, tb = ptrs(Ad, d), ptrs(Bd, d)
    K.smlm_lora_forward_multi(ys, [xd, xd], [ta, ta], [tb, tb], plan, r, beta=1.0, v_out=vs, dropout=spec)
    outs = []
    for i in range(2):
        xdrop = oracle.dropout_rows(x, rp, seed, offset + i, dt)
        assert (xdrop[:train_rows] != x[:train_rows]).any() and np.array_equal(xdrop[train_rows:], x[train_rows:])
        yo, vo = oracle.lora_fused(y0, xdrop, [A[j] for j in ids], [B[j] for j in ids], seg, None, 1.0, dt)
        covered = np.zeros(T, bool)
        for j in range(len(ids)):
            covered[seg[j]:seg[j + 1]] = True
        assert np.array_equal(to_np(vs[i])[covered], vo[covered])
        assert np.array_equal(to_np(ys[i]), yo)
        outs.append(yo)
    assert not np.array_equal(outs[0], outs[1])   # the two masks differ
    # without the descriptor nothing is dropped
    y_plain = dev_t(y0, dt, d)
    K.smlm_lora_forward(y_plain, xd, ta, tb, plan, r, beta=1.0)
    yo, _ = oracle.lora_fused(y0, x, [A[j] for j in ids], [B[j] for j in ids], seg, None, 1.0, dt)
    assert np.array_equal(to_np(y_plain), yo)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("p", [0.05, 0.1, 0.3])
def test_forward_dropout_gaussian(K, oracle, gpu_device, dt, p):
    case = ("g", 200, [0, 64, 128, 200], [0, 1, 0], 2, 1024, 256, 16, 128, [p, p / 2])
    name, T, seg, ids, NA, h_in, h_out, r, train_rows, ad_p = case
    d = gpu_device
    rng = np.random.default_rng(22)
    x, A, B, xd, Ad, Bd, plan, seg_p = setup(K, rng, case, dt, d, dy=False)
    spec = K.DropoutSpec(torch.from_numpy(seg_p).to(d), train_rows, 77, 5)
    v = torch.zeros(T, r, dtype=TDT[dt], device=d)
    y = torch.zeros(T, h_out, dtype=TDT[dt], device=d)
    K.smlm_lora_forward(y, xd, ptrs(Ad, d), ptrs(Bd, d), plan, r, v_out=v, dropout=spec)
    xdrop = oracle.dropout_rows(x, row_probs(seg, seg_p, T, train_rows), 77, 5, dt)
    _, vo = oracle.lora_fused(np.zeros((T, h_out), np.float32), xdrop, [A[j] for j in ids],
                              [B[j] for j in ids], seg, None, 0.0, dt)
    close(to_np(v), vo)
    y_stage = np.zeros((T, h_out), np.float32)
    oracle.smlm_gemm(y_stage, to_np(v), [B[j] for j in ids], seg, False, dt)
    close(to_np(y), y_stage)
