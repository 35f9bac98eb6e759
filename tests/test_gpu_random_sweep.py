"""Randomised shapes and routings, forward and backward, against the oracle bit for bit
(dyadic inputs: every partial sum is exact, so any correct summation order gives the same
bits).  Widths that are not multiples of the kernels' 64-column chunks, ragged and empty
segments, rows outside every segment, ranks 8..64, with and without the per-segment scale,
dropout (p = 0.5: factor 2, still exact) and true ranks."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

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


def draw_case(seed):
    rng = np.random.default_rng(seed)
    big = seed % 5 == 0
    T = int(rng.integers(1100, 2600)) if big else int(rng.integers(1, 400))
    S = int(rng.integers(1, 12 if big else 40))
    cuts = np.sort(rng.integers(0, T + 1, S + 1))
    if seed % 3 == 0:
        cuts[0] = 0          # segments from row 0 (the usual batch); otherwise leading rows stay uncovered
    seg = cuts.tolist()
    NA = int(rng.integers(1, 6))
    ids = rng.integers(0, NA, S).tolist()
    r = int(rng.choice([8, 16, 24, 32, 48, 64]))
    h_in = int(rng.choice([64, 72, 136, 256, 520, 1000, 2048]))
    h_out = int(rng.choice([64, 88, 192, 328, 1024]))
    dt = "fp16" if seed % 2 else "bf16"
    return rng, T, seg, ids, NA, r, h_in, h_out, dt


@pytest.mark.parametrize("seed", range(24))
def test_random_forward(K, oracle, gpu_device, seed):
    rng, T, seg, ids, NA, r, h_in, h_out, dt = draw_case(seed)
    d = gpu_device
    true_r = [int(rng.choice([q for q in (8, 16, 24, 32, 48, 64) if q <= r])) for _ in range(NA)]
    x = dyadic(rng, (T, h_in), 16, 8)
    A = [dyadic(rng, (r, h_in), 8, 64) for _ in range(NA)]
    B = [dyadic(rng, (h_out, r), 8, 8) for _ in range(NA)]
    use_rank = seed % 4 == 1
    if use_rank:
        for a in range(NA):
            A[a][true_r[a]:] = 0
            B[a][:, true_r[a]:] = 0
    y0 = dyadic(rng, (T, h_out), 16, 8)
    S = len(ids)
    scale = rng.choice([0.5, 1.0, 2.0, 4.0], S).astype(np.float32) if seed % 2 else None
    train_rows = seg[min(2, S)] if seed % 3 == 0 else 0
    seg_p = np.where(rng.random(S) < 0.7, 0.5, 0.0).astype(np.float32)
    xd, yd = dev_t(x, dt, d), dev_t(y0, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    plan = K.SegmentPlan(torch.tensor(seg, dtype=torch.int32, device=d),
                         torch.tensor(ids, dtype=torch.int32, device=d), T)
    spec = K.DropoutSpec(torch.from_numpy(seg_p).to(d), train_rows, 1000 + seed, seed) if train_rows else None
    v = torch.zeros(T, r, dtype=TDT[dt], device=d)
    K.smlm_lora_forward(yd, xd, ptrs(Ad, d), ptrs(Bd, d), plan, r,
                        seg_scale=None if scale is None else torch.from_numpy(scale).to(d), beta=1.0, v_out=v,
                        dropout=spec,
                        adapter_rank=torch.tensor(true_r, dtype=torch.int32, device=d) if use_rank else None)
    xo = x
    if train_rows:
        rp = np.zeros(T, np.float32)
        for i in range(S):
            rp[seg[i]:seg[i + 1]] = seg_p[i]
        rp[train_rows:] = 0
        xo = oracle.dropout_rows(x, rp, 1000 + seed, seed, dt)
    yo, vo = oracle.lora_fused(y0, xo, [A[i] for i in ids], [B[i] for i in ids], seg,
                               None if scale is None else scale.tolist(), 1.0, dt)
    covered = np.zeros(T, bool)
    for i in range(S):
        covered[seg[i]:seg[i + 1]] = True
    assert np.array_equal(to_np(v)[covered], vo[covered]), "v"
    assert np.array_equal(to_np(yd), yo), "y"


@pytest.mark.parametrize("seed", range(100, 118))
def test_random_backward(K, oracle, gpu_device, seed):
    rng, T, seg, ids, NA, r, h_in, h_out, dt = draw_case(seed)
    d = gpu_device
    # the training partitions are the segments, from row 0, each adapter possibly several times
    tp = [c - seg[0] for c in seg]
    n_rows = tp[-1]
    if n_rows == 0:
        pytest.skip("drawn batch has no rows")
    part_ad = ids
    x = dyadic(rng, (n_rows, h_in), 16, 8)
    A = [dyadic(rng, (r, h_in), 8, 64) for _ in range(NA)]
    B = [dyadic(rng, (h_out, r), 8, 8) for _ in range(NA)]
    g = dyadic(rng, (n_rows, h_out), 16, 8)
    use_drop = seed % 2 == 0
    ad_p = np.where(rng.random(NA) < 0.7, 0.5, 0.0).astype(np.float32)
    seg_p = ad_p[part_ad]
    xd, gd = dev_t(x, dt, d), dev_t(g, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    dA, dB = [torch.empty_like(a) for a in Ad], [torch.empty_like(b) for b in Bd]
    dx = torch.empty(n_rows, h_in, dtype=TDT[dt], device=d)
    plan = K.SegmentPlan(torch.tensor(tp, dtype=torch.int32, device=d),
                         torch.tensor(part_ad, dtype=torch.int32, device=d), n_rows)
    spec = K.DropoutSpec(torch.from_numpy(seg_p).to(d), n_rows, 7, seed) if use_drop else None
    K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), gd, xd, None, ptrs(Ad, d), ptrs(Bd, d), plan, r,
                         dropout=spec)
    xo = x
    if use_drop:
        rp = np.zeros(n_rows, np.float32)
        for i in range(len(part_ad)):
            rp[tp[i]:tp[i + 1]] = seg_p[i]
        xo = oracle.dropout_rows(x, rp, 7, seed, dt)
    gx, ga, gb = oracle.add_lora_backward(g, xo, A, B, tp, part_ad, dt)
    if use_drop:
        gx = oracle.dropout_rows(gx, rp, 7, seed, dt)
    assert np.array_equal(to_np(dx), gx), "dX"
    for a in range(NA):
        assert np.array_equal(to_np(dA[a]), ga[a]), f"dA[{a}]"
        assert np.array_equal(to_np(dB[a]), gb[a]), f"dB[{a}]"
