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
    bits = torch.full((2, train_rows, h_in // 8), 0xAA, dtype=torch.uint8, device=d)
    assert bits.numel() == K.DropoutSpec.mask_nbytes(train_rows, [h_in, h_in])
    spec = K.DropoutSpec(torch.from_numpy(seg_p).to(d), train_rows, seed, offset, mask_bits=bits)
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
        # the keep bits the forward left behind: bit e of byte b of a row = element 8b + e is kept;
        # rows that are not dropped (p = 0, outside every segment) keep the buffer's old bytes
        keep = oracle.dropout_mask(train_rows, h_in, rp[:train_rows], seed, offset + i)
        want_bits = np.packbits(keep, axis=1, bitorder="little")
        dropped = covered[:train_rows] & (rp[:train_rows] > 0)
        got_bits = bits[i].cpu().numpy()
        assert np.array_equal(got_bits[dropped], want_bits[dropped])
        assert np.all(got_bits[~dropped] == 0xAA)
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


# name, tp, part_ad, NA, h_in, h_out, r, per-adapter p
BWD_CASES = [
    ("two-parts", [0, 5, 12], [0, 1], 2, 64, 96, 8, [0.5, 0.5]),
    ("shared-adapter", [0, 40, 70, 100], [1, 0, 1], 2, 128, 256, 16, [0.5, 0.0]),   # adapter 0 trains without dropout
    ("empty-part", [0, 17, 17, 50], [0, 1, 2], 3, 256, 128, 32, [0.5, 0.5, 0.5]),
    ("rank64", [0, 33, 90], [0, 1], 2, 192, 320, 64, [0.5, 0.5]),
    ("in-place", [0, 500, 520, 1300], [2, 0, 2], 3, 256, 192, 16, [0.5, 0.0, 0.5]),  # tile blocks: no transposes
    ("many-rows", [0, 1100, 2300], [0, 1], 2, 320, 128, 32, [0.5, 0.5]),             # four-wave weight gradient
    ("long-k", [0, 30, 75], [1, 0], 2, 4096, 2048, 16, [0.5, 0.5]),
]


def run_backward(K, d, dt, x, A, B, g, tp, part_ad, r, spec, v=None):
    n_rows = tp[-1]
    xd, gd = dev_t(x, dt, d), dev_t(g, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    dA, dB = [torch.empty_like(a) for a in Ad], [torch.empty_like(b) for b in Bd]
    dx = torch.full((n_rows + 3, x.shape[1]), 9.0, dtype=TDT[dt], device=d)
    pi = torch.tensor(tp, dtype=torch.int32, device=d)
    pa = torch.tensor(part_ad, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(pi, pa, n_rows)
    K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), gd, xd, v, ptrs(Ad, d), ptrs(Bd, d), plan, r,
                         dropout=spec)
    return to_np(dx), [to_np(t) for t in dA], [to_np(t) for t in dB]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("with_v,with_bits", [(False, False), (True, False), (True, True)],
                         ids=["recompute", "saved-v", "saved-v-and-bits"])
@pytest.mark.parametrize("case", BWD_CASES, ids=[c[0] for c in BWD_CASES])
def test_backward_dropout_exact(K, oracle, gpu_device, case, dt, with_v, with_bits):
    """dX, dA, dB of a forward that ran with dropout: the oracle's backward on the dropped x,
    then the mask and factor once more on its dX (autograd's dropout backward)."""
    name, tp, part_ad, NA, h_in, h_out, r, ad_p = case
    d = gpu_device
    n_rows = tp[-1]
    rng = np.random.default_rng(31)
    x = oracle.round_to(dyadic(rng, (n_rows, h_in), 16, 8), dt)
    A = [dyadic(rng, (r, h_in), 8, 64) for _ in range(NA)]
    B = [dyadic(rng, (h_out, r), 8, 8) for _ in range(NA)]
    g = dyadic(rng, (n_rows, h_out), 16, 8)
    seg_p = np.array([ad_p[a] for a in part_ad], np.float32)
    seed, offset = 4242, 9
    spec = K.DropoutSpec(torch.from_numpy(seg_p).to(d), n_rows, seed, offset)
    rp = row_probs(tp, seg_p, n_rows, n_rows)
    xdrop = oracle.dropout_rows(x, rp, seed, offset, dt)
    v = None
    if with_v:  # the v the forward saved (of the dropped x)
        _, vo = oracle.add_lora_forward(xdrop, [A[a] for a in part_ad], [B[a] for a in part_ad], tp, h_out, dt)
        v = dev_t(vo, dt, d)
    if with_bits:  # and the keep bits a forward call left (here: the fused forward over the same rows)
        bits = torch.zeros(n_rows, h_in // 8, dtype=torch.uint8, device=d)
        spec = K.DropoutSpec(spec.seg_p, n_rows, seed, offset, mask_bits=bits)
        Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
        plan = K.SegmentPlan(torch.tensor(tp, dtype=torch.int32, device=d),
                             torch.tensor(part_ad, dtype=torch.int32, device=d), n_rows)
        K.smlm_lora_forward(torch.zeros(n_rows, h_out, dtype=TDT[dt], device=d), dev_t(x, dt, d), ptrs(Ad, d),
                            ptrs(Bd, d), plan, r, dropout=spec)
        assert bits.any()
    dx, dA, dB = run_backward(K, d, dt, x, A, B, g, tp, part_ad, r, spec, v)
    gx, ga, gb = oracle.add_lora_backward(g, xdrop, A, B, tp, part_ad, dt)
    gx = oracle.dropout_rows(gx, rp, seed, offset, dt)
    covered = np.zeros(n_rows, bool)
    for p in range(len(part_ad)):
        covered[tp[p]:tp[p + 1]] = True
    assert np.array_equal(dx[:n_rows][covered], gx[covered])
    assert np.all(dx[n_rows:] == 9.0)
    for a in range(NA):
        assert np.array_equal(dA[a], ga[a]), f"dA[{a}]"
        assert np.array_equal(dB[a], gb[a]), f"dB[{a}]"
    # and the mask matters: without the descriptor dA differs wherever an adapter drops
    _, dA_plain, _ = run_backward(K, d, dt, x, A, B, g, tp, part_ad, r, None)
    for a in set(part_ad):
        rows = sum(tp[i + 1] - tp[i] for i in range(len(part_ad)) if part_ad[i] == a)
        if rows:
            assert np.array_equal(dA_plain[a], dA[a]) == (ad_p[a] == 0.0)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_backward_dropout_gaussian(K, oracle, gpu_device, dt):
    tp, part_ad, NA, h_in, h_out, r, ad_p = [0, 200, 500], [0, 1], 2, 512, 384, 16, [0.1, 0.25]
    d = gpu_device
    n_rows = tp[-1]
    rng = np.random.default_rng(32)
    x = oracle.round_to(rng.standard_normal((n_rows, h_in)), dt)
    A = [oracle.round_to(rng.standard_normal((r, h_in)) / np.sqrt(h_in), dt) for _ in range(NA)]
    B = [oracle.round_to(rng.standard_normal((h_out, r)) / np.sqrt(r), dt) for _ in range(NA)]
    g = oracle.round_to(rng.standard_normal((n_rows, h_out)), dt)
    seg_p = np.array([ad_p[a] for a in part_ad], np.float32)
    spec = K.DropoutSpec(torch.from_numpy(seg_p).to(d), n_rows, 1, 2)
    rp = row_probs(tp, seg_p, n_rows, n_rows)
    xdrop = oracle.dropout_rows(x, rp, 1, 2, dt)
    dx, dA, dB = run_backward(K, d, dt, x, A, B, g, tp, part_ad, r, spec)
    gx, ga, gb = oracle.add_lora_backward(g, xdrop, A, B, tp, part_ad, dt)
    keep = oracle.dropout_mask(n_rows, h_in, rp, 1, 2).astype(bool)
    gx = oracle.dropout_rows(gx, rp, 1, 2, dt)
    assert not dx[:n_rows][~keep].any()               # dropped positions: exactly zero
    close(dx[:n_rows], gx, atol=ATOL if dt == "fp16" else 6e-3)
    for a in range(NA):
        close(dA[a], ga[a], atol=ATOL * max(1.0, float(np.abs(ga[a]).max())))
        close(dB[a], gb[a], atol=ATOL * max(1.0, float(np.abs(gb[a]).max())))


def test_mixed_lora_linear_layer_with_dropout(K, oracle, gpu_device):
    """MixedLoraLinear(fused=True) with nn.Dropout adapters: the layer hands the kernels a
    descriptor (seed = torch's seed, offset from the context's host-side call counter) instead of
    dropping x itself; forward and gradients equal the oracle's on the dropped x."""
    from loquetier_amd.kernel_utils import BatchLenInfo
    from loquetier_amd.mixed_lora import MixedLoraContext, MixedLoraLinear, NamedLoraLayer
    from loquetier_amd.segments import build_segments
    dt, tdt = "bf16", torch.bfloat16
    d = gpu_device
    h_in, h_out, r, NA = 256, 384, 16, 4
    rng = np.random.default_rng(41)
    W = oracle.round_to(rng.standard_normal((h_out, h_in)) / 16, dt)
    A = [oracle.round_to(rng.standard_normal((r, h_in)) / 16, dt) for _ in range(NA)]
    B = [oracle.round_to(rng.standard_normal((h_out, r)) / 4, dt) for _ in range(NA)]
    # train (1x24) on adapter 1, train (1x16) on adapter 3, prefill 9 on 3 (merges with the
    # partition before it into one segment), decode on 2, 2, 1
    req_ids, req_len = [1, 3, 3, 2, 2, 1], [24, 16, 9, 1, 1, 1]
    T = sum(req_len)
    xs = oracle.round_to(rng.standard_normal((T, h_in)), dt)
    drops = [torch.nn.Identity(), torch.nn.Dropout(0.5), torch.nn.Dropout(0.9), torch.nn.Dropout(0.25)]
    base = torch.nn.Linear(h_in, h_out, bias=False, device=d, dtype=tdt)
    base.weight.data.copy_(dev_t(W, dt, d))
    base.weight.requires_grad_(False)
    adapters = [NamedLoraLayer(f"a{i}", dev_t(A[i], dt, d), dev_t(B[i], dt, d), drops[i], 1.0) for i in range(NA)]
    ctx = MixedLoraContext()
    layer = MixedLoraLinear(ctx, base, adapters, r, tdt, is_scaled=True, fused=True)
    layer.set_trainable([1, 3])
    lora_ids, lora_len, segment = build_segments(req_ids, req_len, d)
    assert lora_ids == [1, 3, 2, 1]
    blen = BatchLenInfo([(1, 24), (1, 16)], [9], 3, [], d)
    ctx.update(blen=blen, lora_ids=lora_ids, lora_len=lora_len, segment=segment, train_idx=[1, 3])
    torch.manual_seed(777)
    xd = dev_t(xs, dt, d).requires_grad_(True)
    out = layer(xd)
    # the first dropout call of a fresh context: its salt (drawn from torch's CPU generator at that call,
    # after the seed above was set) plus eight (MixedLoraContext.next_dropout_offset)
    salt, calls = ctx.dropout_state()
    assert calls == 1 and salt is not None
    offset = salt + 8
    # rows 0..23 drop with 0.5, rows 24..39 with 0.25, the prefill rows of adapter 3 and the decode
    # rows (adapter 2 has p = 0.9 but never trains here) are not dropped
    rp = np.zeros(T, np.float32)
    rp[:24], rp[24:40] = 0.5, 0.25
    xdrop = oracle.dropout_rows(xs, rp, 777, offset, dt)
    seg = segment.cpu().numpy()
    base_np = oracle.round_to(xs.astype(np.float64) @ W.T.astype(np.float64), dt)
    want, _ = oracle.lora_fused(base_np, xdrop, [A[i] for i in lora_ids], [B[i] for i in lora_ids], seg,
                                None, 1.0, dt)
    close(to_np(out), want, atol=2e-2)
    plain, _ = oracle.lora_fused(base_np, xs, [A[i] for i in lora_ids], [B[i] for i in lora_ids], seg,
                                 None, 1.0, dt)
    assert np.abs(to_np(out)[:40] - plain[:40]).max() > 0.1   # the mask was applied
    close(to_np(out)[40:], plain[40:], atol=2e-2)              # and only to the training rows
    g = oracle.round_to(rng.standard_normal((T, h_out)), dt)
    out.backward(dev_t(g, dt, d))
    tp = [0, 24, 40]
    gx, ga, gb = oracle.add_lora_backward(g[:40], xdrop[:40], [A[1], A[3]], [B[1], B[3]], tp, [0, 1], "fp32")
    gx = oracle.dropout_rows(gx, rp[:40], 777, offset, "fp32")
    for k, idx in enumerate((1, 3)):
        pa = layer.get_parameter(f"lora-{idx}-A").grad
        pb = layer.get_parameter(f"lora-{idx}-B").grad
        close(to_np(pa), ga[k], rtol=2e-2, atol=2e-2 * float(np.abs(ga[k]).max()))
        close(to_np(pb), gb[k], rtol=2e-2, atol=2e-2 * float(np.abs(gb[k]).max()))
    want_dx = g.astype(np.float64) @ W.astype(np.float64)
    want_dx[:40] += gx
    close(to_np(xd.grad), want_dx, rtol=2e-2, atol=5e-2)
    # a second call draws a new offset: another mask
    out2 = layer(dev_t(xs, dt, d))
    assert not torch.equal(out2[:40], out.detach()[:40]) and torch.equal(out2[40:], out.detach()[40:])
