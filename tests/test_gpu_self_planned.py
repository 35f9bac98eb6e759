"""A plan that the first fused forward builds itself (SegmentPlan(defer=True);
smlm_lora_opts.build_seg_indptr / build_seg_adapter).  Decode batches build it inside the
shrink launch: every workgroup derives its own tile from the segment table and one more
workgroup writes the plan.  Whatever route the library takes, the call must leave the very
plan smlm_plan_build writes (byte for byte) and the very outputs a call over a prebuilt plan
gives (bit for bit); the outputs are also held against the oracle."""
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


def ptrs(ts, dev):
    return torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=dev)


def decode_ids(n, na, seed):
    return np.random.default_rng(seed).integers(0, na, n).tolist()


def ragged(seed, n_seg, max_len, na):
    rng = np.random.default_rng(seed)
    lens = rng.integers(0, max_len + 1, n_seg)
    seg = np.concatenate([[0], np.cumsum(lens)]).tolist()
    return seg, rng.integers(0, na, n_seg).tolist()


# name, seg, ids, NA (table entries), T (rows of x; rows past seg[-1] belong to no segment), rank, [(h_in, h_out)]
CASES = [
    ("decode256-qkvo", list(range(257)), decode_ids(256, 32, 2), 32, 256, 16, [(4096, 4096)] * 4),
    ("one-projection", list(range(257)), decode_ids(256, 32, 3), 32, 256, 16, [(4096, 1024)]),
    ("ragged-empty-uncovered",) + ragged(4, 90, 9, 12) + (12, 0, 16, [(2048, 512), (2048, 256)]),
    ("one-adapter-many-tiles", [0, 300, 301, 640], [5, 5, 5], 8, 700, 32, [(2048, 320)]),
    ("absent-adapters", list(range(0, 200, 2)), [(7 * i) % 600 for i in range(99)], 1024, 198, 8, [(2048, 128)]),
    ("1024-segments", list(range(0, 1000)) + [1000] * 25, [(i * 37) % 1000 for i in range(1024)], 1000, 1000, 16,
     [(2048, 256)]),
    ("512-segments", list(range(0, 500)) + [500] * 13, [(i * 37) % 300 for i in range(512)], 300, 500, 16, [(2048, 256)]),
    ("513-segments", list(range(0, 513)) + [513], [(i * 11) % 40 for i in range(513)], 40, 513, 16, [(2048, 128)]),
    ("1023-rows", [0, 1000, 1023], [1, 0], 2, 1023, 16, [(2048, 128)]),
    ("1024-rows", [0, 1000, 1024], [1, 0], 2, 1024, 16, [(2048, 128)]),
    ("700-segments-ragged-k", list(range(0, 701)), [(i * 3) % 50 for i in range(700)], 50, 700, 16, [(3400, 72), (2048, 64)]),
    ("rank64", list(range(0, 130, 2)), decode_ids(64, 6, 7), 6, 130, 64, [(4096, 512)]),
    ("rank128", list(range(0, 100, 2)), decode_ids(49, 5, 9), 5, 98, 128, [(4096, 256)]),
    ("rank72-tile-blocks", [0, 600, 1200, 1210], [1, 0, 1], 2, 1210, 72, [(512, 128)]),
    ("short-k-falls-back", list(range(41)), decode_ids(40, 4, 8), 4, 40, 16, [(512, 256)]),   # four-wave shrink: plan launch first
    # larger batches (from 512 rows at rank 64, 2560 at rank 16): the tile-block shrink finds its tile blocks (up to 256 segments)
    ("tile-blocks", [0, 700, 1100, 1101, 1500], [0, 1, 3, 2], 4, 1500, 64, [(2048, 320)]),
    ("tile-blocks-finetune-serve", [0, 1024, 2048, 3072, 4096] + list(range(4097, 4225)),
     [0, 1, 2, 3] + [4 + i % 32 for i in range(128)], 36, 4224, 16, [(4096, 512)]),
    ("tile-blocks-prefill-mlp", [0, 512, 1024, 1536, 2048] + list(range(2049, 2113)), [i % 16 for i in range(68)], 16, 2112,
     32, [(1024, 704), (1024, 704), (2752, 256)]),
    ("tile-blocks-256-segments", [5 * i for i in range(257)], [(i * 7) % 300 for i in range(256)], 300, 1300, 64,
     [(512, 128)]),
    ("tile-blocks-257-segments-odd-split-falls-back", [5 * i for i in range(258)], [(i * 7) % 300 for i in range(257)], 300,
     1300, 64, [(512, 128)]),
    # beyond 256 segments: two groups of four waves a workgroup (the k splits must be even)
    ("tile-blocks-300-segments", [5 * i for i in range(301)], [(i * 7) % 300 for i in range(300)], 300, 1510, 64,
     [(2048, 128), (4096, 64)]),
    ("tile-blocks-300-segments-ragged-k", [5 * i for i in range(301)], [(i * 7) % 30 for i in range(300)], 30, 1510, 64,
     [(3400, 72)]),   # four k slices of 1024, the last one 328 long
    ("tile-blocks-512-segments", [3 * i for i in range(513)], [(i * 5) % 37 for i in range(512)], 37, 1540, 32,
     [(2048, 192)]),
    ("tile-blocks-513-segments-fall-back", [3 * i for i in range(514)], [(i * 5) % 37 for i in range(513)], 37, 1540, 32,
     [(2048, 192)]),
]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_deferred_plan_equals_built_plan(K, gpu_device, case, dt):
    name, seg, ids, NA, T, r, projs = case
    T = max(T, seg[-1])
    d, tdt = gpu_device, TDT[dt]
    gen = torch.Generator().manual_seed(61)
    S = len(ids)
    seg_t = torch.tensor(seg, dtype=torch.int32, device=d)
    ids_t = torch.tensor(ids, dtype=torch.int32, device=d)
    used = sorted(set(ids))
    xs, y0, A, B = [], [], [], []
    for h_in, h_out in projs:
        xs.append((torch.randn(T, h_in, generator=gen)).to(tdt).to(d))
        y0.append(torch.randn(T, h_out, generator=gen).to(tdt).to(d))
        # only the adapters in use get weights; the other table entries hold an address that must never be read
        wa = {a: (torch.randn(r, h_in, generator=gen) / h_in ** 0.5).to(tdt).to(d) for a in used}
        wb = {a: (torch.randn(h_out, r, generator=gen) / r ** 0.5).to(tdt).to(d) for a in used}
        A.append(wa)
        B.append(wb)
    tab = lambda w: torch.tensor([w[a].data_ptr() if a in w else 16 for a in range(NA)], dtype=torch.int64, device=d)
    a_tabs, b_tabs = [tab(w) for w in A], [tab(w) for w in B]
    sc = (torch.rand(S, generator=gen) + 0.5).to(d)

    def run(plan):
        ys = [y.clone() for y in y0]
        vs = [torch.full((T, r), 3.0, dtype=tdt, device=d) for _ in projs]
        K.smlm_lora_forward_multi(ys, xs, a_tabs, b_tabs, plan, r, seg_scale=sc, beta=1.0, v_out=vs)
        return ys, vs

    nbytes = max(K.SegmentPlan.nbytes(T, S), 64)
    fresh = lambda: torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=d)  # bytes no build writes stay as they are
    built = K.SegmentPlan(seg_t, ids_t, T, buf=fresh())
    ys_ref, vs_ref = run(built)
    deferred = K.SegmentPlan(seg_t, ids_t, T, buf=fresh(), defer=True)
    assert not deferred.built
    ys, vs = run(deferred)
    assert deferred.built
    torch.cuda.synchronize()
    assert torch.equal(deferred.buf, built.buf), "the call must leave the plan smlm_plan_build writes"
    for i in range(len(projs)):
        assert torch.equal(ys[i], ys_ref[i]) and torch.equal(vs[i], vs_ref[i])
    # the plan it left serves later calls
    ys2, vs2 = run(deferred)
    for i in range(len(projs)):
        assert torch.equal(ys2[i], ys_ref[i]) and torch.equal(vs2[i], vs_ref[i])

    # and the outputs are the oracle's
    from oracle import torch_segments as ref
    for i, (h_in, h_out) in enumerate(projs[:1]):
        wa = [A[i][a].cpu() for a in ids]
        wb = [B[i][a].cpu() for a in ids]
        y_o, v_o = ref.add_lora_forward(xs[i].cpu(), wa, wb, seg, y=y0[i].cpu().clone(), beta=1.0,
                                        seg_scale=sc.cpu().tolist())
        assert torch.allclose(vs[i].cpu().float()[:seg[-1]], v_o.float()[:seg[-1]], rtol=1e-2, atol=1e-3 if dt == "fp16" else 8e-3)
        # y against the oracle fed with the kernel's own v (a rounding flip of v moves a whole row of y)
        vk = vs[i].cpu().float()
        for s_i in range(S):
            lo, hi = seg[s_i], seg[s_i + 1]
            if hi <= lo:
                continue
            want = (y0[i].cpu().float()[lo:hi] + float(sc[s_i]) * (vk[lo:hi] @ wb[s_i].float().t())).to(tdt).float()
            assert torch.allclose(ys[i].cpu().float()[lo:hi], want, rtol=1e-2, atol=2e-2 if dt == "bf16" else 4e-3)
    if T > seg[-1]:  # rows past the last segment are left alone
        for i in range(len(projs)):
            assert torch.equal(ys[i][seg[-1]:], y0[i][seg[-1]:])


def test_deferred_plan_is_built_by_other_users_first(K, gpu_device):
    d = gpu_device
    seg = torch.tensor([0, 3, 9], dtype=torch.int32, device=d)
    ids = torch.tensor([1, 0], dtype=torch.int32, device=d)
    fresh = lambda: torch.full((max(K.SegmentPlan.nbytes(9, 2), 64),), 0xA5, dtype=torch.uint8, device=d)
    p1 = K.SegmentPlan(seg, ids, 9, buf=fresh())
    p2 = K.SegmentPlan(seg, ids, 9, buf=fresh(), defer=True)
    assert not p2.built
    assert p2.header() == p1.header() and p2.built
    torch.cuda.synchronize()
    assert torch.equal(p1.buf, p2.buf)
    # pointer-keyed plans are never deferred
    p3 = K.SegmentPlan(seg, torch.tensor([32, 16], dtype=torch.int64, device=d), 9, defer=True)
    assert p3.built


@pytest.mark.parametrize("seed", range(12, 20))
def test_random_tile_block_batches(K, gpu_device, seed):
    """The same for larger batches (tile blocks of up to 64 rows of one adapter; a batch of 1024 to
    2560 rows takes them or the single tiles according to its rank)."""
    rng = np.random.default_rng(800 + seed)
    d, tdt = gpu_device, [torch.float16, torch.bfloat16][seed % 2]
    NA = int(rng.choice([2, 9, 64, 100, 300, 1024]))
    S = int(rng.integers(2, 257)) if seed % 2 else int(rng.integers(257, 513))
    lens = rng.integers(0, 12, S) if S < 257 else rng.integers(0, 5, S)
    big = rng.random(S) < 0.08
    lens[big] = rng.integers(100, 700, int(big.sum()))
    r = int(rng.choice([8, 16, 32, 64]))
    rows = {8: 2560, 16: 2560, 32: 1280, 64: 512}[r]   # where the forward changes over to tile blocks at this rank
    if lens.sum() < rows:
        lens[0] += rows + 76
    seg = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ids = rng.integers(0, NA, S).astype(np.int32)
    ids[rng.random(S) < 0.03] = -1
    T = int(seg[-1]) + int(rng.integers(0, 40))
    h_in, h_out = int(rng.choice([256, 1024, 2048])), int(rng.choice([64, 136]))
    gen = torch.Generator().manual_seed(int(seed))
    used = sorted(set(int(i) for i in ids if i >= 0))
    wa = {a: (torch.randn(r, h_in, generator=gen) / h_in ** 0.5).to(tdt).to(d) for a in used}
    wb = {a: (torch.randn(h_out, r, generator=gen) / r ** 0.5).to(tdt).to(d) for a in used}
    tab = lambda w: torch.tensor([w[a].data_ptr() if a in w else 16 for a in range(NA)], dtype=torch.int64, device=d)
    ta, tb = tab(wa), tab(wb)
    x = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    y0 = torch.randn(T, h_out, generator=gen).to(tdt).to(d)
    seg_t, ids_t = torch.tensor(seg, device=d), torch.tensor(ids, device=d)
    sc = (torch.rand(S, generator=gen) + 0.5).to(d)
    nbytes = max(K.SegmentPlan.nbytes(T, S), 64)
    out = []
    for defer in (False, True):
        plan = K.SegmentPlan(seg_t, ids_t, T, buf=torch.full((nbytes,), 0x5A, dtype=torch.uint8, device=d), defer=defer)
        y, v = y0.clone(), torch.full((T, r), 3.0, dtype=tdt, device=d)
        K.smlm_lora_forward(y, x, ta, tb, plan, r, seg_scale=sc, beta=1.0, v_out=v)
        torch.cuda.synchronize()
        out.append((y, v, plan.buf))
    served = np.zeros(T, dtype=bool)  # v of rows that no adapter serves is undefined
    for i in range(S):
        if ids[i] >= 0:
            served[seg[i]:seg[i + 1]] = True
    keep = torch.tensor(served, device=d)
    assert torch.equal(out[0][0], out[1][0]) and torch.equal(out[0][1][keep], out[1][1][keep])
    assert torch.equal(out[0][2], out[1][2])
    assert torch.equal(out[1][0][~keep], y0[~keep]) and not torch.equal(out[1][0][keep], y0[keep])


@pytest.mark.parametrize("seed", range(12))
def test_random_decode_batches(K, gpu_device, seed):
    """Random segment tables (empty segments, several rows a segment, uncovered rows, adapters that own
    nothing, a few negative ids = segments no adapter serves): deferred and prebuilt plans agree."""
    rng = np.random.default_rng(700 + seed)
    d, tdt = gpu_device, [torch.float16, torch.bfloat16][seed % 2]
    NA = int(rng.choice([1, 3, 40, 64, 65, 200, 257, 900]))
    S = int(rng.integers(1, 400)) if seed % 3 else int(rng.integers(513, 1025))   # beyond 512: two groups of waves a workgroup
    lens = rng.integers(0, 4, S) if S < 400 else rng.integers(0, 2, S)
    lens[rng.random(S) < 0.05] = int(rng.integers(10, 60))
    while lens.sum() >= 1000:
        lens[int(np.argmax(lens))] = 1
    seg = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ids = rng.integers(0, NA, S).astype(np.int32)
    ids[rng.random(S) < 0.03] = -1
    T = int(seg[-1]) + int(rng.integers(0, 20))
    if T == 0:
        T = 8
    r = int(rng.choice([8, 16, 32, 64]))
    h_in, h_out = 2048, int(rng.choice([64, 136, 512]))
    gen = torch.Generator().manual_seed(int(seed))
    used = sorted(set(int(i) for i in ids if i >= 0))
    wa = {a: (torch.randn(r, h_in, generator=gen) / h_in ** 0.5).to(tdt).to(d) for a in used}
    wb = {a: (torch.randn(h_out, r, generator=gen) / r ** 0.5).to(tdt).to(d) for a in used}
    tab = lambda w: torch.tensor([w[a].data_ptr() if a in w else 16 for a in range(NA)], dtype=torch.int64, device=d)
    ta, tb = tab(wa), tab(wb)
    x = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    y0 = torch.randn(T, h_out, generator=gen).to(tdt).to(d)
    seg_t, ids_t = torch.tensor(seg, device=d), torch.tensor(ids, device=d)
    sc = (torch.rand(S, generator=gen) + 0.5).to(d)
    nbytes = max(K.SegmentPlan.nbytes(T, S), 64)
    out = []
    for defer in (False, True):
        plan = K.SegmentPlan(seg_t, ids_t, T, buf=torch.full((nbytes,), 0x5A, dtype=torch.uint8, device=d), defer=defer)
        y, v = y0.clone(), torch.full((T, r), 3.0, dtype=tdt, device=d)
        K.smlm_lora_forward(y, x, ta, tb, plan, r, seg_scale=sc, beta=1.0, v_out=v)
        torch.cuda.synchronize()
        out.append((y, v, plan.buf))
    for a, b in zip(*out):
        assert torch.equal(a, b)
    # rows that belong to no served segment keep their y
    served = np.zeros(T, dtype=bool)
    for i in range(S):
        if ids[i] >= 0:
            served[seg[i]:seg[i + 1]] = True
    idle = torch.tensor(~served, device=d)
    assert torch.equal(out[1][0][idle], y0[idle])
    assert not torch.equal(out[1][0][~idle], y0[~idle]) or not served.any()


@pytest.mark.parametrize("rows", [40, 400], ids=["single-tiles", "tile-blocks"])
def test_segments_without_adapter_are_left_alone(K, gpu_device, rows):
    """A negative adapter id marks a segment that no adapter serves (a request without LoRA in a mixed
    batch): its rows of y stay as they are, the other segments get the oracle's result."""
    d, tdt = gpu_device, torch.float16
    h_in, h_out, r = 256, 192, 16
    seg = [0, rows, 2 * rows, 2 * rows + 7, 3 * rows + 7, 4 * rows]
    ids = [1, -1, 0, -1, 1]
    T = seg[-1]
    gen = torch.Generator().manual_seed(5)
    A = [(torch.randn(r, h_in, generator=gen) / h_in ** 0.5).to(tdt).to(d) for _ in range(2)]
    B = [(torch.randn(h_out, r, generator=gen) / r ** 0.5).to(tdt).to(d) for _ in range(2)]
    x = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    y0 = torch.randn(T, h_out, generator=gen).to(tdt).to(d)
    plan = K.SegmentPlan(torch.tensor(seg, dtype=torch.int32, device=d), torch.tensor(ids, dtype=torch.int32, device=d), T)
    y = y0.clone()
    K.smlm_lora_forward(y, x, ptrs(A, d), ptrs(B, d), plan, r, beta=1.0)
    from oracle import torch_segments as ref
    for i, a in enumerate(ids):
        lo, hi = seg[i], seg[i + 1]
        if a < 0:
            assert torch.equal(y[lo:hi], y0[lo:hi])
        else:
            want, _ = ref.add_lora_forward(x[lo:hi].cpu(), [A[a].cpu()], [B[a].cpu()], [0, hi - lo],
                                           y=y0[lo:hi].cpu().clone(), beta=1.0)
            assert torch.allclose(y[lo:hi].cpu().float(), want.float(), rtol=1e-2, atol=4e-3)


# name, train partitions, adapter of each, NA, h_in, h_out, rank, v given
BWD_CASES = [
    ("tile-blocks", [0, 500, 520, 1300], [2, 0, 2], 3, 256, 192, 16, True),
    ("finetune-batch", [0, 1024, 2048, 3072, 4096], [0, 1, 2, 3], 4, 1024, 512, 16, True),
    ("rank64-many-parts", [0] + [37 * i + 900 for i in range(1, 200)], [i % 5 for i in range(199)], 5, 320, 128, 64, True),
    ("300-partitions", [0] + [7 * i + 100 for i in range(1, 301)], [i % 9 for i in range(300)], 9, 256, 2048, 16, True),
    ("v-recomputed-falls-back", [0, 700, 1400], [0, 1], 2, 256, 128, 32, False),
    ("few-rows", [0, 35, 90], [0, 1], 2, 192, 320, 16, True),
    ("rank72-single-tiles-fall-back", [0, 35, 90], [0, 1], 2, 192, 320, 72, True),
]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", BWD_CASES, ids=[c[0] for c in BWD_CASES])
def test_backward_deferred_plan_equals_built_plan(K, gpu_device, case, dt):
    """The backward builds a deferred plan too -- inside its dV shrink when that is the first launch to
    need it (ranks up to 64, v given, no dropout), with the plan launch otherwise."""
    name, tp, part_ad, NA, h_in, h_out, r, with_v = case
    d, tdt = gpu_device, TDT[dt]
    n_rows = tp[-1]
    gen = torch.Generator().manual_seed(71)
    A = [(torch.randn(r, h_in, generator=gen) / h_in ** 0.5).to(tdt).to(d) for _ in range(NA)]
    B = [(torch.randn(h_out, r, generator=gen) / r ** 0.5).to(tdt).to(d) for _ in range(NA)]
    x = torch.randn(n_rows, h_in, generator=gen).to(tdt).to(d)
    g = torch.randn(n_rows, h_out, generator=gen).to(tdt).to(d)
    tp_t = torch.tensor(tp, dtype=torch.int32, device=d)
    ad_t = torch.tensor(part_ad, dtype=torch.int32, device=d)
    sc = (torch.rand(len(part_ad), generator=gen) + 0.5).to(d)
    nbytes = max(K.SegmentPlan.nbytes(n_rows, len(part_ad)), 64)
    fresh = lambda: torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=d)
    built = K.SegmentPlan(tp_t, ad_t, n_rows, buf=fresh())
    v = None
    if with_v:
        v = torch.zeros(n_rows, r, dtype=tdt, device=d)
        K.smlm_lora_forward(torch.zeros(n_rows, h_out, dtype=tdt, device=d), x, ptrs(A, d), ptrs(B, d), built, r, v_out=v)

    def run(plan):
        dA, dB = [torch.full_like(a, 5.0) for a in A], [torch.full_like(b, 5.0) for b in B]
        dx = torch.full((n_rows, h_in), 5.0, dtype=tdt, device=d)
        K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), g, x, v, ptrs(A, d), ptrs(B, d), plan, r, sc)
        torch.cuda.synchronize()
        return [dx] + dA + dB

    ref = run(built)
    deferred = K.SegmentPlan(tp_t, ad_t, n_rows, buf=fresh(), defer=True)
    assert not deferred.built
    out = run(deferred)
    assert deferred.built and torch.equal(deferred.buf, built.buf)
    for a, b in zip(ref, out):
        assert torch.equal(a, b)
    for a, b in zip(ref, run(deferred)):   # the plan it left serves the next call
        assert torch.equal(a, b)


@pytest.mark.parametrize("packed", [False, True], ids=["padded", "packed"])
@pytest.mark.parametrize("rows", [60, 1400], ids=["single-tiles", "tile-blocks"])
def test_deferred_plans_with_true_ranks(K, gpu_device, rows, packed):
    """Adapters of different ranks (padded to one rank, or stored at their own): the routes that build
    the plan themselves read the rank table as the planned ones do, forward and backward."""
    d, tdt = gpu_device, torch.bfloat16
    h_in, h_out, r_pad, NA = 2048, 256, 64, 4
    ranks = [8, 16, 32, 64]
    seg = [0, rows // 3, rows // 3 + 1, 2 * rows // 3, rows]
    ids = [2, 0, 3, 1]
    T = rows
    gen = torch.Generator().manual_seed(81)
    A, B = [], []
    for a in range(NA):
        wa, wb = torch.zeros(r_pad, h_in), torch.zeros(h_out, r_pad)
        wa[:ranks[a]] = torch.randn(ranks[a], h_in, generator=gen) / h_in ** 0.5
        wb[:, :ranks[a]] = torch.randn(h_out, ranks[a], generator=gen) / ranks[a] ** 0.5
        if packed:
            wa, wb = wa[:ranks[a]].contiguous(), wb[:, :ranks[a]].contiguous()
        A.append(wa.to(tdt).to(d))
        B.append(wb.to(tdt).to(d))
    x = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    y0 = torch.randn(T, h_out, generator=gen).to(tdt).to(d)
    g = torch.randn(T, h_out, generator=gen).to(tdt).to(d)
    seg_t, ids_t = torch.tensor(seg, dtype=torch.int32, device=d), torch.tensor(ids, dtype=torch.int32, device=d)
    rk = torch.tensor(ranks, dtype=torch.int32, device=d)
    sc = torch.full((len(ids),), 0.5, device=d)
    nbytes = max(K.SegmentPlan.nbytes(T, len(ids)), 64)
    outs = []
    for defer in (False, True):
        fresh = lambda: torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=d)
        plan = K.SegmentPlan(seg_t, ids_t, T, buf=fresh(), defer=defer)
        y, v = y0.clone(), torch.zeros(T, r_pad, dtype=tdt, device=d)
        K.smlm_lora_forward(y, x, ptrs(A, d), ptrs(B, d), plan, r_pad, seg_scale=sc, beta=1.0, v_out=v,
                            adapter_rank=rk, packed_ranks=packed)
        bplan = K.SegmentPlan(seg_t, ids_t, T, buf=fresh(), defer=defer)   # every segment trains here
        dA, dB = [torch.full_like(a, 5.0) for a in A], [torch.full_like(b, 5.0) for b in B]
        dx = torch.full((T, h_in), 5.0, dtype=tdt, device=d)
        K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), g, x, v, ptrs(A, d), ptrs(B, d), bplan, r_pad, sc,
                             adapter_rank=rk, packed_ranks=packed)
        torch.cuda.synchronize()
        outs.append([y, v, dx, plan.buf, bplan.buf] + dA + dB)
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert not torch.isnan(outs[1][2].float()).any()
