"""The backward of several projections in one set of launches (smlm_lora_bwd_multi_ex) against
per-projection calls (bit for bit: the same kernels run with the same launch shapes per
projection) and against the CPU oracle (bit for bit on exactly representable inputs, to the
BASELINE tolerance on Gaussian ones).  Replaces the reference's per-layer Python backward
(src/loquetier_src/kernel_utils.py:128-147)."""
import numpy as np
import pytest
import torch

from test_gpu_parity import ATOL, TDT, K, close, dev_t, dyadic, make_case, ptrs, to_np  # noqa: F401

pytestmark = pytest.mark.gpu

# name, partition indptr, partition adapter, NA, [(h_in, h_out), ...], r
CASES = [
    ("qkv-small", [0, 40, 64, 100], [1, 0, 1], 2, [(256, 256), (256, 64), (256, 64)], 16),
    ("mlp-mixed-widths", [0, 300, 700], [1, 0], 3, [(512, 1408), (512, 1408), (1408, 512)], 32),
    ("rank64-gqa", [0, 33, 90, 130], [0, 2, 1], 4, [(192, 192), (192, 64), (320, 192)], 64),
    ("rank128-one-tile-route", [0, 33, 90], [0, 1], 2, [(192, 320), (320, 192)], 128),
    ("many-rows", [0, 1100, 2300], [0, 1], 2, [(256, 512), (512, 256), (256, 256), (256, 128)], 16),
    ("eight-projections", [0, 50, 75], [0, 0], 1, [(64, 128)] * 8, 8),
]


def _setup(oracle, d, case, dt, dy):
    name, tp, part_ad, NA, dims, r = case
    n_rows = tp[-1]
    projs = []
    for i, (h_in, h_out) in enumerate(dims):
        x, A, B = make_case(oracle, 300 + i, n_rows, None, None, NA, h_in, h_out, r, dt, dy=dy)
        rng = np.random.default_rng(40 + i)
        g = dyadic(rng, (n_rows, h_out), 16, 8) if dy else oracle.round_to(rng.standard_normal((n_rows, h_out)), dt)
        Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
        projs.append(dict(x=x, A=A, B=B, g=g, xd=dev_t(x, dt, d), gd=dev_t(g, dt, d), Ad=Ad, Bd=Bd,
                          a_tab=ptrs(Ad, d), b_tab=ptrs(Bd, d)))
    pi = torch.tensor(tp, dtype=torch.int32, device=d)
    pa = torch.tensor(part_ad, dtype=torch.int32, device=d)
    return projs, pi, pa


def _outputs(projs, d, dt, n_rows):
    out = []
    for p in projs:
        dA, dB = [torch.full_like(a, 7.0) for a in p["Ad"]], [torch.full_like(b, 7.0) for b in p["Bd"]]
        out.append(dict(dx=torch.full((n_rows, p["x"].shape[1]), 7.0, dtype=TDT[dt], device=d), dA=dA, dB=dB,
                        da_tab=ptrs(dA, d), db_tab=ptrs(dB, d)))
    return out


def _multi(K, projs, outs, plan, r, vs=None, scale=None, **kw):
    K.smlm_lora_backward_multi([o["dx"] for o in outs], [o["da_tab"] for o in outs], [o["db_tab"] for o in outs],
                               [p["gd"] for p in projs], [p["xd"] for p in projs], vs,
                               [p["a_tab"] for p in projs], [p["b_tab"] for p in projs], plan, r,
                               part_scale=scale, **kw)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("with_v", [False, True])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_multi_equals_single_calls_and_oracle(K, oracle, gpu_device, case, dt, with_v):
    """Gaussian inputs: one multi call == one call per projection, bit for bit; both within the
    tolerance of the oracle (bf16 dX: atol 4e-3, one bf16 step of a dV element times |A|; dA / dB: atol
    scaled to the size of the sums)."""
    name, tp, part_ad, NA, dims, r = case
    d, n_rows = gpu_device, tp[-1]
    projs, pi, pa = _setup(oracle, d, case, dt, dy=False)
    scale = torch.full((len(part_ad),), 0.5, device=d)
    vs = None
    if with_v:
        vs = []
        for p in projs:
            _, vo = oracle.add_lora_forward(p["x"], [p["A"][a] for a in part_ad], [p["B"][a] for a in part_ad],
                                            tp, p["g"].shape[1], dt)
            vs.append(dev_t(vo, dt, d))
    multi = _outputs(projs, d, dt, n_rows)
    _multi(K, projs, multi, K.SegmentPlan(pi, pa, n_rows), r, vs=vs, scale=scale)
    single = _outputs(projs, d, dt, n_rows)
    plan = K.SegmentPlan(pi, pa, n_rows)
    for i, (p, o) in enumerate(zip(projs, single)):
        K.smlm_lora_backward(o["dx"], o["da_tab"], o["db_tab"], p["gd"], p["xd"], None if vs is None else vs[i],
                             p["a_tab"], p["b_tab"], plan, r, part_scale=scale)
    covered = np.zeros(n_rows, bool)
    for q in range(len(part_ad)):
        covered[tp[q]:tp[q + 1]] = True
    for i, (p, m, s) in enumerate(zip(projs, multi, single)):
        assert torch.equal(m["dx"], s["dx"]), f"dX of projection {i}"
        # the scale 0.5 is a power of two: every scaled value is exactly half the unscaled one
        gx, ga, gb = oracle.add_lora_backward(p["g"], p["x"], p["A"], p["B"], tp, part_ad, dt)
        gx, ga, gb = 0.5 * gx, [0.5 * m for m in ga], [0.5 * m for m in gb]
        close(to_np(m["dx"])[covered], gx[covered], atol=ATOL if dt == "fp16" else 4e-3)
        assert np.all(to_np(m["dx"])[~covered] == 7.0)
        for a in range(NA):
            assert torch.equal(m["dA"][a], s["dA"][a]) and torch.equal(m["dB"][a], s["dB"][a]), (i, a)
            close(to_np(m["dA"][a]), ga[a], atol=ATOL * max(1.0, float(np.abs(ga[a]).max())))
            close(to_np(m["dB"][a]), gb[a], atol=ATOL * max(1.0, float(np.abs(gb[a]).max())))


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_multi_dyadic_bit_exact(K, oracle, gpu_device, case, dt):
    """Exactly representable sums: every projection's dX, dA, dB equal the oracle bit for bit; the plan is
    built by the call itself (deferred)."""
    name, tp, part_ad, NA, dims, r = case
    d, n_rows = gpu_device, tp[-1]
    projs, pi, pa = _setup(oracle, d, case, dt, dy=True)
    outs = _outputs(projs, d, dt, n_rows)
    plan = K.SegmentPlan(pi, pa, n_rows, defer=True)
    _multi(K, projs, outs, plan, r)
    assert plan.built
    covered = np.zeros(n_rows, bool)
    for q in range(len(part_ad)):
        covered[tp[q]:tp[q + 1]] = True
    for i, (p, o) in enumerate(zip(projs, outs)):
        gx, ga, gb = oracle.add_lora_backward(p["g"], p["x"], p["A"], p["B"], tp, part_ad, dt)
        assert np.array_equal(to_np(o["dx"])[covered], gx[covered]), f"dX of projection {i}"
        for a in range(NA):
            assert np.array_equal(to_np(o["dA"][a]), ga[a]), f"dA[{a}] of projection {i}"
            assert np.array_equal(to_np(o["dB"][a]), gb[a]), f"dB[{a}] of projection {i}"


def test_multi_with_dropout_equals_single_calls(K, oracle, gpu_device):
    """Dropout: projection i of a multi call uses the stream offset + i and its part of the keep bits,
    as a per-projection call told that offset and those bits does."""
    case, dt = CASES[1], "bf16"
    name, tp, part_ad, NA, dims, r = case
    d, n_rows = gpu_device, tp[-1]
    projs, pi, pa = _setup(oracle, d, case, dt, dy=False)
    seg_p = torch.tensor([0.25, 0.1], device=d)
    widths = [h_in for h_in, _ in dims]
    for keep_bits in (False, True):
        bits = None
        if keep_bits:  # the forward of the same projections leaves the bits behind
            bits = torch.zeros(K.DropoutSpec.mask_nbytes(n_rows, widths), dtype=torch.uint8, device=d)
            ys = [torch.zeros(n_rows, h_out, dtype=TDT[dt], device=d) for _, h_out in dims]
            K.smlm_lora_forward_multi(ys, [p["xd"] for p in projs], [p["a_tab"] for p in projs],
                                      [p["b_tab"] for p in projs], K.SegmentPlan(pi, pa, n_rows), r,
                                      dropout=K.DropoutSpec(seg_p, n_rows, 5, 16, bits))
        multi = _outputs(projs, d, dt, n_rows)
        _multi(K, projs, multi, K.SegmentPlan(pi, pa, n_rows), r, dropout=K.DropoutSpec(seg_p, n_rows, 5, 16, bits))
        single = _outputs(projs, d, dt, n_rows)
        starts = [K.DropoutSpec.mask_nbytes(n_rows, widths[:i]) for i in range(len(widths))]
        for i, (p, o) in enumerate(zip(projs, single)):
            spec = K.DropoutSpec(seg_p, n_rows, 5, 16 + i, None if bits is None else bits[starts[i]:])
            K.smlm_lora_backward(o["dx"], o["da_tab"], o["db_tab"], p["gd"], p["xd"], None, p["a_tab"], p["b_tab"],
                                 K.SegmentPlan(pi, pa, n_rows), r, dropout=spec)
        for i, (m, s) in enumerate(zip(multi, single)):
            assert torch.equal(m["dx"], s["dx"]), (keep_bits, i)
            for a in range(NA):
                assert torch.equal(m["dA"][a], s["dA"][a]) and torch.equal(m["dB"][a], s["dB"][a]), (keep_bits, i, a)


def test_multi_argument_errors(K, oracle, gpu_device):
    case, dt = CASES[0], "fp16"
    name, tp, part_ad, NA, dims, r = case
    d, n_rows = gpu_device, tp[-1]
    projs, pi, pa = _setup(oracle, d, case, dt, dy=True)
    outs = _outputs(projs, d, dt, n_rows)
    plan = K.SegmentPlan(pi, pa, n_rows)
    with pytest.raises(RuntimeError):  # lists of different lengths
        K.smlm_lora_backward_multi([o["dx"] for o in outs][:2], [o["da_tab"] for o in outs],
                                   [o["db_tab"] for o in outs], [p["gd"] for p in projs], [p["xd"] for p in projs],
                                   None, [p["a_tab"] for p in projs], [p["b_tab"] for p in projs], plan, r)
    with pytest.raises(RuntimeError):  # v of some projections only
        v0 = torch.zeros(n_rows, r, dtype=TDT[dt], device=d)
        _multi(K, projs, outs, plan, r, vs=[v0, None, None])


def test_checked_call_cache_changes_nothing(K, oracle, gpu_device):
    """A layer's dict of checked calls: the second call with the same shapes skips the argument checks and
    reuses the argument blocks; its results equal an uncached call's, other shapes or a tensor the checks
    refuse never take the short way."""
    case, dt = CASES[1], "bf16"
    name, tp, part_ad, NA, dims, r = case
    d, n_rows = gpu_device, tp[-1]
    cache = {}
    projs, pi, pa = _setup(oracle, d, case, dt, dy=False)
    for shift in (0, 1, 2):   # the first call fills the cache, the later ones use it with other data
        for p in projs:
            p["xd"] = p["xd"] + shift
        plan = K.SegmentPlan(pi, pa, n_rows)
        ys = [[torch.zeros(n_rows, h_out, dtype=TDT[dt], device=d) for _, h_out in dims] for _ in range(2)]
        vs = [[torch.zeros(n_rows, r, dtype=TDT[dt], device=d) for _ in dims] for _ in range(2)]
        for which, c in ((0, cache), (1, None)):
            K.smlm_lora_forward_multi(ys[which], [p["xd"] for p in projs], [p["a_tab"] for p in projs],
                                      [p["b_tab"] for p in projs], plan, r, v_out=vs[which], cache=c)
        for a, b in zip(ys[0] + vs[0], ys[1] + vs[1]):
            assert torch.equal(a, b)
        cached, plain = _outputs(projs, d, dt, n_rows), _outputs(projs, d, dt, n_rows)
        _multi(K, projs, cached, plan, r, vs=vs[0], cache=cache)
        _multi(K, projs, plain, plan, r, vs=vs[0])
        for m, s in zip(cached, plain):
            assert torch.equal(m["dx"], s["dx"])
            for a in range(NA):
                assert torch.equal(m["dA"][a], s["dA"][a]) and torch.equal(m["dB"][a], s["dB"][a])
    assert len(cache) == 2
    # a strided x of the same shape is still refused
    wide = torch.zeros(n_rows, 2 * dims[0][0], dtype=TDT[dt], device=d)
    with pytest.raises(RuntimeError):
        K.smlm_lora_forward_multi(ys[0], [wide[:, ::2]] + [p["xd"] for p in projs[1:]], [p["a_tab"] for p in projs],
                                  [p["b_tab"] for p in projs], plan, r, v_out=vs[0], cache=cache)
    # fewer rows than the plan covers: checked and refused, not cut short
    with pytest.raises(RuntimeError):
        K.smlm_lora_forward_multi([y[:-16] for y in ys[0]], [p["xd"] for p in projs], [p["a_tab"] for p in projs],
                                  [p["b_tab"] for p in projs], plan, r, cache=cache)


SIDE_CASES = [
    ("q-o-wide", [0, 600, 1100], [1, 0], 2, [(512, 2048), (2048, 2048)], 16),
    ("mlp-rank64", [0, 300, 700, 1300], [1, 0, 2], 3, [(512, 2816), (512, 2816), (2816, 512)], 64),
]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", SIDE_CASES, ids=[c[0] for c in SIDE_CASES])
def test_fold_writes_what_the_weight_gradients_read(K, oracle, gpu_device, case, dt):
    """Wide outputs: the dV product of every projection is folded from k-split partials and the fold leaves the
    scaled, transposed dV and v behind for the weight-gradient launch (narrow outputs leave that to dX's
    launch: the cases further up).  Values against the oracle, staged calls and a captured call replayed with
    new inputs against the call in one piece, bit for bit."""
    name, tp, part_ad, NA, dims, r = case
    d, n_rows = gpu_device, tp[-1]
    projs, pi, pa = _setup(oracle, d, case, dt, dy=False)
    scales = [0.5, 2.0, 1.0][: len(part_ad)]   # (powers of two: scaled values are the unscaled ones' exact multiples)
    scale = torch.tensor(scales, device=d)
    vs = []
    for p in projs:
        _, vo = oracle.add_lora_forward(p["x"], [p["A"][a] for a in part_ad], [p["B"][a] for a in part_ad],
                                        tp, p["g"].shape[1], dt)
        vs.append(dev_t(vo, dt, d))
    plan = K.SegmentPlan(pi, pa, n_rows)
    whole, staged = _outputs(projs, d, dt, n_rows), _outputs(projs, d, dt, n_rows)
    _multi(K, projs, whole, plan, r, vs=vs, scale=scale)
    for st in (1, 2, 4):   # SMLM_BWD_PRODUCTS, _DX, _WGRAD
        _multi(K, projs, staged, plan, r, vs=vs, scale=scale, stages=st)

    def same(got, want, what):
        for i, (m, s) in enumerate(zip(got, want)):
            assert torch.equal(m["dx"], s["dx"]), (what, i)
            for a in range(NA):
                assert torch.equal(m["dA"][a], s["dA"][a]) and torch.equal(m["dB"][a], s["dB"][a]), (what, i, a)
    same(staged, whole, "staged")
    for i, (p, m) in enumerate(zip(projs, whole)):
        gx, ga, gb = oracle.add_lora_backward(p["g"], p["x"], p["A"], p["B"], tp, part_ad, dt)
        for q, a in enumerate(part_ad):   # (every adapter trains one partition here)
            close(to_np(m["dA"][a]), scales[q] * ga[a], atol=ATOL * max(1.0, float(np.abs(scales[q] * ga[a]).max())))
            close(to_np(m["dB"][a]), scales[q] * gb[a], atol=ATOL * max(1.0, float(np.abs(scales[q] * gb[a]).max())))

    cap = torch.cuda.Stream()
    static = _outputs(projs, d, dt, n_rows)
    with torch.cuda.stream(cap):
        _multi(K, projs, static, plan, r, vs=vs, scale=scale)   # (sizes the workspace of this stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=cap):
        _multi(K, projs, static, plan, r, vs=vs, scale=scale)
    for k in range(3):
        for p in projs:
            p["gd"].copy_(p["gd"] * 0.5 + k)
        for o in static:
            o["dx"].fill_(7.0)
            for t in o["dA"] + o["dB"]:
                t.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        eager = _outputs(projs, d, dt, n_rows)
        _multi(K, projs, eager, plan, r, vs=vs, scale=scale)
        torch.cuda.synchronize()
        same(static, eager, f"replay {k}")


@pytest.mark.parametrize("case", [CASES[0], SIDE_CASES[0]], ids=["dx-launch-writes-the-side-products", "fold-writes-them"])
def test_rows_of_dx_past_the_training_rows_are_cleared_by_the_call(K, oracle, gpu_device, case):
    """dx buffers that cover the whole batch (autograd wants the gradient of all of x): zero_dx_tail makes the call
    clear the rows past the plan's -- inside the fold's launch where there is one for every projection, by a small
    launch of its own otherwise -- and changes nothing else; staged calls do it in their first stage."""
    name, tp, part_ad, NA, dims, r = case
    d, dt, n_rows, extra = gpu_device, "bf16", tp[-1], 37
    projs, pi, pa = _setup(oracle, d, case, dt, dy=False)
    plan = K.SegmentPlan(pi, pa, n_rows)
    plain = _outputs(projs, d, dt, n_rows)
    _multi(K, projs, plain, plan, r)
    for stages in ((0,), (1, 2, 4)):
        wide = _outputs(projs, d, dt, n_rows + extra)
        for st in stages:
            _multi(K, projs, wide, plan, r, zero_dx_tail=True, stages=st)
        for i, (m, s_) in enumerate(zip(wide, plain)):
            assert torch.equal(m["dx"][:n_rows], s_["dx"]), (stages, i)
            assert torch.count_nonzero(m["dx"][n_rows:]) == 0, (stages, i)
            for a in range(NA):
                assert torch.equal(m["dA"][a], s_["dA"][a]) and torch.equal(m["dB"][a], s_["dB"][a]), (stages, i, a)
    with pytest.raises(RuntimeError):  # dx tensors of different heights
        wide = _outputs(projs, d, dt, n_rows + extra)
        wide[0]["dx"] = wide[0]["dx"][:-1]
        _multi(K, projs, wide, plan, r, zero_dx_tail=True)
