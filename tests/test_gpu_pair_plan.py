"""Plans keyed by a PAIR of weight addresses per segment (smlm_plan_build2, SMLM_KEY_PTR2): what the
reference's add_lora.forward is handed -- wa_ptr[i], wb_ptr[i] per problem
(src/loquetier_src/kernel_utils.py:115-119) -- served by ONE plan and one fused call.  Segments that
share both addresses share tiles; segments that share A and differ in B (or the other way round) do not.
The plan a fused call builds itself equals the one the plan launch builds, byte for byte, and the outputs
equal the oracle's bit for bit on exactly representable inputs."""
import numpy as np
import pytest
import torch

from test_gpu_parity import TDT, K, dev_t, dyadic, ptrs, to_np  # noqa: F401

pytestmark = pytest.mark.gpu

# name, seg, A index per segment, B index per segment, h_in, h_out, r
CASES = [
    ("decode-shared-pairs", list(range(201)), [i % 5 for i in range(200)], [i % 5 for i in range(200)], 2048, 256, 16),
    ("decode-a-shared-b-not", list(range(121)), [i % 3 for i in range(120)], [i % 7 for i in range(120)], 2048, 192, 16),
    ("ragged-empty-segments", [0, 10, 10, 25, 26, 40, 60, 60], [0, 1, 0, 1, 0, 1, 0], [0, 1, 1, 1, 0, 0, 0], 256, 192, 16),
    ("tile-blocks", [0, 700, 1100, 1101, 1500, 2300], [0, 1, 0, 1, 0], [2, 1, 2, 0, 2], 512, 320, 64),
    ("600-segments", list(range(0, 1200, 2)) + [1200], [(i * 7) % 11 for i in range(600)], [(i * 3) % 4 for i in range(600)],
     2048, 128, 16),
    # more tiles (tile blocks) than the launch has rows of workgroups -- a table entry per segment, so the launch
    # is sized for the usual batch (rows / 16 + 33 tiles): its workgroups go round again
    ("100-distinct-pairs-three-rounds", list(range(101)), [i % 10 for i in range(100)], [(i // 10) % 10 for i in range(100)],
     2048, 128, 16),
    ("80-distinct-pairs-tile-blocks-two-rounds", list(range(0, 644, 4)), [i % 10 for i in range(160)],
     [(i // 10) % 8 for i in range(160)], 2048, 192, 64),
    ("1500-segments-two-launch-plan", list(range(1501)), [(i * 7) % 9 for i in range(1500)],
     [(i * 5) % 6 for i in range(1500)], 256, 128, 8),
]


def _inputs(case, dt, d):
    name, seg, a_of, b_of, h_in, h_out, r = case
    rng = np.random.default_rng(91)
    T = seg[-1]
    x, base = dyadic(rng, (T, h_in), 16, 8), dyadic(rng, (T, h_out), 16, 8)
    A = [dyadic(rng, (r, h_in), 8, 64) for _ in range(max(a_of) + 1)]
    B = [dyadic(rng, (h_out, r), 8, 8) for _ in range(max(b_of) + 1)]
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    wa, wb = ptrs([Ad[i] for i in a_of], d), ptrs([Bd[i] for i in b_of], d)
    return T, x, base, A, B, Ad, Bd, wa, wb


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_pair_plan_fused_forward_bit_exact(K, oracle, gpu_device, case, dt):
    name, seg, a_of, b_of, h_in, h_out, r = case
    d = gpu_device
    T, x, base, A, B, Ad, Bd, wa, wb = _inputs(case, dt, d)
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    S = len(a_of)
    scale = (np.random.default_rng(92).integers(1, 5, S) / 2.0).astype(np.float32)
    want, v_want = oracle.lora_fused(base, x, [A[i] for i in a_of], [B[i] for i in b_of], seg, scale, 1.0, dt)
    plans = []
    nbytes = max(K.SegmentPlan.nbytes(T, S), 64)
    fresh = lambda: torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=d)  # bytes no build writes stay as they are
    for defer in (False, True):
        y = dev_t(base, dt, d)
        v = torch.zeros(T, r, dtype=TDT[dt], device=d)
        plan = K.SegmentPlan(s, (wa, wb), T, buf=fresh(), defer=defer)
        assert plan.built != defer
        K.smlm_lora_forward(y, dev_t(x, dt, d), wa, wb, plan, r, seg_scale=torch.from_numpy(scale).to(d), beta=1.0,
                            v_out=v)
        torch.cuda.synchronize()
        assert plan.built
        assert np.array_equal(to_np(y), want), f"y (defer={defer})"
        covered = np.zeros(T, bool)
        for i in range(S):
            covered[seg[i]:seg[i + 1]] = True
        assert np.array_equal(to_np(v)[covered], v_want[covered]), f"v (defer={defer})"
        plans.append(plan)
    # the plan the call built itself is the plan the plan launch builds
    assert torch.equal(plans[0].buf, plans[1].buf)
    # groups: one per distinct pair that has rows (a plan of at most 1024 segments; the two-launch route may split
    # pairs that share A into more groups, never fewer)
    n_tiles, n_groups, rows, kind = plans[1].header()
    pairs = {(a_of[i], b_of[i]) for i in range(S) if seg[i + 1] > seg[i]}
    all_pairs = {(a_of[i], b_of[i]) for i in range(S)}
    assert rows == T
    if S <= 1024:
        assert n_groups == len(all_pairs)
    else:
        assert n_groups >= len(pairs)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_add_lora_apply_one_plan_one_call(K, oracle, gpu_device, dt, monkeypatch):
    """add_lora.apply (the surface MixedLoraLinear calls, kernel_utils.py:101-120) issues one fused call over one
    plan that the call builds itself: no plan launch of its own for a decode batch, results the oracle's."""
    from loquetier_amd import kernel_utils as ku
    d = gpu_device
    case = CASES[1]
    name, seg, a_of, b_of, h_in, h_out, r = case
    T, x, base, A, B, Ad, Bd, wa, wb = _inputs(case, dt, d)
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    calls = []
    real = ku.kernel.smlm_lora_forward_multi

    def spy(*a, **kw):
        calls.append((kw.get("stages", 3), a[4].built))
        return real(*a, **kw)
    monkeypatch.setattr(ku.kernel, "smlm_lora_forward_multi", spy)
    y = ku.add_lora.apply((T, h_out), dev_t(x, dt, d), wa, wb, s, r, 0, [])
    want, _ = oracle.add_lora_forward(x, [A[i] for i in a_of], [B[i] for i in b_of], seg, h_out, dt)
    assert np.array_equal(to_np(y), want)
    assert calls == [(3, False)]   # both stages in one call, the plan not built beforehand
