"""Pins the CPU oracle (oracle/smlm_oracle.c) before anything is checked
against it.  The reference has no golden vector or known-answer test for the
SMLM path, so every function of the oracle is pinned by what the mathematics
fixes: library GEMMs per segment, brute force on tiny inputs, autograd of the
float64 composite, finite differences, invariants, exact small-integer cases.
"""
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "smlm_small.npz")


def _rand_case(rng, T, seg, ids, NA, h_in, h_out, r):
    x = rng.standard_normal((T, h_in)).astype(np.float32)
    A = [(rng.standard_normal((r, h_in)) / np.sqrt(h_in)).astype(np.float32) for _ in range(NA)]
    B = [(rng.standard_normal((h_out, r)) / np.sqrt(r)).astype(np.float32) for _ in range(NA)]
    return x, A, B


# ---------------------------------------------------------------- rounding --
@pytest.mark.parametrize("dtype,tdt", [("fp16", torch.float16), ("bf16", torch.bfloat16)])
def test_round_matches_torch_cast(oracle, dtype, tdt):
    rng = np.random.default_rng(1)
    vals = [rng.standard_normal(50000) * s for s in (1e-8, 1e-5, 1e-3, 1.0, 100.0, 3e4, 7e4)]
    # exact ties between neighbouring 16-bit values, both parities of the lower neighbour
    bits = np.arange(0, 0x7BFF if dtype == "fp16" else 0x7F7F, dtype=np.uint16)
    lo = torch.from_numpy(bits.view(np.int16)).view(tdt).to(torch.float64).numpy()
    ties = (lo[:-1] + lo[1:]) / 2
    special = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e30, -1e30, np.inf, -np.inf,
                        5.96e-8, 2.98e-8, 2.981e-8, 6.1e-5, 1e-45, 3.3895e38, 3.4e38])
    allv = np.concatenate(vals + [ties, -ties, special]).astype(np.float32)
    got = oracle.round_to(allv, dtype)
    want = torch.from_numpy(allv).to(tdt).to(torch.float32).numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    nan = oracle.round_to(np.array([np.nan], np.float32), dtype)
    assert np.isnan(nan[0])


def test_round_fp32_is_identity(oracle):
    a = np.random.default_rng(2).standard_normal(1000).astype(np.float32)
    assert np.array_equal(oracle.round_to(a, "fp32"), a)


# ----------------------------------------------------------- grouped GEMM ---
@pytest.mark.parametrize("row_major", [False, True])
def test_gemm_matches_numpy_per_segment(oracle, row_major):
    rng = np.random.default_rng(3)
    T, d_in, d_out = 23, 40, 24
    seg = [2, 7, 7, 15, 20]  # starts after row 0, one empty segment, ends before T
    x = rng.standard_normal((T, d_in)).astype(np.float32)
    W = [rng.standard_normal((d_in, d_out)).astype(np.float32) for _ in range(4)]
    w_in = [w if row_major else np.ascontiguousarray(w.T) for w in W]
    y = np.full((T, d_out), 7.5, np.float32)
    oracle.smlm_gemm(y, x, w_in, seg, row_major, "fp32", acc64=True)
    want = np.full((T, d_out), 7.5)
    for i in range(4):
        want[seg[i]:seg[i + 1]] = x[seg[i]:seg[i + 1]].astype(np.float64) @ W[i].astype(np.float64)
    np.testing.assert_allclose(y, want, rtol=1e-6, atol=1e-6)
    # rows outside every segment are untouched (beta = 0 overwrites only covered rows)
    assert np.all(y[:2] == 7.5) and np.all(y[20:] == 7.5)


def test_gemm_single_segment_is_one_library_gemm(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((9, 32)).astype(np.float32)
    w = rng.standard_normal((16, 32)).astype(np.float32)  # column-major view of a 32x16 matrix
    y = np.zeros((9, 16), np.float32)
    oracle.smlm_gemm(y, x, [w], [0, 9], False, "fp32")
    np.testing.assert_allclose(y, x.astype(np.float64) @ w.T.astype(np.float64), rtol=1e-6, atol=1e-6)


def test_gemm_float_accumulate_is_index_order(oracle):
    # acc64 = False: plain float accumulation in k order, reproduced here by a Python loop
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 50)).astype(np.float32)
    w = rng.standard_normal((8, 50)).astype(np.float32)
    y = np.zeros((3, 8), np.float32)
    oracle.smlm_gemm(y, x, [w], [0, 3], False, "fp32", acc64=False)
    for i in range(3):
        for j in range(8):
            acc = np.float32(0)
            for k in range(50):
                acc = np.float32(acc + np.float32(x[i, k] * w[j, k]))
            assert y[i, j] == acc


def test_routing_brute_force_and_exact_integers(oracle):
    # small integers: every product and sum is exact in fp16, so routing errors
    # (wrong adapter, shifted row, wrong segment edge) change bits
    rng = np.random.default_rng(6)
    T, h_in, h_out, r, NA = 19, 16, 24, 8, 3
    seg = [0, 1, 1, 6, 7, 19]
    ids = [1, 2, 0, 1, 2]
    x = rng.integers(-2, 3, (T, h_in)).astype(np.float32)
    A = [rng.integers(-1, 2, (r, h_in)).astype(np.float32) for _ in range(NA)]
    B = [rng.integers(-1, 2, (h_out, r)).astype(np.float32) for _ in range(NA)]
    y, v = oracle.add_lora_forward(x, [A[i] for i in ids], [B[i] for i in ids], seg, h_out, "fp16")
    for t in range(T):  # closed form: the unique i with seg[i] <= t < seg[i+1]
        owner = [i for i in range(len(ids)) if seg[i] <= t < seg[i + 1]]
        assert len(owner) == 1
        a = ids[owner[0]]
        vt = [sum(int(x[t, k]) * int(A[a][j, k]) for k in range(h_in)) for j in range(r)]
        yt = [sum(vt[j] * int(B[a][n, j]) for j in range(r)) for n in range(h_out)]
        assert v[t].tolist() == vt
        assert y[t].tolist() == yt


def test_forward_is_two_gemm_calls_with_rounded_v(oracle):
    rng = np.random.default_rng(7)
    T, h_in, h_out, r = 12, 48, 40, 16
    seg, ids = [0, 4, 12], [1, 0]
    x, A, B = _rand_case(rng, T, seg, ids, 2, h_in, h_out, r)
    for dt, tdt in (("fp16", torch.float16), ("bf16", torch.bfloat16)):
        xr = oracle.round_to(x, dt)
        Ar = [oracle.round_to(a, dt) for a in A]
        Br = [oracle.round_to(b, dt) for b in B]
        y, v = oracle.add_lora_forward(xr, [Ar[i] for i in ids], [Br[i] for i in ids], seg, h_out, dt)
        for i, a in enumerate(ids):
            s0, s1 = seg[i], seg[i + 1]
            v64 = xr[s0:s1].astype(np.float64) @ Ar[a].T.astype(np.float64)
            vw = torch.from_numpy(v64).to(torch.float32).to(tdt).to(torch.float64).numpy()
            assert np.array_equal(v[s0:s1].astype(np.float64), vw)
            y64 = vw @ Br[a].T.astype(np.float64)
            yw = torch.from_numpy(y64).to(torch.float32).to(tdt).to(torch.float32).numpy()
            assert np.array_equal(y[s0:s1], yw)


def test_baseline_config_1_cpu(oracle):
    """BASELINE config 1: fp32, 64 tokens in 4 segments of 16 -> adapters
    [0,1,2,3], h=4096, r=16, scale 2, accumulate into zero y."""
    rng = np.random.default_rng(1)
    T, h, r = 64, 4096, 16
    seg = [0, 16, 32, 48, 64]
    x = rng.standard_normal((T, h)).astype(np.float32)
    A = [(rng.standard_normal((r, h)) / 64.0).astype(np.float32) for _ in range(4)]
    B = [(rng.standard_normal((h, r)) / 4.0).astype(np.float32) for _ in range(4)]
    y, v = oracle.lora_fused(np.zeros((T, h), np.float32), x, A, B, seg, seg_scale=[2.0] * 4,
                             beta=1.0, dtype="fp32", acc64=False)
    want = np.zeros((T, h))
    for i in range(4):
        xs = x[seg[i]:seg[i + 1]].astype(np.float64)
        want[seg[i]:seg[i + 1]] = 2.0 * (xs @ A[i].T.astype(np.float64)) @ B[i].T.astype(np.float64)
    np.testing.assert_allclose(y, want, rtol=1e-4, atol=1e-4)
    # float accumulation against double accumulation: the fp32 path is what config 1 names
    y64, _ = oracle.lora_fused(np.zeros((T, h), np.float32), x, A, B, seg, seg_scale=[2.0] * 4,
                               beta=1.0, dtype="fp32", acc64=True)
    np.testing.assert_allclose(y64, want, rtol=2e-6, atol=2e-6)


def test_fused_and_reference_tail_agree_without_rounding(oracle):
    # in fp32 the fused epilogue and the reference's three-step tail are the same arithmetic
    rng = np.random.default_rng(8)
    T, h_in, h_out, r = 10, 32, 24, 8
    seg, ids = [0, 3, 10], [0, 1]
    x, A, B = _rand_case(rng, T, seg, ids, 2, h_in, h_out, r)
    base = rng.standard_normal((T, h_out)).astype(np.float32)
    sc = [2.0, 0.5]
    a = oracle.mixed_lora_linear(base, x, [A[i] for i in ids], [B[i] for i in ids], seg, sc, "fp32")
    b, _ = oracle.lora_fused(base, x, [A[i] for i in ids], [B[i] for i in ids], seg, sc, 1.0, "fp32")
    np.testing.assert_allclose(a, b, rtol=1e-6, atol=1e-6)
    want = base.astype(np.float64).copy()
    for i, ad in enumerate(ids):
        xs = x[seg[i]:seg[i + 1]].astype(np.float64)
        want[seg[i]:seg[i + 1]] += sc[i] * (xs @ A[ad].T.astype(np.float64)) @ B[ad].T.astype(np.float64)
    np.testing.assert_allclose(b, want, rtol=1e-5, atol=1e-5)


def test_rank_padding_is_exact(oracle):
    # an adapter zero-padded to the layer rank gives bit-identical outputs
    rng = np.random.default_rng(9)
    T, h_in, h_out, r0, r = 7, 32, 40, 8, 32
    x = oracle.round_to(rng.standard_normal((T, h_in)), "bf16")
    A0 = rng.standard_normal((r0, h_in)).astype(np.float32) / 6
    B0 = rng.standard_normal((h_out, r0)).astype(np.float32) / 3
    A0r, B0r = oracle.round_to(A0, "bf16"), oracle.round_to(B0, "bf16")
    Ap = oracle.prepare_weight(A0, 0, r, None, "bf16")
    Bp = oracle.prepare_weight(B0, 1, r, None, "bf16")
    assert Ap.shape == (r, h_in) and Bp.shape == (h_out, r)
    assert np.array_equal(Ap[:r0], A0r) and not Ap[r0:].any()
    assert np.array_equal(Bp[:, :r0], B0r) and not Bp[:, r0:].any()
    y0, _ = oracle.add_lora_forward(x, [A0r], [B0r], [0, T], h_out, "bf16")
    y1, _ = oracle.add_lora_forward(x, [Ap], [Bp], [0, T], h_out, "bf16")
    assert np.array_equal(y0, y1)
    # scale folding: multiply, then cast (mixed_lora.py:509-521)
    As = oracle.prepare_weight(A0, 0, r, 2.0, "bf16")
    assert np.array_equal(As[:r0], oracle.round_to(A0 * np.float32(2.0), "bf16"))


# ---------------------------------------------------------------- backward --
def _autograd_reference(x, A, B, g, tp, part_ad):
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    At = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in A]
    Bt = [torch.tensor(b, dtype=torch.float64, requires_grad=True) for b in B]
    gt = torch.tensor(g, dtype=torch.float64)
    tot = torch.zeros((), dtype=torch.float64)
    for p, ad in enumerate(part_ad):
        s0, s1 = tp[p], tp[p + 1]
        tot = tot + ((xt[s0:s1] @ At[ad].T @ Bt[ad].T) * gt[s0:s1]).sum()
    tot.backward()
    z = lambda t, like: np.zeros_like(like, dtype=np.float64) if t.grad is None else t.grad.numpy()
    return xt.grad.numpy(), [z(a, A[i]) for i, a in enumerate(At)], [z(b, B[i]) for i, b in enumerate(Bt)]


def test_backward_matches_autograd_of_composite(oracle):
    rng = np.random.default_rng(10)
    T, h_in, h_out, r, NA = 17, 24, 32, 8, 3
    tp, part_ad = [0, 4, 9, 9, 14], [1, 0, 2, 1]   # adapter 1 trains twice, one empty partition
    x, A, B = _rand_case(rng, T, None, None, NA, h_in, h_out, r)
    g = rng.standard_normal((T, h_out)).astype(np.float32)
    gx, ga, gb = oracle.add_lora_backward(g, x, A, B, tp, part_ad, "fp32")
    wx, wa, wb = _autograd_reference(x, A, B, g, tp, part_ad)
    np.testing.assert_allclose(gx, wx, rtol=1e-5, atol=1e-5)
    assert not gx[14:].any()  # rows past the train partitions get zero gradient
    for i in range(NA):
        np.testing.assert_allclose(ga[i], wa[i], rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(gb[i], wb[i], rtol=1e-5, atol=1e-5)
    # adapter 2 owns only the empty partition -> exact zeros
    assert not ga[2].any() and not gb[2].any()


def test_backward_finite_differences(oracle):
    rng = np.random.default_rng(11)
    T, h_in, h_out, r = 5, 6, 7, 8
    x = rng.standard_normal((T, h_in))
    A = rng.standard_normal((r, h_in))
    B = rng.standard_normal((h_out, r))
    g = rng.standard_normal((T, h_out))
    f = lambda x_, A_, B_: float(((x_ @ A_.T @ B_.T) * g).sum())
    gx, ga, gb = oracle.add_lora_backward(g, x, [A], [B], [0, T], [0], "fp32")
    eps = 1e-3
    for arr, grad, name in ((x, gx, "x"), (A, ga[0], "A"), (B, gb[0], "B")):
        for idx in [(0, 0), (1, 3), (arr.shape[0] - 1, arr.shape[1] - 1)]:
            p, m = arr.copy(), arr.copy()
            p[idx] += eps
            m[idx] -= eps
            args_p = {"x": (p, A, B), "A": (x, p, B), "B": (x, A, p)}[name]
            args_m = {"x": (m, A, B), "A": (x, m, B), "B": (x, A, m)}[name]
            fd = (f(*args_p) - f(*args_m)) / (2 * eps)
            assert abs(fd - grad[idx]) < 2e-3 * max(1.0, abs(fd)), (name, idx, fd, grad[idx])


def test_backward_homogeneity_identity(oracle):
    # y is linear in each of x, A, B: <dY, Y> = <dX, x> = <dA, A> = <dB, B>
    rng = np.random.default_rng(12)
    T, h_in, h_out, r = 11, 40, 24, 16
    x, A, B = _rand_case(rng, T, None, None, 1, h_in, h_out, r)
    g = rng.standard_normal((T, h_out)).astype(np.float32)
    y, _ = oracle.add_lora_forward(x, A, B, [0, T], h_out, "fp32")
    gx, ga, gb = oracle.add_lora_backward(g, x, A, B, [0, T], [0], "fp32")
    ref = float((g.astype(np.float64) * y).sum())
    for val in ((gx.astype(np.float64) * x).sum(), (ga[0].astype(np.float64) * A[0]).sum(),
                (gb[0].astype(np.float64) * B[0]).sum()):
        assert abs(val - ref) < 1e-4 * max(1.0, abs(ref))


def test_backward_literal_rowmajor_is_transpose_of_layout_used(oracle):
    """The reference's backward lines are valid for wa [h_in,r], wb [r,h_out];
    with wa = A^T, wb = B^T they must give the transposes of the gradients for
    A [r,h_in], B [h_out,r]."""
    rng = np.random.default_rng(13)
    T, h_in, h_out, r = 13, 24, 40, 8
    tp = [0, 6, 13]
    x, A, B = _rand_case(rng, T, None, None, 2, h_in, h_out, r)
    g = rng.standard_normal((T, h_out)).astype(np.float32)
    gx, ga, gb = oracle.add_lora_backward(g, x, A, B, tp, [0, 1], "fp32")
    gx2, gwa, gwb = oracle.add_lora_backward_rowmajor(
        g, x, [np.ascontiguousarray(a.T) for a in A], [np.ascontiguousarray(b.T) for b in B], tp, "fp32")
    np.testing.assert_allclose(gx, gx2, rtol=1e-6, atol=1e-6)
    for i in range(2):
        np.testing.assert_allclose(ga[i], gwa[i].T, rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(gb[i], gwb[i].T, rtol=1e-5, atol=1e-5)
    # and the literal lines against numpy, term by term (kernel_utils.py:141-144)
    for p in range(2):
        s0, s1 = tp[p], tp[p + 1]
        wa, wb = A[p].T.astype(np.float64), B[p].T.astype(np.float64)
        gp, xp = g[s0:s1].astype(np.float64), x[s0:s1].astype(np.float64)
        mid = gp @ wb.T
        np.testing.assert_allclose(gx2[s0:s1], mid @ wa.T, rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(gwa[p], xp.T @ mid, rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(gwb[p], wa.T @ xp.T @ gp, rtol=1e-5, atol=1e-5)


def test_backward_shared_adapter_is_sum_of_partitions(oracle):
    rng = np.random.default_rng(14)
    T, h_in, h_out, r = 12, 16, 24, 8
    x, A, B = _rand_case(rng, T, None, None, 1, h_in, h_out, r)
    g = rng.standard_normal((T, h_out)).astype(np.float32)
    _, ga, gb = oracle.add_lora_backward(g, x, A, B, [0, 5, 12], [0, 0], "fp32")
    _, ga1, gb1 = oracle.add_lora_backward(g, x, A, B, [0, 5], [0], "fp32")
    g2, x2 = g[5:], x[5:]
    _, ga2, gb2 = oracle.add_lora_backward(g2, x2, A, B, [0, 7], [0], "fp32")
    np.testing.assert_allclose(ga[0], ga1[0] + ga2[0], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(gb[0], gb1[0] + gb2[0], rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------ index makers --
def test_build_segments_brute_force(oracle):
    rng = np.random.default_rng(15)
    for _ in range(50):
        n = int(rng.integers(1, 30))
        ids = rng.integers(0, 4, n).tolist()
        lens = rng.integers(1, 9, n).tolist()
        got_ids, got_len, got_seg = oracle.build_segments(ids, lens)
        exp_ids, exp_len = [], []
        for i, l in zip(ids, lens):
            if exp_ids and exp_ids[-1] == i:
                exp_len[-1] += l
            else:
                exp_ids.append(i)
                exp_len.append(l)
        assert got_ids == exp_ids
        assert got_len.tolist() == exp_len
        assert got_seg.tolist() == np.concatenate([[0], np.cumsum(exp_len)]).tolist()
        assert all(a != b for a, b in zip(got_ids, got_ids[1:]))  # neighbours differ
        assert got_seg[-1] == sum(lens)


def test_batch_len_info(oracle):
    tp, tlen, doff = oracle.batch_len_info([(2, 8), (1, 5)], [3, 4])
    assert tp.tolist() == [0, 16, 21] and tlen == 21 and doff == 28
    tp, tlen, doff = oracle.batch_len_info([], [])
    assert tp.tolist() == [0] and tlen == 0 and doff == 0


# ------------------------------------------------------------ golden file ---
@pytest.mark.parametrize("dt", ["fp32", "fp16", "bf16"])
def test_oracle_matches_golden_fixture(oracle, dt):
    z = np.load(GOLDEN)
    seg, ids, tp, tp_ad = z["seg"], z["ids"], z["tp"], z["tp_ad"]
    x, A, B, g = z[f"{dt}_x"], z[f"{dt}_A"], z[f"{dt}_B"], z[f"{dt}_g"]
    y, v = oracle.add_lora_forward(x, [A[i] for i in ids], [B[i] for i in ids], seg, B.shape[1], dt)
    tol = dict(rtol=1e-6, atol=1e-6) if dt == "fp32" else dict(rtol=0, atol=0)
    np.testing.assert_allclose(v, z[f"{dt}_v"], **tol)
    np.testing.assert_allclose(y, z[f"{dt}_y"], **tol)
    gx, ga, gb = oracle.add_lora_backward(g, x, list(A), list(B), tp, tp_ad, dt)
    np.testing.assert_allclose(gx, z[f"{dt}_dx"], **tol)
    np.testing.assert_allclose(np.stack(ga), z[f"{dt}_dA"], **tol)
    np.testing.assert_allclose(np.stack(gb), z[f"{dt}_dB"], **tol)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_reference_tail_rounding_points_against_torch_16bit_ops(oracle, dt):
    """oracle_mixed_lora_linear in 16 bits, bit for bit against torch's CPU fp16 / bf16 tensor ops
    applied as the reference applies them (src/loquetier_src/models/mixed_lora.py:214-217):
    lora_res (a 16-bit tensor) * scaling[lora_ids] repeated per row (a 16-bit tensor, so the
    scale itself is rounded) -> rounded; result + lora_res -> rounded.  The scales are not
    representable in 16 bits and the values are random, so a rounding that is skipped, moved
    behind the add, or taken with the unrounded scale changes bits."""
    import torch
    tdt = torch.float16 if dt == "fp16" else torch.bfloat16
    rng = np.random.default_rng(77)
    T, h_in, h_out, r = 37, 64, 96, 8
    seg, ids = [0, 5, 5, 20, 37], [1, 0, 2, 1]
    x, A, B = _rand_case(rng, T, seg, ids, 3, h_in, h_out, r)
    x = oracle.round_to(x, dt)
    A = [oracle.round_to(a, dt) for a in A]
    B = [oracle.round_to(b, dt) for b in B]
    base = oracle.round_to(rng.standard_normal((T, h_out)), dt)
    sc = [0.3, 1.7, 0.123, 2.9]   # none exact in fp16 or bf16
    wa, wb = [A[i] for i in ids], [B[i] for i in ids]
    got = oracle.mixed_lora_linear(base, x, wa, wb, seg, sc, dt)
    # the LoRA term as the kernel hands it back: a 16-bit tensor (pinned by the GEMM tests above)
    lora, _ = oracle.add_lora_forward(x, wa, wb, seg, h_out, dt)
    lora_t = torch.from_numpy(lora).to(tdt)
    scaling = torch.tensor(sc, dtype=tdt)                       # mixed_lora.py:163-166
    lens = torch.tensor([seg[i + 1] - seg[i] for i in range(len(ids))])
    lora_t = lora_t * torch.repeat_interleave(scaling, lens).unsqueeze(-1)   # :214-216
    result = torch.from_numpy(base).to(tdt) + lora_t                          # :217
    assert np.array_equal(got, result.float().numpy())
    # and the roundings matter on this input: one rounding at the end gives other bits
    fused, _ = oracle.lora_fused(base, x, wa, wb, seg, sc, 1.0, dt)
    assert not np.array_equal(got, fused)
    # without a scale only the add is rounded
    got1 = oracle.mixed_lora_linear(base, x, wa, wb, seg, None, dt)
    want1 = torch.from_numpy(base).to(tdt) + torch.from_numpy(lora).to(tdt)
    assert np.array_equal(got1, want1.float().numpy())
