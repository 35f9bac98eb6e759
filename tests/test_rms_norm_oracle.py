"""Pins the RMSNorm part of the CPU oracle (oracle/rms_norm_oracle.c).  The
reference holds no test or fixture for its rms_norm operator, so the oracle is
pinned by the mathematics: the float64 closed form, special cases with known
answers, invariances, torch.autograd of the float64 composite and finite
differences -- chosen so that a dropped term, a wrong sign or a wrong power of
rms fails one of them.
"""
import numpy as np
import pytest
import torch


def _case(seed, rows=7, cols=48):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    w = (1.0 + 0.3 * rng.standard_normal(cols)).astype(np.float32)
    g = rng.standard_normal((rows, cols)).astype(np.float32)
    return x, w, g


@pytest.mark.parametrize("eps", [1e-6, 1e-5, 0.5])
def test_forward_closed_form(oracle, eps):
    x, w, _ = _case(0)
    out, rms = oracle.rms_norm_fwd(x, w, eps, "fp32")
    x64 = x.astype(np.float64)
    want_rms = 1.0 / np.sqrt((x64 ** 2).mean(axis=1) + eps)
    assert np.allclose(rms, want_rms, rtol=1e-6, atol=0)
    assert np.allclose(out, x64 * want_rms[:, None] * w, rtol=1e-6, atol=1e-7)
    # float accumulation in index order agrees with the double one to float precision
    out32, rms32 = oracle.rms_norm_fwd(x, w, eps, "fp32", acc64=False)
    assert np.allclose(rms32, rms, rtol=1e-5) and np.allclose(out32, out, rtol=1e-5, atol=1e-6)


def test_forward_known_answers(oracle):
    cols = 16
    # a row of equal values c normalises to c / sqrt(c^2 + eps)
    for c, eps in ((2.0, 0.0), (-3.0, 1.0), (0.5, 0.25)):
        x = np.full((1, cols), c, np.float32)
        out, rms = oracle.rms_norm_fwd(x, np.ones(cols, np.float32), eps, "fp32")
        assert np.allclose(out, c / np.sqrt(c * c + eps), rtol=1e-6)
        assert np.allclose(rms, 1.0 / np.sqrt(c * c + eps), rtol=1e-6)
    # a one-hot row: mean of squares = v^2 / cols
    x = np.zeros((1, cols), np.float32)
    x[0, 3] = 4.0
    w = np.arange(1, cols + 1, dtype=np.float32)
    out, rms = oracle.rms_norm_fwd(x, w, 0.0, "fp32")
    assert np.allclose(rms, np.sqrt(cols) / 4.0, rtol=1e-6)
    assert np.allclose(out[0, 3], np.sqrt(cols) * 4.0, rtol=1e-6) and np.count_nonzero(out) == 1
    # an all-zero row stays zero and rms = 1 / sqrt(eps)
    out, rms = oracle.rms_norm_fwd(np.zeros((2, cols), np.float32), w, 1e-4, "fp32")
    assert not out.any() and np.allclose(rms, 100.0, rtol=1e-6)


def test_forward_invariances(oracle):
    x, w, _ = _case(1)
    out, rms = oracle.rms_norm_fwd(x, w, 0.0, "fp32")
    out4, rms4 = oracle.rms_norm_fwd(4.0 * x, w, 0.0, "fp32")  # scaling a row by a power of two
    assert np.allclose(out4, out, rtol=1e-6, atol=1e-7) and np.allclose(rms4, rms / 4.0, rtol=1e-6)
    # the unit-weight output has unit mean square
    unit, _ = oracle.rms_norm_fwd(x, np.ones_like(w), 0.0, "fp32")
    assert np.allclose((unit.astype(np.float64) ** 2).mean(axis=1), 1.0, rtol=1e-5)
    # rows are independent
    one, _ = oracle.rms_norm_fwd(x[2:3], w, 0.0, "fp32")
    assert np.array_equal(one[0], out[2])


@pytest.mark.parametrize("dtype,tdt", [("fp16", torch.float16), ("bf16", torch.bfloat16)])
def test_forward_rounds_once(oracle, dtype, tdt):
    x, w, _ = _case(2)
    x, w = oracle.round_to(x, dtype), oracle.round_to(w, dtype)
    out, _ = oracle.rms_norm_fwd(x, w, 1e-6, dtype)
    exact, _ = oracle.rms_norm_fwd(x, w, 1e-6, "fp32")
    want = torch.from_numpy(exact).to(tdt).float().numpy()
    assert np.array_equal(out, want)


@pytest.mark.parametrize("eps", [1e-6, 0.3])
def test_backward_matches_autograd_and_finite_differences(oracle, eps):
    x, w, g = _case(3, rows=5, cols=24)
    _, rms = oracle.rms_norm_fwd(x, w, eps, "fp32")
    dx, dw = oracle.rms_norm_bwd(g, x, w, rms, "fp32")
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    y = xt * torch.rsqrt((xt ** 2).mean(dim=1, keepdim=True) + eps) * wt
    y.backward(torch.tensor(g, dtype=torch.float64))
    assert np.allclose(dx, xt.grad.numpy(), rtol=1e-5, atol=1e-6)
    assert np.allclose(dw, wt.grad.numpy(), rtol=1e-5, atol=1e-6)

    def loss(xv, wv):
        xv = xv.astype(np.float64)
        return float((xv / np.sqrt((xv ** 2).mean(axis=1, keepdims=True) + eps) * wv * g).sum())

    h = 1e-4
    rng = np.random.default_rng(4)
    for _ in range(12):
        t, j = int(rng.integers(0, x.shape[0])), int(rng.integers(0, x.shape[1]))
        xp, xm = x.astype(np.float64).copy(), x.astype(np.float64).copy()
        xp[t, j] += h
        xm[t, j] -= h
        assert abs((loss(xp, w) - loss(xm, w)) / (2 * h) - dx[t, j]) < 1e-5
        wp, wm = w.astype(np.float64).copy(), w.astype(np.float64).copy()
        wp[j] += h
        wm[j] -= h
        assert abs((loss(x, wp) - loss(x, wm)) / (2 * h) - dw[j]) < 1e-5


def test_backward_invariants(oracle):
    x, w, g = _case(5)
    _, rms = oracle.rms_norm_fwd(x, w, 0.0, "fp32")
    dx, dw = oracle.rms_norm_bwd(g, x, w, rms, "fp32")
    # with eps = 0 the output does not change when a row is scaled: <dx_t, x_t> = 0
    assert np.abs((dx.astype(np.float64) * x).sum(axis=1)).max() < 1e-5
    # dw is linear in g and additive over rows
    dx2, dw2 = oracle.rms_norm_bwd(2.0 * g, x, w, rms, "fp32")
    assert np.allclose(dw2, 2.0 * dw, rtol=1e-6) and np.allclose(dx2, 2.0 * dx, rtol=1e-6, atol=1e-7)
    parts = [oracle.rms_norm_bwd(g[t:t + 1], x[t:t + 1], w, rms[t:t + 1], "fp32") for t in range(x.shape[0])]
    assert np.allclose(sum(p[1].astype(np.float64) for p in parts), dw, rtol=1e-5, atol=1e-6)
    assert np.array_equal(np.concatenate([p[0] for p in parts]), dx)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_literal_reference_rounding_stays_close(oracle, dtype):
    """The reference's Python backward rounds intermediates to 16 bits
    (kernel_utils.py:169-176); restated literally it stays within a few 16-bit
    ulps of the exact gradient -- the bound the GPU kernel (float throughout) is
    held to against the exact mode."""
    x, w, g = _case(6, rows=9, cols=256)
    x, w, g = (oracle.round_to(a, dtype) for a in (x, w, g))
    _, rms = oracle.rms_norm_fwd(x, w, 1e-6, dtype)
    dx, dw = oracle.rms_norm_bwd(g, x, w, rms, dtype)
    dxl, dwl = oracle.rms_norm_bwd(g, x, w, rms, dtype, literal=True)
    ulp = 2.0 ** -10 if dtype == "fp16" else 2.0 ** -7
    assert np.abs(dxl - dx).max() <= 8 * ulp * max(1.0, np.abs(dx).max())
    assert np.abs(dwl - dw).max() <= 4 * ulp * max(1.0, np.abs(dw).max())
