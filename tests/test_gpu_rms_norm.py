"""GPU parity of the RMSNorm kernels (through the C ABI, behind the reference's
`kernel.rms_norm` / `rms_norm.apply` surface) against the CPU oracle.

Bars: where the arithmetic is exact (rows whose mean square is a power of four,
dyadic weights and gradients) the result must equal the oracle exactly (value
for value; the sign of an exactly-zero product is not compared -- the compiler
forms the last multiply and the 16-bit conversion as one fused multiply-add with
a +0 addend, which turns a -0 product into +0);
Gaussian inputs must be within one 16-bit ulp of the oracle's exact-mode output
(the only freedom is the order of the float sum of squares and the last bit of
1/sqrt), which is far inside the rtol 1e-2 / atol 1e-3 stated for this build.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}
ULP = {"fp16": 2.0 ** -10, "bf16": 2.0 ** -7}


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


def run_fwd(K, x, w, eps, dt, dev):
    xd, wd = dev_t(x, dt, dev), dev_t(w, dt, dev)
    o = torch.empty_like(xd)
    m = torch.empty((x.shape[0], 1), dtype=torch.float32, device=dev)
    K.rms_norm(o, m, xd, wd, eps)
    torch.cuda.synchronize()
    return to_np(o), m.cpu().numpy()[:, 0], (xd, wd, m)


def within_ulps(got, want, dt, n):
    tol = n * ULP[dt] * np.maximum(np.abs(want), 2.0 ** -14)
    return np.all(np.abs(got - want) <= tol)


SHAPES = [(1, 8), (3, 64), (4, 4096), (5, 4096), (257, 4096), (33, 1000), (7, 4104), (9, 11008),
          (130, 14336), (2, 16384), (1024, 4096),
          # wider than four waves' registers hold: the two-pass kernels
          (3, 16392), (5, 20480), (2, 32768)]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_forward_gaussian(K, oracle, gpu_device, dt, rows, cols):
    rng = np.random.default_rng(rows * 131 + cols)
    x = oracle.round_to(rng.standard_normal((rows, cols)) * 1.5, dt)
    w = oracle.round_to(1.0 + 0.2 * rng.standard_normal(cols), dt)
    got, rms, _ = run_fwd(K, x, w, 1e-6, dt, gpu_device)
    want, want_rms = oracle.rms_norm_fwd(x, w, 1e-6, dt)
    assert np.allclose(rms, want_rms, rtol=2e-6, atol=0)
    assert within_ulps(got, want, dt, 1)
    assert (got == want).mean() > 0.97
    assert np.allclose(got, want, rtol=1e-2, atol=1e-3)  # the stated bar


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("rows,cols", [(6, 64), (9, 4096), (5, 14336)])
def test_forward_exact(K, oracle, gpu_device, dt, rows, cols):
    """|x| = 2^k along a row: mean square 4^k, rms = 2^-k exactly, out = x * rms * w exact."""
    rng = np.random.default_rng(cols + rows)
    k = rng.integers(-3, 4, rows)
    x = (np.where(rng.random((rows, cols)) < 0.5, -1.0, 1.0) * (2.0 ** k)[:, None]).astype(np.float32)
    w = (rng.integers(-64, 65, cols) / 32.0).astype(np.float32)
    got, rms, _ = run_fwd(K, x, w, 0.0, dt, gpu_device)
    want, want_rms = oracle.rms_norm_fwd(x, w, 0.0, dt)
    assert np.array_equal(rms, want_rms) and np.array_equal(rms, (2.0 ** -k).astype(np.float32))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("rows,cols", [(1, 8), (3, 64), (4, 4096), (5, 4096), (300, 4096), (33, 1000),
                                        (9, 11008), (70, 14336), (2, 16384), (4096, 4096),
                                        (3, 16392), (140, 20480), (2, 32768)])  # the last three: two-pass kernels
def test_backward_gaussian(K, oracle, gpu_device, dt, rows, cols):
    rng = np.random.default_rng(rows * 7 + cols)
    x = oracle.round_to(rng.standard_normal((rows, cols)), dt)
    w = oracle.round_to(1.0 + 0.2 * rng.standard_normal(cols), dt)
    g = oracle.round_to(rng.standard_normal((rows, cols)), dt)
    _, _, (xd, wd, m) = run_fwd(K, x, w, 1e-6, dt, gpu_device)
    gd = dev_t(g, dt, gpu_device)
    dx, dw = torch.empty_like(xd), torch.empty_like(wd)
    K.rms_norm_backward(dx, dw, gd, xd, wd, m)
    torch.cuda.synchronize()
    want_dx, want_dw = oracle.rms_norm_bwd(g, x, w, m.cpu().numpy()[:, 0], dt)
    assert within_ulps(to_np(dx), want_dx, dt, 2)
    assert np.allclose(to_np(dx), want_dx, rtol=1e-2, atol=1e-3)
    # dw sums `rows` terms in float in another order than the oracle's double
    scale = np.sqrt(rows)
    assert np.all(np.abs(to_np(dw) - want_dw) <= 1.5 * ULP[dt] * np.maximum(np.abs(want_dw), scale * 2.0 ** -6))


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_backward_exact(K, oracle, gpu_device, dt):
    """Unit-magnitude rows, dyadic w and g: dot, coef and every term are exact in float."""
    rows, cols = 37, 4096
    rng = np.random.default_rng(11)
    x = np.where(rng.random((rows, cols)) < 0.5, -1.0, 1.0).astype(np.float32)
    w = (rng.integers(-8, 9, cols) / 4.0).astype(np.float32)
    g = (rng.integers(-8, 9, (rows, cols)) / 8.0).astype(np.float32)
    _, rms, (xd, wd, m) = run_fwd(K, x, w, 0.0, dt, gpu_device)
    assert np.array_equal(rms, np.ones(rows, np.float32))
    dx, dw = torch.empty_like(xd), torch.empty_like(wd)
    K.rms_norm_backward(dx, dw, dev_t(g, dt, gpu_device), xd, wd, m)
    torch.cuda.synchronize()
    want_dx, want_dw = oracle.rms_norm_bwd(g, x, w, rms, dt)
    assert np.array_equal(to_np(dx), want_dx)
    assert np.array_equal(to_np(dw), want_dw)


def test_autograd_function_matches_float64_autograd(K, gpu_device):
    from loquetier_amd.kernel_utils import rms_norm
    torch.manual_seed(3)
    x = torch.randn(50, 4096, device=gpu_device).to(torch.bfloat16).requires_grad_()
    w = (1 + 0.1 * torch.randn(4096, device=gpu_device)).to(torch.bfloat16).requires_grad_()
    g = torch.randn(50, 4096, device=gpu_device).to(torch.bfloat16)
    rms_norm.apply(x, w, 1e-5).backward(g)
    x64 = x.detach().double().requires_grad_()
    w64 = w.detach().double().requires_grad_()
    (x64 * torch.rsqrt((x64 ** 2).mean(dim=1, keepdim=True) + 1e-5) * w64).backward(g.double())
    assert torch.allclose(x.grad.double(), x64.grad, rtol=1e-2, atol=4e-3)  # one bf16 ulp at |dx| ~ 0.5
    assert torch.allclose(w.grad.double(), w64.grad, rtol=1e-2, atol=4e-2)  # one bf16 ulp at |dw| ~ 5


def test_deterministic_and_rows_independent(K, oracle, gpu_device):
    rng = np.random.default_rng(5)
    x = oracle.round_to(rng.standard_normal((64, 4096)), "fp16")
    w = oracle.round_to(rng.standard_normal(4096), "fp16")
    a, ra, _ = run_fwd(K, x, w, 1e-6, "fp16", gpu_device)
    b, rb, _ = run_fwd(K, x, w, 1e-6, "fp16", gpu_device)
    assert np.array_equal(a, b) and np.array_equal(ra, rb)
    c, rc, _ = run_fwd(K, x[10:13], w, 1e-6, "fp16", gpu_device)  # same rows in another batch
    assert np.array_equal(c, a[10:13]) and np.array_equal(rc, ra[10:13])


def test_errors_and_empty(K, gpu_device):
    from loquetier_amd import _lib
    dev = gpu_device
    x = torch.zeros(4, 60, dtype=torch.float16, device=dev)
    w = torch.zeros(60, dtype=torch.float16, device=dev)
    o, m = torch.empty_like(x), torch.empty(4, 1, dtype=torch.float32, device=dev)
    with pytest.raises(RuntimeError, match="No suitable kernel"):
        K.rms_norm(o, m, x, w, 1e-6)  # columns not a multiple of 8 (rms_norm_cutlass.cu:166-168)
    x32 = torch.zeros(4, 64, dtype=torch.float32, device=dev)
    with pytest.raises(RuntimeError, match="No suitable kernel"):
        K.rms_norm(torch.empty_like(x32), m, x32, torch.zeros(64, device=dev), 1e-6)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        K.rms_norm(o.cpu(), m, x, w, 1e-6)
    L = _lib.load()
    assert L.smlm_rms_norm_fwd(x.data_ptr(), m.data_ptr(), x.data_ptr(), x.data_ptr(), 1, (1 << 24) + 8, 1e-6,
                               0, None) == -6   # refused before any launch
    empty = torch.zeros(0, 64, dtype=torch.float16, device=dev)
    K.rms_norm(torch.empty_like(empty), torch.empty(0, 1, dtype=torch.float32, device=dev), empty,
               torch.zeros(64, dtype=torch.float16, device=dev), 1e-6)  # no rows: nothing to do
    torch.cuda.synchronize()
