"""Error budgets of the 16-bit backward.

The operator keeps its rank-r intermediates (v, dV) in the I/O dtype, as the reference does
(`mid = g @ wb.T` is a 16-bit tensor, src/loquetier_src/kernel_utils.py:141).  One element of dV
rounding the other way moves a whole row of dX, so the comparisons with the 16-bit oracle in
tests/test_gpu_parity.py carry an absolute tolerance wider than 1e-3 for bf16 gradients.  These
tests bound what hides inside that tolerance: against the exact result (the oracle in float64
with no intermediate rounding) the HIP kernels must not err more than the reference's own
semantics do (the oracle with 16-bit intermediates, double accumulation), beyond one rounding of
the output:

    rms(gpu - exact)  <= 1.10 * rms(oracle16 - exact) + tiny
    max|gpu - exact|  <= 1.5 * max|oracle16 - exact| + ulp(max|exact|)

A kernel that loses a few ulp somewhere (a product rounded twice, a partial sum kept in 16 bits)
fails the first line; a wrong element fails the second.  Full-size Gaussian inputs of the
fine-tune + serve batch are checked the same way."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}
ULP = {"fp16": 2.0 ** -10, "bf16": 2.0 ** -7}   # spacing of the dtype just below 2.0, relative to 1


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


def within_budget(name, gpu, ref16, exact, dt):
    e_gpu, e_ref = gpu.astype(np.float64) - exact, ref16.astype(np.float64) - exact
    rms_gpu, rms_ref = np.sqrt(np.mean(e_gpu ** 2)), np.sqrt(np.mean(e_ref ** 2))
    ulp = ULP[dt] * float(np.abs(exact).max())
    assert rms_gpu <= 1.10 * rms_ref + 1e-7, f"{name}: rms error {rms_gpu:.4g} vs reference semantics {rms_ref:.4g}"
    assert np.abs(e_gpu).max() <= 1.5 * np.abs(e_ref).max() + ulp, \
        f"{name}: max error {np.abs(e_gpu).max():.4g} vs reference semantics {np.abs(e_ref).max():.4g} (+ {ulp:.3g})"


def run_backward(K, d, dt, x, A, B, g, tp, part_ad, r, v=None, scale=None):
    n_rows = tp[-1]
    xd, gd = dev_t(x, dt, d), dev_t(g, dt, d)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    dA, dB = [torch.empty_like(a) for a in Ad], [torch.empty_like(b) for b in Bd]
    dx = torch.empty(n_rows, x.shape[1], dtype=TDT[dt], device=d)
    plan = K.SegmentPlan(torch.tensor(tp, dtype=torch.int32, device=d),
                         torch.tensor(part_ad, dtype=torch.int32, device=d), n_rows)
    K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), gd, xd, None if v is None else dev_t(v, dt, d),
                         ptrs(Ad, d), ptrs(Bd, d), plan, r, scale)
    return to_np(dx), [to_np(t) for t in dA], [to_np(t) for t in dB]


def gaussian(oracle, seed, n_rows, NA, h_in, h_out, r, dt):
    rng = np.random.default_rng(seed)
    x = oracle.round_to(rng.standard_normal((n_rows, h_in)), dt)
    g = oracle.round_to(rng.standard_normal((n_rows, h_out)), dt)
    A = [oracle.round_to(rng.standard_normal((r, h_in)) / np.sqrt(h_in), dt) for _ in range(NA)]
    B = [oracle.round_to(rng.standard_normal((h_out, r)) / np.sqrt(r), dt) for _ in range(NA)]
    return x, g, A, B


CASES = [
    # name, tp, part_ad, NA, h_in, h_out, r  (the shapes whose tolerances are widened in test_gpu_parity.py)
    ("two-parts", [0, 5, 12], [0, 1], 2, 64, 96, 8),
    ("blocks", [0, 500, 520, 1300], [2, 0, 2], 3, 256, 192, 16),
    ("shared-adapter", [0, 40, 70, 100], [1, 0, 1], 2, 128, 256, 16),
    ("rank64", [0, 33, 90], [0, 1], 2, 192, 320, 64),
    ("long", [0, 300, 700], [1, 0], 2, 512, 384, 16),
    ("long-k", [0, 30, 75], [1, 0], 2, 4096, 2048, 16),
    ("rank128", [0, 33, 90], [0, 1], 2, 192, 320, 128),
]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_backward_error_no_larger_than_the_reference_semantics(K, oracle, gpu_device, case, dt):
    name, tp, part_ad, NA, h_in, h_out, r = case
    x, g, A, B = gaussian(oracle, 301, tp[-1], NA, h_in, h_out, r, dt)
    dx, dA, dB = run_backward(K, gpu_device, dt, x, A, B, g, tp, part_ad, r)
    x16, a16, b16 = oracle.add_lora_backward(g, x, A, B, tp, part_ad, dt)        # 16-bit intermediates
    x64, a64, b64 = oracle.add_lora_backward(g, x, A, B, tp, part_ad, "fp32")    # exact
    within_budget("dX", dx, x16, x64, dt)
    for a in sorted(set(part_ad)):
        within_budget(f"dA[{a}]", dA[a], a16[a], a64[a], dt)
        within_budget(f"dB[{a}]", dB[a], b16[a], b64[a], dt)


def test_forward_error_no_larger_than_the_reference_semantics(K, oracle, gpu_device):
    """The same budget for the forward in bf16, where v is rounded to 8 bits between the products."""
    d, dt = gpu_device, "bf16"
    T, NA, h_in, h_out, r = 300, 4, 1024, 768, 16
    rng = np.random.default_rng(302)
    seg = [0, 40, 41, 200, 300]
    ids = [2, 0, 3, 1]
    x, _, A, B = gaussian(oracle, 303, T, NA, h_in, h_out, r, dt)
    base = oracle.round_to(rng.standard_normal((T, h_out)), dt)
    y = dev_t(base, dt, d)
    s = torch.tensor(seg, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(s, torch.tensor(ids, dtype=torch.int32, device=d), T)
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    K.smlm_lora_forward(y, dev_t(x, dt, d), ptrs(Ad, d), ptrs(Bd, d), plan, r,
                        seg_scale=torch.full((4,), 2.0, device=d), beta=1.0)
    wa, wb = [A[i] for i in ids], [B[i] for i in ids]
    y16, _ = oracle.lora_fused(base, x, wa, wb, seg, [2.0] * 4, 1.0, dt)
    y64, _ = oracle.lora_fused(base, x, wa, wb, seg, [2.0] * 4, 1.0, "fp32")
    within_budget("y", to_np(y), y16, y64, dt)


def test_full_size_gaussian_backward_finetune_batch(K, oracle, gpu_device):
    """Gaussian inputs at the size of the fine-tune + serve batch (4 x 1024 training rows on adapters
    0-3, h = 4096, r = 16, bf16, upstream gradient ~ N(0,1)): dX, dA, dB within the stated tolerance
    of the 16-bit oracle and within the error budget of the exact one; with the v the forward kernel
    saved, as a training step runs it, and per-segment scale 2."""
    d, dt, r, NA = gpu_device, "bf16", 16, 4
    tp, part_ad = [0, 1024, 2048, 3072, 4096], [0, 1, 2, 3]
    x, g, A, B = gaussian(oracle, 304, 4096, NA, 4096, 4096, r, dt)
    # forward on the device: its rounded v is what the backward reuses
    Ad, Bd = [dev_t(a, dt, d) for a in A], [dev_t(b, dt, d) for b in B]
    s = torch.tensor(tp, dtype=torch.int32, device=d)
    plan = K.SegmentPlan(s, torch.tensor(part_ad, dtype=torch.int32, device=d), 4096)
    y = torch.zeros(4096, 4096, dtype=TDT[dt], device=d)
    v = torch.zeros(4096, r, dtype=TDT[dt], device=d)
    K.smlm_lora_forward(y, dev_t(x, dt, d), ptrs(Ad, d), ptrs(Bd, d), plan, r, v_out=v)
    _, v16 = oracle.add_lora_forward(x, A, B, tp, 4096, dt)
    v_np = to_np(v)
    assert np.abs(v_np - v16).max() <= 1e-3 + 1e-2 * np.abs(v16).max()
    scale = torch.full((4,), 2.0, device=d)
    dx, dA, dB = run_backward(K, d, dt, x, A, B, g, tp, part_ad, r, v=v_np, scale=scale)
    x16, a16, b16 = oracle.add_lora_backward(g, x, A, B, tp, part_ad, dt)
    x64, a64, b64 = oracle.add_lora_backward(g, x, A, B, tp, part_ad, "fp32")
    # tolerance against the 16-bit oracle: rtol 1e-2; atol = one bf16 step of the intermediate (|dV| < 16:
    # 2^-4) times |A| ~ 1/64 per element over r terms for dX, and 1e-3 of the largest entry for the sums
    # over 1024 tokens
    def close(got, want, atol):
        err = np.abs(got - want)
        assert (err <= atol + 1e-2 * np.abs(want)).all(), f"max err {err.max():.4g} (atol {atol:.3g})"
    close(dx, 2.0 * x16, 8e-3)
    for a in range(NA):
        close(dA[a], 2.0 * a16[a], 1e-3 * float(np.abs(a16[a]).max()) * 2.0)
        close(dB[a], 2.0 * b16[a], 1e-3 * float(np.abs(b16[a]).max()) * 2.0)
    within_budget("dX", dx, 2.0 * x16, 2.0 * x64.astype(np.float64), dt)
    for a in range(NA):
        within_budget(f"dA[{a}]", dA[a], 2.0 * a16[a], 2.0 * a64[a].astype(np.float64), dt)
        within_budget(f"dB[{a}]", dB[a], 2.0 * b16[a], 2.0 * b64[a].astype(np.float64), dt)
