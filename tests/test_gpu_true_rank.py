"""Adapters of different true ranks stored zero-padded to one rank, as the reference keeps
them (MixedLoraModel._prepare_weight, src/loquetier_src/models/mixed_lora.py:501-521): with
`adapter_rank` the kernels skip the padding.  The result must equal the padded computation
bit for bit -- and must not depend on what the padding holds, which is checked by filling it
with NaN."""
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


def padded_adapters(gen, NA, ranks, r_pad, h_in, h_out, tdt, d, poison):
    A, B = [], []
    for a in range(NA):
        ra = ranks[a % len(ranks)]
        wa = torch.zeros(r_pad, h_in)
        wb = torch.zeros(h_out, r_pad)
        wa[:ra] = torch.randn(ra, h_in, generator=gen) / h_in ** 0.5
        wb[:, :ra] = torch.randn(h_out, ra, generator=gen) / ra ** 0.5
        if poison:  # whatever lies past the rank (rounded up to 8) must never be read
            r8 = (ra + 7) // 8 * 8
            wa[r8:] = float("nan")
            wb[:, r8:] = float("nan")
        A.append(wa.to(tdt).to(d))
        B.append(wb.to(tdt).to(d))
    return A, B


# name, T, seg, ids, NA, h_in, h_out, r_pad, true ranks by adapter
CASES = [
    ("small", 90, [0, 20, 41, 41, 60, 77, 90], [0, 1, 2, 3, 1, 2], 4, 256, 192, 64, [8, 16, 32, 64]),
    ("decode-route", 48, list(range(49)), [i % 4 for i in range(48)], 4, 512, 256, 64, [8, 16, 32, 64]),
    ("tile-blocks", 1500, [0, 700, 1100, 1101, 1500], [0, 1, 3, 2], 4, 512, 320, 64, [8, 16, 32, 64]),
    ("rank32-pad", 200, [0, 64, 200], [1, 0], 2, 1024, 128, 32, [8, 24]),
    ("odd-rank", 70, [0, 30, 70], [0, 1], 2, 256, 64, 16, [4, 12]),      # rounded up to 8 and 16 by the kernels
    ("long-k", 70, [0, 33, 70], [1, 0], 2, 4096, 64, 64, [16, 8]),        # k split and folded
]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_forward_with_true_ranks_equals_padded(K, gpu_device, case, dt):
    name, T, seg, ids, NA, h_in, h_out, r_pad, ranks = case
    d, tdt = gpu_device, TDT[dt]
    gen = torch.Generator().manual_seed(51)
    A, B = padded_adapters(gen, NA, ranks, r_pad, h_in, h_out, tdt, d, poison=False)
    gen = torch.Generator().manual_seed(51)
    An, Bn = padded_adapters(gen, NA, ranks, r_pad, h_in, h_out, tdt, d, poison=True)
    x = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    y0 = torch.randn(T, h_out, generator=gen).to(tdt).to(d)
    plan = K.SegmentPlan(torch.tensor(seg, dtype=torch.int32, device=d),
                         torch.tensor(ids, dtype=torch.int32, device=d), T)
    sc = torch.full((len(ids),), 2.0, device=d)
    rk = torch.tensor([ranks[a % len(ranks)] for a in range(NA)], dtype=torch.int32, device=d)

    def run(Aw, Bw, rank_arg):
        y, v = y0.clone(), torch.full((T, r_pad), 7.0, dtype=tdt, device=d)
        K.smlm_lora_forward(y, x, ptrs(Aw, d), ptrs(Bw, d), plan, r_pad, seg_scale=sc, beta=1.0, v_out=v,
                            adapter_rank=rank_arg)
        return y, v

    y_pad, v_pad = run(A, B, None)
    y_rk, v_rk = run(A, B, rk)
    assert torch.equal(y_pad, y_rk) and torch.equal(v_pad, v_rk)
    y_nan, v_nan = run(An, Bn, rk)          # the padding is poisoned and never read
    assert torch.equal(y_pad, y_nan) and torch.equal(v_pad, v_nan)
    assert not torch.isnan(y_nan).any()


BWD_CASES = [
    ("two-parts", [0, 35, 90], [0, 1], 2, 192, 320, 64, [8, 32]),
    ("shared", [0, 40, 70, 100], [1, 0, 1], 2, 128, 256, 32, [16, 8]),
    ("in-place", [0, 500, 520, 1300], [2, 0, 2], 3, 256, 192, 64, [8, 16, 64]),
    ("many-rows", [0, 1100, 2300], [0, 1], 2, 320, 128, 64, [32, 16]),
]


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("with_v", [False, True])
@pytest.mark.parametrize("case", BWD_CASES, ids=[c[0] for c in BWD_CASES])
def test_backward_with_true_ranks_equals_padded(K, gpu_device, case, dt, with_v):
    name, tp, part_ad, NA, h_in, h_out, r_pad, ranks = case
    d, tdt = gpu_device, TDT[dt]
    n_rows = tp[-1]
    gen = torch.Generator().manual_seed(52)
    A, B = padded_adapters(gen, NA, ranks, r_pad, h_in, h_out, tdt, d, poison=False)
    gen = torch.Generator().manual_seed(52)
    An, Bn = padded_adapters(gen, NA, ranks, r_pad, h_in, h_out, tdt, d, poison=True)
    x = torch.randn(n_rows, h_in, generator=gen).to(tdt).to(d)
    g = torch.randn(n_rows, h_out, generator=gen).to(tdt).to(d)
    plan = K.SegmentPlan(torch.tensor(tp, dtype=torch.int32, device=d),
                         torch.tensor(part_ad, dtype=torch.int32, device=d), n_rows)
    rk = torch.tensor([ranks[a % len(ranks)] for a in range(NA)], dtype=torch.int32, device=d)
    v = None
    if with_v:
        v = torch.zeros(n_rows, r_pad, dtype=tdt, device=d)
        K.smlm_lora_forward(torch.zeros(n_rows, h_out, dtype=tdt, device=d), x, ptrs(A, d), ptrs(B, d), plan,
                            r_pad, v_out=v)

    def run(Aw, Bw, rank_arg):
        dA, dB = [torch.full_like(a, 5.0) for a in Aw], [torch.full_like(b, 5.0) for b in Bw]
        dx = torch.empty(n_rows, h_in, dtype=tdt, device=d)
        K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), g, x, v, ptrs(Aw, d), ptrs(Bw, d), plan, r_pad,
                             adapter_rank=rank_arg)
        return [dx] + dA + dB

    pad, rkd, nan = run(A, B, None), run(A, B, rk), run(An, Bn, rk)
    for a, b, c in zip(pad, rkd, nan):
        assert torch.equal(a, b)
        assert torch.equal(a, c)     # gradients of the padding are zeros either way, and no NaN leaks in


def packed(ws, ranks, dim):
    """The same adapters stored at their true rank rounded up to 8 (rows of A, columns of B), each
    inside a guard band that must stay untouched."""
    out = []
    for a, w in enumerate(ws):
        r8 = (ranks[a % len(ranks)] + 7) // 8 * 8
        w = (w[:r8] if dim == 0 else w[:, :r8]).contiguous()
        out.append(w)
    return out


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_forward_with_packed_ranks_equals_padded(K, gpu_device, case, dt):
    """Adapters stored at their true rank (A_a [r_a, h_in], B_a [h_out, r_a]): the bits of the padded run."""
    name, T, seg, ids, NA, h_in, h_out, r_pad, ranks = case
    d, tdt = gpu_device, TDT[dt]
    gen = torch.Generator().manual_seed(51)
    A, B = padded_adapters(gen, NA, ranks, r_pad, h_in, h_out, tdt, d, poison=False)
    x = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    y0 = torch.randn(T, h_out, generator=gen).to(tdt).to(d)
    plan = K.SegmentPlan(torch.tensor(seg, dtype=torch.int32, device=d),
                         torch.tensor(ids, dtype=torch.int32, device=d), T)
    sc = torch.full((len(ids),), 2.0, device=d)
    rk = torch.tensor([ranks[a % len(ranks)] for a in range(NA)], dtype=torch.int32, device=d)

    def run(Aw, Bw, rank_arg, pk):
        y, v = y0.clone(), torch.full((T, r_pad), 7.0, dtype=tdt, device=d)
        K.smlm_lora_forward(y, x, ptrs(Aw, d), ptrs(Bw, d), plan, r_pad, seg_scale=sc, beta=1.0, v_out=v,
                            adapter_rank=rank_arg, packed_ranks=pk)
        return y, v

    y_pad, v_pad = run(A, B, None, False)
    y_pk, v_pk = run(packed(A, ranks, 0), packed(B, ranks, 1), rk, True)
    assert torch.equal(y_pad, y_pk) and torch.equal(v_pad, v_pk)
    with pytest.raises(RuntimeError, match="adapter_rank"):
        run(A, B, None, True)


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("with_v", [False, True])
@pytest.mark.parametrize("case", BWD_CASES, ids=[c[0] for c in BWD_CASES])
def test_backward_with_packed_ranks_equals_padded(K, gpu_device, case, dt, with_v):
    """Packed storage in the backward: dX as padded; dA_a [r_a, h_in] and dB_a [h_out, r_a] are the
    leading rows / columns of the padded gradients, and nothing is written outside them."""
    name, tp, part_ad, NA, h_in, h_out, r_pad, ranks = case
    d, tdt = gpu_device, TDT[dt]
    n_rows = tp[-1]
    gen = torch.Generator().manual_seed(52)
    A, B = padded_adapters(gen, NA, ranks, r_pad, h_in, h_out, tdt, d, poison=False)
    x = torch.randn(n_rows, h_in, generator=gen).to(tdt).to(d)
    g = torch.randn(n_rows, h_out, generator=gen).to(tdt).to(d)
    plan = K.SegmentPlan(torch.tensor(tp, dtype=torch.int32, device=d),
                         torch.tensor(part_ad, dtype=torch.int32, device=d), n_rows)
    rk = torch.tensor([ranks[a % len(ranks)] for a in range(NA)], dtype=torch.int32, device=d)
    v = None
    if with_v:
        v = torch.zeros(n_rows, r_pad, dtype=tdt, device=d)
        K.smlm_lora_forward(torch.zeros(n_rows, h_out, dtype=tdt, device=d), x, ptrs(A, d), ptrs(B, d), plan,
                            r_pad, v_out=v)
    dA, dB = [torch.full_like(a, 5.0) for a in A], [torch.full_like(b, 5.0) for b in B]
    dx = torch.empty(n_rows, h_in, dtype=tdt, device=d)
    K.smlm_lora_backward(dx, ptrs(dA, d), ptrs(dB, d), g, x, v, ptrs(A, d), ptrs(B, d), plan, r_pad)
    Ap, Bp = packed(A, ranks, 0), packed(B, ranks, 1)
    # gradients inside guard bands: 64 elements of 9.0 either side of every packed matrix
    guard = 64
    bufs = [torch.full((w.numel() + 2 * guard,), 9.0, dtype=tdt, device=d) for w in Ap + Bp]
    views = [b[guard: guard + w.numel()].view(w.shape) for b, w in zip(bufs, Ap + Bp)]
    dAp, dBp = views[:NA], views[NA:]
    dxp = torch.empty(n_rows, h_in, dtype=tdt, device=d)
    K.smlm_lora_backward(dxp, ptrs(dAp, d), ptrs(dBp, d), g, x, v, ptrs(Ap, d), ptrs(Bp, d), plan, r_pad,
                         adapter_rank=rk, packed_ranks=True)
    assert torch.equal(dx, dxp)
    for a in range(NA):
        r8 = Ap[a].size(0)
        assert torch.equal(dAp[a], dA[a][:r8]) and torch.equal(dBp[a], dB[a][:, :r8])
    for b in bufs:
        assert bool((b[:guard] == 9.0).all()) and bool((b[-guard:] == 9.0).all())


def test_layer_with_true_ranks_equals_padded_layer(K, gpu_device):
    """MixedLoraLinear: adapters that carry their true rank give the bits (output and
    gradients) of the same adapters treated as full-rank."""
    from loquetier_amd.kernel_utils import BatchLenInfo
    from loquetier_amd.mixed_lora import MixedLoraContext, MixedLoraLinear, NamedLoraLayer, prepare_weight
    from loquetier_amd.segments import build_segments
    d, tdt = gpu_device, torch.bfloat16
    h_in, h_out, r_pad, ranks = 256, 320, 32, [8, 32, 16]
    gen = torch.Generator().manual_seed(71)
    raw = [((torch.randn(q, h_in, generator=gen) / 16), (torch.randn(h_out, q, generator=gen) / 4)) for q in ranks]
    req_ids, req_len = [2, 0, 0, 1, 1, 2], [40, 24, 5, 1, 1, 1]   # train on adapters 2 and 0
    T = sum(req_len)
    x0 = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    g = torch.randn(T, h_out, generator=gen).to(tdt).to(d)
    base = torch.nn.Linear(h_in, h_out, bias=False, device=d, dtype=tdt)
    base.weight.requires_grad_(False)
    results = []
    for with_rank in (False, True):
        adapters = [NamedLoraLayer(f"a{i}", prepare_weight(wa, r_pad, tdt, d, rank_dim=0),
                                   prepare_weight(wb, r_pad, tdt, d, rank_dim=1), torch.nn.Identity(), 2.0,
                                   true_rank=ranks[i] if with_rank else None) for i, (wa, wb) in enumerate(raw)]
        ctx = MixedLoraContext()
        layer = MixedLoraLinear(ctx, base, adapters, r_pad, tdt, is_scaled=False, fused=True)
        assert (layer.adapter_rank is not None) == with_rank
        layer.set_trainable([2, 0])
        lora_ids, lora_len, segment = build_segments(req_ids, req_len, d)
        ctx.update(blen=BatchLenInfo([(1, 40), (1, 24)], [5], 3, [], d), lora_ids=lora_ids, lora_len=lora_len,
                   segment=segment, train_idx=[2, 0])
        x = x0.clone().requires_grad_(True)
        out = layer(x)
        out.backward(g)
        results.append([out.detach(), x.grad] + [layer.get_parameter(f"lora-{i}-{m}").grad for i in (2, 0) for m in "AB"])
    for a, b in zip(*results):
        assert torch.equal(a, b)
    assert not (results[1][2][16:] != 0).any()  # dA of adapter 2 (true rank 16): the padding rows get zero gradient


def test_layer_with_packed_adapters_equals_padded_layer(K, gpu_device):
    """MixedLoraLinear over adapters stored at their own rank (prepare_weight(pack=True)): output, dX
    and the parameters' gradients (in the parameters' packed shapes) are those of the padded layer."""
    from loquetier_amd.kernel_utils import BatchLenInfo
    from loquetier_amd.mixed_lora import MixedLoraContext, MixedLoraLinear, NamedLoraLayer, prepare_weight
    from loquetier_amd.segments import build_segments
    d, tdt = gpu_device, torch.bfloat16
    h_in, h_out, r_pad, ranks = 256, 320, 32, [8, 32, 12]
    gen = torch.Generator().manual_seed(72)
    raw = [((torch.randn(q, h_in, generator=gen) / 16), (torch.randn(h_out, q, generator=gen) / 4)) for q in ranks]
    req_ids, req_len = [2, 0, 0, 1, 1, 2], [40, 24, 5, 1, 1, 1]   # train on adapters 2 and 0
    T = sum(req_len)
    x0 = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    g = torch.randn(T, h_out, generator=gen).to(tdt).to(d)
    base = torch.nn.Linear(h_in, h_out, bias=False, device=d, dtype=tdt)
    base.weight.requires_grad_(False)
    results = []
    for pack in (False, True):
        adapters = [NamedLoraLayer(f"a{i}", prepare_weight(wa, r_pad, tdt, d, rank_dim=0, pack=pack),
                                   prepare_weight(wb, r_pad, tdt, d, rank_dim=1, pack=pack), torch.nn.Identity(), 2.0,
                                   true_rank=ranks[i]) for i, (wa, wb) in enumerate(raw)]
        ctx = MixedLoraContext()
        layer = MixedLoraLinear(ctx, base, adapters, r_pad, tdt, is_scaled=False, fused=True)
        assert layer.packed == pack
        if pack:
            assert [tuple(a.wa.shape) for a in adapters] == [(8, h_in), (32, h_in), (16, h_in)]
            assert [tuple(a.wb.shape) for a in adapters] == [(h_out, 8), (h_out, 32), (h_out, 16)]
        layer.set_trainable([2, 0])
        lora_ids, lora_len, segment = build_segments(req_ids, req_len, d)
        ctx.update(blen=BatchLenInfo([(1, 40), (1, 24)], [5], 3, [], d), lora_ids=lora_ids, lora_len=lora_len,
                   segment=segment, train_idx=[2, 0])
        x = x0.clone().requires_grad_(True)
        out = layer(x)
        out.backward(g)
        results.append([out.detach(), x.grad] + [layer.get_parameter(f"lora-{i}-{m}").grad for i in (2, 0) for m in "AB"])
    pad, pk = results
    assert torch.equal(pad[0], pk[0]) and torch.equal(pad[1], pk[1])
    r8 = {2: 16, 0: 8}
    for k, (i, m) in enumerate([(2, "A"), (2, "B"), (0, "A"), (0, "B")]):
        want = pad[2 + k][: r8[i]] if m == "A" else pad[2 + k][:, : r8[i]]
        assert pk[2 + k].shape == want.shape and torch.equal(pk[2 + k], want)
    with pytest.raises(RuntimeError, match="fused"):
        MixedLoraLinear(MixedLoraContext(), base, adapters, r_pad, tdt, is_scaled=False, fused=False)
