"""The entry points under HIP graph capture: nothing in them synchronises, allocates or
clears memory with a memset node, so a captured step must give the eager result on every
replay.  The graph is replayed several times with new inputs, with eager work and
synchronisations in between, and every replay is compared with an eager run bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K(gpu_device):
    from loquetier_amd import _lib
    from loquetier_amd.ops import _kernels
    _lib.load()
    return _kernels


def ptrs(ts, dev):
    return torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=dev)


@pytest.mark.parametrize("T_train,n_dec", [(96, 24), (1200, 40)], ids=["single-tiles", "tile-blocks"])
def test_captured_step_replays_like_eager(K, gpu_device, T_train, n_dec):
    d, tdt = gpu_device, torch.bfloat16
    h_in, h_out, r, NA = 512, 384, 16, 5
    T = T_train + n_dec
    half = T_train // 2
    seg = [0, half, T_train] + [T_train + i + 1 for i in range(n_dec)]
    ids = [0, 1] + [2 + i % 3 for i in range(n_dec)]
    S = len(ids)
    gen = torch.Generator().manual_seed(61)
    A = [(torch.randn(r, h_in, generator=gen) / h_in ** 0.5).to(tdt).to(d) for _ in range(NA)]
    B = [(torch.randn(h_out, r, generator=gen) / r ** 0.5).to(tdt).to(d) for _ in range(NA)]
    ta, tb = ptrs(A, d), ptrs(B, d)
    seg_t = torch.tensor(seg, dtype=torch.int32, device=d)
    ids_t = torch.tensor(ids, dtype=torch.int32, device=d)
    scale = torch.full((S,), 2.0, device=d)
    seg_p = torch.zeros(S, device=d)
    seg_p[:2] = 0.1
    part_t = torch.tensor(seg[:3], dtype=torch.int32, device=d)
    part_ad = torch.tensor([0, 1], dtype=torch.int32, device=d)
    part_scale = torch.full((2,), 2.0, device=d)

    def buffers():
        b = dict(x=torch.empty(T, h_in, dtype=tdt, device=d), y=torch.empty(T, h_out, dtype=tdt, device=d),
                 g=torch.empty(T_train, h_out, dtype=tdt, device=d), v=torch.empty(T, r, dtype=tdt, device=d),
                 dx=torch.empty(T_train, h_in, dtype=tdt, device=d),
                 dA=[torch.empty_like(A[i]) for i in range(2)], dB=[torch.empty_like(B[i]) for i in range(2)],
                 bits=torch.empty(K.DropoutSpec.mask_nbytes(T_train, h_in), dtype=torch.uint8, device=d),
                 plan=torch.empty(K.SegmentPlan.nbytes(T, S), dtype=torch.uint8, device=d),
                 bplan=torch.empty(K.SegmentPlan.nbytes(T_train, 2), dtype=torch.uint8, device=d))
        b["da_tab"], b["db_tab"] = ptrs(b["dA"], d), ptrs(b["dB"], d)
        b["ta2"], b["tb2"] = ptrs(A[:2], d), ptrs(B[:2], d)
        return b

    def step(b):
        plan = K.SegmentPlan(seg_t, ids_t, T, buf=b["plan"])
        drop = K.DropoutSpec(seg_p, T_train, 9, 3, b["bits"])
        K.smlm_lora_forward(b["y"], b["x"], ta, tb, plan, r, seg_scale=scale, beta=1.0, v_out=b["v"], dropout=drop)
        bplan = K.SegmentPlan(part_t, part_ad, T_train, buf=b["bplan"])
        bdrop = K.DropoutSpec(seg_p[:2], T_train, 9, 3, b["bits"])
        K.smlm_lora_backward(b["dx"], b["da_tab"], b["db_tab"], b["g"], b["x"], b["v"], b["ta2"], b["tb2"], bplan,
                             r, part_scale, dropout=bdrop)

    def fill(b, k):
        gk = torch.Generator().manual_seed(100 + k)
        b["x"].copy_(torch.randn(T, h_in, generator=gk).to(tdt))
        b["y"].copy_(torch.randn(T, h_out, generator=gk).to(tdt))
        b["g"].copy_(torch.randn(T_train, h_out, generator=gk).to(tdt))

    def outputs(b):
        return [b["y"], b["v"], b["dx"], b["bits"]] + b["dA"] + b["dB"]

    static, eager = buffers(), buffers()
    side = torch.cuda.Stream()
    fill(static, 0)
    with torch.cuda.stream(side):   # once outside capture: sizes the wrappers' workspace on this stream
        step(static)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    fill(static, 0)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        step(static)
    for k in range(1, 5):
        fill(static, k)
        fill(eager, k)
        torch.cuda.synchronize()
        graph.replay()
        step(eager)                 # eager work of the same kind between the replays
        torch.cuda.synchronize()
        for a, b_ in zip(outputs(static), outputs(eager)):
            assert torch.equal(a, b_), f"replay {k} differs from the eager run"
        assert not torch.isnan(static["dx"].float()).any()


def test_captured_decode_step_builds_its_plan_on_every_replay(K, gpu_device):
    """A decode step captured with a deferred plan: the shrink launch derives the tiles and writes the
    plan itself, so a replay follows whatever routing the segment and adapter tensors hold by then."""
    d, tdt = gpu_device, torch.float16
    T, h_in, h_out, r, NA = 96, 2048, 512, 16, 7
    gen = torch.Generator().manual_seed(62)
    A = [(torch.randn(r, h_in, generator=gen) / h_in ** 0.5).to(tdt).to(d) for _ in range(NA)]
    B = [(torch.randn(h_out, r, generator=gen) / r ** 0.5).to(tdt).to(d) for _ in range(NA)]
    ta, tb = ptrs(A, d), ptrs(B, d)
    seg_t = torch.arange(T + 1, dtype=torch.int32, device=d)
    scale = torch.full((T,), 0.5, device=d)

    def buffers():
        return dict(x=torch.empty(T, h_in, dtype=tdt, device=d), y=torch.empty(T, h_out, dtype=tdt, device=d),
                    v=torch.empty(T, r, dtype=tdt, device=d), ids=torch.zeros(T, dtype=torch.int32, device=d),
                    plan=torch.zeros(K.SegmentPlan.nbytes(T, T), dtype=torch.uint8, device=d))

    def step(b, defer):
        plan = K.SegmentPlan(seg_t, b["ids"], T, buf=b["plan"], defer=defer)
        K.smlm_lora_forward(b["y"], b["x"], ta, tb, plan, r, seg_scale=scale, beta=1.0, v_out=b["v"])
        # a second layer of the step reuses the plan the first one left
        K.smlm_lora_forward(b["y"], b["x"], ta, tb, plan, r, seg_scale=scale, beta=1.0)

    def fill(b, k):
        gk = torch.Generator().manual_seed(200 + k)
        b["x"].copy_(torch.randn(T, h_in, generator=gk).to(tdt))
        b["y"].copy_(torch.randn(T, h_out, generator=gk).to(tdt))
        b["ids"].copy_(torch.randint(0, NA, (T,), generator=gk).to(torch.int32))

    static, eager = buffers(), buffers()
    side = torch.cuda.Stream()
    fill(static, 0)
    with torch.cuda.stream(side):
        step(static, True)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step(static, True)
    for k in range(1, 5):
        fill(static, k)
        fill(eager, k)
        torch.cuda.synchronize()
        graph.replay()
        step(eager, False)          # eager, with the plan launch
        torch.cuda.synchronize()
        for name in ("y", "v"):
            assert torch.equal(static[name], eager[name]), f"replay {k}: {name} differs from the eager run"
        # the plans' headers agree (entries past the live counts keep whatever an earlier batch left)
        assert torch.equal(static["plan"][:64], eager["plan"][:64])
