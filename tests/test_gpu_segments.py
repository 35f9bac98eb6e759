"""The device segment builder against the oracle's restatement of the host loop
(src/loquetier_src/model_generation.py:267-283), bit for bit, and the forward
fed with its padded outputs against the forward fed with the host's."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from loquetier_amd.ops import _kernels
    return _kernels


def requests(name, rng):
    if name == "one":
        return [3], [7]
    if name == "all-same":
        return [5] * 40, list(rng.integers(1, 9, 40))
    if name == "all-different":
        return list(range(300)), [1] * 300
    if name == "zero-lengths":  # a request without tokens still opens a segment when its id differs
        return [1, 1, 2, 2, 1, 3, 3], [4, 0, 0, 5, 0, 0, 0]
    if name == "decode-mix":
        return list(rng.integers(0, 4, 700)), list(rng.integers(0, 3, 700))
    if name == "beyond-one-pass":  # more requests than the workgroup has threads: the carry is used
        ids = np.repeat(rng.integers(0, 50, 1500), rng.integers(1, 5, 1500))[:3000]
        return list(ids), list(rng.integers(0, 20, len(ids)))
    if name == "pass-boundary":  # a run that straddles request 1024
        return [0] * 1000 + [9] * 48 + [4] * 10, [1] * 1058
    raise KeyError(name)


CASES = ["one", "all-same", "all-different", "zero-lengths", "decode-mix", "beyond-one-pass", "pass-boundary"]


@pytest.mark.parametrize("name", CASES)
def test_device_segments_equal_the_host_loop(K, oracle, gpu_device, name):
    ids, lens = requests(name, np.random.default_rng(11))
    R = len(ids)
    o_ids, o_len, o_seg = oracle.build_segments(ids, lens)
    S, rows = len(o_ids), int(o_seg[-1])
    d_ids = torch.tensor(ids, dtype=torch.int32, device=gpu_device)
    d_len = torch.tensor(lens, dtype=torch.int32, device=gpu_device)
    seg_adapter, seg_len, seg_indptr, n_seg = K.segments_build(d_ids, d_len)
    assert n_seg.tolist() == [S, rows]
    assert seg_adapter.shape == (R,) and seg_len.shape == (R,) and seg_indptr.shape == (R + 1,)
    assert seg_adapter[:S].tolist() == o_ids
    assert np.array_equal(seg_len[:S].cpu().numpy(), o_len)
    assert np.array_equal(seg_indptr[:S + 1].cpu().numpy(), o_seg)
    # the unused capacity describes empty segments at the end of the batch
    assert (seg_indptr[S:] == rows).all() and (seg_len[S:] == 0).all()
    assert (seg_adapter[S:] == ids[-1]).all()


def test_no_requests(K, gpu_device):
    e = torch.empty(0, dtype=torch.int32, device=gpu_device)
    seg_adapter, seg_len, seg_indptr, n_seg = K.segments_build(e, e)
    assert seg_indptr.tolist() == [0] and n_seg.tolist() == [0, 0] and seg_adapter.numel() == 0


def test_rejects_wrong_inputs(K, gpu_device):
    i32 = torch.zeros(4, dtype=torch.int32, device=gpu_device)
    with pytest.raises(RuntimeError, match="int32"):
        K.segments_build(i32.long(), i32)
    with pytest.raises(RuntimeError, match="one entry per request"):
        K.segments_build(i32, i32[:3].contiguous())
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        K.segments_build(i32.cpu(), i32.cpu())


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_forward_from_device_built_segments(K, oracle, gpu_device, dt):
    """The padded device outputs (S = R, empty segments at the end) drive the fused
    forward to the same bits as the host-built segments."""
    rng = np.random.default_rng(12)
    ids = list(np.repeat(rng.integers(0, 6, 60), rng.integers(1, 4, 60)))
    lens = list(rng.integers(0, 7, len(ids)))
    lens[0] = 33
    o_ids, o_len, o_seg = oracle.build_segments(ids, lens)
    T, NA, h_in, h_out, r = int(o_seg[-1]) + 5, 6, 256, 192, 16
    d = gpu_device
    g = torch.Generator(device="cpu").manual_seed(12)
    x = torch.randn(T, h_in, generator=g).to(dt).to(d)
    A = [(torch.randn(r, h_in, generator=g) / 16).to(dt).to(d) for _ in range(NA)]
    B = [(torch.randn(h_out, r, generator=g) / 4).to(dt).to(d) for _ in range(NA)]
    ta = torch.tensor([a.data_ptr() for a in A], dtype=torch.int64, device=d)
    tb = torch.tensor([b.data_ptr() for b in B], dtype=torch.int64, device=d)
    y0 = torch.randn(T, h_out, generator=g).to(dt).to(d)

    def run(seg_indptr, seg_adapter):
        plan = K.SegmentPlan(seg_indptr, seg_adapter, T)
        y = y0.clone()
        K.smlm_lora_forward(y, x, ta, tb, plan, r, beta=1.0)
        return y

    y_host = run(torch.tensor(o_seg, dtype=torch.int32, device=d), torch.tensor(o_ids, dtype=torch.int32, device=d))
    seg_adapter, _, seg_indptr, _ = K.segments_build(torch.tensor(ids, dtype=torch.int32, device=d),
                                                     torch.tensor(lens, dtype=torch.int32, device=d))
    y_dev = run(seg_indptr, seg_adapter)
    assert torch.equal(y_host, y_dev)
    assert torch.equal(y_dev[int(o_seg[-1]):], y0[int(o_seg[-1]):])  # rows past the last request untouched
    assert not torch.equal(y_dev[:33], y0[:33])


def test_layer_from_device_built_segments(K, oracle, gpu_device):
    """MixedLoraLinear (fused) driven by the device segment builder's padded arrays gives the
    bits it gives with the host loop's segments."""
    from loquetier_amd.kernel_utils import BatchLenInfo
    from loquetier_amd.mixed_lora import MixedLoraContext, MixedLoraLinear, NamedLoraLayer
    from loquetier_amd.segments import build_segments, build_segments_device
    d, tdt = gpu_device, torch.float16
    h_in, h_out, r, NA = 128, 192, 16, 3
    g = torch.Generator().manual_seed(13)
    req_ids, req_len = [1, 1, 0, 2, 2, 2, 1], [9, 1, 30, 1, 1, 1, 1]
    T = sum(req_len)
    base = torch.nn.Linear(h_in, h_out, bias=False, device=d, dtype=tdt)
    adapters = [NamedLoraLayer(f"a{i}", (torch.randn(r, h_in, generator=g) / 8).to(tdt).to(d),
                               (torch.randn(h_out, r, generator=g) / 4).to(tdt).to(d), torch.nn.Identity(), 2.0)
                for i in range(NA)]
    x = torch.randn(T, h_in, generator=g).to(tdt).to(d)
    blen = BatchLenInfo([], [40], 4, [], d)
    outs = []
    for on_device in (False, True):
        ctx = MixedLoraContext()
        layer = MixedLoraLinear(ctx, base, adapters, r, tdt, is_scaled=False, fused=True)
        if on_device:
            ids, lens, segment, _ = build_segments_device(torch.tensor(req_ids, dtype=torch.int32, device=d),
                                                          torch.tensor(req_len, dtype=torch.int32, device=d))
        else:
            ids, lens, segment = build_segments(req_ids, req_len, d)
        ctx.update(blen=blen, lora_ids=ids, lora_len=lens, segment=segment, train_idx=[])
        with torch.no_grad():
            outs.append(layer(x))
    assert torch.equal(outs[0], outs[1])
