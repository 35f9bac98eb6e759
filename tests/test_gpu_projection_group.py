"""ProjectionGroup: layers that read one input (q/k/v, gate/up) share one shrink launch in a serving
step.  Grouping must never change a result: the grouped layers' outputs equal the ungrouped layers'
bit for bit, whatever order the members are called in and whatever else happens between their calls."""
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


def build(d, tdt, widths, h_in, r, NA, seed, true_ranks=None):
    """One context and, for every width, a pair of identical fused layers: [0] to be grouped, [1] left alone."""
    from loquetier_amd.mixed_lora import MixedLoraContext, MixedLoraLinear, NamedLoraLayer
    gen = torch.Generator().manual_seed(seed)
    ctx = MixedLoraContext()
    pairs = []
    for h_out in widths:
        base = torch.nn.Linear(h_in, h_out, bias=False, device=d, dtype=tdt)
        base.weight.data.copy_((torch.randn(h_out, h_in, generator=gen) / h_in ** 0.5).to(tdt))
        base.weight.requires_grad_(False)
        ads = []
        for a in range(NA):
            ra = r if true_ranks is None else true_ranks[a % len(true_ranks)]
            wa, wb = torch.zeros(r, h_in), torch.zeros(h_out, r)
            wa[:ra] = torch.randn(ra, h_in, generator=gen) / h_in ** 0.5
            wb[:, :ra] = torch.randn(h_out, ra, generator=gen) / ra ** 0.5
            ads.append(NamedLoraLayer(f"a{a}", wa.to(tdt).to(d), wb.to(tdt).to(d), torch.nn.Identity(), 0.5 + a,
                                      true_rank=None if true_ranks is None else ra))
        pairs.append([MixedLoraLinear(ctx, base, list(ads), r, tdt, is_scaled=False, fused=True) for _ in range(2)])
    return ctx, pairs


def serve_step(ctx, d, req_ids, req_len):
    from loquetier_amd.kernel_utils import BatchLenInfo
    from loquetier_amd.segments import build_segments
    lora_ids, lora_len, segment = build_segments(req_ids, req_len, d)
    n_dec = sum(1 for n in req_len if n == 1)
    blen = BatchLenInfo([], [n for n in req_len if n > 1], n_dec, [], d)
    ctx.update(blen=blen, lora_ids=lora_ids, lora_len=lora_len, segment=segment, train_idx=[])


@pytest.mark.parametrize("case", ["decode-qkv", "prefill-gate-up", "true-ranks"])
def test_grouped_layers_equal_ungrouped(K, gpu_device, case):
    from loquetier_amd.mixed_lora import ProjectionGroup
    d, tdt = gpu_device, torch.float16
    if case == "decode-qkv":
        h_in, widths, r, NA, ranks = 2048, [2048, 512, 512], 16, 6, None
        req_ids, req_len = [int(i) for i in np.random.default_rng(3).integers(0, 6, 70)], [1] * 70
    elif case == "prefill-gate-up":
        h_in, widths, r, NA, ranks = 1024, [2752, 2752], 32, 3, None
        req_ids, req_len = [0, 2, 1, 1, 0], [700, 500, 1, 1, 1]
    else:
        h_in, widths, r, NA, ranks = 2048, [256, 256, 128], 64, 4, [8, 16, 32, 64]
        req_ids, req_len = [3, 0, 1, 2, 2, 1], [40, 1, 1, 1, 30, 1]
    ctx, pairs = build(d, tdt, widths, h_in, r, NA, 5, ranks)
    group = ProjectionGroup([p[0] for p in pairs])
    T = sum(req_len)
    gen = torch.Generator().manual_seed(9)
    with torch.no_grad():
        for step in range(3):                     # several steps: the group's state must not leak across them
            serve_step(ctx, d, req_ids, req_len)
            x = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
            want = [p[1](x) for p in pairs]
            order = [(i + step) % len(pairs) for i in range(len(pairs))]   # any order of the members
            got = [None] * len(pairs)
            for i in order:
                got[i] = pairs[i][0](x)
            for a, b in zip(got, want):
                assert torch.equal(a, b)
    assert "open_group" not in ctx._step


def test_grouping_survives_misuse(K, gpu_device):
    """Members called with different tensors, twice, with the input changed in between, or interleaved
    with another group: every call still gives the ungrouped result."""
    from loquetier_amd.mixed_lora import ProjectionGroup
    d, tdt = gpu_device, torch.bfloat16
    h_in, r, NA = 2048, 16, 4
    ctx, pairs = build(d, tdt, [256, 256, 384, 384], h_in, r, NA, 6)
    g1 = ProjectionGroup([pairs[0][0], pairs[1][0]])
    g2 = ProjectionGroup([pairs[2][0], pairs[3][0]])
    req_ids, req_len = [1, 0, 3, 2, 1, 0, 0], [1, 1, 1, 1, 1, 1, 17]
    T = sum(req_len)
    gen = torch.Generator().manual_seed(10)
    x1 = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    x2 = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    with torch.no_grad():
        serve_step(ctx, d, req_ids, req_len)
        ref = lambda i, x: pairs[i][1](x)
        grp = lambda i, x: pairs[i][0](x)
        # a member of one group, then a member of the other, then the first group's second member
        a0, c0, b0 = grp(0, x1), grp(2, x1), grp(1, x1)
        assert torch.equal(a0, ref(0, x1)) and torch.equal(c0, ref(2, x1)) and torch.equal(b0, ref(1, x1))
        # different inputs within one group
        a1, b1 = grp(0, x1), grp(1, x2)
        assert torch.equal(a1, ref(0, x1)) and torch.equal(b1, ref(1, x2))
        # the same member twice
        d1, d2 = grp(3, x2), grp(3, x2)
        assert torch.equal(d1, ref(3, x2)) and torch.equal(d2, ref(3, x2))
        # the input modified in place between the members' calls
        a2 = grp(0, x1)
        want_a2 = ref(0, x1)
        x1.mul_(0.5)
        b2 = grp(1, x1)
        assert torch.equal(a2, want_a2) and torch.equal(b2, ref(1, x1))
        # an ordinary layer call between the members of a group (it uses the context's other workspace)
        a3, mid, b3 = grp(0, x2), ref(2, x2), grp(1, x2)
        assert torch.equal(a3, ref(0, x2)) and torch.equal(b3, ref(1, x2)) and torch.equal(mid, ref(2, x2))


def test_training_steps_are_not_grouped(K, gpu_device):
    """With training rows in the batch the grouped layers take the ordinary path (autograd, dropout)."""
    from loquetier_amd.kernel_utils import BatchLenInfo
    from loquetier_amd.mixed_lora import ProjectionGroup
    from loquetier_amd.segments import build_segments
    d, tdt = gpu_device, torch.bfloat16
    h_in, r, NA = 512, 16, 3
    ctx, pairs = build(d, tdt, [256, 256], h_in, r, NA, 7)
    ProjectionGroup([p[0] for p in pairs])
    for p in pairs:
        for l in p:
            l.set_trainable([1])
    req_ids, req_len = [1, 0, 2], [24, 1, 1]
    lora_ids, lora_len, segment = build_segments(req_ids, req_len, d)
    ctx.update(blen=BatchLenInfo([(1, 24)], [], 2, [], d), lora_ids=lora_ids, lora_len=lora_len, segment=segment,
               train_idx=[1])
    x = torch.randn(26, h_in, generator=torch.Generator().manual_seed(1)).to(tdt).to(d)
    outs = []
    for k in range(2):
        xs = x.clone().requires_grad_(True)
        y = pairs[0][k](xs) .float().sum() + pairs[1][k](xs).float().sum()
        y.backward()
        outs.append((xs.grad.clone(), pairs[0][k].get_parameter("lora-1-A").grad.clone()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    assert "open_group" not in ctx._step


def test_deferred_group_adds_everything_with_the_last_member(K, gpu_device):
    """deferred=True: a member's output lacks its LoRA term until the group's last member has been
    called; from then on every output equals the ungrouped layer's, bit for bit."""
    from loquetier_amd.mixed_lora import ProjectionGroup
    d, tdt = gpu_device, torch.float16
    h_in, widths, r, NA = 2048, [2048, 512, 512], 16, 6
    req_ids, req_len = [int(i) for i in np.random.default_rng(4).integers(0, NA, 90)], [1] * 90
    ctx, pairs = build(d, tdt, widths, h_in, r, NA, 8)
    ProjectionGroup([p[0] for p in pairs], deferred=True)
    gen = torch.Generator().manual_seed(12)
    with torch.no_grad():
        for step in range(3):
            serve_step(ctx, d, req_ids, req_len)
            x = torch.randn(sum(req_len), h_in, generator=gen).to(tdt).to(d)
            want = [p[1](x) for p in pairs]
            order = [(i + step) % 3 for i in range(3)]
            got = [None] * 3
            for n_called, i in enumerate(order):
                got[i] = pairs[i][0](x)
                if n_called < 2:   # still the base layer's output: the add is owed
                    assert torch.equal(got[i], pairs[i][0].base_layer(x))
                    assert not torch.equal(got[i], want[i])
            for a, b in zip(got, want):
                assert torch.equal(a, b)
            assert "open_group" not in ctx._step


def test_deferred_group_cut_short(K, gpu_device):
    """A deferred pass that never sees its last member pays what it owes when the next pass or the
    next step starts; a member whose output tensor is not the one handed out is expanded at once."""
    from loquetier_amd.mixed_lora import ProjectionGroup
    d, tdt = gpu_device, torch.bfloat16
    h_in, r, NA = 2048, 16, 4
    ctx, pairs = build(d, tdt, [256, 256, 384], h_in, r, NA, 9)
    ProjectionGroup([p[0] for p in pairs], deferred=True)
    req_ids, req_len = [1, 0, 3, 2, 1, 0, 0], [1, 1, 1, 1, 1, 1, 17]
    T = sum(req_len)
    gen = torch.Generator().manual_seed(13)
    x1 = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    x2 = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    with torch.no_grad():
        serve_step(ctx, d, req_ids, req_len)
        want1 = [p[1](x1) for p in pairs]
        want2 = [p[1](x2) for p in pairs]
        a, b = pairs[0][0](x1), pairs[1][0](x1)       # two of three members ...
        c = pairs[0][0](x2)                           # ... then another input: the first pass is settled
        assert torch.equal(a, want1[0]) and torch.equal(b, want1[1])
        assert not torch.equal(c, want2[0])
        serve_step(ctx, d, req_ids, req_len)          # the next step settles the second pass
        assert torch.equal(c, want2[0])
        assert "open_group" not in ctx._step
        # a base layer that answers in float32: the layer hands out a converted copy, so its term is added at once
        pairs[2][0].base_layer.float()
        pairs[2][1].base_layer.float()
        xf = x1.float()
        want_c = pairs[2][1](xf)
        got_c = pairs[2][0](xf)
        assert got_c.dtype == torch.float32 and torch.equal(got_c, want_c)


@pytest.mark.parametrize("deferred", [False, True])
def test_grouped_layers_under_graph_capture(K, gpu_device, deferred):
    """A serving step of grouped layers captured once and replayed with new inputs: every replay gives
    what ungrouped layers give eagerly (the group's bookkeeping is host-side and done at capture time)."""
    from loquetier_amd.mixed_lora import ProjectionGroup
    d, tdt = gpu_device, torch.float16
    h_in, widths, r, NA = 2048, [1024, 256, 256], 16, 5
    req_ids, req_len = [int(i) for i in np.random.default_rng(6).integers(0, NA, 48)], [1] * 48
    T = sum(req_len)
    ctx, pairs = build(d, tdt, widths, h_in, r, NA, 14)
    ProjectionGroup([p[0] for p in pairs], deferred=deferred)
    gen = torch.Generator().manual_seed(15)
    x = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
    outs = [torch.empty(T, w, dtype=tdt, device=d) for w in widths]
    cap = torch.cuda.Stream()
    from loquetier_amd.kernel_utils import BatchLenInfo
    from loquetier_amd.segments import build_segments
    lora_ids, lora_len, segment = build_segments(req_ids, req_len, d)   # staged on the device before the capture
    lora_ids = torch.tensor(lora_ids, dtype=torch.int32, device=d) if not isinstance(lora_ids, torch.Tensor) else lora_ids
    blen = BatchLenInfo([], [], T, [], d)

    def update():
        ctx.update(blen=blen, lora_ids=lora_ids, lora_len=lora_len, segment=segment, train_idx=[])

    def step():
        update()
        got = [p[0](x) for p in pairs]   # (a deferred group's outputs are complete after the last member's call)
        for o, t in zip(outs, got):
            o.copy_(t)
    with torch.no_grad():
        with torch.cuda.stream(cap):
            step()                             # eager once: sizes the workspaces outside the capture
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=cap):
            step()
        for rep in range(3):
            x.copy_(torch.randn(T, h_in, generator=gen).to(tdt))
            g.replay()
            torch.cuda.synchronize()
            serve_step(ctx, d, req_ids, req_len)
            want = [p[1](x) for p in pairs]
            for a, b in zip(outs, want):
                assert torch.equal(a, b)


def test_group_under_inference_mode_and_with_a_strided_input(K, gpu_device, monkeypatch):
    """A serving loop under torch.inference_mode (tensors without a version counter) and an input that is a
    strided view (the layer works on a contiguous copy): the members still share ONE shrink launch and
    the results equal the ungrouped layers'."""
    from loquetier_amd import mixed_lora as ml
    d, tdt = gpu_device, torch.float16
    h_in, r, NA = 2048, 16, 4
    ctx, pairs = build(d, tdt, [256, 512, 256], h_in, r, NA, 8)
    ml.ProjectionGroup([p[0] for p in pairs])
    req_ids, req_len = [1, 0, 3, 2, 1, 0, 0], [1, 1, 1, 1, 1, 1, 9]
    T = sum(req_len)
    shrinks = []
    real = ml.kernel.smlm_lora_forward_multi

    def counting(*a, **kw):
        if kw.get("stages") == 1:
            shrinks.append(1)
        return real(*a, **kw)
    monkeypatch.setattr(ml.kernel, "smlm_lora_forward_multi", counting)
    gen = torch.Generator().manual_seed(12)
    with torch.inference_mode():
        serve_step(ctx, d, req_ids, req_len)
        x = torch.randn(T, h_in, generator=gen).to(tdt).to(d)
        got = [p[0](x) for p in pairs]
        assert len(shrinks) == 1
        for g_, p in zip(got, pairs):
            assert torch.equal(g_, p[1](x))
        # a strided view: every member is handed the same view object, each makes its own contiguous copy
        wide = torch.randn(T, 2 * h_in, generator=gen).to(tdt).to(d)
        view = wide[:, ::2]
        assert not view.is_contiguous()
        del shrinks[:]
        got = [p[0](view) for p in pairs]
        assert len(shrinks) == 1
        for g_, p in zip(got, pairs):
            assert torch.equal(g_, p[1](view.contiguous()))
    # and outside inference mode, with no_grad, a strided view of an ordinary tensor
    with torch.no_grad():
        serve_step(ctx, d, req_ids, req_len)
        wide = torch.randn(T, 2 * h_in, generator=gen).to(tdt).to(d)
        del shrinks[:]
        got = [p[0](wide[:, 1::2]) for p in pairs]     # equal views made anew for every call
        assert len(shrinks) == 1
        for g_, p in zip(got, pairs):
            assert torch.equal(g_, p[1](wide[:, 1::2].contiguous()))
