"""CPU-only checks of the boundary and the host logic: the C-ABI library loads
and exports every symbol include/smlm.h declares, argument validation returns
the documented codes before any GPU work, and the Python mirrors of the
reference's host-side helpers agree with the oracle.  No kernel is launched.
"""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from loquetier_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from loquetier_amd.build import build_library
        build_library()
    return _lib


def test_every_declared_symbol_is_exported_and_bound(lib):
    header = open(os.path.join(ROOT, "include", "smlm.h")).read()
    declared = set(re.findall(r"SMLM_API\s+[\w\s\*]+?\b(smlm_\w+)\s*\(", header))
    assert len(declared) >= 15
    handle = ctypes.CDLL(lib.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), f"{name} is declared in smlm.h but not exported"
    assert declared == set(lib.SIGNATURES), "ctypes binding and header disagree"
    assert lib.load().smlm_abi_version() == 5


def test_missing_library_fails_loudly(lib, monkeypatch):
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "LIB_PATH", "/nonexistent/libsmlm_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        lib.load()


def test_size_queries(lib):
    assert lib.size_query("smlm_tmp_size", 0) == 0
    assert lib.size_query("smlm_tmp_size", 256) == 64 * 256
    small = lib.size_query("smlm_plan_size", 256, 256)
    big = lib.size_query("smlm_plan_size", 8192, 1075)
    assert 0 < small < big
    # the plan must hold a row and a segment index for every slot of every possible tile
    assert big >= (8192 // 16 + 1075 + 1) * 16 * 8
    assert lib.size_query("smlm_gemm_workspace_size", 4224, 132, 4096, 16) > \
        lib.size_query("smlm_plan_size", 4224, 132)
    assert lib.size_query("smlm_lora_fwd_workspace_size", 4224, 132, 4096, 4096, 16) >= 4224 * 16 * 4
    assert lib.size_query("smlm_lora_bwd_workspace_size", 4096, 4, 4, 4096, 4096, 16) > 0
    out = ctypes.c_size_t(0)
    assert lib.load().smlm_plan_size(-1, 4, ctypes.byref(out)) == -1
    assert lib.load().smlm_plan_size(16, 1 << 20, ctypes.byref(out)) == -6


def test_argument_validation_codes(lib):
    L = lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p = (p + 255) // 256 * 256  # 16-byte aligned fake "device" address; never dereferenced
    big = 1 << 30
    gemm = lambda **k: L.smlm_gemm(k.get("y", p), p, p, p, p, k.get("ws", big), k.get("T", 16), 2,
                                   k.get("d_in", 64), k.get("d_out", 8), k.get("ld", 64), 0,
                                   k.get("dtype", 0), 0.0, None, None)
    assert gemm(dtype=2) == -2                      # fp32 etc.: "No suitable kernel."
    assert lib.strerror(-2) == "No suitable kernel."
    assert gemm(d_in=60, ld=60) == -3               # not a multiple of 8
    assert gemm(y=p + 2) == -3                      # misaligned matrix
    assert gemm(y=None) == -1
    assert gemm(ws=128) == -4                       # workspace too small
    assert gemm(T=-1) == -1
    assert gemm(T=0) == 0                           # empty batch: nothing to do, no launch
    assert L.smlm_plan_build(p, big, p, None, 2, 16, 2, None) == -1   # key kind needs keys
    assert L.smlm_plan_build(p, big, p, p, 9, 16, 2, None) == -1      # unknown key kind
    assert L.smlm_plan_build(p, 64, p, None, 0, 16, 2, None) == -4
    assert L.smlm_lora_fwd(p, p, None, p, p, 2, p, p, big, 16, 2, 64, 64, 12, 0, 0.0, None, None) == -3
    assert L.smlm_lora_bwd(p, p, p, p, p, None, p, p, p, p, big, 16, 1, 1, 64, 64, 12, 1,
                           None, None) == -3        # rank not a multiple of 8
    # the entry point that carries its own scratch refuses batches beyond it before touching the device
    st = lambda T, d_in, d_out, dtype=0: L.smlm_gemm_static(p, p, p, p, T, 2, d_in, d_out, d_in, 0, dtype,
                                                             0.0, None, None)
    assert st(1 << 20, 4096, 64) == lib.SMLM_ERR_SCRATCH
    assert "scratch" in lib.strerror(lib.SMLM_ERR_SCRATCH)
    assert st(16, 64, 8, dtype=2) == -2
    assert st(0, 64, 8) == 0                         # empty batch
    need = lib.size_query("smlm_gemm_workspace_size", 4224, 132, 4096, 16)
    assert need <= lib.SMLM_STATIC_SCRATCH_BYTES     # the fine-tune + serve batch fits
    assert L.smlm_lora_bwd(p, p, p, p, p, None, p, p, p, p, 16, 16, 1, 1, 64, 64, 8, 1,
                           None, None) == -4


def test_plan_on_first_use_argument_validation(lib):
    """smlm_lora_opts.build_seg_indptr / build_seg_adapter: both or neither, and only with the shrink stage."""
    L = lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256  # aligned fake "device" address; never dereferenced
    VP, CI = ctypes.c_void_p * 1, ctypes.c_int * 1

    def call(opts, stages=3, T=16):
        return L.smlm_lora_fwd_multi_ex(1, VP(p), VP(p), None, VP(p), VP(p), 2, CI(64), CI(64), p, p, 1 << 30,
                                        T, 2, 16, 0, 0.0, None, stages, ctypes.byref(opts), None)
    o = lib.LoraOpts()
    o.build_seg_indptr = p
    assert call(o) == -1                  # the adapter ids are missing
    o.build_seg_adapter = p
    assert call(o, stages=2) == -1        # the plan is built with the shrink
    assert call(o, T=0) == 0              # empty batch: nothing to build, nothing launched
    assert ctypes.sizeof(lib.LoraOpts) == 64  # as the C struct: four pointers, three ints (one padded), two pointers
    # stage-by-stage calls: only a call that runs one stage may leave out the other stage's tensors
    full = lambda y, x, stages: L.smlm_lora_fwd_multi(1, VP(y), VP(x), None, VP(p), VP(p), 2, CI(64), CI(64), p, p,
                                                       1 << 30, 16, 2, 16, 0, 0.0, None, stages, None)
    assert full(None, p, 3) == -1 and full(p, None, 3) == -1
    assert full(p, None, 1) == -1                     # the shrink needs x


def test_rms_norm_argument_validation_codes(lib):
    L = lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256  # aligned fake "device" address; never dereferenced
    fwd = lambda **k: L.smlm_rms_norm_fwd(k.get("out", p), p, p, p, k.get("rows", 4), k.get("cols", 64), 1e-6,
                                          k.get("dtype", 0), None)
    assert fwd(dtype=2) == -2
    assert fwd(cols=60) == -3          # the reference refuses columns % 8 != 0 (rms_norm_cutlass.cu:166-168)
    assert fwd(cols=(1 << 24) + 8) == -6   # beyond what the kernels index
    assert fwd(out=None) == -1
    assert fwd(out=p + 2) == -3
    assert fwd(rows=0) == 0            # nothing to do, no launch
    assert fwd(rows=-1) == -1
    assert lib.size_query("smlm_rms_norm_bwd_workspace_size", 4096, 4096) >= 4096 * 4
    assert L.smlm_rms_norm_bwd(p, p, p, p, p, p, p, 16, 64, 4096, 0, None) == -4   # workspace too small
    assert L.smlm_rms_norm_bwd(p, p, p, p, p, p, None, 1 << 30, 64, 4096, 0, None) == -1


def test_python_surface_rejects_host_tensors(lib):
    from loquetier_amd.ops import _kernels as K
    y, x = torch.zeros(4, 8, dtype=torch.float16), torch.zeros(4, 16, dtype=torch.float16)
    w, s = torch.zeros(1, dtype=torch.int64), torch.tensor([0, 4], dtype=torch.int32)
    tmp = torch.zeros(K.smlm_forward_cutlass_tmp_size(1), dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        K.smlm_forward_cutlass(y, x, w, s, tmp, False)


def test_batch_len_info_mirror(oracle):
    from loquetier_amd.kernel_utils import BatchLenInfo
    cases = [([(2, 8), (1, 5)], [3, 4], 6, []), ([], [7], 2, []), ([(1, 1024)], [], 128, [(1, 4)]),
             ([], [], 5, [])]
    for trains, prefills, decode, evals in cases:
        b = BatchLenInfo(trains, prefills, decode, evals, torch.device("cpu"))
        tp, tlen, doff = oracle.batch_len_info(trains, prefills)
        assert list(b.train_partition) == (tp.tolist() if trains else [])
        assert b.tlen == tlen and b.doff == doff and b.decode == decode
        if prefills:
            assert b.indptr.dtype == torch.int32
            assert b.indptr.tolist() == np.concatenate([[0], np.cumsum(prefills)]).tolist()
        else:
            assert b.indptr is None
        if evals:
            assert list(b.eval_partition) == np.cumsum([tlen] + [e[0] * e[1] for e in evals]).tolist()


def test_build_segments_mirror(oracle):
    from loquetier_amd.segments import build_segments
    rng = np.random.default_rng(0)
    for _ in range(30):
        n = int(rng.integers(1, 40))
        ids = rng.integers(0, 5, n).tolist()
        lens = rng.integers(1, 20, n).tolist()
        lora_ids, lora_len, segment = build_segments(ids, lens, "cpu")
        o_ids, o_len, o_seg = oracle.build_segments(ids, lens)
        assert lora_ids == o_ids
        assert lora_len.dtype == torch.int32 and segment.dtype == torch.int32
        assert lora_len.tolist() == o_len.tolist() and segment.tolist() == o_seg.tolist()
    with pytest.raises(IndexError):
        build_segments([], [], "cpu")


def test_prepare_weight_mirror(oracle):
    from loquetier_amd.mixed_lora import prepare_weight
    rng = np.random.default_rng(1)
    w = rng.standard_normal((8, 32)).astype(np.float32)
    for dt, tdt in (("fp16", torch.float16), ("bf16", torch.bfloat16)):
        for scaling in (None, 2.0):
            got = prepare_weight(torch.from_numpy(w), 16, tdt, "cpu", 0, scaling).float().numpy()
            assert np.array_equal(got, oracle.prepare_weight(w, 0, 16, scaling, dt))
            got = prepare_weight(torch.from_numpy(w.T.copy()), 16, tdt, "cpu", 1, scaling).float().numpy()
            assert np.array_equal(got, oracle.prepare_weight(w.T.copy(), 1, 16, scaling, dt))
        same = prepare_weight(torch.from_numpy(w), 8, tdt, "cpu", 0, None)
        assert same.shape == (8, 32)


def test_segments_build_argument_validation_codes(lib):
    L = lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256  # fake "device" address; never dereferenced
    assert L.smlm_segments_build(p, p, -1, p, p, p, p, None) == -1
    assert L.smlm_segments_build(None, p, 4, p, p, p, p, None) == -1
    assert L.smlm_segments_build(p, p, 4, p, p, None, p, None) == -1
    assert L.smlm_segments_build(p, p, 4, p, p, p, None, None) == -1
    assert L.smlm_segments_build(p, p, (1 << 20) + 1, p, p, p, p, None) == -6   # beyond the plan's segment limit


def test_dropout_entry_points_validate_like_their_plain_forms(lib):
    L = lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256  # fake "device" address; never dereferenced
    big = 1 << 30
    VP, CI = ctypes.c_void_p * 1, ctypes.c_int * 1
    drop = lib.Dropout(p, -1, 1, 2, None)
    opts = lib.LoraOpts(ctypes.pointer(drop), None)
    fwd = lambda dr, **k: L.smlm_lora_fwd_multi_ex(
        1, VP(p), VP(p), None, VP(p), VP(p), 2, CI(64), CI(64), p, p, big, k.get("T", 16), 2, k.get("r", 16),
        k.get("dtype", 0), 0.0, None, 3, dr, None)
    assert fwd(ctypes.byref(opts)) == -1            # negative row count
    assert fwd(None, r=12) == -3 and fwd(None, dtype=2) == -2 and fwd(None, T=0) == 0
    bwd = lambda dr, **k: L.smlm_lora_bwd_ex(p, p, p, p, p, None, p, p, p, p, k.get("ws", big), 16, 1, 1, 64,
                                                  64, k.get("r", 8), 1, None, dr, None)
    assert bwd(ctypes.byref(opts)) == -1
    assert bwd(None, r=12) == -3 and bwd(None, ws=16) == -4


def test_layer_state_dict_saves_one_adapter_under_peft_names():
    """MixedLoraLinear._save_to_state_dict (reference mixed_lora.py:220-234): only the adapter chosen
    with set_saving_lora_id is saved, renamed lora-{idx}-A -> lora_A.weight."""
    import torch
    from loquetier_amd import mixed_lora as ml

    class Base(torch.nn.Module):  # a CPU stand-in: construction and state_dict launch no kernel
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.zeros(8, 16), requires_grad=False)

    adapters = [ml.NamedLoraLayer(f"a{i}", torch.full((8, 16), float(i)), torch.full((8, 8), 10.0 + i),
                                  torch.nn.Identity(), 2.0) for i in range(3)]
    layer = ml.MixedLoraLinear(ml.MixedLoraContext(), Base(), adapters, 8, torch.float32, is_scaled=False)
    layer.set_trainable([0, 2])
    assert sorted(n for n, _ in layer.named_parameters() if n.startswith("lora-")) == \
        ["lora-0-A", "lora-0-B", "lora-2-A", "lora-2-B"]
    sd = {k: v for k, v in layer.state_dict().items() if k.startswith("lora_")}
    assert sorted(sd) == ["lora_A.weight", "lora_B.weight"] and float(sd["lora_A.weight"][0, 0]) == 0.0
    with ml.set_saving_lora_id(2):
        sd2 = {k: v for k, v in layer.state_dict(prefix="m.").items() if "lora_" in k}
    assert sorted(sd2) == ["m.lora_A.weight", "m.lora_B.weight"]
    assert float(sd2["m.lora_A.weight"][0, 0]) == 2.0 and float(sd2["m.lora_B.weight"][0, 0]) == 12.0
    assert not sd2["m.lora_A.weight"].requires_grad          # detached unless keep_vars
    assert ml.CURRENT_TRAINER_LORA_ID == 0                   # restored on exit
    with ml.set_saving_lora_id(1):                           # adapter 1 does not train here: nothing saved
        assert not [k for k in layer.state_dict() if k.startswith("lora_")]
    # the parameters share the adapters' storage (mixed_lora.py:168-171): an optimizer step moves no address
    assert layer.get_parameter("lora-2-A").data_ptr() == adapters[2].wa.data_ptr()


def test_layer_adapter_list_management():
    """add_adapter / del_adapter / update_adapters (reference mixed_lora.py:106-166): the layer's own
    list is changed in place and the pointer and scale tables follow it."""
    import torch
    from loquetier_amd import mixed_lora as ml

    class Base(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.zeros(8, 16), requires_grad=False)

    def adapter(i, scale):
        return ml.NamedLoraLayer(f"a{i}", torch.full((8, 16), float(i)), torch.full((8, 8), 10.0 + i),
                                 torch.nn.Identity(), scale)
    held = [adapter(0, 2.0), adapter(1, 0.5)]
    layer = ml.MixedLoraLinear(ml.MixedLoraContext(), Base(), held, 8, torch.float32, is_scaled=False)
    assert layer.adapters is held and layer.wa_ptrs.tolist() == [a.wa.data_ptr() for a in held]
    layer.add_adapter(adapter(2, 4.0))
    assert layer.adapters is held and len(held) == 3
    assert layer.wa_ptrs.tolist() == [a.wa.data_ptr() for a in held]
    assert layer.wb_ptrs.tolist() == [a.wb.data_ptr() for a in held]
    assert layer.scaling.tolist() == [2.0, 0.5, 4.0]
    layer.del_adapter(0)
    assert layer.adapters is held and [a.adapter_name for a in held] == ["a1", "a2"]
    assert layer.wa_ptrs.tolist() == [a.wa.data_ptr() for a in held] and layer.scaling.tolist() == [0.5, 4.0]
    import pytest
    with pytest.raises(AssertionError):
        layer.del_adapter(5)
    scaled = ml.MixedLoraLinear(ml.MixedLoraContext(), Base(), [adapter(0, 2.0)], 8, torch.float32, is_scaled=True)
    assert scaled.scaling is None
    scaled.add_adapter(adapter(1, 3.0))
    assert scaled.scaling is None and scaled.wb_ptrs.numel() == 2


def _cpu_layer(ml, n_adapters=2, rank=8, fused=True):
    class Base(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.zeros(8, 16), requires_grad=False)
    ads = [ml.NamedLoraLayer(f"a{i}", torch.full((rank, 16), float(i)), torch.full((8, rank), 10.0 + i),
                             torch.nn.Identity(), 2.0) for i in range(n_adapters)]
    ctx = ml.MixedLoraContext()
    return ctx, ml.MixedLoraLinear(ctx, Base(), ads, rank, torch.float32, is_scaled=False, fused=fused)


def test_host_adapter_ids_must_index_the_layers_adapters():
    """A host list of adapter ids with an id at or past the number of adapters is refused before any
    launch (the kernels, which are also told the table length, would skip such segments); negative ids
    (segments no adapter serves) and ids that live on the device pass."""
    from loquetier_amd import mixed_lora as ml
    ctx, layer = _cpu_layer(ml, n_adapters=3)
    ctx.update(lora_ids=[0, 2, -1, 1])
    ctx.check_adapter_ids(3)
    with pytest.raises(IndexError, match="adapter id 2"):
        ctx.check_adapter_ids(2)
    ctx.update(lora_ids=[0, 3])
    with pytest.raises(IndexError):
        ctx.check_adapter_ids(len(layer.adapters))
    ctx.update(lora_ids=torch.tensor([0, 7], dtype=torch.int32))  # device-side ids: not read back
    ctx.check_adapter_ids(3)
    ctx.update(lora_ids=[])
    ctx.check_adapter_ids(1)


def test_projection_group_input_key():
    """The key a projection group recognises its input by: no version counter is read from inference
    tensors (they have none), a strided tensor is keyed by its own address and strides, and an in-place
    change of an ordinary tensor changes the key."""
    from loquetier_amd.mixed_lora import ProjectionGroup
    x = torch.zeros(6, 8)
    k0 = ProjectionGroup.input_key(x)
    assert k0 == ProjectionGroup.input_key(x)
    x.add_(1.0)
    assert ProjectionGroup.input_key(x) != k0
    with torch.inference_mode():
        y = torch.zeros(6, 8)
        ky = ProjectionGroup.input_key(y)     # would raise if it asked for y._version
        assert ky[1] is None and ky == ProjectionGroup.input_key(y)
    s1, s2 = x[:, ::2], x[:, 1::2]
    assert not s1.is_contiguous()
    assert ProjectionGroup.input_key(s1) == ProjectionGroup.input_key(x[:, ::2])
    assert ProjectionGroup.input_key(s1) != ProjectionGroup.input_key(s2)
    assert ProjectionGroup.input_key(s1) != ProjectionGroup.input_key(s1.contiguous())


def test_dropout_offsets_differ_between_contexts_and_can_be_restored():
    from loquetier_amd import mixed_lora as ml
    torch.manual_seed(1234)
    a, b = ml.MixedLoraContext(), ml.MixedLoraContext()
    oa, ob = [a.next_dropout_offset() for _ in range(3)], [b.next_dropout_offset() for _ in range(3)]
    assert oa[1] - oa[0] == 8 and oa[2] - oa[1] == 8          # eight projections' worth apart
    assert not set(range(oa[0], oa[2] + 8)) & set(range(ob[0], ob[2] + 8))  # two contexts: different streams
    torch.manual_seed(1234)                                    # a fresh context after re-seeding repeats the run
    c = ml.MixedLoraContext()
    assert [c.next_dropout_offset() for _ in range(3)] == oa
    state = a.dropout_state()
    nxt = a.next_dropout_offset()
    d = ml.MixedLoraContext()
    d.set_dropout_state(state)                                 # a resumed run continues the sequence
    assert d.next_dropout_offset() == nxt
    assert 0 <= nxt < 2 ** 63


def test_refused_adapter_set_leaves_the_layer_unchanged():
    """add_adapter with an adapter the layer cannot serve raises and changes neither the caller's list
    nor the layer's tables (an unfused layer cannot take an adapter stored below the layer's rank)."""
    from loquetier_amd import mixed_lora as ml
    ctx, layer = _cpu_layer(ml, n_adapters=2, rank=16, fused=False)
    held, ptrs = layer.adapters, layer.wa_ptrs.tolist()
    bad = ml.NamedLoraLayer("short", torch.zeros(8, 16), torch.zeros(8, 8), torch.nn.Identity(), 1.0)
    with pytest.raises(RuntimeError, match="fused path"):
        layer.add_adapter(bad)
    assert layer.adapters is held and len(held) == 2 and layer.wa_ptrs.tolist() == ptrs
    assert layer.scaling.numel() == 2 and layer.adapter_rank is None and not layer.packed
    # a fused layer takes no adapter whose A and B are stored at different ranks
    ctx2, fused = _cpu_layer(ml, n_adapters=2, rank=16, fused=True)
    odd = ml.NamedLoraLayer("odd", torch.zeros(8, 16), torch.zeros(8, 16), torch.nn.Identity(), 1.0)
    with pytest.raises(RuntimeError, match="packed storage"):
        fused.add_adapter(odd)
    assert len(fused.adapters) == 2 and fused.wa_ptrs.numel() == 2 and not fused.packed
    fused.add_adapter(bad)  # stored at its own rank beside padded ones: served (packed_ranks)
    assert len(fused.adapters) == 3 and fused.packed and fused.adapter_rank.tolist() == [16, 16, 8]


def test_checked_call_signature_compares_what_the_checks_look_at():
    """The record a checked operator call leaves behind (ops/_kernels._Checked): a later call takes the short way
    only with tensors of the same shapes, dtypes, devices and contiguity and the very same table objects."""
    from loquetier_amd.ops import _kernels as K
    x, y, tab_a, tab_b = torch.zeros(8, 16), torch.zeros(8, 32), torch.zeros(4, dtype=torch.int64), torch.zeros(4, dtype=torch.int64)
    hit = K._Checked()
    hit.descs = K._descs(([x], [y], ()))
    hit.same = (tab_a, tab_b, None)
    assert hit.matches(([torch.ones(8, 16)], [torch.ones(8, 32)], ()), (tab_a, tab_b, None))
    assert not hit.matches(([torch.ones(8, 16)], [torch.ones(8, 32)], ()), (tab_a.clone(), tab_b, None))   # another table
    assert not hit.matches(([torch.ones(9, 16)], [torch.ones(8, 32)], ()), (tab_a, tab_b, None))           # other rows
    assert not hit.matches(([torch.ones(8, 16).half()], [torch.ones(8, 32)], ()), (tab_a, tab_b, None))    # other dtype
    assert not hit.matches(([torch.ones(8, 32)[:, ::2]], [torch.ones(8, 32)], ()), (tab_a, tab_b, None))   # strided
    assert not hit.matches(([None], [torch.ones(8, 32)], ()), (tab_a, tab_b, None))                        # left out
    assert not hit.matches(([torch.ones(8, 16)], [torch.ones(8, 32)], [torch.ones(8, 4)]), (tab_a, tab_b, None))  # one more
    assert not hit.matches(([torch.ones(8, 16)], [torch.ones(8, 32)], ()), (tab_a, tab_b, tab_a))          # a rank table now
    assert K._mask([x, None, y]) == 0b101
