"""The entry point that allocates nothing (smlm_gemm_static) against smlm_gemm, through the C
ABI: same kernels, scratch in the library's static device array instead of a caller's
workspace.  Results must be bit-identical; two calls in a row share the array, the second on
a smaller batch, so anything the first call left behind must not matter."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}


def _case(dev, dt, seed, T, S, NA, d_in, d_out):
    g = torch.Generator(device="cpu").manual_seed(seed)
    cuts = torch.sort(torch.randperm(T - 1, generator=g)[: S - 1] + 1).values.tolist() if S > 1 else []
    seg = [0] + cuts + [T]
    ids = torch.randint(0, NA, (S,), generator=g).tolist()
    x = torch.randn(T, d_in, generator=g).to(dev).to(dt)
    # w [d_out, d_in] per adapter: the layout the reference passes (is_row_major = False)
    W = [(torch.randn(d_out, d_in, generator=g) / d_in ** 0.5).to(dev).to(dt) for _ in range(NA)]
    y0 = torch.randn(T, d_out, generator=g).to(dev).to(dt)
    return dict(T=T, S=S, d_in=d_in, d_out=d_out, x=x, W=W, y0=y0,
                s=torch.tensor(seg, dtype=torch.int32, device=dev),
                w=torch.tensor([W[i].data_ptr() for i in ids], dtype=torch.int64, device=dev),
                scale=(torch.rand(S, generator=g) + 0.5).to(dev))


def _run(L, lib, c, static, code, stream):
    y = c["y0"].clone()
    common = (c["T"], c["S"], c["d_in"], c["d_out"], c["d_in"], 0, code, 1.0, c["scale"].data_ptr(), stream)
    if static:
        rc = L.smlm_gemm_static(y.data_ptr(), c["x"].data_ptr(), c["w"].data_ptr(), c["s"].data_ptr(), *common)
    else:
        need = lib.size_query("smlm_gemm_workspace_size", c["T"], c["S"], c["d_in"], c["d_out"])
        ws = torch.empty(need, dtype=torch.uint8, device=y.device)
        rc = L.smlm_gemm(y.data_ptr(), c["x"].data_ptr(), c["w"].data_ptr(), c["s"].data_ptr(),
                         ws.data_ptr(), ws.numel(), *common)
    assert rc == 0, lib.strerror(rc)
    return y


@pytest.mark.parametrize("dt", ["fp16", "bf16"])
@pytest.mark.parametrize("shapes", [
    # (T, S, NA, d_in, d_out) of the first call, then of the smaller second call
    ((1500, 40, 7, 2048, 16), (300, 9, 7, 2048, 16)),      # shrink with k split: partial sums in the scratch
    ((700, 700, 5, 4096, 32), (17, 17, 5, 4096, 32)),      # decode-style shrink, one row per segment
    ((1200, 33, 6, 32, 1024), (90, 4, 6, 32, 1024)),       # expand: only the plan lives in the scratch
], ids=["shrink-ksplit", "shrink-decode", "expand"])
def test_static_scratch_equals_workspace_call(gpu_device, dt, shapes):
    from loquetier_amd import _lib as lib
    L = lib.load()
    dev = gpu_device
    code = lib.SMLM_DTYPE_F16 if dt == "fp16" else lib.SMLM_DTYPE_BF16
    stream = torch.cuda.current_stream(dev).cuda_stream
    first, second = (_case(dev, TDT[dt], 70 + i, *sh) for i, sh in enumerate(shapes))
    want = [_run(L, lib, c, False, code, stream) for c in (first, second)]
    got = [_run(L, lib, c, True, code, stream) for c in (first, second)]   # two calls in a row
    torch.cuda.synchronize()
    for g_, w_, c in zip(got, want, (first, second)):
        assert torch.equal(g_, w_)
        assert not torch.equal(g_, c["y0"])      # something was computed
    # and once more in the other order: a larger batch after a smaller one
    again = _run(L, lib, first, True, code, stream)
    torch.cuda.synchronize()
    assert torch.equal(again, want[0])


def test_static_scratch_refuses_what_does_not_fit(gpu_device):
    from loquetier_amd import _lib as lib
    L = lib.load()
    dev = gpu_device
    T, S, d_in, d_out = 70000, 4, 4096, 64
    assert lib.size_query("smlm_gemm_workspace_size", T, S, d_in, d_out) > lib.SMLM_STATIC_SCRATCH_BYTES
    x = torch.zeros(8, dtype=torch.float16, device=dev)  # never read: the call returns before any launch
    rc = L.smlm_gemm_static(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), T, S, d_in, d_out, d_in, 0,
                            lib.SMLM_DTYPE_F16, 0.0, None, torch.cuda.current_stream(dev).cuda_stream)
    assert rc == lib.SMLM_ERR_SCRATCH and "scratch" in lib.strerror(rc)


def test_static_scratch_python_surface(gpu_device):
    """The wrapper with the reference's argument order (no tmp) against smlm_forward_cutlass."""
    from loquetier_amd.ops import _kernels as K
    dev = gpu_device
    c = _case(dev, torch.float16, 77, 260, 31, 4, 1024, 16)
    tmp = torch.empty(K.smlm_forward_cutlass_tmp_size(c["S"]), dtype=torch.uint8, device=dev)
    y1, y2 = torch.zeros_like(c["y0"]), torch.zeros_like(c["y0"])
    K.smlm_forward_cutlass(y1, c["x"], c["w"], c["s"], tmp, False)
    K.smlm_forward_cutlass_static(y2, c["x"], c["w"], c["s"], False)
    torch.cuda.synchronize()
    assert torch.equal(y1, y2) and bool(y1.abs().sum() > 0)
