"""Python surface of the HIP library, with the names and argument order of the
reference's pybind module `loquetier.ops._kernels`
(kernel_src/csrc/loquetier_ops.cc:365-374) for the SMLM entries, plus the
fused forward, the backward and the plan builder this build adds.

Tensors are torch tensors on a ROCm device; the calls are asynchronous on
torch's current stream of that device.  Nothing here computes on the host.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Optional, Tuple

import torch

from .. import _lib

_DTYPE_CODE = {torch.float16: _lib.SMLM_DTYPE_F16, torch.bfloat16: _lib.SMLM_DTYPE_BF16}

class Workspace:
    """Scratch memory for the kernels (k-split partial sums, the rounded v, transposed weights).

    The C ABI allocates nothing: every call is handed a buffer at least as large as its
    `*_workspace_size` query says.  A Workspace owns such a buffer.  It only ever grows, a
    buffer that was handed out is never freed while the Workspace lives (a captured HIP graph
    keeps the raw address of the buffer it was captured with), and it refuses to grow while
    its stream is being captured: size it first, with `reserve` or with one eager pass.
    Calls that share a Workspace must be ordered on one stream."""

    def __init__(self, device: torch.device, nbytes: int = 0):
        self.device = torch.device(device)
        self._buf: Optional[torch.Tensor] = None
        self._retired = []
        if nbytes:
            self.reserve(nbytes)

    def reserve(self, nbytes: int) -> torch.Tensor:
        if self._buf is None or self._buf.numel() < nbytes:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError(
                    f"the workspace must grow to {nbytes} bytes during a graph capture: reserve it "
                    "before capturing (Workspace.reserve, or one eager pass of the same calls)")
            if self._buf is not None:
                self._retired.append(self._buf)
            self._buf = torch.empty(max(nbytes, 1 << 20) * 3 // 2, dtype=torch.uint8, device=self.device)
        return self._buf


# default workspaces, one per (device index, stream handle): calls on one stream are ordered,
# so they can share one buffer.  Callers that want to own the memory pass `workspace=`.
_WORKSPACES: Dict[Tuple[int, int], Workspace] = {}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(dev: torch.device) -> int:
    # (the handle itself where torch hands it out: building a torch.cuda.Stream object around it costs
    # microseconds per call)
    if _raw_stream is None:
        return torch.cuda.current_stream(dev).cuda_stream
    return _raw_stream(dev.index if dev.index is not None else torch.cuda.current_device())


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on(dev: torch.device):
    """Context that makes `dev` the current device; nothing to do (and nothing spent) when it already is."""
    if dev.index is None or dev.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(dev)


def _workspace(dev: torch.device, nbytes: int, own: Optional[Workspace] = None) -> torch.Tensor:
    if own is not None:
        buf = own.reserve(nbytes)
        if buf.device != dev:
            raise RuntimeError(f"workspace lives on {buf.device}, the tensors on {dev}")
        return buf
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), _stream(dev))
    ws = _WORKSPACES.get(key)
    if ws is None:
        ws = _WORKSPACES[key] = Workspace(dev)
    return ws.reserve(nbytes)


def _check_input(t: torch.Tensor, name: str) -> None:
    # CHECK_INPUT of kernel_src/csrc/loquetier_ops.cc:32-38
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _check_dim(d: int, t: torch.Tensor, name: str) -> None:
    if t.dim() != d:
        raise RuntimeError(f"{name} must be a {d}D tensor")


def _dtype_code(t: torch.Tensor) -> int:
    code = _DTYPE_CODE.get(t.dtype)
    if code is None:
        raise RuntimeError(f"No suitable kernel. dtype={t.dtype}")
    return code


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def smlm_forward_cutlass_tmp_size(num_problems: int) -> int:
    """Bytes of the `tmp` tensor `smlm_forward_cutlass` expects
    (reference: smlm_forward_tmp_size, smlm_forward_cutlass.cuh:48-52)."""
    return _lib.size_query("smlm_tmp_size", int(num_problems))


def smlm_forward_cutlass_workspace_size(T: int, num_problems: int, d_in: int, d_out: int) -> int:
    """Bytes of a `tmp` that smlm_forward_cutlass uses as its ONLY scratch (plan and k-split partial sums of a
    [T, d_in] x [d_in, d_out] batch of num_problems segments): a caller that passes a tmp of at least this size
    owns every byte the call touches.  No counterpart in the reference, whose 60 bytes a problem hold all it needs."""
    return _lib.size_query("smlm_gemm_workspace_size", int(T), int(num_problems), int(d_in), int(d_out))


def smlm_forward_cutlass(y: torch.Tensor, x: torch.Tensor, w_ptr: torch.Tensor, s: torch.Tensor,
                         tmp: torch.Tensor, is_row_major: bool) -> None:
    """Grouped GEMM y[s_i:s_{i+1}] = x[s_i:s_{i+1}] @ W_i, overwriting y.

    Same contract as dispatch_smlm_forward_cutlass
    (kernel_src/csrc/loquetier_ops.cc:277-319): y [T,d_out], x [T,d_in] fp16 or
    bf16, w_ptr int64 [S] device addresses, s int32 [S+1], tmp uint8 of exactly
    smlm_forward_cutlass_tmp_size(S) bytes.  Unlike the reference it does not
    block the host.  The kernels here need more scratch than that tmp holds: with a tmp of the
    reference's size it comes from a buffer this module keeps per (device, stream); a tmp of
    smlm_forward_cutlass_workspace_size(T, S, d_in, d_out) bytes or more (16-byte aligned) is
    used itself, and the call then touches no memory the caller did not hand it.
    """
    for t, n in ((y, "y"), (x, "x"), (w_ptr, "w_ptr"), (s, "s"), (tmp, "tmp")):
        _check_input(t, n)
    _check_dim(2, y, "y")
    _check_dim(2, x, "x")
    _check_dim(1, w_ptr, "w_ptr")
    _check_dim(1, s, "s")
    _check_dim(1, tmp, "tmp")
    num_problems = s.size(0) - 1
    d_in, d_out = x.size(1), y.size(1)
    w_ld = d_out if is_row_major else d_in
    if w_ptr.dtype != torch.int64 or s.dtype != torch.int32:
        raise RuntimeError("w_ptr must be int64 and s must be int32")
    if w_ptr.size(0) != num_problems or y.size(0) != x.size(0) or y.dtype != x.dtype:
        raise RuntimeError("inconsistent shapes: w_ptr [S], s [S+1], x [T,d_in], y [T,d_out]")
    code = _dtype_code(x)
    T = x.size(0)
    dev = tmp.device
    with _on(dev):
        need = _lib.size_query("smlm_gemm_workspace_size", T, num_problems, d_in, d_out)
        own = tmp.size(0) >= need and tmp.size(0) != smlm_forward_cutlass_tmp_size(num_problems)
        if not own and tmp.size(0) != smlm_forward_cutlass_tmp_size(num_problems):
            raise RuntimeError(f"CHECK_EQ(tmp.size(0), smlm_forward_tmp_size(num_problems)) failed: "
                               f"{tmp.size(0)} vs {smlm_forward_cutlass_tmp_size(num_problems)}")
        if own and tmp.data_ptr() % 16:
            raise RuntimeError("a tmp that serves as the workspace must be 16-byte aligned")
        ws = tmp if own else _workspace(dev, need)
        rc = _lib.load().smlm_gemm(y.data_ptr(), x.data_ptr(), w_ptr.data_ptr(), s.data_ptr(),
                                   ws.data_ptr(), ws.numel(), T, num_problems, d_in, d_out, w_ld,
                                   int(bool(is_row_major)), code, 0.0, None, _stream(dev))
    if rc == _lib.SMLM_ERR_DTYPE:
        raise RuntimeError(f"No suitable kernel. dtype={x.dtype}")
    _lib.check(rc, "smlm_forward_cutlass")


def smlm_forward_cutlass_static(y: torch.Tensor, x: torch.Tensor, w_ptr: torch.Tensor, s: torch.Tensor,
                                is_row_major: bool, beta: float = 0.0,
                                seg_scale: Optional[torch.Tensor] = None) -> None:
    """smlm_forward_cutlass without `tmp` and without any allocation (smlm_gemm_static): the
    scratch is an array inside the library, SMLM_STATIC_SCRATCH_BYTES per GPU, shared by all
    calls on that GPU -- keep them on one stream.  Raises when the batch needs more."""
    for t, n in ((y, "y"), (x, "x"), (w_ptr, "w_ptr"), (s, "s")):
        _check_input(t, n)
    _check_dim(2, y, "y")
    _check_dim(2, x, "x")
    _check_dim(1, w_ptr, "w_ptr")
    _check_dim(1, s, "s")
    num_problems = s.size(0) - 1
    if w_ptr.dtype != torch.int64 or s.dtype != torch.int32:
        raise RuntimeError("w_ptr must be int64 and s must be int32")
    if w_ptr.size(0) != num_problems or y.size(0) != x.size(0) or y.dtype != x.dtype:
        raise RuntimeError("inconsistent shapes: w_ptr [S], s [S+1], x [T,d_in], y [T,d_out]")
    if seg_scale is not None and (seg_scale.dtype != torch.float32 or seg_scale.numel() != num_problems
                                  or not seg_scale.is_cuda):
        raise RuntimeError("seg_scale must be a device float32 tensor with one entry per segment")
    code = _dtype_code(x)
    d_in, d_out = x.size(1), y.size(1)
    dev = x.device
    with _on(dev):
        rc = _lib.load().smlm_gemm_static(y.data_ptr(), x.data_ptr(), w_ptr.data_ptr(), s.data_ptr(),
                                          x.size(0), num_problems, d_in, d_out,
                                          d_out if is_row_major else d_in, int(bool(is_row_major)), code,
                                          float(beta), _ptr(seg_scale), _stream(dev))
    _lib.check(rc, "smlm_forward_cutlass_static")


class SegmentPlan:
    """Tile plan of one flat batch: built once from (segment, adapter ids) and
    shared by every LoRA linear of the step (the reference rebuilds its
    per-problem table inside every kernel call,
    smlm_forward_cutlass.cuh:76-79).

    seg_key: None (every segment its own group), int32 adapter ids, int64 weight addresses, or a
    PAIR of int64 address tensors (wa_ptr, wb_ptr) as the reference's add_lora.forward is handed
    them (kernel_utils.py:115-119): segments are then grouped where both addresses agree, and one
    plan serves both GEMMs of the fused forward (per-segment tables).

    defer=True (plans keyed by int32 adapter ids or by a pair of address tensors): nothing is
    launched here; the first smlm_lora_forward(_multi) or smlm_lora_backward call that gets the
    plan builds it -- for batches of few enough segments inside its first launch, at no launch of
    its own -- and every other user builds it with the plan launch first (ensure_built)."""

    def __init__(self, segment: torch.Tensor, seg_key: Optional[torch.Tensor], T: int,
                 buf: Optional[torch.Tensor] = None, defer: bool = False):
        _check_input(segment, "segment")
        if segment.dtype != torch.int32 or segment.dim() != 1:
            raise RuntimeError("segment must be a 1D int32 tensor")
        self.segment = segment
        self.S = segment.size(0) - 1
        self.T = int(T)
        self.seg_key2 = None
        if isinstance(seg_key, (tuple, list)):
            if len(seg_key) != 2 or any(k.dtype != torch.int64 for k in seg_key):
                raise RuntimeError("a pair key is two int64 tensors of weight addresses")
            seg_key, self.seg_key2 = seg_key
        self.seg_key = seg_key
        if seg_key is None:
            kind = _lib.SMLM_KEY_NONE
        elif self.seg_key2 is not None:
            kind = _lib.SMLM_KEY_PTR2
        elif seg_key.dtype == torch.int32:
            kind = _lib.SMLM_KEY_I32
        elif seg_key.dtype == torch.int64:
            kind = _lib.SMLM_KEY_PTR
        else:
            raise RuntimeError("seg_key must be int32 adapter ids or int64 addresses")
        for key in (seg_key, self.seg_key2):
            if key is not None:
                _check_input(key, "seg_key")
                if key.dim() != 1 or key.size(0) != self.S:
                    raise RuntimeError("seg_key must have one entry per segment")
        self.kind = kind
        dev = segment.device
        nbytes = _lib.size_query("smlm_plan_size", self.T, self.S)
        if buf is None:
            buf = torch.empty(max(nbytes, 64), dtype=torch.uint8, device=dev)
        elif buf.dtype != torch.uint8 or buf.numel() < nbytes or buf.device != dev:
            raise RuntimeError(f"plan buffer must be a uint8 tensor of >= {nbytes} bytes on {dev}")
        self.buf = buf
        self.built = False
        if not (defer and kind in (_lib.SMLM_KEY_I32, _lib.SMLM_KEY_PTR2)):
            self.ensure_built()

    def ensure_built(self) -> None:
        if self.built:
            return
        dev = self.segment.device
        with _on(dev):
            if self.kind == _lib.SMLM_KEY_PTR2:
                rc = _lib.load().smlm_plan_build2(self.buf.data_ptr(), self.buf.numel(), self.segment.data_ptr(),
                                                  self.seg_key.data_ptr(), self.seg_key2.data_ptr(), self.T,
                                                  self.S, _stream(dev))
            else:
                rc = _lib.load().smlm_plan_build(self.buf.data_ptr(), self.buf.numel(), self.segment.data_ptr(),
                                                 _ptr(self.seg_key), self.kind, self.T, self.S, _stream(dev))
        _lib.check(rc, "smlm_plan_build")
        self.built = True

    @staticmethod
    def nbytes(T: int, S: int) -> int:
        return _lib.size_query("smlm_plan_size", int(T), int(S))

    def header(self) -> Tuple[int, int, int, int]:
        """(n_tiles, n_groups, rows covered, key kind used) -- synchronises; for tests."""
        self.ensure_built()
        h = self.buf[:16].view(torch.int32).cpu()
        return int(h[0]), int(h[1]), int(h[2]), int(h[3])


def _check_table(t: torch.Tensor, plan: SegmentPlan, name: str) -> None:
    _check_input(t, name)
    if t.dtype != torch.int64 or t.dim() != 1:
        raise RuntimeError(f"{name} must be a 1D int64 tensor of device addresses")
    if plan.kind != _lib.SMLM_KEY_I32 and t.size(0) != plan.S:
        raise RuntimeError(f"{name} needs one entry per segment unless the plan is keyed by adapter id")


def _check_scale(seg_scale: Optional[torch.Tensor], plan: SegmentPlan) -> None:
    if seg_scale is not None and (seg_scale.dtype != torch.float32 or seg_scale.dim() != 1
                                  or seg_scale.size(0) != plan.S or not seg_scale.is_cuda):
        raise RuntimeError("seg_scale must be a device float32 tensor with one entry per segment")


def smlm_gemm_planned(y: torch.Tensor, x: torch.Tensor, w_ptrs: torch.Tensor, plan: SegmentPlan,
                      is_row_major: bool = False, seg_scale: Optional[torch.Tensor] = None,
                      beta: float = 0.0, workspace: Optional[Workspace] = None) -> None:
    """Grouped GEMM over a prebuilt plan: y[seg] = beta*y[seg] + scale*x[seg] @ W_seg.
    w_ptrs is indexed by adapter id when the plan was built from int32 adapter ids,
    by segment otherwise."""
    for t, n in ((y, "y"), (x, "x")):
        _check_input(t, n)
    _check_dim(2, y, "y")
    _check_dim(2, x, "x")
    _check_table(w_ptrs, plan, "w_ptrs")
    _check_scale(seg_scale, plan)
    plan.ensure_built()
    if y.dtype != x.dtype or y.size(0) != x.size(0) or x.size(0) != plan.T:
        raise RuntimeError("x [T,d_in] and y [T,d_out] must share dtype and T with the plan")
    code = _dtype_code(x)
    T, d_in, d_out = x.size(0), x.size(1), y.size(1)
    w_ld = d_out if is_row_major else d_in
    dev = x.device
    with _on(dev):
        need = _lib.size_query("smlm_gemm_planned_workspace_size", T, d_in, d_out)
        ws = _workspace(dev, need, workspace)
        rc = _lib.load().smlm_gemm_planned(y.data_ptr(), x.data_ptr(), w_ptrs.data_ptr(), w_ptrs.size(0),
                                           plan.buf.data_ptr(), ws.data_ptr(), ws.numel(), T, plan.S,
                                           d_in, d_out, w_ld, int(bool(is_row_major)), code,
                                           float(beta), _ptr(seg_scale), _stream(dev))
    _lib.check(rc, "smlm_gemm_planned")


class DropoutSpec:
    """Dropout of the training rows of x inside the operator (struct smlm_dropout):
    seg_p float32 [S] on the device, the dropout probability of each segment's
    adapter; rows = number of training rows (they come first in the batch);
    (seed, offset) name the mask stream -- the backward of a layer must be given
    the pair its forward used.  Replaces the nn.Dropout calls and the torch.cat of
    MixedLoraLinear.forward (src/loquetier_src/models/mixed_lora.py:185-192)."""

    def __init__(self, seg_p: torch.Tensor, rows: int, seed: int, offset: int,
                 mask_bits: Optional[torch.Tensor] = None):
        _check_input(seg_p, "seg_p")
        if seg_p.dtype != torch.float32 or seg_p.dim() != 1:
            raise RuntimeError("seg_p must be a 1D float32 tensor")
        if rows < 0:
            raise RuntimeError("rows must not be negative")
        if mask_bits is not None:
            _check_input(mask_bits, "mask_bits")
            if mask_bits.dtype != torch.uint8:
                raise RuntimeError("mask_bits must be a uint8 tensor")
        self.seg_p, self.rows = seg_p, int(rows)
        self.seed, self.offset = int(seed) & (2 ** 64 - 1), int(offset) & (2 ** 64 - 1)
        self.mask_bits = mask_bits

    @staticmethod
    def mask_nbytes(rows: int, h_in) -> int:
        """Size of mask_bits for `rows` training rows; h_in: one width or one per projection."""
        widths = [h_in] if isinstance(h_in, int) else list(h_in)
        return sum(int(rows) * (int(h) // 8) for h in widths)

    def with_offset(self, offset: int) -> "DropoutSpec":
        return DropoutSpec(self.seg_p, self.rows, self.seed, offset, self.mask_bits)

    def struct(self, plan: "SegmentPlan", widths):
        if self.seg_p.size(0) != plan.S or self.seg_p.device != plan.segment.device:
            raise RuntimeError("seg_p must have one entry per segment of the plan, on its device")
        if self.mask_bits is not None and self.mask_bits.numel() < self.mask_nbytes(self.rows, widths):
            raise RuntimeError(f"mask_bits needs {self.mask_nbytes(self.rows, widths)} bytes")
        return _lib.Dropout(self.seg_p.data_ptr(), self.rows, self.seed, self.offset, _ptr(self.mask_bits))


def _opts(plan: SegmentPlan, dropout: Optional["DropoutSpec"], widths, adapter_rank: Optional[torch.Tensor],
          n_weights: int, packed_ranks: bool = False, checked: bool = False):
    """struct smlm_lora_opts for a call (None when there is nothing to say).  The returned
    object keeps the dropout struct alive.  checked: the arguments were looked at by an earlier call."""
    if packed_ranks and adapter_rank is None:
        raise RuntimeError("packed_ranks needs adapter_rank: the kernels must know each adapter's stored rank")
    if dropout is None and adapter_rank is None:
        return None
    if adapter_rank is not None and not checked:
        _check_input(adapter_rank, "adapter_rank")
        if adapter_rank.dtype != torch.int32 or adapter_rank.dim() != 1 or adapter_rank.size(0) < n_weights:
            raise RuntimeError("adapter_rank must be a 1D int32 tensor with one entry per weight table entry")
    opts = _lib.LoraOpts()
    if dropout is not None:
        opts._drop = dropout.struct(plan, widths)
        opts.dropout = C.pointer(opts._drop)
    opts.adapter_rank = _ptr(adapter_rank)
    opts.packed_ranks = int(bool(packed_ranks))
    return opts


def smlm_lora_forward(y: torch.Tensor, x: torch.Tensor, a_ptrs: torch.Tensor, b_ptrs: torch.Tensor,
                      plan: SegmentPlan, rank: int, seg_scale: Optional[torch.Tensor] = None,
                      beta: float = 0.0, v_out: Optional[torch.Tensor] = None,
                      dropout: Optional[DropoutSpec] = None,
                      adapter_rank: Optional[torch.Tensor] = None,
                      workspace: Optional[Workspace] = None, packed_ranks: bool = False,
                      cache: Optional[dict] = None) -> None:
    """y = beta*y + seg_scale * round(x A^T) B^T in one stream-ordered call (two launches).
    a_ptrs / b_ptrs are indexed by adapter id when the plan was built from int32
    adapter ids, by segment otherwise.  cache: see smlm_lora_forward_multi."""
    smlm_lora_forward_multi([y], [x], [a_ptrs], [b_ptrs], plan, rank, seg_scale=seg_scale, beta=beta,
                            v_out=None if v_out is None else [v_out], dropout=dropout,
                            adapter_rank=adapter_rank, workspace=workspace, packed_ranks=packed_ranks,
                            cache=cache)


_FWD_MULTI_SIZES: Dict[Tuple, int] = {}


class _Checked:
    """What a checked call leaves behind for the next call from the same place: what its tensors looked
    like (a later call is compared with that, cheaply) and the argument blocks that do not change."""
    __slots__ = ("descs", "same", "code", "dev", "arrs", "h_in", "h_out", "a_arr", "b_arr", "n_weights", "need",
                 "opts")

    def matches(self, tensor_lists, objects) -> bool:
        """tensor_lists: the call's data tensors, list by list; objects: the tables and other tensors that are
        expected to be the very objects of the checked call."""
        for o, mine in zip(objects, self.same):
            if o is not mine:
                return False
        k = 0
        descs = self.descs
        for ts in tensor_lists:
            for t in ts:
                if k == len(descs):
                    return False
                d = descs[k]
                k += 1
                if t is None:
                    if d is not None:
                        return False
                elif d is None or t.shape != d[0] or t.dtype != d[1] or t.device != d[2] or not t.is_contiguous():
                    return False
        return k == len(descs)


def _descs(tensor_lists):
    return [None if t is None else (t.shape, t.dtype, t.device) for ts in tensor_lists for t in ts]


def _mask(ts) -> int:
    m = 0
    for i, t in enumerate(ts):
        if t is not None:
            m |= 1 << i
    return m


def _fill(arr, ts):
    for i, t in enumerate(ts):
        arr[i] = None if t is None else t.data_ptr()
    return arr


def _remember(cache: dict, key, hit: "_Checked") -> None:
    if len(cache) >= 32:
        cache.clear()
    cache[key] = hit


def _fwd_multi_workspace_size(T: int, widths_in: Tuple[int, ...], rank: int) -> int:
    key = (T, widths_in, rank)
    n = _FWD_MULTI_SIZES.get(key)
    if n is None:
        need = C.c_size_t(0)
        arr = (C.c_int * len(widths_in))(*widths_in)
        _lib.check(_lib.load().smlm_lora_fwd_multi_workspace_size(len(widths_in), T, arr, rank, C.byref(need)),
                   "smlm_lora_fwd_multi_workspace_size")
        n = _FWD_MULTI_SIZES[key] = need.value
    return n


def smlm_lora_forward_multi(ys, xs, a_ptrs, b_ptrs, plan: SegmentPlan, rank: int,
                            seg_scale: Optional[torch.Tensor] = None, beta: float = 0.0,
                            v_out=None, stages: int = 3, dropout: Optional[DropoutSpec] = None,
                            adapter_rank: Optional[torch.Tensor] = None,
                            workspace: Optional[Workspace] = None, packed_ranks: bool = False,
                            dims=None, cache: Optional[dict] = None) -> None:
    """The fused forward for several projections of one batch (q/k/v/o, gate/up/down)
    in two launches.  Lists of equal length; entries of xs may be the same tensor.
    stages: 1 = shrink only, 2 = expand only (after a shrink call with the same
    arguments, workspace and stream), 3 = both.  A shrink-only call may pass None for
    the ys, an expand-only call None for the xs, and an expand-only call skips the
    projections whose y is None (q, k and v of one shrink call can be expanded one at a
    time); `dims` = [(h_in, h_out), ...] then names the shapes the missing tensors have.  dropout: the training rows of x are
    dropped inside the shrink kernel; projection i uses the stream offset + i.
    adapter_rank (int32, indexed like the tables): true ranks of adapters stored
    zero-padded to `rank`; the padding is then not read.  packed_ranks: the adapters are stored
    AT their true rank rounded up to 8 (A_a [r_a, h_in], B_a [h_out, r_a]) instead of padded.
    cache: a dict the caller keeps (one per layer): after a call has been checked, later calls with
    tensors of the same shapes, dtype, device and contiguity and the same tables skip the checks and
    reuse the argument blocks that do not change."""
    n = len(ys)
    key = None
    if cache is not None and dropout is None and len(xs) == n:  # (a dropout descriptor is checked call by call)
        scale_list = () if seg_scale is None else (seg_scale,)
        key = ("fwd", n, stages, plan.T, plan.S, plan.kind, rank, bool(packed_ranks), _mask(xs), _mask(ys),
               None if v_out is None else _mask(v_out), len(scale_list),
               dims if dims is None or isinstance(dims, tuple) else tuple(tuple(d_) for d_ in dims))
        hit = cache.get(key)
        if hit is not None and hit.matches((xs, ys, v_out or (), scale_list), (*a_ptrs, *b_ptrs, adapter_rank)):
            dev = hit.dev
            with _on(dev):
                ws = _workspace(dev, hit.need, workspace)
                opts = hit.opts
                if not plan.built and not (stages & _lib.SMLM_STAGE_SHRINK):
                    plan.ensure_built()
                if not plan.built:  # a deferred plan: this call builds it
                    opts = _opts(plan, None, None, adapter_rank, hit.n_weights, packed_ranks, checked=True) \
                        or _lib.LoraOpts()
                    opts.build_seg_indptr = plan.segment.data_ptr()
                    if plan.kind == _lib.SMLM_KEY_PTR2:
                        opts.build_seg_key_a = plan.seg_key.data_ptr()
                        opts.build_seg_key_b = plan.seg_key2.data_ptr()
                    else:
                        opts.build_seg_adapter = plan.seg_key.data_ptr()
                y_arr, x_arr, v_arr = hit.arrs
                rc = _lib.load().smlm_lora_fwd_multi_ex(
                    n, _fill(y_arr, ys), _fill(x_arr, xs), None if v_out is None else _fill(v_arr, v_out),
                    hit.a_arr, hit.b_arr, hit.n_weights, hit.h_in, hit.h_out, plan.buf.data_ptr(), ws.data_ptr(),
                    ws.numel(), plan.T, plan.S, rank, hit.code, float(beta), _ptr(seg_scale), int(stages),
                    None if opts is None else C.byref(opts), _stream(dev))
            _lib.check(rc, "smlm_lora_forward")
            plan.built = True
            return
    if not (1 <= n <= 8) or len(xs) != n or len(a_ptrs) != n or len(b_ptrs) != n or \
            (v_out is not None and len(v_out) != n):
        raise RuntimeError("between 1 and 8 projections, all lists of one length")
    _check_scale(seg_scale, plan)
    given = [t for t in list(xs) + list(ys) if t is not None]
    if not given:
        raise RuntimeError("nothing to work on: every x and y is None")
    first = given[0]
    for i in range(n):
        if (ys[i] is None and stages == 3) or (xs[i] is None and stages != 2):
            raise RuntimeError("only a shrink-only call may leave out y, only an expand-only call x")
        if (xs[i] is None or ys[i] is None) and dims is None:
            raise RuntimeError("dims=[(h_in, h_out), ...] must name the shapes of the tensors left out")
        for t, name in ((ys[i], "y"), (xs[i], "x")):
            if t is None:
                continue
            _check_input(t, name)
            _check_dim(2, t, name)
            if t.dtype != first.dtype or t.size(0) != plan.T or t.device != first.device:
                raise RuntimeError("x [T,h_in] and y [T,h_out] must share dtype, device and T with the plan")
            if dims is not None and t.size(1) != dims[i][0 if name == "x" else 1]:
                raise RuntimeError(f"{name} of projection {i} does not have the width dims names")
        _check_table(a_ptrs[i], plan, "a_ptrs")
        _check_table(b_ptrs[i], plan, "b_ptrs")
        if v_out is not None and v_out[i] is not None:
            vo = v_out[i]
            if vo.dtype != first.dtype or tuple(vo.shape) != (plan.T, rank) or not vo.is_contiguous():
                raise RuntimeError("v_out must be a contiguous [T, rank] tensor of x's dtype")
    code = _dtype_code(first)
    dev = first.device
    VP, CI = C.c_void_p * n, C.c_int * n
    widths_in = [dims[i][0] if xs[i] is None else xs[i].size(1) for i in range(n)]
    h_in = CI(*widths_in)
    h_out = CI(*[dims[i][1] if ys[i] is None else ys[i].size(1) for i in range(n)])
    vo_arr = None if v_out is None else VP(*[_ptr(t) for t in v_out])
    with _on(dev):
        need = _fwd_multi_workspace_size(plan.T, tuple(widths_in), rank)
        ws = _workspace(dev, need, workspace)
        n_weights = min(t.size(0) for t in list(a_ptrs) + list(b_ptrs))
        opts = _opts(plan, dropout, widths_in, adapter_rank, n_weights, packed_ranks)
        a_arr, b_arr = VP(*[t.data_ptr() for t in a_ptrs]), VP(*[t.data_ptr() for t in b_ptrs])
        if key is not None:  # (every check has passed: the next call like this one takes the short way)
            hit = _Checked()
            hit.descs = _descs((xs, ys, v_out or (), () if seg_scale is None else (seg_scale,)))
            hit.same = (*a_ptrs, *b_ptrs, adapter_rank)
            hit.code, hit.dev, hit.arrs, hit.h_in, hit.h_out = code, dev, (VP(), VP(), VP()), h_in, h_out
            hit.a_arr, hit.b_arr, hit.n_weights, hit.need = a_arr, b_arr, n_weights, need
            hit.opts = _opts(plan, None, None, adapter_rank, n_weights, packed_ranks, checked=True)
            _remember(cache, key, hit)
        if not plan.built:
            if stages & _lib.SMLM_STAGE_SHRINK:  # a deferred plan: this call builds it
                opts = opts or _lib.LoraOpts()
                opts.build_seg_indptr = plan.segment.data_ptr()
                if plan.kind == _lib.SMLM_KEY_PTR2:
                    opts.build_seg_key_a = plan.seg_key.data_ptr()
                    opts.build_seg_key_b = plan.seg_key2.data_ptr()
                else:
                    opts.build_seg_adapter = plan.seg_key.data_ptr()
            else:
                plan.ensure_built()
        rc = _lib.load().smlm_lora_fwd_multi_ex(
            n, VP(*[_ptr(t) for t in ys]), VP(*[_ptr(t) for t in xs]), vo_arr,
            a_arr, b_arr,
            n_weights, h_in, h_out,
            plan.buf.data_ptr(), ws.data_ptr(), ws.numel(), plan.T, plan.S, rank, code, float(beta),
            _ptr(seg_scale), int(stages), None if opts is None else C.byref(opts), _stream(dev))
    _lib.check(rc, "smlm_lora_forward")
    plan.built = True


def smlm_lora_backward(dx: torch.Tensor, da_ptrs: torch.Tensor, db_ptrs: torch.Tensor,
                       dy: torch.Tensor, x: torch.Tensor, v: Optional[torch.Tensor],
                       a_ptrs: torch.Tensor, b_ptrs: torch.Tensor, plan: SegmentPlan, rank: int,
                       part_scale: Optional[torch.Tensor] = None,
                       dropout: Optional[DropoutSpec] = None,
                       adapter_rank: Optional[torch.Tensor] = None,
                       workspace: Optional[Workspace] = None, packed_ranks: bool = False,
                       is_row_major: bool = False, cache: Optional[dict] = None,
                       zero_dx_tail: bool = False) -> None:
    """dX rows of the train partitions and per-adapter dA / dB (see include/smlm.h).
    `plan` = SegmentPlan(part_indptr, part_adapter int32, n_rows).  dropout: the
    forward's stream with seg_p per partition; x is the tensor before dropout.
    is_row_major: weights and gradients in the reference's other layout, A [h_in, r], B [r, h_out]."""
    smlm_lora_backward_multi([dx], [da_ptrs], [db_ptrs], [dy], [x], None if v is None else [v], [a_ptrs],
                             [b_ptrs], plan, rank, part_scale=part_scale, dropout=dropout,
                             adapter_rank=adapter_rank, workspace=workspace, packed_ranks=packed_ranks,
                             is_row_major=is_row_major, cache=cache, zero_dx_tail=zero_dx_tail)


_BWD_MULTI_SIZES: Dict[Tuple, int] = {}


def _bwd_opts(plan, adapter_rank, n_weights, packed_ranks, stages, is_row_major, checked, dropout=None, widths=None,
              dx_rows=0):
    """struct smlm_lora_opts of a backward call (None when there is nothing to say)."""
    opts = _opts(plan, dropout, widths, adapter_rank, n_weights, packed_ranks, checked=checked)
    if dx_rows:
        opts = opts or _lib.LoraOpts()
        opts.dx_rows = int(dx_rows)
    if stages:
        opts = opts or _lib.LoraOpts()
        opts.bwd_stages = int(stages)
    if is_row_major:
        opts = opts or _lib.LoraOpts()
        opts.w_row_major = 1
    return opts


def _bwd_multi_workspace_size(n_rows: int, P: int, NA: int, widths_in: Tuple[int, ...],
                              widths_out: Tuple[int, ...], rank: int) -> int:
    key = (n_rows, P, NA, widths_in, widths_out, rank)
    n = _BWD_MULTI_SIZES.get(key)
    if n is None:
        need = C.c_size_t(0)
        CI = C.c_int * len(widths_in)
        _lib.check(_lib.load().smlm_lora_bwd_multi_workspace_size(len(widths_in), n_rows, P, NA, CI(*widths_in),
                                                                  CI(*widths_out), rank, C.byref(need)),
                   "smlm_lora_bwd_multi_workspace_size")
        n = _BWD_MULTI_SIZES[key] = need.value
    return n


def smlm_lora_backward_multi(dxs, da_ptrs, db_ptrs, dys, xs, vs, a_ptrs, b_ptrs, plan: SegmentPlan, rank: int,
                             part_scale: Optional[torch.Tensor] = None,
                             dropout: Optional[DropoutSpec] = None,
                             adapter_rank: Optional[torch.Tensor] = None,
                             workspace: Optional[Workspace] = None, packed_ranks: bool = False,
                             stages: int = 0, is_row_major: bool = False,
                             cache: Optional[dict] = None, zero_dx_tail: bool = False) -> None:
    """The backward of several projections of one batch (q/k/v/o, gate/up/down) in one set of
    launches; lists of equal length, one entry per projection, each what smlm_lora_backward
    takes.  vs: None, or the saved intermediate of every projection.  The results equal
    per-projection calls bit for bit.  dropout: projection i uses the stream offset + i and
    the keep bits of the projections lie end to end (as smlm_lora_forward_multi leaves them).
    stages: 0 = everything; else SMLM_BWD_* bits (1 products v / dV, 2 dX, 4 weight gradients): the stages
    may be issued as separate calls with the same arguments, workspace and stream, in that order.
    is_row_major: the weights and their gradients are A [h_in, r], B [r, h_out] (the layout the reference's
    backward lines are written for, kernel_utils.py:139-145) instead of PEFT's A [r, h_in], B [h_out, r].
    cache: as in smlm_lora_forward_multi (the same dict may serve a layer's forward and backward).
    zero_dx_tail: the dx tensors cover more rows than the plan (the whole batch): the call also sets their rows from
    plan.T on to zero, inside one of its launches where it can (all dx must then have the same number of rows)."""
    n = len(dxs)
    key = None
    if cache is not None and dropout is None:  # (a dropout descriptor is checked call by call)
        scale_list = () if part_scale is None else (part_scale,)
        key = ("bwd", n, stages, plan.T, plan.S, plan.kind, rank, bool(packed_ranks), bool(is_row_major),
               vs is None, len(scale_list), bool(zero_dx_tail))
        hit = cache.get(key)
        if hit is not None and hit.matches((dxs, dys, xs, vs or (), da_ptrs, db_ptrs, scale_list),
                                           (*a_ptrs, *b_ptrs, adapter_rank)):
            dev = hit.dev
            with _on(dev):
                ws = _workspace(dev, hit.need, workspace)
                opts = hit.opts
                if not plan.built and stages and not (stages & _lib.SMLM_BWD_PRODUCTS):
                    plan.ensure_built()
                if not plan.built:  # a deferred plan: this call builds it
                    opts = _bwd_opts(plan, adapter_rank, hit.n_weights, packed_ranks, stages, is_row_major, True,
                                     dx_rows=dxs[0].size(0) if zero_dx_tail else 0) or _lib.LoraOpts()
                    opts.build_seg_indptr = plan.segment.data_ptr()
                    opts.build_seg_adapter = plan.seg_key.data_ptr()
                dx_arr, dy_arr, x_arr, v_arr, da_arr, db_arr = hit.arrs
                rc = _lib.load().smlm_lora_bwd_multi_ex(
                    n, _fill(dx_arr, dxs), _fill(da_arr, da_ptrs), _fill(db_arr, db_ptrs), _fill(dy_arr, dys),
                    _fill(x_arr, xs), None if vs is None else _fill(v_arr, vs), hit.a_arr, hit.b_arr,
                    plan.buf.data_ptr(), ws.data_ptr(), ws.numel(), plan.T, plan.S, hit.n_weights, hit.h_in,
                    hit.h_out, rank, hit.code, _ptr(part_scale), None if opts is None else C.byref(opts),
                    _stream(dev))
            _lib.check(rc, "smlm_lora_backward")
            plan.built = True
            return
    lists = (da_ptrs, db_ptrs, dys, xs, a_ptrs, b_ptrs) + (() if vs is None else (vs,))
    if not (1 <= n <= 8) or any(len(l) != n for l in lists):
        raise RuntimeError("between 1 and 8 projections, all lists of one length")
    if plan.kind != _lib.SMLM_KEY_I32:
        raise RuntimeError("the backward plan must be built from int32 adapter ids")
    n_rows = plan.T
    NA = a_ptrs[0].size(0)
    dtype = dys[0].dtype
    for i in range(n):
        for t, name in ((dxs[i], "dx"), (dys[i], "dy"), (xs[i], "x"), (da_ptrs[i], "da_ptrs"),
                        (db_ptrs[i], "db_ptrs"), (a_ptrs[i], "a_ptrs"), (b_ptrs[i], "b_ptrs")):
            _check_input(t, name)
        if dys[i].size(0) < n_rows or xs[i].size(0) < n_rows or dxs[i].size(0) < n_rows:
            raise RuntimeError("dy, x and dx need at least plan.T rows")
        v = None if vs is None else vs[i]
        if dxs[i].dtype != dtype or xs[i].dtype != dtype or dys[i].dtype != dtype or \
                (v is not None and v.dtype != dtype):
            raise RuntimeError("dx, dy, x, v must share one dtype")
        if any(t.size(0) != NA for t in (a_ptrs[i], b_ptrs[i], da_ptrs[i], db_ptrs[i])):
            raise RuntimeError("pointer tables must all have one entry per adapter")
        if vs is not None and (v is None or v.size(0) < n_rows or v.size(1) != rank or not v.is_contiguous()):
            raise RuntimeError("v must be a contiguous [>=n_rows, rank] tensor (of every projection or of none)")
        if dxs[i].size(1) != xs[i].size(1):
            raise RuntimeError("dx and x must have the same width")
    code = _dtype_code(dys[0])
    widths_in = tuple(t.size(1) for t in xs)
    widths_out = tuple(t.size(1) for t in dys)
    dev = dys[0].device
    VP, CI = C.c_void_p * n, C.c_int * n
    with _on(dev):
        need = _bwd_multi_workspace_size(n_rows, plan.S, NA, widths_in, widths_out, rank)
        ws = _workspace(dev, need, workspace)
        if dropout is not None and dropout.rows < n_rows:
            raise RuntimeError("the dropout descriptor must cover the backward's rows")
        dx_rows = 0
        if zero_dx_tail:
            dx_rows = dxs[0].size(0)
            if any(t.size(0) != dx_rows for t in dxs):
                raise RuntimeError("zero_dx_tail: every dx must have the same number of rows")
        opts = _bwd_opts(plan, adapter_rank, NA, packed_ranks, stages, is_row_major, False, dropout,
                         list(widths_in), dx_rows)
        arr = lambda ts: VP(*[t.data_ptr() for t in ts])
        a_arr, b_arr, h_in, h_out = arr(a_ptrs), arr(b_ptrs), CI(*widths_in), CI(*widths_out)
        if key is not None:  # (every check has passed: the next call like this one takes the short way)
            hit = _Checked()
            hit.descs = _descs((dxs, dys, xs, vs or (), da_ptrs, db_ptrs, () if part_scale is None else (part_scale,)))
            hit.same = (*a_ptrs, *b_ptrs, adapter_rank)
            hit.code, hit.dev, hit.arrs, hit.h_in, hit.h_out = code, dev, tuple(VP() for _ in range(6)), h_in, h_out
            hit.a_arr, hit.b_arr, hit.n_weights, hit.need = a_arr, b_arr, NA, need
            hit.opts = _bwd_opts(plan, adapter_rank, NA, packed_ranks, stages, is_row_major, True, dx_rows=dx_rows)
            _remember(cache, key, hit)
        if not plan.built:  # a deferred plan: this call builds it (inside its first launch where it can)
            if stages and not (stages & _lib.SMLM_BWD_PRODUCTS):
                plan.ensure_built()
            else:
                opts = opts or _lib.LoraOpts()
                opts.build_seg_indptr = plan.segment.data_ptr()
                opts.build_seg_adapter = plan.seg_key.data_ptr()
        rc = _lib.load().smlm_lora_bwd_multi_ex(
            n, arr(dxs), arr(da_ptrs), arr(db_ptrs), arr(dys), arr(xs), None if vs is None else arr(vs),
            a_arr, b_arr, plan.buf.data_ptr(), ws.data_ptr(), ws.numel(), n_rows, plan.S, NA,
            h_in, h_out, rank, code, _ptr(part_scale),
            None if opts is None else C.byref(opts), _stream(dev))
    _lib.check(rc, "smlm_lora_backward")
    plan.built = True


def rms_norm(output: torch.Tensor, rms_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
             epsilon: float) -> None:
    """output = input * rms * weight, rms_output = 1 / sqrt(mean(input^2) + epsilon) per row.

    Same arguments and checks as dispatch_rms_norm
    (kernel_src/csrc/loquetier_ops.cc:326-358): input/output [rows, cols] fp16
    or bf16, weight [cols] of the same dtype, rms_output float32 [rows, 1].
    """
    for t, n in ((output, "output"), (rms_output, "rms_output"), (input, "input"), (weight, "weight")):
        _check_input(t, n)
    _check_dim(2, input, "input")
    _check_dim(2, rms_output, "rms_output")
    _check_dim(1, weight, "weight")
    if output.shape != input.shape:
        raise RuntimeError("output and input must have the same shape")
    if rms_output.size(0) != input.size(0) or rms_output.size(1) != 1:
        raise RuntimeError("rms_output must be [rows, 1]")
    if rms_output.dtype != torch.float32:
        raise RuntimeError("rms_output must be float32")
    if weight.size(0) != input.size(1):
        raise RuntimeError("weight must have one entry per column of input")
    if input.dtype != weight.dtype or input.dtype != output.dtype:
        raise RuntimeError("input, weight and output must share one dtype")
    rows, cols = input.shape
    if input.dtype not in _DTYPE_CODE or cols % 8 != 0:
        raise RuntimeError(f"No suitable kernel. dtype={input.dtype} columns={cols}")
    dev = input.device
    with _on(dev):
        rc = _lib.load().smlm_rms_norm_fwd(output.data_ptr(), rms_output.data_ptr(), input.data_ptr(),
                                           weight.data_ptr(), rows, cols, float(epsilon),
                                           _DTYPE_CODE[input.dtype], _stream(dev))
    _lib.check(rc, "rms_norm")


def rms_norm_backward(dx: torch.Tensor, dw: torch.Tensor, grad_output: torch.Tensor, x: torch.Tensor,
                      w: torch.Tensor, rms: torch.Tensor) -> None:
    """dx [rows, cols] and dw [cols] of RMSNorm from the upstream gradient and the
    forward's saved tensors (the reference computes them with tensor expressions,
    src/loquetier_src/kernel_utils.py:169-176)."""
    for t, n in ((dx, "dx"), (dw, "dw"), (grad_output, "grad_output"), (x, "x"), (w, "w"), (rms, "rms")):
        _check_input(t, n)
    if dx.shape != x.shape or grad_output.shape != x.shape or dw.shape != w.shape:
        raise RuntimeError("dx / grad_output must match x and dw must match w")
    if rms.dtype != torch.float32 or rms.numel() != x.size(0):
        raise RuntimeError("rms must be float32 with one entry per row")
    if not (dx.dtype == dw.dtype == grad_output.dtype == x.dtype == w.dtype):
        raise RuntimeError("dx, dw, grad_output, x, w must share one dtype")
    rows, cols = x.shape
    code = _dtype_code(x)
    dev = x.device
    with _on(dev):
        need = _lib.size_query("smlm_rms_norm_bwd_workspace_size", rows, cols)
        ws = _workspace(dev, need)
        rc = _lib.load().smlm_rms_norm_bwd(dx.data_ptr(), dw.data_ptr(), grad_output.data_ptr(),
                                           x.data_ptr(), w.data_ptr(), rms.data_ptr(), ws.data_ptr(),
                                           ws.numel(), rows, cols, code, _stream(dev))
    _lib.check(rc, "rms_norm_backward")


def segments_build(req_adapter: torch.Tensor, req_len: torch.Tensor):
    """Run-length segments from per-request (adapter id, token count), on the device.

    The device version of the loop in ModelGeneration.generate
    (src/loquetier_src/model_generation.py:267-283).  Both inputs are int32 [R]
    device tensors.  Returns (seg_adapter [R], seg_len [R], seg_indptr [R+1],
    n_seg [2]) as int32 device tensors; n_seg holds (segment count, total rows)
    and is not read back here, so nothing waits for the device.  Entries past
    n_seg[0] are empty segments; pass the arrays on whole (S = R)."""
    for t, n in ((req_adapter, "req_adapter"), (req_len, "req_len")):
        _check_input(t, n)
        _check_dim(1, t, n)
        if t.dtype != torch.int32:
            raise RuntimeError(f"{n} must be int32")
    if req_adapter.numel() != req_len.numel():
        raise RuntimeError("req_adapter and req_len must have one entry per request")
    dev, R = req_adapter.device, req_adapter.numel()
    seg_adapter = torch.empty(R, dtype=torch.int32, device=dev)
    seg_len = torch.empty(R, dtype=torch.int32, device=dev)
    seg_indptr = torch.empty(R + 1, dtype=torch.int32, device=dev)
    n_seg = torch.empty(2, dtype=torch.int32, device=dev)
    with _on(dev):
        rc = _lib.load().smlm_segments_build(_ptr(req_adapter), _ptr(req_len), R, _ptr(seg_adapter),
                                             _ptr(seg_len), seg_indptr.data_ptr(), n_seg.data_ptr(),
                                             _stream(dev))
    _lib.check(rc, "segments_build")
    return seg_adapter, seg_len, seg_indptr, n_seg
