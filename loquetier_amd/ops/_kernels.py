"""Python surface of the HIP library, with the names and argument order of the
reference's pybind module `loquetier.ops._kernels`
(kernel_src/csrc/loquetier_ops.cc:365-374) for the SMLM entries, plus the
fused forward, the backward and the plan builder this build adds.

Tensors are torch tensors on a ROCm device; the calls are asynchronous on
torch's current stream of that device.  Nothing here computes on the host.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .. import _lib

_DTYPE_CODE = {torch.float16: _lib.SMLM_DTYPE_F16, torch.bfloat16: _lib.SMLM_DTYPE_BF16}

# (device index, stream handle) -> uint8 workspace tensor, grown on demand.
# Calls on one stream are ordered, so they can share one buffer.
_WORKSPACES: Dict[Tuple[int, int], torch.Tensor] = {}


def _stream(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def _workspace(dev: torch.device, nbytes: int, tag: int = 0) -> torch.Tensor:
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), _stream(dev), tag)
    buf = _WORKSPACES.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20) * 3 // 2, dtype=torch.uint8, device=dev)
        _WORKSPACES[key] = buf
    return buf


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


def smlm_forward_cutlass(y: torch.Tensor, x: torch.Tensor, w_ptr: torch.Tensor, s: torch.Tensor,
                         tmp: torch.Tensor, is_row_major: bool) -> None:
    """Grouped GEMM y[s_i:s_{i+1}] = x[s_i:s_{i+1}] @ W_i, overwriting y.

    Same contract as dispatch_smlm_forward_cutlass
    (kernel_src/csrc/loquetier_ops.cc:277-319): y [T,d_out], x [T,d_in] fp16 or
    bf16, w_ptr int64 [S] device addresses, s int32 [S+1], tmp uint8 of exactly
    smlm_forward_cutlass_tmp_size(S) bytes.  Unlike the reference it does not
    block the host.
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
    if tmp.size(0) != smlm_forward_cutlass_tmp_size(num_problems):
        raise RuntimeError(f"CHECK_EQ(tmp.size(0), smlm_forward_tmp_size(num_problems)) failed: "
                           f"{tmp.size(0)} vs {smlm_forward_cutlass_tmp_size(num_problems)}")
    if w_ptr.dtype != torch.int64 or s.dtype != torch.int32:
        raise RuntimeError("w_ptr must be int64 and s must be int32")
    if w_ptr.size(0) != num_problems or y.size(0) != x.size(0) or y.dtype != x.dtype:
        raise RuntimeError("inconsistent shapes: w_ptr [S], s [S+1], x [T,d_in], y [T,d_out]")
    code = _dtype_code(x)
    T = x.size(0)
    dev = tmp.device
    with torch.cuda.device(dev):
        need = _lib.size_query("smlm_gemm_workspace_size", T, num_problems, d_in, d_out)
        ws = _workspace(dev, need)
        rc = _lib.load().smlm_gemm(y.data_ptr(), x.data_ptr(), w_ptr.data_ptr(), s.data_ptr(),
                                   ws.data_ptr(), ws.numel(), T, num_problems, d_in, d_out, w_ld,
                                   int(bool(is_row_major)), code, 0.0, None, _stream(dev))
    if rc == _lib.SMLM_ERR_DTYPE:
        raise RuntimeError(f"No suitable kernel. dtype={x.dtype}")
    _lib.check(rc, "smlm_forward_cutlass")


class SegmentPlan:
    """Tile plan of one flat batch: built once from (segment, adapter ids) and
    shared by every LoRA linear of the step (the reference rebuilds its
    per-problem table inside every kernel call,
    smlm_forward_cutlass.cuh:76-79)."""

    def __init__(self, segment: torch.Tensor, seg_key: Optional[torch.Tensor], T: int):
        _check_input(segment, "segment")
        if segment.dtype != torch.int32 or segment.dim() != 1:
            raise RuntimeError("segment must be a 1D int32 tensor")
        self.segment = segment
        self.S = segment.size(0) - 1
        self.T = int(T)
        self.seg_key = seg_key
        if seg_key is None:
            kind = _lib.SMLM_KEY_NONE
        elif seg_key.dtype == torch.int32:
            kind = _lib.SMLM_KEY_I32
        elif seg_key.dtype == torch.int64:
            kind = _lib.SMLM_KEY_PTR
        else:
            raise RuntimeError("seg_key must be int32 adapter ids or int64 addresses")
        if seg_key is not None:
            _check_input(seg_key, "seg_key")
            if seg_key.dim() != 1 or seg_key.size(0) != self.S:
                raise RuntimeError("seg_key must have one entry per segment")
        dev = segment.device
        nbytes = _lib.size_query("smlm_plan_size", self.T, self.S)
        self.buf = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = _lib.load().smlm_plan_build(self.buf.data_ptr(), self.buf.numel(), segment.data_ptr(),
                                             _ptr(seg_key), kind, self.T, self.S, _stream(dev))
        _lib.check(rc, "smlm_plan_build")

    def header(self) -> Tuple[int, int, int, int]:
        """(n_tiles, n_groups, rows covered, key kind used) -- synchronises; for tests."""
        h = self.buf[:16].view(torch.int32).cpu()
        return int(h[0]), int(h[1]), int(h[2]), int(h[3])


def smlm_lora_forward(y: torch.Tensor, x: torch.Tensor, a_ptrs: torch.Tensor, b_ptrs: torch.Tensor,
                      plan: SegmentPlan, rank: int, seg_adapter: Optional[torch.Tensor] = None,
                      seg_scale: Optional[torch.Tensor] = None, beta: float = 0.0,
                      v_out: Optional[torch.Tensor] = None) -> None:
    """y = beta*y + seg_scale * round(x A^T) B^T in one stream-ordered call."""
    for t, n in ((y, "y"), (x, "x"), (a_ptrs, "a_ptrs"), (b_ptrs, "b_ptrs")):
        _check_input(t, n)
    _check_dim(2, y, "y")
    _check_dim(2, x, "x")
    if y.dtype != x.dtype or y.size(0) != x.size(0) or x.size(0) != plan.T:
        raise RuntimeError("x [T,h_in] and y [T,h_out] must share dtype and T with the plan")
    if a_ptrs.dtype != torch.int64 or b_ptrs.dtype != torch.int64:
        raise RuntimeError("pointer tables must be int64")
    if seg_adapter is None and (a_ptrs.size(0) != plan.S or b_ptrs.size(0) != plan.S):
        raise RuntimeError("per-segment pointer tables must have one entry per segment")
    if seg_adapter is not None and (seg_adapter.dtype != torch.int32 or seg_adapter.size(0) != plan.S
                                    or not seg_adapter.is_cuda):
        raise RuntimeError("seg_adapter must be a device int32 tensor with one entry per segment")
    if seg_scale is not None and (seg_scale.dtype != torch.float32 or seg_scale.size(0) != plan.S
                                  or not seg_scale.is_cuda):
        raise RuntimeError("seg_scale must be a device float32 tensor with one entry per segment")
    if v_out is not None and (v_out.dtype != x.dtype or tuple(v_out.shape) != (x.size(0), rank)
                              or not v_out.is_contiguous()):
        raise RuntimeError("v_out must be a contiguous [T, rank] tensor of x's dtype")
    code = _dtype_code(x)
    T, h_in, h_out = x.size(0), x.size(1), y.size(1)
    dev = x.device
    with torch.cuda.device(dev):
        need = _lib.size_query("smlm_lora_fwd_workspace_size", T, plan.S, h_in, h_out, rank)
        ws = _workspace(dev, need)
        rc = _lib.load().smlm_lora_fwd(y.data_ptr(), x.data_ptr(), _ptr(v_out), a_ptrs.data_ptr(),
                                       b_ptrs.data_ptr(), _ptr(seg_adapter), plan.segment.data_ptr(),
                                       plan.buf.data_ptr(), ws.data_ptr(), ws.numel(), T, plan.S, h_in,
                                       h_out, rank, code, float(beta), _ptr(seg_scale), _stream(dev))
    _lib.check(rc, "smlm_lora_forward")


def smlm_lora_backward(dx: torch.Tensor, da_ptrs: torch.Tensor, db_ptrs: torch.Tensor,
                       dy: torch.Tensor, x: torch.Tensor, v: Optional[torch.Tensor],
                       a_ptrs: torch.Tensor, b_ptrs: torch.Tensor, part_adapter: torch.Tensor,
                       plan: SegmentPlan, rank: int, part_scale: Optional[torch.Tensor] = None) -> None:
    """dX rows of the train partitions and per-adapter dA / dB (see include/smlm.h)."""
    for t, n in ((dx, "dx"), (dy, "dy"), (x, "x"), (da_ptrs, "da_ptrs"), (db_ptrs, "db_ptrs"),
                 (a_ptrs, "a_ptrs"), (b_ptrs, "b_ptrs"), (part_adapter, "part_adapter")):
        _check_input(t, n)
    n_rows = plan.T
    if dy.size(0) < n_rows or x.size(0) < n_rows or dx.size(0) < n_rows:
        raise RuntimeError("dy, x and dx need at least plan.T rows")
    if dx.dtype != dy.dtype or x.dtype != dy.dtype or (v is not None and v.dtype != dy.dtype):
        raise RuntimeError("dx, dy, x, v must share one dtype")
    if part_adapter.dtype != torch.int32 or part_adapter.size(0) != plan.S:
        raise RuntimeError("part_adapter must be int32 with one entry per partition")
    NA = a_ptrs.size(0)
    if b_ptrs.size(0) != NA or da_ptrs.size(0) != NA or db_ptrs.size(0) != NA:
        raise RuntimeError("pointer tables must all have one entry per adapter")
    if v is not None and (v.size(0) < n_rows or v.size(1) != rank or not v.is_contiguous()):
        raise RuntimeError("v must be a contiguous [>=n_rows, rank] tensor")
    code = _dtype_code(dy)
    h_in, h_out = x.size(1), dy.size(1)
    dev = dy.device
    with torch.cuda.device(dev):
        need = _lib.size_query("smlm_lora_bwd_workspace_size", n_rows, plan.S, NA, h_in, h_out, rank)
        ws = _workspace(dev, need)
        rc = _lib.load().smlm_lora_bwd(dx.data_ptr(), da_ptrs.data_ptr(), db_ptrs.data_ptr(),
                                       dy.data_ptr(), x.data_ptr(), _ptr(v), a_ptrs.data_ptr(),
                                       b_ptrs.data_ptr(), part_adapter.data_ptr(),
                                       plan.segment.data_ptr(), plan.buf.data_ptr(), ws.data_ptr(),
                                       ws.numel(), n_rows, plan.S, NA, h_in, h_out, rank, code,
                                       _ptr(part_scale), _stream(dev))
    _lib.check(rc, "smlm_lora_backward")
