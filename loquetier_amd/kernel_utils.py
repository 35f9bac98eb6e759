"""Host-side mirror of src/loquetier_src/kernel_utils.py for the SMLM path:
`BatchLenInfo` (row layout of the flat batch) and the `add_lora` autograd
Function, with the reference's positional arguments and `None`-padded backward
tuple, running on the HIP kernels; and the `rms_norm` autograd Function
(kernel_utils.py:149-176).
"""
from __future__ import annotations

from collections.abc import Sequence
from typing import List, Optional, Tuple

import numpy as np
import torch
from torch.autograd.function import Function, FunctionCtx

from .ops import _kernels as kernel


class BatchLenInfo:
    """Row layout [train | eval | prefill | decode] of one flat batch
    (reference: src/loquetier_src/kernel_utils.py:11-98, same properties)."""

    def __init__(self, trains: List[Tuple[int, ...]], prefills: List[int], decode: int,
                 evals: List[Tuple[int, ...]], indptr_device: torch.device,
                 indptr_dtype: torch.dtype = torch.int32):
        self._train_batches = trains
        tlen = [t[0] * t[1] for t in trains]
        if tlen:
            self._train_partition = np.cumsum([0] + tlen)
            self._tlen = int(self._train_partition[-1])
        else:
            self._train_partition = []
            self._tlen = 0
        self._eval_batches = evals
        if evals:
            self._eval_partition = np.cumsum([self._tlen] + [e[0] * e[1] for e in evals])
        else:
            self._eval_partition = []
        self._prefills = list(prefills)
        self._decode = decode
        if prefills:
            cumsum = np.cumsum([0] + list(prefills))
            self._indptr = torch.tensor(cumsum, dtype=indptr_dtype, device=indptr_device)
            self._doff = int(cumsum[-1]) + self._tlen
        else:
            self._indptr = None
            self._doff = self._tlen

    @property
    def train_batches(self) -> List[Tuple[int, ...]]:
        return self._train_batches

    @property
    def train_partition(self) -> Sequence[int]:
        return self._train_partition

    @property
    def eval_batches(self) -> List[Tuple[int, ...]]:
        return self._eval_batches

    @property
    def eval_partition(self) -> Sequence[int]:
        return self._eval_partition

    @property
    def prefills(self) -> List[int]:
        return self._prefills

    @property
    def decode(self) -> int:
        return self._decode

    @property
    def tlen(self) -> int:
        return self._tlen

    @property
    def doff(self) -> int:
        return self._doff

    @property
    def indptr(self) -> Optional[torch.Tensor]:
        return self._indptr


def _ptr_table(tensors: Sequence[torch.Tensor], device: torch.device) -> torch.Tensor:
    return torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64, device=device)


def _unique_adapters(weight_list: Sequence[torch.Tensor]):
    """Train partitions -> indices into the list of distinct (A, B) pairs."""
    pairs, index, part_adapter = [], {}, []
    for wa, wb in zip(weight_list[::2], weight_list[1::2]):
        key = (wa.data_ptr(), wb.data_ptr())
        if key not in index:
            index[key] = len(pairs)
            pairs.append((wa, wb))
        part_adapter.append(index[key])
    return pairs, part_adapter


def lora_backward(grad_output: torch.Tensor, x_train: torch.Tensor, v_train: Optional[torch.Tensor],
                  weight_list: Sequence[torch.Tensor], tp: Sequence[int], lora_rank: int,
                  part_scale: Optional[torch.Tensor] = None, dropout=None,
                  adapter_rank: Optional[torch.Tensor] = None, step=None):
    """Shared backward: returns (grad_x [T, h_in], [grad per weight occurrence]).

    Partitions that train the same adapter contribute to one summed gradient,
    returned for the first occurrence of that adapter; later occurrences get
    None (autograd adds per-occurrence gradients, so the total is the same as
    the reference's, src/loquetier_src/models/mixed_lora.py:201-204).

    `step` (mixed_lora.LayerStep or None): the backward's plan, the partitions'
    adapters, the weights' pointer tables and the layout of one buffer for all the
    gradients, prepared outside the layer loop; without it they are built here
    (five small host-to-device copies and a plan launch per call)."""
    dev, dt = grad_output.device, grad_output.dtype
    T = grad_output.size(0)
    h_in = x_train.size(1)
    n_parts = min(len(weight_list) // 2, len(tp) - 1)
    tp = [int(t) for t in tp][: n_parts + 1]
    tl = tp[-1]
    grad_x = torch.empty((T, h_in), dtype=dt, device=dev)
    # rows past the training rows: cleared by the backward call itself (inside one of its launches) when one follows
    tail_in_call = 0 < tl < T
    if tl == 0:
        grad_x.zero_()
    if tp[0] > 0:
        grad_x[: tp[0]].zero_()
    prepared = step is not None and step.bwd_plan is not None and step.grad_layout is not None
    if prepared:
        part_adapter = step.part_adapter
        lay = step.grad_layout
        uniform, known = lay["grad_uniform"], lay["grad_tabs"]
        # addresses of the gradients: device arithmetic, no copy from the host; torch's allocator hands the
        # same blocks out step after step, so the tables of an address are kept
        if uniform is not None:   # matrices of one shape: one tensor for the dA, one for the dB
            NA, sa, sb = uniform
            ga, gb = torch.empty((NA,) + sa, dtype=dt, device=dev), torch.empty((NA,) + sb, dtype=dt, device=dev)
            da, db = ga.unbind(0), gb.unbind(0)
            bufs, where = (ga, gb), (ga.data_ptr(), gb.data_ptr())
            tabs = known.get(where)
            if tabs is None:
                tabs = (lay["grad_offsets_a"] + where[0], lay["grad_offsets_b"] + where[1])
        else:                     # all dA, then all dB, in one allocation
            buf = torch.empty(lay["grad_numel"], dtype=dt, device=dev)
            mats = [buf[o: o + shape[0] * shape[1]].view(shape) for o, shape in lay["grad_shapes"]]
            NA = len(mats) // 2
            da, db = mats[:NA], mats[NA:]
            bufs, where = (buf,), buf.data_ptr()
            tabs = known.get(where)
            if tabs is None:
                both = lay["grad_offsets"] + where
                tabs = (both[:NA], both[NA:])
        if where not in known:
            if len(known) >= 64:
                known.clear()
            known[where] = tabs
        if tl > 0:
            g = grad_output if grad_output.is_contiguous() else grad_output.contiguous()
            kernel.smlm_lora_backward(grad_x, tabs[0], tabs[1], g, x_train, v_train, step.a_tab, step.b_tab,
                                      step.bwd_plan, lora_rank, part_scale, dropout=dropout,
                                      adapter_rank=adapter_rank, workspace=step.workspace,
                                      packed_ranks=step.packed, cache=step.cache, zero_dx_tail=tail_in_call)
        else:
            for b in bufs:
                b.zero_()
    else:
        pairs, part_adapter = _unique_adapters(weight_list[: 2 * n_parts])
        da = [torch.empty_like(wa) for wa, _ in pairs]
        db = [torch.empty_like(wb) for _, wb in pairs]
        if tl > 0:
            g = grad_output if grad_output.is_contiguous() else grad_output.contiguous()
            part_indptr = torch.tensor(tp, dtype=torch.int32, device=dev)
            part_ad = torch.tensor(part_adapter, dtype=torch.int32, device=dev)
            plan = kernel.SegmentPlan(part_indptr, part_ad, tl)
            kernel.smlm_lora_backward(
                grad_x, _ptr_table(da, dev), _ptr_table(db, dev), g, x_train, v_train,
                _ptr_table([p[0] for p in pairs], dev), _ptr_table([p[1] for p in pairs], dev),
                plan, lora_rank, part_scale, dropout=dropout, adapter_rank=adapter_rank,
                workspace=None if step is None else step.workspace,
                packed_ranks=step is not None and step.packed, zero_dx_tail=tail_in_call)
        else:
            for t in da + db:
                t.zero_()
    grads: List[Optional[torch.Tensor]] = []
    seen = set()
    for ad in part_adapter:
        if ad in seen:
            grads += [None, None]
        else:
            seen.add(ad)
            grads += [da[ad], db[ad]]
    grads += [None] * (len(weight_list) - len(grads))
    return grad_x, grads


class add_lora(Function):
    """Reference: src/loquetier_src/kernel_utils.py:101-147.

    forward(y_shape, x, wa_ptr, wb_ptr, s, lora_rank, train_len, train_partition, *weights)
    returns y = (x @ A_seg^T) @ B_seg^T per segment (A [r,h_in], B [h_out,r]).
    The two grouped GEMMs of the reference run as one fused call; v (rounded to
    x's dtype, as the reference materialises it) is kept for backward instead
    of being recomputed.  backward returns gradients for x and for each
    trainable weight, written for the layout the forward uses.
    """

    @staticmethod
    def forward(ctx: FunctionCtx, y_shape, x, wa_ptr, wb_ptr, s, lora_rank, train_len,
                train_partition, *args):
        y = torch.empty(y_shape, dtype=x.dtype, device=x.device)
        need_v = len(args) > 0 and train_len > 0
        v = torch.empty((x.size(0), lora_rank), dtype=x.dtype, device=x.device) if need_v else None
        # The reference looks up wa_ptr[i] and wb_ptr[i] per problem, so two segments may share A and
        # differ in B: the plan groups the segments where BOTH addresses agree, and is built by the
        # fused call itself (for batches of few segments inside its shrink launch).
        plan = kernel.SegmentPlan(s, (wa_ptr, wb_ptr), x.size(0), defer=True)
        kernel.smlm_lora_forward(y, x, wa_ptr, wb_ptr, plan, lora_rank, v_out=v)
        # what the reference's setup_context keeps (kernel_utils.py:122-126), plus v
        ctx.tp = train_partition
        ctx.rank = lora_rank
        ctx.has_v = v is not None
        if v is not None:
            ctx.save_for_backward(x[:train_len, ...], v[:train_len, ...], *args)
        else:
            ctx.save_for_backward(x[:train_len, ...], *args)
        return y

    @staticmethod
    def backward(ctx: FunctionCtx, grad_output: torch.Tensor):
        if ctx.has_v:
            x, v, *weight_list = ctx.saved_tensors
        else:
            x, *weight_list = ctx.saved_tensors
            v = None
        if len(weight_list) == 0:
            return None, None, None, None, None, None, None, None
        assert len(weight_list) % 2 == 0
        grad_x, grads = lora_backward(grad_output, x, v, weight_list, ctx.tp, ctx.rank)
        return (None, grad_x, None, None, None, None, None, None, *grads)



class rms_norm(Function):
    """RMSNorm with the reference's call signature `rms_norm.apply(x, w, eps)`
    (src/loquetier_src/kernel_utils.py:149-176).  x: [rows, cols] fp16/bf16,
    w: [cols].  The backward runs as one fused kernel in float instead of the
    reference's chain of 16-bit tensor expressions."""

    @staticmethod
    def forward(ctx: FunctionCtx, x: torch.Tensor, w: torch.Tensor, eps: float = 1e-6):
        m = torch.empty((x.size(0), 1), dtype=torch.float32, device=x.device)
        o = torch.empty_like(x)
        kernel.rms_norm(o, m, x, w, eps)
        ctx.save_for_backward(x, w, m)
        return o

    @staticmethod
    def backward(ctx: FunctionCtx, grad_output: torch.Tensor):
        x, w, rms_1 = ctx.saved_tensors
        dx = torch.empty_like(x)
        d_weight = torch.empty_like(w)
        kernel.rms_norm_backward(dx, d_weight, grad_output.contiguous(), x, w, rms_1)
        return dx, d_weight, None
