"""Minimal counterpart of the reference's LoRA layer for the SMLM path:
`MixedLoraContext`, `NamedLoraLayer`, `MixedLoraLinear`
(src/loquetier_src/models/mixed_lora.py:24-235) and the rank padding / scale
folding of `MixedLoraModel._prepare_weight` (:501-521).

`MixedLoraLinear.forward` keeps the reference's data flow -- base layer, per
train-partition dropout, LoRA term, scale, residual add -- but by default runs
the last three as one fused in-place kernel call and lets the kernel do the
`wa_ptrs[lora_ids]` gather.  `fused=False` reproduces the reference's sequence
of separate tensor ops (same operator calls, same rounding points).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List, Optional, Sequence, Union

import torch
from torch import nn
from torch.autograd.function import Function, FunctionCtx

from .kernel_utils import BatchLenInfo, add_lora, lora_backward
from .ops import _kernels as kernel


class MixedLoraContext:
    """Per-step routing record shared by every LoRA linear of a model
    (reference: mixed_lora.py:24-64).  `update` also builds the tile plan and
    the device copy of the adapter ids once, for all layers of the step."""

    def __init__(self):
        self._blen = None
        self._lora_ids = None
        self._lora_len = None
        self._segment = None
        self._train_idx: List[int] = []
        self._plan: Optional[kernel.SegmentPlan] = None
        self._seg_adapter: Optional[torch.Tensor] = None

    def update(self, blen: Optional[BatchLenInfo] = None, lora_ids: Optional[List[int]] = None,
               lora_len: Optional[torch.Tensor] = None, segment: Optional[torch.Tensor] = None,
               train_idx: Sequence[int] = ()):
        self._blen = blen
        self._lora_ids = lora_ids
        self._lora_len = lora_len
        self._segment = segment
        self._train_idx = list(train_idx)
        self._plan = None
        self._seg_adapter = None

    @property
    def blen(self) -> Optional[BatchLenInfo]:
        return self._blen

    @property
    def lora_ids(self) -> Optional[List[int]]:
        return self._lora_ids

    @property
    def lora_len(self) -> Optional[torch.Tensor]:
        return self._lora_len

    @property
    def segment(self) -> Optional[torch.Tensor]:
        return self._segment

    @property
    def train_idx(self) -> List[int]:
        return self._train_idx

    def seg_adapter(self, device: torch.device) -> torch.Tensor:
        """Adapter id of every segment as a device tensor.  `lora_ids` may already be one (int32,
        e.g. from segments.build_segments_device, whose arrays keep the request count as capacity
        and describe empty segments past the real ones): it is then used as it is, and the fused
        path never brings the ids to the host."""
        if self._seg_adapter is None or self._seg_adapter.device != device:
            if isinstance(self._lora_ids, torch.Tensor):
                self._seg_adapter = self._lora_ids.to(device=device, dtype=torch.int32)
            else:
                self._seg_adapter = torch.tensor(self._lora_ids, dtype=torch.int32, device=device)
        return self._seg_adapter

    def plan(self, device: torch.device, T: int) -> kernel.SegmentPlan:
        if self._plan is None or self._plan.T != T or self._plan.buf.device != device:
            self._plan = kernel.SegmentPlan(self._segment.to(device), self.seg_adapter(device), T)
        return self._plan


@dataclass
class NamedLoraLayer:
    adapter_name: str
    wa: torch.Tensor  # [rank, h_in]
    wb: torch.Tensor  # [h_out, rank]
    dropout: Union[nn.Dropout, nn.Identity]
    scaling: Optional[float] = None
    # Rank of the adapter before prepare_weight padded it to the layer's rank (None: the layer's
    # rank).  Not in the reference's record; with it the fused kernels skip the zero padding.
    true_rank: Optional[int] = None


def prepare_weight(weight: torch.Tensor, rank: int, dtype: torch.dtype, device, rank_dim: int = 0,
                   scaling: Optional[float] = None) -> torch.Tensor:
    """Cast, optionally pre-scale, and zero-pad a LoRA weight to the layer rank
    (reference: MixedLoraModel._prepare_weight, mixed_lora.py:501-521)."""
    weight = weight.detach()
    if weight.size(rank_dim) == rank:
        w = weight if scaling is None else weight * scaling
        return w.to(dtype=dtype, device=device).contiguous()
    new_size = list(weight.size())
    new_size[rank_dim] = rank
    new_weight = torch.zeros(new_size, dtype=dtype, device=device)
    src = weight if scaling is None else weight * scaling
    new_weight[: weight.size(0), : weight.size(1)].copy_(src, non_blocking=True)
    return new_weight


class fused_add_lora(Function):
    """result <- result + scale_seg * (x A_seg^T) B_seg^T, in place, one call.

    Arguments: (result, x, wa_table, wb_table, seg_scale, plan, lora_rank,
    train_len, train_partition, dropout, adapter_rank, *weights); the tables hold
    one address per adapter and the plan is keyed by adapter id.  `adapter_rank`
    (None, or a pair of int32 device tensors: the true rank of every adapter, and
    of the training adapters in order of first appearance among the partitions)
    tells the kernels which adapters are stored zero-padded.  `dropout` (a
    kernel.DropoutSpec or None) drops the training rows of x inside the kernels,
    in place of the reference's nn.Dropout calls and torch.cat before the op
    (src/loquetier_src/models/mixed_lora.py:185-192); x is the tensor before
    dropout.  Returns `result`.
    Gradients: result -> passed through, x -> dX on train rows (zero elsewhere),
    each trainable weight -> its summed gradient (None when not training)."""

    @staticmethod
    def forward(ctx: FunctionCtx, result, x, wa_table, wb_table, seg_scale, plan, lora_rank,
                train_len, train_partition, dropout, adapter_rank, *weights):
        need_v = len(weights) > 0 and train_len > 0
        adapter_rank, train_rank = adapter_rank if adapter_rank is not None else (None, None)
        v = torch.empty((x.size(0), lora_rank), dtype=x.dtype, device=x.device) if need_v else None
        if dropout is not None and need_v and dropout.mask_bits is None:
            # the backward reads the forward's keep bits (1/16 of x's bytes) instead of making them again
            bits = torch.empty(kernel.DropoutSpec.mask_nbytes(dropout.rows, x.size(1)), dtype=torch.uint8,
                               device=x.device)
            dropout = kernel.DropoutSpec(dropout.seg_p, dropout.rows, dropout.seed, dropout.offset, bits)
        kernel.smlm_lora_forward(result, x, wa_table, wb_table, plan, lora_rank, seg_scale=seg_scale,
                                 beta=1.0, v_out=v, dropout=dropout, adapter_rank=adapter_rank)
        ctx.mark_dirty(result)
        ctx.tp = train_partition
        ctx.rank = lora_rank
        ctx.has_v = v is not None
        ctx.n_parts = len(weights) // 2
        # scale of each train partition = scale of the segment that starts it;
        # kept as a device gather so nothing is read back to the host
        ctx.part_scale = None
        ctx.part_drop = None
        ctx.train_rank = train_rank if need_v else None
        if need_v and (seg_scale is not None or dropout is not None):
            starts = torch.tensor([int(t) for t in train_partition][: ctx.n_parts],
                                  dtype=torch.int32, device=x.device)
            seg_of = (torch.searchsorted(plan.segment, starts, right=True) - 1).clamp_(0, plan.S - 1)
            if seg_scale is not None:
                ctx.part_scale = seg_scale[seg_of].contiguous()
            if dropout is not None:  # the same stream, probabilities by train partition
                ctx.part_drop = kernel.DropoutSpec(dropout.seg_p[seg_of].contiguous(), train_len,
                                                   dropout.seed, dropout.offset, dropout.mask_bits)
        if need_v:
            ctx.save_for_backward(x[:train_len, ...], v[:train_len, ...], *weights)
        return result

    @staticmethod
    def backward(ctx: FunctionCtx, grad_output: torch.Tensor):
        n_fixed = 11
        if not ctx.has_v:
            return (grad_output, None) + (None,) * (n_fixed - 2) + (None,) * (2 * ctx.n_parts)
        x, v, *weight_list = ctx.saved_tensors
        grad_x, grads = lora_backward(grad_output, x, v, weight_list, ctx.tp, ctx.rank,
                                      part_scale=ctx.part_scale, dropout=ctx.part_drop,
                                      adapter_rank=ctx.train_rank)
        return (grad_output, grad_x) + (None,) * (n_fixed - 2) + tuple(grads)


class MixedLoraLinear(nn.Module):
    """A linear layer plus the LoRA terms of every resident adapter
    (reference: mixed_lora.py:86-218)."""

    def __init__(self, root_context: MixedLoraContext, base_layer: Any, adapters: List[NamedLoraLayer],
                 rank: int, dtype: torch.dtype, is_scaled: bool = False, fused: bool = True):
        super().__init__()
        self.root_context = root_context
        self.base_layer = base_layer
        self.device = base_layer.weight.device
        self.dtype = dtype
        self.is_scaled = is_scaled
        self.fused = fused
        self.scaling = None
        self.update_adapters(adapters, rank)

    def _ptrs(self, tensors) -> torch.Tensor:
        return torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64, device=self.device)

    def update_adapters(self, adapters: List[NamedLoraLayer], rank: int):
        self.adapters = adapters
        self.rank = rank
        self.wa_ptrs = self._ptrs([a.wa for a in adapters])
        self.wb_ptrs = self._ptrs([a.wb for a in adapters])
        if not self.is_scaled:
            self.scaling = torch.tensor([a.scaling for a in adapters], dtype=self.dtype,
                                        device=self.device)
        ranks = [rank if a.true_rank is None else min(int(a.true_rank), rank) for a in adapters]
        self.adapter_rank = (torch.tensor(ranks, dtype=torch.int32, device=self.device)
                             if any(q < rank for q in ranks) else None)
        self._train_rank_key, self._train_rank = None, None

    def _rank_args(self, train_idx):
        """(ranks of all adapters, ranks of the training adapters in order of first appearance),
        or None when every adapter has the layer's rank."""
        if self.adapter_rank is None:
            return None
        order = list(dict.fromkeys(int(i) for i in train_idx))
        key = tuple(order)
        if self._train_rank_key != key:
            self._train_rank_key = key
            self._train_rank = (self.adapter_rank[torch.tensor(order, dtype=torch.long, device=self.device)]
                                if order else None)
        return self.adapter_rank, self._train_rank

    def add_adapter(self, adapter: NamedLoraLayer):
        """New adapter must have the rank of the existing ones."""
        self.update_adapters(self.adapters + [adapter], self.rank)

    def del_adapter(self, adapter_idx: int):
        assert adapter_idx < len(self.adapters)
        adapters = list(self.adapters)
        del adapters[adapter_idx]
        self.update_adapters(adapters, self.rank)

    def set_trainable(self, train_idx: List[int]):
        for idx in train_idx:
            self.register_parameter(f"lora-{idx}-A", nn.Parameter(self.adapters[idx].wa))
            self.register_parameter(f"lora-{idx}-B", nn.Parameter(self.adapters[idx].wb))

    def forward(self, x: torch.Tensor, *args: Any, **kwargs: Any) -> torch.Tensor:
        result = self.base_layer(x, *args, **kwargs)
        torch_result_dtype = result.dtype
        ctx = self.root_context
        blen = ctx.blen
        lora_ids = ctx.lora_ids
        train_idx = ctx.train_idx

        x = x.to(self.dtype)
        drop_spec = None
        if blen.tlen > 0 and self.fused:
            # the kernels drop the training rows themselves: no dropped copy, no torch.cat
            probs = [float(a.dropout.p) if isinstance(a.dropout, nn.Dropout) and a.dropout.training else 0.0
                     for a in self.adapters]
            if any(probs[idx] > 0.0 for idx in train_idx):
                seg_p = torch.tensor(probs, dtype=torch.float32, device=self.device)[
                    ctx.seg_adapter(self.device).long()]
                # the stream: torch's seed, and an offset drawn from torch's generator so that every
                # call (layer, step) gets its own mask and torch.manual_seed makes runs repeatable
                offset = int(torch.randint(0, 2 ** 62, (1,)).item())
                drop_spec = kernel.DropoutSpec(seg_p, blen.tlen, torch.initial_seed(), offset)
        elif blen.tlen > 0:
            dropped_x = []
            for idx, pi in zip(train_idx, range(len(blen.train_partition) - 1)):
                start, end = blen.train_partition[pi], blen.train_partition[pi + 1]
                dropped_x.append(self.adapters[idx].dropout(x[start:end, :]))
            x = torch.cat(dropped_x + [x[blen.tlen:, :]])
        weights = [w for idx in train_idx for w in (self.get_parameter(f"lora-{idx}-A"),
                                                    self.get_parameter(f"lora-{idx}-B"))]
        if self.fused:
            seg_adapter = ctx.seg_adapter(self.device)
            seg_scale = None if self.is_scaled else self.scaling.float()[seg_adapter.long()]
            result = result.to(self.dtype).contiguous()
            if not x.is_contiguous():
                x = x.contiguous()
            result = fused_add_lora.apply(result, x, self.wa_ptrs, self.wb_ptrs, seg_scale,
                                          ctx.plan(self.device, x.size(0)), self.rank, blen.tlen,
                                          blen.train_partition, drop_spec, self._rank_args(train_idx), *weights)
            return result.to(torch_result_dtype)

        segment = ctx.segment.to(self.device)
        wa_ptr, wb_ptr = self.wa_ptrs[lora_ids], self.wb_ptrs[lora_ids]
        lora_res = add_lora.apply(result.shape, x, wa_ptr, wb_ptr, segment, self.rank, blen.tlen,
                                  blen.train_partition, *weights)
        if not self.is_scaled:
            lora_res = lora_res * torch.repeat_interleave(self.scaling[lora_ids],
                                                          ctx.lora_len).unsqueeze(-1)
        result = result + lora_res
        return result.to(torch_result_dtype)
