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

from contextlib import contextmanager
from dataclasses import dataclass
from typing import Any, List, Optional, Sequence, Union

import torch
from torch import nn
from torch.autograd.function import Function, FunctionCtx

from .kernel_utils import BatchLenInfo, add_lora, lora_backward
from .ops import _kernels as kernel


class MixedLoraContext:
    """Per-step routing record shared by every LoRA linear of a model
    (reference: mixed_lora.py:24-64).  Everything that depends only on the step's
    routing is built here ONCE per `update` and shared by all layers: the device
    copy of the adapter ids, the tile plan of the forward, the partition plan of
    the backward, the partition -> segment map.  The context also owns the scratch
    memory the kernels use, so that no layer allocates or copies anything from the
    host inside the layer loop."""

    def __init__(self):
        self._blen = None
        self._lora_ids = None
        self._lora_len = None
        self._segment = None
        self._train_idx: List[int] = []
        self._train_key: tuple = ()
        self._train_order: Optional[List[int]] = None
        self._plan: Optional[kernel.SegmentPlan] = None
        self._seg_adapter: Optional[torch.Tensor] = None
        self._step: dict = {}          # per-step memo, dropped by update()
        self._workspaces: dict = {}    # device -> kernel.Workspace, kept across steps
        self._dropout_calls = 0        # host-side counter: every dropout call gets its own mask stream
        self._dropout_salt: Optional[int] = None  # drawn from torch's CPU generator at the first dropout call

    def update(self, blen: Optional[BatchLenInfo] = None, lora_ids: Optional[List[int]] = None,
               lora_len: Optional[torch.Tensor] = None, segment: Optional[torch.Tensor] = None,
               train_idx: Sequence[int] = ()):
        self._blen = blen
        self._lora_ids = lora_ids
        self._lora_len = lora_len
        self._segment = segment
        open_group = self._step.get("open_group")
        if open_group is not None:   # a deferred group whose last member was never called: its adds happen now
            open_group["group"].flush(open_group)
        self._train_idx = list(train_idx)
        self._train_key = tuple(self._train_idx)   # (what the layers key their per-training-set tables on)
        self._train_order = None
        self._plan = None
        self._seg_adapter = None
        self._step = {}

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

    @property
    def train_key(self) -> tuple:
        """train_idx as a tuple, made once per update."""
        return self._train_key

    def memo(self, key, build):
        """Value built once per step (per `update`) and shared by every layer that asks for `key`."""
        if key not in self._step:
            self._step[key] = build()
        return self._step[key]

    def workspace(self, device: torch.device) -> "kernel.Workspace":
        """Scratch memory of the kernels, owned by the context (grow-only; size it with one eager
        step before capturing a graph)."""
        ws = self._workspaces.get(device)
        if ws is None:
            ws = self._workspaces[device] = kernel.Workspace(device)
        return ws

    def group_workspace(self, device: torch.device) -> "kernel.Workspace":
        """Scratch memory that holds the shrink results of ONE open projection group (ProjectionGroup)
        between the group's members' calls; apart from `workspace`, which any layer call overwrites."""
        ws = self._workspaces.get(("group", device))
        if ws is None:
            ws = self._workspaces[("group", device)] = kernel.Workspace(device)
        return ws

    def next_dropout_offset(self) -> int:
        """Offset of the next dropout mask stream: a per-context salt plus a host-side counter (eight
        projections' worth of offsets apart), so drawing it waits for nothing on the device.  The salt
        is drawn ONCE, at the context's first dropout call, from torch's CPU generator: two contexts of
        one process get different masks, and `torch.manual_seed(s)` followed by the same sequence of
        calls on a fresh context repeats a run.  A run that is resumed, or re-seeded without a fresh
        context, continues the sequence where `dropout_state()` says; hand that to
        `set_dropout_state` to repeat from there."""
        if self._dropout_salt is None:
            self._dropout_salt = int(torch.randint(0, 1 << 40, (1,), dtype=torch.int64).item()) << 20
        self._dropout_calls += 1
        return self._dropout_salt + self._dropout_calls * 8

    def dropout_state(self):
        """(salt, calls made): what a trainer checkpoints beside torch's seed to repeat the masks."""
        return self._dropout_salt, self._dropout_calls

    def set_dropout_state(self, state) -> None:
        self._dropout_salt, self._dropout_calls = (None if state[0] is None else int(state[0])), int(state[1])

    def check_adapter_ids(self, n_adapters: int) -> None:
        """Adapter ids handed over as a host list must index the layer's adapters (negative: a segment no
        adapter serves).  Ids that only exist on the device cannot be looked at without waiting for it: the
        kernels skip segments whose id is not below the table length.  Checked once per step and table length."""
        if isinstance(self._lora_ids, torch.Tensor) or self._lora_ids is None:
            return

        def check():
            top = max((int(i) for i in self._lora_ids), default=-1)
            if top >= n_adapters:
                raise IndexError(f"adapter id {top} in lora_ids, but the layer holds {n_adapters} adapters")
            return True
        self.memo(("ids_ok", n_adapters), check)

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

    def seg_adapter_long(self, device: torch.device) -> torch.Tensor:
        return self.memo(("seg_adapter_long", device), lambda: self.seg_adapter(device).long())

    def plan(self, device: torch.device, T: int) -> kernel.SegmentPlan:
        if self._plan is None or self._plan.T != T or self._plan.buf.device != device:
            # deferred: the step's first fused forward builds the plan (decode batches inside its
            # shrink launch), any other first user builds it with the plan launch
            self._plan = kernel.SegmentPlan(self._segment.to(device), self.seg_adapter(device), T, defer=True)
        return self._plan

    def train_order(self) -> List[int]:
        """Training adapters in order of first appearance among the train partitions: the backward
        numbers them 0..NA-1 in this order."""
        if self._train_order is None:
            self._train_order = list(dict.fromkeys(int(i) for i in self._train_idx))
        return self._train_order

    def backward_tables(self, device: torch.device):
        """(partition plan, partition -> training adapter list) of the step's backward: a function
        of the train partitions and their adapters only, so one serves every layer."""
        def build():
            tp = [int(t) for t in self._blen.train_partition]
            n_parts = min(len(self._train_idx), len(tp) - 1)
            tp = tp[: n_parts + 1]
            order = self.train_order()
            part_adapter = [order.index(int(i)) for i in self._train_idx[:n_parts]]
            if n_parts == 0 or tp[-1] == 0:
                return None, part_adapter
            plan = kernel.SegmentPlan(torch.tensor(tp, dtype=torch.int32, device=device),
                                      torch.tensor(part_adapter, dtype=torch.int32, device=device), tp[-1],
                                      defer=True)  # built by the step's first backward call
            return plan, part_adapter
        return self.memo(("backward", device), build)

    def part_segments(self, device: torch.device, plan: kernel.SegmentPlan) -> torch.Tensor:
        """Segment that starts every train partition (int64 device indices): the partition's scale
        and dropout probability are those of that segment."""
        def build():
            n_parts = min(len(self._train_idx), len(self._blen.train_partition) - 1)
            starts = torch.tensor([int(t) for t in self._blen.train_partition][:n_parts],
                                  dtype=torch.int32, device=device)
            return (torch.searchsorted(plan.segment, starts, right=True) - 1).clamp_(0, max(plan.S - 1, 0))
        return self.memo(("part_segments", device), build)

    def train_bundle(self, device: torch.device, plan: kernel.SegmentPlan):
        """(training adapters in order, backward plan, partition -> training adapter, partition -> segment):
        what a training layer call needs of the step beyond the forward's plan, in one look-up."""
        def build():
            bwd_plan, part_adapter = self.backward_tables(device)
            return self.train_order(), bwd_plan, part_adapter, self.part_segments(device, plan)
        return self.memo(("train_bundle", device), build)


# Adapter whose parameters a state_dict() call saves (reference: CURRENT_TRAINER_LORA_ID and
# set_saving_lora_id, mixed_lora.py:66-76).
CURRENT_TRAINER_LORA_ID = 0


@contextmanager
def set_saving_lora_id(num: int):
    """Within the block, state_dict() of every MixedLoraLinear saves adapter `num`."""
    global CURRENT_TRAINER_LORA_ID
    original_lora_id = CURRENT_TRAINER_LORA_ID
    CURRENT_TRAINER_LORA_ID = num
    try:
        yield
    finally:
        CURRENT_TRAINER_LORA_ID = original_lora_id


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
                   scaling: Optional[float] = None, pack: bool = False) -> torch.Tensor:
    """Cast, optionally pre-scale, and zero-pad a LoRA weight to the layer rank
    (reference: MixedLoraModel._prepare_weight, mixed_lora.py:501-521).

    pack=True pads only to the next multiple of 8 instead of the layer rank: the adapter is then
    stored at its own rank (A [r_a, h_in], B [h_out, r_a]) and the fused kernels read it so
    (`packed_ranks`); results are those of the padded storage, bit for bit."""
    weight = weight.detach()
    target = min(rank, (weight.size(rank_dim) + 7) // 8 * 8) if pack else rank
    if weight.size(rank_dim) == target:
        w = weight if scaling is None else weight * scaling
        return w.to(dtype=dtype, device=device).contiguous()
    new_size = list(weight.size())
    new_size[rank_dim] = target
    new_weight = torch.zeros(new_size, dtype=dtype, device=device)
    src = weight if scaling is None else weight * scaling
    new_weight[: weight.size(0), : weight.size(1)].copy_(src, non_blocking=True)
    return new_weight


class fused_add_lora(Function):
    """result <- result + scale_seg * (x A_seg^T) B_seg^T, in place, one call.

    Arguments: (result, x, call, *weights).  `call` (a LayerStep) names everything that is not
    differentiated, so that autograd has three arguments to look at besides the weights: the tables
    (one address per adapter; the plan is keyed by adapter id), the per-segment scale, the plan, the
    rank, the training rows and partitions, `adapter_rank` (None, or a pair of int32 device tensors:
    the true rank of every adapter, and of the training adapters in order of first appearance among
    the partitions; tells the kernels which adapters are stored zero-padded), `dropout` (a
    kernel.DropoutSpec or None: drops the training rows of x inside the kernels, in place of the
    reference's nn.Dropout calls and torch.cat before the op,
    src/loquetier_src/models/mixed_lora.py:185-192; x is the tensor before dropout), and what the
    step's context and the layer have prepared once: scratch memory, the backward's plan and pointer
    tables.  Returns `result`.
    Gradients: result -> passed through, x -> dX on train rows (zero elsewhere),
    each trainable weight -> its summed gradient (None when not training)."""

    @staticmethod
    def forward(ctx: FunctionCtx, result, x, step, *weights):
        wa_table, wb_table, seg_scale, plan, lora_rank = step.wa_table, step.wb_table, step.seg_scale, step.plan, step.rank
        train_len, train_partition, dropout = step.train_len, step.train_partition, step.dropout
        need_v = len(weights) > 0 and train_len > 0
        adapter_rank, train_rank = step.adapter_rank if step.adapter_rank is not None else (None, None)
        v = torch.empty((x.size(0), lora_rank), dtype=x.dtype, device=x.device) if need_v else None
        if dropout is not None and need_v and dropout.mask_bits is None:
            # the backward reads the forward's keep bits (1/16 of x's bytes) instead of making them again
            bits = torch.empty(kernel.DropoutSpec.mask_nbytes(dropout.rows, x.size(1)), dtype=torch.uint8,
                               device=x.device)
            dropout = kernel.DropoutSpec(dropout.seg_p, dropout.rows, dropout.seed, dropout.offset, bits)
        kernel.smlm_lora_forward(result, x, wa_table, wb_table, plan, lora_rank, seg_scale=seg_scale,
                                 beta=1.0, v_out=v, dropout=dropout, adapter_rank=adapter_rank,
                                 workspace=step.workspace, packed_ranks=step.packed, cache=step.cache)
        ctx.mark_dirty(result)
        ctx.tp = train_partition
        ctx.rank = lora_rank
        ctx.has_v = v is not None
        ctx.n_parts = len(weights) // 2
        ctx.step = step
        # scale of each train partition = scale of the segment that starts it;
        # kept as a device gather so nothing is read back to the host
        ctx.part_scale = None
        ctx.part_drop = None
        ctx.train_rank = train_rank if need_v else None
        if need_v and (seg_scale is not None or dropout is not None):
            seg_of = step.part_segments
            if seg_of is None:
                starts = torch.tensor([int(t) for t in train_partition][: ctx.n_parts],
                                      dtype=torch.int32, device=x.device)
                seg_of = (torch.searchsorted(plan.segment, starts, right=True) - 1).clamp_(0, plan.S - 1)
                gather = lambda t: t[seg_of].contiguous()
            else:  # (gathers of one step's tensors are shared by the layers that use the same tensors)
                gather = lambda t: step.gather(t, seg_of)
            if seg_scale is not None:
                ctx.part_scale = gather(seg_scale)
            if dropout is not None:  # the same stream, probabilities by train partition
                ctx.part_drop = kernel.DropoutSpec(gather(dropout.seg_p), train_len,
                                                   dropout.seed, dropout.offset, dropout.mask_bits)
        if need_v:
            ctx.save_for_backward(x, v, *weights)  # (whole: the backward reads the plan's rows of them)
        return result

    @staticmethod
    def backward(ctx: FunctionCtx, grad_output: torch.Tensor):
        n_fixed = 3
        if not ctx.has_v:
            return (grad_output, None) + (None,) * (n_fixed - 2) + (None,) * (2 * ctx.n_parts)
        x, v, *weight_list = ctx.saved_tensors
        grad_x, grads = lora_backward(grad_output, x, v, weight_list, ctx.tp, ctx.rank,
                                      part_scale=ctx.part_scale, dropout=ctx.part_drop,
                                      adapter_rank=ctx.train_rank, step=ctx.step)
        return (grad_output, grad_x) + (None,) * (n_fixed - 2) + tuple(grads)


class LayerStep:
    """What one layer call hands to the operator besides the tensors it differentiates: the call's own
    arguments, and what was prepared once per step by the context (shared by all layers) or once per
    adapter set by the layer, never inside the call."""
    __slots__ = ("workspace", "memo", "packed", "cache", "wa_table", "wb_table", "seg_scale", "plan", "rank",
                 "train_len", "train_partition", "dropout", "adapter_rank", "part_segments", "bwd_plan",
                 "part_adapter", "a_tab", "b_tab", "grad_layout")

    def __init__(self, workspace, memo=None, packed=False, cache=None):
        self.workspace = workspace      # kernel.Workspace owned by the context
        self.memo = memo                # the context's per-step memo (MixedLoraContext.memo)
        self.packed = packed            # the adapters are stored at their true ranks
        self.cache = cache              # the layer's checked operator calls (kernel.smlm_lora_forward_multi)
        # the call: pointer tables by adapter, per-segment scale, plan, rank, training rows and partitions,
        # dropout descriptor, (ranks of all adapters, ranks of the training adapters) or None
        self.wa_table = self.wb_table = self.seg_scale = self.plan = self.dropout = self.adapter_rank = None
        self.rank = self.train_len = 0
        self.train_partition = ()
        self.part_segments = None       # segment that starts every train partition
        self.bwd_plan = None            # kernel.SegmentPlan over the train partitions
        self.part_adapter = None        # training-adapter index of every partition
        self.a_tab = self.b_tab = None  # addresses of the training adapters' A / B, in order
        # where the gradients go (MixedLoraLinear._train_tables): byte offsets of dA_0.., dB_0.. inside one buffer
        # (grad_offsets) or inside one buffer for the dA and one for the dB (grad_offsets_a / _b, when the matrices
        # have one shape: grad_uniform), [(offset in elements, shape)] in the same order (grad_shapes, grad_numel),
        # and the device tables of the gradients' addresses by buffer address (grad_tabs)
        self.grad_layout = None

    def gather(self, table: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
        """table[index], computed once per step for a given pair of tensors."""
        build = lambda: table[index].contiguous()
        return build() if self.memo is None else self.memo(("gather", id(table), id(index)), build)


class ProjectionGroup:
    """Layers that read the SAME input tensor in one pass -- q/k/v of an attention block, gate/up of
    an MLP.  In a serving step (no training rows) the first member to be called shrinks the input for
    all of them in one launch (three projections cost little more than one there: the launch is
    mostly fixed cost), and every member then expands only its own projection onto its base layer's
    output.  Results are those of the ungrouped calls, bit for bit.  No counterpart in the reference,
    whose layers each run both GEMMs themselves (mixed_lora.py:198-205).

    The members must be fused layers of one rank, dtype, device and set of true ranks, and must be
    handed the same tensor object (same storage, not modified in between); a member that is called
    with anything else, or twice, or after another group has started its pass, simply shrinks
    again -- grouping never changes a result.  Call ProjectionGroup([q, k, v]) once after the layers
    are built.

    deferred=True also gives the members ONE expand launch: a member's call returns its base layer's
    output with the LoRA term still missing, and the call of the group's last member adds the terms
    of all of them, in place.  The values are the same, but they are complete only once every member
    has been called: use it only where nothing reads a member's output before the last member's call
    returns -- the reference's attention does (q, k and v are projected one after the other,
    models/mixed_llama.py:113-115), its MLP does not (the activation reads gate's output before up is
    called, mixed_llama.py:77).  A pass that is cut short (another group or another input starts, or
    the context's next update arrives) adds what it still owes at that point.  A member whose call
    cannot hand out the very tensor the expand writes (its base layer's output is of another dtype)
    is expanded at once."""

    def __init__(self, layers, deferred: bool = False):
        self.layers = list(layers)
        self.deferred = deferred
        first = self.layers[0]
        for l in self.layers:
            if not (l.fused and l.rank == first.rank and l.dtype == first.dtype and l.device == first.device
                    and l.packed == first.packed and l.root_context is first.root_context):
                raise ValueError("the layers of a group must be fused layers of one context, rank, dtype and device")
            ra, rb = l.adapter_rank, first.adapter_rank
            if (ra is None) != (rb is None) or (ra is not None and not torch.equal(ra, rb)):
                raise ValueError("the layers of a group must hold adapters of the same true ranks")
        self.suspended = False  # set while the members' adapter sets disagree (one of them was changed alone)
        self._call_cache: dict = {}  # argument blocks of the group's operator calls that have been checked once
        for i, l in enumerate(self.layers):
            l._group = (self, i)

    def dims(self):
        return [(l.adapters[0].wa.size(1), l.adapters[0].wb.size(0)) for l in self.layers]

    def _expand(self, ys, seg_scale, plan) -> None:
        first, n = self.layers[0], len(self.layers)
        kernel.smlm_lora_forward_multi(ys, [None] * n, [l.wa_ptrs for l in self.layers],
                                       [l.wb_ptrs for l in self.layers], plan, first.rank, seg_scale=seg_scale,
                                       beta=1.0, stages=2, adapter_rank=first.adapter_rank,
                                       workspace=first.root_context.group_workspace(first.device),
                                       packed_ranks=first.packed, dims=self.dims(), cache=self._call_cache)

    def flush(self, state) -> None:
        """The expands a deferred pass still owes: one launch per distinct scale tensor (normally one)."""
        waiting, state["waiting"] = state.get("waiting", []), []
        while waiting:
            scale = waiting[0][2]
            ys = [None] * len(self.layers)
            rest = []
            for i, result, sc in waiting:
                if sc is scale and ys[i] is None:
                    ys[i] = result
                else:
                    rest.append((i, result, sc))
            self._expand(ys, scale, state["plan"])
            waiting = rest

    @staticmethod
    def input_key(src: torch.Tensor):
        """What identifies the input of a pass: the tensor the caller handed to the layer (before any
        cast or copy the layer makes of it), its layout and -- where torch keeps one -- its version
        counter.  Inference tensors (torch.inference_mode) have no version counter; they cannot be
        modified in place outside inference mode either, so address and layout are all there is."""
        try:
            version = None if src.is_inference() else src._version
        except RuntimeError:
            version = None
        return (src.data_ptr(), version, tuple(src.shape), tuple(src.stride()), src.dtype)

    def expand_member(self, i: int, result: torch.Tensor, x: torch.Tensor, seg_scale, plan,
                      may_defer: bool = False, src: Optional[torch.Tensor] = None) -> None:
        """result += scale * v_i B^T for member i, shrinking x for the whole group first when this is
        the first member to see x.  may_defer: the caller hands `result` itself on to its own caller,
        so a deferred group may add to it later.  src: the tensor the layer was called with, of which
        x is the contiguous copy in the layer's dtype (None: x itself); the pass is keyed on src, so
        members that are handed one strided or differently typed tensor still share one shrink."""
        first, n = self.layers[0], len(self.layers)
        ctx = first.root_context
        key = self.input_key(x if src is None else src)
        state = ctx._step.get("open_group")
        if state is None or state["group"] is not self or state["key"] != key or i not in state["pending"]:
            if state is not None:
                state["group"].flush(state)
            kernel.smlm_lora_forward_multi([None] * n, [x] * n, [l.wa_ptrs for l in self.layers],
                                           [l.wb_ptrs for l in self.layers], plan, first.rank, stages=1,
                                           adapter_rank=first.adapter_rank,
                                           workspace=ctx.group_workspace(first.device),
                                           packed_ranks=first.packed, dims=self.dims(),
                                           cache=self._call_cache)
            # (the tensors are kept so that their addresses cannot be handed to others while the pass is open)
            state = ctx._step["open_group"] = {"group": self, "key": key, "pending": set(range(n)), "x": x,
                                               "src": src, "plan": plan, "waiting": []}
        state["pending"].discard(i)
        if self.deferred and may_defer:
            state["waiting"].append((i, result, seg_scale))
        else:
            ys = [None] * n
            ys[i] = result
            self._expand(ys, seg_scale, plan)
        if not state["pending"]:
            self.flush(state)
            del ctx._step["open_group"]


class MixedLoraLinear(nn.Module):
    """A linear layer plus the LoRA terms of every resident adapter
    (reference: mixed_lora.py:86-218)."""

    def __init__(self, root_context: MixedLoraContext, base_layer: Any, adapters: List[NamedLoraLayer],
                 rank: int, dtype: torch.dtype, is_scaled: bool = False, fused: bool = True):
        super().__init__()
        self.root_context = root_context
        self._group = None  # (ProjectionGroup, index) once the layer shares its input with siblings
        self.base_layer = base_layer
        self.device = base_layer.weight.device
        self.dtype = dtype
        self.is_scaled = is_scaled
        self.fused = fused
        self.scaling = None
        self.update_adapters(adapters, rank)

    def _ptrs(self, tensors) -> torch.Tensor:
        return torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64, device=self.device)

    def _true_ranks(self, adapters: List[NamedLoraLayer], rank: int):
        """(packed, true rank of every adapter); raises when the set cannot be served.  Touches nothing."""
        # adapters stored at their own rank (prepare_weight(pack=True)): every one must be, consistently
        packed = any(a.wa.size(0) < rank or a.wb.size(1) < rank for a in adapters)
        ranks = []
        for a in adapters:
            stored = a.wa.size(0)
            q = min(int(a.true_rank), rank) if a.true_rank is not None else min(stored, rank)
            if packed and not (stored == a.wb.size(1) == min(rank, (q + 7) // 8 * 8)):
                raise RuntimeError(f"adapter {a.adapter_name}: packed storage needs A [r8, h_in] and B [h_out, r8] "
                                   f"with r8 = true rank rounded up to 8; got {tuple(a.wa.shape)}, {tuple(a.wb.shape)}")
            ranks.append(q)
        if packed and not self.fused:
            raise RuntimeError("adapters stored at their true rank need the fused path")
        return packed, ranks

    def update_adapters(self, adapters: List[NamedLoraLayer], rank: int):
        # everything that can refuse the set comes first: a refused set leaves the layer as it was
        packed, ranks = self._true_ranks(adapters, rank)
        adapter_rank = (torch.tensor(ranks, dtype=torch.int32, device=self.device)
                        if packed or any(q < rank for q in ranks) else None)
        if self._group is not None:  # the members of a projection group hold adapters of the same true ranks
            for other in self._group[0].layers:
                if other is self:
                    continue
                ra = other.adapter_rank
                if other.packed != packed or (ra is None) != (adapter_rank is None) or (
                        ra is not None and not torch.equal(ra, adapter_rank)):
                    # the siblings may be about to get the same change: the group stops sharing until they agree
                    self._group[0].suspended = True
                    break
            else:
                self._group[0].suspended = False
        self.adapters = adapters
        self.rank = rank
        self.packed = packed
        self.adapter_rank = adapter_rank
        self.wa_ptrs = self._ptrs([a.wa for a in adapters])
        self.wb_ptrs = self._ptrs([a.wb for a in adapters])
        if not self.is_scaled:
            self.scaling = torch.tensor([a.scaling for a in adapters], dtype=self.dtype,
                                        device=self.device)
        self._train_rank_key, self._train_rank = None, None
        self._scaling_f32 = None if self.is_scaled else self.scaling.float()
        self._scaling_key = None if self.is_scaled else tuple(float(a.scaling) for a in adapters)
        self._train_tabs: dict = {}   # training-adapter order -> pointer tables and gradient layout
        self._drop_probs: dict = {}   # adapter dropout probabilities -> device tensor
        self._train_weights: dict = {}  # training adapters of a step -> their parameters, A and B in turn
        self._call_cache: dict = {}   # argument blocks of operator calls that have been checked once

    def _train_tables(self, order):
        """Pointer tables of the training adapters' weights and the layout of one buffer holding all
        their gradients; built once per set of training adapters (addresses of the weights are
        stable: the parameters share the adapters' storage)."""
        key = tuple(order)
        tabs = self._train_tabs.get(key)
        if tabs is None:
            idx = torch.tensor(list(order), dtype=torch.long, device=self.device)
            shapes, offsets, off = [], [], 0
            for group in ("wa", "wb"):
                for i in order:
                    w = getattr(self.adapters[i], group)
                    shapes.append((off, tuple(w.shape)))
                    offsets.append(off * w.element_size())
                    off += (w.numel() + 7) // 8 * 8   # every matrix 16-byte aligned
            was = [tuple(self.adapters[i].wa.shape) for i in order]
            wbs = [tuple(self.adapters[i].wb.shape) for i in order]
            # matrices of one shape lie evenly spaced: the gradients are then views taken in one go
            uniform = ((len(order), was[0], wbs[0]) if order and len(set(was)) == 1 and len(set(wbs)) == 1
                       and (was[0][0] * was[0][1]) % 8 == 0 and (wbs[0][0] * wbs[0][1]) % 8 == 0 else None)
            grad_offsets = torch.tensor(offsets, dtype=torch.int64, device=self.device)
            n_ad = len(key)
            tabs = dict(a_tab=self.wa_ptrs[idx].contiguous(), b_tab=self.wb_ptrs[idx].contiguous(),
                        grad_offsets=grad_offsets, grad_shapes=shapes, grad_numel=off, grad_uniform=uniform,
                        # (offsets of the dA inside a buffer of their own, and of the dB likewise)
                        grad_offsets_a=grad_offsets[:n_ad].contiguous(),
                        grad_offsets_b=(grad_offsets[n_ad:] - grad_offsets[n_ad:n_ad + 1]).contiguous(),
                        grad_tabs={})
            self._train_tabs[key] = tabs
        return tabs

    def _seg_dropout(self, ctx, train_idx):
        """Dropout probability of every segment (device float32) or None when no training adapter drops."""
        for idx in train_idx:
            d = self.adapters[idx].dropout
            if isinstance(d, nn.Dropout) and d.training and d.p > 0.0:
                break
        else:
            return None
        probs = tuple(float(a.dropout.p) if isinstance(a.dropout, nn.Dropout) and a.dropout.training else 0.0
                      for a in self.adapters)
        table = self._drop_probs.get(probs)
        if table is None:
            table = self._drop_probs[probs] = torch.tensor(probs, dtype=torch.float32, device=self.device)
        return ctx.memo(("seg_p", probs, self.device), lambda: table[ctx.seg_adapter_long(self.device)])

    def _weights_of(self, train_idx):
        """The parameters of the step's training adapters, A and B in turn (looked up once per set: the
        parameters are registered by set_trainable and stay the same objects)."""
        key = train_idx if isinstance(train_idx, tuple) else tuple(train_idx)
        weights = self._train_weights.get(key)
        if weights is None:
            weights = [w for idx in key for w in (self.get_parameter(f"lora-{idx}-A"),
                                                  self.get_parameter(f"lora-{idx}-B"))]
            if len(self._train_weights) >= 64:
                self._train_weights.clear()
            self._train_weights[key] = weights
        return weights

    def _rank_args(self, train_idx):
        """(ranks of all adapters, ranks of the training adapters in order of first appearance),
        or None when every adapter has the layer's rank."""
        if self.adapter_rank is None:
            return None
        order = list(dict.fromkeys(int(i) for i in train_idx))   # (a no-op on the context's own order)
        key = tuple(order)
        if self._train_rank_key != key:
            self._train_rank_key = key
            self._train_rank = (self.adapter_rank[torch.tensor(order, dtype=torch.long, device=self.device)]
                                if order else None)
        return self.adapter_rank, self._train_rank

    def add_adapter(self, adapter: NamedLoraLayer):
        """New adapter must have the rank of the existing ones.  A set that the layer cannot serve raises
        and leaves the layer and its list as they were."""
        self._true_ranks(self.adapters + [adapter], self.rank)
        self.adapters.append(adapter)   # (in place, as the reference does: the caller may hold the list)
        self.update_adapters(self.adapters, self.rank)

    def del_adapter(self, adapter_idx: int):
        assert adapter_idx < len(self.adapters)
        self._true_ranks(self.adapters[:adapter_idx] + self.adapters[adapter_idx + 1:], self.rank)
        del self.adapters[adapter_idx]
        self.update_adapters(self.adapters, self.rank)

    def set_trainable(self, train_idx: List[int]):
        for idx in train_idx:
            self.register_parameter(f"lora-{idx}-A", nn.Parameter(self.adapters[idx].wa))
            self.register_parameter(f"lora-{idx}-B", nn.Parameter(self.adapters[idx].wb))
        self._train_weights = {}

    def forward(self, x: torch.Tensor, *args: Any, **kwargs: Any) -> torch.Tensor:
        result = self.base_layer(x, *args, **kwargs)
        torch_result_dtype = result.dtype
        ctx = self.root_context
        blen = ctx.blen
        lora_ids = ctx.lora_ids
        train_idx = ctx.train_idx

        x_arg = x  # the tensor the caller handed over (a projection group recognises its input by it)
        if x.dtype != self.dtype:
            x = x.to(self.dtype)
        drop_spec = None
        if blen.tlen > 0 and self.fused:
            # the kernels drop the training rows themselves: no dropped copy, no torch.cat
            seg_p = self._seg_dropout(ctx, train_idx)
            if seg_p is not None:
                # the stream: torch's seed, and an offset from the context's host-side counter, so that
                # every call (layer, step) gets its own mask, torch.manual_seed makes runs repeatable
                # and nothing waits for the device
                drop_spec = kernel.DropoutSpec(seg_p, blen.tlen, torch.initial_seed(), ctx.next_dropout_offset())
        elif blen.tlen > 0:
            dropped_x = []
            for idx, pi in zip(train_idx, range(len(blen.train_partition) - 1)):
                start, end = blen.train_partition[pi], blen.train_partition[pi + 1]
                dropped_x.append(self.adapters[idx].dropout(x[start:end, :]))
            x = torch.cat(dropped_x + [x[blen.tlen:, :]])
        weights = self._weights_of(ctx.train_key)
        if self.fused:
            # per-step tables come from the context (built once for all layers), per-layer ones from
            # the layer (built once per adapter set): nothing is copied from the host in here
            seg_scale = None
            if not self.is_scaled:
                # (layers whose adapters have the same scales share one gather per step)
                seg_scale = ctx.memo(("seg_scale", self._scaling_key, self.device),
                                     lambda: self._scaling_f32[ctx.seg_adapter_long(self.device)])
            if result.dtype != self.dtype:
                result = result.to(self.dtype)
            if not result.is_contiguous():
                result = result.contiguous()
            if not x.is_contiguous():
                x = x.contiguous()
            same_dtype = result.dtype == torch_result_dtype
            ctx.check_adapter_ids(len(self.adapters))
            plan = ctx.plan(self.device, x.size(0))
            if self._group is not None and not self._group[0].suspended and blen.tlen == 0 and not weights and not (
                    torch.is_grad_enabled() and (x.requires_grad or result.requires_grad)):
                # a serving step: the group's members share one shrink launch
                self._group[0].expand_member(self._group[1], result, x, seg_scale, plan,
                                             may_defer=same_dtype, src=x_arg)
                return result if same_dtype else result.to(torch_result_dtype)
            if not weights and drop_spec is None and not (
                    torch.is_grad_enabled() and (x.requires_grad or result.requires_grad)):
                # nothing to differentiate: the operator is called directly, without autograd's bookkeeping
                kernel.smlm_lora_forward(result, x, self.wa_ptrs, self.wb_ptrs, plan, self.rank,
                                         seg_scale=seg_scale, beta=1.0, adapter_rank=self.adapter_rank,
                                         workspace=ctx.workspace(self.device), packed_ranks=self.packed,
                                         cache=self._call_cache)
                return result if same_dtype else result.to(torch_result_dtype)
            step = LayerStep(ctx.workspace(self.device), ctx.memo, self.packed, self._call_cache)
            step.wa_table, step.wb_table, step.seg_scale, step.plan, step.rank = \
                self.wa_ptrs, self.wb_ptrs, seg_scale, plan, self.rank
            step.train_len, step.train_partition, step.dropout = blen.tlen, blen.train_partition, drop_spec
            step.adapter_rank = None if self.adapter_rank is None else self._rank_args(ctx.train_order())
            if weights and blen.tlen > 0:
                order, step.bwd_plan, step.part_adapter, step.part_segments = ctx.train_bundle(self.device, plan)
                tabs = self._train_tables(order)
                step.a_tab, step.b_tab = tabs["a_tab"], tabs["b_tab"]
                step.grad_layout = tabs
            result = fused_add_lora.apply(result, x, step, *weights)
            return result if same_dtype else result.to(torch_result_dtype)

        segment = ctx.segment.to(self.device)
        wa_ptr, wb_ptr = self.wa_ptrs[lora_ids], self.wb_ptrs[lora_ids]
        lora_res = add_lora.apply(result.shape, x, wa_ptr, wb_ptr, segment, self.rank, blen.tlen,
                                  blen.train_partition, *weights)
        if not self.is_scaled:
            lora_res = lora_res * torch.repeat_interleave(self.scaling[lora_ids],
                                                          ctx.lora_len).unsqueeze(-1)
        result = result + lora_res
        return result.to(torch_result_dtype)

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        """LoRA-only state dict of ONE adapter under PEFT's names: the parameters `lora-{idx}-A` /
        `lora-{idx}-B` of the adapter selected with set_saving_lora_id are saved as
        `lora_A.weight` / `lora_B.weight`, other adapters' parameters are left out
        (reference: mixed_lora.py:220-234).  The base layer is a plain attribute, not a
        submodule's parameter of this module, so its weights are saved by whoever owns it."""
        for name, param in self._parameters.items():
            lora_info = name.split('-')
            if len(lora_info) != 3 or param is None:
                continue
            lora_id, a_b = int(lora_info[1]), lora_info[2]
            if lora_id == CURRENT_TRAINER_LORA_ID:
                destination[prefix + 'lora_' + a_b + '.weight'] = param if keep_vars else param.detach()
        for name, buf in self._buffers.items():
            if buf is not None and name not in self._non_persistent_buffers_set:
                destination[prefix + name] = buf if keep_vars else buf.detach()
