#!/usr/bin/env python3
"""Benchmark of the SMLM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg2|cfg3|cfg4|cfg5|rmsnorm]

A step is one pass of the hot path over one synthetic batch: the tile plan is
built from the batch's (segment, adapter-id) arrays, then every projection of
the workload runs the fused LoRA forward (shrink + expand, accumulating in
place into a base-layer output); configs with training rows add the backward
(dX, dA, dB).  The default workload is the decode-heavy batch BASELINE.json's
metric is quoted on (configs[1]); the other configs are selectable for
profiling.  Steps are HIP-graph replays so the GPU, not Python, sets the pace;
consecutive steps use different buffer sets, more than the 256 MB Infinity
Cache holds in total, so weights and activations come from HBM.

Prints one JSON line (see the keys below); `roofline` is for the dominant
kernel measured alone with HIP events on the launch stream, `cpu_baseline` is
the per-segment torch restatement of the reference timed on the host cores.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np

HBM_PEAK_GBPS = 8000.0
METRIC = "SMLM tokens/s + HBM GB/s (% of 8 TB/s), Llama-2-7B shapes, 1 GPU"


def workload(name: str):
    """Shapes and routing of BASELINE.json's configs 2-5 (seeds = config number)."""
    if name in ("cfg2", "cfg2mod", "cfg2one", "cfg2layer"):
        # adapters drawn uniformly (the headline workload) or dealt round-robin, i % 32 (the variant);
        # cfg2one is the headline batch through ONE projection, what a single layer call of the reference issues
        ids = [i % 32 for i in range(256)] if name == "cfg2mod" else np.random.default_rng(2).integers(0, 32, 256).tolist()
        proj = [("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096)]
        w = dict(name=f"{name}: 256 single-token segments over 32 adapters"
                      f"{' dealt round-robin' if name == 'cfg2mod' else ''}, r=16, "
                      f"{'q' if name == 'cfg2one' else 'q/k/v/o'} 4096->4096, "
                      "fp16, forward", dtype="fp16", r=16, NA=32, seg=list(range(257)), ids=ids,
                 proj=proj[:1] if name == "cfg2one" else proj, n_train_parts=0)
        if name == "cfg2layer":
            # as a decoder layer can issue it: q, k, v read ONE input and go out in one call, o (whose input is the
            # attention's output) in a call of its own
            w["name"] = ("cfg2layer: the cfg2 batch as one decoder layer issues it -- q/k/v of one shared input in "
                         "one call, then o in its own call, fp16, forward")
            w["calls"], w["shared_x"] = [[0, 1, 2], [3]], {1: 0, 2: 0}
        return w
    if name == "cfg3":
        return dict(name="cfg3: 4x512 prefill + 64 decode, 16 adapters, r=32, gate/up 4096->11008, "
                         "down 11008->4096, fp16, forward", dtype="fp16", r=32, NA=16,
                    seg=[0, 512, 1024, 1536, 2048] + list(range(2049, 2113)),
                    ids=[i % 16 for i in range(68)],
                    proj=[("gate", 4096, 11008), ("up", 4096, 11008), ("down", 11008, 4096)],
                    n_train_parts=0)
    if name == "cfg4":
        return dict(name="cfg4: 4x1024 training rows (fwd+bwd) + 128 decode, 36 adapters, r=16, "
                         "4096->4096, bf16", dtype="bf16", r=16, NA=36,
                    seg=[0, 1024, 2048, 3072, 4096] + list(range(4097, 4225)),
                    ids=[0, 1, 2, 3] + [4 + i % 32 for i in range(128)],
                    proj=[("h", 4096, 4096)], n_train_parts=4)
    if name == "cfg5":
        rng = np.random.default_rng(5)
        lens = []
        while sum(lens) < 8192:
            lens.append(int(np.clip(rng.geometric(1 / 8), 1, 2048)))
        lens[-1] -= sum(lens) - 8192
        seg = np.concatenate([[0], np.cumsum(lens)]).tolist()
        S = len(lens)
        return dict(name="cfg5: 64 adapters of ranks {8,16,32,64}, geometric segments, 8192 "
                         "rows, Llama-3-8B shapes, bf16, fwd + bwd on first quarter of segments",
                    dtype="bf16", r=64, NA=64, seg=seg, ids=[i % 64 for i in range(S)],
                    proj=[("q", 4096, 4096), ("k", 4096, 1024), ("v", 4096, 1024),
                          ("gate", 4096, 14336), ("up", 4096, 14336), ("down", 14336, 4096)],
                    n_train_parts=S // 4, true_ranks=[8, 16, 32, 64])
    raise SystemExit(f"unknown config {name}")


def adapter_sorted(w):
    """The same requests handed over grouped by adapter (training part and serving part each on
    its own): what a scheduler that batches by adapter would pass.  Neighbouring segments of one
    adapter merge, as the run-length segment builder merges them, so the rows of an adapter are
    one contiguous run instead of many short ones."""
    seg, ids, P = w["seg"], w["ids"], w["n_train_parts"]
    lens = [seg[i + 1] - seg[i] for i in range(len(ids))]

    def group(lo, hi):
        out = {}
        for i in range(lo, hi):
            out[ids[i]] = out.get(ids[i], 0) + lens[i]
        return sorted(out.items())
    train, serve = group(0, P), group(P, len(ids))
    new_ids = [a for a, _ in train + serve]
    new_seg = np.concatenate([[0], np.cumsum([n for _, n in train + serve])]).tolist()
    w = dict(w, seg=new_seg, ids=new_ids, n_train_parts=len(train))
    w["name"] += ", requests grouped by adapter"
    return w


def single_tiles(T: int, r: int) -> bool:
    """Whether the forward of a batch of T rows at rank r runs on single 16-row tiles (the decode route)
    or on tile blocks: the library's rule, loquetier_amd/csrc/smlm_api.hip (tiles_per_wave); only used
    here to say in the output how the step's plan is built."""
    return T < (2048 if r <= 16 else 768 if r <= 32 else 512 if r <= 48 else 128 if r <= 64 else 1024)


def algorithmic_bytes(w, h_in, h_out, accumulate=True, own_x=True):
    """Forward bytes of one projection: x and y once (y read too when accumulating),
    A and B of each distinct active adapter once, v written and read once at I/O width.
    own_x False: the projection reads an input that another projection of the call is charged for."""
    T = w["seg"][-1]
    active = sorted(set(w["ids"]))
    ranks = w.get("true_ranks")
    rsum = sum((ranks[a % 4] if ranks else w["r"]) for a in active)
    vbytes = 0
    for i, a in enumerate(w["ids"]):
        n = w["seg"][i + 1] - w["seg"][i]
        vbytes += 2 * n * (ranks[a % 4] if ranks else w["r"]) * 2
    return (T * h_in * (1 if own_x else 0) + T * h_out * (2 if accumulate else 1)) * 2 + rsum * (h_in + h_out) * 2 + vbytes


def backward_bytes(w, h_in, h_out):
    """dY and x read once, dX written, A/B read and dA/dB written per training adapter, v and dV."""
    P = w["n_train_parts"]
    n = w["seg"][P]
    train = sorted(set(w["ids"][:P]))
    ranks = w.get("true_ranks")
    rsum = sum((ranks[a % 4] if ranks else w["r"]) for a in train)
    return n * (h_out + 2 * h_in) * 2 + 2 * rsum * (h_in + h_out) * 2 + 3 * n * w["r"] * 2


def rmsnorm_bench(args, torch, K):
    """RMSNorm forward + backward on the rows of the fine-tune + serve batch (4224 x 4096, bf16):
    the other native operator of the reference's model (rms_norm_cutlass.cu, kernel_utils.py:149-176).
    A step = forward over all rows + backward over the 4096 training rows."""
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    T, n_train, n, tdt = 4224, 4096, 4096, torch.bfloat16
    fwd_bytes = T * n * 2 * 2 + n * 2 + T * 4
    bwd_bytes = n_train * n * 2 * 3 + n * 2 * 2 + n_train * 4
    R = max(2, math.ceil(640e6 / (T * n * 2 * 2 + n_train * n * 2 * 2)))
    gen = torch.Generator(device="cpu").manual_seed(7)
    sets = []
    for _ in range(R):
        x = torch.randn(T, n, generator=gen).to(dev).to(tdt)
        sets.append(dict(x=x, w=(1 + 0.1 * torch.randn(n, generator=gen)).to(dev).to(tdt), o=torch.empty_like(x),
                         m=torch.empty(T, 1, dtype=torch.float32, device=dev),
                         g=torch.randn(n_train, n, generator=gen).to(dev).to(tdt),
                         dx=torch.empty(n_train, n, dtype=tdt, device=dev), dw=torch.empty(n, dtype=tdt, device=dev)))

    def fwd(s):
        K.rms_norm(s["o"], s["m"], s["x"], s["w"], 1e-5)

    def bwd(s):
        K.rms_norm_backward(s["dx"], s["dw"], s["g"], s["x"][:n_train], s["w"], s["m"][:n_train])

    cap = torch.cuda.Stream()
    with torch.cuda.stream(cap):
        for s_ in sets:
            fwd(s_), bwd(s_)
    torch.cuda.synchronize()

    def graph_of(fn, n_rep):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=cap):
            for i in range(n_rep):
                fn(sets[i % R])
        return g

    def timed(g, reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b)

    g_step = graph_of(lambda s_: (fwd(s_), bwd(s_)), R)
    timed(g_step, max(1, args.warmup // R))
    n_rep = max(1, args.steps // R)
    ms_per_step = timed(g_step, n_rep) / (n_rep * R)
    g_f, g_b = graph_of(fwd, R), graph_of(bwd, R)
    timed(g_f, 2), timed(g_b, 2)
    fwd_us = timed(g_f, 10) * 1e3 / (10 * R)
    bwd_us = timed(g_b, 10) * 1e3 / (10 * R)
    achieved = fwd_bytes / (fwd_us * 1e-6) / 1e9
    cpu = None
    if not args.no_cpu_baseline:
        import numpy as np
        from oracle import smlm_oracle as O
        xs = sets[0]["x"][:64].float().cpu().numpy()
        ws = sets[0]["w"].float().cpu().numpy()
        gs = sets[0]["g"][:64].float().cpu().numpy()
        t0, reps = time.perf_counter(), 0
        while time.perf_counter() - t0 < 10.0:
            _, rms = O.rms_norm_fwd(xs, ws, 1e-5, "bf16")
            O.rms_norm_bwd(gs, xs, ws, rms, "bf16")
            reps += 1
        el = time.perf_counter() - t0
        cpu = dict(value=round(64 * reps / el, 1), unit="tokens/s", cores=1, kind="port",
                   sample=f"{reps} passes of forward + backward over 64 rows x 4096 ({el:.1f} s), "
                          "oracle/rms_norm_oracle.c, scalar C")
    print(json.dumps({
        "metric": "RMSNorm tokens/s + HBM GB/s (% of 8 TB/s), Llama-2-7B hidden size, 1 GPU",
        "value": round(T / (ms_per_step * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": n_rep * R, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "rmsnorm: forward over 4224 rows x 4096 + backward over the 4096 training rows, "
                               "bf16", "buffer_sets_rotated": R, "graph_replay": True},
        "step_algorithmic_bytes": fwd_bytes + bwd_bytes,
        "step_hbm_gbps": round((fwd_bytes + bwd_bytes) / (ms_per_step * 1e-3) / 1e9, 1),
        "roofline": dict(kernel="rms_fwd_kernel", bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBPS,
                         unit="GB/s", frac=round(achieved / HBM_PEAK_GBPS, 4), traffic=None,
                         us_per_launch=round(fwd_us, 3), algorithmic_bytes=fwd_bytes),
        "kernels": {"fwd_us": round(fwd_us, 3), "fwd_gbps": round(achieved, 1), "bwd_us": round(bwd_us, 3),
                    "bwd_gbps": round(bwd_bytes / (bwd_us * 1e-6) / 1e9, 1)},
        "cpu_baseline": cpu}), flush=True)


def model_step_bench(args, torch, K, finetune=True):
    """The path as the reference drives it (src/loquetier_src/models/mixed_lora.py:173-218, 224 LoRA linears
    per model forward): 32 layers x (q, k, v, o, gate, up, down) of Llama-2-7B through MixedLoraLinear(fused=True)
    with ONE MixedLoraContext.update per step.  The base layers hand back preallocated outputs (their GEMMs
    are not part of this path).  Reports, per layer call: host time of an eager step (Python + ctypes + launch),
    GPU time of the same step replayed from a graph, for the decode batch (forward) and, eager only, for the
    fine-tune + serve batch (forward + backward through autograd)."""
    from loquetier_amd.kernel_utils import BatchLenInfo
    from loquetier_amd.mixed_lora import MixedLoraContext, MixedLoraLinear, NamedLoraLayer
    dev = torch.device("cuda:0")
    shapes = [("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
              ("gate", 4096, 11008), ("up", 4096, 11008), ("down", 11008, 4096)]
    n_layers = 32

    class Base(torch.nn.Module):
        """Stands in for the frozen base projection: returns its (preallocated) output."""

        def __init__(self, out):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.empty(1, device=dev), requires_grad=False)
            self.out = out

        def forward(self, x):
            return self.out.detach()  # a fresh tensor object over the same memory: no autograd history

    def build(cfg, trainable):
        w = workload(cfg)
        tdt = torch.float16 if w["dtype"] == "fp16" else torch.bfloat16
        T, r, NA = w["seg"][-1], w["r"], w["NA"]
        gen = torch.Generator(device="cpu").manual_seed(11)
        ctx = MixedLoraContext()
        pool = {h: [torch.randn(T, h, generator=gen).to(dev).to(tdt) for _ in range(8)] for h in (4096, 11008)}
        outs = {h: [torch.randn(T, h, generator=gen).to(dev).to(tdt) for _ in range(8)] for h in (4096, 11008)}
        layers = []
        for li in range(n_layers):
            for pi, (_, hi, ho) in enumerate(shapes):
                A = (torch.randn(NA, r, hi, generator=gen) * hi ** -0.5).to(dev).to(tdt)
                B = (torch.randn(NA, ho, r, generator=gen) * r ** -0.5).to(dev).to(tdt)
                ad = [NamedLoraLayer(f"a{a}", A[a], B[a], torch.nn.Identity(), 2.0) for a in range(NA)]
                k = (li * len(shapes) + pi) % 8
                layer = MixedLoraLinear(ctx, Base(outs[ho][k]), ad, r, tdt, is_scaled=False, fused=True)
                if trainable:
                    layer.set_trainable(trainable)
                layers.append((layer, pool[hi][k]))
        return w, ctx, layers, tdt

    staged = {}

    def update(w, ctx, trainable):
        # what ModelGeneration.generate hands over once per step (model_generation.py:267-283); the index
        # arrays are staged on the device once (a serving loop builds them there, smlm_segments_build)
        P = w["n_train_parts"] if trainable else 0
        key = (w["name"], P)
        if key not in staged:
            lens = [w["seg"][i + 1] - w["seg"][i] for i in range(len(w["ids"]))]
            staged[key] = (BatchLenInfo([(1, n) for n in lens[:P]], [], sum(lens[P:]), [], dev),
                           torch.tensor(w["ids"], dtype=torch.int32, device=dev),
                           torch.tensor(lens, dtype=torch.int32, device=dev),
                           torch.tensor(w["seg"], dtype=torch.int32, device=dev))
        blen, ids_t, lens_t, seg_t = staged[key]
        ctx.update(blen=blen, lora_ids=ids_t, lora_len=lens_t, segment=seg_t, train_idx=w["ids"][:P])

    out = {"metric": "SMLM layer path: per-call time of MixedLoraLinear(fused=True), 224 calls per model step",
           "n_gpus": 1, "data": "synthetic", "config": {"workload": "model-step: 32 layers x q,k,v,o,gate,up,down, "
                                                                 "Llama-2-7B shapes"}}
    # ---- decode batch, forward
    w, ctx, layers, tdt = build("cfg2", [])
    cap = torch.cuda.Stream()

    def measure_decode(layers):
        def fwd_step():
            update(w, ctx, [])
            for layer, x in layers:
                layer(x)
        with torch.no_grad(), torch.cuda.stream(cap):
            for _ in range(3):
                fwd_step()
            torch.cuda.synchronize()
            n_eager = max(1, min(args.steps, 50))
            t0 = time.perf_counter()
            for _ in range(n_eager):
                fwd_step()
            host_us = (time.perf_counter() - t0) * 1e6 / (n_eager * len(layers))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n_eager):
                fwd_step()
            torch.cuda.synchronize()
            eager_us = (time.perf_counter() - t0) * 1e6 / (n_eager * len(layers))
        g = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(g, stream=cap):
            fwd_step()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(2):
            g.replay()
        a.record()
        for _ in range(10):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        return host_us, eager_us, a.elapsed_time(b) * 1e3 / (10 * len(layers))

    host_us, eager_us, graph_us = measure_decode(layers)
    # the same step with q/k/v and gate/up of every layer sharing their input tensor and one shrink
    # launch (ProjectionGroup: not in the reference, whose layers each run both GEMMs)
    from loquetier_amd.mixed_lora import ProjectionGroup
    n_sh = len(shapes)
    grouped = list(layers)
    for li in range(n_layers):
        q, gate = li * n_sh, li * n_sh + 4
        ProjectionGroup([grouped[q + i][0] for i in range(3)])
        ProjectionGroup([grouped[gate + i][0] for i in range(2)])
        for i in (1, 2):
            grouped[q + i] = (grouped[q + i][0], grouped[q][1])
        grouped[gate + 1] = (grouped[gate + 1][0], grouped[gate][1])
    g_host_us, _, g_graph_us = measure_decode(grouped)
    # and with q/k/v also sharing ONE expand launch (deferred=True: the terms of all three are added when
    # v is called, which the reference's attention allows, mixed_llama.py:113-115; gate/up stay as they are,
    # its MLP reads gate's output before it calls up, mixed_llama.py:77)
    for li in range(n_layers):
        ProjectionGroup([grouped[li * n_sh + i][0] for i in range(3)], deferred=True)
    d_host_us, _, d_graph_us = measure_decode(grouped)
    T = w["seg"][-1]
    step_bytes = sum(algorithmic_bytes(w, hi, ho) for _, hi, ho in shapes) * n_layers
    out["decode_forward"] = dict(workload=w["name"], calls_per_step=len(layers), host_us_per_call=round(host_us, 2),
                                 eager_us_per_call=round(eager_us, 2), graph_gpu_us_per_call=round(graph_us, 2),
                                 graph_ms_per_model_step=round(graph_us * len(layers) / 1e3, 4),
                                 step_hbm_gbps=round(step_bytes / (graph_us * len(layers) * 1e-6) / 1e9, 1),
                                 tokens_per_s=round(T / (graph_us * len(layers) * 1e-6), 1),
                                 grouped_qkv_gate_up=dict(host_us_per_call=round(g_host_us, 2),
                                                          graph_gpu_us_per_call=round(g_graph_us, 2),
                                                          graph_ms_per_model_step=round(g_graph_us * len(layers) / 1e3, 4),
                                                          tokens_per_s=round(T / (g_graph_us * len(layers) * 1e-6), 1)),
                                 grouped_qkv_one_expand=dict(host_us_per_call=round(d_host_us, 2),
                                                             graph_gpu_us_per_call=round(d_graph_us, 2),
                                                             graph_ms_per_model_step=round(d_graph_us * len(layers) / 1e3, 4),
                                                             tokens_per_s=round(T / (d_graph_us * len(layers) * 1e-6), 1)))
    del grouped
    del layers
    torch.cuda.empty_cache()
    if not finetune:
        return out

    # ---- fine-tune + serve batch, forward + backward through autograd (eager)
    w, ctx, layers, tdt = build("cfg4", [0, 1, 2, 3])
    n_train = w["seg"][w["n_train_parts"]]
    gen = torch.Generator(device="cpu").manual_seed(12)
    grads = {h: torch.randn(w["seg"][-1], h, generator=gen).to(dev).to(tdt) for h in (4096, 11008)}

    params = [p for layer, _ in layers for p in layer.parameters() if p.requires_grad]

    def train_step(one_engine_run=False):
        for p in params:  # what optimizer.zero_grad() does by default: the backward then hands its buffers over
            p.grad = None
        update(w, ctx, [0, 1, 2, 3])
        outs = []
        for layer, x in layers:
            outs.append(layer(x))  # dX is computed and handed to autograd, which has no use for it here
        t_f = time.perf_counter()
        if one_engine_run:  # as loss.backward() of a model does: autograd's engine starts once for all the layers
            torch.autograd.backward(outs[::-1], [grads[o.size(1)] for o in outs[::-1]])
        else:               # the engine is started (and its device thread woken) once per layer
            for o in reversed(outs):
                o.backward(grads[o.size(1)])
        return t_f

    def timed(one_engine_run, n=7):
        rows = []
        for _ in range(n):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            t_f = train_step(one_engine_run)
            t1 = time.perf_counter()
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            rows.append(((t_f - t0) * 1e6 / len(layers), (t1 - t_f) * 1e6 / len(layers), (t2 - t0) * 1e6 / len(layers)))
        return rows
    med = lambda rows, i: round(float(np.median([r[i] for r in rows])), 2)
    with torch.cuda.stream(cap):
        for _ in range(2 + max(0, min(args.steps, 50) - 5) // 4):  # (more steps on request: copy-trace runs)
            train_step()
            train_step(True)
        per_layer, one_run = timed(False), timed(True)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record(cap)
        train_step(True)
        b.record(cap)
        torch.cuda.synchronize()
    out["finetune_forward_backward"] = dict(
        workload=w["name"], calls_per_step=len(layers), training_rows=n_train,
        timing="median of 7 steps, each started on an idle GPU",
        host_us_per_call_forward=med(per_layer + one_run, 0),
        host_us_per_call_backward=med(one_run, 1),
        host_us_per_call_backward_one_backward_call_per_layer=med(per_layer, 1),
        eager_us_per_call_incl_gpu=med(one_run, 2),
        eager_us_per_call_incl_gpu_one_backward_call_per_layer=med(per_layer, 2),
        event_us_per_call=round(a.elapsed_time(b) * 1e3 / len(layers), 2))
    return out


def reference_surface_bench(args, torch, K):
    """One LoRA layer call of the decode batch through the surface the reference's own code calls, next to the
    fused call: (1) the lines of the reference's add_lora.forward (src/loquetier_src/kernel_utils.py:113-119)
    against this library's `_kernels` module -- three allocations and two smlm_forward_cutlass calls with
    per-segment pointer tables -- followed by the caller's scale multiply and residual add
    (models/mixed_lora.py:214-217); (2) the mirror `add_lora.apply` with the same tensors and the same two
    caller ops; (3) the fused call (scale, residual add and the adapter gather inside the op) over a plan the
    step's layers share.  GPU time per call from graph replays over rotating buffer sets."""
    from loquetier_amd.kernel_utils import add_lora
    dev = torch.device("cuda:0")
    w = workload("cfg2one")
    tdt = torch.float16
    T, S, r, NA = w["seg"][-1], len(w["ids"]), w["r"], w["NA"]
    _, hi, ho = w["proj"][0]
    gen = torch.Generator(device="cpu").manual_seed(21)
    seg_t = torch.tensor(w["seg"], dtype=torch.int32, device=dev)
    ids_t = torch.tensor(w["ids"], dtype=torch.int32, device=dev)
    lens_t = torch.ones(S, dtype=torch.int32, device=dev)
    scaling = torch.full((NA,), 2.0, dtype=tdt, device=dev)
    R = 16
    sets = []
    for _ in range(R):
        A = (torch.randn(NA, r, hi, generator=gen) * hi ** -0.5).to(dev).to(tdt)
        B = (torch.randn(NA, ho, r, generator=gen) * r ** -0.5).to(dev).to(tdt)
        a_tab = torch.tensor([A[a].data_ptr() for a in range(NA)], dtype=torch.int64, device=dev)
        b_tab = torch.tensor([B[a].data_ptr() for a in range(NA)], dtype=torch.int64, device=dev)
        sets.append(dict(x=torch.randn(T, hi, generator=gen).to(dev).to(tdt), base=torch.randn(T, ho, generator=gen).to(dev).to(tdt),
                         A=A, B=B, a_tab=a_tab, b_tab=b_tab, wa_ptr=a_tab[ids_t.long()], wb_ptr=b_tab[ids_t.long()]))
    plan = K.SegmentPlan(seg_t, ids_t, T)
    scale_seg = torch.full((S,), 2.0, device=dev)

    def caller_tail(st, lora_res):  # mixed_lora.py:214-217
        lora_res = lora_res * torch.repeat_interleave(scaling[ids_t.long()], lens_t.long(), output_size=T)[:, None]
        return st["base"] + lora_res

    def two_call(st):
        x, s_, wa_ptr, wb_ptr = st["x"], seg_t, st["wa_ptr"], st["wb_ptr"]
        y = torch.empty((T, ho), dtype=x.dtype, device=x.device)
        tmp = torch.empty((K.smlm_forward_cutlass_tmp_size(s_.size(0) - 1),), dtype=torch.uint8, device=x.device)
        v = torch.empty((x.size(0), r), dtype=x.dtype, device=x.device)
        K.smlm_forward_cutlass(v, x, wa_ptr, s_, tmp, False)
        K.smlm_forward_cutlass(y, v, wb_ptr, s_, tmp, False)
        return caller_tail(st, y)

    def mirror(st):
        return caller_tail(st, add_lora.apply((T, ho), st["x"], st["wa_ptr"], st["wb_ptr"], seg_t, r, 0, []))

    def fused(st):
        K.smlm_lora_forward(st["base"], st["x"], st["a_tab"], st["b_tab"], plan, r, seg_scale=scale_seg, beta=1.0)

    cap = torch.cuda.Stream()

    def per_call_us(fn):
        with torch.no_grad(), torch.cuda.stream(cap):
            for st in sets[:2]:
                fn(st)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(g, stream=cap):
            for _ in range(2):
                for st in sets:
                    fn(st)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(2):
            g.replay()
        a.record()
        for _ in range(10):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / (10 * 2 * R)

    t_two, t_mirror, t_fused = per_call_us(two_call), per_call_us(mirror), per_call_us(fused)
    tmp_t = torch.empty(K.smlm_forward_cutlass_tmp_size(S), dtype=torch.uint8, device=dev)
    for st in sets:
        st["v"], st["y"] = torch.empty(T, r, dtype=tdt, device=dev), torch.empty(T, ho, dtype=tdt, device=dev)

    def two_call_kernels(st):  # the two GEMM calls alone: no allocation, no caller ops
        K.smlm_forward_cutlass(st["v"], st["x"], st["wa_ptr"], seg_t, tmp_t, False)
        K.smlm_forward_cutlass(st["y"], st["v"], st["wb_ptr"], seg_t, tmp_t, False)
    t_two_k = per_call_us(two_call_kernels)
    # the mirror's operator alone (one plan grouped by the (A, B) address pairs, built inside the shrink launch)
    t_mirror_k = per_call_us(lambda st: add_lora.apply((T, ho), st["x"], st["wa_ptr"], st["wb_ptr"], seg_t, r, 0, []))
    # the fused call when it has to build its plan itself, as every call of the reference surface must
    for st in sets:
        st["plan_buf"] = torch.empty(K.SegmentPlan.nbytes(T, S), dtype=torch.uint8, device=dev)

    def fused_own_plan(st):
        K.smlm_lora_forward(st["base"], st["x"], st["a_tab"], st["b_tab"],
                            K.SegmentPlan(seg_t, ids_t, T, buf=st["plan_buf"], defer=True), r,
                            seg_scale=scale_seg, beta=1.0)
    t_fused_own = per_call_us(fused_own_plan)
    nbytes = algorithmic_bytes(w, hi, ho)
    return dict(workload=w["name"] + ", one layer call",
                fused_call_us=round(t_fused, 2),
                reference_lines_two_calls_us=round(t_two, 2),
                reference_lines_two_calls_kernels_only_us=round(t_two_k, 2),
                add_lora_mirror_us=round(t_mirror, 2),
                add_lora_mirror_kernels_only_us=round(t_mirror_k, 2),
                fused_call_building_its_plan_us=round(t_fused_own, 2),
                ratio_two_calls_vs_fused=round(t_two / t_fused, 2),
                ratio_kernels_only_vs_fused=round(t_two_k / t_fused, 2),
                ratio_mirror_vs_fused=round(t_mirror / t_fused, 2),
                ratio_mirror_kernels_only_vs_fused=round(t_mirror_k / t_fused, 2),
                ratio_mirror_kernels_only_vs_fused_building_its_plan=round(t_mirror_k / t_fused_own, 2),
                fused_call_hbm_gbps=round(nbytes / (t_fused * 1e-6) / 1e9, 1),
                note="GPU time per layer call, graph replay over 16 rotating buffer sets; the reference-surface "
                     "legs include the caller's scale multiply and residual add (two more passes over y) unless "
                     "marked kernels only; the fused call reuses the step's plan")


def load_probe():
    """The plain streaming kernels (loquetier_amd/lib/libsmlm_probe.so); None when not built."""
    import ctypes as C
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "loquetier_amd", "lib", "libsmlm_probe.so")
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path)
    lib.smlm_probe_rmw.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p]
    lib.smlm_probe_read.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]
    return lib


def run_workload(args, cfg, torch, K, probe, brief=False):
    """One workload: the whole step, the two forward launches alone, the plain streaming kernels at the
    same launch sizes and the CPU baseline.  brief: fewer side measurements and a short CPU sample (the
    non-headline workloads of the default run)."""
    dev = torch.device("cuda:0")
    w = workload(cfg)
    if args.sorted:
        w = adapter_sorted(w)
    tdt = torch.float16 if w["dtype"] == "fp16" else torch.bfloat16
    T, S, r, NA = w["seg"][-1], len(w["ids"]), w["r"], w["NA"]
    P = w["n_train_parts"]
    n_train = w["seg"][P] if P else 0

    shared_x = w.get("shared_x", {})  # projection -> the projection whose input it reads
    calls = w.get("calls", [list(range(len(w["proj"])))])  # projections issued together, call by call
    fwd_bytes = sum(algorithmic_bytes(w, hi, ho, own_x=i not in shared_x) for i, (_, hi, ho) in enumerate(w["proj"]))
    bwd_bytes = sum(backward_bytes(w, hi, ho) for _, hi, ho in w["proj"]) if P else 0
    footprint = sum((T * (hi + ho) + NA * r * (hi + ho)) * 2 for _, hi, ho in w["proj"])
    if P:
        footprint += sum(n_train * (hi + ho) * 2 for _, hi, ho in w["proj"])
    R = 1 if args.no_rotate else max(2, math.ceil(640e6 / footprint))
    R = min(R, 16)

    gen = torch.Generator(device="cpu").manual_seed(int("".join(ch for ch in cfg if ch.isdigit())))
    seg_t = torch.tensor(w["seg"], dtype=torch.int32, device=dev)
    ids_t = torch.tensor(w["ids"], dtype=torch.int32, device=dev)
    scale_t = torch.full((S,), 2.0, device=dev)

    def randn(*shape, std=1.0):
        return (torch.randn(*shape, generator=gen) * std).to(dev).to(tdt)

    ranks = w.get("true_ranks")
    # adapters below the launch's rank (cfg5) are stored at their own rank unless asked otherwise
    packed = bool(ranks) and not args.padded_ranks and not args.padded_storage
    sets = []
    for _ in range(R):
        projs = []
        for pi, (_, hi, ho) in enumerate(w["proj"]):
            A = randn(NA, r, hi, std=hi ** -0.5)
            B = randn(NA, ho, r, std=r ** -0.5)
            if ranks:  # true rank below the padded rank: zero the padding (mixed_lora.py:501-521)
                for a in range(NA):
                    A[a, ranks[a % 4]:] = 0
                    B[a, :, ranks[a % 4]:] = 0
            Aw, Bw = [A[a] for a in range(NA)], [B[a] for a in range(NA)]
            if packed:  # every adapter stored at its own rank: what prepare_weight(pack=True) produces
                Aw = [A[a, :ranks[a % 4]].contiguous() for a in range(NA)]
                Bw = [B[a, :, :ranks[a % 4]].contiguous() for a in range(NA)]
            d = dict(x=projs[shared_x[pi]]["x"] if pi in shared_x else randn(T, hi), y=randn(T, ho), A=Aw, B=Bw,
                     a_tab=torch.tensor([w_.data_ptr() for w_ in Aw], dtype=torch.int64, device=dev),
                     b_tab=torch.tensor([w_.data_ptr() for w_ in Bw], dtype=torch.int64, device=dev))
            if P:
                train = sorted(set(w["ids"][:P]))
                d.update(g=randn(n_train, ho), dx=torch.empty(n_train, hi, dtype=tdt, device=dev),
                         v=torch.empty(T, r, dtype=tdt, device=dev),
                         dA=[torch.empty_like(Aw[a]) for a in train], dB=[torch.empty_like(Bw[a]) for a in train])
                d["ta_tab"] = torch.tensor([Aw[a].data_ptr() for a in train], dtype=torch.int64, device=dev)
                d["tb_tab"] = torch.tensor([Bw[a].data_ptr() for a in train], dtype=torch.int64, device=dev)
                d["da_tab"] = torch.tensor([t_.data_ptr() for t_ in d["dA"]], dtype=torch.int64, device=dev)
                d["db_tab"] = torch.tensor([t_.data_ptr() for t_ in d["dB"]], dtype=torch.int64, device=dev)
            projs.append(d)
        sets.append(dict(proj=projs,
                         plan_buf=torch.empty(K.SegmentPlan.nbytes(T, S), dtype=torch.uint8, device=dev),
                         bplan_buf=torch.empty(K.SegmentPlan.nbytes(max(n_train, 1), max(P, 1)),
                                               dtype=torch.uint8, device=dev)))
    if P:
        train = sorted(set(w["ids"][:P]))
        part_indptr = torch.tensor(w["seg"][:P + 1], dtype=torch.int32, device=dev)
        part_ad = torch.tensor([train.index(a) for a in w["ids"][:P]], dtype=torch.int32, device=dev)
        part_scale = torch.full((P,), 2.0, device=dev)
    # adapters below the padded rank (cfg5): the kernels are told the true ranks and skip the padding
    rank_f = rank_b = None
    if ranks and not args.padded_ranks:
        rank_f = torch.tensor([ranks[a % 4] for a in range(NA)], dtype=torch.int32, device=dev)
        if P:
            rank_b = torch.tensor([ranks[a % 4] for a in train], dtype=torch.int32, device=dev)
    drop_f = drop_b = None
    if P and args.dropout > 0:
        seg_p = torch.zeros(S, device=dev)
        seg_p[:P] = args.dropout
        # the forward leaves the keep bits of every projection's mask end to end; the backward of
        # projection i reads its part
        widths = [hi for _, hi, _ in w["proj"]]
        bits = torch.empty(K.DropoutSpec.mask_nbytes(n_train, widths), dtype=torch.uint8, device=dev)
        drop_f = K.DropoutSpec(seg_p, n_train, 1, 0, bits)
        starts = [K.DropoutSpec.mask_nbytes(n_train, widths[:i]) for i in range(len(widths))]
        drop_b = [K.DropoutSpec(seg_p[:P].contiguous(), n_train, 1, i, bits[starts[i]:]) for i in range(len(widths))]

    def fwd(st, stages=3):
        for call in calls:
            pr = [st["proj"][i] for i in call]
            K.smlm_lora_forward_multi([d["y"] for d in pr], [d["x"] for d in pr], [d["a_tab"] for d in pr],
                                      [d["b_tab"] for d in pr], st["plan"], r, seg_scale=scale_t, beta=1.0,
                                      v_out=[d["v"] for d in pr] if P else None, stages=stages, dropout=drop_f,
                                      adapter_rank=rank_f, packed_ranks=packed)

    def bwd(st, stages=0):
        # every projection's backward in one set of launches (--bwd-per-projection: a call per projection)
        pr, bplan = st["proj"], st["bplan"]
        if args.bwd_per_projection and not stages:
            for i, d in enumerate(pr):
                K.smlm_lora_backward(d["dx"], d["da_tab"], d["db_tab"], d["g"], d["x"], d["v"],
                                     d["ta_tab"], d["tb_tab"], bplan, r, part_scale,
                                     dropout=drop_b[i] if drop_b else None, adapter_rank=rank_b,
                                     packed_ranks=packed)
            return
        K.smlm_lora_backward_multi([d["dx"] for d in pr], [d["da_tab"] for d in pr], [d["db_tab"] for d in pr],
                                   [d["g"] for d in pr], [d["x"] for d in pr], [d["v"] for d in pr],
                                   [d["ta_tab"] for d in pr], [d["tb_tab"] for d in pr], bplan, r, part_scale,
                                   dropout=drop_b[0] if drop_b else None, adapter_rank=rank_b,
                                   packed_ranks=packed, stages=stages)

    def step(st, build_plan=True):
        if build_plan:
            # deferred: the forward call builds the plan itself -- decode batches inside their
            # shrink launch, the others with the plan launch first (--plan-launch: always that)
            st["plan"] = K.SegmentPlan(seg_t, ids_t, T, buf=st["plan_buf"], defer=not args.plan_launch)
        fwd(st)
        if P:
            if build_plan or "bplan" not in st:
                st["bplan"] = K.SegmentPlan(part_indptr, part_ad, n_train, buf=st["bplan_buf"],
                                            defer=not args.plan_launch)
            bwd(st)

    # eager once on the capture stream (sizes its workspace outside any capture)
    cap_stream = torch.cuda.Stream()
    with torch.cuda.stream(cap_stream):
        for st in sets:
            step(st)
    torch.cuda.synchronize()

    if args.calibration_copy:
        src = torch.empty(128 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    class Eager:
        """Stands in for a captured graph: replay() launches the work directly."""

        def __init__(self, fn):
            self.fn = fn

        def replay(self):
            with torch.cuda.stream(cap_stream):
                self.fn()

    def capture(fn):
        if args.eager:
            return Eager(fn)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=cap_stream):
            fn()
        return g

    def timed(graph_runs):
        """graph_runs: list of (graph, times).  Returns elapsed ms between HIP events
        recorded on the stream the graphs are launched on."""
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        run_stream = cap_stream if args.eager else torch.cuda.current_stream()
        a.record(run_stream)
        for g, n in graph_runs:
            for _ in range(n):
                g.replay()
        b.record(run_stream)
        torch.cuda.synchronize()
        return a.elapsed_time(b)

    # One graph holds one step on each of the R buffer sets (launching a graph costs the host
    # tens of microseconds, more than a decode step takes on the GPU); a second graph holds the
    # K mod R steps left over, so that exactly K steps are timed.
    def steps_graph(n):
        return capture(lambda: [step(sets[i % R]) for i in range(n)])

    g_round = steps_graph(R)
    g_rest = steps_graph(args.steps % R) if args.steps % R else None
    g_warm = steps_graph(args.warmup % R) if args.warmup % R else None
    torch.cuda.synchronize()

    timed([(g_round, args.warmup // R)] + ([(g_warm, 1)] if g_warm else []))
    # the timed region of exactly K steps, repeated: the median region is the reported one
    regions, wall = [], []
    for _ in range(3 if brief else 9):
        t0 = time.perf_counter()
        regions.append(timed([(g_round, args.steps // R)] + ([(g_rest, 1)] if g_rest else [])) / args.steps)
        wall.append((time.perf_counter() - t0) * 1e3)
    ms_per_step = float(np.median(regions))
    wall_ms = float(np.median(wall))
    tokens_per_s = T / (ms_per_step * 1e-3)
    step_gbps = (fwd_bytes + bwd_bytes) / (ms_per_step * 1e-3) / 1e9

    if args.step_only:
        return {"config": cfg, "ms_per_step": round(ms_per_step, 5), "step_hbm_gbps": round(step_gbps, 1)}

    # ---- the two forward launches alone (all projections of the batch each): shrink v = x A^T and
    # expand y += s * v B^T, launched back to back from a graph over the rotating buffer sets and timed
    # with HIP events on the stream.
    reps = max(2, 48 // R)
    rsum = sum((ranks[a % 4] if ranks else r) for a in set(w["ids"]))

    def stage_us(stages):
        g = capture(lambda: [fwd(st, stages) for _ in range(reps) for st in sets])
        timed([(g, 2)])
        return timed([(g, 10)]) * 1e3 / (10 * reps * R)  # us per launch

    # the same step with the batch's plans built once and reused, as the layers of one model
    # step reuse them (reported beside the headline value, never as it)
    for st in sets[1:]:  # one plan for every buffer set: the routing is the same, as across the layers of a step
        st["plan"] = sets[0]["plan"]
        if P:
            st["bplan"] = sets[0]["bplan"]
    g_reuse = capture(lambda: [step(st, build_plan=False) for st in sets])
    timed([(g_reuse, 2)])
    reuse_ms = timed([(g_reuse, max(1, args.steps // R))]) / (max(1, args.steps // R) * R)

    expand_us = stage_us(2)
    shrink_us = stage_us(1)
    # decode batches: the shrink launch that also builds the plan (what the step's first forward launches)
    self_planned = single_tiles(T, r) and not args.plan_launch and not P
    if self_planned:
        bufs = [st["plan_buf"] for st in sets]

        def planning_shrink():
            for _ in range(reps):
                for st, buf in zip(sets, bufs):
                    keep, st["plan"] = st["plan"], K.SegmentPlan(seg_t, ids_t, T, buf=buf, defer=True)
                    fwd(st, 1)
                    st["plan"] = keep
        g = capture(planning_shrink)
        timed([(g, 2)])
        shrink_plan_us = timed([(g, 10)]) * 1e3 / (10 * reps * R)
    expand_bytes = sum(T * ho * 2 * 2 + rsum * ho * 2 + T * r * 2 for _, hi, ho in w["proj"])
    shrink_bytes = sum((T * hi * 2 if i not in shared_x else 0) + rsum * hi * 2 + T * r * 2
                       for i, (_, hi, ho) in enumerate(w["proj"]))
    traffic = {}
    tpath = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        traffic = json.load(open(tpath)).get(cfg, {})

    def launch_line(kernel, us, nbytes, key):
        gbps = nbytes / (us * 1e-6) / 1e9
        return dict(kernel=kernel, bound="hbm", achieved=round(gbps, 1), peak=HBM_PEAK_GBPS, unit="GB/s",
                    frac=round(gbps / HBM_PEAK_GBPS, 4), traffic=traffic.get(key), us_per_launch=round(us, 3),
                    algorithmic_bytes=nbytes)
    lines = [launch_line("shrink launch (v = x A^T, all projections of the step)", shrink_us, shrink_bytes,
                         "shrink_bytes_per_launch"),
             launch_line("expand launch (y += s v B^T, all projections of the step)", expand_us, expand_bytes,
                         "expand_bytes_per_launch")]
    if self_planned:
        lines.append(launch_line("shrink launch that also builds the plan (the step's first forward call)",
                                 shrink_plan_us, shrink_bytes, "shrink_self_planned_bytes_per_launch"))
    # the forward launch furthest below the HBM peak is the one the roofline entry names
    roofline = min(lines, key=lambda l: l["frac"])

    # ---- the backward's launches alone (training workloads), each stage of all projections: the products
    # (dV = dY B with its fold launch; v comes from the forward), dX = s dV A, the weight gradients.  Each line
    # counts what that launch has to move by itself -- dY is read by the first and the third -- while the
    # roll-up below them counts the step's algorithmic bytes (dY once) against the backward's own time.
    backward = None
    if P:
        train_ids = sorted(set(w["ids"][:P]))
        rsum_t = sum((ranks[a % 4] if ranks else r) for a in train_ids)
        n = n_train

        def bwd_stage_us(stages):
            g = capture(lambda: [bwd(st, stages) for _ in range(reps) for st in sets])
            timed([(g, 2)])
            return timed([(g, 10)]) * 1e3 / (10 * reps * R)
        dv_bytes = sum(n * ho * 2 + rsum_t * ho * 2 + n * r * 2 for _, hi, ho in w["proj"])
        dx_bytes = sum(n * hi * 2 + rsum_t * hi * 2 + n * r * 2 for _, hi, ho in w["proj"])
        wg_bytes = sum(n * (hi + ho) * 2 + rsum_t * (hi + ho) * 2 + 2 * n * r * 2 for _, hi, ho in w["proj"])
        dv_us, dx_us, wg_us, all_us = bwd_stage_us(1), bwd_stage_us(2), bwd_stage_us(4), bwd_stage_us(0)
        lines += [launch_line("backward: dV = dY B over all projections (shrink launch + fold launch)", dv_us,
                              dv_bytes, "bwd_dv_bytes_per_launch"),
                  launch_line("backward: dX = s dV A over all projections (expand launch)", dx_us, dx_bytes,
                              "bwd_dx_bytes_per_launch"),
                  launch_line("backward: dA, dB of all projections (weight-gradient launch)", wg_us, wg_bytes,
                              "bwd_wgrad_bytes_per_launch")]
        gbps = bwd_bytes / (all_us * 1e-6) / 1e9
        backward = dict(algorithmic_bytes=bwd_bytes, us=round(all_us, 3), achieved=round(gbps, 1), unit="GB/s",
                        frac=round(gbps / HBM_PEAK_GBPS, 4), launches_per_step=4,
                        note="all projections in one set of launches (smlm_lora_bwd_multi_ex), plan reused; "
                             "algorithmic bytes count dY, x once, dX, A/B and dA/dB of the training adapters, v, dV")

    # ---- what plain streaming kernels reach at these launch sizes (loquetier_amd/csrc/stream_probe.hip:
    # a read-modify-write moving the expand launch's bytes, a read moving the shrink launch's), cold over
    # rotating buffers and hot in the Infinity Cache.  HBM-bound launches on this part climb with the bytes
    # per launch, so these, not the 8 TB/s peak, are what the launches above can be held against.
    streaming = None
    if probe is not None and not brief:
        stream_h = cap_stream.cuda_stream

        def probe_us(nbytes, write, cold):
            n = max(2, min(64, math.ceil(640e6 / nbytes))) if cold else 1
            bufs = [torch.zeros(nbytes // 4, dtype=torch.int32, device=dev) for _ in range(n)]
            sink = torch.zeros(4, dtype=torch.int32, device=dev)
            pr = max(2, 48 // n)

            def go():
                for _ in range(pr):
                    for b in bufs:
                        if write:
                            probe.smlm_probe_rmw(b.data_ptr(), nbytes, stream_h)
                        else:
                            probe.smlm_probe_read(b.data_ptr(), nbytes, sink.data_ptr(), stream_h)
            with torch.cuda.stream(cap_stream):
                go()
            torch.cuda.synchronize()
            g = capture(go)
            timed([(g, 2)])
            return timed([(g, 10)]) * 1e3 / (10 * pr * n)
        rmw_c, rmw_h = probe_us(expand_bytes // 2, True, True), probe_us(expand_bytes // 2, True, False)
        rd_c, rd_h = probe_us(shrink_bytes, False, True), probe_us(shrink_bytes, False, False)
        tb = lambda nbytes, us: round(nbytes / (us * 1e-6) / 1e9, 1)
        streaming = dict(kernel="loquetier_amd/csrc/stream_probe.hip (16-byte non-temporal accesses, 8 in flight a thread)",
                         rmw_bytes=expand_bytes, rmw_cold_us=round(rmw_c, 3), rmw_cold_gbps=tb(expand_bytes, rmw_c),
                         rmw_hot_us=round(rmw_h, 3), rmw_hot_gbps=tb(expand_bytes, rmw_h),
                         read_bytes=shrink_bytes, read_cold_us=round(rd_c, 3), read_cold_gbps=tb(shrink_bytes, rd_c),
                         read_hot_us=round(rd_h, 3), read_hot_gbps=tb(shrink_bytes, rd_h))

    # ---- CPU baseline: per-segment torch matmuls on the host cores (bounded sample)
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import torch_segments as ref
        torch.set_num_threads(min(os.cpu_count() or 1, 16))
        cores = torch.get_num_threads()
        st = sets[0]
        host = [dict(x=d["x"].cpu(), y=d["y"].cpu(), A=[a.cpu() for a in d["A"]],
                     B=[b.cpu() for b in d["B"]], g=d["g"].cpu() if P else None) for d in st["proj"]]
        seg, ids = w["seg"], w["ids"]

        def cpu_step():
            for h in host:
                ref.add_lora_forward(h["x"], [h["A"][a] for a in ids], [h["B"][a] for a in ids], seg,
                                     y=h["y"], beta=1.0, seg_scale=[2.0] * S)
                if P:
                    ref.add_lora_backward(h["g"], h["x"][:n_train], h["A"], h["B"], seg[:P + 1], ids[:P])

        budget = 3.0 if brief else 10.0
        if not brief:
            cpu_step()
        n, t_begin = 0, time.perf_counter()
        while True:
            cpu_step()
            n += 1
            el = time.perf_counter() - t_begin
            if el > budget or n >= 200:
                break
        cpu = dict(value=round(T * n / el, 1), unit="tokens/s", cores=cores, kind="port",
                   sample=f"{n} whole step{'s' if n > 1 else ''} of the same workload ({el:.1f} s), per-segment "
                          f"torch.matmul in fp32 on {w['dtype']} data (oracle/torch_segments.py)")

    # whether the library builds this batch's plan inside the forward's shrink launch (the limits of
    # the route, include/smlm.h: segments, possible tiles)
    in_launch = not args.plan_launch and not (args.dropout and P) and (
        S <= 1024 if single_tiles(T, r) else (S <= 512 and T // 16 + S + 1 <= 1024))
    out = {
        "metric": METRIC, "value": round(tokens_per_s, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if w["dtype"] == "fp16" else "bf16", "data": "synthetic",
        "config": {"workload": w["name"], "tokens_per_step": T, "segments": S, "adapters": NA, "rank": r,
                   "projections": [f"{n}:{a}->{b}" for n, a, b in w["proj"]],
                   "buffer_sets_rotated": R, "step_includes": "plan build (" + ("inside the shrink launch" if in_launch else "own launch")
                   + ") + fused forward per projection"
                   + (" + backward" if P else ""), "graph_replay": not args.eager,
                   "dropout": args.dropout if P else 0.0,
                   "true_ranks_passed": bool(ranks and not args.padded_ranks),
                   "adapters_stored_at_true_rank": packed},
        "step_algorithmic_bytes": fwd_bytes + bwd_bytes,
        "step_hbm_gbps": round(step_gbps, 1), "step_frac_of_8TBps": round(step_gbps / HBM_PEAK_GBPS, 4),
        "host_wall_ms_per_step": round(wall_ms / args.steps, 5),
        "ms_per_step_plan_reused": round(reuse_ms, 5),
        "timed_regions": {"count": len(regions), "steps_each": args.steps, "ms_per_step_median": round(ms_per_step, 5),
                          "ms_per_step_min": round(min(regions), 5), "ms_per_step_max": round(max(regions), 5)},
        "roofline": roofline,
        "launches": lines,
        "backward": backward,
        "streaming_reference": streaming,
        "cpu_baseline": cpu,
    }
    del sets
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="all",
                    help="all (default): the headline workload cfg2 in full, then cfg3, cfg4 and cfg5 in brief "
                         "under 'configs', plus per-projection / layer-issue / reference-surface / model-step legs; or one "
                         "of cfg2 | cfg2mod | cfg2one | cfg2layer | cfg2ref | cfg3 | cfg4 | cfg5 | rmsnorm | model-step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-rotate", action="store_true", help="one buffer set (cache-hot numbers)")
    ap.add_argument("--step-only", action="store_true", help="skip the single-kernel and CPU legs")
    ap.add_argument("--eager", action="store_true",
                    help="launch the steps one by one instead of replaying a graph (for counter runs)")
    ap.add_argument("--sorted", action="store_true",
                    help="hand the same requests over grouped by adapter (a scheduler that batches by adapter)")
    ap.add_argument("--padded-ranks", action="store_true",
                    help="workloads with adapters below the padded rank: do not pass the true ranks "
                         "(the kernels then read the zero padding, as the reference's do)")
    ap.add_argument("--plan-launch", action="store_true",
                    help="build the forward plan with its own launch before the forward call, also for decode "
                         "batches (default: the forward call builds it, decode batches inside the shrink launch)")
    ap.add_argument("--padded-storage", action="store_true",
                    help="workloads with adapters below the padded rank: pass the true ranks but keep the "
                         "adapters zero-padded in memory (default: stored at their own rank, packed)")
    ap.add_argument("--bwd-per-projection", action="store_true",
                    help="workloads with a backward: one backward call per projection instead of one for all")
    ap.add_argument("--dropout", type=float, default=0.0,
                    help="dropout probability of the training adapters (workloads with a backward): the "
                         "kernels regenerate the mask in the forward and the backward; default 0 = off")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a 128 MiB device copy three times before the timed region: a kernel "
                         "of known traffic to scale FETCH_SIZE / WRITE_SIZE readings with")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; every box has one MI355X and no collective, "
              "sharding or rank code exists in it. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU (torch.cuda.is_available() is False)")
    from loquetier_amd import _lib
    from loquetier_amd.ops import _kernels as K
    _lib.load()  # no fallback: raises when the HIP library is missing
    torch.cuda.set_device(torch.device("cuda:0"))
    if args.config == "rmsnorm":
        return rmsnorm_bench(args, torch, K)
    if args.config == "model-step":
        print(json.dumps(model_step_bench(args, torch, K)), flush=True)
        return
    if args.config == "cfg2ref":
        print(json.dumps(reference_surface_bench(args, torch, K)), flush=True)
        return
    probe = load_probe()
    if args.config != "all":
        print(json.dumps(run_workload(args, args.config, torch, K, probe)), flush=True)
        return
    # the headline: BASELINE.json's configs[1]; the other GPU workloads ride along in brief
    out = run_workload(args, "cfg2", torch, K, probe)
    if not args.step_only:
        keys = ("value", "unit", "ms_per_step", "ms_per_step_plan_reused", "timed_regions", "dtype",
                "step_algorithmic_bytes", "step_hbm_gbps", "step_frac_of_8TBps", "roofline", "launches", "backward",
                "cpu_baseline")
        quiet = argparse.Namespace(**dict(vars(args), no_cpu_baseline=True))
        # what a model gets out of the headline batch: one projection per call (a layer call of the reference), the
        # launches one decoder layer can issue (q/k/v of one input together, o alone), the reference's own call
        # sequence, and the whole layer path (224 MixedLoraLinear calls a model step)
        for name, cfg in (("per_projection", "cfg2one"), ("layer_issue", "cfg2layer")):
            o = run_workload(quiet, cfg, torch, K, probe, brief=True)
            out[name] = {k: o[k] for k in keys if k != "cpu_baseline"}
            out[name]["workload"] = o["config"]["workload"]
        out["reference_surface"] = reference_surface_bench(args, torch, K)
        out["model_step_decode"] = model_step_bench(args, torch, K, finetune=False)["decode_forward"]
        out["configs"] = {}
        for cfg in ("cfg3", "cfg4", "cfg5"):
            o = run_workload(args, cfg, torch, K, probe, brief=True)
            out["configs"][cfg] = {k: o[k] for k in keys}
            out["configs"][cfg]["workload"] = o["config"]["workload"]
        # cfg5 with the adapters kept zero-padded to rank 64 in memory, as the reference keeps them
        padded = argparse.Namespace(**dict(vars(args), padded_storage=True, step_only=True))
        out["configs"]["cfg5"]["ms_per_step_adapters_padded_in_memory"] = run_workload(padded, "cfg5", torch, K, probe,
                                                                                      brief=True)["ms_per_step"]
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
