"""Per-segment torch restatement of the reference's SMLM semantics on the host.

TEST INFRASTRUCTURE ONLY (tests/, the smoke check, bench.py's cpu_baseline leg).
It is the multi-threaded companion of oracle/smlm_oracle.c for sizes where the
scalar C loops take too long: the same per-segment products, expressed as one
`torch.matmul` per segment the way the reference's backward does
(src/loquetier_src/kernel_utils.py:139-145) and the way its forward is defined
(one GEMM problem per segment,
kernel_src/csrc/smlm_forward/smlm_forward_cutlass.cuh:31-46).

Inputs are CPU tensors in the I/O dtype (fp16 / bf16 / fp32); products are
computed in fp32 and rounded to the I/O dtype where the reference materialises
a tensor in that dtype (v, mid, every returned gradient).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch


def add_lora_forward(x: torch.Tensor, wa: Sequence[torch.Tensor], wb: Sequence[torch.Tensor],
                     seg: Sequence[int], y: Optional[torch.Tensor] = None, beta: float = 0.0,
                     seg_scale: Optional[Sequence[float]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """y[s_i:s_{i+1}] = beta*y + scale_i * round(x_i A_i^T) B_i^T; returns (y, v).

    wa[i] is [r_i, h_in], wb[i] is [h_out, r_i] (per segment; the ranks may differ, v then has
    the largest and zeros past a segment's own).  With beta = 0 and no scale this is
    add_lora.forward (kernel_utils.py:102-120)."""
    T = x.shape[0]
    dt = x.dtype
    h_out = wb[0].shape[0]
    r = max(w.shape[0] for w in wa)
    if y is None:
        y = torch.zeros(T, h_out, dtype=dt)
    v = torch.zeros(T, r, dtype=dt)
    xf = x.float()
    for i in range(len(seg) - 1):
        a, b = int(seg[i]), int(seg[i + 1])
        if b <= a:
            continue
        vi = (xf[a:b] @ wa[i].float().t()).to(dt)
        v[a:b, :vi.shape[1]] = vi
        yi = vi.float() @ wb[i].float().t()
        if seg_scale is not None:
            yi = yi * float(seg_scale[i])
        if beta != 0.0:
            yi = yi + beta * y[a:b].float()
        y[a:b] = yi.to(dt)
    return y, v


def add_lora_backward(g: torch.Tensor, x: torch.Tensor, a_w: Sequence[torch.Tensor],
                      b_w: Sequence[torch.Tensor], tp: Sequence[int], part_adapter: Sequence[int]
                      ) -> Tuple[torch.Tensor, List[torch.Tensor], List[torch.Tensor]]:
    """Layout-corrected add_lora.backward (A [r,h_in], B [h_out,r]).

    Same loop structure as kernel_utils.py:139-145: per train partition
    dV = g B, dX = dV A, dA += dV^T x, dB += g^T v; gradients of partitions that
    share an adapter are summed.  Returns (grad_x, [dA_a], [dB_a])."""
    dt = g.dtype
    T = g.shape[0]
    h_in = x.shape[1]
    gx = torch.zeros(T, h_in, dtype=dt)
    da = [torch.zeros(a.shape, dtype=torch.float32) for a in a_w]
    db = [torch.zeros(b.shape, dtype=torch.float32) for b in b_w]
    for p in range(len(tp) - 1):
        s0, s1 = int(tp[p]), int(tp[p + 1])
        if s1 <= s0:
            continue
        ad = int(part_adapter[p])
        A, B = a_w[ad].float(), b_w[ad].float()
        gp, xp = g[s0:s1].float(), x[s0:s1].float()
        dv = (gp @ B).to(dt).float()
        v = (xp @ A.t()).to(dt).float()
        gx[s0:s1] = (dv @ A).to(dt)
        da[ad] += dv.t() @ xp
        db[ad] += gp.t() @ v
    return gx, [d.to(dt) for d in da], [d.to(dt) for d in db]
