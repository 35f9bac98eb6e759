"""Segment construction for a flat batch (the producer of the operator's index
inputs; reference: ModelGeneration.generate,
src/loquetier_src/model_generation.py:267-281)."""
from __future__ import annotations

from typing import List, Sequence, Tuple

import torch


def build_segments(req_lora_id: Sequence[int], req_len: Sequence[int], device
                   ) -> Tuple[List[int], torch.Tensor, torch.Tensor]:
    """Run-length merge consecutive requests with equal adapter id.

    Returns (lora_ids, lora_len int32 [S], segment int32 [S+1] = cumsum of the
    lengths, starting at 0), the tensors on `device`.  Adjacent requests with
    the same adapter merge whatever their kind (train / prefill / decode), as
    in the reference."""
    if len(req_lora_id) == 0:
        raise IndexError("no requests")  # the reference indexes requests[0]
    lora_ids, lora_lens = [int(req_lora_id[0])], [0]
    for lid, n in zip(req_lora_id, req_len):
        if lora_ids[-1] == lid:
            lora_lens[-1] += int(n)
        else:
            lora_ids.append(int(lid))
            lora_lens.append(int(n))
    lora_len = torch.tensor(lora_lens, dtype=torch.int32, device=device)
    segment = torch.cumsum(torch.tensor([0] + lora_lens, dtype=torch.int32, device=device), dim=0,
                           dtype=torch.int32)
    return lora_ids, lora_len, segment


def build_segments_device(req_lora_id: torch.Tensor, req_len: torch.Tensor
                          ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """The same merge for request arrays that already live on the GPU (int32
    [R] each): returns (lora_ids [R], lora_len [R], segment [R+1], n_seg [2])
    as device tensors without waiting for the GPU.  n_seg = (segment count,
    total rows); the arrays keep the capacity R and describe empty segments
    past the count, so they are handed on whole."""
    from .ops import _kernels
    return _kernels.segments_build(req_lora_id, req_len)
