"""Per-request decode geometry of one batched step (reference
``integration/common/batched_seam.py:36-118``).

Pure host arithmetic over ``WindowSpec``: packed token count, bf16 tail length and tail
positions per request, plus which groups completed since the slot's previous step.  The GPU
path does not need the returned tensors (the tail-gather kernel derives the same numbers from
the sequence length on the device); adapters that plan on the host get the reference's record.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ...attention.kv_window import WindowSpec


@dataclass
class BatchedDecodePlan:
    b_seq_len: torch.Tensor          # [B] int32, packed tokens
    b_tail_len: torch.Tensor         # [B] int32, bf16 rows
    tail_pos: torch.Tensor           # [B, max_tail_len] int64, absolute positions, 0-padded
    regroup: List[Tuple[int, int]]   # per request (groups packed before, groups due now)
    max_seq_len: int
    max_tail_len: int
    seq_lens: List[int]


class BatchedStepPlanner:
    """Remembers, per request slot, how many groups were due at the previous step."""

    def __init__(self, window: WindowSpec, max_context: int, device="cpu") -> None:
        self.window = window
        self.max_context = int(max_context)
        self.device = torch.device(device)
        self.max_tail_len = int(window.max_tail_len(self.max_context))
        self._prev_groups: Dict[int, int] = {}

    def reset(self, slot: Optional[int] = None) -> None:
        if slot is None:
            self._prev_groups.clear()
        else:
            self._prev_groups.pop(int(slot), None)

    def plan(self, seq_lens: Sequence[int], slots: Optional[Sequence[int]] = None) -> BatchedDecodePlan:
        seq_lens = [int(s) for s in seq_lens]
        B = len(seq_lens)
        slots = [int(s) for s in (slots if slots is not None else range(B))]
        win, T = self.window, self.max_tail_len
        b_seq = torch.zeros(B, dtype=torch.int32)
        b_tail = torch.zeros(B, dtype=torch.int32)
        tail_pos = torch.zeros(B, T, dtype=torch.int64)
        regroup: List[Tuple[int, int]] = []
        for i, (seq, slot) in enumerate(zip(seq_lens, slots)):
            groups = win.num_groups(seq)
            tail = win.tail_indices(seq)[:T]          # readers mask by b_tail_len
            b_seq[i] = groups * win.group_tokens
            b_tail[i] = len(tail)
            if tail:
                tail_pos[i, :len(tail)] = torch.tensor(tail, dtype=torch.int64)
            prev = 0 if seq <= 0 else self._prev_groups.get(slot, 0)
            regroup.append((prev, groups))
            self._prev_groups[slot] = groups
        max_seq = max(1, int(b_seq.max().item())) if B else 1
        dev = self.device
        return BatchedDecodePlan(b_seq.to(dev), b_tail.to(dev), tail_pos.to(dev), regroup,
                                 max_seq, T, seq_lens)


__all__ = ["BatchedDecodePlan", "BatchedStepPlanner"]
