"""Sink / packed-prefix / recent-window geometry of an OMMX KV sequence.

A sequence of ``n`` tokens is served from three places: the first ``sink`` tokens and the
last ``recent .. recent+group-1`` tokens stay bf16 (the "tail" the decode kernel reads from
``k_tail``/``v_tail``), everything between is packed in whole 32-token groups.  The split
is a pure function of ``n``; same closed forms as the reference
``ommx_gpu_serve/attention/kv_window.py:35-141``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List

CANONICAL_GROUP_TOKENS = 32


def packed_boundary(seq_len: int, sink_tokens: int, recent_window: int,
                    group_tokens: int = CANONICAL_GROUP_TOKENS) -> int:
    """First token index after the packed prefix (``kv_window.py:35-51``)."""
    n, s, r, g = int(seq_len), int(sink_tokens), int(recent_window), int(group_tokens)
    if g <= 0:
        raise ValueError(f"group_tokens must be > 0; got {g}")
    spare = n - s - r
    return min(s, n) if spare <= 0 else s + g * (spare // g)


def packed_len(seq_len: int, sink_tokens: int, recent_window: int,
               group_tokens: int = CANONICAL_GROUP_TOKENS) -> int:
    """Packed token count, a multiple of ``group_tokens`` (``kv_window.py:54-58``)."""
    return max(0, packed_boundary(seq_len, sink_tokens, recent_window, group_tokens) - int(sink_tokens))


def num_packed_groups(seq_len: int, sink_tokens: int, recent_window: int,
                      group_tokens: int = CANONICAL_GROUP_TOKENS) -> int:
    return packed_len(seq_len, sink_tokens, recent_window, group_tokens) // int(group_tokens)


def newly_completed_groups(prev_seq_len: int, new_seq_len: int, sink_tokens: int,
                           recent_window: int, group_tokens: int = CANONICAL_GROUP_TOKENS) -> int:
    """Groups to pack when a sequence grows from ``prev`` to ``new`` tokens (``kv_window.py:67-77``)."""
    a = num_packed_groups(prev_seq_len, sink_tokens, recent_window, group_tokens)
    b = num_packed_groups(new_seq_len, sink_tokens, recent_window, group_tokens)
    return max(0, b - a)


def tail_token_indices(seq_len: int, sink_tokens: int, recent_window: int,
                       group_tokens: int = CANONICAL_GROUP_TOKENS) -> List[int]:
    """Token indices of the bf16 rows, sink first (``kv_window.py:80-92``)."""
    n = int(seq_len)
    edge = packed_boundary(n, sink_tokens, recent_window, group_tokens)
    return [*range(min(int(sink_tokens), n)), *range(edge, n)]


def sink_page_shift(sink_tokens: int, page_size: int) -> int:
    return int(sink_tokens) // max(1, int(page_size))


def sink_token_offset(sink_tokens: int, page_size: int) -> int:
    return int(sink_tokens) % max(1, int(page_size))


@dataclass(frozen=True)
class WindowSpec:
    """Window constants of one serving configuration (``kv_window.py:104-141``)."""

    sink_tokens: int = 8
    recent_window: int = 32
    group_tokens: int = CANONICAL_GROUP_TOKENS
    page_size: int = 16

    def _a(self):
        return self.sink_tokens, self.recent_window, self.group_tokens

    def boundary(self, seq_len: int) -> int:
        return packed_boundary(seq_len, *self._a())

    def packed_len(self, seq_len: int) -> int:
        return packed_len(seq_len, *self._a())

    def num_groups(self, seq_len: int) -> int:
        return num_packed_groups(seq_len, *self._a())

    def newly_completed_groups(self, prev_seq_len: int, new_seq_len: int) -> int:
        return newly_completed_groups(prev_seq_len, new_seq_len, *self._a())

    def tail_indices(self, seq_len: int) -> List[int]:
        return tail_token_indices(seq_len, *self._a())

    def packed_start_offset(self) -> int:
        return sink_token_offset(self.sink_tokens, self.page_size)

    def sink_page_shift(self) -> int:
        return sink_page_shift(self.sink_tokens, self.page_size)

    def max_tail_len(self, max_seq_len: int = 0) -> int:
        """Largest possible tail: sink + recent + one incomplete group."""
        return int(self.sink_tokens) + int(self.recent_window) + int(self.group_tokens)


__all__ = ["CANONICAL_GROUP_TOKENS", "WindowSpec", "packed_boundary", "packed_len",
           "num_packed_groups", "newly_completed_groups", "tail_token_indices",
           "sink_page_shift", "sink_token_offset"]
