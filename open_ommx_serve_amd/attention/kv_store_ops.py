"""Allocation-free copies for the bf16 residual ring of the KV store (HIP kernels).

Mirror of ``ommx_gpu_serve/attention/kv_store_ops.py:63-76`` (``write_token`` /
``gather_tail``, same arguments), plus the batched forms the multi-sequence pool uses:
``write_tokens`` (one row per request, optional device-side advance of the position
counter) and ``gather_tails`` (window arithmetic of ``attention/kv_pool.py:1048-1105`` done
in the kernel).  Only bf16 rows move here; quantisation stays in the packer.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _hip


def ring_slot(pos: int, sink: int, span: int) -> int:
    """History row of absolute position ``pos`` (kv_store.py:301-313).  ``span == 0``: identity."""
    p = int(pos)
    if span <= 0 or p < sink:
        return p
    return sink + (p - sink) % span


def _check_hist(k_hist: torch.Tensor, v_hist: torch.Tensor) -> None:
    if k_hist.dtype != torch.bfloat16 or v_hist.dtype != torch.bfloat16:
        raise ValueError("k_hist / v_hist must be bfloat16")
    if k_hist.shape != v_hist.shape or not k_hist.is_contiguous() or not v_hist.is_contiguous():
        raise ValueError("k_hist / v_hist must be contiguous and of one shape")


def _check_i64(name: str, t: Optional[torch.Tensor], n: int, device) -> None:
    if t is None:
        return
    if t.dtype != torch.int64 or t.device != device or not t.is_contiguous() or t.numel() < n:
        raise ValueError(f"{name} must be a contiguous int64 tensor of at least {n} entries on {device}")


def write_tokens(k_hist: torch.Tensor, v_hist: torch.Tensor, pos: torch.Tensor, k: torch.Tensor,
                 v: torch.Tensor, sink: int, recent: int, *, slots: Optional[torch.Tensor] = None,
                 pos_next: Optional[torch.Tensor] = None,
                 err_flag: Optional[torch.Tensor] = None) -> None:
    """``k_hist[slot_b, ring_slot(pos[b])] = k[b]`` (and V) for every request, one launch.

    ``k_hist`` / ``v_hist``: ``[num_slots, rows, H, D]`` bf16; ``k`` / ``v``: ``[B, H, D]`` bf16
    (last dim contiguous); ``pos``: int64 ``[B]`` on the device; ``recent`` is the sliding span
    of the ring (0: whole history).  ``pos_next`` (may be ``pos``) receives ``pos + 1``.
    """
    _check_hist(k_hist, v_hist)
    if k_hist.dim() != 4:
        raise ValueError("k_hist must be [num_slots, rows, H, D]")
    N, rows, H, D = (int(x) for x in k_hist.shape)
    if k.dim() != 3 or v.shape != k.shape or tuple(k.shape[1:]) != (H, D):
        raise ValueError(f"k / v must be [B, {H}, {D}]; got {tuple(k.shape)} / {tuple(v.shape)}")
    if k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
        raise ValueError("k / v must be bfloat16")
    if k.stride(-1) != 1 or v.stride(-1) != 1:
        raise ValueError("k / v need a contiguous last dimension")
    B = int(k.shape[0])
    dev = k_hist.device
    _check_i64("pos", pos, B, dev)
    _check_i64("slots", slots, B, dev)
    _check_i64("pos_next", pos_next, B, dev)
    if slots is None and B > N:
        raise ValueError(f"{B} requests but only {N} history slots")
    _hip.require_gpu(dev)
    lib = _hip.load()
    _hip.check(lib.ommx_ring_write(
        k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
        k_hist.data_ptr(), v_hist.data_ptr(), k_hist.stride(0), rows,
        _hip.ptr(slots), pos.data_ptr(), _hip.ptr(pos_next),
        B, H, D, int(sink), int(recent), _hip.ptr(err_flag), _hip.current_stream_ptr(dev)),
        "ommx_ring_write")


def write_token(k_hist: torch.Tensor, v_hist: torch.Tensor, pos: torch.Tensor, k: torch.Tensor,
                v: torch.Tensor, sink: int, recent: int, *,
                err_flag: Optional[torch.Tensor] = None) -> None:
    """Single-sequence form, arguments as the reference: ``k_hist [rows, H, D]``, ``pos [1]``.
    A position outside the history sets ``ERR_RING_RANGE`` in ``err_flag`` (the reference
    asserts there, kv_store_ops.py:33-34); without a flag the row is dropped silently."""
    if k_hist.dim() != 3:
        raise ValueError("k_hist must be [rows, H, D]")
    H, D = int(k_hist.shape[1]), int(k_hist.shape[2])
    write_tokens(k_hist.unsqueeze(0), v_hist.unsqueeze(0), pos, k.reshape(1, H, D),
                 v.reshape(1, H, D), sink, recent, err_flag=err_flag)


def gather_tails(k_hist: torch.Tensor, v_hist: torch.Tensor, k_tail: torch.Tensor,
                 v_tail: torch.Tensor, sink: int, recent_span: int, *,
                 seq: Optional[torch.Tensor] = None, tail_idx: Optional[torch.Tensor] = None,
                 slots: Optional[torch.Tensor] = None, b_tail_len: Optional[torch.Tensor] = None,
                 b_seq_len: Optional[torch.Tensor] = None, window_sink: Optional[int] = None,
                 window_recent: int = 32, group_tokens: int = 32, packed_lag: int = 0,
                 err_flag: Optional[torch.Tensor] = None) -> None:
    """Gather the tail rows of ``B`` requests into ``k_tail`` / ``v_tail`` ``[B, T, H, D]``.

    Either ``seq`` (int64 ``[B]`` absolute lengths: the kernel derives the sink ++ recent
    positions and writes ``b_tail_len`` / ``b_seq_len``) or ``tail_idx`` (int64 ``[B, T]``
    absolute positions).  ``sink`` / ``recent_span`` describe the ring (span 0: whole
    history); ``window_sink`` / ``window_recent`` / ``group_tokens`` the attention window.
    ``packed_lag``: tokens appended since the planes were last packed (``seq`` form only).  A
    step that appends and decodes before the host packs passes 1: the boundary is then the one
    the host has packed for, and the rows since come from the ring.
    """
    _check_hist(k_hist, v_hist)
    if k_hist.dim() != 4:
        raise ValueError("k_hist must be [num_slots, rows, H, D]")
    N, rows, H, D = (int(x) for x in k_hist.shape)
    if k_tail.dim() != 4 or k_tail.shape != v_tail.shape or tuple(k_tail.shape[2:]) != (H, D):
        raise ValueError(f"k_tail / v_tail must be [B, T, {H}, {D}]")
    if k_tail.dtype != torch.bfloat16 or v_tail.dtype != torch.bfloat16:
        raise ValueError("k_tail / v_tail must be bfloat16")
    if not k_tail.is_contiguous() or not v_tail.is_contiguous():
        raise ValueError("k_tail / v_tail must be contiguous")
    B, T = int(k_tail.shape[0]), int(k_tail.shape[1])
    dev = k_hist.device
    if (seq is None) == (tail_idx is None):
        raise ValueError("pass exactly one of seq, tail_idx")
    _check_i64("seq", seq, B, dev)
    _check_i64("tail_idx", tail_idx, B * T, dev)
    _check_i64("slots", slots, B, dev)
    for name, t in (("b_tail_len", b_tail_len), ("b_seq_len", b_seq_len)):
        if t is not None and (t.dtype != torch.int32 or t.device != dev or t.numel() < B
                              or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous int32 tensor of at least {B} entries")
    if slots is None and B > N:
        raise ValueError(f"{B} requests but only {N} history slots")
    _hip.require_gpu(dev)
    lib = _hip.load()
    wsink = int(sink if window_sink is None else window_sink)
    _hip.check(lib.ommx_tail_gather(
        k_hist.data_ptr(), v_hist.data_ptr(), k_hist.stride(0), rows,
        _hip.ptr(slots), _hip.ptr(seq), _hip.ptr(tail_idx),
        k_tail.data_ptr(), v_tail.data_ptr(), _hip.ptr(b_tail_len), _hip.ptr(b_seq_len),
        B, T, H, D, wsink, int(window_recent), int(group_tokens), int(recent_span),
        int(packed_lag), _hip.ptr(err_flag), _hip.current_stream_ptr(dev)), "ommx_tail_gather")


def gather_tail(k_hist: torch.Tensor, v_hist: torch.Tensor, indices: torch.Tensor,
                k_tail: torch.Tensor, v_tail: torch.Tensor, sink: int, recent: int, *,
                err_flag: Optional[torch.Tensor] = None) -> None:
    """Single-sequence form, arguments as the reference: ``k_hist [rows, H, D]``, ``indices [T]``
    absolute positions, ``k_tail`` / ``v_tail`` ``[1, T, H, D]``.  A position outside the history
    yields a zero row and sets ``ERR_RING_RANGE`` in ``err_flag`` (kv_store_ops.py:52-53 asserts)."""
    if k_hist.dim() != 3:
        raise ValueError("k_hist must be [rows, H, D]")
    idx = indices if indices.dtype == torch.int64 else indices.to(torch.int64)
    gather_tails(k_hist.unsqueeze(0), v_hist.unsqueeze(0), k_tail, v_tail, sink, recent,
                 tail_idx=idx.reshape(1, -1).contiguous(), err_flag=err_flag)


__all__ = ["ring_slot", "write_token", "write_tokens", "gather_tail", "gather_tails"]
