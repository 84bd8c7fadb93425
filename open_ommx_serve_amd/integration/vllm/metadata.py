"""Per-step host seam between a vLLM-style scheduler and the OMMX stores (reference
``integration/vllm/metadata.py:39-878``).

``build()`` of the attention-metadata builder runs on the host every step, outside any captured
region.  It hands the step's ``CommonAttentionMetadata`` (duck-typed: ``seq_lens[_cpu]``,
``query_start_loc[_cpu]``, ``block_table_tensor``) to a step manager, which
  * maps batch rows to stable pool slots (keyed by the request's first physical block),
  * packs every group that completed (one store launch per layer), and
  * refreshes fixed-address device buffers that the (capturable) forward reads.

What differs from the reference is the amount of host work per step.  The tail-gather kernel
derives boundary, packed length, tail length and tail positions from the sequence length on the
device, so the batched manager uploads ONE ``[3, B]`` int64 block per step (slot, write column,
current length) where the reference fills a ``[B, T]`` index matrix row by row and issues five
copies; the single-sequence manager uploads its write position and tail positions in one copy
and the two lengths in another, where the reference issues six small device operations.

Layout of this module: ``StepShape`` reads a metadata object once; ``SlotLedger`` owns the
key -> slot allocator (``assign_slots`` is its functional form, kept for callers of the
reference's API); ``_Stoppable`` is the "dead manager" behaviour both managers share.
"""
from __future__ import annotations

import os
import sys
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import torch

from .config import OMMXServingConfig

_UNSAFE_ROW_INDEX_ENV = "OMMX_UNSAFE_ROW_INDEX_SLOTS"
# The scheduler reserves block id 0 as its null block.  A step whose rows all show it in column 0
# names no request at all (memory-profiling and graph-capture dummies).
_NULL_BLOCK_ID = 0
# Batch size reported for a step that could not be read.  It is negative so that no consumer can
# mistake it for an empty (0) or single-request (1) step.
STEP_ROUTE_UNCLASSIFIED = -1

_LENGTH_FIELDS = ("seq_lens_cpu", "seq_lens_cpu_upper_bound", "seq_lens")
_OFFSET_FIELDS = ("query_start_loc_cpu", "query_start_loc")
_BLOCK_TABLE_FIELDS = ("block_table_tensor", "block_table")
_said: set = set()


def _flag_set(name: str) -> bool:
    return os.environ.get(name, "").strip().lower() not in ("", "0", "false", "off", "no")


def _warn_once(tag: str, text: str) -> None:
    """Print a warning the first time ``tag`` is seen in this process (metadata.py:244-262)."""
    if tag not in _said:
        _said.add(tag)
        sys.stderr.write(f"[OMMX] WARNING: {text}\n")
        sys.stderr.flush()


def _ints(value: Any) -> Optional[List[int]]:
    """A metadata field as a flat list of python ints; ``None`` when it is absent or not a
    sequence.  Device tensors are copied to the host (a synchronisation)."""
    if isinstance(value, torch.Tensor):
        return [int(x) for x in value.detach().cpu().flatten().tolist()]
    if value is None or isinstance(value, (str, bytes)):
        return None
    try:
        return [int(x) for x in value]
    except TypeError:
        return None


def _first_present(meta: Any, fields: Sequence[str]) -> Optional[List[int]]:
    for field in fields:
        got = _ints(getattr(meta, field, None))
        if got is not None:
            return got
    return None


@dataclass(frozen=True)
class StepShape:
    """What one step's metadata says about its batch: per-request lengths after the step and the
    cumulative query offsets (``None`` when the scheduler exposes none)."""
    lengths: Optional[List[int]]
    offsets: Optional[List[int]]

    @classmethod
    def read(cls, meta: Any) -> "StepShape":
        return cls(_first_present(meta, _LENGTH_FIELDS), _first_present(meta, _OFFSET_FIELDS))

    @property
    def batch(self) -> int:
        return STEP_ROUTE_UNCLASSIFIED if self.lengths is None else len(self.lengths)

    def _query_counts(self) -> Optional[List[int]]:
        if self.lengths is None or self.offsets is None or len(self.offsets) != len(self.lengths) + 1:
            return None
        return [b - a for a, b in zip(self.offsets, self.offsets[1:])]

    @property
    def one_token_each(self) -> bool:
        counts = self._query_counts()
        return bool(counts) and all(c == 1 for c in counts)

    @property
    def whole_sequences(self) -> bool:
        counts = self._query_counts()
        return bool(counts) and counts == list(self.lengths)


def detect_step_route(common_attn_metadata: Any) -> Tuple[int, bool]:
    """``(B, every request contributes exactly one query token)``; ``(-1, False)`` when the step
    cannot be read at all (metadata.py:800-840)."""
    try:
        shape = StepShape.read(common_attn_metadata)
        return shape.batch, shape.batch >= 1 and shape.one_token_each
    except Exception:
        return STEP_ROUTE_UNCLASSIFIED, False


def detect_full_prefill(common_attn_metadata: Any) -> bool:
    """True iff every request's query span is its whole sequence, so the step's own K/V hold each
    request's complete causal context; False on any doubt (metadata.py:843-873)."""
    try:
        return StepShape.read(common_attn_metadata).whole_sequences
    except Exception:
        return False


def _window_for_seam(cfg: OMMXServingConfig):
    """The attention window of a configuration, refused when it keeps no recent row: both
    managers pack completed groups BEFORE the forward writes token ``seq - 1``, which is sound
    only while that token lies behind the packed boundary (``boundary <= seq - recent``)."""
    win = cfg.window()
    if int(win.recent_window) < 1:
        raise ValueError(f"recent_window={win.recent_window}: the step seam needs at least one "
                         "recent bf16 row, or it would pack a group whose last token is unwritten")
    return win


class _Stoppable:
    """A manager that, once something went wrong at the seam, refuses further steps and keeps
    the reason (``dead`` / ``dead_reason``); ``OMMX_STRICT=1`` raises to the caller instead."""
    dead: bool = False
    dead_reason: Optional[str] = None
    _what = "OMMX store"

    def _guarded(self, work: Callable[[], None], tag: str) -> None:
        if self.dead:
            return
        try:
            work()
        except Exception as exc:
            if self.cfg.strict:
                raise
            self._stop(f"{type(exc).__name__}: {exc}", tag)

    def _stop(self, reason: str, tag: Optional[str]) -> None:
        self.dead, self.dead_reason = True, reason
        self._forget_step()
        if tag:
            _warn_once(tag, f"{self._what} stopped in this worker ({reason}); its decode route is "
                            "refused from now on.  OMMX_STRICT=1 raises at the seam instead.")

    def _forget_step(self) -> None:
        pass


# ── single request ───────────────────────────────────────────────────────────────────────

class OMMXStepManager(_Stoppable):
    """Shared fixed-address step buffers of the one-request route; drives every layer's
    ``CanonicalKVStore`` (metadata.py:39-204).

    ``write_pos [1]`` int64 (slot of the token the forward is about to write, ``seq - 1``),
    ``tail_idx [T]`` int64 (sink ++ recent absolute positions, zero padded), ``b_seq_len [1]`` /
    ``b_tail_len [1]`` int32.  The positions are absolute; the stores map them into their ring.
    """
    _what = "single-request OMMX store"

    def __init__(self, cfg: OMMXServingConfig, device: Any) -> None:
        self.cfg, self.device = cfg, torch.device(device)
        self.window = _window_for_seam(cfg)
        self.capturing = False
        self.kv_ring = _flag_set("OMMX_KV_RING")
        self._ring_rec = int(self.window.recent_window) + 2 * int(self.window.group_tokens)
        self.max_seq_len_fixed = max(int(cfg.max_context), 1)
        self.max_tail_cap = int(self.window.max_tail_len(cfg.max_context))
        # one int64 block [write position | tail positions] and one int32 pair [packed | tail]
        words = 1 + self.max_tail_cap
        self._ctl_host = torch.zeros(words, dtype=torch.long)
        self._ctl = torch.zeros(words, dtype=torch.long, device=self.device)
        self.write_pos, self.tail_idx = self._ctl[:1], self._ctl[1:]
        self._lens_host = torch.zeros(2, dtype=torch.int32)
        self._lens = torch.zeros(2, dtype=torch.int32, device=self.device)
        self.b_seq_len, self.b_tail_len = self._lens[:1], self._lens[1:]
        self._seq_pin: Optional[torch.Tensor] = None
        self.reset()

    def reset(self) -> None:
        self.stores: Dict[int, Any] = {}
        self.dead, self.dead_reason = False, None
        self.cur_seq, self._last_boundary = 0, -1

    def register(self, layer_id: int, store) -> None:
        """Attach a layer's store; a store not seen before must get the next ``advance_to``."""
        if self.stores.get(int(layer_id)) is store:
            return
        self.stores[int(layer_id)] = store
        self._last_boundary = -1

    @property
    def max_seq_len(self) -> int:
        return self.max_seq_len_fixed

    @property
    def max_tail_len(self) -> int:
        return self.max_tail_cap

    def on_build(self, common_attn_metadata: Any, *, new_request=None) -> None:
        """Host half of one step (metadata.py:95-159): read the request's length, move the stores,
        upload the step's positions and lengths."""
        def work():
            starts = detect_full_prefill(common_attn_metadata) if new_request is None else new_request
            self._refresh(self._length_of_request(common_attn_metadata), new_request=bool(starts))
        self._guarded(work, "single-store-fault")

    def _length_of_request(self, meta: Any) -> int:
        """Length of request 0: from a host copy of ``seq_lens`` when the scheduler keeps one,
        else from the device tensor through a pinned one-element buffer."""
        for field in _LENGTH_FIELDS[:2]:
            host = getattr(meta, field, None)
            if host is not None:
                return int(host[0])
        dev = getattr(meta, "seq_lens", None)
        if dev is None:
            raise RuntimeError("CommonAttentionMetadata: no seq_lens field found")
        if not (isinstance(dev, torch.Tensor) and dev.is_cuda):
            return int(dev[0])
        if self._seq_pin is None:
            self._seq_pin = torch.empty(1, dtype=dev.dtype, pin_memory=True)
        self._seq_pin.copy_(dev.reshape(-1)[:1], non_blocking=False)
        return int(self._seq_pin[0])

    def _check_ring_holds(self, seq: int, boundary: int) -> None:
        """With a ring history the rows still needed are the group being packed and everything
        after it up to the newest token; they must fit the ring span."""
        if not (self.kv_ring and seq > 0):
            return
        group = int(self.window.group_tokens)
        oldest = max(self.window.sink_tokens, boundary - group)
        needed = max(0, seq - oldest)
        if needed > self._ring_rec:
            raise AssertionError(
                f"ring history too short: {needed} rows are still live at seq={seq} "
                f"(boundary {boundary}, group {group}) but the ring spans {self._ring_rec}; "
                "rows would alias")

    def _refresh(self, seq: int, *, new_request: bool = False) -> None:
        seq = int(seq)
        edge = self.window.boundary(seq)
        self.cur_seq = seq
        # stores: a new request rewinds them in place (the writer packs the prompt after this
        # build, metadata.py:148-155); otherwise they move only when the boundary did
        if new_request or edge != self._last_boundary:
            for store in self.stores.values():
                if new_request:
                    store.reset_inplace()
                else:
                    store.advance_to(seq)
            self._last_boundary = edge
        self._check_ring_holds(seq, edge)
        positions = self.window.tail_indices(seq)[:self.max_tail_cap]
        block = self._ctl_host
        block.zero_()
        block[0] = max(seq - 1, 0)
        if positions:
            block[1:1 + len(positions)] = torch.tensor(positions, dtype=torch.long)
        self._lens_host[0], self._lens_host[1] = self.window.packed_len(seq), len(positions)
        self._ctl.copy_(block, non_blocking=True)
        self._lens.copy_(self._lens_host, non_blocking=True)


# ── slot allocator ───────────────────────────────────────────────────────────────────────

class OMMXSlotAllocationError(RuntimeError):
    """The static slot pool cannot serve this step's request set without putting two live
    requests on one slot (metadata.py:265-273)."""


def assign_slots(keys: list, key_to_slot: dict, free_slots: list, num_seqs: int) -> Tuple[list, list]:
    """Request keys of this step (batch-row order) -> pool slots (metadata.py:276-359).

    ``key_to_slot`` / ``free_slots`` are the allocator's persistent state.  The step is planned on
    copies and committed at the end, so a refused step leaves both untouched.  A key seen before
    keeps its slot whatever row it sits in now; a key that is gone returns its slot to the back
    of the free queue; a new key takes the front of the queue.  Returns ``(row -> slot, slots
    given to new keys)``; the caller clears the pool state behind the latter.  Raises
    ``OMMXSlotAllocationError`` for a key that appears twice, for more new keys than free slots,
    and for a free queue that names a slot outside the pool or one a live key holds.
    """
    pool_size = int(num_seqs)
    wanted = [int(k) for k in keys]
    rows_of: Dict[int, List[int]] = {}
    for row, key in enumerate(wanted):
        rows_of.setdefault(key, []).append(row)
    twice = {key: rows for key, rows in rows_of.items() if len(rows) > 1}
    if twice:
        raise OMMXSlotAllocationError(
            f"slot pool: duplicate request key in one step, {dict(list(sorted(twice.items()))[:8])} "
            f"(key -> batch rows, {len(wanted)} rows in all).  The key is a request's first "
            "physical block; two rows showing the same one means the scheduler shares blocks "
            "between requests (prefix caching), and both would write one slot.  Turn prefix "
            "caching off for this backend.")
    kept = {int(k): int(v) for k, v in key_to_slot.items() if int(k) in rows_of}
    given_back = [int(v) for k, v in key_to_slot.items() if int(k) not in rows_of]
    queue = [int(x) for x in free_slots] + given_back
    arrivals = [key for key in wanted if key not in kept]
    if len(arrivals) > len(queue):
        raise OMMXSlotAllocationError(
            f"slot pool EXHAUSTED: {len(kept)} request(s) stay, {len(arrivals)} arrive, "
            f"{len(queue)} of {pool_size} slots are free (first key without a slot: "
            f"{arrivals[len(queue)]}).  The pool is sized once from OMMX_ATTN_MAX_NUM_SEQS, which "
            "must cover the engine's max_num_seqs; a slot in use is never handed out again.")
    in_use = set(kept.values())
    handed: List[int] = []
    for key, slot in zip(arrivals, queue):
        if slot < 0 or slot >= pool_size:
            raise OMMXSlotAllocationError(
                f"slot pool: out-of-range slot {slot} in the free queue of a {pool_size}-slot pool")
        if slot in in_use:
            raise OMMXSlotAllocationError(
                f"slot pool: the free queue offers slot {slot}, but a live request owns it "
                f"(slots in use: {sorted(in_use)[:8]}); it was freed twice")
        in_use.add(slot)
        kept[key] = slot
        handed.append(slot)
    key_to_slot.clear()
    key_to_slot.update(kept)
    free_slots[:] = queue[len(arrivals):]
    return [kept[key] for key in wanted], handed


class SlotLedger:
    """The allocator state of one worker: which request key holds which slot, and the queue of
    free slots (oldest first)."""

    def __init__(self, size: int) -> None:
        self.size = int(size)
        self.by_key: Dict[int, int] = {}
        self.free: List[int] = list(range(self.size))

    def place(self, keys: Sequence[int]) -> Tuple[List[int], List[int]]:
        return assign_slots(list(keys), self.by_key, self.free, self.size)

    def lend(self, count: int) -> List[int]:
        """``count`` free slots for rows that are nobody's request; nothing is recorded, so the
        next real step still finds them free."""
        if count > len(self.free):
            raise OMMXSlotAllocationError(
                f"slot pool: {count} identity-less rows (null block in column 0 of every row) but "
                f"only {len(self.free)} free slot(s) out of {self.size}; such rows are never put "
                "on a slot a live request holds")
        return [int(s) for s in self.free[:count]]


# ── batch of requests ────────────────────────────────────────────────────────────────────

class OMMXBatchedStepManager(_Stoppable):
    """Host seam of the batched route: one ``MultiSeqKVPool`` per layer, one slot allocator for
    all of them (metadata.py:362-786).

    Fixed-address device buffers for the captured forward, ``cap = num_seqs`` entries each:
    ``b_sel`` (row -> slot), ``b_write_col`` (absolute write position ``seq - 1``) and
    ``b_cur_seq`` (current length) are rows of one int64 block refreshed by one copy per step;
    ``b_seq_len`` / ``b_tail_len`` (int32) are written by the tail-gather launch of the forward,
    which derives them — and the tail positions the reference keeps in ``b_tail_idx`` — from
    ``b_cur_seq`` on the device.
    """
    _what = "batched OMMX pool"

    def __init__(self, cfg: OMMXServingConfig, device: Any, num_seqs: int, graph: bool = False,
                 *, pool_cls: Optional[Callable] = None, pool_kwargs: Optional[dict] = None) -> None:
        self.cfg, self.device = cfg, torch.device(device)
        self.window = _window_for_seam(cfg)
        self.graph = bool(graph)
        self.num_seqs = self.cap = max(int(num_seqs), 1)
        self._make_pool = pool_cls
        self._pool_kwargs = dict(pool_kwargs or {})
        self.max_seq_len_fixed = max(int(cfg.max_context), 1)
        self.max_tail_cap = int(self.window.max_tail_len(cfg.max_context))
        self._ctl_host = torch.zeros(3, self.cap, dtype=torch.long)
        self._ctl = torch.zeros(3, self.cap, dtype=torch.long, device=self.device)
        self.b_sel, self.b_write_col, self.b_cur_seq = self._ctl.unbind(0)
        self.b_seq_len = torch.zeros(self.cap, dtype=torch.int32, device=self.device)
        self.b_tail_len = torch.zeros(self.cap, dtype=torch.int32, device=self.device)
        self.capturing = False
        self.pools: Dict[int, Any] = {}
        self.reset()

    def reset(self) -> None:
        self.pools.clear()
        self.dead, self.dead_reason = False, None
        self._ledger = SlotLedger(self.num_seqs)
        self._keys_are_row_index = False
        self.step_tables = None
        self._forget_step()
        self.q_start: Optional[List[int]] = []

    def _forget_step(self) -> None:
        """No step is current: nothing captured may run on the previous step's slots."""
        self.seq_lens: List[int] = []
        self.slots: List[int] = []
        self.cur_B = 0
        self.is_uniform_decode = False

    # the allocator state under the names callers of the reference's manager know
    @property
    def _key_to_slot(self) -> Dict[int, int]:
        return self._ledger.by_key

    @property
    def _free_slots(self) -> List[int]:
        return self._ledger.free

    @property
    def max_seq_len(self) -> int:
        return self.max_seq_len_fixed

    @property
    def max_tail_len(self) -> int:
        return self.max_tail_cap

    def pool(self, layer_id: int, device: Any):
        """The layer's pool, built on first use from the serving configuration."""
        key = int(layer_id)
        if key not in self.pools:
            make = self._make_pool
            if make is None:
                from ...attention.kv_pool import MultiSeqKVPool as make
            cfg = self.cfg
            self.pools[key] = make(head_dim=cfg.head_dim, n_kv_heads=cfg.n_kv_heads,
                                   num_seqs=self.num_seqs, max_seq_len=int(cfg.max_context),
                                   device=device, **cfg.store_kwargs(), **self._pool_kwargs)
        return self.pools[key]

    # ── host seam ────────────────────────────────────────────────────────────────

    def on_build(self, common_attn_metadata: Any) -> None:
        """Host half of one batched step.  Any failure stops the manager for this worker (reason
        kept in ``dead_reason``); with ``OMMX_STRICT=1`` it is raised to the caller instead."""
        self._guarded(lambda: self._refresh(common_attn_metadata), "batched-seam-fault")

    def _refresh(self, meta: Any) -> None:
        shape = StepShape.read(meta)
        if shape.lengths is None:
            raise RuntimeError("CommonAttentionMetadata: no seq_lens field found")
        rows = len(shape.lengths)
        if rows > self.num_seqs:
            # more rows than the pool has slots only happens for the engine's start-up dummies:
            # there is nothing to store, and the next real step must still be served
            # (metadata.py:526-539)
            self._forget_step()
            self.q_start = None
            return
        self.seq_lens, self.q_start = list(shape.lengths), shape.offsets
        self.slots = self._slots(meta, rows)
        self.is_uniform_decode = rows > 0 and shape.one_token_each
        # (The reference also runs its planner here, every step, for per-slot regroup deltas that
        # only its own pools read; the pools here count their packed groups themselves, and the
        # planner's position matrix costs more host time than the rest of the seam.)
        if self.graph and self.is_uniform_decode:
            self._refresh_graph_buffers(self.seq_lens, self.slots)

    def _refresh_graph_buffers(self, seq_lens: List[int], slots: List[int]) -> None:
        """Advance every pool to this step's lengths, pack what completed, refresh the device
        block (metadata.py:558-643).  The step's own token (``seq - 1``) is written by the forward
        after this seam; it lies in the bf16 tail (``boundary <= seq - recent``), so packing never
        needs it.  A pool may therefore be exactly one token behind and no more: a larger gap
        means rows nobody wrote would be packed, and the manager stops instead."""
        pairs = [(int(slot), int(seq)) for slot, seq in zip(slots, seq_lens)]
        for slot, seq in pairs:
            for pool in self.pools.values():
                written = int(pool.seq_len[slot])
                if seq - written > 1:
                    self._stop(
                        f"slot {slot}: pool holds {written} written tokens, the scheduler reports "
                        f"seq={seq} ({seq - written - 1} never reached the pool).  Regrouping to "
                        f"seq would pack unwritten rows into "
                        f"{self.window.num_groups(seq) - int(pool.packed_groups[slot])} group(s).",
                        f"seam-seq-ahead-{slot}")
                    return
                pool.seq_len[slot] = seq
                if self.window.num_groups(seq) > pool.packed_groups[slot]:
                    pool.regroup(slot)
        n = len(pairs)
        self.cur_B = n
        self.step_tables = None      # (req_to_token, req_to_group) rows of this step, set by the first layer
        self._ctl_host[:, :n] = torch.tensor(
            [[slot for slot, _ in pairs], [max(seq - 1, 0) for _, seq in pairs], [seq for _, seq in pairs]],
            dtype=torch.long).reshape(3, n)
        self._ctl[:, :n].copy_(self._ctl_host[:, :n], non_blocking=True)

    @staticmethod
    def _first_blocks(table: Any, B: int) -> List[int]:
        """Column 0 of the first ``B`` rows of a block table (tensor, array or nested list)."""
        column = table[:B, 0] if hasattr(table, "shape") else [row[0] for row in list(table)[:B]]
        values = _ints(column)
        if values is None or len(values) != B:
            got = "nothing" if values is None else f"{len(values)} entries"
            raise ValueError(f"column 0 gave {got} for {B} rows")
        return values

    def _req_keys(self, common: Any, B: int) -> List[int]:
        """One key per batch row: the id of the request's first physical block, which stays with
        the request when the scheduler reorders rows (metadata.py:660-720).  A step without a
        readable block table has no such identity and is refused, unless
        ``OMMX_UNSAFE_ROW_INDEX_SLOTS=1`` accepts the row index (single-request benches)."""
        tried: Dict[str, str] = {}
        for field in _BLOCK_TABLE_FIELDS:
            table = getattr(common, field, None)
            if table is None:
                tried[field] = "absent"
                continue
            try:
                keys = self._first_blocks(table, B)
            except Exception as exc:
                tried[field] = f"{type(exc).__name__}: {exc}"
                continue
            self._keys_are_row_index = False
            return keys
        why = ", ".join(f"{k}: {v}" for k, v in tried.items())
        if not _flag_set(_UNSAFE_ROW_INDEX_ENV):
            raise OMMXSlotAllocationError(
                f"slot pool: this step has no readable block table ({why}), hence no request "
                "identity to key slots by, and batch rows move between steps.  "
                f"{_UNSAFE_ROW_INDEX_ENV}=1 accepts row indices for a one-request bench.")
        _warn_once("row-index-slots",
                   f"{_UNSAFE_ROW_INDEX_ENV}=1 and no readable block table ({why}): slots follow "
                   "the batch ROW INDEX.  Any reordering of the batch swaps KV between requests.")
        self._keys_are_row_index = True
        return list(range(B))

    def _slots(self, meta: Any, rows: int) -> List[int]:
        """Slots of this step's rows.  A step without rows changes nothing (in particular it
        frees nothing); a step whose rows all carry the null block borrows free slots
        (metadata.py:733-764); any other step goes through the ledger."""
        if rows < 1:
            return []
        keys = self._req_keys(meta, rows)
        anonymous = not self._keys_are_row_index and set(keys) == {_NULL_BLOCK_ID}
        if anonymous:
            borrowed = self._ledger.lend(rows)
            if not self.capturing:
                _warn_once("null-block-keys",
                           f"a step of {rows} row(s) shows the null block in column 0 of every "
                           "block-table row; it is served as a start-up / profiling dummy on "
                           "free slots.  If requests are live, their identity is lost.")
            return borrowed
        placed, newly = self._ledger.place(keys)
        for slot in newly:
            # the slot's cursors still describe whoever held it before, and packing only ever
            # moves forward: start the newcomer from zero in every layer
            for pool in self.pools.values():
                pool.seq_len[slot] = pool.packed_groups[slot] = 0
        return placed


__all__ = ["OMMXStepManager", "OMMXBatchedStepManager", "OMMXSlotAllocationError", "SlotLedger",
           "StepShape", "assign_slots", "detect_step_route", "detect_full_prefill",
           "STEP_ROUTE_UNCLASSIFIED"]
