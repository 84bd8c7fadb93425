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
"""
from __future__ import annotations

import os
import sys
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

from ..common.batched_seam import BatchedStepPlanner
from .config import OMMXServingConfig

_OFF = {"", "0", "false", "off", "no"}
_UNSAFE_ROW_INDEX_ENV = "OMMX_UNSAFE_ROW_INDEX_SLOTS"
# Block id 0 is the scheduler's reserved null block: a step whose every row shows it in column 0
# carries no request identity (memory-profiling and capture dummies).
_NULL_BLOCK_ID = 0
_WARNED_ONCE: set = set()

# ``B`` of a step that could not be classified at all.  Negative on purpose: 0 is a genuinely
# empty batch and 1 a single request; consumers must refuse this value, not treat it as small.
STEP_ROUTE_UNCLASSIFIED = -1


def _env_on(name: str) -> bool:
    return os.environ.get(name, "").strip().lower() not in _OFF


def _warn_once(key: str, msg: str) -> None:
    """One warning per process and key, on stderr (metadata.py:244-262)."""
    if key in _WARNED_ONCE:
        return
    _WARNED_ONCE.add(key)
    print(f"[OMMX] WARNING: {msg}", file=sys.stderr, flush=True)


def _host_list(v: Any) -> Optional[list]:
    """Metadata field (tensor / numpy / list) -> python list of ints, or None."""
    if v is None:
        return None
    if isinstance(v, torch.Tensor):
        return v.detach().to("cpu").reshape(-1).tolist()
    try:
        return [int(x) for x in v]
    except TypeError:
        return None


def _first_field(common: Any, names) -> Optional[list]:
    for attr in names:
        lst = _host_list(getattr(common, attr, None))
        if lst is not None:
            return [int(x) for x in lst]
    return None


_SEQ_FIELDS = ("seq_lens_cpu", "seq_lens_cpu_upper_bound", "seq_lens")
_QSL_FIELDS = ("query_start_loc_cpu", "query_start_loc")


# ── single request ───────────────────────────────────────────────────────────────────────

class OMMXStepManager:
    """Shared fixed-address step buffers of the one-request route; drives every layer's
    ``CanonicalKVStore`` (metadata.py:39-204).

    ``write_pos [1]`` int64 (slot of the token the forward is about to write, ``seq - 1``),
    ``tail_idx [T]`` int64 (sink ++ recent absolute positions, zero padded), ``b_seq_len [1]`` /
    ``b_tail_len [1]`` int32.  The positions are absolute; the stores map them into their ring.
    """

    def __init__(self, cfg: OMMXServingConfig, device: Any) -> None:
        self.cfg = cfg
        self.device = torch.device(device)
        self.window = cfg.window()
        self.stores: Dict[int, Any] = {}
        self.dead = False
        self.dead_reason: Optional[str] = None
        self.capturing = False
        dev = self.device
        t_max = int(self.window.max_tail_len(cfg.max_context))
        self.max_tail_cap = t_max
        self._ctl = torch.zeros(1 + t_max, dtype=torch.long, device=dev)
        self._ctl_host = torch.zeros(1 + t_max, dtype=torch.long)
        self.write_pos = self._ctl[:1]
        self.tail_idx = self._ctl[1:]
        self._lens = torch.zeros(2, dtype=torch.int32, device=dev)
        self._lens_host = torch.zeros(2, dtype=torch.int32)
        self.b_seq_len = self._lens[:1]
        self.b_tail_len = self._lens[1:]
        self.max_seq_len_fixed = max(1, int(cfg.max_context))
        self.cur_seq = 0
        self.kv_ring = _env_on("OMMX_KV_RING")
        gt = int(self.window.group_tokens)
        self._ring_rec = int(self.window.recent_window) + 2 * gt
        self._last_boundary = -1
        self._seq_pin = None

    def register(self, layer_id: int, store) -> None:
        layer_id = int(layer_id)
        if self.stores.get(layer_id) is not store:
            self.stores[layer_id] = store
            self._last_boundary = -1       # a new store must see the next advance_to

    def reset(self) -> None:
        self.stores = {}
        self.cur_seq = 0
        self.dead = False
        self.dead_reason = None
        self._last_boundary = -1

    def on_build(self, common_attn_metadata: Any, *, new_request=None) -> None:
        if self.dead:
            return
        try:
            seq = self._current_seq(common_attn_metadata)
            if new_request is None:
                new_request = detect_full_prefill(common_attn_metadata)
            self._refresh(seq, new_request=bool(new_request))
        except Exception as exc:
            if self.cfg.strict:
                raise
            self.dead = True
            self.dead_reason = f"{type(exc).__name__}: {exc}"
            _warn_once("single-store-fault",
                       f"{self.dead_reason}\n  -> the single-sequence OMMX store is dead for this "
                       "worker; the backend refuses its decode route from here.  Set "
                       "OMMX_STRICT=1 to re-raise at the seam instead.")

    def _current_seq(self, common: Any) -> int:
        for attr in ("seq_lens_cpu", "seq_lens_cpu_upper_bound"):
            v = getattr(common, attr, None)
            if v is not None:
                return int(v[0])
        v = getattr(common, "seq_lens", None)
        if v is None:
            raise RuntimeError("CommonAttentionMetadata: no seq_lens field found")
        if isinstance(v, torch.Tensor) and v.is_cuda:
            if self._seq_pin is None:
                self._seq_pin = torch.empty(1, dtype=v.dtype, pin_memory=True)
            self._seq_pin.copy_(v.reshape(-1)[:1], non_blocking=False)
            return int(self._seq_pin[0])
        return int(v[0])

    def _refresh(self, seq: int, *, new_request: bool = False) -> None:
        seq = int(seq)
        self.cur_seq = seq
        win = self.window
        sink = win.sink_tokens
        boundary = win.boundary(seq)
        if new_request:
            # This build precedes the prompt's write: only the cursors move, every tensor keeps
            # its address; the writer packs the prompt (metadata.py:148-155).
            for st in self.stores.values():
                st.reset_inplace()
            self._last_boundary = boundary
        elif boundary != self._last_boundary:
            for st in self.stores.values():
                st.advance_to(seq)
            self._last_boundary = boundary
        valid_sink = min(sink, seq)
        n_rec = max(0, seq - boundary)
        if self.kv_ring and seq > 0:
            gt = int(win.group_tokens)
            lo = max(sink, boundary - gt)
            live_span = max(0, (seq - 1) - lo + 1)
            if live_span > self._ring_rec:
                raise AssertionError(
                    f"OMMX_KV_RING live span {live_span} > ring span {self._ring_rec} "
                    f"(seq={seq}, boundary={boundary}, gt={gt}): live rows would alias")
        if valid_sink + n_rec > self.max_tail_cap:
            n_rec = self.max_tail_cap - sink
        n_tail = valid_sink + n_rec
        h = self._ctl_host
        h.zero_()
        h[0] = max(0, seq - 1)
        if valid_sink:
            h[1:1 + valid_sink] = torch.arange(valid_sink)
        if n_rec > 0:
            h[1 + valid_sink:1 + n_tail] = torch.arange(boundary, boundary + n_rec)
        self._lens_host[0] = max(0, boundary - sink)
        self._lens_host[1] = n_tail
        self._ctl.copy_(h, non_blocking=True)
        self._lens.copy_(self._lens_host, non_blocking=True)

    @property
    def max_seq_len(self) -> int:
        return self.max_seq_len_fixed

    @property
    def max_tail_len(self) -> int:
        return self.max_tail_cap


# ── slot allocator ───────────────────────────────────────────────────────────────────────

class OMMXSlotAllocationError(RuntimeError):
    """The static slot pool cannot serve this step's request set without putting two live
    requests on one slot (metadata.py:265-273)."""


def assign_slots(keys: list, key_to_slot: dict, free_slots: list, num_seqs: int) -> Tuple[list, list]:
    """Request keys of this step (batch-row order) -> pool slots (metadata.py:276-359).

    ``key_to_slot`` / ``free_slots`` are the persistent allocator state and are changed in
    place: keys that left the batch give their slot back, new keys take the oldest free one.
    Returns ``(row -> slot, slots handed to a new key)``; the caller clears the pool state behind
    the latter.  Raises ``OMMXSlotAllocationError`` — before touching the state — on duplicate
    keys, and on exhaustion or a corrupt free list; it never hands out a slot a live request owns.
    """
    num_seqs = int(num_seqs)
    keys = [int(k) for k in keys]
    if len(set(keys)) != len(keys):
        dup = sorted({k for k in keys if keys.count(k) > 1})
        raise OMMXSlotAllocationError(
            f"OMMX batched slot pool: {len(dup)} duplicate request key(s) {dup[:8]} in a batch of "
            f"{len(keys)} rows (keys[:16]={keys[:16]}).  Two rows share their first physical block "
            "(prefix caching hands requests with a common prompt prefix one block), so the block "
            "id no longer names one request and both rows would write one slot.  Run the OMMX "
            "backend with prefix caching off (enable_prefix_caching=False).")
    live = set(keys)
    for k in list(key_to_slot):
        if k not in live:
            free_slots.append(int(key_to_slot.pop(k)))
    owned = set(int(v) for v in key_to_slot.values())
    out: list = []
    fresh: list = []
    for k in keys:
        slot = key_to_slot.get(k)
        if slot is None:
            if not free_slots:
                raise OMMXSlotAllocationError(
                    f"OMMX batched slot pool EXHAUSTED: {len(key_to_slot)} live request key(s) "
                    f"hold all {num_seqs} slots and request key {k} has nowhere to go.  The pool "
                    "is sized once at OMMX_ATTN_MAX_NUM_SEQS and must be >= the engine's "
                    "max_num_seqs.  (A live slot is never recycled: two requests on one slot "
                    "overwrite each other's KV.)")
            slot = int(free_slots.pop(0))
            if not 0 <= slot < num_seqs:
                raise OMMXSlotAllocationError(
                    f"OMMX batched slot pool: free list yielded out-of-range slot {slot} "
                    f"(num_seqs={num_seqs}); the allocator state is corrupt.")
            if slot in owned:
                raise OMMXSlotAllocationError(
                    f"OMMX batched slot pool: free list yielded slot {slot}, which a live request "
                    f"already owns (owned={sorted(owned)[:8]}): double-freed slot, refusing to "
                    "alias two requests onto it.")
            key_to_slot[k] = slot
            owned.add(slot)
            fresh.append(slot)
        out.append(int(slot))
    return out, fresh


# ── batch of requests ────────────────────────────────────────────────────────────────────

class OMMXBatchedStepManager:
    """Host seam of the batched route: one ``MultiSeqKVPool`` per layer, one slot allocator for
    all of them (metadata.py:362-786).

    Fixed-address device buffers for the captured forward, ``cap = num_seqs`` entries each:
    ``b_sel`` (row -> slot), ``b_write_col`` (absolute write position ``seq - 1``) and
    ``b_cur_seq`` (current length) are rows of one int64 block refreshed by one copy per step;
    ``b_seq_len`` / ``b_tail_len`` (int32) are written by the tail-gather launch of the forward,
    which derives them — and the tail positions the reference keeps in ``b_tail_idx`` — from
    ``b_cur_seq`` on the device.
    """

    def __init__(self, cfg: OMMXServingConfig, device: Any, num_seqs: int, graph: bool = False,
                 *, pool_cls: Optional[Callable] = None, pool_kwargs: Optional[dict] = None) -> None:
        self._pool_cls = pool_cls
        self._pool_kwargs = dict(pool_kwargs or {})
        self.cfg = cfg
        self.device = torch.device(device)
        self.window = cfg.window()
        self.graph = bool(graph)
        self.num_seqs = max(1, int(num_seqs))
        self.dead = False
        self.dead_reason: Optional[str] = None
        self.pools: Dict[int, Any] = {}
        self.planner = BatchedStepPlanner(self.window, cfg.max_context)
        self.seq_lens: List[int] = []
        self.q_start: Optional[List[int]] = []
        self.slots: List[int] = []
        self.is_uniform_decode = False
        self.max_seq_len_fixed = max(1, int(cfg.max_context))
        cap = self.num_seqs
        dev = self.device
        self.cap = cap
        self.max_tail_cap = int(self.window.max_tail_len(cfg.max_context))
        self._ctl = torch.zeros(3, cap, dtype=torch.long, device=dev)
        self._ctl_host = torch.zeros(3, cap, dtype=torch.long)
        self.b_sel, self.b_write_col, self.b_cur_seq = self._ctl[0], self._ctl[1], self._ctl[2]
        self.b_seq_len = torch.zeros(cap, dtype=torch.int32, device=dev)
        self.b_tail_len = torch.zeros(cap, dtype=torch.int32, device=dev)
        self.cur_B = 0
        self.step_tables = None
        self.capturing = False
        self._key_to_slot: Dict[int, int] = {}
        self._free_slots: List[int] = list(range(self.num_seqs))
        self._keys_are_row_index = False

    # ── pools ─────────────────────────────────────────────────────────────────────

    def pool(self, layer_id: int, device: Any):
        p = self.pools.get(int(layer_id))
        if p is None:
            cls = self._pool_cls
            if cls is None:
                from ...attention.kv_pool import MultiSeqKVPool as cls
            c = self.cfg
            p = cls(head_dim=c.head_dim, n_kv_heads=c.n_kv_heads, num_seqs=self.num_seqs,
                    max_seq_len=int(c.max_context), device=device, **c.store_kwargs(),
                    **self._pool_kwargs)
            self.pools[int(layer_id)] = p
        return p

    def reset(self) -> None:
        self.pools = {}
        self.planner.reset()
        self.seq_lens, self.q_start, self.slots = [], [], []
        self.is_uniform_decode = False
        self.dead = False
        self.dead_reason = None
        self._key_to_slot = {}
        self._free_slots = list(range(self.num_seqs))
        self._keys_are_row_index = False
        self.cur_B = 0
        self.step_tables = None

    # ── host seam ────────────────────────────────────────────────────────────────

    def on_build(self, common_attn_metadata: Any) -> None:
        if self.dead:
            return
        try:
            self._refresh(common_attn_metadata)
        except OMMXSlotAllocationError as exc:
            _warn_once("slot-fault", f"{exc}\n  -> the OMMX batched pool is dead for this worker. "
                       "Set OMMX_STRICT=1 to fail hard instead.")
            if self.cfg.strict:
                raise
            self.dead = True
            self.dead_reason = f"{type(exc).__name__}: {exc}"
        except Exception as exc:
            if self.cfg.strict:
                raise
            self.dead = True
            self.dead_reason = f"{type(exc).__name__}: {exc}"
            _warn_once("batched-refresh-fault", f"{self.dead_reason}\n  -> the OMMX batched pool is "
                       "dead for this worker.  Set OMMX_STRICT=1 to re-raise instead.")

    def _refresh(self, common: Any) -> None:
        seq_lens = self._seq_lens(common)
        q_start = self._query_start_loc(common)
        B = len(seq_lens)
        self.seq_lens, self.q_start = seq_lens, q_start
        if B > self.num_seqs:
            # An init dummy batch larger than the pool: nothing real to store.  Not a fault, the
            # next real step must still route (metadata.py:526-539).
            self.seq_lens, self.q_start, self.slots = [], None, []
            self.is_uniform_decode = False
            self.cur_B = 0
            return
        self.slots = self._slots(common, B)
        self.is_uniform_decode = bool(
            q_start is not None and len(q_start) == B + 1
            and all(q_start[i + 1] - q_start[i] == 1 for i in range(B)))
        # (The reference also runs its planner here, every step, for per-slot regroup deltas that
        # only its own pools read; the pools here count their packed groups themselves, and the
        # planner's position matrix costs more host time than the rest of the seam.)
        if B and self.is_uniform_decode and self.graph:
            self._refresh_graph_buffers(seq_lens, self.slots)

    def _refresh_graph_buffers(self, seq_lens: List[int], slots: List[int]) -> None:
        """Advance every pool to this step's lengths, pack what completed, refresh the device
        block (metadata.py:558-643).  The step's own token (``seq - 1``) is written by the forward
        after this seam; it lies in the bf16 tail (``boundary <= seq - recent``), so packing never
        needs it.  A pool may therefore be exactly one token behind and no more: a larger gap
        means rows nobody wrote would be packed, and the manager stops instead."""
        B = len(seq_lens)
        win = self.window
        cols: List[int] = []
        for i in range(B):
            r, seq = int(slots[i]), int(seq_lens[i])
            for pool in self.pools.values():
                prev = int(pool.seq_len[r])
                if seq > prev + 1:
                    self.dead = True
                    self.dead_reason = (
                        f"slot {r}: pool holds {prev} written tokens, the scheduler reports "
                        f"seq={seq} ({seq - prev - 1} never reached the pool).  Regrouping to seq "
                        f"would pack unwritten rows into "
                        f"{win.num_groups(seq) - int(pool.packed_groups[r])} group(s).")
                    _warn_once(f"seam-seq-ahead-{r}", "OMMX batched-graph disabled: " + self.dead_reason)
                    return
                pool.seq_len[r] = seq
                if win.num_groups(seq) > pool.packed_groups[r]:
                    pool.regroup(r)
            cols.append(max(0, seq - 1))
        self.cur_B = B
        self.step_tables = None        # (req_to_token, req_to_group) rows of this step, set by the first layer
        self._ctl_host[:, :B] = torch.tensor([[int(r) for r in slots], cols, [int(x) for x in seq_lens]],
                                             dtype=torch.long)
        self._ctl[:, :B].copy_(self._ctl_host[:, :B], non_blocking=True)

    def _seq_lens(self, common: Any) -> List[int]:
        lst = _first_field(common, _SEQ_FIELDS)
        if lst is None:
            raise RuntimeError("CommonAttentionMetadata: no seq_lens field found")
        return lst

    def _query_start_loc(self, common: Any) -> Optional[List[int]]:
        return _first_field(common, _QSL_FIELDS)

    def _req_keys(self, common: Any, B: int) -> List[int]:
        """First physical block id per row: the only request identity that survives the
        scheduler's row reordering (metadata.py:660-720).  Without a block table this raises,
        unless ``OMMX_UNSAFE_ROW_INDEX_SLOTS=1`` accepts row indices (one-request benches)."""
        causes: List[str] = []
        for attr in ("block_table_tensor", "block_table"):
            bt = getattr(common, attr, None)
            if bt is None:
                causes.append(f"{attr}=absent")
                continue
            try:
                host = _host_list(bt[:B, 0] if hasattr(bt, "shape") else bt)
                if host is None:
                    raise TypeError(f"{type(bt).__name__} column 0 did not coerce to a host list")
                keys = [int(x) for x in host[:B]]
            except Exception as exc:
                causes.append(f"{attr}={type(exc).__name__}: {exc}")
                continue
            if len(keys) != B:
                causes.append(f"{attr}=got {len(keys)} column-0 entries for B={B}")
                continue
            self._keys_are_row_index = False
            return keys
        detail = "; ".join(causes) if causes else "no candidates"
        if _env_on(_UNSAFE_ROW_INDEX_ENV):
            _warn_once("row-index-slots",
                       f"{_UNSAFE_ROW_INDEX_ENV}=1: no usable block table ({detail}); pool slots are "
                       "keyed by BATCH ROW INDEX.  Safe only while the batch order cannot change; "
                       "under continuous batching this swaps KV between requests.")
            self._keys_are_row_index = True
            return list(range(B))
        raise OMMXSlotAllocationError(
            f"OMMX batched slot pool: no usable per-request block table ({detail}), so there is no "
            "stable request identity to key pool slots by.  Refusing the batch row index: rows are "
            f"reordered across steps.  For a one-request bench set {_UNSAFE_ROW_INDEX_ENV}=1.")

    def _slots(self, common: Any, B: int) -> List[int]:
        if B <= 0:
            return []          # a request-less step releases nothing
        keys = self._req_keys(common, B)
        if not self._keys_are_row_index and all(k == _NULL_BLOCK_ID for k in keys):
            # Dummy batch without identity: rows go onto currently free slots and are not
            # registered, so no live request's slot is touched (metadata.py:733-764).
            if len(self._free_slots) < B:
                raise OMMXSlotAllocationError(
                    f"OMMX batched slot pool: dummy batch of B={B} rows (every column 0 is the "
                    f"null block) but only {len(self._free_slots)} free slot(s) of {self.num_seqs}; "
                    "refusing to place dummy rows on live requests' slots.")
            if not self.capturing:
                _warn_once("null-block-keys",
                           f"OMMX batched slots: every row of a B={B} step shows the null block in "
                           "block-table column 0; treated as an init / profiling dummy.  During "
                           "real serving this means request identity is broken.")
            return [int(s) for s in self._free_slots[:B]]
        slots, fresh = assign_slots(keys, self._key_to_slot, self._free_slots, self.num_seqs)
        for slot in fresh:
            # A recycled slot still names the previous occupant's groups, and packing only moves
            # forward, so its cursors are cleared where the assignment is known to be new.
            for pool in self.pools.values():
                pool.seq_len[slot] = 0
                pool.packed_groups[slot] = 0
            self.planner.reset(slot)
        return slots

    @property
    def max_seq_len(self) -> int:
        return self.max_seq_len_fixed

    @property
    def max_tail_len(self) -> int:
        return self.max_tail_cap


# ── step classification ──────────────────────────────────────────────────────────────────

def detect_step_route(common_attn_metadata: Any) -> Tuple[int, bool]:
    """``(B, every request contributes exactly one query token)``; ``(-1, False)`` when the step
    cannot be read at all (metadata.py:800-840)."""
    try:
        seq_lens = _first_field(common_attn_metadata, _SEQ_FIELDS)
        if seq_lens is None:
            return STEP_ROUTE_UNCLASSIFIED, False
        B = len(seq_lens)
        q_start = _first_field(common_attn_metadata, _QSL_FIELDS)
        uniform = bool(B >= 1 and q_start is not None and len(q_start) == B + 1
                       and all(q_start[i + 1] - q_start[i] == 1 for i in range(B)))
        return B, uniform
    except Exception:
        return STEP_ROUTE_UNCLASSIFIED, False


def detect_full_prefill(common_attn_metadata: Any) -> bool:
    """True iff every request's query span is its whole sequence, so the step's own K/V hold each
    request's complete causal context; False on any doubt (metadata.py:843-873)."""
    try:
        seq_lens = _first_field(common_attn_metadata, _SEQ_FIELDS)
        if not seq_lens:
            return False
        B = len(seq_lens)
        q_start = _first_field(common_attn_metadata, _QSL_FIELDS)
        if q_start is None or len(q_start) != B + 1:
            return False
        return all(q_start[i + 1] - q_start[i] == seq_lens[i] for i in range(B))
    except Exception:
        return False


__all__ = ["OMMXStepManager", "OMMXBatchedStepManager", "OMMXSlotAllocationError",
           "assign_slots", "detect_step_route", "detect_full_prefill", "STEP_ROUTE_UNCLASSIFIED"]
