"""Attention-backend surface over the OMMX store and decode operators (reference
``integration/vllm/backend.py:988-2119``).

Three classes with the reference's names and method signatures:

* ``OMMXCanonicalMetadataBuilder.build(common_prefix_len, common_attn_metadata)`` — classifies the
  step (``detect_step_route`` / ``detect_full_prefill``), decides the write and read routes and
  runs the step managers' host seam;
* ``OMMXCanonicalImpl.do_kv_cache_update(layer, key, value, kv_cache, slot_mapping)`` — the step's
  K/V rows go into the layer's ``CanonicalKVStore`` (one request) or ``MultiSeqKVPool`` (batch),
  which quantize completed groups on store;
* ``OMMXCanonicalImpl.forward(layer, query, key, value, kv_cache, attn_metadata, output)`` — a
  uniform one-token step runs the paged decode operator over the packed planes and the bf16 tail;
  a full-prefill step attends causally over the step's own K/V.

The OMMX planes are the only KV cache (the reference's packed-only mode): ``kv_cache`` and
``slot_mapping`` are accepted and ignored, there is no bf16 shadow cache and therefore nothing to
fall back to — a step that cannot be served raises.  Chunked prefill and prefix caching are
refused like in the reference's packed-only mode (``backend.py:1846-1918``).

vLLM is not a dependency.  When ``vllm`` is importable the three classes take vLLM's
FlashAttention backend / builder / impl as bases, so the engine's plugin loader accepts them;
otherwise they are plain classes with the same methods, which is what the tests drive with
duck-typed metadata (``seq_lens``, ``query_start_loc``, ``block_table_tensor``).
"""
from __future__ import annotations

import math
import os
from typing import Any, Callable, Dict, Optional

import torch

from ...attention.kv_store import CanonicalKVStore
from ...attention.reference_op import ommx_paged_decode
from .config import OMMXServingConfig, resolve_serving_config
from .metadata import (STEP_ROUTE_UNCLASSIFIED, OMMXBatchedStepManager, OMMXStepManager,
                       detect_full_prefill, detect_step_route)

try:                                                     # engine present: real bases
    from vllm.v1.attention.backends.flash_attn import (FlashAttentionBackend as _BackendBase,
                                                       FlashAttentionImpl as _ImplBase,
                                                       FlashAttentionMetadataBuilder as _BuilderBase)
    HAVE_VLLM = True
except Exception:                                        # standalone: same surface, no engine
    _BackendBase = _ImplBase = _BuilderBase = object
    HAVE_VLLM = False

OMMX_BACKEND_CLASS_PATH = "open_ommx_serve_amd.integration.vllm.backend.OMMXCanonicalBackend"
_OFF = {"", "0", "false", "off", "no"}


def _env_on(name: str) -> bool:
    return os.environ.get(name, "").strip().lower() not in _OFF


def _env_int(name: str, default: int) -> int:
    v = os.environ.get(name, "").strip()
    return int(v) if v else int(default)


class _WorkerState:
    """Per-worker step state shared by the builder and every layer's impl (the reference keeps
    the same items as module globals, ``backend.py:100-165, 814-831``)."""

    def __init__(self) -> None:
        self.configure()

    def configure(self, *, graph: Optional[bool] = None, batched: Optional[bool] = None,
                  batched_graph: Optional[bool] = None, max_num_seqs: Optional[int] = None) -> None:
        self.graph = _env_on("OMMX_ATTN_GRAPH") if graph is None else bool(graph)
        self.batched_graph = (_env_on("OMMX_ATTN_BATCHED_GRAPH") if batched_graph is None
                              else bool(batched_graph))
        pre = _env_on("OMMX_ATTN_BATCHED") if batched is None else bool(batched)
        self.batched_session = bool(pre or self.batched_graph)
        self.max_num_seqs = (_env_int("OMMX_ATTN_MAX_NUM_SEQS", 256) if max_num_seqs is None
                             else int(max_num_seqs))
        self.step: Dict[str, Any] = {"B": 0, "uniform": False, "full_prefill": False,
                                     "batched_write": False, "batched_read": False}
        self.last_common = None
        self.manager: Optional[OMMXStepManager] = None
        self.bmanager: Optional[OMMXBatchedStepManager] = None
        self.fires = {"single": 0, "batched": 0, "prefill": 0}


_STATE = _WorkerState()


def reset_worker_state(**kw) -> _WorkerState:
    """Drop managers, stores and counters; re-read the route switches (``graph``, ``batched``,
    ``batched_graph``, ``max_num_seqs``) from the arguments or the environment."""
    _STATE.configure(**kw)
    return _STATE


def ommx_route_health() -> dict:
    """How many steps each route served, and whether a manager went dead
    (``backend.py:600-700``)."""
    s = _STATE
    return {"decode_single": s.fires["single"], "decode_batched": s.fires["batched"],
            "prefill": s.fires["prefill"],
            "single_dead": bool(s.manager and s.manager.dead),
            "batched_dead": bool(s.bmanager and s.bmanager.dead),
            "dead_reason": (s.manager and s.manager.dead_reason) or
                           (s.bmanager and s.bmanager.dead_reason) or None}


def _manager(cfg: OMMXServingConfig, device) -> OMMXStepManager:
    if _STATE.manager is None:
        _STATE.manager = OMMXStepManager(cfg, device)
    return _STATE.manager


def _bmanager(cfg: OMMXServingConfig, device) -> OMMXBatchedStepManager:
    if _STATE.bmanager is None:
        _STATE.bmanager = OMMXBatchedStepManager(cfg, device, _STATE.max_num_seqs,
                                                 graph=_STATE.batched_graph)
    return _STATE.bmanager


# ── metadata builder ─────────────────────────────────────────────────────────────────────

class OMMXCanonicalMetadataBuilder(_BuilderBase):
    def build(self, common_prefix_len, common_attn_metadata, fast_build=False):
        if HAVE_VLLM:
            md = super().build(common_prefix_len=common_prefix_len,
                               common_attn_metadata=common_attn_metadata, fast_build=fast_build)
        else:
            md = common_attn_metadata
        self._ommx_on_build(common_attn_metadata)
        return md

    @staticmethod
    def _ommx_on_build(common) -> None:
        """Route decisions of one step (``backend.py:1080-1151``)."""
        s = _STATE
        s.last_common = common
        B, uniform = detect_step_route(common)
        st = s.step
        st["B"], st["uniform"] = int(B), bool(uniform)
        if B == STEP_ROUTE_UNCLASSIFIED and (s.graph or s.batched_graph):
            raise RuntimeError("OMMX refuses graph replay with unclassified batch metadata")
        st["full_prefill"] = detect_full_prefill(common)
        if s.graph and B > 1:
            raise RuntimeError(
                "OMMX_ATTN_GRAPH supports one request only; restart with OMMX_ATTN_GRAPH=0 and "
                "OMMX_ATTN_BATCHED_GRAPH=1 for batched serving.")
        if not s.graph and B > 1:
            if not s.batched_session and not st["full_prefill"]:
                raise RuntimeError(
                    "OMMX cannot migrate a live single-sequence KV history into the batched pool. "
                    "Set OMMX_ATTN_BATCHED=1 before starting the engine for staggered requests, or "
                    "submit a full batched prefill.")
            s.batched_session = True
        in_batched = bool(s.batched_session) and not s.graph
        st["batched_write"] = in_batched
        st["batched_read"] = bool(in_batched and uniform and B >= 1)
        if not in_batched and s.manager is not None and B == 1:
            s.manager.on_build(common, new_request=st["full_prefill"])
            if s.manager.dead:
                raise RuntimeError("OMMX refuses to decode with stale KV metadata: "
                                   f"{s.manager.dead_reason}")
        if in_batched and s.bmanager is not None:
            s.bmanager.on_build(common)
            if s.bmanager.dead:
                raise RuntimeError("OMMX refuses to serve this step from the batched pool: "
                                   f"{s.bmanager.dead_reason}")

    def build_for_cudagraph_capture(self, common_attn_metadata):
        s = _STATE
        for m in (s.manager, s.bmanager):
            if m is not None:
                m.capturing = True
        try:
            if s.bmanager is not None and s.bmanager.graph:
                s.bmanager.on_build(common_attn_metadata)
            if HAVE_VLLM:
                return super().build_for_cudagraph_capture(common_attn_metadata)
            return common_attn_metadata
        finally:
            for m in (s.manager, s.bmanager):
                if m is not None:
                    m.capturing = False


# ── per-layer implementation ─────────────────────────────────────────────────────────────

def causal_prefill_attention(query, key, value, q_start, scale, n_rep):
    """Causal attention of each request over its own rows of a full-prefill step, fp32 math on
    the device through torch (a library call; prefill is outside the decode path).
    ``query [n, Hq, D]``, ``key`` / ``value [n, Hkv, D]``, ``q_start`` cumulative row offsets;
    returns fp32 ``[n, Hq, D]``."""
    out = torch.empty(query.shape, dtype=torch.float32, device=query.device)
    for i in range(len(q_start) - 1):
        t0, t1 = int(q_start[i]), int(q_start[i + 1])
        if t1 <= t0:
            continue
        q = query[t0:t1].transpose(0, 1).unsqueeze(0).float()
        k = key[t0:t1].transpose(0, 1).repeat_interleave(n_rep, 0).unsqueeze(0).float()
        v = value[t0:t1].transpose(0, 1).repeat_interleave(n_rep, 0).unsqueeze(0).float()
        o = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale)
        out[t0:t1] = o[0].transpose(0, 1)
    return out


class OMMXCanonicalImpl(_ImplBase):
    """One attention layer.  ``prefill_attention`` may replace the torch prefill read by the
    engine's varlen kernel: ``f(query, key, value, q_start, scale, n_rep) -> [n, Hq, D]``."""

    prefill_attention: Callable = staticmethod(causal_prefill_attention)

    def __init__(self, num_heads: int, head_size: int, scale: Optional[float] = None,
                 num_kv_heads: Optional[int] = None, *args, **kwargs) -> None:
        if HAVE_VLLM:
            super().__init__(num_heads, head_size, scale, num_kv_heads, *args, **kwargs)
        self.num_heads = int(num_heads)
        self.head_size = int(head_size)
        self.num_kv_heads = int(num_kv_heads if num_kv_heads is not None else num_heads)
        self.scale = float(scale if scale is not None else 1.0 / math.sqrt(head_size))
        self._ommx_serving_cfg: Optional[OMMXServingConfig] = None

    # ── configuration and per-layer state ─────────────────────────────────────────

    def _ommx_cfg(self) -> OMMXServingConfig:
        if self._ommx_serving_cfg is None:
            self._ommx_serving_cfg = resolve_serving_config(
                head_dim=self.head_size, n_q_heads=self.num_heads, n_kv_heads=self.num_kv_heads)
        return self._ommx_serving_cfg

    def _ommx_store(self, layer, device, max_ctx) -> CanonicalKVStore:
        st = getattr(layer, "_ommx_store_obj", None)
        if st is None or st.max_seq_len < int(max_ctx):
            c = self._ommx_cfg()
            st = CanonicalKVStore(c.head_dim, c.n_kv_heads, int(max_ctx), device=device,
                                  **c.store_kwargs())
            layer._ommx_store_obj = st
            layer._ommx_single_ws = None
        return st

    def _ommx_reset(self, layer, device, max_ctx) -> CanonicalKVStore:
        """The layer's store ready for a new sequence: same tensors, cursors at zero, so
        addresses that a captured forward reads stay valid (``backend.py:1269-1288``)."""
        st = self._ommx_store(layer, device, max_ctx)
        st.reset_inplace()
        return st

    # ── write ────────────────────────────────────────────────────────────────────

    def do_kv_cache_update(self, layer, key, value, kv_cache=None, slot_mapping=None) -> None:
        n = int(key.shape[0])
        if n == 0:
            return
        s, st = _STATE, _STATE.step
        cfg = self._ommx_cfg()
        key = key.reshape(n, self.num_kv_heads, self.head_size)
        value = value.reshape(n, self.num_kv_heads, self.head_size)
        if st["B"] == STEP_ROUTE_UNCLASSIFIED and not st["batched_write"]:
            raise RuntimeError(
                "[ommx] cannot classify this step: the metadata exposed no readable per-request "
                f"seq_lens, so the number of requests is unknown (n={n} rows in this write). "
                "Refusing to write rather than risk resetting a live sequence.")
        if st["batched_write"]:
            m = s.bmanager
            if m is not None and m.dead:
                raise RuntimeError(f"[ommx] batched pool dead: {m.dead_reason}")
            if (m is not None and m.graph and m.is_uniform_decode and n == int(m.cur_B) > 0):
                self._batched_kv_update_captured(layer, key, value)
            else:
                self._batched_kv_update(layer, key, value)
            return
        mgr = _manager(cfg, key.device)
        if st["full_prefill"] or (n > 1 and st["B"] == 0):
            store = self._ommx_reset(layer, key.device, max(cfg.max_context, n))
            store.append_block(key, value)
            mgr.register(id(layer), store)
            mgr._last_boundary = store.window.boundary(store.seq_len)
        elif n == 1:
            store = self._ommx_store(layer, key.device, cfg.max_context)
            mgr.register(id(layer), store)
            if mgr.cur_seq <= 0:                       # manager created after this step's build
                mgr.on_build(s.last_common, new_request=False)
            store.write_token(mgr.write_pos, key[0], value[0])
        else:
            raise RuntimeError("OMMX single-sequence route does not support chunked prefill")

    def _batched_kv_update(self, layer, key, value) -> None:
        """Split the step's rows per request into the pool (``backend.py:1290-1356``): blocks go
        through ``append_block``, a uniform one-token step is one write and one pack launch."""
        cfg = self._ommx_cfg()
        mgr = _bmanager(cfg, key.device)
        if not mgr.seq_lens and _STATE.last_common is not None:
            mgr.on_build(_STATE.last_common)           # manager created after this step's build
        if mgr.dead:
            raise RuntimeError(f"OMMX batched manager dead: {mgr.dead_reason}")
        n, B = int(key.shape[0]), len(mgr.seq_lens)
        if B == 0:
            return
        pool = mgr.pool(id(layer), key.device)
        q_start = mgr.q_start
        if q_start is not None and len(q_start) == B + 1 and int(q_start[-1]) == n:
            bounds = q_start
        elif n == B:
            bounds = list(range(B + 1))
        else:
            raise RuntimeError(f"batched write: cannot map {n} tokens to {B} requests")
        uniform = n == B and all(bounds[i + 1] - bounds[i] == 1 for i in range(B))
        if uniform and not any(int(mgr.seq_lens[i]) - 1 <= 0 for i in range(B)):
            for i, slot in enumerate(mgr.slots):
                if int(pool.seq_len[slot]) != int(mgr.seq_lens[i]) - 1:
                    raise RuntimeError(
                        f"batched write: slot {slot} holds {pool.seq_len[slot]} tokens but the "
                        f"scheduler reports {mgr.seq_lens[i]} after this step")
            pool.append_decode_batched(mgr.slots, key, value)
            return
        for i in range(B):
            slot = mgr.slots[i]
            t0, t1 = int(bounds[i]), int(bounds[i + 1])
            if t1 <= t0:
                continue
            seq_before = int(mgr.seq_lens[i]) - (t1 - t0)
            if seq_before <= 0:
                pool.reset_slot(slot)
            elif int(pool.seq_len[slot]) != seq_before:
                raise RuntimeError(f"batched write: slot {slot} holds {pool.seq_len[slot]} tokens, "
                                   f"the step continues from {seq_before}")
            if t1 - t0 > 1:
                pool.append_block(slot, key[t0:t1], value[t0:t1])
            else:
                pool.append(slot, key[t0], value[t0])

    def _batched_kv_update_captured(self, layer, key, value) -> None:
        """Launch-only write of a uniform one-token step at the host-refreshed slots and columns
        (``backend.py:1358-1378``); the host seam already advanced and packed the pools."""
        mgr = _STATE.bmanager
        B = int(mgr.cur_B)
        pool = mgr.pool(id(layer), key.device)
        pool.append_decode_captured(mgr.b_sel[:B], mgr.b_write_col[:B], key, value)

    # ── read ─────────────────────────────────────────────────────────────────────

    def forward(self, layer, query, key, value, kv_cache=None, attn_metadata=None, output=None,
                output_scale=None, output_block_scale=None):
        H, D = self.num_heads, self.head_size
        q = query.reshape(-1, H, D)
        if output is None:
            output = torch.empty_like(query)
        out = output.view(-1, H, D)
        st = _STATE.step
        if st["B"] == STEP_ROUTE_UNCLASSIFIED:
            raise RuntimeError("[ommx] unclassified step: request count unknown, refusing to "
                               "serve it through any route")
        if st["batched_read"]:
            m = _STATE.bmanager
            if m is not None and m.graph and int(m.cur_B) == int(q.shape[0]) > 0:
                self._route_decode_batched_graph(layer, q, out)
            else:
                self._route_decode_batched(layer, q, out)
            return output
        if st["full_prefill"]:
            q_start = (_STATE.bmanager.q_start if st["batched_write"] and _STATE.bmanager
                       else None) or [0, int(q.shape[0])]
            self._prefill_rows(q, key, value, out, q_start)
            return output
        if st["uniform"] and st["B"] == 1 and not st["batched_write"]:
            self._route_decode(layer, q, out)
            return output
        if st["batched_write"] and st["B"] >= 1:
            self._route_mixed_batched(layer, q, key, value, out)
            return output
        raise RuntimeError(
            f"[ommx] step with B={st['B']} is neither a uniform one-token decode nor a full "
            "prefill; chunked prefill and prefix caching are not served from packed planes")

    def _prefill_rows(self, q, key, value, out, q_start) -> None:
        n, D = int(q_start[-1]), self.head_size
        k = key.reshape(-1, self.num_kv_heads, D)
        v = value.reshape(-1, self.num_kv_heads, D)
        t0 = int(q_start[0])
        res = type(self).prefill_attention(q[t0:n], k[t0:n], v[t0:n], [x - t0 for x in q_start],
                                           self.scale, self.num_heads // self.num_kv_heads)
        out[t0:n].copy_(res)
        _STATE.fires["prefill"] += 1

    def _route_mixed_batched(self, layer, q, key, value, out) -> None:
        """A step that carries whole prompts of new requests next to one-token rows of running
        ones (continuous batching).  Each prompt attends over its own rows; the one-token rows
        are one decode launch over their pool slots.  A request whose query span is neither its
        whole sequence nor one token (chunked prefill, prefix-cache hit) is refused.  The
        reference's packed-only read refuses every mixed step (``backend.py:1846-1918``)."""
        mgr = _STATE.bmanager
        if mgr is None or mgr.dead:
            raise RuntimeError(f"[ommx] batched pool dead: {getattr(mgr, 'dead_reason', None)}")
        pool = mgr.pools.get(id(layer))
        qs, seqs = mgr.q_start, mgr.seq_lens
        if pool is None or qs is None or len(qs) != len(seqs) + 1:
            raise RuntimeError("[ommx] mixed step without per-request query spans")
        dec_rows, dec_slots = [], []
        for i, seq in enumerate(seqs):
            n_q = int(qs[i + 1]) - int(qs[i])
            if n_q == int(seq):
                self._prefill_rows(q, key, value, out, [int(qs[i]), int(qs[i + 1])])
            elif n_q == 1:
                dec_rows.append(int(qs[i]))
                dec_slots.append(int(mgr.slots[i]))
            elif n_q != 0:
                raise RuntimeError(
                    f"[ommx] request {i}: {n_q} query tokens of a {seq}-token sequence; chunked "
                    "prefill and prefix caching are not served from packed planes")
        if dec_rows:
            rows = torch.tensor(dec_rows, dtype=torch.long).to(q.device, non_blocking=True)
            bundle = pool.decode_inputs_batched(dec_slots)
            tmp = torch.empty(len(dec_rows), self.num_heads, self.head_size, dtype=out.dtype,
                              device=out.device)
            self._decode(layer, q.index_select(0, rows), tmp, bundle, bundle["max_seq_len"])
            out.index_copy_(0, rows, tmp)
            _STATE.fires["batched"] += 1

    def _ommx_ws(self, layer, B: int, max_seq: int, dev) -> dict:
        """Per-layer workspace of fixed capacity: output, lse and split partials."""
        ws = getattr(layer, "_ommx_ws_cache", None)
        if ws is not None and ws["o"].shape[0] >= B and ws["max_seq"] >= max_seq:
            return ws
        cap = max(B, _STATE.max_num_seqs if B > 1 else 1)
        H, D = self.num_heads, self.head_size
        ws = {"o": torch.empty(cap, H, D, dtype=torch.float32, device=dev),
              "lse": torch.empty(cap, H, dtype=torch.float32, device=dev), "max_seq": int(max_seq)}
        layer._ommx_ws_cache = ws
        return ws

    def _decode(self, layer, q, out, bundle, max_seq_len) -> None:
        B = int(q.shape[0])
        ws = self._ommx_ws(layer, B, max_seq_len, q.device)
        cfg = self._ommx_cfg()
        o, _ = ommx_paged_decode(
            q, bundle["planes"], bundle["k_tail"], bundle["v_tail"], bundle["b_tail_len"],
            bundle["b_seq_len"], sm_scale=self.scale, out=ws["o"][:B], lse_out=ws["lse"][:B],
            max_seq_len=int(max_seq_len), max_tail_len=int(bundle["max_tail_len"]),
            combinadic_read=cfg.resolved_combinadic_read(), bitmap_read=cfg.resolved_bitmap_read(),
            packed_start_offset=int(bundle["packed_start_offset"]),
            req_to_token=bundle.get("req_to_token"), req_to_group=bundle.get("req_to_group"))
        out[:B].copy_(o)

    def _route_decode(self, layer, q, out) -> None:
        """One request: fixed-address buffers of the step manager, launch-only
        (``backend.py:1950-2080``)."""
        mgr = _STATE.manager
        store = getattr(layer, "_ommx_store_obj", None)
        if mgr is None or store is None or mgr.dead:
            raise RuntimeError("[ommx] single-sequence decode without a live store: "
                               f"{getattr(mgr, 'dead_reason', None) or 'no prefill reached it'}")
        ws = getattr(layer, "_ommx_single_ws", None)
        T = mgr.max_tail_cap
        if ws is None:
            ws = {"kt": torch.zeros(1, T, store.H, store.D, dtype=torch.bfloat16, device=q.device)}
            ws["vt"] = torch.zeros_like(ws["kt"])
            layer._ommx_single_ws = ws
        store.gather_tail_into(mgr.tail_idx, ws["kt"], ws["vt"], T)
        bundle = {"planes": store.decode_planes_full(), "k_tail": ws["kt"], "v_tail": ws["vt"],
                  "b_tail_len": mgr.b_tail_len, "b_seq_len": mgr.b_seq_len,
                  "max_tail_len": T, "packed_start_offset": 0}
        self._decode(layer, q[:1], out, bundle, mgr.max_seq_len)
        _STATE.fires["single"] += 1

    def _route_decode_batched(self, layer, q, out) -> None:
        mgr = _STATE.bmanager
        if mgr is None or mgr.dead or not mgr.is_uniform_decode:
            raise RuntimeError("[ommx] batched decode without a live pool: "
                               f"{getattr(mgr, 'dead_reason', None)}")
        pool = mgr.pools.get(id(layer))
        if pool is None:
            raise RuntimeError("[ommx] batched decode before any write reached this layer's pool")
        B = len(mgr.slots)
        bundle = pool.decode_inputs_batched(mgr.slots)
        self._decode(layer, q[:B], out, bundle, bundle["max_seq_len"])
        _STATE.fires["batched"] += 1

    def _route_decode_batched_graph(self, layer, q, out) -> None:
        """Launch-only batched read from the manager's fixed buffers (``backend.py:1477-1549``)."""
        mgr = _STATE.bmanager
        if mgr.dead:
            raise RuntimeError(f"[ommx] batched pool dead: {mgr.dead_reason}")
        pool = mgr.pools.get(id(layer))
        if pool is None:
            raise RuntimeError("[ommx] batched decode before any write reached this layer's pool")
        B = int(mgr.cur_B)
        # every layer's pool has the same slot geometry: the page / group table rows of this
        # step's slots are selected by the first layer that runs and shared by the others
        bundle = pool.decode_inputs_seq(mgr.b_sel[:B], mgr.b_cur_seq[:B], mgr.b_seq_len[:B],
                                        mgr.b_tail_len[:B], mgr.max_seq_len, tables=mgr.step_tables)
        mgr.step_tables = (bundle["req_to_token"], bundle["req_to_group"])
        self._decode(layer, q[:B], out, bundle, mgr.max_seq_len)
        _STATE.fires["batched"] += 1


# ── backend ──────────────────────────────────────────────────────────────────────────────

class OMMXCanonicalBackend(_BackendBase):
    @staticmethod
    def get_name() -> str:
        return "CUSTOM"

    @staticmethod
    def get_impl_cls():
        return OMMXCanonicalImpl

    @staticmethod
    def get_builder_cls():
        return OMMXCanonicalMetadataBuilder

    @staticmethod
    def get_kv_cache_shape(num_blocks, block_size, num_kv_heads, head_size, cache_dtype_str="auto"):
        """The engine's paged cache is not used; a one-byte page keeps its allocator satisfied.
        (The reference's packed-only mode sizes an engine-owned byte arena here,
        ``backend.py:2098-2107``; this package keeps the planes in its own pools.)"""
        return (int(num_blocks), 1)

    @staticmethod
    def get_kv_cache_stride_order(include_num_layers_dimension=False):
        if include_num_layers_dimension:
            raise NotImplementedError("OMMX planes do not support cross-layer KV transfer")
        return (0, 1)

    @staticmethod
    def get_supported_kernel_block_sizes():
        return [16]


__all__ = ["OMMXCanonicalBackend", "OMMXCanonicalImpl", "OMMXCanonicalMetadataBuilder",
           "OMMX_BACKEND_CLASS_PATH", "ommx_route_health", "reset_worker_state",
           "causal_prefill_attention", "HAVE_VLLM"]
