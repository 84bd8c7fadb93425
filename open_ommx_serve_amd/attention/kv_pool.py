"""Multi-sequence KV pool: shared packed planes + per-request bf16 residual histories.

Same class, methods and argument bundles as the reference
``ommx_gpu_serve/attention/kv_pool.py:93-1105`` (``MultiSeqKVPool``), with the data movement
done by the HIP kernels of this package:

* a decode append is one ``ommx_ring_write`` launch (all requests, ring slot computed on the
  device, the device-side sequence counter advanced by the same launch);
* a completed 32-token group is packed by one ``ommx_store_pack`` launch that reads the
  rows through their ring slots and writes straight into the request's page / group slots
  (the reference packs into temporaries and copies plane by plane, ``kv_pool.py:552-635``);
* the decode inputs (tail rows, ``b_seq_len``, ``b_tail_len``) come from one
  ``ommx_tail_gather`` launch that does the window arithmetic of ``kv_pool.py:1048-1105``.

Slot arithmetic (``kv_pool.py:165-170, 273-276, 711-734``): request ``r`` owns group slots
``[r*G_per_seq, (r+1)*G_per_seq)`` and pages ``[r*P_per_seq, (r+1)*P_per_seq)`` with
``G_per_seq = ceil(max_seq_len/gt) + 1``; the tables are ``arange`` slices.

Only the serving recipe is implemented (i2f4, signed outliers, flat bitmap, power-of-two
int8 exponents, dedicated FP4 map, 32x32 groups, i2 V); other recipes raise
``NotImplementedError``.  The pool lives on a ROCm GPU; there is no CPU path.
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _hip
from .kv_store_ops import gather_tails, ring_slot, write_tokens
from .kv_window import CANONICAL_GROUP_TOKENS, WindowSpec
from .pack import index_plane_bytes, raise_for_store_errors, store_pack_into

_FALSE = {"0", "false", "off", "no"}


def _env_flag(name: str, default: bool) -> bool:
    raw = os.environ.get(name)
    if not raw:
        return default
    return raw.strip().lower() not in _FALSE


def check_serving_recipe(*, k_format: str, outlier_select: str, outlier_repr: str, use_pow2: bool,
                         kv_outlier_map: Optional[bool], kv_int8_scale: Optional[bool],
                         group_tokens: int, group_channels: int, scale_dtype: torch.dtype,
                         outliers_per_vector: int, v_format: str = "i2") -> None:
    """Accept the serving recipe, refuse every other one with its name."""
    k = int(outliers_per_vector)
    if str(k_format).lower() not in ("i2f4", "itf4"):
        raise ValueError(f"k_format must be i2f4|itf4; got {k_format!r}")
    if str(outlier_repr).lower() not in ("relidx7", "combinadic", "bitmap"):
        raise ValueError(f"outlier_repr must be one of relidx7|combinadic|bitmap; got {outlier_repr!r}")
    if group_channels not in (16, 32, 64, 128):
        raise ValueError(f"group_channels must be in {{16,32,64,128}}; got {group_channels}")
    if group_tokens not in (16, 32, 64, 128):
        raise ValueError(f"group_tokens must be in {{16,32,64,128}}; got {group_tokens}")
    bad = []
    if str(v_format).lower() not in ("i2", "bf16"):
        bad.append(f"v_format={v_format!r}")
    if str(outlier_repr).lower() == "combinadic" and k > 8:
        bad.append("combinadic ranks with more than 8 outliers (their decode twin is the bitmask plane)")
    if k > 0 and str(outlier_select).lower() not in ("signed", "abs"):
        bad.append(f"outlier_select={outlier_select!r}")
    if scale_dtype != torch.bfloat16:
        bad.append(f"scale_dtype={scale_dtype}")
    if not 0 <= k <= min(16, int(group_tokens)):
        bad.append(f"outliers_per_vector={k}")
    if bad:
        raise NotImplementedError(
            "the HIP KV store implements the serving recipe and its near variants only (i2f4, "
            "signed or abs selection, bitmap, relidx7 or combinadic index plane, power-of-two or plain bf16 steps, "
            "dedicated or base-shared FP4 outliers, bf16 zero points, 0..16 outliers); "
            "unsupported: " + ", ".join(bad))


class MultiSeqKVPool:
    """Per-layer shared plane pool + per-request tables for batched paged decode."""

    def __init__(
        self,
        head_dim: int,
        n_kv_heads: int,
        num_seqs: int,
        max_seq_len: int,
        *,
        k_format: str = "i2f4",
        outliers_per_vector: int = 3,
        outlier_select: str = "signed",
        outlier_repr: str = "relidx7",
        use_pow2: bool = False,
        kv_outlier_map: Optional[bool] = None,
        kv_int8_scale: Optional[bool] = None,
        window: Optional[WindowSpec] = None,
        group_channels: int = 32,
        scale_dtype: torch.dtype = torch.bfloat16,
        device="cuda",
        kv_ring: Optional[bool] = None,
    ) -> None:
        if head_dim % 32 != 0:
            raise ValueError(f"head_dim must be a multiple of 32; got {head_dim}")
        self.window = window or WindowSpec()
        self.gt = int(self.window.group_tokens) or CANONICAL_GROUP_TOKENS
        self.ps = int(self.window.page_size)
        if self.gt % self.ps != 0:
            raise ValueError(f"group_tokens ({self.gt}) must be a multiple of page_size ({self.ps})")
        if kv_outlier_map is None:
            kv_outlier_map = _env_flag("OMMX_KV_OUTLIER_MAP", True)
        if kv_int8_scale is None:
            kv_int8_scale = _env_flag("OMMX_KV_INT8_SCALE", bool(use_pow2))
        check_serving_recipe(k_format=k_format, outlier_select=outlier_select,
                             outlier_repr=outlier_repr, use_pow2=use_pow2,
                             kv_outlier_map=kv_outlier_map, kv_int8_scale=kv_int8_scale,
                             group_tokens=self.gt, group_channels=int(group_channels),
                             scale_dtype=scale_dtype, outliers_per_vector=outliers_per_vector)
        self.D, self.H = int(head_dim), int(n_kv_heads)
        self.num_seqs, self.max_seq_len = int(num_seqs), int(max_seq_len)
        self.k_format = str(k_format).lower()          # "i2f4" and "itf4" name the same planes
        self.k = int(outliers_per_vector)
        self.outlier_select = str(outlier_select).lower()
        self.outlier_repr = str(outlier_repr).lower()
        self.use_pow2 = bool(use_pow2)
        self.kv_outlier_map = bool(kv_outlier_map)
        self.kv_int8_scale = bool(kv_int8_scale) and bool(use_pow2)      # pack.py:397
        self.scale_dtype = scale_dtype
        self.device = torch.device(device)
        _hip.require_gpu(self.device)
        _hip.load()
        self.pages_per_group = self.gt // self.ps
        self.gc = int(group_channels)
        self.k_base_bits, self.oval_bits = 2, 4
        self.k_base_w = self.D // 4
        self.NGV = self.D // self.gc

        # capacity: one group of slack per request (kv_pool.py:165-170)
        self.G_per_seq = max(1, (self.max_seq_len + self.gt - 1) // self.gt + 1)
        self.P_per_seq = self.G_per_seq * self.pages_per_group
        self.G_cap = self.num_seqs * self.G_per_seq
        self.P_cap = self.num_seqs * self.P_per_seq

        dev, bf = self.device, torch.bfloat16
        z = torch.zeros
        self.k_base = z(self.P_cap, self.ps, self.H, self.k_base_w, dtype=torch.uint8, device=dev)
        self.v_main = z(self.P_cap, self.ps, self.H, self.D // 4, dtype=torch.uint8, device=dev)
        sdt = torch.int8 if self.kv_int8_scale else bf      # exponents, or the steps themselves
        self.k_scale = z(self.G_cap, self.H, self.D, dtype=sdt, device=dev)
        self.k_zp = z(self.G_cap, self.H, self.D, dtype=bf, device=dev)
        self.v_scale = z(self.P_cap, self.ps, self.H, self.NGV, dtype=sdt, device=dev)
        self.v_zp = z(self.P_cap, self.ps, self.H, self.NGV, dtype=bf, device=dev)
        self.k_oidx = None
        self.k_crank = None
        if self.k > 0:
            if self.kv_outlier_map:     # base-shared outliers carry no map planes (pack.py:502-506)
                self.k_fp4_mapscale = z(self.G_cap, self.H, self.D, dtype=bf, device=dev)
                self.k_fp4_mapcenter = z(self.G_cap, self.H, self.D, dtype=bf, device=dev)
            else:
                self.k_fp4_mapscale = self.k_fp4_mapcenter = None
            # index plane of the recipe: flat bitmask, or 7-bit position streams (pack.py:128-164)
            if self.outlier_repr == "relidx7":
                self.k_obmp = None
                self.k_oidx = z(self.G_cap, self.H, self.D, (7 * self.k + 7) // 8, dtype=torch.uint8, device=dev)
            elif self.outlier_repr == "combinadic":
                # The ranks are the stored form (pack.py:552-557).  The store kernel writes the flat
                # bitmask first and one launch ranks it, so the bitmask plane stays beside the ranks
                # as their decode-ready twin: the decode kernels read positions, not ranks.
                self.k_crank = z(self.G_cap, self.H, self.D, index_plane_bytes("combinadic", self.gt, self.k),
                                 dtype=torch.uint8, device=dev)
                self.k_obmp = z(self.G_cap, self.H, self.D, (self.gt + 7) // 8, dtype=torch.uint8, device=dev)
            else:
                self.k_obmp = z(self.G_cap, self.H, self.D, (self.gt + 7) // 8, dtype=torch.uint8, device=dev)
            self.k_oval = z(self.G_cap, self.H, self.D, (self.k + 1) // 2, dtype=torch.uint8, device=dev)
        else:
            self.k_fp4_mapscale = self.k_fp4_mapcenter = self.k_obmp = self.k_oval = None

        # bf16 residual history: whole sequence, or a ring of the live rows
        # (kv_pool.py:228-262; ring span = recent + 2 groups so live rows never alias)
        self.kv_ring = _env_flag("OMMX_KV_RING", False) if kv_ring is None else bool(kv_ring)
        if self.kv_ring:
            self._ring_sink = int(self.window.sink_tokens)
            self._ring_rec = int(self.window.recent_window) + 2 * self.gt
            self.ring_cap = self._ring_sink + self._ring_rec
        else:
            self._ring_sink = 0
            self._ring_rec = 0
            self.ring_cap = self.max_seq_len
        self.S_ring = int(self.ring_cap)
        self.k_hist = z(self.num_seqs, self.ring_cap, self.H, self.D, dtype=bf, device=dev)
        self.v_hist = z(self.num_seqs, self.ring_cap, self.H, self.D, dtype=bf, device=dev)
        self.seq_len: List[int] = [0] * self.num_seqs
        self.packed_groups: List[int] = [0] * self.num_seqs

        self._req_to_group = torch.arange(self.G_cap, dtype=torch.int32, device=dev).reshape(
            self.num_seqs, self.G_per_seq)
        self._req_to_token = torch.arange(self.P_cap, dtype=torch.int32, device=dev).reshape(
            self.num_seqs, self.P_per_seq)
        self.max_tail_len = int(self.window.max_tail_len(self.max_seq_len))
        # device error bits of the store / ring kernels; read by check_errors()
        self.err_flag = torch.zeros(1, dtype=torch.int32, device=dev)
        self.wide_steps = False      # a packed K step above 2^15 was seen: decode on the plain kernel
        self._dbuf: Optional[Dict[str, object]] = None
        self._planes_cache: Optional[dict] = None

    # ── ring address mapping ───────────────────────────────────────────────────────

    def _ring_slot_host(self, pos: int) -> int:
        return ring_slot(pos, self._ring_sink, self._ring_rec) if self.kv_ring else int(pos)

    def _ring_slot_dev(self, pos: torch.Tensor) -> torch.Tensor:
        if not self.kv_ring:
            return pos
        rel = (pos - self._ring_sink) % self._ring_rec + self._ring_sink
        return torch.where(pos < self._ring_sink, pos, rel)

    def check_errors(self) -> None:
        """Read the device error bits (host sync) and raise what the reference would have."""
        bits = int(self.err_flag.item())
        if bits:
            self.err_flag.zero_()
        if bits & _hip.NOTE_WIDE_STEP:
            # not an error: some packed K step is above 2^15, beyond the f16 operands of the matrix-core
            # decode kernels; from here on this cache is decoded by the plain fp32 kernel
            self.wide_steps = True
        if bits & _hip.ERR_VALUE_RANGE:
            self.wide_steps = True
            raise ValueError("OMMX decode: a K step above 2^15 (K values beyond some 1e5) met the matrix-core "
                             "kernel, whose f16 operands held it at 2^15: outputs since the last check are off "
                             "for the requests that hold such a group.  This cache is served by the plain "
                             "kernel from now on (_force_reference_kernel=True)")
        if bits & _hip.ERR_TABLE_RANGE:
            raise IndexError("OMMX decode: a page id or group slot of the request tables lies outside the planes "
                             "(it was clamped; the output of that request is not meaningful)")
        if bits & _hip.ERR_RING_RANGE:
            raise IndexError("OMMX KV write/gather outside residual capacity")  # kv_store_ops.py:34,53
        raise_for_store_errors(bits)

    def reset_slot(self, req: int) -> None:
        """Start a new sequence in slot ``req`` (tensors are kept; stale slots are never read)."""
        self.seq_len[int(req)] = 0
        self.packed_groups[int(req)] = 0

    # ── write path ───────────────────────────────────────────────────────────────

    def _planes_for_store(self) -> dict:
        return {"k_base": self.k_base, "k_scale": self.k_scale, "k_zp": self.k_zp,
                "k_fp4_mapscale": self.k_fp4_mapscale, "k_fp4_mapcenter": self.k_fp4_mapcenter,
                "k_obmp": self.k_obmp, "k_oidx": self.k_oidx, "k_oval": self.k_oval,
                "k_crank": self.k_crank,
                "_k_obmp_scratch": self.k_obmp if self.outlier_repr == "combinadic" else None,
                "v_main": self.v_main, "v_scale": self.v_scale, "v_zp": self.v_zp}

    def _as_rows(self, t: torch.Tensor, what: str) -> torch.Tensor:
        if t.device != self.device:
            t = t.to(self.device)
        if t.dtype not in (torch.bfloat16, torch.float32):
            t = t.to(torch.bfloat16)
        if t.dim() != 3 or tuple(t.shape[1:]) != (self.H, self.D):
            raise ValueError(f"{what} must be [T, {self.H}, {self.D}]; got {tuple(t.shape)}")
        return t

    def append_block(self, req: int, K: torch.Tensor, V: torch.Tensor) -> int:
        """Stash request ``req``'s prefill block ``[T, H, D]`` then pack its completed groups.

        Returns the number of groups packed (kv_pool.py:310-368).
        """
        r = int(req)
        K, V = self._as_rows(K, "K"), self._as_rows(V, "V")
        T = int(K.shape[0])
        s = self.seq_len[r]
        if not self.kv_ring:
            if s + T > self.max_seq_len:
                raise RuntimeError(f"MultiSeqKVPool req {r} capacity {self.max_seq_len} exceeded")
            self.k_hist[r, s:s + T] = K.to(torch.bfloat16)
            self.v_hist[r, s:s + T] = V.to(torch.bfloat16)
            self.seq_len[r] = s + T
            return self.regroup(r)
        if s != 0:
            raise RuntimeError(
                f"ring append_block expects a fresh request slot (seq_len==0); chunked prefill "
                f"under the ring is unsupported (it cannot retain unpacked rows across chunks). "
                f"Reset pool slot {r} before each prefill block.")
        Kb, Vb = K.to(torch.bfloat16), V.to(torch.bfloat16)
        self.seq_len[r] = T
        target = self.window.num_groups(T)
        if target > 0:
            sink = self.window.sink_tokens
            self._pack_block_into_pool(r, Kb[sink:sink + target * self.gt],
                                       Vb[sink:sink + target * self.gt], 0, target)
            self.packed_groups[r] = target
        # only the live rows enter the ring: sink, and [boundary - gt, T)
        boundary = self.window.boundary(T)
        sink_tokens = self.window.sink_tokens
        lo = max(sink_tokens, boundary - self.gt)
        parts = [torch.arange(0, min(sink_tokens, T), device=self.device)]
        if lo < T:
            parts.append(torch.arange(lo, T, device=self.device))
        live = torch.cat(parts).to(torch.long)
        slots = self._ring_slot_dev(live)
        self.k_hist[r].index_copy_(0, slots, Kb.index_select(0, live))
        self.v_hist[r].index_copy_(0, slots, Vb.index_select(0, live))
        return target

    def append(self, req: int, k: torch.Tensor, v: torch.Tensor) -> int:
        """One decode step's K/V row ``[H, D]`` for request ``req`` (kv_pool.py:370-381)."""
        r = int(req)
        s = self.seq_len[r]
        if not self.kv_ring and s >= self.max_seq_len:
            raise RuntimeError(f"MultiSeqKVPool req {r} capacity {self.max_seq_len} exceeded")
        slot = self._ring_slot_host(s)
        self.k_hist[r, slot] = k.reshape(self.H, self.D).to(self.device, torch.bfloat16)
        self.v_hist[r, slot] = v.reshape(self.H, self.D).to(self.device, torch.bfloat16)
        self.seq_len[r] = s + 1
        return self.regroup(r)

    def _bf16_batch(self, t: torch.Tensor, B: int) -> torch.Tensor:
        t = t.reshape(B, self.H, self.D)
        if t.dtype != torch.bfloat16 or t.device != self.device:
            t = t.to(self.device, torch.bfloat16)
        return t if t.stride(-1) == 1 else t.contiguous()

    def _advance_host_and_pack(self, slots: Sequence[int]) -> int:
        pend: List[Tuple[int, int, int]] = []
        total = 0
        for r in slots:
            self.seq_len[r] += 1
            target = self.window.num_groups(self.seq_len[r])
            if target > self.packed_groups[r]:
                pend.append((r, self.packed_groups[r], target))
                total += target - self.packed_groups[r]
        if pend:
            self._regroup_pack_batched_device(pend)
            for r, _g0, g1 in pend:
                self.packed_groups[r] = g1
        return total

    def append_decode_batched(self, slots: Sequence[int], K: torch.Tensor, V: torch.Tensor) -> int:
        """B new rows ``[B, H, D]`` in one launch, then one pack launch for every group that
        completed this step (kv_pool.py:383-438).  Returns the number of groups packed."""
        slots = [int(s) for s in slots]
        B = len(slots)
        if B == 0:
            return 0
        for r in slots:
            if not self.kv_ring and self.seq_len[r] >= self.max_seq_len:
                raise RuntimeError(f"MultiSeqKVPool req {r} capacity {self.max_seq_len} exceeded")
        meta = torch.tensor([slots, [self.seq_len[r] for r in slots]], dtype=torch.int64).to(
            self.device, non_blocking=True)
        write_tokens(self.k_hist, self.v_hist, meta[1], self._bf16_batch(K, B), self._bf16_batch(V, B),
                     self._ring_sink, self._ring_rec, slots=meta[0], err_flag=self.err_flag)
        return self._advance_host_and_pack(slots)

    def append_decode_captured(self, rows: torch.Tensor, cols: torch.Tensor, K: torch.Tensor,
                               V: torch.Tensor) -> None:
        """Write B rows by device indices only: ``rows`` = pool slots, ``cols`` = absolute
        positions, both int64 ``[B]`` fixed-address buffers (kv_pool.py:490-524).  Host state is
        not touched; an out-of-range slot sets the ring error bit (see ``check_errors``)."""
        B = int(rows.shape[0])
        write_tokens(self.k_hist, self.v_hist, cols, self._bf16_batch(K, B), self._bf16_batch(V, B),
                     self._ring_sink, self._ring_rec, slots=rows, err_flag=self.err_flag)

    def append_decode_device(self, K: torch.Tensor, V: torch.Tensor, B: int) -> int:
        """Decode write driven by the device sequence counter: one launch writes the B rows at
        ``seq_dev`` and advances it; the host mirror then packs completed groups
        (kv_pool.py:440-488).  Batch row b is pool slot b, as in the reference."""
        d = self._decode_buffers(B)
        write_tokens(self.k_hist, self.v_hist, d["seq_dev"], self._bf16_batch(K, B),
                     self._bf16_batch(V, B), self._ring_sink, self._ring_rec, slots=d["rows"],
                     pos_next=d["seq_dev"], err_flag=self.err_flag)
        return self._advance_host_and_pack(range(B))

    def _regroup_pack_batched_device(self, pend: Sequence[Tuple[int, int, int]]) -> None:
        """Pack every completing group of this step with ONE store launch (kv_pool.py:552-635).

        The launch reads the source rows in place (``src_rows`` = flat history rows through
        the ring map) and writes to each request's own page / group slots.
        """
        gt, ppg, sink = self.gt, self.pages_per_group, self.window.sink_tokens
        src: List[int] = []
        pages: List[int] = []
        groups: List[int] = []
        for (r, g0, g1) in pend:
            base = r * self.S_ring
            for g in range(g0, g1):
                t0 = sink + g * gt
                src.extend(base + self._ring_slot_host(t) for t in range(t0, t0 + gt))
                groups.append(r * self.G_per_seq + g)
                pages.extend(r * self.P_per_seq + g * ppg + i for i in range(ppg))
        idx = torch.tensor(src + pages + groups, dtype=torch.int32).to(self.device, non_blocking=True)
        n_s, n_p = len(src), len(pages)
        flat_k = self.k_hist.view(self.num_seqs * self.S_ring, self.H, self.D)
        flat_v = self.v_hist.view(self.num_seqs * self.S_ring, self.H, self.D)
        store_pack_into(flat_k, flat_v, self._planes_for_store(), outliers_per_vector=self.k,
                        outlier_repr=self.outlier_repr, outlier_select=self.outlier_select,
                        use_pow2=self.use_pow2, kv_int8_scale=self.kv_int8_scale,
                        group_tokens=self.gt, group_channels=self.gc,
                        page_size=self.ps, src_rows=idx[:n_s], dst_pages=idx[n_s:n_s + n_p],
                        dst_groups=idx[n_s + n_p:], err_flag=self.err_flag, num_tokens=n_s)

    def regroup(self, req: int) -> int:
        """Pack request ``req``'s newly completed groups (kv_pool.py:637-652)."""
        r = int(req)
        target = self.window.num_groups(self.seq_len[r])
        if target <= self.packed_groups[r]:
            return 0
        n = target - self.packed_groups[r]
        self._regroup_pack_range(r, self.packed_groups[r], target)
        self.packed_groups[r] = target
        return n

    def _regroup_pack_range(self, req: int, g0: int, g1: int) -> None:
        r = int(req)
        if self.kv_ring:
            self._regroup_pack_batched_device([(r, g0, g1)])
            return
        sink = self.window.sink_tokens
        t0, t1 = sink + g0 * self.gt, sink + g1 * self.gt
        self._pack_block_into_pool(r, self.k_hist[r, t0:t1], self.v_hist[r, t0:t1], g0, g1)

    def _pack_block_into_pool(self, req: int, K_blk: torch.Tensor, V_blk: torch.Tensor,
                              g0: int, g1: int) -> None:
        """Pack a source block of exactly ``(g1-g0)*gt`` tokens into request ``req``'s group /
        page slots ``[g0, g1)`` with one store launch (kv_pool.py:677-734)."""
        r = int(req)
        n_tok = (g1 - g0) * self.gt
        if int(K_blk.shape[0]) != n_tok or int(V_blk.shape[0]) != n_tok:
            raise ValueError(f"source block must hold {n_tok} tokens; got {int(K_blk.shape[0])}")
        gp0 = r * self.G_per_seq + g0
        pp0 = r * self.P_per_seq + g0 * self.pages_per_group
        store_pack_into(K_blk, V_blk, self._planes_for_store(), outliers_per_vector=self.k,
                        outlier_repr=self.outlier_repr, outlier_select=self.outlier_select,
                        use_pow2=self.use_pow2, kv_int8_scale=self.kv_int8_scale,
                        group_tokens=self.gt, group_channels=self.gc,
                        page_size=self.ps,
                        dst_pages=self._req_to_token.view(-1)[pp0:pp0 + (g1 - g0) * self.pages_per_group],
                        dst_groups=self._req_to_group.view(-1)[gp0:gp0 + (g1 - g0)],
                        err_flag=self.err_flag)

    # ── read path ────────────────────────────────────────────────────────────────

    def pool_planes(self) -> dict:
        """Whole-pool plane dict + batched tables, built once (kv_pool.py:738-774)."""
        if self._planes_cache is None:
            self._planes_cache = self._build_pool_planes()
        return self._planes_cache

    def _build_pool_planes(self) -> dict:
        return {
            "k_base": self.k_base, "k_scale": self.k_scale, "k_zp": self.k_zp,
            "k_oidx": self.k_oidx, "k_oval": self.k_oval, "k_crank": self.k_crank,
            "k_obmp": self.k_obmp,
            "k_fp4_mapscale": self.k_fp4_mapscale, "k_fp4_mapcenter": self.k_fp4_mapcenter,
            "v_main": self.v_main, "v_scale": self.v_scale, "v_zp": self.v_zp,
            "req_to_token": self._req_to_token, "req_to_group": self._req_to_group,
            "page_size": self.ps, "outliers_per_vector": self.k,
            "outlier_repr": self.outlier_repr, "outlier_select": self.outlier_select,
            "k_format": self.k_format, "head_dim": self.D, "n_kv_heads": self.H,
            "group_tokens": self.gt, "group_channels": self.gc,
            "k_base_bits": self.k_base_bits, "oval_bits": self.oval_bits,
            "kv_outlier_map": bool(self.kv_outlier_map and self.k > 0),
            "kv_int8_scale": self.kv_int8_scale,
        }

    def request_planes(self, req: int) -> dict:
        """Dense per-request plane dict gathered through the tables (kv_pool.py:776-816)."""
        r = int(req)
        G = self.packed_groups[r]
        P = G * self.pages_per_group
        gidx = self._req_to_group[r, :G].to(torch.long)
        pidx = self._req_to_token[r, :P].to(torch.long)

        def sel(t, idx):
            return None if t is None else t.index_select(0, idx)

        return {
            "k_base": sel(self.k_base, pidx), "k_scale": sel(self.k_scale, gidx),
            "k_zp": sel(self.k_zp, gidx), "k_oidx": sel(self.k_oidx, gidx), "k_crank": sel(self.k_crank, gidx),
            "k_oval": sel(self.k_oval, gidx), "k_obmp": sel(self.k_obmp, gidx),
            "k_fp4_mapscale": sel(self.k_fp4_mapscale, gidx),
            "k_fp4_mapcenter": sel(self.k_fp4_mapcenter, gidx),
            "v_main": sel(self.v_main, pidx), "v_scale": sel(self.v_scale, pidx),
            "v_zp": sel(self.v_zp, pidx),
            "head_dim": self.D, "n_kv_heads": self.H, "num_tokens": G * self.gt, "n_groups": G,
            "page_size": self.ps, "outliers_per_vector": self.k,
            "outlier_repr": self.outlier_repr, "outlier_select": self.outlier_select,
            "group_tokens": self.gt, "group_channels": self.gc, "k_format": self.k_format,
            "k_base_bits": self.k_base_bits, "oval_bits": self.oval_bits,
            "kv_outlier_map": bool(self.kv_outlier_map and self.k > 0), "kv_int8_scale": self.kv_int8_scale,
        }

    def _gather(self, kt, vt, *, seq=None, tail_idx=None, slots=None, b_tail=None, b_seq=None):
        gather_tails(self.k_hist, self.v_hist, kt, vt, self._ring_sink, self._ring_rec,
                     seq=seq, tail_idx=tail_idx, slots=slots, b_tail_len=b_tail, b_seq_len=b_seq,
                     window_sink=self.window.sink_tokens, window_recent=self.window.recent_window,
                     group_tokens=self.gt, err_flag=self.err_flag)

    def tail_bf16_batched(self, slots: Sequence[int]):
        """``(k_tail [B,T,H,D], v_tail, b_tail_len [B])`` of the given slots (kv_pool.py:818-842).
        Rows past ``b_tail_len`` repeat position 0 of the request; readers mask them."""
        slots = [int(s) for s in slots]
        B, T = len(slots), self.max_tail_len
        dev = self.device
        kt = torch.empty(B, T, self.H, self.D, dtype=torch.bfloat16, device=dev)
        vt = torch.empty_like(kt)
        b_tail = torch.zeros(B, dtype=torch.int32, device=dev)
        if B:
            meta = torch.tensor([slots, [self.seq_len[r] for r in slots]], dtype=torch.int64).to(dev)
            self._gather(kt, vt, seq=meta[1], slots=meta[0], b_tail=b_tail)
        return kt, vt, b_tail

    def _ensure_decode_buffers(self, B: int) -> None:
        """Persistent fixed-address decode buffers, allocated once (kv_pool.py:844-884)."""
        if self._dbuf is not None and self._dbuf["cap"] >= B:
            return
        cap = max(B, self.num_seqs)
        T, dev = self.max_tail_len, self.device
        self._dbuf = {
            "cap": cap,
            "kt": torch.zeros(cap, T, self.H, self.D, dtype=torch.bfloat16, device=dev),
            "vt": torch.zeros(cap, T, self.H, self.D, dtype=torch.bfloat16, device=dev),
            "b_tail": torch.zeros(cap, dtype=torch.int32, device=dev),
            "b_seq": torch.zeros(cap, dtype=torch.int32, device=dev),
            "sel": torch.zeros(cap, dtype=torch.long, device=dev),
            "tidx_dev": torch.zeros(cap, T, dtype=torch.long, device=dev),
            "seq_dev": torch.zeros(cap, dtype=torch.long, device=dev),
            "rows": torch.zeros(cap, dtype=torch.long, device=dev),
            "cols": torch.zeros(cap, dtype=torch.long, device=dev),
        }

    def _decode_buffers(self, B: int) -> Dict[str, torch.Tensor]:
        self._ensure_decode_buffers(B)
        d = self._dbuf
        return {k: (v[:B] if isinstance(v, torch.Tensor) else v) for k, v in d.items()}

    def _bundle(self, sel: torch.Tensor, b_seq: torch.Tensor, b_tail: torch.Tensor,
                kt: torch.Tensor, vt: torch.Tensor, max_seq_len: int, tables=None) -> dict:
        planes = dict(self.pool_planes())
        if tables is None:
            tables = (self._req_to_token.index_select(0, sel), self._req_to_group.index_select(0, sel))
        planes["req_to_token"], planes["req_to_group"] = tables
        # beside the planes: where the decode kernels report, and whether this cache needs the plain kernel
        planes["err_flag"], planes["force_reference_kernel"] = self.err_flag, self.wide_steps
        return {
            "planes": planes, "k_tail": kt, "v_tail": vt,
            "b_tail_len": b_tail, "b_seq_len": b_seq,
            "req_to_token": planes["req_to_token"], "req_to_group": planes["req_to_group"],
            "packed_start_offset": 0, "max_seq_len": int(max_seq_len),
            "max_tail_len": self.max_tail_len,
        }

    def decode_inputs_captured(self, sel: torch.Tensor, b_seq_len: torch.Tensor,
                               b_tail_len: torch.Tensor, tidx_dev: torch.Tensor,
                               kt: torch.Tensor, vt: torch.Tensor, max_seq_len: int) -> dict:
        """Decode bundle from caller-filled fixed buffers: ``tidx_dev [B,T]`` absolute tail
        positions are gathered (through the ring map) into ``kt`` / ``vt``
        (kv_pool.py:886-936).  Device-only work."""
        self._gather(kt, vt, tail_idx=tidx_dev, slots=sel)
        return self._bundle(sel, b_seq_len, b_tail_len, kt, vt, max_seq_len)

    def decode_inputs_seq(self, sel: torch.Tensor, seq: torch.Tensor, b_seq_len: torch.Tensor,
                          b_tail_len: torch.Tensor, max_seq_len: int, tables=None) -> dict:
        """Decode bundle from caller-owned fixed buffers that hold the pool slots (``sel``,
        int64 ``[B]``) and the CURRENT sequence lengths (``seq``, int64 ``[B]``): the gather
        launch derives the tail positions and writes ``b_seq_len`` / ``b_tail_len`` (int32
        ``[B]``).  Device-only work; the reference's counterpart takes a host-filled ``[B, T]``
        position matrix (kv_pool.py:886-936).  ``tables``: the ``(req_to_token, req_to_group)`` rows
        of ``sel`` when the caller already holds them (pools of one geometry share them: every
        layer of a model), else they are selected here."""
        B = int(sel.shape[0])
        d = self._decode_buffers(B)
        self._gather(d["kt"], d["vt"], seq=seq, slots=sel, b_tail=b_tail_len, b_seq=b_seq_len)
        return self._bundle(sel, b_seq_len, b_tail_len, d["kt"], d["vt"], max_seq_len, tables)

    def decode_inputs_batched(self, slots: Sequence[int]) -> dict:
        """Decode bundle for ``slots`` from the host sequence lengths (kv_pool.py:938-1013):
        one small host-to-device copy, then one gather launch."""
        slots = [int(s) for s in slots]
        B = len(slots)
        d = self._decode_buffers(B)
        meta = torch.tensor([slots, [self.seq_len[r] for r in slots]], dtype=torch.int64).to(
            self.device, non_blocking=True)
        d["sel"].copy_(meta[0])
        self._gather(d["kt"], d["vt"], seq=meta[1], slots=d["sel"], b_tail=d["b_tail"], b_seq=d["b_seq"])
        max_pg = max([self.packed_groups[r] for r in slots], default=0)
        return self._bundle(d["sel"], d["b_seq"], d["b_tail"], d["kt"], d["vt"], max(1, max_pg * self.gt))

    # ── device decode path ───────────────────────────────────────────────────────────

    def decode_seed_seq_device(self, slots: Sequence[int]) -> torch.Tensor:
        """Seed the device sequence counter and the row -> slot map from the host state
        (kv_pool.py:1015-1035); called once before a decode loop."""
        slots = [int(s) for s in slots]
        B = len(slots)
        d = self._decode_buffers(B)
        meta = torch.tensor([slots, [self.seq_len[r] for r in slots]], dtype=torch.int64).to(
            self.device, non_blocking=True)
        d["rows"].copy_(meta[0])
        d["sel"].copy_(meta[0])
        d["seq_dev"].copy_(meta[1])
        return d["seq_dev"]

    def advance_seq_device(self, B: int) -> None:
        """``seq_dev += 1`` on the device (kv_pool.py:1037-1046).  ``append_decode_device``
        already does this inside its write launch; this is for callers that write through
        ``append_decode_captured``."""
        d = self._decode_buffers(B)
        d["seq_dev"].add_(1)
        d["cols"].copy_(d["seq_dev"] - 1)

    def decode_inputs_device(self, B: int, max_seq_len: int) -> dict:
        """Decode bundle built entirely on the device from ``seq_dev`` (kv_pool.py:1048-1105):
        boundary, packed / tail lengths, tail positions and the gather are one launch."""
        d = self._decode_buffers(B)
        self._gather(d["kt"], d["vt"], seq=d["seq_dev"], slots=d["sel"], b_tail=d["b_tail"],
                     b_seq=d["b_seq"])
        return self._bundle(d["sel"], d["b_seq"], d["b_tail"], d["kt"], d["vt"], max_seq_len)


__all__ = ["MultiSeqKVPool", "check_serving_recipe"]
