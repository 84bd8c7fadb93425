"""Single-sequence KV store: packed planes + bf16 residual history of ONE request.

Same class and methods as the reference ``ommx_gpu_serve/attention/kv_store.py:93-710``
(``CanonicalKVStore``), backed by the HIP kernels of this package: ``write_token`` and
``gather_tail_into`` are the ring copy kernels, every pack is one ``ommx_store_pack`` launch
that writes straight into the plane slots of the completed groups (the reference packs into
temporaries on the host seam and copies plane by plane, ``kv_store.py:551-610``).  The store
kernel does not synchronise with the host, so packing is legal at any point of a step;
non-finite input is reported through ``err_flag`` / ``check_errors()``.

Only the serving recipe is implemented (see ``kv_pool.check_serving_recipe``).  The store
lives on a ROCm GPU; there is no CPU path.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _hip
from .kv_pool import _env_flag, check_serving_recipe
from .kv_store_ops import gather_tail, ring_slot, write_token
from .kv_window import CANONICAL_GROUP_TOKENS, WindowSpec
from .pack import index_plane_bytes, raise_for_store_errors, store_pack_into


class CanonicalKVStore:
    """Per-layer packed planes + bf16 tail of one sequence."""

    def __init__(
        self,
        head_dim: int,
        n_kv_heads: int,
        max_seq_len: int,
        *,
        k_format: str = "i2f4",
        v_format: str = "i2",
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
        if str(v_format).lower() not in ("i2", "bf16"):
            raise ValueError(f"v_format must be i2|bf16; got {v_format!r}")
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
                             scale_dtype=scale_dtype, outliers_per_vector=outliers_per_vector,
                             v_format=v_format)
        self.D, self.H, self.max_seq_len = int(head_dim), int(n_kv_heads), int(max_seq_len)
        # "itf4" names the same K planes; V is INT2 codes or, with "bf16", the rows as they came
        # (kv_store.py:120-127, 183-188)
        self.k_format, self.v_format = str(k_format).lower(), str(v_format).lower()
        self.k = int(outliers_per_vector)
        self.outlier_select = str(outlier_select).lower()
        self.outlier_repr = str(outlier_repr).lower()
        self.use_pow2 = bool(use_pow2)
        self.kv_int8_scale = bool(kv_int8_scale) and bool(use_pow2)      # pack.py:397
        self.kv_outlier_map = bool(kv_outlier_map)
        self.scale_dtype = scale_dtype
        self.device = torch.device(device)
        _hip.require_gpu(self.device)
        _hip.load()
        self.pages_per_group = self.gt // self.ps
        self.gc = int(group_channels)
        self.k_base_bits, self.oval_bits = 2, 4
        self.k_base_w = self.D // 4
        self.NGV = self.D // self.gc
        # one group of slack so a just-completed group always has a slot (kv_store.py:172-174)
        self.G_cap = max(1, (self.max_seq_len + self.gt - 1) // self.gt + 1)
        self.P_cap = self.G_cap * self.pages_per_group

        dev, bf, z = self.device, torch.bfloat16, torch.zeros
        self.k_base = z(self.P_cap, self.ps, self.H, self.k_base_w, dtype=torch.uint8, device=dev)
        if self.v_format == "bf16":
            self.v_main = z(self.P_cap, self.ps, self.H, self.D, dtype=bf, device=dev)
        else:
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

        self.kv_ring = _env_flag("OMMX_KV_RING", False) if kv_ring is None else bool(kv_ring)
        self._fused_io = True
        self.kv_cap = self.max_seq_len
        if self.kv_ring:   # kv_store.py:196-214
            self._ring_sink = int(self.window.sink_tokens)
            self._ring_rec = int(self.window.recent_window) + 2 * self.gt
            self.ring_cap = self._ring_sink + self._ring_rec
        else:
            self._ring_sink, self._ring_rec, self.ring_cap = 0, 0, self.kv_cap
        self.k_hist = z(self.ring_cap, self.H, self.D, dtype=bf, device=dev)
        self.v_hist = z(self.ring_cap, self.H, self.D, dtype=bf, device=dev)
        self.seq_len = 0
        self.packed_groups = 0

        self._req_to_token_full = torch.arange(self.P_cap, dtype=torch.int32, device=dev).reshape(1, self.P_cap)
        self._req_to_group_full = torch.arange(self.G_cap, dtype=torch.int32, device=dev).reshape(1, self.G_cap)
        self.tail_cap = int(self.window.sink_tokens + self.window.recent_window + self.window.group_tokens)
        self.k_tail_buf = z(1, self.tail_cap, self.H, self.D, dtype=bf, device=dev)
        self.v_tail_buf = z(1, self.tail_cap, self.H, self.D, dtype=bf, device=dev)
        self.err_flag = torch.zeros(1, dtype=torch.int32, device=dev)
        self.wide_steps = False      # a packed K step above 2^15 was seen: decode on the plain kernel

    # ── ring address mapping (kv_store.py:301-327) ────────────────────────────────────

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
            raise IndexError("OMMX KV write/gather outside residual capacity")
        raise_for_store_errors(bits)

    # ── lifecycle ─────────────────────────────────────────────────────────────────

    def reset_inplace(self) -> None:
        """New sequence, same tensors (kv_store.py:331-345): only the cursors move."""
        self.seq_len = 0
        self.packed_groups = 0

    # ── write path ───────────────────────────────────────────────────────────────

    def append(self, k: torch.Tensor, v: torch.Tensor) -> None:
        """Stash one decode step's K/V row ``[H, D]`` (kv_store.py:349-357)."""
        if not self.kv_ring and self.seq_len >= self.kv_cap:
            raise RuntimeError(f"CanonicalKVStore capacity {self.kv_cap} exceeded (seq_len)")
        slot = self._ring_slot_host(self.seq_len)
        self.k_hist[slot] = k.reshape(self.H, self.D).to(self.device, torch.bfloat16)
        self.v_hist[slot] = v.reshape(self.H, self.D).to(self.device, torch.bfloat16)
        self.seq_len += 1

    def write_token(self, pos: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> None:
        """Write one K/V row at the absolute position held in the device tensor ``pos``
        ([1] int64); launch-only, ``seq_len`` is not touched (kv_store.py:361-385)."""
        kb = k.reshape(self.H, self.D)
        vb = v.reshape(self.H, self.D)
        if kb.dtype != torch.bfloat16 or kb.device != self.device:
            kb = kb.to(self.device, torch.bfloat16)
        if vb.dtype != torch.bfloat16 or vb.device != self.device:
            vb = vb.to(self.device, torch.bfloat16)
        if kb.stride(-1) != 1:
            kb = kb.contiguous()
        if vb.stride(-1) != 1:
            vb = vb.contiguous()
        if pos.dtype != torch.int64 or pos.device != self.device:
            pos = pos.to(self.device, torch.int64)
        write_token(self.k_hist, self.v_hist, pos.reshape(-1)[:1].contiguous(), kb, vb,
                    self._ring_sink, self._ring_rec, err_flag=self.err_flag)

    def advance_to(self, seq_len: int) -> int:
        """Set the sequence length and pack completed groups (kv_store.py:387-395)."""
        self.seq_len = int(seq_len)
        return self.maybe_regroup()

    def gather_tail_into(self, tail_idx: torch.Tensor, k_tail: torch.Tensor, v_tail: torch.Tensor,
                         n_valid: int) -> None:
        """Gather the rows at absolute positions ``tail_idx [T]`` into the fixed buffers
        ``k_tail`` / ``v_tail [1, T, H, D]``; launch-only (kv_store.py:397-427)."""
        if tail_idx.device != self.device:
            tail_idx = tail_idx.to(self.device)
        gather_tail(self.k_hist, self.v_hist, tail_idx, k_tail, v_tail, self._ring_sink, self._ring_rec,
                    err_flag=self.err_flag)

    def append_block(self, K: torch.Tensor, V: torch.Tensor) -> None:
        """Stash a prefill block ``[T, H, D]`` and pack its completed groups (kv_store.py:429-490)."""
        T = int(K.shape[0])
        Kb = K.to(self.device, torch.bfloat16)
        Vb = V.to(self.device, torch.bfloat16)
        if not self.kv_ring:
            if self.seq_len + T > self.kv_cap:
                raise RuntimeError("CanonicalKVStore capacity exceeded (block)")
            self.k_hist[self.seq_len:self.seq_len + T] = Kb
            self.v_hist[self.seq_len:self.seq_len + T] = Vb
            self.seq_len += T
            self.maybe_regroup()
            return
        if self.seq_len != 0:
            raise RuntimeError(
                "ring append_block expects a fresh sequence (seq_len==0); chunked prefill under "
                "the ring is not supported. Reset the store before each prefill block.")
        self.seq_len = T
        target = self.window.num_groups(T)
        if target > 0:
            sink = self.window.sink_tokens
            self._pack_block_into_planes(Kb[sink:sink + target * self.gt],
                                         Vb[sink:sink + target * self.gt], 0, target)
            self.packed_groups = target
        boundary = self.window.boundary(T)
        sink_tokens = self.window.sink_tokens
        lo = max(sink_tokens, boundary - self.gt)
        parts = [torch.arange(0, min(sink_tokens, T), device=self.device)]
        if lo < T:
            parts.append(torch.arange(lo, T, device=self.device))
        live = torch.cat(parts).to(torch.long)
        slots = self._ring_slot_dev(live)
        self.k_hist.index_copy_(0, slots, Kb.index_select(0, live))
        self.v_hist.index_copy_(0, slots, Vb.index_select(0, live))

    def maybe_regroup(self) -> int:
        """Pack any newly completed groups; returns how many (kv_store.py:492-526)."""
        target = self.window.num_groups(self.seq_len)
        if target <= self.packed_groups:
            return 0
        n = target - self.packed_groups
        if self.kv_ring:
            for g in range(self.packed_groups, target):   # one ring span per call
                self._regroup_pack_range(g, g + 1)
        else:
            self._regroup_pack_range(self.packed_groups, target)
        self.packed_groups = target
        return n

    def _planes_for_store(self) -> dict:
        return {"k_base": self.k_base, "k_scale": self.k_scale, "k_zp": self.k_zp,
                "k_fp4_mapscale": self.k_fp4_mapscale, "k_fp4_mapcenter": self.k_fp4_mapcenter,
                "k_obmp": self.k_obmp, "k_oidx": self.k_oidx, "k_oval": self.k_oval,
                "k_crank": self.k_crank,
                "_k_obmp_scratch": self.k_obmp if self.outlier_repr == "combinadic" else None,
                "v_main": self.v_main, "v_scale": self.v_scale, "v_zp": self.v_zp}

    def _regroup_pack_range(self, g0: int, g1: int) -> None:
        sink = self.window.sink_tokens
        t0, t1 = sink + g0 * self.gt, sink + g1 * self.gt
        if self.kv_ring:
            rows = torch.tensor([self._ring_slot_host(t) for t in range(t0, t1)], dtype=torch.int32).to(
                self.device, non_blocking=True)
            self._pack_block_into_planes(self.k_hist, self.v_hist, g0, g1, src_rows=rows)
        else:
            self._pack_block_into_planes(self.k_hist[t0:t1], self.v_hist[t0:t1], g0, g1)

    def _pack_block_into_planes(self, K_blk: torch.Tensor, V_blk: torch.Tensor, g0: int, g1: int,
                                src_rows: Optional[torch.Tensor] = None) -> None:
        """Pack ``(g1-g0)*gt`` tokens into group slots ``[g0, g1)`` with one store launch
        (kv_store.py:551-610)."""
        n_tok = (g1 - g0) * self.gt
        ppg = self.pages_per_group
        store_pack_into(K_blk, V_blk, self._planes_for_store(), outliers_per_vector=self.k,
                        outlier_repr=self.outlier_repr, outlier_select=self.outlier_select,
                        use_pow2=self.use_pow2, kv_int8_scale=self.kv_int8_scale,
                        group_tokens=self.gt, group_channels=self.gc, v_format=self.v_format,
                        page_size=self.ps, src_rows=src_rows,
                        dst_pages=self._req_to_token_full.view(-1)[g0 * ppg:g1 * ppg],
                        dst_groups=self._req_to_group_full.view(-1)[g0:g1],
                        err_flag=self.err_flag, num_tokens=n_tok)

    # ── read path ────────────────────────────────────────────────────────────────

    def _meta(self) -> dict:
        return {"head_dim": self.D, "n_kv_heads": self.H, "page_size": self.ps,
                "outliers_per_vector": self.k, "outlier_repr": self.outlier_repr,
                "outlier_select": self.outlier_select, "group_tokens": self.gt,
                "group_channels": self.gc, "k_format": self.k_format, "v_format": self.v_format,
                "k_base_bits": self.k_base_bits, "oval_bits": self.oval_bits,
                "kv_outlier_map": bool(self.kv_outlier_map and self.k > 0), "kv_int8_scale": self.kv_int8_scale}

    def decode_planes(self) -> dict:
        """Plane dict over the filled slots (kv_store.py:614-649)."""
        G = self.packed_groups
        P = G * self.pages_per_group

        def cut(t, n):
            return None if t is None else t[:n]

        out = {"k_base": self.k_base[:P], "k_scale": self.k_scale[:G], "k_zp": self.k_zp[:G],
               "k_oidx": cut(self.k_oidx, G), "k_crank": cut(self.k_crank, G), "k_oval": cut(self.k_oval, G),
               "k_obmp": cut(self.k_obmp, G), "k_fp4_mapscale": cut(self.k_fp4_mapscale, G),
               "k_fp4_mapcenter": cut(self.k_fp4_mapcenter, G),
               "v_main": self.v_main[:P], "v_scale": self.v_scale[:P], "v_zp": self.v_zp[:P],
               "req_to_token": self._req_to_token_full[:, :P],
               "req_to_group": self._req_to_group_full[:, :G],
               "num_tokens": G * self.gt, "n_groups": G}
        out.update(self._meta())
        out["err_flag"], out["force_reference_kernel"] = self.err_flag, self.wide_steps
        return out

    def decode_planes_full(self) -> dict:
        """Full-capacity, fixed-address plane dict (kv_store.py:651-676)."""
        out = {"k_base": self.k_base, "k_scale": self.k_scale, "k_zp": self.k_zp,
               "k_oidx": self.k_oidx, "k_oval": self.k_oval, "k_crank": self.k_crank, "k_obmp": self.k_obmp,
               "k_fp4_mapscale": self.k_fp4_mapscale, "k_fp4_mapcenter": self.k_fp4_mapcenter,
               "v_main": self.v_main, "v_scale": self.v_scale, "v_zp": self.v_zp,
               "req_to_token": self._req_to_token_full, "req_to_group": self._req_to_group_full}
        out.update(self._meta())
        out["err_flag"], out["force_reference_kernel"] = self.err_flag, self.wide_steps
        return out

    def tail_bf16(self) -> Tuple[torch.Tensor, torch.Tensor, int]:
        """``(k_tail [1,n,H,D], v_tail, n)``: the sink + recent rows (kv_store.py:678-694)."""
        idx = self.window.tail_indices(self.seq_len)
        n = len(idx)
        kt = torch.empty(1, n, self.H, self.D, dtype=torch.bfloat16, device=self.device)
        vt = torch.empty_like(kt)
        if n:
            ti = torch.tensor(idx, dtype=torch.int64).to(self.device)
            gather_tail(self.k_hist, self.v_hist, ti, kt, vt, self._ring_sink, self._ring_rec,
                        err_flag=self.err_flag)
        return kt, vt, n

    def decode_inputs(self) -> dict:
        """Argument bundle of the decode operator at the current state (kv_store.py:696-710)."""
        planes = self.decode_planes()
        kt, vt, n_tail = self.tail_bf16()
        packed_tokens = self.packed_groups * self.gt
        return {
            "planes": planes, "k_tail": kt, "v_tail": vt,
            "b_tail_len": torch.tensor([n_tail], dtype=torch.int32).to(self.device),
            "b_seq_len": torch.tensor([packed_tokens], dtype=torch.int32).to(self.device),
            "packed_start_offset": 0,
            "max_seq_len": max(1, packed_tokens),
            "max_tail_len": self.window.max_tail_len(self.max_seq_len),
        }


__all__ = ["CanonicalKVStore"]
