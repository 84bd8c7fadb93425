"""Deterministic synthetic KV caches and decode requests in the shapes the benchmarks use.

Everything is drawn from numpy's counter-based Philox generator, so a (seed, shape) pair
gives the same bf16 tensors on every machine.  ``build_decode_case`` stores the packed
prefix of each request with the HIP quantize-on-store kernel into one shared pool of
16-token pages and 32-token group slots (optionally through shuffled tables) and returns
every argument of the decode operator.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence

import numpy as np
import torch

from .attention.kv_window import WindowSpec
from .attention.pack import alloc_planes, raise_for_store_errors, store_pack_into


def _rng(seed: int, stream: int) -> np.random.Generator:
    return np.random.Generator(np.random.Philox(key=[int(seed), int(stream)]))


def synth_kv(num_tokens: int, kv_heads: int, head_dim: int, seed: int, *,
             outlier_channels: int = 4, outlier_gain: float = 12.0,
             sparse_frac: float = 0.0, sparse_gain: float = 8.0, stream: int = 0):
    """bf16 ``(K, V)`` ``[T, H, D]`` ~ N(0,1).  ``outlier_channels`` fixed channels of every
    K head are scaled by ``outlier_gain``; a further ``sparse_frac`` of K elements, at
    random positions, by ``sparse_gain``."""
    g = _rng(seed, stream)
    shape = (num_tokens, kv_heads, head_dim)
    K = g.standard_normal(shape, dtype=np.float32)
    V = g.standard_normal(shape, dtype=np.float32)
    if outlier_channels > 0:
        gc = _rng(seed, 7777)                      # channel choice does not depend on T
        for h in range(kv_heads):
            ch = gc.choice(head_dim, size=outlier_channels, replace=False)
            K[:, h, ch] *= outlier_gain
    if sparse_frac > 0:
        K[g.random(shape, dtype=np.float32) < sparse_frac] *= sparse_gain
    return torch.from_numpy(K).to(torch.bfloat16), torch.from_numpy(V).to(torch.bfloat16)


def synth_q(batch: int, q_heads: int, head_dim: int, seed: int):
    """bf16 queries ``[B, Hq, D]`` ~ N(0,1)."""
    g = _rng(seed, 1_000_003)
    return torch.from_numpy(g.standard_normal((batch, q_heads, head_dim), dtype=np.float32)).to(torch.bfloat16)


@dataclass
class DecodeCase:
    """All operands of one batched decode call, on ``device``, plus what a checker needs."""
    q: torch.Tensor
    planes: Dict[str, Any]
    k_tail: torch.Tensor
    v_tail: torch.Tensor
    b_tail_len: torch.Tensor
    req_to_token: torch.Tensor
    req_to_group: torch.Tensor
    b_seq_len: torch.Tensor
    sm_scale: float
    page_size: int
    q_heads: int
    kv_heads: int
    head_dim: int
    seq_lens: List[int]
    outliers_per_vector: int = 6
    outlier_repr: str = "bitmap"
    extra: Dict[str, Any] = field(default_factory=dict)

    def decode_kwargs(self) -> Dict[str, Any]:
        p = self.planes
        return dict(sm_scale=self.sm_scale, page_size=self.page_size,
                    k_outliers_per_vector=self.outliers_per_vector, k_format="i2f4",
                    bitmap_read=self.outliers_per_vector > 0 and self.outlier_repr == "bitmap",
                    k_obmp=p["k_obmp"],
                    k_fp4_mapscale=p["k_fp4_mapscale"], k_fp4_mapcenter=p["k_fp4_mapcenter"],
                    kv_outlier_map=self.outliers_per_vector > 0 and p["k_fp4_mapscale"] is not None,
                    kv_int8_scale=p["k_scale"].dtype == torch.int8,
                    max_seq_len=max(1, int(max(self.packed_lens))),
                    max_tail_len=int(self.k_tail.shape[1]))

    @property
    def packed_lens(self) -> List[int]:
        return [int(x) for x in self.extra["packed_lens"]]

    def decode_args(self, o: torch.Tensor, lse: torch.Tensor):
        p = self.planes
        return (self.q, p["k_base"], p["k_scale"], p["k_zp"], p.get("k_oidx"), p["k_oval"],
                p["v_main"], p["v_scale"], p["v_zp"], self.k_tail, self.v_tail, self.b_tail_len,
                o, lse, self.req_to_token, self.req_to_group, self.b_seq_len)

    def algorithmic_bytes(self) -> int:
        """Bytes the decode must read: every plane byte of the live packed prefix plus the
        bf16 tail rows (K and V); q, partials and outputs are not counted."""
        D, H, k = self.head_dim, self.kv_heads, self.outliers_per_vector
        per_tok = D // 4 + D // 4 + D // 32 + 2 * (D // 32)
        nidx = 4 if self.outlier_repr == "bitmap" else (7 * k + 7) // 8
        nmap = 4 if self.planes.get("k_fp4_mapscale") is not None else 0
        per_grp = D * (1 + 2 + (nmap + nidx + (k + 1) // 2 if k > 0 else 0))
        tails = [int(x) for x in self.b_tail_len.tolist()]
        tot = 0
        for L, tl in zip(self.packed_lens, tails):
            tot += L * H * per_tok + (L // 32) * H * per_grp + tl * H * D * 2 * 2
        return tot


def build_decode_case(seq_lens: Sequence[int], *, q_heads: int = 32, kv_heads: int = 8,
                      head_dim: int = 128, page_size: int = 16, seed: int = 42,
                      permute_tables: bool = False, sparse_frac: float = 0.0,
                      outliers_per_vector: int = 6, window: Optional[WindowSpec] = None,
                      device: Any = "cuda", keep_source: bool = False,
                      table_dtype: torch.dtype = torch.int32, sparse_gain: float = 8.0,
                      outlier_repr: str = "bitmap", kv_outlier_map: bool = True,
                      use_pow2: bool = True, kv_int8_scale: bool = True,
                      group_tokens: int = 32, group_channels: int = 32, v_format: str = "i2",
                      outlier_gain: float = 12.0) -> DecodeCase:
    """Synthesize ``len(seq_lens)`` requests, store their packed prefixes, gather their tails.

    Each request gets its own slice of page / group-slot ids out of one shared pool; with
    ``permute_tables`` the ids of all requests are shuffled together, so consecutive
    logical pages of a request land anywhere in the pool.
    """
    gt, gc = int(group_tokens), int(group_channels)
    win = window or WindowSpec(page_size=page_size, group_tokens=gt)
    assert win.group_tokens == gt
    dev = torch.device(device)
    B, H, D, ps = len(seq_lens), kv_heads, head_dim, page_size
    packed = [win.packed_len(int(n)) for n in seq_lens]
    n_pages = [p // ps for p in packed]
    n_groups = [p // gt for p in packed]
    # at least one whole group (gt // ps pages), so the planes keep the group geometry
    tot_pages, tot_groups = max(max(1, gt // ps), sum(n_pages)), max(1, sum(n_groups))
    g = _rng(seed, 424242)
    page_ids = g.permutation(tot_pages) if permute_tables else np.arange(tot_pages)
    # group slots follow their pages only through the tables, so shuffle them separately
    group_ids = g.permutation(tot_groups) if permute_tables else np.arange(tot_groups)
    planes = alloc_planes(tot_pages, tot_groups, H, D, page_size=ps,
                          outliers_per_vector=outliers_per_vector, device=dev,
                          outlier_repr=outlier_repr, kv_outlier_map=kv_outlier_map,
                          int8_scale=bool(use_pow2) and bool(kv_int8_scale),
                          group_tokens=gt, group_channels=gc, v_format=v_format)
    planes["outlier_repr"] = str(outlier_repr).lower()
    planes["group_tokens"], planes["group_channels"] = gt, gc
    for t in planes.values():
        if torch.is_tensor(t):
            t.zero_()
    max_pages, max_groups = max(1, max(n_pages)), max(1, max(n_groups))
    rt = np.zeros((B, max_pages), dtype=np.int64)
    rg = np.zeros((B, max_groups), dtype=np.int64)
    max_tail = max(1, max(len(win.tail_indices(int(n))) for n in seq_lens))
    k_tail = torch.zeros(B, max_tail, H, D, dtype=torch.bfloat16)
    v_tail = torch.zeros(B, max_tail, H, D, dtype=torch.bfloat16)
    tails = []
    err = torch.zeros(1, dtype=torch.int32, device=dev)
    src = []
    po = go = 0
    for b, n in enumerate(int(x) for x in seq_lens):
        K, V = synth_kv(n, H, D, seed, sparse_frac=sparse_frac, sparse_gain=sparse_gain, stream=b,
                        outlier_gain=outlier_gain)
        edge = win.boundary(n)
        ti = win.tail_indices(n)
        tails.append(len(ti))
        if ti:
            idx = torch.tensor(ti, dtype=torch.int64)
            k_tail[b, :len(ti)] = K[idx]
            v_tail[b, :len(ti)] = V[idx]
        rt[b, :n_pages[b]] = page_ids[po:po + n_pages[b]]
        rg[b, :n_groups[b]] = group_ids[go:go + n_groups[b]]
        if packed[b] > 0:
            Kd = K[win.sink_tokens:edge].to(dev)
            Vd = V[win.sink_tokens:edge].to(dev)
            store_pack_into(Kd, Vd, planes, outliers_per_vector=outliers_per_vector, page_size=ps,
                            dst_pages=torch.from_numpy(rt[b, :n_pages[b]].astype(np.int32)).to(dev),
                            dst_groups=torch.from_numpy(rg[b, :n_groups[b]].astype(np.int32)).to(dev),
                            err_flag=err, outlier_repr=outlier_repr, use_pow2=use_pow2,
                            kv_int8_scale=kv_int8_scale, group_tokens=gt, group_channels=gc,
                            v_format=v_format)
        po += n_pages[b]
        go += n_groups[b]
        if keep_source:
            src.append((K, V))
    raise_for_store_errors(int(err.item()))
    case = DecodeCase(
        q=synth_q(B, q_heads, D, seed).to(dev), planes=planes,
        k_tail=k_tail.to(dev), v_tail=v_tail.to(dev),
        b_tail_len=torch.tensor(tails, dtype=torch.int32, device=dev),
        req_to_token=torch.from_numpy(rt).to(table_dtype).to(dev),
        req_to_group=torch.from_numpy(rg).to(table_dtype).to(dev),
        b_seq_len=torch.tensor(packed, dtype=torch.int32, device=dev),
        sm_scale=1.0 / math.sqrt(D), page_size=ps, q_heads=q_heads, kv_heads=H, head_dim=D,
        seq_lens=[int(x) for x in seq_lens], outliers_per_vector=outliers_per_vector,
        outlier_repr=str(outlier_repr).lower(),
        extra={"packed_lens": packed, "window": win})
    if keep_source:
        case.extra["source"] = src
    return case
