"""CPU restatement of the OMMX paged decode-attention path.  TEST INFRASTRUCTURE ONLY.

This module is the checker the HIP kernels are compared against.  Nothing in the
shipped package may import it: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do.  It runs on torch-CPU because the reference's
own packer is torch-CPU code whose results depend on torch's fp32 ``log2`` / ``log`` /
``round`` / stable ``sort`` routines; calling the same library routines is what makes a
bit-exact comparison meaningful.

Every function names the reference lines it restates (paths relative to the reference
checkout, ``ommx_gpu_serve/attention/``).

Parity status of each function (what pins it, besides reading):

  fp4_encode / fp4_decode      closed form + the 16 fixed points + brute-force
                               nearest-in-log check            (tests/test_oracle_pins.py)
  pack_int2 / unpack_int2      closed form, round trip
  bitmap_pack / bitmap_unpack  closed form, popcount / rank-rule invariants
  relidx7_pack / relidx7_unpack  closed form (7-bit LSB-first stream) against big-integer
                               arithmetic and hand-computed bytes; positions equal the
                               bitmap's for the same input; planes the reference packer
                               wrote (tests/golden/variant_relidx7.npz, ..._k16_relidx7)
  combinadic_pack / _unpack    the combinatorial number system: every k-subset of a small set
                               enumerated in colexicographic order takes the ranks 0, 1, 2 ...
                               in turn; first / last subset, a hand-computed rank, field widths
                               of the reference's recipes; a plane the reference packer
                               wrote (tests/golden/variant_combinadic.npz)
  pow2_exponent                rule 2^rint(log2(x)) incl. exact-tie vectors
  select_outliers_signed       brute-force rank counting on small vectors with ties
  select_outliers_abs          the same, on magnitudes
  pack_kv                      golden planes written by the reference packer itself: five
                               blocks of the serving recipe (tests/golden/pack_*.npz) and one
                               block per variant branch -- index planes, base-shared outliers,
                               magnitude selector, free / bf16 steps, 16/64/128-element
                               vectors with 0..16 outliers, bf16 V (tests/golden/variant_*.npz)
  dequant_kv                   the reference's dequant of every one of those plane sets;
                               encode/decode identity
  attend / decode_reference    softmax closed forms, fp64 cross-check, split-merge
                               associativity
  WindowSpec arithmetic        closed forms + the invariant recent <= seq-boundary < recent+gt
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence, Tuple

import torch

GROUP_TOKENS = 32
GROUP_CHANNELS = 32
FP4_LEVELS = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


# ---------------------------------------------------------------------------------------
# FP4 E2M1 codec                                                       codec.py:29-80
# ---------------------------------------------------------------------------------------

def _fp4_log_levels() -> torch.Tensor:
    # codec.py:38-41: log of the level table with the zero level clamped to 1e-8
    lv = torch.tensor(FP4_LEVELS, dtype=torch.float32)
    return torch.log(lv.clamp_min(1e-8))


def fp4_encode(x: torch.Tensor) -> torch.Tensor:
    """Float -> 4-bit code ``sign<<3 | exp<<1 | mant`` (uint8).  codec.py:45-65.

    Nearest level in fp32 log magnitude, first minimum wins (ties go to the lower
    level), exact zero encodes to level 0, sign bit is ``x < 0`` whatever the level.
    """
    xf = x.to(torch.float32)
    if not bool(torch.isfinite(xf).all()):
        raise ValueError("fp4_encode: non-finite input")
    a = xf.abs()
    d = (torch.log(a.clamp_min(1e-8)).unsqueeze(-1) - _fp4_log_levels()).abs()
    idx = torch.argmin(d, dim=-1)
    idx = torch.where(a == 0, torch.zeros_like(idx), idx)
    exp = (idx >= 2).to(torch.int64) + (idx >= 4).to(torch.int64) + (idx >= 6).to(torch.int64)
    mant = idx & 1
    sign = (xf < 0).to(torch.int64)
    return ((sign << 3) | (exp << 1) | mant).to(torch.uint8)


def fp4_decode(code: torch.Tensor) -> torch.Tensor:
    """4-bit code -> signed fp32 level.  codec.py:68-80."""
    c = code.to(torch.int64) & 0xF
    # exp==0 -> 0.5*mant, else (1+0.5*mant)*2^(exp-1): exactly the level table indexed
    # by the low three bits (exp<<1 | mant).
    v = torch.tensor(FP4_LEVELS, dtype=torch.float32)[c & 7]
    return torch.where(((c >> 3) & 1).bool(), -v, v)


# ---------------------------------------------------------------------------------------
# bit layouts                                         pack.py:97-125, codec.py:330-406
# ---------------------------------------------------------------------------------------

def pack_int2(codes: torch.Tensor) -> torch.Tensor:
    """codes 0..3 ``[..., D]`` -> uint8 ``[..., D/4]``; channel c sits in byte c//4 at
    bits ``2*(c%4)+1 : 2*(c%4)``.  pack.py:97-104."""
    c = (codes.to(torch.int64) & 3).reshape(*codes.shape[:-1], codes.shape[-1] // 4, 4)
    w = torch.tensor([1, 4, 16, 64], dtype=torch.int64)
    return (c * w).sum(-1).to(torch.uint8)


def unpack_int2(plane: torch.Tensor) -> torch.Tensor:
    """Inverse of :func:`pack_int2`.  pack.py:107-113."""
    p = plane.to(torch.int64).unsqueeze(-1)
    sh = torch.tensor([0, 2, 4, 6], dtype=torch.int64)
    return ((p >> sh) & 3).reshape(*plane.shape[:-1], plane.shape[-1] * 4)


def bitmap_pack(pos: torch.Tensor, n: int = GROUP_TOKENS) -> torch.Tensor:
    """Ascending distinct positions ``[..., k]`` -> ``[..., n/8]`` bytes, position p in
    byte p>>3 bit p&7.  codec.py:330-372."""
    p = pos.to(torch.int64)
    if bool((p < 0).any()) or bool((p >= n).any()):
        raise ValueError("bitmap_pack: position out of range")
    occ = torch.zeros(*p.shape[:-1], n, dtype=torch.int64)
    occ.scatter_(-1, p, 1)
    if bool((occ.sum(-1) != p.shape[-1]).any()):
        raise ValueError("bitmap_pack: duplicate position")
    w = 1 << torch.arange(8, dtype=torch.int64)
    return (occ.reshape(*p.shape[:-1], n // 8, 8) * w).sum(-1).to(torch.uint8)


def bitmap_unpack(bmp: torch.Tensor, k: int, n: int = GROUP_TOKENS) -> torch.Tensor:
    """``[..., n/8]`` bytes -> ascending set positions ``[..., k]``.  codec.py:375-406."""
    b = bmp.to(torch.int64).unsqueeze(-1)
    occ = ((b >> torch.arange(8, dtype=torch.int64)) & 1).reshape(*bmp.shape[:-1], n).bool()
    if bool((occ.sum(-1) != k).any()):
        raise ValueError("bitmap_unpack: a frame does not hold exactly k set bits")
    idx = torch.arange(n, dtype=torch.int64).expand_as(occ)
    return torch.where(occ, idx, torch.full_like(idx, n)).sort(-1)[0][..., :k]


def relidx7_pack(pos: torch.Tensor) -> torch.Tensor:
    """Ascending positions ``[..., k]`` -> ``[..., ceil(7k/8)]`` bytes: position s occupies
    bits [7s, 7s+7) of a little-endian bit stream, least significant bit first.
    pack.py:128-164, codec.py:91-107."""
    p = pos.to(torch.int64)
    if bool((p < 0).any()) or bool((p > 127).any()):
        raise ValueError("relidx7_pack: position out of range")
    k = int(p.shape[-1])
    nbytes = (7 * k + 7) // 8
    bits = ((p.unsqueeze(-1) >> torch.arange(7, dtype=torch.int64)) & 1).reshape(*p.shape[:-1], 7 * k)
    pad = nbytes * 8 - 7 * k
    if pad:
        bits = torch.cat([bits, torch.zeros(*p.shape[:-1], pad, dtype=torch.int64)], dim=-1)
    w = 1 << torch.arange(8, dtype=torch.int64)
    return (bits.reshape(*p.shape[:-1], nbytes, 8) * w).sum(-1).to(torch.uint8)


def relidx7_unpack(plane: torch.Tensor, k: int) -> torch.Tensor:
    """Inverse of :func:`relidx7_pack`: ``[..., ceil(7k/8)]`` bytes -> positions ``[..., k]``.
    pack.py:167-174, codec.py:110-121."""
    b = plane.to(torch.int64).unsqueeze(-1)
    bits = ((b >> torch.arange(8, dtype=torch.int64)) & 1).reshape(*plane.shape[:-1], plane.shape[-1] * 8)
    bits = bits[..., : 7 * k].reshape(*plane.shape[:-1], k, 7)
    return (bits * (1 << torch.arange(7, dtype=torch.int64))).sum(-1)


def combinadic_bytes(k: int, n: int = GROUP_TOKENS) -> int:
    """Bytes of one combinadic rank: ``ceil(log2 C(n, k))`` bits, at least one.
    codec.py:131-143."""
    if k <= 0 or k >= n:
        return 0
    return (max(1, (math.comb(n, k) - 1).bit_length()) + 7) // 8


def combinadic_pack(pos: torch.Tensor, n: int = GROUP_TOKENS) -> torch.Tensor:
    """Ascending distinct positions ``[..., k]`` -> ``[..., combinadic_bytes]`` little-endian
    ranks: the rank of ``p_1 < ... < p_k`` is ``sum_i C(p_i, i)`` (the combinatorial number
    system; codec.py:146-158 sums ``C(c_j, k-j)`` over the descending order, the same terms).
    Python integers, so no width limit.  pack.py:179-206."""
    k = int(pos.shape[-1])
    nb = combinadic_bytes(k, n)
    flat = pos.reshape(-1, k).tolist()
    out = torch.zeros(len(flat), nb, dtype=torch.uint8)
    for r, cols in enumerate(flat):
        cols = sorted(int(c) for c in cols)
        if len(set(cols)) != k or cols[0] < 0 or cols[-1] >= n:
            raise ValueError("combinadic_pack: positions must be distinct and inside the group")
        rank = sum(math.comb(c, i + 1) for i, c in enumerate(cols))
        out[r] = torch.tensor(list(rank.to_bytes(nb, "little")), dtype=torch.uint8)
    return out.reshape(*pos.shape[:-1], nb)


def combinadic_unpack(plane: torch.Tensor, k: int, n: int = GROUP_TOKENS) -> torch.Tensor:
    """Ranks ``[..., bytes]`` -> ascending positions ``[..., k]`` by the greedy inverse: for
    ``i = k .. 1`` take the largest ``c`` with ``C(c, i) <= rest``.  codec.py:161-180,
    pack.py:209-223."""
    flat = plane.reshape(-1, int(plane.shape[-1])).tolist()
    out = torch.zeros(len(flat), k, dtype=torch.int64)
    for r, bs in enumerate(flat):
        rem = int.from_bytes(bytes(bs), "little")
        cols = []
        for i in range(k, 0, -1):
            c = n - 1
            while c >= i - 1 and math.comb(c, i) > rem:
                c -= 1
            if c < i - 1:
                raise ValueError("invalid combinadic rank")
            rem -= math.comb(c, i)
            cols.append(c)
        if rem != 0 or len(set(cols)) != k:
            raise ValueError("invalid combinadic rank")
        out[r] = torch.tensor(sorted(cols), dtype=torch.int64)
    return out.reshape(*plane.shape[:-1], k)


def outlier_positions(planes: Dict[str, object], gsel, k: int, gt: int = GROUP_TOKENS) -> torch.Tensor:
    """Ascending outlier positions ``[n, H, D, k]`` of the group slots ``gsel`` from whichever
    index plane the pack carries (both decode to the same positions, pack.py:323-326)."""
    if str(planes.get("outlier_repr", "bitmap")).lower() == "relidx7":
        return relidx7_unpack(planes["k_oidx"][gsel], k)
    if str(planes.get("outlier_repr", "bitmap")).lower() == "combinadic":
        return combinadic_unpack(planes["k_crank"][gsel], k, gt)
    return bitmap_unpack(planes["k_obmp"][gsel], k, gt)


def nibbles_pack(val: torch.Tensor) -> torch.Tensor:
    """k 4-bit values ``[..., k]`` -> ``[..., ceil(k/2)]`` bytes, even slot = low nibble.
    pack.py:116-125."""
    v = val.to(torch.int64) & 0xF
    if v.shape[-1] % 2:
        v = torch.cat([v, torch.zeros(*v.shape[:-1], 1, dtype=torch.int64)], -1)
    return (v[..., 0::2] | (v[..., 1::2] << 4)).to(torch.uint8)


def nibbles_unpack(plane: torch.Tensor, k: int) -> torch.Tensor:
    """Inverse of :func:`nibbles_pack`.  pack.py:732-734."""
    p = plane.to(torch.int64)
    return torch.stack([(p[..., s // 2] >> (4 * (s % 2))) & 0xF for s in range(k)], -1)


# ---------------------------------------------------------------------------------------
# quantiser pieces                                                    pack.py:428-501
# ---------------------------------------------------------------------------------------

def _bf16_rt(x: torch.Tensor) -> torch.Tensor:
    """Round to bf16 (nearest even) and back, the ``.to(scale_dtype).to(float32)`` of
    pack.py:463-464, 495-496."""
    return x.to(torch.bfloat16).to(torch.float32)


def pow2_exponent(raw: torch.Tensor) -> torch.Tensor:
    """``rint(log2(max(raw, 1e-12)))`` as fp32 integers.  pack.py:462, 612."""
    return torch.round(torch.log2(raw.clamp_min(1e-12)))


def select_outliers_signed(gw: torch.Tensor, k: int) -> torch.Tensor:
    """Boolean outlier mask over the last axis.  pack.py:436-445.

    The ``ceil(k/2)`` largest values by stable descending sort, then the ``k//2``
    smallest of what is left (already-chosen lanes replaced by +1e9) by stable
    ascending sort; equal values keep ascending index order in both sorts.
    """
    kt = (k + 1) // 2
    kb = k - kt
    mask = torch.zeros_like(gw, dtype=torch.bool)
    if k == 0:
        return mask
    top = torch.sort(gw, dim=-1, descending=True, stable=True)[1][..., :kt]
    mask.scatter_(-1, top, True)
    if kb > 0:
        rest = torch.where(mask, torch.tensor(1e9, dtype=torch.float32), gw)
        bot = torch.sort(rest, dim=-1, descending=False, stable=True)[1][..., :kb]
        mask.scatter_(-1, bot, True)
    return mask


def select_outliers_abs(gw: torch.Tensor, k: int) -> torch.Tensor:
    """Boolean outlier mask: the ``k`` largest magnitudes by stable descending sort of ``|w|``
    (equal magnitudes keep ascending index order).  pack.py:446-448."""
    mask = torch.zeros_like(gw, dtype=torch.bool)
    if k == 0:
        return mask
    top = torch.sort(gw.abs(), dim=-1, descending=True, stable=True)[1][..., :k]
    return mask.scatter_(-1, top, True)


def _masked_min_max(gw: torch.Tensor, keep: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """min / max over lanes where ``keep``; sentinels +-1e9, an empty set gives 0.
    pack.py:455-458 and 486-489."""
    big = torch.tensor(1e9, dtype=torch.float32)
    mn = torch.where(keep, gw, big).min(-1, keepdim=True)[0]
    mx = torch.where(keep, gw, -big).max(-1, keepdim=True)[0]
    mn = torch.where(mn > 1e8, torch.zeros_like(mn), mn)
    mx = torch.where(mx < -1e8, torch.zeros_like(mx), mx)
    return mn, mx


def pack_kv(K: torch.Tensor, V: torch.Tensor, *, page_size: int = 16,
            outliers_per_vector: int = 6, outlier_repr: str = "bitmap",
            kv_outlier_map: bool = True, outlier_select: str = "signed",
            use_pow2: bool = True, kv_int8_scale: bool = True,
            group_tokens: int = GROUP_TOKENS, group_channels: int = GROUP_CHANNELS,
            v_format: str = "i2") -> Dict[str, object]:
    """The pinned serving recipe of ``ommx_pack_kv_canonical_block`` (pack.py:293-655):
    i2f4, signed select, bitmap (or relidx7) index plane, pow2 scales stored as int8
    exponents, dedicated FP4 map, 32-token K vectors, 32-channel V vectors, bf16 side planes.
    ``kv_outlier_map=False`` is the base-shared outlier variant (pack.py:502-506): the FP4 code
    is taken of ``(w - zp) / scale`` and there are no map planes.  ``use_pow2=False`` keeps the
    step ``bf16((max - min) / 3)`` as it comes; the step planes are then bf16, as they are with
    ``kv_int8_scale=False`` (pack.py:397, 459-463, 586-590).

    ``K``/``V`` are ``[T, H, D]`` bf16 or fp32 with T a multiple of 32 and of
    ``page_size``.  Returns the ten planes, identity tables and the metadata keys.
    """
    T, H, D = (int(s) for s in K.shape)
    gt, gc, k = int(group_tokens), int(group_channels), int(outliers_per_vector)
    if gt not in (16, 32, 64, 128) or gc not in (16, 32, 64, 128):          # pack.py:405-408
        raise ValueError("group sizes must be in {16, 32, 64, 128}")
    if tuple(V.shape) != (T, H, D):
        raise ValueError("K/V shape mismatch")
    if T % gt or T % page_size or D % gc:
        raise ValueError("bad block shape")
    if not 0 <= k <= gt:
        raise ValueError("outliers_per_vector out of range")
    G, NGV, pages = T // gt, D // gc, T // page_size
    Kf, Vf = K.to(torch.float32), V.to(torch.float32)

    # ---- K, vector = (head, channel, group) over 32 tokens            pack.py:428-501
    gw = Kf.permute(1, 2, 0).contiguous().reshape(H, D, G, gt)
    sel = str(outlier_select).lower()
    if sel not in ("signed", "abs"):
        raise ValueError("outlier_select must be signed or abs")
    omask = select_outliers_signed(gw, k) if sel == "signed" else select_outliers_abs(gw, k)
    mn, mx = _masked_min_max(gw, ~omask)
    int8_scale = bool(kv_int8_scale) and bool(use_pow2)                  # pack.py:397
    raw = (mx - mn).clamp_min(1e-8) / 3.0
    scale = _bf16_rt(torch.pow(2.0, pow2_exponent(raw)) if use_pow2 else raw)
    zp = _bf16_rt(mn)
    code = torch.round((gw - zp) / scale).clamp(0, 3).to(torch.int64)

    repr_l = str(outlier_repr).lower()
    if repr_l not in ("bitmap", "relidx7", "combinadic"):
        raise ValueError("outlier_repr must be bitmap, relidx7 or combinadic")
    planes: Dict[str, object] = {"k_oidx": None, "k_crank": None}
    if k > 0:
        if kv_outlier_map:                                  # pack.py:486-498
            omn, omx = _masked_min_max(gw, omask)
            center = _bf16_rt((omx + omn) / 2.0)
            # (scalar / tensor is reciprocal-then-multiply in torch: two roundings; written out so that
            # the oracle does not depend on how a torch version spells Tensor.__rtruediv__)
            mscale = _bf16_rt(torch.reciprocal((omx - omn).clamp_min(1e-8)) * 12.0)
            mapped = (gw - center) * mscale
        else:                                               # pack.py:502-506
            mapped = (gw - zp) / scale
        fpc = fp4_encode(mapped).to(torch.int64)
        cols = torch.arange(gt).expand_as(gw)
        pos = torch.where(omask, cols, torch.full_like(cols, gt)).sort(-1)[0][..., :k]
        if int(pos.max()) >= gt:
            # pack.py:515-538: the selector under-filled a vector (non-finite input)
            raise IndexError("outlier index out of range")
        oval = fpc.gather(-1, pos)
        pos = pos.permute(2, 0, 1, 3).contiguous()          # [G,H,D,k]
        oval = oval.permute(2, 0, 1, 3).contiguous()
        if repr_l == "bitmap":                              # pack.py:559-573
            planes["k_obmp"] = bitmap_pack(pos, gt)
        elif repr_l == "combinadic":                        # pack.py:552-557
            planes["k_obmp"] = None
            planes["k_crank"] = combinadic_pack(pos, gt)
        else:
            planes["k_obmp"] = None
            planes["k_oidx"] = relidx7_pack(pos)
        planes["k_oval"] = nibbles_pack(oval)
        if kv_outlier_map:
            planes["k_fp4_mapscale"] = mscale.squeeze(-1).permute(2, 0, 1).contiguous().to(torch.bfloat16)
            planes["k_fp4_mapcenter"] = center.squeeze(-1).permute(2, 0, 1).contiguous().to(torch.bfloat16)
        else:
            planes["k_fp4_mapscale"] = planes["k_fp4_mapcenter"] = None
    else:
        planes["k_obmp"] = planes["k_oval"] = None
        planes["k_fp4_mapscale"] = planes["k_fp4_mapcenter"] = None

    codes_tok = code.reshape(H, D, T).permute(2, 0, 1)                    # [T,H,D]
    planes["k_base"] = pack_int2(codes_tok).reshape(pages, page_size, H, D // 4).contiguous()
    scale_ghd = scale.squeeze(-1).permute(2, 0, 1).contiguous()
    planes["k_scale"] = pow2_exponent(scale_ghd).to(torch.int8) if int8_scale \
        else scale_ghd.to(torch.bfloat16)                                 # pack.py:586-590
    planes["k_zp"] = zp.squeeze(-1).permute(2, 0, 1).contiguous().to(torch.bfloat16)

    # ---- V, vector = (token, head, 32 channels)                         pack.py:604-623
    vfmt = str(v_format).lower()
    if vfmt not in ("i2", "bf16"):
        raise ValueError("v_format must be i2 or bf16")
    if vfmt == "bf16":                                                    # pack.py:596-602
        planes["v_main"] = V.to(torch.bfloat16).reshape(pages, page_size, H, D).contiguous()
        planes["v_scale"] = torch.ones(pages, page_size, H, NGV, dtype=torch.int8 if int8_scale else torch.bfloat16)
        planes["v_zp"] = torch.zeros(pages, page_size, H, NGV, dtype=torch.bfloat16)
        return _finish_planes(planes, locals())
    gv = Vf.reshape(T, H, NGV, gc)
    if not bool(torch.isfinite(gv).all()):
        raise ValueError("V pack: non-finite input")
    vmn = gv.min(-1, keepdim=True)[0]
    vmx = gv.max(-1, keepdim=True)[0]
    vraw = (vmx - vmn).clamp_min(1e-8) / 3.0
    vscale = _bf16_rt(torch.pow(2.0, pow2_exponent(vraw)) if use_pow2 else vraw)
    vzp = _bf16_rt(vmn)
    vcode = torch.round((gv - vzp) / vscale).clamp(0, 3).to(torch.int64)
    planes["v_main"] = pack_int2(vcode.reshape(T, H, D)).reshape(pages, page_size, H, D // 4).contiguous()
    vs_flat = vscale.squeeze(-1).reshape(pages, page_size, H, NGV).contiguous()
    planes["v_scale"] = pow2_exponent(vs_flat).to(torch.int8) if int8_scale else vs_flat.to(torch.bfloat16)
    planes["v_zp"] = vzp.squeeze(-1).to(torch.bfloat16).reshape(pages, page_size, H, NGV).contiguous()
    return _finish_planes(planes, locals())


def _finish_planes(planes: Dict[str, object], v: Dict[str, object]) -> Dict[str, object]:
    """Identity tables and the metadata keys of pack.py:628-654."""
    gt, k = v["gt"], v["k"]
    planes.update(
        k_field_bytes=((gt + 7) // 8 if v["repr_l"] == "bitmap" else
                       combinadic_bytes(k, gt) if v["repr_l"] == "combinadic" else 0) if k > 0 else 0,
        req_to_token=torch.arange(v["pages"], dtype=torch.int32).reshape(1, v["pages"]),
        req_to_group=torch.arange(v["G"], dtype=torch.int32).reshape(1, v["G"]),
        head_dim=v["D"], n_kv_heads=v["H"], num_tokens=v["T"], n_groups=v["G"], page_size=int(v["page_size"]),
        outliers_per_vector=k, outlier_repr=v["repr_l"], outlier_select=v["sel"],
        group_tokens=gt, group_channels=v["gc"], k_format="i2f4", v_format=v["vfmt"],
        k_base_bits=2, oval_bits=4, use_pow2=bool(v["use_pow2"]),
        kv_outlier_map=bool(v["kv_outlier_map"]) and k > 0, kv_int8_scale=v["int8_scale"])
    return planes


# ---------------------------------------------------------------------------------------
# dequant                                                             pack.py:701-781
# ---------------------------------------------------------------------------------------

def _steps(plane: torch.Tensor) -> torch.Tensor:
    """fp32 quantisation steps from a step plane: 2^e for an int8 exponent plane, the stored
    values for a bf16 plane.  pack.py:719-726, 770-776."""
    if plane.dtype == torch.int8:
        return torch.exp2(plane.to(torch.float32))
    return plane.to(torch.float32)


def dequant_kv(planes: Dict[str, object]) -> Tuple[torch.Tensor, torch.Tensor]:
    """Planes (slot-linear, tables ignored) -> fp32 ``(K, V)`` each ``[T, H, D]``.

    ``K = code * 2^e + zp`` with outlier lanes overwritten by
    ``level / map_scale + center``; ``V = code * 2^e + zp``.  pack.py:719-779.
    """
    k_base = planes["k_base"]
    P, ps, H, D4 = (int(s) for s in k_base.shape)
    T, D = P * ps, D4 * 4
    gt = int(planes.get("group_tokens", GROUP_TOKENS))
    gc = int(planes.get("group_channels", GROUP_CHANNELS))
    G = T // gt
    k = int(planes["outliers_per_vector"])
    code = unpack_int2(k_base.reshape(T, H, D4)).to(torch.float32)
    scale = _steps(planes["k_scale"])[:G]
    zp = planes["k_zp"].to(torch.float32)[:G]
    Kd = code * scale.repeat_interleave(gt, 0) + zp.repeat_interleave(gt, 0)
    if k > 0:
        pos = outlier_positions(planes, slice(0, G), k, gt)                  # [G,H,D,k]
        lvl = fp4_decode(nibbles_unpack(planes["k_oval"][:G], k))
        if planes.get("k_fp4_mapscale") is not None:                         # pack.py:749-755
            ms = planes["k_fp4_mapscale"].to(torch.float32)[:G].unsqueeze(-1)
            mc = planes["k_fp4_mapcenter"].to(torch.float32)[:G].unsqueeze(-1)
            dq = lvl / ms + mc
        else:                                                                # pack.py:756-757
            dq = lvl * scale.unsqueeze(-1) + zp.unsqueeze(-1)
        Kg = Kd.reshape(G, gt, H, D).permute(0, 2, 3, 1).contiguous()        # [G,H,D,gt]
        Kg.scatter_(-1, pos, dq)
        Kd = Kg.permute(0, 3, 1, 2).reshape(T, H, D)
    if planes["v_main"].dtype == torch.bfloat16:                             # pack.py:766-769
        return Kd, planes["v_main"].to(torch.float32).reshape(T, H, D)
    vcode = unpack_int2(planes["v_main"].reshape(T, H, D4)).to(torch.float32)
    NGV = D // gc
    vs = _steps(planes["v_scale"]).reshape(T, H, NGV, 1)
    vz = planes["v_zp"].to(torch.float32).reshape(T, H, NGV, 1)
    Vd = (vcode.reshape(T, H, NGV, gc) * vs + vz).reshape(T, H, D)
    return Kd, Vd


# ---------------------------------------------------------------------------------------
# window arithmetic                                                kv_window.py:35-141
# ---------------------------------------------------------------------------------------

def packed_boundary(seq_len: int, sink: int = 8, recent: int = 32, gt: int = GROUP_TOKENS) -> int:
    """End of the quantised prefix: ``sink + ((seq-sink-recent)//gt)*gt`` once the
    sequence is longer than sink+recent, else ``min(sink, seq)``.  kv_window.py:35-51."""
    extra = seq_len - sink - recent
    if extra <= 0:
        return min(sink, seq_len)
    return sink + (extra // gt) * gt


def tail_indices(seq_len: int, sink: int = 8, recent: int = 32, gt: int = GROUP_TOKENS):
    """bf16 rows = sink rows then ``[boundary, seq)``.  kv_window.py:80-92."""
    b = packed_boundary(seq_len, sink, recent, gt)
    return list(range(0, min(sink, seq_len))) + list(range(b, seq_len))


# ---------------------------------------------------------------------------------------
# attention                                oracle.py:33-49, paged_decode.py:1428-1432,
#                                          2262-2284, 2407-2410, 2483-2500
# ---------------------------------------------------------------------------------------

def attend(q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, sm_scale: float,
           dtype=torch.float32) -> Tuple[torch.Tensor, torch.Tensor]:
    """Textbook GQA attention of one query row set.  oracle.py:33-49.

    ``q [Hq, D]``; ``K, V [T, Hkv, D]``.  Returns ``(o [Hq, D], lse [Hq])`` in ``dtype``
    arithmetic; ``T == 0`` gives ``o = 0`` and ``lse = -inf`` (paged_decode.py:2262-2284).
    """
    Hq, D = int(q.shape[0]), int(q.shape[1])
    Hkv = int(K.shape[1])
    per = Hq // Hkv
    o = torch.zeros(Hq, D, dtype=dtype)
    lse = torch.full((Hq,), -math.inf, dtype=dtype)
    if int(K.shape[0]) == 0:
        return o, lse
    for h in range(Hq):
        kh = h // per
        s = (K[:, kh, :].to(dtype) @ q[h].to(dtype)) * sm_scale
        m = s.max()
        w = torch.exp(s - m)
        z = w.sum()
        o[h] = (w.unsqueeze(-1) * V[:, kh, :].to(dtype)).sum(0) / z
        lse[h] = m + torch.log(z)
    return o, lse


def merge_states(o_parts: torch.Tensor, lse_parts: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``o = sum w_p o_p / sum w_p``, ``lse = m + log sum w_p`` with
    ``w_p = exp(lse_p - m)``; parts with ``lse = -inf`` weigh nothing and an all-empty
    row gives ``o = 0``.  paged_decode.py:2483-2500, 3566-3567."""
    m = lse_parts.max(0)[0]
    m_safe = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    w = torch.exp(lse_parts - m_safe)
    w = torch.where(torch.isinf(lse_parts), torch.zeros_like(w), w)
    z = w.sum(0)
    z_safe = torch.where(z > 0, z, torch.ones_like(z))
    o = (w.unsqueeze(-1) * o_parts).sum(0) / z_safe.unsqueeze(-1)
    return o, m + torch.log(z)


def split_bounds(seq_len: int, num_splits: int, gt: int = GROUP_TOKENS):
    """Token ranges of the KV splits: ``per = ceil(ceil(L/S)/gt)*gt``, split s covers
    ``[s*per, min((s+1)*per, L))`` and is empty when that is void.
    paged_decode.py:1429-1432, 2407-2410."""
    per = -(-(-(-seq_len // num_splits)) // gt) * gt
    return [(s * per, min((s + 1) * per, seq_len)) for s in range(num_splits)]


def gather_request(planes: Dict[str, object], req_to_token: torch.Tensor,
                   req_to_group: torch.Tensor, seq_len: int, *, page_size: int,
                   packed_start_offset: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dequantised packed rows ``[seq_len, H, D]`` of ONE request read through its page and
    group-slot tables the way the decode kernel addresses them: packed token p lives in
    physical row ``req_to_token[(p+off)//ps]*ps + (p+off)%ps`` and uses group slot
    ``req_to_group[p//gt]``.  paged_decode.py:1668-1677."""
    gt = int(planes.get("group_tokens", GROUP_TOKENS))
    gc = int(planes.get("group_channels", GROUP_CHANNELS))
    k_base = planes["k_base"]
    P, ps, H, D4 = (int(s) for s in k_base.shape)
    assert ps == page_size
    D = D4 * 4
    L = int(seq_len)
    if L == 0:
        z = torch.zeros(0, H, D, dtype=torch.float32)
        return z, z.clone()
    p = torch.arange(L, dtype=torch.int64) + int(packed_start_offset)
    rows = req_to_token.to(torch.int64)[p // ps] * ps + p % ps
    gslot = req_to_group.to(torch.int64)[torch.arange(L, dtype=torch.int64) // gt]
    n_g = (L + gt - 1) // gt
    gs = req_to_group.to(torch.int64)[:n_g]
    code = unpack_int2(k_base.reshape(P * ps, H, D4)[rows]).to(torch.float32)
    scale = _steps(planes["k_scale"])[gslot]
    zp = planes["k_zp"].to(torch.float32)[gslot]
    Kd = code * scale + zp
    k = int(planes["outliers_per_vector"])
    if k > 0:
        Lp = n_g * gt
        pos = outlier_positions(planes, gs, k, gt)
        lvl = fp4_decode(nibbles_unpack(planes["k_oval"][gs], k))
        if planes.get("k_fp4_mapscale") is not None:
            ms = planes["k_fp4_mapscale"].to(torch.float32)[gs].unsqueeze(-1)
            mc = planes["k_fp4_mapcenter"].to(torch.float32)[gs].unsqueeze(-1)
            dq = lvl / ms + mc
        else:
            gsc = _steps(planes["k_scale"])[gs].unsqueeze(-1)
            dq = lvl * gsc + planes["k_zp"].to(torch.float32)[gs].unsqueeze(-1)
        Kp = torch.zeros(Lp, H, D, dtype=torch.float32)
        Kp[:L] = Kd
        Kg = Kp.reshape(n_g, gt, H, D).permute(0, 2, 3, 1).contiguous()
        Kg.scatter_(-1, pos, dq)
        Kd = Kg.permute(0, 3, 1, 2).reshape(Lp, H, D)[:L]
    if planes["v_main"].dtype == torch.bfloat16:
        return Kd, planes["v_main"].reshape(P * ps, H, D)[rows].to(torch.float32)
    vcode = unpack_int2(planes["v_main"].reshape(P * ps, H, D4)[rows]).to(torch.float32)
    NGV = D // gc
    vs = _steps(planes["v_scale"].reshape(P * ps, H, NGV)[rows]).unsqueeze(-1)
    vz = planes["v_zp"].reshape(P * ps, H, NGV)[rows].to(torch.float32).unsqueeze(-1)
    Vd = (vcode.reshape(L, H, NGV, gc) * vs + vz).reshape(L, H, D)
    return Kd, Vd


def decode_reference(q: torch.Tensor, planes: Dict[str, object], k_tail: torch.Tensor,
                     v_tail: torch.Tensor, b_tail_len: Sequence[int],
                     req_to_token: torch.Tensor, req_to_group: torch.Tensor,
                     b_seq_len: Sequence[int], *, sm_scale: float, page_size: int = 16,
                     packed_start_offset: int = 0, dtype=torch.float64
                     ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dequantise-then-attend result of the decode operator for a batch.

    Attended set of request b = its ``b_seq_len[b]`` packed tokens (through the tables)
    plus the first ``b_tail_len[b]`` bf16 tail rows; order is irrelevant
    (paged_decode.py:2308-2312).  Returns ``o [B, Hq, D]`` and ``lse [B, Hq]``.
    """
    B, Hq, D = (int(s) for s in q.shape)
    o = torch.zeros(B, Hq, D, dtype=dtype)
    lse = torch.zeros(B, Hq, dtype=dtype)
    for b in range(B):
        Kd, Vd = gather_request(planes, req_to_token[b], req_to_group[b], int(b_seq_len[b]),
                                page_size=page_size, packed_start_offset=packed_start_offset)
        tl = int(b_tail_len[b])
        Kf = torch.cat([Kd, k_tail[b, :tl].to(torch.float32)])
        Vf = torch.cat([Vd, v_tail[b, :tl].to(torch.float32)])
        o[b], lse[b] = attend(q[b], Kf, Vf, sm_scale, dtype=dtype)
    return o, lse


def plane_bytes_per_token_head(D: int = 128, k: int = 6) -> float:
    """Bytes of packed planes per (token, kv head): k_base D/4 + v_main D/4 + v_scale D/32
    + v_zp 2*D/32 per token, plus per 32-token group D*(1 + 2 + 2 + 2 + 4 + ceil(k/2))
    bytes of k_scale, k_zp, map scale, map centre, bitmap, nibbles.  132 at D=128, k=6.
    integration/vllm/packed_only.py:352-388."""
    per_tok = D // 4 + D // 4 + D // 32 + 2 * (D // 32)
    per_grp = D * (1 + 2 + 2 + 2 + 4 + (k + 1) // 2)
    return per_tok + per_grp / GROUP_TOKENS
