"""Quantize-on-store for the OMMX KV cache: host side of the HIP store kernel.

``ommx_pack_kv_canonical_block`` keeps the signature, plane dictionary and error behaviour of
the reference packer (``ommx_gpu_serve/attention/pack.py:293-655``); the arithmetic runs in
``ommx_store_pack`` (``csrc/ommx_store.hip``).  ``store_pack_into`` is the same kernel writing
straight into the page / group slots of caller-owned pool planes, the placement the
reference does with a pack followed by indexed copies (``attention/kv_pool.py:552-735``).

Only the serving recipe is implemented on the device: ``k_format="i2f4"``, signed outlier
selection, the flat-bitmask index plane, power-of-two scales stored as int8 exponents, the
dedicated FP4 outlier map, 32-token K vectors, 32-channel V vectors, bf16 side planes.
Other recipes raise ``NotImplementedError``.
"""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from . import _hip

CANONICAL_GROUP_TOKENS = 32
CANONICAL_GROUP_CHANNELS = 32
OUTLIER_REPRS = ("relidx7", "combinadic", "bitmap")

_FP4_MAGNITUDES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
_table_host: Optional[torch.Tensor] = None
_table_dev: Dict[str, torch.Tensor] = {}


# -- decision tables ----------------------------------------------------------------------

def _ulp_window(center: torch.Tensor, half: int) -> torch.Tensor:
    """fp32 neighbours of ``center`` (shape [n]) from -half to +half ulps -> [n, 2*half+1]."""
    steps = torch.arange(-half, half + 1, dtype=torch.int32)
    return (center.view(torch.int32).unsqueeze(-1) + steps).view(torch.float32)


def _first_true_monotone(flags: torch.Tensor, what: str) -> torch.Tensor:
    """Index of the first True of each row; every row must be False...False True...True."""
    first = flags.to(torch.int8).argmax(-1)
    cols = torch.arange(flags.shape[-1]).expand_as(flags)
    if not bool(((cols >= first.unsqueeze(-1)) == flags).all()) or not bool(flags[:, -1].all()) \
            or bool(flags[:, 0].any()):
        raise RuntimeError(f"{what}: this libm's rounding is not a single threshold per interval")
    return first


def measure_store_table() -> torch.Tensor:
    """The store kernel's decision table measured from this machine's torch-CPU routines.

    The packer's power-of-two exponent is ``round(log2(x))`` in fp32 and its FP4 level is an
    ``argmin`` over fp32 ``log`` distances (reference ``pack.py:462`` and ``codec.py:58-62``);
    both are step functions of ``x`` whose steps sit within a few ulps of ``sqrt(2)*2^k`` and
    of the geometric means of neighbouring levels, on whichever side the library's last-bit
    rounding puts them.  Scanning those few ulps with the very same torch expressions gives
    thresholds the kernel can compare against, so device and host agree bit for bit.
    """
    lib = _hip.load()
    table = torch.zeros(_hip.STORE_TABLE_FLOATS, dtype=torch.float32)
    lib.ommx_store_default_table(table.data_ptr())
    half = 64
    # pow2 exponents that a clamped scale can take: 1e-12 <= x < 2^127
    kbs = torch.arange(127 - 39, 254, dtype=torch.int64)
    win = _ulp_window(table[kbs].clone(), half)
    got = torch.round(torch.log2(win.clamp_min(1e-12)))
    up = got >= (kbs - 127 + 1).to(torch.float32).unsqueeze(-1)
    first = _first_true_monotone(up, "log2")
    table[kbs] = win.gather(-1, first.unsqueeze(-1)).squeeze(-1)
    # FP4 level boundaries
    lv = torch.tensor(_FP4_MAGNITUDES, dtype=torch.float32)
    loglv = torch.log(lv.clamp_min(1e-8))
    win = _ulp_window(table[257:264].clone(), half)
    idx = (torch.log(win.clamp_min(1e-8)).unsqueeze(-1) - loglv).abs().argmin(-1)
    up = idx >= torch.arange(1, 8).unsqueeze(-1)
    first = _first_true_monotone(up, "log")
    table[257:264] = win.gather(-1, first.unsqueeze(-1)).squeeze(-1)
    # the kernels walk down the FP4 boundaries by halves, which takes them in ascending order
    if not bool((table[257:264].diff() > 0).all()):
        raise RuntimeError("measured FP4 level boundaries are not ascending")
    return table


def store_table(device: torch.device) -> torch.Tensor:
    """Device copy of the decision table (measured once per process, cached per device)."""
    global _table_host
    if _table_host is None:
        _table_host = measure_store_table()
    device = torch.device(device)
    if device.type == "cuda" and device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    key = str(device)
    if key not in _table_dev:
        _table_dev[key] = _table_host.to(device)    # first use on a device uploads (not capturable)
    return _table_dev[key]


# -- launch -------------------------------------------------------------------------------

def _check_rows(name: str, t: torch.Tensor) -> None:
    if t.dim() != 3:
        raise ValueError(f"{name} must be [num_tokens, n_kv_heads, head_dim]; got {tuple(t.shape)}")
    if t.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"{name} must be bf16 or fp32; got {t.dtype}")
    if t.stride(-1) != 1:
        raise ValueError(f"{name} must be contiguous along head_dim")


def store_pack_into(K: torch.Tensor, V: torch.Tensor, planes: Dict[str, Any], *,
                    outliers_per_vector: int = 6, page_size: int = 16,
                    src_rows: Optional[torch.Tensor] = None,
                    dst_pages: Optional[torch.Tensor] = None,
                    dst_groups: Optional[torch.Tensor] = None,
                    err_flag: Optional[torch.Tensor] = None,
                    num_tokens: Optional[int] = None,
                    outlier_repr: str = "bitmap", outlier_select: str = "signed",
                    use_pow2: bool = True, kv_int8_scale: bool = True,
                    group_tokens: int = 32, group_channels: int = 32, v_format: str = "i2") -> None:
    """Pack ``num_tokens`` (default: all rows) tokens of ``K``/``V`` into ``planes`` in place.

    ``src_rows`` int32[T] picks the source row of each packed token (a ring gather);
    ``dst_pages`` int32[T/page_size] and ``dst_groups`` int32[T/32] give the physical page
    and group slot of each logical page / group (identity when ``None``).  No host
    synchronisation happens here: non-finite input or an under-filled outlier set is
    reported by bits OR-ed into ``err_flag`` (int32[1]), which the caller reads when it
    can afford to.  Launches on the current stream.  ``outlier_repr`` names the index plane
    that is written: ``planes["k_obmp"]`` (``"bitmap"``) or ``planes["k_oidx"]`` (``"relidx7"``).
    """
    _check_rows("K", K)
    _check_rows("V", V)
    if K.dtype != V.dtype or K.device != V.device:
        raise ValueError("K and V must share dtype and device")
    _hip.require_gpu(K.device)
    H, D = int(K.shape[1]), int(K.shape[2])
    T = int(num_tokens) if num_tokens is not None else (
        int(src_rows.numel()) if src_rows is not None else int(K.shape[0]))
    gt, gc = int(group_tokens), int(group_channels)
    for t, n in ((src_rows, T), (dst_pages, T // max(1, page_size)), (dst_groups, T // max(1, gt))):
        if t is not None and (t.dtype != torch.int32 or not t.is_contiguous()
                              or int(t.numel()) < n or t.device != K.device):
            raise ValueError("index tables must be contiguous int32 device tensors of the right length")
    k = int(outliers_per_vector)
    combinadic = k > 0 and str(outlier_repr).lower() == "combinadic"
    if combinadic:
        # the store kernel writes the flat bitmask into a scratch plane kept beside k_crank;
        # the ranks of the groups just written come from one conversion launch after it
        crank = planes.get("k_crank")
        fb = index_plane_bytes("combinadic", gt, k)
        if crank is None or int(crank.shape[-1]) != fb:
            raise ValueError(f"combinadic needs a k_crank plane of {fb} bytes per frame")
        scratch = planes.get("_k_obmp_scratch")
        if scratch is None or tuple(scratch.shape[:3]) != tuple(crank.shape[:3]):
            scratch = torch.zeros(*crank.shape[:3], (gt + 7) // 8, dtype=torch.uint8, device=crank.device)
            planes["_k_obmp_scratch"] = scratch
        index_repr, index_plane = _hip.INDEX_BITMAP, scratch
    else:
        index_repr, index_plane = _index_plane(planes, outlier_repr, k, gt)
    sel = str(outlier_select).lower()
    if sel not in ("signed", "abs"):
        raise ValueError(f"outlier_select must be signed|abs; got {outlier_select!r}")
    v_bf16 = str(v_format).lower() == "bf16"
    if (planes["v_main"].dtype == torch.bfloat16) != v_bf16:
        raise ValueError("v_main must be bf16 [pages, page_size, H, D] for v_format='bf16', else uint8 codes")
    mode = _hip.scale_mode(bool(use_pow2), bool(kv_int8_scale))
    want_dt = torch.int8 if mode == _hip.SCALE_POW2_INT8 else torch.bfloat16
    if planes["k_scale"].dtype != want_dt or planes["v_scale"].dtype != want_dt:
        raise ValueError(f"k_scale / v_scale planes must be {want_dt} for this recipe")
    lib = _hip.load()
    with torch.cuda.device(K.device):
        rc = lib.ommx_store_pack(
            K.data_ptr(), V.data_ptr(), 1 if K.dtype == torch.float32 else 0,
            K.stride(0), K.stride(1), V.stride(0), V.stride(1),
            _hip.ptr(src_rows), T, H, D, int(page_size), k, index_repr, 1 if sel == "abs" else 0, mode,
            gt, gc, 1 if v_bf16 else 0, _hip.ptr(dst_pages), _hip.ptr(dst_groups), store_table(K.device).data_ptr(),
            planes["k_base"].data_ptr(), planes["k_scale"].data_ptr(), planes["k_zp"].data_ptr(),
            _hip.ptr(planes.get("k_fp4_mapscale")), _hip.ptr(planes.get("k_fp4_mapcenter")),
            _hip.ptr(index_plane), _hip.ptr(planes.get("k_oval")),
            planes["v_main"].data_ptr(), planes["v_scale"].data_ptr(), planes["v_zp"].data_ptr(),
            _hip.ptr(err_flag), _hip.current_stream_ptr(K.device))
    _hip.check(rc, "ommx_store_pack")
    if combinadic and T >= gt:
        convert_index_plane(index_plane, planes["k_crank"], group_tokens=gt, k=k, src_repr="bitmap",
                            dst_repr="combinadic", groups=dst_groups, n_groups=T // gt, err_flag=err_flag)


_REPR_CODE = {"bitmap": _hip.INDEX_BITMAP, "relidx7": _hip.INDEX_RELIDX7, "combinadic": _hip.INDEX_COMBINADIC}


def index_plane_bytes(outlier_repr: str, group_tokens: int, k: int) -> int:
    """Bytes per K vector of an index plane: ``group_tokens/8`` (bitmap), ``ceil(7k/8)`` (relidx7),
    ``ceil(log2 C(group_tokens, k) / 8)`` (combinadic; reference ``codec.py:131-143``).  Raises
    ``NotImplementedError`` for what the library does not convert (more than 16 outliers, ranks
    wider than 64 bits)."""
    if int(k) <= 0:
        return 0
    n = _hip.load().ommx_index_plane_bytes(_REPR_CODE[str(outlier_repr).lower()], int(group_tokens), int(k))
    if n <= 0:
        raise NotImplementedError(f"index plane {outlier_repr!r} with group_tokens={group_tokens}, k={k}")
    return int(n)


def convert_index_plane(src: torch.Tensor, dst: torch.Tensor, *, group_tokens: int, k: int,
                        src_repr: str, dst_repr: str, groups: Optional[torch.Tensor] = None,
                        n_groups: Optional[int] = None, err_flag: Optional[torch.Tensor] = None) -> None:
    """Rewrite the outlier index plane ``src [slots, H, D, bytes]`` in another encoding into
    ``dst`` (same slots), one launch on the current stream; ``groups`` int32 names the slots to
    convert (default: the first ``n_groups``, default all).  A vector that does not hold exactly
    ``k`` positions sets ``ERR_INDEX_PLANE`` in ``err_flag`` and is written as zeros."""
    gt, k = int(group_tokens), int(k)
    sb, db = index_plane_bytes(src_repr, gt, k), index_plane_bytes(dst_repr, gt, k)
    for name, t, nb in (("src", src, sb), ("dst", dst, db)):
        if t.dtype != torch.uint8 or t.dim() != 4 or int(t.shape[-1]) != nb or not t.is_contiguous():
            raise ValueError(f"{name} index plane must be contiguous u8 [slots, H, D, {nb}]")
    if tuple(src.shape[:3]) != tuple(dst.shape[:3]) or src.device != dst.device:
        raise ValueError("src and dst index planes must cover the same slots on one device")
    _hip.require_gpu(src.device)
    if groups is not None:
        if groups.dtype != torch.int32 or not groups.is_contiguous() or groups.device != src.device:
            raise ValueError("groups must be a contiguous int32 device tensor")
        n = int(groups.numel()) if n_groups is None else int(n_groups)
        if n > int(groups.numel()):
            raise ValueError("n_groups exceeds the slot list")
    else:
        n = int(src.shape[0]) if n_groups is None else int(n_groups)
        if n > int(src.shape[0]):
            raise ValueError("n_groups exceeds the plane")
    with torch.cuda.device(src.device):
        rc = _hip.load().ommx_index_convert(
            src.data_ptr(), dst.data_ptr(), _hip.ptr(groups), n, int(src.shape[1]) * int(src.shape[2]),
            gt, k, _REPR_CODE[str(src_repr).lower()], _REPR_CODE[str(dst_repr).lower()],
            _hip.ptr(err_flag), _hip.current_stream_ptr(src.device))
    _hip.check(rc, "ommx_index_convert")


def _derive(planes: dict, dst_repr: str) -> dict:
    if str(planes.get("outlier_repr")) != "combinadic" or planes.get("k_crank") is None:
        return planes
    k, gt = int(planes["outliers_per_vector"]), int(planes.get("group_tokens", 32))
    crank = planes["k_crank"]
    dev = crank.device if crank.device.type == "cuda" else torch.device("cuda", torch.cuda.current_device())
    src = crank.to(dev).contiguous()
    dst = torch.empty(*src.shape[:3], index_plane_bytes(dst_repr, gt, k), dtype=torch.uint8, device=dev)
    err = torch.zeros(1, dtype=torch.int32, device=dev)
    convert_index_plane(src, dst, group_tokens=gt, k=k, src_repr="combinadic", dst_repr=dst_repr, err_flag=err)
    if int(err.item()) & _hip.ERR_INDEX_PLANE:
        raise ValueError(f"invalid combinadic rank for k={k}, tile={gt}")          # codec.py:173-178
    out = dict(planes)
    out["k_oidx" if dst_repr == "relidx7" else "k_obmp"] = dst.to(crank.device)
    out["outlier_repr"] = dst_repr
    out["k_field_bytes"] = int(dst.shape[-1]) if dst_repr == "bitmap" else 0
    out["outlier_repr_storage"] = "combinadic"
    return out


def derive_relidx7_from_combinadic(planes: dict) -> dict:
    """Combinadic-stored outliers -> a new pack dict with the position-stream plane ``k_oidx`` the
    decode kernels read; ``k_crank`` stays as the stored form (reference ``pack.py:662-699``, which
    unranks on the host).  A pack with another index plane is returned unchanged."""
    return _derive(planes, "relidx7")


def derive_bitmap_from_combinadic(planes: dict) -> dict:
    """Same, to the flat bitmask plane ``k_obmp``."""
    return _derive(planes, "bitmap")


def _index_plane(planes: Dict[str, Any], outlier_repr: str, k: int, gt: int = 32):
    """(index_repr code of the C ABI, index plane tensor) for an ``outlier_repr`` name."""
    repr_l = str(outlier_repr).lower()
    if repr_l == "bitmap":
        t = planes.get("k_obmp")
        if k > 0 and (t is None or int(t.shape[-1]) != (gt + 7) // 8):
            raise ValueError("bitmap needs a k_obmp plane of group_tokens/8 bytes per frame")
        return _hip.INDEX_BITMAP, t
    if repr_l == "relidx7":
        t = planes.get("k_oidx")
        if k > 0 and (t is None or int(t.shape[-1]) != (7 * k + 7) // 8):
            raise ValueError("relidx7 needs a k_oidx plane of ceil(7k/8) bytes per frame")
        return _hip.INDEX_RELIDX7, t
    raise NotImplementedError(f"outlier_repr={outlier_repr!r} has no HIP kernel")


def alloc_planes(num_pages: int, num_group_slots: int, n_kv_heads: int, head_dim: int, *,
                 page_size: int = 16, outliers_per_vector: int = 6,
                 device: Any = "cuda", outlier_repr: str = "bitmap",
                 kv_outlier_map: bool = True, int8_scale: bool = True,
                 group_tokens: int = 32, group_channels: int = 32, v_format: str = "i2") -> Dict[str, Any]:
    """Empty planes with the shapes and dtypes of reference ``pack.py:576-623``;
    ``num_group_slots`` counts K groups of ``group_tokens`` tokens."""
    P, G, H, D, ps, k = num_pages, num_group_slots, n_kv_heads, head_dim, page_size, outliers_per_vector
    dev = torch.device(device)
    u8, bf = torch.uint8, torch.bfloat16
    i8 = torch.int8 if int8_scale else torch.bfloat16       # dtype of the two step planes (pack.py:586-590)
    out: Dict[str, Any] = {
        "k_base": torch.empty(P, ps, H, D // 4, dtype=u8, device=dev),
        "k_scale": torch.empty(G, H, D, dtype=i8, device=dev),
        "k_zp": torch.empty(G, H, D, dtype=bf, device=dev),
        "v_main": (torch.empty(P, ps, H, D, dtype=bf, device=dev) if str(v_format).lower() == "bf16"
                   else torch.empty(P, ps, H, D // 4, dtype=u8, device=dev)),     # pack.py:596-598
        "v_scale": torch.empty(P, ps, H, D // int(group_channels), dtype=i8, device=dev),
        "v_zp": torch.empty(P, ps, H, D // int(group_channels), dtype=bf, device=dev),
        "k_oidx": None, "k_crank": None,
        "k_obmp": None, "k_oval": None, "k_fp4_mapscale": None, "k_fp4_mapcenter": None,
    }
    if k > 0:
        if str(outlier_repr).lower() == "relidx7":      # pack.py:128-164: ceil(7k/8) bytes per frame
            out["k_oidx"] = torch.empty(G, H, D, (7 * k + 7) // 8, dtype=u8, device=dev)
        elif str(outlier_repr).lower() == "combinadic":  # pack.py:552-557: one rank per frame
            out["k_crank"] = torch.empty(G, H, D, index_plane_bytes("combinadic", int(group_tokens), k),
                                         dtype=u8, device=dev)
        else:
            out["k_obmp"] = torch.empty(G, H, D, (int(group_tokens) + 7) // 8, dtype=u8, device=dev)
        out["k_oval"] = torch.empty(G, H, D, (k + 1) // 2, dtype=u8, device=dev)
        if kv_outlier_map:       # base-shared outliers carry no map planes (pack.py:502-506)
            out["k_fp4_mapscale"] = torch.empty(G, H, D, dtype=bf, device=dev)
            out["k_fp4_mapcenter"] = torch.empty(G, H, D, dtype=bf, device=dev)
    return out


def raise_for_store_errors(bits: int) -> None:
    """Turn the device error bits into the exceptions the reference packer raises."""
    if bits & _hip.ERR_NONFINITE_V:
        raise ValueError("V pack: non-finite input (NaN/inf)")               # pack.py:605-607
    if bits & _hip.ERR_UNDERFILLED:
        raise IndexError("OMMX KV pack: the outlier selector chose fewer than k distinct "
                         "positions in some group (non-finite or out-of-range K)")  # pack.py:520-538
    if bits & _hip.ERR_NONFINITE_K:
        raise ValueError("encode_fp4_e2m1f: non-finite input")               # codec.py:55-57
    if bits & _hip.ERR_EXP_RANGE:
        raise ValueError("KV pack: a scale exponent does not fit the int8 plane")
    if bits & _hip.ERR_INDEX_PLANE:
        raise ValueError("outlier index plane: a vector does not name exactly k positions")


def ommx_pack_kv_canonical_block(
    K, V, *,
    outliers_per_vector: int = 3,
    scale_dtype: Any = None,
    page_size: int = 16,
    device: Any = None,
    outlier_repr: str = "relidx7",
    outlier_select: str = "abs",
    k_format: str = "i2f4",
    use_pow2: bool = False,
    kv_outlier_map: Any = None,
    kv_int8_scale: Any = None,
    group_tokens: int = CANONICAL_GROUP_TOKENS,
    group_channels: int = CANONICAL_GROUP_CHANNELS,
    v_format: str = "i2",
):
    """Pack a ``[num_tokens, n_kv_heads, head_dim]`` K/V block into the canonical planes.

    Same keywords, defaults, returned keys and exceptions as the reference
    (``pack.py:293-309, 367-417, 628-654``).  The block is packed on the GPU (``K``'s
    device if it is one, else the current GPU); the planes are returned on ``device``
    (default ``"cpu"`` like the reference).  Recipes other than the serving one raise
    ``NotImplementedError`` after the reference's own argument checks.
    """
    if device is None:
        device = "cpu"
    if scale_dtype is None:
        scale_dtype = torch.bfloat16
    repr_l = str(outlier_repr).lower()
    if repr_l not in OUTLIER_REPRS:
        raise ValueError(f"outlier_repr must be one of {OUTLIER_REPRS}; got {outlier_repr!r}")
    kfmt = str(k_format).lower()
    if kfmt not in ("i2f4", "itf4"):
        raise ValueError(f"k_format must be i2f4|itf4; got {k_format!r}")
    if kv_outlier_map is None:
        kv_outlier_map = True
    if kv_int8_scale is None:
        kv_int8_scale = True
    T, H, D = (int(s) for s in K.shape)
    if tuple(V.shape) != (T, H, D):
        raise ValueError(f"K/V shape mismatch: {tuple(K.shape)} vs {tuple(V.shape)}")
    gt, gc = int(group_tokens), int(group_channels)
    if gt not in (16, 32, 64, 128):
        raise ValueError(f"group_tokens (K vector_length) must be in {{16,32,64,128}}; got {gt}")
    if gc not in (16, 32, 64, 128):
        raise ValueError(f"group_channels (V vector_length) must be in {{16,32,64,128}}; got {gc}")
    if T % gt != 0 or T % int(page_size) != 0:
        raise ValueError(f"num_tokens={T} must be a multiple of {gt} and page_size")
    if D % gc != 0 or D % 4 != 0:
        raise ValueError(f"head_dim={D} must be a multiple of {gc}")
    k = int(outliers_per_vector)
    if k < 0 or k > gt:
        raise ValueError(f"outliers_per_vector={k} out of range [0, {gt}]")
    vfmt = str(v_format).lower()
    if vfmt not in ("i2", "bf16"):
        raise ValueError(f"v_format must be i2|bf16; got {v_format!r}")

    unsupported = []
    if 0 < k <= 16 and repr_l == "combinadic" and \
            _hip.load().ommx_index_plane_bytes(_hip.INDEX_COMBINADIC, gt, k) <= 0:
        unsupported.append(f"combinadic ranks wider than 64 bits (group_tokens={gt}, k={k})")
    if str(outlier_select).lower() not in ("signed", "abs"):
        unsupported.append(f"outlier_select={outlier_select!r}")
    if k > 16:
        unsupported.append("more than 16 outliers per vector")
    if scale_dtype != torch.bfloat16:
        unsupported.append(f"scale_dtype={scale_dtype}")
    if D > 256 or D % 32 != 0:
        unsupported.append("head_dim above 256 or not a multiple of 32")
    if unsupported:
        raise NotImplementedError(
            "the HIP store kernel implements the serving recipe only; not: " + ", ".join(unsupported))

    if K.device.type == "cuda":
        dev = K.device
    else:
        if not torch.cuda.is_available():
            raise RuntimeError("ommx_pack_kv_canonical_block needs a ROCm GPU (no CPU fallback)")
        dev = torch.device("cuda", torch.cuda.current_device())
    Kd = K.to(dev)
    Vd = V.to(dev)
    if Kd.dtype not in (torch.bfloat16, torch.float32):
        Kd = Kd.to(torch.float32)
    Vd = Vd.to(Kd.dtype)
    if Kd.stride(-1) != 1:
        Kd = Kd.contiguous()
    if Vd.stride(-1) != 1:
        Vd = Vd.contiguous()
    G, pages = T // gt, T // int(page_size)
    planes = alloc_planes(pages, G, H, D, page_size=int(page_size), outliers_per_vector=k, device=dev,
                          outlier_repr=repr_l, kv_outlier_map=bool(kv_outlier_map),
                          int8_scale=bool(use_pow2) and bool(kv_int8_scale),
                          group_tokens=gt, group_channels=gc, v_format=vfmt)
    err = torch.zeros(1, dtype=torch.int32, device=dev)
    if T > 0:
        store_pack_into(Kd, Vd, planes, outliers_per_vector=k, page_size=int(page_size), err_flag=err,
                        outlier_repr=repr_l, outlier_select=outlier_select,
                        use_pow2=bool(use_pow2), kv_int8_scale=bool(kv_int8_scale),
                        group_tokens=gt, group_channels=gc, v_format=vfmt)
    raise_for_store_errors(int(err.item()))

    def _to(t):
        return t.to(device) if t is not None else None

    out = {name: _to(planes[name]) for name in (
        "k_base", "k_scale", "k_zp", "k_oidx", "k_oval", "k_crank", "k_obmp",
        "k_fp4_mapscale", "k_fp4_mapcenter")}
    out["k_field_bytes"] = 0                                                      # pack.py:468,557,568
    if k > 0 and repr_l == "bitmap":
        out["k_field_bytes"] = (gt + 7) // 8
    elif k > 0 and repr_l == "combinadic":
        out["k_field_bytes"] = int(planes["k_crank"].shape[-1])
    out.update({name: _to(planes[name]) for name in ("v_main", "v_scale", "v_zp")})
    out.update(
        req_to_token=torch.arange(pages, dtype=torch.int32, device=device).reshape(1, pages),
        req_to_group=torch.arange(G, dtype=torch.int32, device=device).reshape(1, G),
        head_dim=D, n_kv_heads=H, num_tokens=T, n_groups=G, page_size=int(page_size),
        outliers_per_vector=k, outlier_repr=repr_l, outlier_select=str(outlier_select).lower(),
        group_tokens=gt, group_channels=gc, k_format=kfmt, v_format=vfmt,
        k_base_bits=2, oval_bits=4, use_pow2=bool(use_pow2),
        kv_outlier_map=bool(kv_outlier_map and k > 0),
        kv_int8_scale=bool(use_pow2) and bool(kv_int8_scale))
    return out


__all__ = ["CANONICAL_GROUP_TOKENS", "CANONICAL_GROUP_CHANNELS", "OUTLIER_REPRS",
           "ommx_pack_kv_canonical_block", "store_pack_into", "alloc_planes",
           "measure_store_table", "store_table", "raise_for_store_errors", "index_plane_bytes",
           "convert_index_plane", "derive_relidx7_from_combinadic", "derive_bitmap_from_combinadic"]
