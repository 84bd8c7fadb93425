"""OMMX paged decode attention: host launcher of the HIP split-KV and combine kernels.

``ommx_paged_decode_attention_canonical`` keeps the positional and keyword signature of the
reference launcher (``ommx_gpu_serve/attention/paged_decode.py:2768-2798``), its argument
checks and exception types (``:2916-3064``, ``:3323-3325``), the workspace shape
``[B, Hq, splits+1, D+1]`` (``:247-253``) and the split rounding (``:1429-1432``).  It
writes ``o`` and ``lse`` in place on the current stream, allocates nothing when
``attn_logits`` is passed, and never synchronises when ``max_seq_len`` is passed.

Implemented on the device: INT2 base with 0..16 FP4 outliers per vector behind any of the three
index planes (bitmap, 7-bit position stream, combinadic rank), dedicated or base-shared outlier
map, int8 exponent or bf16 step planes, 16/32/64/128-element vectors, INT2 or bf16 V.  The
serving recipe (bitmap, 6 outliers, dedicated map, int8 exponents, 32/32 vectors, INT2 V) takes
the fastest kernel; the library picks per call.  The reference's environment knobs are not read; ``num_stages`` / ``num_warps`` / ``qzp_buf`` are accepted
and ignored (they tune Triton, not this kernel).
"""
from __future__ import annotations

from typing import Any, Optional

import torch

from . import _hip

_CU_COUNT = {}


def _cu_count(device: torch.device) -> int:
    key = str(device)
    if key not in _CU_COUNT:
        _CU_COUNT[key] = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return _CU_COUNT[key]


MAX_KV_SPLITS = 512


def auto_num_kv_splits(max_seq_len: int, batch: int, kv_heads: int, n_cu: int = 256,
                       q_per_kv: int = 4, group_tokens: int = 32,
                       mean_seq_len: Optional[float] = None, resident: int = 2) -> int:
    """Split count for one decode call.  A workgroup is four waves of one split (a wave covers one
    kv head and all of its q heads, so ``q_per_kv`` does not enter); ``resident`` workgroups fit a
    compute unit at a time (3 for the serving-recipe kernel with up to 4 q heads per kv head, 2
    otherwise).  Requests about equally long (``mean_seq_len`` at least 0.9 of the longest) get one
    round of workgroups: little is left to even out, and a second round mostly pays the start-up of
    a workgroup (about one step) again.  Requests of different length get two rounds, so that they
    even out, and four when a workgroup would otherwise run for more than sixteen steps.  Never
    less than one 64-token step per split (one 32-token group when even that leaves units idle): a
    wave's time is a fixed part plus a few microseconds per step, so while compute units are idle
    more splits are faster.  The kernel with ``resident`` 3 deals whole groups out evenly by itself;
    for the others the count is chosen so that their rounding leaves no split empty.  At most 512,
    the number of partial states the combine kernel keeps on chip.  Splits are whole K groups
    (``group_tokens``), so longer groups mean coarser steps."""
    wgs_per_split = max(1, int(batch) * max(1, int(kv_heads) // 4))
    gt = max(32, int(group_tokens))
    step_tokens = max(64, gt)
    steps = max(1, (int(max_seq_len) + step_tokens - 1) // step_tokens)
    groups = max(1, (int(max_seq_len) + gt - 1) // gt)
    equal = int(batch) == 1 or (mean_seq_len is not None and float(mean_seq_len) >= 0.9 * float(max_seq_len))
    rounds = 1 if equal else 2

    def count(res: int) -> int:
        want = max(1, min(MAX_KV_SPLITS, (rounds * res * int(n_cu)) // wgs_per_split))
        if not equal and int(batch) > 1 and (steps + min(want, steps) - 1) // min(want, steps) > 16:
            # long splits of requests of different length: four rounds even out better (3-6 % on
            # 96-128 requests of 1K..16K tokens), the start-up they add is small against 16 steps
            want = max(1, min(MAX_KV_SPLITS, (4 * res * int(n_cu)) // wgs_per_split))
        return want

    res = max(1, int(resident))
    want = count(res)
    if res >= 3 and steps < 4 * want:
        # a third resident workgroup pays only while every wave keeps four steps or more: below that
        # the start-up of the extra waves costs more than their overlap returns (one request of 64K
        # tokens: 27.7 us with 256 splits of four steps, 28.9 us with 384 of fewer than three)
        res = 2
        want = count(res)
    if want >= 2 * steps:          # plenty of idle units: splits of one K group
        return int(min(want, groups))
    if res >= 3:
        # the kernel deals the groups out evenly whatever the count: fill the chip
        return int(max(1, min(want, groups)))
    target = max(1, min(want, steps))
    # equal whole steps per split, no empty split: the slowest wave sets the kernel's time
    steps_per_split = (steps + target - 1) // target
    return int((steps + steps_per_split - 1) // steps_per_split)


def make_attn_logits(batch: int, q_heads: int, num_kv_splits: int, head_dim: int, device) -> torch.Tensor:
    """fp32 workspace ``[B, Hq, splits + 1, D + 1]`` (reference ``paged_decode.py:247-253, 3220-3222``)."""
    return torch.empty(batch, q_heads, num_kv_splits + 1, head_dim + 1,
                       dtype=torch.float32, device=device)


def ommx_paged_decode_attention_canonical(
    q,
    k_base, k_scale, k_zp, k_oidx, k_oval,
    v_main, v_scale, v_zp,
    k_tail, v_tail, b_tail_len,
    o, lse,
    req_to_token, req_to_group, b_seq_len,
    *,
    sm_scale: float = 1.0,
    page_size: int = 16,
    logit_cap: float = 0.0,
    k_outliers_per_vector: int = 3,
    k_format: str = "i2f4",
    combinadic_read: bool = False,
    k_crank: Any = None,
    bitmap_read: bool = False,
    k_obmp: Any = None,
    k_fp4_mapscale: Any = None,
    k_fp4_mapcenter: Any = None,
    kv_outlier_map: bool = False,
    kv_int8_scale: bool = False,
    num_kv_splits: Optional[int] = None,
    num_stages: Optional[int] = None,
    num_warps: Optional[int] = None,
    max_seq_len: Optional[int] = None,
    max_tail_len: Optional[int] = None,
    attn_logits: Any = None,
    qzp_buf: Any = None,
    packed_start_offset: int = 0,
    seg_group_base: int = 0,
    _force_reference_kernel: bool = False,
    mean_seq_len: Optional[float] = None,
    err_flag: Any = None,
) -> None:
    """Canonical-KV paged decode attention.  Writes ``o [B,Hq,D]`` / ``lse [B,Hq]`` in place.

    Plane layouts, tables and the tail are as documented for the reference launcher
    (``paged_decode.py:2856-2887``).  ``seg_group_base > 0`` emits the un-merged state of a
    group-range segment without the tail (``:2892-2902``).

    ``mean_seq_len`` (not in the reference's signature) is a hint for the automatic split count
    only: a caller that passes ``max_seq_len`` to avoid the host sync may also say how long the
    requests are on average, see :func:`auto_num_kv_splits`.  ``err_flag`` (not in the reference's
    signature either): an int32 device tensor that receives ``_hip.ERR_TABLE_RANGE`` when a page id
    or group slot of the tables lies outside the planes (the kernels clamp such an entry, so nothing
    is read out of bounds; the reference leaves these checks to the pools, ``kv_pool.py:526-550``),
    and ``_hip.ERR_VALUE_RANGE`` when a K step lies above 2^15 (K values beyond some 1e5), which the
    f16 operands of the matrix-core kernel cannot carry: the output is finite but off, and
    ``_force_reference_kernel=True`` serves such a cache.
    """
    pages, ngroups = int(k_base.shape[0]), int(k_scale.shape[0])
    ps = int(page_size)
    if pages == 0 or ngroups == 0:
        group_tokens = 32
    else:
        group_tokens = (pages * ps) // ngroups
        if group_tokens not in (16, 32, 64, 128):
            raise ValueError(
                f"derived GROUP_TOKENS={group_tokens} (pages={pages} page_size={ps} "
                f"n_group_slots={ngroups}) must be in {{16,32,64,128}}")
    vsc = int(v_scale.shape[-1])
    v_bf16 = v_main.dtype == torch.bfloat16            # rows kept unquantised (pack.py:596-602)
    v_width = int(v_main.shape[-1]) if v_bf16 else int(v_main.shape[-1]) * 4
    group_channels = 32 if vsc == 0 else v_width // vsc
    if group_channels not in (16, 32, 64, 128):
        raise ValueError(f"derived GROUP_CHANNELS={group_channels} must be in {{16,32,64,128}}")
    kfmt = str(k_format).lower()
    if kfmt not in ("i2f4", "itf4"):
        raise ValueError(f"k_format must be i2f4|itf4; got {k_format!r}")
    if bitmap_read and combinadic_read:
        raise ValueError("combinadic_read and bitmap_read are mutually exclusive outlier-index sources")
    B, Hq = int(q.shape[0]), int(q.shape[1])
    D = int(k_base.shape[-1]) * 4
    Dv = v_width
    Hkv = int(k_base.shape[-2])
    if Dv % group_channels != 0:
        raise ValueError(f"canonical KV requires head_dim % {group_channels} == 0; got Lv={Dv}.")
    if Hkv < 1 or Hq < Hkv or Hq % Hkv != 0:
        raise NotImplementedError(
            "ommx_paged_decode_attention_canonical requires q_head_num to be an integer "
            f"multiple of n_kv_heads; got q_head_num={Hq} n_kv_heads={Hkv}.")
    for name, t in (("k_base", k_base), ("v_main", v_main), ("v_scale", v_scale), ("v_zp", v_zp)):
        # the kernels address a row as page*page_size + token and a head as a fixed-width slice of
        # it: the whole plane must be dense, a view that keeps only some heads or columns is not
        if t.dim() != 4 or not t.is_contiguous() or int(t.shape[0]) != pages or int(t.shape[1]) != ps \
                or int(t.shape[2]) != Hkv:
            raise ValueError(f"{name} must be a contiguous [pages={pages}, page_size={ps}, Hkv={Hkv}, w] "
                             f"plane; got shape {tuple(t.shape)} strides {tuple(t.stride())}")
    if q.dim() != 3 or int(q.shape[2]) != D:
        raise ValueError(f"q must be [B, Hq, D={D}]; got {tuple(q.shape)}")
    if tuple(k_scale.shape) != (ngroups, Hkv, D) or tuple(k_zp.shape) != (ngroups, Hkv, D) \
            or k_zp.dtype != torch.bfloat16:
        raise ValueError(f"k_scale / k_zp must be [group_slots={ngroups}, Hkv={Hkv}, D={D}] (k_zp bf16); "
                         f"got {tuple(k_scale.shape)} / {tuple(k_zp.shape)} {k_zp.dtype}")
    if tuple(o.shape) != (B, Hq, D) or tuple(lse.shape) != (B, Hq):
        raise ValueError(f"o must be [B={B}, Hq={Hq}, D={D}] and lse [B, Hq]; got {tuple(o.shape)} / "
                         f"{tuple(lse.shape)}")
    for name, t in (("b_seq_len", b_seq_len), ("b_tail_len", b_tail_len)):
        if t is not None and (int(t.numel()) < B or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous tensor of at least B={B} entries")
    for name, t in (("req_to_token", req_to_token), ("req_to_group", req_to_group)):
        if t.dim() != 2 or int(t.shape[0]) < B:
            raise ValueError(f"{name} must be [>= B={B}, columns]; got {tuple(t.shape)}")
    for name, t in (("k_base", k_base), ("k_scale", k_scale), ("v_main", v_main), ("o", o), ("lse", lse),
                    ("req_to_token", req_to_token), ("req_to_group", req_to_group),
                    ("b_seq_len", b_seq_len)):
        if t.device != q.device:
            raise ValueError(f"{name} is on {t.device}, q on {q.device}")
    off = int(packed_start_offset or 0)
    if off < 0 or off >= ps:
        raise ValueError(f"packed_start_offset={off} must be in [0, page_size={ps})")
    gbase = int(seg_group_base or 0)
    if gbase < 0:
        raise ValueError(f"seg_group_base={gbase} must be >= 0")
    k = int(k_outliers_per_vector)
    if k > 0 and k_oval is None:
        raise ValueError("k_outliers_per_vector > 0 requires the k_oval sidecar plane.")
    if combinadic_read and k > 0 and k_crank is None:
        raise ValueError("combinadic_read=True requires the k_crank combinadic-rank plane.")
    if bitmap_read and k > 0 and k_obmp is None:
        raise ValueError("bitmap_read=True requires the k_obmp flat-bitmask plane "
                         "(pack with ommx_pack_kv_canonical_block(..., outlier_repr='bitmap')).")
    if bitmap_read and k > 8:
        raise ValueError("bitmap_read packs the k_oval value stream into ONE int32 word, "
                         f"i.e. k <= 8; got k={k}. Use relidx7.")
    if (not combinadic_read) and (not bitmap_read) and k > 0 and k_oidx is None:
        raise ValueError("k_outliers_per_vector > 0 requires the k_oidx relidx7 sidecar plane "
                         "(or bitmap_read=True with a k_obmp plane).")
    use_map = bool(kv_outlier_map) and k > 0
    if use_map and (k_fp4_mapscale is None or k_fp4_mapcenter is None):
        raise ValueError("kv_outlier_map=True requires k_fp4_mapscale + k_fp4_mapcenter planes.")
    if use_map:
        for name, t in (("k_fp4_mapscale", k_fp4_mapscale), ("k_fp4_mapcenter", k_fp4_mapcenter)):
            if t.dtype != torch.bfloat16 or tuple(t.shape) != (ngroups, Hkv, D):
                raise ValueError(f"{name} must be bf16 [group_slots={ngroups}, Hkv={Hkv}, D={D}]; "
                                 f"got {t.dtype} {tuple(t.shape)}")
    if k > 0 and (k_oval.dtype != torch.uint8 or tuple(k_oval.shape) != (ngroups, Hkv, D, (k + 1) // 2)):
        raise ValueError(f"k_oval must be u8 [group_slots={ngroups}, Hkv={Hkv}, D={D}, {(k + 1) // 2}]; "
                         f"got {k_oval.dtype} {tuple(k_oval.shape)}")

    unsupported = []
    if k > 16:
        unsupported.append("more than 16 outliers per vector")
    # int8 exponent planes (kv_int8_scale) or the steps themselves as bf16 (paged_decode.py:1846-1855)
    scale_bf16 = k_scale.dtype == torch.bfloat16
    if k_scale.dtype != v_scale.dtype or k_scale.dtype not in (torch.int8, torch.bfloat16) \
            or scale_bf16 == bool(kv_int8_scale):
        unsupported.append(f"k_scale {k_scale.dtype} / v_scale {v_scale.dtype} with kv_int8_scale={bool(kv_int8_scale)}")
    if D != Dv or D not in (64, 128) or (Hq // Hkv) not in (1, 2, 4, 8):
        unsupported.append(f"head_dim {D}/{Dv} or GQA ratio {Hq // Hkv}")
    if group_tokens % ps != 0:
        unsupported.append("page_size not dividing the K group")
    if q.dtype != torch.bfloat16 or q.stride(-1) != 1:
        unsupported.append("q that is not bf16 with unit inner stride")
    if unsupported:
        raise NotImplementedError(
            "not covered by the HIP decode kernels: " + ", ".join(unsupported))
    if combinadic_read and k > 0:
        # The kernels read positions, not ranks: the rank plane is unranked into a position plane
        # by one launch ahead of the decode (paged_decode.py:969-1010 unranks inside the tile loop
        # and is 2.3-4.5x slower for it, pack.py:668).  A caller that decodes the same planes step
        # after step converts once with pack.derive_bitmap_from_combinadic instead.
        from .pack import convert_index_plane, index_plane_bytes
        if k_crank.dtype != torch.uint8 or tuple(k_crank.shape[:3]) != tuple(k_scale.shape) \
                or int(k_crank.shape[-1]) != index_plane_bytes("combinadic", group_tokens, k):
            raise ValueError("k_crank must be u8 [group_slots, Hkv, D, ceil(log2 C(group_tokens, k) / 8)]")
        to = "bitmap" if k <= 8 else "relidx7"          # the bitmask read serves up to 8 outliers
        plane = k_obmp if to == "bitmap" else k_oidx
        if plane is None or plane.dtype != torch.uint8 or tuple(plane.shape) != (
                *k_crank.shape[:3], index_plane_bytes(to, group_tokens, k)):
            # no unranked twin came with the ranks (the pool and store classes keep one)
            plane = torch.empty(*k_crank.shape[:3], index_plane_bytes(to, group_tokens, k),
                                dtype=torch.uint8, device=k_crank.device)
            convert_index_plane(k_crank.contiguous(), plane, group_tokens=group_tokens, k=k,
                                src_repr="combinadic", dst_repr=to)
        bitmap_read = to == "bitmap"
        k_obmp, k_oidx = (plane, k_oidx) if bitmap_read else (k_obmp, plane)
    # which index plane the kernels read (paged_decode.py:945-968 bitmap, :843-913 relidx7)
    k_index, index_repr = (k_obmp, _hip.INDEX_BITMAP) if bitmap_read else (k_oidx, _hip.INDEX_RELIDX7)
    if k > 0 and (k_index.dtype != torch.uint8 or tuple(k_index.shape[:3]) != tuple(k_scale.shape)
                  or int(k_index.shape[-1]) != ((group_tokens + 7) // 8 if bitmap_read else (7 * k + 7) // 8)):
        raise ValueError("outlier index plane must be u8 [group_slots, Hkv, D, group_tokens/8 (bitmap) "
                         "or ceil(7k/8) (relidx7)]")
    for name, t in (("k_scale", k_scale), ("k_zp", k_zp), ("k_oval", k_oval), ("k_index", k_index),
                    ("k_fp4_mapscale", k_fp4_mapscale), ("k_fp4_mapcenter", k_fp4_mapcenter)):
        if t is not None and not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
    if req_to_token.dtype != req_to_group.dtype or req_to_token.dtype not in (torch.int32, torch.int64):
        raise ValueError("req_to_token / req_to_group must both be int32 or both int64")
    if req_to_token.stride(-1) != 1 or req_to_group.stride(-1) != 1:
        raise ValueError("page / group tables must be contiguous along their last axis")
    if b_seq_len.dtype != torch.int32 or (b_tail_len is not None and b_tail_len.dtype != torch.int32):
        raise ValueError("b_seq_len / b_tail_len must be int32")
    if o.dtype != torch.float32 or lse.dtype != torch.float32 or o.stride(-1) != 1 or lse.stride(-1) != 1:
        raise ValueError("o / lse must be fp32 with unit inner stride")

    has_tail = gbase == 0 and k_tail is not None and v_tail is not None and b_tail_len is not None \
        and int(k_tail.shape[1]) > 0 \
        and (max_tail_len is None or int(max_tail_len) > 0)
    if has_tail:
        if k_tail.dtype != torch.bfloat16 or v_tail.dtype != torch.bfloat16 \
                or k_tail.stride(-1) != 1 or v_tail.stride(-1) != 1 or k_tail.dim() != 4 \
                or k_tail.shape != v_tail.shape or int(k_tail.shape[0]) < B \
                or tuple(k_tail.shape[2:]) != (Hkv, D):
            raise ValueError(f"k_tail / v_tail must be bf16 [>= B={B}, T, Hkv={Hkv}, D={D}] with unit inner "
                             f"stride; got {tuple(k_tail.shape)} / {tuple(v_tail.shape)}")

    _hip.require_gpu(q.device)
    if max_seq_len is not None:
        max_seq = max(1, int(max_seq_len))
    elif num_kv_splits is None and int(b_seq_len.numel()) > 0:
        lens = b_seq_len.tolist()                      # the one host sync of this path
        max_seq = max(1, max(lens))
        if mean_seq_len is None:
            mean_seq_len = sum(lens) / len(lens)
    else:
        max_seq = int(b_seq_len.max().item()) if int(b_seq_len.numel()) > 0 else 1
    # the serving-recipe kernel keeps three workgroups per compute unit resident with up to 4 q heads
    # per kv head (two with 8, and so do the other kernels); it also serves the call in one launch
    tuned = D == 128 and Hq // Hkv <= 4 and k == 6
    general4 = bitmap_read and 1 <= k <= 6 and ((D == 128 and Hq // Hkv <= 4) or      # (7, 8 outliers: two resident)
                                                (D == 64 and Hq // Hkv <= 2 and Hkv % 2 == 0))
    lean = ((tuned or general4) and group_tokens == 32 and group_channels == 32
            and not scale_bf16 and not v_bf16 and not _force_reference_kernel)
    if num_kv_splits is None:
        # (at head_dim 64 a wave of that kernel takes a pair of kv heads)
        paired = D == 64 and bitmap_read and 1 <= k <= 8 and Hq // Hkv <= 4 and Hkv % 2 == 0 and not (
            scale_bf16 or v_bf16 or _force_reference_kernel) and group_tokens == 32 and group_channels == 32
        num_kv_splits = auto_num_kv_splits(max_seq, B, Hkv // 2 if paired else Hkv, _cu_count(q.device),
                                           Hq // Hkv, group_tokens, mean_seq_len, resident=3 if lean else 2)
    S = max(1, int(num_kv_splits))
    if attn_logits is None:
        attn_logits = make_attn_logits(B, Hq, S, D, q.device)
    else:
        if attn_logits.dtype != torch.float32 or attn_logits.dim() != 4 \
                or tuple(attn_logits.shape[:2]) != (B, Hq) or int(attn_logits.shape[2]) < S \
                or int(attn_logits.shape[3]) < D + 1 or attn_logits.stride(-1) != 1:
            raise ValueError(f"attn_logits must be fp32 [B={B}, Hq={Hq}, >= {S}, >= {D + 1}] "
                             f"with unit inner stride; got {tuple(attn_logits.shape)}")
    if err_flag is not None and (err_flag.dtype != torch.int32 or err_flag.device != q.device):
        raise ValueError("err_flag must be an int32 tensor on the device of q")
    lib = _hip.load()
    stream = _hip.current_stream_ptr(q.device)
    splitkv = lib.ommx_decode_splitkv_ref if _force_reference_kernel else lib.ommx_decode_splitkv
    tail_args = ((k_tail.data_ptr(), v_tail.data_ptr(), k_tail.stride(0), k_tail.stride(1), k_tail.stride(2),
                  v_tail.stride(0), v_tail.stride(1), v_tail.stride(2), b_tail_len.data_ptr())
                 if has_tail else (None, None, 0, 0, 0, 0, 0, 0, None))
    planes = (k_base.data_ptr(), k_scale.data_ptr(), k_zp.data_ptr(),
              _hip.ptr(k_fp4_mapscale) if use_map else None, _hip.ptr(k_fp4_mapcenter) if use_map else None,
              _hip.ptr(k_index) if k > 0 else None, _hip.ptr(k_oval) if k > 0 else None,
              v_main.data_ptr(), v_scale.data_ptr(), v_zp.data_ptr(),
              req_to_token.data_ptr(), req_to_token.stride(0),
              req_to_group.data_ptr(), req_to_group.stride(0),
              1 if req_to_token.dtype == torch.int64 else 0,
              b_seq_len.data_ptr(),
              attn_logits.data_ptr(), attn_logits.stride(0), attn_logits.stride(1), attn_logits.stride(2))
    shape = (B, Hq, Hkv, D, ps, k, index_repr, 1 if scale_bf16 else 0, group_tokens, group_channels,
             1 if v_bf16 else 0, S, float(sm_scale), float(logit_cap), off, gbase,
             pages, ngroups, _hip.ptr(err_flag), stream)
    with torch.cuda.device(q.device):
        rc = splitkv(q.data_ptr(), q.stride(0), q.stride(1), *planes, *shape)
        _hip.check(rc, "ommx_decode_splitkv")
        rc = lib.ommx_decode_combine(
            attn_logits.data_ptr(), attn_logits.stride(0), attn_logits.stride(1), attn_logits.stride(2),
            q.data_ptr(), q.stride(0), q.stride(1), *tail_args[:8], tail_args[8], b_seq_len.data_ptr(),
            o.data_ptr(), o.stride(0), o.stride(1), lse.data_ptr(), lse.stride(0),
            B, Hq, Hkv, D, S, group_tokens, int(k_tail.shape[1]) if has_tail else 0,
            float(sm_scale), float(logit_cap), stream)
        _hip.check(rc, "ommx_decode_combine")


def merge_attention_states(o_parts: torch.Tensor, lse_parts: torch.Tensor, *, valid_lens=None,
                           out=None, lse_out=None):
    """Merge ``P`` partial attention states of the same query rows, computed over disjoint KV
    segments, into the state over their union (reference ``paged_decode.py:3556-3624``):
    ``m = max lse_p; w_p = exp(lse_p - m); o = sum w_p o_p / sum w_p; lse = m + log sum w_p``.

    ``o_parts [P, R, D]``, ``lse_parts [P, R]``; ``valid_lens [R]`` (optional) is the number of
    leading parts each row uses.  Returns ``(o [R, D] in o_parts' dtype, lse [R] fp32)``;
    ``out`` / ``lse_out`` are written in place when given.  One HIP launch, fp32 arithmetic.
    """
    if o_parts.dim() != 3:
        raise ValueError(
            f"o_parts must be [P, R, D]; got shape {tuple(o_parts.shape)}. "
            "Reshape any [P, ..., D] structure to a flat row axis R first.")
    if lse_parts.dim() != 2 or tuple(lse_parts.shape) != tuple(o_parts.shape[:2]):
        raise ValueError(
            f"lse_parts must be [P, R] matching o_parts[:2]; got "
            f"{tuple(lse_parts.shape)} vs {tuple(o_parts.shape[:2])}.")
    P, R, D = (int(x) for x in o_parts.shape)
    dev = o_parts.device
    if valid_lens is not None and int(valid_lens.numel()) != R:
        raise ValueError(f"valid_lens must have R={R} entries; got {valid_lens.numel()}.")
    _hip.require_gpu(dev)
    op = o_parts if (o_parts.dtype == torch.float32 and o_parts.stride(-1) == 1) \
        else o_parts.to(torch.float32).contiguous()
    lp = lse_parts if (lse_parts.dtype == torch.float32 and lse_parts.stride(-1) == 1
                       and lse_parts.device == dev) else lse_parts.to(dev, torch.float32).contiguous()
    valid = None if valid_lens is None else valid_lens.to(device=dev, dtype=torch.int32).contiguous()
    if out is None:
        out = torch.empty(R, D, dtype=o_parts.dtype, device=dev)
    if lse_out is None:
        lse_out = torch.empty(R, dtype=torch.float32, device=dev)
    direct = out.dtype == torch.float32 and out.stride(-1) == 1 and lse_out.dtype == torch.float32 \
        and lse_out.is_contiguous()
    o32 = out if direct else torch.empty(R, D, dtype=torch.float32, device=dev)
    l32 = lse_out if direct else torch.empty(R, dtype=torch.float32, device=dev)
    lib = _hip.load()
    with torch.cuda.device(dev):
        _hip.check(lib.ommx_merge_states(
            op.data_ptr(), lp.data_ptr(), _hip.ptr(valid), o32.data_ptr(), l32.data_ptr(),
            P, R, D, op.stride(0), op.stride(1), lp.stride(0), o32.stride(0),
            _hip.current_stream_ptr(dev)), "ommx_merge_states")
    if not direct:
        out.copy_(o32)
        lse_out.copy_(l32)
    return out, lse_out


__all__ = ["ommx_paged_decode_attention_canonical", "merge_attention_states", "auto_num_kv_splits",
           "make_attn_logits"]
