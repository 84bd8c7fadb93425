"""ctypes binding of ``libommx_hip.so`` (the C ABI declared in ``include/ommx_hip.h``).

The library is built in-tree by ``open_ommx_serve_amd.csrc.build``.  There is no fallback:
if it is missing or an entry point fails, the caller gets an exception.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                         "csrc", "libommx_hip.so")
_lib: Optional[C.CDLL] = None

STORE_TABLE_FLOATS = 264
ABI_VERSION = 8
INDEX_BITMAP, INDEX_RELIDX7, INDEX_COMBINADIC = 0, 1, 2
SCALE_POW2_INT8, SCALE_POW2_BF16, SCALE_BF16 = 0, 1, 2


def scale_mode(use_pow2: bool, kv_int8_scale: bool) -> int:
    """C-ABI scale_mode of a recipe: the int8 exponent plane exists only for power-of-two
    steps (reference pack.py:397 ``use_int8_scale = kv_int8_scale and use_pow2``)."""
    if not use_pow2:
        return SCALE_BF16
    return SCALE_POW2_INT8 if kv_int8_scale else SCALE_POW2_BF16
ERR_NONFINITE_K, ERR_NONFINITE_V, ERR_UNDERFILLED, ERR_EXP_RANGE, ERR_RING_RANGE = 1, 2, 4, 8, 16
ERR_INDEX_PLANE = 32
ERR_TABLE_RANGE = 64
ERR_VALUE_RANGE = 128
NOTE_WIDE_STEP = 256        # not an error: the store wrote a K step above 2^15 (see kv_pool.check_errors)

_P, _I, _L, _F = C.c_void_p, C.c_int, C.c_int64, C.c_float

_DECODE_ARGS = [
    _P, _L, _L,                       # q, strides
    _P, _P, _P, _P, _P, _P, _P,       # k planes
    _P, _P, _P,                       # v planes
    _P, _L, _P, _L, _I,               # tables
    _P,                               # b_seq_len
    _P, _L, _L, _L,                   # attn_logits, strides
    _I, _I, _I, _I, _I, _I, _I, _I,       # B Hq Hkv D ps kout index_repr scale_bf16
    _I, _I, _I, _I,                       # group_tokens group_channels v_bf16 S
    _F, _F, _I, _I,                   # sm_scale cap off gbase
    _I, _I, _P, _P,                   # num_pages num_group_slots err_flag stream
]

_SIGNATURES = {
    "ommx_abi_version": (_I, []),
    "ommx_last_error": (C.c_char_p, []),
    "ommx_store_default_table": (None, [_P]),
    "ommx_store_pack": (_I, [_P, _P, _I, _L, _L, _L, _L, _P] + [_I] * 11 + [_P, _P, _P,
                             _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "ommx_decode_splitkv": (_I, _DECODE_ARGS),
    "ommx_decode_splitkv_ref": (_I, _DECODE_ARGS),
    "ommx_clamp_table_id": (_I, [_I, _I, _P]),
    "ommx_decode_combine": (_I, [_P, _L, _L, _L, _P, _L, _L, _P, _P, _L, _L, _L, _L, _L, _L,
                                 _P, _P, _P, _L, _L, _P, _L, _I, _I, _I, _I, _I, _I, _I, _F, _F, _P]),
    "ommx_decode_attention_noalloc": (_I, [
        _P, _L, _L, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P,      # q, K planes, V planes
        _P, _L, _P, _L, _I, _P,                                  # tables, b_seq_len
        _P, _P, _L, _L, _L, _L, _L, _L, _P,                      # tail rows, strides, b_tail_len
        _P, _L, _L, _P, _L,                                      # o, lse
        _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I,      # B Hq Hkv D ps kout repr scale_bf16 gt gc v_bf16 S tail_rows
        _F, _F, _I, _I, _I, _P, _P]),                            # sm_scale cap off num_pages num_group_slots err stream
    "ommx_ring_write": (_I, [_P, _P, _L, _L, _L, _L, _P, _P, _L, _I, _P, _P, _P,
                             _I, _I, _I, _I, _I, _P, _P]),
    "ommx_merge_states": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _L, _L, _L, _L, _P]),
    "ommx_index_plane_bytes": (_I, [_I, _I, _I]),
    "ommx_index_convert": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _P]),
    "ommx_tail_gather": (_I, [_P, _P, _L, _I, _P, _P, _P, _P, _P, _P, _P,
                              _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P]),
}


def lib_path() -> str:
    return _LIB_PATH


def load() -> C.CDLL:
    """Load the shared library (once) and declare every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"{_LIB_PATH} is missing: build it with `python -m open_ommx_serve_amd.csrc.build` "
            "(the OMMX operators have no fallback path)")
    lib = C.CDLL(_LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.ommx_abi_version() != ABI_VERSION:
        raise RuntimeError("libommx_hip.so ABI version mismatch; rebuild it")
    _lib = lib
    return lib


def exported_symbols():
    return tuple(_SIGNATURES)


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().ommx_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (rc={rc}): {msg}")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(device: torch.device) -> None:
    if device.type != "cuda":
        raise RuntimeError(
            f"OMMX HIP operators need tensors on a ROCm GPU; got device {device}. "
            "There is no CPU fallback.")
