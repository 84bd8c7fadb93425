"""Serving recipe + per-model geometry (reference ``integration/vllm/config.py:219-440``).

Same field names, defaults and environment knobs as the reference's ``OMMXServingConfig``;
the defaults are the serving recipe the tuned kernels are built for (i2f4, 6 signed outliers,
flat bitmask, power-of-two steps, dedicated FP4 map, 32-token / 32-channel groups, sink 8,
recent 32, page 16).
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Any, Optional

from ...attention.kv_window import WindowSpec

DEFAULT_OUTLIER_REPR = "bitmap"
DEFAULT_OUTLIERS = 6
DEFAULT_POW2 = True
GROUP_TOKENS = 32
OUTLIER_REPRS = ("relidx7", "combinadic", "bitmap")
_OFF = {"", "0", "false", "off", "no"}


def _env_present(name: str) -> bool:
    return os.environ.get(name, "").strip() != ""


def _env_str(name: str, default: str) -> str:
    v = os.environ.get(name, "").strip()
    return v.lower() if v else default


def _env_int(name: str, default: int) -> int:
    v = os.environ.get(name, "").strip()
    return int(v) if v else int(default)


def _env_float(name: str, default: float) -> float:
    v = os.environ.get(name, "").strip()
    return float(v) if v else float(default)


def _env_bool(name: str, default: bool) -> bool:
    if not _env_present(name):
        return bool(default)
    return os.environ[name].strip().lower() not in _OFF


def _env_int_alias(canonical: str, alias: str, default: int) -> int:
    return _env_int(canonical, _env_int(alias, default))


@dataclass
class OMMXServingConfig:
    k_format: str = "i2f4"
    outliers_per_vector: int = DEFAULT_OUTLIERS
    outlier_select: str = "signed"
    outlier_repr: str = DEFAULT_OUTLIER_REPR
    use_pow2: bool = DEFAULT_POW2
    combinadic_read: Any = None
    bitmap_read: Optional[bool] = None
    sink_tokens: int = 8
    recent_window: int = 32
    group_tokens: int = GROUP_TOKENS
    group_channels: int = GROUP_TOKENS
    kv_outlier_map: bool = True
    strict: bool = False
    head_dim: int = 128
    n_q_heads: int = 32
    n_kv_heads: int = 8
    page_size: int = 16
    max_context: int = 4096
    extra: dict = field(default_factory=dict)

    def window(self) -> WindowSpec:
        return WindowSpec(sink_tokens=self.sink_tokens, recent_window=self.recent_window,
                          group_tokens=self.group_tokens, page_size=self.page_size)

    def resolved_bitmap_read(self) -> bool:
        """The index plane the decode kernel reads follows the one the store wrote
        (config.py:280-295); an explicit bool is for A/B runs only."""
        if self.bitmap_read is None:
            return self.outlier_repr == "bitmap"
        return bool(self.bitmap_read)

    def resolved_combinadic_read(self) -> bool:
        if self.combinadic_read is None:
            return self.outlier_repr == "combinadic"
        return bool(self.combinadic_read)

    def store_kwargs(self) -> dict:
        """Constructor arguments shared by ``CanonicalKVStore`` and ``MultiSeqKVPool``."""
        return dict(k_format=self.k_format, outliers_per_vector=self.outliers_per_vector,
                    outlier_select=self.outlier_select, outlier_repr=self.outlier_repr,
                    use_pow2=self.use_pow2, kv_outlier_map=self.kv_outlier_map,
                    window=self.window(), group_channels=self.group_channels)


def resolve_serving_config(*, head_dim: Optional[int] = None, n_q_heads: Optional[int] = None,
                           n_kv_heads: Optional[int] = None, page_size: Optional[int] = None,
                           max_context: Optional[int] = None) -> OMMXServingConfig:
    """Environment knobs + model geometry -> config (config.py:342-440).  Named presets
    (``OMMX_RECIPE``) belong to the reference's recipe registry, which this package does not
    carry: a set variable raises instead of silently serving the default recipe."""
    if _env_present("OMMX_RECIPE"):
        raise NotImplementedError(
            "OMMX_RECIPE presets are not available here; set the OMMX_ATTN_* / OMMX_KV_* knobs")
    gt = _env_int_alias("OMMX_KV_GROUP_TOKENS", "OMMX_ATTN_GROUP_TOKENS", GROUP_TOKENS)
    gc = _env_int_alias("OMMX_KV_GROUP_CHANNELS", "OMMX_ATTN_GROUP_CHANNELS", GROUP_TOKENS)
    if _env_present("OMMX_OUTLIER_PERCENT"):
        pct = _env_float("OMMX_OUTLIER_PERCENT", 0.0)
        npv = max(1, int(round(gt * pct))) if pct > 0 else 0
    else:
        npv = _env_int("OMMX_ATTN_OUTLIERS", DEFAULT_OUTLIERS)
    cfg = OMMXServingConfig(
        k_format=_env_str("OMMX_ATTN_K_FORMAT", "i2f4"),
        outliers_per_vector=npv,
        outlier_select=_env_str("OMMX_ATTN_OUTLIER_SELECT", "signed"),
        outlier_repr=_env_str("OMMX_ATTN_OUTLIER_REPR", DEFAULT_OUTLIER_REPR),
        use_pow2=_env_bool("OMMX_ATTN_POW2", DEFAULT_POW2),
        combinadic_read=(_env_bool("OMMX_ATTN_COMBINADIC_READ", False)
                         if _env_present("OMMX_ATTN_COMBINADIC_READ") else None),
        bitmap_read=(_env_bool("OMMX_ATTN_BITMAP_READ", False)
                     if _env_present("OMMX_ATTN_BITMAP_READ") else None),
        sink_tokens=_env_int_alias("OMMX_KV_SINK", "OMMX_ATTN_SINK", 8),
        recent_window=_env_int_alias("OMMX_KV_RECENT", "OMMX_ATTN_RECENT", 32),
        group_tokens=gt, group_channels=gc,
        kv_outlier_map=_env_bool("OMMX_KV_OUTLIER_MAP", True),
        strict=_env_bool("OMMX_STRICT", False),
        max_context=_env_int("OMMX_ATTN_MAXCTX", 4096),
    )
    for name, val in (("head_dim", head_dim), ("n_q_heads", n_q_heads), ("n_kv_heads", n_kv_heads),
                      ("page_size", page_size), ("max_context", max_context)):
        if val is not None:
            setattr(cfg, name, int(val))
    if cfg.recent_window < 1 or cfg.sink_tokens < 0:
        # the step seam packs completed groups before the forward writes token seq-1; that token
        # stays outside the packed region only while at least one recent row is kept as bf16
        raise ValueError(f"OMMX_KV_RECENT must be >= 1 and OMMX_KV_SINK >= 0; got recent="
                         f"{cfg.recent_window}, sink={cfg.sink_tokens}: with no recent row the "
                         "seam would pack a group whose last token is not written yet")
    if cfg.k_format not in ("i2f4", "itf4"):
        raise ValueError(f"OMMX_ATTN_K_FORMAT must be i2f4|itf4; got {cfg.k_format!r}")
    if cfg.outlier_repr not in OUTLIER_REPRS:
        raise ValueError(f"OMMX_ATTN_OUTLIER_REPR must be one of {OUTLIER_REPRS}; got {cfg.outlier_repr!r}")
    if cfg.resolved_bitmap_read() and cfg.resolved_combinadic_read():
        raise ValueError("OMMX_ATTN_BITMAP_READ and OMMX_ATTN_COMBINADIC_READ are mutually exclusive "
                         "outlier-index sources (a pack carries exactly one index plane)")
    if cfg.bitmap_read and cfg.outlier_repr != "bitmap":
        raise ValueError("OMMX_ATTN_BITMAP_READ=1 needs OMMX_ATTN_OUTLIER_REPR=bitmap: the store "
                         f"allocates no k_obmp plane under outlier_repr={cfg.outlier_repr!r}")
    if cfg.combinadic_read and cfg.outlier_repr != "combinadic":
        raise ValueError("OMMX_ATTN_COMBINADIC_READ=1 needs OMMX_ATTN_OUTLIER_REPR=combinadic: the "
                         f"store allocates no k_crank plane under outlier_repr={cfg.outlier_repr!r}")
    if cfg.resolved_bitmap_read() and cfg.outliers_per_vector > 8:
        raise ValueError(f"outlier_repr=bitmap cannot serve outliers_per_vector={cfg.outliers_per_vector}: "
                         "the bitmask read is limited to k <= 8 (config.py:458-465).  Set "
                         "OMMX_ATTN_OUTLIER_REPR=relidx7, or lower OMMX_ATTN_OUTLIERS / OMMX_OUTLIER_PERCENT.")
    return cfg


__all__ = ["OMMXServingConfig", "resolve_serving_config", "DEFAULT_OUTLIER_REPR",
           "DEFAULT_OUTLIERS", "DEFAULT_POW2", "GROUP_TOKENS", "OUTLIER_REPRS"]
