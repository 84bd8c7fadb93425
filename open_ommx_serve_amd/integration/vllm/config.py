"""Serving recipe + per-model geometry (reference ``integration/vllm/config.py:219-440``).

The dataclass keeps the reference's field names and defaults, and the resolver reads the
reference's environment names, because those two lists are the interface a deployment
already has.  The defaults are the serving recipe the tuned kernels are built for (i2f4,
6 signed outliers, flat bitmask, power-of-two steps, dedicated FP4 map, 32-token /
32-channel groups, sink 8, recent 32, page 16).

How a value is found is one table (``KNOBS``): per field the environment names that may
carry it, in order of precedence, and the parser for its text.  ``explain_knobs()`` prints
that table, so the list of knobs a worker honours can be read from a running process.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field, fields
from typing import Any, Callable, Dict, Mapping, NamedTuple, Optional, Tuple

from ...attention.kv_window import WindowSpec

DEFAULT_OUTLIER_REPR = "bitmap"
DEFAULT_OUTLIERS = 6
DEFAULT_POW2 = True
GROUP_TOKENS = 32
OUTLIER_REPRS = ("relidx7", "combinadic", "bitmap")
K_FORMATS = ("i2f4", "itf4")


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


# ── the knob table ─────────────────────────────────────────────────────────────────────────

def _word(text: str) -> str:
    return text.lower()


def _switch(text: str) -> bool:
    """A knob that is set is on unless its text is one of the usual spellings of "off"."""
    return text.lower() not in ("0", "false", "off", "no")


class Knob(NamedTuple):
    target: str                                  # field of OMMXServingConfig
    names: Tuple[str, ...]                       # environment names, the first one that is set wins
    parse: Callable[[str], Any]


KNOBS: Tuple[Knob, ...] = (
    Knob("k_format", ("OMMX_ATTN_K_FORMAT",), _word),
    Knob("outliers_per_vector", ("OMMX_ATTN_OUTLIERS",), int),
    Knob("outlier_select", ("OMMX_ATTN_OUTLIER_SELECT",), _word),
    Knob("outlier_repr", ("OMMX_ATTN_OUTLIER_REPR",), _word),
    Knob("use_pow2", ("OMMX_ATTN_POW2",), _switch),
    Knob("combinadic_read", ("OMMX_ATTN_COMBINADIC_READ",), _switch),
    Knob("bitmap_read", ("OMMX_ATTN_BITMAP_READ",), _switch),
    Knob("sink_tokens", ("OMMX_KV_SINK", "OMMX_ATTN_SINK"), int),
    Knob("recent_window", ("OMMX_KV_RECENT", "OMMX_ATTN_RECENT"), int),
    Knob("group_tokens", ("OMMX_KV_GROUP_TOKENS", "OMMX_ATTN_GROUP_TOKENS"), int),
    Knob("group_channels", ("OMMX_KV_GROUP_CHANNELS", "OMMX_ATTN_GROUP_CHANNELS"), int),
    Knob("kv_outlier_map", ("OMMX_KV_OUTLIER_MAP",), _switch),
    Knob("strict", ("OMMX_STRICT",), _switch),
    Knob("max_context", ("OMMX_ATTN_MAXCTX",), int),
)
# Knobs that are not a field of their own: the outlier count as a share of the group, and the
# reference's named presets (its recipe registry is not part of this package).
SHARE_KNOB = "OMMX_OUTLIER_PERCENT"
PRESET_KNOB = "OMMX_RECIPE"
GEOMETRY = ("head_dim", "n_q_heads", "n_kv_heads", "page_size", "max_context")


def _set_text(env: Mapping[str, str], name: str) -> Optional[str]:
    """The knob's text, or None when it is unset or blank (a blank variable counts as unset)."""
    text = env.get(name, "").strip()
    return text or None


def read_knobs(env: Optional[Mapping[str, str]] = None) -> Dict[str, Any]:
    """Field values the environment asks for; fields nobody set are absent from the result."""
    env = os.environ if env is None else env
    found: Dict[str, Any] = {}
    for knob in KNOBS:
        for name in knob.names:
            text = _set_text(env, name)
            if text is None:
                continue
            try:
                found[knob.target] = knob.parse(text)
            except ValueError as exc:
                raise ValueError(f"{name}={text!r} does not read as {knob.parse.__name__}") from exc
            break
    share = _set_text(env, SHARE_KNOB)
    if share is not None:
        # a share of the K vector, at least one outlier once the share is positive; it outranks the count
        gt = found.get("group_tokens", GROUP_TOKENS)
        frac = float(share)
        found["outliers_per_vector"] = max(1, int(round(gt * frac))) if frac > 0 else 0
    return found


def explain_knobs() -> str:
    """One line per knob: field, environment names in order of precedence, current text."""
    rows = [f"{k.target:22s} {' > '.join(k.names):55s} {next((t for t in (_set_text(os.environ, n) for n in k.names) if t), '-')}"
            for k in KNOBS]
    rows.append(f"{'outliers_per_vector':22s} {SHARE_KNOB + ' (share of group_tokens, outranks the count)':55s} "
                f"{_set_text(os.environ, SHARE_KNOB) or '-'}")
    return "\n".join(rows)


def _refuse(cfg: OMMXServingConfig) -> Optional[str]:
    """Why this configuration cannot be served, or None.  Every rule is the reference's
    (config.py:398-465) except the first, which belongs to the step seam of this package."""
    bitmap, ranks = cfg.resolved_bitmap_read(), cfg.resolved_combinadic_read()
    rules = (
        (cfg.recent_window < 1 or cfg.sink_tokens < 0,
         f"OMMX_KV_RECENT must be >= 1 and OMMX_KV_SINK >= 0 (got recent={cfg.recent_window}, "
         f"sink={cfg.sink_tokens}): the seam packs a completed group before the forward writes the "
         "step's own token, which is safe only while that token still sits among the bf16 recent rows"),
        (cfg.k_format not in K_FORMATS,
         f"OMMX_ATTN_K_FORMAT={cfg.k_format!r}: the K base format is one of {K_FORMATS}"),
        (cfg.outlier_repr not in OUTLIER_REPRS,
         f"OMMX_ATTN_OUTLIER_REPR={cfg.outlier_repr!r}: the index plane is one of {OUTLIER_REPRS}"),
        (bitmap and ranks,
         "OMMX_ATTN_BITMAP_READ and OMMX_ATTN_COMBINADIC_READ both on: a pack holds one index plane, "
         "so the decode can read positions from one of them only"),
        (bool(cfg.bitmap_read) and cfg.outlier_repr != "bitmap",
         f"OMMX_ATTN_BITMAP_READ=1 with outlier_repr={cfg.outlier_repr!r}: that store writes no "
         "k_obmp plane to read; set OMMX_ATTN_OUTLIER_REPR=bitmap"),
        (bool(cfg.combinadic_read) and cfg.outlier_repr != "combinadic",
         f"OMMX_ATTN_COMBINADIC_READ=1 with outlier_repr={cfg.outlier_repr!r}: that store writes no "
         "k_crank plane to read; set OMMX_ATTN_OUTLIER_REPR=combinadic"),
        (bitmap and cfg.outliers_per_vector > 8,
         f"{cfg.outliers_per_vector} outliers per vector on the bitmask plane: the bitmask read stops "
         "at 8; use OMMX_ATTN_OUTLIER_REPR=relidx7 or a lower OMMX_ATTN_OUTLIERS / OMMX_OUTLIER_PERCENT"),
    )
    return next((why for hit, why in rules if hit), None)


def resolve_serving_config(*, head_dim: Optional[int] = None, n_q_heads: Optional[int] = None,
                           n_kv_heads: Optional[int] = None, page_size: Optional[int] = None,
                           max_context: Optional[int] = None) -> OMMXServingConfig:
    """Defaults, then environment knobs, then the model's geometry (reference config.py:342-440).
    A named preset raises: serving the default recipe under a preset's name would be silent."""
    if _set_text(os.environ, PRESET_KNOB) is not None:
        raise NotImplementedError(f"{PRESET_KNOB} presets come from the reference's recipe registry, which "
                                  "is not part of this package; spell the recipe with the OMMX_ATTN_* / "
                                  "OMMX_KV_* knobs (explain_knobs() lists them)")
    cfg = OMMXServingConfig(**read_knobs())
    given = dict(head_dim=head_dim, n_q_heads=n_q_heads, n_kv_heads=n_kv_heads, page_size=page_size,
                 max_context=max_context)
    for name in GEOMETRY:
        if given[name] is not None:
            setattr(cfg, name, int(given[name]))
    why = _refuse(cfg)
    if why is not None:
        raise ValueError(why)
    return cfg


assert {k.target for k in KNOBS} <= {f.name for f in fields(OMMXServingConfig)}

__all__ = ["OMMXServingConfig", "resolve_serving_config", "read_knobs", "explain_knobs", "KNOBS",
           "DEFAULT_OUTLIER_REPR", "DEFAULT_OUTLIERS", "DEFAULT_POW2", "GROUP_TOKENS", "OUTLIER_REPRS"]
