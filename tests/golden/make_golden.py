"""Write golden vectors for the composed KV packer by running the reference's own packer.

Run ONCE in the build container, where the reference checkout is mounted:

    python tests/golden/make_golden.py /root/reference
    python tests/golden/make_golden.py /root/reference --only map_scale_rounding   (adds one case)

The bit pattern of ``ommx_pack_kv_canonical_block`` (outlier tie order, fp32 operation
order, bf16 rounding, log2/log ulps) is the one thing on this path that no closed form or
invariant fixes, so it is recorded here as data: the inputs (bf16 bit patterns) and every
plane the reference writes for them, plus ``dequant_kv_canonical`` of those planes.  The
fixtures are small ``.npz`` files; tests only read them.  Nothing from the reference's
source text is stored.

Besides the serving recipe (``pack_<case>.npz``) one small block per format variant is
written (``variant_<name>.npz``): the other two index planes, base-shared outliers, the
magnitude selector, steps that are not powers of two, bf16 step planes, 16/64/128-element
vectors with up to 10 outliers, and bf16 V.  Each holds the recipe it was packed with.
"""
from __future__ import annotations

import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
PLANES = ("k_base", "k_scale", "k_zp", "k_obmp", "k_oval", "k_fp4_mapscale",
          "k_fp4_mapcenter", "v_main", "v_scale", "v_zp")
SEEDS = {"tiny_ties": 101, "small_gauss": 202, "layer_outliers": 303, "wide_range": 404,
         "fp32_inputs": 505, "map_scale_rounding": 606}
RECIPE = dict(outliers_per_vector=6, outlier_select="signed", outlier_repr="bitmap",
              k_format="i2f4", use_pow2=True, kv_outlier_map=True, kv_int8_scale=True,
              group_tokens=32, group_channels=32, page_size=16, v_format="i2")


# name -> (recipe overrides, (T, H, D), seed)
VARIANTS = {
    "relidx7": (dict(outlier_repr="relidx7"), (128, 2, 64), 611),
    "combinadic": (dict(outlier_repr="combinadic"), (128, 2, 64), 612),
    "base_shared": (dict(kv_outlier_map=False), (128, 2, 64), 613),
    "abs_select": (dict(outlier_select="abs"), (128, 2, 64), 614),
    "abs_relidx7_k3": (dict(outlier_select="abs", outlier_repr="relidx7", outliers_per_vector=3),
                       (64, 1, 64), 615),
    "free_steps": (dict(use_pow2=False), (128, 2, 64), 616),
    "bf16_steps": (dict(kv_int8_scale=False), (128, 2, 64), 617),
    "gt64_gc64_k10": (dict(group_tokens=64, group_channels=64, outliers_per_vector=10,
                           kv_outlier_map=False), (128, 1, 128), 618),
    "gt64_gc64_k10_map": (dict(group_tokens=64, group_channels=64, outliers_per_vector=10),
                          (128, 1, 64), 619),
    "gt128_gc128_k10": (dict(group_tokens=128, group_channels=128, outliers_per_vector=10,
                             kv_outlier_map=False), (256, 1, 128), 620),
    "gt128_gc32_k16_relidx7": (dict(group_tokens=128, outliers_per_vector=16,
                                    outlier_repr="relidx7"), (128, 1, 64), 621),
    "gt16_k3": (dict(group_tokens=16, outliers_per_vector=3), (64, 2, 64), 622),
    "gt16_gc16_k2": (dict(group_tokens=16, group_channels=16, outliers_per_vector=2),
                     (64, 1, 64), 623),
    "k0": (dict(outliers_per_vector=0), (64, 2, 64), 624),
    "k1": (dict(outliers_per_vector=1), (64, 2, 64), 625),
    "v_bf16": (dict(v_format="bf16"), (64, 2, 64), 626),
    "v_bf16_bf16_steps": (dict(v_format="bf16", kv_int8_scale=False), (64, 1, 64), 627),
}
INDEX_PLANES = ("k_oidx", "k_crank")


def _bits(t: torch.Tensor) -> np.ndarray:
    """Raw storage of a tensor as a numpy integer array (bf16 -> uint16)."""
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float32:
        return t.contiguous().view(torch.int32).numpy().view(np.uint32)
    return t.contiguous().numpy()


def main(ref_root: str) -> None:
    sys.path.insert(0, ref_root)
    from ommx_gpu_serve.attention.pack import (  # type: ignore
        dequant_kv_canonical, ommx_pack_kv_canonical_block)

    only = sys.argv[3:] if len(sys.argv) > 3 and sys.argv[2] == "--only" else None
    index = {}
    if only:      # add cases to the fixtures already written: the other files stay as they are
        with open(os.path.join(HERE, "pack_index.json")) as f:
            index = json.load(f)["sha256"]
    for name in (only or SEEDS):
        g = torch.Generator().manual_seed(SEEDS[name])
        K, V = _case_inputs(name, g)
        planes = ommx_pack_kv_canonical_block(K, V, **RECIPE)
        Kd, Vd = dequant_kv_canonical(planes)
        out = {"K_bits": _bits(K), "V_bits": _bits(V),
               "K_dq_bits": _bits(Kd), "V_dq_bits": _bits(Vd)}
        for p in PLANES:
            out[p] = _bits(planes[p])
        np.savez_compressed(os.path.join(HERE, f"pack_{name}.npz"), **out)
        index[name] = {p: hashlib.sha256(_bits(planes[p]).tobytes()).hexdigest() for p in PLANES}
        print(name, {p: tuple(planes[p].shape) for p in PLANES})
    with open(os.path.join(HERE, "pack_index.json"), "w") as f:
        json.dump({"recipe": RECIPE, "torch": torch.__version__, "sha256": index}, f, indent=1)
    if only:
        return

    vindex = {}
    for name, (over, shape, seed) in VARIANTS.items():
        g = torch.Generator().manual_seed(seed)
        K, V = _variant_inputs(shape, g)
        recipe = dict(RECIPE, **over)
        planes = ommx_pack_kv_canonical_block(K, V, **recipe)
        Kd, Vd = dequant_kv_canonical(planes)
        out = {"K_bits": _bits(K), "V_bits": _bits(V),
               "K_dq_bits": _bits(Kd), "V_dq_bits": _bits(Vd)}
        held = []
        for p in PLANES + INDEX_PLANES:
            if torch.is_tensor(planes.get(p)):
                out[p] = _bits(planes[p])
                held.append(p)
        np.savez_compressed(os.path.join(HERE, f"variant_{name}.npz"), **out)
        vindex[name] = {"recipe": recipe, "shape": list(shape), "planes": {
            p: [str(planes[p].dtype).replace("torch.", ""), list(planes[p].shape)] for p in held}}
        print(name, vindex[name]["planes"])
    with open(os.path.join(HERE, "variant_index.json"), "w") as f:
        json.dump(vindex, f, indent=1)


def _variant_inputs(shape, g: torch.Generator):
    """Gaussian rows with a few heavy channels, some exact ties and a constant vector."""
    T, H, D = shape
    K = torch.randn(T, H, D, generator=g)
    V = torch.randn(T, H, D, generator=g) * 2.0
    K[:, :, [3, 17, 40]] *= 9.0
    K[:, 0, 5] = torch.randint(-3, 4, (T,), generator=g).float() * 0.5      # many ties
    K[:, 0, 6] = 0.25                                                        # constant
    V[1, 0, :16] = 1.0
    return K.to(torch.bfloat16), V.to(torch.bfloat16)


def _case_inputs(name: str, g: torch.Generator):
    if name == "tiny_ties":
        T, H, D = 64, 2, 64
        lv = torch.tensor([-2.0, -1.0, -0.5, 0.0, 0.0, 0.5, 1.0, 2.0, 4.0])
        K = lv[torch.randint(0, 9, (T, H, D), generator=g)]
        V = lv[torch.randint(0, 9, (T, H, D), generator=g)]
    elif name == "small_gauss":
        T, H, D = 128, 2, 64
        K = torch.randn(T, H, D, generator=g)
        V = torch.randn(T, H, D, generator=g)
    elif name == "layer_outliers":
        T, H, D = 128, 8, 128
        K = torch.randn(T, H, D, generator=g)
        V = torch.randn(T, H, D, generator=g)
        K[:, :, [3, 40, 77, 120]] *= 12.0
    elif name == "wide_range":
        T, H, D = 64, 1, 64
        K = torch.randn(T, H, D, generator=g) * torch.exp2(
            torch.randint(-12, 9, (1, H, D), generator=g).float())
        V = torch.randn(T, H, D, generator=g) * torch.exp2(
            torch.randint(-12, 9, (T, H, 1), generator=g).float())
        K[:32, 0, 0] = 1.5
        V[0, 0, :32] = -0.75
        K[:32, 0, 1] = 0.0
        K[5, 0, 1] = -0.0
    elif name == "fp32_inputs":
        # fp32 K/V: the zero point and the map parameters are then genuinely rounded
        T, H, D = 64, 2, 64
        return torch.randn(T, H, D, generator=g), torch.randn(T, H, D, generator=g) * 3.0
    elif name == "map_scale_rounding":
        # ``12.0 / o_range`` (pack.py:492) has the Python scalar on the left, which torch evaluates as
        # reciprocal(o_range) * 12.0: two roundings.  About six ranges in a million give another bf16
        # map scale than one correctly rounded division; every K vector here has such a range
        # (smallest value 0, largest the range), found by search from this seed.
        T, H, D = 32, 1, 64
        r = torch.exp2(torch.rand(4_000_000, generator=g) * 20 - 8) * (1 + torch.rand(4_000_000, generator=g))
        one = (torch.tensor(12.0) / r).to(torch.bfloat16).view(torch.int16)
        two = (torch.reciprocal(r) * 12.0).to(torch.bfloat16).view(torch.int16)
        hits = r[(one != two).nonzero().flatten()]
        assert len(hits) >= 16, len(hits)
        K = torch.empty(T, H, D)
        for c in range(D):
            rc = hits[c % len(hits)]
            col = (0.3 + 0.4 * torch.rand(T, generator=g)) * rc
            col[(3 * c) % T] = 0.0
            col[(3 * c + 7) % T] = rc
            K[:, 0, c] = col
        return K, torch.randn(T, H, D, generator=g)
    else:
        raise KeyError(name)
    return K.to(torch.bfloat16), V.to(torch.bfloat16)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
