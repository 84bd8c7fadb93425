"""Write golden vectors for the composed KV packer by running the reference's own packer.

Run ONCE in the build container, where the reference checkout is mounted:

    python tests/golden/make_golden.py /root/reference

The bit pattern of ``ommx_pack_kv_canonical_block`` (outlier tie order, fp32 operation
order, bf16 rounding, log2/log ulps) is the one thing on this path that no closed form or
invariant fixes, so it is recorded here as data: the inputs (bf16 bit patterns) and every
plane the reference writes for them, plus ``dequant_kv_canonical`` of those planes.  The
fixtures are small ``.npz`` files; tests only read them.  Nothing from the reference's
source text is stored.
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
         "fp32_inputs": 505}
RECIPE = dict(outliers_per_vector=6, outlier_select="signed", outlier_repr="bitmap",
              k_format="i2f4", use_pow2=True, kv_outlier_map=True, kv_int8_scale=True,
              group_tokens=32, group_channels=32, page_size=16, v_format="i2")


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

    index = {}
    for name in SEEDS:
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
    else:
        raise KeyError(name)
    return K.to(torch.bfloat16), V.to(torch.bfloat16)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
