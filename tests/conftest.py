"""Shared fixtures.  Tests marked ``gpu`` need one ROCm GPU; the rest run on the CPU."""
import json
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")
PLANE_NAMES = ("k_base", "k_scale", "k_zp", "k_obmp", "k_oval", "k_fp4_mapscale",
               "k_fp4_mapcenter", "v_main", "v_scale", "v_zp")
GOLDEN_CASES = ("tiny_ties", "small_gauss", "layer_outliers", "wide_range", "fp32_inputs",
                "map_scale_rounding")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for it in items:
        if "gpu" in it.keywords:
            it.add_marker(skip)


def tensor_from_bits(a: np.ndarray) -> torch.Tensor:
    """Inverse of the fixture writer: uint16 -> bf16, uint32 -> fp32, else as stored."""
    t = torch.from_numpy(a.copy())
    if a.dtype == np.uint16:
        return t.view(torch.int16).view(torch.bfloat16)
    if a.dtype == np.uint32:
        return t.view(torch.int32).view(torch.float32)
    return t


def bits_of(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy().view(np.uint32)
    return t.numpy()


def load_golden(name: str):
    z = np.load(os.path.join(GOLDEN_DIR, f"pack_{name}.npz"))
    return {k: z[k] for k in z.files}


ZERO_SIGN_FREE = ("k_zp", "v_zp", "k_fp4_mapcenter")


def assert_planes_equal(got, want_bits, what="", zero_sign_free=False):
    """Bit-exact comparison of a plane dict against raw golden arrays (or another dict).

    ``zero_sign_free``: a zero point or map centre that is a zero may differ in sign.  Which
    of -0 / +0 a minimum over mixed-sign zeros returns is not defined by the reference (its
    vectorised reduction keeps one or the other depending on lane order and vector width);
    the device kernel always returns -0.  Both stand for the same number everywhere downstream.
    """
    for name in PLANE_NAMES:
        w = want_bits[name]
        if torch.is_tensor(w):
            w = bits_of(w)
        g = bits_of(got[name])
        assert g.shape == w.shape, f"{what} {name}: shape {g.shape} != {w.shape}"
        if zero_sign_free and name in ZERO_SIGN_FREE:
            g = np.where(g == 0x8000, 0, g)
            w = np.where(w == 0x8000, 0, w)
        bad = int((g != w).sum())
        assert bad == 0, f"{what} {name}: {bad} of {g.size} elements differ"


# ---- one reference-written block per format variant (tests/golden/variant_*.npz) --------

with open(os.path.join(GOLDEN_DIR, "variant_index.json")) as _f:
    VARIANT_INDEX = json.load(_f)
VARIANT_CASES = tuple(VARIANT_INDEX)
ALL_PLANE_NAMES = PLANE_NAMES + ("k_oidx", "k_crank")


def load_variant(name: str):
    """``(arrays, recipe)`` of a variant fixture: raw plane bits plus the keyword arguments
    the reference packer was called with."""
    z = np.load(os.path.join(GOLDEN_DIR, f"variant_{name}.npz"))
    return {k: z[k] for k in z.files}, dict(VARIANT_INDEX[name]["recipe"])


def variant_planes(z, recipe):
    """Plane dict (tensors + the metadata keys a dequant needs) of a variant fixture."""
    planes = {p: (tensor_from_bits(z[p]) if p in z else None) for p in ALL_PLANE_NAMES}
    planes.update(outliers_per_vector=recipe["outliers_per_vector"],
                  group_tokens=recipe["group_tokens"], group_channels=recipe["group_channels"],
                  outlier_repr=recipe["outlier_repr"], page_size=recipe["page_size"])
    return planes


def assert_variant_planes_equal(got, z, what=""):
    """Every plane the reference wrote is matched bit for bit (dtype included); every plane it
    left out must be absent from ``got`` as well."""
    for name in ALL_PLANE_NAMES:
        g = got.get(name)
        if name not in z:
            assert g is None, f"{what} {name}: reference wrote no such plane"
            continue
        assert g is not None, f"{what} {name}: plane missing"
        want_dtype = VARIANT_INDEX[what]["planes"][name][0] if what in VARIANT_INDEX else None
        if want_dtype:
            assert str(g.dtype).replace("torch.", "") == want_dtype, f"{what} {name}: dtype {g.dtype}"
        gb, w = bits_of(g), z[name]
        assert gb.shape == w.shape, f"{what} {name}: shape {gb.shape} != {w.shape}"
        bad = int((gb != w).sum())
        assert bad == 0, f"{what} {name}: {bad} of {gb.size} elements differ"
