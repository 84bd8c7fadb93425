"""HIP quantize-on-store against the reference packer's golden planes and the CPU oracle.
Bit-exact on every plane.  All calls go through the C ABI (ctypes)."""
import numpy as np
import pytest
import torch

import oracle.ommx_oracle as O
from conftest import (GOLDEN_CASES, PLANE_NAMES, VARIANT_CASES, assert_planes_equal,
                      assert_variant_planes_equal, bits_of, load_golden, load_variant,
                      tensor_from_bits)
from open_ommx_serve_amd.attention import pack as hip_pack
from open_ommx_serve_amd.attention.pack import (alloc_planes, ommx_pack_kv_canonical_block,
                                                store_pack_into)
from open_ommx_serve_amd.synth import synth_kv

pytestmark = pytest.mark.gpu

RECIPE = dict(outliers_per_vector=6, outlier_select="signed", outlier_repr="bitmap",
              k_format="i2f4", use_pow2=True, page_size=16)


def _hip(K, V, **kw):
    r = dict(RECIPE); r.update(kw)
    return ommx_pack_kv_canonical_block(K.cuda(), V.cuda(), **r)


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_store_matches_reference_golden_planes(name):
    z = load_golden(name)
    K, V = tensor_from_bits(z["K_bits"]), tensor_from_bits(z["V_bits"])
    planes = _hip(K, V)
    assert planes["k_base"].device.type == "cpu"            # default output device, like the reference
    assert_planes_equal(planes, z, what=name)
    for key in ("head_dim", "n_kv_heads", "num_tokens", "n_groups", "page_size",
                "outliers_per_vector", "outlier_repr", "outlier_select", "group_tokens",
                "group_channels", "k_format", "v_format", "k_base_bits", "oval_bits",
                "use_pow2", "kv_outlier_map", "kv_int8_scale", "k_field_bytes",
                "req_to_token", "req_to_group", "k_oidx", "k_crank"):
        assert key in planes
    assert planes["k_field_bytes"] == 4 and planes["k_oidx"] is None


@pytest.mark.parametrize("name", VARIANT_CASES)
def test_store_variant_matches_reference_golden_planes(name):
    """One block per format variant (index planes, base-shared outliers, magnitude selector,
    free and bf16 steps, 16/64/128-element vectors, bf16 V): every plane the reference packer
    wrote for it, bit for bit, and no plane it did not write."""
    z, recipe = load_variant(name)
    K, V = tensor_from_bits(z["K_bits"]), tensor_from_bits(z["V_bits"])
    planes = ommx_pack_kv_canonical_block(K.cuda(), V.cuda(), **recipe)
    assert_variant_planes_equal(planes, z, what=name)
    assert planes["outlier_repr"] == recipe["outlier_repr"]
    assert planes["group_tokens"] == recipe["group_tokens"]


@pytest.mark.parametrize("seed,T,H,D", [(1, 32, 1, 32), (2, 96, 3, 64), (3, 256, 8, 128),
                                        (4, 64, 2, 256), (5, 960, 8, 128)])
def test_store_matches_oracle_random_bf16(seed, T, H, D):
    K, V = synth_kv(T, H, D, seed, outlier_channels=min(4, D // 8), sparse_frac=0.01)
    assert_planes_equal(_hip(K, V), O.pack_kv(K, V), what=f"seed{seed}")


@pytest.mark.parametrize("k,T,H,D", [(6, 256, 8, 128), (6, 64, 2, 64), (1, 64, 2, 32), (3, 96, 1, 64),
                                     (5, 64, 2, 128), (8, 64, 2, 256)])
def test_store_relidx7_index_plane(k, T, H, D):
    """The 7-bit position-stream index plane (the reference packer's default ``outlier_repr``):
    bit-exact against the oracle, every other plane unchanged against the bitmap pack."""
    K, V = synth_kv(T, H, D, 300 + k, outlier_channels=min(4, D // 8), sparse_frac=0.01)
    want = O.pack_kv(K, V, outliers_per_vector=k, outlier_repr="relidx7")
    got = _hip(K, V, outliers_per_vector=k, outlier_repr="relidx7")
    assert got["k_obmp"] is None and got["outlier_repr"] == "relidx7" and got["k_field_bytes"] == 0
    assert tuple(got["k_oidx"].shape) == (T // 32, H, D, (7 * k + 7) // 8)
    for n in ("k_oidx", "k_base", "k_scale", "k_zp", "k_oval", "k_fp4_mapscale", "k_fp4_mapcenter",
              "v_main", "v_scale", "v_zp"):
        assert np.array_equal(bits_of(got[n]), bits_of(want[n])), n
    bm = _hip(K, V, outliers_per_vector=k)
    assert torch.equal(O.relidx7_unpack(got["k_oidx"], k), O.bitmap_unpack(bm["k_obmp"], k))


@pytest.mark.parametrize("k,T,H,D,rep", [(6, 256, 8, 128, "bitmap"), (6, 64, 2, 64, "relidx7"),
                                         (3, 96, 1, 64, "bitmap"), (8, 64, 2, 256, "bitmap")])
def test_store_base_shared_outliers(k, T, H, D, rep):
    """kv_outlier_map=False: the FP4 code of (w - zp) / scale, no map planes (pack.py:502-506)."""
    K, V = synth_kv(T, H, D, 400 + k, outlier_channels=min(4, D // 8), sparse_frac=0.01)
    want = O.pack_kv(K, V, outliers_per_vector=k, outlier_repr=rep, kv_outlier_map=False)
    got = _hip(K, V, outliers_per_vector=k, outlier_repr=rep, kv_outlier_map=False)
    assert got["k_fp4_mapscale"] is None and got["k_fp4_mapcenter"] is None and got["kv_outlier_map"] is False
    idx = "k_obmp" if rep == "bitmap" else "k_oidx"
    for n in (idx, "k_base", "k_scale", "k_zp", "k_oval", "v_main", "v_scale", "v_zp"):
        assert np.array_equal(bits_of(got[n]), bits_of(want[n])), n
    # the nibbles differ from the dedicated-map pack of the same block: it is another code
    assert not np.array_equal(bits_of(got["k_oval"]), bits_of(_hip(K, V, outliers_per_vector=k)["k_oval"]))


@pytest.mark.parametrize("k,T,H,D", [(6, 256, 8, 128), (3, 64, 2, 64), (1, 64, 1, 32), (8, 64, 2, 256)])
def test_store_abs_selection(k, T, H, D):
    """outlier_select="abs" (the reference packer's default argument): the k largest magnitudes.
    Includes a block of heavy ties between values of both signs."""
    K, V = synth_kv(T, H, D, 500 + k, outlier_channels=min(4, D // 8), sparse_frac=0.01)
    g = torch.Generator().manual_seed(k)
    lv = torch.tensor([-3.0, -1.0, 1.0, 0.0, -0.0, 0.5, -0.5, 2.0, -2.0, 3.0])
    K[:32] = lv[torch.randint(0, 10, (32, H, D), generator=g)].to(torch.bfloat16)
    want = O.pack_kv(K, V, outliers_per_vector=k, outlier_select="abs")
    got = _hip(K, V, outliers_per_vector=k, outlier_select="abs")
    assert got["outlier_select"] == "abs"
    assert_planes_equal(got, want, what=f"abs k{k}", zero_sign_free=True)


@pytest.mark.parametrize("kw", [dict(use_pow2=False), dict(use_pow2=True, kv_int8_scale=False),
                                dict(use_pow2=False, kv_outlier_map=False, outlier_repr="relidx7"),
                                dict(use_pow2=False, outlier_select="abs", outliers_per_vector=3)])
@pytest.mark.parametrize("T,H,D", [(256, 8, 128), (64, 2, 64)])
def test_store_bf16_step_planes(kw, T, H, D):
    """use_pow2=False (the step bf16((max - min) / 3) as it comes: true division for the codes)
    and kv_int8_scale=False (power-of-two steps stored as bf16): bit-exact against the oracle.
    The last two rows are the reference packer's default arguments but for the outlier count
    / selection: relidx7, abs, no power-of-two rounding."""
    K, V = synth_kv(T, H, D, 600 + T, outlier_channels=min(4, D // 8), sparse_frac=0.01)
    args = dict(outliers_per_vector=6, outlier_repr="bitmap", outlier_select="signed")
    args.update(kw)
    want = O.pack_kv(K, V, **args)
    got = _hip(K, V, **args)
    assert got["k_scale"].dtype == torch.bfloat16 and got["v_scale"].dtype == torch.bfloat16
    assert got["kv_int8_scale"] is False and got["use_pow2"] is bool(args.get("use_pow2", True))
    names = ["k_base", "k_scale", "k_zp", "k_oval", "v_main", "v_scale", "v_zp",
             "k_oidx" if args["outlier_repr"] == "relidx7" else "k_obmp"]
    if args.get("kv_outlier_map", True):
        names += ["k_fp4_mapscale", "k_fp4_mapcenter"]
    for n in names:
        assert np.array_equal(bits_of(got[n]), bits_of(want[n])), n


def test_store_reference_default_arguments():
    """ommx_pack_kv_canonical_block(K, V) with nothing else: 3 outliers by magnitude, relidx7,
    plain bf16 steps, dedicated map (pack.py:293-309)."""
    K, V = synth_kv(128, 4, 128, 77, sparse_frac=0.01)
    got = ommx_pack_kv_canonical_block(K.cuda(), V.cuda())
    want = O.pack_kv(K, V, outliers_per_vector=3, outlier_repr="relidx7", outlier_select="abs",
                     use_pow2=False)
    assert (got["outliers_per_vector"], got["outlier_repr"], got["outlier_select"], got["use_pow2"]) == \
        (3, "relidx7", "abs", False)
    for n in ("k_base", "k_scale", "k_zp", "k_oidx", "k_oval", "k_fp4_mapscale", "k_fp4_mapcenter",
              "v_main", "v_scale", "v_zp"):
        assert np.array_equal(bits_of(got[n]), bits_of(want[n])), n


GROUP_RECIPES = [
    # the two other named recipes of the reference: "low-bit lever" and "paper-kv"
    dict(group_tokens=64, group_channels=64, outliers_per_vector=6, outlier_repr="relidx7", kv_outlier_map=False),
    dict(group_tokens=128, group_channels=128, outliers_per_vector=10, outlier_repr="relidx7"),
    dict(group_tokens=128, group_channels=32, outliers_per_vector=8, outlier_repr="bitmap"),
    dict(group_tokens=16, group_channels=16, outliers_per_vector=3, outlier_repr="bitmap"),
    dict(group_tokens=64, group_channels=128, outliers_per_vector=16, outlier_repr="bitmap", outlier_select="abs"),
    dict(group_tokens=16, group_channels=64, outliers_per_vector=2, outlier_repr="relidx7", use_pow2=False),
    dict(group_tokens=32, group_channels=32, outliers_per_vector=12, outlier_repr="relidx7"),
    dict(group_tokens=64, group_channels=64, outliers_per_vector=0),
]


@pytest.mark.parametrize("recipe", GROUP_RECIPES)
@pytest.mark.parametrize("T,H,D,fp32", [(256, 8, 128, False), (128, 2, 256, True)])
def test_store_other_group_sizes(recipe, T, H, D, fp32):
    """K vectors of 16 / 64 / 128 tokens, V vectors of 16 / 64 / 128 channels, up to 16 outliers,
    multi-word bitmaps and position streams: bit-exact against the oracle on every plane."""
    K, V = synth_kv(T, H, D, 700 + T, outlier_channels=4, sparse_frac=0.01)
    if fp32:
        K, V = K.float() * 1.0009765625, V.float() * 0.99951171875       # leave the bf16 grid
    args = dict(outlier_repr="bitmap", outlier_select="signed")
    args.update(recipe)
    want = O.pack_kv(K, V, **args)
    got = _hip(K, V, **args)
    gt, gc, k = args["group_tokens"], args["group_channels"], args["outliers_per_vector"]
    assert (got["group_tokens"], got["group_channels"], got["n_groups"]) == (gt, gc, T // gt)
    names = ["k_base", "k_scale", "k_zp", "v_main", "v_scale", "v_zp"]
    if k > 0:
        names += ["k_oval", "k_oidx" if args["outlier_repr"] == "relidx7" else "k_obmp"]
        if args.get("kv_outlier_map", True):
            names += ["k_fp4_mapscale", "k_fp4_mapcenter"]
    for n in names:
        assert got[n].shape == want[n].shape, n
        assert np.array_equal(bits_of(got[n]), bits_of(want[n])), n
    assert got["k_field_bytes"] == want["k_field_bytes"]


@pytest.mark.parametrize("kw", [dict(), dict(group_tokens=64, group_channels=64, outlier_repr="relidx7"),
                                dict(use_pow2=False)])
@pytest.mark.parametrize("fp32", [False, True])
def test_store_bf16_v_rows(kw, fp32):
    """v_format="bf16" (pack.py:596-602): V is kept as bf16 rows [pages, ps, H, D], the step planes
    are ones and zeros; K is packed as usual."""
    K, V = synth_kv(128, 4, 128, 900, sparse_frac=0.01)
    if fp32:
        K, V = K.float() * 1.0009765625, V.float() * 0.99951171875
    args = dict(outliers_per_vector=6, outlier_repr="bitmap", outlier_select="signed", v_format="bf16")
    args.update(kw)
    want = O.pack_kv(K, V, **args)
    got = _hip(K, V, **args)
    assert got["v_format"] == "bf16" and got["v_main"].dtype == torch.bfloat16
    assert tuple(got["v_main"].shape) == (8, 16, 4, 128)
    for n in ("v_main", "v_scale", "v_zp", "k_base", "k_scale", "k_zp", "k_oval",
              "k_oidx" if args["outlier_repr"] == "relidx7" else "k_obmp", "k_fp4_mapscale", "k_fp4_mapcenter"):
        assert got[n].dtype == want[n].dtype and got[n].shape == want[n].shape, n
        assert np.array_equal(bits_of(got[n]), bits_of(want[n])), n


def test_store_randomised_recipes():
    """Sixty random draws over the recipe space (group sizes, outlier count / selection / index
    plane / map, step mode, V format, page size, head shapes, input dtype, value patterns with
    ties): every plane bit for bit against the oracle."""
    g = torch.Generator().manual_seed(77)

    def pick(*xs):
        return xs[int(torch.randint(0, len(xs), (1,), generator=g))]

    for it in range(60):
        gt, gc = pick(16, 32, 64, 128), pick(16, 32, 64, 128)
        D = pick(32, 64, 128, 256)
        gc = min(gc, D)
        H = pick(1, 2, 5, 8)
        ps = pick(8, 16, 32)
        T = gt * pick(1, 2, 5)
        while T % ps:
            T += gt
        rep = pick("bitmap", "relidx7")
        k = min(pick(0, 1, 2, 3, 6, 7, 8, 11, 16), gt)
        recipe = dict(group_tokens=gt, group_channels=gc, outliers_per_vector=k, outlier_repr=rep,
                      outlier_select=pick("signed", "abs"), kv_outlier_map=pick(True, False),
                      use_pow2=pick(True, False), kv_int8_scale=pick(True, False),
                      v_format=pick("i2", "i2", "bf16"), page_size=ps)
        K, V = synth_kv(T, H, D, 4000 + it, outlier_channels=min(4, D // 8), sparse_frac=pick(0.0, 0.02))
        if pick(0, 1, 2) == 0:                      # a block of heavy ties between values of both signs
            lv = torch.tensor([-3.0, -1.0, 1.0, 0.5, -0.5, 2.0, -2.0, 3.0, 0.25])
            n = min(T, 2 * gt)
            K[:n] = lv[torch.randint(0, 9, (n, H, D), generator=g)].to(torch.bfloat16)
            V[:n] = lv[torch.randint(0, 9, (n, H, D), generator=g)].to(torch.bfloat16)
        if pick(0, 1):
            K, V = K.float() * 1.0009765625, V.float() * 0.99951171875
        what = f"case {it}: T={T} H={H} D={D} {K.dtype} {recipe}"
        want = O.pack_kv(K, V, **recipe)
        got = _hip(K, V, **recipe)
        for n in ("k_base", "k_scale", "k_zp", "k_obmp", "k_oidx", "k_oval", "k_fp4_mapscale",
                  "k_fp4_mapcenter", "v_main", "v_scale", "v_zp"):
            if want[n] is None:
                assert got[n] is None, (what, n)
                continue
            assert got[n].dtype == want[n].dtype and got[n].shape == want[n].shape, (what, n)
            a, b = bits_of(got[n]), bits_of(want[n])
            if n in ("k_zp", "k_fp4_mapcenter", "v_zp"):        # the sign of a zero is free (conftest)
                a, b = np.where(a == 0x8000, 0, a), np.where(b == 0x8000, 0, b)
            assert np.array_equal(a, b), f"{what}: plane {n}"


@pytest.mark.parametrize("k", [0, 1, 2, 5, 8])
def test_store_other_outlier_counts(k):
    K, V = synth_kv(128, 2, 64, 10 + k)
    want = O.pack_kv(K, V, outliers_per_vector=k)
    got = _hip(K, V, outliers_per_vector=k)
    names = PLANE_NAMES if k > 0 else ("k_base", "k_scale", "k_zp", "v_main", "v_scale", "v_zp")
    for n in names:
        assert np.array_equal(bits_of(got[n]), bits_of(want[n])), n
    if k == 0:
        assert got["k_obmp"] is None and got["k_oval"] is None and got["kv_outlier_map"] is False


def test_store_heavy_ties_and_degenerate_vectors():
    g = torch.Generator().manual_seed(77)
    lv = torch.tensor([-4.0, -1.0, -1.0, 0.0, 0.0, 0.0, 0.25, 2.0, 2.0, 8.0])
    K = lv[torch.randint(0, 10, (128, 2, 64), generator=g)].to(torch.bfloat16)
    V = lv[torch.randint(0, 10, (128, 2, 64), generator=g)].to(torch.bfloat16)
    K[:32, 0, 0] = 3.0            # constant K vector: every range clamps to 1e-8
    V[0, 0, :32] = -7.0           # constant V vector
    K[32:64, 1, 5] = 0.0
    assert_planes_equal(_hip(K, V), O.pack_kv(K, V), what="ties")


def test_store_huge_constant_vectors_take_the_two_step_code_path():
    """The INT2 codes come from one fused multiply-add w * 2^-e - zp * 2^-e; a constant vector of huge
    values has a tiny step (the 1e-8 range floor) and a zero point whose scaled value overflows, so the
    kernel must fall back to (w - zp) * 2^-e there: K at the selector's limit, V at the end of bf16."""
    K, V = synth_kv(128, 2, 128, 31, sparse_frac=0.01)
    K[:32, 0, 3] = 9.0e8
    K[32:64, 1, 7] = -9.0e8
    V[5, 0, :32] = 3.0e38
    V[6, 1, 32:64] = -3.0e38
    V[7, 0, 64:96] = torch.linspace(1.0e38, 3.0e38, 32).to(torch.bfloat16)
    for fp32 in (False, True):
        Kx, Vx = (K.float(), V.float()) if fp32 else (K, V)
        assert_planes_equal(_hip(Kx, Vx), O.pack_kv(Kx, Vx), what=f"huge fp32={fp32}")


def test_store_fp32_inputs_round_zero_point_and_map():
    g = torch.Generator().manual_seed(9)
    K = torch.randn(128, 2, 64, generator=g) * 3.0
    V = torch.randn(128, 2, 64, generator=g) * torch.exp2(torch.randint(-10, 8, (128, 2, 1), generator=g).float())
    assert_planes_equal(_hip(K, V), O.pack_kv(K, V), what="fp32")


def test_store_scale_rounding_points_across_binades():
    """Vectors whose range/3 sits within a few ulps of sqrt(2)*2^n, where the reference's fp32
    log2 decides the exponent: the kernel has to take the same side for every n."""
    rows = []
    for n in range(-20, 12):
        c = torch.tensor([3.0 * 2.0 ** (n + 0.5)], dtype=torch.float32)
        rows.append((c.view(torch.int32) + torch.arange(-16, 16, dtype=torch.int32)).view(torch.float32))
    m = torch.stack(rows)                                    # [32 binades, 32 neighbours]
    ramp = torch.arange(32, dtype=torch.float32) / 31.0
    # V: token t = (binade), channel group j = neighbour  -> vector = m[t, j] * ramp
    V = (m.unsqueeze(-1) * ramp).reshape(32, 1, 32 * 32)[:, :, :256].contiguous()
    V = torch.cat([V, (m[:, 8:16].unsqueeze(-1) * ramp).reshape(32, 1, 256)], 1)
    K = V.clone()
    got = _hip(K, V, outliers_per_vector=0)
    want = O.pack_kv(K, V, outliers_per_vector=0)
    for nme in ("k_base", "k_scale", "k_zp", "v_main", "v_scale", "v_zp"):
        assert np.array_equal(bits_of(got[nme]), bits_of(want[nme])), nme


def test_store_fp4_rounding_points():
    """Outliers whose mapped value sits within a few ulps of an FP4 level boundary."""
    bounds = [7.0710678e-05, 0.70710678, 1.2247449, 1.7320508, 2.4494897, 3.4641016, 4.8989795]
    K = torch.zeros(32, 1, 256)
    g = torch.Generator().manual_seed(3)
    K[:] = torch.randn(32, 1, 256, generator=g) * 0.01
    col = 0
    for b in bounds:
        c = torch.tensor([b], dtype=torch.float32)
        for step in range(-18, 18):
            x = (c.view(torch.int32) + step).view(torch.float32).item()
            # outliers +6-ish top and -6 bottom fix the map to centre 0, scale 1
            K[0, 0, col], K[1, 0, col], K[2, 0, col] = 6.0, 5.0, x if x > 0.05 else 5.5
            K[3, 0, col], K[4, 0, col], K[5, 0, col] = -6.0, -5.0, -x if x > 0.05 else -5.5
            col += 1
            if col == 256:
                break
        if col == 256:
            break
    V = torch.randn(32, 1, 256, generator=g)
    assert_planes_equal(_hip(K, V), O.pack_kv(K, V), what="fp4-bounds")


def test_store_into_pool_with_tables_and_ring_gather():
    """Pages and group slots chosen by tables, source rows gathered from a shuffled ring."""
    T, H, D, ps = 128, 2, 64, 16
    K, V = synth_kv(T, H, D, 21)
    want = O.pack_kv(K, V)
    g = torch.Generator().manual_seed(4)
    perm = torch.randperm(T, generator=g)
    ringK = torch.empty(T + 5, H, D, dtype=torch.bfloat16); ringV = torch.empty_like(ringK)
    ringK[perm] = K; ringV[perm] = V                               # token t lives in ring row perm[t]
    pool_pages, pool_groups = 20, 9
    planes = alloc_planes(pool_pages, pool_groups, H, D, page_size=ps, device="cuda")
    for t in planes.values():
        if torch.is_tensor(t):
            t.fill_(0x5A if t.dtype == torch.uint8 else 1)
    pages = torch.randperm(pool_pages, generator=g)[:T // ps].to(torch.int32)
    groups = torch.randperm(pool_groups, generator=g)[:T // 32].to(torch.int32)
    err = torch.zeros(1, dtype=torch.int32, device="cuda")
    store_pack_into(ringK.cuda(), ringV.cuda(), planes, page_size=ps,
                    src_rows=perm.to(torch.int32).cuda(), dst_pages=pages.cuda(),
                    dst_groups=groups.cuda(), err_flag=err)
    assert int(err.item()) == 0
    for n in ("k_base", "v_main", "v_scale", "v_zp"):
        assert np.array_equal(bits_of(planes[n][pages.long().cuda()]), bits_of(want[n])), n
        untouched = torch.ones(pool_pages, dtype=torch.bool); untouched[pages.long()] = False
        ref = torch.full_like(planes[n][untouched.cuda()].cpu(), 0x5A if planes[n].dtype == torch.uint8 else 1)
        assert torch.equal(planes[n][untouched.cuda()].cpu(), ref), f"{n}: a foreign page was written"
    for n in ("k_scale", "k_zp", "k_obmp", "k_oval", "k_fp4_mapscale", "k_fp4_mapcenter"):
        assert np.array_equal(bits_of(planes[n][groups.long().cuda()]), bits_of(want[n])), n


def test_store_page_sizes():
    K, V = synth_kv(64, 2, 64, 31)
    for ps in (8, 16, 32):
        assert_planes_equal(_hip(K, V, page_size=ps), O.pack_kv(K, V, page_size=ps), what=f"ps{ps}")


def test_store_refuses_nonfinite_and_bad_arguments():
    K, V = synth_kv(64, 1, 64, 41)
    Kb = K.clone(); Kb[3, 0, 5] = float("inf")
    with pytest.raises((ValueError, IndexError)):
        _hip(Kb, V)
    Kn = K.clone(); Kn[:, 0, 7] = float("nan")
    with pytest.raises((ValueError, IndexError)):
        _hip(Kn, V)
    Vb = V.clone(); Vb[0, 0, 0] = float("nan")
    with pytest.raises(ValueError):
        _hip(K, Vb)
    with pytest.raises(ValueError):
        _hip(K[:48], V[:48])                       # not a multiple of 32
    with pytest.raises(ValueError):
        _hip(K, V[:32])
    with pytest.raises(ValueError):
        _hip(K, V, outlier_repr="nope")
    with pytest.raises(ValueError):
        _hip(K, V, outliers_per_vector=33)
    with pytest.raises(NotImplementedError):
        _hip(K, V, outliers_per_vector=17, outlier_repr="relidx7")
    _hip(K, V)                                     # and a good call still works afterwards


def test_store_prefill_sized_block_is_bit_exact():
    """4032 tokens of the 8-head, 128-channel layer (the store of the ctx-4096 case)."""
    K, V = synth_kv(4032, 8, 128, 42, sparse_frac=0.005)
    assert_planes_equal(_hip(K, V), O.pack_kv(K, V), what="ctx4096")


def test_store_bulk_32k_block_is_bit_exact_in_every_group():
    """32704 tokens of the 8-head layer (the bulk prefill store of the batch-8 / ctx-32768 case): all ten
    planes of all 1022 groups x 8 heads are held against the oracle packer, which packs the block in
    pieces of 128 groups (groups are packed independently, reference kv_pool.py:563-566); every frame
    holds exactly 6 outliers."""
    T, H, D = 32704, 8, 128
    K, V = synth_kv(T, H, D, 43, sparse_frac=0.005)
    planes = _hip(K, V, device="cuda")
    bm = planes["k_obmp"].view(torch.int32).reshape(-1)
    pop = torch.zeros_like(bm)
    for i in range(32):
        pop += (bm >> i) & 1
    assert bool((pop == 6).all())
    got = {n: planes[n].cpu() for n in PLANE_NAMES}
    step = 4096                                   # tokens per oracle call: 128 groups, 256 pages
    for t0 in range(0, T, step):
        t1 = min(t0 + step, T)
        want = O.pack_kv(K[t0:t1], V[t0:t1])
        g0, g1, p0, p1 = t0 // 32, t1 // 32, t0 // 16, t1 // 16
        for n in ("k_scale", "k_zp", "k_obmp", "k_oval", "k_fp4_mapscale", "k_fp4_mapcenter"):
            assert np.array_equal(bits_of(got[n][g0:g1]), bits_of(want[n])), (n, t0)
        for n in ("k_base", "v_main", "v_scale", "v_zp"):
            assert np.array_equal(bits_of(got[n][p0:p1]), bits_of(want[n])), (n, t0)


def test_decision_table_measured_on_this_host_is_monotone_and_near_the_exact_one():
    t = hip_pack.measure_store_table()
    d = torch.zeros(264)
    from open_ommx_serve_amd.attention import _hip as H
    H.load().ommx_store_default_table(d.data_ptr())
    ulps = (t[88:254].view(torch.int32) - d[88:254].view(torch.int32)).abs()
    assert int(ulps.max()) <= 64
    assert bool((t[257:264][1:] > t[257:264][:-1]).all())


def test_store_replayed_from_a_hip_graph():
    """The store launch neither allocates nor synchronises: captured once, replayed on new rows
    (three replays with eager work between them), each time equal to the oracle's planes."""
    T, H, D = 128, 2, 128
    store_table_ready = hip_pack.store_table(torch.device("cuda"))     # upload outside the capture
    assert store_table_ready.numel() == 264
    K = torch.zeros(T, H, D, dtype=torch.bfloat16, device="cuda")
    V = torch.zeros_like(K)
    planes = alloc_planes(T // 16, T // 32, H, D, device="cuda")
    err = torch.zeros(1, dtype=torch.int32, device="cuda")
    K0, V0 = synth_kv(T, H, D, seed=90)
    K.copy_(K0)
    V.copy_(V0)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            store_pack_into(K, V, planes, err_flag=err)
    torch.cuda.current_stream().wait_stream(stream)
    for rep in range(3):
        Kr, Vr = synth_kv(T, H, D, seed=91 + rep, sparse_frac=0.01)
        K.copy_(Kr)
        V.copy_(Vr)
        graph.replay()
        torch.cuda.synchronize()
        assert int(err.item()) == 0
        want = O.pack_kv(Kr, Vr)
        for name in PLANE_NAMES:
            assert torch.equal(planes[name].cpu().view(torch.uint8), want[name].view(torch.uint8)), (rep, name)
        (K.float().sum() + V.float().sum()).item()                      # eager work between replays


def test_store_randomised_tie_patterns_signed_zeros_and_extremes():
    """Thirty random blocks drawn from small value sets (so that ties reach into the chosen
    lanes in every pattern), with signed zeros, bf16 denormals, huge magnitudes and vectors that
    are constant or constant but for one to five lanes; bf16 and fp32 input; bit-exact."""
    g = torch.Generator().manual_seed(31337)

    def rnd(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    pools = [
        torch.tensor([-0.0, 0.0, 1.0, -1.0]),
        torch.tensor([-0.0, 0.0]),
        torch.tensor([3.0, 3.0, 3.0, 3.0, 3.0, -2.0, 7.0]),
        torch.tensor([9.1835e-41, -9.1835e-41, 0.0, 1e-38, -1e-38]),          # bf16 denormals
        torch.tensor([1e30, -1e30, 5e8, 2e9, -3e9, 1.0]),
        torch.tensor([-4.0, -1.0, -1.0, 0.0, 0.0, 0.25, 2.0, 2.0, 8.0, 8.0, 8.0]),
        torch.arange(-16, 17).float() * 0.5,
    ]
    for it in range(30):
        H, D, T = (1, 2, 8)[rnd(0, 2)], (32, 64, 128)[rnd(0, 2)], 32 * rnd(1, 4)
        pk = pools[rnd(0, len(pools) - 1)]
        pv = pools[rnd(0, len(pools) - 1)]
        K = pk[torch.randint(0, len(pk), (T, H, D), generator=g)]
        V = pv[torch.randint(0, len(pv), (T, H, D), generator=g)]
        # a few vectors that are constant but for n lanes
        for _ in range(4):
            h, d, n = rnd(0, H - 1), rnd(0, D - 1), rnd(0, 5)
            K[:32, h, d] = float(pk[0])
            for i in torch.randperm(32, generator=g)[:n].tolist():
                K[i, h, d] = float(pk[rnd(0, len(pk) - 1)]) + 1.0
        if rnd(0, 1):
            K, V = K.to(torch.bfloat16), V.to(torch.bfloat16)
        what = f"random block {it} {tuple(K.shape)} {K.dtype}"
        try:
            want = O.pack_kv(K, V)
        except (IndexError, ValueError) as exc:
            # magnitudes of 1e9 and more defeat the +1e9 sentinel of the selector: the
            # reference refuses such a block, and so must the store
            with pytest.raises(type(exc)):
                _hip(K, V)
            continue
        assert_planes_equal(_hip(K, V), want, what=what, zero_sign_free=True)
