"""Pins of the CPU oracle: golden planes from the reference packer, closed forms, invariants
and brute force.  Each check is chosen so that a plausible slip in the oracle (wrong tie
order, wrong rounding, transposed index, dropped term) fails it.  Runs on the CPU."""
import math

import numpy as np
import pytest
import torch

import oracle.ommx_oracle as O
from conftest import (GOLDEN_CASES, VARIANT_CASES, assert_planes_equal,
                      assert_variant_planes_equal, bits_of, load_golden, load_variant,
                      tensor_from_bits, variant_planes)


# ---- the composed packer against the reference's own output ---------------------------

@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_pack_matches_reference_golden_planes(name):
    z = load_golden(name)
    K, V = tensor_from_bits(z["K_bits"]), tensor_from_bits(z["V_bits"])
    planes = O.pack_kv(K, V, page_size=16, outliers_per_vector=6)
    assert_planes_equal(planes, z, what=name)


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_dequant_matches_reference_golden(name):
    z = load_golden(name)
    planes = {k: tensor_from_bits(z[k]) for k in z if not k.endswith("_bits")}
    planes["outliers_per_vector"] = 6
    Kd, Vd = O.dequant_kv(planes)
    assert np.array_equal(bits_of(Kd), z["K_dq_bits"])
    assert np.array_equal(bits_of(Vd), z["V_dq_bits"])


def _oracle_kwargs(recipe):
    kw = dict(recipe)
    assert kw.pop("k_format") == "i2f4"
    return kw


@pytest.mark.parametrize("name", VARIANT_CASES)
def test_pack_variant_matches_reference_golden_planes(name):
    """Each format variant's branch of the packer, against planes the reference packer wrote
    for the same block with the same keyword arguments."""
    z, recipe = load_variant(name)
    K, V = tensor_from_bits(z["K_bits"]), tensor_from_bits(z["V_bits"])
    planes = O.pack_kv(K, V, **_oracle_kwargs(recipe))
    assert_variant_planes_equal(planes, z, what=name)


@pytest.mark.parametrize("name", VARIANT_CASES)
def test_dequant_variant_matches_reference_golden(name):
    z, recipe = load_variant(name)
    Kd, Vd = O.dequant_kv(variant_planes(z, recipe))
    assert np.array_equal(bits_of(Kd), z["K_dq_bits"])
    assert np.array_equal(bits_of(Vd), z["V_dq_bits"])


def test_gather_through_identity_tables_equals_linear_dequant():
    z = load_golden("layer_outliers")
    planes = {k: tensor_from_bits(z[k]) for k in z if not k.endswith("_bits")}
    planes["outliers_per_vector"] = 6
    Kd, Vd = O.dequant_kv(planes)
    T = Kd.shape[0]
    Kg, Vg = O.gather_request(planes, torch.arange(T // 16), torch.arange(T // 32), T, page_size=16)
    assert torch.equal(Kg, Kd) and torch.equal(Vg, Vd)
    # a shorter request sees a prefix
    Kg2, _ = O.gather_request(planes, torch.arange(T // 16), torch.arange(T // 32), 64, page_size=16)
    assert torch.equal(Kg2, Kd[:64])


def test_gather_through_permuted_tables():
    """Move pages and group slots around physically; the logical rows must not change."""
    z = load_golden("layer_outliers")
    planes = {k: tensor_from_bits(z[k]) for k in z if not k.endswith("_bits")}
    planes["outliers_per_vector"] = 6
    Kd, Vd = O.dequant_kv(planes)
    T, P, G = Kd.shape[0], Kd.shape[0] // 16, Kd.shape[0] // 32
    g = torch.Generator().manual_seed(3)
    pp, gp = torch.randperm(P, generator=g), torch.randperm(G, generator=g)
    moved = dict(planes)
    for n in ("k_base", "v_main", "v_scale", "v_zp"):
        t = torch.empty_like(planes[n]); t[pp] = planes[n]; moved[n] = t
    for n in ("k_scale", "k_zp", "k_obmp", "k_oval", "k_fp4_mapscale", "k_fp4_mapcenter"):
        t = torch.empty_like(planes[n]); t[gp] = planes[n]; moved[n] = t
    Kg, Vg = O.gather_request(moved, pp, gp, T, page_size=16)
    assert torch.equal(Kg, Kd) and torch.equal(Vg, Vd)


# ---- FP4 codec --------------------------------------------------------------------------

def test_fp4_levels_are_fixed_points_and_codes_cover_the_table():
    lv = torch.tensor(O.FP4_LEVELS)
    x = torch.cat([lv, -lv])
    assert torch.equal(O.fp4_decode(O.fp4_encode(x)), x)        # -0.0 == 0.0 under torch.equal
    codes = torch.arange(16, dtype=torch.uint8)
    want = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6])
    assert torch.equal(O.fp4_decode(codes), want)
    # sign bit follows x < 0 even when the level is 0; +-0 give code 0
    assert O.fp4_encode(torch.tensor([-1e-9, 0.0, -0.0])).tolist() == [8, 0, 0]


def test_fp4_encode_is_nearest_in_log_with_ties_down():
    """Brute force in float64 away from the boundaries; exact geometric means go down."""
    g = torch.Generator().manual_seed(5)
    x = torch.exp(torch.rand(20000, generator=g) * 14 - 11)         # 1.7e-5 .. 20
    lv = np.array([1e-8, .5, 1, 1.5, 2, 3, 4, 6])
    d = np.abs(np.log(x.double().numpy())[:, None] - np.log(lv)[None, :])
    srt = np.sort(d, axis=1)
    clear = (srt[:, 1] - srt[:, 0]) > 1e-4                           # not within fp32 noise of a tie
    want = d.argmin(1)
    got = (O.fp4_encode(x).to(torch.int64) & 7).numpy()
    assert clear.sum() > 19000 and np.array_equal(got[clear], want[clear])
    assert O.fp4_encode(torch.tensor([100.0, 6.0, 4.9, 4.89, 2.0])).tolist() == [7, 7, 7, 6, 4]


def test_fp4_encode_monotone_over_all_floats_near_boundaries():
    for lo, hi in zip(O.FP4_LEVELS[1:-1], O.FP4_LEVELS[2:]):
        c = torch.tensor([math.sqrt(lo * hi)], dtype=torch.float32)
        win = (c.view(torch.int32) + torch.arange(-200, 201, dtype=torch.int32)).view(torch.float32)
        idx = (O.fp4_encode(win).to(torch.int64) & 7)
        assert bool((idx[1:] >= idx[:-1]).all()) and idx[0] != idx[-1]


# ---- bit layouts ------------------------------------------------------------------------

def test_int2_layout_closed_form_and_round_trip():
    codes = torch.tensor([[1, 2, 3, 0, 3, 3, 0, 1]])
    plane = O.pack_int2(codes)
    assert plane.tolist() == [[1 | 2 << 2 | 3 << 4 | 0 << 6, 3 | 3 << 2 | 0 << 4 | 1 << 6]]
    g = torch.Generator().manual_seed(1)
    c = torch.randint(0, 4, (7, 3, 64), generator=g)
    assert torch.equal(O.unpack_int2(O.pack_int2(c)), c)


def test_bitmap_layout_popcount_and_rank_rule():
    pos = torch.tensor([[0, 7, 8, 15, 30, 31]])
    bm = O.bitmap_pack(pos)
    assert bm.tolist() == [[0x81, 0x81, 0x00, 0xC0]]
    word = int.from_bytes(bytes(bm[0].tolist()), "little")
    assert bin(word).count("1") == 6 and word >> 32 == 0
    # nibble ordinal of a set bit == popcount of the lower set bits
    for s, p in enumerate(pos[0].tolist()):
        assert bin(word & ((1 << p) - 1)).count("1") == s
    assert torch.equal(O.bitmap_unpack(bm, 6), pos)
    with pytest.raises(ValueError):
        O.bitmap_pack(torch.tensor([[1, 1, 2, 3, 4, 5]]))
    with pytest.raises(ValueError):
        O.bitmap_pack(torch.tensor([[1, 2, 3, 4, 5, 32]]))
    with pytest.raises(ValueError):
        O.bitmap_unpack(torch.tensor([[0xFF, 0, 0, 0]], dtype=torch.uint8), 6)


def test_relidx7_stream_layout_against_big_integers_and_hand_bytes():
    # hand-computed: 1 -> bits 0..6 = 1000000, 127 -> bits 7..13 all ones
    assert O.relidx7_pack(torch.tensor([[1, 127]])).tolist() == [[0x81, 0x3F]]
    # positions 0..5: value sum(p << 7p) written little-endian in ceil(42/8) = 6 bytes
    assert O.relidx7_pack(torch.tensor([[0, 1, 2, 3, 4, 5]])).tolist() == \
        [list((sum(p << (7 * p) for p in range(6))).to_bytes(6, "little"))]
    g = torch.Generator().manual_seed(11)
    for k in (1, 2, 3, 5, 6, 8):
        pos = torch.stack([torch.randperm(32, generator=g)[:k].sort()[0] for _ in range(50)])
        plane = O.relidx7_pack(pos)
        assert plane.shape == (50, (7 * k + 7) // 8)
        for row, p in zip(plane.tolist(), pos.tolist()):
            # the scalar rule of codec.py:91-107 as one big integer
            assert int.from_bytes(bytes(row), "little") == sum(v << (7 * s) for s, v in enumerate(p))
        assert torch.equal(O.relidx7_unpack(plane, k), pos)
    with pytest.raises(ValueError):
        O.relidx7_pack(torch.tensor([[0, 128]]))


def test_relidx7_pack_carries_the_same_positions_and_values_as_the_bitmap_pack():
    """The index planes are membership-equivalent (pack.py:323-326): same positions, every other
    plane identical, identical dequantised K."""
    from open_ommx_serve_amd.synth import synth_kv
    K, V = synth_kv(128, 2, 64, 77, sparse_frac=0.02)
    a = O.pack_kv(K, V, outlier_repr="bitmap")
    b = O.pack_kv(K, V, outlier_repr="relidx7")
    assert b["k_obmp"] is None and a["k_oidx"] is None
    assert b["k_oidx"].shape == (4, 2, 64, 6) and b["k_oidx"].dtype == torch.uint8
    assert b["k_field_bytes"] == 0 and a["k_field_bytes"] == 4          # pack.py:468,568
    assert torch.equal(O.relidx7_unpack(b["k_oidx"], 6), O.bitmap_unpack(a["k_obmp"], 6))
    for n in ("k_base", "k_scale", "k_zp", "k_oval", "k_fp4_mapscale", "k_fp4_mapcenter",
              "v_main", "v_scale", "v_zp"):
        assert torch.equal(a[n], b[n]), n
    Ka, Va = O.dequant_kv(a)
    Kb, Vb = O.dequant_kv(b)
    assert torch.equal(Ka, Kb) and torch.equal(Va, Vb)


def test_combinadic_ranks_are_the_combinatorial_number_system():
    """Pins independent of the formula: the k-subsets of a small set, enumerated in
    colexicographic order (compare the largest elements first), take the ranks 0, 1, 2, ... in
    turn - so the map is a bijection onto [0, C(n, k)); the first subset ranks 0 and the last
    C(n, k) - 1; one rank worked by hand; the plane widths of the reference's recipes."""
    import itertools
    for n, k in ((8, 3), (10, 4), (7, 1), (9, 8)):
        subsets = sorted(itertools.combinations(range(n), k), key=lambda c: tuple(reversed(c)))
        assert len(subsets) == math.comb(n, k)
        planes = O.combinadic_pack(torch.tensor(subsets), n)
        nb = planes.shape[-1]
        ranks = [int.from_bytes(bytes(r), "little") for r in planes.tolist()]
        assert ranks == list(range(len(subsets))), (n, k)
        assert torch.equal(O.combinadic_unpack(planes, k, n), torch.tensor(subsets))
        assert nb == O.combinadic_bytes(k, n) == (max(1, (len(subsets) - 1).bit_length()) + 7) // 8
    # {1, 4, 6}: C(1,1) + C(4,2) + C(6,3) = 1 + 6 + 20
    assert O.combinadic_pack(torch.tensor([[1, 4, 6]]), 32).tolist() == [[27, 0]]
    assert O.combinadic_pack(torch.tensor([[6, 1, 4]]), 32).tolist() == [[27, 0]]      # order is irrelevant
    last = torch.arange(26, 32).reshape(1, 6)
    assert int.from_bytes(bytes(O.combinadic_pack(last, 32)[0].tolist()), "little") == 906192 - 1
    # widths: 32 choose 6 needs 20 bits, 128 choose 10 needs 48 (codec.py:131-143)
    assert (O.combinadic_bytes(6, 32), O.combinadic_bytes(10, 128), O.combinadic_bytes(3, 32),
            O.combinadic_bytes(16, 32), O.combinadic_bytes(0, 32)) == (3, 6, 2, 4, 0)
    with pytest.raises(ValueError):
        O.combinadic_unpack(torch.tensor([[0xD0, 0xD3, 0x0D]], dtype=torch.uint8), 6, 32)   # = C(32, 6)
    with pytest.raises(ValueError):
        O.combinadic_pack(torch.tensor([[1, 1, 2]]), 32)


def test_combinadic_pack_carries_the_same_positions_as_the_bitmap_pack():
    from open_ommx_serve_amd.synth import synth_kv
    K, V = synth_kv(128, 2, 64, 78, sparse_frac=0.02)
    a = O.pack_kv(K, V, outlier_repr="bitmap")
    c = O.pack_kv(K, V, outlier_repr="combinadic")
    assert c["k_obmp"] is None and c["k_oidx"] is None and a["k_crank"] is None
    assert c["k_crank"].shape == (4, 2, 64, 3) and c["k_field_bytes"] == 3
    assert torch.equal(O.combinadic_unpack(c["k_crank"], 6), O.bitmap_unpack(a["k_obmp"], 6))
    for n in ("k_base", "k_scale", "k_zp", "k_oval", "k_fp4_mapscale", "k_fp4_mapcenter",
              "v_main", "v_scale", "v_zp"):
        assert torch.equal(a[n], c[n]), n
    Ka, _ = O.dequant_kv(a)
    Kc, _ = O.dequant_kv(c)
    assert torch.equal(Ka, Kc)


def test_base_shared_outliers_hand_built_vector():
    """kv_outlier_map=False (pack.py:502-506, dequant :756-757), every stored value derived on
    paper.  Channel 0 over 32 tokens: base lanes 0, 1, 2, 3 repeating -> min 0, max 3, scale
    2^0, zp 0.  Outliers (top three, bottom three): +6.5, +4.9, +3.4 and -6, -2.4, -0.2.
    (w - zp) / scale = w, so the FP4 codes are those of the raw values: 6.5 -> level 6 (code 7),
    4.9 -> nearest in log to 4 vs 6: boundary sqrt(24) = 4.899 -> 6 (code 7), 3.4 -> boundary
    sqrt(12) = 3.46 -> 3 (code 5), -6 -> sign | 7 = 15, -2.4 -> boundary sqrt(6) = 2.449 -> 2
    (code 4 | 8 = 12), -0.2 -> boundary sqrt(0.5e-8)... 0.2 is nearer to 0.5 than to 1e-8 in
    log -> 0.5 (code 1 | 8 = 9).  Dequant = level * 1 + 0."""
    w = torch.tensor([float(i % 4) for i in range(32)])
    put = {3: 6.5, 7: 4.9, 12: 3.4, 16: -6.0, 21: -2.4, 30: -0.2}
    for p, v in put.items():
        w[p] = v
    K = torch.zeros(32, 1, 32)
    K[:, 0, 0] = w
    K[:, 0, 1:] = torch.arange(32).float().unsqueeze(1) * 0.01      # other channels: anything finite
    pl = O.pack_kv(K, K.clone(), kv_outlier_map=False)
    assert pl["k_fp4_mapscale"] is None and pl["k_fp4_mapcenter"] is None and pl["kv_outlier_map"] is False
    assert int(pl["k_scale"][0, 0, 0]) == 0 and float(pl["k_zp"][0, 0, 0]) == 0.0
    assert O.bitmap_unpack(pl["k_obmp"], 6)[0, 0, 0].tolist() == sorted(put)
    assert O.nibbles_unpack(pl["k_oval"], 6)[0, 0, 0].tolist() == [7, 7, 5, 15, 12, 9]
    Kd, _ = O.dequant_kv(pl)
    want = w.clone()
    for p, v in zip(sorted(put), [6.0, 6.0, 3.0, -6.0, -2.0, -0.5]):
        want[p] = v
    assert torch.equal(Kd[:, 0, 0], want)
    # with the dedicated map the same vector stores other nibbles and planes
    assert O.pack_kv(K, K.clone())["k_fp4_mapscale"] is not None


def test_plain_bf16_steps_hand_built_vectors():
    """use_pow2=False (pack.py:459-465): the step is bf16((max - min) / 3), not a power of two,
    and the bf16 rounding of the step happens BEFORE the codes are formed.  No outliers, so the
    whole vector is the base.
    Channel 0: values in [0, 4.5] -> step 1.5 (exact in bf16); 1.4 / 1.5 = 0.93 -> 1,
               2.3 / 1.5 = 1.53 -> 2, 0.75 / 1.5 = 0.5 -> ties to even -> 0, 2.25 / 1.5 = 1.5 -> 2.
    Channel 1: values in [0, 1] -> 1/3 = 0.33333 rounds to bf16 0.333984375 (0x3EAB);
               0.5 / 0.333984375 = 1.497 -> 1 (with the unrounded third it would be a tie -> 2).
    Power-of-two twin of channel 0: 2^rint(log2(1.5)) = 2^1 -> codes rint(w / 2)."""
    w0 = [0.0, 4.5, 1.4, 2.3, 0.75, 2.25] + [3.0] * 26
    w1 = [0.0, 1.0, 0.5] + [0.25] * 29
    K = torch.zeros(32, 1, 32)
    K[:, 0, 0] = torch.tensor(w0)
    K[:, 0, 1] = torch.tensor(w1)
    pl = O.pack_kv(K, K.clone(), outliers_per_vector=0, use_pow2=False)
    assert pl["k_scale"].dtype == torch.bfloat16 and pl["v_scale"].dtype == torch.bfloat16
    assert pl["use_pow2"] is False and pl["kv_int8_scale"] is False
    assert float(pl["k_scale"][0, 0, 0]) == 1.5 and float(pl["k_scale"][0, 0, 1]) == 0.333984375
    codes = O.unpack_int2(pl["k_base"].reshape(32, 1, 8))
    assert codes[:6, 0, 0].tolist() == [0, 3, 1, 2, 0, 2] and codes[6, 0, 0].item() == 2
    assert codes[:4, 0, 1].tolist() == [0, 3, 1, 1]
    Kd, _ = O.dequant_kv(pl)
    assert Kd[:6, 0, 0].tolist() == [0.0, 4.5, 1.5, 3.0, 0.0, 3.0]
    assert Kd[2, 0, 1].item() == 0.333984375
    # the power-of-two recipe on the same data, stored either way, is another quantiser
    p2 = O.pack_kv(K, K.clone(), outliers_per_vector=0)
    assert int(p2["k_scale"][0, 0, 0]) == 1
    assert O.unpack_int2(p2["k_base"].reshape(32, 1, 8))[:6, 0, 0].tolist() == [0, 2, 1, 1, 0, 1]
    p3 = O.pack_kv(K, K.clone(), outliers_per_vector=0, kv_int8_scale=False)
    assert p3["k_scale"].dtype == torch.bfloat16 and float(p3["k_scale"][0, 0, 0]) == 2.0
    assert torch.equal(p3["k_base"], p2["k_base"]) and torch.equal(p3["v_main"], p2["v_main"])
    assert torch.equal(O.dequant_kv(p3)[0], O.dequant_kv(p2)[0])
    # V vector (token 1, channels 0..31): values 4.5, 1.0, zeros -> step 1.5, codes 3, 1 (0.67 -> 1), 0
    vc = O.unpack_int2(pl["v_main"].reshape(32, 1, 8))[1, 0]
    assert float(pl["v_scale"].reshape(32, 1, 1)[1, 0, 0]) == 1.5 and vc[:3].tolist() == [3, 1, 0]


def test_nibble_stream_even_slot_low():
    v = torch.tensor([[1, 2, 3, 4, 5, 6]])
    assert O.nibbles_pack(v).tolist() == [[0x21, 0x43, 0x65]]
    assert torch.equal(O.nibbles_unpack(O.nibbles_pack(v), 6), v)
    assert O.nibbles_pack(torch.tensor([[9, 8, 7]])).tolist() == [[0x89, 0x07]]


def test_bytes_per_token_head_is_8_25_bits_per_pair():
    assert O.plane_bytes_per_token_head(128, 6) == 132.0
    assert O.plane_bytes_per_token_head(128, 6) * 8 / (2 * 128) == 4.125      # per element
    assert 2 * 4.125 == 8.25


# ---- power-of-two scale -----------------------------------------------------------------

def test_pow2_rule_away_from_ties_and_exact_powers():
    g = torch.Generator().manual_seed(2)
    x = torch.exp(torch.rand(50000, generator=g) * 40 - 20)
    e = O.pow2_exponent(x)
    frac = np.log2(x.double().numpy()) - np.floor(np.log2(x.double().numpy()))
    clear = np.abs(frac - 0.5) > 1e-4
    assert np.array_equal(e.numpy()[clear], np.rint(np.log2(x.double().numpy()))[clear])
    n = torch.arange(-39, 61, dtype=torch.float32)      # the rule clamps below 1e-12 ~ 2^-39.9
    p = torch.pow(2.0, n)
    assert torch.equal(p, torch.ldexp(torch.ones_like(n), n.to(torch.int32)))   # exact powers
    assert torch.equal(O.pow2_exponent(p), n)                                    # lossless exponent
    assert torch.equal(torch.exp2(n), p)


def test_pow2_exact_log2_ties_round_half_to_even():
    """Vectors whose (max-min)/3 has fp32 log2 exactly n+0.5 must land on the even exponent;
    the same construction as the reference's tie test."""
    hits = []
    for n in range(-12, 6):
        t = torch.tensor([3.0 * 2.0 ** (n + 0.5)], dtype=torch.float32)
        cand = (t.view(torch.int32) + torch.arange(-8192, 8193, dtype=torch.int32)).view(torch.float32)
        raw = cand.clamp_min(1e-8) / 3.0
        hit = torch.log2(raw.clamp_min(1e-12)) == (n + 0.5)
        if bool(hit.any()):
            hits.append((n, float(cand[hit][0])))
    if not hits:
        pytest.skip("this libm produces no exact n+0.5 ties")
    T = 32
    K = torch.rand(T, 1, 32, generator=torch.Generator().manual_seed(7)) + 0.5
    V = K.clone()
    ramp = torch.arange(32, dtype=torch.float32) / 31.0
    hits = hits[:32]
    for j, (_, m) in enumerate(hits):
        K[:, 0, j] = m * ramp
        V[j, 0, :] = m * ramp
    p = O.pack_kv(K, V, outliers_per_vector=0)
    want = [n if n % 2 == 0 else n + 1 for n, _ in hits]
    assert p["k_scale"][0, 0, :len(hits)].tolist() == want
    assert p["v_scale"].reshape(T)[:len(hits)].tolist() == want


# ---- outlier selection ------------------------------------------------------------------

def _brute_select(w, k):
    """Rank counting: lane i is in the top set iff fewer than kt lanes beat it, where j
    beats i when w[j] > w[i] or (w[j] == w[i] and j < i); likewise for the bottom set on the
    vector with the top lanes replaced by 1e9."""
    kt, kb = (k + 1) // 2, k // 2
    n = len(w)
    top = [i for i in range(n)
           if sum(1 for j in range(n) if w[j] > w[i] or (w[j] == w[i] and j < i)) < kt]
    rest = [1e9 if i in top else w[i] for i in range(n)]
    bot = [i for i in range(n)
           if sum(1 for j in range(n) if rest[j] < rest[i] or (rest[j] == rest[i] and j < i)) < kb]
    return sorted(set(top) | set(bot))


@pytest.mark.parametrize("k", [2, 5, 6, 8])
def test_signed_selection_matches_brute_force_with_heavy_ties(k):
    g = torch.Generator().manual_seed(11 + k)
    lv = torch.tensor([-3.0, -1.0, -1.0, 0.0, 0.0, 0.0, 0.5, 2.0, 2.0])
    w = lv[torch.randint(0, 9, (200, 32), generator=g)]
    w[0] = 1.25                                              # a constant vector
    w[1, :16] = -2.0; w[1, 16:] = 2.0                        # two plateaus
    mask = O.select_outliers_signed(w, k)
    for r in range(w.shape[0]):
        assert mask[r].nonzero().flatten().tolist() == _brute_select(w[r].tolist(), k), r
    assert bool((mask.sum(-1) == k).all())


@pytest.mark.parametrize("k", [1, 3, 6, 8])
def test_abs_selection_matches_brute_force_with_heavy_ties(k):
    """Largest magnitudes, equal magnitudes (of either sign) to the lower index: lane i is chosen
    iff fewer than k lanes beat it, where j beats i when |w_j| > |w_i| or (equal and j < i)."""
    g = torch.Generator().manual_seed(21 + k)
    lv = torch.tensor([-3.0, -1.0, 1.0, 0.0, -0.0, 0.5, -0.5, 2.0, -2.0, 3.0])
    w = lv[torch.randint(0, 10, (200, 32), generator=g)]
    w[0] = -1.25
    w[1, ::2] = -2.0; w[1, 1::2] = 2.0
    mask = O.select_outliers_abs(w, k)
    for r in range(w.shape[0]):
        a = [abs(x) for x in w[r].tolist()]
        want = [i for i in range(32)
                if sum(1 for j in range(32) if a[j] > a[i] or (a[j] == a[i] and j < i)) < k]
        assert mask[r].nonzero().flatten().tolist() == want, r
    # and through the packer: positions are those lanes, in ascending order
    K = torch.zeros(32, 1, 32); K[:, 0, :] = w[:32].t()
    pl = O.pack_kv(K, K.clone(), outliers_per_vector=k, outlier_select="abs")
    assert pl["outlier_select"] == "abs"
    pos = O.bitmap_unpack(pl["k_obmp"], k)[0, 0]
    for c in range(32):
        assert pos[c].tolist() == mask[c].nonzero().flatten().tolist()


def test_base_range_excludes_outliers_and_map_closed_form():
    """One hand-built vector: the scale comes from the 26 inner lanes only, the FP4 map is
    centred on the 6 outliers, and every stored value follows the closed forms."""
    w = torch.linspace(-1.0, 1.0, 26).tolist() + [50.0, 40.0, 30.0, -50.0, -40.0, -20.0]
    K = torch.tensor(w, dtype=torch.float32).reshape(32, 1, 1).repeat(1, 1, 32)
    V = torch.zeros(32, 1, 32)
    p = O.pack_kv(K, V, outliers_per_vector=6)
    assert p["k_scale"][0, 0, 0].item() == round(math.log2(2.0 / 3.0))          # range 2 -> 2^-1
    assert p["k_zp"][0, 0, 0].item() == -1.0
    assert O.bitmap_unpack(p["k_obmp"], 6)[0, 0, 0].tolist() == [26, 27, 28, 29, 30, 31]
    assert p["k_fp4_mapcenter"][0, 0, 0].item() == 0.0                           # (50 + -50)/2
    ms = torch.tensor(12.0 / 100.0).to(torch.bfloat16)
    assert p["k_fp4_mapscale"][0, 0, 0] == ms
    lvl = O.fp4_decode(O.nibbles_unpack(p["k_oval"], 6))[0, 0, 0]
    assert lvl.tolist() == [6.0, 4.0, 4.0, -6.0, -4.0, -2.0]                      # 50*.12=6, 4.8->4, 3.6->4, -2.4->-2
    Kd, Vd = O.dequant_kv(p)
    assert torch.equal(Kd[26:, 0, 0], lvl / ms.float() + 0.0)
    inner = Kd[:26, 0, 0]
    assert torch.equal(inner, torch.round((torch.tensor(w[:26]) + 1.0) / 0.5).clamp(0, 3) * 0.5 - 1.0)
    # V all zeros: range clamps to 1e-8, exponent rint(log2(1e-8/3)) = -28, codes 0
    assert int(p["v_scale"].flatten()[0]) == round(math.log2(1e-8 / 3.0)) and int(p["v_main"].sum()) == 0
    assert torch.equal(Vd, torch.zeros_like(Vd))


def test_pack_refuses_nonfinite_like_the_reference():
    K = torch.randn(32, 1, 32); V = torch.randn(32, 1, 32)
    Kbad = K.clone(); Kbad[3, 0, 5] = float("inf")
    with pytest.raises((ValueError, IndexError)):
        O.pack_kv(Kbad, V)
    Vbad = V.clone(); Vbad[0, 0, 0] = float("nan")
    with pytest.raises(ValueError):
        O.pack_kv(K, Vbad)


# ---- attention and the split merge --------------------------------------------------------

def test_attend_equals_torch_softmax_and_fp64():
    g = torch.Generator().manual_seed(4)
    K = torch.randn(300, 2, 64, generator=g); V = torch.randn(300, 2, 64, generator=g)
    q = torch.randn(4, 64, generator=g)
    o32, l32 = O.attend(q, K, V, 0.125, dtype=torch.float32)
    o64, l64 = O.attend(q, K, V, 0.125, dtype=torch.float64)
    for h in range(4):
        s = (K[:, h // 2].double() @ q[h].double()) * 0.125
        want = torch.softmax(s, 0) @ V[:, h // 2].double()
        assert torch.allclose(o64[h], want, atol=1e-12)
        assert abs(l64[h].item() - torch.logsumexp(s, 0).item()) < 1e-12
    assert (o32.double() - o64).abs().max() < 1e-5 and (l32.double() - l64).abs().max() < 1e-5
    # one token: output is that token's V; uniform K: output is the mean of V
    o1, l1 = O.attend(q, K[:1], V[:1], 0.5, dtype=torch.float64)
    assert torch.allclose(o1[3], V[0, 1].double())
    ou, _ = O.attend(q, torch.zeros(10, 2, 64), V[:10], 1.0, dtype=torch.float64)
    assert torch.allclose(ou[0], V[:10, 0].double().mean(0))
    oe, le = O.attend(q, K[:0], V[:0], 1.0)
    assert float(oe.abs().sum()) == 0.0 and bool(torch.isinf(le).all())


@pytest.mark.parametrize("S", [1, 2, 3, 8, 64])
def test_split_merge_is_independent_of_the_split_count(S):
    g = torch.Generator().manual_seed(6)
    L = 1000
    K = torch.randn(L, 1, 32, generator=g); V = torch.randn(L, 1, 32, generator=g)
    q = torch.randn(2, 32, generator=g)
    want_o, want_l = O.attend(q, K, V, 0.2, dtype=torch.float64)
    parts = [O.attend(q, K[a:b], V[a:b], 0.2, dtype=torch.float64) for a, b in O.split_bounds(L, S)]
    o, l = O.merge_states(torch.stack([p[0] for p in parts]), torch.stack([p[1] for p in parts]))
    assert torch.allclose(o, want_o, atol=1e-12) and torch.allclose(l, want_l, atol=1e-12)


def test_split_bounds_rounding_and_empty_splits():
    assert O.split_bounds(960, 4) == [(0, 256), (256, 512), (512, 768), (768, 960)]
    b = O.split_bounds(96, 8)                       # per = 32: five splits are empty
    assert b[:3] == [(0, 32), (32, 64), (64, 96)] and all(a >= e for a, e in b[3:])
    o, l = O.merge_states(torch.zeros(3, 2, 4), torch.full((3, 2), -math.inf))
    assert float(o.abs().sum()) == 0.0 and bool(torch.isinf(l).all())


def test_window_closed_forms_and_invariant():
    assert O.packed_boundary(1024) == 968 and O.packed_boundary(4096) == 4040
    assert O.packed_boundary(65536) == 65480 and O.packed_boundary(40) == 8 and O.packed_boundary(5) == 5
    for n in range(0, 400):
        b = O.packed_boundary(n)
        if n >= 40:
            assert 32 <= n - b < 64 and (b - 8) % 32 == 0
        ti = O.tail_indices(n)
        assert len(ti) == len(set(ti)) and len(ti) <= 72
        assert sorted(ti + list(range(min(8, n), max(min(8, n), b)))) == list(range(n))
