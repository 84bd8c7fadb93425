"""HIP split-KV decode + combine against the dequantise-then-attend oracle.

Tolerance (fp32 accumulation on the device, fp64 in the oracle): max-abs 2e-3 and
mean-abs 2e-4 on ``o``; ``lse`` within 2e-3.  All calls go through the C ABI."""
import math

import pytest
import torch

import oracle.ommx_oracle as O
from open_ommx_serve_amd.attention import _hip
from open_ommx_serve_amd.attention.kv_window import WindowSpec
from open_ommx_serve_amd.attention.paged_decode import (make_attn_logits,
                                                        ommx_paged_decode_attention_canonical)
from open_ommx_serve_amd.synth import build_decode_case

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-3, 2e-4


def _cpu_planes(case):
    return {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in case.planes.items()} | {
        "outliers_per_vector": case.outliers_per_vector}


def _oracle(case, **kw):
    return O.decode_reference(
        case.q.cpu(), _cpu_planes(case), case.k_tail.cpu(), case.v_tail.cpu(),
        case.b_tail_len.tolist(), case.req_to_token.cpu(), case.req_to_group.cpu(),
        case.b_seq_len.tolist(), sm_scale=case.sm_scale, page_size=case.page_size, **kw)


def _run(case, num_kv_splits=None, ref_kernel=False, **over):
    B, Hq, D = case.q.shape
    o = torch.full((B, Hq, D), float("nan"), dtype=torch.float32, device=case.q.device)
    lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=case.q.device)
    kw = case.decode_kwargs()
    kw.update(over)
    ommx_paged_decode_attention_canonical(*case.decode_args(o, lse), num_kv_splits=num_kv_splits,
                                          _force_reference_kernel=ref_kernel, **kw)
    torch.cuda.synchronize()
    return o.cpu(), lse.cpu()


def _check(got, want, what=""):
    (o, lse), (wo, wl) = got, want
    assert torch.isfinite(o).all(), f"{what}: non-finite output"
    err = (o.double() - wo).abs()
    assert err.max().item() <= MAX_ABS, f"{what}: max-abs {err.max().item():.3e}"
    assert err.mean().item() <= MEAN_ABS, f"{what}: mean-abs {err.mean().item():.3e}"
    fin = torch.isfinite(wl)
    assert torch.equal(torch.isfinite(lse), fin), f"{what}: lse finiteness"
    assert (lse.double()[fin] - wl[fin]).abs().max().item() <= 2e-3 if fin.any() else True, f"{what}: lse"


@pytest.mark.parametrize("ref_kernel", [False, True])
@pytest.mark.parametrize("seq_len", [128, 136, 200, 232])
def test_small_gqa2_d64_like_the_reference_parity_test(seq_len, ref_kernel):
    """H_KV=2, H_Q=4, D=64, page 16, sink 8, recent 32, k=6: 2/3/5/6 packed groups."""
    case = build_decode_case([seq_len], q_heads=4, kv_heads=2, head_dim=64, seed=11)
    _check(_run(case, ref_kernel=ref_kernel), _oracle(case), f"seq{seq_len}")


@pytest.mark.parametrize("ref_kernel", [False, True])
@pytest.mark.parametrize("splits", [1, 2, 4])
def test_forced_splits_4k_d64(splits, ref_kernel):
    case = build_decode_case([4096 + 40], q_heads=4, kv_heads=2, head_dim=64, seed=23,
                             table_dtype=torch.int64)
    _check(_run(case, num_kv_splits=splits, ref_kernel=ref_kernel), _oracle(case), f"S{splits}")


@pytest.mark.parametrize("ref_kernel", [False, True])
def test_layer_ctx1024(ref_kernel):
    """32 q / 8 kv heads, d=128, ctx 1024: 960 packed tokens + 64 tail rows."""
    case = build_decode_case([1024], seed=42)
    assert case.b_seq_len.tolist() == [960] and case.b_tail_len.tolist() == [64]
    assert case.algorithmic_bytes() == 960 * 8 * 132 + 64 * 8 * 128 * 4
    want = _oracle(case)
    for S in (None, 1, 3, 8):
        _check(_run(case, num_kv_splits=S, ref_kernel=ref_kernel), want, f"S{S}")


@pytest.mark.parametrize("ref_kernel", [False, True])
def test_layer_ctx4096_identity_tables(ref_kernel):
    case = build_decode_case([4096], seed=42)
    assert case.b_seq_len.tolist() == [4032]
    want = _oracle(case)
    for S in (None, 4, 16):
        _check(_run(case, num_kv_splits=S, ref_kernel=ref_kernel), want, f"S{S}")


@pytest.mark.parametrize("ref_kernel", [False, True])
def test_permuted_tables_ctx8192(ref_kernel):
    case = build_decode_case([8192], seed=7, permute_tables=True, sparse_frac=0.005)
    want = _oracle(case)
    for S in (1, 8, 32):
        _check(_run(case, num_kv_splits=S, ref_kernel=ref_kernel), want, f"S{S}")


def test_long_context_64k_permuted_all_split_counts():
    """ctx 65536, permuted page and group tables, sparse x8 outliers; 1, 8, 32, 64 splits."""
    case = build_decode_case([65536], seed=42, permute_tables=True, sparse_frac=0.005)
    assert case.b_seq_len.tolist() == [65472]
    assert case.algorithmic_bytes() == 65472 * 8 * 132 + 64 * 8 * 128 * 4
    want = _oracle(case)
    for S in (1, 8, 32, 64, 384, None):
        _check(_run(case, num_kv_splits=S), want, f"S{S}")
    _check(_run(case, num_kv_splits=64, ref_kernel=True), want, "ref S64")


def test_long_context_128k_int64_tables_and_the_split_limit():
    """ctx 131072 (the longest the reference serves), int64 tables, 512 splits (the limit) and
    odd split counts that leave the last splits short or empty."""
    case = build_decode_case([131072], seed=43, permute_tables=True, sparse_frac=0.005,
                             table_dtype=torch.int64)
    assert case.b_seq_len.tolist() == [131008]
    want = _oracle(case, dtype=torch.float32)
    for S in (None, 512, 256, 255, 100, 3):
        _check(_run(case, num_kv_splits=S), want, f"S{S}")
    _check(_run(case, num_kv_splits=300, ref_kernel=True), want, "ref S300")


@pytest.mark.parametrize("ref_kernel", [False, True])
def test_ragged_batch_shared_pool(ref_kernel):
    """Twelve requests of different lengths sharing one shuffled pool, incl. one with no
    packed tokens at all and one with an empty tail slot beyond its length."""
    lens = [1024, 40, 4000, 71, 72, 2047, 16384, 9, 1500, 333, 8192, 5000]
    case = build_decode_case(lens, seed=5, permute_tables=True, sparse_frac=0.005)
    want = _oracle(case)
    for S in (None, 1, 7, 16):
        _check(_run(case, num_kv_splits=S, ref_kernel=ref_kernel), want, f"S{S}")


def test_ragged_batch_32_requests():
    g = torch.Generator().manual_seed(4)
    lens = torch.randint(1024, 16385, (32,), generator=g).tolist()
    case = build_decode_case(lens, seed=6, permute_tables=True, sparse_frac=0.005)
    _check(_run(case), _oracle(case), "B32")


@pytest.mark.parametrize("batch", [2, 64, 65, 70, 130, 256, 257])
def test_longest_first_request_order(batch):
    """The matrix-core kernel serves up to 256 requests longest first (by counting up to 64, by a
    radix select beyond; more keep the grid order): equal lengths, zero lengths and both sides
    of the two limits give every request its own result."""
    g = torch.Generator().manual_seed(batch)
    lens = torch.randint(40, 700, (batch,), generator=g).tolist()
    lens[0] = lens[-1] = 500                      # ties
    lens[batch // 2] = 9                          # nothing packed
    if batch > 2:
        lens[1] = lens[2] = lens[3] = 168
    case = build_decode_case(lens, seed=batch, permute_tables=True, sparse_frac=0.005)
    want = _oracle(case)
    for S in (None, 3):
        _check(_run(case, num_kv_splits=S), want, f"B{batch} S{S}")


def _run_one(case, i, **over):
    """Request i of a batch as a one-request call (same planes and tables, row i of the rest)."""
    B, Hq, D = case.q.shape
    o = torch.full((1, Hq, D), float("nan"), dtype=torch.float32, device=case.q.device)
    lse = torch.full((1, Hq), float("nan"), dtype=torch.float32, device=case.q.device)
    args = list(case.decode_args(o, lse))
    for k in (0, 9, 10, 11, 14, 15, 16):          # q, tails, tables, lengths
        args[k] = args[k][i:i + 1].contiguous()
    kw = case.decode_kwargs()
    kw.update(over)
    ommx_paged_decode_attention_canonical(*args, **kw)
    torch.cuda.synchronize()
    return o.cpu()[0], lse.cpu()[0]


@pytest.mark.parametrize("hq,hkv,D,kw", [
    (32, 8, 128, {}), (64, 8, 128, {}), (16, 4, 64, {}), (32, 4, 64, {}),
    (32, 8, 128, dict(group_tokens=128, group_channels=128, outlier_repr="relidx7")),   # tails past 128 rows
])
def test_batches_combine_per_kv_head(hq, hkv, D, kw):
    """With 512 or more (request, kv head) pairs and at most 64 splits the combine serves a whole
    kv head per workgroup: against the oracle over split counts, and -- capped logits, segment
    form -- against the same requests sent one by one (which take the per-head kernel)."""
    B = 512 // hkv + 3
    pool = [9, 40, 71, 72, 200, 1000, 1500, 333, 2047, 640, 4100, 136, 168, 900, 77]
    lens = [pool[i % len(pool)] + 3 * (i // len(pool)) for i in range(B)]
    case = build_decode_case(lens, q_heads=hq, kv_heads=hkv, head_dim=D, seed=31 + hq + D,
                             permute_tables=True, sparse_frac=0.005, **kw)
    assert B * hkv >= 512
    if kw:
        assert max(case.b_tail_len.tolist()) > 128
    want = _oracle(case)
    for S in (None, 1, 5, 64):
        _check(_run(case, num_kv_splits=S), want, f"S{S}")
    for over in (dict(logit_cap=4.0), dict(seg_group_base=0, max_tail_len=0)):
        o, lse = _run(case, num_kv_splits=6, **over)
        for i in (0, 1, 5, B - 1):
            o1, l1 = _run_one(case, i, num_kv_splits=6, **over)
            assert torch.equal(torch.isfinite(lse[i]), torch.isfinite(l1))
            fin = torch.isfinite(l1)
            assert (o[i] - o1).abs().max().item() <= 2e-5, (over, i)
            assert (lse[i][fin] - l1[fin]).abs().max().item() <= 2e-5 if fin.any() else True


@pytest.mark.parametrize("ref_kernel", [False, True])
def test_gqa8_64_q_heads(ref_kernel):
    case = build_decode_case([2048, 3000], q_heads=64, kv_heads=8, seed=8, sparse_frac=0.005)
    want = _oracle(case)
    for S in (None, 5):
        _check(_run(case, num_kv_splits=S, ref_kernel=ref_kernel), want, f"S{S}")


@pytest.mark.parametrize("ref_kernel", [False, True])
def test_other_head_ratios(ref_kernel):
    for hq, hkv in ((8, 8), (8, 4), (2, 1)):
        case = build_decode_case([520], q_heads=hq, kv_heads=hkv, seed=9)
        _check(_run(case, ref_kernel=ref_kernel), _oracle(case), f"{hq}/{hkv}")


@pytest.mark.parametrize("ref_kernel", [False, True])
@pytest.mark.parametrize("hq,hkv", [(32, 8), (64, 8), (8, 2)])
def test_relidx7_index_plane(hq, hkv, ref_kernel):
    """Positions from the 7-bit streams (k_oidx, bitmap_read=False) instead of the bitmaps:
    same tolerance against the oracle, and the same result as the bitmap pack of the same
    cache (the two planes hold the same positions)."""
    kw = dict(q_heads=hq, kv_heads=hkv, seed=31, permute_tables=True, sparse_frac=0.005)
    lens = [3000, 72, 1500]
    case = build_decode_case(lens, outlier_repr="relidx7", **kw)
    assert case.planes["k_obmp"] is None and case.planes["k_oidx"].shape[-1] == 6
    assert case.decode_kwargs()["bitmap_read"] is False
    want = _oracle(case)
    twin = _run(build_decode_case(lens, **kw), ref_kernel=ref_kernel)
    for S in (None, 3):
        got = _run(case, num_kv_splits=S, ref_kernel=ref_kernel)
        _check(got, want, f"relidx7 S{S}")
        if S is None:
            assert (got[0] - twin[0]).abs().max().item() <= 1e-5


def test_relidx7_other_outlier_counts_and_head_dim():
    for k, D in ((3, 64), (8, 128), (1, 64)):
        case = build_decode_case([700], q_heads=4, kv_heads=2, head_dim=D, seed=32 + k,
                                 outliers_per_vector=k, outlier_repr="relidx7")
        assert case.planes["k_oidx"].shape[-1] == (7 * k + 7) // 8
        _check(_run(case), _oracle(case), f"relidx7 k{k} D{D}")


@pytest.mark.parametrize("ref_kernel", [False, True])
@pytest.mark.parametrize("hq,hkv,rep", [(32, 8, "bitmap"), (64, 8, "relidx7"), (8, 2, "bitmap")])
def test_base_shared_outliers(hq, hkv, rep, ref_kernel):
    """kv_outlier_map=False: outliers decode as level * 2^e + zp, no map planes."""
    case = build_decode_case([2100, 40, 700], q_heads=hq, kv_heads=hkv, seed=41, permute_tables=True,
                             sparse_frac=0.005, outlier_repr=rep, kv_outlier_map=False)
    assert case.planes["k_fp4_mapscale"] is None and case.decode_kwargs()["kv_outlier_map"] is False
    want = _oracle(case)
    for S in (None, 4):
        _check(_run(case, num_kv_splits=S, ref_kernel=ref_kernel), want, f"base-shared S{S}")


@pytest.mark.parametrize("kw", [dict(use_pow2=False), dict(kv_int8_scale=False),
                                dict(use_pow2=False, outlier_repr="relidx7", kv_outlier_map=False)])
@pytest.mark.parametrize("hq,hkv,D", [(32, 8, 128), (4, 2, 64)])
def test_bf16_step_planes(hq, hkv, D, kw):
    """Planes whose k_scale / v_scale hold the steps as bf16 (use_pow2=False: not powers of two;
    kv_int8_scale=False: powers of two stored as bf16) decode through the plain kernel."""
    case = build_decode_case([1300, 90], q_heads=hq, kv_heads=hkv, head_dim=D, seed=51,
                             permute_tables=True, sparse_frac=0.005, **kw)
    assert case.planes["k_scale"].dtype == torch.bfloat16 and case.decode_kwargs()["kv_int8_scale"] is False
    want = _oracle(case)
    for S in (None, 3):
        _check(_run(case, num_kv_splits=S), want, f"bf16 steps {kw} S{S}")
    if "use_pow2" not in kw:         # same numbers as the int8-exponent twin of the same cache
        twin = build_decode_case([1300, 90], q_heads=hq, kv_heads=hkv, head_dim=D, seed=51,
                                 permute_tables=True, sparse_frac=0.005)
        a, b = _run(case, ref_kernel=True), _run(twin, ref_kernel=True)
        assert torch.equal(a[0], b[0])


@pytest.mark.parametrize("recipe", [
    dict(group_tokens=64, group_channels=64, outliers_per_vector=6, outlier_repr="relidx7", kv_outlier_map=False),
    dict(group_tokens=128, group_channels=128, outliers_per_vector=10, outlier_repr="relidx7"),
    dict(group_tokens=128, group_channels=32, outliers_per_vector=8, outlier_repr="bitmap"),
    dict(group_tokens=16, group_channels=16, outliers_per_vector=3, outlier_repr="bitmap"),
    dict(group_tokens=16, group_channels=64, outliers_per_vector=2, outlier_repr="relidx7", use_pow2=False),
    dict(group_tokens=64, group_channels=128, outliers_per_vector=16, outlier_repr="relidx7"),
    dict(group_tokens=32, group_channels=32, outliers_per_vector=12, outlier_repr="relidx7"),
    dict(group_tokens=64, group_channels=64, outliers_per_vector=0),
])
@pytest.mark.parametrize("hq,hkv,D", [(32, 8, 128), (4, 2, 64)])
def test_other_group_sizes(hq, hkv, D, recipe):
    """K groups of 16 / 64 / 128 tokens, V vectors of 16 / 64 / 128 channels, up to 16 outliers:
    the window boundary, the split rounding and both tables follow the group size.  The first
    two rows are the reference's "low-bit lever" and "paper-kv" recipes."""
    if D % recipe["group_channels"]:
        recipe = {**recipe, "group_channels": D}          # a V vector cannot be wider than the head
    case = build_decode_case([1500, 300, 40], q_heads=hq, kv_heads=hkv, head_dim=D, seed=61,
                             permute_tables=True, sparse_frac=0.005, **recipe)
    gt = recipe["group_tokens"]
    assert all(n % gt == 0 for n in case.packed_lens) and case.packed_lens[0] > 0
    want = _oracle(case)
    for S in (None, 1, 7):
        _check(_run(case, num_kv_splits=S), want, f"{recipe} S{S}")


@pytest.mark.parametrize("kw", [dict(), dict(group_tokens=64, group_channels=64, outlier_repr="relidx7")])
def test_bf16_v_rows(kw):
    """v_format="bf16": P.V from unquantised bf16 rows (pack.py:596-602, dequant :766-769)."""
    case = build_decode_case([900, 50], q_heads=32, kv_heads=8, seed=71, permute_tables=True,
                             sparse_frac=0.005, v_format="bf16", **kw)
    assert case.planes["v_main"].dtype == torch.bfloat16
    want = _oracle(case)
    for S in (None, 2):
        _check(_run(case, num_kv_splits=S), want, f"bf16 V {kw} S{S}")


@pytest.mark.parametrize("gt,gc,k", [(64, 64, 6), (64, 32, 6), (128, 128, 6), (128, 64, 6), (64, 128, 6),
                                     (128, 128, 10), (128, 32, 10)])
@pytest.mark.parametrize("hq,own_map", [(32, False), (64, True), (32, True), (64, False)])
def test_longer_groups_on_the_matrix_core_kernel(gt, gc, k, hq, own_map):
    """K groups of 64 / 128 tokens with position streams and 6 outliers (10 with 128-token
    groups: the reference's 2.75-bit "paper-kv" recipe) run on the matrix-core kernel as
    32-token pieces of a group: against the oracle and against the plain kernel, ragged
    lengths, permuted tables, several split counts."""
    case = build_decode_case([2900, 700, 150], q_heads=hq, kv_heads=8, seed=81, permute_tables=True,
                             sparse_frac=0.005, group_tokens=gt, group_channels=gc, outliers_per_vector=k,
                             outlier_repr="relidx7", kv_outlier_map=own_map)
    want = _oracle(case)
    ref = _run(case, ref_kernel=True)
    for S in (None, 1, 5):
        got = _run(case, num_kv_splits=S)
        _check(got, want, f"gt{gt} gc{gc} k{k} S{S}")
        assert (got[0] - ref[0]).abs().max().item() <= MAX_ABS


def test_randomised_recipes_against_the_oracle():
    """Forty random draws over the whole recipe space the kernels accept (group sizes, outlier
    count, index plane, outlier map, step mode, V format, head shapes, table dtype, splits,
    ragged lengths cut inside the last group), each against the fp64 oracle."""
    g = torch.Generator().manual_seed(2024)

    def pick(*xs):
        return xs[int(torch.randint(0, len(xs), (1,), generator=g))]

    for it in range(40):
        gt, gc = pick(16, 32, 64, 128), pick(16, 32, 64)
        D = pick(64, 128)
        rep = pick("bitmap", "relidx7")
        k = pick(0, 1, 3, 6, 8) if rep == "bitmap" else pick(0, 2, 6, 10, 16)
        k = min(k, gt)
        hkv = pick(1, 2, 4)
        r = pick(1, 2, 4, 8)
        recipe = dict(group_tokens=gt, group_channels=gc, outliers_per_vector=k, outlier_repr=rep,
                      kv_outlier_map=pick(True, False), use_pow2=pick(True, True, False),
                      kv_int8_scale=pick(True, False), v_format=pick("i2", "i2", "bf16"))
        B = pick(1, 2, 3)
        lens = [int(torch.randint(1, 1400, (1,), generator=g)) for _ in range(B)]
        case = build_decode_case(lens, q_heads=hkv * r, kv_heads=hkv, head_dim=D, seed=3000 + it,
                                 permute_tables=pick(True, False), sparse_frac=pick(0.0, 0.01),
                                 table_dtype=pick(torch.int32, torch.int64), **recipe)
        if pick(0, 1):
            cut = torch.tensor([max(0, n - int(torch.randint(0, gt, (1,), generator=g)))
                                for n in case.b_seq_len.tolist()], dtype=torch.int32)
            case.b_seq_len.copy_(cut)
        S = pick(None, 1, 3, 16, 200)
        _check(_run(case, num_kv_splits=S), _oracle(case), f"case {it}: lens={lens} D={D} r={r} hkv={hkv} S={S} {recipe}")


@pytest.mark.parametrize("ref_kernel", [False, True])
def test_no_outliers_recipe(ref_kernel):
    case = build_decode_case([1000], q_heads=8, kv_heads=2, seed=10, outliers_per_vector=0)
    _check(_run(case, ref_kernel=ref_kernel), _oracle(case), "k0")


def test_tail_only_and_nothing_attended():
    case = build_decode_case([33, 1], q_heads=8, kv_heads=2, seed=12)
    assert case.b_seq_len.tolist() == [0, 0]
    _check(_run(case, num_kv_splits=4), _oracle(case), "tail-only")
    # zero tail rows as well: o = 0, lse = -inf
    case.b_tail_len.zero_()
    o, lse = _run(case, num_kv_splits=2)
    assert float(o.abs().sum()) == 0.0 and bool(torch.isinf(lse).all()) and bool((lse < 0).all())


def test_partial_last_group_is_masked():
    """b_seq_len need not be a whole number of groups: tokens past it are ignored."""
    case = build_decode_case([2048], q_heads=8, kv_heads=2, seed=13)
    for L in (1, 31, 33, 1000, 1971):
        case.b_seq_len.fill_(L)
        case.extra["packed_lens"] = [L]
        want = _oracle(case)
        for S in (1, 3):
            _check(_run(case, num_kv_splits=S), want, f"L{L} S{S}")


def test_logit_cap_and_caller_workspace():
    case = build_decode_case([3000], q_heads=8, kv_heads=2, seed=14)
    S = 6
    ws = make_attn_logits(1, 8, S, 128, "cuda")
    ws.fill_(float("nan"))
    got = _run(case, num_kv_splits=S, attn_logits=ws)
    _check(got, _oracle(case), "workspace")
    # partial states: splits x (D+1), lse column finite, tail slot untouched by stage 1
    assert torch.isfinite(ws[:, :, :S, :]).all()
    # capped logits: compare with an oracle that caps
    cap = 5.0
    Kd, Vd = O.gather_request(_cpu_planes(case), case.req_to_token[0].cpu(), case.req_to_group[0].cpu(),
                              case.b_seq_len.tolist()[0], page_size=16)
    tl = case.b_tail_len.tolist()[0]
    Kf = torch.cat([Kd, case.k_tail[0, :tl].cpu().float()]).double()
    Vf = torch.cat([Vd, case.v_tail[0, :tl].cpu().float()]).double()
    want = torch.zeros(8, 128, dtype=torch.float64)
    for h in range(8):
        s = (Kf[:, h // 4] @ case.q[0, h].cpu().double()) * case.sm_scale
        s = cap * torch.tanh(s / cap)
        want[h] = torch.softmax(s, 0) @ Vf[:, h // 4]
    o, _ = _run(case, num_kv_splits=S, logit_cap=cap)
    assert (o[0].double() - want).abs().max().item() <= MAX_ABS


@pytest.mark.parametrize("D,hq,hkv", [(128, 32, 8), (128, 16, 2), (128, 2, 2), (64, 4, 2), (64, 16, 4), (64, 4, 4),
                                      (64, 8, 8)])
@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 7, 8])
def test_other_outlier_counts_and_head_dim_64_on_the_matrix_core_kernel(D, hq, hkv, k):
    """1..8 outliers per vector (bitmap plane) and head_dim 64 run on the serving-recipe kernel's general
    form: against the oracle and against the plain kernel, ragged lengths cut inside a group, permuted
    tables, several split counts, both outlier maps."""
    for own_map in (True, False):
        case = build_decode_case([1700, 90, 600], q_heads=hq, kv_heads=hkv, head_dim=D, seed=700 + 10 * k + D,
                                 permute_tables=True, sparse_frac=0.005,
                                 outliers_per_vector=k, kv_outlier_map=own_map)
        cut = torch.tensor([1700 - 13, 90, 600 - 31], dtype=torch.int32)
        cut = torch.minimum(cut, case.b_seq_len.cpu()).to(case.b_seq_len.device)
        case.b_seq_len.copy_(cut)
        case.extra["packed_lens"] = cut.tolist()
        want = _oracle(case)
        ref = _run(case, num_kv_splits=4, ref_kernel=True)
        for S in (None, 1, 5):
            got = _run(case, num_kv_splits=S)
            _check(got, want, f"D{D} {hq}/{hkv} k{k} map{own_map} S{S}")
            assert (got[0] - ref[0]).abs().max().item() <= MAX_ABS


def test_head_dim_64_serving_recipe_with_cap_and_int64_tables():
    case = build_decode_case([2100, 333], q_heads=8, kv_heads=2, head_dim=64, seed=77, permute_tables=True,
                             sparse_frac=0.005, table_dtype=torch.int64)
    _check(_run(case, num_kv_splits=6), _oracle(case), "d64 k6")
    cap = 4.0
    planes = _cpu_planes(case)
    o, _ = _run(case, num_kv_splits=3, logit_cap=cap)
    for b in range(2):
        Kd, Vd = O.gather_request(planes, case.req_to_token[b].cpu(), case.req_to_group[b].cpu(),
                                  case.b_seq_len.tolist()[b], page_size=16)
        tl = case.b_tail_len.tolist()[b]
        Kf = torch.cat([Kd, case.k_tail[b, :tl].cpu().float()]).double()
        Vf = torch.cat([Vd, case.v_tail[b, :tl].cpu().float()]).double()
        for h in range(8):
            s_ = (Kf[:, h // 4] @ case.q[b, h].cpu().double()) * case.sm_scale
            want = torch.softmax(cap * torch.tanh(s_ / cap), 0) @ Vf[:, h // 4]
            assert (o[b, h].double() - want).abs().max().item() <= MAX_ABS, f"cap, request {b} head {h}"


@pytest.mark.parametrize("B", [2, 70])
def test_tail_length_outside_the_buffer_is_held_inside_it(B):
    """b_tail_len is a device tensor nobody checks on the host: with the buffer's row count known to the
    combine (tail_rows), a length above it reads as the row count and a negative one as 0, in the kernel
    with one workgroup per q head and in the one with one per kv head (70 requests of 8 kv heads)."""
    case = build_decode_case([200] * B, q_heads=32, kv_heads=8, seed=19)
    T = int(case.k_tail.shape[1])
    good = case.b_tail_len.clone()
    case.b_tail_len.fill_(T)
    case.b_tail_len[1] = 0
    want = _run(case, num_kv_splits=3)
    case.b_tail_len.fill_(T + 100000)
    case.b_tail_len[1] = -7
    got = _run(case, num_kv_splits=3)
    case.b_tail_len.copy_(good)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_head_dim_64_eight_outliers_many_requests_stay_inside_the_tolerance():
    """At head_dim 64 a logit weighs 64^-0.5 instead of 128^-0.5, so the f16 rounding of an outlier's
    tile entry shows more: the kernel lowers the size from which an entry's residual is added exactly
    in step (this shape measured 2.2e-3 with the head_dim-128 threshold)."""
    g = torch.Generator().manual_seed(5)
    lens = [int(torch.randint(1, 2500, (1,), generator=g)) for _ in range(70)]
    case = build_decode_case(lens, q_heads=16, kv_heads=8, head_dim=64, seed=9132, permute_tables=True,
                             sparse_frac=0.02, outliers_per_vector=8)
    _check(_run(case, num_kv_splits=5), _oracle(case), "d64 k8 70 requests")


@pytest.mark.parametrize("hq,hkv,D,k,own_map", [(32, 8, 128, 6, True), (64, 8, 128, 6, True), (32, 8, 128, 5, False),
                                                 (8, 8, 128, 3, True), (16, 8, 64, 6, True)])
def test_large_steps_take_the_operand_without_its_constant(hq, hkv, D, k, own_map):
    """Channels whose every value is large (x150 here), or vectors that hold more large values than they
    have outlier slots, get steps of 2^6 and more; the base operand (1 + code * 2^-j) * 2^e then carries
    a constant that cancels badly in fp32 (one such case measured 4.7e-3), so those groups use
    code * 2^(e-j) and no 2^e bias column."""
    case = build_decode_case([1500, 333, 2100], q_heads=hq, kv_heads=hkv, head_dim=D, seed=15, permute_tables=True,
                             sparse_frac=0.02, sparse_gain=40.0, outlier_gain=150.0, outliers_per_vector=k,
                             kv_outlier_map=own_map)
    exps = case.planes["k_scale"].to(torch.int32)
    assert int((exps >= 6).sum()) > 100 and int(exps.max()) <= 15
    err = torch.zeros(1, dtype=torch.int32, device=case.q.device)
    wo, wl = _oracle(case)
    for S in (None, 3):
        o, lse = _run(case, num_kv_splits=S, err_flag=err)
        e = (o.double() - wo).abs()
        assert e.max().item() <= MAX_ABS and e.mean().item() <= MEAN_ABS, f"S{S}: {e.max().item():.3e}"
        # the logits run into the thousands here: an fp32 lse carries 1e-4 of rounding per thousand
        assert ((lse.double() - wl).abs() <= 2e-3 + 2e-6 * wl.abs()).all(), f"S{S}: lse"
    assert int(err.item()) == 0


def test_a_step_beyond_the_f16_operands_is_reported():
    """K values around 1e6 give steps above 2^15, which the f16 operands of the matrix-core kernel cannot
    carry: the step is held at 2^15, the result stays finite, and the error word says so.  The plain
    kernel serves such a cache (fp32 throughout)."""
    case = build_decode_case([700], q_heads=32, kv_heads=8, seed=16, outlier_gain=3.0e5)
    assert int(case.planes["k_scale"].to(torch.int32).max()) > 15
    err = torch.zeros(1, dtype=torch.int32, device=case.q.device)
    o, lse = _run(case, num_kv_splits=2, err_flag=err)
    assert int(err.item()) & _hip.ERR_VALUE_RANGE
    assert torch.isfinite(o).all()
    err.zero_()
    po, pl = _run(case, num_kv_splits=2, ref_kernel=True, err_flag=err)
    wo, wl = _oracle(case)
    assert (po.double() - wo).abs().max().item() <= MAX_ABS
    assert ((pl.double() - wl).abs() <= 2e-3 + 2e-6 * wl.abs()).all()       # logits in the 1e5 range
    assert int(err.item()) == 0


@pytest.mark.parametrize("q_heads,kv_heads,head_dim", [(32, 8, 128), (16, 2, 128), (8, 4, 64)])
def test_query_elements_of_several_hundred(q_heads, kv_heads, head_dim):
    """The matrix-core kernel's QK operand is q * 2^(10-2m) as f16, up to q * 2^8: a query element of 256 or
    more would saturate it.  The kernel divides such a query by a power of two first (exact) and lets the
    softmax scale carry the factor; the result is held against the oracle like any other, with the lse bound
    widened by 1e-5 of its value (logits now run into the thousands, where 2e-3 is eight fp32 ulps)."""
    case = build_decode_case([900, 330], q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, seed=31,
                             permute_tables=True, sparse_frac=0.005)
    g = torch.Generator().manual_seed(7)
    q = case.q.float().cpu()
    flat = q.view(-1)
    where = torch.randperm(flat.numel(), generator=g)[:20]
    flat[where] = torch.tensor([300.0, -512.0, 1000.0, -776.0, 256.0] * 4)
    case.q.copy_(q.to(case.q.dtype))
    err = torch.zeros(1, dtype=torch.int32, device=case.q.device)
    wo, wl = _oracle(case)
    for S in (1, 3):
        o, lse = _run(case, num_kv_splits=S, err_flag=err)
        assert torch.isfinite(o).all()
        d = (o.double() - wo).abs()
        assert d.max().item() <= MAX_ABS and d.mean().item() <= MEAN_ABS, f"S{S}: {d.max().item():.3e}"
        assert ((lse.double() - wl).abs() <= 2e-3 + 1e-5 * wl.abs()).all(), f"S{S}: lse"
    assert int(err.item()) == 0


def test_a_v_step_beyond_the_f16_operands_is_reported():
    """V values around 1e6 give V steps above 2^15: held at 2^15 and reported, like the K steps above."""
    case = build_decode_case([300], q_heads=32, kv_heads=8, seed=18)
    vs = case.planes["v_scale"]
    vs.view(-1)[5::97] = 17                      # a handful of vectors with a step of 2^17
    err = torch.zeros(1, dtype=torch.int32, device=case.q.device)
    o, lse = _run(case, num_kv_splits=2, err_flag=err)
    assert int(err.item()) & _hip.ERR_VALUE_RANGE
    assert torch.isfinite(o).all()
    err.zero_()
    po, pl = _run(case, num_kv_splits=2, ref_kernel=True, err_flag=err)
    wo, wl = _oracle(case)
    assert ((po.double() - wo).abs() <= MAX_ABS + 1e-5 * wo.abs()).all()      # outputs in the thousands, fp32 sums
    assert int(err.item()) == 0


@pytest.mark.parametrize("B,hq", [(3, 32), (33, 32), (70, 32), (40, 64)])
def test_long_tails_take_several_passes_in_every_combine_kernel(B, hq):
    """A recent window of 300 tokens gives tails of up to 339 bf16 rows: several chunks of 64 rows in the
    combine with one workgroup per q head (3 requests), several passes of 128 in the one per kv head,
    with the first pass asked for early (33 and 40 requests of 8 kv heads) and without (70)."""
    win = WindowSpec(sink_tokens=8, recent_window=300, group_tokens=32, page_size=16)
    g = torch.Generator().manual_seed(B)
    lens = [int(torch.randint(20, 1500, (1,), generator=g)) for _ in range(B)]
    case = build_decode_case(lens, q_heads=hq, kv_heads=8, seed=21, permute_tables=True, sparse_frac=0.005,
                             window=win)
    assert int(case.b_tail_len.max()) > 256
    _check(_run(case, num_kv_splits=4), _oracle(case), f"B{B}")


def test_eight_q_heads_per_kv_head_partial_groups_empty_splits_and_cap():
    """The serving-recipe kernel laid out for 8 q heads per kv head (a lane keeps four heads of one
    token of either group): lengths that end inside the first / second group of a 64-token step,
    more splits than groups, one kv head alone in its workgroup, and capped logits."""
    case = build_decode_case([2048, 700], q_heads=16, kv_heads=2, seed=17, permute_tables=True, sparse_frac=0.01,
                             sparse_gain=40.0)
    full = case.b_seq_len.clone()
    for cut in ((1, 31), (33, 64), (65, 97), (1000, 2), (1971, 640)):
        case.b_seq_len.copy_(torch.tensor(cut, dtype=torch.int32))
        case.extra["packed_lens"] = list(cut)
        want = _oracle(case)
        for S in (1, 3, 40):
            _check(_run(case, num_kv_splits=S), want, f"cut {cut} S{S}")
    case.b_seq_len.copy_(full)
    case.extra["packed_lens"] = full.tolist()
    one = build_decode_case([900], q_heads=8, kv_heads=1, seed=18, sparse_frac=0.005)
    _check(_run(one, num_kv_splits=5), _oracle(one), "one kv head")
    cap = 5.0
    planes = _cpu_planes(case)
    o, _ = _run(case, num_kv_splits=7, logit_cap=cap)
    for b in range(2):
        Kd, Vd = O.gather_request(planes, case.req_to_token[b].cpu(), case.req_to_group[b].cpu(),
                                  case.b_seq_len.tolist()[b], page_size=16)
        tl = case.b_tail_len.tolist()[b]
        Kf = torch.cat([Kd, case.k_tail[b, :tl].cpu().float()]).double()
        Vf = torch.cat([Vd, case.v_tail[b, :tl].cpu().float()]).double()
        want = torch.zeros(16, 128, dtype=torch.float64)
        for h in range(16):
            s_ = (Kf[:, h // 8] @ case.q[b, h].cpu().double()) * case.sm_scale
            want[h] = torch.softmax(cap * torch.tanh(s_ / cap), 0) @ Vf[:, h // 8]
        assert (o[b].double() - want).abs().max().item() <= MAX_ABS, f"cap, request {b}"


@pytest.mark.parametrize("gt,kw", [(32, {}), (64, dict(group_tokens=64, group_channels=64, outlier_repr="relidx7")),
                                   (128, dict(group_tokens=128, group_channels=128, outlier_repr="relidx7",
                                              outliers_per_vector=10)),
                                   (16, dict(group_tokens=16, group_channels=16, outliers_per_vector=3))])
def test_segment_partial_emit_composes_to_the_full_result(gt, kw):
    """Two group-range segments plus the tail, merged with the textbook state merge; the segment
    base counts K groups of the recipe's size."""
    case = build_decode_case([4096], q_heads=8, kv_heads=2, seed=15, **kw)
    want = _oracle(case)
    L = case.b_seq_len.tolist()[0]
    g_split = (L // gt) // 3
    parts = []
    for gb, n in ((0, g_split * gt), (g_split, L - g_split * gt)):
        case.b_seq_len.fill_(n)
        o, lse = _run(case, num_kv_splits=4, seg_group_base=gb,
                      max_tail_len=0 if gb > 0 else None)
        parts.append((o, lse))
    case.b_seq_len.fill_(L)
    # first call (gb=0) included the tail; second is a pure segment
    o, lse = O.merge_states(torch.stack([p[0][0].double() for p in parts]),
                            torch.stack([p[1][0].double() for p in parts]))
    assert (o - want[0][0]).abs().max().item() <= MAX_ABS
    assert (lse - want[1][0]).abs().max().item() <= 2e-3


def test_host_argument_checks_raise_before_launch():
    case = build_decode_case([200], q_heads=4, kv_heads=2, head_dim=64, seed=16)
    B, Hq, D = case.q.shape
    o = torch.empty(B, Hq, D, dtype=torch.float32, device="cuda")
    lse = torch.empty(B, Hq, dtype=torch.float32, device="cuda")
    args = list(case.decode_args(o, lse))
    kw = case.decode_kwargs()
    with pytest.raises(ValueError):
        ommx_paged_decode_attention_canonical(*args, **{**kw, "packed_start_offset": 16})
    with pytest.raises(ValueError):
        ommx_paged_decode_attention_canonical(*args, **{**kw, "k_obmp": None})
    with pytest.raises(ValueError):
        ommx_paged_decode_attention_canonical(*args, **{**kw, "combinadic_read": True})
    with pytest.raises(ValueError):
        ommx_paged_decode_attention_canonical(*args, **{**kw, "k_fp4_mapscale": None})
    with pytest.raises(ValueError):
        ommx_paged_decode_attention_canonical(*args, **{**kw, "k_format": "i4"})
    bad = list(args); bad[0] = case.q[:, :3]
    with pytest.raises(NotImplementedError):
        ommx_paged_decode_attention_canonical(*bad, **kw)
    bad = list(args); bad[1] = case.planes["k_base"].transpose(0, 1)
    with pytest.raises(ValueError):
        ommx_paged_decode_attention_canonical(*bad, **kw)
    with pytest.raises(ValueError):          # k > 0 with no index plane at all
        ommx_paged_decode_attention_canonical(*args, **{**kw, "bitmap_read": False})
    ommx_paged_decode_attention_canonical(*args, **kw)
    torch.cuda.synchronize()


def test_randomised_shapes_two_kernels_and_the_oracle():
    """A hundred random cases (batch, lengths, GQA ratio, split count, table type, outlier mix with
    magnitudes up to x200, partial last groups): the matrix-core kernel against the plain
    fp32 kernel on the device (both within tolerance of each other's oracle), and against the
    oracle itself on every fourth case."""
    g = torch.Generator().manual_seed(2024)

    def rnd(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    for it in range(100):
        B = rnd(1, 5)
        lens = [rnd(1, 6000) if rnd(0, 4) else rnd(1, 80) for _ in range(B)]
        r = (4, 8)[rnd(0, 1)]
        hkv = (1, 2, 4, 8)[rnd(0, 3)]
        gain = (12.0, 40.0, 200.0)[rnd(0, 2)]
        case = build_decode_case(lens, q_heads=hkv * r, kv_heads=hkv, seed=1000 + it,
                                 permute_tables=bool(rnd(0, 1)), sparse_frac=(0.0, 0.005, 0.03)[rnd(0, 2)],
                                 table_dtype=(torch.int32, torch.int64)[rnd(0, 1)], sparse_gain=gain)
        if rnd(0, 2) == 0:                         # cut into the last group of every request
            cut = torch.tensor([max(0, n - rnd(0, 31)) for n in case.b_seq_len.tolist()], dtype=torch.int32)
            case.b_seq_len.copy_(cut)
        S = (None, 1, 2, 5, 16, 37, 256)[rnd(0, 6)]
        what = f"case {it}: B={B} lens={lens} r={r} hkv={hkv} gain={gain} S={S}"
        fast = _run(case, num_kv_splits=S)
        ref = _run(case, num_kv_splits=S, ref_kernel=True)
        assert torch.isfinite(fast[0]).all(), what
        err = (fast[0] - ref[0]).abs()
        assert err.max().item() <= MAX_ABS and err.mean().item() <= MEAN_ABS, f"{what}: {err.max().item():.3e}"
        fin = torch.isfinite(ref[1])
        assert torch.equal(torch.isfinite(fast[1]), fin), what
        # x200 outliers push lse into the hundreds, where 2e-3 is a few dozen fp32 ulps of the
        # logits' own accumulation: allow 1e-5 relative on top
        if fin.any():
            d = (fast[1][fin] - ref[1][fin]).abs() - 1e-5 * ref[1][fin].abs()
            assert d.max().item() <= 2e-3, what
        if it % 4 == 0:
            wo, wl = _oracle(case, dtype=torch.float32)
            e = (fast[0].double() - wo).abs()
            assert e.max().item() <= MAX_ABS and e.mean().item() <= MEAN_ABS, what
            f2 = torch.isfinite(wl)
            if f2.any():
                assert ((fast[1].double()[f2] - wl[f2]).abs() - 1e-5 * wl[f2].abs()).max().item() <= 2e-3, what


def test_plane_extents_are_passed_and_in_range_tables_raise_no_flag():
    """The launcher hands the plane extents to the kernels, which clamp every table entry into them
    and report one that was outside.  With tables in range nothing is reported (both kernels);
    a negative packed length counts as nothing packed and is reported."""
    from open_ommx_serve_amd.attention import _hip
    case = build_decode_case([2048 + 40, 777], seed=9, permute_tables=True, sparse_frac=0.005)
    want = _oracle(case)
    for ref in (False, True):
        err = torch.zeros(1, dtype=torch.int32, device=case.q.device)
        _check(_run(case, ref_kernel=ref, err_flag=err), want, f"ref={ref}")
        assert int(err.item()) == 0
    neg = case.b_seq_len.clone()
    neg[1] = -5
    err = torch.zeros(1, dtype=torch.int32, device=case.q.device)
    B, Hq, D = case.q.shape
    o = torch.full((B, Hq, D), float("nan"), dtype=torch.float32, device=case.q.device)
    lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=case.q.device)
    args = list(case.decode_args(o, lse))
    args[-1] = neg
    ommx_paged_decode_attention_canonical(*args, err_flag=err, **case.decode_kwargs())
    torch.cuda.synchronize()
    assert int(err.item()) & _hip.ERR_TABLE_RANGE
    assert torch.isfinite(o).all()
    # request 1 attends its tail rows only; request 0 is untouched
    assert (o[0].cpu().double() - want[0][0]).abs().max().item() <= MAX_ABS
