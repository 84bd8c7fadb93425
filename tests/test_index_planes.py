"""Outlier index planes: widths (CPU, through the C ABI's host-side entry point) and the
conversion kernel, the combinadic packer and the combinadic decode read (GPU) against the
oracle's big-integer ranking."""
import math
import random

import pytest
import torch

import oracle.ommx_oracle as O
from open_ommx_serve_amd.attention import _hip
from open_ommx_serve_amd.attention.pack import (alloc_planes, convert_index_plane,
                                                derive_bitmap_from_combinadic,
                                                derive_relidx7_from_combinadic, index_plane_bytes,
                                                ommx_pack_kv_canonical_block, store_pack_into)
from open_ommx_serve_amd.synth import build_decode_case, synth_kv

DEV = "cuda"
SHAPES = [(32, 6), (32, 16), (32, 1), (16, 3), (64, 6), (64, 16), (128, 10), (128, 15)]


def test_plane_widths_match_the_closed_forms():
    lib = _hip.load()
    for gt in (16, 32, 64, 128):
        for k in range(1, 17):
            if k >= gt:
                continue
            want = O.combinadic_bytes(k, gt)
            got = lib.ommx_index_plane_bytes(_hip.INDEX_COMBINADIC, gt, k)
            assert got == (want if math.comb(gt, k) < 2 ** 64 else 0), (gt, k)
            assert lib.ommx_index_plane_bytes(_hip.INDEX_BITMAP, gt, k) == gt // 8
            assert lib.ommx_index_plane_bytes(_hip.INDEX_RELIDX7, gt, k) == (7 * k + 7) // 8
    assert index_plane_bytes("combinadic", 32, 6) == 3 and index_plane_bytes("combinadic", 128, 10) == 6
    assert lib.ommx_index_plane_bytes(_hip.INDEX_COMBINADIC, 128, 16) == 0     # C(128, 16) > 2^64
    assert lib.ommx_index_plane_bytes(_hip.INDEX_COMBINADIC, 32, 17) == 0
    with pytest.raises(NotImplementedError):
        index_plane_bytes("combinadic", 128, 16)


def _random_positions(gt, k, shape, seed):
    rng = random.Random(seed)
    n = shape[0] * shape[1] * shape[2]
    rows = [sorted(rng.sample(range(gt), k)) for _ in range(n)]
    rows[0] = list(range(k))                        # rank 0
    rows[1] = list(range(gt - k, gt))               # rank C(gt, k) - 1
    return torch.tensor(rows, dtype=torch.int64).reshape(*shape, k)


def _planes_of(pos, gt):
    return {"bitmap": O.bitmap_pack(pos, gt), "relidx7": O.relidx7_pack(pos),
            "combinadic": O.combinadic_pack(pos, gt)}


@pytest.mark.gpu
@pytest.mark.parametrize("gt,k", SHAPES)
def test_conversion_kernel_matches_the_oracle_between_every_pair_of_planes(gt, k):
    pos = _random_positions(gt, k, (5, 2, 48), seed=gt * 100 + k)
    want = _planes_of(pos, gt)
    err = torch.zeros(1, dtype=torch.int32, device=DEV)
    for a in want:
        for b in want:
            dst = torch.full(want[b].shape, 0xAB, dtype=torch.uint8, device=DEV)
            convert_index_plane(want[a].to(DEV), dst, group_tokens=gt, k=k, src_repr=a, dst_repr=b, err_flag=err)
            assert torch.equal(dst.cpu(), want[b]), (a, b)
    assert int(err.item()) == 0


@pytest.mark.gpu
def test_conversion_of_selected_slots_and_invalid_vectors():
    gt, k = 32, 6
    pos = _random_positions(gt, k, (6, 2, 32), seed=5)
    want = _planes_of(pos, gt)
    src = want["combinadic"].clone()
    src[4, 1, 7] = torch.tensor([0xD0, 0xD3, 0x0D], dtype=torch.uint8)        # = C(32, 6): no such subset
    groups = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    dst = torch.full(want["bitmap"].shape, 0xAB, dtype=torch.uint8, device=DEV)
    err = torch.zeros(1, dtype=torch.int32, device=DEV)
    convert_index_plane(src.to(DEV), dst, group_tokens=gt, k=k, src_repr="combinadic", dst_repr="bitmap",
                        groups=groups, err_flag=err)
    got = dst.cpu()
    assert int(err.item()) == _hip.ERR_INDEX_PLANE
    assert not got[4, 1, 7].any()                                            # refused vector: zeros
    ok = torch.ones(6, 2, 32, dtype=torch.bool)
    ok[4, 1, 7] = False
    for g in (1, 4):
        assert torch.equal(got[g][ok[g]], want["bitmap"][g][ok[g]])
    for g in (0, 2, 3, 5):
        assert bool((got[g] == 0xAB).all())                                  # untouched slots
    # a bitmask with five bits is refused as well
    bad = want["bitmap"].clone()
    bad[0, 0, 0, 0] = 0
    bad[0, 0, 0, 1] = 0x1F
    bad[0, 0, 0, 2:] = 0
    err.zero_()
    out = torch.empty(want["combinadic"].shape, dtype=torch.uint8, device=DEV)
    convert_index_plane(bad.to(DEV), out, group_tokens=gt, k=k, src_repr="bitmap", dst_repr="combinadic", err_flag=err)
    assert int(err.item()) == _hip.ERR_INDEX_PLANE and not out[0, 0, 0].any()
    with pytest.raises(ValueError):
        convert_index_plane(want["bitmap"].to(DEV), out[..., :2].contiguous(), group_tokens=gt, k=k,
                            src_repr="bitmap", dst_repr="combinadic")


@pytest.mark.gpu
@pytest.mark.parametrize("gt,gc,k,dtype", [(32, 32, 6, torch.bfloat16), (32, 32, 3, torch.float32),
                                           (128, 128, 10, torch.bfloat16), (64, 64, 6, torch.bfloat16)])
def test_packer_writes_the_combinadic_plane_bit_for_bit(gt, gc, k, dtype):
    T, H, D = 4 * gt, 2, 128
    K, V = synth_kv(T, H, D, seed=31 + gt, sparse_frac=0.01)
    K, V = K.to(dtype), V.to(dtype)
    got = ommx_pack_kv_canonical_block(K, V, outliers_per_vector=k, outlier_repr="combinadic",
                                       outlier_select="signed", use_pow2=True, group_tokens=gt,
                                       group_channels=gc)
    want = O.pack_kv(K, V, outliers_per_vector=k, outlier_repr="combinadic", group_tokens=gt, group_channels=gc)
    assert got["k_obmp"] is None and got["k_oidx"] is None
    assert got["k_field_bytes"] == want["k_field_bytes"] == O.combinadic_bytes(k, gt)
    assert got["outlier_repr"] == "combinadic"
    for name in ("k_crank", "k_base", "k_scale", "k_zp", "k_oval", "k_fp4_mapscale", "k_fp4_mapcenter",
                 "v_main", "v_scale", "v_zp"):
        a, b = got[name], want[name]
        assert a.shape == b.shape and a.dtype == b.dtype, name
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), name
    # the stored ranks rewritten for the decode kernels: the planes the other recipes pack
    for derive, repr_name, plane in ((derive_relidx7_from_combinadic, "relidx7", "k_oidx"),
                                     (derive_bitmap_from_combinadic, "bitmap", "k_obmp")):
        d = derive(got)
        twin = O.pack_kv(K, V, outliers_per_vector=k, outlier_repr=repr_name, group_tokens=gt, group_channels=gc)
        assert d["outlier_repr"] == repr_name and torch.equal(d[plane], twin[plane])
        assert d["k_crank"] is got["k_crank"] and derive(twin) is twin


@pytest.mark.gpu
def test_store_into_pool_slots_ranks_only_the_groups_it_wrote():
    gt, k, H, D = 32, 6, 2, 128
    K, V = synth_kv(3 * gt, H, D, seed=9, sparse_frac=0.01)
    planes = alloc_planes(12, 8, H, D, outlier_repr="combinadic", device=DEV)
    planes["k_crank"].fill_(0xEE)
    slots = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    pages = torch.tensor([11, 10, 1, 0, 7, 6], dtype=torch.int32, device=DEV)
    err = torch.zeros(1, dtype=torch.int32, device=DEV)
    store_pack_into(K.to(DEV), V.to(DEV), planes, outlier_repr="combinadic", dst_groups=slots,
                    dst_pages=pages, err_flag=err)
    want = O.pack_kv(K, V, outlier_repr="combinadic")
    got = planes["k_crank"].cpu()
    assert int(err.item()) == 0
    for g, s in enumerate((6, 0, 3)):
        assert torch.equal(got[s], want["k_crank"][g])
    for s in (1, 2, 4, 5, 7):
        assert bool((got[s] == 0xEE).all())


@pytest.mark.gpu
@pytest.mark.parametrize("k", [6, 10])
def test_decode_reads_the_rank_plane(k):
    """``combinadic_read`` gives what the same cache gives through its position plane, and stays
    within tolerance of the oracle decoding the rank plane itself."""
    from open_ommx_serve_amd.attention.paged_decode import ommx_paged_decode_attention_canonical
    repr_twin = "bitmap" if k <= 8 else "relidx7"
    case = build_decode_case([700, 333], seed=12, permute_tables=True, sparse_frac=0.005,
                             outliers_per_vector=k, outlier_repr=repr_twin)
    p = case.planes
    src = p["k_obmp"] if repr_twin == "bitmap" else p["k_oidx"]
    crank = torch.empty(*src.shape[:3], index_plane_bytes("combinadic", 32, k), dtype=torch.uint8, device=DEV)
    convert_index_plane(src, crank, group_tokens=32, k=k, src_repr=repr_twin, dst_repr="combinadic")
    B, Hq, Dh = case.q.shape
    outs = []
    for comb in (False, True):
        o = torch.empty(B, Hq, Dh, dtype=torch.float32, device=DEV)
        lse = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
        kw = case.decode_kwargs()
        args = list(case.decode_args(o, lse))
        if comb:
            kw.update(bitmap_read=False, k_obmp=None, combinadic_read=True, k_crank=crank)
            args[4] = None                       # no k_oidx either
        ommx_paged_decode_attention_canonical(*args, **kw)
        torch.cuda.synchronize()
        outs.append((o.cpu(), lse.cpu()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    planes = {n: (v.cpu() if torch.is_tensor(v) else v) for n, v in p.items()}
    planes.update(k_crank=crank.cpu(), k_obmp=None, k_oidx=None, outlier_repr="combinadic", outliers_per_vector=k)
    wo, wl = O.decode_reference(case.q.cpu(), planes, case.k_tail.cpu(), case.v_tail.cpu(),
                                case.b_tail_len.tolist(), case.req_to_token.cpu(), case.req_to_group.cpu(),
                                case.b_seq_len.tolist(), sm_scale=case.sm_scale, page_size=case.page_size,
                                dtype=torch.float64)
    err = (outs[1][0].double() - wo.double()).abs()
    assert err.max().item() <= 2e-3 and err.mean().item() <= 2e-4
    assert (outs[1][1].double() - wl.double()).abs().max().item() <= 2e-3
