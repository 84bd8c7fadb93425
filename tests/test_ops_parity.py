"""torch.library ops and the state merge: segment decode + merge against the full decode and
the oracle; registration and fake (shape-only) implementations on the CPU."""
import math

import pytest
import torch

import oracle.ommx_oracle as O
from open_ommx_serve_amd.attention import reference_op as R
from open_ommx_serve_amd.attention.paged_decode import merge_attention_states
from open_ommx_serve_amd.synth import build_decode_case

MAX_ABS, MEAN_ABS = 2e-3, 2e-4


def test_ops_are_registered_with_fake_implementations():
    """Importing the module registers the three ops; fake mode runs the shape contract only."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    ns = torch.ops.ommx_gpu_serve
    for name in ("paged_decode", "paged_decode_segment", "merge_attention_states"):
        assert hasattr(ns, name)
    with FakeTensorMode():
        o_parts = torch.empty(3, 10, 128)
        lse_parts = torch.empty(3, 10)
        o, lse = ns.merge_attention_states(o_parts, lse_parts, None)
        assert tuple(o.shape) == (10, 128) and tuple(lse.shape) == (10,) and lse.dtype == torch.float32
        q = torch.empty(2, 32, 128, dtype=torch.bfloat16)
        kb = torch.empty(8, 16, 8, 32, dtype=torch.uint8)
        sc = torch.empty(4, 8, 128, dtype=torch.int8)
        zp = torch.empty(4, 8, 128, dtype=torch.bfloat16)
        vs = torch.empty(8, 16, 8, 4, dtype=torch.int8)
        vz = torch.empty(8, 16, 8, 4, dtype=torch.bfloat16)
        tail = torch.empty(2, 72, 8, 128, dtype=torch.bfloat16)
        i32 = torch.empty(2, dtype=torch.int32)
        tbl = torch.empty(2, 8, dtype=torch.int32)
        out, l2 = torch.empty(2, 32, 128), torch.empty(2, 32)
        ns.paged_decode(q, kb, sc, zp, None, None, None, None, zp, zp, kb, vs, vz, tail, tail, i32, out, l2,
                        tbl, tbl, i32, 0.1, 16, 6, "i2f4", False, True, True, True, 128, 72, 0)
        ns.paged_decode_segment(q, kb, sc, zp, None, None, None, None, zp, zp, kb, vs, vz, out, l2,
                                tbl, tbl, i32, 0.1, 16, 6, "i2f4", False, True, True, True, 128, 0, 0)
        with pytest.raises(Exception, match="lse must be"):
            ns.paged_decode(q, kb, sc, zp, None, None, None, None, zp, zp, kb, vs, vz, tail, tail, i32, out,
                            torch.empty(2, 31), tbl, tbl, i32, 0.1, 16, 6, "i2f4", False, True, True, True,
                            128, 72, 0)


def test_merge_argument_checks_and_no_cpu_path():
    with pytest.raises(ValueError, match="o_parts must be"):
        merge_attention_states(torch.zeros(2, 3), torch.zeros(2, 3))
    with pytest.raises(ValueError, match="lse_parts must be"):
        merge_attention_states(torch.zeros(2, 3, 4), torch.zeros(3, 2))
    with pytest.raises(ValueError, match="valid_lens"):
        merge_attention_states(torch.zeros(2, 3, 4), torch.zeros(2, 3), valid_lens=torch.zeros(2))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        merge_attention_states(torch.zeros(2, 3, 4), torch.zeros(2, 3))
    with pytest.raises(ValueError, match="k_obmp"):
        R._resolve_bitmap_read({"outlier_repr": "bitmap", "outliers_per_vector": 6, "k_obmp": None}, None)
    assert R._resolve_bitmap_read({"outlier_repr": "relidx7"}, None) is False


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_merge_states_matches_the_oracle(dtype):
    g = torch.Generator().manual_seed(5)
    P, Rr, D = 5, 37, 128
    o_parts = torch.randn(P, Rr, D, generator=g)
    lse_parts = torch.randn(P, Rr, generator=g) * 3
    lse_parts[1, 4] = float("-inf")
    lse_parts[:, 9] = float("-inf")                  # a row nothing attended
    valid = torch.full((Rr,), -1, dtype=torch.int32)
    valid[3], valid[11], valid[12] = 2, 5, 1
    op = o_parts.to(dtype)
    o, lse = R.merge_attention_states(op.cuda(), lse_parts.cuda(), valid_lens=valid.cuda())
    assert o.dtype == dtype and lse.dtype == torch.float32
    for r in range(Rr):
        n = P if valid[r] < 0 else int(valid[r])
        wo, wl = O.merge_states(op[:n, r:r + 1].double(), lse_parts[:n, r:r + 1].double())
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        if torch.isinf(wl).all():
            assert torch.isinf(lse[r].cpu()) and not o[r].any()
        else:
            assert (o[r].cpu().double() - wo[0]).abs().max() <= tol
            assert abs(float(lse[r]) - float(wl[0])) <= 1e-5
    # all parts valid, no valid_lens, preallocated strided output
    out = torch.zeros(Rr, 2 * D, device="cuda")[:, :D]
    lo = torch.zeros(Rr, device="cuda")
    merge_attention_states(o_parts.cuda(), lse_parts.cuda(), out=out, lse_out=lo)
    wo, wl = O.merge_states(o_parts[:, :9].double(), lse_parts[:, :9].double())
    assert (out[:9].cpu().double() - wo).abs().max() <= 1e-5 and (lo[:9].cpu().double() - wl).abs().max() <= 1e-5


@pytest.mark.gpu
def test_segments_merged_through_the_ops_equal_the_full_decode():
    """Three group-range segments + the bf16 tail as its own state, merged: the cascade /
    context-parallel composition (reference_op.py:151-271)."""
    case = build_decode_case([3000, 1500], seed=21, permute_tables=True, sparse_frac=0.005)
    planes = dict(case.planes) | {"outliers_per_vector": case.outliers_per_vector, "page_size": case.page_size,
                                  "k_format": "i2f4", "outlier_repr": "bitmap", "kv_outlier_map": True,
                                  "kv_int8_scale": True}
    q, B = case.q, 2
    full_o, full_lse = R.ommx_paged_decode(q, planes, case.k_tail, case.v_tail, case.b_tail_len, case.b_seq_len,
                                           sm_scale=case.sm_scale, req_to_token=case.req_to_token,
                                           req_to_group=case.req_to_group)
    seq = case.b_seq_len.tolist()
    cuts = [0, 20, 45, 10 ** 6]                    # group boundaries of the segments
    parts_o, parts_l = [], []
    for a, b in zip(cuts, cuts[1:]):
        seg = torch.tensor([max(0, min(n, b * 32) - a * 32) for n in seq], dtype=torch.int32, device=q.device)
        o, l = R.ommx_paged_decode_segment(q, planes, seg, a, sm_scale=case.sm_scale,
                                           req_to_token=case.req_to_token, req_to_group=case.req_to_group)
        parts_o.append(o)
        parts_l.append(l)
    # the tail alone: a decode with zero packed tokens
    zero = torch.zeros(B, dtype=torch.int32, device=q.device)
    o, l = R.ommx_paged_decode(q, planes, case.k_tail, case.v_tail, case.b_tail_len, zero, sm_scale=case.sm_scale,
                               req_to_token=case.req_to_token, req_to_group=case.req_to_group, max_seq_len=1)
    parts_o.append(o)
    parts_l.append(l)
    Hq, D = q.shape[1], q.shape[2]
    mo, ml = R.merge_attention_states(torch.stack(parts_o).reshape(-1, B * Hq, D),
                                      torch.stack(parts_l).reshape(-1, B * Hq))
    torch.cuda.synchronize()
    # the two routes round their softmax weights at different split boundaries
    assert (mo.reshape(B, Hq, D) - full_o).abs().max().item() <= 3e-4
    assert (ml.reshape(B, Hq) - full_lse).abs().max().item() <= 3e-4
    cpu_planes = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in planes.items()}
    wo, wl = O.decode_reference(q.cpu(), cpu_planes, case.k_tail.cpu(), case.v_tail.cpu(), case.b_tail_len.tolist(),
                                case.req_to_token.cpu(), case.req_to_group.cpu(), seq, sm_scale=case.sm_scale,
                                page_size=case.page_size)
    err = (mo.reshape(B, Hq, D).cpu().double() - wo).abs()
    assert err.max().item() <= MAX_ABS and err.mean().item() <= MEAN_ABS
