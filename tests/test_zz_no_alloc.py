"""``ommx_decode_attention_noalloc``: the whole decode step with the split states in the
library's built-in device array instead of a caller workspace.

Checked through the C ABI against the existing pair of entry points
(``ommx_decode_splitkv`` + ``ommx_decode_combine`` over a torch workspace) on the same inputs,
to the decode tolerance (max-abs 2e-3 / mean-abs 2e-4 on ``o``, 2e-3 on ``lse``; the same
kernels run, so the results normally agree to the last bits), and against the CPU oracle; two
calls in a row, the second with a smaller input, so that stale contents of the shared array
would show.  Also: the driver's free device memory is the same before and after the second call
(the call allocates nothing), and sizes beyond the array are refused with a message."""
import pytest
import torch

import oracle.ommx_oracle as O
from open_ommx_serve_amd.attention import _hip
from open_ommx_serve_amd.attention.paged_decode import (make_attn_logits,
                                                        ommx_paged_decode_attention_canonical)
from open_ommx_serve_amd.synth import build_decode_case

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-3, 2e-4


def _noalloc(case, S):
    B, Hq, D = case.q.shape
    dev = case.q.device
    o = torch.full((B, Hq, D), float("nan"), dtype=torch.float32, device=dev)
    lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=dev)
    p = case.planes
    lib = _hip.load()
    with torch.cuda.device(dev):
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]       # device memory the driver has left (hipMemGetInfo)
        rc = lib.ommx_decode_attention_noalloc(
            case.q.data_ptr(), case.q.stride(0), case.q.stride(1),
            p["k_base"].data_ptr(), p["k_scale"].data_ptr(), p["k_zp"].data_ptr(),
            p["k_fp4_mapscale"].data_ptr(), p["k_fp4_mapcenter"].data_ptr(),
            p["k_obmp"].data_ptr(), p["k_oval"].data_ptr(),
            p["v_main"].data_ptr(), p["v_scale"].data_ptr(), p["v_zp"].data_ptr(),
            case.req_to_token.data_ptr(), case.req_to_token.stride(0),
            case.req_to_group.data_ptr(), case.req_to_group.stride(0),
            1 if case.req_to_token.dtype == torch.int64 else 0, case.b_seq_len.data_ptr(),
            case.k_tail.data_ptr(), case.v_tail.data_ptr(),
            case.k_tail.stride(0), case.k_tail.stride(1), case.k_tail.stride(2),
            case.v_tail.stride(0), case.v_tail.stride(1), case.v_tail.stride(2),
            case.b_tail_len.data_ptr(),
            o.data_ptr(), o.stride(0), o.stride(1), lse.data_ptr(), lse.stride(0),
            B, Hq, case.kv_heads, D, case.page_size, case.outliers_per_vector, _hip.INDEX_BITMAP, 0,
            32, 32, 0, S, int(case.k_tail.shape[1]), float(case.sm_scale), 0.0, 0, int(p["k_base"].shape[0]), int(p["k_scale"].shape[0]), None,
            _hip.current_stream_ptr(dev))
        torch.cuda.synchronize()
        _noalloc.taken = free_before - torch.cuda.mem_get_info()[0]
    return rc, o, lse


def _existing(case, S):
    B, Hq, D = case.q.shape
    dev = case.q.device
    o = torch.full((B, Hq, D), float("nan"), dtype=torch.float32, device=dev)
    lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=dev)
    ws = make_attn_logits(B, Hq, S, D, dev)
    ommx_paged_decode_attention_canonical(*case.decode_args(o, lse), num_kv_splits=S, attn_logits=ws,
                                          **case.decode_kwargs())
    return o, lse


def _oracle(case):
    planes = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in case.planes.items()} | {
        "outliers_per_vector": case.outliers_per_vector}
    return O.decode_reference(
        case.q.cpu(), planes, case.k_tail.cpu(), case.v_tail.cpu(), case.b_tail_len.tolist(),
        case.req_to_token.cpu(), case.req_to_group.cpu(), case.b_seq_len.tolist(),
        sm_scale=case.sm_scale, page_size=case.page_size)


def _close(o, lse, wo, wl, what):
    o, lse, wo, wl = o.cpu().double(), lse.cpu().double(), wo.cpu().double(), wl.cpu().double()
    assert torch.isfinite(o).all(), f"{what}: non-finite output"
    err = (o - wo).abs()
    assert err.max().item() <= MAX_ABS, f"{what}: max-abs {err.max().item():.3e}"
    assert err.mean().item() <= MEAN_ABS, f"{what}: mean-abs {err.mean().item():.3e}"
    assert (lse - wl).abs().max().item() <= 2e-3, f"{what}: lse"


def test_two_calls_in_a_row_second_smaller_match_the_workspace_entry_points():
    # first a ragged batch with many splits, then one short request with few: the second call
    # reuses the front of the array the first one filled
    big = build_decode_case([8192 + 40, 3000, 5121], seed=5, permute_tables=True, sparse_frac=0.005)
    small = build_decode_case([1024], seed=42)
    for case, S, name in ((big, 64, "big"), (small, 7, "small")):
        rc, o, lse = _noalloc(case, S)
        assert rc == 0, _hip.load().ommx_last_error()
        torch.cuda.synchronize()
        if name == "small":
            # the first call on a device may load the array's symbol; from the second call on the
            # driver's free memory must read the same before and after the call
            assert _noalloc.taken == 0, f"the call took {_noalloc.taken} bytes of device memory"
        wo, wl = _existing(case, S)
        torch.cuda.synchronize()
        _close(o, lse, wo, wl, f"{name} vs workspace entry points")
        assert (o - wo).abs().max().item() <= 1e-5, f"{name}: same kernels, same split count"
        oo, ol = _oracle(case)
        _close(o, lse, oo, ol, f"{name} vs oracle")


def test_head_dim_64_and_eight_q_heads_per_kv_head_through_the_same_entry_point():
    # the layouts of the serving-recipe kernel that came later: pairs of 64-channel kv heads, 8 q heads per kv head
    for case, S, name in ((build_decode_case([900, 70], q_heads=8, kv_heads=2, head_dim=64, seed=6), 4, "d64"),
                          (build_decode_case([1300], q_heads=64, kv_heads=8, seed=7, sparse_frac=0.005), 9, "gqa8")):
        rc, o, lse = _noalloc(case, S)
        assert rc == 0, _hip.load().ommx_last_error()
        torch.cuda.synchronize()
        wo, wl = _existing(case, S)
        torch.cuda.synchronize()
        assert (o - wo).abs().max().item() <= 1e-5, f"{name}: same kernels, same split count"
        oo, ol = _oracle(case)
        _close(o, lse, oo, ol, f"{name} vs oracle")


def test_sizes_beyond_the_built_in_array_are_refused():
    case = build_decode_case([1024] * 64, seed=3)          # 64 * 32 * 257 * 129 floats > 2 Mi
    rc, _, _ = _noalloc(case, 256)
    assert rc == -1
    msg = _hip.load().ommx_last_error().decode()
    assert "exceed" in msg and "8 MiB" in msg
