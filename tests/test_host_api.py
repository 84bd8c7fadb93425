"""Host-side checks that need no GPU: the C-ABI library loads and exports every entry point
the header declares, the decision tables behave, argument validation raises the
reference's exception types before anything is launched, and the operators refuse to run
without a GPU instead of falling back."""
import ctypes
import os
import re

import pytest
import torch

import oracle.ommx_oracle as O
from open_ommx_serve_amd.attention import _hip, kv_window
from open_ommx_serve_amd.attention import pack as hip_pack
from open_ommx_serve_amd.attention.paged_decode import (auto_num_kv_splits,
                                                        ommx_paged_decode_attention_canonical)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "ommx_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ommx_[a-z0-9_]+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = _hip.load()
    names = _declared_functions()
    assert {"ommx_store_pack", "ommx_decode_splitkv", "ommx_decode_combine",
            "ommx_store_default_table", "ommx_abi_version", "ommx_last_error"} <= set(names)
    raw = ctypes.CDLL(_hip.lib_path())
    for n in names:
        assert getattr(raw, n) is not None, n
    assert set(_hip.exported_symbols()) == set(names)
    assert lib.ommx_abi_version() == _hip.ABI_VERSION == 8


def test_default_decision_table_is_the_exact_arithmetic_one():
    lib = _hip.load()
    t = torch.zeros(_hip.STORE_TABLE_FLOATS)
    lib.ommx_store_default_table(t.data_ptr())
    for kb in (100, 126, 127, 128, 140):
        x = t[kb].double().item()
        assert x > 2.0 ** (kb - 127 + 0.5) > torch.nextafter(t[kb], torch.tensor(0.0)).double().item()
    want = [(1e-8 * 0.5) ** 0.5, 0.5 ** 0.5, 1.5 ** 0.5, 3 ** 0.5, 6 ** 0.5, 12 ** 0.5, 24 ** 0.5]
    for j, w in enumerate(want, start=1):
        assert abs(t[256 + j].item() - w) / w < 1e-6 and t[256 + j].double().item() > w


def test_measured_decision_table_reproduces_the_torch_rounding():
    """Thresholds measured from torch-CPU must give, for every float near every rounding
    point, the exponent / FP4 level the oracle's own expressions give."""
    t = hip_pack.measure_store_table()
    for kb in range(95, 150):
        c = t[kb:kb + 1]
        win = (c.view(torch.int32) + torch.arange(-40, 41, dtype=torch.int32)).view(torch.float32)
        got = (kb - 127) + (win >= c).to(torch.float32)
        assert torch.equal(got, O.pow2_exponent(win)), kb
    for j in range(2, 8):
        c = t[256 + j:256 + j + 1]
        win = (c.view(torch.int32) + torch.arange(-40, 41, dtype=torch.int32)).view(torch.float32)
        idx = sum((win >= t[256 + k]).to(torch.int64) for k in range(1, 8))
        assert torch.equal(idx, O.fp4_encode(win).to(torch.int64) & 7), j


def test_window_arithmetic_matches_the_oracle_closed_forms():
    w = kv_window.WindowSpec()
    for n in list(range(0, 300)) + [1024, 4096, 32768, 65536]:
        assert w.boundary(n) == O.packed_boundary(n)
        assert w.tail_indices(n) == O.tail_indices(n)
        assert w.packed_len(n) == max(0, O.packed_boundary(n) - 8)
        assert w.num_groups(n) * 32 == w.packed_len(n)
    assert (w.packed_len(1024), w.packed_len(4096), w.packed_len(65536)) == (960, 4032, 65472)
    assert w.newly_completed_groups(71, 72) == 1 and w.newly_completed_groups(72, 103) == 0
    assert w.max_tail_len() == 72 and w.packed_start_offset() == 8 and w.sink_page_shift() == 0
    w64 = kv_window.WindowSpec(group_tokens=64)
    assert w64.boundary(200) == 8 + 128
    with pytest.raises(ValueError):
        kv_window.packed_boundary(10, 8, 32, 0)


def test_split_heuristic_bounds():
    assert auto_num_kv_splits(960, 1, 8, 256) >= 1
    assert auto_num_kv_splits(65472, 1, 8, 256) == 256
    assert auto_num_kv_splits(960, 1, 8, 256) == 30          # one 32-token group per split
    assert auto_num_kv_splits(16320, 32, 8, 256) == 16
    assert auto_num_kv_splits(65472, 32, 8, 256) == 32         # long splits, lengths may differ: finer
    # equal lengths (mean close to the longest) and short splits: two workgroups per compute unit
    # instead of four
    assert auto_num_kv_splits(8128, 32, 8, 256, mean_seq_len=8128) == 8
    assert auto_num_kv_splits(8128, 32, 8, 256) == 16
    assert auto_num_kv_splits(65472, 32, 8, 256, mean_seq_len=65472) == 8       # long splits too
    assert auto_num_kv_splits(65472, 32, 8, 256, mean_seq_len=30000) == 32
    assert auto_num_kv_splits(32704, 8, 8, 256, 8, mean_seq_len=32704) == 32
    assert auto_num_kv_splits(65472, 1, 8, 256, mean_seq_len=65472) == 256
    assert 1 <= auto_num_kv_splits(1, 1, 1, 256) <= 256
    # the kernel that keeps three workgroups per compute unit deals groups out evenly: fill the chip
    assert auto_num_kv_splits(65472, 1, 8, 256, resident=3) == 256          # fewer than four steps per wave at 384
    assert auto_num_kv_splits(960, 1, 8, 256, resident=3) == 30
    assert auto_num_kv_splits(65472, 2, 8, 256, mean_seq_len=65472, resident=3) == 192
    assert auto_num_kv_splits(10 ** 6, 1, 8, 1024, resident=3) <= 512
    assert auto_num_kv_splits(131008, 1, 8, 256, resident=3) == 384         # 128K tokens: 5.3 steps per wave


def test_pack_argument_errors_match_the_reference():
    K = torch.zeros(64, 2, 64, dtype=torch.bfloat16)
    good = dict(outliers_per_vector=6, outlier_select="signed", outlier_repr="bitmap",
                k_format="i2f4", use_pow2=True, page_size=16)
    P = hip_pack.ommx_pack_kv_canonical_block
    with pytest.raises(ValueError):
        P(K, K[:32], **good)
    with pytest.raises(ValueError):
        P(K[:48], K[:48], **good)
    with pytest.raises(ValueError):
        P(K, K, **{**good, "outlier_repr": "bogus"})
    with pytest.raises(ValueError):
        P(K, K, **{**good, "k_format": "i4"})
    with pytest.raises(ValueError):
        P(K, K, **{**good, "group_tokens": 48})
    with pytest.raises(ValueError):
        P(K, K, **{**good, "outliers_per_vector": 33})
    with pytest.raises(ValueError):
        P(K, K, **{**good, "v_format": "fp8"})
    with pytest.raises(NotImplementedError, match="64 bits"):      # C(128, 16) does not fit a 64-bit rank
        P(torch.zeros(128, 2, 64), torch.zeros(128, 2, 64),
          **{**good, "outlier_repr": "combinadic", "group_tokens": 128, "outliers_per_vector": 16})
    with pytest.raises(NotImplementedError):
        P(K, K, **{**good, "scale_dtype": torch.float16})
    with pytest.raises(NotImplementedError):
        P(K, K, **{**good, "outliers_per_vector": 17, "outlier_repr": "relidx7"})
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            P(K, K, **good)


def test_store_error_bits_become_reference_exceptions():
    hip_pack.raise_for_store_errors(0)
    with pytest.raises(ValueError):
        hip_pack.raise_for_store_errors(_hip.ERR_NONFINITE_V)
    with pytest.raises(IndexError):
        hip_pack.raise_for_store_errors(_hip.ERR_UNDERFILLED | _hip.ERR_NONFINITE_K)
    with pytest.raises(ValueError):
        hip_pack.raise_for_store_errors(_hip.ERR_NONFINITE_K)


def _cpu_decode_args(Hq=4, Hkv=2, D=64, T=64):
    planes = O.pack_kv(torch.randn(T, Hkv, D).to(torch.bfloat16), torch.randn(T, Hkv, D).to(torch.bfloat16))
    q = torch.zeros(1, Hq, D, dtype=torch.bfloat16)
    tail = torch.zeros(1, 8, Hkv, D, dtype=torch.bfloat16)
    o = torch.zeros(1, Hq, D)
    lse = torch.zeros(1, Hq)
    args = [q, planes["k_base"], planes["k_scale"], planes["k_zp"], None, planes["k_oval"],
            planes["v_main"], planes["v_scale"], planes["v_zp"], tail, tail,
            torch.tensor([8], dtype=torch.int32), o, lse, planes["req_to_token"],
            planes["req_to_group"], torch.tensor([T], dtype=torch.int32)]
    kw = dict(sm_scale=0.125, page_size=16, k_outliers_per_vector=6, bitmap_read=True,
              k_obmp=planes["k_obmp"], k_fp4_mapscale=planes["k_fp4_mapscale"],
              k_fp4_mapcenter=planes["k_fp4_mapcenter"], kv_outlier_map=True, kv_int8_scale=True,
              max_seq_len=T, max_tail_len=8)
    return args, kw


def test_decode_argument_errors_precede_any_launch():
    args, kw = _cpu_decode_args()
    D = ommx_paged_decode_attention_canonical
    with pytest.raises(ValueError, match="packed_start_offset"):
        D(*args, **{**kw, "packed_start_offset": 16})
    with pytest.raises(ValueError, match="seg_group_base"):
        D(*args, **{**kw, "seg_group_base": -1})
    with pytest.raises(ValueError, match="k_obmp"):
        D(*args, **{**kw, "k_obmp": None})
    with pytest.raises(ValueError, match="mutually exclusive"):
        D(*args, **{**kw, "combinadic_read": True})
    with pytest.raises(ValueError, match="k_fp4_mapscale"):
        D(*args, **{**kw, "k_fp4_mapscale": None})
    with pytest.raises(ValueError, match="k_format"):
        D(*args, **{**kw, "k_format": "i8"})
    with pytest.raises(ValueError, match="k_oval"):
        bad = list(args); bad[5] = None
        D(*bad, **kw)
    with pytest.raises(NotImplementedError, match="integer multiple"):
        bad = list(args); bad[0] = args[0][:, :3]
        D(*bad, **kw)
    with pytest.raises(ValueError, match="contiguous"):
        bad = list(args); bad[6] = args[6][:, ::2]
        D(*bad, **{**kw, "page_size": 8})
    # operands whose shape or layout the kernels would otherwise take on trust
    with pytest.raises(ValueError, match="k_base must be a contiguous"):
        bad = list(args); bad[1] = args[1][:, :, :1]                  # a view that keeps one kv head
        D(*bad, **kw)
    with pytest.raises(ValueError, match="v_zp must be a contiguous"):
        bad = list(args); bad[8] = args[8].transpose(2, 3).contiguous().transpose(2, 3)
        D(*bad, **kw)
    with pytest.raises(ValueError, match="o must be"):
        bad = list(args); bad[12] = torch.zeros(1, 4, 32)
        D(*bad, **kw)
    with pytest.raises(ValueError, match="lse"):
        bad = list(args); bad[13] = torch.zeros(1, 3)
        D(*bad, **kw)
    with pytest.raises(ValueError, match="b_seq_len"):
        bad = list(args); bad[16] = torch.zeros(0, dtype=torch.int32)
        D(*bad, **kw)
    with pytest.raises(ValueError, match="req_to_group"):
        bad = list(args); bad[15] = args[15].reshape(-1)
        D(*bad, **kw)
    with pytest.raises(ValueError, match="k_oval must be"):
        bad = list(args); bad[5] = args[5][..., :2]
        D(*bad, **kw)
    with pytest.raises(ValueError, match="k_fp4_mapcenter must be"):
        D(*args, **{**kw, "k_fp4_mapcenter": kw["k_fp4_mapcenter"][:1]})
    with pytest.raises(ValueError, match="k_scale / k_zp"):
        bad = list(args); bad[3] = args[3][:, :1]
        D(*bad, **kw)
    with pytest.raises(ValueError, match="k_tail / v_tail"):
        bad = list(args); bad[9] = bad[10] = torch.zeros(1, 8, 1, 64, dtype=torch.bfloat16)
        D(*bad, **kw)
    with pytest.raises(ValueError, match="k_crank must be"):          # the rank plane's own shape check
        D(*args, **{**kw, "combinadic_read": True, "bitmap_read": False,
                    "k_crank": torch.zeros(2, 2, 64, 4, dtype=torch.uint8)})
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            D(*args, **kw)


def test_missing_library_is_a_loud_error(monkeypatch):
    monkeypatch.setattr(_hip, "_lib", None)
    monkeypatch.setattr(_hip, "_LIB_PATH", "/nonexistent/libommx_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _hip.load()


# ── KV store host logic ──────────────────────────────────────────────────────────────────

def test_ring_slot_pins_the_sink_and_never_aliases_live_rows():
    """Ring map of kv_store.py:301-313.  At every length the rows that can still be read
    (sink, and [boundary - group, seq)) must land on distinct ring rows."""
    from open_ommx_serve_amd.attention.kv_store_ops import ring_slot
    win = kv_window.WindowSpec()
    sink, span = win.sink_tokens, win.recent_window + 2 * win.group_tokens
    assert [ring_slot(p, sink, span) for p in range(sink)] == list(range(sink))
    assert ring_slot(sink, sink, span) == sink and ring_slot(sink + span, sink, span) == sink
    assert ring_slot(12345, sink, 0) == 12345
    for n in range(1, 700):
        edge = win.boundary(n)
        live = list(range(min(sink, n))) + list(range(max(sink, edge - win.group_tokens), n))
        slots = [ring_slot(p, sink, span) for p in live]
        assert len(set(slots)) == len(slots) and max(slots) < sink + span, n


def test_store_classes_refuse_other_recipes_and_the_cpu():
    from open_ommx_serve_amd.attention import CanonicalKVStore, MultiSeqKVPool
    from open_ommx_serve_amd.attention.kv_pool import check_serving_recipe
    good = dict(k_format="i2f4", outliers_per_vector=6, outlier_select="signed",
                outlier_repr="bitmap", use_pow2=True)
    check_serving_recipe(**good, kv_outlier_map=True, kv_int8_scale=True, group_tokens=32,
                         group_channels=32, scale_dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError, match="combinadic"):      # the bitmask twin serves up to 8
        MultiSeqKVPool(128, 8, 2, 256, device="cpu",
                       **{**good, "outlier_repr": "combinadic", "outliers_per_vector": 10})
    check_serving_recipe(**{**good, "outlier_repr": "combinadic"}, kv_outlier_map=True, kv_int8_scale=True,
                         group_tokens=32, group_channels=32, scale_dtype=torch.bfloat16)
    check_serving_recipe(**{**good, "outlier_repr": "relidx7"}, kv_outlier_map=True, kv_int8_scale=True,
                         group_tokens=32, group_channels=32, scale_dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="v_format"):
        CanonicalKVStore(128, 8, 256, device="cpu", v_format="fp8", **good)
    with pytest.raises(RuntimeError, match="no CPU fallback"):          # bf16 V rows are a served recipe
        CanonicalKVStore(128, 8, 256, device="cpu", v_format="bf16", **good)
    with pytest.raises(ValueError, match="k_format"):
        MultiSeqKVPool(128, 8, 2, 256, device="cpu", **{**good, "k_format": "i3"})
    with pytest.raises(ValueError, match="multiple of 32"):
        CanonicalKVStore(100, 8, 256, device="cpu", **good)
    with pytest.raises(ValueError, match="multiple of page_size"):
        MultiSeqKVPool(128, 8, 2, 256, device="cpu", window=kv_window.WindowSpec(page_size=24), **good)
    # the serving recipe on a CPU device: there is no CPU path
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        MultiSeqKVPool(128, 8, 2, 256, device="cpu", **good)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        CanonicalKVStore(128, 8, 256, device="cpu", **good)


def test_ring_ops_validate_before_touching_the_device():
    from open_ommx_serve_amd.attention import gather_tails, write_tokens
    kh = torch.zeros(1, 16, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        write_tokens(kh, kh.clone(), torch.zeros(1, dtype=torch.int64), kh[0, :1], kh[0, :1], 0, 0)
    with pytest.raises(ValueError, match="bfloat16"):
        write_tokens(kh.float(), kh.float(), torch.zeros(1, dtype=torch.int64), kh[0, :1], kh[0, :1], 0, 0)
    with pytest.raises(ValueError, match="num_slots"):
        gather_tails(kh[0], kh[0], kh, kh, 0, 0, seq=torch.zeros(1, dtype=torch.int64))


def test_tail_gather_refuses_a_buffer_shorter_than_the_longest_tail():
    """In the length-driven form a request's tail can hold sink + recent + group - 1 + lag rows and the kernel
    writes min(rows, T), sink rows first: a shorter buffer would drop the newest tokens, so the entry point
    refuses it before any launch (the pointers below are never followed)."""
    lib = _hip.load()
    fake = 4096
    args = dict(sink=8, recent=32, gt=32)
    need = args["sink"] + args["recent"] + args["gt"] - 1

    def call(T, lag):
        return lib.ommx_tail_gather(fake, fake, 100 * 2 * 64, 100, None, fake, None, fake, fake, None, None,
                                    1, T, 2, 64, args["sink"], args["recent"], args["gt"], 0, lag, None, None)

    assert call(need - 1, 0) == -1 and b"T is below" in lib.ommx_last_error()
    assert call(need, 1) == -1 and b"T is below" in lib.ommx_last_error()
    assert call(need + 4, 5) == -1


def test_table_id_clamp_arithmetic():
    """The clamp every decode kernel applies to the page ids and group slots it reads: ids inside
    the plane pass, anything else (negative ids included) lands on the nearest valid id and is
    reported; an extent of 0 means not given."""
    lib = _hip.load()
    flag = ctypes.c_int(0)
    for ident, extent, want, bad in [(0, 10, 0, 0), (9, 10, 9, 0), (10, 10, 9, 1), (10 ** 9, 10, 9, 1),
                                     (-1, 10, 9, 1), (-2 ** 31, 10, 9, 1), (5, 1, 0, 1), (0, 1, 0, 0),
                                     (123456, 0, 123456, 0), (-7, 0, -7, 0), (2 ** 31 - 1, 2 ** 31 - 1, 2 ** 31 - 2, 1)]:
        got = lib.ommx_clamp_table_id(ident, extent, ctypes.byref(flag))
        assert (got, flag.value) == (want, bad), (ident, extent, got, flag.value)
        assert extent == 0 or 0 <= got < extent
