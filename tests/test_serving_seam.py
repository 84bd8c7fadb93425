"""Host seam of the serving integration (CPU): slot allocator, step classification, the step
managers' buffers and their refusal rules, serving config.  The cases follow the reference's
``tests/test_slot_allocator.py``, ``test_slot_recycle_state.py``, ``test_seam_write_highwater.py``
and ``test_build_seam_ordering.py``; pools and stores are small stand-ins that record calls, so
nothing here needs a GPU."""
import random
from types import SimpleNamespace as NS

import pytest
import torch

from open_ommx_serve_amd.attention.kv_window import WindowSpec, packed_boundary
from open_ommx_serve_amd.integration.vllm import backend as BK
from open_ommx_serve_amd.integration.vllm.config import OMMXServingConfig, resolve_serving_config
from open_ommx_serve_amd.integration.vllm.metadata import (
    STEP_ROUTE_UNCLASSIFIED, OMMXBatchedStepManager, OMMXSlotAllocationError, OMMXStepManager,
    assign_slots, detect_full_prefill, detect_step_route)


# ── allocator ────────────────────────────────────────────────────────────────────────────

def _fresh(n):
    return {}, list(range(n))


def _ok(out, keys, n):
    assert len(out) == len(keys) and all(0 <= s < n for s in out) and len(set(out)) == len(out)


def test_surviving_key_keeps_its_slot_and_slots_follow_the_key_not_the_row():
    k2s, free = _fresh(4)
    a, fresh = assign_slots([10, 20, 30], k2s, free, 4)
    _ok(a, [10, 20, 30], 4)
    assert sorted(fresh) == sorted(a)
    b, fresh = assign_slots([30, 10, 20], k2s, free, 4)
    assert fresh == [] and b == [a[2], a[0], a[1]]


def test_departed_key_frees_its_slot_for_a_new_request():
    k2s, free = _fresh(2)
    a, _ = assign_slots([1, 2], k2s, free, 2)
    b, fresh = assign_slots([2, 3], k2s, free, 2)
    assert b[0] == a[1] and b[1] == a[0] and fresh == [a[0]]
    assert 1 not in k2s


def test_exhaustion_and_duplicates_raise_and_never_alias():
    k2s, free = _fresh(2)
    assign_slots([1, 2], k2s, free, 2)
    with pytest.raises(OMMXSlotAllocationError, match="EXHAUSTED"):
        assign_slots([1, 2, 3], k2s, free, 2)
    with pytest.raises(OMMXSlotAllocationError, match="EXHAUSTED"):
        assign_slots([7, 8, 9], *_fresh(2), 2)
    k2s, free = _fresh(8)
    assign_slots([1, 2], k2s, free, 8)
    before = (dict(k2s), list(free))
    with pytest.raises(OMMXSlotAllocationError, match="duplicate"):
        assign_slots([5, 2, 5], k2s, free, 8)
    assert (k2s, free) == before           # a refused step leaves the state untouched


def test_double_freed_or_out_of_range_slot_is_refused():
    k2s, free = {1: 0}, [0, 1]
    with pytest.raises(OMMXSlotAllocationError, match="already owns|already owned|owns"):
        assign_slots([1, 2], k2s, free, 2)
    with pytest.raises(OMMXSlotAllocationError, match="out-of-range"):
        assign_slots([4], {}, [9], 2)


def test_randomized_churn_never_aliases_two_live_requests():
    rng = random.Random(7)
    n = 6
    k2s, free = _fresh(n)
    live, nxt, owner = [], 100, {}
    for _ in range(400):
        live = [k for k in live if rng.random() > 0.25]
        while len(live) < n and rng.random() < 0.6:
            live.append(nxt)
            nxt += 1
        rng.shuffle(live)
        out, fresh = assign_slots(live, k2s, free, n)
        _ok(out, live, n)
        for k, s in zip(live, out):
            assert owner.setdefault(k, s) == s      # a request never moves
        assert sorted(free + list(k2s.values())) == list(range(n))
        assert set(fresh) <= set(out)


# ── classification ───────────────────────────────────────────────────────────────────────

def test_step_classification():
    assert detect_step_route(NS(seq_lens_cpu=[5, 9], query_start_loc_cpu=[0, 1, 2])) == (2, True)
    assert detect_step_route(NS(seq_lens=torch.tensor([5, 9]), query_start_loc=torch.tensor([0, 5, 6]))) == (2, False)
    assert detect_step_route(NS(seq_lens_cpu=[], query_start_loc_cpu=[0])) == (0, False)
    assert detect_step_route(NS()) == (STEP_ROUTE_UNCLASSIFIED, False)
    assert detect_step_route(NS(seq_lens_cpu=[3])) == (1, False)          # no query spans
    assert detect_full_prefill(NS(seq_lens_cpu=[5, 9], query_start_loc_cpu=[0, 5, 14]))
    assert not detect_full_prefill(NS(seq_lens_cpu=[5, 9], query_start_loc_cpu=[0, 5, 13]))
    assert not detect_full_prefill(NS(seq_lens_cpu=[5, 9]))
    assert not detect_full_prefill(NS())
    assert detect_full_prefill(NS(seq_lens_cpu=[1], query_start_loc_cpu=[0, 1]))   # one-token prompt


@pytest.mark.parametrize("sink,recent,gt", [(8, 32, 32), (0, 32, 32), (8, 1, 32), (128, 128, 128),
                                            (8, 32, 1), (4, 7, 3)])
def test_the_current_token_is_never_inside_the_packed_region(sink, recent, gt):
    """The seam packs before the forward writes token ``seq - 1``; that is sound because the
    token always lies in the bf16 tail, with a margin of at least the recent window."""
    for seq in range(1, 600):
        b = packed_boundary(seq, sink, recent, gt)
        assert not (sink <= seq - 1 < b)
        if b > sink:
            assert b <= seq - recent


def test_a_window_without_recent_rows_is_refused_at_the_seam(monkeypatch):
    """recent = 0 would let the boundary reach seq itself: the seam packs before the forward
    writes token seq-1, so that group would be packed with an unwritten row."""
    assert any(packed_boundary(seq, 8, 0, 32) == seq for seq in range(1, 200))
    with pytest.raises(ValueError, match="recent"):
        OMMXStepManager(_cfg(recent_window=0), "cpu")
    with pytest.raises(ValueError, match="recent"):
        OMMXBatchedStepManager(_cfg(recent_window=0), "cpu", 2)
    monkeypatch.setenv("OMMX_KV_RECENT", "0")
    from open_ommx_serve_amd.integration.vllm.config import resolve_serving_config
    with pytest.raises(ValueError, match="OMMX_KV_RECENT"):
        resolve_serving_config(head_dim=64, n_q_heads=4, n_kv_heads=2)


# ── single-request manager ───────────────────────────────────────────────────────────────

class _Store:
    def __init__(self):
        self.calls = []

    def reset_inplace(self):
        self.calls.append("reset")

    def advance_to(self, n):
        self.calls.append(("advance", n))


def _cfg(**kw):
    return OMMXServingConfig(max_context=kw.pop("max_context", 512), head_dim=64, n_kv_heads=2,
                             n_q_heads=4, **kw)


def test_single_manager_buffers_follow_the_window_arithmetic():
    cfg = _cfg()
    win = cfg.window()
    m = OMMXStepManager(cfg, "cpu")
    st = _Store()
    m.register(0, st)
    T = m.max_tail_len
    assert T == win.max_tail_len(cfg.max_context) and m.tail_idx.shape == (T,)
    last = None
    for seq in list(range(1, 140)) + [300, 301, 511]:
        m.on_build(NS(seq_lens_cpu=[seq], query_start_loc_cpu=[0, 1]), new_request=False)
        tail = win.tail_indices(seq)
        assert int(m.write_pos) == seq - 1
        assert int(m.b_seq_len) == win.packed_len(seq)
        assert int(m.b_tail_len) == len(tail)
        assert m.tail_idx[:len(tail)].tolist() == tail and not m.tail_idx[len(tail):].any()
        b = win.boundary(seq)
        assert (st.calls[-1] == ("advance", seq)) == (b != last) or last is None
        last = b
    n_adv = sum(1 for c in st.calls if c != "reset")
    assert n_adv == len({win.boundary(s) for s in list(range(1, 140)) + [300, 301, 511]})
    m.on_build(NS(seq_lens_cpu=[77], query_start_loc_cpu=[0, 77]))        # full prefill detected
    assert st.calls[-1] == "reset" and int(m.b_seq_len) == win.packed_len(77)


def test_single_manager_records_why_it_died_and_strict_reraises():
    m = OMMXStepManager(_cfg(), "cpu")
    m.on_build(NS())
    assert m.dead and "seq_lens" in m.dead_reason
    with pytest.raises(RuntimeError):
        OMMXStepManager(_cfg(strict=True), "cpu").on_build(NS())


def test_ring_span_guard(monkeypatch):
    monkeypatch.setenv("OMMX_KV_RING", "1")
    m = OMMXStepManager(_cfg(strict=True), "cpu")
    for seq in range(1, 400):                      # the shipped window never trips it
        m.on_build(NS(seq_lens_cpu=[seq], query_start_loc_cpu=[0, 1]), new_request=False)
    m._ring_rec = 40
    with pytest.raises(AssertionError, match="alias"):
        m._refresh(200)


# ── batched manager ──────────────────────────────────────────────────────────────────────

class _Pool:
    def __init__(self, num_seqs, window, **kw):
        self.window = window
        self.seq_len = [0] * num_seqs
        self.packed_groups = [0] * num_seqs
        self.regrouped = []

    def regroup(self, r):
        self.regrouped.append((r, self.seq_len[r]))
        self.packed_groups[r] = self.window.num_groups(self.seq_len[r])


def _bmgr(num_seqs=4, graph=True, **kw):
    cfg = _cfg(**kw)
    m = OMMXBatchedStepManager(cfg, "cpu", num_seqs, graph=graph,
                               pool_cls=lambda **a: _Pool(a["num_seqs"], a["window"]))
    return m, m.pool(0, "cpu")


def _md(seqs, keys, q=None):
    q = q if q is not None else list(range(len(seqs) + 1))
    return NS(seq_lens_cpu=list(seqs), query_start_loc_cpu=list(q),
              block_table_tensor=torch.tensor([[k, k + 1] for k in keys]).reshape(len(keys), 2))


def test_the_one_token_anticipation_is_allowed_and_buffers_are_refreshed():
    m, pool = _bmgr()
    m.on_build(_md([200, 90], [11, 12], q=[0, 200, 290]))        # prefill step: slots only
    s0, s1 = m.slots
    pool.seq_len[s0], pool.seq_len[s1] = 200, 90                 # what the writer would do
    pool.packed_groups[s0] = m.window.num_groups(200)
    pool.packed_groups[s1] = m.window.num_groups(90)
    m.on_build(_md([201, 91], [12, 11][::-1]))
    assert not m.dead and m.cur_B == 2 and m.is_uniform_decode
    assert m.b_sel[:2].tolist() == [s0, s1]
    assert m.b_write_col[:2].tolist() == [200, 90] and m.b_cur_seq[:2].tolist() == [201, 91]
    assert pool.seq_len[s0] == 201
    for seq in range(202, 240):                                   # crossing a group boundary packs
        m.on_build(_md([seq, seq - 110], [11, 12]))
    assert not m.dead
    assert {r for r, _ in pool.regrouped} == {s0, s1}
    assert pool.packed_groups[s0] == m.window.num_groups(239)
    m.on_build(_md([239, 129], [11, 12]))                         # an exactly current length is fine
    assert not m.dead


def test_a_pool_that_never_saw_the_prompt_stops_instead_of_packing():
    m, pool = _bmgr()
    m.on_build(_md([1357, 50], [5, 6], q=[0, 1357, 1407]))
    s0, s1 = m.slots
    pool.seq_len[s0] = 1                       # one token reached the pool, not the prompt
    pool.seq_len[s1] = 50
    m.on_build(_md([1358, 51], [5, 6]))
    assert m.dead and pool.regrouped == []
    assert "1358" in m.dead_reason and "1356" in m.dead_reason and f"slot {s0}" in m.dead_reason
    assert pool.packed_groups[s1] == 0         # the healthy slot was not packed either


@pytest.mark.parametrize("written,seq,ok", [(100, 100, True), (100, 101, True), (100, 102, False)])
def test_the_boundary_is_exactly_one_token(written, seq, ok):
    m, pool = _bmgr()
    m.on_build(_md([written], [9], q=[0, written]))
    pool.seq_len[m.slots[0]] = written
    m.on_build(_md([seq], [9]))
    assert m.dead == (not ok)


def test_a_recycled_slot_starts_with_clear_cursors():
    m, pool = _bmgr(num_seqs=1)
    m.on_build(_md([300], [21], q=[0, 300]))
    s = m.slots[0]
    pool.seq_len[s], pool.packed_groups[s] = 300, 8
    m.on_build(_md([40], [22], q=[0, 40]))     # request 21 left, 22 takes its slot
    assert m.slots == [s] and pool.seq_len[s] == 0 and pool.packed_groups[s] == 0


def test_dummy_and_oversized_batches_touch_no_live_slot():
    m, pool = _bmgr(num_seqs=3, graph=False)
    m.on_build(_md([10], [31], q=[0, 10]))
    live = dict(m._key_to_slot)
    m.capturing = True
    m.on_build(_md([1, 1], [0, 0]))            # null block ids: a capture / profiling dummy
    assert m._key_to_slot == live and set(m.slots).isdisjoint(live.values()) and len(m.slots) == 2
    m.on_build(_md([1] * 5, [0] * 5))          # larger than the pool: skipped, not a fault
    assert not m.dead and m.slots == [] and m.cur_B == 0
    m.on_build(NS(seq_lens_cpu=[], query_start_loc_cpu=[0]))
    assert m._key_to_slot == live              # a request-less step releases nothing
    m.on_build(_md([1, 1, 1], [0, 0, 0]))      # three dummies, two free slots
    assert m.dead and "free slot" in m.dead_reason


def test_identity_is_required_unless_the_unsafe_hatch_is_set(monkeypatch):
    m, _ = _bmgr(graph=False)
    m.on_build(NS(seq_lens_cpu=[5, 6], query_start_loc_cpu=[0, 1, 2]))
    assert m.dead and "block table" in m.dead_reason
    with pytest.raises(OMMXSlotAllocationError):
        _bmgr(graph=False, strict=True)[0].on_build(NS(seq_lens_cpu=[5], query_start_loc_cpu=[0, 1]))
    monkeypatch.setenv("OMMX_UNSAFE_ROW_INDEX_SLOTS", "1")
    m2, _ = _bmgr(graph=False)
    m2.on_build(NS(seq_lens_cpu=[5, 6], query_start_loc_cpu=[0, 1, 2]))
    assert not m2.dead and sorted(m2.slots) == [0, 1]   # row 0 is a real request, not a null block
    with pytest.raises(OMMXSlotAllocationError, match="duplicate"):
        _bmgr(graph=False, strict=True)[0].on_build(_md([5, 6], [4, 4]))


# ── config and route decisions ───────────────────────────────────────────────────────────

def test_config_defaults_are_the_serving_recipe_and_env_knobs_apply(monkeypatch):
    for k in ("OMMX_RECIPE", "OMMX_ATTN_OUTLIERS", "OMMX_ATTN_OUTLIER_REPR", "OMMX_KV_GROUP_TOKENS",
              "OMMX_ATTN_GROUP_TOKENS", "OMMX_OUTLIER_PERCENT", "OMMX_ATTN_BITMAP_READ",
              "OMMX_KV_OUTLIER_MAP", "OMMX_ATTN_POW2", "OMMX_STRICT"):
        monkeypatch.delenv(k, raising=False)
    c = resolve_serving_config(head_dim=128, n_kv_heads=8, max_context=9000)
    assert (c.k_format, c.outliers_per_vector, c.outlier_select, c.outlier_repr, c.use_pow2,
            c.kv_outlier_map, c.group_tokens, c.group_channels, c.sink_tokens, c.recent_window,
            c.page_size, c.max_context) == ("i2f4", 6, "signed", "bitmap", True, True, 32, 32, 8, 32,
                                            16, 9000)
    assert c.resolved_bitmap_read() and not c.resolved_combinadic_read()
    monkeypatch.setenv("OMMX_ATTN_OUTLIER_REPR", "relidx7")
    monkeypatch.setenv("OMMX_ATTN_GROUP_TOKENS", "64")
    monkeypatch.setenv("OMMX_OUTLIER_PERCENT", "0.1")
    c = resolve_serving_config()
    assert c.outlier_repr == "relidx7" and c.group_tokens == 64 and c.outliers_per_vector == 6
    assert not c.resolved_bitmap_read() and c.window().group_tokens == 64
    monkeypatch.setenv("OMMX_ATTN_BITMAP_READ", "1")
    with pytest.raises(ValueError, match="BITMAP_READ"):
        resolve_serving_config()
    monkeypatch.delenv("OMMX_ATTN_BITMAP_READ")
    monkeypatch.setenv("OMMX_ATTN_OUTLIER_REPR", "nibbles")
    with pytest.raises(ValueError, match="OUTLIER_REPR"):
        resolve_serving_config()
    monkeypatch.setenv("OMMX_ATTN_OUTLIER_REPR", "bitmap")
    monkeypatch.setenv("OMMX_RECIPE", "paper-kv")
    with pytest.raises(NotImplementedError):
        resolve_serving_config()


def test_builder_route_decisions():
    b = BK.OMMXCanonicalMetadataBuilder()
    s = BK.reset_worker_state(graph=False, batched=False, batched_graph=False, max_num_seqs=4)
    md = _md([50], [3], q=[0, 50])
    assert b.build(0, md) is md
    assert s.step == {"B": 1, "uniform": False, "full_prefill": True, "batched_write": False,
                      "batched_read": False}
    with pytest.raises(RuntimeError, match="migrate"):
        b.build(0, _md([51, 9], [3, 4]))               # staggered second request, no batched session
    b.build(0, _md([20, 30], [3, 4], q=[0, 20, 50]))   # a full batched prefill opens the session
    assert s.batched_session and s.step["batched_write"] and not s.step["batched_read"]
    b.build(0, _md([21, 31], [3, 4]))
    assert s.step["batched_read"]
    s = BK.reset_worker_state(graph=True, batched=False, batched_graph=False)
    with pytest.raises(RuntimeError, match="one request only"):
        b.build(0, _md([21, 31], [3, 4]))
    with pytest.raises(RuntimeError, match="unclassified"):
        b.build(0, NS())
    s = BK.reset_worker_state(graph=False, batched=False, batched_graph=False)
    b.build(0, NS())
    assert s.step["B"] == STEP_ROUTE_UNCLASSIFIED
    impl = BK.OMMXCanonicalImpl(4, 64, None, 2)
    with pytest.raises(RuntimeError, match="classif"):
        impl.forward(NS(), torch.zeros(1, 4, 64), None, None)
    with pytest.raises(RuntimeError, match="classify"):
        impl.do_kv_cache_update(NS(), torch.zeros(1, 2, 64), torch.zeros(1, 2, 64))
    assert BK.OMMXCanonicalBackend.get_impl_cls() is BK.OMMXCanonicalImpl
    assert BK.OMMXCanonicalBackend.get_builder_cls() is BK.OMMXCanonicalMetadataBuilder
    assert BK.OMMXCanonicalBackend.get_supported_kernel_block_sizes() == [16]
    BK.reset_worker_state()
