"""KV store write seams on the GPU: ring copies, incremental packing, decode through the pool.

What pins what:
* ring copies are pure row moves: compared with torch indexing of the same history;
* the window arithmetic done inside the gather kernel is compared with the host closed forms
  (``WindowSpec``), which the CPU suite pins against brute force;
* incremental packing must equal, bit for bit, the oracle packer run once over the whole
  packed prefix (32-token groups are packed independently, reference kv_pool.py:563-566);
* decode through the pool's argument bundle is compared with the oracle's
  dequantise-then-attend result on the full token history (tolerance: max-abs 2e-3,
  mean-abs 2e-4).
"""
import math

import pytest
import torch

import oracle.ommx_oracle as O
from conftest import PLANE_NAMES
from open_ommx_serve_amd.attention import (CanonicalKVStore, MultiSeqKVPool, WindowSpec,
                                           gather_tails, ommx_paged_decode_attention_canonical,
                                           write_tokens)
from open_ommx_serve_amd.attention.kv_store_ops import ring_slot
from open_ommx_serve_amd.synth import synth_kv, synth_q

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-3, 2e-4
RECIPE = dict(k_format="i2f4", outliers_per_vector=6, outlier_select="signed",
              outlier_repr="bitmap", use_pow2=True)
DEV = "cuda"


def _rows(n, H, D, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, H, D, generator=g).to(torch.bfloat16)


# ── ring copies ────────────────────────────────────────────────────────────────────────

@pytest.mark.parametrize("span", [0, 96])
def test_write_tokens_matches_indexing_and_advances_the_counter(span):
    N, H, D, sink = 5, 8, 128, 8
    rows = sink + span if span else 300
    kh = torch.zeros(N, rows, H, D, dtype=torch.bfloat16, device=DEV)
    vh = torch.zeros_like(kh)
    want_k, want_v = kh.cpu().clone(), vh.cpu().clone()
    slots = torch.tensor([3, 0, 4], dtype=torch.int64, device=DEV)
    pos = torch.tensor([5, 150, 299], dtype=torch.int64, device=DEV)
    for step in range(3):
        k, v = _rows(3, H, D, 10 + step), _rows(3, H, D, 20 + step)
        p_host = pos.cpu().tolist()
        write_tokens(kh, vh, pos, k.to(DEV), v.to(DEV), sink if span else 0, span, slots=slots,
                     pos_next=pos)
        for b, s in enumerate(slots.cpu().tolist()):
            r = ring_slot(p_host[b], sink, span) if span else p_host[b]
            if r < rows:
                want_k[s, r], want_v[s, r] = k[b], v[b]
        assert pos.cpu().tolist() == [p + 1 for p in p_host]
    assert torch.equal(kh.cpu(), want_k) and torch.equal(vh.cpu(), want_v)


def test_write_outside_the_history_sets_the_error_bit_and_writes_nothing():
    kh = torch.zeros(1, 16, 2, 64, dtype=torch.bfloat16, device=DEV)
    vh = torch.zeros_like(kh)
    err = torch.zeros(1, dtype=torch.int32, device=DEV)
    pos = torch.tensor([16], dtype=torch.int64, device=DEV)
    write_tokens(kh, vh, pos, _rows(1, 2, 64, 1).to(DEV), _rows(1, 2, 64, 2).to(DEV), 0, 0, err_flag=err)
    assert int(err.item()) == 16 and not kh.any() and not vh.any()


def test_strided_source_rows_take_the_elementwise_path():
    H, D = 4, 64
    kh = torch.zeros(2, 40, H, D, dtype=torch.bfloat16, device=DEV)
    vh = torch.zeros_like(kh)
    big = _rows(2, H, D + 3, 5).to(DEV)          # rows are not 16-byte aligned
    k, v = big[:, :, 1:D + 1], big[:, :, 2:D + 2]
    pos = torch.tensor([7, 39], dtype=torch.int64, device=DEV)
    write_tokens(kh, vh, pos, k, v, 0, 0)
    assert torch.equal(kh[0, 7], k[0]) and torch.equal(kh[1, 39], k[1])
    assert torch.equal(vh[0, 7], v[0]) and torch.equal(vh[1, 39], v[1])


@pytest.mark.parametrize("ring", [False, True])
def test_gather_window_arithmetic_matches_the_host_closed_forms(ring):
    win = WindowSpec()
    sink, recent, gt = win.sink_tokens, win.recent_window, win.group_tokens
    span = recent + 2 * gt if ring else 0
    seqs = [0, 1, 5, 8, 9, 39, 40, 41, 71, 72, 73, 103, 104, 105, 135, 1000, 4096, 4097, 4135]
    N, H, D = len(seqs), 2, 64
    rows = sink + span if ring else max(seqs) + 1
    T = win.max_tail_len()
    # history row r of slot s holds the value that identifies (s, r)
    kh = (torch.arange(N * rows, dtype=torch.float32).reshape(N, rows, 1, 1) % 251).expand(
        N, rows, H, D).to(torch.bfloat16).contiguous().to(DEV)
    vh = (kh.float() + 1).to(torch.bfloat16)
    kt = torch.full((N, T, H, D), -1.0, dtype=torch.bfloat16, device=DEV)
    vt = torch.full_like(kt, -1.0)
    b_tail = torch.full((N,), -1, dtype=torch.int32, device=DEV)
    b_seq = torch.full((N,), -1, dtype=torch.int32, device=DEV)
    seq = torch.tensor(seqs, dtype=torch.int64, device=DEV)
    gather_tails(kh, vh, kt, vt, sink if ring else 0, span, seq=seq, b_tail_len=b_tail, b_seq_len=b_seq,
                 window_sink=sink, window_recent=recent, group_tokens=gt)
    kt, vt, khc, vhc = kt.cpu(), vt.cpu(), kh.cpu(), vh.cpu()
    for b, n in enumerate(seqs):
        idx = win.tail_indices(n)
        assert int(b_tail[b]) == min(len(idx), T), (n, int(b_tail[b]))
        assert int(b_seq[b]) == win.packed_len(n), (n, int(b_seq[b]))
        for t in range(T):
            p = idx[t] if t < len(idx) else 0
            r = ring_slot(p, sink, span) if ring else p
            assert torch.equal(kt[b, t], khc[b, r]) and torch.equal(vt[b, t], vhc[b, r]), (n, t)


def test_gather_explicit_positions_through_slots():
    N, rows, H, D, T = 3, 50, 2, 64, 6
    kh = _rows(N * rows, H, D, 3).reshape(N, rows, H, D).to(DEV)
    vh = _rows(N * rows, H, D, 4).reshape(N, rows, H, D).to(DEV)
    slots = torch.tensor([2, 0], dtype=torch.int64, device=DEV)
    idx = torch.tensor([[0, 1, 49, 7, 0, 0], [3, 3, 3, 10, 11, 12]], dtype=torch.int64, device=DEV)
    kt = torch.empty(2, T, H, D, dtype=torch.bfloat16, device=DEV)
    vt = torch.empty_like(kt)
    gather_tails(kh, vh, kt, vt, 0, 0, tail_idx=idx, slots=slots)
    for b in range(2):
        assert torch.equal(kt[b], kh[slots[b]].index_select(0, idx[b]))
        assert torch.equal(vt[b], vh[slots[b]].index_select(0, idx[b]))


# ── pool: incremental packing and decode ─────────────────────────────────────────────────

def _decode_bundle(q, bundle, sm_scale, k):
    pl = bundle["planes"]
    B, Hq, D = q.shape
    o = torch.full((B, Hq, D), float("nan"), dtype=torch.float32, device=q.device)
    lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=q.device)
    ommx_paged_decode_attention_canonical(
        q, pl["k_base"], pl["k_scale"], pl["k_zp"], pl.get("k_oidx"), pl["k_oval"],
        pl["v_main"], pl["v_scale"], pl["v_zp"], bundle["k_tail"], bundle["v_tail"],
        bundle["b_tail_len"], o, lse, bundle.get("req_to_token", pl["req_to_token"]),
        bundle.get("req_to_group", pl["req_to_group"]), bundle["b_seq_len"],
        sm_scale=sm_scale, page_size=pl["page_size"], k_outliers_per_vector=k,
        bitmap_read=pl.get("outlier_repr", "bitmap") == "bitmap", k_obmp=pl["k_obmp"],
        k_fp4_mapscale=pl["k_fp4_mapscale"],
        k_fp4_mapcenter=pl["k_fp4_mapcenter"], kv_outlier_map=True, kv_int8_scale=True,
        max_seq_len=bundle["max_seq_len"], max_tail_len=bundle["max_tail_len"],
        packed_start_offset=bundle["packed_start_offset"])
    torch.cuda.synchronize()
    return o.cpu(), lse.cpu()


def _oracle_decode(q, K_hist, V_hist, win, sm_scale, packed_for=None, v_format="i2"):
    """Dequantise-then-attend over the full history of every request (fp64).  ``packed_for``:
    the lengths the planes were last packed for (default: the current ones); rows past that
    boundary are attended as bf16."""
    outs, lses = [], []
    for b, (K, V) in enumerate(zip(K_hist, V_hist)):
        n = int(K.shape[0])
        edge = win.boundary(n if packed_for is None else packed_for[b])
        rows = list(range(min(n, win.sink_tokens))) + list(range(max(edge, min(n, win.sink_tokens)), n))
        assert packed_for is not None or rows == win.tail_indices(n)
        Kf = [K[i].float() for i in rows]
        Vf = [V[i].float() for i in rows]
        Kd = torch.stack(Kf) if Kf else torch.zeros(0, *K.shape[1:])
        Vd = torch.stack(Vf) if Vf else torch.zeros(0, *V.shape[1:])
        if edge > win.sink_tokens:
            planes = O.pack_kv(K[win.sink_tokens:edge], V[win.sink_tokens:edge], page_size=win.page_size,
                               v_format=v_format)
            Kp, Vp = O.dequant_kv(planes)
            Kd, Vd = torch.cat([Kp, Kd]), torch.cat([Vp, Vd])
        o, lse = O.attend(q[b].cpu(), Kd, Vd, sm_scale, dtype=torch.float64)
        outs.append(o)
        lses.append(lse)
    return torch.stack(outs), torch.stack(lses)


def _assert_planes_equal_oracle(got: dict, K, V, win, what, outlier_repr="bitmap"):
    n = int(K.shape[0])
    edge = win.boundary(n)
    assert got["num_tokens"] == max(0, edge - win.sink_tokens), what
    if edge <= win.sink_tokens:
        return
    want = O.pack_kv(K[win.sink_tokens:edge], V[win.sink_tokens:edge], page_size=win.page_size,
                     outlier_repr=outlier_repr)
    for name in PLANE_NAMES:
        if outlier_repr == "relidx7" and name == "k_obmp":
            assert got["k_obmp"] is None
            name = "k_oidx"
        a, b = got[name].cpu(), want[name]
        assert a.shape == b.shape and a.dtype == b.dtype, (what, name)
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"{what}: plane {name} differs"


def _check_out(got, want, what):
    (o, lse), (wo, wl) = got, want
    err = (o.double() - wo).abs()
    assert torch.isfinite(o).all(), what
    assert err.max().item() <= MAX_ABS, f"{what}: max-abs {err.max().item():.3e}"
    assert err.mean().item() <= MEAN_ABS, f"{what}: mean-abs {err.mean().item():.3e}"
    assert (lse.double() - wl).abs().max().item() <= 2e-3, f"{what}: lse"


@pytest.mark.parametrize("ring", [False, True])
@pytest.mark.parametrize("q_heads", [32, 64])
def test_pool_prefill_then_decode_steps(ring, q_heads):
    """Ragged prefill, then 70 appended tokens per request: every request crosses two group
    boundaries.  Planes are compared after every pack, decode output every 9th step."""
    H, D, B = 8, 128, 3
    win = WindowSpec()
    prefill = [700, 1029, 37]
    steps = 70
    sm_scale = 1.0 / math.sqrt(D)
    Ks, Vs = zip(*[synth_kv(n + steps, H, D, seed=100 + i, sparse_frac=0.005) for i, n in enumerate(prefill)])
    pool = MultiSeqKVPool(D, H, num_seqs=4, max_seq_len=1200, window=win, device=DEV, kv_ring=ring, **RECIPE)
    slot_of = [2, 0, 3]                       # requests do not sit in batch order
    for i, r in enumerate(slot_of):
        n_packed = pool.append_block(r, Ks[i][:prefill[i]].to(DEV), Vs[i][:prefill[i]].to(DEV))
        assert n_packed == win.num_groups(prefill[i])
        _assert_planes_equal_oracle(pool.request_planes(r), Ks[i][:prefill[i]], Vs[i][:prefill[i]], win,
                                    f"prefill req {i}")
    q_all = synth_q(steps, B * q_heads, D, seed=5).reshape(steps, B, q_heads, D)
    for s in range(steps):
        newK = torch.stack([Ks[i][prefill[i] + s] for i in range(B)]).to(DEV)
        newV = torch.stack([Vs[i][prefill[i] + s] for i in range(B)]).to(DEV)
        packed = pool.append_decode_batched(slot_of, newK, newV)
        cur = [prefill[i] + s + 1 for i in range(B)]
        if packed:
            for i, r in enumerate(slot_of):
                _assert_planes_equal_oracle(pool.request_planes(r), Ks[i][:cur[i]], Vs[i][:cur[i]], win,
                                            f"step {s} req {i}")
        if s % 9 == 0 or s == steps - 1:
            bundle = pool.decode_inputs_batched(slot_of)
            assert bundle["b_seq_len"].tolist() == [win.packed_len(n) for n in cur]
            assert bundle["b_tail_len"].tolist() == [len(win.tail_indices(n)) for n in cur]
            q = q_all[s].to(DEV)
            got = _decode_bundle(q, bundle, sm_scale, 6)
            want = _oracle_decode(q, [Ks[i][:cur[i]] for i in range(B)], [Vs[i][:cur[i]] for i in range(B)],
                                  win, sm_scale)
            _check_out(got, want, f"ring={ring} Hq={q_heads} step {s}")
    pool.check_errors()


@pytest.mark.parametrize("ring", [False, True])
def test_pool_with_the_relidx7_index_plane(ring):
    """The pool on the 7-bit position-stream recipe: prefill, 40 appended tokens (every request
    crosses a group boundary), planes against the oracle after every pack, decode at the end
    of each 10 steps; and a single-sequence store on the same recipe."""
    H, D, B, q_heads = 8, 128, 2, 32
    win = WindowSpec()
    prefill, steps = [300, 71], 40
    sm_scale = 1.0 / math.sqrt(D)
    recipe = {**RECIPE, "outlier_repr": "relidx7"}
    Ks, Vs = zip(*[synth_kv(n + steps, H, D, seed=500 + i, sparse_frac=0.005) for i, n in enumerate(prefill)])
    pool = MultiSeqKVPool(D, H, num_seqs=2, max_seq_len=400, window=win, device=DEV, kv_ring=ring, **recipe)
    assert pool.k_obmp is None and tuple(pool.k_oidx.shape[2:]) == (D, 6)
    for r in range(B):
        pool.append_block(r, Ks[r][:prefill[r]].to(DEV), Vs[r][:prefill[r]].to(DEV))
        _assert_planes_equal_oracle(pool.request_planes(r), Ks[r][:prefill[r]], Vs[r][:prefill[r]], win,
                                    f"prefill req {r}", "relidx7")
    q_all = synth_q(steps, B * q_heads, D, seed=6).reshape(steps, B, q_heads, D)
    for s in range(steps):
        newK = torch.stack([Ks[i][prefill[i] + s] for i in range(B)]).to(DEV)
        newV = torch.stack([Vs[i][prefill[i] + s] for i in range(B)]).to(DEV)
        packed = pool.append_decode_batched(range(B), newK, newV)
        cur = [prefill[i] + s + 1 for i in range(B)]
        if packed:
            for r in range(B):
                _assert_planes_equal_oracle(pool.request_planes(r), Ks[r][:cur[r]], Vs[r][:cur[r]], win,
                                            f"step {s} req {r}", "relidx7")
        if s % 10 == 9:
            bundle = pool.decode_inputs_batched(range(B))
            assert bundle["planes"]["outlier_repr"] == "relidx7"
            q = q_all[s].to(DEV)
            want = _oracle_decode(q, [Ks[i][:cur[i]] for i in range(B)], [Vs[i][:cur[i]] for i in range(B)],
                                  win, sm_scale)
            _check_out(_decode_bundle(q, bundle, sm_scale, 6), want, f"relidx7 ring={ring} step {s}")
    pool.check_errors()
    store = CanonicalKVStore(D, H, max_seq_len=400, window=win, device=DEV, kv_ring=ring, **recipe)
    store.append_block(Ks[0][:prefill[0]].to(DEV), Vs[0][:prefill[0]].to(DEV))
    _assert_planes_equal_oracle(store.decode_planes(), Ks[0][:prefill[0]], Vs[0][:prefill[0]], win,
                                "store", "relidx7")


@pytest.mark.parametrize("ring", [False, True])
@pytest.mark.parametrize("recipe", [
    # the reference's "low-bit lever" and "paper-kv" recipes (pack.py:334-362, recipes.py:183-200)
    dict(group_tokens=64, group_channels=64, outliers_per_vector=6, outlier_repr="relidx7", kv_outlier_map=False),
    dict(group_tokens=128, group_channels=128, outliers_per_vector=10, outlier_repr="relidx7"),
    dict(group_tokens=16, group_channels=32, outliers_per_vector=2, outlier_repr="bitmap", use_pow2=False),
])
def test_pool_other_group_sizes(recipe, ring):
    """Pool and single-sequence store with K groups of 16 / 64 / 128 tokens: the window, the ring
    span, the page / group-slot tables and the incremental packs follow the group size.  Planes
    against the oracle packer after every pack, decode against the oracle at the end."""
    H, D, B, q_heads = 4, 128, 2, 16
    gt, gc, k = recipe["group_tokens"], recipe["group_channels"], recipe["outliers_per_vector"]
    win = WindowSpec(group_tokens=gt)
    prefill, steps = [300, 45], 2 * gt + 5
    sm_scale = 1.0 / math.sqrt(D)
    okw = dict(outliers_per_vector=k, outlier_repr=recipe["outlier_repr"], group_tokens=gt, group_channels=gc,
               kv_outlier_map=recipe.get("kv_outlier_map", True), use_pow2=recipe.get("use_pow2", True))
    kw = {**RECIPE, **recipe}
    kw.pop("group_tokens")
    Ks, Vs = zip(*[synth_kv(n + steps, H, D, seed=800 + i, sparse_frac=0.005) for i, n in enumerate(prefill)])
    pool = MultiSeqKVPool(D, H, num_seqs=2, max_seq_len=1024, window=win, device=DEV, kv_ring=ring, **kw)

    def planes_equal(got, n_tok, r, what):
        edge = win.boundary(n_tok)
        assert got["num_tokens"] == max(0, edge - win.sink_tokens), what
        if edge <= win.sink_tokens:
            return
        want = O.pack_kv(Ks[r][win.sink_tokens:edge], Vs[r][win.sink_tokens:edge], page_size=win.page_size, **okw)
        for name in ("k_base", "k_scale", "k_zp", "k_obmp", "k_oidx", "k_oval", "k_fp4_mapscale",
                     "k_fp4_mapcenter", "v_main", "v_scale", "v_zp"):
            if want[name] is None:
                assert got[name] is None, (what, name)
                continue
            a, b = got[name].cpu(), want[name]
            assert a.shape == b.shape and a.dtype == b.dtype, (what, name, a.shape, b.shape)
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"{what}: plane {name} differs"

    for r in range(B):
        pool.append_block(r, Ks[r][:prefill[r]].to(DEV), Vs[r][:prefill[r]].to(DEV))
        planes_equal(pool.request_planes(r), prefill[r], r, f"prefill req {r}")
    q_all = synth_q(steps, B * q_heads, D, seed=7).reshape(steps, B, q_heads, D)
    n_packs = 0
    for s in range(steps):
        newK = torch.stack([Ks[i][prefill[i] + s] for i in range(B)]).to(DEV)
        newV = torch.stack([Vs[i][prefill[i] + s] for i in range(B)]).to(DEV)
        packed = pool.append_decode_batched(range(B), newK, newV)
        cur = [prefill[i] + s + 1 for i in range(B)]
        if packed:
            n_packs += 1
            for r in range(B):
                planes_equal(pool.request_planes(r), cur[r], r, f"step {s} req {r}")
        if s % 16 == 15 or s == steps - 1:
            bundle = pool.decode_inputs_batched(range(B))
            assert bundle["b_seq_len"].tolist() == [win.packed_len(n) for n in cur]
            pl = bundle["planes"]
            q = q_all[s].to(DEV)
            o = torch.full((B, q_heads, D), float("nan"), dtype=torch.float32, device=DEV)
            lse = torch.full((B, q_heads), float("nan"), dtype=torch.float32, device=DEV)
            ommx_paged_decode_attention_canonical(
                q, pl["k_base"], pl["k_scale"], pl["k_zp"], pl.get("k_oidx"), pl["k_oval"],
                pl["v_main"], pl["v_scale"], pl["v_zp"], bundle["k_tail"], bundle["v_tail"],
                bundle["b_tail_len"], o, lse, bundle["req_to_token"], bundle["req_to_group"], bundle["b_seq_len"],
                sm_scale=sm_scale, page_size=pl["page_size"], k_outliers_per_vector=k,
                bitmap_read=pl["outlier_repr"] == "bitmap", k_obmp=pl["k_obmp"],
                k_fp4_mapscale=pl["k_fp4_mapscale"], k_fp4_mapcenter=pl["k_fp4_mapcenter"],
                kv_outlier_map=pl["kv_outlier_map"], kv_int8_scale=pl["kv_int8_scale"],
                max_seq_len=bundle["max_seq_len"], max_tail_len=bundle["max_tail_len"],
                packed_start_offset=bundle["packed_start_offset"])
            torch.cuda.synchronize()
            outs, lses = [], []
            for b in range(B):
                n = cur[b]
                edge = win.boundary(n)
                ti = win.tail_indices(n)
                Kd = torch.stack([Ks[b][i].float() for i in ti])
                Vd = torch.stack([Vs[b][i].float() for i in ti])
                if edge > win.sink_tokens:
                    Kp, Vp = O.dequant_kv(O.pack_kv(Ks[b][win.sink_tokens:edge], Vs[b][win.sink_tokens:edge],
                                                    page_size=win.page_size, **okw))
                    Kd, Vd = torch.cat([Kp, Kd]), torch.cat([Vp, Vd])
                ob, lb = O.attend(q[b].cpu(), Kd, Vd, sm_scale, dtype=torch.float64)
                outs.append(ob); lses.append(lb)
            _check_out((o.cpu(), lse.cpu()), (torch.stack(outs), torch.stack(lses)), f"{recipe} ring={ring} step {s}")
    assert n_packs >= 2
    pool.check_errors()
    store = CanonicalKVStore(D, H, max_seq_len=1024, window=win, device=DEV, kv_ring=ring, **kw)
    store.append_block(Ks[0][:prefill[0]].to(DEV), Vs[0][:prefill[0]].to(DEV))
    planes_equal(store.decode_planes(), prefill[0], 0, "store")


def test_pool_device_counter_path_equals_the_host_path():
    """append_decode_device / decode_inputs_device (device sequence counter) against
    append_decode_batched / decode_inputs_batched on a second pool fed the same rows."""
    H, D, B, steps = 2, 64, 3, 40
    win = WindowSpec()
    prefill = [45, 72, 100]
    Ks, Vs = zip(*[synth_kv(n + steps, H, D, seed=300 + i) for i, n in enumerate(prefill)])
    pools = [MultiSeqKVPool(D, H, num_seqs=B, max_seq_len=200, window=win, device=DEV, kv_ring=True, **RECIPE)
             for _ in range(2)]
    for p in pools:
        for i in range(B):
            p.append_block(i, Ks[i][:prefill[i]].to(DEV), Vs[i][:prefill[i]].to(DEV))
    pools[0].decode_seed_seq_device(range(B))
    for s in range(steps):
        newK = torch.stack([Ks[i][prefill[i] + s] for i in range(B)]).to(DEV)
        newV = torch.stack([Vs[i][prefill[i] + s] for i in range(B)]).to(DEV)
        n0 = pools[0].append_decode_device(newK, newV, B)
        n1 = pools[1].append_decode_batched(range(B), newK, newV)
        assert n0 == n1
        a = pools[0].decode_inputs_device(B, 200)
        b = pools[1].decode_inputs_batched(range(B))
        assert torch.equal(a["b_seq_len"], b["b_seq_len"]) and torch.equal(a["b_tail_len"], b["b_tail_len"])
        for i in range(B):
            n = int(a["b_tail_len"][i])
            assert torch.equal(a["k_tail"][i, :n], b["k_tail"][i, :n])
            assert torch.equal(a["v_tail"][i, :n], b["v_tail"][i, :n])
    for name in PLANE_NAMES:
        assert torch.equal(getattr(pools[0], name), getattr(pools[1], name)), name
    assert pools[0]._dbuf["seq_dev"][:B].tolist() == [prefill[i] + steps for i in range(B)]
    pools[0].check_errors()


def test_pool_with_values_beyond_the_f16_operands_is_served_by_the_plain_kernel():
    """K values in the millions give steps above 2^15, which the matrix-core decode cannot carry.  Nobody
    passes a flag: the store kernel notes such a step in the pool's own error word, the pool's plane dicts
    carry that word to the decode, and ``check_errors`` (a) raises if a decode already met such a step and
    (b) sends every later decode of this pool to the plain kernel, whose output matches the oracle."""
    from open_ommx_serve_amd.attention.reference_op import ommx_paged_decode
    H, D, Hq = 8, 128, 32
    win = WindowSpec()
    n = 400
    K, V = synth_kv(n, H, D, seed=77, sparse_frac=0.0)
    K = (K.float() * 1.0e6).to(torch.bfloat16)
    q = synth_q(1, Hq, D, seed=9).reshape(1, Hq, D).to(DEV)
    q = (q.float() * 1.0e-6).to(torch.bfloat16)          # keeps the logits of order one
    sm_scale = 1.0 / math.sqrt(D)
    want = _oracle_decode(q, [K], [V], win, sm_scale)

    def decode(pool):
        b = pool.decode_inputs_batched([1])
        o, lse = ommx_paged_decode(q, b["planes"], b["k_tail"], b["v_tail"], b["b_tail_len"], b["b_seq_len"],
                                   sm_scale=sm_scale, max_seq_len=b["max_seq_len"], max_tail_len=b["max_tail_len"])
        torch.cuda.synchronize()
        return o.cpu(), lse.cpu()

    # (a) decode before anybody looked at the error word: reported at the next check
    pool = MultiSeqKVPool(D, H, num_seqs=2, max_seq_len=512, window=win, device=DEV, **RECIPE)
    pool.append_block(1, K.to(DEV), V.to(DEV))
    assert int(pool.k_scale.to(torch.int32).max()) > 15
    decode(pool)
    with pytest.raises(ValueError, match="2\\^15"):
        pool.check_errors()
    assert pool.wide_steps
    got = decode(pool)                                     # now on the plain kernel
    assert (got[0].double() - want[0]).abs().max().item() <= MAX_ABS
    assert ((got[1].double() - want[1]).abs() <= 2e-3 + 2e-6 * want[1].abs()).all()
    pool.check_errors()
    # (b) checked after the pack, before the first decode: nothing is ever served wrong
    pool = MultiSeqKVPool(D, H, num_seqs=2, max_seq_len=512, window=win, device=DEV, **RECIPE)
    pool.append_block(1, K.to(DEV), V.to(DEV))
    pool.check_errors()
    assert pool.wide_steps
    got = decode(pool)
    assert (got[0].double() - want[0]).abs().max().item() <= MAX_ABS
    pool.check_errors()


def test_pool_raises_for_a_table_entry_outside_the_planes():
    from open_ommx_serve_amd.attention.reference_op import ommx_paged_decode
    H, D, Hq = 8, 128, 32
    K, V = synth_kv(200, H, D, seed=78)
    pool = MultiSeqKVPool(D, H, num_seqs=2, max_seq_len=256, window=WindowSpec(), device=DEV, **RECIPE)
    pool.append_block(0, K.to(DEV), V.to(DEV))
    b = pool.decode_inputs_batched([0])
    b["planes"]["req_to_token"] = b["planes"]["req_to_token"].clone()
    b["planes"]["req_to_token"][0, 2] = 1 << 20             # a page far outside the pool
    q = synth_q(1, Hq, D, seed=3).reshape(1, Hq, D).to(DEV)
    o, _ = ommx_paged_decode(q, b["planes"], b["k_tail"], b["v_tail"], b["b_tail_len"], b["b_seq_len"],
                             sm_scale=0.1, max_seq_len=b["max_seq_len"], max_tail_len=b["max_tail_len"])
    assert torch.isfinite(o).all()                           # the entry was held inside the planes
    with pytest.raises(IndexError, match="outside the planes"):
        pool.check_errors()


def test_pool_reports_non_finite_rows_lazily():
    H, D = 2, 64
    pool = MultiSeqKVPool(D, H, num_seqs=1, max_seq_len=200, device=DEV, kv_ring=False, **RECIPE)
    K, V = synth_kv(80, H, D, seed=1)
    K[20, 1, 5] = float("nan")
    pool.append_block(0, K.to(DEV), V.to(DEV))
    with pytest.raises((ValueError, IndexError)):
        pool.check_errors()
    pool.check_errors()                      # the flag was cleared by the first read


# ── single-sequence store ───────────────────────────────────────────────────────────────

@pytest.mark.parametrize("ring", [False, True])
def test_store_prefill_write_token_advance_and_decode(ring):
    H, D, Hq = 8, 128, 32
    win = WindowSpec()
    prefill, steps = 300, 40
    K, V = synth_kv(prefill + steps, H, D, seed=77, sparse_frac=0.005)
    st = CanonicalKVStore(D, H, max_seq_len=512, window=win, device=DEV, kv_ring=ring, **RECIPE)
    st.append_block(K[:prefill].to(DEV), V[:prefill].to(DEV))
    pos = torch.zeros(1, dtype=torch.int64, device=DEV)
    sm_scale = 1.0 / math.sqrt(D)
    qs = synth_q(steps, Hq, D, seed=9)
    for s in range(steps):
        n = prefill + s + 1
        pos.fill_(n - 1)
        st.write_token(pos, K[n - 1].to(DEV), V[n - 1].to(DEV))
        packed = st.advance_to(n)
        assert packed == win.newly_completed_groups(n - 1, n)
        if packed or s == 0:
            got = st.decode_planes()
            _assert_planes_equal_oracle(got, K[:n], V[:n], win, f"store step {s}")
        # fixed-buffer gather (the graph path) and the allocating one agree
        idx = win.tail_indices(n)
        tidx = torch.zeros(st.tail_cap, dtype=torch.int64, device=DEV)
        tidx[:len(idx)] = torch.tensor(idx)
        st.gather_tail_into(tidx, st.k_tail_buf, st.v_tail_buf, len(idx))
        kt, vt, nt = st.tail_bf16()
        assert nt == len(idx)
        assert torch.equal(st.k_tail_buf[0, :nt], kt[0]) and torch.equal(kt[0].cpu(), K[idx])
        assert torch.equal(st.v_tail_buf[0, :nt], vt[0]) and torch.equal(vt[0].cpu(), V[idx])
        if s % 13 == 0 or s == steps - 1:
            bundle = st.decode_inputs()
            q = qs[s:s + 1].to(DEV)
            got = _decode_bundle(q, bundle, sm_scale, 6)
            want = _oracle_decode(q, [K[:n]], [V[:n]], win, sm_scale)
            _check_out(got, want, f"store ring={ring} step {s}")
    st.check_errors()
    st.reset_inplace()
    assert st.seq_len == 0 and st.packed_groups == 0


@pytest.mark.parametrize("ring", [False, True])
def test_store_with_v_kept_as_bf16_rows(ring):
    """``v_format="bf16"`` on the single-sequence store (kv_store.py:120-127, 183-188): V rows go
    into ``v_main`` as they come, K is packed as always.  Planes bit for bit against the oracle
    packer after the prefill and after every incremental pack, decode against the oracle."""
    H, D, Hq = 4, 128, 16
    win = WindowSpec()
    prefill, steps = 200, 40
    K, V = synth_kv(prefill + steps, H, D, seed=91, sparse_frac=0.005)
    st = CanonicalKVStore(D, H, max_seq_len=400, window=win, device=DEV, kv_ring=ring, v_format="bf16", **RECIPE)
    assert st.v_main.dtype == torch.bfloat16 and tuple(st.v_main.shape[1:]) == (win.page_size, H, D)

    def planes_equal(n, what):
        got, edge = st.decode_planes(), win.boundary(n)
        assert got["v_format"] == "bf16" and got["num_tokens"] == edge - win.sink_tokens
        want = O.pack_kv(K[win.sink_tokens:edge], V[win.sink_tokens:edge], page_size=win.page_size, v_format="bf16")
        for name in PLANE_NAMES:
            a, b = got[name].cpu(), want[name]
            assert a.shape == b.shape and a.dtype == b.dtype, (what, name, a.shape, b.shape, a.dtype, b.dtype)
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"{what}: plane {name} differs"

    st.append_block(K[:prefill].to(DEV), V[:prefill].to(DEV))
    planes_equal(prefill, "prefill")
    pos = torch.zeros(1, dtype=torch.int64, device=DEV)
    sm_scale = 1.0 / math.sqrt(D)
    qs = synth_q(steps, Hq, D, seed=10)
    packs = 0
    for s in range(steps):
        n = prefill + s + 1
        pos.fill_(n - 1)
        st.write_token(pos, K[n - 1].to(DEV), V[n - 1].to(DEV))
        if st.advance_to(n):
            packs += 1
            planes_equal(n, f"step {s}")
        if s % 13 == 0 or s == steps - 1:
            q = qs[s:s + 1].to(DEV)
            got = _decode_bundle(q, st.decode_inputs(), sm_scale, 6)
            want = _oracle_decode(q, [K[:n]], [V[:n]], win, sm_scale, v_format="bf16")
            _check_out(got, want, f"bf16 V store ring={ring} step {s}")
    assert packs >= 1
    st.check_errors()


def test_store_reports_a_position_outside_its_history():
    """The launch-only write and gather of the single-sequence store carry the store's error
    flag: a position beyond the history is dropped / zero-filled on the device and
    ``check_errors`` raises what the reference's assert would have."""
    H, D = 2, 64
    st = CanonicalKVStore(D, H, max_seq_len=128, device=DEV, kv_ring=False, **RECIPE)
    K, V = synth_kv(4, H, D, seed=5)
    rows = int(st.k_hist.shape[0])
    st.write_token(torch.tensor([3], device=DEV), K[0].to(DEV), V[0].to(DEV))
    st.check_errors()
    before = st.k_hist.clone()
    st.write_token(torch.tensor([rows + 7], device=DEV), K[1].to(DEV), V[1].to(DEV))
    with pytest.raises(IndexError):
        st.check_errors()
    assert torch.equal(st.k_hist, before)
    st.check_errors()                                   # the flag was cleared by the raise
    T = 8
    kt = torch.ones(1, T, H, D, dtype=torch.bfloat16, device=DEV)
    vt = torch.ones_like(kt)
    idx = torch.tensor([3, 0, 0, rows + 1, 0, 0, 0, 0], dtype=torch.int64, device=DEV)
    st.gather_tail_into(idx, kt, vt, 4)
    with pytest.raises(IndexError):
        st.check_errors()
    assert torch.equal(kt[0, 0].cpu(), K[0]) and not kt[0, 3].any()


def test_eager_append_matches_write_token():
    H, D = 2, 64
    K, V = synth_kv(120, H, D, seed=3)
    a = CanonicalKVStore(D, H, max_seq_len=128, device=DEV, kv_ring=True, **RECIPE)
    b = CanonicalKVStore(D, H, max_seq_len=128, device=DEV, kv_ring=True, **RECIPE)
    pos = torch.zeros(1, dtype=torch.int64, device=DEV)
    for n in range(120):
        a.append(K[n].to(DEV), V[n].to(DEV))
        a.maybe_regroup()
        pos.fill_(n)
        b.write_token(pos, K[n].to(DEV), V[n].to(DEV))
        b.advance_to(n + 1)
    assert a.packed_groups == b.packed_groups == WindowSpec().num_groups(120)
    assert torch.equal(a.k_hist, b.k_hist) and torch.equal(a.v_hist, b.v_hist)
    for name in PLANE_NAMES:
        assert torch.equal(getattr(a, name), getattr(b, name)), name


def test_config5_bulk_pack_then_128_decode_steps_at_full_size():
    """64 q / 8 kv heads, 8 requests of 32768 tokens: bulk-pack 32704 tokens per request, then
    128 decode steps, each appending one token per request (4 incremental packs per request)
    and decoding.  Full-size checks are properties plus the oracle on one request:
    * after the last step the pool planes of every request equal ONE store launch over the
      whole packed prefix of its history (incremental == bulk, bit for bit), and request 0's
      also equal the oracle packer's planes;
    * tails equal the history rows the window names;
    * decode output of request 0 against the oracle at the first, a middle and the last
      step; every step's output is finite and every request's lse is consistent with a
      second decode through a different split count."""
    from open_ommx_serve_amd.attention.pack import alloc_planes, store_pack_into
    H, D, Hq, B = 8, 128, 64, 8
    ctx, steps = 32768, 128
    win = WindowSpec()
    sm_scale = 1.0 / math.sqrt(D)
    pool = MultiSeqKVPool(D, H, num_seqs=B, max_seq_len=ctx + steps, window=win, device=DEV,
                          kv_ring=True, **RECIPE)
    Ks, Vs = [], []
    for i in range(B):
        K, V = synth_kv(ctx + steps, H, D, seed=500 + i, sparse_frac=0.005)
        Ks.append(K)
        Vs.append(V)
        assert pool.append_block(i, K[:ctx].to(DEV), V[:ctx].to(DEV)) == 1022
    assert pool.packed_groups == [1022] * B          # 32704 packed tokens per request
    pool.decode_seed_seq_device(range(B))
    qs = synth_q(steps, B * Hq, D, seed=6).reshape(steps, B, Hq, D)
    packs = 0
    for s in range(steps):
        newK = torch.stack([Ks[i][ctx + s] for i in range(B)]).to(DEV)
        newV = torch.stack([Vs[i][ctx + s] for i in range(B)]).to(DEV)
        packs += pool.append_decode_device(newK, newV, B)
        bundle = pool.decode_inputs_device(B, ctx + steps)
        q = qs[s].to(DEV)
        o, lse = _decode_bundle(q, bundle, sm_scale, 6)
        assert torch.isfinite(o).all() and torch.isfinite(lse).all(), s
        n = ctx + s + 1
        if s in (0, 70, steps - 1):
            want = _oracle_decode(q[:1], [Ks[0][:n]], [Vs[0][:n]], win, sm_scale)
            _check_out((o[:1], lse[:1]), want, f"config 5 step {s}")
    assert packs == 4 * B and pool.packed_groups == [1026] * B
    pool.check_errors()
    n = ctx + steps
    edge = win.boundary(n)
    for i in range(B):
        got = pool.request_planes(i)
        ref = alloc_planes(got["k_base"].shape[0], got["k_scale"].shape[0], H, D, device=DEV)
        store_pack_into(Ks[i][win.sink_tokens:edge].to(DEV), Vs[i][win.sink_tokens:edge].to(DEV), ref)
        for name in PLANE_NAMES:
            assert torch.equal(got[name], ref[name]), f"req {i} plane {name}: incremental != bulk"
        kt, vt, bt = pool.tail_bf16_batched([i])
        idx = win.tail_indices(n)
        assert int(bt[0]) == len(idx)
        assert torch.equal(kt[0, :len(idx)].cpu(), Ks[i][idx]) and torch.equal(vt[0, :len(idx)].cpu(), Vs[i][idx])
    _assert_planes_equal_oracle(pool.request_planes(0), Ks[0][:n], Vs[0][:n], win, "config 5 req 0")


def test_decode_step_replayed_from_a_hip_graph():
    """One captured step = ring write (device counter advanced in the launch) + tail gather with
    the window arithmetic + split-KV decode + combine.  Replayed 40 times while the host packs
    completed groups between replays, and compared with an eager pool fed the same rows."""
    H, D, Hq, B, steps = 8, 128, 32, 2, 40
    win = WindowSpec()
    prefill = [500, 333]
    sm_scale = 1.0 / math.sqrt(D)
    Ks, Vs = zip(*[synth_kv(n + steps, H, D, seed=700 + i, sparse_frac=0.005) for i, n in enumerate(prefill)])
    pools = [MultiSeqKVPool(D, H, num_seqs=B, max_seq_len=600, window=win, device=DEV, kv_ring=True, **RECIPE)
             for _ in range(2)]
    for p in pools:
        for i in range(B):
            p.append_block(i, Ks[i][:prefill[i]].to(DEV), Vs[i][:prefill[i]].to(DEV))
    g_pool, e_pool = pools
    g_pool.decode_seed_seq_device(range(B))
    d = g_pool._decode_buffers(B)
    # fixed-address inputs and outputs of the captured step
    newK = torch.zeros(B, H, D, dtype=torch.bfloat16, device=DEV)
    newV = torch.zeros_like(newK)
    q = torch.zeros(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    o = torch.zeros(B, Hq, D, dtype=torch.float32, device=DEV)
    lse = torch.zeros(B, Hq, dtype=torch.float32, device=DEV)
    from open_ommx_serve_amd.attention import make_attn_logits
    S = 16
    ws = make_attn_logits(B, Hq, S, D, DEV)
    pl = g_pool.pool_planes()

    def step():
        write_tokens(g_pool.k_hist, g_pool.v_hist, d["seq_dev"], newK, newV, g_pool._ring_sink,
                     g_pool._ring_rec, slots=d["rows"], pos_next=d["seq_dev"], err_flag=g_pool.err_flag)
        gather_tails(g_pool.k_hist, g_pool.v_hist, d["kt"], d["vt"], g_pool._ring_sink, g_pool._ring_rec,
                     seq=d["seq_dev"], slots=d["sel"], b_tail_len=d["b_tail"], b_seq_len=d["b_seq"],
                     window_sink=win.sink_tokens, window_recent=win.recent_window, group_tokens=win.group_tokens,
                     packed_lag=1, err_flag=g_pool.err_flag)
        ommx_paged_decode_attention_canonical(
            q, pl["k_base"], pl["k_scale"], pl["k_zp"], None, pl["k_oval"], pl["v_main"], pl["v_scale"],
            pl["v_zp"], d["kt"], d["vt"], d["b_tail"], o, lse, pl["req_to_token"], pl["req_to_group"],
            d["b_seq"], sm_scale=sm_scale, page_size=win.page_size, k_outliers_per_vector=6,
            bitmap_read=True, k_obmp=pl["k_obmp"], k_fp4_mapscale=pl["k_fp4_mapscale"],
            k_fp4_mapcenter=pl["k_fp4_mapcenter"], kv_outlier_map=True, kv_int8_scale=True,
            max_seq_len=600, max_tail_len=g_pool.max_tail_len, num_kv_splits=S, attn_logits=ws)

    # The host packs between replays, so the captured step decodes BEFORE the pack of its own
    # append: its tail gather is told that the planes lag the sequence by one token
    # (packed_lag=1) and reads the group that token may have completed from the ring.
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    qs = synth_q(steps, B * Hq, D, seed=8).reshape(steps, B, Hq, D)
    with torch.cuda.stream(stream):
        newK.copy_(torch.stack([Ks[i][prefill[i]] for i in range(B)]))
        newV.copy_(torch.stack([Vs[i][prefill[i]] for i in range(B)]))
        q.copy_(qs[0])
        seq_before = d["seq_dev"].clone()
        with torch.cuda.graph(graph, stream=stream):
            step()
        d["seq_dev"].copy_(seq_before)          # capture does not run the kernels
    torch.cuda.current_stream().wait_stream(stream)
    completed_steps = 0
    for s in range(steps):
        newK.copy_(torch.stack([Ks[i][prefill[i] + s] for i in range(B)]))
        newV.copy_(torch.stack([Vs[i][prefill[i] + s] for i in range(B)]))
        q.copy_(qs[s])
        graph.replay()
        torch.cuda.synchronize()
        # eager mirror: same write, same decode inputs (before packing), then pack
        write_tokens(e_pool.k_hist, e_pool.v_hist,
                     torch.tensor([e_pool.seq_len[i] for i in range(B)], dtype=torch.int64, device=DEV),
                     newK, newV, e_pool._ring_sink, e_pool._ring_rec)
        cur = [prefill[i] + s + 1 for i in range(B)]
        assert d["seq_dev"].tolist() == cur
        # what the captured step attended: packed prefix as of the last host pack + tail as of now
        want_o, want_l = [], []
        completing = 0
        for i in range(B):
            n, packed_groups = cur[i], g_pool.packed_groups[i]
            assert int(d["b_seq"][i]) == win.packed_len(n - 1) == packed_groups * win.group_tokens
            assert int(d["b_tail"][i]) == n - win.packed_len(n - 1)
            completing += win.packed_len(n) != win.packed_len(n - 1)
            wo, wl = _oracle_decode(q[i:i + 1], [Ks[i][:n]], [Vs[i][:n]], win, sm_scale, packed_for=[n - 1])
            _check_out((o[i:i + 1].cpu(), lse[i:i + 1].cpu()), (wo, wl), f"replay {s} req {i}")
        completed_steps += completing
        # host seam between replays: advance the mirrors and pack what completed
        packed = g_pool._advance_host_and_pack(range(B))
        assert packed == e_pool._advance_host_and_pack(range(B))
    assert completed_steps >= B                 # steps whose token completed a group were checked too
    for name in PLANE_NAMES:
        assert torch.equal(getattr(g_pool, name), getattr(e_pool, name)), name
    assert torch.equal(g_pool.k_hist, e_pool.k_hist) and torch.equal(g_pool.v_hist, e_pool.v_hist)
    g_pool.check_errors()
