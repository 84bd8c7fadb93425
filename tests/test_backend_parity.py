"""The attention-backend surface driven like a serving engine drives it (GPU): every step runs
``builder.build`` -> per layer ``do_kv_cache_update`` -> ``forward`` with duck-typed scheduler
metadata.  Decode rows are checked against the fp64 dequantise-then-attend oracle over the
request's whole history, prompt rows against textbook causal attention."""
import math
import random
from types import SimpleNamespace as NS

import pytest
import torch

import oracle.ommx_oracle as O
from open_ommx_serve_amd.attention import WindowSpec
from open_ommx_serve_amd.integration.vllm import backend as BK
from open_ommx_serve_amd.integration.vllm.config import OMMXServingConfig
from open_ommx_serve_amd.synth import synth_kv, synth_q
from test_kv_store_parity import _oracle_decode

pytestmark = pytest.mark.gpu
DEV = "cuda"
HQ, HKV, D, LAYERS = 32, 8, 128, 2
MAX_ABS, MEAN_ABS = 2e-3, 2e-4
SCALE = 1.0 / math.sqrt(D)


class _Request:
    def __init__(self, key, prompt, total, seed):
        self.key, self.prompt, self.seq = key, prompt, 0
        kv = [synth_kv(total, HKV, D, seed=seed + 17 * l, sparse_frac=0.005) for l in range(LAYERS)]
        self.K = [k for k, _ in kv]
        self.V = [v for _, v in kv]
        self.q = synth_q(total, HQ, D, seed=seed + 5)          # one query row per position


class _Engine:
    def __init__(self, max_context, recipe=None, **state):
        self.state = BK.reset_worker_state(**state)
        self.builder = BK.OMMXCanonicalMetadataBuilder()
        self.layers = [NS() for _ in range(LAYERS)]
        self.impls = [BK.OMMXCanonicalImpl(HQ, D, SCALE, HKV) for _ in range(LAYERS)]
        for im in self.impls:
            im._ommx_serving_cfg = OMMXServingConfig(max_context=max_context, head_dim=D,
                                                     n_q_heads=HQ, n_kv_heads=HKV, **(recipe or {}))
        self.win = WindowSpec()

    def step(self, batch, check):
        """``batch``: requests in row order; a request with ``seq == 0`` sends its prompt, the
        others one token.  Returns the number of rows compared."""
        spans, q_start = [], [0]
        for r in batch:
            n = r.prompt if r.seq == 0 else 1
            spans.append((r.seq, r.seq + n))
            q_start.append(q_start[-1] + n)
        md = NS(seq_lens_cpu=[b for _, b in spans], query_start_loc_cpu=q_start,
                block_table_tensor=torch.tensor([[r.key, r.key + 1] for r in batch]))
        self.builder.build(0, md)
        checked = 0
        for l, (layer, impl) in enumerate(zip(self.layers, self.impls)):
            key = torch.cat([r.K[l][a:b] for r, (a, b) in zip(batch, spans)]).to(DEV)
            val = torch.cat([r.V[l][a:b] for r, (a, b) in zip(batch, spans)]).to(DEV)
            qry = torch.cat([r.q[a:b] for r, (a, b) in zip(batch, spans)]).to(DEV)
            out = torch.full((q_start[-1], HQ, D), float("nan"), dtype=torch.float32, device=DEV)
            impl.do_kv_cache_update(layer, key, val, None, None)
            impl.forward(layer, qry, key, val, None, md, out)
            if not check:
                continue
            got = out.cpu()
            assert torch.isfinite(got).all()
            for i, (r, (a, b)) in enumerate(zip(batch, spans)):
                row = got[q_start[i + 1] - 1]
                if a == 0:       # prompt: last row against exact causal attention
                    want, _ = O.attend(r.q[b - 1], r.K[l][:b], r.V[l][:b], SCALE, dtype=torch.float64)
                    assert (row.double() - want).abs().max().item() <= 2e-5, (l, i, "prefill")
                else:
                    want, _ = _oracle_decode(r.q[b - 1:b], [r.K[l][:b]], [r.V[l][:b]], self.win, SCALE)
                    err = (row.double() - want[0]).abs()
                    assert err.max().item() <= MAX_ABS, f"layer {l} row {i} seq {b}: {err.max().item():.3e}"
                    assert err.mean().item() <= MEAN_ABS, f"layer {l} row {i} seq {b}"
                checked += 1
        for r, (_, b) in zip(batch, spans):
            r.seq = b
        return checked


@pytest.mark.parametrize("graph", [False, True])
def test_continuous_batching_with_reordered_rows_and_a_recycled_slot(graph):
    """Batched prefill, decode steps whose row order changes every step, a request that leaves,
    a new one that arrives as a whole prompt beside running one-token rows and inherits the freed
    slot, and a one-token prompt.  ``graph`` selects the launch-only write / read routes."""
    eng = _Engine(1400, graph=False, batched=True, batched_graph=graph, max_num_seqs=3)
    rng = random.Random(3)
    r0, r1, r2 = _Request(11, 700, 820, 100), _Request(25, 1029, 1150, 200), _Request(40, 37, 100, 300)
    live = [r0, r1, r2]
    assert eng.step(live, check=True) == 3 * LAYERS
    for s in range(30):
        rng.shuffle(live)
        eng.step(live, check=(s % 9 == 0))
    slot_r2 = eng.state.bmanager._key_to_slot[40]
    r3 = _Request(77, 45, 120, 400)
    live = [r0, r3, r1]                                   # r2 left; r3's prompt sits between decodes
    assert eng.step(live, check=True) == 3 * LAYERS
    assert eng.state.bmanager._key_to_slot[77] == slot_r2
    for s in range(45):
        rng.shuffle(live)
        eng.step(live, check=(s % 9 == 0 or s == 44))
    r4 = _Request(90, 1, 40, 500)                          # one-token prompt replaces r1
    live = [r4, r0, r3]
    eng.step(live, check=True)
    for s in range(12):
        eng.step(live, check=(s == 11))
    h = BK.ommx_route_health()
    assert not h["batched_dead"] and h["decode_batched"] >= LAYERS * 88 and h["decode_single"] == 0
    for p in eng.state.bmanager.pools.values():
        p.check_errors()
    assert len(eng.state.bmanager.pools) == LAYERS
    BK.reset_worker_state()


def test_single_request_route_across_two_prompts():
    """One request at a time: prompt, decode steps across group boundaries, then a new prompt that
    reuses the stores in place (same tensors, cursors reset)."""
    eng = _Engine(1200, graph=False, batched=False, batched_graph=False)
    a = _Request(5, 300, 380, 600)
    assert eng.step([a], check=True) == LAYERS
    stores = [l._ommx_store_obj for l in eng.layers]
    for s in range(75):
        eng.step([a], check=(s % 8 == 0 or s == 74))
    b = _Request(6, 1, 80, 700)                            # one-token prompt
    eng.step([b], check=True)
    for s in range(70):
        eng.step([b], check=(s % 8 == 0 or s == 69))
    c = _Request(7, 1100, 1140, 800)
    eng.step([c], check=True)
    for s in range(35):
        eng.step([c], check=(s % 8 == 0 or s == 34))
    assert [l._ommx_store_obj for l in eng.layers] == stores
    h = BK.ommx_route_health()
    assert h["decode_single"] == LAYERS * 180 and not h["single_dead"] and h["decode_batched"] == 0
    for st in stores:
        st.check_errors()
    BK.reset_worker_state()


def test_unservable_steps_raise():
    eng = _Engine(600, graph=False, batched=True, batched_graph=False, max_num_seqs=2)
    a = _Request(3, 100, 140, 900)
    eng.step([a], check=False)
    a.seq = 50                                             # pretend: 30 query rows of an 80-token sequence
    md = NS(seq_lens_cpu=[80], query_start_loc_cpu=[0, 30], block_table_tensor=torch.tensor([[3, 4]]))
    eng.builder.build(0, md)
    k = torch.zeros(30, HKV, D, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="continues from"):
        eng.impls[0].do_kv_cache_update(eng.layers[0], k, k)
    with pytest.raises(RuntimeError, match="chunked"):
        eng.impls[0].forward(eng.layers[0], torch.zeros(30, HQ, D, dtype=torch.bfloat16, device=DEV), k, k)
    BK.reset_worker_state()


def test_batched_graph_route_replays_from_a_hip_graph():
    """The launch-only write + read of every layer captured once and replayed for 40 steps; the
    host seam (slots, packing, the one control-block upload) runs between replays, and the row
    order changes from replay to replay because rows reach their slots through device buffers."""
    B, steps = 3, 40
    eng = _Engine(900, graph=False, batched=True, batched_graph=True, max_num_seqs=B)
    reqs = [_Request(11, 500, 560, 1100), _Request(25, 333, 400, 1200), _Request(40, 61, 130, 1300)]
    eng.step(reqs, check=False)
    for _ in range(3):                                      # eager steps allocate every workspace
        eng.step(reqs, check=False)
    key = [torch.zeros(B, HKV, D, dtype=torch.bfloat16, device=DEV) for _ in range(LAYERS)]
    val = [torch.zeros_like(k) for k in key]
    qry = torch.zeros(B, HQ, D, dtype=torch.bfloat16, device=DEV)
    out = [torch.zeros(B, HQ, D, dtype=torch.float32, device=DEV) for _ in range(LAYERS)]

    def forward_all():
        for l, (layer, impl) in enumerate(zip(eng.layers, eng.impls)):
            impl.do_kv_cache_update(layer, key[l], val[l], None, None)
            impl.forward(layer, qry, key[l], val[l], None, None, out[l])

    rng = random.Random(9)
    graph = None
    for s in range(steps):
        rng.shuffle(reqs)
        md = NS(seq_lens_cpu=[r.seq + 1 for r in reqs], query_start_loc_cpu=list(range(B + 1)),
                block_table_tensor=torch.tensor([[r.key, r.key + 1] for r in reqs]))
        eng.builder.build(0, md)
        for l in range(LAYERS):
            key[l].copy_(torch.stack([r.K[l][r.seq] for r in reqs]))
            val[l].copy_(torch.stack([r.V[l][r.seq] for r in reqs]))
        qry.copy_(torch.stack([r.q[r.seq] for r in reqs]))
        if graph is None:
            stream = torch.cuda.Stream()
            stream.wait_stream(torch.cuda.current_stream())
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(stream):
                with torch.cuda.graph(graph, stream=stream):
                    forward_all()
            torch.cuda.current_stream().wait_stream(stream)
        graph.replay()
        torch.cuda.synchronize()
        for r in reqs:
            r.seq += 1
        if s % 6 == 0 or s == steps - 1:
            for l in range(LAYERS):
                got = out[l].cpu()
                for i, r in enumerate(reqs):
                    want, _ = _oracle_decode(r.q[r.seq - 1:r.seq], [r.K[l][:r.seq]], [r.V[l][:r.seq]],
                                             eng.win, SCALE)
                    err = (got[i].double() - want[0]).abs()
                    assert err.max().item() <= MAX_ABS and err.mean().item() <= MEAN_ABS, (s, l, i)
    assert not eng.state.bmanager.dead
    for p in eng.state.bmanager.pools.values():
        p.check_errors()
        assert sorted(p.seq_len) == sorted(r.seq for r in reqs)
    BK.reset_worker_state()


@pytest.mark.parametrize("graph,outlier_repr", [(False, "relidx7"), (True, "relidx7"), (True, "combinadic")])
def test_ring_history_and_the_other_index_planes_through_the_backend(graph, outlier_repr, monkeypatch):
    """``OMMX_KV_RING=1`` (the pools and stores keep 104 bf16 rows per request instead of the
    whole history) with the relidx7 or the combinadic index plane chosen through the serving
    config.  The index planes name the same outlier positions, so the dequantised history — and
    the oracle — is the one of the bitmap recipe; the stored ranks are compared with the oracle's."""
    monkeypatch.setenv("OMMX_KV_RING", "1")
    recipe = {"outlier_repr": outlier_repr}
    eng = _Engine(700, recipe=recipe, graph=False, batched=True, batched_graph=graph, max_num_seqs=2)
    a, b = _Request(8, 420, 520, 1500), _Request(9, 75, 180, 1600)
    eng.step([a, b], check=True)
    for s in range(80):
        eng.step([b, a] if s % 2 else [a, b], check=(s % 10 == 0 or s == 79))
    pool = next(iter(eng.state.bmanager.pools.values()))
    assert pool.kv_ring and pool.k_hist.shape[1] == 104
    if outlier_repr == "relidx7":
        assert pool.k_oidx is not None and pool.k_obmp is None and pool.k_crank is None
    else:
        assert pool.k_crank.shape[-1] == 3 and pool.k_oidx is None
        slot = eng.state.bmanager._key_to_slot[a.key]
        got = pool.request_planes(slot)
        edge = eng.win.boundary(a.seq)
        want = O.pack_kv(a.K[0][8:edge], a.V[0][8:edge], outlier_repr="combinadic")
        assert got["outlier_repr"] == "combinadic" and got["num_tokens"] == edge - 8
        assert torch.equal(got["k_crank"].cpu(), want["k_crank"])
        assert torch.equal(got["k_obmp"].cpu(), O.bitmap_pack(O.combinadic_unpack(want["k_crank"], 6)))
    for p in eng.state.bmanager.pools.values():
        p.check_errors()
    eng = _Engine(700, recipe=recipe, graph=False, batched=False, batched_graph=False)
    c = _Request(4, 200, 300, 1700)
    eng.step([c], check=True)
    for s in range(90):
        eng.step([c], check=(s % 10 == 0 or s == 89))
    st = eng.layers[0]._ommx_store_obj
    assert st.kv_ring and st.k_hist.shape[0] == 104
    assert eng.state.manager.kv_ring and not eng.state.manager.dead
    st.check_errors()
    BK.reset_worker_state()
