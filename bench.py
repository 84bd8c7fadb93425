"""Decode-attention benchmark: p50 microseconds per layer-step of the OMMX paged decode
operator (split-KV kernel + combine kernel) on one MI355X, Llama-3.1-8B attention shape
(32 q heads, 8 kv heads, d=128), batch 1, synthetic caches, context 1K..64K.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--ctx 65536] [--no-ladder]
                    [--no-cpu-baseline] [--batch B] [--q-heads H] [--ragged]

One step = one decode call over one batch: the split-KV launch followed by the combine
launch, operands resident in HBM, workspace preallocated.  Steps are replayed from HIP
graphs of 32 consecutive steps (the 32 layers of one model forward; eager launches if
capture fails), so K is rounded up to a multiple of 32 (``steps_requested`` /
``warmup_requested`` keep what was asked for).  Every one of the 32 layers reads its own
copy of the cache, query, tail and workspace, at its own addresses, as the layers of a model
do: 32 x 69 MB at the headline context, far beyond the 256 MB last-level cache, so every
step reads its planes from HBM.  Before anything is timed the outputs are filled with NaN,
every layer is run once and compared with the CPU checker (``parity_before_timing``); a
mismatch ends the run.  Prints ONE JSON line.  ``value`` is the p50 over the K timed steps
at the headline context; ``roofline`` is the split-KV kernel alone (algorithmic bytes of the
packed planes it must read over its average duration, against 8 TB/s); ``store`` is the
quantize-on-store kernel over the same cache (its own roofline figures); ``cpu_baseline``
is the CPU checker (dequantise-then-attend, torch on the host cores) timed on the same
workload for a bounded number of runs, and on the 1024-token configuration.
"""
from __future__ import annotations

import argparse
import dataclasses
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the split-KV kernel at the default workload (ctx 65536, 256
# splits), from rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a 256 MiB copy kernel
# (profiles/decode_ctx64k_hbm_traffic.txt); counters cannot be read from inside this script.
TRAFFIC_BYTES_CTX64K = 74.03e6
STAGE1_REP = 20
STORE_REP = 8
LAYERS = 32                  # decode steps (layers) per graph replay
H200_P50_US_64K = 563.0      # reference Triton kernel, H200 NVL, B=1 ctx 65536 (other hardware)


def _graph_or_eager(fn):
    import torch
    try:
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        g.replay()
        torch.cuda.synchronize()
        return g.replay, "hip_graph"
    except Exception as exc:                      # capture unsupported: time eager launches
        print(f"graph capture failed ({type(exc).__name__}: {exc}); timing eager launches",
              file=sys.stderr)
        torch.cuda.synchronize()
        return fn, "eager"


def _time_steps(fn, calls, warmup, per_call=1):
    """Time `calls` invocations of fn, each worth `per_call` steps.  Returns (wall ms per
    step over the whole timed region, GPU microseconds per step of each invocation)."""
    import torch
    for _ in range(warmup):
        fn()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(calls)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / (calls * per_call)
    return wall_ms, [a.elapsed_time(b) * 1e3 / per_call for a, b in ev]


def _layer_copies(case, n):
    """``n`` cases with the same contents at different addresses: the caches of n layers."""
    import torch

    def dup(v):
        return v.clone() if torch.is_tensor(v) else v
    out = [case]
    for _ in range(n - 1):
        out.append(dataclasses.replace(
            case, planes={k: dup(v) for k, v in case.planes.items()}, q=case.q.clone(),
            k_tail=case.k_tail.clone(), v_tail=case.v_tail.clone(),
            req_to_token=case.req_to_token.clone(), req_to_group=case.req_to_group.clone()))
    return out


def _make_runner(cases, splits=None):
    """Closures ``step(i)`` / ``stage1(i)`` launching the full step / the split-KV kernel alone
    on layer ``i`` with fixed buffers; ``outs[i] = (o, lse)`` of that layer."""
    import torch
    case = cases[0]
    from open_ommx_serve_amd.attention import _hip
    from open_ommx_serve_amd.attention.paged_decode import (auto_num_kv_splits, make_attn_logits,
                                                            ommx_paged_decode_attention_canonical)
    B, Hq, D = case.q.shape
    dev = case.q.device
    kw = case.decode_kwargs()
    n_cu = torch.cuda.get_device_properties(dev).multi_processor_count
    # the lengths of the synthetic requests are known on the host: pass their mean as the hint a
    # serving caller would take from its own bookkeeping
    mean_len = sum(case.packed_lens) / len(case.packed_lens)
    S = splits or auto_num_kv_splits(kw["max_seq_len"], B, case.kv_heads, n_cu, Hq // case.kv_heads,
                                     mean_seq_len=mean_len, resident=3 if Hq // case.kv_heads <= 4 else 2)
    wss = [make_attn_logits(B, Hq, S, D, dev) for _ in cases]
    outs = [(torch.empty(B, Hq, D, dtype=torch.float32, device=dev),
             torch.empty(B, Hq, dtype=torch.float32, device=dev)) for _ in cases]
    argss = [c.decode_args(*ol) for c, ol in zip(cases, outs)]
    kws = [c.decode_kwargs() for c in cases]

    def step(i=0):
        ommx_paged_decode_attention_canonical(*argss[i], num_kv_splits=S, attn_logits=wss[i], **kws[i])

    lib = _hip.load()

    def stage1(i=0):
        case, ws, p = cases[i], wss[i], cases[i].planes
        rc = lib.ommx_decode_splitkv(
            case.q.data_ptr(), case.q.stride(0), case.q.stride(1),
            p["k_base"].data_ptr(), p["k_scale"].data_ptr(), p["k_zp"].data_ptr(),
            _hip.ptr(p.get("k_fp4_mapscale")), _hip.ptr(p.get("k_fp4_mapcenter")),
            _hip.ptr(p.get("k_obmp")), _hip.ptr(p.get("k_oval")),
            p["v_main"].data_ptr(), p["v_scale"].data_ptr(), p["v_zp"].data_ptr(),
            case.req_to_token.data_ptr(), case.req_to_token.stride(0),
            case.req_to_group.data_ptr(), case.req_to_group.stride(0),
            1 if case.req_to_token.dtype == torch.int64 else 0, case.b_seq_len.data_ptr(),
            ws.data_ptr(), ws.stride(0), ws.stride(1), ws.stride(2),
            B, Hq, case.kv_heads, D, case.page_size, case.outliers_per_vector, _hip.INDEX_BITMAP, 0, 32, 32, 0, S,
            float(case.sm_scale), 0.0, 0, 0, int(p["k_base"].shape[0]), int(p["k_scale"].shape[0]), None,
            torch.cuda.current_stream(dev).cuda_stream)
        _hip.check(rc, "ommx_decode_splitkv")

    return step, stage1, outs, S


def _parity_gate(case, outs, run_layer, want=None):
    """NaN-fill the outputs, run every layer once, compare each with the CPU checker's result for
    the (shared) inputs.  Returns ``(figures, want)``; raises on a mismatch."""
    import torch
    for o, lse in outs:
        o.fill_(float("nan"))
        lse.fill_(float("nan"))
    for i in range(len(outs)):
        run_layer(i)
    torch.cuda.synchronize()
    if want is None:
        want = _cpu_reference(case, 1)[1]
    wo, wl = want[0].double(), want[1].double()
    worst = {"max_abs": 0.0, "mean_abs": 0.0, "lse_max_abs": 0.0}
    for i, (o, lse) in enumerate(outs):
        err = (o.cpu().double() - wo).abs()
        lerr = (lse.cpu().double() - wl).abs()
        fig = {"max_abs": float(err.max()), "mean_abs": float(err.mean()), "lse_max_abs": float(lerr.max())}
        if not (fig["max_abs"] <= 2e-3 and fig["mean_abs"] <= 2e-4 and fig["lse_max_abs"] <= 2e-3):
            raise RuntimeError(f"parity failure before timing, layer {i}: {fig}")
        worst = {k: max(worst[k], fig[k]) for k in worst}
    worst["layers_checked"] = len(outs)
    return worst, want


def _time_store(ctx, kv_heads=8, head_dim=128):
    """Quantize-on-store kernel over one ctx-token cache (bf16 K and V resident in HBM, serving
    recipe, identity tables): launches replayed from a graph of STORE_REP, HIP events around each
    replay.  Algorithmic bytes per (token, kv head): 512 read + 132 written."""
    import torch
    from open_ommx_serve_amd.attention.kv_window import WindowSpec
    from open_ommx_serve_amd.attention.pack import alloc_planes, store_pack_into
    from open_ommx_serve_amd.synth import synth_kv
    T = WindowSpec().packed_len(ctx)
    K, V = synth_kv(T, kv_heads, head_dim, seed=42, sparse_frac=0.005)
    K, V = K.cuda(), V.cuda()
    planes = alloc_planes(T // 16, T // 32, kv_heads, head_dim, device="cuda")
    err = torch.zeros(1, dtype=torch.int32, device="cuda")

    def rep():
        for _ in range(STORE_REP):
            store_pack_into(K, V, planes, err_flag=err)
    run, mode = _graph_or_eager(rep)
    _, us = _time_steps(run, 10, 2, per_call=STORE_REP)
    if int(err.item()):
        raise RuntimeError(f"store kernel reported error bits {int(err.item())}")
    k = statistics.mean(us)
    nbytes = T * kv_heads * (4 * head_dim + 132)
    gbps = nbytes / (k * 1e-6) / 1e9
    return {"kernel": "store_pack", "bound": "hbm", "tokens": T, "bytes_per_launch": nbytes,
            "avg_kernel_us": round(k, 2), "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS,
            "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4), "launch": mode}


def _pool_step(batch, ctx, q_heads, steps, warmup, splits=0):
    """One decode step of a serving loop on MultiSeqKVPool (ring history): the new K/V row of every
    request is written (the launch advances the device sequence counter), the sink + recent rows are
    gathered with the window arithmetic on the device, then split-KV + combine.  These four launches
    are one HIP graph; after each replay the host advances its mirror and packs the groups that
    completed (one store launch, outside the timed replay), so the gather is told that the planes
    lag the sequence by one token.  Every request gets the same synthetic rows (the kernels do not
    care).  The outputs of the first replay whose token completes a group, and of the last replay,
    are compared with the CPU checker.  Returns the JSON object."""
    import torch
    from open_ommx_serve_amd.attention import MultiSeqKVPool, WindowSpec, gather_tails, write_tokens
    from open_ommx_serve_amd.attention.paged_decode import (auto_num_kv_splits, make_attn_logits,
                                                            ommx_paged_decode_attention_canonical)
    from open_ommx_serve_amd.synth import synth_kv, synth_q
    H, D, B = 8, 128, batch
    win = WindowSpec()
    total = steps + warmup + 2
    pool = MultiSeqKVPool(D, H, num_seqs=B, max_seq_len=ctx + total + 64, window=win, device="cuda",
                          kv_ring=True, k_format="i2f4", outliers_per_vector=6, outlier_select="signed",
                          outlier_repr="bitmap", use_pow2=True)
    K, V = synth_kv(ctx + total, H, D, seed=42, sparse_frac=0.005)
    Kd, Vd = K.cuda(), V.cuda()
    for r in range(B):
        pool.append_block(r, Kd[:ctx], Vd[:ctx])
    pool.decode_seed_seq_device(range(B))
    d = pool._decode_buffers(B)
    pl = pool.pool_planes()
    newK = torch.zeros(B, H, D, dtype=torch.bfloat16, device="cuda")
    newV = torch.zeros_like(newK)
    q = synth_q(B, q_heads, D, 42).cuda()
    o = torch.empty(B, q_heads, D, dtype=torch.float32, device="cuda")
    lse = torch.empty(B, q_heads, dtype=torch.float32, device="cuda")
    n_cu = torch.cuda.get_device_properties(0).multi_processor_count
    max_seq = win.packed_len(ctx + total)
    S = splits or auto_num_kv_splits(max_seq, B, H, n_cu, q_heads // H, mean_seq_len=win.packed_len(ctx),
                                     resident=3 if q_heads // H <= 4 else 2)
    ws = make_attn_logits(B, q_heads, S, D, "cuda")

    def step():
        write_tokens(pool.k_hist, pool.v_hist, d["seq_dev"], newK, newV, pool._ring_sink, pool._ring_rec,
                     slots=d["rows"], pos_next=d["seq_dev"], err_flag=pool.err_flag)
        gather_tails(pool.k_hist, pool.v_hist, d["kt"], d["vt"], pool._ring_sink, pool._ring_rec,
                     seq=d["seq_dev"], slots=d["sel"], b_tail_len=d["b_tail"], b_seq_len=d["b_seq"],
                     window_sink=win.sink_tokens, window_recent=win.recent_window,
                     group_tokens=win.group_tokens, packed_lag=1, err_flag=pool.err_flag)
        ommx_paged_decode_attention_canonical(
            q, pl["k_base"], pl["k_scale"], pl["k_zp"], None, pl["k_oval"], pl["v_main"], pl["v_scale"],
            pl["v_zp"], d["kt"], d["vt"], d["b_tail"], o, lse, pl["req_to_token"], pl["req_to_group"],
            d["b_seq"], sm_scale=D ** -0.5, page_size=win.page_size, k_outliers_per_vector=6,
            bitmap_read=True, k_obmp=pl["k_obmp"], k_fp4_mapscale=pl["k_fp4_mapscale"],
            k_fp4_mapcenter=pl["k_fp4_mapcenter"], kv_outlier_map=True, kv_int8_scale=True,
            max_seq_len=max_seq, max_tail_len=pool.max_tail_len, num_kv_splits=S, attn_logits=ws)

    seq0 = d["seq_dev"].clone()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            step()
    torch.cuda.current_stream().wait_stream(stream)
    d["seq_dev"].copy_(seq0)                      # capture ran no kernel
    def check(s):
        """Replay s has run and the host has not packed yet: request 0 against the CPU checker."""
        import oracle.ommx_oracle as O
        n = ctx + s + 1
        edge = win.boundary(n - 1)                 # what the planes hold
        rows = list(range(min(n, win.sink_tokens))) + list(range(edge, n))
        if int(d["b_seq"][0]) != edge - win.sink_tokens or int(d["b_tail"][0]) != len(rows):
            raise RuntimeError(f"pool step {s}: lengths {int(d['b_seq'][0])}/{int(d['b_tail'][0])}, "
                               f"expected {edge - win.sink_tokens}/{len(rows)}")
        if not torch.equal(d["kt"][0, :len(rows)].cpu(), K[rows]) or \
                not torch.equal(d["vt"][0, :len(rows)].cpu(), V[rows]):
            raise RuntimeError(f"pool step {s}: gathered tail rows differ from the appended rows")
        planes = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in pool.request_planes(0).items()}
        G = planes["k_scale"].shape[0]
        wo, _ = O.decode_reference(q[:1].cpu(), planes, d["kt"][:1].cpu(), d["vt"][:1].cpu(), [len(rows)],
                                   torch.arange(2 * G).reshape(1, -1), torch.arange(G).reshape(1, -1),
                                   [edge - win.sink_tokens], sm_scale=D ** -0.5, page_size=win.page_size,
                                   dtype=torch.float32)
        err = (o[:1].cpu().double() - wo.double()).abs()
        if not (float(err.max()) <= 2e-3 and float(err.mean()) <= 2e-4):
            raise RuntimeError(f"pool step {s}: parity failure, max {float(err.max())} mean {float(err.mean())}")
        return float(err.max())

    us, packed, checked = [], 0, {}
    t0 = time.perf_counter()
    for s in range(warmup + steps):
        newK.copy_(Kd[ctx + s].unsqueeze(0).expand(B, H, D))
        newV.copy_(Vd[ctx + s].unsqueeze(0).expand(B, H, D))
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        graph.replay()
        b.record()
        completes = win.boundary(ctx + s + 1) != win.boundary(ctx + s)
        if (completes and "group_completing_step" not in checked) or s == warmup + steps - 1:
            torch.cuda.synchronize()
            checked["group_completing_step" if completes else "last_step"] = round(check(s), 6)
        packed += pool._advance_host_and_pack(range(B))      # host mirror + pack of completed groups
        torch.cuda.synchronize()
        if s == warmup:
            t0 = time.perf_counter()
        if s >= warmup:
            us.append(a.elapsed_time(b) * 1e3)
    wall_ms = (time.perf_counter() - t0) * 1e3 / max(1, steps - 1)
    pool.check_errors()
    if not bool(torch.isfinite(o).all()):
        raise RuntimeError("pool step produced non-finite output")
    p50 = statistics.median(us)
    nbytes = B * (win.packed_len(ctx) * H * 132 + 64 * H * D * 2 * 2)
    return {"metric": "p50 serving-step us/layer (ring write + tail gather + split-KV + combine)",
            "value": round(p50, 3), "unit": "us/step/layer", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(wall_ms, 6), "higher_is_better": False, "scaling": "weak",
            "vs_baseline": None, "dtype": "u8 planes, bf16 q, f32 accumulate", "data": "synthetic",
            "config": {"workload": f"MultiSeqKVPool serving step, {q_heads} q / 8 kv heads, d=128, batch {B}, "
                                   f"ctx {ctx} growing by one token per step, ring history, page 16",
                       "num_kv_splits": S, "launch": "hip_graph", "bytes_per_step": nbytes,
                       "hbm_frac_step": round(nbytes / (p50 * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                       "groups_packed_between_replays": packed, "parity_max_abs": checked,
                       "note": "ms_per_step is wall time per step including the host mirror, the pack "
                               "launches and a synchronisation per step"},
            "roofline": None, "cpu_baseline": None}


def _cpu_reference(case, runs):
    """Dequantise-then-attend on the host cores; (seconds per step list, o, lse)."""
    import torch
    import oracle.ommx_oracle as O
    planes = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in case.planes.items()}
    planes["outliers_per_vector"] = case.outliers_per_vector
    a = (case.q.cpu(), planes, case.k_tail.cpu(), case.v_tail.cpu(), case.b_tail_len.tolist(),
         case.req_to_token.cpu(), case.req_to_group.cpu(), case.b_seq_len.tolist())
    times, out = [], None
    for _ in range(runs):
        t0 = time.perf_counter()
        out = O.decode_reference(*a, sm_scale=case.sm_scale, page_size=case.page_size,
                                 dtype=torch.float32)
        times.append(time.perf_counter() - t0)
    return times, out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=640)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--ctx", type=int, default=65536)
    ap.add_argument("--splits", type=int, default=0)
    ap.add_argument("--batch", type=int, default=1,
                    help="requests per step (other workloads than the headline one, e.g. "
                         "--batch 8 --ctx 32768 --q-heads 64 for the 8-request GQA-8 configuration)")
    ap.add_argument("--q-heads", type=int, default=32)
    ap.add_argument("--ragged", action="store_true",
                    help="with --batch: request lengths uniform in [1024, ctx] (seeded) instead of "
                         "all ctx, e.g. --batch 32 --ctx 16384 --ragged")
    ap.add_argument("--no-ladder", action="store_true")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-store", action="store_true",
                    help="skip the timing of the quantize-on-store kernel (headline workload only)")
    ap.add_argument("--pool-step", action="store_true",
                    help="measure the launch-only serving step of MultiSeqKVPool instead: ring write of "
                         "one new row per request + tail gather + split-KV + combine, replayed from a "
                         "HIP graph while the host packs completed groups between replays "
                         "(e.g. --pool-step --batch 8 --ctx 32768 --q-heads 64)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy kernel (3 times), the known-size "
                         "reference that scales the FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the decode operator has no collective and every box "
              "here has a single GPU; run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    from open_ommx_serve_amd.attention import _hip
    from open_ommx_serve_amd.synth import build_decode_case
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        return 2
    if not os.path.exists(_hip.lib_path()):
        import __graft_entry__
        __graft_entry__.build()
    torch.cuda.set_device(0)
    if args.pool_step:
        print(json.dumps(_pool_step(args.batch, args.ctx, args.q_heads, args.steps, args.warmup, args.splits)))
        return 0

    def measure(ctx, steps, warmup):
        lens = [ctx] * args.batch
        if args.ragged:
            g = torch.Generator().manual_seed(4)
            lens = torch.randint(1024, ctx + 1, (args.batch,), generator=g).tolist()
        case = build_decode_case(lens, q_heads=args.q_heads, seed=42, permute_tables=True,
                                 sparse_frac=0.005)
        # one cache per layer while they fit in 48 GiB, and never fewer than 4 (4 x 69 MB is
        # already past the 256 MB last-level cache at the headline context)
        n_copies = max(4, min(LAYERS, (48 << 30) // max(1, case.algorithmic_bytes())))
        cases = _layer_copies(case, n_copies)
        step, stage1, outs, S = _make_runner(cases, args.splits or None)
        parity, want = _parity_gate(case, outs, step)
        _parity_gate(case, outs, lambda i: (stage1(i), step(i)), want)   # both closures, same result
        # one model forward runs this operator once per layer inside a single graph, so the
        # steps are timed in graphs of LAYERS consecutive steps (steps is rounded up to that)
        def layers():
            for i in range(LAYERS):
                step(i % n_copies)
        run, mode = _graph_or_eager(layers)
        calls = -(-steps // LAYERS)
        wall_ms, us = _time_steps(run, calls, max(1, -(-warmup // LAYERS)), per_call=LAYERS)
        # the kernel alone: REP launches back to back inside one graph, so that the event
        # pair brackets kernel time and not the launch latency of a one-kernel graph
        def stage1_rep():
            for i in range(STAGE1_REP):
                stage1(i % n_copies)
        run1, _ = _graph_or_eager(stage1_rep)
        _, us1 = _time_steps(run1, max(5, steps // STAGE1_REP), 2, per_call=STAGE1_REP)
        return dict(case=case, outs=outs, S=S, mode=mode, wall_ms=wall_ms, us=us, us1=us1,
                    parity=parity, want=want, layer_copies=n_copies)

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    headline = args.batch == 1 and args.q_heads == 32
    if not headline:                   # another workload: no ladder, no CPU run (it scales with the batch)
        args.no_ladder = args.no_cpu_baseline = True
    ladder = {}
    if not args.no_ladder:
        for ctx in (1024, 4096, 16384, 32768):
            if ctx == args.ctx:
                continue
            m = measure(ctx, max(LAYERS, args.steps // 2), max(3, args.warmup // 4))
            ab = m["case"].algorithmic_bytes()
            p50 = statistics.median(m["us"])
            ladder[str(ctx)] = {"p50_us": round(p50, 2), "splits": m["S"], "bytes": ab,
                                "hbm_frac": round(ab / (p50 * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}
            del m
            torch.cuda.empty_cache()

    m = measure(args.ctx, args.steps, args.warmup)
    case = m["case"]
    p50 = statistics.median(m["us"])
    step_bytes = case.algorithmic_bytes()
    L = case.packed_lens[0]
    packed_bytes = sum(case.packed_lens) * case.kv_heads * 132
    k1 = statistics.mean(m["us1"])
    achieved = packed_bytes / (k1 * 1e-6) / 1e9
    ladder[str(args.ctx)] = {"p50_us": round(p50, 2), "splits": m["S"], "bytes": step_bytes,
                             "hbm_frac": round(step_bytes / (p50 * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}

    store = None
    if headline and not args.no_store:
        store = _time_store(args.ctx)

    # the outputs the timed replays left behind must still be the checked ones
    wo = m["want"][0].double()
    after = max(float((o.cpu().double() - wo).abs().max()) for o, _ in m["outs"])
    if not after <= 2e-3:
        print(f"PARITY FAILURE after timing: max_abs {after}", file=sys.stderr)
        return 1
    parity = dict(m["parity"], max_abs_after_timing=after)

    cpu = None
    if not args.no_cpu_baseline:
        runs = 15 if args.ctx >= 32768 else 40          # about ten seconds of CPU work
        times, _ = _cpu_reference(case, runs)
        small = build_decode_case([1024], q_heads=args.q_heads, seed=42, permute_tables=True,
                                  sparse_frac=0.005)
        times_1k, _ = _cpu_reference(small, 200)
        cpu = {"value": round(statistics.median(times) * 1e6, 1), "unit": "us/step/layer",
               "cores": torch.get_num_threads(), "kind": "port",
               "sample": f"{runs} runs of the same ctx-{args.ctx} step (dequantise all planes, "
                         f"fp32 attention per q head) on {os.cpu_count()} logical CPUs",
               "ctx1024": {"value": round(statistics.median(times_1k) * 1e6, 1), "unit": "us/step/layer",
                           "sample": "200 runs of the ctx-1024 step of the same shape (the "
                                     "configuration the reference's CPU path is quoted on)"}}

    out = {
        "metric": "p50 decode-attn us/step/layer, 8B shape bs1" if headline
                  else "p50 decode-attn us/step/layer",
        "value": round(p50, 3), "unit": "us/step/layer", "n_gpus": 1,
        "steps": -(-args.steps // LAYERS) * LAYERS, "warmup": -(-args.warmup // LAYERS) * LAYERS,
        "steps_requested": args.steps, "warmup_requested": args.warmup,
        "ms_per_step": round(m["wall_ms"], 6), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": round(p50 / H200_P50_US_64K, 5) if (args.ctx == 65536 and headline) else None,
        "dtype": "u8 planes, bf16 q, f32 accumulate", "data": "synthetic",
        "config": {"workload": f"OMMX paged decode attention, {args.q_heads} q / 8 kv heads, d=128, "
                               f"batch {args.batch}, ctx {'1024..' if args.ragged else ''}{args.ctx} "
                               f"({sum(case.packed_lens) if args.ragged else L} packed tokens"
                               f"{' in all' if args.ragged else ''} + {int(case.b_tail_len[0])} bf16 "
                               f"tail rows), page 16, permuted page/group tables, K outliers 4 "
                               f"channels x12 + 0.5% x8",
                   "num_kv_splits": m["S"], "launch": m["mode"], "layer_caches": m["layer_copies"],
                   "bytes_per_step": step_bytes, "hbm_frac_step": round(
                       step_bytes / (p50 * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                   "ladder": ladder, "baseline_note": "vs_baseline = value / 563 us "
                   "(reference Triton kernel on H200 NVL, page 32; other hardware)"},
        "roofline": {"bound": "hbm", "kernel": "decode_splitkv", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": TRAFFIC_BYTES_CTX64K if (args.ctx == 65536 and not args.splits and headline) else None,
                     "traffic_source": ("profiles/decode_ctx64k_hbm_traffic.txt (rocprofv3 FETCH_SIZE + WRITE_SIZE of "
                                        "this kernel and workload, scaled by a copy kernel; a constant of the script, "
                                        "not a counter read in this run)")
                     if (args.ctx == 65536 and not args.splits and headline) else None,
                     "bytes_per_launch": packed_bytes,
                     "avg_kernel_us": round(k1, 3)},
        "cpu_baseline": cpu,
        "parity_before_timing": parity,
        "store": store,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
