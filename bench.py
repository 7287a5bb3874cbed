#!/usr/bin/env python3
"""Decode-step attention benchmark of the OmniKV selection path on one MI355X.

Workload (default, `ctx128k_bs1`): batch 1, Llama-3-8B geometry (32 q heads, 8 kv
heads, head_dim 128), bf16, 131072 prompt tokens with all 32 layers' K and V
resident in HBM, first decode step (one generated token in the tail).  Layer
schedule of the reference's example configuration: filter layers 2, 8, 18 (dense
attention + scoring of the prompt tokens in the same pass, then top-k of
int(0.067*N) tokens), one wait-load dense layer after each filter layer, dense
layers 0-1, sparse attention over the selected rows + tail everywhere else.
One step = the attention work of one decode step over all 32 layers.

Prints ONE JSON line: metric = microseconds of attention per layer (step time /
32), plus `roofline` for the dominant kernel (dense split attention) and
`cpu_baseline` (the CPU oracle timed on this host on a bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dense split pass from rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE
# (profiles/dense_split_pass_pmc.txt), keyed by (context, tail, dtype); None when not measured.
TRAFFIC_BYTES = {(131072, 1, "bf16"): 537.1e6 + 1.04e6}
HQ, HKV, D, LAYERS = 32, 8, 128, 32
FILTER_LAYERS = (2, 8, 18)
WAIT = 1


def schedule():
    """layer -> ('dense' | 'filter' | 'sparse', filter layer feeding it)."""
    sel = list(FILTER_LAYERS)
    full = list(range(0, sel[0])) + sel + [LAYERS]
    kind = {}
    for lo in full[:-1]:
        hi = min(x for x in full if x > lo)
        for i in range(lo, min(hi, lo + WAIT + 1)):
            kind[i] = ("filter" if i in sel else "dense", lo)
        for i in range(min(hi, lo + WAIT + 1), hi):
            kind[i] = ("sparse", lo)
    return kind


def build_cache(n, tail_cap, dtype, device, layout):
    """Per layer K and V as (1, HKV, n + tail_cap, D) views; filter layers carry
    the seeded sink / heavy-hitter distribution, the others device-side N(0,1)."""
    from omnikv_amd import synth

    ks, vs, qs = [], [], []
    gen = torch.Generator(device=device).manual_seed(4321)
    for l in range(LAYERS):
        rows = n + tail_cap
        if layout == "token_major":
            kbuf = torch.empty((1, rows, HKV, D), dtype=dtype, device=device).permute(0, 2, 1, 3)
            vbuf = torch.empty((1, rows, HKV, D), dtype=dtype, device=device).permute(0, 2, 1, 3)
        else:
            kbuf = torch.empty((1, HKV, rows, D), dtype=dtype, device=device)
            vbuf = torch.empty((1, HKV, rows, D), dtype=dtype, device=device)
        if l in FILTER_LAYERS:
            q, k, v = synth.filter_layer_inputs(n, HQ, HKV, D, seed=synth.SEED_DATA + l)
            kbuf[:, :, :n].copy_(k.to(dtype))
            vbuf[:, :, :n].copy_(v.to(dtype))
            kbuf[:, :, n:].normal_(generator=gen)
            vbuf[:, :, n:].normal_(generator=gen)
            qs.append(q.to(dtype).to(device))
            del k, v
        else:
            kbuf.normal_(generator=gen)
            vbuf.normal_(generator=gen)
            qs.append(torch.randn((1, HQ, 1, D), generator=gen, device=device, dtype=torch.float32).to(dtype))
        ks.append(kbuf)
        vs.append(vbuf)
    return ks, vs, qs


def make_step(ks, vs, qs, n, tail, k_sel, selector):
    from omnikv_amd import ops

    kinds = schedule()

    def step():
        idx = {}
        outs = []
        for l in range(LAYERS):
            kind, src = kinds[l]
            kfull, vfull = ks[l][:, :, : n + tail], vs[l][:, :, : n + tail]
            if kind == "dense":
                outs.append(ops.dense_attn(qs[l], kfull, vfull))
            elif kind == "filter":
                o, sc = ops.dense_attn(qs[l], kfull, vfull, selector=selector, score_len=n)
                idx[l] = ops.topk(sc, k_sel)
                outs.append(o)
            else:
                outs.append(ops.sparse_attn(qs[l], ks[l][:, :, :n], vs[l][:, :, :n], idx=idx[src],
                                            tail_k=ks[l][:, :, n: n + tail], tail_v=vs[l][:, :, n: n + tail]))
        return outs, idx

    return step


def time_events(fn, reps, stream):
    """Average milliseconds of fn() between two events on `stream`."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        fn()
    e1.record(stream)
    e1.synchronize()
    return e0.elapsed_time(e1) / reps


def cpu_baseline(n, k_sel, selector, budget_s=25.0):
    """The CPU oracle on this host: one dense layer, one filter layer (score +
    top-k + dense attention) and one sparse layer (gather + cat + attention) at
    the benchmark's context length in fp32, scaled to the 32-layer schedule."""
    from omnikv_amd import synth
    from oracle import okv_oracle as orc

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    q, k, v = synth.filter_layer_inputs(n, HQ, HKV, D)
    qn = synth.fresh_q()
    tk, tv = torch.randn(1, HKV, 1, D), torch.randn(1, HKV, 1, D)

    def t(fn, reps):
        best = []
        for _ in range(reps):
            s = time.perf_counter()
            r = fn()
            best.append(time.perf_counter() - s)
        best.sort()
        return best[len(best) // 2], r

    t0 = time.perf_counter()
    dense_s, _ = t(lambda: orc.gqa_attention(q, k, v), 1)
    reps = 3 if (time.perf_counter() - t0) * 8 < budget_s else 1
    dense_s, _ = t(lambda: orc.gqa_attention(q, k, v), reps)
    score_s, sc = t(lambda: orc.score_tokens(q, k, n, selector), reps)
    topk_s, idx = t(lambda: orc.select_topk(sc, k_sel), reps)

    def sparse():
        pk = torch.cat([orc.gather_rows(k, idx[0]), tk], dim=-2)
        pv = torch.cat([orc.gather_rows(v, idx[0]), tv], dim=-2)
        return orc.gqa_attention(qn, pk, pv)

    sparse_s, _ = t(sparse, max(reps, 3))
    kinds = schedule()
    nd = sum(1 for x in kinds.values() if x[0] in ("dense", "filter"))
    nf = sum(1 for x in kinds.values() if x[0] == "filter")
    ns = sum(1 for x in kinds.values() if x[0] == "sparse")
    step_s = nd * dense_s + nf * (score_s + topk_s) + ns * sparse_s
    return {
        "value": step_s * 1e6 / LAYERS,
        "unit": "us/layer",
        "cores": cores,
        "kind": "port",
        "sample": (f"torch fp32 CPU oracle at N={n}: 1 dense layer {dense_s*1e3:.1f} ms, score {score_s*1e3:.1f} ms, "
                   f"top-k {topk_s*1e3:.2f} ms, 1 sparse layer (gather+cat+attention, k={k_sel}) {sparse_s*1e3:.2f} ms; "
                   f"median of {reps}; scaled to {nd} dense + {nf} score/top-k + {ns} sparse layers"),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--ctx", type=int, default=131072)
    ap.add_argument("--tail", type=int, default=1)
    ap.add_argument("--ratio", type=float, default=0.067)
    ap.add_argument("--selector", default="softmax_sum_last",
                    choices=["last", "softmax_before_last", "softmax_sum_last"])
    ap.add_argument("--layout", default="hf", choices=["token_major", "hf"],
                    help="hf = (1, Hkv, N, D) as the reference stores it; token_major = (1, N, Hkv, D)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16", "f32"])
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of a HIP graph replay")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--detail", action="store_true", help="print per-op timings to stderr")
    ap.add_argument("--split-rows", type=int, default=0, help="override rows per split (0 = automatic)")
    ap.add_argument("--attn-variant", type=int, default=0, help="1 = portable VALU stage 1 for every dtype")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    from omnikv_amd import ops
    from omnikv_amd._lib import check, lib

    check(lib().okv_set_option(b"split_rows", args.split_rows))
    check(lib().okv_set_option(b"attn_variant", args.attn_variant))
    device = torch.device("cuda:0")
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[args.dtype]
    esize = 4 if dtype == torch.float32 else 2
    n, tail = args.ctx, args.tail
    k_sel = int(args.ratio * n)  # the reference truncates: modeling/omnikv.py:169-171
    ks, vs, qs = build_cache(n, max(tail, 1), dtype, device, args.layout)
    step = make_step(ks, vs, qs, n, tail, k_sel, args.selector)

    stream = torch.cuda.Stream()
    graph = None
    with torch.cuda.stream(stream):
        for _ in range(max(args.warmup, 1)):
            outs, idx = step()
        stream.synchronize()
        ref_out = [o.clone() for o in outs]
        if not args.no_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                g_outs, g_idx = step()
            for _ in range(3):  # replays must reproduce the eager results
                graph.replay()
                stream.synchronize()
                for a, b in zip(g_outs, ref_out):
                    if not torch.equal(a, b):
                        raise SystemExit("graph replay differs from the eager step")
        run = graph.replay if graph is not None else step
        for _ in range(args.warmup):
            run()
        stream.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            run()
        stream.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

        # ---- spread of single steps (outside the timed region): one event pair per step
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
               for _ in range(max(args.steps, 20))]
        for e0, e1 in evs:
            e0.record(stream)
            run()
            e1.record(stream)
        stream.synchronize()
        per_step = sorted(e0.elapsed_time(e1) for e0, e1 in evs)

        def pct(p):
            return per_step[min(len(per_step) - 1, int(p * len(per_step)))]

        # ---- dominant kernel: dense split attention over N+tail rows, eager, events
        dense_layers = [l for l, kd in schedule().items() if kd[0] == "dense"]
        reps = 10

        def dense_pass():
            for l in dense_layers:
                ops.dense_attn(qs[l], ks[l][:, :, : n + tail], vs[l][:, :, : n + tail])

        dense_pass()
        dense_ms = time_events(dense_pass, reps, stream) / len(dense_layers)
        # the split pass alone (the dominant kernel), merge launch left out
        check(lib().okv_set_option(b"skip_merge", 1))
        dense_pass()
        split_ms = time_events(dense_pass, reps, stream) / len(dense_layers)
        check(lib().okv_set_option(b"skip_merge", 0))
        detail = {}
        if args.detail:
            fl = FILTER_LAYERS[0]
            sp = [l for l, kd in schedule().items() if kd[0] == "sparse"]
            _, sc = ops.dense_attn(qs[fl], ks[fl][:, :, : n + tail], vs[fl][:, :, : n + tail],
                                   selector=args.selector, score_len=n)
            ix = ops.topk(sc, k_sel)
            detail["fused_filter_ms"] = time_events(
                lambda: [ops.dense_attn(qs[l], ks[l][:, :, : n + tail], vs[l][:, :, : n + tail],
                                        selector=args.selector, score_len=n) for l in FILTER_LAYERS], reps, stream) / 3
            detail["score_only_ms"] = time_events(
                lambda: [ops.score(qs[l], ks[l][:, :, :n], selector=args.selector) for l in FILTER_LAYERS], reps, stream) / 3
            detail["score_raw_max_ms"] = time_events(
                lambda: [ops.score(qs[l], ks[l][:, :, :n], selector="last") for l in FILTER_LAYERS], reps, stream) / 3
            detail["topk_ms"] = time_events(lambda: ops.topk(sc, k_sel), 20, stream)
            detail["sparse_ms"] = time_events(
                lambda: [ops.sparse_attn(qs[l], ks[l][:, :, :n], vs[l][:, :, :n], idx=ix,
                                         tail_k=ks[l][:, :, n: n + tail], tail_v=vs[l][:, :, n: n + tail]) for l in sp],
                reps, stream) / len(sp)
            detail["dense_ms"] = dense_ms
            print(json.dumps(detail), file=sys.stderr)

    dense_bytes = 2.0 * (n + tail) * HKV * D * esize  # K and V rows once each
    achieved = dense_bytes / (split_ms * 1e-3) / 1e9
    kinds = schedule()
    step_bytes = 0.0
    for l, (kind, _) in kinds.items():
        if kind in ("dense", "filter"):
            step_bytes += dense_bytes + (4.0 * n if kind == "filter" else 0.0)
        else:
            step_bytes += 2.0 * (k_sel + tail) * HKV * D * esize + 4.0 * k_sel
    res = {
        "metric": "omnikv_decode_step_attn_us_per_layer",
        "value": wall_ms * 1e3 / LAYERS,
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {
            "workload": "ctx128k_bs1" if n == 131072 else f"ctx{n}_bs1",
            "context": n, "tail": tail, "selected": k_sel, "selector": args.selector,
            "filter_layers": list(FILTER_LAYERS), "num_wait_load_layers": WAIT, "layers": LAYERS,
            "q_heads": HQ, "kv_heads": HKV, "head_dim": D, "kv_layout": args.layout,
            "launch": "hip_graph_replay" if graph is not None else "eager",
            "kv_resident_gb": round(2 * LAYERS * (n + max(tail, 1)) * HKV * D * esize / 1e9, 2),
        },
        "decode_tokens_per_s_attention_only": 1e3 / wall_ms,
        "step_hbm_gbs": step_bytes / (wall_ms * 1e-3) / 1e9,
        "step_ms_p10_p50_p90": [round(pct(0.1), 4), round(pct(0.5), 4), round(pct(0.9), 4)],
        "roofline": {
            "kernel": "okv::attn_stage1_mfma<BF16,4,true,0,false> (dense split pass over N+tail rows of K and V)"
            if dtype != torch.float32 else "okv::attn_stage1_generic<float,4,true> (dense split pass)",
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": TRAFFIC_BYTES.get((n, tail, args.dtype)),
            "bytes_per_launch": dense_bytes, "avg_launch_us": split_ms * 1e3,
            "with_merge_launch_us": dense_ms * 1e3,
        },
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(n, k_sel, args.selector)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
