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

Other workloads (`--workload`): `ctx450k_bs1`, the same step at 450000 tokens (59 GB of K/V resident), and
`batch16_paged`, the batched serving shape: 16 requests of 8192..32768 tokens in one paged pool per layer (pages
of 16 tokens, page table shuffled from a seed), per-request k = int(0.067 N_b), the same 32-layer schedule; a
filter layer composes the selected tokens' pool slots once (PagedKV.slot_index) and the group's sparse layers read
through them.  Same JSON shape for all.

Prints ONE JSON line: metric = microseconds of attention per layer (step time /
32); `roofline` for the dominant kernel (dense split attention), its `traffic` read from the
hardware's byte counters in two short child runs of rocprofv3 after the timed region
(`--no-live-traffic` to skip them); `roofline_by_kernel`
for every kernel of the step (scoring, filter pass, sparse gather-attention, top-k, and
the load-only floor of the sparse layer), each timed live with events around a replayed
graph of that kernel alone; `variants` (the reference's `last` selector; k = round
instead of floor); `cpu_baseline` (the CPU oracle at this context on a bounded sample)
and `cpu_baseline_config0` (the CPU-runnable 4096-token configuration).
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
# HBM bytes per launch of the dense split pass from an earlier rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE run
# (profiles/dense_split_pass_pmc.txt), keyed by (context, tail, dtype): what the line carries when the live
# measurement (live_traffic) cannot run.
TRAFFIC_BYTES = {(131072, 1, "bf16"): 537.1e6 + 1.04e6, (450000, 1, "bf16"): 1843.4e6 + 2.11e6}
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


def make_step(ks, vs, qs, n, tail, k_sel, selector, overlap_select=False):
    """One decode step's attention over the 32 layers.  With overlap_select the top-k of a filter layer runs
    on a stream of its own under the wait-load layer that follows it -- only the group's sparse layers need its
    result, which is what num_wait_load_layers is for (modeling/spec_cache.py:271-281) -- and the first sparse
    layer of the group waits for it.  Measured, the replayed graph is SLOWER that way (1.197 against 1.166 ms per
    step at 128K: three forks and joins cost more than the 3 x 18 us they hide, and the top-k's workgroups slow
    the dense pass they run beside), so it is off unless asked for.  Scores and indices live in fixed buffers."""
    from omnikv_amd import ops

    kinds = schedule()
    dev = ks[0].device
    side = torch.cuda.Stream(device=dev) if overlap_select else None
    scores = {l: torch.empty((1, n), dtype=torch.float32, device=dev) for l in FILTER_LAYERS}
    idx = {l: torch.empty((1, min(k_sel, n)), dtype=torch.int32, device=dev) for l in FILTER_LAYERS}
    done = {l: torch.cuda.Event() for l in FILTER_LAYERS}

    def step():
        outs = []
        main = torch.cuda.current_stream(dev)
        waited = set()
        for l in range(LAYERS):
            kind, src = kinds[l]
            kfull, vfull = ks[l][:, :, : n + tail], vs[l][:, :, : n + tail]
            if kind == "dense":
                outs.append(ops.dense_attn(qs[l], kfull, vfull))
            elif kind == "filter":
                if side is None:  # attention, scores and selection in one call
                    o, sc, _ = ops.dense_attn(qs[l], kfull, vfull, selector=selector, score_len=n,
                                              scores_out=scores[l], select_k=k_sel, idx_out=idx[l])
                    outs.append(o)
                else:
                    o, sc = ops.dense_attn(qs[l], kfull, vfull, selector=selector, score_len=n, scores_out=scores[l])
                    outs.append(o)
                    side.wait_stream(main)
                    with torch.cuda.stream(side):
                        ops.topk(sc, k_sel, out=idx[l])
                        done[l].record(side)
            else:
                if side is not None and src not in waited:
                    main.wait_event(done[src])
                    waited.add(src)
                outs.append(ops.sparse_attn(qs[l], ks[l][:, :, :n], vs[l][:, :, :n], idx=idx[src],
                                            tail_k=ks[l][:, :, n: n + tail], tail_v=vs[l][:, :, n: n + tail]))
        return outs, idx

    return step


def traffic_from_counters(path, counter, copy_bytes, mode=0):
    """One rocprofv3 counter_collection CSV -> bytes per launch of the dense split pass: the average reading over its
    dispatches (the attention pass itself -- with V, row mode `mode` (0 contiguous, 3 paged), no logits -- not the
    scoring pass of the set-up), scaled by the reading of the run's last three dispatches of the runtime's copy kernel, which moved
    `copy_bytes` each way.  (dict, "") or (None, reason)."""
    import csv

    dense, copy = [], []  # in dispatch order
    for r in csv.DictReader(open(path)):
        if r["Counter_Name"] != counter:
            continue
        name = r["Kernel_Name"]
        if ("attn_stage1_mfma" in name and f", true, {mode}, false>" in name) or \
                ("attn_stage1_generic" in name and ", true>" in name):
            dense.append(float(r["Counter_Value"]))
        elif "copyBuffer" in name:
            copy.append(float(r["Counter_Value"]))
    copy = copy[-3:]
    if len(dense) < 4 or len(copy) < 3 or min(copy) <= 0:
        return None, f"{len(dense)} dense and {len(copy)} copy dispatches"
    raw_dense, raw_copy = sum(dense) / len(dense) * 1024.0, sum(copy) / len(copy) * 1024.0  # the counters count KiB
    return {"raw_bytes": raw_dense, "scale": copy_bytes / raw_copy, "bytes": raw_dense * copy_bytes / raw_copy,
            "dispatches": len(dense)}, ""


def live_traffic(n, tail, dtype, budget_s=150.0, paged=False):
    """HBM bytes per launch of the dense split pass by the hardware's counters, taken now: two child runs of
    `rocprofv3 --pmc` (FETCH_SIZE, then WRITE_SIZE; one counter per run) around
    `python -m omnikv_amd.microbench --op dense --then-copy 3` at this shape (`--op paged_dense` for the paged
    batch: the same requests and pool, without the decode step's own token).  Each counter is scaled by what it
    reads, in the same process, for the runtime's copy kernel moving one K tensor (a transfer of known size).
    Returns (dict | None, note): None with the reason when the profiler is absent, fails or runs out of time."""
    import shutil
    import signal
    import subprocess
    import tempfile

    exe = shutil.which("rocprofv3")
    if exe is None:
        return None, "rocprofv3 is not on PATH"
    if "rocprofiler" in os.environ.get("LD_PRELOAD", ""):
        return None, "this run is itself being profiled"
    env = dict(os.environ, TMPDIR="/tmp", PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""))
    got = {}
    with tempfile.TemporaryDirectory(dir="/tmp") as td:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            out_dir = os.path.join(td, counter)
            cmd = [exe, "--pmc", counter, "--kernel-trace", "--output-format", "csv", "-d", out_dir, "-o", "p", "--",
                   sys.executable, "-m", "omnikv_amd.microbench", "--dtype", dtype, "--layers", "2", "--reps", "4",
                   "--warmup", "1", "--then-copy", "3"]
            cmd += ["--op", "paged_dense"] if paged else ["--op", "dense", "--ctx", str(n), "--tail", str(tail)]
            with open(os.path.join(td, counter + ".log"), "w") as log:
                child = subprocess.Popen(cmd, cwd="/tmp", env=env, stdout=log, stderr=log, start_new_session=True)
                try:
                    rc = child.wait(timeout=budget_s / 2)
                except subprocess.TimeoutExpired:
                    os.killpg(child.pid, signal.SIGKILL)  # the group this call started, nothing else
                    child.wait()
                    return None, f"the {counter} run did not finish in {budget_s / 2:.0f} s"
            if rc != 0:
                return None, f"the {counter} run ended with status {rc}"
            copy_bytes = None
            for line in open(os.path.join(td, counter + ".log")):
                if line.startswith("{"):
                    copy_bytes = json.loads(line).get("copy_bytes_each_way")
            path = os.path.join(out_dir, "p_counter_collection.csv")
            if copy_bytes is None or not os.path.exists(path):
                return None, f"the {counter} run left no counters"
            got[counter], why = traffic_from_counters(path, counter, copy_bytes, 3 if paged else 0)
            if got[counter] is None:
                return None, f"the {counter} run: {why}"
    return got, "measured in this run"


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

    # beyond ~200K tokens the 4x repeated K of the whole-tensor functions is held one kv head at a time
    attend = orc.gqa_attention_by_kv_head if n > 200000 else orc.gqa_attention
    score = orc.score_tokens_by_kv_head if n > 200000 else orc.score_tokens
    t0 = time.perf_counter()
    dense_s, _ = t(lambda: attend(q, k, v), 1)
    reps = 3 if (time.perf_counter() - t0) * 8 < budget_s else 1
    dense_s, _ = t(lambda: attend(q, k, v), reps)
    score_s, sc = t(lambda: score(q, k, n, selector), reps)
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


def time_graph(fn, launches, reps, stream):
    """Microseconds per launch of fn()'s `launches` launches: captured once, replayed between two events."""
    fn()
    stream.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        fn()
    g.replay()
    stream.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        g.replay()
    e1.record(stream)
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (reps * launches)


def measure_kernels(ops, l, check, stream, ks, vs, qs, n, tail, k_sel, selector, dtype, esize, dense_layers,
                    sparse_layers, filter_layers, idx):
    """Per-kernel microseconds and fraction of the HBM roofline (algorithmic bytes / time / 8 TB/s) for the
    kernels the decode step is made of.  `..._split_pass` entries time the split pass alone (the library's
    measurement hook suppresses the merge / finishing launch), `..._op` entries the whole entry point."""
    import ctypes as C

    from omnikv_amd import _lib

    reps = 20
    kv_row = HKV * D * esize
    tname = {torch.bfloat16: "BF16", torch.float16: "F16", torch.float32: "float"}[dtype]
    mfma = dtype != torch.float32
    out = {}

    def entry(name, kernel, us, nbytes, launches_per_op=1, note=None):
        e = {"kernel": kernel, "us": us, "launches": launches_per_op}
        if nbytes:
            e.update({"bytes": nbytes, "achieved": nbytes / (us * 1e-6) / 1e9, "frac": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                      "bound": "hbm", "unit": "GB/s"})
        else:
            e.update({"bound": "latency"})
        if note:
            e["note"] = note
        out[name] = e

    def full(layer):
        return ks[layer][:, :, : n + tail], vs[layer][:, :, : n + tail]

    def split_only(fn, launches):
        check(l.okv_diag_split_pass_only(1))
        try:
            return time_graph(fn, launches, reps, stream)
        finally:
            check(l.okv_diag_split_pass_only(0))

    def dense():
        for layer in dense_layers:
            ops.dense_attn(qs[layer], *full(layer))

    dense_bytes = 2.0 * (n + tail) * kv_row
    stage1 = "okv::attn_stage1_mfma<%s,4,%%s,%%d,%%s>" % tname if mfma else "okv::attn_stage1_generic<float,4,%s> [mode %d, logits %s]"
    entry("dense_split_pass", stage1 % ("true", 0, "false") + " (dense split pass over N+tail rows of K and V)",
          split_only(dense, len(dense_layers)), dense_bytes)
    entry("dense_attention_op", "split pass + okv::attn_merge", time_graph(dense, len(dense_layers), reps, stream), dense_bytes, 2)

    def fused():
        for layer in filter_layers:
            ops.dense_attn(qs[layer], *full(layer), selector=selector, score_len=n)

    fused_bytes = dense_bytes + 4.0 * n
    entry("filter_layer_split_pass", stage1 % ("true", 0, "true") + f" (attention + {selector} logits in one pass over K)",
          split_only(fused, len(filter_layers)), fused_bytes)
    entry("filter_layer_op", "split pass + okv::merge_and_finish", time_graph(fused, len(filter_layers), reps, stream),
          fused_bytes, 2)

    score_bytes = 1.0 * n * kv_row + 4.0 * n

    def score_last():
        for layer in filter_layers:
            ops.score(qs[layer], ks[layer][:, :, :n], selector="last")

    entry("score_last_op", "okv::score_raw_mfma<%s,4,false> (raw logits, head max: one launch)" % tname if mfma
          else "split pass + finish", time_graph(score_last, len(filter_layers), reps, stream), score_bytes, 1 if mfma else 2)

    def score_soft():
        for layer in filter_layers:
            ops.score(qs[layer], ks[layer][:, :, :n], selector="softmax_sum_last")

    entry("score_softmax_split_pass", stage1 % ("false", 0, "true") + " (softmax_sum_last: logits + per-split log-sum-exp)",
          split_only(score_soft, len(filter_layers)), score_bytes)
    entry("score_softmax_op", "split pass + okv::merge_and_finish", time_graph(score_soft, len(filter_layers), reps, stream),
          score_bytes, 2)

    any_idx = next(iter(idx.values()))
    sc = ops.score(qs[filter_layers[0]], ks[filter_layers[0]][:, :, :n], selector=selector)
    entry("topk_op", "okv::topk_mb_hist + topk_mb_cand + topk_mb_write (k = %d of %d)" % (k_sel, n),
          time_graph(lambda: [ops.topk(sc, k_sel) for _ in range(4)], 4, reps, stream), None, 3)

    def fused_select():
        for layer in filter_layers:
            ops.dense_attn(qs[layer], *full(layer), selector=selector, score_len=n, select_k=k_sel)

    entry("filter_layer_with_selection",
          "split pass + okv::merge_and_finish + topk_mb_hist + topk_mb_cand + topk_mb_write: "
          "attention, scores and the k = %d selection of a filter layer in one call" % k_sel,
          time_graph(fused_select, len(filter_layers), reps, stream), fused_bytes, 5)

    def sparse():
        for layer in sparse_layers:
            ops.sparse_attn(qs[layer], ks[layer][:, :, :n], vs[layer][:, :, :n], idx=any_idx,
                            tail_k=ks[layer][:, :, n: n + tail], tail_v=vs[layer][:, :, n: n + tail])

    sparse_bytes = 2.0 * (k_sel + tail) * kv_row + 4.0 * k_sel
    entry("sparse_split_pass", stage1 % ("true", 1, "false") + " (fused gather + attention over the selected rows + tail)",
          split_only(sparse, len(sparse_layers)), sparse_bytes)
    entry("sparse_attention_op", "split pass + okv::attn_merge", time_graph(sparse, len(sparse_layers), reps, stream),
          sparse_bytes, 2)
    if mfma:
        # the attainable bound on this device: a kernel with the same grid, index lookups, load shapes and
        # bytes that does nothing with what it loads
        shape = _lib.Shape(1, HQ, HKV, D, k_sel, tail, 0)
        rows_, splits_ = C.c_int32(0), C.c_int32(0)
        check(l.okv_diag_split_geometry(_lib.OKV_OP_SPARSE_ATTN, C.byref(shape), C.byref(rows_), C.byref(splits_)))
        sink = torch.zeros(4, dtype=torch.int32, device=any_idx.device)
        k0 = ks[sparse_layers[0]]
        lay = _lib.KVLayout(_lib.OKV_BF16 if dtype == torch.bfloat16 else _lib.OKV_F16, HQ, HKV, D, k0.stride(2),
                            k0.stride(1), k0.stride(0), None, 0, 0, 0)

        def floor():
            for layer in sparse_layers:
                check(l.okv_diag_gather_floor(ks[layer].data_ptr(), vs[layer].data_ptr(), C.byref(lay), any_idx.data_ptr(),
                                              any_idx.stride(0), None, k_sel, 1, rows_.value, 4, sink.data_ptr(),
                                              stream.cuda_stream))

        entry("sparse_load_only_floor", "okv::gather_floor_kernel (same grid, index lookups and loads; no arithmetic, no output)",
              time_graph(floor, len(sparse_layers), reps, stream), 2.0 * k_sel * kv_row + 4.0 * k_sel,
              note="split_rows %d, %d splits x %d kv heads" % (rows_.value, (k_sel + rows_.value - 1) // rows_.value, HKV))

        def empty():
            for _ in range(24):
                check(l.okv_diag_empty_launch(sink.data_ptr(), stream.cuda_stream))

        entry("empty_launch", "okv::empty_kernel (one wave, no work): the cost of a launch inside a replayed graph",
              time_graph(empty, 24, reps, stream), None)
    return out


def cpu_baseline_config0(n=4096, ratio=0.067):
    """The CPU-runnable configuration itself (batch 1, fp32, 4096 tokens): the oracle's whole filter-layer op
    -- score, top-k, gather, one downstream layer's attention over the selected rows -- for both selectors."""
    from omnikv_amd import synth
    from oracle import okv_oracle as orc

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    q, k, v = synth.filter_layer_inputs(n, HQ, HKV, D)
    _, k2, v2 = synth.filter_layer_inputs(n, HQ, HKV, D, seed=synth.SEED_DATA + 100)
    qn = synth.fresh_q()
    res = {"context": n, "dtype": "f32", "cores": cores, "kind": "port", "unit": "us per filter-layer op",
           "sample": "median of 20 runs after 3 warm-ups of okv_oracle.filter_layer_op (score + top-k + gather + sparse attention)"}
    for sel in ("last", "softmax_sum_last"):
        for kk in sorted({int(ratio * n), int(round(ratio * n))}):
            ts = []
            for i in range(23):
                t0 = time.perf_counter()
                orc.filter_layer_op(q, k, v2, k2, qn, kk, sel)
                ts.append(time.perf_counter() - t0)
            ts = sorted(ts[3:])
            res[f"{sel}_k{kk}"] = ts[len(ts) // 2] * 1e6
    return res


# --------------------------------------------------------------------------------------------------
# batch16_paged: the batched serving shape
# --------------------------------------------------------------------------------------------------
def main_batch16_paged(args):
    """16 requests of 8192..32768 prompt tokens (seeded) + the decode step's own token each, one paged pool per
    layer (16-token pages, one page table shuffled from a seed), per-request k = int(ratio * N_b).  Layer
    schedule as in the default workload.  A filter layer is one okv_dense_attn_select call (attention over
    N_b + 1 rows, scores of the N_b prompt rows, ragged top-k) followed by PagedKV.slot_index, which composes
    index and page table once per selection; the group's sparse layers read the pool through those slots
    (the table the reference's serving stack keeps per request, common/req_manager.py:12-17) and a tail buffer."""
    from omnikv_amd import _lib as okv_lib
    okv_lib.use_diag_build()
    import ctypes as C

    from omnikv_amd import ops, synth
    from omnikv_amd._lib import check, lib

    check(lib().okv_set_option(b"split_rows", args.split_rows))
    check(lib().okv_set_option(b"attn_variant", args.attn_variant))
    dev = torch.device("cuda:0")
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16}[args.dtype]
    esize, batch, page, tail = 2, 16, 16, 1
    selector = args.selector
    lens = synth.ragged_lengths(batch)
    lens1 = lens + 1
    table, total = synth.shuffled_page_table(lens1, page)
    table_d, lens_d, lens1_d = table.to(dev), lens.to(dev), lens1.to(dev)
    nmax, nmax1 = int(lens.max()), int(lens1.max())
    k_per = torch.tensor([max(1, int(args.ratio * int(x))) for x in lens], dtype=torch.int32)
    kmax, k_per_d = int(k_per.max()), k_per.to(dev)
    gen = torch.Generator(device=dev).manual_seed(4321)
    pools, qs, tails = [], [], []
    t_idx = [torch.arange(int(x)) for x in lens]
    for l in range(LAYERS):
        pk = torch.empty((total, page, HKV, D), dtype=dtype, device=dev).normal_(generator=gen)
        pv = torch.empty((total, page, HKV, D), dtype=dtype, device=dev).normal_(generator=gen)
        q = torch.randn((batch, HQ, 1, D), generator=gen, device=dev, dtype=torch.float32).to(dtype)
        if l in FILTER_LAYERS:  # the benchmark's key distribution (sink + heavy hitters) for every request
            for b in range(batch):
                qb, kb, _ = synth.filter_layer_inputs(int(lens[b]), HQ, HKV, D, seed=synth.SEED_DATA + 100 * l + b)
                pages = table[b, t_idx[b] // page].long().to(dev)
                pk[pages, (t_idx[b] % page).to(dev)] = kb[0].permute(1, 0, 2).to(dtype).to(dev)
                q[b] = qb[0].to(dtype).to(dev)
        pools.append(ops.PagedKV(pk, pv, table_d, page))
        qs.append(q)
        tails.append((torch.empty((batch, HKV, tail, D), dtype=dtype, device=dev).normal_(generator=gen),
                      torch.empty((batch, HKV, tail, D), dtype=dtype, device=dev).normal_(generator=gen)))
    kinds = schedule()
    scores = {l: torch.empty((batch, nmax), dtype=torch.float32, device=dev) for l in FILTER_LAYERS}
    idx = {l: torch.full((batch, kmax), -1, dtype=torch.int32, device=dev) for l in FILTER_LAYERS}

    def step():
        outs, slots = [], {}
        for l in range(LAYERS):
            kind, src = kinds[l]
            if kind == "dense":
                outs.append(ops.dense_attn(qs[l], pools[l], seq_len=nmax1, seq_lens=lens1_d))
            elif kind == "filter":
                o, _, _ = ops.dense_attn(qs[l], pools[l], seq_len=nmax1, seq_lens=lens1_d, selector=selector, score_len=nmax,
                                         score_lens=lens_d, scores_out=scores[l], select_k=kmax, k_per_seg=k_per_d,
                                         idx_out=idx[l])
                slots[l] = pools[l].slot_index(idx[l])
                outs.append(o)
            else:
                outs.append(ops.sparse_attn(qs[l], pools[l], slots=slots[src], sel_len=kmax, sel_lens=k_per_d,
                                            tail_k=tails[l][0], tail_v=tails[l][1]))
        return outs, slots

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(max(args.warmup, 1)):
            outs, slots = step()
        stream.synchronize()
        ref_out = [o.clone() for o in outs]
        graph = None
        if not args.no_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                g_outs, _ = step()
            for _ in range(3):
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
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(max(args.steps, 20))]
        for e0, e1 in evs:
            e0.record(stream)
            run()
            e1.record(stream)
        stream.synchronize()
        per_step = sorted(e0.elapsed_time(e1) for e0, e1 in evs)

        # ---- single kernels, each over rotating layers in a replayed graph of its own
        l_ = lib()
        reps = 20
        tokens, tokens1, sel_total = int(lens.sum()), int(lens1.sum()), int(k_per.sum())
        kv_row = HKV * D * esize
        dense_layers = [l for l, kd in kinds.items() if kd[0] == "dense"]
        sparse_layers = [l for l, kd in kinds.items() if kd[0] == "sparse"]
        fl = list(FILTER_LAYERS)
        tname = "BF16" if dtype == torch.bfloat16 else "F16"
        by = {}

        def entry(name, kernel, us, nbytes, launches=1, note=None):
            e = {"kernel": kernel, "us": us, "launches": launches}
            if nbytes:
                e.update({"bytes": nbytes, "achieved": nbytes / (us * 1e-6) / 1e9, "frac": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                          "bound": "hbm", "unit": "GB/s"})
            else:
                e.update({"bound": "latency"})
            if note:
                e["note"] = note
            by[name] = e

        def split_only(fn, launches):
            check(l_.okv_diag_split_pass_only(1))
            try:
                return time_graph(fn, launches, reps, stream)
            finally:
                check(l_.okv_diag_split_pass_only(0))

        def dense():
            for l in dense_layers:
                ops.dense_attn(qs[l], pools[l], seq_len=nmax1, seq_lens=lens1_d)

        def fused():
            for l in fl:
                ops.dense_attn(qs[l], pools[l], seq_len=nmax1, seq_lens=lens1_d, selector=selector, score_len=nmax, score_lens=lens_d)

        def fused_select():
            for l in fl:
                ops.dense_attn(qs[l], pools[l], seq_len=nmax1, seq_lens=lens1_d, selector=selector, score_len=nmax,
                               score_lens=lens_d, select_k=kmax, k_per_seg=k_per_d)

        def score_of(sel):
            def f():
                for l in fl:
                    ops.score(qs[l], pools[l], score_len=nmax, selector=sel, score_lens=lens_d)
            return f

        any_slots = next(iter(slots.values()))
        any_idx = idx[fl[0]]

        def sparse_slots():
            for l in sparse_layers:
                ops.sparse_attn(qs[l], pools[l], slots=any_slots, sel_len=kmax, sel_lens=k_per_d, tail_k=tails[l][0], tail_v=tails[l][1])

        def sparse_two_lookups():
            for l in sparse_layers[:8]:
                ops.sparse_attn(qs[l], pools[l], idx=any_idx, sel_len=kmax, sel_lens=k_per_d, tail_k=tails[l][0], tail_v=tails[l][1])

        stage1 = "okv::attn_stage1_mfma<%s,4,%%s,%%d,%%s>" % tname
        dense_bytes = 2.0 * tokens1 * kv_row
        fused_bytes = dense_bytes + 4.0 * tokens
        score_bytes = 1.0 * tokens * kv_row + 4.0 * tokens
        sparse_bytes = 2.0 * (sel_total + batch * tail) * kv_row + 4.0 * sel_total
        entry("dense_split_pass", stage1 % ("true", 3, "false") + " (paged dense split pass, one page lookup per 16-row tile)",
              split_only(dense, len(dense_layers)), dense_bytes)
        entry("dense_attention_op", "split pass + okv::attn_merge", time_graph(dense, len(dense_layers), reps, stream), dense_bytes, 2)
        entry("filter_layer_split_pass", stage1 % ("true", 3, "true") + f" (attention + {selector} logits in one pass over K)",
              split_only(fused, len(fl)), fused_bytes)
        entry("filter_layer_op", "split pass + okv::merge_and_finish", time_graph(fused, len(fl), reps, stream), fused_bytes, 2)
        entry("score_last_op", "okv::score_raw_mfma<%s,4,true> (raw logits, head max: one launch)" % tname,
              time_graph(score_of("last"), len(fl), reps, stream), score_bytes, 1)
        entry("score_softmax_split_pass", stage1 % ("false", 3, "true"), split_only(score_of("softmax_sum_last"), len(fl)), score_bytes)
        entry("score_softmax_op", "split pass + okv::merge_and_finish", time_graph(score_of("softmax_sum_last"), len(fl), reps, stream),
              score_bytes, 2)
        sc0 = scores[fl[0]]
        entry("topk_op", "ragged top-k: okv::topk_mb_hist + topk_mb_cand + topk_mb_write (k_b = int(%.3f N_b))" % args.ratio,
              time_graph(lambda: [ops.topk(sc0, kmax, seq_lens=lens_d, k_per_seg=k_per_d) for _ in range(4)], 4, reps, stream), None, 3)
        entry("filter_layer_with_selection", "split pass + okv::merge_and_finish + the three top-k launches, one call",
              time_graph(fused_select, len(fl), reps, stream), fused_bytes, 5)
        entry("slot_index", "PagedKV.slot_index: index and page table composed once per selection (torch ops)",
              time_graph(lambda: [pools[l].slot_index(idx[l]) for l in fl], len(fl), reps, stream), None)
        entry("sparse_split_pass", stage1 % ("true", 1, "false") + " (selected rows of the pool through composed token slots + tail)",
              split_only(sparse_slots, len(sparse_layers)), sparse_bytes)
        entry("sparse_attention_op", "split pass + okv::attn_merge", time_graph(sparse_slots, len(sparse_layers), reps, stream),
              sparse_bytes, 2)
        entry("sparse_attention_two_lookups_op", stage1 % ("true", 2, "false") + " + okv::attn_merge (index, then page table, per row)",
              time_graph(sparse_two_lookups, 8, reps, stream), sparse_bytes, 2)
        shape = okv_lib.Shape(batch, HQ, HKV, D, kmax, tail, 0)
        rows_, splits_ = C.c_int32(0), C.c_int32(0)
        check(l_.okv_diag_split_geometry(okv_lib.OKV_OP_SPARSE_ATTN, C.byref(shape), C.byref(rows_), C.byref(splits_)))
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        pk0 = pools[0].pool_k
        lay = okv_lib.KVLayout(okv_lib.OKV_BF16 if dtype == torch.bfloat16 else okv_lib.OKV_F16, HQ, HKV, D, pk0.stride(1),
                               pk0.stride(2), 0, None, 0, 0, 0)

        def floor():
            for l in sparse_layers:
                check(l_.okv_diag_gather_floor(pools[l].pool_k.data_ptr(), pools[l].pool_v.data_ptr(), C.byref(lay),
                                               any_slots.data_ptr(), any_slots.stride(0), k_per_d.data_ptr(), kmax, batch,
                                               rows_.value, 4, sink.data_ptr(), stream.cuda_stream))

        entry("sparse_load_only_floor", "okv::gather_floor_kernel (same grid, slot lookups and loads; no arithmetic, no output)",
              time_graph(floor, len(sparse_layers), reps, stream), 2.0 * sel_total * kv_row + 4.0 * sel_total,
              note="split_rows %d, %d splits x %d kv heads x %d requests" % (rows_.value, (kmax + rows_.value - 1) // rows_.value, HKV, batch))

        def empty():
            for _ in range(24):
                check(l_.okv_diag_empty_launch(sink.data_ptr(), stream.cuda_stream))

        entry("empty_launch", "okv::empty_kernel", time_graph(empty, 24, reps, stream), None)

    step_bytes = 0.0
    for l, (kind, _) in kinds.items():
        step_bytes += (dense_bytes + (4.0 * tokens if kind == "filter" else 0.0)) if kind != "sparse" else sparse_bytes
    dom = by["dense_split_pass"]

    def pct(p):
        return per_step[min(len(per_step) - 1, int(p * len(per_step)))]

    traffic, traffic_source, traffic_detail = None, None, None
    if not args.no_live_traffic and args.dtype != "f32":
        live, note = live_traffic(0, 0, args.dtype, paged=True)
        if live is not None:
            traffic = live["FETCH_SIZE"]["bytes"] + live["WRITE_SIZE"]["bytes"]
            traffic_source = ("live: rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, in two child processes of this run around "
                              "`python -m omnikv_amd.microbench --op paged_dense --then-copy 3` (the same requests, pages "
                              "and page table, without the decode step's own token: 16 rows fewer); each counter scaled by "
                              "its reading for the runtime's copy kernel moving one layer's K pool in the same process")
            traffic_detail = {"fetched_bytes": live["FETCH_SIZE"]["bytes"], "written_bytes": live["WRITE_SIZE"]["bytes"],
                              "fetch_scale": live["FETCH_SIZE"]["scale"], "write_scale": live["WRITE_SIZE"]["scale"],
                              "dispatches": live["FETCH_SIZE"]["dispatches"]}
        else:
            traffic_source = f"not measured: {note}"
    res = {
        "metric": "omnikv_decode_step_attn_us_per_layer", "value": wall_ms * 1e3 / LAYERS, "unit": "us/layer", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall_ms, "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {
            "workload": "batch16_paged", "batch": batch, "prompt_tokens": [int(x) for x in lens], "tokens_total": tokens,
            "page_size": page, "page_table": "shuffled (seeded)", "tail": tail, "selected_total": sel_total,
            "selected_per_request": "int(%.3f * N_b)" % args.ratio, "selector": selector, "filter_layers": list(FILTER_LAYERS),
            "num_wait_load_layers": WAIT, "layers": LAYERS, "q_heads": HQ, "kv_heads": HKV, "head_dim": D,
            "launch": "hip_graph_replay" if graph is not None else "eager",
            "kv_resident_gb": round(2 * LAYERS * total * page * HKV * D * esize / 1e9, 2),
        },
        "decode_tokens_per_s_attention_only": batch * 1e3 / wall_ms,
        "step_hbm_gbs": step_bytes / (wall_ms * 1e-3) / 1e9,
        "step_ms_p10_p50_p90": [round(pct(0.1), 4), round(pct(0.5), 4), round(pct(0.9), 4)],
        "roofline": {"kernel": dom["kernel"], "bound": "hbm", "achieved": dom["achieved"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": dom["frac"], "traffic": traffic, "traffic_source": traffic_source,
                     "traffic_detail": traffic_detail, "bytes_per_launch": dense_bytes,
                     "avg_launch_us": dom["us"], "with_merge_launch_us": by["dense_attention_op"]["us"]},
        "roofline_by_kernel": by,
        "variants": {},
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_batch(lens, args.ratio, selector, tokens)
    print(json.dumps(res))


def cpu_baseline_batch(lens, ratio, selector, tokens_total, sample=3):
    """The CPU oracle on the first `sample` requests of the batch (dense attention, scoring + top-k, one sparse
    layer each, fp32), scaled to all 16 by token count and to the 32-layer schedule."""
    from omnikv_amd import synth
    from oracle import okv_oracle as orc

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    dense_s = score_s = sparse_s = 0.0
    toks = 0
    for b in range(sample):
        n = int(lens[b])
        q, k, v = synth.filter_layer_inputs(n, HQ, HKV, D, seed=synth.SEED_DATA + b)
        qn = synth.fresh_q()
        kk = max(1, int(ratio * n))
        t0 = time.perf_counter()
        orc.gqa_attention(q, k, v)
        t1 = time.perf_counter()
        idx = orc.select_topk(orc.score_tokens(q, k, n, selector), kk)
        t2 = time.perf_counter()
        orc.gqa_attention(qn, orc.gather_rows(k, idx[0]), orc.gather_rows(v, idx[0]))
        t3 = time.perf_counter()
        dense_s, score_s, sparse_s, toks = dense_s + t1 - t0, score_s + t2 - t1, sparse_s + t3 - t2, toks + n
    scale = tokens_total / toks
    kinds = schedule()
    nd = sum(1 for x in kinds.values() if x[0] in ("dense", "filter"))
    nf = sum(1 for x in kinds.values() if x[0] == "filter")
    ns = sum(1 for x in kinds.values() if x[0] == "sparse")
    step_s = scale * (nd * dense_s + nf * score_s + ns * sparse_s)
    return {"value": step_s * 1e6 / LAYERS, "unit": "us/layer", "cores": cores, "kind": "port",
            "sample": f"torch fp32 CPU oracle on requests 0..{sample - 1} of the batch ({toks} of {tokens_total} tokens), one pass "
                      f"each: dense {dense_s*1e3:.1f} ms, score + top-k {score_s*1e3:.1f} ms, sparse {sparse_s*1e3:.2f} ms; scaled by "
                      f"token count to 16 requests and to {nd} dense + {nf} score/top-k + {ns} sparse layers"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=None, choices=["ctx128k_bs1", "ctx450k_bs1", "batch16_paged"],
                    help="ctx128k_bs1 (default): the configuration the metric is quoted on; ctx450k_bs1: the same step "
                         "at 450000 tokens; batch16_paged: 16 ragged requests on a paged pool")
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
    ap.add_argument("--overlap-select", action="store_true",
                    help="run each filter layer's top-k on a stream of its own under the wait-load layer (measured slower)")
    ap.add_argument("--no-variants", action="store_true", help="skip the extra steps (selector last, k = round(ratio N))")
    ap.add_argument("--no-live-traffic", action="store_true",
                    help="do not re-measure roofline.traffic with rocprofv3 --pmc in child processes (two short runs)")
    ap.add_argument("--split-rows", type=int, default=0, help="override rows per split (0 = automatic)")
    ap.add_argument("--attn-variant", type=int, default=0, help="1 = portable VALU stage 1 for every dtype")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    if args.workload == "ctx450k_bs1":
        args.ctx = 450000
    elif args.workload == "ctx128k_bs1":
        args.ctx = 131072
    elif args.workload == "batch16_paged":
        return main_batch16_paged(args)

    from omnikv_amd import _lib as okv_lib
    okv_lib.use_diag_build()  # the product's kernels + the measurement hooks (split pass alone, load-only floor)
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
    step = make_step(ks, vs, qs, n, tail, k_sel, args.selector, args.overlap_select)

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

        # ---- single kernels, timed live: each measurement captures one pass over its layers in a HIP
        # graph (so short kernels are not paced by the host's launch rate) and replays it between two
        # events on this stream; the layers rotate, so no launch finds its rows in cache
        kinds = schedule()
        dense_layers = [l for l, kd in kinds.items() if kd[0] == "dense"]
        sparse_layers = [l for l, kd in kinds.items() if kd[0] == "sparse"]
        fl = list(FILTER_LAYERS)
        by_kernel = measure_kernels(ops, lib(), check, stream, ks, vs, qs, n, tail, k_sel, args.selector, dtype, esize,
                                    dense_layers, sparse_layers, fl, idx)
        dom = by_kernel["dense_split_pass"]
        split_us, dense_us = dom["us"], by_kernel["dense_attention_op"]["us"]

        # ---- the same step with the reference's own selector and with BASELINE's k = round(0.067 N)
        variants = {}
        if not args.no_variants:
            for name, sel_v, k_v in (("selector_last", "last", k_sel), ("selected_%d" % round(args.ratio * n), args.selector,
                                                                         int(round(args.ratio * n)))):
                step_v = make_step(ks, vs, qs, n, tail, k_v, sel_v, args.overlap_select)
                step_v()
                stream.synchronize()
                gv = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gv, stream=stream):
                    step_v()
                gv.replay()
                stream.synchronize()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    gv.replay()
                stream.synchronize()
                ms = (time.perf_counter() - t0) * 1e3 / args.steps
                variants[name] = {"selector": sel_v, "selected": k_v, "ms_per_step": ms, "us_per_layer": ms * 1e3 / LAYERS}

    dense_bytes = 2.0 * (n + tail) * HKV * D * esize  # K and V rows once each
    step_bytes = 0.0
    for l, (kind, _) in kinds.items():
        if kind in ("dense", "filter"):
            step_bytes += dense_bytes + (4.0 * n if kind == "filter" else 0.0)
        else:
            step_bytes += 2.0 * (k_sel + tail) * HKV * D * esize + 4.0 * k_sel
    traffic = TRAFFIC_BYTES.get((n, tail, args.dtype))
    traffic_source = ("profiles/dense_split_pass_pmc.txt (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE of an earlier run of this "
                      "kernel at this shape; not measured in this run)") if traffic else None
    traffic_detail = None
    if not args.no_live_traffic and args.layout == "hf":
        live, note = live_traffic(n, tail, args.dtype)
        if live is not None:
            traffic = live["FETCH_SIZE"]["bytes"] + live["WRITE_SIZE"]["bytes"]
            traffic_source = ("live: rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, in two child processes of this run around "
                              "`python -m omnikv_amd.microbench --op dense --then-copy 3` at this shape; each counter scaled by "
                              "its reading for the runtime's copy kernel moving one K tensor in the same process")
            traffic_detail = {"fetched_bytes": live["FETCH_SIZE"]["bytes"], "written_bytes": live["WRITE_SIZE"]["bytes"],
                              "fetch_scale": live["FETCH_SIZE"]["scale"], "write_scale": live["WRITE_SIZE"]["scale"],
                              "dispatches": live["FETCH_SIZE"]["dispatches"]}
        elif traffic_source:
            traffic_source += f"; the live measurement was skipped: {note}"
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
            "workload": {131072: "ctx128k_bs1", 450000: "ctx450k_bs1"}.get(n, f"ctx{n}_bs1"),
            "context": n, "tail": tail, "selected": k_sel, "selector": args.selector,
            "filter_layers": list(FILTER_LAYERS), "num_wait_load_layers": WAIT, "layers": LAYERS,
            "q_heads": HQ, "kv_heads": HKV, "head_dim": D, "kv_layout": args.layout,
            "launch": "hip_graph_replay" if graph is not None else "eager",
            "topk_stream": "own stream, under the wait-load layer" if args.overlap_select else "main",
            "kv_resident_gb": round(2 * LAYERS * (n + max(tail, 1)) * HKV * D * esize / 1e9, 2),
        },
        "decode_tokens_per_s_attention_only": 1e3 / wall_ms,
        "step_hbm_gbs": step_bytes / (wall_ms * 1e-3) / 1e9,
        "step_ms_p10_p50_p90": [round(pct(0.1), 4), round(pct(0.5), 4), round(pct(0.9), 4)],
        "roofline": {
            "kernel": dom["kernel"],
            "bound": "hbm", "achieved": dom["achieved"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": dom["frac"], "traffic": traffic, "traffic_source": traffic_source, "traffic_detail": traffic_detail,
            "bytes_per_launch": dense_bytes, "avg_launch_us": split_us,
            "with_merge_launch_us": dense_us,
        },
        "roofline_by_kernel": by_kernel,
        "variants": variants,
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(n, k_sel, args.selector)
        res["cpu_baseline_config0"] = cpu_baseline_config0()
    print(json.dumps(res))


if __name__ == "__main__":
    main()
