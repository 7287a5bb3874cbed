"""Single-op timing of the HIP kernels at benchmark shapes, for profiling.

    python -m omnikv_amd.microbench --op sparse --ctx 131072 --reps 50

Runs `--op` back to back over `--layers` rotating K/V buffers (so no launch reads
what the previous one left in cache), times the whole run with events on the
launch stream and prints one JSON line with the average microseconds per call and
the algorithmic GB/s.  Meant to sit behind `rocprofv3 --kernel-trace --stats` or
`--pmc`: every kernel of the run belongs to the one op.
"""
from __future__ import annotations

import argparse
import json

import torch

from . import ops, synth
from ._lib import check, lib

HQ, HKV, D = 32, 8, 128


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--op", required=True,
                    choices=["dense", "fused", "fused_select", "fused_then_topk", "score", "topk", "sparse", "sparse_packed", "sparse_floor", "sparse_timeline",
                             "empty", "gather", "copy",
                             "offload_memcpy", "offload_zero_copy", "offload_incremental", "h2d", "window", "window_loop", "window_fused", "window_then_dense",
                             "paged_dense", "paged_fused", "paged_fused_select", "paged_score", "paged_topk", "paged_sparse", "paged_sparse_slots",
                             "paged_sparse_floor"])
    ap.add_argument("--batch", type=int, default=16, help="requests of the paged_* ops (ragged lengths 8192..32768)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--pages-in-order", action="store_true", help="paged_* ops: identity page table instead of shuffled")
    ap.add_argument("--contiguous", action="store_true",
                    help="paged_* ops: the same ragged batch in (bsz, Hkv, Nmax, D) tensors, no page table")
    ap.add_argument("--window", type=int, default=16, help="query positions of the window selectors")
    ap.add_argument("--cpu-threads", type=int, default=8, help="packing threads of the offload tier")
    ap.add_argument("--tiles-in-flight", type=int, default=4, choices=[1, 2, 4],
                    help="sparse_floor: tiles whose loads a wave keeps outstanding")
    ap.add_argument("--overlap", type=float, default=0.9,
                    help="offload_incremental: share of a selection's tokens that the previous selection already held")
    ap.add_argument("--ctx", type=int, default=131072)
    ap.add_argument("--ratio", type=float, default=0.067)
    ap.add_argument("--tail", type=int, default=1)
    ap.add_argument("--layers", type=int, default=6)
    ap.add_argument("--reps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--selector", default="softmax_sum_last")
    ap.add_argument("--layout", default="hf", choices=["token_major", "hf", "interleaved"],
                    help="hf = (1, Hkv, N, D) as the reference stores it; token_major = (1, N, Hkv, D); "
                         "interleaved = (1, Hkv, N, 2, D), K and V rows of a token side by side (times like hf)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16", "f32"])
    ap.add_argument("--split-rows", type=int, default=0)
    ap.add_argument("--attn-variant", type=int, default=0)
    ap.add_argument("--then-copy", type=int, default=0,
                    help="after the op, copy one K tensor this many times with the runtime's copy kernel: a transfer of "
                         "known size in the same process, against which hardware byte counters are scaled")
    args = ap.parse_args()

    from . import _lib as okv_lib
    okv_lib.use_diag_build(stamps=args.op == "sparse_timeline")  # the product's kernels + the measurement hooks
    check(lib().okv_set_option(b"split_rows", args.split_rows))
    check(lib().okv_set_option(b"attn_variant", args.attn_variant))
    dev = torch.device("cuda:0")
    if args.op.startswith("paged_"):
        return paged(args, dev)
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[args.dtype]
    es = 4 if dtype == torch.float32 else 2
    n, tail, nl = args.ctx, args.tail, args.layers
    k_sel = int(args.ratio * n)
    gen = torch.Generator(device=dev).manual_seed(7)
    ks, vs, qs = [], [], []
    for _ in range(nl):
        if args.layout == "interleaved":  # (1, Hkv, N, 2, D): a token's K and V rows of a head side by side
            kvb = torch.empty((1, HKV, n + tail, 2, D), dtype=dtype, device=dev).normal_(generator=gen)
            kb, vb = kvb[:, :, :, 0], kvb[:, :, :, 1]
        else:
            shape = (1, n + tail, HKV, D) if args.layout == "token_major" else (1, HKV, n + tail, D)
            kb = torch.empty(shape, dtype=dtype, device=dev).normal_(generator=gen)
            vb = torch.empty(shape, dtype=dtype, device=dev).normal_(generator=gen)
        if args.layout == "token_major":
            kb, vb = kb.permute(0, 2, 1, 3), vb.permute(0, 2, 1, 3)
        ks.append(kb)
        vs.append(vb)
        qs.append(torch.randn((1, HQ, 1, D), generator=gen, device=dev).to(dtype))
    # scores with the benchmark's distribution, and their selection
    q0, k0, _ = synth.filter_layer_inputs(n, HQ, HKV, D)
    ks[0][:, :, :n].copy_(k0.to(dtype))
    qs[0] = q0.to(dtype).to(dev)
    del k0
    scores = ops.score(qs[0], ks[0][:, :, :n], selector=args.selector)
    idx = ops.topk(scores, k_sel)
    packed = [(ops.gather_rows(ks[l][:, :, :n], idx), ops.gather_rows(vs[l][:, :, :n], idx)) for l in range(nl)] \
        if args.op == "sparse_packed" else None
    dst = torch.empty_like(ks[0]) if args.op == "copy" else None
    qw = [torch.randn((1, HQ, args.window, D), generator=gen, device=dev).to(dtype) for _ in range(nl)] \
        if args.op.startswith("window") else None
    off = None
    if args.op.startswith("offload") or args.op == "h2d":
        # one offloaded layer group: `nl` layers whose prompt K/V live in pinned host memory
        from .cache import OmniKVMultiStageCache
        off = OmniKVMultiStageCache([0, nl + 2], nl + 2, num_wait_load_layers=1, real_offload=True,
                                    offload_mode={"offload_zero_copy": "zero_copy", "offload_incremental": "incremental"}.get(
                                        args.op, "memcpy"),
                                    cpu_num_threads=args.cpu_threads)
        for l in range(nl + 2):
            off.append(ks[l % nl][:, :, :n], vs[l % nl][:, :, :n], l)
        torch.cuda.synchronize()
        off.stage = "decoding"
        if args.op == "h2d":
            hsrc = torch.empty(k_sel * 2 * HKV * D * es, dtype=torch.uint8).pin_memory()
            hdst = torch.empty(k_sel * 2 * HKV * D * es, dtype=torch.uint8, device=dev)
        if args.op == "offload_incremental":
            # a chain of selections, each keeping `overlap` of the previous one's tokens (seeded, on the device)
            gsel = torch.Generator(device=dev).manual_seed(5)
            keep_n = int(round(args.overlap * k_sel))
            sels = [idx]
            for _ in range(args.warmup + args.reps + 1):
                prev = sels[-1][0].long()
                held = torch.zeros(n, dtype=torch.bool, device=dev)
                held[prev] = True
                keep = prev[torch.randperm(k_sel, generator=gsel, device=dev)[:keep_n]]
                rest = torch.nonzero(~held)[:, 0]
                fresh = rest[torch.randperm(rest.numel(), generator=gsel, device=dev)[: k_sel - keep_n]]
                sels.append(torch.cat([keep, fresh]).sort().values.to(torch.int32)[None].contiguous())
            off.set_idx_on_gpu(sels[0], 0)  # the first selection fetches everything; not timed
            torch.cuda.synchronize()

    floor = None
    if args.op in ("sparse_floor", "empty"):
        # measurement kernels of the library: a load-only pass with the sparse layer's grid, index lookups,
        # load shapes and bytes (what merely fetching the rows costs here), and an empty launch
        import ctypes as C

        from . import _lib
        shape = _lib.Shape(1, HQ, HKV, D, k_sel, tail, 0)
        rows_, splits_ = C.c_int32(0), C.c_int32(0)
        check(lib().okv_diag_split_geometry(_lib.OKV_OP_SPARSE_ATTN, C.byref(shape), C.byref(rows_), C.byref(splits_)))
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        lay = _lib.KVLayout(ops._DTYPES[dtype], HQ, HKV, D, ks[0].stride(2), ks[0].stride(1), ks[0].stride(0), None, 0, 0, 0)
        floor = (rows_.value, sink, lay, C)

    def call(i):
        l = i % nl
        if args.op == "sparse_floor":
            rows, sink, lay, C = floor
            return check(lib().okv_diag_gather_floor(ks[l].data_ptr(), vs[l].data_ptr(), C.byref(lay), idx.data_ptr(),
                                                     idx.stride(0), None, k_sel, 1, rows, args.tiles_in_flight,
                                                     sink.data_ptr(), torch.cuda.current_stream().cuda_stream))
        if args.op == "empty":
            return check(lib().okv_diag_empty_launch(floor[1].data_ptr(), torch.cuda.current_stream().cuda_stream))
        if args.op == "dense":
            return ops.dense_attn(qs[l], ks[l], vs[l])
        if args.op == "fused":
            return ops.dense_attn(qs[l], ks[l], vs[l], selector=args.selector, score_len=n)
        if args.op == "fused_select":  # the filter layer in one call
            return ops.dense_attn(qs[l], ks[l], vs[l], selector=args.selector, score_len=n, select_k=k_sel)
        if args.op == "fused_then_topk":  # the same as two calls
            return ops.topk(ops.dense_attn(qs[l], ks[l], vs[l], selector=args.selector, score_len=n)[1], k_sel)
        if args.op == "score":
            return ops.score(qs[l], ks[l][:, :, :n], selector=args.selector)
        if args.op == "topk":
            return ops.topk(scores, k_sel)
        if args.op == "window":
            return ops.score_window(qw[l], ks[l][:, :, :n], selector="uniform")
        if args.op == "window_fused":  # a window-selector filter layer in two passes over K
            return ops.dense_attn_window(qs[l], qw[l], ks[l], vs[l], selector="uniform", score_len=n)
        if args.op == "window_then_dense":  # the same as two calls: three passes over K
            ops.score_window(qw[l], ks[l][:, :, :n], selector="uniform")
            return ops.dense_attn(qs[l], ks[l], vs[l])
        if args.op == "window_loop":
            acc = None
            for t in range(args.window):
                s = ops.score(qw[l][:, :, t:t + 1], ks[l][:, :, :n], selector="softmax_before_last")
                acc = s if acc is None else acc + s
            return acc
        if args.op in ("sparse", "sparse_timeline"):
            return ops.sparse_attn(qs[l], ks[l][:, :, :n], vs[l][:, :, :n], idx=idx,
                                   tail_k=ks[l][:, :, n:], tail_v=vs[l][:, :, n:])
        if args.op == "sparse_packed":
            return ops.sparse_attn(qs[l], packed[l][0], packed[l][1],
                                   tail_k=ks[l][:, :, n:], tail_v=vs[l][:, :, n:])
        if args.op == "gather":
            return ops.gather_rows(ks[l][:, :, :n], idx)
        if args.op == "copy":
            return dst.copy_(ks[l])
        if args.op == "h2d":
            return hdst.copy_(hsrc, non_blocking=True)
        if off is not None:
            # select once, stage the rows of all `nl` layers, wait for the last of them
            off.set_idx_on_gpu(sels[i + 1] if args.op == "offload_incremental" else idx, 0)
            for l2 in range(2, nl + 2):
                off._wait_part(l2)
            return None

    row = HKV * D * es
    algo = {
        "dense": 2.0 * (n + tail) * row,
        "fused": 2.0 * (n + tail) * row + 4.0 * n,
        "fused_select": 2.0 * (n + tail) * row + 4.0 * n + 4.0 * k_sel,
        "fused_then_topk": 2.0 * (n + tail) * row + 4.0 * n + 4.0 * k_sel,
        "score": 1.0 * n * row + 4.0 * n,
        "topk": 4.0 * n + 4.0 * k_sel,
        "window": 1.0 * n * row + 4.0 * n,  # one reading of K; the kernels read it twice
        "window_fused": 2.0 * (n + tail) * row + 4.0 * n,  # one reading of K and V; K is read twice
        "window_then_dense": 2.0 * (n + tail) * row + 4.0 * n,
        "window_loop": 1.0 * n * row + 4.0 * n,
        "sparse": 2.0 * (k_sel + tail) * row + 4.0 * k_sel,
        "sparse_timeline": 2.0 * (k_sel + tail) * row + 4.0 * k_sel,
        "sparse_packed": 2.0 * (k_sel + tail) * row,
        "sparse_floor": 2.0 * k_sel * row + 4.0 * k_sel,
        "empty": 0.0,
        "gather": 2.0 * k_sel * row + 4.0 * k_sel,
        "copy": 2.0 * (n + tail) * row,
        "h2d": 2.0 * k_sel * row,
        "offload_memcpy": 2.0 * k_sel * row * nl,
        "offload_zero_copy": 2.0 * k_sel * row * nl,
        "offload_incremental": 2.0 * (k_sel - int(round(args.overlap * k_sel))) * row * nl,  # rows that are new
    }[args.op]
    stream = torch.cuda.current_stream()
    for i in range(args.warmup):
        call(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for i in range(args.reps):
        call(args.warmup + i)
    e1.record(stream)
    e1.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / args.reps
    res = {"op": args.op, "ctx": n, "selected": k_sel, "tail": tail, "dtype": args.dtype,
           "layout": args.layout, "us_per_call": us, "algorithmic_bytes": algo,
           "algorithmic_GBps": algo / us / 1e3 if algo else None, "frac_of_8TBps": algo / us / 1e3 / 8000.0}
    if args.op == "sparse_timeline":
        res["timeline_ns"] = sparse_timeline()
    if args.op.startswith("offload"):
        res.update({"layers_per_selection": nl, "host_link_GBps": algo / us / 1e3})
        if args.op == "offload_incremental":
            res.update({"overlap": args.overlap, "rows_fetched_per_layer": off.last_fetch_count(0),
                        "full_restage_bytes": 2.0 * k_sel * row * nl})
    if args.then_copy > 0:
        cdst = torch.empty_like(ks[0])
        for _ in range(args.then_copy):
            cdst.copy_(ks[0])
        torch.cuda.synchronize()
        res["copy_bytes_each_way"] = ks[0].numel() * es
    print(json.dumps(res))


def sparse_timeline():
    """Device timestamps of the LAST sparse-layer call (timeline build): nanoseconds after the first workgroup's
    entry, over the workgroups whose first wave took the three-tile path (split pass) and the q heads (merge);
    (min, median, p90, max) per point, then the same for the intervals between consecutive points."""
    import ctypes as C

    import numpy as np

    out = {}
    for which, names in ((0, ["entry", "query loads issued", "index loads issued", "first tile's row loads issued",
                              "all row loads issued", "first tile consumed", "last tile consumed", "end"]),
                         (1, ["entry", "arguments and lengths there", "own splits folded", "after the barrier", "end"])):
        buf = (C.c_ulonglong * (4096 * 8))()
        check(lib().okv_stamps_read(which, buf, 0))
        a = np.frombuffer(buf, dtype=np.uint64).astype(np.int64).reshape(4096, 8)[:, :len(names)]
        a = a[(a > 0).all(axis=1)]
        a = (a - a[:, 0].min()) * 10

        def q(c):
            return [int(c.min()), int(np.median(c)), int(np.percentile(c, 90)), int(c.max())]

        d = np.diff(a, axis=1)
        out["split_pass" if which == 0 else "merge"] = {
            "workgroups": int(len(a)), "columns": "min, median, p90, max",
            "at": {nm: q(a[:, i]) for i, nm in enumerate(names)},
            "between": {f"{names[i]} -> {names[i + 1]}": q(d[:, i]) for i in range(len(names) - 1)}}
    return out


def paged(args, dev):
    """The batched serving shape: `--batch` requests of ragged length in one paged pool
    (pages shuffled from a seed), per-request k = int(ratio * length)."""
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[args.dtype]
    es = 4 if dtype == torch.float32 else 2
    lens = synth.ragged_lengths(args.batch)
    table, total = synth.shuffled_page_table(lens, args.page_size)
    if args.pages_in_order:
        flat = torch.sort(table.flatten()[table.flatten() >= 0]).values  # same pages, ascending per request
        pages = [(int(l) + args.page_size - 1) // args.page_size for l in lens]
        o = 0
        for b, pcount in enumerate(pages):
            table[b, :pcount] = torch.arange(o, o + pcount, dtype=torch.int32)
            o += pcount
    gen = torch.Generator(device=dev).manual_seed(11)
    nl = args.layers
    pools = []
    for _ in range(nl):
        if args.contiguous:
            nmax_ = int(lens.max())
            pools.append((torch.empty((args.batch, HKV, nmax_, D), dtype=dtype, device=dev).normal_(generator=gen),
                          torch.empty((args.batch, HKV, nmax_, D), dtype=dtype, device=dev).normal_(generator=gen)))
            continue
        pk = torch.empty((total, args.page_size, HKV, D), dtype=dtype, device=dev).normal_(generator=gen)
        pv = torch.empty((total, args.page_size, HKV, D), dtype=dtype, device=dev).normal_(generator=gen)
        pools.append(ops.PagedKV(pk, pv, table.to(dev), args.page_size))
    if args.contiguous:
        dense_ = lambda q, kv, **kw: ops.dense_attn(q, kv[0], kv[1], **kw)
        sparse_ = lambda q, kv, **kw: ops.sparse_attn(q, kv[0], kv[1], **kw)
        score_ = lambda q, kv, **kw: ops.score(q, kv[0], **kw)
    else:
        dense_, sparse_, score_ = ops.dense_attn, ops.sparse_attn, ops.score
    qs = [torch.randn((args.batch, HQ, 1, D), generator=gen, device=dev).to(dtype) for _ in range(nl)]
    lens_d = lens.to(dev)
    nmax = int(lens.max())
    k_per = torch.tensor([max(1, int(args.ratio * int(n))) for n in lens], dtype=torch.int32)
    kmax, k_per_d = int(k_per.max()), k_per.to(dev)
    _, scores = dense_(qs[0], pools[0], seq_len=nmax, seq_lens=lens_d, selector=args.selector, score_len=nmax,
                               score_lens=lens_d)
    idx = torch.zeros((args.batch, kmax), dtype=torch.int32, device=dev)
    ops.topk(scores, kmax, seq_lens=lens_d, k_per_seg=k_per_d, out=idx)

    slots = pools[0].slot_index(idx) if args.op in ("paged_sparse_slots", "paged_sparse_floor") else None
    floor = None
    if args.op == "paged_sparse_floor":
        # the load-only counterpart of paged_sparse_slots: same grid, slot lookups, loads and bytes, no arithmetic
        import ctypes as C

        from . import _lib
        shape = _lib.Shape(args.batch, HQ, HKV, D, kmax, 0, 0)
        rows_, splits_ = C.c_int32(0), C.c_int32(0)
        check(lib().okv_diag_split_geometry(_lib.OKV_OP_SPARSE_ATTN, C.byref(shape), C.byref(rows_), C.byref(splits_)))
        pk0 = pools[0].pool_k
        floor = (rows_.value, torch.zeros(4, dtype=torch.int32, device=dev),
                 _lib.KVLayout(ops._DTYPES[dtype], HQ, HKV, D, pk0.stride(1), pk0.stride(2), 0, None, 0, 0, 0), C)

    def call(i):
        l = i % nl
        if args.op == "paged_dense":
            return dense_(qs[l], pools[l], seq_len=nmax, seq_lens=lens_d)
        if args.op == "paged_fused":
            return dense_(qs[l], pools[l], seq_len=nmax, seq_lens=lens_d, selector=args.selector,
                                  score_len=nmax, score_lens=lens_d)
        if args.op == "paged_fused_select":
            return dense_(qs[l], pools[l], seq_len=nmax, seq_lens=lens_d, selector=args.selector, score_len=nmax,
                          score_lens=lens_d, select_k=kmax, k_per_seg=k_per_d)
        if args.op == "paged_score":
            return score_(qs[l], pools[l], score_len=nmax, selector=args.selector, score_lens=lens_d)
        if args.op == "paged_topk":
            return ops.topk(scores, kmax, seq_lens=lens_d, k_per_seg=k_per_d, out=idx)
        if args.op == "paged_sparse_floor":
            rows, sink, lay, C = floor
            return check(lib().okv_diag_gather_floor(pools[l].pool_k.data_ptr(), pools[l].pool_v.data_ptr(), C.byref(lay),
                                                     slots.data_ptr(), slots.stride(0), k_per_d.data_ptr(), kmax, args.batch,
                                                     rows, 4, sink.data_ptr(), torch.cuda.current_stream().cuda_stream))
        if args.op == "paged_sparse_slots":
            return ops.sparse_attn(qs[l], pools[l], slots=slots, sel_len=kmax, sel_lens=k_per_d)
        return sparse_(qs[l], pools[l], idx=idx, sel_len=kmax, sel_lens=k_per_d)

    tokens, sel = int(lens.sum()), int(k_per.sum())
    row = HKV * D * es
    algo = {"paged_dense": 2.0 * tokens * row, "paged_fused": 2.0 * tokens * row + 4.0 * tokens,
            "paged_fused_select": 2.0 * tokens * row + 4.0 * tokens + 4.0 * sel,
            "paged_score": 1.0 * tokens * row + 4.0 * tokens, "paged_topk": 4.0 * tokens + 4.0 * sel,
            "paged_sparse": 2.0 * sel * row + 4.0 * sel, "paged_sparse_slots": 2.0 * sel * row + 4.0 * sel,
            "paged_sparse_floor": 2.0 * sel * row + 4.0 * sel}[args.op]
    for i in range(args.warmup):
        call(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream = torch.cuda.current_stream()
    e0.record(stream)
    for i in range(args.reps):
        call(i)
    e1.record(stream)
    e1.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / args.reps
    res = {"op": args.op, "batch": args.batch, "page_size": args.page_size, "tokens": tokens,
           "selected": sel, "dtype": args.dtype, "us_per_call": us, "algorithmic_bytes": algo,
           "algorithmic_GBps": algo / us / 1e3, "frac_of_8TBps": algo / us / 1e3 / 8000.0}
    if args.then_copy > 0:
        csrc = pools[0].pool_k
        cdst = torch.empty_like(csrc)
        for _ in range(args.then_copy):
            cdst.copy_(csrc)
        torch.cuda.synchronize()
        res["copy_bytes_each_way"] = csrc.numel() * es
    print(json.dumps(res))


if __name__ == "__main__":
    main()
