"""End-to-end greedy decode of a random-init Llama-3-8B-shaped model on one MI355X.

    python -m omnikv_amd.e2e --ctx 131072 --steps 256 --real-offload

Seeded N(0, 0.02) weights (bf16), a prompt of uniform-random token ids, one prefill
call, then `--steps` greedy decode steps with OmniKV at layers 2, 8, 18 (one wait
layer).  GEMMs, norms and the prefill attention are PyTorch-ROCm; selection and decode
attention are the HIP kernels.  Prints one JSON line with prefill seconds, decode
milliseconds per token and tokens per second.
"""
from __future__ import annotations

import argparse
import json
import time

import torch

from .config import OmniKVConfig
from .model import LlamaShape, OmniKVMulLM


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ctx", type=int, default=131072)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--ratio", type=float, default=0.067)
    ap.add_argument("--selector", default="last")
    ap.add_argument("--select-layers", default="2,8,18")
    ap.add_argument("--real-offload", action="store_true")
    ap.add_argument("--offload-mode", default="zero_copy", choices=["zero_copy", "memcpy", "incremental"])
    ap.add_argument("--full-attention", action="store_true", help="no selection: every layer attends to everything")
    ap.add_argument("--graph", action="store_true", help="replay the decode step from a HIP graph")
    ap.add_argument("--trace", default=None, metavar="DESC",
                    help="every layer reports its own selection each step (full attention, eager); writes "
                         "debug_logs/selected_index_DESC.pt and prints the filter layers the run suggests")
    args = ap.parse_args()
    if args.trace:
        args.full_attention, args.graph = True, False

    dev = torch.device("cuda:0")
    shape = LlamaShape(num_hidden_layers=args.layers)
    sel = args.select_layers
    if args.full_attention:  # a filter layer that never hands anything on: all layers stay dense
        sel = str(args.layers - 1)
    cfg = OmniKVConfig(model_cls="multi", cache_cls="multi", do_select_layers=sel, num_wait_load_layers=1,
                       real_offload=args.real_offload and not args.full_attention, dense_more=True,
                       num_of_selected_tokens=args.ratio, selector_cls=args.selector, window_size=16)
    torch.set_default_dtype(torch.bfloat16)
    with torch.device(dev):
        lm = OmniKVMulLM(shape, cfg)
    lm.init_weights(seed=0, std=0.02)
    torch.set_default_dtype(torch.float32)
    ids = torch.randint(0, shape.vocab_size, (1, args.ctx), generator=torch.Generator().manual_seed(1)).to(dev)

    tracer = None
    if args.trace:
        from . import trace
        tracer = trace.SelectedIndexTracer(desc=args.trace, num_selected_tokens=args.ratio)
        trace.set_tracer(tracer)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    # room for the warm-up steps, and for the eager steps a window selector takes before a capture
    logits, cache = lm.forward(ids, None, max_new_tokens=args.steps + 48, offload_mode=args.offload_mode)
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    tok = logits[:, -1].argmax(-1, keepdim=True)
    toks = [int(tok)]
    if args.graph:
        graph, token, _ = lm.capture_decode(cache, tok, warmup=3)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        toks.append(int(token))
    else:
        for _ in range(3):  # warm-up steps (workspace growth, first selection)
            logits, cache = lm.forward(tok, cache)
            tok = logits[:, -1].argmax(-1, keepdim=True)
            toks.append(int(tok))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            logits, cache = lm.forward(tok, cache)
            tok = logits[:, -1].argmax(-1, keepdim=True)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    if args.real_offload:
        cache._join_worker()
    extra = {}
    if args.real_offload and args.offload_mode == "incremental" and not args.full_attention:
        # rows per layer the last selection of each filter layer had to fetch (of `selected`)
        extra["rows_fetched_per_layer_last_step"] = {str(f): cache.last_fetch_count(f) for f in sorted(cache._plan)}
    if tracer is not None:
        mass, _ = tracer.matrices()
        layers, quality = trace.suggest_filter_layers(mass, num_filters=len(args.select_layers.split(",")))
        extra = {**extra, "trace_file": tracer.save_idx(), "suggested_select_layers": layers, "suggested_quality": quality,
                 "configured_quality": trace.schedule_quality(mass, [int(i) for i in args.select_layers.split(",")])[0]}
    print(json.dumps({
        **extra,
        "model": f"random-init Llama-3-8B shape, {args.layers} layers, bf16", "context": args.ctx,
        "decode_steps": args.steps, "select_layers": sel, "selected": int(args.ratio * args.ctx),
        "selector": args.selector, "real_offload": bool(args.real_offload and not args.full_attention),
        "offload_mode": args.offload_mode if args.real_offload else None, "full_attention": args.full_attention, "launch": "hip_graph_replay" if args.graph else "eager",
        "prefill_s": prefill_s, "decode_ms_per_token": dt * 1e3 / args.steps, "decode_tokens_per_s": args.steps / dt,
        "hbm_gb_allocated": round(torch.cuda.max_memory_allocated() / 1e9, 1),
        "first_tokens": toks,
    }))


if __name__ == "__main__":
    main()
