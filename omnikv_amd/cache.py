"""OmniKVMultiStageCache on MI355X: the reference's `cache_cls: multi`
(modeling/spec_cache.py:253-385) with the same constructor, attributes and
update / set_idx_on_gpu / from_dynamic_cache behaviour, over storage laid out for
the HIP kernels.

Storage.  Every layer owns preallocated buffers in the reference's own layout,
(bsz, Hkv, capacity, D) -- each kv head one contiguous stream of 256-byte rows, which
is what the split pass reads fastest -- and hands out (bsz, Hkv, L, D) VIEWS of them,
so appending a decode token writes Hkv rows instead of re-allocating the layer (the
reference's torch.cat, spec_cache.py:363-368).  With real_offload the layers that only
ever read selected rows keep their prompt K/V in PINNED host memory as interleaved
(N, 2, Hkv, D) rows, so one host row carries a token's K and V.

Two ways to consume it:
  * the reference's: `update()` returns the tensors a third-party attention
    would read (full cache, or gathered rows ++ tail), bit-identical to the
    reference's values;
  * the native one: `append()` + `attend()` / `attend_and_select()` run the HIP
    attention kernels straight on the storage; the gather is fused into the sparse
    attention, nothing is concatenated.
"""
from __future__ import annotations

import threading
from typing import Any, Dict, List, Optional, Tuple

import torch

from . import ops
from ._lib import check, lib

__all__ = ["OmniKVMultiStageCache", "WOPackCache", "OmniKVLazyCache", "get_cache_cls", "get_idx_iou_score",
           "layer_schedule"]


def layer_schedule(full_attn_layers, num_hidden_layers: int, num_wait_load_layers: int):
    """layer -> (reads selected rows only, its filter layer, next full layer);
    modeling/spec_cache.py:271-281."""
    state = {}
    full = list(full_attn_layers)
    for lo in full:
        hi = num_hidden_layers
        for i in range(lo + 1, num_hidden_layers):
            if i in full:
                hi = i
                break
        for i in range(lo, min(hi, lo + num_wait_load_layers + 1)):
            state[i] = (False, lo, hi)
        for i in range(min(hi, lo + num_wait_load_layers + 1), hi):
            state[i] = (True, lo, hi)
    return state


class _Store:
    """K and V of one layer, (bsz, Hkv, capacity, D) with room to append."""

    def __init__(self, bsz, capacity, hkv, d, dtype, device):
        self.k = torch.empty((bsz, hkv, capacity, d), dtype=dtype, device=device)
        self.v = torch.empty((bsz, hkv, capacity, d), dtype=dtype, device=device)
        self.len = 0

    @property
    def capacity(self):
        return self.k.shape[2]

    def reserve(self, n):
        if n <= self.capacity:
            return
        cap = max(n, int(self.capacity * 1.5) + 64)
        for name in ("k", "v"):
            old = getattr(self, name)
            new = torch.empty(tuple(old.shape[:2]) + (cap, old.shape[3]), dtype=old.dtype, device=old.device)
            new[:, :, : self.len].copy_(old[:, :, : self.len])
            setattr(self, name, new)

    def append(self, key_states, value_states):
        """key_states / value_states: (bsz, Hkv, n, D)."""
        n = key_states.shape[2]
        self.reserve(self.len + n)
        self.k[:, :, self.len: self.len + n].copy_(key_states)
        self.v[:, :, self.len: self.len + n].copy_(value_states)
        self.len += n

    def views(self, lo=0, hi=None):
        hi = self.len if hi is None else hi
        return self.k[:, :, lo:hi], self.v[:, :, lo:hi]


class OmniKVMultiStageCache:
    """Drop-in for the reference class of the same name (default DenseMore=True)."""

    def __init__(self, full_attn_layers: List, num_hidden_layers, num_wait_load_layers=2, real_offload=True,
                 max_new_tokens: int = 1024, offload_mode: str = "zero_copy", cpu_num_threads: int = 8,
                 skip_threshold: Optional[float] = None):
        self.stage = "prefill"
        # lazy re-selection (OmniKVLazyCache.set_out_idx, modeling/spec_cache.py:539-557): a new
        # selection whose IoU with the one in use exceeds the threshold is dropped
        self.skip_threshold = skip_threshold
        self.num_skipped_selections = 0
        self.full_attn_layers = full_attn_layers
        self.num_hidden_layers = num_hidden_layers
        self.num_wait_layers = num_wait_load_layers
        self.layer_state = layer_schedule(full_attn_layers, num_hidden_layers, num_wait_load_layers)
        self.need_cat_layers = []
        self.device = "cpu" if real_offload else None
        self.real_offload = bool(real_offload)
        if offload_mode not in ("memcpy", "zero_copy", "incremental"):
            raise ValueError("offload_mode must be 'memcpy', 'zero_copy' or 'incremental'")
        if offload_mode == "incremental" and not self._stage_at_selection:
            raise ValueError("incremental staging plans one exchange per selection for the whole group of layers; "
                             "a cache that stages layer by layer at layer time takes 'zero_copy' or 'memcpy'")
        self.offload_mode = offload_mode
        self.cpu_num_threads = int(cpu_num_threads)
        self.max_new_tokens = int(max_new_tokens)
        self._seen_tokens = 0
        # reference-visible containers
        self.key_cache: List[torch.Tensor] = []
        self.value_cache: List[torch.Tensor] = []
        self.part_key: Dict[int, torch.Tensor] = {}
        self.part_value: Dict[int, torch.Tensor] = {}
        self.tail_k: Dict[int, torch.Tensor] = {}
        self.tail_v: Dict[int, torch.Tensor] = {}
        # storage behind them
        self._store: Dict[int, _Store] = {}        # GPU K/V (all layers unless offloaded)
        self._host_kv: Dict[int, torch.Tensor] = {}  # pinned (N, 2, Hkv, D) of offloaded layers
        self._tail: Dict[int, _Store] = {}
        self._idx: Dict[int, torch.Tensor] = {}    # filter layer -> (bsz, k) int32 on the GPU
        self._part: Dict[int, torch.Tensor] = {}   # sparse layer -> (bsz, k, 2, Hkv, D) staged rows
        self._sel_gen: Dict[int, int] = {}         # filter layer -> how many selections it has made
        self._part_src: Dict[int, int] = {}        # sparse layer -> selection number it was gathered with
        self._staged_for: Dict[int, int] = {}      # sparse layer -> selection number its rows were staged with
        self._staging: Dict[int, torch.Tensor] = {}
        self._plan: Dict[int, Dict[str, torch.Tensor]] = {}  # filter layer -> slot maps of its group (incremental mode)
        self._events: Dict[int, torch.cuda.Event] = {}
        self._recorded: Dict[int, threading.Event] = {}
        self._copy_stream: Optional[torch.cuda.Stream] = None
        self._d2h_stream: Optional[torch.cuda.Stream] = None
        self._d2h_pending = False
        self._d2h_staging: Optional[torch.Tensor] = None
        self._worker: Optional[threading.Thread] = None
        self._prefill_len: Optional[int] = None
        # static decode (enable_static_decode): lengths and write positions live on the device
        self._static = False
        self._pos = self._len32 = self._tail_pos = self._tail_len32 = None

    # ------------------------------------------------------------ storage
    def _gpu_store(self, layer_idx, like: torch.Tensor, n_first: int) -> _Store:
        st = self._store.get(layer_idx)
        if st is None:
            b, hkv, _, d = like.shape
            st = _Store(b, n_first + self.max_new_tokens, hkv, d, like.dtype, like.device)
            self._store[layer_idx] = st
        return st

    def _sync_lists(self, layer_idx):
        """Keep key_cache / value_cache (the reference's public lists) pointing at views."""
        while len(self.key_cache) <= layer_idx:
            self.key_cache.append(None)
            self.value_cache.append(None)
        if layer_idx in self._host_kv:
            h = self._host_kv[layer_idx]
            self.key_cache[layer_idx] = h[:, 0].permute(1, 0, 2)[None]
            self.value_cache[layer_idx] = h[:, 1].permute(1, 0, 2)[None]
        else:
            self.key_cache[layer_idx], self.value_cache[layer_idx] = self._store[layer_idx].views()

    def get_seq_length(self, layer_idx: int = 0) -> int:
        return self._seen_tokens

    # ------------------------------------------------------------ reference API
    # ------------------------------------------------------------ static decode (graph capture)
    def enable_static_decode(self) -> None:
        """After the prefill: switch the decode path to one whose launches never change
        shape, so that a whole decode step can be captured in a HIP graph and replayed.
        Sequence lengths and append positions become device scalars (the kernels read
        per-request lengths from device memory); every buffer a step touches is
        preallocated.  With real_offload only the zero-copy mode qualifies: there the GPU
        fetches the selected pinned rows itself, on the copy stream, and the fork and join of
        that stream become part of the graph; the memcpy mode packs rows on host threads."""
        if self.real_offload and self.offload_mode == "memcpy":
            raise NotImplementedError("static decode with real_offload needs offload_mode='zero_copy' or 'incremental'")
        if self._static:
            return
        any_store = next(iter(self._store.values()))
        dev = any_store.k.device
        n = self._seen_tokens
        self._finish_prefill_offload()
        for layer_idx, sparse in ((i, s[0]) for i, s in self.layer_state.items()):
            if sparse:
                if layer_idx not in self._tail:
                    if self.real_offload:
                        host = self._host_kv[layer_idx]
                        b, hkv, d, dt = 1, host.shape[2], host.shape[3], host.dtype
                    else:
                        st = self._store[layer_idx]
                        (b, hkv, _, d), dt = st.k.shape, st.k.dtype
                    self._tail[layer_idx] = _Store(b, self.max_new_tokens, hkv, d, dt, dev)
            else:
                self._store[layer_idx].reserve(n + self.max_new_tokens)
        tails = [t.len for t in self._tail.values()]
        t0 = tails[0] if tails else 0
        self._pos = torch.tensor([n], dtype=torch.int64, device=dev)
        self._len32 = torch.tensor([n + 1], dtype=torch.int32, device=dev)
        self._tail_pos = torch.tensor([t0], dtype=torch.int64, device=dev)
        self._tail_len32 = torch.tensor([t0 + 1], dtype=torch.int32, device=dev)
        # how many static steps the preallocated buffers take: every step writes one row at
        # _pos into the dense stores and one at _tail_pos into the tails
        dense_caps = [self._store[i].capacity for i, s in self.layer_state.items() if not s[0]]
        tail_caps = [t.capacity for t in self._tail.values()]
        self._static_caps = (min(dense_caps) if dense_caps else n + self.max_new_tokens,
                             min(tail_caps) if tail_caps else t0 + self.max_new_tokens)
        self._static_budget = min(self._static_caps[0] - n, self._static_caps[1] - t0)
        self._static_steps = 0
        self._static = True

    @property
    def static_steps_left(self) -> int:
        """Static decode steps (eager or graph replays) the preallocated buffers still take."""
        return self._static_budget - self._static_steps

    def note_static_step(self) -> None:
        """Host-side count of static steps, taken BEFORE a step runs (each replay of a captured
        step counts: the graph itself cannot).  The appends of a static step write at device
        positions that nothing on the device checks, so running past the buffers must be
        refused here."""
        if self._static_steps >= self._static_budget:
            raise RuntimeError(
                f"static decode buffers are full after {self._static_steps} steps "
                f"(max_new_tokens={self.max_new_tokens}): build the cache with a larger max_new_tokens")
        self._static_steps += 1

    def advance_static(self) -> None:
        """End of a static decode step: one more token everywhere (device-side adds).  The
        positions stop at the last row of the buffers even if a caller replays a captured
        step more often than note_static_step allows."""
        dense_cap, tail_cap = self._static_caps
        self._pos.add_(1).clamp_(max=dense_cap - 1)
        self._len32.add_(1).clamp_(max=dense_cap)
        self._tail_pos.add_(1).clamp_(max=tail_cap - 1)
        self._tail_len32.add_(1).clamp_(max=tail_cap)

    def append(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int) -> None:
        """Store the new rows of `layer_idx` (what update() does before it returns;
        modeling/spec_cache.py:308-369)."""
        if layer_idx == 0:
            self._seen_tokens += key_states.shape[-2]
        sparse = self.layer_state[layer_idx][0]
        if self._static:
            st = self._tail[layer_idx] if sparse else self._store[layer_idx]
            where = self._tail_pos if sparse else self._pos
            st.k.index_copy_(2, where, key_states)
            st.v.index_copy_(2, where, value_states)
            return
        if sparse and self.stage != "prefill":
            tl = self._tail.get(layer_idx)
            if tl is None:
                b, hkv, _, d = key_states.shape
                tl = _Store(b, self.max_new_tokens, hkv, d, key_states.dtype, key_states.device)
                self._tail[layer_idx] = tl
            tl.append(key_states, value_states)
            self.tail_k[layer_idx], self.tail_v[layer_idx] = tl.views()
            return
        if sparse and self.real_offload:
            # prompt K/V of a selected-rows-only layer go to pinned host memory
            if key_states.shape[0] != 1:
                raise NotImplementedError("real_offload keeps one request (the reference is bs=1 too)")
            n = key_states.shape[2]
            host = self._host_kv.get(layer_idx)
            if host is None:
                hkv, d = key_states.shape[1], key_states.shape[3]
                host = torch.empty((n, 2, hkv, d), dtype=key_states.dtype, pin_memory=True)
                self._host_kv[layer_idx] = host
            elif host.shape[0] != n:
                raise NotImplementedError("an offloaded layer takes its prompt in one prefill call")
            else:
                # the same pinned rows are about to hold another prompt: whatever was staged from them,
                # and the incremental mode's record of which tokens sit in which slots, is stale
                self._plan.pop(self.layer_state[layer_idx][1], None)
                self._staged_for.pop(layer_idx, None)
                self._part_src.pop(layer_idx, None)
                self.part_key.pop(layer_idx, None)
                self.part_value.pop(layer_idx, None)
            if not key_states.is_cuda:  # rows that already live on the host (an adopted cache)
                host[:, 0].copy_(key_states[0].permute(1, 0, 2))
                host[:, 1].copy_(value_states[0].permute(1, 0, 2))
                self._sync_lists(layer_idx)
                return
            # device-to-host on a stream of its own: the next layer's prefill compute runs
            # meanwhile; the stream is drained when decoding starts (_finish_prefill_offload)
            cur = torch.cuda.current_stream(key_states.device)
            if self._d2h_stream is None:
                self._d2h_stream = torch.cuda.Stream(device=key_states.device)
            self._d2h_stream.wait_stream(cur)
            with torch.cuda.stream(self._d2h_stream):
                # into the host layout on the GPU first (a strided device-to-host copy crawls at a
                # few GB/s), then one contiguous copy at link speed; the staging buffer is reused
                # layer after layer, in stream order
                stg = self._d2h_staging
                if stg is None or stg.shape != host.shape or stg.dtype != host.dtype:
                    stg = torch.empty(host.shape, dtype=host.dtype, device=key_states.device)
                    self._d2h_staging = stg
                stg[:, 0].copy_(key_states[0].permute(1, 0, 2))
                stg[:, 1].copy_(value_states[0].permute(1, 0, 2))
                host.copy_(stg, non_blocking=True)
            key_states.record_stream(self._d2h_stream)
            value_states.record_stream(self._d2h_stream)
            self._d2h_pending = True
            self._sync_lists(layer_idx)
            return
        st = self._gpu_store(layer_idx, key_states, key_states.shape[2])
        st.append(key_states, value_states)
        self._sync_lists(layer_idx)

    def append_projected(self, q_lin: torch.Tensor, k_lin: torch.Tensor, v_lin: torch.Tensor, cos: torch.Tensor,
                         sin: torch.Tensor, layer_idx: int, num_q_heads: int) -> torch.Tensor:
        """Static decode: the rotary embedding of the new token's q and k and the append of its k and v rows
        in one launch (what append() stores, written by the kernel that rotates).  q_lin / k_lin / v_lin are the
        projections' outputs (bsz, 1, heads * D); returns the rotated q (bsz, Hq, 1, D)."""
        if not self._static:
            raise RuntimeError("append_projected serves static decode; elsewhere rotate, then append()")
        if layer_idx == 0:
            self._seen_tokens += 1
        sparse = self.layer_state[layer_idx][0]
        st = self._tail[layer_idx] if sparse else self._store[layer_idx]
        return ops.rope_append(q_lin, k_lin, v_lin, cos, sin, num_q_heads, st.k.shape[1], st.k, st.v,
                               self._tail_pos if sparse else self._pos)

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """modeling/spec_cache.py:308-369: store the new rows and return what this
        layer's attention reads."""
        self.append(key_states, value_states, layer_idx)
        if self.layer_state[layer_idx][0]:
            if self.stage == "prefill":
                return key_states, value_states
            pk, pv = self._materialised_part(layer_idx)
            return (torch.cat([pk, self.tail_k[layer_idx]], dim=-2),
                    torch.cat([pv, self.tail_v[layer_idx]], dim=-2))
        return self.key_cache[layer_idx], self.value_cache[layer_idx]

    def set_idx_on_gpu(self, idx: torch.Tensor, sel_layer_idx: int) -> None:
        """modeling/spec_cache.py:290-306.  idx: (bsz, k) ascending token indices
        (int64 as the reference's selector returns them, or int32)."""
        if idx.dim() == 1:
            idx = idx[None]
        idx32 = idx if idx.dtype == torch.int32 else idx.to(torch.int32)
        idx32 = idx32.contiguous()
        old = self._idx.get(sel_layer_idx)
        if self.skip_threshold is not None and old is not None and not self._static:
            if get_idx_iou_score(idx32.view(-1), old.view(-1)) > self.skip_threshold:
                self.num_skipped_selections += 1
                return
        self._idx[sel_layer_idx] = idx32
        self._sel_gen[sel_layer_idx] = self._sel_gen.get(sel_layer_idx, 0) + 1
        hi = self.layer_state[sel_layer_idx][2]
        lo = sel_layer_idx + self.num_wait_layers + 1
        for i in range(lo, hi):
            self.part_key.pop(i, None)
            self.part_value.pop(i, None)
            self._part_src.pop(i, None)
        if self.real_offload and lo < hi and self._stage_at_selection:
            self._start_offload(idx32, list(range(lo, hi)))

    _stage_at_selection = True  # False: each sparse layer stages its own rows when it runs

    @staticmethod
    def from_dynamic_cache(cache, full_attn_layers: List, num_hidden_layers, num_wait_load_layers=2,
                           real_offload=True, **kwargs):
        """modeling/spec_cache.py:371-385; `cache` is anything with key_cache /
        value_cache lists (or transformers >= 4.54 `.layers[i].keys/.values`), usually empty
        (the reference adopts the fresh DynamicCache of the first forward, omnikv.py:339-341).
        A populated cache is taken in as a prompt: its rows are COPIED into this cache's own
        storage and tiered as the constructor arguments say -- with real_offload the
        selected-rows-only layers go to pinned host memory whichever device they came on,
        where the reference keeps the adopted tensors as they are."""
        c = kwargs.pop("_cls", OmniKVMultiStageCache)(full_attn_layers, num_hidden_layers, num_wait_load_layers,
                                                       real_offload, **kwargs)
        keys = getattr(cache, "key_cache", None)
        vals = getattr(cache, "value_cache", None)
        if keys is None and hasattr(cache, "layers"):
            keys = [l.keys for l in cache.layers if getattr(l, "keys", None) is not None]
            vals = [l.values for l in cache.layers if getattr(l, "values", None) is not None]
        seen = getattr(cache, "_seen_tokens", None)
        on_gpu = [k.device for k in (keys or []) if k.is_cuda]
        dev = on_gpu[0] if on_gpu else torch.device("cuda", torch.cuda.current_device())
        for i, (k, v) in enumerate(zip(keys or [], vals or [])):
            to_host = c.real_offload and c.layer_state[i][0]
            if not to_host:  # stays (or becomes) GPU resident
                k, v = k.to(dev), v.to(dev)
            c.append(k, v, i)
        c._seen_tokens = seen if seen is not None else (keys[0].shape[-2] if keys else 0)
        return c

    # ------------------------------------------------------------ offload tier
    def _finish_prefill_offload(self) -> None:
        """The prompt's host copies are complete before anything reads them (host threads
        of the memcpy mode included)."""
        if self._d2h_pending:
            self._d2h_stream.synchronize()
            self._d2h_pending = False
            self._d2h_staging = None  # half a gigabyte per layer at 128K: not kept past the prefill

    def _start_offload(self, idx32: torch.Tensor, layers: List[int]) -> None:
        if idx32.shape[0] != 1:
            raise NotImplementedError("real_offload keeps one request")
        self._finish_prefill_offload()
        self._join_worker()
        dev = idx32.device
        if self._copy_stream is None:
            self._copy_stream = torch.cuda.Stream(device=dev)
        k = idx32.shape[1]
        for i in layers:
            host = self._host_kv[i]
            part = self._part.get(i)
            if part is None or part.shape[1] != k:
                self._part[i] = torch.empty((1, k) + tuple(host.shape[1:]), dtype=host.dtype, device=dev)
            self._recorded[i] = threading.Event()
            if i not in self._events:
                self._events[i] = torch.cuda.Event()
        if self.offload_mode == "incremental":
            self._copy_stream.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(self._copy_stream):
                self._stage_incremental(idx32, layers)
                for i in layers:
                    self._recorded[i].set()
            return
        if self.offload_mode == "zero_copy":
            # the GPU reads the pinned rows itself: one gather per layer on the copy stream
            self._copy_stream.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(self._copy_stream):
                for i in layers:
                    host = self._host_kv[i]
                    src = host.view(1, host.shape[0], 1, -1).permute(0, 2, 1, 3)  # (1, 1, N, 2*Hkv*D) rows
                    dst = self._part[i].view(1, k, 1, -1).permute(0, 2, 1, 3)
                    _gather_wide(src, idx32, dst)
                    self._events[i].record(self._copy_stream)
                    self._recorded[i].set()
            return
        host_idx = idx32[0].cpu()  # synchronises with the selection, as the reference's idx.cpu()
        copy_stream = self._copy_stream

        def work():
            for i in layers:
                host = self._host_kv[i]
                row_bytes = host.stride(0) * host.element_size()
                stg = self._staging.get(i)
                if stg is None or stg.numel() < k * row_bytes:
                    stg = torch.empty(k * row_bytes, dtype=torch.uint8, pin_memory=True)
                    self._staging[i] = stg
                else:
                    self._events[i].synchronize()  # last step's copy out of this staging is done
                check(lib().okv_offload_stage(
                    host.data_ptr(), row_bytes, host_idx.data_ptr(), k, stg.data_ptr(), self.cpu_num_threads,
                    self._part[i].data_ptr(), copy_stream.cuda_stream, None))
                self._events[i].record(copy_stream)
                self._recorded[i].set()

        self._worker = threading.Thread(target=work, daemon=True)
        self._worker.start()

    def _stage_incremental(self, idx32: torch.Tensor, layers: List[int]) -> None:
        """On the current (copy) stream: plan which rows the new selection does not find staged and
        which slots the dropped rows free (okv_offload_plan, once for the group), then fetch those
        rows of every layer from pinned memory into the freed slots (okv_offload_fetch) and record
        the layer's event.  Nothing here touches the host; the row count lives on the device."""
        sel = self.layer_state[layers[0]][1]
        dev, k = idx32.device, idx32.shape[1]
        n_tok = self._host_kv[layers[0]].shape[0]
        plan = self._plan.get(sel)
        if plan is None or plan["slot_tok"].shape[0] != k or plan["slot_of"].shape[0] != n_tok:
            plan = {"slot_tok": torch.full((k,), -1, dtype=torch.int32, device=dev),
                    "slot_of": torch.full((n_tok,), -1, dtype=torch.int32, device=dev),
                    "fetch_tok": torch.empty((k,), dtype=torch.int32, device=dev),
                    "fetch_slot": torch.empty((k,), dtype=torch.int32, device=dev),
                    "fetch_count": torch.zeros((1,), dtype=torch.int32, device=dev)}
            self._plan[sel] = plan
        stream = torch.cuda.current_stream(dev).cuda_stream
        check(lib().okv_offload_plan(idx32.data_ptr(), k, plan["slot_tok"].data_ptr(), plan["slot_of"].data_ptr(), n_tok,
                                     plan["fetch_tok"].data_ptr(), plan["fetch_slot"].data_ptr(),
                                     plan["fetch_count"].data_ptr(), stream))
        for i in layers:
            host = self._host_kv[i]
            part = self._part.get(i)
            if part is None or part.shape[1] != k:
                part = torch.empty((1, k) + tuple(host.shape[1:]), dtype=host.dtype, device=dev)
                self._part[i] = part
            if i not in self._events:
                self._events[i] = torch.cuda.Event()
            check(lib().okv_offload_fetch(host.data_ptr(), host.stride(0) * host.element_size(), plan["fetch_tok"].data_ptr(),
                                          plan["fetch_slot"].data_ptr(), plan["fetch_count"].data_ptr(), k,
                                          part.data_ptr(), stream))
            self._events[i].record(torch.cuda.current_stream(dev))

    def last_fetch_count(self, sel_layer_idx: int) -> int:
        """Rows per layer the latest selection of this filter layer had to fetch over the host link
        (incremental mode); synchronises with the device."""
        return int(self._plan[sel_layer_idx]["fetch_count"].item())

    def _stage_static(self, sel_layer_idx: int, idx32: torch.Tensor) -> None:
        """Static decode with the host tier: the copy stream gathers the selected pinned rows
        of every layer of the group (the GPU reads host memory itself), one event per layer.
        Nothing here touches the host, so the whole exchange is captured with the step."""
        hi = self.layer_state[sel_layer_idx][2]
        lo = sel_layer_idx + self.num_wait_layers + 1
        if lo >= hi:
            return
        dev, k = idx32.device, idx32.shape[1]
        if self._copy_stream is None:
            self._copy_stream = torch.cuda.Stream(device=dev)
        self._copy_stream.wait_stream(torch.cuda.current_stream(dev))
        if self.offload_mode == "incremental":
            with torch.cuda.stream(self._copy_stream):
                self._stage_incremental(idx32, list(range(lo, hi)))
            return
        with torch.cuda.stream(self._copy_stream):
            for i in range(lo, hi):
                host = self._host_kv[i]
                part = self._part.get(i)
                if part is None or part.shape[1] != k:
                    part = torch.empty((1, k) + tuple(host.shape[1:]), dtype=host.dtype, device=dev)
                    self._part[i] = part
                if i not in self._events:
                    self._events[i] = torch.cuda.Event()
                _gather_wide(host.view(1, host.shape[0], 1, -1).permute(0, 2, 1, 3), idx32,
                             part.view(1, k, 1, -1).permute(0, 2, 1, 3))
                self._events[i].record(self._copy_stream)

    def _join_worker(self):
        if self._worker is not None:
            self._worker.join()
            self._worker = None

    def _wait_part(self, layer_idx: int) -> torch.Tensor:
        """Staged rows of an offloaded layer, ordered behind their copy on the current stream."""
        sel = self.layer_state[layer_idx][1]
        if not self._stage_at_selection and self._staged_for.get(layer_idx) != self._sel_gen[sel]:
            self._start_offload(self._idx[sel], [layer_idx])  # this layer only, now
            self._staged_for[layer_idx] = self._sel_gen[sel]
        self._recorded[layer_idx].wait()
        torch.cuda.current_stream(self._part[layer_idx].device).wait_event(self._events[layer_idx])
        return self._part[layer_idx]

    # ------------------------------------------------------------ gathered views
    def _materialised_part(self, layer_idx: int):
        """(bsz, Hkv, k, D) K and V rows of the current selection; gathers on first use."""
        sel = self.layer_state[layer_idx][1]
        idx32 = self._idx[sel]
        if self._part_src.get(layer_idx) != self._sel_gen[sel]:
            if self.real_offload:
                part = self._wait_part(layer_idx)
                if self.offload_mode == "incremental":
                    # the staged rows are a set; the reference hands them out in ascending token order
                    order = self._plan[sel]["slot_of"][idx32[0].long()].long()
                    part = part.index_select(1, order)
                pk = part[:, :, 0].permute(0, 2, 1, 3)
                pv = part[:, :, 1].permute(0, 2, 1, 3)
            else:
                kview, vview = self._store[layer_idx].views(0, self._prefill_rows(layer_idx))
                pk = ops.gather_rows(kview, idx32)
                pv = ops.gather_rows(vview, idx32)
            self.part_key[layer_idx], self.part_value[layer_idx] = pk, pv
            self._part_src[layer_idx] = self._sel_gen[sel]
        return self.part_key[layer_idx], self.part_value[layer_idx]

    def _prefill_rows(self, layer_idx: int) -> int:
        return self._store[layer_idx].len

    # ------------------------------------------------------------ native attention
    def attend(self, query_states: torch.Tensor, layer_idx: int, scale: Optional[float] = None) -> torch.Tensor:
        """Decode attention of `layer_idx` over what update() would have returned,
        without building it.  query_states: (bsz, Hq, 1, D); returns (bsz, Hq, D)."""
        if self._static:
            if self.layer_state[layer_idx][0] and self.real_offload:
                # rows staged by the copy stream since the filter layer ran (_stage_static)
                torch.cuda.current_stream(query_states.device).wait_event(self._events[layer_idx])
                part, tl = self._part[layer_idx], self._tail[layer_idx]
                return ops.sparse_attn(query_states, part[:, :, 0].permute(0, 2, 1, 3), part[:, :, 1].permute(0, 2, 1, 3),
                                       tail_k=tl.k, tail_v=tl.v, tail_len=tl.capacity, tail_lens=self._tail_len32,
                                       scale=scale)
            st = self._store[layer_idx]
            if self.layer_state[layer_idx][0]:
                tl = self._tail[layer_idx]
                kview, vview = st.views()
                return ops.sparse_attn(query_states, kview, vview, idx=self._idx[self.layer_state[layer_idx][1]],
                                       tail_k=tl.k, tail_v=tl.v, tail_len=tl.capacity, tail_lens=self._tail_len32,
                                       scale=scale)
            return ops.dense_attn(query_states, st.k, st.v, seq_len=st.capacity, seq_lens=self._len32, scale=scale)
        if self.layer_state[layer_idx][0] and self.stage != "prefill":
            sel = self.layer_state[layer_idx][1]
            tk = self.tail_k.get(layer_idx)
            tv = self.tail_v.get(layer_idx)
            if self.real_offload:
                part = self._wait_part(layer_idx)
                pk = part[:, :, 0].permute(0, 2, 1, 3)
                pv = part[:, :, 1].permute(0, 2, 1, 3)
                return ops.sparse_attn(query_states, pk, pv, tail_k=tk, tail_v=tv, scale=scale)
            kview, vview = self._store[layer_idx].views()
            return ops.sparse_attn(query_states, kview, vview, idx=self._idx[sel], tail_k=tk, tail_v=tv, scale=scale)
        kview, vview = self._store[layer_idx].views()
        return ops.dense_attn(query_states, kview, vview, scale=scale)

    def select_with_query(self, query_states: torch.Tensor, layer_idx: int, num_selected_tokens: int,
                          consider_len: int, selector_cls: str, forced_tail: int = 0) -> torch.Tensor:
        """Filter layer with a selector that scores separately from the layer's attention (the
        window selectors `uniform` / `exp`, modeling/omnikv.py:59-105,177-210): scores of the first
        `consider_len` cached tokens from the rotated query block (bsz, Hq, W, D), top-k, the last
        `forced_tail` prompt positions appended (the window still inside the prompt), then
        set_idx_on_gpu.  In static decode everything has a fixed shape and lands in a fixed index
        buffer, so the step can be captured.  Returns the int32 (bsz, k) selection."""
        from . import selector
        if not self._static:
            idx = selector.select_from_query(query_states, self.key_cache[layer_idx], num_selected_tokens, consider_len,
                                             selector_cls)
            if forced_tail:
                end = consider_len + forced_tail
                tail_idx = torch.arange(end - forced_tail, end, device=idx.device)
                idx = torch.cat([idx, tail_idx[None, :].repeat(idx.shape[0], 1)], dim=1)
            self.set_idx_on_gpu(idx, layer_idx)
            return self._idx[layer_idx]
        if forced_tail:
            raise RuntimeError("static decode with a window selector starts once the window has left the prompt")
        scores = selector.score_from_query(query_states, self._store[layer_idx].k, consider_len, selector_cls)
        k = min(num_selected_tokens, consider_len)
        buf = self._idx.get(layer_idx)
        if buf is None or buf.shape[1] != k:
            buf = torch.empty((scores.shape[0], k), dtype=torch.int32, device=scores.device)
            self._idx[layer_idx] = buf  # the sparse layers keep reading this very buffer
        ops.topk(scores, k, out=buf)
        self._sel_gen[layer_idx] = self._sel_gen.get(layer_idx, 0) + 1
        if self.real_offload:
            self._stage_static(layer_idx, buf)
        return buf

    def attend_and_select_window(self, query_states: torch.Tensor, query_window: torch.Tensor, layer_idx: int,
                                 num_selected_tokens: int, consider_len: int, selector_cls: str, forced_tail: int = 0,
                                 scale: Optional[float] = None):
        """Filter layer with a window selector (`uniform` / `exp`) whose first scoring pass rides on the
        layer's own attention: what select_with_query followed by attend do, in two passes over K
        instead of three.  query_states: (bsz, Hq, 1, D), the attention's query; query_window:
        (bsz, Hq, W, D), rotated.  Returns (attention output, idx int32 (bsz, k)).  Operands the
        kernel does not take (fp32, more than 64 window columns per kv head) go the separate way."""
        st = self._store[layer_idx]
        if not ops.window_supported(query_window, st.k):
            idx = self.select_with_query(query_window, layer_idx, num_selected_tokens, consider_len, selector_cls,
                                         forced_tail=forced_tail)
            return self.attend(query_states, layer_idx, scale=scale), idx
        k = min(num_selected_tokens, consider_len)
        if self._static:
            if forced_tail:
                raise RuntimeError("static decode with a window selector starts once the window has left the prompt")
            out, scores = ops.dense_attn_window(query_states, query_window, st.k, st.v, selector=selector_cls,
                                                seq_len=st.capacity, seq_lens=self._len32, score_len=consider_len,
                                                scale=scale)
            buf = self._idx.get(layer_idx)
            if buf is None or buf.shape[1] != k:
                buf = torch.empty((scores.shape[0], k), dtype=torch.int32, device=scores.device)
                self._idx[layer_idx] = buf  # the sparse layers keep reading this very buffer
            ops.topk(scores, k, out=buf)
            self._sel_gen[layer_idx] = self._sel_gen.get(layer_idx, 0) + 1
            if self.real_offload:
                self._stage_static(layer_idx, buf)
            return out, buf
        kview, vview = st.views()
        out, scores = ops.dense_attn_window(query_states, query_window, kview, vview, selector=selector_cls,
                                            score_len=consider_len, scale=scale)
        idx = ops.topk(scores, k).to(torch.int64)
        if forced_tail:
            end = consider_len + forced_tail
            tail_idx = torch.arange(end - forced_tail, end, device=idx.device)
            idx = torch.cat([idx, tail_idx[None, :].repeat(idx.shape[0], 1)], dim=1)
        self.set_idx_on_gpu(idx, layer_idx)
        return out, self._idx[layer_idx]

    def attend_and_select(self, query_states: torch.Tensor, layer_idx: int, num_selected_tokens: int,
                          consider_len: int, selector_cls: str = "last", scale: Optional[float] = None):
        """Filter layer: dense attention, the filter-layer scores from the same pass over K and
        the top-k of those scores in one library call, then set_idx_on_gpu
        (modeling/omnikv.py:189-212 followed by the layer's own attention).  Returns
        (attention output, idx int32 (bsz, k))."""
        k = min(num_selected_tokens, consider_len)
        if self._static:
            st = self._store[layer_idx]
            buf = self._idx.get(layer_idx)
            if buf is None or buf.shape[1] != k:
                buf = torch.empty((query_states.shape[0], k), dtype=torch.int32, device=query_states.device)
                self._idx[layer_idx] = buf  # the sparse layers keep reading this very buffer
            out, _, _ = ops.dense_attn(query_states, st.k, st.v, seq_len=st.capacity, seq_lens=self._len32,
                                       selector=selector_cls, score_len=consider_len, scale=scale, select_k=k,
                                       idx_out=buf)
            self._sel_gen[layer_idx] = self._sel_gen.get(layer_idx, 0) + 1  # same buffer, new selection
            if self.real_offload:
                self._stage_static(layer_idx, buf)
            return out, buf
        kview, vview = self._store[layer_idx].views()
        out, _, idx = ops.dense_attn(query_states, kview, vview, selector=selector_cls, score_len=consider_len,
                                     scale=scale, select_k=k)
        self.set_idx_on_gpu(idx, layer_idx)
        return out, idx


def _gather_wide(src: torch.Tensor, idx32: torch.Tensor, dst: torch.Tensor) -> None:
    """Row gather with one 'head' as wide as the whole interleaved K|V row."""
    import ctypes as C

    from ._lib import KVLayout

    width = src.shape[-1]
    if width % 128:
        raise ValueError("row width must be a multiple of 128 elements")
    # present each row as (width/128) heads of 128 elements
    heads = width // 128
    lay = KVLayout(ops._DTYPES[src.dtype], heads, heads, 128, src.stride(2), 128, 0, None, 0, 0, 0)
    check(lib().okv_gather_rows(src.data_ptr(), C.byref(lay), idx32.data_ptr(), idx32.stride(0), None,
                                idx32.shape[1], 1, dst.data_ptr(), dst.stride(2), 128, 0,
                                torch.cuda.current_stream(idx32.device).cuda_stream))


class WOPackCache(OmniKVMultiStageCache):
    """`cache_cls: without_pack` (modeling/spec_cache.py:388-520): set_idx_on_gpu only
    records the selection; with real_offload each sparse layer fetches its own rows
    when it runs (spec_cache.py:477-483) instead of all layers of the group being staged
    ahead at selection time.  Without offload there is nothing to pack in this build
    (the sparse kernel reads the rows in place), so the two classes then coincide."""

    _stage_at_selection = False

    @staticmethod
    def from_dynamic_cache(cache, full_attn_layers: List, num_hidden_layers, num_wait_load_layers=2,
                           real_offload=True, **kwargs):
        return OmniKVMultiStageCache.from_dynamic_cache(cache, full_attn_layers, num_hidden_layers,
                                                        num_wait_load_layers, real_offload, _cls=WOPackCache, **kwargs)


def get_idx_iou_score(new_idx: torch.Tensor, old_idx: torch.Tensor) -> float:
    """Overlap of two 1-D index tensors as the reference scores it
    (modeling/spec_cache.py:10-32): |new & old| / |new| -- despite its name not divided by
    the union.  Synchronises with the device, as the reference's Python float does."""
    assert new_idx.dim() == 1 and old_idx.dim() == 1, "Both tensors should be 1D"
    un = torch.cat([new_idx, old_idx], dim=0).unique().shape[0]
    inter = new_idx.shape[0] + old_idx.shape[0] - un
    return inter / new_idx.shape[0]


class OmniKVLazyCache(OmniKVMultiStageCache):
    """`cache_cls: lazy` (modeling/spec_cache.py:523-557): the multi-stage cache that keeps the rows it has
    staged when a new selection overlaps the one in use by more than `skip_threshold` of its indices
    (OmniKVLazyCache.set_out_idx; the reference's default threshold is 0.4 of `get_idx_iou_score`).  The
    reference pairs it with a model class of its own that feeds it one selection per step; here it is the
    `multi` cache with that threshold switched on, behind the same interface."""

    DEFAULT_SKIP_THRESHOLD = 0.4

    def __init__(self, full_attn_layers: List, num_hidden_layers, num_wait_load_layers=2, real_offload=True,
                 **kwargs):
        if kwargs.get("skip_threshold") is None:
            kwargs["skip_threshold"] = self.DEFAULT_SKIP_THRESHOLD
        super().__init__(full_attn_layers, num_hidden_layers, num_wait_load_layers, real_offload, **kwargs)

    @staticmethod
    def from_dynamic_cache(cache, full_attn_layers: List, num_hidden_layers, num_wait_load_layers=2,
                           real_offload=True, **kwargs):
        return OmniKVMultiStageCache.from_dynamic_cache(cache, full_attn_layers, num_hidden_layers,
                                                        num_wait_load_layers, real_offload, _cls=OmniKVLazyCache, **kwargs)


def get_cache_cls(config):
    """modeling/spec_cache.py:829-837.  `lazy` is the multi-stage cache with re-selection skipping on;
    `default` (the baseline without selection) and `eff` (broken upstream) belong to other model paths."""
    name2cls = {"multi": OmniKVMultiStageCache, "without_pack": WOPackCache, "lazy": OmniKVLazyCache}
    name = config.get("cache_cls", "default")
    if name not in name2cls:
        raise NotImplementedError(f"cache_cls={name!r}: 'multi', 'without_pack' and 'lazy' are built here")
    return name2cls[name]
