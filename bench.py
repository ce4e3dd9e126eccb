#!/usr/bin/env python3
"""Benchmark of the paged-KV attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--all]

Default workload (config c2): Qwen3-32B attention shape, decode. A step is one
pass over 64 layers' worth of independent KV pools: one step plan (the cut of
the batch's pages into equal chunks, shared by all layers), then per layer the
KV append of the batch's new tokens fused into paged flash-decoding, and the
merge of its partial results. All inputs are resident in HBM before the timed
region. One JSON line is printed on
stdout; `--all` adds one line per other configuration on stderr and in
`bench_all.jsonl` under `--out-dir`.

`value` is algorithmic bytes of the whole step divided by its wall-clock time.
`roofline` describes the dominant kernel (the decode kernel): algorithmic bytes
of one launch over its mean duration, taken from HIP events attached to every
one of its launches inside the timed region, on the stream the kernels run on. `cpu_baseline` times the PyTorch-CPU restatement of the
reference's own torch path (oracle/cpu_ref.py) on this machine's host cores for
one layer of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, published


METRIC = "paged decode attn HBM GB/s (% of 8 TB/s peak); KV-append GB/s; us/layer"
TRAFFIC_FILE = ROOT / "profiles" / "traffic.json"


def measured_traffic(config: str, schedule: str, kv_dtype: str):
    """HBM bytes per launch of a configuration's roofline kernel(s) as rocprofv3 counted them
    (FETCH_SIZE + WRITE_SIZE scaled by a copy of known size; profiles/traffic.json names the
    summary each figure comes from). A figure only describes the kernel source it was taken on:
    the file's SHA-256 at that time is stored with it, and a source that has changed since gives
    None. Returns (bytes or None, the stamp that is printed with the result)."""
    import hashlib

    try:
        entries = json.loads(TRAFFIC_FILE.read_text())["entries"]
    except (OSError, ValueError, KeyError):
        return None, None
    for e in entries:
        if (e["config"], e["schedule"], e["kv_dtype"]) != (config, schedule, kv_dtype):
            continue
        current = True
        for rel, digest in e["kernel_sources"].items():
            try:
                current &= hashlib.sha256((ROOT / rel).read_bytes()).hexdigest() == digest
            except OSError:
                current = False
        stamp = {"profile": e["profile"], "taken_at_commit": e["commit"], "kernel_sources_unchanged": current}
        return (float(e["bytes_per_launch"]) if current else None), stamp
    return None, None


def _median(xs):
    xs = sorted(xs)
    n = len(xs)
    return xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])


class HipEvents:
    """HIP events created through the runtime PyTorch already loaded; they are attached to the decode
    kernel's own dispatch (litekv_profile_next_decode), so they time the kernel on its stream without
    adding packets between launches."""

    def __init__(self):
        import ctypes
        import torch

        self.ct = ctypes
        self.hip = ctypes.CDLL(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def create(self):
        e = self.ct.c_void_p()
        rc = self.hip.hipEventCreate(self.ct.byref(e))
        if rc != 0:
            raise RuntimeError(f"hipEventCreate failed: {rc}")
        return e

    def elapsed_ms(self, a, b) -> float:
        ms = self.ct.c_float()
        rc = self.hip.hipEventElapsedTime(self.ct.byref(ms), a, b)
        if rc != 0:
            raise RuntimeError(f"hipEventElapsedTime failed: {rc}")
        return ms.value

    def destroy(self, e) -> None:
        self.hip.hipEventDestroy(e)


class DecodeLayerSet:
    """`layers` independent KV pools sharing one batch's block tables, with pre-bound launches.

    A step = one plan launch (the cuts are shared by every layer of a decode step) + per layer one
    balanced decode call with the KV append fused in (decode kernel + merge kernel)."""

    def __init__(self, case, layers: int, device: str, schedule: str = "balanced", shared_pages: int = 0,
                 kv_dtype: str = "f16", splits: int = 1):
        import torch
        from llama_lite_npu_amd import _lib, ops

        self.torch = torch
        self.case = case
        self.layers = layers
        self.schedule = schedule
        lib = _lib.load()
        self.lib = lib
        c = case
        b, hq, hkv = c.batch, c.num_q_heads, c.num_kv_heads
        slots = c.num_pages * 16
        gen = torch.Generator(device=device).manual_seed(4242)
        self.fp8 = kv_dtype in ("fp8", "int8")       # 8-bit codes with one scale per head
        self.q8 = kv_dtype
        if self.fp8:
            if schedule == "splits":
                raise ValueError("8-bit pools are read with the append fused in in this benchmark")
            # E4M3 codes (no NaN codes) or int8 codes (no -128), and one scale per head
            if kv_dtype == "fp8":
                pools = torch.randint(0, 0x7F, (layers, slots, 2 * hkv, 128), generator=gen, device=device,
                                      dtype=torch.uint8)
            else:
                pools = torch.randint(-127, 128, (layers, slots, 2 * hkv, 128), generator=gen, device=device,
                                      dtype=torch.int8)
            self.scales = torch.full((2 * hkv,), 0.02, dtype=torch.float32, device=device)
        else:
            pools = torch.empty((layers, slots, 2 * hkv, 128), dtype=torch.float16, device=device)
            for l in range(layers):
                pools[l].normal_(generator=gen)
        self.pools = pools
        self.q = c.q
        self.out = torch.empty((layers, b, hq, 128), dtype=torch.float16, device=device)
        self.table = c.block_table.contiguous()
        self.seq_lens = c.seq_lens.contiguous()
        self.slot_mapping = c.slot_mapping.contiguous()
        stream = torch.cuda.current_stream().cuda_stream
        self.stream = stream
        bts = self.table.stride(0)
        if schedule == "balanced":
            self.shared_pages = shared_pages
            self.chunks = c.extra.get("chunks") or (
                lib.litekv_paged_decode_prefix_chunks(b, hq, hkv, 128, 16, shared_pages, 1 if kv_dtype == "f16" else 0)
                if shared_pages > 0 else lib.litekv_paged_decode_balanced_chunks(hkv))
            self.plan_bytes = lib.litekv_decode_plan_bytes(b, bts, hkv, self.chunks)
            self.plan = torch.empty(self.plan_bytes // 4, dtype=torch.int32, device=device)
            ws_bytes = lib.litekv_paged_decode_prefix_workspace_bytes(b, hq, 128, self.chunks)
            self.ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=device)
            # per-step metadata on the device: the batch's rows are gathered from the request tables
            # (here request i is batch row i) and slots / positions recomputed; increment 0 keeps the
            # workload's lengths fixed from step to step
            self.req_ids = torch.arange(b, dtype=torch.int32, device=device)
            self.batch_table = torch.zeros_like(self.table)
            self.slot_out = torch.empty(b, dtype=torch.int32, device=device)
            self.pos_out = torch.empty(b, dtype=torch.int64, device=device)
            self.advance_args = (self.table.data_ptr(), bts, b, self.req_ids.data_ptr(), None,
                                 self.seq_lens.data_ptr(), None, self.slot_out.data_ptr(), self.pos_out.data_ptr(),
                                 self.batch_table.data_ptr(), bts, self.table.shape[1], None, b, 16, c.num_pages,
                                 0, stream)
            self.plan_args = (self.batch_table.data_ptr(), bts, self.seq_lens.data_ptr(), b, hkv, 16, c.num_pages,
                              self.chunks, shared_pages, self.plan.data_ptr(), self.plan_bytes, stream)
            self.decode_args = [
                (self.q.data_ptr(), hq * 128, pools[l].data_ptr(), self.batch_table.data_ptr(), self.seq_lens.data_ptr(),
                 self.plan.data_ptr(), self.plan_bytes, c.k_new.data_ptr(), c.v_new.data_ptr(), hkv * 128,
                 hkv * 128, self.out[l].data_ptr(), self.ws.data_ptr(), ws_bytes, b, hq, hkv, 128, 16,
                 c.num_pages, bts, self.chunks, shared_pages, c.softmax_scale, stream)
                for l in range(layers)
            ]
            if self.fp8:
                self.decode_args = [
                    (self.q.data_ptr(), hq * 128, pools[l].data_ptr(), self.scales.data_ptr(),
                     self.batch_table.data_ptr(), self.seq_lens.data_ptr(), self.plan.data_ptr(), self.plan_bytes,
                     c.k_new.data_ptr(), c.v_new.data_ptr(), hkv * 128, hkv * 128, self.out[l].data_ptr(),
                     self.ws.data_ptr(), ws_bytes, b, hq, hkv, 128, 16, c.num_pages, bts, self.chunks,
                     shared_pages, c.softmax_scale, stream)
                    for l in range(layers)
                ]
            self.plan_info = {"schedule": "balanced", "chunks": self.chunks, "shared_pages": shared_pages,
                              "kv_dtype": kv_dtype}
        elif schedule == "per_sequence":
            # `splits` wavefronts per (sequence, kv head) with the append fused in, then (more than
            # one split) the merge launch; per-step metadata on the device as on the balanced schedule
            self.max_splits = int(splits)
            self.ws = ops.decode_workspace(b, hq, self.max_splits, device)
            ws_ptr = None if self.ws is None else self.ws.data_ptr()
            ws_bytes = 0 if self.ws is None else self.ws.numel() * 4
            self.req_ids = torch.arange(b, dtype=torch.int32, device=device)
            self.batch_table = torch.zeros_like(self.table)
            self.slot_out = torch.empty(b, dtype=torch.int32, device=device)
            self.pos_out = torch.empty(b, dtype=torch.int64, device=device)
            self.advance_args = (self.table.data_ptr(), bts, b, self.req_ids.data_ptr(), None,
                                 self.seq_lens.data_ptr(), None, self.slot_out.data_ptr(), self.pos_out.data_ptr(),
                                 self.batch_table.data_ptr(), bts, self.table.shape[1], None, b, 16, c.num_pages,
                                 0, stream)
            scales = (self.scales.data_ptr(),) if self.fp8 else ()
            self.decode_args = [
                (self.q.data_ptr(), hq * 128, pools[l].data_ptr(), *scales, self.batch_table.data_ptr(), bts,
                 self.seq_lens.data_ptr(), c.k_new.data_ptr(), c.v_new.data_ptr(), hkv * 128, hkv * 128,
                 self.out[l].data_ptr(), ws_ptr, ws_bytes, b, hq, hkv, 128, 16, c.num_pages, self.max_splits, 1,
                 c.softmax_scale, stream)
                for l in range(layers)
            ]
            self.plan_info = {"schedule": "per_sequence", "splits_per_sequence": self.max_splits,
                              "kv_dtype": kv_dtype}
        else:
            self.max_splits, self.min_pps = ops.decode_split_plan(b, hkv, self.table.shape[1], c.num_splits)
            self.ws = ops.decode_workspace(b, hq, self.max_splits, device)
            ws_ptr = None if self.ws is None else self.ws.data_ptr()
            ws_bytes = 0 if self.ws is None else self.ws.numel() * 4
            self.append_args, self.split_args, self.merge_args = [], [], []
            for l in range(layers):
                pool_ptr = pools[l].data_ptr()
                self.append_args.append((c.k_new.data_ptr(), c.v_new.data_ptr(), hkv * 128, hkv * 128,
                                         self.slot_mapping.data_ptr(), pool_ptr, b, hkv, 128, slots, stream))
                self.split_args.append((self.q.data_ptr(), hq * 128, pool_ptr, self.table.data_ptr(), bts,
                                        self.seq_lens.data_ptr(), self.out[l].data_ptr(), ws_ptr, ws_bytes, b, hq,
                                        hkv, 128, 16, c.num_pages, self.max_splits, self.min_pps,
                                        c.softmax_scale, stream))
                self.merge_args.append((self.seq_lens.data_ptr(), self.out[l].data_ptr(), ws_ptr, ws_bytes, b, hq,
                                        128, 16, self.max_splits, self.min_pps, stream))
            self.plan_info = {"schedule": "splits", "max_splits": self.max_splits,
                              "min_pages_per_split": self.min_pps}

    def step(self, events=None, stream=None):
        """One pass over all layers. `events[l]`: (start, stop) raw HIP events for layer l's decode kernel
        (balanced, per_sequence) or 3 torch events bracketing split and merge (splits). `stream`:
        launch there instead of the stream the set was built on (used under graph capture)."""
        lib = self.lib
        rc = 0
        if self.schedule == "balanced":
            on = (lambda a: a) if stream is None else (lambda a: a[:-1] + (stream,))
            rc |= lib.litekv_decode_advance(*on(self.advance_args))
            rc |= lib.litekv_decode_plan_prefix(*on(self.plan_args))
            dec = (getattr(lib, "litekv_paged_decode_prefix_" + self.q8) if self.fp8
                   else lib.litekv_paged_decode_prefix)
            prof = lib.litekv_profile_next_decode
            for l in range(self.layers):
                if events is not None:
                    prof(events[l][0], events[l][1])
                rc |= dec(*on(self.decode_args[l]))
        elif self.schedule == "per_sequence":
            on = (lambda a: a) if stream is None else (lambda a: a[:-1] + (stream,))
            rc |= lib.litekv_decode_advance(*on(self.advance_args))
            dec = (getattr(lib, "litekv_paged_decode_append_" + self.q8) if self.fp8
                   else lib.litekv_paged_decode_append)
            prof = lib.litekv_profile_next_decode
            for l in range(self.layers):
                if events is not None:
                    prof(events[l][0], events[l][1])
                rc |= dec(*on(self.decode_args[l]))
        else:
            ap, sp, mg = lib.litekv_kv_append, lib.litekv_paged_decode_split, lib.litekv_paged_decode_merge
            for l in range(self.layers):
                rc |= ap(*self.append_args[l])
                if events is not None:
                    e = events[l]
                    e[0].record()
                    rc |= sp(*self.split_args[l])
                    e[1].record()
                    rc |= mg(*self.merge_args[l])
                    e[2].record()
                else:
                    rc |= sp(*self.split_args[l])
                    rc |= mg(*self.merge_args[l])
        if rc:
            raise RuntimeError(f"liblitekv launch failed: {lib.litekv_last_error().decode()}")

    def capture(self):
        """The whole step (metadata, plan, every layer) recorded once as a HIP graph."""
        from llama_lite_npu_amd.executor.decode_graph import quiet_capture

        torch = self.torch
        graph = torch.cuda.CUDAGraph()
        with quiet_capture(graph):
            self.step(stream=torch.cuda.current_stream().cuda_stream)
        return graph


def run_decode(case, layers: int, steps: int, warmup: int, device: str, label: str,
               schedule: str = "balanced", shared_pages: int = 0, graph: bool = True,
               kv_dtype: str = "f16", splits: int = 1) -> dict:
    import torch

    ls = DecodeLayerSet(case, layers, device, schedule, shared_pages, kv_dtype, splits)
    for _ in range(max(1, warmup)):
        ls.step()
    torch.cuda.synchronize()
    balanced = schedule in ("balanced", "per_sequence")      # one fused call per layer, timed by its own events
    if balanced:
        hip = HipEvents()
        events = [[(hip.create(), hip.create()) for _ in range(layers)] for _ in range(steps)]
    else:
        events = [[[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(layers)]
                  for _ in range(steps)]
    # timed region: exactly `steps` steps, synchronised on both sides
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        ls.step(events[s])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_ms = []
    for s in range(steps):
        for l in range(layers):
            e = events[s][l]
            kernel_ms.append(hip.elapsed_ms(e[0], e[1]) if balanced else e[0].elapsed_time(e[1]))
    if balanced:
        for s in range(steps):
            for l in range(layers):
                hip.destroy(events[s][l][0])
                hip.destroy(events[s][l][1])
    ms_per_step = wall * 1e3 / steps
    decode_bytes = case.decode_bytes()
    append_bytes = case.append_bytes()
    if kv_dtype in ("fp8", "int8"):
        # one byte per cached element: K/V traffic halves; the appended rows arrive as fp16
        kv_read = int(case.seq_lens.sum()) * case.tok_bytes
        decode_bytes -= kv_read // 2
        append_bytes = case.batch * (case.tok_bytes + case.tok_bytes // 2 + 4)
    step_bytes = layers * (decode_bytes + append_bytes)
    replay = None
    if balanced and graph:
        # the same step replayed as one HIP graph (how the executor runs decode steps by default)
        g = ls.capture()
        for _ in range(max(1, warmup)):
            g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            g.replay()
        torch.cuda.synchronize()
        replay_ms = (time.perf_counter() - t0) * 1e3 / steps
        replay = {"ms_per_step": replay_ms, "us_per_layer": replay_ms * 1e3 / layers,
                  "value": step_bytes / (replay_ms * 1e-3) / 1e9}
    k_mean = sum(kernel_ms) / len(kernel_ms)
    # the fused kernel also moves the appended rows; they are part of its algorithmic bytes
    kernel_bytes = decode_bytes + (append_bytes if balanced else 0)
    achieved = kernel_bytes / (k_mean * 1e-3) / 1e9
    res = {
        "label": label,
        "ms_per_step": ms_per_step,
        "value": step_bytes / (ms_per_step * 1e-3) / 1e9,
        "us_per_layer": ms_per_step * 1e3 / layers,
        "decode_kernel_us_mean": k_mean * 1e3,
        "decode_kernel_us_median": _median(kernel_ms) * 1e3,
        "decode_kernel_us_min": min(kernel_ms) * 1e3,
        "decode_bytes_per_layer": decode_bytes,
        "append_bytes_per_layer": append_bytes,
        "layers": layers,
        "roofline": {
            "kernel": "paged_decode_balanced_kernel" if schedule == "balanced" else "paged_decode_split_kernel",
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": None,
        },
    }
    if shared_pages > 0:
        # two launches share the work (the two-role kernel that attends the shared pages and streams
        # the private ones, then the merge): the rate is taken over the layer's wall-clock share of
        # the step instead of one kernel's duration
        res["prefix_step_kernel_us_mean"] = k_mean * 1e3
        k_mean = ms_per_step / layers
        res["roofline"]["kernel"] = "prefix_step_kernel (shared-prefix role + balanced role) + merge"
        res["roofline"]["duration_us"] = k_mean * 1e3
    unique = case.unique_decode_bytes() + (append_bytes if balanced else 0)
    if kv_dtype in ("fp8", "int8"):
        unique -= (case.unique_decode_bytes() - (case.decode_bytes() - int(case.seq_lens.sum()) * case.tok_bytes)) // 2
    if unique < kernel_bytes:
        # Pages shared between block tables: the roofline fraction is taken on the bytes that must
        # come from HBM at least once; the logical rate (every reader counted) is kept beside it.
        res["roofline"].update(achieved=unique / (k_mean * 1e-3) / 1e9,
                               frac=unique / (k_mean * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                               logical_gbps=kernel_bytes / (k_mean * 1e-3) / 1e9, unique_bytes_per_launch=unique,
                               logical_bytes_per_launch=kernel_bytes)
    res.update(ls.plan_info)
    res["launch"] = "eager"
    if replay is not None:
        # Both ways of issuing the same step are timed; the reported step is the faster one (a graph
        # wins when launches are short against their issue cost, eager launches win for a step of one
        # long kernel, where a graph launch's fixed cost is not spread over many nodes).
        res["eager_launch"] = {"ms_per_step": res["ms_per_step"], "us_per_layer": res["us_per_layer"],
                               "value": res["value"]}
        res["graph_replay"] = replay
        if replay["ms_per_step"] < res["ms_per_step"]:
            res.update(replay)
            res["launch"] = "hipgraph replay"
            if shared_pages > 0:
                k = replay["ms_per_step"] / layers
                scale = res["roofline"]["duration_us"] / (k * 1e3)
                res["roofline"]["duration_us"] = k * 1e3
                for key in ("achieved", "frac", "logical_gbps"):
                    if key in res["roofline"]:
                        res["roofline"][key] *= scale
    return res


def _time_us(fn, reps: int = 10, warm: int = 2) -> float:
    """Mean device time of one `fn()` in microseconds: `reps` launches recorded back to back in one
    HIP graph and replayed between two events (an event pair around a single short launch measures
    mostly the events and the Python call, 10-15 us on this stack)."""
    import torch
    from llama_lite_npu_amd.executor.decode_graph import quiet_capture

    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with quiet_capture(graph):
        for _ in range(reps):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    graph.replay()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps * 1e3


def time_qk_epilogue(tokens: int, hq: int, hkv: int, slot_mapping, pool) -> dict:
    """The fused QK-norm + RoPE + append launch on `tokens` rows of the workload's head layout."""
    import torch
    from llama_lite_npu_amd import ops

    dev = pool.device
    g = torch.Generator(device=dev).manual_seed(99)
    q = torch.randn((tokens, hq, 128), generator=g, device=dev, dtype=torch.float16)
    k = torch.randn((tokens, hkv, 128), generator=g, device=dev, dtype=torch.float16)
    v = torch.randn((tokens, hkv, 128), generator=g, device=dev, dtype=torch.float16)
    w = torch.ones(128, device=dev, dtype=torch.float16)
    ang = torch.rand((tokens, 128), generator=g, device=dev) * 6.28
    cos, sin = ang.cos().half(), ang.sin().half()
    us = _time_us(lambda: ops.qk_norm_rope_append(q, k, v, slot_mapping, pool, w, w, cos, sin, 1e-6), reps=20)
    nbytes = tokens * ((2 * hq + 4 * hkv) * 256 + 2 * 128 + 4)
    return {"qk_epilogue_us": us, "qk_epilogue_gbps": nbytes / (us * 1e-6) / 1e9, "qk_epilogue_bytes": nbytes}


def cow_step(case) -> dict:
    """C4: the copy-on-write move before a step appends into a shared last page: every sequence's
    last page is copied into its spare page (page_copy, one launch)."""
    import torch
    from llama_lite_npu_amd import ops

    n_last = (case.seq_lens.cpu().to(torch.int64) - 1) // 16
    src = case.block_table.cpu().gather(1, n_last[:, None])[:, 0].to(torch.int32).to(case.kv_pool.device)
    dst = case.extra["spare_pages"].to(case.kv_pool.device)
    us = _time_us(lambda: ops.page_copy(case.kv_pool, src, dst))
    nbytes = 2 * src.numel() * case.tok_bytes * 16 + 8 * src.numel()
    return {"cow_pages": int(src.numel()), "cow_us": us, "cow_gbps": nbytes / (us * 1e-6) / 1e9}


def compaction_step(case) -> dict:
    """C5: out-of-place compaction. Every live page is gathered into the dense prefix of a second
    pool, the block table is rewritten, and the decode result must not change by a bit."""
    import torch
    from llama_lite_npu_amd import ops

    dev = case.kv_pool.device
    lens = case.seq_lens.cpu().to(torch.int64)
    n_pages = ((lens + 15) // 16).tolist()
    table = case.block_table.cpu()
    live = torch.cat([table[b, :n] for b, n in enumerate(n_pages)])
    new_table = torch.zeros_like(table)
    cur = 0
    for b, n in enumerate(n_pages):
        new_table[b, :n] = torch.arange(cur, cur + n, dtype=torch.int32)
        cur += n
    dense = torch.empty((cur * 16,) + tuple(case.kv_pool.shape[1:]), dtype=case.kv_pool.dtype, device=dev)
    src = live.to(torch.int32).to(dev)
    us = _time_us(lambda: ops.page_gather(case.kv_pool, dense, src, None), reps=5, warm=1)
    nbytes = 2 * cur * case.tok_bytes * 16 + 4 * cur
    before = ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale)
    after = ops.paged_decode(case.q, dense, new_table.to(dev), case.seq_lens, case.softmax_scale)
    again = ops.paged_decode(case.q, dense, new_table.to(dev), case.seq_lens, case.softmax_scale)
    torch.cuda.synchronize()
    return {"gather_pages": cur, "gather_us": us, "gather_gbps": nbytes / (us * 1e-6) / 1e9,
            "decode_same_bits_after_compaction": bool(torch.equal(before, after)),
            "decode_repeat_same_bits": bool(torch.equal(after, again))}


def _host_threads() -> int:
    """Threads for the CPU baseline: what the environment grants (OMP_NUM_THREADS), else the
    visible cores, never more than 16 (one GPU's share of a host)."""
    try:
        granted = int(os.environ.get("OMP_NUM_THREADS", "0"))
    except ValueError:
        granted = 0
    return max(1, min(granted if granted > 0 else (os.cpu_count() or 1), 16))


def _cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline_prefill(case, budget_s: float = 10.0) -> dict:
    """Per-sequence causal attention of the whole C3 workload in torch on the host cores
    (restates flashattention2_nopad.py:250-274), min over repetitions for about `budget_s` s."""
    import torch
    from oracle import cpu_ref

    cores = _host_threads()
    torch.set_num_threads(cores)
    c = case.to("cpu")
    starts = c.cu_q_lens[:-1]

    def one():
        t0 = time.perf_counter()
        cpu_ref.varlen_prefill_ref(c.q, c.k, c.v, starts, c.seq_lens, c.softmax_scale)
        return time.perf_counter() - t0

    first = one()
    times, used = [], first
    for _ in range(64):
        if used > budget_s:
            break
        dt = one()
        times.append(dt)
        used += dt
    best = min(times) if times else first
    return {"value": case.flops() / best / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "cpu_model": _cpu_model(),
            "sample": f"the whole workload ({case.flops() / 1e12:.3f} TFLOP causal), torch CPU restatement, "
                      f"min of {max(1, len(times))} reps after 1 warm-up, {best:.3f} s"}


def time_append(case_tokens_k, case_tokens_v, slot_mapping, pool, reps: int = 20) -> float:
    """Mean microseconds of one KV-append launch."""
    from llama_lite_npu_amd import ops

    return _time_us(lambda: ops.kv_append(case_tokens_k, case_tokens_v, slot_mapping, pool), reps=reps, warm=3)


def run_prefill(case, steps: int, warmup: int, device: str, label: str) -> dict:
    import torch
    from llama_lite_npu_amd import ops

    out = torch.empty_like(case.q)
    max_q_len = case.max_q_len  # one host read, outside the timed steps

    def step(ev=None):
        ops.kv_append(case.k, case.v, case.slot_mapping, case.kv_pool)
        if ev is not None:
            ev[0].record()
        ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, None, max_q_len,
                          case.softmax_scale, out=out)
        if ev is not None:
            ev[1].record()

    for _ in range(max(1, warmup)):
        step()
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for s in range(steps):
        step(events[s])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = [a.elapsed_time(b) for a, b in events]
    mean_ms = sum(ms) / len(ms)
    flops = case.flops()
    tokens = int(case.seq_lens.sum())
    append_us = time_append(case.k, case.v, case.slot_mapping, case.kv_pool)
    append_bytes = tokens * (2 * 2 * case.num_kv_heads * 128 * 2 + 4)
    achieved = flops / (mean_ms * 1e-3) / 1e12
    return {
        "label": label,
        "ms_per_step": wall * 1e3 / steps,
        "prefill_us_mean": mean_ms * 1e3,
        "prefill_tflops": achieved,
        "prefill_min_bytes_gbps": case.min_bytes() / (mean_ms * 1e-3) / 1e9,
        "append_us": append_us,
        "append_gbps": append_bytes / (append_us * 1e-6) / 1e9,
        "tokens": tokens,
        "flops": flops,
        "roofline": {
            "kernel": "varlen_prefill_tiled_kernel<paged>",
            "bound": "mfma",
            "achieved": achieved,
            "peak": MFMA_FP16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / MFMA_FP16_PEAK_TFLOPS,
            "traffic": None,
        },
    }


def time_chunk_prefill(device: str, rows: int = 128, history: int = 32768, hq: int = 64, hkv: int = 8) -> dict:
    """One request's prefill chunk (the reference's chunked prefill) of `rows` tokens over `history`
    cached tokens: too few query rows to fill the device, so the library also cuts the launch along
    the keys (ops.paged_prefill, key_slices chosen by the library) -- timed beside the same launch
    with the cut switched off. Median of 20 launches each, torch events around each launch."""
    import torch
    from llama_lite_npu_amd import _lib, ops

    g = torch.Generator(device=device).manual_seed(77)
    pages = (history + rows + 15) // 16
    pool = torch.empty((pages * 16, 2 * hkv, 128), dtype=torch.float16, device=device).normal_(generator=g)
    q = torch.empty((rows, hq, 128), dtype=torch.float16, device=device).normal_(generator=g)
    table = torch.randperm(pages, generator=g, device=device).to(torch.int32).reshape(1, pages)
    cu = torch.tensor([0, rows], dtype=torch.int32, device=device)
    ctx = torch.tensor([history], dtype=torch.int32, device=device)
    out = torch.empty_like(q)
    slices = int(_lib.load().litekv_paged_prefill_key_slices(1, hq, hkv, 128, rows, history + rows))
    ws = torch.empty(max(4, ops.paged_prefill_workspace_floats(rows, hq, 128, max(slices, 1))), dtype=torch.float32,
                     device=device)

    def timed(key_slices):
        run = lambda: ops.paged_prefill(q, pool, table, cu, ctx, rows, None, out=out, key_slices=key_slices,
                                        workspace=ws if key_slices > 1 else None)
        for _ in range(3):
            run()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(20)]
        for a, b in evs:
            a.record()
            run()
            b.record()
        torch.cuda.synchronize()
        return _median([a.elapsed_time(b) for a, b in evs]) * 1e3

    flops = 4.0 * hq * 128 * rows * (history + (rows + 1) / 2.0)
    plain, cut = timed(1), timed(slices)
    return {"chunk_prefill": {"rows": rows, "history_tokens": history, "key_slices": slices,
                              "us_uncut": plain, "us": cut, "tflops": flops / (cut * 1e-6) / 1e12,
                              "tflops_uncut": flops / (plain * 1e-6) / 1e12}}


def cpu_baseline_decode(case, budget_s: float = 10.0, max_sequences=None, kv_dtype: str = "f16") -> dict:
    """The reference's torch CPU path (append + gathered fp32 attention) for ONE layer of `case`,
    on the host cores: 1 warm-up, then repetitions for about `budget_s` seconds, min taken.
    `max_sequences`: time only the first that many sequences and scale the rate as measured (the
    result is then flagged as extrapolated; the pool stays on the GPU side, only those sequences'
    pages are brought to the host). `kv_dtype` fp8 / int8: the pool holds 8-bit codes, the CPU
    path quantises the appended rows, decodes the pool's codes (oracle/fp8.py, oracle/int8.py) and
    attends the decoded values; the rate is over the 8-bit algorithmic bytes."""
    import numpy as np
    import torch
    from oracle import cpu_ref, fp8 as fp8_codec, int8 as int8_codec

    cores = _host_threads()
    torch.set_num_threads(cores)
    extrapolated = max_sequences is not None and max_sequences < case.batch
    if extrapolated:
        c = _first_sequences(case, int(max_sequences))
    else:
        c = case.to("cpu")
    kv = torch.cat([c.k_new, c.v_new], dim=1)
    pool = c.kv_pool
    q8 = kv_dtype in ("fp8", "int8")
    if q8:
        codec = fp8_codec if kv_dtype == "fp8" else int8_codec
        scales = np.full(2 * c.num_kv_heads, 0.02, dtype=np.float32)
        rng = np.random.default_rng(4242)     # random codes, as the GPU leg's pools hold (no NaN codes, no -128)
        if kv_dtype == "fp8":
            codes = rng.integers(0, 0x7F, size=tuple(pool.shape), dtype=np.uint8)
        else:
            codes = rng.integers(-127, 128, size=tuple(pool.shape), dtype=np.int8)
        k_new, v_new, slots = c.k_new.numpy(), c.v_new.numpy(), c.slot_mapping.numpy()

    def one():
        t0 = time.perf_counter()
        if q8:
            codec.kv_append(k_new, v_new, slots, codes, scales)
            values = torch.from_numpy(codec.dequantize_pool(codes, scales))
            cpu_ref.paged_decode_ref(c.q, values, c.block_table, c.seq_lens, c.softmax_scale)
        else:
            cpu_ref.kv_append_ref(kv, c.slot_mapping, pool)
            cpu_ref.paged_decode_ref(c.q, pool, c.block_table, c.seq_lens, c.softmax_scale)
        return time.perf_counter() - t0

    first = one()
    times = []
    t_used = first
    for _ in range(64):
        if t_used > budget_s:
            break
        dt = one()
        times.append(dt)
        t_used += dt
    best = min(times) if times else first
    nbytes = c.decode_bytes() + c.append_bytes()
    whole = case.decode_bytes() + case.append_bytes()
    if q8:   # one byte per cached element (see run_decode)
        nbytes -= int(c.seq_lens.sum()) * c.tok_bytes // 2 + c.batch * c.tok_bytes // 2
        whole -= int(case.seq_lens.sum()) * case.tok_bytes // 2 + case.batch * case.tok_bytes // 2
    return {
        "value": nbytes / best / 1e9,
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "cpu_model": _cpu_model(),
        "sample": (f"the first {c.batch} of {case.batch} sequences of one layer (rate extrapolated to the "
                   f"whole layer), " if extrapolated else "1 of the layers of the same workload, ")
                  + (f"quantising append + decoding the {kv_dtype} pool + decode, " if q8 else "append + decode, ")
                  + f"{nbytes / 1e6:.1f} MB algorithmic, torch CPU restatement, "
                    f"min of {max(1, len(times))} reps after 1 warm-up, {best:.3f} s",
        "extrapolated": extrapolated,
        "seconds_per_layer": best * whole / nbytes,
    }


def _first_sequences(case, n: int):
    """The first n sequences of a decode case as a case of their own on the CPU: their pages are
    pulled out of the pool into a dense one (same bytes, new page ids)."""
    import torch
    from llama_lite_npu_amd import workloads

    lens = case.seq_lens[:n].cpu().to(torch.int64)
    n_pages = ((lens + 15) // 16).tolist()
    table = case.block_table[:n].cpu()
    live = torch.cat([table[b, :p] for b, p in enumerate(n_pages)]).to(torch.long)
    pool = case.kv_pool.view(case.num_pages, 16, *case.kv_pool.shape[1:])[live.to(case.kv_pool.device)].cpu()
    new_table = torch.zeros((n, max(n_pages)), dtype=torch.int32)
    cur = 0
    for b, p in enumerate(n_pages):
        new_table[b, :p] = torch.arange(cur, cur + p, dtype=torch.int32)
        cur += p
    ctx = case.context_lens[:n].cpu()
    slots = torch.tensor([int(new_table[b, int(ctx[b]) // 16]) * 16 + int(ctx[b]) % 16 for b in range(n)],
                         dtype=torch.int32)
    return workloads.DecodeCase(
        name=case.name, num_q_heads=case.num_q_heads, num_kv_heads=case.num_kv_heads, context_lens=ctx,
        seq_lens=case.seq_lens[:n].cpu(), block_table=new_table, slot_mapping=slots, num_pages=cur,
        q=case.q[:n].cpu(), k_new=case.k_new[:n].cpu(), v_new=case.v_new[:n].cpu(),
        kv_pool=pool.reshape(cur * 16, *case.kv_pool.shape[1:]), num_splits=case.num_splits)


CONFIGS = ("c1", "c2", "c3", "c4", "c5")


def measure(name: str, args, device: str, cpu_budget_s: float, schedule=None, kv_dtype=None,
            cpu: bool = True) -> dict:
    """One configuration measured in full: the step (value, ms_per_step), the roofline of its
    dominant kernel(s), the launches beside it, and the CPU baseline, in the schema of the
    headline line."""
    import torch
    from llama_lite_npu_amd import workloads

    schedule = schedule or args.schedule
    steps = args.steps if args.steps is not None else (30 if name == "c3" else 10)
    warmup = args.warmup if args.warmup is not None else (10 if name == "c3" else 3)
    if name == "c3":
        case = workloads.config_c3(device)
        res = run_prefill(case, steps, warmup, device, case.name)
        kv_dtype = "f16"
    else:
        layers = args.layers or {"c1": 64, "c2": 64, "c4": 16, "c5": 1}[name]
        case = {"c1": workloads.config_c1, "c2": workloads.config_c2, "c4": workloads.config_c4,
                "c5": workloads.config_c5}[name](device)
        if args.chunks:
            case.extra["chunks"] = args.chunks
        shared = 0
        if schedule in ("auto", "balanced") and not args.no_shared_prefix and not case.extra.get("private_prefix"):
            shared = int(case.extra.get("n_shared", 0))
        kv_dtype = (kv_dtype or args.kv_dtype) if schedule != "splits" else "f16"
        splits = args.splits
        if schedule == "auto":
            # what the library's host rule picks for this step from the lengths the host knows
            # (ops.DecodePlan.choose_schedule): balanced, or so many splits per sequence
            from llama_lite_npu_amd import ops

            pages = [(int(n) + 15) // 16 for n in case.seq_lens.tolist() if n > 0]
            splits = 0 if shared > 0 or args.chunks else ops.decode_schedule(
                case.batch, case.num_kv_heads, max(pages), sum(pages),
                case.tok_bytes // (1 if kv_dtype == "f16" else 2), heads_per_kv_head=case.num_q_heads // case.num_kv_heads)
            schedule = "per_sequence" if splits > 0 else "balanced"
        res = run_decode(case, layers, steps, warmup, device, case.name, schedule, shared,
                         graph=not args.no_graph, kv_dtype=kv_dtype, splits=splits)
    traffic, stamp = measured_traffic(name, None if name == "c3" else schedule, kv_dtype)
    res["roofline"]["traffic_source"] = stamp
    if traffic is not None and (name != "c4" or not args.no_shared_prefix):
        if name == "c3":
            duration_us, algorithmic = res["prefill_us_mean"], case.min_bytes()
        else:
            duration_us = res["roofline"].get("duration_us", res["decode_kernel_us_mean"])
            algorithmic = res["roofline"].get("unique_bytes_per_launch",
                                              res["decode_bytes_per_layer"] + res["append_bytes_per_layer"])
        res["roofline"]["traffic"] = traffic / (duration_us * 1e-6) / 1e9
        res["roofline"]["traffic_bytes_per_launch"] = traffic
        res["roofline"]["algorithmic_bytes_per_launch"] = algorithmic
    row = {
        "value": res.get("value", res.get("prefill_tflops")),
        "unit": "GB/s" if "value" in res else "TFLOP/s",
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": res["ms_per_step"],
        "dtype": "f16",
        "config": {"workload": res["label"], "config": name, "launch": res.get("launch", "eager"),
                   "kv_dtype": kv_dtype, "schedule": schedule if name != "c3" else None},
        "roofline": res["roofline"],
        "detail": {k: v for k, v in res.items() if k not in ("roofline", "label", "value", "ms_per_step", "launch")},
    }
    if name != "c3":
        row["config"].update(batch=case.batch, num_q_heads=case.num_q_heads, num_kv_heads=case.num_kv_heads,
                             head_dim=128, page_size=16, layers=res["layers"],
                             tokens_attended=int(case.seq_lens.sum()))
        row["pct_of_hbm_peak"] = 100.0 * res["roofline"]["frac"]
        ap_us = time_append(case.k_new, case.v_new, case.slot_mapping, case.kv_pool)
        row["detail"]["append_us"] = ap_us
        row["detail"]["append_gbps"] = case.append_bytes() / (ap_us * 1e-6) / 1e9
        row["detail"].update(time_qk_epilogue(case.batch, case.num_q_heads, case.num_kv_heads,
                                              case.slot_mapping, case.kv_pool))
        if name == "c4":
            row["detail"].update(cow_step(case))
        if name == "c5" and schedule == "balanced":
            row["detail"].update(compaction_step(case))
        if cpu and not args.no_cpu_baseline:
            row["cpu_baseline"] = cpu_baseline_decode(case, cpu_budget_s, max_sequences=8 if name == "c5" else None,
                                                      kv_dtype=kv_dtype)
    else:
        row["pct_of_mfma_peak"] = 100.0 * res["roofline"]["frac"]
        row["detail"].update(time_qk_epilogue(int(case.seq_lens.sum()), case.num_q_heads, case.num_kv_heads,
                                              case.slot_mapping, case.kv_pool))
        if not args.no_chunk_prefill:
            row["detail"].update(time_chunk_prefill(device))
        if not args.no_cpu_baseline:
            row["cpu_baseline"] = cpu_baseline_prefill(case, cpu_budget_s)
    del case
    torch.cuda.empty_cache()
    return row


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 10; 30 for c3)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps first (default 3; 10 for c3)")
    ap.add_argument("--config", default="c2", choices=list(CONFIGS))
    ap.add_argument("--layers", type=int, default=None, help="independent KV pools per step (c2 default 64)")
    ap.add_argument("--only", action="store_true",
                    help="measure --config alone (default: the other configurations follow in detail.configs)")
    ap.add_argument("--all", action="store_true",
                    help="also write one line per configuration, same schema, to bench_all.jsonl under --out-dir")
    ap.add_argument("--schedule", default="auto", choices=["auto", "balanced", "per_sequence", "splits"],
                    help="decode work decomposition (auto: what the library's host rule picks for the step; "
                         "per_sequence: --splits wavefronts per sequence and kv head with the append fused in; "
                         "splits: the workload's split count as separate append, split and merge launches)")
    ap.add_argument("--splits", type=int, default=1, help="splits per sequence of --schedule per_sequence")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--chunks", type=int, default=None,
                    help="balanced schedule: pieces per kv head (default: one workgroup per compute unit)")
    ap.add_argument("--no-shared-prefix", action="store_true",
                    help="c4: read the shared prefix pages once per sequence like any other page")
    ap.add_argument("--kv-dtype", default="f16", choices=["f16", "fp8", "int8"],
                    help="storage of the KV pools (fp8: E4M3 codes, int8: signed codes, both with per-head "
                         "scales; decode configs only)")
    ap.add_argument("--no-chunk-prefill", action="store_true",
                    help="c3: skip the chunk-over-a-long-history launches timed beside the workload (they run the "
                         "same kernel at another shape, which a per-kernel profile of the run would mix in)")
    ap.add_argument("--no-graph", action="store_true",
                    help="skip the leg that replays the decode step as one HIP graph")
    ap.add_argument("--out-dir", default="bench_out",
                    help="where --all writes bench_all.jsonl (relative to the repository root)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one page_gather of exactly 1 GiB (read) + 1 GiB (write): a plain copy of "
                         "known size against which profiler byte counters can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures the path on ONE GPU (one process, one device); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2

    import torch
    from llama_lite_npu_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the path has no CPU implementation", file=sys.stderr)
        return 2
    _lib.load()
    device = "cuda:0"
    torch.cuda.set_device(0)

    if args.calibrate_copy:
        from llama_lite_npu_amd import ops
        n_cal = 16384                                   # pages of 64 KiB = 1 GiB
        src = torch.empty((n_cal * 16, 16, 128), dtype=torch.float16, device=device).normal_()
        dst = torch.empty_like(src)
        ids = torch.randperm(n_cal, device=device).to(torch.int32)
        ops.page_gather(src, dst, ids, None)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    head = measure(args.config, args, device, cpu_budget_s=10.0)
    line = {
        "metric": METRIC,
        "value": head["value"],
        "unit": head["unit"],
        "n_gpus": 1,
        "steps": head["steps"],
        "warmup": head["warmup"],
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": head["config"],
        "roofline": head["roofline"],
        "detail": head["detail"],
    }
    for key in ("pct_of_hbm_peak", "pct_of_mfma_peak", "cpu_baseline"):
        if key in head:
            line[key] = head[key]
    rows = {args.config: head}
    if not args.only:
        # Every other configuration, each with its own roofline and CPU baseline (a few seconds of
        # host time each). C5 is reported on both schedules: the balanced cut (the default) and the
        # 16 per-sequence splits its description names.
        others = {}
        for name in CONFIGS:
            if name == args.config:
                continue
            others[name] = measure(name, args, device, cpu_budget_s=3.0)
            if name == "c5":
                others["c5_16_splits"] = measure("c5", args, device, cpu_budget_s=0.0, schedule="splits", cpu=False)
                if "cpu_baseline" in others["c5"]:   # the CPU path has one schedule: the same work, timed once
                    others["c5_16_splits"]["cpu_baseline"] = dict(others["c5"]["cpu_baseline"])
        if args.config == "c2" and args.kv_dtype == "f16":
            # the headline workload over pools of 8-bit codes (half the K/V bytes per token)
            for q8 in ("fp8", "int8"):
                others[f"c2_{q8}"] = measure("c2", args, device, cpu_budget_s=3.0, kv_dtype=q8)
        rows.update(others)
        line["detail"]["configs"] = others
    print(json.dumps(line), flush=True)

    if args.all:
        out_dir = ROOT / args.out_dir
        out_dir.mkdir(parents=True, exist_ok=True)
        with open(out_dir / "bench_all.jsonl", "w") as f:
            for name, row in rows.items():
                full = {"metric": METRIC, "n_gpus": 1, "higher_is_better": True, "scaling": "weak",
                        "vs_baseline": None, "data": "synthetic", **row}
                f.write(json.dumps(full) + "\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
