"""Measures the decode schedules over a grid of batch shapes and scores the host rule that
chooses between them (``ops.decode_schedule``).

    python -m llama_lite_npu_amd.tune_decode_schedule [--heads HQ HKV] [--kv-dtype f16|fp8] [--quick]

Per shape: microseconds per layer of the balanced schedule (fused step + merge) and of the
per-sequence schedule with the append fused in, at one wavefront per sequence and kv head (one
launch) and at 4, 8 and 16 splits per sequence (+ merge launch), each recorded 16 times into a HIP
graph and replayed, minimum of 3 replays; then what the rule picks. Shapes: equal lengths, ragged
U[len/4, len], and one long sequence among short ones. The last line gives the rule's mean and
worst time relative to always picking the fastest schedule. The rule's constants are fits to this
table on an MI355X; on other parts, refit them from it.
"""

from __future__ import annotations

import argparse

import torch

from . import ops, workloads
from .executor.decode_graph import quiet_capture

DEV = "cuda:0"


def _replayed_us(fn, inner: int = 16, reps: int = 5) -> float:
    fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        fn()
        torch.cuda.synchronize()
        with quiet_capture(graph, stream=side):
            for _ in range(inner):
                fn()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(reps):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        graph.replay()
        stop.record()
        torch.cuda.synchronize()
        best = min(best, start.elapsed_time(stop) * 1e3 / inner)
    return best


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--heads", type=int, nargs=2, default=(64, 8), metavar=("HQ", "HKV"))
    ap.add_argument("--quick", action="store_true", help="a dozen shapes instead of the whole grid")
    ap.add_argument("--kv-dtype", default="f16", choices=["f16", "fp8"], help="storage of the KV pool")
    args = ap.parse_args()
    hq, hkv = args.heads
    fp8 = args.kv_dtype == "fp8"
    batches = (2, 16, 128) if args.quick else (1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048)
    lengths = (64, 512, 4096) if args.quick else (32, 64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384)
    token_bytes = 2 * hkv * 128 * (1 if fp8 else 2)
    scales = torch.full((2 * hkv,), 0.02, dtype=torch.float32, device=DEV) if fp8 else None
    schedules = (0, 1) + ops.SPLIT_COUNTS
    print(f"heads {hq}/{hkv}, {args.kv_dtype} pool; us per layer: balanced, then per-sequence in "
          f"{', '.join(map(str, schedules[1:]))} splits", flush=True)
    ratio_rule, ratio_balanced, worst, shapes = 0.0, 0.0, 0.0, 0
    for b in batches:
        for hi in lengths:
            for kind in ("equal", "ragged", "one long"):
                if b * hi > 600_000 or (b == 1 and kind != "equal"):
                    continue
                if kind == "equal":
                    lens = [hi] * b
                elif kind == "ragged":
                    lens = workloads.uniform_lens(b + hi, b, max(1, hi // 4), hi)
                else:
                    lens = [hi] + [max(1, hi // 16)] * (b - 1)
                case = workloads.make_decode_case("tune", 5, lens, hq, hkv, device=DEV)
                plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages)
                out = torch.empty_like(case.q)
                pool = case.kv_pool
                if fp8:  # the same values as codes
                    pool = torch.empty(case.kv_pool.shape, dtype=torch.uint8, device=DEV)
                    every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
                    ops.kv_append_fp8(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every_slot, pool, scales)
                pages = [(n + 1 + 15) // 16 for n in lens]
                times = {}
                for n in schedules:
                    if n > 1 and b * n * hkv > 4096:
                        continue                                  # far outside what the rule considers
                    plan.set_schedule(n)
                    times[n] = _replayed_us(lambda: ops.decode_step(case.q, pool, plan, case.k_new, case.v_new,
                                                                    case.softmax_scale, out=out, kv_scales=scales),
                                            reps=3)
                pick = ops.decode_schedule(b, hkv, max(pages), sum(pages), token_bytes, heads_per_kv_head=hq // hkv)
                best = min(times.values())
                ratio_rule += times[pick] / best
                ratio_balanced += times[0] / best
                worst = max(worst, times[pick] / best)
                shapes += 1
                print(f"B {b:5d} {kind:8s} len {hi:6d}  tokens {sum(lens):7d}  "
                      + "  ".join(f"{n}: {t:7.1f}" for n, t in times.items())
                      + f"  rule picks {pick} ({times[pick] / best:.2f} x the fastest)", flush=True)
                del case, plan, pool
        torch.cuda.empty_cache()
    print(f"{shapes} shapes: rule / fastest = {ratio_rule / shapes:.3f} on average, {worst:.2f} at worst; "
          f"always balanced / fastest = {ratio_balanced / shapes:.3f}", flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
