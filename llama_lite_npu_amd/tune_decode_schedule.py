"""Measures both decode schedules over a grid of batch shapes and scores the host rule that
chooses between them (``ops.per_sequence_decode_is_faster``).

    python -m llama_lite_npu_amd.tune_decode_schedule [--heads HQ HKV] [--kv-dtype f16|fp8] [--quick]

Per shape: microseconds per layer of the balanced schedule (fused step + merge) and of the
per-sequence schedule (one wavefront per sequence and kv head, append fused in), each recorded 16
times into a HIP graph and replayed, minimum of 5 replays; then what the rule picks. The last line
gives the rule's mean and worst time relative to always picking the faster schedule. The rule's
constants are fits to this table on an MI355X; on other parts, refit them from it.
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
    batches = (8, 64, 512) if args.quick else (8, 16, 32, 64, 128, 256, 512, 1024, 2048)
    lengths = (32, 256, 2048) if args.quick else (32, 64, 128, 256, 512, 1024, 2048, 4096)
    token_bytes = 2 * hkv * 128 * (1 if fp8 else 2)
    scales = torch.full((2 * hkv,), 0.02, dtype=torch.float32, device=DEV) if fp8 else None
    print(f"heads {hq}/{hkv}, {args.kv_dtype} pool; us per layer", flush=True)
    ratio_rule, ratio_balanced, worst, shapes = 0.0, 0.0, 0.0, 0
    for b in batches:
        for hi in lengths:
            for ragged in (False, True):
                if b * hi > 600_000:
                    continue
                lens = workloads.uniform_lens(b + hi, b, max(1, hi // 4), hi) if ragged else [hi] * b
                case = workloads.make_decode_case("tune", 5, lens, hq, hkv, device=DEV)
                plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages)
                out = torch.empty_like(case.q)
                pool = case.kv_pool
                if fp8:  # the same values as codes
                    pool = torch.empty(case.kv_pool.shape, dtype=torch.uint8, device=DEV)
                    every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
                    ops.kv_append_fp8(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every_slot, pool, scales)
                t_bal = _replayed_us(lambda: ops.decode_step(case.q, pool, plan, case.k_new, case.v_new,
                                                             case.softmax_scale, out=out, kv_scales=scales))
                t_seq = _replayed_us(lambda: ops.paged_decode(case.q, pool, case.block_table, case.seq_lens,
                                                              case.softmax_scale, schedule="splits", num_splits=1,
                                                              out=out, kv_scales=scales, k_new=case.k_new,
                                                              v_new=case.v_new))
                pages = [(n + 1 + 15) // 16 for n in lens]
                pick_seq = ops.per_sequence_decode_is_faster(b, hkv, max(pages), sum(pages), token_bytes,
                                                             heads_per_kv_head=hq // hkv)
                picked, best = (t_seq if pick_seq else t_bal), min(t_seq, t_bal)
                ratio_rule += picked / best
                ratio_balanced += t_bal / best
                worst = max(worst, picked / best)
                shapes += 1
                name = f"U[{max(1, hi // 4)},{hi}]" if ragged else str(hi)
                print(f"B {b:5d} len {name:>12}  tokens {sum(lens):7d}  balanced {t_bal:7.1f}  per-sequence {t_seq:7.1f}"
                      f"  rule picks {'per-sequence' if pick_seq else 'balanced'}", flush=True)
                del case, plan, pool
        torch.cuda.empty_cache()
    print(f"{shapes} shapes: rule / best = {ratio_rule / shapes:.3f} on average, {worst:.2f} at worst; "
          f"always balanced / best = {ratio_balanced / shapes:.3f}", flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
