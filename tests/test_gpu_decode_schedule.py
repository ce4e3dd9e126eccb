"""GPU: the per-sequence decode schedule chosen by a plan from host-known lengths (append fused
into one wavefront per sequence and kv head) gives the same result as the balanced one (attention
tolerance against the oracle, pool bit for bit), for fp16 and fp8 pools, and across a change of
schedule under graph replay; the fused append of the splits schedule with several splits."""

import math
import random

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import ops, workloads
from oracle import c_oracle, cpu_ref, fp8
from tests.parity import assert_attention_close, to_np16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _plans(case, hq, hkv, lens, token_bytes=None):
    routed = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages,
                            host_seq_lens=[n + 1 for n in lens], token_bytes=token_bytes)
    balanced = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages)
    return routed, balanced


@pytest.mark.parametrize("hq,hkv", [(64, 8), (32, 4), (16, 2), (40, 8), (8, 1)])
def test_short_batches_take_the_per_sequence_schedule_with_the_same_result(hq, hkv):
    rng = random.Random(hq + hkv)
    lens = [rng.choice([0, rng.randint(1, 40), rng.randint(1, 120)]) for _ in range(48)]
    print(f"per-sequence schedule: heads {hq}/{hkv} lens {lens[:10]}...", flush=True)
    case = workloads.make_decode_case("sched", 31, lens, hq, hkv, device=DEV)
    routed, balanced = _plans(case, hq, hkv, lens)
    assert routed.per_sequence and not balanced.per_sequence
    pool_a, pool_b = case.kv_pool.clone(), case.kv_pool.clone()
    out_a = ops.decode_step(case.q, pool_a, routed, case.k_new, case.v_new, case.softmax_scale)
    out_b = ops.decode_step(case.q, pool_b, balanced, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(pool_a.view(torch.int16), pool_b.view(torch.int16))
    ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_a), case.block_table.cpu().numpy(),
                                case.seq_lens.cpu().numpy(), case.softmax_scale)
    assert_attention_close(out_a, ref, "per-sequence")
    assert_attention_close(out_b, ref, "balanced")
    # rows already stored (the fused epilogue did it): no append, same attention
    again = ops.decode_step(case.q, pool_a, routed, None, None, case.softmax_scale)
    assert torch.equal(again, out_a)


def test_long_sequences_and_shared_prefixes_stay_balanced():
    print("per-sequence schedule: cases that must not take it", flush=True)
    lens = [37, 128, 511, 12000]
    case = workloads.make_decode_case("sched", 32, lens, 16, 8, device=DEV)
    routed, _ = _plans(case, 16, 8, lens)
    assert not routed.per_sequence
    shared = workloads.config_c4(DEV, batch=8, prefix=256, lo=8, hi=40)
    plan = ops.DecodePlan(shared.block_table, shared.seq_lens, 64, 8, shared.num_pages, shared_pages=16,
                          host_seq_lens=shared.seq_lens.tolist())
    assert not plan.per_sequence


def test_fp8_pools_take_it_too():
    hq, hkv = 32, 8
    rng = random.Random(9)
    lens = [rng.randint(1, 120) for _ in range(64)]
    print("per-sequence schedule over an fp8 pool", flush=True)
    case = workloads.make_decode_case("sched", 34, lens, hq, hkv, device=DEV)
    scales = torch.cat([0.02 * (1 + 0.1 * torch.arange(hkv)), 0.015 * (1 + 0.2 * torch.arange(hkv))]).float().to(DEV)
    pool = torch.empty(case.kv_pool.shape, dtype=torch.uint8, device=DEV)
    every = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
    ops.kv_append_fp8(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every, pool, scales)
    routed, balanced = _plans(case, hq, hkv, lens, token_bytes=2 * hkv * 128)
    assert routed.per_sequence
    pool_a, pool_b = pool.clone(), pool.clone()
    out_a = ops.decode_step(case.q, pool_a, routed, case.k_new, case.v_new, case.softmax_scale, kv_scales=scales)
    out_b = ops.decode_step(case.q, pool_b, balanced, case.k_new, case.v_new, case.softmax_scale, kv_scales=scales)
    torch.cuda.synchronize()
    a, b = pool_a.cpu().numpy(), pool_b.cpu().numpy()
    assert int(((a != b) & ~(((a & 0x7F) == 0) & ((b & 0x7F) == 0))).sum()) == 0
    values = torch.from_numpy(fp8.dequantize_pool(a, scales.cpu().numpy()))
    ref = cpu_ref.paged_decode_ref(case.q.cpu(), values, case.block_table.cpu(), case.seq_lens.cpu(),
                                   case.softmax_scale).numpy()
    assert_attention_close(out_a, ref, "fp8 per-sequence")
    assert_attention_close(out_b, ref, "fp8 balanced")


def test_graph_replay_follows_a_change_of_schedule(monkeypatch):
    """A small batch starts with one wavefront per sequence, moves to several splits per sequence
    and then to the balanced schedule as it grows: the device batch follows, the runner captures
    one graph per schedule, and every step still matches an executor that builds its metadata on
    the host. (The thresholds are set by the test: the measured rule keeps four sequences off the
    balanced schedule up to thousands of tokens.)"""
    from tests.test_gpu_decode_graph import TinyModel, _executor, _host_step, _next_tokens, _prefill

    print("graph replay across changes of decode schedule", flush=True)

    def by_longest(batch, num_kv_heads, max_pages, total_pages, token_bytes, page_size=16, heads_per_kv_head=8,
                   current=None, hysteresis=1.0):
        return 1 if max_pages <= 8 else 8 if max_pages <= 12 else 0

    monkeypatch.setattr(ops, "decode_schedule", by_longest)
    host, graphed = _executor(num_pages=400, max_seq_len=512), _executor(num_pages=400, max_seq_len=512)
    model_h, model_g = TinyModel(), TinyModel()
    lens = [100, 20, 90, 5]
    ids_h, ids_g = _prefill(host, lens, 4), _prefill(graphed, lens, 4)
    graphed.attach_model(model_g, "qwen3")
    batch = graphed.activate_device_decode_batch(ids_g, reserve_tokens=32)
    assert batch.decode_plan.schedule == 1
    tok_h = tok_g = torch.tensor([[7], [8], [9], [10]], device=DEV)
    seen = []
    for step in range(160):
        out_h = _host_step(host, model_h, ids_h, tok_h)
        graphed.extend_paged_requests(ids_g)
        out_g = graphed.forward(tok_g)
        torch.cuda.synchronize()
        if batch.decode_plan.schedule not in seen:
            seen.append(batch.decode_plan.schedule)
        assert float((out_h - out_g).abs().max()) <= 3 * 2e-3, f"step {step}"     # three layers summed
        tok_h = tok_g = _next_tokens(out_h)
    assert seen == [1, 8, 0] and not batch.decode_plan.per_sequence
    assert graphed.graph_runner.capture_count == 3
    batch.check()


def test_small_batches_take_several_splits_per_sequence_with_the_same_result():
    """Where the host rule picks several splits per sequence (a few sequences of some hundred
    tokens), the step appends and attends like the balanced one: pool bit for bit, attention within
    the tolerance of the oracle; a plan keeps its partial-result buffer between steps."""
    for hq, hkv, lens in ((64, 8, [300, 1000, 37, 512]), (16, 8, [420, 16, 0, 500, 300]), (32, 4, [900])):
        print(f"several splits per sequence: heads {hq}/{hkv} lens {lens}", flush=True)
        case = workloads.make_decode_case("sched", 36, lens, hq, hkv, device=DEV)
        routed, balanced = _plans(case, hq, hkv, lens, token_bytes=2 * hkv * 128 * 2)
        assert routed.per_sequence and routed.splits in ops.SPLIT_COUNTS and routed.schedule == routed.splits
        assert routed.split_workspace is not None and balanced.schedule == 0
        pool_a, pool_b = case.kv_pool.clone(), case.kv_pool.clone()
        out_a = ops.decode_step(case.q, pool_a, routed, case.k_new, case.v_new, case.softmax_scale)
        out_b = ops.decode_step(case.q, pool_b, balanced, case.k_new, case.v_new, case.softmax_scale)
        torch.cuda.synchronize()
        assert torch.equal(pool_a.view(torch.int16), pool_b.view(torch.int16))
        ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_a), case.block_table.cpu().numpy(),
                                    case.seq_lens.cpu().numpy(), case.softmax_scale)
        assert_attention_close(out_a, ref, "several splits")
        assert_attention_close(out_b, ref, "balanced")
        held = routed.split_workspace.data_ptr()
        again = ops.decode_step(case.q, pool_a, routed, None, None, case.softmax_scale)
        assert torch.equal(again, out_a) and routed.split_workspace.data_ptr() == held
        # moving the plan to another split count (or back to balanced) needs no new plan
        routed.set_schedule(4)
        four = ops.decode_step(case.q, pool_a, routed, None, None, case.softmax_scale)
        routed.set_schedule(0)
        routed.refresh()
        cut = ops.decode_step(case.q, pool_a, routed, None, None, case.softmax_scale)
        torch.cuda.synchronize()
        assert_attention_close(four, ref, "four splits")
        assert_attention_close(cut, ref, "back to balanced")


@pytest.mark.parametrize("splits", [1, 2, 5, 16])
def test_append_fused_into_the_splits_schedule(splits):
    """litekv_paged_decode_append[_fp8]: pool = separate append bit for bit, attention = the oracle
    on that pool, whatever the number of splits (the last split's wavefront writes the token)."""
    rng = random.Random(40 + splits)
    for hq, hkv in ((64, 8), (16, 2), (12, 4)):
        lens = [rng.choice([0, 15, 16, 17, rng.randint(0, 70), rng.randint(100, 1500)]) for _ in range(9)]
        print(f"fused append, {splits} splits, heads {hq}/{hkv}, lens {lens}", flush=True)
        case = workloads.make_decode_case("fa", 50 + splits, lens, hq, hkv, device=DEV)
        want = case.kv_pool.clone()
        ops.kv_append(case.k_new, case.v_new, case.slot_mapping, want)
        pool = case.kv_pool.clone()
        out = ops.paged_decode(case.q, pool, case.block_table, case.seq_lens, case.softmax_scale, schedule="splits",
                               num_splits=splits, k_new=case.k_new, v_new=case.v_new)
        torch.cuda.synchronize()
        assert torch.equal(pool.view(torch.int16), want.view(torch.int16))
        ref = c_oracle.paged_decode(to_np16(case.q), to_np16(want), case.block_table.cpu().numpy(),
                                    case.seq_lens.cpu().numpy(), case.softmax_scale)
        assert_attention_close(out, ref, f"fused append {splits}")
        # fp8 pool: the codes of a separate quantising append, attention over the decoded codes
        scales = torch.cat([0.02 * (1 + 0.1 * torch.arange(hkv)), 0.015 * (1 + 0.2 * torch.arange(hkv))]).float().to(DEV)
        codes = torch.empty(case.kv_pool.shape, dtype=torch.uint8, device=DEV)
        every = torch.arange(codes.shape[0], dtype=torch.int32, device=DEV)
        ops.kv_append_fp8(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every, codes, scales)
        want8 = codes.clone()
        ops.kv_append_fp8(case.k_new, case.v_new, case.slot_mapping, want8, scales)
        out8 = ops.paged_decode(case.q, codes, case.block_table, case.seq_lens, case.softmax_scale, schedule="splits",
                                num_splits=splits, kv_scales=scales, k_new=case.k_new, v_new=case.v_new)
        torch.cuda.synchronize()
        a, b = codes.cpu().numpy(), want8.cpu().numpy()
        assert int(((a != b) & ~(((a & 0x7F) == 0) & ((b & 0x7F) == 0))).sum()) == 0
        values = torch.from_numpy(fp8.dequantize_pool(a, scales.cpu().numpy()))
        ref8 = cpu_ref.paged_decode_ref(case.q.cpu(), values, case.block_table.cpu(), case.seq_lens.cpu(),
                                        case.softmax_scale).numpy()
        assert_attention_close(out8, ref8, f"fused append fp8 {splits}")


def test_fused_append_argument_checks():
    case = workloads.make_decode_case("fa", 60, [20, 30], 16, 8, device=DEV)
    with pytest.raises(ValueError, match="k_new and v_new go together"):
        ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, schedule="splits", num_splits=1,
                         k_new=case.k_new)
    with pytest.raises(ValueError, match="both stages"):
        ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, schedule="splits", num_splits=2,
                         stage="split", k_new=case.k_new, v_new=case.v_new)
    with pytest.raises(ValueError, match="decode_step"):
        ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, schedule="balanced",
                         k_new=case.k_new, v_new=case.v_new)
    with pytest.raises(ValueError, match=r"\[B, Hkv, D\]"):
        ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, schedule="splits", num_splits=1,
                         k_new=case.k_new[:1], v_new=case.v_new[:1])


@pytest.mark.parametrize("lens,expected", [([30, 100, 64, 7], 8), ([40, 1200, 900, 16], 16), ([40, 9000, 900, 16], 0)],
                         ids=["short", "long", "longer"])
def test_drop_in_flash_decoding_on_either_schedule(lens, expected):
    """The reference-signature wrapper picks the schedule from the batch size and the longest
    sequence it is told; each choice gives the oracle's attention."""
    from llama_lite_npu_amd import kernels as compat

    hq, hkv = 16, 8
    print(f"flash_decoding wrapper, lens {lens}", flush=True)
    case = workloads.make_decode_case("compat", 70, lens, hq, hkv, device=DEV)
    pool = case.kv_pool
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool)
    # the reference's per-token table: slot of every logical position
    token_table = (case.block_table.long()[:, :, None] * 16 + torch.arange(16, device=DEV)).reshape(len(lens), -1)
    max_len = max(lens) + 1
    picked = ops.decode_schedule(len(lens), hkv, (max_len + 15) // 16, len(lens) * ((max_len + 15) // 16),
                                 2 * hkv * 128 * 2, heads_per_kv_head=hq // hkv)
    assert picked == expected
    out = compat.flash_decoding(case.q, pool[:, :hkv], pool[:, hkv:], case.softmax_scale,
                                token_table.to(torch.int32), case.seq_lens.long(), max_len)
    torch.cuda.synchronize()
    ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool), case.block_table.cpu().numpy(),
                                case.seq_lens.cpu().numpy(), case.softmax_scale)
    assert_attention_close(out, ref, "flash_decoding wrapper")
