"""GPU: seeded random varlen prefills against the oracle -- ragged chunk lengths over ragged
histories (including none), every head layout, chunks of one row, sequences that end on and next
to page and tile boundaries; the packed entry point on the same rows when there is no history."""

import random

import pytest
import torch

from llama_lite_npu_amd import ops, workloads
from oracle import cpu_ref
from tests.parity import assert_attention_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HEADS = [(64, 8), (32, 4), (16, 8), (8, 8), (16, 1), (4, 2), (32, 16), (6, 3), (16, 2)]
EDGES = [1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129]


@pytest.mark.parametrize("seed", range(3))
def test_random_chunks_over_random_histories(seed):
    rng = random.Random(400 + seed)
    for case_no in range(8):
        hq, hkv = rng.choice(HEADS)
        b = rng.choice([1, 2, 3, 5])
        q_lens = [rng.choice([rng.choice(EDGES), rng.randint(1, 400)]) for _ in range(b)]
        with_history = rng.random() < 0.7
        ctx = [rng.choice([0, rng.choice(EDGES), rng.randint(0, 700)]) if with_history else 0 for _ in range(b)]
        print(f"random prefill {seed}.{case_no}: heads {hq}/{hkv} chunks {q_lens} histories {ctx}", flush=True)
        case = workloads.make_prefill_case("random", 7000 + 100 * seed + case_no, q_lens, hq, hkv,
                                           context_lens=ctx, device=DEV)
        # the chunk's own K/V go through the append; the history is whatever the pool already holds
        ops.kv_append(case.k, case.v, case.slot_mapping, case.kv_pool)
        ctx_dev = case.context_lens if with_history else None
        out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, ctx_dev, case.max_q_len,
                                case.softmax_scale)
        again = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, ctx_dev, case.max_q_len,
                                  case.softmax_scale)
        torch.cuda.synchronize()
        ref = cpu_ref.paged_prefill_ref(case.q.cpu(), case.kv_pool.cpu(), case.block_table.cpu(),
                                        case.cu_q_lens.cpu(), case.context_lens.cpu() if with_history else None,
                                        case.softmax_scale).numpy()
        assert_attention_close(out, ref, f"random prefill {seed}.{case_no}")
        assert torch.equal(out, again)
        if not with_history:
            packed = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1].contiguous(), case.seq_lens,
                                        case.max_q_len, case.softmax_scale)
            assert_attention_close(packed, ref, f"random packed prefill {seed}.{case_no}")


@pytest.mark.parametrize("seed", range(2))
def test_random_chunks_at_head_dim_64_and_larger_pages(seed):
    """The same at head dim 64 (the tiled kernel's second build) with pages of 16, 32 or 64 tokens."""
    rng = random.Random(900 + seed)
    for case_no in range(8):
        hq, hkv = rng.choice(HEADS)
        page_size = rng.choice([16, 32, 64])
        b = rng.choice([1, 2, 3, 5])
        q_lens = [rng.choice([rng.choice(EDGES), rng.randint(1, 400)]) for _ in range(b)]
        with_history = rng.random() < 0.7
        ctx = [rng.choice([0, rng.choice(EDGES), rng.randint(0, 700)]) if with_history else 0 for _ in range(b)]
        print(f"random prefill hd64 {seed}.{case_no}: heads {hq}/{hkv} page {page_size} chunks {q_lens} histories {ctx}",
              flush=True)
        case = workloads.make_prefill_case("random64", 9000 + 100 * seed + case_no, q_lens, hq, hkv,
                                           context_lens=ctx, device=DEV, head_dim=64, page_size=page_size)
        ops.kv_append(case.k, case.v, case.slot_mapping, case.kv_pool)
        ctx_dev = case.context_lens if with_history else None
        out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, ctx_dev, case.max_q_len,
                                case.softmax_scale, page_size=page_size)
        again = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, ctx_dev, case.max_q_len,
                                  case.softmax_scale, page_size=page_size)
        torch.cuda.synchronize()
        ref = cpu_ref.paged_prefill_ref(case.q.cpu(), case.kv_pool.cpu(), case.block_table.cpu(),
                                        case.cu_q_lens.cpu(), case.context_lens.cpu() if with_history else None,
                                        case.softmax_scale, page_size=page_size).numpy()
        assert_attention_close(out, ref, f"random prefill hd64 {seed}.{case_no}")
        assert torch.equal(out, again)
        if not with_history:
            packed = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1].contiguous(), case.seq_lens,
                                        case.max_q_len, case.softmax_scale)
            assert torch.equal(packed, out)
