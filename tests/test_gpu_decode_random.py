"""GPU: seeded random decode steps against the oracle.

Head layouts, batch sizes, length mixes (empty, one token, page-boundary, long), chunk counts from
one workgroup walking every sequence to more chunks than pages, empty rows in the middle of the
batch: the fused step (append + attention) must write the pool bit for bit like the append kernel,
attend within the attention tolerance of the fp32 oracle, zero the rows of empty sequences and
repeat bit for bit; the same over fp8 pools (codes bit-equal to the quantising append) and behind
a shared prefix, declared fully or partly.
"""

import random

import pytest
import torch

from llama_lite_npu_amd import ops, workloads
from oracle import c_oracle, cpu_ref, fp8
from tests.parity import assert_attention_close, to_np16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HEADS = [(64, 8), (32, 4), (16, 8), (8, 8), (16, 1), (4, 2), (32, 16), (24, 12), (6, 3), (16, 2)]
CHUNKS = [None, 1, 2, 3, 7, 37, 64, 256, 300]


def _lengths(rng, kind, b):
    def one():
        if kind == "tiny":
            return rng.choice([0, 1, 2, 15, 16, 17, 31, 33])
        if kind == "short":
            return rng.randint(0, 200)
        if kind == "long":
            return rng.randint(500, 3000)
        return rng.choice([rng.randint(0, 40), rng.randint(100, 900), rng.randint(0, 3000)])
    return [one() for _ in range(b)]


@pytest.mark.parametrize("seed", range(4))
def test_random_fused_steps(seed):
    rng = random.Random(100 + seed)
    for case_no in range(12):
        hq, hkv = rng.choice(HEADS)
        b = rng.choice([1, 2, 3, 5, 8, 13, 32, 70])
        kind = rng.choice(["short", "mixed", "long", "tiny"])
        lens = _lengths(rng, kind, b)
        chunks = rng.choice(CHUNKS)
        case = workloads.make_decode_case("random", 1000 + 100 * seed + case_no, lens, hq, hkv, device=DEV)
        empty = [i for i in range(b) if rng.random() < 0.1]
        live = [i for i in range(b) if i not in empty]
        for i in empty:
            case.seq_lens[i] = 0
        print(f"random step {seed}.{case_no}: heads {hq}/{hkv} batch {b} {kind} chunks {chunks} empty {empty}", flush=True)
        pool_ref = case.kv_pool.clone()
        ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool_ref)
        keep = torch.ones(case.kv_pool.shape[0], dtype=torch.bool, device=DEV)
        for i in empty:                      # an empty sequence appends nothing
            keep[case.slot_mapping[i].long()] = False
        ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                    case.seq_lens.cpu().numpy(), case.softmax_scale)
        plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, chunks)
        out = ops.decode_step(case.q, case.kv_pool, plan, case.k_new, case.v_new, case.softmax_scale)
        again = ops.decode_step(case.q, case.kv_pool, plan, None, None, case.softmax_scale)
        torch.cuda.synchronize()
        assert torch.equal(case.kv_pool[keep].view(torch.int16), pool_ref[keep].view(torch.int16))
        assert_attention_close(out, ref, f"random step {seed}.{case_no}")
        for i in empty:
            assert float(out[i].abs().max()) == 0.0
        assert torch.equal(again[live], out[live])


@pytest.mark.parametrize("seed", range(2))
def test_random_steps_over_fp8_pools(seed):
    rng = random.Random(200 + seed)
    for case_no in range(10):
        hq, hkv = rng.choice([(64, 8), (32, 4), (16, 8), (8, 8), (4, 2), (16, 2)])
        b = rng.choice([1, 2, 5, 8, 33])
        lens = _lengths(rng, "mixed", b)
        chunks = rng.choice([None, 1, 3, 37, 256])
        print(f"random fp8 step {seed}.{case_no}: heads {hq}/{hkv} batch {b} chunks {chunks}", flush=True)
        case = workloads.make_decode_case("random", 3000 + 100 * seed + case_no, lens, hq, hkv, device=DEV)
        scales = torch.cat([0.02 * (1 + 0.1 * torch.arange(hkv)), 0.015 * (1 + 0.2 * torch.arange(hkv))]).float().to(DEV)
        pool = torch.empty(case.kv_pool.shape, dtype=torch.uint8, device=DEV)
        every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
        ops.kv_append_fp8(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every_slot, pool, scales)
        want = pool.clone()
        ops.kv_append_fp8(case.k_new, case.v_new, case.slot_mapping, want, scales)
        plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, chunks)
        out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale, kv_scales=scales)
        torch.cuda.synchronize()
        got, exp = pool.cpu().numpy(), want.cpu().numpy()
        differ = (got != exp) & ~(((got & 0x7F) == 0) & ((exp & 0x7F) == 0))      # the sign of zero is free
        assert int(differ.sum()) == 0
        values = torch.from_numpy(fp8.dequantize_pool(got, scales.cpu().numpy()))
        ref = cpu_ref.paged_decode_ref(case.q.cpu(), values, case.block_table.cpu(), case.seq_lens.cpu(),
                                       case.softmax_scale).numpy()
        assert_attention_close(out, ref, f"random fp8 step {seed}.{case_no}")


@pytest.mark.parametrize("seed", range(2))
def test_random_steps_behind_a_shared_prefix(seed):
    rng = random.Random(300 + seed)
    for case_no in range(10):
        hq, hkv = rng.choice([(64, 8), (32, 4), (16, 8), (8, 8), (4, 2), (16, 2)])
        b = rng.choice([1, 2, 5, 8, 33])
        shared = rng.choice([4, 6, 17, 40])
        ctx = [shared * 16 + n for n in _lengths(rng, "mixed", b)]
        chunks = rng.choice([None, 1, 3, 37, 256])
        declared = rng.choice([shared, max(1, shared // 2)])
        print(f"random prefix step {seed}.{case_no}: heads {hq}/{hkv} batch {b} shared {shared} declared {declared} "
              f"chunks {chunks}", flush=True)
        pages = [(c + 1 + 15) // 16 for c in ctx]
        num_pages = shared + sum(p - shared for p in pages) + 9
        perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(10 * seed + case_no)).to(torch.int32)
        lists, cur = [], shared
        for p in pages:
            lists.append(torch.cat([perm[:shared], perm[cur:cur + p - shared]]))
            cur += p - shared
        case = workloads.make_decode_case("random", 5000 + 100 * seed + case_no, ctx, hq, hkv, num_pages=num_pages,
                                          device=DEV, page_lists=lists)
        pool_ref = case.kv_pool.clone()
        ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool_ref)
        ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                    case.seq_lens.cpu().numpy(), case.softmax_scale)
        plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, chunks, shared_pages=declared)
        pool0 = case.kv_pool.clone()
        out = ops.decode_step(case.q, case.kv_pool, plan, case.k_new, case.v_new, case.softmax_scale)
        torch.cuda.synchronize()
        assert torch.equal(case.kv_pool.view(torch.int16), pool_ref.view(torch.int16))
        assert_attention_close(out, ref, f"random prefix step {seed}.{case_no}")
        # the same step over fp8 pools: codes as the quantising append writes them, attention
        # within tolerance of the oracle on the decoded pool, equal to the step without the
        # shared-prefix kernel up to the order of the sums
        scales = torch.cat([0.02 * (1 + 0.1 * torch.arange(hkv)), 0.015 * (1 + 0.2 * torch.arange(hkv))]).float().to(DEV)
        pool8 = torch.empty(pool0.shape, dtype=torch.uint8, device=DEV)
        every_slot = torch.arange(pool8.shape[0], dtype=torch.int32, device=DEV)
        ops.kv_append_fp8(pool0[:, :hkv], pool0[:, hkv:], every_slot, pool8, scales)
        want8 = pool8.clone()
        ops.kv_append_fp8(case.k_new, case.v_new, case.slot_mapping, want8, scales)
        plain = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, chunks)
        out_plain = ops.decode_step(case.q, want8.clone(), plain, None, None, case.softmax_scale, kv_scales=scales)
        out8 = ops.decode_step(case.q, pool8, plan, case.k_new, case.v_new, case.softmax_scale, kv_scales=scales)
        torch.cuda.synchronize()
        got, exp = pool8.cpu().numpy(), want8.cpu().numpy()
        assert int(((got != exp) & ~(((got & 0x7F) == 0) & ((exp & 0x7F) == 0))).sum()) == 0
        values = torch.from_numpy(fp8.dequantize_pool(got, scales.cpu().numpy()))
        ref8 = cpu_ref.paged_decode_ref(case.q.cpu(), values, case.block_table.cpu(), case.seq_lens.cpu(),
                                        case.softmax_scale).numpy()
        assert_attention_close(out8, ref8, f"random fp8 prefix step {seed}.{case_no}")
        assert float((out8.float() - out_plain.float()).abs().max()) <= 1e-3


@pytest.mark.parametrize("batch", [200, 600])
def test_large_batches_take_the_packed_merge(batch):
    """More than 8192 (sequence, head) rows: four rows per merge workgroup; more sequences than
    twice the chunk boundaries (600 >= 512): merge by boundary. One long sequence among the short ones spans
    more than 16 chunks, so the long-row merge runs inside the packed launch too."""
    rng = random.Random(500 + batch)
    lens = [rng.randint(0, 300 if batch < 400 else 90) for _ in range(batch)]
    lens[batch // 3] = 6000
    lens[5] = 0
    print(f"large batch {batch}", flush=True)
    case = workloads.make_decode_case("large", 9000 + batch, lens, 64, 8, device=DEV)
    case.seq_lens[11] = 0                     # an empty row
    pool_ref = case.kv_pool.clone()
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool_ref)
    ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                case.seq_lens.cpu().numpy(), case.softmax_scale)
    plan = ops.DecodePlan(case.block_table, case.seq_lens, 64, 8, case.num_pages)
    assert plan.chunks == 256
    out = ops.decode_step(case.q, case.kv_pool, plan, case.k_new, case.v_new, case.softmax_scale)
    again = ops.decode_step(case.q, case.kv_pool, plan, None, None, case.softmax_scale)
    torch.cuda.synchronize()
    assert_attention_close(out, ref, f"large batch {batch}")
    assert float(out[11].abs().max()) == 0.0
    live = [i for i in range(batch) if i != 11]
    assert torch.equal(again[live], out[live])


@pytest.mark.parametrize("seed", range(2))
def test_random_fused_steps_at_head_dim_64_and_larger_pages(seed):
    """The same at head dim 64 (the second build of the decode kernels) with pages of 16, 32 or 64
    tokens, both schedules."""
    rng = random.Random(700 + seed)
    for case_no in range(10):
        hq, hkv = rng.choice(HEADS)
        page_size = rng.choice([16, 32, 64])
        b = rng.choice([1, 2, 3, 5, 8, 13, 32])
        kind = rng.choice(["short", "mixed", "long", "tiny"])
        lens = _lengths(rng, kind, b)
        chunks = rng.choice(CHUNKS)
        case = workloads.make_decode_case("random64", 5000 + 100 * seed + case_no, lens, hq, hkv, device=DEV,
                                          head_dim=64, page_size=page_size)
        empty = [i for i in range(b) if rng.random() < 0.1]
        live = [i for i in range(b) if i not in empty]
        for i in empty:
            case.seq_lens[i] = 0
        print(f"random step hd64 {seed}.{case_no}: heads {hq}/{hkv} page {page_size} batch {b} {kind} chunks {chunks} "
              f"empty {empty}", flush=True)
        pool_ref = case.kv_pool.clone()
        ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool_ref)
        keep = torch.ones(case.kv_pool.shape[0], dtype=torch.bool, device=DEV)
        for i in empty:
            keep[case.slot_mapping[i].long()] = False
        ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                    case.seq_lens.cpu().numpy(), case.softmax_scale, page_size=page_size)
        plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, chunks, page_size=page_size)
        pool = case.kv_pool.clone()
        out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale)
        again = ops.decode_step(case.q, pool, plan, None, None, case.softmax_scale)
        split_pool = case.kv_pool.clone()
        split = ops.paged_decode(case.q, split_pool, case.block_table, case.seq_lens, case.softmax_scale,
                                 max_splits=rng.choice([1, 3, 8]), min_pages_per_split=rng.choice([1, 4]),
                                 k_new=case.k_new, v_new=case.v_new, page_size=page_size)
        torch.cuda.synchronize()
        assert torch.equal(pool[keep].view(torch.int16), pool_ref[keep].view(torch.int16))
        assert torch.equal(split_pool[keep].view(torch.int16), pool_ref[keep].view(torch.int16))
        assert_attention_close(out, ref, f"random step hd64 {seed}.{case_no}")
        assert_attention_close(split, ref, f"random step hd64 {seed}.{case_no}, splits schedule")
        for i in empty:
            assert float(out[i].abs().max()) == 0.0
        assert torch.equal(again[live], out[live])
