"""GPU: the benchmark configurations at their full sizes.

The smaller parity tests compare every kernel with the oracle element by element. Here the same
entry points run on the workloads the benchmark times -- C2 (32 sequences up to 4096 tokens),
C3 (8 prompts up to 2048 tokens), C4 (64 sequences behind 2048 shared tokens), C5 (128 sequences
up to 32768 tokens in a pool with holes) -- and are checked by what does not depend on size:
the appended pool is the closed form `pool[slots] = rows` bit for bit, a repeated launch gives
the same bits, moving pages and rewriting the tables gives the same bits, another schedule or a
chunked prompt gives the same attention within tolerance. Where the fp32 oracle finishes in
seconds it is compared directly (C2, C3, C4 and C5 whole; C5's pages are pulled out of the 7 GB
pool eight sequences at a time).
"""

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import ops, workloads
from oracle import c_oracle, cpu_ref
from tests.parity import assert_attention_close, assert_bit_exact, to_np16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PS = 16


def _pages_of(lens: torch.Tensor) -> list[int]:
    return ((lens.cpu().to(torch.int64) + PS - 1) // PS).tolist()


def _oracle_rows(q, pool, table, seq_lens, rows, scale):
    """fp32 oracle for the chosen sequences: their pages are copied out of the device pool into a
    small host pool addressed by an identity table."""
    paged = pool.view(-1, PS, *pool.shape[1:])
    n_pages = _pages_of(seq_lens)
    parts, lists, cur = [], [], 0
    for b in rows:
        ids = table[b, :n_pages[b]].to(torch.long)
        parts.append(paged[ids].cpu())
        lists.append(torch.arange(cur, cur + n_pages[b], dtype=torch.int32))
        cur += n_pages[b]
    small = torch.cat(parts).view(-1, *pool.shape[1:])
    idx = torch.tensor(rows, dtype=torch.long)
    return cpu_ref.paged_decode_ref(q.cpu()[idx], small, workloads.table_from_lists(lists),
                                    seq_lens.cpu()[idx], scale).numpy()


def _appended_on_host(pool0, k_new, v_new, slots):
    host = to_np16(pool0).copy()
    c_oracle.kv_append(to_np16(torch.cat([k_new, v_new], dim=1)), slots.cpu().numpy(), host)
    return host


def _move_pages(case, seed):
    """The same logical KV under another physical placement: every page moved by page_gather."""
    perm = torch.randperm(case.num_pages, generator=torch.Generator().manual_seed(seed)).to(torch.int32).to(DEV)
    moved = torch.empty_like(case.kv_pool)
    ops.page_gather(case.kv_pool, moved, torch.arange(case.num_pages, dtype=torch.int32, device=DEV), perm)
    return moved, perm[case.block_table.to(torch.long)].contiguous()


def test_c2_decode_step_at_full_size():
    print("full size: C2 decode step", flush=True)
    case = workloads.config_c2(DEV)
    assert case.q.shape == (32, 64, 128) and int(case.seq_lens.max()) <= 4097
    pool0 = case.kv_pool.clone()
    plan = ops.DecodePlan(case.block_table, case.seq_lens, 64, 8, case.num_pages)
    out = ops.decode_step(case.q, case.kv_pool, plan, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    print("  pool against pool[slots] = rows", flush=True)
    assert_bit_exact(case.kv_pool, _appended_on_host(pool0, case.k_new, case.v_new, case.slot_mapping),
                     "C2 fused append")
    print("  oracle, all 32 sequences", flush=True)
    ref = cpu_ref.paged_decode_ref(case.q.cpu(), case.kv_pool.cpu(), case.block_table.cpu(),
                                   case.seq_lens.cpu(), case.softmax_scale).numpy()
    assert_attention_close(out, ref, "C2 balanced step")
    # the pool now holds the step's rows: a plain launch over it must repeat the step bit for bit
    again = ops.decode_step(case.q, case.kv_pool, plan, None, None, case.softmax_scale)
    third = ops.decode_step(case.q, case.kv_pool, plan, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(again, out) and torch.equal(third, out)
    print("  other schedules", flush=True)
    for kw in ({"num_splits": 1}, {"num_splits": 16}, {"schedule": "balanced", "chunks": 100},
               {"schedule": "balanced", "chunks": 1024}):
        other = ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale, **kw)
        assert_attention_close(other, ref, f"C2 {kw}")
    print("  pages moved", flush=True)
    moved, table = _move_pages(case, 7)
    plan2 = ops.DecodePlan(table, case.seq_lens, 64, 8, case.num_pages)
    elsewhere = ops.decode_step(case.q, moved, plan2, None, None, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(elsewhere, out), "the result depends on where the pages lie"


def test_c3_prefill_at_full_size():
    print("full size: C3 varlen prefill", flush=True)
    case = workloads.config_c3(DEV)
    assert case.batch == 8 and case.q.shape[1:] == (64, 128) and case.max_q_len <= 2048
    pool0 = case.kv_pool.clone()
    ops.kv_append(case.k, case.v, case.slot_mapping, case.kv_pool)
    out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, None, case.max_q_len,
                            case.softmax_scale)
    torch.cuda.synchronize()
    assert_bit_exact(case.kv_pool, _appended_on_host(pool0, case.k, case.v, case.slot_mapping), "C3 append")
    print("  oracle, all prompts", flush=True)
    ref = cpu_ref.paged_prefill_ref(case.q.cpu(), case.kv_pool.cpu(), case.block_table.cpu(),
                                    case.cu_q_lens.cpu(), None, case.softmax_scale).numpy()
    assert_attention_close(out, ref, "C3 paged prefill")
    again = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, None, case.max_q_len,
                              case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(again, out)
    print("  packed K/V", flush=True)
    packed = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1].contiguous(), case.seq_lens,
                                case.max_q_len, case.softmax_scale)
    assert_attention_close(packed, ref, "C3 packed prefill")
    print("  second halves as chunks over their history", flush=True)
    lens = case.seq_lens.cpu().to(torch.int64)
    cu = case.cu_q_lens.cpu().to(torch.int64)
    first = lens // 2
    rows = torch.cat([torch.arange(int(cu[i] + first[i]), int(cu[i + 1])) for i in range(case.batch)]).to(DEV)
    cu_half = torch.zeros(case.batch + 1, dtype=torch.int32)
    cu_half[1:] = torch.cumsum(lens - first, 0)
    chunk = ops.paged_prefill(case.q[rows].contiguous(), case.kv_pool, case.block_table, cu_half.to(DEV),
                              first.to(torch.int32).to(DEV), int((lens - first).max()), case.softmax_scale)
    assert_attention_close(chunk, ref[rows.cpu().numpy()], "C3 second halves")


def test_c4_copy_on_write_then_shared_prefix_step_at_full_size():
    print("full size: C4 copy-on-write + shared-prefix step", flush=True)
    case = workloads.config_c4(DEV)
    n_shared = case.extra["n_shared"]
    assert case.q.shape == (64, 64, 128) and n_shared == 128
    pool0 = case.kv_pool.clone()
    # every sequence's last page is held by someone else too: it moves to the spare page first
    last = ((case.seq_lens.to(torch.long) - 1) // PS)[:, None]
    src = case.block_table.gather(1, last)[:, 0].contiguous()
    dst = case.extra["spare_pages"].to(DEV)
    ops.page_copy(case.kv_pool, src, dst)
    table = case.block_table.clone()
    table.scatter_(1, last, dst[:, None])
    slots = (dst.to(torch.long) * PS + (case.seq_lens.to(torch.long) - 1) % PS).to(torch.int32)
    plan = ops.DecodePlan(table, case.seq_lens, 64, 8, case.num_pages, shared_pages=n_shared)
    out = ops.decode_step(case.q, case.kv_pool, plan, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    print("  pool: old last pages untouched, copies hold the page plus the new row", flush=True)
    host = to_np16(pool0).copy()
    host_pages = host.reshape(case.num_pages, -1)       # a view: one row per page
    host_pages[dst.cpu().numpy()] = host_pages[src.cpu().numpy()]
    c_oracle.kv_append(to_np16(torch.cat([case.k_new, case.v_new], dim=1)), slots.cpu().numpy(), host)
    assert_bit_exact(case.kv_pool, host, "C4 copy-on-write + fused append")
    print("  oracle, all 64 sequences", flush=True)
    ref = cpu_ref.paged_decode_ref(case.q.cpu(), case.kv_pool.cpu(), table.cpu(), case.seq_lens.cpu(),
                                   case.softmax_scale).numpy()
    assert_attention_close(out, ref, "C4 shared-prefix step")
    print("  every sequence with its own copy of the prefix pages", flush=True)
    extra = 64 * n_shared
    wide = torch.empty(((case.num_pages + extra) * PS,) + tuple(case.kv_pool.shape[1:]), dtype=torch.float16,
                       device=DEV)
    wide[:case.num_pages * PS] = case.kv_pool
    own = torch.arange(case.num_pages, case.num_pages + extra, dtype=torch.int32, device=DEV)
    ops.page_copy(wide, table[:, :n_shared].reshape(-1).contiguous(), own)
    table_own = table.clone()
    table_own[:, :n_shared] = own.view(64, n_shared)
    private = ops.paged_decode(case.q, wide, table_own, case.seq_lens, case.softmax_scale, schedule="balanced")
    assert_attention_close(private, ref, "C4 private prefix copies")
    assert float((private.float() - out.float()).abs().max()) <= 1e-3
    again = ops.decode_step(case.q, case.kv_pool, plan, None, None, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(again, out)


def test_c5_long_context_decode_and_compaction_at_full_size():
    print("full size: C5 long-context decode + compaction", flush=True)
    case = workloads.config_c5(DEV)
    lens = case.seq_lens.cpu().to(torch.int64)
    assert case.q.shape == (128, 32, 128) and int(lens.min()) > 8192 and int(lens.max()) <= 32769
    n_pages = _pages_of(case.seq_lens)
    n_live = sum(n_pages)
    assert case.num_pages * 3 // 4 - 1 <= n_live <= case.num_pages * 3 // 4 + 1      # a quarter of the pool is holes
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, case.kv_pool)
    # the oracle on every sequence, eight at a time (their pages leave the 7 GB pool in pieces of
    # about 330 MB)
    sample = list(range(case.batch))
    print("  oracle on all 128 sequences", flush=True)
    ref = np.concatenate([_oracle_rows(case.q, case.kv_pool, case.block_table, case.seq_lens,
                                       sample[i:i + 8], case.softmax_scale) for i in range(0, case.batch, 8)])
    runs = {}
    for name, kw in (("16 splits", {"num_splits": 16}), ("balanced", {"schedule": "balanced"})):
        print(f"  {name}", flush=True)
        out = ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale, **kw)
        again = ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale, **kw)
        torch.cuda.synchronize()
        assert torch.equal(out, again), f"C5 {name}: two launches differ"
        assert_attention_close(out[sample], ref, f"C5 {name}")
        assert bool(torch.isfinite(out.float()).all())
        runs[name] = out
    assert float((runs["16 splits"].float() - runs["balanced"].float()).abs().max()) <= 1e-3

    print("  out-of-place compaction: live pages gathered into a dense pool", flush=True)
    table = case.block_table.cpu()
    live = torch.cat([table[b, :n] for b, n in enumerate(n_pages)])
    dense_table = torch.zeros_like(table)
    cur = 0
    for b, n in enumerate(n_pages):
        dense_table[b, :n] = torch.arange(cur, cur + n, dtype=torch.int32)
        cur += n
    dense = torch.empty((n_live * PS,) + tuple(case.kv_pool.shape[1:]), dtype=torch.float16, device=DEV)
    ops.page_gather(case.kv_pool, dense, live.to(DEV), None)
    for name, kw in (("16 splits", {"num_splits": 16}), ("balanced", {"schedule": "balanced"})):
        after = ops.paged_decode(case.q, dense, dense_table.to(DEV), case.seq_lens, case.softmax_scale, **kw)
        torch.cuda.synchronize()
        assert torch.equal(after, runs[name]), f"C5 {name}: compaction changed the result"
    del dense

    print("  in-place compaction: pages past the live count move into the holes below it", flush=True)
    is_live = torch.zeros(case.num_pages, dtype=torch.bool)
    is_live[live.to(torch.long)] = True
    movers = live[live >= n_live]
    holes = torch.nonzero(~is_live[:n_live])[:, 0].to(torch.int32)
    assert movers.numel() == holes.numel() and movers.numel() > n_live // 8
    ops.page_copy(case.kv_pool, movers.to(DEV), holes.to(DEV))
    remap = torch.arange(case.num_pages, dtype=torch.int32)
    remap[movers.to(torch.long)] = holes
    packed_table = torch.zeros_like(table)
    for b, n in enumerate(n_pages):
        packed_table[b, :n] = remap[table[b, :n].to(torch.long)]
    assert int(packed_table.max()) < n_live
    front = case.kv_pool[:n_live * PS]          # the pool could now be cut back to the live pages
    after = ops.paged_decode(case.q, front, packed_table.to(DEV), case.seq_lens, case.softmax_scale,
                             schedule="balanced")
    torch.cuda.synchronize()
    assert torch.equal(after, runs["balanced"]), "C5: in-place compaction changed the result"


def test_c2_decode_step_over_an_fp8_pool_at_full_size():
    print("full size: C2 decode step over an fp8 pool", flush=True)
    from oracle import fp8

    case = workloads.config_c2(DEV)
    hkv = 8
    scales = torch.cat([0.02 * (1 + 0.1 * torch.arange(hkv)), 0.015 * (1 + 0.2 * torch.arange(hkv))]).float().to(DEV)
    slots_all = torch.arange(case.kv_pool.shape[0], dtype=torch.int32, device=DEV)
    pool = torch.empty(case.kv_pool.shape, dtype=torch.uint8, device=DEV)
    # the whole fp16 pool quantised by one append of 81 k rows (K and V halves are strided views)
    ops.kv_append_fp8(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], slots_all, pool, scales)
    plan = ops.DecodePlan(case.block_table, case.seq_lens, 64, hkv, case.num_pages)
    out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale, kv_scales=scales)
    torch.cuda.synchronize()
    print("  codes of sampled rows and of the step's rows against the oracle", flush=True)
    new_slots = case.slot_mapping.cpu().numpy()
    rows = np.setdiff1d(np.random.default_rng(3).choice(case.kv_pool.shape[0], 3000, replace=False), new_slots)
    want = np.zeros((rows.size + new_slots.size, 2 * hkv, 128), dtype=np.uint8)
    src = case.kv_pool.cpu().numpy()
    fp8.kv_append(src[rows, :hkv], src[rows, hkv:], np.arange(rows.size, dtype=np.int32), want, scales.cpu().numpy())
    fp8.kv_append(to_np16(case.k_new), to_np16(case.v_new),
                  np.arange(rows.size, rows.size + new_slots.size, dtype=np.int32), want, scales.cpu().numpy())
    got = pool.cpu().numpy()
    got_rows = got[np.concatenate([rows, new_slots])]
    differ = (got_rows != want) & ~(((got_rows & 0x7F) == 0) & ((want & 0x7F) == 0))   # the sign of zero is free
    assert int(differ.sum()) == 0, f"{int(differ.sum())} codes differ"
    print("  oracle on the decoded pool, all 32 sequences", flush=True)
    values = torch.from_numpy(fp8.dequantize_pool(got, scales.cpu().numpy()))
    ref = cpu_ref.paged_decode_ref(case.q.cpu(), values, case.block_table.cpu(), case.seq_lens.cpu(),
                                   case.softmax_scale).numpy()
    assert_attention_close(out, ref, "C2 fp8 step")
    again = ops.decode_step(case.q, pool, plan, None, None, case.softmax_scale, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(again, out)
    moved = torch.empty_like(pool)
    perm = torch.randperm(case.num_pages, generator=torch.Generator().manual_seed(11)).to(torch.int32).to(DEV)
    ops.page_gather(pool, moved, torch.arange(case.num_pages, dtype=torch.int32, device=DEV), perm)
    plan2 = ops.DecodePlan(perm[case.block_table.to(torch.long)].contiguous(), case.seq_lens, 64, hkv, case.num_pages)
    elsewhere = ops.decode_step(case.q, moved, plan2, None, None, case.softmax_scale, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(elsewhere, out), "the result depends on where the fp8 pages lie"
