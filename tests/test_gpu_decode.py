"""GPU parity of paged flash-decoding against the CPU oracle, through the C ABI."""

import pytest
import torch

from llama_lite_npu_amd import ops, workloads
from oracle import c_oracle
from tests.parity import assert_attention_close, to_np16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _oracle(case, seq_lens=None):
    sl = case.seq_lens if seq_lens is None else seq_lens
    return c_oracle.paged_decode(to_np16(case.q), to_np16(case.kv_pool), case.block_table.cpu().numpy(),
                                 sl.cpu().numpy(), case.softmax_scale, page_size=case.page_size)


def _run(case, **kw):
    out = ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale,
                           page_size=case.page_size, **kw)
    torch.cuda.synchronize()
    return out


def test_c1_append_then_decode():
    print("decode C1", flush=True)
    case = workloads.config_c1(DEV)
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, case.kv_pool)
    ref = _oracle(case)
    for kw in ({}, {"schedule": "balanced", "chunks": 16}, {"num_splits": 1}, {"num_splits": 4},
               {"max_splits": 8, "min_pages_per_split": 8}):
        print("  ", kw, flush=True)
        assert_attention_close(_run(case, **kw), ref, f"C1 {kw}")


@pytest.mark.parametrize("hq,hkv", [(16, 8), (64, 8), (32, 4), (8, 8), (16, 1), (4, 2)])
def test_head_layouts_and_ragged_lengths(hq, hkv):
    print(f"decode heads {hq}/{hkv}", flush=True)
    lens = [0, 1, 15, 16, 17, 255, 256, 700]  # context; +1 appended => 1, 2, 16, 17, 18, ...
    case = workloads.make_decode_case("ragged", 50 + hq + hkv, lens, hq, hkv, device=DEV)
    ref = _oracle(case)
    for kw in ({"num_splits": 1}, {"num_splits": 3}, {"max_splits": 16, "min_pages_per_split": 2}):
        assert_attention_close(_run(case, **kw), ref, f"ragged {hq}/{hkv} {kw}")


@pytest.mark.parametrize("hq,hkv", [(64, 8), (32, 4), (16, 1), (6, 3), (32, 16), (24, 12)])
@pytest.mark.parametrize("chunks", [1, 3, 37, 256, 1000])
def test_balanced_schedule_any_chunk_count(hq, hkv, chunks):
    """Equal-share schedule: chunks cut across sequence boundaries, empty sequences in between."""
    print(f"decode balanced {hq}/{hkv} chunks={chunks}", flush=True)
    lens = [300, 0, 1, 15, 16, 17, 700, 64, 2, 1200]
    case = workloads.make_decode_case("balanced", 60 + hq + hkv, lens, hq, hkv, device=DEV)
    case.seq_lens[1] = 0            # an empty sequence in the middle of the line
    case.seq_lens[8] = 0
    ref = _oracle(case)
    out = _run(case, schedule="balanced", chunks=chunks)
    assert_attention_close(out, ref, f"balanced {hq}/{hkv} chunks={chunks}")
    assert float(out[1].abs().max()) == 0.0 and float(out[8].abs().max()) == 0.0
    again = _run(case, schedule="balanced", chunks=chunks)
    assert torch.equal(out, again)


@pytest.mark.parametrize("hq,hkv,chunks", [(64, 8, None), (32, 4, 7), (16, 8, 64), (8, 1, 3)])
def test_fused_append_decode_step(hq, hkv, chunks):
    """One launch = append of the step's token + attention: pool bit exact, output as append->decode."""
    print(f"decode fused step {hq}/{hkv} chunks={chunks}", flush=True)
    lens = [37, 128, 511, 1000, 0, 15, 16, 31, 1]      # contexts; 128 -> new page, 15 -> fills a page
    case = workloads.make_decode_case("fused", 70 + hq, lens, hq, hkv, device=DEV)
    pool0 = case.kv_pool.clone()
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, case.kv_pool)
    want_out = _run(case, num_splits=1)
    ref = _oracle(case)
    pool = pool0.clone()
    plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, chunks)
    out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(pool.view(torch.int16), case.kv_pool.view(torch.int16)), "fused append not bit exact"
    assert_attention_close(out, ref, "fused step vs oracle")
    assert float((out.float() - want_out.float()).abs().max()) <= 1e-3
    # the plan is reusable: a second layer (other pool) through the same plan
    pool2 = pool0.clone()
    out2 = ops.decode_step(case.q, pool2, plan, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(out2, out) and torch.equal(pool2.view(torch.int16), pool.view(torch.int16))


def test_plan_refresh_follows_growing_sequences():
    """Decode steps: lengths grow by one per step; the plan is refreshed, not rebuilt."""
    print("decode plan refresh", flush=True)
    case = workloads.make_decode_case("grow", 71, [14, 300, 47], 16, 8, num_pages=64, device=DEV)
    plan = ops.DecodePlan(case.block_table, case.seq_lens, 16, 8, case.num_pages, chunks=8)
    lens = case.seq_lens.clone()
    for step in range(3):
        out = ops.decode_step(case.q, case.kv_pool, plan, None, None, case.softmax_scale)
        torch.cuda.synchronize()
        ref = _oracle(case, lens)
        assert_attention_close(out, ref, f"refresh step {step}")
        lens = lens + 1
        plan.refresh(seq_lens=lens)


def test_balanced_all_sequences_empty():
    print("decode balanced all empty", flush=True)
    case = workloads.make_decode_case("empty", 61, [5, 9], 16, 8, device=DEV)
    case.seq_lens[:] = 0
    out = _run(case, schedule="balanced")
    assert float(out.abs().max()) == 0.0


def test_zero_length_sequence_gives_zeros():
    print("decode zero length", flush=True)
    case = workloads.make_decode_case("zero", 77, [40, 3, 90], 16, 8, device=DEV)
    case.seq_lens[1] = 0
    ref = _oracle(case)
    for kw in ({"num_splits": 1}, {"num_splits": 4}):
        out = _run(case, **kw)
        assert_attention_close(out, ref, f"zero {kw}")
        assert float(out[1].abs().max()) == 0.0


@pytest.mark.parametrize("chunks", [2, 4, 9])
def test_balanced_many_short_rows_with_empty_ones_between(chunks):
    """Twice as many sequences as chunks and more: the merge then runs over the chunk boundaries
    (only a sequence that crosses one has pieces). Empty rows sit at the start, at the end, next
    to each other and right where chunks are cut."""
    print(f"decode balanced, short rows with empty ones, chunks={chunks}", flush=True)
    lens = [5, 33, 0, 18, 70, 0, 0, 2, 47, 16, 0, 90, 31, 1, 0, 64, 15, 17, 0, 40, 8, 0, 29, 12]
    case = workloads.make_decode_case("short-empty", 83 + chunks, lens, 16, 4, device=DEV)
    empty = [i for i, n in enumerate(lens) if n == 0] + [0, len(lens) - 1]
    for i in empty:
        case.seq_lens[i] = 0
    assert len(lens) >= 2 * chunks
    ref = _oracle(case)
    out = _run(case, schedule="balanced", chunks=chunks)
    assert_attention_close(out, ref, f"short rows with empty ones, chunks={chunks}")
    for i in empty:
        assert float(out[i].abs().max()) == 0.0
    assert torch.equal(out, _run(case, schedule="balanced", chunks=chunks))
    # the same step with the append fused in
    plan = ops.DecodePlan(case.block_table, case.seq_lens, 16, 4, case.num_pages, chunks=chunks)
    pool = case.kv_pool.clone()
    fused = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    want_pool = case.kv_pool.clone()
    live = [i for i in range(len(lens)) if i not in empty]
    for b in live:
        want_pool[int(case.slot_mapping[b]), :4], want_pool[int(case.slot_mapping[b]), 4:] = case.k_new[b], case.v_new[b]
    assert torch.equal(pool, want_pool)
    ref2 = c_oracle.paged_decode(to_np16(case.q), to_np16(want_pool), case.block_table.cpu().numpy(),
                                 case.seq_lens.cpu().numpy(), case.softmax_scale)
    assert_attention_close(fused, ref2, f"fused append, short rows with empty ones, chunks={chunks}")


@pytest.mark.parametrize("spike_at", [5, 70, 301, 590])
def test_score_spike_far_above_the_running_maximum(spike_at):
    """One key scores about 2^40 times higher than all the keys before it, so its probability
    against the running maximum would overflow fp16: the maximum has to follow it, in whichever
    lane group of its page the key sits and under every schedule."""
    print(f"decode score spike at key {spike_at}", flush=True)
    case = workloads.make_decode_case("spike", 90 + spike_at, [599, 130, 40], 16, 2, device=DEV)
    gen = torch.Generator().manual_seed(91)
    direction = torch.randn(workloads.HEAD_DIM, generator=gen)
    direction = direction / direction.norm()
    case.q.copy_((6.0 * direction + 0.3 * torch.randn(case.q.shape, generator=gen)).half())
    pool = 0.3 * torch.randn(case.kv_pool.shape, generator=gen)
    table = case.block_table.cpu()
    for b, at in ((0, spike_at), (1, min(spike_at, 100)), (2, 17)):
        slot = int(table[b, at // 16]) * 16 + at % 16
        pool[slot, :2] += 52.0 * direction          # K heads: 6 * 52 / sqrt(128) * log2(e), about +40
    case.kv_pool.copy_(pool.half())
    ref = _oracle(case)
    for kw in ({}, {"schedule": "balanced", "chunks": 7}, {"num_splits": 1}, {"num_splits": 5}):
        assert_attention_close(_run(case, **kw), ref, f"spike at {spike_at} {kw}")


def test_split_count_and_page_permutation_invariance():
    """Same logical KV under another physical page assignment and any split count."""
    print("decode invariance", flush=True)
    case = workloads.make_decode_case("inv", 91, [1500, 333, 2047, 64], 64, 8, device=DEV)
    ref = _oracle(case)
    base = _run(case, num_splits=1)
    assert_attention_close(base, ref, "inv base")
    for s in (2, 5, 16, 200):
        out = _run(case, num_splits=s)
        assert_attention_close(out, ref, f"inv splits={s}")
        assert float((out.float() - base.float()).abs().max()) <= 1e-3
    # move every page to a new physical location; logical content unchanged
    n = case.num_pages
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(5)).to(DEV)
    pool2 = torch.empty_like(case.kv_pool)
    pool2.view(n, -1)[perm] = case.kv_pool.view(n, -1)
    table2 = perm[case.block_table.long()].to(torch.int32)
    out2 = ops.paged_decode(case.q, pool2, table2, case.seq_lens, case.softmax_scale, num_splits=1)
    torch.cuda.synchronize()
    assert torch.equal(out2, base), "page permutation changed the result"


def test_deterministic_bitwise():
    print("decode determinism", flush=True)
    case = workloads.make_decode_case("det", 93, [3000, 4096, 257, 1024] * 4, 64, 8, device=DEV)
    a = _run(case)
    b = _run(case)
    assert torch.equal(a, b)


def test_closed_forms():
    """One token: out == v. Equal keys: out == mean(V) over the sequence."""
    print("decode closed forms", flush=True)
    case = workloads.make_decode_case("one", 95, [0, 0], 16, 8, device=DEV)
    out = _run(case, num_splits=1)
    for b in range(2):
        slot = int(case.block_table[b, 0]) * 16
        v = case.kv_pool[slot, 8:].float()                     # [Hkv, D]
        want = v.repeat_interleave(2, dim=0)
        assert float((out[b].float() - want).abs().max()) <= 1e-3
    case = workloads.make_decode_case("mean", 96, [199], 16, 8, device=DEV)
    n = int(case.seq_lens[0])
    slots = (case.block_table[0].long()[torch.arange(n, device=DEV) // 16] * 16 + torch.arange(n, device=DEV) % 16)
    case.kv_pool[slots, :8] = case.kv_pool[slots[0], :8]
    out = _run(case, num_splits=2)
    want = case.kv_pool[slots, 8:].float().mean(dim=0).repeat_interleave(2, dim=0)
    assert float((out[0].float() - want).abs().max()) <= 2e-3


def test_stages_can_be_called_separately():
    print("decode stages", flush=True)
    case = workloads.make_decode_case("stages", 97, [900, 2000, 100], 64, 8, device=DEV)
    both = _run(case, max_splits=8, min_pages_per_split=4)
    ws = ops.decode_workspace(case.batch, 64, 8, DEV)
    out = torch.zeros_like(both)
    ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale,
                     max_splits=8, min_pages_per_split=4, out=out, workspace=ws, stage="split")
    ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale,
                     max_splits=8, min_pages_per_split=4, out=out, workspace=ws, stage="merge")
    torch.cuda.synchronize()
    assert torch.equal(out, both)


def test_unwritten_tail_slots_do_not_leak():
    """NaN/Inf bit patterns in slots past the sequence end must not reach the output."""
    print("decode tail garbage", flush=True)
    case = workloads.make_decode_case("tail", 98, [20, 37], 16, 8, device=DEV)
    ref = _oracle(case)
    for b in range(2):
        n = int(case.seq_lens[b])
        page = int(case.block_table[b, (n - 1) // 16])
        case.kv_pool[page * 16 + n % 16: page * 16 + 16] = float("nan")
    assert_attention_close(_run(case, num_splits=1), ref, "tail NaN")


def test_invalid_arguments_raise():
    print("decode errors", flush=True)
    case = workloads.make_decode_case("err", 99, [10], 16, 8, device=DEV)
    from llama_lite_npu_amd._lib import LiteKVError
    with pytest.raises(LiteKVError, match="head_dim"):
        ops.paged_decode(case.q[..., :96].contiguous(), case.kv_pool[..., :96].contiguous(), case.block_table,
                         case.seq_lens)
    with pytest.raises(LiteKVError, match="workspace"):
        ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, max_splits=4,
                         min_pages_per_split=1, workspace=torch.empty(4, device=DEV))


def _shared_prefix_case(seed, hq, hkv, shared_pages, suffix_ctx, page_size=16):
    """Every block-table row starts with the same `shared_pages` pages; context = prefix + suffix."""
    ctx = [shared_pages * page_size + s for s in suffix_ctx]
    priv = [(c + 1 + page_size - 1) // page_size - shared_pages for c in ctx]
    num_pages = shared_pages + sum(priv) + 7
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(seed)).to(torch.int32)
    shared, cur, lists = perm[:shared_pages], shared_pages, []
    for n in priv:
        lists.append(torch.cat([shared, perm[cur:cur + n]]))
        cur += n
    return workloads.make_decode_case("shared", seed, ctx, hq, hkv, num_pages=num_pages, device=DEV,
                                      page_lists=lists, page_size=page_size)


@pytest.mark.parametrize("hq,hkv,shared_pages,suffix", [
    (64, 8, 13, [0, 5, 15, 16, 40, 300]),          # 208 prefix keys: not a multiple of the key tile
    (16, 8, 1, [3, 0, 90]),                        # one shared page
    (32, 4, 40, list(range(0, 170, 10))),          # 17 sequences x 8 heads: two column blocks
    (16, 1, 64, [1, 2, 3, 500]),                   # 16 query heads per kv head
    (28, 4, 9, [7, 0, 33, 64, 65]),                # 7 heads per kv head
])
def test_shared_prefix_decode(hq, hkv, shared_pages, suffix):
    """Pages common to all sequences attended once for the batch == the plain decode."""
    print(f"decode shared prefix {hq}/{hkv} pages={shared_pages}", flush=True)
    case = _shared_prefix_case(700 + hq + shared_pages, hq, hkv, shared_pages, suffix)
    ref = _oracle(case)
    for chunks in (None, 5):
        out = _run(case, schedule="balanced", chunks=chunks, shared_pages=shared_pages)
        assert_attention_close(out, ref, f"shared prefix {hq}/{hkv} chunks={chunks}")
    # fewer pages declared shared than really are: still the same attention
    out = _run(case, schedule="balanced", shared_pages=max(1, shared_pages // 2))
    assert_attention_close(out, ref, "shared prefix, half declared")


def test_shared_prefix_fused_append_and_empty_rows():
    """The fused append writes the same bits with a shared prefix; empty sequences give zero rows."""
    print("decode shared prefix + fused append", flush=True)
    case = _shared_prefix_case(760, 64, 8, 6, [0, 14, 15, 16, 31, 100, 7])
    pool_ref = case.kv_pool.clone()
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool_ref)
    lens = case.seq_lens.clone()
    lens[2] = 0
    plan = ops.DecodePlan(case.block_table, lens, 64, 8, case.num_pages, shared_pages=6)
    out = ops.decode_step(case.q, case.kv_pool, plan, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    keep = torch.ones(case.kv_pool.shape[0], dtype=torch.bool, device=DEV)
    keep[case.slot_mapping[2].long()] = False       # sequence 2 is empty: its row is not appended
    assert torch.equal(case.kv_pool[keep], pool_ref[keep])
    ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                lens.cpu().numpy(), case.softmax_scale)
    assert_attention_close(out, ref, "shared prefix + fused append")
    assert float(out[2].abs().max()) == 0.0


# ---- pools with pages of 32 to 256 tokens (the reference's --page_size, server.py:1038-1161;
# "typically 16-256", executor/paged_attention.py:27) ----

PAGE_SIZES = [32, 64, 128, 256]
EDGE_CONTEXTS = [0, 1, 15, 16, 17, 31, 32, 33, 47, 48, 63, 64, 65, 127, 128, 129, 255, 256, 257, 700, 1200]


@pytest.mark.parametrize("page_size", PAGE_SIZES)
@pytest.mark.parametrize("hq,hkv", [(64, 8), (16, 4), (8, 1)])
def test_page_sizes_every_schedule(page_size, hq, hkv):
    """Both schedules on a pool of larger pages: lengths that end on, before and after every
    16-token boundary inside a page and on the page boundary itself."""
    print(f"decode page_size {page_size} heads {hq}/{hkv}", flush=True)
    case = workloads.make_decode_case("pages", 300 + page_size + hq, EDGE_CONTEXTS, hq, hkv, device=DEV,
                                      page_size=page_size)
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, case.kv_pool)
    ref = _oracle(case)
    for kw in ({"num_splits": 1}, {"num_splits": 3}, {"max_splits": 16, "min_pages_per_split": 2},
               {"schedule": "balanced"}, {"schedule": "balanced", "chunks": 7},
               {"schedule": "balanced", "chunks": 1000}):
        print("  ", kw, flush=True)
        assert_attention_close(_run(case, **kw), ref, f"page_size {page_size} {hq}/{hkv} {kw}")


@pytest.mark.parametrize("page_size", PAGE_SIZES)
def test_page_sizes_fused_append_step(page_size):
    """The fused append on larger pages: pool bit exact with the append kernel, output as the oracle's;
    empty rows in between."""
    print(f"decode fused step, page_size {page_size}", flush=True)
    case = workloads.make_decode_case("pages-fused", 340 + page_size, EDGE_CONTEXTS, 32, 4, device=DEV,
                                      page_size=page_size)
    lens = case.seq_lens.clone()
    lens[3] = 0
    lens[9] = 0
    pool_ref = case.kv_pool.clone()
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool_ref)
    ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                lens.cpu().numpy(), case.softmax_scale, page_size=page_size)
    keep = torch.ones(case.kv_pool.shape[0], dtype=torch.bool, device=DEV)
    keep[case.slot_mapping[[3, 9]].long()] = False      # empty sequences append nothing
    for chunks in (None, 5):
        pool = case.kv_pool.clone()
        plan = ops.DecodePlan(case.block_table, lens, 32, 4, case.num_pages, chunks, page_size=page_size)
        out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale)
        torch.cuda.synchronize()
        assert torch.equal(pool[keep].view(torch.int16), pool_ref[keep].view(torch.int16)), "append not bit exact"
        assert_attention_close(out, ref, f"fused step page_size {page_size} chunks {chunks}")
        assert float(out[3].abs().max()) == 0.0 and float(out[9].abs().max()) == 0.0
    # the per-sequence schedule with its fused append
    pool = case.kv_pool.clone()
    out = ops.paged_decode(case.q, pool, case.block_table, lens, case.softmax_scale, num_splits=1,
                           page_size=page_size, k_new=case.k_new, v_new=case.v_new)
    torch.cuda.synchronize()
    assert torch.equal(pool[keep].view(torch.int16), pool_ref[keep].view(torch.int16))
    assert_attention_close(out, ref, f"per-sequence fused step page_size {page_size}")


@pytest.mark.parametrize("page_size", PAGE_SIZES)
@pytest.mark.parametrize("hq,hkv,shared_pages,suffix", [
    (64, 8, 5, [0, 5, 15, 16, 40, 300]),
    (16, 8, 1, [3, 0, 90]),
    (32, 4, 11, list(range(0, 170, 10))),
])
def test_page_sizes_shared_prefix(page_size, hq, hkv, shared_pages, suffix):
    print(f"decode shared prefix page_size {page_size} {hq}/{hkv} pages={shared_pages}", flush=True)
    case = _shared_prefix_case(800 + hq + shared_pages + page_size, hq, hkv, shared_pages, suffix, page_size)
    ref = _oracle(case)
    for chunks in (None, 5):
        out = _run(case, schedule="balanced", chunks=chunks, shared_pages=shared_pages)
        assert_attention_close(out, ref, f"shared prefix page_size {page_size} chunks={chunks}")


def test_unsupported_page_size_is_refused():
    from llama_lite_npu_amd._lib import LiteKVError
    case = workloads.make_decode_case("p48", 391, [40, 3, 90], 16, 8, device=DEV, page_size=48)
    with pytest.raises(LiteKVError, match="page_size"):
        ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, page_size=48, num_splits=1)
    with pytest.raises((LiteKVError, ValueError), match="page_size"):
        ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, page_size=48, schedule="balanced")


# ---- head dims other than 128 (the reference kernels take any block size, flashdecoding.py:305) ----

@pytest.mark.parametrize("head_dim", [64, 32, 256])
@pytest.mark.parametrize("hq,hkv,page_size", [(64, 8, 16), (14, 2, 16), (16, 4, 64), (8, 8, 32)])
def test_head_dims_every_schedule(head_dim, hq, hkv, page_size):
    """Decode at head dims 32, 64 and 256 through every entry point: both schedules, the plan made
    on the device, the fused append, a shared prefix, empty rows."""
    print(f"decode head_dim {head_dim} heads {hq}/{hkv} page_size {page_size}", flush=True)
    case = workloads.make_decode_case("dims", 500 + head_dim + hq, [0, 1, 15, 16, 17, 63, 64, 65, 255, 700], hq, hkv,
                                      device=DEV, page_size=page_size, head_dim=head_dim)
    lens = case.seq_lens.clone()
    lens[4] = 0
    pool_ref = case.kv_pool.clone()
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool_ref)
    ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                lens.cpu().numpy(), case.softmax_scale, page_size=page_size)
    for kw in ({"num_splits": 1}, {"num_splits": 3}, {"schedule": "balanced"}, {"schedule": "balanced", "chunks": 7}):
        out = ops.paged_decode(case.q, pool_ref, case.block_table, lens, case.softmax_scale, page_size=page_size, **kw)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"head_dim {head_dim} {kw}")
        assert float(out[4].abs().max()) == 0.0
    keep = torch.ones(case.kv_pool.shape[0], dtype=torch.bool, device=DEV)
    keep[case.slot_mapping[4].long()] = False           # the empty sequence appends nothing
    # fused append, balanced entry (page ids from the plan) and per-sequence entry
    pool = case.kv_pool.clone()
    plan = ops.DecodePlan(case.block_table, lens, hq, hkv, case.num_pages, 5, page_size=page_size)
    out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(pool[keep].view(torch.int16), pool_ref[keep].view(torch.int16))
    assert_attention_close(out, ref, f"head_dim {head_dim} fused step")
    pool = case.kv_pool.clone()
    out = ops.paged_decode(case.q, pool, case.block_table, lens, case.softmax_scale, num_splits=1,
                           page_size=page_size, k_new=case.k_new, v_new=case.v_new)
    torch.cuda.synchronize()
    assert torch.equal(pool[keep].view(torch.int16), pool_ref[keep].view(torch.int16))
    assert_attention_close(out, ref, f"head_dim {head_dim} per-sequence fused step")


@pytest.mark.parametrize("head_dim", [64, 256])
def test_head_dims_shared_prefix(head_dim):
    print(f"decode shared prefix head_dim {head_dim}", flush=True)
    shared_pages, suffix = 5, [0, 5, 15, 16, 40, 300]
    ctx = [shared_pages * 16 + s for s in suffix]
    priv = [(c + 1 + 15) // 16 - shared_pages for c in ctx]
    num_pages = shared_pages + sum(priv) + 7
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(head_dim)).to(torch.int32)
    shared, cur, lists = perm[:shared_pages], shared_pages, []
    for n in priv:
        lists.append(torch.cat([shared, perm[cur:cur + n]]))
        cur += n
    case = workloads.make_decode_case("shared-dims", 560 + head_dim, ctx, 32, 4, num_pages=num_pages, device=DEV,
                                      page_lists=lists, head_dim=head_dim)
    ref = _oracle(case)
    out = _run(case, schedule="balanced", shared_pages=shared_pages)
    assert_attention_close(out, ref, f"shared prefix head_dim {head_dim}")


def test_head_dim_64_at_a_larger_size():
    """Head dim 64 on the MFMA kernels at a size where chunks cross many sequences and sequences
    span many chunks: both schedules against the oracle, fused append bit exact, repeatable."""
    print("decode head_dim 64, larger batch", flush=True)
    lens = workloads.uniform_lens(641, 24, 1, 3000) + [0, 15, 16, 4095]
    case = workloads.make_decode_case("d64-large", 642, lens, 32, 8, device=DEV, head_dim=64)
    pool_ref = case.kv_pool.clone()
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool_ref)
    ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                case.seq_lens.cpu().numpy(), case.softmax_scale)
    plan = ops.DecodePlan(case.block_table, case.seq_lens, 32, 8, case.num_pages)
    pool = case.kv_pool.clone()
    out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale)
    again = ops.decode_step(case.q, pool, plan, None, None, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(pool.view(torch.int16), pool_ref.view(torch.int16))
    assert_attention_close(out, ref, "head_dim 64 balanced, fused append")
    assert_attention_close(again, ref, "head_dim 64 balanced")
    for kw in ({"num_splits": 1}, {"num_splits": 5}, {"max_splits": 16, "min_pages_per_split": 4},
               {"schedule": "balanced", "chunks": 37}):
        got = ops.paged_decode(case.q, pool_ref, case.block_table, case.seq_lens, case.softmax_scale, **kw)
        torch.cuda.synchronize()
        assert_attention_close(got, ref, f"head_dim 64 {kw}")


@pytest.mark.parametrize("page_size,shared_tokens", [(16, 1040), (32, 640), (64, 2048)])
def test_head_dim_64_long_shared_prefix(page_size, shared_tokens):
    """Head dim 64 behind a long shared prefix: the prefix goes through the tiled prefix kernel in
    several key slices, the private pages through the balanced kernel, and the merge joins them."""
    print(f"decode head_dim 64 shared prefix of {shared_tokens} tokens, page_size {page_size}", flush=True)
    shared_pages = shared_tokens // page_size
    suffix = [0, 1, page_size - 1, page_size, 3 * page_size + 5, 700, 64, 333]
    ctx = [shared_tokens + s for s in suffix]
    priv = [(c + 1 + page_size - 1) // page_size - shared_pages for c in ctx]
    num_pages = shared_pages + sum(priv) + 5
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(page_size)).to(torch.int32)
    shared, cur, lists = perm[:shared_pages], shared_pages, []
    for n in priv:
        lists.append(torch.cat([shared, perm[cur:cur + n]]))
        cur += n
    case = workloads.make_decode_case("shared-64", 1560 + page_size, ctx, 32, 8, num_pages=num_pages, device=DEV,
                                      page_lists=lists, head_dim=64, page_size=page_size)
    ref = _oracle(case)
    out = _run(case, schedule="balanced", shared_pages=shared_pages)
    assert_attention_close(out, ref, "shared prefix at head_dim 64")
    partly = _run(case, schedule="balanced", shared_pages=shared_pages // 2)
    assert_attention_close(partly, ref, "half the shared prefix declared, head_dim 64")
    assert torch.equal(out, _run(case, schedule="balanced", shared_pages=shared_pages))


# ---- more than 16 query heads per kv head (the reference's grid is per query head,
# flashdecoding.py:44, 170-175: no bound on the group) ----

@pytest.mark.parametrize("head_dim", [128, 64, 32])
@pytest.mark.parametrize("hq,hkv", [(32, 1), (64, 2), (96, 4), (20, 1), (51, 3), (64, 1)])
def test_more_than_16_query_heads_per_kv_head(head_dim, hq, hkv):
    """Groups of 17 to 32 query heads run as two slices of their kv head (up to 16 columns each):
    both schedules, the fused append (written once per slice, the same bits), a shared prefix."""
    print(f"decode {hq}/{hkv} heads, head_dim {head_dim}", flush=True)
    lens = [0, 1, 15, 16, 17, 255, 256, 700, 40]
    case = workloads.make_decode_case("wide-group", 1700 + hq + head_dim, lens, hq, hkv, device=DEV,
                                      head_dim=head_dim)
    seq = case.seq_lens.clone()
    seq[8] = 0
    pool_ref = case.kv_pool.clone()
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, pool_ref)
    ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                seq.cpu().numpy(), case.softmax_scale)
    keep = torch.ones(case.kv_pool.shape[0], dtype=torch.bool, device=DEV)
    keep[case.slot_mapping[8].long()] = False           # the empty sequence appends nothing
    for kw in ({"num_splits": 1}, {"num_splits": 3}, {"max_splits": 16, "min_pages_per_split": 2},
               {"schedule": "balanced"}, {"schedule": "balanced", "chunks": 5}):
        out = ops.paged_decode(case.q, pool_ref, case.block_table, seq, case.softmax_scale, **kw)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"{hq}/{hkv} d={head_dim} {kw}")
        assert float(out[8].abs().max()) == 0.0
    for chunks in (None, 3):
        pool = case.kv_pool.clone()
        plan = ops.DecodePlan(case.block_table, seq, hq, hkv, case.num_pages, chunks)
        out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale)
        torch.cuda.synchronize()
        assert torch.equal(pool[keep].view(torch.int16), pool_ref[keep].view(torch.int16))
        assert_attention_close(out, ref, f"{hq}/{hkv} d={head_dim} fused step chunks={chunks}")
    pool = case.kv_pool.clone()
    out = ops.paged_decode(case.q, pool, case.block_table, seq, case.softmax_scale, num_splits=1,
                           k_new=case.k_new, v_new=case.v_new)
    torch.cuda.synchronize()
    assert torch.equal(pool[keep].view(torch.int16), pool_ref[keep].view(torch.int16))
    assert_attention_close(out, ref, f"{hq}/{hkv} d={head_dim} per-sequence fused step")


@pytest.mark.parametrize("head_dim", [128, 64])
def test_more_than_16_query_heads_per_kv_head_behind_a_shared_prefix(head_dim):
    print(f"decode 64/2 heads behind a shared prefix, head_dim {head_dim}", flush=True)
    shared_pages, suffix = 13, [0, 5, 15, 16, 40, 300]
    ctx = [shared_pages * 16 + s for s in suffix]
    priv = [(c + 1 + 15) // 16 - shared_pages for c in ctx]
    num_pages = shared_pages + sum(priv) + 7
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(head_dim + 3)).to(torch.int32)
    shared, cur, lists = perm[:shared_pages], shared_pages, []
    for n in priv:
        lists.append(torch.cat([shared, perm[cur:cur + n]]))
        cur += n
    case = workloads.make_decode_case("wide-shared", 1760 + head_dim, ctx, 64, 2, num_pages=num_pages, device=DEV,
                                      page_lists=lists, head_dim=head_dim)
    ref = _oracle(case)
    for chunks in (None, 5):
        out = _run(case, schedule="balanced", chunks=chunks, shared_pages=shared_pages)
        assert_attention_close(out, ref, f"64/2 shared prefix d={head_dim} chunks={chunks}")


# ---- a length beyond what the block table can name (lengths live on the device: no host check) ----

@pytest.mark.parametrize("head_dim", [128, 32])
def test_length_beyond_the_block_table_row_touches_no_other_page(head_dim):
    """Sequence 1 claims 100 tokens against a table whose rows name 4 pages (64 tokens): the
    kernels re-read the row's last entry instead of reading past the row, and the fused append
    writes nothing for it; the other sequences are attended and appended as usual."""
    print(f"decode length beyond the table, head_dim {head_dim}", flush=True)
    hq, hkv = 16, 4
    case = workloads.make_decode_case("beyond", 1790 + head_dim, [39, 63, 63, 20], hq, hkv, device=DEV,
                                      head_dim=head_dim)
    assert case.block_table.shape[1] == 4
    seq = case.seq_lens.clone()
    seq[1] = 100
    good = [0, 2, 3]
    pool_ref = case.kv_pool.clone()
    ops.kv_append(case.k_new[good], case.v_new[good], case.slot_mapping[good], pool_ref)
    ref = c_oracle.paged_decode(to_np16(case.q), to_np16(pool_ref), case.block_table.cpu().numpy(),
                                case.seq_lens.cpu().numpy(), case.softmax_scale)
    for kw in ({"num_splits": 1}, {"num_splits": 3}):
        pool = case.kv_pool.clone()
        out = ops.paged_decode(case.q, pool, case.block_table, seq, case.softmax_scale, k_new=case.k_new,
                               v_new=case.v_new, **kw)
        torch.cuda.synchronize()
        assert torch.equal(pool.view(torch.int16), pool_ref.view(torch.int16)), f"pool changed elsewhere {kw}"
        assert_attention_close(out[good], ref[good], f"length beyond the table {kw}")
        assert bool(torch.isfinite(out).all())
    pool = case.kv_pool.clone()
    plan = ops.DecodePlan(case.block_table, seq, hq, hkv, case.num_pages, 3)
    out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(pool.view(torch.int16), pool_ref.view(torch.int16)), "pool changed elsewhere (balanced)"
    assert_attention_close(out[good], ref[good], "length beyond the table, balanced")


@pytest.mark.parametrize("hq,hkv,fused", [(64, 8, False), (32, 4, True), (16, 8, False)])
def test_split_schedule_dispatched_longest_first(hq, hkv, fused):
    """A split launch with more workgroups than the device holds at once walks the sequences from
    the longest down. Which workgroup attends which sequence must not show in the result: every
    row equals, bit for bit, the row of the same sequence decoded in a batch of one (no ordering,
    the same split boundaries); lengths with ties, empty rows and one-token rows among them."""
    print(f"decode splits, longest first {hq}/{hkv} fused={fused}", flush=True)
    lens = [(37 * i * i + 11 * i) % 900 for i in range(96)]
    for i in (3, 40, 41, 77):
        lens[i] = 0                                  # empty rows
    lens[10] = lens[11] = lens[60] = 512             # ties
    lens[20] = 1
    case = workloads.make_decode_case("lpt", 4100 + hq, lens, hq, hkv, device=DEV)
    pool0 = case.kv_pool.clone()
    ops.kv_append(case.k_new, case.v_new, case.slot_mapping, case.kv_pool)
    for i in (3, 40, 41, 77):
        case.seq_lens[i] = 0
    ref = _oracle(case)
    kw = dict(max_splits=16, min_pages_per_split=1)
    if fused:
        pool = pool0.clone()
        out = ops.paged_decode(case.q, pool, case.block_table, case.seq_lens, case.softmax_scale,
                               k_new=case.k_new, v_new=case.v_new, **kw)
        torch.cuda.synchronize()
        live = case.seq_lens > 0
        slots = case.slot_mapping[live].long()
        assert torch.equal(pool[slots].view(torch.int16), case.kv_pool[slots].view(torch.int16))
    else:
        out = _run(case, **kw)
    assert_attention_close(out, ref, "splits, longest first")
    for b in (0, 10, 11, 20, 41, 60, 95, max(range(96), key=lambda i: lens[i])):
        alone = ops.paged_decode(case.q[b:b + 1].contiguous(), case.kv_pool, case.block_table[b:b + 1].contiguous(),
                                 case.seq_lens[b:b + 1].contiguous(), case.softmax_scale, **kw)
        torch.cuda.synchronize()
        assert torch.equal(alone[0], out[b]), f"sequence {b} of length {int(case.seq_lens[b])}"


def test_prefix_chunk_count_leaves_room_for_the_prefix_role():
    """The chunk count a plan takes for a step behind a shared prefix: the compute units the
    prefix workgroups leave, less a sixteenth of the device, never under a quarter of it; shapes
    the helper cannot judge get the plain balanced count."""
    print("decode prefix chunk count", flush=True)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    plain = ops.balanced_chunks(8)
    c4 = ops.prefix_chunks(64, 64, 8, 128)
    assert c4 == cus - 64 - cus // 16                     # 64 prefix workgroups of 8 wavefronts on this shape
    small = ops.prefix_chunks(2, 8, 8, 128)               # too few columns for wide workgroups
    assert cus // 4 <= small <= cus
    assert ops.prefix_chunks(64, 64, 8, 8, page_size=256) == c4      # 8 pages of 256 tokens are the same 2048 keys
    eight_bit = ops.prefix_chunks(64, 64, 8, 128, fp16_pool=False)
    assert cus // 4 <= eight_bit <= cus
    assert ops.prefix_chunks(64, 64, 8, 0) == plain       # no shared pages: the plain count
    assert ops.prefix_chunks(64, 64, 8, 128, page_size=48) == plain
    plan = ops.DecodePlan(torch.zeros((64, 160), dtype=torch.int32, device=DEV),
                          torch.full((64,), 2100, dtype=torch.int32, device=DEV), 64, 8, 4096,
                          shared_pages=128, kv_dtype=torch.float16)
    assert plan.chunks == c4


@pytest.mark.parametrize("head_dim", [128, 64])
@pytest.mark.parametrize("hq,hkv", [(64, 8), (16, 2)])
def test_few_long_sequences_merge_their_many_pieces(hq, hkv, head_dim):
    """One to three long sequences on the balanced schedule: each spans far more than 16 chunks,
    and with so few rows the merge shares every row's elements out among several workgroups (more
    than 256 pieces: several sweeps). A short and an empty sequence ride along (fewer pieces: the
    ordinary paths of the same launch). Against the oracle, and twice bit for bit; nine such
    sequences take the one-workgroup-per-row merge of long rows."""
    for lens, chunks in (([9000], None), ([5000, 70, 0, 4100], None), ([9000, 3000, 33], 700), ([2600] * 9, None)):
        print(f"long rows {hq}/{hkv} d{head_dim} lens {lens} chunks {chunks}", flush=True)
        case = workloads.make_decode_case("long", 1300 + hq + head_dim, lens, hq, hkv, device=DEV, head_dim=head_dim)
        ops.kv_append(case.k_new, case.v_new, case.slot_mapping, case.kv_pool)
        for i, n in enumerate(lens):
            if n == 0:
                case.seq_lens[i] = 0
        ref = _oracle(case)
        kw = dict(schedule="balanced") if chunks is None else dict(schedule="balanced", chunks=chunks)
        out = _run(case, **kw)
        again = _run(case, **kw)
        assert torch.equal(out, again)
        assert_attention_close(out, ref, f"long rows {lens}")
