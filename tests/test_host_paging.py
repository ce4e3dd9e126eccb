"""Page pool, request tables and executor metadata on the CPU: the integer examples held by the
reference's tests (tests/test_decode_p0.py:48-113, tests/test_paged_attention_refcount.py:28-135,
tests/test_continuous_batching.py:524-553) and its worked token-table example
(lite_llama/executor/paged_attention.py:125-129), re-expressed against this package's classes."""

import pytest
import torch

from llama_lite_npu_amd.executor import ModelExecutor, PagedKVCacheManager, PagedReqTokensManager


def _managers(num_pages=4, max_requests=1, max_seq_len=16, page_size=4):
    page_mgr = PagedKVCacheManager(num_layers=1, num_kv_heads=1, head_dim=8, num_pages=num_pages,
                                   page_size=page_size, dtype=torch.float16, device="cpu")
    req_mgr = PagedReqTokensManager(max_requests=max_requests, max_seq_len=max_seq_len, page_manager=page_mgr,
                                    device="cpu")
    return page_mgr, req_mgr


def test_token_table_worked_example():
    page_mgr, _ = _managers(num_pages=16)
    table = torch.zeros((2, 16), dtype=torch.int32)
    mapped = page_mgr.build_token_table(torch.tensor([3, 7, 12]), 10, table, 1)
    assert mapped == 10
    assert table[1, :10].tolist() == [12, 13, 14, 15, 28, 29, 30, 31, 48, 49]
    assert page_mgr.slots_of([3, 7, 12], 10).tolist() == [12, 13, 14, 15, 28, 29, 30, 31, 48, 49]


def test_extend_updates_only_new_mapping():
    page_mgr, req_mgr = _managers()
    assert req_mgr.alloc_req(0, 3)
    page_mgr.build_token_table = None   # a full rebuild would crash
    assert req_mgr.extend_req(0, 1)
    assert req_mgr.req_token_count[0] == 4
    assert req_mgr.b_req_tokens_table[0, :4].tolist() == [0, 1, 2, 3]
    assert req_mgr.block_table[0, 0].item() == 0


def test_extend_across_page_boundary_maps_new_page():
    _, req_mgr = _managers()
    assert req_mgr.alloc_req(0, 4)
    assert req_mgr.extend_req(0, 1)
    assert len(req_mgr.req_page_table[0]) == 2
    assert req_mgr.b_req_tokens_table[0, 4].item() == 4
    assert req_mgr.block_table[0, :2].tolist() == [0, 1]


def test_reserve_req_assigns_and_reuses_request_id():
    _, req_mgr = _managers()
    first = req_mgr.reserve_req(3)
    assert first == 0
    assert req_mgr.reserve_req(1) is None
    req_mgr.free_req(first)
    reused = req_mgr.reserve_req(2)
    assert reused == 0 and req_mgr.req_token_count[reused] == 2


def test_batch_metadata_uses_each_request_length_and_last_token():
    _, req_mgr = _managers(num_pages=8, max_requests=2)
    assert req_mgr.alloc_req(0, 3) and req_mgr.alloc_req(1, 5)
    req_ids, seq_lens, last = req_mgr.batch_metadata([1, 0])
    assert req_ids.tolist() == [1, 0] and req_ids.dtype == torch.int32
    assert seq_lens.tolist() == [5, 3] and seq_lens.dtype == torch.long
    table = req_mgr.b_req_tokens_table
    assert last.tolist() == [table[1, 4].item(), table[0, 2].item()]
    with pytest.raises(ValueError):
        req_mgr.batch_metadata([])
    with pytest.raises(KeyError):
        req_mgr.batch_metadata([5])


def test_shared_page_is_not_returned_to_free_pool_until_last_ref():
    manager, _ = _managers()
    pages = manager.alloc(4)
    assert manager.num_free_pages == 3
    manager.add_ref(pages)
    assert int(manager.page_refcount[pages[0]]) == 2
    manager.free(pages)
    assert manager.num_free_pages == 3 and not bool(manager.page_free[pages[0]])
    manager.free(pages)
    assert manager.num_free_pages == 4 and bool(manager.page_free[pages[0]])
    with pytest.raises(ValueError):
        manager.free(pages)
    with pytest.raises(ValueError):
        manager.add_ref(pages)


def test_alloc_hands_out_lowest_free_ids_and_fails_cleanly():
    manager, _ = _managers(num_pages=6)
    a = manager.alloc(9)              # 3 pages
    assert a.tolist() == [0, 1, 2]
    b = manager.alloc(4)
    assert b.tolist() == [3]
    manager.free(a[1:2])
    assert manager.alloc(4).tolist() == [1]
    assert manager.alloc(100) is None and manager.num_free_pages == 2
    manager.free_all()
    assert manager.num_free_pages == 6 and manager.alloc(4).tolist() == [0]


def test_request_pages_returns_host_page_ids():
    _, req_mgr = _managers(max_requests=2)
    assert req_mgr.alloc_req(0, 5)
    pages = req_mgr.request_pages(0)
    assert len(pages) == 2 and all(isinstance(p, int) for p in pages)
    with pytest.raises(KeyError):
        req_mgr.request_pages(1)


def test_reserved_capacity_does_not_advance_logical_length():
    page_mgr, req_mgr = _managers(max_requests=2)
    req_idx = req_mgr.reserve_req(num_tokens=1, reserved_tokens=9)
    assert req_idx == 0 and req_mgr.req_token_count[0] == 1
    assert len(req_mgr.req_page_table[0]) == 3 and page_mgr.num_free_pages == 1
    assert req_mgr.extend_req(0, 8)
    assert req_mgr.req_token_count[0] == 9 and len(req_mgr.req_page_table[0]) == 3
    assert page_mgr.num_free_pages == 1
    assert req_mgr.get_token_indices(0, 9).tolist() == list(range(9))


def test_share_req_from_pages_reuses_existing_pages_with_refcounts():
    page_mgr, req_mgr = _managers(max_requests=2)
    assert req_mgr.alloc_req(0, 5)
    pages = req_mgr.req_page_table[0]
    assert req_mgr.share_req_from_pages(1, pages, 5)
    assert req_mgr.get_token_indices(1, 5).tolist() == [0, 1, 2, 3, 4]
    assert int(page_mgr.page_refcount[pages[0]]) == 2
    req_mgr.free_req(0)
    assert not bool(page_mgr.page_free[pages[0]])
    req_mgr.free_req(1)
    assert bool(page_mgr.page_free[pages[0]])


def test_capacity_and_length_failures_are_distinct_and_side_effect_free():
    page_mgr, req_mgr = _managers(num_pages=2, max_requests=2, max_seq_len=8)
    assert not req_mgr.alloc_req(0, 9)                       # beyond max_seq_len
    assert not req_mgr.alloc_req(0, 0)
    assert not req_mgr.alloc_req(0, 4, reserved_tokens=2)    # capacity below length
    assert page_mgr.num_free_pages == 2 and req_mgr.free_req_indices == [0, 1]
    assert req_mgr.alloc_req(0, 8)
    assert not req_mgr.alloc_req(1, 1)                       # pool exhausted
    assert not req_mgr.extend_req(0, 1)                      # would exceed max_seq_len
    assert req_mgr.req_token_count[0] == 8
    assert req_mgr.ensure_req_capacity(0, 4) and not req_mgr.ensure_req_capacity(0, 9)
    assert not req_mgr.ensure_req_capacity(1, 4)


def _executor(num_pages=16, max_seq_len=32, max_requests=4, page_size=4):
    return ModelExecutor(num_layers=1, num_q_heads=2, num_kv_heads=1, head_dim=8, num_pages=num_pages,
                         max_seq_len=max_seq_len, max_requests=max_requests, page_size=page_size, device="cpu")


def test_packed_prefill_metadata():
    ex = _executor()
    ids = ex.reserve_paged_requests([2, 1, 2])
    assert ids == (0, 1, 2)
    positions, sample = ex.activate_paged_packed_prefill_batch(ids, [2, 1, 2])
    info = ex.atten_info
    assert info.b_start_loc.tolist() == [0, 2, 3]
    assert positions.tolist() == [0, 1, 0, 0, 1] and sample.tolist() == [1, 2, 4]
    assert info.b_seq_len.tolist() == [2, 1, 2] and info.b_seq_len.dtype == torch.long
    assert info.cu_q_lens.tolist() == [0, 2, 3, 5]
    # each request got its own page (page_size 4): slots page*4 + offset
    assert info.cur_select_index.tolist() == [0, 1, 4, 8, 9]
    assert info.block_table.tolist() == [[0], [1], [2]]
    assert info.max_actual_seq_len == 2 and not info.is_paged_chunk_prefill
    with pytest.raises(ValueError, match="length mismatch"):
        ex.activate_paged_packed_prefill_batch(ids, [2, 2, 2])


def test_chunk_prefill_and_decode_metadata():
    ex = _executor()
    (rid,) = ex.reserve_paged_requests([3], reserved_lengths=[10])
    ex.activate_paged_packed_prefill_batch((rid,), [3])
    positions, sample = ex.activate_paged_chunk_prefill_batch((rid,), [3], [4])
    info = ex.atten_info
    assert info.is_paged_chunk_prefill and info.max_actual_q_seq_len == 4
    assert positions.tolist() == [3, 4, 5, 6] and sample.tolist() == [3]
    assert info.chunk_context_len.tolist() == [3] and info.chunk_q_seq_len.tolist() == [4]
    assert info.b_seq_len.tolist() == [7] and info.cur_select_index.tolist() == [3, 4, 5, 6]
    with pytest.raises(ValueError, match="context length mismatch"):
        ex.activate_paged_chunk_prefill_batch((rid,), [3], [1])
    ex.extend_paged_requests((rid,))
    info = ex.atten_info
    assert not info.is_paged_chunk_prefill and info.b_seq_len.tolist() == [8]
    assert info.cur_select_index.tolist() == [7] and info.max_actual_seq_len == 8
    assert info.cu_q_lens.tolist() == [0, 1]
    ex.release_paged_request_ids((rid,))
    assert ex.kv_mem_manager.num_free_pages == 16


def test_reservation_rolls_back_and_reports_exhaustion():
    ex = _executor(num_pages=3)
    with pytest.raises(RuntimeError, match="capacity is exhausted"):
        ex.reserve_paged_requests([4, 4, 4, 4])
    assert ex.kv_mem_manager.num_free_pages == 3 and ex.req_tokens_manager.free_req_indices == [0, 1, 2, 3]
    (rid,) = ex.reserve_paged_requests([12])
    with pytest.raises(RuntimeError, match="Paged KV allocation failed for request"):
        ex.extend_paged_requests((rid,))


def test_prefix_cache_exact_and_block_hits_hold_page_references():
    ex = _executor()
    prompt = tuple(range(100, 110))                      # 10 tokens, page_size 4: 2 full blocks + 2
    (rid,) = ex.reserve_paged_requests([10])
    ex.store_paged_request_prefix(prompt, rid, first_token_id=7)
    pages = ex.req_tokens_manager.request_pages(rid)
    mgr = ex.kv_mem_manager
    assert [mgr.refcount(p) for p in pages] == [3, 3, 2]  # request + exact entry (+ block entry)
    hit = ex.share_paged_request_from_cache(prompt)
    assert hit == (1, 7)
    assert ex.req_tokens_manager.request_pages(1) == pages
    part = ex.share_paged_prefix_from_cache(prompt[:8] + (1, 2, 3))
    assert part == (2, 8, None)                          # two full blocks matched, suffix to replay
    assert ex.req_tokens_manager.request_pages(2) == pages[:2]
    assert ex.share_paged_prefix_from_cache((5, 5, 5, 5, 5)) is None
    ex.release_paged_request_ids((0, 1, 2))
    assert [mgr.refcount(p) for p in pages] == [2, 2, 1]  # the caches keep the pages alive


def test_compaction_plan_moves_high_pages_into_holes(monkeypatch):
    ex = _executor(num_pages=8, max_requests=4)
    ids = ex.reserve_paged_requests([4, 4, 4, 4, ][:4])   # pages 0..3
    ex.req_tokens_manager.extend_req(ids[3], 8)           # request 3 now owns pages 3, 4, 5
    ex.release_paged_request_ids((ids[0], ids[2]))        # holes at 0 and 2; live = {1, 3, 4, 5}
    moved = []
    monkeypatch.setattr(ex.kv_mem_manager, "copy_pages", lambda s, d: moved.append((list(s), list(d))))
    moves = ex.compact_kv_pool()
    assert moves == [(4, 0), (5, 2)] and moved == [([4, 5], [0, 2])]
    assert ex.req_tokens_manager.request_pages(ids[3]) == (3, 0, 2)
    assert ex.req_tokens_manager.request_pages(ids[1]) == (1,)
    mgr = ex.kv_mem_manager
    assert mgr.page_free.tolist() == [False, False, False, False, True, True, True, True]
    assert mgr.alloc(4).tolist() == [4]
    assert ex.req_tokens_manager.block_table[ids[3], :3].tolist() == [3, 0, 2]


def test_copy_on_write_leaves_the_page_to_its_last_holder(monkeypatch):
    """Two requests share a partly filled page that nobody else holds: one of them moves to a
    private copy, the other keeps the page (one allocation, one copy). A full last page and
    reserved pages behind the logical end are left alone."""
    page_mgr, req_mgr = _managers(num_pages=6, max_requests=4, max_seq_len=16)
    copies = []
    monkeypatch.setattr(page_mgr, "copy_pages", lambda s, d: copies.append((list(s), list(d))))
    assert req_mgr.alloc_req(0, 6)                                   # pages 0, 1; page 1 holds 2 of 4 tokens
    pages = req_mgr.req_page_table[0]
    assert req_mgr.share_req_from_pages(1, pages, 6)
    moves = req_mgr.copy_on_write((0, 1))
    assert moves == [(1, 2)] and copies == [([1], [2])]
    assert req_mgr.request_pages(0) == (0, 2) and req_mgr.request_pages(1) == (0, 1)
    assert int(page_mgr.page_refcount[1]) == 1 and int(page_mgr.page_refcount[2]) == 1
    assert int(page_mgr.page_refcount[0]) == 2
    assert req_mgr.copy_on_write((0, 1)) == []                       # now private: nothing left to do
    # a full last page: the next token opens a new page, the shared one is never written
    assert req_mgr.alloc_req(2, 4)                                   # page 3, full
    assert req_mgr.share_req_from_pages(3, req_mgr.req_page_table[2], 4)
    assert req_mgr.copy_on_write((2, 3)) == [] and len(copies) == 1
    # reserved pages behind the logical end are not the page the next token goes into
    req_mgr.free_req(3)
    req_mgr.free_req(2)
    assert req_mgr.alloc_req(2, 2, 8)                                # 2 tokens, two pages reserved
    first = req_mgr.req_page_table[2][:1]
    assert req_mgr.share_req_from_pages(3, first, 2)
    (move,) = req_mgr.copy_on_write((3,))
    assert move[0] == int(first[0])


def test_shared_prefix_pages_counts_full_common_pages():
    """Requests that map the same cached pages (block prefix cache) share them in a decode step;
    the page receiving a request's next token never counts."""
    ex = _executor(num_pages=32, max_seq_len=64, max_requests=4, page_size=4)
    ex.shared_prefix_min_pages = 2
    system = tuple(range(100, 112))                      # 3 full pages of 4 tokens
    (a,) = ex.reserve_paged_requests([12])
    ex.activate_paged_packed_prefill_batch((a,), [12])
    ex.store_paged_request_prefix(system, a, first_token_id=1)
    b, matched, first = ex.share_paged_prefix_from_cache(system + (7, 8, 9))
    assert (matched, first) == (12, None)
    ex.ensure_paged_request_capacity(b, 20)
    ex.activate_paged_chunk_prefill_batch((b,), [12], [3])
    pages_a, pages_b = ex.req_tokens_manager.request_pages(a), ex.req_tokens_manager.request_pages(b)
    assert pages_a[:3] == pages_b[:3]
    assert ex.shared_prefix_pages((a,)) == 0             # nothing to share with
    assert ex.shared_prefix_pages((a, b)) == 2           # a holds 12 tokens: its page 2 takes no part yet
    ex.extend_paged_requests((a, b))                     # a -> 13 tokens on a private 4th page
    assert ex.shared_prefix_pages((a, b)) == 3
    ex.shared_prefix_min_pages = 4
    assert ex.shared_prefix_pages((a, b)) == 0           # too short to pay for the extra launches
