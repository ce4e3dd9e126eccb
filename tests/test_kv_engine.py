"""Host scheduling metadata: the integer examples the reference's own tests hold for
lite_llama/kv_engine.py (tests/test_kv_engine.py:19-87), plus edge cases."""

import pytest

from llama_lite_npu_amd import kv_engine as kv


def test_ref_counter_acquire_release():
    refs = kv.KVBlockRefCounter(total_blocks=4)
    assert refs.acquire(2) == (0, 1)
    assert refs.refcount(0) == 1 and refs.available_count == 2
    refs.add_ref((0,))
    assert refs.refcount(0) == 2
    refs.release((0, 1))
    assert refs.refcount(0) == 1 and refs.refcount(1) == 0 and refs.available_count == 3
    # lowest free id first, also after a release out of order
    assert refs.acquire(2) == (1, 2)


def test_ref_counter_errors():
    refs = kv.KVBlockRefCounter(total_blocks=1)
    with pytest.raises(ValueError):
        refs.release((0,))
    with pytest.raises(ValueError):
        refs.add_ref((0,))
    with pytest.raises(IndexError):
        refs.refcount(3)
    with pytest.raises(ValueError):
        kv.KVBlockRefCounter(0)
    refs.acquire(1)
    with pytest.raises(RuntimeError, match="insufficient KV blocks"):
        refs.acquire(1)


def test_prefix_cache_longest_block_aligned_match():
    cache = kv.PrefixCache(block_size=4)
    cache.put((1, 2, 3, 4, 5, 6, 7, 8), (10, 11))
    m = cache.match((1, 2, 3, 4, 5, 6, 9, 9))
    assert m.matched_tokens == 4 and m.block_ids == (10,)
    full = cache.match((1, 2, 3, 4, 5, 6, 7, 8, 1))
    assert full.matched_tokens == 8 and full.block_ids == (10, 11)


def test_prefix_cache_ignores_partial_blocks():
    cache = kv.PrefixCache(block_size=4)
    cache.put((1, 2, 3), (10,))
    m = cache.match((1, 2, 3, 4))
    assert m.matched_tokens == 0 and m.block_ids == ()
    with pytest.raises(ValueError):
        cache.put((1, 2, 3, 4, 5, 6, 7, 8), (1,))
    with pytest.raises(ValueError):
        kv.PrefixCache(0)


def test_chunked_prefill_planner():
    chunks = kv.ChunkedPrefillPlanner(chunk_size=4).plan(prompt_length=10)
    assert [(c.start, c.end) for c in chunks] == [(0, 4), (4, 8), (8, 10)]
    assert [c.length for c in chunks] == [4, 4, 2]
    assert kv.ChunkedPrefillPlanner(4).plan(0) == ()
    with pytest.raises(ValueError):
        kv.ChunkedPrefillPlanner(chunk_size=0)
    with pytest.raises(ValueError):
        kv.ChunkedPrefillPlanner(4).plan(-1)


def test_mixed_length_packer():
    plan = kv.MixedLengthPrefillPacker().pack(((10, 11), (20,), (30, 31, 32)))
    assert plan.flat_token_ids == (10, 11, 20, 30, 31, 32)
    assert plan.flat_position_ids == (0, 1, 0, 0, 1, 2)
    assert [(r.request_index, r.start, r.length, r.end) for r in plan.requests] == [
        (0, 0, 2, 2), (1, 2, 1, 3), (2, 3, 3, 6)]
    assert plan.total_tokens == 6 and plan.batch_size == 3
