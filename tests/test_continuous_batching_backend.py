"""Host logic of the continuous-batching backend against a recording stand-in for the executor (CPU).

The cases and the expected executor call sequences are those of the reference's own tests of its
backend (tests/test_continuous_batching.py:422-941): what is packed into one forward, what the
prefill budget splits, which tokens are replayed at which positions, what a prefix-cache hit skips,
and what chunked prefill does for first and later chunks. The stand-in answers ``forward`` with
logits whose arg-max is 40 + request id at each request's sampling row.
"""

from types import SimpleNamespace

import pytest
import torch

from llama_lite_npu_amd.continuous_batching import (BatchRequest, ContinuousBatchModelBackend,
                                                    KVCacheCapacityError, sample_next_token)


class RecordingExecutor:
    """Counts tokens per request like the paged managers do and records every call."""

    def __init__(self, max_prefill_tokens=None):
        self.device = "cpu"
        self.use_paged_attn = True
        self.max_prefill_tokens = max_prefill_tokens
        self.max_seq_len = 64
        self.lengths = {}
        self.req_tokens_manager = SimpleNamespace(req_token_count=self.lengths, max_seq_len=64)
        self.next_id = 0
        self.calls = []            # (name, args) in order
        self.forwards = []         # (input_ids, position_ids)
        self.active = ()
        self.rows = None           # sampling rows of a packed forward
        self.released = []
        self.logits_are_sharded = False

    def _log(self, name, *args):
        self.calls.append((name, args))

    def named(self, name):
        return [args for n, args in self.calls if n == name]

    def reserve_paged_requests(self, prompt_lengths, reserved_lengths=None):
        self._log("reserve", tuple(prompt_lengths), None if reserved_lengths is None else tuple(reserved_lengths))
        ids = []
        for n in prompt_lengths:
            self.lengths[self.next_id] = int(n)
            ids.append(self.next_id)
            self.next_id += 1
        return tuple(ids)

    def ensure_paged_request_capacity(self, req_idx, total_tokens):
        self._log("ensure", req_idx, total_tokens)

    def activate_paged_prefill_batch(self, request_ids, prompt_length):
        self._log("prefill_batch", tuple(request_ids), prompt_length)
        self.active, self.rows = tuple(request_ids), None

    def activate_paged_packed_prefill_batch(self, request_ids, prompt_lengths):
        self._log("packed_batch", tuple(request_ids), tuple(prompt_lengths))
        self.active = tuple(request_ids)
        ends, pos = [], []
        for n in prompt_lengths:
            pos.extend(range(int(n)))
            ends.append(len(pos) - 1)
        self.rows = tuple(ends)
        return torch.tensor(pos), torch.tensor(ends)

    def activate_paged_decode_batch(self, request_ids):
        self._log("decode_batch", tuple(request_ids))
        self.active, self.rows = tuple(request_ids), None

    def extend_paged_requests(self, request_ids):
        self._log("extend", tuple(request_ids))
        for r in request_ids:
            self.lengths[r] += 1

    def release_paged_request_ids(self, request_ids):
        self.released.extend(request_ids)
        for r in request_ids:
            self.lengths.pop(r, None)

    def share_paged_request_from_cache(self, prompt_tokens):
        return None

    def store_paged_request_prefix(self, prompt_tokens, req_idx, first_token_id):
        self._log("store", tuple(prompt_tokens), req_idx, first_token_id)

    def forward(self, input_ids, position_ids):
        self.forwards.append((input_ids.clone(), position_ids.clone()))
        b, t = input_ids.shape
        logits = torch.zeros((b, t, 128))
        if self.rows is not None:
            for req, row in zip(self.active, self.rows):
                logits[0, row, 40 + req] = 10.0
            self.rows = None
        else:
            for row, req in enumerate(self.active):
                logits[row, -1, 40 + req] = 10.0
        return logits


class ChunkingExecutor(RecordingExecutor):
    def activate_paged_chunk_prefill_batch(self, request_ids, context_lengths, chunk_lengths):
        self._log("chunk_batch", tuple(request_ids), tuple(context_lengths), tuple(chunk_lengths))
        self.active = tuple(request_ids)
        pos, ends = [], []
        for c, n in zip(context_lengths, chunk_lengths):
            pos.extend(range(int(c), int(c) + int(n)))
            ends.append(len(pos) - 1)
        self.rows = tuple(ends)
        return torch.tensor(pos), torch.tensor(ends)


def _backend(executor, **kw):
    tokenizer = SimpleNamespace(eos_token_id=99, decode=lambda ids, skip_special_tokens=True: " ".join(map(str, ids)),
                                encode=lambda text, add_special_tokens=True: [7, 8])
    return ContinuousBatchModelBackend(SimpleNamespace(model_executor=executor, tokenizer=tokenizer), **kw)


def _req(name, tokens, temperature=0.0, top_p=1.0):
    return BatchRequest(name, tokens, 4, temperature, top_p)


def test_facts_the_scheduler_reads():
    ex = RecordingExecutor(max_prefill_tokens=9)
    be = _backend(ex)
    assert be.eos_token_id == 99 and be.max_context_tokens == 64 and be.max_prefill_tokens == 9
    assert be.tokenize("x") == [7, 8] and be.decode_tokens([1, 2]) == "1 2"
    assert not be.device_decode                      # this executor has no device-side decode batches
    ex.use_paged_attn = False
    with pytest.raises(RuntimeError, match="page_size"):
        _backend(ex)
    with pytest.raises(ValueError):
        BatchRequest("bad", [1], 0, 0.0, 1.0)
    r = _req("r", [1, 2])
    r.generated_token_ids += [10, 11]
    assert r.model_context_tokens == [1, 2, 10, 11] and r.last_token_id == 11      # what a preempted request replays
    r.model_request_id = 3
    r.mark_preempted()
    assert r.preemptions == 1 and r.model_request_id is None


def test_mixed_lengths_go_into_one_packed_forward():
    ex = RecordingExecutor()
    be = _backend(ex)
    reqs = [_req("a", [1, 2]), _req("b", [3]), _req("c", [4, 5])]
    assert be.prefill(reqs) == [40, 41, 42]
    assert ex.named("prefill_batch") == []
    assert ex.named("packed_batch") == [((0, 1, 2), (2, 1, 2))]
    (ids, pos), = ex.forwards
    assert ids.tolist() == [[1, 2, 3, 4, 5]] and pos.tolist() == [[0, 1, 0, 0, 1]]
    assert [r.model_request_id for r in reqs] == [0, 1, 2]
    assert ex.named("extend") == [((0, 1, 2),)]       # the slot of each first generated token
    assert [a[0] for a in ex.named("store")] == [(1, 2), (3,), (4, 5)]
    assert be._device_positions[2].item() == 2 and be._device_tokens[1].item() == 41


def test_equal_lengths_go_into_one_rectangular_forward():
    ex = RecordingExecutor()
    be = _backend(ex)
    assert be.prefill([_req("a", [1, 2, 3]), _req("b", [4, 5, 6])]) == [40, 41]
    assert ex.named("packed_batch") == [] and ex.named("prefill_batch") == [((0, 1), 3)]
    (ids, pos), = ex.forwards
    assert ids.tolist() == [[1, 2, 3], [4, 5, 6]] and pos.tolist() == [[0, 1, 2], [0, 1, 2]]


def test_the_prefill_budget_splits_the_forwards():
    ex = RecordingExecutor(max_prefill_tokens=3)
    be = _backend(ex)
    assert be.prefill([_req("a", [1, 2]), _req("b", [3, 4]), _req("c", [5])]) == [40, 41, 42]
    assert ex.named("reserve") == [((2, 2, 1), None)]            # reserved together, run in two forwards
    assert ex.named("prefill_batch") == [((0,), 2)]
    assert ex.named("packed_batch") == [((1, 2), (2, 1))]
    assert len(ex.forwards) == 2


def test_a_prompt_over_the_budget_is_replayed_token_by_token():
    ex = RecordingExecutor(max_prefill_tokens=2)
    be = _backend(ex)
    assert be.prefill([_req("long", [1, 2, 3, 4])]) == [40]
    assert ex.named("reserve") == [((1,), (5,))]                  # room for the prompt and the first new token
    assert ex.named("prefill_batch") == [] and ex.named("packed_batch") == []
    assert [f[0].tolist() for f in ex.forwards] == [[[1]], [[2]], [[3]], [[4]]]
    assert [f[1].tolist() for f in ex.forwards] == [[[0]], [[1]], [[2]], [[3]]]
    assert ex.lengths[0] == 5


def test_a_failed_forward_gives_the_reservations_back():
    class Failing(RecordingExecutor):
        def forward(self, input_ids, position_ids):
            raise RuntimeError("Paged KV allocation failed for request 0")

    ex = Failing()
    be = _backend(ex)
    reqs = [_req("a", [1, 2]), _req("b", [3])]
    with pytest.raises(RuntimeError, match="allocation failed"):
        be.prefill(reqs)
    assert sorted(ex.released) == [0, 1] and all(r.model_request_id is None for r in reqs)


def test_decode_takes_its_batch_as_given_and_books_the_next_slot():
    ex = RecordingExecutor()
    be = _backend(ex)
    reqs = [_req("a", [1]), _req("b", [2])]
    be.prefill(reqs)
    assert be.decode([reqs[1]]) == [41]
    assert ex.named("decode_batch")[-1] == ((1,),)
    assert ex.lengths[1] == 3                                     # prompt, first token, the one just booked
    assert be.decode([]) == []


def test_decode_feeds_the_tokens_and_positions_it_kept_itself():
    ex = RecordingExecutor()
    be = _backend(ex)
    r = _req("a", [1, 2])
    assert be.prefill([r]) == [40]
    r.generated_token_ids[:] = [77]                               # whatever the host believes ...
    ex.lengths[0] = 999
    be.decode([r])
    ids, pos = ex.forwards[-1]
    assert ids.tolist() == [[40]] and pos.tolist() == [[2]]       # ... the device-side state decides
    be.decode([r])                                                # same batch again: last step's samples go straight in
    ids, pos = ex.forwards[-1]
    assert ids.tolist() == [[40]] and pos.tolist() == [[3]]


def test_a_worker_keeps_tokens_on_the_device():
    ex = RecordingExecutor()
    be = _backend(ex, return_host_tokens=False)
    r = _req("w", [1])
    assert be.prefill([r]) == []
    assert be._device_tokens[r.model_request_id].item() == 40
    assert ex.named("store") == []                                # storing a prefix needs the token on the host
    assert be.decode([r]) == []


class CachingExecutor(RecordingExecutor):
    def __init__(self):
        super().__init__()
        self.cache, self.shared, self.cow = {}, [], []

    def share_paged_request_from_cache(self, prompt_tokens):
        hit = self.cache.get(tuple(prompt_tokens))
        if hit is None:
            return None
        length, token = hit
        req = self.next_id
        self.next_id += 1
        self.lengths[req] = length
        self.shared.append((req, tuple(prompt_tokens)))
        return req, token

    def store_paged_request_prefix(self, prompt_tokens, req_idx, first_token_id):
        self.cache[tuple(prompt_tokens)] = (self.lengths[req_idx], first_token_id)

    def copy_on_write(self, request_ids):
        self.cow.append(tuple(request_ids))
        return []


def test_an_exact_cache_hit_needs_no_forward_and_gets_its_own_last_page():
    ex = CachingExecutor()
    be = _backend(ex)
    first, second = _req("first", [1, 2, 3]), _req("second", [1, 2, 3])
    assert be.prefill([first]) == [40]
    assert be.prefill([second]) == [40]
    assert len(ex.forwards) == 1 and ex.named("reserve") == [((3,), None)]
    assert ex.shared == [(1, (1, 2, 3))] and second.model_request_id == 1
    assert ex.cow == [(1,)]                    # the slot of the first new token lay in a shared page
    assert be._device_positions[1].item() == 3 and second.prefill_cursor == 3
    assert be.decode([second]) == [41]         # continues from the cached token
    assert ex.forwards[-1][0].tolist() == [[40]] and ex.forwards[-1][1].tolist() == [[3]]


def test_sampling_requests_neither_use_nor_fill_the_cache():
    ex = CachingExecutor()
    be = _backend(ex)
    assert be.prefill([_req("first", [1, 2, 3], 0.6, 0.9)]) == [40]
    assert be.prefill([_req("second", [1, 2, 3], 0.6, 0.9)]) == [41]
    assert len(ex.forwards) == 2 and ex.cache == {} and ex.shared == []


def test_out_of_pages_during_copy_on_write_is_a_capacity_error():
    class Full(CachingExecutor):
        def copy_on_write(self, request_ids):
            raise RuntimeError("Paged KV allocation failed during copy-on-write")

    ex = Full()
    be = _backend(ex)
    be.prefill([_req("first", [1, 2, 3])])
    with pytest.raises(KVCacheCapacityError):
        be.prefill([_req("second", [1, 2, 3])])
    assert ex.released == [1]


class BlockPrefixExecutor(RecordingExecutor):
    def __init__(self):
        super().__init__()
        self.next_id = 3
        self.lengths.update({0: 4, 1: 4})
        self.lookups = 0

    def share_paged_prefix_from_cache(self, prompt_tokens):
        self.lookups += 1
        return (1, 4, None) if tuple(prompt_tokens) == (1, 2, 3, 4, 5, 6) else None


def test_block_prefix_lookups_are_off_unless_asked_for():
    ex = BlockPrefixExecutor()
    be = _backend(ex)
    assert be.prefill([_req("p", [1, 2, 3, 4, 5, 6])]) == [43]
    assert ex.lookups == 0
    assert [f[0].tolist()[0] for f in ex.forwards] == [[1, 2, 3, 4, 5, 6]]


def test_a_block_prefix_hit_replays_only_the_suffix():
    ex = BlockPrefixExecutor()
    be = _backend(ex, enable_partial_prefix_cache=True)
    r = _req("p", [1, 2, 3, 4, 5, 6])
    assert be.prefill([r]) == [41]
    assert r.model_request_id == 1
    assert [f[0].tolist() for f in ex.forwards] == [[[5]], [[6]]]
    assert [f[1].tolist() for f in ex.forwards] == [[[4]], [[5]]]
    assert ex.lengths[1] == 7


def _mid_prefill(ex, name, tokens, req_idx, cursor):
    r = _req(name, tokens)
    r.model_request_id, r.prefill_cursor = req_idx, cursor
    ex.lengths[req_idx] = cursor
    return r


def test_first_chunks_are_packed_with_room_reserved_for_the_whole_prompt():
    ex = RecordingExecutor()
    be = _backend(ex)
    a, b = _req("a", [1, 2, 3, 4]), _req("b", [5, 6, 7])
    assert be.prefill_chunk([a, b], chunk_size=2) == [None, None]
    assert (a.prefill_cursor, b.prefill_cursor) == (2, 2)
    assert ex.named("reserve") == [((2, 2), (5, 4))]
    assert ex.named("packed_batch") == [((0, 1), (2, 2))] and ex.named("decode_batch") == []
    (ids, pos), = ex.forwards
    assert ids.tolist() == [[1, 2, 5, 6]] and pos.tolist() == [[0, 1, 0, 1]]
    assert ex.named("extend") == []                 # nobody's context is complete yet


def test_a_first_chunk_that_covers_the_prompt_completes_it():
    ex = RecordingExecutor()
    be = _backend(ex)
    a, b = _req("a", [1, 2]), _req("b", [5, 6, 7])
    assert be.prefill_chunk([a, b], chunk_size=2) == [40, None]
    assert ex.named("extend") == [((0,),)] and [s[0] for s in ex.named("store")] == [(1, 2)]


def test_later_chunks_without_a_history_kernel_are_replayed_in_micro_batches():
    ex = RecordingExecutor()
    be = _backend(ex)
    a = _mid_prefill(ex, "a", [1, 2, 3, 4], 0, 2)
    b = _mid_prefill(ex, "b", [5, 6, 7], 1, 2)
    assert be.prefill_chunk([a, b], chunk_size=2) == [40, 41]
    assert (a.prefill_cursor, b.prefill_cursor) == (4, 3)
    assert ex.named("packed_batch") == []
    assert [f[0].tolist() for f in ex.forwards] == [[[3], [7]], [[4]]]
    assert [f[1].tolist() for f in ex.forwards] == [[[2], [2]], [[3]]]
    assert ex.named("decode_batch") == [((0, 1),), ((0,),)]


def test_later_chunks_use_attention_over_cached_history_when_the_executor_has_it():
    ex = ChunkingExecutor()
    be = _backend(ex)
    a = _mid_prefill(ex, "a", [1, 2, 3, 4], 0, 2)
    b = _mid_prefill(ex, "b", [5, 6, 7, 8, 9], 1, 2)
    assert be.prefill_chunk([a, b], chunk_size=2) == [40, None]
    assert (a.prefill_cursor, b.prefill_cursor) == (4, 4)
    assert ex.named("chunk_batch") == [((0, 1), (2, 2), (2, 2))] and ex.named("decode_batch") == []
    (ids, pos), = ex.forwards
    assert ids.tolist() == [[3, 4, 7, 8]] and pos.tolist() == [[2, 3, 2, 3]]
    assert ("ensure", (0, 5)) in ex.calls and ("ensure", (1, 5)) in ex.calls


def test_fresh_and_running_requests_share_a_chunk_step():
    ex = ChunkingExecutor()
    be = _backend(ex)
    ex.next_id = 1
    running = _mid_prefill(ex, "run", [1, 2, 3, 4, 5], 0, 2)
    fresh = _req("new", [6, 7, 8])
    assert be.prefill_chunk([running, fresh], chunk_size=2) == [None, None]
    assert ex.named("packed_batch") == [((1,), (2,))] and ex.named("chunk_batch") == [((0,), (2,), (2,))]
    assert be.prefill_chunk([running, fresh], chunk_size=2) == [40, 41]
    assert ex.named("chunk_batch")[-1] == ((0, 1), (4, 2), (1, 1))


def test_preparing_a_chunk_reserves_for_running_requests_only():
    ex = RecordingExecutor()
    be = _backend(ex)
    fresh = _req("first", [1, 2, 3, 4])
    running = _mid_prefill(ex, "run", [1, 2, 3, 4, 5, 6], 4, 2)
    be.prepare_prefill_chunk([fresh, running], chunk_size=2)
    assert fresh.model_request_id is None and fresh.prefill_cursor == 0 and ex.named("reserve") == []
    assert ex.named("ensure") == [(4, 5)]


def test_capacity_failures_name_the_request():
    class Tight(RecordingExecutor):
        def ensure_paged_request_capacity(self, req_idx, total_tokens):
            raise RuntimeError("Paged KV capacity reservation failed")

    ex = Tight()
    be = _backend(ex)
    running = _mid_prefill(ex, "run", [1, 2, 3, 4], 0, 2)
    with pytest.raises(KVCacheCapacityError, match="request_id=run.*target_tokens=5"):
        be.prepare_prefill_chunk([running], chunk_size=2)
    with pytest.raises(RuntimeError, match="empty prompts"):
        be.prefill_chunk([_req("empty", [])], chunk_size=2)


def test_release_and_preempt_forget_the_request():
    ex = RecordingExecutor()
    be = _backend(ex)
    reqs = [_req("a", [1]), _req("b", [2, 3])]
    be.prefill(reqs)
    be.decode(reqs)
    be.preempt([reqs[0]])
    assert ex.released == [0] and reqs[0].model_request_id is None
    assert 0 not in be._device_tokens and 0 not in be._positions
    be.release([reqs[0], reqs[1]])                 # releasing twice is harmless
    assert ex.released == [0, 1] and be._device_tokens == {}
    reqs[0].generated_token_ids.append(40)         # the preempted request comes back with its history
    assert be.prefill([reqs[0]]) == [42]
    assert ex.forwards[-1][0].tolist() == [[1, 40]]


def test_sampler_is_greedy_at_temperature_zero_and_respects_top_p():
    logits = torch.tensor([[0.0, 5.0, 1.0, 4.9], [3.0, 0.0, 0.0, 2.9]])
    assert sample_next_token(logits, [0.0, 0.0], [1.0, 1.0]).tolist() == [1, 0]
    assert sample_next_token(logits[:, None, :].expand(2, 3, 4), [0.0, 0.0], [1.0, 1.0]).tolist() == [1, 0]
    torch.manual_seed(0)
    seen = set()
    for _ in range(200):
        seen.add(tuple(sample_next_token(logits, [1.0, 0.0], [0.9, 1.0]).tolist()))
    assert {s[1] for s in seen} == {0}                     # the greedy row never moves
    assert {s[0] for s in seen} == {1, 3}                  # 0.9 of the mass is tokens 1 and 3; 0 and 2 are cut
    tiny = sample_next_token(logits, [1.0, 1.0], [1e-6, 1e-6])
    assert tiny.tolist() == [1, 0]                         # top_p -> 0 leaves the most likely token
    with pytest.raises(NotImplementedError):
        sample_next_token(logits, [0.0, 0.0], [1.0, 1.0], vocab_parallel=True)
