"""The oracle and the host code against the committed fixture of the reference's integer examples."""

import json
from pathlib import Path
from types import SimpleNamespace

import torch

from llama_lite_npu_amd.continuous_batching import BatchRequest, ContinuousBatchModelBackend
from llama_lite_npu_amd.executor import DecodeGraphRunner, ModelExecutor, PagedKVCacheManager
from oracle import decode_metadata

GOLDEN = json.loads((Path(__file__).parent / "golden" / "reference_integer_examples.json").read_text())


def test_token_table_example():
    ex = GOLDEN["token_table"]
    assert decode_metadata.token_slots(ex["pages"], ex["num_tokens"], ex["page_size"]).tolist() == ex["slots"]
    mgr = PagedKVCacheManager(num_layers=1, num_kv_heads=1, head_dim=8, num_pages=16, page_size=ex["page_size"],
                              dtype=torch.float16, device="cpu")
    assert mgr.slots_of(ex["pages"], ex["num_tokens"]).tolist() == ex["slots"]
    table = torch.zeros((1, 16), dtype=torch.int32)
    assert mgr.build_token_table(torch.tensor(ex["pages"]), ex["num_tokens"], table, 0) == ex["num_tokens"]
    assert table[0, :ex["num_tokens"]].tolist() == ex["slots"]


def test_graph_keys_with_the_reference_partition():
    ex = GOLDEN["graph_buckets"]

    class Bucketed(DecodeGraphRunner):
        PARTITION_SIZE = ex["partition_size"]

    assert [Bucketed.sequence_bucket(n) for n in ex["sequence_lengths"]] == ex["buckets"]
    runner = Bucketed(model=None, graph_api=SimpleNamespace(available=False))
    ids = torch.zeros((4, 1), dtype=torch.long)
    for length, key in ex["batch_4_keys"].items():
        assert list(runner.graph_key(ids, int(length))) == key


def _cpu_executor():
    ex = ModelExecutor(num_layers=1, num_q_heads=2, num_kv_heads=1, head_dim=128, num_pages=32, max_seq_len=64,
                       max_requests=8, device="cpu")
    ex.forwards = []

    class Model:
        def forward(self, input_ids, position_ids, atten_info):
            ex.forwards.append((input_ids.clone(), position_ids.clone()))
            ex.seen = dict(chunked=atten_info.is_paged_chunk_prefill, starts=atten_info.b_start_loc.tolist(),
                           context=None if atten_info.chunk_context_len is None else atten_info.chunk_context_len.tolist(),
                           chunk=None if atten_info.chunk_q_seq_len is None else atten_info.chunk_q_seq_len.tolist())
            logits = torch.zeros((*input_ids.shape, 16))
            logits[..., 3] = 1.0
            return logits

    ex.attach_model(Model(), use_graph=False)
    return ex


def test_packing_of_mixed_length_prompts_through_the_real_metadata_builders():
    ex_data = GOLDEN["packed_prefill"]
    ex = _cpu_executor()
    backend = ContinuousBatchModelBackend(SimpleNamespace(model_executor=ex, tokenizer=SimpleNamespace(eos_token_id=9)))
    requests = [BatchRequest(str(i), p, 4, 0.0, 1.0) for i, p in enumerate(ex_data["prompts"])]
    assert backend.prefill(requests) == [3, 3, 3]
    assert [r.model_request_id for r in requests] == ex_data["request_ids"]
    (ids, pos), = ex.forwards
    assert ids.tolist() == [ex_data["flat_input_ids"]] and pos.tolist() == [ex_data["flat_position_ids"]]
    assert ex.seen["starts"] == ex_data["starts"] and not ex.seen["chunked"]


def test_chunked_prefill_examples():
    first = GOLDEN["chunked_prefill"]["first_chunk"]
    ex = _cpu_executor()
    backend = ContinuousBatchModelBackend(SimpleNamespace(model_executor=ex, tokenizer=SimpleNamespace(eos_token_id=9)))
    requests = [BatchRequest(str(i), p, 4, 0.0, 1.0) for i, p in enumerate(first["prompts"])]
    assert backend.prefill_chunk(requests, first["chunk_size"]) == first["tokens"]
    (ids, pos), = ex.forwards
    assert ids.tolist() == [first["flat_input_ids"]] and pos.tolist() == [first["flat_position_ids"]]
    assert [r.prefill_cursor for r in requests] == first["cursors_after"]
    assert ex.seen["starts"] == [0, 2] and not ex.seen["chunked"]

    later = GOLDEN["chunked_prefill"]["later_chunk"]
    ex = _cpu_executor()
    backend = ContinuousBatchModelBackend(SimpleNamespace(model_executor=ex, tokenizer=SimpleNamespace(eos_token_id=9)))
    requests = [BatchRequest(str(i), p, 4, 0.0, 1.0) for i, p in enumerate(later["prompts"])]
    backend.prefill_chunk(requests, later["chunk_size"])          # first chunks: cursors 2, 2
    assert [r.prefill_cursor for r in requests] == later["cursors_before"]
    ex.forwards.clear()
    tokens = backend.prefill_chunk(requests, later["chunk_size"])
    (ids, pos), = ex.forwards
    assert ids.tolist() == [later["flat_input_ids"]] and pos.tolist() == [later["flat_position_ids"]]
    assert [r.prefill_cursor for r in requests] == later["cursors_after"]
    assert [t is not None for t in tokens] == later["completed"]
    assert ex.seen["chunked"] and ex.seen["context"] == later["context_lengths"]
    assert ex.seen["chunk"] == later["chunk_lengths"]


def test_static_batch_prefill_then_decode_select_indices():
    """The worked example in the docstring of the reference's prefill_alloc_kv_cache: four padded
    prompts, then two decode steps whose tokens land right behind each prompt's own length."""
    ex = GOLDEN["static_batch_prefill"]
    stride = ex["slots_per_request"]                 # one page per request reproduces the example's slot ranges
    executor = ModelExecutor(num_layers=1, num_q_heads=2, num_kv_heads=1, head_dim=8, num_pages=4,
                             max_seq_len=stride, max_requests=4, page_size=stride, device="cpu")
    select, patches = executor.prefill_alloc_kv_cache(ex["max_prompt_len"], torch.tensor(ex["b_seq_len"]),
                                                      torch.arange(4, dtype=torch.int32))
    assert patches is None
    info = executor.atten_info
    assert select.tolist() == sum(ex["prefill_select_index"], [])
    assert info.b_start_loc.tolist() == [i * ex["max_prompt_len"] for i in range(4)]
    assert info.b_seq_len.tolist() == ex["b_seq_len"] and info.max_actual_seq_len == ex["max_prompt_len"]
    assert info.b_req_idx.tolist() == [0, 1, 2, 3]
    assert [p[0] * stride for p in map(executor.req_tokens_manager.request_pages, range(4))] == ex["start_index"]
    for step in ex["decode_steps"]:
        assert executor.decode_alloc_kv_cache(4).tolist() == step["cur_select_index"]
        assert info.b_seq_len.tolist() == step["cur_b_seq_len"]
    # a batch that does not fit gives the reference's error and leaves nothing allocated behind
    executor.release_paged_requests()
    small = ModelExecutor(num_layers=1, num_q_heads=2, num_kv_heads=1, head_dim=8, num_pages=2,
                          max_seq_len=8, max_requests=4, page_size=4, device="cpu")
    try:
        small.prefill_alloc_kv_cache(8, [8, 3], [0, 1])
    except RuntimeError as exc:
        assert "Paged KV allocation failed during prefill" in str(exc)
    else:
        raise AssertionError("allocation beyond the pool did not fail")
    assert small.kv_mem_manager.num_free_pages == 2


def test_static_batch_decode_steps_never_attend_a_padding_row():
    """After the padded static-batch prefill every decode step writes request r's token at
    slots(r)[tokens so far] (the first one over the first padding row) and attends exactly the
    prompt's own tokens plus the tokens decoded so far: the slots a step can reach never include
    a padding row that has not been overwritten. The reference's paged branch counts the padded
    length instead (model_executor.py:450-455); this pins the behaviour chosen here."""
    page = 4
    lens = [3, 7, 1, 5]
    longest = 7
    executor = ModelExecutor(num_layers=1, num_q_heads=2, num_kv_heads=1, head_dim=8, num_pages=16,
                             max_seq_len=16, max_requests=4, page_size=page, device="cpu")
    select, _ = executor.prefill_alloc_kv_cache(longest, torch.tensor(lens), torch.arange(4, dtype=torch.int32))
    mgr = executor.req_tokens_manager
    rows = select.reshape(4, longest)
    written = [set(rows[r, :lens[r]].tolist()) for r in range(4)]           # slots holding real tokens
    padding = [set(rows[r, lens[r]:].tolist()) for r in range(4)]
    info = executor.atten_info
    for step in range(1, 6):
        slots = executor.decode_alloc_kv_cache(4).tolist()
        for r in range(4):
            have = lens[r] + step
            assert slots[r] == mgr.slots(r, 0, have)[have - 1]                # right behind what the request holds
            assert int(info.b_seq_len[r]) == have
            written[r].add(slots[r])
            padding[r].discard(slots[r])
            # what a kernel reaches: the first `have` tokens of the step's block-table row
            pages = info.block_table[r].tolist()
            attended = {pages[t // page] * page + t % page for t in range(int(info.seq_lens_i32[r]))}
            assert attended == written[r], (r, step)
            assert not (attended & padding[r])
