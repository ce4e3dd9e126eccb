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
