"""Host logic of the decode graph runner, with a stand-in for the graph calls (no GPU needed).

Follows the cases of the reference's own tests for its runner (tests/test_decode_p0.py:116-262):
model families that may capture, the key of a step, capture once / replay every step, and a key
whose capture failed is never tried again.
"""

from contextlib import contextmanager
from types import SimpleNamespace

import pytest
import torch

from llama_lite_npu_amd.executor.decode_graph import DecodeGraphRunner, supports_decode_graph


class FakeGraph:
    def __init__(self):
        self.replay_count = 0

    def replay(self):
        self.replay_count += 1


class FakeGraphs:
    """The calls DecodeGraphRunner makes on its graph API; capture just runs the body once."""

    available = True

    def __init__(self):
        self.graphs = []
        self.pool_requests = 0

    def Graph(self):
        self.graphs.append(FakeGraph())
        return self.graphs[-1]

    @contextmanager
    def graph(self, graph, pool=None):
        assert pool == "shared-pool"
        yield

    def synchronize(self):
        pass

    def graph_pool_handle(self):
        self.pool_requests += 1
        return "shared-pool"


def _info(length=65):
    return SimpleNamespace(max_actual_seq_len=length,
                           cur_select_index=torch.tensor([3], dtype=torch.int32),
                           b_seq_len=torch.tensor([length], dtype=torch.int64),
                           b_req_idx=torch.tensor([0], dtype=torch.int32))


def test_model_families_that_may_capture():
    assert supports_decode_graph("qwen3") and supports_decode_graph("qwen3_moe")
    assert supports_decode_graph("qwen3_moe", moe_parallel_mode="tp")
    assert not supports_decode_graph("qwen3_moe", moe_parallel_mode="ep")
    assert not supports_decode_graph("Qwen3_VL") and not supports_decode_graph("llava")


def test_one_bucket_for_every_length_by_default():
    assert DecodeGraphRunner.sequence_bucket(1) == 0
    assert DecodeGraphRunner.sequence_bucket(4097) == 0
    runner = DecodeGraphRunner(model=None, graph_api=FakeGraphs())
    ids = torch.zeros((4, 1), dtype=torch.long)
    assert runner.graph_key(ids, 65) == (4, 0) == runner.graph_key(ids, 4000)


def test_partition_buckets_as_in_the_reference_when_asked_for():
    class Bucketed(DecodeGraphRunner):
        PARTITION_SIZE = 128

    assert [Bucketed.sequence_bucket(n) for n in (1, 127, 128, 129)] == [128, 128, 128, 256]
    runner = Bucketed(model=None, graph_api=FakeGraphs())
    ids = torch.zeros((4, 1), dtype=torch.long)
    assert runner.graph_key(ids, 65) == (4, 128)
    assert runner.graph_key(ids, 120) == (4, 128)
    assert runner.graph_key(ids, 129) == (4, 256)


def test_same_key_captures_once_and_replays_each_step():
    class Model:
        forward_count = 0

        def forward(self, input_ids, position_ids, atten_info):
            self.forward_count += 1
            return input_ids.float()

    api = FakeGraphs()
    model = Model()
    runner = DecodeGraphRunner(model, graph_api=api)
    info = _info(65)
    runner(torch.tensor([[1]]), torch.tensor([[64]]), info)
    info.max_actual_seq_len = 300                  # far beyond a 128-token partition: same graph
    info.b_seq_len.fill_(300)
    info.cur_select_index.fill_(4)
    runner(torch.tensor([[2]]), torch.tensor([[299]]), info)

    assert runner.capture_count == 1 and runner.capture_attempt_count == 1
    assert runner.replay_count == 2 and runner.fallback_count == 0
    assert model.forward_count == 2                # the eager run on the static copies + the capture
    assert api.pool_requests == 1 and len(api.graphs) == 1 and api.graphs[0].replay_count == 2
    captured = runner._graphs[(1, 0)]
    # the replay refreshed the static copies, which are not the caller's tensors
    assert captured.b_seq_len.item() == 300 and captured.cur_select_index.item() == 4
    assert captured.input_ids.item() == 2 and captured.position_ids.item() == 299
    assert captured.b_seq_len is not info.b_seq_len


def test_failed_key_is_not_captured_again():
    class Failing:
        forward_count = 0

        def forward(self, input_ids, position_ids, atten_info):
            self.forward_count += 1
            raise RuntimeError("unsupported graph operator")

    model = Failing()
    runner = DecodeGraphRunner(model, model_type="qwen3_moe", graph_api=FakeGraphs())
    info = _info()
    for token in (1, 2):
        with pytest.raises(RuntimeError, match="unsupported graph operator"):
            runner(torch.tensor([[token]]), torch.tensor([[64]]), info)
    assert model.forward_count == 3                # one capture attempt + two eager fallbacks
    assert runner.capture_attempt_count == 1 and runner.capture_count == 0
    assert runner.fallback_count == 2 and not runner.captured


def test_without_graph_support_every_step_is_eager():
    class Model:
        def forward(self, input_ids, position_ids, atten_info):
            return input_ids + 1

    api = FakeGraphs()
    api.available = False
    runner = DecodeGraphRunner(Model(), graph_api=api)
    out = runner(torch.tensor([[5]]), torch.tensor([[0]]), _info())
    assert out.item() == 6 and runner.fallback_count == 1 and runner.capture_attempt_count == 0
    assert api.pool_requests == 0


def test_a_trimmed_block_table_keys_the_graph_by_its_width():
    class Model:
        def forward(self, input_ids, position_ids, atten_info):
            return atten_info.block_table.sum()

    runner = DecodeGraphRunner(Model(), graph_api=FakeGraphs())            # no max_blocks given
    info = _info()
    info.seq_lens_i32 = torch.tensor([65], dtype=torch.int32)
    info.block_table = torch.tensor([[1, 2, 3, 4, 5]], dtype=torch.int32)
    runner(torch.tensor([[1]]), torch.tensor([[64]]), info)
    info.block_table = torch.tensor([[1, 2, 3, 4, 5, 6]], dtype=torch.int32)   # the request grew a page
    runner(torch.tensor([[1]]), torch.tensor([[80]]), info)
    assert runner.capture_count == 2

    wide = DecodeGraphRunner(Model(), graph_api=FakeGraphs(), max_blocks=8)
    info.block_table = torch.tensor([[1, 2, 3, 4, 5]], dtype=torch.int32)
    wide(torch.tensor([[1]]), torch.tensor([[64]]), info)
    info.block_table = torch.tensor([[1, 2, 3, 4, 5, 6]], dtype=torch.int32)
    out = wide(torch.tensor([[1]]), torch.tensor([[80]]), info)
    assert wide.capture_count == 1
    static = wide._graphs[(1, 0)].block_table
    assert static.shape == (1, 8) and static[0].tolist() == [1, 2, 3, 4, 5, 6, 0, 0]
