"""litekv_paged_decode_static (the entry point that allocates nothing) against
litekv_paged_decode with a caller's workspace, through the C ABI: same kernels, same cuts, so the
outputs must agree bit for bit; attention tolerance against the fp32 oracle on top."""

import pytest
import torch

from llama_lite_npu_amd import _lib, ops, workloads
from oracle import c_oracle
from tests.parity import assert_attention_close, assert_bit_exact, to_np16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(case, max_splits, min_pages):
    """(static-scratch result, workspace result, oracle) of one decode case."""
    b, hq, d = case.q.shape
    bt = case.block_table.to(torch.int32).contiguous()
    sl = case.seq_lens.to(torch.int32).contiguous()
    ref_out = ops.paged_decode(case.q, case.kv_pool, bt, sl, case.softmax_scale, max_splits=max_splits,
                               min_pages_per_split=min_pages)
    out = torch.full((b, hq, d), float("nan"), dtype=torch.float16, device=DEV)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    torch_before = torch.cuda.memory_allocated()
    ops.paged_decode_static(case.q, case.kv_pool, bt, sl, out, max_splits, min_pages, case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == torch_before
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory changed hands during the call"
    oracle = c_oracle.paged_decode(to_np16(case.q), to_np16(case.kv_pool), bt.cpu().numpy(), sl.cpu().numpy(),
                                   case.softmax_scale)
    return out, ref_out, oracle


def test_static_scratch_decode_equals_workspace_decode_twice_in_a_row():
    print("static decode: large then small", flush=True)
    big = workloads.make_decode_case("static-big", 7101, [1500, 0, 33, 700, 16, 2047, 255, 1], 64, 8, device=DEV)
    big.seq_lens[1] = 0  # an empty row between live ones
    out, ref_out, oracle = _both(big, 8, 4)
    assert float(out[1].abs().max()) == 0.0
    assert_bit_exact(out, ref_out, "static vs workspace (first call)")
    assert_attention_close(out, oracle, "static vs oracle (first call)")
    # a smaller step right after: fewer sequences, other head layout, fewer splits; whatever the
    # first call left in the scratch array must not reach this result
    small = workloads.make_decode_case("static-small", 7102, [300, 17, 64], 16, 8, device=DEV)
    out, ref_out, oracle = _both(small, 3, 2)
    assert_bit_exact(out, ref_out, "static vs workspace (second, smaller call)")
    assert_attention_close(out, oracle, "static vs oracle (second, smaller call)")
    # one split per sequence needs no partial results at all
    out, ref_out, oracle = _both(small, 1, 1)
    assert_bit_exact(out, ref_out, "static vs workspace (one split)")


def test_static_scratch_limit_is_enforced():
    print("static decode: limit", flush=True)
    case = workloads.make_decode_case("static-limit", 7103, [64, 64], 64, 8, device=DEV)
    b, hq, d = case.q.shape
    out = torch.empty((b, hq, d), dtype=torch.float16, device=DEV)
    bt = case.block_table.to(torch.int32).contiguous()
    sl = case.seq_lens.to(torch.int32).contiguous()
    too_many = (32 << 20) // (b * hq * (d + 1) * 4) + 1
    with pytest.raises(_lib.LiteKVError, match="built-in scratch holds"):
        ops.paged_decode_static(case.q, case.kv_pool, bt, sl, out, too_many, 1, case.softmax_scale)
    # the largest admissible split count still runs (the grid is mostly idle)
    ops.paged_decode_static(case.q, case.kv_pool, bt, sl, out, too_many - 1, 1, case.softmax_scale)
    torch.cuda.synchronize()
    ref_out = ops.paged_decode(case.q, case.kv_pool, bt, sl, case.softmax_scale, max_splits=too_many - 1,
                               min_pages_per_split=1)
    assert_bit_exact(out, ref_out, "static vs workspace at the limit")
