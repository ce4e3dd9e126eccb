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


_CAPTURE_SCRIPT = r"""
import sys
import torch
sys.path.insert(0, sys.argv[1])
from llama_lite_npu_amd import _lib, ops, workloads

dev = "cuda:0"
case = workloads.make_decode_case("static-capture", 7201, [300, 17, 64, 900], 16, 8, device=dev)
bt = case.block_table.to(torch.int32).contiguous()
sl = case.seq_lens.to(torch.int32).contiguous()
want = ops.paged_decode(case.q, case.kv_pool, bt, sl, case.softmax_scale, max_splits=3, min_pages_per_split=2)
out = torch.zeros_like(want)
torch.cuda.synchronize()

# the very first call of this process on the device, inside a capture: refused, capture intact
g = torch.cuda.CUDAGraph()
refused = ""
with torch.cuda.graph(g):
    out.add_(0)
    try:
        ops.paged_decode_static(case.q, case.kv_pool, bt, sl, out, 3, 2, case.softmax_scale)
    except _lib.LiteKVError as e:
        refused = str(e)
assert "capture" in refused, refused
g.replay()
torch.cuda.synchronize()
assert float(out.abs().max()) == 0.0
print("refused:", refused, flush=True)

# the warm-up call (batch 0) resolves the array's address; then the same capture holds the step
empty = torch.empty((0,) + tuple(case.q.shape[1:]), dtype=torch.float16, device=dev)
ops.paged_decode_static(empty, case.kv_pool, bt[:0], sl[:0], empty.clone(), 3, 2, case.softmax_scale)
g2 = torch.cuda.CUDAGraph()
with torch.cuda.graph(g2):
    ops.paged_decode_static(case.q, case.kv_pool, bt, sl, out, 3, 2, case.softmax_scale)
for replay in range(3):
    out.fill_(float("nan"))
    torch.cuda.synchronize()
    g2.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want), f"replay {replay} differs"
print("captured after warm-up: ok", flush=True)
"""


def test_first_static_call_inside_a_capture_is_refused_and_a_warm_up_call_enables_it():
    """The array's address is looked up on the first call on a device, which a stream capture
    cannot hold: such a call is refused with a message, and a call with batch 0 beforehand makes
    the entry point capturable. Needs a process that has not called the entry point yet."""
    import subprocess
    import sys
    from pathlib import Path

    print("static decode: first call under capture (own process)", flush=True)
    root = str(Path(__file__).resolve().parents[1])
    proc = subprocess.run([sys.executable, "-u", "-c", _CAPTURE_SCRIPT, root], capture_output=True, text=True,
                          timeout=300)
    print(proc.stdout, proc.stderr[-2000:], flush=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "captured after warm-up: ok" in proc.stdout
