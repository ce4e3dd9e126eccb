"""GPU: decode metadata advanced on the device and decode steps replayed as HIP graphs.

The device metadata is compared word for word with what the host builders produce (and with the
numpy oracle for the refusal cases); replayed steps are compared bit for bit with the same steps
run eagerly from host-built metadata on a second executor, every replay, with eager work and
synchronisations between replays.
"""

import math

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import ops
from llama_lite_npu_amd.attention import Attention
from llama_lite_npu_amd.executor import DecodeGraphRunner, ModelExecutor
from oracle import c_oracle, decode_metadata
from tests.parity import assert_attention_close, to_np16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HQ, HKV, D = 8, 2, 128
LAYERS = 3
VOCAB = 64
SCALE = 1.0 / math.sqrt(D)
LOG2E = 1.4426950408889634


def _executor(num_pages=160, max_requests=8, max_seq_len=256):
    ex = ModelExecutor(num_layers=LAYERS, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D, num_pages=num_pages,
                       max_seq_len=max_seq_len, max_requests=max_requests, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(5)
    for pool in ex.kv_mem_manager.gpu_kv_buffer:       # the same stale data in every executor of a test
        pool.copy_(torch.randn(pool.shape, generator=g, device=DEV, dtype=torch.float16))
    return ex


class TinyModel:
    """Three attention layers fed from an embedding table: enough to exercise the per-layer calls
    (fused QKV epilogue on even layers, append fused into the decode kernel on odd ones)."""

    def __init__(self, seed=3, max_pos=512):
        g = torch.Generator(device=DEV).manual_seed(seed)
        self.table = torch.randn((VOCAB, LAYERS, HQ + 2 * HKV, D), generator=g, device=DEV, dtype=torch.float16)
        self.wq = (1.0 + 0.1 * torch.randn(D, generator=g, device=DEV)).half()
        self.wk = (1.0 + 0.1 * torch.randn(D, generator=g, device=DEV)).half()
        pos = torch.arange(max_pos, device=DEV, dtype=torch.float64)
        inv = 10000.0 ** (-torch.arange(0, D, 2, device=DEV, dtype=torch.float64) / D)
        emb = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=1)
        self.cos, self.sin = emb.cos().half(), emb.sin().half()
        self.attn = Attention(HQ, HKV, D)
        self.forward_count = 0

    def forward(self, input_ids, position_ids, atten_info):
        self.forward_count += 1
        tokens = input_ids.reshape(-1)
        pos = position_ids.reshape(-1)
        cos, sin = self.cos.index_select(0, pos), self.sin.index_select(0, pos)
        x = self.table.index_select(0, tokens)                     # [B, layers, Hq + 2 Hkv, D]
        acc = torch.zeros((tokens.numel(), HQ, D), dtype=torch.float32, device=DEV)
        for layer in range(LAYERS):
            q, k, v = x[:, layer, :HQ], x[:, layer, HQ:HQ + HKV], x[:, layer, HQ + HKV:]
            if layer % 2 == 0:
                q = self.attn.qkv_epilogue(q, k, v, atten_info, layer, self.wq, self.wk, (cos, sin))
                out = self.attn.token_forward(q, None, None, atten_info, layer, SCALE)
            else:
                out = self.attn.token_forward(q, k, v, atten_info, layer, SCALE)
            acc += out.float()
        return acc


def _next_tokens(out):
    """Token ids of the next step from this step's output, on the device (no host round trip)."""
    return ((out.sum(dim=(1, 2)).abs() * 997.0).long() % VOCAB).reshape(-1, 1)


def _prefill(ex, lens, seed):
    """Reserves one request per length and fills its pages with seeded K/V rows in every layer."""
    ids = ex.reserve_paged_requests(lens)
    ex.activate_paged_packed_prefill_batch(ids, lens)
    g = torch.Generator(device=DEV).manual_seed(seed)
    for layer in range(LAYERS):
        k = torch.randn((sum(lens), HKV, D), generator=g, device=DEV, dtype=torch.float16)
        v = torch.randn((sum(lens), HKV, D), generator=g, device=DEV, dtype=torch.float16)
        ops.kv_append(k, v, ex.atten_info.cur_select_index, ex.atten_info.kv_buffer[layer])
    return ids


def _host_step(ex, model, ids, tokens):
    ex.extend_paged_requests(ids)
    pos = (ex.atten_info.b_seq_len - 1)
    return model.forward(tokens, pos, ex.atten_info)


def _pools_equal(a, b):
    return all(torch.equal(x, y) for x, y in zip(a.kv_mem_manager.gpu_kv_buffer, b.kv_mem_manager.gpu_kv_buffer))


def test_device_metadata_equals_host_metadata_step_by_step():
    print("decode_advance vs host builders", flush=True)
    host, dev = _executor(), _executor()
    lens = [1, 17, 48, 100, 31]
    ids_h, ids_d = _prefill(host, lens, 1), _prefill(dev, lens, 1)
    assert ids_h == ids_d
    batch = dev.activate_device_decode_batch(ids_d, reserve_tokens=8)
    torch.cuda.synchronize()
    # loaded, not advanced: the metadata of the last prompt token
    assert batch.seq_lens_i32.tolist() == lens and batch.position_ids.tolist() == [n - 1 for n in lens]
    for step in range(40):                         # the 8-token reserve runs out on the way
        host.extend_paged_requests(ids_h)
        dev.extend_paged_requests(ids_d)
        assert batch.pending
        batch.enqueue_advance()
        torch.cuda.synchronize()
        hi, di = host.atten_info, dev.atten_info
        assert di.device_decode is batch
        assert torch.equal(hi.b_seq_len, di.b_seq_len) and torch.equal(hi.seq_lens_i32, di.seq_lens_i32)
        assert torch.equal(hi.cur_select_index, di.cur_select_index), step
        assert torch.equal(hi.b_req_idx, di.b_req_idx)
        assert torch.equal(batch.position_ids, hi.b_seq_len - 1)
        w = hi.block_table.shape[1]
        used = (hi.seq_lens_i32 + 15) // 16
        for b in range(len(lens)):                 # beyond a request's pages the host rows hold other padding
            n = int(used[b])
            assert torch.equal(hi.block_table[b, :n], di.block_table[b, :n])
        assert di.block_table.shape[1] == dev.req_tokens_manager.max_pages_per_req >= w
        assert hi.max_actual_seq_len == di.max_actual_seq_len
    batch.check()


def test_decode_advance_refusals_match_the_oracle():
    print("decode_advance refusal cases", flush=True)
    ps, width, num_pages = 16, 3, 16
    tables = np.array([[1, 2, 3, 9], [4, 5, 6, 9]], dtype=np.int32)
    ids = np.array([0, 1, 7, 1, -1], dtype=np.int32)             # 7, -1: no such request
    lens = np.array([48, 32, 3, 0, 5], dtype=np.int32)           # row 0 is at the table's end
    cap = np.array([48, 32, 48, 48, 48], dtype=np.int32)         # row 1 has reached its reserved pages
    for capacity in (cap, None):
        for increment in (1, 0):
            want = decode_metadata.decode_advance(tables, ids, lens, capacity, width, ps, num_pages, increment)
            t = torch.from_numpy(tables).to(DEV)
            seq = torch.from_numpy(lens.copy()).to(DEV)
            seq64 = torch.zeros(5, dtype=torch.int64, device=DEV)
            slot = torch.zeros(5, dtype=torch.int32, device=DEV)
            pos = torch.zeros(5, dtype=torch.int64, device=DEV)
            rows = torch.full((5, width), -7, dtype=torch.int32, device=DEV)
            flag = torch.zeros(1, dtype=torch.int32, device=DEV)
            ops.decode_advance(t, torch.from_numpy(ids).to(DEV), seq, slot, rows, num_pages,
                               capacity=None if capacity is None else torch.from_numpy(capacity).to(DEV),
                               seq_lens_i64=seq64, position_ids=pos, overflow=flag, page_size=ps,
                               increment=increment)
            torch.cuda.synchronize()
            new_lens, slots, positions, table_rows, overflow = want
            assert seq.tolist() == new_lens.tolist() == seq64.tolist()
            assert slot.tolist() == slots.tolist()
            assert pos.tolist() == positions.tolist()
            assert np.array_equal(rows.cpu().numpy(), table_rows)
            assert int(flag.item()) == overflow
    with pytest.raises(Exception, match="increment"):
        ops.decode_advance(t, torch.from_numpy(ids).to(DEV), seq, slot, rows, num_pages, increment=2)
    with pytest.raises(ValueError, match="seq_lens"):
        ops.decode_advance(t, torch.from_numpy(ids).to(DEV), seq.long(), slot, rows, num_pages)


def test_refused_row_appends_nothing_and_attends_nothing():
    """A row whose reserved pages are used up is refused by the device advance; the step's append
    (fused into either decode schedule, or through the slot mapping) must leave its cached tokens
    alone, its output is zero, and the other rows are attended as if it were not there."""
    print("decode step with a refused row", flush=True)
    from llama_lite_npu_amd import workloads

    case = workloads.make_decode_case("refused", 31, [30, 15, 47], HQ, HKV, device=DEV)
    capacity = torch.tensor([32, 15, 48], dtype=torch.int32, device=DEV)     # row 1: 15 cached, no room
    ids = torch.arange(3, dtype=torch.int32, device=DEV)
    for per_sequence in (0, 1, 4):                       # balanced, one wavefront, four splits per sequence
        pool = case.kv_pool.clone()
        seq = case.context_lens.to(DEV).to(torch.int32).clone()
        slot = torch.zeros(3, dtype=torch.int32, device=DEV)
        rows = torch.zeros_like(case.block_table)
        flag = torch.zeros(1, dtype=torch.int32, device=DEV)
        ops.decode_advance(case.block_table, ids, seq, slot, rows, case.num_pages, capacity=capacity, overflow=flag)
        torch.cuda.synchronize()
        assert seq.tolist() == [31, -1, 48] and int(flag.item()) == 1 and int(slot[1]) == -1
        plan = ops.DecodePlan(rows, seq, HQ, HKV, case.num_pages, chunks=5)
        plan.set_schedule(per_sequence)
        out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, SCALE)
        torch.cuda.synchronize()
        want_pool = case.kv_pool.clone()                 # index assignment of the two live rows only
        for b in (0, 2):
            want_pool[int(slot[b]), :HKV], want_pool[int(slot[b]), HKV:] = case.k_new[b], case.v_new[b]
        assert torch.equal(pool, want_pool), "the refused row's pages (or any other slot) were written"
        separate = case.kv_pool.clone()
        ops.kv_append(case.k_new, case.v_new, slot, separate)
        assert torch.equal(separate, want_pool)
        assert float(out[1].abs().max()) == 0.0
        live = torch.tensor([31, 0, 48], dtype=torch.int32)
        ref = c_oracle.paged_decode(to_np16(case.q), to_np16(want_pool), case.block_table.cpu().numpy(),
                                    live.numpy(), SCALE)
        assert_attention_close(out, ref, f"refused row, per_sequence={per_sequence}")
        # the next step refuses the row again instead of restarting it at token 0
        ops.decode_advance(case.block_table, ids, seq, slot, rows, case.num_pages, capacity=capacity, overflow=flag)
        torch.cuda.synchronize()
        assert seq.tolist() == [32, -1, -1] and slot.tolist()[1:] == [-1, -1]


@pytest.mark.parametrize("pinned", [0, 1, 8], ids=["balanced", "one_wavefront", "eight_splits"])
def test_replayed_steps_equal_eager_steps_bit_for_bit(pinned, monkeypatch):
    """Both executors are held on one decode schedule (the host rule would let the device batch keep
    a schedule a little longer than a plan built afresh every step, and two schedules differ in the
    order of their sums)."""
    print(f"graph replay (device metadata) vs eager host metadata, schedule {pinned}", flush=True)
    monkeypatch.setattr(ops, "decode_schedule", lambda *args, **kwargs: pinned)
    host, dev = _executor(), _executor()
    model_h, model_d = TinyModel(), TinyModel()
    lens = [1, 17, 48, 100, 31]
    ids_h, ids_d = _prefill(host, lens, 2), _prefill(dev, lens, 2)
    dev.attach_model(model_d, "qwen3")
    runner = dev.graph_runner
    assert isinstance(runner, DecodeGraphRunner) and runner.available
    batch = dev.activate_device_decode_batch(ids_d, reserve_tokens=8)
    tok_h = tok_d = torch.arange(len(lens), device=DEV).reshape(-1, 1) % VOCAB
    scratch = torch.zeros(1 << 20, device=DEV)
    for step in range(30):
        out_h = _host_step(host, model_h, ids_h, tok_h)
        dev.extend_paged_requests(ids_d)
        out_d = dev.forward(tok_d)                  # positions come from the device batch
        scratch.add_(1.0)                           # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(out_h, out_d), f"step {step}: max diff {(out_h - out_d).abs().max().item()}"
        tok_h, tok_d = _next_tokens(out_h), _next_tokens(out_d)
    assert runner.capture_count == 1 and runner.capture_attempt_count == 1
    assert runner.replay_count == 29 and runner.fallback_count == 0    # the first step ran eagerly, then was captured
    assert model_d.forward_count == 2               # that eager step + the capture; replays never enter Python
    batch.check()
    assert _pools_equal(host, dev)
    # the result is also right, not only equal: last step against the fp32 oracle, layer by layer
    info = dev.atten_info
    g = torch.Generator(device=DEV).manual_seed(12)
    q = torch.randn((len(lens), HQ, D), generator=g, device=DEV, dtype=torch.float16)
    for layer in range(LAYERS):
        got = ops.paged_decode(q, info.kv_buffer[layer], info.block_table, info.seq_lens_i32, SCALE)
        torch.cuda.synchronize()
        ref = c_oracle.paged_decode(to_np16(q), to_np16(info.kv_buffer[layer]), info.block_table.cpu().numpy(),
                                    info.seq_lens_i32.cpu().numpy(), SCALE)
        assert_attention_close(got, ref, "decode over the pages the replays wrote")

    # another set of requests of the same count re-targets the same tensors and the same graph
    for ex, ids in ((host, ids_h), (dev, ids_d)):
        ex.release_paged_request_ids((ids[1],))
    (new_h,), (new_d,) = _prefill(host, [20], 9), _prefill(dev, [20], 9)
    ids_h = (ids_h[0], new_h, *ids_h[2:])
    ids_d = (ids_d[0], new_d, *ids_d[2:])
    assert dev.activate_device_decode_batch(ids_d, reserve_tokens=4) is batch
    for step in range(6):
        out_h = _host_step(host, model_h, ids_h, tok_h)
        dev.extend_paged_requests(ids_d)
        out_d = dev.forward(tok_d)
        torch.cuda.synchronize()
        assert torch.equal(out_h, out_d), f"re-targeted step {step}"
        tok_h, tok_d = _next_tokens(out_h), _next_tokens(out_d)
    assert runner.capture_count == 1 and runner.replay_count == 35
    batch.check()
    assert _pools_equal(host, dev)


def test_host_metadata_steps_replay_through_static_copies(monkeypatch):
    print("graph replay (host metadata, static copies) vs eager", flush=True)
    # one decode schedule for the whole run: a change of schedule is a graph of its own, which
    # test_graph_replay_follows_a_change_of_schedule covers
    monkeypatch.setattr(ops, "decode_schedule", lambda *args, **kwargs: 1)
    host, graphed = _executor(), _executor()
    model_h, model_g = TinyModel(), TinyModel()
    lens = [30, 5, 64]
    ids_h, ids_g = _prefill(host, lens, 4), _prefill(graphed, lens, 4)
    graphed.attach_model(model_g, "qwen3")
    tok_h = tok_g = torch.tensor([[7], [8], [9]], device=DEV)
    for step in range(20):                          # 30 -> 50 and 64 -> 84 open pages: the step's table widens
        out_h = _host_step(host, model_h, ids_h, tok_h)
        graphed.extend_paged_requests(ids_g)
        out_g = graphed.forward(tok_g, graphed.atten_info.b_seq_len - 1)
        torch.cuda.synchronize()
        assert torch.equal(out_h, out_g), f"step {step}"
        tok_h, tok_g = _next_tokens(out_h), _next_tokens(out_g)
    runner = graphed.graph_runner
    assert runner.capture_count == 1 and runner.replay_count == 20 and runner.fallback_count == 0
    assert _pools_equal(host, graphed)


def _shared_prefix_batch(ex, model):
    """Three requests whose first 6 pages are one cached system prompt; returns their ids."""
    attn = model.attn
    system = tuple(range(2000, 2096))           # 6 full pages
    g = torch.Generator(device=DEV).manual_seed(77)

    def rows(n, heads):
        return torch.randn((n, heads, D), generator=g, device=DEV, dtype=torch.float16)

    (a,) = ex.reserve_paged_requests([96])
    ex.activate_paged_packed_prefill_batch((a,), [96])
    for layer in range(LAYERS):
        attn.context_forward(rows(96, HQ), rows(96, HKV), rows(96, HKV), ex.atten_info, layer, SCALE * LOG2E)
    ex.store_paged_request_prefix(system, a, first_token_id=5)
    batch_ids = [a]
    for i, extra in enumerate((20, 3)):
        prompt = system + tuple(range(3000 + 100 * i, 3000 + 100 * i + extra))
        req, matched, _ = ex.share_paged_prefix_from_cache(prompt)
        assert matched == 96
        ex.ensure_paged_request_capacity(req, 96 + extra + 8)
        ex.activate_paged_chunk_prefill_batch((req,), [96], [extra])
        for layer in range(LAYERS):
            attn.context_forward(rows(extra, HQ), rows(extra, HKV), rows(extra, HKV), ex.atten_info, layer,
                                 SCALE * LOG2E)
        batch_ids.append(req)
    return tuple(batch_ids)


def test_graph_of_a_shared_prefix_batch_is_not_replayed_for_a_batch_sharing_nothing(monkeypatch):
    """Host-metadata steps replay through a static plan made at capture. A batch that shares a
    cached prefix and a batch of the same size that shares nothing need different plans: each
    must get its own graph, every replay equal to the eager step bit for bit."""
    print("graph replay: shared-prefix batch, then a same-size batch without one", flush=True)
    monkeypatch.setattr(ops, "decode_schedule", lambda *args, **kwargs: 1)   # the private batch on one schedule
    host, graphed = _executor(num_pages=200, max_requests=8), _executor(num_pages=200, max_requests=8)
    model_h, model_g = TinyModel(), TinyModel()
    shared_h, shared_g = _shared_prefix_batch(host, model_h), _shared_prefix_batch(graphed, model_g)
    private_h, private_g = _prefill(host, [40, 7, 70], 9), _prefill(graphed, [40, 7, 70], 9)
    assert shared_h == shared_g and private_h == private_g
    graphed.attach_model(model_g, "qwen3")
    tok_h = tok_g = torch.tensor([[1], [2], [3]], device=DEV)
    for phase, (ids_h, ids_g, shared) in enumerate(((shared_h, shared_g, 6), (private_h, private_g, 0),
                                                    (shared_h, shared_g, 6), (private_h, private_g, 0))):
        for step in range(3):
            out_h = _host_step(host, model_h, ids_h, tok_h)
            assert host.atten_info.decode_plan.shared_pages == shared
            graphed.extend_paged_requests(ids_g)
            out_g = graphed.forward(tok_g, graphed.atten_info.b_seq_len - 1)
            torch.cuda.synchronize()
            assert torch.equal(out_h, out_g), f"phase {phase} step {step}"
            tok_h, tok_g = _next_tokens(out_h), _next_tokens(out_g)
    runner = graphed.graph_runner
    assert runner.capture_count == 2 and runner.replay_count == 12 and runner.fallback_count == 0
    assert _pools_equal(host, graphed)


def test_shared_prefix_batch_steps_on_the_device():
    print("graph replay over a shared cached prefix", flush=True)
    outs = []
    for use_device in (False, True):
        ex = _executor(num_pages=160)
        model = TinyModel()
        ids = _shared_prefix_batch(ex, model)
        tok = torch.tensor([[1], [2], [3]], device=DEV)
        steps = []
        if use_device:
            ex.attach_model(model, "qwen3")
            batch = ex.activate_device_decode_batch(ids, reserve_tokens=16)
            assert batch.shared_pages == 6 and batch.decode_plan.shared_pages == 6
        for step in range(12):
            if use_device:
                ex.extend_paged_requests(ids)
                out = ex.forward(tok)
            else:
                out = _host_step(ex, model, ids, tok)
                assert ex.atten_info.decode_plan.shared_pages == 6
            torch.cuda.synchronize()
            steps.append(out.clone())
            tok = _next_tokens(out)
        if use_device:
            batch.check()
            assert ex.graph_runner.replay_count == 11
        outs.append(steps)
    for step, (h, d) in enumerate(zip(*outs)):
        assert torch.equal(h, d), f"step {step}"
