"""GPU: the continuous-batching backend driving the real executor and HIP kernels end to end.

A small language model (embedding table -> three attention layers on the paged cache -> vocabulary
projection) is generated from greedily. The same requests are run through differently configured
backends -- device-side decode metadata with graph replay against the reference's per-step host
metadata, chunked against one-shot prefill, prefix-cache hits against cold runs -- and must
produce the same tokens; the page bookkeeping of a cache hit is checked directly.
"""

import math
from types import SimpleNamespace

import pytest
import torch

from llama_lite_npu_amd.attention import Attention
from llama_lite_npu_amd.continuous_batching import BatchRequest, ContinuousBatchModelBackend
from llama_lite_npu_amd.executor import ModelExecutor

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HQ, HKV, D = 8, 2, 128
LAYERS = 3
VOCAB = 96
SCALE = 1.0 / math.sqrt(D)
LOG2E = 1.4426950408889634


class TinyLM:
    def __init__(self, seed=21, max_pos=512):
        g = torch.Generator(device=DEV).manual_seed(seed)
        self.table = torch.randn((VOCAB, LAYERS, HQ + 2 * HKV, D), generator=g, device=DEV, dtype=torch.float16)
        self.wq = (1.0 + 0.1 * torch.randn(D, generator=g, device=DEV)).half()
        self.wk = (1.0 + 0.1 * torch.randn(D, generator=g, device=DEV)).half()
        self.head = torch.randn((D, VOCAB), generator=g, device=DEV, dtype=torch.float32)
        pos = torch.arange(max_pos, device=DEV, dtype=torch.float64)
        inv = 10000.0 ** (-torch.arange(0, D, 2, device=DEV, dtype=torch.float64) / D)
        emb = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=1)
        self.cos, self.sin = emb.cos().half(), emb.sin().half()
        self.attn = Attention(HQ, HKV, D)
        self.calls = 0              # graph replays do not come through here

    def forward(self, input_ids, position_ids, atten_info):
        self.calls += 1
        tokens, pos = input_ids.reshape(-1), position_ids.reshape(-1)
        decode = input_ids.shape[1] == 1
        cos, sin = self.cos.index_select(0, pos), self.sin.index_select(0, pos)
        x = self.table.index_select(0, tokens)
        acc = torch.zeros((tokens.numel(), HQ, D), dtype=torch.float32, device=DEV)
        for layer in range(LAYERS):
            q, k, v = x[:, layer, :HQ], x[:, layer, HQ:HQ + HKV], x[:, layer, HQ + HKV:]
            q = self.attn.qkv_epilogue(q, k, v, atten_info, layer, self.wq, self.wk, (cos, sin))
            if decode:
                out = self.attn.token_forward(q, None, None, atten_info, layer, SCALE)
            else:
                out = self.attn.context_forward(q, None, None, atten_info, layer, SCALE * LOG2E)
            acc += out.float()
        logits = acc.mean(dim=1) @ self.head
        return logits.reshape(*input_ids.shape, VOCAB)


def _backend(use_graph=True, device_decode=True, num_pages=200, max_prefill_tokens=None, **kw):
    ex = ModelExecutor(num_layers=LAYERS, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D, num_pages=num_pages,
                       max_seq_len=256, max_requests=12, device=DEV)
    for pool in ex.kv_mem_manager.gpu_kv_buffer:
        pool.zero_()
    if max_prefill_tokens is not None:
        ex.max_prefill_tokens = max_prefill_tokens
    ex.attach_model(TinyLM(), "qwen3", use_graph=use_graph)
    tokenizer = SimpleNamespace(eos_token_id=VOCAB + 1)
    be = ContinuousBatchModelBackend(SimpleNamespace(model_executor=ex, tokenizer=tokenizer),
                                     device_decode=device_decode, **kw)
    return be, ex


def _prompt(seed, n):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, VOCAB, (n,), generator=g).tolist()


def _accept(requests, tokens):
    for r, t in zip(requests, tokens):
        r.generated_token_ids.append(int(t))


def _script(be, steps_before=10, steps_after=14):
    """Five requests, ten decode steps, one request leaves and another joins, fourteen more."""
    reqs = [BatchRequest(f"r{i}", _prompt(i, n), 64, 0.0, 1.0) for i, n in enumerate((5, 33, 16, 70, 1))]
    log = [list(be.prefill(reqs))]
    _accept(reqs, log[-1])
    for _ in range(steps_before):
        log.append(list(be.decode(reqs)))
        _accept(reqs, log[-1])
    be.release([reqs[1]])
    newcomer = BatchRequest("late", _prompt(9, 21), 64, 0.0, 1.0)
    log.append(list(be.prefill([newcomer])))
    _accept([newcomer], log[-1])
    reqs = [reqs[0], newcomer, *reqs[2:]]
    for _ in range(steps_after):
        log.append(list(be.decode(reqs)))
        _accept(reqs, log[-1])
    torch.cuda.synchronize()
    return log, reqs


def test_device_decode_with_graph_replay_generates_the_same_tokens():
    print("backend: device decode + graph vs host metadata, eager", flush=True)
    plain, ex_plain = _backend(use_graph=False, device_decode=False)
    fast, ex_fast = _backend(use_graph=True, device_decode=True, decode_reserve_tokens=8)
    assert fast.device_decode and not plain.device_decode
    want, _ = _script(plain)
    got, reqs = _script(fast)
    assert got == want
    runner = ex_fast.graph_runner
    assert runner.capture_count >= 1 and runner.replay_count >= 20 and runner.fallback_count == 0
    ex_fast._device_batch.check()
    counts = ex_fast.req_tokens_manager.req_token_count
    for r in reqs:                      # the last sampled token has its slot, its K/V come with the next step
        assert counts[r.model_request_id] == len(r.model_context_tokens)
    assert ex_fast.model.calls < ex_plain.model.calls - 15      # most decode steps never entered Python


def test_device_decode_without_graphs_and_host_decode_with_graphs_agree_too():
    print("backend: the two mixed configurations", flush=True)
    want, _ = _script(_backend(use_graph=False, device_decode=False)[0], 6, 6)
    assert _script(_backend(use_graph=False, device_decode=True)[0], 6, 6)[0] == want
    assert _script(_backend(use_graph=True, device_decode=False)[0], 6, 6)[0] == want


def test_an_exact_cache_hit_shares_full_pages_and_owns_its_last_page():
    print("backend: exact prefix hit with copy-on-write", flush=True)
    be, ex = _backend()
    mgr, pages = ex.req_tokens_manager, ex.kv_mem_manager
    prompt = _prompt(3, 20)                               # one full page + 4 tokens
    first = BatchRequest("first", prompt, 32, 0.0, 1.0)
    (t0,) = be.prefill([first])
    _accept([first], [t0])
    forwards_before = ex.model.calls
    second = BatchRequest("second", prompt, 32, 0.0, 1.0)
    (t1,) = be.prefill([second])
    assert t1 == t0 and second.prefill_cursor == 20
    assert ex.model.calls == forwards_before              # nothing was computed for the hit
    pa, pb = mgr.request_pages(first.model_request_id), mgr.request_pages(second.model_request_id)
    assert pa[0] == pb[0] and pa[1] != pb[1]              # full page shared, partly filled page copied
    assert pages.refcount(pa[0]) == 4                     # two requests, the exact entry and the block entry
    assert pages.refcount(pa[1]) == 2 and pages.refcount(pb[1]) == 1
    for pool in pages.gpu_kv_buffer:                      # the copy holds the cached rows
        assert torch.equal(pool[pa[1] * 16: pa[1] * 16 + 4], pool[pb[1] * 16: pb[1] * 16 + 4])
    _accept([second], [t1])
    # the first request runs ahead for three steps, then both decode together
    solo = [be.decode([first])[0] for _ in range(3)]
    _accept([first], solo[:1]); _accept([first], solo[1:2]); _accept([first], solo[2:3])
    both = []
    for _ in range(3):
        a, b = be.decode([first, second])
        _accept([first, second], [a, b])
        both.append((a, b))
    assert [b for _, b in both] == solo                   # the sharer repeats what the first one generated
    # a cold run on a fresh executor gives the same continuation
    cold_be, _ = _backend()
    cold = BatchRequest("cold", prompt, 32, 0.0, 1.0)
    tokens = list(cold_be.prefill([cold]))
    _accept([cold], tokens)
    for _ in range(6):
        tokens += cold_be.decode([cold])
        _accept([cold], tokens[-1:])
    assert tokens == first.generated_token_ids
    # the cached entry still serves a third request after both have appended
    third = BatchRequest("third", prompt, 32, 0.0, 1.0)
    assert be.prefill([third]) == [t0]
    _accept([third], [t0])
    assert be.decode([third])[0] == solo[0]


def test_chunked_prefill_generates_what_one_shot_prefill_generates():
    print("backend: chunked prefill vs one shot", flush=True)
    lengths = (40, 7, 33)
    whole_be, _ = _backend()
    whole = [BatchRequest(f"w{i}", _prompt(30 + i, n), 16, 0.0, 1.0) for i, n in enumerate(lengths)]
    want = list(whole_be.prefill(whole))
    _accept(whole, want)
    chunk_be, ex = _backend()
    chunked = [BatchRequest(f"c{i}", _prompt(30 + i, n), 16, 0.0, 1.0) for i, n in enumerate(lengths)]
    got = [None] * 3
    rounds = 0
    while any(t is None for t in got):
        waiting = [i for i, t in enumerate(got) if t is None]
        chunk_be.prepare_prefill_chunk([chunked[i] for i in waiting], 16)
        for i, t in zip(waiting, chunk_be.prefill_chunk([chunked[i] for i in waiting], 16)):
            got[i] = t
        rounds += 1
    assert rounds == 3 and got == want                    # 40 tokens need three chunks of 16
    _accept(chunked, got)
    for _ in range(5):
        a, b = whole_be.decode(whole), chunk_be.decode(chunked)
        assert a == b
        _accept(whole, a)
        _accept(chunked, b)
    counts = ex.req_tokens_manager.req_token_count
    assert [counts[r.model_request_id] for r in chunked] == [n + 6 for n in lengths]


def test_a_block_prefix_hit_replays_the_suffix_over_shared_pages():
    print("backend: block prefix hit", flush=True)
    be, ex = _backend(enable_partial_prefix_cache=True)
    base = _prompt(50, 40)
    first = BatchRequest("first", base, 16, 0.0, 1.0)
    be.prefill([first])
    other = base[:32] + _prompt(51, 9)                    # two cached blocks, then its own tokens
    second = BatchRequest("second", other, 16, 0.0, 1.0)
    (got,) = be.prefill([second])
    mgr = ex.req_tokens_manager
    pa, pb = mgr.request_pages(first.model_request_id), mgr.request_pages(second.model_request_id)
    assert pa[:2] == pb[:2] and pa[2] != pb[2]
    assert second.prefill_cursor == 41
    cold_be, _ = _backend()
    cold = BatchRequest("cold", other, 16, 0.0, 1.0)
    (want,) = cold_be.prefill([cold])
    assert got == want
    _accept([second], [got]); _accept([cold], [want])
    for _ in range(4):
        (a,), (b,) = be.decode([second]), cold_be.decode([cold])
        assert a == b
        _accept([second], [a]); _accept([cold], [b])


def test_prompts_over_the_prefill_budget_are_replayed_and_still_agree():
    print("backend: prefill budget", flush=True)
    roomy, _ = _backend()
    tight, _ = _backend(max_prefill_tokens=24)
    lengths = (30, 10, 12, 5)
    a = [BatchRequest(f"a{i}", _prompt(70 + i, n), 8, 0.0, 1.0) for i, n in enumerate(lengths)]
    b = [BatchRequest(f"b{i}", _prompt(70 + i, n), 8, 0.0, 1.0) for i, n in enumerate(lengths)]
    assert list(roomy.prefill(a)) == list(tight.prefill(b))
