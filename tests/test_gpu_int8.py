"""GPU parity of the int8 KV pool (signed 8-bit codes, one fp32 scale per kv head) through the C ABI:
codes written by the append, by the fused epilogue and by the append fused into decode are
bit-equal to the numpy oracle's, page dequantisation is bit-equal to code * scale rounded to fp16,
and attention over an int8 pool (decode, both schedules; chunk prefill; shared prefix) is within
the attention tolerance of the fp32 oracle applied to the decoded pool."""

import math
import random

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import ops, workloads
from oracle import cpu_ref, int8
from tests.parity import assert_attention_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = 128
SCALE = 1.0 / math.sqrt(D)


def _head_scales(hkv, k_scale=6.0 / 127, v_scale=5.0 / 127):
    return torch.cat([k_scale * (1 + 0.1 * torch.arange(hkv)), v_scale * (1 + 0.2 * torch.arange(hkv))]).float().to(DEV)


def test_append_codes_equal_the_oracle_for_every_fp16_input():
    print("int8 append: every fp16 value", flush=True)
    hkv = 2
    halves = np.arange(0x10000, dtype=np.uint16).view(np.float16)
    vals = halves[np.isfinite(halves) & (np.abs(halves.astype(np.float32)) <= 2000.0)]   # saturation included
    t = (vals.size + hkv * D - 1) // (hkv * D)
    flat = np.zeros(t * hkv * D, dtype=np.float16)
    flat[:vals.size] = vals
    k = flat.reshape(t, hkv, D)
    v = k[::-1].copy()
    scales = np.array([1.0, 0.37, 3.0, 0.011], dtype=np.float32)
    slots = np.random.default_rng(0).permutation(t + 16)[:t].astype(np.int32)
    slots[5] = -1                                            # a padded row
    pool = torch.full((t + 16, 2 * hkv, D), 0x55, dtype=torch.int8, device=DEV)
    ops.kv_append_quantised(torch.from_numpy(k).to(DEV), torch.from_numpy(v).to(DEV), torch.from_numpy(slots).to(DEV),
                            pool, torch.from_numpy(scales).to(DEV))
    torch.cuda.synchronize()
    want = np.full((t + 16, 2 * hkv, D), 0x55, dtype=np.int8)
    int8.kv_append(k, v, slots, want, scales)
    got = pool.cpu().numpy()
    assert int((got != want).sum()) == 0, f"{int((got != want).sum())} codes differ"
    assert got.min() >= -127                                 # -128 is never stored


def test_page_dequant_is_code_times_scale():
    print("int8 page dequant", flush=True)
    hkv, pages = 2, 6
    codes = np.arange(pages * 16 * 2 * hkv * D, dtype=np.uint32)
    codes = ((codes * 2654435761) >> 13).astype(np.uint8).view(np.int8)   # every code many times, in no order
    pool = torch.from_numpy(codes.reshape(pages * 16, 2 * hkv, D).copy()).to(DEV)
    scales = np.array([0.5, 0.013, 1.7, 0.25], dtype=np.float32)
    dst = torch.zeros((4 * 16, 2 * hkv, D), dtype=torch.float16, device=DEV)
    src_ids = torch.tensor([5, 0, 9, 2], dtype=torch.int32, device=DEV)   # 9: out of range, skipped
    ops.page_dequant(pool, dst, src_ids, None, torch.from_numpy(scales).to(DEV))
    torch.cuda.synchronize()
    full = int8.dequantize_pool(codes.reshape(pages * 16, 2 * hkv, D), scales).astype(np.float16)
    got = dst.cpu().numpy()
    for i, page in enumerate((5, 0, None, 2)):
        block = got[16 * i: 16 * i + 16]
        if page is None:
            assert np.all(block == 0)
        else:
            assert np.array_equal(block.view(np.uint16), full[16 * page: 16 * page + 16].view(np.uint16))


def _int8_case(seed, lens, hq, hkv, page_size=16):
    """Random fp16 K/V quantised into a shuffled int8 pool by the append kernel; returns what decode needs."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    b = len(lens)
    pages_per = [(n + page_size - 1) // page_size for n in lens]
    num_pages = sum(pages_per) + 7
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    table = torch.zeros((b, max(1, max(pages_per))), dtype=torch.int32)
    slots, cur = [], 0
    for i, n in enumerate(lens):
        ids = perm[cur:cur + pages_per[i]]
        cur += pages_per[i]
        table[i, :len(ids)] = torch.tensor(ids, dtype=torch.int32)
        slots += [ids[t // page_size] * page_size + t % page_size for t in range(n)]
    total = sum(lens)
    k = torch.randn((total, hkv, D), generator=g, device=DEV, dtype=torch.float16)
    v = torch.randn((total, hkv, D), generator=g, device=DEV, dtype=torch.float16)
    scales = _head_scales(hkv)
    pool = torch.randint(-127, 128, (num_pages * page_size, 2 * hkv, D), generator=g, device=DEV, dtype=torch.int8)
    ops.kv_append_quantised(k, v, torch.tensor(slots, dtype=torch.int32, device=DEV), pool, scales)
    q = torch.randn((b, hq, D), generator=g, device=DEV, dtype=torch.float16)
    return q, pool, scales, table.to(DEV), torch.tensor(lens, dtype=torch.int32, device=DEV)


def _oracle(q, pool, scales, table, lens, page_size=16):
    values = torch.from_numpy(int8.dequantize_pool(pool.cpu().numpy(), scales.cpu().numpy()))
    return cpu_ref.paged_decode_ref(q.cpu(), values, table.cpu(), lens.cpu(), SCALE, page_size=page_size).numpy()


@pytest.mark.parametrize("hq,hkv", [(8, 2), (64, 8), (16, 16), (4, 1)])
def test_decode_over_an_int8_pool_matches_the_oracle_on_the_decoded_values(hq, hkv):
    print(f"int8 decode hq={hq} hkv={hkv}", flush=True)
    lens = [1, 16, 17, 250, 0, 999, 64]
    q, pool, scales, table, seq_lens = _int8_case(11 + hq, lens, hq, hkv)
    ref = _oracle(q, pool, scales, table, seq_lens)
    out = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    assert_attention_close(out, ref, "int8 decode")
    assert torch.all(out[4] == 0)                            # the empty sequence
    again = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales)
    other = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales, chunks=37)
    torch.cuda.synchronize()
    assert torch.equal(out, again)
    assert_attention_close(other, ref, "int8 decode, 37 chunks")
    for kw in ({"num_splits": 1}, {"num_splits": 4}, {"max_splits": 16, "min_pages_per_split": 2}):
        out = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales, **kw)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"int8 splits {kw}")
        assert float(out[4].abs().max()) == 0.0


def test_int8_pool_with_pages_of_64_tokens():
    print("int8 decode, page_size 64", flush=True)
    lens = [1, 16, 17, 63, 64, 65, 250, 0, 999]
    q, pool, scales, table, seq_lens = _int8_case(17, lens, 32, 4, page_size=64)
    ref = _oracle(q, pool, scales, table, seq_lens, page_size=64)
    for kw in ({}, {"chunks": 5}, {"num_splits": 1}, {"num_splits": 3}):
        out = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales, page_size=64, **kw)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"int8 page_size 64 {kw}")


def test_quantisation_error_is_the_only_difference_from_fp16():
    """The same K/V in an fp16 pool: outputs differ by what 127 levels over +-6 sigma allow, not more."""
    print("int8 vs fp16 decode", flush=True)
    hq, hkv, lens = 16, 4, [300, 77]
    g = torch.Generator(device=DEV).manual_seed(5)
    k = torch.randn((sum(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    v = torch.randn((sum(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    q = torch.randn((2, hq, D), generator=g, device=DEV, dtype=torch.float16)
    slots = torch.cat([torch.arange(lens[0]) + 16, torch.arange(lens[1]) + 24 * 16]).to(torch.int32).to(DEV)
    table = torch.zeros((2, 20), dtype=torch.int32, device=DEV)
    table[0, :19] = torch.arange(1, 20)
    table[1, :5] = torch.arange(24, 29)
    pool16 = torch.zeros((30 * 16, 2 * hkv, D), dtype=torch.float16, device=DEV)
    pool8 = torch.zeros((30 * 16, 2 * hkv, D), dtype=torch.int8, device=DEV)
    scales = torch.full((2 * hkv,), 6.0 / 127.0, device=DEV)
    ops.kv_append(k, v, slots, pool16)
    ops.kv_append_quantised(k, v, slots, pool8, scales)
    seq_lens = torch.tensor(lens, dtype=torch.int32, device=DEV)
    o16 = ops.paged_decode(q, pool16, table, seq_lens, SCALE)
    o8 = ops.paged_decode(q, pool8, table, seq_lens, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    err = (o16.float() - o8.float()).abs().max().item()
    assert 1e-5 < err < 2e-2, err                          # visibly quantised, and bounded


def test_fused_append_writes_the_same_codes_and_attends_them():
    print("int8 decode with fused append", flush=True)
    hq, hkv = 16, 4
    lens = [33, 16, 1, 130]                                # lengths already counting the new token
    q, pool, scales, table, seq_lens = _int8_case(23, lens, hq, hkv)
    g = torch.Generator(device=DEV).manual_seed(99)
    k_new = torch.randn((len(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16) * 3   # some codes saturate
    v_new = torch.randn((len(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    last_slots = torch.stack([table[i, (n - 1) // 16] * 16 + (n - 1) % 16 for i, n in enumerate(lens)]).int()
    separate = pool.clone()
    ops.kv_append_quantised(k_new, v_new, last_slots, separate, scales)
    want_out = ops.paged_decode(q, separate, table, seq_lens, SCALE, kv_scales=scales)
    plan = ops.DecodePlan(table, seq_lens, hq, hkv, pool.shape[0] // 16)
    fused = pool.clone()
    got_out = ops.decode_step(q, fused, plan, k_new, v_new, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(fused, separate)                    # same codes in the same slots, nothing else touched
    assert torch.equal(got_out, want_out)
    assert_attention_close(got_out, _oracle(q, fused, scales, table, seq_lens), "int8 fused append + decode")
    # the per-sequence schedule with its fused append
    fused2 = pool.clone()
    out2 = ops.paged_decode(q, fused2, table, seq_lens, SCALE, kv_scales=scales, num_splits=1, k_new=k_new, v_new=v_new)
    torch.cuda.synchronize()
    assert torch.equal(fused2, separate)
    assert_attention_close(out2, _oracle(q, fused2, scales, table, seq_lens), "int8 per-sequence fused append")


def test_int8_pages_move_with_the_page_copy_and_gather_kernels():
    print("int8 page moves", flush=True)
    q, pool, scales, table, seq_lens = _int8_case(31, [40, 90], 8, 2)
    before = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales)
    n_pages = pool.shape[0] // 16
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(1)).to(torch.int32).to(DEV)
    moved = torch.zeros_like(pool)
    ops.page_gather(pool, moved, torch.arange(n_pages, dtype=torch.int32, device=DEV), order)
    remapped = order[table.long()]
    after = ops.paged_decode(q, moved, remapped.int(), seq_lens, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(before, after)


def test_argument_checks():
    q, pool, scales, table, seq_lens = _int8_case(41, [20], 8, 2)
    with pytest.raises(ValueError, match="scales"):
        ops.paged_decode(q, pool, table, seq_lens, SCALE)
    with pytest.raises(ValueError, match="scales"):
        ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales[:3])


@pytest.mark.parametrize("t", [77, 8197])          # one token per lane, and four (prefill-sized launches)
def test_fused_epilogue_into_an_int8_pool_equals_epilogue_then_quantising_append(t):
    print(f"int8: fused QK-norm + RoPE + quantising append, {t} tokens", flush=True)
    hq, hkv = 16, 4
    n_slots = max(256, 2 * t)
    g = torch.Generator(device=DEV).manual_seed(61)
    qkv = torch.randn((t, hq + 2 * hkv, D), generator=g, device=DEV, dtype=torch.float16) * 1.5
    q, k, v = qkv[:, :hq], qkv[:, hq:hq + hkv], qkv[:, hq + hkv:]
    wq = (1.0 + 0.2 * torch.randn(D, generator=g, device=DEV)).half()
    wk = (1.0 + 0.2 * torch.randn(D, generator=g, device=DEV)).half()
    pos = torch.randint(0, 4096, (t,), generator=g, device=DEV).double()
    inv = 10000.0 ** (-torch.arange(0, D, 2, device=DEV, dtype=torch.float64) / D)
    emb = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=1)
    cos, sin = emb.cos().half(), emb.sin().half()
    slots = torch.randperm(n_slots, generator=torch.Generator().manual_seed(3))[:t].to(torch.int32).to(DEV)
    slots[7] = -1
    scales = torch.tensor([0.02, 0.03, 0.025, 0.04, 0.015, 0.02, 0.01, 0.03], device=DEV)
    q_a = q.clone()
    rows = torch.empty((t, 2 * hkv, D), dtype=torch.float16, device=DEV)
    ops.qk_norm_rope_append(q_a, k, v, torch.arange(t, dtype=torch.int32, device=DEV), rows, wq, wk, cos, sin)
    pool_a = torch.full((n_slots, 2 * hkv, D), 0x55, dtype=torch.int8, device=DEV)
    ops.kv_append_quantised(rows[:, :hkv], rows[:, hkv:], slots, pool_a, scales)
    q_b = q.clone()
    pool_b = torch.full((n_slots, 2 * hkv, D), 0x55, dtype=torch.int8, device=DEV)
    ops.qk_norm_rope_append(q_b, k, v, slots, pool_b, wq, wk, cos, sin, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(q_a, q_b)
    assert torch.equal(pool_a, pool_b)
    assert int((pool_b != 0x55).any(dim=(1, 2)).sum()) == t - 1          # the padded token stored nothing


@pytest.mark.parametrize("seed", range(2))
def test_chunk_prefill_reads_an_int8_pool_directly(seed):
    """Chunk rows over an int8 history (and their own rows, appended as codes): the oracle on the
    decoded pool, within the attention tolerance; agrees with dequantising the pages first."""
    rng = random.Random(700 + seed)
    for case_no in range(6):
        hq, hkv = rng.choice([(64, 8), (32, 4), (16, 8), (8, 8), (4, 2), (16, 1)])
        b = rng.choice([1, 2, 4])
        edges = [1, 15, 16, 17, 63, 64, 65, 128]
        q_lens = [rng.choice([rng.choice(edges), rng.randint(1, 300)]) for _ in range(b)]
        ctx = [rng.choice([0, rng.choice(edges), rng.randint(0, 900)]) for _ in range(b)]
        print(f"int8 chunk prefill {seed}.{case_no}: heads {hq}/{hkv} chunks {q_lens} histories {ctx}", flush=True)
        case = workloads.make_prefill_case("int8", 8100 + 100 * seed + case_no, q_lens, hq, hkv, context_lens=ctx,
                                           device=DEV)
        scales = _head_scales(hkv)
        pool = torch.empty(case.kv_pool.shape, dtype=torch.int8, device=DEV)
        every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
        ops.kv_append_quantised(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every_slot, pool, scales)   # the history
        ops.kv_append_quantised(case.k, case.v, case.slot_mapping, pool, scales)                          # the chunk
        out = ops.paged_prefill(case.q, pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len,
                                SCALE, kv_scales=scales)
        again = ops.paged_prefill(case.q, pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len,
                                  SCALE, kv_scales=scales)
        torch.cuda.synchronize()
        values = torch.from_numpy(int8.dequantize_pool(pool.cpu().numpy(), scales.cpu().numpy()))
        ref = cpu_ref.paged_prefill_ref(case.q.cpu(), values, case.block_table.cpu(), case.cu_q_lens.cpu(),
                                        case.context_lens.cpu(), SCALE).numpy()
        assert_attention_close(out, ref, f"int8 chunk prefill {seed}.{case_no}")
        assert torch.equal(out, again)
        scratch = torch.zeros(case.kv_pool.shape, dtype=torch.float16, device=DEV)
        all_pages = torch.arange(case.num_pages, dtype=torch.int32, device=DEV)
        ops.page_dequant(pool, scratch, all_pages, all_pages, scales)
        two_pass = ops.paged_prefill(case.q, scratch, case.block_table, case.cu_q_lens, case.context_lens,
                                     case.max_q_len, SCALE)
        assert float((two_pass.float() - out.float()).abs().max()) <= 2e-3


def _rows(tokens, heads, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return torch.randn((tokens, heads, D), generator=g, device=DEV, dtype=torch.float16)


def test_executor_on_int8_pools_with_a_shared_system_prompt():
    """Three requests share a 96-token prefix through the block cache of an int8 executor: prompts
    and chunks are quantised on their way in, the decode step gets a shared-prefix plan, and every
    step equals the oracle on the decoded pool."""
    print("int8: executor, chunk prefill, shared prefix decode", flush=True)
    from llama_lite_npu_amd.attention import Attention
    from llama_lite_npu_amd.executor import ModelExecutor

    hq, hkv = 16, 8
    ex = ModelExecutor(num_layers=1, num_q_heads=hq, num_kv_heads=hkv, head_dim=D, num_pages=128,
                       max_seq_len=512, max_requests=8, device=DEV, dtype=torch.int8)
    ex.kv_mem_manager.gpu_kv_buffer[0].fill_(0x55)
    ex.kv_mem_manager.set_kv_scales(0, [6.0 / 127 + 0.001 * h for h in range(hkv)], [5.0 / 127 + 0.002 * h for h in range(hkv)])
    assert ex.atten_info.kv_scales[0] is not None
    attn = Attention(hq, hkv, D)
    log2e = 1.4426950408889634

    def decoded():
        pool = ex.kv_mem_manager.gpu_kv_buffer[0].cpu().numpy()
        return torch.from_numpy(int8.dequantize_pool(pool, ex.kv_mem_manager.kv_scales[0].cpu().numpy()))

    system = tuple(range(2000, 2096))               # 6 full pages
    (a,) = ex.reserve_paged_requests([96])
    ex.activate_paged_packed_prefill_batch((a,), [96])
    attn.context_forward(_rows(96, hq, 61), _rows(96, hkv, 62), _rows(96, hkv, 63), ex.atten_info, 0, SCALE * log2e)
    ex.store_paged_request_prefix(system, a, first_token_id=5)
    others = []
    for i, extra in enumerate((20, 3)):
        prompt = system + tuple(range(3000 + 100 * i, 3000 + 100 * i + extra))
        req, matched, first = ex.share_paged_prefix_from_cache(prompt)
        assert matched == 96 and first is None
        ex.ensure_paged_request_capacity(req, 96 + extra + 8)
        ex.activate_paged_chunk_prefill_batch((req,), [96], [extra])
        q = _rows(extra, hq, 70 + i)
        out = attn.context_forward(q, _rows(extra, hkv, 80 + i), _rows(extra, hkv, 90 + i), ex.atten_info, 0, SCALE * log2e)
        torch.cuda.synchronize()
        info = ex.atten_info
        ref = cpu_ref.paged_prefill_ref(q.cpu(), decoded(), info.block_table.cpu(), info.cu_q_lens.cpu(),
                                        info.context_lens_i32.cpu(), SCALE).numpy()
        assert_attention_close(out, ref, f"int8 pool, chunk {i} over the cached prefix")
        others.append(req)
    batch = (a, *others)
    for step in range(3):
        ex.extend_paged_requests(batch)
        assert ex.atten_info.decode_plan.shared_pages == 6
        qd, kd, vd = _rows(3, hq, 95 + step), _rows(3, hkv, 96 + step), _rows(3, hkv, 97 + step)
        out = attn.token_forward(qd, kd, vd, ex.atten_info, 0, SCALE)
        torch.cuda.synchronize()
        info = ex.atten_info
        ref = cpu_ref.paged_decode_ref(qd.cpu(), decoded(), info.block_table.cpu(), info.seq_lens_i32.cpu(), SCALE).numpy()
        assert_attention_close(out, ref, f"int8 decode step {step} over a shared system prompt")


@pytest.mark.parametrize("dtype", [torch.int8, torch.uint8])
def test_quantised_pools_at_head_dim_64(dtype):
    """8-bit pools (int8 and fp8) at head dim 64: quantising append, decode through both schedules
    with the fused append, and a chunk over cached history."""
    from oracle import fp8
    codec = int8 if dtype == torch.int8 else fp8
    print(f"head_dim 64, pool dtype {dtype}", flush=True)
    d, hq, hkv = 64, 16, 4
    scale = 1.0 / math.sqrt(d)
    case = workloads.make_decode_case("q64", 77, [0, 15, 16, 17, 200, 63], hq, hkv, device=DEV, head_dim=d)
    scales = _head_scales(hkv) if dtype == torch.int8 else _head_scales(hkv, 0.02, 0.015)
    pool = torch.zeros(case.kv_pool.shape, dtype=dtype, device=DEV)
    every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
    ops.kv_append_quantised(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every_slot, pool, scales)
    want_codes = np.zeros(pool.shape, dtype=np.int8 if dtype == torch.int8 else np.uint8)
    codec.kv_append(case.kv_pool[:, :hkv].cpu().numpy(), case.kv_pool[:, hkv:].cpu().numpy(), every_slot.cpu().numpy(),
                    want_codes, scales.cpu().numpy())
    got = pool.cpu().numpy()
    if dtype == torch.int8:
        assert np.array_equal(got, want_codes)
    else:
        assert (((got == want_codes) | (((got & 0x7F) == 0) & ((want_codes & 0x7F) == 0)))).all()
    ref_pool = pool.clone()
    ops.kv_append_quantised(case.k_new, case.v_new, case.slot_mapping, ref_pool, scales)
    values = torch.from_numpy(codec.dequantize_pool(ref_pool.cpu().numpy(), scales.cpu().numpy()))
    ref = cpu_ref.paged_decode_ref(case.q.cpu(), values, case.block_table.cpu(), case.seq_lens.cpu(), scale).numpy()
    for kw in ({"num_splits": 1}, {"schedule": "balanced", "chunks": 3}):
        fused = pool.clone()
        if "schedule" in kw:
            plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, 3)
            out = ops.decode_step(case.q, fused, plan, case.k_new, case.v_new, scale, kv_scales=scales)
        else:
            out = ops.paged_decode(case.q, fused, case.block_table, case.seq_lens, scale, kv_scales=scales,
                                   k_new=case.k_new, v_new=case.v_new, **kw)
        torch.cuda.synchronize()
        assert torch.equal(fused, ref_pool)
        assert_attention_close(out, ref, f"head_dim 64 {dtype} {kw}")
    pre = workloads.make_prefill_case("q64p", 78, [40, 7, 65], hq, hkv, context_lens=[33, 0, 100], device=DEV, head_dim=d)
    pool = torch.zeros(pre.kv_pool.shape, dtype=dtype, device=DEV)
    every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
    ops.kv_append_quantised(pre.kv_pool[:, :hkv], pre.kv_pool[:, hkv:], every_slot, pool, scales)
    ops.kv_append_quantised(pre.k, pre.v, pre.slot_mapping, pool, scales)
    out = ops.paged_prefill(pre.q, pool, pre.block_table, pre.cu_q_lens, pre.context_lens, pre.max_q_len, scale,
                            kv_scales=scales)
    torch.cuda.synchronize()
    values = torch.from_numpy(codec.dequantize_pool(pool.cpu().numpy(), scales.cpu().numpy()))
    ref = cpu_ref.paged_prefill_ref(pre.q.cpu(), values, pre.block_table.cpu(), pre.cu_q_lens.cpu(),
                                    pre.context_lens.cpu(), scale).numpy()
    assert_attention_close(out, ref, f"head_dim 64 {dtype} chunk prefill")


@pytest.mark.parametrize("dtype", [torch.int8, torch.uint8])
@pytest.mark.parametrize("page_size", [16, 32])
def test_quantised_chunk_prefill_at_head_dim_64_many_tiles(dtype, page_size):
    """Chunks over long 8-bit histories at head dim 64 (the MFMA-tiled kernel's staging of 64-wide
    code rows): many key tiles, ragged ends, 3 and 8 query heads per KV head."""
    from oracle import fp8
    codec = int8 if dtype == torch.int8 else fp8
    d = 64
    scale = 1.0 / math.sqrt(d)
    for hq, hkv, lens, ctx in ((24, 8, [300, 65, 129], [700, 1, 450]), (32, 4, [513], [1000])):
        print(f"head_dim 64 {dtype} page_size {page_size} {hq}/{hkv} {lens} ctx {ctx}", flush=True)
        pre = workloads.make_prefill_case("q64t", 91 + hq, lens, hq, hkv, context_lens=ctx, device=DEV, head_dim=d,
                                          page_size=page_size)
        scales = _head_scales(hkv) if dtype == torch.int8 else _head_scales(hkv, 0.02, 0.015)
        pool = torch.zeros(pre.kv_pool.shape, dtype=dtype, device=DEV)
        every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
        ops.kv_append_quantised(pre.kv_pool[:, :hkv], pre.kv_pool[:, hkv:], every_slot, pool, scales)
        ops.kv_append_quantised(pre.k, pre.v, pre.slot_mapping, pool, scales)
        out = ops.paged_prefill(pre.q, pool, pre.block_table, pre.cu_q_lens, pre.context_lens, pre.max_q_len, scale,
                                kv_scales=scales, page_size=page_size)
        torch.cuda.synchronize()
        values = torch.from_numpy(codec.dequantize_pool(pool.cpu().numpy(), scales.cpu().numpy()))
        ref = cpu_ref.paged_prefill_ref(pre.q.cpu(), values, pre.block_table.cpu(), pre.cu_q_lens.cpu(),
                                        pre.context_lens.cpu(), scale, page_size=page_size).numpy()
        assert_attention_close(out, ref, f"head_dim 64 {dtype} chunk prefill over {ctx}")


@pytest.mark.parametrize("dtype", [torch.int8, torch.uint8])
def test_codes_of_rows_that_are_not_finite(dtype):
    """NaN and +-Inf elements of a row: +-Inf saturate, NaN is stored as the most negative code
    (the clamp drops a NaN operand), by the append kernel and by the appends fused into decode;
    no other element's code changes."""
    from oracle import fp8
    codec = int8 if dtype == torch.int8 else fp8
    print(f"codes of non-finite inputs, pool dtype {dtype}", flush=True)
    hq, hkv = 8, 2
    case = workloads.make_decode_case("nonfinite", 88, [20, 47, 15], hq, hkv, device=DEV)
    for row in (case.k_new, case.v_new):
        row[0, 0, 3], row[0, 1, 64], row[1, 0, 127] = float("nan"), float("inf"), float("-inf")
        row[2, 1, 0] = float("nan")
    scales = _head_scales(hkv) if dtype == torch.int8 else _head_scales(hkv, 0.02, 0.015)
    pool0 = torch.zeros(case.kv_pool.shape, dtype=dtype, device=DEV)
    every_slot = torch.arange(pool0.shape[0], dtype=torch.int32, device=DEV)
    ops.kv_append_quantised(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every_slot, pool0, scales)
    want = pool0.cpu().numpy().copy()
    codec.kv_append(case.k_new.cpu().numpy(), case.v_new.cpu().numpy(), case.slot_mapping.cpu().numpy(), want,
                    scales.cpu().numpy())
    lowest, highest = (-127, 127) if dtype == torch.int8 else (0xFE, 0x7E)
    slot0 = int(case.slot_mapping[0])
    assert want[slot0, 0, 3] == lowest and want[slot0, 1, 64] == highest
    pool = pool0.clone()
    ops.kv_append_quantised(case.k_new, case.v_new, case.slot_mapping, pool, scales)
    torch.cuda.synchronize()

    def same_codes(got):
        got = got.cpu().numpy()
        if dtype == torch.int8:
            return np.array_equal(got, want)
        return bool((((got == want) | (((got & 0x7F) == 0) & ((want & 0x7F) == 0)))).all())   # zero's sign is free

    assert same_codes(pool), "append kernel"
    for chunks in (None, 2):
        fused = pool0.clone()
        plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, chunks)
        ops.decode_step(case.q, fused, plan, case.k_new, case.v_new, SCALE, kv_scales=scales)
        torch.cuda.synchronize()
        assert same_codes(fused), f"append fused into the balanced step, chunks={chunks}"
    fused = pool0.clone()
    ops.paged_decode(case.q, fused, case.block_table, case.seq_lens, SCALE, kv_scales=scales, num_splits=1,
                     k_new=case.k_new, v_new=case.v_new)
    torch.cuda.synchronize()
    assert same_codes(fused), "append fused into the per-sequence step"


@pytest.mark.parametrize("dtype", [torch.int8, torch.uint8])
@pytest.mark.parametrize("head_dim", [128, 64])
@pytest.mark.parametrize("hq,hkv,lens,ctx,slices", [
    (64, 8, [256], [4096], 3),
    (16, 8, [77, 20], [2100, 130], 4),
    (8, 8, [130], [1500], 2),
])
def test_chunk_prefill_over_key_slices_of_a_pool_of_codes(dtype, head_dim, hq, hkv, lens, ctx, slices):
    """A lone chunk over a long 8-bit history, cut along its keys: the oracle on the decoded pool,
    the unsplit launch within 1e-3, the same bits twice."""
    from oracle import fp8
    codec = int8 if dtype == torch.int8 else fp8
    print(f"{dtype} chunk prefill over {slices} key slices d={head_dim} {hq}/{hkv} {lens} ctx {ctx}", flush=True)
    case = workloads.make_prefill_case("q8ks", 8800 + hq + slices, lens, hq, hkv, context_lens=ctx, device=DEV,
                                       head_dim=head_dim)
    scale = 1.0 / math.sqrt(head_dim)
    scales = _head_scales(hkv) if dtype == torch.int8 else _head_scales(hkv, 6.0 / 448, 5.0 / 448)
    pool = torch.empty(case.kv_pool.shape, dtype=dtype, device=DEV)
    every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
    ops.kv_append_quantised(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every_slot, pool, scales)
    ops.kv_append_quantised(case.k, case.v, case.slot_mapping, pool, scales)
    args = (case.q, pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len, scale)
    plain = ops.paged_prefill(*args, kv_scales=scales, key_slices=1)
    split = ops.paged_prefill(*args, kv_scales=scales, key_slices=slices)
    again = ops.paged_prefill(*args, kv_scales=scales, key_slices=slices)
    torch.cuda.synchronize()
    values = torch.from_numpy(codec.dequantize_pool(pool.cpu().numpy(), scales.cpu().numpy()))
    ref = cpu_ref.paged_prefill_ref(case.q.cpu(), values, case.block_table.cpu(), case.cu_q_lens.cpu(),
                                    case.context_lens.cpu(), scale).numpy()
    assert_attention_close(split, ref, f"{dtype} {slices} key slices")
    assert torch.equal(split, again)
    assert float((split.float() - plain.float()).abs().max()) <= 1e-3
