"""GPU parity of the fp8 (E4M3FN) KV pool through the C ABI: codes written by the append and by the
append fused into decode are bit-equal to the numpy oracle's, page dequantisation is bit-equal to
decode * scale rounded to fp16, and decode attention over an fp8 pool is within the attention
tolerance of the fp32 oracle applied to the decoded pool."""

import math

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import ops
from oracle import cpu_ref, fp8
from tests.parity import assert_attention_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = 128
SCALE = 1.0 / math.sqrt(D)


def _all_halves_in_range(limit):
    halves = np.arange(0x10000, dtype=np.uint16).view(np.float16)
    keep = np.isfinite(halves) & (np.abs(halves.astype(np.float32)) <= limit)
    return halves[keep]


def test_append_codes_equal_the_oracle_for_every_fp16_input():
    print("fp8 append: every fp16 value", flush=True)
    hkv = 2
    vals = _all_halves_in_range(2000.0)                      # well past 448 * scale: saturation included
    t = (vals.size + hkv * D - 1) // (hkv * D)
    flat = np.zeros(t * hkv * D, dtype=np.float16)
    flat[:vals.size] = vals
    k = flat.reshape(t, hkv, D)
    v = k[::-1].copy()
    scales = np.array([1.0, 0.37, 3.0, 0.011], dtype=np.float32)
    slots = np.random.default_rng(0).permutation(t + 16)[:t].astype(np.int32)
    slots[5] = -1                                            # a padded row
    pool = torch.full((t + 16, 2 * hkv, D), 0x55, dtype=torch.uint8, device=DEV)
    ops.kv_append_fp8(torch.from_numpy(k).to(DEV), torch.from_numpy(v).to(DEV), torch.from_numpy(slots).to(DEV),
                      pool, torch.from_numpy(scales).to(DEV))
    torch.cuda.synchronize()
    want = np.full((t + 16, 2 * hkv, D), 0x55, dtype=np.uint8)
    fp8.kv_append(k, v, slots, want, scales)
    got = pool.cpu().numpy()
    diff = got != want
    # the sign of a zero code is free (0x00 and 0x80 decode to the same value)
    diff &= ~(((got & 0x7F) == 0) & ((want & 0x7F) == 0))
    assert int(diff.sum()) == 0, f"{int(diff.sum())} codes differ, e.g. {got[diff][:8]} vs {want[diff][:8]}"


def test_page_dequant_is_decode_times_scale():
    print("fp8 page dequant", flush=True)
    hkv, pages = 2, 6
    codes = np.arange(pages * 16 * 2 * hkv * D, dtype=np.uint32)
    codes = ((codes * 2654435761) >> 13).astype(np.uint8)   # every code many times, in no order
    codes[(codes & 0x7F) == 0x7F] = 0x3C                    # NaN codes never get written by the append
    pool = torch.from_numpy(codes.reshape(pages * 16, 2 * hkv, D)).to(DEV)
    scales = np.array([0.5, 0.013, 1.7, 0.25], dtype=np.float32)
    dst = torch.zeros((4 * 16, 2 * hkv, D), dtype=torch.float16, device=DEV)
    src_ids = torch.tensor([5, 0, 9, 2], dtype=torch.int32, device=DEV)          # 9: out of range, skipped
    ops.page_dequant(pool, dst, src_ids, None, torch.from_numpy(scales).to(DEV))
    torch.cuda.synchronize()
    full = fp8.dequantize_pool(codes.reshape(pages * 16, 2 * hkv, D), scales).astype(np.float16)
    got = dst.cpu().numpy()
    for i, page in enumerate((5, 0, None, 2)):
        block = got[16 * i: 16 * i + 16]
        if page is None:
            assert np.all(block == 0)
        else:
            assert np.array_equal(block.view(np.uint16), full[16 * page: 16 * page + 16].view(np.uint16))
    # a view of the pool as torch's float8 type is accepted too
    dst2 = torch.zeros_like(dst)
    ops.page_dequant(pool.view(torch.float8_e4m3fn), dst2, src_ids, torch.tensor([3, 2, 1, 0], dtype=torch.int32, device=DEV),
                     torch.from_numpy(scales).to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(dst2[48:64], dst[0:16]) and torch.equal(dst2[0:16], dst[48:64])


def _fp8_case(seed, lens, hq, hkv, k_scale=0.02, v_scale=0.015):
    """Random fp16 K/V quantised into a shuffled fp8 pool by the append kernel; returns what decode needs."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    b = len(lens)
    pages_per = [(n + 15) // 16 for n in lens]
    num_pages = sum(pages_per) + 7
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    width = max(1, max(pages_per))
    table = torch.zeros((b, width), dtype=torch.int32)
    slots = []
    cur = 0
    for i, n in enumerate(lens):
        ids = perm[cur:cur + pages_per[i]]
        cur += pages_per[i]
        table[i, :len(ids)] = torch.tensor(ids, dtype=torch.int32)
        slots += [ids[t // 16] * 16 + t % 16 for t in range(n)]
    total = sum(lens)
    k = torch.randn((total, hkv, D), generator=g, device=DEV, dtype=torch.float16)
    v = torch.randn((total, hkv, D), generator=g, device=DEV, dtype=torch.float16)
    scales = torch.cat([k_scale * (1 + 0.1 * torch.arange(hkv)), v_scale * (1 + 0.2 * torch.arange(hkv))]).float().to(DEV)
    pool = torch.randint(0, 0x7F, (num_pages * 16, 2 * hkv, D), generator=g, device=DEV, dtype=torch.uint8)
    ops.kv_append_fp8(k, v, torch.tensor(slots, dtype=torch.int32, device=DEV), pool, scales)
    q = torch.randn((b, hq, D), generator=g, device=DEV, dtype=torch.float16)
    return q, pool, scales, table.to(DEV), torch.tensor(lens, dtype=torch.int32, device=DEV)


def _oracle(q, pool, scales, table, lens):
    values = torch.from_numpy(fp8.dequantize_pool(pool.cpu().numpy(), scales.cpu().numpy()))
    return cpu_ref.paged_decode_ref(q.cpu(), values, table.cpu(), lens.cpu(), SCALE).numpy()


@pytest.mark.parametrize("hq,hkv", [(8, 2), (64, 8), (16, 16), (4, 1)])
def test_decode_over_an_fp8_pool_matches_the_oracle_on_the_decoded_values(hq, hkv):
    print(f"fp8 decode hq={hq} hkv={hkv}", flush=True)
    lens = [1, 16, 17, 250, 0, 999, 64]
    q, pool, scales, table, seq_lens = _fp8_case(11 + hq, lens, hq, hkv)
    out = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle(q, pool, scales, table, seq_lens), "fp8 decode")
    assert torch.all(out[4] == 0)                            # the empty sequence
    # chunk count is free: same result within tolerance, and a repeat is bit-identical
    again = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales)
    other = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales, chunks=37)
    torch.cuda.synchronize()
    assert torch.equal(out, again)
    assert_attention_close(other, _oracle(q, pool, scales, table, seq_lens), "fp8 decode, 37 chunks")


def test_per_sequence_splits_read_an_fp8_pool_too():
    print("fp8 decode, per-sequence splits", flush=True)
    q, pool, scales, table, seq_lens = _fp8_case(57, [0, 1, 16, 17, 300, 1000, 64], 32, 4)
    ref = _oracle(q, pool, scales, table, seq_lens)
    for kw in ({"num_splits": 1}, {"num_splits": 4}, {"max_splits": 16, "min_pages_per_split": 2}):
        out = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales, **kw)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"fp8 splits {kw}")
        assert float(out[0].abs().max()) == 0.0


def test_quantisation_error_is_the_only_difference_from_fp16():
    """The same K/V in an fp16 pool: outputs differ by what E4M3's 3 mantissa bits allow, not more."""
    print("fp8 vs fp16 decode", flush=True)
    hq, hkv, lens = 16, 4, [300, 77]
    g = torch.Generator(device=DEV).manual_seed(5)
    k = torch.randn((sum(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    v = torch.randn((sum(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    q = torch.randn((2, hq, D), generator=g, device=DEV, dtype=torch.float16)
    # sequence 0 in pages 1..19, sequence 1 in pages 24..28
    slots = torch.cat([torch.arange(lens[0]) + 16, torch.arange(lens[1]) + 24 * 16]).to(torch.int32).to(DEV)
    table = torch.zeros((2, 20), dtype=torch.int32, device=DEV)
    table[0, :19] = torch.arange(1, 20)
    table[1, :5] = torch.arange(24, 29)
    pool16 = torch.zeros((30 * 16, 2 * hkv, D), dtype=torch.float16, device=DEV)
    pool8 = torch.zeros((30 * 16, 2 * hkv, D), dtype=torch.uint8, device=DEV)
    scales = torch.full((2 * hkv,), 6.0 / 448.0, device=DEV)                 # +-6 sigma before saturation
    ops.kv_append(k, v, slots, pool16)
    ops.kv_append_fp8(k, v, slots, pool8, scales)
    seq_lens = torch.tensor(lens, dtype=torch.int32, device=DEV)
    o16 = ops.paged_decode(q, pool16, table, seq_lens, SCALE)
    o8 = ops.paged_decode(q, pool8, table, seq_lens, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    err = (o16.float() - o8.float()).abs().max().item()
    assert 1e-4 < err < 3e-2, err                          # visibly quantised, and bounded


def test_fused_append_writes_the_same_codes_and_attends_them():
    print("fp8 decode with fused append", flush=True)
    hq, hkv = 16, 4
    lens = [33, 16, 1, 130]                                # lengths already counting the new token
    q, pool, scales, table, seq_lens = _fp8_case(23, lens, hq, hkv)
    g = torch.Generator(device=DEV).manual_seed(99)
    k_new = torch.randn((len(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    v_new = torch.randn((len(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    last_slots = torch.stack([table[i, (n - 1) // 16] * 16 + (n - 1) % 16 for i, n in enumerate(lens)]).int()
    separate = pool.clone()
    ops.kv_append_fp8(k_new, v_new, last_slots, separate, scales)
    want_out = ops.paged_decode(q, separate, table, seq_lens, SCALE, kv_scales=scales)
    plan = ops.DecodePlan(table, seq_lens, hq, hkv, pool.shape[0] // 16)
    fused = pool.clone()
    got_out = ops.decode_step(q, fused, plan, k_new, v_new, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(fused, separate)                    # same codes in the same slots, nothing else touched
    assert torch.equal(got_out, want_out)
    assert_attention_close(got_out, _oracle(q, fused, scales, table, seq_lens), "fp8 fused append + decode")


def test_fp8_pages_move_with_the_page_copy_and_gather_kernels():
    print("fp8 page moves", flush=True)
    q, pool, scales, table, seq_lens = _fp8_case(31, [40, 90], 8, 2)
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
    q, pool, scales, table, seq_lens = _fp8_case(41, [20], 8, 2)
    with pytest.raises(ValueError, match="scales"):
        ops.paged_decode(q, pool, table, seq_lens, SCALE)
    with pytest.raises(ValueError, match="scales"):
        ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales[:3])
    with pytest.raises(ValueError, match="both stages"):
        ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales, num_splits=2, stage="split")
    with pytest.raises(ValueError, match="fp8"):
        ops.kv_append_fp8(q[:, :2], q[:, :2], seq_lens, pool.half(), scales)


# ---- the executor and the attention layer on fp8 pools ------------------------------------------

def _fp8_executor(layers=2, hq=16, hkv=8, num_pages=96):
    from llama_lite_npu_amd.executor import ModelExecutor

    ex = ModelExecutor(num_layers=layers, num_q_heads=hq, num_kv_heads=hkv, head_dim=D, num_pages=num_pages,
                       max_seq_len=512, max_requests=8, device=DEV, dtype=torch.float8_e4m3fn)
    for layer, pool in enumerate(ex.kv_mem_manager.gpu_kv_buffer):
        pool.view(torch.uint8).fill_(0x55)
        ex.kv_mem_manager.set_kv_scales(layer, [0.02 + 0.001 * h for h in range(hkv)],
                                        [0.015 + 0.002 * h for h in range(hkv)])
    return ex


def _rows(tokens, heads, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return torch.randn((tokens, heads, D), generator=g, device=DEV, dtype=torch.float16)


def _decoded_pool(ex, layer):
    pool = ex.kv_mem_manager.gpu_kv_buffer[layer].view(torch.uint8).cpu().numpy()
    return torch.from_numpy(fp8.dequantize_pool(pool, ex.kv_mem_manager.kv_scales[layer].cpu().numpy()))


def test_executor_flow_on_fp8_pools():
    print("fp8: executor prefill / chunked prefill / decode / compaction", flush=True)
    from llama_lite_npu_amd.attention import Attention
    from oracle import c_oracle
    from tests.parity import to_np16

    hq, hkv = 16, 8
    ex = _fp8_executor(hq=hq, hkv=hkv)
    assert ex.kv_mem_manager.is_fp8 and ex.atten_info.kv_scales[0] is not None
    attn = Attention(hq, hkv, D)
    log2e = 1.4426950408889634
    lens = [37, 16, 90, 5]
    ids = ex.reserve_paged_requests(lens)
    ex.activate_paged_packed_prefill_batch(ids, lens)
    info = ex.atten_info
    for layer in range(2):
        q, k, v = _rows(sum(lens), hq, 10 + layer), _rows(sum(lens), hkv, 20 + layer), _rows(sum(lens), hkv, 30 + layer)
        out = attn.context_forward(q, k, v, info, layer, SCALE * log2e)
        torch.cuda.synchronize()
        # a fresh prompt attends to its own fp16 K/V ...
        ref = c_oracle.varlen_prefill(to_np16(q), to_np16(k), to_np16(v), info.b_start_loc.cpu().numpy(),
                                      np.asarray(lens, dtype=np.int32), SCALE)
        assert_attention_close(out, ref, f"fp8 pool, fresh prefill, layer {layer}")
        # ... and what went into the pages are the oracle's codes
        scales = ex.kv_mem_manager.kv_scales[layer].cpu().numpy()
        want = np.concatenate([fp8.quantize_rows(to_np16(k), scales[:hkv]), fp8.quantize_rows(to_np16(v), scales[hkv:])], axis=1)
        got = ex.kv_mem_manager.gpu_kv_buffer[layer].view(torch.uint8)[info.cur_select_index.long()].cpu().numpy()
        same = (got == want) | (((got & 0x7F) == 0) & ((want & 0x7F) == 0))
        assert same.all()
    # a later chunk of request 3 attends to cached (quantised) history through the scratch pool
    ex.ensure_paged_request_capacity(ids[3], 5 + 40)
    ex.activate_paged_chunk_prefill_batch((ids[3],), [5], [30])
    info = ex.atten_info
    q, k, v = _rows(30, hq, 41), _rows(30, hkv, 42), _rows(30, hkv, 43)
    out = attn.context_forward(q, k, v, info, 0, SCALE * log2e)
    torch.cuda.synchronize()
    ref = cpu_ref.paged_prefill_ref(q.cpu(), _decoded_pool(ex, 0), info.block_table.cpu(), info.cu_q_lens.cpu(),
                                    info.context_lens_i32.cpu(), SCALE).numpy()
    assert_attention_close(out, ref, "fp8 pool, chunk over cached history")
    # layer 1 has to see the chunk too before the requests decode together
    attn.context_forward(_rows(30, hq, 44), _rows(30, hkv, 45), _rows(30, hkv, 46), info, 1, SCALE * log2e)
    for step in range(18):
        ex.extend_paged_requests(ids)
        info = ex.atten_info
        assert info.decode_plan is not None and info.decode_plan.shared_pages == 0
        for layer in range(2):
            q, k, v = _rows(4, hq, 100 + 2 * step + layer), _rows(4, hkv, 200 + 2 * step + layer), _rows(4, hkv, 300 + step)
            out = attn.token_forward(q, k, v, info, layer, SCALE)
            torch.cuda.synchronize()
            ref = cpu_ref.paged_decode_ref(q.cpu(), _decoded_pool(ex, layer), info.block_table.cpu(),
                                           info.seq_lens_i32.cpu(), SCALE).numpy()
            assert_attention_close(out, ref, f"fp8 decode step {step} layer {layer}")
    # pages of an fp8 pool move like any others: free a request, compact, same answers bit for bit
    q = _rows(3, hq, 999)
    ex.release_paged_request_ids((ids[1],))
    keep = (ids[0], ids[2], ids[3])
    ex.activate_paged_decode_batch(keep)
    before = attn.token_forward(q, None, None, ex.atten_info, 0, SCALE).clone()
    moves = ex.compact_kv_pool()
    assert moves
    ex.activate_paged_decode_batch(keep)
    after = attn.token_forward(q, None, None, ex.atten_info, 0, SCALE)
    torch.cuda.synchronize()
    assert torch.equal(before, after)


def test_fp8_decode_steps_replay_as_graphs():
    print("fp8: device metadata + graph replay vs eager", flush=True)
    from tests import test_gpu_decode_graph as dg

    def build():
        from llama_lite_npu_amd.executor import ModelExecutor

        ex = ModelExecutor(num_layers=dg.LAYERS, num_q_heads=dg.HQ, num_kv_heads=dg.HKV, head_dim=D, num_pages=160,
                           max_seq_len=256, max_requests=8, device=DEV, dtype=torch.float8_e4m3fn)
        for layer, pool in enumerate(ex.kv_mem_manager.gpu_kv_buffer):
            pool.view(torch.uint8).fill_(0x31)
            ex.kv_mem_manager.set_kv_scales(layer, [0.03] * dg.HKV, [0.02] * dg.HKV)
        return ex

    def prefill(ex, lens, seed):
        ids = ex.reserve_paged_requests(lens)
        ex.activate_paged_packed_prefill_batch(ids, lens)
        for layer in range(dg.LAYERS):
            ops.kv_append_fp8(_rows(sum(lens), dg.HKV, seed + layer), _rows(sum(lens), dg.HKV, seed + 50 + layer),
                              ex.atten_info.cur_select_index, ex.atten_info.kv_buffer[layer],
                              ex.atten_info.kv_scales[layer])
        return ids

    host, dev = build(), build()
    model_h, model_d = dg.TinyModel(), dg.TinyModel()
    lens = [1, 17, 48, 100, 31]
    ids_h, ids_d = prefill(host, lens, 7), prefill(dev, lens, 7)
    dev.attach_model(model_d, "qwen3")
    batch = dev.activate_device_decode_batch(ids_d, reserve_tokens=8)
    tok_h = tok_d = torch.arange(len(lens), device=DEV).reshape(-1, 1) % dg.VOCAB
    for step in range(20):
        out_h = dg._host_step(host, model_h, ids_h, tok_h)
        dev.extend_paged_requests(ids_d)
        out_d = dev.forward(tok_d)
        torch.cuda.synchronize()
        assert torch.equal(out_h, out_d), f"step {step}"
        tok_h, tok_d = dg._next_tokens(out_h), dg._next_tokens(out_d)
    assert dev.graph_runner.replay_count == 19 and dev.graph_runner.fallback_count == 0
    batch.check()
    for a, b in zip(host.kv_mem_manager.gpu_kv_buffer, dev.kv_mem_manager.gpu_kv_buffer):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("t", [77, 8197])          # one token per lane, and four (prefill-sized launches)
def test_fused_epilogue_into_an_fp8_pool_equals_epilogue_then_quantising_append(t):
    print(f"fp8: fused QK-norm + RoPE + quantising append, {t} tokens", flush=True)
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
    # two launches: epilogue into fp16 rows, then the quantising append
    q_a = q.clone()
    rows = torch.empty((t, 2 * hkv, D), dtype=torch.float16, device=DEV)
    ops.qk_norm_rope_append(q_a, k, v, torch.arange(t, dtype=torch.int32, device=DEV), rows, wq, wk, cos, sin)
    pool_a = torch.full((n_slots, 2 * hkv, D), 0x55, dtype=torch.uint8, device=DEV)
    ops.kv_append_fp8(rows[:, :hkv], rows[:, hkv:], slots, pool_a, scales)
    # one launch
    q_b = q.clone()
    pool_b = torch.full((n_slots, 2 * hkv, D), 0x55, dtype=torch.uint8, device=DEV)
    ops.qk_norm_rope_append(q_b, k, v, slots, pool_b, wq, wk, cos, sin, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(q_a, q_b)
    assert torch.equal(pool_a, pool_b)
    assert int((pool_b != 0x55).any(dim=(1, 2)).sum()) == t - 1          # the padded token stored nothing
    # without norm and rotation it is the plain quantising append
    pool_c = torch.full_like(pool_b, 0x55)
    pool_d = torch.full_like(pool_b, 0x55)
    ops.qk_norm_rope_append(q.clone(), k, v, slots, pool_c, kv_scales=scales)
    ops.kv_append_fp8(k, v, slots, pool_d, scales)
    torch.cuda.synchronize()
    assert torch.equal(pool_c, pool_d)
    with pytest.raises(ValueError, match="scales"):
        ops.qk_norm_rope_append(q.clone(), k, v, slots, pool_c)


@pytest.mark.parametrize("seed", range(3))
def test_chunk_prefill_reads_an_fp8_pool_directly(seed):
    """Chunk rows over an fp8 history (and their own rows, appended as codes): the oracle on the
    decoded pool, within the attention tolerance; agrees with dequantising the pages first."""
    import random
    from llama_lite_npu_amd import workloads

    rng = random.Random(600 + seed)
    for case_no in range(6):
        hq, hkv = rng.choice([(64, 8), (32, 4), (16, 8), (8, 8), (4, 2), (16, 1)])
        b = rng.choice([1, 2, 4])
        edges = [1, 15, 16, 17, 63, 64, 65, 128]
        q_lens = [rng.choice([rng.choice(edges), rng.randint(1, 300)]) for _ in range(b)]
        ctx = [rng.choice([0, rng.choice(edges), rng.randint(0, 900)]) for _ in range(b)]
        print(f"fp8 chunk prefill {seed}.{case_no}: heads {hq}/{hkv} chunks {q_lens} histories {ctx}", flush=True)
        case = workloads.make_prefill_case("fp8", 8000 + 100 * seed + case_no, q_lens, hq, hkv, context_lens=ctx,
                                           device=DEV)
        scales = torch.cat([0.02 * (1 + 0.1 * torch.arange(hkv)), 0.015 * (1 + 0.2 * torch.arange(hkv))]).float().to(DEV)
        pool = torch.empty(case.kv_pool.shape, dtype=torch.uint8, device=DEV)
        every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=DEV)
        ops.kv_append_fp8(case.kv_pool[:, :hkv], case.kv_pool[:, hkv:], every_slot, pool, scales)   # the history
        ops.kv_append_fp8(case.k, case.v, case.slot_mapping, pool, scales)                          # the chunk
        out = ops.paged_prefill(case.q, pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len,
                                SCALE, kv_scales=scales)
        again = ops.paged_prefill(case.q, pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len,
                                  SCALE, kv_scales=scales)
        torch.cuda.synchronize()
        values = torch.from_numpy(fp8.dequantize_pool(pool.cpu().numpy(), scales.cpu().numpy()))
        ref = cpu_ref.paged_prefill_ref(case.q.cpu(), values, case.block_table.cpu(), case.cu_q_lens.cpu(),
                                        case.context_lens.cpu(), SCALE).numpy()
        assert_attention_close(out, ref, f"fp8 chunk prefill {seed}.{case_no}")
        assert torch.equal(out, again)
        # the two-pass way: pages to fp16 (rounding code * scale), then the fp16 kernel
        scratch = torch.zeros(case.kv_pool.shape, dtype=torch.float16, device=DEV)
        all_pages = torch.arange(case.num_pages, dtype=torch.int32, device=DEV)
        ops.page_dequant(pool, scratch, all_pages, all_pages, scales)
        two_pass = ops.paged_prefill(case.q, scratch, case.block_table, case.cu_q_lens, case.context_lens,
                                     case.max_q_len, SCALE)
        assert float((two_pass.float() - out.float()).abs().max()) <= 2e-3


def test_cached_system_prompt_over_fp8_pools_is_attended_once_for_the_batch():
    """Three requests share a 96-token prefix through the block cache of an fp8 executor: the
    decode step gets a shared-prefix plan and the codes of the shared pages are read once."""
    print("fp8: executor, shared prefix decode", flush=True)
    from llama_lite_npu_amd.attention import Attention

    hq, hkv = 16, 8
    ex = _fp8_executor(layers=1, hq=hq, hkv=hkv, num_pages=128)
    attn = Attention(hq, hkv, D)
    log2e = 1.4426950408889634
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
        attn.context_forward(_rows(extra, hq, 70 + i), _rows(extra, hkv, 80 + i), _rows(extra, hkv, 90 + i),
                             ex.atten_info, 0, SCALE * log2e)
        others.append(req)
    batch = (a, *others)
    ex.extend_paged_requests(batch)
    assert ex.atten_info.decode_plan.shared_pages == 6
    qd, kd, vd = _rows(3, hq, 95), _rows(3, hkv, 96), _rows(3, hkv, 97)
    out = attn.token_forward(qd, kd, vd, ex.atten_info, 0, SCALE)
    torch.cuda.synchronize()
    info = ex.atten_info
    ref = cpu_ref.paged_decode_ref(qd.cpu(), _decoded_pool(ex, 0), info.block_table.cpu(), info.seq_lens_i32.cpu(),
                                   SCALE).numpy()
    assert_attention_close(out, ref, "fp8 decode over a shared system prompt")
