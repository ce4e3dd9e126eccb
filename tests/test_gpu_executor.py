"""GPU: the reference's call surface end to end -- executor metadata -> Attention.context_forward /
token_forward -> HIP kernels -- checked against the CPU oracle; prefix sharing with copy-on-write,
pool compaction, and the lite_llama.kernels-compatible wrappers."""

import math

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import kernels as compat
from llama_lite_npu_amd import ops
from llama_lite_npu_amd.attention import Attention
from llama_lite_npu_amd.executor import ModelExecutor
from oracle import c_oracle
from tests.parity import assert_attention_close, assert_bit_exact, to_np16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HQ, HKV, D = 16, 8, 128
SCALE = 1.0 / math.sqrt(D)
LOG2E = 1.4426950408889634


def _executor(num_pages=96, layers=2, max_requests=8, max_seq_len=512):
    ex = ModelExecutor(num_layers=layers, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D, num_pages=num_pages,
                       max_seq_len=max_seq_len, max_requests=max_requests, device=DEV)
    for pool in ex.kv_mem_manager.gpu_kv_buffer:
        pool.normal_()          # stale data everywhere: only written slots may matter
    return ex


def _qkv(tokens, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    q = torch.randn((tokens, HQ, D), generator=g, device=DEV, dtype=torch.float16)
    k = torch.randn((tokens, HKV, D), generator=g, device=DEV, dtype=torch.float16)
    v = torch.randn((tokens, HKV, D), generator=g, device=DEV, dtype=torch.float16)
    return q, k, v


def _oracle_decode(ex, q, layer):
    info = ex.atten_info
    return c_oracle.paged_decode(to_np16(q), to_np16(info.kv_buffer[layer]), info.block_table.cpu().numpy(),
                                 info.seq_lens_i32.cpu().numpy(), SCALE)


def test_packed_prefill_then_fused_decode_steps():
    print("executor: packed prefill + decode", flush=True)
    ex = _executor()
    attn = Attention(HQ, HKV, D)
    lens = [37, 16, 90, 5]
    ids = ex.reserve_paged_requests(lens)
    ex.activate_paged_packed_prefill_batch(ids, lens)
    info = ex.atten_info
    total = sum(lens)
    for layer in range(2):
        q, k, v = _qkv(total, 10 + layer)
        out = attn.context_forward(q, k, v, info, layer, qk_scale=SCALE * LOG2E)
        torch.cuda.synchronize()
        ref = c_oracle.varlen_prefill(to_np16(q), to_np16(k), to_np16(v), info.b_start_loc.cpu().numpy(),
                                      np.asarray(lens, dtype=np.int32), SCALE)
        assert_attention_close(out, ref, f"prefill layer {layer}")
        # the K/V rows landed in the slots the metadata names
        pool = info.kv_buffer[layer]
        sel = info.cur_select_index.long()
        assert_bit_exact(pool[sel][:, :HKV], k, "K rows in pages")
        assert_bit_exact(pool[sel][:, HKV:], v, "V rows in pages")
    for step in range(20):             # 16 -> 17 opens a page, 37 + 11 = 48 fills one
        ex.extend_paged_requests(ids)
        info = ex.atten_info
        assert info.decode_plan is not None
        for layer in range(2):
            q, k, v = _qkv(len(ids), 100 + 2 * step + layer)
            out = attn.token_forward(q, k, v, info, layer, qk_scale=SCALE)
            torch.cuda.synchronize()
            pool = info.kv_buffer[layer]
            sel = info.cur_select_index.long()
            assert_bit_exact(pool[sel][:, :HKV], k, "appended K")
            assert_bit_exact(pool[sel][:, HKV:], v, "appended V")
            assert_attention_close(out, _oracle_decode(ex, q, layer), f"decode step {step} layer {layer}")
    assert info.b_seq_len.tolist() == [n + 20 for n in lens]


def test_chunked_prefill_matches_one_shot_prefill():
    print("executor: chunked prefill", flush=True)
    attn = Attention(HQ, HKV, D)
    n = 150
    q, k, v = _qkv(n, 7)
    whole = _executor(layers=1)
    (rid,) = whole.reserve_paged_requests([n])
    whole.activate_paged_packed_prefill_batch((rid,), [n])
    out_whole = attn.context_forward(q, k, v, whole.atten_info, 0, SCALE * LOG2E)

    ex = _executor(layers=1)
    (rid,) = ex.reserve_paged_requests([64], reserved_lengths=[n])
    ex.activate_paged_packed_prefill_batch((rid,), [64])
    outs = [attn.context_forward(q[:64], k[:64], v[:64], ex.atten_info, 0, SCALE * LOG2E)]
    done = 64
    for chunk in (50, 36):
        ex.activate_paged_chunk_prefill_batch((rid,), [done], [chunk])
        sl = slice(done, done + chunk)
        outs.append(attn.context_forward(q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(),
                                         ex.atten_info, 0, SCALE * LOG2E))
        done += chunk
    torch.cuda.synchronize()
    got = torch.cat(outs)
    assert float((got.float() - out_whole.float()).abs().max()) <= 1e-3
    ref = c_oracle.varlen_prefill(to_np16(q), to_np16(k), to_np16(v), np.array([0], dtype=np.int32),
                                  np.array([n], dtype=np.int32), SCALE)
    assert_attention_close(got, ref, "chunked prefill")


def test_lone_chunk_over_a_long_history_is_cut_along_its_keys():
    """One request prefilled 128 rows at a time: a chunk's launch has too few row blocks for the
    device, and once the history is long enough for a cut to pay the attention layer's prefill call
    cuts it along its keys (the executor's host-side lengths say how far the rows see). Every chunk
    against the oracle on the whole prompt."""
    print("executor: chunked prefill over a long history", flush=True)
    attn = Attention(HQ, HKV, D)
    n, chunk = 4608, 128
    q, k, v = _qkv(n, 17)
    ex = _executor(num_pages=320, layers=1, max_requests=2, max_seq_len=5120)
    (rid,) = ex.reserve_paged_requests([chunk], reserved_lengths=[n])
    ex.activate_paged_packed_prefill_batch((rid,), [chunk])
    outs = [attn.context_forward(q[:chunk], k[:chunk], v[:chunk], ex.atten_info, 0, SCALE * LOG2E)]
    sliced = 0
    for done in range(chunk, n, chunk):
        ex.activate_paged_chunk_prefill_batch((rid,), [done], [chunk])
        info = ex.atten_info
        sliced += int(ops._lib.load().litekv_paged_prefill_key_slices(1, HQ, HKV, D, chunk, int(info.max_actual_seq_len))) > 1
        sl = slice(done, done + chunk)
        outs.append(attn.context_forward(q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), info, 0,
                                         SCALE * LOG2E))
    torch.cuda.synchronize()
    assert sliced >= 3                      # the last chunks see 4224 keys and more
    ref = c_oracle.varlen_prefill(to_np16(q), to_np16(k), to_np16(v), np.array([0], dtype=np.int32),
                                  np.array([n], dtype=np.int32), SCALE)
    assert_attention_close(torch.cat(outs), ref, "chunks over a growing history")


def test_prefix_sharing_with_copy_on_write():
    print("executor: prefix sharing + COW", flush=True)
    ex = _executor(layers=1)
    attn = Attention(HQ, HKV, D)
    prompt = tuple(range(1000, 1040))                # 40 tokens: 2 full pages + 8 tokens
    (a,) = ex.reserve_paged_requests([40])
    ex.activate_paged_packed_prefill_batch((a,), [40])
    q, k, v = _qkv(40, 21)
    attn.context_forward(q, k, v, ex.atten_info, 0, SCALE * LOG2E)
    ex.store_paged_request_prefix(prompt, a, first_token_id=3)
    b, first = ex.share_paged_request_from_cache(prompt)
    assert first == 3
    pages_a = ex.req_tokens_manager.request_pages(a)
    assert ex.req_tokens_manager.request_pages(b) == pages_a
    pool = ex.atten_info.kv_buffer[0]
    before = pool.clone()
    # both requests are about to append token 40 into the shared, partly filled third page
    moves = ex.copy_on_write((a, b))
    torch.cuda.synchronize()
    # the cache entry still holds the original page, so both requests get a private copy of it
    assert len(moves) == 2 and {m[0] for m in moves} == {pages_a[2]}
    pages_a2, pages_b2 = ex.req_tokens_manager.request_pages(a), ex.req_tokens_manager.request_pages(b)
    assert pages_a2[:2] == pages_b2[:2] == pages_a[:2] and len({pages_a[2], pages_a2[2], pages_b2[2]}) == 3
    for src, dst in moves:
        assert_bit_exact(pool[dst * 16:(dst + 1) * 16], before[src * 16:(src + 1) * 16], "COW page copy")
    ex.extend_paged_requests((a, b))
    qd, kd, vd = _qkv(2, 22)
    out = attn.token_forward(qd, kd, vd, ex.atten_info, 0, SCALE)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_decode(ex, qd, 0), "decode after COW")
    # the cached page was not touched by either append
    shared = pages_a[2]
    assert_bit_exact(pool[shared * 16:(shared + 1) * 16], before[shared * 16:(shared + 1) * 16], "cached page")
    # the two requests read the same prefix but their own new token
    assert float((out[0].float() - out[1].float()).abs().max()) > 1e-3


def test_cached_system_prompt_is_attended_once_for_the_batch():
    """Three requests share a 96-token prompt prefix through the block cache; each replays its own
    suffix; the decode step then runs with a shared-prefix plan and matches the oracle."""
    print("executor: shared prefix decode", flush=True)
    ex = _executor(num_pages=128, layers=1)
    attn = Attention(HQ, HKV, D)
    system = tuple(range(2000, 2096))               # 6 full pages
    (a,) = ex.reserve_paged_requests([96])
    ex.activate_paged_packed_prefill_batch((a,), [96])
    q, k, v = _qkv(96, 31)
    attn.context_forward(q, k, v, ex.atten_info, 0, SCALE * LOG2E)
    ex.store_paged_request_prefix(system, a, first_token_id=5)
    others = []
    for i, extra in enumerate((20, 3)):
        prompt = system + tuple(range(3000 + 100 * i, 3000 + 100 * i + extra))
        req, matched, first = ex.share_paged_prefix_from_cache(prompt)
        assert matched == 96 and first is None
        ex.ensure_paged_request_capacity(req, 96 + extra + 8)
        ex.activate_paged_chunk_prefill_batch((req,), [96], [extra])
        qs, ks, vs = _qkv(extra, 40 + i)
        attn.context_forward(qs, ks, vs, ex.atten_info, 0, SCALE * LOG2E)
        others.append(req)
    batch = (a, *others)
    assert ex.shared_prefix_pages(batch) == 5       # not extended yet: page 5 still ends request a
    ex.extend_paged_requests(batch)
    assert ex.atten_info.decode_plan.shared_pages == 6
    qd, kd, vd = _qkv(3, 50)
    out = attn.token_forward(qd, kd, vd, ex.atten_info, 0, SCALE)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_decode(ex, qd, 0), "decode over a shared system prompt")


def test_compaction_keeps_results_bitwise():
    print("executor: compaction", flush=True)
    ex = _executor(num_pages=64, layers=2)
    attn = Attention(HQ, HKV, D)
    lens = [70, 33, 120, 48, 9]
    ids = ex.reserve_paged_requests(lens)
    ex.activate_paged_packed_prefill_batch(ids, lens)
    for layer in range(2):
        q, k, v = _qkv(sum(lens), 30 + layer)
        attn.context_forward(q, k, v, ex.atten_info, layer, SCALE * LOG2E)
    ex.release_paged_request_ids((ids[0], ids[3]))        # punch holes into the pool
    keep = (ids[1], ids[2], ids[4])
    ex.activate_paged_decode_batch(keep)
    qd = _qkv(3, 40)[0]
    before = [ops.paged_decode(qd, ex.atten_info.kv_buffer[l], ex.atten_info.block_table,
                               ex.atten_info.seq_lens_i32, SCALE, num_splits=1) for l in range(2)]
    moves = ex.compact_kv_pool()
    assert moves, "expected at least one page move"
    n_live = sum(len(ex.req_tokens_manager.request_pages(r)) for r in keep)
    assert all(dst < n_live <= src for src, dst in moves)
    assert sorted(p for r in keep for p in ex.req_tokens_manager.request_pages(r)) == list(range(n_live))
    ex.activate_paged_decode_batch(keep)
    after = [ops.paged_decode(qd, ex.atten_info.kv_buffer[l], ex.atten_info.block_table,
                              ex.atten_info.seq_lens_i32, SCALE, num_splits=1) for l in range(2)]
    torch.cuda.synchronize()
    for l in range(2):
        assert torch.equal(before[l], after[l]), "compaction changed the attention result"


def test_lite_llama_kernels_signatures():
    """The four reference functions, called the way lite_llama/models/qwen3.py:20-75 calls them."""
    print("compat wrappers", flush=True)
    ex = _executor(layers=1)
    lens = [45, 130, 17]
    ids = ex.reserve_paged_requests(lens)
    ex.activate_paged_packed_prefill_batch(ids, lens)
    info = ex.atten_info
    pool = info.kv_buffer[0]
    q, k, v = _qkv(sum(lens), 50)
    compat.update_kv_buffer(torch.cat([k, v], dim=-2), info.cur_select_index, pool)
    out = compat.flash_attention2_no_pad(q, k, v, SCALE * LOG2E, info.b_start_loc, info.b_seq_len,
                                         info.max_actual_seq_len)
    torch.cuda.synchronize()
    sel = info.cur_select_index.long()
    assert_bit_exact(pool[sel], torch.cat([k, v], dim=-2), "update_kv_buffer")
    ref = c_oracle.varlen_prefill(to_np16(q), to_np16(k), to_np16(v), info.b_start_loc.cpu().numpy(),
                                  np.asarray(lens, dtype=np.int32), SCALE)
    assert_attention_close(out, ref, "flash_attention2_no_pad")

    table = ex.req_tokens_manager.b_req_tokens_table          # the reference's per-token table
    ex.extend_paged_requests(ids)
    info = ex.atten_info
    table = ex.req_tokens_manager.b_req_tokens_table
    qd, kd, vd = _qkv(3, 51)
    compat.update_kv_buffer(torch.cat([kd, vd], dim=-2), info.cur_select_index, pool)
    out = compat.flash_decoding(qd, pool[:, :HKV, :], pool[:, HKV:, :], SCALE, table, info.b_seq_len,
                                info.max_actual_seq_len)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_decode(ex, qd, 0), "flash_decoding")

    # later chunk of a chunked prefill through the paged function
    ctx = [int(n) for n in info.b_seq_len.tolist()]
    chunk = [20, 3, 31]
    ex.activate_paged_chunk_prefill_batch(ids, ctx, chunk)
    info = ex.atten_info
    table = ex.req_tokens_manager.b_req_tokens_table
    qc, kc, vc = _qkv(sum(chunk), 52)
    compat.update_kv_buffer(torch.cat([kc, vc], dim=-2), info.cur_select_index, pool)
    out = compat.paged_chunk_flash_attention(qc, pool[:, :HKV, :], pool[:, HKV:, :], SCALE * LOG2E, table,
                                             info.b_req_idx, info.b_start_loc, info.chunk_context_len,
                                             info.chunk_q_seq_len, info.max_actual_q_seq_len)
    torch.cuda.synchronize()
    ref = c_oracle.paged_prefill(to_np16(qc), to_np16(pool), info.block_table.cpu().numpy(),
                                 info.cu_q_lens.cpu().numpy(), np.asarray(ctx, dtype=np.int32), SCALE)
    assert_attention_close(out, ref, "paged_chunk_flash_attention")
    with pytest.raises(ValueError, match="halves of one"):
        compat.flash_decoding(qd, pool[:, :HKV, :].contiguous(), pool[:, HKV:, :], SCALE, table, info.b_seq_len, 8)


def test_qkv_epilogue_then_attention_equals_separate_steps():
    """Executor flow with the fused QK-norm + RoPE + append in front of prefill and decode."""
    print("executor: fused qkv epilogue", flush=True)
    from oracle import qk_epilogue

    ex = _executor(layers=1)
    attn = Attention(HQ, HKV, D)
    g = torch.Generator(device=DEV).manual_seed(77)
    wq = (1.0 + 0.1 * torch.randn(D, generator=g, device=DEV)).half()
    wk = (1.0 + 0.1 * torch.randn(D, generator=g, device=DEV)).half()

    def rows(positions):
        pos = torch.tensor(positions, device=DEV, dtype=torch.float64)
        inv = 10000.0 ** (-torch.arange(0, D, 2, device=DEV, dtype=torch.float64) / D)
        emb = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=1)
        return emb.cos().half(), emb.sin().half()

    ids = ex.reserve_paged_requests([21, 40])
    ex.activate_paged_packed_prefill_batch(ids, [21, 40])
    q, k, v = _qkv(61, 60)
    cos, sin = rows(list(range(21)) + list(range(40)))
    q_ref = torch.from_numpy(qk_epilogue.rope(qk_epilogue.rms_norm(to_np16(q), to_np16(wq), 1e-6),
                                             to_np16(cos), to_np16(sin))).to(DEV)
    attn.qkv_epilogue(q, k, v, ex.atten_info, 0, wq, wk, (cos, sin), 1e-6)
    out = attn.context_forward(q, None, None, ex.atten_info, 0, SCALE * LOG2E)
    torch.cuda.synchronize()
    assert float((q.float() - q_ref.float()).abs().max()) <= 4e-3
    info = ex.atten_info
    ref = c_oracle.paged_prefill(to_np16(q), to_np16(info.kv_buffer[0]), info.block_table.cpu().numpy(),
                                 info.cu_q_lens.cpu().numpy(), np.zeros(2, np.int32), SCALE)
    assert_attention_close(out, ref, "prefill after fused epilogue")
    ex.extend_paged_requests(ids)
    qd, kd, vd = _qkv(2, 61)
    cos, sin = rows([21, 40])
    attn.qkv_epilogue(qd, kd, vd, ex.atten_info, 0, wq, wk, (cos, sin), 1e-6)
    out = attn.token_forward(qd, None, None, ex.atten_info, 0, SCALE)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_decode(ex, qd, 0), "decode after fused epilogue")


def test_static_batch_prefill_then_decode_equals_the_packed_flow():
    """prefill_alloc_kv_cache (prompts padded to the longest) followed by decode_alloc_kv_cache
    steps gives, on the prompts' own rows and on every decode step, what the packed no-pad flow
    gives for the same prompts."""
    print("executor: static batch (padded) vs packed flow", flush=True)
    lens = [20, 7, 33]
    longest = max(lens)
    attn = Attention(HQ, HKV, D)
    q, k, v = _qkv(sum(lens), 71)                        # the prompts' rows, packed
    starts = np.concatenate([[0], np.cumsum(lens)[:-1]])
    # --- packed flow
    packed = _executor(layers=1)
    ids_p = packed.reserve_paged_requests(lens, [n + 8 for n in lens])
    packed.activate_paged_packed_prefill_batch(ids_p, lens)
    out_p = attn.context_forward(q, k, v, packed.atten_info, 0, qk_scale=SCALE * LOG2E)
    # --- static batch: the same rows at the head of each padded block, noise behind them
    static = _executor(layers=1)
    qs, ks, vs = _qkv(len(lens) * longest, 72)
    for i, (s, n) in enumerate(zip(starts, lens)):
        qs[i * longest:i * longest + n] = q[s:s + n]
        ks[i * longest:i * longest + n] = k[s:s + n]
        vs[i * longest:i * longest + n] = v[s:s + n]
    select, _ = static.prefill_alloc_kv_cache(longest, torch.tensor(lens), torch.arange(len(lens), dtype=torch.int32))
    assert select.numel() == len(lens) * longest
    out_s = attn.context_forward(qs, ks, vs, static.atten_info, 0, qk_scale=SCALE * LOG2E)
    torch.cuda.synchronize()
    for i, (s, n) in enumerate(zip(starts, lens)):
        diff = (out_s[i * longest:i * longest + n].float() - out_p[s:s + n].float()).abs().max()
        assert float(diff) <= 1e-3, f"prompt {i}: {float(diff)}"
    ref = c_oracle.varlen_prefill(to_np16(q), to_np16(k), to_np16(v), starts.astype(np.int32),
                                  np.array(lens, dtype=np.int32), SCALE)
    assert_attention_close(out_p, ref, "packed prefill")
    # --- decode steps: the token goes behind each prompt's own length, over the padding row
    for step in range(3):
        qd, kd, vd = _qkv(len(lens), 80 + step)
        packed.extend_paged_requests(ids_p)
        o_p = attn.token_forward(qd, kd, vd, packed.atten_info, 0, SCALE)
        static.decode_alloc_kv_cache(len(lens))
        assert static.atten_info.b_seq_len.tolist() == [n + step + 1 for n in lens]
        o_s = attn.token_forward(qd, kd, vd, static.atten_info, 0, SCALE)
        torch.cuda.synchronize()
        assert float((o_s.float() - o_p.float()).abs().max()) <= 1e-3, f"decode step {step}"
        assert_attention_close(o_s, _oracle_decode(static, qd, 0), f"static batch decode step {step}")


@pytest.mark.parametrize("page_size,head_dim", [(32, 128), (64, 64), (16, 64), (16, 256), (128, 128), (256, 128),
                                                (256, 64), (128, 32)])
def test_executor_flow_at_other_page_sizes_and_head_dims(page_size, head_dim):
    """The same host flow -- packed prefill, a chunk over cached history, fused decode steps --
    on pools with larger pages and other head dims."""
    print(f"executor: page_size {page_size}, head_dim {head_dim}", flush=True)
    hq, hkv = 16, 4
    scale = 1.0 / math.sqrt(head_dim)
    ex = ModelExecutor(num_layers=1, num_q_heads=hq, num_kv_heads=hkv, head_dim=head_dim, num_pages=64,
                       max_seq_len=512, max_requests=8, device=DEV, page_size=page_size)
    ex.kv_mem_manager.gpu_kv_buffer[0].normal_()
    attn = Attention(hq, hkv, head_dim)

    def rows(tokens, heads, seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        return torch.randn((tokens, heads, head_dim), generator=g, device=DEV, dtype=torch.float16)

    lens = [37, 16, 90, 5]
    if page_size > 64:
        lens.append(page_size - 6)           # crosses into its second page during the decode steps
    ids = ex.reserve_paged_requests(lens, reserved_lengths=[n + 60 for n in lens])
    ex.activate_paged_packed_prefill_batch(ids, lens)
    info = ex.atten_info
    assert info.page_size == page_size
    q, k, v = rows(sum(lens), hq, 1), rows(sum(lens), hkv, 2), rows(sum(lens), hkv, 3)
    out = attn.context_forward(q, k, v, info, 0, scale * LOG2E)
    torch.cuda.synchronize()
    ref = c_oracle.varlen_prefill(to_np16(q), to_np16(k), to_np16(v), info.b_start_loc.cpu().numpy(),
                                  np.asarray(lens, dtype=np.int32), scale)
    assert_attention_close(out, ref, "prefill")
    # a chunk of 30 more tokens for request 2, over its 90 cached ones
    ex.activate_paged_chunk_prefill_batch((ids[2],), [90], [30])
    info = ex.atten_info
    q, k, v = rows(30, hq, 4), rows(30, hkv, 5), rows(30, hkv, 6)
    out = attn.context_forward(q, k, v, info, 0, scale * LOG2E)
    torch.cuda.synchronize()
    ref = c_oracle.paged_prefill(to_np16(q), to_np16(info.kv_buffer[0]), info.block_table.cpu().numpy(),
                                 info.cu_q_lens.cpu().numpy(), info.context_lens_i32.cpu().numpy(), scale,
                                 page_size=page_size)
    assert_attention_close(out, ref, "chunk over history")
    for step in range(20):
        ex.extend_paged_requests(ids)
        info = ex.atten_info
        q, k, v = rows(len(ids), hq, 100 + step), rows(len(ids), hkv, 200 + step), rows(len(ids), hkv, 300 + step)
        out = attn.token_forward(q, k, v, info, 0, qk_scale=scale)
        torch.cuda.synchronize()
        sel = info.cur_select_index.long()
        assert_bit_exact(info.kv_buffer[0][sel][:, :hkv], k, "appended K")
        ref = c_oracle.paged_decode(to_np16(q), to_np16(info.kv_buffer[0]), info.block_table.cpu().numpy(),
                                    info.seq_lens_i32.cpu().numpy(), scale, page_size=page_size)
        assert_attention_close(out, ref, f"decode step {step}")
