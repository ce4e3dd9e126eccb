"""Drop-in replacements for the four attention-path functions of ``lite_llama.kernels``
(lite_llama/kernels/__init__.py:1-16), same names, argument order and return values, running on the
HIP kernels of liblitekv:

    update_kv_buffer(KV_Values, Select_Index, KV_Buffer)
    flash_decoding(q, k_cache, v_cache, qk_scale, b_req_tokens_table, b_seq_len, max_actual_seq_len)
    flash_attention2_no_pad(q, k, v, sm_scale, b_start_loc, b_seq_len, max_seq_len)
    paged_chunk_flash_attention(q, k_cache, v_cache, sm_scale, req_token_table, req_ids,
                                q_start_loc, context_lens, q_seq_lens, max_q_len)

The reference's callers pass a per-token slot table and K/V as the two strided halves of one
pool; the wrappers recover the pool and the per-page block table from them on the device
(slot // page_size of every page_size-th column), without a host round trip. Code that already
holds block tables should call ``llama_lite_npu_amd.ops`` directly.
"""

from __future__ import annotations

import torch

from .. import ops

PAGE_SIZE = ops.PAGE_SIZE
LOG2E = 1.4426950408889634


def update_kv_buffer(KV_Values: torch.Tensor, Select_Index: torch.Tensor, KV_Buffer: torch.Tensor) -> None:
    """KV_Buffer[Select_Index[i], :, :] = KV_Values[i, :, :] (lite_llama/kernels/update_kv_buffer.py:46-81).
    KV_Values is [tokens, 2 * Hkv, D]: K heads then V heads, as torch.cat([xk, xv], dim=-2) builds it."""
    assert KV_Values.shape[1] == KV_Buffer.shape[1] and KV_Values.shape[2] == KV_Buffer.shape[2]
    hkv = KV_Values.shape[1] // 2
    ops.kv_append(KV_Values[:, :hkv], KV_Values[:, hkv:], Select_Index, KV_Buffer)


def _pool_of(k_cache: torch.Tensor, v_cache: torch.Tensor) -> torch.Tensor:
    """The [slots, 2 * Hkv, D] pool whose halves are k_cache = pool[:, :Hkv], v_cache = pool[:, Hkv:]
    (lite_llama/models/qwen3.py:68-69)."""
    slots, hkv, d = k_cache.shape
    ok = (k_cache.stride() == (2 * hkv * d, d, 1) and v_cache.stride() == k_cache.stride()
          and v_cache.data_ptr() == k_cache.data_ptr() + hkv * d * k_cache.element_size())
    if not ok:
        raise ValueError("k_cache / v_cache must be the K and V halves of one [slots, 2*Hkv, D] pool")
    return torch.as_strided(k_cache, (slots, 2 * hkv, d), (2 * hkv * d, d, 1))


def _block_table_of(token_table_rows: torch.Tensor, page_size: int = PAGE_SIZE) -> torch.Tensor:
    """Per-page table from a per-token slot table: a page's slots are consecutive
    (lite_llama/executor/paged_attention.py:141-146), so column p * page_size holds page * page_size."""
    return torch.div(token_table_rows[:, ::page_size], page_size, rounding_mode="floor").to(torch.int32).contiguous()


def flash_decoding(q, k_cache, v_cache, qk_scale, b_req_tokens_table, b_seq_len, max_actual_seq_len):
    """Decode attention, out [B, Hq, D] (lite_llama/kernels/flashdecoding.py:294-342). Row i of the
    table belongs to batch row i, as in the reference kernel (:48, :84-88)."""
    assert q.shape[-1] == k_cache.shape[-1] == v_cache.shape[-1]
    pool = _pool_of(k_cache, v_cache)
    b = q.shape[0]
    cols = ((int(max_actual_seq_len) + PAGE_SIZE - 1) // PAGE_SIZE) * PAGE_SIZE
    table = _block_table_of(b_req_tokens_table[:b, :cols])
    # The host knows the batch size and the longest sequence: with every sequence taken to be that
    # long, small steps go one or several wavefronts per sequence and kv head, the rest balanced.
    hkv, d = k_cache.shape[1], k_cache.shape[2]
    max_pages = cols // PAGE_SIZE
    splits = ops.decode_schedule(b, hkv, max_pages, b * max_pages, 2 * hkv * d * q.element_size(),
                                 heads_per_kv_head=q.shape[1] // hkv)
    if splits:
        return ops.paged_decode(q, pool, table, b_seq_len, float(qk_scale), num_splits=splits, schedule="splits")
    return ops.paged_decode(q, pool, table, b_seq_len, float(qk_scale))


def flash_attention2_no_pad(q, k, v, sm_scale, b_start_loc, b_seq_len, max_seq_len):
    """Causal varlen prefill over packed contiguous K/V (lite_llama/kernels/flashattention2_nopad.py:169-221).
    ``sm_scale`` carries the log2(e) factor the reference's callers fold in (qwen3.py:295-298)."""
    return ops.varlen_prefill(q.half(), k.half(), v.half(), b_start_loc, b_seq_len, int(max_seq_len),
                              float(sm_scale) / LOG2E)


def paged_chunk_flash_attention(q, k_cache, v_cache, sm_scale, req_token_table, req_ids, q_start_loc,
                                context_lens, q_seq_lens, max_q_len):
    """Causal attention of packed query chunks over paged history + chunk
    (lite_llama/kernels/paged_chunk_flashattention.py:225-327). ``sm_scale`` carries log2(e)."""
    if q.numel() == 0:
        return torch.empty_like(q)
    pool = _pool_of(k_cache, v_cache)
    rows = req_token_table.index_select(0, req_ids.to(torch.long))
    table = _block_table_of(rows)
    q_lens = q_seq_lens.to(torch.int32)
    cu = torch.cat([q_start_loc.to(torch.int32), (q_start_loc[-1:].to(torch.int32) + q_lens[-1:])])
    return ops.paged_prefill(q.half(), pool, table, cu, context_lens, int(max_q_len), float(sm_scale) / LOG2E)


__all__ = ["update_kv_buffer", "flash_decoding", "flash_attention2_no_pad", "paged_chunk_flash_attention"]
