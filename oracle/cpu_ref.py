"""PyTorch-CPU restatement of the reference's own torch implementations of the
paged-KV attention path. TEST INFRASTRUCTURE (and the timed `cpu_baseline`):
never imported by the product package.

Each function follows the torch code the reference keeps next to its Triton
kernels, with two deliberate differences that the target tolerance (max-abs
2e-3, max-rel 1e-2 against an fp32-accumulated result) calls for: scores,
softmax and the PV product stay in fp32 (the reference casts probabilities to
fp16 before PV), and the natural softmax scale is used throughout.
Kernel-level parity with the Triton-Ascend kernels themselves is unpinned: the
reference stores no numeric golden vectors for them.
"""

from __future__ import annotations

import math
from typing import Optional

import torch


def slots_of(block_row: torch.Tensor, n_tokens: int, page_size: int) -> torch.Tensor:
    """Physical slot of logical tokens 0..n-1: page * page_size + offset
    (lite_llama/executor/paged_attention.py:141-146, 347-354)."""
    t = torch.arange(n_tokens, dtype=torch.long)
    pages = block_row.to(torch.long)[t // page_size]
    return pages * page_size + t % page_size


def kv_append_ref(kv_values: torch.Tensor, select_index: torch.Tensor, kv_buffer: torch.Tensor) -> None:
    """KV_Buffer[Select_Index[i]] = KV_Values[i]
    (lite_llama/kernels/update_kv_buffer.py:47-56; torch form `dest[dest_loc] = src`, :104-105)."""
    kv_buffer[select_index.to(torch.long)] = kv_values


def page_copy_ref(pool: torch.Tensor, src_ids: torch.Tensor, dst_ids: torch.Tensor, page_size: int = 16) -> None:
    """pool[page dst] = pool[page src]; closed form, no counterpart in the reference."""
    paged = pool.view(pool.shape[0] // page_size, page_size, *pool.shape[1:])
    paged[dst_ids.to(torch.long)] = paged[src_ids.to(torch.long)].clone()


def page_gather_ref(src_pool: torch.Tensor, dst_pool: torch.Tensor, src_ids: torch.Tensor,
                    dst_ids: Optional[torch.Tensor] = None, page_size: int = 16) -> None:
    """dst_pool[page dst_ids[i]] = src_pool[page src_ids[i]]; dst_ids None means page i."""
    s = src_pool.view(src_pool.shape[0] // page_size, page_size, *src_pool.shape[1:])
    d = dst_pool.view(dst_pool.shape[0] // page_size, page_size, *dst_pool.shape[1:])
    if dst_ids is None:
        dst_ids = torch.arange(src_ids.numel())
    d[dst_ids.to(torch.long)] = s[src_ids.to(torch.long)].clone()


def _attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
            mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [H, M, D], k/v [H, N, D] fp32 -> softmax(q k^T scale + mask) v in fp32."""
    scores = torch.matmul(q, k.transpose(1, 2)) * scale
    if mask is not None:
        scores = scores.masked_fill(~mask, float("-inf"))
    return torch.matmul(torch.softmax(scores, dim=-1), v)


def paged_decode_ref(q: torch.Tensor, kv_pool: torch.Tensor, block_table: torch.Tensor,
                     seq_lens: torch.Tensor, scale: Optional[float] = None, page_size: int = 16,
                     dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Decode attention, one query token per sequence.

    The reference's torch decode (lite_llama/kernels/flashdecoding.py:348-374:
    per-sequence matmul -> fp32 softmax -> matmul) applied after gathering K/V
    through the table, i.e. lite_llama/kernels/paged_chunk_flashattention.py:196-221
    with q_len = 1; kv head = head // (Hq / Hkv) (:186, :211).
    Returns fp32 (or fp64) [B, Hq, D], not rounded to fp16.
    """
    b, hq, d = q.shape
    hkv = kv_pool.shape[1] // 2
    group = hq // hkv
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    out = torch.zeros((b, hq, d), dtype=dtype)
    for i in range(b):
        n = int(seq_lens[i])
        if n <= 0:
            continue
        slots = slots_of(block_table[i], n, page_size)
        rows = kv_pool[slots].to(dtype)                              # [n, 2*Hkv, D]
        k = rows[:, :hkv].transpose(0, 1).repeat_interleave(group, dim=0)   # [Hq, n, D]
        v = rows[:, hkv:].transpose(0, 1).repeat_interleave(group, dim=0)
        out[i] = _attend(q[i].to(dtype).unsqueeze(1), k, v, scale).squeeze(1)
    return out


def flash_decoding_ref(q: torch.Tensor, kv_pool: torch.Tensor, block_table: torch.Tensor,
                       seq_lens: torch.Tensor, scale: float, partition: int = 128, page_size: int = 16):
    """The reference's two-stage algorithm in fp32: per-partition online softmax giving
    mid_o = acc / d and lse = m + log d (lite_llama/kernels/flashdecoding.py:96-138), then the
    sequential merge (:242-267). Returns (out [B, Hq, D], mid_o, mid_lse)."""
    b, hq, d = q.shape
    hkv = kv_pool.shape[1] // 2
    group = hq // hkv
    parts = max(1, (int(seq_lens.max()) + partition - 1) // partition)
    mid_o = torch.zeros((b, hq, parts, d))
    mid_lse = torch.full((b, hq, parts), float("-inf"))
    out = torch.zeros((b, hq, d))
    for i in range(b):
        n = int(seq_lens[i])
        slots = slots_of(block_table[i], n, page_size)
        rows = kv_pool[slots].float()
        k = rows[:, :hkv].transpose(0, 1).repeat_interleave(group, dim=0)
        v = rows[:, hkv:].transpose(0, 1).repeat_interleave(group, dim=0)
        qi = q[i].float()
        n_parts = (n + partition - 1) // partition
        for p in range(n_parts):
            sl = slice(p * partition, min(n, (p + 1) * partition))
            s = torch.einsum("hd,hnd->hn", qi, k[:, sl]) * scale
            m = s.max(dim=-1).values
            e = torch.exp(s - m[:, None])
            den = e.sum(dim=-1)
            mid_o[i, :, p] = torch.einsum("hn,hnd->hd", e, v[:, sl]) / den[:, None]
            mid_lse[i, :, p] = m + torch.log(den)
        m_run = torch.full((hq,), float("-inf"))
        d_run = torch.zeros(hq)
        acc = torch.zeros((hq, d))
        for p in range(n_parts):
            m_new = torch.maximum(m_run, mid_lse[i, :, p])
            alpha = torch.exp(m_run - m_new)
            w = torch.exp(mid_lse[i, :, p] - m_new)
            acc = alpha[:, None] * acc + w[:, None] * mid_o[i, :, p]
            d_run = alpha * d_run + w
            m_run = m_new
        if n_parts:
            out[i] = acc / d_run[:, None]
    return out, mid_o, mid_lse


def paged_prefill_ref(q: torch.Tensor, kv_pool: torch.Tensor, block_table: torch.Tensor,
                      cu_q_lens: torch.Tensor, context_lens: Optional[torch.Tensor],
                      scale: Optional[float] = None, page_size: int = 16,
                      dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Causal chunk attention over paged KV
    (lite_llama/kernels/paged_chunk_flashattention.py:179-222): query row m sits at logical
    position ctx + m, mask is q_pos >= key_pos (:203-210), keys gathered through the table
    (:196). Returns fp32 [T, Hq, D]."""
    t, hq, d = q.shape
    hkv = kv_pool.shape[1] // 2
    group = hq // hkv
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    out = torch.zeros((t, hq, d), dtype=dtype)
    for i in range(cu_q_lens.numel() - 1):
        q0, q1 = int(cu_q_lens[i]), int(cu_q_lens[i + 1])
        qn = q1 - q0
        if qn <= 0:
            continue
        ctx = 0 if context_lens is None else int(context_lens[i])
        n = ctx + qn
        rows = kv_pool[slots_of(block_table[i], n, page_size)].to(dtype)
        k = rows[:, :hkv].transpose(0, 1).repeat_interleave(group, dim=0)
        v = rows[:, hkv:].transpose(0, 1).repeat_interleave(group, dim=0)
        q_pos = torch.arange(ctx, ctx + qn)
        mask = q_pos[:, None] >= torch.arange(n)[None, :]
        out[q0:q1] = _attend(q[q0:q1].to(dtype).transpose(0, 1), k, v, scale, mask).transpose(0, 1)
    return out


def varlen_prefill_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_starts: torch.Tensor,
                       seq_lens: torch.Tensor, scale: Optional[float] = None) -> torch.Tensor:
    """Per-sequence causal attention over packed contiguous K/V with the library routine the
    reference itself uses (lite_llama/kernels/flashattention2_nopad.py:250-274:
    `scaled_dot_product_attention(..., is_causal=True)` per sequence), GQA by head repeat.
    Returns fp32 [T, Hq, D]."""
    t, hq, d = q.shape
    group = hq // k.shape[1]
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    out = torch.zeros((t, hq, d), dtype=torch.float32)
    for i in range(seq_lens.numel()):
        s0, n = int(seq_starts[i]), int(seq_lens[i])
        if n <= 0:
            continue
        qi = q[s0:s0 + n].float().transpose(0, 1).unsqueeze(0)
        ki = k[s0:s0 + n].float().transpose(0, 1).repeat_interleave(group, dim=0).unsqueeze(0)
        vi = v[s0:s0 + n].float().transpose(0, 1).repeat_interleave(group, dim=0).unsqueeze(0)
        oi = torch.nn.functional.scaled_dot_product_attention(qi, ki, vi, is_causal=True, scale=scale)
        out[s0:s0 + n] = oi.squeeze(0).transpose(0, 1)
    return out
