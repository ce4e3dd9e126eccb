"""The per-layer attention step of the models: append this step's K/V, then attend.

Mirror of ``Attention.context_forward / token_forward`` in the reference's model files
(lite_llama/models/qwen3.py:12-75, same in qwen2.py and llama.py): same method names and
arguments, driven by the same ``AttentionInfo``. Differences:

* no ``torch.cat([xk, xv])``: K and V rows go to the pool straight from their own tensors;
* decode follows the step's ``DecodePlan``: one fused launch (append + attention) and a merge
  on the balanced schedule, or the append fused into one wavefront (no merge) or several splits
  (+ merge) per (sequence, kv head) where the plan found the step small enough for that to be
  faster;
* prefill reads K/V through the block table (context 0 for a fresh prompt, history for later
  chunks), so one kernel serves both branches of the reference;
* ``qkv_epilogue`` folds the step before the append (QK RMSNorm, rotary embedding,
  qwen3.py:124-129) into the append itself; the forward calls are then made with ``xk=None``;
* a layer whose pool holds fp8 or int8 codes (``atten_info.kv_scales[layer]`` set) quantises on append
  and attends straight from the codes, in decode and in chunks over cached history; fresh
  prompts attend to their own fp16 K/V.

``qk_scale`` follows the reference's convention (qwen3.py:295-298): the natural 1/sqrt(D) for
decode, multiplied by log2(e) for prefill; it is un-folded here.
"""

from __future__ import annotations

import math

import torch

from . import ops

LOG2E = 1.4426950408889634


def _page_size(atten_info) -> int:
    """Tokens per page of the step's pools (metadata built by other code may not carry it: 16)."""
    return int(getattr(atten_info, "page_size", 16) or 16)


class Attention:
    def __init__(self, num_q_heads: int, num_kv_heads: int, head_dim: int):
        self.num_q_heads = num_q_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.hidden_size = num_q_heads * head_dim

    def qkv_epilogue(self, xq, xk, xv, atten_info, layer_index: int, q_norm_weight=None,
                     k_norm_weight=None, position_embeddings=None, rms_eps: float = 1e-6) -> torch.Tensor:
        """The tail of ``_get_qkv`` (qwen3.py:124-129) fused with the KV append: per-head RMSNorm of
        xq / xk (weights None: skipped), rotary embedding with the (cos, sin) rows of the tokens'
        positions, and k / v written into their slots. xq is updated in place and returned; call
        ``context_forward`` / ``token_forward`` afterwards with ``xk=None, xv=None``."""
        cos, sin = position_embeddings if position_embeddings is not None else (None, None)
        pool = atten_info.kv_buffer[layer_index]
        scales = atten_info.kv_scales[layer_index] if ops.is_quantised_pool(pool) else None
        return ops.qk_norm_rope_append(xq, xk, xv, atten_info.cur_select_index, pool, q_norm_weight,
                                       k_norm_weight, cos, sin, rms_eps, kv_scales=scales)

    def context_forward(self, xq, xk, xv, atten_info, layer_index: int, qk_scale=None) -> torch.Tensor:
        """Prefill: xq [T, Hq, D], xk / xv [T, Hkv, D] packed rows of the batch's prompts or chunks
        (None when ``qkv_epilogue`` already stored them)."""
        pool = atten_info.kv_buffer[layer_index]
        scale = (1.0 / math.sqrt(self.head_dim)) if qk_scale is None else float(qk_scale) / LOG2E
        if ops.is_quantised_pool(pool):
            return self._context_forward_fp8(xq, xk, xv, atten_info, pool, atten_info.kv_scales[layer_index], scale)
        if xk is not None:
            ops.kv_append(xk, xv, atten_info.cur_select_index, pool)
        # max_kv_len: the longest history + chunk of the batch, which the executor knows on the host;
        # a lone chunk over a long history is then cut along its keys as well (ops.paged_prefill)
        if getattr(atten_info, "is_paged_chunk_prefill", False):
            return ops.paged_prefill(xq, pool, atten_info.block_table, atten_info.cu_q_lens,
                                     atten_info.context_lens_i32, int(atten_info.max_actual_q_seq_len), scale,
                                     page_size=_page_size(atten_info),
                                     max_kv_len=int(atten_info.max_actual_seq_len))
        return ops.paged_prefill(xq, pool, atten_info.block_table, atten_info.cu_q_lens, None,
                                 int(atten_info.max_actual_seq_len), scale, page_size=_page_size(atten_info),
                                 max_kv_len=int(atten_info.max_actual_seq_len))

    def _context_forward_fp8(self, xq, xk, xv, atten_info, pool, scales, scale) -> torch.Tensor:
        chunked = getattr(atten_info, "is_paged_chunk_prefill", False)
        if xk is not None:
            ops.kv_append_quantised(xk, xv, atten_info.cur_select_index, pool, scales)
            if not chunked:
                # a fresh prompt attends to its own K/V as computed, not as stored
                return ops.varlen_prefill(xq, xk, xv, atten_info.b_start_loc, atten_info.seq_lens_i32,
                                          int(atten_info.max_actual_seq_len), scale)
        # history (or rows already stored by the epilogue): the kernel reads the codes themselves
        if chunked:
            return ops.paged_prefill(xq, pool, atten_info.block_table, atten_info.cu_q_lens,
                                     atten_info.context_lens_i32, int(atten_info.max_actual_q_seq_len), scale,
                                     kv_scales=scales, page_size=_page_size(atten_info),
                                     max_kv_len=int(atten_info.max_actual_seq_len))
        return ops.paged_prefill(xq, pool, atten_info.block_table, atten_info.cu_q_lens, None,
                                 int(atten_info.max_actual_seq_len), scale, kv_scales=scales,
                                 page_size=_page_size(atten_info), max_kv_len=int(atten_info.max_actual_seq_len))

    def token_forward(self, xq, xk, xv, atten_info, layer_index: int, qk_scale=None) -> torch.Tensor:
        """Decode: xq [B, Hq, D], xk / xv [B, Hkv, D], one new token per sequence (None when
        ``qkv_epilogue`` already stored them)."""
        pool = atten_info.kv_buffer[layer_index]
        scale = (1.0 / math.sqrt(self.head_dim)) if qk_scale is None else float(qk_scale)
        plan = getattr(atten_info, "decode_plan", None)
        scales = atten_info.kv_scales[layer_index] if ops.is_quantised_pool(pool) else None
        if plan is not None:
            return ops.decode_step(xq, pool, plan, xk, xv, scale, kv_scales=scales)
        if xk is not None:
            if scales is not None:
                ops.kv_append_quantised(xk, xv, atten_info.cur_select_index, pool, scales)
            else:
                ops.kv_append(xk, xv, atten_info.cur_select_index, pool)
        return ops.paged_decode(xq, pool, atten_info.block_table, atten_info.seq_lens_i32, scale, kv_scales=scales,
                                page_size=_page_size(atten_info))
