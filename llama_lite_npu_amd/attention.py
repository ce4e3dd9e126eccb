"""The per-layer attention step of the models: append this step's K/V, then attend.

Mirror of ``Attention.context_forward / token_forward`` in the reference's model files
(lite_llama/models/qwen3.py:12-75, same in qwen2.py and llama.py): same method names and
arguments, driven by the same ``AttentionInfo``. Differences:

* no ``torch.cat([xk, xv])``: K and V rows go to the pool straight from their own tensors;
* decode is one fused launch (append + attention) when the step carries a ``DecodePlan``;
* prefill reads K/V through the block table (context 0 for a fresh prompt, history for later
  chunks), so one kernel serves both branches of the reference.

``qk_scale`` follows the reference's convention (qwen3.py:295-298): the natural 1/sqrt(D) for
decode, multiplied by log2(e) for prefill; it is un-folded here.
"""

from __future__ import annotations

import math

import torch

from . import ops

LOG2E = 1.4426950408889634


class Attention:
    def __init__(self, num_q_heads: int, num_kv_heads: int, head_dim: int):
        self.num_q_heads = num_q_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.hidden_size = num_q_heads * head_dim

    def context_forward(self, xq, xk, xv, atten_info, layer_index: int, qk_scale=None) -> torch.Tensor:
        """Prefill: xq [T, Hq, D], xk / xv [T, Hkv, D] packed rows of the batch's prompts or chunks."""
        pool = atten_info.kv_buffer[layer_index]
        ops.kv_append(xk, xv, atten_info.cur_select_index, pool)
        scale = (1.0 / math.sqrt(self.head_dim)) if qk_scale is None else float(qk_scale) / LOG2E
        if getattr(atten_info, "is_paged_chunk_prefill", False):
            return ops.paged_prefill(xq, pool, atten_info.block_table, atten_info.cu_q_lens,
                                     atten_info.context_lens_i32, int(atten_info.max_actual_q_seq_len), scale)
        return ops.paged_prefill(xq, pool, atten_info.block_table, atten_info.cu_q_lens, None,
                                 int(atten_info.max_actual_seq_len), scale)

    def token_forward(self, xq, xk, xv, atten_info, layer_index: int, qk_scale=None) -> torch.Tensor:
        """Decode: xq [B, Hq, D], xk / xv [B, Hkv, D], one new token per sequence."""
        pool = atten_info.kv_buffer[layer_index]
        scale = (1.0 / math.sqrt(self.head_dim)) if qk_scale is None else float(qk_scale)
        plan = getattr(atten_info, "decode_plan", None)
        if plan is not None:
            return ops.decode_step(xq, pool, plan, xk, xv, scale)
        ops.kv_append(xk, xv, atten_info.cur_select_index, pool)
        return ops.paged_decode(xq, pool, atten_info.block_table, atten_info.seq_lens_i32, scale)
