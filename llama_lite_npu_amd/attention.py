"""The per-layer attention step of the models: append this step's K/V, then attend.

Mirror of ``Attention.context_forward / token_forward`` in the reference's model files
(lite_llama/models/qwen3.py:12-75, same in qwen2.py and llama.py): same method names and
arguments, driven by the same ``AttentionInfo``. Differences:

* no ``torch.cat([xk, xv])``: K and V rows go to the pool straight from their own tensors;
* decode is one fused launch (append + attention) when the step carries a ``DecodePlan``;
* prefill reads K/V through the block table (context 0 for a fresh prompt, history for later
  chunks), so one kernel serves both branches of the reference;
* ``qkv_epilogue`` folds the step before the append (QK RMSNorm, rotary embedding,
  qwen3.py:124-129) into the append itself; the forward calls are then made with ``xk=None``.

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

    def qkv_epilogue(self, xq, xk, xv, atten_info, layer_index: int, q_norm_weight=None,
                     k_norm_weight=None, position_embeddings=None, rms_eps: float = 1e-6) -> torch.Tensor:
        """The tail of ``_get_qkv`` (qwen3.py:124-129) fused with the KV append: per-head RMSNorm of
        xq / xk (weights None: skipped), rotary embedding with the (cos, sin) rows of the tokens'
        positions, and k / v written into their slots. xq is updated in place and returned; call
        ``context_forward`` / ``token_forward`` afterwards with ``xk=None, xv=None``."""
        cos, sin = position_embeddings if position_embeddings is not None else (None, None)
        return ops.qk_norm_rope_append(xq, xk, xv, atten_info.cur_select_index,
                                       atten_info.kv_buffer[layer_index], q_norm_weight, k_norm_weight,
                                       cos, sin, rms_eps)

    def context_forward(self, xq, xk, xv, atten_info, layer_index: int, qk_scale=None) -> torch.Tensor:
        """Prefill: xq [T, Hq, D], xk / xv [T, Hkv, D] packed rows of the batch's prompts or chunks
        (None when ``qkv_epilogue`` already stored them)."""
        pool = atten_info.kv_buffer[layer_index]
        if xk is not None:
            ops.kv_append(xk, xv, atten_info.cur_select_index, pool)
        scale = (1.0 / math.sqrt(self.head_dim)) if qk_scale is None else float(qk_scale) / LOG2E
        if getattr(atten_info, "is_paged_chunk_prefill", False):
            return ops.paged_prefill(xq, pool, atten_info.block_table, atten_info.cu_q_lens,
                                     atten_info.context_lens_i32, int(atten_info.max_actual_q_seq_len), scale)
        return ops.paged_prefill(xq, pool, atten_info.block_table, atten_info.cu_q_lens, None,
                                 int(atten_info.max_actual_seq_len), scale)

    def token_forward(self, xq, xk, xv, atten_info, layer_index: int, qk_scale=None) -> torch.Tensor:
        """Decode: xq [B, Hq, D], xk / xv [B, Hkv, D], one new token per sequence (None when
        ``qkv_epilogue`` already stored them)."""
        pool = atten_info.kv_buffer[layer_index]
        scale = (1.0 / math.sqrt(self.head_dim)) if qk_scale is None else float(qk_scale)
        plan = getattr(atten_info, "decode_plan", None)
        if plan is not None:
            return ops.decode_step(xq, pool, plan, xk, xv, scale)
        if xk is not None:
            ops.kv_append(xk, xv, atten_info.cur_select_index, pool)
        return ops.paged_decode(xq, pool, atten_info.block_table, atten_info.seq_lens_i32, scale)
