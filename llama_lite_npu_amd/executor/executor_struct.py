"""Per-step attention metadata handed from the executor to the attention layers.

Field names follow the reference's ``AttentionInfo``
(lite_llama/executor/executor_struct.py:30-40, filled by
lite_llama/executor/model_executor.py:685-911); the block-table fields at the
end are what the HIP kernels consume.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional

import torch


@dataclass
class AttentionInfo:
    kv_buffer: list = field(default_factory=list)        # per layer [slots, 2*Hkv, D] pool (fp16, or E4M3 codes)
    kv_scales: list = field(default_factory=list)        # per layer float32 [2*Hkv] scales of an fp8 pool, else None
    cur_select_index: Optional[torch.Tensor] = None      # slot mapping of the step's new tokens (int32)
    b_req_tokens_table: Any = None                       # per-token slot table, or None (built on demand)
    b_start_loc: Optional[torch.Tensor] = None           # packed-row start of each sequence (int32)
    b_req_idx: Optional[torch.Tensor] = None             # request ids of the batch (int32)
    b_seq_len: Optional[torch.Tensor] = None             # tokens visible to attention per sequence (int64)
    max_actual_seq_len: int = 0
    is_paged_chunk_prefill: bool = False
    chunk_context_len: Optional[torch.Tensor] = None     # tokens cached before the chunk (int64)
    chunk_q_seq_len: Optional[torch.Tensor] = None       # chunk lengths (int64)
    max_actual_q_seq_len: Optional[int] = None
    # block-table view of the same batch
    block_table: Optional[torch.Tensor] = None           # [B, max_blocks] int32 page ids, batch order
    seq_lens_i32: Optional[torch.Tensor] = None          # b_seq_len as int32
    cu_q_lens: Optional[torch.Tensor] = None             # [B+1] int32 packed-row offsets (prefill)
    context_lens_i32: Optional[torch.Tensor] = None      # chunk_context_len as int32
    page_size: int = 16                                  # tokens per page of the pools (16, 32, 64, 128 or 256)
    decode_plan: Any = None                              # ops.DecodePlan of the step (decode only)
    device_decode: Any = None                            # DeviceDecodeBatch that owns the tensors above, if any
