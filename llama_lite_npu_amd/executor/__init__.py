"""Executor-side metadata of the paged KV cache (mirror of the reference's lite_llama/executor)."""

from .executor_struct import AttentionInfo
from .paged_attention import PagedKVCacheManager, PagedReqTokensManager
from .model_executor import ModelExecutor
from .decode_graph import DecodeGraphRunner, DeviceDecodeBatch, supports_decode_graph

__all__ = ["AttentionInfo", "PagedKVCacheManager", "PagedReqTokensManager", "ModelExecutor",
           "DecodeGraphRunner", "DeviceDecodeBatch", "supports_decode_graph"]
