"""Paged-KV metadata API of the executor: request reservation, prefix-cache sharing and the
per-step ``AttentionInfo`` builders.

Method names, arguments, return values and error texts follow the paged half of the reference's
``ModelExecutor`` (lite_llama/executor/model_executor.py:496-987); model loading, tensor-parallel
weight sharding and graph capture are not part of this package. Differences underneath:

* every builder assembles its slot mappings and lengths on the host and uploads each tensor
  once (the reference concatenates per-request device views);
* the batch's block-table rows travel with the metadata (``atten_info.block_table``), and a
  decode step carries a ``DecodePlan`` shared by all layers;
* ``copy_on_write`` runs before appends into shared pages, and ``compact_kv_pool`` exists.
"""

from __future__ import annotations

from collections import OrderedDict
from typing import Optional, Sequence

import numpy as np
import torch

from .executor_struct import AttentionInfo
from .paged_attention import PagedKVCacheManager, PagedReqTokensManager


class ModelExecutor:
    """Owns the page pool, the request tables, the prefix caches and the step metadata."""

    def __init__(self, num_layers: int, num_q_heads: int, num_kv_heads: int, head_dim: int,
                 num_pages: int, max_seq_len: int, max_requests: Optional[int] = None,
                 page_size: int = 16, device: str = "cuda:0", dtype: torch.dtype = torch.float16,
                 tp_world_size: int = 1, build_decode_plans: bool = True):
        if page_size <= 0:
            raise ValueError("this executor only runs the paged path (page_size > 0)")
        self.device = device
        # heads are sharded over tensor-parallel ranks exactly as in the reference (:249-250)
        self.local_q_heads = num_q_heads // tp_world_size
        self.local_kv_heads = num_kv_heads // tp_world_size
        self.head_dim = head_dim
        self.num_layers = num_layers
        self.max_seq_len = int(max_seq_len)
        self.page_size = int(page_size)
        self.use_paged_attn = True
        self.kv_mem_manager = PagedKVCacheManager(num_layers, self.local_kv_heads, head_dim, num_pages,
                                                  page_size, dtype, device)
        if max_requests is None:
            max_requests = max(1, (num_pages * page_size) // self.max_seq_len)
        self.max_request_num = int(max_requests)
        self.req_tokens_manager = PagedReqTokensManager(self.max_request_num, self.max_seq_len,
                                                        self.kv_mem_manager, device=device)
        self.atten_info = AttentionInfo()
        self.atten_info.kv_buffer = self.kv_mem_manager.gpu_kv_buffer
        self.atten_info.kv_scales = self.kv_mem_manager.kv_scales
        self.atten_info.page_size = self.page_size
        self.build_decode_plans = build_decode_plans and torch.device(device).type == "cuda"
        # K + V bytes of one token in a layer's pool (what a decode step reads per token attended)
        self.kv_token_bytes = 2 * self.local_kv_heads * head_dim * torch.empty((), dtype=dtype).element_size()
        self.shared_prefix_min_pages = 4  # below that the two extra launches cost more than they save
        self._decode_plan = None
        self._paged_request_ids: tuple[int, ...] = ()
        self._device_batch = None            # DeviceDecodeBatch in charge of the running decode batch
        self._decode_meta_sig = None         # what the decode metadata in atten_info was last built from
        self._device_batches: dict = {}      # (batch size, shared pages) -> DeviceDecodeBatch
        self.model = None
        self.graph_runner = None
        # exact-prompt cache: prompt -> (pages, token count, first generated token), LRU of 128
        self._paged_prefix_cache: OrderedDict = OrderedDict()
        self._paged_prefix_cache_max_entries = 128
        # block cache: (fingerprint of the parent chain, block tokens) -> (page, tokens covered), LRU of 4096
        self._paged_block_prefix_cache: OrderedDict = OrderedDict()
        self._paged_block_prefix_cache_max_entries = 4096
        self.max_prefill_tokens = max(1, 60000 // max(1, self.local_q_heads))

    # ---- reservation -----------------------------------------------------------------------
    def reserve_paged_requests(self, prompt_lengths: Sequence[int],
                               reserved_lengths: Optional[Sequence[int]] = None) -> tuple[int, ...]:
        """One request id per prompt; on failure everything reserved by the call is released."""
        if reserved_lengths is not None and len(reserved_lengths) != len(prompt_lengths):
            raise ValueError("reserved_lengths must match prompt_lengths")
        made: list[int] = []
        try:
            for i, length in enumerate(prompt_lengths):
                cap = None if reserved_lengths is None else int(reserved_lengths[i])
                req_idx = self.req_tokens_manager.reserve_req(int(length), cap)
                if req_idx is None:
                    raise RuntimeError("Paged KV request or page capacity is exhausted")
                made.append(req_idx)
        except BaseException:
            for req_idx in made:
                self.req_tokens_manager.free_req(req_idx)
            raise
        return tuple(made)

    def ensure_paged_request_capacity(self, req_idx: int, total_tokens: int) -> None:
        if not self.req_tokens_manager.ensure_req_capacity(req_idx, total_tokens):
            raise RuntimeError(f"Paged KV capacity reservation failed for request {req_idx}")

    # ---- prefix caches ---------------------------------------------------------------------
    @staticmethod
    def _paged_block_key(parent_fingerprint, block_tokens):
        return parent_fingerprint, tuple(int(t) for t in block_tokens)

    def share_paged_request_from_cache(self, prompt_tokens) -> Optional[tuple[int, int]]:
        """Exact prompt hit: a new request sharing the cached pages, and the cached first token."""
        key = tuple(int(t) for t in prompt_tokens)
        hit = self._paged_prefix_cache.get(key)
        if hit is None:
            return None
        self._paged_prefix_cache.move_to_end(key)
        pages, num_tokens, first_token = hit
        req_idx = self.req_tokens_manager.reserve_shared_req(pages, num_tokens)
        return None if req_idx is None else (int(req_idx), int(first_token))

    def share_paged_prefix_from_cache(self, prompt_tokens) -> Optional[tuple[int, int, Optional[int]]]:
        """(request id, matched tokens, first token or None): the exact prompt if cached, else the
        longest chain of cached full pages (the caller then replays only the suffix)."""
        key = tuple(int(t) for t in prompt_tokens)
        if not key:
            return None
        exact = self._paged_prefix_cache.get(key)
        if exact is not None:
            self._paged_prefix_cache.move_to_end(key)
            pages, num_tokens, first_token = exact
            req_idx = self.req_tokens_manager.reserve_shared_req(pages, num_tokens)
            return None if req_idx is None else (int(req_idx), len(key), int(first_token))
        chain: list[torch.Tensor] = []
        matched, parent, ps = 0, None, self.page_size
        for first in range(0, len(key) - ps + 1, ps):
            block_key = self._paged_block_key(parent, key[first:first + ps])
            hit = self._paged_block_prefix_cache.get(block_key)
            if hit is None:
                break
            self._paged_block_prefix_cache.move_to_end(block_key)
            page, covered = hit
            chain.append(page.reshape(-1))
            matched = int(covered)
            parent = hash(block_key)
        if not chain or matched <= 0:
            return None
        req_idx = self.req_tokens_manager.reserve_shared_req(torch.cat(chain), matched)
        return None if req_idx is None else (int(req_idx), matched, None)

    def _store_paged_prompt_blocks(self, prompt_tokens: tuple[int, ...], page_indices: torch.Tensor) -> None:
        ps = self.page_size
        parent = None
        for block in range(len(prompt_tokens) // ps):
            block_key = self._paged_block_key(parent, prompt_tokens[block * ps:(block + 1) * ps])
            parent = hash(block_key)
            if block_key in self._paged_block_prefix_cache:
                self._paged_block_prefix_cache.move_to_end(block_key)
                continue
            page = page_indices[block:block + 1].clone()
            self.kv_mem_manager.add_ref(page)
            self._paged_block_prefix_cache[block_key] = (page, (block + 1) * ps)
            while len(self._paged_block_prefix_cache) > self._paged_block_prefix_cache_max_entries:
                _, (old_page, _) = self._paged_block_prefix_cache.popitem(last=False)
                self.kv_mem_manager.free(old_page)

    def store_paged_request_prefix(self, prompt_tokens, req_idx: int, first_token_id: int) -> None:
        """Caches a finished prefill: one page reference for the exact prompt, one per full block."""
        if req_idx not in self.req_tokens_manager.req_page_table:
            return
        key = tuple(int(t) for t in prompt_tokens)
        if key in self._paged_prefix_cache:
            return
        pages = self.req_tokens_manager.req_page_table[int(req_idx)]
        self.kv_mem_manager.add_ref(pages)
        self._paged_prefix_cache[key] = (pages.clone(), int(self.req_tokens_manager.req_token_count[int(req_idx)]),
                                         int(first_token_id))
        self._store_paged_prompt_blocks(key, pages)
        while len(self._paged_prefix_cache) > self._paged_prefix_cache_max_entries:
            _, (old_pages, _, _) = self._paged_prefix_cache.popitem(last=False)
            self.kv_mem_manager.free(old_pages)

    # ---- step metadata ---------------------------------------------------------------------
    def _reset_paged_chunk_prefill_metadata(self) -> None:
        info = self.atten_info
        info.is_paged_chunk_prefill = False
        info.chunk_context_len = info.chunk_q_seq_len = info.max_actual_q_seq_len = None
        info.context_lens_i32 = None
        info.decode_plan = None
        info.device_decode = None
        self._device_batch = None
        self._decode_meta_sig = None

    def _i32(self, values) -> torch.Tensor:
        return torch.as_tensor(np.asarray(values, dtype=np.int32), device=self.device)

    def _i64(self, values) -> torch.Tensor:
        return torch.as_tensor(np.asarray(values, dtype=np.int64), device=self.device)

    def _set_batch(self, request_ids: tuple[int, ...], kv_lens: Sequence[int], q_lens: Sequence[int],
                   slot_parts: list[np.ndarray]) -> None:
        """Common tail of the builders: ids, lengths, slot mapping, packed starts, block-table rows."""
        info, mgr = self.atten_info, self.req_tokens_manager
        self._paged_request_ids = request_ids
        info.b_req_idx = self._i32(request_ids)
        info.b_seq_len = self._i64(kv_lens)
        info.seq_lens_i32 = self._i32(kv_lens)
        info.cur_select_index = self._i32(np.concatenate(slot_parts) if slot_parts else [])
        cu = np.zeros(len(q_lens) + 1, dtype=np.int32)
        cu[1:] = np.cumsum(q_lens)
        info.cu_q_lens = self._i32(cu)
        info.b_start_loc = self._i32(cu[:-1])
        info.block_table = mgr.block_table_rows(request_ids)
        info.b_req_tokens_table = None   # derived from the block table only if somebody asks
        info.max_actual_seq_len = int(max(kv_lens))

    def activate_paged_prefill_batch(self, request_ids: tuple[int, ...], prompt_length: int) -> None:
        """Equal-length prompts, one prefill forward."""
        self._reset_paged_chunk_prefill_metadata()
        if not request_ids:
            raise ValueError("request_ids must not be empty")
        mgr = self.req_tokens_manager
        for req_idx in request_ids:
            actual = mgr.req_token_count[req_idx]
            if actual != prompt_length:
                raise ValueError("continuous prefill groups must have equal prompt "
                                 f"lengths: expected={prompt_length}, request={req_idx}, actual={actual}")
        ids = tuple(int(r) for r in request_ids)
        lens = [int(prompt_length)] * len(ids)
        self._set_batch(ids, lens, lens, [mgr.slots(r, 0, prompt_length) for r in ids])

    def activate_paged_packed_prefill_batch(self, request_ids, prompt_lengths):
        """Mixed-length prompts packed without padding. Returns (flat position ids, flat index of
        each request's last prompt token), both int64 on the device."""
        self._reset_paged_chunk_prefill_metadata()
        if not request_ids:
            raise ValueError("request_ids must not be empty")
        if len(request_ids) != len(prompt_lengths):
            raise ValueError("request_ids and prompt_lengths must have same length")
        lens = [int(n) for n in prompt_lengths]
        if any(n <= 0 for n in lens):
            raise ValueError("prompt_lengths must be positive")
        mgr = self.req_tokens_manager
        ids = tuple(int(r) for r in request_ids)
        for req_idx, n in zip(ids, lens):
            actual = mgr.req_token_count[req_idx]
            if actual != n:
                raise ValueError("packed prefill request length mismatch: "
                                 f"request={req_idx}, expected={n}, actual={actual}")
        self._set_batch(ids, lens, lens, [mgr.slots(r, 0, n) for r, n in zip(ids, lens)])
        ends = np.cumsum(lens)
        positions = np.concatenate([np.arange(n) for n in lens])
        return self._i64(positions), self._i64(ends - 1)

    def activate_paged_chunk_prefill_batch(self, request_ids, context_lengths, chunk_lengths):
        """Later chunks of a chunked prefill: extends each request by its chunk, then describes a
        batch whose queries are the chunks and whose keys are history + chunk, read through the
        pages. Returns (flat position ids, flat index of each chunk's last token)."""
        if not request_ids:
            raise ValueError("request_ids must not be empty")
        if len(request_ids) != len(context_lengths) or len(request_ids) != len(chunk_lengths):
            raise ValueError("request_ids, context_lengths and chunk_lengths must have same length")
        ids = tuple(int(r) for r in request_ids)
        ctx = [int(n) for n in context_lengths]
        chunk = [int(n) for n in chunk_lengths]
        if any(n < 0 for n in ctx):
            raise ValueError("context_lengths must be non-negative")
        if any(n <= 0 for n in chunk):
            raise ValueError("chunk_lengths must be positive")
        mgr = self.req_tokens_manager
        for req_idx, c, q in zip(ids, ctx, chunk):
            actual = mgr.req_token_count[req_idx]
            if actual != c:
                raise ValueError("paged chunk prefill context length mismatch: "
                                 f"request={req_idx}, expected={c}, actual={actual}")
            if not mgr.extend_req(req_idx, q):
                raise RuntimeError(
                    "Paged KV allocation failed for chunked prefill request "
                    f"{req_idx}: context_tokens={c}, chunk_tokens={q}, "
                    f"current_tokens={mgr.req_token_count.get(req_idx, 'unknown')}, "
                    f"max_seq_len={mgr.max_seq_len}, free_pages={mgr.page_mgr.num_free_pages}")
        self._reset_paged_chunk_prefill_metadata()
        total = [c + q for c, q in zip(ctx, chunk)]
        self._set_batch(ids, total, chunk, [mgr.slots(r, c, t) for r, c, t in zip(ids, ctx, total)])
        info = self.atten_info
        info.max_actual_q_seq_len = max(chunk)
        info.chunk_context_len = self._i64(ctx)
        info.chunk_q_seq_len = self._i64(chunk)
        info.context_lens_i32 = self._i32(ctx)
        info.is_paged_chunk_prefill = True
        ends = np.cumsum(chunk)
        positions = np.concatenate([np.arange(c, c + q) for c, q in zip(ctx, chunk)])
        return self._i64(positions), self._i64(ends - 1)

    def activate_paged_decode_batch(self, request_ids: tuple[int, ...]) -> None:
        """Metadata of one decode step: each sequence's length already counts the token whose K/V
        this step appends, and ``cur_select_index`` is that token's slot."""
        mgr = self.req_tokens_manager
        ids = tuple(int(r) for r in request_ids)
        # The backend activates the batch before a step and extend_paged_requests does after it:
        # the second of two calls with nothing changed in between (same requests, lengths and page
        # lists, no other batch activated) finds the metadata and the step plan already in place.
        sig = (ids, mgr.table_epoch, tuple(mgr.req_token_count.get(r) for r in ids))
        if sig == self._decode_meta_sig:
            return
        self._reset_paged_chunk_prefill_metadata()
        req_ids, seq_lens, last = mgr.batch_metadata(list(ids))
        info = self.atten_info
        self._paged_request_ids = ids
        info.b_req_idx, info.b_seq_len, info.cur_select_index = req_ids, seq_lens, last
        info.seq_lens_i32 = seq_lens.to(torch.int32)
        info.b_start_loc = torch.zeros(len(ids), dtype=torch.int32, device=self.device)
        info.cu_q_lens = torch.arange(len(ids) + 1, dtype=torch.int32, device=self.device)
        info.block_table = mgr.block_table_rows(ids)
        info.b_req_tokens_table = None
        info.max_actual_seq_len = max(mgr.req_token_count[r] for r in ids)
        if self.build_decode_plans:
            from .. import ops

            info.decode_plan = ops.DecodePlan(info.block_table, info.seq_lens_i32, self.local_q_heads,
                                              self.local_kv_heads, self.kv_mem_manager.num_pages,
                                              page_size=self.page_size,
                                              shared_pages=self.shared_prefix_pages(ids),
                                              host_seq_lens=[mgr.req_token_count[r] for r in ids],
                                              token_bytes=self.kv_token_bytes,
                                              kv_dtype=self.kv_mem_manager.gpu_kv_buffer[0].dtype)
        self._decode_meta_sig = sig

    def common_leading_pages(self, request_ids: Sequence[int], upcoming_tokens: int = 0) -> int:
        """How many leading pages are the same physical pages, and full, in every request of the
        batch. ``upcoming_tokens``: tokens the next step will add to each request before it attends
        (0 when ``extend_req`` has already booked them)."""
        mgr = self.req_tokens_manager
        ids = list(request_ids)
        if len(ids) < 2:
            return 0
        lists = [mgr.request_pages(r) for r in ids]
        # the page that receives this step's token, and everything after it, is private
        limit = min((mgr.req_token_count[r] + int(upcoming_tokens) - 1) // self.page_size for r in ids)
        limit = min(limit, min(len(p) for p in lists))
        first = lists[0]
        n = 0
        while n < limit and all(p[n] == first[n] for p in lists[1:]):
            n += 1
        return n

    def shared_prefix_pages(self, request_ids: Sequence[int], upcoming_tokens: int = 0) -> int:
        """Leading pages the decode step attends once for the whole batch (prefix-cache hits map one
        page list into many requests, :547-620). 0 when the batch shares fewer than
        ``shared_prefix_min_pages`` pages."""
        n = self.common_leading_pages(request_ids, upcoming_tokens)
        return n if n >= self.shared_prefix_min_pages else 0

    def activate_device_decode_batch(self, request_ids: Sequence[int], reserve_tokens: int = 0,
                                     host_ahead: bool = False):
        """Decode metadata that steps on the device (see ``DeviceDecodeBatch``): call once when the
        set of running requests changes, instead of ``activate_paged_decode_batch`` every step.
        Afterwards ``extend_paged_requests`` with the same ids only books the token on the host;
        the device half runs with the step (``forward``, a ``DecodeGraphRunner``, or
        ``device_batch.enqueue_advance()``). Batches are kept per (size, shared pages) so that
        graphs captured on their tensors stay valid. ``host_ahead``: the requests' lengths already
        count the token of the first step (``extend_paged_requests`` was called after the previous
        forward, as the reference's backend does); each later step is then forward first,
        ``extend_paged_requests`` afterwards."""
        from .decode_graph import DeviceDecodeBatch

        self._reset_paged_chunk_prefill_metadata()
        ids = tuple(int(r) for r in request_ids)
        shared = self.shared_prefix_pages(ids, upcoming_tokens=0 if host_ahead else 1)
        batch = self._device_batches.get((len(ids), shared))
        if batch is None:
            batch = DeviceDecodeBatch(self, ids, reserve_tokens, shared_pages=shared, host_ahead=host_ahead)
            self._device_batches[(len(ids), shared)] = batch
        else:
            batch.load(ids, reserve_tokens, host_ahead)
        batch.bind(self.atten_info)
        self._paged_request_ids = ids
        self._device_batch = batch
        return batch

    def extend_paged_requests(self, request_ids: tuple[int, ...]) -> None:
        """Reserves the KV position of the next decode input of every request, then activates the batch."""
        mgr = self.req_tokens_manager
        batch = self._device_batch
        if batch is not None and batch.request_ids == tuple(int(r) for r in request_ids):
            batch.host_advance()
            self.atten_info.max_actual_seq_len = batch.max_actual_seq_len
            return
        self._device_batch = None
        self.atten_info.device_decode = None
        for req_idx in request_ids:
            if not mgr.extend_req(req_idx, 1):
                raise RuntimeError(
                    "Paged KV allocation failed for request "
                    f"{req_idx}: current_tokens={mgr.req_token_count.get(req_idx, 'unknown')}, "
                    f"max_seq_len={mgr.max_seq_len}, free_pages={mgr.page_mgr.num_free_pages}")
        self.activate_paged_decode_batch(tuple(request_ids))

    def prefill_alloc_kv_cache(self, max_prompt_len: int, actual_prompt_lens, b_req_idx,
                               image_batch_size=None, debug_mode: bool = False):
        """Static-batch prefill (:411-494, the entry ``generate_stream.py:155-174`` calls before
        ``decode_alloc_kv_cache``): prompts padded to ``max_prompt_len`` rows each. Request
        ``b_req_idx[i]`` gets pages for ``max_prompt_len`` tokens and the logical length
        ``actual_prompt_lens[i]``; ``cur_select_index`` lists the slots of all ``max_prompt_len`` rows
        of every request (the padding rows are stored too, as the reference does), ``b_start_loc`` is
        ``i * max_prompt_len``. The first decode step then writes its token at position
        ``actual_prompt_lens[i]``, over the first padding row, and attends ``actual + 1`` tokens,
        which is what the reference's own worked example shows (:419-429: select index
        ``start + len``). Its paged branch instead counts ``max_prompt_len`` tokens per request
        (:450-455), so that a shorter prompt's first decode step appends behind the padding and
        attends a padding row; that is not reproduced. Returns ``(cur_select_index, None)``."""
        if image_batch_size is not None:
            raise RuntimeError("image prompts are outside the paged attention path")
        self._reset_paged_chunk_prefill_metadata()
        max_prompt_len = int(max_prompt_len)
        ids = tuple(int(r) for r in (b_req_idx.detach().cpu().tolist() if torch.is_tensor(b_req_idx) else b_req_idx))
        lens = [int(n) for n in (actual_prompt_lens.detach().cpu().reshape(-1).tolist()
                                 if torch.is_tensor(actual_prompt_lens) else actual_prompt_lens)]
        if len(lens) != len(ids) or not ids:
            raise ValueError("actual_prompt_lens and b_req_idx must name the same, non-empty batch")
        if any(n < 1 or n > max_prompt_len for n in lens):
            raise ValueError("prompt lengths must lie in [1, max_prompt_len]")
        mgr = self.req_tokens_manager
        made: list[int] = []
        for req_idx, n in zip(ids, lens):
            if not mgr.alloc_req(req_idx, n, max_prompt_len):
                for done in made:
                    mgr.free_req(done)
                raise RuntimeError("Paged KV allocation failed during prefill")
            made.append(req_idx)
        padded = [max_prompt_len] * len(ids)
        self._set_batch(ids, padded, padded, [mgr.slots(r, 0, max_prompt_len) for r in ids])
        info = self.atten_info
        info.b_seq_len = self._i64(lens)          # the prompts' own lengths, as the reference keeps them
        info.max_actual_seq_len = max_prompt_len
        if debug_mode:
            print(f"context_num_tokens: {max_prompt_len * len(ids)}, max_prompt_len: {max_prompt_len},\n"
                  f" cur_select_index: {info.cur_select_index},\n b_seq_len: {info.b_seq_len},\n"
                  f" b_start_loc: {info.b_start_loc}")
        return info.cur_select_index, None

    def decode_alloc_kv_cache(self, batch_size: int) -> torch.Tensor:
        """Static-batch decode step over the request ids cached at prefill time."""
        if len(self._paged_request_ids) != batch_size:
            raise RuntimeError("Paged request id cache is not initialized for the "
                               f"decode batch: cached={len(self._paged_request_ids)}, batch_size={batch_size}")
        for req_idx in self._paged_request_ids:
            if not self.req_tokens_manager.extend_req(req_idx, 1):
                raise RuntimeError("Paged KV allocation failed during decode")
        self.activate_paged_decode_batch(self._paged_request_ids)
        return self.atten_info.cur_select_index

    def release_paged_request_ids(self, request_ids: tuple[int, ...]) -> None:
        batch = self._device_batch
        if batch is not None and any(int(r) in batch.request_ids for r in request_ids):
            self._device_batch = None            # its tensors describe a request that is gone
            self.atten_info.device_decode = None
        for req_idx in request_ids:
            self.req_tokens_manager.free_req(req_idx)
        if tuple(request_ids) == self._paged_request_ids:
            self._paged_request_ids = ()

    def release_paged_requests(self) -> None:
        self.release_paged_request_ids(self._paged_request_ids)

    # ---- the step itself -------------------------------------------------------------------
    def attach_model(self, model, model_type: str = "unknown", use_graph: bool = True,
                     moe_parallel_mode: str = "tp") -> None:
        """``model.forward(input_ids, position_ids, atten_info)`` is what ``forward`` runs; decode
        steps go through a graph runner when the model family allows it (:306-314, :380-386)."""
        from .decode_graph import DecodeGraphRunner, supports_decode_graph

        self.model = model
        self.graph_runner = None
        if use_graph and supports_decode_graph(model_type, moe_parallel_mode):
            self.graph_runner = DecodeGraphRunner(model, model_type,
                                                  max_blocks=self.req_tokens_manager.max_pages_per_req)

    def forward(self, input_ids, position_ids=None, **kwargs):
        """One model step on the active batch (:977-987). Decode steps (one token per sequence)
        take the graph runner; with a device decode batch ``position_ids`` may be None (the batch
        computes them) and the device half of the step's metadata is enqueued here."""
        if self.model is None:
            raise RuntimeError("no model attached (attach_model)")
        batch = self._device_batch
        is_decode = input_ids.dim() == 2 and input_ids.shape[1] == 1
        if batch is not None and not is_decode:
            raise ValueError("a device decode batch is active: forward takes one token per sequence")
        if self.graph_runner is not None and is_decode and not kwargs:
            return self.graph_runner(input_ids, position_ids, self.atten_info)
        if batch is not None:
            batch.enqueue_advance()
            position_ids = batch.position_ids
        return self.model.forward(input_ids, position_ids, self.atten_info, **kwargs)

    # ---- page moves ------------------------------------------------------------------------
    def copy_on_write(self, request_ids: Sequence[int]):
        """Private copies of shared last pages before a step appends into them."""
        return self.req_tokens_manager.copy_on_write(request_ids)

    def compact_kv_pool(self):
        """Moves live pages into the dense prefix of the pool (all layers), fixing every table and
        every prefix-cache entry that names a moved page."""
        holders = [entry[0] for entry in self._paged_prefix_cache.values()]
        holders += [entry[0] for entry in self._paged_block_prefix_cache.values()]
        return self.req_tokens_manager.compact(holders)
