"""Page pool and per-request page tables of the paged KV cache (host logic + device tables).

Public surface of the reference's ``lite_llama/executor/paged_attention.py``
(PagedKVCacheManager :19-147, PagedReqTokensManager :153-384) with the same
method names, arguments, return values and failure modes, so the executor and
scheduler code written against it keeps working. What differs is underneath:

* the kernels consume a per-page **block table** ``[max_requests, max_pages]
  int32`` kept on the device and patched incrementally; the reference's
  per-token ``b_req_tokens_table`` (16x larger) is only materialised when a
  caller asks for it (slot = page * page_size + offset, reference :141-146);
* free pages live in a min-heap, so "lowest free ids first" (reference :79)
  costs O(log n) instead of a scan of the whole pool;
* all bookkeeping reads host arrays only; nothing here reads a device tensor
  back, so no call synchronises the stream;
* page moves exist: copy-on-write of shared pages and in-place compaction,
  both carried out by the page-copy kernel for every layer.
"""

from __future__ import annotations

import heapq
from typing import Iterable, List, Optional, Sequence, Tuple

import numpy as np
import torch


def _as_page_array(page_indices) -> np.ndarray:
    if isinstance(page_indices, torch.Tensor):
        return page_indices.detach().to("cpu", torch.long).numpy().reshape(-1)
    return np.asarray(list(page_indices), dtype=np.int64).reshape(-1)


class PagedKVCacheManager:
    """Fixed pool of ``num_pages`` KV pages of ``page_size`` tokens, reference counted.

    ``gpu_kv_buffer[l]`` is layer l's pool ``[num_pages * page_size, 2 * num_kv_heads,
    head_dim]``: K heads first, then V heads (reference :54-62). With ``dtype``
    ``torch.float8_e4m3fn`` (or ``torch.uint8``) the pools hold E4M3 codes and
    ``kv_scales[l]`` (float32 ``[2 * num_kv_heads]``, K heads then V heads, 1.0 until
    ``set_kv_scales``) the per-head scales; for fp16 pools ``kv_scales[l]`` is None.
    """

    def __init__(self, num_layers: int, num_kv_heads: int, head_dim: int, num_pages: int,
                 page_size: int = 16, dtype: torch.dtype = torch.float16, device: str = "cuda:0"):
        self.num_layers = int(num_layers)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.num_pages = int(num_pages)
        self.page_size = int(page_size)
        self.dtype = dtype
        self.device = device
        self.max_tokens = self.num_pages * self.page_size
        self.max_num_tokens = self.max_tokens
        self.gpu_kv_buffer = [
            torch.empty((self.max_tokens, 2 * self.num_kv_heads, self.head_dim), dtype=dtype, device=device)
            for _ in range(self.num_layers)
        ]
        # pools of 8-bit codes (fp8 E4M3 or int8) carry one scale per head
        self.is_fp8 = dtype in (torch.uint8, torch.float8_e4m3fn, torch.int8)
        self.kv_scales = [
            torch.ones(2 * self.num_kv_heads, dtype=torch.float32, device=device) if self.is_fp8 else None
            for _ in range(self.num_layers)
        ]
        self._refcount = np.zeros(self.num_pages, dtype=np.int32)
        self._free_mask = np.ones(self.num_pages, dtype=np.bool_)
        # host views with the reference's attribute names (shared memory with the arrays above)
        self.page_refcount = torch.from_numpy(self._refcount)
        self.page_free = torch.from_numpy(self._free_mask)
        self._heap = list(range(self.num_pages))
        self.num_free_pages = self.num_pages

    def set_kv_scales(self, layer: int, k_scales, v_scales) -> None:
        """Per-head scales of an fp8 or int8 layer (value = code * scale); set them before anything is cached."""
        if not self.is_fp8:
            raise ValueError("fp16 pools have no scales")
        both = torch.cat([torch.as_tensor(k_scales, dtype=torch.float32).reshape(-1),
                          torch.as_tensor(v_scales, dtype=torch.float32).reshape(-1)])
        if both.numel() != 2 * self.num_kv_heads or not bool((both > 0).all()):
            raise ValueError("need one positive scale per K head and per V head")
        self.kv_scales[layer].copy_(both)

    # ---- allocation ------------------------------------------------------------------------
    def pages_for(self, num_tokens: int) -> int:
        return (int(num_tokens) + self.page_size - 1) // self.page_size

    def alloc(self, num_tokens: int) -> Optional[torch.Tensor]:
        """Pages for ``num_tokens`` tokens, lowest free ids first; None if the pool cannot serve it."""
        need = self.pages_for(num_tokens)
        if need > self.num_free_pages:
            return None
        ids = np.fromiter((heapq.heappop(self._heap) for _ in range(need)), dtype=np.int64, count=need)
        self._free_mask[ids] = False
        self._refcount[ids] = 1
        self.num_free_pages -= need
        return torch.from_numpy(ids)

    def add_ref(self, page_indices) -> None:
        ids = _as_page_array(page_indices)
        if ids.size == 0:
            return
        if np.any(self._refcount[ids] <= 0):
            raise ValueError("cannot add ref to a free KV page")
        np.add.at(self._refcount, ids, 1)

    def free(self, page_indices) -> None:
        """Drops one reference per listed page; pages reaching zero return to the pool."""
        ids = _as_page_array(page_indices)
        if ids.size == 0:
            return
        if np.any(self._refcount[ids] <= 0):
            raise ValueError("KV page refcount would become negative")
        np.subtract.at(self._refcount, ids, 1)
        released = np.unique(ids[self._refcount[ids] == 0])
        released = released[~self._free_mask[released]]
        for page in released.tolist():
            heapq.heappush(self._heap, page)
        self._free_mask[released] = True
        self.num_free_pages += int(released.size)

    def free_all(self) -> None:
        self._refcount[:] = 0
        self._free_mask[:] = True
        self._heap = list(range(self.num_pages))
        self.num_free_pages = self.num_pages

    def refcount(self, page: int) -> int:
        return int(self._refcount[int(page)])

    # ---- tables ----------------------------------------------------------------------------
    def slots_of(self, page_indices, num_tokens: int) -> np.ndarray:
        """Physical slots of logical tokens 0..num_tokens-1: page * page_size + offset."""
        pages = _as_page_array(page_indices)
        t = np.arange(min(int(num_tokens), pages.size * self.page_size), dtype=np.int64)
        return pages[t // self.page_size] * self.page_size + t % self.page_size

    def build_token_table(self, page_indices, num_tokens: int, token_table: torch.Tensor, req_idx: int) -> int:
        """Writes the slots of a request into row ``req_idx`` of a per-token table; returns how many
        tokens were mapped (page_size 4, 10 tokens, pages [3, 7, 12] ->
        [12, 13, 14, 15, 28, 29, 30, 31, 48, 49], reference :125-129)."""
        slots = self.slots_of(page_indices, num_tokens)
        if slots.size:
            token_table[req_idx, :slots.size] = torch.from_numpy(slots).to(token_table.device, token_table.dtype)
        return int(slots.size)

    # ---- page moves ------------------------------------------------------------------------
    def copy_pages(self, src_ids: Sequence[int], dst_ids: Sequence[int]) -> None:
        """pool[dst] = pool[src] in every layer (device copy, bit exact, enqueued on the stream)."""
        from .. import ops

        src = torch.as_tensor(np.asarray(src_ids, dtype=np.int32), device=self.device)
        dst = torch.as_tensor(np.asarray(dst_ids, dtype=np.int32), device=self.device)
        if src.numel() == 0:
            return
        for pool in self.gpu_kv_buffer:
            ops.page_copy(pool, src, dst, self.page_size)


class PagedReqTokensManager:
    """Request slots and their page lists; builds the per-step metadata of a batch."""

    def __init__(self, max_requests: int, max_seq_len: int, page_manager: PagedKVCacheManager,
                 device: str = "cuda:0"):
        self.max_requests = int(max_requests)
        self.max_seq_len = int(max_seq_len)
        self.page_mgr = page_manager
        self.device = device
        self.max_pages_per_req = page_manager.pages_for(self.max_seq_len)
        self._table_host = np.zeros((self.max_requests, self.max_pages_per_req), dtype=np.int32)
        self.block_table = torch.zeros((self.max_requests, self.max_pages_per_req), dtype=torch.int32,
                                       device=device)
        self.req_page_table: dict[int, torch.Tensor] = {}
        self.req_page_count: dict[int, int] = {}      # len(req_page_table[r]) without touching the tensor
        self.req_token_count: dict[int, int] = {}
        self.req_active = torch.zeros(self.max_requests, dtype=torch.bool, device="cpu")
        self.free_req_indices = list(range(self.max_requests))
        self.table_epoch = 0    # grows whenever a request's page list changes or a request is freed

    # ---- device tables ---------------------------------------------------------------------
    def _publish_pages(self, req_idx: int, first: int = 0) -> None:
        """Copies page-list entries [first, len) of a request to the host mirror and the device table."""
        pages = self.req_page_table[req_idx].numpy().astype(np.int32)
        if first >= pages.size:
            return
        self.table_epoch += 1
        self._table_host[req_idx, first:pages.size] = pages[first:]
        self.block_table[req_idx, first:pages.size] = torch.from_numpy(pages[first:]).to(self.device)

    @property
    def b_req_tokens_table(self) -> torch.Tensor:
        """Per-token slot table ``[max_requests, max_seq_len] int32`` derived from the block table
        (the layout the reference's kernels take, reference :166-170). Built on demand."""
        ps = self.page_mgr.page_size
        offs = torch.arange(ps, dtype=torch.int32, device=self.block_table.device)
        slots = self.block_table.unsqueeze(-1) * ps + offs
        return slots.view(self.max_requests, -1)[:, :self.max_seq_len].contiguous()

    def block_table_rows(self, req_indices: Sequence[int]) -> torch.Tensor:
        """Block-table rows of a batch, in batch order, trimmed to the longest page list."""
        width = max(1, max(self.req_page_count[r] for r in req_indices))
        rows = np.ascontiguousarray(self._table_host[list(req_indices), :width])
        return torch.from_numpy(rows).to(self.device)

    # ---- request lifecycle -----------------------------------------------------------------
    def alloc_req(self, req_idx: int, num_tokens: int, reserved_tokens: int | None = None) -> bool:
        """Binds pages to an explicit request id. ``num_tokens`` is the logical length visible to
        attention; ``reserved_tokens`` (>= num_tokens) the capacity to reserve up front."""
        if req_idx not in self.free_req_indices:
            return False
        num_tokens = int(num_tokens)
        capacity = num_tokens if reserved_tokens is None else int(reserved_tokens)
        if num_tokens < 1 or capacity < num_tokens or capacity > self.max_seq_len:
            return False
        pages = self.page_mgr.alloc(capacity)
        if pages is None:
            return False
        self._bind(req_idx, pages, num_tokens)
        return True

    def _bind(self, req_idx: int, pages: torch.Tensor, num_tokens: int) -> None:
        self.free_req_indices.remove(req_idx)
        self.req_page_table[req_idx] = pages
        self.req_page_count[req_idx] = len(pages)
        self.req_token_count[req_idx] = num_tokens
        self.req_active[req_idx] = True
        self._publish_pages(req_idx)

    def reserve_req(self, num_tokens: int, reserved_tokens: int | None = None) -> Optional[int]:
        """Lowest free request id with freshly allocated pages, or None."""
        if not self.free_req_indices:
            return None
        req_idx = self.free_req_indices[0]
        return req_idx if self.alloc_req(req_idx, num_tokens, reserved_tokens) else None

    def ensure_req_capacity(self, req_idx: int, total_tokens: int) -> bool:
        """Grows the page list so ``total_tokens`` fit; the logical length is unchanged."""
        if req_idx not in self.req_page_table:
            return False
        total_tokens = int(total_tokens)
        if total_tokens < self.req_token_count[req_idx]:
            return True
        if total_tokens > self.max_seq_len:
            return False
        return self._grow(req_idx, self.page_mgr.pages_for(total_tokens))

    def _grow(self, req_idx: int, pages_needed: int) -> bool:
        have = self.req_page_count[req_idx]
        if pages_needed <= have:
            return True
        extra = self.page_mgr.alloc((pages_needed - have) * self.page_mgr.page_size)
        if extra is None:
            return False
        self.req_page_table[req_idx] = torch.cat([self.req_page_table[req_idx], extra])
        self.req_page_count[req_idx] = pages_needed
        self._publish_pages(req_idx, have)
        return True

    def share_req_from_pages(self, req_idx: int, page_indices, num_tokens: int) -> bool:
        """Maps a request onto existing pages (one more reference each)."""
        if req_idx not in self.free_req_indices:
            return False
        num_tokens = int(num_tokens)
        if num_tokens < 1 or num_tokens > self.max_seq_len:
            return False
        need = self.page_mgr.pages_for(num_tokens)
        ids = _as_page_array(page_indices)
        if ids.size < need:
            return False
        pages = torch.from_numpy(ids[:need].copy())
        self.page_mgr.add_ref(pages)
        self._bind(req_idx, pages, num_tokens)
        return True

    def reserve_shared_req(self, page_indices, num_tokens: int) -> Optional[int]:
        if not self.free_req_indices:
            return None
        req_idx = self.free_req_indices[0]
        return req_idx if self.share_req_from_pages(req_idx, page_indices, num_tokens) else None

    def extend_req(self, req_idx: int, num_new_tokens: int) -> bool:
        """Advances the logical length, allocating pages only when the reserved ones run out."""
        if num_new_tokens <= 0:
            return True
        new_total = self.req_token_count[req_idx] + int(num_new_tokens)
        if new_total > self.max_seq_len:
            return False
        ps = self.page_mgr.page_size
        if new_total > self.req_page_count[req_idx] * ps and not self._grow(req_idx, (new_total + ps - 1) // ps):
            return False
        self.req_token_count[req_idx] = new_total
        return True

    def free_req(self, req_idx: int) -> None:
        if req_idx in self.req_page_table:
            self.table_epoch += 1
            self.page_mgr.free(self.req_page_table.pop(req_idx))
            del self.req_token_count[req_idx]
            del self.req_page_count[req_idx]
        self.req_active[req_idx] = False
        if req_idx not in self.free_req_indices:
            self.free_req_indices.append(req_idx)
            self.free_req_indices.sort()

    def request_pages(self, req_idx: int) -> Tuple[int, ...]:
        if req_idx not in self.req_page_table:
            raise KeyError(f"request {req_idx} is not allocated")
        return tuple(int(p) for p in self.req_page_table[req_idx].tolist())

    # ---- per-step metadata -----------------------------------------------------------------
    def slots(self, req_idx: int, first: int = 0, last: Optional[int] = None) -> np.ndarray:
        """Host array of the physical slots of logical tokens [first, last) of a request."""
        last = self.req_token_count[req_idx] if last is None else int(last)
        return self.page_mgr.slots_of(self.req_page_table[req_idx], last)[first:]

    def get_token_indices(self, req_idx: int, num_tokens: Optional[int] = None) -> torch.Tensor:
        """Physical slots of a request's first ``num_tokens`` tokens (int32, on the device)."""
        return torch.from_numpy(self.slots(req_idx, 0, num_tokens).astype(np.int32)).to(self.device)

    def batch_metadata(self, req_indices: List[int]) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """(request ids int32, lengths int64, slot of each request's last token int32), on the device.
        Computed from host page lists only: no device tensor is read."""
        if not req_indices:
            raise ValueError("req_indices must not be empty")
        for req_idx in req_indices:
            if req_idx not in self.req_token_count:
                raise KeyError(f"request {req_idx} is not allocated")
        ps = self.page_mgr.page_size
        lens = [self.req_token_count[r] for r in req_indices]
        table = self._table_host
        last = [int(table[r, (n - 1) // ps]) * ps + (n - 1) % ps for r, n in zip(req_indices, lens)]
        return (torch.tensor(req_indices, dtype=torch.int32, device=self.device),
                torch.tensor(lens, dtype=torch.long, device=self.device),
                torch.tensor(last, dtype=torch.int32, device=self.device))

    # ---- page moves ------------------------------------------------------------------------
    def copy_on_write(self, req_indices: Iterable[int]) -> list[tuple[int, int]]:
        """Gives every listed request a private copy of the partly filled page its next token goes
        into if that page is shared (refcount > 1, counting the holders this call has not already
        moved away): a fresh page is allocated, the bytes are copied in every layer, the table
        entry is swapped and the old reference dropped. Returns the (src, dst) moves made.
        Needed before appending into a page another holder can still read; the reference shares
        such pages without copying (model_executor.py:672-678)."""
        moves: list[tuple[int, int]] = []
        touched: list[tuple[int, int]] = []
        dropping: dict[int, int] = {}      # references this call has already decided to drop, per page
        ps = self.page_mgr.page_size
        for req_idx in req_indices:
            pages = self.req_page_table[req_idx]
            count = self.req_token_count[req_idx]
            if count % ps == 0:
                continue                   # the next token opens a page of its own: nothing to protect
            last = (count - 1) // ps       # the page the next token goes into (reserved pages may follow it)
            old = int(pages[last])
            if self.page_mgr.refcount(old) - dropping.get(old, 0) <= 1:
                continue                   # the last holder left keeps the page
            dropping[old] = dropping.get(old, 0) + 1
            fresh = self.page_mgr.alloc(1)
            if fresh is None:
                raise RuntimeError("Paged KV allocation failed during copy-on-write")
            pages = pages.clone()
            pages[last] = fresh[0]
            self.req_page_table[req_idx] = pages
            moves.append((old, int(fresh[0])))
            touched.append((req_idx, last))
        if moves:
            self.page_mgr.copy_pages([m[0] for m in moves], [m[1] for m in moves])
            for (req_idx, last), (old, _) in zip(touched, moves):
                self._publish_pages(req_idx, last)
                self.page_mgr.free(torch.tensor([old]))
        return moves

    def compact(self, extra_holders: Sequence[torch.Tensor] = ()) -> list[tuple[int, int]]:
        """Moves live pages with id >= (number of live pages) into the free holes below, so the
        live set becomes the dense prefix of the pool; sources and destinations are disjoint.
        ``extra_holders`` are page-id tensors kept outside this manager (prefix-cache entries);
        they are rewritten in place. Returns the (src, dst) moves."""
        mgr = self.page_mgr
        live = np.flatnonzero(~mgr._free_mask)
        n_live = int(live.size)
        src = live[live >= n_live]
        holes = np.flatnonzero(mgr._free_mask[:n_live])
        assert src.size == holes.size
        if src.size == 0:
            return []
        mgr.copy_pages(src.tolist(), holes.tolist())
        remap = np.arange(mgr.num_pages, dtype=np.int64)
        remap[src] = holes
        mgr._refcount[holes] = mgr._refcount[src]
        mgr._refcount[src] = 0
        mgr._free_mask[holes] = False
        mgr._free_mask[src] = True
        mgr._heap = np.flatnonzero(mgr._free_mask).tolist()
        for req_idx, pages in self.req_page_table.items():
            new = torch.from_numpy(remap[pages.numpy()])
            if not torch.equal(new, pages):
                self.req_page_table[req_idx] = new
                self._publish_pages(req_idx)
        for holder in extra_holders:
            holder.copy_(torch.from_numpy(remap[holder.numpy()]))
        return list(zip(src.tolist(), holes.tolist()))
