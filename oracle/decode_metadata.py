"""TEST INFRASTRUCTURE ONLY -- CPU restatement (numpy, integer arithmetic) of the per-step metadata
of a decode batch on the reference's paged path. Nothing under llama_lite_npu_amd/ may import this.

Reference lines followed:
  token_slots     lite_llama/executor/paged_attention.py:116-146 (`build_token_table`): logical token
                  t of a request lives at slot  pages[t // page_size] * page_size + t % page_size
  decode_advance  lite_llama/executor/paged_attention.py:320-359 (`extend_req`: the logical length grows by
                  one, failing beyond max_seq_len / the pages at hand) followed by :287-318
                  (`batch_metadata`: request ids, lengths, slot of each request's last token) and the
                  position ids of a decode step (length - 1). The block-table rows in batch order
                  are what the reference's kernels reach through b_req_idx
                  (lite_llama/kernels/flashdecoding.py:84-94).

Pinned in tests/test_oracle.py by: the worked example in the reference's docstring (page_size 4,
10 tokens, pages [3, 7, 12] -> slots [12, 13, 14, 15, 28, 29, 30, 31, 48, 49], paged_attention.py:125-129);
brute force over every token of random page lists against an explicit per-token table; the
invariant that N single steps from length L give the slots token_slots lists at L .. L+N-1; and
the refusal cases (capacity reached, request id out of range): such a row ends empty (length -1,
slot -1) and stays refused, so nothing is appended over a cached token (the reference raises on
the host at this point, paged_attention.py:333-337, before anything is written).
"""

from __future__ import annotations

from typing import Optional

import numpy as np


def token_slots(pages, num_tokens: int, page_size: int) -> np.ndarray:
    """Slots of logical tokens 0 .. num_tokens-1 of one request."""
    pages = np.asarray(pages, dtype=np.int64)
    t = np.arange(int(num_tokens), dtype=np.int64)
    return pages[t // page_size] * page_size + t % page_size


def decode_advance(request_tables: np.ndarray, request_ids: np.ndarray, seq_lens: np.ndarray,
                   capacity: Optional[np.ndarray], width: int, page_size: int, num_pages: int,
                   increment: int = 1):
    """One step for a batch. request_tables [max_requests, >= width] page lists, request_ids [B],
    seq_lens [B] lengths before the step. Returns (new seq_lens int32, slot of the last token
    int32 (-1: none), position ids int64, block-table rows [B, width] int32, overflow flag)."""
    request_tables = np.asarray(request_tables)
    b = len(request_ids)
    new_lens = np.zeros(b, dtype=np.int32)
    slots = np.full(b, -1, dtype=np.int32)
    positions = np.zeros(b, dtype=np.int64)
    rows = np.zeros((b, width), dtype=np.int32)
    overflow = 0
    room = width * page_size
    for i in range(b):
        r = int(request_ids[i])
        known = 0 <= r < request_tables.shape[0]
        if known:
            rows[i] = request_tables[r, :width]
        length = int(seq_lens[i])
        cap = room if capacity is None else min(int(capacity[i]), room)
        ok = known and length >= 0 and length + increment <= cap
        if ok:
            nxt = length + increment
        else:
            # a refused row becomes empty for good (length -1, no slot): the step's append writes at
            # position length - 1, so a row that kept its length would lose its last cached token
            overflow = 1
            nxt = -1
        new_lens[i] = nxt
        if ok and nxt >= 1:
            page = int(request_tables[r, (nxt - 1) // page_size])
            if 0 <= page < num_pages:
                slots[i] = page * page_size + (nxt - 1) % page_size
        positions[i] = max(nxt - 1, 0)
    return new_lens, slots, positions, rows, overflow
