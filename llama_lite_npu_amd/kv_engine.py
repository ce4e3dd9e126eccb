"""Host-side scheduling metadata of the KV cache (no tensors, no device).

Same public names and behaviour as the reference's ``lite_llama/kv_engine.py``
(dataclasses :14-62, MixedLengthPrefillPacker :65-89, KVBlockRefCounter
:92-147, PrefixCache :150-194, ChunkedPrefillPlanner :197-215) so schedulers
written against it keep working; the implementations are this package's own
(free blocks live in a heap instead of being rescanned, the prefix cache walks
block by block, plans are built with running offsets).
"""

from __future__ import annotations

import heapq
from dataclasses import dataclass
from typing import Iterable, Sequence


def _checked(name: str, value, low: int = 1) -> int:
    """`value` as int; ValueError("<name> must be positive" / "... non-negative") below `low`."""
    number = int(value)
    if number < low:
        raise ValueError(f"{name} must be {'positive' if low == 1 else 'non-negative'}")
    return number


@dataclass(frozen=True)
class PrefixCacheMatch:
    """Longest cached block-aligned prefix: token count and the logical blocks holding it."""

    matched_tokens: int
    block_ids: tuple[int, ...]


@dataclass(frozen=True)
class PrefillChunk:
    """Half-open token range [start, end) of one prefill chunk."""

    start: int
    end: int

    @property
    def length(self) -> int:
        return self.end - self.start


@dataclass(frozen=True)
class PackedPrefillRequest:
    """Where one request's tokens sit in a packed (no padding) prefill batch."""

    request_index: int
    start: int
    length: int

    @property
    def end(self) -> int:
        return self.start + self.length


@dataclass(frozen=True)
class PackedPrefillPlan:
    """Flattened tokens, per-token positions and per-request rows of a packed prefill."""

    flat_token_ids: tuple[int, ...]
    flat_position_ids: tuple[int, ...]
    requests: tuple[PackedPrefillRequest, ...]

    @property
    def total_tokens(self) -> int:
        return len(self.flat_token_ids)

    @property
    def batch_size(self) -> int:
        return len(self.requests)


class MixedLengthPrefillPacker:
    """Concatenates prompts of different lengths; positions restart at 0 for every request."""

    def pack(self, prompt_token_ids: Sequence[Sequence[int]]) -> PackedPrefillPlan:
        tokens: list[int] = []
        positions: list[int] = []
        rows: list[PackedPrefillRequest] = []
        for index, prompt in enumerate(prompt_token_ids):
            row = PackedPrefillRequest(request_index=index, start=len(tokens), length=len(prompt))
            rows.append(row)
            tokens += [int(t) for t in prompt]
            positions += list(range(row.length))
        return PackedPrefillPlan(tuple(tokens), tuple(positions), tuple(rows))


class KVBlockRefCounter:
    """Reference counts of logical KV blocks; free blocks are handed out lowest id first."""

    def __init__(self, total_blocks: int) -> None:
        total_blocks = _checked("total_blocks", total_blocks)
        self._counts = [0] * total_blocks
        self._free = list(range(total_blocks))  # already a valid min-heap

    @property
    def total_blocks(self) -> int:
        return len(self._counts)

    @property
    def available_count(self) -> int:
        return len(self._free)

    def refcount(self, block_id: int) -> int:
        return self._counts[self._index(block_id)]

    def acquire(self, count: int) -> tuple[int, ...]:
        count = _checked("count", count)
        if count > len(self._free):
            raise RuntimeError(f"insufficient KV blocks: need {count}, available {len(self._free)}")
        taken = tuple(heapq.heappop(self._free) for _ in range(count))
        for block in taken:
            self._counts[block] = 1
        return taken

    def add_ref(self, block_ids: Iterable[int]) -> None:
        for block_id in block_ids:
            i = self._index(block_id)
            if self._counts[i] == 0:
                raise ValueError(f"cannot add ref to free KV block {i}")
            self._counts[i] += 1

    def release(self, block_ids: Iterable[int]) -> None:
        for block_id in block_ids:
            i = self._index(block_id)
            if self._counts[i] == 0:
                raise ValueError(f"KV block {i} refcount would become negative")
            self._counts[i] -= 1
            if self._counts[i] == 0:
                heapq.heappush(self._free, i)

    def _index(self, block_id: int) -> int:
        i = int(block_id)
        if not 0 <= i < len(self._counts):
            raise IndexError(f"KV block id out of range: {i}")
        return i


class PrefixCache:
    """Block-aligned prefix lookup: full token blocks map to logical block ids; a match ends at the
    first block that is not cached and never covers a partial block."""

    def __init__(self, block_size: int) -> None:
        block_size = _checked("block_size", block_size)
        self.block_size = block_size
        self._blocks: dict[tuple[int, ...], int] = {}

    def _full_blocks(self, token_ids: Sequence[int]):
        size = self.block_size
        for first in range(0, len(token_ids) - size + 1, size):
            yield tuple(int(t) for t in token_ids[first:first + size])

    def put(self, token_ids: Sequence[int], block_ids: Sequence[int]) -> None:
        keys = list(self._full_blocks(token_ids))
        if not keys:
            return
        if len(block_ids) < len(keys):
            raise ValueError("not enough block ids for full token blocks")
        for key, block_id in zip(keys, block_ids):
            self._blocks[key] = int(block_id)

    def match(self, token_ids: Sequence[int]) -> PrefixCacheMatch:
        found: list[int] = []
        for key in self._full_blocks(token_ids):
            block_id = self._blocks.get(key)
            if block_id is None:
                break
            found.append(block_id)
        return PrefixCacheMatch(matched_tokens=len(found) * self.block_size, block_ids=tuple(found))


class ChunkedPrefillPlanner:
    """Cuts a prompt into consecutive chunks of at most ``chunk_size`` tokens."""

    def __init__(self, chunk_size: int) -> None:
        chunk_size = _checked("chunk_size", chunk_size)
        self.chunk_size = chunk_size

    def plan(self, prompt_length: int) -> tuple[PrefillChunk, ...]:
        prompt_length = _checked("prompt_length", prompt_length, low=0)
        starts = range(0, prompt_length, self.chunk_size)
        return tuple(PrefillChunk(s, min(s + self.chunk_size, prompt_length)) for s in starts)
