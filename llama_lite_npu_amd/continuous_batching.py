"""The model side of continuous batching: what a scheduler calls to prefill, decode, release and
preempt requests on the paged KV cache.

Counterpart of ``ContinuousBatchModelBackend`` in the reference
(lite_llama/continuous_batching.py:614-1612) with the same constructor, methods, return values and
executor call order, so the reference's scheduler (:194-611, not rebuilt here: it is model-agnostic
control plane) can drive it unchanged. ``BatchRequest`` below carries exactly the fields of the
reference's request object (:77-173) that the backend reads and writes.

What is different underneath:

* every way a prompt can finish (one-shot, packed, first chunk, later chunk, token replay) ends in
  one routine, ``_complete``: sample, remember the token and position on the device, book the next
  token's slot, hand the host its token, store the prefix;
* an exact prefix-cache hit maps the cached pages into the new request and then gives it a private
  copy of the partly filled last page (``ModelExecutor.copy_on_write``) before anything appends
  into it; the reference lets both requests append into the shared page and relies on greedy
  decoding being deterministic (:908-928, model_executor.py:672-678);
* ``decode`` keeps a batch's metadata on the device while its set of requests is unchanged
  (``ModelExecutor.activate_device_decode_batch``): a step is then one graph replay plus host
  dictionary bookkeeping, and the sampled tokens feed the next step without being re-stacked.
  Executors without that call (the reference's) get the reference's per-step sequence (:1574-1595);
* positions are host integers (one upload per step) instead of one device scalar per request
  incremented by one kernel each (:1590-1591).
"""

from __future__ import annotations

import logging
from typing import Callable, Optional, Sequence

import torch

logger = logging.getLogger(__name__)


class KVCacheCapacityError(RuntimeError):
    """The live KV cache cannot admit or extend a request (reference :25-26)."""


class BatchRequest:
    """The request fields the backend uses (reference :77-121); streaming, text decoding and
    completion events belong to the scheduler and are not modelled."""

    def __init__(self, request_id: str, prompt_tokens: Sequence[int], max_new_tokens: int,
                 temperature: float, top_p: float, control_id: Optional[int] = None) -> None:
        if max_new_tokens < 1:
            raise ValueError("max_new_tokens must be positive")
        self.request_id = request_id
        self.control_id = control_id
        self.prompt_tokens = list(prompt_tokens)
        self.max_new_tokens = max_new_tokens
        self.temperature = temperature
        self.top_p = top_p
        self.generated_token_ids: list[int] = []
        self.preemptions = 0
        self.prefill_cursor = 0          # context tokens already in the KV cache
        self.model_request_id: Optional[int] = None
        self.finished = False
        self.cancelled = False

    @property
    def last_token_id(self) -> int:
        if not self.generated_token_ids:
            raise RuntimeError("request has no generated token")
        return self.generated_token_ids[-1]

    @property
    def model_context_tokens(self) -> list[int]:
        """Tokens whose K/V must be cached before the next token is sampled (a preempted request
        replays its prompt and what it had generated)."""
        return self.prompt_tokens + self.generated_token_ids

    def mark_preempted(self) -> None:
        self.preemptions += 1
        self.model_request_id = None


def sample_next_token(logits: torch.Tensor, temperature: Sequence[float], top_p: Sequence[float],
                      vocab_parallel: bool = False) -> torch.Tensor:
    """One token per row of ``logits`` [n, vocab] (or [n, seq, vocab]: last position). Rows with
    temperature 0 take the arg-max; the others sample from the smallest set of tokens whose
    probability mass reaches top_p, after temperature scaling. Same call as the reference's
    ``lite_llama.sampling.sample_next_token`` as the backend uses it (:654-664); sharded logits
    (tensor parallelism) are not supported on one GPU."""
    if vocab_parallel:
        raise NotImplementedError("vocabulary-parallel sampling needs several ranks")
    rows = logits[:, -1, :] if logits.dim() == 3 else logits
    rows = rows.float()
    greedy = rows.argmax(dim=-1)
    if all(float(t) == 0.0 for t in temperature):
        return greedy
    temp = torch.tensor([float(t) if float(t) > 0 else 1.0 for t in temperature], device=rows.device)
    probs = torch.softmax(rows / temp[:, None], dim=-1)
    ordered, order = probs.sort(dim=-1, descending=True)
    before = ordered.cumsum(dim=-1) - ordered                  # mass of the more likely tokens
    keep = before < torch.tensor([float(p) for p in top_p], device=rows.device)[:, None]
    keep[:, 0] = True
    ordered = torch.where(keep, ordered, torch.zeros_like(ordered))
    pick = torch.multinomial(ordered / ordered.sum(dim=-1, keepdim=True), 1)
    drawn = order.gather(1, pick).reshape(-1)
    is_greedy = torch.tensor([float(t) == 0.0 for t in temperature], device=rows.device)
    return torch.where(is_greedy, greedy, drawn)


class _TokenRows(dict):
    """request id -> its last sampled token as a 0-d device tensor. Entries are kept as (batch
    tensor, row) and sliced only when somebody asks, so remembering a step's samples costs no
    device work per request."""

    def remember(self, req_idx: int, sampled: torch.Tensor, row: int) -> None:
        dict.__setitem__(self, req_idx, (sampled, row))

    def __getitem__(self, req_idx: int) -> torch.Tensor:
        sampled, row = dict.__getitem__(self, req_idx)
        return sampled[row].reshape(())


class ContinuousBatchModelBackend:
    """Paged-KV model adapter between a continuous-batching scheduler and ``ModelExecutor``."""

    def __init__(self, generator, return_host_tokens: bool = True, enable_partial_prefix_cache: bool = False,
                 device_decode: bool = True, decode_reserve_tokens: int = 64,
                 sampler: Optional[Callable] = None) -> None:
        """``generator``: an object with ``model_executor`` and ``tokenizer``. ``return_host_tokens``
        False (a tensor-parallel worker in the reference) keeps sampled tokens on the device and
        returns no token lists. ``device_decode``: use device-side decode metadata when the executor
        offers it; ``decode_reserve_tokens`` pages are then reserved that many tokens ahead."""
        self.generator = generator
        self.executor = generator.model_executor
        self.tokenizer = generator.tokenizer
        self.return_host_tokens = bool(return_host_tokens)
        self.enable_partial_prefix_cache = bool(enable_partial_prefix_cache)
        self.device_decode = bool(device_decode) and hasattr(self.executor, "activate_device_decode_batch")
        self.decode_reserve_tokens = int(decode_reserve_tokens)
        self._sampler = sampler if sampler is not None else sample_next_token
        self._device_tokens = _TokenRows()                    # last sampled token of each request (0-d)
        self._positions: dict[int, int] = {}                  # position of that token
        self._step_ids: tuple[int, ...] = ()                  # requests of the last decode step ...
        self._step_tokens: Optional[torch.Tensor] = None      # ... and what it sampled, [B]
        self._announced_paths = False
        self._warned_replay = False
        if not self.executor.use_paged_attn:
            raise RuntimeError("continuous batching requires --page_size greater than zero")

    # ---- what the scheduler asks about ---------------------------------------------------------
    @property
    def eos_token_id(self) -> int:
        return int(self.tokenizer.eos_token_id)

    @property
    def max_context_tokens(self) -> Optional[int]:
        return int(getattr(self.executor, "max_seq_len", 0)) or None

    @property
    def max_prefill_tokens(self) -> Optional[int]:
        value = getattr(self.executor, "max_prefill_tokens", None)
        return None if value is None else int(value)

    def tokenize(self, prompt: str) -> list[int]:
        return self.tokenizer.encode(prompt, add_special_tokens=True)

    def decode_tokens(self, token_ids: Sequence[int]) -> str:
        return self.tokenizer.decode([int(t) for t in token_ids], skip_special_tokens=True)

    @property
    def _device_positions(self) -> dict[int, torch.Tensor]:
        """Positions as 0-d device tensors, the form the reference keeps them in (:666-683)."""
        return {req: torch.tensor(pos, dtype=torch.long, device=self.executor.device)
                for req, pos in self._positions.items()}

    # ---- shared pieces -------------------------------------------------------------------------
    def _tensor(self, values) -> torch.Tensor:
        return torch.tensor(values, dtype=torch.long, device=self.executor.device)

    def _sample(self, logits, requests: Sequence[BatchRequest]) -> torch.Tensor:
        return self._sampler(logits, temperature=[r.temperature for r in requests],
                             top_p=[r.top_p for r in requests],
                             vocab_parallel=bool(getattr(self.executor, "logits_are_sharded", False)))

    def _remember(self, requests: Sequence[BatchRequest], sampled: torch.Tensor,
                  positions: Optional[Sequence[int]] = None) -> None:
        for row, request in enumerate(requests):
            req_idx = int(request.model_request_id)
            self._device_tokens.remember(req_idx, sampled, row)
            if positions is not None:
                self._positions[req_idx] = int(positions[row])

    def _complete(self, requests: Sequence[BatchRequest], logits) -> list[Optional[int]]:
        """The prompts of ``requests`` are cached and ``logits`` holds one row per request for the
        last prompt token: sample the first generated token, book its slot, store the prefix."""
        sampled = self._sample(logits, requests)
        self._remember(requests, sampled, [len(r.model_context_tokens) for r in requests])
        ids = tuple(int(r.model_request_id) for r in requests)
        self.executor.extend_paged_requests(ids)
        if not self.return_host_tokens:
            return [None] * len(requests)
        tokens = [int(t) for t in sampled.detach().cpu().tolist()]
        if hasattr(self.executor, "store_paged_request_prefix"):
            for request, token in zip(requests, tokens):
                if request.temperature == 0:        # only greedy continuations are reusable
                    self.executor.store_paged_request_prefix(request.model_context_tokens,
                                                             int(request.model_request_id), token)
        return tokens

    def _adopt_cached(self, request: BatchRequest) -> Optional[tuple[int, Optional[int]]]:
        """Looks the request's context up in the prefix caches (greedy requests only). On a hit the
        request owns a model request mapped onto cached pages and ``prefill_cursor`` says how many
        tokens they cover. Returns (matched tokens, first token or None), or None on a miss."""
        if request.temperature != 0:
            return None
        context = request.model_context_tokens
        ex = self.executor
        if self.enable_partial_prefix_cache and hasattr(ex, "share_paged_prefix_from_cache"):
            hit = ex.share_paged_prefix_from_cache(context)
            if hit is not None:
                req_idx, matched, token = hit
                request.model_request_id, request.prefill_cursor = int(req_idx), int(matched)
                if token is not None:
                    self._own_last_page(int(req_idx))
                return int(matched), None if token is None else int(token)
        if hasattr(ex, "share_paged_request_from_cache"):
            hit = ex.share_paged_request_from_cache(context)
            if hit is not None:
                req_idx, token = hit
                request.model_request_id, request.prefill_cursor = int(req_idx), len(context)
                self._own_last_page(int(req_idx))
                return len(context), int(token)
        return None

    def _own_last_page(self, req_idx: int) -> None:
        """After an exact hit the slot of the first generated token lies in a page the cache entry
        (and possibly other requests) also hold: copy it before this request appends."""
        if hasattr(self.executor, "copy_on_write"):
            try:
                self.executor.copy_on_write((req_idx,))
            except RuntimeError as error:
                self.executor.release_paged_request_ids((req_idx,))
                raise KVCacheCapacityError(f"Paged KV capacity exhausted during copy-on-write: {error}") from error

    def _use_cached_token(self, request: BatchRequest, token: int) -> int:
        self._remember([request], self._tensor([token]), [len(request.model_context_tokens)])
        return token

    def _ensure_capacity(self, request: BatchRequest, target_tokens: int) -> None:
        if not hasattr(self.executor, "ensure_paged_request_capacity"):
            return
        req_idx = int(request.model_request_id)
        try:
            self.executor.ensure_paged_request_capacity(req_idx, int(target_tokens))
        except RuntimeError as error:
            limit = getattr(self.executor.req_tokens_manager, "max_seq_len", "unknown")
            raise KVCacheCapacityError(
                "chunked prefill KV capacity check failed: "
                f"request_id={request.request_id}, model_request_id={req_idx}, "
                f"target_tokens={int(target_tokens)}, max_seq_len={limit}, "
                f"prompt_tokens={len(request.prompt_tokens)}, "
                f"generated_tokens={len(request.generated_token_ids)}") from error

    @staticmethod
    def _context(request: BatchRequest) -> list[int]:
        context = request.model_context_tokens
        if not context:
            raise RuntimeError("empty prompts are not supported by chunked prefill")
        return context

    # ---- token-by-token replay (fallback; also the suffix after a block-prefix hit) ------------
    def _replay(self, requests: Sequence[BatchRequest], chunk_size: Optional[int]) -> list[Optional[int]]:
        """Feeds context tokens [prefill_cursor, prefill_cursor + chunk_size) of every request
        through decode steps, all requests that still have tokens left in one micro-batch per
        step (:966-1133). Requests without a model request get one with room for the whole context
        and the first generated token."""
        ex = self.executor
        results: list[Optional[int]] = [None] * len(requests)
        ends = []
        for request in requests:
            context = self._context(request)
            whole = len(context) + 1
            if request.model_request_id is None:
                (req_idx,) = ex.reserve_paged_requests((1,), reserved_lengths=(whole,))
                request.model_request_id, request.prefill_cursor = int(req_idx), 0
            else:
                self._ensure_capacity(request, whole)
            end = len(context) if chunk_size is None else min(len(context), request.prefill_cursor + int(chunk_size))
            self._ensure_capacity(request, end + 1)
            ends.append(end)
        counts = ex.req_tokens_manager.req_token_count
        while True:
            rows = [(i, r) for i, (r, end) in enumerate(zip(requests, ends)) if r.prefill_cursor < end]
            if not rows:
                return results
            ids = []
            for _, request in rows:
                req_idx = int(request.model_request_id)
                while counts[req_idx] <= request.prefill_cursor:
                    ex.extend_paged_requests((req_idx,))
                ids.append(req_idx)
            ex.activate_paged_decode_batch(tuple(ids))
            tokens = [[int(r.model_context_tokens[r.prefill_cursor])] for _, r in rows]
            positions = [[int(r.prefill_cursor)] for _, r in rows]
            logits = ex.forward(self._tensor(tokens), self._tensor(positions))
            done_rows, done = [], []
            for row, (index, request) in enumerate(rows):
                request.prefill_cursor += 1
                if request.prefill_cursor >= len(request.model_context_tokens):
                    done_rows.append(row)
                    done.append((index, request))
            if done:
                picked = logits[self._tensor(done_rows).to(logits.device), -1, :]
                for (index, _), token in zip(done, self._complete([r for _, r in done], picked)):
                    results[index] = token

    # ---- one-shot prefill ----------------------------------------------------------------------
    def _split_by_budget(self, items: Sequence[tuple[int, BatchRequest]]) -> list[list[tuple[int, BatchRequest]]]:
        """Consecutive groups whose context tokens stay within ``max_prefill_tokens`` (a group is
        closed as soon as it reaches the budget; :740-765)."""
        budget = self.max_prefill_tokens
        if budget is None or budget <= 0:
            return [list(items)]
        groups, current, used = [], [], 0
        for item in items:
            cost = len(item[1].model_context_tokens)
            if current and used + cost > budget:
                groups.append(current)
                current, used = [], 0
            current.append(item)
            used += cost
            if used >= budget:
                groups.append(current)
                current, used = [], 0
        if current:
            groups.append(current)
        return groups

    def _prefill_group(self, items: Sequence[tuple[int, BatchRequest]], results: list) -> None:
        """One forward for requests that already own model requests of their context length: packed
        when lengths differ (:822-871), one [B, L] batch per length otherwise (:873-906)."""
        ex = self.executor
        requests = [r for _, r in items]
        lengths = [len(r.model_context_tokens) for r in requests]
        if len(set(lengths)) > 1 and hasattr(ex, "activate_paged_packed_prefill_batch"):
            ids = tuple(int(r.model_request_id) for r in requests)
            positions, last_rows = ex.activate_paged_packed_prefill_batch(ids, lengths)
            flat = [int(t) for r in requests for t in r.model_context_tokens]
            logits = ex.forward(self._tensor([flat]), positions.reshape(1, -1))
            for (index, _), token in zip(items, self._complete(requests, logits[0, last_rows, :])):
                results[index] = token
            return
        for length in dict.fromkeys(lengths):
            same = [(i, r) for (i, r), n in zip(items, lengths) if n == length]
            group = [r for _, r in same]
            ex.activate_paged_prefill_batch(tuple(int(r.model_request_id) for r in group), length)
            input_ids = self._tensor([r.model_context_tokens for r in group])
            positions = torch.arange(length, dtype=torch.long, device=ex.device).unsqueeze(0).expand(len(group), -1)
            logits = ex.forward(input_ids, positions)
            for (index, _), token in zip(same, self._complete(group, logits[:, -1, :])):
                results[index] = token

    def prefill(self, requests: Sequence[BatchRequest]) -> Sequence[int]:
        """Caches the whole context of every request and returns each one's first generated token
        (:1428-1505): prefix-cache hits first, contexts longer than the prefill budget by token
        replay, the rest in as few forwards as the budget allows."""
        if not requests:
            return []
        ex = self.executor
        results: list[Optional[int]] = [None] * len(requests)
        misses: list[tuple[int, BatchRequest]] = []
        for index, request in enumerate(requests):
            hit = self._adopt_cached(request)
            if hit is None:
                misses.append((index, request))
                continue
            _, token = hit
            if token is not None:
                results[index] = self._use_cached_token(request, token)
                continue
            (results[index],) = self._replay([request], None)
            if results[index] is None and self.return_host_tokens:
                raise RuntimeError("partial prefix replay did not produce a token")
        budget = self.max_prefill_tokens
        direct = []
        for index, request in misses:
            if budget is not None and len(request.model_context_tokens) > budget:
                (results[index],) = self._replay([request], None)       # too long for one forward
            else:
                direct.append((index, request))
        if direct:
            ids = ex.reserve_paged_requests([len(r.model_context_tokens) for _, r in direct])
            for (_, request), req_idx in zip(direct, ids):
                request.model_request_id = req_idx
            try:
                for group in self._split_by_budget(direct):
                    self._prefill_group(group, results)
            except BaseException:
                ex.release_paged_request_ids(ids)
                for _, request in direct:
                    request.model_request_id = None
                raise
        return [int(t) for t in results] if self.return_host_tokens else []

    # ---- chunked prefill -----------------------------------------------------------------------
    def _first_chunks_packed(self, requests: Sequence[BatchRequest], chunk_size: int) -> Optional[list]:
        """First chunks of fresh requests in one packed forward (no history to attend to);
        pages for the whole context and the first generated token are reserved up front (:1272-1396).
        None if the executor cannot pack."""
        ex = self.executor
        if not requests:
            return []
        if not hasattr(ex, "activate_paged_packed_prefill_batch"):
            return None
        chunks = [min(len(self._context(r)), int(chunk_size)) for r in requests]
        ids = ex.reserve_paged_requests(chunks, reserved_lengths=[len(r.model_context_tokens) + 1 for r in requests])
        for request, req_idx in zip(requests, ids):
            request.model_request_id = int(req_idx)
        try:
            positions, _ = ex.activate_paged_packed_prefill_batch(tuple(int(i) for i in ids), chunks)
            flat = [int(t) for r, n in zip(requests, chunks) for t in r.model_context_tokens[:n]]
            logits = ex.forward(self._tensor([flat]), positions.reshape(1, -1))
        except BaseException:
            ex.release_paged_request_ids(ids)
            for request in requests:
                request.model_request_id, request.prefill_cursor = None, 0
            raise
        return self._after_chunks(requests, [0] * len(requests), chunks, logits)

    def _later_chunks_paged(self, requests: Sequence[BatchRequest], chunk_size: int) -> Optional[list]:
        """Next chunks of requests that already have history in the cache, in one forward whose
        attention reads history and chunk through the pages (:1135-1270). None if the executor
        has no such path or a request has no history yet."""
        ex = self.executor
        if not requests:
            return []
        if not hasattr(ex, "activate_paged_chunk_prefill_batch"):
            return None
        if any(r.model_request_id is None or r.prefill_cursor <= 0 for r in requests):
            return None
        where, live, starts, chunks = [], [], [], []
        for index, request in enumerate(requests):
            context = self._context(request)
            start = int(request.prefill_cursor)
            end = min(len(context), start + int(chunk_size))
            if end > start:
                self._ensure_capacity(request, end + 1)
                where.append(index)
                live.append(request)
                starts.append(start)
                chunks.append(end - start)
        results: list[Optional[int]] = [None] * len(requests)
        if not live:
            return results
        ids = tuple(int(r.model_request_id) for r in live)
        positions, _ = ex.activate_paged_chunk_prefill_batch(ids, tuple(starts), tuple(chunks))
        flat = [int(t) for r, s, n in zip(live, starts, chunks) for t in r.model_context_tokens[s:s + n]]
        logits = ex.forward(self._tensor([flat]), positions.reshape(1, -1))
        for index, token in zip(where, self._after_chunks(live, starts, chunks, logits)):
            results[index] = token
        return results

    def _after_chunks(self, requests, starts, chunks, logits) -> list[Optional[int]]:
        """Moves the cursors past the chunks just cached and completes the requests whose context
        is now whole; ``logits`` [1, total chunk tokens, vocab] in request order."""
        results: list[Optional[int]] = [None] * len(requests)
        done, rows, offset = [], [], 0
        for index, (request, start, n) in enumerate(zip(requests, starts, chunks)):
            request.prefill_cursor = int(start) + int(n)
            offset += int(n)
            if request.prefill_cursor >= len(request.model_context_tokens):
                done.append(index)
                rows.append(offset - 1)
        if done:
            picked = logits[0, self._tensor(rows).to(logits.device), :]
            for index, token in zip(done, self._complete([requests[i] for i in done], picked)):
                results[index] = token
        return results

    def prepare_prefill_chunk(self, requests: Sequence[BatchRequest], chunk_size: int) -> None:
        """Reserves the pages the next chunk needs, without computing (:1398-1426). Requests that
        have no model request yet are left alone: their reservation belongs to ``prefill_chunk``."""
        for request in requests:
            context = self._context(request)
            if request.model_request_id is None:
                continue
            end = min(len(context), request.prefill_cursor + int(chunk_size))
            self._ensure_capacity(request, end + 1)

    def prefill_chunk(self, requests: Sequence[BatchRequest], chunk_size: int) -> Sequence[Optional[int]]:
        """Advances every request by one chunk of its context; a request whose context is complete
        afterwards gets its first generated token, the others None (:1507-1572)."""
        if not self._announced_paths:
            later = "paged chunk attention" if hasattr(self.executor, "activate_paged_chunk_prefill_batch") \
                else "token replay"
            logger.info("chunked prefill: first chunks packed, later chunks by %s", later)
            self._announced_paths = True
        results: list[Optional[int]] = [None] * len(requests)
        fresh, later = [], []
        for index, request in enumerate(requests):
            if request.model_request_id is None:
                hit = self._adopt_cached(request)
                if hit is not None:
                    _, token = hit
                    if token is not None:
                        self._use_cached_token(request, token)
                        results[index] = token if self.return_host_tokens else None
                        continue
                    self._ensure_capacity(request, len(request.model_context_tokens) + 1)
            if request.model_request_id is None and request.prefill_cursor == 0:
                fresh.append(index)
            else:
                later.append(index)
        first = self._first_chunks_packed([requests[i] for i in fresh], chunk_size)
        if first is None:
            later = fresh + later
        else:
            for index, token in zip(fresh, first):
                results[index] = token
        rest = [requests[i] for i in later]
        tokens = self._later_chunks_paged(rest, chunk_size)
        if tokens is None:
            if not self._warned_replay:
                logger.warning("chunked prefill falls back to token-by-token replay: the executor offers no "
                               "attention over cached history for this batch")
                self._warned_replay = True
            tokens = self._replay(rest, chunk_size)
        for index, token in zip(later, tokens):
            results[index] = token
        return results

    # ---- decode --------------------------------------------------------------------------------
    def decode(self, requests: Sequence[BatchRequest]) -> Sequence[int]:
        """One token for every request (:1574-1595): the last sampled tokens go in, the next ones
        come out, and the slot of the following step is booked."""
        if not requests:
            return []
        ex = self.executor
        ids = tuple(int(r.model_request_id) for r in requests)
        if self._step_tokens is not None and ids == self._step_ids:
            input_ids = self._step_tokens.reshape(-1, 1)       # same batch as last step: no re-stacking
        else:
            input_ids = torch.stack([self._device_tokens[i] for i in ids]).reshape(-1, 1)
        if self.device_decode:
            batch = getattr(ex, "_device_batch", None)
            if batch is None or batch.request_ids != ids:
                try:
                    ex.activate_device_decode_batch(ids, reserve_tokens=self.decode_reserve_tokens, host_ahead=True)
                except RuntimeError:
                    # the pool cannot hold the look-ahead: pages are then taken step by step
                    ex.activate_device_decode_batch(ids, reserve_tokens=0, host_ahead=True)
            logits = ex.forward(input_ids)                     # positions are the device batch's
        else:
            ex.activate_paged_decode_batch(ids)
            position_ids = self._tensor([[self._positions[i]] for i in ids])
            logits = ex.forward(input_ids, position_ids)
        sampled = self._sample(logits, requests)
        self._remember(requests, sampled)
        self._step_ids, self._step_tokens = ids, sampled
        for req_idx in ids:
            self._positions[req_idx] += 1
        ex.extend_paged_requests(ids)
        if not self.return_host_tokens:
            return []
        tokens = [int(t) for t in sampled.detach().cpu().tolist()]
        # the readback above has waited for the step: the device batch's refusal flag is current
        batch = getattr(ex, "_device_batch", None) if self.device_decode else None
        if batch is not None and int(batch.overflow.item()) != 0:
            raise RuntimeError("Paged KV allocation failed during decode: a step on the device ran past a "
                               "request's reserved pages")
        return tokens

    # ---- release -------------------------------------------------------------------------------
    def release(self, requests: Sequence[BatchRequest]) -> None:
        ids = tuple(int(r.model_request_id) for r in requests if r.model_request_id is not None)
        if ids:
            self.executor.release_paged_request_ids(ids)
            for req_idx in ids:
                self._device_tokens.pop(req_idx, None)
                self._positions.pop(req_idx, None)
            if any(i in self._step_ids for i in ids):
                self._step_ids, self._step_tokens = (), None
        for request in requests:
            request.model_request_id = None

    def preempt(self, requests: Sequence[BatchRequest]) -> None:
        """A preempted request gives its pages back; it is prefilled again later from
        ``model_context_tokens`` (:1611-1612)."""
        self.release(requests)
