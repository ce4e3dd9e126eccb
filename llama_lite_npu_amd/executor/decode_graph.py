"""Decode steps as replayed HIP graphs, with the batch's metadata advanced on the device.

Counterpart of the reference's ``lite_llama/executor/npu_graph.py`` (NpuGraphRunner :66-217,
supports_decode_graph :35-52): same entry points (``graph_key``, ``capture``, ``replay``,
``__call__``), same counters and the same rule that a key whose capture failed is not tried
again. Two things differ:

* **No length buckets by default.** The reference recaptures every 128 tokens because its
  decode launch is sized by the context length. Here no launch dimension depends on it: the
  decode kernel's grid is (chunks, kv heads), the cuts live in a plan buffer that a kernel
  rewrites each step, and the block table has its full width. One graph per batch size serves
  every length (``PARTITION_SIZE = None``; set it to 128 for the reference's keys).

* **Metadata can step inside the graph.** With a ``DeviceDecodeBatch`` the lengths, slots,
  positions, block-table rows and the plan are advanced by two small launches at the head of
  the captured step, so a replay uploads nothing but the new token ids. Without one the runner
  works like the reference's: it keeps static copies of the step's tensors and refreshes them
  before each replay (:183-197).
"""

from __future__ import annotations

import contextlib
import copy
import gc
import logging
from dataclasses import dataclass
from typing import Any, Callable, Optional, Sequence

import numpy as np
import torch

logger = logging.getLogger(__name__)


def supports_decode_graph(model_type: str, moe_parallel_mode: str = "tp") -> bool:
    """Whether decode-graph capture may be attempted for a model family (reference :35-52).
    Vision-language models feed per-step image tensors; expert-parallel MoE compacts its
    assignments with a data-dependent ``nonzero`` that cannot run under capture."""
    model_type = model_type.lower()
    if model_type in {"qwen3_vl", "llava"}:
        return False
    if model_type == "qwen3_moe" and moe_parallel_mode == "ep":
        return False
    return True


class DeviceDecodeBatch:
    """Metadata of a decode batch in fixed device tensors, stepped by ``litekv_decode_advance``.

    Host side per step: ``host_advance()`` (dictionary bookkeeping of the request manager; a page
    is allocated and its id uploaded only when a request outgrows its reserved pages). Device
    side per step: ``enqueue_advance()`` (two launches: metadata, plan), which a graph can hold.
    The tensors keep their addresses for the life of the object; ``load`` re-targets them at
    another set of requests of the same count.
    """

    def __init__(self, executor, request_ids: Sequence[int], reserve_tokens: int = 0,
                 shared_pages: Optional[int] = None, host_ahead: bool = False):
        from .. import ops

        self.executor = executor
        mgr = executor.req_tokens_manager
        dev = executor.device
        b = len(request_ids)
        if b == 0:
            raise ValueError("request_ids must not be empty")
        self.batch = b
        self.width = mgr.max_pages_per_req
        self.b_req_idx = torch.zeros(b, dtype=torch.int32, device=dev)
        self.seq_lens_i32 = torch.zeros(b, dtype=torch.int32, device=dev)
        self.b_seq_len = torch.zeros(b, dtype=torch.int64, device=dev)
        self.cur_select_index = torch.full((b,), -1, dtype=torch.int32, device=dev)
        self.position_ids = torch.zeros(b, dtype=torch.int64, device=dev)
        self.capacity = torch.zeros(b, dtype=torch.int32, device=dev)
        self.block_table = torch.zeros((b, self.width), dtype=torch.int32, device=dev)
        self.overflow = torch.zeros(1, dtype=torch.int32, device=dev)
        self.b_start_loc = torch.zeros(b, dtype=torch.int32, device=dev)
        self.cu_q_lens = torch.arange(b + 1, dtype=torch.int32, device=dev)
        self.request_ids: tuple[int, ...] = ()
        self.pending = False      # host_advance() done, enqueue_advance() (or a replay) still due
        self.steps = 0
        self.look_ahead = 0       # tokens of page reserve taken again whenever a request runs out
        self._capacity_host = np.zeros(b, dtype=np.int32)
        if shared_pages is None:
            shared_pages = executor.shared_prefix_pages(request_ids, upcoming_tokens=0 if host_ahead else 1)
        self.shared_pages = int(shared_pages)
        self.decode_plan = ops.DecodePlan(self.block_table, self.seq_lens_i32, executor.local_q_heads,
                                          executor.local_kv_heads, executor.kv_mem_manager.num_pages,
                                          page_size=executor.page_size, shared_pages=self.shared_pages,
                                          token_bytes=getattr(executor, "kv_token_bytes", None),
                                          kv_dtype=executor.kv_mem_manager.gpu_kv_buffer[0].dtype)
        self.load(request_ids, reserve_tokens, host_ahead)

    # ---- host side -------------------------------------------------------------------------
    def _upload_capacity(self) -> None:
        mgr = self.executor.req_tokens_manager
        ps = self.executor.page_size
        cap = np.asarray([min(mgr.req_page_count[r] * ps, mgr.max_seq_len) for r in self.request_ids],
                         dtype=np.int32)
        if not np.array_equal(cap, self._capacity_host):
            self._capacity_host = cap
            self.capacity.copy_(torch.from_numpy(cap))

    def load(self, request_ids: Sequence[int], reserve_tokens: int = 0, host_ahead: bool = False) -> None:
        """Points the batch at ``request_ids`` (same count): uploads ids and current lengths, then
        recomputes slots, positions, table rows and the plan on the device for those lengths.
        ``host_ahead``: the host has already booked the next step's token for every request (the
        reference's order: ``extend_paged_requests`` follows each forward, model_executor.py:913-933,
        continuous_batching.py:1574-1595), so the device starts one token behind and the first
        step needs no ``host_advance()``."""
        mgr = self.executor.req_tokens_manager
        ids = tuple(int(r) for r in request_ids)
        if len(ids) != self.batch:
            raise ValueError(f"this batch holds {self.batch} requests, got {len(ids)}")
        for r in ids:
            if r not in mgr.req_token_count:
                raise KeyError(f"request {r} is not allocated")
        ahead = 1 if host_ahead else 0
        if any(mgr.req_token_count[r] - ahead < 1 for r in ids):
            raise ValueError("every request needs at least one token in the cache before it decodes")
        if self.shared_pages and self.executor.common_leading_pages(ids, upcoming_tokens=1 - ahead) < self.shared_pages:
            raise ValueError(f"requests do not share the {self.shared_pages} leading pages this batch was built for")
        self.request_ids = ids
        self.look_ahead = int(reserve_tokens)
        self.b_req_idx.copy_(torch.tensor(ids, dtype=torch.int32))
        self.seq_lens_i32.copy_(torch.tensor([mgr.req_token_count[r] - ahead for r in ids], dtype=torch.int32))
        self._capacity_host = np.zeros(self.batch, dtype=np.int32)
        self.reserve(reserve_tokens)
        self.overflow.zero_()
        self.pending = bool(host_ahead)
        self._choose_schedule()
        self._launch_advance(0)

    def reserve(self, tokens_ahead: int) -> None:
        """Reserves pages so every request can grow by ``tokens_ahead`` tokens without the host
        touching the page tables (capped at the executor's max_seq_len)."""
        mgr = self.executor.req_tokens_manager
        for r in self.request_ids:
            want = min(mgr.req_token_count[r] + int(tokens_ahead), mgr.max_seq_len)
            if not mgr.ensure_req_capacity(r, want):
                raise RuntimeError(f"Paged KV capacity reservation failed for request {r}")
        self._upload_capacity()

    def host_advance(self) -> None:
        """Books one more token for every request (allocating a page where the reserve ran out)."""
        if self.pending:
            raise RuntimeError("the previous host_advance() has not been followed by a device step")
        mgr = self.executor.req_tokens_manager
        counts, reserved = mgr.req_token_count, self._capacity_host
        grew = False
        for i, r in enumerate(self.request_ids):
            if counts[r] >= reserved[i]:                  # this token needs a page beyond the reserve:
                grew = True                               # take the look-ahead again in one go
                if self.look_ahead > 0:
                    mgr.ensure_req_capacity(r, min(counts[r] + 1 + self.look_ahead, mgr.max_seq_len))
            if not mgr.extend_req(r, 1):
                raise RuntimeError(
                    "Paged KV allocation failed for request "
                    f"{r}: current_tokens={mgr.req_token_count.get(r, 'unknown')}, "
                    f"max_seq_len={mgr.max_seq_len}, free_pages={mgr.page_mgr.num_free_pages}")
        if grew:
            self._upload_capacity()
        self.pending = True
        self.steps += 1
        if self.steps % 16 == 0:       # lengths drift slowly: a look every few steps is enough
            self._choose_schedule()

    def _choose_schedule(self) -> None:
        """Balanced or per-sequence decode (and its split count) for the coming steps, from the
        host's lengths. The schedule in use keeps a 10 % advantage so that a batch near a boundary
        does not flip (a graph runner holds one graph per schedule)."""
        plan = self.decode_plan
        counts = self.executor.req_tokens_manager.req_token_count
        plan.choose_schedule([counts[r] for r in self.request_ids], hysteresis=1.1)

    @property
    def max_actual_seq_len(self) -> int:
        mgr = self.executor.req_tokens_manager
        return max(mgr.req_token_count[r] for r in self.request_ids)

    # ---- device side -----------------------------------------------------------------------
    def _launch_advance(self, increment: int) -> None:
        from .. import ops

        ex = self.executor
        ops.decode_advance(ex.req_tokens_manager.block_table, self.b_req_idx, self.seq_lens_i32,
                           self.cur_select_index, self.block_table, ex.kv_mem_manager.num_pages,
                           capacity=self.capacity, seq_lens_i64=self.b_seq_len, position_ids=self.position_ids,
                           overflow=self.overflow, page_size=ex.page_size, increment=increment)
        self.decode_plan.refresh()

    def enqueue_advance(self) -> None:
        """The device half of a step (capturable): lengths + 1, new slots and positions, table rows, plan."""
        if not self.pending:
            raise RuntimeError("host_advance() must book the step's token before the device advances")
        self._launch_advance(1)
        self.pending = False

    def step(self) -> None:
        self.host_advance()
        self.enqueue_advance()

    def bind(self, atten_info) -> None:
        """Makes ``atten_info`` describe this batch through the fixed tensors."""
        info = atten_info
        info.b_req_idx, info.b_seq_len, info.seq_lens_i32 = self.b_req_idx, self.b_seq_len, self.seq_lens_i32
        info.cur_select_index = self.cur_select_index
        info.b_start_loc, info.cu_q_lens = self.b_start_loc, self.cu_q_lens
        info.block_table = self.block_table
        info.b_req_tokens_table = None
        info.decode_plan = self.decode_plan
        info.device_decode = self
        info.max_actual_seq_len = self.max_actual_seq_len

    def check(self) -> None:
        """Reads the overflow flag back (synchronises) and checks the device lengths against the host's."""
        mgr = self.executor.req_tokens_manager
        if int(self.overflow.item()) != 0:
            raise RuntimeError("a decode step on the device ran past a request's reserved pages")
        want = [mgr.req_token_count[r] - (1 if self.pending else 0) for r in self.request_ids]
        got = self.seq_lens_i32.tolist()
        if got != want:
            raise RuntimeError(f"device sequence lengths {got} differ from the host's {want}")


@contextlib.contextmanager
def quiet_capture(graph, **kwargs):
    """``torch.cuda.graph`` with Python's cyclic collector held off. A collection that starts
    while the stream is capturing can destroy an older graph or return pool memory to the
    driver; HIP refuses both during a capture and the process aborts. Dead cycles are collected
    before the capture begins instead (PyTorch no longer does that on its own)."""
    gc.collect()
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph, **kwargs):
            yield
    finally:
        if was_enabled:
            gc.enable()


class _TorchHipGraphs:
    """The graph calls the runner needs, as PyTorch-ROCm exposes hipGraph."""

    @property
    def available(self) -> bool:
        return torch.cuda.is_available() and hasattr(torch.cuda, "CUDAGraph")

    def Graph(self):
        return torch.cuda.CUDAGraph()

    def graph(self, graph, pool=None):
        return quiet_capture(graph, pool=pool)

    def synchronize(self) -> None:
        torch.cuda.synchronize()

    def graph_pool_handle(self):
        return torch.cuda.graph_pool_handle()


@dataclass
class _CapturedGraph:
    graph: Any
    output: Any
    input_ids: torch.Tensor
    position_ids: torch.Tensor
    cur_select_index: Optional[torch.Tensor]
    b_seq_len: Optional[torch.Tensor]
    b_req_idx: Optional[torch.Tensor]
    seq_lens_i32: Optional[torch.Tensor] = None
    block_table: Optional[torch.Tensor] = None
    device_decode: Optional[DeviceDecodeBatch] = None
    static_info: Any = None     # keeps everything the graph reads or writes alive (the step's plan and workspace too)


class DecodeGraphRunner:
    """Captures ``model.forward(input_ids, position_ids, atten_info)`` of a decode step once per key
    and replays it afterwards."""

    PARTITION_SIZE: Optional[int] = None

    def __init__(self, model, model_type: str = "unknown", graph_api=None, max_blocks: Optional[int] = None):
        """``max_blocks``: width every static block table is given (the executor's
        ``max_pages_per_req``), needed without length buckets when the step's table is trimmed."""
        self.model = model
        self.model_type = model_type
        self.max_blocks = max_blocks
        self._api = graph_api if graph_api is not None else _TorchHipGraphs()
        self._graphs: dict[tuple, _CapturedGraph] = {}
        self._failed_keys: set[tuple] = set()
        self._pool = self._api.graph_pool_handle() if self.available else None
        self.capture_count = 0
        self.capture_attempt_count = 0
        self.replay_count = 0
        self.fallback_count = 0

    @property
    def available(self) -> bool:
        return bool(self._api.available)

    @property
    def captured(self) -> bool:
        return bool(self._graphs)

    @classmethod
    def sequence_bucket(cls, sequence_length: int) -> int:
        """Lengths that share a graph: multiples of PARTITION_SIZE as in the reference (:94-99), or
        one bucket (0) for all lengths when PARTITION_SIZE is None."""
        if cls.PARTITION_SIZE is None:
            return 0
        sequence_length = max(1, int(sequence_length))
        return ((sequence_length + cls.PARTITION_SIZE - 1) // cls.PARTITION_SIZE) * cls.PARTITION_SIZE

    def graph_key(self, input_ids: torch.Tensor, sequence_length: int) -> tuple[int, int]:
        return input_ids.shape[0], self.sequence_bucket(sequence_length)

    def _key(self, input_ids, atten_info) -> tuple:
        key = self.graph_key(input_ids, atten_info.max_actual_seq_len)
        device = getattr(atten_info, "device_decode", None)
        plan = getattr(atten_info, "decode_plan", None)
        # a graph holds the kernels of the decode schedule it was captured with
        per_sequence = int(plan.schedule) if plan is not None else 0   # 0 balanced, else splits per sequence
        if device is not None:
            return key + (id(device), per_sequence)   # the graph is tied to that batch's tensors
        # Host-metadata steps replay through a static plan built at capture: the graph holds that
        # plan's launches, so a batch that shares another number of leading pages (a cached
        # prefix attended once for the batch) needs a graph of its own. A graph captured with a
        # shared prefix would otherwise make every later batch of that size attend row 0's pages.
        shared = int(getattr(plan, "shared_pages", 0) or 0) if plan is not None else 0
        extra = (("shared", shared),) if shared > 0 else ()
        table = getattr(atten_info, "block_table", None)
        if self.PARTITION_SIZE is None and self.max_blocks is None and table is not None:
            return key + (int(table.shape[1]), per_sequence) + extra   # a trimmed table: its width sizes the plan
        return key + ((per_sequence,) if per_sequence else ()) + extra

    # ---- capture ---------------------------------------------------------------------------
    def _static_info(self, atten_info):
        """Copies of the step's dynamic tensors at fixed addresses; the large pools are shared."""
        info = copy.copy(atten_info)
        for name in ("cur_select_index", "b_seq_len", "b_req_idx", "seq_lens_i32"):
            value = getattr(atten_info, name, None)
            setattr(info, name, value.clone() if value is not None else None)
        table = getattr(atten_info, "block_table", None)
        if table is not None:
            width = max(int(table.shape[1]), int(self.max_blocks or 0))
            info.block_table = torch.zeros((table.shape[0], width), dtype=table.dtype, device=table.device)
            info.block_table[:, :table.shape[1]] = table
        plan = getattr(atten_info, "decode_plan", None)
        if plan is not None:
            from .. import ops

            info.decode_plan = ops.DecodePlan(info.block_table, info.seq_lens_i32, plan.num_q_heads,
                                              plan.num_kv_heads, plan.num_pages, plan.chunks, plan.page_size,
                                              plan.shared_pages, token_bytes=plan.token_bytes,
                                              kv_dtype=getattr(plan, "kv_dtype", None))
            info.decode_plan.set_schedule(plan.schedule)
        return info

    def capture(self, input_ids: torch.Tensor, position_ids: torch.Tensor, atten_info) -> bool:
        """Captures one graph for the step's key. Host-metadata steps are run once eagerly on the
        static copies first, as the reference does (:126-134); a device-metadata step is captured
        right after its eager run, so nothing is executed twice."""
        if not self.available:
            return False
        key = self._key(input_ids, atten_info)
        if key in self._graphs:
            return True
        if key in self._failed_keys:
            return False
        self.capture_attempt_count += 1
        device = getattr(atten_info, "device_decode", None)
        try:
            static_input_ids = input_ids.clone()
            if device is None:
                static_position_ids = position_ids.clone()
                static_info = self._static_info(atten_info)
                static_info.max_actual_seq_len = key[1] or atten_info.max_actual_seq_len
                plan = getattr(static_info, "decode_plan", None)
                prologue: Optional[Callable[[], None]] = plan.refresh if plan is not None else None
                _ = self.model.forward(static_input_ids, static_position_ids, static_info)
            else:
                static_position_ids = device.position_ids
                static_info = copy.copy(atten_info)
                prologue = lambda: device._launch_advance(1)   # the step's host half is booked per replay
            self._api.synchronize()

            graph = self._api.Graph()
            with self._api.graph(graph, pool=self._pool):
                if prologue is not None:
                    prologue()
                graph_output = self.model.forward(static_input_ids, static_position_ids, static_info)

            self._graphs[key] = _CapturedGraph(
                graph=graph, output=graph_output, input_ids=static_input_ids, position_ids=static_position_ids,
                cur_select_index=static_info.cur_select_index, b_seq_len=static_info.b_seq_len,
                b_req_idx=getattr(static_info, "b_req_idx", None),
                seq_lens_i32=getattr(static_info, "seq_lens_i32", None),
                block_table=getattr(static_info, "block_table", None), device_decode=device,
                static_info=static_info)
            self.capture_count += 1
            logger.info("Captured decode graph for model=%s batch=%d bucket=%d", self.model_type, key[0], key[1])
            return True
        except Exception as exc:
            self._failed_keys.add(key)
            logger.warning("decode graph capture failed for model=%s batch=%d bucket=%d; using eager execution: %s",
                           self.model_type, key[0], key[1], exc)
            return False

    # ---- replay ----------------------------------------------------------------------------
    def replay(self, input_ids: torch.Tensor, position_ids: torch.Tensor, atten_info):
        """Replays the step's graph after refreshing its inputs; None if the key has no graph."""
        captured = self._graphs.get(self._key(input_ids, atten_info))
        if captured is None:
            return None
        captured.input_ids.copy_(input_ids)
        if captured.device_decode is None:
            captured.position_ids.copy_(position_ids)
            for name in ("cur_select_index", "b_seq_len", "b_req_idx", "seq_lens_i32"):
                static, value = getattr(captured, name), getattr(atten_info, name, None)
                if static is not None and value is not None:
                    static.copy_(value)
            table = getattr(atten_info, "block_table", None)
            if captured.block_table is not None and table is not None:
                captured.block_table[:, :table.shape[1]].copy_(table)
        captured.graph.replay()
        if captured.device_decode is not None:
            captured.device_decode.pending = False
        self.replay_count += 1
        return captured.output

    def __call__(self, input_ids, position_ids, atten_info):
        device = getattr(atten_info, "device_decode", None)
        if device is not None and not device.pending:
            raise RuntimeError("host_advance() must book the step's token before the step runs")
        if not self.available:
            self.fallback_count += 1
            return self._eager(input_ids, position_ids, atten_info, device)
        key = self._key(input_ids, atten_info)
        if device is not None:
            if key in self._graphs:
                return self.replay(input_ids, position_ids, atten_info)
            result = self._eager(input_ids, position_ids, atten_info, device)
            if key not in self._failed_keys:
                self.capture(input_ids, position_ids, atten_info)
            else:
                self.fallback_count += 1
            return result
        if key not in self._graphs and key not in self._failed_keys:
            self.capture(input_ids, position_ids, atten_info)
        result = self.replay(input_ids, position_ids, atten_info)
        if result is None:
            self.fallback_count += 1
            return self.model.forward(input_ids, position_ids, atten_info)
        return result

    def _eager(self, input_ids, position_ids, atten_info, device):
        if device is not None:
            device.enqueue_advance()
            position_ids = device.position_ids
        return self.model.forward(input_ids, position_ids, atten_info)
