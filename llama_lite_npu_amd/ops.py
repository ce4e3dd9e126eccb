"""Block-table-native operators over liblitekv (PyTorch-ROCm tensors in, C ABI out).

PyTorch supplies device memory and the current stream; every byte of the path
is moved or computed by the HIP kernels behind include/litekv.h. All calls only
enqueue work on ``torch.cuda.current_stream()``.
"""

from __future__ import annotations

import math
from typing import Optional, Sequence

import torch

from . import _lib

PAGE_SIZE = 16
HEAD_DIM = 128


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _dev_half(name: str, t: torch.Tensor) -> None:
    _need(t.is_cuda, f"{name} must live on the GPU")
    _need(t.dtype == torch.float16, f"{name} must be float16, got {t.dtype}")


FP8_DTYPES = (torch.uint8, torch.float8_e4m3fn)
INT8_DTYPES = (torch.int8,)


def _dev_pool(name: str, t: torch.Tensor) -> None:
    _need(t.is_cuda, f"{name} must live on the GPU")
    _need(t.dtype == torch.float16 or t.dtype in FP8_DTYPES + INT8_DTYPES,
          f"{name} must be float16, fp8 or int8, got {t.dtype}")


def is_fp8_pool(kv_pool: torch.Tensor) -> bool:
    """An fp8 pool holds one E4M3 code per element (a uint8 or float8_e4m3fn tensor)."""
    return kv_pool.dtype in FP8_DTYPES


def is_int8_pool(kv_pool: torch.Tensor) -> bool:
    """An int8 pool holds one signed 8-bit code per element (a torch.int8 tensor)."""
    return kv_pool.dtype in INT8_DTYPES


def is_quantised_pool(kv_pool: torch.Tensor) -> bool:
    """A pool of 8-bit codes (fp8 or int8) with one fp32 scale per kv head: value = code * scale."""
    return is_fp8_pool(kv_pool) or is_int8_pool(kv_pool)


def _q8_entry(lib, stem: str, kv_pool: torch.Tensor):
    """The library's entry point `stem` for the pool's 8-bit format (litekv_<stem>_fp8 / _int8)."""
    return getattr(lib, f"litekv_{stem}_{'int8' if is_int8_pool(kv_pool) else 'fp8'}")


def _dev_fp8_pool(kv_pool: torch.Tensor, scales: Optional[torch.Tensor], num_kv_heads: int) -> None:
    _need(kv_pool.is_cuda and is_quantised_pool(kv_pool),
          f"kv_pool must be an fp8 (uint8 / float8_e4m3fn) or int8 GPU tensor, got {kv_pool.dtype}")
    _need(scales is not None, "a pool of 8-bit codes needs its per-head scales")
    _need(scales.is_cuda and scales.dtype == torch.float32 and scales.is_contiguous()
          and scales.numel() == 2 * num_kv_heads, "scales must be float32 [2 * Hkv] on the GPU (K heads, then V heads)")


def _dev_i32(name: str, t: torch.Tensor) -> torch.Tensor:
    _need(t.is_cuda, f"{name} must live on the GPU")
    if t.dtype != torch.int32:
        t = t.to(torch.int32)  # device-side cast, no host sync
    return t.contiguous()


def _rows(name: str, t: torch.Tensor) -> int:
    """Token stride of a [T, H, D] tensor whose [H, D] block is contiguous."""
    _need(t.dim() == 3, f"{name} must be [tokens, heads, head_dim]")
    _need(t.stride(2) == 1 and t.stride(1) == t.shape[2], f"{name}: [heads, head_dim] block must be contiguous")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1] * t.shape[2])


def pool_geometry(kv_pool: torch.Tensor, page_size: int = PAGE_SIZE):
    """(num_slots, num_kv_heads, head_dim, num_pages, page_bytes) of a [slots, 2*Hkv, D] pool."""
    _need(kv_pool.dim() == 3 and kv_pool.is_contiguous(), "kv_pool must be contiguous [slots, 2*Hkv, D]")
    slots, two_h, d = kv_pool.shape
    _need(two_h % 2 == 0, "kv_pool dim 1 must be 2 * num_kv_heads")
    _need(slots % page_size == 0, "kv_pool slots must be a multiple of page_size")
    return slots, two_h // 2, d, slots // page_size, page_size * two_h * d * kv_pool.element_size()


def kv_append(k: torch.Tensor, v: torch.Tensor, slot_mapping: torch.Tensor, kv_pool: torch.Tensor) -> None:
    """kv_pool[slot_mapping[t]] = concat(k[t], v[t]) for every token t (bit exact, in place)."""
    _dev_half("k", k), _dev_half("v", v), _dev_half("kv_pool", kv_pool)
    slots, hkv, d, _, _ = pool_geometry(kv_pool, 1)
    _need(k.shape == v.shape, "k and v must have the same shape")
    _need(k.shape[1] == hkv and k.shape[2] == d, f"k/v heads {tuple(k.shape[1:])} do not match pool ({hkv}, {d})")
    slot_mapping = _dev_i32("slot_mapping", slot_mapping)
    t = k.shape[0]
    _need(slot_mapping.numel() == t, "slot_mapping must hold one slot per token")
    lib = _lib.load()
    _lib.check(lib.litekv_kv_append(_ptr(k), _ptr(v), _rows("k", k), _rows("v", v), _ptr(slot_mapping),
                                    _ptr(kv_pool), t, hkv, d, slots, _stream()))


def kv_append_quantised(k: torch.Tensor, v: torch.Tensor, slot_mapping: torch.Tensor, kv_pool: torch.Tensor,
                        scales: torch.Tensor) -> None:
    """kv_pool[slot_mapping[t]] = code(concat(k[t], v[t]) / scale of the head) for every token t, in the
    pool's format (E4M3 for a uint8 / float8_e4m3fn pool, int8 for a torch.int8 pool);
    scales is float32 [2 * Hkv]: K-head scales, then V-head scales."""
    _dev_half("k", k), _dev_half("v", v)
    slots, hkv, d, _, _ = pool_geometry(kv_pool, 1)
    _dev_fp8_pool(kv_pool, scales, hkv)
    _need(k.shape == v.shape and k.shape[1] == hkv and k.shape[2] == d, "k / v must be [T, Hkv, D] matching the pool")
    slot_mapping = _dev_i32("slot_mapping", slot_mapping)
    t = k.shape[0]
    _need(slot_mapping.numel() == t, "slot_mapping must hold one slot per token")
    lib = _lib.load()
    _lib.check(_q8_entry(lib, "kv_append", kv_pool)(_ptr(k), _ptr(v), _rows("k", k), _rows("v", v),
                                                    _ptr(slot_mapping), _ptr(kv_pool), _ptr(scales), t, hkv, d,
                                                    slots, _stream()))


kv_append_fp8 = kv_append_quantised     # the name from before int8 pools


def page_dequant(kv_pool: torch.Tensor, dst_pool: torch.Tensor, src_ids: torch.Tensor,
                 dst_ids: Optional[torch.Tensor], scales: torch.Tensor, page_size: int = PAGE_SIZE) -> None:
    """dst_pool[page dst_ids[i]] (fp16) = decoded page src_ids[i] of the fp8 pool; dst_ids None means page i."""
    _dev_half("dst_pool", dst_pool)
    _, hkv, d, n_src, _ = pool_geometry(kv_pool, page_size)
    _, hkv_d, d_d, n_dst, _ = pool_geometry(dst_pool, page_size)
    _dev_fp8_pool(kv_pool, scales, hkv)
    _need((hkv, d) == (hkv_d, d_d), "pools differ in head geometry")
    src_ids = _dev_i32("src_ids", src_ids)
    if dst_ids is not None:
        dst_ids = _dev_i32("dst_ids", dst_ids)
        _need(dst_ids.numel() == src_ids.numel(), "src_ids and dst_ids differ in length")
    lib = _lib.load()
    fn = lib.litekv_page_dequant_int8 if is_int8_pool(kv_pool) else lib.litekv_page_dequant
    _lib.check(fn(_ptr(kv_pool), _ptr(dst_pool), _ptr(src_ids), _ptr(dst_ids), src_ids.numel(),
                  _ptr(scales), hkv, d, page_size, n_src, n_dst, _stream()))


def qk_norm_rope_append(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, slot_mapping: torch.Tensor,
                        kv_pool: torch.Tensor, q_norm_weight: Optional[torch.Tensor] = None,
                        k_norm_weight: Optional[torch.Tensor] = None, cos: Optional[torch.Tensor] = None,
                        sin: Optional[torch.Tensor] = None, rms_eps: float = 1e-6,
                        kv_scales: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per-head RMSNorm (optional) and rotary embedding (optional) of q [T, Hq, D] in place and of
    k [T, Hkv, D] on its way into the pool, plus the append of v: one launch for the reference's
    skip_rmsnorm x2 + rope_emb_forward + cat + update_kv_buffer. cos / sin are [T, >= D/2] rows of
    each token's position. An fp8 pool (with its ``kv_scales``) receives the quantised rows. Returns q."""
    _dev_half("q", q), _dev_half("k", k), _dev_half("v", v)
    slots, hkv, d, _, _ = pool_geometry(kv_pool, 1)
    fp8 = is_quantised_pool(kv_pool)
    if fp8:
        _dev_fp8_pool(kv_pool, kv_scales, hkv)
    else:
        _dev_half("kv_pool", kv_pool)
    t, hq = q.shape[0], q.shape[1]
    _need(q.dim() == 3 and q.shape[2] == d, "q must be [T, Hq, D]")
    _need(k.shape == (t, hkv, d) and v.shape == (t, hkv, d), "k / v must be [T, Hkv, D] matching the pool")
    _need((q_norm_weight is None) == (k_norm_weight is None), "q_norm_weight and k_norm_weight go together")
    _need((cos is None) == (sin is None), "cos and sin go together")
    if q_norm_weight is not None:
        _dev_half("q_norm_weight", q_norm_weight), _dev_half("k_norm_weight", k_norm_weight)
        _need(q_norm_weight.numel() == d and k_norm_weight.numel() == d and q_norm_weight.is_contiguous()
              and k_norm_weight.is_contiguous(), "norm weights must be contiguous [D]")
    cs_stride = 0
    if cos is not None:
        _dev_half("cos", cos), _dev_half("sin", sin)
        cos, sin = cos.reshape(-1, cos.shape[-1]), sin.reshape(-1, sin.shape[-1])
        _need(cos.shape == sin.shape and cos.shape[0] == t and cos.shape[1] >= d // 2, "cos / sin must be [T, >= D/2]")
        _need(cos.stride(1) == 1 and sin.stride(1) == 1 and cos.stride(0) == sin.stride(0),
              "cos / sin rows must be contiguous with equal row strides")
        cs_stride = cos.stride(0)
    slot_mapping = _dev_i32("slot_mapping", slot_mapping)
    _need(slot_mapping.numel() == t, "slot_mapping must hold one slot per token")
    lib = _lib.load()
    if fp8:
        _lib.check(_q8_entry(lib, "qk_norm_rope_append", kv_pool)(
            _ptr(q), _rows("q", q), _ptr(k), _rows("k", k), _ptr(v), _rows("v", v), _ptr(q_norm_weight),
            _ptr(k_norm_weight), _ptr(cos), _ptr(sin), cs_stride, _ptr(slot_mapping), _ptr(kv_pool),
            _ptr(kv_scales), t, hq, hkv, d, slots, float(rms_eps), _stream()))
        return q
    _lib.check(lib.litekv_qk_norm_rope_append(
        _ptr(q), _rows("q", q), _ptr(k), _rows("k", k), _ptr(v), _rows("v", v), _ptr(q_norm_weight),
        _ptr(k_norm_weight), _ptr(cos), _ptr(sin), cs_stride, _ptr(slot_mapping), _ptr(kv_pool), t, hq, hkv, d,
        slots, float(rms_eps), _stream()))
    return q


def page_gather(src_pool: torch.Tensor, dst_pool: torch.Tensor, src_ids: torch.Tensor,
                dst_ids: Optional[torch.Tensor] = None, page_size: int = PAGE_SIZE) -> None:
    """dst_pool[page dst_ids[i]] = src_pool[page src_ids[i]]; dst_ids None means page i. Pages are
    moved as bytes: fp16 pools or fp8 pools, both of the same kind."""
    _dev_pool("src_pool", src_pool), _dev_pool("dst_pool", dst_pool)
    _need(src_pool.element_size() == dst_pool.element_size(), "pools differ in element size")
    _, hs, ds, n_src, page_bytes = pool_geometry(src_pool, page_size)
    _, hd, dd, n_dst, page_bytes_d = pool_geometry(dst_pool, page_size)
    _need((hs, ds) == (hd, dd) and page_bytes == page_bytes_d, "pools differ in page geometry")
    src_ids = _dev_i32("src_ids", src_ids)
    if dst_ids is not None:
        dst_ids = _dev_i32("dst_ids", dst_ids)
        _need(dst_ids.numel() == src_ids.numel(), "src_ids and dst_ids differ in length")
    lib = _lib.load()
    _lib.check(lib.litekv_page_gather(_ptr(src_pool), _ptr(dst_pool), _ptr(src_ids), _ptr(dst_ids),
                                      src_ids.numel(), page_bytes, n_src, n_dst, _stream()))


def page_copy(kv_pool: torch.Tensor, src_ids: torch.Tensor, dst_ids: torch.Tensor,
              page_size: int = PAGE_SIZE) -> None:
    """kv_pool[page dst_ids[i]] = kv_pool[page src_ids[i]] (copy-on-write move inside one pool, fp16 or fp8)."""
    _dev_pool("kv_pool", kv_pool)
    _, _, _, n_pages, page_bytes = pool_geometry(kv_pool, page_size)
    src_ids = _dev_i32("src_ids", src_ids)
    dst_ids = _dev_i32("dst_ids", dst_ids)
    _need(dst_ids.numel() == src_ids.numel(), "src_ids and dst_ids differ in length")
    lib = _lib.load()
    _lib.check(lib.litekv_page_copy(_ptr(kv_pool), _ptr(src_ids), _ptr(dst_ids), src_ids.numel(),
                                    page_bytes, n_pages, _stream()))


def decode_split_plan(batch: int, num_kv_heads: int, max_blocks: int,
                      num_splits: Optional[int] = None) -> tuple[int, int]:
    """(max_splits, min_pages_per_split) for a decode launch.

    ``num_splits`` fixes the split count per sequence (every sequence with at
    least that many pages uses exactly that many). Otherwise pages per split
    are chosen so the launch has a few thousand wavefronts of at least 8 pages.
    """
    if num_splits is not None:
        return max(1, int(num_splits)), 1
    items = max(1, batch * num_kv_heads)
    target_waves = 4096
    pps = max(8, min(64, (items * max_blocks + target_waves - 1) // target_waves))
    return max(1, (max_blocks + pps - 1) // pps), pps


def decode_workspace(batch: int, num_q_heads: int, max_splits: int, device) -> Optional[torch.Tensor]:
    nbytes = _lib.load().litekv_paged_decode_workspace_bytes(batch, num_q_heads, HEAD_DIM, max_splits)
    if nbytes == 0:
        return None
    return torch.empty(nbytes // 4, dtype=torch.float32, device=device)


def balanced_chunks(num_kv_heads: int) -> int:
    """Chunks per kv head that give every CU of the current device one workgroup."""
    return int(_lib.load().litekv_paged_decode_balanced_chunks(int(num_kv_heads)))


def prefix_chunks(batch: int, num_q_heads: int, num_kv_heads: int, shared_pages: int,
                  page_size: int = PAGE_SIZE, head_dim: int = HEAD_DIM, fp16_pool: bool = True) -> int:
    """Chunks per kv head for a step behind ``shared_pages`` shared pages: the private pages get the
    compute units that the workgroups attending the shared pages (same launch) leave free."""
    return int(_lib.load().litekv_paged_decode_prefix_chunks(int(batch), int(num_q_heads), int(num_kv_heads),
                                                             int(head_dim), int(page_size), int(shared_pages),
                                                             1 if fp16_pool else 0))


SPLIT_COUNTS = (4, 8, 16)


def decode_schedule_estimates(batch: int, num_kv_heads: int, max_pages: int, total_pages: int, token_bytes: int,
                              page_size: int = PAGE_SIZE, heads_per_kv_head: int = 8) -> dict:
    """Estimated microseconds per layer of every decode schedule a step could take, keyed as
    ``decode_schedule`` returns them. Fits to 554 measured shapes on an MI355X (1 to 2048 sequences
    of 32 to 16384 tokens: equal, ragged, one long among short; 64/8 and 16/8 heads; every
    schedule replayed from a graph; ``tune_decode_schedule`` re-measures the table):

    * 1, one wavefront per (sequence, kv head), one launch: 4.3 us + the largest (a 3.6-norm) of the
      longest sequence's dependent chain of 16-token steps at 0.58 us each -- up to half as much
      again when the launch has 2048 wavefronts or more, whose loads share the compute units'
      memory paths with the chain's --, the placement of the launch's wavefronts at 2.9 ns each,
      and the bytes at 5.7 MB/us (unbalanced streams).
    * 4 / 8 / 16 splits per sequence + the merge launch, for launches of at most 2048 wavefronts:
      6.8 us for the two launches, the chain of a split against the bytes at 6.1 MB/us (a 3.1-norm),
      1.3 ns per wavefront; where the bytes dominate, uneven sequences make uneven splits, which
      the balanced cut does not have: up to 15 % more with the bytes' share.
    * 0, balanced (fused step + merge): 7.6 us, 0.17 us per piece the merge folds for the longest
      sequence (up to 36; 0.06 us where a step of few rows shares a long row out among several
      workgroups), 3.4 ns + 0.26 ns per query head for every sequence, and the bytes at
      6.8 MB/us against the chain inside one of the 256 chunks; a tenth more with over 8 query
      heads per kv head (two column tiles, twice the rows to merge)."""
    steps = max(1, page_size // PAGE_SIZE)                 # the kernels step by 16 tokens
    chain = max_pages * steps
    total = total_pages * steps
    nbytes = float(total_pages) * page_size * token_bytes
    num_q_heads = num_kv_heads * heads_per_kv_head
    slices = (heads_per_kv_head + 15) // 16                # wavefronts per kv head
    norm = lambda p, *xs: sum(x ** p for x in xs) ** (1.0 / p)
    lone = batch * num_kv_heads * slices                   # wavefronts of a launch with one per sequence
    pieces = chain / max(1.0, total / 256.0)
    # rows of more than 16 pieces are merged by several workgroups each while the step has few rows
    per_piece = 0.057 if pieces > 16 and batch * num_q_heads <= 256 else 0.170
    estimates = {
        0: (7.6 + per_piece * min(pieces, 36.0) + (3.4e-3 + 2.6e-4 * num_q_heads) * batch
            + norm(2.0, nbytes / 6.81e6, 0.82 * ((total + 255) // 256))) * (1.1 if heads_per_kv_head > 8 else 1.0),
        1: 4.27 + norm(3.6, 0.584 * chain * (1.0 + 0.49 * min(1.0, lone / 2048.0)), 2.9e-3 * lone, nbytes / 5.70e6),
    }
    for n in SPLIT_COUNTS:
        wavefronts = batch * n * num_kv_heads * slices
        if wavefronts > 2048:
            continue
        split_chain = 0.634 * ((chain + n - 1) // n)
        stream = nbytes / 6.06e6
        estimates[n] = ((6.76 + norm(3.1, split_chain, stream) + 1.3e-3 * wavefronts)
                        * (1.0 + 0.15 * stream / (split_chain + stream)))
    return estimates


def decode_schedule(batch: int, num_kv_heads: int, max_pages: int, total_pages: int, token_bytes: int,
                    page_size: int = PAGE_SIZE, heads_per_kv_head: int = 8, current: Optional[int] = None,
                    hysteresis: float = 1.0) -> int:
    """Which decode schedule a step should take, from what the host knows about it: 0 = balanced,
    1 = one wavefront per (sequence, kv head) in one launch, 4 / 8 / 16 = that many splits per
    sequence and the merge launch: the smallest of ``decode_schedule_estimates``. Choosing by this
    rule is 1.1 % slower on average than always choosing the fastest schedule on the measured
    shapes (30 % at worst; 1.3 to 1.7 % and 27 to 32 % on three head layouts the constants were not
    fitted on); always balanced is 19 % slower on average. ``current``: the schedule
    in use; another must be estimated ``hysteresis`` times faster to replace it."""
    if batch <= 0 or total_pages <= 0 or max_pages <= 0:
        return 0
    estimates = decode_schedule_estimates(batch, num_kv_heads, max_pages, total_pages, token_bytes, page_size,
                                          heads_per_kv_head)
    if current in estimates:
        estimates[current] /= hysteresis
    return min(estimates, key=estimates.get)


class DecodePlan:
    """Per-step decision how the batch's pages are attended, shared by every layer of the step.

    Balanced schedule (default): the cut of the batch's pages into equal chunks (one launch), the
    device plan buffer (chunk entries) and the partial-result workspace. Launches that share a
    plan share its workspace and must run one after the other (same stream).
    Per-sequence schedule (``per_sequence`` True, see ``choose_schedule``): no cut to build;
    ``decode_step`` then runs ``splits`` wavefronts per (sequence, kv head), the append fused in,
    and with more than one split the merge launch over ``split_workspace``.
    """

    def __init__(self, block_table: torch.Tensor, seq_lens: torch.Tensor, num_q_heads: int,
                 num_kv_heads: int, num_pages: int, chunks: Optional[int] = None,
                 page_size: int = PAGE_SIZE, shared_pages: int = 0,
                 host_seq_lens: Optional[Sequence[int]] = None, token_bytes: Optional[int] = None,
                 kv_dtype: Optional[torch.dtype] = None):
        """``shared_pages``: leading block-table entries that are the same physical pages in every
        row (a shared cached prefix); they are then attended once for the whole batch.
        ``host_seq_lens``: the lengths as the host knows them; with them the plan picks the
        per-sequence schedule (and its split count) where ``decode_schedule`` says so. ``token_bytes``:
        K + V bytes of one token in the pool (default: fp16). ``kv_dtype``: the pool's element type
        (default fp16); with a shared prefix it decides how the default chunk count is chosen."""
        lib = _lib.load()
        self.shared_pages = int(shared_pages)
        self.kv_dtype = kv_dtype
        self.per_sequence = False
        self.splits = 1
        self.split_workspace: Optional[torch.Tensor] = None
        self.token_bytes = int(token_bytes) if token_bytes is not None else 2 * int(num_kv_heads) * HEAD_DIM * 2
        _need(0 <= self.shared_pages <= block_table.shape[1], "shared_pages out of range")
        _need(block_table.dim() == 2, "block_table must be [B, max_blocks]")
        self.block_table = _dev_i32("block_table", block_table)
        self.seq_lens = _dev_i32("seq_lens", seq_lens)
        self.batch = int(self.block_table.shape[0])
        _need(self.seq_lens.numel() == self.batch, "seq_lens must be [B]")
        self.num_q_heads, self.num_kv_heads = int(num_q_heads), int(num_kv_heads)
        self.num_pages, self.page_size = int(num_pages), int(page_size)
        self.bt_stride = int(self.block_table.stride(0))
        if chunks is not None:
            self.chunks = int(chunks)
        elif self.shared_pages > 0 and block_table.shape[0] > 0:
            self.chunks = prefix_chunks(block_table.shape[0], num_q_heads, num_kv_heads, self.shared_pages, page_size,
                                        fp16_pool=kv_dtype in (None, torch.float16))
        else:
            self.chunks = balanced_chunks(num_kv_heads)
        dev = self.block_table.device
        self.plan_bytes = int(lib.litekv_decode_plan_bytes_paged(self.batch, self.bt_stride, self.num_kv_heads,
                                                                 self.chunks, self.page_size))
        _need(self.plan_bytes > 0 or self.batch == 0, f"page_size {self.page_size} unsupported (16, 32, 64, 128 or 256)")
        self.buffer = torch.empty(max(4, self.plan_bytes // 4), dtype=torch.int32, device=dev)
        ws_fn = (lib.litekv_paged_decode_prefix_workspace_bytes if self.shared_pages > 0
                 else lib.litekv_paged_decode_balanced_workspace_bytes)
        ws_bytes = int(ws_fn(self.batch, self.num_q_heads, HEAD_DIM, self.chunks))
        self.workspace = torch.empty(max(4, ws_bytes // 4), dtype=torch.float32, device=dev)
        self.workspace_bytes = ws_bytes
        if host_seq_lens is not None:
            self.choose_schedule(host_seq_lens)
        self.refresh()

    def set_schedule(self, splits: int) -> None:
        """0: balanced; otherwise the per-sequence schedule with that many splits per sequence
        (the partial-result buffer of several splits is allocated here, not at the launch)."""
        self.per_sequence = splits > 0
        self.splits = max(1, int(splits))
        if self.splits > 1:
            need = int(_lib.load().litekv_paged_decode_workspace_bytes(self.batch, self.num_q_heads, HEAD_DIM,
                                                                       self.splits)) // 4
            if self.split_workspace is None or self.split_workspace.numel() < need:
                self.split_workspace = torch.empty(need, dtype=torch.float32, device=self.block_table.device)

    @property
    def schedule(self) -> int:
        """0 on the balanced schedule, else the splits per sequence."""
        return self.splits if self.per_sequence else 0

    def choose_schedule(self, host_seq_lens: Sequence[int], hysteresis: float = 1.0) -> bool:
        """Sets the schedule from the lengths as the host knows them (no device read): see
        ``decode_schedule``; the schedule in use keeps a ``hysteresis`` advantage. A plan with a
        shared prefix stays balanced. Returns ``per_sequence``."""
        if self.shared_pages > 0:
            self.set_schedule(0)
            return False
        pages = [(int(n) + self.page_size - 1) // self.page_size for n in host_seq_lens if n > 0]
        if not pages:
            self.set_schedule(0)
            return False
        self.set_schedule(decode_schedule(self.batch, self.num_kv_heads, max(pages), sum(pages), self.token_bytes,
                                          self.page_size, self.num_q_heads // self.num_kv_heads,
                                          current=self.schedule, hysteresis=hysteresis))
        return self.per_sequence

    def refresh(self, block_table: Optional[torch.Tensor] = None, seq_lens: Optional[torch.Tensor] = None) -> None:
        """Recomputes the cuts after the tables or lengths changed (same shapes). Nothing to do
        while the plan is on the per-sequence schedule."""
        if block_table is not None:
            bt = _dev_i32("block_table", block_table)
            _need(bt.shape == self.block_table.shape and bt.stride(0) == self.bt_stride, "block_table shape changed")
            self.block_table = bt
        if seq_lens is not None:
            sl = _dev_i32("seq_lens", seq_lens)
            _need(sl.numel() == self.batch, "seq_lens shape changed")
            self.seq_lens = sl
        if self.per_sequence:
            return
        lib = _lib.load()
        _lib.check(lib.litekv_decode_plan_prefix(_ptr(self.block_table), self.bt_stride, _ptr(self.seq_lens),
                                                 self.batch, self.num_kv_heads, self.page_size, self.num_pages,
                                                 self.chunks, self.shared_pages, _ptr(self.buffer),
                                                 self.plan_bytes, _stream()))


def _fixed(name: str, t: Optional[torch.Tensor], dtype: torch.dtype, numel: Optional[int] = None) -> None:
    """An output (or in/out) tensor must already have its final form: nothing is cast or copied."""
    if t is None:
        return
    _need(t.is_cuda and t.dtype == dtype and t.is_contiguous(), f"{name} must be a contiguous {dtype} GPU tensor")
    _need(numel is None or t.numel() == numel, f"{name} must hold {numel} elements")


def decode_advance(request_tables: torch.Tensor, request_ids: torch.Tensor, seq_lens: torch.Tensor,
                   slot_mapping: torch.Tensor, block_table: torch.Tensor, num_pages: int,
                   capacity: Optional[torch.Tensor] = None, seq_lens_i64: Optional[torch.Tensor] = None,
                   position_ids: Optional[torch.Tensor] = None, overflow: Optional[torch.Tensor] = None,
                   page_size: int = PAGE_SIZE, increment: int = 1) -> None:
    """One decode step of metadata on the device, in place: seq_lens += increment, slot_mapping[b] =
    slot of logical token seq_lens[b] - 1 in request request_ids[b]'s page list (a row of
    request_tables [max_requests, max_pages]), position_ids[b] = seq_lens[b] - 1, and block_table
    [B, width] = the batch's page lists. Rows that cannot advance (capacity reached, bad request id)
    raise the overflow flag and end empty for good (length -1, slot -1): every kernel of the path
    treats them as holding no tokens, so the step's append never lands on a cached token."""
    _need(request_tables.dim() == 2 and request_tables.stride(1) == 1, "request_tables must be [max_requests, max_pages]")
    _fixed("request_tables", request_tables, torch.int32)
    b = request_ids.numel()
    _fixed("request_ids", request_ids, torch.int32)
    _fixed("seq_lens", seq_lens, torch.int32, b)
    _fixed("slot_mapping", slot_mapping, torch.int32, b)
    _fixed("capacity", capacity, torch.int32, b)
    _fixed("seq_lens_i64", seq_lens_i64, torch.int64, b)
    _fixed("position_ids", position_ids, torch.int64, b)
    _fixed("overflow", overflow, torch.int32, 1)
    _need(block_table.is_cuda and block_table.dtype == torch.int32 and block_table.dim() == 2
          and block_table.shape[0] == b and block_table.stride(1) == 1, "block_table must be int32 [B, width] on the GPU")
    width = int(block_table.shape[1])
    _need(width <= request_tables.shape[1], "block_table is wider than request_tables")
    lib = _lib.load()
    _lib.check(lib.litekv_decode_advance(
        _ptr(request_tables), request_tables.stride(0), request_tables.shape[0], _ptr(request_ids), _ptr(capacity),
        _ptr(seq_lens), _ptr(seq_lens_i64), _ptr(slot_mapping), _ptr(position_ids), _ptr(block_table),
        block_table.stride(0) if b > 1 else max(block_table.stride(0), width), width, _ptr(overflow), b,
        int(page_size), int(num_pages), int(increment), _stream()))


def decode_step(q: torch.Tensor, kv_pool: torch.Tensor, plan: DecodePlan,
                k_new: Optional[torch.Tensor] = None, v_new: Optional[torch.Tensor] = None,
                softmax_scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                kv_scales: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One layer of a decode step under ``plan``. Balanced schedule: optional append of k_new / v_new
    ([B, Hkv, D]) at logical position seq_lens[b] - 1 fused into the attention of q [B, Hq, D] over
    the planned pages, then the merge of the sequences that span several chunks. Per-sequence
    schedule (``plan.per_sequence``): the same by ``plan.splits`` wavefronts per (sequence, kv
    head); one launch and no merge with one split. An fp8 pool (uint8 / float8_e4m3fn) comes with
    its per-head ``kv_scales``."""
    if plan.per_sequence:
        return paged_decode(q, kv_pool, plan.block_table, plan.seq_lens, softmax_scale, num_splits=plan.splits,
                            out=out, workspace=plan.split_workspace if plan.splits > 1 else None,
                            page_size=plan.page_size, schedule="splits", kv_scales=kv_scales,
                            k_new=k_new, v_new=v_new)
    _dev_half("q", q)
    fp8 = is_quantised_pool(kv_pool)
    if not fp8:
        _dev_half("kv_pool", kv_pool)
    _need(q.dim() == 3 and q.stride(2) == 1 and q.stride(1) == q.shape[2], "q must be [B, Hq, D] with contiguous heads")
    b, hq, d = q.shape
    _, hkv, dk, n_pages, _ = pool_geometry(kv_pool, plan.page_size)
    _need(d == dk, "q and kv_pool differ in head_dim")
    _need((b, hq, hkv, n_pages) == (plan.batch, plan.num_q_heads, plan.num_kv_heads, plan.num_pages),
          "plan was made for another batch / head / pool geometry")
    _need((k_new is None) == (v_new is None), "k_new and v_new go together")
    kn_stride = vn_stride = 0
    if k_new is not None:
        _dev_half("k_new", k_new), _dev_half("v_new", v_new)
        _need(k_new.shape == (b, hkv, d) and v_new.shape == (b, hkv, d), "k_new / v_new must be [B, Hkv, D]")
        kn_stride, vn_stride = _rows("k_new", k_new), _rows("v_new", v_new)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    if out is None:
        out = torch.empty((b, hq, d), dtype=torch.float16, device=q.device)
    else:
        _dev_half("out", out)
        _need(out.shape == (b, hq, d) and out.is_contiguous(), "out must be contiguous [B, Hq, D]")
    q_stride = q.stride(0) if b > 1 else max(q.stride(0), hq * d)
    lib = _lib.load()
    if fp8:
        _dev_fp8_pool(kv_pool, kv_scales, hkv)
        if plan.shared_pages > 0:
            _lib.check(_q8_entry(lib, "paged_decode_prefix", kv_pool)(
                _ptr(q), q_stride, _ptr(kv_pool), _ptr(kv_scales), _ptr(plan.block_table), _ptr(plan.seq_lens),
                _ptr(plan.buffer), plan.plan_bytes, _ptr(k_new), _ptr(v_new), kn_stride, vn_stride, _ptr(out),
                _ptr(plan.workspace), plan.workspace_bytes, b, hq, hkv, d, plan.page_size, n_pages, plan.bt_stride,
                plan.chunks, plan.shared_pages, float(softmax_scale), _stream()))
            return out
        _lib.check(_q8_entry(lib, "paged_decode_balanced", kv_pool)(
            _ptr(q), q_stride, _ptr(kv_pool), _ptr(kv_scales), _ptr(plan.seq_lens), _ptr(plan.buffer),
            plan.plan_bytes, _ptr(k_new), _ptr(v_new), kn_stride, vn_stride, _ptr(out), _ptr(plan.workspace),
            plan.workspace_bytes, b, hq, hkv, d, plan.page_size, n_pages, plan.bt_stride, plan.chunks,
            float(softmax_scale), _stream()))
        return out
    if plan.shared_pages > 0:
        _lib.check(lib.litekv_paged_decode_prefix(
            _ptr(q), q_stride, _ptr(kv_pool), _ptr(plan.block_table), _ptr(plan.seq_lens), _ptr(plan.buffer),
            plan.plan_bytes, _ptr(k_new), _ptr(v_new), kn_stride, vn_stride, _ptr(out), _ptr(plan.workspace),
            plan.workspace_bytes, b, hq, hkv, d, plan.page_size, n_pages, plan.bt_stride, plan.chunks,
            plan.shared_pages, float(softmax_scale), _stream()))
        return out
    _lib.check(lib.litekv_paged_decode_balanced(
        _ptr(q), q_stride, _ptr(kv_pool), _ptr(plan.seq_lens), _ptr(plan.buffer), plan.plan_bytes,
        _ptr(k_new), _ptr(v_new), kn_stride, vn_stride, _ptr(out), _ptr(plan.workspace), plan.workspace_bytes,
        b, hq, hkv, d, plan.page_size, n_pages, plan.bt_stride, plan.chunks, float(softmax_scale), _stream()))
    return out


_STAGES = ("both", "split", "merge")


def paged_decode(q: torch.Tensor, kv_pool: torch.Tensor, block_table: torch.Tensor,
                 seq_lens: torch.Tensor, softmax_scale: Optional[float] = None,
                 num_splits: Optional[int] = None, min_pages_per_split: Optional[int] = None,
                 max_splits: Optional[int] = None, out: Optional[torch.Tensor] = None,
                 workspace: Optional[torch.Tensor] = None, page_size: int = PAGE_SIZE,
                 stage: str = "both", schedule: Optional[str] = None,
                 chunks: Optional[int] = None, plan: Optional[DecodePlan] = None,
                 shared_pages: int = 0, kv_scales: Optional[torch.Tensor] = None,
                 k_new: Optional[torch.Tensor] = None, v_new: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Decode attention of q [B, Hq, D] over the pages named by block_table [B, max_blocks].

    ``shared_pages`` (balanced schedule): the first that many entries of every block-table row are
    the same physical pages; they are attended once for the whole batch.

    schedule "balanced" (default): all pages of the batch are cut into `chunks` equal pieces per
    kv head (default: one workgroup per CU); a DecodePlan is built for the call unless one is
    passed. schedule "splits" (chosen when num_splits, max_splits or min_pages_per_split is
    given): every sequence is cut into its own splits; two launches (`stage` selects one).
    An fp8 pool comes with its ``kv_scales``; either schedule reads it.
    ``k_new`` / ``v_new`` [B, Hkv, D] (splits schedule, both stages): the step's new token of every
    sequence is written at logical position seq_lens[b] - 1 by the same launch and attended.
    """
    _dev_half("q", q)
    if not is_quantised_pool(kv_pool):
        _dev_half("kv_pool", kv_pool)
    _need(q.dim() == 3 and q.stride(2) == 1 and q.stride(1) == q.shape[2], "q must be [B, Hq, D] with contiguous heads")
    b, hq, d = q.shape
    _, hkv, dk, n_pages, _ = pool_geometry(kv_pool, page_size)
    _need(d == dk, "q and kv_pool differ in head_dim")
    _need(stage in _STAGES, f"unknown stage {stage!r}")
    if schedule is None:
        split_args = (num_splits, max_splits, min_pages_per_split)
        schedule = "splits" if any(x is not None for x in split_args) or stage != "both" else "balanced"
    _need(schedule in ("balanced", "splits"), f"unknown schedule {schedule!r}")

    _need((k_new is None) == (v_new is None), "k_new and v_new go together")
    if schedule == "balanced":
        _need(stage == "both", "the balanced schedule is a single launch")
        _need(k_new is None, "the balanced schedule appends through decode_step")
        if plan is None:
            plan = DecodePlan(block_table, seq_lens, hq, hkv, n_pages, chunks, page_size, shared_pages,
                              kv_dtype=kv_pool.dtype)
        return decode_step(q, kv_pool, plan, None, None, softmax_scale, out, kv_scales)

    fp8 = is_quantised_pool(kv_pool)
    if fp8:
        _dev_fp8_pool(kv_pool, kv_scales, hkv)
        _need(stage == "both", "an fp8 pool is read by both stages in one call")
    _need(block_table.dim() == 2 and block_table.shape[0] == b, "block_table must be [B, max_blocks]")
    block_table = _dev_i32("block_table", block_table)
    seq_lens = _dev_i32("seq_lens", seq_lens)
    _need(seq_lens.numel() == b, "seq_lens must be [B]")
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    if out is None:
        out = torch.empty((b, hq, d), dtype=torch.float16, device=q.device)
    else:
        _dev_half("out", out)
        _need(out.shape == (b, hq, d) and out.is_contiguous(), "out must be contiguous [B, Hq, D]")
    lib = _lib.load()
    q_stride = q.stride(0) if b > 1 else max(q.stride(0), hq * d)
    if max_splits is None or min_pages_per_split is None:
        s, pps = decode_split_plan(b, hkv, block_table.shape[1], num_splits)
        max_splits = s if max_splits is None else max_splits
        min_pages_per_split = pps if min_pages_per_split is None else min_pages_per_split
    if workspace is None:
        workspace = decode_workspace(b, hq, max_splits, q.device)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    if k_new is not None:
        _need(stage == "both", "the fused append belongs to the call that runs both stages")
        _dev_half("k_new", k_new), _dev_half("v_new", v_new)
        _need(k_new.shape == (b, hkv, d) and v_new.shape == (b, hkv, d), "k_new / v_new must be [B, Hkv, D]")
        rows = (_ptr(k_new), _ptr(v_new), _rows("k_new", k_new), _rows("v_new", v_new))
        tail = (_ptr(out), _ptr(workspace), ws_bytes, b, hq, hkv, d, page_size, n_pages, max_splits,
                min_pages_per_split, float(softmax_scale), _stream())
        if fp8:
            _lib.check(_q8_entry(lib, "paged_decode_append", kv_pool)(_ptr(q), q_stride, _ptr(kv_pool), _ptr(kv_scales),
                                                          _ptr(block_table), block_table.stride(0), _ptr(seq_lens),
                                                          *rows, *tail))
        else:
            _lib.check(lib.litekv_paged_decode_append(_ptr(q), q_stride, _ptr(kv_pool), _ptr(block_table),
                                                      block_table.stride(0), _ptr(seq_lens), *rows, *tail))
    elif fp8:
        _lib.check(_q8_entry(lib, "paged_decode", kv_pool)(_ptr(q), q_stride, _ptr(kv_pool), _ptr(kv_scales), _ptr(block_table),
                                               block_table.stride(0), _ptr(seq_lens), _ptr(out), _ptr(workspace),
                                               ws_bytes, b, hq, hkv, d, page_size, n_pages, max_splits,
                                               min_pages_per_split, float(softmax_scale), _stream()))
    elif stage in ("both", "split"):
        fn = lib.litekv_paged_decode if stage == "both" else lib.litekv_paged_decode_split
        _lib.check(fn(_ptr(q), q_stride, _ptr(kv_pool), _ptr(block_table), block_table.stride(0),
                      _ptr(seq_lens), _ptr(out), _ptr(workspace), ws_bytes, b, hq, hkv, d, page_size,
                      n_pages, max_splits, min_pages_per_split, float(softmax_scale), _stream()))
    else:
        _lib.check(lib.litekv_paged_decode_merge(_ptr(seq_lens), _ptr(out), _ptr(workspace), ws_bytes, b,
                                                 hq, d, page_size, max_splits, min_pages_per_split,
                                                 _stream()))
    return out


def paged_decode_static(q: torch.Tensor, kv_pool: torch.Tensor, block_table: torch.Tensor,
                        seq_lens: torch.Tensor, out: torch.Tensor, max_splits: int,
                        min_pages_per_split: int, softmax_scale: Optional[float] = None,
                        page_size: int = PAGE_SIZE) -> torch.Tensor:
    """``paged_decode`` on the splits schedule without any allocation: ``out`` comes from the
    caller, index tensors must already be int32 on the device, and the partial results live in
    the scratch array built into the library (at most STATIC_SCRATCH_BYTES of them, else
    LiteKVError). Calls that overlap in time on one GPU share that array and race."""
    _dev_half("q", q), _dev_half("kv_pool", kv_pool), _dev_half("out", out)
    _need(q.dim() == 3 and q.stride(2) == 1 and q.stride(1) == q.shape[2], "q must be [B, Hq, D] with contiguous heads")
    b, hq, d = q.shape
    _, hkv, dk, n_pages, _ = pool_geometry(kv_pool, page_size)
    _need(d == dk, "q and kv_pool differ in head_dim")
    _need(out.shape == (b, hq, d) and out.is_contiguous(), "out must be contiguous [B, Hq, D]")
    for name, t in (("block_table", block_table), ("seq_lens", seq_lens)):
        _need(t.is_cuda and t.dtype == torch.int32, f"{name} must be an int32 device tensor")
    _need(block_table.dim() == 2 and block_table.shape[0] == b and block_table.stride(1) == 1,
          "block_table must be [B, max_blocks]")
    _need(seq_lens.numel() == b and seq_lens.is_contiguous(), "seq_lens must be contiguous [B]")
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    q_stride = q.stride(0) if b > 1 else max(q.stride(0), hq * d)
    _lib.check(_lib.load().litekv_paged_decode_static(
        _ptr(q), q_stride, _ptr(kv_pool), _ptr(block_table), block_table.stride(0), _ptr(seq_lens),
        _ptr(out), b, hq, hkv, d, page_size, n_pages, int(max_splits), int(min_pages_per_split),
        float(softmax_scale), _stream()))
    return out


def paged_prefill(q: torch.Tensor, kv_pool: torch.Tensor, block_table: torch.Tensor,
                  cu_q_lens: torch.Tensor, context_lens: Optional[torch.Tensor], max_q_len: int,
                  softmax_scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                  page_size: int = PAGE_SIZE, kv_scales: Optional[torch.Tensor] = None,
                  key_slices: Optional[int] = None, max_kv_len: Optional[int] = None,
                  workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal varlen attention of packed q [T, Hq, D] over paged KV (history + the chunk itself).
    An fp8 pool (uint8 / float8_e4m3fn) comes with its per-head ``kv_scales``.

    A launch with too few query rows to fill the device (one request's chunk over a long history)
    is cut along the keys as well: ``key_slices`` workgroups per row block and a merge launch
    (head_dim 64 / 128, any pool format). None lets the library choose from the launch shape and
    ``max_kv_len`` (the most keys a row sees: history + chunk, as the host knows it; without it
    the launch is not cut); 1 switches it off. ``workspace`` (float32, see ``paged_prefill_workspace_floats``) is
    allocated when not given."""
    _dev_half("q", q)
    fp8 = is_quantised_pool(kv_pool)
    if not fp8:
        _dev_half("kv_pool", kv_pool)
        _need(kv_scales is None, "kv_scales belong to an fp8 pool")
    q_stride = _rows("q", q)
    t, hq, d = q.shape
    _, hkv, dk, n_pages, _ = pool_geometry(kv_pool, page_size)
    if fp8:
        _dev_fp8_pool(kv_pool, kv_scales, hkv)
    _need(d == dk, "q and kv_pool differ in head_dim")
    cu_q_lens = _dev_i32("cu_q_lens", cu_q_lens)
    b = cu_q_lens.numel() - 1
    _need(block_table.dim() == 2 and block_table.shape[0] == b, "block_table must be [B, max_blocks]")
    block_table = _dev_i32("block_table", block_table)
    if context_lens is not None:
        context_lens = _dev_i32("context_lens", context_lens)
        _need(context_lens.numel() == b, "context_lens must be [B]")
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    if out is None:
        out = torch.empty((t, hq, d), dtype=torch.float16, device=q.device)
    lib = _lib.load()
    if key_slices is None:
        # a workgroup takes 128 (row, head) columns: beyond 512 of them the device is full as it is;
        # and without the lengths on the host there is nothing to choose by (what the block table
        # could name says little: a fresh prompt cut into eight slices takes twice as long)
        few_rows = 0 < t * hq <= 128 * 512 and max_kv_len is not None
        key_slices = int(lib.litekv_paged_prefill_key_slices(b, hq, hkv, d, int(max_q_len), int(max_kv_len))) if few_rows else 1
    key_slices = int(key_slices)
    if key_slices > 1:
        need = paged_prefill_workspace_floats(t, hq, d, key_slices)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.float32, device=q.device)
        _need(workspace.is_cuda and workspace.dtype == torch.float32 and workspace.is_contiguous() and
              workspace.numel() >= need, f"workspace must be {need} contiguous float32 on the device")
    if fp8:
        if key_slices > 1:
            _lib.check(lib.litekv_paged_prefill_split_q8(
                _ptr(q), q_stride, _ptr(kv_pool), _ptr(kv_scales), 1 if is_int8_pool(kv_pool) else 0,
                _ptr(block_table), block_table.stride(0), _ptr(cu_q_lens), _ptr(context_lens), _ptr(out),
                _rows("out", out), b, hq, hkv, d, page_size, n_pages, int(max_q_len), t, key_slices,
                _ptr(workspace), workspace.numel() * 4, float(softmax_scale), _stream()))
            return out
        _lib.check(_q8_entry(lib, "paged_prefill", kv_pool)(_ptr(q), q_stride, _ptr(kv_pool), _ptr(kv_scales), _ptr(block_table),
                                                block_table.stride(0), _ptr(cu_q_lens), _ptr(context_lens),
                                                _ptr(out), _rows("out", out), b, hq, hkv, d, page_size, n_pages,
                                                int(max_q_len), float(softmax_scale), _stream()))
        return out
    if key_slices > 1:
        _lib.check(lib.litekv_paged_prefill_split(_ptr(q), q_stride, _ptr(kv_pool), _ptr(block_table),
                                                  block_table.stride(0), _ptr(cu_q_lens), _ptr(context_lens),
                                                  _ptr(out), _rows("out", out), b, hq, hkv, d, page_size, n_pages,
                                                  int(max_q_len), t, key_slices, _ptr(workspace),
                                                  workspace.numel() * 4, float(softmax_scale), _stream()))
        return out
    _lib.check(lib.litekv_paged_prefill(_ptr(q), q_stride, _ptr(kv_pool), _ptr(block_table),
                                        block_table.stride(0), _ptr(cu_q_lens), _ptr(context_lens),
                                        _ptr(out), _rows("out", out), b, hq, hkv, d, page_size, n_pages,
                                        int(max_q_len), float(softmax_scale), _stream()))
    return out


def paged_prefill_workspace_floats(num_tokens: int, num_q_heads: int, head_dim: int, key_slices: int) -> int:
    """float32 elements of the workspace a paged prefill over ``key_slices`` key slices needs."""
    nbytes = int(_lib.load().litekv_paged_prefill_split_workspace_bytes(int(num_tokens), int(num_q_heads),
                                                                        int(head_dim), int(key_slices)))
    return nbytes // 4


def varlen_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_starts: torch.Tensor,
                   seq_lens: torch.Tensor, max_seq_len: int, softmax_scale: Optional[float] = None,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal varlen attention of packed q over packed contiguous k, v ([T, Hkv, D])."""
    _dev_half("q", q), _dev_half("k", k), _dev_half("v", v)
    q_stride, k_stride, v_stride = _rows("q", q), _rows("k", k), _rows("v", v)
    t, hq, d = q.shape
    _need(k.shape == v.shape and k.shape[0] == t and k.shape[2] == d, "k/v shape mismatch")
    hkv = k.shape[1]
    seq_starts = _dev_i32("seq_starts", seq_starts)
    seq_lens = _dev_i32("seq_lens", seq_lens)
    b = seq_lens.numel()
    _need(seq_starts.numel() == b, "seq_starts and seq_lens differ in length")
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    if out is None:
        out = torch.empty((t, hq, d), dtype=torch.float16, device=q.device)
    lib = _lib.load()
    _lib.check(lib.litekv_varlen_prefill(_ptr(q), q_stride, _ptr(k), k_stride, _ptr(v), v_stride,
                                         _ptr(seq_starts), _ptr(seq_lens), _ptr(out), _rows("out", out),
                                         b, hq, hkv, d, int(max_seq_len), t, float(softmax_scale),
                                         _stream()))
    return out
