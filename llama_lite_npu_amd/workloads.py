"""Seeded synthetic inputs for the five benchmark configurations of the paged-KV
attention path (used by bench.py and the parity tests).

Everything random comes from ``torch.Generator().manual_seed(seed)`` on the
CPU for metadata (lengths, page permutation) so block tables are identical on
every machine; bulk fp16 data (~N(0,1)) is drawn on the target device.
"Context length L, append 1 token": the pool already holds L tokens, the append
writes logical position L and decode attends over L + 1 tokens
(lite_llama/executor/model_executor.py:893-911 counts the new token in b_seq_len).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional, Sequence

import torch

PAGE_SIZE = 16
HEAD_DIM = 128


def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(int(seed))


def _randn_half(shape, seed: int, device) -> torch.Tensor:
    g = torch.Generator(device=device).manual_seed(int(seed))
    if torch.device(device).type == "cpu":
        return torch.randn(shape, generator=g, dtype=torch.float32).to(torch.float16)
    return torch.randn(shape, generator=g, dtype=torch.float16, device=device)


@dataclass
class DecodeCase:
    """One layer's decode step: append one token per sequence, then attend."""

    name: str
    num_q_heads: int
    num_kv_heads: int
    context_lens: torch.Tensor          # [B] int32 (CPU): tokens already cached
    seq_lens: torch.Tensor              # [B] int32 = context_lens + 1
    block_table: torch.Tensor           # [B, max_blocks] int32, unused entries 0
    slot_mapping: torch.Tensor          # [B] int32 slot of the appended token
    num_pages: int
    q: torch.Tensor                     # [B, Hq, D] fp16
    k_new: torch.Tensor                 # [B, Hkv, D] fp16
    v_new: torch.Tensor
    kv_pool: torch.Tensor               # [num_pages*page_size, 2*Hkv, D] fp16
    softmax_scale: float = 1.0 / math.sqrt(HEAD_DIM)
    num_splits: Optional[int] = None
    extra: dict = field(default_factory=dict)
    page_size: int = PAGE_SIZE
    head_dim: int = HEAD_DIM

    @property
    def batch(self) -> int:
        return int(self.seq_lens.numel())

    @property
    def tok_bytes(self) -> int:
        return 2 * self.num_kv_heads * self.head_dim * 2

    def decode_bytes(self) -> int:
        """Algorithmic bytes of one decode-attention launch: K/V of every attended token,
        q and out rows, the block-table entries and the lengths."""
        toks = int(self.seq_lens.sum())
        pages = int(((self.seq_lens + self.page_size - 1) // self.page_size).sum())
        return (toks * self.tok_bytes + 2 * self.batch * self.num_q_heads * self.head_dim * 2
                + pages * 4 + self.batch * 4)

    def append_bytes(self) -> int:
        return self.batch * (2 * self.tok_bytes + 4)

    def unique_decode_bytes(self) -> int:
        """decode_bytes() with every physical page counted once (pages shared between block tables
        are fetched from HBM once if the cache keeps them): the conservative figure for C4."""
        lens = self.seq_lens.cpu().tolist()
        table = self.block_table.cpu()
        fill = {}
        pages = 0
        for b, n in enumerate(lens):
            n_pages = (n + self.page_size - 1) // self.page_size
            pages += n_pages
            ids = table[b, :n_pages].tolist()
            for j, pid in enumerate(ids):
                used = min(self.page_size, n - j * self.page_size)
                if used > fill.get(pid, 0):
                    fill[pid] = used
        toks = sum(fill.values())
        return (toks * self.tok_bytes + 2 * self.batch * self.num_q_heads * self.head_dim * 2
                + pages * 4 + self.batch * 4)

    def to(self, device) -> "DecodeCase":
        kw = dict(self.__dict__)
        for key in ("context_lens", "seq_lens", "block_table", "slot_mapping", "q", "k_new", "v_new", "kv_pool"):
            kw[key] = kw[key].to(device)
        return DecodeCase(**kw)


def assign_pages(pages_per_seq: Sequence[int], num_pages: int, seed: int):
    """Consecutive chunks of a seeded permutation of the pool -> per-sequence page lists."""
    perm = torch.randperm(num_pages, generator=_gen(seed)).to(torch.int32)
    out, cur = [], 0
    for n in pages_per_seq:
        out.append(perm[cur:cur + n])
        cur += n
    assert cur <= num_pages, "pool too small"
    return out


def table_from_lists(page_lists, max_blocks: Optional[int] = None) -> torch.Tensor:
    max_blocks = max_blocks or max(1, max(len(p) for p in page_lists))
    table = torch.zeros((len(page_lists), max_blocks), dtype=torch.int32)
    for i, p in enumerate(page_lists):
        table[i, :len(p)] = p
    return table


def make_decode_case(name: str, seed: int, context_lens: Sequence[int], num_q_heads: int,
                     num_kv_heads: int, num_pages: Optional[int] = None, slack: float = 0.10,
                     device="cpu", num_splits: Optional[int] = None,
                     page_lists=None, page_size: int = PAGE_SIZE, head_dim: int = HEAD_DIM) -> DecodeCase:
    ctx = torch.tensor(list(context_lens), dtype=torch.int32)
    seq = ctx + 1
    pages = ((seq + page_size - 1) // page_size).tolist()
    if page_lists is None:
        if num_pages is None:
            num_pages = int(math.ceil(sum(pages) * (1.0 + slack)))
        page_lists = assign_pages(pages, num_pages, seed + 1)
    assert num_pages is not None
    table = table_from_lists(page_lists)
    b = len(pages)
    slot = torch.tensor(
        [int(page_lists[i][int(ctx[i]) // page_size]) * page_size + int(ctx[i]) % page_size for i in range(b)],
        dtype=torch.int32)
    return DecodeCase(
        name=name, num_q_heads=num_q_heads, num_kv_heads=num_kv_heads, context_lens=ctx, seq_lens=seq,
        block_table=table, slot_mapping=slot, num_pages=num_pages,
        q=_randn_half((b, num_q_heads, head_dim), seed + 2, device),
        k_new=_randn_half((b, num_kv_heads, head_dim), seed + 3, device),
        v_new=_randn_half((b, num_kv_heads, head_dim), seed + 4, device),
        kv_pool=_randn_half((num_pages * page_size, 2 * num_kv_heads, head_dim), seed + 5, device),
        softmax_scale=1.0 / math.sqrt(head_dim), num_splits=num_splits, page_size=page_size, head_dim=head_dim,
    ).to(device)


def uniform_lens(seed: int, n: int, lo: int, hi: int) -> list[int]:
    return torch.randint(lo, hi + 1, (n,), generator=_gen(seed)).tolist()


def config_c1(device="cpu") -> DecodeCase:
    """Qwen3-0.6B-shaped layer: B 4, contexts {37,128,511,1000}, 16 Q / 8 KV heads, 512-page pool."""
    return make_decode_case("C1 qwen3-0.6b decode", 1001, [37, 128, 511, 1000], 16, 8, num_pages=512,
                            device=device)


def config_c2(device="cpu", batch: int = 32, lo: int = 256, hi: int = 4096) -> DecodeCase:
    """Qwen3-32B decode: B 32, contexts U[256,4096], 64 Q / 8 KV heads, pool = pages + 10 %."""
    return make_decode_case("C2 qwen3-32b decode", 1002, uniform_lens(1002, batch, lo, hi), 64, 8,
                            device=device)


def config_c5(device="cpu", batch: int = 128, lo: int = 8192, hi: int = 32768) -> DecodeCase:
    """Qwen3-30B-A3B long context: B 128, contexts U[8192,32768], 32 Q / 4 KV heads, 16 splits,
    pool with 25 % holes (pool = live / 0.75, live pages scattered by a permutation)."""
    lens = uniform_lens(1005, batch, lo, hi)
    pages = sum((l + 1 + PAGE_SIZE - 1) // PAGE_SIZE for l in lens)
    return make_decode_case("C5 qwen3-30b-a3b long decode", 1005, lens, 32, 4,
                            num_pages=int(math.ceil(pages / 0.75)), device=device, num_splits=16)


def config_c4(device="cpu", batch: int = 64, prefix: int = 2048, lo: int = 64, hi: int = 512,
              private_prefix: bool = False) -> DecodeCase:
    """Prefix sharing: every block table starts with the same prefix/16 physical pages; the suffix
    U[lo,hi] lives in private pages (last one partial). ``private_prefix`` duplicates the prefix
    pages per sequence (same bytes) to check that sharing does not change the result."""
    assert prefix % PAGE_SIZE == 0
    suffix = uniform_lens(1004, batch, lo, hi)
    ctx = [prefix + s for s in suffix]
    n_shared = prefix // PAGE_SIZE
    priv = [(c + 1 + PAGE_SIZE - 1) // PAGE_SIZE - n_shared for c in ctx]
    extra_pages = batch  # one spare page per sequence: destination of the copy-on-write move
    total = n_shared * (batch if private_prefix else 1) + sum(priv) + extra_pages
    num_pages = int(math.ceil(total * 1.10))
    perm = torch.randperm(num_pages, generator=_gen(1004 + 1)).to(torch.int32)
    shared = perm[:n_shared]
    cur = n_shared
    lists, spare = [], []
    for i in range(batch):
        if private_prefix:
            own = perm[cur:cur + n_shared]
            cur += n_shared
        else:
            own = shared
        lists.append(torch.cat([own, perm[cur:cur + priv[i]]]))
        cur += priv[i]
    for i in range(batch):
        spare.append(int(perm[cur]))
        cur += 1
    case = make_decode_case("C4 prefix sharing decode", 1004, ctx, 64, 8, num_pages=num_pages,
                            device=device, page_lists=lists)
    case.extra.update(shared_pages=shared, spare_pages=torch.tensor(spare, dtype=torch.int32),
                      n_shared=n_shared, private_prefix=private_prefix)
    if private_prefix:  # make the duplicated prefix pages byte-identical to the first sequence's
        pool = case.kv_pool.view(num_pages, PAGE_SIZE, 2 * 8, HEAD_DIM)
        src = lists[0][:n_shared].to(torch.long).to(pool.device)
        for i in range(1, batch):
            pool[lists[i][:n_shared].to(torch.long).to(pool.device)] = pool[src]
    return case


@dataclass
class PrefillCase:
    """Packed varlen causal prefill: K/V of all tokens appended into pages, then attention."""

    name: str
    num_q_heads: int
    num_kv_heads: int
    seq_lens: torch.Tensor        # [B] int32 query (= chunk) lengths
    context_lens: torch.Tensor    # [B] int32 tokens already cached before the chunk
    cu_q_lens: torch.Tensor       # [B+1] int32
    block_table: torch.Tensor     # [B, max_blocks] int32
    slot_mapping: torch.Tensor    # [T] int32 slots of the chunk's tokens
    num_pages: int
    q: torch.Tensor               # [T, Hq, D]
    k: torch.Tensor               # [T, Hkv, D]
    v: torch.Tensor
    kv_pool: torch.Tensor
    softmax_scale: float = 1.0 / math.sqrt(HEAD_DIM)
    page_size: int = PAGE_SIZE
    head_dim: int = HEAD_DIM

    @property
    def batch(self) -> int:
        return int(self.seq_lens.numel())

    @property
    def max_q_len(self) -> int:
        return int(self.seq_lens.max())

    def flops(self) -> int:
        """2 * Hq * D * L * (L + 1) per sequence (QK^T and PV over the causal half) plus
        4 * Hq * D * ctx * q for the rectangular history part."""
        l = self.seq_lens.to(torch.int64)
        c = self.context_lens.to(torch.int64)
        return int((2 * self.num_q_heads * self.head_dim * (l * (l + 1) + 2 * c * l)).sum())

    def min_bytes(self) -> int:
        t = int(self.seq_lens.sum()) + int(self.context_lens.sum())
        tq = int(self.seq_lens.sum())
        return 2 * tq * self.num_q_heads * self.head_dim * 2 + t * 2 * self.num_kv_heads * self.head_dim * 2

    def to(self, device) -> "PrefillCase":
        kw = dict(self.__dict__)
        for key in ("seq_lens", "context_lens", "cu_q_lens", "block_table", "slot_mapping", "q", "k", "v",
                    "kv_pool"):
            kw[key] = kw[key].to(device)
        return PrefillCase(**kw)


def make_prefill_case(name: str, seed: int, seq_lens: Sequence[int], num_q_heads: int, num_kv_heads: int,
                      context_lens: Optional[Sequence[int]] = None, device="cpu",
                      slack: float = 0.10, page_size: int = PAGE_SIZE, head_dim: int = HEAD_DIM) -> PrefillCase:
    ql = torch.tensor(list(seq_lens), dtype=torch.int32)
    ctx = torch.zeros_like(ql) if context_lens is None else torch.tensor(list(context_lens), dtype=torch.int32)
    total = ql + ctx
    pages = ((total + page_size - 1) // page_size).tolist()
    num_pages = int(math.ceil(sum(pages) * (1.0 + slack))) + 1
    lists = assign_pages(pages, num_pages, seed + 1)
    table = table_from_lists(lists)
    cu = torch.zeros(len(pages) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(ql, 0)
    slots = []
    for i in range(len(pages)):
        t = torch.arange(int(ctx[i]), int(total[i]))
        slots.append(lists[i].to(torch.long)[t // page_size] * page_size + t % page_size)
    slot_mapping = torch.cat(slots).to(torch.int32)
    t_total = int(ql.sum())
    return PrefillCase(
        name=name, num_q_heads=num_q_heads, num_kv_heads=num_kv_heads, seq_lens=ql, context_lens=ctx,
        cu_q_lens=cu, block_table=table, slot_mapping=slot_mapping, num_pages=num_pages,
        q=_randn_half((t_total, num_q_heads, head_dim), seed + 2, device),
        k=_randn_half((t_total, num_kv_heads, head_dim), seed + 3, device),
        v=_randn_half((t_total, num_kv_heads, head_dim), seed + 4, device),
        kv_pool=_randn_half((num_pages * page_size, 2 * num_kv_heads, head_dim), seed + 5, device),
        softmax_scale=1.0 / math.sqrt(head_dim), page_size=page_size, head_dim=head_dim,
    ).to(device)


def config_c3(device="cpu", batch: int = 8, lo: int = 128, hi: int = 2048) -> PrefillCase:
    """Qwen3-32B varlen prefill: 8 sequences U[128,2048], 64 Q / 8 KV heads, context 0."""
    return make_prefill_case("C3 qwen3-32b varlen prefill", 1003, uniform_lens(1003, batch, lo, hi), 64, 8,
                             device=device)
