"""GPU parity (bit exact) of KV append, page copy and page gather, through the C ABI."""

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import ops, workloads
from oracle import c_oracle, cpu_ref
from tests.parity import assert_bit_exact

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _sentinel_pool(slots, hkv, seed):
    g = torch.Generator().manual_seed(seed)
    bits = torch.randint(-32768, 32767, (slots, 2 * hkv, 128), generator=g, dtype=torch.int16)
    return bits.view(torch.float16)


@pytest.mark.parametrize("tokens,hkv", [(1, 8), (4, 8), (33, 4), (257, 8), (5000, 8), (3, 1)])
def test_kv_append_matches_oracle(tokens, hkv):
    print(f"kv_append tokens={tokens} hkv={hkv}", flush=True)
    slots = 64 * 16
    g = torch.Generator().manual_seed(7 + tokens)
    pool = _sentinel_pool(slots, hkv, 11)
    kv = torch.randint(-32768, 32767, (tokens, 2 * hkv, 128), generator=g, dtype=torch.int16).view(torch.float16)
    if tokens <= slots:
        sel = torch.randperm(slots, generator=g)[:tokens].to(torch.int32)
    else:  # duplicates: last writer is not defined, so use a bigger pool instead
        slots = 512 * 16
        pool = _sentinel_pool(slots, hkv, 12)
        sel = torch.randperm(slots, generator=g)[:tokens].to(torch.int32)
    want = pool.clone().numpy()
    c_oracle.kv_append(kv.numpy(), sel.numpy(), want)
    want_t = pool.clone()
    cpu_ref.kv_append_ref(kv, sel, want_t)
    assert np.array_equal(want.view(np.int16), want_t.numpy().view(np.int16))

    pool_d = pool.to(DEV)
    kv_d = kv.to(DEV)
    # the reference's calling convention: halves of one concatenated tensor
    ops.kv_append(kv_d[:, :hkv], kv_d[:, hkv:], sel.to(DEV), pool_d)
    torch.cuda.synchronize()
    assert_bit_exact(pool_d, want, "kv_append (concatenated halves)")

    pool_d2 = pool.to(DEV)
    ops.kv_append(kv_d[:, :hkv].contiguous(), kv_d[:, hkv:].contiguous(), sel.to(DEV), pool_d2)
    torch.cuda.synchronize()
    assert_bit_exact(pool_d2, want, "kv_append (separate k, v)")


def test_kv_append_skips_out_of_range_slots_and_empty_batch():
    print("kv_append out-of-range", flush=True)
    pool = _sentinel_pool(32, 2, 3)
    kv = _sentinel_pool(4, 2, 4)
    sel = torch.tensor([5, -1, 32, 7], dtype=torch.int32)
    want = pool.clone()
    want[5], want[7] = kv[0], kv[3]
    pool_d = pool.to(DEV)
    ops.kv_append(kv.to(DEV)[:, :2], kv.to(DEV)[:, 2:], sel.to(DEV), pool_d)
    ops.kv_append(kv.to(DEV)[:0, :2], kv.to(DEV)[:0, 2:], sel.to(DEV)[:0], pool_d)
    torch.cuda.synchronize()
    assert_bit_exact(pool_d, want, "kv_append skip")


def test_kv_append_c1_page_crossings():
    """C1: contexts {37,128,511,1000}: 128 -> 129 opens a new page, 511 -> 512 fills one."""
    print("kv_append C1", flush=True)
    case = workloads.config_c1("cpu")
    kv = torch.cat([case.k_new, case.v_new], dim=1)
    want = case.kv_pool.clone()
    cpu_ref.kv_append_ref(kv, case.slot_mapping, want)
    for i, ctx in enumerate(case.context_lens.tolist()):
        page = int(case.block_table[i, ctx // 16])
        assert int(case.slot_mapping[i]) == page * 16 + ctx % 16
    d = case.to(DEV)
    ops.kv_append(d.k_new, d.v_new, d.slot_mapping, d.kv_pool)
    torch.cuda.synchronize()
    assert_bit_exact(d.kv_pool, want, "C1 append")
    untouched = torch.ones(case.kv_pool.shape[0], dtype=torch.bool)
    untouched[case.slot_mapping.long()] = False
    assert_bit_exact(d.kv_pool.cpu()[untouched], case.kv_pool[untouched], "C1 untouched slots")


@pytest.mark.parametrize("hkv,n_pages,n_moves", [(8, 64, 17), (4, 40, 40), (8, 300, 1)])
def test_page_gather_and_copy(hkv, n_pages, n_moves):
    print(f"page ops hkv={hkv} pages={n_pages} moves={n_moves}", flush=True)
    g = torch.Generator().manual_seed(21 + n_moves)
    src = _sentinel_pool(n_pages * 16, hkv, 5)
    dst = _sentinel_pool(n_pages * 16, hkv, 6)
    perm = torch.randperm(n_pages, generator=g).to(torch.int32)
    src_ids, dst_ids = perm[:n_moves], torch.randperm(n_pages, generator=g)[:n_moves].to(torch.int32)

    want = dst.clone().numpy()
    c_oracle.page_gather(src.numpy(), want, src_ids.numpy(), dst_ids.numpy())
    want_t = dst.clone()
    cpu_ref.page_gather_ref(src, want_t, src_ids, dst_ids)
    assert np.array_equal(want.view(np.int16), want_t.numpy().view(np.int16))
    dst_d = dst.to(DEV)
    ops.page_gather(src.to(DEV), dst_d, src_ids.to(DEV), dst_ids.to(DEV))
    torch.cuda.synchronize()
    assert_bit_exact(dst_d, want, "page_gather")

    # dst_ids None: compaction into the dense prefix
    want2 = dst.clone()
    cpu_ref.page_gather_ref(src, want2, src_ids, None)
    dst_d2 = dst.to(DEV)
    ops.page_gather(src.to(DEV), dst_d2, src_ids.to(DEV), None)
    torch.cuda.synchronize()
    assert_bit_exact(dst_d2, want2, "page_gather dense")

    # in-pool copy with disjoint sources / destinations (copy-on-write)
    half = n_pages // 2
    s_ids = perm[:min(n_moves, half)]
    d_ids = perm[half:half + s_ids.numel()]
    want3 = src.clone()
    cpu_ref.page_copy_ref(want3, s_ids, d_ids)
    pool_d = src.to(DEV)
    ops.page_copy(pool_d, s_ids.to(DEV), d_ids.to(DEV))
    torch.cuda.synchronize()
    assert_bit_exact(pool_d, want3, "page_copy")


def test_gather_of_scatter_is_identity():
    """Scatter pages by a permutation, gather them back by the same permutation: every byte returns."""
    print("page gather(scatter) == id", flush=True)
    n_pages = 96
    pool = _sentinel_pool(n_pages * 16, 8, 9).to(DEV)
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(2)).to(torch.int32).to(DEV)
    scattered = torch.zeros_like(pool)
    ops.page_gather(pool, scattered, torch.arange(n_pages, dtype=torch.int32, device=DEV), perm)
    back = torch.zeros_like(pool)
    ops.page_gather(scattered, back, perm, None)
    torch.cuda.synchronize()
    assert_bit_exact(back, pool, "gather(scatter)")
