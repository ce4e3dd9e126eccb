"""GPU parity of the fp8 (E4M3FN) KV pool through the C ABI: codes written by the append and by the
append fused into decode are bit-equal to the numpy oracle's, page dequantisation is bit-equal to
decode * scale rounded to fp16, and decode attention over an fp8 pool is within the attention
tolerance of the fp32 oracle applied to the decoded pool."""

import math

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import ops
from oracle import cpu_ref, fp8
from tests.parity import assert_attention_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = 128
SCALE = 1.0 / math.sqrt(D)


def _all_halves_in_range(limit):
    halves = np.arange(0x10000, dtype=np.uint16).view(np.float16)
    keep = np.isfinite(halves) & (np.abs(halves.astype(np.float32)) <= limit)
    return halves[keep]


def test_append_codes_equal_the_oracle_for_every_fp16_input():
    print("fp8 append: every fp16 value", flush=True)
    hkv = 2
    vals = _all_halves_in_range(2000.0)                      # well past 448 * scale: saturation included
    t = (vals.size + hkv * D - 1) // (hkv * D)
    flat = np.zeros(t * hkv * D, dtype=np.float16)
    flat[:vals.size] = vals
    k = flat.reshape(t, hkv, D)
    v = k[::-1].copy()
    scales = np.array([1.0, 0.37, 3.0, 0.011], dtype=np.float32)
    slots = np.random.default_rng(0).permutation(t + 16)[:t].astype(np.int32)
    slots[5] = -1                                            # a padded row
    pool = torch.full((t + 16, 2 * hkv, D), 0x55, dtype=torch.uint8, device=DEV)
    ops.kv_append_fp8(torch.from_numpy(k).to(DEV), torch.from_numpy(v).to(DEV), torch.from_numpy(slots).to(DEV),
                      pool, torch.from_numpy(scales).to(DEV))
    torch.cuda.synchronize()
    want = np.full((t + 16, 2 * hkv, D), 0x55, dtype=np.uint8)
    fp8.kv_append(k, v, slots, want, scales)
    got = pool.cpu().numpy()
    diff = got != want
    # the sign of a zero code is free (0x00 and 0x80 decode to the same value)
    diff &= ~(((got & 0x7F) == 0) & ((want & 0x7F) == 0))
    assert int(diff.sum()) == 0, f"{int(diff.sum())} codes differ, e.g. {got[diff][:8]} vs {want[diff][:8]}"


def test_page_dequant_is_decode_times_scale():
    print("fp8 page dequant", flush=True)
    hkv, pages = 2, 6
    codes = np.arange(pages * 16 * 2 * hkv * D, dtype=np.uint32)
    codes = ((codes * 2654435761) >> 13).astype(np.uint8)   # every code many times, in no order
    codes[(codes & 0x7F) == 0x7F] = 0x3C                    # NaN codes never get written by the append
    pool = torch.from_numpy(codes.reshape(pages * 16, 2 * hkv, D)).to(DEV)
    scales = np.array([0.5, 0.013, 1.7, 0.25], dtype=np.float32)
    dst = torch.zeros((4 * 16, 2 * hkv, D), dtype=torch.float16, device=DEV)
    src_ids = torch.tensor([5, 0, 9, 2], dtype=torch.int32, device=DEV)          # 9: out of range, skipped
    ops.page_dequant(pool, dst, src_ids, None, torch.from_numpy(scales).to(DEV))
    torch.cuda.synchronize()
    full = fp8.dequantize_pool(codes.reshape(pages * 16, 2 * hkv, D), scales).astype(np.float16)
    got = dst.cpu().numpy()
    for i, page in enumerate((5, 0, None, 2)):
        block = got[16 * i: 16 * i + 16]
        if page is None:
            assert np.all(block == 0)
        else:
            assert np.array_equal(block.view(np.uint16), full[16 * page: 16 * page + 16].view(np.uint16))
    # a view of the pool as torch's float8 type is accepted too
    dst2 = torch.zeros_like(dst)
    ops.page_dequant(pool.view(torch.float8_e4m3fn), dst2, src_ids, torch.tensor([3, 2, 1, 0], dtype=torch.int32, device=DEV),
                     torch.from_numpy(scales).to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(dst2[48:64], dst[0:16]) and torch.equal(dst2[0:16], dst[48:64])


def _fp8_case(seed, lens, hq, hkv, k_scale=0.02, v_scale=0.015):
    """Random fp16 K/V quantised into a shuffled fp8 pool by the append kernel; returns what decode needs."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    b = len(lens)
    pages_per = [(n + 15) // 16 for n in lens]
    num_pages = sum(pages_per) + 7
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    width = max(1, max(pages_per))
    table = torch.zeros((b, width), dtype=torch.int32)
    slots = []
    cur = 0
    for i, n in enumerate(lens):
        ids = perm[cur:cur + pages_per[i]]
        cur += pages_per[i]
        table[i, :len(ids)] = torch.tensor(ids, dtype=torch.int32)
        slots += [ids[t // 16] * 16 + t % 16 for t in range(n)]
    total = sum(lens)
    k = torch.randn((total, hkv, D), generator=g, device=DEV, dtype=torch.float16)
    v = torch.randn((total, hkv, D), generator=g, device=DEV, dtype=torch.float16)
    scales = torch.cat([k_scale * (1 + 0.1 * torch.arange(hkv)), v_scale * (1 + 0.2 * torch.arange(hkv))]).float().to(DEV)
    pool = torch.randint(0, 0x7F, (num_pages * 16, 2 * hkv, D), generator=g, device=DEV, dtype=torch.uint8)
    ops.kv_append_fp8(k, v, torch.tensor(slots, dtype=torch.int32, device=DEV), pool, scales)
    q = torch.randn((b, hq, D), generator=g, device=DEV, dtype=torch.float16)
    return q, pool, scales, table.to(DEV), torch.tensor(lens, dtype=torch.int32, device=DEV)


def _oracle(q, pool, scales, table, lens):
    values = torch.from_numpy(fp8.dequantize_pool(pool.cpu().numpy(), scales.cpu().numpy()))
    return cpu_ref.paged_decode_ref(q.cpu(), values, table.cpu(), lens.cpu(), SCALE).numpy()


@pytest.mark.parametrize("hq,hkv", [(8, 2), (64, 8), (16, 16), (4, 1)])
def test_decode_over_an_fp8_pool_matches_the_oracle_on_the_decoded_values(hq, hkv):
    print(f"fp8 decode hq={hq} hkv={hkv}", flush=True)
    lens = [1, 16, 17, 250, 0, 999, 64]
    q, pool, scales, table, seq_lens = _fp8_case(11 + hq, lens, hq, hkv)
    out = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle(q, pool, scales, table, seq_lens), "fp8 decode")
    assert torch.all(out[4] == 0)                            # the empty sequence
    # chunk count is free: same result within tolerance, and a repeat is bit-identical
    again = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales)
    other = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales, chunks=37)
    torch.cuda.synchronize()
    assert torch.equal(out, again)
    assert_attention_close(other, _oracle(q, pool, scales, table, seq_lens), "fp8 decode, 37 chunks")


def test_quantisation_error_is_the_only_difference_from_fp16():
    """The same K/V in an fp16 pool: outputs differ by what E4M3's 3 mantissa bits allow, not more."""
    print("fp8 vs fp16 decode", flush=True)
    hq, hkv, lens = 16, 4, [300, 77]
    g = torch.Generator(device=DEV).manual_seed(5)
    k = torch.randn((sum(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    v = torch.randn((sum(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    q = torch.randn((2, hq, D), generator=g, device=DEV, dtype=torch.float16)
    # sequence 0 in pages 1..19, sequence 1 in pages 24..28
    slots = torch.cat([torch.arange(lens[0]) + 16, torch.arange(lens[1]) + 24 * 16]).to(torch.int32).to(DEV)
    table = torch.zeros((2, 20), dtype=torch.int32, device=DEV)
    table[0, :19] = torch.arange(1, 20)
    table[1, :5] = torch.arange(24, 29)
    pool16 = torch.zeros((30 * 16, 2 * hkv, D), dtype=torch.float16, device=DEV)
    pool8 = torch.zeros((30 * 16, 2 * hkv, D), dtype=torch.uint8, device=DEV)
    scales = torch.full((2 * hkv,), 6.0 / 448.0, device=DEV)                 # +-6 sigma before saturation
    ops.kv_append(k, v, slots, pool16)
    ops.kv_append_fp8(k, v, slots, pool8, scales)
    seq_lens = torch.tensor(lens, dtype=torch.int32, device=DEV)
    o16 = ops.paged_decode(q, pool16, table, seq_lens, SCALE)
    o8 = ops.paged_decode(q, pool8, table, seq_lens, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    err = (o16.float() - o8.float()).abs().max().item()
    assert 1e-4 < err < 3e-2, err                          # visibly quantised, and bounded


def test_fused_append_writes_the_same_codes_and_attends_them():
    print("fp8 decode with fused append", flush=True)
    hq, hkv = 16, 4
    lens = [33, 16, 1, 130]                                # lengths already counting the new token
    q, pool, scales, table, seq_lens = _fp8_case(23, lens, hq, hkv)
    g = torch.Generator(device=DEV).manual_seed(99)
    k_new = torch.randn((len(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    v_new = torch.randn((len(lens), hkv, D), generator=g, device=DEV, dtype=torch.float16)
    last_slots = torch.stack([table[i, (n - 1) // 16] * 16 + (n - 1) % 16 for i, n in enumerate(lens)]).int()
    separate = pool.clone()
    ops.kv_append_fp8(k_new, v_new, last_slots, separate, scales)
    want_out = ops.paged_decode(q, separate, table, seq_lens, SCALE, kv_scales=scales)
    plan = ops.DecodePlan(table, seq_lens, hq, hkv, pool.shape[0] // 16)
    fused = pool.clone()
    got_out = ops.decode_step(q, fused, plan, k_new, v_new, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(fused, separate)                    # same codes in the same slots, nothing else touched
    assert torch.equal(got_out, want_out)
    assert_attention_close(got_out, _oracle(q, fused, scales, table, seq_lens), "fp8 fused append + decode")


def test_fp8_pages_move_with_the_page_copy_and_gather_kernels():
    print("fp8 page moves", flush=True)
    q, pool, scales, table, seq_lens = _fp8_case(31, [40, 90], 8, 2)
    before = ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales)
    n_pages = pool.shape[0] // 16
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(1)).to(torch.int32).to(DEV)
    moved = torch.zeros_like(pool)
    ops.page_gather(pool, moved, torch.arange(n_pages, dtype=torch.int32, device=DEV), order)
    remapped = order[table.long()]
    after = ops.paged_decode(q, moved, remapped.int(), seq_lens, SCALE, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(before, after)


def test_argument_checks():
    q, pool, scales, table, seq_lens = _fp8_case(41, [20], 8, 2)
    with pytest.raises(ValueError, match="scales"):
        ops.paged_decode(q, pool, table, seq_lens, SCALE)
    with pytest.raises(ValueError, match="scales"):
        ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales[:3])
    with pytest.raises(ValueError, match="balanced"):
        ops.paged_decode(q, pool, table, seq_lens, SCALE, kv_scales=scales, num_splits=2)
    with pytest.raises(ValueError, match="fp8"):
        ops.kv_append_fp8(q[:, :2], q[:, :2], seq_lens, pool.half(), scales)
