"""Pins the CPU oracle (oracle/litekv_oracle.c and oracle/cpu_ref.py) before it is trusted as the
checker of the HIP kernels: closed forms, brute force on tiny inputs, library routines, invariants.
A dropped term, a wrong GQA map, a transposed K/V half or an off-by-one in the causal mask fails
at least one of these."""

import math

import numpy as np
import torch

from llama_lite_npu_amd import workloads
from oracle import c_oracle, cpu_ref


def test_half_conversion_matches_numpy_for_every_bit_pattern():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([c_oracle.half_to_float(int(b)) for b in bits[::97]], dtype=np.float32)
    w = want[::97]
    both_nan = np.isnan(w) & np.isnan(got)
    assert np.array_equal(got[~both_nan], w[~both_nan])
    for special in (0x0000, 0x8000, 0x0001, 0x03ff, 0x0400, 0x7bff, 0x7c00, 0xfc00, 0x3c00):
        assert c_oracle.half_to_float(special) == np.uint16(special).view(np.float16).astype(np.float32)


def _random_half(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(-32768, 32767, shape, generator=g, dtype=torch.int16).view(torch.float16)


def test_kv_append_is_index_assignment():
    pool = _random_half((64, 6, 8), 1)
    kv = _random_half((5, 6, 8), 2)
    idx = torch.tensor([9, 0, 63, 17, 33], dtype=torch.int32)
    want = pool.clone()
    for i, s in enumerate(idx.tolist()):
        want[s] = kv[i]
    got_c = pool.clone().numpy()
    c_oracle.kv_append(kv.numpy(), idx.numpy(), got_c)
    got_t = pool.clone()
    cpu_ref.kv_append_ref(kv, idx, got_t)
    assert np.array_equal(got_c.view(np.int16), want.numpy().view(np.int16))
    assert torch.equal(got_t.view(torch.int16), want.view(torch.int16))
    untouched = np.setdiff1d(np.arange(64), idx.numpy())
    assert np.array_equal(got_c.view(np.int16)[untouched], pool.numpy().view(np.int16)[untouched])
    # idempotent
    again = got_c.copy()
    c_oracle.kv_append(kv.numpy(), idx.numpy(), again)
    assert np.array_equal(again.view(np.int16), got_c.view(np.int16))


def test_page_gather_scatter_round_trip():
    n_pages, ps = 12, 4
    pool = _random_half((n_pages * ps, 2, 8), 3)
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(4)).to(torch.int32)
    scattered = np.zeros_like(pool.numpy())
    c_oracle.page_gather(pool.numpy(), scattered, np.arange(n_pages), perm.numpy(), page_size=ps)
    back = np.zeros_like(scattered)
    c_oracle.page_gather(scattered, back, perm.numpy(), None, page_size=ps)
    assert np.array_equal(back.view(np.int16), pool.numpy().view(np.int16))
    paged = pool.view(n_pages, ps, 2, 8)
    want = torch.zeros_like(paged)
    want[perm.long()] = paged
    assert np.array_equal(scattered.view(np.int16), want.view(n_pages * ps, 2, 8).numpy().view(np.int16))
    t = torch.zeros_like(pool)
    cpu_ref.page_gather_ref(pool, t, torch.arange(n_pages), perm, page_size=ps)
    assert torch.equal(t.view(torch.int16), want.view(n_pages * ps, 2, 8).view(torch.int16))


def _brute_decode(q, pool, table, lens, scale, ps):
    """Plain Python loops, one (sequence, head) at a time; GQA map h // (Hq / Hkv); K heads are
    pool[:, :Hkv], V heads pool[:, Hkv:]."""
    b, hq, d = q.shape
    hkv = pool.shape[1] // 2
    out = np.zeros((b, hq, d))
    for i in range(b):
        for h in range(hq):
            kvh = h // (hq // hkv)
            scores, values = [], []
            for t in range(int(lens[i])):
                slot = int(table[i][t // ps]) * ps + t % ps
                k = pool[slot, kvh].astype(np.float64)
                scores.append(float(np.dot(q[i, h].astype(np.float64), k)) * scale)
                values.append(pool[slot, hkv + kvh].astype(np.float64))
            if not scores:
                continue
            m = max(scores)
            w = [math.exp(s - m) for s in scores]
            out[i, h] = sum(wi * vi for wi, vi in zip(w, values)) / sum(w)
    return out


def test_decode_against_brute_force_tiny():
    ps, hq, hkv, d = 4, 4, 2, 8
    g = torch.Generator().manual_seed(5)
    pool = torch.randn((10 * ps, 2 * hkv, d), generator=g).half()
    q = torch.randn((3, hq, d), generator=g).half()
    table = torch.tensor([[7, 2, 9], [0, 0, 0], [4, 1, 0]], dtype=torch.int32)
    lens = torch.tensor([11, 1, 8], dtype=torch.int32)
    want = _brute_decode(q.numpy(), pool.numpy(), table.tolist(), lens.tolist(), 0.37, ps)
    for wide in (False, True):
        got = c_oracle.paged_decode(q.numpy(), pool.numpy(), table.numpy(), lens.numpy(), 0.37, page_size=ps,
                                    wide=wide)
        assert np.abs(got - want).max() < (1e-6 if wide else 2e-6)
    got_t = cpu_ref.paged_decode_ref(q, pool, table, lens, 0.37, page_size=ps, dtype=torch.float64).numpy()
    assert np.abs(got_t - want).max() < 1e-12


def test_decode_closed_forms():
    case = workloads.make_decode_case("cf", 6, [0, 30], 8, 4)
    # one token: out == v of that token (GQA: heads 2k, 2k+1 share kv head k)
    out = c_oracle.paged_decode(case.q.numpy(), case.kv_pool.numpy(), case.block_table.numpy(),
                                case.seq_lens.numpy(), case.softmax_scale)
    slot = int(case.block_table[0, 0]) * 16
    v = case.kv_pool[slot, 4:].float().numpy()
    assert np.array_equal(out[0], np.repeat(v, 2, axis=0))
    # equal keys: out == mean of V over the sequence
    n = int(case.seq_lens[1])
    slots = cpu_ref.slots_of(case.block_table[1], n, 16)
    pool = case.kv_pool.clone()
    pool[slots, :4] = pool[slots[0], :4]
    out = c_oracle.paged_decode(case.q.numpy(), pool.numpy(), case.block_table.numpy(), case.seq_lens.numpy(),
                                case.softmax_scale, wide=True)
    want = np.repeat(pool[slots, 4:].double().mean(dim=0).numpy(), 2, axis=0)
    assert np.abs(out[1] - want).max() < 1e-6


def test_c_and_torch_oracles_agree_on_c1_and_lse_is_logsumexp():
    case = workloads.config_c1()
    a, lse = c_oracle.paged_decode(case.q.numpy(), case.kv_pool.numpy(), case.block_table.numpy(),
                                   case.seq_lens.numpy(), case.softmax_scale, return_lse=True)
    b = cpu_ref.paged_decode_ref(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale)
    assert np.abs(a - b.numpy()).max() < 5e-6
    i, h = 2, 5
    slots = cpu_ref.slots_of(case.block_table[i], int(case.seq_lens[i]), 16)
    s = (case.kv_pool[slots, h // 2].double() @ case.q[i, h].double()) * case.softmax_scale
    assert abs(float(torch.logsumexp(s, 0)) - float(lse[i, h])) < 1e-5


def test_partitioned_decode_equals_one_pass_for_any_partition():
    case = workloads.make_decode_case("part", 8, [100, 257, 15], 8, 2)
    one = c_oracle.paged_decode(case.q.numpy(), case.kv_pool.numpy(), case.block_table.numpy(),
                                case.seq_lens.numpy(), case.softmax_scale, wide=True)
    for part in (16, 128, 4096):
        out, mid_o, mid_lse = c_oracle.decode_partitioned(case.q.numpy(), case.kv_pool.numpy(),
                                                          case.block_table.numpy(), case.seq_lens.numpy(),
                                                          case.softmax_scale, partition=part)
        assert np.abs(out - one).max() < 2e-6, part
    t_out, t_mid, t_lse = cpu_ref.flash_decoding_ref(case.q, case.kv_pool, case.block_table, case.seq_lens,
                                                      case.softmax_scale, partition=128)
    out, mid_o, mid_lse = c_oracle.decode_partitioned(case.q.numpy(), case.kv_pool.numpy(),
                                                      case.block_table.numpy(), case.seq_lens.numpy(),
                                                      case.softmax_scale, partition=128)
    assert np.abs(t_out.numpy() - one).max() < 5e-6
    valid = np.isfinite(mid_lse)
    assert np.abs(t_lse.numpy()[valid] - mid_lse[valid]).max() < 1e-5
    assert np.abs(t_mid.numpy() - mid_o).max() < 5e-6


def test_lse_merge_is_associative_and_order_free():
    rng = np.random.default_rng(9)
    o = rng.standard_normal((6, 16)).astype(np.float32)
    lse = rng.standard_normal(6).astype(np.float32) * 3
    full = c_oracle.lse_merge(o, lse)
    w = np.exp(lse.astype(np.float64) - lse.max())
    want = (w[:, None] * o).sum(0) / w.sum()
    assert np.abs(full - want).max() < 1e-6
    left = c_oracle.lse_merge(o[:3], lse[:3])
    right = c_oracle.lse_merge(o[3:], lse[3:])
    lse_l = np.log(np.exp(lse[:3].astype(np.float64)).sum())
    lse_r = np.log(np.exp(lse[3:].astype(np.float64)).sum())
    two = c_oracle.lse_merge(np.stack([left, right]), np.array([lse_l, lse_r], dtype=np.float32))
    assert np.abs(two - full).max() < 1e-6
    assert np.abs(c_oracle.lse_merge(o[::-1].copy(), lse[::-1].copy()) - full).max() < 1e-6


def test_prefill_matches_sdpa_and_brute_force_mask():
    case = workloads.make_prefill_case("pf", 10, [5, 33, 1, 17], 4, 2)
    pool = case.kv_pool.clone()
    cpu_ref.kv_append_ref(torch.cat([case.k, case.v], 1), case.slot_mapping, pool)
    got = c_oracle.paged_prefill(case.q.numpy(), pool.numpy(), case.block_table.numpy(), case.cu_q_lens.numpy(),
                                 None, case.softmax_scale)
    sdpa = cpu_ref.varlen_prefill_ref(case.q, case.k, case.v, case.cu_q_lens[:-1], case.seq_lens,
                                      case.softmax_scale).numpy()
    assert np.abs(got - sdpa).max() < 5e-6
    packed = c_oracle.varlen_prefill(case.q.numpy(), case.k.numpy(), case.v.numpy(), case.cu_q_lens[:-1].numpy(),
                                     case.seq_lens.numpy(), case.softmax_scale)
    assert np.abs(packed - got).max() < 1e-6
    torch_paged = cpu_ref.paged_prefill_ref(case.q, pool, case.block_table, case.cu_q_lens, None,
                                            case.softmax_scale).numpy()
    assert np.abs(torch_paged - got).max() < 5e-6
    # row m of a sequence == decode over its first m + 1 tokens
    b, m = 1, 20
    row = int(case.cu_q_lens[b]) + m
    dec = c_oracle.paged_decode(case.q[row:row + 1].numpy(), pool.numpy(), case.block_table[b:b + 1].numpy(),
                                np.array([m + 1]), case.softmax_scale)
    assert np.abs(dec[0] - got[row]).max() < 1e-6


def test_chunked_prefill_equals_rows_of_full_prefill():
    full = workloads.make_prefill_case("full", 11, [40, 23], 4, 2)
    pool = full.kv_pool.clone()
    cpu_ref.kv_append_ref(torch.cat([full.k, full.v], 1), full.slot_mapping, pool)
    whole = c_oracle.paged_prefill(full.q.numpy(), pool.numpy(), full.block_table.numpy(), full.cu_q_lens.numpy(),
                                   None, full.softmax_scale)
    ctx = np.array([25, 0], dtype=np.int32)
    chunk = full.seq_lens.numpy() - ctx
    cu = np.concatenate([[0], np.cumsum(chunk)]).astype(np.int32)
    rows = np.concatenate([np.arange(int(full.cu_q_lens[i]) + ctx[i], int(full.cu_q_lens[i + 1])) for i in range(2)])
    part = c_oracle.paged_prefill(full.q.numpy()[rows], pool.numpy(), full.block_table.numpy(), cu, ctx,
                                  full.softmax_scale)
    assert np.abs(part - whole[rows]).max() < 1e-6
    part_t = cpu_ref.paged_prefill_ref(full.q[torch.from_numpy(rows)], pool, full.block_table,
                                       torch.from_numpy(cu), torch.from_numpy(ctx), full.softmax_scale).numpy()
    assert np.abs(part_t - whole[rows]).max() < 5e-6


def test_workload_generators_are_seeded_and_consistent():
    a, b = workloads.config_c1(), workloads.config_c1()
    assert torch.equal(a.block_table, b.block_table) and torch.equal(a.q, b.q)
    assert a.seq_lens.tolist() == [38, 129, 512, 1001] and a.num_pages == 512
    pages = sorted(p for i in range(4) for p in a.block_table[i, :(int(a.seq_lens[i]) + 15) // 16].tolist())
    assert len(set(pages)) == len(pages)                      # no page is assigned twice
    c4 = workloads.config_c4(batch=4, prefix=64, lo=5, hi=40)
    n = c4.extra["n_shared"]
    assert all(torch.equal(c4.block_table[i, :n], c4.block_table[0, :n]) for i in range(4))
    assert c4.decode_bytes() > 0 and c4.append_bytes() == 4 * (2 * 4096 + 4)


# ---- QK-norm + RoPE + append (oracle/qk_epilogue.py) ---------------------------------------------

def _rows(seed, t, h, d=128):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((t, h, d)).astype(np.float16)


def _angles(seed, t, d=128):
    """cos / sin rows the way RotaryEmbedding.forward builds them: theta_i = pos * base^(-2i/d),
    both halves of the row equal (RotaryEmbedding.py:190-200)."""
    rng = np.random.default_rng(seed)
    pos = rng.integers(0, 4096, size=t).astype(np.float64)
    inv = 10000.0 ** (-np.arange(0, d, 2, dtype=np.float64) / d)
    theta = pos[:, None] * inv[None, :]
    emb = np.concatenate([theta, theta], axis=1)
    return theta, np.cos(emb).astype(np.float16), np.sin(emb).astype(np.float16)


def test_rms_norm_is_the_closed_form():
    from oracle import qk_epilogue

    x = _rows(1, 5, 3) * np.float16(3.0)
    w = (1.0 + 0.1 * np.random.default_rng(2).standard_normal(128)).astype(np.float16)
    got = qk_epilogue.rms_norm(x, w, 1e-6).astype(np.float64)
    xd = x.astype(np.float64)
    want = xd / np.sqrt((xd * xd).mean(axis=-1, keepdims=True) + 1e-6) * w.astype(np.float64)
    assert np.abs(got - want).max() <= 2.5e-3          # two fp16 roundings of O(1..4) values
    # unit weight and a row of equal entries: every output is +-1
    ones = np.full((1, 1, 128), 2.5, dtype=np.float16)
    assert np.all(qk_epilogue.rms_norm(ones, np.ones(128, np.float16), 0.0) == np.float16(1.0))
    # a missing term (no mean: sum instead) would scale by sqrt(128)
    assert abs(float(np.abs(got).mean()) / float(np.abs(want).mean()) - 1.0) < 1e-2


def test_rope_is_complex_multiplication():
    from oracle import qk_epilogue

    t, h = 7, 4
    x = _rows(3, t, h)
    theta, cos, sin = _angles(4, t)
    got = qk_epilogue.rope(x, cos, sin).astype(np.float64)
    # (x1 + i x2) * exp(i theta) with the cos / sin the kernel sees (fp16-rounded)
    z = x[..., :64].astype(np.float64) + 1j * x[..., 64:].astype(np.float64)
    rot = cos[:, None, :64].astype(np.float64) + 1j * sin[:, None, :64].astype(np.float64)
    want = np.concatenate([(z * rot).real, (z * rot).imag], axis=-1)
    assert np.abs(got - want).max() <= 2e-3            # one fp16 rounding of |x| < 4
    # pair norms survive the rotation (up to the rounding of cos / sin and of the result)
    n_in = np.abs(z)
    n_out = np.hypot(got[..., :64], got[..., 64:])
    assert np.abs(n_in - n_out).max() <= 6e-3
    # position 0: cos 1, sin 0 -> identity, bit for bit
    one, zero = np.ones((t, 128), np.float16), np.zeros((t, 128), np.float16)
    assert np.array_equal(qk_epilogue.rope(x, one, zero), x)


def test_rope_angles_add():
    from oracle import qk_epilogue

    x = _rows(5, 3, 2)
    inv = 10000.0 ** (-np.arange(0, 128, 2, dtype=np.float64) / 128)

    def rows(pos):
        th = np.asarray(pos, dtype=np.float64)[:, None] * inv[None, :]
        e = np.concatenate([th, th], axis=1)
        return np.cos(e).astype(np.float16), np.sin(e).astype(np.float16)

    c1, s1 = rows([3, 10, 100])
    c2, s2 = rows([4, 1, 28])
    c3, s3 = rows([7, 11, 128])
    twice = qk_epilogue.rope(qk_epilogue.rope(x, c1, s1), c2, s2).astype(np.float64)
    once = qk_epilogue.rope(x, c3, s3).astype(np.float64)
    assert np.abs(twice - once).max() <= 1.5e-2        # fp16 cos / sin and two result roundings


def test_qk_epilogue_append_is_index_assignment():
    from oracle import qk_epilogue

    t, hq, hkv = 6, 4, 2
    q, k, v = _rows(6, t, hq), _rows(7, t, hkv), _rows(8, t, hkv)
    _, cos, sin = _angles(9, t)
    w = np.ones(128, np.float16)
    pool = np.full((32, 2 * hkv, 128), 7.0, dtype=np.float16)
    slots = np.array([5, 31, -1, 0, 40, 17], dtype=np.int32)       # two out of range
    q_out, new_pool = qk_epilogue.qk_norm_rope_append(q, k, v, slots, pool, w, w, cos, sin, 1e-6)
    k_out = qk_epilogue.rope(qk_epilogue.rms_norm(k, w, 1e-6), cos, sin)
    assert np.array_equal(q_out, qk_epilogue.rope(qk_epilogue.rms_norm(q, w, 1e-6), cos, sin))
    for i, s in enumerate(slots):
        if 0 <= s < 32:
            assert np.array_equal(new_pool[s, :hkv], k_out[i]) and np.array_equal(new_pool[s, hkv:], v[i])
    untouched = np.setdiff1d(np.arange(32), slots)
    assert np.all(new_pool[untouched] == np.float16(7.0))
    # no norm, no rope: plain KV append (same result as the append oracle)
    _, plain = qk_epilogue.qk_norm_rope_append(q, k, v, slots, pool)
    want = pool.copy()
    c_oracle.kv_append(np.concatenate([k, v], axis=1), slots, want)
    assert np.array_equal(plain, want)


# ---- decode metadata (integer arithmetic) -------------------------------------------------------

def test_token_slots_reference_docstring_example():
    from oracle import decode_metadata

    # worked example of build_token_table (lite_llama/executor/paged_attention.py:125-129)
    got = decode_metadata.token_slots([3, 7, 12], 10, page_size=4)
    assert got.tolist() == [12, 13, 14, 15, 28, 29, 30, 31, 48, 49]


def test_decode_advance_walks_the_per_token_table():
    from oracle import decode_metadata

    rng = np.random.default_rng(11)
    ps, width, num_pages, max_req = 4, 6, 64, 5
    tables = np.zeros((max_req, width), dtype=np.int32)
    for r in range(max_req):
        tables[r] = rng.choice(num_pages, size=width, replace=False)
    # explicit per-token table, built page by page as the reference does
    per_token = np.zeros((max_req, width * ps), dtype=np.int64)
    for r in range(max_req):
        for p in range(width):
            for o in range(ps):
                per_token[r, p * ps + o] = int(tables[r, p]) * ps + o
    ids = np.array([4, 0, 2], dtype=np.int32)
    lens = np.array([1, 7, 12], dtype=np.int32)
    for step in range(8):
        new_lens, slots, pos, rows, overflow = decode_metadata.decode_advance(tables, ids, lens, None, width, ps,
                                                                              num_pages)
        assert overflow == 0
        assert new_lens.tolist() == (lens + 1).tolist()
        assert pos.tolist() == lens.tolist()                       # position of the new token = old length
        assert slots.tolist() == [per_token[r, n] for r, n in zip(ids, lens)]
        assert np.array_equal(rows, tables[ids])
        lens = new_lens
    # increment 0 recomputes for the lengths as they are
    same, slots0, pos0, _, _ = decode_metadata.decode_advance(tables, ids, lens, None, width, ps, num_pages, 0)
    assert same.tolist() == lens.tolist() and pos0.tolist() == (lens - 1).tolist()
    assert slots0.tolist() == [per_token[r, n - 1] for r, n in zip(ids, lens)]


def test_decode_advance_refused_rows_end_empty_and_stay_refused():
    from oracle import decode_metadata

    ps, width, num_pages = 4, 3, 16
    tables = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.int32)
    ids = np.array([0, 1, 7, 1], dtype=np.int32)            # 7: no such request
    lens = np.array([12, 8, 3, 0], dtype=np.int32)          # row 0 is at the table's end
    cap = np.array([12, 8, 12, 12], dtype=np.int32)         # row 1 has reached its reserved pages
    new_lens, slots, pos, rows, overflow = decode_metadata.decode_advance(tables, ids, lens, cap, width, ps, num_pages)
    assert overflow == 1
    assert new_lens.tolist() == [-1, -1, -1, 1]             # refused rows: no tokens, no slot
    assert slots.tolist() == [-1, -1, -1, 4 * 4 + 0]
    assert pos.tolist() == [0, 0, 0, 0]
    assert rows[2].tolist() == [0, 0, 0]
    # a refused row stays refused (a fresh start at length 0 would write over its first page)
    again, slots2, _, _, overflow2 = decode_metadata.decode_advance(tables, ids, new_lens, cap, width, ps, num_pages)
    assert overflow2 == 1 and again.tolist() == [-1, -1, -1, 2] and slots2.tolist() == [-1, -1, -1, 4 * 4 + 1]
    # recomputing for the lengths as they are (increment 0) refuses nothing that fits
    same, slots0, pos0, _, overflow0 = decode_metadata.decode_advance(tables, ids[:2], lens[:2], cap[:2], width, ps,
                                                                      num_pages, increment=0)
    assert overflow0 == 0 and same.tolist() == [12, 8] and slots0.tolist() == [3 * 4 + 3, 5 * 4 + 3]
    assert pos0.tolist() == [11, 7]


# ---- fp8 (E4M3FN) storage ----------------------------------------------------------------------

def test_fp8_code_values_closed_form():
    from oracle import fp8

    vals = fp8.code_values()
    assert vals[0x00] == 0.0 and vals[0x80] == 0.0 and np.signbit(vals[0x80])
    assert vals[0x01] == 2.0 ** -9 and vals[0x07] == 7 * 2.0 ** -9          # subnormals
    assert vals[0x08] == 2.0 ** -6 and vals[0x38] == 1.0 and vals[0x3C] == 1.5
    assert vals[0x7E] == 448.0 and vals[0xFE] == -448.0                      # largest finite values
    assert np.isnan(vals[0x7F]) and np.isnan(vals[0xFF])
    finite = vals[:0x7F]
    assert np.all(np.diff(finite) > 0)                                       # codes order like their values
    assert np.array_equal(vals[0x80:0xFF], -finite)


def test_fp8_encode_decode_against_torch_float8():
    import torch
    from oracle import fp8

    # every finite fp16 value in range, as the kernels see them (fp16 -> fp32)
    halves = np.arange(0x10000, dtype=np.uint16).view(np.float16)
    x = halves[np.isfinite(halves) & (np.abs(halves.astype(np.float32)) <= 448.0)].astype(np.float32)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = fp8.encode(x)
    zero = x == 0
    assert np.array_equal(got[~zero], want[~zero])
    assert np.all((got[zero] & 0x7F) == 0)
    # decode: torch's own table
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    mine = fp8.decode(codes)
    assert np.array_equal(np.isnan(ref), np.isnan(mine))
    assert np.array_equal(ref[~np.isnan(ref)], mine[~np.isnan(mine)])


def test_fp8_rounding_saturation_and_round_trip():
    from oracle import fp8

    vals = fp8.code_values()
    finite_codes = np.array([c for c in range(256) if not np.isnan(vals[c]) and c != 0x80], dtype=np.uint8)
    assert np.array_equal(fp8.encode(vals[finite_codes]), finite_codes)        # representable values are fixed points
    pos = np.sort(vals[:0x7F])
    mid = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)   # exact in fp32
    tie = fp8.encode(mid)
    assert np.all(tie % 2 == 0)                                                # ties go to the even code
    assert np.all((tie == np.arange(0x7E)) | (tie == np.arange(1, 0x7F)))
    big = np.array([449.0, 1e4, 65504.0, -500.0, np.inf, -np.inf], dtype=np.float32)
    assert fp8.encode(big).tolist() == [0x7E, 0x7E, 0x7E, 0xFE, 0x7E, 0xFE]
    rng = np.random.default_rng(3)
    x = rng.normal(scale=30.0, size=4096).astype(np.float32)
    err = np.abs(fp8.decode(fp8.encode(x)) - np.clip(x, -448, 448))
    assert np.all(err <= np.maximum(np.abs(x) * 2.0 ** -4, 2.0 ** -10))       # half a spacing of 2^-3 relative
    assert np.all(np.diff(fp8.decode(fp8.encode(np.sort(x)))) >= 0)           # monotone


def test_fp8_append_uses_the_head_scales():
    from oracle import fp8

    rng = np.random.default_rng(4)
    k = rng.normal(size=(5, 2, 128)).astype(np.float16)
    v = rng.normal(size=(5, 2, 128)).astype(np.float16)
    scales = np.array([0.01, 0.02, 0.5, 0.004], dtype=np.float32)
    pool = np.full((8, 4, 128), 0x55, dtype=np.uint8)
    fp8.kv_append(k, v, np.array([3, 0, -1, 9, 7]), pool, scales)
    assert np.all(pool[[1, 2, 4, 5, 6]] == 0x55)                               # untouched slots
    back = fp8.dequantize_pool(pool, scales)
    for t, slot in ((0, 3), (1, 0), (4, 7)):
        for h in range(2):
            want_k = np.clip(k[t, h].astype(np.float32), -448 * scales[h], 448 * scales[h])
            assert np.all(np.abs(back[slot, h] - want_k) <= np.maximum(np.abs(want_k) * 2.0 ** -4, scales[h] * 2.0 ** -10))
            want_v = np.clip(v[t, h].astype(np.float32), -448 * scales[2 + h], 448 * scales[2 + h])
            assert np.all(np.abs(back[slot, 2 + h] - want_v) <= np.maximum(np.abs(want_v) * 2.0 ** -4,
                                                                           scales[2 + h] * 2.0 ** -10))
    assert np.all(np.abs(back[3, 3]) <= 448 * 0.004 + 1e-6)                    # a small scale saturates


# ---- int8 storage ---------------------------------------------------------------------------------

def test_int8_rounding_saturation_and_round_trip():
    from oracle import int8

    every = np.arange(-127, 128, dtype=np.float32)
    assert np.array_equal(int8.encode(every), every.astype(np.int8))            # integers are fixed points
    assert np.array_equal(int8.decode(int8.encode(every)), every)
    ties = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5], dtype=np.float32)
    assert int8.encode(ties).tolist() == [0, 2, 2, 0, -2, -2, 126, -126]        # halves go to the even integer
    big = np.array([127.49, 127.5, 128.0, 1e9, -127.5, -128.0, -1e9], dtype=np.float32)
    assert int8.encode(big).tolist() == [127, 127, 127, 127, -127, -127, -127]  # -128 is never produced
    x = np.random.default_rng(5).normal(scale=60.0, size=4096).astype(np.float32)
    back = int8.decode(int8.encode(x))
    assert np.all(np.abs(back - np.clip(x, -127, 127)) <= 0.5)                  # half a step
    assert np.all(np.diff(int8.decode(int8.encode(np.sort(x)))) >= 0)           # monotone


def test_codes_of_inputs_that_are_not_finite():
    """+-Inf saturate; NaN is dropped by the clamp's maxNum (IEEE 754-2008) and stored as the most
    negative code. Stated independently of the oracle's own expression: through torch.fmax / fmin,
    which implement maxNum / minNum, and as literal codes."""
    import torch
    from oracle import fp8, int8

    x = np.array([np.nan, -np.nan, np.inf, -np.inf, 1.0], dtype=np.float32)
    assert int8.encode(x).tolist() == [-127, -127, 127, -127, 1]
    assert fp8.encode(x).tolist() == [0xFE, 0xFE, 0x7E, 0xFE, 0x38]
    t = torch.from_numpy(x)
    clamped = torch.fmin(torch.fmax(t, torch.tensor(-127.0)), torch.tensor(127.0))
    assert clamped.tolist() == [-127.0, -127.0, 127.0, -127.0, 1.0]
    # through the append: a NaN / Inf element of a row changes no other element's code
    k = np.ones((1, 1, 128), dtype=np.float16)
    k[0, 0, 5], k[0, 0, 9], k[0, 0, 11] = np.nan, np.inf, -np.inf
    for codec, dtype, lowest, highest, one in ((int8, np.int8, -127, 127, 2), (fp8, np.uint8, 0xFE, 0x7E, 0x40)):
        pool = np.zeros((1, 2, 128), dtype=dtype)
        codec.kv_append(k, k, np.array([0]), pool, np.array([0.5, 0.5], dtype=np.float32))
        row = pool[0, 0].tolist()
        assert (row[5], row[9], row[11]) == (lowest, highest, lowest)
        assert all(c == one for i, c in enumerate(row) if i not in (5, 9, 11))


def test_int8_encode_against_torch_round_and_clamp():
    """An independent statement of the same rule: torch.round (half to even) then clamp, on every fp16
    input of moderate size divided by a scale in fp32."""
    import torch
    from oracle import int8

    halves = np.arange(0x10000, dtype=np.uint16).view(np.float16)
    halves = halves[np.isfinite(halves) & (np.abs(halves.astype(np.float32)) <= 40.0)]
    for scale in (1.0, 0.37, 0.011, 3.0):
        y = halves.astype(np.float32) * (np.float32(1.0) / np.float32(scale))
        want = torch.clamp(torch.round(torch.from_numpy(y)), -127, 127).to(torch.int8).numpy()
        assert np.array_equal(int8.encode(y), want), scale


def test_int8_append_uses_the_head_scales():
    from oracle import int8

    k = np.zeros((2, 2, 128), dtype=np.float16)
    v = np.zeros((2, 2, 128), dtype=np.float16)
    k[0, 0, :4] = [0.05, -0.05, 0.126, 10.0]       # scale 0.1: 0.5 -> 0, -0.5 -> 0, 1.26 -> 1, 100 -> 100
    k[0, 1, :3] = [1.0, -3.0, 100.0]               # scale 0.5: 2, -6, 200 -> 127
    v[1, 0, :2] = [0.25, -0.75]                    # scale 0.25: 1, -3
    v[1, 1, :2] = [0.006, -2.0]                    # scale 0.004: 1.5 -> 2, -500 -> -127
    scales = np.array([0.1, 0.5, 0.25, 0.004], dtype=np.float32)
    pool = np.full((4, 4, 128), 0x55, dtype=np.int8)
    int8.kv_append(k, v, np.array([2, 0]), pool, scales)
    assert np.all(pool[[1, 3]] == 0x55)
    # the fp16 inputs are not exactly the decimals written above: 0.05 (fp16) / 0.1 (fp32) is just
    # under one half, -0.05 / 0.1 just above minus one half; both round to 0 either way
    assert pool[2, 0, :4].tolist() == [0, 0, 1, 100]
    assert pool[2, 1, :3].tolist() == [2, -6, 127]
    assert pool[0, 2, :2].tolist() == [1, -3]
    assert pool[0, 3, :2].tolist() == [2, -127]
    back = int8.dequantize_pool(pool, scales)
    assert back[2, 1, 2] == np.float32(127) * np.float32(0.5) and back[0, 3, 1] == np.float32(-127) * np.float32(0.004)
