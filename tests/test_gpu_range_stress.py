"""Range-stress parity of every attention instantiation, through the C ABI.

N(0,1) inputs keep every score within a few units of its column's maximum, so a softmax whose
running maximum follows only part of the keys still passes them. Two kinds of input here do not:

* a planted key whose score lies about 2^40 above everything before it (its probability against
  the old maximum overflows fp16, so the maximum has to follow it wherever the key sits);
* heavy-tailed inputs: a few channels of q (x48) and K (x1.6) scaled up so that the scores of one
  row span about +-40 in log2 units.

Both run over pool format {fp16, fp8, int8} x head dim {64, 128} x {balanced schedule,
per-sequence splits, fused append on either schedule, shared prefix, paged prefill, chunk over
cached history}, and over head dims 32 and 256 on the general kernel. The reference for a pool of
8-bit codes is the fp32 oracle applied to the decoded pool (codes are exact in fp16, the scale is
applied in fp32), so quantisation error is not part of the comparison.
"""

import math

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import ops, workloads
from oracle import cpu_ref, fp8, int8
from tests.parity import assert_attention_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

FORMATS = ["f16", "fp8", "int8"]
POOL_DTYPE = {"fp8": torch.uint8, "int8": torch.int8}
CODEC = {"fp8": fp8, "int8": int8}
CODE_MAX = {"fp8": 448.0, "int8": 127.0}


def _unit(d, seed):
    v = torch.randn(d, generator=torch.Generator().manual_seed(seed))
    return v / v.norm()


def _spike_gain(d):
    """|k| of a planted key: with |q| = 6 along the same direction the score is 6 * gain / sqrt(d)
    natural units = about +40 in log2 units at every head dim."""
    return 52.0 * math.sqrt(d / 128.0)


def _quantise(values, fmt, hkv):
    """values: fp16 pool [slots, 2*Hkv, D] on the device -> (pool, scales, reference values fp32 on
    the CPU). Scales: the tightest the head's largest element allows for even heads, eight times
    looser (codes use an eighth of their range, score multiplier eight times larger) for odd ones."""
    if fmt == "f16":
        return values, None, values.float().cpu()
    top = values.float().abs().amax(dim=(0, 2)).clamp_min(1e-3) / CODE_MAX[fmt]      # [2*Hkv]
    loose = torch.tensor([8.0 if h % 2 else 1.0 for h in range(2 * hkv)], device=values.device)
    scales = (top * 1.02 * loose).float().contiguous()
    pool = torch.zeros(values.shape, dtype=POOL_DTYPE[fmt], device=values.device)
    every_slot = torch.arange(pool.shape[0], dtype=torch.int32, device=values.device)
    ops.kv_append_quantised(values[:, :hkv], values[:, hkv:], every_slot, pool, scales)
    torch.cuda.synchronize()
    return pool, scales, _decoded(pool, scales, fmt)


def _decoded(pool, scales, fmt):
    if fmt == "f16":
        return pool.float().cpu()
    return torch.from_numpy(CODEC[fmt].dequantize_pool(pool.cpu().numpy(), scales.cpu().numpy()))


def _decode_ref(case, values, seq_lens=None):
    sl = case.seq_lens if seq_lens is None else seq_lens
    return cpu_ref.paged_decode_ref(case.q.cpu(), values, case.block_table.cpu(), sl.cpu(), case.softmax_scale,
                                    page_size=case.page_size).numpy()


def _slot(case, b, at):
    ps = case.page_size
    return int(case.block_table[b, at // ps]) * ps + at % ps


def _spiked_decode_case(seed, ctx, hq, hkv, d, spikes, page_lists=None, num_pages=None, page_size=16):
    """q along one direction, K/V small noise, and for every (sequence, key) of `spikes` a K row far
    along that direction in every kv head."""
    case = workloads.make_decode_case("stress", seed, ctx, hq, hkv, device=DEV, head_dim=d, page_lists=page_lists,
                                      num_pages=num_pages, page_size=page_size)
    gen = torch.Generator().manual_seed(seed + 7)
    direction = _unit(d, seed + 8)
    case.q.copy_((6.0 * direction + 0.3 * torch.randn(case.q.shape, generator=gen)).half())
    pool = 0.3 * torch.randn(case.kv_pool.shape, generator=gen)
    for b, at in spikes:
        pool[_slot(case, b, at), :hkv] += _spike_gain(d) * direction
    case.kv_pool.copy_(pool.half())
    case.k_new.copy_((0.3 * torch.randn(case.k_new.shape, generator=gen)).half())
    case.v_new.copy_((0.3 * torch.randn(case.v_new.shape, generator=gen)).half())
    return case, direction


DECODE_RUNS = ({}, {"schedule": "balanced", "chunks": 7}, {"num_splits": 1}, {"num_splits": 5})


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("spike_at", [5, 70, 301, 590])
def test_decode_spike_every_format_and_schedule(fmt, d, spike_at):
    """The planted key in the first, a middle and the last pages of a sequence (each lane group of
    its page over the four positions), under the balanced schedule and per-sequence splits."""
    print(f"stress decode spike fmt={fmt} d={d} at={spike_at}", flush=True)
    hq, hkv = 16, 2
    spikes = [(0, spike_at), (1, min(spike_at, 100)), (2, 17), (3, 0)]
    case, _ = _spiked_decode_case(2000 + spike_at + d, [599, 130, 40, 75], hq, hkv, d, spikes)
    pool, scales, values = _quantise(case.kv_pool, fmt, hkv)
    ref = _decode_ref(case, values)
    for kw in DECODE_RUNS:
        out = ops.paged_decode(case.q, pool, case.block_table, case.seq_lens, case.softmax_scale, kv_scales=scales, **kw)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"spike {fmt} d={d} at {spike_at} {kw}")


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("d", [64, 128])
def test_fused_append_of_a_spiking_row(fmt, d):
    """The step's own token is the key that scores far above the rest (and, for one sequence, an
    earlier key does while the new one does not): the row patched into the page registers by the
    fused append has to move the maximum like a row read from the pool. Both schedules."""
    print(f"stress fused append fmt={fmt} d={d}", flush=True)
    hq, hkv = 32, 4
    ctx = [37, 128, 511, 15, 16, 0, 300]
    case, direction = _spiked_decode_case(2100 + d, ctx, hq, hkv, d, [(2, 200), (6, 290)])
    for b in (0, 1, 3, 4, 5, 6):
        case.k_new[b] += (_spike_gain(d) * direction).half().to(DEV)
    pool0, scales, _ = _quantise(case.kv_pool, fmt, hkv)
    want_pool = pool0.clone()
    if fmt == "f16":
        ops.kv_append(case.k_new, case.v_new, case.slot_mapping, want_pool)
    else:
        ops.kv_append_quantised(case.k_new, case.v_new, case.slot_mapping, want_pool, scales)
    torch.cuda.synchronize()
    ref = _decode_ref(case, _decoded(want_pool, scales, fmt))
    for chunks in (None, 5):
        pool = pool0.clone()
        plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, chunks)
        out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale, kv_scales=scales)
        torch.cuda.synchronize()
        assert torch.equal(pool, want_pool), "fused append differs from the append kernel"
        assert_attention_close(out, ref, f"fused spike {fmt} d={d} balanced chunks={chunks}")
    pool = pool0.clone()
    out = ops.paged_decode(case.q, pool, case.block_table, case.seq_lens, case.softmax_scale, num_splits=1,
                           kv_scales=scales, k_new=case.k_new, v_new=case.v_new)
    torch.cuda.synchronize()
    assert torch.equal(pool, want_pool)
    assert_attention_close(out, ref, f"fused spike {fmt} d={d} per sequence")


def _shared_lists(seed, shared_pages, suffix_ctx, page_size=16):
    ctx = [shared_pages * page_size + s for s in suffix_ctx]
    priv = [(c + 1 + page_size - 1) // page_size - shared_pages for c in ctx]
    num_pages = shared_pages + sum(priv) + 7
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(seed)).to(torch.int32)
    shared, cur, lists = perm[:shared_pages], shared_pages, []
    for n in priv:
        lists.append(torch.cat([shared, perm[cur:cur + n]]))
        cur += n
    return ctx, lists, num_pages


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("where", ["prefix-first-slice", "prefix-last-slice", "suffix", "both"])
def test_shared_prefix_spike(fmt, d, where):
    """The planted key inside the shared pages (first or last key slice of the prefix kernel), inside
    a private suffix, or one in each: prefix partials and private partials then differ by 2^40 in
    weight when the merge joins them."""
    print(f"stress shared prefix fmt={fmt} d={d} spike in {where}", flush=True)
    hq, hkv, shared_pages = 16, 2, 40           # 640 shared keys: several key slices
    suffix = [0, 5, 15, 16, 40, 300]
    ctx, lists, num_pages = _shared_lists(2200 + d, shared_pages, suffix)
    spikes = []
    if where in ("prefix-first-slice", "both"):
        spikes.append((0, 37))
    if where == "prefix-last-slice":
        spikes.append((0, 630))
    if where in ("suffix", "both"):
        spikes += [(5, 640 + 250), (3, 640 + 9)]
    case, _ = _spiked_decode_case(2210 + d, ctx, hq, hkv, d, spikes, page_lists=lists, num_pages=num_pages)
    pool, scales, values = _quantise(case.kv_pool, fmt, hkv)
    ref = _decode_ref(case, values)
    for chunks in (None, 5):
        out = ops.paged_decode(case.q, pool, case.block_table, case.seq_lens, case.softmax_scale, schedule="balanced",
                               chunks=chunks, shared_pages=shared_pages, kv_scales=scales)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"shared prefix spike {fmt} d={d} {where} chunks={chunks}")
    plain = ops.paged_decode(case.q, pool, case.block_table, case.seq_lens, case.softmax_scale, schedule="balanced",
                             kv_scales=scales)
    torch.cuda.synchronize()
    assert_attention_close(plain, ref, f"shared pages undeclared {fmt} d={d} {where}")


def _prefill_ref(case, values, ctx):
    return cpu_ref.paged_prefill_ref(case.q.cpu(), values, case.block_table.cpu(), case.cu_q_lens.cpu(),
                                     case.context_lens.cpu() if ctx else None, case.softmax_scale,
                                     page_size=case.page_size).numpy()


def _spiked_prefill_case(seed, lens, ctx, hq, hkv, d, spikes):
    """`spikes`: (sequence, logical key) pairs; keys below the sequence's context sit in the cached
    history, the others in the chunk's own rows."""
    case = workloads.make_prefill_case("stress", seed, lens, hq, hkv, context_lens=ctx, device=DEV, head_dim=d)
    gen = torch.Generator().manual_seed(seed + 7)
    direction = _unit(d, seed + 8)
    case.q.copy_((6.0 * direction + 0.3 * torch.randn(case.q.shape, generator=gen)).half())
    pool = 0.3 * torch.randn(case.kv_pool.shape, generator=gen)
    k = 0.3 * torch.randn(case.k.shape, generator=gen)
    v = 0.3 * torch.randn(case.v.shape, generator=gen)
    table = case.block_table.cpu()
    for b, at in spikes:
        c = int(case.context_lens[b])
        if at < c:
            pool[int(table[b, at // 16]) * 16 + at % 16, :hkv] += _spike_gain(d) * direction
        else:
            k[int(case.cu_q_lens[b]) + at - c] += _spike_gain(d) * direction
    case.kv_pool.copy_(pool.half())
    case.k.copy_(k.half())
    case.v.copy_(v.half())
    # the chunk's own rows join the history in the pool
    every = torch.cat([case.k, case.v], dim=1)
    case.kv_pool[case.slot_mapping.long()] = every
    return case


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("spike_at", [70, 300, 321, 1000])
def test_prefill_spike_every_format(fmt, d, spike_at):
    """Prompts (context 0) read from the paged pool in every format: the planted key in the first
    or second half of its tile, below the diagonal or on it."""
    print(f"stress prefill spike fmt={fmt} d={d} at={spike_at}", flush=True)
    hq, hkv = 16, 2
    case = _spiked_prefill_case(2300 + spike_at + d, [1100, 400], None, hq, hkv, d, [(0, spike_at), (1, 200)])
    pool, scales, values = _quantise(case.kv_pool, fmt, hkv)
    out = ops.paged_prefill(case.q, pool, case.block_table, case.cu_q_lens, None, case.max_q_len, case.softmax_scale,
                            kv_scales=scales)
    torch.cuda.synchronize()
    assert_attention_close(out, _prefill_ref(case, values, None), f"prefill spike {fmt} d={d} at {spike_at}")
    if fmt == "f16":
        packed = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1], case.seq_lens, case.max_q_len,
                                    case.softmax_scale)
        torch.cuda.synchronize()
        assert torch.equal(out, packed)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("hq,hkv", [(16, 2), (12, 4)])
def test_chunk_over_history_spike(fmt, d, hq, hkv):
    """Chunks over cached history: one sequence has its planted key deep in the history (every row of
    the chunk sees it from its first tile on), one in the chunk itself, one in both (the later key
    twice as far out), one has a history that ends inside a tile with the key right at its end."""
    print(f"stress chunk over history fmt={fmt} d={d} heads {hq}/{hkv}", flush=True)
    lens, ctx = [200, 333, 150, 40], [700, 100, 450, 77]
    case = _spiked_prefill_case(2400 + d + hq, lens, ctx, hq, hkv, d,
                                [(0, 130), (1, 100 + 170), (2, 31), (2, 450 + 149), (3, 76)])
    # sequence 2's later key lies further out than its earlier one
    row = int(case.cu_q_lens[2]) + 149
    case.k[row] = (case.k[row].float() * 2).half()
    case.kv_pool[case.slot_mapping[row].long(), :hkv] = case.k[row]
    pool, scales, values = _quantise(case.kv_pool, fmt, hkv)
    out = ops.paged_prefill(case.q, pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len,
                            case.softmax_scale, kv_scales=scales)
    again = ops.paged_prefill(case.q, pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len,
                              case.softmax_scale, kv_scales=scales)
    torch.cuda.synchronize()
    assert_attention_close(out, _prefill_ref(case, values, ctx), f"chunk spike {fmt} d={d} {hq}/{hkv}")
    assert torch.equal(out, again)


@pytest.mark.parametrize("d", [32, 256])
@pytest.mark.parametrize("fmt", ["f16", "int8"])
def test_general_kernel_spikes(d, fmt):
    """Head dims 32 and 256 (the general kernel): decode on both schedules, fused append of a
    spiking row, prefill and a chunk over history."""
    print(f"stress general kernel d={d} fmt={fmt}", flush=True)
    hq, hkv = 8, 2
    case, direction = _spiked_decode_case(2500 + d, [599, 130, 40, 0], hq, hkv, d, [(0, 301), (1, 5), (2, 39)])
    pool0, scales, values = _quantise(case.kv_pool, fmt, hkv)
    lens_before = case.seq_lens - 1
    ref = _decode_ref(case, values)
    for kw in DECODE_RUNS:
        out = ops.paged_decode(case.q, pool0, case.block_table, case.seq_lens, case.softmax_scale, kv_scales=scales, **kw)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"general kernel spike d={d} {fmt} {kw}")
    del lens_before
    case.k_new[3] += (_spike_gain(d) * direction).half().to(DEV)
    case.k_new[1] += (_spike_gain(d) * direction).half().to(DEV)
    want_pool = pool0.clone()
    if fmt == "f16":
        ops.kv_append(case.k_new, case.v_new, case.slot_mapping, want_pool)
    else:
        ops.kv_append_quantised(case.k_new, case.v_new, case.slot_mapping, want_pool, scales)
    ref = _decode_ref(case, _decoded(want_pool, scales, fmt))
    pool = pool0.clone()
    plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, 3)
    out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale, kv_scales=scales)
    torch.cuda.synchronize()
    assert torch.equal(pool, want_pool)
    assert_attention_close(out, ref, f"general kernel fused spike d={d} {fmt}")
    pre = _spiked_prefill_case(2510 + d, [150, 40], [100, 0], hq, hkv, d, [(0, 60), (0, 100 + 120), (1, 33)])
    pool, scales, values = _quantise(pre.kv_pool, fmt, hkv)
    out = ops.paged_prefill(pre.q, pool, pre.block_table, pre.cu_q_lens, pre.context_lens, pre.max_q_len,
                            pre.softmax_scale, kv_scales=scales)
    torch.cuda.synchronize()
    assert_attention_close(out, _prefill_ref(pre, values, [100, 0]), f"general kernel prefill spike d={d} {fmt}")


# ---- heavy-tailed inputs ------------------------------------------------------------------------

def _heavy_tail(t, gen, channels, gain):
    """N(0,1) with `channels` scaled by `gain`."""
    x = torch.randn(t.shape, generator=gen)
    x[..., channels] *= gain
    return x


def _tail_channels(d, seed):
    return torch.randperm(d, generator=torch.Generator().manual_seed(seed))[:4]


Q_GAIN, K_GAIN, V_GAIN = 48.0, 1.6, 0.5
# V is kept within +-2.5 or so: with a softmax this peaked an output row is close to one V row,
# and from magnitude 4 on the final rounding to fp16 alone (half a spacing of 2^-8) reaches the
# absolute tolerance.


def _score_span_log2(q, k, scale):
    """Largest minus smallest score of a query row against the given keys, in log2 units; the
    largest such span over the rows of q [rows, D] against k [keys, D]."""
    s = (q.float() @ k.float().T) * scale * 1.4426950408889634
    return float((s.amax(dim=-1) - s.amin(dim=-1)).max())


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("d", [64, 128])
def test_heavy_tailed_decode(fmt, d):
    """Four channels of q scaled x48 and of K x1.6: the scores of a row span about +-40 in log2
    units, with many keys between the extremes. Every schedule, the fused append and a shared prefix."""
    print(f"stress heavy-tailed decode fmt={fmt} d={d}", flush=True)
    hq, hkv, shared_pages = 32, 4, 12
    ctx, lists, num_pages = _shared_lists(2600 + d, shared_pages, [0, 9, 100, 700, 31, 250])
    case = workloads.make_decode_case("heavy", 2601 + d, ctx, hq, hkv, device=DEV, head_dim=d, page_lists=lists,
                                      num_pages=num_pages)
    gen = torch.Generator().manual_seed(2602 + d)
    ch = _tail_channels(d, 2603 + d)
    gain = math.sqrt(d / 128.0)      # the same span at either head dim
    case.q.copy_(_heavy_tail(case.q, gen, ch, Q_GAIN * gain).half())
    pool = torch.randn(case.kv_pool.shape, generator=gen)
    pool[:, :hkv, ch] *= K_GAIN
    pool[:, hkv:] *= V_GAIN
    case.kv_pool.copy_(pool.half())
    case.k_new.copy_(_heavy_tail(case.k_new, gen, ch, K_GAIN).half())
    case.v_new.mul_(V_GAIN)
    span = _score_span_log2(case.q[:, 0].cpu(), case.kv_pool[:700, 0].cpu(), case.softmax_scale)
    assert span > 70.0, f"scores span only {span:.1f} log2 units"
    pool0, scales, values = _quantise(case.kv_pool, fmt, hkv)
    lens = case.seq_lens - 1                                  # before the step's token
    ref = _decode_ref(case, values, lens)
    for kw in DECODE_RUNS + ({"schedule": "balanced", "shared_pages": shared_pages},):
        out = ops.paged_decode(case.q, pool0, case.block_table, lens, case.softmax_scale, kv_scales=scales, **kw)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"heavy-tailed decode {fmt} d={d} {kw}")
    want_pool = pool0.clone()
    if fmt == "f16":
        ops.kv_append(case.k_new, case.v_new, case.slot_mapping, want_pool)
    else:
        ops.kv_append_quantised(case.k_new, case.v_new, case.slot_mapping, want_pool, scales)
    ref = _decode_ref(case, _decoded(want_pool, scales, fmt))
    for shared in (0, shared_pages):
        pool = pool0.clone()
        plan = ops.DecodePlan(case.block_table, case.seq_lens, hq, hkv, case.num_pages, shared_pages=shared)
        out = ops.decode_step(case.q, pool, plan, case.k_new, case.v_new, case.softmax_scale, kv_scales=scales)
        torch.cuda.synchronize()
        assert torch.equal(pool, want_pool)
        assert_attention_close(out, ref, f"heavy-tailed fused step {fmt} d={d} shared={shared}")


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("d", [64, 128])
def test_heavy_tailed_prefill(fmt, d):
    """The same inputs through prefill: prompts from the pool (and packed K/V), chunks over history."""
    print(f"stress heavy-tailed prefill fmt={fmt} d={d}", flush=True)
    hq, hkv = 16, 2
    gain = math.sqrt(d / 128.0)
    for lens, ctx in (([900, 130, 333], None), ([200, 65, 129], [700, 1, 450])):
        case = workloads.make_prefill_case("heavy", 2700 + d + len(lens), lens, hq, hkv, context_lens=ctx, device=DEV,
                                           head_dim=d)
        gen = torch.Generator().manual_seed(2701 + d)
        ch = _tail_channels(d, 2702 + d)
        case.q.copy_(_heavy_tail(case.q, gen, ch, Q_GAIN * gain).half())
        pool = torch.randn(case.kv_pool.shape, generator=gen)
        pool[:, :hkv, ch] *= K_GAIN
        pool[:, hkv:] *= V_GAIN
        case.kv_pool.copy_(pool.half())
        case.k.copy_(_heavy_tail(case.k, gen, ch, K_GAIN).half())
        case.v.mul_(V_GAIN)
        case.kv_pool[case.slot_mapping.long()] = torch.cat([case.k, case.v], dim=1)
        span = _score_span_log2(case.q[:200, 0].cpu(), case.k[:200, 0].cpu(), case.softmax_scale)
        assert span > 70.0, f"scores span only {span:.1f} log2 units"
        pool, scales, values = _quantise(case.kv_pool, fmt, hkv)
        out = ops.paged_prefill(case.q, pool, case.block_table, case.cu_q_lens,
                                case.context_lens if ctx else None, case.max_q_len, case.softmax_scale,
                                kv_scales=scales)
        torch.cuda.synchronize()
        assert_attention_close(out, _prefill_ref(case, values, ctx), f"heavy-tailed prefill {fmt} d={d} ctx={ctx}")
        if fmt == "f16" and ctx is None:
            packed = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1], case.seq_lens, case.max_q_len,
                                        case.softmax_scale)
            torch.cuda.synchronize()
            assert torch.equal(out, packed)


@pytest.mark.parametrize("d", [32, 256])
def test_heavy_tailed_general_kernel(d):
    print(f"stress heavy-tailed general kernel d={d}", flush=True)
    hq, hkv = 8, 2
    gain = math.sqrt(d / 128.0)
    case = workloads.make_decode_case("heavy-g", 2800 + d, [599, 130, 40, 0], hq, hkv, device=DEV, head_dim=d)
    gen = torch.Generator().manual_seed(2801 + d)
    ch = _tail_channels(d, 2802 + d)
    case.q.copy_(_heavy_tail(case.q, gen, ch, Q_GAIN * gain).half())
    pool = torch.randn(case.kv_pool.shape, generator=gen)
    pool[:, :hkv, ch] *= K_GAIN
    pool[:, hkv:] *= V_GAIN
    case.kv_pool.copy_(pool.half())
    ref = _decode_ref(case, case.kv_pool.float().cpu())
    for kw in DECODE_RUNS:
        out = ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale, **kw)
        torch.cuda.synchronize()
        assert_attention_close(out, ref, f"heavy-tailed general kernel d={d} {kw}")
    pre = workloads.make_prefill_case("heavy-gp", 2810 + d, [150, 40], hq, hkv, context_lens=[100, 0], device=DEV,
                                      head_dim=d)
    pre.q.copy_(_heavy_tail(pre.q, gen, ch, Q_GAIN * gain).half())
    pool = torch.randn(pre.kv_pool.shape, generator=gen)
    pool[:, :hkv, ch] *= K_GAIN
    pool[:, hkv:] *= V_GAIN
    pre.kv_pool.copy_(pool.half())
    out = ops.paged_prefill(pre.q, pre.kv_pool, pre.block_table, pre.cu_q_lens, pre.context_lens, pre.max_q_len,
                            pre.softmax_scale)
    torch.cuda.synchronize()
    assert_attention_close(out, _prefill_ref(pre, pre.kv_pool.float().cpu(), [100, 0]),
                           f"heavy-tailed general kernel prefill d={d}")
