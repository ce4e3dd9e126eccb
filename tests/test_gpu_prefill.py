"""GPU parity of varlen causal prefill (paged and packed) against the CPU oracle."""

import pytest
import torch

from llama_lite_npu_amd import ops, workloads
from oracle import c_oracle
from tests.parity import assert_attention_close, to_np16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _append(case):
    ops.kv_append(case.k, case.v, case.slot_mapping, case.kv_pool)


def _oracle_paged(case):
    return c_oracle.paged_prefill(to_np16(case.q), to_np16(case.kv_pool), case.block_table.cpu().numpy(),
                                  case.cu_q_lens.cpu().numpy(), case.context_lens.cpu().numpy(),
                                  case.softmax_scale, page_size=case.page_size)


@pytest.mark.parametrize("hq,hkv,lens", [
    (16, 8, [1, 2, 15, 16, 17, 33]),
    (64, 8, [128, 77, 200]),
    (32, 4, [300, 5]),
    (8, 8, [65]),
    (16, 1, [130, 40]),        # 16 query heads per kv head: two workgroups per kv head
    (28, 4, [260, 31]),        # 7 heads per kv head: one idle column tile
    (4, 4, [520, 129]),        # no grouping: 128 query rows per workgroup
    (64, 8, [700, 333]),       # long enough for tiles wholly below the diagonal
])
def test_paged_prefill_context_zero(hq, hkv, lens):
    print(f"prefill paged {hq}/{hkv} {lens}", flush=True)
    case = workloads.make_prefill_case("p", 300 + hq + len(lens), lens, hq, hkv, device=DEV)
    _append(case)
    out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, None, case.max_q_len,
                            case.softmax_scale)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_paged(case), "paged prefill ctx=0")
    # the packed-K/V entry point must agree bit for bit: same arithmetic, other addressing
    out2 = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1], case.seq_lens, case.max_q_len,
                              case.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


def test_chunked_prefill_over_history():
    """Chunk rows attend to history + chunk; equals rows [ctx, ctx+q) of the full prefill."""
    print("prefill chunked", flush=True)
    full = workloads.make_prefill_case("full", 400, [150, 40, 97], 16, 8, device=DEV)
    _append(full)
    out_full = ops.paged_prefill(full.q, full.kv_pool, full.block_table, full.cu_q_lens, None,
                                 full.max_q_len, full.softmax_scale)
    ctx = torch.tensor([100, 16, 0], dtype=torch.int32)
    chunk = full.seq_lens.cpu() - ctx
    cu = torch.zeros(4, dtype=torch.int32)
    cu[1:] = torch.cumsum(chunk, 0)
    rows = torch.cat([torch.arange(int(full.cu_q_lens[i]) + int(ctx[i]), int(full.cu_q_lens[i + 1]))
                      for i in range(3)]).to(DEV)
    q_chunk = full.q[rows].contiguous()
    out_chunk = ops.paged_prefill(q_chunk, full.kv_pool, full.block_table, cu.to(DEV), ctx.to(DEV),
                                  int(chunk.max()), full.softmax_scale)
    torch.cuda.synchronize()
    ref = c_oracle.paged_prefill(to_np16(q_chunk), to_np16(full.kv_pool), full.block_table.cpu().numpy(),
                                 cu.numpy(), ctx.numpy(), full.softmax_scale)
    assert_attention_close(out_chunk, ref, "chunk vs oracle")
    assert float((out_chunk.float() - out_full[rows].float()).abs().max()) <= 1e-3


def test_decode_equals_prefill_of_one_row():
    print("prefill q_len=1 == decode", flush=True)
    case = workloads.make_decode_case("d", 410, [500, 31, 1024], 64, 8, device=DEV)
    dec = ops.paged_decode(case.q, case.kv_pool, case.block_table, case.seq_lens, case.softmax_scale,
                           num_splits=1)
    cu = torch.arange(4, dtype=torch.int32, device=DEV)
    pre = ops.paged_prefill(case.q, case.kv_pool, case.block_table, cu, case.seq_lens - 1, 1,
                            case.softmax_scale)
    torch.cuda.synchronize()
    assert float((dec.float() - pre.float()).abs().max()) <= 1e-3


def test_prefill_running_maximum_keeps_growing():
    """Scores rise steadily along the keys, so every tile moves the running maximum by far more
    than the slack the lazy rescale allows."""
    print("prefill growing maximum", flush=True)
    case = workloads.make_prefill_case("g", 420, [600, 190], 16, 2, device=DEV)
    gen = torch.Generator().manual_seed(421)
    direction = torch.randn(workloads.HEAD_DIM, generator=gen)
    direction = direction / direction.norm()
    t_total = case.q.shape[0]
    pos = torch.cat([torch.arange(int(n)) for n in case.seq_lens.tolist()]).float()
    noise_q = 0.1 * torch.randn(case.q.shape, generator=gen)
    noise_k = 0.1 * torch.randn(case.k.shape, generator=gen)
    case.q.copy_((8.0 * direction + noise_q).half())
    # score ~ 8 * 0.3 * pos: about +0.3 in log2 units per key after scaling, +10 per 32 keys
    case.k.copy_((direction * (0.3 * pos)[:, None, None] + noise_k).half())
    assert case.k.shape[0] == t_total
    _append(case)
    out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, None, case.max_q_len,
                            case.softmax_scale)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_paged(case), "growing maximum")


@pytest.mark.parametrize("spike_at", [70, 300, 321, 1000])
def test_prefill_score_spike_far_above_the_running_maximum(spike_at):
    """One key scores about 2^40 times higher than everything before it (its probability would
    overflow fp16 against the running maximum): the tile has to be redone with a rescale, whether
    the key sits in the first or second half of its tile, below the diagonal or on it."""
    print(f"prefill score spike at key {spike_at}", flush=True)
    case = workloads.make_prefill_case("spike", 430 + spike_at, [1100, 400], 16, 2, device=DEV)
    gen = torch.Generator().manual_seed(431)
    direction = torch.randn(workloads.HEAD_DIM, generator=gen)
    direction = direction / direction.norm()
    case.q.copy_((6.0 * direction + 0.3 * torch.randn(case.q.shape, generator=gen)).half())
    k = 0.3 * torch.randn(case.k.shape, generator=gen)
    k[spike_at] += 52.0 * direction              # 6 * 52 / sqrt(128) * log2(e): about +40 in log2 units
    k[1100 + 200] += 52.0 * direction            # second sequence: a spike of its own
    case.k.copy_(k.half())
    _append(case)
    out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, None, case.max_q_len,
                            case.softmax_scale)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_paged(case), f"spike at {spike_at}")
    packed = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1], case.seq_lens, case.max_q_len,
                                case.softmax_scale)
    torch.cuda.synchronize()
    assert_attention_close(packed, _oracle_paged(case), f"spike at {spike_at}, packed K/V")


def test_prefill_never_reads_values_past_the_sequence_end():
    """Slots after the last token of a page (and unowned pages) hold NaN: they must not leak."""
    print("prefill NaN in unused slots", flush=True)
    case = workloads.make_prefill_case("n", 430, [70, 17, 100, 1], 16, 8, device=DEV)
    case.kv_pool.fill_(float("nan"))
    _append(case)
    out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, None, case.max_q_len,
                            case.softmax_scale)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    assert_attention_close(out, _oracle_paged(case), "NaN outside the sequences")


def test_prefill_repeats_bit_for_bit():
    """Same inputs, same bits: nothing in the kernel may depend on wavefront timing."""
    print("prefill repeatability", flush=True)
    case = workloads.make_prefill_case("r", 440, [700, 333], 64, 8, device=DEV)
    _append(case)
    outs = []
    for _ in range(6):
        outs.append(ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, None,
                                      case.max_q_len, case.softmax_scale))
    torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.equal(outs[0], o)


@pytest.mark.parametrize("page_size", [32, 64, 128, 256])
@pytest.mark.parametrize("hq,hkv,lens,ctx", [
    (16, 8, [1, 2, 15, 16, 17, 33, 47, 48, 63, 64, 65, 127, 128, 129, 255, 256, 257], None),
    (64, 8, [128, 77, 200], None),
    (32, 4, [300, 5, 96], [100, 31, 64]),       # chunks over cached history
    (16, 1, [130, 40], [17, 700]),
])
def test_paged_prefill_page_sizes(page_size, hq, hkv, lens, ctx):
    """Pools with pages of 32 to 256 tokens (the reference's --page_size): prompts and chunks over
    history whose ends fall on every kind of boundary inside and between pages."""
    print(f"prefill page_size {page_size} {hq}/{hkv} {lens} ctx {ctx}", flush=True)
    case = workloads.make_prefill_case("pp", 900 + page_size + hq, lens, hq, hkv, context_lens=ctx, device=DEV,
                                       page_size=page_size)
    _append(case)
    out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens,
                            case.context_lens if ctx is not None else None, case.max_q_len, case.softmax_scale,
                            page_size=page_size)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_paged(case), f"paged prefill page_size {page_size}")


@pytest.mark.parametrize("head_dim", [64, 32, 256])
@pytest.mark.parametrize("hq,hkv,lens,ctx,page_size", [
    (16, 8, [1, 2, 15, 16, 17, 33, 64, 65], None, 16),
    (14, 2, [128, 77], None, 16),
    (32, 4, [100, 5, 96], [100, 31, 64], 32),       # chunks over cached history
    (16, 1, [70, 40], [17, 200], 64),
    (8, 8, [45, 1, 18], [3, 70, 0], 16),            # no grouping: 16 query rows per wavefront at 32 / 256
    (12, 3, [33, 64, 7], None, 32),                 # 4 heads per kv head: 4 rows per wavefront, ragged last blocks
    (40, 2, [20, 9], [5, 0], 16),                   # 20 heads per kv head: two slices of 10, one row each
])
def test_prefill_head_dims(head_dim, hq, hkv, lens, ctx, page_size):
    """Prefill at head dims 32, 64 and 256: prompts (paged and packed entry points agree bit for
    bit) and chunks over cached history."""
    print(f"prefill head_dim {head_dim} {hq}/{hkv} {lens} ctx {ctx} page_size {page_size}", flush=True)
    case = workloads.make_prefill_case("pd", 950 + head_dim + hq, lens, hq, hkv, context_lens=ctx, device=DEV,
                                       page_size=page_size, head_dim=head_dim)
    _append(case)
    out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens,
                            case.context_lens if ctx is not None else None, case.max_q_len, case.softmax_scale,
                            page_size=page_size)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_paged(case), f"paged prefill head_dim {head_dim}")
    if ctx is None:
        out2 = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1], case.seq_lens, case.max_q_len,
                                  case.softmax_scale)
        torch.cuda.synchronize()
        assert torch.equal(out, out2)


@pytest.mark.parametrize("hq,hkv,lens,ctx,page_size", [
    (32, 8, [700, 333, 1500], None, 16),            # Llama-3.2-1B's heads; many key tiles, ragged ends
    (64, 4, [257, 1023], None, 16),                 # 16 query heads per kv head: two workgroups per group
    (24, 8, [129, 64, 900], [513, 1, 250], 32),     # 3 heads per kv head; chunks over long histories
    (8, 8, [1100], [2000], 64),                     # no grouping
])
def test_prefill_head_dim_64_on_the_tiled_kernel(hq, hkv, lens, ctx, page_size):
    """Head dim 64 with fp16 K/V runs on the MFMA-tiled kernel (rows of 128 bytes, their own LDS
    swizzle): sequences long enough for the pipelined loop, the masked diagonal and rescales, and
    repeated launches agree bit for bit."""
    print(f"prefill head_dim 64 tiled {hq}/{hkv} {lens} ctx {ctx} page_size {page_size}", flush=True)
    case = workloads.make_prefill_case("p64", 4200 + hq, lens, hq, hkv, context_lens=ctx, device=DEV,
                                       page_size=page_size, head_dim=64)
    _append(case)
    outs = [ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens,
                              case.context_lens if ctx is not None else None, case.max_q_len,
                              case.softmax_scale, page_size=page_size) for _ in range(3)]
    torch.cuda.synchronize()
    assert_attention_close(outs[0], _oracle_paged(case), "paged prefill head_dim 64")
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    if ctx is None:
        out2 = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1], case.seq_lens, case.max_q_len,
                                  case.softmax_scale)
        torch.cuda.synchronize()
        assert torch.equal(outs[0], out2)


@pytest.mark.parametrize("head_dim", [128, 64])
@pytest.mark.parametrize("hq,hkv,lens,ctx", [
    (32, 1, [130, 40], None),                  # 32 heads per kv head: four workgroups per kv head
    (96, 4, [70, 200], None),                  # 24
    (40, 2, [260, 31], [100, 700]),            # 20, chunks over history
    (64, 1, [90, 33], [0, 150]),               # 64: the most a kv head may carry
])
def test_prefill_more_than_16_query_heads_per_kv_head(head_dim, hq, hkv, lens, ctx):
    """The reference's grid is per query head (flashattention2_nopad.py:195): no bound on the group."""
    print(f"prefill {hq}/{hkv} heads d={head_dim} {lens} ctx {ctx}", flush=True)
    case = workloads.make_prefill_case("wg", 1300 + hq + head_dim, lens, hq, hkv, context_lens=ctx, device=DEV,
                                       head_dim=head_dim)
    _append(case)
    out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens,
                            case.context_lens if ctx is not None else None, case.max_q_len, case.softmax_scale)
    torch.cuda.synchronize()
    assert_attention_close(out, _oracle_paged(case), f"prefill {hq}/{hkv}")
    if ctx is None:
        out2 = ops.varlen_prefill(case.q, case.k, case.v, case.cu_q_lens[:-1], case.seq_lens, case.max_q_len,
                                  case.softmax_scale)
        torch.cuda.synchronize()
        assert torch.equal(out, out2)


def test_prefill_length_beyond_the_block_table_row():
    """A chunk whose history claims more tokens than its block-table row names: the row's last
    entry is re-read instead of the memory behind the row; the other sequences are unaffected."""
    print("prefill length beyond the table", flush=True)
    case = workloads.make_prefill_case("pb", 1390, [20, 30, 17], 16, 4, context_lens=[40, 30, 0], device=DEV)
    _append(case)
    ref = _oracle_paged(case)
    ctx = case.context_lens.clone()
    ctx[1] = 500                                # the table has 4 entries per row
    assert case.block_table.shape[1] == 4
    out = ops.paged_prefill(case.q, case.kv_pool, case.block_table, case.cu_q_lens, ctx, case.max_q_len,
                            case.softmax_scale)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    rows = torch.cat([torch.arange(0, 20), torch.arange(50, 67)])
    assert_attention_close(out[rows.to(DEV)], ref[rows.numpy()], "rows of the other sequences")


@pytest.mark.parametrize("head_dim", [128, 64])
@pytest.mark.parametrize("hq,hkv,lens,ctx,slices,page_size", [
    (64, 8, [512], [4096], 2, 16),              # one request's chunk over a long history
    (64, 8, [200], [3000], 4, 16),              # ragged last row block
    (32, 4, [77, 130], [1000, 17], 3, 32),      # a sequence whose slices are mostly empty beside a long one
    (16, 8, [16], [2049], 8, 16),               # a single row block, eight slices
    (8, 8, [300], [0], 2, 16),                  # no history: 128 rows per block, the diagonal in the last slice only
    (14, 2, [64], [63], 5, 64),                 # fewer plain tiles than slices
    (32, 1, [40], [900], 2, 16),                # 32 heads per kv head: four workgroups per kv head
    (64, 8, [1, 3], [640, 5000], 4, 128),       # one and three rows
])
def test_paged_prefill_over_key_slices(head_dim, hq, hkv, lens, ctx, slices, page_size):
    """A chunk whose row blocks are cut along their keys (key_slices workgroups per block and a merge
    launch): within tolerance of the oracle and of the unsplit launch, the same bits on a second
    launch, and with one slice the plain kernel itself."""
    print(f"prefill over {slices} key slices d={head_dim} {hq}/{hkv} {lens} ctx {ctx} page_size {page_size}", flush=True)
    case = workloads.make_prefill_case("ks", 7300 + hq + slices, lens, hq, hkv, context_lens=ctx, device=DEV,
                                       page_size=page_size, head_dim=head_dim)
    _append(case)
    args = (case.q, case.kv_pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len,
            case.softmax_scale)
    plain = ops.paged_prefill(*args, page_size=page_size, key_slices=1)
    split = ops.paged_prefill(*args, page_size=page_size, key_slices=slices)
    again = ops.paged_prefill(*args, page_size=page_size, key_slices=slices)
    torch.cuda.synchronize()
    ref = _oracle_paged(case)
    assert_attention_close(split, ref, f"{slices} key slices")
    assert_attention_close(plain, ref, "one slice")
    assert torch.equal(split, again)
    assert float((split.float() - plain.float()).abs().max()) <= 1e-3
    # the workspace may be the caller's, and larger than needed
    need = ops.paged_prefill_workspace_floats(case.q.shape[0], hq, head_dim, slices)
    ws = torch.full((need + 64,), float("nan"), dtype=torch.float32, device=DEV)
    mine = ops.paged_prefill(*args, page_size=page_size, key_slices=slices, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(mine, split)


def test_key_slices_are_chosen_for_launches_that_leave_the_device_idle():
    print("prefill key slice rule", flush=True)
    lib = ops._lib.load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rule = lambda *a: int(lib.litekv_paged_prefill_key_slices(*a))
    # 512 rows x 64/8 heads = 32 row blocks x 8 kv heads = 256 workgroups on 2 per compute unit
    assert rule(1, 64, 8, 128, 128, 32768) >= 4
    if cus == 256:
        assert rule(1, 64, 8, 128, 512, 32768 + 512) == 2         # measured 609 -> 551 us
        assert rule(1, 64, 8, 128, 128, 32768) == 8               # 64 workgroups: eight slices fill the slots
        assert rule(1, 64, 8, 128, 128, 2048 + 128) == 4           # measured 40 -> 30 us
        assert rule(1, 64, 8, 128, 64, 8192 + 64) == 8             # measured 130 -> 36 us
    assert rule(4, 64, 8, 128, 512, 32768) == 1                    # four such chunks fill it
    assert rule(1, 64, 8, 128, 512, 700) == 1                      # too few keys to share out
    assert rule(1, 64, 8, 128, 512, 2048 + 512) == 1               # two slices would not pay (49 -> 60 us)
    assert rule(1, 64, 8, 128, 512, 4096 + 512) == 1               # nor here (82 -> 88 us)
    for rows in (64, 128, 256, 512):                               # a fresh prompt is never cut (14 -> 29 us in eight)
        assert rule(1, 64, 8, 128, rows, rows) == 1 and rule(1, 64, 8, 128, rows, 256 + rows) == 1
    assert rule(1, 64, 8, 256, 128, 32768) == 1 and rule(1, 64, 8, 32, 128, 32768) == 1
    assert rule(1, 32, 8, 64, 256, 16384) >= 2                     # head dim 64 has its own build
    # chosen by default from the longest row's keys as the caller knows them; not at all without them
    case = workloads.make_prefill_case("ksr", 7400, [256], 64, 8, context_lens=[6000], device=DEV)
    _append(case)
    args = (case.q, case.kv_pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len,
            case.softmax_scale)
    picked = rule(1, 64, 8, 128, 256, 6256)
    assert picked > 1
    auto = ops.paged_prefill(*args, max_kv_len=6256)
    forced = ops.paged_prefill(*args, key_slices=picked)
    blind = ops.paged_prefill(*args)
    plain = ops.paged_prefill(*args, key_slices=1)
    torch.cuda.synchronize()
    assert torch.equal(auto, forced) and torch.equal(blind, plain)
    assert_attention_close(auto, _oracle_paged(case), "key slices by default")


def test_key_slices_argument_errors():
    print("prefill key slice errors", flush=True)
    case = workloads.make_prefill_case("kse", 7500, [64], 16, 8, context_lens=[1024], device=DEV)
    _append(case)
    args = (case.q, case.kv_pool, case.block_table, case.cu_q_lens, case.context_lens, case.max_q_len,
            case.softmax_scale)
    with pytest.raises(ops._lib.LiteKVError, match="key_slices"):
        ops.paged_prefill(*args, key_slices=9)
    with pytest.raises(ValueError, match="workspace"):
        ops.paged_prefill(*args, key_slices=2, workspace=torch.empty(16, dtype=torch.float32, device=DEV))
    case32 = workloads.make_prefill_case("kse32", 7501, [64], 16, 8, context_lens=[1024], device=DEV, head_dim=32)
    ops.kv_append(case32.k, case32.v, case32.slot_mapping, case32.kv_pool)
    with pytest.raises(ops._lib.LiteKVError, match="head_dim"):
        ops.paged_prefill(case32.q, case32.kv_pool, case32.block_table, case32.cu_q_lens, case32.context_lens,
                          case32.max_q_len, case32.softmax_scale, key_slices=2,
                          workspace=torch.empty(1 << 20, dtype=torch.float32, device=DEV))
