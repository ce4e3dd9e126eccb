"""Host rule that picks the decode schedule of a step (no GPU): the qualitative behaviour the
measurements behind its constants showed, at the sizes the benchmark configurations name."""

from llama_lite_npu_amd.ops import per_sequence_decode_is_faster as per_sequence

TOK = 4096  # K + V bytes of a token: 8 kv heads, fp16


def pages(n):
    return (n + 15) // 16


def test_many_short_sequences_take_one_wavefront_each():
    for batch in (32, 64, 128, 256):
        assert per_sequence(batch, 8, pages(64), batch * pages(64), TOK)
    assert per_sequence(128, 8, pages(256), 128 * pages(256), TOK)
    assert per_sequence(8, 8, pages(40), 8 * pages(40), TOK)


def test_long_or_ragged_batches_stay_balanced():
    assert not per_sequence(8, 8, pages(4096), 8 * pages(4096), TOK)
    assert not per_sequence(1, 8, pages(32768), pages(32768), TOK)
    # one long sequence among many short ones: the chain of its pages decides
    assert not per_sequence(128, 8, pages(8192), 127 * pages(64) + pages(8192), TOK)
    # large batches of a few hundred tokens are bound by bytes, which the balanced cut streams faster
    assert not per_sequence(1024, 8, pages(512), 1024 * pages(512), TOK)


def test_benchmark_configurations_stay_balanced():
    c1 = [38, 129, 512, 1001]
    assert not per_sequence(4, 8, max(map(pages, c1)), sum(map(pages, c1)), TOK)
    assert not per_sequence(32, 8, pages(4097), 32 * pages(2200), TOK)             # C2
    assert not per_sequence(128, 4, pages(32769), 128 * pages(20000), TOK // 2)    # C5


def test_the_choice_is_monotonic_in_the_longest_sequence():
    flips = [per_sequence(64, 8, mp, 64 * mp, TOK) for mp in range(1, 300)]
    assert flips[0] and not flips[-1]
    assert sum(a != b for a, b in zip(flips, flips[1:])) == 1


def test_degenerate_inputs():
    assert not per_sequence(0, 8, 0, 0, TOK)
    assert not per_sequence(4, 8, 0, 0, TOK)
    # a wider margin only ever moves steps to the balanced schedule
    for mp in range(1, 200):
        if per_sequence(32, 8, mp, 32 * mp, TOK, margin=1.2):
            assert per_sequence(32, 8, mp, 32 * mp, TOK, margin=1.0)


def test_wide_head_groups_lean_towards_one_wavefront_per_sequence():
    # 16 query heads per kv head slow the balanced schedule only: some steps change sides, none the other way
    moved = 0
    for batch in (8, 16, 64, 128):
        for mp in range(1, 80):
            narrow = per_sequence(batch, 8, mp, batch * mp, TOK)
            wide = per_sequence(batch, 8, mp, batch * mp, TOK, heads_per_kv_head=16)
            assert wide or not narrow
            moved += wide and not narrow
    assert moved > 0
