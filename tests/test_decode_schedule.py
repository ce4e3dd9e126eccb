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


# ---- the three-way rule: balanced / one wavefront / several splits per sequence ----------------

from llama_lite_npu_amd.ops import SPLIT_COUNTS, decode_schedule  # noqa: E402


def uniform(batch, tokens, **kw):
    return decode_schedule(batch, 8, pages(tokens), batch * pages(tokens), TOK, **kw)


def test_small_batches_take_several_splits_per_sequence():
    # measured: 1 to 8 sequences of 256 to 2048 tokens run 1.3 to 1.5 times faster in 8 or 16 splits
    for batch in (1, 2, 4, 8):
        for tokens in (256, 1024, 2048):
            assert uniform(batch, tokens) in (8, 16), (batch, tokens)
    c1 = [38, 129, 512, 1001]
    assert decode_schedule(4, 8, max(map(pages, c1)), sum(map(pages, c1)), TOK, heads_per_kv_head=2) in (8, 16)


def test_the_other_regimes_keep_their_schedule():
    for batch in (32, 64, 128):
        assert uniform(batch, 64) == 1                       # many short sequences: one wavefront each
    assert uniform(8, 16384) == 0 and uniform(16, 8192) == 0 and uniform(128, 2048) == 0
    assert decode_schedule(32, 8, pages(4097), 32 * pages(2200), TOK) == 0             # C2
    assert decode_schedule(128, 4, pages(32769), 128 * pages(20000), TOK // 2) == 0    # C5
    assert uniform(1, 32768) == 0                             # one long sequence: the balanced cut
    assert decode_schedule(0, 8, 0, 0, TOK) == 0 and decode_schedule(4, 8, 0, 0, TOK) == 0


def test_splits_are_bounded_by_the_wavefronts_of_the_launch():
    for batch in (1, 2, 4, 8, 16, 32, 64, 128, 256, 1024):
        for tokens in (16, 64, 256, 1024, 4096, 16384):
            pick = uniform(batch, tokens)
            assert pick in (0, 1) + SPLIT_COUNTS
            assert pick <= 1 or batch * pick * 8 <= 2048
            wide = uniform(batch, tokens, heads_per_kv_head=32)     # two wavefronts per kv head
            assert wide <= 1 or batch * wide * 8 * 2 <= 2048


def test_the_schedule_in_use_keeps_an_advantage():
    changed = kept = 0
    for batch in (1, 4, 8, 16, 32):
        for mp in range(1, 700, 3):
            free = decode_schedule(batch, 8, mp, batch * mp, TOK)
            for current in (0, 1, 4, 8, 16):
                sticky = decode_schedule(batch, 8, mp, batch * mp, TOK, current=current, hysteresis=1.1)
                assert sticky in (free, current)             # hysteresis only ever keeps the current one
                kept += sticky == current != free
                changed += sticky != current
    assert kept > 0 and changed > 0
    # and a schedule that is not a candidate for the step (too many wavefronts) is not kept
    assert decode_schedule(512, 8, 4, 2048, TOK, current=16, hysteresis=2.0) in (0, 1)


def test_page_size_does_not_change_the_choice_for_the_same_tokens():
    for batch, tokens in ((2, 1024), (8, 512), (64, 64), (16, 16384)):
        picks = {decode_schedule(batch, 8, tokens // ps, batch * tokens // ps, TOK, page_size=ps)
                 for ps in (16, 64, 256)}
        assert len(picks) == 1, (batch, tokens, picks)
