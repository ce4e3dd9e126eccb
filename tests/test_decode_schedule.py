"""Host rule that picks the decode schedule of a step (no GPU): the qualitative behaviour the
measurements behind its constants showed, at the sizes the benchmark configurations name.
0 = balanced, 1 = one wavefront per (sequence, kv head), 4 / 8 / 16 = splits per sequence + merge."""

from llama_lite_npu_amd.ops import SPLIT_COUNTS, decode_schedule, decode_schedule_estimates

TOK = 4096  # K + V bytes of a token: 8 kv heads, fp16


def pages(n):
    return (n + 15) // 16


def uniform(batch, tokens, **kw):
    return decode_schedule(batch, 8, pages(tokens), batch * pages(tokens), TOK, **kw)


def test_many_short_sequences_take_one_wavefront_each():
    for batch in (32, 64, 128, 256, 1024):
        assert uniform(batch, 64) == 1
    assert uniform(128, 256) == 1
    assert uniform(8, 40) == 1


def test_small_batches_take_several_splits_per_sequence():
    # measured: 1 to 8 sequences of 256 to 1024 tokens run 1.2 to 1.5 times faster in 8 or 16 splits
    for batch in (1, 2, 4, 8):
        for tokens in (256, 1024):
            assert uniform(batch, tokens) in (8, 16), (batch, tokens)
    assert uniform(8, 2048) in (8, 16)
    # from a few thousand tokens on, a step of few rows merges its long rows over several workgroups
    # and the balanced cut is the faster one again
    assert uniform(1, 4096) == 0 and uniform(2, 8192) == 0 and uniform(4, 8192) == 0
    c1 = [38, 129, 512, 1001]
    assert decode_schedule(4, 8, max(map(pages, c1)), sum(map(pages, c1)), TOK, heads_per_kv_head=2) in (8, 16)


def test_long_or_large_batches_stay_balanced():
    assert uniform(8, 16384) == 0 and uniform(16, 8192) == 0 and uniform(128, 2048) == 0
    assert uniform(1, 32768) == 0                             # one long sequence: the balanced cut
    # one long sequence among many short ones: the chain of its pages decides
    assert decode_schedule(128, 8, pages(8192), 127 * pages(64) + pages(8192), TOK) == 0
    # large batches of a few hundred tokens are bound by bytes, which the balanced cut streams faster
    assert uniform(1024, 512) == 0
    assert decode_schedule(32, 8, pages(4097), 32 * pages(2200), TOK) == 0             # C2
    assert decode_schedule(128, 4, pages(32769), 128 * pages(20000), TOK // 2) == 0    # C5


def test_the_choice_moves_one_way_with_the_longest_sequence():
    # one wavefront, then (small batches) several splits, then balanced: apart from a few pages
    # around a boundary (pages per split and per chunk are whole numbers) the choice never moves back
    for batch in (1, 4, 16, 64, 256):
        picks = [decode_schedule(batch, 8, mp, batch * mp, TOK) for mp in range(1, 2200)]
        order = [0 if p == 1 else 2 if p == 0 else 1 for p in picks]
        assert picks[0] == 1 and picks[-1] == 0
        backwards = [i for i in range(1, len(order)) if order[i] < order[i - 1]]
        assert len(backwards) <= 4, (batch, backwards)
        for i in backwards:                      # and it is back within 32 pages
            assert max(order[i:i + 32]) >= order[i - 1]


def test_degenerate_inputs():
    assert decode_schedule(0, 8, 0, 0, TOK) == 0 and decode_schedule(4, 8, 0, 0, TOK) == 0
    estimates = decode_schedule_estimates(4, 8, 10, 30, TOK)
    assert set(estimates) == {0, 1} | set(SPLIT_COUNTS) and all(t > 0 for t in estimates.values())


def test_splits_are_bounded_by_the_wavefronts_of_the_launch():
    for batch in (1, 2, 4, 8, 16, 32, 64, 128, 256, 1024):
        for tokens in (16, 64, 256, 1024, 4096, 16384):
            pick = uniform(batch, tokens)
            assert pick in (0, 1) + SPLIT_COUNTS
            assert pick <= 1 or batch * pick * 8 <= 2048
            wide = uniform(batch, tokens, heads_per_kv_head=32)     # two wavefronts per kv head
            assert wide <= 1 or batch * wide * 8 * 2 <= 2048


def test_wide_head_groups_lean_away_from_the_balanced_schedule():
    # 16 query heads per kv head slow the balanced schedule only: some steps leave it, none joins it
    moved = 0
    for batch in (8, 16, 64, 128):
        for mp in range(1, 400):
            narrow = decode_schedule(batch, 8, mp, batch * mp, TOK)
            wide = decode_schedule(batch, 8, mp, batch * mp, TOK, heads_per_kv_head=16)
            assert narrow != 0 or wide in (0, 1) + SPLIT_COUNTS
            assert wide != 0 or narrow == 0
            moved += narrow == 0 and wide != 0
    assert moved > 0


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
    for batch, tokens in ((2, 1024), (8, 512), (64, 256), (16, 16384)):
        picks = {decode_schedule(batch, 8, tokens // ps, batch * tokens // ps, TOK, page_size=ps)
                 for ps in (16, 64, 256)}
        assert len(picks) == 1, (batch, tokens, picks)
