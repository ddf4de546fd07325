"""The host-side plan of the matrix-core attention kernels: every (query row, key) pair that the
mask allows is covered by exactly one work item, partial slots are held once, and every partial
result has exactly one reduce item that reads it.  Runs without a GPU: it follows the kernels'
reading of the items (`wllm_amd/csrc/attention_mfma.hip`, `attention_prefill.hip`)."""
import numpy as np
import pytest

from wllm_amd.kernels import attention_plan as ap


def covered(q_len, ctx_len, group, nkv, window, page_size, rows_per_item=64, workgroup_slots=512, tiles_only=False):
    items, reduces, slots, prefill, prefill_rows = ap.build_work_items(
        np.array(q_len), np.array(ctx_len), group, nkv, window, page_size, rows_per_item, workgroup_slots, tiles_only)
    assert not (tiles_only and prefill.shape[0])
    assert prefill_rows == rows_per_item
    cover = {}          # (seg, kvh, row) -> list of (first key, end key, slot)
    slot_users = {}
    def hold(slot, who):
        assert 0 <= slot < slots, (slot, slots)
        assert slot not in slot_users, f"slot {slot} held by {slot_users[slot]} and {who}"
        slot_users[slot] = who
    for n, it in enumerate(items):
        seg, head_and_row, new_tokens, first_token, kb, ke, slot, context = (int(v) for v in it)
        kvh, row0 = head_and_row & 0xffff, (head_and_row >> 16) * 16      # the tile's number in the high 16 bits
        rows = q_len[seg] * group
        # short: at most 16 rows, or one token whose group of heads fills several tiles of 16
        assert rows <= 16 or q_len[seg] == 1 or tiles_only
        assert row0 % 16 == 0 and row0 < rows
        # the item carries the segment's lengths and the place of its first token in the step
        assert new_tokens == q_len[seg] and context == ctx_len[seg] and first_token == sum(q_len[:seg])
        # the kernel gives each of its four wavefronts one block of 32 keys of an aligned group of 128
        assert kb < ke and kb // 128 == (ke - 1) // 128, (kb, ke)
        first_pos = ctx_len[seg] - q_len[seg]
        assert kb >= (max(0, first_pos - window + 1) if window > 0 else 0) and ke <= ctx_len[seg]
        if slot >= 0:
            hold(slot, ("short", n))
        for r in range(row0, min(rows, row0 + 16)):
            cover.setdefault((seg, kvh, r), []).append((kb, ke, slot))
    for n, it in enumerate(prefill):
        seg, kvh, row0, kb, ke, slot = (int(v) for v in it[:6])
        rows = q_len[seg] * group
        assert rows > 16 and q_len[seg] > 1 and row0 % prefill_rows == 0 and row0 < rows
        first_pos = ctx_len[seg] - q_len[seg]
        last = min(rows - 1, row0 + prefill_rows - 1)
        b_hi = first_pos + last // group + 1
        b_lo = max(0, first_pos + row0 // group - window + 1) if window > 0 else 0
        lo, hi = max(b_lo, kb), min(b_hi, ke)
        assert lo < hi, "an item without keys"
        assert kb % 32 == 0 and ke % 32 == 0
        first_page, last_page = (lo // 32 * 32) // page_size, (min(-(-hi // 32) * 32, ctx_len[seg]) - 1) // page_size
        assert last_page - first_page + 1 <= ap.PREFILL_TABLE_PAGES
        for tile in range(prefill_rows // 16):
            if slot >= 0 and row0 + 16 * tile < rows:
                hold(slot + tile, ("prefill", n, tile))
        for r in range(row0, last + 1):
            cover.setdefault((seg, kvh, r), []).append((lo, hi, slot + (r - row0) // 16 if slot >= 0 else -1))
    reduce_of = {}
    for it in reduces:
        seg, kvh, first, splits, row0, stride = (int(v) for v in it[:6])
        for r in range(row0, min(row0 + 16, q_len[seg] * group)):
            assert (seg, kvh, r) not in reduce_of
            reduce_of[(seg, kvh, r)] = {first + j * stride for j in range(splits)}
    for seg in range(len(q_len)):
        first_pos = ctx_len[seg] - q_len[seg]
        for kvh in range(nkv):
            for r in range(q_len[seg] * group):
                pos = first_pos + r // group
                lo = max(0, pos - window + 1) if window > 0 else 0
                pieces = sorted(cover[(seg, kvh, r)])
                # pieces are disjoint, in order, and hold every key lo..pos
                assert pieces[0][0] <= lo and pieces[-1][1] > pos, (seg, kvh, r, pieces, lo, pos)
                for a, b in zip(pieces, pieces[1:]):
                    assert a[1] == b[0], (seg, kvh, r, pieces)
                if len(pieces) == 1 and pieces[0][2] < 0:
                    assert (seg, kvh, r) not in reduce_of
                else:
                    assert all(p[2] >= 0 for p in pieces)
                    assert reduce_of[(seg, kvh, r)] == {p[2] for p in pieces}
    assert len(slot_users) <= slots      # tiles beyond a segment's last row leave their slots unused
    return items, reduces, slots, prefill


@pytest.mark.parametrize("seed", range(24))
def test_every_pair_is_covered_once(seed, monkeypatch):
    rng = np.random.default_rng(seed)
    # small targets so that small cases split the way large ones do
    monkeypatch.setattr(ap, "PREFILL_MIN_PIECE", int(rng.choice([1, 4, 12])))
    monkeypatch.setattr(ap, "PREFILL_TABLE_PAGES", int(rng.choice([34, 1024])))
    group, nkv = int(rng.choice([1, 2, 3, 8, 17, 24, 32, 40])), int(rng.choice([1, 2, 3]))
    window = int(rng.choice([0, 0, 40, 300]))
    page_size = int(rng.choice([4, 12, 16, 64]))
    n = int(rng.integers(1, 5))
    q_len = [int(rng.choice([1, 2, 5, 17, 70, 130, 400])) for _ in range(n)]
    ctx_len = [q + int(rng.choice([0, 1, 31, 128, 500, 1500])) for q in q_len]
    covered(q_len, ctx_len, group, nkv, window, page_size, int(rng.choice([64, 128])), int(rng.choice([2, 16, 128, 512])))


def test_a_late_portion_of_a_long_prompt_is_split_over_the_keys():
    # 512 tokens at the end of 2,560, 8 query heads on one key/value head: 64 blocks of rows alone
    # would leave most compute units idle
    _, reduces, slots, prefill = covered([512], [2560], 8, 1, 0, 16)
    assert prefill.shape[0] >= 256
    assert slots > 0 and reduces.shape[0] == 512 * 8 // 16


def test_prefill_items_fill_the_workgroup_slots_once_where_they_can():
    """2,048 tokens of 8 heads on one key/value head: 256 blocks of rows over 1 to 64 groups of 32 keys.  The pieces
    are as short as 512 workgroups allow, and the items come longest first, every second run of 256 turned round."""
    _, _, _, prefill = covered([2048], [2048], 8, 1, 0, 16)
    assert 400 < prefill.shape[0] <= 512
    length = np.minimum(prefill[:, 4], (prefill[:, 2] + 63) // 8 + 1) - prefill[:, 3]     # up to the block's last row's key
    assert length.max() <= 32 * ap.prefill_piece_length(np.arange(1, 65).repeat(4), 1, 512, 4096)
    assert (np.diff(length[:256]) <= 0).all() and (np.diff(length[256:]) >= 0).all()
    assert length[:256].min() >= length[256:].max()
    # twice the prompt: 512 blocks of rows cannot be cut at all within one round, nor is any cut in two
    _, reduces, slots, prefill = covered([4096], [4096], 8, 1, 0, 16)
    assert prefill.shape[0] == 512 and slots == 0 and reduces.shape[0] == 0


def test_piece_length():
    span = np.array([64] * 8)
    assert ap.prefill_piece_length(span, 1, 16, 128) == 32          # two pieces a block fill 16 slots
    assert ap.prefill_piece_length(span, 2, 16, 128) == 64          # two heads: one piece a block
    assert ap.prefill_piece_length(span, 4, 16, 128) == 64          # two rounds, uncut
    assert ap.prefill_piece_length(span, 1, 512, 128) == ap.PREFILL_MIN_PIECE      # never shorter than this
    assert ap.prefill_piece_length(span, 1, 4, 16) == 16            # the longest piece allowed: 4 a block, 8 rounds


def test_a_whole_prompt_of_many_heads_is_not_split():
    _, reduces, slots, prefill = covered([300], [300], 1, 1, 0, 16)
    assert slots == 0 and reduces.shape[0] == 0
    assert (prefill[:, 5] == -1).all()


def test_a_decoded_token_of_a_large_group_stays_short():
    """More than 16 query heads a key/value head: the token's rows fill several tiles of 16, each with
    its own work items, partial slots and reduce item; nothing goes to the kernel for prompt portions,
    so a captured decode graph can hold it."""
    items, reduces, slots, prefill = covered([1, 1, 1], [50, 300, 129], 40, 2, 0, 16)
    assert prefill.shape[0] == 0
    assert sorted(set(int(v) >> 16 for v in items[:, 1])) == [0, 1, 2]
    # 1 + 3 + 2 chunks of keys, for 2 key/value heads and 3 tiles of rows
    assert items.shape[0] == (1 + 3 + 2) * 2 * 3
    assert reduces.shape[0] == 2 * 2 * 3 and slots == (3 + 2) * 2 * 3


@pytest.mark.parametrize("seed", range(12))
def test_tiles_only_covers_every_pair_once(seed):
    """The float32 kernel's plan: every segment, prompts too, as tiles of 16 rows with chunks of 128 keys."""
    rng = np.random.default_rng(100 + seed)
    group, nkv = int(rng.choice([1, 2, 3, 8, 17, 24])), int(rng.choice([1, 2, 3]))
    window = int(rng.choice([0, 0, 40, 300]))
    n = int(rng.integers(1, 5))
    q_len = [int(rng.choice([1, 2, 5, 17, 70, 130, 400])) for _ in range(n)]
    ctx_len = [q + int(rng.choice([0, 1, 31, 128, 500, 1500])) for q in q_len]
    items, reduces, slots, prefill = covered(q_len, ctx_len, group, nkv, window, 16, tiles_only=True)
    assert prefill.shape[0] == 0 and items.shape[0] > 0


def test_a_prompts_tiles_stop_at_their_last_rows_position():
    # 300 tokens of one head: tile 0 (tokens 0..15) needs keys 0..15 only, the last tile (tokens 288..299) keys 0..299
    items, reduces, slots, _ = covered([300], [300], 1, 1, 0, 16, tiles_only=True)
    by_tile = {}
    for it in items:
        by_tile.setdefault(int(it[1]) >> 16, []).append((int(it[4]), int(it[5])))
    assert by_tile[0] == [(0, 16)]
    assert sorted(by_tile[18]) == [(0, 128), (128, 256), (256, 300)]
    assert len(by_tile) == 19
