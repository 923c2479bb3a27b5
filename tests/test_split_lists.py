"""The lists that give every single row of a batch splits of its own for the decode attention
(host side only): every row present with consecutive splits, the budget kept, no split shorter than
the least, the list's length a function of the batch's shape alone."""
import numpy as np

from flambeau_amd.kernels import tuned


def test_every_row_gets_consecutive_splits_within_the_budget():
    rng = np.random.default_rng(0)
    for _ in range(1500):
        n = int(rng.integers(1, 70))
        per_row = int(rng.choice([1, 2, 8, 16, 64]))
        pos = rng.integers(0, int(rng.choice([50, 300, 5000, 70000])), n)
        window = int(rng.choice([0, 0, 64, 4096]))
        rows = np.stack([np.arange(n), pos, np.arange(n), np.zeros(n, int)], 1).astype(np.int32)
        items, firsts = tuned.balanced_items(rows, per_row, window)
        assert len(items) == tuned.decode_item_budget(n, per_row)
        used = items[items[:, 0] >= 0]
        assert (items[len(used):, 0] < 0).all()                       # the unused places are the last ones
        by_row = {}
        for r, p, q, w in used:
            assert p == pos[r] and q == r
            by_row.setdefault(int(r), []).append(int(w))
        assert list(by_row) == list(range(n))                          # in the order of the rows
        for r, ws in by_row.items():
            k = ws[0] >> 8
            assert [w & 255 for w in ws] == list(range(k)) and all(w >> 8 == k for w in ws)
            keys = min(pos[r] + 1, window) if window else pos[r] + 1
            assert 1 <= k <= tuned.DECODE_MAX_SPLITS and (k == 1 or keys / k > tuned.DECODE_MIN_KEYS_PER_SPLIT / 2)
        assert all(items[f, 0] == r and items[f, 3] == 256 * k for r, f, k, _ in firsts)


def test_long_contexts_get_the_splits_of_a_ragged_batch():
    pos = [8000, 100, 100, 100, 4000, 100, 100, 100]
    rows = np.array([[i, p, i, 0] for i, p in enumerate(pos)], dtype=np.int32)
    items, _ = tuned.balanced_items(rows, 8)
    splits = {int(r): int(w) >> 8 for r, _, _, w in items if r >= 0}
    assert splits[1] == 1 and splits[0] > splits[4] > 8
    # the longest split is not much longer than the mean of the work per place
    longest = max((p + 1) / splits[i] for i, p in enumerate(pos))
    assert longest < 2.0 * sum(p + 1 for p in pos) / len(items) + tuned.DECODE_MIN_KEYS_PER_SPLIT
    # rows of one length share a block per unit and no more; 64 of them get a split each
    even, _ = tuned.balanced_items(np.array([[i, 2099, i, 0] for i in range(8)], dtype=np.int32), 8)
    assert [int(w) >> 8 for r, _, _, w in even if r >= 0 and w & 255 == 0] == [8] * 8
    even, _ = tuned.balanced_items(np.array([[i, 2099, i, 0] for i in range(16)], dtype=np.int32), 8)
    assert [int(w) >> 8 for r, _, _, w in even if r >= 0 and w & 255 == 0] == [2] * 16
    many, _ = tuned.balanced_items(np.array([[i, 2099, i, 0] for i in range(64)], dtype=np.int32), 8)
    assert len(many) == 256 and (many[:64, 3] == 256).all() and (many[64:, 0] < 0).all()
    # no rows, one row
    assert tuned.balanced_items(rows[:0], 8)[0].shape == (0, 4)
    one, first = tuned.balanced_items(rows[:1], 8)
    assert (one[:, 0] >= 0).sum() == 63 and first[0].tolist() == [0, 0, 63, 0]
