"""The mask-producer oracle against the golden vectors written from the reference's
prune_algo.py, and its summation-order / percentile models against NumPy itself."""
import json
import os

import numpy as np
import pytest

from oracle import tw_prune_oracle as po

GOLD = os.path.join(os.path.dirname(__file__), "golden", "prune_vectors.npz")


def load_gold():
    z = np.load(GOLD)
    meta = json.loads(bytes(z["meta"]).decode())
    return z, meta


def parse_sparsity(text):
    return int(text) if text.lstrip("-").isdigit() else float(text)


def gold_cases():
    z, meta = load_gold()
    for case in meta["cases"]:
        for sp in case["sparsities"]:
            yield case["name"], sp


@pytest.mark.parametrize("name,sp", list(gold_cases()))
def test_oracle_matches_reference_vectors(name, sp):
    z, meta = load_gold()
    case = next(c for c in meta["cases"] if c["name"] == name)
    weights = [z["%s/w%d" % (name, i)] for i in range(len(case["shapes"]))]
    scores = [po.img2col(w) for w in weights]
    sparsity = parse_sparsity(sp)
    m1, _, _ = po.tiled_wise_1d(scores, sparsity, case["granularity"])
    m2, _, _, _ = po.tiled_wise_2d(scores, sparsity, case["granularity"])
    for fn, masks in (("tiled_wise_1d", m1), ("tiled_wise_2d", m2)):
        for i, m in enumerate(masks):
            want = np.unpackbits(z["%s/%s/%s/m%d" % (name, fn, sp, i)])[:m.size].reshape(m.shape).astype(bool)
            assert np.array_equal(m, want), (name, fn, sp, i)


def gold_mix_cases():
    _, meta = load_gold()
    for name, calls in meta["mix"].items():
        for fn, sp, g1 in calls:
            yield name, fn, sp, g1


@pytest.mark.parametrize("name,fn,sp,g1", list(gold_mix_cases()))
def test_mix_oracle_matches_reference_vectors(name, fn, sp, g1):
    z, meta = load_gold()
    case = next(c for c in meta["cases"] if c["name"] == name)
    scores = [po.img2col(z["%s/w%d" % (name, i)]) for i in range(len(case["shapes"]))]
    masks = getattr(po, fn)(scores, parse_sparsity(sp), case["granularity"], parse_sparsity(g1))
    for i, m in enumerate(masks):
        want = np.unpackbits(z["%s/%s/%s/%s/m%d" % (name, fn, sp, g1, i)])[:m.size].reshape(m.shape)
        assert np.array_equal(m, want.astype(bool)), (name, fn, sp, g1, i)


def test_mix_adds_exactly_the_largest_unkept_elements():
    """Property check of tw_mix_fn against a sort: without ties, the added elements are the
    top g1percent of the shifted scores, and nothing kept by the TW mask is lost."""
    rng = np.random.default_rng(21)
    scores = [np.abs(rng.standard_normal(s)).astype(np.float32) for s in [(40, 64), (30, 50)]]
    tw_masks, _, _ = po.tiled_wise_1d(scores, 80, 16)
    mixed, thr = po.tw_mix_fn(scores, 5, tw_masks)
    shifted = np.concatenate([(s - m).ravel() for s, m in zip(scores, tw_masks)])
    n_extra = int(np.sum(shifted > thr))
    assert abs(n_extra - 0.05 * shifted.size) <= 1
    top = np.sort(shifted)[-n_extra:]
    assert top[0] > thr >= np.sort(shifted)[-n_extra - 1]
    for m0, m1 in zip(tw_masks, mixed):
        assert np.all(m1[m0])


def test_fixture_was_written_by_this_numpy_family():
    _, meta = load_gold()
    # np.percentile keeps float32 arithmetic for float32 data since NumPy 2; the fixture and the
    # oracle must run under the same rule
    assert meta["numpy"].split(".")[0] == np.__version__.split(".")[0]


def test_tile_tables_known_answers():
    assert po.tiles_every_g_columns(300, 128) == [(0, 128), (128, 128), (256, 44)]
    assert po.tiles_every_g_columns(128, 128) == [(0, 128)]
    assert po.tiles_every_g_columns(5, 8) == [(0, 5)]
    # every 2 kept columns; a split is not opened after the last column
    cm = np.array([1, 0, 1, 1, 0, 0, 1, 0, 1, 1], bool)
    assert po.tiles_every_g_kept_columns(cm, 2) == [(0, 3), (3, 4), (7, 3)]
    assert po.tiles_every_g_kept_columns(np.array([1, 1], bool), 2) == [(0, 2)]
    assert po.tiles_every_g_kept_columns(np.zeros(4, bool), 2) == [(0, 4)]


def test_row_norm_model_is_numpys_order():
    rng = np.random.default_rng(5)
    for w in list(range(1, 140)) + [200, 255, 256, 257, 300, 511, 1000]:
        x = rng.standard_normal((3, w + 5)).astype(np.float32)[:, 2:2 + w]
        ref = np.linalg.norm(x, axis=1) / x.shape[1]
        for i in range(3):
            assert po.row_norm_model(x[i]).tobytes() == ref[i].tobytes(), w


def test_col_norm_model_is_numpys_order():
    rng = np.random.default_rng(6)
    for K in (1, 2, 7, 8, 9, 100, 1000, 3000):
        x = rng.standard_normal((K, 33)).astype(np.float32)
        ref = np.linalg.norm(x, axis=0) / x.shape[0]
        assert np.array_equal(po.col_norm_model(x).view(np.uint32), ref.view(np.uint32)), K


@pytest.mark.parametrize("f64", [False, True])
def test_percentile_model_is_numpys(f64):
    rng = np.random.default_rng(7)
    for n in (1, 2, 3, 10, 101, 1000, 4097):
        for q in (0, 0.1, 25, 33.3, 50, 66.6, 75, 90, 99.9, 100):
            for quant in (0, 8):
                v = rng.random(n).astype(np.float32)
                if quant:
                    v = (np.round(v * quant) / quant).astype(np.float32)
                qq = np.float64(q) if f64 else q
                want = np.percentile(v, qq)
                got = po.percentile_model(v, q, f64)
                assert got.dtype == want.dtype and got.tobytes() == want.tobytes(), (n, q, quant)


def test_strict_comparison_prunes_ties():
    # all rows of a tile share one norm: the threshold equals it and nothing is kept
    s = np.ones((8, 4), np.float32)
    masks, thr, _ = po.tiled_wise_1d([s], 50, 4)
    assert not masks[0].any() and thr == np.float32(0.5)


def test_granularity_pruning_per_tile_threshold():
    rng = np.random.default_rng(8)
    s = np.abs(rng.standard_normal((32, 64))).astype(np.float32)
    m = po.granularity_pruning(s, 75, 16)
    for c0 in range(0, 64, 16):
        rows = m[:, c0]
        assert np.array_equal(m[:, c0:c0 + 16], np.repeat(rows[:, None], 16, 1))
        assert rows.sum() == 8          # 25 % of 32 rows survive in every tile


def test_granularity_pruning_brute_force():
    """Pins WHICH rows survive (MyHook.py:202-214: per tile, rows whose L2 norm is strictly
    above the tile's own percentile): the percentile is worked out by hand from the two order
    statistics around rank q (n - 1) / 100, the norms with plain Python sums."""
    rng = np.random.default_rng(81)
    for (K, N, G, q) in ((7, 6, 3, 40), (12, 8, 4, 75), (9, 10, 5, 50), (5, 4, 2, 0), (6, 6, 3, 100)):
        s = np.abs(rng.standard_normal((K, N))).astype(np.float32)
        got = po.granularity_pruning(s, q, G)
        for c0 in range(0, N, G):
            norms = [float(np.float32(np.sqrt(np.float32(sum(
                np.float32(s[r, c]) * np.float32(s[r, c]) for c in range(c0, c0 + G))))))
                for r in range(K)]
            order = sorted(norms)
            pos = q / 100.0 * (K - 1)
            lo = int(np.floor(pos))
            hi = min(lo + 1, K - 1)
            thr = order[lo] + (order[hi] - order[lo]) * (pos - lo)
            # rows far from the threshold decide by the hand value; a row within rounding of it
            # (float32 vs double interpolation) is left to the bit-exact percentile model tests
            for r in range(K):
                if abs(norms[r] - thr) > 1e-5 * max(1.0, thr):
                    assert got[r, c0] == (norms[r] > thr), (K, N, G, q, c0, r)
            assert (got[:, c0:c0 + G] == got[:, c0:c0 + 1]).all()
    # q = 0 keeps all rows but the smallest, q = 100 keeps none (strict comparison)
    s = np.abs(rng.standard_normal((5, 4))).astype(np.float32)
    assert po.granularity_pruning(s, 0, 2).sum(axis=0).tolist() == [4, 4, 4, 4]
    assert not po.granularity_pruning(s, 100, 2).any()


def test_granularity_pruning_one_tile_equals_tiled_wise_1d():
    """With one tile as wide as the layer, the per-tile threshold is the layer's threshold:
    the kept rows are those of tiled_wise_1d on the same scores (whose norms are divided by
    the tile width on both sides of the comparison, a positive factor; pinned by the golden
    vectors)."""
    rng = np.random.default_rng(82)
    for (K, N, q) in ((64, 16, 75), (100, 8, 50), (33, 32, 90)):
        s = np.abs(rng.standard_normal((K, N))).astype(np.float32) + np.float32(0.5)
        g = po.granularity_pruning(s, q, N)
        m1, _, _ = po.tiled_wise_1d([s], q, N)
        # the division by the width can move a row across the threshold only on a last-bit tie
        diff = g != m1[0]
        assert diff.sum() == 0 or diff[:, 0].sum() <= 1
        assert np.array_equal(g[:, 0], m1[0][:, 0]) or diff[:, 0].sum() <= 1


def test_masks_are_tile_wise():
    rng = np.random.default_rng(9)
    s = [np.abs(rng.standard_normal((50, 70))).astype(np.float32)]
    m1, _, t1 = po.tiled_wise_1d(s, 60, 32)
    tiles = po.plan_tiles_from_mask(m1[0], t1[0])
    assert sum(len(t["kept_k"]) for t in tiles) == int(m1[0][:, [c for c, _ in t1[0]]].sum())
    m2, _, t2, cm = po.tiled_wise_2d(s, 60, 8)
    po.plan_tiles_from_mask(m2[0], t2[0])
    # a column the 2-D producer pruned holds no kept element, and its tiles end on kept columns
    assert not m2[0][:, ~cm[0]].any()
    assert all(cm[0][c0 + w - 1] or not cm[0][c0:c0 + w].any() for c0, w in t2[0])
