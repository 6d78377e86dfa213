"""CPU tests of the on-disk hand-off: the exported pruned model (exportPrunedModel,
Pruning/BERT/utils/MyHook.py:54-89), the restricted unpickler and the tile table derived from
a stored mask.  No GPU work: only host entry points of the library are called."""
import io
import pickle

import numpy as np
import pytest

from oracle import tw_prune_oracle as po


@pytest.fixture(scope="module")
def ex():
    from tilesparsity_amd import twexport
    return twexport


def random_layers(rng, shapes):
    layers = []
    for i, (K, N) in enumerate(shapes):
        mi = (rng.random(K) < 0.5).astype(np.float32)
        mo = (rng.random(N) < 0.6).astype(np.float32)
        layers.append(("bert/encoder/layer_%d/dense" % i, mi, mo,
                       rng.standard_normal((K, N)).astype(np.float32),
                       rng.standard_normal(N).astype(np.float32)))
    return layers


def test_oracle_export_known_answer(oracle):
    mi = np.array([1, 0, 1, 1], np.float32)
    mo = np.array([0, 1, 1], np.float32)
    kernel = np.arange(12, dtype=np.float32).reshape(4, 3)
    bias = np.array([5, 6, 7], np.float32)
    ck = oracle.export_pruned_model([("l", mi, mo, kernel, bias)])
    assert list(ck) == ["l/mask-i:0", "l/mask-o:0", "l/kernel:0", "l/bias:0"]
    assert ck["l/mask-i:0"].tolist() == [0, 1, 1]          # kept rows 0, 2, 3
    assert ck["l/mask-o:0"].tolist() == [1, 1]             # kept columns 1, 2
    assert ck["l/kernel:0"].tolist() == [[1, 2], [7, 8], [10, 11]]
    assert ck["l/bias:0"].tolist() == [0, 6, 7]


def test_oracle_export_scatters_back_to_the_masked_kernel(oracle):
    rng = np.random.default_rng(5)
    for scope, mi, mo, kernel, bias in random_layers(rng, [(37, 50), (64, 9), (5, 130)]):
        ck = oracle.export_pruned_model([(scope, mi, mo, kernel, bias)])
        kk = oracle.offsets_to_kept(ck[scope + "/mask-i:0"])
        kn = oracle.offsets_to_kept(ck[scope + "/mask-o:0"])
        assert np.array_equal(kk, np.flatnonzero(mi)) and np.array_equal(kn, np.flatnonzero(mo))
        back = np.zeros_like(kernel)
        back[np.ix_(kk, kn)] = ck[scope + "/kernel:0"]
        assert np.array_equal(back, kernel * np.outer(mi, mo))


def test_product_export_equals_oracle(ex, oracle, tmp_path):
    rng = np.random.default_rng(6)
    layers = random_layers(rng, [(40, 48), (96, 33), (8, 8)])
    want = oracle.export_pruned_model(layers)
    path = tmp_path / "pruned_model.pkl"
    got = ex.export_pruned_model(layers, path)
    assert list(got) == list(want)
    for k in want:
        assert np.array_equal(got[k], want[k]) and got[k].dtype == want[k].dtype, k
    loaded = ex.load_pickle(path)
    assert list(loaded) == list(want)
    for k in want:
        assert np.array_equal(loaded[k], want[k])
    # the same bytes the reference's hook writes load as well: plain pickle.dump of the dict
    buf = io.BytesIO()
    pickle.dump(want, buf, pickle.HIGHEST_PROTOCOL)
    again = ex.load_pickle(buf.getvalue())
    assert all(np.array_equal(again[k], want[k]) for k in want)


@pytest.mark.parametrize("protocol", [2, 4, pickle.HIGHEST_PROTOCOL])
def test_unpickler_admits_arrays_and_containers(ex, protocol):
    obj = {"a": np.arange(6, dtype=np.int64).reshape(2, 3), "b": [np.ones(3, bool), 2.5, "x"],
           "c": np.float32(1.5), "d": np.zeros((2, 2, 1, 3), np.int32)[:, :, :, ::2]}
    back = ex.load_pickle(pickle.dumps(obj, protocol))
    assert np.array_equal(back["a"], obj["a"]) and np.array_equal(back["d"], obj["d"])
    assert back["b"][1:] == [2.5, "x"] and back["c"] == np.float32(1.5)


def test_unpickler_refuses_code(ex):
    class Evil:
        def __reduce__(self):
            import os
            return (os.getcwd, ())

    for payload in (pickle.dumps({"x": Evil()}), pickle.dumps(print), pickle.dumps(io.BytesIO)):
        with pytest.raises(pickle.UnpicklingError):
            ex.load_pickle(payload)


def test_layer_grouping_errors(ex, tw):
    ok = {"s/mask-i:0": np.array([0]), "s/mask-o:0": np.array([0]), "s/kernel:0": np.ones((1, 1)),
          "s/bias:0": np.ones(1)}
    assert [g[0] for g in ex._layer_groups(ok)] == ["s"]
    assert list(ex._layer_groups({"global_step:0": np.array(3)})) == []
    bad = dict(list(ok.items())[:3])
    with pytest.raises(tw.TwError):
        list(ex._layer_groups(bad))
    swapped = {"s/mask-i:0": ok["s/mask-i:0"], "s/kernel:0": ok["s/kernel:0"],
               "s/mask-o:0": ok["s/mask-o:0"], "s/bias:0": ok["s/bias:0"]}
    with pytest.raises(tw.TwError):
        list(ex._layer_groups(swapped))
    with pytest.raises(tw.TwError):
        ex.export_pruned_model([("s", np.ones(2), np.ones(3), np.ones((3, 2)), np.ones(3))])
    with pytest.raises(tw.TwError):
        ex.mask_2d(np.ones((2, 3, 4)))


# --------------------------------------------------------------------------------------
# tile table from a stored mask
# --------------------------------------------------------------------------------------
def check_table(mask, table, g):
    """The table covers [0,N), every tile is rows x columns and holds at most g kept columns."""
    n = mask.shape[1]
    assert table[0][0] == 0 and sum(w for _, w in table) == n
    assert all(table[i][0] + table[i][1] == table[i + 1][0] for i in range(len(table) - 1))
    tiles = po.plan_tiles_from_mask(mask, table)       # raises unless rows x columns
    if g > 0:
        assert max(len(t["kept_n"]) for t in tiles) <= g


@pytest.mark.parametrize("g", [0, 16, 32])
def test_tiles_from_mask_on_producer_masks(tw, g):
    rng = np.random.default_rng(9)
    scores = [np.abs(rng.standard_normal(s)).astype(np.float32) for s in [(40, 50), (64, 130), (17, 16)]]
    m1, _, _ = po.tiled_wise_1d(scores, 60, 16)
    m2, _, _, _ = po.tiled_wise_2d(scores, 60, 16)
    for mask in m1 + m2:
        want = po.tiles_from_mask(mask, g)
        got = tw.tiles_from_mask(mask, g)
        assert got == want
        check_table(mask, got, g)


def test_tiles_from_mask_edge_cases(tw):
    assert tw.tiles_from_mask(np.zeros((4, 9), np.uint8)) == [(0, 9)]
    assert tw.tiles_from_mask(np.ones((4, 9), np.uint8)) == [(0, 9)]
    assert tw.tiles_from_mask(np.ones((4, 9), np.uint8), 4) == [(0, 4), (4, 4), (8, 1)]
    assert tw.tiles_from_mask(np.ones((1, 1), np.uint8), 128) == [(0, 1)]
    # rows that differ only in position must not share a tile
    m = np.zeros((3, 4), np.uint8)
    m[0, 0] = m[1, 1] = m[2, 2] = m[0, 3] = 1
    assert tw.tiles_from_mask(m) == po.tiles_from_mask(m) == [(0, 1), (1, 1), (2, 1), (3, 1)]
    with pytest.raises(tw.TwError):
        tw.tiles_from_mask(np.zeros((0, 4), np.uint8))


def test_tiles_from_mask_accepts_any_mask(tw):
    """An element-wise mask is not tile-wise, yet the derived tiles are all rows x columns."""
    rng = np.random.default_rng(10)
    for shape, density in [((30, 40), 0.5), ((64, 64), 0.05), ((7, 200), 0.9)]:
        mask = rng.random(shape) < density
        got = tw.tiles_from_mask(mask, 32)
        assert got == po.tiles_from_mask(mask, 32)
        check_table(mask, got, 32)


# --------------------------------------------------------------------------------------
# host logic of the producer mirror (no GPU call)
# --------------------------------------------------------------------------------------
def test_percentile_type_follows_the_type_of_q():
    """np.percentile keeps float32 arithmetic for a Python number and switches to float64 for a
    NumPy float64; the mirror passes that choice to the library."""
    from tilesparsity_amd import twprune
    assert twprune._q_type(75) == twprune.Q_F32 and twprune._q_type(75.0) == twprune.Q_F32
    assert twprune._q_type(np.float64(75)) == twprune.Q_F64
    assert twprune._q_type(np.float32(75)) == twprune.Q_F32
    assert twprune._q_type(100 - np.sqrt(10000 - 75 * 100)) == twprune.Q_F64   # tiled_wise_2d's own
    assert twprune._q_type(100 - 5) == twprune.Q_F32 and twprune._q_type(75 + np.float64(5)) == twprune.Q_F64
    # and NumPy really behaves that way (the reason the switch exists)
    v = np.random.default_rng(3).random(1001).astype(np.float32)
    assert np.percentile(v, 33.3).dtype == np.float32 and np.percentile(v, np.float64(33.3)).dtype == np.float64


def test_img2col_forward_shapes_and_sign():
    from tilesparsity_amd import twprune
    rng = np.random.default_rng(4)
    conv, dense = rng.standard_normal((3, 3, 8, 16)).astype(np.float32), rng.standard_normal((5, 7)).astype(np.float32)
    out = twprune.img2col_forward([conv, dense])
    assert out[0].shape == (72, 16) and out[1].shape == (5, 7)
    assert np.array_equal(out[0], po.img2col(conv)) and np.array_equal(out[1], np.abs(dense))
    # HWIO -> (H*W*I) x O keeps the output channel as the column
    assert np.array_equal(out[0][:, 3], np.abs(conv[..., 3]).ravel())
