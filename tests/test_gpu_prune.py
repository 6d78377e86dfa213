"""GPU parity of the TW mask producers (tw_prune_tiled_wise_1d / _2d through the C ABI)
against the CPU oracle and the golden vectors of the reference's prune_algo.py.

Masks are integer results: the bar is bit-exact.  The oracle computes with NumPy itself
(np.linalg.norm, np.percentile), so these tests also check that the HIP kernels repeat
NumPy's float32 summation order and percentile arithmetic."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "prune_vectors.npz")


@pytest.fixture(scope="module")
def twprune(tw):
    from tilesparsity_amd import twprune as m
    return m


@pytest.fixture(scope="module")
def po():
    from oracle import tw_prune_oracle
    return tw_prune_oracle


def parse_sparsity(text):
    return int(text) if text.lstrip("-").isdigit() else float(text)


def test_golden_vectors(twprune):
    z = np.load(GOLD)
    meta = json.loads(bytes(z["meta"]).decode())
    for case in meta["cases"]:
        name, g = case["name"], case["granularity"]
        weights = [z["%s/w%d" % (name, i)] for i in range(len(case["shapes"]))]
        scores = twprune.img2col_forward(weights)
        for sp in case["sparsities"]:
            print("case", name, sp, flush=True)
            got = {"tiled_wise_1d": twprune.tiled_wise_1d(scores, parse_sparsity(sp), g),
                   "tiled_wise_2d": twprune.tiled_wise_2d(scores, parse_sparsity(sp), g)}
            for fn, masks in got.items():
                for i, m in enumerate(masks):
                    want = np.unpackbits(z["%s/%s/%s/m%d" % (name, fn, sp, i)])[:m.size]
                    assert np.array_equal(m.ravel(), want.astype(bool)), (name, fn, sp, i)


def test_norms_are_numpys_bits(twprune, po):
    rng = np.random.default_rng(20)
    for K, N, g in ((37, 300, 8), (300, 1000, 8), (64, 520, 128), (16, 1500, 700), (5, 7, 3)):
        x = rng.standard_normal((K, N)).astype(np.float32)
        table = po.tiles_every_g_columns(N, g)
        print("norms", K, N, g, flush=True)
        assert np.array_equal(twprune.tile_row_norms(x, table).view(np.uint32),
                              po.tile_row_norms(x, table).view(np.uint32))
        keep = rng.random(N) < 0.6
        want = po.tile_row_norms(x * keep[None, :], table)
        assert np.array_equal(twprune.tile_row_norms(x, table, keep).view(np.uint32), want.view(np.uint32))
        assert np.array_equal(twprune.col_norms(x).view(np.uint32), po.col_norms(x).view(np.uint32))


def test_percentile_is_numpys_bits(twprune):
    rng = np.random.default_rng(19)
    for n in (1, 2, 3, 10, 101, 1000, 37500, 300001):
        for quant in (0, 64):
            v = rng.random(n).astype(np.float32)
            if quant:
                v = (np.round(v * quant) / quant).astype(np.float32)
            for q in (0, 0.1, 25, 33.3, 50, 66.6, 75.0, 99.9, 100, np.float64(50.0), np.float64(87.3)):
                want = np.percentile(v, q)
                got = twprune.percentile(v, q)
                assert got.dtype == want.dtype and got.tobytes() == want.tobytes(), (n, quant, q, got, want)


SHAPES = [
    [(64, 256), (128, 384)],
    [(100, 130), (33, 500), (257, 64)],          # ragged last tiles
    [(300, 1000)],
    [(3, 3, 16, 48), (48, 72)],                  # conv + dense
]


@pytest.mark.parametrize("shapes", SHAPES)
@pytest.mark.parametrize("g", [8, 32, 128, 200])
@pytest.mark.parametrize("sparsity", [50, 75.0, 87.5, np.float64(60.0)])
def test_1d_matches_oracle(twprune, po, shapes, g, sparsity):
    rng = np.random.default_rng(abs(hash((str(shapes), g, float(sparsity)))) % 2 ** 31)
    scores = twprune.img2col_forward([rng.standard_normal(s).astype(np.float32) for s in shapes])
    print("1d", shapes, g, repr(sparsity), flush=True)
    want, thr, _ = po.tiled_wise_1d(scores, sparsity, g)
    got = twprune.tiled_wise_1d(scores, sparsity, g)
    assert np.float64(thr) == twprune.tiled_wise_1d.last_threshold
    for w, m in zip(want, got):
        assert np.array_equal(w, m)


@pytest.mark.parametrize("shapes", SHAPES)
@pytest.mark.parametrize("g", [8, 32, 128])
@pytest.mark.parametrize("sparsity,transform", [(50, True), (75.0, True), (60, False),
                                                (np.float64(80.0), False)])
def test_2d_matches_oracle(twprune, po, shapes, g, sparsity, transform):
    rng = np.random.default_rng(abs(hash((str(shapes), g, float(sparsity), transform))) % 2 ** 31)
    scores = twprune.img2col_forward([rng.standard_normal(s).astype(np.float32) for s in shapes])
    print("2d", shapes, g, repr(sparsity), transform, flush=True)
    want, thrs, tables, _ = po.tiled_wise_2d(scores, sparsity, g, transform=transform)
    got, got_tables = twprune.tiled_wise_2d(scores, sparsity, g, transform=transform, return_tiles=True)
    assert (np.float64(thrs[0]), np.float64(thrs[1])) == twprune.tiled_wise_2d.last_thresholds
    for w, m in zip(want, got):
        assert np.array_equal(w, m)
    assert got_tables == tables


def test_ties_and_extremes(twprune, po):
    rng = np.random.default_rng(21)
    # scores on a coarse grid: many rows share a norm, some tie with the threshold
    scores = [(np.round(rng.standard_normal((96, 128)) * 2) / 2).astype(np.float32) for _ in range(2)]
    scores = twprune.img2col_forward(scores)
    for sp in (0, 100, 50, 33.3, np.float64(66.6)):
        for g in (16, 64):
            w1, _, _ = po.tiled_wise_1d(scores, sp, g)
            g1 = twprune.tiled_wise_1d(scores, sp, g)
            w2 = po.tiled_wise_2d(scores, sp, g)[0]
            g2 = twprune.tiled_wise_2d(scores, sp, g)
            for a, b in zip(w1 + w2, g1 + g2):
                assert np.array_equal(a, b), (sp, g)
    # a constant layer: the threshold equals every norm, nothing is kept
    ones = [np.ones((8, 8), np.float32)]
    assert not twprune.tiled_wise_1d(ones, 50, 4)[0].any()


def test_wide_tiles_use_the_recursive_sum(twprune, po):
    rng = np.random.default_rng(22)
    scores = [np.abs(rng.standard_normal((40, 1500))).astype(np.float32)]
    for g in (129, 256, 700, 1500):
        want, _, _ = po.tiled_wise_1d(scores, 70, g)
        got = twprune.tiled_wise_1d(scores, 70, g)
        assert np.array_equal(want[0], got[0]), g


def test_masks_feed_plans(tw, twprune, po, oracle):
    """1-D masks go through tw_plan_from_mask, 2-D masks through tw_plan_from_mask_tiles with
    the kept-column tile table; the plans hold the lists the oracle derives from the mask."""
    rng = np.random.default_rng(23)
    K, N, G = 192, 320, 64
    W = rng.standard_normal((K, N)).astype(np.float32)
    scores = twprune.img2col_forward([W])
    m1 = twprune.tiled_wise_1d(scores, 75, G)[0]
    with tw.Plan.from_mask(m1, G, "f16", W) as plan:
        ex, _ = plan.export(with_weight=False)
        want = po.plan_tiles_from_mask(m1, po.tiles_every_g_columns(N, G))
        for t, wt in zip(ex, want):
            assert t["kept_k"].tolist() == wt["kept_k"] and t["kept_n"].tolist() == wt["kept_n"]
    m2, tables = twprune.tiled_wise_2d(scores, 75, G, return_tiles=True)
    with tw.Plan.from_mask_tiles(m2[0], tables[0], "f16", W) as plan:
        ex, _ = plan.export(with_weight=False)
        want = po.plan_tiles_from_mask(m2[0], tables[0])
        assert [(t["col0"], t["width"]) for t in ex] == tables[0]
        for t, wt in zip(ex, want):
            assert t["kept_k"].tolist() == wt["kept_k"] and t["kept_n"].tolist() == wt["kept_n"]
        # and the GEMM on that plan is the masked dense product
        A = rng.standard_normal((64, K)).astype(np.float32)
        from tests.test_gpu_gemm import run_gemm
        C, _ = run_gemm(tw, oracle, plan, A, "f16", N, pruned=1)
        ref = oracle.quantize(A, "f16").astype(np.float64) @ (oracle.quantize(W, "f16") * m2[0]).astype(np.float64)
        assert oracle.rel_error(C, ref) <= 1e-2


def test_granularity_pruning_matches_oracle(twprune, po):
    rng = np.random.default_rng(24)
    for K, N, g in ((64, 128, 16), (768, 768, 64), (300, 512, 128), (5, 8, 2)):
        s = np.abs(rng.standard_normal((K, N))).astype(np.float32)
        for sp in (50, 75.0, 90, np.float64(33.3), 0, 100):
            print("granularity", K, N, g, repr(sp), flush=True)
            assert np.array_equal(twprune.granularity_pruning(s, sp, g), po.granularity_pruning(s, sp, g))
    # ties inside a tile
    s = (np.round(np.abs(rng.standard_normal((96, 64))) * 2) / 2).astype(np.float32)
    assert np.array_equal(twprune.granularity_pruning(s, 60, 8), po.granularity_pruning(s, 60, 8))


def test_error_paths(tw, twprune):
    with pytest.raises(tw.TwError):
        twprune.tiled_wise_1d([np.ones((4, 4), np.float32)], 150, 2)
    with pytest.raises(tw.TwError):
        twprune.tiled_wise_1d([np.ones((4, 4), np.float32)], 50, 0)
    with pytest.raises(tw.TwError):
        twprune.granularity_pruning(np.ones((4, 6), np.float32), 50, 4)
    with pytest.raises(tw.TwError):
        tw.Plan.from_mask_tiles(np.ones((4, 8), np.uint8), [(0, 4), (5, 3)], "f16", np.ones((4, 8), np.float32))
