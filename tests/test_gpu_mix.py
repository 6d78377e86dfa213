"""GPU parity of the mixed (TW + element-wise remainder) producers, tw_prune_mix through the C
ABI, against the golden vectors of the reference's prune_algo.py:151-193 and the CPU oracle;
and of the covering plan that runs such masks on the TW kernel.

Masks: bit-exact.  GEMM on a covering plan: max relative error <= 1e-2 (fp16) / 2e-2 (bf16)
against the float64 product of the 16-bit operands with the mask applied."""
import json
import os

import numpy as np
import pytest

from tests.test_gpu_gemm import run_gemm

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


def parse(text):
    return int(text) if text.lstrip("-").isdigit() else float(text)


def test_golden_vectors_mix(twprune):
    z = np.load(GOLD)
    meta = json.loads(bytes(z["meta"]).decode())
    for case in meta["cases"]:
        name, g = case["name"], case["granularity"]
        scores = twprune.img2col_forward([z["%s/w%d" % (name, i)] for i in range(len(case["shapes"]))])
        for fn, sp, g1 in meta["mix"][name]:
            print("case", name, fn, sp, g1, flush=True)
            got = getattr(twprune, fn)(scores, parse(sp), g, parse(g1))
            for i, m in enumerate(got):
                want = np.unpackbits(z["%s/%s/%s/%s/m%d" % (name, fn, sp, g1, i)])[:m.size]
                assert np.array_equal(m.ravel(), want.astype(bool)), (name, fn, sp, g1, i)


SHAPES = [
    [(64, 256), (128, 384)],
    [(100, 130), (33, 500), (257, 64)],
    [(3, 3, 16, 48), (48, 72)],
    [(1, 1)],
]


@pytest.mark.parametrize("shapes", SHAPES)
@pytest.mark.parametrize("g1", [5, 1, 2.5, 0, np.float64(3.0)])
def test_mix_matches_oracle(twprune, po, shapes, g1):
    rng = np.random.default_rng(abs(hash((str(shapes), float(g1)))) % 2 ** 31)
    scores = twprune.img2col_forward([rng.standard_normal(s).astype(np.float32) for s in shapes])
    for sp, g in ((75, 32), (50.0, 128), (90, 8)):
        print("mix", shapes, repr(g1), sp, g, flush=True)
        for fn in ("tiled_wise_1d_mix", "tiled_wise_2d_mix"):
            want = getattr(po, fn)(scores, sp, g, g1)
            got = getattr(twprune, fn)(scores, sp, g, g1)
            for w, m in zip(want, got):
                assert np.array_equal(w, m), (fn, sp, g)
    # the second stage alone, on masks that are not tile-wise at all
    masks = [rng.random(s.shape) < 0.3 for s in scores]
    want, thr = po.tw_mix_fn(scores, g1, masks)
    got = twprune.tw_mix_fn(scores, g1, masks)
    assert np.float64(thr) == twprune.tw_mix_fn.last_threshold
    for w, m in zip(want, got):
        assert np.array_equal(w, m)


def test_mix_ties_and_extremes(twprune, po):
    rng = np.random.default_rng(41)
    scores = [(np.round(rng.standard_normal((96, 128)) * 2) / 2).astype(np.float32) for _ in range(2)]
    scores = twprune.img2col_forward(scores)
    for sp, g1 in ((50, 5), (0, 100), (95, 5), (60, 33.3), (99, 1)):
        want = po.tiled_wise_1d_mix(scores, sp, 16, g1)
        got = twprune.tiled_wise_1d_mix(scores, sp, 16, g1)
        for a, b in zip(want, got):
            assert np.array_equal(a, b), (sp, g1)


def test_mix_error_paths(tw, twprune):
    with pytest.raises(tw.TwError):
        twprune.tiled_wise_1d_mix([np.ones((4, 4), np.float32)], 50, 2, 120)   # percentile < 0
    with pytest.raises(tw.TwError):
        twprune.tiled_wise_1d_mix([np.ones((4, 4), np.float32)], 98, 2, 5)     # TW stage > 100


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_cover_plan_runs_mixed_masks(tw, twprune, po, oracle, dtype):
    """A mixed mask is not tile-wise (the plain builder refuses it); the covering plan computes
    A (B (.) mask) exactly as masked, and its lists are the union of each tile's elements."""
    rng = np.random.default_rng(42)
    K, N, G, M = 320, 384, 128, 200
    W = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    # structured magnitudes, so that the remainder does not touch every row of every tile
    W *= (rng.random((K, 1)) < 0.5) * 0.9 + 0.1
    scores = twprune.img2col_forward([W])
    mask = twprune.tiled_wise_1d_mix(scores, 70, G, 2)[0]
    table = po.tiles_every_g_columns(N, G)
    with pytest.raises(tw.TwError) as e:
        tw.Plan.from_mask_tiles(mask, table, dtype, W)
    assert e.value.status == tw.ERR_NOT_TW
    with tw.Plan.from_mask_tiles(mask, table, dtype, W, cover=True) as plan:
        ex, _ = plan.export(with_weight=False)
        want = po.cover_tiles_from_mask(mask, table)
        for t, wt in zip(ex, want):
            assert t["kept_k"].tolist() == wt["kept_k"] and t["kept_n"].tolist() == wt["kept_n"]
        A = rng.standard_normal((M, K)).astype(np.float32)
        C, _ = run_gemm(tw, oracle, plan, A, dtype, N, pruned=1)
        ref = oracle.quantize(A, dtype).astype(np.float64) @ (oracle.quantize(W, dtype) * mask).astype(np.float64)
        assert oracle.rel_error(C, ref) <= (1e-2 if dtype == "f16" else 2e-2)
    # a tile-wise mask gives the same plan with and without `cover`
    m1 = twprune.tiled_wise_1d(scores, 70, G)[0]
    with tw.Plan.from_mask_tiles(m1, table, dtype, W) as p1, \
            tw.Plan.from_mask_tiles(m1, table, dtype, W, cover=True) as p2:
        (t1, b1), (t2, b2) = p1.export(), p2.export()
        assert np.array_equal(b1, b2)
        for a, b in zip(t1, t2):
            assert np.array_equal(a["kept_k"], b["kept_k"]) and np.array_equal(a["kept_n"], b["kept_n"])


VGG16_LAYERS = [(27, 64), (576, 64), (576, 128), (1152, 128), (1152, 256), (2304, 256), (2304, 256),
                (2304, 512), (4608, 512), (4608, 512), (4608, 512), (4608, 512), (4608, 512),
                (4096, 4096)]


def test_full_size_network_all_producers(twprune, po):
    """A VGG16-sized list of score matrices (31.6 M elements, the 13 conv layers as im2col
    matrices and one 4096 x 4096 dense layer): every producer returns the oracle's masks bit for
    bit, and the kept fractions are the requested ones."""
    rng = np.random.default_rng(20200615)
    scores = [np.abs(rng.standard_normal(s)).astype(np.float32) for s in VGG16_LAYERS]
    total = sum(k * n for k, n in VGG16_LAYERS)
    print("full size: 1d", flush=True)
    want, _, _ = po.tiled_wise_1d(scores, 75, 128)
    got = twprune.tiled_wise_1d(scores, 75, 128)
    assert all(np.array_equal(w, g) for w, g in zip(want, got))
    assert abs(sum(int(g.sum()) for g in got) / total - 0.25) < 0.01
    print("full size: 2d", flush=True)
    want = po.tiled_wise_2d(scores, 75, 128)[0]
    got = twprune.tiled_wise_2d(scores, 75, 128)
    assert all(np.array_equal(w, g) for w, g in zip(want, got))
    print("full size: 1d mix", flush=True)
    want = po.tiled_wise_1d_mix(scores, 75, 128, 5)
    got = twprune.tiled_wise_1d_mix(scores, 75, 128, 5)
    assert all(np.array_equal(w, g) for w, g in zip(want, got))
    # TW at 80 % plus the top 5 % of the shifted element scores: between 20 % and 25 % kept
    kept = sum(int(g.sum()) for g in got) / total
    assert 0.20 < kept <= 0.2501
    print("full size: 2d mix", flush=True)
    want = po.tiled_wise_2d_mix(scores, 75, 128, 1)
    got = twprune.tiled_wise_2d_mix(scores, 75, 128, 1)
    assert all(np.array_equal(w, g) for w, g in zip(want, got))


def _mixed_layer(rng, twprune, K, N, G, sparsity, g1, structured):
    """Weight, the TW mask of the mixed producer's first stage and the mixed mask."""
    W = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    if structured:
        W *= (rng.random((K, 1)) < 0.5) * 0.9 + 0.1
    scores = twprune.img2col_forward([W])
    mask = twprune.tiled_wise_1d_mix(scores, sparsity, G, g1)[0]
    mask0 = twprune.tiled_wise_1d(scores, sparsity + g1, G)[0]
    assert not (mask0 & ~mask).any()          # the mixed mask only adds elements
    return W, mask0, mask


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M", [200, 513, 2100, 4300])
def test_side_kernel_runs_the_remainder(tw, twprune, po, oracle, dtype, M):
    """TW plan of the first stage's mask + tw_side_gemm on what the second stage adds = the masked
    layer A (B (.) mask) of the mixed mask.  The two passes round their results to 16 bits one
    after the other, so an element's error is relative to the larger of the tile-wise part and
    the sum (where the remainder cancels the tile-wise part, the first rounding stays): within
    the GEMM tolerance of the float64 products of the 16-bit operands on that scale.  The side
    call alone adds exactly the remainder's product (checked against a launch on zeros, one
    rounding: plain relative error), leaves columns without remainder elements and the padding
    beyond M untouched, and repeats bit for bit.  A die takes whole 256-row chunks in rounds of
    eight and the chunks left over are shared: M = 200 and 513 have left-over chunks only, 2100
    (nine chunks) one round and one left over, 4300 (seventeen) two rounds and one left over."""
    import torch
    from tests.test_gpu_gemm import to_device_bits, from_device_bits, round_up, SENTINEL
    rng = np.random.default_rng(77 + M)
    K, N, G = 320, 384, 128
    W, mask0, mask = _mixed_layer(rng, twprune, K, N, G, 70, 2, structured=True)
    rem = mask & ~mask0
    rem[:, 5] = False                          # a column without remainder elements
    rem[:, 300:310] = False
    mask = mask0 | rem
    table = po.tiles_every_g_columns(N, G)
    A = rng.standard_normal((M, K)).astype(np.float32)
    lda = ldc = round_up(M, 8) + 8
    At = np.zeros((K, lda), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    dA = to_device_bits(At, At.shape)
    s = torch.cuda.current_stream().cuda_stream
    tol = 1e-2 if dtype == "f16" else 2e-2
    with tw.Plan.from_mask_tiles(mask0, table, dtype, W) as plan, tw.Side(rem, dtype, W) as side:
        assert side.nnz == int(rem.sum())
        outs = []
        for rep in range(2):
            dC = to_device_bits(np.full((N, ldc), SENTINEL, np.uint16), (N, ldc))
            print("side test: plan + side", M, dtype, rep, flush=True)
            plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, pruned_cols=tw.PRUNED_ZERO, stream=s)
            side.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, stream=s)
            torch.cuda.synchronize()
            outs.append(from_device_bits(dC))
        assert np.array_equal(outs[0], outs[1])
        assert (outs[0][:, M:] == SENTINEL).all()
        C = oracle.bits_to_f32(outs[0][:, :M], dtype).reshape(N, M).T
        Aq, Wq = oracle.quantize(A, dtype).astype(np.float64), oracle.quantize(W, dtype).astype(np.float64)
        ref, ref_tw = Aq @ (Wq * mask), Aq @ (Wq * mask0)
        floor = 1e-2 * np.sqrt(np.mean(ref * ref))
        assert np.max(np.abs(C - ref) / np.maximum(np.maximum(np.abs(ref), np.abs(ref_tw)), floor)) <= tol
        # the side call alone, on zeros, with alpha: exactly alpha * A (W (.) rem), one rounding
        dZ = to_device_bits(np.zeros((N, ldc), np.uint16), (N, ldc))
        side.gemm(dA.data_ptr(), dZ.data_ptr(), M, lda=lda, ldc=ldc, alpha=-0.5, stream=s)
        torch.cuda.synchronize()
        Z = from_device_bits(dZ)
        untouched = ~rem.any(axis=0)
        assert (Z[untouched] == 0).all() and (Z[:, M:] == 0).all()
        Zf = oracle.bits_to_f32(Z[:, :M], dtype).reshape(N, M).T
        assert oracle.rel_error(Zf, -0.5 * (Aq @ (Wq * rem))) <= tol


def test_side_edge_cases_and_errors(tw):
    import torch
    K, N, M = 64, 40, 16
    W = np.ones((K, N), np.float32)
    dA = torch.ones((K, M), dtype=torch.float16, device="cuda")
    dC = torch.full((N, M), 3.0, dtype=torch.float16, device="cuda")
    with tw.Side(np.zeros((K, N), bool), "f16", W) as side:       # an empty remainder does nothing
        assert side.nnz == 0
        side.gemm(dA.data_ptr(), dC.data_ptr(), M)
        torch.cuda.synchronize()
        assert (dC == 3.0).all()
    full = np.ones((K, N), bool)
    with tw.Side(full, "f16", W) as side:                         # every element: a dense product
        assert side.nnz == K * N
        side.gemm(dA.data_ptr(), dC.data_ptr(), 0)                # M = 0: nothing
        side.gemm(dA.data_ptr(), dC.data_ptr(), M)
        torch.cuda.synchronize()
        assert (dC == 3.0 + K).all()
        with pytest.raises(tw.TwError):
            side.gemm(0, dC.data_ptr(), M)
        with pytest.raises(tw.TwError):
            side.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=M - 8)
        with pytest.raises(tw.TwError):
            side.gemm(dA.data_ptr(), dC.data_ptr(), M, ldc=M + 4)
        with pytest.raises(tw.TwError):
            side.gemm(dA.data_ptr() + 2, dC.data_ptr(), M)
    with pytest.raises(ValueError):
        tw.Side(full, "f16", W[:, :3])
