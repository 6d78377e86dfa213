"""GPU tests of the on-disk hand-off: an exported pruned model (exportPrunedModel,
Pruning/BERT/utils/MyHook.py:54-89) and stored mask dictionaries become plans whose GEMM equals
the reference's masked dense layer (mask_dense, Pruning/BERT/utils/modeling.py:992-1007) on the
same 16-bit operands; and layers chain, the K-major C of one being the K-major A of the next.

Tolerance: max relative error <= 1e-2 (fp16) / 2e-2 (bf16) with the 1e-2 * rms floor; pruned
columns are exactly zero (the exported bias is bias * mask_o)."""
import pickle

import numpy as np
import pytest

from tests.test_gpu_epilogue import run as run_ex
from tests.test_gpu_gemm import run_gemm

pytestmark = pytest.mark.gpu

TOL = {"f16": 1e-2, "bf16": 2e-2}


@pytest.fixture(scope="module")
def ex(tw):
    from tilesparsity_amd import twexport
    return twexport


@pytest.fixture(scope="module")
def twprune(tw):
    from tilesparsity_amd import twprune as m
    return m


@pytest.fixture(scope="module")
def po():
    from oracle import tw_prune_oracle
    return tw_prune_oracle


def random_layers(rng, shapes, keep_k=0.4, keep_n=0.7):
    layers = []
    for i, (K, N) in enumerate(shapes):
        mi = (rng.random(K) < keep_k).astype(np.float32)
        mo = (rng.random(N) < keep_n).astype(np.float32)
        layers.append(("bert/encoder/layer_%d/intermediate/dense" % i, mi, mo,
                       (rng.standard_normal((K, N)) * 0.08).astype(np.float32),
                       rng.standard_normal(N).astype(np.float32)))
    return layers


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_exported_model_runs_as_mask_dense(tw, ex, oracle, dtype, tmp_path):
    rng = np.random.default_rng(51)
    shapes = [(256, 384), (100, 520), (768, 96), (40, 8)]
    layers = random_layers(rng, shapes)
    # one layer loses every row, one keeps everything
    layers[3] = layers[3][:1] + (np.zeros(40, np.float32),) + layers[3][2:]
    layers[2] = layers[2][:1] + (np.ones(768, np.float32), np.ones(96, np.float32)) + layers[2][3:]
    path = tmp_path / "pruned_model.pkl"
    with open(path, "wb") as f:      # the reference's writer: a plain pickle of the oracle's dict
        pickle.dump(oracle.export_pruned_model(layers), f, pickle.HIGHEST_PROTOCOL)
    loaded = ex.load_pruned_model(path, dtype, K={l[0]: s[0] for l, s in zip(layers, shapes)})
    assert [l.name for l in loaded] == [l[0] for l in layers]
    for (scope, mi, mo, kernel, bias), L, (K, N) in zip(layers, loaded, shapes):
        print("layer", scope, K, N, dtype, flush=True)
        assert (L.K, L.N) == (K, N)
        assert np.array_equal(L.kept_k, np.flatnonzero(mi)) and np.array_equal(L.kept_n, np.flatnonzero(mo))
        assert np.array_equal(L.bias, bias * mo)
        M = 130
        x = rng.standard_normal((M, K)).astype(np.float32)
        C = run_ex(tw, oracle, L.plan, x, dtype, N, L.bias, tw.ACT_GELU)
        ref = oracle.mask_dense(oracle.quantize(x, dtype).astype(np.float64),
                                oracle.quantize(kernel, dtype).astype(np.float64),
                                np.outer(mi, mo), (bias * mo).astype(np.float64), "gelu")
        assert oracle.rel_error(C, ref) <= TOL[dtype]
        assert not C[:, mo == 0].any()
        L.plan.destroy()
    # without K the smallest sufficient K is used and the product is the same
    again = ex.load_pruned_model(oracle.export_pruned_model(layers[:1]), dtype)
    assert again[0].K == int(np.flatnonzero(layers[0][1])[-1]) + 1
    x = rng.standard_normal((64, again[0].K)).astype(np.float32)
    C = run_ex(tw, oracle, again[0].plan, x, dtype, again[0].N, again[0].bias, tw.ACT_NONE)
    _, mi, mo, kernel, bias = layers[0]
    k = again[0].K
    ref = oracle.mask_dense(oracle.quantize(x, dtype).astype(np.float64),
                            oracle.quantize(kernel[:k], dtype).astype(np.float64),
                            np.outer(mi[:k], mo), (bias * mo).astype(np.float64))
    assert oracle.rel_error(C, ref) <= TOL[dtype]


def test_export_argument_errors(tw):
    k = np.ones((2, 2), np.float32)
    with pytest.raises(tw.TwError):
        tw.Plan.from_export(4, 4, "f16", [0, 0], [0, 0], np.ones((3, 2), np.float32))
    with pytest.raises(tw.TwError) as e:
        tw.Plan.from_export(4, 4, "f16", [0, 3], [0, 0], k)       # row 4 is outside K = 4
    assert e.value.status == tw.ERR_INDEX_LIST
    with pytest.raises(tw.TwError):
        tw.Plan.from_export(4, 4, "f16", [1, -1], [0, 0], k)      # not ascending
    with pytest.raises(tw.TwError):
        tw.Plan.from_export(0, 4, "f16", [], [0, 0], np.ones((0, 2), np.float32))


def test_mask_dictionaries_become_plans(tw, ex, twprune, po, oracle):
    """masks.pkl of a pruning run: name -> mask in the weight's shape (conv masks HWIO)."""
    rng = np.random.default_rng(52)
    weights = {"conv3/kernel": (rng.standard_normal((3, 3, 32, 160)) * 0.1).astype(np.float32),
               "fc/kernel": (rng.standard_normal((200, 300)) * 0.1).astype(np.float32)}
    names = list(weights)
    scores = twprune.img2col_forward([weights[n] for n in names])
    for fn in ("tiled_wise_1d", "tiled_wise_2d"):
        masks2d = getattr(twprune, fn)(scores, 70, 64)
        stored = {n: m.reshape(weights[n].shape).astype(np.int64) for n, m in zip(names, masks2d)}
        blob = pickle.dumps(stored, pickle.HIGHEST_PROTOCOL)
        plans = ex.plans_from_masks(blob, weights, granularity=64)
        for n, m in zip(names, masks2d):
            K, N = m.shape
            print("masks.pkl", fn, n, K, N, flush=True)
            W = weights[n].reshape(K, N)
            tiles, _ = plans[n].export(with_weight=False)
            want = po.plan_tiles_from_mask(m, po.tiles_from_mask(m, 64))
            assert len(tiles) == len(want)
            for t, wt in zip(tiles, want):
                assert (t["col0"], t["width"]) == (wt["col0"], wt["width"])
                assert t["kept_k"].tolist() == wt["kept_k"] and t["kept_n"].tolist() == wt["kept_n"]
            A = rng.standard_normal((96, K)).astype(np.float32)
            C, _ = run_gemm(tw, oracle, plans[n], A, "f16", N, pruned=1)
            ref = oracle.quantize(A, "f16").astype(np.float64) @ (oracle.quantize(W, "f16") * m).astype(np.float64)
            assert oracle.rel_error(C, ref) <= 1e-2
            plans[n].destroy()
    # mixed masks load through the covering plan
    mixed = twprune.tiled_wise_1d_mix(scores, 70, 64, 2)
    plans = ex.plans_from_masks(dict(zip(names, mixed)), weights, granularity=64, cover=True)
    for n, m in zip(names, mixed):
        K, N = m.shape
        A = rng.standard_normal((64, K)).astype(np.float32)
        C, _ = run_gemm(tw, oracle, plans[n], A, "f16", N, pruned=1)
        ref = oracle.quantize(A, "f16").astype(np.float64) @ (oracle.quantize(weights[n].reshape(K, N), "f16") * m).astype(np.float64)
        assert oracle.rel_error(C, ref) <= 1e-2


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_layers_chain_without_a_transpose(tw, oracle, dtype):
    """C of one layer (K-major: column n at n*ldc) is the A of the next (row k at k*lda): two
    masked dense layers with fused bias + activation run back to back on device buffers."""
    import torch
    from tests.helpers import from_device_bits, random_tiles, to_device_bits
    rng = np.random.default_rng(53)
    M, K1, N1, N2, G = 264, 192, 384, 256, 128
    x = rng.standard_normal((M, K1)).astype(np.float32)
    W1 = (rng.standard_normal((K1, N1)) * 0.08).astype(np.float32)
    W2 = (rng.standard_normal((N1, N2)) * 0.08).astype(np.float32)
    b1, b2 = rng.standard_normal(N1).astype(np.float32), rng.standard_normal(N2).astype(np.float32)
    t1 = random_tiles(rng, K1, N1, G, k_keep=0.5, n_keep=0.8)
    t2 = random_tiles(rng, N1, N2, G, k_keep=0.5, n_keep=0.9)
    ld = M
    Ab = np.ascontiguousarray(oracle.cast_bits(x, dtype).reshape(M, K1).T)
    dA = to_device_bits(Ab, Ab.shape)
    dH = torch.full((N1, ld), 0x7E00, dtype=torch.int16, device="cuda")     # NaN patterns
    dY = torch.full((N2, ld), 0x7E00, dtype=torch.int16, device="cuda")
    db1, db2 = torch.from_numpy(b1).cuda(), torch.from_numpy(b2).cuda()
    s = torch.cuda.current_stream().cuda_stream
    with tw.Plan.create(K1, N1, dtype, t1, W1) as p1, tw.Plan.create(N1, N2, dtype, t2, W2) as p2:
        p1.gemm(dA.data_ptr(), dH.data_ptr(), M, lda=ld, ldc=ld, pruned_cols=tw.PRUNED_ZERO, stream=s,
                bias_ptr=db1.data_ptr(), activation=tw.ACT_RELU)
        p2.gemm(dH.data_ptr(), dY.data_ptr(), M, lda=ld, ldc=ld, pruned_cols=tw.PRUNED_ZERO, stream=s,
                bias_ptr=db2.data_ptr(), activation=tw.ACT_TANH)
        torch.cuda.synchronize()
    Y = oracle.bits_to_f32(from_device_bits(dY), dtype).reshape(N2, M).T
    m1, m2 = oracle.plan_mask(K1, N1, t1), oracle.plan_mask(N1, N2, t2)
    h = oracle.mask_dense(oracle.quantize(x, dtype).astype(np.float64), oracle.quantize(W1, dtype).astype(np.float64),
                          m1, b1.astype(np.float64), "relu")
    h = oracle.quantize(h.astype(np.float32), dtype).astype(np.float64)      # the 16-bit hand-over
    ref = oracle.mask_dense(h, oracle.quantize(W2, dtype).astype(np.float64), m2, b2.astype(np.float64), "tanh")
    assert oracle.rel_error(Y, ref) <= 2 * TOL[dtype]
