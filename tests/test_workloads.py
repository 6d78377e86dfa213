"""CPU checks of the seeded workload generators (tilesparsity_amd/workloads.py)."""
import importlib.util
import json
import os

import numpy as np

from tilesparsity_amd import workloads as W

HERE = os.path.dirname(os.path.abspath(__file__))


def _maker():
    spec = importlib.util.spec_from_file_location(
        "make_workload_digests", os.path.join(HERE, "golden", "make_workload_digests.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_tile_tables_match_committed_digests():
    golden = json.load(open(os.path.join(HERE, "golden", "workload_digests.json")))
    mk = _maker()
    seen = set()
    for name, wl in mk.configs():
        assert golden[name]["sha256"] == mk.digest(wl["tiles"]), name
        assert golden[name]["seed"] == wl["seed"]
        seen.add(name)
    assert seen == set(golden)


def test_configurations_have_the_stated_structure():
    w = W.bert_base_ffn()
    assert (w["M"], w["K"], w["N"], w["G"], len(w["tiles"])) == (4096, 768, 3072, 128, 24)
    assert all(len(t["kept_k"]) == 192 and len(t["kept_n"]) == 128 for t in w["tiles"])
    w = W.vgg16_conv4_2()
    assert (w["M"], w["K"], w["N"], len(w["tiles"])) == (12544, 4608, 512, 4)
    assert all(692 <= len(t["kept_k"]) <= 1612 and len(t["kept_n"]) == 115 for t in w["tiles"])
    w = W.nmt_lstm_gates()
    assert (w["M"], w["K"], w["N"], len(w["tiles"])) == (128, 2048, 4096, 32)
    assert all(len(t["kept_k"]) == 512 for t in w["tiles"])
    w = W.imbalance_stress()
    kts = np.array([len(t["kept_k"]) for t in w["tiles"]])
    assert len(kts) == 128 and (kts == 0).sum() == 13 and all(len(t["kept_n"]) == 51 for t in w["tiles"])
    assert 0.12 < kts[kts > 0].mean() / 4096 < 0.30      # Beta(0.5, 2) has mean 0.2
    for t in w["tiles"]:
        assert np.all(np.diff(t["kept_k"]) > 0) and np.all(np.diff(t["kept_n"]) > 0)


def test_beta_inverse_cdf_is_exact_at_known_points():
    # F(x) = 1.5 sqrt(x) - 0.5 x^1.5: the median solves s^3 - 3 s + 1 = 0, s = 2 cos(4 pi / 9)
    s = 2 * np.cos(4 * np.pi / 9)
    K = 1 << 20
    orig = W.stream_u64
    try:
        W.stream_u64 = lambda key, n: np.array([np.uint64(1) << np.uint64(63)], np.uint64)  # u = 0.5
        assert abs(W.beta_half_two_count(0, K) - round(s * s * K)) <= 1
        W.stream_u64 = lambda key, n: np.array([0], np.uint64)                               # u = 0
        assert W.beta_half_two_count(0, K) == 0
    finally:
        W.stream_u64 = orig


def test_top_l1_selection_prefers_lower_index_on_ties():
    w = W.bert_large_ffn(1, 0.25, M=8)
    _, B = w["values"]()
    t = w["tiles"][0]
    score = np.abs(B[:, :128]).astype(np.float64).sum(axis=1)
    kept = set(t["kept_k"].tolist())
    assert len(kept) == 256
    assert min(score[list(kept)]) >= max(score[[i for i in range(1024) if i not in kept]])


def test_work_accounting():
    w = W.vgg16_conv4_2()
    fk = W.flops_kept(w["M"], w["tiles"])
    assert fk == 2 * 12544 * 115 * sum(len(t["kept_k"]) for t in w["tiles"])
    assert W.flops_dense(12544, 4608, 512) == 2 * 12544 * 4608 * 512
    by = W.algorithmic_bytes(12544, 4608, 512, w["tiles"])
    assert abs(by - 128.2e6) < 0.2e6
