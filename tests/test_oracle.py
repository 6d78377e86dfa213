"""Pins the CPU oracle (oracle/) before anything is checked against it.

The reference ships no golden vectors for the TW-GEMM path, so each oracle function
is pinned by known answers derived by hand from the reference's text, by closed
forms and invariants, by brute force on tiny inputs, by the standard library's own
std::random_shuffle, and by agreement of independently written forms.
"""
import ctypes

import numpy as np
import pytest

from tests.helpers import random_tiles

i32 = ctypes.c_int32


def P(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


# ----------------------------------------------------------------------------- offsets
def test_offsets_known_answer(oracle):
    # hand-derived from convert_mask_to_offset: kept indices 1,4,5,7 minus ranks 0..3
    mask = np.array([0, 1, 0, 0, 1, 1, 0, 1], np.uint8)
    assert oracle.mask_to_offsets(mask).tolist() == [1, 3, 3, 4]
    out = np.zeros(8, np.int32)
    n = oracle.clib().ora_mask_to_offsets(P(mask, ctypes.c_uint8), 8, P(out, i32))
    assert n == 4 and out[:4].tolist() == [1, 3, 3, 4]


def test_offsets_invariants_and_round_trip(oracle):
    rng = np.random.default_rng(0)
    for n in (0, 1, 7, 64, 1000):
        for p in (0.0, 0.1, 0.5, 1.0):
            mask = (rng.random(n) < p).astype(np.uint8)
            off = oracle.mask_to_offsets(mask)
            cout = np.zeros(max(n, 1), np.int32)
            cn = oracle.clib().ora_mask_to_offsets(P(mask, ctypes.c_uint8), n, P(cout, i32))
            assert cn == off.size and np.array_equal(cout[:cn], off)
            kept = oracle.offsets_to_kept(off)
            assert np.array_equal(kept, np.flatnonzero(mask))
            if off.size:
                assert np.all(np.diff(off) >= 0) and off[0] >= 0 and off[-1] <= n - off.size
            back = np.zeros(n, np.uint8)
            back[kept] = 1
            assert np.array_equal(back, mask)


# ----------------------------------------------------------------------------- mask_gen
def test_rand_stream_known_answer(oracle):
    # glibc rand() with seed 1 starts 1804289383, 846930886, ...; init_matrix maps a
    # draw r to float(r / RAND_MAX - 0.5)  (basic_nn.cu:618)
    L = oracle.clib()
    L.ora_srand(1)
    m = np.zeros((1, 2), np.float32)
    L.ora_init_matrix(P(m, ctypes.c_float), 1, 2)
    expect = [np.float32(1804289383 / 2147483647 - 0.5), np.float32(846930886 / 2147483647 - 0.5)]
    assert m[0].tolist() == expect


@pytest.mark.parametrize("n,keep", [(8, 3), (768, 384), (256, 128), (4608, 1152), (5, 5), (3, 0)])
def test_mask_gen_matches_std_random_shuffle(oracle, n, keep):
    L, S = oracle.clib(), oracle.shuffle_lib()
    for seed in (1, 2, 12345):
        a, b = np.zeros(max(keep, 1), np.int32), np.zeros(max(keep, 1), np.int32)
        L.ora_srand(seed)
        L.ora_mask_gen(n, keep, P(a, i32))
        S.ora_std_srand(seed)
        S.ora_std_mask_gen(n, keep, P(b, i32))
        assert np.array_equal(a, b)
        kept = oracle.offsets_to_kept(a[:keep])
        assert np.all(np.diff(kept) > 0) and (keep == 0 or (kept[0] >= 0 and kept[-1] < n))


# ----------------------------------------------------------------------------- tile partition
def test_tile_partition_readme_cases(oracle):
    # StreamMaskedGEMM/README.md: 768 -> 384 kept columns, 3072 -> 1536
    p = oracle.tile_partition(12800, 768, 768, 384, 384)
    assert p["block_num"] == 3 and p["N_ori"] == [256] * 3 and p["N_cal"] == [128] * 3
    assert p["K_cal"] == [384] * 3
    assert p["off_B"] == [0, 768 * 256, 768 * 512] and p["off_C"] == [0, 12800 * 256, 12800 * 512]
    p = oracle.tile_partition(12800, 3072, 768, 1536, 384)
    assert p["block_num"] == 12 and p["N_ori"] == [256] * 12 and p["N_cal"] == [128] * 12


@pytest.mark.parametrize("args", [(64, 100, 40, 70, 10, 32), (8, 1000, 16, 333, 8, 128),
                                  (128, 128, 128, 128, 128, 128), (16, 520, 64, 200, 32, 64)])
def test_tile_partition_c_equals_python(oracle, args):
    M, N, K, Np, Kp, nd = args
    p = oracle.tile_partition(M, N, K, Np, Kp, nd)
    bn = p["block_num"]
    arrs = [np.zeros(bn, np.int32) for _ in range(5)]
    got = oracle.clib().ora_tile_partition(M, N, K, Np, Kp, nd, *[P(a, i32) for a in arrs])
    assert got == bn
    for a, key in zip(arrs, ("N_ori", "N_cal", "K_cal", "off_B", "off_C")):
        assert a.tolist() == p[key]
    assert sum(p["N_ori"]) == N and sum(p["N_cal"]) == Np


# ----------------------------------------------------------------------------- weights
def brute_weights(B, tiles):
    K, N = B.shape
    dense = np.zeros_like(B)
    stream = np.zeros(K * N, np.float32)
    for t in tiles:
        for i, k in enumerate(t["kept_k"]):
            for j, n in enumerate(t["kept_n"]):
                c = t["col0"] + int(n)
                dense[k, c] = B[k, c]
                stream[(j + t["col0"]) * K + i] = B[k, c]
    return dense, stream


def test_weights_against_brute_force_and_c(oracle):
    rng = np.random.default_rng(1)
    K, N, G = 24, 40, 16
    B = rng.standard_normal((K, N)).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=0.7, empty_every=3)
    dense, stream = brute_weights(B, tiles)
    assert np.array_equal(oracle.masked_dense_weight(B, tiles), dense)
    assert np.array_equal(oracle.stream_weight(B, tiles), stream)
    assert np.array_equal(dense, B * oracle.plan_mask(K, N, tiles))
    # plain-C restatement, driven with relative offsets like the reference
    cd, cs = np.zeros_like(B), np.zeros(K * N, np.float32)
    L = oracle.clib()
    for t in tiles:
        mk = oracle.mask_to_offsets(np.isin(np.arange(K), t["kept_k"]).astype(np.uint8))
        mn = oracle.mask_to_offsets(np.isin(np.arange(t["width"]), t["kept_n"]).astype(np.uint8))
        mk = np.ascontiguousarray(np.append(mk, 0), np.int32)
        mn = np.ascontiguousarray(np.append(mn, 0), np.int32)
        for fn, dst in ((L.ora_gen_cutlass_weight, cd), (L.ora_gen_stream_weight, cs)):
            fn(P(dst, ctypes.c_float), P(B, ctypes.c_float), K, N, P(mk, i32), P(mn, i32),
               len(t["kept_k"]), len(t["kept_n"]), t["col0"])
    assert np.array_equal(cd, dense) and np.array_equal(cs, stream)
    # identity: compact tile == (B*mask)[kept_k][:, kept_n], column-major with ld = K
    for t in tiles:
        comp = dense[np.ix_(t["kept_k"], t["kept_n"] + t["col0"])]
        blk = stream.reshape(N, K)[t["col0"]:t["col0"] + len(t["kept_n"]), :len(t["kept_k"])]
        assert np.array_equal(blk.T, comp)


def test_plan_from_mask_round_trip(oracle):
    rng = np.random.default_rng(2)
    K, N, G = 50, 70, 32
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.8, empty_every=2)
    back = oracle.plan_from_mask(oracle.plan_mask(K, N, tiles), G)
    for a, b in zip(tiles, back):
        if len(a["kept_k"]) == 0 or len(a["kept_n"]) == 0:
            assert len(b["kept_k"]) == 0 and len(b["kept_n"]) == 0
        else:
            assert np.array_equal(a["kept_k"], b["kept_k"]) and np.array_equal(a["kept_n"], b["kept_n"])


# ----------------------------------------------------------------------------- casts
def test_f16_cast_matches_numpy(oracle):
    rng = np.random.default_rng(3)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000),
        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, 65519.9, 65520.0, 1e-8, 6e-8,
                  5.96e-8, 2.98e-8, 2.99e-8, 6.1e-5, 6.097e-5, 1.0, 1.00048828125, 1.0009765625],
                 np.float32)]).astype(np.float32)
    got = np.zeros(x.size, np.uint16)
    oracle.clib().ora_cast_f32(P(x, ctypes.c_float), P(got, ctypes.c_uint16), x.size, 0)
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], ref[~nan])
    assert np.all((got[nan] & 0x7C00) == 0x7C00) and np.all((got[nan] & 0x3FF) != 0)
    assert np.array_equal(oracle.cast_bits(x, "f16")[~nan], ref[~nan])
    # every half value converts back and forth exactly
    allh = np.arange(65536, dtype=np.uint16)
    f = np.zeros(65536, np.float32)
    oracle.clib().ora_uncast_f32(P(allh, ctypes.c_uint16), P(f, ctypes.c_float), 65536, 0)
    ok = ~np.isnan(allh.view(np.float16))
    assert np.array_equal(f[ok], allh.view(np.float16).astype(np.float32)[ok])
    back = np.zeros(65536, np.uint16)
    oracle.clib().ora_cast_f32(P(f, ctypes.c_float), P(back, ctypes.c_uint16), 65536, 0)
    assert np.array_equal(back[ok], allh[ok])


def test_bf16_cast_round_to_nearest_even(oracle):
    # exact halfway cases: the 16 dropped bits are 0x8000 -> round to the even neighbour
    hi = np.array([0x3F80, 0x3F81, 0x4000, 0x7F7F, 0x0001, 0x8000 | 0x3F81], np.uint32)
    x = ((hi << 16) | 0x8000).astype(np.uint32).view(np.float32)
    expect = np.where(hi & 1, hi + 1, hi).astype(np.uint16)
    assert np.array_equal(oracle.cast_bits(x, "bf16"), expect)
    got = np.zeros(x.size, np.uint16)
    oracle.clib().ora_cast_f32(P(x, ctypes.c_float), P(got, ctypes.c_uint16), x.size, 1)
    assert np.array_equal(got, expect)
    # just below / above halfway
    below = ((hi << 16) | 0x7FFF).astype(np.uint32).view(np.float32)
    above = ((hi << 16) | 0x8001).astype(np.uint32).view(np.float32)
    assert np.array_equal(oracle.cast_bits(below, "bf16"), hi.astype(np.uint16))
    assert np.array_equal(oracle.cast_bits(above, "bf16"), (hi + 1).astype(np.uint16))
    # second formulation on random data: nearest representable, ties to even, via float64
    rng = np.random.default_rng(4)
    r = (rng.standard_normal(50000) * 10.0 ** rng.integers(-20, 20, 50000)).astype(np.float32)
    bits = oracle.cast_bits(r, "bf16")
    c = np.zeros(r.size, np.uint16)
    oracle.clib().ora_cast_f32(P(r, ctypes.c_float), P(c, ctypes.c_uint16), r.size, 1)
    assert np.array_equal(bits, c)
    val = oracle.bits_to_f32(bits, "bf16").astype(np.float64)
    lo = oracle.bits_to_f32((bits.astype(np.int32) - 1).astype(np.uint16), "bf16").astype(np.float64)
    up = oracle.bits_to_f32((bits.astype(np.int32) + 1).astype(np.uint16), "bf16").astype(np.float64)
    fin = np.isfinite(val) & np.isfinite(lo) & np.isfinite(up)
    d = np.abs(val - r)[fin]
    assert np.all(d <= np.abs(lo - r)[fin]) and np.all(d <= np.abs(up - r)[fin])
    assert oracle.cast_bits(np.array([np.inf, -np.inf], np.float32), "bf16").tolist() == [0x7F80, 0xFF80]
    nanb = oracle.cast_bits(np.array([np.nan], np.float32), "bf16")[0]
    assert (nanb & 0x7F80) == 0x7F80 and (nanb & 0x7F) != 0


# ----------------------------------------------------------------------------- GEMM forms
def c_stream_gemm(oracle, A, B, tiles, alpha, beta, C0):
    """Drives the plain-C Stream_Gemm_NN_reference restatement with reference layouts."""
    M, K = A.shape
    N = B.shape[1]
    L = oracle.clib()
    At = np.ascontiguousarray(A.T, np.float32)            # column-major M x K
    Bs = oracle.stream_weight(B, tiles)
    Ct = np.ascontiguousarray(C0.T, np.float32)           # column-major M x N
    bn = len(tiles)
    N_cal = np.array([len(t["kept_n"]) for t in tiles], np.int32)
    K_cal = np.array([len(t["kept_k"]) for t in tiles], np.int32)
    mks = [np.ascontiguousarray(np.append(t["kept_k"] - np.arange(len(t["kept_k"])), 0), np.int32)
           for t in tiles]
    mns = [np.ascontiguousarray(np.append(t["kept_n"] - np.arange(len(t["kept_n"])), 0), np.int32)
           for t in tiles]
    i32p = ctypes.POINTER(i32)
    mk = (i32p * bn)(*[P(a, i32) for a in mks])
    mn = (i32p * bn)(*[P(a, i32) for a in mns])
    off_B = np.array([K * t["col0"] for t in tiles], np.int64)
    off_C = np.array([M * t["col0"] for t in tiles], np.int64)
    L.ora_stream_gemm_nn(M, N, K, alpha, P(At, ctypes.c_float), P(Bs, ctypes.c_float), beta,
                         P(Ct, ctypes.c_float), bn, P(N_cal, i32), P(K_cal, i32), mn, mk,
                         P(off_B, ctypes.c_int64), P(off_C, ctypes.c_int64))
    return Ct.T


@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.5, 0.0), (1.0, 1.0), (-2.0, 0.25)])
def test_gemm_forms_agree(oracle, alpha, beta):
    rng = np.random.default_rng(5)
    M, K, N, G = 37, 48, 80, 32
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.75, empty_every=3)
    ref = oracle.tw_gemm_reference(A, B, tiles, alpha, beta, C0)
    form2 = oracle.stream_gemm_nn(A, B, tiles, alpha, beta, C0)
    form3 = c_stream_gemm(oracle, A, B, tiles, alpha, beta, C0)
    np.testing.assert_allclose(form2, ref, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(form3, ref, rtol=2e-6, atol=2e-6)
    # textbook: matmul with the masked weight on the kept columns, C untouched elsewhere
    mask = oracle.plan_mask(K, N, tiles)
    kept_cols = np.zeros(N, bool)
    for t in tiles:
        kept_cols[t["kept_n"] + t["col0"]] = True
    plain = alpha * (A.astype(np.float64) @ (B * mask).astype(np.float64)) + beta * C0
    np.testing.assert_allclose(ref[:, kept_cols], plain[:, kept_cols], rtol=1e-12, atol=1e-12)
    assert np.array_equal(ref[:, ~kept_cols], C0[:, ~kept_cols].astype(np.float64))


def test_gemm_special_cases(oracle):
    rng = np.random.default_rng(6)
    M, K, N, G = 20, 32, 64, 16
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    # all kept -> plain GEMM
    full = [dict(col0=c, width=G, kept_k=np.arange(K, dtype=np.int32),
                 kept_n=np.arange(G, dtype=np.int32)) for c in range(0, N, G)]
    np.testing.assert_allclose(oracle.tw_gemm_reference(A, B, full),
                               A.astype(np.float64) @ B.astype(np.float64), rtol=1e-12)
    # identity weight, one tile, G = N = K: C = A with pruned rows zeroed / columns dropped
    eye = np.eye(K, dtype=np.float32)
    kk = np.array([1, 5, 6, 30], np.int32)
    one = [dict(col0=0, width=K, kept_k=kk, kept_n=np.arange(K, dtype=np.int32))]
    out = oracle.tw_gemm_reference(A, eye, one)
    expect = np.zeros((M, K))
    expect[:, kk] = A[:, kk]
    assert np.array_equal(out, expect)
    # K_t == 0 -> zeros on the kept columns; N_t == 0 -> nothing written
    empty = [dict(col0=0, width=N, kept_k=np.zeros(0, np.int32), kept_n=np.arange(3, dtype=np.int32))]
    C0 = np.full((M, N), 7.0, np.float32)
    out = oracle.tw_gemm_reference(A, B, empty, C=C0)
    assert np.all(out[:, :3] == 0) and np.all(out[:, 3:] == 7)
    # mask_dense == numpy matmul (+ bias), C restatement agrees
    mask = oracle.plan_mask(K, N, random_tiles(rng, K, N, G))
    bias = rng.standard_normal(N).astype(np.float32)
    y = oracle.mask_dense(A, B, mask, bias)
    np.testing.assert_allclose(y, A @ (B * mask) + bias, rtol=1e-6, atol=1e-6)
    yc = np.zeros((M, N), np.float32)
    oracle.clib().ora_mask_dense(P(A, ctypes.c_float), P(B, ctypes.c_float), P(mask, ctypes.c_uint8),
                                 P(bias, ctypes.c_float), P(yc, ctypes.c_float), M, K, N)
    np.testing.assert_allclose(yc, y, rtol=1e-5, atol=1e-5)


def test_delete_insert_row(oracle):
    rng = np.random.default_rng(7)
    rows, cols = 9, 5
    src = rng.standard_normal((rows, cols)).astype(np.float32)
    kept = np.array([0, 3, 4, 8], np.int32)
    rel = np.ascontiguousarray(kept - np.arange(4), np.int32)
    out = np.zeros((4, cols), np.float32)
    oracle.clib().ora_delete_row(P(src, ctypes.c_float), P(out, ctypes.c_float), 4, cols, P(rel, i32))
    assert np.array_equal(out, src[kept])
    dst = np.zeros((rows, cols), np.float32)
    oracle.clib().ora_insert_row(P(dst, ctypes.c_float), P(out, ctypes.c_float), 4, cols, P(rel, i32))
    expect = np.zeros_like(dst)
    expect[kept] = src[kept]
    assert np.array_equal(dst, expect)


# ----------------------------------------------------------------------------- checkout
def test_checkout_rule(oracle):
    a = np.array([[1.0, 2.0, 0.0, 100.0]], np.float32)
    assert oracle.checkout(a, a.copy(), err=1e-10) == 0            # includes 0/0 -> passes
    b = a.copy()
    b[0, 3] = 100.5                                                 # ratio 1.005 ok, |diff| 0.5 > 0.01
    assert oracle.checkout(a, b, err=1e-2) == 1
    c = a.copy()
    c[0, 0] = 1.02                                                  # ratio 1.02 > 1.01
    assert oracle.checkout(a, c, err=1e-2) == 1
    d = a.copy()
    d[0, 1] = 2.005                                                 # within both bounds
    assert oracle.checkout(a, d, err=1e-2) == 0
    # C restatement agrees, including the transposed read of the reference operand
    rng = np.random.default_rng(8)
    x = rng.standard_normal((6, 4)).astype(np.float32)
    y = (x + rng.standard_normal((6, 4)).astype(np.float32) * 0.01).astype(np.float32)
    yt = np.ascontiguousarray(y.T)
    n_py = oracle.checkout(x, y, err=1e-2)
    n_c = oracle.clib().ora_checkout(P(x, ctypes.c_float), P(yt, ctypes.c_float), 6, 4, 1, 1e-2)
    assert n_py == n_c == oracle.checkout(x, yt, trans=True, err=1e-2)


def test_ref_compat_problem(oracle):
    A, B, tiles, part = oracle.ref_compat_problem(16, 768, 64, 384, 32)
    assert A[0, 0] == np.float32(1804289383 / 2147483647 - 0.5)
    assert part["block_num"] == 3 and [t["width"] for t in tiles] == [256] * 3
    assert all(len(t["kept_k"]) == 32 and len(t["kept_n"]) == 128 for t in tiles)
    A2, B2, tiles2, _ = oracle.ref_compat_problem(16, 768, 64, 384, 32)
    assert np.array_equal(A, A2) and np.array_equal(B, B2)
    assert all(np.array_equal(a["kept_k"], b["kept_k"]) for a, b in zip(tiles, tiles2))


def test_gelu_and_mask_dense_epilogue():
    """gelu: known values of the tanh form (0 -> 0, large x -> x, large -x -> 0, odd part x/2);
    mask_dense with bias and activation against a loop."""
    from oracle import tw_oracle as o
    import math
    assert o.gelu(0.0) == 0.0
    assert abs(o.gelu(10.0) - 10.0) < 1e-6 and abs(o.gelu(-10.0)) < 1e-6
    for x in (0.3, 1.0, 2.5):
        assert abs((o.gelu(x) - o.gelu(-x)) - x) < 1e-12        # gelu(x) - gelu(-x) = x
        want = 0.5 * x * (1 + math.tanh(math.sqrt(2 / math.pi) * (x + 0.044715 * x ** 3)))
        assert abs(o.gelu(x) - want) < 1e-12
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 7)).astype(np.float32)
    w = rng.standard_normal((7, 6)).astype(np.float32)
    m = (rng.random((7, 6)) < 0.5).astype(np.float32)
    b = rng.standard_normal(6).astype(np.float32)
    y = o.mask_dense(x, w, m, b, "relu")
    for i in range(5):
        for j in range(6):
            v = sum(float(x[i, k]) * float(w[k, j]) * float(m[k, j]) for k in range(7)) + float(b[j])
            assert abs(y[i, j] - max(v, 0.0)) < 1e-4
    # a fully pruned column still gets its bias
    m[:, 2] = 0
    assert np.allclose(o.mask_dense(x, w, m, b)[:, 2], b[2])


def test_basic_lstm_cell_closed_forms(oracle):
    """BasicLSTMCell's gate arithmetic against library routines and its limits."""
    from scipy.special import expit
    rng = np.random.default_rng(77)
    M, H = 9, 16
    g = rng.standard_normal((M, 4 * H)) * 2
    c = rng.standard_normal((M, H))
    nc, nh = oracle.basic_lstm_cell(g, c, 1.0)
    i, j, f, o = g[:, :H], g[:, H:2 * H], g[:, 2 * H:3 * H], g[:, 3 * H:]
    want_c = c * expit(f + 1.0) + expit(i) * np.tanh(j)
    assert np.allclose(nc, want_c, rtol=1e-12, atol=1e-12)
    assert np.allclose(nh, np.tanh(want_c) * expit(o), rtol=1e-12, atol=1e-12)
    # saturated gates: forget open / input shut keeps c; the opposite replaces it by tanh(j)
    big = 40.0
    keep = np.concatenate([np.full((M, H), -big), g[:, H:2 * H], np.full((M, H), big), np.full((M, H), big)], 1)
    nc, nh = oracle.basic_lstm_cell(keep, c, 0.0)
    assert np.allclose(nc, c) and np.allclose(nh, np.tanh(c))
    repl = np.concatenate([np.full((M, H), big), g[:, H:2 * H], np.full((M, H), -big), np.full((M, H), -big)], 1)
    nc, nh = oracle.basic_lstm_cell(repl, c, 0.0)
    assert np.allclose(nc, np.tanh(j)) and np.allclose(nh, 0.0, atol=1e-15)
    # zero pre-activations: c/2 (+ forget bias 0), h = tanh(c/2)/2
    nc, nh = oracle.basic_lstm_cell(np.zeros((M, 4 * H)), c, 0.0)
    assert np.allclose(nc, c / 2) and np.allclose(nh, np.tanh(c / 2) / 2)
    # the gate order is i, j, f, o: a transposed split would fail this
    one = np.zeros((1, 4)); one[0, 2] = big                    # only f saturated, H = 1
    nc, _ = oracle.basic_lstm_cell(one, np.array([[3.0]]), 0.0)
    assert np.allclose(nc, 3.0)
