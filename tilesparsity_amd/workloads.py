"""Seeded synthetic TW-GEMM workloads: the five benchmark configurations.

Tile tables (kept-K counts, kept rows, kept columns) come from one integer-only
counter-based generator (splitmix64 keyed by seed, configuration, tile and
stream), so they are identical on every machine and NumPy version.  Value
tensors come from numpy's PCG64 (`default_rng(seed)`).

A workload is a dict: name, M, K, N, G, dtype, tiles (list of dicts with col0,
width, kept_k, kept_n), seed, and `values()` -> (A[M,K] fp32, B[K,N] fp32).
"""
import numpy as np

DEFAULT_SEED = 20200613
_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_MASK = (1 << 64) - 1


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def _mix_int(z):
    z &= _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def stream_key(seed, cfg, tile, stream_id):
    """64-bit key of one random stream."""
    k = _mix_int(seed + 0x9E3779B97F4A7C15)
    for v in (cfg, tile, stream_id):
        k = _mix_int(k ^ _mix_int(v + 0x9E3779B97F4A7C15))
    return k


def stream_u64(key, n):
    """n values of splitmix64 started at `key`."""
    with np.errstate(over="ignore"):
        ctr = np.uint64(key) + np.arange(1, n + 1, dtype=np.uint64) * _GAMMA
        return _mix(ctr)


def choose_sorted(key, n, n_keep):
    """n_keep distinct indices of range(n), ascending: the n_keep smallest random keys."""
    if n_keep <= 0:
        return np.zeros(0, np.int32)
    order = np.argsort(stream_u64(key, n), kind="stable")
    return np.sort(order[:n_keep]).astype(np.int32)


def uniform_int(key, lo, hi):
    return lo + int(stream_u64(key, 1)[0] % np.uint64(hi - lo + 1))


def beta_half_two_count(key, K):
    """round(K * X), X ~ Beta(0.5, 2), by exact integer inversion of the CDF
    F(x) = 1.5 sqrt(x) - 0.5 x^1.5: with s = sqrt(x) in Q31, the smallest s with
    3 s 2^62 - s^3 >= 2 u 2^62."""
    u = int(stream_u64(key, 1)[0] >> np.uint64(33))  # 31 random bits, Q31
    target = (2 * u) << 62
    lo, hi = 0, 1 << 31
    while lo < hi:
        mid = (lo + hi) // 2
        if 3 * mid * (1 << 62) - mid ** 3 >= target:
            hi = mid
        else:
            lo = mid + 1
    return int((lo * lo * K + (1 << 61)) >> 62)


def _uniform_tiles(N, G):
    return [(c, min(G, N - c)) for c in range(0, N, G)]


def _finish(name, M, K, N, G, dtype, tiles, seed, values):
    return dict(name=name, M=M, K=K, N=N, G=G, dtype=dtype, tiles=tiles, seed=seed, values=values)


def bert_base_ffn(seed=None, M=4096, K=768, N=3072, G=128):
    """Config 1: BERT-base FFN-in; 75 % of the K rows pruned per tile, rows chosen
    uniformly per tile, no column pruning.  A ~ N(0,1), B ~ N(0,0.02)."""
    seed = DEFAULT_SEED + 1 if seed is None else seed
    tiles = []
    for t, (c0, w) in enumerate(_uniform_tiles(N, G)):
        tiles.append(dict(col0=c0, width=w,
                          kept_k=choose_sorted(stream_key(seed, 1, t, 0), K, K // 4),
                          kept_n=np.arange(w, dtype=np.int32)))

    def values():
        rng = np.random.default_rng(seed)
        return (rng.standard_normal((M, K), dtype=np.float32),
                (rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)))
    return _finish("bert_base_ffn_in", M, K, N, G, "f16", tiles, seed, values)


def vgg16_conv4_2(seed=None, M=12544, K=4608, N=512, G=128):
    """Config 2: VGG16 conv4_2 as im2col; per-tile kept-K uniform in [0.15K, 0.35K],
    10 % of the columns pruned per tile.  A = ReLU(N(0,1)), B ~ N(0, sqrt(2/K))."""
    seed = DEFAULT_SEED + 2 if seed is None else seed
    lo, hi = -(-15 * K // 100), 35 * K // 100
    tiles = []
    for t, (c0, w) in enumerate(_uniform_tiles(N, G)):
        kt = uniform_int(stream_key(seed, 2, t, 2), lo, hi)
        n_pruned = (w * 10 + 50) // 100  # 10 % of the tile's columns, rounded
        tiles.append(dict(col0=c0, width=w,
                          kept_k=choose_sorted(stream_key(seed, 2, t, 0), K, kt),
                          kept_n=choose_sorted(stream_key(seed, 2, t, 1), w, w - n_pruned)))

    def values():
        rng = np.random.default_rng(seed)
        A = np.maximum(rng.standard_normal((M, K), dtype=np.float32), 0)
        B = rng.standard_normal((K, N), dtype=np.float32) * np.float32(np.sqrt(2.0 / K))
        return A, B
    return _finish("vgg16_conv4_2_im2col", M, K, N, G, "f16", tiles, seed, values)


def nmt_lstm_gates(seed=None, M=128, K=2048, N=4096, G=128):
    """Config 3: NMT LSTM gate GEMM, skinny M; 75 % uniform sparsity.
    A ~ U(-1,1), B ~ N(0,0.03)."""
    seed = DEFAULT_SEED + 3 if seed is None else seed
    tiles = []
    for t, (c0, w) in enumerate(_uniform_tiles(N, G)):
        tiles.append(dict(col0=c0, width=w,
                          kept_k=choose_sorted(stream_key(seed, 3, t, 0), K, K // 4),
                          kept_n=np.arange(w, dtype=np.int32)))

    def values():
        rng = np.random.default_rng(seed)
        A = rng.uniform(-1.0, 1.0, (M, K)).astype(np.float32)
        B = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.03)
        return A, B
    return _finish("nmt_lstm_gates", M, K, N, G, "f16", tiles, seed, values)


def bert_large_ffn(which=1, keep=0.25, seed=None, M=8192, G=128):
    """Config 4: BERT-large FFN pair in bf16; `which` 1: K=1024,N=4096; 2: K=4096,N=1024.
    Per tile the round(keep*K) rows with the largest L1 score sum_j |w[r,j]| are kept
    (ties -> lower index).  A ~ N(0,1), W ~ N(0,0.02)."""
    seed = DEFAULT_SEED + 4 if seed is None else seed
    K, N = (1024, 4096) if which == 1 else (4096, 1024)
    rng = np.random.default_rng(seed + 1000 * which)
    B = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)
    kt = int(np.floor(keep * K + 0.5))
    tiles = []
    for c0, w in _uniform_tiles(N, G):
        score = np.abs(B[:, c0:c0 + w]).astype(np.float64).sum(axis=1)
        order = np.argsort(-score, kind="stable")[:kt]
        tiles.append(dict(col0=c0, width=w, kept_k=np.sort(order).astype(np.int32),
                          kept_n=np.arange(w, dtype=np.int32)))

    def values():
        rng_a = np.random.default_rng(seed + 1000 * which + 1)
        return rng_a.standard_normal((M, K), dtype=np.float32), B
    return _finish("bert_large_ffn%d_keep%02d" % (which, int(round(keep * 100))), M, K, N, G,
                   "bf16", tiles, seed, values)


def imbalance_stress(seed=None, M=16384, K=4096, N=8192, G=64, empty_frac=0.10):
    """Config 5: load-imbalance stress; per-tile kept-K = round(Beta(0.5,2)*K), 20 % of
    the columns pruned per tile, a tenth of the tiles fully pruned (K_t = 0, kept
    columns then receive zeros).  A ~ N(0,1), B ~ N(0,0.02)."""
    seed = DEFAULT_SEED + 5 if seed is None else seed
    tt = _uniform_tiles(N, G)
    empty = set(choose_sorted(stream_key(seed, 5, 0, 3), len(tt),
                              int(np.floor(empty_frac * len(tt) + 0.5))).tolist())
    tiles = []
    for t, (c0, w) in enumerate(tt):
        kt = 0 if t in empty else beta_half_two_count(stream_key(seed, 5, t, 2), K)
        n_pruned = (w * 20 + 50) // 100
        tiles.append(dict(col0=c0, width=w,
                          kept_k=choose_sorted(stream_key(seed, 5, t, 0), K, kt),
                          kept_n=choose_sorted(stream_key(seed, 5, t, 1), w, w - n_pruned)))

    def values():
        rng = np.random.default_rng(seed)
        return (rng.standard_normal((M, K), dtype=np.float32),
                rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02))
    return _finish("imbalance_stress", M, K, N, G, "f16", tiles, seed, values)


def dense_tiles(K, N, G):
    """The 0 %-sparse tile table."""
    return [dict(col0=c0, width=w, kept_k=np.arange(K, dtype=np.int32),
                 kept_n=np.arange(w, dtype=np.int32)) for c0, w in _uniform_tiles(N, G)]


# --------------------------------------------------------------------------- work accounting
def flops_kept(M, tiles):
    return 2 * M * sum(len(t["kept_k"]) * len(t["kept_n"]) for t in tiles)


def flops_dense(M, K, N):
    return 2 * M * K * N


def algorithmic_bytes(M, K, N, tiles, elem=2, pruned_untouched=True):
    """A once + packed weight once + C once (kept columns only when pruned columns
    stay untouched) + the index lists."""
    kept_w = sum(len(t["kept_k"]) * len(t["kept_n"]) for t in tiles)
    sum_n = sum(len(t["kept_n"]) for t in tiles)
    idx = 4 * sum(len(t["kept_k"]) + len(t["kept_n"]) for t in tiles)
    c_cols = sum_n if pruned_untouched else N
    return M * K * elem + kept_w * elem + M * c_cols * elem + idx
