"""CPU oracle of the tile-wise mask producers (test infrastructure only).

Restates, with NumPy, what the reference's pruning scripts compute when they turn a
network's importance scores into tile-wise (TW) masks:

* ``tiled_wise_1d``  - Pruning/VGG/prune_algo.py:114-148 (BERT pruning type 7,
  Pruning/BERT/utils/MyHook.py:226-259, is the same computation for N % G == 0);
* ``tiled_wise_2d``  - Pruning/VGG/prune_algo.py:55-112 (BERT type 8,
  MyHook.py:261-313, is the same without the sparsity transform of line 61);
* ``granularity_pruning`` - MyHook.py:202-214 (one threshold per tile);
* ``tw_mix_fn``, ``tiled_wise_1d_mix``, ``tiled_wise_2d_mix`` - prune_algo.py:151-193 (a TW mask
  plus the largest remaining single elements).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module; the product path (tilesparsity_amd.twprune -> libtwgemm.so) never does.

What the masks depend on, bit for bit, and how this file pins it:

* the norms: ``np.linalg.norm(w, axis=1) / w.shape[1]`` on float32 data is
  ``sqrt(add.reduce(w*w, axis=1))`` in float32.  ``row_norm_model`` / ``col_norm_model``
  restate the summation order (NumPy's pairwise sum with 8 accumulators along the
  contiguous axis, plain row-by-row accumulation along axis 0); tests compare them with
  ``np.linalg.norm`` itself on all widths 1..300, so the HIP kernels can be checked against
  either.
* the threshold: ``np.percentile(values, q)`` with linear interpolation.  Its arithmetic type
  follows the type of ``q`` (a Python number is divided by float32(100) and everything stays
  float32; a NumPy float64 keeps the quantile, the virtual index and the interpolation in
  float64).  ``percentile_model`` restates that; tests compare it with ``np.percentile`` on
  random and tie-heavy inputs.
* the comparisons are strict (``>``): an element equal to the threshold is pruned.

Parity with the reference's own files is pinned by tests/golden/prune_vectors.npz, written
by tests/golden/make_prune_vectors.py from Pruning/VGG/prune_algo.py under the NumPy of this
image (2.2.6).  The reference's published environment used an older NumPy whose percentile
interpolates in float64 for every input; the two can differ only when a norm ties with the
threshold to the last bit.  granularity_pruning has no vectors from the reference (MyHook.py
imports TensorFlow, which this image lacks); it is pinned by a brute-force check on small inputs
(norms by plain sums, the percentile from the two order statistics by hand, kept rows = those
strictly above it) and by its one-tile case, which must keep the rows tiled_wise_1d keeps.
"""
import numpy as np

F32 = np.float32


# --------------------------------------------------------------------------------------
# tile tables
# --------------------------------------------------------------------------------------
def tiles_every_g_columns(n_cols, g):
    """(col0, width) of consecutive tiles of g original columns, last one ragged
    (prune_algo.py:119-128)."""
    return [(c, min(g, n_cols - c)) for c in range(0, n_cols, g)]


def tiles_every_g_kept_columns(col_mask, g):
    """(col0, width) of tiles that end right after their g-th kept column; the last tile
    takes what is left (prune_algo.py:76-88)."""
    n = len(col_mask)
    tiles, start, kept = [], 0, 0
    for c in range(n):
        kept += int(bool(col_mask[c]))
        if kept == g and c + 1 < n:
            tiles.append((start, c + 1 - start))
            start, kept = c + 1, 0
    tiles.append((start, n - start))
    return tiles


# --------------------------------------------------------------------------------------
# norms
# --------------------------------------------------------------------------------------
def tile_row_norms(score, tiles):
    """[len(tiles), K] float32: L2 norm of every row inside every tile, divided by the
    tile's width (prune_algo.py:92, 130)."""
    score = np.asarray(score, F32)
    return np.stack([np.linalg.norm(score[:, c0:c0 + w], axis=1) / w for c0, w in tiles])


def col_norms(score):
    """[N] float32: L2 norm of every column divided by K (prune_algo.py:64)."""
    score = np.asarray(score, F32)
    return np.linalg.norm(score, axis=0) / score.shape[0]


def _pairwise(a):
    n = len(a)
    if n < 8:
        r = F32(0)
        for v in a:
            r = F32(r + v)
        return r
    if n <= 128:
        r = [F32(a[j]) for j in range(8)]
        i = 8
        while i < n - (n % 8):
            for j in range(8):
                r[j] = F32(r[j] + a[i + j])
            i += 8
        res = F32(F32(F32(r[0] + r[1]) + F32(r[2] + r[3])) + F32(F32(r[4] + r[5]) + F32(r[6] + r[7])))
        while i < n:
            res = F32(res + a[i])
            i += 1
        return res
    n2 = n // 2
    n2 -= n2 % 8
    return F32(_pairwise(a[:n2]) + _pairwise(a[n2:]))


def row_norm_model(row):
    """float32 norm of one tile row, divided by its width, in the exact operation order
    NumPy uses (pure Python: small inputs only)."""
    row = np.asarray(row, F32)
    sq = (row * row).astype(F32)
    return F32(np.sqrt(_pairwise(sq))) / F32(len(row))


def col_norm_model(score):
    """float32 column norms / K with the rows accumulated one after the other."""
    score = np.asarray(score, F32)
    acc = np.zeros(score.shape[1], F32)
    for i in range(score.shape[0]):
        acc = (acc + score[i] * score[i]).astype(F32)
    return np.sqrt(acc).astype(F32) / F32(score.shape[0])


# --------------------------------------------------------------------------------------
# threshold
# --------------------------------------------------------------------------------------
def percentile_model(values, q, q_is_f64):
    """np.percentile(values, q) for a float32 vector, restated: the k-th and (k+1)-th order
    statistics and NumPy's two-sided linear interpolation, in float32 when ``q`` is a Python
    number and in float64 when it is a NumPy float64."""
    v = np.sort(np.asarray(values, F32))
    n = len(v)
    if q_is_f64:
        quant = np.float64(q) / np.float64(100)
        virt = np.float64(n - 1) * quant
        T = np.float64
    else:
        quant = F32(q) / F32(100)
        virt = F32(n - 1) * quant
        T = F32
    if virt >= n - 1:
        lo = hi = n - 1
    elif virt < 0:
        lo = hi = 0
    else:
        lo = int(np.floor(virt))
        hi = lo + 1
    gamma = T(virt - T(np.floor(virt)))
    a, b = v[lo], v[hi]
    diff = F32(b - a)                      # float32 - float32
    if gamma >= 0.5:
        return T(b) - T(T(diff) * T(T(1) - gamma)) if q_is_f64 else F32(b - F32(diff * F32(F32(1) - gamma)))
    return T(a) + T(T(diff) * gamma) if q_is_f64 else F32(a + F32(diff * gamma))


# --------------------------------------------------------------------------------------
# the producers
# --------------------------------------------------------------------------------------
def tiled_wise_1d(scores, sparsity, granularity=128):
    """One global threshold over every (layer, tile, row) norm; a tile row is kept iff its
    norm is above it.  ``scores``: list of float32 [K_l, N_l].  Returns (masks, threshold,
    tile tables); masks are bool [K_l, N_l].  prune_algo.py:114-148."""
    scores = [np.asarray(s, F32) for s in scores]
    tables = [tiles_every_g_columns(s.shape[1], granularity) for s in scores]
    norms = [tile_row_norms(s, t) for s, t in zip(scores, tables)]
    pool = np.concatenate([n.ravel() for n in norms])
    thr = np.percentile(pool, sparsity)
    masks = []
    for s, t, n in zip(scores, tables, norms):
        m = np.zeros(s.shape, bool)
        for (c0, w), row_norm in zip(t, n):
            m[:, c0:c0 + w] = (row_norm > thr)[:, None]
        masks.append(m)
    return masks, thr, tables


def tiled_wise_2d(scores, sparsity, granularity=128, transform=True):
    """Columns first (global threshold over every column norm / K), then tiles that end
    after every ``granularity`` kept columns, then tile rows as in the 1-D case but on the
    column-pruned scores; the mask is the product.  With ``transform`` the sparsity is
    first mapped to 100 - sqrt(10000 - 100*s) so that the two prunings compose to it
    (prune_algo.py:61); BERT's type 8 (MyHook.py:261-313) passes it unchanged.
    Returns (masks, (thr_cols, thr_rows), tile tables, column masks)."""
    scores = [np.asarray(s, F32) for s in scores]
    if transform:
        sparsity = 100 - np.sqrt(10000 - sparsity * 100)
    cn = [col_norms(s) for s in scores]
    thr_c = np.percentile(np.concatenate(cn), sparsity)
    col_masks = [n > thr_c for n in cn]
    pruned = [s * cm[None, :] for s, cm in zip(scores, col_masks)]
    tables = [tiles_every_g_kept_columns(cm, granularity) for cm in col_masks]
    norms = [tile_row_norms(s, t) for s, t in zip(pruned, tables)]
    thr_r = np.percentile(np.concatenate([n.ravel() for n in norms]), sparsity)
    masks = []
    for s, t, n, cm in zip(scores, tables, norms, col_masks):
        m = np.zeros(s.shape, bool)
        for (c0, w), row_norm in zip(t, n):
            m[:, c0:c0 + w] = (row_norm > thr_r)[:, None]
        masks.append(m & cm[None, :])
    return masks, (thr_c, thr_r), tables, col_masks


def tw_mix_fn(scores, g1percent, layer_masks):
    """Second stage of the mixed (TEW) producers, prune_algo.py:151-179: every element scores
    ||x|| over a tile of one column (sqrt(x*x) / 1 in float32) minus the TW mask (so kept
    elements drop by 1); the elements strictly above the (100 - g1percent)-th percentile of
    all of them are added to the masks.  Returns (masks, threshold)."""
    scores = [np.asarray(s, F32) for s in scores]
    vals = []
    for s, m in zip(scores, layer_masks):
        nrm = np.sqrt((s * s).astype(F32)).astype(F32) / F32(1)          # :158
        vals.append((nrm - np.asarray(m, bool).astype(F32)).astype(F32))  # :160
    thr = np.percentile(np.concatenate([v.ravel() for v in vals]), 100 - g1percent)   # :166
    return [np.asarray(m, bool) | (v > thr) for m, v in zip(layer_masks, vals)], thr


def tiled_wise_1d_mix(scores, sparsity, granularity=128, g1percent=5):
    """prune_algo.py:182-186."""
    masks, _, _ = tiled_wise_1d(scores, sparsity + g1percent, granularity)
    return tw_mix_fn(scores, g1percent, masks)[0]


def tiled_wise_2d_mix(scores, sparsity, granularity=128, g1percent=1):
    """prune_algo.py:189-193."""
    masks, _, _, _ = tiled_wise_2d(scores, sparsity + g1percent, granularity)
    return tw_mix_fn(scores, g1percent, masks)[0]


def granularity_pruning(score, sparsity, granularity):
    """One threshold per tile over that tile's row norms (not divided by the width); N must
    be a multiple of the granularity.  MyHook.py:202-214."""
    score = np.asarray(score, F32)
    assert score.shape[1] % granularity == 0
    m = np.zeros(score.shape, bool)
    for c0 in range(0, score.shape[1], granularity):
        n = np.linalg.norm(score[:, c0:c0 + granularity], axis=1)
        m[:, c0:c0 + granularity] = (n > np.percentile(n, sparsity))[:, None]
    return m


def img2col(score):
    """|w| as a 2-D [K, N] matrix: HWIO conv kernels become (H*W*I) x O
    (prune_algo.py:16-24)."""
    score = np.abs(np.asarray(score, F32))
    return score.reshape(-1, score.shape[-1]) if score.ndim == 4 else score


def tiles_from_mask(mask, g=0):
    """(col0, width) tiles for a mask whose tiling is unknown: left to right a tile takes
    columns while their kept rows equal those of its first non-empty column, at most g of them
    (0: no limit); empty columns join the tile they fall into.  Columns are compared exactly."""
    mask = np.asarray(mask) != 0
    n = mask.shape[1]
    tiles, start, kept, cur = [], 0, 0, None
    for c in range(n):
        col = mask[:, c]
        if not col.any():
            continue
        if kept > 0 and (not np.array_equal(col, cur) or (g > 0 and kept == g)):
            tiles.append((start, c - start))
            start, kept = c, 0
        cur = col
        kept += 1
    tiles.append((start, n - start))
    return tiles


def cover_tiles_from_mask(mask, table):
    """Tile dicts whose rows / columns are every row / column holding a kept element of the
    tile (the covering plan of an arbitrary mask)."""
    mask = np.asarray(mask) != 0
    return [dict(col0=int(c0), width=int(w), kept_k=np.flatnonzero(mask[:, c0:c0 + w].any(axis=1)).tolist(),
                 kept_n=np.flatnonzero(mask[:, c0:c0 + w].any(axis=0)).tolist()) for c0, w in table]


def plan_tiles_from_mask(mask, table):
    """Tile dicts (col0, width, kept_k, kept_n) of a TW mask for the given tile table; raises
    if a tile is not rows x columns."""
    mask = np.asarray(mask, bool)
    tiles = []
    for c0, w in table:
        sub = mask[:, c0:c0 + w]
        rows, cols = sub.any(axis=1), sub.any(axis=0)
        if not np.array_equal(sub, rows[:, None] & cols[None, :]):
            raise ValueError("tile at column %d is not an outer product" % c0)
        tiles.append(dict(col0=int(c0), width=int(w), kept_k=np.flatnonzero(rows).tolist(),
                          kept_n=np.flatnonzero(cols).tolist()))
    return tiles
