"""TW mask producers on the GPU, with the reference's function names and argument meaning
(Pruning/VGG/prune_algo.py: img2col_forward, tiled_wise_1d, tiled_wise_2d, tw_mix_fn,
tiled_wise_1d_mix, tiled_wise_2d_mix; BERT pruning types 7 and 8 of Pruning/BERT/utils/MyHook.py
are tiled_wise_1d and tiled_wise_2d(transform=False)).

    masks = tiled_wise_1d(scores, sparsity, granularity)     # list of bool [K, N] arrays

`scores` is a list of float32 arrays (2-D, or 4-D HWIO conv kernels, which are viewed as
(H*W*I) x O).  The work runs in libtwgemm.so (HIP); there is no CPU path.  As in NumPy, the type
of `sparsity` selects the arithmetic of the percentile: a Python int/float keeps it in float32,
a numpy.float64 in float64.
"""
import ctypes

import numpy as np

from . import twgemm as tw

Q_F32, Q_F64 = 0, 1


def _q_type(sparsity):
    # np.percentile: a Python number adapts to the float32 data, a NumPy float64 does not
    return Q_F64 if isinstance(sparsity, np.floating) and np.dtype(type(sparsity)).itemsize == 8 else Q_F32


def img2col_forward(accumulated_scores):
    """|w| of every layer as a 2-D matrix (prune_algo.py:16-24)."""
    out = []
    for w in accumulated_scores:
        w = np.abs(np.asarray(w, np.float32))
        out.append(w.reshape(-1, w.shape[-1]) if w.ndim == 4 else w)
    return out


class _DeviceLayers:
    """Scores uploaded to the GPU and mask buffers, as pointer tables for the C ABI."""

    def __init__(self, scores):
        import torch
        self.torch = torch
        self.shapes = []
        self.d_scores, self.d_masks, self.d_cols = [], [], []
        for s in scores:
            if isinstance(s, torch.Tensor):
                t = s.detach().to(device="cuda", dtype=torch.float32)
            else:
                t = torch.from_numpy(np.ascontiguousarray(s, dtype=np.float32)).cuda()
            if t.dim() == 4:
                t = t.reshape(-1, t.shape[-1])
            if t.dim() != 2:
                raise tw.TwError(tw.ERR_SHAPE, "a score tensor must be 2-D or 4-D")
            t = t.contiguous()
            self.shapes.append(tuple(t.shape))
            self.d_scores.append(t)
            self.d_masks.append(torch.empty(t.shape, dtype=torch.uint8, device="cuda"))
            self.d_cols.append(torch.empty(t.shape[1], dtype=torch.uint8, device="cuda"))
        n = len(scores)
        self.K = np.array([s[0] for s in self.shapes], np.int32)
        self.N = np.array([s[1] for s in self.shapes], np.int32)
        self.p_scores = (ctypes.c_void_p * n)(*[t.data_ptr() for t in self.d_scores])
        self.p_masks = (ctypes.c_void_p * n)(*[t.data_ptr() for t in self.d_masks])
        self.p_cols = (ctypes.c_void_p * n)(*[t.data_ptr() for t in self.d_cols])
        self.stream = torch.cuda.current_stream().cuda_stream

    def masks(self):
        return [m.cpu().numpy().astype(bool) for m in self.d_masks]


def tiled_wise_1d(accumulated_scores, sparsity, granularity=128, return_device=False):
    """prune_algo.py:114-148.  Returns the list of masks (bool arrays; uint8 CUDA tensors with
    return_device=True)."""
    L = tw.lib()
    d = _DeviceLayers(accumulated_scores)
    thr = ctypes.c_double()
    tw._check(L.tw_prune_tiled_wise_1d(
        len(d.shapes), tw._ptr(d.K, ctypes.c_int32), tw._ptr(d.N, ctypes.c_int32),
        ctypes.cast(d.p_scores, ctypes.POINTER(ctypes.c_void_p)), float(sparsity), _q_type(sparsity),
        int(granularity), ctypes.cast(d.p_masks, ctypes.POINTER(ctypes.c_void_p)),
        ctypes.byref(thr), d.stream))
    tiled_wise_1d.last_threshold = thr.value
    return d.d_masks if return_device else d.masks()


def tiled_wise_2d(accumulated_scores, sparsity, granularity=128, transform=True, return_device=False,
                  return_tiles=False):
    """prune_algo.py:55-112 (transform=False: BERT pruning type 8).  With return_tiles=True
    also returns, per layer, the tile table [(col0, width), ...] the masks are tile-wise on."""
    L = tw.lib()
    d = _DeviceLayers(accumulated_scores)
    thr = (ctypes.c_double * 2)()
    tw._check(L.tw_prune_tiled_wise_2d(
        len(d.shapes), tw._ptr(d.K, ctypes.c_int32), tw._ptr(d.N, ctypes.c_int32),
        ctypes.cast(d.p_scores, ctypes.POINTER(ctypes.c_void_p)), float(sparsity), _q_type(sparsity),
        1 if transform else 0, int(granularity),
        ctypes.cast(d.p_masks, ctypes.POINTER(ctypes.c_void_p)),
        ctypes.cast(d.p_cols, ctypes.POINTER(ctypes.c_void_p)), thr, d.stream))
    tiled_wise_2d.last_thresholds = (thr[0], thr[1])
    masks = d.d_masks if return_device else d.masks()
    if not return_tiles:
        return masks
    tables = [tiles_every_g_kept_columns(c.cpu().numpy(), granularity) for c in d.d_cols]
    return masks, tables


def _mix(d, g1percent, return_device):
    """Second stage of the mixed producers on the device masks already in ``d``."""
    thr = ctypes.c_double()
    pm = ctypes.cast(d.p_masks, ctypes.POINTER(ctypes.c_void_p))
    tw._check(tw.lib().tw_prune_mix(
        len(d.shapes), tw._ptr(d.K, ctypes.c_int32), tw._ptr(d.N, ctypes.c_int32),
        ctypes.cast(d.p_scores, ctypes.POINTER(ctypes.c_void_p)), pm, float(g1percent),
        _q_type(100 - g1percent), pm, ctypes.byref(thr), d.stream))
    tw_mix_fn.last_threshold = thr.value
    return d.d_masks if return_device else d.masks()


def tw_mix_fn(accumulated_scores, g1percent, layer_mask, return_device=False):
    """prune_algo.py:151-179: the elements whose |score| (minus 1 where ``layer_mask`` keeps
    them) lies above the (100 - g1percent)-th percentile of the whole network join the masks."""
    d = _DeviceLayers(accumulated_scores)
    for dst, m in zip(d.d_masks, layer_mask):
        if isinstance(m, d.torch.Tensor):
            dst.copy_(m.reshape(dst.shape).to(device="cuda", dtype=d.torch.uint8))
        else:
            dst.copy_(d.torch.from_numpy(np.ascontiguousarray(np.asarray(m) != 0).view(np.uint8)
                                         .reshape(dst.shape)))
    return _mix(d, g1percent, return_device)


def tiled_wise_1d_mix(accumulated_scores, sparsity, granularity=128, g1percent=5, return_device=False):
    """prune_algo.py:182-186: tiled_wise_1d at sparsity + g1percent, then tw_mix_fn."""
    d = _DeviceLayers(accumulated_scores)
    q = sparsity + g1percent
    tw._check(tw.lib().tw_prune_tiled_wise_1d(
        len(d.shapes), tw._ptr(d.K, ctypes.c_int32), tw._ptr(d.N, ctypes.c_int32),
        ctypes.cast(d.p_scores, ctypes.POINTER(ctypes.c_void_p)), float(q), _q_type(q),
        int(granularity), ctypes.cast(d.p_masks, ctypes.POINTER(ctypes.c_void_p)), None, d.stream))
    return _mix(d, g1percent, return_device)


def tiled_wise_2d_mix(accumulated_scores, sparsity, granularity=128, g1percent=1, return_device=False):
    """prune_algo.py:189-193: tiled_wise_2d at sparsity + g1percent, then tw_mix_fn."""
    d = _DeviceLayers(accumulated_scores)
    q = sparsity + g1percent
    tw._check(tw.lib().tw_prune_tiled_wise_2d(
        len(d.shapes), tw._ptr(d.K, ctypes.c_int32), tw._ptr(d.N, ctypes.c_int32),
        ctypes.cast(d.p_scores, ctypes.POINTER(ctypes.c_void_p)), float(q), _q_type(q), 1,
        int(granularity), ctypes.cast(d.p_masks, ctypes.POINTER(ctypes.c_void_p)),
        ctypes.cast(d.p_cols, ctypes.POINTER(ctypes.c_void_p)), None, d.stream))
    return _mix(d, g1percent, return_device)


def granularity_pruning(score, sparsity, granularity):
    """One threshold per tile (Pruning/BERT/utils/MyHook.py:202-214); `score` is one 2-D layer
    whose width is a multiple of the granularity.  Returns a bool [K, N] mask."""
    import torch
    L = tw.lib()
    t = torch.from_numpy(np.ascontiguousarray(score, dtype=np.float32)).cuda()
    K, N = t.shape
    m = torch.empty((K, N), dtype=torch.uint8, device="cuda")
    tw._check(L.tw_prune_granularity(K, N, t.data_ptr(), float(sparsity), _q_type(sparsity),
                                     int(granularity), m.data_ptr(),
                                     torch.cuda.current_stream().cuda_stream))
    return m.cpu().numpy().astype(bool)


def tiles_every_g_columns(n_cols, granularity):
    L = tw.lib()
    col0 = np.zeros(n_cols, np.int32)
    width = np.zeros(n_cols, np.int32)
    n = ctypes.c_int()
    tw._check(L.tw_tiles_every_g_columns(int(n_cols), int(granularity), tw._ptr(col0, ctypes.c_int32),
                                         tw._ptr(width, ctypes.c_int32), ctypes.byref(n)))
    return [(int(col0[i]), int(width[i])) for i in range(n.value)]


def tiles_every_g_kept_columns(col_mask, granularity):
    L = tw.lib()
    cm = np.ascontiguousarray(col_mask, dtype=np.uint8)
    col0 = np.zeros(cm.size, np.int32)
    width = np.zeros(cm.size, np.int32)
    n = ctypes.c_int()
    tw._check(L.tw_tiles_every_g_kept_columns(cm.size, int(granularity), tw._ptr(cm, ctypes.c_uint8),
                                              tw._ptr(col0, ctypes.c_int32),
                                              tw._ptr(width, ctypes.c_int32), ctypes.byref(n)))
    return [(int(col0[i]), int(width[i])) for i in range(n.value)]


def tile_row_norms(score, tile_table, col_keep=None):
    """float32 [n_tiles, K]: np.linalg.norm(score[:, tile], axis=1) / width for every tile, with
    the columns where col_keep is 0 counted as zeros."""
    import torch
    L = tw.lib()
    t = torch.from_numpy(np.ascontiguousarray(score, dtype=np.float32)).cuda()
    K, N = t.shape
    col0 = np.array([c for c, _ in tile_table], np.int32)
    width = np.array([w for _, w in tile_table], np.int32)
    out = torch.empty((len(tile_table), K), dtype=torch.float32, device="cuda")
    ck = None if col_keep is None else torch.from_numpy(np.ascontiguousarray(col_keep, dtype=np.uint8)).cuda()
    tw._check(L.tw_prune_tile_row_norms(K, N, t.data_ptr(), len(tile_table), tw._ptr(col0, ctypes.c_int32),
                                        tw._ptr(width, ctypes.c_int32), None if ck is None else ck.data_ptr(),
                                        out.data_ptr(), torch.cuda.current_stream().cuda_stream))
    return out.cpu().numpy()


def col_norms(score):
    """float32 [N]: np.linalg.norm(score, axis=0) / K."""
    import torch
    L = tw.lib()
    t = torch.from_numpy(np.ascontiguousarray(score, dtype=np.float32)).cuda()
    K, N = t.shape
    out = torch.empty(N, dtype=torch.float32, device="cuda")
    tw._check(L.tw_prune_col_norms(K, N, t.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def percentile(values, q):
    """np.percentile(values, q) for float32 values, computed on the GPU."""
    import torch
    L = tw.lib()
    t = torch.from_numpy(np.ascontiguousarray(values, dtype=np.float32).ravel()).cuda()
    r = ctypes.c_double()
    tw._check(L.tw_percentile_linear(t.data_ptr(), t.numel(), float(q), _q_type(q), ctypes.byref(r),
                                     torch.cuda.current_stream().cuda_stream))
    return np.float64(r.value) if _q_type(q) == Q_F64 else np.float32(r.value)
