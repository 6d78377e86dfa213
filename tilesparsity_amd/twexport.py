"""The on-disk hand-off between the reference's pruning runs and the TW-GEMM engine.

Two file formats leave the reference's Python side, both pickles of plain dictionaries of
NumPy arrays:

* the exported pruned model (exportPrunedModel, Pruning/BERT/utils/MyHook.py:54-89): for every
  masked dense layer four consecutive entries, keyed by the TensorFlow variable names
  ``.../mask-i:0``, ``.../mask-o:0``, ``.../kernel:0``, ``.../bias:0``: the relative offsets of
  the kept rows and columns (convert_mask_to_offset, :66-74), the compacted kernel
  ``kernel[mask_i][:, mask_o]`` and ``bias * mask_o``;
* the mask dictionaries name -> 0/1 array in the weight's own shape, 2-D or HWIO
  (Pruning/VGG/pruning.py:580-581, 639-640; Pruning/NMT/nmt/train.py:741-742).

``export_pruned_model`` writes the first format from masks and weights (the reference's hook
reads them out of a TensorFlow session), ``load_pruned_model`` turns it into device plans, and
``plans_from_masks`` does the same for the second format given the weights.  Files are read
with an unpickler that only admits NumPy arrays and plain containers, so loading a file runs
no code from it.
"""
import collections
import io
import pickle

import numpy as np

from . import twgemm

PrunedLayer = collections.namedtuple("PrunedLayer", "name plan bias K N kept_k kept_n")

_ALLOWED = {
    ("numpy.core.multiarray", "_reconstruct"), ("numpy._core.multiarray", "_reconstruct"),
    ("numpy.core.multiarray", "scalar"), ("numpy._core.multiarray", "scalar"),
    ("numpy", "ndarray"), ("numpy", "dtype"),
    ("numpy.core.numeric", "_frombuffer"), ("numpy._core.numeric", "_frombuffer"),
    ("collections", "OrderedDict"),
    ("_codecs", "encode"),      # protocol <= 2 stores an array's bytes as an encoded string
}


class _ArrayUnpickler(pickle.Unpickler):
    def find_class(self, module, name):
        if (module, name) in _ALLOWED:
            return super().find_class(module, name)
        raise pickle.UnpicklingError("refusing to load %s.%s: only NumPy arrays and plain "
                                     "containers are accepted" % (module, name))


def load_pickle(source):
    """The object stored in a pickle (path, bytes or binary file) made of dicts, lists, numbers,
    strings and NumPy arrays; anything else raises pickle.UnpicklingError."""
    if isinstance(source, (bytes, bytearray)):
        return _ArrayUnpickler(io.BytesIO(source)).load()
    if hasattr(source, "read"):
        return _ArrayUnpickler(source).load()
    with open(source, "rb") as f:
        return _ArrayUnpickler(f).load()


def convert_mask_to_offset(mask):
    """0/1 keep vector -> relative offsets kept[i] - i (MyHook.py:66-74)."""
    return twgemm.mask_to_offsets(np.asarray(mask) != 0)


def export_pruned_model(layers, path=None):
    """The dictionary exportPrunedModel pickles (MyHook.py:54-89).  ``layers``: iterable of
    (scope, mask_i [K], mask_o [N], kernel [K,N], bias [N]); the keys are
    ``scope/mask-i:0`` ... in the order the hook inserts them.  With ``path`` the dictionary is
    also written there with the highest pickle protocol, as the hook does."""
    ckpt = {}
    for scope, mi, mo, kernel, bias in layers:
        mi, mo = np.asarray(mi), np.asarray(mo)
        kernel = np.asarray(kernel)
        if kernel.shape != (mi.size, mo.size) or np.asarray(bias).shape != (mo.size,):
            raise twgemm.TwError(twgemm.ERR_SHAPE, "layer %s: kernel %r, masks %d x %d, bias %r"
                                 % (scope, kernel.shape, mi.size, mo.size, np.asarray(bias).shape))
        ckpt[scope + "/mask-i:0"] = convert_mask_to_offset(mi).astype(np.int64)
        ckpt[scope + "/mask-o:0"] = convert_mask_to_offset(mo).astype(np.int64)
        ckpt[scope + "/kernel:0"] = kernel[mi != 0][:, mo != 0]
        ckpt[scope + "/bias:0"] = np.asarray(bias) * mo
    if path is not None:
        with open(path, "wb") as f:
            pickle.dump(ckpt, f, pickle.HIGHEST_PROTOCOL)
    return ckpt


def _layer_groups(ckpt):
    """(scope, mask-i, mask-o, kernel, bias) for every ``mask-i`` entry and the three entries
    that follow it (the hook's insertion order, MyHook.py:59-63)."""
    items = list(ckpt.items())
    i = 0
    while i < len(items):
        name = items[i][0]
        if "mask-i" not in name:
            i += 1
            continue
        if i + 3 >= len(items):
            raise twgemm.TwError(twgemm.ERR_SHAPE, "entry %s is not followed by mask-o, kernel "
                                 "and bias" % name)
        for want, (got, _) in zip(("mask-o", "kernel", "bias"), items[i + 1:i + 4]):
            if want not in got:
                raise twgemm.TwError(twgemm.ERR_SHAPE, "entry after %s is %s, expected a %s"
                                     % (name, got, want))
        yield (name.split("mask-i")[0].rstrip("/"),) + tuple(v for _, v in items[i:i + 4])
        i += 4


def load_pruned_model(source, dtype="f16", K=None):
    """Plans for every layer of an exported pruned model.  ``source``: the dictionary itself or
    a pickle of it (path, bytes or file).  The file does not hold a layer's unpruned K;
    ``K`` may give it per scope (dict) or for all layers (int); otherwise the smallest K that
    holds the last kept row is used, which gives the same product.  Returns a list of
    PrunedLayer(name, plan, bias, K, N, kept_k, kept_n); ``bias`` is the exported fp32 vector of
    N entries (zero on pruned columns), ready for ``Plan.gemm(bias_ptr=...)``."""
    ckpt = source if isinstance(source, dict) else load_pickle(source)
    out = []
    for scope, mi, mo, kernel, bias in _layer_groups(ckpt):
        mi, mo = np.asarray(mi, np.int64).ravel(), np.asarray(mo, np.int64).ravel()
        bias = np.ascontiguousarray(bias, np.float32).ravel()
        N = bias.size
        need = int(mi[-1]) + mi.size if mi.size else 1
        k = K.get(scope) if isinstance(K, dict) else K
        k = need if k is None else int(k)
        kernel = np.asarray(kernel, np.float32).reshape(mi.size, mo.size)
        plan = twgemm.Plan.from_export(k, N, dtype, mi, mo, kernel)
        out.append(PrunedLayer(scope, plan, bias, k, N, twgemm.offsets_to_kept(mi, k),
                               twgemm.offsets_to_kept(mo, N)))
    return out


def mask_2d(mask):
    """A stored mask as a [K, N] matrix: HWIO conv masks become (H*W*I) x O, the inverse of
    img2col_back_ward (Pruning/VGG/prune_algo.py:26-36)."""
    mask = np.asarray(mask)
    if mask.ndim == 4:
        return mask.reshape(-1, mask.shape[-1])
    if mask.ndim != 2:
        raise twgemm.TwError(twgemm.ERR_SHAPE, "mask of shape %r is neither 2-D nor HWIO"
                             % (mask.shape,))
    return mask


def plans_from_masks(masks, weights, granularity=128, dtype="f16", cover=False):
    """Plans from a stored mask dictionary (or pickle of one) and the weights under the same
    names.  The tile table is derived from each mask (``twgemm.tiles_from_mask`` with at most
    ``granularity`` kept columns per tile), so masks of tiled_wise_1d and tiled_wise_2d load
    alike; with ``cover`` the mixed masks (TW plus an element-wise remainder) load too, on the
    tiles of every ``granularity`` columns.  Returns {name: Plan}."""
    if not isinstance(masks, dict):
        masks = load_pickle(masks)
    plans = {}
    for name, mask in masks.items():
        m = (mask_2d(mask) != 0).astype(np.uint8)
        w = np.asarray(weights[name], np.float32).reshape(m.shape)
        if cover:
            table = [(c, min(granularity, m.shape[1] - c)) for c in range(0, m.shape[1], granularity)]
        else:
            table = twgemm.tiles_from_mask(m, granularity)
        plans[name] = twgemm.Plan.from_mask_tiles(m, table, dtype, w, cover=cover)
    return plans
