"""ctypes binding of libtwgemm.so and the host-side mirror of the reference's
TW-GEMM driver interface (StreamMaskedGEMM/perf/basic_nn.cu).

The names follow the reference: ``mask_to_offsets`` (convert_mask_to_offset,
Pruning/BERT/utils/MyHook.py:66-74), ``tile_partition`` (basic_nn.cu:836-885),
``Plan`` (the per-tile mask_k / mask_n / compacted weight that
basic_nn.cu:891-914 builds), ``Plan.gemm`` / ``stream_gemm_nn`` (Stream_Gemm_NN,
basic_nn.cu:378-445).  Device memory is passed as raw pointers (integers), e.g.
``torch.Tensor.data_ptr()``; this module itself does not import torch.

There is no CPU fallback: if the HIP library is missing, loading fails loudly.
"""
import ctypes
import importlib.util
import os
import sys

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TWGEMM_LIB") or os.path.join(_PKG, "libtwgemm.so")

F16, BF16 = 0, 1
KMAJOR, ROWMAJOR = 0, 1
PRUNED_UNTOUCHED, PRUNED_ZERO = 0, 1
ACT_NONE, ACT_RELU, ACT_GELU, ACT_TANH = 0, 1, 2, 3
OPT_SHAPE, OPT_WGS_PER_CU, OPT_PIECE, OPT_XCD_QUEUES, OPT_SPIN_LIMIT, OPT_BALANCE, OPT_LDS_DMA, OPT_LSTM_LOOK = 0, 1, 2, 3, 4, 5, 6, 7
SHAPE_AS64, SHAPE_AS32, SHAPE_SKINNY, SHAPE_BS = 7, 8, 9, 10
SHAPE_WIDE, SHAPE_128x128, SHAPE_512x64, SHAPE_128x64, SHAPE_256x128, SHAPE_128x32, SHAPE_256x64 = range(7)
SHAPE_NAMES = ("tw_gemm_kmajor_kernel 256x128", "tw_gemm_ws_kernel 128x128", "tw_gemm_ws_kernel 512x64",
               "tw_gemm_ws_kernel 128x64", "tw_gemm_ws_kernel 256x128", "tw_gemm_ws_kernel 128x32",
               "tw_gemm_ws_kernel 256x64", "tw_gemm_as_kernel 64 rows", "tw_gemm_as_kernel 32 rows",
               "tw_gemm_skinny_kernel", "tw_gemm_bs_kernel")


class Epilogue(ctypes.Structure):
    """tw_epilogue of include/twgemm.h."""
    _fields_ = [("bias", ctypes.c_void_p), ("activation", ctypes.c_int)]

OK = 0
ERR_NULL, ERR_SHAPE, ERR_TILE_TABLE, ERR_INDEX_LIST, ERR_DTYPE = -1, -2, -3, -4, -5
ERR_LAYOUT, ERR_ALIGNMENT, ERR_NOT_TW, ERR_DEVICE, ERR_ALLOC, ERR_BUFFER = -6, -7, -8, -9, -10, -11

_DTYPES = {"f16": F16, "fp16": F16, "half": F16, "bf16": BF16, F16: F16, BF16: BF16}

# every symbol include/twgemm.h declares
EXPORTED_SYMBOLS = (
    "tw_version", "tw_last_error", "tw_status_string",
    "tw_mask_to_offsets", "tw_offsets_to_kept", "tw_tile_partition",
    "tw_plan_create", "tw_plan_create_dense", "tw_plan_from_mask",
    "tw_plan_from_stream_operands", "tw_plan_info", "tw_plan_export", "tw_plan_destroy",
    "tw_gemm", "tw_stream_gemm_nn", "tw_cast_f32", "tw_delete_row", "tw_insert_row",
    "tw_plan_from_mask_tiles", "tw_prune_tiled_wise_1d", "tw_prune_tiled_wise_2d",
    "tw_tiles_every_g_columns", "tw_tiles_every_g_kept_columns",
    "tw_prune_tile_row_norms", "tw_prune_col_norms", "tw_percentile_linear", "tw_gemm_ex",
    "tw_prune_granularity", "tw_plan_from_export", "tw_plan_from_mask_cover", "tw_tiles_from_mask",
    "tw_prune_mix", "tw_lstm_gates", "tw_plan_from_device_mask", "tw_set_option", "tw_gemm_static",
    "tw_gemm_staged", "tw_gemm_staged_workspace",
    "tw_side_create", "tw_side_destroy", "tw_side_nnz", "tw_side_gemm", "tw_plan_reset", "tw_lstm_step",
    "tw_lstm_steps", "tw_lstm_steps_status", "tw_gemm_choice",
)


class TwError(RuntimeError):
    """A libtwgemm call returned a negative status."""

    def __init__(self, status, message):
        super().__init__("libtwgemm status %d: %s" % (status, message))
        self.status = status
        self.message = message


_lib = None


def _share_torch_hip_runtime():
    """A process must hold ONE HIP runtime.  PyTorch wheels bundle their own
    libamdhip64 (same soname as the system one); if it is loaded after the system copy
    that libtwgemm.so would otherwise pull in, the second runtime finds no GPU.  So when
    PyTorch is installed but not yet imported, its runtime is loaded first and
    libtwgemm.so binds to it by soname.  TWGEMM_SYSTEM_HIP=1 skips this."""
    if "torch" in sys.modules or os.environ.get("TWGEMM_SYSTEM_HIP") == "1":
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    if spec is None or not spec.origin:
        return
    path = os.path.join(os.path.dirname(spec.origin), "lib", "libamdhip64.so")
    if os.path.exists(path):
        ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


def lib():
    """The loaded library (raises if libtwgemm.so has not been built)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `python -m tilesparsity_amd.build` "
            "(there is no CPU fallback)" % LIB_PATH)
    _share_torch_hip_runtime()
    L = ctypes.CDLL(LIB_PATH)
    c_int, c_i64, c_f, vp = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p
    i32p = ctypes.POINTER(ctypes.c_int32)
    i64p = ctypes.POINTER(ctypes.c_int64)
    u8p = ctypes.POINTER(ctypes.c_uint8)
    u16p = ctypes.POINTER(ctypes.c_uint16)
    f32p = ctypes.POINTER(ctypes.c_float)
    pp = ctypes.POINTER(vp)
    sig = {
        "tw_version": (c_int, []),
        "tw_last_error": (ctypes.c_char_p, []),
        "tw_status_string": (ctypes.c_char_p, [c_int]),
        "tw_mask_to_offsets": (c_int, [u8p, c_int, i32p, ctypes.POINTER(c_int)]),
        "tw_offsets_to_kept": (c_int, [i32p, c_int, c_int, i32p]),
        "tw_tile_partition": (c_int, [c_int] * 7 + [ctypes.POINTER(c_int), i32p, i32p, i32p,
                                                     i64p, i64p]),
        "tw_plan_create": (c_int, [c_int, c_int, c_int, c_int, i32p, i32p, i32p, i32p, i32p,
                                   i32p, f32p, pp]),
        "tw_plan_create_dense": (c_int, [c_int, c_int, c_int, c_int, f32p, pp]),
        "tw_plan_from_mask": (c_int, [c_int, c_int, c_int, c_int, u8p, f32p, pp]),
        "tw_plan_from_stream_operands": (c_int, [c_int, c_int, c_int, c_int, vp, c_int, i32p,
                                                 i32p, pp, pp, i64p, i64p, pp]),
        "tw_plan_info": (c_int, [vp, i64p, c_int]),
        "tw_plan_export": (c_int, [vp, i32p, i32p, i32p, i32p, i32p, i32p, i32p, i32p, u16p]),
        "tw_plan_destroy": (c_int, [vp]),
        "tw_gemm": (c_int, [vp, vp, c_int, c_i64, vp, c_int, c_i64, c_int, c_f, c_f, c_int, vp]),
        "tw_gemm_ex": (c_int, [vp, vp, c_int, c_i64, vp, c_int, c_i64, c_int, c_f, c_f, c_int,
                               ctypes.POINTER(Epilogue), vp]),
        "tw_gemm_static": (c_int, [vp, vp, c_int, c_i64, vp, c_int, c_i64, c_int, c_f, c_f, c_int,
                                   ctypes.POINTER(Epilogue), vp]),
        "tw_gemm_staged": (c_int, [vp, vp, c_int, c_i64, vp, c_int, c_i64, c_int, c_f, c_f, c_int,
                                   ctypes.POINTER(Epilogue), vp, c_i64, vp]),
        "tw_gemm_staged_workspace": (c_i64, [vp, c_int, c_int, c_int]),
        "tw_stream_gemm_nn": (c_int, [c_int, c_int, c_int, c_int, c_f, vp, vp, c_f, vp, c_int,
                                      i32p, i32p, pp, pp, i64p, i64p, vp]),
        "tw_cast_f32": (c_int, [vp, vp, c_i64, c_int, vp]),
        "tw_delete_row": (c_int, [vp, vp, c_int, c_int, vp, vp]),
        "tw_insert_row": (c_int, [vp, vp, c_int, c_int, vp, vp]),
        "tw_plan_from_mask_tiles": (c_int, [c_int, c_int, c_int, c_int, i32p, i32p, u8p, f32p, pp]),
        "tw_prune_tiled_wise_1d": (c_int, [c_int, i32p, i32p, pp, ctypes.c_double, c_int, c_int,
                                           pp, ctypes.POINTER(ctypes.c_double), vp]),
        "tw_prune_tiled_wise_2d": (c_int, [c_int, i32p, i32p, pp, ctypes.c_double, c_int, c_int,
                                           c_int, pp, pp, ctypes.POINTER(ctypes.c_double), vp]),
        "tw_tiles_every_g_columns": (c_int, [c_int, c_int, i32p, i32p, ctypes.POINTER(c_int)]),
        "tw_prune_tile_row_norms": (c_int, [c_int, c_int, vp, c_int, i32p, i32p, vp, vp, vp]),
        "tw_prune_col_norms": (c_int, [c_int, c_int, vp, vp, vp]),
        "tw_prune_granularity": (c_int, [c_int, c_int, vp, ctypes.c_double, c_int, c_int, vp, vp]),
        "tw_percentile_linear": (c_int, [vp, c_i64, ctypes.c_double, c_int,
                                         ctypes.POINTER(ctypes.c_double), vp]),
        "tw_tiles_every_g_kept_columns": (c_int, [c_int, c_int, u8p, i32p, i32p,
                                                  ctypes.POINTER(c_int)]),
        "tw_prune_mix": (c_int, [c_int, i32p, i32p, pp, pp, ctypes.c_double, c_int, pp,
                                 ctypes.POINTER(ctypes.c_double), vp]),
        "tw_lstm_gates": (c_int, [c_int, c_int, c_int, vp, c_i64, c_f, vp, c_i64, vp, c_i64, vp, c_i64, vp]),
        "tw_plan_from_device_mask": (c_int, [c_int, c_int, c_int, c_int, i32p, i32p, vp, vp, c_int, vp, pp]),
        "tw_set_option": (c_int, [c_int, c_int]),
        "tw_plan_from_export": (c_int, [c_int, c_int, c_int, c_int, i32p, c_int, i32p, f32p, pp]),
        "tw_plan_from_mask_cover": (c_int, [c_int, c_int, c_int, c_int, i32p, i32p, u8p, f32p, pp]),
        "tw_tiles_from_mask": (c_int, [c_int, c_int, c_int, u8p, i32p, i32p, ctypes.POINTER(c_int)]),
        "tw_plan_reset": (c_int, [vp, vp]),
        "tw_lstm_step": (c_int, [vp, vp, c_i64, c_int, vp, c_f, vp, c_i64, vp, c_i64, vp, c_i64, vp, c_i64, vp]),
        "tw_lstm_steps": (c_int, [vp, c_int, vp, c_i64, c_i64, c_int, vp, c_f, vp, c_i64, vp, c_i64, vp]),
        "tw_lstm_steps_status": (c_int, [vp, vp]),
        "tw_gemm_choice": (c_int, [vp, c_int, c_i64, c_i64, c_f, i32p]),
        "tw_side_create": (c_int, [c_int, c_int, c_int, u8p, f32p, pp]),
        "tw_side_destroy": (None, [vp]),
        "tw_side_nnz": (c_i64, [vp]),
        "tw_side_gemm": (c_int, [vp, vp, c_i64, vp, c_i64, c_int, c_f, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def _check(status):
    if status != OK:
        raise TwError(status, lib().tw_last_error().decode())


def set_option(option, value):
    """tw_set_option: process-wide tuning switch of the GEMM launches (OPT_*), -1 = automatic."""
    _check(lib().tw_set_option(int(option), int(value)))


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _ptr(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def dtype_code(dtype):
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TwError(ERR_DTYPE, "unknown dtype %r" % (dtype,))


def version():
    return lib().tw_version()


# --------------------------------------------------------------------------- integer helpers
def mask_to_offsets(mask):
    """0/1 keep vector -> relative offsets kept[i]-i (convert_mask_to_offset)."""
    mask = np.ascontiguousarray(mask, dtype=np.uint8)
    out = np.empty(max(mask.size, 1), dtype=np.int32)
    n = ctypes.c_int(0)
    _check(lib().tw_mask_to_offsets(_ptr(mask, ctypes.c_uint8), mask.size,
                                    _ptr(out, ctypes.c_int32), ctypes.byref(n)))
    return out[:n.value].copy()


def offsets_to_kept(offsets, limit):
    """Relative offsets -> ascending kept indices in [0, limit)."""
    offsets = _i32(offsets)
    out = np.empty(max(offsets.size, 1), dtype=np.int32)
    _check(lib().tw_offsets_to_kept(_ptr(offsets, ctypes.c_int32), offsets.size, limit,
                                    _ptr(out, ctypes.c_int32)))
    return out[:offsets.size].copy()


def tile_partition(M, N, K, N_pruned, K_pruned, n_dim=128, max_tiles=4096):
    """Tile partition of TestCutlassGemm (basic_nn.cu:836-885)."""
    bn = ctypes.c_int(0)
    N_ori = np.zeros(max_tiles, np.int32)
    N_cal = np.zeros(max_tiles, np.int32)
    K_cal = np.zeros(max_tiles, np.int32)
    off_B = np.zeros(max_tiles, np.int64)
    off_C = np.zeros(max_tiles, np.int64)
    _check(lib().tw_tile_partition(M, N, K, N_pruned, K_pruned, n_dim, max_tiles,
                                   ctypes.byref(bn), _ptr(N_ori, ctypes.c_int32),
                                   _ptr(N_cal, ctypes.c_int32), _ptr(K_cal, ctypes.c_int32),
                                   _ptr(off_B, ctypes.c_int64), _ptr(off_C, ctypes.c_int64)))
    n = bn.value
    return dict(block_num=n, N_ori=N_ori[:n].tolist(), N_cal=N_cal[:n].tolist(),
                K_cal=K_cal[:n].tolist(), off_B=off_B[:n].tolist(), off_C=off_C[:n].tolist())


def tiles_from_mask(mask, G=0):
    """[(col0, width), ...] for a mask [K,N] whose tiling is not known: a tile takes columns
    while their kept rows equal those of its first non-empty column, at most G of them (0: no
    limit).  Host only."""
    mask = np.ascontiguousarray(mask, dtype=np.uint8)
    K, N = mask.shape
    col0, width = np.zeros(N, np.int32), np.zeros(N, np.int32)
    n = ctypes.c_int(0)
    _check(lib().tw_tiles_from_mask(K, N, int(G), _ptr(mask, ctypes.c_uint8),
                                    _ptr(col0, ctypes.c_int32), _ptr(width, ctypes.c_int32),
                                    ctypes.byref(n)))
    return [(int(col0[t]), int(width[t])) for t in range(n.value)]


def tiles_to_csr(tiles):
    """list of tile dicts (col0, width, kept_k, kept_n) -> the six flat arrays."""
    col0 = _i32([t["col0"] for t in tiles])
    width = _i32([t["width"] for t in tiles])
    kp = np.zeros(len(tiles) + 1, np.int32)
    npt = np.zeros(len(tiles) + 1, np.int32)
    for i, t in enumerate(tiles):
        kp[i + 1] = kp[i] + len(t["kept_k"])
        npt[i + 1] = npt[i] + len(t["kept_n"])
    ki = _i32(np.concatenate([_i32(t["kept_k"]) for t in tiles])) if tiles else _i32([])
    ni = _i32(np.concatenate([_i32(t["kept_n"]) for t in tiles])) if tiles else _i32([])
    return col0, width, kp, ki, npt, ni


# --------------------------------------------------------------------------- plans
class Plan:
    """Device-resident TW weight: tile table, kept-K / kept-N lists, packed weight."""

    def __init__(self, handle, K, N, dtype):
        self._h = ctypes.c_void_p(handle)
        self.K, self.N, self.dtype = K, N, dtype

    # -- constructors
    @classmethod
    def create(cls, K, N, dtype, tiles, B):
        """From an explicit tile table (list of dicts) and the fp32 weight B[K,N]."""
        col0, width, kp, ki, npt, ni = tiles_to_csr(tiles)
        return cls.create_csr(K, N, dtype, col0, width, kp, ki, npt, ni, B)

    @classmethod
    def create_csr(cls, K, N, dtype, col0, width, kp, ki, npt, ni, B):
        B = np.ascontiguousarray(B, dtype=np.float32)
        if B.size != K * N:
            raise TwError(ERR_SHAPE, "B has %d elements, expected K*N=%d" % (B.size, K * N))
        col0, width, kp, ki, npt, ni = map(_i32, (col0, width, kp, ki, npt, ni))
        h = ctypes.c_void_p()
        i32 = ctypes.c_int32
        _check(lib().tw_plan_create(K, N, dtype_code(dtype), col0.size, _ptr(col0, i32),
                                    _ptr(width, i32), _ptr(kp, i32), _ptr(ki, i32),
                                    _ptr(npt, i32), _ptr(ni, i32), _ptr(B, ctypes.c_float),
                                    ctypes.byref(h)))
        return cls(h.value, K, N, dtype_code(dtype))

    @classmethod
    def dense(cls, K, N, G, dtype, B):
        """The 0 %-sparse plan (every row and column kept)."""
        B = np.ascontiguousarray(B, dtype=np.float32)
        if B.size != K * N:
            raise TwError(ERR_SHAPE, "B has %d elements, expected K*N=%d" % (B.size, K * N))
        h = ctypes.c_void_p()
        _check(lib().tw_plan_create_dense(K, N, G, dtype_code(dtype), _ptr(B, ctypes.c_float),
                                          ctypes.byref(h)))
        return cls(h.value, K, N, dtype_code(dtype))

    @classmethod
    def from_mask(cls, mask, G, dtype, B):
        """From a dense 0/1 mask [K,N]; the integer pre-pass runs on the GPU."""
        mask = np.ascontiguousarray(mask, dtype=np.uint8)
        K, N = mask.shape
        B = np.ascontiguousarray(B, dtype=np.float32)
        if B.size != K * N:
            raise TwError(ERR_SHAPE, "B has %d elements, expected K*N=%d" % (B.size, K * N))
        h = ctypes.c_void_p()
        _check(lib().tw_plan_from_mask(K, N, G, dtype_code(dtype), _ptr(mask, ctypes.c_uint8),
                                       _ptr(B, ctypes.c_float), ctypes.byref(h)))
        return cls(h.value, K, N, dtype_code(dtype))

    @classmethod
    def from_mask_tiles(cls, mask, tile_table, dtype, B, cover=False):
        """From a dense 0/1 mask [K,N] and an explicit tile table [(col0, width), ...].  With
        ``cover`` a tile need not be rows x columns: it keeps every row and column that holds a
        kept element and stores the dropped elements inside as zeros (any mask is accepted)."""
        mask = np.ascontiguousarray(mask, dtype=np.uint8)
        K, N = mask.shape
        B = np.ascontiguousarray(B, dtype=np.float32)
        if B.size != K * N:
            raise TwError(ERR_SHAPE, "B has %d elements, expected K*N=%d" % (B.size, K * N))
        col0 = _i32([t[0] for t in tile_table])
        width = _i32([t[1] for t in tile_table])
        h = ctypes.c_void_p()
        fn = lib().tw_plan_from_mask_cover if cover else lib().tw_plan_from_mask_tiles
        _check(fn(K, N, dtype_code(dtype), len(tile_table), _ptr(col0, ctypes.c_int32),
                  _ptr(width, ctypes.c_int32), _ptr(mask, ctypes.c_uint8), _ptr(B, ctypes.c_float),
                  ctypes.byref(h)))
        return cls(h.value, K, N, dtype_code(dtype))

    @classmethod
    def from_device_mask(cls, K, N, mask_ptr, tile_table, dtype, B_ptr, cover=False, stream=0):
        """As from_mask_tiles, with the mask (K x N bytes) and the fp32 weight in device memory
        (raw pointers): nothing is uploaded.  The build runs on `stream` and waits for it."""
        col0 = _i32([t[0] for t in tile_table])
        width = _i32([t[1] for t in tile_table])
        h = ctypes.c_void_p()
        _check(lib().tw_plan_from_device_mask(K, N, dtype_code(dtype), len(tile_table),
                                              _ptr(col0, ctypes.c_int32), _ptr(width, ctypes.c_int32),
                                              ctypes.c_void_p(int(mask_ptr or 0)),
                                              ctypes.c_void_p(int(B_ptr or 0)), 1 if cover else 0,
                                              ctypes.c_void_p(int(stream or 0)), ctypes.byref(h)))
        return cls(h.value, K, N, dtype_code(dtype))

    @classmethod
    def from_export(cls, K, N, dtype, mask_i, mask_o, kernel):
        """From one layer of an exported pruned model: relative offsets of the kept rows and
        columns and the compacted fp32 weight [len(mask_i), len(mask_o)]."""
        mask_i, mask_o = _i32(mask_i), _i32(mask_o)
        kernel = np.ascontiguousarray(kernel, dtype=np.float32)
        if kernel.size != mask_i.size * mask_o.size:
            raise TwError(ERR_SHAPE, "kernel has %d elements, expected %d x %d"
                          % (kernel.size, mask_i.size, mask_o.size))
        h = ctypes.c_void_p()
        _check(lib().tw_plan_from_export(K, N, dtype_code(dtype), mask_i.size,
                                         _ptr(mask_i, ctypes.c_int32), mask_o.size,
                                         _ptr(mask_o, ctypes.c_int32), _ptr(kernel, ctypes.c_float),
                                         ctypes.byref(h)))
        return cls(h.value, K, N, dtype_code(dtype))

    @classmethod
    def from_stream_operands(cls, M, N, K, dtype, B_stream_ptr, N_cal, K_cal, mask_n_ptrs,
                             mask_k_ptrs, off_B, off_C):
        """From the device operands of the reference's Stream_Gemm_NN."""
        N_cal, K_cal = _i32(N_cal), _i32(K_cal)
        off_B = np.ascontiguousarray(off_B, dtype=np.int64)
        off_C = np.ascontiguousarray(off_C, dtype=np.int64)
        bn = N_cal.size
        mn = (ctypes.c_void_p * bn)(*[int(p) for p in mask_n_ptrs])
        mk = (ctypes.c_void_p * bn)(*[int(p) for p in mask_k_ptrs])
        h = ctypes.c_void_p()
        _check(lib().tw_plan_from_stream_operands(
            M, N, K, dtype_code(dtype), ctypes.c_void_p(int(B_stream_ptr)), bn,
            _ptr(N_cal, ctypes.c_int32), _ptr(K_cal, ctypes.c_int32), mn, mk,
            _ptr(off_B, ctypes.c_int64), _ptr(off_C, ctypes.c_int64), ctypes.byref(h)))
        return cls(h.value, K, N, dtype_code(dtype))

    # -- inspection
    def lstm_step(self, A_ptr, M, c_prev_ptr, c_new_ptr, h_new_ptr, lda=None, ldc_prev=None,
                  ldc_new=None, ldh=None, bias_ptr=None, forget_bias=1.0, gates_ptr=None, ldg=None,
                  stream=0):
        """One LSTM time step on K-major device buffers (see tw_lstm_step): the gate GEMM of this
        plan (N = 4H) and the cell arithmetic in one launch where the plan allows it, else
        tw_gemm_ex into `gates_ptr` followed by tw_lstm_gates."""
        vp = ctypes.c_void_p
        ld = lambda v: M if v is None else v
        _check(lib().tw_lstm_step(self._h, vp(int(A_ptr or 0)), ld(lda), M, vp(int(bias_ptr or 0)),
                                  forget_bias, vp(int(c_prev_ptr or 0)), ld(ldc_prev),
                                  vp(int(c_new_ptr or 0)), ld(ldc_new), vp(int(h_new_ptr or 0)), ld(ldh),
                                  vp(int(gates_ptr or 0)), ld(ldg), vp(int(stream or 0))))

    def lstm_steps(self, T, A_ptr, M, c_ptr, lda=None, a_step=None, ldc=None, bias_ptr=None, forget_bias=1.0,
                   gates_ptr=None, ldg=None, stream=0):
        """T LSTM time steps on T + 1 K-major matrices A_t = [x_t ; h_(t-1)] at a_step elements from
        each other (see tw_lstm_steps): one persistent launch where the plan and the chip allow it,
        else T calls of tw_lstm_step.  Asynchronous; lstm_steps_status() tells whether it completed."""
        vp = ctypes.c_void_p
        lda = M if lda is None else lda
        a_step = self.K * lda if a_step is None else a_step
        _check(lib().tw_lstm_steps(self._h, T, vp(int(A_ptr or 0)), lda, a_step, M, vp(int(bias_ptr or 0)),
                                   forget_bias, vp(int(c_ptr or 0)), M if ldc is None else ldc,
                                   vp(int(gates_ptr or 0)), M if ldg is None else ldg, vp(int(stream or 0))))

    def lstm_steps_status(self, stream=0):
        """Waits for the stream; raises TwError(ERR_DEVICE) if a persistent lstm_steps launch gave up."""
        _check(lib().tw_lstm_steps_status(self._h, ctypes.c_void_p(int(stream or 0))))

    def choice(self, M, lda=None, ldc=None, beta=0.0):
        """The kernel a K-major launch on M rows would run: dict(shape, name, piece, per_cu, xcd_queues)."""
        out = np.zeros(4, np.int32)
        _check(lib().tw_gemm_choice(self._h, M, M if lda is None else lda, M if ldc is None else ldc, beta,
                                    _ptr(out, ctypes.c_int32)))
        return dict(shape=int(out[0]), name=SHAPE_NAMES[int(out[0])], piece=int(out[1]), per_cu=int(out[2]),
                    xcd_queues=bool(out[3]))

    def reset(self, stream=0):
        """Re-arms the plan's work-queue counters (after a launch of it was aborted mid-flight)."""
        _check(lib().tw_plan_reset(self._h, ctypes.c_void_p(int(stream or 0))))

    def info(self):
        v = np.zeros(12, np.int64)
        _check(lib().tw_plan_info(self._h, _ptr(v, ctypes.c_int64), 12))
        keys = ("K", "N", "dtype", "n_tiles", "sum_k", "sum_n", "kept_elems", "packed_bytes",
                "max_k", "max_n", "empty_tiles", "total_width")
        return dict(zip(keys, (int(x) for x in v)))

    def export(self, with_weight=True):
        """Tile table, kept lists, relative offsets and (optionally) the compacted
        weight in the reference's stream layout, as 16-bit patterns [K*N]."""
        inf = self.info()
        nt, sk, sn = inf["n_tiles"], inf["sum_k"], inf["sum_n"]
        i32 = ctypes.c_int32
        col0, width = np.zeros(nt, np.int32), np.zeros(nt, np.int32)
        kp, npt = np.zeros(nt + 1, np.int32), np.zeros(nt + 1, np.int32)
        ki, rk = np.zeros(max(sk, 1), np.int32), np.zeros(max(sk, 1), np.int32)
        ni, rn = np.zeros(max(sn, 1), np.int32), np.zeros(max(sn, 1), np.int32)
        Bs = np.zeros(self.K * self.N, np.uint16) if with_weight else None
        _check(lib().tw_plan_export(
            self._h, _ptr(col0, i32), _ptr(width, i32), _ptr(kp, i32), _ptr(ki, i32),
            _ptr(rk, i32), _ptr(npt, i32), _ptr(ni, i32), _ptr(rn, i32),
            _ptr(Bs, ctypes.c_uint16) if with_weight else None))
        tiles = []
        for t in range(nt):
            tiles.append(dict(col0=int(col0[t]), width=int(width[t]),
                              kept_k=ki[kp[t]:kp[t + 1]].copy(), kept_n=ni[npt[t]:npt[t + 1]].copy(),
                              mask_k=rk[kp[t]:kp[t + 1]].copy(), mask_n=rn[npt[t]:npt[t + 1]].copy()))
        return tiles, Bs

    # -- the GEMM
    def staged_workspace(self, M, a_layout, c_layout):
        """Bytes of workspace `gemm(..., workspace_ptr=...)` needs for these layouts."""
        return int(lib().tw_gemm_staged_workspace(self._h, M, a_layout, c_layout))

    def gemm(self, A_ptr, C_ptr, M, lda=None, ldc=None, alpha=1.0, beta=0.0,
             a_layout=KMAJOR, c_layout=KMAJOR, pruned_cols=PRUNED_UNTOUCHED, stream=0,
             bias_ptr=None, activation=ACT_NONE, static=False, workspace_ptr=None,
             workspace_bytes=0):
        """C = act(alpha * A (B (.) mask) + beta * C + bias) on device pointers; asynchronous.
        bias_ptr: device fp32 [N] or None; activation: ACT_NONE / ACT_RELU / ACT_GELU / ACT_TANH.
        static=True goes through tw_gemm_static (work-queue counters in the library's own device
        array; calls that overlap on one GPU race).  With a workspace (device memory of
        staged_workspace(...) bytes) row-major operands go through tw_gemm_staged: K-major copies
        in the workspace around the K-major kernel, instead of the layout-generic kernel."""
        if lda is None:
            lda = M if a_layout == KMAJOR else self.K
        if ldc is None:
            ldc = M if c_layout == KMAJOR else self.N
        if workspace_ptr is not None:
            ep = Epilogue(ctypes.c_void_p(int(bias_ptr or 0)), int(activation))
            _check(lib().tw_gemm_staged(self._h, ctypes.c_void_p(int(A_ptr or 0)), a_layout, lda,
                                        ctypes.c_void_p(int(C_ptr or 0)), c_layout, ldc, M, alpha, beta,
                                        pruned_cols, ctypes.byref(ep),
                                        ctypes.c_void_p(int(workspace_ptr or 0)), int(workspace_bytes),
                                        ctypes.c_void_p(int(stream or 0))))
            return
        if bias_ptr is None and activation == ACT_NONE and not static:
            _check(lib().tw_gemm(self._h, ctypes.c_void_p(int(A_ptr or 0)), a_layout, lda,
                                 ctypes.c_void_p(int(C_ptr or 0)), c_layout, ldc, M, alpha, beta,
                                 pruned_cols, ctypes.c_void_p(int(stream or 0))))
            return
        ep = Epilogue(ctypes.c_void_p(int(bias_ptr or 0)), int(activation))
        fn = lib().tw_gemm_static if static else lib().tw_gemm_ex
        _check(fn(self._h, ctypes.c_void_p(int(A_ptr or 0)), a_layout, lda,
                                ctypes.c_void_p(int(C_ptr or 0)), c_layout, ldc, M, alpha, beta,
                                pruned_cols, ctypes.byref(ep), ctypes.c_void_p(int(stream or 0))))

    def destroy(self):
        if self._h is not None and self._h.value:
            lib().tw_plan_destroy(self._h)
        self._h = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.destroy()


def stream_gemm_nn(M, N, K, dtype, alpha, A_ptr, B_ptr, beta, C_ptr, N_cal, K_cal, mask_n_ptrs,
                   mask_k_ptrs, off_B, off_C, stream=0):
    """One-shot drop-in for Stream_Gemm_NN (basic_nn.cu:378-393), device pointers."""
    N_cal, K_cal = _i32(N_cal), _i32(K_cal)
    off_B = np.ascontiguousarray(off_B, dtype=np.int64)
    off_C = np.ascontiguousarray(off_C, dtype=np.int64)
    bn = N_cal.size
    mn = (ctypes.c_void_p * bn)(*[int(p) for p in mask_n_ptrs])
    mk = (ctypes.c_void_p * bn)(*[int(p) for p in mask_k_ptrs])
    _check(lib().tw_stream_gemm_nn(M, N, K, dtype_code(dtype), alpha, ctypes.c_void_p(int(A_ptr)),
                                   ctypes.c_void_p(int(B_ptr)), beta, ctypes.c_void_p(int(C_ptr)),
                                   bn, _ptr(N_cal, ctypes.c_int32), _ptr(K_cal, ctypes.c_int32),
                                   mn, mk, _ptr(off_B, ctypes.c_int64), _ptr(off_C, ctypes.c_int64),
                                   ctypes.c_void_p(int(stream or 0))))


class Side:
    """The element-wise remainder of a mixed mask (tw_side_*): ``remainder`` is a K x N mask, normally
    ``mask & ~mask0`` of tiled_wise_1d_mix / tiled_wise_2d_mix (Pruning/VGG/prune_algo.py:151-193),
    ``B`` the fp32 weight.  ``gemm`` adds ``alpha * A @ (B * remainder)`` to a K-major C after the
    plan of mask0 has written it."""

    def __init__(self, remainder, dtype, B):
        m = np.ascontiguousarray(np.asarray(remainder) != 0, dtype=np.uint8)
        B = np.ascontiguousarray(B, dtype=np.float32)
        if m.ndim != 2 or B.shape != m.shape:
            raise ValueError("remainder and B must be K x N matrices of one shape")
        self.K, self.N, self.dtype = m.shape[0], m.shape[1], dtype
        h = ctypes.c_void_p()
        _check(lib().tw_side_create(self.K, self.N, dtype_code(dtype),
                                    m.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)),
                                    B.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), ctypes.byref(h)))
        self._h = h

    @property
    def nnz(self):
        return int(lib().tw_side_nnz(self._h))

    def gemm(self, A_ptr, C_ptr, M, lda=None, ldc=None, alpha=1.0, stream=0):
        vp = ctypes.c_void_p
        _check(lib().tw_side_gemm(self._h, vp(int(A_ptr or 0)), M if lda is None else lda,
                                  vp(int(C_ptr or 0)), M if ldc is None else ldc, M, alpha,
                                  vp(int(stream or 0))))

    def destroy(self):
        if self._h:
            lib().tw_side_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.destroy()


def lstm_gates(M, H, dtype, gates_ptr, ldg, forget_bias, c_prev_ptr, ldc_prev, c_new_ptr, ldc_new,
               h_new_ptr, ldh, stream=0):
    """BasicLSTMCell gate arithmetic on K-major device buffers (see tw_lstm_gates)."""
    vp = ctypes.c_void_p
    _check(lib().tw_lstm_gates(M, H, dtype_code(dtype), vp(int(gates_ptr or 0)), ldg, forget_bias,
                               vp(int(c_prev_ptr or 0)), ldc_prev, vp(int(c_new_ptr or 0)), ldc_new,
                               vp(int(h_new_ptr or 0)), ldh, vp(int(stream or 0))))


def cast_f32(src_ptr, dst_ptr, n, dtype, stream=0):
    """Device fp32 -> 16-bit cast (float_to_half)."""
    _check(lib().tw_cast_f32(ctypes.c_void_p(int(src_ptr or 0)), ctypes.c_void_p(int(dst_ptr or 0)),
                             n, dtype_code(dtype), ctypes.c_void_p(int(stream or 0))))


def delete_row(matrix_ptr, matrix_2_ptr, rows, columns, mask_ptr, stream=0):
    _check(lib().tw_delete_row(ctypes.c_void_p(int(matrix_ptr or 0)),
                               ctypes.c_void_p(int(matrix_2_ptr or 0)), rows, columns,
                               ctypes.c_void_p(int(mask_ptr or 0)), ctypes.c_void_p(int(stream or 0))))


def insert_row(matrix_ptr, matrix_2_ptr, rows, columns, mask_ptr, stream=0):
    _check(lib().tw_insert_row(ctypes.c_void_p(int(matrix_ptr or 0)),
                               ctypes.c_void_p(int(matrix_2_ptr or 0)), rows, columns,
                               ctypes.c_void_p(int(mask_ptr or 0)), ctypes.c_void_p(int(stream or 0))))
