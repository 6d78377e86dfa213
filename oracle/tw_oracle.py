"""CPU oracle for the tile-wise-sparse (TW) GEMM path.  TEST INFRASTRUCTURE ONLY.

NumPy restatement of the reference's host-side algorithm plus a ctypes loader
for the plain-C restatement in ``tw_oracle.c``.  Only the test-suite, the smoke
check and the benchmark's CPU-baseline leg may import this module; the product
package never does.  Reference citations are relative to the reference tree.

A *plan* here is a list of tiles; each tile is a dict with
``col0`` (first original column), ``width`` (original columns in the tile),
``kept_k`` (ascending int32 kept K rows) and ``kept_n`` (ascending int32 kept
columns, relative to ``col0``).

Pins (the reference holds no golden vectors for this path):
  mask_to_offsets        closed form, hand known answer, round trip
  tile_partition         README known answers (768,384) and (3072,1536)
  masked_dense_weight,   brute-force element loops on small inputs and the
  stream_weight          identity  compact_t == (B*mask)[kept_k][:, kept_n]
  cast_bits              numpy.float16; bf16 checked against a second form
  tw_gemm_reference      numpy.matmul on B*mask  vs  the per-tile
                         gather -> GEMM -> scatter form (stream_gemm_nn)
  mask_dense             numpy.matmul
  export_pruned_model    hand known answer; export -> scatter back == kernel * outer(mi, mo)
  basic_lstm_cell        closed form of a third-party routine (TensorFlow is absent): limits
                         (saturated gates), zero input, scipy.special.expit / numpy.tanh
  checkout               hand cases
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


# --------------------------------------------------------------------------- C library
def build(force=False):
    """Compile tw_oracle.c / shuffle_check.cpp with gcc/g++ (see oracle/Makefile)."""
    targets = [os.path.join(_HERE, n) for n in ("libtworacle.so", "libshufflecheck.so")]
    if force or not all(os.path.exists(t) for t in targets):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []),
                              stdout=subprocess.DEVNULL)
    return targets


_clib = None
_shuffle = None


def clib():
    """ctypes handle of libtworacle.so with argument types declared."""
    global _clib
    if _clib is None:
        build()
        L = ctypes.CDLL(os.path.join(_HERE, "libtworacle.so"))
        i32p = ctypes.POINTER(ctypes.c_int32)
        u8p = ctypes.POINTER(ctypes.c_uint8)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        f32p = ctypes.POINTER(ctypes.c_float)
        L.ora_mask_to_offsets.argtypes = [u8p, ctypes.c_int, i32p]
        L.ora_mask_to_offsets.restype = ctypes.c_int
        L.ora_offsets_to_kept.argtypes = [i32p, ctypes.c_int, i32p]
        L.ora_offsets_to_kept.restype = None
        L.ora_mask_gen.argtypes = [ctypes.c_int, ctypes.c_int, i32p]
        L.ora_mask_gen.restype = None
        L.ora_init_matrix.argtypes = [f32p, ctypes.c_int, ctypes.c_int]
        L.ora_init_matrix.restype = None
        L.ora_srand.argtypes = [ctypes.c_uint]
        L.ora_srand.restype = None
        L.ora_transpose_matrix.argtypes = [f32p, f32p, ctypes.c_int, ctypes.c_int]
        L.ora_transpose_matrix.restype = None
        L.ora_tile_partition.argtypes = [ctypes.c_int] * 6 + [i32p] * 5
        L.ora_tile_partition.restype = ctypes.c_int
        for fn in (L.ora_gen_cutlass_weight, L.ora_gen_stream_weight):
            fn.argtypes = [f32p, f32p, ctypes.c_int, ctypes.c_int, i32p, i32p,
                           ctypes.c_int, ctypes.c_int, ctypes.c_int]
            fn.restype = None
        L.ora_cast_f32.argtypes = [f32p, u16p, ctypes.c_int64, ctypes.c_int]
        L.ora_cast_f32.restype = None
        L.ora_uncast_f32.argtypes = [u16p, f32p, ctypes.c_int64, ctypes.c_int]
        L.ora_uncast_f32.restype = None
        L.ora_delete_row.argtypes = [f32p, f32p, ctypes.c_int, ctypes.c_int, i32p]
        L.ora_delete_row.restype = None
        L.ora_insert_row.argtypes = [f32p, f32p, ctypes.c_int, ctypes.c_int, i32p]
        L.ora_insert_row.restype = None
        L.ora_stream_gemm_nn.argtypes = [
            ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float, f32p, f32p,
            ctypes.c_float, f32p, ctypes.c_int, i32p, i32p,
            ctypes.POINTER(i32p), ctypes.POINTER(i32p),
            ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)]
        L.ora_stream_gemm_nn.restype = None
        L.ora_mask_dense.argtypes = [f32p, f32p, u8p, f32p, f32p,
                                     ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.ora_mask_dense.restype = None
        L.ora_checkout.argtypes = [f32p, f32p, ctypes.c_int, ctypes.c_int,
                                   ctypes.c_int, ctypes.c_double]
        L.ora_checkout.restype = ctypes.c_int64
        _clib = L
    return _clib


def shuffle_lib():
    """ctypes handle of libshufflecheck.so (the real std::random_shuffle)."""
    global _shuffle
    if _shuffle is None:
        build()
        L = ctypes.CDLL(os.path.join(_HERE, "libshufflecheck.so"))
        L.ora_std_srand.argtypes = [ctypes.c_uint]
        L.ora_std_mask_gen.argtypes = [ctypes.c_int, ctypes.c_int,
                                       ctypes.POINTER(ctypes.c_int32)]
        _shuffle = L
    return _shuffle


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


# --------------------------------------------------------------------------- integer logic
def mask_to_offsets(mask):
    """0/1 keep vector -> relative offsets kept[i]-i.
    Pruning/BERT/utils/MyHook.py:66-74; basic_nn.cu:713-716."""
    kept = np.flatnonzero(np.asarray(mask) == 1).astype(np.int32)
    return kept - np.arange(kept.size, dtype=np.int32)


def offsets_to_kept(offsets):
    """Relative offsets -> ascending kept indices (i + mask[i], basic_nn.cu:154)."""
    offsets = np.asarray(offsets, dtype=np.int32)
    return offsets + np.arange(offsets.size, dtype=np.int32)


def export_pruned_model(layers):
    """The dictionary the reference's export hook pickles, Pruning/BERT/utils/MyHook.py:54-89,
    restated with its own loop: per layer (scope, mi [K], mo [N], kernel [K,N], bias [N]) the
    entries scope/mask-i:0, mask-o:0 (relative offsets), kernel:0 (kept rows, then kept
    columns) and bias:0 (bias * mo), in that order."""
    def convert_mask_to_offset(mask):          # :66-74
        offset = []
        for index in range(len(mask)):
            if mask[index] == 1:
                offset.append(index - len(offset))
        return np.array(offset, dtype=np.int64)

    ckpt = {}
    for scope, mi, mo, kernel, bias in layers:
        mi, mo = np.asarray(mi), np.asarray(mo)
        k = np.asarray(kernel)[np.array(mi, dtype=bool)]          # :80
        k = (k.T[np.array(mo, dtype=bool)]).T                     # :81
        ckpt[scope + "/mask-i:0"] = convert_mask_to_offset(mi)
        ckpt[scope + "/mask-o:0"] = convert_mask_to_offset(mo)
        ckpt[scope + "/kernel:0"] = k
        ckpt[scope + "/bias:0"] = np.asarray(bias) * mo           # :79
    return ckpt


def tile_partition(M, N, K, N_pruned, K_pruned, n_dim=128):
    """basic_nn.cu:836-885 -> dict of block_num, N_ori, N_cal, K_cal, off_B, off_C."""
    block_num = (N_pruned + n_dim - 1) // n_dim
    K_cal = [K_pruned] * block_num
    N_ori = [N // block_num] * (block_num - 1)
    N_cal = [n_dim] * (block_num - 1)
    N_ori.append(N - sum(N_ori))
    N_cal.append(N_pruned - sum(N_cal))
    off_B, off_C, ob, oc = [], [], 0, 0
    for i in range(block_num):
        off_B.append(ob)
        off_C.append(oc)
        ob += K * N_ori[i]
        oc += M * N_ori[i]
    return dict(block_num=block_num, N_ori=N_ori, N_cal=N_cal, K_cal=K_cal,
                off_B=off_B, off_C=off_C)


def plan_mask(K, N, tiles):
    """Dense 0/1 mask [K,N] of a plan: mask[k, col0+n] = 1 iff k kept and n kept."""
    mask = np.zeros((K, N), dtype=np.uint8)
    for t in tiles:
        kk = np.asarray(t["kept_k"], dtype=np.int64)
        nn = np.asarray(t["kept_n"], dtype=np.int64) + t["col0"]
        if kk.size and nn.size:
            mask[np.ix_(kk, nn)] = 1
    return mask


def plan_from_mask(mask, G):
    """Tile table of a TW mask split every G original columns (tiled_wise_1d style,
    Pruning/VGG/prune_algo.py:119-126): per tile the kept rows are those with any
    kept element and the kept columns those with any kept element."""
    mask = np.asarray(mask)
    K, N = mask.shape
    tiles = []
    for col0 in range(0, N, G):
        w = min(G, N - col0)
        sub = mask[:, col0:col0 + w] != 0
        tiles.append(dict(col0=col0, width=w,
                          kept_k=np.flatnonzero(sub.any(axis=1)).astype(np.int32),
                          kept_n=np.flatnonzero(sub.any(axis=0)).astype(np.int32)))
    return tiles


def masked_dense_weight(B, tiles):
    """gen_cutlass_weight, basic_nn.cu:743-755: B (.) mask, row-major [K,N]."""
    B = np.asarray(B, dtype=np.float32)
    return B * plan_mask(B.shape[0], B.shape[1], tiles)


def stream_weight(B, tiles):
    """gen_masked_stream_weight, basic_nn.cu:757-769: flat fp32 buffer of K*N
    elements; tile t is a K_t x N_t block, column-major with ld=K, starting at
    element K*col0; unused slots are 0."""
    B = np.asarray(B, dtype=np.float32)
    K, N = B.shape
    dst = np.zeros(K * N, dtype=np.float32)
    view = dst.reshape(N, K)  # view[c, i] == dst[c*K + i]
    for t in tiles:
        kk = np.asarray(t["kept_k"], dtype=np.int64)
        nn = np.asarray(t["kept_n"], dtype=np.int64)
        if kk.size and nn.size:
            comp = B[np.ix_(kk, nn + t["col0"])]  # [K_t, N_t]
            view[t["col0"]:t["col0"] + nn.size, :kk.size] = comp.T
    return dst


# --------------------------------------------------------------------------- casts
def cast_bits(x, dtype):
    """fp32 -> 16-bit patterns, round-to-nearest-even (float_to_half, basic_nn.cu:122-137)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dtype == "f16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16).view(np.uint16)
    if dtype == "bf16":
        u = x.view(np.uint32)
        nan = ((u & 0x7F800000) == 0x7F800000) & ((u & 0x007FFFFF) != 0)
        r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
        return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)
    raise ValueError(dtype)


def bits_to_f32(bits, dtype):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    if dtype == "f16":
        return bits.view(np.float16).astype(np.float32)
    if dtype == "bf16":
        return (bits.astype(np.uint32) << 16).view(np.float32)
    raise ValueError(dtype)


def quantize(x, dtype):
    """Values of x after a round trip through the 16-bit type, as fp32."""
    return bits_to_f32(cast_bits(x, dtype), dtype).reshape(np.shape(x))


# --------------------------------------------------------------------------- GEMM
def gelu(x):
    """Pruning/BERT/utils/modeling.py:264-277: the tanh form of GELU."""
    x = np.asarray(x)
    cdf = 0.5 * (1.0 + np.tanh(np.sqrt(2 / np.pi) * (x + 0.044715 * np.power(x, 3))))
    return x * cdf


ACTIVATIONS = {
    None: lambda v: v, "linear": lambda v: v, "none": lambda v: v,
    "relu": lambda v: np.maximum(v, 0), "gelu": gelu, "tanh": np.tanh,
}


def mask_dense(x, kernel, mask, bias=None, activation=None):
    """Pruning/BERT/utils/modeling.py:992-1007: activation(x @ (kernel * mask) + bias) in
    fp32; activation by name as in get_activation (modeling.py:280-305).  This is the
    reference's CPU/TF operator (BLAS-backed here, as TF's matmul is)."""
    y = np.asarray(x, dtype=np.float32) @ (np.asarray(kernel, dtype=np.float32) * mask)
    if bias is not None:
        y = y + bias
    return ACTIVATIONS[activation](y)


def basic_lstm_cell(gate_inputs, c, forget_bias=1.0):
    """The gate arithmetic of TensorFlow 1.x BasicLSTMCell.call, the cell of the reference's NMT
    model (Pruning/NMT/nmt/model_helper.py:400-402): gate_inputs [M, 4H] = concat([x, h]) @
    kernel + bias, split into i, j, f, o; returns (new_c, new_h) in the input's precision."""
    g = np.asarray(gate_inputs)
    i, j, f, o = np.split(g, 4, axis=1)
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    new_c = c * sig(f + forget_bias) + sig(i) * np.tanh(j)
    return new_c, np.tanh(new_c) * sig(o)


def tw_gemm_reference(A, B, tiles, alpha=1.0, beta=0.0, C=None, acc=np.float64):
    """C[M,N] = alpha * A[M,K] @ (B (.) mask) + beta * C on the kept columns; pruned
    columns are returned untouched (C) or zero (C is None).  Dense-matmul form."""
    A = np.asarray(A)
    Bm = masked_dense_weight(B, tiles).astype(acc)
    P = (A.astype(acc) @ Bm) * alpha
    N = Bm.shape[1]
    keep_cols = np.zeros(N, dtype=bool)
    for t in tiles:  # kept columns are always written, even when the tile keeps no K row
        keep_cols[np.asarray(t["kept_n"], dtype=np.int64) + t["col0"]] = True
    out = np.zeros((A.shape[0], N), dtype=acc) if C is None else np.array(C, dtype=acc)
    if beta != 0.0 and C is not None:
        out[:, keep_cols] = P[:, keep_cols] + beta * out[:, keep_cols]
    else:
        out[:, keep_cols] = P[:, keep_cols]
    return out


def stream_gemm_nn(A, B, tiles, alpha=1.0, beta=0.0, C=None, acc=np.float64):
    """Stream_Gemm_NN_reference, basic_nn.cu:450-503, as a second, independent form:
    per tile gather the kept K columns of A, multiply with the compact tile, scatter
    into the kept C columns.  Same argument meaning as tw_gemm_reference."""
    A = np.asarray(A)
    B = np.asarray(B, dtype=np.float32)
    M = A.shape[0]
    N = B.shape[1]
    out = np.zeros((M, N), dtype=acc) if C is None else np.array(C, dtype=acc)
    for t in tiles:
        kk = np.asarray(t["kept_k"], dtype=np.int64)
        nn = np.asarray(t["kept_n"], dtype=np.int64) + t["col0"]
        if nn.size == 0:
            continue
        comp = B[np.ix_(kk, nn)].astype(acc) if kk.size else np.zeros((0, nn.size), acc)
        A2 = A[:, kk].astype(acc)
        C2 = alpha * (A2 @ comp)
        if beta != 0.0 and C is not None:
            C2 = C2 + beta * out[:, nn]
        out[:, nn] = C2
    return out


def rel_error(C, C_ref, floor_frac=1e-2):
    """max |C - C_ref| / max(|C_ref|, floor), floor = floor_frac * rms(C_ref)."""
    C = np.asarray(C, dtype=np.float64)
    C_ref = np.asarray(C_ref, dtype=np.float64)
    if C_ref.size == 0:
        return 0.0
    rms = float(np.sqrt(np.mean(C_ref * C_ref)))
    floor = max(floor_frac * rms, 1e-30)
    return float(np.max(np.abs(C - C_ref) / np.maximum(np.abs(C_ref), floor)))


def checkout(host_cutlass, host_reference, trans=False, err=1e-2):
    """basic_nn.cu:771-798: number of elements failing
    v1/v2 > 1+err or v2/v1 > 1+err or |v2-v1| > err (NaN compares false)."""
    v2 = np.asarray(host_cutlass, dtype=np.float32)
    v1 = np.asarray(host_reference, dtype=np.float32)
    if trans:
        v1 = v1.T
    with np.errstate(divide="ignore", invalid="ignore"):
        bad = (v1 / v2 > np.float32(1 + err)) | (v2 / v1 > np.float32(1 + err)) \
            | (np.abs(v2 - v1) > np.float32(err))
    return int(np.count_nonzero(bad))


# --------------------------------------------------------------------------- reference-compatible inputs
def ref_compat_problem(M, N, K, N_pruned, K_pruned, n_dim=128, seed=1):
    """Regenerates the inputs of `test_basic_nn M N K N_pruned K_pruned` exactly as
    the reference draws them: glibc rand() (never seeded => seed 1), consumed in the
    order init_matrix(A) -> init_matrix(B) -> per tile mask_gen(K) then mask_gen(N_ori)
    (basic_nn.cu:822-825, 891-903)."""
    L = clib()
    L.ora_srand(seed)
    A = np.empty((M, K), dtype=np.float32)
    B = np.empty((K, N), dtype=np.float32)
    L.ora_init_matrix(_p(A, ctypes.c_float), M, K)
    L.ora_init_matrix(_p(B, ctypes.c_float), K, N)
    part = tile_partition(M, N, K, N_pruned, K_pruned, n_dim)
    tiles, col0 = [], 0
    for i in range(part["block_num"]):
        mk = np.empty(part["K_cal"][i], dtype=np.int32)
        mn = np.empty(part["N_cal"][i], dtype=np.int32)
        L.ora_mask_gen(K, part["K_cal"][i], _p(mk, ctypes.c_int32))
        L.ora_mask_gen(part["N_ori"][i], part["N_cal"][i], _p(mn, ctypes.c_int32))
        tiles.append(dict(col0=col0, width=part["N_ori"][i],
                          kept_k=offsets_to_kept(mk), kept_n=offsets_to_kept(mn),
                          mask_k=mk, mask_n=mn))
        col0 += part["N_ori"][i]
    return A, B, tiles, part
