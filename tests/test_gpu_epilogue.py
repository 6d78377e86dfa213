"""GPU parity of the fused epilogue (tw_gemm_ex: bias and activation) against the oracle's
mask_dense (Pruning/BERT/utils/modeling.py:992-1007) on the same 16-bit inputs.

Floating point: tolerance as for the plain GEMM (max relative error <= 1e-2 fp16, 2e-2 bf16,
with the 1e-2 * rms floor); pruned columns under TW_PRUNED_ZERO must equal act(bias) rounded to
the output type, bit for bit for the identity and ReLU."""
import numpy as np
import pytest

from tests.helpers import from_device_bits, random_tiles, to_device_bits
from tests.test_gpu_gemm import kept_columns, round_up

pytestmark = pytest.mark.gpu

TOL = {"f16": 1e-2, "bf16": 2e-2}
ACTS = [("none", 0), ("relu", 1), ("gelu", 2), ("tanh", 3)]


def run(tw, oracle, plan, A, dtype, N, bias, act, alpha=1.0, beta=0.0, C0=None, pruned=1,
        row_major=False):
    import torch
    M, K = A.shape
    if row_major:
        lda, ldc = round_up(K, 8), round_up(N, 8)
        Ab = np.zeros((M, lda), np.uint16)
        Ab[:, :K] = oracle.cast_bits(A, dtype).reshape(M, K)
        Cb = np.zeros((M, ldc), np.uint16)
        if C0 is not None:
            Cb[:, :N] = oracle.cast_bits(C0, dtype).reshape(M, N)
        dA, dC = to_device_bits(Ab, Ab.shape), to_device_bits(Cb, Cb.shape)
        lay = tw.ROWMAJOR
    else:
        lda = ldc = round_up(M, 8)
        Ab = np.zeros((K, lda), np.uint16)
        Ab[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
        Cb = np.zeros((N, ldc), np.uint16)
        if C0 is not None:
            Cb[:, :M] = oracle.cast_bits(C0, dtype).reshape(M, N).T
        dA, dC = to_device_bits(Ab, Ab.shape), to_device_bits(Cb, Cb.shape)
        lay = tw.KMAJOR
    dbias = None if bias is None else torch.from_numpy(np.ascontiguousarray(bias, np.float32)).cuda()
    plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, alpha=alpha, beta=beta,
              a_layout=lay, c_layout=lay, pruned_cols=pruned,
              stream=torch.cuda.current_stream().cuda_stream,
              bias_ptr=None if dbias is None else dbias.data_ptr(), activation=act)
    torch.cuda.synchronize()
    bits = from_device_bits(dC)
    if row_major:
        return oracle.bits_to_f32(bits[:, :N], dtype).reshape(M, N)
    return oracle.bits_to_f32(bits[:, :M], dtype).reshape(N, M).T.copy()


def reference(oracle, A, B, tiles, dtype, bias, act_name, alpha=1.0, beta=0.0, C0=None):
    Aq, Bq = oracle.quantize(A, dtype).astype(np.float64), oracle.quantize(B, dtype).astype(np.float64)
    mask = oracle.plan_mask(B.shape[0], B.shape[1], tiles).astype(np.float64)
    y = alpha * (Aq @ (Bq * mask))
    if beta != 0.0:
        y = y + beta * oracle.quantize(C0, dtype).astype(np.float64)
    if bias is not None:
        y = y + bias.astype(np.float64)
    return oracle.ACTIVATIONS[None if act_name == "none" else act_name](y)


CASES = [
    # M,   K,   N,   G,  k_keep n_keep
    (512, 256, 512, 128, 0.25, 0.9),    # wide tiles: the wave-specialised kernel
    (100, 96, 200, 128, 0.3, 0.9),      # few items: 128 x 128 shape, ragged M
    (520, 300, 320, 64, 0.2, 0.8),      # G = 64: narrow shapes
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("act_name,act", ACTS)
@pytest.mark.parametrize("case", CASES)
def test_bias_and_activation(tw, oracle, case, act_name, act, dtype):
    M, K, N, G, kk, nk = case
    rng = np.random.default_rng(abs(hash((case, act_name))) % 2 ** 31)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.08).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=kk, n_keep=nk)
    print("case", case, act_name, dtype, flush=True)
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        C = run(tw, oracle, plan, A, dtype, N, bias, act)
        ref = reference(oracle, A, B, tiles, dtype, bias, act_name)
        assert oracle.rel_error(C, ref) <= TOL[dtype]
        # pruned columns: act(bias), one rounding
        keep = kept_columns(tiles, N)
        if (~keep).any() and act_name in ("none", "relu"):
            want = oracle.quantize(oracle.ACTIVATIONS[None if act_name == "none" else act_name](bias), dtype)
            assert np.array_equal(C[:, ~keep], np.broadcast_to(want[~keep], (M, int((~keep).sum()))))
        # activation without bias, and bias with beta
        C2 = run(tw, oracle, plan, A, dtype, N, None, act)
        assert oracle.rel_error(C2, reference(oracle, A, B, tiles, dtype, None, act_name)) <= TOL[dtype]
        C0 = rng.standard_normal((M, N)).astype(np.float32)
        C3 = run(tw, oracle, plan, A, dtype, N, bias, act, alpha=0.5, beta=-1.5, C0=C0)
        ref3 = reference(oracle, A, B, tiles, dtype, bias, act_name, alpha=0.5, beta=-1.5, C0=C0)
        assert oracle.rel_error(C3, ref3) <= TOL[dtype]


@pytest.mark.parametrize("act_name,act", ACTS)
def test_row_major_epilogue(tw, oracle, act_name, act):
    rng = np.random.default_rng(31)
    M, K, N, G = 130, 160, 256, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.08).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.8)
    with tw.Plan.create(K, N, "f16", tiles, B) as plan:
        C = run(tw, oracle, plan, A, "f16", N, bias, act, row_major=True)
        assert oracle.rel_error(C, reference(oracle, A, B, tiles, "f16", bias, act_name)) <= 1e-2


def test_untouched_columns_stay_untouched(tw, oracle):
    rng = np.random.default_rng(32)
    M, K, N, G = 256, 128, 256, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.08).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=0.5)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    with tw.Plan.create(K, N, "f16", tiles, B) as plan:
        C = run(tw, oracle, plan, A, "f16", N, bias, 2, C0=C0, pruned=0)
        keep = kept_columns(tiles, N)
        assert np.array_equal(C[:, ~keep], oracle.quantize(C0, "f16")[:, ~keep])


def test_plain_gemm_is_the_null_epilogue(tw, oracle):
    import torch
    rng = np.random.default_rng(33)
    M, K, N, G = 384, 192, 256, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.08).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=0.9)
    with tw.Plan.create(K, N, "f16", tiles, B) as plan:
        C1 = run(tw, oracle, plan, A, "f16", N, None, 0)
        zero = np.zeros(N, np.float32)
        C2 = run(tw, oracle, plan, A, "f16", N, zero, 0)
        assert np.array_equal(C1, C2)
        with pytest.raises(tw.TwError):
            plan.gemm(1, 1, M, activation=9, bias_ptr=torch.zeros(N, device="cuda").data_ptr())
