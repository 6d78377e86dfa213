"""The weight-stationary kernel (TW_SHAPE_BS: a unit's packed weight in registers, the kept rows of A
streamed through LDS by loads that write LDS directly) against the streaming 256 x 128 kernel, bit
for bit, and against the oracle (max relative error 1e-2 fp16 / 2e-2 bf16).  It takes plans whose
tiles keep at most 192 rows, K-major operands and beta == 0; a forced shape it does not take falls
back to the automatic choice."""
import numpy as np
import pytest

from tests.helpers import from_device_bits, to_device_bits

pytestmark = pytest.mark.gpu

TOL = {"f16": 1e-2, "bf16": 2e-2}
SENTINEL = 0x1234


def make_tiles(rng, K, G, spec):
    tiles = []
    for t, (kt, nt) in enumerate(spec):
        tiles.append(dict(col0=t * G, width=G,
                          kept_k=np.sort(rng.choice(K, size=kt, replace=False)).astype(np.int32),
                          kept_n=np.sort(rng.choice(G, size=nt, replace=False)).astype(np.int32)))
    return tiles


CASES = [
    # M, K, G, (kept rows, kept columns) per tile
    (333, 700, 128, ((192, 128), (64, 100), (0, 128), (191, 128), (130, 7), (1, 33))),    # up to three steps
    (1000, 300, 128, ((128, 128), (65, 96), (100, 128))),                                  # two steps
    (4100, 520, 64, ((190, 64), (3, 51), (129, 33), (0, 10), (64, 64))),                   # three steps, G = 64
    (64, 200, 32, ((10, 32), (70, 20))),                                                   # one range, few rows
    (2500, 256, 128, tuple((60 + 3 * t, 128 - t) for t in range(40))),                     # more units than argument slots
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_weight_stationary_kernel(tw, oracle, dtype, case):
    import torch
    M, K, G, spec = CASES[case]
    N = G * len(spec)
    rng = np.random.default_rng(900 + case)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = make_tiles(rng, K, G, spec)
    keep = np.zeros(N, bool)
    for t in tiles:
        keep[t["col0"] + t["kept_n"]] = True
    dbias = torch.from_numpy(bias).cuda()
    lda = ldc = (M + 7) // 8 * 8 + 8
    At = np.zeros((K, lda), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    dA = to_device_bits(At, At.shape)
    s = torch.cuda.current_stream().cuda_stream

    def launch(plan, shape, alpha, pruned, with_bias, act, per_cu=-1):
        dC = torch.full((N, ldc), SENTINEL, dtype=torch.int16, device="cuda")
        tw.set_option(tw.OPT_SHAPE, shape)
        tw.set_option(tw.OPT_WGS_PER_CU, per_cu)
        print("weight-stationary test: case", case, "shape", shape, alpha, pruned, with_bias, act, per_cu, dtype, flush=True)
        plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, alpha=alpha, pruned_cols=pruned,
                  bias_ptr=dbias.data_ptr() if with_bias else None, activation=act, stream=s)
        torch.cuda.synchronize()
        return from_device_bits(dC)

    try:
        with tw.Plan.create(K, N, dtype, tiles, B) as plan:
            for (alpha, pruned, with_bias, act) in ((1.0, tw.PRUNED_UNTOUCHED, False, tw.ACT_NONE),
                                                    (0.5, tw.PRUNED_ZERO, True, tw.ACT_RELU),
                                                    (1.0, tw.PRUNED_ZERO, True, tw.ACT_TANH)):
                want = launch(plan, tw.SHAPE_256x128, alpha, pruned, with_bias, act)
                for per_cu in (-1, 1, 8):     # few and many ranges of rows
                    got = launch(plan, tw.SHAPE_BS, alpha, pruned, with_bias, act, per_cu)
                    if act == tw.ACT_TANH:
                        a = oracle.bits_to_f32(got[:, :M], dtype)
                        b = oracle.bits_to_f32(want[:, :M], dtype)
                        assert oracle.rel_error(a, b) <= 0.5 * TOL[dtype]
                        assert np.array_equal(got[:, M:], want[:, M:])
                    else:
                        assert np.array_equal(got, want), (alpha, pruned, with_bias, act, per_cu)
                    again = launch(plan, tw.SHAPE_BS, alpha, pruned, with_bias, act, per_cu)
                    assert np.array_equal(got, again)
                if not with_bias:
                    Cf = oracle.bits_to_f32(got[:, :M], dtype).reshape(N, M).T
                    ref = oracle.stream_gemm_nn(oracle.quantize(A, dtype), oracle.quantize(B, dtype), tiles, alpha)
                    assert oracle.rel_error(Cf[:, keep], ref[:, keep]) <= TOL[dtype]
                    assert np.all(got[~keep, :] == SENTINEL) and np.all(got[:, M:] == SENTINEL)
    finally:
        tw.set_option(tw.OPT_SHAPE, -1)
        tw.set_option(tw.OPT_WGS_PER_CU, -1)


def test_weight_stationary_kernel_declines(tw, oracle):
    """Tiles with more than 192 kept rows, or beta != 0: the forced shape does not apply and the
    launch runs what it would have run anyway (same bits as the automatic choice)."""
    import torch
    rng = np.random.default_rng(77)
    M, K, G = 300, 600, 128
    tiles = make_tiles(rng, K, G, ((300, 128), (100, 128)))
    N = 2 * G
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    At = np.ascontiguousarray(oracle.cast_bits(A, "f16").reshape(M, K).T)
    ld = 304
    Ap = np.zeros((K, ld), np.uint16)
    Ap[:, :M] = At
    dA = to_device_bits(Ap, Ap.shape)
    s = torch.cuda.current_stream().cuda_stream
    out = []
    try:
        with tw.Plan.create(K, N, "f16", tiles, B) as plan:
            for shape in (-1, tw.SHAPE_BS):
                tw.set_option(tw.OPT_SHAPE, shape)
                dC = torch.zeros((N, ld), dtype=torch.int16, device="cuda")
                plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=ld, ldc=ld, stream=s)
                torch.cuda.synchronize()
                out.append(from_device_bits(dC).copy())
    finally:
        tw.set_option(tw.OPT_SHAPE, -1)
    assert np.array_equal(out[0], out[1])
