"""Rows of A that no tile keeps never reach a product: the reference's gathered load reads the
kept rows only (cutlass/tile_iterator.h:786-816; the gather -> GEMM -> scatter restatement,
basic_nn.cu:450-503), so Inf and NaN in a row a tile prunes leave its columns finite.  The
engine pads a tile's list of kept rows to whole steps of 64; whatever is fetched for the padding
has to be discarded, not multiplied by the zero weight behind it (Inf * 0 = NaN).

Every kernel family is forced in turn on tiles whose kept-row counts are no multiples of 64,
with +Inf, -Inf and NaN in rows 0, 5 and K - 1, which no tile keeps.  The result must be finite
and within the GEMM tolerance (1e-2 fp16, 2e-2 bf16) of the oracle's gather form on the same
operands."""
import numpy as np
import pytest

from tests.helpers import from_device_bits, to_device_bits

pytestmark = pytest.mark.gpu

TOL = {"f16": 1e-2, "bf16": 2e-2}
F16_BITS = {"inf": 0x7C00, "ninf": 0xFC00, "nan": 0x7E00}
BF16_BITS = {"inf": 0x7F80, "ninf": 0xFF80, "nan": 0x7FC0}


def poisoned_problem(rng, oracle, M, K, N, G, kts, dtype, n_keep=1.0):
    """Tiles that keep none of the rows 0, 5, K-1; A (K-major bits) with non-finite values there."""
    dead = np.array([0, 5, K - 1])
    live = np.setdiff1d(np.arange(K), dead)
    tiles = []
    for t, c0 in enumerate(range(0, N, G)):
        w = min(G, N - c0)
        kt = kts[t % len(kts)]
        nt = int(round(w * n_keep))
        tiles.append(dict(col0=c0, width=w,
                          kept_k=np.sort(rng.choice(live, size=kt, replace=False)).astype(np.int32),
                          kept_n=np.sort(rng.choice(w, size=nt, replace=False)).astype(np.int32)))
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    ld = (M + 7) // 8 * 8
    At = np.zeros((K, ld), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    bits = F16_BITS if dtype == "f16" else BF16_BITS
    At[0, :] = bits["inf"]
    At[0, 1::2] = bits["nan"]
    At[5, :] = bits["ninf"]
    At[K - 1, :] = bits["nan"]
    A_clean = A.copy()
    A_clean[:, dead] = 0.0          # what the oracle's gather never looks at anyway
    return tiles, A_clean, B, At, ld


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_unkept_rows_with_inf_and_nan_leave_c_finite(tw, oracle, dtype):
    import torch
    rng = np.random.default_rng(2024)
    cases = (
        # M, K, N, G, kept rows per tile (none a multiple of 64), shapes to force
        (200, 300, 384, 128, (70, 130, 1),
         (tw.SHAPE_AS64, tw.SHAPE_AS32, tw.SHAPE_SKINNY, tw.SHAPE_BS, tw.SHAPE_256x128, tw.SHAPE_128x128,
          tw.SHAPE_128x64, tw.SHAPE_WIDE, -1)),
        (96, 520, 256, 64, (3, 190, 65, 127),
         (tw.SHAPE_AS64, tw.SHAPE_AS32, tw.SHAPE_SKINNY, tw.SHAPE_BS, tw.SHAPE_512x64, tw.SHAPE_256x64,
          tw.SHAPE_128x32, -1)),
    )
    s = torch.cuda.current_stream().cuda_stream
    try:
        for (M, K, N, G, kts, shapes) in cases:
            tiles, A_clean, B, At, ld = poisoned_problem(rng, oracle, M, K, N, G, kts, dtype, n_keep=0.9)
            ref = oracle.stream_gemm_nn(oracle.quantize(A_clean, dtype), oracle.quantize(B, dtype), tiles)
            keep = np.zeros(N, bool)
            for t in tiles:
                keep[t["col0"] + t["kept_n"]] = True
            dA = to_device_bits(At, At.shape)
            with tw.Plan.create(K, N, dtype, tiles, B) as plan:
                for shape in shapes:
                    for layout in ("kmajor", "rowmajor", "mixed"):
                        if layout != "kmajor" and shape != -1:
                            continue
                        tw.set_option(tw.OPT_SHAPE, shape)
                        print("non-finite rows: shape", shape, layout, M, K, N, G, dtype, flush=True)
                        if layout == "kmajor":
                            dC = torch.zeros((N, ld), dtype=torch.int16, device="cuda")
                            plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=ld, ldc=ld, stream=s)
                            torch.cuda.synchronize()
                            C = oracle.bits_to_f32(from_device_bits(dC)[:, :M], dtype).reshape(N, M).T
                        else:
                            # row-major A: with a row-major C the A-stationary kernel in its
                            # row-major form, with a K-major C the layout-generic kernel
                            ldk = (K + 7) // 8 * 8
                            Ar = np.zeros((M, ldk), np.uint16)
                            Ar[:, :K] = At[:, :M].T
                            dAr = to_device_bits(Ar, Ar.shape)
                            if layout == "rowmajor":
                                dC = torch.zeros((M, N), dtype=torch.int16, device="cuda")
                                plan.gemm(dAr.data_ptr(), dC.data_ptr(), M, lda=ldk, ldc=N,
                                          a_layout=tw.ROWMAJOR, c_layout=tw.ROWMAJOR, stream=s)
                                torch.cuda.synchronize()
                                C = oracle.bits_to_f32(from_device_bits(dC), dtype).reshape(M, N)
                            else:
                                dC = torch.zeros((N, ld), dtype=torch.int16, device="cuda")
                                plan.gemm(dAr.data_ptr(), dC.data_ptr(), M, lda=ldk, ldc=ld,
                                          a_layout=tw.ROWMAJOR, c_layout=tw.KMAJOR, stream=s)
                                torch.cuda.synchronize()
                                C = oracle.bits_to_f32(from_device_bits(dC)[:, :M], dtype).reshape(N, M).T
                        assert np.all(np.isfinite(C)), (shape, layout)
                        assert oracle.rel_error(C[:, keep], ref[:, keep]) <= TOL[dtype], (shape, layout)
    finally:
        tw.set_option(tw.OPT_SHAPE, -1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_lstm_step_ignores_unkept_rows(tw, oracle, dtype):
    """The fused time step gathers the same padded lists: non-finite values in rows of [x, h] that
    no gate tile keeps leave h and c finite and equal to the step on a clean A, bit for bit."""
    import torch
    rng = np.random.default_rng(77)
    M, I, H, G = 72, 44, 128, 128
    K, N = I + H, 4 * H
    tiles, A_clean, W, At, ld = poisoned_problem(rng, oracle, M, K, N, G, (50, 70, 100, 33), dtype)
    At_clean = At.copy()
    At_clean[[0, 5, K - 1], :] = 0
    c0 = (rng.standard_normal((H, ld)) * 0.5).astype(np.float32)
    s = torch.cuda.current_stream().cuda_stream
    out = []
    with tw.Plan.create(K, N, dtype, tiles, W) as plan:
        for a in (At, At_clean):
            dA = to_device_bits(a, a.shape)
            dC = torch.from_numpy(c0.copy()).cuda()
            dH = torch.zeros((H, ld), dtype=torch.int16, device="cuda")
            print("non-finite rows: lstm step", dtype, flush=True)
            plan.lstm_step(dA.data_ptr(), M, dC.data_ptr(), dC.data_ptr(), dH.data_ptr(), lda=ld,
                           ldc_prev=ld, ldc_new=ld, ldh=ld, stream=s)
            torch.cuda.synchronize()
            out.append((from_device_bits(dH).copy(), dC.cpu().numpy().copy()))
    h_bits, c = out[0]
    assert np.all(np.isfinite(c[:, :M]))
    assert np.all(np.isfinite(oracle.bits_to_f32(h_bits[:, :M], dtype)))
    assert np.array_equal(h_bits, out[1][0]) and np.array_equal(c, out[1][1])
    # and the clean step is the oracle's cell on the oracle's gate GEMM
    q = lambda v: oracle.quantize(np.asarray(v, np.float32), dtype).astype(np.float64)
    gates = oracle.stream_gemm_nn(q(A_clean), q(W), tiles)
    want_c, want_h = oracle.basic_lstm_cell(gates, c0[:, :M].T.astype(np.float64), 1.0)
    got_h = oracle.bits_to_f32(h_bits[:, :M], dtype).reshape(H, M).T
    assert oracle.rel_error(got_h, want_h) <= 2 * TOL[dtype]
    assert oracle.rel_error(c[:, :M].T, want_c) <= 2 * TOL[dtype]
