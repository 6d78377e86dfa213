"""tw_gemm_static, the entry point that allocates nothing (work-queue counters in the library's
own device array), through the C ABI: its output equals tw_gemm_ex's bit for bit and matches the
oracle, on two calls in a row, the second with a smaller input.

Only the streaming kernels draw work from counters (the A-stationary, weight-stationary and skinny
kernels map workgroups to work directly), and at these sizes the launch would pick one of the
latter by itself.  The streaming kernels are therefore forced with tw_set_option, so that the
kernels under test read, advance and re-arm the static array: 256 x 128 items, 128 x 64 items of
64-column pieces, and the per-die queue layout."""
import numpy as np
import pytest

from tests.helpers import from_device_bits, random_tiles, to_device_bits

pytestmark = pytest.mark.gpu

TOL = {"f16": 1e-2, "bf16": 2e-2}
SENTINEL = 0x1234


def _run(tw, oracle, plan, A, dtype, N, static, bias=None, act=0, pruned=0):
    import torch
    M, K = A.shape
    ld = (M + 7) // 8 * 8
    At = np.zeros((K, ld), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    dA = to_device_bits(At, (K, ld))
    dC = to_device_bits(np.full((N, ld), SENTINEL, np.uint16), (N, ld))
    d_bias = None if bias is None else torch.from_numpy(bias).cuda()
    plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=ld, ldc=ld, pruned_cols=pruned,
              stream=torch.cuda.current_stream().cuda_stream,
              bias_ptr=None if d_bias is None else d_bias.data_ptr(), activation=act, static=static)
    torch.cuda.synchronize()
    bits = from_device_bits(dC)
    return oracle.bits_to_f32(bits[:, :M], dtype).reshape(N, M).T.copy(), bits


def _forced(tw):
    """(kernel shape, piece width, per-die queues) of the launches that use the counters; the last
    entry leaves the choice to the launch (a kernel without counters at these sizes)."""
    return ((tw.SHAPE_256x128, -1, 0), (tw.SHAPE_128x64, 64, 0), (tw.SHAPE_256x128, -1, 1),
            (tw.SHAPE_128x64, 64, 1), (-1, -1, -1))


def _force(tw, shape, piece, xcd):
    tw.set_option(tw.OPT_SHAPE, shape)
    tw.set_option(tw.OPT_PIECE, piece)
    tw.set_option(tw.OPT_XCD_QUEUES, xcd)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_static_entry_point_equals_tw_gemm_ex(tw, oracle, dtype):
    rng = np.random.default_rng(4711)
    K, N, G = 448, 640, 128
    B = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.3, n_keep=0.9)
    keep = np.concatenate([t["col0"] + np.asarray(t["kept_n"]) for t in tiles])
    Bq = oracle.quantize(B, dtype)
    bias = rng.standard_normal(N).astype(np.float32)
    try:
        with tw.Plan.create(K, N, dtype, tiles, B) as plan:
            for shape, piece, xcd in _forced(tw):
                _force(tw, shape, piece, xcd)
                if shape >= 0:
                    assert plan.choice(1500, 1504, 1504)["shape"] == shape
                # two calls in a row through the new entry point, the second with a smaller input;
                # the existing entry point on the same inputs in between must not disturb it either
                for M in (1500, 130):
                    A = rng.standard_normal((M, K)).astype(np.float32)
                    ref = oracle.tw_gemm_reference(oracle.quantize(A, dtype), Bq, tiles)
                    print("tw_gemm_static", dtype, "shape", shape, "piece", piece, "xcd", xcd, "M", M, flush=True)
                    C_s, bits_s = _run(tw, oracle, plan, A, dtype, N, static=True)
                    C_e, bits_e = _run(tw, oracle, plan, A, dtype, N, static=False)
                    assert np.array_equal(bits_s, bits_e), "differs from tw_gemm_ex (M=%d)" % M
                    assert oracle.rel_error(C_s[:, keep], ref[:, keep]) <= TOL[dtype]
                    # pruned columns and the padding rows keep the sentinel
                    pruned_cols = np.setdiff1d(np.arange(N), keep)
                    assert (bits_s[pruned_cols] == SENTINEL).all()
                # the fused epilogue and the zero-fill of pruned columns go through the same counters
                A = rng.standard_normal((700, K)).astype(np.float32)
                print("tw_gemm_static", dtype, "epilogue", flush=True)
                _, bits_s = _run(tw, oracle, plan, A, dtype, N, True, bias=bias, act=tw.ACT_RELU, pruned=1)
                _, bits_e = _run(tw, oracle, plan, A, dtype, N, False, bias=bias, act=tw.ACT_RELU, pruned=1)
                assert np.array_equal(bits_s, bits_e)
    finally:
        _force(tw, -1, -1, -1)


def test_static_entry_point_in_a_graph(tw, oracle):
    """Launches through the static counters recorded into a HIP graph (a kernel clears the
    counters, so no memset node is recorded): every replay, with eager launches through the same
    counters in between, gives the eager result bit for bit.  The plan was built before the
    capture began, which is all the set-up the entry point needs."""
    import torch
    rng = np.random.default_rng(99)
    M, K, N, G = 900, 320, 512, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.9)
    ld = (M + 7) // 8 * 8
    At = np.zeros((K, ld), np.uint16)
    At[:, :M] = oracle.cast_bits(A, "f16").reshape(M, K).T
    dA = to_device_bits(At, At.shape)
    dH = torch.zeros((N, ld), dtype=torch.int16, device="cuda")
    dC = torch.zeros((N, ld), dtype=torch.int16, device="cuda")
    s = torch.cuda.Stream()
    try:
        _force(tw, tw.SHAPE_128x64, 64, 1)
        with tw.Plan.create(K, N, "f16", tiles, B) as plan:
            assert plan.choice(M, ld, ld)["shape"] == tw.SHAPE_128x64

            def chain():
                plan.gemm(dA.data_ptr(), dH.data_ptr(), M, lda=ld, ldc=ld, pruned_cols=tw.PRUNED_ZERO,
                          stream=s.cuda_stream, static=True)
                plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=ld, ldc=ld, alpha=0.5, pruned_cols=tw.PRUNED_ZERO,
                          stream=s.cuda_stream, static=True)
                plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=ld, ldc=ld, alpha=1.0, beta=1.0,
                          stream=s.cuda_stream, static=True)
            with torch.cuda.stream(s):
                print("tw_gemm_static in a graph: eager", flush=True)
                chain()
                s.synchronize()
                want_h, want_c = dH.clone(), dC.clone()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=s):
                    chain()
                for rep in range(4):
                    print("tw_gemm_static in a graph: replay", rep, flush=True)
                    dH.fill_(0x1234)
                    dC.fill_(0x1234)
                    plan.gemm(dA.data_ptr(), dH.data_ptr(), M, lda=ld, ldc=ld, stream=s.cuda_stream, static=True)
                    s.synchronize()
                    g.replay()
                    s.synchronize()
                    assert torch.equal(dH[:, :M], want_h[:, :M]) and torch.equal(dC[:, :M], want_c[:, :M]), rep
                    assert bool((dH[:, M:] == 0x1234).all()) and bool((dC[:, M:] == 0x1234).all())
    finally:
        _force(tw, -1, -1, -1)


def test_static_entry_point_row_major_and_errors(tw, oracle):
    """Layouts that need no counters also go through the entry point; argument errors come
    back as they do from tw_gemm_ex."""
    import torch
    rng = np.random.default_rng(12)
    M, K, N, G = 200, 192, 256, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=1.0)
    with tw.Plan.create(K, N, "f16", tiles, B) as plan:
        dA = to_device_bits(oracle.cast_bits(A, "f16").reshape(M, K), (M, K))
        outs = []
        for static in (True, False):
            dC = to_device_bits(np.zeros((M, N), np.uint16), (M, N))
            plan.gemm(dA.data_ptr(), dC.data_ptr(), M, a_layout=tw.ROWMAJOR, c_layout=tw.ROWMAJOR,
                      stream=torch.cuda.current_stream().cuda_stream, static=static)
            torch.cuda.synchronize()
            outs.append(from_device_bits(dC))
        assert np.array_equal(outs[0], outs[1])
        with pytest.raises(tw.TwError) as e:
            plan.gemm(0, 0, M, static=True)
        assert e.value.status == tw.ERR_NULL
        with pytest.raises(tw.TwError) as e:
            plan.gemm(dA.data_ptr(), dA.data_ptr(), -1, static=True)
        assert e.value.status == tw.ERR_SHAPE
