"""GPU parity of the LSTM gate arithmetic (tw_lstm_gates) against the oracle's BasicLSTMCell
restatement, alone and inside a two-step recurrence that runs the reference's NMT gate GEMM
(concat([x, h]) @ (kernel * mask) + bias) through tw_gemm_ex with the new h written straight
into the next step's K-major A.

Tolerances: c (fp32) 1e-5 relative to max |c|; h (16-bit) max relative error 1e-2 (fp16) /
2e-2 (bf16) with the 1e-2 * rms floor, as for the GEMM."""
import numpy as np
import pytest

from tests.helpers import from_device_bits, random_tiles, to_device_bits

pytestmark = pytest.mark.gpu

TOL = {"f16": 1e-2, "bf16": 2e-2}


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,H", [(128, 256), (100, 96), (7, 8), (264, 1024)])
def test_gates_match_oracle(tw, oracle, M, H, dtype):
    import torch
    rng = np.random.default_rng(M * 1000 + H)
    ld = (M + 7) // 8 * 8
    g = (rng.standard_normal((M, 4 * H)) * 2).astype(np.float32)
    c = rng.standard_normal((M, H)).astype(np.float32)
    gb = np.zeros((4 * H, ld), np.uint16)
    gb[:, :M] = oracle.cast_bits(g, dtype).reshape(M, 4 * H).T
    cp = np.zeros((H, ld), np.float32)
    cp[:, :M] = c.T
    dg, dc = to_device_bits(gb, gb.shape), torch.from_numpy(cp).cuda()
    dcn = torch.full((H, ld), 7.0, dtype=torch.float32, device="cuda")
    dh = torch.full((H, ld), 0x3C00, dtype=torch.int16, device="cuda")
    print("gates", M, H, dtype, flush=True)
    tw.lstm_gates(M, H, dtype, dg.data_ptr(), ld, 1.0, dc.data_ptr(), ld, dcn.data_ptr(), ld,
                  dh.data_ptr(), ld, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want_c, want_h = oracle.basic_lstm_cell(oracle.quantize(g, dtype).astype(np.float64), c.astype(np.float64), 1.0)
    got_c = dcn.cpu().numpy()
    got_h = oracle.bits_to_f32(from_device_bits(dh), dtype).reshape(H, ld)
    assert np.max(np.abs(got_c[:, :M].T - want_c)) <= 1e-5 * np.max(np.abs(want_c))
    assert oracle.rel_error(got_h[:, :M].T, want_h) <= TOL[dtype]
    # padding beyond M is not written
    if ld > M:
        assert np.all(got_c[:, M:] == 7.0) and np.all(from_device_bits(dh)[:, M:] == 0x3C00)
    # in place on c
    tw.lstm_gates(M, H, dtype, dg.data_ptr(), ld, 1.0, dc.data_ptr(), ld, dc.data_ptr(), ld,
                  dh.data_ptr(), ld, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert np.array_equal(dc.cpu().numpy()[:, :M], got_c[:, :M])


def test_gate_argument_errors(tw):
    with pytest.raises(tw.TwError):
        tw.lstm_gates(8, 8, "f16", 0, 8, 1.0, 0, 8, 0, 8, 0, 8)
    with pytest.raises(tw.TwError):
        tw.lstm_gates(8, 8, "f16", 16, 4, 1.0, 16, 8, 16, 8, 16, 8)      # ldg < M
    with pytest.raises(tw.TwError):
        tw.lstm_gates(8, 8, "f16", 16, 12, 1.0, 16, 8, 16, 8, 16, 8)     # ldg not a multiple of 8
    with pytest.raises(tw.TwError):
        tw.lstm_gates(8, 0, "f16", 16, 8, 1.0, 16, 8, 16, 8, 16, 8)
    tw.lstm_gates(0, 8, "f16", 0, 8, 1.0, 0, 8, 0, 8, 0, 8)               # M = 0: no-op


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_two_step_recurrence(tw, oracle, dtype):
    """x_t and h_{t-1} share one K-major A; the gate kernel writes h_t into the rows of the next
    step's A, the masked gate GEMM adds the bias in its epilogue."""
    import torch
    rng = np.random.default_rng(91)
    M, I, H, G = 128, 192, 256, 128
    K, N = I + H, 4 * H
    W = (rng.standard_normal((K, N)) * 0.08).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.5).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=1.0)
    mask = oracle.plan_mask(K, N, tiles)
    xs = [rng.standard_normal((M, I)).astype(np.float32) for _ in range(2)]
    h0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    c0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    ld = M
    s = torch.cuda.current_stream().cuda_stream
    # A_t = [x_t ; h_{t-1}] as K-major rows
    A = []
    for t in range(3):
        a = np.zeros((K, ld), np.uint16)
        if t < 2:
            a[:I] = oracle.cast_bits(xs[t], dtype).reshape(M, I).T
        A.append(a)
    A[0][I:] = oracle.cast_bits(h0, dtype).reshape(M, H).T
    dA = [to_device_bits(a, a.shape) for a in A]
    dC = torch.from_numpy(np.ascontiguousarray(c0.T)).cuda()
    dG = torch.zeros((N, ld), dtype=torch.int16, device="cuda")
    dbias = torch.from_numpy(bias).cuda()
    esz = 2
    with tw.Plan.create(K, N, dtype, tiles, W) as plan:
        for t in range(2):
            plan.gemm(dA[t].data_ptr(), dG.data_ptr(), M, lda=ld, ldc=ld, pruned_cols=tw.PRUNED_ZERO,
                      stream=s, bias_ptr=dbias.data_ptr())
            tw.lstm_gates(M, H, dtype, dG.data_ptr(), ld, 1.0, dC.data_ptr(), ld, dC.data_ptr(), ld,
                          dA[t + 1].data_ptr() + I * ld * esz, ld, s)
        torch.cuda.synchronize()
    # oracle: the same recurrence with the 16-bit hand-overs
    q = lambda v: oracle.quantize(np.asarray(v, np.float32), dtype).astype(np.float64)
    h, c = q(h0), c0.astype(np.float64)
    for t in range(2):
        gates = oracle.mask_dense(np.concatenate([q(xs[t]), h], 1), q(W), mask, bias.astype(np.float64))
        c, h = oracle.basic_lstm_cell(q(gates), c, 1.0)
        h = q(h)
    got_h = oracle.bits_to_f32(from_device_bits(dA[2])[I:], dtype).reshape(H, M).T
    got_c = dC.cpu().numpy().T
    assert oracle.rel_error(got_h, h) <= 2 * TOL[dtype]
    assert oracle.rel_error(got_c, c) <= 2 * TOL[dtype]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,G,k_keep", [(128, 128, 0.5), (100, 64, 0.3), (33, 32, 0.6), (1, 128, 0.25)])
def test_fused_step_recurrence(tw, oracle, dtype, M, G, k_keep):
    """tw_lstm_step: gate GEMM, bias and cell in one launch, two time steps in a row with h_t
    written into the next step's A (two A buffers in turn).  Against the oracle's recurrence with
    fp32 pre-activations (the fused kernel never rounds the gate matrix), and against the
    two-kernel form (tw_gemm_ex then tw_lstm_gates), which rounds it to 16 bits in between.
    Ragged M; rows and padding beyond M stay untouched."""
    import torch
    rng = np.random.default_rng(97 + M + G)
    I, H = 160, 256
    K, N = I + H, 4 * H
    W = (rng.standard_normal((K, N)) * 0.08).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.5).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=k_keep, n_keep=1.0, empty_every=7 if G == 32 else 0)
    mask = oracle.plan_mask(K, N, tiles)
    xs = [rng.standard_normal((M, I)).astype(np.float32) for _ in range(2)]
    h0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    c0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    ld = (M + 7) // 8 * 8
    PAD = 0x5a5a
    s = torch.cuda.current_stream().cuda_stream

    def operands():
        A = []
        for t in range(3):
            a = np.full((K, ld), PAD, np.uint16)
            a[:, :M] = 0
            if t < 2:
                a[:I, :M] = oracle.cast_bits(xs[t], dtype).reshape(M, I).T
            A.append(a)
        A[0][I:, :M] = oracle.cast_bits(h0, dtype).reshape(M, H).T
        c = np.full((H, ld), 7.5, np.float32)
        c[:, :M] = c0.T
        return [to_device_bits(a, a.shape) for a in A], torch.from_numpy(c).cuda()

    dbias = torch.from_numpy(bias).cuda()
    with tw.Plan.create(K, N, dtype, tiles, W) as plan:
        dA, dC = operands()
        for t in range(2):
            plan.lstm_step(dA[t].data_ptr(), M, dC.data_ptr(), dC.data_ptr(),
                           dA[t + 1].data_ptr() + I * ld * 2, lda=ld, ldc_prev=ld, ldc_new=ld, ldh=ld,
                           bias_ptr=dbias.data_ptr(), forget_bias=1.0, stream=s)
        torch.cuda.synchronize()
        dA2, dC2 = operands()
        dG = torch.zeros((N, ld), dtype=torch.int16, device="cuda")
        for t in range(2):
            plan.gemm(dA2[t].data_ptr(), dG.data_ptr(), M, lda=ld, ldc=ld, pruned_cols=tw.PRUNED_ZERO,
                      stream=s, bias_ptr=dbias.data_ptr())
            tw.lstm_gates(M, H, dtype, dG.data_ptr(), ld, 1.0, dC2.data_ptr(), ld, dC2.data_ptr(), ld,
                          dA2[t + 1].data_ptr() + I * ld * 2, ld, s)
        torch.cuda.synchronize()
    q = lambda v: oracle.quantize(np.asarray(v, np.float32), dtype).astype(np.float64)
    h, c = q(h0), c0.astype(np.float64)
    for t in range(2):
        gates = oracle.mask_dense(np.concatenate([q(xs[t]), h], 1), q(W), mask, bias.astype(np.float64))
        c, h = oracle.basic_lstm_cell(gates, c, 1.0)
        h = q(h)
    out = from_device_bits(dA[2])
    got_h = oracle.bits_to_f32(np.ascontiguousarray(out[I:, :M]), dtype).reshape(H, M).T
    got_c = dC.cpu().numpy()
    assert oracle.rel_error(got_h, h) <= 2 * TOL[dtype]
    assert oracle.rel_error(got_c[:, :M].T, c) <= 2 * TOL[dtype]
    # nothing beyond M, and the x rows of the last A, were written
    assert np.all(out[:, M:] == PAD) and np.all(out[:I, :M] == 0)
    assert np.all(got_c[:, M:] == 7.5)
    # the two-kernel form rounds the pre-activations to 16 bits (an absolute error of 2^-11 or
    # 2^-8 of a gate's magnitude, which can be most of a small h): close in absolute terms
    two_h = oracle.bits_to_f32(np.ascontiguousarray(from_device_bits(dA2[2])[I:, :M]), dtype).reshape(H, M).T
    bound = {"f16": 5e-3, "bf16": 4e-2}[dtype]      # |h| < 1, |c| of order 1, gates of order 4
    assert np.max(np.abs(got_h - two_h)) <= bound
    assert np.max(np.abs(got_c[:, :M].T - dC2.cpu().numpy()[:, :M].T)) <= bound


def test_fused_step_without_bias_and_fallback(tw, oracle):
    """No bias; and a plan the fused kernel does not take (pruned columns): the call then runs
    tw_gemm_ex + tw_lstm_gates through the caller's gate matrix, and fails without one."""
    import torch
    rng = np.random.default_rng(131)
    M, I, H, G, dtype = 64, 64, 128, 128, "f16"
    K, N = I + H, 4 * H
    W = (rng.standard_normal((K, N)) * 0.08).astype(np.float32)
    x = rng.standard_normal((M, I)).astype(np.float32)
    h0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    c0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    q = lambda v: oracle.quantize(np.asarray(v, np.float32), dtype).astype(np.float64)
    a = np.zeros((K, M), np.uint16)
    a[:I] = oracle.cast_bits(x, dtype).reshape(M, I).T
    a[I:] = oracle.cast_bits(h0, dtype).reshape(M, H).T
    s = torch.cuda.current_stream().cuda_stream
    for n_keep in (1.0, 0.8):
        tiles = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=n_keep)
        mask = oracle.plan_mask(K, N, tiles)
        dA = to_device_bits(a, a.shape)
        dC = torch.from_numpy(np.ascontiguousarray(c0.T)).cuda()
        dH = torch.zeros((H, M), dtype=torch.int16, device="cuda")
        dG = torch.zeros((N, M), dtype=torch.int16, device="cuda")
        with tw.Plan.create(K, N, dtype, tiles, W) as plan:
            if n_keep < 1.0:
                with pytest.raises(tw.TwError) as e:
                    plan.lstm_step(dA.data_ptr(), M, dC.data_ptr(), dC.data_ptr(), dH.data_ptr(), stream=s)
                assert e.value.status == tw.ERR_LAYOUT
            plan.lstm_step(dA.data_ptr(), M, dC.data_ptr(), dC.data_ptr(), dH.data_ptr(),
                           gates_ptr=dG.data_ptr(), stream=s)
            torch.cuda.synchronize()
        gates = oracle.mask_dense(np.concatenate([q(x), q(h0)], 1), q(W), mask, np.zeros(N))
        c, h = oracle.basic_lstm_cell(gates if n_keep == 1.0 else q(gates), c0.astype(np.float64), 1.0)
        got_h = oracle.bits_to_f32(from_device_bits(dH), dtype).reshape(H, M).T
        assert oracle.rel_error(got_h, h) <= 2 * TOL[dtype]
        assert oracle.rel_error(dC.cpu().numpy().T, c) <= 2 * TOL[dtype]
        # the fused path leaves the caller's gate matrix alone
        assert (int(dG.abs().max()) == 0) == (n_keep == 1.0)


def test_fused_step_limits(tw, oracle):
    """H = 1024 is the widest cell the fused kernel takes (bf16, ragged M); H = 1056 needs the
    caller's gate matrix.  Both against the oracle."""
    import torch
    rng = np.random.default_rng(137)
    s = torch.cuda.current_stream().cuda_stream
    for H, G, dtype in ((1024, 128, "bf16"), (1056, 96, "f16")):
        M, I = 40, 32
        K, N = I + H, 4 * H
        W = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
        bias = (rng.standard_normal(N) * 0.3).astype(np.float32)
        tiles = random_tiles(rng, K, N, G, k_keep=0.3, n_keep=1.0)
        mask = oracle.plan_mask(K, N, tiles)
        xh = (rng.standard_normal((M, K)) * 0.7).astype(np.float32)
        c0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
        q = lambda v: oracle.quantize(np.asarray(v, np.float32), dtype).astype(np.float64)
        a = np.zeros((K, M), np.uint16)
        a[:] = oracle.cast_bits(xh, dtype).reshape(M, K).T
        dA = to_device_bits(a, a.shape)
        dC = torch.from_numpy(np.ascontiguousarray(c0.T)).cuda()
        dH = torch.zeros((H, M), dtype=torch.int16, device="cuda")
        dG = torch.zeros((N, M), dtype=torch.int16, device="cuda")
        dbias = torch.from_numpy(bias).cuda()
        with tw.Plan.create(K, N, dtype, tiles, W) as plan:
            if H > 1024:
                with pytest.raises(tw.TwError) as e:
                    plan.lstm_step(dA.data_ptr(), M, dC.data_ptr(), dC.data_ptr(), dH.data_ptr(),
                                   bias_ptr=dbias.data_ptr(), stream=s)
                assert e.value.status == tw.ERR_LAYOUT
            plan.lstm_step(dA.data_ptr(), M, dC.data_ptr(), dC.data_ptr(), dH.data_ptr(),
                           bias_ptr=dbias.data_ptr(), gates_ptr=dG.data_ptr(), stream=s)
            torch.cuda.synchronize()
        assert (int(dG.abs().max()) == 0) == (H <= 1024)
        gates = oracle.mask_dense(q(xh), q(W), mask, bias.astype(np.float64))
        c, h = oracle.basic_lstm_cell(gates if H <= 1024 else q(gates), c0.astype(np.float64), 1.0)
        got_h = oracle.bits_to_f32(from_device_bits(dH), dtype).reshape(H, M).T
        assert oracle.rel_error(got_h, h) <= 2 * TOL[dtype]
        assert oracle.rel_error(dC.cpu().numpy().T, c) <= 2 * TOL[dtype]


def _sequence_problem(rng, oracle, M, I, H, G, k_keep, T, dtype, ld, pad_bits=0x5a5a):
    """x_0 .. x_(T-1), h_(-1), c_(-1) and the T + 1 K-major matrices A_t the engine takes."""
    K, N = I + H, 4 * H
    W = (rng.standard_normal((K, N)) * 0.08).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.5).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=k_keep, n_keep=1.0)
    xs = [rng.standard_normal((M, I)).astype(np.float32) for _ in range(T)]
    h0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    c0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    A = np.full((T + 1, K, ld), pad_bits, np.uint16)
    A[:, :, :M] = 0
    for t in range(T):
        A[t, :I, :M] = oracle.cast_bits(xs[t], dtype).reshape(M, I).T
    A[0, I:, :M] = oracle.cast_bits(h0, dtype).reshape(M, H).T
    c = np.full((H, ld), 7.5, np.float32)
    c[:, :M] = c0.T
    return W, bias, tiles, xs, h0, c0, A, c


def _oracle_recurrence(oracle, W, bias, tiles, xs, h0, c0, dtype):
    """The oracle's cell on the oracle's gate GEMM, step after step, h rounded to 16 bits between
    the steps as the engine hands it over; returns every h_t and the last c."""
    q = lambda v: oracle.quantize(np.asarray(v, np.float32), dtype).astype(np.float64)
    mask = oracle.plan_mask(W.shape[0], W.shape[1], tiles)
    h, c, hs = q(h0), c0.astype(np.float64), []
    for x in xs:
        gates = oracle.mask_dense(np.concatenate([q(x), h], 1), q(W), mask, bias.astype(np.float64))
        c, h = oracle.basic_lstm_cell(gates, c, 1.0)
        h = q(h)
        hs.append(h)
    return hs, c


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,I,H,G,k_keep,T", [(128, 160, 256, 128, 0.5, 6), (100, 96, 128, 64, 0.3, 5),
                                              (33, 40, 64, 32, 0.6, 9), (1, 64, 256, 128, 0.25, 3),
                                              (200, 64, 1024, 128, 0.25, 3),    # 224 workgroups
                                              (120, 1024, 1024, 128, 0.25, 4)])  # the NMT cell
def test_multi_step_launch(tw, oracle, dtype, M, I, H, G, k_keep, T):
    """tw_lstm_steps: T time steps in one persistent launch (weights, row numbers and the cell state
    stay in registers; the rows of h are handed from step to step through memory).  Every h_t and the final c
    against the oracle's recurrence (2 x the GEMM tolerance: errors of h feed the next step), within
    the same bound of T calls of tw_lstm_step, the same bits on a second launch, nothing written beyond
    M or into the rows of x, and a clean status."""
    import torch
    rng = np.random.default_rng(1000 + M + H + T)
    K = I + H
    ld = (M + 7) // 8 * 8
    W, bias, tiles, xs, h0, c0, A, c = _sequence_problem(rng, oracle, M, I, H, G, k_keep, T, dtype, ld)
    want_h, want_c = _oracle_recurrence(oracle, W, bias, tiles, xs, h0, c0, dtype)
    dbias = torch.from_numpy(bias).cuda()
    s = torch.cuda.current_stream().cuda_stream
    outs = []
    with tw.Plan.create(K, 4 * H, dtype, tiles, W) as plan:
        for mode in ("steps", "steps", "single", "reuse"):
            dA = to_device_bits(A, A.shape)
            dC = torch.from_numpy(c.copy()).cuda()
            print("multi-step launch:", mode, M, I, H, G, T, dtype, flush=True)
            if mode == "reuse":
                # the same buffers once more after a launch from another cell state: nothing of that
                # launch's h may be read again (its rows of h linger in the caches)
                dC.add_(0.75)
                plan.lstm_steps(T, dA.data_ptr(), M, dC.data_ptr(), lda=ld, a_step=K * ld, ldc=ld,
                                bias_ptr=dbias.data_ptr(), stream=s)
                dA.copy_(to_device_bits(A, A.shape))
                dC.copy_(torch.from_numpy(c.copy()).cuda())
            if mode in ("steps", "reuse"):
                plan.lstm_steps(T, dA.data_ptr(), M, dC.data_ptr(), lda=ld, a_step=K * ld, ldc=ld,
                                bias_ptr=dbias.data_ptr(), stream=s)
                plan.lstm_steps_status(s)          # waits; raises if a wave gave up
            else:
                for t in range(T):
                    plan.lstm_step(dA[t].data_ptr(), M, dC.data_ptr(), dC.data_ptr(),
                                   dA[t + 1].data_ptr() + I * ld * 2, lda=ld, ldc_prev=ld, ldc_new=ld, ldh=ld,
                                   bias_ptr=dbias.data_ptr(), stream=s)
                torch.cuda.synchronize()
            outs.append((from_device_bits(dA).copy(), dC.cpu().numpy().copy()))
    a_bits, c_out = outs[0]
    for t in range(T):
        got = oracle.bits_to_f32(np.ascontiguousarray(a_bits[t + 1, I:, :M]), dtype).reshape(H, M).T
        assert oracle.rel_error(got, want_h[t]) <= 2 * TOL[dtype], t
    assert oracle.rel_error(c_out[:, :M].T, want_c) <= 2 * TOL[dtype]
    # rows of x, and everything beyond M, are as the caller left them
    assert np.array_equal(a_bits[:, :I, :], A[:, :I, :]) and np.all(a_bits[:, :, M:] == 0x5a5a)
    assert np.all(c_out[:, M:] == 7.5)
    # a second launch gives the same bits; the T single launches differ from it in last bits only
    # (the two kernels' cell arithmetic is contracted into fused multiply-adds differently, and a
    # last-bit difference of h_t then feeds every later step)
    assert np.array_equal(a_bits, outs[1][0]) and np.array_equal(c_out, outs[1][1])
    assert np.array_equal(a_bits, outs[3][0]) and np.array_equal(c_out, outs[3][1])
    single_h = oracle.bits_to_f32(np.ascontiguousarray(outs[2][0][1:, I:, :M]), dtype)
    steps_h = oracle.bits_to_f32(np.ascontiguousarray(a_bits[1:, I:, :M]), dtype)
    assert oracle.rel_error(steps_h, single_h) <= 2 * TOL[dtype]
    assert oracle.rel_error(c_out[:, :M], outs[2][1][:, :M]) <= 2 * TOL[dtype]
    assert np.array_equal(outs[2][0][:, :I, :], A[:, :I, :])


def test_multi_step_launch_in_a_graph(tw, oracle):
    """tw_lstm_steps records into a HIP graph (its fill of the rows of h is a kernel, not a memset):
    the graph is replayed four times on inputs restored in between, with eager launches of the same
    plan between the replays, and every replay gives the eager call's bits."""
    import torch
    rng = np.random.default_rng(77)
    M, I, H, G, T, dtype = 96, 128, 256, 128, 5, "bf16"
    K, ld = I + H, 96
    W, bias, tiles, xs, h0, c0, A, c = _sequence_problem(rng, oracle, M, I, H, G, 0.4, T, dtype, ld)
    dbias = torch.from_numpy(bias).cuda()
    s = torch.cuda.Stream()
    with tw.Plan.create(K, 4 * H, dtype, tiles, W) as plan:
        with torch.cuda.stream(s):
            A0, C0 = to_device_bits(A, A.shape), torch.from_numpy(c.copy()).cuda()
            dA, dC = A0.clone(), C0.clone()
            other_a, other_c = A0.clone(), C0.clone()

            def steps(a, cc):
                plan.lstm_steps(T, a.data_ptr(), M, cc.data_ptr(), lda=ld, a_step=K * ld, ldc=ld,
                                bias_ptr=dbias.data_ptr(), stream=s.cuda_stream)
            print("multi-step launch, eager then in a graph", flush=True)
            steps(dA, dC)
            plan.lstm_steps_status(s.cuda_stream)
            want_a, want_c = dA.clone(), dC.clone()
            dA.copy_(A0)
            dC.copy_(C0)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=s):
                steps(dA, dC)
            for rep in range(4):
                dA.copy_(A0)
                dC.copy_(C0)
                other_c.copy_(C0 + rep)              # eager work of the same plan between the replays
                steps(other_a, other_c)
                s.synchronize()
                g.replay()
                plan.lstm_steps_status(s.cuda_stream)
                assert torch.equal(dA, want_a) and torch.equal(dC, want_c), rep
    want_h, want_cc = _oracle_recurrence(oracle, W, bias, tiles, xs, h0, c0, dtype)
    got = oracle.bits_to_f32(np.ascontiguousarray(from_device_bits(want_a)[T, I:, :M]), dtype).reshape(H, M).T
    assert oracle.rel_error(got, want_h[-1]) <= 2 * TOL[dtype]


def test_multi_step_launch_without_the_first_look(tw, oracle):
    """TW_OPT_LSTM_LOOK = 0: the waves fetch a step's rows of h at once and again until none shows
    the fill pattern (the path a wave otherwise takes only for a line that was fetched too early).
    Same bits as the default form."""
    import torch
    rng = np.random.default_rng(78)
    M, I, H, G, T, dtype = 120, 192, 512, 128, 6, "f16"
    K, ld = I + H, 120
    W, bias, tiles, xs, h0, c0, A, c = _sequence_problem(rng, oracle, M, I, H, G, 0.3, T, dtype, ld)
    dbias = torch.from_numpy(bias).cuda()
    s = torch.cuda.current_stream().cuda_stream
    outs = []
    with tw.Plan.create(K, 4 * H, dtype, tiles, W) as plan:
        try:
            for look in (-1, 0, 0):
                tw.set_option(tw.OPT_LSTM_LOOK, look)
                dA = to_device_bits(A, A.shape)
                dC = torch.from_numpy(c.copy()).cuda()
                print("multi-step launch, first look", look, flush=True)
                plan.lstm_steps(T, dA.data_ptr(), M, dC.data_ptr(), lda=ld, a_step=K * ld, ldc=ld,
                                bias_ptr=dbias.data_ptr(), stream=s)
                plan.lstm_steps_status(s)
                outs.append((from_device_bits(dA).copy(), dC.cpu().numpy().copy()))
        finally:
            tw.set_option(tw.OPT_LSTM_LOOK, -1)
    for a_bits, c_out in outs[1:]:
        assert np.array_equal(a_bits, outs[0][0]) and np.array_equal(c_out, outs[0][1])
    want_h, want_c = _oracle_recurrence(oracle, W, bias, tiles, xs, h0, c0, dtype)
    got = oracle.bits_to_f32(np.ascontiguousarray(outs[0][0][T, I:, :M]), dtype).reshape(H, M).T
    assert oracle.rel_error(got, want_h[-1]) <= 2 * TOL[dtype]


def test_multi_step_launch_gives_up_cleanly(tw, oracle):
    """The loads a wave spends looking for a step's h are bounded.  With none allowed at all every
    wave that needs rows of h gives up at the second step; every workgroup then leaves normally,
    the call after it reports TW_ERR_DEVICE once, and the plan works again afterwards."""
    import torch
    rng = np.random.default_rng(5)
    M, I, H, G, T, dtype = 128, 64, 256, 128, 4, "f16"
    K, ld = I + H, 128
    W, bias, tiles, xs, h0, c0, A, c = _sequence_problem(rng, oracle, M, I, H, G, 0.4, T, dtype, ld)
    s = torch.cuda.current_stream().cuda_stream
    with tw.Plan.create(K, 4 * H, dtype, tiles, W) as plan:
        dA = to_device_bits(A, A.shape)
        dC = torch.from_numpy(c.copy()).cuda()
        try:
            tw.set_option(tw.OPT_SPIN_LIMIT, 0)
            print("multi-step launch with no polls", flush=True)
            plan.lstm_steps(T, dA.data_ptr(), M, dC.data_ptr(), lda=ld, a_step=K * ld, ldc=ld, stream=s)
            with pytest.raises(tw.TwError) as e:
                plan.lstm_steps_status(s)
            assert e.value.status == tw.ERR_DEVICE
        finally:
            tw.set_option(tw.OPT_SPIN_LIMIT, -1)
        plan.lstm_steps_status(s)                  # the status was cleared by the report
        dA = to_device_bits(A, A.shape)
        dC = torch.from_numpy(c.copy()).cuda()
        plan.lstm_steps(T, dA.data_ptr(), M, dC.data_ptr(), lda=ld, a_step=K * ld, ldc=ld, stream=s)
        plan.lstm_steps_status(s)
        want_h, want_c = _oracle_recurrence(oracle, W, np.zeros(4 * H, np.float32), tiles, xs, h0, c0, dtype)
        got = oracle.bits_to_f32(np.ascontiguousarray(from_device_bits(dA)[T, I:, :M]), dtype).reshape(H, M).T
        assert oracle.rel_error(got, want_h[-1]) <= 2 * TOL[dtype]


def test_multi_step_launch_falls_back(tw, oracle):
    """A plan the persistent kernel does not take (pruned columns) runs step by step through the
    caller's gate matrix; without one the call fails like tw_lstm_step."""
    import torch
    rng = np.random.default_rng(6)
    M, I, H, G, T, dtype = 64, 64, 128, 128, 3, "f16"
    K, N, ld = I + H, 4 * H, 64
    W = (rng.standard_normal((K, N)) * 0.08).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=0.8)
    xs = [rng.standard_normal((M, I)).astype(np.float32) for _ in range(T)]
    h0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    c0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    A = np.zeros((T + 1, K, ld), np.uint16)
    for t in range(T):
        A[t, :I] = oracle.cast_bits(xs[t], dtype).reshape(M, I).T
    A[0, I:] = oracle.cast_bits(h0, dtype).reshape(M, H).T
    s = torch.cuda.current_stream().cuda_stream
    q = lambda v: oracle.quantize(np.asarray(v, np.float32), dtype).astype(np.float64)
    mask = oracle.plan_mask(K, N, tiles)
    with tw.Plan.create(K, N, dtype, tiles, W) as plan:
        dA = to_device_bits(A, A.shape)
        dC = torch.from_numpy(np.ascontiguousarray(c0.T)).cuda()
        dG = torch.zeros((N, ld), dtype=torch.int16, device="cuda")
        with pytest.raises(tw.TwError) as e:
            plan.lstm_steps(T, dA.data_ptr(), M, dC.data_ptr(), stream=s)
        assert e.value.status == tw.ERR_LAYOUT
        plan.lstm_steps(T, dA.data_ptr(), M, dC.data_ptr(), gates_ptr=dG.data_ptr(), stream=s)
        plan.lstm_steps_status(s)
    h, cc = q(h0), c0.astype(np.float64)
    for x in xs:
        gates = oracle.mask_dense(np.concatenate([q(x), h], 1), q(W), mask, np.zeros(N))
        cc, h = oracle.basic_lstm_cell(q(gates), cc, 1.0)   # the two-kernel form rounds the gate matrix
        h = q(h)
    got = oracle.bits_to_f32(np.ascontiguousarray(from_device_bits(dA)[T, I:]), dtype).reshape(H, M).T
    # (the gate matrix goes through 16 bits here: an absolute error of 2^-11 of a gate's magnitude,
    # which can be most of a small h, so the bound is absolute: |h| < 1, |c| of order 1)
    assert np.max(np.abs(got - h)) <= 1e-2
    assert np.max(np.abs(dC.cpu().numpy().T - cc)) <= 1e-2
