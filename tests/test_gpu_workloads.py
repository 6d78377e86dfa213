"""The five benchmark configurations on the GPU, at full size where memory allows.

At full size the oracle is evaluated on a sample of rows (a row of C depends on the same
row of A only, so C[rows] = A[rows] @ (B (.) mask) is exact for the sample), and
size-independent properties are checked on the whole result: pruned columns untouched,
linearity in A, and agreement of the two kernel shapes.
"""
import numpy as np
import pytest

from tests.helpers import from_device_bits

pytestmark = pytest.mark.gpu

TOL = {"f16": 1e-2, "bf16": 2e-2}


def run(tw, wl, A_dev, M, plan, alpha=1.0):
    import torch
    C = torch.full((wl["N"], M), 0x1234, dtype=torch.int16, device="cuda")
    plan.gemm(A_dev.data_ptr(), C.data_ptr(), M, alpha=alpha,
              stream=torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return C


def check_workload(tw, oracle, wl, sample_rows=96):
    import torch
    M, K, N, dtype, tiles = wl["M"], wl["K"], wl["N"], wl["dtype"], wl["tiles"]
    A, B = wl["values"]()
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    At = torch.from_numpy(A).cuda().to(tdt).t().contiguous()
    keep = np.zeros(N, bool)
    for t in tiles:
        keep[np.asarray(t["kept_n"], np.int64) + t["col0"]] = True
    rng = np.random.default_rng(wl["seed"])
    rows = np.sort(rng.choice(M, size=min(sample_rows, M), replace=False))
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        C = run(tw, wl, At, M, plan)
        bits = from_device_bits(C)
        got = oracle.bits_to_f32(np.ascontiguousarray(bits[:, rows]), dtype).reshape(N, rows.size).T
        Aq = oracle.bits_to_f32(from_device_bits(At.view(torch.int16)[:, rows].contiguous()), dtype)
        ref = oracle.tw_gemm_reference(Aq.reshape(K, rows.size).T, oracle.quantize(B, dtype), tiles)
        err = oracle.rel_error(got[:, keep], ref[:, keep])
        assert err <= TOL[dtype], (wl["name"], err)
        assert np.all(bits[~keep] == 0x1234), "pruned columns were written"
        # linearity: tw_gemm(2A) == 2 tw_gemm(A) exactly (scaling by 2 is exact in fp16/bf16)
        C2 = run(tw, wl, At * 2, M, plan)
        a = oracle.bits_to_f32(from_device_bits(C)[keep][:, :4096].copy(), dtype)
        b = oracle.bits_to_f32(from_device_bits(C2)[keep][:, :4096].copy(), dtype)
        fin = np.isfinite(b) & (np.abs(a) > 1e-3)
        assert np.array_equal((2 * a)[fin], b[fin])
    return err


def test_config1_bert_base_ffn(tw, oracle):
    from tilesparsity_amd import workloads as W
    check_workload(tw, oracle, W.bert_base_ffn())


def test_config1_row_major_operands(tw, oracle):
    """Config 1 with the operands of the reference's Python operator: x[M,K] and the result
    [M,N] row-major, bias in the epilogue, pruned columns receive the bias (mask_dense,
    Pruning/BERT/utils/modeling.py:992-1007).  At full size, through tw_gemm_staged (which hands
    operands a GEMM kernel takes as they are straight on: K = 768 fits the A-stationary kernel's
    panel) and with A alone row-major (staged): sampled rows against the oracle, and the whole
    result bit for bit against the K-major launch."""
    import torch
    from tilesparsity_amd import workloads as W
    wl = W.bert_base_ffn()
    M, K, N, dtype, tiles = wl["M"], wl["K"], wl["N"], wl["dtype"], wl["tiles"]
    A, B = wl["values"]()
    rng = np.random.default_rng(wl["seed"])
    bias = rng.standard_normal(N).astype(np.float32)
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    Ar = torch.from_numpy(A).cuda().to(tdt).contiguous()
    At = Ar.t().contiguous()
    dbias = torch.from_numpy(bias).cuda()
    Cr = torch.full((M, N), 0x1234, dtype=torch.int16, device="cuda")
    Ck = torch.full((N, M), 0x1234, dtype=torch.int16, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        nbytes = plan.staged_workspace(M, tw.ROWMAJOR, tw.ROWMAJOR)
        ws = torch.empty((nbytes,), dtype=torch.uint8, device="cuda")
        plan.gemm(Ar.data_ptr(), Cr.data_ptr(), M, lda=K, ldc=N, a_layout=tw.ROWMAJOR,
                  c_layout=tw.ROWMAJOR, pruned_cols=tw.PRUNED_ZERO, bias_ptr=dbias.data_ptr(),
                  stream=s, workspace_ptr=ws.data_ptr(), workspace_bytes=nbytes)
        plan.gemm(At.data_ptr(), Ck.data_ptr(), M, pruned_cols=tw.PRUNED_ZERO,
                  bias_ptr=dbias.data_ptr(), stream=s)
        torch.cuda.synchronize()
        Ck2 = torch.full((N, M), 0x1234, dtype=torch.int16, device="cuda")
        plan.gemm(Ar.data_ptr(), Ck2.data_ptr(), M, lda=K, a_layout=tw.ROWMAJOR, pruned_cols=tw.PRUNED_ZERO,
                  bias_ptr=dbias.data_ptr(), stream=s, workspace_ptr=ws.data_ptr(), workspace_bytes=nbytes)
        torch.cuda.synchronize()
    assert torch.equal(Cr, Ck.t())
    assert torch.equal(Ck2, Ck)
    rows = np.sort(rng.choice(M, size=96, replace=False))
    got = oracle.bits_to_f32(from_device_bits(Cr[torch.from_numpy(rows).cuda()].contiguous()), dtype)
    mask = oracle.plan_mask(K, N, tiles)
    ref = oracle.mask_dense(oracle.quantize(A[rows], dtype), oracle.quantize(B, dtype), mask,
                            bias.astype(np.float64))
    assert oracle.rel_error(got.reshape(rows.size, N), ref) <= TOL[dtype]


def test_config2_vgg16_conv4_2(tw, oracle):
    from tilesparsity_amd import workloads as W
    check_workload(tw, oracle, W.vgg16_conv4_2())


def test_config3_nmt_lstm_gates_50_steps(tw, oracle):
    """Fixed plan, 50 back-to-back steps: every step must reproduce the first bit for bit."""
    import torch
    from tilesparsity_amd import workloads as W
    wl = W.nmt_lstm_gates()
    check_workload(tw, oracle, wl, sample_rows=128)
    A, B = wl["values"]()
    At = torch.from_numpy(A).cuda().half().t().contiguous()
    with tw.Plan.create(wl["K"], wl["N"], "f16", wl["tiles"], B) as plan:
        first = from_device_bits(run(tw, wl, At, wl["M"], plan))
        C = torch.zeros((wl["N"], wl["M"]), dtype=torch.int16, device="cuda")
        for _ in range(50):
            plan.gemm(At.data_ptr(), C.data_ptr(), wl["M"],
                      stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert np.array_equal(from_device_bits(C), first)


def test_config3_fused_time_steps(tw, oracle):
    """The NMT configuration at full size through tw_lstm_step: three time steps of the fused
    launch (gate GEMM, bias, cell) against the oracle's recurrence, with h handed on in fp16
    through the rows of the next step's A; and the same launches once more, bit for bit."""
    import torch
    from tilesparsity_amd import workloads as W
    wl = W.nmt_lstm_gates()
    M, K, N = wl["M"], wl["K"], wl["N"]
    H = N // 4
    I = K - H
    A, B = wl["values"]()
    rng = np.random.default_rng(5)
    bias = (rng.standard_normal(N) * 0.3).astype(np.float32)
    c0 = (rng.standard_normal((M, H)) * 0.5).astype(np.float32)
    mask = oracle.plan_mask(K, N, wl["tiles"])
    q = lambda v: oracle.quantize(np.asarray(v, np.float32), "f16").astype(np.float64)
    s = torch.cuda.current_stream().cuda_stream
    dbias = torch.from_numpy(bias).cuda()
    At = torch.from_numpy(A).cuda().half().t().contiguous()        # [K, M]: x rows, then h rows
    with tw.Plan.create(K, N, "f16", wl["tiles"], B) as plan:
        runs = []
        for rep in range(2):
            bufs = [At.clone(), At.clone()]
            cell = torch.from_numpy(np.ascontiguousarray(c0.T)).cuda()
            for t in range(3):
                a, a_next = bufs[t % 2], bufs[(t + 1) % 2]
                plan.lstm_step(a.data_ptr(), M, cell.data_ptr(), cell.data_ptr(),
                               a_next.data_ptr() + I * M * 2, bias_ptr=dbias.data_ptr(), stream=s)
            torch.cuda.synchronize()
            runs.append((bufs[1][I:].clone(), cell.clone()))
        assert torch.equal(runs[0][0], runs[1][0]) and torch.equal(runs[0][1], runs[1][1])
    x = q(A[:, :I])
    h, c = q(A[:, I:]), c0.astype(np.float64)
    for t in range(3):
        gates = oracle.mask_dense(np.concatenate([x, h], 1), q(B), mask, bias.astype(np.float64))
        c, h = oracle.basic_lstm_cell(gates, c, 1.0)
        h = q(h)
    got_h = runs[0][0].float().cpu().numpy().T
    got_c = runs[0][1].cpu().numpy().T
    assert oracle.rel_error(got_h, h) <= 2e-2
    assert oracle.rel_error(got_c, c) <= 2e-2


@pytest.mark.parametrize("which,keep", [(1, 0.5), (1, 0.25), (1, 0.10), (2, 0.5), (2, 0.25), (2, 0.10)])
def test_config4_bert_large_ffn_bf16(tw, oracle, which, keep):
    from tilesparsity_amd import workloads as W
    wl = W.bert_large_ffn(which, keep)
    K = wl["K"]
    assert all(len(t["kept_k"]) == int(np.floor(keep * K + 0.5)) for t in wl["tiles"])
    check_workload(tw, oracle, wl)


def test_config5_imbalance_stress(tw, oracle):
    from tilesparsity_amd import workloads as W
    wl = W.imbalance_stress()
    kts = [len(t["kept_k"]) for t in wl["tiles"]]
    assert kts.count(0) >= 13 and max(kts) > 2500      # empty tiles and near-dense tiles
    check_workload(tw, oracle, wl)


@pytest.mark.parametrize("name", ["vgg16_conv4_2", "bert_large_ffn2_75", "bert_large_ffn1_50"])
def test_direct_loads_repeat_under_back_to_back_launches(tw, name):
    """The 256 x 128 kernel with loads that write LDS directly relies on exact counts of the loads
    in flight.  At full size, with launches queued back to back (a launch then starts while the
    memory system is still busy with its predecessor's stores, which is when a count that is one
    too generous shows), every launch gives the bits of the register-staged form of the kernel:
    one item per workgroup (VGG16 conv4_2, BERT-large FFN2) and four chained items with deferred
    stores (BERT-large FFN1)."""
    import torch
    from tilesparsity_amd import workloads
    wl = {"vgg16_conv4_2": workloads.vgg16_conv4_2, "bert_large_ffn2_75": lambda: workloads.bert_large_ffn(2, 0.25),
          "bert_large_ffn1_50": lambda: workloads.bert_large_ffn(1, 0.50)}[name]()
    M, K, N, dtype, tiles = wl["M"], wl["K"], wl["N"], wl["dtype"], wl["tiles"]
    A, B = wl["values"]()
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    At = torch.from_numpy(A).cuda().to(tdt).t().contiguous()
    s = torch.cuda.current_stream().cuda_stream
    try:
        tw.set_option(tw.OPT_SHAPE, tw.SHAPE_256x128)
        with tw.Plan.create(K, N, dtype, tiles, B) as plan:
            tw.set_option(tw.OPT_LDS_DMA, 0)
            want = torch.zeros((N, M), dtype=torch.int16, device="cuda")
            plan.gemm(At.data_ptr(), want.data_ptr(), M, stream=s)
            torch.cuda.synchronize()
            tw.set_option(tw.OPT_LDS_DMA, 1)
            outs = [torch.zeros((N, M), dtype=torch.int16, device="cuda") for _ in range(3)]
            for rep in range(8):
                print("direct loads, back to back:", name, rep, flush=True)
                for c in outs:
                    c.zero_()
                for i in range(9):
                    plan.gemm(At.data_ptr(), outs[i % 3].data_ptr(), M, stream=s)
                torch.cuda.synchronize()
                for c in outs:
                    assert torch.equal(c, want), (name, rep)
    finally:
        tw.set_option(tw.OPT_SHAPE, -1)
        tw.set_option(tw.OPT_LDS_DMA, -1)


def test_cpp_driver_reference_command_line():
    """The C++ perf driver with the reference's command line (`./test_basic_nn M N K N_kept K_kept`,
    StreamMaskedGEMM/README.md:12-13) at a reduced M: its three self-checks (fused == gather /
    dense / scatter bit for bit, fused vs a host fp32 product, dense baseline vs fused) pass."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                       "tilesparsity_amd", "test_basic_nn")
    assert os.path.exists(exe), "build the driver with `python -m tilesparsity_amd.build`"
    for args in (["1280", "768", "768", "384", "384"], ["520", "768", "3072", "384", "1536"]):
        print("driver", args, flush=True)
        res = subprocess.run([exe] + args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                             timeout=100)
        assert res.returncode == 0, res.stdout[-2000:]
        assert res.stdout.count("PASSED !!!") == 3 and "FAILED" not in res.stdout, res.stdout[-2000:]
        assert "Stream  GEMM :" in res.stdout and "Dense   GEMM :" in res.stdout
