#!/usr/bin/env python3
"""Benchmark of the tile-wise-sparse GEMM engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--headline-only]

A step is one TW GEMM  C = A * (B (.) mask)  over one batch of synthetic input that
is already resident in HBM.  The default workload is VGG16 conv4_2 as an im2col GEMM
(M=12544, K=4608, N=512, G=128, 75 % tile-wise sparsity, fp16 in / fp32 accumulate).
Prints ONE JSON line: effective TFLOP/s (dense flops / time), with the speedup over the
same kernel on the 0 %-sparse plan, the roofline of the kernel and the CPU baseline
(NumPy masked dense matmul, the reference's CPU path) timed on this box's host cores.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense fp16 / bf16

# HBM bytes per sparse launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per
# dispatch), each scaled by what the same counter reads for a 256 MiB copy in the same run
# (reads x 2.0, writes x 1.0).  Constants copied from the profile named beside them, not read in
# this run: `traffic_source` in the line says which file, and for which kernel, they stand.
# Keyed by the workload's own name.
PREWARM_SECONDS = 0.03  # untimed launches before a configuration's warm-up steps (clock ramp-up)

MEASURED_TRAFFIC = {
    "vgg16_conv4_2_im2col": ((2 * 62014 + 11282) * 1024, "profiles/tw_gemm_ws_kernel__vgg16_conv4_2.md (tw_gemm_ws_kernel 256x128)"),
    "bert_base_ffn_in": ((2 * 7897 + 24576) * 1024, "profiles/tw_gemm_as_kernel__bert_base_ffn.md (tw_gemm_as_kernel 64 rows)"),
    "nmt_lstm_gates": ((2 * 3558.5 + 1024) * 1024, "profiles/tw_gemm_skinny_kernel__nmt_lstm_gates.md (tw_gemm_skinny_kernel)"),
    "imbalance_stress": ((2 * 922921 + 209150) * 1024, "profiles/tw_gemm_ws_kernel__imbalance_stress.md (tw_gemm_ws_kernel 256x64)"),
    "bert_large_ffn1_keep50": ((2 * 25220 + 65570) * 1024, "profiles/tw_gemm_ws_kernel__bert_large_ffn1_50.md (tw_gemm_ws_kernel 256x128)"),
    "bert_large_ffn2_keep10": ((2 * 22280 + 16400) * 1024, "profiles/tw_gemm_ws_kernel__bert_large_ffn2.md (tw_gemm_ws_kernel 256x128)"),
    "bert_large_ffn2_keep50": ((2 * 49480 + 16400) * 1024, "profiles/tw_gemm_ws_kernel__bert_large_ffn2.md (tw_gemm_ws_kernel 256x128)"),
    "bert_large_ffn1_keep25": ((2 * 16649 + 65536) * 1024, "profiles/tw_gemm_as_kernel__bert_large_ffn1.md (tw_gemm_as_kernel 64 rows)"),
    "bert_large_ffn1_keep10": ((2 * 12319 + 65536) * 1024, "profiles/tw_gemm_bs_kernel__bert_large_ffn1_90.md (tw_gemm_bs_kernel)"),
    "bert_large_ffn2_keep25": ((2 * 38160 + 16400) * 1024, "profiles/tw_gemm_ws_kernel__bert_large_ffn2.md (tw_gemm_ws_kernel 256x128)"),
}


def make_workload(name):
    from tilesparsity_amd import workloads as W
    table = {
        "vgg16_conv4_2": W.vgg16_conv4_2,
        "bert_base_ffn": W.bert_base_ffn,
        "nmt_lstm_gates": W.nmt_lstm_gates,
        "bert_large_ffn1_50": lambda: W.bert_large_ffn(1, 0.50),
        "bert_large_ffn1_75": lambda: W.bert_large_ffn(1, 0.25),
        "bert_large_ffn1_90": lambda: W.bert_large_ffn(1, 0.10),
        "bert_large_ffn2_50": lambda: W.bert_large_ffn(2, 0.50),
        "bert_large_ffn2_75": lambda: W.bert_large_ffn(2, 0.25),
        "bert_large_ffn2_90": lambda: W.bert_large_ffn(2, 0.10),
        "imbalance_stress": W.imbalance_stress,
    }
    return table[name]()


def time_steps(launch, steps, warmup, torch):
    """Average seconds per step over exactly `steps` back-to-back calls of launch(i), timed with
    events on the stream the kernels run on, after `warmup` untimed calls."""
    stream = torch.cuda.current_stream()
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(stream)
    for i in range(steps):
        launch(i)
    stop.record(stream)
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / steps


def time_plan(plan, bufs, M, steps, warmup, torch):
    """Seconds per launch of a plan; buffers rotate so that A and C come from HBM."""
    s = torch.cuda.current_stream().cuda_stream
    n = len(bufs)

    def launch(i):
        a, c = bufs[i % n]
        plan.gemm(a.data_ptr(), c.data_ptr(), M, stream=s)
    return time_steps(launch, steps, warmup, torch)


def time_plan_streams(plan, bufs, M, steps, warmup, torch, n_streams=2):
    """Seconds per launch when the launches, which do not depend on each other (each has its own
    A and C), are issued on `n_streams` streams in turn, as the reference issues its per-tile
    GEMMs on streams of their own (Stream_Gemm_NN, basic_nn.cu:396-430): the last workgroups of
    one launch then run next to the first of the next.  Throughput of independent launches, not
    the duration of one: the headline figure and the roofline stay with the single stream."""
    main = torch.cuda.current_stream()
    streams = [torch.cuda.Stream() for _ in range(n_streams)]
    n = len(bufs)

    def run(count):
        for i in range(count):
            a, c = bufs[i % n]
            plan.gemm(a.data_ptr(), c.data_ptr(), M, stream=streams[i % n_streams].cuda_stream)
    run(warmup)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(main)
    for st in streams:
        st.wait_event(start)
    run(steps)
    for st in streams:
        main.wait_stream(st)
    stop.record(main)
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / steps


def time_plan_graph(plan, bufs, M, steps, warmup, torch):
    """The same with the `steps` launches recorded once into a HIP graph and the graph replayed:
    for launches of a few microseconds, which the host cannot issue as fast as the GPU runs them
    (the NMT recurrence: 50 time steps back to back with fixed weights)."""
    n = len(bufs)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            s = torch.cuda.current_stream().cuda_stream
            for i in range(steps):
                a, c = bufs[i % n]
                plan.gemm(a.data_ptr(), c.data_ptr(), M, stream=s)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream()
    for _ in range(max(1, warmup // max(1, steps) + 1)):
        graph.replay()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(stream)
    graph.replay()          # exactly `steps` launches
    stop.record(stream)
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / steps


def time_row_major(wl, steps, warmup, torch):
    """The operands of the reference's Python operator: x[M,K] and the result [M,N] row-major,
    pruned columns filled.  Seconds per launch of tw_gemm_ex on them as they are (for a K that
    fits a panel of A in LDS the A-stationary kernel takes them directly) and, for scale, of
    tw_gemm_staged with the result K-major (A alone goes through its K-major copy)."""
    from tilesparsity_amd import twgemm as tw
    M, K, N, dtype = wl["M"], wl["K"], wl["N"], wl["dtype"]
    A, B = wl["values"]()
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    Ar = torch.from_numpy(A).cuda().to(tdt).contiguous()
    Cr = torch.zeros((M, N), dtype=tdt, device="cuda")
    plan = tw.Plan.create(K, N, dtype, wl["tiles"], B)
    nbytes = plan.staged_workspace(M, tw.ROWMAJOR, tw.ROWMAJOR)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    kw = dict(lda=K, ldc=N, a_layout=tw.ROWMAJOR, c_layout=tw.ROWMAJOR, pruned_cols=tw.PRUNED_ZERO,
              stream=s)
    t_direct = time_steps(lambda i: plan.gemm(Ar.data_ptr(), Cr.data_ptr(), M, **kw), steps, warmup, torch)
    Ck = torch.zeros((N, M), dtype=tdt, device="cuda")
    kw.update(c_layout=tw.KMAJOR, ldc=M)
    t_a_staged = time_steps(lambda i: plan.gemm(Ar.data_ptr(), Ck.data_ptr(), M, workspace_ptr=ws.data_ptr(),
                                                workspace_bytes=nbytes, **kw), steps, warmup, torch)
    plan.destroy()
    return t_direct, t_a_staged


def time_nmt_recurrence(wl, steps, torch):
    """One NMT time step is the masked gate GEMM (bias in its epilogue) followed by the LSTM gate
    arithmetic, which writes h_t into the rows of the next step's A (A_t = [x_t ; h_{t-1}],
    K-major).  `steps` time steps are recorded into a HIP graph and replayed; returns seconds per
    step for the pair, for the gate kernel alone, for the fused step (tw_lstm_step: GEMM, bias
    and cell in one launch), and for all `steps` time steps as one persistent launch
    (tw_lstm_steps, timed with events around the call)."""
    from tilesparsity_amd import twgemm as tw
    M, K, N, dtype = wl["M"], wl["K"], wl["N"], wl["dtype"]
    H = N // 4
    A, B = wl["values"]()
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    At = [torch.from_numpy(A).cuda().to(tdt).t().contiguous() for _ in range(2)]
    gates = torch.zeros((N, M), dtype=tdt, device="cuda")
    cell = torch.zeros((H, M), dtype=torch.float32, device="cuda")
    bias = torch.zeros((N,), dtype=torch.float32, device="cuda")
    plan = tw.Plan.create(K, N, dtype, wl["tiles"], B)
    out = []
    for mode in ("pair", "gates", "fused"):
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                s = torch.cuda.current_stream().cuda_stream
                for i in range(steps):
                    a, a_next = At[i % 2], At[(i + 1) % 2]
                    if mode == "fused":
                        plan.lstm_step(a.data_ptr(), M, cell.data_ptr(), cell.data_ptr(),
                                       a_next.data_ptr() + (K - H) * M * 2, bias_ptr=bias.data_ptr(),
                                       gates_ptr=gates.data_ptr(), stream=s)
                        continue
                    if mode == "pair":
                        plan.gemm(a.data_ptr(), gates.data_ptr(), M, pruned_cols=tw.PRUNED_ZERO,
                                  stream=s, bias_ptr=bias.data_ptr())
                    tw.lstm_gates(M, H, dtype, gates.data_ptr(), M, 1.0, cell.data_ptr(), M,
                                  cell.data_ptr(), M, a_next.data_ptr() + (K - H) * M * 2, M, s)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        stream = torch.cuda.current_stream()
        ts = []
        for _ in range(6):
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(stream)
            graph.replay()
            stop.record(stream)
            torch.cuda.synchronize()
            ts.append(start.elapsed_time(stop) * 1e-3 / steps)
        out.append(float(np.median(ts[1:])))
        del graph
    # the same `steps` time steps as ONE persistent launch (tw_lstm_steps), on steps + 1 matrices A_t
    seq = torch.from_numpy(A).cuda().to(tdt).t().contiguous().unsqueeze(0).repeat(steps + 1, 1, 1).contiguous()
    s = torch.cuda.current_stream().cuda_stream
    ts = []
    for _ in range(7):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(torch.cuda.current_stream())
        plan.lstm_steps(steps, seq.data_ptr(), M, cell.data_ptr(), bias_ptr=bias.data_ptr(), stream=s)
        stop.record(torch.cuda.current_stream())
        plan.lstm_steps_status(s)      # waits, and raises if the launch gave up
        ts.append(start.elapsed_time(stop) * 1e-3 / steps)
    out.append(float(np.median(ts[1:])))
    plan.destroy()
    return out[0], out[1], out[2], out[3]


def roofline_of(M, K, N, tiles, t, traffic=None, traffic_source=None):
    """Roofline block of one launch that took t seconds: the binding roof is the larger of the
    ideal HBM time (algorithmic bytes at 8 TB/s) and the ideal MFMA time (kept flops at the dense
    16-bit peak)."""
    from tilesparsity_amd import workloads as W
    by, fk = W.algorithmic_bytes(M, K, N, tiles), W.flops_kept(M, tiles)
    if by / (HBM_PEAK_GBS * 1e9) >= fk / (MFMA_PEAK_TFLOPS * 1e12):
        ach = by / t / 1e9
        return {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": ach / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": traffic_source,
                "algorithmic_bytes": by}
    ach = fk / t / 1e12
    return {"bound": "mfma", "achieved": ach, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": ach / MFMA_PEAK_TFLOPS, "traffic": traffic, "traffic_source": traffic_source,
            "algorithmic_flops": fk}


def traffic_of(name, kernel):
    """(bytes, source) of the committed counter measurement of a workload, or (None, None) when
    there is none or the launch now runs another kernel than the one that was measured."""
    if name not in MEASURED_TRAFFIC:
        return None, None
    by, src = MEASURED_TRAFFIC[name]
    if "(%s)" % kernel not in src:
        return None, "%s: measured on another kernel than this launch's %s" % (src, kernel)
    return by, src


def run_workload(wl, steps, warmup, torch, rotate_bytes=768 << 20, repeats=5, graph=False,
                 two_streams=False):
    """Times the TW plan (`steps` launches after `warmup`: the headline figure), then `repeats`
    more rounds of the same length each for the TW plan, for the 0 %-sparse plan of the same
    kernel and for the library's dense GEMM (torch.matmul, i.e. hipBLASLt / rocBLAS) on the same
    operands, layout and rotating buffers; the ratios are taken between the medians."""
    from tilesparsity_amd import twgemm as tw
    from tilesparsity_amd import workloads as W
    M, K, N, G, dtype, tiles = wl["M"], wl["K"], wl["N"], wl["G"], wl["dtype"], wl["tiles"]
    A, B = wl["values"]()
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    # K-major operands: A^T [K, M], C^T [N, M]
    At = torch.from_numpy(A).cuda().to(tdt).t().contiguous()
    per_set = (At.numel() + N * M) * 2
    n_sets = max(2, min(8, -(-rotate_bytes // per_set)))
    bufs = [(At if i == 0 else At.clone(), torch.zeros((N, M), dtype=tdt, device="cuda"))
            for i in range(n_sets)]
    sparse = tw.Plan.create(K, N, dtype, tiles, B)
    dense = tw.Plan.dense(K, N, G, dtype, B)
    kernel_sparse, kernel_dense = sparse.choice(M)["name"], dense.choice(M)["name"]
    timer = time_plan_graph if graph else time_plan
    # After an idle stretch (the plans were just built on the host) the GPU's clocks take ~10 ms of
    # work to come back up: the first 100 launches of the headline shape then read 32.0 us instead
    # of 31.0.  So the GPU is kept busy with untimed launches of the plan for PREWARM_SECONDS
    # before the warm-up steps and the timed steps, which measure the steady state.
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < PREWARM_SECONDS:
        timer(sparse, bufs, M, steps, 0, torch)
    t_sparse = timer(sparse, bufs, M, steps, warmup, torch)
    reps_sparse = [timer(sparse, bufs, M, steps, 2, torch) for _ in range(repeats)]
    reps_dense = [timer(dense, bufs, M, steps, 2, torch) for _ in range(repeats)]
    two = None
    if two_streams and not graph:
        two = [float(np.median([time_plan_streams(pl, bufs, M, steps, 2, torch) for _ in range(3)]))
               for pl in (sparse, dense)]
    sparse.destroy()
    dense.destroy()
    # the library's dense GEMM in the same layout: C^T [N, M] = W^T [N, K] . A^T [K, M]
    Wt = torch.from_numpy(np.ascontiguousarray(B.T)).cuda().to(tdt)

    def lib_launch(i):
        a, c = bufs[i % n_sets]
        torch.matmul(Wt, a, out=c)
    reps_lib = [time_steps(lib_launch, steps, 2, torch) for _ in range(repeats)]
    t_sp, t_de, t_lib = (float(np.median(x)) for x in (reps_sparse, reps_dense, reps_lib))
    fk, fd = W.flops_kept(M, tiles), W.flops_dense(M, K, N)
    by = W.algorithmic_bytes(M, K, N, tiles)
    res = dict(
        workload=wl["name"], M=M, K=K, N=N, G=G, dtype=dtype, seed=wl["seed"], n_tiles=len(tiles),
        us_sparse=t_sparse * 1e6, us_sparse_median=t_sp * 1e6, us_dense=t_de * 1e6,
        us_dense_library=t_lib * 1e6, timed_with="hip graph replay" if graph else "stream launches",
        repeats=repeats,
        effective_tflops=fd / t_sparse / 1e12, actual_tflops=fk / t_sparse / 1e12,
        dense_tflops=fd / t_de / 1e12, dense_library_tflops=fd / t_lib / 1e12,
        speedup_vs_dense=t_de / t_sp, speedup_vs_dense_library=t_lib / t_sp,
        mfma_util_kept=fk / t_sparse / 1e12 / MFMA_PEAK_TFLOPS,
        mfma_util_dense_run=fd / t_de / 1e12 / MFMA_PEAK_TFLOPS,
        algorithmic_bytes=by, hbm_gbs=by / t_sparse / 1e9, rotating_buffer_sets=n_sets,
        kept_flops=fk, dense_flops=fd, kernel_sparse=kernel_sparse, kernel_dense_plan=kernel_dense,
        roofline=roofline_of(M, K, N, tiles, t_sparse, *traffic_of(wl["name"], kernel_sparse)))
    if two:
        # independent launches on two streams in turn (throughput, see time_plan_streams)
        res["two_streams"] = dict(us_sparse=two[0] * 1e6, us_dense_plan=two[1] * 1e6,
                                  speedup_vs_dense_plan=two[1] / two[0],
                                  effective_tflops=fd / two[0] / 1e12, hbm_gbs=by / two[0] / 1e9)
    del bufs, At, Wt
    torch.cuda.empty_cache()
    return res, (A, B)


def cpu_baseline(wl, A, B, budget_s=20.0):
    """The reference's CPU path, y = x @ (kernel * mask) in fp32 (mask_dense,
    Pruning/BERT/utils/modeling.py:992-1007), timed with NumPy's BLAS on the host cores."""
    from oracle import tw_oracle
    M, K, N = wl["M"], wl["K"], wl["N"]
    mask = tw_oracle.plan_mask(K, N, wl["tiles"]).astype(np.float32)
    rows = M
    t0 = time.perf_counter()
    tw_oracle.mask_dense(A[:min(M, 256)], B, mask)          # warm-up / probe
    probe = time.perf_counter() - t0
    if probe * (M / min(M, 256)) * 5 > budget_s:             # bound the sample
        rows = max(256, int(M * budget_s / (probe * (M / min(M, 256)) * 5)) // 8 * 8)
    x = np.ascontiguousarray(A[:rows])
    tw_oracle.mask_dense(x, B, mask)
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 10 and (len(times) < 3 or time.perf_counter() < t_end):
        t0 = time.perf_counter()
        tw_oracle.mask_dense(x, B, mask)
        times.append(time.perf_counter() - t0)
    t = float(np.median(times))
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count()
    env_threads = os.environ.get("OMP_NUM_THREADS")
    threads = min(cores, int(env_threads)) if env_threads else cores
    return dict(value=2.0 * rows * K * N / t / 1e12, unit="TFLOP/s (dense flops, fp32)",
                cores=threads, kind="port",
                sample="numpy x @ (kernel*mask), %d of %d rows of the same workload, mask multiply "
                       "inside the timed region, median of %d runs (%.3f s each)"
                       % (rows, M, len(times), t))


def bench_prepass(wl, steps, warmup):
    """The integer pre-pass behind tw_plan_from_mask on the workload's mask: host mask and fp32
    weight in, device plan out (upload, row / column flags, tile-wise check, compaction of the
    kept lists and relative offsets, weight packing and cast).  A step is one plan build; the
    CPU baseline is the oracle's NumPy restatement of the same pre-pass."""
    from tilesparsity_amd import twgemm as tw
    from oracle import tw_oracle
    K, N, G, tiles = wl["K"], wl["N"], wl["G"], wl["tiles"]
    _, B = wl["values"]()
    mask = tw_oracle.plan_mask(K, N, tiles).astype(np.uint8)
    for _ in range(warmup):
        tw.Plan.from_mask(mask, G, wl["dtype"], B).destroy()
    t0 = time.perf_counter()
    for _ in range(steps):
        tw.Plan.from_mask(mask, G, wl["dtype"], B).destroy()
    t = (time.perf_counter() - t0) / steps
    with tw.Plan.from_mask(mask, G, wl["dtype"], B) as plan:
        info = plan.info()
    # the same with the mask and the weight already on the device (as a producer leaves them)
    import torch
    d_mask, d_B = torch.from_numpy(mask).cuda(), torch.from_numpy(np.ascontiguousarray(B, np.float32)).cuda()
    table = [(c, min(G, N - c)) for c in range(0, N, G)]
    for _ in range(warmup):
        tw.Plan.from_device_mask(K, N, d_mask.data_ptr(), table, wl["dtype"], d_B.data_ptr()).destroy()
    t0 = time.perf_counter()
    for _ in range(steps):
        tw.Plan.from_device_mask(K, N, d_mask.data_ptr(), table, wl["dtype"], d_B.data_ptr()).destroy()
    t_dev = (time.perf_counter() - t0) / steps
    # bytes the device must move: the mask is read three times (row flags, column flags, check),
    # the fp32 weight once at the kept positions, the packed 16-bit weight is written once
    by = 3 * K * N + 4 * info["kept_elems"] + info["packed_bytes"]
    t1 = time.perf_counter()
    got = tw_oracle.plan_from_mask(mask, G)
    tw_oracle.cast_bits(tw_oracle.stream_weight(B, got), wl["dtype"])
    t_cpu = time.perf_counter() - t1
    return {
        "metric": "TW pre-pass: plan builds per second, operands resident in HBM "
                  "(mask -> lists -> offsets -> packed weight)",
        "value": 1.0 / t_dev, "unit": "plans/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": t_dev * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": "%s mask %d x %d, G=%d, %d tiles" % (wl["name"], K, N, G, len(tiles))},
        "device_to_plan_ms": t_dev * 1e3, "host_to_plan_ms": t * 1e3, "uploaded_bytes": K * N * 5,
        "roofline": {"bound": "hbm", "achieved": by / t_dev / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": by / t_dev / 1e9 / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes": by},
        "cpu_baseline": {"value": 1.0 / t_cpu, "unit": "plans/s", "cores": 1, "kind": "port",
                         "sample": "NumPy oracle: lists from the mask, compacted weight and cast, "
                                   "one run (%.1f ms)" % (t_cpu * 1e3)},
    }


# VGG16's 13 conv layers as im2col score matrices (H*W*I) x O, plus a 4096 x 4096 dense layer
PRODUCER_LAYERS = [(27, 64), (576, 64), (576, 128), (1152, 128), (1152, 256), (2304, 256),
                   (2304, 256), (2304, 512), (4608, 512), (4608, 512), (4608, 512), (4608, 512),
                   (4608, 512), (4096, 4096)]


def bench_producers(steps, warmup, torch):
    """The TW mask producers (tiled_wise_1d / tiled_wise_2d at 75 % sparsity, G=128) on a
    VGG16-sized list of score matrices resident in HBM; the NumPy oracle is the CPU baseline."""
    import ctypes
    from tilesparsity_amd import twgemm as tw
    from tilesparsity_amd import twprune
    from oracle import tw_prune_oracle as po
    rng = np.random.default_rng(20200615)
    scores = [np.abs(rng.standard_normal(s)).astype(np.float32) for s in PRODUCER_LAYERS]
    elems = sum(k * n for k, n in PRODUCER_LAYERS)
    d = twprune._DeviceLayers(scores)
    L = tw.lib()
    pp = ctypes.POINTER(ctypes.c_void_p)
    i32 = ctypes.c_int32

    def run1d():
        thr = ctypes.c_double()
        tw._check(L.tw_prune_tiled_wise_1d(len(d.shapes), tw._ptr(d.K, i32), tw._ptr(d.N, i32),
                                           ctypes.cast(d.p_scores, pp), 75.0, 0, 128,
                                           ctypes.cast(d.p_masks, pp), ctypes.byref(thr), d.stream))

    def run2d():
        thr = (ctypes.c_double * 2)()
        tw._check(L.tw_prune_tiled_wise_2d(len(d.shapes), tw._ptr(d.K, i32), tw._ptr(d.N, i32),
                                           ctypes.cast(d.p_scores, pp), 75.0, 0, 1, 128,
                                           ctypes.cast(d.p_masks, pp), ctypes.cast(d.p_cols, pp),
                                           thr, d.stream))

    def run1dmix():
        # tiled_wise_1d at 75 + 5 %, then the element-wise remainder (5 %) over all elements
        tw._check(L.tw_prune_tiled_wise_1d(len(d.shapes), tw._ptr(d.K, i32), tw._ptr(d.N, i32),
                                           ctypes.cast(d.p_scores, pp), 80.0, 0, 128,
                                           ctypes.cast(d.p_masks, pp), None, d.stream))
        thr = ctypes.c_double()
        tw._check(L.tw_prune_mix(len(d.shapes), tw._ptr(d.K, i32), tw._ptr(d.N, i32),
                                 ctypes.cast(d.p_scores, pp), ctypes.cast(d.p_masks, pp), 5.0, 0,
                                 ctypes.cast(d.p_masks, pp), ctypes.byref(thr), d.stream))

    out = {}
    # bytes: scores read once per stage, one mask byte written; the mixed producer also writes and
    # reads the 4-byte element scores, reads the TW mask and rewrites it
    for name, fn, passes in (("tiled_wise_1d", run1d, 1), ("tiled_wise_2d", run2d, 2),
                             ("tiled_wise_1d_mix", run1dmix, 4)):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()                      # every call returns with its masks complete
        t = (time.perf_counter() - t0) / steps
        by = elems * (4 * passes + 1)  # scores read once per stage, one mask byte written
        out[name] = dict(ms=t * 1e3, algorithmic_bytes=by, gbs=by / t / 1e9)
    t0 = time.perf_counter()
    po.tiled_wise_1d(scores, 75.0, 128)
    t1 = time.perf_counter()
    po.tiled_wise_2d(scores, 75.0, 128)
    t2 = time.perf_counter()
    one = out["tiled_wise_1d"]
    return {
        "metric": "TW mask producer throughput (tiled_wise_1d, 14 VGG16-sized layers, 75 %, G=128)",
        "value": one["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": one["ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "mask producers, %d layers, %.1f M score elements" % (
            len(PRODUCER_LAYERS), elems / 1e6)},
        "tiled_wise_2d": out["tiled_wise_2d"],
        "tiled_wise_1d_mix": out["tiled_wise_1d_mix"],
        "roofline": {"bound": "hbm", "achieved": one["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": one["gbs"] / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes": one["algorithmic_bytes"]},
        "cpu_baseline": {"value": elems * 5 / (t1 - t0) / 1e9, "unit": "GB/s", "cores": 1,
                         "kind": "port",
                         "sample": "NumPy oracle on the same layers: tiled_wise_1d %.1f ms, "
                                   "tiled_wise_2d %.1f ms (one run each)" % ((t1 - t0) * 1e3,
                                                                             (t2 - t1) * 1e3)},
    }


def bench_shape_grid(torch, Ms=(128, 512, 2048, 8192, 16384), Ks=(512, 1024, 2048, 4096),
                     Ns=(512, 2048, 4096), Gs=(64, 128), keeps=(0.25, 0.5)):
    """The automatic shape choice against every kernel shape forced in turn, on a grid of
    problems (random tiles, kept-K within +-30 % of keep * K, 90 % of the columns kept).  One line
    per problem: the automatic choice's time, the best forced shape and its time, and their
    ratio; a summary line at the end.  A forced shape that cannot take a plan falls back to the
    automatic one, so its time then repeats that."""
    import itertools
    from tilesparsity_amd import twgemm as tw
    rng = np.random.default_rng(7)
    s = torch.cuda.current_stream().cuda_stream
    shapes = [(tw.SHAPE_128x128, -1), (tw.SHAPE_512x64, -1), (tw.SHAPE_128x64, 64), (tw.SHAPE_256x128, -1),
              (tw.SHAPE_128x32, 32), (tw.SHAPE_256x64, -1), (tw.SHAPE_AS64, -1), (tw.SHAPE_AS32, -1)]
    worst, n_all, n_off = 1.0, 0, 0
    for M, K, N, G, keep in itertools.product(Ms, Ks, Ns, Gs, keeps):
        tiles = []
        for c0 in range(0, N, G):
            w = min(G, N - c0)
            kt = int(np.clip(round(K * keep * rng.uniform(0.7, 1.3)), 1, K))
            tiles.append(dict(col0=c0, width=w,
                              kept_k=np.sort(rng.choice(K, kt, replace=False)).astype(np.int32),
                              kept_n=np.sort(rng.choice(w, max(1, round(w * 0.9)), replace=False)).astype(np.int32)))
        B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
        plan = tw.Plan.create(K, N, "f16", tiles, B)
        n_sets = max(2, min(6, (256 << 20) // ((K + N) * M * 2)))
        bufs = [(torch.randn((K, M), device="cuda").half(),
                 torch.zeros((N, M), dtype=torch.float16, device="cuda")) for _ in range(n_sets)]
        steps = 30 if M * K * N < 1 << 34 else 10
        time_plan(plan, bufs, M, 60, 0, torch)        # the first launches of a new plan run slower
        t_auto = min(time_plan(plan, bufs, M, steps, 3, torch) for _ in range(2))
        res = []
        for shape, piece in shapes:
            if shape in ((tw.SHAPE_128x128, tw.SHAPE_256x128) if G == 64 else (tw.SHAPE_512x64, tw.SHAPE_256x64)):
                continue    # 128-column shapes on 64-column tiles and the other way round
            tw.set_option(tw.OPT_SHAPE, shape)
            tw.set_option(tw.OPT_PIECE, piece)
            res.append((min(time_plan(plan, bufs, M, steps, 3, torch) for _ in range(2)), shape))
        tw.set_option(tw.OPT_SHAPE, -1)
        tw.set_option(tw.OPT_PIECE, -1)
        t_auto = min(t_auto, min(time_plan(plan, bufs, M, steps, 3, torch) for _ in range(2)))
        t_best, s_best = min(res)
        n_all += 1
        n_off += t_auto > 1.08 * t_best
        worst = max(worst, t_auto / t_best)
        print("M=%d K=%d N=%d G=%d keep=%.2f: automatic %.1f us, best forced shape %d %.1f us, ratio %.2f" % (
            M, K, N, G, keep, t_auto * 1e6, s_best, t_best * 1e6, t_auto / t_best), flush=True)
        plan.destroy()
        del bufs
        torch.cuda.empty_cache()
    print(json.dumps({"problems": n_all, "automatic_more_than_8_percent_off_the_best": n_off,
                      "worst_ratio": worst}), flush=True)


def bench_mix(torch, g1s=(0.1, 0.25, 0.5, 1.0, 5.0), steps=30, warmup=5):
    """The two ways to run a mixed mask (tiled_wise_1d_mix at 75 %, i.i.d. weights) on the headline
    shape: the covering plan, and the plan of the tile-wise stage followed by tw_side_gemm on the
    element-wise remainder.  One JSON line per g1percent with the times in us."""
    from tilesparsity_amd import twgemm as tw, twprune
    M, K, N, G = 12544, 4608, 512, 128
    rng = np.random.default_rng(3)
    W = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    scores = twprune.img2col_forward([W])
    n_tiles = (N + G - 1) // G
    table = [(t * G, min(G, N - t * G)) for t in range(n_tiles)]
    bufs = [(torch.randn((K, M), device="cuda").half(), torch.zeros((N, M), dtype=torch.float16, device="cuda"))
            for _ in range(4)]
    s = torch.cuda.current_stream().cuda_stream
    for g1 in g1s:
        mask = twprune.tiled_wise_1d_mix(scores, 75, G, g1)[0]
        mask0 = twprune.tiled_wise_1d(scores, 75 + g1, G)[0]
        with tw.Plan.from_mask_tiles(mask0, table, "f16", W) as plan0, \
                tw.Plan.from_mask_tiles(mask, table, "f16", W, cover=True) as cover, \
                tw.Side(mask & ~mask0, "f16", W) as side:
            def run_tw(i):
                a, c = bufs[i % 4]
                plan0.gemm(a.data_ptr(), c.data_ptr(), M, pruned_cols=tw.PRUNED_ZERO, stream=s)

            def run_side(i):
                a, c = bufs[i % 4]
                side.gemm(a.data_ptr(), c.data_ptr(), M, stream=s)

            def run_pair(i):
                run_tw(i)
                run_side(i)

            def run_cover(i):
                a, c = bufs[i % 4]
                cover.gemm(a.data_ptr(), c.data_ptr(), M, pruned_cols=tw.PRUNED_ZERO, stream=s)
            t = {name: min(time_steps(fn, steps, warmup, torch) for _ in range(3)) * 1e6
                 for name, fn in (("us_tw_stage", run_tw), ("us_side", run_side), ("us_tw_then_side", run_pair),
                                  ("us_covering_plan", run_cover))}
            print(json.dumps(dict(workload="vgg16_conv4_2 M=12544 K=4608 N=512 G=128, tiled_wise_1d_mix 75 %",
                                  g1percent=g1, remainder_elements=side.nnz, **t)), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=None,
                    help="one configuration only (default: vgg16_conv4_2 with the full report: the "
                         "other target shapes and the two-stream leg)")
    ap.add_argument("--two-streams", action="store_true",
                    help="also time independent launches issued on two streams in turn")
    ap.add_argument("--all", action="store_true", help="(kept for old command lines: every configuration runs by default)")
    ap.add_argument("--headline-only", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--rows", type=int, default=None,
                    help="launch the configuration's plan on its first ROWS rows of A only (how long "
                         "an item takes with few of them on the chip); implies --headline-only")
    ap.add_argument("--producers", action="store_true",
                    help="benchmark the TW mask producers instead of the GEMM (one JSON line)")
    ap.add_argument("--prepass", action="store_true",
                    help="time the mask -> kept lists -> offsets -> compaction pre-pass instead")
    ap.add_argument("--shape-grid", action="store_true",
                    help="time the automatic kernel-shape choice against every forced shape on a "
                         "grid of problems (several minutes)")
    ap.add_argument("--mix", action="store_true",
                    help="time the two ways to run a mixed (tile-wise + element-wise) mask: the covering "
                         "plan and the tile-wise plan followed by the side kernel")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (4 launches over rotating buffers), "
                         "so that FETCH_SIZE / WRITE_SIZE read under rocprofv3 can be scaled by what "
                         "the same counters show for a copy of known size")
    args = ap.parse_args()
    full_report = args.workload is None   # no configuration named: the headline with everything
    if full_report:
        args.workload = "vgg16_conv4_2"
    if args.gpus != 1:
        print("bench.py: this engine and this benchmark use exactly one GPU; "
              "--gpus %d is not supported (run with --gpus 1)" % args.gpus, file=sys.stderr)
        return 2
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    from tilesparsity_amd import twgemm as tw
    tw.lib()  # fails loudly if the HIP library has not been built
    if args.shape_grid:
        bench_shape_grid(torch)
        return 0
    if args.mix:
        bench_mix(torch)
        return 0
    if args.producers:
        print(json.dumps(bench_producers(min(args.steps, 20), min(args.warmup, 3), torch)), flush=True)
        return 0
    if args.prepass:
        print(json.dumps(bench_prepass(make_workload(args.workload), min(args.steps, 20),
                                       min(args.warmup, 3))), flush=True)
        return 0

    if args.copy_calibration:
        n = (256 << 20) // 4
        srcs = [torch.full((n,), float(i), dtype=torch.float32, device="cuda") for i in range(4)]
        dsts = [torch.empty_like(x) for x in srcs]
        torch.cuda.synchronize()
        for x, y in zip(srcs, dsts):          # each source was written long ago: it comes from HBM
            y.copy_(x)
        torch.cuda.synchronize()
        del srcs, dsts
        torch.cuda.empty_cache()

    two_streams = args.two_streams or full_report
    wl = make_workload(args.workload)
    if args.rows is not None:
        if not 0 < args.rows <= wl["M"]:
            print("bench.py: --rows must be in 1 .. %d" % wl["M"], file=sys.stderr)
            return 2
        full_values, rows = wl["values"], args.rows
        wl = dict(wl, M=rows, values=lambda: (lambda ab: (np.ascontiguousarray(ab[0][:rows]), ab[1]))(full_values()))
        args.headline_only = True
        two_streams = args.two_streams
    res, (A, B) = run_workload(wl, args.steps, args.warmup, torch, two_streams=two_streams)
    roof = dict(res["roofline"])
    out = {
        "metric": "effective TFLOP/s (dense flops / time) at 75% TW sparsity, G=128",
        "value": res["effective_tflops"], "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": res["us_sparse"] * 1e-3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": wl["dtype"], "data": "synthetic",
        "config": {"workload": "%s M=%d K=%d N=%d G=%d, %d tiles, seed %d" % (
            wl["name"], wl["M"], wl["K"], wl["N"], wl["G"], len(wl["tiles"]), wl["seed"])},
        "speedup_vs_dense_plan": res["speedup_vs_dense"],
        "speedup_vs_dense_library": res["speedup_vs_dense_library"],
        "actual_tflops": res["actual_tflops"], "dense_plan_tflops": res["dense_tflops"],
        "dense_library_tflops": res["dense_library_tflops"],
        "mfma_utilisation_kept_flops": res["mfma_util_kept"],
        "mfma_utilisation_dense_run": res["mfma_util_dense_run"],
        "us_sparse": res["us_sparse"], "us_sparse_median": res["us_sparse_median"],
        "us_dense": res["us_dense"], "us_dense_library": res["us_dense_library"],
        "repeats_for_medians": res["repeats"], "untimed_prewarm_seconds": PREWARM_SECONDS,
        "kernel_sparse": res["kernel_sparse"], "kernel_dense_plan": res["kernel_dense_plan"],
        "roofline": roof,
    }
    if "two_streams" in res:
        out["independent_launches_on_two_streams"] = res["two_streams"]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wl, A, B)
    del A, B
    # the other configurations: BERT-base FFN (small K per tile), the NMT gate GEMM (skinny M; its
    # 50 time steps are recorded into a graph and replayed), the BERT-large FFN pair at three
    # sparsities and the imbalance stress shape, each with the roofline of its own launch and the
    # names of the kernels its sparse and its 0 %-sparse plan ran
    names = ["bert_base_ffn", "nmt_lstm_gates", "bert_large_ffn1_50", "bert_large_ffn1_75", "bert_large_ffn1_90",
             "bert_large_ffn2_50", "bert_large_ffn2_75", "bert_large_ffn2_90", "imbalance_stress"]
    if args.workload != "vgg16_conv4_2" or args.headline_only:
        names = []
    others = {}
    for name in names:
        nmt = name == "nmt_lstm_gates"
        big = name == "imbalance_stress"   # (launches of 0.3 - 1.5 ms: fewer of them)
        r, _ = run_workload(make_workload(name), 50 if nmt else (min(args.steps, 30) if big else args.steps),
                            args.warmup, torch, repeats=3, graph=nmt, two_streams=two_streams and not big)
        others[name] = {k: r[k] for k in ("us_sparse", "us_sparse_median", "us_dense",
                                          "us_dense_library", "effective_tflops", "actual_tflops",
                                          "speedup_vs_dense", "speedup_vs_dense_library",
                                          "mfma_util_kept", "hbm_gbs", "dtype", "timed_with", "kernel_sparse",
                                          "kernel_dense_plan", "roofline")}
        if "two_streams" in r:
            others[name]["independent_launches_on_two_streams"] = r["two_streams"]
        if name == "bert_base_ffn":
            t_direct, t_a_staged = time_row_major(make_workload(name), args.steps, args.warmup, torch)
            others[name]["us_row_major_a_and_c"] = t_direct * 1e6
            others[name]["us_row_major_a_staged_c_k_major"] = t_a_staged * 1e6
        if nmt:
            t_step, t_gates, t_fused, t_persistent = time_nmt_recurrence(make_workload(name), 50, torch)
            others[name]["us_step_gemm_and_gates"] = t_step * 1e6
            others[name]["us_gates_alone"] = t_gates * 1e6
            others[name]["us_step_fused"] = t_fused * 1e6
            others[name]["us_step_persistent"] = t_persistent * 1e6
        print("# %s %s" % (name, json.dumps(others[name])), file=sys.stderr, flush=True)
    if others:
        out["other_workloads"] = others
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
