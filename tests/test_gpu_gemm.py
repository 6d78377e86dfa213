"""GPU parity of the TW GEMM against the CPU oracle, through the C ABI.

Tolerance (stated by the task): max relative error <= 1e-2 for fp16 and <= 2e-2 for
bf16, measured as max |C - C_ref| / max(|C_ref|, 1e-2 * rms(C_ref)) against the
oracle's fp64 dense matmul of the masked weight on the same 16-bit inputs.  Integer
outcomes (which columns are written, untouched sentinels) are checked bit-exactly.
"""
import numpy as np
import pytest

from tests.helpers import from_device_bits, random_tiles, to_device_bits

pytestmark = pytest.mark.gpu

TOL = {"f16": 1e-2, "bf16": 2e-2}
SENTINEL = 0x1234  # 16-bit pattern pre-filled into C


def round_up(v, m):
    return (v + m - 1) // m * m


def run_gemm(tw, oracle, plan, A, dtype, N, alpha=1.0, beta=0.0, C0=None, pruned=0, pad=0):
    """A: fp32 [M,K] -> device K-major 16-bit; returns (C as fp32 [M,N], raw C bits [N,ldc])."""
    import torch
    M, K = A.shape
    lda = round_up(M, 8) + pad
    ldc = round_up(M, 8) + pad
    At = np.zeros((K, lda), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    Cb = np.full((N, ldc), SENTINEL, np.uint16)
    if C0 is not None:
        Cb[:, :M] = oracle.cast_bits(C0, dtype).reshape(M, N).T
    dA = to_device_bits(At, (K, lda))
    dC = to_device_bits(Cb, (N, ldc))
    plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, alpha=alpha, beta=beta,
              pruned_cols=pruned, stream=torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    bits = from_device_bits(dC)
    return oracle.bits_to_f32(bits[:, :M], dtype).reshape(N, M).T.copy(), bits


def reference(oracle, A, B, tiles, dtype, alpha=1.0, beta=0.0, C0=None):
    Aq, Bq = oracle.quantize(A, dtype), oracle.quantize(B, dtype)
    Cq = None if C0 is None else oracle.quantize(C0, dtype)
    return oracle.tw_gemm_reference(Aq, Bq, tiles, alpha, beta, Cq)


def kept_columns(tiles, N):
    keep = np.zeros(N, bool)
    for t in tiles:
        keep[np.asarray(t["kept_n"], np.int64) + t["col0"]] = True
    return keep


CASES = [
    # M,  K,   N,   G,  k_keep n_keep empty
    (128, 64, 128, 128, 0.5, 1.0, 0),
    (256, 128, 256, 128, 0.25, 1.0, 0),
    (100, 96, 200, 128, 0.3, 0.9, 0),     # ragged M, ragged last tile, K_t not multiples of 32
    (8, 40, 64, 64, 0.5, 0.8, 0),         # tiny M, G = 64 kernel
    (520, 300, 320, 64, 0.2, 0.8, 3),     # G = 64, empty tiles
    (333, 257, 384, 128, 0.25, 0.9, 4),   # M not a multiple of 8
    (1024, 768, 512, 128, 0.25, 1.0, 0),
    (64, 512, 130, 128, 0.1, 0.5, 0),     # last tile 2 columns wide
    (257, 64, 96, 32, 0.5, 0.75, 2),      # G = 32
    (192, 200, 512, 256, 0.3, 0.9, 0),    # tiles wider than one work unit
    (300, 96, 5120, 128, 0.5, 1.0, 7),    # more units than fit the kernel-argument table
    (2048, 64, 4224, 128, 0.6, 0.9, 0),   # several items per workgroup, one 64-row step each
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("case", CASES)
def test_gemm_matches_oracle(tw, oracle, case, dtype):
    M, K, N, G, kk, nk, empty = case
    rng = np.random.default_rng(hash(case) % (2 ** 31))
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=kk, n_keep=nk, empty_every=empty)
    print("case", case, dtype, flush=True)
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        C, bits = run_gemm(tw, oracle, plan, A, dtype, N, pad=8)
    ref = reference(oracle, A, B, tiles, dtype)
    keep = kept_columns(tiles, N)
    err = oracle.rel_error(C[:, keep], ref[:, keep])
    assert err <= TOL[dtype], err
    # pruned columns and the padding rows beyond M were never written
    assert np.all(bits[~keep, :] == SENTINEL)
    assert np.all(bits[:, M:] == SENTINEL)
    # the reference's own acceptance rule (basic_nn.cu:771-798, err 1e-2) on the kept part
    big = np.abs(ref[:, keep]) > 0.05
    assert oracle.checkout(np.where(big, C[:, keep], 0), np.where(big, ref[:, keep], 0),
                           err=2e-2 if dtype == "bf16" else 1e-2) == 0


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_alpha_beta_and_zero_mode(tw, oracle, dtype):
    rng = np.random.default_rng(21)
    M, K, N, G = 200, 160, 256, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.7)
    keep = kept_columns(tiles, N)
    C0q = oracle.quantize(C0, dtype)
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        # beta != 0: C read only on kept columns, pruned ones untouched (bit-exact)
        C, bits = run_gemm(tw, oracle, plan, A, dtype, N, alpha=0.5, beta=-1.5, C0=C0)
        ref = reference(oracle, A, B, tiles, dtype, 0.5, -1.5, C0)
        assert oracle.rel_error(C[:, keep], ref[:, keep]) <= TOL[dtype]
        assert np.array_equal(C[:, ~keep], C0q[:, ~keep])
        # zero mode, beta == 0: pruned columns become exact zeros
        C, bits = run_gemm(tw, oracle, plan, A, dtype, N, alpha=2.0, C0=C0, pruned=tw.PRUNED_ZERO)
        ref = reference(oracle, A, B, tiles, dtype, 2.0)
        assert oracle.rel_error(C[:, keep], ref[:, keep]) <= TOL[dtype]
        assert np.all(bits[~keep, :M] == 0)
        assert np.all(bits[:, M:] == SENTINEL)
        # zero mode with beta: pruned columns receive beta * C, the full product's value
        C, _ = run_gemm(tw, oracle, plan, A, dtype, N, alpha=1.0, beta=0.5, C0=C0,
                        pruned=tw.PRUNED_ZERO)
        full = oracle.quantize(A, dtype).astype(np.float64) @ oracle.masked_dense_weight(
            oracle.quantize(B, dtype), tiles).astype(np.float64) + 0.5 * C0q
        assert oracle.rel_error(C, full) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_row_major_columns_in_groups_of_four(tw, oracle, dtype):
    """Row-major A and C on a plan whose kept columns are neighbours in C (no column pruned: the
    A-stationary kernel then stores 16-byte pieces of rows) or come in groups of four (element-wise
    stores in the blocks that hold an odd group).  Bit for bit the K-major result with bias and
    ReLU, within tolerance with GELU; ragged M, padding and pruned columns untouched, a C that
    starts 16 bytes into its buffer, a bias that is not 16-byte aligned."""
    import torch
    rng = np.random.default_rng(77)
    M, K, N, G = 203, 320, 512, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = []
    for t in range(N // G):
        quads = np.arange(G // 4) if t % 2 == 0 else np.sort(rng.choice(G // 4, 19, replace=False))
        kept_n = (quads[:, None] * 4 + np.arange(4)).reshape(-1).astype(np.int32)
        kept_k = np.sort(rng.choice(K, K * 2 // 5, replace=False)).astype(np.int32)
        tiles.append(dict(col0=t * G, width=G, kept_k=kept_k, kept_n=kept_n))
    keep = kept_columns(tiles, N)
    Ab = oracle.cast_bits(A, dtype).reshape(M, K)
    d_bias = torch.from_numpy(bias).cuda()
    d_bias1 = torch.from_numpy(np.concatenate([[0.0], bias]).astype(np.float32)).cuda()
    ld8 = round_up(M, 8)
    Ak = np.zeros((K, ld8), np.uint16)
    Ak[:, :M] = Ab.T
    lda = K + 8
    Ar = np.zeros((M, lda), np.uint16)
    Ar[:, :K] = Ab
    pre = 0.75 * reference(oracle, A, B, tiles, dtype) + bias
    refs = {tw.ACT_RELU: np.maximum(pre, 0.0),
            tw.ACT_GELU: 0.5 * pre * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (pre + 0.044715 * pre ** 3)))}
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        dAk, dAr = to_device_bits(Ak, Ak.shape), to_device_bits(Ar, Ar.shape)
        for act, ref in refs.items():
            dCk = to_device_bits(np.full((N, ld8), SENTINEL, np.uint16), (N, ld8))
            tw.set_option(tw.OPT_SHAPE, tw.SHAPE_AS32)   # (the default for so few rows sums k in four slices)
            try:
                plan.gemm(dAk.data_ptr(), dCk.data_ptr(), M, lda=ld8, ldc=ld8, alpha=0.75,
                          bias_ptr=d_bias.data_ptr(), activation=act)
            finally:
                tw.set_option(tw.OPT_SHAPE, -1)
            torch.cuda.synchronize()
            want = from_device_bits(dCk)[:, :M].T
            want_f = oracle.bits_to_f32(np.ascontiguousarray(want), dtype).reshape(M, N)
            assert oracle.rel_error(want_f[:, keep], ref[:, keep]) <= TOL[dtype]
            # 8-byte stores; a bias that is not 16-byte aligned: element-wise stores
            for ldc, shift, bias_shift in ((N + 8, 0, 0), (N + 16, 8, 0), (N + 8, 0, 1)):
                full = torch.full((M * ldc + 16,), SENTINEL, dtype=torch.int16, device="cuda")
                plan.gemm(dAr.data_ptr(), full.data_ptr() + 2 * shift, M, lda=lda, ldc=ldc, alpha=0.75,
                          a_layout=tw.ROWMAJOR, c_layout=tw.ROWMAJOR,
                          bias_ptr=(d_bias1.data_ptr() + 4) if bias_shift else d_bias.data_ptr(),
                          activation=act)
                torch.cuda.synchronize()
                flat = full.cpu().numpy().view(np.uint16)
                assert np.all(flat[:shift] == SENTINEL) and np.all(flat[shift + M * ldc:] == SENTINEL)
                got = flat[shift:shift + M * ldc].reshape(M, ldc)
                assert np.all(got[:, N:] == SENTINEL)
                assert np.all(got[:, :N][:, ~keep] == SENTINEL)
                if act == tw.ACT_RELU:      # the same arithmetic in every kernel: the same bits
                    assert np.array_equal(got[:, :N][:, keep], want[:, keep])
                else:
                    got_f = oracle.bits_to_f32(np.ascontiguousarray(got[:, :N]), dtype).reshape(M, N)
                    assert oracle.rel_error(got_f[:, keep], ref[:, keep]) <= TOL[dtype]
                    assert oracle.rel_error(got_f[:, keep], want_f[:, keep]) <= 0.5 * TOL[dtype]


@pytest.mark.parametrize("staged", [False, True])
@pytest.mark.parametrize("a_layout,c_layout", [(1, 1), (1, 0), (0, 1)])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_row_major_layouts(tw, oracle, a_layout, c_layout, dtype, staged):
    """Row-major A[M,K] (lda >= K) and/or C[M,N] (ldc >= N): through the layout-generic kernel, and
    staged through K-major copies in a caller's workspace (tw_gemm_staged).  Ragged sizes: M, K
    and N are no multiples of 8, the leading dimensions leave padding that must stay untouched."""
    import torch
    rng = np.random.default_rng(31 + 2 * a_layout + c_layout)
    M, K, N, G = 203, 150, 330, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.8, empty_every=3)
    keep = kept_columns(tiles, N)
    Ab, Cb = oracle.cast_bits(A, dtype).reshape(M, K), oracle.cast_bits(C0, dtype).reshape(M, N)
    if a_layout == tw.ROWMAJOR:
        lda = round_up(K, 8) + 8
        Ah = np.zeros((M, lda), np.uint16)
        Ah[:, :K] = Ab
    else:
        lda = round_up(M, 8)
        Ah = np.zeros((K, lda), np.uint16)
        Ah[:, :M] = Ab.T
    for alpha, beta, pruned in ((1.0, 0.0, tw.PRUNED_UNTOUCHED), (0.5, 2.0, tw.PRUNED_ZERO)):
        if c_layout == tw.ROWMAJOR:
            ldc = round_up(N, 8) + 8
            Ch = np.full((M, ldc), SENTINEL, np.uint16)
            Ch[:, :N] = Cb
        else:
            ldc = round_up(M, 8)
            Ch = np.full((N, ldc), SENTINEL, np.uint16)
            Ch[:, :M] = Cb.T
        dA, dC = to_device_bits(Ah, Ah.shape), to_device_bits(Ch, Ch.shape)
        with tw.Plan.create(K, N, dtype, tiles, B) as plan:
            kw = {}
            if staged:
                nbytes = plan.staged_workspace(M, a_layout, c_layout)
                assert nbytes == 2 * round_up(M, 64) * (K * (a_layout == tw.ROWMAJOR) +
                                                        N * (c_layout == tw.ROWMAJOR))
                ws = torch.full((nbytes // 2 + 64,), 0x7bcd, dtype=torch.int16, device="cuda")
                kw = dict(workspace_ptr=ws.data_ptr(), workspace_bytes=nbytes)
                # (beta != 0: C is read, so the launch has to stage whatever the layouts are; with
                # beta == 0 and this short K two row-major operands need no workspace at all)
                with pytest.raises(tw.TwError) as e:
                    plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, beta=1.0, a_layout=a_layout,
                              c_layout=c_layout, workspace_ptr=ws.data_ptr(), workspace_bytes=nbytes - 2)
                assert e.value.status == tw.ERR_BUFFER
            plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, alpha=alpha, beta=beta,
                      a_layout=a_layout, c_layout=c_layout, pruned_cols=pruned, **kw)
            torch.cuda.synchronize()
            if staged:
                assert torch.all(ws[nbytes // 2:] == 0x7bcd)   # nothing beyond the stated size
                # the staged path is the K-major kernel on transposed copies: bit for bit what
                # that kernel gives on K-major operands
                Ak = np.zeros((K, round_up(M, 8)), np.uint16)
                Ak[:, :M] = Ab.T
                Ck = np.full((N, round_up(M, 8)), SENTINEL, np.uint16)
                Ck[:, :M] = Cb.T
                dAk, dCk = to_device_bits(Ak, Ak.shape), to_device_bits(Ck, Ck.shape)
                plan.gemm(dAk.data_ptr(), dCk.data_ptr(), M, lda=round_up(M, 8), ldc=round_up(M, 8),
                          alpha=alpha, beta=beta, pruned_cols=pruned)
                torch.cuda.synchronize()
                want = from_device_bits(dCk)[:, :M].T
                have = from_device_bits(dC)
                have = have[:, :N] if c_layout == tw.ROWMAJOR else have[:, :M].T
                assert np.array_equal(np.ascontiguousarray(have), np.ascontiguousarray(want))
        out = from_device_bits(dC)
        got = out[:, :N] if c_layout == tw.ROWMAJOR else out[:, :M].T
        pad = out[:, N:] if c_layout == tw.ROWMAJOR else out[:, M:]
        assert np.all(pad == SENTINEL)
        Cf = oracle.bits_to_f32(np.ascontiguousarray(got), dtype).reshape(M, N)
        ref = reference(oracle, A, B, tiles, dtype, alpha, beta, C0)
        assert oracle.rel_error(Cf[:, keep], ref[:, keep]) <= TOL[dtype]
        if pruned == tw.PRUNED_UNTOUCHED:
            assert np.array_equal(np.ascontiguousarray(got)[:, ~keep], Cb[:, ~keep])
        else:
            expect = oracle.cast_bits(beta * oracle.quantize(C0, dtype)[:, ~keep], dtype)
            assert np.array_equal(np.ascontiguousarray(got)[:, ~keep], expect.reshape(M, -1))


def test_gemm_degenerate_plans(tw, oracle):
    rng = np.random.default_rng(22)
    M, K, N, G = 96, 64, 256, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    e = np.zeros(0, np.int32)
    # tile 0 keeps columns but no K row -> zeros there; tile 1 keeps no column -> untouched
    tiles = [dict(col0=0, width=128, kept_k=e, kept_n=np.arange(0, 128, 3, dtype=np.int32)),
             dict(col0=128, width=128, kept_k=np.arange(K, dtype=np.int32), kept_n=e)]
    with tw.Plan.create(K, N, "f16", tiles, B) as plan:
        assert plan.info()["empty_tiles"] == 2
        C, bits = run_gemm(tw, oracle, plan, A, "f16", N)
        keep = kept_columns(tiles, N)
        assert np.all(bits[keep, :M] == 0) and np.all(bits[~keep, :] == SENTINEL)
        # M == 0 is a no-op
        plan.gemm(0, 0, 0)
    # identity weight: C is the gathered A columns, exactly
    K = N = 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    kk = np.sort(rng.choice(K, 37, replace=False)).astype(np.int32)
    one = [dict(col0=0, width=N, kept_k=kk, kept_n=np.arange(N, dtype=np.int32))]
    with tw.Plan.create(K, N, "f16", one, np.eye(K, dtype=np.float32)) as plan:
        C, _ = run_gemm(tw, oracle, plan, A, "f16", N)
    expect = np.zeros((M, N), np.float32)
    expect[:, kk] = oracle.quantize(A, "f16")[:, kk]
    assert np.array_equal(C, expect)


def test_dense_plan_equals_plain_gemm(tw, oracle):
    import torch
    rng = np.random.default_rng(23)
    M, K, N, G = 512, 384, 640, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    with tw.Plan.dense(K, N, G, "f16", B) as plan:
        C, _ = run_gemm(tw, oracle, plan, A, "f16", N)
    Aq, Bq = oracle.quantize(A, "f16"), oracle.quantize(B, "f16")
    assert oracle.rel_error(C, Aq.astype(np.float64) @ Bq.astype(np.float64)) <= TOL["f16"]
    # a library routine on the same inputs (hipBLASLt/rocBLAS through torch)
    lib = (torch.from_numpy(Aq).cuda().half() @ torch.from_numpy(Bq).cuda().half()).float().cpu().numpy()
    assert oracle.rel_error(C, lib) <= TOL["f16"]


def test_fused_equals_gather_dense_scatter_bitwise(tw, oracle):
    """The reference's first self-check (basic_nn.cu:1081, tolerance 1e-10 = exact): the
    fused masked GEMM equals gather rows -> dense GEMM on the compact tile -> scatter,
    run through the engine's own kernel and its deleteRow / insertRow kernels."""
    import torch
    rng = np.random.default_rng(24)
    M, K, N, G, dtype = 264, 320, 384, 128, "f16"
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.3, n_keep=0.8)
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        _, fused = run_gemm(tw, oracle, plan, A, dtype, N)
    At = oracle.cast_bits(A, dtype).reshape(M, K).T.copy()
    dA = to_device_bits(At, (K, M))
    out = np.full((N, M), SENTINEL, np.uint16)
    for t in tiles:
        kt, nt = len(t["kept_k"]), len(t["kept_n"])
        rel_k = torch.from_numpy(t["kept_k"] - np.arange(kt, dtype=np.int32)).cuda()
        rel_n = torch.from_numpy(t["kept_n"] - np.arange(nt, dtype=np.int32)).cuda()
        dA2 = torch.zeros((kt, M), dtype=torch.int16, device="cuda")
        tw.delete_row(dA.data_ptr(), dA2.data_ptr(), kt, M, rel_k.data_ptr())
        comp = B[np.ix_(t["kept_k"], t["kept_n"] + t["col0"])]
        dC2 = torch.zeros((nt, M), dtype=torch.int16, device="cuda")
        with tw.Plan.dense(kt, nt, max(nt, 1), dtype, comp) as dense:
            dense.gemm(dA2.data_ptr(), dC2.data_ptr(), M)
            torch.cuda.synchronize()
        dCt = to_device_bits(out[t["col0"]:t["col0"] + t["width"]], (t["width"], M))
        tw.insert_row(dCt.data_ptr(), dC2.data_ptr(), nt, M, rel_n.data_ptr())
        torch.cuda.synchronize()
        out[t["col0"]:t["col0"] + t["width"]] = from_device_bits(dCt)
    assert np.array_equal(fused[:, :M], out)


def test_tile_order_does_not_change_a_bit(tw, oracle):
    """Work-queue order must not matter: the same tiles with kept-K counts arranged so
    that the queue sorts them differently give bit-identical columns."""
    rng = np.random.default_rng(25)
    M, K, N, G, dtype = 300, 256, 512, 128, "f16"
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.3, n_keep=0.9)
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        _, base = run_gemm(tw, oracle, plan, A, dtype, N)
    # reverse the column-tile order of the weight (and of the plan): each tile's columns
    # must come out identical, at their new position
    perm = list(reversed(range(len(tiles))))
    B2 = np.concatenate([B[:, tiles[i]["col0"]:tiles[i]["col0"] + G] for i in perm], axis=1)
    tiles2 = [dict(col0=j * G, width=G, kept_k=tiles[i]["kept_k"], kept_n=tiles[i]["kept_n"])
              for j, i in enumerate(perm)]
    with tw.Plan.create(K, N, dtype, tiles2, B2) as plan:
        _, moved = run_gemm(tw, oracle, plan, A, dtype, N)
    for j, i in enumerate(perm):
        assert np.array_equal(moved[j * G:(j + 1) * G], base[i * G:(i + 1) * G])


def test_repeated_launches_and_slot_reuse(tw, oracle):
    """More launches than ticket slots on one plan: every launch must see a re-armed queue."""
    import torch
    rng = np.random.default_rng(26)
    M, K, N, G, dtype = 136, 96, 256, 128, "f16"
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=0.9)
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        _, first = run_gemm(tw, oracle, plan, A, dtype, N)
        At = oracle.cast_bits(A, dtype).reshape(M, K).T.copy()
        dA = to_device_bits(At, (K, M))
        dC = torch.zeros((N, M), dtype=torch.int16, device="cuda")
        for _ in range(600):
            plan.gemm(dA.data_ptr(), dC.data_ptr(), M,
                      stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        keep = kept_columns(tiles, N)
        assert np.array_equal(from_device_bits(dC)[keep], first[keep, :M])


def test_plan_reset_leaves_results_unchanged(tw, oracle):
    """tw_plan_reset between launches (the call that re-arms every ticket slot after an aborted
    launch): the launches after it give the bits of the launches before it."""
    import torch
    rng = np.random.default_rng(28)
    M, K, N, G, dtype = 300, 192, 640, 128, "f16"
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=0.9)
    stream = torch.cuda.current_stream().cuda_stream
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        _, first = run_gemm(tw, oracle, plan, A, dtype, N)
        ld = (M + 7) // 8 * 8
        At = np.zeros((K, ld), np.uint16)
        At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
        dA = to_device_bits(At, (K, ld))
        keep = kept_columns(tiles, N)
        for _ in range(3):
            plan.reset(stream)
            dC = torch.zeros((N, ld), dtype=torch.int16, device="cuda")
            for _ in range(5):
                plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=ld, ldc=ld, stream=stream)
            torch.cuda.synchronize()
            assert np.array_equal(from_device_bits(dC)[keep, :M], first[keep, :M])
    assert tw.lib().tw_plan_reset(None, None) == tw.ERR_NULL


def test_queue_is_rearmed_between_launches_of_different_sizes(tw, oracle):
    """Launches with few items (one per workgroup), with several rounds of items per workgroup,
    and with items that have no step or only fill zeros alternate on one plan, through every
    ticket slot more than once: each launch re-arms the queue for the next, whatever its grid
    was, so every result repeats bit for bit."""
    import torch
    rng = np.random.default_rng(27)
    K, N, G, dtype = 320, 1536, 128, "bf16"
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.85, empty_every=5)
    Ms = (8, 520, 33000)                  # 12 items; 36 items; 129 row blocks x 12 units
    stream = torch.cuda.current_stream().cuda_stream
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        dA, dC, want = {}, {}, {}
        for M in Ms:
            ld = (M + 7) // 8 * 8
            g = torch.Generator(device="cuda")
            g.manual_seed(M)
            dA[M] = torch.randn((K, ld), generator=g, device="cuda").to(torch.bfloat16)
            dC[M] = torch.zeros((N, ld), dtype=torch.bfloat16, device="cuda")
            plan.gemm(dA[M].data_ptr(), dC[M].data_ptr(), M, lda=ld, ldc=ld, stream=stream,
                      pruned_cols=tw.PRUNED_ZERO)
            torch.cuda.synchronize()
            want[M] = dC[M].clone()
            ref = (dA[M][:, :M].float().T.cpu().numpy() @
                   (oracle.quantize(B, dtype) * oracle.plan_mask(K, N, tiles)))
            got = dC[M][:, :M].float().T.cpu().numpy()
            assert oracle.rel_error(got, ref) <= TOL[dtype], M
        print("re-arm over mixed sizes", Ms, flush=True)
        for i in range(3 * 256 + 5):
            M = Ms[i % 3] if i % 7 else Ms[2 - i % 3]
            ld = (M + 7) // 8 * 8
            dC[M].fill_(1.0)
            plan.gemm(dA[M].data_ptr(), dC[M].data_ptr(), M, lda=ld, ldc=ld, stream=stream,
                      pruned_cols=tw.PRUNED_ZERO)
            if i % 64 == 63 or i > 3 * 256:
                torch.cuda.synchronize()
                assert torch.equal(dC[M][:, :M], want[M][:, :M]), (i, M)


def test_gemm_argument_errors(tw):
    import torch
    K, N, M = 64, 128, 64
    with tw.Plan.dense(K, N, 128, "f16", np.zeros((K, N), np.float32)) as plan:
        a = torch.zeros((K, M), dtype=torch.int16, device="cuda")
        c = torch.zeros((N, M), dtype=torch.int16, device="cuda")
        for kwargs, status in ((dict(lda=M - 8), tw.ERR_SHAPE), (dict(ldc=M + 4), tw.ERR_ALIGNMENT),
                               (dict(a_layout=5), tw.ERR_LAYOUT), (dict(pruned_cols=3), tw.ERR_LAYOUT)):
            with pytest.raises(tw.TwError) as e:
                plan.gemm(a.data_ptr(), c.data_ptr(), M, **kwargs)
            assert e.value.status == status
        with pytest.raises(tw.TwError) as e:
            plan.gemm(a.data_ptr() + 2, c.data_ptr(), M)
        assert e.value.status == tw.ERR_ALIGNMENT
        with pytest.raises(tw.TwError) as e:
            plan.gemm(0, c.data_ptr(), M)
        assert e.value.status == tw.ERR_NULL
        with pytest.raises(tw.TwError) as e:
            plan.gemm(a.data_ptr(), c.data_ptr(), -1)
        assert e.value.status == tw.ERR_SHAPE


def test_stream_gemm_nn_drop_in(tw, oracle):
    """The reference's own problem (`test_basic_nn 64 768 256 384 128`, its rand() stream)
    driven through the Stream_Gemm_NN-shaped entry point with the reference's operands."""
    import torch
    M, N, K, Np, Kp = 64, 768, 256, 384, 128
    A, B, tiles, part = oracle.ref_compat_problem(M, N, K, Np, Kp)
    dtype = "f16"
    dA = to_device_bits(oracle.cast_bits(A, dtype).reshape(M, K).T.copy(), (K, M))
    dB = to_device_bits(oracle.cast_bits(oracle.stream_weight(B, tiles), dtype), (K * N,))
    dC = torch.zeros((N, M), dtype=torch.int16, device="cuda")
    mk = [torch.from_numpy(t["mask_k"]).cuda() for t in tiles]
    mn = [torch.from_numpy(t["mask_n"]).cuda() for t in tiles]
    tw.stream_gemm_nn(M, N, K, dtype, 1.0, dA.data_ptr(), dB.data_ptr(), 0.0, dC.data_ptr(),
                      part["N_cal"], part["K_cal"], [x.data_ptr() for x in mn],
                      [x.data_ptr() for x in mk], part["off_B"], part["off_C"])
    C = oracle.bits_to_f32(from_device_bits(dC), dtype).reshape(N, M).T
    ref = reference(oracle, A, B, tiles, dtype)
    assert oracle.rel_error(C, ref) <= TOL[dtype]
    # and a plan built from those operands exports the same lists and weight bits
    with tw.Plan.from_stream_operands(M, N, K, dtype, dB.data_ptr(), part["N_cal"], part["K_cal"],
                                      [x.data_ptr() for x in mn], [x.data_ptr() for x in mk],
                                      part["off_B"], part["off_C"]) as plan:
        got, Bs = plan.export()
        for g, t in zip(got, tiles):
            assert np.array_equal(g["kept_k"], t["kept_k"]) and np.array_equal(g["mask_n"], t["mask_n"])
        assert np.array_equal(Bs, from_device_bits(dB))


@pytest.mark.parametrize("forced", ["auto", "streaming"])
def test_graph_capture_replays_bitwise(tw, oracle, forced):
    """tw_gemm allocates nothing, clears nothing from the host and re-arms its work queue inside
    the kernel, so a sequence of launches can be captured into a HIP graph; every replay (with
    eager launches and synchronisations in between) gives the eager result bit for bit.  Once with
    the kernel the launch picks by itself (none that uses the queue at this size) and once with a
    streaming kernel forced, whose recorded launches keep a ticket slot of the plan's captured
    range across the replays and re-arm it each time."""
    import torch
    rng = np.random.default_rng(77)
    M, K, N, G = 384, 256, 512, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.9)
    At = np.ascontiguousarray(oracle.cast_bits(A, "f16").reshape(M, K).T)
    dA = to_device_bits(At, At.shape)
    dH = torch.zeros((N, M), dtype=torch.int16, device="cuda")
    dC = torch.zeros((N, M), dtype=torch.int16, device="cuda")
    s = torch.cuda.Stream()
    try:
        if forced == "streaming":
            tw.set_option(tw.OPT_SHAPE, tw.SHAPE_128x64)
            tw.set_option(tw.OPT_PIECE, 64)
            tw.set_option(tw.OPT_XCD_QUEUES, 1)
        with tw.Plan.create(K, N, "f16", tiles, B) as plan:
            if forced == "streaming":
                assert plan.choice(M)["shape"] == tw.SHAPE_128x64

            def chain():
                # two dependent launches: C = A (B.mask), then C += 0.5 * A (B.mask) on top of it
                plan.gemm(dA.data_ptr(), dH.data_ptr(), M, pruned_cols=tw.PRUNED_ZERO, stream=s.cuda_stream)
                plan.gemm(dA.data_ptr(), dC.data_ptr(), M, alpha=0.5, beta=0.0, pruned_cols=tw.PRUNED_ZERO,
                          stream=s.cuda_stream)
                plan.gemm(dA.data_ptr(), dC.data_ptr(), M, alpha=1.0, beta=1.0, stream=s.cuda_stream)
            with torch.cuda.stream(s):
                print("graph capture", forced, flush=True)
                chain()
                s.synchronize()
                want_h, want_c = dH.clone(), dC.clone()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=s):
                    chain()
                for rep in range(4):
                    dH.fill_(0x1234)
                    dC.fill_(0x1234)
                    plan.gemm(dA.data_ptr(), dH.data_ptr(), M, stream=s.cuda_stream)   # eager work between replays
                    s.synchronize()
                    g.replay()
                    s.synchronize()
                    assert torch.equal(dH, want_h) and torch.equal(dC, want_c), rep
    finally:
        for opt in (tw.OPT_SHAPE, tw.OPT_PIECE, tw.OPT_XCD_QUEUES):
            tw.set_option(opt, -1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_every_kernel_shape_agrees(tw, oracle, dtype):
    """The launch picks a kernel shape, the width of a unit piece and the queue layout from the
    plan and M; tw_set_option forces each combination a plan can run with in turn: all match the
    oracle, and each repeats itself bit for bit."""
    rng = np.random.default_rng(88)
    W, S1, S2, S3, S4, S5 = (tw.SHAPE_WIDE, tw.SHAPE_128x128, tw.SHAPE_512x64, tw.SHAPE_128x64,
                             tw.SHAPE_256x128, tw.SHAPE_128x32)
    A6, A3, SK, BS, S6 = tw.SHAPE_AS64, tw.SHAPE_AS32, tw.SHAPE_SKINNY, tw.SHAPE_BS, tw.SHAPE_256x64
    cases = (
        (600, 320, 384, 128, ((W, -1), (S1, -1), (S4, -1), (S3, 64), (S5, 32), (S1, 64), (S4, 32),
                              (A6, -1), (A3, -1), (SK, -1), (BS, -1))),
        (1100, 200, 256, 64, ((S2, -1), (S3, -1), (S5, 32), (S1, -1), (S4, -1), (W, -1), (A6, -1),
                              (A3, -1), (SK, -1), (BS, -1), (S6, -1), (S6, 32))),
        (2500, 130, 96, 32, ((S5, -1), (S3, -1), (S2, -1), (A6, -1), (A3, -1), (SK, -1), (BS, -1), (S6, -1), (S6, 32))),
    )
    try:
        for (M, K, N, G, combos) in cases:
            A = rng.standard_normal((M, K)).astype(np.float32)
            B = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
            tiles = random_tiles(rng, K, N, G, k_keep=0.45, n_keep=0.85)
            ref = reference(oracle, A, B, tiles, dtype)
            keep = kept_columns(tiles, N)
            with tw.Plan.create(K, N, dtype, tiles, B) as plan:
                for shape, piece in combos:
                    for xcd in (1, 0, 2):
                        tw.set_option(tw.OPT_SHAPE, shape)
                        tw.set_option(tw.OPT_PIECE, piece)
                        tw.set_option(tw.OPT_XCD_QUEUES, xcd)
                        print("shape", shape, "piece", piece, "xcd", xcd, M, K, N, G, dtype, flush=True)
                        C1, bits1 = run_gemm(tw, oracle, plan, A, dtype, N)
                        C2, bits2 = run_gemm(tw, oracle, plan, A, dtype, N)
                        assert oracle.rel_error(C1[:, keep], ref[:, keep]) <= TOL[dtype], (shape, piece)
                        assert np.array_equal(bits1, bits2), (shape, piece)
                        if shape in (S4, S6):
                            # the 256-row kernels load straight into LDS by default; their
                            # register-staged form gives the same bits
                            tw.set_option(tw.OPT_LDS_DMA, 0)
                            C3, bits3 = run_gemm(tw, oracle, plan, A, dtype, N)
                            tw.set_option(tw.OPT_LDS_DMA, -1)
                            assert np.array_equal(bits1, bits3), (shape, piece, "register-staged")
    finally:
        for opt in (tw.OPT_SHAPE, tw.OPT_PIECE, tw.OPT_XCD_QUEUES, tw.OPT_LDS_DMA):
            tw.set_option(opt, -1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_a_stationary_shapes(tw, oracle, dtype):
    """The A-stationary kernels (a panel of A resident in LDS, kept rows gathered inside LDS) are
    forced with tw_set_option here.  Tiles from no kept row to all of them (one to nine segments of
    two steps), ragged M, bias + activation, filled pruned columns: bit for bit what the streaming
    256 x 128 kernel gives, and within tolerance of the oracle.  With beta != 0 (C is read) the
    forced shape does not apply and the launch takes the default kernel (for these few rows the
    skinny one, whose sums run in slices: within half the tolerance)."""
    rng = np.random.default_rng(4321)
    M, K, N, G = 333, 1040, 640, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = []
    for t, (kt, nt) in enumerate(((1040, 128), (64, 100), (0, 128), (333, 128), (700, 7))):
        tiles.append(dict(col0=t * G, width=G,
                          kept_k=np.sort(rng.choice(K, size=kt, replace=False)).astype(np.int32),
                          kept_n=np.sort(rng.choice(G, size=nt, replace=False)).astype(np.int32)))
    keep = kept_columns(tiles, N)
    import torch
    dbias = torch.from_numpy(bias).cuda()
    lda = ldc = round_up(M, 8)
    At = np.zeros((K, lda), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    dA = to_device_bits(At, At.shape)

    def launch(plan, shape, alpha, beta, pruned, with_bias, act):
        Cb = np.full((N, ldc), SENTINEL, np.uint16)
        Cb[:, :M] = oracle.cast_bits(C0, dtype).reshape(M, N).T
        dC = to_device_bits(Cb, Cb.shape)
        tw.set_option(tw.OPT_SHAPE, shape)
        print("a-stationary test: shape", shape, alpha, beta, pruned, with_bias, act, dtype, flush=True)
        plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, alpha=alpha, beta=beta,
                  pruned_cols=pruned, bias_ptr=dbias.data_ptr() if with_bias else None, activation=act,
                  stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return from_device_bits(dC)

    try:
        with tw.Plan.create(K, N, dtype, tiles, B) as plan:
            for (alpha, beta, pruned, with_bias, act) in (
                    (1.0, 0.0, tw.PRUNED_UNTOUCHED, False, tw.ACT_NONE),
                    (0.5, 0.0, tw.PRUNED_ZERO, True, tw.ACT_RELU),
                    (1.0, 0.0, tw.PRUNED_ZERO, True, tw.ACT_GELU),
                    (2.0, 0.75, tw.PRUNED_ZERO, False, tw.ACT_NONE)):
                want = launch(plan, tw.SHAPE_256x128, alpha, beta, pruned, with_bias, act)
                for shape in (tw.SHAPE_AS64, tw.SHAPE_AS32):
                    got = launch(plan, shape, alpha, beta, pruned, with_bias, act)
                    if act == tw.ACT_GELU or beta != 0.0:
                        # the two kernels evaluate the polynomial inside GELU in loops of their
                        # own; the compiler fuses their multiply-adds differently: last-bit ties
                        a = oracle.bits_to_f32(got[:, :M], dtype)
                        b = oracle.bits_to_f32(want[:, :M], dtype)
                        assert oracle.rel_error(a, b) <= 0.5 * TOL[dtype]
                        assert np.array_equal(got[:, M:], want[:, M:])
                    else:
                        assert np.array_equal(got, want), (shape, alpha, beta, pruned, with_bias, act)
                if not with_bias and act == tw.ACT_NONE:
                    Cf = oracle.bits_to_f32(want[:, :M], dtype).reshape(N, M).T
                    ref = reference(oracle, A, B, tiles, dtype, alpha, beta, C0)
                    assert oracle.rel_error(Cf[:, keep], ref[:, keep]) <= TOL[dtype]
    finally:
        tw.set_option(tw.OPT_SHAPE, -1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_row_blocks_sized_per_tile(tw, oracle, dtype):
    """A launch whose items would not fill the chip once gives the tiles with more kept rows lower
    row blocks (multiples of 64 rows).  Tiles of 40 to 900 kept rows, one without any, ragged M,
    pruned columns filled, bias + activation, beta: every streaming shape gives the same bits with
    TW_OPT_BALANCE 0 and 1 and stays within tolerance of the oracle; nothing is written past M."""
    import torch
    rng = np.random.default_rng(8086)
    M, K, N, G = 5003, 1000, 640, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = []
    for t, (kt, nt) in enumerate(((900, 128), (40, 100), (0, 128), (333, 128), (520, 77))):
        tiles.append(dict(col0=t * G, width=G,
                          kept_k=np.sort(rng.choice(K, size=kt, replace=False)).astype(np.int32),
                          kept_n=np.sort(rng.choice(G, size=nt, replace=False)).astype(np.int32)))
    keep = kept_columns(tiles, N)
    dbias = torch.from_numpy(bias).cuda()
    lda = ldc = round_up(M, 8) + 8
    At = np.zeros((K, lda), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    dA = to_device_bits(At, At.shape)

    def launch(plan, shape, balance, alpha, beta, pruned, with_bias, act):
        Cb = np.full((N, ldc), SENTINEL, np.uint16)
        Cb[:, :M] = oracle.cast_bits(C0, dtype).reshape(M, N).T
        dC = to_device_bits(Cb, Cb.shape)
        tw.set_option(tw.OPT_SHAPE, shape)
        tw.set_option(tw.OPT_BALANCE, balance)
        print("row blocks per tile: shape", shape, balance, alpha, beta, pruned, with_bias, act, dtype, flush=True)
        plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, alpha=alpha, beta=beta,
                  pruned_cols=pruned, bias_ptr=dbias.data_ptr() if with_bias else None, activation=act,
                  stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return from_device_bits(dC)

    try:
        with tw.Plan.create(K, N, dtype, tiles, B) as plan:
            for (alpha, beta, pruned, with_bias, act) in (
                    (1.0, 0.0, tw.PRUNED_UNTOUCHED, False, tw.ACT_NONE),
                    (0.5, 0.0, tw.PRUNED_ZERO, True, tw.ACT_RELU),
                    (2.0, 0.75, tw.PRUNED_ZERO, False, tw.ACT_NONE)):
                for shape in (tw.SHAPE_256x128, tw.SHAPE_128x128):
                    want = launch(plan, shape, 0, alpha, beta, pruned, with_bias, act)
                    got = launch(plan, shape, 1, alpha, beta, pruned, with_bias, act)
                    assert np.array_equal(got, want), (shape, alpha, beta, pruned, with_bias, act)
                    assert (got[:, M:] == SENTINEL).all()
                    if not with_bias and act == tw.ACT_NONE:
                        Cf = oracle.bits_to_f32(got[:, :M], dtype).reshape(N, M).T
                        ref = reference(oracle, A, B, tiles, dtype, alpha, beta, C0)
                        assert oracle.rel_error(Cf[:, keep], ref[:, keep]) <= TOL[dtype]
    finally:
        tw.set_option(tw.OPT_SHAPE, -1)
        tw.set_option(tw.OPT_BALANCE, -1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape_bn", [128, 64])
def test_streaming_kernel_several_items_per_workgroup(tw, oracle, dtype, shape_bn):
    """The 256-row streaming kernels with more items than workgroups, so that every workgroup runs
    several one after the other: the first steps of the next item are loaded over the epilogue of
    the current one, and a full C tile (every column kept, 256 rows) is stored by the moving waves
    during the next item's first time slot.  Tiles of 1 to 7 steps, one without kept rows, full
    and partly kept columns, a ragged last row block: the same bits as the register-staged form of
    the kernel (TW_OPT_LDS_DMA = 0) and as a second launch, within tolerance of the oracle, with
    bias + activation and filled pruned columns as well."""
    import torch
    rng = np.random.default_rng(31337 + shape_bn)
    G = shape_bn
    n_tiles = 40 if G == 128 else 72
    M, K, N = 2048 + 256 * 5 + 77, 448, n_tiles * G          # 14 row blocks, the last one ragged
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = []
    for t in range(n_tiles):
        kt = (64, 128, 200, 448, 0, 130, 70, 256)[t % 8]
        nt = G if t % 3 else int(G * 0.8)
        tiles.append(dict(col0=t * G, width=G,
                          kept_k=np.sort(rng.choice(K, size=kt, replace=False)).astype(np.int32),
                          kept_n=np.sort(rng.choice(G, size=nt, replace=False)).astype(np.int32)))
    keep = kept_columns(tiles, N)
    ref = reference(oracle, A, B, tiles, dtype)
    dbias = torch.from_numpy(bias).cuda()
    lda = ldc = round_up(M, 8)
    At = np.zeros((K, lda), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    dA = to_device_bits(At, At.shape)
    shape = tw.SHAPE_256x128 if G == 128 else tw.SHAPE_256x64

    def launch(plan, dma, pruned, with_bias, act):
        dC = to_device_bits(np.full((N, ldc), SENTINEL, np.uint16), (N, ldc))
        tw.set_option(tw.OPT_LDS_DMA, dma)
        print("several items per workgroup:", G, dma, pruned, with_bias, act, dtype, flush=True)
        assert plan.choice(M, lda, ldc)["shape"] == shape
        plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, pruned_cols=pruned,
                  bias_ptr=dbias.data_ptr() if with_bias else None, activation=act,
                  stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return from_device_bits(dC)

    try:
        tw.set_option(tw.OPT_SHAPE, shape)
        with tw.Plan.create(K, N, dtype, tiles, B) as plan:
            for (pruned, with_bias, act) in ((tw.PRUNED_UNTOUCHED, False, tw.ACT_NONE),
                                             (tw.PRUNED_ZERO, True, tw.ACT_RELU)):
                want = launch(plan, 0, pruned, with_bias, act)
                for rep in range(2):
                    got = launch(plan, 1, pruned, with_bias, act)
                    assert np.array_equal(got, want), (rep, pruned, with_bias, act)
                assert (want[:, M:] == SENTINEL).all()
                if not with_bias:
                    Cf = oracle.bits_to_f32(want[:, :M], dtype).reshape(N, M).T
                    assert oracle.rel_error(Cf[:, keep], ref[:, keep]) <= TOL[dtype]
                    assert (want[~keep] == SENTINEL).all()
    finally:
        tw.set_option(tw.OPT_SHAPE, -1)
        tw.set_option(tw.OPT_LDS_DMA, -1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_256x64_shape_epilogues(tw, oracle, dtype):
    """The 256 x 64 streaming shape (64-wide tiles of plans with few items) with every epilogue:
    alpha / beta, bias + activation, filled pruned columns, both queue layouts and both piece
    widths it takes: bit for bit what the 128 x 64 shape gives (same step order over k, same
    epilogue code), within tolerance of the oracle, nothing written past M."""
    import torch
    rng = np.random.default_rng(6464)
    M, K, N, G = 777, 300, 320, 64
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.8)
    keep = kept_columns(tiles, N)
    dbias = torch.from_numpy(bias).cuda()
    lda = ldc = round_up(M, 8) + 8
    At = np.zeros((K, lda), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    dA = to_device_bits(At, At.shape)

    def launch(plan, shape, piece, xcd, alpha, beta, pruned, with_bias, act):
        Cb = np.full((N, ldc), SENTINEL, np.uint16)
        Cb[:, :M] = oracle.cast_bits(C0, dtype).reshape(M, N).T
        dC = to_device_bits(Cb, Cb.shape)
        tw.set_option(tw.OPT_SHAPE, shape)
        tw.set_option(tw.OPT_PIECE, piece)
        tw.set_option(tw.OPT_XCD_QUEUES, xcd)
        print("256x64 test: shape", shape, piece, xcd, alpha, beta, pruned, with_bias, act, dtype, flush=True)
        assert plan.choice(M, lda, ldc, beta)["shape"] == shape
        plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, alpha=alpha, beta=beta,
                  pruned_cols=pruned, bias_ptr=dbias.data_ptr() if with_bias else None, activation=act,
                  stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return from_device_bits(dC)

    try:
        with tw.Plan.create(K, N, dtype, tiles, B) as plan:
            for (alpha, beta, pruned, with_bias, act) in (
                    (1.0, 0.0, tw.PRUNED_UNTOUCHED, False, tw.ACT_NONE),
                    (0.5, 0.0, tw.PRUNED_ZERO, True, tw.ACT_RELU),
                    (1.0, 0.0, tw.PRUNED_ZERO, True, tw.ACT_GELU),
                    (2.0, 0.75, tw.PRUNED_ZERO, False, tw.ACT_NONE)):
                want = launch(plan, tw.SHAPE_128x64, -1, 0, alpha, beta, pruned, with_bias, act)
                for piece, xcd in ((-1, 0), (-1, 1), (32, 0), (32, 1)):
                    got = launch(plan, tw.SHAPE_256x64, piece, xcd, alpha, beta, pruned, with_bias, act)
                    assert np.array_equal(got, want), (piece, xcd, alpha, beta, pruned, with_bias, act)
                assert (want[:, M:] == SENTINEL).all()
                if not with_bias and act == tw.ACT_NONE:
                    Cf = oracle.bits_to_f32(want[:, :M], dtype).reshape(N, M).T
                    ref = reference(oracle, A, B, tiles, dtype, alpha, beta, C0)
                    assert oracle.rel_error(Cf[:, keep], ref[:, keep]) <= TOL[dtype]
    finally:
        for opt in (tw.OPT_SHAPE, tw.OPT_PIECE, tw.OPT_XCD_QUEUES):
            tw.set_option(opt, -1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M", [1, 31, 64, 100, 129, 200])
def test_skinny_kernel(tw, oracle, dtype, M):
    """The skinny kernel (32 rows of A and half a unit per workgroup, the kept rows split over its
    waves, the partial sums added in wave order) is what few rows of A get by default.  Tiles from
    no kept row over one step to 23 steps (three rounds of pairs, the last one odd), 7 to 128
    kept columns, ragged M, alpha / beta, bias + activation, filled pruned columns: within half
    the tolerance of the streaming 256 x 128 kernel (the sum over k runs in four slices), bit for
    bit what it gives where nothing is summed (pruned columns, tiles without kept rows), nothing
    written outside, and the same bits on a second launch."""
    rng = np.random.default_rng(555 + M)
    K, N, G = 1500, 768, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tiles = []
    for t, (kt, nt) in enumerate(((1460, 128), (64, 100), (0, 128), (333, 65), (700, 7), (1, 33))):
        tiles.append(dict(col0=t * G, width=G,
                          kept_k=np.sort(rng.choice(K, size=kt, replace=False)).astype(np.int32),
                          kept_n=np.sort(rng.choice(G, size=nt, replace=False)).astype(np.int32)))
    keep = kept_columns(tiles, N)
    import torch
    dbias = torch.from_numpy(bias).cuda()
    lda = ldc = round_up(M, 8) + 8
    At = np.zeros((K, lda), np.uint16)
    At[:, :M] = oracle.cast_bits(A, dtype).reshape(M, K).T
    dA = to_device_bits(At, At.shape)

    def launch(plan, shape, alpha, beta, pruned, with_bias, act):
        Cb = np.full((N, ldc), SENTINEL, np.uint16)
        Cb[:, :M] = oracle.cast_bits(C0, dtype).reshape(M, N).T
        dC = to_device_bits(Cb, Cb.shape)
        tw.set_option(tw.OPT_SHAPE, shape)
        print("skinny test: shape", shape, M, alpha, beta, pruned, with_bias, act, dtype, flush=True)
        plan.gemm(dA.data_ptr(), dC.data_ptr(), M, lda=lda, ldc=ldc, alpha=alpha, beta=beta,
                  pruned_cols=pruned, bias_ptr=dbias.data_ptr() if with_bias else None, activation=act,
                  stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return from_device_bits(dC)

    no_sum = np.ones(N, bool)                   # columns whose value does not come from a sum over k
    for t in tiles:
        if len(t["kept_k"]):
            no_sum[t["col0"] + t["kept_n"]] = False
    try:
        with tw.Plan.create(K, N, dtype, tiles, B) as plan:
            for (alpha, beta, pruned, with_bias, act) in (
                    (1.0, 0.0, tw.PRUNED_UNTOUCHED, False, tw.ACT_NONE),
                    (0.5, 0.0, tw.PRUNED_ZERO, True, tw.ACT_RELU),
                    (1.0, 0.0, tw.PRUNED_ZERO, True, tw.ACT_TANH),
                    (2.0, 0.75, tw.PRUNED_ZERO, False, tw.ACT_NONE),
                    (1.0, -0.5, tw.PRUNED_UNTOUCHED, True, tw.ACT_GELU)):
                want = launch(plan, tw.SHAPE_256x128, alpha, beta, pruned, with_bias, act)
                got = launch(plan, -1, alpha, beta, pruned, with_bias, act)     # the default: skinny
                forced = launch(plan, tw.SHAPE_SKINNY, alpha, beta, pruned, with_bias, act)
                assert np.array_equal(got, forced)
                assert np.array_equal(got[:, M:], want[:, M:])                  # padding untouched
                if act != tw.ACT_GELU:
                    assert np.array_equal(got[no_sum], want[no_sum])
                a = oracle.bits_to_f32(got[:, :M], dtype)
                b = oracle.bits_to_f32(want[:, :M], dtype)
                assert oracle.rel_error(a, b) <= 0.5 * TOL[dtype], (alpha, beta, pruned, with_bias, act)
                if not with_bias and act == tw.ACT_NONE:
                    Cf = a.reshape(N, M).T
                    ref = reference(oracle, A, B, tiles, dtype, alpha, beta, C0)
                    assert oracle.rel_error(Cf[:, keep], ref[:, keep]) <= TOL[dtype]
    finally:
        tw.set_option(tw.OPT_SHAPE, -1)


def test_skinny_kernel_many_units(tw, oracle):
    """More units than travel in the kernel arguments (40 tiles of 64 and 128 columns): the skinny
    kernel reads its unit from the plan's table in memory.  Against the oracle, the streaming
    kernel and itself."""
    rng = np.random.default_rng(909)
    M, K = 96, 700
    widths = [128, 64] * 20
    N = sum(widths)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    tiles, c0 = [], 0
    for t, w in enumerate(widths):
        kt = int(rng.integers(0, 400))
        nt = int(rng.integers(1, w + 1))
        tiles.append(dict(col0=c0, width=w,
                          kept_k=np.sort(rng.choice(K, size=kt, replace=False)).astype(np.int32),
                          kept_n=np.sort(rng.choice(w, size=nt, replace=False)).astype(np.int32)))
        c0 += w
    keep = kept_columns(tiles, N)
    ref = reference(oracle, A, B, tiles, "f16")
    try:
        with tw.Plan.create(K, N, "f16", tiles, B) as plan:
            assert plan.info()["n_tiles"] > 32
            tw.set_option(tw.OPT_SHAPE, tw.SHAPE_SKINNY)
            print("skinny, many units: launch", flush=True)
            C1, bits1 = run_gemm(tw, oracle, plan, A, "f16", N, pruned=1)
            C2, bits2 = run_gemm(tw, oracle, plan, A, "f16", N, pruned=1)
            tw.set_option(tw.OPT_SHAPE, tw.SHAPE_128x64)
            tw.set_option(tw.OPT_PIECE, 64)
            C3, _ = run_gemm(tw, oracle, plan, A, "f16", N, pruned=1)
            assert np.array_equal(bits1, bits2)
            assert oracle.rel_error(C1[:, keep], ref[:, keep]) <= TOL["f16"]
            assert oracle.rel_error(C1, C3) <= 0.5 * TOL["f16"]
            assert (C1[:, ~keep] == 0).all()
    finally:
        tw.set_option(tw.OPT_SHAPE, -1)
        tw.set_option(tw.OPT_PIECE, -1)


def test_operand_beyond_four_gib(tw, oracle):
    """A of 4.4 GiB: byte offsets into A no longer fit 32 bits, the launch falls back to the
    kernel with 64-bit addressing.  Checked on sampled rows (a row of C depends on the same row
    of A only) at both ends of M."""
    import torch
    K, N, G = 2304, 128, 128
    M = 1024 * 1000                        # K * M * 2 bytes = 4.4 GiB
    rng = np.random.default_rng(99)
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.25, n_keep=0.9)
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    dA = torch.empty((K, M), dtype=torch.float16, device="cuda")
    for k0 in range(0, K, 256):            # filled in slabs: no 2x temporary
        dA[k0:k0 + 256].normal_(generator=g)
    dC = torch.full((N, M), 7.0, dtype=torch.float16, device="cuda")
    print("4 GiB operand: launch", flush=True)
    with tw.Plan.create(K, N, "f16", tiles, B) as plan:
        plan.gemm(dA.data_ptr(), dC.data_ptr(), M, stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
    rows = np.concatenate([np.arange(0, 40), rng.integers(0, M, 60), np.arange(M - 40, M)])
    idx = torch.from_numpy(rows).cuda()
    A_rows = dA[:, idx].float().cpu().numpy().T          # [rows, K], exact fp16 values
    C_rows = dC[:, idx].float().cpu().numpy().T
    ref = oracle.tw_gemm_reference(A_rows, oracle.quantize(B, "f16"), tiles)
    keep = kept_columns(tiles, N)
    assert oracle.rel_error(C_rows[:, keep], ref[:, keep]) <= 1e-2
    assert np.all(C_rows[:, ~keep] == 7.0)               # pruned columns untouched


def test_concurrent_host_threads_and_streams(tw, oracle):
    """One immutable plan, four host threads, each launching on its own stream into its own C:
    every thread gets the single-stream result bit for bit."""
    import threading
    import torch
    rng = np.random.default_rng(111)
    M, K, N, G = 1024, 384, 512, 128
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.4, n_keep=0.9)
    At = np.ascontiguousarray(oracle.cast_bits(A, "f16").reshape(M, K).T)
    dA = to_device_bits(At, At.shape)
    with tw.Plan.create(K, N, "f16", tiles, B) as plan:
        want = torch.zeros((N, M), dtype=torch.int16, device="cuda")
        plan.gemm(dA.data_ptr(), want.data_ptr(), M, pruned_cols=tw.PRUNED_ZERO,
                  stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        outs = [torch.full((N, M), 0x1234, dtype=torch.int16, device="cuda") for _ in range(4)]
        streams = [torch.cuda.Stream() for _ in range(4)]
        errors = []

        def work(i):
            try:
                for _ in range(60):
                    plan.gemm(dA.data_ptr(), outs[i].data_ptr(), M, pruned_cols=tw.PRUNED_ZERO,
                              stream=streams[i].cuda_stream)
                streams[i].synchronize()
            except Exception as e:           # surfaced by the main thread
                errors.append(e)

        threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not errors, errors
        for o in outs:
            assert torch.equal(o, want)
