"""GPU parity of the integer pre-pass (mask -> kept lists -> relative offsets ->
compaction) and of the small boundary kernels, bit-exact against the oracle."""
import numpy as np
import pytest

from tests.helpers import from_device_bits, random_tiles, to_device_bits

pytestmark = pytest.mark.gpu


def check_export(oracle, plan, tiles, B, dtype):
    got, Bs = plan.export()
    assert len(got) == len(tiles)
    for g, t in zip(got, tiles):
        assert g["col0"] == t["col0"] and g["width"] == t["width"]
        assert np.array_equal(g["kept_k"], t["kept_k"])
        assert np.array_equal(g["kept_n"], t["kept_n"])
        # relative offsets: kept[i] - i, and the oracle's mask -> offsets routine
        assert np.array_equal(g["mask_k"], t["kept_k"] - np.arange(len(t["kept_k"])))
        assert np.array_equal(g["mask_n"], t["kept_n"] - np.arange(len(t["kept_n"])))
    K, N = B.shape
    assert np.array_equal(g["mask_k"], oracle.mask_to_offsets(
        np.isin(np.arange(K), tiles[-1]["kept_k"]).astype(np.uint8)))
    # compacted weight, reference stream layout, after the 16-bit cast: bit-exact
    expect = oracle.cast_bits(oracle.stream_weight(B, tiles), dtype)
    assert np.array_equal(Bs, expect)


@pytest.mark.parametrize("K,N,G,dtype", [(64, 128, 32, "f16"), (100, 200, 64, "bf16"),
                                         (257, 300, 128, "f16"), (768, 512, 128, "bf16"),
                                         (33, 40, 64, "f16")])
def test_plan_create_compaction_bit_exact(tw, oracle, K, N, G, dtype):
    rng = np.random.default_rng(K * 1000 + N)
    B = rng.standard_normal((K, N)).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.3, n_keep=0.8, empty_every=4)
    with tw.Plan.create(K, N, dtype, tiles, B) as plan:
        check_export(oracle, plan, tiles, B, dtype)
        inf = plan.info()
        assert inf["sum_k"] == sum(len(t["kept_k"]) for t in tiles)
        assert inf["kept_elems"] == sum(len(t["kept_k"]) * len(t["kept_n"]) for t in tiles)
        assert inf["total_width"] == N


@pytest.mark.parametrize("K,N,G,dtype", [(64, 128, 32, "f16"), (300, 520, 128, "bf16"),
                                         (1000, 77, 64, "f16"), (768, 3072, 128, "f16")])
def test_plan_from_mask_bit_exact(tw, oracle, K, N, G, dtype):
    rng = np.random.default_rng(K + N)
    B = rng.standard_normal((K, N)).astype(np.float32)
    tiles = random_tiles(rng, K, N, G, k_keep=0.25, n_keep=0.9, empty_every=5)
    mask = oracle.plan_mask(K, N, tiles)
    expect = oracle.plan_from_mask(mask, G)   # empty tiles lose their lists, as a mask cannot hold them
    with tw.Plan.from_mask(mask, G, dtype, B) as plan:
        check_export(oracle, plan, expect, B, dtype)


@pytest.mark.parametrize("name", ["vgg16_conv4_2", "imbalance_stress"])
def test_plan_from_mask_full_size_configurations(tw, oracle, name):
    """The mask -> kept lists -> relative offsets -> compaction pre-pass at the full size of the
    benchmark configurations, from the 0/1 mask of the configuration's tile table (VGG16 conv4_2:
    4608 x 512, ragged kept-row counts, 13 of 128 columns pruned a tile; imbalance stress:
    4096 x 8192, tiles of 64 columns from empty to dense): tile table, kept lists, relative offsets
    and the compacted 16-bit weight in the reference's stream layout (basic_nn.cu:697-769), bit
    for bit against the oracle on the same seed."""
    from tilesparsity_amd import workloads
    wl = workloads.vgg16_conv4_2() if name == "vgg16_conv4_2" else workloads.imbalance_stress()
    K, N, G, dtype, tiles = wl["K"], wl["N"], wl["G"], wl["dtype"], wl["tiles"]
    _, B = wl["values"]()
    mask = oracle.plan_mask(K, N, tiles)
    expect = oracle.plan_from_mask(mask, G)   # what a mask can hold: empty tiles lose their lists
    assert sum(len(t["kept_k"]) * len(t["kept_n"]) for t in expect) == int(mask.sum())
    print("full-size pre-pass:", name, K, N, G, dtype, flush=True)
    with tw.Plan.from_mask(mask, G, dtype, B) as plan:
        check_export(oracle, plan, expect, B, dtype)
        inf = plan.info()
        assert inf["kept_elems"] == int(mask.sum()) and inf["total_width"] == N


def test_plan_from_mask_rejects_non_tw_mask(tw):
    K, N, G = 64, 128, 32
    mask = np.zeros((K, N), np.uint8)
    mask[::2, :16] = 1
    mask[5, 3] = 1          # an element outside the (rows x columns) product
    mask[0, 1] = 0          # and a hole inside it
    with pytest.raises(tw.TwError) as e:
        tw.Plan.from_mask(mask, G, "f16", np.zeros((K, N), np.float32))
    assert e.value.status == tw.ERR_NOT_TW
    mask[5, 3] = 0
    mask[0, 1] = 1
    tw.Plan.from_mask(mask, G, "f16", np.zeros((K, N), np.float32)).destroy()


def test_dense_plan(tw, oracle):
    K, N, G = 96, 200, 64
    B = np.random.default_rng(9).standard_normal((K, N)).astype(np.float32)
    with tw.Plan.dense(K, N, G, "f16", B) as plan:
        tiles, Bs = plan.export()
        assert [t["width"] for t in tiles] == [64, 64, 64, 8]
        assert all(len(t["kept_k"]) == K and len(t["kept_n"]) == t["width"] for t in tiles)
        # all kept: the stream layout is simply B transposed
        assert np.array_equal(Bs.reshape(N, K), oracle.cast_bits(B.T, "f16").reshape(N, K))


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_cast_kernel_bit_exact(tw, oracle, dtype):
    import torch
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(100003) * 10.0 ** rng.integers(-8, 6, 100003)).astype(np.float32)
    x[:8] = [0.0, -0.0, np.inf, -np.inf, 65504.0, 65520.0, 1e-8, 3e-5]
    src = torch.from_numpy(x).cuda()
    dst = torch.full((x.size + 1,), 0x5555, dtype=torch.int16, device="cuda")
    tw.cast_f32(src.data_ptr(), dst.data_ptr(), x.size, dtype)
    torch.cuda.synchronize()
    got = from_device_bits(dst)
    assert np.array_equal(got[:-1], oracle.cast_bits(x, dtype))
    assert got[-1] == 0x5555    # no write past the end (the reference's bound is off by one)


def test_delete_insert_row_kernels(tw):
    import torch
    rng = np.random.default_rng(12)
    rows, cols = 300, 77
    src = rng.integers(0, 65536, (rows, cols)).astype(np.uint16)
    kept = np.sort(rng.choice(rows, 120, replace=False)).astype(np.int32)
    rel = torch.from_numpy(kept - np.arange(120, dtype=np.int32)).cuda()
    d_src = to_device_bits(src, (rows, cols))
    d_out = torch.zeros((120, cols), dtype=torch.int16, device="cuda")
    tw.delete_row(d_src.data_ptr(), d_out.data_ptr(), 120, cols, rel.data_ptr())
    d_back = torch.zeros((rows, cols), dtype=torch.int16, device="cuda")
    tw.insert_row(d_back.data_ptr(), d_out.data_ptr(), 120, cols, rel.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(from_device_bits(d_out), src[kept])
    expect = np.zeros_like(src)
    expect[kept] = src[kept]
    assert np.array_equal(from_device_bits(d_back), expect)
    # more rows than one grid dimension holds (the reference's kernels take any row count)
    rows, cols, n_keep = 70000, 9, 66000
    src = rng.integers(0, 65536, (rows, cols)).astype(np.uint16)
    kept = np.sort(rng.choice(rows, n_keep, replace=False)).astype(np.int32)
    rel = torch.from_numpy(kept - np.arange(n_keep, dtype=np.int32)).cuda()
    d_src = to_device_bits(src, (rows, cols))
    d_out = torch.zeros((n_keep, cols), dtype=torch.int16, device="cuda")
    tw.delete_row(d_src.data_ptr(), d_out.data_ptr(), n_keep, cols, rel.data_ptr())
    d_back = torch.zeros((rows, cols), dtype=torch.int16, device="cuda")
    tw.insert_row(d_back.data_ptr(), d_out.data_ptr(), n_keep, cols, rel.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(from_device_bits(d_out), src[kept])
    expect = np.zeros_like(src)
    expect[kept] = src[kept]
    assert np.array_equal(from_device_bits(d_back), expect)


def test_device_operands_give_the_same_plan(tw, oracle):
    """tw_plan_from_device_mask on device copies of the mask and the weight builds the plan the
    host entry points build: same lists, same packed weight bits; also for covering plans and
    for the masks a producer leaves on the device."""
    import torch
    from oracle import tw_prune_oracle as po
    from tilesparsity_amd import twprune
    rng = np.random.default_rng(17)
    for K, N, G in ((192, 320, 64), (300, 200, 128), (64, 64, 16)):
        W = rng.standard_normal((K, N)).astype(np.float32)
        scores = twprune.img2col_forward([W])
        dW = torch.from_numpy(W).cuda()
        table = po.tiles_every_g_columns(N, G)
        # a producer's device mask goes straight into the plan
        dmask = twprune.tiled_wise_1d(scores, 70, G, return_device=True)[0]
        print("device pre-pass", K, N, G, flush=True)
        with tw.Plan.from_device_mask(K, N, dmask.data_ptr(), table, "f16", dW.data_ptr()) as pd, \
                tw.Plan.from_mask_tiles(dmask.cpu().numpy(), table, "f16", W) as ph:
            (td, bd), (th, bh) = pd.export(), ph.export()
            assert np.array_equal(bd, bh)
            for a, b in zip(td, th):
                assert np.array_equal(a["kept_k"], b["kept_k"]) and np.array_equal(a["kept_n"], b["kept_n"])
                assert np.array_equal(a["mask_k"], b["mask_k"]) and np.array_equal(a["mask_n"], b["mask_n"])
        # an arbitrary mask: refused without cover, identical to the host path with it
        m = (rng.random((K, N)) < 0.1).astype(np.uint8)
        dm = torch.from_numpy(m).cuda()
        with pytest.raises(tw.TwError) as e:
            tw.Plan.from_device_mask(K, N, dm.data_ptr(), table, "bf16", dW.data_ptr())
        assert e.value.status == tw.ERR_NOT_TW
        with tw.Plan.from_device_mask(K, N, dm.data_ptr(), table, "bf16", dW.data_ptr(), cover=True) as pd, \
                tw.Plan.from_mask_tiles(m, table, "bf16", W, cover=True) as ph:
            (td, bd), (th, bh) = pd.export(), ph.export()
            assert np.array_equal(bd, bh)
            assert np.array_equal(bd, oracle.cast_bits(oracle.stream_weight(np.where(m != 0, W, np.float32(0)), po.cover_tiles_from_mask(m, table)), "bf16"))
        # on a stream of the caller: the mask is produced on that stream right before the build
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            dm2 = torch.zeros_like(dm)
            dm2.copy_(dm)
            with tw.Plan.from_device_mask(K, N, dm2.data_ptr(), table, "bf16", dW.data_ptr(), cover=True,
                                          stream=side.cuda_stream) as ps:
                _, bs = ps.export()
        assert np.array_equal(bs, bd)
    with pytest.raises(tw.TwError):
        tw.Plan.from_device_mask(8, 8, 0, [(0, 8)], "f16", 0)


def test_long_rows_and_wide_tiles_span_several_segments(tw, oracle):
    """Counting and compaction work on segments of 1024 flags: a mask with more rows than that,
    tiles wider than that (one of them not starting at a multiple of 16) and a narrow tile between
    them gives the oracle's lists and packed weight."""
    rng = np.random.default_rng(23)
    K, widths = 2500, [1500, 40, 2101, 7]
    N = sum(widths)
    table, tiles, c0 = [], [], 0
    for w in widths:
        kk = np.sort(rng.choice(K, int(K * 0.3), replace=False)).astype(np.int32)
        kn = np.sort(rng.choice(w, max(1, int(w * 0.7)), replace=False)).astype(np.int32)
        table.append((c0, w))
        tiles.append(dict(col0=c0, width=w, kept_k=kk, kept_n=kn))
        c0 += w
    B = rng.standard_normal((K, N)).astype(np.float32)
    mask = oracle.plan_mask(K, N, tiles)
    print("segmented pre-pass", K, N, widths, flush=True)
    with tw.Plan.from_mask_tiles(mask, table, "f16", B) as plan:
        check_export(oracle, plan, tiles, B, "f16")
    # rows kept only in the last segment, columns only in a tile's last segment
    mask2 = np.zeros((K, N), np.uint8)
    mask2[2400:2500:3, 1400:1500:2] = 1
    mask2[5, 1540 + 2090] = 1
    with tw.Plan.from_mask_tiles(mask2, table, "bf16", B) as plan:
        got, _ = plan.export()
        assert np.array_equal(got[0]["kept_k"], np.arange(2400, 2500, 3))
        assert np.array_equal(got[0]["kept_n"], np.arange(1400, 1500, 2))
        assert len(got[1]["kept_k"]) == 0 and len(got[1]["kept_n"]) == 0
        assert np.array_equal(got[2]["kept_k"], [5]) and np.array_equal(got[2]["kept_n"], [2090])
        assert np.array_equal(got[2]["mask_k"], [5]) and np.array_equal(got[2]["mask_n"], [2090])
        assert len(got[3]["kept_k"]) == 0
