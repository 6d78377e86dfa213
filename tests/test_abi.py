"""CPU-only checks of the C-ABI library: it loads, exports every declared symbol,
and its host-side logic (integer helpers, validation, error paths) behaves.  No
compute call is made here; nothing in this file needs a GPU."""
import ctypes
import os
import re

import numpy as np
import pytest

from tests.helpers import random_tiles

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "twgemm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tw_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(tw):
    names = declared_symbols()
    assert len(names) >= 18
    assert sorted(tw.EXPORTED_SYMBOLS) == names
    raw = ctypes.CDLL(tw.LIB_PATH)
    for n in names:
        assert getattr(raw, n) is not None
    assert tw.version() == 100
    assert tw.lib().tw_status_string(tw.ERR_NOT_TW) == b"mask is not tile-wise"


def test_mask_to_offsets_matches_oracle(tw, oracle):
    assert tw.mask_to_offsets([0, 1, 0, 0, 1, 1, 0, 1]).tolist() == [1, 3, 3, 4]
    rng = np.random.default_rng(0)
    for n in (0, 1, 33, 500):
        mask = (rng.random(n) < 0.3).astype(np.uint8)
        off = tw.mask_to_offsets(mask)
        assert np.array_equal(off, oracle.mask_to_offsets(mask))
        assert np.array_equal(tw.offsets_to_kept(off, n), np.flatnonzero(mask))
    with pytest.raises(tw.TwError) as e:
        tw.mask_to_offsets([0, 2, 1])
    assert e.value.status == tw.ERR_INDEX_LIST


def test_offsets_to_kept_rejects_bad_lists(tw):
    for bad, limit in (([0, -1], 10), ([5, 5], 6), ([-1], 4)):
        with pytest.raises(tw.TwError) as e:
            tw.offsets_to_kept(bad, limit)
        assert e.value.status == tw.ERR_INDEX_LIST
    assert tw.offsets_to_kept([], 0).size == 0


def test_tile_partition_matches_oracle(tw, oracle):
    for args in ((12800, 768, 768, 384, 384, 128), (12800, 3072, 768, 1536, 384, 128),
                 (64, 1000, 16, 333, 8, 128), (16, 520, 64, 200, 32, 64), (0, 128, 8, 128, 8, 128)):
        assert tw.tile_partition(*args) == oracle.tile_partition(*args)
    # beyond the reference's 32-tile cap
    assert tw.tile_partition(8, 8192, 8, 8192, 8, 64)["block_num"] == 128
    for bad in ((8, 100, 8, 200, 8, 128), (8, 100, 8, 0, 8, 128), (8, 100, 8, 50, 9, 128),
                (8, 250, 8, 250, 8, 128)):
        with pytest.raises(tw.TwError) as e:
            tw.tile_partition(*bad)
        assert e.value.status == tw.ERR_SHAPE
    with pytest.raises(tw.TwError) as e:
        tw.tile_partition(8, 8192, 8, 8192, 8, 64, max_tiles=16)
    assert e.value.status == tw.ERR_BUFFER


def test_plan_create_validation_errors(tw):
    """Every rejection happens before the first HIP call, so it runs without a GPU."""
    rng = np.random.default_rng(1)
    K, N, G = 16, 48, 16
    B = np.zeros((K, N), np.float32)
    good = random_tiles(rng, K, N, G, k_keep=0.5, n_keep=0.5)

    def expect(status, tiles=None, K_=K, N_=N, dtype="f16"):
        with pytest.raises(tw.TwError) as e:
            tw.Plan.create(K_, N_, dtype, good if tiles is None else tiles, B)
        assert e.value.status == status, e.value

    gap = [dict(t) for t in good]
    gap[1]["col0"] += 1
    expect(tw.ERR_TILE_TABLE, gap)
    expect(tw.ERR_TILE_TABLE, good[:2])                       # does not reach N
    over = [dict(t) for t in good]
    over[2]["width"] += 8
    expect(tw.ERR_TILE_TABLE, over)
    unsorted = [dict(t) for t in good]
    unsorted[0]["kept_k"] = np.array([3, 2], np.int32)
    expect(tw.ERR_INDEX_LIST, unsorted)
    dup = [dict(t) for t in good]
    dup[0]["kept_n"] = np.array([1, 1], np.int32)
    expect(tw.ERR_INDEX_LIST, dup)
    oob = [dict(t) for t in good]
    oob[0]["kept_k"] = np.array([0, K], np.int32)
    expect(tw.ERR_INDEX_LIST, oob)
    oobn = [dict(t) for t in good]
    oobn[1]["kept_n"] = np.array([G], np.int32)
    expect(tw.ERR_INDEX_LIST, oobn)
    expect(tw.ERR_DTYPE, dtype="f32")
    L = tw.lib()
    h = ctypes.c_void_p()
    assert L.tw_plan_create(K, N, 0, 0, None, None, None, None, None, None, None,
                            ctypes.byref(h)) == tw.ERR_SHAPE
    assert L.tw_plan_create(K, N, 0, 3, None, None, None, None, None, None, None,
                            ctypes.byref(h)) == tw.ERR_NULL
    assert L.tw_plan_create(K, N, 0, 3, None, None, None, None, None, None, None, None) == tw.ERR_NULL
    assert b"NULL" in L.tw_last_error()
    assert L.tw_plan_create_dense(0, N, G, 0, None, ctypes.byref(h)) == tw.ERR_SHAPE
    assert L.tw_plan_from_mask(K, N, 0, 0, None, None, ctypes.byref(h)) == tw.ERR_SHAPE
    assert L.tw_plan_from_mask(K, N, G, 0, None, None, ctypes.byref(h)) == tw.ERR_NULL
    assert L.tw_plan_from_mask(K, N, G, 7, None, None, ctypes.byref(h)) == tw.ERR_DTYPE


def test_gemm_and_small_entry_points_reject_bad_arguments(tw):
    L = tw.lib()
    assert L.tw_gemm(None, None, 0, 8, None, 0, 8, 8, 1.0, 0.0, 0, None) == tw.ERR_NULL
    assert L.tw_plan_info(None, None, 0) == tw.ERR_NULL
    assert L.tw_plan_export(None, *([None] * 9)) == tw.ERR_NULL
    assert L.tw_plan_destroy(None) == tw.OK
    assert L.tw_cast_f32(None, None, 4, 9, None) == tw.ERR_DTYPE
    assert L.tw_cast_f32(None, None, -1, 0, None) == tw.ERR_SHAPE
    assert L.tw_cast_f32(None, None, 0, 0, None) == tw.OK
    assert L.tw_cast_f32(None, None, 4, 0, None) == tw.ERR_NULL
    assert L.tw_delete_row(None, None, 4, 4, None, None) == tw.ERR_NULL
    assert L.tw_insert_row(None, None, -1, 4, None, None) == tw.ERR_SHAPE
    assert L.tw_stream_gemm_nn(8, 8, 8, 5, 1.0, None, None, 0.0, None, 1, None, None, None, None,
                               None, None, None) == tw.ERR_DTYPE
    assert L.tw_stream_gemm_nn(8, 8, 8, 0, 1.0, None, None, 0.0, None, 1, None, None, None, None,
                               None, None, None) == tw.ERR_NULL
