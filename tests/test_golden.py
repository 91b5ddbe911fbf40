"""The oracle against the committed fixtures of its own outputs (tests/golden/kx_golden.npz, written by
tests/golden/make_golden.py), and the GPU against the same fixtures."""
import ctypes as C
import importlib.util
import os

import numpy as np
import pytest

import oracle as O
from oracle import ptr

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = np.load(os.path.join(HERE, "golden", "kx_golden.npz"))


def test_oracle_reproduces_the_fixtures(ox):
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    now = mod.build()
    assert sorted(now) == sorted(GOLD.files)
    for k in GOLD.files:
        a, b = np.asarray(now[k]), GOLD[k]
        assert a.dtype == b.dtype and a.shape == b.shape, k
        assert (a.view(np.uint8) == b.view(np.uint8)).all(), k


@pytest.mark.gpu
def test_gpu_reproduces_the_fixtures(kxlib):
    from kxt import check, dev
    from blok_amd.lib import DevBuf
    rows, cols = 4, 1024
    dp, ds, dx = dev(GOLD["i4_packed"]), dev(GOLD["i4_scale"]), dev(GOLD["i4_x"])
    dq, dw, dy = DevBuf(rows * cols), DevBuf(rows * cols * 2), DevBuf(2 * rows * 2)
    check(kxlib.kx_i4_unpack(dp.ptr, dq.ptr, rows, cols, None))
    check(kxlib.kx_i4_dequant(dp.ptr, ds.ptr, dw.ptr, rows, cols, None))
    check(kxlib.kx_i4_gemv(dp.ptr, ds.ptr, dx.ptr, dy.ptr, rows, cols, 2, None))
    check(kxlib.kx_sync(None))
    assert (dq.to_numpy(np.int8, (rows, cols))[:, :64] == GOLD["i4_q"]).all()
    assert (dw.to_numpy(np.uint16, (rows, cols))[:, :64] == GOLD["i4_w"]).all()
    assert (dy.to_numpy(np.uint16, (2, rows)) == GOLD["i4_y_mode1"]).all()
    dl, db = dev(GOLD["router_logits"]), dev(GOLD["router_bias"])
    di, dwt = DevBuf(2 * 8 * 2), DevBuf(2 * 8 * 4)
    check(kxlib.kx_router_topk(dl.ptr, db.ptr, di.ptr, dwt.ptr, 2, 384, 8, 2.827, None))
    check(kxlib.kx_sync(None))
    assert (di.to_numpy(np.uint16, (2, 8)) == GOLD["router_ids"]).all()
    assert (dwt.to_numpy(np.uint32, (2, 8)) == GOLD["router_weights"].view(np.uint32)).all()
    cfg = O.small_config()
    tab = np.empty((4, 64), np.uint16)
    check(kxlib.kx_rope_table(C.byref(cfg), 1000, 4, ptr(tab)))
    assert (tab == GOLD["rope_rows_1000"]).all()
    cfg.heads = 4
    nbytes = C.c_size_t()
    check(kxlib.kx_mla_workspace_bytes(C.byref(cfg), 1, 8, C.byref(nbytes)))
    dc, dqa, dws, do = dev(GOLD["mla_cache"]), dev(GOLD["mla_qabs"]), DevBuf(nbytes.value), DevBuf(4 * 512 * 2)
    check(kxlib.kx_mla_decode(C.byref(cfg), dc.ptr, 8 * 576, dqa.ptr, dws.ptr, do.ptr, 1, 8, 0, None))
    check(kxlib.kx_sync(None))
    assert (do.to_numpy(np.uint16, (1, 4, 512))[:, :, :64] == GOLD["mla_o_mode1"]).all()
    cfg = O.small_config(batch=2)
    h = C.c_void_p()
    check(kxlib.kx_model_create(C.byref(cfg), C.byref(h)))
    out = np.zeros((2, 6), np.uint32); counts = np.zeros(2, np.int32)
    check(kxlib.kx_generate(h, ptr(np.ascontiguousarray(GOLD["stack_prompt"])), 2, 6, 6, 1, ptr(out), ptr(counts)))
    check(kxlib.kx_model_destroy(h))
    assert (out == GOLD["stack_ids_mode1"]).all()
