"""GPU parity of the router, the bucketing and one routed-MoE decode layer.

Bars: expert ids, bucketing and (kx schedule) every tensor of the layer are
bit-exact; against the reference schedule the layer output is within max-rel 1e-2.
"""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from kxt import (NEAR_TIE, check, dev, moe_case, moe_cfg, moe_device_weights, moe_oracle_weights, say)
from oracle import ptr

pytestmark = pytest.mark.gpu
from blok_amd.lib import DevBuf  # noqa: E402


def _router(kxlib, logits, bias, topk, scale=2.827):
    T, E = logits.shape
    dl, db = dev(logits), dev(bias)
    di, dw = DevBuf(T * topk * 2), DevBuf(T * topk * 4)
    check(kxlib.kx_router_topk(dl.ptr, db.ptr, di.ptr, dw.ptr, T, E, topk, scale, None))
    check(kxlib.kx_sync(None))
    return di.to_numpy(np.uint16, (T, topk)), dw.to_numpy(np.float32, (T, topk))


@pytest.mark.parametrize("T,E,topk", [(1, 384, 8), (64, 384, 8), (5, 16, 4), (3, 1000, 8), (2, 8, 8)])
def test_router_topk_bit_exact(kxlib, ox, T, E, topk):
    say(f"router T={T} E={E} topk={topk}")
    logits = O.normal_f32(T * E, 5, 1, 1.0).reshape(T, E)
    bias = O.normal_f32(E, 5, 2, 0.01)
    ids, w = _router(kxlib, logits, bias, topk)
    ids1, w1 = np.empty_like(ids), np.empty_like(w)
    ox.ox_router_topk(ptr(logits), ptr(bias), ptr(ids1), ptr(w1), T, E, topk, 2.827, 1)
    assert (ids == ids1).all()
    assert (w.view(np.uint32) == w1.view(np.uint32)).all()
    ids0, w0 = np.empty_like(ids), np.empty_like(w)
    ox.ox_router_topk(ptr(logits), ptr(bias), ptr(ids0), ptr(w0), T, E, topk, 2.827, 0)
    assert (ids == ids0).all()
    assert np.allclose(w, w0, rtol=1e-5)


def test_router_ties_take_lowest_index(kxlib, ox):
    E, topk = 384, 8
    logits = np.zeros((3, E), dtype=np.float32)          # every score equal
    logits[1, 100:110] = 2.0                              # ten equal winners, eight slots
    logits[2, ::7] = 1.0
    bias = np.zeros(E, dtype=np.float32)
    ids, w = _router(kxlib, logits, bias, topk)
    assert ids[0].tolist() == list(range(8))
    assert ids[1].tolist() == list(range(100, 108))
    assert ids[2].tolist() == [0, 7, 14, 21, 28, 35, 42, 49]
    ids1, w1 = np.empty_like(ids), np.empty_like(w)
    ox.ox_router_topk(ptr(logits), ptr(bias), ptr(ids1), ptr(w1), 3, E, topk, 2.827, 1)
    assert (ids == ids1).all() and (w.view(np.uint32) == w1.view(np.uint32)).all()


@pytest.mark.parametrize("T,E,topk", [(1, 384, 8), (8, 384, 8), (64, 384, 8), (2048, 384, 8), (7, 16, 4), (301, 384, 8), (259, 16, 4)])
def test_bucket_bit_exact(kxlib, ox, T, E, topk):
    say(f"bucket T={T} E={E} topk={topk}")
    logits = O.normal_f32(T * E, 6, 1, 1.0).reshape(T, E)
    bias = O.normal_f32(E, 6, 2, 0.01)
    ids = np.empty((T, topk), dtype=np.uint16)
    wts = np.empty((T, topk), dtype=np.float32)
    ox.ox_router_topk(ptr(logits), ptr(bias), ptr(ids), ptr(wts), T, E, topk, 2.827, 1)
    di = dev(ids)
    dc, do, dp, da, dn = DevBuf(E * 4), DevBuf((E + 1) * 4), DevBuf(T * topk * 4), DevBuf(E * 16), DevBuf(4)
    check(kxlib.kx_bucket(di.ptr, T, E, topk, dc.ptr, do.ptr, dp.ptr, da.ptr, dn.ptr, None))
    check(kxlib.kx_sync(None))
    counts = np.empty(E, dtype=np.int32)
    offsets = np.empty(E + 1, dtype=np.int32)
    pairs = np.empty(T * topk, dtype=np.int32)
    active = np.empty(E, dtype=np.int32)
    na = ox.ox_bucket(ptr(ids), T, E, topk, ptr(counts), ptr(offsets), ptr(pairs), ptr(active))
    assert (dc.to_numpy(np.int32, (E,)) == counts).all()
    assert (do.to_numpy(np.int32, (E + 1,)) == offsets).all()
    assert (dp.to_numpy(np.int32, (T * topk,)) == pairs).all()
    assert dn.to_numpy(np.int32, (1,))[0] == na
    work = da.to_numpy(np.int32, (E, 4))
    act = active[:na]
    assert (work[:na, 0] == act).all()
    assert (work[:na, 1] == offsets[act]).all() and (work[:na, 2] == offsets[act + 1]).all()
    assert (work[:na, 3] == pairs[offsets[act]]).all()
    assert (work[na:] == np.array([-1, 0, 0, 0])).all()


def _run_layer(kxlib, ox, H, I, SI, E, K, T, seed, flags=0, gpu_flags=0, mode0_tokens=None):
    """One layer on the GPU and through both oracle schedules.  mode0_tokens: run the (slower) reference schedule on
    these token rows only (tokens do not interact); its tensors then hold those rows."""
    host, n, x = moe_case(kxlib, H, I, SI, E, K, T, seed)
    cfg = moe_cfg(H, I, SI, E, K)
    w, bufs = moe_device_weights(host)
    ws = C.c_void_p()
    check(kxlib.kx_moe_workspace_create(C.byref(cfg), T, C.byref(ws)))
    dn, dx = dev(n), dev(x)
    check(kxlib.kx_moe_decode_layer(C.byref(cfg), C.byref(w), ws, dn.ptr, dx.ptr, T, flags | gpu_flags, None))
    check(kxlib.kx_sync(None))
    views = [C.c_void_p() for _ in range(8)]
    check(kxlib.kx_moe_workspace_views(ws, *[C.byref(v) for v in views]))
    got = {"x": dx.to_numpy(np.uint16, (T, H))}
    tmp = DevBuf.__new__(DevBuf)
    def grab(v, dtype, shape):
        tmp.ptr, tmp.nbytes = v.value, int(np.prod(shape)) * np.dtype(dtype).itemsize
        return tmp.to_numpy(dtype, shape)
    got["logits"] = grab(views[0], np.float32, (T, E))
    got["ids"] = grab(views[1], np.uint16, (T, K))
    got["weights"] = grab(views[2], np.float32, (T, K))
    got["mid"] = grab(views[6], np.uint16, (T * K, I))
    got["eout"] = grab(views[7], np.uint16, (T * K, H))
    # the bucketing the layer's own routing launch did (for up to 32 tokens with more than 64 pairs: by bit masks per
    # expert), against the oracle's on the same ids
    counts, offsets, pairs = np.empty(E, np.int32), np.empty(E + 1, np.int32), np.empty(T * K, np.int32)
    active = np.empty(E, np.int32)
    ids = np.ascontiguousarray(got["ids"])
    ox.ox_bucket(ptr(ids), T, E, K, ptr(counts), ptr(offsets), ptr(pairs), ptr(active))
    assert (grab(views[3], np.int32, (E,)) == counts).all(), "expert counts of the layer's routing differ"
    assert (grab(views[4], np.int32, (E + 1,)) == offsets).all(), "expert offsets of the layer's routing differ"
    assert (grab(views[5], np.int32, (T * K,)) == pairs).all(), "sorted pairs of the layer's routing differ"
    tmp.ptr = None
    check(kxlib.kx_moe_workspace_destroy(ws))
    exp = {}
    for mode in (1, 0):
        rows = np.arange(T) if (mode == 1 or mode0_tokens is None) else np.asarray(mode0_tokens)
        Tm = len(rows)
        xo, nm = np.ascontiguousarray(x[rows]), np.ascontiguousarray(n[rows])
        o = {"logits": np.empty((Tm, E), np.float32), "ids": np.empty((Tm, K), np.uint16),
             "weights": np.empty((Tm, K), np.float32), "mid": np.empty((Tm * K, I), np.uint16),
             "eout": np.empty((Tm * K, H), np.uint16)}
        wo = moe_oracle_weights(host)
        ox.ox_moe_layer(C.byref(wo), ptr(nm), ptr(xo), Tm, H, I, SI, E, K, 2.827, flags, mode,
                        ptr(o["logits"]), ptr(o["ids"]), ptr(o["weights"]), ptr(o["mid"]), ptr(o["eout"]))
        o["x"], o["rows"] = xo, rows
        exp[mode] = o
    exp["bias"] = host["router_bias"]
    return got, exp


def _assert_layer(got, exp):
    e1, e0 = exp[1], exp[0]
    assert (got["logits"].view(np.uint32) == e1["logits"].view(np.uint32)).all(), "router logits differ (kx schedule)"
    assert (got["ids"] == e1["ids"]).all(), "expert ids differ"
    assert (got["weights"].view(np.uint32) == e1["weights"].view(np.uint32)).all()
    assert (got["mid"] == e1["mid"]).all(), f"{np.count_nonzero(got['mid'] != e1['mid'])} mid values differ"
    assert (got["eout"] == e1["eout"]).all()
    assert (got["x"] == e1["x"]).all()
    rows = e0["rows"]
    K, I = got["ids"].shape[1], got["mid"].shape[1]
    same = (e0["ids"] == e1["ids"][rows]).all(axis=1)   # tokens with the same experts under both schedules: compare values
    # a token the reference schedule routes differently must sit on a near-tie of the selection: the gap between the
    # K-th and the (K+1)-th score, sigmoid(logit) + bias, of the kx schedule is then below NEAR_TIE -- checked per token
    score = np.sort(1.0 / (1.0 + np.exp(-e1["logits"][rows].astype(np.float64))) + exp["bias"].astype(np.float64), axis=1)
    gap = score[:, -K] - score[:, -K - 1]
    for t in np.flatnonzero(~same):
        assert gap[t] < NEAR_TIE, f"token {rows[t]}: the two oracle schedules pick different experts at a selection gap of {gap[t]:.2e}"
    if not same.all():
        print(f"tokens routed differently by the reference schedule, all on near-ties: {[(int(rows[t]), float('%.1e' % gap[t])) for t in np.flatnonzero(~same)]}", flush=True)
    assert same.any()
    gx, gm = O.bf16_to_f32(got["x"][rows][same]), O.bf16_to_f32(got["mid"].reshape(-1, K, I)[rows][same])
    rx, rm = O.bf16_to_f32(e0["x"][same]), O.bf16_to_f32(e0["mid"].reshape(-1, K, I)[same])
    errs = (O.max_rel(gx, rx), O.elem_err(gx, rx), O.max_rel(gm, rm), O.elem_err(gm, rm))
    print("vs reference schedule: x max-rel %.2e elem %.2e, mid max-rel %.2e elem %.2e" % errs, flush=True)
    # 1e-2 on the normalised maximum (the bar BASELINE states); the element-wise figure is held to 2e-2: one bf16
    # step is up to 2^-7 of a value's own size, and mid = bf(bf(silu(g)) * u) passes three roundings whose boundary
    # cases fall differently under another summation order
    assert max(errs[0], errs[2]) < 1e-2 and max(errs[1], errs[3]) < 2e-2


@pytest.mark.parametrize("T", [1, 8, 23, 32, 64])
def test_moe_layer_small_shape(kxlib, ox, T):
    say(f"moe layer small T={T}")
    got, exp = _run_layer(kxlib, ox, 1024, 1024, 512, 32, 4, T, 7)
    _assert_layer(got, exp)


def test_moe_layer_flags_write_down_only(kxlib, ox):
    got, exp = _run_layer(kxlib, ox, 1024, 1024, 512, 16, 8, 3, 8, flags=1)
    _assert_layer(got, exp)


@pytest.mark.parametrize("T", [1, 8, 64])
def test_moe_layer_kimi_shape(kxlib, ox, T):
    # BASELINE config 2: hidden 7168, 384 experts top-8, moe_inter 2048, shared 2048.  T = 64 (512 pairs on 384
    # experts) takes the two-launch plan: experts with one pair through the one-token kernel, the others two tokens
    # per pass.  Every tensor to the bit against the kx schedule for all tokens; the reference schedule (about four
    # times the CPU time) on eight of the 64 tokens.
    say(f"moe layer kimi shape T={T}")
    got, exp = _run_layer(kxlib, ox, 7168, 2048, 2048, 384, 8, T, 9, mode0_tokens=None if T <= 8 else range(3, 64, 8))
    _assert_layer(got, exp)


@pytest.mark.parametrize("T,bits", [(16, 0x600), (32, 0x600), (32, 0x200), (32, 0x400), (7, 0x600), (48, 0x400), (64, 0x600)])
def test_moe_layer_kimi_shape_matrix_core_forms(kxlib, ox, T, bits):
    _matrix_core_forms(kxlib, ox, T, bits, ())


def test_moe_layer_kimi_shape_matrix_core_forms_with_every_token_on_two_experts(kxlib, ox):
    # 48 tokens that all select experts 5 and 200 (a large router bias): 48 pairs on each, more than the 32 tokens of
    # one pass of the kernel that takes the experts of several pairs from 32 tokens on -- two passes, the second with 16
    _matrix_core_forms(kxlib, ox, 48, 0x400, (5, 200))


def _matrix_core_forms(kxlib, ox, T, bits, hot):
    # What the stack runs from 5 (bit 9: shared expert as bf16 matrix-core products) and 12 sequences on (bit 10:
    # routed experts with several pairs as W4A16 grouped GEMMs -- from 32 tokens on through the kernel that dequantizes
    # in registers and multiplies in f16 --, the others through the one-token GEMV kernel), reached
    # through the C ABI.  The layer output `down` (flag bit 0: no residual, so the bar is on the layer's own result):
    # within 1e-2 as normalised maximum (2e-2 element-wise: see _assert_layer) of the default GEMV form for every token, and of the
    # oracle's reference schedule given the GPU's routing on a sample of tokens; the routing itself must be the
    # default's to the bit (neither bit touches the router).
    say(f"moe layer kimi shape T={T} flags={bits:#x}")
    H, I, SI, E, K = 7168, 2048, 2048, 384, 8
    host, n, x = moe_case(kxlib, H, I, SI, E, K, T, 9)
    if hot:
        host = dict(host)   # the cached case stays as it is
        host["router_bias"] = host["router_bias"].copy()
        host["router_bias"][list(hot)] += 10.0
    cfg = moe_cfg(H, I, SI, E, K)
    w, bufs = moe_device_weights(host)
    ws = C.c_void_p()
    check(kxlib.kx_moe_workspace_create(C.byref(cfg), T, C.byref(ws)))
    dn = dev(n)
    res = {}
    for flags in (1, 1 | bits):
        dx = dev(x)
        check(kxlib.kx_moe_decode_layer(C.byref(cfg), C.byref(w), ws, dn.ptr, dx.ptr, T, flags, None))
        check(kxlib.kx_sync(None))
        views = [C.c_void_p() for _ in range(8)]
        check(kxlib.kx_moe_workspace_views(ws, *[C.byref(v) for v in views]))
        tmp = DevBuf.__new__(DevBuf)
        tmp.ptr, tmp.nbytes = views[1].value, T * K * 2
        ids = tmp.to_numpy(np.uint16, (T, K))
        tmp.ptr, tmp.nbytes = views[2].value, T * K * 4
        wts = tmp.to_numpy(np.float32, (T, K))
        tmp.ptr = None
        res[flags] = (O.bf16_to_f32(dx.to_numpy(np.uint16, (T, H))), ids, wts)
    check(kxlib.kx_moe_workspace_destroy(ws))
    (d0, ids0, w0), (d1, ids1, w1) = res[1], res[1 | bits]
    assert (ids0 == ids1).all() and (w0.view(np.uint32) == w1.view(np.uint32)).all()
    pairs = np.bincount(ids0.ravel(), minlength=E)
    for e in hot:
        assert pairs[e] == T, f"expert {e} was meant to be selected by every token, has {pairs[e]} pairs"
    e_max, e_el = O.max_rel(d1, d0), O.elem_err(d1, d0)
    print(f"{(pairs > 0).sum()} experts, {(pairs > 1).sum()} with several pairs (most: {pairs.max()}); "
          f"vs the GEMV form: max-rel {e_max:.2e}, element-wise {e_el:.2e}", flush=True)
    assert e_max < 1e-2 and e_el < 2e-2
    rows = np.arange(T)[:: max(1, T // 6)]
    xo, no = np.ascontiguousarray(x[rows]), np.ascontiguousarray(n[rows])
    io, wr = np.ascontiguousarray(ids1[rows]), np.ascontiguousarray(w1[rows])
    wo = moe_oracle_weights(host)
    ox.ox_moe_layer_routed(C.byref(wo), ptr(no), ptr(xo), len(rows), H, I, SI, E, K, 1, 0, ptr(io), ptr(wr))
    ref = O.bf16_to_f32(xo)
    r_max, r_el = O.max_rel(d1[rows], ref), O.elem_err(d1[rows], ref)
    print(f"vs the reference schedule on tokens {rows.tolist()}: max-rel {r_max:.2e}, element-wise {r_el:.2e}", flush=True)
    assert r_max < 1e-2 and r_el < 2e-2


@pytest.mark.parametrize("flags,gpu_flags", [(0, 0x100), (1, 0), (1, 0x100)])
def test_moe_layer_kimi_shape_one_token_tail(kxlib, ox, flags, gpu_flags):
    # one token: by default the routed down launch also runs the shared expert's down GEMV and combines (bit 8 of
    # the flags keeps them a launch of their own); both forms, with and without the residual add, against the oracle
    say(f"moe layer kimi shape T=1 flags={flags} gpu_flags={gpu_flags:#x}")
    got, exp = _run_layer(kxlib, ox, 7168, 2048, 2048, 384, 8, 1, 10, flags=flags, gpu_flags=gpu_flags)
    _assert_layer(got, exp)


def test_moe_errors(kxlib):
    cfg = moe_cfg(1000, 1024, 512, 16, 4)
    ws = C.c_void_p()
    assert kxlib.kx_moe_workspace_create(C.byref(cfg), 4, C.byref(ws)) != 0
    assert b"hidden" in kxlib.kx_last_error()
    cfg = moe_cfg(1024, 1024, 512, 16, 4)
    check(kxlib.kx_moe_workspace_create(C.byref(cfg), 4, C.byref(ws)))
    from blok_amd.lib import KxMoeWeights
    w = KxMoeWeights()
    b = DevBuf(64)
    assert kxlib.kx_moe_decode_layer(C.byref(cfg), C.byref(w), ws, b.ptr, b.ptr, 5, 0, None) != 0
    assert b"tokens" in kxlib.kx_last_error()
    check(kxlib.kx_moe_workspace_destroy(ws))
