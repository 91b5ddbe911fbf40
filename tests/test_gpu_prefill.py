"""GPU parity of the prefill chunk path (W4A16 grouped GEMM on the matrix cores, BASELINE config 4).

Routing (ids, weights, bucketing) is bit-exact against the oracle given the GPU's own router logits;
the layer output is within max-rel 1e-2 of the oracle's per-token reference schedule run with that
routing (MFMA's internal summation order is not documented, so no bit-exact claim is made here).
"""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from kxt import check, dev, moe_case, moe_cfg, moe_device_weights, moe_oracle_weights, say
from oracle import ptr

pytestmark = pytest.mark.gpu
from blok_amd.lib import DevBuf  # noqa: E402


def _zipf_bias(E, seed, c=0.1):
    """noaux bias plus c*ln(1/rank): a roughly Zipf-skewed expert load"""
    return (O.normal_f32(E, seed, 11, 0.01) + c * np.log(1.0 / np.arange(1, E + 1))).astype(np.float32)


def _prefill(kxlib, ox, H, I, SI, E, K, T, seed, sample=None):
    host, n, x = moe_case(kxlib, H, I, SI, E, K, T, seed)
    host["router_bias"] = _zipf_bias(E, seed)
    cfg = moe_cfg(H, I, SI, E, K)
    w, bufs = moe_device_weights(host)
    ws = C.c_void_p()
    check(kxlib.kx_moe_workspace_create(C.byref(cfg), T, C.byref(ws)))
    dn, dx = dev(n), dev(x)
    check(kxlib.kx_moe_prefill_layer(C.byref(cfg), C.byref(w), ws, dn.ptr, dx.ptr, T, 0, None))
    check(kxlib.kx_sync(None))
    got = dx.to_numpy(np.uint16, (T, H))
    views = [C.c_void_p() for _ in range(8)]
    check(kxlib.kx_moe_workspace_views(ws, *[C.byref(v) for v in views]))
    tmp = DevBuf.__new__(DevBuf)
    def grab(v, dtype, shape):
        tmp.ptr, tmp.nbytes = v.value, int(np.prod(shape)) * np.dtype(dtype).itemsize
        return tmp.to_numpy(dtype, shape)
    logits = grab(views[0], np.float32, (T, E))
    ids = grab(views[1], np.uint16, (T, K))
    wts = grab(views[2], np.float32, (T, K))
    counts = grab(views[3], np.int32, (E,))
    tmp.ptr = None
    check(kxlib.kx_moe_workspace_destroy(ws))
    # routing: bit-exact given the same logits
    ids1, w1 = np.empty_like(ids), np.empty_like(wts)
    ox.ox_router_topk(ptr(logits), ptr(host["router_bias"]), ptr(ids1), ptr(w1), T, E, K, 2.827, 1)
    assert (ids == ids1).all() and (wts.view(np.uint32) == w1.view(np.uint32)).all()
    assert counts.sum() == T * K
    # expert arithmetic: per-token reference schedule with that routing, on all tokens or a sample
    sel = np.arange(T) if sample is None else np.sort(np.random.default_rng(seed).choice(T, sample, replace=False))
    xo = np.ascontiguousarray(x[sel])
    ns, idss, wtss = np.ascontiguousarray(n[sel]), np.ascontiguousarray(ids[sel]), np.ascontiguousarray(wts[sel])
    wo = moe_oracle_weights(host)
    ox.ox_moe_layer_routed(C.byref(wo), ptr(ns), ptr(xo), len(sel), H, I, SI, E, K, 0, 0, ptr(idss), ptr(wtss))
    err = O.max_rel(O.bf16_to_f32(got[sel]), O.bf16_to_f32(xo))
    print(f"prefill T={T}: max-rel {err:.3e} over {len(sel)} tokens; busiest expert {counts.max()} tokens, "
          f"{np.count_nonzero(counts)} experts used")
    assert err < 1e-2, err
    return counts


@pytest.mark.parametrize("T", [1, 37, 300])
def test_prefill_small_shape(kxlib, ox, T):
    say(f"prefill small T={T}")
    _prefill(kxlib, ox, 1024, 1024, 512, 32, 4, T, 21)


def test_prefill_kimi_shape_chunk(kxlib, ox):
    # BASELINE config 4: 2048 tokens, 384 experts top-8, Zipf-skewed load; a sample of tokens is checked
    say("prefill kimi shape T=2048")
    counts = _prefill(kxlib, ox, 7168, 2048, 2048, 384, 8, 2048, 22, sample=24)
    assert counts.max() > 4 * counts[counts > 0].mean() or counts.max() > 200   # the load is skewed
