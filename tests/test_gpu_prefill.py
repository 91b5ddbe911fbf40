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


def _check_expert(ox, host, n, ids, eout, e, H, I, K, what):
    """Every (token, slot) pair of expert e: the GPU's expert output row against the oracle's reference schedule
    (mode 0: per-weight dequant, 256-thread tree) of gate/up GEMV, SwiGLU, down GEMV on that token."""
    toks, slots = np.nonzero(ids == e)
    assert len(toks), f"expert {e} has no token"
    per = I * H // 8
    gp, gs = host["gate_packed"][e * per:(e + 1) * per], host["gate_scale"][e * per // 4:(e + 1) * per // 4]
    up, us = host["up_packed"][e * per:(e + 1) * per], host["up_scale"][e * per // 4:(e + 1) * per // 4]
    dp, ds = host["down_packed"][e * per:(e + 1) * per], host["down_scale"][e * per // 4:(e + 1) * per // 4]
    xs = np.ascontiguousarray(n[toks])
    g, u = np.empty((len(toks), I), dtype=np.uint16), np.empty((len(toks), I), dtype=np.uint16)
    ox.ox_i4_gemv(ptr(gp), ptr(gs), ptr(xs), ptr(g), I, H, len(toks), 0)
    ox.ox_i4_gemv(ptr(up), ptr(us), ptr(xs), ptr(u), I, H, len(toks), 0)
    gf, uf = O.bf16_to_f32(g), O.bf16_to_f32(u)
    silu = O.bf16_to_f32(O.f32_to_bf16(gf / (1.0 + np.exp(-gf))))               # :255 (libm exp in float32)
    mid = O.f32_to_bf16(silu * uf)
    y = np.empty((len(toks), H), dtype=np.uint16)
    ox.ox_i4_gemv(ptr(dp), ptr(ds), ptr(mid), ptr(y), H, I, len(toks), 0)
    got = O.bf16_to_f32(eout[toks * K + slots])
    exp = O.bf16_to_f32(y)
    errs = np.abs(got.astype(np.float64) - exp).max(axis=1) / np.abs(exp).max(axis=1)
    print(f"expert {e} ({what}): {len(toks)} tokens, expert output rows max-rel worst {errs.max():.3e}", flush=True)
    assert errs.max() < 1e-2, f"expert {e} ({what}): token {toks[int(errs.argmax())]} max-rel {errs.max():.3e}"
    return len(toks)


def _prefill(kxlib, ox, H, I, SI, E, K, T, seed, sample=None, bias=None, detail=False):
    host, n, x = moe_case(kxlib, H, I, SI, E, K, T, seed)
    host = dict(host)
    host["router_bias"] = _zipf_bias(E, seed) if bias is None else bias
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
    eout = grab(views[7], np.uint16, (T * K, H)) if detail else None
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
    if detail:
        return counts, host, n, ids, eout
    return counts


@pytest.mark.parametrize("T", [1, 37, 300])
def test_prefill_small_shape(kxlib, ox, T):
    say(f"prefill small T={T}")
    _prefill(kxlib, ox, 1024, 1024, 512, 32, 4, T, 21)


def _m_bucket(count):
    """the token-tile class of an expert in the grouped GEMM: 32-token blocks of its last 128-token tile, and
    whether it has more than one tile"""
    last = (count - 1) % 128 + 1
    return ((last + 31) // 32, count > 128)


def test_prefill_kimi_shape_chunk(kxlib, ox):
    # BASELINE config 4: 2048 tokens, 384 experts top-8, Zipf-skewed load.  The grouped GEMM's work depends on an
    # expert's token count (128-token tiles whose K loop is specialised on the number of 32-token blocks), so besides
    # a random sample of tokens (whole layer output) the experts themselves are checked, every token of each: the
    # busiest expert (nine full tiles and a remainder), the expert whose count lies closest above a tile edge, one
    # expert per block count of a single tile that the routing offers, and three single-token experts.
    say("prefill kimi shape T=2048")
    H, I, K = 7168, 2048, 8
    counts, host, n, ids, eout = _prefill(kxlib, ox, H, I, 2048, 384, K, 2048, 22, sample=24, detail=True)
    assert counts.max() > 4 * counts[counts > 0].mean() or counts.max() > 200   # the load is skewed
    chosen = {int(counts.argmax()): "busiest"}
    over = [(int(c) % 128, e) for e, c in enumerate(counts) if c > 128 and e not in chosen]
    if over:
        chosen[min(over)[1]] = "closest above a tile edge"
    for blocks in (1, 2, 3, 4):
        for e, c in enumerate(counts):
            if 1 < c <= 128 and _m_bucket(int(c))[0] == blocks and e not in chosen:
                chosen[e] = f"single tile of {blocks} block(s)"
                break
    for e in np.nonzero(counts == 1)[0][:3]:
        chosen[int(e)] = "one token"
    buckets = set()
    for e, what in chosen.items():
        got = _check_expert(ox, host, n, ids, eout, e, H, I, K, what)
        assert got == counts[e]
        buckets.add(_m_bucket(got))
    print(f"experts checked in full: {len(chosen)}, tile classes covered: {sorted(buckets)}", flush=True)
    assert len(buckets) >= 3 and any(counts[e] == 1 for e in chosen) and any(counts[e] > 256 for e in chosen)


@pytest.mark.parametrize("T", [128, 129, 33])
def test_prefill_kimi_shape_tile_edges(kxlib, ox, T):
    # exact tile edges at Kimi shape: a bias of +4 makes every token select expert 5, so that expert has exactly T
    # tokens -- one full 128-token tile, a full tile plus a one-token tile, one tile of two blocks with one token in
    # the second.  Every token of that expert is checked, and the whole layer output of every token.
    say(f"prefill kimi shape, forced expert, T={T}")
    H, I, K, E = 7168, 2048, 8, 384
    bias = O.normal_f32(E, 22, 11, 0.01)
    bias[5] += 4.0
    counts, host, n, ids, eout = _prefill(kxlib, ox, H, I, 2048, E, K, T, 22, bias=bias, detail=True)
    assert counts[5] == T
    _check_expert(ox, host, n, ids, eout, 5, H, I, K, f"all {T} tokens")
