"""Pins the rest of the oracle (exp, bf16 rounding, RMSNorm, bf16 matvec, router, bucketing, generator,
MoE layer composition) against what the mathematics fixes.  Reference: src/kimi_exec.cu:240-298, :372-407."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from oracle import ptr


def test_bf16_rounding_is_nearest_even(ox):
    cases = {0x3F800000: 0x3F80, 0x3F808000: 0x3F80, 0x3F818000: 0x3F82, 0x3F808001: 0x3F81,
             0x3F80FFFF: 0x3F81, 0xBF808000: 0xBF80, 0x7F7FFFFF: 0x7F80, 0x00000000: 0x0000, 0x80000000: 0x8000}
    for bits, want in cases.items():
        f = np.array([bits], dtype=np.uint32).view(np.float32)[0]
        assert ox.ox_bf16(C.c_float(f)) == want, hex(bits)
    f = O.normal_f32(200000, 1, 1, 3.0)
    got = np.array([ox.ox_bf16(C.c_float(v)) for v in f[:5000]], dtype=np.uint16)
    assert (got == O.f32_to_bf16(f[:5000])).all()


def test_exp_kx_within_2_ulp_of_libm(ox):
    xs = np.concatenate([np.linspace(-103.0, 88.5, 40001), np.linspace(-1, 1, 20001), [0.0, -0.0]]).astype(np.float32)
    got = np.array([ox.ox_expf(C.c_float(x), 1) for x in xs], dtype=np.float32)
    want = np.exp(xs.astype(np.float64))
    normal = want > 1.2e-38
    rel = np.abs(got[normal].astype(np.float64) - want[normal]) / want[normal]
    assert rel.max() < 2.5e-7, rel.max()          # 2 ulp of binary32
    assert ox.ox_expf(C.c_float(0.0), 1) == 1.0
    assert ox.ox_expf(C.c_float(-200.0), 1) == 0.0 and np.isinf(ox.ox_expf(C.c_float(100.0), 1))
    assert ox.ox_expf(C.c_float(float("-inf")), 1) == 0.0
    assert np.all(np.diff(got[:40001]) >= 0)        # monotone over the sweep


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("n", [7168, 1536, 512, 64])
def test_rmsnorm_against_float64(ox, mode, n):
    x = O.normal_bf16(3 * n, 2, 1, 2.0).reshape(3, n)
    w = O.normal_bf16(n, 2, 2, 1.0)
    y = np.empty_like(x)
    ox.ox_rmsnorm(ptr(x), ptr(w), ptr(y), 3, n, 1e-5, mode)
    xf, wf = O.bf16_to_f32(x).astype(np.float64), O.bf16_to_f32(w).astype(np.float64)
    ref = xf / np.sqrt((xf ** 2).mean(axis=1, keepdims=True) + 1e-5) * wf
    assert np.allclose(O.bf16_to_f32(y), ref, rtol=2 ** -7, atol=1e-30)     # two bf16 roundings
    # unit weight, constant input: y = bf(bf(c * rsqrt(c^2 + eps)))
    c = np.full((1, n), 0x4040, dtype=np.uint16)        # 3.0
    one = np.full(n, 0x3F80, dtype=np.uint16)
    ox.ox_rmsnorm(ptr(c), ptr(one), ptr(y[:1]), 1, n, 1e-5, mode)
    assert (y[0] == O.f32_to_bf16(np.float32(3.0 / np.sqrt(9.0 + 1e-5)))).all()


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("rows,cols,f32", [(50, 7168, 0), (384, 1024, 1), (16, 512, 0)])
def test_gemv_bf16_against_float64(ox, mode, rows, cols, f32):
    w = O.normal_bf16(rows * cols, 3, 1, 0.02).reshape(rows, cols)
    x = O.normal_bf16(2 * cols, 3, 2, 1.0).reshape(2, cols)
    y = np.empty((2, rows), dtype=np.float32 if f32 else np.uint16)
    ox.ox_gemv_bf16(ptr(w), ptr(x), ptr(y), rows, cols, 2, f32, mode)
    ref = O.bf16_to_f32(x).astype(np.float64) @ O.bf16_to_f32(w).astype(np.float64).T
    got = y if f32 else O.bf16_to_f32(y)
    assert O.max_rel(got, ref) < (1e-5 if f32 else 5e-3)
    # x = e_k reads back column k exactly
    xk = np.zeros((1, cols), dtype=np.uint16); xk[0, 77] = 0x3F80
    y1 = np.empty((1, rows), dtype=np.uint16)
    ox.ox_gemv_bf16(ptr(w), ptr(xk), ptr(y1), rows, cols, 1, 0, mode)
    assert (y1[0] == w[:, 77]).all()


@pytest.mark.parametrize("mode", [0, 1])
def test_router_against_sort_and_invariants(ox, mode):
    T, E, K = 50, 384, 8
    logits = O.normal_f32(T * E, 4, 1, 1.0).reshape(T, E)
    bias = O.normal_f32(E, 4, 2, 0.01)
    ids = np.empty((T, K), dtype=np.uint16)
    w = np.empty((T, K), dtype=np.float32)
    ox.ox_router_topk(ptr(logits), ptr(bias), ptr(ids), ptr(w), T, E, K, 2.827, mode)
    score = 1.0 / (1.0 + np.exp(-logits.astype(np.float64)))
    sel = (score + bias).astype(np.float32)
    for t in range(T):
        order = np.lexsort((np.arange(E), -sel[t].astype(np.float64)))[:K]     # descending select, lowest index on ties
        assert (ids[t] == order).all()
        assert np.allclose(w[t], score[t, order] / score[t, order].sum() * 2.827, rtol=1e-5)
    assert np.allclose(w.sum(axis=1), 2.827, rtol=1e-5)
    # constructed ties: equal logits and bias everywhere -> the first K experts, equal weights
    z = np.zeros((1, E), dtype=np.float32)
    ox.ox_router_topk(ptr(z), ptr(np.zeros(E, dtype=np.float32)), ptr(ids[:1]), ptr(w[:1]), 1, E, K, 2.827, mode)
    assert ids[0].tolist() == list(range(K)) and np.allclose(w[0], 2.827 / K)


def test_bucket_invariants(ox):
    T, E, K = 64, 384, 8
    rng = np.random.default_rng(0)
    ids = np.stack([rng.choice(E, K, replace=False) for _ in range(T)]).astype(np.uint16)
    counts, offsets = np.empty(E, np.int32), np.empty(E + 1, np.int32)
    pairs, active = np.empty(T * K, np.int32), np.empty(E, np.int32)
    na = ox.ox_bucket(ptr(ids), T, E, K, ptr(counts), ptr(offsets), ptr(pairs), ptr(active))
    assert counts.sum() == T * K and (counts == np.bincount(ids.ravel(), minlength=E)).all()
    assert offsets[0] == 0 and (np.diff(offsets) == counts).all()
    assert sorted(pairs.tolist()) == list(range(T * K))                       # a permutation
    flat = ids.ravel()
    for e in range(E):
        seg = pairs[offsets[e]:offsets[e + 1]]
        assert (flat[seg] == e).all() and (np.diff(seg) > 0).all()            # right expert, (token, slot) order
    assert na == np.count_nonzero(counts) and (active[:na] == np.nonzero(counts)[0]).all()


def test_generator_statistics_and_determinism(ox):
    z = O.normal_f32(400000, 9, 1, 1.0)
    assert abs(z.mean()) < 0.01 and abs(z.std() - 1.0) < 0.01
    assert (z == O.normal_f32(400000, 9, 1, 1.0)).all() and not (z == O.normal_f32(400000, 9, 2, 1.0)).all()
    s = O.bf16_to_f32(O.normal_bf16(100000, 9, 3, 0.02, 1))
    assert s.min() >= 0 and abs(s.mean() - 0.02 * np.sqrt(2 / np.pi)) < 3e-4     # |N(0, 0.02)|
    w = O.words_u32(100000, 9, 4)
    nib = np.stack([(w >> (4 * j)) & 0xF for j in range(8)]).ravel()
    assert abs(np.bincount(nib, minlength=16) / nib.size - 1 / 16).max() < 2e-3  # q uniform on [-8, 7]
    tok = O.tokens_u32(10000, 9, 5, 163840)
    assert tok.max() < 163840 and tok.min() >= 0


def test_moe_layer_composition(ox):
    # the layer is router -> top-k -> per slot (gate, up, SwiGLU, down) weighted in slot order -> shared expert
    # -> residual; rebuilt here in float64 from the oracle's own INT4 dequant, so a dropped term fails
    H, I, SI, E, K, T = 1024, 1024, 512, 16, 4, 3
    import kxt
    host, n, x = kxt.moe_case(None, H, I, SI, E, K, T, 31)
    wo = kxt.moe_oracle_weights(host)
    xo = x.copy()
    ids = np.empty((T, K), np.uint16); wts = np.empty((T, K), np.float32)
    ox.ox_moe_layer(C.byref(wo), ptr(n), ptr(xo), T, H, I, SI, E, K, 2.827, 0, 0, None, ptr(ids), ptr(wts), None, None)
    f = lambda a: O.bf16_to_f32(a).astype(np.float64)
    def deq(packed, scale, rows, cols, e):
        p = packed.reshape(E, rows, cols // 8)[e]; s = scale.reshape(E, rows, cols // 32)[e]
        out = np.empty((rows, cols), np.uint16)
        ox.ox_i4_dequant(ptr(np.ascontiguousarray(p)), ptr(np.ascontiguousarray(s)), ptr(out), rows, cols)
        return f(out)
    silu = lambda a: a / (1 + np.exp(-a))
    nf, ref = f(n), f(x).copy()
    for t in range(T):
        down = np.zeros(H)
        for k in range(K):
            e = int(ids[t, k])
            g = deq(host["gate_packed"], host["gate_scale"], I, H, e) @ nf[t]
            u = deq(host["up_packed"], host["up_scale"], I, H, e) @ nf[t]
            down += wts[t, k] * (deq(host["down_packed"], host["down_scale"], H, I, e) @ (silu(g) * u))
        sg = f(host["shared_gate"]).reshape(SI, H) @ nf[t]
        su = f(host["shared_up"]).reshape(SI, H) @ nf[t]
        down += f(host["shared_down"]).reshape(H, SI) @ (silu(sg) * su)
        ref[t] += down
    assert O.max_rel(f(xo), ref) < 1e-2
    # mode 1 agrees with mode 0 when the routing agrees
    x1 = x.copy(); ids1 = np.empty_like(ids)
    ox.ox_moe_layer(C.byref(wo), ptr(n), ptr(x1), T, H, I, SI, E, K, 2.827, 0, 1, None, ptr(ids1), None, None, None)
    assert (ids1 == ids).all() and O.max_rel(f(x1), f(xo)) < 1e-2
