"""Helpers shared by the GPU tests: device buffers and case builders."""
import ctypes as C

import numpy as np

import oracle as O
from blok_amd.lib import DevBuf, KxConfig, KxMoeWeights, check, default_config  # noqa: F401


def dev(arr):
    return DevBuf.from_numpy(arr)


def say(msg):
    print("[case] " + msg, flush=True)


_moe_host_cache = {}


def moe_case(lib, hidden, inter, shared, experts, topk, tokens, seed, gate_sigma=None):
    """Seeded weights of one MoE layer on host (numpy) and device, plus activations.  The weights of the last
    (shape, seed) are kept: at Kimi-K2 shape they are 10 GB and take the generator 20 s."""
    H, I, SI, E = hidden, inter, shared, experts
    gate_sigma = gate_sigma if gate_sigma is not None else float(H) ** -0.5
    key = (H, I, SI, E, seed, gate_sigma)
    if key not in _moe_host_cache:
        _moe_host_cache.clear()
        _moe_host_cache[key] = _moe_host(H, I, SI, E, seed, gate_sigma)
    host = _moe_host_cache[key]
    n = O.normal_bf16(tokens * H, seed, 30, 1.0).reshape(tokens, H)
    x = O.normal_bf16(tokens * H, seed, 31, 1.0).reshape(tokens, H)
    return host, n, x


def _moe_host(H, I, SI, E, seed, gate_sigma):
    host = {
        "router_gate": O.normal_bf16(E * H, seed, 10, gate_sigma),
        "router_bias": O.normal_f32(E, seed, 11, 0.01),
        "gate_packed": O.words_u32(E * I * H // 8, seed, 12),
        "gate_scale": O.normal_bf16(E * I * H // 32, seed, 13, 0.02, 1),
        "up_packed": O.words_u32(E * I * H // 8, seed, 14),
        "up_scale": O.normal_bf16(E * I * H // 32, seed, 15, 0.02, 1),
        "down_packed": O.words_u32(E * H * I // 8, seed, 16),
        "down_scale": O.normal_bf16(E * H * I // 32, seed, 17, 0.02, 1),
        "shared_gate": O.normal_bf16(SI * H, seed, 18, 0.02),
        "shared_up": O.normal_bf16(SI * H, seed, 19, 0.02),
        "shared_down": O.normal_bf16(H * SI, seed, 20, 0.02),
    }
    return host


def routing_of(lib, model_handle, cfg, batch):
    """Per MoE layer of the last step of a kx_model with the routing record on: the selected experts of every
    sequence as sorted tuples, and the gap between the last selected and the first rejected selection score.  The
    router bias is the generator's tensor (layer + 1) * 64 + 13 of a random-init model."""
    res = {}
    for layer in range(cfg.first_dense, cfg.n_layers):
        logits = np.empty((batch, cfg.experts), dtype=np.float32)
        check(lib.kx_model_routing(model_handle, layer, logits.ctypes.data, None))
        bias = O.normal_f32(cfg.experts, cfg.seed, (layer + 1) * 64 + 13, 0.01)
        sel = 1.0 / (1.0 + np.exp(-logits.astype(np.float64))) + bias
        order = np.argsort(-sel, axis=1, kind="stable")
        srt = np.take_along_axis(sel, order, axis=1)
        res[layer] = ([tuple(sorted(order[b, :cfg.topk].tolist())) for b in range(batch)],
                      srt[:, cfg.topk - 1] - srt[:, cfg.topk])
    return res


# a selection-score gap below this is a near-tie: a 1e-2 change of the router's input (another summation order in
# the layers before it) moves a sigmoid score by a few 1e-3
NEAR_TIE = 5e-3


class Excuse(str):
    """The text of an excuse; `key` = (sequence name, "router" or "argmax", layer or None) is what a test pins."""
    key = None


def _excuse(text, key):
    e = Excuse(text)
    e.key = key
    return e


def judge_sequences(names, errs, bar, routes_a, routes_ref, ids_a, ids_ref, logits_ref):
    """Per-sequence verdict of a tolerance path against a reference path of the same stack.  A sequence must meet
    `bar` on its logits and sample the same id, unless (a) its expert set differs from the reference's in some MoE
    layer and the reference's selection there was a near-tie (the first such layer is named), or (b) only the id
    differs and the reference's two largest logits lie closer together than the bar allows to resolve.
    Returns the list of excused sequences; raises AssertionError for any other failure."""
    excused = []
    for b, name in enumerate(names):
        flipped = None
        for layer in sorted(routes_ref):
            if routes_a[layer][0][b] != routes_ref[layer][0][b]:
                flipped = layer
                break
        if flipped is not None:
            gap = float(routes_ref[flipped][1][b])
            assert gap < NEAR_TIE, f"{name}: experts differ in layer {flipped} but the reference's selection gap there is {gap:.2e}"
            excused.append(_excuse(f"{name}: router near-tie in layer {flipped} (gap {gap:.1e}), logits err {errs[b]:.2e}", (name, "router", flipped)))
            continue
        assert errs[b] < bar, f"{name}: same experts in every layer, logits err {errs[b]:.3e} >= {bar}"
        if ids_a[b] != ids_ref[b]:
            top = np.sort(logits_ref[b])[-2:]
            gap = float(top[1] - top[0]) / float(np.max(np.abs(logits_ref[b])))
            assert gap < bar, f"{name}: id {ids_a[b]} vs {ids_ref[b]} although the top-2 logit gap is {gap:.2e}"
            excused.append(_excuse(f"{name}: argmax near-tie (top-2 gap {gap:.1e} of the largest logit)", (name, "argmax", None)))
    return excused


def assert_excused(excused, expected, what):
    """The excused sequences of a fixed seed are a fixed set: anything else excused, or a sequence no longer excused,
    is a change of the kernels' arithmetic and has to be looked at, not absorbed by a budget.  An entry with a fourth
    element, (sequence, "argmax", None, "either way"), names a sequence whose two largest reference logits are so close
    (equal to the bit, in the cases recorded) that every change of a summation order may break the tie the other way:
    it may be excused or not; judge_sequences has checked the gap when it is."""
    got = sorted(e.key for e in excused)
    print(f"{what}: excused keys {got}", flush=True)
    required = sorted(e[:3] for e in expected if len(e) == 3)
    optional = [e[:3] for e in expected if len(e) == 4]
    left = sorted(k for k in got if k not in optional)
    assert left == required, f"{what}: excused {got}, expected {required} (and possibly {optional})"


def moe_device_weights(host):
    bufs = {k: dev(v) for k, v in host.items()}
    w = KxMoeWeights()
    for k, b in bufs.items():
        setattr(w, "d_" + k, b.ptr)
    return w, bufs


def moe_oracle_weights(host):
    w = O.OxMoeWeights()
    for k, v in host.items():
        setattr(w, k, v.ctypes.data)
    return w


def moe_cfg(hidden, inter, shared, experts, topk):
    cfg = default_config()
    cfg.hidden, cfg.moe_inter, cfg.shared_inter, cfg.experts, cfg.topk = hidden, inter, shared, experts, topk
    return cfg
