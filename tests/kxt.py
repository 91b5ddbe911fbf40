"""Helpers shared by the GPU tests: device buffers and case builders."""
import ctypes as C

import numpy as np

import oracle as O
from blok_amd.lib import DevBuf, KxConfig, KxMoeWeights, check, default_config  # noqa: F401


def dev(arr):
    return DevBuf.from_numpy(arr)


def say(msg):
    print("[case] " + msg, flush=True)


def moe_case(lib, hidden, inter, shared, experts, topk, tokens, seed, gate_sigma=None):
    """Seeded weights of one MoE layer on host (numpy) and device, plus activations."""
    H, I, SI, E = hidden, inter, shared, experts
    gate_sigma = gate_sigma if gate_sigma is not None else float(H) ** -0.5
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
    n = O.normal_bf16(tokens * H, seed, 30, 1.0).reshape(tokens, H)
    x = O.normal_bf16(tokens * H, seed, 31, 1.0).reshape(tokens, H)
    return host, n, x


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
