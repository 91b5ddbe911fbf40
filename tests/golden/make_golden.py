#!/usr/bin/env python3
"""Writes tests/golden/kx_golden.npz: small inputs and the oracle's outputs for them.

The reference (akhilnairCSE110/blok) holds no golden vector for the arithmetic of this path, so these
fixtures come from this repository's own oracle (oracle/kx_oracle.cpp), after it has been pinned by the
closed-form tests.  They make a silent change of the oracle, or of the generator, visible.
Run from the repository root:  python tests/golden/make_golden.py
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle as O  # noqa: E402
from oracle import ptr  # noqa: E402


def build():
    ox = O.load()
    g = {}
    # generator
    g["rng_normal_bf16"] = O.normal_bf16(64, 5, 1, 1.0)
    g["rng_scale_bf16"] = O.normal_bf16(64, 5, 2, 0.02, 1)
    g["rng_words"] = O.words_u32(32, 5, 3)
    g["rng_tokens"] = O.tokens_u32(16, 5, 4, 163840)
    # INT4 tile: 4 rows x 1024 columns
    rows, cols = 4, 1024
    packed = O.words_u32(rows * cols // 8, 6, 1).reshape(rows, cols // 8)
    scale = O.normal_bf16(rows * cols // 32, 6, 2, 0.02, 1).reshape(rows, cols // 32)
    x = O.normal_bf16(2 * cols, 6, 3, 1.0).reshape(2, cols)
    q = np.empty((rows, cols), np.int8); w = np.empty((rows, cols), np.uint16)
    ox.ox_i4_unpack(ptr(packed), ptr(q), rows, cols)
    ox.ox_i4_dequant(ptr(packed), ptr(scale), ptr(w), rows, cols)
    g.update(i4_packed=packed, i4_scale=scale, i4_x=x, i4_q=q[:, :64].copy(), i4_w=w[:, :64].copy())
    for mode in (0, 1):
        y = np.empty((2, rows), np.uint16)
        ox.ox_i4_gemv(ptr(packed), ptr(scale), ptr(x), ptr(y), rows, cols, 2, mode)
        g[f"i4_y_mode{mode}"] = y
    # router: 2 tokens x 384 experts
    logits = O.normal_f32(2 * 384, 7, 1, 1.0).reshape(2, 384)
    bias = O.normal_f32(384, 7, 2, 0.01)
    ids = np.empty((2, 8), np.uint16); wts = np.empty((2, 8), np.float32)
    ox.ox_router_topk(ptr(logits), ptr(bias), ptr(ids), ptr(wts), 2, 384, 8, 2.827, 1)
    g.update(router_logits=logits, router_bias=bias, router_ids=ids, router_weights=wts)
    # rope table rows and the score scale
    cfg = O.small_config()
    tab = np.empty((4, 64), np.uint16)
    ox.ox_rope_table(C.byref(cfg), 1000, 4, ptr(tab))
    rs, ms = C.c_float(), C.c_float()
    ox.ox_softmax_scale(C.byref(cfg), C.byref(rs), C.byref(ms))
    g.update(rope_rows_1000=tab, softmax_scale=np.array([rs.value, ms.value], np.float32))
    # MLA: 4 heads x 8 positions
    cfg.heads = 4
    cache = O.normal_bf16(8 * 576, 8, 1, 1.0).reshape(1, 8, 576)
    qabs = O.bf16_to_f32(O.normal_bf16(4 * 576, 8, 2, 0.25)).reshape(1, 4, 576)
    g.update(mla_cache=cache, mla_qabs=qabs)
    for mode in (0, 1):
        o = np.empty((1, 4, 512), np.uint16)
        ox.ox_mla_decode(C.byref(cfg), ptr(cache), 8 * 576, ptr(qabs), ptr(o), 1, 8, mode)
        g[f"mla_o_mode{mode}"] = o[:, :, :64].copy()
    # stack: greedy ids of the small configuration
    cfg = O.small_config(batch=2)
    prompt = O.tokens_u32(2 * 6, cfg.seed, 4, cfg.vocab).reshape(2, 6)
    m = O.OxModel(cfg, 1)
    rc, out, _ = m.generate(prompt, 6)
    m.close()
    g.update(stack_prompt=prompt, stack_ids_mode1=out)
    return g


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "kx_golden.npz"), **build())
    print("wrote", os.path.join(HERE, "kx_golden.npz"))
