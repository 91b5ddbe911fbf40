#!/usr/bin/env python3
"""bench.py -- throughput of the kimi_exec forward hot path on one MI355X.

One "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM.  Workloads (BASELINE.json configs):
  stack     : (default) config 5, the truncated Kimi-K2-shaped stack: a step is one greedy
              decode step of `--batch` sequences after a `--prompt`-token prompt.  `value` is
              its decode tok/s.  The same run then times config 2 (one MoE decode layer,
              T = batch, cold weights) for `roofline`, whose dominant kernel is the fused INT4
              gate/up GEMV, and the scalar oracle on a bounded sample for `cpu_baseline`.
  moe_layer : config 2 alone, one routed-MoE decode layer at Kimi-K2 shape for `--tokens`
              tokens.  Weights of several independent layers are cycled so that neither L2
              nor the 256 MB Infinity Cache can serve them.
Prints ONE JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0


def build_if_missing():
    from blok_amd.lib import lib_path
    if not os.path.exists(lib_path()):
        import __graft_entry__
        __graft_entry__.build()


# HBM bytes of one i4_gemv_k<dual> launch at T=1 (8 experts) as rocprofv3's FETCH_SIZE / WRITE_SIZE counters saw them,
# scaled by what the same counters read for a 1 GiB kx_dev_copy.  Counters cannot be read inside this run; the figure is
# taken from the committed summary of the counter runs of this same workload, which carries it on a line of the form
# `traffic_bytes_per_launch: N`, and the JSON line names that file.
TRAFFIC_PROFILE = "profiles/moe_layer_t1_pmc.md"


def profiled_traffic():
    return _profile_figure(TRAFFIC_PROFILE, "traffic_bytes_per_launch:", int)


# Average duration of the same kernel in the committed `rocprofv3 --kernel-trace --stats` summary of the same
# command (a line `kernel_avg_us: N` there).  The profiler widens the launches and the event figure includes the
# gap between launches, so the line carries both, and the fraction each gives.
KERNEL_PROFILE = "profiles/moe_layer_t1.md"


def _profile_figure(path, key, kind):
    try:
        for line in open(os.path.join(ROOT, path)):
            if line.startswith(key):
                return kind(line.split(":")[1].split()[0].replace(",", ""))
    except OSError:
        pass
    return None


# The launches of one MoE layer of a batch-1 decode step: algorithmic bytes from the shapes, kernel time from the
# committed `rocprofv3 --kernel-trace --stats` summary of the default run's batch-1 leg (a table row per kernel).
STACK_PROFILE = "profiles/stack_decode.md"


def stack_launches(args):
    from blok_amd.lib import default_config
    c = default_config()
    H, qk, VD = c.hidden, c.qk_nope + c.qk_rope, c.heads * c.v_head
    attn_front = 2 * ((c.q_rank + c.kv_rank + c.qk_rope) * H + c.heads * qk * c.q_rank + c.heads * c.qk_nope * c.kv_rank)
    attn_back = 2 * (c.heads * c.v_head * c.kv_rank + H * VD)
    head = 2 * (2 * c.shared_inter * H + c.experts * H)
    routed = c.topk * 3 * (c.moe_inter * H // 2 + c.moe_inter * (H // 32) * 2) + 2 * H * c.shared_inter
    rows = {"attn_front_k": attn_front, "attn_back_k<true>": attn_back + head, "i4_routed_shared_k": routed}
    out = {}
    try:
        text = open(os.path.join(ROOT, STACK_PROFILE)).read()
    except OSError:
        return None
    for name, nbytes in rows.items():
        for line in text.splitlines():
            cells = [x.strip() for x in line.split("|")]
            if len(cells) > 3 and cells[1] == f"`{name}`":
                us = float(cells[3])
                out[name] = {"algorithmic_bytes": int(nbytes), "profile_avg_us": us,
                             "frac_of_hbm_peak": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
    return dict(out, profile_from=STACK_PROFILE) if out else None


def device_tokens(lib, n, seed, vocab):
    """n uniform-random token ids generated on the device (tensor id 4 of the seed) and copied back: what kx_prefill
    takes is a host array, as the reference's executor takes its prompt from argv."""
    from blok_amd.lib import DevBuf, check
    buf = DevBuf(n * 4)
    check(lib.kx_fill_tokens_u32(buf.ptr, n, seed, 4, vocab, None))
    check(lib.kx_sync(None))
    return buf.to_numpy(np.uint32, (n,))


def moe_layer_bytes(cfg, tokens, distinct):
    """Algorithmic HBM bytes of one MoE decode layer (unique bytes that must cross once)."""
    H, I, SI, E = cfg.hidden, cfg.moe_inter, cfg.shared_inter, cfg.experts
    per_matrix = I * H // 2 + I * H // 32 * 2              # packed + scales (gate, up and down alike)
    expert = 3 * per_matrix
    shared = 3 * SI * H * 2
    router = E * H * 2
    io = tokens * H * 2 * 2
    return {"expert": expert, "gate_up": 2 * per_matrix, "down": per_matrix,
            "routed": distinct * expert, "shared": shared, "router": router,
            "layer": distinct * expert + shared + router + io}


class MoeLayerSet:
    """n_layers independent MoE layers generated in place on the device."""

    TENSORS = ("router_gate", "router_bias", "gate_packed", "gate_scale", "up_packed", "up_scale",
               "down_packed", "down_scale", "shared_gate", "shared_up", "shared_down")

    def __init__(self, lib, cfg, n_layers, seed):
        from blok_amd.lib import DevBuf, KxMoeWeights, check
        H, I, SI, E = cfg.hidden, cfg.moe_inter, cfg.shared_inter, cfg.experts
        self.spec = {  # name: (kind, elements, sigma, tensor id)
            "router_gate": ("bf16", E * H, float(H) ** -0.5, 10), "router_bias": ("f32", E, 0.01, 11),
            "gate_packed": ("u32", E * I * H // 8, 0, 12), "gate_scale": ("abs", E * I * H // 32, 0.02, 13),
            "up_packed": ("u32", E * I * H // 8, 0, 14), "up_scale": ("abs", E * I * H // 32, 0.02, 15),
            "down_packed": ("u32", E * H * I // 8, 0, 16), "down_scale": ("abs", E * H * I // 32, 0.02, 17),
            "shared_gate": ("bf16", SI * H, 0.02, 18), "shared_up": ("bf16", SI * H, 0.02, 19),
            "shared_down": ("bf16", H * SI, 0.02, 20)}
        self.layers, self.bufs, self.seed = [], [], seed
        for layer in range(n_layers):
            w = KxMoeWeights()
            for name in self.TENSORS:
                kind, n, sigma, tid = self.spec[name]
                b = DevBuf(n * (2 if kind in ("bf16", "abs") else 4))
                s = seed + 1000 * layer
                if kind == "u32":
                    check(lib.kx_fill_words_u32(b.ptr, n, s, tid, None))
                elif kind == "f32":
                    check(lib.kx_fill_normal_f32(b.ptr, n, s, tid, sigma, None))
                else:
                    check(lib.kx_fill_normal_bf16(b.ptr, n, s, tid, sigma, 1 if kind == "abs" else 0, None))
                setattr(w, "d_" + name, b.ptr)
                self.bufs.append(b)
            self.layers.append(w)
        check(lib.kx_sync(None))

    def host_layer(self, layer):
        """The same tensors regenerated on the host by the oracle's generator."""
        import oracle as O
        out = {}
        s = self.seed + 1000 * layer
        for name in self.TENSORS:
            kind, n, sigma, tid = self.spec[name]
            if kind == "u32":
                out[name] = O.words_u32(n, s, tid)
            elif kind == "f32":
                out[name] = O.normal_f32(n, s, tid, sigma)
            else:
                out[name] = O.normal_bf16(n, s, tid, sigma, 1 if kind == "abs" else 0)
        return out


def run_moe_layer(args, emit=True):
    from blok_amd.lib import DevBuf, check, default_config, kx
    lib = kx()
    cfg = default_config()
    T = args.tokens
    name = C.create_string_buffer(256)
    cus, hbm = C.c_int32(), C.c_uint64()
    check(lib.kx_device_info(name, 256, C.byref(cus), C.byref(hbm)))
    n_layers = args.layers
    layers = MoeLayerSet(lib, cfg, n_layers, args.seed)
    ws = C.c_void_p()
    check(lib.kx_moe_workspace_create(C.byref(cfg), T, C.byref(ws)))
    dn, dx = DevBuf(T * cfg.hidden * 2), DevBuf(T * cfg.hidden * 2)     # activations generated on the device
    check(lib.kx_fill_normal_bf16(dn.ptr, T * cfg.hidden, args.seed, 30, 1.0, 0, None))
    check(lib.kx_fill_normal_bf16(dx.ptr, T * cfg.hidden, args.seed, 31, 1.0, 0, None))
    views = [C.c_void_p() for _ in range(8)]
    check(lib.kx_moe_workspace_views(ws, *[C.byref(v) for v in views]))

    def step(i, timed=None):
        w = layers.layers[i % n_layers]
        if timed is None:
            check(lib.kx_moe_decode_layer(C.byref(cfg), C.byref(w), ws, dn.ptr, dx.ptr, T, args.moe_flags, None))
        else:
            check(lib.kx_moe_decode_layer_timed(C.byref(cfg), C.byref(w), ws, dn.ptr, dx.ptr, T, args.moe_flags, None, timed))

    for i in range(args.warmup):
        step(i)
    check(lib.kx_sync(None))
    # timed region: K steps, events on the launch stream
    e0, e1 = C.c_void_p(), C.c_void_p()
    check(lib.kx_event_create(C.byref(e0)))
    check(lib.kx_event_create(C.byref(e1)))
    check(lib.kx_sync(None))
    t0 = time.perf_counter()
    check(lib.kx_event_record(e0, None))
    for i in range(args.steps):
        step(args.warmup + i)
    check(lib.kx_event_record(e1, None))
    check(lib.kx_sync(None))
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms = C.c_float()
    check(lib.kx_event_elapsed_ms(e0, e1, C.byref(ms)))
    ms_per_step = ms.value / args.steps

    # per-kernel durations (events around each launch) and distinct experts, same steps
    phases = np.zeros(5)
    distinct = []
    ms5 = (C.c_float * 5)()
    counts = np.empty(cfg.experts, dtype=np.int32)
    for i in range(args.steps):
        step(args.warmup + i, ms5)
        phases += np.array(list(ms5))
        check(lib.kx_d2h(counts.ctypes.data, views[3].value, counts.nbytes))
        distinct.append(int(np.count_nonzero(counts)))
    phases /= args.steps
    U = float(np.mean(distinct))
    by = moe_layer_bytes(cfg, T, U)
    # the two routed-expert kernels alone, launched back to back over the cycled layers (cold weights), on the
    # routing of the last step: average launch duration = elapsed / launches, events on the launch stream
    alone = []
    for which in (0, 1):
        for i in range(n_layers):
            check(lib.kx_moe_routed_only(C.byref(cfg), C.byref(layers.layers[i]), ws, dn.ptr, T, which, None))
        check(lib.kx_sync(None))
        reps = max(args.steps, 20)
        check(lib.kx_event_record(e0, None))
        for i in range(reps):
            check(lib.kx_moe_routed_only(C.byref(cfg), C.byref(layers.layers[i % n_layers]), ws, dn.ptr, T, which, None))
        check(lib.kx_event_record(e1, None))
        check(lib.kx_sync(None))
        check(lib.kx_event_elapsed_ms(e0, e1, C.byref(ms)))
        alone.append(ms.value / reps)
    check(lib.kx_d2h(counts.ctypes.data, views[3].value, counts.nbytes))
    U_last = int(np.count_nonzero(counts))
    gate_up_gbs = U_last * by["gate_up"] / (alone[0] * 1e-3) / 1e9
    down_gbs = U_last * by["down"] / (alone[1] * 1e-3) / 1e9
    routed_gbs = U_last * (by["gate_up"] + by["down"]) / ((alone[0] + alone[1]) * 1e-3) / 1e9
    layer_gbs = by["layer"] / (ms_per_step * 1e-3) / 1e9

    # CPU baseline: the oracle's reference schedule on the same layer-0 weights, bounded sample
    cpu = None
    if not args.no_cpu:
        import oracle as O
        from kxt import moe_oracle_weights
        ox = O.load()
        n_host = dn.to_numpy(np.uint16, (T, cfg.hidden))
        x_host = dx.to_numpy(np.uint16, (T, cfg.hidden))
        host = layers.host_layer(0)
        wo = moe_oracle_weights(host)
        tc = min(T, 4)
        xo = x_host[:tc].copy()
        t0 = time.perf_counter()
        reps = 0
        while True:
            ox.ox_moe_layer(C.byref(wo), n_host[:tc].ctypes.data, xo.ctypes.data, tc, cfg.hidden, cfg.moe_inter,
                            cfg.shared_inter, cfg.experts, cfg.topk, cfg.routed_scale, 1, 0,
                            None, None, None, None, None)
            reps += 1
            if time.perf_counter() - t0 > args.cpu_seconds or reps >= 64:
                break
        dt = time.perf_counter() - t0
        cpu = {"value": round(tc * reps / dt, 3), "unit": "tok/s", "cores": ox.ox_num_threads(), "kind": "port",
               "sample": f"{reps} x one MoE decode layer, {tc} token(s), layer-0 weights, reference schedule "
                         f"(oracle mode 0), OpenMP over output rows, {dt:.1f} s"}
    check(lib.kx_moe_workspace_destroy(ws))

    out = {
        "metric": "decode tok/s + INT4 expert GEMV HBM GB/s (% of peak), Kimi-K2 shapes, 1 GPU",
        "value": round(T / (ms_per_step * 1e-3), 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int4 weights x bf16 activations, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": f"moe_decode_layer (BASELINE config 2), T={T}, hidden 7168, 384 experts top-8, "
                               f"moe_inter 2048, shared 2048; {n_layers} independent layers cycled (cold weights)",
                   "tokens": T, "distinct_experts_per_step": round(U, 2), "layer_flags": hex(args.moe_flags),
                   "layer_gbs": round(layer_gbs, 1), "device": name.value.decode(),
                   "compute_units": cus.value},
        "roofline": {"bound": "hbm", "achieved": round(gate_up_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gate_up_gbs / HBM_PEAK_GBS, 4),
                     "traffic": profiled_traffic() if (T == 1 and U_last == cfg.topk) else None,
                     "traffic_from": TRAFFIC_PROFILE if (T == 1 and U_last == cfg.topk) else None,
                     "kernel": "i4_gemv_k<dual> (routed gate+up + SwiGLU)",
                     "algorithmic_bytes_per_launch": int(U_last * by["gate_up"]),
                     "avg_launch_ms": round(alone[0], 5),
                     "how": "launched back to back over the cycled layers, HIP events on the launch stream"},
        "int4_expert_gemv": {"routed_gbs": round(routed_gbs, 1), "routed_frac_of_peak": round(routed_gbs / HBM_PEAK_GBS, 4),
                             "gate_up_gbs": round(gate_up_gbs, 1), "down_gbs": round(down_gbs, 1),
                             "gate_up_ms": round(alone[0], 5), "down_ms": round(alone[1], 5),
                             "distinct_experts": U_last, "layer_gbs": round(layer_gbs, 1)},
        "phase_ms": {"shared_gate_up_router_route": round(float(phases[0]), 5), "routed_gate_up": round(float(phases[1]), 5),
                     "routed_down": round(float(phases[2]), 5), "shared_down_combine": round(float(phases[3] + phases[4]), 5),
                     "note": "events around each launch inside the layer; they include the event commands themselves; "
                             "for one token the routed down launch also runs the shared down GEMV and the combine"},
        "wall_ms_per_step": round(wall_ms / args.steps, 5),
        "cpu_baseline": cpu,
    }
    if emit:
        print(json.dumps(out), flush=True)
    return out


def stack_bytes_per_token(cfg, distinct_per_layer):
    """Algorithmic HBM bytes of the weights one decode step of the truncated stack reads (each once), with
    distinct_per_layer routed experts selected per MoE layer (8 at batch 1; measured for a batch)."""
    H, V = cfg.hidden, cfg.vocab
    KD, VD = cfg.heads * (cfg.qk_nope + cfg.qk_rope), cfg.heads * cfg.v_head
    KVA, KVB = cfg.kv_rank + cfg.qk_rope, cfg.heads * (cfg.qk_nope + cfg.v_head)
    attn = 2 * ((cfg.q_rank + KVA) * H + KD * cfg.q_rank + KVB * cfg.kv_rank + H * VD)
    dense = 2 * 3 * cfg.dense_inter * H
    per_matrix = cfg.moe_inter * H // 2 + cfg.moe_inter * H // 32 * 2
    moe = distinct_per_layer * 3 * per_matrix + 2 * 3 * cfg.shared_inter * H + 2 * cfg.experts * H
    n_moe = cfg.n_layers - cfg.first_dense
    return cfg.n_layers * attn + cfg.first_dense * dense + n_moe * moe + 2 * V * H


def stack_leg(lib, cfg, model, st, B, P, K, W, seed, prefill_chunk):
    """One timed run of the stack on an existing model: prefill B prompts of P tokens, W warm-up and K timed greedy
    decode steps; ids never leave the device inside the timed region."""
    from blok_amd.lib import check
    prompt = device_tokens(lib, B * P, seed, cfg.vocab).reshape(B, P)
    e = [C.c_void_p() for _ in range(4)]
    for ev in e:
        check(lib.kx_event_create(C.byref(ev)))
    check(lib.kx_model_set_prefill_chunk(model, max(1, prefill_chunk)))  # 1: token by token, the reference's loop
    check(lib.kx_event_record(e[0], st))
    check(lib.kx_prefill(model, prompt.ctypes.data, B, P))
    check(lib.kx_event_record(e[3], st))
    for _ in range(W):
        check(lib.kx_decode_step(model, None))
    check(lib.kx_event_record(e[1], st))
    check(lib.kx_sync(st))
    t0 = time.perf_counter()
    for i in range(K):                      # K timed decode steps; ids stay on the device
        check(lib.kx_decode_step(model, None))
    check(lib.kx_event_record(e[2], st))
    check(lib.kx_sync(st))
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_pre, ms_dec = C.c_float(), C.c_float()
    check(lib.kx_event_elapsed_ms(e[0], e[3], C.byref(ms_pre)))
    check(lib.kx_event_elapsed_ms(e[1], e[2], C.byref(ms_dec)))
    for ev in e:
        check(lib.kx_event_destroy(ev))
    last = np.zeros(B, dtype=np.uint32)
    check(lib.kx_greedy_sample(model, last.ctypes.data))
    # distinct routed experts per MoE layer, which is what a batch's weight traffic depends on: counted over a few more
    # (untimed) decode steps with the model's routing record switched on
    distinct = float(cfg.topk)
    if B > 1 and cfg.n_layers > cfg.first_dense:
        check(lib.kx_model_set_routing_record(model, 1))
        seen, d = [], C.c_int32()
        for _ in range(6):
            check(lib.kx_decode_step(model, None))
            for layer in range(cfg.first_dense, cfg.n_layers):
                check(lib.kx_model_routing(model, layer, None, C.byref(d)))
                seen.append(d.value)
        distinct = float(np.mean(seen))
        check(lib.kx_model_set_routing_record(model, 0))
    ms_per_step = ms_dec.value / K
    weights = stack_bytes_per_token(cfg, distinct)
    kv = B * (P + W + K // 2) * (cfg.kv_rank + cfg.qk_rope) * 2 * cfg.n_layers   # latent cache rows read by a mid-run step
    algo = weights if B == 1 else weights + kv
    return {
        "value": round(B * 1e3 / ms_per_step, 2), "ms_per_step": round(ms_per_step, 5), "wall_ms_per_step": round(wall_ms / K, 5),
        "prefill_ms_per_token": round(ms_pre.value / P, 5), "last_ids": last.tolist(),
        "prefill": "token by token" if prefill_chunk <= 1 else f"{min(prefill_chunk, max(1, 2048 // B))} positions per step",
        "stack_hbm": {"algorithmic_bytes_per_step": int(algo), "weight_bytes": int(weights), "kv_cache_bytes": int(kv),
                      "counted": "weights once per step" + ("" if B == 1 else " + latent cache rows of every sequence"),
                      "distinct_experts_per_moe_layer": round(distinct, 1),
                      "achieved_gbs": round(algo / (ms_per_step * 1e-3) / 1e9, 1),
                      "frac_of_peak": round(algo / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                      "roof_tok_s": round(B * HBM_PEAK_GBS * 1e9 / algo, 1)},
    }


def run_stack(args, extra_batches=()):
    """BASELINE config 5: the truncated Kimi-K2-shaped stack, greedy decode after a uniform-random prompt.  The model
    is created once, for the largest batch asked for; the headline leg (--batch) runs first, then one leg per extra
    batch on the same resident weights."""
    from blok_amd.lib import check, default_config, kx
    lib = kx()
    cfg = default_config()
    B, P, K, W = args.batch, args.prompt, args.steps, args.warmup
    cfg.n_layers, cfg.max_batch, cfg.max_context, cfg.seed = args.stack_layers, max((B,) + tuple(extra_batches)), P + K + W + 9, args.seed
    name = C.create_string_buffer(256)
    cus, hbm = C.c_int32(), C.c_uint64()
    check(lib.kx_device_info(name, 256, C.byref(cus), C.byref(hbm)))
    wb, cb, sb = C.c_uint64(), C.c_uint64(), C.c_uint64()
    check(lib.kx_model_bytes(C.byref(cfg), C.byref(wb), C.byref(cb), C.byref(sb)))
    t0 = time.perf_counter()
    model = C.c_void_p()
    check(lib.kx_model_create(C.byref(cfg), C.byref(model)))
    check(lib.kx_sync(None))
    t_create = time.perf_counter() - t0
    st = C.c_void_p()
    check(lib.kx_model_stream(model, C.byref(st)))
    if args.fusion is not None:             # which steps ride inside the launch before them (KX_FUSE_* of include/kx.h); same results
        check(lib.kx_model_set_fusion(model, args.fusion))
    out = stack_leg(lib, cfg, model, st, B, P, K, W, args.seed, args.prefill_chunk)
    out["extra"] = {b: stack_leg(lib, cfg, model, st, b, P, K, W, args.seed, args.prefill_chunk) for b in extra_batches}
    check(lib.kx_model_destroy(model))
    out.update({
        "workload": f"truncated Kimi-K2 stack (BASELINE config 5): {cfg.n_layers} layers (1 dense + {cfg.n_layers - 1} MoE), "
                    f"vocab {cfg.vocab}, batch {B}, {P}-token uniform-random prompt prefilled {out['prefill']}, then "
                    f"{W} warm-up and {K} timed greedy decode steps; seeded random-init weights resident in HBM",
        "resident_gb": {"weights": round(wb.value / 1e9, 2), "kv_cache": round(cb.value / 1e9, 3), "scratch": round(sb.value / 1e9, 3)},
        "model_create_s": round(t_create, 2), "device": name.value.decode(), "compute_units": cus.value})
    return out


def run_cpu_stack(args):
    """CPU baseline: the oracle's reference schedule (mode 0) on config 5's stack itself -- all --cpu-layers layers
    (default 24), full vocabulary, batch 1 -- for a bounded number of token steps.  The oracle holds the dense tensors
    and produces a routed expert when a token first selects it, so the stack fits in host memory; producing the
    experts is part of what is timed (the reference reads its tiles from NVMe inside the layer loop, too)."""
    import oracle as O
    from blok_amd.lib import default_config
    cfg = default_config()
    cfg.n_layers, cfg.max_batch, cfg.max_context, cfg.seed = args.cpu_layers, 1, 64, args.seed
    t0 = time.perf_counter()
    m = O.OxModel(cfg, 0, experts_on_demand=True)
    t_init = time.perf_counter() - t0
    ids = O.tokens_u32(1, args.seed, 4, cfg.vocab)
    t0 = time.perf_counter()
    steps = 0
    while steps < args.cpu_tokens and (steps < 2 or time.perf_counter() - t0 < args.cpu_seconds * 2):
        ids = m.step(ids, steps, True)          # every step samples, as a decode step does
        steps += 1
    dt = time.perf_counter() - t0
    m.close()
    per_step = dt / steps
    full = default_config()
    scaled = per_step * ((full.n_layers - 1) / max(1, cfg.n_layers - 1)) if cfg.n_layers != full.n_layers else per_step
    return {"value": round(1.0 / per_step, 4), "unit": "tok/s", "cores": O.load().ox_num_threads(), "kind": "port",
            "layers": cfg.n_layers, "steps": steps, "seconds": round(dt, 2),
            "scaled_to_24_layers_tok_s": round(1.0 / scaled, 4),
            "sample": f"oracle reference schedule (mode 0) on config 5's stack, {cfg.n_layers} layers (1 dense + "
                      f"{cfg.n_layers - 1} MoE, 384 experts produced on demand, full vocabulary), batch 1: {steps} sampled token "
                      f"steps in {dt:.1f} s after {t_init:.1f} s of dense-weight generation; OpenMP over output rows"}


def run_default(args):
    """Config 5 for `value`, plus the routed INT4 gate/up kernel of config 2 (T = batch) for `roofline`."""
    extra = (32,) if (args.batch == 1 and not args.no_b32) else ()
    stack = run_stack(args, extra)
    margs = argparse.Namespace(**vars(args))
    margs.tokens, margs.steps, margs.warmup, margs.no_cpu = args.batch, 40, 8, True
    moe = run_moe_layer(margs, emit=False)
    moe8 = None
    if args.batch == 1:   # the same two kernels at T = 8 (BASELINE config 2 names T in {1, 8, 64}), where a launch is 7.5 waves of workgroups
        margs8 = argparse.Namespace(**vars(margs))
        margs8.tokens = 8
        moe8 = run_moe_layer(margs8, emit=False)
    cpu = None if args.no_cpu else run_cpu_stack(args)
    roof = {k: v for k, v in moe["roofline"].items()}
    prof_us = _profile_figure(KERNEL_PROFILE, "kernel_avg_us:", float) if args.batch == 1 else None
    if prof_us:
        roof["profile_kernel_avg_us"] = prof_us
        roof["profile_frac"] = round(roof["algorithmic_bytes_per_launch"] / (prof_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)
        roof["profile_from"] = KERNEL_PROFILE
    out = {
        "metric": "decode tok/s + INT4 expert GEMV HBM GB/s (% of peak), Kimi-K2 shapes, 1 GPU",
        "value": stack["value"], "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": stack["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights x bf16 activations, f32 accumulate", "data": "synthetic",
        "config": {"workload": stack["workload"], "batch": args.batch, "prompt": args.prompt, "device": stack["device"],
                   "compute_units": stack["compute_units"], "resident_gb": stack["resident_gb"]},
        "roofline": roof,
        "int4_expert_gemv": dict(moe["int4_expert_gemv"], workload=moe["config"]["workload"], phase_ms=moe["phase_ms"]),
        "stack": {k: stack[k] for k in ("wall_ms_per_step", "prefill_ms_per_token", "model_create_s", "stack_hbm", "last_ids")},
        "cpu_baseline": cpu,
    }
    launches = stack_launches(args) if args.batch == 1 else None
    if launches:
        out["stack"]["launches_per_moe_layer"] = launches
    for b, leg in stack["extra"].items():     # config 5 names batch 32 too: the same resident model, same prompt length
        out[f"stack_b{b}"] = {"tok_s": leg["value"], "ms_per_step": leg["ms_per_step"], "steps": args.steps, "warmup": args.warmup,
                              "prompt": args.prompt, "prefill": leg["prefill"], "prefill_ms_per_token": leg["prefill_ms_per_token"],
                              "distinct_experts": leg["stack_hbm"]["distinct_experts_per_moe_layer"], "stack_hbm": leg["stack_hbm"]}
    if moe8 is not None:
        out["int4_expert_gemv_t8"] = dict(moe8["int4_expert_gemv"], workload=moe8["config"]["workload"],
                                          gate_up_frac_of_peak=moe8["roofline"]["frac"])
    print(json.dumps(out), flush=True)
    return out


def run_prefill(args):
    """BASELINE config 4: a 2048-token prefill chunk through one MoE layer on the matrix cores."""
    import oracle as O
    from blok_amd.lib import DevBuf, check, default_config, kx
    lib = kx()
    cfg = default_config()
    T = args.tokens
    layers = MoeLayerSet(lib, cfg, 2, args.seed)
    # Zipf-like load: bias += c*ln(1/rank)
    for li, w in enumerate(layers.layers):
        bias = (O.normal_f32(cfg.experts, args.seed + 1000 * li, 11, 0.01) + 0.1 * np.log(1.0 / np.arange(1, cfg.experts + 1))).astype(np.float32)
        check(lib.kx_h2d(w.d_router_bias, bias.ctypes.data, cfg.experts * 4))   # `bias` stays alive across the call
    ws = C.c_void_p()
    check(lib.kx_moe_workspace_create(C.byref(cfg), T, C.byref(ws)))
    n_host = O.normal_bf16(T * cfg.hidden, args.seed, 30, 1.0)
    x_host = O.normal_bf16(T * cfg.hidden, args.seed, 31, 1.0)
    dn, dx = DevBuf.from_numpy(n_host), DevBuf.from_numpy(x_host)
    views = [C.c_void_p() for _ in range(8)]
    check(lib.kx_moe_workspace_views(ws, *[C.byref(v) for v in views]))
    e0, e1 = C.c_void_p(), C.c_void_p()
    check(lib.kx_event_create(C.byref(e0)))
    check(lib.kx_event_create(C.byref(e1)))
    for i in range(args.warmup):
        check(lib.kx_moe_prefill_layer(C.byref(cfg), C.byref(layers.layers[i % 2]), ws, dn.ptr, dx.ptr, T, 1, None))
    check(lib.kx_sync(None))
    check(lib.kx_event_record(e0, None))
    for i in range(args.steps):
        check(lib.kx_moe_prefill_layer(C.byref(cfg), C.byref(layers.layers[i % 2]), ws, dn.ptr, dx.ptr, T, 1, None))
    check(lib.kx_event_record(e1, None))
    ms = C.c_float()
    check(lib.kx_event_elapsed_ms(e0, e1, C.byref(ms)))
    counts = np.empty(cfg.experts, dtype=np.int32)
    check(lib.kx_d2h(counts.ctypes.data, views[3].value, counts.nbytes))
    check(lib.kx_moe_workspace_destroy(ws))
    ms_step = ms.value / args.steps
    U = int(np.count_nonzero(counts))
    by = moe_layer_bytes(cfg, T, U)
    flops = 2.0 * T * cfg.topk * 3 * cfg.moe_inter * cfg.hidden + 2.0 * T * 3 * cfg.shared_inter * cfg.hidden
    out = {"metric": "prefill tok/s through one MoE layer (BASELINE config 4)", "value": round(T / (ms_step * 1e-3), 1),
           "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "int4 weights dequantized to bf16, bf16 MFMA, f32 accumulate", "data": "synthetic",
           "config": {"workload": f"moe_prefill_layer, T={T}, Zipf-skewed gate bias", "experts_used": U,
                      "busiest_expert_tokens": int(counts.max())},
           "roofline": {"bound": "mfma", "achieved": round(flops / (ms_step * 1e-3) / 1e12, 2), "peak": 2500.0,
                        "unit": "TFLOP/s", "frac": round(flops / (ms_step * 1e-3) / 1e12 / 2500.0, 4), "traffic": None},
           "hbm_gbs": round(by["layer"] / (ms_step * 1e-3) / 1e9, 1)}
    print(json.dumps(out), flush=True)
    return out


def run_mla(args):
    """BASELINE config 3: MLA decode attention on the latent cache, one query position per sequence."""
    from blok_amd.lib import check, default_config, kx
    lib = kx()
    cfg = default_config()
    B, L = args.batch, args.context
    kva = cfg.kv_rank + cfg.qk_rope
    cache_bytes = B * L * kva * 2
    cache, qabs, wsp, o_lat = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
    check(lib.kx_dev_malloc(C.byref(cache), cache_bytes))
    check(lib.kx_fill_normal_bf16(cache, B * L * kva, args.seed, 40, 1.0, 0, None))
    check(lib.kx_dev_malloc(C.byref(qabs), B * cfg.heads * kva * 4))
    check(lib.kx_fill_normal_f32(qabs, B * cfg.heads * kva, args.seed, 41, 1.0, None))
    ws_bytes = C.c_size_t()
    check(lib.kx_mla_workspace_bytes(C.byref(cfg), B, L, C.byref(ws_bytes)))
    check(lib.kx_dev_malloc(C.byref(wsp), ws_bytes.value))
    check(lib.kx_dev_malloc(C.byref(o_lat), B * cfg.heads * cfg.kv_rank * 2))
    e0, e1 = C.c_void_p(), C.c_void_p()
    check(lib.kx_event_create(C.byref(e0)))
    check(lib.kx_event_create(C.byref(e1)))
    steps = args.steps if args.steps != 256 else 20
    for _ in range(min(args.warmup, 3)):
        check(lib.kx_mla_decode(C.byref(cfg), cache, L * kva, qabs, wsp, o_lat, B, L, 0, None))
    check(lib.kx_sync(None))
    check(lib.kx_event_record(e0, None))
    for _ in range(steps):
        check(lib.kx_mla_decode(C.byref(cfg), cache, L * kva, qabs, wsp, o_lat, B, L, 0, None))
    check(lib.kx_event_record(e1, None))
    check(lib.kx_sync(None))
    ms = C.c_float()
    check(lib.kx_event_elapsed_ms(e0, e1, C.byref(ms)))
    per = ms.value / steps
    flops = 2.0 * B * L * cfg.heads * (kva + cfg.kv_rank)
    gbs = cache_bytes / (per * 1e-3) / 1e9
    print(json.dumps({"metric": "MLA decode attention, latent-cache GB/s (BASELINE config 3)", "value": round(gbs, 1),
                      "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": min(args.warmup, 3), "ms_per_step": round(per, 4),
                      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 cache, f32 accumulate",
                      "data": "synthetic",
                      "config": {"workload": f"kx_mla_decode, B={B}, L={L}, 64 heads, latent 512+64", "batch": B, "context": L},
                      "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                                   "algorithmic_bytes_per_launch": cache_bytes},
                      "compute": {"tflops": round(flops / (per * 1e-3) / 1e12, 2),
                                  "kernel": "mla_partial_mfma_k (bf16 MFMA)" if L >= 2048 else "mla_partial_k (fp32 VALU)",
                                  "frac_of_mfma_bf16_peak": round(flops / (per * 1e-3) / 1e12 / 2500.0, 4),
                                  "frac_of_valu_fp32_peak": round(flops / (per * 1e-3) / 1e12 / 157.3, 4)}}), flush=True)


def run_copy(args):
    """Plain copy of a known size: the kernel whose FETCH_SIZE / WRITE_SIZE readings calibrate the traffic figures."""
    from blok_amd.lib import check, kx
    lib = kx()
    nbytes = args.copy_mib << 20
    src, dst = C.c_void_p(), C.c_void_p()
    check(lib.kx_dev_malloc(C.byref(src), nbytes))
    check(lib.kx_dev_malloc(C.byref(dst), nbytes))
    check(lib.kx_fill_words_u32(src, nbytes // 4, 1, 1, None))
    e0, e1 = C.c_void_p(), C.c_void_p()
    check(lib.kx_event_create(C.byref(e0)))
    check(lib.kx_event_create(C.byref(e1)))
    for _ in range(args.warmup):
        check(lib.kx_dev_copy(dst, src, nbytes, None))
    check(lib.kx_sync(None))
    check(lib.kx_event_record(e0, None))
    for _ in range(args.steps):
        check(lib.kx_dev_copy(dst, src, nbytes, None))
    check(lib.kx_event_record(e1, None))
    check(lib.kx_sync(None))
    ms = C.c_float()
    check(lib.kx_event_elapsed_ms(e0, e1, C.byref(ms)))
    per = ms.value / args.steps
    print(json.dumps({"metric": "copy16_k read+write GB/s", "value": round(2 * nbytes / (per * 1e-3) / 1e9, 1),
                      "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                      "ms_per_step": round(per, 5), "higher_is_better": True,
                      "config": {"workload": f"kx_dev_copy of {args.copy_mib} MiB (reads {nbytes} B, writes {nbytes} B per launch)"}}),
          flush=True)


def run_load(args):
    """kx_model_load on a Kimi-K2-shaped checkpoint of --stack-layers layers whose shards are sparse files
    (headers written, data holes): what the reader threads, staging buffers and host-to-device copies sustain
    when the disk is not the limit.  Not a disk benchmark."""
    import struct
    import tempfile
    from blok_amd import model_index
    from blok_amd.lib import check, default_config, kx
    lib = kx()
    cfg = default_config()
    cfg.n_layers = args.stack_layers if args.stack_layers != 24 else 2
    cfg.max_batch, cfg.max_context = 1, 64
    H, V, E, I, SI, D = cfg.hidden, cfg.vocab, cfg.experts, cfg.moe_inter, cfg.shared_inter, cfg.dense_inter
    KD, VD = cfg.heads * (cfg.qk_nope + cfg.qk_rope), cfg.heads * cfg.v_head
    KVA, KVB = cfg.kv_rank + cfg.qk_rope, cfg.heads * (cfg.qk_nope + cfg.v_head)
    lm = "language_model."
    shards = [[(lm + "model.embed_tokens.weight", "BF16", (V, H)), (lm + "model.norm.weight", "BF16", (H,)),
               (lm + "lm_head.weight", "BF16", (V, H))]]
    for l in range(cfg.n_layers):
        p, t = f"{lm}model.layers.{l}.", []
        for n, shp in (("input_layernorm", (H,)), ("post_attention_layernorm", (H,)), ("self_attn.q_a_proj", (cfg.q_rank, H)),
                       ("self_attn.q_a_layernorm", (cfg.q_rank,)), ("self_attn.q_b_proj", (KD, cfg.q_rank)),
                       ("self_attn.kv_a_proj_with_mqa", (KVA, H)), ("self_attn.kv_a_layernorm", (cfg.kv_rank,)),
                       ("self_attn.kv_b_proj", (KVB, cfg.kv_rank)), ("self_attn.o_proj", (H, VD))):
            t.append((p + n + ".weight", "BF16", shp))
        if l < cfg.first_dense:
            t += [(p + "mlp.gate_proj.weight", "BF16", (D, H)), (p + "mlp.up_proj.weight", "BF16", (D, H)),
                  (p + "mlp.down_proj.weight", "BF16", (H, D))]
        else:
            t += [(p + "mlp.gate.weight", "BF16", (E, H)), (p + "mlp.gate.e_score_correction_bias", "BF16", (E,))]
            for n, shp in (("gate_proj", (SI, H)), ("up_proj", (SI, H)), ("down_proj", (H, SI))):
                t.append((p + f"mlp.shared_experts.{n}.weight", "BF16", shp))
            for e in range(E):
                for n, (r, c) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
                    t.append((p + f"mlp.experts.{e}.{n}.weight_packed", "I32", (r, c // 8)))
                    t.append((p + f"mlp.experts.{e}.{n}.weight_scale", "BF16", (r, c // 32)))
        shards.append(t)
    root = tempfile.mkdtemp(prefix="kx_load_", dir=args.load_dir)
    try:
        for i, tensors in enumerate(shards):
            header, at = {}, 0
            for name, dtype, shape in tensors:
                n = int(np.prod(shape)) * (2 if dtype == "BF16" else 4)
                header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [at, at + n]}
                at += n
            body = json.dumps(header, separators=(",", ":")).encode()
            with open(os.path.join(root, f"model-{i + 1:05d}-of-{len(shards):06d}.safetensors"), "wb") as f:
                f.write(struct.pack("<Q", len(body)))
                f.write(body)
                f.truncate(8 + len(body) + at)
        report = model_index.materialize(root, os.path.join(root, "meta"))
        times = []
        for _ in range(max(1, min(args.steps, 3))):
            h = C.c_void_p()
            check(lib.kx_model_load(C.byref(cfg), report["index"].encode(), C.byref(h)))
            nbytes, secs = C.c_uint64(), C.c_double()
            check(lib.kx_model_load_info(h, C.byref(nbytes), C.byref(secs)))
            check(lib.kx_model_destroy(h))
            times.append(secs.value)
    finally:
        import shutil
        shutil.rmtree(root, ignore_errors=True)
    best = min(times)
    print(json.dumps({"metric": "checkpoint load GB/s (sparse shards, no disk reads)", "value": round(nbytes.value / best / 1e9, 2),
                      "unit": "GB/s", "n_gpus": 1, "steps": len(times), "warmup": 0, "ms_per_step": round(best * 1e3, 1),
                      "higher_is_better": True, "data": "synthetic",
                      "config": {"workload": f"kx_model_load, Kimi-K2 shapes, {cfg.n_layers} layers, {report['tensors']} tensors, "
                                             f"{nbytes.value / 1e9:.2f} GB", "threads": int(os.environ.get("KX_LOAD_THREADS", "8")),
                                 "direct": os.environ.get("KX_LOAD_DIRECT", "1") != "0", "seconds_each": [round(t, 3) for t in times]}}),
          flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default="stack", choices=["stack", "moe_layer", "prefill", "mla", "copy", "load"])
    ap.add_argument("--load-dir", default=None, help="where the load workload writes its sparse shards (default: the temp dir)")
    ap.add_argument("--context", type=int, default=32768)
    ap.add_argument("--copy-mib", type=int, default=1024)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--prompt", type=int, default=1024)
    ap.add_argument("--prefill-chunk", type=int, default=1, help="prompt positions per prefill step (1: the reference's token-by-token prefill)")
    ap.add_argument("--stack-layers", type=int, default=24)
    ap.add_argument("--fusion", type=lambda v: int(v, 0), default=None, help="stack: mask for kx_model_set_fusion (default: the library's, all on)")
    ap.add_argument("--cpu-layers", type=int, default=24)
    ap.add_argument("--no-b32", action="store_true", help="default run: skip the batch-32 leg of config 5")
    ap.add_argument("--tokens", type=int, default=1)
    ap.add_argument("--moe-flags", type=lambda v: int(v, 0), default=0,
                    help="moe_layer: flags of kx_moe_decode_layer (0: the bit-reproducible kernels; 0x400: routed experts with "
                         "several pairs on the matrix cores, 0x200: the shared expert too, both within 1e-2 of the default)")
    ap.add_argument("--layers", type=int, default=4, help="independent layers cycled to keep weights cold")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=12)
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    build_if_missing()
    if args.workload == "copy":
        run_copy(args)
        return
    if args.workload == "load":
        run_load(args)
        return
    if args.workload == "mla":
        run_mla(args)
        return
    if args.workload == "prefill":
        if args.tokens == 1:
            args.tokens = 2048
        if args.steps == 256:
            args.steps = 10
        run_prefill(args)
    elif args.workload == "moe_layer":
        if args.steps == 256:
            args.steps = 40
        run_moe_layer(args)
    else:
        run_default(args)


if __name__ == "__main__":
    main()
