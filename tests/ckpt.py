"""Test helper: a synthetic checkpoint in the on-disk form the reference loads.

Writes safetensors shards whose tensors carry the Hugging Face names of the Kimi-K2.6 text decoder
(`language_model.model.layers.<l>...`, README.md:17 of the reference) for a small kx_config, plus decoys
the index writer must skip, and returns the same tensors as arrays for the oracle.  The shards are
written here byte by byte (8-byte length, JSON header, data), so the reader under test is not its own
witness.
"""
import json
import struct
from pathlib import Path

import numpy as np

import oracle as O

# tensor ids of the seeded model (kx_model.hip / kx_oracle.cpp): globals use the id, layers TL_*
TID_EMBED, TID_FINAL_NORM, TID_LM_HEAD = 1, 2, 3
(TL_INPUT_LN, TL_QA, TL_QA_LN, TL_QB, TL_KVA, TL_KV_LN, TL_KVB, TL_O, TL_POST_LN, TL_DENSE_GATE, TL_DENSE_UP,
 TL_DENSE_DOWN, TL_ROUTER, TL_ROUTER_BIAS, TL_GATE_P, TL_GATE_S, TL_UP_P, TL_UP_S, TL_DOWN_P, TL_DOWN_S, TL_SH_GATE,
 TL_SH_UP, TL_SH_DOWN) = range(23)


def _ln(n, seed, tid):
    out = np.empty(n, dtype=np.uint16)
    O.load().ox_fill_affine_bf16(O.ptr(out), n, seed, tid, 1.0, 0.02)
    return out


def model_tensors(cfg, seed):
    """[(hf_name, st_dtype, shape, array, (layer, tid, expert), oracle_array)] for every tensor of the stack."""
    H, V, E, I, SI, D = cfg.hidden, cfg.vocab, cfg.experts, cfg.moe_inter, cfg.shared_inter, cfg.dense_inter
    KD, VD = cfg.heads * (cfg.qk_nope + cfg.qk_rope), cfg.heads * cfg.v_head
    KVA, KVB = cfg.kv_rank + cfg.qk_rope, cfg.heads * (cfg.qk_nope + cfg.v_head)
    sg, es = cfg.init_sigma, cfg.expert_scale_sigma
    out = []

    def bf(name, shape, arr, key):
        out.append((name, "BF16", shape, arr, key, arr))

    lm = "language_model."
    bf(lm + "model.embed_tokens.weight", (V, H), O.normal_bf16(V * H, seed, TID_EMBED, 1.0), (-1, TID_EMBED, -1))
    bf(lm + "model.norm.weight", (H,), _ln(H, seed, TID_FINAL_NORM), (-1, TID_FINAL_NORM, -1))
    bf(lm + "lm_head.weight", (V, H), O.normal_bf16(V * H, seed, TID_LM_HEAD, sg), (-1, TID_LM_HEAD, -1))
    for l in range(cfg.n_layers):
        b = (l + 1) * 64
        p = f"{lm}model.layers.{l}."
        a = p + "self_attn."
        bf(p + "input_layernorm.weight", (H,), _ln(H, seed, b + TL_INPUT_LN), (l, TL_INPUT_LN, -1))
        bf(a + "q_a_proj.weight", (cfg.q_rank, H), O.normal_bf16(cfg.q_rank * H, seed, b + TL_QA, sg), (l, TL_QA, -1))
        bf(a + "q_a_layernorm.weight", (cfg.q_rank,), _ln(cfg.q_rank, seed, b + TL_QA_LN), (l, TL_QA_LN, -1))
        bf(a + "q_b_proj.weight", (KD, cfg.q_rank), O.normal_bf16(KD * cfg.q_rank, seed, b + TL_QB, sg), (l, TL_QB, -1))
        bf(a + "kv_a_proj_with_mqa.weight", (KVA, H), O.normal_bf16(KVA * H, seed, b + TL_KVA, sg), (l, TL_KVA, -1))
        bf(a + "kv_a_layernorm.weight", (cfg.kv_rank,), _ln(cfg.kv_rank, seed, b + TL_KV_LN), (l, TL_KV_LN, -1))
        bf(a + "kv_b_proj.weight", (KVB, cfg.kv_rank), O.normal_bf16(KVB * cfg.kv_rank, seed, b + TL_KVB, sg), (l, TL_KVB, -1))
        bf(a + "o_proj.weight", (H, VD), O.normal_bf16(H * VD, seed, b + TL_O, sg), (l, TL_O, -1))
        bf(p + "post_attention_layernorm.weight", (H,), _ln(H, seed, b + TL_POST_LN), (l, TL_POST_LN, -1))
        m = p + "mlp."
        if l < cfg.first_dense:
            bf(m + "gate_proj.weight", (D, H), O.normal_bf16(D * H, seed, b + TL_DENSE_GATE, sg), (l, TL_DENSE_GATE, -1))
            bf(m + "up_proj.weight", (D, H), O.normal_bf16(D * H, seed, b + TL_DENSE_UP, sg), (l, TL_DENSE_UP, -1))
            bf(m + "down_proj.weight", (H, D), O.normal_bf16(H * D, seed, b + TL_DENSE_DOWN, sg), (l, TL_DENSE_DOWN, -1))
            continue
        bf(m + "gate.weight", (E, H), O.normal_bf16(E * H, seed, b + TL_ROUTER, float(H) ** -0.5), (l, TL_ROUTER, -1))
        bias16 = O.f32_to_bf16(O.normal_f32(E, seed, b + TL_ROUTER_BIAS, 0.01))  # the checkpoint keeps it in bf16
        out.append((m + "gate.e_score_correction_bias", "BF16", (E,), bias16, (l, TL_ROUTER_BIAS, -1), O.bf16_to_f32(bias16)))
        bf(m + "shared_experts.gate_proj.weight", (SI, H), O.normal_bf16(SI * H, seed, b + TL_SH_GATE, sg), (l, TL_SH_GATE, -1))
        bf(m + "shared_experts.up_proj.weight", (SI, H), O.normal_bf16(SI * H, seed, b + TL_SH_UP, sg), (l, TL_SH_UP, -1))
        bf(m + "shared_experts.down_proj.weight", (H, SI), O.normal_bf16(H * SI, seed, b + TL_SH_DOWN, sg), (l, TL_SH_DOWN, -1))
        packed = {k: O.words_u32(E * I * H // 8, seed, b + t) for k, t in (("gate", TL_GATE_P), ("up", TL_UP_P), ("down", TL_DOWN_P))}
        scales = {k: O.normal_bf16(E * I * H // 32, seed, b + t, es, 1) for k, t in (("gate", TL_GATE_S), ("up", TL_UP_S), ("down", TL_DOWN_S))}
        ids = {"gate": (TL_GATE_P, TL_GATE_S, I, H), "up": (TL_UP_P, TL_UP_S, I, H), "down": (TL_DOWN_P, TL_DOWN_S, H, I)}
        for e in range(E):
            for k, (tp, ts, rows, cols) in ids.items():
                pw = packed[k].reshape(E, -1)[e]
                sc = scales[k].reshape(E, -1)[e]
                x = f"{m}experts.{e}.{k}_proj."
                out.append((x + "weight_packed", "I32", (rows, cols // 8), pw, (l, tp, e), pw))
                out.append((x + "weight_scale", "BF16", (rows, cols // 32), sc, (l, ts, e), sc))
                # compressed-tensors also stores the logical shape; the index writer skips it
                out.append((x + "weight_shape", "I32", (2,), np.array([rows, cols], dtype=np.int32), None, None))
    # decoys: another tower, and a dtype the executor does not run
    out.append(("vision_tower.patch_embed.weight", "BF16", (4, 8), np.arange(32, dtype=np.uint16), None, None))
    out.append((lm + "model.rotary_emb.inv_freq", "F32", (32,), np.arange(32, dtype=np.float32), None, None))
    return out


def write_safetensors(path, entries, pad_to=None):
    """entries: [(name, st_dtype, shape, array)].  pad_to: header length is padded with spaces to a multiple of it."""
    header, blobs, at = {"__metadata__": {"format": "pt"}}, [], 0
    for name, dtype, shape, arr in entries:
        raw = np.ascontiguousarray(arr).tobytes()
        header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    body = json.dumps(header, separators=(",", ":")).encode()
    if pad_to:
        body += b" " * (-len(body) % pad_to)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(body)))
        f.write(body)
        for raw in blobs:
            f.write(raw)


def write_checkpoint(root, cfg, seed, shards=3):
    """Shards under root/; returns [(key, oracle_array)] for the tensors the forward pass reads."""
    root = Path(root)
    root.mkdir(parents=True, exist_ok=True)
    all_t = model_tensors(cfg, seed)
    per = -(-len(all_t) // shards)
    for s in range(shards):
        part = all_t[s * per:(s + 1) * per]
        # odd header lengths put the data at unaligned file offsets, one shard is padded as real files are
        write_safetensors(root / f"model-{s + 1:05d}-of-{shards:06d}.safetensors", [t[:4] for t in part], pad_to=8 if s == 1 else None)
    return [(t[4], t[5]) for t in all_t if t[4] is not None]
