"""A float64 numpy forward pass of the DeepSeek-V3 / Kimi-K2 decoder stack, written from the published model
formulation (the DeepseekV3 model code of the transformers library: RMSNorm, the low-rank q and kv projections,
kv_b_proj split into K-nope and V per head, rotary embedding on de-interleaved pairs with YaRN frequencies,
softmax(q.k * scale) with scale = (nope+rope)^-1/2 * mscale^2, sigmoid router with a selection bias, SwiGLU
experts), NOT from the oracle: whole-prompt causal attention on expanded K/V, no cache, no absorbed form, no
intermediate rounding.  It is the independent witness that pins the wiring of the oracle's model_step
(reference: run(), src/kimi_exec.cu:801-884) and its RoPE rotation (:346-357).

`mutate` names one deliberate mistake; the tests require that each of them breaks the agreement.
"""
import math

import numpy as np

MUTATIONS = ("swap_ln", "drop_attn_residual", "drop_mlp_residual", "norm_all_kva", "rope_sign", "rope_half_split",
             "swap_uk_uv", "no_mscale", "bias_in_weight", "no_routed_scale", "rope_on_nope", "final_norm_skipped",
             "qa_norm_skipped", "shared_dropped")


def bf16_round(a):
    """float -> nearest-even bf16 bit patterns (uint16)"""
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_f64(h):
    return (np.asarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def random_weights(cfg, seed):
    """Every tensor of the stack as the bit patterns the oracle keeps (bf16 -> uint16, packed words uint32,
    router bias float32), from numpy's generator.  Norm weights are spread widely (0.5 .. 1.5) so that a
    mix-up of two of them is visible."""
    rng = np.random.default_rng(seed)
    H, V, E, I, SI, D = cfg.hidden, cfg.vocab, cfg.experts, cfg.moe_inter, cfg.shared_inter, cfg.dense_inter
    KD, VD = cfg.heads * (cfg.qk_nope + cfg.qk_rope), cfg.heads * cfg.v_head
    KVA, KVB = cfg.kv_rank + cfg.qk_rope, cfg.heads * (cfg.qk_nope + cfg.v_head)
    nrm = lambda shape, s: bf16_round(rng.standard_normal(shape) * s)
    ln = lambda n: bf16_round(rng.uniform(0.5, 1.5, n))
    w = {"embed": nrm((V, H), 0.1), "final_norm": ln(H), "lm_head": nrm((V, H), 0.02), "layers": []}
    for l in range(cfg.n_layers):
        L = {"input_ln": ln(H), "qa": nrm((cfg.q_rank, H), 0.02), "qa_ln": ln(cfg.q_rank), "qb": nrm((KD, cfg.q_rank), 0.02),
             "kva": nrm((KVA, H), 0.02), "kv_ln": ln(cfg.kv_rank), "kvb": nrm((KVB, cfg.kv_rank), 0.02),
             "o": nrm((H, VD), 0.02), "post_ln": ln(H)}
        if l < cfg.first_dense:
            L.update(dgate=nrm((D, H), 0.02), dup=nrm((D, H), 0.02), ddown=nrm((H, D), 0.02))
        else:
            L.update(router=nrm((E, H), H ** -0.5), router_bias=(rng.standard_normal(E) * 0.25).astype(np.float32),
                     gate_p=rng.integers(0, 2 ** 32, (E, I, H // 8), dtype=np.uint32),
                     gate_s=bf16_round(np.abs(rng.standard_normal((E, I, H // 32))) * 0.004),
                     up_p=rng.integers(0, 2 ** 32, (E, I, H // 8), dtype=np.uint32),
                     up_s=bf16_round(np.abs(rng.standard_normal((E, I, H // 32))) * 0.004),
                     down_p=rng.integers(0, 2 ** 32, (E, H, I // 8), dtype=np.uint32),
                     down_s=bf16_round(np.abs(rng.standard_normal((E, H, I // 32))) * 0.004),
                     sh_gate=nrm((SI, H), 0.02), sh_up=nrm((SI, H), 0.02), sh_down=nrm((H, SI), 0.04))
        w["layers"].append(L)
    return w


def dequant(packed, scale):
    """compressed-tensors pack_quantized, symmetric INT4, group 32: nibble j of word i is column 8i+j, value q+8."""
    rows, words = packed.shape
    q = ((packed[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 15).astype(np.float64) - 8.0
    q = q.reshape(rows, words * 8)
    return q * np.repeat(bf16_f64(scale), 32, axis=1)


def yarn_inv_freq(cfg):
    """YaRN ("NTK by parts") inverse frequencies, as transformers' _compute_yarn_parameters does them."""
    dim, base, factor = cfg.qk_rope, float(cfg.rope_theta), float(cfg.yarn_factor)
    pos_freqs = base ** (np.arange(0, dim, 2, dtype=np.float64) / dim)
    extrapolation, interpolation = 1.0 / pos_freqs, 1.0 / (factor * pos_freqs)
    corr = lambda rot: dim * math.log(cfg.yarn_orig_ctx / (rot * 2 * math.pi)) / (2 * math.log(base))
    low, high = max(math.floor(corr(cfg.yarn_beta_fast)), 0), min(math.ceil(corr(cfg.yarn_beta_slow)), dim - 1)
    ramp = np.clip((np.arange(dim // 2, dtype=np.float64) - low) / (high - low), 0.0, 1.0)
    extrapolation_factor = 1.0 - ramp
    return interpolation * (1.0 - extrapolation_factor) + extrapolation * extrapolation_factor


def rotate(x, pos, inv_freq, mutate=None):
    """apply_rotary_pos_emb_interleave: x[..., 64] with pairs (2p, 2p+1) is first regrouped into halves
    (even elements, then odd ones), then q*cos + rotate_half(q)*sin.  pos: array broadcastable to x[..., 0]."""
    ang = np.asarray(pos, dtype=np.float64)[..., None] * inv_freq
    cos, sin = np.cos(ang), np.sin(ang)
    if mutate == "rope_sign":
        sin = -sin
    if mutate == "rope_half_split":
        a, b = x[..., :32], x[..., 32:]
    else:
        a, b = x[..., 0::2], x[..., 1::2]
    return np.concatenate([a * cos - b * sin, b * cos + a * sin], axis=-1)


def rms(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def silu(a):
    return a / (1.0 + np.exp(-a))


def forward(cfg, w, ids, mutate=None):
    """ids: int array [P] (one sequence).  Returns dict(hidden [P, H] after the last layer, logits [vocab] of the last
    position, latent: per layer [P, kv_rank + qk_rope] = (normed compressed kv | rotated rope key), margins: per MoE
    layer the smallest gap between the last selected and the first rejected selection score)."""
    assert mutate is None or mutate in MUTATIONS
    P = len(ids)
    nh, dn, dr, dv, R = cfg.heads, cfg.qk_nope, cfg.qk_rope, cfg.v_head, cfg.kv_rank
    eps = float(cfg.rms_eps)
    inv_freq = yarn_inv_freq(cfg)
    mscale = 0.1 * cfg.yarn_mscale_all_dim * math.log(cfg.yarn_factor) + 1.0
    scale = (dn + dr) ** -0.5 * (1.0 if mutate == "no_mscale" else mscale * mscale)
    pos = np.arange(P)
    x = bf16_f64(w["embed"])[np.asarray(ids)]
    latents, margins = [], []
    for l, L in enumerate(w["layers"]):
        W = {k: (bf16_f64(v) if v.dtype == np.uint16 else v) for k, v in L.items()}
        ln_in, ln_post = (W["post_ln"], W["input_ln"]) if mutate == "swap_ln" else (W["input_ln"], W["post_ln"])
        n = rms(x, ln_in, eps)
        qa = n @ W["qa"].T
        if mutate != "qa_norm_skipped":
            qa = rms(qa, W["qa_ln"], eps)
        q = (qa @ W["qb"].T).reshape(P, nh, dn + dr)
        kva = n @ W["kva"].T
        if mutate == "norm_all_kva":
            full = kva / np.sqrt(np.mean(kva * kva, axis=-1, keepdims=True) + eps)
            ckv, kr = full[:, :R] * W["kv_ln"], full[:, R:]
        else:
            ckv, kr = rms(kva[:, :R], W["kv_ln"], eps), kva[:, R:]
        kv = (ckv @ W["kvb"].T).reshape(P, nh, dn + dv)
        k_nope, v = (kv[..., dv:], kv[..., :dv]) if mutate == "swap_uk_uv" else (kv[..., :dn], kv[..., dn:])
        q_nope, q_rope = q[..., :dn], q[..., dn:]
        if mutate == "rope_on_nope":
            q_nope, q_rope = q[..., dr:], q[..., :dr]
        q_rot = rotate(q_rope, pos[:, None], inv_freq, mutate)
        k_rot = rotate(kr, pos, inv_freq, mutate)
        latents.append(np.concatenate([ckv, k_rot], axis=-1))
        s = (np.einsum("phd,thd->hpt", q_nope, k_nope) + np.einsum("phd,td->hpt", q_rot, k_rot)) * scale
        s = np.where(pos[None, :, None] >= pos[None, None, :], s, -np.inf)
        p = np.exp(s - s.max(axis=-1, keepdims=True))
        p /= p.sum(axis=-1, keepdims=True)
        attn = np.einsum("hpt,thd->phd", p, v).reshape(P, nh * dv)
        a_out = attn @ W["o"].T
        x = a_out if mutate == "drop_attn_residual" else x + a_out
        n = rms(x, ln_post, eps)
        if l < cfg.first_dense:
            y = (silu(n @ W["dgate"].T) * (n @ W["dup"].T)) @ W["ddown"].T
        else:
            sc = 1.0 / (1.0 + np.exp(-(n @ W["router"].T)))
            sel = sc + W["router_bias"].astype(np.float64)
            order = np.argsort(-sel, axis=-1, kind="stable")
            top = order[:, :cfg.topk]
            srt = np.take_along_axis(sel, order, axis=-1)
            margins.append(float(np.min(srt[:, cfg.topk - 1] - srt[:, cfg.topk])))
            picked = np.take_along_axis(sel if mutate == "bias_in_weight" else sc, top, axis=-1)
            rw = picked / (picked.sum(axis=-1, keepdims=True) + 1e-20)
            if mutate != "no_routed_scale":
                rw = rw * float(cfg.routed_scale)
            y = np.zeros_like(x)
            for e in np.unique(top):
                tok, slot = np.nonzero(top == e)
                g, u = dequant(L["gate_p"][e], L["gate_s"][e]), dequant(L["up_p"][e], L["up_s"][e])
                d = dequant(L["down_p"][e], L["down_s"][e])
                y[tok] += ((silu(n[tok] @ g.T) * (n[tok] @ u.T)) @ d.T) * rw[tok, slot][:, None]
            if mutate != "shared_dropped":
                y = y + (silu(n @ W["sh_gate"].T) * (n @ W["sh_up"].T)) @ W["sh_down"].T
        x = y if mutate == "drop_mlp_residual" else x + y
    last = x[-1] if mutate == "final_norm_skipped" else rms(x[-1], bf16_f64(w["final_norm"]), eps)
    return dict(hidden=x, logits=last @ bf16_f64(w["lm_head"]).T, latent=latents, margins=margins)
