"""Pins the two oracle functions that both of its schedules share -- the RoPE rotation (rope_apply, restating
rope_k, src/kimi_exec.cu:346-357) and the wiring of a decode step (model_step, restating run(), :801-884) -- against
witnesses that do not come from the oracle: closed-form properties of a rotation, a float64 numpy forward pass
written from the published DeepSeek-V3 formulation (tests/witness.py), and the DeepseekV3 model of the
transformers library given the same weights.  Every check is one that a plausible mistake fails; the witness's
`mutate` cases prove that for the wiring.
"""
import ctypes as C

import numpy as np
import pytest

import oracle as O
import witness as W
from oracle import ptr

TL = dict(input_ln=0, qa=1, qa_ln=2, qb=3, kva=4, kv_ln=5, kvb=6, o=7, post_ln=8, dgate=9, dup=10, ddown=11, router=12,
          router_bias=13, gate_p=14, gate_s=15, up_p=16, up_s=17, down_p=18, down_s=19, sh_gate=20, sh_up=21, sh_down=22)
PER_EXPERT = ("gate_p", "gate_s", "up_p", "up_s", "down_p", "down_s")


# ---- rope_apply ---------------------------------------------------------------------------------
def _table(ox, cfg, pos):
    tab = np.empty(64, dtype=np.uint16)
    ox.ox_rope_table(C.byref(cfg), pos, 1, ptr(tab))
    return tab


def _rope(ox, x, tab):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    ox.ox_rope_apply(ptr(x), ptr(y), ptr(tab), 64)
    return y


def test_rope_position_zero_is_the_deinterleave_permutation(ox):
    cfg = O.small_config()
    x = O.bf16_to_f32(O.normal_bf16(64, 5, 1, 1.0))
    y = _rope(ox, x, _table(ox, cfg, 0))
    assert (y[:32] == x[0::2]).all() and (y[32:] == x[1::2]).all()


def test_rope_is_a_rotation_of_each_pair(ox):
    cfg = O.small_config()
    x = O.bf16_to_f32(O.normal_bf16(64, 5, 2, 1.0))
    for pos in (1, 7, 300, 4095):
        y = _rope(ox, x, _table(ox, cfg, pos)).astype(np.float64)
        n_in = x[0::2].astype(np.float64) ** 2 + x[1::2].astype(np.float64) ** 2
        n_out = y[:32] ** 2 + y[32:] ** 2
        # two bf16 roundings per product and sum, and a rounded cos/sin: 2^-7 relative on the squared norm
        assert np.allclose(n_out, n_in, rtol=2 ** -6, atol=1e-3)
        # against the float64 rotation in the half-split convention of the DeepSeek-V3 model code
        ref = W.rotate(x.astype(np.float64), pos, W.yarn_inv_freq(cfg))
        assert np.max(np.abs(y - ref)) < 2 ** -6 * np.max(np.abs(x))
        # the mistakes this is meant to catch do not pass it
        for bad in ("rope_sign", "rope_half_split"):
            assert np.max(np.abs(y - W.rotate(x.astype(np.float64), pos, W.yarn_inv_freq(cfg), bad))) > 0.1


def test_rope_scores_depend_on_relative_position_only(ox):
    cfg = O.small_config()
    q = O.bf16_to_f32(O.normal_bf16(64, 5, 3, 1.0))
    k = O.bf16_to_f32(O.normal_bf16(64, 5, 4, 1.0))
    dot = lambda m, n: float(_rope(ox, q, _table(ox, cfg, m)).astype(np.float64) @ _rope(ox, k, _table(ox, cfg, n)).astype(np.float64))
    norm = float(np.linalg.norm(q) * np.linalg.norm(k))
    for d in (0, 1, 5, 40):
        vals = [dot(m + d, m) for m in (0, 3, 50, 1000)]
        assert max(vals) - min(vals) < 0.03 * norm, (d, vals)   # rounding only: a sign or pairing slip moves it by O(norm)
    assert abs(dot(40, 0) - dot(0, 0)) > 0.03 * norm            # and the position does matter


# ---- model_step against the float64 witness ------------------------------------------------------
def _load_oracle(cfg, w, mode):
    m = O.OxModel(cfg, mode)
    m.set_tensor(-1, 1, -1, w["embed"])
    m.set_tensor(-1, 2, -1, w["final_norm"])
    m.set_tensor(-1, 3, -1, w["lm_head"])
    for l, L in enumerate(w["layers"]):
        for name, arr in L.items():
            if name in PER_EXPERT:
                for e in range(cfg.experts):
                    m.set_tensor(l, TL[name], e, arr[e])
            else:
                m.set_tensor(l, TL[name], -1, arr)
    return m


@pytest.fixture(scope="module")
def wiring_case():
    cfg = O.small_config(n_layers=3, first_dense=1, batch=1, context=16)
    w = W.random_weights(cfg, 20240607)
    ids = np.random.default_rng(11).integers(0, cfg.vocab, 7).astype(np.uint32)
    runs = {}
    for mode in (0, 1):
        m = _load_oracle(cfg, w, mode)
        rc, out, _ = m.generate(ids.reshape(1, -1), 1)
        assert rc == 0
        runs[mode] = dict(hidden=O.bf16_to_f32(m.hidden(1))[0].astype(np.float64), logits=m.logits(1)[0].astype(np.float64),
                          latent=[O.bf16_to_f32(m.latent(l))[0, :len(ids)].astype(np.float64) for l in range(cfg.n_layers)],
                          first=int(out[0, 0]))
        m.close()
    return cfg, w, ids, runs


def _errors(ref, run):
    """normalised maximum errors of the oracle run against a witness result"""
    e = {"hidden": O.max_rel(run["hidden"], ref["hidden"][-1]), "logits": O.max_rel(run["logits"], ref["logits"])}
    for l, lat in enumerate(ref["latent"]):
        e[f"latent{l}"] = O.max_rel(run["latent"][l], lat)
    return e


@pytest.mark.parametrize("mode", [0, 1])
def test_model_step_agrees_with_float64_witness(wiring_case, mode):
    cfg, w, ids, runs = wiring_case
    ref = W.forward(cfg, w, ids)
    # the routing of the witness must not hang on a near-tie, or a legitimate rounding difference could flip it
    assert min(ref["margins"]) > 2e-3, ref["margins"]
    err = _errors(ref, runs[mode])
    assert max(err.values()) < 2e-2, err
    assert int(np.argmax(ref["logits"])) == runs[mode]["first"]


@pytest.mark.parametrize("mutation", W.MUTATIONS)
def test_witness_mutations_are_noticed(wiring_case, mutation):
    """Each deliberate mistake in the witness must break the agreement: then the same mistake in the oracle would."""
    cfg, w, ids, runs = wiring_case
    err = _errors(W.forward(cfg, w, ids, mutation), runs[1])
    assert max(err.values()) > 5e-2, (mutation, err)


# ---- model_step against the transformers library's DeepseekV3 ------------------------------------
def test_model_step_agrees_with_transformers_deepseek_v3(wiring_case):
    torch = pytest.importorskip("torch")
    pytest.importorskip("transformers")
    from transformers.models.deepseek_v3 import DeepseekV3Config, DeepseekV3ForCausalLM
    cfg, w, ids, runs = wiring_case
    rope = dict(rope_type="yarn", rope_theta=float(cfg.rope_theta), factor=float(cfg.yarn_factor),
                beta_fast=float(cfg.yarn_beta_fast), beta_slow=float(cfg.yarn_beta_slow), mscale=1.0,
                mscale_all_dim=float(cfg.yarn_mscale_all_dim), original_max_position_embeddings=int(cfg.yarn_orig_ctx))
    hc = DeepseekV3Config(
        vocab_size=cfg.vocab, hidden_size=cfg.hidden, intermediate_size=cfg.dense_inter, moe_intermediate_size=cfg.moe_inter,
        num_hidden_layers=cfg.n_layers, num_attention_heads=cfg.heads, num_key_value_heads=cfg.heads, n_shared_experts=1,
        n_routed_experts=cfg.experts, routed_scaling_factor=float(cfg.routed_scale), kv_lora_rank=cfg.kv_rank,
        q_lora_rank=cfg.q_rank, qk_rope_head_dim=cfg.qk_rope, v_head_dim=cfg.v_head, qk_nope_head_dim=cfg.qk_nope, n_group=1,
        topk_group=1, num_experts_per_tok=cfg.topk, first_k_dense_replace=cfg.first_dense, norm_topk_prob=True,
        hidden_act="silu", max_position_embeddings=4096 * 32, rms_norm_eps=float(cfg.rms_eps), rope_parameters=rope,
        rope_interleave=True, attention_bias=False, attention_dropout=0.0, tie_word_embeddings=False,
        attn_implementation="eager", experts_implementation="eager")
    # the shared expert of this stack is narrower than a routed one; the library sizes it moe_inter * n_shared
    assert cfg.shared_inter * 2 == cfg.moe_inter
    torch.manual_seed(0)
    with torch.device("cpu"):
        model = DeepseekV3ForCausalLM(hc).to(torch.float64).eval()
    t = lambda a: torch.from_numpy(W.bf16_f64(a).copy())
    sd = {"model.embed_tokens.weight": t(w["embed"]), "model.norm.weight": t(w["final_norm"]), "lm_head.weight": t(w["lm_head"])}
    for l, L in enumerate(w["layers"]):
        p = f"model.layers.{l}."
        sd.update({p + "input_layernorm.weight": t(L["input_ln"]), p + "post_attention_layernorm.weight": t(L["post_ln"]),
                   p + "self_attn.q_a_proj.weight": t(L["qa"]), p + "self_attn.q_a_layernorm.weight": t(L["qa_ln"]),
                   p + "self_attn.q_b_proj.weight": t(L["qb"]), p + "self_attn.kv_a_proj_with_mqa.weight": t(L["kva"]),
                   p + "self_attn.kv_a_layernorm.weight": t(L["kv_ln"]), p + "self_attn.kv_b_proj.weight": t(L["kvb"]),
                   p + "self_attn.o_proj.weight": t(L["o"])})
        if l < cfg.first_dense:
            sd.update({p + "mlp.gate_proj.weight": t(L["dgate"]), p + "mlp.up_proj.weight": t(L["dup"]),
                       p + "mlp.down_proj.weight": t(L["ddown"])})
        else:
            gu = np.stack([np.concatenate([W.dequant(L["gate_p"][e], L["gate_s"][e]), W.dequant(L["up_p"][e], L["up_s"][e])])
                           for e in range(cfg.experts)])
            dn = np.stack([W.dequant(L["down_p"][e], L["down_s"][e]) for e in range(cfg.experts)])
            zero = lambda a: np.concatenate([W.bf16_f64(a), np.zeros_like(W.bf16_f64(a))])      # pad the shared expert to moe_inter
            sd.update({p + "mlp.gate.weight": t(L["router"]),
                       p + "mlp.gate.e_score_correction_bias": torch.from_numpy(L["router_bias"].astype(np.float64)),
                       p + "mlp.experts.gate_up_proj": torch.from_numpy(gu), p + "mlp.experts.down_proj": torch.from_numpy(dn),
                       p + "mlp.shared_experts.gate_proj.weight": torch.from_numpy(zero(L["sh_gate"])),
                       p + "mlp.shared_experts.up_proj.weight": torch.from_numpy(zero(L["sh_up"])),
                       p + "mlp.shared_experts.down_proj.weight": torch.from_numpy(
                           np.concatenate([W.bf16_f64(L["sh_down"]), np.zeros_like(W.bf16_f64(L["sh_down"]))], axis=1))})
    missing, unexpected = model.load_state_dict(sd, strict=False)
    assert not unexpected and all("rotary" in k or "inv_freq" in k for k in missing), (missing, unexpected)
    with torch.no_grad():
        out = model(input_ids=torch.from_numpy(ids.astype(np.int64))[None], output_hidden_states=True, use_cache=False)
    logits = out.logits[0, -1].numpy()
    for mode in (0, 1):
        assert O.max_rel(runs[mode]["logits"], logits) < 2e-2
        assert int(np.argmax(logits)) == runs[mode]["first"]
    # and the float64 witness is the same function as the library's model, far below the rounding of the oracle
    # (the library norms, rotates and normalises the softmax in float32 whatever the model's dtype)
    ref = W.forward(cfg, w, ids)
    assert O.max_rel(ref["logits"], logits) < 1e-4
