"""Pins the oracle's RoPE/YaRN, attention and stack functions without a GPU.

The reference holds no vector for them (src/kimi_exec.cu:325-357, :414-475, :780-893), so the
checks are closed forms and the algebraic identity between the reference's expanded K/V
attention (mode 0) and the absorbed latent form the kernels use (mode 1).
"""
import ctypes as C
import math

import numpy as np
import pytest

import oracle as O
from oracle import ptr


def test_yarn_frequencies_closed_form(ox):
    cfg = O.small_config()
    inv = np.array([ox.ox_yarn_inv_freq(C.byref(cfg), p) for p in range(32)], dtype=np.float32)
    extra = np.array([50000.0 ** (-2.0 * p / 64.0) for p in range(32)])
    # correction range for theta 50000, 64 rotary dims, original context 4096: low 8, high 20
    cd = lambda rot: 64 * math.log(4096 / (rot * 2 * math.pi)) / (2 * math.log(50000.0))
    assert math.floor(cd(32)) == 8 and math.ceil(cd(1)) == 20
    assert np.allclose(inv[:9], extra[:9], rtol=1e-6)                 # below the ramp: unscaled
    assert np.allclose(inv[20:], extra[20:] / 32.0, rtol=1e-6)        # above: divided by the factor
    ramp = (np.arange(9, 20) - 8) / 12.0
    assert np.allclose(inv[9:20], extra[9:20] / 32.0 * ramp + extra[9:20] * (1 - ramp), rtol=1e-5)
    assert np.all(np.diff(inv) < 0)


def test_rope_table_and_scale(ox):
    cfg = O.small_config()
    tab = np.empty((40, 64), dtype=np.uint16)
    ox.ox_rope_table(C.byref(cfg), 0, 40, ptr(tab))
    f = O.bf16_to_f32(tab)
    assert (f[0, :32] == 1.0).all() and (f[0, 32:] == 0.0).all()      # position 0 is the identity
    inv = np.array([ox.ox_yarn_inv_freq(C.byref(cfg), p) for p in range(32)], dtype=np.float64)
    pos = np.arange(40)[:, None]
    assert np.allclose(f[:, :32], np.cos(pos * inv), atol=2 ** -8)
    assert np.allclose(f[:, 32:], np.sin(pos * inv), atol=2 ** -8)
    assert np.allclose(f[:, :32] ** 2 + f[:, 32:] ** 2, 1.0, atol=2 ** -6)
    rs, ms = C.c_float(), C.c_float()
    ox.ox_softmax_scale(C.byref(cfg), C.byref(rs), C.byref(ms))
    assert abs(ms.value - 1.346574) < 1e-5                             # 0.1 * ln(32) + 1
    assert abs(rs.value * ms.value ** 2 - 0.130861) < 1e-5             # BASELINE config 3 scale
    cfg.yarn_factor = 64.0                                              # the reference's pinned factor (:184)
    ox.ox_softmax_scale(C.byref(cfg), C.byref(rs), C.byref(ms))
    assert abs(rs.value * ms.value ** 2 - 0.144680) < 1e-5


def test_span_policy(ox):
    assert [ox.ox_mla_span_tiles(s) for s in (1, 64, 4096, 4097, 32768, 131072)] == [1, 1, 1, 2, 8, 32]


@pytest.fixture(scope="module")
def small_runs():
    """Both schedules on the same seeded small stack: prompt 20, 12 new tokens, batch 2."""
    cfg = O.small_config(batch=2)
    prompt = O.tokens_u32(2 * 20, cfg.seed, 4, cfg.vocab).reshape(2, 20)
    res = {}
    for mode in (0, 1):
        m = O.OxModel(cfg, mode)
        rc, out, counts = m.generate(prompt, 12)
        assert rc == 0
        res[mode] = dict(out=out, counts=counts, logits=m.logits(2), hidden=m.hidden(2), latent=m.latent(1))
        m.close()
    return cfg, prompt, res


def test_absorbed_attention_equals_expanded(small_runs):
    # mode 0 runs the reference's expanded K/V three-pass softmax, mode 1 the absorbed latent form with
    # the online softmax: same mathematics, different rounding.  Compared where both have seen the same
    # tokens: the latent cache rows of the prompt and the first sampled ids.
    cfg, prompt, res = small_runs
    l0, l1 = res[0]["latent"][:, :20], res[1]["latent"][:, :20]
    assert O.max_rel(O.bf16_to_f32(l1), O.bf16_to_f32(l0)) < 1e-2
    assert (res[0]["out"][:, 0] == res[1]["out"][:, 0]).all()


def test_generate_is_deterministic_and_batch_independent(ox):
    cfg2 = O.small_config(batch=2)
    prompt = O.tokens_u32(2 * 12, cfg2.seed, 4, cfg2.vocab).reshape(2, 12)
    m = O.OxModel(cfg2, 1)
    rc, out2, _ = m.generate(prompt, 6)
    m.close()
    cfg1 = O.small_config(batch=1)
    for b in range(2):
        m = O.OxModel(cfg1, 1)
        rc, out1, _ = m.generate(prompt[b:b + 1], 6)
        m.close()
        assert (out1[0] == out2[b]).all()       # a sequence does not depend on its batch neighbours


@pytest.mark.parametrize("mode", [0, 1])
def test_experts_on_demand_equal_the_whole_tensors(ox, mode):
    # A model that produces a routed expert when a token first selects it (what lets the 24-layer stack fit in host
    # memory) must be the model that holds every expert: ids, logits, hidden state, cache rows to the bit -- also when
    # it keeps at most three experts at a time (each step then produces its experts again), and with an expert's
    # tensors handed over from outside, which must survive the dropping.
    cfg = O.small_config(batch=2, context=40)
    prompt = O.tokens_u32(2 * 9, cfg.seed, 4, cfg.vocab).reshape(2, 9)
    whole = O.OxModel(cfg, mode)
    given = O.words_u32(cfg.moe_inter * cfg.hidden // 8, 99, 1)
    runs = []
    for m, keep in ((whole, None), (O.OxModel(cfg, mode, experts_on_demand=True), None),
                    (O.OxModel(cfg, mode, experts_on_demand=True), 3)):
        if keep:
            ox.ox_model_keep_experts(m.h, keep)
        for e in range(cfg.experts):      # every expert of layer 1 gets the same foreign gate_proj words
            m.set_tensor(1, 14, e, given)
        rc, out, counts = m.generate(prompt, 7)
        assert rc == 0
        runs.append((out, counts, m.logits(2).view(np.uint32), m.hidden(2), m.latent(1), m.latent(2)))
        if m is not whole:
            made = ox.ox_model_experts_produced(m.h)
            # 2 MoE layers x 16 experts exist; with room for all of them none is produced twice
            assert (made <= 32) if keep is None else (made > 32), made
        m.close()
    for other in runs[1:]:
        assert all((a == b).all() for a, b in zip(runs[0], other))
    # and the foreign words did change the result (the hand-over is not a no-op)
    plain = O.OxModel(cfg, mode, experts_on_demand=True)
    rc, out_p, _ = plain.generate(prompt, 7)
    assert not (plain.logits(2).view(np.uint32) == runs[0][2]).all()
    plain.close()


def test_step_by_step_equals_generate(ox):
    cfg = O.small_config(batch=2, context=24)
    prompt = O.tokens_u32(2 * 6, cfg.seed, 4, cfg.vocab).reshape(2, 6)
    m = O.OxModel(cfg, 1)
    rc, out, _ = m.generate(prompt, 5)
    logits, hidden = m.logits(2), m.hidden(2)
    m.close()
    m = O.OxModel(cfg, 1, experts_on_demand=True)
    got, nxt = [], None
    for pos in range(6 + 4):
        ids = prompt[:, pos] if pos < 6 else nxt
        nxt = m.step(ids, pos, pos >= 5)
        if nxt is not None:
            got.append(nxt)
    assert (np.stack(got, axis=1) == out).all()
    assert (m.logits(2).view(np.uint32) == logits.view(np.uint32)).all() and (m.hidden(2) == hidden).all()
    with pytest.raises(ValueError):
        m.step(np.array([cfg.vocab, 0]), 3, False)
    with pytest.raises(ValueError):
        m.step(prompt[:, 0], cfg.max_context, False)
    m.close()


def test_generate_eos_and_argument_rules(ox):
    cfg = O.small_config()
    prompt = O.tokens_u32(10, cfg.seed, 4, cfg.vocab).reshape(1, 10)
    m = O.OxModel(cfg, 1)
    rc, out, counts = m.generate(prompt, 8)
    assert rc == 0 and counts[0] == 8
    m.close()
    # make the third generated id the end-of-sequence id: generation stops before emitting it (:887-888)
    cfg.eos_id = int(out[0, 2])
    first = int(np.argmax(out[0] == out[0, 2]))
    m = O.OxModel(cfg, 1)
    rc, out_e, counts_e = m.generate(prompt, 8, ignore_eos=False)
    assert rc == 0 and counts_e[0] == first and (out_e[0, :first] == out[0, :first]).all()
    rc, out_i, counts_i = m.generate(prompt, 8, ignore_eos=True)
    assert counts_i[0] == 8 and (out_i == out).all()
    # requested sequence exceeds the context (:784); token id outside the vocabulary (:552)
    assert m.generate(prompt, cfg.max_context)[0] == 1
    bad = prompt.copy(); bad[0, 3] = cfg.vocab
    assert m.generate(bad, 2)[0] == 1
    m.close()


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("seq", [1, 64, 65, 300])
def test_mla_decode_against_float64_softmax(ox, mode, seq):
    from blok_amd.lib import default_config
    cfg = default_config()
    H, KVA, R = cfg.heads, 576, 512
    cache = O.normal_bf16(seq * KVA, 3, 1, 1.0).reshape(1, seq, KVA)
    qabs = O.bf16_to_f32(O.normal_bf16(H * KVA, 3, 2, 0.25)).reshape(1, H, KVA)
    out = np.empty((1, H, R), dtype=np.uint16)
    ox.ox_mla_decode(C.byref(cfg), ptr(cache), seq * KVA, ptr(qabs), ptr(out), 1, seq, mode)
    rs, ms = C.c_float(), C.c_float()
    ox.ox_softmax_scale(C.byref(cfg), C.byref(rs), C.byref(ms))
    c = O.bf16_to_f32(cache).astype(np.float64)
    s = np.einsum("bhk,btk->bht", qabs.astype(np.float64), c) * rs.value * ms.value ** 2
    p = np.exp(s - s.max(axis=2, keepdims=True))
    p /= p.sum(axis=2, keepdims=True)
    ref = np.einsum("bht,btr->bhr", p, c[:, :, :R])
    # the scores are rounded to bf16 twice (:429), which moves a probability by up to 2^-8 * |s|
    assert O.max_rel(O.bf16_to_f32(out), ref) < 1.5e-2
    if seq == 1:
        assert (out[0] == cache[0, 0, :R]).all()      # softmax over one position: the latent itself
