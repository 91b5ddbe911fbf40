"""GPU parity of the decoder stack (prefill, decode step, greedy sample, generate) and of the
attention operators, through the C ABI, against the oracle.

Bar: greedy token ids identical to the oracle's kx schedule; hidden state, logits and latent
cache bit-exact against it; first-step logits within max-rel 1e-2 of the reference schedule.
"""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from kxt import assert_excused, check, dev, judge_sequences, routing_of, say
from oracle import ptr

pytestmark = pytest.mark.gpu
from blok_amd.lib import DevBuf, default_config  # noqa: E402


class KxModel:
    def __init__(self, lib, cfg):
        self.lib, self.cfg = lib, cfg
        self.h = C.c_void_p()
        check(lib.kx_model_create(C.byref(cfg), C.byref(self.h)))

    def generate(self, prompt, n_tokens, ignore_eos=True):
        B, P = prompt.shape
        out = np.zeros((B, n_tokens), dtype=np.uint32)
        counts = np.zeros(B, dtype=np.int32)
        rc = self.lib.kx_generate(self.h, ptr(np.ascontiguousarray(prompt)), B, P, n_tokens, int(ignore_eos), ptr(out), ptr(counts))
        return rc, out, counts

    def hidden(self, B):
        out = np.empty((B, self.cfg.hidden), dtype=np.uint16)
        check(self.lib.kx_model_hidden(self.h, ptr(out)))
        return out

    def logits(self, B):
        out = np.empty((B, self.cfg.vocab), dtype=np.float32)
        check(self.lib.kx_model_logits(self.h, ptr(out)))
        return out

    def latent(self, layer, b, n):
        out = np.empty((n, self.cfg.kv_rank + self.cfg.qk_rope), dtype=np.uint16)
        check(self.lib.kx_model_latent(self.h, layer, b, 0, n, ptr(out)))
        return out

    def close(self):
        if self.h:
            self.lib.kx_model_destroy(self.h)
            self.h = None



# The sequences a tolerance path may differ on, for the fixed seeds of the tests below: (sequence, "router" or
# "argmax", first MoE layer whose expert set differs).  Every entry was checked when it was recorded -- the reference
# run's selection gap in that layer is below kxt.NEAR_TIE, or its two largest logits lie closer than the bar -- and
# judge_sequences checks it again on every run.  A set that changes means the arithmetic of a kernel changed.
EITHER = "either way"  # a tie of the reference's two largest logits: see kxt.assert_excused
EXCUSED_SMALL_STACK = {(16, 1): [], (16, 0): [], (8, 1): [], (8, 0): [], (5, 1): [], (5, 0): [],
                       (40, 1): [("sequence 16", "argmax", None, EITHER)], (40, 0): [("sequence 16", "argmax", None, EITHER)]}
EXCUSED_ATTENTION_PATHS = []
# sequence 7: the reference run's two largest logits are equal to the bit; the matrix-core attention kernel with the
# two products on different waves broke the tie one way, the f16 routed kernel of 32 sequences the other
EXCUSED_AGAINST_SINGLE = {16: [("sequence 0", "router", 1), ("sequence 7", "argmax", None, EITHER)],
                          32: [("sequence 0", "router", 1), ("sequence 20", "router", 1), ("sequence 29", "argmax", None),
                               ("sequence 7", "argmax", None, EITHER)]}


def test_rope_table_matches_oracle(kxlib, ox):
    cfg = O.small_config()
    a = np.empty((300, 64), dtype=np.uint16)
    b = np.empty((300, 64), dtype=np.uint16)
    check(kxlib.kx_rope_table(C.byref(cfg), 5, 300, ptr(a)))
    ox.ox_rope_table(C.byref(cfg), 5, 300, ptr(b))
    assert (a == b).all()
    r1, m1, r2, m2 = C.c_float(), C.c_float(), C.c_float(), C.c_float()
    check(kxlib.kx_softmax_scale(C.byref(cfg), C.byref(r1), C.byref(m1)))
    ox.ox_softmax_scale(C.byref(cfg), C.byref(r2), C.byref(m2))
    assert r1.value == r2.value and m1.value == m2.value


@pytest.mark.parametrize("batch,prompt_len,n_tokens", [(1, 20, 24), (3, 9, 10), (2, 70, 6)])
def test_small_stack_tokens_identical(kxlib, ox, batch, prompt_len, n_tokens):
    say(f"small stack batch={batch} prompt={prompt_len} tokens={n_tokens}")
    cfg = O.small_config(batch=batch, context=96)
    prompt = O.tokens_u32(batch * prompt_len, cfg.seed, 4, cfg.vocab).reshape(batch, prompt_len)
    km = KxModel(kxlib, cfg)
    rc, out, counts = km.generate(prompt, n_tokens)
    assert rc == 0, kxlib.kx_last_error()
    om = O.OxModel(cfg, 1)
    rc, out1, counts1 = om.generate(prompt, n_tokens)
    assert rc == 0
    total = prompt_len + n_tokens - 1
    for layer in range(cfg.n_layers):
        lat = om.latent(layer)
        for b in range(batch):
            got = km.latent(layer, b, total)
            assert (got == lat[b, :total]).all(), f"latent cache layer {layer} seq {b} differs"
    assert (km.hidden(batch) == om.hidden(batch)).all()
    assert (km.logits(batch).view(np.uint32) == om.logits(batch).view(np.uint32)).all()
    assert (out == out1).all(), f"tokens differ:\n{out}\n{out1}"
    assert (counts == counts1).all()
    # reference schedule (expanded K/V, three-pass softmax, per-weight dequant) on the same prompt.  The
    # 1e-2 bar is per operator on identical inputs (operator tests); through a whole stack the bf16
    # rounding differences of every layer compound, so the logits of the first sampled step are held
    # to 3e-2 here and the sampled ids must agree.
    om0 = O.OxModel(cfg, 0)
    rc, out0, _ = om0.generate(prompt, 1)
    km1 = KxModel(kxlib, cfg)
    rc, o1, _ = km1.generate(prompt, 1)
    err = O.max_rel(km1.logits(batch), om0.logits(batch))
    print(f"stack logits vs reference schedule: max-rel {err:.3e}")
    assert err < 3e-2
    assert (o1 == out0).all()
    for m in (km, km1, om, om0):
        m.close()


@pytest.mark.parametrize("batch", [16, 8, 5, 40])
def test_small_stack_matrix_core_projections(kxlib, ox, batch):
    # from 5 sequences on the dense projections and the shared expert run as MFMA GEMMs (another summation order): the logits of the first
    # sampled step are held to the stack-level 3e-2 against both oracle schedules, not to the bits (batch 40: beyond
    # one 32-token tile the projections take the prefill GEMM kernel)
    say(f"small stack batch={batch} (dense projections on the matrix cores)")
    # Per sequence: logits within 3e-2 and the same first id.  The only excuses are the two a tolerance path has in a
    # MoE stack, and each is checked and named: the sequence's expert set differs from the bit-exact path's because
    # that path's own selection was a near-tie there, or the two largest logits lie closer than the tolerance.  The
    # routing of the bit-exact path comes from the same sequences run four at a time (GEMV kernels, equal to the
    # oracle's kx schedule to the bit, as the tests above establish).
    prompt_len = 5
    cfg = O.small_config(batch=batch, context=32)
    prompt = O.tokens_u32(batch * prompt_len, cfg.seed, 4, cfg.vocab).reshape(batch, prompt_len)
    km = KxModel(kxlib, cfg)
    check(kxlib.kx_model_set_routing_record(km.h, 1))
    rc, out, _ = km.generate(prompt, 1)
    assert rc == 0, kxlib.kx_last_error()
    got, routes = km.logits(batch), routing_of(kxlib, km.h, cfg, batch)
    ref_routes = {l: ([], []) for l in routes}
    for b0 in range(0, batch, 4):
        nb = min(4, batch - b0)
        rc, _, _ = km.generate(prompt[b0:b0 + nb], 1)
        assert rc == 0, kxlib.kx_last_error()
        for l, (sets, gaps) in routing_of(kxlib, km.h, cfg, nb).items():
            ref_routes[l][0].extend(sets)
            ref_routes[l][1].extend(gaps.tolist())
    km.close()
    names = [f"sequence {b}" for b in range(batch)]
    for mode in (1, 0):
        om = O.OxModel(cfg, mode)
        rc, out_o, _ = om.generate(prompt, 1)
        assert rc == 0
        ref = om.logits(batch)
        errs = [O.max_rel(got[b], ref[b]) for b in range(batch)]
        excused = judge_sequences(names, errs, 3e-2, routes, ref_routes, out[:, 0], out_o[:, 0], ref)
        print(f"batch-{batch} stack vs oracle mode {mode}: worst logits max-rel {max(errs):.3e}; excused: {excused or 'none'}", flush=True)
        assert_excused(excused, EXCUSED_SMALL_STACK[batch, mode], f"small stack, batch {batch}, oracle mode {mode}")
        om.close()


def test_prefill_decode_sample_entry_points(kxlib, ox):
    cfg = O.small_config(batch=2, context=64)
    prompt = O.tokens_u32(2 * 7, cfg.seed, 4, cfg.vocab).reshape(2, 7)
    km = KxModel(kxlib, cfg)
    rc, ref, _ = km.generate(prompt, 5)
    assert rc == 0
    check(kxlib.kx_prefill(km.h, ptr(prompt), 2, 7))
    ids = np.zeros(2, dtype=np.uint32)
    got = []
    check(kxlib.kx_greedy_sample(km.h, ptr(ids)))
    got.append(ids.copy())
    check(kxlib.kx_decode_step(km.h, None))           # feeds the device-resident ids
    check(kxlib.kx_greedy_sample(km.h, ptr(ids)))
    got.append(ids.copy())
    check(kxlib.kx_decode_step(km.h, ptr(ids)))       # feeds host ids
    check(kxlib.kx_greedy_sample(km.h, ptr(ids)))
    got.append(ids.copy())
    assert (np.stack(got, axis=1) == ref[:, :3]).all()
    km.close()


def test_eos_and_errors(kxlib, ox):
    cfg = O.small_config(batch=1, context=40)
    prompt = O.tokens_u32(10, cfg.seed, 4, cfg.vocab).reshape(1, 10)
    km = KxModel(kxlib, cfg)
    rc, out, counts = km.generate(prompt, 8)
    assert rc == 0 and counts[0] == 8
    km.close()
    cfg.eos_id = int(out[0, 2])
    first = int(np.argmax(out[0] == out[0, 2]))
    km = KxModel(kxlib, cfg)
    rc, out_e, counts_e = km.generate(prompt, 8, ignore_eos=False)
    assert rc == 0 and counts_e[0] == first and (out_e[0, :first] == out[0, :first]).all()
    # the loop ends once every sequence has sampled the end-of-sequence id (:887-888); the ids are looked at every
    # eighth step, so of 28 steps asked for 8 are decoded; with ignore_eos all of them
    steps = C.c_int32()
    rc, out_l, counts_l = km.generate(prompt, 28, ignore_eos=False)
    assert rc == 0 and counts_l[0] == first and (out_l[0, :first] == out[0, :first]).all()
    check(kxlib.kx_model_steps_decoded(km.h, C.byref(steps)))
    assert steps.value == 8
    rc, out_l, counts_l = km.generate(prompt, 28, ignore_eos=True)
    check(kxlib.kx_model_steps_decoded(km.h, C.byref(steps)))
    assert rc == 0 and counts_l[0] == 28 and steps.value == 28 and (out_l[0, :8] == out[0]).all()
    assert km.generate(prompt, 31)[0] != 0 and b"context" in kxlib.kx_last_error()
    bad = prompt.copy(); bad[0, 1] = cfg.vocab
    assert km.generate(bad, 2)[0] != 0 and b"vocabulary" in kxlib.kx_last_error()
    two = np.zeros((2, 4), dtype=np.uint32)
    assert km.generate(two, 2)[0] != 0 and b"batch" in kxlib.kx_last_error()
    km.close()
    bad_cfg = O.small_config()
    bad_cfg.kv_rank = 256
    h = C.c_void_p()
    assert kxlib.kx_model_create(C.byref(bad_cfg), C.byref(h)) != 0


@pytest.mark.parametrize("batch,plen,n_tokens", [(1, 70, 32), (3, 6, 5)])
def test_config5_24_layer_stack_tokens_identical_to_the_oracle(kxlib, ox, capsys, batch, plen, n_tokens):
    # BASELINE config 5's stack at its full depth and width -- 24 layers (one dense, 23 MoE of 384 experts), vocabulary
    # 163840, 231 GB resident on the GPU -- against the CPU oracle's kx schedule (generate(), :885-890; run(),
    # :801-884).  The oracle holds the dense tensors and produces a routed expert when a token first selects it (the
    # generator is a function of seed, tensor and index; the CPU suite checks that such a model equals the one holding
    # every expert), which makes 24 layers fit in host memory.  One sequence: a 70-token prompt crosses the 64-position
    # tile of the attention kernel; 32 greedy tokens follow (the path of the resident launches).  Three sequences, a
    # short run: the kernels that take two to four tokens per pass, at the full depth.  Required: every sampled id
    # identical, the logits of every sampled step identical to the bit, and at the end the hidden state and the cache
    # rows of all 24 layers identical to the bit.  The top-1/top-2 margin of every sampled step is printed: identity
    # is not owed to wide margins alone when some of them are a few bf16 steps.  The oracle takes about half a second
    # a step and sequence on sixteen cores: progress is printed.
    import time
    say(f"config 5, 24 layers, batch {batch}, prompt {plen}, {n_tokens} tokens against the oracle")
    cfg = default_config()
    cfg.max_batch, cfg.max_context, cfg.seed = batch, plen + n_tokens, 0
    assert cfg.n_layers == 24 and cfg.first_dense == 1 and cfg.experts == 384 and cfg.vocab == 163840
    prompt = O.tokens_u32(batch * plen, cfg.seed, 4, cfg.vocab).reshape(batch, plen)

    def note(msg):
        with capsys.disabled():
            print("  " + msg, flush=True)

    km = KxModel(kxlib, cfg)
    check(kxlib.kx_prefill(km.h, ptr(prompt), batch, plen))
    ids_gpu, logits_gpu = [], []
    got = np.zeros(batch, dtype=np.uint32)
    for i in range(n_tokens):
        if i:
            check(kxlib.kx_decode_step(km.h, None))        # feeds the ids sampled on the device
        check(kxlib.kx_greedy_sample(km.h, ptr(got)))
        ids_gpu.append(got.copy())
        logits_gpu.append(km.logits(batch).view(np.uint32).copy())
    hidden_gpu = km.hidden(batch)
    total = plen + n_tokens - 1
    rows_gpu = [[km.latent(layer, b, total) for b in range(batch)] for layer in range(cfg.n_layers)]
    km.close()
    note(f"GPU ids {[g.tolist() for g in ids_gpu]}")

    om = O.OxModel(cfg, 1, experts_on_demand=True)
    t0 = time.time()
    for pos in range(plen - 1):
        om.step(np.ascontiguousarray(prompt[:, pos]), pos, False)
        if pos % 8 == 7:
            note(f"oracle: prompt position {pos + 1} of {plen}, {time.time() - t0:.0f} s")
    cur = np.ascontiguousarray(prompt[:, plen - 1])
    for i in range(n_tokens):
        nxt = om.step(cur, plen - 1 + i, True)
        lg = om.logits(batch)
        margins = []
        for b in range(batch):
            top = np.sort(lg[b])[-2:]
            margins.append(float((top[1] - top[0]) / (abs(top[1]) * 2.0 ** -8)))      # in bf16 steps of the winner
        note(f"token {i}: oracle {nxt.tolist()} GPU {ids_gpu[i].tolist()}; top-1 and top-2 "
             f"{', '.join('%.1f' % m for m in margins)} bf16 steps apart; {time.time() - t0:.0f} s")
        assert (nxt == ids_gpu[i]).all(), f"token {i}: the oracle samples {nxt.tolist()}, the GPU {ids_gpu[i].tolist()}"
        bad = int(np.count_nonzero(lg.view(np.uint32) != logits_gpu[i]))
        assert bad == 0, f"token {i}: {bad} of {lg.size} logits differ"
        cur = nxt.copy()
    assert (om.hidden(batch) == hidden_gpu).all(), "final hidden state differs"
    for layer in range(cfg.n_layers):
        lat = om.latent(layer)
        for b in range(batch):
            assert (lat[b, :total] == rows_gpu[layer][b]).all(), f"cache rows of layer {layer}, sequence {b} differ"
    note(f"24 layers: {n_tokens} x {batch} ids, their logits, the hidden states and {cfg.n_layers} x {batch} x {total} cache rows "
         f"identical; {ox.ox_model_experts_produced(om.h)} experts produced by the oracle")
    om.close()


def test_kimi_shape_truncated_stack_tokens_identical(kxlib, ox):
    # Kimi-K2 shapes (BASELINE config 5) truncated to the dense layer and one MoE layer, full vocabulary
    say("kimi shape 2-layer stack")
    cfg = default_config()
    cfg.n_layers, cfg.first_dense, cfg.max_batch, cfg.max_context, cfg.seed = 2, 1, 1, 32, 7
    prompt = O.tokens_u32(6, cfg.seed, 4, cfg.vocab).reshape(1, 6)
    km = KxModel(kxlib, cfg)
    rc, out, _ = km.generate(prompt, 4)
    assert rc == 0, kxlib.kx_last_error()
    om = O.OxModel(cfg, 1, experts_on_demand=True)
    rc, out1, _ = om.generate(prompt, 4)
    assert rc == 0
    assert (km.hidden(1) == om.hidden(1)).all()
    assert (out == out1).all(), f"{out} vs {out1}"
    km.close(); om.close()


def test_kimi_shape_stack_batch_invariance(kxlib, ox):
    # Properties that need no oracle, at Kimi-K2 shapes (4 layers: 1 dense + 3 MoE, full vocabulary): the summation
    # order of every kernel on the path is independent of the batch, so identical prompts in a batch of 2, 3 or 4 (the
    # 2- and 4-token kernel variants with their own launch plans, fused prologues) give the ids, hidden state and
    # logits of the batch-1 run (1-token variants) to the bit, run after run, and a longer generation extends a
    # shorter one.
    say("kimi shape 4-layer stack, batch invariance")
    cfg = default_config()
    cfg.n_layers, cfg.first_dense, cfg.max_context, cfg.seed = 4, 1, 48, 5
    prompt_len, n_tokens = 9, 12
    one = O.tokens_u32(prompt_len, cfg.seed, 4, cfg.vocab).reshape(1, prompt_len)
    runs = {}
    for batch in (1, 2, 3, 4, 1):
        cfg.max_batch = batch
        km = KxModel(kxlib, cfg)
        rc, out, counts = km.generate(np.repeat(one, batch, axis=0), n_tokens)
        assert rc == 0, kxlib.kx_last_error()
        got = (out, km.hidden(batch), km.logits(batch).view(np.uint32))
        if batch in runs:   # the same run again: deterministic
            assert all((a == b).all() for a, b in zip(got, runs[batch]))
        runs[batch] = got
        if batch == 1:
            rc, short, _ = km.generate(one, 5)
            assert rc == 0 and (short[0] == out[0, :5]).all()
        km.close()
    o1, h1, l1 = runs[1]
    for batch in (2, 3, 4):
        ob, hb, lb = runs[batch]
        for b in range(batch):
            assert (ob[b] == o1[0]).all(), f"batch {batch}, row {b}: {ob[b]} vs {o1[0]}"
            assert (hb[b] == h1[0]).all() and (lb[b] == l1[0]).all(), f"batch {batch}, row {b}"


@pytest.mark.parametrize("shape", ["small-1", "small-3", "kimi"])
def test_fused_and_separate_launches_agree(kxlib, ox, shape):
    # the q_b GEMV that finishes the query in its own launch, (batch 1) the routed down launch that finishes the MoE
    # layer, and (batch 1, Kimi shapes) the resident launches that run the whole front of the attention block and its
    # back (bit 3; with bit 4 the head of the MoE layer behind it: norm, router, routing, shared gate/up) and the routed
    # experts with the layer's tail (bit 5), against the same steps as kernels of their own: cache rows, hidden state, logits and ids to the bit (the oracle
    # comparisons above run the fused forms)
    say(f"fusion on/off {shape}")
    if shape == "kimi":
        cfg = default_config()
        cfg.n_layers, cfg.first_dense, cfg.max_batch, cfg.max_context, cfg.seed = 2, 1, 1, 32, 11
        batch, prompt_len, n_tokens = 1, 5, 4
    else:
        batch = int(shape[-1])
        cfg = O.small_config(batch=batch, context=64)
        prompt_len, n_tokens = 11, 9
    prompt = O.tokens_u32(batch * prompt_len, cfg.seed, 4, cfg.vocab).reshape(batch, prompt_len)
    got = []
    for mask in (63, 0, 1, 2, 3, 4, 8, 15, 24, 31, 34):
        km = KxModel(kxlib, cfg)
        check(kxlib.kx_model_set_fusion(km.h, mask))
        rc, out, _ = km.generate(prompt, n_tokens)
        assert rc == 0, kxlib.kx_last_error()
        total = prompt_len + n_tokens - 1
        lat = [km.latent(layer, b, total) for layer in range(cfg.n_layers) for b in range(batch)]
        got.append((out, km.hidden(batch), km.logits(batch).view(np.uint32), lat))
        km.close()
    assert kxlib.kx_model_set_fusion(None, 1) != 0
    km = KxModel(kxlib, cfg)
    assert kxlib.kx_model_set_fusion(km.h, 64) != 0 and b"mask" in kxlib.kx_last_error()
    km.close()
    o0, h0, l0, c0 = got[1]   # every launch on its own
    for (o1, h1, l1, c1) in got[:1] + got[2:]:
        assert all((a == b).all() for a, b in zip(c1, c0)), "latent cache differs"
        assert (h1 == h0).all() and (l1 == l0).all() and (o1 == o0).all()


def test_resident_launches_at_and_past_their_span_limit(kxlib, ox):
    # The back launch of the attention block holds up to 32 span partials per thread.  With the bit-reproducible
    # attention kernel kept at every length, positions 1985 .. 2048 are 32 spans -- the last the launch takes -- and from
    # 2049 on there are 33 and the model goes back to the W_UV GEMV that merges while it loads.  A generation that
    # crosses that line must equal, to the bit, the same generation with every step a launch of its own.
    say("kimi shape 2-layer stack across 2048 positions: resident launches against separate ones")
    cfg = default_config()
    plen, n_tokens = 2030, 40
    cfg.n_layers, cfg.first_dense, cfg.max_batch, cfg.max_context, cfg.seed = 2, 1, 1, plen + n_tokens, 13
    prompt = O.tokens_u32(plen, cfg.seed, 4, cfg.vocab).reshape(1, plen)
    got = []
    for mask in (63, 3):
        km = KxModel(kxlib, cfg)
        check(kxlib.kx_model_set_fusion(km.h, mask))
        check(kxlib.kx_model_set_attention_kernel(km.h, 1))     # KX_MLA_VALU at every length
        rc, out, _ = km.generate(prompt, n_tokens)
        assert rc == 0, kxlib.kx_last_error()
        total = plen + n_tokens - 1
        got.append((out.copy(), km.hidden(1), km.logits(1).view(np.uint32), km.latent(1, 0, total)))
        km.close()
    for a, b in zip(*got):
        assert (a == b).all(), "the resident launches and the separate ones differ"


@pytest.mark.parametrize("tokens", [1, 3, 9, 32, 70])
def test_q_absorb_operator(kxlib, ox, tokens):
    # bf(W_UK^T q_nope): eight fp32 chains over d = j, j+8, ... summed ((0+1)+(2+3))+((4+5)+(6+7)) (bf16 products are
    # exact in fp32, so numpy's add of the product is the fma).  From 8 tokens on a workgroup takes four tokens: every
    # row, rope part included, must equal the row the one-token launch gives, to the bit.
    say(f"q_absorb tokens={tokens}")
    cfg = default_config()
    Hd, nope, rope, vh, R = cfg.heads, cfg.qk_nope, cfg.qk_rope, cfg.v_head, cfg.kv_rank
    q = O.normal_bf16(tokens * Hd * (nope + rope), 9, 1, 1.0).reshape(tokens, Hd, nope + rope)
    kvb = O.normal_bf16(Hd * (nope + vh) * R, 9, 2, 0.05).reshape(Hd, nope + vh, R)
    tab = np.empty((1, rope), dtype=np.uint16)
    check(kxlib.kx_rope_table(C.byref(cfg), 77, 1, ptr(tab)))
    dq, dk, dr = dev(q), dev(kvb), dev(tab)
    do = DevBuf(tokens * Hd * (R + rope) * 4)
    check(kxlib.kx_q_absorb(C.byref(cfg), dq.ptr, dk.ptr, dr.ptr, do.ptr, tokens, None))
    check(kxlib.kx_sync(None))
    got = do.to_numpy(np.float32, (tokens, Hd, R + rope))
    d1 = DevBuf(Hd * (R + rope) * 4)
    for t in range(tokens):
        check(kxlib.kx_q_absorb(C.byref(cfg), dq.ptr + t * Hd * (nope + rope) * 2, dk.ptr, dr.ptr, d1.ptr, 1, None))
        check(kxlib.kx_sync(None))
        one = d1.to_numpy(np.float32, (Hd, R + rope))
        assert (one.view(np.uint32) == got[t].view(np.uint32)).all(), f"token {t} differs from the one-token launch"
    qf, wf = O.bf16_to_f32(q), O.bf16_to_f32(kvb)
    acc = np.zeros((8, tokens, Hd, R), dtype=np.float32)
    for d in range(nope):
        acc[d % 8] = acc[d % 8] + wf[None, :, d, :] * qf[:, :, d, None]
    tot = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]))
    exp = O.bf16_to_f32(O.f32_to_bf16(tot))
    assert (exp.view(np.uint32) == got[:, :, :R].view(np.uint32)).all()


@pytest.mark.parametrize("batch,seq", [(1, 1), (1, 100), (2, 700), (1, 1100), (1, 1500), (1, 2000), (1, 5000)])
def test_mla_decode_operator(kxlib, ox, batch, seq):
    # BASELINE config 3 shapes (64 heads, latent 512+64) at lengths the scalar oracle finishes quickly; 1100, 2 x 700,
    # 1500 and 2000 positions take workgroups of six, six, seven and eight waves (one head each) instead of four
    say(f"mla decode batch={batch} seq={seq}")
    cfg = default_config()
    H, KVA, R = cfg.heads, 576, 512
    cache = O.normal_bf16(batch * seq * KVA, 3, 1, 1.0).reshape(batch, seq, KVA)
    qabs = O.bf16_to_f32(O.normal_bf16(batch * H * KVA, 3, 2, 0.5)).reshape(batch, H, KVA)
    nbytes = C.c_size_t()
    check(kxlib.kx_mla_workspace_bytes(C.byref(cfg), batch, seq, C.byref(nbytes)))
    dc, dq, dw, do = dev(cache), dev(qabs), DevBuf(nbytes.value), DevBuf(batch * H * R * 2)
    # kernel 1: the VALU kernel, whose summation order the oracle's mode 1 restates
    check(kxlib.kx_mla_decode(C.byref(cfg), dc.ptr, seq * KVA, dq.ptr, dw.ptr, do.ptr, batch, seq, 1, None))
    check(kxlib.kx_sync(None))
    got = do.to_numpy(np.uint16, (batch, H, R))
    exp1, exp0 = np.empty_like(got), np.empty_like(got)
    ox.ox_mla_decode(C.byref(cfg), ptr(cache), seq * KVA, ptr(qabs), ptr(exp1), batch, seq, 1)
    ox.ox_mla_decode(C.byref(cfg), ptr(cache), seq * KVA, ptr(qabs), ptr(exp0), batch, seq, 0)
    assert (got == exp1).all(), f"{np.count_nonzero(got != exp1)} of {got.size} differ from the kx schedule"
    assert O.max_rel(O.bf16_to_f32(got), O.bf16_to_f32(exp0)) < 1e-2
    if seq == 1:
        assert (got == cache[:, 0:1, :R]).all()   # one position: the latent itself


@pytest.mark.parametrize("batch,seq", [(1, 1), (1, 31), (1, 100), (2, 700), (1, 4133), (1, 5000), (8, 4200)])
def test_mla_decode_matrix_core_kernel(kxlib, ox, batch, seq):
    # the MFMA variant sums in another order: max-rel 1e-2 against both oracle schedules, and against the VALU kernel.
    # From 4097 positions on, one to eight sequences are cut into more than 64 spans (both merge kernels, in groups)
    say(f"mla decode (matrix cores) batch={batch} seq={seq}")
    cfg = default_config()
    H, KVA, R = cfg.heads, 576, 512
    cache = O.normal_bf16(batch * seq * KVA, 5, 1, 1.0).reshape(batch, seq, KVA)
    qabs = O.bf16_to_f32(O.normal_bf16(batch * H * KVA, 5, 2, 0.5)).reshape(batch, H, KVA)
    nbytes = C.c_size_t()
    check(kxlib.kx_mla_workspace_bytes(C.byref(cfg), batch, seq, C.byref(nbytes)))
    dc, dq, dw, do = dev(cache), dev(qabs), DevBuf(nbytes.value), DevBuf(batch * H * R * 2)
    outs = {}
    for mode in (2, 1):
        check(kxlib.kx_mla_decode(C.byref(cfg), dc.ptr, seq * KVA, dq.ptr, dw.ptr, do.ptr, batch, seq, mode, None))
        check(kxlib.kx_sync(None))
        outs[mode] = O.bf16_to_f32(do.to_numpy(np.uint16, (batch, H, R)))
    exp1, exp0 = np.empty((batch, H, R), dtype=np.uint16), np.empty((batch, H, R), dtype=np.uint16)
    ox.ox_mla_decode(C.byref(cfg), ptr(cache), seq * KVA, ptr(qabs), ptr(exp1), batch, seq, 1)
    ox.ox_mla_decode(C.byref(cfg), ptr(cache), seq * KVA, ptr(qabs), ptr(exp0), batch, seq, 0)
    e_valu = O.max_rel(outs[2], outs[1])
    e1, e0 = O.max_rel(outs[2], O.bf16_to_f32(exp1)), O.max_rel(outs[2], O.bf16_to_f32(exp0))
    print(f"matrix-core MLA seq={seq}: max-rel {e_valu:.2e} vs VALU kernel, {e1:.2e} vs mode 1, {e0:.2e} vs mode 0", flush=True)
    assert e_valu < 1e-2 and e1 < 1e-2 and e0 < 1e-2


@pytest.mark.parametrize("batch,seq", [(1, 4096), (1, 32768), (1, 131072), (16, 4096), (16, 32768), (16, 131072)])
def test_mla_decode_baseline_sizes(kxlib, ox, batch, seq):
    # BASELINE config 3 at its own sizes.  The cache is generated on the device, sequence b from tensor id b, so the
    # host can regenerate single sequences.  The scalar oracle runs on a sample -- the first and the last sequence,
    # eight of the 64 heads (heads do not interact: a config with heads = 8 on that slice of q) -- in both schedules;
    # the matrix-core kernel (the one these sizes take) is held to 1e-2 on it, normalised maximum and element-wise,
    # and the VALU kernel to the kx schedule's bits.  On the full output: finite, every element inside the range of
    # its cache column (a softmax-weighted mean cannot leave it), and matrix-core against VALU kernel within 1e-2.
    # The element-wise figure is held to 2e-2: a score is rounded to bf16 twice (:429), so another summation order
    # flips the rounding of a few scores by one bf16 step, 2^-8 |s|, which moves that position's probability by
    # percents; over half a million outputs the largest such move reaches 1.2e-2 of an output's own size.
    say(f"mla decode at BASELINE size batch={batch} seq={seq}")
    cfg = default_config()
    H, KVA, R = cfg.heads, 576, 512
    dc = DevBuf(batch * seq * KVA * 2)
    for b in range(batch):
        check(kxlib.kx_fill_normal_bf16(dc.ptr + b * seq * KVA * 2, seq * KVA, 77, b, 1.0, 0, None))
    qabs = O.bf16_to_f32(O.normal_bf16(batch * H * KVA, 77, 1000, 0.5)).reshape(batch, H, KVA)
    nbytes = C.c_size_t()
    check(kxlib.kx_mla_workspace_bytes(C.byref(cfg), batch, seq, C.byref(nbytes)))
    dq, dw, do = dev(qabs), DevBuf(nbytes.value), DevBuf(batch * H * R * 2)
    outs = {}
    for kernel in (2, 1, 0):
        check(kxlib.kx_dev_memset(do.ptr, 0xFF, batch * H * R * 2, None))
        check(kxlib.kx_mla_decode(C.byref(cfg), dc.ptr, seq * KVA, dq.ptr, dw.ptr, do.ptr, batch, seq, kernel, None))
        check(kxlib.kx_sync(None))
        outs[kernel] = do.to_numpy(np.uint16, (batch, H, R))
    assert (outs[0] == outs[2]).all()          # these sizes take the matrix-core kernel by default
    f2, f1 = O.bf16_to_f32(outs[2]), O.bf16_to_f32(outs[1])
    assert np.isfinite(f2).all() and np.isfinite(f1).all()
    e_k, e_k_el = O.max_rel(f2, f1), O.elem_err(f2, f1)
    cfg8 = default_config()
    cfg8.heads = 8
    for b in sorted({0, batch - 1}):
        cache = O.normal_bf16(seq * KVA, 77, b, 1.0).reshape(1, seq, KVA)
        cf = O.bf16_to_f32(cache[0, :, :R])
        lo, hi = cf.min(axis=0), cf.max(axis=0)
        for f in (f2, f1):
            assert (f[b] >= lo - 1e-6).all() and (f[b] <= hi + 1e-6).all(), "an output lies outside the range of its cache column"
        for h0 in (0, 40):
            q8 = np.ascontiguousarray(qabs[b:b + 1, h0:h0 + 8])
            exp1, exp0 = np.empty((1, 8, R), dtype=np.uint16), np.empty((1, 8, R), dtype=np.uint16)
            ox.ox_mla_decode(C.byref(cfg8), ptr(cache), seq * KVA, ptr(q8), ptr(exp1), 1, seq, 1)
            ox.ox_mla_decode(C.byref(cfg8), ptr(cache), seq * KVA, ptr(q8), ptr(exp0), 1, seq, 0)
            assert (outs[1][b, h0:h0 + 8] == exp1[0]).all(), f"VALU kernel differs from the kx schedule (sequence {b}, heads {h0}..)"
            g = f2[b, h0:h0 + 8]
            e1 = (O.max_rel(g, O.bf16_to_f32(exp1[0])), O.elem_err(g, O.bf16_to_f32(exp1[0])))
            e0 = (O.max_rel(g, O.bf16_to_f32(exp0[0])), O.elem_err(g, O.bf16_to_f32(exp0[0])))
            print(f"sequence {b} heads {h0}-{h0 + 7}: matrix-core kernel vs kx schedule max-rel {e1[0]:.2e} elem {e1[1]:.2e}, "
                  f"vs reference schedule max-rel {e0[0]:.2e} elem {e0[1]:.2e}", flush=True)
            assert max(e1[0], e0[0]) < 1e-2 and max(e1[1], e0[1]) < 2e-2
    print(f"matrix-core vs VALU kernel, all {batch} x 64 heads: max-rel {e_k:.2e}, element-wise {e_k_el:.2e}", flush=True)
    assert e_k < 1e-2 and e_k_el < 2e-2


def test_config5_full_stack_batch_invariance_and_prefix(kxlib, ox):
    # BASELINE config 5 at full size: 24 layers (231 GB resident), 1024-token uniform-random prompts, 256 greedy tokens.
    # The scalar oracle cannot walk 24 layers x 1280 positions (the oracle comparisons run on the truncated stacks
    # above); what holds at any size is checked here: three different sequences decoded together come out, each of
    # them, exactly as that sequence decoded alone -- ids, final hidden state and logits to the bit -- (the batch-1
    # run is the driver-timed benchmark path), a rerun reproduces itself, ids stay inside the vocabulary and a shorter
    # generation is a prefix of the longer one.
    say("config 5: 24 layers, prompt 1024, 256 tokens, batch 3 against batch 1")
    cfg = default_config()
    plen, n_tokens = 1024, 256
    cfg.max_batch, cfg.max_context, cfg.seed = 3, plen + n_tokens, 0
    assert cfg.n_layers == 24 and cfg.first_dense == 1 and cfg.vocab == 163840
    prompt = O.tokens_u32(3 * plen, cfg.seed, 4, cfg.vocab).reshape(3, plen)
    km = KxModel(kxlib, cfg)
    rc, out3, counts = km.generate(prompt, n_tokens)
    assert rc == 0, kxlib.kx_last_error()
    assert (counts == n_tokens).all() and (out3 < cfg.vocab).all()
    h3, l3 = km.hidden(3), km.logits(3).view(np.uint32)
    print(f"batch 3 decoded; first ids {out3[:, :6].tolist()}", flush=True)
    for b in (1, 2):
        rc, out1, _ = km.generate(prompt[b:b + 1], n_tokens)
        assert rc == 0, kxlib.kx_last_error()
        same = int(np.argmax(np.append(out1[0] != out3[b], True)))
        assert (out1[0] == out3[b]).all(), f"sequence {b}: ids differ from position {same} on"
        assert (km.hidden(1)[0] == h3[b]).all() and (km.logits(1).view(np.uint32)[0] == l3[b]).all()
    rc, short, _ = km.generate(prompt[2:3], 40)
    assert rc == 0 and (short[0] == out3[2, :40]).all()
    km.close()


def test_kimi_shape_long_context_stack_attention_paths(kxlib, ox):
    # batch 1 past 4096 positions: the matrix-core attention kernel cuts the sequence into more than 64 spans, which
    # the stack merges with a kernel of its own instead of inside the W_UV GEMV.  Held against the same stack with the
    # VALU kernel forced (the bit-exact path): logits of the first sampled step within the stack-level 3e-2, same id.
    say("kimi shape 2-layer stack, 4200-token prompt, attention paths")
    cfg = default_config()
    cfg.n_layers, cfg.first_dense, cfg.max_batch, cfg.max_context, cfg.seed = 2, 1, 1, 4300, 3
    prompt = O.tokens_u32(4200, cfg.seed, 4, cfg.vocab).reshape(1, 4200)
    got = {}
    for mode in (0, 1):
        km = KxModel(kxlib, cfg)
        check(kxlib.kx_model_set_attention_kernel(km.h, mode))
        rc, out, _ = km.generate(prompt, 1)
        assert rc == 0, kxlib.kx_last_error()
        got[mode] = (out.copy(), km.logits(1))
        km.close()
    err = O.max_rel(got[0][1], got[1][1])
    print(f"long-context stack, matrix-core vs VALU attention: logits max-rel {err:.3e}", flush=True)
    assert err < 3e-2 and (got[0][0] == got[1][0]).all()


def test_kimi_shape_batched_stack_attention_paths(kxlib, ox):
    # five sequences and more take the matrix-core attention kernel from 128 cached positions on (their projections run
    # on the matrix cores as well).  Held against the same stack with the VALU attention kernel forced, sequence by
    # sequence: logits of the first sampled step within the stack-level 3e-2 and the same first id, unless the
    # sequence sits on a router or argmax near-tie, which is then named.
    say("kimi shape 2-layer stack, batch 8, 160-token prompts, attention paths")
    cfg = default_config()
    batch, plen = 8, 160
    cfg.n_layers, cfg.first_dense, cfg.max_batch, cfg.max_context, cfg.seed = 2, 1, batch, 192, 5
    prompt = O.tokens_u32(batch * plen, cfg.seed, 4, cfg.vocab).reshape(batch, plen)
    got = {}
    for mode in (0, 1):
        km = KxModel(kxlib, cfg)
        check(kxlib.kx_model_set_attention_kernel(km.h, mode))
        check(kxlib.kx_model_set_routing_record(km.h, 1))
        rc, out, _ = km.generate(prompt, 1)
        assert rc == 0, kxlib.kx_last_error()
        got[mode] = (out.copy(), km.logits(batch), routing_of(kxlib, km.h, cfg, batch))
        km.close()
    errs = [O.max_rel(got[0][1][b], got[1][1][b]) for b in range(batch)]
    excused = judge_sequences([f"sequence {b}" for b in range(batch)], errs, 3e-2, got[0][2], got[1][2], got[0][0][:, 0],
                              got[1][0][:, 0], got[1][1])
    print(f"batch-8 stack, matrix-core vs VALU attention: worst logits max-rel {max(errs):.3e}; excused: {excused or 'none'}", flush=True)
    assert_excused(excused, EXCUSED_ATTENTION_PATHS, "Kimi-shape stack, batch 8, attention paths")


@pytest.mark.parametrize("shape,batch,prompt_len,chunk", [
    ("small", 1, 21, 8), ("small", 3, 23, 32), ("small", 1, 3, 2), ("small", 1, 70, 12), ("kimi", 1, 150, 32),
    ("kimi", 4, 40, 8), ("kimi", 1, 150, 24), ("kimi", 1, 2100, 32), ("small", 2, 100, 40), ("kimi", 1, 300, 256),
    ("kimi", 3, 130, 64), ("kimi-dense", 3, 130, 64), ("kimi", 1, 2100, 2048), ("small", 2, 300, 1024)])
def test_chunked_prefill_against_token_by_token(kxlib, ox, shape, batch, prompt_len, chunk):
    # several prompt positions per prefill step: the step runs as a batch of positions x sequences tokens (matrix-core
    # projections from 5 tokens on, so another summation order).  Held against the token-by-token prefill of the same
    # model (the reference's loop, the path the token-identity checks pin to the oracle).  Both runs keep the router
    # logits of every position (routing record level 2), so every verdict is per row and per sequence:
    #  * a cache row of the last layer (it comes out of a whole layer, and one bf16 step of the largest entry is 7.8e-3
    #    already) within 2e-2, unless that position's expert set differs in a MoE layer before it and the
    #    token-by-token run's selection there was a near-tie (the token then took another expert; counted and named);
    #  * per sequence, the logits of the first sampled step within the stack-level 3e-2 and the same first id, unless
    #    the last position sits on such a router near-tie or on an argmax near-tie (judge_sequences checks and names it).
    # Chunks that leave at most 4 tokens a step take the same GEMV kernels as the token-by-token path and must match
    # it to the bit.  (small, 70, 12) and (kimi, 150, 24) have a step that straddles a 64-position tile, so that the
    # early positions of the step leave the last span empty (VALU and matrix-core attention kernel); (kimi, 2100)
    # crosses 2048 positions.  Steps of more than 32 tokens take the prefill GEMM kernel for the projections and the
    # grouped GEMMs of kx_moe_prefill_layer for the experts: (small, 2 x 40), (kimi, 256) and (kimi, 3 x 64).
    from kxt import NEAR_TIE
    say(f"chunked prefill shape={shape} batch={batch} prompt={prompt_len} chunk={chunk}")
    if shape == "small":
        cfg = O.small_config(batch=batch, context=prompt_len + 8)
    else:
        cfg = default_config()
        cfg.n_layers, cfg.first_dense, cfg.max_batch, cfg.max_context, cfg.seed = 2, 1, batch, prompt_len + 8, 7
        if shape == "kimi-dense":  # two dense layers: no router at all
            cfg.first_dense = 2
    prompt = O.tokens_u32(batch * prompt_len, cfg.seed, 4, cfg.vocab).reshape(batch, prompt_len)
    moe_layers = list(range(cfg.first_dense, cfg.n_layers))
    got = {}
    for c in (1, chunk):
        km = KxModel(kxlib, cfg)
        check(kxlib.kx_model_set_prefill_chunk(km.h, c))
        if moe_layers:
            check(kxlib.kx_model_set_routing_record(km.h, 2))
        rc, out, _ = km.generate(prompt, 4)
        assert rc == 0, kxlib.kx_last_error()
        rc, out1, _ = km.generate(prompt, 1)
        assert rc == 0, kxlib.kx_last_error()
        rows = np.stack([km.latent(cfg.n_layers - 1, b, prompt_len) for b in range(batch)])
        sets, gaps = {}, {}
        for l in moe_layers:       # expert sets and selection gaps of every (position, sequence)
            lg = np.empty((prompt_len, batch, cfg.experts), dtype=np.float32)
            check(kxlib.kx_model_routing_history(km.h, l, 0, prompt_len, ptr(lg)))
            bias = O.normal_f32(cfg.experts, cfg.seed, (l + 1) * 64 + 13, 0.01)
            sel = 1.0 / (1.0 + np.exp(-lg.astype(np.float64))) + bias
            order = np.argsort(-sel, axis=2, kind="stable")
            srt = np.take_along_axis(sel, order[:, :, :cfg.topk + 1], axis=2)
            sets[l], gaps[l] = np.sort(order[:, :, :cfg.topk], axis=2), srt[:, :, cfg.topk - 1] - srt[:, :, cfg.topk]
        got[c] = (out.copy(), km.logits(batch), rows, sets, gaps)
        km.close()
    (ids1, log1, rows1, sets1, gaps1), (idsc, logc, rowsc, setsc, _) = got[1], got[chunk]
    tokens_per_step = min(chunk, 2048 // batch) * batch
    if tokens_per_step <= 4:
        assert (rows1 == rowsc).all() and (log1.view(np.uint32) == logc.view(np.uint32)).all() and (ids1 == idsc).all()
        return
    # cache rows of the last layer, every (sequence, position)
    fc, f1 = O.bf16_to_f32(rowsc), O.bf16_to_f32(rows1)
    row_err = np.abs(fc.astype(np.float64) - f1).max(axis=2) / np.abs(f1).max()
    before = [l for l in moe_layers if l < cfg.n_layers - 1]     # MoE layers whose output reaches the last layer's rows
    flipped_rows, worst_same = [], 0.0
    for b in range(batch):
        for p in range(prompt_len):
            first = next((l for l in before if (sets1[l][p, b] != setsc[l][p, b]).any()), None)
            if first is None:
                worst_same = max(worst_same, float(row_err[b, p]))
                assert row_err[b, p] < 2e-2, f"sequence {b}, position {p}: same experts, cache row max-rel {row_err[b, p]:.3e}"
            else:
                gap = float(gaps1[first][p, b])
                assert gap < NEAR_TIE, f"sequence {b}, position {p}: experts differ in layer {first}, selection gap {gap:.2e}"
                flipped_rows.append(f"sequence {b} position {p}: router near-tie in layer {first} (gap {gap:.1e}), row err {row_err[b, p]:.1e}")
    # the first sampled step, per sequence
    last = prompt_len - 1
    routes_c = {l: ([tuple(setsc[l][last, b]) for b in range(batch)], None) for l in moe_layers}
    routes_1 = {l: ([tuple(sets1[l][last, b]) for b in range(batch)], gaps1[l][last]) for l in moe_layers}
    e_log = [O.max_rel(logc[b], log1[b]) for b in range(batch)]
    excused = judge_sequences([f"sequence {b}" for b in range(batch)], e_log, 3e-2, routes_c, routes_1, idsc[:, 0], ids1[:, 0], log1)
    print(f"chunked prefill: {batch * prompt_len} cache rows, worst max-rel among rows with the same experts "
          f"{worst_same:.1e}; "
          f"rows excused: {flipped_rows or 'none'}; logits max-rel per sequence {np.array2string(np.array(e_log), precision=3)}; "
          f"sequences excused: {excused or 'none'}", flush=True)


def test_prefill_chunk_errors(kxlib):
    cfg = O.small_config(batch=1, context=16)
    km = KxModel(kxlib, cfg)
    assert kxlib.kx_model_set_prefill_chunk(km.h, 0) != 0
    assert kxlib.kx_model_set_prefill_chunk(km.h, 2049) != 0
    assert kxlib.kx_model_set_prefill_chunk(None, 4) != 0
    assert kxlib.kx_model_set_prefill_chunk(km.h, 2048) == 0
    km.close()


@pytest.mark.parametrize("batch", [16, 32])
def test_kimi_shape_batched_stack_against_single_sequences(kxlib, ox, batch):
    # BASELINE config 5's batch 32 (and 16) at Kimi shapes, 2 layers: projections, shared expert, attention (from 128
    # positions) and the routed experts with several pairs run on the matrix cores.  Sequences do not interact, so each
    # must come out as it does alone at batch 1 -- the bit-exact path that the tests above hold to the oracle -- within
    # the stack-level tolerance: last-layer cache rows within 2e-2, logits of the first sampled step within 3e-2 and
    # the same first id.  Every sequence is checked; one that sits on a router near-tie of the batch-1 run (another
    # expert is then legitimately picked) or an argmax near-tie is excused by name.
    say(f"kimi shape 2-layer stack, batch {batch} against the same sequences alone")
    cfg = default_config()
    plen = 140
    cfg.n_layers, cfg.first_dense, cfg.max_batch, cfg.max_context, cfg.seed = 2, 1, batch, plen + 4, 11
    prompt = O.tokens_u32(batch * plen, cfg.seed, 4, cfg.vocab).reshape(batch, plen)
    km = KxModel(kxlib, cfg)
    check(kxlib.kx_model_set_routing_record(km.h, 1))
    rc, out, _ = km.generate(prompt, 1)
    assert rc == 0, kxlib.kx_last_error()
    logits, routes = km.logits(batch), routing_of(kxlib, km.h, cfg, batch)
    rows = [O.bf16_to_f32(km.latent(1, b, plen)) for b in range(batch)]
    ref_routes = {l: ([], []) for l in routes}
    ref_logits, ref_ids, errs = [], [], []
    for b in range(batch):
        rc, o1, _ = km.generate(prompt[b:b + 1], 1)      # the same model, one sequence: GEMV kernels, VALU attention
        assert rc == 0, kxlib.kx_last_error()
        for l, (sets, gaps) in routing_of(kxlib, km.h, cfg, 1).items():
            ref_routes[l][0].extend(sets)
            ref_routes[l][1].extend(gaps.tolist())
        ref_logits.append(km.logits(1)[0])
        ref_ids.append(int(o1[0, 0]))
        errs.append(O.max_rel(logits[b], ref_logits[-1]))
        e_rows = O.max_rel(rows[b], O.bf16_to_f32(km.latent(1, 0, plen)))
        assert e_rows < 2e-2, f"sequence {b}: cache rows max-rel {e_rows:.3e}"
    km.close()
    excused = judge_sequences([f"sequence {b}" for b in range(batch)], errs, 3e-2, routes, ref_routes, out[:, 0], ref_ids,
                              np.stack(ref_logits))
    print(f"batch {batch}: logits max-rel per sequence: median {np.median(errs):.2e}, worst {max(errs):.2e}; excused: {excused or 'none'}", flush=True)
    assert_excused(excused, EXCUSED_AGAINST_SINGLE[batch], f"Kimi-shape stack, batch {batch} against the sequences alone")


def test_config5_batch32_full_size_step_by_step_against_the_exact_path(kxlib, ox, capsys):
    # BASELINE config 5 at batch 32 and full size: 24 layers, 32 uniform-random prompts of 1024 tokens, 256 greedy
    # tokens.  At this batch the projections, the shared expert, the attention and the routed experts with several
    # tokens run on the matrix cores: another summation order, a tolerance path.  The reference is the same model with
    # kx_model_set_exact: the GEMV kernels and the VALU attention kernel at batch 32, whose sums do not depend on the
    # batch.  The exact path prefills the prompts and decodes greedily; every one of the 256 decode steps is run
    # three times from the same cache and the same input ids -- twice on the default path, then, after
    # kx_model_rewind(1), on the exact path, which also leaves the exact cache row behind -- so what is compared is
    # one step's own deviation.  Checked:
    #  1. the exact path's sequences 0..3 equal, to the bit, the same sequences decoded four at a time (the path the
    #     tests above hold to the oracle, at 24 layers too): ids, logits, router logits of the first three tokens;
    #  2. the two default runs of every step agree to the bit (ids, logits, the router logits of all 23 MoE layers of
    #     all 32 sequences): two streams per MoE layer and arrival counters leave no room for a run-to-run difference
    #     unless something races;
    #  3. for every (sequence, step): the router logits of the first MoE layer -- what the dense layer and two
    #     attention blocks on the matrix cores hand to the first router -- within max-rel 1e-2 of the exact path's;
    #  4. for every (sequence, step), one of three verdicts, each checked:
    #     "agrees": the same expert set in all 23 MoE layers, logits within the stack-level 3e-2, the same sampled id;
    #     "argmax near-tie": as before, but another id, and the exact path's two largest logits closer than the bar;
    #     "router flip": the expert sets differ first in layer j, and the exact path's selection gap there is below
    #        2.5e-2, i.e. what a router-logit change of a few percent can cross.  A token that took another expert is
    #        off by tens of percent in the next layer, so such a pair is not judged further in this step.
    # Why the bars of a 24-layer stack are wider than the operator bars (1e-2 given identical inputs, held in the
    # operator tests): with INT4 values in [-8, 7] times group scales |N(0, 0.02)| a routed expert has a gain of
    # several hundred, every MoE layer's output swamps the residual stream it is added to, and a deviation of 4e-3 in
    # layer 1 is 1e-2 to 6e-2 a few layers later for some sequences before it decays again -- with any one of the
    # matrix-core parts switched on alone, the others exact.  The counts of the three verdicts and the worst figures are
    # printed.
    import time
    batch, plen, n_tokens = 32, 1024, 256
    say(f"config 5 at full size: 24 layers, batch {batch}, prompt {plen}, {n_tokens} tokens, default path against exact path step by step")
    cfg = default_config()
    cfg.max_batch, cfg.max_context, cfg.seed = batch, plen + n_tokens, 0
    assert cfg.n_layers == 24 and cfg.first_dense == 1 and cfg.vocab == 163840
    prompt = O.tokens_u32(batch * plen, cfg.seed, 4, cfg.vocab).reshape(batch, plen)
    moe_layers = list(range(cfg.first_dense, cfg.n_layers))
    bias = np.stack([O.normal_f32(cfg.experts, cfg.seed, (l + 1) * 64 + 13, 0.01).astype(np.float64) for l in moe_layers])
    t0 = time.time()

    def note(msg):
        with capsys.disabled():
            print(f"  [{time.time() - t0:4.0f} s] {msg}", flush=True)

    km = KxModel(kxlib, cfg)
    check(kxlib.kx_model_set_routing_record(km.h, 1))

    def observe(nb):
        """sampled ids, logits (as bits), router logits [nb, layers, experts] of the last step"""
        ids = np.zeros(nb, dtype=np.uint32)
        check(kxlib.kx_greedy_sample(km.h, ptr(ids)))
        rl = np.empty((nb, len(moe_layers), cfg.experts), dtype=np.float32)
        lg = np.empty((nb, cfg.experts), dtype=np.float32)
        for j, l in enumerate(moe_layers):
            check(kxlib.kx_model_routing(km.h, l, ptr(lg), None))
            rl[:, j] = lg
        return ids, km.logits(nb), rl

    def same_bits(a, b):
        return all((x.view(np.uint32) == y.view(np.uint32)).all() for x, y in zip(a, b))

    # four sequences at a time, default path (GEMV kernels at this batch): prompt + 3 tokens
    four = []
    check(kxlib.kx_prefill(km.h, ptr(np.ascontiguousarray(prompt[:4])), 4, plen))
    for i in range(3):
        if i:
            check(kxlib.kx_decode_step(km.h, None))
        four.append(observe(4))
    note("sequences 0..3 decoded four at a time")
    # exact path at batch 32: prefill, then step back onto the last prompt position
    check(kxlib.kx_model_set_exact(km.h, 15))
    check(kxlib.kx_prefill(km.h, ptr(prompt), batch, plen))
    check(kxlib.kx_sync(None))
    note("exact path: 32 prompts prefilled")
    check(kxlib.kx_model_rewind(km.h, 1))
    feed = np.ascontiguousarray(prompt[:, plen - 1])
    verdicts = {"agrees": 0, "argmax near-tie": 0, "router flip": 0}
    worst = {"first router": 0.0, "logits": 0.0, "flipped gap": 0.0}
    for i in range(n_tokens):
        runs = []
        for mask in (0, 0, 15):
            if runs:
                check(kxlib.kx_model_rewind(km.h, 1))
            check(kxlib.kx_model_set_exact(km.h, mask))
            check(kxlib.kx_decode_step(km.h, ptr(feed)))
            runs.append(observe(batch))
        assert same_bits(runs[0], runs[1]), f"token {i}: two runs of the default path differ"
        (ids_f, log_f, rl_f), (ids_e, log_e, rl_e) = runs[0], runs[2]
        if i < 3:
            assert same_bits([x[:4] for x in runs[2]], four[i]), f"token {i}: the exact path at batch 32 differs from four at a time"
        first_router = np.abs(rl_f[:, 0] - rl_e[:, 0]).max(axis=1) / np.abs(rl_e[:, 0]).max(axis=1)
        worst["first router"] = max(worst["first router"], float(first_router.max()))
        assert first_router.max() < 1e-2, f"token {i}, sequence {int(first_router.argmax())}: router logits of the first MoE layer differ by max-rel {first_router.max():.3e}"
        sel_f = 1.0 / (1.0 + np.exp(-rl_f.astype(np.float64))) + bias[None]
        sel_e = 1.0 / (1.0 + np.exp(-rl_e.astype(np.float64))) + bias[None]
        order_e = np.argsort(-sel_e, axis=2, kind="stable")
        set_e = np.sort(order_e[:, :, :cfg.topk], axis=2)
        set_f = np.sort(np.argsort(-sel_f, axis=2, kind="stable")[:, :, :cfg.topk], axis=2)
        srt_e = np.take_along_axis(sel_e, order_e[:, :, :cfg.topk + 1], axis=2)
        gap_e = srt_e[:, :, cfg.topk - 1] - srt_e[:, :, cfg.topk]
        errs = np.abs(log_f - log_e).max(axis=1) / np.abs(log_e).max(axis=1)
        for b in range(batch):
            differs = np.nonzero((set_f[b] != set_e[b]).any(axis=1))[0]
            if len(differs):
                j = int(differs[0])
                assert gap_e[b, j] < 2.5e-2, (f"sequence {b}, token {i}: experts differ in layer {moe_layers[j]} although the exact path's "
                                              f"selection gap there is {gap_e[b, j]:.2e}")
                worst["flipped gap"] = max(worst["flipped gap"], float(gap_e[b, j]))
                verdicts["router flip"] += 1
                continue
            worst["logits"] = max(worst["logits"], float(errs[b]))
            assert errs[b] < 3e-2, f"sequence {b}, token {i}: the same experts in every layer, logits err {errs[b]:.3e}"
            if ids_f[b] != ids_e[b]:
                top = np.sort(log_e[b])[-2:]
                gap = float(top[1] - top[0]) / float(np.abs(log_e[b]).max())
                assert gap < 3e-2, f"sequence {b}, token {i}: id {ids_f[b]} vs {ids_e[b]} although the top-2 logit gap is {gap:.2e}"
                verdicts["argmax near-tie"] += 1
                continue
            verdicts["agrees"] += 1
        feed = ids_e.copy()
        if i % 32 == 31:
            note(f"{i + 1} steps: verdicts {verdicts}; worst {({k: float(f'{v:.2e}') for k, v in worst.items()})}")
    km.close()
    note(f"{batch * n_tokens} (sequence, step) pairs: {verdicts}; worst first-router max-rel {worst['first router']:.2e}, worst logits max-rel among "
         f"pairs with the same experts everywhere {worst['logits']:.2e}, largest selection gap "
         f"flipped {worst['flipped gap']:.2e}; default path deterministic over {n_tokens} steps")
    assert sum(verdicts.values()) == batch * n_tokens


def test_a_wait_given_up_inside_a_resident_launch_is_reported(kxlib, ox):
    # The workgroups of the resident launches wait for each other's values with a bounded number of polls; one that
    # gives up sets a flag, the launch ends normally, and the model reports the flag at its next synchronisation.
    # Forced from the host: with the flag set beforehand, every workgroup whose first poll fails gives up at once, so
    # all launches drain (nothing hangs) and generate must come back with an error that names the way out.
    say("resident launches: a wait given up is reported, the launches still end")
    cfg = default_config()
    cfg.n_layers, cfg.first_dense, cfg.max_batch, cfg.max_context, cfg.seed = 2, 1, 1, 32, 11
    prompt = O.tokens_u32(5, cfg.seed, 4, cfg.vocab).reshape(1, 5)
    km = KxModel(kxlib, cfg)
    check(kxlib.kx_model_debug_fail_waits(km.h))
    rc, _, _ = km.generate(prompt, 3)
    assert rc != 0 and b"kx_model_set_fusion" in kxlib.kx_last_error(), kxlib.kx_last_error()
    rc, _, _ = km.generate(prompt, 3)   # the flag stays: so does the error
    assert rc != 0
    km.close()
    assert kxlib.kx_model_debug_fail_waits(None) != 0
    # the process is fine: a new model, with and without the resident launches, decodes the same ids
    outs = []
    for mask in (63, 3):
        km = KxModel(kxlib, cfg)
        check(kxlib.kx_model_set_fusion(km.h, mask))
        rc, out, _ = km.generate(prompt, 3)
        assert rc == 0, kxlib.kx_last_error()
        outs.append(out.copy())
        km.close()
    assert (outs[0] == outs[1]).all()


def test_model_form_of_the_handover_gives_the_same_bits(kxlib, ox):
    # blok_amd/libkx_strict.so is the library with the hand-over between workgroups of one launch (the q_b GEMV that
    # finishes a head's query, the router GEMV whose last workgroup routes, the routed down launch that combines)
    # compiled in its memory-model form: release increment, acquire by the finisher.  The library that ships orders
    # the same accesses by what the gfx950 instructions do, which is faster.  Both run here, on the paths that
    # use the protocol (up to 4 sequences), and must agree to the bit on ids, hidden state, logits and cache rows.
    import os
    from blok_amd.lib import load_library
    say("hand-over protocol: shipped form against the memory-model form")
    strict = load_library(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "blok_amd", "libkx_strict.so"))
    # (name, config, sequences, prompt, tokens, fusion masks): the small stack at 3 sequences; Kimi shapes at one
    # sequence with the launches that use the protocol (mask 3: the q_b GEMV finishes the query, the routed down
    # launch finishes the layer; mask 1: the layer's tail as launches of its own), with the resident launches of the
    # attention block (31: their hand-over is another one; the routed down launch finishes the layer) and with the
    # default (63: the routed experts' resident launch finishes it); Kimi shapes at 3 sequences (the router
    # and shared gate/up pair launch whose last router workgroup routes, the q_b GEMV at several tokens)
    cases = [("small", O.small_config(batch=3, context=64), 3, 11, 9, (63,))]
    kimi = default_config()
    kimi.n_layers, kimi.first_dense, kimi.max_batch, kimi.max_context, kimi.seed = 3, 1, 1, 48, 11
    cases.append(("kimi", kimi, 1, 24, 8, (3, 1, 31, 63)))
    kimi3 = default_config()
    kimi3.n_layers, kimi3.first_dense, kimi3.max_batch, kimi3.max_context, kimi3.seed = 2, 1, 3, 24, 12
    cases.append(("kimi, 3 sequences", kimi3, 3, 9, 4, (63,)))
    for name, cfg, batch, prompt_len, n_tokens, masks in cases:
        prompt = O.tokens_u32(batch * prompt_len, cfg.seed, 4, cfg.vocab).reshape(batch, prompt_len)
        for mask in masks:
            got = []
            for lib in (kxlib, strict):
                km = KxModel(lib, cfg)
                assert lib.kx_model_set_fusion(km.h, mask) == 0
                rc, out, _ = km.generate(prompt, n_tokens)
                assert rc == 0, lib.kx_last_error()
                total = prompt_len + n_tokens - 1
                h = np.empty((batch, cfg.hidden), dtype=np.uint16)
                lg = np.empty((batch, cfg.vocab), dtype=np.float32)
                assert lib.kx_model_hidden(km.h, ptr(h)) == 0 and lib.kx_model_logits(km.h, ptr(lg)) == 0
                rows = np.empty((batch, total, cfg.kv_rank + cfg.qk_rope), dtype=np.uint16)
                for b in range(batch):
                    assert lib.kx_model_latent(km.h, cfg.n_layers - 1, b, 0, total, ptr(rows[b])) == 0
                got.append((out.copy(), h, lg.view(np.uint32), rows))
                km.close()
            for a, b in zip(*got):
                assert (a == b).all(), f"{name}, fusion mask {mask}: the two forms differ"


def test_executor_json_line(kxlib):
    import json
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "blok_amd", "kx-kimi-exec")
    r = subprocess.run([exe, "--prompt-tokens", "11,12,13", "--tokens", "3", "--layers", "2", "--seed", "7",
                        "--ignore-eos"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    doc = json.loads(r.stdout)                       # blok/runtime.py:88-94
    assert doc["status"] == "ok" and len(doc["token_ids"]) == 3
    assert all(isinstance(t, int) and 0 <= t < 163840 for t in doc["token_ids"])
    assert r.stdout.startswith('{"status":"ok","token_ids":[') and r.stdout.endswith("]}\n")
