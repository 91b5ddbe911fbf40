"""runtime-index.blok: the index writer (blok_amd/model_index.py) and the C++ reader / forward contract
(kx_index_check, kx_index_infer_config) on CPU.

What pins them: the one index fixture the reference's own test holds (scripts/test_host.py:28-39: the row
("language_model.model.norm.weight", "resident", "bf16", "1", shard, 8, 2) gives a 14-field line, key
(-1, "resident", "norm", -1), aligned extent (0, 4096)); the keys validate_forward_contract()
(src/kimi_exec.cu:746-777) and scripts/check_kimi_contract.py:50-73 look up, which the writer must produce
from the Hugging Face tensor names; and the error messages of runtime_index() (:561-583).
"""
import ctypes as C

import numpy as np

import pytest

import ckpt
import oracle as O
from blok_amd import model_index as MI
from blok_amd.lib import KxConfig, kx


def _check(cfg, index):
    n, b = C.c_uint64(), C.c_uint64()
    rc = kx().kx_index_check(C.byref(cfg), str(index).encode(), C.byref(n), C.byref(b))
    return rc, n.value, b.value, kx().kx_last_error().decode()


def test_reference_fixture_row_gives_the_reference_line():
    row = ("language_model.model.norm.weight", "resident", "bf16", "1", "/tmp/model-00001-of-00064.safetensors", 8, 2)
    lines = MI.index_lines([row])
    assert lines[0] == "blok-runtime-index-v1"
    f = lines[1].split()
    assert len(f) == 14                                            # scripts/test_host.py:34
    assert f[0] == "tensor" and f[1] == row[0] and f[2] == "resident"
    assert (int(f[3]), int(f[4]), f[5]) == (-1, -1, "norm")        # key (-1, "resident", "norm", -1), :39
    assert (f[6], f[7]) == ("bf16", "1")
    assert (int(f[8]), int(f[9]), int(f[10])) == (0, 4096, 4096)   # read_required_ranges == [(0, 4096)], :40
    assert (int(f[11]), int(f[12]), f[13]) == (8, 2, row[4])


@pytest.mark.parametrize("name,key", [
    # (layer, role, slot, expert) as check_kimi_contract.py:50-73 / kimi_exec.cu:746-777 look them up
    ("language_model.model.embed_tokens.weight", (-1, "resident", "embed_tokens", -1)),
    ("language_model.lm_head.weight", (-1, "resident", "lm_head", -1)),
    ("language_model.model.layers.3.input_layernorm.weight", (3, "resident", "input_layernorm", -1)),
    ("language_model.model.layers.3.post_attention_layernorm.weight", (3, "resident", "post_attention_layernorm", -1)),
    ("language_model.model.layers.60.self_attn.kv_a_proj_with_mqa.weight", (60, "attention_resident", "kv_a_proj_with_mqa", -1)),
    ("language_model.model.layers.2.self_attn.q_a_layernorm.weight", (2, "attention_resident", "q_a_layernorm", -1)),
    ("language_model.model.layers.0.mlp.gate_proj.weight", (0, "dense_ffn_rowcol", "gate_proj", -1)),
    ("language_model.model.layers.0.mlp.down_proj.weight", (0, "dense_ffn_rowcol", "down_proj", -1)),
    ("language_model.model.layers.5.mlp.gate.weight", (5, "router", "gate", -1)),
    ("language_model.model.layers.5.mlp.gate.e_score_correction_bias", (5, "router", "e_score_correction_bias", -1)),
    ("language_model.model.layers.5.mlp.shared_experts.up_proj.weight", (5, "shared_expert_resident", "up_proj", -1)),
    ("language_model.model.layers.5.mlp.experts.383.down_proj.weight_packed", (5, "routed_expert", "down_proj.weight_packed", 383)),
    ("language_model.model.layers.5.mlp.experts.0.gate_proj.weight_scale", (5, "routed_expert", "gate_proj.weight_scale", 0)),
])
def test_writer_keys_are_the_contract_keys(name, key):
    layer, expert, slot = MI.runtime_slot(name)
    assert (layer, MI.role(name), slot, expert) == key


def _small(tmp_path, **kw):
    cfg = O.small_config(**kw)
    keyed = ckpt.write_checkpoint(tmp_path / "hf", cfg, seed=77)
    report = MI.materialize(tmp_path / "hf", tmp_path / "meta")
    return cfg, keyed, report


def test_writer_and_reader_agree_on_a_small_checkpoint(tmp_path):
    cfg, keyed, report = _small(tmp_path)
    assert report["tensors"] == len(keyed)             # decoys (other tower, weight_shape, f32) are not indexed
    rc, n, nbytes, err = _check(cfg, report["index"])
    assert rc == 0, err
    assert n == len(keyed)
    assert nbytes == sum(a.nbytes // (2 if k[1] == ckpt.TL_ROUTER_BIAS and k[0] >= 0 else 1) for k, a in keyed)
    # a truncated stack reads a prefix of the layers from the same index
    cfg.n_layers = 2
    rc, n2, _, err = _check(cfg, report["index"])
    assert rc == 0 and n2 < n, err
    # data of the shards starts at unaligned offsets: extents must still be whole 4096-byte blocks
    for line in open(report["index"]).read().splitlines()[1:]:
        f = line.split()
        off, ext, data, size = int(f[8]), int(f[9]), int(f[11]), int(f[12])
        assert off % 4096 == 0 and ext % 4096 == 0 and off <= data and data + size <= off + ext and data - off < 4096


def test_infer_config_recovers_the_shapes(tmp_path):
    cfg, _, report = _small(tmp_path)
    got = KxConfig()
    kx().kx_config_default(C.byref(got))
    got.topk = cfg.topk
    assert kx().kx_index_infer_config(report["index"].encode(), C.byref(got)) == 0, kx().kx_last_error()
    for f in ("vocab", "hidden", "n_layers", "first_dense", "q_rank", "kv_rank", "heads", "dense_inter", "experts",
              "shared_inter", "moe_inter", "topk", "qk_nope", "qk_rope", "v_head"):
        assert getattr(got, f) == getattr(cfg, f), f
    rc, _, _, err = _check(got, report["index"])
    assert rc == 0, err
    # the numeric constants after the call are the reference's for a checkpoint (src/kimi_exec.cu:181-186): a caller
    # of the C ABI that loads one computes RoPE and the softmax scale with YARN_FACTOR 64, not the 32 of the
    # library's random-init default
    assert got.yarn_factor == 64.0 and (got.yarn_beta_fast, got.yarn_beta_slow, got.yarn_orig_ctx) == (32.0, 1.0, 4096.0)
    assert got.rope_theta == 50000.0 and abs(got.rms_eps - 1e-5) < 1e-12 and abs(got.routed_scale - 2.827) < 1e-6
    assert got.eos_id == 163586 and got.yarn_mscale_all_dim == 1.0
    rs, ms = C.c_float(), C.c_float()
    assert kx().kx_softmax_scale(C.byref(got), C.byref(rs), C.byref(ms)) == 0
    assert abs(ms.value - (0.1 * np.log(64.0) + 1.0)) < 1e-6                   # :428


def _rewrite(index, fn):
    lines = open(index).read().splitlines()
    lines = fn(lines)
    open(index, "w").write("\n".join(lines) + "\n")


def _sub(lines, pick, fn):
    i = next(i for i, l in enumerate(lines) if pick in l)
    f = lines[i].split()
    fn(f)
    lines[i] = " ".join(f)
    return lines


@pytest.mark.parametrize("edit,msg", [
    (lambda ls: ["blok-runtime-index-v0"] + ls[1:], "bad runtime index header"),                       # :565
    (lambda ls: ls[:3] + ["tensors x"] + ls[3:], "bad runtime index line"),                             # :567
    (lambda ls: ls[:2] + [" ".join(ls[2].split()[:13])] + ls[3:], "incomplete runtime tensor line"),    # :572
    (lambda ls: ls[:2] + [ls[2] + " tail"] + ls[3:], "runtime tensor path cannot contain whitespace"),  # :574
    (lambda ls: ls + [ls[5]], "duplicate runtime tensor key"),                                          # :580
    (lambda ls: ls[:1], "runtime index has no file-backed tensors"),                                    # :583
    (lambda ls: [l for l in ls if ".layers.1.self_attn.o_proj." not in l], "missing runtime tensor: 1:-1:attention_resident:o_proj"),  # :590
    (lambda ls: _sub(ls, ".layers.0.self_attn.q_b_proj.", lambda f: f.__setitem__(7, "1x2")), "bad bf16 tensor contract"),          # :598
    (lambda ls: _sub(ls, ".layers.1.mlp.experts.3.up_proj.weight_packed", lambda f: f.__setitem__(6, "bf16")), "bad routed expert packed shape"),
    (lambda ls: _sub(ls, ".layers.2.mlp.experts.0.down_proj.weight_scale", lambda f: f.__setitem__(12, "10")), "bad routed expert scale shape"),
    (lambda ls: _sub(ls, ".layers.1.mlp.gate.e_score_correction_bias", lambda f: f.__setitem__(7, "17")), "bad router correction bias"),  # :764
    (lambda ls: _sub(ls, "model.norm.weight", lambda f: f.__setitem__(10, "512")), "runtime index has invalid tensor extent"),   # :742
    (lambda ls: _sub(ls, "model.norm.weight", lambda f: f.__setitem__(8, str(int(f[8]) + 4096))), "runtime index has invalid tensor extent"),
    (lambda ls: _sub(ls, ".layers.1.mlp.experts.3.up_proj.weight_scale", lambda f: f.__setitem__(4, "16")), "out-of-range Kimi coordinates"),  # :740
    (lambda ls: _sub(ls, "lm_head", lambda f: f.__setitem__(3, "x")), "bad layer"),                     # :575
])
def test_reader_rejects_what_the_reference_rejects(tmp_path, edit, msg):
    cfg, _, report = _small(tmp_path)
    _rewrite(report["index"], edit)
    rc, _, _, err = _check(cfg, report["index"])
    assert rc != 0 and msg in err, err


def test_missing_index_names_the_file(tmp_path):
    rc, _, _, err = _check(O.small_config(), tmp_path / "runtime-index.blok")
    assert rc != 0 and "missing runtime-index.blok" in err   # :561


def _kimi_index_lines(layers=61):
    """Index lines of the full Kimi-K2 checkpoint layout (no files behind them): the shapes of
    scripts/check_kimi_contract.py:50-73, data packed back to back into one imaginary shard."""
    H, D, I, E, V = 7168, 18432, 2048, 384, 163840
    rows, at = [], [8]

    def add(name, dtype, *shape):
        n = 1
        for d in shape:
            n *= d
        size = n * (2 if dtype == "bf16" else 4)
        rows.append((name, MI.role(name), dtype, "x".join(map(str, shape)), "/ckpt/model-00001-of-000064.safetensors", at[0], size))
        at[0] += size

    lm = "language_model."
    add(lm + "model.embed_tokens.weight", "bf16", V, H)
    add(lm + "model.norm.weight", "bf16", H)
    add(lm + "lm_head.weight", "bf16", V, H)
    for l in range(layers):
        p = f"{lm}model.layers.{l}."
        add(p + "input_layernorm.weight", "bf16", H)
        add(p + "post_attention_layernorm.weight", "bf16", H)
        for n, shp in (("q_a_proj", (1536, H)), ("q_a_layernorm", (1536,)), ("q_b_proj", (64 * 192, 1536)), ("kv_a_proj_with_mqa", (576, H)),
                       ("kv_a_layernorm", (512,)), ("kv_b_proj", (64 * 256, 512)), ("o_proj", (H, 64 * 128))):
            add(p + "self_attn." + n + ".weight", "bf16", *shp)
        if l == 0:
            add(p + "mlp.gate_proj.weight", "bf16", D, H)
            add(p + "mlp.up_proj.weight", "bf16", D, H)
            add(p + "mlp.down_proj.weight", "bf16", H, D)
            continue
        add(p + "mlp.gate.weight", "bf16", E, H)
        add(p + "mlp.gate.e_score_correction_bias", "bf16", E)
        for n, shp in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            add(p + f"mlp.shared_experts.{n}.weight", "bf16", *shp)
            for e in range(E):
                add(p + f"mlp.experts.{e}.{n}.weight_packed", "i32", shp[0], shp[1] // 8)
                add(p + f"mlp.experts.{e}.{n}.weight_scale", "bf16", shp[0], shp[1] // 32)
    return MI.index_lines(rows), at[0] - 8


def test_full_kimi_k2_contract_and_checker(tmp_path):
    # all 61 layers x 384 experts at the real shapes, through the writer's naming rules and the C++ contract
    from blok_amd import check_contract as CC
    from blok_amd.lib import default_config
    lines, data_bytes = _kimi_index_lines()
    index = tmp_path / "runtime-index.blok"
    index.write_text("\n".join(lines) + "\n")
    cfg = default_config()
    cfg.n_layers = 61
    rc, n, nbytes, err = _check(cfg, index)
    assert rc == 0, err
    assert n == len(lines) - 1 == 3 + 61 * 9 + 3 + 60 * (2 + 3 + 384 * 6)
    assert nbytes == data_bytes
    cfg.n_layers = 24            # the truncation that fits one GPU reads a prefix
    rc, n24, b24, err = _check(cfg, index)
    assert rc == 0 and n24 == 3 + 24 * 9 + 3 + 23 * (2 + 3 + 384 * 6), err
    assert abs(b24 - 231.29e9) < 0.3e9   # the resident weights of the 24-layer stack
    # the checker: index ok, tokenizer missing, then present with the real ids of the words involved
    with pytest.raises(SystemExit, match="missing or bad tokenizer.blok"):
        CC.check(tmp_path)
    import test_tokenizer as TT
    ranks = {bytes([b]): i for i, b in enumerate(TT.byte_order())}
    ranks.update({b"user": 2482, b"hello": 22931, b"assistant": 69702, b"123": 6694, b"456": 12972, b"789": 16242})
    special = {"<|im_end|>": 163586, "<|im_user|>": 163587, "<|im_assistant|>": 163588, "<|im_middle|>": 163601, "<think>": 163606, "</think>": 163607}
    TT.write_blok(tmp_path / "tokenizer.blok", ranks, special)
    assert CC.check(tmp_path) == (n, nbytes)
    ranks[b"hello"] = 22930
    TT.write_blok(tmp_path / "tokenizer.blok", ranks, special)
    with pytest.raises(SystemExit, match="tokenizer mismatch for 'hello'"):
        CC.check(tmp_path)
    with pytest.raises(SystemExit, match="missing runtime-index.blok"):
        CC.check(tmp_path / "nowhere")
