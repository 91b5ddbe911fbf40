"""GPU parity of the checkpoint path: safetensors shards -> runtime-index.blok -> kx_model_load -> tokens.

The oracle gets the same tensors as arrays (ox_model_set_tensor) on top of a model seeded differently, so a
tensor that either side dropped, misplaced or mis-sliced changes the tokens.  Bar: ids, hidden state and
logits bit-exact against the oracle's kx schedule.
"""
import ctypes as C
import json
import os
import subprocess

import numpy as np
import pytest

import ckpt
import oracle as O
from blok_amd import model_index as MI
from kxt import check, say
from oracle import ptr
from test_gpu_model import KxModel

pytestmark = pytest.mark.gpu


class KxLoaded(KxModel):
    def __init__(self, lib, cfg, index):
        self.lib, self.cfg = lib, cfg
        self.h = C.c_void_p()
        check(lib.kx_model_load(C.byref(cfg), str(index).encode(), C.byref(self.h)))

    def load_info(self):
        b, s = C.c_uint64(), C.c_double()
        check(self.lib.kx_model_load_info(self.h, C.byref(b), C.byref(s)))
        return b.value, s.value


def _oracle_with(cfg, keyed, mode=1):
    om = O.OxModel(cfg, mode)
    for (layer, tid, expert), arr in keyed:
        om.set_tensor(layer, tid, expert, arr)
    return om


@pytest.mark.parametrize("batch,prompt_len,n_tokens,direct", [(1, 12, 10, "1"), (2, 7, 6, "0")])
def test_loaded_stack_tokens_identical(kxlib, ox, tmp_path, monkeypatch, batch, prompt_len, n_tokens, direct):
    say(f"checkpoint load batch={batch} prompt={prompt_len} tokens={n_tokens} direct={direct}")
    monkeypatch.setenv("KX_LOAD_DIRECT", direct)
    monkeypatch.setenv("KX_LOAD_THREADS", "3")
    cfg = O.small_config(batch=batch, context=64)
    keyed = ckpt.write_checkpoint(tmp_path / "hf", cfg, seed=4242)
    report = MI.materialize(tmp_path / "hf", tmp_path / "meta")
    cfg.seed = 99  # neither side may fall back to the seeded weights
    km = KxLoaded(kxlib, cfg, report["index"])
    nbytes, secs = km.load_info()
    assert nbytes == sum(a.nbytes // (2 if k[1] == ckpt.TL_ROUTER_BIAS and k[0] >= 0 else 1) for k, a in keyed)
    print(f"loaded {nbytes / 1e6:.1f} MB in {secs * 1e3:.1f} ms", flush=True)
    prompt = O.tokens_u32(batch * prompt_len, 5, 4, cfg.vocab).reshape(batch, prompt_len)
    rc, out, counts = km.generate(prompt, n_tokens)
    assert rc == 0, kxlib.kx_last_error()
    om = _oracle_with(cfg, keyed)
    rc, out1, counts1 = om.generate(prompt, n_tokens)
    assert rc == 0
    assert (km.hidden(batch) == om.hidden(batch)).all()
    assert (km.logits(batch).view(np.uint32) == om.logits(batch).view(np.uint32)).all()
    assert (out == out1).all() and (counts == counts1).all(), f"tokens differ:\n{out}\n{out1}"
    # the loaded weights are not the seeded ones
    ks = KxModel(kxlib, cfg)
    rc, out_seeded, _ = ks.generate(prompt, n_tokens)
    assert rc == 0 and not (out_seeded == out).all()
    for m in (km, ks, om):
        m.close()


def test_truncated_stack_loads_a_layer_prefix(kxlib, ox, tmp_path):
    say("checkpoint load, 2 of 3 layers")
    cfg = O.small_config(batch=1, context=32)
    keyed = ckpt.write_checkpoint(tmp_path / "hf", cfg, seed=31)
    report = MI.materialize(tmp_path / "hf", tmp_path / "meta")
    cfg.n_layers = 2
    km = KxLoaded(kxlib, cfg, report["index"])
    om = _oracle_with(cfg, [(k, a) for k, a in keyed if k[0] < 2])
    prompt = O.tokens_u32(6, 5, 4, cfg.vocab).reshape(1, 6)
    rc, out, _ = km.generate(prompt, 5)
    assert rc == 0, kxlib.kx_last_error()
    rc, out1, _ = om.generate(prompt, 5)
    assert (out == out1).all()
    assert (km.logits(1).view(np.uint32) == om.logits(1).view(np.uint32)).all()
    km.close()
    om.close()


def test_short_shard_is_an_error(kxlib, tmp_path):
    say("checkpoint load from a shard cut short")
    cfg = O.small_config(batch=1, context=16)
    ckpt.write_checkpoint(tmp_path / "hf", cfg, seed=31)
    report = MI.materialize(tmp_path / "hf", tmp_path / "meta")
    shard = sorted((tmp_path / "hf").glob("*.safetensors"))[-1]
    os.truncate(shard, os.path.getsize(shard) // 2)
    h = C.c_void_p()
    rc = kxlib.kx_model_load(C.byref(cfg), report["index"].encode(), C.byref(h))
    assert rc != 0 and "ends inside tensor" in kxlib.kx_last_error().decode(), kxlib.kx_last_error()
    assert not h.value


def test_executor_reads_the_index(kxlib, ox, tmp_path):
    # the reference's process boundary (blok/runtime.py:70-83): --index, --prompt-tokens, --tokens in, one JSON line out
    say("executor with --index")
    cfg = O.small_config(batch=1, context=32)
    keyed = ckpt.write_checkpoint(tmp_path / "hf", cfg, seed=8)
    report = MI.materialize(tmp_path / "hf", tmp_path / "meta")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "blok_amd", "kx-kimi-exec")
    prompt = O.tokens_u32(5, 5, 4, cfg.vocab).reshape(1, 5)
    r = subprocess.run([exe, "--index", report["index"], "--prompt-tokens", ",".join(str(t) for t in prompt[0]), "--tokens", "4",
                        "--topk", str(cfg.topk), "--ignore-eos"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    doc = json.loads(r.stdout)
    cfg.max_context = 9
    cfg.yarn_factor = 64.0      # a checkpoint run uses the reference's YARN_FACTOR (src/kimi_exec.cu:184)
    om = _oracle_with(cfg, keyed)
    rc, out1, _ = om.generate(prompt, 4)
    assert doc["status"] == "ok" and doc["token_ids"] == [int(t) for t in out1[0]]
    om.close()
    r = subprocess.run([exe, "--index", str(tmp_path / "nowhere" / "runtime-index.blok"), "--prompt-tokens", "1", "--tokens", "1"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "missing runtime-index.blok" in r.stderr and r.stdout == ""
