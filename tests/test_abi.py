"""CPU-side checks of the drop-in boundary: the C-ABI library loads without a GPU and exports every
entry point include/kx.h declares; the executor keeps the reference's argv / JSON / exit-code contract
(reference: src/kimi_exec.cu:532-557, :895-904; scripts/test_host.py:43-54 pins the same boundary)."""
import ctypes as C
import json
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "kx.h")
EXEC = os.path.join(ROOT, "blok_amd", "kx-kimi-exec")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from blok_amd.lib import kx, _SIGS
    lib = kx()
    names = declared_functions()
    assert len(names) > 40
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/kx.h but not exported by libkx.so"
    missing = [n for n in names if n not in _SIGS and n != "kx_last_error"]
    assert not missing, f"no ctypes signature for {missing}"


def _print_config(*argv):
    r = subprocess.run([EXEC, "--prompt-tokens", "1,2,3", "--tokens", "5", "--print-config", *argv], capture_output=True, text=True, timeout=60)
    return r.returncode, (json.loads(r.stdout) if r.returncode == 0 else None), r.stderr


def test_executor_config_for_a_checkpoint_is_the_reference_constants(tmp_path):
    # src/kimi_exec.cu:176-186: with --index the executor must compute with the reference's constants, YARN_FACTOR 64
    # (:184) among them; the seeded random-init run (the synthetic benchmark configurations) keeps factor 32.
    # A checkpoint that does not fit one GPU is not truncated silently.
    import test_index as TI
    rc, doc, err = _print_config()
    assert rc == 0 and doc["yarn_factor"] == 32.0 and doc["n_layers"] == 24 and doc["layers_in_checkpoint"] == 0
    lines, _ = TI._kimi_index_lines()
    index = tmp_path / "runtime-index.blok"
    index.write_text("\n".join(lines) + "\n")
    rc, doc, err = _print_config("--index", str(index))
    assert rc == 1 and "61 layers" in err and "--layers" in err
    rc, doc, err = _print_config("--index", str(index), "--layers", "24")
    assert rc == 0, err
    assert (doc["hidden"], doc["vocab"], doc["q_rank"], doc["kv_rank"], doc["heads"]) == (7168, 163840, 1536, 512, 64)   # :176-178
    assert (doc["qk_nope"], doc["qk_rope"], doc["v_head"]) == (128, 64, 128)                                             # :178
    assert (doc["experts"], doc["topk"], doc["moe_inter"], doc["dense_inter"]) == (384, 8, 2048, 18432)                  # :179
    assert doc["first_dense"] == 1 and doc["n_layers"] == 24 and doc["layers_in_checkpoint"] == 61
    assert abs(doc["rms_eps"] - 1e-5) < 1e-12 and doc["rope_theta"] == 50000.0 and abs(doc["routed_scale"] - 2.827) < 1e-6   # :181-183
    assert (doc["yarn_factor"], doc["yarn_beta_fast"], doc["yarn_beta_slow"], doc["yarn_orig_ctx"]) == (64.0, 32.0, 1.0, 4096.0)  # :184-185
    assert doc["eos_id"] == 163586                                                                                       # :186
    rc, doc, err = _print_config("--index", str(index), "--layers", "24", "--yarn-factor", "32")
    assert rc == 0 and doc["yarn_factor"] == 32.0
    rc, doc, err = _print_config("--prefill-chunk", "4096")
    assert rc == 1 and "prefill chunk" in err


def test_config_default_is_kimi_k2():
    from blok_amd.lib import default_config
    c = default_config()
    # src/kimi_exec.cu:176-186 (yarn_factor follows BASELINE config 3, not the reference's 64)
    assert (c.hidden, c.heads, c.qk_nope, c.qk_rope, c.v_head) == (7168, 64, 128, 64, 128)
    assert (c.q_rank, c.kv_rank, c.experts, c.topk) == (1536, 512, 384, 8)
    assert (c.dense_inter, c.moe_inter, c.shared_inter, c.vocab) == (18432, 2048, 2048, 163840)
    assert c.eos_id == 163586 and c.first_dense == 1 and c.n_layers == 24
    assert abs(c.routed_scale - 2.827) < 1e-6 and c.yarn_factor == 32.0 and c.rope_theta == 50000.0


def test_errors_are_reported_not_fatal():
    from blok_amd.lib import kx, default_config
    lib = kx()
    assert lib.kx_config_default(None) != 0
    assert b"null" in lib.kx_last_error()
    cfg = default_config()
    w, k, s = C.c_uint64(), C.c_uint64(), C.c_uint64()
    assert lib.kx_model_bytes(C.byref(cfg), C.byref(w), C.byref(k), C.byref(s)) == 0
    assert 231.0e9 < w.value < 231.6e9          # the resident footprint of BASELINE config 5
    cfg.hidden = 1000
    assert lib.kx_model_bytes(C.byref(cfg), C.byref(w), C.byref(k), C.byref(s)) != 0
    assert b"hidden" in lib.kx_last_error()


def _run(*args):
    return subprocess.run([EXEC, *args], capture_output=True, text=True, timeout=60)


@pytest.mark.skipif(not os.path.exists(EXEC), reason="executor not built")
def test_executor_argument_errors_exit_1_with_a_message():
    for args, msg in [((), "bad args"), (("--prompt-tokens", "1,2"), "bad args"),
                      (("--bogus", "1"), "unknown flag: --bogus"), (("--tokens",), "usage:"),
                      (("--prompt-tokens", "1,x", "--tokens", "2"), "bad prompt token"),
                      (("--prompt-tokens", "1,163840", "--tokens", "2"), "prompt token outside vocabulary"),
                      (("--prompt-tokens", "1", "--tokens", "262144"), "requested sequence exceeds Kimi context")]:
        r = _run(*args)
        assert r.returncode == 1 and msg in r.stderr and r.stdout == "", (args, r)
