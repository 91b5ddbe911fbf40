"""AddressSanitizer + UndefinedBehaviorSanitizer over the host-side code (no GPU): the library's checkpoint-index
parser and tokenizer (blok_amd/csrc/kx_index.hip, kx_tok.hip, compiled as plain C++) and the CPU oracle, driven by
tests/sanitize_driver.cpp on valid inputs, on every malformed index the reference's reader rejects
(src/kimi_exec.cu:559-606, :736-778), on malformed tokenizer.blok files (blok/runtime.py:121-134) and on awkward
strings.  The reference's build has no sanitizer target (CMakeLists.txt:14-16: warnings as errors only).
"""
import os
import struct
import subprocess

import pytest

import ckpt
import oracle as O
import test_index as TI
import test_tokenizer as TT
from blok_amd import model_index as MI

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "blok_amd", "csrc")


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("san") / "sanitize_driver")
    cmd = ["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer",
           "-ffp-contract=off", "-mfma", "-fopenmp", "-Wall", "-Wextra", "-Werror", "-Wno-unused-parameter", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
           "-x", "c++", os.path.join(CSRC, "kx_index.hip"), os.path.join(CSRC, "kx_tok.hip"),
           os.path.join(ROOT, "oracle", "kx_oracle.cpp"), os.path.join(ROOT, "tests", "sanitize_driver.cpp"), "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    if r.returncode != 0 and "libasan" in r.stderr:
        pytest.skip("the sanitizer runtimes are not installed for g++ here")
    assert r.returncode == 0, r.stderr[-4000:]
    return exe


def test_host_code_is_clean_under_asan_and_ubsan(driver, tmp_path):
    cfg = O.small_config()
    ckpt.write_checkpoint(tmp_path / "hf", cfg, seed=5)
    report = MI.materialize(tmp_path / "hf", tmp_path / "good")
    good = open(report["index"]).read().splitlines()
    # absolute shard paths, so that the edited copies next to the good index still point at the files
    edits = [p[0] for p in TI.test_reader_rejects_what_the_reference_rejects.pytestmark[0].args[1]]
    edits += [lambda ls: TI._sub(ls, "model.norm.weight", lambda f: f.__setitem__(8, str(2 ** 64 - 4096))),    # extent wraps around
              lambda ls: TI._sub(ls, "model.norm.weight", lambda f: f.__setitem__(11, str(2 ** 64 - 1))),
              lambda ls: [ls[0], "tensor " + "x" * 70000],                                                   # one very long field
              lambda ls: ls[:2] + ["tensor a b 99999999999999999999 0 c bf16 1 0 4096 4096 0 2 /dev/null"]]
    for i, edit in enumerate(edits):
        (tmp_path / f"bad_{i}.blok").write_text("\n".join(edit(list(good))) + "\n")
    ranks = TT.train_vocab(TT.CORPUS, 120)
    TT.write_blok(tmp_path / "tokenizer.blok", ranks, TT.SPECIAL)
    rows = (tmp_path / "tokenizer.blok").read_text().splitlines()
    bad_tok = [["blok-tokenizer-v1"] + rows[1:], rows + [rows[5]], rows[:3] + ["tok 7 zz"] + rows[3:], rows + ["tok 4294967295 41"],
               rows + ["tok 2147483647 4141"], rows + ["special 99 "], rows[:1], rows[:40], rows + ["tok 5000 414"], rows + ["frob 1 41"]]
    for i, r in enumerate(bad_tok):
        (tmp_path / f"tok_bad_{i}.blok").write_text("\n".join(r) + "\n")
    strings = [b"", b" ", b"hello world", "it's 12345 we'll  \n\n x".encode(), "你好 世界 naïve".encode(), b"\xff\xfe\x80abc\xc3", b"\xe4\xbd",
               b"<|im_end|><|im_end", b"a" * 5000, bytes(range(256)) * 3, " 　\t\r\n ".encode() * 7, b"<think></think>" * 50]
    with open(tmp_path / "strings.bin", "wb") as f:
        for s in strings:
            f.write(struct.pack("<I", len(s)) + s)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1", OMP_NUM_THREADS="2")
    r = subprocess.run([driver, str(tmp_path)], capture_output=True, text=True, timeout=600, env=env)
    assert r.returncode == 0 and "0 failure(s)" in r.stdout, r.stdout[-2000:] + r.stderr[-6000:]
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr and "LeakSanitizer" not in r.stderr, r.stderr[-6000:]
