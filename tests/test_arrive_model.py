"""The cross-workgroup hand-over of blok_amd/csrc/kx_arrive.h as a thread model under ThreadSanitizer (no GPU).

The reference has no such protocol (every step is a launch of its own, src/kimi_exec.cu:812-877); the GPU kernels
that use it are held to the oracle by the GPU tests.  Here the protocol's ordering itself is checked against the
C++ memory model: race-free as written, reported when the release/acquire is taken out.
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def _build_and_run(tmp_path, name, extra):
    exe = str(tmp_path / name)
    cmd = ["g++", "-O1", "-g", "-std=c++17", "-fsanitize=thread", *extra, os.path.join(HERE, "arrive_model.cpp"), "-o", exe, "-lpthread"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    if r.returncode != 0 and "sanitize" in r.stderr:
        pytest.skip("ThreadSanitizer is not available to g++ here")
    assert r.returncode == 0, r.stderr
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=0 exitcode=66")
    return subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)


def test_protocol_is_race_free_and_finishes_each_block_once(tmp_path):
    r = _build_and_run(tmp_path, "arrive_ok", [])
    assert r.returncode == 0, r.stdout + r.stderr[-2000:]
    assert "errors=0" in r.stdout and "data race" not in r.stderr


def test_relaxed_ordering_is_reported(tmp_path):
    r = _build_and_run(tmp_path, "arrive_relaxed", ["-DKX_ARRIVE_ORDER=__ATOMIC_RELAXED"])
    assert r.returncode == 66 and "data race" in r.stderr, (r.returncode, r.stderr[-500:])
