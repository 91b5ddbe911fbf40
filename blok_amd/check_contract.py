"""Checks a metadata directory against what the executor will ask of it.

Reference: scripts/check_kimi_contract.py -- every tensor of the 61-layer Kimi-K2 forward pass present in
runtime-index.blok with the right role, slot, dtype, shape and byte count (:47-74), tokenizer.blok present with its
header, and the chat-templated prompts "hello" and "1234567890" encoding to the ids the real tokenizer gives (:31-33).
The tensor contract is the C++ one the loader itself applies (kx_index_check, include/kx.h).

usage: python -m blok_amd.check_contract <runtime-index-or-directory>
"""
import ctypes as C
import sys
from pathlib import Path

from .lib import default_config, kx
from .runtime import encode_prompt

GOLDEN = (
    ("hello", [163587, 2482, 163601, 22931, 163586, 163588, 69702, 163601, 163606, 163607]),
    ("1234567890", [163587, 2482, 163601, 6694, 12972, 16242, 15, 163586, 163588, 69702, 163601, 163606, 163607]),
)


def check(arg, layers=61):
    """Raises SystemExit with the reference's messages; returns (tensors, weight bytes) when everything holds."""
    path = Path(arg)
    if path.is_dir():
        path = path / "runtime-index.blok"
    if path.name != "runtime-index.blok" or not path.is_file():
        raise SystemExit(f"missing runtime-index.blok: {path}")
    cfg = default_config()
    cfg.n_layers = layers
    n, nbytes = C.c_uint64(), C.c_uint64()
    if kx().kx_index_check(C.byref(cfg), str(path).encode(), C.byref(n), C.byref(nbytes)) != 0:
        raise SystemExit(kx().kx_last_error().decode("utf-8", "replace"))
    tokenizer = path.parent / "tokenizer.blok"
    if not tokenizer.is_file() or tokenizer.open().readline().strip() != "blok-tokenizer-v2":
        raise SystemExit("missing or bad tokenizer.blok")
    for prompt, expected in GOLDEN:
        if encode_prompt(tokenizer, prompt) != expected:
            raise SystemExit(f"tokenizer mismatch for {prompt!r}")
    return n.value, nbytes.value


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if len(argv) != 1:
        raise SystemExit("usage: python -m blok_amd.check_contract <runtime-index-or-directory>")
    check(argv[0])
    print("ok: Kimi runtime and tokenizer contract")


if __name__ == "__main__":
    main()
