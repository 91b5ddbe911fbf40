"""Host side of the executor: prompt -> token ids -> kx-kimi-exec -> text.

Reference: blok/runtime.py.  The public names and their behaviour are the reference's -- generate() :51-95,
runtime_index() :98-118, tokenizer_encoding() :121-134, encode_prompt() :137-140, answer() :143-149,
BlokRuntimeError :7-8, KIMI_TEXT :11-36 -- with two differences: the byte-pair encoder is libkx's
(kx_tokenizer_*, include/kx.h) instead of tiktoken, and the executor needs no uGDS device, map or KV scratch
range (BLOK_UGDS_*, BLOK_KV_UGDS_*), because weights and cache live in HBM.
"""
import ctypes as C
import json
import os
import subprocess
from pathlib import Path

from .lib import KxError, kx


class BlokRuntimeError(RuntimeError):
    pass


# the text decoder this executor is built for (config.json `text_config` of the checkpoint, runtime.py:11-36)
KIMI_TEXT = dict(
    model_type="kimi_k2", num_hidden_layers=61, hidden_size=7168, intermediate_size=18432, first_k_dense_replace=1,
    num_attention_heads=64, q_lora_rank=1536, kv_lora_rank=512, qk_nope_head_dim=128, qk_rope_head_dim=64, v_head_dim=128,
    n_routed_experts=384, num_experts_per_tok=8, n_shared_experts=1, n_group=1, topk_group=1, moe_intermediate_size=2048,
    routed_scaling_factor=2.827, scoring_func="sigmoid", norm_topk_prob=True, rms_norm_eps=1e-5, rope_theta=50000.0,
    max_position_embeddings=262144, vocab_size=163840,
)
CHAT_HEAD = "<|im_user|>user<|im_middle|>"
CHAT_TAIL = "<|im_end|><|im_assistant|>assistant<|im_middle|><think></think>"


class Encoding:
    """What the reference gets from tiktoken.Encoding: encode (special tokens allowed) and decode."""

    def __init__(self, path):
        self._lib = kx()
        self._h = C.c_void_p()
        if self._lib.kx_tokenizer_open(str(path).encode(), C.byref(self._h)) != 0:
            raise BlokRuntimeError(self._lib.kx_last_error().decode("utf-8", "replace"))

    def _ids(self, call, data):
        n = C.c_size_t()
        cap = 2 * len(data) + 32  # a token covers at least one byte; the template adds ten ids
        buf = (C.c_uint32 * cap)()
        if call(data, len(data), buf, cap, C.byref(n)) != 0:
            raise BlokRuntimeError(self._lib.kx_last_error().decode("utf-8", "replace"))
        return list(buf[:n.value])

    def encode(self, text, allowed_special="all"):
        special = 1 if allowed_special == "all" else 0
        return self._ids(lambda d, n, b, c, out: self._lib.kx_tokenizer_encode(self._h, d, n, special, b, c, out), text.encode("utf-8"))

    def encode_prompt(self, prompt):
        return self._ids(lambda d, n, b, c, out: self._lib.kx_encode_prompt(self._h, d, n, b, c, out), prompt.encode("utf-8"))

    def decode_bytes(self, ids):
        arr = (C.c_uint32 * len(ids))(*ids)
        n = C.c_size_t()
        self._lib.kx_tokenizer_decode(self._h, arr, len(ids), None, 0, C.byref(n))  # asks for the size
        buf = C.create_string_buffer(max(1, n.value))
        if self._lib.kx_tokenizer_decode(self._h, arr, len(ids), buf, n.value, C.byref(n)) != 0:
            raise BlokRuntimeError(self._lib.kx_last_error().decode("utf-8", "replace"))
        return buf.raw[:n.value]

    def decode(self, ids):
        return self.decode_bytes(ids).decode("utf-8", errors="replace")

    def close(self):
        if self._h:
            self._lib.kx_tokenizer_close(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def tokenizer_encoding(tokenizer):
    try:
        return Encoding(tokenizer)
    except KxError as error:
        raise BlokRuntimeError(str(error)) from error


def encode_prompt(tokenizer, prompt, encoding=None):
    """Token ids of the chat-templated prompt (runtime.py:137-140)."""
    if encoding is None:
        return tokenizer_encoding(tokenizer).encode_prompt(prompt)
    if isinstance(encoding, Encoding):
        return encoding.encode_prompt(prompt)
    return encoding.encode(CHAT_HEAD + prompt + CHAT_TAIL, allowed_special="all")  # any object with tiktoken's interface


PLACEHOLDER_MODELS = ("<kimi k2 model directory", "<kimi k2 model directory>")
INDEX_NAME = "runtime-index.blok"


def _check_kimi_config(directory):
    """A checkpoint directory's config.json, when there is one, must describe Kimi-K2 (KIMI_TEXT)."""
    config = directory / "config.json"
    if not config.is_file():
        return
    fields = json.loads(config.read_text())
    fields = fields.get("text_config", fields)
    wrong = [name for name in KIMI_TEXT if fields.get(name) != KIMI_TEXT[name]]
    if wrong:
        raise BlokRuntimeError("unsupported Kimi config fields: " + ", ".join(wrong))


def default_index():
    """Where the index of the pinned model lives when no model argument names one: BLOK_META_ROOT, else
    $BLOK_HOME/metadata, else ~/.blok/metadata."""
    meta_root = os.getenv("BLOK_META_ROOT")
    if meta_root is None:
        meta_root = Path(os.getenv("BLOK_HOME", Path.home() / ".blok")) / "metadata"
    return Path(meta_root) / "moonshotai/Kimi-K2.6" / INDEX_NAME


def runtime_index(model):
    """Path of runtime-index.blok for a model argument (blok/runtime.py:98-118 resolves it the same way): the index
    file itself, a directory holding it (a checkpoint directory's config.json must then describe Kimi-K2), the
    BLOK_MODEL environment variable when the argument is the command line's placeholder, and last the default
    metadata directory."""
    named = os.getenv("BLOK_MODEL", "") if str(model) in PLACEHOLDER_MODELS else str(model)
    places = []
    if named:
        base = Path(named).expanduser().resolve()
        places = [base, base / INDEX_NAME]
        _check_kimi_config(base)
    places.append(default_index())
    found = next((p for p in places if p.name == INDEX_NAME and p.is_file()), None)
    if found is None:
        raise BlokRuntimeError("runtime-index.blok not found; run python -m blok_amd.model_index <checkpoint-dir> <metadata-dir>")
    return found


def executor_path():
    return Path(os.getenv("BLOK_KIMI_EXEC_BIN", Path(__file__).parent / "kx-kimi-exec"))


def _run_executor(argv, max_time):
    """The executor's token ids: one JSON line on stdout, a non-zero exit code means failure with the reason on
    stderr (src/kimi_exec.cu:495-498, :901-903)."""
    try:
        done = subprocess.run(argv, text=True, capture_output=True, timeout=max_time)
    except subprocess.TimeoutExpired as error:
        raise BlokRuntimeError(f"generation exceeded {max_time:g} seconds") from error
    if done.returncode != 0:
        raise BlokRuntimeError(done.stderr.strip() or done.stdout.strip())
    try:
        report = json.loads(done.stdout)
    except json.JSONDecodeError as error:
        raise BlokRuntimeError(f"executor returned invalid JSON: {done.stdout!r}") from error
    ids = report.get("token_ids") if report.get("status") == "ok" else None
    vocab = KIMI_TEXT["vocab_size"]
    if not isinstance(ids, list) or any(type(i) is not int or not 0 <= i < vocab for i in ids):
        raise BlokRuntimeError(f"executor failed: {report}")
    return ids


def generate(*, model_dir, prompt, max_tokens, max_time):
    """Text generated for `prompt` by the executor (blok/runtime.py:51-95): at most max_tokens ids, max_time seconds.
    The executor computes with the reference's constants for a checkpoint (YaRN factor 64) and refuses a checkpoint
    that does not fit one GPU; BLOK_KIMI_LAYERS=n runs the first n layers of it (a truncation: not the full model's
    output)."""
    if not prompt or max_tokens <= 0 or max_time <= 0:
        raise BlokRuntimeError("prompt must be non-empty and limits must be positive")
    index = runtime_index(model_dir)
    needed = {"index": index, "tokenizer": index.parent / "tokenizer.blok", "executor": executor_path()}
    absent = [str(p) for p in needed.values() if not p.is_file()]
    if absent:
        raise BlokRuntimeError("missing required file(s): " + ", ".join(absent))
    encoding = tokenizer_encoding(needed["tokenizer"])
    ids = encode_prompt(needed["tokenizer"], prompt, encoding)
    argv = [str(needed["executor"]), "--index", str(index), "--prompt-tokens", ",".join(map(str, ids)), "--tokens", str(max_tokens)]
    layers = os.getenv("BLOK_KIMI_LAYERS")
    if layers:
        argv += ["--layers", layers]
    return encoding.decode(_run_executor(argv, max_time))


def answer(text):
    """The reference's normalisation of a reply for its smoke test (runtime.py:143-149): what follows the last
    </think>, the inside of a leading <...>, lower-cased letters, digits and spaces only."""
    _, found, tail = text.rpartition("</think>")
    text = (tail if found else text).strip()
    if text.startswith("<") and ">" in text:
        text = text[1:text.index(">")]
    return "".join(ch for ch in text.lower() if ch.isalnum() or ch.isspace()).strip()
