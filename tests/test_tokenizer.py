"""tokenizer.blok, the pre-tokenizer, byte-pair merging, the chat template and the Python host (CPU only).

Pins:
* the split: the `regex` module (an independent backtracking engine with its own Unicode tables) running the
  pattern of blok/runtime.py:37-48 on curated and random strings -- the C++ matcher must cut the same pieces;
* byte-pair merging: a plain Python restatement of merge-lowest-rank-first on a vocabulary trained here;
  decode(encode(x)) == x;
* the chat template and special-token handling: the ids the reference expects for "hello" and "1234567890"
  (scripts/check_kimi_contract.py:31-32, scripts/test_host.py:43-46), reproduced with a tokenizer.blok that
  gives the few words involved the ids the real vocabulary gives them.  The real vocabulary is not in the
  container (tiktoken.model ships with the checkpoint): parity with it is unpinned beyond this.
* the host: scripts/test_host.py:48-54 (argv tail, JSON line, answer()).
"""
import ctypes as C
import json
import os
import random
import stat

import pytest

from blok_amd import model_index as MI
from blok_amd import runtime as RT
from blok_amd.lib import kx

regex = pytest.importorskip("regex")

KIMI_PATTERN = "|".join([  # blok/runtime.py:37-48
    r"[\p{Han}]+",
    r"[^\r\n\p{L}\p{N}]?[\p{Lu}\p{Lt}\p{Lm}\p{Lo}\p{M}&&[^\p{Han}]]*[\p{Ll}\p{Lm}\p{Lo}\p{M}&&[^\p{Han}]]+(?i:'s|'t|'re|'ve|'m|'ll|'d)?",
    r"[^\r\n\p{L}\p{N}]?[\p{Lu}\p{Lt}\p{Lm}\p{Lo}\p{M}&&[^\p{Han}]]+[\p{Ll}\p{Lm}\p{Lo}\p{M}&&[^\p{Han}]]*(?i:'s|'t|'re|'ve|'m|'ll|'d)?",
    r"\p{N}{1,3}",
    r" ?[^\s\p{L}\p{N}]+[\r\n]*",
    r"\s*[\r\n]+",
    r"\s+(?!\S)",
    r"\s+",
])
WITNESS = regex.compile(KIMI_PATTERN, regex.V1)


def split(text):
    data = text.encode("utf-8")
    n = C.c_size_t()
    cap = len(data) + 1
    ends = (C.c_uint32 * cap)()
    assert kx().kx_pretokenize(data, len(data), ends, cap, C.byref(n)) == 0, kx().kx_last_error()
    out, at = [], 0
    for e in ends[:n.value]:
        out.append(data[at:e].decode("utf-8"))
        at = e
    assert at == len(data)
    return out


CURATED = [
    "Hello world's  test\n\n  x", "1234567890", "你好世界abc", "あAあ", "あA", "I'LL go, they'Ve DONE it; we'd", "a'ſ b's",
    "x \n y", "tab\t\tz", "ΑΒγ ΑΒ", "naïve café", "  leading", "trailing   ", "a\r\n\r\nb", " \n \n ", "\n", " ", "",
    "foo(bar) -> baz!!\n", "emoji 😀😀 ok", "mixed漢字とかなkana", "ǅemal ǅ", "ʰabc", "é́x", "٣٤٥٦ Ⅷ ²³",
    "a b　c d", "don't DON'T don'T", "'s", "''s", "x's's", "\x00\x1f\x7f", "��", "𝒜𝒷 𝟘𝟙𝟚𝟛",
    "CamelCaseWordsHere", "snake_case_words", "HTTPServer2Go", "...", " ...\n\n", "a" * 50 + " " * 7 + "b", "〇一二", "⺀⺁",
    "<|im_user|>user<|im_middle|>hello<|im_end|>",
]
ALPHABET = (list("abcdefgxyzABCXYZ") * 3 + list("0123456789") + [" "] * 8 + ["\n", "\r", "\t", "\n", " \n"] + list(".,!?()'\"-_") + ["'"] * 4
            + ["'s", "'T", "'re", "'VE", "'m", "'LL", "'d", "'ſ"] + list("你好世界漢字") + list("あいアイ") + list("ΑΒΓαβγ") + list("ДЖдж")
            + ["ǅ", "ʰ", "́", "̀", "٣", "Ⅷ", "²", " ", "　", " ", "\u0085", "😀", "ſ", "\x00", "\x1f", "�", "𝒜", "𝟘", "〇", "⺀", "ß", "İ", "ı"])


def test_split_on_curated_strings():
    for text in CURATED:
        assert split(text) == WITNESS.findall(text), repr(text)


def test_split_on_random_strings():
    rng = random.Random(20240607)
    for _ in range(6000):
        text = "".join(rng.choice(ALPHABET) for _ in range(rng.randint(1, 40)))
        assert split(text) == WITNESS.findall(text), repr(text)


def test_split_agrees_on_every_single_character_class():
    # one representative of every run of the generated tables, alone and between a letter and a space
    import itertools
    reps = [chr(cp) for cp in itertools.chain(range(0, 0x3000, 7), range(0x3000, 0x11000, 97), range(0x11000, 0x110000, 1009)) if not 0xD800 <= cp <= 0xDFFF]
    for ch in reps:
        for text in (ch, "a" + ch + " b", " " + ch + ch + "1"):
            assert split(text) == WITNESS.findall(text), repr(text)


# ---- a small vocabulary ------------------------------------------------------------------------------
def byte_order():
    """The 256 single-byte tokens in the order byte-level vocabularies use: printable ASCII first ('0' is id 15)."""
    first = list(range(33, 127)) + list(range(161, 173)) + list(range(174, 256))
    return first + [b for b in range(256) if b not in first]


def train_vocab(corpus, merges):
    """Plain byte-pair training: repeatedly make the most frequent adjacent pair a token."""
    ranks = {bytes([b]): i for i, b in enumerate(byte_order())}
    words = [[bytes([b]) for b in piece.encode("utf-8")] for text in corpus for piece in WITNESS.findall(text)]
    for _ in range(merges):
        count = {}
        for w in words:
            for a, b in zip(w, w[1:]):
                count[a + b] = count.get(a + b, 0) + 1
        count = {k: v for k, v in count.items() if k not in ranks}
        if not count:
            break
        best = max(sorted(count), key=lambda k: count[k])
        ranks[best] = len(ranks)
        for w in words:
            i = 0
            while i + 1 < len(w):
                if w[i] + w[i + 1] == best:
                    w[i:i + 2] = [best]
                else:
                    i += 1
    return ranks


def py_bpe(ranks, piece):
    """Merge the adjacent pair of lowest rank (leftmost on ties) until none is in the vocabulary."""
    if piece in ranks:
        return [ranks[piece]]
    parts = [bytes([b]) for b in piece]
    while True:
        best, at = None, -1
        for i in range(len(parts) - 1):
            r = ranks.get(parts[i] + parts[i + 1])
            if r is not None and (best is None or r < best):
                best, at = r, i
        if best is None:
            return [ranks[p] for p in parts]
        parts[at:at + 2] = [parts[at] + parts[at + 1]]


def write_blok(path, ranks, special):
    rows = ["blok-tokenizer-v2"] + [f"tok {i} {b.hex()}" for b, i in sorted(ranks.items(), key=lambda kv: kv[1])]
    rows += [f"special {i} {s.encode().hex()}" for s, i in sorted(special.items(), key=lambda kv: kv[1])]
    path.write_text("\n".join(rows) + "\n")


CORPUS = ["the quick brown fox jumps over the lazy dog " * 3, "hello hello user assistant the then there",
          "it's what's don't we'll 123 456 1234", "你好世界 你好 世界", "naïve café déjà vu", "x = f(a, b) + g(c);\n\treturn x;\n"] * 2
SPECIAL = {"<|im_end|>": 1000, "<|im_user|>": 1001, "<|im_assistant|>": 1002, "<|im_middle|>": 1003, "<think>": 1004, "</think>": 1005,
           "[EOS]": 1006, "<|reserved_token_1|>": 1007, "<|reserved_token_10|>": 1008}


@pytest.fixture(scope="module")
def small_tok(tmp_path_factory):
    ranks = train_vocab(CORPUS, 300)
    path = tmp_path_factory.mktemp("tok") / "tokenizer.blok"
    write_blok(path, ranks, SPECIAL)
    return ranks, path, RT.tokenizer_encoding(path)


def test_merges_match_the_plain_restatement(small_tok):
    ranks, _, enc = small_tok
    rng = random.Random(7)
    texts = CORPUS + CURATED + ["".join(rng.choice(ALPHABET + list("thequickhello ")) for _ in range(rng.randint(1, 60))) for _ in range(1500)]
    for text in texts:
        want = [i for piece in WITNESS.findall(text) for i in py_bpe(ranks, piece.encode("utf-8"))]
        assert enc.encode(text, allowed_special=()) == want, repr(text)
        assert enc.decode_bytes(enc.encode(text)) == text.encode("utf-8"), repr(text)


def test_special_tokens_are_ids_only_when_allowed(small_tok):
    ranks, _, enc = small_tok
    text = "a<|im_end|>b<|reserved_token_10|><think>c</think>[EOS]"
    ids = enc.encode(text)
    assert [i for i in ids if i >= 1000] == [1000, 1008, 1004, 1005, 1006]
    assert enc.decode(ids) == text
    plain = enc.encode(text, allowed_special=())
    assert all(i < 1000 for i in plain) and enc.decode(plain) == text
    assert plain == [i for piece in WITNESS.findall(text) for i in py_bpe(ranks, piece.encode())]
    assert enc.encode("") == [] and enc.decode([]) == ""


def test_reference_golden_prompts(tmp_path):
    # the ids the real vocabulary gives these words and special tokens, as the reference's own checks hold them
    # (scripts/check_kimi_contract.py:31-32): the template, the special-token handling and the 1-3 digit split
    # must then give exactly the reference's lists
    ranks = {bytes([b]): i for i, b in enumerate(byte_order())}
    assert ranks[b"0"] == 15
    ranks.update({b"user": 2482, b"hello": 22931, b"assistant": 69702, b"123": 6694, b"456": 12972, b"789": 16242})
    special = {f"<|reserved_token_{i}|>": i for i in range(163584, 163840)}
    special = {k: v for k, v in special.items() if v not in (163586, 163587, 163588, 163601, 163606, 163607)}
    special.update({"<|im_end|>": 163586, "<|im_user|>": 163587, "<|im_assistant|>": 163588, "<|im_middle|>": 163601,
                    "<think>": 163606, "</think>": 163607})
    path = tmp_path / "tokenizer.blok"
    write_blok(path, ranks, special)
    expected = {
        "hello": [163587, 2482, 163601, 22931, 163586, 163588, 69702, 163601, 163606, 163607],
        "1234567890": [163587, 2482, 163601, 6694, 12972, 16242, 15, 163586, 163588, 69702, 163601, 163606, 163607],
    }
    for prompt, ids in expected.items():
        assert RT.encode_prompt(path, prompt) == ids
    enc = RT.tokenizer_encoding(path)
    assert enc.decode(expected["hello"]) == "<|im_user|>user<|im_middle|>hello<|im_end|><|im_assistant|>assistant<|im_middle|><think></think>"
    n_tok, n_sp, max_id = C.c_int32(), C.c_int32(), C.c_int32()
    assert kx().kx_tokenizer_info(enc._h, C.byref(n_tok), C.byref(n_sp), C.byref(max_id)) == 0
    assert (n_tok.value, n_sp.value, max_id.value) == (262, 256, 163839)


@pytest.mark.parametrize("text", ["", "blok-tokenizer-v1\ntok 0 61\n", "blok-tokenizer-v2\ntok 0 6\n", "blok-tokenizer-v2\nword 0 61\n",
                                  "blok-tokenizer-v2\ntok 0 61\ntok 0 62\n", "blok-tokenizer-v2\ntok 0 61\n", "blok-tokenizer-v2\ntok 0 zz\n"])
def test_bad_tokenizer_files(tmp_path, text):
    path = tmp_path / "tokenizer.blok"
    path.write_text(text)
    with pytest.raises(RT.BlokRuntimeError, match="bad tokenizer"):   # blok/runtime.py:128
        RT.tokenizer_encoding(path)
    with pytest.raises(RT.BlokRuntimeError, match="missing tokenizer.blok"):
        RT.tokenizer_encoding(tmp_path / "nothing.blok")


def test_tokenizer_blok_writer(tmp_path, small_tok):
    import base64
    ranks, _, _ = small_tok
    n = len(ranks)
    (tmp_path / "tiktoken.model").write_bytes(b"".join(base64.b64encode(b) + b" %d\n" % i for b, i in ranks.items()))
    added = {str(n + k): {"content": s} for k, s in enumerate(sorted(SPECIAL))}
    (tmp_path / "tokenizer_config.json").write_text(json.dumps({"added_tokens_decoder": added}))
    text = MI.tokenizer(tmp_path, n_tokens=n, n_special=len(SPECIAL))
    lines = text.splitlines()
    assert lines[0] == "blok-tokenizer-v2" and len(lines) == 1 + n + len(SPECIAL)
    assert lines[1] == f"tok 0 {bytes([byte_order()[0]]).hex()}" and lines[n + 1].startswith(f"special {n} ")
    (tmp_path / "meta").mkdir()
    (tmp_path / "meta" / "tokenizer.blok").write_text(text)
    enc = RT.tokenizer_encoding(tmp_path / "meta" / "tokenizer.blok")
    assert enc.decode(enc.encode("hello user<think>")) == "hello user<think>"
    with pytest.raises(SystemExit, match="unexpected Kimi tokenizer rank contract"):   # scripts/model_fetch.py:93-94
        MI.tokenizer(tmp_path)
    os.remove(tmp_path / "tiktoken.model")
    with pytest.raises(SystemExit, match="requires tiktoken.model"):                   # :84-85
        MI.tokenizer(tmp_path)


# ---- the host: prompt in, text out (scripts/test_host.py:43-54) ------------------------------------------
def _fake_executor(path, log, stdout, code=0, stderr=""):
    path.write_text(f"#!/bin/sh\nprintf '%s\\n' \"$@\" > {log}\nprintf '%s' '{stdout}'\nprintf '%s' '{stderr}' >&2\nexit {code}\n")
    path.chmod(path.stat().st_mode | stat.S_IXUSR)


def test_generate_spawns_the_executor_and_decodes(tmp_path, small_tok, monkeypatch):
    ranks, tok_path, enc = small_tok
    meta = tmp_path / "meta"
    meta.mkdir()
    (meta / "runtime-index.blok").write_text("blok-runtime-index-v1\n")
    (meta / "tokenizer.blok").write_text(tok_path.read_text())
    reply = enc.encode("<think>hm</think> <Paris>")
    exe, log = tmp_path / "exec", tmp_path / "argv.txt"
    _fake_executor(exe, log, json.dumps({"status": "ok", "token_ids": reply}, separators=(",", ":")))
    monkeypatch.setenv("BLOK_KIMI_EXEC_BIN", str(exe))
    text = RT.generate(model_dir=meta, prompt="Paris?", max_tokens=7, max_time=20)
    assert RT.answer(text) == "paris"
    argv = log.read_text().split("\n")[:-1]
    want_ids = enc.encode("<|im_user|>user<|im_middle|>Paris?<|im_end|><|im_assistant|>assistant<|im_middle|><think></think>")
    assert argv == ["--index", str(meta / "runtime-index.blok"), "--prompt-tokens", ",".join(map(str, want_ids)), "--tokens", "7"]
    # failures surface as BlokRuntimeError with the executor's words (blok/runtime.py:84-94)
    _fake_executor(exe, log, "", code=1, stderr="missing runtime tensor: 0:-1:resident:norm")
    with pytest.raises(RT.BlokRuntimeError, match="missing runtime tensor"):
        RT.generate(model_dir=meta, prompt="x", max_tokens=1, max_time=20)
    _fake_executor(exe, log, "not json")
    with pytest.raises(RT.BlokRuntimeError, match="invalid JSON"):
        RT.generate(model_dir=meta, prompt="x", max_tokens=1, max_time=20)
    _fake_executor(exe, log, json.dumps({"status": "ok", "token_ids": [163840]}))
    with pytest.raises(RT.BlokRuntimeError, match="executor failed"):
        RT.generate(model_dir=meta, prompt="x", max_tokens=1, max_time=20)
    for bad in (dict(prompt="", max_tokens=1, max_time=1), dict(prompt="x", max_tokens=0, max_time=1), dict(prompt="x", max_tokens=1, max_time=0)):
        with pytest.raises(RT.BlokRuntimeError, match="must be non-empty"):
            RT.generate(model_dir=meta, **bad)
    os.remove(meta / "tokenizer.blok")
    with pytest.raises(RT.BlokRuntimeError, match="missing required file"):
        RT.generate(model_dir=meta, prompt="x", max_tokens=1, max_time=20)


def test_runtime_index_resolution(tmp_path, monkeypatch):
    monkeypatch.setenv("BLOK_HOME", str(tmp_path / "home"))
    with pytest.raises(RT.BlokRuntimeError, match="runtime-index.blok not found"):
        RT.runtime_index(tmp_path)
    (tmp_path / "runtime-index.blok").write_text("blok-runtime-index-v1\n")
    assert RT.runtime_index(tmp_path) == (tmp_path / "runtime-index.blok").resolve()
    assert RT.runtime_index(tmp_path / "runtime-index.blok") == (tmp_path / "runtime-index.blok").resolve()
    (tmp_path / "config.json").write_text(json.dumps({"text_config": dict(RT.KIMI_TEXT, hidden_size=4096)}))
    with pytest.raises(RT.BlokRuntimeError, match="unsupported Kimi config fields: hidden_size"):
        RT.runtime_index(tmp_path)
    (tmp_path / "config.json").write_text(json.dumps({"text_config": RT.KIMI_TEXT}))
    assert RT.runtime_index(tmp_path).name == "runtime-index.blok"


def test_answer_normalisation():
    assert RT.answer("<think>no</think> <Paris>") == "paris"          # scripts/test_host.py:53
    assert RT.answer("  The Answer, is: 42! ") == "the answer is 42"
    assert RT.answer("a</think>b</think> C d") == "c d"
    assert RT.answer("<x") == "x"
