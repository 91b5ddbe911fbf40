"""Writes runtime-index.blok for a directory of safetensors shards.

Reference: scripts/model_fetch.py -- role() :62-69, runtime_slot() :71-79, tensors() :99-113 and
materialize() :115-131.  The index is plain text: the header line, then for every checkpoint tensor

    tensor <name> <role> <layer> <expert> <slot> <dtype> <shape> <off> <bytes> <align> <data> <data_bytes> <file>

where [data, data+data_bytes) is the tensor's byte range in <file> and [off, off+bytes) the enclosing
4096-aligned extent.  The executor (kx_model_load in include/kx.h, runtime_index() in the reference,
src/kimi_exec.cu:559-585) finds tensors by (layer, expert, role, slot), never by name.

Only the safetensors header is read here: 8 bytes little-endian length, then that many bytes of JSON
mapping names to {dtype, shape, data_offsets}; offsets count from the end of the header.
"""
import base64
import json
import re
import struct
import sys
from pathlib import Path

HEADER = "blok-runtime-index-v1"
ALIGN = 4096
PREFIX = "language_model."                     # the text decoder of the checkpoint; other towers are skipped (:107)
DTYPES = {"BF16": "bf16", "I32": "i32"}        # what the executor can run (:7, :108)
_LAYER = re.compile(r"\.layers\.(\d+)\.")
_EXPERT = re.compile(r"\.experts?\.(\d+)\.")
_FFN_WORDS = ("up_proj", "gate_proj", "w1", "w3", "down_proj", "w2")


def role(name):
    """Residency class of a tensor, first match wins (:62-69)."""
    if name.endswith((".mlp.gate.weight", ".mlp.gate.e_score_correction_bias")):
        return "router"
    rules = (
        (lambda n: "shared_experts" in n, "shared_expert_resident"),
        (lambda n: _EXPERT.search(n) is not None, "routed_expert"),
        (lambda n: ".self_attn." in n, "attention_resident"),
        (lambda n: any(w in n for w in _FFN_WORDS), "dense_ffn_rowcol"),
    )
    for test, value in rules:
        if test(name):
            return value
    return "resident"


def runtime_slot(name):
    """(layer, expert, slot): -1 where the name has no such coordinate (:71-79).

    The slot is the module name for `<module>.weight`, `<module>.weight_packed` style suffixes keep the
    module in front (`gate_proj.weight_packed`), any other last component is the slot itself
    (`e_score_correction_bias`)."""
    found = _LAYER.search(name)
    layer = int(found.group(1)) if found else -1
    found = _EXPERT.search(name)
    expert = int(found.group(1)) if found else -1
    parts = name.split(".")
    last = parts[-1]
    module = parts[-2] if len(parts) > 1 else last
    if last == "weight":
        slot = module
    elif last.startswith("weight_"):
        slot = module + "." + last
    else:
        slot = last
    return layer, expert, slot


def read_header(path):
    """(header dict, file offset of the data section) of one safetensors file."""
    with open(path, "rb") as f:
        raw = f.read(8)
        if len(raw) != 8:
            raise ValueError(f"{path}: not a safetensors file")
        (n,) = struct.unpack("<Q", raw)
        body = f.read(n)
        if len(body) != n:
            raise ValueError(f"{path}: truncated safetensors header")
    return json.loads(body), 8 + n


def tensors(local_dir):
    """Rows (name, role, dtype, shape, file, data_start, data_bytes) of every executable tensor (:99-113)."""
    rows = []
    for path in sorted(Path(local_dir).glob("*.safetensors")):
        header, base = read_header(path)
        for name, meta in header.items():
            if name == "__metadata__" or not name.startswith(PREFIX) or name.endswith(".weight_shape"):
                continue
            dtype = DTYPES.get(meta["dtype"])
            if dtype is None:
                continue
            begin, end = meta["data_offsets"]
            shape = "x".join(str(d) for d in meta["shape"])
            rows.append((name, role(name), dtype, shape, str(path), base + begin, end - begin))
    return rows


def index_lines(rows, align=ALIGN):
    lines = [HEADER]
    for name, kind, dtype, shape, file, start, size in rows:
        if any(ch.isspace() for ch in file):
            raise ValueError("model path cannot contain whitespace")  # :118
        off = start // align * align
        end = -(-(start + size) // align) * align
        layer, expert, slot = runtime_slot(name)
        lines.append(f"tensor {name} {kind} {layer} {expert} {slot} {dtype} {shape} {off} {end - off} {align} {start} {size} {file}")
    return lines


TOKENIZER_HEADER = "blok-tokenizer-v2"


def _tiktoken_ranks(path):
    """{rank: bytes} of a tiktoken.model file: one `<base64 of the byte string> <rank>` per non-empty line."""
    table = {}
    for number, raw in enumerate(path.read_bytes().split(b"\n"), 1):
        fields = raw.split()
        if not fields:
            continue
        if len(fields) != 2:
            raise SystemExit(f"{path.name}:{number}: expected '<base64> <rank>'")
        table[int(fields[1])] = base64.b64decode(fields[0])
    return table


def _special_tokens(path):
    """{id: utf-8 bytes} from the added_tokens_decoder map of tokenizer_config.json."""
    decoder = json.loads(path.read_text()).get("added_tokens_decoder") or {}
    return {int(token_id): entry["content"].encode() for token_id, entry in decoder.items()}


def tokenizer(local_dir, n_tokens=163584, n_special=256):
    """Text of tokenizer.blok (scripts/model_fetch.py:81-97 writes the same file): the header, `tok <id> <hex>` for every
    mergeable byte string in rank order, `special <id> <hex>` for every added token in id order.  The ranks must be
    exactly 0..n_tokens-1 and the special ids the n_special that follow (Kimi-K2: 163584 + 256 = the 163840-row
    embedding); n_tokens=None skips that check."""
    sources = [Path(local_dir) / name for name in ("tiktoken.model", "tokenizer_config.json")]
    if not all(p.is_file() for p in sources):
        raise SystemExit("pinned checkpoint requires tiktoken.model and tokenizer_config.json")
    sections = (("tok", _tiktoken_ranks(sources[0])), ("special", _special_tokens(sources[1])))
    if n_tokens is not None:
        expected = (range(n_tokens), range(n_tokens, n_tokens + n_special))
        if any(sorted(table) != list(ids) for (_, table), ids in zip(sections, expected)):
            raise SystemExit("unexpected Kimi tokenizer rank contract")
    out = [TOKENIZER_HEADER]
    for tag, table in sections:
        out.extend(f"{tag} {token_id} {table[token_id].hex()}" for token_id in sorted(table))
    return "\n".join(out) + "\n"


def materialize(local_dir, meta_dir, tokenizer_ranks=(163584, 256)):
    """Writes <meta_dir>/runtime-index.blok for the shards in local_dir and, when the checkpoint carries
    tiktoken.model, <meta_dir>/tokenizer.blok; returns a small report (:115-131)."""
    meta = Path(meta_dir)
    meta.mkdir(parents=True, exist_ok=True)
    report = {}
    if (Path(local_dir) / "tiktoken.model").is_file():
        n_tokens, n_special = tokenizer_ranks if tokenizer_ranks else (None, None)
        (meta / "tokenizer.blok").write_text(tokenizer(local_dir, n_tokens, n_special))
        report["tokenizer"] = str(meta / "tokenizer.blok")
    lines = index_lines(tensors(local_dir))
    index = meta / "runtime-index.blok"
    index.write_text("\n".join(lines) + "\n")
    report.update(tensors=len(lines) - 1, index=str(index))
    return report


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if len(argv) != 2:
        print("usage: python -m blok_amd.model_index <checkpoint-dir> <metadata-dir>", file=sys.stderr)
        return 64
    print(json.dumps(materialize(argv[0], argv[1]), separators=(",", ":")))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
