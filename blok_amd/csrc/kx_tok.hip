// kx_tok.hip -- tokenizer.blok: the byte-pair encoder on the caller's side of the executor (host code only).
//
// Reference: blok/runtime.py -- tokenizer_encoding() :121-134 hands the ranks and special tokens of tokenizer.blok
// and the split pattern KIMI_PATTERN (:37-48) to tiktoken; encode_prompt() :137-140 wraps the prompt in the chat
// template and encodes it with every special token allowed.  tokenizer.blok is written by scripts/model_fetch.py
// tokenizer() :81-97: a header line `blok-tokenizer-v2`, then `tok <id> <hex bytes>` and `special <id> <hex bytes>`.
// tiktoken itself (a dependency of the reference, requirements.txt; not part of it) is restated here from its
// published behaviour: split the text at special tokens, split the rest with the pattern, and merge the bytes of
// every piece by lowest rank first.
//
// The pattern is matched by hand instead of by a regex engine.  Its eight alternatives, tried in order at every
// position as a backtracking engine does (first alternative that matches wins, not the longest):
//   1  [\p{Han}]+
//   2  [^\r\n\p{L}\p{N}]? UP* LOW+ (?i:'s|'t|'re|'ve|'m|'ll|'d)?    UP  = [\p{Lu}\p{Lt}\p{Lm}\p{Lo}\p{M}] minus Han
//   3  [^\r\n\p{L}\p{N}]? UP+ LOW* (?i:'s|'t|'re|'ve|'m|'ll|'d)?    LOW = [\p{Ll}\p{Lm}\p{Lo}\p{M}] minus Han
//   4  \p{N}{1,3}
//   5  " "? [^\s\p{L}\p{N}]+ [\r\n]*
//   6  \s* [\r\n]+         7  \s+ (?!\S)         8  \s+
// UP and LOW overlap (Lm, Lo, M), so alternative 2 needs the engine's backtracking: UP* gives characters back until
// LOW+ finds one.  The character classes come from kx_unicode_tables.h.
#include <stdlib.h>
#include <string.h>
#include <string>
#include <unordered_map>
#include <vector>
#include "kx_common.h"
#include "kx_unicode_tables.h"

struct kx_tokenizer {
  std::unordered_map<std::string, uint32_t> ranks;      // mergeable byte strings
  std::vector<std::pair<std::string, uint32_t>> special;  // text, id
  std::vector<std::string> bytes_of;                     // id -> bytes (both kinds); empty = unused id
  bool special_first[256] = {};
  int32_t n_tokens = 0, n_special = 0;
};

namespace {

uint32_t class_of(uint32_t c) {
  size_t lo = 0, hi = sizeof(kx_unicode_ranges) / sizeof(kx_unicode_ranges[0]);
  while (lo < hi) {
    const size_t mid = (lo + hi) / 2;
    if (c > kx_unicode_ranges[mid].last) lo = mid + 1;
    else if (c < kx_unicode_ranges[mid].first) hi = mid;
    else return kx_unicode_ranges[mid].flags;
  }
  return 0;
}

struct Cp {
  uint32_t c, cls, off;  // code point, class flags, byte offset
};

// UTF-8 -> code points; a byte that is not part of a well-formed sequence becomes U+FFFD on its own
void decode_utf8(const unsigned char *s, size_t n, std::vector<Cp> &out) {
  out.clear();
  out.reserve(n + 1);
  size_t i = 0;
  while (i < n) {
    uint32_t c = s[i];
    size_t len = 1;
    if (c >= 0xC2 && c <= 0xDF && i + 1 < n && (s[i + 1] & 0xC0) == 0x80) {
      c = ((c & 0x1F) << 6) | (s[i + 1] & 0x3F);
      len = 2;
    } else if (c >= 0xE0 && c <= 0xEF && i + 2 < n && (s[i + 1] & 0xC0) == 0x80 && (s[i + 2] & 0xC0) == 0x80) {
      const uint32_t v = ((c & 0x0F) << 12) | ((s[i + 1] & 0x3F) << 6) | (s[i + 2] & 0x3F);
      if (v >= 0x800 && !(v >= 0xD800 && v <= 0xDFFF)) { c = v; len = 3; } else c = 0xFFFD;
    } else if (c >= 0xF0 && c <= 0xF4 && i + 3 < n && (s[i + 1] & 0xC0) == 0x80 && (s[i + 2] & 0xC0) == 0x80 &&
               (s[i + 3] & 0xC0) == 0x80) {
      const uint32_t v = ((c & 0x07) << 18) | ((s[i + 1] & 0x3F) << 12) | ((s[i + 2] & 0x3F) << 6) | (s[i + 3] & 0x3F);
      if (v >= 0x10000 && v <= 0x10FFFF) { c = v; len = 4; } else c = 0xFFFD;
    } else if (c >= 0x80) {
      c = 0xFFFD;
    }
    out.push_back(Cp{c, class_of(c), (uint32_t)i});
    i += len;
  }
  out.push_back(Cp{0, 0, (uint32_t)n});  // end marker
}

inline bool is_newline(const Cp &p) { return p.c == '\r' || p.c == '\n'; }
inline bool is_lead(const Cp &p) { return !is_newline(p) && !(p.cls & (KXU_L | KXU_N)); }  // [^\r\n\p{L}\p{N}]

bool fold_eq(uint32_t c, char lower) {  // case-insensitive as Unicode simple folding has it for these letters
  if (c == (uint32_t)lower || c == (uint32_t)(lower - 32)) return true;
  return lower == 's' && c == 0x17F;  // LATIN SMALL LETTER LONG S folds to s
}
// (?i:'s|'t|'re|'ve|'m|'ll|'d)? at index e of a text of n code points
size_t contraction(const std::vector<Cp> &t, size_t e, size_t n) {
  if (e + 1 >= n || t[e].c != '\'') return e;
  const uint32_t a = t[e + 1].c, b = e + 2 < n ? t[e + 2].c : 0;
  if (fold_eq(a, 's') || fold_eq(a, 't')) return e + 2;
  if ((fold_eq(a, 'r') || fold_eq(a, 'v')) && fold_eq(b, 'e')) return e + 3;
  if (fold_eq(a, 'm')) return e + 2;
  if (fold_eq(a, 'l') && fold_eq(b, 'l')) return e + 3;
  if (fold_eq(a, 'd')) return e + 2;
  return e;
}

// end index of the piece that starts at i (n = code points without the end marker); i when nothing matches
size_t piece_end(const std::vector<Cp> &t, size_t i, size_t n) {
  auto run = [&](size_t from, uint32_t mask) {
    size_t j = from;
    while (j < n && (t[j].cls & mask)) ++j;
    return j;
  };
  // 1
  if (t[i].cls & KXU_HAN) return run(i, KXU_HAN);
  // 2 and 3, each first with the optional lead character taken, then without it
  for (int alt = 2; alt <= 3; ++alt) {
    for (int lead = is_lead(t[i]) ? 1 : 0; lead >= 0; --lead) {
      const size_t p = i + lead;
      if (p >= n) continue;
      const size_t up_end = run(p, KXU_UP);
      if (alt == 2) {
        for (size_t q = up_end + 1; q-- > p;) {  // UP* gives back one character at a time
          const size_t low_end = run(q, KXU_LOW);
          if (low_end > q) return contraction(t, low_end, n);
        }
      } else if (up_end > p) {
        return contraction(t, run(up_end, KXU_LOW), n);
      }
    }
  }
  // 4
  if (t[i].cls & KXU_N) {
    size_t j = i;
    while (j < n && j < i + 3 && (t[j].cls & KXU_N)) ++j;
    return j;
  }
  // 5
  {
    size_t p = i + (t[i].c == ' ' ? 1 : 0), j = p;
    while (j < n && !(t[j].cls & (KXU_WS | KXU_L | KXU_N))) ++j;
    if (j > p) {
      while (j < n && is_newline(t[j])) ++j;
      return j;
    }
  }
  // 6, 7, 8 on the whitespace run that starts here
  const size_t ws_end = run(i, KXU_WS);
  if (ws_end > i) {
    for (size_t q = ws_end; q-- > i;)
      if (is_newline(t[q])) return q + 1;        // 6: up to the last line break of the run
    if (ws_end == n) return ws_end;              // 7: nothing follows
    if (ws_end - i >= 2) return ws_end - 1;      // 7: leave one whitespace character to the next piece
    return ws_end;                               // 8
  }
  return i;
}

// byte-pair merge of one piece: lowest rank first, leftmost on ties, until no adjacent pair is in the vocabulary
void bpe(const kx_tokenizer &tk, const std::string &piece, std::vector<uint32_t> &out) {
  auto whole = tk.ranks.find(piece);
  if (whole != tk.ranks.end()) {
    out.push_back(whole->second);
    return;
  }
  const uint32_t NONE = 0xffffffffu;
  struct Part { uint32_t start, rank; };  // rank of this part merged with the next one
  std::vector<Part> parts(piece.size() + 1);
  for (size_t k = 0; k <= piece.size(); ++k) parts[k] = Part{(uint32_t)k, NONE};
  std::string key;
  auto pair_rank = [&](size_t k) {
    if (k + 2 >= parts.size()) return NONE;
    key.assign(piece, parts[k].start, parts[k + 2].start - parts[k].start);
    auto f = tk.ranks.find(key);
    return f == tk.ranks.end() ? NONE : f->second;
  };
  for (size_t k = 0; k + 2 < parts.size(); ++k) parts[k].rank = pair_rank(k);
  for (;;) {
    uint32_t best = NONE;
    size_t at = 0;
    for (size_t k = 0; k + 1 < parts.size(); ++k)
      if (parts[k].rank < best) { best = parts[k].rank; at = k; }
    if (best == NONE) break;
    parts.erase(parts.begin() + (long)at + 1);
    parts[at].rank = pair_rank(at);
    if (at > 0) parts[at - 1].rank = pair_rank(at - 1);
  }
  for (size_t k = 0; k + 1 < parts.size(); ++k) {
    key.assign(piece, parts[k].start, parts[k + 1].start - parts[k].start);
    out.push_back(tk.ranks.at(key));  // single bytes are always present (checked when the file is read)
  }
}

void encode_ordinary(const kx_tokenizer &tk, const char *text, size_t len, std::vector<uint32_t> &out) {
  std::vector<Cp> cps;
  decode_utf8((const unsigned char *)text, len, cps);
  const size_t n = cps.size() - 1;
  std::string piece;
  for (size_t i = 0; i < n;) {
    size_t e = piece_end(cps, i, n);
    if (e == i) { ++i; continue; }  // the pattern covers every character; kept for safety
    piece.assign(text + cps[i].off, cps[e].off - cps[i].off);
    bpe(tk, piece, out);
    i = e;
  }
}

int hex_val(char c) { return c >= '0' && c <= '9' ? c - '0' : c >= 'a' && c <= 'f' ? c - 'a' + 10 : c >= 'A' && c <= 'F' ? c - 'A' + 10 : -1; }

int copy_out(const std::vector<uint32_t> &ids, uint32_t *h_ids, size_t cap, size_t *n, const char *who) {
  if (n) *n = ids.size();
  KX_REQUIRE(ids.size() <= cap && (h_ids || ids.empty()), "%s: %zu ids do not fit a buffer of %zu", who, ids.size(), cap);
  if (!ids.empty()) memcpy(h_ids, ids.data(), ids.size() * 4);
  return KX_OK;
}

}  // namespace

// ids index a table, so a hostile file must not be able to ask for gigabytes: no tokenizer.blok the reference
// writes goes beyond 163,840 ids (scripts/model_fetch.py:92)
constexpr unsigned long KX_TOK_MAX_ID = 1ul << 24;

static int kx_tokenizer_open_body(const char *path, kx_tokenizer **out) {
  KX_REQUIRE(path && out, "kx_tokenizer_open: null argument");
  *out = nullptr;
  FILE *f = fopen(path, "rb");
  KX_REQUIRE(f, "missing tokenizer.blok: %s", path);
  kx_tokenizer *tk = new kx_tokenizer();
  char *buf = nullptr;
  size_t cap = 0;
  ssize_t got;
  long lineno = 0;
  bool ok = true;
  while (ok && (got = getline(&buf, &cap, f)) >= 0) {
    ++lineno;
    while (got > 0 && (buf[got - 1] == '\n' || buf[got - 1] == '\r')) buf[--got] = 0;
    if (lineno == 1) {
      ok = strcmp(buf, "blok-tokenizer-v2") == 0;  // runtime.py:127-128
      continue;
    }
    if (got == 0) continue;
    char kind[16];
    unsigned long id = 0;
    int used = 0;
    if (sscanf(buf, "%15s %lu %n", kind, &id, &used) < 2 || (strcmp(kind, "tok") && strcmp(kind, "special")) || id >= KX_TOK_MAX_ID) { ok = false; break; }
    const char *hex = buf + used;
    const size_t hl = strlen(hex);
    if (hl == 0 || hl % 2) { ok = false; break; }
    std::string bytes(hl / 2, '\0');
    for (size_t k = 0; k < hl / 2 && ok; ++k) {
      const int a = hex_val(hex[2 * k]), b = hex_val(hex[2 * k + 1]);
      if (a < 0 || b < 0) ok = false;
      bytes[k] = (char)(a * 16 + b);
    }
    if (!ok) break;
    if (tk->bytes_of.size() <= id) tk->bytes_of.resize(id + 1);
    if (!tk->bytes_of[id].empty()) { ok = false; break; }  // an id twice
    tk->bytes_of[id] = bytes;
    if (kind[0] == 't') {
      ok = tk->ranks.emplace(bytes, (uint32_t)id).second;
      ++tk->n_tokens;
    } else {
      tk->special.emplace_back(bytes, (uint32_t)id);
      tk->special_first[(unsigned char)bytes[0]] = true;
      ++tk->n_special;
    }
  }
  free(buf);
  fclose(f);
  for (int b = 0; ok && b < 256 && tk->n_tokens > 0; ++b) ok = tk->ranks.count(std::string(1, (char)b)) == 1;  // byte fallback
  if (!ok || lineno < 1 || tk->n_tokens == 0) {
    delete tk;
    kx_set_error("bad tokenizer: %s (line %ld)", path, lineno);  // runtime.py:128
    return KX_ERR_ARG;
  }
  *out = tk;
  return KX_OK;
}

extern "C" int kx_tokenizer_close(kx_tokenizer *tk) {
  delete tk;
  return KX_OK;
}

extern "C" int kx_tokenizer_info(const kx_tokenizer *tk, int32_t *n_tokens, int32_t *n_special, int32_t *max_id) {
  KX_REQUIRE(tk, "kx_tokenizer_info: null tokenizer");
  if (n_tokens) *n_tokens = tk->n_tokens;
  if (n_special) *n_special = tk->n_special;
  if (max_id) *max_id = (int32_t)tk->bytes_of.size() - 1;
  return KX_OK;
}

static int kx_pretokenize_body(const char *text, size_t len, uint32_t *h_ends, size_t cap, size_t *n) {
  KX_REQUIRE(text || len == 0, "kx_pretokenize: null text");
  std::vector<Cp> cps;
  decode_utf8((const unsigned char *)text, len, cps);
  const size_t m = cps.size() - 1;
  std::vector<uint32_t> ends;
  for (size_t i = 0; i < m;) {
    size_t e = piece_end(cps, i, m);
    if (e == i) e = i + 1;
    ends.push_back(cps[e].off);
    i = e;
  }
  return copy_out(ends, h_ends, cap, n, "kx_pretokenize");
}

static int kx_tokenizer_encode_body(const kx_tokenizer *tk, const char *text, size_t len, int allow_special, uint32_t *h_ids,
                                   size_t cap, size_t *n) {
  KX_REQUIRE(tk && (text || len == 0), "kx_tokenizer_encode: null argument");
  std::vector<uint32_t> ids;
  size_t from = 0;
  if (allow_special && !tk->special.empty()) {
    for (size_t i = 0; i < len;) {
      const std::pair<std::string, uint32_t> *hit = nullptr;
      if (tk->special_first[(unsigned char)text[i]])
        for (const auto &sp : tk->special)
          if (sp.first.size() <= len - i && memcmp(text + i, sp.first.data(), sp.first.size()) == 0 &&
              (!hit || sp.first.size() > hit->first.size()))
            hit = &sp;
      if (!hit) { ++i; continue; }
      encode_ordinary(*tk, text + from, i - from, ids);
      ids.push_back(hit->second);
      i += hit->first.size();
      from = i;
    }
  }
  encode_ordinary(*tk, text + from, len - from, ids);
  return copy_out(ids, h_ids, cap, n, "kx_tokenizer_encode");
}

static int kx_tokenizer_decode_body(const kx_tokenizer *tk, const uint32_t *h_ids, size_t n_ids, char *h_bytes, size_t cap, size_t *len) {
  KX_REQUIRE(tk && (h_ids || n_ids == 0), "kx_tokenizer_decode: null argument");
  std::string out;
  for (size_t k = 0; k < n_ids; ++k) {
    KX_REQUIRE(h_ids[k] < tk->bytes_of.size() && !tk->bytes_of[h_ids[k]].empty(), "kx_tokenizer_decode: id %u is not in the tokenizer", h_ids[k]);
    out += tk->bytes_of[h_ids[k]];
  }
  if (len) *len = out.size();
  KX_REQUIRE(out.size() <= cap && (h_bytes || out.empty()), "kx_tokenizer_decode: %zu bytes do not fit a buffer of %zu", out.size(), cap);
  if (!out.empty()) memcpy(h_bytes, out.data(), out.size());
  return KX_OK;
}

static int kx_encode_prompt_body(const kx_tokenizer *tk, const char *prompt, size_t len, uint32_t *h_ids, size_t cap, size_t *n) {
  KX_REQUIRE(tk && (prompt || len == 0), "kx_encode_prompt: null argument");
  std::string text = "<|im_user|>user<|im_middle|>";  // runtime.py:139
  text.append(prompt, len);
  text += "<|im_end|><|im_assistant|>assistant<|im_middle|><think></think>";
  return kx_tokenizer_encode(tk, text.data(), text.size(), 1, h_ids, cap, n);
}

// ---- the C ABI: every body above runs under kx_guard, so that no exception leaves the library ----
extern "C" int kx_tokenizer_open(const char *path, kx_tokenizer **out) {
  return kx_guard("kx_tokenizer_open", [&] { return kx_tokenizer_open_body(path, out); });
}
extern "C" int kx_pretokenize(const char *text, size_t len, uint32_t *h_ends, size_t cap, size_t *n) {
  return kx_guard("kx_pretokenize", [&] { return kx_pretokenize_body(text, len, h_ends, cap, n); });
}
extern "C" int kx_tokenizer_encode(const kx_tokenizer *tk, const char *text, size_t len, int allow_special, uint32_t *h_ids, size_t cap, size_t *n) {
  return kx_guard("kx_tokenizer_encode", [&] { return kx_tokenizer_encode_body(tk, text, len, allow_special, h_ids, cap, n); });
}
extern "C" int kx_tokenizer_decode(const kx_tokenizer *tk, const uint32_t *h_ids, size_t n_ids, char *h_bytes, size_t cap, size_t *len) {
  return kx_guard("kx_tokenizer_decode", [&] { return kx_tokenizer_decode_body(tk, h_ids, n_ids, h_bytes, cap, len); });
}
extern "C" int kx_encode_prompt(const kx_tokenizer *tk, const char *prompt, size_t len, uint32_t *h_ids, size_t cap, size_t *n) {
  return kx_guard("kx_encode_prompt", [&] { return kx_encode_prompt_body(tk, prompt, len, h_ids, cap, n); });
}
