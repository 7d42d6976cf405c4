// Byte-pair-encoding tokenizer of the GPT-2 demo: what caten/llm's BPETokenizer does on the host
// (external/llm/bpe.lisp, external/llm/tokenizers.lisp) before and after the decode loop of
// gpt2-generate (apps/gpt2/gpt2.lisp:97-113).  Host code only; no device work.
//
//   make-bpe-tokenizer (bpe.lisp:14-38): `tokens` is split at single spaces and the first piece dropped,
//     the rest are numbered from 0; `merges` is split at newlines, the first line dropped, each remaining
//     line split at its space into a pair ranked by its line number.
//   encode (bpe.lisp:85-100): pre-tokenise with the GPT-2 pattern (bpe.lisp:3), spell every piece in the
//     byte alphabet (utils.lisp:15-272), merge pairs by rank (bpe-split, bpe.lisp:48-83), look the merged
//     symbols up; a symbol the vocabulary lacks becomes id 0.
//   decode (bpe.lisp:102-114): concatenate the symbols and map the byte alphabet back.
//
// Two deliberate differences, both outside what the reference's own test covers (test-tokenizer.lisp:26-37,
// ASCII sentences checked against tiktoken): text is spelled by its UTF-8 BYTES, as the vocabulary was built
// (the reference indexes the byte alphabet with character codes, which only agrees for ASCII), and decode
// applies the true inverse of the byte alphabet (the reference turns every symbol above U+00FF into a space,
// which is right for the space symbol and wrong for e.g. the newline symbol).
#include <stdint.h>
#include <string.h>

#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"
#include "unicode_tables.h"

namespace {

struct PairHash {
  size_t operator()(const std::pair<std::string, std::string> &p) const {
    return std::hash<std::string>()(p.first) * 1000003u ^ std::hash<std::string>()(p.second);
  }
};

struct BPE {
  std::unordered_map<std::string, int> encoder;
  std::vector<std::string> decoder;
  std::unordered_map<std::pair<std::string, std::string>, int, PairHash> merges;
  std::unordered_map<std::string, std::vector<int>> cache;  // piece (byte alphabet) -> ids
  std::string byte2uni[256];                                 // byte -> UTF-8 of its alphabet symbol
  std::unordered_map<uint32_t, uint8_t> uni2byte;           // alphabet code point -> byte
};

void append_utf8(std::string &s, uint32_t cp) {
  if (cp < 0x80) {
    s.push_back((char)cp);
  } else if (cp < 0x800) {
    s.push_back((char)(0xC0 | (cp >> 6)));
    s.push_back((char)(0x80 | (cp & 0x3F)));
  } else if (cp < 0x10000) {
    s.push_back((char)(0xE0 | (cp >> 12)));
    s.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
    s.push_back((char)(0x80 | (cp & 0x3F)));
  } else {
    s.push_back((char)(0xF0 | (cp >> 18)));
    s.push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
    s.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
    s.push_back((char)(0x80 | (cp & 0x3F)));
  }
}

// one code point of UTF-8 text at byte i; malformed bytes decode as themselves (one byte, class "other")
uint32_t next_cp(const char *s, size_t n, size_t i, size_t *len) {
  const unsigned char c = (unsigned char)s[i];
  auto cont = [&](size_t k) { return i + k < n && ((unsigned char)s[i + k] & 0xC0) == 0x80; };
  if (c < 0x80) {
    *len = 1;
    return c;
  }
  if ((c & 0xE0) == 0xC0 && cont(1)) {
    *len = 2;
    return ((c & 0x1Fu) << 6) | ((unsigned char)s[i + 1] & 0x3Fu);
  }
  if ((c & 0xF0) == 0xE0 && cont(1) && cont(2)) {
    *len = 3;
    return ((c & 0x0Fu) << 12) | (((unsigned char)s[i + 1] & 0x3Fu) << 6) | ((unsigned char)s[i + 2] & 0x3Fu);
  }
  if ((c & 0xF8) == 0xF0 && cont(1) && cont(2) && cont(3)) {
    *len = 4;
    return ((c & 0x07u) << 18) | (((unsigned char)s[i + 1] & 0x3Fu) << 12) | (((unsigned char)s[i + 2] & 0x3Fu) << 6) |
           ((unsigned char)s[i + 3] & 0x3Fu);
  }
  *len = 1;
  return 0xFFFFFFFFu;
}

template <size_t N>
bool in_ranges(const unsigned (&t)[N][2], uint32_t cp) {
  size_t lo = 0, hi = N;
  while (lo < hi) {
    const size_t mid = (lo + hi) / 2;
    if (cp < t[mid][0]) hi = mid;
    else if (cp > t[mid][1]) lo = mid + 1;
    else return true;
  }
  return false;
}

enum { C_SPACE, C_LETTER, C_NUMBER, C_OTHER };
int classify(uint32_t cp) {
  // \s of the reference's regex engine: the ASCII whitespace characters
  if (cp == ' ' || cp == '\t' || cp == '\n' || cp == '\r' || cp == '\f' || cp == '\v') return C_SPACE;
  if (cp == 0xFFFFFFFFu) return C_OTHER;
  if (in_ranges(kUnicodeLetters, cp)) return C_LETTER;
  if (in_ranges(kUnicodeNumbers, cp)) return C_NUMBER;
  return C_OTHER;
}

// 's|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+(?!\S)|\s+   (leftmost alternative that matches)
void pretokenize(const char *s, size_t n, std::vector<std::pair<size_t, size_t>> &out) {
  static const char *contractions[] = {"'s", "'t", "'re", "'ve", "'m", "'ll", "'d"};
  size_t i = 0;
  while (i < n) {
    if (s[i] == '\'') {
      bool hit = false;
      for (const char *c : contractions) {
        const size_t l = strlen(c);
        if (i + l <= n && memcmp(s + i, c, l) == 0) {
          out.push_back({i, l});
          i += l;
          hit = true;
          break;
        }
      }
      if (hit) continue;
    }
    // " ?X+" for X = letter, number, other: the class of the first character after an optional single space
    size_t j = i, len;
    if (s[j] == ' ' && j + 1 < n) {
      size_t l2;
      const int c2 = classify(next_cp(s, n, j + 1, &l2));
      if (c2 != C_SPACE) j++;
    }
    const int cls = classify(next_cp(s, n, j, &len));
    if (cls != C_SPACE) {
      size_t k = j;
      while (k < n) {
        size_t l3;
        if (classify(next_cp(s, n, k, &l3)) != cls) break;
        k += l3;
      }
      out.push_back({i, k - i});
      i = k;
      continue;
    }
    // a run of whitespace: all of it at the end of the text, all but its last character before a word
    // (that one is left for the " ?X+" alternatives), the single character otherwise
    size_t k = i;
    while (k < n && classify((unsigned char)s[k]) == C_SPACE) k++;
    size_t take = k - i;
    if (k < n && take > 1) take--;
    out.push_back({i, take});
    i += take;
  }
}

// bpe-split: merge the best-ranked adjacent pair, every occurrence left to right, until none is ranked
void bpe_split(const BPE &b, std::vector<std::string> &word) {
  while (word.size() > 1) {
    int best = -1;
    size_t at = 0;
    for (size_t i = 0; i + 1 < word.size(); i++) {
      auto it = b.merges.find({word[i], word[i + 1]});
      if (it != b.merges.end() && (best < 0 || it->second < best)) {
        best = it->second;
        at = i;
      }
    }
    if (best < 0) break;
    const std::string first = word[at], second = word[at + 1];
    std::vector<std::string> merged;
    merged.reserve(word.size());
    for (size_t i = 0; i < word.size();) {
      if (i + 1 < word.size() && word[i] == first && word[i + 1] == second) {
        merged.push_back(first + second);
        i += 2;
      } else {
        merged.push_back(word[i]);
        i++;
      }
    }
    word.swap(merged);
  }
}

}  // namespace

using cthip::fail;

extern "C" {

int cthip_bpe_create(void **out, const char *tokens, size_t tokens_len, const char *merges, size_t merges_len) {
  if (!out || !tokens || !merges) return fail(CTHIP_E_BAD_ARG, "cthip_bpe_create: null argument");
  BPE *b = new BPE();
  // the byte alphabet (utils.lisp:15-272): printable Latin-1 bytes stand for themselves, the other 68 bytes
  // take the code points 256, 257, ... in byte order
  int extra = 0;
  for (int byte = 0; byte < 256; byte++) {
    const bool keep = (byte >= 33 && byte <= 126) || (byte >= 161 && byte <= 172) || (byte >= 174 && byte <= 255);
    const uint32_t cp = keep ? (uint32_t)byte : 256u + (uint32_t)extra++;
    append_utf8(b->byte2uni[byte], cp);
    b->uni2byte[cp] = (uint8_t)byte;
  }
  // tokens: pieces between single spaces, the first dropped
  {
    size_t i = 0;
    int piece = 0;
    while (i <= tokens_len) {
      size_t j = i;
      while (j < tokens_len && tokens[j] != ' ') j++;
      if (piece > 0) {
        std::string t(tokens + i, j - i);
        b->encoder[t] = (int)b->decoder.size();  // a repeated spelling keeps its last id, as a hash table would
        b->decoder.push_back(t);
      }
      piece++;
      i = j + 1;
    }
  }
  // merges: lines, the first dropped; "a b" -> rank = line number - 1
  {
    size_t i = 0;
    int line = 0, rank = 0;
    while (i <= merges_len) {
      size_t j = i;
      while (j < merges_len && merges[j] != '\n') j++;
      if (line > 0) {
        const char *sp = (const char *)memchr(merges + i, ' ', j - i);
        if (sp) {
          std::string a(merges + i, sp - (merges + i));
          const char *rest = sp + 1;
          size_t rl = (merges + j) - rest;
          const char *sp2 = (const char *)memchr(rest, ' ', rl);  // anything after a second space is not part of the pair
          if (sp2) rl = sp2 - rest;
          b->merges[{a, std::string(rest, rl)}] = rank;
        }
        rank++;
      }
      line++;
      i = j + 1;
    }
  }
  *out = b;
  return 0;
}

int cthip_bpe_destroy(void *h) {
  delete (BPE *)h;
  return 0;
}

int cthip_bpe_vocab_size(const void *h) { return h ? (int)((const BPE *)h)->decoder.size() : -1; }

int cthip_bpe_encode(void *h, const char *text, size_t len, int *ids, size_t cap, size_t *n_out) {
  if (!h || (!text && len) || !n_out) return fail(CTHIP_E_BAD_ARG, "cthip_bpe_encode: null argument");
  BPE *b = (BPE *)h;
  std::vector<std::pair<size_t, size_t>> pieces;
  pretokenize(text, len, pieces);
  size_t n = 0;
  for (auto &p : pieces) {
    std::string spelled;
    for (size_t k = 0; k < p.second; k++) spelled += b->byte2uni[(unsigned char)text[p.first + k]];
    auto it = b->cache.find(spelled);
    if (it == b->cache.end()) {
      std::vector<std::string> word;
      for (size_t k = 0; k < p.second; k++) word.push_back(b->byte2uni[(unsigned char)text[p.first + k]]);
      bpe_split(*b, word);
      std::vector<int> v;
      for (const std::string &w : word) {
        auto e = b->encoder.find(w);
        v.push_back(e == b->encoder.end() ? 0 : e->second);  // (or (gethash bpetoken encoder) 0)
      }
      it = b->cache.emplace(spelled, std::move(v)).first;
    }
    for (int id : it->second) {
      if (ids && n < cap) ids[n] = id;
      n++;
    }
  }
  *n_out = n;
  if (ids && n > cap) return fail(CTHIP_E_BAD_ARG, "cthip_bpe_encode: %zu ids do not fit a buffer of %zu", n, cap);
  return 0;
}

int cthip_bpe_decode(const void *h, const int *ids, size_t n, char *out, size_t cap, size_t *len_out) {
  if (!h || (!ids && n) || !len_out) return fail(CTHIP_E_BAD_ARG, "cthip_bpe_decode: null argument");
  const BPE *b = (const BPE *)h;
  std::string bytes;
  for (size_t i = 0; i < n; i++) {
    if (ids[i] < 0 || ids[i] >= (int)b->decoder.size())
      return fail(CTHIP_E_BAD_ARG, "cthip_bpe_decode: id %d is outside the vocabulary of %zu", ids[i], b->decoder.size());
    const std::string &sym = b->decoder[ids[i]];
    for (size_t k = 0; k < sym.size();) {
      size_t l;
      const uint32_t cp = next_cp(sym.data(), sym.size(), k, &l);
      auto it = b->uni2byte.find(cp);
      if (it != b->uni2byte.end()) bytes.push_back((char)it->second);
      else bytes.append(sym, k, l);  // a symbol outside the byte alphabet (special tokens) is kept as spelled
      k += l;
    }
  }
  *len_out = bytes.size();
  if (out) {
    if (bytes.size() > cap) return fail(CTHIP_E_BAD_ARG, "cthip_bpe_decode: %zu bytes do not fit a buffer of %zu", bytes.size(), cap);
    memcpy(out, bytes.data(), bytes.size());
  }
  return 0;
}

}  // extern "C"
