// Byte-level BPE tokenizer behind the C ABI the reference binds (shim/gigatoken_wrapper/src/lib.rs:19-93, used by
// prototypes/decode.ts:78-86): gt_init(path to a Hugging Face tokenizer.json) / gt_encode / gt_encode_mt / gt_free.  The reference's
// wrapper is Rust over the gigatoken crate (a path dependency outside its tree, Cargo.toml:11); this is a C++ restatement
// of the published algorithm those files implement:
//   1. added tokens ("added_tokens": content -> id) are cut out of the text first, leftmost-longest;
//   2. the rest is split by the pre-tokenizer's regular expression (the Qwen / cl100k family, matched by a hand-written
//      scanner over code points with the Unicode general categories of unicode_tables.h);
//   3. every piece goes through the GPT-2 byte -> printable-character map and is merged pair by pair in rank order
//      ("merges"), lowest rank first, leftmost on ties; "ignore_merges" emits a piece that is a vocabulary entry as is.
// Not done: Unicode normalisation (a "normalizer" of type NFC in the file is accepted; the text is taken as already
// normalised), lstrip / rstrip / single_word flags of added tokens, case folding beyond ASCII in the contraction branch.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "unicode_tables.h"

namespace {

// ------------------------------------------------------------------ minimal JSON reader (objects, arrays, strings, scalars)
struct JValue {
  enum Kind { NUL, BOOL, NUM, STR, ARR, OBJ } kind = NUL;
  bool b = false;
  double num = 0;
  std::string str;
  std::vector<JValue> arr;
  std::vector<std::pair<std::string, JValue>> obj;
  const JValue* get(const char* key) const {
    for (const auto& kv : obj)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
};

struct JParser {
  const char* p;
  const char* end;
  bool ok = true;
  void ws() { while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) p++; }
  static void put_utf8(std::string& s, uint32_t cp) {
    if (cp < 0x80) s += (char)cp;
    else if (cp < 0x800) { s += (char)(0xC0 | (cp >> 6)); s += (char)(0x80 | (cp & 0x3F)); }
    else if (cp < 0x10000) { s += (char)(0xE0 | (cp >> 12)); s += (char)(0x80 | ((cp >> 6) & 0x3F)); s += (char)(0x80 | (cp & 0x3F)); }
    else { s += (char)(0xF0 | (cp >> 18)); s += (char)(0x80 | ((cp >> 12) & 0x3F)); s += (char)(0x80 | ((cp >> 6) & 0x3F)); s += (char)(0x80 | (cp & 0x3F)); }
  }
  uint32_t hex4() {
    uint32_t v = 0;
    for (int i = 0; i < 4 && p < end; i++, p++) {
      const char c = *p;
      v = v * 16 + (c >= '0' && c <= '9' ? c - '0' : c >= 'a' && c <= 'f' ? c - 'a' + 10 : c >= 'A' && c <= 'F' ? c - 'A' + 10 : (ok = false, 0));
    }
    return v;
  }
  std::string string() {
    std::string s;
    if (p >= end || *p != '"') { ok = false; return s; }
    p++;
    while (p < end && *p != '"') {
      if (*p == '\\') {
        p++;
        if (p >= end) { ok = false; break; }
        const char c = *p++;
        switch (c) {
          case 'n': s += '\n'; break; case 't': s += '\t'; break; case 'r': s += '\r'; break;
          case 'b': s += '\b'; break; case 'f': s += '\f'; break;
          case 'u': {
            uint32_t cp = hex4();
            if (cp >= 0xD800 && cp < 0xDC00 && p + 1 < end && p[0] == '\\' && p[1] == 'u') {   // surrogate pair
              p += 2;
              const uint32_t lo = hex4();
              cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
            }
            put_utf8(s, cp);
            break;
          }
          default: s += c;      // \" \\ \/
        }
      } else {
        s += *p++;
      }
    }
    if (p >= end) ok = false; else p++;
    return s;
  }
  JValue value() {
    JValue v;
    ws();
    if (p >= end) { ok = false; return v; }
    if (*p == '{') {
      v.kind = JValue::OBJ; p++; ws();
      if (p < end && *p == '}') { p++; return v; }
      while (ok) {
        ws();
        std::string k = string();
        ws();
        if (p >= end || *p != ':') { ok = false; break; }
        p++;
        v.obj.emplace_back(std::move(k), value());
        ws();
        if (p < end && *p == ',') { p++; continue; }
        if (p < end && *p == '}') { p++; break; }
        ok = false;
      }
    } else if (*p == '[') {
      v.kind = JValue::ARR; p++; ws();
      if (p < end && *p == ']') { p++; return v; }
      while (ok) {
        v.arr.push_back(value());
        ws();
        if (p < end && *p == ',') { p++; continue; }
        if (p < end && *p == ']') { p++; break; }
        ok = false;
      }
    } else if (*p == '"') {
      v.kind = JValue::STR; v.str = string();
    } else if (!strncmp(p, "true", 4)) { v.kind = JValue::BOOL; v.b = true; p += 4; }
    else if (!strncmp(p, "false", 5)) { v.kind = JValue::BOOL; v.b = false; p += 5; }
    else if (!strncmp(p, "null", 4)) { v.kind = JValue::NUL; p += 4; }
    else {
      char* e = nullptr;
      v.kind = JValue::NUM; v.num = strtod(p, &e);
      if (e == p) ok = false;
      p = e;
    }
    return v;
  }
};

// ------------------------------------------------------------------ code points and classes
bool in_ranges(const uint32_t (*t)[2], int n, uint32_t cp) {
  int lo = 0, hi = n - 1;
  while (lo <= hi) {
    const int mid = (lo + hi) / 2;
    if (cp < t[mid][0]) hi = mid - 1;
    else if (cp > t[mid][1]) lo = mid + 1;
    else return true;
  }
  return false;
}
bool is_letter(uint32_t cp) { return cp < 0x80 ? ((cp | 0x20) >= 'a' && (cp | 0x20) <= 'z') : in_ranges(UNI_LETTER, UNI_LETTER_count, cp); }
bool is_number(uint32_t cp) { return cp < 0x80 ? (cp >= '0' && cp <= '9') : in_ranges(UNI_NUMBER, UNI_NUMBER_count, cp); }
bool is_space(uint32_t cp) {       // the White_Space property (what \s means in the file's regular expression)
  return (cp >= 0x09 && cp <= 0x0D) || cp == 0x20 || cp == 0x85 || cp == 0xA0 || cp == 0x1680 || (cp >= 0x2000 && cp <= 0x200A) ||
         cp == 0x2028 || cp == 0x2029 || cp == 0x202F || cp == 0x205F || cp == 0x3000;
}

// Classes of the ASCII range in one table (bit 0 letter, 1 number, 2 space, 3 line break); the rest by range search.
enum : uint8_t { C_LETTER = 1, C_NUMBER = 2, C_SPACE = 4, C_NEWLINE = 8 };
struct AsciiClass {
  uint8_t t[128];
  constexpr AsciiClass() : t() {
    for (int c = 0; c < 128; c++) {
      uint8_t k = 0;
      if ((c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z')) k |= C_LETTER;
      if (c >= '0' && c <= '9') k |= C_NUMBER;
      if ((c >= 0x09 && c <= 0x0D) || c == 0x20) k |= C_SPACE;
      if (c == '\r' || c == '\n') k |= C_NEWLINE;
      t[c] = k;
    }
  }
};
constexpr AsciiClass ASCII_CLASS;
inline uint8_t classes(uint32_t cp) {
  if (cp < 0x80) return ASCII_CLASS.t[cp];
  return (is_letter(cp) ? C_LETTER : 0) | (is_number(cp) ? C_NUMBER : 0) | (is_space(cp) ? C_SPACE : 0);
}

// ------------------------------------------------------------------ the pre-tokenizer's regular expression, by hand
//   (?i:'s|'t|'re|'ve|'m|'ll|'d) | [^\r\n\p{L}\p{N}]?\p{L}+ | \p{N}{1,D} | ?[^\s\p{L}\p{N}]+[\r\n]* | \s*[\r\n]+ | \s+(?!\S) | \s+
// Alternatives are tried in this order at every position and the first that matches wins; D = 1 (Qwen) or 3 (cl100k).
// The scanner walks the UTF-8 bytes themselves: a code point is decoded where it is looked at (one table lookup for
// ASCII), and a malformed byte counts as one code point U+FFFD that covers that byte.
struct Scanner {
  int max_digits = 1;

  struct At { uint32_t cp; uint32_t len; uint8_t cls; };      // code point at a byte offset, its length, its classes; len 0 = end
  __attribute__((always_inline)) static inline At at(const uint8_t* s, size_t n, size_t i) {
    if (i >= n) return {0, 0, 0};
    const uint8_t c = s[i];
    if (c < 0x80) return {c, 1, ASCII_CLASS.t[c]};
    return at_multibyte(s, n, i);
  }
  static At at_multibyte(const uint8_t* s, size_t n, size_t i) {
    const uint8_t c = s[i];
    uint32_t cp = 0xFFFD, len = 1;
    if ((c & 0xE0) == 0xC0 && i + 1 < n && (s[i + 1] & 0xC0) == 0x80) { cp = ((c & 0x1F) << 6) | (s[i + 1] & 0x3F); len = 2; }
    else if ((c & 0xF0) == 0xE0 && i + 2 < n && (s[i + 1] & 0xC0) == 0x80 && (s[i + 2] & 0xC0) == 0x80) {
      cp = ((c & 0x0F) << 12) | ((s[i + 1] & 0x3F) << 6) | (s[i + 2] & 0x3F); len = 3;
    } else if ((c & 0xF8) == 0xF0 && i + 3 < n && (s[i + 1] & 0xC0) == 0x80 && (s[i + 2] & 0xC0) == 0x80 && (s[i + 3] & 0xC0) == 0x80) {
      cp = ((c & 0x07) << 18) | ((s[i + 1] & 0x3F) << 12) | ((s[i + 2] & 0x3F) << 6) | (s[i + 3] & 0x3F); len = 4;
    }
    return {cp, len, classes(cp)};
  }

  // returns the number of bytes of the piece that starts at s[i] (i < n)
  size_t next(const uint8_t* s, size_t n, size_t i) const {
    auto lower = [](uint8_t x) -> uint8_t { return x >= 'A' && x <= 'Z' ? x + 32 : x; };
    const At x = at(s, n, i);
    if (x.cp == '\'' && i + 1 < n) {
      const uint8_t a = lower(s[i + 1]), b = i + 2 < n ? lower(s[i + 2]) : 0;     // a byte >= 0x80 matches none of these
      if (a == 's' || a == 't') return 2;
      if ((a == 'r' && b == 'e') || (a == 'v' && b == 'e')) return 3;
      if (a == 'm') return 2;
      if (a == 'l' && b == 'l') return 3;
      if (a == 'd') return 2;
    }
    {   // [^\r\n\p{L}\p{N}]?\p{L}+
      size_t k = i;
      At y = x;
      if (!(x.cls & (C_NEWLINE | C_LETTER | C_NUMBER))) {
        const At z = at(s, n, i + x.len);
        if (z.cls & C_LETTER) { k = i + x.len; y = z; }
      }
      if (y.cls & C_LETTER) {
        do { k += y.len; y = at(s, n, k); } while (y.cls & C_LETTER);
        return k - i;
      }
    }
    if (x.cls & C_NUMBER) {
      size_t k = i; int digits = 0;
      At y = x;
      while (digits < max_digits && (y.cls & C_NUMBER)) { k += y.len; digits++; y = at(s, n, k); }
      return k - i;
    }
    {   //  ?[^\s\p{L}\p{N}]+[\r\n]*
      size_t k = i;
      At y = x;
      if (x.cp == ' ' && i + 1 < n) { k = i + 1; y = at(s, n, k); }
      if (y.len && !(y.cls & (C_SPACE | C_LETTER | C_NUMBER))) {
        do { k += y.len; y = at(s, n, k); } while (y.len && !(y.cls & (C_SPACE | C_LETTER | C_NUMBER)));
        while (y.cls & C_NEWLINE) { k += y.len; y = at(s, n, k); }
        return k - i;
      }
    }
    if (x.cls & C_SPACE) {
      size_t e = i, last_start = i, nl_end = 0;         // end of the run, start of its last character, end of its last line break
      At y = x;
      while (y.cls & C_SPACE) {
        last_start = e;
        e += y.len;
        if (y.cls & C_NEWLINE) nl_end = e;
        y = at(s, n, e);
      }
      if (nl_end) return nl_end - i;                      // \s*[\r\n]+ : up to and including the last line break of the run
      if (e == n) return e - i;                           // \s+(?!\S) : the whole run at the end of the text,
      if (last_start > i) return last_start - i;          //               else all but its last character
      return x.len;                                       // \s+
    }
    return x.len;     // not reachable for well-formed input: every code point is a letter, number, space or "other"
  }
};

// ------------------------------------------------------------------ the tokenizer
struct PairHash {
  size_t operator()(uint64_t k) const { return (size_t)(k * 0x9E3779B97F4A7C15ull >> 17); }
};

struct Tokenizer {
  std::unordered_map<std::string, uint32_t> vocab;
  std::unordered_map<uint64_t, std::pair<uint32_t, uint32_t>, PairHash> merges;     // (left id, right id) -> (rank, merged id)
  std::vector<std::pair<std::string, uint32_t>> added;                              // content, id
  bool added_first[256] = {};     // some added token begins with this byte
  uint32_t byte_id[256];          // id of the one-character token of every byte
  std::string byte_char[256];     // the printable character (UTF-8) a byte maps to
  bool ignore_merges = false;
  Scanner scan;
  std::string error;

  bool load(const char* path) {
    FILE* f = fopen(path, "rb");
    if (!f) { error = std::string("cannot open ") + path; return false; }
    std::string text;
    char buf[1 << 16];
    size_t got;
    while ((got = fread(buf, 1, sizeof buf, f)) > 0) text.append(buf, got);
    fclose(f);
    JParser jp{text.data(), text.data() + text.size()};
    const JValue root = jp.value();
    if (!jp.ok || root.kind != JValue::OBJ) { error = "tokenizer.json: not valid JSON"; return false; }
    const JValue* model = root.get("model");
    if (!model || !model->get("vocab") || !model->get("merges")) { error = "tokenizer.json: no model.vocab / model.merges"; return false; }
    if (const JValue* t = model->get("type")) if (t->kind == JValue::STR && t->str != "BPE") { error = "tokenizer.json: model type is not BPE"; return false; }
    if (const JValue* im = model->get("ignore_merges")) ignore_merges = im->kind == JValue::BOOL && im->b;
    for (const auto& kv : model->get("vocab")->obj) vocab.emplace(kv.first, (uint32_t)kv.second.num);
    // GPT-2 byte map: printable bytes map to themselves, the others to U+0100 onwards in byte order
    int extra = 0;
    for (int b = 0; b < 256; b++) {
      const bool printable = (b >= 0x21 && b <= 0x7E) || (b >= 0xA1 && b <= 0xAC) || (b >= 0xAE && b <= 0xFF);
      const uint32_t cp = printable ? (uint32_t)b : 0x100u + extra++;
      JParser::put_utf8(byte_char[b], cp);
      auto it = vocab.find(byte_char[b]);
      if (it == vocab.end()) { error = "tokenizer.json: the vocabulary lacks a byte-level base token"; return false; }
      byte_id[b] = it->second;
    }
    uint32_t rank = 0;
    for (const JValue& m : model->get("merges")->arr) {
      std::string a, b;
      if (m.kind == JValue::ARR && m.arr.size() == 2) { a = m.arr[0].str; b = m.arr[1].str; }
      else if (m.kind == JValue::STR) {
        const size_t sp = m.str.find(' ');
        if (sp == std::string::npos) { error = "tokenizer.json: malformed merge"; return false; }
        a = m.str.substr(0, sp); b = m.str.substr(sp + 1);
      } else { error = "tokenizer.json: malformed merge"; return false; }
      auto ia = vocab.find(a), ib = vocab.find(b), iab = vocab.find(a + b);
      if (ia == vocab.end() || ib == vocab.end() || iab == vocab.end()) { error = "tokenizer.json: merge of unknown tokens"; return false; }
      merges.emplace(((uint64_t)ia->second << 32) | ib->second, std::make_pair(rank, iab->second));
      rank++;
    }
    if (const JValue* at = root.get("added_tokens"))
      for (const JValue& t : at->arr) {
        const JValue *c = t.get("content"), *id = t.get("id");
        if (c && id && !c->str.empty()) { added.emplace_back(c->str, (uint32_t)id->num); added_first[(uint8_t)c->str[0]] = true; }
      }
    // the split pattern decides how many digits form one piece
    if (const JValue* pt = root.get("pre_tokenizer")) {
      std::string all;
      collect_strings(*pt, all);
      if (all.find("\\p{N}{1,3}") != std::string::npos) scan.max_digits = 3;
    }
    return true;
  }
  static void collect_strings(const JValue& v, std::string& out) {
    if (v.kind == JValue::STR) { out += v.str; out += '\n'; }
    for (const JValue& e : v.arr) collect_strings(e, out);
    for (const auto& kv : v.obj) collect_strings(kv.second, out);
  }

  // one pre-token (raw bytes) -> ids
  void bpe(const uint8_t* s, size_t n, std::vector<uint32_t>& out) const {
    if (n == 0) return;
    if (ignore_merges) {
      std::string whole;
      for (size_t i = 0; i < n; i++) whole += byte_char[s[i]];
      auto it = vocab.find(whole);
      if (it != vocab.end()) { out.push_back(it->second); return; }
    }
    // lowest rank first, leftmost on ties, until no neighbouring pair is a merge.  rank[i] / into[i] describe the pair
    // (sym[i], sym[i + 1]); a merge changes the two pairs beside it only, so the table is looked up once per new pair
    uint32_t stack_buf[3 * 64];
    std::vector<uint32_t> heap_buf;
    uint32_t* sym = stack_buf;
    if (n > 64) { heap_buf.resize(3 * n); sym = heap_buf.data(); }
    uint32_t* rank = sym + n;
    uint32_t* into = rank + n;
    auto look = [&](size_t i) {
      auto it = merges.find(((uint64_t)sym[i] << 32) | sym[i + 1]);
      if (it == merges.end()) { rank[i] = 0xFFFFFFFFu; into[i] = 0; }
      else { rank[i] = it->second.first; into[i] = it->second.second; }
    };
    for (size_t i = 0; i < n; i++) sym[i] = byte_id[s[i]];
    size_t len = n;
    for (size_t i = 0; i + 1 < len; i++) look(i);
    while (len > 1) {
      uint32_t best = 0xFFFFFFFFu; size_t at = 0;
      for (size_t i = 0; i + 1 < len; i++)
        if (rank[i] < best) { best = rank[i]; at = i; }
      if (best == 0xFFFFFFFFu) break;
      sym[at] = into[at];
      for (size_t i = at + 1; i + 1 < len; i++) { sym[i] = sym[i + 1]; rank[i] = rank[i + 1]; into[i] = into[i + 1]; }
      len--;
      if (at + 1 < len) look(at);
      if (at > 0) look(at - 1);
    }
    out.insert(out.end(), sym, sym + len);
  }

  // Pieces repeat (words, indentation, punctuation runs): the ids of a piece of up to 24 bytes are kept for the rest of
  // the call.  The table belongs to the call, not to the tokenizer, so calls on several threads share nothing.
  struct PieceCache {
    struct Entry { uint8_t len = 0xFF, nids = 0; uint8_t bytes[24]; uint32_t ids[8]; };
    std::vector<Entry> slots;
    // sized from the input (a slot per 8 bytes, 256 to 16384 slots): a chat-sized call does not pay for a megabyte
    explicit PieceCache(size_t input_bytes) {
      size_t want = 256;
      while (want < (1u << 14) && want < input_bytes / 8) want <<= 1;
      slots.resize(want);
    }
    static size_t hash(const uint8_t* s, size_t n) {
      uint64_t h = 0xcbf29ce484222325ull ^ n;
      for (size_t i = 0; i < n; i++) h = (h ^ s[i]) * 0x100000001b3ull;
      return (size_t)(h ^ (h >> 29));
    }
  };

  void encode_plain(const uint8_t* s, size_t n, std::vector<uint32_t>& out, PieceCache& cache) const {
    size_t i = 0;
    while (i < n) {
      const size_t pn = scan.next(s, n, i);
      if (pn <= 24) {
        PieceCache::Entry& e = cache.slots[PieceCache::hash(s + i, pn) & (cache.slots.size() - 1)];
        if (e.len == pn && !memcmp(e.bytes, s + i, pn)) {
          out.insert(out.end(), e.ids, e.ids + e.nids);
        } else {
          const size_t before = out.size();
          bpe(s + i, pn, out);
          const size_t got = out.size() - before;
          if (got <= 8) {
            e.len = (uint8_t)pn; e.nids = (uint8_t)got;
            memcpy(e.bytes, s + i, pn);
            memcpy(e.ids, out.data() + before, got * sizeof(uint32_t));
          }
        }
      } else {
        bpe(s + i, pn, out);
      }
      i += pn;
    }
  }

  void encode(const uint8_t* s, size_t n, std::vector<uint32_t>& out) const {
    PieceCache cache(n);
    size_t start = 0, i = 0;
    while (i < n && !added.empty()) {
      if (!added_first[s[i]]) { i++; continue; }       // no added token begins with this byte
      // leftmost-longest added token at i
      size_t best_len = 0; uint32_t best_id = 0;
      for (const auto& a : added)
        if (a.first.size() > best_len && a.first.size() <= n - i && (uint8_t)a.first[0] == s[i] && !memcmp(a.first.data(), s + i, a.first.size())) {
          best_len = a.first.size(); best_id = a.second;
        }
      if (best_len) {
        encode_plain(s + start, i - start, out, cache);
        out.push_back(best_id);
        i += best_len;
        start = i;
      } else {
        i++;
      }
    }
    encode_plain(s + start, n - start, out, cache);
  }
};

thread_local std::string g_last_error;

}  // namespace

extern "C" {

// shim/gigatoken_wrapper/src/lib.rs:19-33: null on failure
__attribute__((visibility("default"))) void* gt_init(const char* path) {
  if (!path) { g_last_error = "gt_init: null path"; return nullptr; }
  Tokenizer* t = new Tokenizer();
  if (!t->load(path)) { g_last_error = t->error; delete t; return nullptr; }
  return t;
}

// lib.rs:35-46: ids of `text` into out_buf; returns the number written (at most out_max), -1 on a null argument
__attribute__((visibility("default"))) int gt_encode(void* tok, const uint8_t* text, size_t text_len, uint32_t* out_buf, size_t out_max) {
  if (!tok || !text || !out_buf) return -1;
  std::vector<uint32_t> ids;
  ids.reserve(text_len);
  ((const Tokenizer*)tok)->encode(text, text_len, ids);
  const size_t n = ids.size() < out_max ? ids.size() : out_max;
  memcpy(out_buf, ids.data(), n * sizeof(uint32_t));
  return (int)n;
}

// lib.rs:47-88: the text is cut into one chunk per hardware thread, each chunk ending behind the first space at or past
// its share of the bytes, and the chunks are encoded side by side; a chunk is encoded on its own, so the ids are those
// of gt_encode over each chunk (a piece that spans a cut is split there, as in the reference).  Returns the number of
// ids of all chunks together, which may exceed out_max: a chunk whose ids do not fit behind the ones before it is left
// out.  The reference hands chunks their place in out_buf in the order they finish; here chunk i follows chunk i - 1.
__attribute__((visibility("default"))) int gt_encode_mt(void* tok, const uint8_t* text, size_t text_len, uint32_t* out_buf, size_t out_max) {
  if (!tok || !text || !out_buf) return -1;
  const Tokenizer* t = (const Tokenizer*)tok;
  size_t n_threads = std::thread::hardware_concurrency();
  if (n_threads == 0) n_threads = 32;                       // lib.rs:26
  const size_t chunk_size = (text_len + n_threads - 1) / n_threads;
  std::vector<std::pair<size_t, size_t>> chunks;            // (start, end)
  for (size_t s = 0; s < text_len;) {
    size_t e = s + chunk_size < text_len ? s + chunk_size : text_len;
    if (e < text_len) {
      while (e < text_len && text[e] != ' ') e++;
      if (e < text_len) e++;
    }
    chunks.emplace_back(s, e);
    s = e;
  }
  std::vector<std::vector<uint32_t>> ids(chunks.size());
  std::vector<std::thread> workers;
  const size_t nw = chunks.size() < n_threads ? chunks.size() : n_threads;
  for (size_t w = 0; w < nw; w++)
    workers.emplace_back([&, w] {
      for (size_t c = w; c < chunks.size(); c += nw) {
        ids[c].reserve(chunks[c].second - chunks[c].first);
        t->encode(text + chunks[c].first, chunks[c].second - chunks[c].first, ids[c]);
      }
    });
  for (auto& th : workers) th.join();
  size_t cursor = 0;
  for (const auto& v : ids) {
    if (cursor + v.size() <= out_max) memcpy(out_buf + cursor, v.data(), v.size() * sizeof(uint32_t));
    cursor += v.size();
  }
  return (int)cursor;
}

// lib.rs:90-93
__attribute__((visibility("default"))) void gt_free(void* tok) { delete (Tokenizer*)tok; }

// why the last gt_init of this thread returned null (not in the reference's wrapper, which only returns null)
__attribute__((visibility("default"))) const char* gt_last_error(void) { return g_last_error.c_str(); }

}
