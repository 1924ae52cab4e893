// Byte-level BPE tokenizer of the Qwen2 family (GPT-2 style), the text side of the decode
// path: vocabulary, merges and control tokens come from a GGUF file's tokenizer.ggml.*
// metadata. Same surface and same results as the reference's tl::tokenizer
// (include/tokenizer.h: encode, decode, eos_id, bos_id, control tokens matched atomically,
// no BOS/EOS added), written as:
//   * a scanner over code points for the pre-tokenizer regex
//       (?i:'s|'t|'re|'ve|'m|'ll|'d) | [^\r\n\p{L}\p{N}]?\p{L}+ | \p{N}
//       | ?[^\s\p{L}\p{N}]+[\r\n]* | \s*[\r\n]+ | \s+(?!\S) | \s+
//     (first alternative that matches wins, each greedy),
//   * the GPT-2 byte -> printable code point map, computed, not tabulated,
//   * BPE merging on a linked list with a heap of candidate pairs: lowest merge rank first,
//     leftmost among equals - the order the reference's quadratic rescans produce
//     (tokenizer.h:262-282) at O(n log n).
#pragma once

#include <cstdint>
#include <queue>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "gguf.h"
#include "unicode_tables.h"

namespace tl {

class tokenizer {
 public:
  explicit tokenizer(const std::string& gguf_path) : tokenizer(gguf::model(gguf_path)) {}

  explicit tokenizer(const gguf::model& m) {
    pieces_ = m.kv("tokenizer.ggml.tokens").as_str_array();
    id_of_.reserve(pieces_.size() * 2);
    for (size_t i = 0; i < pieces_.size(); i++) id_of_.emplace(pieces_[i], static_cast<int>(i));   // first id wins

    const std::vector<std::string> merges = m.kv("tokenizer.ggml.merges").as_str_array();
    rank_of_.reserve(merges.size() * 2);
    for (size_t i = 0; i < merges.size(); i++) rank_of_.emplace(merges[i], static_cast<int>(i));   // "left right"

    // control tokens (type 3) are cut out of the text before anything else sees it
    const gguf::metadata_value& types = m.kv("tokenizer.ggml.token_type");
    for (size_t i = 0; i < types.arr.size() && i < pieces_.size(); i++)
      if (types.arr[i].i == 3) controls_.emplace_back(pieces_[i], static_cast<int>(i));

    eos_ = static_cast<int>(m.kv("tokenizer.ggml.eos_token_id").as_u32());
    bos_ = static_cast<int>(m.kv("tokenizer.ggml.bos_token_id").as_u32());

    // GPT-2's bytes_to_unicode: printable Latin-1 bytes stand for themselves, the other 68
    // bytes take code points 256, 257, ... in byte order.
    uint32_t next = 256;
    for (uint32_t b = 0; b < 256; b++) {
      const bool keeps = (b >= 33 && b <= 126) || (b >= 161 && b <= 172) || (b >= 174);
      const uint32_t cp = keeps ? b : next++;
      append_utf8(byte_piece_[b], cp);
      byte_of_.emplace(cp, static_cast<uint8_t>(b));
    }
  }

  int eos_id() const { return eos_; }
  int bos_id() const { return bos_; }
  size_t vocab_size() const { return pieces_.size(); }

  // UTF-8 text -> ids. Control-token strings inside the text become their id; the text
  // between them is pre-tokenized and merged.
  std::vector<int> encode(const std::string& text) const {
    std::vector<int> ids;
    size_t plain_from = 0, at = 0;
    while (at < text.size()) {
      int hit = -1;
      size_t hit_len = 0;
      for (const auto& c : controls_)   // longest control token starting here
        if (c.first.size() > hit_len && text.compare(at, c.first.size(), c.first) == 0) {
          hit = c.second;
          hit_len = c.first.size();
        }
      if (hit < 0) {
        at++;
        continue;
      }
      plain(text, plain_from, at, ids);
      ids.push_back(hit);
      at += hit_len;
      plain_from = at;
    }
    plain(text, plain_from, text.size(), ids);
    return ids;
  }

  // ids -> the raw bytes they stand for (control tokens give their literal text).
  std::string decode(const std::vector<int>& ids) const {
    std::string shown;
    for (int id : ids) {
      if (id < 0 || static_cast<size_t>(id) >= pieces_.size()) throw std::runtime_error("tokenizer: id out of range");
      shown += pieces_[static_cast<size_t>(id)];
    }
    std::string bytes;
    bytes.reserve(shown.size());
    for (size_t p = 0; p < shown.size();) {
      const auto it = byte_of_.find(read_utf8(shown, p));
      if (it == byte_of_.end()) throw std::runtime_error("tokenizer: codepoint not in byte map");
      bytes.push_back(static_cast<char>(it->second));
    }
    return bytes;
  }

 private:
  // One code point at s[p], p advanced. A lead byte without all of its continuation bytes
  // inside the string, and any other stray byte, counts as a code point of its own value
  // (the reference's rule, tokenizer.h:113-137: the classes below then see e.g. 0xAA as a letter).
  static uint32_t read_utf8(const std::string& s, size_t& p) {
    const auto at = [&s](size_t i) { return static_cast<uint32_t>(static_cast<uint8_t>(s[i])); };
    const uint32_t lead = at(p);
    int extra = 0;
    uint32_t cp = lead;
    if (lead >= 0xC0 && lead < 0xE0) { extra = 1; cp = lead & 0x1Fu; }
    else if (lead >= 0xE0 && lead < 0xF0) { extra = 2; cp = lead & 0x0Fu; }
    else if (lead >= 0xF0 && lead < 0xF8) { extra = 3; cp = lead & 0x07u; }
    if (extra == 0 || p + (size_t)extra >= s.size()) {
      p += 1;
      return lead;
    }
    for (int k = 1; k <= extra; k++) cp = (cp << 6) | (at(p + (size_t)k) & 0x3Fu);
    p += (size_t)extra + 1;
    return cp;
  }

  static void append_utf8(std::string& s, uint32_t cp) {
    if (cp < 0x80) {
      s.push_back(static_cast<char>(cp));
      return;
    }
    const int extra = cp < 0x800 ? 1 : cp < 0x10000 ? 2 : 3;
    static const uint8_t lead_bits[4] = {0, 0xC0, 0xE0, 0xF0};
    s.push_back(static_cast<char>(lead_bits[extra] | (cp >> (6 * extra))));
    for (int k = extra - 1; k >= 0; k--) s.push_back(static_cast<char>(0x80 | ((cp >> (6 * k)) & 0x3F)));
  }

  static bool newline(uint32_t c) { return c == '\r' || c == '\n'; }
  static bool other(uint32_t c) {   // [^\s\p{L}\p{N}]
    return !unicode::is_space(c) && !unicode::is_letter(c) && !unicode::is_number(c);
  }

  // End (exclusive, in code points) of the pre-token that starts at cps[i].
  static size_t pretoken_end(const std::vector<uint32_t>& cps, size_t i) {
    const size_t n = cps.size();
    const uint32_t c = cps[i];
    // 's 't 'm 'd 're 've 'll, ASCII case-insensitive
    if (c == '\'' && i + 1 < n) {
      const auto low = [](uint32_t x) { return x >= 'A' && x <= 'Z' ? x + 32 : x; };
      const uint32_t a = low(cps[i + 1]);
      if (a == 's' || a == 't' || a == 'm' || a == 'd') return i + 2;
      if (i + 2 < n) {
        const uint32_t b = low(cps[i + 2]);
        if ((a == 'r' && b == 'e') || (a == 'v' && b == 'e') || (a == 'l' && b == 'l')) return i + 3;
      }
    }
    // letters, with at most one leading character that is no letter, number, CR or LF
    {
      size_t j = n;
      if (unicode::is_letter(c)) j = i;
      else if (!newline(c) && !unicode::is_number(c) && i + 1 < n && unicode::is_letter(cps[i + 1])) j = i + 1;
      if (j < n) {
        while (j < n && unicode::is_letter(cps[j])) j++;
        return j;
      }
    }
    if (unicode::is_number(c)) return i + 1;   // digits one at a time
    // a run of other characters, optionally led by one space, with trailing CR / LF
    {
      size_t j = i;
      bool led = true;
      if (c == ' ') {
        led = i + 1 < n && other(cps[i + 1]);
        j = i + 1;
      }
      if (led && j < n && other(cps[j])) {
        while (j < n && other(cps[j])) j++;
        while (j < n && newline(cps[j])) j++;
        return j;
      }
    }
    // whitespace: up to its last CR / LF; else the whole run at the end of the text; else
    // all but its last character (which then leads the next pre-token); else that one character
    size_t w = i;
    while (w < n && unicode::is_space(cps[w])) w++;
    for (size_t k = w; k > i; k--)
      if (newline(cps[k - 1])) return k;
    if (w == n) return w;
    return w - i > 1 ? w - 1 : w;
  }

  // text[from, to): no control tokens inside
  void plain(const std::string& text, size_t from, size_t to, std::vector<int>& ids) const {
    if (to <= from) return;
    const std::string seg = text.substr(from, to - from);
    std::vector<uint32_t> cps;
    std::vector<size_t> starts;   // byte offset of each code point, plus the end
    for (size_t p = 0; p < seg.size();) {
      starts.push_back(p);
      cps.push_back(read_utf8(seg, p));
    }
    starts.push_back(seg.size());
    for (size_t i = 0; i < cps.size();) {
      const size_t e = pretoken_end(cps, i);
      merge(seg.data() + starts[i], starts[e] - starts[i], ids);
      i = e;
    }
  }

  // BPE over the bytes of one pre-token.
  void merge(const char* bytes, size_t n, std::vector<int>& ids) const {
    struct node { std::string text; int prev, next; bool alive; };
    std::vector<node> nodes(n);
    for (size_t k = 0; k < n; k++)
      nodes[k] = node{byte_piece_[static_cast<uint8_t>(bytes[k])], (int)k - 1, k + 1 < n ? (int)k + 1 : -1, true};
    // candidate = (rank, left node, lengths of both sides when pushed): stale entries are
    // recognised by the lengths having changed or a side having died
    struct cand { int rank, left; size_t llen, rlen; };
    const auto later = [](const cand& a, const cand& b) { return a.rank != b.rank ? a.rank > b.rank : a.left > b.left; };
    std::priority_queue<cand, std::vector<cand>, decltype(later)> heap(later);
    std::string key;
    const auto consider = [&](int left) {
      if (left < 0) return;
      const int right = nodes[(size_t)left].next;
      if (right < 0) return;
      key.assign(nodes[(size_t)left].text);
      key += ' ';
      key += nodes[(size_t)right].text;
      const auto it = rank_of_.find(key);
      if (it != rank_of_.end())
        heap.push(cand{it->second, left, nodes[(size_t)left].text.size(), nodes[(size_t)right].text.size()});
    };
    for (size_t k = 0; k + 1 < n; k++) consider((int)k);
    while (!heap.empty()) {
      const cand c = heap.top();
      heap.pop();
      node& l = nodes[(size_t)c.left];
      if (!l.alive || l.next < 0 || l.text.size() != c.llen) continue;
      node& r = nodes[(size_t)l.next];
      if (r.text.size() != c.rlen) continue;
      l.text += r.text;
      r.alive = false;
      l.next = r.next;
      if (r.next >= 0) nodes[(size_t)r.next].prev = c.left;
      consider(l.prev);
      consider(c.left);
    }
    for (int k = n ? 0 : -1; k >= 0; k = nodes[(size_t)k].next) {
      const auto it = id_of_.find(nodes[(size_t)k].text);
      if (it == id_of_.end()) throw std::runtime_error("tokenizer: symbol not in vocab: " + nodes[(size_t)k].text);
      ids.push_back(it->second);
    }
  }

  std::vector<std::string> pieces_;                        // id -> piece
  std::unordered_map<std::string, int> id_of_;
  std::unordered_map<std::string, int> rank_of_;           // "left right" -> merge rank
  std::vector<std::pair<std::string, int>> controls_;
  std::string byte_piece_[256];                            // byte -> its one-character piece
  std::unordered_map<uint32_t, uint8_t> byte_of_;
  int eos_ = -1, bos_ = -1;
};

}  // namespace tl
