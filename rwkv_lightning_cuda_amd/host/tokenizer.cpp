// Greedy longest-match byte-trie tokenizer (reference behaviour: src/utils/trie.h + src/utils/tokenizer.cpp,
// wrapped by src/rwkv_tokenizer.cpp).  Vocabulary lines are `<id> <literal> <byte length>` where the literal
// is a Python str ('...' / "...") or bytes (b'...') literal; str literals are stored as their UTF-8 bytes.
#include "rwkv_tokenizer.hpp"

#include <cstdint>
#include <fstream>
#include <unordered_map>

namespace rwkv7_server {
namespace {

void append_utf8(std::string& out, std::uint32_t cp) {
  if (cp < 0x80) {
    out += static_cast<char>(cp);
  } else if (cp < 0x800) {
    out += static_cast<char>(0xC0 | (cp >> 6));
    out += static_cast<char>(0x80 | (cp & 0x3F));
  } else if (cp < 0x10000) {
    out += static_cast<char>(0xE0 | (cp >> 12));
    out += static_cast<char>(0x80 | ((cp >> 6) & 0x3F));
    out += static_cast<char>(0x80 | (cp & 0x3F));
  } else {
    out += static_cast<char>(0xF0 | (cp >> 18));
    out += static_cast<char>(0x80 | ((cp >> 12) & 0x3F));
    out += static_cast<char>(0x80 | ((cp >> 6) & 0x3F));
    out += static_cast<char>(0x80 | (cp & 0x3F));
  }
}

int hex_value(char c) {
  if (c >= '0' && c <= '9') return c - '0';
  if (c >= 'a' && c <= 'f') return c - 'a' + 10;
  if (c >= 'A' && c <= 'F') return c - 'A' + 10;
  return -1;
}

// Decodes a Python literal body (between the quotes).  In a bytes literal \xNN is one byte; in a str literal
// \xNN, \uNNNN and \UNNNNNNNN are code points encoded as UTF-8.
bool parse_literal(const std::string& lit, std::string& out) {
  size_t i = 0;
  bool is_bytes = false;
  if (i < lit.size() && lit[i] == 'b') {
    is_bytes = true;
    ++i;
  }
  if (i >= lit.size() || (lit[i] != '\'' && lit[i] != '"')) return false;
  const char quote = lit[i++];
  if (lit.size() < i + 1 || lit.back() != quote) return false;
  const size_t end = lit.size() - 1;
  out.clear();
  while (i < end) {
    const char c = lit[i++];
    if (c != '\\') {
      out += c;
      continue;
    }
    if (i >= end) return false;
    const char e = lit[i++];
    switch (e) {
      case 'n': out += '\n'; break;
      case 't': out += '\t'; break;
      case 'r': out += '\r'; break;
      case '\\': out += '\\'; break;
      case '\'': out += '\''; break;
      case '"': out += '"'; break;
      case 'a': out += '\a'; break;
      case 'b': out += '\b'; break;
      case 'f': out += '\f'; break;
      case 'v': out += '\v'; break;
      case '0': out += '\0'; break;
      case 'x':
      case 'u':
      case 'U': {
        const int digits = e == 'x' ? 2 : (e == 'u' ? 4 : 8);
        if (i + digits > end) return false;
        std::uint32_t value = 0;
        for (int d = 0; d < digits; ++d) {
          const int h = hex_value(lit[i++]);
          if (h < 0) return false;
          value = value * 16 + static_cast<std::uint32_t>(h);
        }
        if (is_bytes) {
          out += static_cast<char>(value);
        } else {
          append_utf8(out, value);
        }
        break;
      }
      default: return false;
    }
  }
  return true;
}

struct Node {
  int token = -1;
  int next[256];
  Node() {
    for (int& n : next) n = -1;
  }
};

}  // namespace

struct TrieTokenizer::Impl {
  std::vector<Node> nodes;
  std::unordered_map<int, std::string> id_to_bytes;

  void insert(const std::string& bytes, int id) {
    int cur = 0;
    for (unsigned char b : bytes) {
      if (nodes[cur].next[b] < 0) {
        nodes[cur].next[b] = static_cast<int>(nodes.size());
        nodes.emplace_back();
      }
      cur = nodes[cur].next[b];
    }
    nodes[cur].token = id;
  }
};

TrieTokenizer::TrieTokenizer() : impl_(std::make_unique<Impl>()) {}
TrieTokenizer::~TrieTokenizer() = default;

int TrieTokenizer::load(const std::string& vocab_file) {
  std::ifstream in(vocab_file, std::ios::binary);
  if (!in) return kTokenizerError;
  impl_->nodes.clear();
  impl_->nodes.emplace_back();
  impl_->id_to_bytes.clear();
  std::string line;
  while (std::getline(in, line)) {
    if (!line.empty() && line.back() == '\r') line.pop_back();
    if (line.empty()) continue;
    const size_t first = line.find(' ');
    const size_t last = line.rfind(' ');
    if (first == std::string::npos || last == first) return kTokenizerError;
    int id = 0, length = 0;
    try {
      id = std::stoi(line.substr(0, first));
      length = std::stoi(line.substr(last + 1));
    } catch (...) {
      return kTokenizerError;
    }
    std::string bytes;
    if (!parse_literal(line.substr(first + 1, last - first - 1), bytes)) return kTokenizerError;
    if (static_cast<int>(bytes.size()) != length) return kTokenizerError;
    impl_->insert(bytes, id);
    impl_->id_to_bytes[id] = bytes;
  }
  return impl_->id_to_bytes.empty() ? kTokenizerError : kTokenizerSuccess;
}

std::vector<int> TrieTokenizer::encode(std::string_view text) const {
  std::vector<int> ids;
  size_t pos = 0;
  while (pos < text.size()) {
    int cur = 0, best = -1;
    size_t best_len = 0;
    for (size_t i = pos; i < text.size(); ++i) {
      cur = impl_->nodes[cur].next[static_cast<unsigned char>(text[i])];
      if (cur < 0) break;
      if (impl_->nodes[cur].token >= 0) {
        best = impl_->nodes[cur].token;
        best_len = i - pos + 1;
      }
    }
    if (best < 0) {  // a byte that no token covers: skip it
      ++pos;
      continue;
    }
    ids.push_back(best);
    pos += best_len;
  }
  return ids;
}

std::string TrieTokenizer::decode(int id) const {
  auto it = impl_->id_to_bytes.find(id);
  return it == impl_->id_to_bytes.end() ? std::string() : it->second;
}

std::string TrieTokenizer::decode(const std::vector<int>& ids) const {
  std::string out;
  for (int id : ids) out += decode(id);
  return out;
}

}  // namespace rwkv7_server
