// Greedy longest-match byte-trie tokenizer over the RWKV "world" vocabulary file format
// (lines `<id> <python string or bytes literal> <byte length>`), API as in the reference's
// include/rwkv_tokenizer.hpp.
#pragma once

#include <memory>
#include <string>
#include <string_view>
#include <vector>

namespace rwkv7_server {

inline constexpr int kTokenizerSuccess = 0;
inline constexpr int kTokenizerError = -1;

class TrieTokenizer {
 public:
  TrieTokenizer();
  ~TrieTokenizer();
  TrieTokenizer(const TrieTokenizer&) = delete;
  TrieTokenizer& operator=(const TrieTokenizer&) = delete;

  int load(const std::string& vocab_file);
  std::vector<int> encode(std::string_view text) const;
  std::string decode(const std::vector<int>& ids) const;
  std::string decode(int id) const;

 private:
  struct Impl;
  std::unique_ptr<Impl> impl_;
};

}  // namespace rwkv7_server
