// Vocabulary file reader and the greedy highest-score pair-merging tokenizer:
// behaviour of llama_cu.cu:1312-1437.
#include <algorithm>

#include "host_common.hpp"

namespace llama_cu {

namespace {
// bytes in a UTF-8 sequence from the high nibble of its first byte
size_t utf8_length(char first) {
  static const uint8_t len[16] = {1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 2, 3, 4};
  return len[static_cast<uint8_t>(first) >> 4];
}
}  // namespace

// File layout: uint32 count, then count x {uint32 offset, float score}; offsets (from the start
// of the file) point at NUL-terminated piece texts.  Ids 3..258 are the raw bytes 0..255 whatever
// the file says; only ids >= 259 can be found by text.
llama_vocabulary::llama_vocabulary(mapped_buffer const& buffer) {
  struct record {
    uint32_t offset;
    float score;
  };
  const char* base = static_cast<const char*>(buffer.data());
  const uint32_t count = *reinterpret_cast<const uint32_t*>(base);
  const record* records = reinterpret_cast<const record*>(base + sizeof(uint32_t));
  tokens.reserve(count);
  for (uint32_t i = 0; i < count; ++i) {
    llama_token t;
    t.id = (short)i;
    t.score = records[i].score;
    if (i >= 3 && i < 259) {
      t.text = std::string(1, (char)(i - 3));
    } else {
      t.text = std::string(base + records[i].offset);
    }
    tokens.push_back(std::move(t));
  }
  for (uint32_t i = 259; i < count; ++i) {
    token_lookup.emplace(tokens[i].text, &tokens[i]);  // the first id wins for a repeated text
  }
}

std::vector<short> llama_vocabulary::tokenize(std::string_view text, bool bos) {
  std::vector<short> out;
  if (bos) {
    out.push_back(1);
  }
  if (text.empty()) {
    return out;
  }
  llama_tokenizer tk(*this);
  if (text[0] != ' ') {
    std::string spaced;
    spaced.reserve(text.size() + 1);
    spaced.push_back(' ');
    spaced.append(text);
    tk.tokenize(spaced, out);  // pieces are views into `spaced`, which outlives the call
  } else {
    tk.tokenize(text, out);
  }
  return out;
}

void llama_tokenizer::consider(int left, int right) {
  if (left < 0 || right < 0) {
    return;
  }
  const std::string_view joined(pieces_[left].text.data(), pieces_[left].text.size() + pieces_[right].text.size());
  auto it = vocab_.token_lookup.find(std::string(joined));
  if (it == vocab_.token_lookup.end()) {
    return;
  }
  queue_.push(candidate{left, right, it->second->score, joined.size()});
}

void llama_tokenizer::tokenize(std::string_view text, std::vector<short>& output) {
  // one piece per UTF-8 character, doubly linked by index
  while (!text.empty()) {
    const size_t len = std::min(text.size(), utf8_length(text[0]));
    const int index = (int)pieces_.size();
    piece p;
    p.text = text.substr(0, len);
    p.prev = index - 1;
    text.remove_prefix(len);
    p.next = text.empty() ? -1 : index + 1;
    pieces_.push_back(p);
  }
  for (size_t i = 1; i < pieces_.size(); ++i) {
    consider((int)i - 1, (int)i);
  }
  // merge the best-scoring adjacent pair (leftmost on ties) until no known pair is left
  while (!queue_.empty()) {
    const candidate best = queue_.top();
    queue_.pop();
    piece& l = pieces_[best.left];
    piece& r = pieces_[best.right];
    if (l.text.empty() || r.text.empty() || l.text.size() + r.text.size() != best.size) {
      continue;  // one side was merged away since this candidate was queued
    }
    l.text = std::string_view(l.text.data(), l.text.size() + r.text.size());
    r.text = std::string_view();
    l.next = r.next;
    if (r.next >= 0) {
      pieces_[r.next].prev = best.left;
    }
    consider(l.prev, best.left);
    consider(best.left, l.next);
  }
  if (pieces_.empty()) {
    return;
  }
  for (int i = 0; i != -1; i = pieces_[i].next) {
    const piece& p = pieces_[i];
    auto it = vocab_.token_lookup.find(std::string(p.text));
    if (it != vocab_.token_lookup.end()) {
      output.push_back(it->second->id);
    } else {
      for (unsigned char byte : p.text) {
        output.push_back((short)(byte + 3));  // unknown text falls back to byte tokens
      }
    }
  }
}

}  // namespace llama_cu
