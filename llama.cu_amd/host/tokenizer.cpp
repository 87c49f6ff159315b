// Vocabulary file reader and tokenizer.  Contract (llama_cu.cu:1312-1437): the text is cut into
// UTF-8 characters; the adjacent pair whose concatenation is the best-scoring vocabulary piece is
// merged (the leftmost such pair on equal scores), again and again until no adjacent pair is a
// piece; what is left is looked up, and text that is no piece goes out byte by byte as ids 3..258.
//
// Own structure: segments live in parallel arrays addressed by index into the text, every segment
// carries a version number, and the pending merges sit in a binary heap kept with the standard heap
// algorithms; a pending merge is valid exactly when both versions it recorded are still current.
#include <algorithm>
#include <cstring>

#include "host_common.hpp"

namespace llama_cu {

namespace {

constexpr short BOS_ID = 1;
constexpr uint32_t FIRST_BYTE_ID = 3;   // ids 3..258 stand for the bytes 0..255
constexpr uint32_t FIRST_TEXT_ID = 259;  // only ids from here on are found by their text

// length of the UTF-8 sequence that a byte opens: the run of leading one bits for lead bytes
// (0xC0 and up, capped at four), one for ASCII and for stray continuation bytes
uint32_t sequence_bytes(unsigned char lead) {
  if (lead < 0xC0) {
    return 1;
  }
  const uint32_t ones = (uint32_t)__builtin_clz(~((uint32_t)lead << 24));
  return ones > 4 ? 4 : ones;
}

// heap order: the better merge compares greater (higher score; on equal scores the one further left)
bool merges_before(float score_a, int left_a, float score_b, int left_b) {
  return score_a != score_b ? score_a < score_b : left_a > left_b;
}

}  // namespace

// File layout: uint32 count, then count records {uint32 offset, float score}; an offset counts
// from the start of the file to a NUL-terminated piece.
llama_vocabulary::llama_vocabulary(mapped_buffer const& buffer) {
  const unsigned char* file = static_cast<const unsigned char*>(buffer.data());
  uint32_t count = 0;
  memcpy(&count, file, sizeof(count));
  tokens.resize(count);
  const unsigned char* record = file + sizeof(count);
  for (uint32_t id = 0; id < count; ++id, record += 8) {
    uint32_t offset = 0;
    llama_token& t = tokens[id];
    memcpy(&offset, record, 4);
    memcpy(&t.score, record + 4, 4);
    t.id = (short)id;
    if (id >= FIRST_BYTE_ID && id < FIRST_TEXT_ID) {
      t.text.assign(1, (char)(id - FIRST_BYTE_ID));  // whatever the file says
    } else {
      t.text.assign(reinterpret_cast<const char*>(file + offset));
    }
  }
  // `tokens` never grows again, so the pointers stay good; emplace keeps the first id of a repeated text
  for (uint32_t id = FIRST_TEXT_ID; id < count; ++id) {
    token_lookup.emplace(tokens[id].text, &tokens[id]);
  }
}

std::vector<short> llama_vocabulary::tokenize(std::string_view text, bool bos) {
  std::vector<short> ids;
  if (bos) {
    ids.push_back(BOS_ID);
  }
  if (text.empty()) {
    return ids;
  }
  // the text is tokenized as if it began with a space
  std::string padded;
  if (text.front() != ' ') {
    padded.reserve(text.size() + 1);
    padded += ' ';
    padded += text;
    text = padded;
  }
  llama_tokenizer(*this).tokenize(text, ids);
  return ids;
}

// id of the piece spelled by bytes [begin, begin + bytes) of the text, or -1
short llama_tokenizer::find_piece(size_t begin, size_t bytes, float* score) {
  key_.assign(text_.data() + begin, bytes);
  auto hit = vocab_.token_lookup.find(key_);
  if (hit == vocab_.token_lookup.end()) {
    return -1;
  }
  if (score) {
    *score = hit->second->score;
  }
  return hit->second->id;
}

void llama_tokenizer::queue_merge(int left, int right) {
  if (left < 0 || right < 0) {
    return;
  }
  float score = 0.0f;
  if (find_piece(begin_[left], (size_t)bytes_[left] + bytes_[right], &score) < 0) {
    return;
  }
  heap_.push_back(merge{score, left, right, version_[left], version_[right]});
  std::push_heap(heap_.begin(), heap_.end(), [](merge const& a, merge const& b) {
    return merges_before(a.score, a.left, b.score, b.left);
  });
}

void llama_tokenizer::tokenize(std::string_view text, std::vector<short>& output) {
  text_ = text;
  begin_.clear();
  bytes_.clear();
  heap_.clear();
  for (size_t at = 0; at < text.size();) {
    const size_t n = std::min<size_t>(sequence_bytes((unsigned char)text[at]), text.size() - at);
    begin_.push_back((uint32_t)at);
    bytes_.push_back((uint32_t)n);
    at += n;
  }
  const int count = (int)begin_.size();
  if (count == 0) {
    return;
  }
  version_.assign(count, 0);
  left_of_.resize(count);
  right_of_.resize(count);
  for (int i = 0; i < count; ++i) {
    left_of_[i] = i - 1;
    right_of_[i] = i + 1 < count ? i + 1 : -1;
  }
  for (int i = 0; i + 1 < count; ++i) {
    queue_merge(i, i + 1);
  }
  auto order = [](merge const& a, merge const& b) { return merges_before(a.score, a.left, b.score, b.left); };
  while (!heap_.empty()) {
    std::pop_heap(heap_.begin(), heap_.end(), order);
    const merge m = heap_.back();
    heap_.pop_back();
    if (version_[m.left] != m.left_version || version_[m.right] != m.right_version) {
      continue;  // a side has grown or gone since this merge was queued
    }
    // the left segment swallows the right one
    bytes_[m.left] += bytes_[m.right];
    bytes_[m.right] = 0;
    ++version_[m.left];
    ++version_[m.right];
    const int after = right_of_[m.right];
    right_of_[m.left] = after;
    if (after >= 0) {
      left_of_[after] = m.left;
    }
    queue_merge(left_of_[m.left], m.left);
    queue_merge(m.left, after);
  }
  for (int i = 0; i >= 0; i = right_of_[i]) {
    const short id = find_piece(begin_[i], bytes_[i], nullptr);
    if (id >= 0) {
      output.push_back(id);
      continue;
    }
    for (uint32_t b = 0; b < bytes_[i]; ++b) {
      output.push_back((short)((unsigned char)text[begin_[i] + b] + FIRST_BYTE_ID));
    }
  }
}

}  // namespace llama_cu
