// C handles over the C++ host interface; see llama_cu_c.h.
#include "llama_cu_c.h"

#include <cstring>
#include <memory>
#include <string>

#include "model_impl.hpp"

using namespace llama_cu;

struct lcu_model {
  std::unique_ptr<llama_model> model;
  llama_model_impl* impl() const { return static_cast<llama_model_impl*>(model.get()); }
};

struct lcu_context {
  std::unique_ptr<llama_context> context;
  llama_context_impl* impl() const { return static_cast<llama_context_impl*>(context.get()); }
};

struct lcu_batch {
  std::unique_ptr<llama_batch_context> context;
  int n_vocab;
};

namespace llama_cu {
int batch_context_read(llama_batch_context* ctx, bool probs, uint16_t* out);  // host/batch.cpp
}

struct lcu_vocab {
  mapped_buffer file;
  std::unique_ptr<llama_vocabulary> vocab;
};

namespace {
// uint32 count, count x {uint32 offset, float score}, NUL-terminated pieces at the offsets
bool vocab_file_is_sound(mapped_buffer const& f) {
  if (!f.is_ok() || f.size() < sizeof(uint32_t)) return false;
  const char* base = static_cast<const char*>(f.data());
  uint32_t count;
  memcpy(&count, base, sizeof(count));
  const size_t table_end = sizeof(uint32_t) + (size_t)count * 8;
  if (count > 32767 || table_end > f.size()) return false;
  if (count == 0) return true;
  if (base[f.size() - 1] != '\0') return false;  // every piece ends inside the file
  for (uint32_t i = 0; i < count; ++i) {
    uint32_t offset;
    memcpy(&offset, base + sizeof(uint32_t) + (size_t)i * 8, sizeof(offset));
    const bool by_text = i < 3 || i >= 259;  // ids 3..258 are bytes, their offsets are not read
    if (by_text && (offset < table_end || offset >= f.size())) return false;
  }
  return true;
}
}  // namespace

extern "C" {

lcu_model* lcu_model_create_synthetic(uint32_t dim, uint32_t multiple_of, uint32_t n_heads, uint32_t n_layers,
                                      uint32_t n_vocab, float norm_eps, int q_type, int quantization_block_size,
                                      uint64_t seed, float weight_std) {
  if (lcu_init(0) != 0) {
    fprintf(stderr, "lcu_model_create_synthetic: %s\n", lcu_last_error());
    return nullptr;
  }
  llama_params p{};
  p.magic = LLAMA_CU_MAGIC;
  p.fourcc = LLAMA_CU_MODEL_FOURCC_LLAMA;
  p.dim = dim;
  p.multiple_of = multiple_of;
  p.n_heads = n_heads;
  p.n_layers = n_layers;
  p.n_vocab = n_vocab;
  p.norm_eps = norm_eps;
  p.q_type = q_type == 1 ? quantization_type::uint8 : quantization_type::fp16;
  p.quantization_block_size = (uint16_t)(q_type == 1 ? quantization_block_size : 0);
  if (multiple_of == 0) {
    return nullptr;
  }
  auto m = llama_model::create_synthetic(p, seed, weight_std);
  if (!m) {
    return nullptr;
  }
  return new lcu_model{std::move(m)};
}

lcu_model* lcu_model_load(const char* model_dir, int context_len) {
  if (!model_dir || lcu_init(0) != 0) {
    return nullptr;
  }
  const std::string dir(model_dir);
  mapped_buffer params_buf(dir + "/params");
  llama_params p;
  if (!params_buf.is_ok() || !p.load(params_buf)) {
    fprintf(stderr, "Could not load params file\n");
    return nullptr;
  }
  llama_partition partition;
  partition.autopipe(p, (size_t)context_len);
  if (!partition.is_valid()) {
    fprintf(stderr, "Could not partition model\n");
    return nullptr;
  }
  auto m = llama_model::load(p, partition, dir);
  if (!m) {
    return nullptr;
  }
  return new lcu_model{std::move(m)};
}

void lcu_model_destroy(lcu_model* m) { delete m; }

uint32_t lcu_model_ffn_dim(const lcu_model* m) { return m->model->params.ffn_dim(); }

void lcu_model_describe(const lcu_model* m, uint32_t* dim, uint32_t* multiple_of, uint32_t* n_heads,
                        uint32_t* n_layers, uint32_t* n_vocab, float* norm_eps, int* q_type,
                        int* quantization_block_size) {
  llama_params const& p = m->model->params;
  if (dim) *dim = p.dim;
  if (multiple_of) *multiple_of = p.multiple_of;
  if (n_heads) *n_heads = p.n_heads;
  if (n_layers) *n_layers = p.n_layers;
  if (n_vocab) *n_vocab = p.n_vocab;
  if (norm_eps) *norm_eps = p.norm_eps;
  if (q_type) *q_type = p.q_type == quantization_type::uint8 ? 1 : 0;
  if (quantization_block_size) *quantization_block_size = p.quantization_block_size;
}

int lcu_model_read_tensor(const lcu_model* m, uint64_t stream_id, void* values, void* scales) {
  weight_tensor const* t = m->impl()->tensor_by_stream(stream_id);
  if (!t || !values) {
    return -1;
  }
  if (lcu_d2h(values, t->data.data(), t->data.size(), nullptr) != 0) return -2;
  if (t->quantised && scales) {
    if (lcu_d2h(scales, t->scales.data(), t->scales.size(), nullptr) != 0) return -2;
  }
  return 0;
}

int lcu_model_tensor_ptr(const lcu_model* m, uint64_t stream_id, void** values_dev, void** scales_dev) {
  weight_tensor const* t = m->impl()->tensor_by_stream(stream_id);
  if (!t || !values_dev) {
    return -1;
  }
  *values_dev = t->data.data();
  if (scales_dev) {
    *scales_dev = t->scales.data();
  }
  return 0;
}

void* lcu_model_norm_ptr(const lcu_model* m, int which) {
  llama_model_impl* mi = m->impl();
  if (which == -1) {
    return mi->norm.data();
  }
  if (which < 0 || (size_t)(which / 2) >= mi->layers.size()) {
    return nullptr;
  }
  llama_layer const& L = mi->layers[which / 2];
  return (which & 1) ? L.ffn_norm.data() : L.attn_norm.data();
}

lcu_context* lcu_context_create(lcu_model* m, int context_len, float temperature) {
  if (!m || context_len <= 0 || !(temperature > 0.0f)) {
    return nullptr;
  }
  auto ctx = llama_context::create(m->model.get(), context_len, temperature);
  if (!ctx) {
    return nullptr;  // context length beyond what the attention kernels cover
  }
  return new lcu_context{std::move(ctx)};
}

void lcu_context_destroy(lcu_context* c) { delete c; }
void lcu_context_clear_tokens(lcu_context* c) { c->context->clear_tokens(); }
size_t lcu_context_memory_usage(lcu_context* c) { return c->context->context_memory_usage(); }
size_t lcu_context_tokens_left(lcu_context* c) { return c->context->tokens_left(); }

int lcu_context_next_token(lcu_context* c, const int16_t* tokens, int n) {
  if (!c || !tokens || n <= 0 || (size_t)n > c->context->tokens_left()) {
    return -1;  // the reference asserts (llama_cu.cu:1074)
  }
  const int vocab = (int)c->impl()->model()->params.n_vocab;
  for (int i = 0; i < n; ++i) {
    if (tokens[i] < 0 || tokens[i] >= vocab) {
      return -1;
    }
  }
  std::vector<short> v(tokens, tokens + n);
  return c->context->next_token(v);
}

int lcu_context_read_logits(lcu_context* c, uint16_t* out) {
  auto* ci = c->impl();
  return lcu_d2h(out, ci->logits().data(), ci->logits().size(), ci->stream());
}

int lcu_context_read_probs(lcu_context* c, uint16_t* out) {
  auto* ci = c->impl();
  return lcu_d2h(out, ci->probs().data(), ci->probs().size(), ci->stream());
}

int lcu_context_read_hidden(lcu_context* c, uint16_t* out, int rows) {
  auto* ci = c->impl();
  if (rows <= 0 || rows > ci->last_n()) {
    return -1;
  }
  return lcu_d2h(out, ci->hidden().data(), (size_t)rows * ci->model()->params.dim * 2, ci->stream());
}

int lcu_context_read_kv(lcu_context* c, int layer, uint16_t* k_out, uint16_t* v_out, int T) {
  auto* ci = c->impl();
  if (layer < 0 || (size_t)layer >= ci->kv().size() || T <= 0 || T > ci->context_len()) {
    return -1;
  }
  const size_t bytes = (size_t)T * ci->model()->params.dim * 2;
  if (k_out && lcu_d2h(k_out, ci->kv()[layer].k.data(), bytes, ci->stream()) != 0) return -2;
  if (v_out && lcu_d2h(v_out, ci->kv()[layer].v.data(), bytes, ci->stream()) != 0) return -2;
  return 0;
}

void* lcu_context_stream(lcu_context* c) { return c->impl()->stream(); }

int lcu_context_hand_over_fallbacks(lcu_context* c) { return c->impl()->hand_over_fallbacks(); }

lcu_batch* lcu_batch_create(lcu_model* m, int n_sequences, int context_len, float temperature) {
  if (!m || n_sequences <= 0 || context_len <= 0 || !(temperature > 0.0f)) {
    return nullptr;
  }
  auto ctx = llama_batch_context::create(m->model.get(), n_sequences, context_len, temperature);
  if (!ctx) {
    return nullptr;
  }
  return new lcu_batch{std::move(ctx), (int)m->impl()->params.n_vocab};
}

void lcu_batch_destroy(lcu_batch* b) { delete b; }
int lcu_batch_n_sequences(lcu_batch* b) { return b->context->n_sequences(); }
size_t lcu_batch_memory_usage(lcu_batch* b) { return b->context->context_memory_usage(); }

static bool sequence_ok(lcu_batch* b, int sequence) { return b && sequence >= 0 && sequence < b->context->n_sequences(); }

int lcu_batch_clear_tokens(lcu_batch* b, int sequence) {
  if (!sequence_ok(b, sequence)) return -1;
  b->context->clear_tokens(sequence);
  return 0;
}

long lcu_batch_tokens_left(lcu_batch* b, int sequence) {
  return sequence_ok(b, sequence) ? (long)b->context->tokens_left(sequence) : -1;
}

int lcu_batch_next_token(lcu_batch* b, int sequence, const int16_t* tokens, int n) {
  if (!sequence_ok(b, sequence) || !tokens || n <= 0 || (size_t)n > b->context->tokens_left(sequence)) {
    return -1;
  }
  for (int i = 0; i < n; ++i) {
    if (tokens[i] < 0 || tokens[i] >= b->n_vocab) return -1;
  }
  return b->context->next_token(sequence, std::vector<short>(tokens, tokens + n));
}

int lcu_batch_next_tokens(lcu_batch* b, const int16_t* tokens, int16_t* out_tokens) {
  if (!b || !tokens || !out_tokens) return -1;
  const int n = b->context->n_sequences();
  for (int i = 0; i < n; ++i) {
    if (tokens[i] < 0 || tokens[i] >= b->n_vocab || b->context->tokens_left(i) < 1) return -1;
  }
  const std::vector<short> out = b->context->next_tokens(std::vector<short>(tokens, tokens + n));
  for (int i = 0; i < n; ++i) out_tokens[i] = out[i];
  return 0;
}

int lcu_batch_read_logits(lcu_batch* b, uint16_t* out) { return batch_context_read(b->context.get(), false, out); }
int lcu_batch_read_probs(lcu_batch* b, uint16_t* out) { return batch_context_read(b->context.get(), true, out); }

void lcu_context_set_sampling(lcu_context* c, int enabled, uint64_t seed) {
  if (enabled) {
    c->impl()->sample_with_seed(seed);
  } else {
    c->impl()->greedy();
  }
}

lcu_vocab* lcu_vocab_load(const char* vocab_path) {
  if (!vocab_path) return nullptr;
  mapped_buffer file{std::string(vocab_path)};
  if (!vocab_file_is_sound(file)) {
    fprintf(stderr, "Could not load vocab file\n");
    return nullptr;
  }
  auto* v = new lcu_vocab{std::move(file), nullptr};
  v->vocab = std::make_unique<llama_vocabulary>(v->file);
  return v;
}

void lcu_vocab_destroy(lcu_vocab* v) { delete v; }

int lcu_vocab_size(const lcu_vocab* v) { return v ? (int)v->vocab->tokens.size() : 0; }

int lcu_vocab_tokenize(lcu_vocab* v, const char* text, size_t text_len, int bos, int16_t* out, int capacity) {
  if (!v || (!text && text_len) || (!out && capacity > 0)) return -1;
  const std::vector<short> ids = v->vocab->tokenize(std::string_view(text ? text : "", text_len), bos != 0);
  for (int i = 0; i < capacity && i < (int)ids.size(); ++i) out[i] = ids[i];
  return (int)ids.size();
}

const char* lcu_vocab_piece(const lcu_vocab* v, int id, size_t* len) {
  if (!v || id < 0 || id >= (int)v->vocab->tokens.size()) {
    if (len) *len = 0;
    return nullptr;
  }
  if (len) *len = v->vocab->tokens[id].text.size();
  return v->vocab->tokens[id].text.data();
}

float lcu_vocab_score(const lcu_vocab* v, int id) {
  if (!v || id < 0 || id >= (int)v->vocab->tokens.size()) return 0.0f;
  return v->vocab->tokens[id].score;
}

}  // extern "C"
