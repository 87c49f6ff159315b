// C handles over the C++ host interface; see llama_cu_c.h.
#include "llama_cu_c.h"

#include <memory>

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
  return new lcu_context{llama_context::create(m->model.get(), context_len, temperature)};
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

}  // extern "C"
