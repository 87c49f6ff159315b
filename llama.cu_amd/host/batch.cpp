// llama_batch_context: several sequences decoded together (no counterpart in the reference, whose
// README lists batching as a TODO).  The step is next_token's layer loop (llama_cu.cu:1073-1210)
// with one row per sequence: the matrix products take the rows as M and read every weight once
// for the whole batch; rotary, cache append and attention work per sequence on that sequence's own
// position and caches, which are the caches of an ordinary llama_context per sequence.
#include <cassert>
#include <cstring>

#include "model_impl.hpp"

namespace llama_cu {

namespace {

struct llama_batch_context_impl final : public llama_batch_context {
  llama_batch_context_impl(llama_model* model, int n_sequences, int context_len, float temperature)
      : model_(static_cast<llama_model_impl*>(model)), context_len_(context_len), temperature_(temperature) {
    LCU_CHECK(lcu_init(0));
    device_structure_lock lock(device_structure_mutex());
    LCU_CHECK(lcu_stream_create(&stream_));
    for (int b = 0; b < n_sequences; ++b) {
      seqs_.push_back(std::make_unique<llama_context_impl>(model, context_len, temperature));
    }
    llama_params const& p = model_->params;
    const size_t B = (size_t)n_sequences, dim = p.dim, ffn = p.ffn_dim(), vocab = p.n_vocab;
    t_x_ = gpu_buffer(B * dim * 2);
    t_norm_ = gpu_buffer(B * dim * 2);
    t_q_ = gpu_buffer(B * dim * 2);
    t_k_ = gpu_buffer(B * dim * 2);
    t_v_ = gpu_buffer(B * dim * 2);
    t_out_ = gpu_buffer(B * dim * 2);
    t_w1_ = gpu_buffer(B * ffn * 2);
    t_w3_ = gpu_buffer(B * ffn * 2);
    t_silu_ = gpu_buffer(B * ffn * 2);
    t_logits_ = gpu_buffer(B * vocab * 2);
    t_probs_ = gpu_buffer(B * vocab * 2);
    t_argmax_ = gpu_buffer(B * sizeof(int));
    t_step_ = gpu_buffer(B * (sizeof(int32_t) + sizeof(int16_t)));  // positions, then tokens
    t_cache_ptrs_ = gpu_buffer((size_t)p.n_layers * 2 * B * sizeof(void*));
    upload_cache_pointers();
  }

  ~llama_batch_context_impl() override {
    lcu_sync(stream_);
    device_structure_lock lock(device_structure_mutex());
    lcu_graph_destroy(graph_);
    lcu_stream_destroy(stream_);
  }

  int n_sequences() override { return (int)seqs_.size(); }

  void clear_tokens(int sequence) override {
    LCU_CHECK(lcu_sync(stream_));
    seqs_[sequence]->clear_tokens();  // fresh caches: other addresses
    upload_cache_pointers();
    drop_graph();
  }

  size_t tokens_left(int sequence) override { return seqs_[sequence]->tokens_left(); }

  size_t context_memory_usage() override {
    size_t count = 0;
    for (auto& s : seqs_) {
      count += s->context_memory_usage();
    }
    for (gpu_buffer const* b : {&t_x_, &t_norm_, &t_q_, &t_k_, &t_v_, &t_out_, &t_w1_, &t_w3_, &t_silu_, &t_logits_,
                                &t_probs_, &t_argmax_, &t_step_, &t_cache_ptrs_}) {
      count += b->size();
    }
    return count;
  }

  short next_token(int sequence, std::vector<short> const& new_tokens) override {
    LCU_CHECK(lcu_sync(stream_));
    return seqs_[sequence]->next_token(new_tokens);
  }

  std::vector<short> next_tokens(std::vector<short> const& tokens) override {
    const int B = (int)seqs_.size();
    assert((int)tokens.size() == B);
    // positions and tokens go up in one copy; every kernel of the step reads them on the device,
    // so the step is captured once (on its second run) and replayed afterwards
    std::vector<char> host((size_t)B * 6);
    int max_T = 0;
    for (int b = 0; b < B; ++b) {
      assert(seqs_[b]->tokens_left() >= 1);
      const int32_t pos = seqs_[b]->start_pos();
      memcpy(host.data() + (size_t)b * 4, &pos, 4);
      memcpy(host.data() + (size_t)B * 4 + (size_t)b * 2, &tokens[b], 2);
      max_T = pos + 1 > max_T ? pos + 1 : max_T;
    }
    LCU_CHECK(lcu_h2d(t_step_.data(), host.data(), host.size(), stream_));
    // the attention kernel is given a bound on the rows it may see; a graph is good while the
    // bound holds (bounds: 1024, then the context length)
    const int bound = (max_T <= 1024 && context_len_ > 1024) ? 1024 : context_len_;
    if (graph_ && bound != graph_bound_) {
      drop_graph();
    }
    graph_bound_ = bound;
    ++calls_;
    {
      device_structure_lock lock(device_structure_mutex());  // capture, instantiation, launch: see host_common.hpp
      if (!graph_ && calls_ >= 2) {
        LCU_CHECK(lcu_graph_begin_capture(stream_));
        enqueue_step(bound);
        LCU_CHECK(lcu_graph_end_capture(stream_, &graph_));
      }
      if (graph_) {
        LCU_CHECK(lcu_graph_launch(graph_, stream_));
      } else {
        enqueue_step(bound);
      }
    }
    std::vector<int> idx(B);
    LCU_CHECK(lcu_d2h(idx.data(), t_argmax_.data(), (size_t)B * sizeof(int), stream_));  // blocks
    std::vector<short> out(B);
    for (int b = 0; b < B; ++b) {
      seqs_[b]->advance_one();
      out[b] = (short)idx[b];
    }
    return out;
  }

  // read-back for tests
  gpu_buffer& logits() { return t_logits_; }
  gpu_buffer& probs() { return t_probs_; }
  void* stream() const { return stream_; }
  llama_model_impl* model() const { return model_; }

 private:
  void drop_graph() {
    if (graph_) {
      device_structure_lock lock(device_structure_mutex());
      LCU_CHECK(lcu_graph_destroy(graph_));
      graph_ = nullptr;
    }
    calls_ = 0;
  }

  // device table [layer][k or v][sequence] of cache base pointers
  void upload_cache_pointers() {
    const size_t B = seqs_.size(), L = model_->layers.size();
    std::vector<void*> table(L * 2 * B);
    for (size_t l = 0; l < L; ++l) {
      for (size_t b = 0; b < B; ++b) {
        table[(l * 2 + 0) * B + b] = seqs_[b]->kv()[l].k.data();
        table[(l * 2 + 1) * B + b] = seqs_[b]->kv()[l].v.data();
      }
    }
    LCU_CHECK(lcu_h2d(t_cache_ptrs_.data(), table.data(), table.size() * sizeof(void*), stream_));
    LCU_CHECK(lcu_sync(stream_));
  }

  void matmul(void* out, const void* lhs, weight_tensor const& w, int M, float beta) {
    if (w.quantised) {
      LCU_CHECK(lcu_gemm_f16u8_nt(out, lhs, w.data.data(), w.scales.data(), M, (int)w.cols, (int)w.rows, w.block, beta,
                                  stream_));
    } else {
      LCU_CHECK(lcu_gemm_f16_nt(out, lhs, w.data.data(), M, (int)w.cols, (int)w.rows, beta, stream_));
    }
  }

  void enqueue_step(int bound) {
    llama_params const& p = model_->params;
    const int B = (int)seqs_.size(), dim = p.dim, ffn = p.ffn_dim(), heads = p.n_heads, vocab = p.n_vocab;
    const int block = p.q_type == quantization_type::uint8 ? p.quantization_block_size : 0;
    const void* pos = t_step_.data();
    const void* ids = (char*)t_step_.data() + (size_t)B * 4;
    void* x = t_x_.data();
    if (model_->tok_embeddings.quantised) {  // llama_cu.cu:1087-1097
      LCU_CHECK(lcu_embed_u8(x, ids, B, dim, model_->tok_embeddings.data.data(), model_->tok_embeddings.scales.data(),
                             block, vocab, stream_));
    } else {
      LCU_CHECK(lcu_embed(x, ids, B, dim, model_->tok_embeddings.data.data(), vocab, stream_));
    }
    // Every product is fused with what follows it (lcu_batch_*): rotary + cache append after
    // Wq/Wk/Wv, SiLU after W1/W3, the residual sum and the NEXT norm after Wo and W2 -- so the
    // first norm stands alone and the last W2 carries the final norm.
    LCU_CHECK(lcu_rmsnorm(t_norm_.data(), x, model_->layers[0].attn_norm.data(), B, dim, p.norm_eps, stream_));  // 1129
    const size_t n_layers = model_->layers.size();
    for (size_t l = 0; l < n_layers; ++l) {
      llama_layer const& L = model_->layers[l];
      const char* kp = (char*)t_cache_ptrs_.data() + (l * 2 + 0) * B * sizeof(void*);
      const char* vp = (char*)t_cache_ptrs_.data() + (l * 2 + 1) * B * sizeof(void*);
      const void* const qkv_w[3] = {L.wq.data.data(), L.wk.data.data(), L.wv.data.data()};
      const void* const qkv_s[3] = {L.wq.scales.data(), L.wk.scales.data(), L.wv.scales.data()};
      LCU_CHECK(lcu_batch_qkv(t_q_.data(), t_k_.data(), t_v_.data(), t_norm_.data(), qkv_w, qkv_s, block, B, dim, heads,
                              kp, vp, pos, seqs_[0]->rope_table(), context_len_, stream_));                // 1144-1156
      LCU_CHECK(lcu_attention_decode_batch(t_out_.data(), t_q_.data(), kp, vp, pos, B, bound, dim, heads,
                                           stream_));                                                      // 1161-1171
      LCU_CHECK(lcu_batch_proj_norm(x, t_norm_.data(), t_out_.data(), L.wo.data.data(), L.wo.scales.data(), block, B,
                                    dim, dim, L.ffn_norm.data(), p.norm_eps, stream_));                    // 1174, 1176
      const void* const up_w[2] = {L.w1.data.data(), L.w3.data.data()};
      const void* const up_s[2] = {L.w1.scales.data(), L.w3.scales.data()};
      LCU_CHECK(lcu_batch_ffn_up(t_silu_.data(), t_w1_.data(), t_w3_.data(), t_norm_.data(), up_w, up_s, block, B, dim,
                                 ffn, stream_));                                                           // 1180-1183
      const void* next_norm = l + 1 < n_layers ? model_->layers[l + 1].attn_norm.data() : model_->norm.data();
      LCU_CHECK(lcu_batch_proj_norm(x, t_norm_.data(), t_silu_.data(), L.w2.data.data(), L.w2.scales.data(), block, B,
                                    ffn, dim, next_norm, p.norm_eps, stream_));                            // 1185, 1129 / 1191
    }
    // 1191-1209 for every row (the final norm is already in t_norm_)
    matmul(t_logits_.data(), t_norm_.data(), model_->output, B, 0.0f);
    LCU_CHECK(lcu_softmax_argmax_rows(t_probs_.data(), t_argmax_.data(), t_logits_.data(), B, vocab, temperature_,
                                      stream_));
  }

  llama_model_impl* model_;
  int context_len_;
  float temperature_;
  std::vector<std::unique_ptr<llama_context_impl>> seqs_;
  gpu_buffer t_x_, t_norm_, t_q_, t_k_, t_v_, t_out_, t_w1_, t_w3_, t_silu_, t_logits_, t_probs_, t_argmax_;
  gpu_buffer t_step_;        // int32 positions [B], then int16 tokens [B]
  gpu_buffer t_cache_ptrs_;  // see upload_cache_pointers
  void* stream_{nullptr};
  void* graph_{nullptr};
  int graph_bound_{0};
  int calls_{0};
};

}  // namespace

/* static */ std::unique_ptr<llama_batch_context> llama_batch_context::create(llama_model* model, int n_sequences,
                                                                              int context_len, float temperature) {
  if (model == nullptr || n_sequences < 1 || context_len < 1 || context_len > LLAMA_CU_MAX_CONTEXT) {
    fprintf(stderr, "unsupported batch: %d sequences, context length %d (1..%d)\n", n_sequences, context_len,
            LLAMA_CU_MAX_CONTEXT);
    return nullptr;
  }
  return std::make_unique<llama_batch_context_impl>(model, n_sequences, context_len, temperature);
}

// read-back for the C handles (tests): fp16 logits / probabilities [n_sequences][n_vocab] of the last step
int batch_context_read(llama_batch_context* ctx, bool probs, uint16_t* out) {
  auto* c = static_cast<llama_batch_context_impl*>(ctx);
  gpu_buffer& src = probs ? c->probs() : c->logits();
  return lcu_d2h(out, src.data(), src.size(), c->stream());
}

}  // namespace llama_cu
