// Implementation types behind llama_model / llama_context (the reference keeps its counterparts,
// llama_layer / llama_model_impl / llama_context_impl, private to llama_cu.cu:882-1304).
#pragma once
#include <string>
#include <vector>

#include "host_common.hpp"

namespace llama_cu {

// limit of the attention kernels (csrc/attention.hip): cache rows a call can attend to, whether it
// brings one new token or many
constexpr int LLAMA_CU_MAX_CONTEXT = 4096;


// one weight matrix [rows, cols]: fp16 values, or uint8 codes with fp16 scales [rows, cols/block]
// (the reference's generic_tensor, llama_cu.h:252-270)
struct weight_tensor {
  gpu_buffer data;
  gpu_buffer scales;
  size_t rows{0}, cols{0};
  bool quantised{false};
  int block{0};
};

struct llama_layer {
  weight_tensor wq, wk, wv, wo;
  weight_tensor w1, w2, w3;
  gpu_buffer attn_norm, ffn_norm;
};

struct llama_model_impl : public llama_model {
  llama_model_impl(llama_params params, llama_partition partition) : llama_model(params, partition) {}
  bool load_impl(std::string const& path);
  void synthesize(uint64_t seed, float weight_std);
  weight_tensor const* tensor_by_stream(uint64_t stream_id) const;
  weight_tensor tok_embeddings;
  weight_tensor output;
  gpu_buffer norm;
  std::vector<llama_layer> layers;
};

struct llama_context_impl final : public llama_context {
  llama_context_impl(llama_model* model, int context_len, float temperature);
  ~llama_context_impl() override;
  void clear_tokens() override;
  size_t context_memory_usage() override;
  short next_token(std::vector<short> const& new_tokens) override;
  void sample_with_seed(uint64_t seed) override;
  void greedy() override;

  // read-back used by tests and tools
  llama_model_impl* model() const { return model_; }
  int context_len() const { return context_len_; }
  int start_pos() const { return start_pos_; }
  int last_n() const { return last_n_; }
  void* stream() const { return stream_; }
  gpu_buffer& hidden() { return t_embed_; }
  gpu_buffer& logits() { return t_logits_; }
  gpu_buffer& probs() { return t_probs_; }
  struct kv_cache_layer {
    gpu_buffer k;  // [context_len][dim], rotated
    gpu_buffer v;
  };
  std::vector<kv_cache_layer>& kv() { return kv_; }
  void* rope_table() const { return rope_table_; }
  float temperature() const { return temperature_; }
  // decode steps that were computed a second time because hand-overs inside a launch did not arrive
  int hand_over_fallbacks() const { return hand_over_fallbacks_; }
  // a step taken for this sequence by llama_batch_context: one more cached row
  void advance_one() {
    start_pos_ += 1;
    last_n_ = 1;
  }

 private:
  void matmul(void* out, const void* lhs, weight_tensor const& w, int M, float beta);
  void matmul_multi(void* const* outs, const void* lhs, weight_tensor const* const* ws, int count, int M);
  void enqueue_layers(int n, bool first_norm_ready = false);
  void enqueue_head(int n);
  void drop_graph();
  std::vector<kv_cache_layer> kv_;
  gpu_buffer t_embed_, t_norm_, t_xq_, t_out_, t_w1_, t_w3_, t_silu_;
  gpu_buffer t_tokens_, t_logits_, t_probs_, t_argmax_;
  // step state on the device: {int32 position, int16 token, 64 random bits, uint32 step counter};
  // the decode kernels and the sampler read it from here, so one captured graph replays for every
  // step (the counter differs from step to step: the epoch of the attention kernel's hand-over)
  gpu_buffer t_step_;
  struct step_state {
    int32_t pos;
    int16_t token;
    int16_t pad;
    uint64_t random;  // this step's 64 random bits when sampling
    uint32_t seq;     // counts the one-token steps of this context
    uint32_t pad2;
  } host_step_{};
  bool sampling_{false};
  uint64_t sample_seed_{0};
  uint64_t samples_drawn_{0};
  void* decode_graph_{nullptr};
  int decode_calls_{0};
  int decode_bound_{0};  // the position bound the decode graph was captured with
  int compute_units_{0};
  bool hand_overs_{true};       // one-token steps use the launches that hand results over inside themselves
  unsigned timeouts_seen_{0};   // the stream's count of hand-overs that did not arrive, as last read
  int hand_over_fallbacks_{0};
  void* stream_{nullptr};
  void* rope_table_{nullptr};
  int last_n_{0};
};

}  // namespace llama_cu
