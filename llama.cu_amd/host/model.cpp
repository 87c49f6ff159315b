// Model weights and the forward pass: the host orchestration of llama_cu.cu:882-1310
// (llama_layer, llama_model_impl, llama_context_impl) over the C ABI of llama_cu_hip.h.
//
// What is kept from the reference: the order of operations of next_token, every point where an
// intermediate is rounded to fp16, the [position][dim] KV cache, the per-tensor file format, the
// first-maximum argmax over the fp16 probabilities.  What is not: its zeroed gutter rows, its
// per-layer score-tensor allocation, its side streams, its re-rotation of every cached K row on
// every call (K is cached rotated; RoPE depends only on value and position, so the bits agree),
// and its one-launch-per-operation decode loop (a single new token runs the fused kernels).
#include <assert.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "model_impl.hpp"

namespace llama_cu {

namespace {

constexpr uint16_t FP16_ONE = 0x3C00;

bool load_matrix(weight_tensor& t, llama_params const& params, std::string const& path, std::string const& name,
                 size_t h, size_t w) {
  // llama_cu.cu:929-971: <name>.weight__<h>_<w> holds fp16 values or uint8 codes,
  // <name>.scale__<h>_<w/block> the fp16 scales of a quantised tensor
  t.rows = h;
  t.cols = w;
  const std::string stem = path + "/" + name;
  if (params.q_type == quantization_type::fp16) {
    t.quantised = false;
    t.block = 0;
    t.data = gpu_buffer(h * w * 2);
    mapped_buffer buf(stem + ".weight__" + std::to_string(h) + "_" + std::to_string(w));
    if (!buf.is_ok() || buf.size() != t.data.size()) {
      fprintf(stderr, "failed to load tensor %s (%zu x %zu)\n", name.c_str(), h, w);
      return false;
    }
    t.data.copy_from(buf);
    LCU_CHECK(lcu_sync(nullptr));  // the mapping goes away at the end of this scope
    return true;
  }
  if (params.q_type == quantization_type::uint8) {
    const size_t block = params.quantization_block_size;
    if (block == 0 || w % block != 0) {
      fprintf(stderr, "failed to load tensor %s: width %zu is not a multiple of block %zu\n", name.c_str(), w, block);
      return false;
    }
    t.quantised = true;
    t.block = (int)block;
    t.data = gpu_buffer(h * w);
    t.scales = gpu_buffer(h * (w / block) * 2);
    mapped_buffer wbuf(stem + ".weight__" + std::to_string(h) + "_" + std::to_string(w));
    if (!wbuf.is_ok() || wbuf.size() != t.data.size()) {
      fprintf(stderr, "failed to load tensor %s (%zu x %zu)\n", name.c_str(), h, w);
      return false;
    }
    t.data.copy_from(wbuf);
    mapped_buffer sbuf(stem + ".scale__" + std::to_string(h) + "_" + std::to_string(w / block));
    if (!sbuf.is_ok() || sbuf.size() != t.scales.size()) {
      fprintf(stderr, "failed to load tensor scale %s (%zu x %zu)\n", name.c_str(), h, w / block);
      return false;
    }
    t.scales.copy_from(sbuf);
    LCU_CHECK(lcu_sync(nullptr));
    return true;
  }
  fprintf(stderr, "Unsupported quantization type %d\n", (int)params.q_type);
  return false;
}

bool load_vector(gpu_buffer& t, std::string const& path, std::string const& name, size_t w) {
  // llama_cu.cu:972-984
  t = gpu_buffer(w * 2);
  mapped_buffer buf(path + "/" + name + ".weight__" + std::to_string(w));
  if (!buf.is_ok() || buf.size() != t.size()) {
    fprintf(stderr, "failed to load tensor %s\n", name.c_str());
    return false;
  }
  t.copy_from(buf);
  LCU_CHECK(lcu_sync(nullptr));
  return true;
}

void synth_matrix(weight_tensor& t, llama_params const& params, gpu_buffer& staging, size_t h, size_t w, uint64_t seed,
                  uint64_t stream_id, float std) {
  t.rows = h;
  t.cols = w;
  if (params.q_type == quantization_type::uint8) {
    const int block = params.quantization_block_size;
    t.quantised = true;
    t.block = block;
    t.data = gpu_buffer(h * w);
    t.scales = gpu_buffer(h * (w / block) * 2);
    if (staging.size() < h * w * 2) {
      staging = gpu_buffer();  // release before growing
      staging = gpu_buffer(h * w * 2);
    }
    LCU_CHECK(lcu_fill_normal_f16(staging.data(), h * w, seed, stream_id, std, nullptr));
    LCU_CHECK(lcu_quantize_absmax_u8(t.data.data(), t.scales.data(), staging.data(), h, w, block, nullptr));
  } else {
    t.quantised = false;
    t.block = 0;
    t.data = gpu_buffer(h * w * 2);
    LCU_CHECK(lcu_fill_normal_f16(t.data.data(), h * w, seed, stream_id, std, nullptr));
  }
}

void synth_ones(gpu_buffer& t, size_t w) {
  t = gpu_buffer(w * 2);
  LCU_CHECK(lcu_fill_f16(t.data(), w, FP16_ONE, nullptr));
}

}  // namespace

bool llama_model_impl::load_impl(std::string const& path) {
  // llama_cu.cu:891-922
  const size_t dim = params.dim, ffn = params.ffn_dim(), vocab = params.n_vocab;
  RETURN_UNLESS(load_matrix(tok_embeddings, params, path, "tok_embeddings", vocab, dim));
  RETURN_UNLESS(load_matrix(output, params, path, "output", vocab, dim));
  RETURN_UNLESS(load_vector(norm, path, "norm", dim));
  layers.clear();
  layers.reserve(params.n_layers);
  for (uint32_t i = 0; i < params.n_layers; ++i) {
    llama_layer L;
    const std::string base = "layers." + std::to_string(i) + ".";
    RETURN_UNLESS(load_vector(L.attn_norm, path, base + "attention_norm", dim));
    RETURN_UNLESS(load_vector(L.ffn_norm, path, base + "ffn_norm", dim));
    RETURN_UNLESS(load_matrix(L.wq, params, path, base + "attention.wq", dim, dim));
    RETURN_UNLESS(load_matrix(L.wk, params, path, base + "attention.wk", dim, dim));
    RETURN_UNLESS(load_matrix(L.wv, params, path, base + "attention.wv", dim, dim));
    RETURN_UNLESS(load_matrix(L.wo, params, path, base + "attention.wo", dim, dim));
    RETURN_UNLESS(load_matrix(L.w1, params, path, base + "feed_forward.w1", ffn, dim));
    RETURN_UNLESS(load_matrix(L.w2, params, path, base + "feed_forward.w2", dim, ffn));
    RETURN_UNLESS(load_matrix(L.w3, params, path, base + "feed_forward.w3", ffn, dim));
    layers.emplace_back(std::move(L));
  }
  return true;
}

void llama_model_impl::synthesize(uint64_t seed, float std) {
  const size_t dim = params.dim, ffn = params.ffn_dim(), vocab = params.n_vocab;
  gpu_buffer staging;
  synth_matrix(tok_embeddings, params, staging, vocab, dim, seed, 1, std);
  synth_matrix(output, params, staging, vocab, dim, seed, 2, std);
  synth_ones(norm, dim);
  layers.clear();
  layers.reserve(params.n_layers);
  for (uint32_t i = 0; i < params.n_layers; ++i) {
    llama_layer L;
    const uint64_t base = 16 + 16 * (uint64_t)i;
    synth_matrix(L.wq, params, staging, dim, dim, seed, base + 0, std);
    synth_matrix(L.wk, params, staging, dim, dim, seed, base + 1, std);
    synth_matrix(L.wv, params, staging, dim, dim, seed, base + 2, std);
    synth_matrix(L.wo, params, staging, dim, dim, seed, base + 3, std);
    synth_matrix(L.w1, params, staging, ffn, dim, seed, base + 4, std);
    synth_matrix(L.w2, params, staging, dim, ffn, seed, base + 5, std);
    synth_matrix(L.w3, params, staging, ffn, dim, seed, base + 6, std);
    synth_ones(L.attn_norm, dim);
    synth_ones(L.ffn_norm, dim);
    layers.emplace_back(std::move(L));
  }
  LCU_CHECK(lcu_sync(nullptr));
}

weight_tensor const* llama_model_impl::tensor_by_stream(uint64_t stream_id) const {
  if (stream_id == 1) return &tok_embeddings;
  if (stream_id == 2) return &output;
  if (stream_id < 16) return nullptr;
  const size_t l = (stream_id - 16) / 16, which = (stream_id - 16) % 16;
  if (l >= layers.size() || which > 6) return nullptr;
  llama_layer const& L = layers[l];
  weight_tensor const* tab[7] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.w1, &L.w2, &L.w3};
  return tab[which];
}

static bool shapes_supported(llama_params const& p) {
  if (p.n_heads == 0 || p.dim == 0 || p.dim % p.n_heads != 0 || p.dim / p.n_heads != 128) {
    fprintf(stderr, "unsupported model shape: dim %u with %u heads (head_dim must be 128)\n", p.dim, p.n_heads);
    return false;
  }
  if (p.n_heads > 64 || p.dim > 8192 || p.dim % 16 != 0 || p.ffn_dim() > 24576) {
    fprintf(stderr, "unsupported model shape: dim %u (at most 8192), %u heads (at most 64), ffn %u (at most 24576)\n",
            p.dim, p.n_heads, p.ffn_dim());
    return false;
  }
  if (p.n_vocab == 0 || p.n_vocab > 32767) {
    fprintf(stderr, "unsupported vocabulary size %u (token ids are 16-bit)\n", p.n_vocab);
    return false;
  }
  if (p.q_type == quantization_type::uint8) {
    const uint32_t b = p.quantization_block_size;
    if (b < 16 || b % 16 != 0 || p.dim % b != 0 || p.ffn_dim() % b != 0) {
      fprintf(stderr, "unsupported quantization block size %u for dim %u / ffn %u\n", b, p.dim, p.ffn_dim());
      return false;
    }
  } else if (p.q_type != quantization_type::fp16) {
    fprintf(stderr, "Unsupported quantization type %d\n", (int)p.q_type);
    return false;
  }
  return true;
}

/* static */ std::unique_ptr<llama_model> llama_model::load(llama_params params, llama_partition partition,
                                                            std::string const& path) {
  // llama_cu.cu:987-997
  if (!shapes_supported(params)) {
    return nullptr;
  }
  auto model = std::make_unique<llama_model_impl>(params, partition);
  if (!model->load_impl(path)) {
    return nullptr;
  }
  return model;
}

/* static */ std::unique_ptr<llama_model> llama_model::create_synthetic(llama_params params, uint64_t seed,
                                                                        float weight_std) {
  params.magic = LLAMA_CU_MAGIC;
  params.fourcc = LLAMA_CU_MODEL_FOURCC_LLAMA;
  if (!shapes_supported(params)) {
    return nullptr;
  }
  llama_partition partition;
  partition.use_default(params);
  auto model = std::make_unique<llama_model_impl>(params, partition);
  model->synthesize(seed, weight_std);
  return model;
}

// ------------------------------------------------------------------------------------------------
// context
// ------------------------------------------------------------------------------------------------
llama_context_impl::llama_context_impl(llama_model* model, int context_len, float temperature)
    : llama_context(static_cast<llama_model_impl*>(model), context_len, temperature) {
  device_structure_lock lock(device_structure_mutex());
  LCU_CHECK(lcu_init(0));
  LCU_CHECK(lcu_stream_create(&stream_));
  lcu_device_props props;
  LCU_CHECK(lcu_device_get_props(0, &props));
  compute_units_ = props.compute_units;
  const int head_dim = model_->params.dim / model_->params.n_heads;
  LCU_CHECK(lcu_rope_table_create(&rope_table_, context_len_, head_dim, 10000.0f));  // theta: llama_cu.cu:374
  // The decode launches that hand results over between their own workgroups need those workgroups
  // resident together, which only a device that this process has to itself guarantees.
  // LLAMA_CU_NO_HANDOVER=1 (a GPU shared with other processes) keeps every context on launches that
  // never wait for one another: same results, about a sixth slower.
  const char* no_hand_over = getenv("LLAMA_CU_NO_HANDOVER");
  hand_overs_ = !(no_hand_over != nullptr && atoi(no_hand_over) != 0);
  LCU_CHECK(lcu_sync_timeouts(stream_, &timeouts_seen_));
  clear_tokens();
}

llama_context_impl::~llama_context_impl() {
  lcu_sync(stream_);
  device_structure_lock lock(device_structure_mutex());
  // Every one-token step has looked at the count of hand-overs that did not arrive before it returned
  // its token (next_token), so there is nothing left to judge here; a context whose steps had to be
  // recomputed says so once more when it goes.
  if (hand_over_fallbacks_ > 0) {
    fprintf(stderr, "llama_context: %d decode step(s) of this context were recomputed after hand-overs inside a "
                    "launch did not arrive\n", hand_over_fallbacks_);
  }
  lcu_graph_destroy(decode_graph_);
  lcu_free(rope_table_);
  lcu_stream_destroy(stream_);
}

void llama_context_impl::clear_tokens() {
  // llama_cu.cu:1004-1049: fresh zeroed KV cache and scratch, position 0
  llama_params const& p = model_->params;
  const size_t ctx = (size_t)context_len_, dim = p.dim, ffn = p.ffn_dim();
  LCU_CHECK(lcu_sync(stream_));
  drop_graph();  // it holds pointers into the caches released below
  kv_.clear();
  kv_.resize(p.n_layers);
  for (auto& kv : kv_) {
    kv.k = gpu_buffer(ctx * dim * 2);
    kv.v = gpu_buffer(ctx * dim * 2);
    LCU_CHECK(lcu_memset(kv.k.data(), 0, kv.k.size(), stream_));
    LCU_CHECK(lcu_memset(kv.v.data(), 0, kv.v.size(), stream_));
  }
  if (!t_embed_.is_ok()) {
    t_embed_ = gpu_buffer(ctx * dim * 2);
    t_norm_ = gpu_buffer(ctx * dim * 2);
    t_xq_ = gpu_buffer(ctx * dim * 2);
    t_out_ = gpu_buffer(ctx * dim * 2);
    t_w1_ = gpu_buffer(ctx * ffn * 2);
    t_w3_ = gpu_buffer(ctx * ffn * 2);
    t_silu_ = gpu_buffer(ctx * ffn * 2);
    t_tokens_ = gpu_buffer(ctx * sizeof(short));
    t_logits_ = gpu_buffer((size_t)p.n_vocab * 2);
    t_probs_ = gpu_buffer((size_t)p.n_vocab * 2);
    t_argmax_ = gpu_buffer(2 * sizeof(int));  // {token, count of hand-overs that did not arrive}
    t_step_ = gpu_buffer(sizeof(step_state));
  }
  LCU_CHECK(lcu_sync(stream_));
  start_pos_ = 0;
  last_n_ = 0;
}

size_t llama_context_impl::context_memory_usage() {
  size_t count = 0;
  for (auto& kv : kv_) {
    count += kv.k.size() + kv.v.size();
  }
  for (gpu_buffer const* b : {&t_embed_, &t_norm_, &t_xq_, &t_out_, &t_w1_, &t_w3_, &t_silu_, &t_tokens_, &t_logits_,
                              &t_probs_, &t_argmax_, &t_step_}) {
    count += b->size();
  }
  return count;
}

void llama_context_impl::matmul(void* out, const void* lhs, weight_tensor const& w, int M, float beta) {
  // llama_cu.cu:1498-1523
  if (w.quantised) {
    LCU_CHECK(lcu_gemm_f16u8_nt(out, lhs, w.data.data(), w.scales.data(), M, (int)w.cols, (int)w.rows, w.block, beta,
                                stream_));
  } else {
    LCU_CHECK(lcu_gemm_f16_nt(out, lhs, w.data.data(), M, (int)w.cols, (int)w.rows, beta, stream_));
  }
}

// products of one lhs with several weight matrices of one shape (Wq, Wk, Wv; W1, W3) in one launch
void llama_context_impl::matmul_multi(void* const* outs, const void* lhs, weight_tensor const* const* ws, int count,
                                      int M) {
  const void* values[3];
  const void* scales[3];
  for (int g = 0; g < count; ++g) {
    values[g] = ws[g]->data.data();
    scales[g] = ws[g]->scales.data();
  }
  weight_tensor const& w = *ws[0];
  if (w.quantised) {
    LCU_CHECK(lcu_gemm_f16u8_nt_multi(outs, lhs, values, scales, count, M, (int)w.cols, (int)w.rows, w.block, 0.0f,
                                      stream_));
  } else {
    LCU_CHECK(lcu_gemm_f16_nt_multi(outs, lhs, values, count, M, (int)w.cols, (int)w.rows, 0.0f, stream_));
  }
}

// The layer loop for n new rows sitting in t_embed_; positions start_pos_ .. start_pos_ + n - 1.
// n == 1 takes the fused decode kernels, which read the position from t_step_ on the device.
void llama_context_impl::enqueue_layers(int n, bool first_norm_ready) {
  llama_params const& p = model_->params;
  const int dim = p.dim, ffn = p.ffn_dim(), heads = p.n_heads;
  const int sp = start_pos_, T = sp + n;
  const int block = p.q_type == quantization_type::uint8 ? p.quantization_block_size : 0;
  char* x = (char*)t_embed_.data();
  bool norm_ready = first_norm_ready;  // t_norm_ already holds this layer's normalised input
  for (size_t l = 0; l < model_->layers.size(); ++l) {
    llama_layer const& L = model_->layers[l];
    char* kc = (char*)kv_[l].k.data();
    char* vc = (char*)kv_[l].v.data();
    bool fused_wo = false;
    if (n == 1) {
      // 1129 (unless the previous layer's W2 launch has left the normalised row behind), then
      // 1144-1156 in one launch, then 1161-1171 in one launch
      if (!norm_ready) {
        LCU_CHECK(lcu_rmsnorm(t_norm_.data(), x, L.attn_norm.data(), 1, dim, p.norm_eps, stream_));
      }
      norm_ready = false;
      LCU_CHECK(lcu_decode_qkv(t_xq_.data(), kc, vc, t_norm_.data(), nullptr, L.wq.data.data(), L.wk.data.data(),
                               L.wv.data.data(), L.wq.scales.data(), L.wk.scales.data(), L.wv.scales.data(), block, dim,
                               heads, 0, t_step_.data(), p.norm_eps, rope_table_, context_len_, stream_));
      const void* seq = (char*)t_step_.data() + offsetof(step_state, seq);
      // fp16 weights and rows of up to 1024 scores: attention, the Wo product with the residual sum
      // (1174) and the norm that follows (1176) in one launch
      fused_wo = hand_overs_ && !L.wo.quantised && decode_bound_ <= 1024 && heads * 8 <= compute_units_;
      if (!hand_overs_) {
        // launches whose workgroups never wait for one another (1161-1171)
        LCU_CHECK(lcu_attention_decode(t_out_.data(), t_xq_.data(), kc, vc, t_step_.data(), decode_bound_, dim, heads,
                                       stream_));
      } else if (fused_wo) {
        LCU_CHECK(lcu_decode_attention_wo_norm(x, t_norm_.data(), t_xq_.data(), kc, vc, L.wo.data.data(),
                                               L.ffn_norm.data(), p.norm_eps, t_step_.data(), seq, (int)(l & 1023),
                                               decode_bound_, dim, heads, stream_));
      } else {
        LCU_CHECK(lcu_attention_decode_spread(t_out_.data(), t_xq_.data(), kc, vc, t_step_.data(), seq,
                                              (int)(l & 1023), decode_bound_, dim, heads, stream_));
      }
    } else {
      char* k_new = kc + (size_t)sp * dim * 2;
      char* v_new = vc + (size_t)sp * dim * 2;
      LCU_CHECK(lcu_rmsnorm(t_norm_.data(), x, L.attn_norm.data(), n, dim, p.norm_eps, stream_));            // 1129
      void* const qkv_out[3] = {t_xq_.data(), k_new, v_new};
      weight_tensor const* const qkv_w[3] = {&L.wq, &L.wk, &L.wv};
      matmul_multi(qkv_out, t_norm_.data(), qkv_w, 3, n);                                                    // 1144, 1150, 1156
      LCU_CHECK(lcu_rope_pair(t_xq_.data(), k_new, n, dim, heads, sp, rope_table_, context_len_, stream_));  // 1146, 1152 (new rows only)
      LCU_CHECK(lcu_attention(t_out_.data(), t_xq_.data(), kc, vc, n, T, sp, dim, heads, stream_));          // 1161-1171
    }
    if (n == 1 && hand_overs_ && !fused_wo && dim <= 8192) {
      // 1174 and 1176 in one launch (salts: even for this one, odd for the W2 launch below)
      LCU_CHECK(lcu_decode_proj_norm(x, t_norm_.data(), t_out_.data(), L.wo.data.data(), L.wo.scales.data(), block, dim,
                                     dim, L.ffn_norm.data(), p.norm_eps,
                                     (char*)t_step_.data() + offsetof(step_state, seq), (int)((2 * l) & 1023), stream_));
    } else if (!fused_wo) {
      matmul(x, t_out_.data(), L.wo, n, 1.0f);                                                               // 1174
      LCU_CHECK(lcu_rmsnorm(t_norm_.data(), x, L.ffn_norm.data(), n, dim, p.norm_eps, stream_));             // 1176
    }
    if (n == 1) {
      // 1180-1183 in one launch
      LCU_CHECK(lcu_decode_ffn_up(t_silu_.data(), t_norm_.data(), nullptr, L.w1.data.data(), L.w3.data.data(),
                                  L.w1.scales.data(), L.w3.scales.data(), block, dim, ffn, p.norm_eps, stream_));
    } else {
      void* const up_out[2] = {t_w1_.data(), t_w3_.data()};
      weight_tensor const* const up_w[2] = {&L.w1, &L.w3};
      matmul_multi(up_out, t_norm_.data(), up_w, 2, n);                                                      // 1180, 1181
      LCU_CHECK(lcu_silu_mul(t_silu_.data(), t_w1_.data(), t_w3_.data(), (size_t)n * ffn, stream_));         // 1183
    }
    if (n == 1 && hand_overs_ && l + 1 < model_->layers.size() && dim <= 8192) {
      // 1185 and the next layer's 1129 in one launch
      llama_layer const& next = model_->layers[l + 1];
      LCU_CHECK(lcu_decode_proj_norm(x, t_norm_.data(), t_silu_.data(), L.w2.data.data(), L.w2.scales.data(), block,
                                     ffn, dim, next.attn_norm.data(), p.norm_eps,
                                     (char*)t_step_.data() + offsetof(step_state, seq), (int)((2 * l + 1) & 1023), stream_));
      norm_ready = true;
    } else {
      matmul(x, t_silu_.data(), L.w2, n, 1.0f);                                                              // 1185
    }
  }
}

// final norm of the last row, logits, softmax with temperature, argmax: llama_cu.cu:1191-1209.
// The reference normalises every row and uses the last one.
void llama_context_impl::enqueue_head(int n) {
  llama_params const& p = model_->params;
  const int dim = p.dim, vocab = p.n_vocab;
  const int block = p.q_type == quantization_type::uint8 ? p.quantization_block_size : 0;
  char* x = (char*)t_embed_.data();
  if (block > 0) {
    // uint8 weights: the GEMV is bound by its vector instructions, and normalising the row in each of
    // its 16 000 workgroups costs more there (60 us) than a norm launch of its own (6 + 39 us)
    LCU_CHECK(lcu_rmsnorm(t_norm_.data(), x + (size_t)(n - 1) * dim * 2, model_->norm.data(), 1, dim, p.norm_eps, stream_));
    LCU_CHECK(lcu_gemm_f16u8_nt(t_logits_.data(), t_norm_.data(), model_->output.data.data(),
                                model_->output.scales.data(), 1, dim, vocab, block, 0.0f, stream_));
  } else {
    LCU_CHECK(lcu_decode_logits(t_logits_.data(), x + (size_t)(n - 1) * dim * 2, model_->norm.data(),
                                model_->output.data.data(), model_->output.scales.data(), block, dim, vocab, p.norm_eps,
                                stream_));
  }
  // the first maximum of the fp16 probabilities is found on the device; 4 bytes go back to the host
  // and, next to it, the stream's count of hand-overs that did not arrive, for next_token's one copy back
  LCU_CHECK(lcu_softmax_argmax_status(t_probs_.data(), t_argmax_.data(), t_logits_.data(), vocab, temperature_,
                                      stream_));
  if (sampling_) {  // 1202-1203; the random bits of this step are in t_step_
    LCU_CHECK(lcu_sample_row(t_argmax_.data(), t_probs_.data(), vocab, 0,
                             (char*)t_step_.data() + offsetof(step_state, random), stream_));
  }
}

void llama_context_impl::sample_with_seed(uint64_t seed) {
  if (!sampling_) {
    drop_graph();  // the captured step has no sampler launch
  }
  sampling_ = true;
  sample_seed_ = seed;
  samples_drawn_ = 0;
}

void llama_context_impl::greedy() {
  if (sampling_) {
    drop_graph();
  }
  sampling_ = false;
}

void llama_context_impl::drop_graph() {
  if (decode_graph_) {
    device_structure_lock lock(device_structure_mutex());
    LCU_CHECK(lcu_graph_destroy(decode_graph_));
    decode_graph_ = nullptr;
  }
  decode_calls_ = 0;
}

short llama_context_impl::next_token(std::vector<short> const& new_tokens) {
  llama_params const& p = model_->params;
  const int n = (int)new_tokens.size();
  assert(n > 0);
  assert(new_tokens.size() + start_pos_ <= (size_t)context_len_);  // llama_cu.cu:1074
  const int dim = p.dim, vocab = p.n_vocab;
  const int block = p.q_type == quantization_type::uint8 ? p.quantization_block_size : 0;
  char* x = (char*)t_embed_.data();
  const void* ids = t_tokens_.data();
  host_step_.pos = start_pos_;
  host_step_.token = new_tokens[0];
  if (sampling_) {  // output samples_drawn_ of splitmix64 started at the seed
    uint64_t z = sample_seed_ + (samples_drawn_ + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    host_step_.random = z ^ (z >> 31);
    ++samples_drawn_;
  }
  if (n == 1 || sampling_) {
    // The launches that hand results over inside themselves tell new words from old ones by the low 21 bits of
    // this counter: when those come round, the words are cleared, and the value that cleared words carry is skipped.
    if ((++host_step_.seq & 0x1fffffu) == 0) {
      ++host_step_.seq;
      LCU_CHECK(lcu_sync_reset(stream_));
    }
    LCU_CHECK(lcu_h2d(t_step_.data(), &host_step_, sizeof(host_step_), stream_));
  }
  if (n == 1) {
    ids = (char*)t_step_.data() + offsetof(step_state, token);
  } else {
    LCU_CHECK(lcu_h2d(t_tokens_.data(), new_tokens.data(), n * sizeof(short), stream_));  // 1086
  }
  auto enqueue_all = [&]() {
    // 1087-1097; a one-token step gathers the row and normalises it for the first layer (1129) in one launch
    const bool quantised = model_->tok_embeddings.quantised;
    if (n == 1 && dim % 8 == 0 && dim <= 8192 && (!quantised || block % 8 == 0) && !model_->layers.empty()) {
      LCU_CHECK(lcu_embed_rmsnorm(x, t_norm_.data(), ids, 1, dim, model_->tok_embeddings.data.data(),
                                  quantised ? model_->tok_embeddings.scales.data() : nullptr, quantised ? block : 0, vocab,
                                  model_->layers[0].attn_norm.data(), model_->params.norm_eps, stream_));
      enqueue_layers(n, true);
      enqueue_head(n);
      return;
    }
    if (model_->tok_embeddings.quantised) {
      LCU_CHECK(lcu_embed_u8(x, ids, n, dim, model_->tok_embeddings.data.data(), model_->tok_embeddings.scales.data(),
                             block, vocab, stream_));
    } else {
      LCU_CHECK(lcu_embed(x, ids, n, dim, model_->tok_embeddings.data.data(), vocab, stream_));
    }
    enqueue_layers(n);
    enqueue_head(n);
  };
  // One decode step at a time per process: the launch that joins attention, Wo and norm puts one
  // workgroup on every compute unit and these wait for one another, so two such launches running side
  // by side (two contexts driven from two host threads) could each hold compute units the other needs
  // until their bounded waits run out.  Held from the launch to the token's arrival.
  static std::mutex decode_step_mutex;
  std::unique_lock<std::mutex> one_step(decode_step_mutex, std::defer_lock);
  if (n == 1) {
    one_step.lock();
  }
  if (n == 1) {
    // A decode step is ~260 launches of a few microseconds each: the first one runs eagerly (and
    // loads the kernels), the second is captured into a HIP graph, every later one replays it.
    // Decode attention has a form for short rows and one for long rows, chosen by the bound it is
    // given; the graph is captured again when the position outgrows the short bound.
    const int bound = (start_pos_ + 1 <= 1024 && context_len_ > 1024) ? 1024 : (int)context_len_;
    device_structure_lock lock(device_structure_mutex());  // capture, instantiation, launch: see host_common.hpp
    if (decode_graph_ && bound != decode_bound_) {
      LCU_CHECK(lcu_graph_destroy(decode_graph_));
      decode_graph_ = nullptr;
    }
    decode_bound_ = bound;
    ++decode_calls_;
    // LLAMA_CU_NO_GRAPH=1 keeps every step eager: profilers that instrument graph launches have
    // crashed on the host inside hipGraphLaunch on graphs of more than about 400 kernel nodes
    static const bool no_graph = getenv("LLAMA_CU_NO_GRAPH") != nullptr && atoi(getenv("LLAMA_CU_NO_GRAPH")) != 0;
    if (!decode_graph_ && decode_calls_ >= 2 && !no_graph) {
      LCU_CHECK(lcu_graph_begin_capture(stream_));
      enqueue_all();
      LCU_CHECK(lcu_graph_end_capture(stream_, &decode_graph_));
    }
    if (decode_graph_) {
      LCU_CHECK(lcu_graph_launch(decode_graph_, stream_));
    } else {
      enqueue_all();
    }
  } else {
    enqueue_all();
  }
  struct {
    int token;
    unsigned timeouts;
  } result{0, 0};
  LCU_CHECK(lcu_d2h(&result, t_argmax_.data(), sizeof(result), stream_));  // 1198-1200, blocks
  // The one-token launches hand results over between their workgroups with bounded waits, and a wait
  // that ran out went on with stale words: the count of such waits comes back with the token, and a
  // count that has moved means this step's token is not to be trusted.  It is never returned: the
  // context leaves the hand-over launches for good (something else is holding compute units of this
  // device), and the step is computed again by launches that wait for nobody -- the step is a function
  // of the token, the position and the cache rows below the position, all untouched.  A call whose
  // launches hand nothing over (several tokens, or a context already on the plain launches) does not
  // depend on the count: if it moves there, somebody else is using this stream's workspace, which is
  // reported and otherwise harmless to the result.
  if (result.timeouts != timeouts_seen_) {
    const unsigned moved = result.timeouts - timeouts_seen_;
    timeouts_seen_ = result.timeouts;
    if (hand_overs_ && n == 1) {
      fprintf(stderr, "llama_context: %u hand-over(s) between workgroups of a decode launch did not arrive (is other "
                      "work holding compute units of this device?); the step is recomputed without them\n", moved);
      ++hand_over_fallbacks_;
      hand_overs_ = false;
      drop_graph();
      enqueue_all();
      LCU_CHECK(lcu_d2h(&result, t_argmax_.data(), sizeof(result), stream_));
      timeouts_seen_ = result.timeouts;
    } else {
      fprintf(stderr, "llama_context: the stream's count of failed hand-overs moved by %u during a call that hands "
                      "nothing over (is the stream's workspace shared?); the call's result does not depend on it\n", moved);
    }
  }
  start_pos_ += n;
  last_n_ = n;
  return (short)result.token;
}

/* static */ std::unique_ptr<llama_context> llama_context::create(llama_model* model, int context_len,
                                                                  float temperature) {
  // The reference leaves context_len free (llama_cu.h:376); the attention kernels here hold a row of
  // scores per head in LDS, which bounds it.  Refused at creation, not in the middle of a generation.
  if (model == nullptr || context_len <= 0 || context_len > LLAMA_CU_MAX_CONTEXT) {
    fprintf(stderr, "unsupported context length %d (1..%d)\n", context_len, LLAMA_CU_MAX_CONTEXT);
    return nullptr;
  }
  return std::make_unique<llama_context_impl>(model, context_len, temperature);
}

}  // namespace llama_cu
