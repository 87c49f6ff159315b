// llama_params size arithmetic and llama_partition: llama_cu.cu:749-880.
#include <assert.h>

#include "host_common.hpp"

namespace llama_cu {

int matmul_type = 4;

// The reference pads activation tensors with 128 zeroed "gutter" rows for its 128-row tile
// (llama_cu.cu:749, llama_cu.h:236-242).  The kernels here mask instead, but the size formulas a
// caller prints or plans with (main.cpp:47-52) keep the reference's values.
constexpr size_t GUTTER = 128;
constexpr size_t HALF = 2;

bool llama_params::load(mapped_buffer const& buffer) {
  if (buffer.size() != sizeof(llama_params)) {
    return false;
  }
  auto* p = reinterpret_cast<llama_params const*>(buffer.data());
  if (p->magic != LLAMA_CU_MAGIC || p->fourcc != LLAMA_CU_MODEL_FOURCC_LLAMA) {
    return false;
  }
  *this = *p;
  return true;
}

uint32_t llama_params::ffn_dim() const { return (uint32_t)round_up(dim * 8 / 3, multiple_of); }

size_t llama_params::layer_size() const {
  const size_t d = dim, f = ffn_dim();
  const size_t norms = 2 * d * HALF;
  if (q_type == quantization_type::fp16) {
    return 4 * d * d * HALF + 3 * f * d * HALF + norms;
  }
  assert(q_type == quantization_type::uint8 && "unsupported quantization type");
  const size_t b = quantization_block_size;
  // as llama_cu.cu:774-779, including its count of attention scales (one matrix' worth)
  const size_t attn = 4 * d * d + (d / b * d) * HALF;
  const size_t ffn = 3 * f * d + (f / b * d) * HALF + (d / b * f) * HALF * 2;
  return attn + norms + ffn;
}

size_t llama_params::embedding_size() const { return (size_t)n_vocab * dim * HALF; }
size_t llama_params::output_size() const { return (size_t)n_vocab * dim * HALF + dim * HALF; }

size_t llama_params::shared_context_memory_size(size_t context_len) const {
  const size_t rows = context_len + GUTTER;
  const size_t act = rows * dim * HALF;        // embed, norm, xq, xk, out
  const size_t ffn = rows * ffn_dim() * HALF;  // w1, w3, silu
  const size_t qk = n_heads * rows * context_len * HALF;
  const size_t logits = (1 + GUTTER) * n_vocab * HALF;
  return context_len * sizeof(short) + 5 * act + qk + 3 * ffn + logits;
}

size_t llama_params::kv_cache_size(size_t context_len) const { return (context_len + GUTTER) * dim * 2 * HALF; }

void llama_partition::use_default(llama_params const& params) {
  used_gpus = {0};
  embedding_gpu = 0;
  layer_gpus.assign(params.n_layers, 0);
  output_gpu = 0;
}

// The reference packs tensors onto GPUs 0..n greedily by free memory (llama_cu.cu:819-837,
// 862-880).  Here the answer is device 0 for everything, or an invalid partition if the model
// plus its context does not fit in what device 0 has free.
void llama_partition::autopipe(llama_params const& params, size_t context_len) {
  lcu_device_props props;
  int device = 0;
  LCU_CHECK(lcu_get_device(&device));
  LCU_CHECK(lcu_device_get_props(device, &props));
  const size_t reserved = params.shared_context_memory_size(context_len) + 64 * 1024 * 1024;
  const size_t need = reserved + params.embedding_size() + params.output_size() +
                      (size_t)params.n_layers * (params.layer_size() + params.kv_cache_size(context_len));
  const int gpu = need < props.free_memory ? device : -1;
  used_gpus = {gpu};
  embedding_gpu = gpu;
  layer_gpus.assign(params.n_layers, gpu);
  output_gpu = gpu;
}

bool llama_partition::is_valid() {
  if (embedding_gpu == -1 || output_gpu == -1) {
    return false;
  }
  for (int g : layer_gpus) {
    if (g == -1) {
      return false;
    }
  }
  return true;
}

void llama_partition::debug_print() {
  fprintf(stderr, "Model partition:\n");
  fprintf(stderr, "  Embedding GPU: %d\n", embedding_gpu);
  fprintf(stderr, "  Output GPU: %d\n", output_gpu);
  fprintf(stderr, "  Layers:\n    ");
  for (size_t i = 0; i < layer_gpus.size(); i++) {
    fprintf(stderr, "% 3d: %d ", (int)i, layer_gpus[i]);
    if ((i % 8) == 7 && i != layer_gpus.size() - 1) {
      fprintf(stderr, "\n    ");
    }
  }
  fprintf(stderr, "\n");
}

void initialize() {
  LCU_CHECK(lcu_init(0));
  lcu_device_props props;
  LCU_CHECK(lcu_device_get_props(0, &props));
  printf("Device name: %s\n", props.name);
  printf("Number of CUs: %d\n", props.compute_units);
  printf("LDS size per workgroup: %d bytes\n", props.lds_bytes_per_block);
  printf("L2 cache size: %d bytes\n", props.l2_bytes);
  printf("Device memory: %zu bytes total, %zu free\n", props.total_memory, props.free_memory);
}

}  // namespace llama_cu
