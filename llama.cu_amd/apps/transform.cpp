// transform: tools over model directories in the reference's on-disk format.
//
//   transform quantize  <input_model> <output_model> [block_size = 128]
//   transform histogram <model> [tensor = attention.wq] [layer = 0]
//
// Same operations, file names and report lines as the reference's transform.cu (quantize_one
// 152-202, copy_tensor 204-222, do_quantize 224-267, do_histogram 326-362, main 514-580).  Its svd
// and compare_svd operations exist only in ENABLE_CUBLAS + ENABLE_CUSOLVER builds and are not
// provided.  A model name is looked up as models/<name>, as in the reference; a name that contains
// a '/' is taken as the directory itself.  The output directory is created if it is missing.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <filesystem>
#include <string>
#include <vector>

#include "llama_cu.h"
#include "llama_cu_hip.h"

using namespace llama_cu;

namespace {

std::string model_dir(std::string const& name) {
  return name.find('/') == std::string::npos ? "models/" + name : name;
}

#define CHECK_LCU(call)                                                   \
  do {                                                                    \
    if ((call) != 0) {                                                    \
      fprintf(stderr, "%s failed: %s\n", #call, lcu_last_error());        \
      return false;                                                       \
    }                                                                     \
  } while (0)

struct matrix_spec {
  std::string name;
  size_t h, w;
};

// every weight matrix of the model, in the order the reference visits them, and every norm vector
void model_tensors(llama_params const& p, std::vector<matrix_spec>& matrices, std::vector<std::string>& vectors) {
  const size_t dim = p.dim, ffn = p.ffn_dim(), vocab = p.n_vocab;
  matrices = {{"tok_embeddings", vocab, dim}, {"output", vocab, dim}};
  vectors = {"norm"};
  for (uint32_t l = 0; l < p.n_layers; ++l) {
    const std::string base = "layers." + std::to_string(l) + ".";
    vectors.push_back(base + "attention_norm");
    vectors.push_back(base + "ffn_norm");
    for (const char* m : {"attention.wq", "attention.wk", "attention.wv", "attention.wo"}) {
      matrices.push_back({base + m, dim, dim});
    }
    matrices.push_back({base + "feed_forward.w1", ffn, dim});
    matrices.push_back({base + "feed_forward.w2", dim, ffn});
    matrices.push_back({base + "feed_forward.w3", ffn, dim});
  }
}

bool read_params(std::string const& dir, llama_params& params) {
  mapped_buffer buf(dir + "/params");
  if (!buf.is_ok()) {
    fprintf(stderr, "Could not load params file\n");
    return false;
  }
  if (!params.load(buf)) {
    fprintf(stderr, "Invalid model parameters\n");
    return false;
  }
  return true;
}

std::string matrix_file(std::string const& dir, std::string const& name, const char* kind, size_t h, size_t w) {
  return dir + "/" + name + "." + kind + "__" + std::to_string(h) + "_" + std::to_string(w);
}

// device buffers sized for the largest matrix, reused for every tensor
struct quantize_buffers {
  gpu_buffer input, dequantised, codes, scales, stats;
  explicit quantize_buffers(size_t max_elems, int block)
      : input(max_elems * 2), dequantised(max_elems * 2), codes(max_elems), scales(max_elems / block * 2), stats(12) {}
};

bool quantize_matrix(quantize_buffers& b, std::string const& in_dir, std::string const& out_dir, matrix_spec const& m,
                     int block) {
  printf("quantizing %s (%zu x %zu)\n", m.name.c_str(), m.h, m.w);
  const size_t n = m.h * m.w;
  mapped_buffer src(matrix_file(in_dir, m.name, "weight", m.h, m.w));
  if (!src.is_ok() || src.size() != n * 2) {
    fprintf(stderr, "failed to load tensor %s (%zu x %zu)\n", m.name.c_str(), m.h, m.w);
    return false;
  }
  CHECK_LCU(lcu_h2d(b.input.data(), src.data(), n * 2, nullptr));
  CHECK_LCU(lcu_quantize_absmax_u8(b.codes.data(), b.scales.data(), b.input.data(), m.h, m.w, block, nullptr));
  CHECK_LCU(lcu_dequantize_absmax_u8(b.dequantised.data(), b.scales.data(), b.codes.data(), m.h, m.w, block, nullptr));
  CHECK_LCU(lcu_error_stats(b.stats.data(), b.input.data(), b.dequantised.data(), n, nullptr));
  float stats[3];
  CHECK_LCU(lcu_d2h(stats, b.stats.data(), sizeof(stats), nullptr));
  printf("  rms/max/mean error: %f/%f/%f\n", std::sqrt(stats[0]), stats[1], stats[2]);
  const size_t scale_bytes = m.h * (m.w / block) * 2;
  mapped_buffer code_file(matrix_file(out_dir, m.name, "weight", m.h, m.w), n);
  mapped_buffer scale_file(matrix_file(out_dir, m.name, "scale", m.h, m.w / block), scale_bytes);
  if (!code_file.is_ok()) {
    fprintf(stderr, "failed to create weight tensor %s (%zu x %zu)\n", m.name.c_str(), m.h, m.w);
    return false;
  }
  if (!scale_file.is_ok()) {
    fprintf(stderr, "failed to create scale tensor %s (%zu x %zu)\n", m.name.c_str(), m.h, m.w);
    return false;
  }
  CHECK_LCU(lcu_d2h(scale_file.data(), b.scales.data(), scale_bytes, nullptr));
  CHECK_LCU(lcu_d2h(code_file.data(), b.codes.data(), n, nullptr));
  return true;
}

bool copy_vector(std::string const& in_dir, std::string const& out_dir, std::string const& name, size_t w) {
  const std::string file = "/" + name + ".weight__" + std::to_string(w);
  mapped_buffer src(in_dir + file);
  if (!src.is_ok()) {
    fprintf(stderr, "failed to load tensor %s (%zu)\n", name.c_str(), w);
    return false;
  }
  mapped_buffer dst(out_dir + file, src.size());
  if (!dst.is_ok()) {
    fprintf(stderr, "failed to create tensor %s (%zu)\n", name.c_str(), w);
    return false;
  }
  memcpy(dst.data(), src.data(), src.size());
  return true;
}

bool quantize_model(std::string const& in_name, std::string const& out_name, int block) {
  const std::string in_dir = model_dir(in_name), out_dir = model_dir(out_name);
  llama_params params;
  if (!read_params(in_dir, params)) return false;
  if (params.q_type != quantization_type::fp16) {
    fprintf(stderr, "Input model is not fp16\n");
    return false;
  }
  if (block < 16 || block % 16 != 0 || block > 65535 || params.dim % block != 0 || params.ffn_dim() % block != 0) {
    fprintf(stderr, "Unsupported block size %d (a multiple of 16 dividing %u and %u)\n", block, params.dim,
            params.ffn_dim());
    return false;
  }
  std::error_code ec;
  std::filesystem::create_directories(out_dir, ec);
  std::vector<matrix_spec> matrices;
  std::vector<std::string> vectors;
  model_tensors(params, matrices, vectors);
  size_t largest = 0;
  for (auto const& m : matrices) largest = std::max(largest, m.h * m.w);
  quantize_buffers buffers(largest, block);
  for (auto const& m : matrices) {
    if (!quantize_matrix(buffers, in_dir, out_dir, m, block)) return false;
  }
  for (auto const& v : vectors) {
    if (!copy_vector(in_dir, out_dir, v, params.dim)) return false;
  }
  llama_params out_params = params;
  out_params.q_type = quantization_type::uint8;
  out_params.quantization_block_size = (uint16_t)block;
  mapped_buffer params_file(out_dir + "/params", sizeof(llama_params));
  if (!params_file.is_ok()) {
    fprintf(stderr, "Failed to create params file\n");
    return false;
  }
  memcpy(params_file.data(), &out_params, sizeof(llama_params));
  // the vocabulary belongs to the model directory too; carry it over when the input has one
  mapped_buffer vocab(in_dir + "/vocab");
  if (vocab.is_ok()) {
    mapped_buffer vocab_out(out_dir + "/vocab", vocab.size());
    if (vocab_out.is_ok()) memcpy(vocab_out.data(), vocab.data(), vocab.size());
  }
  return true;
}

bool tensor_shape(llama_params const& p, std::string const& tensor, int layer, size_t& h, size_t& w) {
  if (tensor == "tok_embeddings" || tensor == "output") {
    if (layer != -1) {
      fprintf(stderr, "Invalid layer index %d for tensor %s\n", layer, tensor.c_str());
      return false;
    }
    h = p.n_vocab;
    w = p.dim;
  } else if (tensor == "attention.wq" || tensor == "attention.wk" || tensor == "attention.wv" ||
             tensor == "attention.wo") {
    h = w = p.dim;
  } else if (tensor == "feed_forward.w1" || tensor == "feed_forward.w3") {
    h = p.ffn_dim();
    w = p.dim;
  } else if (tensor == "feed_forward.w2") {
    h = p.dim;
    w = p.ffn_dim();
  } else {
    fprintf(stderr, "Unknown tensor name %s\n", tensor.c_str());
    return false;
  }
  return true;
}

bool histogram(std::string const& name, std::string const& tensor, int layer) {
  const std::string dir = model_dir(name);
  llama_params params;
  if (!read_params(dir, params)) return false;
  if (params.q_type != quantization_type::uint8) {
    fprintf(stderr, "Input model is not uint8\n");
    return false;
  }
  size_t h, w;
  if (!tensor_shape(params, tensor, layer, h, w)) return false;
  const std::string full = (layer >= 0 ? "layers." + std::to_string(layer) + "." : std::string()) + tensor;
  mapped_buffer codes(matrix_file(dir, full, "weight", h, w));
  if (!codes.is_ok() || codes.size() != h * w) {
    fprintf(stderr, "Failed to load tensor %s\n", tensor.c_str());
    return false;
  }
  uint32_t counts[256] = {};
  const uint8_t* q = static_cast<const uint8_t*>(codes.data());
  for (size_t i = 0; i < codes.size(); ++i) counts[q[i]]++;
  printf("      ");
  for (int j = 0; j < 16; ++j) printf("%-8X", j);
  printf("\n");
  for (int i = 0; i < 16; ++i) {
    printf("%4X: ", i);
    for (int j = 0; j < 16; ++j) printf("%-8d", counts[i * 16 + j]);
    printf("\n");
  }
  return true;
}

void usage() {
  fprintf(stderr,
          "usage: transform quantize <input_model> <output_model> [block_size]\n"
          "       transform histogram <model> [tensor] [layer]\n");
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 3) {
    usage();
    return 2;
  }
  const std::string operation = argv[1];
  if (operation == "histogram") {  // host only: no device needed
    return histogram(argv[2], argc > 3 ? argv[3] : "attention.wq", argc > 4 ? atoi(argv[4]) : 0) ? 0 : 1;
  }
  if (operation == "quantize") {
    if (argc < 4) {
      usage();
      return 2;
    }
    initialize();
    return quantize_model(argv[2], argv[3], argc > 4 ? atoi(argv[4]) : 128) ? 0 : 1;
  }
  if (operation == "svd" || operation == "compare_svd") {
    fprintf(stderr, "%s needs the reference's optional cuSOLVER build and is not provided\n", operation.c_str());
    return 1;
  }
  fprintf(stderr, "Unknown operation: %s\n", operation.c_str());
  return 1;
}
