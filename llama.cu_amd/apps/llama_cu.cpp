// llama_cu: greedy text generation from a model directory.
//
//   llama_cu [matmul_type] [model_name] [prompt] [max_tokens = 200] [context_len = 2048] [sample_seed]
//
// The command line, the printed lines, the stop at token 2, the half-context re-prefill when the
// context is full and the times.txt report follow the reference's main.cpp (9-110); the reference's
// own main.cpp also builds unchanged against include/llama_cu.h.  matmul_type is accepted and
// ignored.  A model name is looked up as models/<name>; a name containing '/' is the directory.
// max_tokens and context_len are additions for testing with small contexts; with sample_seed the
// tokens are drawn from the probabilities (the sampler the reference leaves commented out,
// llama_cu.cu:1202-1203) instead of taking the most probable one.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "llama_cu.h"

using namespace llama_cu;
using steady = std::chrono::steady_clock;

namespace {

struct options {
  std::string model = "7B";
  std::string prompt = "Building a website can be done in 10 easy steps:";
  int max_tokens = 200;
  size_t context_len = 2048;
  bool sample = false;
  uint64_t sample_seed = 0;
};

double seconds_since(steady::time_point t0) { return std::chrono::duration<double>(steady::now() - t0).count(); }

std::string model_dir(std::string const& name) {
  return name.find('/') == std::string::npos ? "models/" + name : name;
}

void print_model_facts(llama_params const& p, size_t context_len) {
  const double mb = 1024.0 * 1024.0;
  printf("Dimension: %d\nSwiGLU multiple: %d\nLayers: %d\nHeads: %d\nVocab: %d\nNorm Epsilon: %f\n"
         "Shared Context Memory: %f MB\nPer-Layer Context Memory: %f MB\n",
         p.dim, p.multiple_of, p.n_layers, p.n_heads, p.n_vocab, p.norm_eps,
         p.shared_context_memory_size(context_len) / mb, p.kv_cache_size(context_len) / mb);
}

// Generates up to max_tokens tokens after the prompt; returns the per-token wall times.
std::vector<float> generate(llama_context& context, llama_vocabulary& vocab, std::vector<short> const& prompt,
                            options const& opt, int& generated) {
  std::vector<short> history = prompt;  // everything fed or produced so far
  std::vector<short> feed = prompt;     // what the next call consumes
  std::vector<float> times;
  generated = 0;
  while (generated < opt.max_tokens) {
    const auto t0 = steady::now();
    if (context.tokens_left() == 0) {
      // context full: start over from the most recent half of the history (main.cpp:83-87)
      context.clear_tokens();
      const size_t keep = std::min(history.size(), opt.context_len / 2);
      feed.assign(history.end() - keep, history.end());
    }
    const short token = context.next_token(feed);
    const float dt = (float)seconds_since(t0);
    if (token < 0) {
      fprintf(stderr, "\nnext_token failed: %zu tokens do not fit the context\n", feed.size());
      break;
    }
    if (token == 2) {  // end of sequence
      break;
    }
    fputs(vocab.tokens[token].text.c_str(), stdout);
    fflush(stdout);
    feed.assign(1, token);
    history.push_back(token);
    times.push_back(dt);
    ++generated;
  }
  return times;
}

}  // namespace

int main(int argc, char const** argv) {
  options opt;
  if (argc > 1) matmul_type = atoi(argv[1]);
  if (argc > 2) opt.model = argv[2];
  if (argc > 3) opt.prompt = argv[3];
  if (argc > 4) opt.max_tokens = atoi(argv[4]);
  if (argc > 5) opt.context_len = (size_t)atol(argv[5]);
  if (argc > 6) {
    opt.sample = true;
    opt.sample_seed = strtoull(argv[6], nullptr, 10);
  }
  if (opt.context_len < 2) {
    fprintf(stderr, "context_len must be at least 2\n");
    return 1;
  }
  initialize();
  const std::string dir = model_dir(opt.model);
  mapped_buffer params_buf(dir + "/params");
  mapped_buffer vocab_buf(dir + "/vocab");
  if (!params_buf.is_ok()) {
    fprintf(stderr, "Could not load params file\n");
    return 1;
  }
  if (!vocab_buf.is_ok()) {
    fprintf(stderr, "Could not load vocab file\n");
    return 1;
  }
  llama_params params;
  if (!params.load(params_buf)) {
    fprintf(stderr, "Invalid model parameters\n");
    return 1;
  }
  llama_vocabulary vocab(vocab_buf);
  if (vocab.tokens.size() != params.n_vocab) {
    fprintf(stderr, "Vocab size mismatch\n");
    return 1;
  }
  llama_partition partition;
  partition.autopipe(params, opt.context_len);
  partition.debug_print();
  if (!partition.is_valid()) {
    fprintf(stderr, "Could not partition model\n");
    return 1;
  }
  print_model_facts(params, opt.context_len);
  auto model = llama_model::load(params, partition, dir);
  if (!model) {
    fprintf(stderr, "Could not load model\n");
    return 1;
  }
  auto context = llama_context::create(model.get(), (int)opt.context_len, 0.8f);
  printf("Context memory: %f MB\n", context->context_memory_usage() / 1024.0 / 1024.0);
  if (opt.sample) {
    context->sample_with_seed(opt.sample_seed);
  }

  const std::vector<short> prompt = vocab.tokenize(opt.prompt, true);
  if (prompt.size() > opt.context_len) {
    fprintf(stderr, "Prompt of %zu tokens exceeds the context of %zu\n", prompt.size(), opt.context_len);
    return 1;
  }
  int generated = 0;
  const auto start = steady::now();
  const std::vector<float> times = generate(*context, vocab, prompt, opt, generated);
  printf("\ntokens: %d time: %f\n", generated, seconds_since(start));
  // times.txt: prompt length, then one wall time per generated token (plot_times.py reads it)
  FILE* fp = fopen("times.txt", "w");
  if (!fp) {
    fprintf(stderr, "Could not write times.txt\n");
    return 1;
  }
  fprintf(fp, "%zu\n", prompt.size());
  for (float t : times) fprintf(fp, "%f\n", t);
  fclose(fp);
  return 0;
}
