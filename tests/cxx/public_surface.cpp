// Every public name of the reference's llama_cu.h (64-139, 274-394), used with the reference's
// signatures.  Compiled and linked by tests/test_abi.py against include/llama_cu.h and the built
// library; never run (main returns before touching a device unless an argument is given).
#include <cstdio>
#include <memory>
#include <string>
#include <string_view>
#include <type_traits>
#include <vector>

#include "llama_cu.h"

using namespace llama_cu;

static_assert(sizeof(llama_params) == 40, "params file layout");
static_assert(std::is_same<std::underlying_type<quantization_type>::type, uint8_t>::value, "enum width");
static_assert(!std::is_copy_constructible<mapped_buffer>::value && std::is_move_constructible<mapped_buffer>::value, "");
static_assert(!std::is_copy_constructible<gpu_buffer>::value && std::is_move_constructible<gpu_buffer>::value, "");
static_assert(std::is_base_of<gpu_buffer_view, gpu_buffer>::value, "");
static_assert(LLAMA_CU_MAGIC == 0x000041524F525541 && LLAMA_CU_MODEL_FOURCC_LLAMA == 0x414D4C4C, "");

int main(int argc, char**) {
  if (argc < 2) {
    return 0;
  }
  matmul_type = 4;
  initialize();
  mapped_buffer a;
  mapped_buffer b(std::string("models/7B/params"));
  mapped_buffer c(std::string("scratch.bin"), (size_t)4096);
  mapped_buffer d((size_t)4096);
  a = std::move(d);
  bool ok = b.is_ok() && a.data() != nullptr && a.size() == 4096;
  {
    scoped_gpu on(0);
    gpu_buffer g((size_t)4096);
    gpu_buffer h(std::move(g));
    g = std::move(h);
    g.copy_from(a);
    g.copy_from(a.data(), a.size());
    g.copy_to(a.data(), a.size());
    gpu_buffer_view v(g.data(), g.size());
    ok = ok && v.is_ok() && v.size() == 4096;
  }
  llama_params p;
  ok = ok && p.load(b);
  size_t sizes = p.ffn_dim() + p.layer_size() + p.embedding_size() + p.output_size() +
                 p.shared_context_memory_size(2048) + p.kv_cache_size(2048);
  quantization_type q = p.q_type == quantization_type::uint8 ? quantization_type::uint8 : quantization_type::fp16;
  llama_partition part;
  part.use_default(p);
  part.autopipe(p, 2048);
  part.debug_print();
  ok = ok && part.is_valid() && part.embedding_gpu >= 0 && part.output_gpu >= 0 && !part.layer_gpus.empty() &&
       !part.used_gpus.empty();
  mapped_buffer vocab_file(std::string("models/7B/vocab"));
  llama_vocabulary vocab(vocab_file);
  std::vector<short> ids = vocab.tokenize(std::string_view("hello"), true);
  llama_token const& t = vocab.tokens[0];
  ok = ok && t.id == 0 && t.score <= 0.0f && !t.text.empty() && vocab.token_lookup.count(t.text) == 1;
  llama_tokenizer tokenizer(vocab);
  tokenizer.tokenize(std::string_view("hello"), ids);
  // the reference's single-argument constructors are not explicit (llama_cu.h:72-74, 98, 126, 323,
  // 330): each type converts implicitly from its argument
  mapped_buffer by_path = std::string("models/7B/params");
  mapped_buffer by_size = (size_t)4096;
  gpu_buffer by_bytes = (size_t)256;
  auto takes_scope = [](scoped_gpu const&) {};
  takes_scope(0);
  llama_vocabulary by_buffer = vocab_file;
  llama_tokenizer by_vocab = vocab;
  by_vocab.tokenize(std::string_view("hello"), ids);
  ok = ok && by_path.is_ok() && by_size.is_ok() && by_bytes.is_ok() && !by_buffer.tokens.empty();
  std::unique_ptr<llama_model> model = llama_model::load(p, part, std::string("models/7B"));
  ok = ok && model && model->params.dim == p.dim && model->partition.output_gpu == part.output_gpu;
  std::unique_ptr<llama_context> context = llama_context::create(model.get());
  std::unique_ptr<llama_context> context2 = llama_context::create(model.get(), 2048, 0.8f);
  context->clear_tokens();
  short next = context->next_token(ids);
  printf("%d %zu %zu %zu %d %d\n", (int)next, context->tokens_left(), context->context_memory_usage(), sizes, (int)q,
         (int)ok);
  return 0;
}
