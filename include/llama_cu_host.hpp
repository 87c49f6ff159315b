// Host-side C++17 interface of the MI355X build: the public section of the reference's llama_cu.h
// (llama_cu.h:64-139 and 274-394) with the same names, argument meaning, ownership and error
// behaviour, so that the reference's main.cpp compiles against it unchanged.  Nothing in here
// names a GPU API: device work goes through the C ABI declared in llama_cu_hip.h.
//
// Ownership as in the reference: gpu_buffer owns device memory and views borrow it; mapped_buffer
// owns its mapping; llama_model::load returns an owning pointer; a llama_context borrows its model,
// which must outlive it.  I/O failures give false / nullptr / !is_ok(); a failing GPU call prints
// the error and raises SIGSEGV, like the reference's CHECK_CUDA (llama_cu.h:48-56).  One host
// thread per context.
#pragma once

#if __cplusplus < 201703L
#error "C++17 or higher is required"
#endif

#include <cstddef>
#include <cstdint>
#include <memory>
#include <queue>
#include <string>
#include <string_view>
#include <unordered_map>
#include <vector>

#define LLAMA_CU_API __attribute__((visibility("default")))

namespace llama_cu {

// Kept for source compatibility (llama_cu.h:65-68).  1 selects nothing different here and 0 (the
// reference's cuBLAS path) is not offered: every value runs the gfx950 kernels.
extern LLAMA_CU_API int matmul_type;

// llama_cu.h:70-95 -- read-only file mapping, new read/write file of a given size, or anonymous memory
struct LLAMA_CU_API mapped_buffer {
  mapped_buffer();
  mapped_buffer(std::string const& path);
  mapped_buffer(std::string const& path, size_t size);
  mapped_buffer(size_t size);
  ~mapped_buffer();
  mapped_buffer(mapped_buffer&& other);
  mapped_buffer& operator=(mapped_buffer&& other);
  mapped_buffer(mapped_buffer const&) = delete;
  mapped_buffer& operator=(mapped_buffer const&) = delete;
  bool is_ok() const { return ptr_ != nullptr; }
  void* data() const { return ptr_; }
  size_t size() const { return size_; }

 private:
  void release();
  int fd_{-1};
  void* ptr_{nullptr};
  size_t size_{0};
};

// llama_cu.h:97-107 -- selects a device for the lifetime of the object
struct LLAMA_CU_API scoped_gpu {
  scoped_gpu(int device);
  ~scoped_gpu();
  scoped_gpu(scoped_gpu const&) = delete;
  scoped_gpu& operator=(scoped_gpu const&) = delete;

 private:
  int prev_device_;
};

// llama_cu.h:109-122 -- non-owning window on device memory
struct LLAMA_CU_API gpu_buffer_view {
  gpu_buffer_view() {}
  gpu_buffer_view(void* dev_ptr, size_t size) : dev_ptr_(dev_ptr), size_(size) {}
  void copy_from(mapped_buffer const& buffer);        // asynchronous host -> device, sizes must match
  void copy_from(void const* buffer, size_t size);    // asynchronous host -> device
  void copy_to(void* buffer, size_t size);            // blocking device -> host
  bool is_ok() const { return dev_ptr_ != nullptr; }
  void* data() const { return dev_ptr_; }
  size_t size() const { return size_; }

 protected:
  void* dev_ptr_{nullptr};
  size_t size_{0};
};

// llama_cu.h:124-134 -- owning device allocation
struct LLAMA_CU_API gpu_buffer : public gpu_buffer_view {
  gpu_buffer() {}
  gpu_buffer(size_t size);
  gpu_buffer(gpu_buffer&& other);
  gpu_buffer& operator=(gpu_buffer&& other);
  ~gpu_buffer();
  gpu_buffer(gpu_buffer const&) = delete;
  gpu_buffer& operator=(gpu_buffer const&) = delete;
};

enum class quantization_type : uint8_t {
  fp16,
  uint8,
};

#define LLAMA_CU_MAGIC 0x000041524F525541       // "AURORA\0\0" little endian
#define LLAMA_CU_MODEL_FOURCC_LLAMA 0x414D4C4C  // "LLMA" little endian

// llama_cu.h:280-299 -- the 40-byte `params` file, little endian, no padding
struct LLAMA_CU_API llama_params {
  uint64_t magic;
  uint32_t fourcc;
  uint32_t dim;
  uint32_t multiple_of;
  uint32_t n_heads;
  uint32_t n_layers;
  uint32_t n_vocab;
  float norm_eps;
  quantization_type q_type;
  uint8_t reserved0[1];
  uint16_t quantization_block_size;
  bool load(mapped_buffer const& buffer);
  uint32_t ffn_dim() const;
  size_t layer_size() const;
  size_t embedding_size() const;
  size_t output_size() const;
  size_t shared_context_memory_size(size_t context_len) const;
  size_t kv_cache_size(size_t context_len) const;
};
static_assert(sizeof(llama_params) == 40, "llama_params must match the on-disk layout");

// llama_cu.h:301-314.  One MI355X holds every model the reference was run on, so autopipe puts
// everything on device 0 when it fits and marks the partition invalid (-1) when it does not.
struct LLAMA_CU_API llama_partition {
  llama_partition() {}
  void use_default(llama_params const& params);
  void autopipe(llama_params const& params, size_t context_len);
  bool is_valid();
  void debug_print();
  std::vector<int> used_gpus;
  int embedding_gpu{-1};
  std::vector<int> layer_gpus;
  int output_gpu{-1};
};

// llama_cu.h:316-358
struct llama_token {
  short id;
  float score;
  std::string text;
};

struct LLAMA_CU_API llama_vocabulary {
  llama_vocabulary(mapped_buffer const& buffer);
  std::vector<short> tokenize(std::string_view text, bool bos);
  std::unordered_map<std::string, llama_token*> token_lookup;
  std::vector<llama_token> tokens;
};

struct LLAMA_CU_API llama_tokenizer {
  llama_tokenizer(llama_vocabulary const& vocab) : vocab_(vocab) {}
  void tokenize(std::string_view text, std::vector<short>& output);

 private:
  // Segments of the text being tokenized, as parallel arrays indexed by segment: bytes
  // [begin_[i], begin_[i] + bytes_[i]) of text_, neighbours to either side (-1 at the ends), and a
  // version that goes up whenever the segment grows or is swallowed (bytes_ 0), so that a queued
  // merge can tell whether both of its sides are still what they were when it was queued.
  struct merge {
    float score;
    int left;
    int right;
    uint32_t left_version;
    uint32_t right_version;
  };
  short find_piece(size_t begin, size_t bytes, float* score);
  void queue_merge(int left, int right);
  llama_vocabulary const& vocab_;
  std::string_view text_;
  std::vector<uint32_t> begin_, bytes_, version_;
  std::vector<int> left_of_, right_of_;
  std::vector<merge> heap_;
  std::string key_;
};

struct llama_model_impl;

// llama_cu.h:362-372
struct LLAMA_CU_API llama_model {
  static std::unique_ptr<llama_model> load(llama_params params, llama_partition partition, std::string const& path);
  // Not in the reference: a model whose matrices are seeded pseudo-random N(0, weight_std) values
  // (the recipe of lcu_fill_normal_f16; streams: tok_embeddings 1, output 2, layer l 16+16l + {wq 0,
  // wk 1, wv 2, wo 3, w1 4, w2 5, w3 6}) and whose norm weights are 1, quantised on the device when
  // params.q_type is uint8.  Used by tests and benchmarks, where no checkpoint exists.
  static std::unique_ptr<llama_model> create_synthetic(llama_params params, uint64_t seed, float weight_std);
  virtual ~llama_model() {}
  llama_params params;
  llama_partition partition;

 protected:
  llama_model(llama_params params, llama_partition partition) : params(params), partition(partition) {}
};

// llama_cu.h:374-390
struct LLAMA_CU_API llama_context {
  static std::unique_ptr<llama_context> create(llama_model* model, int context_len = 2048, float temperature = 0.9);
  virtual ~llama_context() {}
  virtual void clear_tokens() = 0;
  virtual size_t context_memory_usage() = 0;
  virtual short next_token(std::vector<short> const& new_tokens) = 0;
  size_t tokens_left() { return context_len_ - start_pos_; }
  // Not in the reference, which always returns the most probable token (its sampler,
  // llama_cu.cu:1202-1203, is commented out): from now on next_token draws the token from the
  // probabilities (index i with probability p[i] / sum p) with the k-th output of the splitmix64
  // generator started at `seed` for the k-th token drawn; greedy() returns to the maximum.
  virtual void sample_with_seed(uint64_t seed) = 0;
  virtual void greedy() = 0;

 protected:
  llama_context(llama_model_impl* model, int context_len, float temperature)
      : model_(model), context_len_(context_len), temperature_(temperature) {}
  llama_model_impl* model_;
  int context_len_;
  int start_pos_{0};
  float temperature_;
};

// Not in the reference, where batching is a TODO (README.md:34): n_sequences independent sequences
// over one model.  Each sequence is a llama_context of its own (next_token(sequence, tokens) is that
// context's next_token: prompts of any length, one sequence at a time); next_tokens advances every
// sequence by one token in a single pass over the weights, the sequences' rows forming the M of
// the matrix products.  Greedy (first maximum) tokens, as llama_context returns them.
struct LLAMA_CU_API llama_batch_context {
  static std::unique_ptr<llama_batch_context> create(llama_model* model, int n_sequences, int context_len = 2048,
                                                     float temperature = 0.9);
  virtual ~llama_batch_context() {}
  virtual int n_sequences() = 0;
  virtual void clear_tokens(int sequence) = 0;
  virtual size_t tokens_left(int sequence) = 0;
  virtual size_t context_memory_usage() = 0;
  virtual short next_token(int sequence, std::vector<short> const& new_tokens) = 0;
  // tokens[b] is the one new token of sequence b; returns the next token of every sequence
  virtual std::vector<short> next_tokens(std::vector<short> const& tokens) = 0;
};

LLAMA_CU_API void initialize();

}  // namespace llama_cu
