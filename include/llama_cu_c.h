/*
 * C handles over the C++ host interface (llama_cu_host.hpp), for callers that cannot include
 * C++ headers: the Python tests and bench.py bind these with ctypes.  Each function names the
 * llama_cu.h member of the reference it forwards to.  Return conventions: pointers are NULL on
 * failure; int functions return 0 / a value >= 0 on success and a negative number on failure.
 * A failing GPU call inside the host layer prints the error and raises SIGSEGV, as the
 * reference's CHECK_CUDA does (llama_cu.h:48-56).
 */
#ifndef LLAMA_CU_C_H
#define LLAMA_CU_C_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct lcu_model lcu_model;
typedef struct lcu_context lcu_context;
typedef struct lcu_batch lcu_batch;
typedef struct lcu_vocab lcu_vocab;

/* llama_params (llama_cu.h:280-291) from its fields; q_type 0 = fp16, 1 = uint8 */
/* llama_model::create_synthetic (no reference counterpart: seeded random weights, norms = 1) */
lcu_model* lcu_model_create_synthetic(uint32_t dim, uint32_t multiple_of, uint32_t n_heads, uint32_t n_layers,
                                      uint32_t n_vocab, float norm_eps, int q_type, int quantization_block_size,
                                      uint64_t seed, float weight_std);
/* mapped_buffer(path + "/params") + llama_params::load + llama_partition::autopipe + llama_model::load
 * (main.cpp:24-57, llama_cu.cu:987-997) */
lcu_model* lcu_model_load(const char* model_dir, int context_len);
void lcu_model_destroy(lcu_model*);
uint32_t lcu_model_ffn_dim(const lcu_model*);                      /* llama_params::ffn_dim */
/* the model's llama_params fields (llama_cu.h:280-291); q_type 0 = fp16, 1 = uint8 */
void lcu_model_describe(const lcu_model*, uint32_t* dim, uint32_t* multiple_of, uint32_t* n_heads, uint32_t* n_layers,
                        uint32_t* n_vocab, float* norm_eps, int* q_type, int* quantization_block_size);
/* copies a weight matrix back to the host: stream id 1 tok_embeddings, 2 output, 16+16l+{0..6}
 * wq wk wv wo w1 w2 w3; `scales` may be NULL for fp16 models */
int lcu_model_read_tensor(const lcu_model*, uint64_t stream_id, void* values, void* scales);

/* device pointers of a weight matrix (values or codes, and scales or NULL) and of the norm weight
 * vectors: which = -1 final norm, 2l attention_norm of layer l, 2l+1 ffn_norm of layer l.  Borrowed;
 * valid while the model lives.  For benchmarks that launch single kernels on the real weights. */
int lcu_model_tensor_ptr(const lcu_model*, uint64_t stream_id, void** values_dev, void** scales_dev);
void* lcu_model_norm_ptr(const lcu_model*, int which);

lcu_context* lcu_context_create(lcu_model*, int context_len, float temperature);   /* llama_context::create */
void lcu_context_destroy(lcu_context*);
void lcu_context_clear_tokens(lcu_context*);                                        /* clear_tokens */
size_t lcu_context_memory_usage(lcu_context*);                                      /* context_memory_usage */
size_t lcu_context_tokens_left(lcu_context*);                                       /* tokens_left */
/* next_token (llama_cu.h:380); -1 if the tokens do not fit the context or an id is out of range */
int lcu_context_next_token(lcu_context*, const int16_t* tokens, int n);
/* results of the last next_token call, fp16: logits and probabilities [n_vocab], the residual
 * stream after the last layer [n][dim] (rows = n of that call) */
int lcu_context_read_logits(lcu_context*, uint16_t* out);
int lcu_context_read_probs(lcu_context*, uint16_t* out);
int lcu_context_read_hidden(lcu_context*, uint16_t* out, int rows);
/* first T rows of one layer's KV cache, [T][dim] each; K is stored rotated */
int lcu_context_read_kv(lcu_context*, int layer, uint16_t* k_out, uint16_t* v_out, int T);
/* the hipStream_t (as void*) the context launches on, for event timing */
void* lcu_context_stream(lcu_context*);
/* How many one-token steps of this context were computed a second time because hand-overs between the
 * workgroups of a decode launch did not arrive in time (other work held compute units of the device).
 * Such a step's first token is never returned; from the first such step on the context uses launches
 * that wait for nobody (what LLAMA_CU_NO_HANDOVER=1 selects from the start).  0 on a device the
 * process has to itself.  No counterpart in the reference. */
int lcu_context_hand_over_fallbacks(lcu_context*);
/* llama_context::sample_with_seed / greedy: draw the next tokens from the probabilities (the
 * sampler the reference leaves commented out, llama_cu.cu:1202-1203) or take the maximum again */
void lcu_context_set_sampling(lcu_context*, int enabled, uint64_t seed);

/* llama_batch_context (no counterpart in the reference, which lists batching as a TODO,
 * README.md:34): n_sequences sequences over one model.  lcu_batch_next_token is
 * lcu_context_next_token on one sequence (prompts); lcu_batch_next_tokens takes one new token per
 * sequence and writes every sequence's next token, in one pass over the weights.  -1 on bad
 * arguments (sequence out of range, token outside the vocabulary, a full context). */
lcu_batch* lcu_batch_create(lcu_model*, int n_sequences, int context_len, float temperature);
void lcu_batch_destroy(lcu_batch*);
int lcu_batch_n_sequences(lcu_batch*);
size_t lcu_batch_memory_usage(lcu_batch*);
int lcu_batch_clear_tokens(lcu_batch*, int sequence);
long lcu_batch_tokens_left(lcu_batch*, int sequence);
int lcu_batch_next_token(lcu_batch*, int sequence, const int16_t* tokens, int n);
int lcu_batch_next_tokens(lcu_batch*, const int16_t* tokens, int16_t* out_tokens);
/* fp16 logits / probabilities [n_sequences][n_vocab] of the last lcu_batch_next_tokens */
int lcu_batch_read_logits(lcu_batch*, uint16_t* out);
int lcu_batch_read_probs(lcu_batch*, uint16_t* out);

/* mapped_buffer(path) + llama_vocabulary(buffer) (main.cpp:25,35; llama_cu.cu:1312-1339).  The
 * file is checked first (entry table and piece offsets inside the file, pieces NUL-terminated):
 * NULL if it cannot be read or is malformed, where the reference would read out of bounds. */
lcu_vocab* lcu_vocab_load(const char* vocab_path);
void lcu_vocab_destroy(lcu_vocab*);
int lcu_vocab_size(const lcu_vocab*);                                /* tokens.size() */
/* llama_vocabulary::tokenize(text, bos) (llama_cu.cu:1341-1360): writes at most `capacity` ids and
 * returns how many the text has */
int lcu_vocab_tokenize(lcu_vocab*, const char* text, size_t text_len, int bos, int16_t* out, int capacity);
/* tokens[id].text (bytes, may contain NUL for the byte tokens 3..258) and .score; NULL / 0 if id is
 * out of range */
const char* lcu_vocab_piece(const lcu_vocab*, int id, size_t* len);
float lcu_vocab_score(const lcu_vocab*, int id);

#ifdef __cplusplus
}
#endif
#endif
