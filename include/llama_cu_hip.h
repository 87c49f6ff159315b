/*
 * C ABI of the MI355X (gfx950) device layer behind the llama_cu host interface.
 *
 * The reference (eiz/llama.cu) has no FFI: its forward pass, llama_context_impl::next_token
 * (llama_cu.cu:1073-1210), launches CUDA kernels directly.  This header declares one entry point
 * per launch site of that function, plus the buffer calls of llama_cu.h:109-134, so that the host
 * code (and any other language) reaches the GPU through plain pointers and sizes.
 *
 * Conventions
 *   - every pointer named *_dev is device memory; fp16 tensors are IEEE binary16, row-major
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); work is asynchronous
 *     unless stated
 *   - every function returns 0 on success and a negative code on failure, never throws, never
 *     exits; lcu_last_error() describes the last failure of the calling thread
 *   - shapes the kernels do not support are rejected before any launch (LCU_E_SHAPE)
 *   - one host thread per stream.  Operators that work in two launches keep partial results in
 *     a 32 MiB workspace: every stream made by lcu_stream_create owns one (so contexts, which each
 *     create a stream, never share scratch), the default stream and streams made elsewhere use one
 *     per device created by lcu_init - calls on those that overlap on one device race
 */
#ifndef LLAMA_CU_HIP_H
#define LLAMA_CU_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LCU_OK 0
#define LCU_E_HIP (-1)      /* a HIP runtime call failed */
#define LCU_E_SHAPE (-2)    /* unsupported or inconsistent shape / null pointer */
#define LCU_E_NOINIT (-3)   /* lcu_init has not run on this device */

typedef struct lcu_device_props {
  char name[128];
  int compute_units;
  int lds_bytes_per_block;
  int l2_bytes;
  int clock_khz;
  int memory_clock_khz;
  int memory_bus_bits;
  size_t total_memory;
  size_t free_memory;
} lcu_device_props;

/* ---- runtime: llama_cu.cu:1525-1542 (initialize), 691-736 (scoped_gpu, gpu_buffer[_view]) ---- */
int lcu_init(int device);
const char* lcu_last_error(void);
int lcu_device_get_props(int device, lcu_device_props* out);
int lcu_get_device(int* out_device);                                            /* scoped_gpu, 691-697 */
int lcu_set_device(int device);
int lcu_malloc(void** out_dev, size_t bytes);                                   /* gpu_buffer ctor, 712-715 */
int lcu_free(void* dev);                                                        /* gpu_buffer dtor, 732-736 */
int lcu_memset(void* dev, int byte_value, size_t bytes, void* stream);          /* llama_cu.h:239-241 */
int lcu_h2d(void* dst_dev, const void* src_host, size_t bytes, void* stream);   /* copy_from, 699-706; async */
int lcu_d2h(void* dst_host, const void* src_dev, size_t bytes, void* stream);   /* copy_to, 707-710; blocks */
int lcu_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream);
int lcu_stream_create(void** out_stream);
int lcu_stream_destroy(void* stream);
/* bounded in-launch waits that ran out on this stream's workspace so far (0 in any healthy run) */
int lcu_sync_timeouts(void* stream, unsigned* out_count);
/* Adds `count` to that counter (stream-ordered), as a wait that ran out would: lets a caller rehearse its
 * handling of a failed hand-over without making any kernel wait.  No counterpart in the reference. */
int lcu_sync_add_timeouts(void* stream, unsigned count);

/* Clears the stream's hand-over words (stream-ordered, not under capture).  A hand-over word is taken for new
 * when it carries the launch's epoch, 21 bits of *seq_dev and the salt: a caller whose step counter has run
 * through 2^21 values clears the words before the epochs repeat, and never uses a counter whose low 21 bits
 * are zero with salt 0 (the epoch of a cleared word).  No counterpart in the reference. */
int lcu_sync_reset(void* stream);
int lcu_sync(void* stream);                                                     /* NULL = whole device */
/* HIP graph capture of the launches made on `stream` between begin and end; every lcu_* kernel
 * entry point may be captured (none of them records a memset node or allocates).  No counterpart
 * in the reference, whose host loop launches ~480 kernels per token one by one. */
int lcu_graph_begin_capture(void* stream);
int lcu_graph_end_capture(void* stream, void** out_graph_exec);
int lcu_graph_launch(void* graph_exec, void* stream);
int lcu_graph_destroy(void* graph_exec);
int lcu_event_create(void** out_event);
int lcu_event_destroy(void* event);
int lcu_event_record(void* event, void* stream);
int lcu_event_elapsed_ms(float* out_ms, void* start_event, void* stop_event);   /* waits for stop */

/* ---- matmul: out[M,N] = lhs[M,K] * rhs[N,K]^T + beta * out ----
 * lcu_gemm_f16_nt replaces matmul_nt(tensor4d_view) and the kernels it selects
 * (llama_cu.cu:1463-1496, 150-220, 225-285): M == 1 runs the streaming GEMV, larger M the MFMA
 * GEMM.  K must be a multiple of 8.  fp32 accumulation, one rounding to fp16 of acc + beta*out.
 * With 2 <= M <= 64 (short prompts) and K a multiple of 128 the K range is split over workgroups
 * and the fp32 partial sums pass through the stream's workspace (both GEMM entry points). */
int lcu_gemm_f16_nt(void* out_dev, const void* lhs_dev, const void* rhs_dev, int M, int K, int N,
                    float beta, void* stream);
/* lcu_gemm_f16u8_nt replaces matmul_nt(generic_tensor&) for quantised weights and
 * matmul_nt_wmma_16x128x256_fp16u8 (llama_cu.cu:1498-1523, 287-366): codes [N,K] uint8, scales
 * [N,K/block] fp16, each weight dequantised as fp16((code - 127.5) * scale) before it is used.
 * K % 16 == 0, block % 16 == 0, K % block == 0. */
int lcu_gemm_f16u8_nt(void* out_dev, const void* lhs_dev, const void* codes_dev,
                      const void* scales_dev, int M, int K, int N, int block, float beta,
                      void* stream);
/* Up to three such products with one lhs and weight matrices of one shape in a single launch
 * (Wq, Wk, Wv at launch sites 1144-1156; W1, W3 at 1180-1181): out_dev, rhs_dev (codes_dev,
 * scales_dev) are host arrays of n_mats device pointers.  Same results as n_mats separate calls;
 * with M == 1 it is n_mats separate calls. */
int lcu_gemm_f16_nt_multi(void* const* out_dev, const void* lhs_dev, const void* const* rhs_dev, int n_mats, int M,
                          int K, int N, float beta, void* stream);
int lcu_gemm_f16u8_nt_multi(void* const* out_dev, const void* lhs_dev, const void* const* codes_dev,
                            const void* const* scales_dev, int n_mats, int M, int K, int N, int block, float beta,
                            void* stream);

/* ---- int8 absmax quantiser: transform.cu:28-72 and 74-87; block in {32, 64, 128, 256, 512, 1024} */
int lcu_quantize_absmax_u8(void* codes_dev, void* scales_dev, const void* in_dev, size_t rows,
                           size_t cols, int block, void* stream);
int lcu_dequantize_absmax_u8(void* out_dev, const void* scales_dev, const void* codes_dev,
                             size_t rows, size_t cols, int block, void* stream);

/* ---- row and element-wise kernels ---- */
/* rms_norm, llama_cu.cu:66-107 (launch sites 1129, 1176, 1191) */
int lcu_rmsnorm(void* out_dev, const void* in_dev, const void* weights_dev, int rows, int cols,
                float eps, void* stream);
/* rotary, llama_cu.cu:368-389 (launch sites 1146, 1152).  The angles cos/sin(pos / theta^(c/head_dim))
 * come from a table built once on the host with the C library's powf/cosf/sinf:
 * table_dev[pos][pair] = {cos, sin} as float2, pair = (c mod head_dim) / 2. */
int lcu_rope_table_create(void** out_table_dev, int positions, int head_dim, float theta);
int lcu_rope(void* out_dev, const void* in_dev, int rows, int cols, int n_heads, int pos_offset,
             const void* table_dev, int table_positions, void* stream);
/* lcu_rope in place on two tensors of one shape in one launch: the new rows of Q and of K of a prompt
 * (launch sites 1146 and 1152; the reference rotates the whole K cache into a scratch copy on every call) */
int lcu_rope_pair(void* a_dev, void* b_dev, int rows, int cols, int n_heads, int pos_offset, const void* table_dev,
                  int table_positions, void* stream);
/* softmax_rows, llama_cu.cu:433-499 (launch sites 1166, 1196); in place allowed */
int lcu_softmax_rows(void* out_dev, const void* in_dev, int rows, int w, float temp, void* stream);
/* e^x on n fp32 values with the exponential that every softmax and SiLU of this library takes
 * (IEEE operations only, within one ulp; the reference calls CUDA's expf at llama_cu.cu:463, 497,
 * 537).  Exported so that the host restatement of the same steps can be held to it bit for bit. */
int lcu_exp_f32(void* out_dev, const void* in_dev, size_t n, void* stream);
/* silu, llama_cu.cu:533-539 (launch site 1183) */
int lcu_silu_mul(void* out_dev, const void* a_dev, const void* b_dev, size_t size, void* stream);
/* embed / embed_uint8, llama_cu.cu:32-62 (launch sites 1090, 1094); ids are int16 */
int lcu_embed(void* out_dev, const void* ids_dev, int n_ids, int dim, const void* table_dev,
              int n_vocab, void* stream);
int lcu_embed_u8(void* out_dev, const void* ids_dev, int n_ids, int dim, const void* codes_dev,
                 const void* scales_dev, int block, int n_vocab, void* stream);
/* embed / embed_uint8 (launch sites 1090, 1094) and the first layer's rms_norm (1129) of the same rows in
 * one launch: x_out gets the rows, norm_out their norm under weights_dev.  block 0: table_dev is the fp16
 * table and scales_dev is ignored; else table_dev holds codes (block a multiple of 8 dividing dim).
 * dim a multiple of 8, at most 8192.  Same values as lcu_embed[_u8] followed by lcu_rmsnorm. */
int lcu_embed_rmsnorm(void* x_out_dev, void* norm_out_dev, const void* ids_dev, int n_ids, int dim,
                      const void* table_dev, const void* scales_dev, int block, int n_vocab,
                      const void* weights_dev, float eps, void* stream);
/* the host argmax of llama_cu.cu:1205-1209 done on the device: index of the first maximum of n
 * fp16 values compared as float, written as int32 */
int lcu_argmax_f16(void* out_index_dev, const void* values_dev, int n, void* stream);
/* softmax_rows over one row of n logits with temperature (launch site 1196) and the argmax of
 * 1205-1209 on its rounded output, in one launch; probs_dev must not alias logits_dev */
int lcu_softmax_argmax(void* probs_dev, void* out_index_dev, const void* logits_dev, int n, float temp,
                       void* stream);
/* lcu_softmax_argmax whose output is two int32: the index, then the stream's count of bounded in-launch
 * waits that ran out (what lcu_sync_timeouts reads) as it stands when this launch runs.  A step that ends
 * with this launch brings its own health back in the copy that fetches the token: a count that has moved
 * since the last step means hand-over words of this step were stale and its token must not be used
 * (the fail-loud rule of llama_cu.h:48-56 applied to the in-launch hand-overs). */
int lcu_softmax_argmax_status(void* probs_dev, void* out_index2_dev, const void* logits_dev, int n, float temp,
                              void* stream);

/* the sampler the reference leaves commented out at llama_cu.cu:1202-1203
 * (std::discrete_distribution over the probabilities): int32 index i drawn with probability
 * p[i] / sum(p) from n fp16 values and 64 random bits, in integer arithmetic (weight = p * 2^24,
 * r = floor(random * total / 2^64), the smallest i whose running weight sum exceeds r; 0 when all
 * weights are 0).  random_dev, when not NULL, points at the 64 bits on the device and replaces
 * `random`, so a captured launch can draw a new number on every replay. */
int lcu_sample_row(void* out_index_dev, const void* probs_dev, int n, uint64_t random, const void* random_dev,
                   void* stream);

/* ---- attention: matmul_qk + softmax_rows + matmul_qkv, llama_cu.cu:400-531, launch sites
 * 1161-1171, without the [n_heads, n, T] score tensor in memory.  q [n_new, dim]; k (already
 * rotated) and v are the first T rows of a [*, dim] cache; causal: row r sees columns
 * c <= r + start_pos.  Scores are rounded to fp16, probabilities are rounded to fp16, the
 * weighted sum runs in fp32: the reference's three rounding points.  head_dim must be 128,
 * T <= 4096 (the multi-row kernel keeps a strip of 16 or 32 rows of scores in LDS).  A call with
 * n_new == 1 hands scores over between workgroups inside its launch when `stream` was made by
 * lcu_stream_create (such a stream owns its hand-over words); on the default stream and on streams
 * made elsewhere, which share the device's, it takes launches that hand nothing over. */
int lcu_attention(void* out_dev, const void* q_dev, const void* k_dev, const void* v_dev,
                  int n_new, int T, int start_pos, int dim, int n_heads, void* stream);

/* lcu_attention for one new token whose position (= T - 1) is read from the device int32 pos_dev
 * when the kernel runs; max_T bounds it (at most the cache length; the position is clamped to it).
 * A bound of 1024 or less selects the single-launch kernel, a larger one the two-launch form that
 * spreads long rows over the chip, so a caller that replays a captured graph keeps the bound at
 * 1024 while the position allows it.  Uses the stream's workspace when max_T > 1024. */
int lcu_attention_decode(void* out_dev, const void* q_dev, const void* k_dev, const void* v_dev,
                         const void* pos_dev, int max_T, int dim, int n_heads, void* stream);

/* lcu_attention_decode with the work of a head spread over eight workgroups, which hand their scores
 * to one another inside the launch through the stream's workspace (same bits as
 * lcu_attention_decode).  Every score travels with the launch's epoch, *seq_dev << 10 | salt: seq_dev is a device
 * uint32 that the caller changes (counts up) before every run of the call, also before every replay
 * of a graph that holds it; salt (0..1023) tells the calls of one such run apart (the layer index).
 * Two consecutive launches on a stream must never have the same epoch.  A hand-over that does not
 * arrive (it cannot on an otherwise idle device) is given up after a bounded wait and counted:
 * lcu_sync_timeouts.  No counterpart in the reference (its score tensor goes through memory
 * between three launches, llama_cu.cu:1161-1171). */
int lcu_attention_decode_spread(void* out_dev, const void* q_dev, const void* k_dev, const void* v_dev,
                                const void* pos_dev, const void* seq_dev, int salt, int max_T, int dim, int n_heads,
                                void* stream);

/* lcu_attention_decode_spread, then x += att . Wo^T (llama_cu.cu:1174, fp16 Wo [dim, dim]) and
 * norm_out = rms_norm(x) with norm_w (1176), in one launch of one 1024-thread workgroup per compute
 * unit: each owns 16 rows of everything, holds its rows of Wo in registers while the attention
 * runs, and takes part in three more hand-overs like the scores' (same epoch rule, same bounded
 * waits).  Same bits as lcu_attention_decode + lcu_gemm_f16_nt (beta 1) + lcu_rmsnorm.  max_T <= 1024;
 * 8 * n_heads workgroups wait for one another and must all be resident, one per compute unit: more
 * heads than a eighth of the compute units are refused (LCU_E_SHAPE), and on a device whose compute
 * units other work holds for good the waits run out (lcu_sync_timeouts) and the result is undefined.
 * Two launches of this entry point must not run at the same time (two streams): each could hold compute
 * units the other is waiting for; the host layer runs one decode step at a time for that reason.
 * x_io_dev: the residual row, updated in place. */
int lcu_decode_attention_wo_norm(void* x_io_dev, void* norm_out_dev, const void* q_dev, const void* k_dev,
                                 const void* v_dev, const void* wo_dev, const void* norm_w_dev, float eps,
                                 const void* pos_dev, const void* seq_dev, int salt, int max_T, int dim, int n_heads,
                                 void* stream);

/* ---- one decode step of several sequences (batching is a TODO of the reference, README.md:34):
 * the GEMMs take the n_seq rows as M; these three handle what differs per sequence.  The caches
 * are given as device arrays of n_seq pointers ([positions][dim] fp16 each), positions as n_seq
 * int32 on the device (row pos[b] is the new one of sequence b). ---- */
/* rotary of row b of q (in place) and of k_new at position pos[b]; rotated k and v_new row b are
 * stored in row pos[b] of sequence b's caches (launch sites 1144-1156 with a position per row) */
int lcu_rope_store_batch(void* q_dev, const void* k_new_dev, const void* v_new_dev, const void* k_cache_ptrs_dev,
                         const void* v_cache_ptrs_dev, const void* pos_dev, int n_seq, int dim, int n_heads,
                         const void* table_dev, int table_positions, void* stream);
/* lcu_attention for one new token (n_new == 1, T cached rows, start_pos = T - 1) that allocates
 * nothing and touches no workspace: no counterpart in the reference; for callers that cannot
 * call hipMalloc (code under HIP graph capture, serving loops and harnesses that forbid it).  The
 * scores of rows longer than 1024 go through a static device array of 64 heads x 4096 rows of
 * fp16 (512 KiB per GPU, held until the process ends): T beyond 4096 or more than 64 heads are
 * rejected (LCU_E_SHAPE), lcu_init must have run on the current device (LCU_E_NOINIT).  Same bits
 * as lcu_attention.  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU
 * (two streams, two threads) race. */
int lcu_attention_decode_static(void* out_dev, const void* q_dev, const void* k_dev, const void* v_dev, int T,
                                int dim, int n_heads, void* stream);
/* lcu_attention_decode for every sequence in one launch: row b of q against rows 0..pos[b] of
 * sequence b's caches -> row b of out; max_T bounds pos[b] + 1 */
int lcu_attention_decode_batch(void* out_dev, const void* q_dev, const void* k_cache_ptrs_dev,
                               const void* v_cache_ptrs_dev, const void* pos_dev, int n_seq, int max_T, int dim,
                               int n_heads, void* stream);
/* The products of a batched step fused with what follows them (for 2..64 sequences the partial sums
 * of the split-K product are added up by the kernel that goes on with them; any other shape runs
 * the separate operators above).  w_dev / scales_dev: host arrays of device pointers (scales NULL
 * and block 0 for fp16 weights); *_tmp_dev: [n_seq][dim] / [n_seq][ffn] fp16 scratch.
 *   lcu_batch_qkv: Wq, Wk, Wv products of lhs [n_seq][dim], then lcu_rope_store_batch (1144-1156)
 *   lcu_batch_ffn_up: W1, W3 products, then fp16(silu(w1) * w3) (1180-1183)
 *   lcu_batch_proj_norm: x += lhs [n_seq][K] * W^T (1174 / 1185), then norm_out = rms_norm(x) with
 *     norm_w (1176, or 1129 of the next layer, or 1191) */
int lcu_batch_qkv(void* q_out_dev, void* k_tmp_dev, void* v_tmp_dev, const void* lhs_dev, const void* const* w_dev,
                  const void* const* scales_dev, int block, int n_seq, int dim, int n_heads,
                  const void* k_cache_ptrs_dev, const void* v_cache_ptrs_dev, const void* pos_dev,
                  const void* table_dev, int table_positions, void* stream);
int lcu_batch_ffn_up(void* out_dev, void* w1_tmp_dev, void* w3_tmp_dev, const void* lhs_dev, const void* const* w_dev,
                     const void* const* scales_dev, int block, int n_seq, int dim, int ffn, void* stream);
int lcu_batch_proj_norm(void* x_dev, void* norm_out_dev, const void* lhs_dev, const void* w_dev, const void* scales_dev,
                        int block, int n_seq, int K, int dim, const void* norm_w_dev, float eps, void* stream);
/* lcu_softmax_argmax on `rows` rows of n logits (n a multiple of 8): probabilities [rows][n],
 * one int32 index per row */
int lcu_softmax_argmax_rows(void* probs_dev, void* out_index_dev, const void* logits_dev, int rows, int n, float temp,
                            void* stream);

/* ---- fused decode steps (n_new == 1), each replacing several launch sites of next_token ---- */
/* rms_norm(x, attn_norm) -> Wq/Wk/Wv GEMV -> RoPE(q, k at position pos) -> q to q_out, k and v into
 * row pos of the caches: llama_cu.cu:1129-1156.  Weight pointers are fp16 [dim, dim], or uint8 codes
 * with fp16 scales when block > 0.  norm_w_dev == NULL means x_dev is already normalised
 * (lcu_rmsnorm ran first); the same holds for lcu_decode_ffn_up.  pos_dev != NULL: the position is
 * read from that device int32 when the kernel runs (`pos` is ignored), so that one captured graph
 * serves every decode step. */
int lcu_decode_qkv(void* q_out_dev, void* k_cache_dev, void* v_cache_dev, const void* x_dev,
                   const void* norm_w_dev, const void* wq_dev, const void* wk_dev, const void* wv_dev,
                   const void* sq_dev, const void* sk_dev, const void* sv_dev, int block, int dim,
                   int n_heads, int pos, const void* pos_dev, float eps, const void* rope_table_dev,
                   int table_positions, void* stream);
/* x += lhs [1, K] . W^T (W [N, K], fp16 or uint8 codes with scales; llama_cu.cu:1185) and then
 * norm_out = rms_norm(x) with norm_w (1129 of the next layer), in one launch: one more workgroup
 * than the GEMV has waits inside the launch for the rows of the new x, which reach it as
 * {two halves, epoch} words through the stream's workspace, and writes x and its norm.  The epoch is
 * *seq_dev << 10 | salt, as for lcu_attention_decode_spread (same rule, same bounded wait).  Same
 * bits as lcu_gemm_f16_nt / lcu_gemm_f16u8_nt (beta 1) + lcu_rmsnorm.  N <= 8192. */
int lcu_decode_proj_norm(void* x_io_dev, void* norm_out_dev, const void* lhs_dev, const void* w_dev,
                         const void* scales_dev, int block, int K, int N, const void* norm_w_dev, float eps,
                         const void* seq_dev, int salt, void* stream);
/* rms_norm(x, ffn_norm) -> W1 and W3 GEMV -> silu(w1) * w3: llama_cu.cu:1176-1183 */
int lcu_decode_ffn_up(void* out_dev, const void* x_dev, const void* norm_w_dev, const void* w1_dev,
                      const void* w3_dev, const void* s1_dev, const void* s3_dev, int block, int dim,
                      int ffn, float eps, void* stream);
/* rms_norm(x, norm) -> output GEMV: llama_cu.cu:1191-1195 for the single row that is used */
int lcu_decode_logits(void* logits_dev, const void* x_dev, const void* norm_w_dev,
                      const void* wout_dev, const void* sout_dev, int block, int dim, int n_vocab,
                      float eps, void* stream);

/* ---- synthetic tensors (no counterpart in the reference, which reads weights from files):
 * value[i] = fp16(float(S - 262140) * scale), S = sum of the eight 16-bit fields of two chained
 * splitmix64 hashes of (seed, stream_id, i), scale = float(std / sqrt(8 * (65536^2 - 1) / 12)).
 * Integer-exact, so any host restating the recipe gets the same bits. */
int lcu_fill_normal_f16(void* out_dev, size_t n, uint64_t seed, uint64_t stream_id, float std,
                        void* stream);
int lcu_fill_f16(void* out_dev, size_t n, uint16_t bits, void* stream);

/* error_stats, transform.cu:99-150 (launch site 175): out3 = {mean squared difference, largest
 * absolute difference, mean absolute difference} of two fp16 arrays of n elements, as fp32.
 * Deterministic (partials are added in index order, where the reference uses atomics).  Uses the
 * stream's workspace. */
int lcu_error_stats(void* out3_dev, const void* a_dev, const void* b_dev, size_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif
