/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the arithmetic of eiz/llama.cu's
 * inference path.  Nothing that ships (the HIP library, the host model code, the
 * command line tools) may include, link or call this file; only tests/, the smoke
 * check and the cpu_baseline leg of bench.py do, and only as the checker.
 *
 * Every function cites the reference lines it restates (paths relative to the
 * reference checkout).  fp16 values travel as uint16_t bit patterns.
 *
 * Parity status of each function (what pins it):
 *   orc_quantize_absmax_u8 / orc_dequantize_absmax_u8 : IEEE-only arithmetic, pinned by the
 *       hand-computed known-answer block, the exhaustive 65536-input sweep against numpy
 *       float32/float16 and the absmax/code-range invariants (tests/test_oracle_quant.py).
 *   orc_matmul_nt[_u8] : pinned by float64 brute force, identity / one-hot / beta special cases;
 *       flavour 2 (the order of this repository's HIP kernels) also by independent numpy
 *       restatements of the lane / wavefront partition, of the matrix cores' steps of eight and of
 *       the dispatcher's cut of K (orc_gemm_plan).
 *   orc_dot2_f32_f16, orc_mfma_f32_f16 : what v_dot2_f32_f16 and the matrix cores of gfx950 return;
 *       not part of the reference (its tensor cores keep their own order).  Pinned by outputs
 *       measured on the GPU (tests/golden/dot2_gfx950.npz, mfma_gfx950.npz, written by the probe
 *       programs beside them), by an independent numpy restatement and by closed forms.
 *   orc_attention_decode_kernel_order, orc_attention_prefill_kernel_order,
 *   orc_softmax_logits_kernel_order : the reference's attention and softmax arithmetic with the
 *       sums in the HIP kernels' order; pinned by independent numpy restatements, against the
 *       reference-ordered functions (last-bit agreement) and float64.
 *   exponentials (softmax, SiLU): the reference calls CUDA's expf, whose last bits no host library
 *       reproduces; restated with IEEE operations only (exp_ieee, within one ulp, pinned against
 *       float64 exp in tests/test_oracle_ops.py) so that host and GPU agree bit for bit.
 *   orc_rms_norm, orc_rotary, orc_softmax_rows, orc_silu_mul, orc_matmul_qk, orc_matmul_qkv,
 *   orc_embed[_u8], orc_argmax_first : pinned by closed forms and float64 restatements written
 *       independently in numpy (tests/test_oracle_ops.py).
 *   orc_error_stats, orc_sample_row : pinned by closed forms (tests/test_oracle_ops.py).
 *   orc_context_next_token : pinned by an independent numpy float64 forward pass on a tiny model
 *       (tolerance) and by the prefill-then-decode == longer-prefill invariant.
 * The reference holds no golden vectors for any of these (it has no tests), and its CUDA sources
 * cannot be compiled here, so no oracle/_ref build exists.
 */
#ifndef LLAMA_ORACLE_H
#define LLAMA_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- seeded synthetic tensors (not from the reference: the shared test-input recipe) ---- */
/* value[i] = fp16_rn( float(S - 262140) * scale ), S = sum of the eight 16-bit fields of
 * splitmix64(key + i) and splitmix64 of that, key = splitmix64(seed ^ stream * 0xD1B54A32D192ED03),
 * scale = float(std / sqrt(8 * (65536^2 - 1) / 12)).  Integer-exact, so host and GPU agree bit for bit. */
void orc_fill_normal_f16(uint16_t* out, size_t n, uint64_t seed, uint64_t stream, float std);

/* ---- int8 absmax block quantiser: transform.cu:28-72 and 74-87 ---- */
void orc_quantize_absmax_u8(uint8_t* codes, uint16_t* scales, const uint16_t* in, size_t rows,
                            size_t cols, int block);
void orc_dequantize_absmax_u8(uint16_t* out, const uint16_t* scales, const uint8_t* codes,
                              size_t rows, size_t cols, int block);

/* ---- matmul: out[M,N] = lhs[M,K] * rhs[N,K]^T + beta * out ----
 * flavour 0: llama_cu.cu:111-122 (and 125-145 for u8), one sequential fp32 sum per output.
 * flavour 1: the tensor-core kernels llama_cu.cu:150-220, 225-285, 294-366: fp16 operands
 *            (u8 weights first rounded to fp16 by dequantize_absmax_one, 287-289), fp32
 *            accumulation in an order the hardware fixes; restated with 16 interleaved partial
 *            sums and a pairwise tree.
 * flavour 2: as flavour 1, except that a single row (M == 1) is summed in the order of this
 *            repository's own decode GEMV kernels (lane-strided partial sums, a pairwise tree over
 *            the 64 lanes, the four wavefronts in order; see dot_gemv_order in oracle.cpp), and a
 *            context created with it also takes the attention and the logits softmax of a
 *            one-token call in the order of the HIP kernels.  Any fp32 order is as good a restatement
 *            of the reference's tensor-core sums as another (their order is the hardware's); this
 *            one lets a decode step be compared with the GPU bit for bit (fp16 and uint8 weights;
 *            the uint8 kernels pair their products through v_dot2_f32_f16, restated from
 *            measured samples: dot2_f32_f16 in oracle.cpp) instead of within a tolerance.  Pinned by the same float64 / identity / one-hot checks as the
 *            other flavours (tests/test_oracle_ops.py). */
void orc_matmul_nt(uint16_t* out, const uint16_t* lhs, const uint16_t* rhs, int M, int K, int N,
                   float beta, int flavour);
void orc_matmul_nt_u8(uint16_t* out, const uint16_t* lhs, const uint8_t* codes,
                      const uint16_t* scales, int M, int K, int N, int block, float beta,
                      int flavour);

/* ---- element-wise and row kernels ---- */
/* llama_cu.cu:66-107 */
void orc_rms_norm(uint16_t* out, const uint16_t* in, const uint16_t* weights, int rows, int cols,
                  float eps);
/* llama_cu.cu:368-389 */
void orc_rotary(uint16_t* out, const uint16_t* in, int rows, int cols, int n_heads, int pos_offset,
                float theta);
/* llama_cu.cu:400-428; out is [n_heads][n_new][T] with row stride T */
void orc_matmul_qk(uint16_t* out, const uint16_t* q, const uint16_t* k, int n_new, int T, int dim,
                   int n_heads, int start_pos);
/* llama_cu.cu:433-499; rows = product of all leading dimensions */
void orc_softmax_rows(uint16_t* out, const uint16_t* in, int rows, int w, float temp);
/* llama_cu.cu:511-531 */
void orc_matmul_qkv(uint16_t* out, const uint16_t* p, const uint16_t* v, int n_new, int T, int dim,
                    int n_heads);
/* llama_cu.cu:533-539 */
void orc_silu_mul(uint16_t* out, const uint16_t* a, const uint16_t* b, size_t size);
/* llama_cu.cu:32-44 and 46-62 */
void orc_embed(uint16_t* out, const int16_t* ids, int n_ids, int dim, const uint16_t* table);
void orc_embed_u8(uint16_t* out, const int16_t* ids, int n_ids, int dim, const uint8_t* table,
                  const uint16_t* scales, int block);
/* llama_cu.cu:1205-1209: first maximum of fp16 values compared as float */
int orc_argmax_first(const uint16_t* probs, int n);

/* Sampler the reference leaves commented out (llama_cu.cu:1202-1203: std::discrete_distribution
 * over the fp16 probabilities): index i is drawn with probability p[i] / sum(p).  Restated in
 * integers so that it has one answer: weight[i] = p[i] * 2^24 (exact for every fp16 in [0, 1];
 * negative and NaN count 0, larger values saturate at 2^24 * 65504), total = sum of the weights,
 * r = floor(random * total / 2^64), result = the smallest i whose running sum of weights exceeds r
 * (0 when total is 0).  Pinned by closed forms: one-hot rows, the 1:3 threshold at random = 2^62,
 * zero weights never drawn, monotone in random, frequencies of a known distribution. */
int orc_sample_row(const uint16_t* probs, int n, uint64_t random);
/* the 64 random bits of the `step`-th sampled token of a context seeded with `seed`: output
 * `step` (from 0) of the splitmix64 generator started at `seed` */
uint64_t orc_step_random(uint64_t seed, uint64_t step);

/* error_stats, transform.cu:99-150: out3 = {mean of d^2, max |d|, mean |d|}, d = a[i] - b[i] in
 * fp32, sums carried in double (the reference adds fp32 partials with atomics in arrival order,
 * so its own result is only defined to fp32 summation accuracy).  Pinned by closed forms:
 * identical arrays -> 0, a constant offset -> {c^2, c, c}, one differing element. */
void orc_error_stats(float* out3, const uint16_t* a, const uint16_t* b, size_t n);

/* e^x as every softmax and SiLU of this oracle takes it: IEEE operations only (the reference calls
 * CUDA's expf, llama_cu.cu:463, 497, 537); pinned against float64 exp to one ulp. */
void orc_exp_f32(float* out, const float* in, size_t n);

/* Flavour 2 for a product that the HIP host code launches together with n_mats - 1 others of the same
 * shape (Wq, Wk, Wv: 3; W1, W3: 2): the dispatcher may then cut K another way.  codes == NULL: fp16
 * weights in rhs; else uint8 codes with scales.  M == 1 takes the GEMV order. */
void orc_matmul_nt_kernel_order(uint16_t* out, const uint16_t* lhs, const uint16_t* rhs, const uint8_t* codes,
                                const uint16_t* scales, int M, int K, int N, int block, float beta, int n_mats);

/* The cut of K that csrc/gemm.hip takes for a product of M > 1 rows on a 256-CU device:
 * returns ks * 1000 + splits (see plan_gemm in oracle.cpp). */
int orc_gemm_plan(int M, int K, int N, int u8, int block, int n_mats);

/* out[i] = the accumulator c[i] after K / 8 steps of eight products a[i][k] * b[i][k] (fp16 bit
 * patterns) as the gfx950 matrix cores take them: K = 16 is v_mfma_f32_32x32x16_f16 for one output
 * element, K = 32 v_mfma_f32_16x16x32_f16.  Restated from measured samples, see mfma_step8. */
void orc_mfma_f32_f16(float* out, const uint16_t* a, const uint16_t* b, const float* c, size_t n, int K);

/* out[i] = v_dot2_f32_f16(a[2i..2i+1], b[2i..2i+1], c[i]) as gfx950 computes it (a, b: fp16 bit
 * patterns); restated from measured samples, see dot2_f32_f16 in oracle.cpp. */
void orc_dot2_f32_f16(float* out, const uint16_t* a, const uint16_t* b, const float* c, size_t n);
/* Attention of one new token (q [dim], the first T rows of k (rotated) and v [T][dim], head_dim 128)
 * and softmax with temperature over one row of n logits (n a multiple of 8 up to 32768): the
 * arithmetic of llama_cu.cu:400-428, 433-499, 511-531 with the sums taken in the order of this
 * repository's HIP kernels (what a context of matmul flavour 2 uses for one-token calls).  Pinned
 * against orc_matmul_qk / orc_softmax_rows / orc_matmul_qkv within fp32 summation accuracy. */
void orc_attention_decode_kernel_order(uint16_t* out, const uint16_t* q, const uint16_t* k, const uint16_t* v, int T,
                                       int dim, int n_heads);
/* lcu_attention with n_new > 1 in the order of csrc/attention.hip (head_dim 128): scores and
 * weighted sums as chains of matrix-core steps, the row softmax summed as its wavefront sums it. */
void orc_attention_prefill_kernel_order(uint16_t* out, const uint16_t* q, const uint16_t* k, const uint16_t* v, int n_new,
                                        int T, int start_pos, int dim, int n_heads);

void orc_softmax_logits_kernel_order(uint16_t* out, const uint16_t* in, int n, float temp);

/* ---- whole model: llama_cu.cu:882-1210 with seeded random weights instead of files ---- */
typedef struct orc_model orc_model;
typedef struct orc_context orc_context;

/* q_type 0 = fp16, 1 = uint8 (weights generated in fp16, then quantised with block `qblock`).
 * Weight streams: tok_embeddings 1, output 2, layer l: 16+16*l + {wq 0, wk 1, wv 2, wo 3, w1 4,
 * w2 5, w3 6}; every matrix ~N(0, weight_std); all norm weights are 1.0. */
orc_model* orc_model_create(int dim, int multiple_of, int n_heads, int n_layers, int n_vocab,
                            float norm_eps, int q_type, int qblock, uint64_t seed,
                            float weight_std);
void orc_model_destroy(orc_model*);
int orc_model_ffn_dim(const orc_model*);
/* borrowed pointers into the model for cross-checks: which = stream id as above, scales may be
 * NULL for fp16 models */
const void* orc_model_tensor(const orc_model*, uint64_t stream, const uint16_t** scales);

/* literal_rope 1 = keep K unrotated and re-rotate all cached rows on every call, exactly as
 * llama_cu.cu:1150-1153; 0 = rotate once when the row is written (same bits, cheaper). */
orc_context* orc_context_create(orc_model*, int context_len, float temperature, int matmul_flavour,
                                int literal_rope);
void orc_context_destroy(orc_context*);
void orc_context_clear(orc_context*);
int orc_context_start_pos(const orc_context*);
/* llama_cu.cu:1073-1210.  Optional outputs (may be NULL): hidden = residual stream after the last
 * layer [n][dim]; logits = fp16 logits of the last row [n_vocab]; probs = softmax(temp) [n_vocab]. */
int orc_context_next_token(orc_context*, const int16_t* tokens, int n, uint16_t* hidden,
                           uint16_t* logits, uint16_t* probs);
/* borrowed KV rows of one layer, [context_len][dim]; K is returned rotated */
void orc_context_kv(orc_context*, int layer, uint16_t* k_rot, uint16_t* v, int T);

int orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
