// Decode-time matrix-vector products (one new token): out[N] = W[N,K] . x[K].
//
// These replace the reference's use of its 16x128x256 tensor-core tile with 15 of 16 rows empty
// (llama_cu.cu:225-285 for fp16 weights, 294-366 for uint8 weights, selected at 1481-1484 and
// 1503-1509).  The work is a pure HBM stream of W, so the kernels are built around that:
//   - one small workgroup (4 wavefronts) per "task" of R whole rows of W; the wavefronts split K
//     between them, so a workgroup reads its rows as one contiguous run, and the hardware
//     dispatcher balances the many uniform workgroups over the 256 compute units
//   - each lane issues 16-byte loads (8 halves or 16 codes), U*R of them per batch, requested
//     before anything else happens in the workgroup (before x is staged or normalised), and the
//     next batch is requested before the current one is consumed (uint8 rows of up to five
//     batches: all of them at once, see with_u8_batches)
//   - each lane loads the pieces of x (or of the norm weights) that match its weights along with
//     them; when x must be RMS-normalised first, every workgroup requests x before its weights
//     (loads return in request order), stages it in LDS, reduces the sum of squares there while
//     the weights are on their way and normalises its pieces in registers (global load
//     instructions per workgroup are what this prologue must keep few)
//   - products accumulate in fp32 per lane, lanes combine with xor shuffles, wavefronts through
//     LDS, thread 0 applies the epilogue (residual add, RoPE, SiLU*mul) and rounds once to fp16
// uint8 weights are dequantised in packed fp16 to bit-for-bit fp16((q - 127.5) * scale), the value
// the reference feeds its tensor cores (287-289, 336-341): see dequant2_fma / dequant2.  The
// products then go through v_dot2_f32_f16 (two multiply-adds per instruction, fp32 accumulate;
// the instruction aligns and cuts its three addends in a way of its own, which the oracle's
// kernel-order flavour restates from measured samples): the dequantisation arithmetic, not HBM,
// is what bounds this kernel on large matrices.
#include "common.hpp"

#include <type_traits>

using namespace lcu;

namespace {

constexpr int GEMV_THREADS = 256;
constexpr int GEMV_WAVES = GEMV_THREADS / WAVE;

// RMS statistics of x inside a GEMV workgroup.  Loads come back in the order they were requested,
// so the pieces of x are requested first (load), before the workgroup's weights: the norm is then
// worked out while the weights are still on their way instead of after them.  reduce() copies x to
// LDS and takes the sum of squares from there in the reference's order (llama_cu.cu:75-100: thread
// t owns elements t, t+256, ...; block256_sum_ref_order), then 1/sqrt(mean + eps) with IEEE
// operations.  Every thread returns the same value; xs holds the raw x afterwards.  XN 16-byte
// pieces per thread cover K <= 2048 * XN; xs holds 2048 * XN halves.
// keeps the memory requests written above it above the ones written below it
__device__ __forceinline__ void issue_order_fence() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

template <int XN>
struct x_stage_t {
  uint4_t v[XN > 0 ? XN : 1];
  __device__ __forceinline__ void load(const half_t* x, int K) {
    // the pointer passes through an empty asm so that these loads are ordinary ones to the
    // compiler: loads from a const __restrict__ kernel argument may cross issue_order_fence()
    asm volatile("" : "+s"(x));
    typedef const __attribute__((address_space(1))) uint4_t* global_ptr_t;
#pragma unroll
    for (int j = 0; j < XN; ++j) {
      const int i = min((int)(threadIdx.x + j * GEMV_THREADS) * 8, K - 8);
      v[j] = *(global_ptr_t)(x + i);
    }
  }
  __device__ __forceinline__ float reduce(half_t* xs, int K, float eps, float* red) const {
#pragma unroll
    for (int j = 0; j < XN; ++j) {
      // unconditional (xs holds 2048 * XN halves): a conditional store lets the compiler move the
      // load down to it, behind the weights
      *reinterpret_cast<uint4_t*>(xs + (threadIdx.x + j * GEMV_THREADS) * 8) = v[j];
    }
    __syncthreads();
    float s = 0.0f;
    for (int i = threadIdx.x; i < K; i += GEMV_THREADS) {
      const float e = (float)xs[i];
      s = fmaf(e, e, s);
    }
    const float total = block256_sum_ref_order(s, red);
    return 1.0f / sqrtf(total / (float)K + eps);
  }
};

// rms_norm applied to 8 elements in registers: fp16(w * fp16(x * rms_inv)), llama_cu.cu:103-106.
// x * rms_inv is rounded to fp32 and then to fp16 (two at a time, v_cvt_pk_f16_f32); the product
// with the weight is one packed fp16 multiply: the fp32 product of two halves is exact, so
// rounding it to fp16 is what the fp16 multiply itself does.  Three instructions per element
// instead of seven: every workgroup of the logits GEMV normalises the whole row.
__device__ __forceinline__ half8_t normed(half8_t x, half8_t w, float rms_inv) {
  typedef float float2_t __attribute__((ext_vector_type(2)));
  half8_t r;
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    float2_t p;
    p.x = (float)x[e] * rms_inv;
    p.y = (float)x[e + 1] * rms_inv;
    asm("" : "+v"(p));  // keeps the multiply and the conversion apart (see round_f16)
    const half2_t inner = __builtin_convertvector(p, half2_t);
    const half2_t ww = {w[e], w[e + 1]};
    const half2_t res = ww * inner;
    r[e] = res.x;
    r[e + 1] = res.y;
  }
  return r;
}

// two codes spread as [b0, 0, b1, 0] -> two dequantised halves; exact for every scale
__device__ __forceinline__ half2_t dequant2(uint32_t spread, half2_t scale2x) {
  const uint32_t bits = (spread << 2) | 0x58005800u;                                  // 128 + q/2, exact
  const half2_t t = __builtin_bit_cast(half2_t, bits) - (half2_t)((half_t)191.75f);   // (q - 127.5)/2, exact
  return t * scale2x;                                                                 // one rounding
}

// The same value in three operations instead of four: bytes [b0, 0x64, b1, 0x64] are the halves
// 1024 + q; minus 1152 is q - 128, exact; fma(q - 128, s, s/2) forms (q - 127.5) * s exactly and
// rounds once.  Needs s/2 to be exact, i.e. not a subnormal scale with an odd last bit: the caller
// checks that and falls back to dequant2.
__device__ __forceinline__ half2_t dequant2_fma(uint32_t biased, half2_t scale, half2_t half_scale) {
  const half2_t q128 = __builtin_bit_cast(half2_t, biased) - (half2_t)((half_t)1152.0f);
  return __builtin_elementwise_fma(q128, scale, half_scale);
}

// ---- one batch in registers: U chunks of R rows of W (16 bytes per lane each), with the matching
// pieces of x and, when x is to be normalised, of the norm weights ------------------------------
template <bool U8, int R, int U, bool NORM>
struct batch_t {
  static constexpr int VEC = U8 ? 16 : 8;          // elements of K per lane per chunk
  static constexpr int CHUNK = VEC * WAVE;         // elements of K covered by one load of a wavefront
  static constexpr int XV = VEC / 8;
  uint4_t w[U][R];                                 // 8 halves or 16 codes
  half_t sc[U8 ? U : 1][U8 ? R : 1];
  half8_t xr[NORM ? 1 : U][NORM ? 1 : XV];        // x itself, unless it is read (raw) from LDS later
  half8_t nw[NORM ? U : 1][NORM ? XV : 1];

  // Loads are unconditional: a chunk past the end of K is read from the last in-range position
  // instead (a predicated load becomes a branch, and the waits the compiler puts around branches
  // serialise the loads); fma() gives such a chunk a zero x.
  // block_shift: log2 of the quantisation block when that is a power of two (a shift instead of
  // the dozen instructions of an integer division per load), else -1
  __device__ __forceinline__ void load(const uint8_t* const (&rows)[R], const half_t* const (&srow)[R],
                                       const half_t* __restrict__ x, const half_t* __restrict__ norm_w, int kb, int K,
                                       int block, int block_shift, int lane) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = min((kb * U + u) * CHUNK + lane * VEC, K - VEC);
      int sidx = 0;
      if constexpr (U8) {
        sidx = block_shift >= 0 ? kk >> block_shift : kk / block;
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        w[u][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(rows[r] + (size_t)kk * (U8 ? 1 : 2)));
        if constexpr (U8) {
          sc[u][r] = srow[r][sidx];
        }
      }
#pragma unroll
      for (int j = 0; j < XV; ++j) {
        if constexpr (NORM) {
          nw[u][j] = *reinterpret_cast<const half8_t*>(norm_w + kk + 8 * j);
        } else {
          xr[u][j] = *reinterpret_cast<const half8_t*>(x + kk + 8 * j);
        }
      }
    }
  }

  // xs: raw x in LDS (NORM only); kb, K, lane as in load().  A piece past the end of K (its load
  // was redirected to the last in-range position) is skipped: per wavefront when the whole chunk
  // lies past K, per lane otherwise.
  __device__ __forceinline__ void fma(const half_t* xs, float rms_inv, int kb, int K, int lane, float (&a0)[R],
                                      float (&a1)[R]) const {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = (kb * U + u) * CHUNK + lane * VEC;
      if ((kb * U + u) * CHUNK >= K) {
        continue;
      }
      if (kk < K) {
        half8_t xv[XV];
#pragma unroll
        for (int j = 0; j < XV; ++j) {
          if constexpr (NORM) {
            xv[j] = normed(*reinterpret_cast<const half8_t*>(xs + kk + 8 * j), nw[u][j], rms_inv);
          } else {
            xv[j] = xr[u][j];
          }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if constexpr (U8) {
            // 16 codes as four words; x as eight words of two halves.  Codes 0,1 of a word go with
            // x word 2j into a0, codes 2,3 with x word 2j + 1 into a1 (v_dot2_f32_f16).
            const uint4_t xw0 = __builtin_bit_cast(uint4_t, xv[0]), xw1 = __builtin_bit_cast(uint4_t, xv[XV - 1]);
            const uint32_t xw[8] = {xw0[0], xw0[1], xw0[2], xw0[3], xw1[0], xw1[1], xw1[2], xw1[3]};
            const half_t sv = sc[u][r];
            const half_t hv = sv * (half_t)0.5f;
            if (hv + hv == sv) {  // s/2 exact (every normal scale): 3-operation dequantisation
              const half2_t s1v = {sv, sv}, h1v = {hv, hv};
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                // selector bytes 4..7 pick from the first operand (0x64 in every byte), 0..3 from the codes
                const half2_t lo = dequant2_fma(__builtin_amdgcn_perm(0x64646464u, w[u][r][j], 0x04010400u), s1v, h1v);
                const half2_t hi = dequant2_fma(__builtin_amdgcn_perm(0x64646464u, w[u][r][j], 0x04030402u), s1v, h1v);
                a0[r] = __builtin_amdgcn_fdot2(lo, __builtin_bit_cast(half2_t, xw[2 * j]), a0[r], false);
                a1[r] = __builtin_amdgcn_fdot2(hi, __builtin_bit_cast(half2_t, xw[2 * j + 1]), a1[r], false);
              }
            } else {  // a subnormal scale with an odd last bit: the four-operation form, same products
              const half_t s2 = sv * (half_t)2.0f;  // exact
              const half2_t s2v = {s2, s2};
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const half2_t lo = dequant2(__builtin_amdgcn_perm(0u, w[u][r][j], 0x0c010c00u), s2v);
                const half2_t hi = dequant2(__builtin_amdgcn_perm(0u, w[u][r][j], 0x0c030c02u), s2v);
                a0[r] = __builtin_amdgcn_fdot2(lo, __builtin_bit_cast(half2_t, xw[2 * j]), a0[r], false);
                a1[r] = __builtin_amdgcn_fdot2(hi, __builtin_bit_cast(half2_t, xw[2 * j + 1]), a1[r], false);
              }
            }
          } else {
            const half8_t wv = __builtin_bit_cast(half8_t, w[u][r]);
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
              a0[r] = fmaf((float)wv[e], (float)xv[0][e], a0[r]);
              a1[r] = fmaf((float)wv[e + 1], (float)xv[0][e + 1], a1[r]);
            }
          }
        }
      }
    }
  }
};

// ---- the streaming loop of one workgroup -------------------------------------------------------
// Tasks: struct with
//   void rows(int task, const uint8_t* (&rows)[R], const half_t* (&srow)[R]) const;   row base pointers
//   void finish(int task, const float (&acc)[R]) const;           epilogue, called by thread 0 only
// The workgroup's wavefronts take the K chunks of the task's rows round-robin: batch b of
// wavefront w covers chunks (b * WAVES + w) * U .. + U.  begin() requests the first batch (weights,
// x, norm weights), or with NB > 0 all NB batches of the rows; the caller may then reduce the norm
// statistics; run() does the rest (NB == 0: a loop that requests one batch ahead; NB > 0: the
// batches summed in the same order, K <= NB * WAVES * U * CHUNK) and ends with the
// cross-wavefront sum.
template <bool U8, int R, int U, bool NORM, class Tasks, int NB = 0>
struct stream_t {
  using batch = batch_t<U8, R, U, NORM>;
  const Tasks tk;  // by value: a reference member kept the struct in scratch memory in some instantiations
  const half_t* x;
  const half_t* norm_w;
  int K, block, block_shift, lane, wave, task, n_batches;
  const uint8_t* rows[R];
  const half_t* srow[R];
  batch held[NB > 0 ? NB : 1];  // NB > 0: every batch of the rows (n_batches <= NB), all requested by begin()

  __device__ __forceinline__ stream_t(const Tasks& t, const half_t* x_, const half_t* norm_w_, int K_, int block_,
                                      int task_)
      : tk(t), x(x_), norm_w(norm_w_), K(K_), block(block_),
        block_shift(block_ > 0 && (block_ & (block_ - 1)) == 0 ? __builtin_ctz(block_) : -1), lane(threadIdx.x & 63),
        wave(threadIdx.x >> 6),
        task(task_), n_batches((K_ + batch::CHUNK * U * GEMV_WAVES - 1) / (batch::CHUNK * U * GEMV_WAVES)) {}

  __device__ __forceinline__ void begin() {
    tk.rows(task, rows, srow);
#pragma unroll
    for (int b = 0; b < (NB > 0 ? NB : 1); ++b) {
      held[b].load(rows, srow, x, norm_w, b * GEMV_WAVES + wave, K, block, block_shift, lane);
    }
  }

  // xs: raw x in LDS when NORM; part: GEMV_WAVES * R floats of LDS
  __device__ __forceinline__ void run(const half_t* xs, float rms_inv, float* part) {
    float a0[R], a1[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      a0[r] = 0.0f;
      a1[r] = 0.0f;
    }
    if constexpr (NB > 0) {
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        held[b].fma(xs, rms_inv, b * GEMV_WAVES + wave, K, lane, a0, a1);
      }
    } else {
      for (int b = 0; b < n_batches; ++b) {
        batch nxt;
        if (b + 1 < n_batches) {
          nxt.load(rows, srow, x, norm_w, (b + 1) * GEMV_WAVES + wave, K, block, block_shift, lane);
        }
        held[0].fma(xs, rms_inv, b * GEMV_WAVES + wave, K, lane, a0, a1);
        held[0] = nxt;
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float s = wave_sum(a0[r] + a1[r]);
      if (lane == 0) {
        part[wave * R + r] = s;
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      float acc[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        acc[r] = 0.0f;
#pragma unroll
        for (int w = 0; w < GEMV_WAVES; ++w) {
          acc[r] += part[w * R + r];
        }
      }
      tk.finish(task, acc);
    }
  }
};

template <bool U8>
__device__ __forceinline__ const uint8_t* row_ptr(const void* W, size_t row, int K) {
  return (const uint8_t*)W + row * (size_t)K * (U8 ? 1 : 2);
}

// ---- tasks --------------------------------------------------------------------------------------
// plain rows: out[n] = fp16(dot + beta * out[n])
template <bool U8, int R>
struct plain_tasks {
  const void* W;
  const half_t* S;
  half_t* out;
  int K, N, nblk;
  float beta;
  __device__ __forceinline__ void rows(int task, const uint8_t* (&rows)[R], const half_t* (&srow)[R]) const {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = min(task * R + r, N - 1);
      rows[r] = row_ptr<U8>(W, n, K);
      srow[r] = U8 ? S + (size_t)n * nblk : nullptr;
    }
  }
  __device__ __forceinline__ void finish(int task, const float (&acc)[R]) const {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = task * R + r;
      if (n < N) {
        float v = acc[r];
        if (beta != 0.0f) {
          v = fmaf(beta, (float)out[n], v);  // llama_cu.cu:279
        }
        out[n] = round_f16(v);
      }
    }
  }
};

// rows of a product whose result is added to the residual row and then normalised (W2 of one layer,
// the attention norm of the next: llama_cu.cu:1185, 1129): x[n] = fp16(dot + x[n]) leaves as a
// {two halves, epoch} word for the workgroup that normalises the row (decode_proj_norm_kernel)
template <bool U8, int R>
struct proj_norm_tasks {
  const void* W;
  const half_t* S;
  const half_t* x_old;
  uint64_t* words;
  int K, N, nblk;
  uint32_t epoch;
  __device__ __forceinline__ void rows(int task, const uint8_t* (&rows)[R], const half_t* (&srow)[R]) const {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = min(task * R + r, N - 1);
      rows[r] = row_ptr<U8>(W, n, K);
      srow[r] = U8 ? S + (size_t)n * nblk : nullptr;
    }
  }
  __device__ __forceinline__ void finish(int task, const float (&acc)[R]) const {
    static_assert(R % 2 == 0, "pairs of rows");
#pragma unroll
    for (int r = 0; r < R; r += 2) {
      const int n = task * R + r;
      if (n < N) {  // N is even
        const half_t h0 = round_f16(fmaf(1.0f, (float)x_old[n], acc[r]));          // llama_cu.cu:279 with beta = 1
        const half_t h1 = round_f16(fmaf(1.0f, (float)x_old[n + 1], acc[r + 1]));
        const uint64_t word = ((uint64_t)epoch << 32) | ((uint32_t)__builtin_bit_cast(unsigned short, h1) << 16) |
                              __builtin_bit_cast(unsigned short, h0);
        __hip_atomic_store(words + n / 2, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
};

// One of Wq / Wk / Wv (chosen per workgroup by the kernel): a task is PAIRS interleaved pairs (rows
// 2p, 2p+1) of that matrix; RoPE on q and k (llama_cu.cu:381-387), results to q_out / the caches'
// row for this position
template <bool U8, int PAIRS>
struct qkv_tasks {
  const void* W;
  const half_t* S;
  half_t* dst;             // q_out, or the K / V cache row of this position
  const float2* rope_row;  // nullptr for V
  int dim, head_dim, nblk, first_task;
  __device__ __forceinline__ void rows(int task, const uint8_t* (&rows)[2 * PAIRS],
                                       const half_t* (&srow)[2 * PAIRS]) const {
    const int p0 = (task - first_task) * PAIRS;
#pragma unroll
    for (int r = 0; r < 2 * PAIRS; ++r) {
      rows[r] = row_ptr<U8>(W, 2 * p0 + r, dim);
      srow[r] = U8 ? S + (size_t)(2 * p0 + r) * nblk : nullptr;
    }
  }
  __device__ __forceinline__ void finish(int task, const float (&acc)[2 * PAIRS]) const {
#pragma unroll
    for (int i = 0; i < PAIRS; ++i) {
      const int p = (task - first_task) * PAIRS + i;
      // the GEMV output is rounded to fp16 before RoPE reads it (llama_cu.cu:1144-1153)
      const half_t h0 = round_f16(acc[2 * i]), h1 = round_f16(acc[2 * i + 1]);
      half2_t o;
      if (rope_row == nullptr) {
        o.x = h0;
        o.y = h1;
      } else {
        const float2 cs = rope_row[((2 * p) % head_dim) / 2];
        const float real = (float)h0, imag = (float)h1;
        o.x = round_f16(fmaf(real, cs.x, -(imag * cs.y)));
        o.y = round_f16(fmaf(real, cs.y, imag * cs.x));
      }
      *reinterpret_cast<half2_t*>(dst + 2 * p) = o;
    }
  }
};

// PAIRS times: W1 row j and W3 row j -> fp16 each -> fp16(silu(w1) * w3)  (llama_cu.cu:1180-1183, 533-539)
template <bool U8, int PAIRS>
struct ffn_up_tasks {
  const void *w1, *w3;
  const half_t *s1, *s3;
  half_t* out;
  int dim, nblk, ffn;
  __device__ __forceinline__ void rows(int task, const uint8_t* (&rows)[2 * PAIRS],
                                       const half_t* (&srow)[2 * PAIRS]) const {
#pragma unroll
    for (int i = 0; i < PAIRS; ++i) {
      const int j = min(task * PAIRS + i, ffn - 1);
      rows[2 * i] = row_ptr<U8>(w1, j, dim);
      rows[2 * i + 1] = row_ptr<U8>(w3, j, dim);
      srow[2 * i] = U8 ? s1 + (size_t)j * nblk : nullptr;
      srow[2 * i + 1] = U8 ? s3 + (size_t)j * nblk : nullptr;
    }
  }
  __device__ __forceinline__ void finish(int task, const float (&acc)[2 * PAIRS]) const {
#pragma unroll
    for (int i = 0; i < PAIRS; ++i) {
      const int j = task * PAIRS + i;
      if (j < ffn) {
        const float val = (float)round_f16(acc[2 * i]);
        const float gate = (float)round_f16(acc[2 * i + 1]);
        out[j] = round_f16(val / (1.0f + exp_ieee(-val)) * gate);
      }
    }
  }
};

// ---- kernels -------------------------------------------------------------------------------------
// one workgroup per task (blockIdx.x)
// XN > 0: x is RMS-normalised first, from XN 16-byte pieces per thread (x_stage_t)
template <bool U8, int R, int U, int XN, int NB = 0>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_kernel(half_t* __restrict__ out, const half_t* __restrict__ x,
                                                            const half_t* __restrict__ norm_w, const void* __restrict__ W,
                                                            const half_t* __restrict__ S, int K, int N, int block,
                                                            float beta, float eps) {
  extern __shared__ half_t xs[];  // 2048 * XN halves
  __shared__ float red[8];
  __shared__ float part[GEMV_WAVES * R];
  constexpr bool NORM = XN > 0;
  plain_tasks<U8, R> tk{W, S, out, K, N, U8 ? K / block : 0, beta};
  stream_t<U8, R, U, NORM, plain_tasks<U8, R>, NB> st(tk, x, norm_w, K, block, blockIdx.x);
  float rms_inv = 1.0f;
  if constexpr (NORM) {
    x_stage_t<XN> xp;
    xp.load(x, K);
    issue_order_fence();
    st.begin();
    issue_order_fence();
    rms_inv = xp.reduce(xs, K, eps, red);
  } else {
    st.begin();
  }
  st.run(xs, rms_inv, part);
}

template <bool U8, int U, int XN, int PAIRS, int NB = 0>
__global__ __launch_bounds__(GEMV_THREADS) void decode_qkv_kernel(
    half_t* __restrict__ q_out, half_t* __restrict__ k_row, half_t* __restrict__ v_row, const half_t* __restrict__ x,
    const half_t* __restrict__ norm_w, const void* __restrict__ wq, const void* __restrict__ wk,
    const void* __restrict__ wv, const half_t* __restrict__ sq, const half_t* __restrict__ sk,
    const half_t* __restrict__ sv, int block, int dim, int head_dim, float eps, const float2* __restrict__ rope_row,
    const int* __restrict__ pos_dev, int max_pos) {
  extern __shared__ half_t xs[];
  __shared__ float red[8];
  __shared__ float part[GEMV_WAVES * 2 * PAIRS];
  if (pos_dev) {  // position kept on the device (graph replay): the row pointers arrive as bases
    const int pos = min(max(*pos_dev, 0), max_pos);
    k_row += (size_t)pos * dim;
    v_row += (size_t)pos * dim;
    rope_row += (size_t)pos * (head_dim / 2);
  }
  // one task per workgroup, so the matrix is chosen here, once, from the kernel arguments (a
  // per-task choice inside the task struct made the compiler index the struct in scratch memory)
  const int tasks_per_matrix = dim / 2 / PAIRS;
  const int which = blockIdx.x / tasks_per_matrix;
  const void* W = which == 0 ? wq : (which == 1 ? wk : wv);
  const half_t* S = which == 0 ? sq : (which == 1 ? sk : sv);
  half_t* dst = which == 0 ? q_out : (which == 1 ? k_row : v_row);
  qkv_tasks<U8, PAIRS> tk{W, S, dst, which == 2 ? nullptr : rope_row, dim, head_dim, U8 ? dim / block : 0,
                          which * tasks_per_matrix};
  constexpr bool NORM = XN > 0;
  stream_t<U8, 2 * PAIRS, U, NORM, qkv_tasks<U8, PAIRS>, NB> st(tk, x, norm_w, dim, block, blockIdx.x);
  float rms_inv = 1.0f;
  if constexpr (NORM) {
    x_stage_t<XN> xp;
    xp.load(x, dim);
    issue_order_fence();
    st.begin();
    issue_order_fence();
    rms_inv = xp.reduce(xs, dim, eps, red);
  } else {
    st.begin();
  }
  st.run(xs, rms_inv, part);
}

template <bool U8, int U, int XN, int PAIRS, int NB = 0>
__global__ __launch_bounds__(GEMV_THREADS) void decode_ffn_up_kernel(
    half_t* __restrict__ out, const half_t* __restrict__ x, const half_t* __restrict__ norm_w,
    const void* __restrict__ w1, const void* __restrict__ w3, const half_t* __restrict__ s1,
    const half_t* __restrict__ s3, int block, int dim, int ffn, float eps) {
  extern __shared__ half_t xs[];
  __shared__ float red[8];
  __shared__ float part[GEMV_WAVES * 2 * PAIRS];
  ffn_up_tasks<U8, PAIRS> tk{w1, w3, s1, s3, out, dim, U8 ? dim / block : 0, ffn};
  constexpr bool NORM = XN > 0;
  stream_t<U8, 2 * PAIRS, U, NORM, ffn_up_tasks<U8, PAIRS>, NB> st(tk, x, norm_w, dim, block, blockIdx.x);
  float rms_inv = 1.0f;
  if constexpr (NORM) {
    x_stage_t<XN> xp;
    xp.load(x, dim);
    issue_order_fence();
    st.begin();
    issue_order_fence();
    rms_inv = xp.reduce(xs, dim, eps, red);
  } else {
    st.begin();
  }
  st.run(xs, rms_inv, part);
}

// x += lhs . W^T followed by norm_out = rms_norm(x) in one launch.  Workgroups 0 .. n_tasks - 1 are
// the GEMV of gemv_kernel (R rows each, same sums); each hands its rows of the new x over as
// {two halves, epoch} words written through to memory.  One more workgroup, the last of the grid,
// asks for the N / 2 words until all of them carry this launch's epoch (a value no earlier launch
// left there: step counter << 10 | salt), then writes the row and its norm (rmsnorm_kernel's
// arithmetic).  It is resident while the last GEMV workgroups run, so the norm costs the hand-over
// and its own arithmetic instead of a launch; its wait is bounded and counts itself when it runs out.
// Diagnostic builds only (-DLCU_PHASE_TIMELINE): thread 0 of every workgroup of the launch notes the
// 100 MHz real-time counter when it starts, when its first batch has been summed, and when its result
// is stored (the follower: start, every word in LDS, norm written, and the sum of squares known); one row per launch (by salt) and
// workgroup, copied out by lcu_debug_timeline_read_proj.  Nothing of this exists in the ordinary build.
#ifdef LCU_PHASE_TIMELINE
constexpr int PTL_POINTS = 4, PTL_LAUNCHES = 64, PTL_GROUPS = 4096;
static __device__ uint64_t proj_timeline[PTL_LAUNCHES * PTL_GROUPS * PTL_POINTS];
#define PTL_MARK(point)                                                                                          \
  do {                                                                                                           \
    if (threadIdx.x == 0 && blockIdx.x < PTL_GROUPS) {                                                           \
      proj_timeline[((ptl_launch & (PTL_LAUNCHES - 1)) * PTL_GROUPS + blockIdx.x) * PTL_POINTS + (point)] =      \
          __builtin_amdgcn_s_memrealtime();                                                                      \
    }                                                                                                            \
  } while (0)
#else
#define PTL_MARK(point) \
  do {                  \
  } while (0)
#endif

constexpr int FOLLOW_SPIN_LIMIT = 1 << 16;
constexpr int FOLLOW_PIECES = 8;  // 16-byte requests per thread: N <= 8192

template <bool U8, int R, int U, int NB = 0>
__global__ __launch_bounds__(GEMV_THREADS) void decode_proj_norm_kernel(
    half_t* __restrict__ x_io, half_t* __restrict__ norm_out, const half_t* __restrict__ lhs,
    const void* __restrict__ W, const half_t* __restrict__ S, const half_t* __restrict__ norm_w, int K, int N, int block,
    float eps, uint64_t* __restrict__ words, const uint32_t* __restrict__ seq_dev, uint32_t epoch,
    uint32_t* __restrict__ timeouts) {
  extern __shared__ half_t xs[];  // N halves: the follower's copy of the row
  __shared__ __attribute__((aligned(16))) float red[8];
  __shared__ float part[GEMV_WAVES * R];
#ifdef LCU_PHASE_TIMELINE
  const uint32_t ptl_launch = epoch >> 1;  // the salt of a W2 launch is 2 * layer + 1
#endif
  PTL_MARK(0);
  epoch = (epoch | (*seq_dev << 10)) & 0x7fffffffu;
  const int n_tasks = (N + R - 1) / R;
  if ((int)blockIdx.x < n_tasks) {
    proj_norm_tasks<U8, R> tk{W, S, x_io, words, K, N, U8 ? K / block : 0, epoch};
    stream_t<U8, R, U, false, proj_norm_tasks<U8, R>, NB> st(tk, lhs, nullptr, K, block, blockIdx.x);
    st.begin();
    st.run(xs, 1.0f, part);
    PTL_MARK(2);
    return;
  }
  const int tid = threadIdx.x;
  // the norm weights of this thread's pieces, requested before the wait (N <= 8192: four pieces)
  half8_t nwp[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = (tid + GEMV_THREADS * j) * 8;
    nwp[j] = i < N ? *reinterpret_cast<const half8_t*>(norm_w + i) : (half8_t)(0.0f);
  }
  // two neighbouring words per request, four requests per statement, and one such group of four at a
  // time (asked for until it is fresh, then put into LDS: sixteen registers for the words instead of
  // thirty-two, which keeps the whole kernel at the GEMV workgroups' register count and so at eight
  // workgroups per compute unit; with 80 registers a quarter of the 2048 workgroups of W2 started
  // only when others had finished).  A piece past the row reads the row's first words instead and
  // is ignored.  The waits of a wavefront share one budget of polls.
  int spins = 0;
  bool gave_up = false;
#pragma unroll
  for (int j = 0; j < FOLLOW_PIECES; j += 4) {
    if (GEMV_THREADS * j * 2 >= N / 2) continue;  // the whole group lies past the row (the same for every thread)
    uint4_t four[4];
    const int w0 = (tid + GEMV_THREADS * j) * 2, w1 = w0 + GEMV_THREADS * 2, w2 = w1 + GEMV_THREADS * 2,
              w3 = w2 + GEMV_THREADS * 2;
    const int wi[4] = {w0, w1, w2, w3};
    while (true) {
      load_word_pairs_device_scope(four, words + (w0 < N / 2 ? w0 : 0), words + (w1 < N / 2 ? w1 : 0),
                                   words + (w2 < N / 2 ? w2 : 0), words + (w3 < N / 2 ? w3 : 0));
      bool stale = false;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (wi[e] < N / 2) stale |= four[e][1] != epoch || four[e][3] != epoch;
      }
      if (__builtin_amdgcn_ballot_w64(stale) == 0 || gave_up) break;
      if (++spins > FOLLOW_SPIN_LIMIT) {
        if ((tid & 63) == 0) atomicAdd(timeouts, 1u);
        gave_up = true;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (wi[e] < N / 2) {
        uint32_t* dst = reinterpret_cast<uint32_t*>(xs + 2 * wi[e]);
        dst[0] = four[e][0];
        dst[1] = four[e][2];
      }
    }
  }
  __syncthreads();
  PTL_MARK(1);
  // rms_norm, llama_cu.cu:66-107, as rmsnorm_kernel: thread t owns elements t, t + 256, ...
  float s = 0.0f;
  {
    // eight LDS reads in flight at a time; the additions stay in ascending order
    int i = tid;
    for (; i + 7 * GEMV_THREADS < N; i += 8 * GEMV_THREADS) {
      float e[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) e[u] = (float)xs[i + u * GEMV_THREADS];
#pragma unroll
      for (int u = 0; u < 8; ++u) s = fmaf(e[u], e[u], s);
    }
    for (; i < N; i += GEMV_THREADS) {
      const float e = (float)xs[i];
      s = fmaf(e, e, s);
    }
  }
  const float total = block256_sum_ref_order_dpp(s, red);
  const float rms_inv = 1.0f / sqrtf(total / (float)N + eps);
  PTL_MARK(3);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = (tid + GEMV_THREADS * j) * 8;
    if (i >= N) continue;
    const half8_t xv = *reinterpret_cast<const half8_t*>(xs + i);
    const half8_t wv = nwp[j];
    half8_t r;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const half_t inner = round_f16((float)xv[e] * rms_inv);
      r[e] = round_f16((float)wv[e] * (float)inner);
    }
    *reinterpret_cast<half8_t*>(x_io + i) = xv;
    *reinterpret_cast<half8_t*>(norm_out + i) = r;
  }
  PTL_MARK(2);
}

// calls f with the number of 16-byte pieces of x per thread (x_stage_t) that covers dim <= 24576
template <class F>
void with_x_pieces(int dim, F&& f) {
  if (dim <= 4096) {
    f(std::integral_constant<int, 2>{});
  } else if (dim <= 8192) {
    f(std::integral_constant<int, 4>{});
  } else {
    f(std::integral_constant<int, 12>{});
  }
}

// uint8 rows at U = 1: a batch of the workgroup covers 4096 codes of a row.  Rows of two to five
// batches have every batch requested at once (NB: same chunks on the same wavefronts in the same
// order as the loop, so the same sums), longer ones keep the loop (NB = 0): 6656 x 17920 uint8
// 23.6 -> 22.0 us, 5120 x 13824 15.5 -> 14.2, 4096 x 11008 10.9 -> 10.2, 8192^2 13.8 -> 13.3,
// 17920 x 6656 20.8 -> 20.5, variants alternating in one process.  (fp16 rows gain at some lengths
// and lose at others, 4096 x 11008 16.6 against 16.1 us, and keep the loop.)
template <class F>
void with_u8_batches(int K, F&& f) {
  const int nb = (K + 4095) / 4096;
  switch (nb) {
    case 2: f(std::integral_constant<int, 2>{}); break;
    case 3: f(std::integral_constant<int, 3>{}); break;
    case 4: f(std::integral_constant<int, 4>{}); break;
    case 5: f(std::integral_constant<int, 5>{}); break;
    default: f(std::integral_constant<int, 0>{}); break;
  }
}

// with_x_pieces and with_u8_batches for a row of dim codes: f(pieces of x per thread, NB)
template <class F>
void with_u8_row_plan(int dim, F&& f) {
  using std::integral_constant;
  if (dim <= 4096) {
    f(integral_constant<int, 2>{}, integral_constant<int, 0>{});
  } else if (dim <= 8192) {
    f(integral_constant<int, 4>{}, integral_constant<int, 2>{});
  } else if (dim <= 12288) {
    f(integral_constant<int, 12>{}, integral_constant<int, 3>{});
  } else if (dim <= 16384) {
    f(integral_constant<int, 12>{}, integral_constant<int, 4>{});
  } else if (dim <= 20480) {
    f(integral_constant<int, 12>{}, integral_constant<int, 5>{});
  } else {
    f(integral_constant<int, 12>{}, integral_constant<int, 0>{});
  }
}

int check_quant_args(const char* who, const void* scales, int K, int block) {
  LCU_REQUIRE(scales != nullptr, "%s: quantised weights need scales", who);
  LCU_REQUIRE(block >= 16 && block % 16 == 0 && K % block == 0 && K % 16 == 0,
              "%s: K %d / block %d unsupported (block multiple of 16 dividing K)", who, K, block);
  return LCU_OK;
}

}  // namespace

namespace lcu {

// M == 1 paths of lcu_gemm_f16_nt / lcu_gemm_f16u8_nt
int gemv_f16(half_t* out, const half_t* x, const half_t* W, int K, int N, float beta, hipStream_t st) {
  if (K > 4096) {
    gemv_kernel<false, 2, 2, 0><<<(N + 1) / 2, GEMV_THREADS, 0, st>>>(out, x, nullptr, W, nullptr, K, N, 0, beta, 0.f);
  } else {
    gemv_kernel<false, 1, 2, 0><<<N, GEMV_THREADS, 0, st>>>(out, x, nullptr, W, nullptr, K, N, 0, beta, 0.f);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int gemv_u8(half_t* out, const half_t* x, const uint8_t* W, const half_t* S, int K, int N, int block, float beta,
            hipStream_t st) {
  // four rows per workgroup where that still gives most compute units eight workgroups: x (as many
  // bytes as two rows of codes) is then fetched half as often (30B shapes: W1/W3 41.5 -> 38.9 us,
  // the logits 216 MB in 34 us); at N = 4096 it would leave half the workgroup slots empty
  with_u8_batches(K, [&](auto nb) {
    if (N >= 6144) {
      gemv_kernel<true, 4, 1, 0, decltype(nb)::value><<<(N + 3) / 4, GEMV_THREADS, 0, st>>>(out, x, nullptr, W, S, K, N,
                                                                                          block, beta, 0.f);
    } else {
      gemv_kernel<true, 2, 1, 0, decltype(nb)::value><<<(N + 1) / 2, GEMV_THREADS, 0, st>>>(out, x, nullptr, W, S, K, N,
                                                                                          block, beta, 0.f);
    }
  });
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

}  // namespace lcu

extern "C" {

int lcu_decode_qkv(void* q_out_dev, void* k_cache_dev, void* v_cache_dev, const void* x_dev,
                   const void* norm_w_dev, const void* wq_dev, const void* wk_dev, const void* wv_dev,
                   const void* sq_dev, const void* sk_dev, const void* sv_dev, int block, int dim, int n_heads,
                   int pos, const void* pos_dev, float eps, const void* rope_table_dev, int table_positions,
                   void* stream) {
  LCU_REQUIRE(q_out_dev && k_cache_dev && v_cache_dev && x_dev && wq_dev && wk_dev && wv_dev &&
                  rope_table_dev,
              "lcu_decode_qkv: null pointer");
  LCU_REQUIRE(dim > 0 && n_heads > 0 && dim % n_heads == 0 && (dim / n_heads) % 2 == 0 && dim % 16 == 0 &&
                  dim <= 24576,
              "lcu_decode_qkv: bad shape dim %d heads %d", dim, n_heads);
  if (pos_dev) {
    pos = 0;  // the kernel adds the device-side position to the base pointers
  }
  LCU_REQUIRE(pos >= 0 && pos < table_positions, "lcu_decode_qkv: position %d outside the RoPE table (%d)", pos,
              table_positions);
  const int head_dim = dim / n_heads;
  half_t* k_row = (half_t*)k_cache_dev + (size_t)pos * dim;
  half_t* v_row = (half_t*)v_cache_dev + (size_t)pos * dim;
  const float2* rope_row = (const float2*)rope_table_dev + (size_t)pos * (head_dim / 2);
  const int grid = 3 * dim / 2;
  hipStream_t st = as_stream(stream);
  if (block > 0) {
    int rc = check_quant_args("lcu_decode_qkv", sq_dev, dim, block);
    if (rc) return rc;
    LCU_REQUIRE(sk_dev && sv_dev, "lcu_decode_qkv: quantised weights need scales");
    if (norm_w_dev) {
      with_u8_row_plan(dim, [&](auto xn, auto nb) {
        decode_qkv_kernel<true, 1, decltype(xn)::value, 1, decltype(nb)::value>
            <<<grid, GEMV_THREADS, decltype(xn)::value * 4096, st>>>(
            (half_t*)q_out_dev, k_row, v_row, (const half_t*)x_dev, (const half_t*)norm_w_dev, wq_dev, wk_dev, wv_dev,
            (const half_t*)sq_dev, (const half_t*)sk_dev, (const half_t*)sv_dev, block, dim, head_dim, eps, rope_row,
            (const int*)pos_dev, table_positions - 1);
      });
    } else {
      with_u8_batches(dim, [&](auto nb) {
        decode_qkv_kernel<true, 1, 0, 2, decltype(nb)::value><<<grid / 2, GEMV_THREADS, 0, st>>>(
            (half_t*)q_out_dev, k_row, v_row, (const half_t*)x_dev, nullptr, wq_dev, wk_dev, wv_dev,
            (const half_t*)sq_dev, (const half_t*)sk_dev, (const half_t*)sv_dev, block, dim, head_dim, eps, rope_row,
            (const int*)pos_dev, table_positions - 1);
      });
    }
  } else {
    if (norm_w_dev) {
      with_x_pieces(dim, [&](auto xn) {
        decode_qkv_kernel<false, 2, decltype(xn)::value, 1><<<grid, GEMV_THREADS, decltype(xn)::value * 4096, st>>>(
            (half_t*)q_out_dev, k_row, v_row, (const half_t*)x_dev, (const half_t*)norm_w_dev, wq_dev, wk_dev, wv_dev,
            nullptr, nullptr, nullptr, 0, dim, head_dim, eps, rope_row, (const int*)pos_dev, table_positions - 1);
      });
    } else {
      decode_qkv_kernel<false, 2, 0, 1><<<grid, GEMV_THREADS, 0, st>>>(
          (half_t*)q_out_dev, k_row, v_row, (const half_t*)x_dev, nullptr, wq_dev, wk_dev, wv_dev, nullptr, nullptr,
          nullptr, 0, dim, head_dim, eps, rope_row, (const int*)pos_dev, table_positions - 1);
    }
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_decode_proj_norm(void* x_io_dev, void* norm_out_dev, const void* lhs_dev, const void* w_dev,
                         const void* scales_dev, int block, int K, int N, const void* norm_w_dev, float eps,
                         const void* seq_dev, int salt, void* stream) {
  LCU_REQUIRE(x_io_dev && norm_out_dev && lhs_dev && w_dev && norm_w_dev && seq_dev, "lcu_decode_proj_norm: null pointer");
  LCU_REQUIRE(K > 0 && K % 16 == 0 && N > 0 && N % 8 == 0 && N <= 2048 * FOLLOW_PIECES / 2,
              "lcu_decode_proj_norm: bad shape K %d N %d (N a multiple of 8, at most %d)", K, N, 2048 * FOLLOW_PIECES / 2);
  LCU_REQUIRE(salt >= 0 && salt < 1024, "lcu_decode_proj_norm: salt %d outside 0..1023", salt);
  hipStream_t st = as_stream(stream);
  const workspace_t ws = workspace_for(st);
  if (ws.sync == nullptr) return set_error(LCU_E_NOINIT, "lcu_decode_proj_norm: lcu_init has not run on this device");
  uint64_t* words = reinterpret_cast<uint64_t*>(ws.sync + SYNC_EXCHANGE) + EXCH_PROJ;
  uint32_t* timeouts = ws.sync + SYNC_TIMEOUTS;
  const size_t lds = (size_t)N * 2;
  if (block > 0) {
    int rc = check_quant_args("lcu_decode_proj_norm", scales_dev, K, block);
    if (rc) return rc;
    // four rows per workgroup (x fetched half as often) where the rows are long; short rows (Wo) finish sooner
    // as twice as many workgroups of two
    with_u8_batches(K, [&](auto nb) {
      if (N >= 6144 && K >= 8192) {
        decode_proj_norm_kernel<true, 4, 1, decltype(nb)::value><<<(N + 3) / 4 + 1, GEMV_THREADS, lds, st>>>(
            (half_t*)x_io_dev, (half_t*)norm_out_dev, (const half_t*)lhs_dev, w_dev, (const half_t*)scales_dev,
            (const half_t*)norm_w_dev, K, N, block, eps, words, (const uint32_t*)seq_dev, (uint32_t)salt, timeouts);
      } else {
        decode_proj_norm_kernel<true, 2, 1, decltype(nb)::value><<<(N + 1) / 2 + 1, GEMV_THREADS, lds, st>>>(
            (half_t*)x_io_dev, (half_t*)norm_out_dev, (const half_t*)lhs_dev, w_dev, (const half_t*)scales_dev,
            (const half_t*)norm_w_dev, K, N, block, eps, words, (const uint32_t*)seq_dev, (uint32_t)salt, timeouts);
      }
    });
  } else {
    decode_proj_norm_kernel<false, 2, 2><<<(N + 1) / 2 + 1, GEMV_THREADS, lds, st>>>(
        (half_t*)x_io_dev, (half_t*)norm_out_dev, (const half_t*)lhs_dev, w_dev, nullptr, (const half_t*)norm_w_dev, K, N,
        0, eps, words, (const uint32_t*)seq_dev, (uint32_t)salt, timeouts);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_decode_ffn_up(void* out_dev, const void* x_dev, const void* norm_w_dev, const void* w1_dev,
                      const void* w3_dev, const void* s1_dev, const void* s3_dev, int block, int dim, int ffn,
                      float eps, void* stream) {
  LCU_REQUIRE(out_dev && x_dev && w1_dev && w3_dev, "lcu_decode_ffn_up: null pointer");
  LCU_REQUIRE(dim > 0 && dim % 16 == 0 && dim <= 24576 && ffn > 0, "lcu_decode_ffn_up: bad shape dim %d ffn %d", dim,
              ffn);
  const int grid = ffn;
  hipStream_t st = as_stream(stream);
  if (block > 0) {
    int rc = check_quant_args("lcu_decode_ffn_up", s1_dev, dim, block);
    if (rc) return rc;
    LCU_REQUIRE(s3_dev != nullptr, "lcu_decode_ffn_up: quantised weights need scales");
    if (norm_w_dev) {
      with_u8_row_plan(dim, [&](auto xn, auto nb) {
        decode_ffn_up_kernel<true, 1, decltype(xn)::value, 1, decltype(nb)::value>
            <<<grid, GEMV_THREADS, decltype(xn)::value * 4096, st>>>(
            (half_t*)out_dev, (const half_t*)x_dev, (const half_t*)norm_w_dev, w1_dev, w3_dev, (const half_t*)s1_dev,
            (const half_t*)s3_dev, block, dim, ffn, eps);
      });
    } else {
      with_u8_batches(dim, [&](auto nb) {
        decode_ffn_up_kernel<true, 1, 0, 2, decltype(nb)::value><<<(grid + 1) / 2, GEMV_THREADS, 0, st>>>(
            (half_t*)out_dev, (const half_t*)x_dev, nullptr, w1_dev, w3_dev, (const half_t*)s1_dev,
            (const half_t*)s3_dev, block, dim, ffn, eps);
      });
    }
  } else {
    if (norm_w_dev) {
      with_x_pieces(dim, [&](auto xn) {
        decode_ffn_up_kernel<false, 2, decltype(xn)::value, 1><<<grid, GEMV_THREADS, decltype(xn)::value * 4096, st>>>(
            (half_t*)out_dev, (const half_t*)x_dev, (const half_t*)norm_w_dev, w1_dev, w3_dev, nullptr, nullptr, 0, dim,
            ffn, eps);
      });
    } else {
      decode_ffn_up_kernel<false, 2, 0, 1><<<grid, GEMV_THREADS, 0, st>>>(
          (half_t*)out_dev, (const half_t*)x_dev, nullptr, w1_dev, w3_dev, nullptr, nullptr, 0, dim, ffn, eps);
    }
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_decode_logits(void* logits_dev, const void* x_dev, const void* norm_w_dev, const void* wout_dev,
                      const void* sout_dev, int block, int dim, int n_vocab, float eps, void* stream) {
  LCU_REQUIRE(logits_dev && x_dev && norm_w_dev && wout_dev, "lcu_decode_logits: null pointer");
  LCU_REQUIRE(dim > 0 && dim % 16 == 0 && dim <= 24576 && n_vocab > 0, "lcu_decode_logits: bad shape dim %d vocab %d",
              dim, n_vocab);
  const int grid = (n_vocab + 1) / 2;
  hipStream_t st = as_stream(stream);
  if (block > 0) {
    int rc = check_quant_args("lcu_decode_logits", sout_dev, dim, block);
    if (rc) return rc;
    with_u8_row_plan(dim, [&](auto xn, auto nb) {
      gemv_kernel<true, 2, 1, decltype(xn)::value, decltype(nb)::value>
          <<<grid, GEMV_THREADS, decltype(xn)::value * 4096, st>>>(
          (half_t*)logits_dev, (const half_t*)x_dev, (const half_t*)norm_w_dev, wout_dev, (const half_t*)sout_dev, dim,
          n_vocab, block, 0.0f, eps);
    });
  } else {
    with_x_pieces(dim, [&](auto xn) {
      gemv_kernel<false, 2, 2, decltype(xn)::value><<<grid, GEMV_THREADS, decltype(xn)::value * 4096, st>>>(
          (half_t*)logits_dev, (const half_t*)x_dev, (const half_t*)norm_w_dev, wout_dev, nullptr, dim, n_vocab, 0,
          0.0f, eps);
    });
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

#ifdef LCU_PHASE_TIMELINE
// diagnostic builds only: clears (out_host == NULL) or copies out the timeline of the W2 launches of
// lcu_decode_proj_norm (odd salts), uint64[64 launches][4096 workgroups][4 points] of the 100 MHz counter
int lcu_debug_timeline_read_proj(void* out_host, size_t bytes) {
  void* dev = nullptr;
  LCU_HIP(hipGetSymbolAddress(&dev, HIP_SYMBOL(proj_timeline)));
  LCU_HIP(hipDeviceSynchronize());
  if (out_host == nullptr) {
    LCU_HIP(hipMemset(dev, 0, sizeof(uint64_t) * PTL_LAUNCHES * PTL_GROUPS * PTL_POINTS));
  } else {
    LCU_REQUIRE(bytes <= sizeof(uint64_t) * PTL_LAUNCHES * PTL_GROUPS * PTL_POINTS,
                "lcu_debug_timeline_read_proj: too many bytes");
    LCU_HIP(hipMemcpy(out_host, dev, bytes, hipMemcpyDeviceToHost));
  }
  return LCU_OK;
}
#endif

}  // extern "C"
