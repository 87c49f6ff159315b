// Decode-time matrix-vector products (one new token): out[N] = W[N,K] . x[K].
//
// These replace the reference's use of its 16x128x256 tensor-core tile with 15 of 16 rows empty
// (llama_cu.cu:225-285 for fp16 weights, 294-366 for uint8 weights, selected at 1481-1484 and
// 1503-1509).  The work is a pure HBM stream of W, so the kernels are built around that:
//   - x (optionally RMS-normalised first) is staged once per workgroup in LDS as fp16
//   - every wavefront owns R whole rows; each lane issues 16-byte loads (8 halves or 16 codes),
//     several in flight, so one load instruction of a wavefront covers 1 KiB of contiguous W
//   - products accumulate in fp32 per lane, lanes combine with xor shuffles, lane 0 applies the
//     epilogue (residual add, RoPE, SiLU*mul) and rounds once to fp16
// uint8 weights are dequantised in packed fp16: (128 + q/2) is built by bit insertion, minus
// 191.75 gives (q - 127.5)/2 exactly, times 2*scale rounds once, which is bit-for-bit
// fp16((q - 127.5) * scale), the value the reference feeds its tensor cores (287-289, 336-341).
#include "common.hpp"

using namespace lcu;

namespace {

constexpr int GEMV_THREADS = 256;
constexpr int GEMV_WAVES = GEMV_THREADS / WAVE;

// ---- staging of x into LDS -------------------------------------------------------------------
// plain copy
__device__ __forceinline__ void stage_x(half_t* xs, const half_t* __restrict__ x, int K) {
  for (int i = threadIdx.x * 8; i < K; i += GEMV_THREADS * 8) {
    *reinterpret_cast<uint4*>(xs + i) = *reinterpret_cast<const uint4*>(x + i);
  }
  __syncthreads();
}

// rms_norm of the single row x (llama_cu.cu:66-107) written to LDS: fp16(w * fp16(x * rms_inv)),
// the sum of squares associated as the reference's 256-thread reduction.
__device__ __forceinline__ void stage_x_normed(half_t* xs, const half_t* __restrict__ x,
                                               const half_t* __restrict__ norm_w, int K, float eps, float* red) {
  float s = 0.0f;
  for (int i = threadIdx.x; i < K; i += GEMV_THREADS) {
    const float v = (float)x[i];
    s = fmaf(v, v, s);
  }
  const float total = block256_sum_ref_order(s, red);
  const float rms_inv = 1.0f / sqrtf(total / (float)K + eps);
  for (int i = threadIdx.x; i < K; i += GEMV_THREADS) {
    const half_t inner = round_f16((float)x[i] * rms_inv);
    xs[i] = round_f16((float)norm_w[i] * (float)inner);
  }
  __syncthreads();
}

// ---- per-wavefront dot products --------------------------------------------------------------
// fp16 rows.  R rows, U chunks of 512 elements in flight.  K % 8 == 0.
template <int R, int U>
__device__ __forceinline__ void wave_dots_f16(const half_t* const (&rows)[R], const half_t* xs, int K, int lane,
                                              float (&acc)[R]) {
  float a0[R], a1[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    a0[r] = 0.0f;
    a1[r] = 0.0f;
  }
  for (int k0 = lane * 8; k0 < K; k0 += 512 * U) {
    half8_t w[U][R];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k0 + u * 512;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (kk < K) {
          w[u][r] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(rows[r] + kk));
        } else {
          w[u][r] = (half8_t)(0.0f);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k0 + u * 512;
      half8_t xv = (half8_t)(0.0f);
      if (kk < K) {
        xv = *reinterpret_cast<const half8_t*>(xs + kk);
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          a0[r] = fmaf((float)w[u][r][e], (float)xv[e], a0[r]);
          a1[r] = fmaf((float)w[u][r][e + 1], (float)xv[e + 1], a1[r]);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    acc[r] = wave_sum(a0[r] + a1[r]);
  }
}

// two codes (the low two bytes of `two`, spread as [b0, 0, b1, 0]) -> two dequantised halves
__device__ __forceinline__ half2_t dequant2(uint32_t spread, half2_t scale2x) {
  const uint32_t bits = (spread << 2) | 0x58005800u;               // 128 + q/2, exact
  const half2_t t = __builtin_bit_cast(half2_t, bits) - (half2_t)((half_t)191.75f);  // (q - 127.5)/2, exact
  return t * scale2x;                                               // one rounding
}

// uint8 rows with per-block scales.  16 codes per lane per load, U loads in flight.
// K % 16 == 0, block % 16 == 0.
template <int R, int U>
__device__ __forceinline__ void wave_dots_u8(const uint8_t* const (&rows)[R], const half_t* const (&srow)[R],
                                             const half_t* xs, int K, int block, int lane, float (&acc)[R]) {
  float a0[R], a1[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    a0[r] = 0.0f;
    a1[r] = 0.0f;
  }
  for (int k0 = lane * 16; k0 < K; k0 += 1024 * U) {
    uint4_t q[U][R];
    half_t sc[U][R];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k0 + u * 1024;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (kk < K) {
          q[u][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(rows[r] + kk));
          sc[u][r] = srow[r][kk / block];
        } else {
          q[u][r] = (uint4_t)(0u);
          sc[u][r] = (half_t)0.0f;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k0 + u * 1024;
      half8_t x0 = (half8_t)(0.0f), x1 = (half8_t)(0.0f);
      if (kk < K) {
        x0 = *reinterpret_cast<const half8_t*>(xs + kk);
        x1 = *reinterpret_cast<const half8_t*>(xs + kk + 8);
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const half_t s2 = sc[u][r] * (half_t)2.0f;  // exact
        const half2_t s2v = {s2, s2};
        const uint32_t d[4] = {q[u][r][0], q[u][r][1], q[u][r][2], q[u][r][3]};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const half2_t lo = dequant2(__builtin_amdgcn_perm(0u, d[j], 0x0c010c00u), s2v);
          const half2_t hi = dequant2(__builtin_amdgcn_perm(0u, d[j], 0x0c030c02u), s2v);
          const half8_t& xv = (j < 2) ? x0 : x1;
          const int e = (j & 1) * 4;
          a0[r] = fmaf((float)lo.x, (float)xv[e], a0[r]);
          a1[r] = fmaf((float)lo.y, (float)xv[e + 1], a1[r]);
          a0[r] = fmaf((float)hi.x, (float)xv[e + 2], a0[r]);
          a1[r] = fmaf((float)hi.y, (float)xv[e + 3], a1[r]);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    acc[r] = wave_sum(a0[r] + a1[r]);
  }
}

// one interface over both weight formats: R consecutive-or-not rows given by index into a matrix
template <bool U8, int R, int U>
__device__ __forceinline__ void wave_dots(const void* const (&mat)[R], const half_t* const (&scales)[R],
                                          const int (&row)[R], const half_t* xs, int K, int block, int lane,
                                          float (&acc)[R]) {
  if constexpr (U8) {
    const uint8_t* rows[R];
    const half_t* srow[R];
    const int nblk = K / block;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rows[r] = (const uint8_t*)mat[r] + (size_t)row[r] * K;
      srow[r] = scales[r] + (size_t)row[r] * nblk;
    }
    wave_dots_u8<R, U>(rows, srow, xs, K, block, lane, acc);
  } else {
    const half_t* rows[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rows[r] = (const half_t*)mat[r] + (size_t)row[r] * K;
    }
    wave_dots_f16<R, U>(rows, xs, K, lane, acc);
  }
}

// ---- kernels ---------------------------------------------------------------------------------
// out[n] = fp16(dot + beta * out[n]); optional RMS norm of x first.
template <bool U8, int R, int U, bool NORM>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_kernel(half_t* __restrict__ out, const half_t* __restrict__ x,
                                                            const half_t* __restrict__ norm_w, const void* __restrict__ W,
                                                            const half_t* __restrict__ S, int K, int N, int block,
                                                            float beta, float eps) {
  extern __shared__ half_t xs[];
  __shared__ float red[8];
  if constexpr (NORM) {
    stage_x_normed(xs, x, norm_w, K, eps, red);
  } else {
    stage_x(xs, x, K);
  }
  const int lane = threadIdx.x & 63;
  const int first = (blockIdx.x * GEMV_WAVES + (threadIdx.x >> 6)) * R;
  if (first >= N) return;
  const void* mat[R];
  const half_t* sc[R];
  int row[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    mat[r] = W;
    sc[r] = S;
    row[r] = min(first + r, N - 1);
  }
  float acc[R];
  wave_dots<U8, R, U>(mat, sc, row, xs, K, block, lane, acc);
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (first + r < N) {
        float v = acc[r];
        if (beta != 0.0f) {
          v = fmaf(beta, (float)out[first + r], v);
        }
        out[first + r] = round_f16(v);
      }
    }
  }
}

// rms_norm -> [Wq; Wk; Wv] . x -> RoPE on q and k -> q_out, k_cache row, v_cache row.
// A wavefront owns one interleaved pair (rows 2p, 2p+1) of one of the three matrices.
template <bool U8, int U>
__global__ __launch_bounds__(GEMV_THREADS) void decode_qkv_kernel(
    half_t* __restrict__ q_out, half_t* __restrict__ k_row, half_t* __restrict__ v_row, const half_t* __restrict__ x,
    const half_t* __restrict__ norm_w, const void* __restrict__ wq, const void* __restrict__ wk,
    const void* __restrict__ wv, const half_t* __restrict__ sq, const half_t* __restrict__ sk,
    const half_t* __restrict__ sv, int block, int dim, int head_dim, float eps, const float2* __restrict__ rope_row) {
  extern __shared__ half_t xs[];
  __shared__ float red[8];
  stage_x_normed(xs, x, norm_w, dim, eps, red);
  const int lane = threadIdx.x & 63;
  const int pair = blockIdx.x * GEMV_WAVES + (threadIdx.x >> 6);  // 0 .. 3*dim/2
  const int pairs_per_mat = dim / 2;
  if (pair >= 3 * pairs_per_mat) return;
  const int which = pair / pairs_per_mat;
  const int p = pair - which * pairs_per_mat;
  const void* W = which == 0 ? wq : (which == 1 ? wk : wv);
  const half_t* S = which == 0 ? sq : (which == 1 ? sk : sv);
  const void* mat[2] = {W, W};
  const half_t* sc[2] = {S, S};
  const int row[2] = {2 * p, 2 * p + 1};
  float acc[2];
  wave_dots<U8, 2, U>(mat, sc, row, xs, dim, block, lane, acc);
  if (lane == 0) {
    // the GEMV output is rounded to fp16 before RoPE reads it (llama_cu.cu:1144-1153)
    const half_t h0 = round_f16(acc[0]), h1 = round_f16(acc[1]);
    half2_t o;
    if (which == 2) {
      o.x = h0;
      o.y = h1;
      *reinterpret_cast<half2_t*>(v_row + 2 * p) = o;
    } else {
      const float2 cs = rope_row[((2 * p) % head_dim) / 2];
      const float real = (float)h0, imag = (float)h1;
      o.x = round_f16(fmaf(real, cs.x, -(imag * cs.y)));
      o.y = round_f16(fmaf(real, cs.y, imag * cs.x));
      *reinterpret_cast<half2_t*>((which == 0 ? q_out : k_row) + 2 * p) = o;
    }
  }
}

// rms_norm -> W1 . x and W3 . x -> fp16 each -> fp16(silu(w1) * w3).  One output per wavefront.
template <bool U8, int U>
__global__ __launch_bounds__(GEMV_THREADS) void decode_ffn_up_kernel(
    half_t* __restrict__ out, const half_t* __restrict__ x, const half_t* __restrict__ norm_w,
    const void* __restrict__ w1, const void* __restrict__ w3, const half_t* __restrict__ s1,
    const half_t* __restrict__ s3, int block, int dim, int ffn, float eps) {
  extern __shared__ half_t xs[];
  __shared__ float red[8];
  stage_x_normed(xs, x, norm_w, dim, eps, red);
  const int lane = threadIdx.x & 63;
  const int j = blockIdx.x * GEMV_WAVES + (threadIdx.x >> 6);
  if (j >= ffn) return;
  const void* mat[2] = {w1, w3};
  const half_t* sc[2] = {s1, s3};
  const int row[2] = {j, j};
  float acc[2];
  wave_dots<U8, 2, U>(mat, sc, row, xs, dim, block, lane, acc);
  if (lane == 0) {
    const float val = (float)round_f16(acc[0]);  // W1 output, rounded as stored (llama_cu.cu:1180)
    const float gate = (float)round_f16(acc[1]); // W3 output (1181)
    out[j] = round_f16(val / (1.0f + expf(-val)) * gate);  // silu, 533-539
  }
}

template <typename F>
int launch_checked(F&& f) {
  f();
  LCU_LAUNCH_CHECK();
  return LCU_OK;
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
  const size_t lds = (size_t)K * 2;
  if (N >= 8192) {
    const int grid = (N + GEMV_WAVES * 2 - 1) / (GEMV_WAVES * 2);
    gemv_kernel<false, 2, 4, false><<<grid, GEMV_THREADS, lds, st>>>(out, x, nullptr, W, nullptr, K, N, 0, beta, 0.f);
  } else {
    const int grid = (N + GEMV_WAVES - 1) / GEMV_WAVES;
    gemv_kernel<false, 1, 8, false><<<grid, GEMV_THREADS, lds, st>>>(out, x, nullptr, W, nullptr, K, N, 0, beta, 0.f);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int gemv_u8(half_t* out, const half_t* x, const uint8_t* W, const half_t* S, int K, int N, int block, float beta,
            hipStream_t st) {
  const size_t lds = (size_t)K * 2;
  if (N >= 8192) {
    const int grid = (N + GEMV_WAVES * 2 - 1) / (GEMV_WAVES * 2);
    gemv_kernel<true, 2, 4, false><<<grid, GEMV_THREADS, lds, st>>>(out, x, nullptr, W, S, K, N, block, beta, 0.f);
  } else {
    const int grid = (N + GEMV_WAVES - 1) / GEMV_WAVES;
    gemv_kernel<true, 1, 4, false><<<grid, GEMV_THREADS, lds, st>>>(out, x, nullptr, W, S, K, N, block, beta, 0.f);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

}  // namespace lcu

extern "C" {

int lcu_decode_qkv(void* q_out_dev, void* k_cache_dev, void* v_cache_dev, const void* x_dev,
                   const void* norm_w_dev, const void* wq_dev, const void* wk_dev, const void* wv_dev,
                   const void* sq_dev, const void* sk_dev, const void* sv_dev, int block, int dim, int n_heads,
                   int pos, float eps, const void* rope_table_dev, int table_positions, void* stream) {
  LCU_REQUIRE(q_out_dev && k_cache_dev && v_cache_dev && x_dev && norm_w_dev && wq_dev && wk_dev && wv_dev &&
                  rope_table_dev,
              "lcu_decode_qkv: null pointer");
  LCU_REQUIRE(dim > 0 && n_heads > 0 && dim % n_heads == 0 && (dim / n_heads) % 2 == 0 && dim % 16 == 0 &&
                  dim <= 24576,
              "lcu_decode_qkv: bad shape dim %d heads %d", dim, n_heads);
  LCU_REQUIRE(pos >= 0 && pos < table_positions, "lcu_decode_qkv: position %d outside the RoPE table (%d)", pos,
              table_positions);
  const int head_dim = dim / n_heads;
  half_t* k_row = (half_t*)k_cache_dev + (size_t)pos * dim;
  half_t* v_row = (half_t*)v_cache_dev + (size_t)pos * dim;
  const float2* rope_row = (const float2*)rope_table_dev + (size_t)pos * (head_dim / 2);
  const int grid = (3 * dim / 2 + GEMV_WAVES - 1) / GEMV_WAVES;
  const size_t lds = (size_t)dim * 2;
  hipStream_t st = as_stream(stream);
  if (block > 0) {
    int rc = check_quant_args("lcu_decode_qkv", sq_dev, dim, block);
    if (rc) return rc;
    LCU_REQUIRE(sk_dev && sv_dev, "lcu_decode_qkv: quantised weights need scales");
    decode_qkv_kernel<true, 4><<<grid, GEMV_THREADS, lds, st>>>(
        (half_t*)q_out_dev, k_row, v_row, (const half_t*)x_dev, (const half_t*)norm_w_dev, wq_dev, wk_dev, wv_dev,
        (const half_t*)sq_dev, (const half_t*)sk_dev, (const half_t*)sv_dev, block, dim, head_dim, eps, rope_row);
  } else {
    decode_qkv_kernel<false, 4><<<grid, GEMV_THREADS, lds, st>>>(
        (half_t*)q_out_dev, k_row, v_row, (const half_t*)x_dev, (const half_t*)norm_w_dev, wq_dev, wk_dev, wv_dev,
        nullptr, nullptr, nullptr, 0, dim, head_dim, eps, rope_row);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_decode_ffn_up(void* out_dev, const void* x_dev, const void* norm_w_dev, const void* w1_dev,
                      const void* w3_dev, const void* s1_dev, const void* s3_dev, int block, int dim, int ffn,
                      float eps, void* stream) {
  LCU_REQUIRE(out_dev && x_dev && norm_w_dev && w1_dev && w3_dev, "lcu_decode_ffn_up: null pointer");
  LCU_REQUIRE(dim > 0 && dim % 16 == 0 && dim <= 24576 && ffn > 0, "lcu_decode_ffn_up: bad shape dim %d ffn %d", dim,
              ffn);
  const int grid = (ffn + GEMV_WAVES - 1) / GEMV_WAVES;
  const size_t lds = (size_t)dim * 2;
  hipStream_t st = as_stream(stream);
  if (block > 0) {
    int rc = check_quant_args("lcu_decode_ffn_up", s1_dev, dim, block);
    if (rc) return rc;
    LCU_REQUIRE(s3_dev != nullptr, "lcu_decode_ffn_up: quantised weights need scales");
    decode_ffn_up_kernel<true, 4><<<grid, GEMV_THREADS, lds, st>>>(
        (half_t*)out_dev, (const half_t*)x_dev, (const half_t*)norm_w_dev, w1_dev, w3_dev, (const half_t*)s1_dev,
        (const half_t*)s3_dev, block, dim, ffn, eps);
  } else {
    decode_ffn_up_kernel<false, 4><<<grid, GEMV_THREADS, lds, st>>>(
        (half_t*)out_dev, (const half_t*)x_dev, (const half_t*)norm_w_dev, w1_dev, w3_dev, nullptr, nullptr, 0, dim,
        ffn, eps);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_decode_logits(void* logits_dev, const void* x_dev, const void* norm_w_dev, const void* wout_dev,
                      const void* sout_dev, int block, int dim, int n_vocab, float eps, void* stream) {
  LCU_REQUIRE(logits_dev && x_dev && norm_w_dev && wout_dev, "lcu_decode_logits: null pointer");
  LCU_REQUIRE(dim > 0 && dim % 16 == 0 && dim <= 24576 && n_vocab > 0, "lcu_decode_logits: bad shape dim %d vocab %d",
              dim, n_vocab);
  const int grid = (n_vocab + GEMV_WAVES * 2 - 1) / (GEMV_WAVES * 2);
  const size_t lds = (size_t)dim * 2;
  hipStream_t st = as_stream(stream);
  if (block > 0) {
    int rc = check_quant_args("lcu_decode_logits", sout_dev, dim, block);
    if (rc) return rc;
    gemv_kernel<true, 2, 4, true><<<grid, GEMV_THREADS, lds, st>>>(
        (half_t*)logits_dev, (const half_t*)x_dev, (const half_t*)norm_w_dev, wout_dev, (const half_t*)sout_dev, dim,
        n_vocab, block, 0.0f, eps);
  } else {
    gemv_kernel<false, 2, 4, true><<<grid, GEMV_THREADS, lds, st>>>(
        (half_t*)logits_dev, (const half_t*)x_dev, (const half_t*)norm_w_dev, wout_dev, nullptr, dim, n_vocab, 0, 0.0f,
        eps);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

}  // extern "C"
