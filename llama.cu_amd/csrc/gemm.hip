// Prefill matrix products on the gfx950 matrix cores: out[M,N] = lhs[M,K] * W[N,K]^T + beta*out.
//
// These replace matmul_nt_wmma_128x64x64 (llama_cu.cu:150-220) and, for uint8 weights,
// matmul_nt_wmma_16x128x256_fp16u8 at M > 1 (294-366).  Both operands are K-contiguous, which is
// the natural operand order of v_mfma_f32_32x32x16_f16: every lane feeds 8 consecutive k of one
// row of lhs (A) and of one row of W (B).
//
//   - 256 threads = 4 wavefronts in a 2x2 grid; block tile BM x BN, K step 64
//   - global -> registers -> LDS with two LDS buffers and two register stages: while the matrix
//     cores work on K step t, step t+1 waits in registers and step t+2 is being fetched; LDS rows
//     are padded by 16 bytes so the 16-byte operand reads of 16 neighbouring lanes fall in
//     distinct banks
//   - the K loop carries no vector address arithmetic and no predication (see load_tile)
//   - uint8 weights are dequantised between the global load and the LDS store, so each weight is
//     converted once per block tile, to exactly fp16((q - 127.5) * scale) (287-289)
//   - block index -> tile mapping keeps the tiles that share a slice of W on one XCD (one L2)
//   - no padding rows: rows >= M and columns >= N are masked instead of the reference's zeroed
//     "gutter" (llama_cu.h:236-242)
#include "common.hpp"

using namespace lcu;

namespace lcu {
int gemv_f16(half_t* out, const half_t* x, const half_t* W, int K, int N, float beta, hipStream_t st);
int gemv_u8(half_t* out, const half_t* x, const uint8_t* W, const half_t* S, int K, int N, int block, float beta,
            hipStream_t st);
}  // namespace lcu

namespace {

constexpr int BK = 64;
constexpr int LDK = BK + 8;  // halves per LDS row
constexpr int THREADS = 256;
constexpr int NUM_XCD = 8;

__device__ __forceinline__ half2_t dequant2(uint32_t spread, half2_t scale2x) {
  const uint32_t bits = (spread << 2) | 0x58005800u;                                  // 128 + q/2
  const half2_t t = __builtin_bit_cast(half2_t, bits) - (half2_t)((half_t)191.75f);   // (q - 127.5)/2
  return t * scale2x;                                                                 // one rounding
}

// KTAIL: K is not a multiple of BK, so the last K step is partly out of range and must be zeroed
// (costs selects in the loop; every model shape takes the KTAIL = false instantiation).
template <int BM, int BN, bool U8, bool KTAIL>
__global__ __launch_bounds__(THREADS, 2) void gemm_kernel(half_t* __restrict__ out, const half_t* __restrict__ A,
                                                          const void* __restrict__ Wv, const half_t* __restrict__ S,
                                                          int M, int K, int N, int block, float beta, int tiles_m,
                                                          int tiles_n) {
  constexpr int TM = BM / 64;  // 32x32 MFMA tiles per wavefront along M
  constexpr int TN = BN / 64;
  constexpr int A_CHUNKS = BM * BK / 8 / THREADS;                  // 16-byte chunks per thread
  constexpr int B_CHUNKS = U8 ? BN * BK / 16 / THREADS : BN * BK / 8 / THREADS;
  static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1, "tile too small for 256 threads");

  __shared__ __attribute__((aligned(16))) half_t As[2][BM * LDK];
  __shared__ __attribute__((aligned(16))) half_t Bs[2][BN * LDK];

  // XCD-aware tile order: hardware deals consecutive workgroups round-robin to the 8 XCDs, so
  // give each XCD one contiguous run of the M-fastest tile sequence.
  const int nb = tiles_m * tiles_n;
  const int bid = blockIdx.x;
  const int q = nb / NUM_XCD, r = nb % NUM_XCD;
  const int xcd = bid % NUM_XCD, idx = bid / NUM_XCD;
  const int logical = xcd * q + min(xcd, r) + idx;
  const int tm = logical % tiles_m, tn = logical / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = (wave & 1) * (BM / 2), wn = (wave >> 1) * (BN / 2);
  const int nblk = U8 ? K / block : 0;

  // Per-thread byte offsets of its chunks from the operand bases; they do not change over the K
  // loop, which only advances a uniform base, so the loop carries no vector address arithmetic.
  // Rows past M or N are clamped to the last row: their products land in accumulator rows and
  // columns that the epilogue never stores, so no zero fill is needed for them.
  uint32_t a_off[A_CHUNKS], b_off[B_CHUNKS], s_off[U8 ? B_CHUNKS : 1];
  int a_k[A_CHUNKS], b_k[B_CHUNKS];
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    const int c = tid + i * THREADS;
    a_k[i] = (c & 7) * 8;
    a_off[i] = ((uint32_t)min(m0 + (c >> 3), M - 1) * (uint32_t)K + a_k[i]) * 2u;
  }
#pragma unroll
  for (int i = 0; i < B_CHUNKS; ++i) {
    const int c = tid + i * THREADS;
    if constexpr (U8) {
      const uint32_t row = (uint32_t)min(n0 + (c >> 2), N - 1);
      b_k[i] = (c & 3) * 16;
      b_off[i] = row * (uint32_t)K + b_k[i];
      s_off[i] = row * (uint32_t)nblk;
    } else {
      b_k[i] = (c & 7) * 8;
      b_off[i] = ((uint32_t)min(n0 + (c >> 3), N - 1) * (uint32_t)K + b_k[i]) * 2u;
    }
  }
  const char* Ab = (const char*)A;
  const char* Wb = (const char*)Wv;

  // one K step of both operands in registers, as loaded from global memory
  struct stage_t {
    half8_t ra[A_CHUNKS];
    half8_t rb[U8 ? 1 : B_CHUNKS];
    uint4_t rq[U8 ? B_CHUNKS : 1];
    half_t rs[U8 ? B_CHUNKS : 1];
    int k0;
  };

  // Unconditional loads: a predicated load becomes a branch, and branches make the compiler wait
  // for every outstanding load before it issues the next ones.  With KTAIL the k offset is
  // clamped into range here and the chunk is zeroed when it is stored to LDS.
  auto load_tile = [&](stage_t& st, int k0) {
    st.k0 = k0;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      int kk = k0;
      if constexpr (KTAIL) kk = min(k0, K - 8 - a_k[i]);
      st.ra[i] = *reinterpret_cast<const half8_t*>(Ab + (ptrdiff_t)kk * 2 + a_off[i]);
    }
    if constexpr (U8) {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; ++i) {
        int kk = k0;
        if constexpr (KTAIL) kk = min(k0, K - 16 - b_k[i]);
        st.rq[i] = *reinterpret_cast<const uint4_t*>(Wb + (ptrdiff_t)kk + b_off[i]);
        st.rs[i] = S[s_off[i] + (uint32_t)(kk + b_k[i]) / (uint32_t)block];
      }
    } else {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; ++i) {
        int kk = k0;
        if constexpr (KTAIL) kk = min(k0, K - 8 - b_k[i]);
        st.rb[i] = *reinterpret_cast<const half8_t*>(Wb + (ptrdiff_t)kk * 2 + b_off[i]);
      }
    }
  };

  auto store_tile = [&](const stage_t& st, int buf) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * THREADS;
      half8_t v = st.ra[i];
      if constexpr (KTAIL) v = (st.k0 + a_k[i] < K) ? v : (half8_t)(0.0f);
      *reinterpret_cast<half8_t*>(&As[buf][(c >> 3) * LDK + (c & 7) * 8]) = v;
    }
    if constexpr (U8) {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; ++i) {
        const int c = tid + i * THREADS;
        half_t s2 = st.rs[i] * (half_t)2.0f;
        if constexpr (KTAIL) s2 = (st.k0 + b_k[i] < K) ? s2 : (half_t)0.0f;  // zero scale: zero weights
        const half2_t s2v = {s2, s2};
        half2_t d[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          d[2 * j] = dequant2(__builtin_amdgcn_perm(0u, st.rq[i][j], 0x0c010c00u), s2v);
          d[2 * j + 1] = dequant2(__builtin_amdgcn_perm(0u, st.rq[i][j], 0x0c030c02u), s2v);
        }
        half8_t lo = {d[0].x, d[0].y, d[1].x, d[1].y, d[2].x, d[2].y, d[3].x, d[3].y};
        half8_t hi = {d[4].x, d[4].y, d[5].x, d[5].y, d[6].x, d[6].y, d[7].x, d[7].y};
        half_t* dst = &Bs[buf][(c >> 2) * LDK + (c & 3) * 16];
        *reinterpret_cast<half8_t*>(dst) = lo;
        *reinterpret_cast<half8_t*>(dst + 8) = hi;
      }
    } else {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; ++i) {
        const int c = tid + i * THREADS;
        half8_t v = st.rb[i];
        if constexpr (KTAIL) v = (st.k0 + b_k[i] < K) ? v : (half8_t)(0.0f);
        *reinterpret_cast<half8_t*>(&Bs[buf][(c >> 3) * LDK + (c & 7) * 8]) = v;
      }
    }
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      acc[i][j] = (float16_t)(0.0f);
    }
  }

  const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
  auto compute = [&](int buf) {
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      half8_t fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        fa[i] = *reinterpret_cast<const half8_t*>(&As[buf][(wm + i * 32 + frag_row) * LDK + ks + frag_k]);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        fb[j] = *reinterpret_cast<const half8_t*>(&Bs[buf][(wn + j * 32 + frag_row) * LDK + ks + frag_k]);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
      }
    }
  };

  // Pipeline: LDS buffer t%2 holds K step t; one register stage holds step t+1 (requested one
  // iteration ago) and the other receives step t+2 while the matrix cores work on step t.
  // Two iterations per trip so that the two register stages keep fixed names.
  stage_t s0, s1;
  const int nt = (K + BK - 1) / BK;
  load_tile(s0, 0);
  if (nt > 1) load_tile(s1, BK);
  store_tile(s0, 0);
  __syncthreads();
  for (int t = 0; t < nt; t += 2) {
    // step t in LDS 0, step t+1 in s1
    if (t + 2 < nt) load_tile(s0, (t + 2) * BK);
    compute(0);
    if (t + 1 < nt) store_tile(s1, 1);
    __syncthreads();
    if (t + 1 >= nt) break;
    // step t+1 in LDS 1, step t+2 in s0
    if (t + 3 < nt) load_tile(s1, (t + 3) * BK);
    compute(1);
    if (t + 2 < nt) store_tile(s0, 0);
    __syncthreads();
  }

  // epilogue, llama_cu.cu:208-215: fp16(acc + beta * old).  Accumulator register v of lane l is
  // element (row 8*(v/4) + 4*(l/32) + v%4, column l%32) of the 32x32 tile.
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int gn = n0 + wn + j * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int gm = m0 + wm + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        if (gm < M && gn < N) {
          half_t* p = out + (size_t)gm * N + gn;
          float val = acc[i][j][v];
          if (beta != 0.0f) {
            val = fmaf(beta, (float)*p, val);
          }
          *p = round_f16(val);
        }
      }
    }
  }
}

template <int BM, int BN, bool U8>
int launch_gemm(half_t* out, const half_t* A, const void* W, const half_t* S, int M, int K, int N, int block,
                float beta, hipStream_t st) {
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  if (K % BK == 0) {
    gemm_kernel<BM, BN, U8, false><<<tiles_m * tiles_n, THREADS, 0, st>>>(out, A, W, S, M, K, N, block, beta, tiles_m,
                                                                          tiles_n);
  } else {
    gemm_kernel<BM, BN, U8, true><<<tiles_m * tiles_n, THREADS, 0, st>>>(out, A, W, S, M, K, N, block, beta, tiles_m,
                                                                         tiles_n);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

template <bool U8>
int dispatch_gemm(half_t* out, const half_t* A, const void* W, const half_t* S, int M, int K, int N, int block,
                  float beta, hipStream_t st) {
  // 128x128 tiles when there are enough of them to give every compute unit one; else 128x64
  const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
  if (tiles128 >= 256) {
    return launch_gemm<128, 128, U8>(out, A, W, S, M, K, N, block, beta, st);
  }
  return launch_gemm<128, 64, U8>(out, A, W, S, M, K, N, block, beta, st);
}

}  // namespace

extern "C" {

int lcu_gemm_f16_nt(void* out_dev, const void* lhs_dev, const void* rhs_dev, int M, int K, int N, float beta,
                    void* stream) {
  LCU_REQUIRE(out_dev && lhs_dev && rhs_dev, "lcu_gemm_f16_nt: null pointer");
  LCU_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 8 == 0, "lcu_gemm_f16_nt: bad shape M %d K %d N %d (K %% 8 == 0)", M, K,
              N);
  if (M == 0) return LCU_OK;
  LCU_REQUIRE((size_t)M * K * 2 < ((size_t)1 << 32) && (size_t)N * K * 2 < ((size_t)1 << 32),
              "lcu_gemm_f16_nt: operands of 4 GiB or more are not supported");
  if (M == 1 && K <= 24576) {
    return gemv_f16((half_t*)out_dev, (const half_t*)lhs_dev, (const half_t*)rhs_dev, K, N, beta, as_stream(stream));
  }
  return dispatch_gemm<false>((half_t*)out_dev, (const half_t*)lhs_dev, rhs_dev, nullptr, M, K, N, 0, beta,
                              as_stream(stream));
}

int lcu_gemm_f16u8_nt(void* out_dev, const void* lhs_dev, const void* codes_dev, const void* scales_dev, int M,
                      int K, int N, int block, float beta, void* stream) {
  LCU_REQUIRE(out_dev && lhs_dev && codes_dev && scales_dev, "lcu_gemm_f16u8_nt: null pointer");
  LCU_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 16 == 0 && block >= 16 && block % 16 == 0 && K % block == 0,
              "lcu_gemm_f16u8_nt: bad shape M %d K %d N %d block %d (K %% 16 == 0, block %% 16 == 0, K %% block == 0)",
              M, K, N, block);
  if (M == 0) return LCU_OK;
  LCU_REQUIRE((size_t)M * K * 2 < ((size_t)1 << 32) && (size_t)N * K < ((size_t)1 << 32),
              "lcu_gemm_f16u8_nt: operands of 4 GiB or more are not supported");
  if (M == 1 && K <= 24576) {
    return gemv_u8((half_t*)out_dev, (const half_t*)lhs_dev, (const uint8_t*)codes_dev, (const half_t*)scales_dev, K,
                   N, block, beta, as_stream(stream));
  }
  return dispatch_gemm<true>((half_t*)out_dev, (const half_t*)lhs_dev, codes_dev, (const half_t*)scales_dev, M, K, N,
                             block, beta, as_stream(stream));
}

}  // extern "C"
