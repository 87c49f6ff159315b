// Prefill matrix products on the gfx950 matrix cores: out[M,N] = lhs[M,K] * W[N,K]^T + beta*out.
//
// These replace matmul_nt_wmma_128x64x64 (llama_cu.cu:150-220) and, for uint8 weights,
// matmul_nt_wmma_16x128x256_fp16u8 at M > 1 (294-366).  Both operands are K-contiguous, which is
// the natural operand order of v_mfma_f32_32x32x16_f16: every lane feeds 8 consecutive k of one
// row of lhs (A) and of one row of W (B).
//
//   - 256 threads = 4 wavefronts in a 2x2 grid; block tile BM x BN, K step 64
//   - global -> registers -> LDS, the next K step's global loads in flight while the matrix cores
//     work on the current one; LDS rows padded by 16 bytes so the 16-byte operand reads of 16
//     neighbouring lanes fall in distinct banks
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

template <int BM, int BN, bool U8>
__global__ __launch_bounds__(THREADS) void gemm_kernel(half_t* __restrict__ out, const half_t* __restrict__ A,
                                                       const void* __restrict__ Wv, const half_t* __restrict__ S,
                                                       int M, int K, int N, int block, float beta, int tiles_m,
                                                       int tiles_n) {
  constexpr int TM = BM / 64;  // 32x32 MFMA tiles per wavefront along M
  constexpr int TN = BN / 64;
  constexpr int A_CHUNKS = BM * BK / 8 / THREADS;                  // 16-byte chunks per thread
  constexpr int B_CHUNKS = U8 ? BN * BK / 16 / THREADS : BN * BK / 8 / THREADS;
  static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1, "tile too small for 256 threads");

  __shared__ __attribute__((aligned(16))) half_t As[BM * LDK];
  __shared__ __attribute__((aligned(16))) half_t Bs[BN * LDK];

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
  const half_t* Wh = (const half_t*)Wv;
  const uint8_t* Wq = (const uint8_t*)Wv;
  const int nblk = U8 ? K / block : 0;

  half8_t ra[A_CHUNKS];
  half8_t rb[U8 ? 1 : B_CHUNKS];
  uint4_t rq[U8 ? B_CHUNKS : 1];
  half_t rs[U8 ? B_CHUNKS : 1];

  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * THREADS;
      const int row = c >> 3, kc = (c & 7) * 8;
      const int gm = m0 + row, gk = k0 + kc;
      ra[i] = (gm < M && gk < K) ? *reinterpret_cast<const half8_t*>(A + (size_t)gm * K + gk) : (half8_t)(0.0f);
    }
    if constexpr (U8) {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; ++i) {
        const int c = tid + i * THREADS;
        const int row = c >> 2, kc = (c & 3) * 16;
        const int gn = n0 + row, gk = k0 + kc;
        const bool ok = gn < N && gk < K;
        rq[i] = ok ? __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(Wq + (size_t)gn * K + gk))
                   : (uint4_t)(0u);
        rs[i] = ok ? S[(size_t)gn * nblk + gk / block] : (half_t)0.0f;
      }
    } else {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; ++i) {
        const int c = tid + i * THREADS;
        const int row = c >> 3, kc = (c & 7) * 8;
        const int gn = n0 + row, gk = k0 + kc;
        rb[i] = (gn < N && gk < K) ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(Wh + (size_t)gn * K + gk))
                                   : (half8_t)(0.0f);
      }
    }
  };

  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * THREADS;
      *reinterpret_cast<half8_t*>(&As[(c >> 3) * LDK + (c & 7) * 8]) = ra[i];
    }
    if constexpr (U8) {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; ++i) {
        const int c = tid + i * THREADS;
        const half_t s2 = rs[i] * (half_t)2.0f;
        const half2_t s2v = {s2, s2};
        half2_t d[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          d[2 * j] = dequant2(__builtin_amdgcn_perm(0u, rq[i][j], 0x0c010c00u), s2v);
          d[2 * j + 1] = dequant2(__builtin_amdgcn_perm(0u, rq[i][j], 0x0c030c02u), s2v);
        }
        half8_t lo = {d[0].x, d[0].y, d[1].x, d[1].y, d[2].x, d[2].y, d[3].x, d[3].y};
        half8_t hi = {d[4].x, d[4].y, d[5].x, d[5].y, d[6].x, d[6].y, d[7].x, d[7].y};
        half_t* dst = &Bs[(c >> 2) * LDK + (c & 3) * 16];
        *reinterpret_cast<half8_t*>(dst) = lo;
        *reinterpret_cast<half8_t*>(dst + 8) = hi;
      }
    } else {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; ++i) {
        const int c = tid + i * THREADS;
        *reinterpret_cast<half8_t*>(&Bs[(c >> 3) * LDK + (c & 7) * 8]) = rb[i];
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
  load_tile(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    store_tile();
    __syncthreads();
    if (k0 + BK < K) {
      load_tile(k0 + BK);
    }
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      half8_t fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        fa[i] = *reinterpret_cast<const half8_t*>(&As[(wm + i * 32 + frag_row) * LDK + ks + frag_k]);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        fb[j] = *reinterpret_cast<const half8_t*>(&Bs[(wn + j * 32 + frag_row) * LDK + ks + frag_k]);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
      }
    }
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
  gemm_kernel<BM, BN, U8><<<tiles_m * tiles_n, THREADS, 0, st>>>(out, A, W, S, M, K, N, block, beta, tiles_m, tiles_n);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

template <bool U8>
int dispatch_gemm(half_t* out, const half_t* A, const void* W, const half_t* S, int M, int K, int N, int block,
                  float beta, hipStream_t st) {
  // enough 128x128 tiles to cover the 256 compute units twice, else the narrower tile
  const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
  if (tiles128 >= 512) {
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
  if (M == 1 && K <= 24576) {
    return gemv_u8((half_t*)out_dev, (const half_t*)lhs_dev, (const uint8_t*)codes_dev, (const half_t*)scales_dev, K,
                   N, block, beta, as_stream(stream));
  }
  return dispatch_gemm<true>((half_t*)out_dev, (const half_t*)lhs_dev, codes_dev, (const half_t*)scales_dev, M, K, N,
                             block, beta, as_stream(stream));
}

}  // extern "C"
