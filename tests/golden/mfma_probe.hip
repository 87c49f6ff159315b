// Measures v_mfma_f32_32x32x16_f16 and v_mfma_f32_16x16x32_f16 on the GPU: seeded tiles A, B, C and
// the D = A B^T + C that one instruction returns, written as raw arrays.  make_mfma_fixture.py picks
// the outputs kept in mfma_gfx950.npz.
//   hipcc --offload-arch=gfx950 -O2 -o mfma_probe tests/golden/mfma_probe.hip && ./mfma_probe mfma.bin
// File: for each of the two shapes (M = N = 32, K = 16; then M = N = 16, K = 32), TILES tiles of
// A[M][K] fp16, then B[N][K] fp16, then C[M][N] fp32, then D[M][N] fp32; then the chains: CHAIN_TILES tiles
// of A[32][CHAIN_K], B[32][CHAIN_K] fp16, then D[CHAIN_TILES][CHAIN_K / 16][32][32] fp32.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <random>
#include <vector>
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));
#define CK(x)                                                                    \
  do {                                                                           \
    hipError_t e = (x);                                                          \
    if (e != hipSuccess) {                                                       \
      printf("%s failed at line %d: %s\n", #x, __LINE__, hipGetErrorString(e)); \
      exit(1);                                                                   \
    }                                                                            \
  } while (0)

constexpr int TILES = 768;

// lane l feeds row l % 32 and k = 8 * (l / 32) .. + 7 of A and of B; accumulator register r of lane l
// is element (8 * (r / 4) + 4 * (l / 32) + r % 4, l % 32)
__global__ __launch_bounds__(64) void mfma_32x32x16(float* D, const _Float16* A, const _Float16* B, const float* C) {
  const int lane = threadIdx.x;
  A += (size_t)blockIdx.x * 512;
  B += (size_t)blockIdx.x * 512;
  C += (size_t)blockIdx.x * 1024;
  D += (size_t)blockIdx.x * 1024;
  const half8_t a = *reinterpret_cast<const half8_t*>(A + (lane & 31) * 16 + (lane >> 5) * 8);
  const half8_t b = *reinterpret_cast<const half8_t*>(B + (lane & 31) * 16 + (lane >> 5) * 8);
  float16_t c;
  for (int r = 0; r < 16; ++r) c[r] = C[((r / 4) * 8 + (lane >> 5) * 4 + (r & 3)) * 32 + (lane & 31)];
  c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  for (int r = 0; r < 16; ++r) D[((r / 4) * 8 + (lane >> 5) * 4 + (r & 3)) * 32 + (lane & 31)] = c[r];
}

// lane l feeds row l % 16 and k = 8 * (l / 16) .. + 7; accumulator register e of lane l is element
// (4 * (l / 16) + e, l % 16)
__global__ __launch_bounds__(64) void mfma_16x16x32(float* D, const _Float16* A, const _Float16* B, const float* C) {
  const int lane = threadIdx.x;
  A += (size_t)blockIdx.x * 512;
  B += (size_t)blockIdx.x * 512;
  C += (size_t)blockIdx.x * 256;
  D += (size_t)blockIdx.x * 256;
  const half8_t a = *reinterpret_cast<const half8_t*>(A + (lane & 15) * 32 + (lane >> 4) * 8);
  const half8_t b = *reinterpret_cast<const half8_t*>(B + (lane & 15) * 32 + (lane >> 4) * 8);
  float4_t c;
  for (int e = 0; e < 4; ++e) c[e] = C[((lane >> 4) * 4 + e) * 16 + (lane & 15)];
  c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  for (int e = 0; e < 4; ++e) D[((lane >> 4) * 4 + e) * 16 + (lane & 15)] = c[e];
}

// Tiles 0 .. 255: normal values, four magnitudes of A and four of C (one of them zero).
// Tiles 256 .. 511: halves drawn by bit pattern (exponent field 0..20, so some are subnormal, one in 16
// zero; in every eighth tile A has exponent field 0..2 only), C placed -6 .. +14 binades from the largest product of its element with a random mantissa.
// Tiles 512 .. 767: as 256 .. 511, but C so close to a power of two, 6..13 binades above the products,
// that the products carry the sum across it.
static void fill(std::vector<_Float16>& A, std::vector<_Float16>& B, std::vector<float>& C, int M, int K,
                 std::mt19937_64& rng) {
  std::normal_distribution<float> nd(0.f, 1.f);
  for (int t = 0; t < TILES; ++t) {
    _Float16* a = &A[(size_t)t * M * K];
    _Float16* b = &B[(size_t)t * M * K];
    float* c = &C[(size_t)t * M * M];
    if (t < 256) {
      const float sa = (t & 3) == 0 ? 0.02f : ((t & 3) == 1 ? 1.f : ((t & 3) == 2 ? 1e-3f : 20.f));
      const int cm = (t >> 2) & 3;
      const float sc = cm == 0 ? 0.f : (cm == 1 ? 0.05f : (cm == 2 ? 5.f : 500.f));
      for (int i = 0; i < M * K; ++i) {
        a[i] = (_Float16)(nd(rng) * sa);
        b[i] = (_Float16)nd(rng);
      }
      for (int i = 0; i < M * M; ++i) c[i] = nd(rng) * sc;
      continue;
    }
    const bool tiny_a = (t & 7) == 7;  // A with exponent field 0..2: mostly subnormal halves
    for (int i = 0; i < 2 * M * K; ++i) {
      const uint64_t r = rng();
      const uint64_t field = tiny_a && i < M * K ? (r >> 20) % 3 : (r >> 20) % 21;
      uint16_t h = (uint16_t)(((r >> 40) & 1) << 15 | field << 10 | (r & 0x3ff));
      if (((r >> 50) & 15) == 0) h = 0;
      memcpy(i < M * K ? (void*)&a[i] : (void*)&b[i - M * K], &h, 2);
    }
    const bool crossing = t >= 512;
    for (int i = 0; i < M; ++i) {
      for (int j = 0; j < M; ++j) {
        float big = 0.f;
        double sum = 0.0;
        for (int k = 0; k < K; ++k) {
          big = fmaxf(big, fabsf((float)a[i * K + k] * (float)b[j * K + k]));
          sum += (double)a[i * K + k] * (double)b[j * K + k];
        }
        const uint64_t r = rng();
        if (crossing && big != 0.f) {
          const double edge = ldexp(1.0, ilogbf(big) + 6 + (int)((r >> 32) % 8));
          const double u = (double)(r & 0xffffff) * 0x1p-24, sign = (r >> 60) & 1 ? -1.0 : 1.0;
          c[i * M + j] = (float)(sign * sum < 0 ? sign * (edge + u * fabs(sum)) : sign * (edge - u * fabs(sum)));
          continue;
        }
        const int gap = (int)((r >> 32) % 21) - 6;
        const float mant = 1.0f + (float)(r & 0x7fffff) * 0x1p-23f;
        float v = big == 0.f ? mant : ldexpf(mant, ilogbf(big) + gap);
        if ((r >> 60) & 1) v = -v;
        c[i * M + j] = v;
      }
    }
  }
}

template <class Kernel>
static void run(FILE* f, Kernel kernel, int M, int K, std::mt19937_64& rng) {
  std::vector<_Float16> A((size_t)TILES * M * K), B((size_t)TILES * M * K);
  std::vector<float> C((size_t)TILES * M * M), D((size_t)TILES * M * M);
  fill(A, B, C, M, K, rng);
  _Float16 *dA, *dB;
  float *dC, *dD;
  CK(hipMalloc(&dA, A.size() * 2));
  CK(hipMalloc(&dB, B.size() * 2));
  CK(hipMalloc(&dC, C.size() * 4));
  CK(hipMalloc(&dD, D.size() * 4));
  CK(hipMemcpy(dA, A.data(), A.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dB, B.data(), B.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dC, C.data(), C.size() * 4, hipMemcpyHostToDevice));
  kernel<<<TILES, 64>>>(dD, dA, dB, dC);
  CK(hipGetLastError());
  CK(hipMemcpy(D.data(), dD, D.size() * 4, hipMemcpyDeviceToHost));
  fwrite(A.data(), 2, A.size(), f);
  fwrite(B.data(), 2, B.size(), f);
  fwrite(C.data(), 4, C.size(), f);
  fwrite(D.data(), 4, D.size(), f);
  // layout check against a plain float64 sum (loose: only a wrong operand layout fails it)
  long gross = 0;
  for (int t = 0; t < TILES; ++t)
    for (int i = 0; i < M; ++i)
      for (int j = 0; j < M; ++j) {
        double s = C[((size_t)t * M + i) * M + j];
        double mag = fabs(s);
        for (int k = 0; k < K; ++k) {
          const double p = (double)A[((size_t)t * M + i) * K + k] * (double)B[((size_t)t * M + j) * K + k];
          s += p;
          mag += fabs(p);
        }
        if (fabs(D[((size_t)t * M + i) * M + j] - s) > 1e-5 * mag) ++gross;
      }
  printf("%dx%dx%d: %d tiles, %ld outputs far from the float64 sum\n", M, M, K, TILES, gross);
  CK(hipFree(dA));
  CK(hipFree(dB));
  CK(hipFree(dC));
  CK(hipFree(dD));
}

// A chain of v_mfma_f32_32x32x16_f16 over K = CHAIN_K as a matrix product runs it, started from
// 0, with the accumulator written out after every instruction: D[step][32][32].
constexpr int CHAIN_TILES = 12, CHAIN_K = 4096;
__global__ __launch_bounds__(64) void mfma_chain(float* D, const _Float16* A, const _Float16* B) {
  const int lane = threadIdx.x;
  A += (size_t)blockIdx.x * 32 * CHAIN_K;
  B += (size_t)blockIdx.x * 32 * CHAIN_K;
  D += (size_t)blockIdx.x * (CHAIN_K / 16) * 1024;
  float16_t c = (float16_t)(0.0f);
  for (int s = 0; s < CHAIN_K / 16; ++s) {
    const half8_t a = *reinterpret_cast<const half8_t*>(A + (size_t)(lane & 31) * CHAIN_K + s * 16 + (lane >> 5) * 8);
    const half8_t b = *reinterpret_cast<const half8_t*>(B + (size_t)(lane & 31) * CHAIN_K + s * 16 + (lane >> 5) * 8);
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    for (int r = 0; r < 16; ++r) D[(size_t)s * 1024 + ((r / 4) * 8 + (lane >> 5) * 4 + (r & 3)) * 32 + (lane & 31)] = c[r];
  }
}

static void run_chains(FILE* f) {
  std::vector<_Float16> A((size_t)CHAIN_TILES * 32 * CHAIN_K), B(A.size());
  std::vector<float> D((size_t)CHAIN_TILES * (CHAIN_K / 16) * 1024);
  std::mt19937_64 rng(11);
  std::normal_distribution<float> nd(0.f, 1.f);
  for (auto& v : A) v = (_Float16)nd(rng);            // activations
  for (auto& v : B) v = (_Float16)(nd(rng) * 0.02f);  // weights
  _Float16 *dA, *dB;
  float* dD;
  CK(hipMalloc(&dA, A.size() * 2));
  CK(hipMalloc(&dB, B.size() * 2));
  CK(hipMalloc(&dD, D.size() * 4));
  CK(hipMemcpy(dA, A.data(), A.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dB, B.data(), B.size() * 2, hipMemcpyHostToDevice));
  mfma_chain<<<CHAIN_TILES, 64>>>(dD, dA, dB);
  CK(hipGetLastError());
  CK(hipMemcpy(D.data(), dD, D.size() * 4, hipMemcpyDeviceToHost));
  fwrite(A.data(), 2, A.size(), f);
  fwrite(B.data(), 2, B.size(), f);
  fwrite(D.data(), 4, D.size(), f);
  printf("chains: %d tiles, K = %d\n", CHAIN_TILES, CHAIN_K);
  CK(hipFree(dA));
  CK(hipFree(dB));
  CK(hipFree(dD));
}

int main(int argc, char** argv) {
  if (argc != 2) {
    printf("usage: %s <output file>\n", argv[0]);
    return 2;
  }
  FILE* f = fopen(argv[1], "wb");
  if (!f) {
    printf("cannot write %s\n", argv[1]);
    return 1;
  }
  std::mt19937_64 rng(3);
  run(f, mfma_32x32x16, 32, 16, rng);
  run(f, mfma_16x16x32, 16, 32, rng);
  run_chains(f);
  fclose(f);
  return 0;
}
