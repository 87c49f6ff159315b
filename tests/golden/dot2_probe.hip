// Measures v_dot2_f32_f16 on the GPU: 3 * 2^20 seeded (a, b, c) samples and what the instruction
// returns for them, written as raw arrays (a: 2 fp16 per sample, b: 2 fp16, c: fp32, out: fp32).
// make_dot2_fixture.py picks the samples kept in dot2_gfx950.npz.
//   hipcc --offload-arch=gfx950 -O2 -o dot2_probe tests/golden/dot2_probe.hip && ./dot2_probe dot2.bin
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <random>
#include <vector>
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
#define CK(x)                                                                              \
  do {                                                                                     \
    hipError_t e = (x);                                                                    \
    if (e != hipSuccess) {                                                                 \
      printf("%s failed at line %d: %s\n", #x, __LINE__, hipGetErrorString(e));           \
      exit(1);                                                                             \
    }                                                                                      \
  } while (0)

__global__ void dot2_kernel(float* out, const half2_t* a, const half2_t* b, const float* c, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = __builtin_amdgcn_fdot2(a[i], b[i], c[i], false);
}

int main(int argc, char** argv) {
  if (argc != 2) {
    printf("usage: %s <output file>\n", argv[0]);
    return 2;
  }
  const int n = 3 << 20, n_first = 1 << 20, n_second = 2 << 20;
  std::vector<float> hc(n), ho(n);
  std::vector<_Float16> fa(2 * n), fb(2 * n);
  std::mt19937_64 rng(1);
  std::normal_distribution<float> nd(0.f, 1.f);
  // four magnitudes of a (so that products land above, around and below c, and some halves are
  // subnormal), two of c, c == 0 for one sample in eight
  for (int i = 0; i < n_first; ++i) {
    const int mode = i & 3;
    const float sa = mode == 0 ? 0.02f : (mode == 1 ? 1.0f : (mode == 2 ? 1e-3f : 30.f));
    fa[2 * i] = (_Float16)(nd(rng) * sa);
    fa[2 * i + 1] = (_Float16)(nd(rng) * sa);
    fb[2 * i] = (_Float16)nd(rng);
    fb[2 * i + 1] = (_Float16)nd(rng);
    hc[i] = nd(rng) * (mode == 3 ? 100.f : 0.05f) * ((i >> 2) & 1 ? 1.f : 0.001f);
    if (((i >> 3) & 7) == 0) hc[i] = 0.f;
  }
  // second half: halves drawn by bit pattern (exponent field 0..20, so one in 21 is subnormal), c
  // placed -6..+14 binades from the larger product with a random 24-bit mantissa
  for (int i = n_first; i < n_second; ++i) {
    uint16_t h[4];
    for (int j = 0; j < 4; ++j) {
      const uint64_t r = rng();
      h[j] = (uint16_t)(((r >> 40) & 1) << 15 | ((r >> 20) % 21) << 10 | (r & 0x3ff));
    }
    memcpy(&fa[2 * i], &h[0], 4);
    memcpy(&fb[2 * i], &h[2], 4);
    const float p0 = fabsf((float)fa[2 * i] * (float)fb[2 * i]), p1 = fabsf((float)fa[2 * i + 1] * (float)fb[2 * i + 1]);
    const float big = p0 > p1 ? p0 : p1;
    const uint64_t r = rng();
    const int gap = (int)((r >> 32) % 21) - 6;
    const float mant = 1.0f + (float)(r & 0x7fffff) * 0x1p-23f;
    hc[i] = big == 0.f ? mant : ldexpf(mant, ilogbf(big) + gap);
    if ((r >> 60) & 1) hc[i] = -hc[i];
  }
  // third part: c so close to a power of two, 6..13 binades above the products, that the products
  // carry the sum across it (the result's exponent is then not that of the largest addend)
  for (int i = n_second; i < n; ++i) {
    uint16_t h[4];
    for (int j = 0; j < 4; ++j) {
      const uint64_t r = rng();
      h[j] = (uint16_t)(((r >> 40) & 1) << 15 | (8 + (r >> 20) % 13) << 10 | (r & 0x3ff));
    }
    memcpy(&fa[2 * i], &h[0], 4);
    memcpy(&fb[2 * i], &h[2], 4);
    const double p0 = (double)fa[2 * i] * (double)fb[2 * i], p1 = (double)fa[2 * i + 1] * (double)fb[2 * i + 1];
    const double sum = p0 + p1, big = fabs(p0) > fabs(p1) ? fabs(p0) : fabs(p1);
    const uint64_t r = rng();
    const double edge = ldexp(1.0, ilogb(big) + 6 + (int)((r >> 32) % 8));
    const double u = (double)(r & 0xffffff) * 0x1p-24, sign = (r >> 60) & 1 ? -1.0 : 1.0;
    // products against c: c just beyond the edge, the sum just inside it; with c: the other way round
    hc[i] = (float)(sign * sum < 0 ? sign * (edge + u * fabs(sum)) : sign * (edge - u * fabs(sum)));
  }
  half2_t *da, *db;
  float *dc, *dout;
  CK(hipMalloc(&da, n * 4));
  CK(hipMalloc(&db, n * 4));
  CK(hipMalloc(&dc, n * 4));
  CK(hipMalloc(&dout, n * 4));
  CK(hipMemcpy(da, fa.data(), n * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(db, fb.data(), n * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(dc, hc.data(), n * 4, hipMemcpyHostToDevice));
  dot2_kernel<<<n / 256, 256>>>(dout, da, db, dc, n);
  CK(hipGetLastError());
  CK(hipMemcpy(ho.data(), dout, n * 4, hipMemcpyDeviceToHost));
  FILE* f = fopen(argv[1], "wb");
  if (!f) {
    printf("cannot write %s\n", argv[1]);
    return 1;
  }
  fwrite(fa.data(), 2, 2 * n, f);
  fwrite(fb.data(), 2, 2 * n, f);
  fwrite(hc.data(), 4, n, f);
  fwrite(ho.data(), 4, n, f);
  fclose(f);
  printf("wrote %d samples to %s\n", n, argv[1]);
  return 0;
}
