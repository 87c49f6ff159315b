// Shared device helpers and the error plumbing of the C ABI.  gfx950 only: 64-wide wavefronts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "llama_cu_hip.h"

namespace lcu {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int WAVE = 64;

int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

#define LCU_HIP(expr)                                                                         \
  do {                                                                                        \
    hipError_t e__ = (expr);                                                                  \
    if (e__ != hipSuccess) {                                                                  \
      return lcu::set_error(LCU_E_HIP, "%s:%d: %s failed: %s", __FILE__, __LINE__, #expr,     \
                            hipGetErrorString(e__));                                          \
    }                                                                                         \
  } while (0)

#define LCU_REQUIRE(cond, ...)                          \
  do {                                                  \
    if (!(cond)) {                                      \
      return lcu::set_error(LCU_E_SHAPE, __VA_ARGS__);  \
    }                                                   \
  } while (0)

#define LCU_LAUNCH_CHECK() LCU_HIP(hipGetLastError())

// per-device state created by lcu_init
struct device_state {
  bool ready = false;
  int compute_units = 0;
  void* workspace = nullptr;  // scratch of the default stream and of streams this library did not create
  size_t workspace_bytes = 0;
  uint32_t* workspace_sync = nullptr;
};
device_state* current_device_state();

// Scratch memory for operators that work in two launches (partial sums of split-K products, scores
// of long decode rows, partial error statistics).  Every stream made by lcu_stream_create owns a
// workspace of its own, so that contexts driven from different host threads (each has its stream)
// never share scratch; the default stream and foreign streams use the device's.  nullptr when
// lcu_init has not run on the current device.
struct workspace_t {
  void* ptr = nullptr;
  size_t bytes = 0;
  // SYNC_WORDS zero-initialised uint32 behind the scratch, never used as scratch: what workgroups
  // of one launch hand to one another (decode attention spread over several workgroups per head).
  // Words 0 .. SYNC_TIMEOUTS are counters; from SYNC_EXCHANGE on, 8-byte {value, epoch} words (64
  // heads x 4096 scores, then three rows of 4096), which no other operator may write: a reader trusts
  // a word by its epoch.
  uint32_t* sync = nullptr;
  // true for the workspace of a stream made by lcu_stream_create: nobody else's launches use it
  bool owned = false;
};
constexpr int SYNC_EXCHANGE = 2048;
// offsets (in 8-byte words) of the hand-over areas: decode attention scores (64 heads x 4096), then
// three rows of up to 8192 halves as {half2, epoch} words: the attention output, the residual row
// behind Wo, the residual row behind W2
constexpr int EXCH_ATT = 64 * 4096;
constexpr int EXCH_X = EXCH_ATT + 4096;
constexpr int EXCH_PROJ = EXCH_X + 4096;
constexpr int SYNC_WORDS = SYNC_EXCHANGE + (EXCH_PROJ + 4096) * 2;
constexpr int SYNC_TIMEOUTS = SYNC_EXCHANGE - 1;  // word that counts bounded waits which ran out
workspace_t workspace_for(hipStream_t stream);

// fp32 -> fp16, round to nearest even, as a separate step.  Written through an opaque register so
// the compiler cannot merge the conversion into the preceding multiply or fused multiply-add
// (v_fma_mixlo_f16 rounds the exact result once to fp16; the reference rounds to fp32 first, and a
// value that lands on an fp16 tie after the fp32 rounding then differs by one ulp).
__device__ __forceinline__ half_t round_f16(float f) {
  asm("" : "+v"(f));
  return (half_t)f;
}

// e^x in fp32 from IEEE operations only (multiply, fused multiply-add, round to nearest even,
// integer scaling), so that the host restatement of the same steps gives the same bits; within
// one ulp of the true value, as the reference's expf is (llama_cu.cu:463, 497, 537 call CUDA's,
// whose last bits no other platform reproduces either).  k = rne(x * log2 e); r = x - k * ln 2 with
// ln 2 split in two; a degree-7 polynomial in r (Cephes' coefficients); the result scaled by 2^k in
// two steps.  Results below the smallest normal number are returned as 0 and arguments above
// 88.72283 as infinity, whatever the denormal mode of the machine.
__device__ __forceinline__ float exp_ieee(float x) {
  if (x > 88.72283f) return __builtin_inff();
  if (x < -87.33654f) return 0.0f;
  const float kf = __builtin_rintf(x * 1.44269504f);
  float r = fmaf(kf, -0.693359375f, x);
  r = fmaf(kf, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = fmaf(p, r, 1.3981999507e-3f);
  p = fmaf(p, r, 8.3334519073e-3f);
  p = fmaf(p, r, 4.1665795894e-2f);
  p = fmaf(p, r, 1.6666665459e-1f);
  p = fmaf(p, r, 5.0000001201e-1f);
  p = fmaf(p * r, r, r) + 1.0f;
  const int k = (int)kf;
  const int k1 = k / 2, k2 = k - k1;
  const float s1 = __builtin_bit_cast(float, (uint32_t)(k1 + 127) << 23);
  const float s2 = __builtin_bit_cast(float, (uint32_t)(k2 + 127) << 23);
  const float res = (p * s1) * s2;
  return res < 1.17549435e-38f ? 0.0f : res;
}

// ---- wavefront reductions (all 64 lanes end with the result) ----
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes with data-parallel-primitive moves (VALU speed; __shfl_xor compiles to
// ds_bpermute, an LDS round trip per step).  Lanes 1, 2 apart by quad permutes, then the mirrors
// within 8 and 16 lanes, then the four 16-lane row sums are read out and added.  The association
// is (((t ^ 1) ^ 2) ^ 4) ^ 8 inside a row, then (r0 + r1) + (r2 + r3).
// sum over each aligned group of 16 lanes, left in every lane of the group
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f32<0x141>(v);  // row_half_mirror
  v += dpp_f32<0x140>(v);  // row_mirror
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  const int vi = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 48));
  return (r0 + r1) + (r2 + r3);
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    v = fmaxf(v, __shfl_xor(v, off, WAVE));
  }
  return v;
}

// Sum over a 256-thread block of one partial per thread, associated exactly as the reference's
// block reduction (llama_cu.cu:81-100 and 476-493): groups of 32 consecutive threads reduce by
// xor distances 16..1, then the eight group sums reduce by xor distances 4, 2, 1.  `red` is 8
// floats of LDS.  Every thread returns the total.
__device__ __forceinline__ float block256_sum_ref_order(float v, float* red) {
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) {
    v += __shfl_xor(v, off, WAVE);
  }
  const int tid = threadIdx.x;
  __syncthreads();  // protects `red` against a previous use
  if ((tid & 31) == 0) {
    red[tid >> 5] = v;
  }
  __syncthreads();
  float w = red[tid & 7];
#pragma unroll
  for (int off = 4; off > 0; off >>= 1) {
    w += __shfl_xor(w, off, WAVE);
  }
  return w;
}

// The same sum, same association, with the xor steps 8, 4, 2, 1 as data-parallel-primitive moves
// (xor 4: a shift by four lanes to the left for lanes 0-3 and 8-11 of a row, to the right for the
// others) and the eight group sums added in registers by every thread: the reference's xor steps
// 4, 2, 1 over lanes holding r0..r7 leave ((r0 + r4) + (r2 + r6)) + ((r1 + r5) + (r3 + r7)) in lane 0
// and, additions being commutative, the same bits in the other seven.  One ds_bpermute and one
// barrier pair instead of eight and two.
__device__ __forceinline__ float block256_sum_ref_order_dpp(float v, float* red) {
  v += __shfl_xor(v, 16, WAVE);
  v += dpp_f32<0x128>(v);  // row_ror:8 = xor 8 inside a row of 16
  {
    const int vi = __builtin_bit_cast(int, v);
    int t = __builtin_amdgcn_update_dpp(0, vi, 0x104, 0xF, 0x5, false);  // row_shl:4 into lanes 0-3, 8-11
    t = __builtin_amdgcn_update_dpp(t, vi, 0x114, 0xF, 0xA, false);      // row_shr:4 into lanes 4-7, 12-15
    v += __builtin_bit_cast(float, t);
  }
  v += dpp_f32<0x4E>(v);  // quad_perm [2,3,0,1]
  v += dpp_f32<0xB1>(v);  // quad_perm [1,0,3,2]
  const int tid = threadIdx.x;
  __syncthreads();  // protects `red` against a previous use
  if ((tid & 31) == 0) {
    red[tid >> 5] = v;
  }
  __syncthreads();
  const float4_t lo = *reinterpret_cast<const float4_t*>(red), hi = *reinterpret_cast<const float4_t*>(red + 4);
  return ((lo[0] + hi[0]) + (lo[2] + hi[2])) + ((lo[1] + hi[1]) + (lo[3] + hi[3]));
}

// maximum over a wavefront with data-parallel-primitive moves (the order of a maximum is free)
__device__ __forceinline__ float wave_max_dpp(float v) {
  v = fmaxf(v, dpp_f32<0xB1>(v));
  v = fmaxf(v, dpp_f32<0x4E>(v));
  v = fmaxf(v, dpp_f32<0x141>(v));
  v = fmaxf(v, dpp_f32<0x140>(v));
  const int vi = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 48));
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}
__device__ __forceinline__ float block256_max_dpp(float v, float* red) {
  v = wave_max_dpp(v);
  const int tid = threadIdx.x;
  __syncthreads();
  if ((tid & 63) == 0) {
    red[tid >> 6] = v;
  }
  __syncthreads();
  const float4_t r = *reinterpret_cast<const float4_t*>(red);
  return fmaxf(fmaxf(r[0], r[1]), fmaxf(r[2], r[3]));
}

__device__ __forceinline__ float block256_max(float v, float* red) {
  v = wave_max(v);
  const int tid = threadIdx.x;
  __syncthreads();
  if ((tid & 63) == 0) {
    red[tid >> 6] = v;
  }
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// ---- hand-over words read at device scope ----
// Loads that bypass the caches another XCD's store does not reach (sc0 sc1), several at a time, and
// the wait for them, in ONE asm statement: when the statement ends the data is in the registers, so
// whatever the compiler does with those registers afterwards (copy, spill, reuse) is safe.  With the
// wait in a statement of its own, the compiler -- which does not know that the registers are still
// being written -- may reuse or spill them in between, and the data then lands on something else.
// Early-clobber outputs: a register written by the first load must not hold a later load's address.
// (The compiler's own device-scope atomic loads are safe too, but it issues them one by one with a
// wait each: 1.7 us more per decoded layer.)
__device__ __forceinline__ void load_words_device_scope(uint64_t (&o)[1], const uint64_t* p0) {
  asm volatile("global_load_dwordx2 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(o[0]) : "v"(p0) : "memory");
}
__device__ __forceinline__ void load_words_device_scope(uint64_t (&o)[4], const uint64_t* p0, const uint64_t* p1,
                                                        const uint64_t* p2, const uint64_t* p3) {
  asm volatile(
      "global_load_dwordx2 %0, %4, off sc0 sc1\n\tglobal_load_dwordx2 %1, %5, off sc0 sc1\n\t"
      "global_load_dwordx2 %2, %6, off sc0 sc1\n\tglobal_load_dwordx2 %3, %7, off sc0 sc1\n\ts_waitcnt vmcnt(0)"
      : "=&v"(o[0]), "=&v"(o[1]), "=&v"(o[2]), "=&v"(o[3])
      : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
      : "memory");
}
// two neighbouring words (16 bytes, 16-byte aligned) per request
__device__ __forceinline__ void load_word_pairs_device_scope(uint4_t (&o)[1], const uint64_t* p0) {
  asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(o[0]) : "v"(p0) : "memory");
}
__device__ __forceinline__ void load_word_pairs_device_scope(uint4_t (&o)[4], const uint64_t* p0, const uint64_t* p1,
                                                             const uint64_t* p2, const uint64_t* p3) {
  asm volatile(
      "global_load_dwordx4 %0, %4, off sc0 sc1\n\tglobal_load_dwordx4 %1, %5, off sc0 sc1\n\t"
      "global_load_dwordx4 %2, %6, off sc0 sc1\n\tglobal_load_dwordx4 %3, %7, off sc0 sc1\n\ts_waitcnt vmcnt(0)"
      : "=&v"(o[0]), "=&v"(o[1]), "=&v"(o[2]), "=&v"(o[3])
      : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
      : "memory");
}

// fp16((code - 127.5) * scale): the product is exact in fp32 (9 x 11 significant bits), so this
// is one rounding, as dequantize_absmax_one (llama_cu.cu:287-289).
__device__ __forceinline__ half_t dequant_one(uint32_t code, float scale) {
  return round_f16(((float)code - 127.5f) * scale);
}

}  // namespace lcu
