// Row-wise and element-wise kernels of the forward pass, the int8 absmax quantiser, and the
// synthetic-tensor fill.  Each kernel keeps the reference's fp16 rounding points; reference
// lines are cited per kernel.
#include "common.hpp"

using namespace lcu;

namespace {

// ---------------------------------------------------------------------------------------------
// rms_norm, llama_cu.cu:66-107.  One 256-thread block per row; the sum of squares is associated
// exactly as the reference's (thread t owns elements t, t+256, ...; see block256_sum_ref_order).
// Two roundings: fp16(x * rms_inv), then fp16(weight * that).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rmsnorm_kernel(half_t* out, const half_t* in,
                                                      const half_t* __restrict__ weights, int cols, float eps) {
  extern __shared__ half_t xs[];  // the row, so that it is read from memory once, with 16-byte loads
  __shared__ __attribute__((aligned(16))) float red[8];
  const half_t* x = in + (size_t)blockIdx.x * cols;
  half_t* y = out + (size_t)blockIdx.x * cols;
  const bool vec = (cols % 8) == 0;
  // rows of up to 8192 elements (every model width): up to four pieces per thread, the weights
  // requested together with the row, so the kernel has one memory round trip before its stores;
  // longer rows take the general loops below
  constexpr int P = 4;
  const bool few = vec && cols <= P * 256 * 8;
  half8_t wp[P];
  if (few) {
    uint4 xp[P];
#pragma unroll
    for (int j = 0; j < P; ++j) {
      const int i = (threadIdx.x + 256 * j) * 8;
      xp[j] = i < cols ? *reinterpret_cast<const uint4*>(x + i) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < P; ++j) {
      const int i = (threadIdx.x + 256 * j) * 8;
      wp[j] = i < cols ? *reinterpret_cast<const half8_t*>(weights + i) : (half8_t)(0.0f);
    }
#pragma unroll
    for (int j = 0; j < P; ++j) {
      const int i = (threadIdx.x + 256 * j) * 8;
      if (i < cols) *reinterpret_cast<uint4*>(xs + i) = xp[j];
    }
  } else if (vec) {
    for (int i = threadIdx.x * 8; i < cols; i += 256 * 8) {
      *reinterpret_cast<uint4*>(xs + i) = *reinterpret_cast<const uint4*>(x + i);
    }
  } else {
    for (int i = threadIdx.x; i < cols; i += 256) xs[i] = x[i];
  }
  __syncthreads();
  float s = 0.0f;
  // eight LDS reads in flight at a time; the additions stay in ascending order
  int i = threadIdx.x;
  for (; i + 7 * 256 < cols; i += 8 * 256) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = (float)xs[i + u * 256];
#pragma unroll
    for (int u = 0; u < 8; ++u) s = fmaf(v[u], v[u], s);
  }
  for (; i < cols; i += 256) {
    float v = (float)xs[i];
    s = fmaf(v, v, s);
  }
  const float total = block256_sum_ref_order_dpp(s, red);
  const float rms_inv = 1.0f / sqrtf(total / (float)cols + eps);
  if (few) {
#pragma unroll
    for (int j = 0; j < P; ++j) {
      const int i = (threadIdx.x + 256 * j) * 8;
      if (i < cols) {
        const half8_t xv = *reinterpret_cast<const half8_t*>(xs + i);
        half8_t r;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const half_t inner = round_f16((float)xv[e] * rms_inv);
          r[e] = round_f16((float)wp[j][e] * (float)inner);
        }
        *reinterpret_cast<half8_t*>(y + i) = r;
      }
    }
  } else if (vec) {
    for (int i = threadIdx.x * 8; i < cols; i += 256 * 8) {
      const half8_t xv = *reinterpret_cast<const half8_t*>(xs + i);
      const half8_t wv = *reinterpret_cast<const half8_t*>(weights + i);
      half8_t r;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const half_t inner = round_f16((float)xv[e] * rms_inv);
        r[e] = round_f16((float)wv[e] * (float)inner);
      }
      *reinterpret_cast<half8_t*>(y + i) = r;
    }
  } else {
    for (int i = threadIdx.x; i < cols; i += 256) {
      half_t inner = round_f16((float)xs[i] * rms_inv);
      y[i] = round_f16((float)weights[i] * (float)inner);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// rotary, llama_cu.cu:368-389.  One thread per interleaved pair; cos/sin from the host-built
// table.  real*cos - imag*sin and real*sin + imag*cos each use one fused multiply-add.
// ---------------------------------------------------------------------------------------------
__global__ void rope_kernel(half_t* out, const half_t* in, int rows, int cols, int head_dim, int pos_offset,
                            const float2* __restrict__ table) {
  const int pair = blockIdx.x * blockDim.x + threadIdx.x;
  const int r = blockIdx.y;
  if (pair * 2 >= cols) return;
  const int c = pair * 2;
  const float2 cs = table[(size_t)(pos_offset + r) * (head_dim / 2) + (c % head_dim) / 2];
  const size_t o = (size_t)r * cols + c;
  const half2_t v = *reinterpret_cast<const half2_t*>(in + o);
  const float real = (float)v.x, imag = (float)v.y;
  half2_t w;
  w.x = round_f16(fmaf(real, cs.x, -(imag * cs.y)));
  w.y = round_f16(fmaf(real, cs.y, imag * cs.x));
  *reinterpret_cast<half2_t*>(out + o) = w;
}

// the same for two tensors of one shape in place (the new rows of Q and of K, llama_cu.cu:1146 and 1152):
// blockIdx.z picks the tensor, so a prompt pays one launch for both
__global__ void rope_pair_kernel(half_t* a, half_t* b, int rows, int cols, int head_dim, int pos_offset,
                                 const float2* __restrict__ table) {
  const int pair = blockIdx.x * blockDim.x + threadIdx.x;
  const int r = blockIdx.y;
  if (pair * 2 >= cols) return;
  half_t* x = blockIdx.z ? b : a;
  const int c = pair * 2;
  const float2 cs = table[(size_t)(pos_offset + r) * (head_dim / 2) + (c % head_dim) / 2];
  const size_t o = (size_t)r * cols + c;
  const half2_t v = *reinterpret_cast<const half2_t*>(x + o);
  const float real = (float)v.x, imag = (float)v.y;
  half2_t w;
  w.x = round_f16(fmaf(real, cs.x, -(imag * cs.y)));
  w.y = round_f16(fmaf(real, cs.y, imag * cs.x));
  *reinterpret_cast<half2_t*>(x + o) = w;
}

// ---------------------------------------------------------------------------------------------
// softmax_rows, llama_cu.cu:433-499.  One 256-thread block per row, thread t owns elements
// t, t+256, ...; the exponential sum is associated as in the reference.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void softmax_rows_kernel(half_t* out, const half_t* in, int w, float temp) {
  __shared__ float red[8];
  const half_t* x = in + (size_t)blockIdx.x * w;
  half_t* y = out + (size_t)blockIdx.x * w;
  float m = -INFINITY;
  for (int i = threadIdx.x; i < w; i += 256) {
    m = fmaxf(m, (float)x[i] / temp);
  }
  m = block256_max(m, red);
  float s = 0.0f;
  for (int i = threadIdx.x; i < w; i += 256) {
    s += exp_ieee((float)x[i] / temp - m);
  }
  const float total = block256_sum_ref_order(s, red);
  for (int i = threadIdx.x; i < w; i += 256) {
    y[i] = round_f16(exp_ieee((float)x[i] / temp - m) / total);
  }
}

// One decode step of several sequences at once: row b of q is rotated in place, row b of k_new is
// rotated and row b of v_new copied into row pos[b] of sequence b's caches (rotary as rope_kernel,
// llama_cu.cu:368-389 and 1144-1156, with a position per row).  pos is clamped into the table.
__global__ void rope_store_batch_kernel(half_t* q, const half_t* __restrict__ k_new, const half_t* __restrict__ v_new,
                                        half_t* const* __restrict__ k_ptrs, half_t* const* __restrict__ v_ptrs,
                                        const int* __restrict__ pos_dev, int dim, int head_dim,
                                        const float2* __restrict__ table, int max_pos) {
  const int pair = blockIdx.x * blockDim.x + threadIdx.x;
  const int b = blockIdx.y;
  if (pair * 2 >= dim) return;
  const int c = pair * 2;
  const int pos = min(max(pos_dev[b], 0), max_pos);
  const float2 cs = table[(size_t)pos * (head_dim / 2) + (c % head_dim) / 2];
  const size_t src = (size_t)b * dim + c, dst = (size_t)pos * dim + c;
  const half2_t qv = *reinterpret_cast<const half2_t*>(q + src);
  const half2_t kv = *reinterpret_cast<const half2_t*>(k_new + src);
  half2_t w;
  w.x = round_f16(fmaf((float)qv.x, cs.x, -((float)qv.y * cs.y)));
  w.y = round_f16(fmaf((float)qv.x, cs.y, (float)qv.y * cs.x));
  *reinterpret_cast<half2_t*>(q + src) = w;
  w.x = round_f16(fmaf((float)kv.x, cs.x, -((float)kv.y * cs.y)));
  w.y = round_f16(fmaf((float)kv.x, cs.y, (float)kv.y * cs.x));
  *reinterpret_cast<half2_t*>(k_ptrs[b] + dst) = w;
  *reinterpret_cast<half2_t*>(v_ptrs[b] + dst) = *reinterpret_cast<const half2_t*>(v_new + src);
}

// Draws index i with probability p[i] / sum(p): the std::discrete_distribution the reference leaves
// commented out (llama_cu.cu:1202-1203), in integers so that the draw is reproducible bit for bit.
// weight = p * 2^24 (exact for fp16 in [0, 1]; negative and NaN count 0, values above 65504
// saturate), r = floor(random * total / 2^64), result = the smallest i whose running sum of weights
// exceeds r; 0 when every weight is 0.  One workgroup: thread t owns the contiguous run
// [t * seg, (t + 1) * seg), prefix sums of the run totals across the workgroup, and the thread
// whose run holds r walks it.
__device__ __forceinline__ uint64_t sample_weight(half_t h) {
  const float f = (float)h;
  if (!(f > 0.0f)) {
    return 0;
  }
  return (uint64_t)(fminf(f, 65504.0f) * 16777216.0f);  // exact: 11 significant bits, at most 2^40
}

__global__ __launch_bounds__(1024) void sample_row_kernel(int* __restrict__ index, const half_t* __restrict__ probs,
                                                          int n, uint64_t random, const uint64_t* __restrict__ random_dev) {
  __shared__ uint64_t wave_total[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (random_dev) {
    random = *random_dev;
  }
  const int seg = (n + 1023) / 1024;
  const int begin = min(tid * seg, n), end = min(begin + seg, n);
  uint64_t own = 0;
  for (int i = begin; i < end; ++i) {
    own += sample_weight(probs[i]);
  }
  // inclusive prefix over the wavefront, then over the 16 wavefront totals
  uint64_t incl = own;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t lo = __shfl_up((uint32_t)incl, off, WAVE), hi = __shfl_up((uint32_t)(incl >> 32), off, WAVE);
    if (lane >= off) {
      incl += ((uint64_t)hi << 32) | lo;
    }
  }
  if (lane == 63) {
    wave_total[wave] = incl;
  }
  __syncthreads();
  uint64_t before = 0, total = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    if (w < wave) {
      before += wave_total[w];
    }
    total += wave_total[w];
  }
  if (total == 0) {
    if (tid == 0) {
      *index = 0;
    }
    return;
  }
  const uint64_t r = __umul64hi(random, total);
  const uint64_t lo_run = before + incl - own;  // weights in front of this thread's run
  if (r >= lo_run && r < lo_run + own) {        // exactly one thread: the runs tile [0, total)
    uint64_t run = lo_run;
    int pick = end - 1;
    for (int i = begin; i < end; ++i) {
      run += sample_weight(probs[i]);
      if (run > r) {
        pick = i;
        break;
      }
    }
    *index = pick;
  }
}

// softmax_rows with temperature over one long row (the logits, llama_cu.cu:1196-1197) followed by
// the first-maximum argmax of the rounded probabilities (1205-1209), in one 1024-thread
// workgroup with 16-byte loads.  The exponential sum is associated differently from the
// 256-thread reference kernel (per-thread partials, then wavefronts, then 16 wavefront sums in
// order), which moves a probability by at most the last fp32 bit of the sum.
__global__ __launch_bounds__(1024) void softmax_argmax_kernel(half_t* __restrict__ probs, int* __restrict__ index,
                                                              const half_t* __restrict__ logits, int n, float temp,
                                                              const uint32_t* __restrict__ status_in) {
  __shared__ float sred[16];
  __shared__ int sidx[16];
  // one row per workgroup (several rows: one sequence of a batch each)
  probs += (size_t)blockIdx.x * n;
  logits += (size_t)blockIdx.x * n;
  index += blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n8 = n / 8;
  if (n % 8 == 0 && n8 <= 4 * 1024) {
    // every vocabulary of the model family (n <= 32768): the row is read once and each element's
    // x / temp, then its exponential, stays in registers -- the same operations in the same order
    // as the general path below, which reads the row three times and takes each exponential twice
    float t[4][8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = tid + j * 1024;
      const half8_t v = c < n8 ? *reinterpret_cast<const half8_t*>(logits + (size_t)c * 8) : (half8_t)(0.0f);
#pragma unroll
      for (int e = 0; e < 8; ++e) t[j][e] = c < n8 ? (float)v[e] / temp : -INFINITY;
    }
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int e = 0; e < 8; ++e) m = fmaxf(m, t[j][e]);
    }
    m = wave_max(m);
    if (lane == 0) sred[wave] = m;
    __syncthreads();
    m = sred[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) m = fmaxf(m, sred[w]);
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (tid + j * 1024 < n8) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          t[j][e] = exp_ieee(t[j][e] - m);
          s += t[j][e];
        }
      }
    }
    s = wave_sum(s);
    if (lane == 0) sred[wave] = s;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < 16; ++w) total += sred[w];
    __syncthreads();
    float best = -INFINITY;
    int idx = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = tid + j * 1024;
      if (c < n8) {
        half8_t p;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          p[e] = round_f16(t[j][e] / total);
          const float f = (float)p[e];
          if (f > best) {  // ascending index within a thread: strict > keeps the first maximum
            best = f;
            idx = c * 8 + e;
          }
        }
        *reinterpret_cast<half8_t*>(probs + (size_t)c * 8) = p;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, WAVE);
      const int oi = __shfl_xor(idx, off, WAVE);
      if (ob > best || (ob == best && oi < idx)) {
        best = ob;
        idx = oi;
      }
    }
    if (lane == 0) {
      sred[wave] = best;
      sidx[wave] = idx;
    }
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < 16; ++w) {
        if (sred[w] > best || (sred[w] == best && sidx[w] < idx)) {
          best = sred[w];
          idx = sidx[w];
        }
      }
      *index = idx == 0x7fffffff ? 0 : idx;
      if (status_in) index[1] = (int)*status_in;
    }
    return;
  }
  float m = -INFINITY;
  for (int c = tid; c < n8; c += 1024) {
    const half8_t v = *reinterpret_cast<const half8_t*>(logits + (size_t)c * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) m = fmaxf(m, (float)v[e] / temp);
  }
  for (int i = n8 * 8 + tid; i < n; i += 1024) m = fmaxf(m, (float)logits[i] / temp);
  m = wave_max(m);
  if (lane == 0) sred[wave] = m;
  __syncthreads();
  m = sred[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) m = fmaxf(m, sred[w]);
  __syncthreads();
  float s = 0.0f;
  for (int c = tid; c < n8; c += 1024) {
    const half8_t v = *reinterpret_cast<const half8_t*>(logits + (size_t)c * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) s += exp_ieee((float)v[e] / temp - m);
  }
  for (int i = n8 * 8 + tid; i < n; i += 1024) s += exp_ieee((float)logits[i] / temp - m);
  s = wave_sum(s);
  if (lane == 0) sred[wave] = s;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < 16; ++w) total += sred[w];
  __syncthreads();
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int c = tid; c < n8; c += 1024) {
    const half8_t v = *reinterpret_cast<const half8_t*>(logits + (size_t)c * 8);
    half8_t p;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      p[e] = round_f16(exp_ieee((float)v[e] / temp - m) / total);
      const float f = (float)p[e];
      if (f > best) {  // ascending index within a thread: strict > keeps the first maximum
        best = f;
        idx = c * 8 + e;
      }
    }
    *reinterpret_cast<half8_t*>(probs + (size_t)c * 8) = p;
  }
  for (int i = n8 * 8 + tid; i < n; i += 1024) {
    const half_t p = round_f16(exp_ieee((float)logits[i] / temp - m) / total);
    probs[i] = p;
    if ((float)p > best || ((float)p == best && i < idx)) {
      best = (float)p;
      idx = i;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ob = __shfl_xor(best, off, WAVE);
    const int oi = __shfl_xor(idx, off, WAVE);
    if (ob > best || (ob == best && oi < idx)) {
      best = ob;
      idx = oi;
    }
  }
  if (lane == 0) {
    sred[wave] = best;
    sidx[wave] = idx;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 16; ++w) {
      if (sred[w] > best || (sred[w] == best && sidx[w] < idx)) {
        best = sred[w];
        idx = sidx[w];
      }
    }
    *index = idx == 0x7fffffff ? 0 : idx;
    if (status_in) index[1] = (int)*status_in;
  }
}

// silu, llama_cu.cu:533-539
__device__ __forceinline__ half_t silu_mul_one(half_t a, half_t b) {
  const float val = (float)a;
  return round_f16(val / (1.0f + exp_ieee(-val)) * (float)b);
}

// eight elements per thread with 16-byte accesses (VEC: every pointer 16-byte aligned), the tail
// and unaligned buffers one by one
template <bool VEC>
__global__ __launch_bounds__(256) void silu_mul_kernel(half_t* out, const half_t* a, const half_t* b, size_t size) {
  const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i >= size) {
    return;
  }
  if (VEC && i + 8 <= size) {
    const half8_t av = *reinterpret_cast<const half8_t*>(a + i), bv = *reinterpret_cast<const half8_t*>(b + i);
    half8_t r;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      r[e] = silu_mul_one(av[e], bv[e]);
    }
    *reinterpret_cast<half8_t*>(out + i) = r;
    return;
  }
  for (size_t j = i; j < min(i + 8, size); ++j) {
    out[j] = silu_mul_one(a[j], b[j]);
  }
}

// embed, llama_cu.cu:32-44: one block per token, 16-byte copies.  An id outside the table gives
// a zero row instead of a stray read.
__global__ void embed_kernel(half_t* __restrict__ out, const short* __restrict__ ids, int dim,
                             const half_t* __restrict__ table, int n_vocab) {
  const int id = ids[blockIdx.x];
  const bool ok = id >= 0 && id < n_vocab;
  const uint4* src = reinterpret_cast<const uint4*>(table + (size_t)(ok ? id : 0) * dim);
  uint4* dst = reinterpret_cast<uint4*>(out + (size_t)blockIdx.x * dim);
  for (int i = threadIdx.x; i < dim / 8; i += blockDim.x) {
    dst[i] = ok ? src[i] : make_uint4(0, 0, 0, 0);
  }
}

// embed_uint8, llama_cu.cu:46-62, sixteen codes per thread (one 16-byte request; they share a scale when
// the block is a multiple of 16): grid (ids, pieces of 4096 codes).  The decode step's single row took
// 15 us with one element per thread and loop trip.
__global__ __launch_bounds__(256) void embed_u8x16_kernel(half_t* __restrict__ out, const short* __restrict__ ids,
                                                          int dim, const uint8_t* __restrict__ codes,
                                                          const half_t* __restrict__ scales, int block, int n_vocab) {
  const int i = (blockIdx.y * 256 + threadIdx.x) * 16;
  if (i >= dim) return;
  const int id = ids[blockIdx.x];
  half8_t r[2] = {(half8_t)(0.0f), (half8_t)(0.0f)};
  if (id >= 0 && id < n_vocab) {
    const uint4_t q = *reinterpret_cast<const uint4_t*>(codes + (size_t)id * dim + i);
    const float s = (float)scales[(size_t)id * (dim / block) + i / block];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      r[e / 8][e % 8] = dequant_one((q[e / 4] >> (8 * (e % 4))) & 0xFF, s);
    }
  }
  half8_t* dst = reinterpret_cast<half8_t*>(out + (size_t)blockIdx.x * dim + i);
  dst[0] = r[0];
  dst[1] = r[1];
}

// any block size and row length: one element per thread and trip
__global__ void embed_u8_kernel(half_t* __restrict__ out, const short* __restrict__ ids, int dim,
                                const uint8_t* __restrict__ codes, const half_t* __restrict__ scales, int block,
                                int n_vocab) {
  const int id = ids[blockIdx.x];
  const bool ok = id >= 0 && id < n_vocab;
  const int nblk = dim / block;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    half_t v = (half_t)0.0f;
    if (ok) {
      v = dequant_one(codes[(size_t)id * dim + i], (float)scales[(size_t)id * nblk + i / block]);
    }
    out[(size_t)blockIdx.x * dim + i] = v;
  }
}

// embed / embed_uint8 followed by rms_norm of the same rows (llama_cu.cu:1087-1097, then 1129 of the
// first layer) in one launch: a block gathers its row (dequantised where the table is uint8), writes it
// and normalises it from LDS with rmsnorm_kernel's arithmetic.  The norm weights are requested before the
// id is known.  cols a multiple of 8, at most 8192; block 0 (fp16 table) or a multiple of 8.
template <bool U8>
__global__ __launch_bounds__(256) void embed_rmsnorm_kernel(half_t* __restrict__ x_out, half_t* __restrict__ norm_out,
                                                            const short* __restrict__ ids, int cols,
                                                            const void* __restrict__ table,
                                                            const half_t* __restrict__ scales, int block, int n_vocab,
                                                            const half_t* __restrict__ weights, float eps) {
  extern __shared__ half_t xs[];
  __shared__ __attribute__((aligned(16))) float red[8];
  constexpr int P = 4;
  half8_t wp[P];
#pragma unroll
  for (int j = 0; j < P; ++j) {
    const int i = (threadIdx.x + 256 * j) * 8;
    wp[j] = i < cols ? *reinterpret_cast<const half8_t*>(weights + i) : (half8_t)(0.0f);
  }
  const int id = ids[blockIdx.x];
  const bool ok = id >= 0 && id < n_vocab;
  half_t* x = x_out + (size_t)blockIdx.x * cols;
  half_t* y = norm_out + (size_t)blockIdx.x * cols;
#pragma unroll
  for (int j = 0; j < P; ++j) {
    const int i = (threadIdx.x + 256 * j) * 8;
    if (i >= cols) continue;
    half8_t v = (half8_t)(0.0f);
    if (ok) {
      if constexpr (U8) {
        const uint2 q = *reinterpret_cast<const uint2*>((const uint8_t*)table + (size_t)id * cols + i);
        const float sc = (float)scales[(size_t)id * (cols / block) + i / block];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[e] = dequant_one(((e < 4 ? q.x : q.y) >> (8 * (e % 4))) & 0xFF, sc);
        }
      } else {
        v = *reinterpret_cast<const half8_t*>((const half_t*)table + (size_t)id * cols + i);
      }
    }
    *reinterpret_cast<half8_t*>(xs + i) = v;
    *reinterpret_cast<half8_t*>(x + i) = v;
  }
  __syncthreads();
  float s = 0.0f;
  int i = threadIdx.x;
  for (; i + 7 * 256 < cols; i += 8 * 256) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = (float)xs[i + u * 256];
#pragma unroll
    for (int u = 0; u < 8; ++u) s = fmaf(v[u], v[u], s);
  }
  for (; i < cols; i += 256) {
    float v = (float)xs[i];
    s = fmaf(v, v, s);
  }
  const float total = block256_sum_ref_order_dpp(s, red);
  const float rms_inv = 1.0f / sqrtf(total / (float)cols + eps);
#pragma unroll
  for (int j = 0; j < P; ++j) {
    const int k = (threadIdx.x + 256 * j) * 8;
    if (k < cols) {
      const half8_t xv = *reinterpret_cast<const half8_t*>(xs + k);
      half8_t r;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const half_t inner = round_f16((float)xv[e] * rms_inv);
        r[e] = round_f16((float)wp[j][e] * (float)inner);
      }
      *reinterpret_cast<half8_t*>(y + k) = r;
    }
  }
}

// exp_ieee on plain fp32 values (a check of the exponential every softmax and SiLU here uses)
__global__ void exp_kernel(float* __restrict__ out, const float* __restrict__ in, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = exp_ieee(in[i]);
}

// first maximum of n fp16 values compared as float, llama_cu.cu:1205-1209
__global__ __launch_bounds__(1024) void argmax_kernel(int* out, const half_t* __restrict__ v, int n) {
  __shared__ float sval[16];
  __shared__ int sidx[16];
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < n; i += 1024) {
    const float f = (float)v[i];
    if (idx == 0x7fffffff || best < f) {  // strict: an equal later value never replaces
      best = f;
      idx = i;
    }
  }
  // (value, index) pairs merge by "larger value, then smaller index"; empty slots are (-inf, INT_MAX)
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ob = __shfl_xor(best, off, WAVE);
    const int oi = __shfl_xor(idx, off, WAVE);
    if (ob > best || (ob == best && oi < idx)) {
      best = ob;
      idx = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    sval[threadIdx.x >> 6] = best;
    sidx[threadIdx.x >> 6] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; ++w) {
      if (sval[w] > best || (sval[w] == best && sidx[w] < idx)) {
        best = sval[w];
        idx = sidx[w];
      }
    }
    *out = idx == 0x7fffffff ? 0 : idx;
  }
}

// ---------------------------------------------------------------------------------------------
// quantize_absmax_uint8, transform.cu:28-72.  One wavefront per (row, block of `block` elements).
// IEEE-only arithmetic: fp32 max, correctly rounded division, round-half-away; the conversion to
// uint8 saturates and maps NaN (all-zero block: 0/0) to 0.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void quantize_kernel(uint8_t* __restrict__ codes, half_t* __restrict__ scales,
                                                       const half_t* __restrict__ in, size_t n_blocks, int block) {
  const size_t b = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (b >= n_blocks) return;
  const int lane = threadIdx.x & 63;
  const half_t* src = in + b * block;
  float absmax = 0.0f;
  for (int i = lane; i < block; i += WAVE) {
    absmax = fmaxf(absmax, fabsf((float)src[i]));
  }
  absmax = wave_max(absmax);
  const half_t sh = round_f16(absmax / 127.5f);
  if (lane == 0) {
    scales[b] = sh;
  }
  const float s = (float)sh;
  uint8_t* dst = codes + b * block;
  for (int i = lane; i < block; i += WAVE) {
    const float v = roundf(127.5f + (float)src[i] / s);
    dst[i] = (v >= 255.0f) ? (uint8_t)255 : (v > 0.0f ? (uint8_t)v : (uint8_t)0);
  }
}

// dequantize_absmax_uint8, transform.cu:74-87: 8 codes per thread
__global__ void dequantize_kernel(half_t* __restrict__ out, const half_t* __restrict__ scales,
                                  const uint8_t* __restrict__ codes, size_t n_chunks, int block) {
  const size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n_chunks) return;
  const uint2 q = *reinterpret_cast<const uint2*>(codes + c * 8);
  const float s = (float)scales[(c * 8) / block];
  half8_t r;
  r[0] = dequant_one(q.x & 0xFF, s);
  r[1] = dequant_one((q.x >> 8) & 0xFF, s);
  r[2] = dequant_one((q.x >> 16) & 0xFF, s);
  r[3] = dequant_one(q.x >> 24, s);
  r[4] = dequant_one(q.y & 0xFF, s);
  r[5] = dequant_one((q.y >> 8) & 0xFF, s);
  r[6] = dequant_one((q.y >> 16) & 0xFF, s);
  r[7] = dequant_one(q.y >> 24, s);
  *reinterpret_cast<half8_t*>(out + c * 8) = r;
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
__device__ __forceinline__ int sum16(uint64_t h) {
  return int(h & 0xFFFF) + int((h >> 16) & 0xFFFF) + int((h >> 32) & 0xFFFF) + int(h >> 48);
}

__global__ void fill_normal_kernel(half_t* out, size_t n, uint64_t key, float scale) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const uint64_t h1 = splitmix64(key + i);
    const uint64_t h2 = splitmix64(h1);
    const int s = sum16(h1) + sum16(h2) - 262140;
    out[i] = round_f16((float)s * scale);
  }
}

__global__ void fill_u16_kernel(uint16_t* out, size_t n, uint16_t bits) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    out[i] = bits;
  }
}

__global__ void fill_bytes_kernel(uint8_t* out, size_t bytes, uint8_t value) {
  // 16-byte stores over the aligned middle, single bytes at the ends
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t head = ((16 - ((uintptr_t)out & 15)) & 15) < bytes ? ((16 - ((uintptr_t)out & 15)) & 15) : bytes;
  const size_t n16 = (bytes - head) / 16;
  const uint32_t w = value * 0x01010101u;
  uint4* mid = reinterpret_cast<uint4*>(out + head);
  for (size_t i = tid; i < n16; i += stride) {
    mid[i] = make_uint4(w, w, w, w);
  }
  const size_t tail_start = head + n16 * 16;
  for (size_t i = tid; i < head; i += stride) out[i] = value;
  for (size_t i = tail_start + tid; i < bytes; i += stride) out[i] = value;
}

inline int grid_for(size_t n, int threads, int cap = 1 << 16) {
  size_t g = (n + threads - 1) / threads;
  return (int)(g < 1 ? 1 : (g > (size_t)cap ? cap : g));
}


// ---- error_stats, transform.cu:99-150: mean squared, largest absolute and mean absolute
// difference of two fp16 arrays.  The reference adds its blocks' contributions with atomics, in
// whatever order they arrive; here each workgroup writes its three partials and the last stage
// adds them in index order, so the result is the same on every run.
constexpr int ERR_BLOCKS = 256;

__global__ __launch_bounds__(256) void error_stats_partial_kernel(float* __restrict__ partials,
                                                                  const half_t* __restrict__ a,
                                                                  const half_t* __restrict__ b, size_t n) {
  __shared__ float red[3][4];
  float sum_sq = 0.0f, mx = 0.0f, sum = 0.0f;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)ERR_BLOCKS * 256) {
    const float d = (float)a[i] - (float)b[i];
    sum_sq = fmaf(d, d, sum_sq);
    mx = fmaxf(mx, fabsf(d));
    sum += fabsf(d);
  }
  sum_sq = wave_sum(sum_sq);
  sum = wave_sum(sum);
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) {
    red[0][threadIdx.x >> 6] = sum_sq;
    red[1][threadIdx.x >> 6] = mx;
    red[2][threadIdx.x >> 6] = sum;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    partials[blockIdx.x * 3 + 0] = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
    partials[blockIdx.x * 3 + 1] = fmaxf(fmaxf(red[1][0], red[1][1]), fmaxf(red[1][2], red[1][3]));
    partials[blockIdx.x * 3 + 2] = (red[2][0] + red[2][1]) + (red[2][2] + red[2][3]);
  }
}

__global__ __launch_bounds__(64) void error_stats_final_kernel(float* __restrict__ out,
                                                               const float* __restrict__ partials, size_t n) {
  if (threadIdx.x != 0) return;
  double sum_sq = 0.0, sum = 0.0;
  float mx = 0.0f;
  for (int i = 0; i < ERR_BLOCKS; ++i) {
    sum_sq += (double)partials[i * 3 + 0];
    mx = fmaxf(mx, partials[i * 3 + 1]);
    sum += (double)partials[i * 3 + 2];
  }
  out[0] = (float)(sum_sq / (double)n);
  out[1] = mx;
  out[2] = (float)(sum / (double)n);
}

}  // namespace

extern "C" {

// A fill kernel rather than hipMemsetAsync, so that the call may be recorded into a HIP graph.
int lcu_memset(void* dev, int byte_value, size_t bytes, void* stream) {
  if (bytes == 0) return LCU_OK;
  LCU_REQUIRE(dev != nullptr, "lcu_memset: null pointer");
  fill_bytes_kernel<<<grid_for(bytes / 16 + 1, 256, 4096), 256, 0, as_stream(stream)>>>((uint8_t*)dev, bytes,
                                                                                         (uint8_t)byte_value);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_rmsnorm(void* out_dev, const void* in_dev, const void* weights_dev, int rows, int cols, float eps,
                void* stream) {
  LCU_REQUIRE(out_dev && in_dev && weights_dev, "lcu_rmsnorm: null pointer");
  LCU_REQUIRE(rows >= 0 && cols > 0, "lcu_rmsnorm: bad shape %d x %d", rows, cols);
  if (rows == 0) return LCU_OK;
  LCU_REQUIRE(cols <= 24576, "lcu_rmsnorm: rows longer than 24576 are not supported");
  rmsnorm_kernel<<<rows, 256, (size_t)cols * 2, as_stream(stream)>>>((half_t*)out_dev, (const half_t*)in_dev,
                                                                     (const half_t*)weights_dev, cols, eps);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_rope_table_create(void** out_table_dev, int positions, int head_dim, float theta) {
  LCU_REQUIRE(out_table_dev && positions > 0 && head_dim > 0 && head_dim % 2 == 0,
              "lcu_rope_table_create: bad arguments (%d positions, head_dim %d)", positions, head_dim);
  const int half = head_dim / 2;
  const size_t n = (size_t)positions * half;
  float2* host = (float2*)malloc(n * sizeof(float2));
  LCU_REQUIRE(host != nullptr, "lcu_rope_table_create: out of host memory");
  for (int pos = 0; pos < positions; ++pos) {
    for (int p = 0; p < half; ++p) {
      // llama_cu.cu:381: angle = pos / powf(theta, float(c mod head_dim) / head_dim), c = 2p
      const float angle = (float)pos / powf(theta, (float)(2 * p) / head_dim);
      host[(size_t)pos * half + p] = make_float2(cosf(angle), sinf(angle));
    }
  }
  void* dev = nullptr;
  hipError_t e = hipMalloc(&dev, n * sizeof(float2));
  if (e == hipSuccess) e = hipMemcpy(dev, host, n * sizeof(float2), hipMemcpyHostToDevice);
  free(host);
  if (e != hipSuccess) {
    if (dev) (void)hipFree(dev);
    return set_error(LCU_E_HIP, "lcu_rope_table_create: %s", hipGetErrorString(e));
  }
  *out_table_dev = dev;
  return LCU_OK;
}

int lcu_rope(void* out_dev, const void* in_dev, int rows, int cols, int n_heads, int pos_offset,
             const void* table_dev, int table_positions, void* stream) {
  LCU_REQUIRE(out_dev && in_dev && table_dev, "lcu_rope: null pointer");
  LCU_REQUIRE(rows >= 0 && cols > 0 && n_heads > 0 && cols % n_heads == 0 && (cols / n_heads) % 2 == 0,
              "lcu_rope: bad shape rows %d cols %d heads %d", rows, cols, n_heads);
  LCU_REQUIRE(pos_offset >= 0 && pos_offset + rows <= table_positions,
              "lcu_rope: positions %d..%d outside the table of %d", pos_offset, pos_offset + rows, table_positions);
  if (rows == 0) return LCU_OK;
  dim3 grid((cols / 2 + 255) / 256, rows);
  rope_kernel<<<grid, 256, 0, as_stream(stream)>>>((half_t*)out_dev, (const half_t*)in_dev, rows, cols,
                                                   cols / n_heads, pos_offset, (const float2*)table_dev);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_rope_pair(void* a_dev, void* b_dev, int rows, int cols, int n_heads, int pos_offset, const void* table_dev,
                  int table_positions, void* stream) {
  LCU_REQUIRE(a_dev && b_dev && table_dev, "lcu_rope_pair: null pointer");
  LCU_REQUIRE(rows >= 0 && cols > 0 && n_heads > 0 && cols % n_heads == 0 && (cols / n_heads) % 2 == 0,
              "lcu_rope_pair: bad shape rows %d cols %d heads %d", rows, cols, n_heads);
  LCU_REQUIRE(pos_offset >= 0 && pos_offset + rows <= table_positions,
              "lcu_rope_pair: positions %d..%d outside the table of %d", pos_offset, pos_offset + rows, table_positions);
  LCU_REQUIRE(rows <= 65535, "lcu_rope_pair: %d rows, a grid holds 65535", rows);
  if (rows == 0) return LCU_OK;
  dim3 grid((cols / 2 + 255) / 256, rows, 2);
  rope_pair_kernel<<<grid, 256, 0, as_stream(stream)>>>((half_t*)a_dev, (half_t*)b_dev, rows, cols, cols / n_heads,
                                                        pos_offset, (const float2*)table_dev);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_softmax_rows(void* out_dev, const void* in_dev, int rows, int w, float temp, void* stream) {
  LCU_REQUIRE(out_dev && in_dev, "lcu_softmax_rows: null pointer");
  LCU_REQUIRE(rows >= 0 && w > 0 && temp > 0.0f, "lcu_softmax_rows: bad arguments rows %d w %d temp %f", rows, w,
              (double)temp);
  if (rows == 0) return LCU_OK;
  softmax_rows_kernel<<<rows, 256, 0, as_stream(stream)>>>((half_t*)out_dev, (const half_t*)in_dev, w, temp);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_sample_row(void* out_index_dev, const void* probs_dev, int n, uint64_t random, const void* random_dev,
                   void* stream) {
  LCU_REQUIRE(out_index_dev && probs_dev, "lcu_sample_row: null pointer");
  LCU_REQUIRE(n > 0 && n <= (1 << 24), "lcu_sample_row: bad length %d", n);
  sample_row_kernel<<<1, 1024, 0, as_stream(stream)>>>((int*)out_index_dev, (const half_t*)probs_dev, n, random,
                                                      (const uint64_t*)random_dev);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_softmax_argmax(void* probs_dev, void* out_index_dev, const void* logits_dev, int n, float temp,
                       void* stream) {
  LCU_REQUIRE(probs_dev && out_index_dev && logits_dev, "lcu_softmax_argmax: null pointer");
  LCU_REQUIRE(n > 0 && temp > 0.0f, "lcu_softmax_argmax: bad arguments n %d temp %f", n, (double)temp);
  LCU_REQUIRE(probs_dev != logits_dev, "lcu_softmax_argmax: probabilities may not overwrite the logits");
  softmax_argmax_kernel<<<1, 1024, 0, as_stream(stream)>>>((half_t*)probs_dev, (int*)out_index_dev,
                                                          (const half_t*)logits_dev, n, temp, nullptr);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_softmax_argmax_status(void* probs_dev, void* out_index2_dev, const void* logits_dev, int n, float temp,
                              void* stream) {
  LCU_REQUIRE(probs_dev && out_index2_dev && logits_dev, "lcu_softmax_argmax_status: null pointer");
  LCU_REQUIRE(n > 0 && temp > 0.0f, "lcu_softmax_argmax_status: bad arguments n %d temp %f", n, (double)temp);
  LCU_REQUIRE(probs_dev != logits_dev, "lcu_softmax_argmax_status: probabilities may not overwrite the logits");
  const workspace_t ws = workspace_for(as_stream(stream));
  if (ws.sync == nullptr) {
    return set_error(LCU_E_NOINIT, "lcu_softmax_argmax_status: lcu_init has not run on this device");
  }
  softmax_argmax_kernel<<<1, 1024, 0, as_stream(stream)>>>((half_t*)probs_dev, (int*)out_index2_dev,
                                                          (const half_t*)logits_dev, n, temp, ws.sync + SYNC_TIMEOUTS);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_softmax_argmax_rows(void* probs_dev, void* out_index_dev, const void* logits_dev, int rows, int n, float temp,
                            void* stream) {
  LCU_REQUIRE(probs_dev && out_index_dev && logits_dev, "lcu_softmax_argmax_rows: null pointer");
  LCU_REQUIRE(rows >= 0 && n > 0 && n % 8 == 0 && temp > 0.0f, "lcu_softmax_argmax_rows: bad arguments rows %d n %d temp %f",
              rows, n, (double)temp);
  LCU_REQUIRE(probs_dev != logits_dev, "lcu_softmax_argmax_rows: probabilities may not overwrite the logits");
  if (rows == 0) return LCU_OK;
  softmax_argmax_kernel<<<rows, 1024, 0, as_stream(stream)>>>((half_t*)probs_dev, (int*)out_index_dev,
                                                             (const half_t*)logits_dev, n, temp, nullptr);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_rope_store_batch(void* q_dev, const void* k_new_dev, const void* v_new_dev, const void* k_cache_ptrs_dev,
                         const void* v_cache_ptrs_dev, const void* pos_dev, int n_seq, int dim, int n_heads,
                         const void* table_dev, int table_positions, void* stream) {
  LCU_REQUIRE(q_dev && k_new_dev && v_new_dev && k_cache_ptrs_dev && v_cache_ptrs_dev && pos_dev && table_dev,
              "lcu_rope_store_batch: null pointer");
  LCU_REQUIRE(n_seq >= 0 && dim > 0 && n_heads > 0 && dim % n_heads == 0 && (dim / n_heads) % 2 == 0 && table_positions > 0,
              "lcu_rope_store_batch: bad shape n_seq %d dim %d heads %d", n_seq, dim, n_heads);
  if (n_seq == 0) return LCU_OK;
  dim3 grid((dim / 2 + 255) / 256, n_seq);
  rope_store_batch_kernel<<<grid, 256, 0, as_stream(stream)>>>(
      (half_t*)q_dev, (const half_t*)k_new_dev, (const half_t*)v_new_dev, (half_t* const*)k_cache_ptrs_dev,
      (half_t* const*)v_cache_ptrs_dev, (const int*)pos_dev, dim, dim / n_heads, (const float2*)table_dev,
      table_positions - 1);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_silu_mul(void* out_dev, const void* a_dev, const void* b_dev, size_t size, void* stream) {
  LCU_REQUIRE(out_dev && a_dev && b_dev, "lcu_silu_mul: null pointer");
  if (size == 0) return LCU_OK;
  LCU_REQUIRE(size <= ((size_t)1 << 40), "lcu_silu_mul: size too large");
  const unsigned grid = (unsigned)((size + 2047) / 2048);
  if ((((uintptr_t)out_dev | (uintptr_t)a_dev | (uintptr_t)b_dev) & 15) == 0) {
    silu_mul_kernel<true><<<grid, 256, 0, as_stream(stream)>>>((half_t*)out_dev, (const half_t*)a_dev,
                                                               (const half_t*)b_dev, size);
  } else {
    silu_mul_kernel<false><<<grid, 256, 0, as_stream(stream)>>>((half_t*)out_dev, (const half_t*)a_dev,
                                                                (const half_t*)b_dev, size);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_embed(void* out_dev, const void* ids_dev, int n_ids, int dim, const void* table_dev, int n_vocab,
              void* stream) {
  LCU_REQUIRE(out_dev && ids_dev && table_dev, "lcu_embed: null pointer");
  LCU_REQUIRE(n_ids >= 0 && dim > 0 && dim % 8 == 0 && n_vocab > 0, "lcu_embed: bad shape n %d dim %d", n_ids, dim);
  if (n_ids == 0) return LCU_OK;
  embed_kernel<<<n_ids, 256, 0, as_stream(stream)>>>((half_t*)out_dev, (const short*)ids_dev, dim,
                                                     (const half_t*)table_dev, n_vocab);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_embed_u8(void* out_dev, const void* ids_dev, int n_ids, int dim, const void* codes_dev,
                 const void* scales_dev, int block, int n_vocab, void* stream) {
  LCU_REQUIRE(out_dev && ids_dev && codes_dev && scales_dev, "lcu_embed_u8: null pointer");
  LCU_REQUIRE(n_ids >= 0 && dim > 0 && block > 0 && dim % block == 0 && n_vocab > 0,
              "lcu_embed_u8: bad shape n %d dim %d block %d", n_ids, dim, block);
  if (n_ids == 0) return LCU_OK;
  if (dim % 16 == 0 && block % 16 == 0) {
    embed_u8x16_kernel<<<dim3(n_ids, (dim + 4095) / 4096), 256, 0, as_stream(stream)>>>(
        (half_t*)out_dev, (const short*)ids_dev, dim, (const uint8_t*)codes_dev, (const half_t*)scales_dev, block,
        n_vocab);
  } else {
    embed_u8_kernel<<<n_ids, 256, 0, as_stream(stream)>>>((half_t*)out_dev, (const short*)ids_dev, dim,
                                                          (const uint8_t*)codes_dev, (const half_t*)scales_dev, block,
                                                          n_vocab);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_embed_rmsnorm(void* x_out_dev, void* norm_out_dev, const void* ids_dev, int n_ids, int dim,
                      const void* table_dev, const void* scales_dev, int block, int n_vocab, const void* weights_dev,
                      float eps, void* stream) {
  LCU_REQUIRE(x_out_dev && norm_out_dev && ids_dev && table_dev && weights_dev, "lcu_embed_rmsnorm: null pointer");
  LCU_REQUIRE(n_ids >= 0 && dim > 0 && dim % 8 == 0 && dim <= 8192 && n_vocab > 0,
              "lcu_embed_rmsnorm: bad shape n %d dim %d (dim a multiple of 8, at most 8192)", n_ids, dim);
  LCU_REQUIRE(block == 0 || (scales_dev && block % 8 == 0 && dim % block == 0),
              "lcu_embed_rmsnorm: block %d unsupported (0 for an fp16 table, else a multiple of 8 dividing dim, with scales)",
              block);
  if (n_ids == 0) return LCU_OK;
  if (block > 0) {
    embed_rmsnorm_kernel<true><<<n_ids, 256, (size_t)dim * 2, as_stream(stream)>>>(
        (half_t*)x_out_dev, (half_t*)norm_out_dev, (const short*)ids_dev, dim, table_dev, (const half_t*)scales_dev, block,
        n_vocab, (const half_t*)weights_dev, eps);
  } else {
    embed_rmsnorm_kernel<false><<<n_ids, 256, (size_t)dim * 2, as_stream(stream)>>>(
        (half_t*)x_out_dev, (half_t*)norm_out_dev, (const short*)ids_dev, dim, table_dev, nullptr, 0, n_vocab,
        (const half_t*)weights_dev, eps);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_exp_f32(void* out_dev, const void* in_dev, size_t n, void* stream) {
  LCU_REQUIRE(out_dev && in_dev, "lcu_exp_f32: null pointer");
  if (n == 0) return LCU_OK;
  exp_kernel<<<(unsigned)((n + 255) / 256), 256, 0, as_stream(stream)>>>((float*)out_dev, (const float*)in_dev, n);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_argmax_f16(void* out_index_dev, const void* values_dev, int n, void* stream) {
  LCU_REQUIRE(out_index_dev && values_dev && n > 0, "lcu_argmax_f16: bad arguments");
  argmax_kernel<<<1, 1024, 0, as_stream(stream)>>>((int*)out_index_dev, (const half_t*)values_dev, n);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_quantize_absmax_u8(void* codes_dev, void* scales_dev, const void* in_dev, size_t rows, size_t cols,
                           int block, void* stream) {
  LCU_REQUIRE(codes_dev && scales_dev && in_dev, "lcu_quantize_absmax_u8: null pointer");
  LCU_REQUIRE(block > 0 && cols % block == 0, "lcu_quantize_absmax_u8: cols %zu not a multiple of block %d", cols,
              block);
  const size_t n_blocks = rows * (cols / block);
  if (n_blocks == 0) return LCU_OK;
  LCU_REQUIRE((n_blocks + 3) / 4 < ((size_t)1 << 31), "lcu_quantize_absmax_u8: tensor too large");
  quantize_kernel<<<(unsigned)((n_blocks + 3) / 4), 256, 0, as_stream(stream)>>>(
      (uint8_t*)codes_dev, (half_t*)scales_dev, (const half_t*)in_dev, n_blocks, block);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_dequantize_absmax_u8(void* out_dev, const void* scales_dev, const void* codes_dev, size_t rows,
                             size_t cols, int block, void* stream) {
  LCU_REQUIRE(out_dev && scales_dev && codes_dev, "lcu_dequantize_absmax_u8: null pointer");
  LCU_REQUIRE(block > 0 && block % 8 == 0 && cols % block == 0,
              "lcu_dequantize_absmax_u8: cols %zu / block %d unsupported (block must be a multiple of 8)", cols, block);
  const size_t n_chunks = rows * cols / 8;
  if (n_chunks == 0) return LCU_OK;
  LCU_REQUIRE((n_chunks + 255) / 256 < ((size_t)1 << 31), "lcu_dequantize_absmax_u8: tensor too large");
  dequantize_kernel<<<(unsigned)((n_chunks + 255) / 256), 256, 0, as_stream(stream)>>>(
      (half_t*)out_dev, (const half_t*)scales_dev, (const uint8_t*)codes_dev, n_chunks, block);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_fill_normal_f16(void* out_dev, size_t n, uint64_t seed, uint64_t stream_id, float std, void* stream) {
  LCU_REQUIRE(out_dev || n == 0, "lcu_fill_normal_f16: null pointer");
  if (n == 0) return LCU_OK;
  uint64_t z = seed ^ (stream_id * 0xD1B54A32D192ED03ull);
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  const uint64_t key = z ^ (z >> 31);
  const double sigma = sqrt(8.0 * (65536.0 * 65536.0 - 1.0) / 12.0);
  const float scale = (float)((double)std / sigma);
  fill_normal_kernel<<<grid_for(n, 256, 8192), 256, 0, as_stream(stream)>>>((half_t*)out_dev, n, key, scale);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_fill_f16(void* out_dev, size_t n, uint16_t bits, void* stream) {
  LCU_REQUIRE(out_dev || n == 0, "lcu_fill_f16: null pointer");
  if (n == 0) return LCU_OK;
  fill_u16_kernel<<<grid_for(n, 256, 4096), 256, 0, as_stream(stream)>>>((uint16_t*)out_dev, n, bits);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_error_stats(void* out3_dev, const void* a_dev, const void* b_dev, size_t n, void* stream) {
  LCU_REQUIRE(out3_dev && a_dev && b_dev && n > 0, "lcu_error_stats: bad arguments");
  const workspace_t ws = workspace_for(as_stream(stream));
  if (ws.ptr == nullptr) return set_error(LCU_E_NOINIT, "lcu_error_stats: lcu_init has not run on this device");
  float* partials = (float*)ws.ptr;  // 256 x 3 floats of the stream's workspace
  error_stats_partial_kernel<<<ERR_BLOCKS, 256, 0, as_stream(stream)>>>(partials, (const half_t*)a_dev,
                                                                        (const half_t*)b_dev, n);
  LCU_LAUNCH_CHECK();
  error_stats_final_kernel<<<1, 64, 0, as_stream(stream)>>>((float*)out3_dev, partials, n);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

}  // extern "C"
