// Causal self-attention over the KV cache: the reference's matmul_qk -> softmax_rows -> matmul_qkv
// chain (llama_cu.cu:400-428, 433-499, 511-531; launch sites 1161-1171) without its
// [n_heads, n, T] score tensor in memory and without its per-layer cudaMalloc (1120-1122).
//
// The reference's three rounding points are kept: scores are rounded to fp16, probabilities are
// rounded to fp16 after a softmax over the whole row (true row maximum and row sum, no online
// rescaling), and the probability-weighted sum of V runs in fp32 and is rounded once.
//
// Layouts: q [n_new, dim]; k, v = first T rows of a [*, dim] cache (K already rotated); head h is
// columns h*128 .. h*128+127.
//
// Decode (n_new == 1), up to 1024 cached rows: one 1024-thread workgroup per head does scores,
// softmax and the weighted sum in one launch; beyond, two launches (see dec_scores_kernel); 16 lanes share one cached row (16 bytes each), 64 rows per pass, 16 passes of
// loads in flight per thread.
// Prefill (n_new > 1), matrix-core bound: one workgroup per (16 or 32 query rows, head); Q.K^T by
// v_mfma_f32_16x16x32_f16 into an LDS score strip [rows][T], softmax in LDS, P.V by MFMA with V
// staged row-major in LDS; the next 64-row chunk of K or V is in flight while the current one is
// multiplied.
#include <atomic>

#include "common.hpp"

using namespace lcu;

namespace {

constexpr int HD = 128;            // head_dim
constexpr int MAX_T_DECODE = 4096;
constexpr int MAX_HEADS = 64;
constexpr int DEC_THREADS = 1024;
constexpr int DEC_GROUPS = DEC_THREADS / 16;  // cache rows per pass: 16 lanes x 16 bytes cover one row of a head
constexpr int DEC_FLIGHT = 16;                // passes whose loads are requested together

// One workgroup per head, the whole attention of one new token in a single launch.  The work is
// a few hundred KB per head, so the kernel is organised around load latency: 1024 threads, every
// thread keeps up to 16 independent 16-byte loads in flight (1024 cached rows per round; rows past
// T are masked off per lane, which costs no load bandwidth), the first V rows are requested before
// the softmax statistics are reduced, and the 16-lane dot products are summed with
// data-parallel-primitive moves instead of LDS shuffles.
__global__ __launch_bounds__(DEC_THREADS) void decode_attention_kernel(half_t* __restrict__ out,
                                                                       const half_t* __restrict__ q,
                                                                       const half_t* __restrict__ k,
                                                                       const half_t* __restrict__ v, int T_cap, int dim,
                                                                       const int* __restrict__ pos_dev,
                                                                       const half_t* const* __restrict__ k_ptrs,
                                                                       const half_t* const* __restrict__ v_ptrs) {
  __shared__ half_t sc[MAX_T_DECODE];  // fp16 scores, then fp16 probabilities
  __shared__ float gsum[DEC_GROUPS][HD + 4];
  __shared__ float red[16];
  // a batch of sequences: blockIdx.y picks the sequence, i.e. its row of q / out, its caches and
  // its position
  if (k_ptrs) {
    const int b = blockIdx.y;
    k = k_ptrs[b];
    v = v_ptrs[b];
    q += (size_t)b * dim;
    out += (size_t)b * dim;
    pos_dev += b;
  }
  const int h = blockIdx.x;
  const int tid = threadIdx.x;
  const int sub = tid & 15, grp = tid >> 4;
  const half_t* kh = k + h * HD + sub * 8;
  const half_t* vh = v + h * HD + sub * 8;
  // position kept on the device (graph replay): the new row is row *pos_dev, T_cap is the cap
  int T = T_cap;
  if (pos_dev) {
    T = min(max(*pos_dev + 1, 1), T_cap);
  }
  const half8_t qh = *reinterpret_cast<const half8_t*>(q + h * HD + sub * 8);
  const float denom = sqrtf((float)HD);

  // ---- scores, llama_cu.cu:400-428 (no mask: the one new row sees every cached row)
  int p0 = 0;
  do {
    half8_t kv[DEC_FLIGHT];
#pragma unroll
    for (int f = 0; f < DEC_FLIGHT; ++f) {
      const int p = p0 + f * DEC_GROUPS + grp;
      kv[f] = p < T ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(kh + (size_t)p * dim))
                    : (half8_t)(0.0f);
    }
#pragma unroll
    for (int f = 0; f < DEC_FLIGHT; ++f) {
      const int p = p0 + f * DEC_GROUPS + grp;
      float s = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s = fmaf((float)qh[e], (float)kv[f][e], s);
      s = row16_sum(s);
      if (sub == 0 && p < T) sc[p] = round_f16(s / denom);  // 425
    }
    p0 += DEC_GROUPS * DEC_FLIGHT;
  } while (p0 < T);
  // first V rows: independent of the statistics below
  half8_t vv[DEC_FLIGHT];
#pragma unroll
  for (int f = 0; f < DEC_FLIGHT; ++f) {
    const int p = f * DEC_GROUPS + grp;
    vv[f] = p < T ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(vh + (size_t)p * dim)) : (half8_t)(0.0f);
  }
  __syncthreads();

  // ---- softmax_rows, llama_cu.cu:433-499: the first 256 threads play the reference's 256 threads
  // (thread t owns elements t, t+256, ...), so the exponential sum is associated identically
  float m = -INFINITY;
  if (tid < 256) {
    for (int i = tid; i < T; i += 256) m = fmaxf(m, (float)sc[i]);
  }
  m = wave_max(m);
  if ((tid & 63) == 0) red[tid >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));  // wavefronts 4..15 hold -inf
  __syncthreads();
  float s = 0.0f;
  if (tid < 256) {
    for (int i = tid; i < T; i += 256) s += exp_ieee((float)sc[i] - m);
  }
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) s += __shfl_xor(s, off, WAVE);
  if (tid < 256 && (tid & 31) == 0) red[tid >> 5] = s;
  __syncthreads();
  float total = red[tid & 7];
#pragma unroll
  for (int off = 4; off > 0; off >>= 1) total += __shfl_xor(total, off, WAVE);
  __syncthreads();
  for (int i = tid; i < T; i += DEC_THREADS) sc[i] = round_f16(exp_ieee((float)sc[i] - m) / total);  // 497
  __syncthreads();

  // ---- matmul_qkv, llama_cu.cu:511-531: group g adds rows g, g+64, ... in ascending order
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
  for (p0 = 0; p0 < T; p0 += DEC_GROUPS * DEC_FLIGHT) {
    if (p0 > 0) {
#pragma unroll
      for (int f = 0; f < DEC_FLIGHT; ++f) {
        const int p = p0 + f * DEC_GROUPS + grp;
        vv[f] = p < T ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(vh + (size_t)p * dim))
                      : (half8_t)(0.0f);
      }
    }
#pragma unroll
    for (int f = 0; f < DEC_FLIGHT; ++f) {
      const int p = p0 + f * DEC_GROUPS + grp;
      if (p < T) {
        const float prob = (float)sc[p];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = fmaf(prob, (float)vv[f][e], acc[e]);
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) gsum[grp][sub * 8 + e] = acc[e];
  __syncthreads();
  if (tid < HD) {
    float o = 0.0f;
#pragma unroll 8
    for (int g = 0; g < DEC_GROUPS; ++g) o += gsum[g][tid];
    out[h * HD + tid] = round_f16(o);  // 529
  }
}

// ---- decode attention in two launches -----------------------------------------------------------
// One compute unit's load path moves about 120 GB/s, so one workgroup per head cannot stream a
// head's K and V (295 KB at T = 576, 1 MB at T = 2048) any faster than that, on 32 of 256 compute
// units.  Split along T the scores need no cross-workgroup step at all, and the second launch
// splits along the head's 128 output columns instead, each workgroup repeating the (cheap) softmax
// of its head's row: no workgroup ever waits for another.
//
// dec_scores_kernel: workgroup (chunk of 64 cache rows, head): 16 lanes per row, 4 rows per
//   thread group in flight; writes the fp16 scores of llama_cu.cu:400-428 to scores[head][t].
// dec_softmax_pv_kernel: workgroup (32-column slice, head), 256 threads: requests its V slice
//   first, then the reference's softmax over the row (the 256 threads are the reference's 256:
//   same association of the sum, llama_cu.cu:433-499), then the weighted sum (511-531).
constexpr int SC_ROWS = 64;      // cache rows per scores workgroup
constexpr int PV_COLS = 32;      // output columns per second-stage workgroup
constexpr int PV_FLIGHT = 16;    // 64-row passes whose loads are requested together (1024 rows)
constexpr int SINGLE_LAUNCH_MAX_T = 1024;

__global__ __launch_bounds__(256) void dec_scores_kernel(half_t* __restrict__ scores, const half_t* __restrict__ q,
                                                         const half_t* __restrict__ k, int T_cap, int dim,
                                                         const int* __restrict__ pos_dev) {
  int T = T_cap;
  if (pos_dev) T = min(max(*pos_dev + 1, 1), T_cap);
  const int t0 = blockIdx.x * SC_ROWS;
  if (t0 >= T) return;
  const int h = blockIdx.y;
  const int tid = threadIdx.x, sub = tid & 15, grp = tid >> 4;  // 16 row groups
  const half8_t qh = *reinterpret_cast<const half8_t*>(q + h * HD + sub * 8);
  const half_t* kh = k + h * HD + sub * 8;
  half8_t kv[SC_ROWS / 16];
#pragma unroll
  for (int f = 0; f < SC_ROWS / 16; ++f) {
    const int p = min(t0 + f * 16 + grp, T - 1);
    kv[f] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(kh + (size_t)p * dim));
  }
  const float denom = sqrtf((float)HD);
#pragma unroll
  for (int f = 0; f < SC_ROWS / 16; ++f) {
    const int p = t0 + f * 16 + grp;
    float s = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s = fmaf((float)qh[e], (float)kv[f][e], s);
    s = row16_sum(s);
    if (sub == 0 && p < T) scores[(size_t)h * T_cap + p] = round_f16(s / denom);  // 425
  }
}

__global__ __launch_bounds__(256) void dec_softmax_pv_kernel(half_t* __restrict__ out,
                                                             const half_t* __restrict__ scores,
                                                             const half_t* __restrict__ v, int T_cap, int dim,
                                                             const int* __restrict__ pos_dev) {
  __shared__ half_t sc[MAX_T_DECODE];  // fp16 scores, then fp16 probabilities
  __shared__ float gsum[64][PV_COLS + 1];
  __shared__ float red[8];
  int T = T_cap;
  if (pos_dev) T = min(max(*pos_dev + 1, 1), T_cap);
  const int slice = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, sub = tid & 3, grp = tid >> 2;  // 4 lanes x 16 bytes = the 32 columns of a row
  const half_t* vh = v + h * HD + slice * PV_COLS + sub * 8;
  // the first 1024 rows of the V slice: independent of everything below
  half8_t vv[PV_FLIGHT];
#pragma unroll
  for (int f = 0; f < PV_FLIGHT; ++f) {
    const int p = f * 64 + grp;
    vv[f] = p < T ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(vh + (size_t)p * dim)) : (half8_t)(0.0f);
  }
  for (int i = tid; i < T; i += 256) sc[i] = scores[(size_t)h * T_cap + i];
  __syncthreads();
  // softmax_rows: thread t owns elements t, t+256, ...
  float m = -INFINITY;
  for (int i = tid; i < T; i += 256) m = fmaxf(m, (float)sc[i]);
  m = block256_max(m, red);
  float s = 0.0f;
  for (int i = tid; i < T; i += 256) s += exp_ieee((float)sc[i] - m);
  const float total = block256_sum_ref_order(s, red);
  for (int i = tid; i < T; i += 256) sc[i] = round_f16(exp_ieee((float)sc[i] - m) / total);  // 497
  __syncthreads();
  // matmul_qkv: row group g adds rows g, g+64, ... in ascending order, then the groups are added
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
  for (int p0 = 0; p0 < T; p0 += 64 * PV_FLIGHT) {
    if (p0 > 0) {
#pragma unroll
      for (int f = 0; f < PV_FLIGHT; ++f) {
        const int p = p0 + f * 64 + grp;
        vv[f] = p < T ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(vh + (size_t)p * dim))
                      : (half8_t)(0.0f);
      }
    }
#pragma unroll
    for (int f = 0; f < PV_FLIGHT; ++f) {
      const int p = p0 + f * 64 + grp;
      if (p < T) {
        const float prob = (float)sc[p];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = fmaf(prob, (float)vv[f][e], acc[e]);
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) gsum[grp][sub * 8 + e] = acc[e];
  __syncthreads();
  if (tid < PV_COLS) {
    float o = 0.0f;
#pragma unroll 8
    for (int g = 0; g < 64; ++g) o += gsum[g][tid];
    out[h * HD + slice * PV_COLS + tid] = round_f16(o);  // 529
  }
}

// ---- decode attention spread over eight workgroups per head, one launch -------------------------
// A compute unit fetches cold cache rows at about 30 GB/s (its count of outstanding misses, not its
// 120 GB/s path, is the limit), so one workgroup per head spends 5 of its 9 us waiting for the
// head's K alone.  Here eight 256-thread workgroups share a head: each takes every eighth block of
// 16 cached rows for the scores and 16 of the head's 128 columns for the weighted sum.  The
// softmax needs the whole row of scores, so the workgroups of a head hand theirs to one another
// inside the launch:
//   * a score travels as an 8-byte word {fp16 score, epoch of the launch}, written with one
//     device-scope store (through to memory) and read with device-scope loads, so the hand-over
//     does not depend on which caches the workgroups share and needs no flag, fence or reset: a
//     reader asks for the words it needs until every one carries this launch's epoch, a value that
//     no earlier launch can have left in them (host-drawn epochs have the top bit set and count
//     up; device epochs are step counter << 10 | salt with the top bit clear);
//   * the wait is bounded: the eight workgroups of a head have neighbouring indices, all are
//     resident at once on any idle device (256 threads, 7 KB of LDS), and a wait that runs out
//     anyway counts itself in the stream's sync area (lcu_sync_timeouts) and goes on;
//   * workgroup b runs on XCD b % 8 (round-robin dispatch), so b = xcd + 8 * (slice + 8 * i) keeps
//     a head's workgroups on one XCD, where they share the L2 lines of the head's K and V rows.
// Every sum is associated as in decode_attention_kernel (16 lanes x 8 elements per score; the
// reference's 256-thread softmax; row groups g, g + 64, ... then the 64 groups in order), so the
// bits are the same.  NJ: the row bound is 256 * NJ.
constexpr int SPREAD = 8;
constexpr int SPREAD_SPIN_LIMIT = 1 << 16;

template <int NJ>
__global__ __launch_bounds__(256) void decode_attention_spread_kernel(
    half_t* __restrict__ out, const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    int T_cap, int dim, int n_heads, const int* __restrict__ pos_dev, uint64_t* __restrict__ scores,
    const uint32_t* __restrict__ seq_dev, uint32_t epoch, uint32_t* __restrict__ timeouts) {
  __shared__ half_t sc[256 * NJ];  // fp16 probabilities
  __shared__ float gsum[64][17];
  __shared__ __attribute__((aligned(16))) float red[8];
  const int b = blockIdx.x, tid = threadIdx.x;
  const int slice = (b >> 3) & 7, h = (b & 7) + 8 * (b >> 6);
  if (h >= n_heads) return;
  int T = T_cap;
  if (pos_dev) T = min(max(*pos_dev + 1, 1), T_cap);
  if (seq_dev) epoch = (epoch | (*seq_dev << 10)) & 0x7fffffffu;

  // ---- scores of rows slice * 16 + grp + 128 f, llama_cu.cu:400-428
  const int sub = tid & 15, grp = tid >> 4;
  const half_t* kh = k + h * HD + sub * 8;
  uint64_t* srow = scores + (size_t)h * T_cap;
  const float denom = sqrtf((float)HD);
  half8_t qh;
  for (int p0 = 0; p0 < T; p0 += 1024) {
    half8_t kv[8];
#pragma unroll
    for (int f = 0; f < 8; ++f) {
      const int p = p0 + slice * 16 + grp + 128 * f;
      kv[f] = p < T ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(kh + (size_t)p * dim))
                    : (half8_t)(0.0f);
    }
    if (p0 == 0) qh = *reinterpret_cast<const half8_t*>(q + h * HD + sub * 8);
#pragma unroll
    for (int f = 0; f < 8; ++f) {
      const int p = p0 + slice * 16 + grp + 128 * f;
      float s = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s = fmaf((float)qh[e], (float)kv[f][e], s);
      s = row16_sum(s);
      if (sub == 0 && p < T) {
        const half_t val = round_f16(s / denom);  // 425
        const uint64_t word = ((uint64_t)epoch << 32) | __builtin_bit_cast(unsigned short, val);
        __hip_atomic_store(srow + p, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  // the first 1024 rows of this workgroup's 16 columns of V: 4 lanes x 8 bytes per row, row group
  // vg takes rows vg + 64 f; on their way during the hand-over and the softmax
  const int vsub = tid & 3, vg = tid >> 2;
  const half_t* vh = v + h * HD + slice * 16 + vsub * 4;
  half4_t vv[16];
#pragma unroll
  for (int f = 0; f < 16; ++f) {
    const int p = vg + 64 * f;
    vv[f] = p < T ? *reinterpret_cast<const half4_t*>(vh + (size_t)p * dim) : (half4_t)(0.0f);
  }

  // ---- hand-over and softmax_rows, llama_cu.cu:433-499: thread t owns elements t, t + 256, ... as
  // there; every wavefront asks for its elements until all of them are this launch's
  float x[NJ];
  {
    uint64_t raw[NJ];
    int spins = 0;
    while (true) {
      // four words per statement; an element past T reads word 0 of the row instead and is ignored
#pragma unroll
      for (int j = 0; j < NJ; j += 4) {
        uint64_t four[4];
        load_words_device_scope(four, srow + (tid + 256 * j < T ? tid + 256 * j : 0),
                                srow + (tid + 256 * (j + 1) < T ? tid + 256 * (j + 1) : 0),
                                srow + (tid + 256 * (j + 2) < T ? tid + 256 * (j + 2) : 0),
                                srow + (tid + 256 * (j + 3) < T ? tid + 256 * (j + 3) : 0));
#pragma unroll
        for (int e = 0; e < 4; ++e) raw[j + e] = tid + 256 * (j + e) < T ? four[e] : ((uint64_t)epoch << 32) | 0xfc00u;
      }
      bool stale = false;
#pragma unroll
      for (int j = 0; j < NJ; ++j) stale |= (uint32_t)(raw[j] >> 32) != epoch;
      if (__builtin_amdgcn_ballot_w64(stale) == 0) break;
      if (++spins > SPREAD_SPIN_LIMIT) {
        if ((tid & 63) == 0) atomicAdd(timeouts, 1u);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) x[j] = (float)__builtin_bit_cast(half_t, (unsigned short)raw[j]);
  }
  float m = x[0];
#pragma unroll
  for (int j = 1; j < NJ; ++j) m = fmaxf(m, x[j]);
  m = block256_max_dpp(m, red);
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    if (tid + 256 * j < T) {
      x[j] = exp_ieee(x[j] - m);
      s += x[j];
    }
  }
  const float total = block256_sum_ref_order_dpp(s, red);
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    if (tid + 256 * j < T) sc[tid + 256 * j] = round_f16(x[j] / total);  // 497
  }
  __syncthreads();

  // ---- matmul_qkv, llama_cu.cu:511-531, for this workgroup's 16 columns
  float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int p0 = 0; p0 < T; p0 += 1024) {
    if (p0 > 0) {
#pragma unroll
      for (int f = 0; f < 16; ++f) {
        const int p = p0 + vg + 64 * f;
        vv[f] = p < T ? *reinterpret_cast<const half4_t*>(vh + (size_t)p * dim) : (half4_t)(0.0f);
      }
    }
#pragma unroll
    for (int f = 0; f < 16; ++f) {
      const int p = p0 + vg + 64 * f;
      if (p < T) {
        const float prob = (float)sc[p];
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] = fmaf(prob, (float)vv[f][c], acc[c]);
      }
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) gsum[vg][vsub * 4 + c] = acc[c];
  __syncthreads();
  if (tid < 16) {
    float o = 0.0f;
#pragma unroll
    for (int g = 0; g < 64; ++g) o += gsum[g][tid];
    out[h * HD + slice * 16 + tid] = round_f16(o);  // 529
  }
}

// ---- decode attention, the Wo product with the residual sum, and the RMS norm that follows, in one
// launch (llama_cu.cu:1161-1176 for one new token, fp16 weights) ---------------------------------
// The attention above leaves HBM idle for its whole length, the Wo product behind it streams 2 dim^2
// bytes and then a one-workgroup norm waits for a launch of its own.  Here workgroup (head h, slice)
// -- 1024 threads, one per compute unit -- owns the 16 rows h * 128 + slice * 16 .. + 15 of
// everything: it computes those 16 columns of the attention output (its first four wavefronts run
// decode_attention_spread_kernel's code), keeps its 16 rows of Wo in the registers of the other
// twelve (requested in batches while the attention runs, so the matrix streams in behind it), and
// after two more hand-overs of the same kind
// ({two halves, epoch} words through memory) finishes those rows of x + Wo . att and of the
// normalised row.  The sums keep the order of the kernels this replaces: a row of Wo is summed by
// four wavefronts as gemv_kernel<false, 1 or 2, 2, 0> does it (chunk c of 512 elements to
// wavefront (c / 2) % 4, two accumulators per lane, wave_sum, wavefronts in order, then
// fmaf(1, x, sum)), the norm by 256 threads as rmsnorm_kernel.  NB: dim <= 4096 * NB.
// ---- phase timeline of the fused launch (diagnostic builds only: -DLCU_PHASE_TIMELINE) ------------
// Thread 0 of every workgroup (and the first lane of its first Wo wavefront) notes the 100 MHz
// real-time counter at the ends of the launch's phases into a device array, one row per launch (by
// salt) and workgroup; lcu_debug_timeline_read copies it out.  Nothing of this exists in the
// ordinary build.
#ifdef LCU_PHASE_TIMELINE
constexpr int TL_POINTS = 16, TL_LAUNCHES = 64, TL_GROUPS = 512;
static __device__ uint64_t phase_timeline[TL_LAUNCHES * TL_GROUPS * TL_POINTS];
#define TL_MARK(point)                                                                                          \
  do {                                                                                                          \
    if (threadIdx.x == ((point) >= 12 ? 256 : 0)) {                                                             \
      phase_timeline[((tl_launch & (TL_LAUNCHES - 1)) * TL_GROUPS + blockIdx.x) * TL_POINTS + (point)] =        \
          __builtin_amdgcn_s_memrealtime();                                                                     \
    }                                                                                                           \
  } while (0)
#else
#define TL_MARK(point) \
  do {                 \
  } while (0)
#endif

constexpr int FUSED_THREADS = 1024;
constexpr int FUSED_PAD_LDS = 72 << 10;  // dynamic LDS nobody touches: a second workgroup does not fit the compute unit

static_assert(EXCH_ATT == MAX_HEADS * MAX_T_DECODE, "the scores' area");

// All threads of the workgroup: waits until the dim / 2 {half2, epoch} words at `words` carry this
// launch's epoch and copies their halves to xs[0 .. dim).  Every thread asks for two words at a time.
__device__ __forceinline__ void gather_row(half_t* xs, const uint64_t* words, int dim, uint32_t epoch,
                                           uint32_t* timeouts) {
  const int tid = threadIdx.x;
  for (int w0 = tid * 2; w0 < dim / 2; w0 += FUSED_THREADS * 2) {
    uint4_t raw[1];
    int spins = 0;
    while (true) {
      load_word_pairs_device_scope(raw, words + w0);
      const bool stale = raw[0][1] != epoch || raw[0][3] != epoch;
      if (__builtin_amdgcn_ballot_w64(stale) == 0) break;
      if (++spins > SPREAD_SPIN_LIMIT) {
        if ((tid & 63) == 0) atomicAdd(timeouts, 1u);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    uint32_t* dst = reinterpret_cast<uint32_t*>(xs + 2 * w0);
    dst[0] = raw[0][0];
    dst[1] = raw[0][2];
  }
}

// threads 0..15 hold one half each (value of row base + tid): pairs go out as {half2, epoch} words
__device__ __forceinline__ void publish16(uint64_t* words, int base, half_t value, uint32_t epoch) {
  const int tid = threadIdx.x;
  const uint32_t mine = __builtin_bit_cast(unsigned short, value);
  const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0xB1, 0xF, 0xF, true);  // lane ^ 1
  if ((tid & 1) == 0) {
    const uint64_t word = ((uint64_t)epoch << 32) | (other << 16) | mine;
    __hip_atomic_store(words + (base + tid) / 2, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <int NB>
__global__ __launch_bounds__(FUSED_THREADS) void decode_attention_wo_norm_kernel(
    half_t* __restrict__ x_io, half_t* __restrict__ norm_out, const half_t* __restrict__ q,
    const half_t* __restrict__ k, const half_t* __restrict__ v, const half_t* __restrict__ wo,
    const half_t* __restrict__ norm_w, float eps, int T_cap, int dim, int n_heads, const int* __restrict__ pos_dev,
    uint64_t* __restrict__ exch, const uint32_t* __restrict__ seq_dev, uint32_t epoch,
    uint32_t* __restrict__ timeouts) {
  constexpr int NJ = 4;  // rows of up to 1024 scores
  __shared__ half_t sc[256 * NJ];
  __shared__ float gsum[64][17];
  __shared__ __attribute__((aligned(16))) float red[8];
  __shared__ __attribute__((aligned(16))) half_t xs[4096 * NB];
  __shared__ float part[16][4];
  const int b = blockIdx.x, tid = threadIdx.x;
  const int slice = (b >> 3) & 7, h = (b & 7) + 8 * (b >> 6);
  if (h >= n_heads) return;
  const int lane = tid & 63, wave = tid >> 6, team = wave >> 2, tw = wave & 3;
  const int row0 = h * HD + slice * 16;  // first of this workgroup's 16 rows / columns
  const bool att = tid < 256;
  int T = T_cap;
  if (pos_dev) T = min(max(*pos_dev + 1, 1), T_cap);
#ifdef LCU_PHASE_TIMELINE
  const uint32_t tl_launch = epoch;  // the salt: the layer
#endif
  TL_MARK(0);
  if (seq_dev) epoch = (epoch | (*seq_dev << 10)) & 0x7fffffffu;
  uint64_t* srow = exch + (size_t)h * T_cap;
  // what the 16 finishing threads need from memory at the very end, requested now
  half_t x_old = (half_t)0.0f, nw_mine = (half_t)0.0f;
  if (tid < 16) {
    x_old = x_io[row0 + tid];
    nw_mine = norm_w[row0 + tid];
  }

  // ---- this workgroup's rows of Wo live in the registers of wavefronts 4-15: row team - 1 + 3 i of
  // the 16 goes to the four wavefronts of `team` (1..3).  The requests go out in four batches, one
  // before the attention starts and one behind each of its first three barriers, and nobody waits
  // for them before the attention output is in: the compute unit's memory pipeline serves requests
  // in order, so the attention's own hand-over reads only ever queue behind one batch.
  constexpr int ROWS = 6, LOADS = ROWS * NB * 2;
  constexpr int B0 = LOADS / 3, B1 = B0 + LOADS / 4, B2 = B1 + LOADS / 4;
  uint4_t wreg[ROWS][NB][2];
  auto load_wo = [&](int first, int last) {
    if (team == 0) return;
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int r = min(team - 1 + 3 * i, 15);
      const half_t* wrow = wo + (size_t)(row0 + r) * dim;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int j = (i * NB + nb) * 2 + u;
          if (j >= first && j < last) {
            const int kk = min(((nb * 4 + tw) * 2 + u) * 512 + lane * 8, dim - 8);
            wreg[i][nb][u] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(wrow + kk));
          }
        }
      }
    }
  };
  if (team > 0) __builtin_amdgcn_s_sleep(24);  // lets the attention's K and V requests go first
  load_wo(0, B0);

  // ---- attention, first part (wavefronts 0-3): scores of this slice, hand-over, row maximum
  const int vsub = tid & 3, vg = tid >> 2;
  half4_t vv[16];
  float x[NJ];
  float m = -INFINITY;
  if (att) {
    const int sub = tid & 15, grp = tid >> 4;
    const half_t* kh = k + h * HD + sub * 8;
    half8_t kv[8];
#pragma unroll
    for (int f = 0; f < 8; ++f) {
      const int p = slice * 16 + grp + 128 * f;
      kv[f] = p < T ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(kh + (size_t)p * dim))
                    : (half8_t)(0.0f);
    }
    const half8_t qh = *reinterpret_cast<const half8_t*>(q + h * HD + sub * 8);
    const half_t* vh = v + row0 + vsub * 4;
#pragma unroll
    for (int f = 0; f < 16; ++f) {
      const int p = vg + 64 * f;
      vv[f] = p < T ? *reinterpret_cast<const half4_t*>(vh + (size_t)p * dim) : (half4_t)(0.0f);
    }
    const float denom = sqrtf((float)HD);
#pragma unroll
    for (int f = 0; f < 8; ++f) {
      const int p = slice * 16 + grp + 128 * f;
      float s = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s = fmaf((float)qh[e], (float)kv[f][e], s);
      s = row16_sum(s);
      if (sub == 0 && p < T) {
        const half_t val = round_f16(s / denom);  // 425
        const uint64_t word = ((uint64_t)epoch << 32) | __builtin_bit_cast(unsigned short, val);
        __hip_atomic_store(srow + p, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    TL_MARK(1);
    uint64_t raw[NJ];
    int spins = 0;
    while (true) {
      // four words per statement; an element past T reads word 0 of the row instead and is ignored
#pragma unroll
      for (int j = 0; j < NJ; j += 4) {
        uint64_t four[4];
        load_words_device_scope(four, srow + (tid + 256 * j < T ? tid + 256 * j : 0),
                                srow + (tid + 256 * (j + 1) < T ? tid + 256 * (j + 1) : 0),
                                srow + (tid + 256 * (j + 2) < T ? tid + 256 * (j + 2) : 0),
                                srow + (tid + 256 * (j + 3) < T ? tid + 256 * (j + 3) : 0));
#pragma unroll
        for (int e = 0; e < 4; ++e) raw[j + e] = tid + 256 * (j + e) < T ? four[e] : ((uint64_t)epoch << 32) | 0xfc00u;
      }
      bool stale = false;
#pragma unroll
      for (int j = 0; j < NJ; ++j) stale |= (uint32_t)(raw[j] >> 32) != epoch;
      if (__builtin_amdgcn_ballot_w64(stale) == 0) break;
      if (++spins > SPREAD_SPIN_LIMIT) {
        if (lane == 0) atomicAdd(timeouts, 1u);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    TL_MARK(2);
#pragma unroll
    for (int j = 0; j < NJ; ++j) x[j] = (float)__builtin_bit_cast(half_t, (unsigned short)raw[j]);
    m = x[0];
#pragma unroll
    for (int j = 1; j < NJ; ++j) m = fmaxf(m, x[j]);
    m = wave_max_dpp(m);
    if (lane == 0) red[wave] = m;
  }
  __syncthreads();  // (1)
  TL_MARK(3);

  load_wo(B0, B1);

  // ---- attention, second part: softmax_rows (433-499) and the weighted sum (511-531)
  float ssum = 0.0f;
  if (att) {
    const float4_t r = *reinterpret_cast<const float4_t*>(red);
    m = fmaxf(fmaxf(r[0], r[1]), fmaxf(r[2], r[3]));
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      if (tid + 256 * j < T) {
        x[j] = exp_ieee(x[j] - m);
        ssum += x[j];
      }
    }
    ssum += __shfl_xor(ssum, 16, WAVE);
    ssum += dpp_f32<0x128>(ssum);
    {
      const int vi = __builtin_bit_cast(int, ssum);
      int t = __builtin_amdgcn_update_dpp(0, vi, 0x104, 0xF, 0x5, false);
      t = __builtin_amdgcn_update_dpp(t, vi, 0x114, 0xF, 0xA, false);
      ssum += __builtin_bit_cast(float, t);
    }
    ssum += dpp_f32<0x4E>(ssum);
    ssum += dpp_f32<0xB1>(ssum);
  }
  __syncthreads();  // (2) every attention wavefront has read the maxima
  load_wo(B1, B2);
  if (att && (tid & 31) == 0) red[tid >> 5] = ssum;
  __syncthreads();  // (3)
  TL_MARK(4);
  load_wo(B2, LOADS);
  TL_MARK(12);
  if (att) {
    const float4_t lo = *reinterpret_cast<const float4_t*>(red), hi = *reinterpret_cast<const float4_t*>(red + 4);
    const float total = ((lo[0] + hi[0]) + (lo[2] + hi[2])) + ((lo[1] + hi[1]) + (lo[3] + hi[3]));
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      if (tid + 256 * j < T) sc[tid + 256 * j] = round_f16(x[j] / total);  // 497
    }
  }
  __syncthreads();  // (4)
  TL_MARK(5);
  if (att) {
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int f = 0; f < 16; ++f) {
      const int p = vg + 64 * f;
      if (p < T) {
        const float prob = (float)sc[p];
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] = fmaf(prob, (float)vv[f][c], acc[c]);
      }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) gsum[vg][vsub * 4 + c] = acc[c];
  }
  __syncthreads();  // (5)
  if (tid < 16) {
    float o = 0.0f;
#pragma unroll
    for (int g = 0; g < 64; ++g) o += gsum[g][tid];
    publish16(exch + EXCH_ATT, row0, round_f16(o), epoch);  // 529
  }
  TL_MARK(6);

  // ---- x + Wo . att for the 16 rows (llama_cu.cu:1174)
  gather_row(xs, exch + EXCH_ATT, dim, epoch, timeouts);
  __syncthreads();  // (6)
  TL_MARK(7);
  if (team > 0) {
    half8_t xp[NB][2];  // this lane's pieces of the attention output, the same for every row
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int kk = min(((nb * 4 + tw) * 2 + u) * 512 + lane * 8, dim - 8);
        xp[nb][u] = *reinterpret_cast<const half8_t*>(xs + kk);
      }
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int r = team - 1 + 3 * i;
      float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int kk = ((nb * 4 + tw) * 2 + u) * 512 + lane * 8;
          if (kk < dim) {
            const half8_t xv = xp[nb][u];
            const half8_t wv = __builtin_bit_cast(half8_t, wreg[i][nb][u]);
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
              a0 = fmaf((float)wv[e], (float)xv[e], a0);
              a1 = fmaf((float)wv[e + 1], (float)xv[e + 1], a1);
            }
          }
        }
      }
      const float s = wave_sum(a0 + a1);
      if (lane == 0 && r < 16) part[r][tw] = s;
    }
  }
  TL_MARK(13);
  __syncthreads();  // (7) also: every read of the attention output in xs is done
  TL_MARK(8);
  if (tid < 16) {
    float acc = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) acc += part[tid][w];
    const half_t xn = round_f16(fmaf(1.0f, (float)x_old, acc));  // llama_cu.cu:279 with beta = 1
    x_io[row0 + tid] = xn;
    publish16(exch + EXCH_X, row0, xn, epoch);
  }
  TL_MARK(9);

  // ---- rms_norm of the new row (llama_cu.cu:1176, 66-107): every workgroup sums the squares, each
  // normalises its own 16 elements
  gather_row(xs, exch + EXCH_X, dim, epoch, timeouts);
  __syncthreads();  // (8)
  TL_MARK(10);
  float sq = 0.0f;
  if (att) {
    // eight LDS reads in flight at a time; the additions stay in ascending order
    int i = tid;
    for (; i + 7 * 256 < dim; i += 8 * 256) {
      float e[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) e[u] = (float)xs[i + u * 256];
#pragma unroll
      for (int u = 0; u < 8; ++u) sq = fmaf(e[u], e[u], sq);
    }
    for (; i < dim; i += 256) {
      const float e = (float)xs[i];
      sq = fmaf(e, e, sq);
    }
    sq += __shfl_xor(sq, 16, WAVE);
    sq += dpp_f32<0x128>(sq);
    {
      const int vi = __builtin_bit_cast(int, sq);
      int t = __builtin_amdgcn_update_dpp(0, vi, 0x104, 0xF, 0x5, false);
      t = __builtin_amdgcn_update_dpp(t, vi, 0x114, 0xF, 0xA, false);
      sq += __builtin_bit_cast(float, t);
    }
    sq += dpp_f32<0x4E>(sq);
    sq += dpp_f32<0xB1>(sq);
    if ((tid & 31) == 0) red[tid >> 5] = sq;
  }
  __syncthreads();  // (9)
  if (tid < 16) {
    const float4_t lo = *reinterpret_cast<const float4_t*>(red), hi = *reinterpret_cast<const float4_t*>(red + 4);
    const float total = ((lo[0] + hi[0]) + (lo[2] + hi[2])) + ((lo[1] + hi[1]) + (lo[3] + hi[3]));
    const float rms_inv = 1.0f / sqrtf(total / (float)dim + eps);
    const half_t inner = round_f16((float)xs[row0 + tid] * rms_inv);
    norm_out[row0 + tid] = round_f16((float)nw_mine * (float)inner);
  }
  TL_MARK(11);
}

// seq_dev == nullptr: the epoch is a number the host draws per launch (never under stream capture:
// a replay would repeat it); else it comes from *seq_dev, which the caller changes before every
// run, and `salt`.  The score words live in the exchange area behind the stream's workspace.
int launch_decode_attention_spread(half_t* out, const half_t* q, const half_t* k, const half_t* v, const int* pos_dev,
                                   int T_cap, int dim, int n_heads, const workspace_t& ws, const uint32_t* seq_dev,
                                   uint32_t salt, hipStream_t s) {
  static std::atomic<uint32_t> host_epoch{1};
  uint32_t epoch = salt & 1023u;
  if (seq_dev == nullptr) {
    epoch = host_epoch.fetch_add(1) | 0x80000000u;
  }
  const int grid = (n_heads + 7) / 8 * 8 * SPREAD;
  uint64_t* scores = reinterpret_cast<uint64_t*>(ws.sync + SYNC_EXCHANGE);
  static_assert(SYNC_WORDS - SYNC_EXCHANGE >= MAX_HEADS * MAX_T_DECODE * 2, "exchange area");
  uint32_t* timeouts = ws.sync + SYNC_TIMEOUTS;
  if (T_cap <= 1024) {
    decode_attention_spread_kernel<4><<<grid, 256, 0, s>>>(out, q, k, v, T_cap, dim, n_heads, pos_dev, scores, seq_dev,
                                                            epoch, timeouts);
  } else if (T_cap <= 2048) {
    decode_attention_spread_kernel<8><<<grid, 256, 0, s>>>(out, q, k, v, T_cap, dim, n_heads, pos_dev, scores, seq_dev,
                                                            epoch, timeouts);
  } else {
    decode_attention_spread_kernel<16><<<grid, 256, 0, s>>>(out, q, k, v, T_cap, dim, n_heads, pos_dev, scores, seq_dev,
                                                             epoch, timeouts);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

// scores: n_heads x T_cap halves of scratch (only touched when T_cap > SINGLE_LAUNCH_MAX_T)
int launch_decode_attention(half_t* out, const half_t* q, const half_t* k, const half_t* v, const int* pos_dev,
                            int T_cap, int dim, int n_heads, half_t* scores, hipStream_t s) {
  // up to 1024 cached rows the single launch wins (10.3 us against 11.0 us at T = 576: the second
  // launch costs more than the spreading saves), beyond that the two launches do (21 us against
  // 28 us at T = 2048)
  if (T_cap <= SINGLE_LAUNCH_MAX_T) {
    decode_attention_kernel<<<n_heads, DEC_THREADS, 0, s>>>(out, q, k, v, T_cap, dim, pos_dev, nullptr, nullptr);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
  }
  dec_scores_kernel<<<dim3((T_cap + SC_ROWS - 1) / SC_ROWS, n_heads), 256, 0, s>>>(scores, q, k, T_cap, dim, pos_dev);
  LCU_LAUNCH_CHECK();
  dec_softmax_pv_kernel<<<dim3(HD / PV_COLS, n_heads), 256, 0, s>>>(out, scores, v, T_cap, dim, pos_dev);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

// ---------------------------------------------------------------------------------------------
// prefill
// ---------------------------------------------------------------------------------------------
constexpr int CW = 64;         // cache rows per staged chunk
constexpr int QLD = HD + 8;    // LDS row stride (halves) of the Q and K tiles
constexpr int MAX_T_PREFILL = 4096;    // 16-row tiles: a strip of 16 x 4096 fp16 scores fits LDS; 32-row tiles reach 2048
constexpr int MAX_T_PREFILL_32 = 2048;

// BR: query rows per workgroup (16 or 32)
// LDS row of position p of a V chunk (a permutation inside every block of 32 positions)
__device__ __forceinline__ int v_row(int p) {
  const int e = p & 7, g = (p >> 3) & 3;
  return (p & ~31) + 4 * g + (e & 3) + 16 * (e >> 2);
}

template <int BR>
__global__ __launch_bounds__(256) void prefill_attention_kernel(half_t* __restrict__ out, const half_t* __restrict__ q,
                                                                const half_t* __restrict__ k, const half_t* __restrict__ v,
                                                                int n_new, int T, int start_pos, int dim, int n_tiles) {
  constexpr int RT = BR / 16;  // 16-row matrix-instruction tiles per workgroup
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // Heaviest work first over the whole grid (a later row tile has the longer causal span): the
  // heads' last tiles, then their second-to-last ones, and so on, so that compute units pick up
  // the short tiles as they run out of long ones instead of some holding only long ones.
  const int n_heads = gridDim.x / n_tiles;
  const int tile = n_tiles - 1 - blockIdx.x / n_heads;
  const int h = blockIdx.x % n_heads;
  const int r0 = tile * BR;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // columns this tile can see: c <= r + start_pos for its last real row
  const int last_row = min(r0 + BR, n_new) - 1;
  const int c_end = min(T, last_row + start_pos + 1);
  const int Tc = (c_end + CW - 1) / CW * CW;
  const int SLD = Tc + 8;

  half_t* Qs = reinterpret_cast<half_t*>(smem);             // [BR][QLD]
  half_t* KVs = Qs + BR * QLD;                              // K or V chunk [CW][QLD]
  half_t* Ss = KVs + CW * QLD;                              // [BR][SLD]

  // Q tile
  for (int c = tid; c < BR * HD / 8; c += 256) {
    const int row = c >> 4, col = (c & 15) * 8;
    const int gr = r0 + row;
    half8_t val = (half8_t)(0.0f);
    if (gr < n_new) val = *reinterpret_cast<const half8_t*>(q + (size_t)gr * dim + h * HD + col);
    *reinterpret_cast<half8_t*>(&Qs[row * QLD + col]) = val;
  }

  const float denom = sqrtf((float)HD);
  const int frow = lane & 15, fk = (lane >> 4) * 8;
  // A chunk of 64 cache rows is 64 x 128 halves = 4 x 16 bytes per thread.  The next chunk is
  // requested into registers before the current one is multiplied, so its latency hides behind
  // the matrix instructions instead of standing between two barriers.
  constexpr int CH = CW * HD / 8 / 256;  // 16-byte pieces per thread and chunk
  auto load_chunk = [&](half8_t (&reg)[CH], const half_t* __restrict__ src, int c0) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = tid + i * 256;
      const int gp = min(c0 + (c >> 4), T - 1);  // rows past T are never used: their scores are masked, their P is 0
      reg[i] = *reinterpret_cast<const half8_t*>(src + (size_t)gp * dim + h * HD + (c & 15) * 8);
    }
  };
  // V rows are stored in a permuted order (see the gather below); K rows in their own
  bool permute_rows = false;
  auto store_chunk = [&](const half8_t (&reg)[CH]) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = tid + i * 256;
      const int p = c >> 4;
      const int row = permute_rows ? v_row(p) : p;
      *reinterpret_cast<half8_t*>(&KVs[row * QLD + (c & 15) * 8]) = reg[i];
    }
  };

  // Three chunks are in flight in registers: one chunk's matrix work is far shorter than a
  // global load, so a single chunk of look-ahead leaves the load latency exposed.
  constexpr int NPF = 3;
  half8_t stage[NPF][CH];
  auto for_chunks = [&](const half_t* __restrict__ src, auto&& body) {
    for (int c0 = 0; c0 < Tc; c0 += NPF * CW) {
#pragma unroll
      for (int j = 0; j < NPF; ++j) {
        const int cc = c0 + j * CW;
        if (cc < Tc) {
          __syncthreads();  // everybody is done with the previous chunk
          store_chunk(stage[j]);
          __syncthreads();
          if (cc + NPF * CW < Tc) load_chunk(stage[j], src, cc + NPF * CW);
          body(cc);
        }
      }
    }
  };
  auto prefetch_first = [&](const half_t* __restrict__ src) {
#pragma unroll
    for (int j = 0; j < NPF; ++j) {
      if (j * CW < Tc) load_chunk(stage[j], src, j * CW);
    }
  };

  // ---- scores: S[BR][Tc] = Q . K^T, wave w owns the 16 columns w*16.. of every 64-column chunk
  prefetch_first(k);
  for_chunks(k, [&](int c0) {
    float4_t acc[RT];
#pragma unroll
    for (int i = 0; i < RT; ++i) acc[i] = (float4_t)(0.0f);
#pragma unroll
    for (int ks = 0; ks < HD; ks += 32) {
      const half8_t fb = *reinterpret_cast<const half8_t*>(&KVs[(wave * 16 + frow) * QLD + ks + fk]);
#pragma unroll
      for (int i = 0; i < RT; ++i) {
        const half8_t fa = *reinterpret_cast<const half8_t*>(&Qs[(i * 16 + frow) * QLD + ks + fk]);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa, fb, acc[i], 0, 0, 0);
      }
    }
    // accumulator register e of lane l is (row 4*(l/16) + e, column l%16)
    const int col = c0 + wave * 16 + (lane & 15);
#pragma unroll
    for (int i = 0; i < RT; ++i) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int row = i * 16 + (lane >> 4) * 4 + e;
        const bool masked = col > r0 + row + start_pos || col >= T;  // llama_cu.cu:415
        Ss[row * SLD + col] = masked ? (half_t)(-INFINITY) : round_f16(acc[i][e] / denom);
      }
    }
  });
  // the first V chunks travel while the softmax runs
  prefetch_first(v);
  __syncthreads();

  // ---- softmax over each row of the strip (llama_cu.cu:433-499): wave w owns rows w*8 .. w*8+7;
  // exp_ieee and a true division, as in every other softmax here
  for (int rr = 0; rr < BR / 4; ++rr) {
    // two neighbouring scores per lane and access (4 bytes: whole LDS words)
    half2_t* srow = reinterpret_cast<half2_t*>(Ss + (wave * (BR / 4) + rr) * SLD);
    const int pairs = Tc / 2;
    float m = -INFINITY;
    for (int i = lane; i < pairs; i += WAVE) {
      const half2_t v = srow[i];
      m = fmaxf(m, fmaxf((float)v.x, (float)v.y));
    }
    m = wave_max(m);
    float s = 0.0f;
    for (int i = lane; i < pairs; i += WAVE) {
      const half2_t v = srow[i];
      s += exp_ieee((float)v.x - m) + exp_ieee((float)v.y - m);
    }
    s = wave_sum(s);
    for (int i = lane; i < pairs; i += WAVE) {
      const half2_t v = srow[i];
      half2_t p;
      p.x = round_f16(exp_ieee((float)v.x - m) / s);
      p.y = round_f16(exp_ieee((float)v.y - m) / s);
      srow[i] = p;
    }
  }

  // ---- out[BR][HD] = P . V: wave w owns output columns w*32 .. w*32+31 (two 16-wide tiles)
  float4_t o[RT][2];
#pragma unroll
  for (int i = 0; i < RT; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) o[i][j] = (float4_t)(0.0f);
  }
  // V chunks stay row-major in LDS, KVs[pos][d] (16-byte stores without bank conflicts); the
  // matrix instruction wants 8 consecutive positions of one output column per lane, which are
  // gathered with 2-byte reads: the 16 lanes of a fragment row group read 16 neighbouring columns
  // (32 bytes), the four groups rows 8 positions apart.  A row is 272 bytes, so 8 rows apart is
  // 128 bytes modulo the 256 bytes of the banks and groups 0 and 2 (1 and 3) would meet in the same
  // banks; v_row() places position 8g + e of a 32-row block at row 4g + e % 4 + 16 (e / 4), which
  // puts the four groups 64 bytes apart.
  permute_rows = true;
  for_chunks(v, [&](int c0) {
#pragma unroll
    for (int ks = 0; ks < CW; ks += 32) {
      half8_t fa[RT], fb[2];
#pragma unroll
      for (int i = 0; i < RT; ++i) fa[i] = *reinterpret_cast<const half8_t*>(&Ss[(i * 16 + frow) * SLD + c0 + ks + fk]);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const half_t* vcol = &KVs[(ks + fk / 2) * QLD + wave * 32 + j * 16 + frow];  // v_row(ks + fk + e) below
#pragma unroll
        for (int e = 0; e < 8; ++e) fb[j][e] = vcol[((e & 3) + 16 * (e >> 2)) * QLD];
      }
#pragma unroll
      for (int i = 0; i < RT; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) o[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[i], fb[j], o[i][j], 0, 0, 0);
      }
    }
  });
#pragma unroll
  for (int i = 0; i < RT; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = h * HD + wave * 32 + j * 16 + (lane & 15);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int gr = r0 + i * 16 + (lane >> 4) * 4 + e;
        if (gr < n_new) out[(size_t)gr * dim + col] = round_f16(o[i][j][e]);  // llama_cu.cu:529
      }
    }
  }
}

// ---- scores of long decode rows for callers that may not allocate --------------------------------
// lcu_attention_decode_static keeps the fp16 scores of dec_scores_kernel in this array instead of
// a workspace from hipMalloc: MAX_HEADS x MAX_T_DECODE halves = 512 KiB per GPU, held until the
// process ends.  In host code the name `scratch` is only a handle: the array's device address is
// fetched once per device with hipGetSymbolAddress (attention_static_init, called by lcu_init
// with that device current) and kept in scratch_dev; kernels and host code use that pointer.
constexpr int STATIC_MAX_DEVICES = 16;
static __device__ __align__(256) half_t scratch[MAX_HEADS * MAX_T_DECODE];
static half_t* scratch_dev[STATIC_MAX_DEVICES] = {};

size_t prefill_lds_bytes(int BR, int Tc) {
  const size_t kv = (size_t)CW * QLD;
  return ((size_t)BR * QLD + kv + (size_t)BR * (Tc + 8)) * sizeof(half_t);
}

}  // namespace

namespace lcu {

// called by lcu_init with `device` current: the address of this device's copy of `scratch`
int attention_static_init(int device) {
  if (device < 0 || device >= STATIC_MAX_DEVICES) {
    return set_error(LCU_E_SHAPE, "attention_static_init: device %d out of range", device);
  }
  if (scratch_dev[device] == nullptr) {
    void* p = nullptr;
    LCU_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    scratch_dev[device] = (half_t*)p;
  }
  return LCU_OK;
}

}  // namespace lcu

extern "C" {

int lcu_attention(void* out_dev, const void* q_dev, const void* k_dev, const void* v_dev, int n_new, int T,
                  int start_pos, int dim, int n_heads, void* stream) {
  LCU_REQUIRE(out_dev && q_dev && k_dev && v_dev, "lcu_attention: null pointer");
  LCU_REQUIRE(n_new >= 0 && start_pos >= 0 && T == start_pos + n_new,
              "lcu_attention: T (%d) must equal start_pos (%d) + n_new (%d)", T, start_pos, n_new);
  LCU_REQUIRE(n_heads > 0 && n_heads <= MAX_HEADS && dim == n_heads * HD,
              "lcu_attention: dim %d / heads %d unsupported (head_dim must be 128, at most %d heads)", dim, n_heads,
              MAX_HEADS);
  if (n_new == 0) return LCU_OK;
  device_state* st = current_device_state();
  if (!st || !st->ready) return set_error(LCU_E_NOINIT, "lcu_attention: lcu_init has not run on this device");
  hipStream_t s = as_stream(stream);
  if (n_new == 1) {
    LCU_REQUIRE(T <= MAX_T_DECODE, "lcu_attention: T %d exceeds %d", T, MAX_T_DECODE);
    const workspace_t ws = workspace_for(s);
    LCU_REQUIRE((size_t)n_heads * T * sizeof(half_t) <= ws.bytes, "lcu_attention: workspace too small");
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (s != nullptr) LCU_HIP(hipStreamIsCapturing(s, &capturing));
    if (capturing == hipStreamCaptureStatusNone && ws.sync != nullptr && ws.owned) {
      // Only on a stream that owns its workspace: the default stream and foreign streams share the
      // device's, where two overlapping calls would overwrite each other's hand-over words.
      // The epoch of this launch is drawn on the host, so the launch must not be replayed.
      return launch_decode_attention_spread((half_t*)out_dev, (const half_t*)q_dev, (const half_t*)k_dev,
                                            (const half_t*)v_dev, nullptr, T, dim, n_heads, ws, nullptr, 0, s);
    }
    return launch_decode_attention((half_t*)out_dev, (const half_t*)q_dev, (const half_t*)k_dev, (const half_t*)v_dev,
                                   nullptr, T, dim, n_heads, (half_t*)ws.ptr, s);
  }
  LCU_REQUIRE(T <= MAX_T_PREFILL, "lcu_attention: T %d exceeds %d for n_new > 1", T, MAX_T_PREFILL);
  // 16-row tiles when 32-row tiles would leave the grid under four workgroups per compute unit
  // and the rows are short (T <= 1024: 22 us against 29 us at n = T = 512, dim 4096); with long
  // rows the per-chunk overhead of the extra workgroups costs more than the balance gains.
  const long wgs32 = (long)((n_new + 31) / 32) * n_heads;
  const int BR = ((wgs32 < 1024 && T <= 1024) || T > MAX_T_PREFILL_32) ? 16 : 32;
  const int n_tiles = (n_new + BR - 1) / BR;
  const int Tc_max = (T + CW - 1) / CW * CW;
  const size_t lds = prefill_lds_bytes(BR, Tc_max);
  static bool attr_set[16] = {};
  int dev = 0;
  LCU_HIP(hipGetDevice(&dev));
  if (!attr_set[dev & 15]) {
    LCU_HIP(hipFuncSetAttribute((const void*)prefill_attention_kernel<16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)prefill_lds_bytes(16, MAX_T_PREFILL)));
    LCU_HIP(hipFuncSetAttribute((const void*)prefill_attention_kernel<32>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)prefill_lds_bytes(32, MAX_T_PREFILL_32)));
    attr_set[dev & 15] = true;
  }
  if (BR == 16) {
    prefill_attention_kernel<16><<<n_tiles * n_heads, 256, lds, s>>>(
        (half_t*)out_dev, (const half_t*)q_dev, (const half_t*)k_dev, (const half_t*)v_dev, n_new, T, start_pos, dim,
        n_tiles);
  } else {
    prefill_attention_kernel<32><<<n_tiles * n_heads, 256, lds, s>>>(
        (half_t*)out_dev, (const half_t*)q_dev, (const half_t*)k_dev, (const half_t*)v_dev, n_new, T, start_pos, dim,
        n_tiles);
  }
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_attention_decode(void* out_dev, const void* q_dev, const void* k_dev, const void* v_dev, const void* pos_dev,
                         int max_T, int dim, int n_heads, void* stream) {
  LCU_REQUIRE(out_dev && q_dev && k_dev && v_dev && pos_dev, "lcu_attention_decode: null pointer");
  LCU_REQUIRE(n_heads > 0 && n_heads <= MAX_HEADS && dim == n_heads * HD,
              "lcu_attention_decode: dim %d / heads %d unsupported (head_dim must be 128, at most %d heads)", dim,
              n_heads, MAX_HEADS);
  LCU_REQUIRE(max_T > 0 && max_T <= MAX_T_DECODE, "lcu_attention_decode: max_T %d outside 1..%d", max_T, MAX_T_DECODE);
  const workspace_t ws = workspace_for(as_stream(stream));
  if (ws.ptr == nullptr) return set_error(LCU_E_NOINIT, "lcu_attention_decode: lcu_init has not run on this device");
  LCU_REQUIRE((size_t)n_heads * max_T * sizeof(half_t) <= ws.bytes, "lcu_attention_decode: workspace too small");
  return launch_decode_attention((half_t*)out_dev, (const half_t*)q_dev, (const half_t*)k_dev, (const half_t*)v_dev,
                                 (const int*)pos_dev, max_T, dim, n_heads, (half_t*)ws.ptr, as_stream(stream));
}

int lcu_attention_decode_spread(void* out_dev, const void* q_dev, const void* k_dev, const void* v_dev,
                                const void* pos_dev, const void* seq_dev, int salt, int max_T, int dim, int n_heads,
                                void* stream) {
  LCU_REQUIRE(out_dev && q_dev && k_dev && v_dev && pos_dev && seq_dev, "lcu_attention_decode_spread: null pointer");
  LCU_REQUIRE(n_heads > 0 && n_heads <= MAX_HEADS && dim == n_heads * HD,
              "lcu_attention_decode_spread: dim %d / heads %d unsupported (head_dim must be 128, at most %d heads)", dim,
              n_heads, MAX_HEADS);
  LCU_REQUIRE(max_T > 0 && max_T <= MAX_T_DECODE, "lcu_attention_decode_spread: max_T %d outside 1..%d", max_T,
              MAX_T_DECODE);
  LCU_REQUIRE(salt >= 0 && salt < 1024, "lcu_attention_decode_spread: salt %d outside 0..1023", salt);
  const workspace_t ws = workspace_for(as_stream(stream));
  if (ws.ptr == nullptr || ws.sync == nullptr) {
    return set_error(LCU_E_NOINIT, "lcu_attention_decode_spread: lcu_init has not run on this device");
  }
  return launch_decode_attention_spread((half_t*)out_dev, (const half_t*)q_dev, (const half_t*)k_dev,
                                        (const half_t*)v_dev, (const int*)pos_dev, max_T, dim, n_heads, ws,
                                        (const uint32_t*)seq_dev, (uint32_t)salt, as_stream(stream));
}

int lcu_decode_attention_wo_norm(void* x_io_dev, void* norm_out_dev, const void* q_dev, const void* k_dev,
                                 const void* v_dev, const void* wo_dev, const void* norm_w_dev, float eps,
                                 const void* pos_dev, const void* seq_dev, int salt, int max_T, int dim, int n_heads,
                                 void* stream) {
  LCU_REQUIRE(x_io_dev && norm_out_dev && q_dev && k_dev && v_dev && wo_dev && norm_w_dev && pos_dev && seq_dev,
              "lcu_decode_attention_wo_norm: null pointer");
  LCU_REQUIRE(n_heads > 0 && n_heads <= MAX_HEADS && dim == n_heads * HD,
              "lcu_decode_attention_wo_norm: dim %d / heads %d unsupported (head_dim must be 128, at most %d heads)",
              dim, n_heads, MAX_HEADS);
  LCU_REQUIRE(max_T > 0 && max_T <= 1024, "lcu_decode_attention_wo_norm: max_T %d outside 1..1024", max_T);
  LCU_REQUIRE(salt >= 0 && salt < 1024, "lcu_decode_attention_wo_norm: salt %d outside 0..1023", salt);
  const workspace_t ws = workspace_for(as_stream(stream));
  if (ws.sync == nullptr) {
    return set_error(LCU_E_NOINIT, "lcu_decode_attention_wo_norm: lcu_init has not run on this device");
  }
  // the workgroups wait for one another, so all of them must be resident at once: one per compute unit
  device_state* ds = current_device_state();
  LCU_REQUIRE(ds != nullptr && n_heads * SPREAD <= ds->compute_units,
              "lcu_decode_attention_wo_norm: %d heads need %d compute units", n_heads, n_heads * SPREAD);
  static_assert(SYNC_WORDS - SYNC_EXCHANGE >= (EXCH_X + 4096) * 2, "exchange area");
  static_assert(MAX_HEADS * HD / 2 <= 4096, "hand-over areas hold dim / 2 words");
  uint64_t* exch = reinterpret_cast<uint64_t*>(ws.sync + SYNC_EXCHANGE);
  const int grid = (n_heads + 7) / 8 * 8 * SPREAD;
  hipStream_t s = as_stream(stream);
  static bool attr_set[16] = {};
  int dev = 0;
  LCU_HIP(hipGetDevice(&dev));
  if (!attr_set[dev & 15]) {
    LCU_HIP(hipFuncSetAttribute((const void*)decode_attention_wo_norm_kernel<1>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, FUSED_PAD_LDS));
    attr_set[dev & 15] = true;
  }
  LCU_REQUIRE(dim <= 4096, "lcu_decode_attention_wo_norm: dim %d beyond 4096", dim);  // 32 heads of 128
  decode_attention_wo_norm_kernel<1><<<grid, FUSED_THREADS, FUSED_PAD_LDS, s>>>(
      (half_t*)x_io_dev, (half_t*)norm_out_dev, (const half_t*)q_dev, (const half_t*)k_dev, (const half_t*)v_dev,
      (const half_t*)wo_dev, (const half_t*)norm_w_dev, eps, max_T, dim, n_heads, (const int*)pos_dev, exch,
      (const uint32_t*)seq_dev, (uint32_t)salt, ws.sync + SYNC_TIMEOUTS);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_attention_decode_static(void* out_dev, const void* q_dev, const void* k_dev, const void* v_dev, int T, int dim,
                                int n_heads, void* stream) {
  LCU_REQUIRE(out_dev && q_dev && k_dev && v_dev, "lcu_attention_decode_static: null pointer");
  LCU_REQUIRE(n_heads > 0 && n_heads <= MAX_HEADS && dim == n_heads * HD,
              "lcu_attention_decode_static: dim %d / heads %d unsupported (head_dim must be 128, at most %d heads)",
              dim, n_heads, MAX_HEADS);
  LCU_REQUIRE(T > 0 && T <= MAX_T_DECODE,
              "lcu_attention_decode_static: %d cached rows, the static scores array holds rows of 1..%d", T,
              MAX_T_DECODE);
  int dev = 0;
  LCU_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= STATIC_MAX_DEVICES || scratch_dev[dev] == nullptr) {
    return set_error(LCU_E_NOINIT, "lcu_attention_decode_static: lcu_init has not run on device %d", dev);
  }
  // n_heads * T <= MAX_HEADS * MAX_T_DECODE halves by the checks above; every score a launch reads
  // it has written itself, so nothing needs clearing between calls
  return launch_decode_attention((half_t*)out_dev, (const half_t*)q_dev, (const half_t*)k_dev, (const half_t*)v_dev,
                                 nullptr, T, dim, n_heads, scratch_dev[dev], as_stream(stream));
}

int lcu_attention_decode_batch(void* out_dev, const void* q_dev, const void* k_cache_ptrs_dev,
                               const void* v_cache_ptrs_dev, const void* pos_dev, int n_seq, int max_T, int dim,
                               int n_heads, void* stream) {
  LCU_REQUIRE(out_dev && q_dev && k_cache_ptrs_dev && v_cache_ptrs_dev && pos_dev, "lcu_attention_decode_batch: null pointer");
  LCU_REQUIRE(n_heads > 0 && n_heads <= MAX_HEADS && dim == n_heads * HD,
              "lcu_attention_decode_batch: dim %d / heads %d unsupported (head_dim must be 128, at most %d heads)", dim,
              n_heads, MAX_HEADS);
  LCU_REQUIRE(max_T > 0 && max_T <= MAX_T_DECODE && n_seq >= 0 && n_seq <= 65535,
              "lcu_attention_decode_batch: max_T %d outside 1..%d or bad n_seq %d", max_T, MAX_T_DECODE, n_seq);
  if (n_seq == 0) return LCU_OK;
  decode_attention_kernel<<<dim3(n_heads, n_seq), DEC_THREADS, 0, as_stream(stream)>>>(
      (half_t*)out_dev, (const half_t*)q_dev, nullptr, nullptr, max_T, dim, (const int*)pos_dev,
      (const half_t* const*)k_cache_ptrs_dev, (const half_t* const*)v_cache_ptrs_dev);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

#ifdef LCU_PHASE_TIMELINE
// diagnostic builds only: clears (out_host == NULL) or copies out the phase timeline of
// lcu_decode_attention_wo_norm, uint64[64 launches][512 workgroups][16 points] of the 100 MHz counter
int lcu_debug_timeline_read(void* out_host, size_t bytes) {
  void* dev = nullptr;
  LCU_HIP(hipGetSymbolAddress(&dev, HIP_SYMBOL(phase_timeline)));
  LCU_HIP(hipDeviceSynchronize());
  if (out_host == nullptr) {
    LCU_HIP(hipMemset(dev, 0, sizeof(uint64_t) * TL_LAUNCHES * TL_GROUPS * TL_POINTS));
  } else {
    LCU_REQUIRE(bytes <= sizeof(uint64_t) * TL_LAUNCHES * TL_GROUPS * TL_POINTS, "lcu_debug_timeline_read: too many bytes");
    LCU_HIP(hipMemcpy(out_host, dev, bytes, hipMemcpyDeviceToHost));
  }
  return LCU_OK;
}
#endif

}  // extern "C"
