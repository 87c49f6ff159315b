// Prefill matrix products on the gfx950 matrix cores: out[M,N] = lhs[M,K] * W[N,K]^T + beta*out.
//
// These replace matmul_nt_wmma_128x64x64 (llama_cu.cu:150-220) and, for uint8 weights,
// matmul_nt_wmma_16x128x256_fp16u8 at M > 1 (294-366).  Both operands are K-contiguous, which is
// the natural operand order of v_mfma_f32_32x32x16_f16: every lane feeds 8 consecutive k of one
// row of lhs (A) and of one row of W (B).
//
// Two kernels:
//   gemm_dl_kernel (K a multiple of 128, every shape of the model family): both operands travel
//     from global memory straight into a ring of 2-3 LDS stages with global_load_lds_dwordx4 (no
//     staging registers, no LDS store instructions); rows are unpadded and the 16-byte chunks of a
//     row are permuted so that neither the requests nor the fragment reads meet in a bank; tiles
//     of 256x128, 128x128 or 128x64 with 4 or 8 wavefronts (a second group of four may take the
//     other half of a 128-wide K stage), chosen by how many tiles the product has; uint8 weights
//     add a ring of codes and of scales and are turned into fp16 -- exactly fp16((q - 127.5) *
//     scale), llama_cu.cu:287-289 -- once per block tile; with 2..64 rows, and with few large tiles
//     and a long K, the K range is split over workgroups and a second launch adds the fp32 partial
//     sums in split order (launch_skinny, large_tile_splits)
//   gemm_kernel (ragged K): global -> registers -> padded LDS with two LDS buffers and two
//     register stages, uint8 weights dequantised between the load and the LDS store
// Both: the K loop carries no vector address arithmetic and no predication; the block index ->
// tile mapping keeps the tiles that share a slice of W on one XCD (one L2); rows >= M and columns
// >= N are masked instead of the reference's zeroed "gutter" rows (llama_cu.h:236-242).
#include <algorithm>
#include <type_traits>

#include "common.hpp"

using namespace lcu;

namespace lcu {
int gemv_f16(half_t* out, const half_t* x, const half_t* W, int K, int N, float beta, hipStream_t st);
int gemv_u8(half_t* out, const half_t* x, const uint8_t* W, const half_t* S, int K, int N, int block, float beta,
            hipStream_t st);
}  // namespace lcu

namespace {

constexpr int BK = 64;        // K extent one group of four wavefronts multiplies per stage
constexpr int NUM_XCD = 8;

// Up to three products lhs * W_g^T with weight matrices of one shape in a single launch (Wq, Wk,
// Wv; W1, W3): the tile index along N runs through matrix 0, then 1, then 2, `tiles_n_per` tiles
// each.  Matrix 0 travels in the kernel's ordinary arguments, the others here.
struct more_matrices_t {
  half_t* out[2];
  const void* W[2];
  const half_t* S[2];
  int tiles_n_per;  // tiles along N of one matrix; 0: a single matrix
};

__device__ __forceinline__ half2_t dequant2(uint32_t spread, half2_t scale2x) {
  const uint32_t bits = (spread << 2) | 0x58005800u;                                  // 128 + q/2
  const half2_t t = __builtin_bit_cast(half2_t, bits) - (half2_t)((half_t)191.75f);   // (q - 127.5)/2
  return t * scale2x;                                                                 // one rounding
}

// KS: groups of four wavefronts per workgroup.  A stage holds KS * 64 of K; group g multiplies
// columns g*64 .. g*64+63 of it into its own accumulators, and the groups' accumulators are added
// through LDS at the end (group 0 + group 1, a fixed order).  With KS = 2 every SIMD holds two
// wavefronts of the same tile, so one can wait for LDS while the other feeds the matrix core --
// what a second resident workgroup does when the grid has one to give, which at M = 512 it has not.
// KTAIL: K is not a multiple of the stage, so the last stage is partly out of range and is zeroed
// (costs selects in the loop; every model shape takes the KTAIL = false instantiation).
template <int BM, int BN, bool U8, bool KTAIL, int KS>
__global__ __launch_bounds__(256 * KS, KS == 1 ? 2 : 1) void gemm_kernel(
    half_t* __restrict__ out, const half_t* __restrict__ A, const void* __restrict__ Wv, const half_t* __restrict__ S,
    int M, int K, int N, int block, float beta, int tiles_m, int tiles_n) {
  constexpr int THREADS = 256 * KS;
  constexpr int BKS = BK * KS;   // K extent of a stage
  constexpr int LDK = BKS + 8;   // halves per LDS row: 16 bytes of padding keep 16-byte reads of 16 lanes in distinct banks
  constexpr int TM = BM / 64;    // 32x32 MFMA tiles per wavefront along M
  constexpr int TN = BN / 64;
  constexpr int A_ROW = BKS / 8;                  // 16-byte chunks per tile row of lhs
  constexpr int B_ROW = U8 ? BKS / 16 : BKS / 8;  // 16-byte chunks per tile row of W
  constexpr int A_CHUNKS = BM * A_ROW / THREADS;  // chunks per thread
  constexpr int B_CHUNKS = BN * B_ROW / THREADS;
  static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1, "tile too small for the workgroup");

  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_lds[];
  half_t* As = reinterpret_cast<half_t*>(gemm_lds);  // [2][BM * LDK]
  half_t* Bs = As + 2 * BM * LDK;                    // [2][BN * LDK]

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
  const int group = wave >> 2, w4 = wave & 3;
  const int wm = (w4 & 1) * (BM / 2), wn = (w4 >> 1) * (BN / 2);
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
    a_k[i] = (c % A_ROW) * 8;
    a_off[i] = ((uint32_t)min(m0 + c / A_ROW, M - 1) * (uint32_t)K + a_k[i]) * 2u;
  }
#pragma unroll
  for (int i = 0; i < B_CHUNKS; ++i) {
    const int c = tid + i * THREADS;
    const uint32_t row = (uint32_t)min(n0 + c / B_ROW, N - 1);
    if constexpr (U8) {
      b_k[i] = (c % B_ROW) * 16;
      b_off[i] = row * (uint32_t)K + b_k[i];
      s_off[i] = row * (uint32_t)nblk;
    } else {
      b_k[i] = (c % B_ROW) * 8;
      b_off[i] = (row * (uint32_t)K + b_k[i]) * 2u;
    }
  }
  const char* Ab = (const char*)A;
  const char* Wb = (const char*)Wv;

  // one stage of both operands in registers, as loaded from global memory
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
    half_t* Ad = As + buf * BM * LDK;
    half_t* Bd = Bs + buf * BN * LDK;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * THREADS;
      half8_t v = st.ra[i];
      if constexpr (KTAIL) v = (st.k0 + a_k[i] < K) ? v : (half8_t)(0.0f);
      *reinterpret_cast<half8_t*>(&Ad[(c / A_ROW) * LDK + a_k[i]]) = v;
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
        half_t* dst = &Bd[(c / B_ROW) * LDK + b_k[i]];
        *reinterpret_cast<half8_t*>(dst) = lo;
        *reinterpret_cast<half8_t*>(dst + 8) = hi;
      }
    } else {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; ++i) {
        const int c = tid + i * THREADS;
        half8_t v = st.rb[i];
        if constexpr (KTAIL) v = (st.k0 + b_k[i] < K) ? v : (half8_t)(0.0f);
        *reinterpret_cast<half8_t*>(&Bd[(c / B_ROW) * LDK + b_k[i]]) = v;
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

  // Operand fragments are read one 16-wide K slice ahead of the matrix instructions that use
  // them (left to itself the compiler reads a fragment and waits for it in front of every
  // instruction, and the matrix core idles for the LDS latency each time).
  const int frag_row = lane & 31, frag_k = group * BK + (lane >> 5) * 8;
  auto compute = [&](int buf) {
    const half_t* Ad = As + buf * BM * LDK + (wm + frag_row) * LDK + frag_k;
    const half_t* Bd = Bs + buf * BN * LDK + (wn + frag_row) * LDK + frag_k;
    half8_t fa[2][TM], fb[2][TN];
    auto read_frags = [&](int slot, int ks) {
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[slot][i] = *reinterpret_cast<const half8_t*>(Ad + i * 32 * LDK + ks);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[slot][j] = *reinterpret_cast<const half8_t*>(Bd + j * 32 * LDK + ks);
    };
    read_frags(0, 0);
#pragma unroll
    for (int s = 0; s < BK / 16; ++s) {
      if (s + 1 < BK / 16) read_frags((s + 1) & 1, (s + 1) * 16);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[s & 1][i], fb[s & 1][j], acc[i][j], 0, 0, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Pipeline: LDS buffer t%2 holds stage t; one register stage holds stage t+1 (requested one
  // iteration ago) and the other receives stage t+2 while the matrix cores work on stage t.
  // Two iterations per trip so that the two register stages keep fixed names.
  stage_t s0, s1;
  const int nt = (K + BKS - 1) / BKS;
  load_tile(s0, 0);
  if (nt > 1) load_tile(s1, BKS);
  store_tile(s0, 0);
  __syncthreads();
  for (int t = 0; t < nt; t += 2) {
    // stage t in LDS 0, stage t+1 in s1
    if (t + 2 < nt) load_tile(s0, (t + 2) * BKS);
    compute(0);
    if (t + 1 < nt) store_tile(s1, 1);
    __syncthreads();
    if (t + 1 >= nt) break;
    // stage t+1 in LDS 1, stage t+2 in s0
    if (t + 3 < nt) load_tile(s1, (t + 3) * BKS);
    compute(1);
    if (t + 2 < nt) store_tile(s0, 0);
    __syncthreads();
  }

  // the groups' partial sums meet in LDS (every wavefront is past its last LDS read: each compute
  // above is followed by a barrier); element (tile, v) of lane l sits at ((w4, tile, v), l)
  if constexpr (KS == 2) {
    float* part = reinterpret_cast<float*>(gemm_lds);
    if (group == 1) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            part[(((w4 * TM + i) * TN + j) * 16 + v) * 64 + lane] = acc[i][j][v];
          }
        }
      }
    }
    __syncthreads();
    if (group == 1) return;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          acc[i][j][v] += part[(((w4 * TM + i) * TN + j) * 16 + v) * 64 + lane];
        }
      }
    }
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

// ---- fp16 weights, K a multiple of the stage: operands go from global memory straight into LDS
// (global_load_lds_dwordx4: no staging registers, no LDS store instructions, and the wavefront
// does not wait for a load before it can go on), through a ring of NS stages.
//
// A load instruction of one wavefront fills 1 KB of LDS, lane l at byte 16*l, so tile rows lie
// densely (ROWB bytes each, no padding) and bank conflicts are avoided by permuting the 16-byte
// chunks inside a row instead: the chunk that holds K offsets 8g..8g+7 of tile row r is stored at
// chunk position g ^ f(r), f(r) = (r / RPB) % CR.  Sixteen lanes reading the same g from sixteen
// consecutive rows then cover all 64 banks exactly once.
//
// Per iteration: wait until this wavefront's loads of stage t have landed, barrier (so everybody's
// have), request stage t+NS-1 into the slot whose reads ended before that barrier, multiply
// stage t.  The compiler does not track these loads against LDS reads; the waits are explicit.
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// WM x WN wavefronts tile the block (each a (BM/WM) x (BN/WN) sub-tile of 32x32 matrix-instruction
// tiles), times KS groups along K.
//
// Tried and dropped: an extra wavefront that touches the lines of a stage several stages ahead so
// that the loaders hit L2.  About a sixth of the requests come from HBM, but the touches (64
// separate lines per instruction) cost the texture addresser more than the misses cost the ring.
//
// uint8 weights (U8): the codes travel the same way, into a ring of their own, one stage further
// ahead than the lhs tile ("batch" b of requests = lhs of stage b + codes of stage b+1).  During
// stage t the workgroup turns the codes of stage t+1 into the fp16 tile the matrix instructions
// read -- every thread one 16-code chunk, each weight exactly fp16((q - 127.5) * scale), written
// at the same permuted chunk positions a direct fp16 load would have filled -- so a weight is
// dequantised once per block tile and the fragment path is the fp16 one.  The chunk's scale comes
// by an ordinary 2-byte load one stage earlier.
//
// SPLIT (few rows, so few tiles): the grid holds `splits` workgroups per tile, each taking a
// contiguous run of the K stages and writing its fp32 sums to part[split][M][N];
// splitk_reduce_kernel adds them in split order and applies the epilogue.
template <int BM, int BN, int WM, int WN, int KS, int NS, bool U8, bool SPLIT = false>
__global__ __launch_bounds__(64 * WM * WN * KS, WM * WN * KS <= 4 ? 2 : 1) void gemm_dl_kernel(
    half_t* __restrict__ out0, const half_t* __restrict__ A, const void* __restrict__ W0, const half_t* __restrict__ S0,
    int M, int K, int N, int block, float beta, int tiles_m, int tiles_n, float* __restrict__ part, int splits,
    more_matrices_t more) {
  constexpr int NG = WM * WN;                // wavefronts of one group
  constexpr int NW = NG * KS;                // wavefronts
  constexpr int BKS = BK * KS;               // K extent of a stage
  constexpr int ROWB = BKS * 2;              // bytes of a tile row in LDS
  constexpr int CR = ROWB / 16;              // 16-byte chunks per row: 8 or 16
  constexpr int RPB = 16 / CR;               // tile rows per 256 bytes (one pass over the banks)
  constexpr int THREADS = 64 * NW;
  constexpr int CPR = BKS / 16;              // 16-code chunks per row of the code tile
  constexpr int PA = BM * CR / 64 / NW;      // load instructions per wavefront per stage, lhs
  constexpr int PB = U8 ? BN * CPR / 64 / NW : BN * CR / 64 / NW;  // and W (fp16 values or codes)
  constexpr int DC = U8 ? BN * CPR / THREADS : 1;                  // code chunks a thread dequantises per stage
  constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, C_BYTES = BN * BKS;
  constexpr int NB = U8 ? 2 : NS;            // fp16 W tiles held: written one stage ahead, or the ring itself
  // fp16: slot s of the ring holds lhs and W tile of a stage side by side; uint8: lhs ring, then the
  // two fp16 W tiles, then the code ring
  constexpr int A_STRIDE = U8 ? A_BYTES : A_BYTES + B_BYTES, B_STRIDE = U8 ? B_BYTES : A_BYTES + B_BYTES;
  constexpr int B_BASE = U8 ? NS * A_BYTES : A_BYTES, C_BASE = NS * A_BYTES + NB * B_BYTES;
  constexpr int S_BYTES = THREADS * 4 * DC;  // scale ring slot: one dword per thread and chunk
  constexpr int S_BASE = C_BASE + NS * C_BYTES;
  constexpr int LDS_BYTES = NS * A_BYTES + NB * B_BYTES + (U8 ? NS * (C_BYTES + S_BYTES) : 0);
  constexpr int TM = BM / (32 * WM), TN = BN / (32 * WN);
  static_assert(PA >= 1 && PB >= 1 && DC >= 1 && NS >= 2 && NS <= 4, "unsupported configuration");
  static_assert(!U8 || NS == 3, "the uint8 schedule is written for a ring of three");
  constexpr int P = PA + PB + (U8 ? DC : 0);  // requests per wavefront and batch
  static_assert(P * (NS - 1) < 64, "vmcnt has 6 bits");

  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_lds[];

  const int nb = tiles_m * tiles_n;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int group = wave / NG, w4 = wave % NG;
  const int wm = (w4 % WM) * (BM / WM), wn = (w4 / WM) * (BN / WN);
  // XCD-aware tile order, as in gemm_kernel
  const int split = SPLIT ? blockIdx.x / nb : 0;
  const int bx = SPLIT ? blockIdx.x - split * nb : blockIdx.x;
  const int q = nb / NUM_XCD, r = nb % NUM_XCD;
  const int xcd = bx % NUM_XCD, idx = bx / NUM_XCD;
  const int logical = xcd * q + min(xcd, r) + idx;
  const int tm = logical % tiles_m;
  int tn = logical / tiles_m;
  // which weight matrix this tile belongs to: chosen once, from kernel arguments (scalar selects)
  half_t* out = out0;
  const void* W = W0;
  const half_t* S = S0;
  if (more.tiles_n_per > 0) {
    const int g = tn / more.tiles_n_per;
    tn -= g * more.tiles_n_per;
    out = g == 0 ? out0 : (g == 1 ? more.out[0] : more.out[1]);
    W = g == 0 ? W0 : (g == 1 ? more.W[0] : more.W[1]);
    S = g == 0 ? S0 : (g == 1 ? more.S[0] : more.S[1]);
    if constexpr (SPLIT) {
      part += (size_t)g * splits * M * N;  // each matrix has its own partial sums
    }
  }
  const int m0 = tm * BM, n0 = tn * BN;

  // beta != 0: the old values of the output tile, asked for now in 16-byte pieces (tile row c / (BN / 8), eight
  // columns from 8 (c % (BN / 8))) and handed to the lanes that need them through LDS after the last stage.
  // Read lane by lane in the accumulators' layout (2-byte requests, two rows of 64 bytes per instruction) they cost
  // the 512 x 4096 x 4096 product 6 us.  Rows of N % 8 != 0 are not 16-byte aligned: those keep the 2-byte reads.
  // Only where a thread holds at most two pieces (the 128 x 64 tile of 512 threads, which carries Wo): the
  // registers that more pieces occupy through the K loop cost the 256 x 128 tile 5 % with beta = 0.
  constexpr int OC = BM * BN / 8 / THREADS;  // pieces per thread
  constexpr int OLD_LD = BN + 8;             // halves per tile row in LDS
  constexpr bool OLD_PIECES = !SPLIT && OC <= 2;
  static_assert(BM * BN / 8 % THREADS == 0 && BM * OLD_LD * 2 <= LDS_BYTES, "old tile staging");
  // 16-byte requests: rows of a multiple of 8 halves from a 16-byte aligned base (anything else keeps
  // the 2-byte reads of the epilogue)
  const bool old_by_pieces = OLD_PIECES && beta != 0.0f && N % 8 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  uint4_t old_piece[OC];
  if constexpr (OLD_PIECES) {
    if (old_by_pieces) {
#pragma unroll
      for (int j = 0; j < OC; ++j) {
        const int c = tid + j * THREADS;
        const int gm = m0 + c / (BN / 8), gn = n0 + (c % (BN / 8)) * 8;
        old_piece[j] = (uint4_t)(0u);
        if (gm < M && gn < N) old_piece[j] = *reinterpret_cast<const uint4_t*>(out + (size_t)gm * N + gn);
      }
    }
  }

  // loader: instruction j of this wavefront fills LDS bytes [(wave + j*NW) * 1024, +1024) of the
  // operand's region; lane l lands on tile row c / CR, chunk position c % CR, c = that index * 64 + l
  uint32_t a_off[PA], b_off[PB];
#pragma unroll
  for (int j = 0; j < PA; ++j) {
    const int c = (wave + j * NW) * 64 + lane;
    const int row = c / CR, g = (c % CR) ^ ((row / RPB) % CR);
    a_off[j] = ((uint32_t)min(m0 + row, M - 1) * (uint32_t)K + g * 8) * 2u;
  }
#pragma unroll
  for (int j = 0; j < PB; ++j) {
    const int c = (wave + j * NW) * 64 + lane;
    if constexpr (U8) {  // codes lie densely and unpermuted: chunk c of the tile at byte 16 c
      b_off[j] = (uint32_t)min(n0 + c / CPR, N - 1) * (uint32_t)K + (c % CPR) * 16;
    } else {
      const int row = c / CR, g = (c % CR) ^ ((row / RPB) % CR);
      b_off[j] = ((uint32_t)min(n0 + row, N - 1) * (uint32_t)K + g * 8) * 2u;
    }
  }
  // this workgroup's K stages: all of them, or its share [stage0, stage0 + nt) of a split
  const int nt_all = K / BKS;
  const int stage0 = SPLIT ? (int)((long)split * nt_all / splits) : 0;
  const int nt = SPLIT ? (int)((long)(split + 1) * nt_all / splits) - stage0 : nt_all;
  const int k_base = stage0 * BKS;
  const char* Ab = (const char*)A + (size_t)k_base * 2;
  const char* Wb = (const char*)W + (size_t)k_base * (U8 ? 1 : 2);
  // uint8: the chunks this thread dequantises (tile row, chunk in the row), their scale index at
  // stage 0, and where the two fp16 chunks of a dequantised chunk go in the W tile
  int d_scale[DC];
  uint32_t d_src[DC], d_dst0[DC], d_dst1[DC];
  const bool hi_first = (tid >> 2) & 1;
  const int nblk = U8 ? K / block : 0;
  if constexpr (U8) {
#pragma unroll
    for (int i = 0; i < DC; ++i) {
      const int c = tid + i * THREADS;
      const int row = c / CPR, kc = c % CPR, f = (row / RPB) % CR;
      d_scale[i] = min(n0 + row, N - 1) * nblk;
      d_src[i] = (uint32_t)c * 16;
      d_dst0[i] = (uint32_t)row * ROWB + (uint32_t)(((2 * kc) ^ f) * 16);
      d_dst1[i] = (uint32_t)row * ROWB + (uint32_t)(((2 * kc + 1) ^ f) * 16);
      // LDS stores see 32 banks (128 bytes): eight consecutive lanes must land on eight different
      // chunk positions modulo 8.  Four lanes share a row (or half a row) and would all write even
      // positions with their first store; so every second group of four lanes writes its odd chunk
      // first (8 conflict cycles per store instruction otherwise).
      if (hi_first) {
        const uint32_t t0 = d_dst0[i];
        d_dst0[i] = d_dst1[i];
        d_dst1[i] = t0;
      }
    }
  }
  // A request is written as inline assembly (M0 = LDS address of the wavefront's 1 KB, then the
  // load), so that the compiler does not know about it: knowing, it treats the request like a FLAT
  // access and waits for every LDS read in front of each matrix instruction.  Nothing else in this
  // kernel uses M0.  The data lands in LDS, not in a register, so there is nothing here the
  // compiler could copy too early; the waits for it (vmcnt) are the explicit ones below.
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)gemm_lds;
  auto request16 = [&](const void* g, uint32_t lds_off) {
    const uint32_t m0 = __builtin_amdgcn_readfirstlane(lds0 + lds_off);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(m0) : "memory", "m0");
  };
  auto request4 = [&](const void* g, uint32_t lds_off) {
    const uint32_t m0 = __builtin_amdgcn_readfirstlane(lds0 + lds_off);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(g), "s"(m0) : "memory", "m0");
  };
  // request `idx` (0 .. P-1) of this wavefront for batch `stage` into ring slot `slot`: the lhs tile
  // of that stage, and the W tile of that stage (fp16) or the codes and scales of the stage after it
  // (uint8; past the end the last stage is fetched again and never used)
  auto issue_one = [&](int stage, int slot, int idx) {
    if (idx < PA) {
      request16(Ab + (size_t)stage * (BKS * 2) + a_off[idx], slot * A_STRIDE + (wave + idx * NW) * 1024);
    } else if constexpr (U8) {
      const int cslot = slot + 1 == NS ? 0 : slot + 1;
      const int st1 = min(stage + 1, nt - 1);
      if (idx < PA + PB) {
        request16(Wb + (size_t)st1 * BKS + b_off[idx - PA], C_BASE + cslot * C_BYTES + (wave + (idx - PA) * NW) * 1024);
      } else {
        const int i = idx - PA - PB;  // the dword that holds this thread's fp16 scale of chunk i
        const int kc = (tid + i * THREADS) % CPR;
        const int at = d_scale[i] + (k_base + st1 * BKS + kc * 16) / block;
        request4(S + (at & ~1), S_BASE + cslot * S_BYTES + (i * NW + wave) * 256);
      }
    } else {
      request16(Wb + (size_t)stage * (BKS * 2) + b_off[idx - PA], B_BASE + slot * B_STRIDE + (wave + (idx - PA) * NW) * 1024);
    }
  };
  auto issue = [&](int stage, int slot) {
#pragma unroll
    for (int idx = 0; idx < P; ++idx) issue_one(stage, slot, idx);
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      acc[i][j] = (float16_t)(0.0f);
    }
  }

  // reader: chunk position of K slice s (16 wide) for this lane; the row term of f() is the same
  // for every 32-row tile of the wavefront because 32 / RPB is a multiple of CR
  const int frag_row = lane & 31;
  const int fr = (frag_row / RPB) % CR;
  const int gbase = group * 8 + (lane >> 5);
  uint32_t pos[BK / 16];
#pragma unroll
  for (int s4 = 0; s4 < BK / 16; ++s4) pos[s4] = (uint32_t)(((gbase + 2 * s4) ^ fr) * 16);
  const uint32_t a_row = (uint32_t)(wm + frag_row) * ROWB, b_row = (uint32_t)B_BASE + (uint32_t)(wn + frag_row) * ROWB;

  // codes and scales in ring slot `cslot` (they belong to K stage `stage`) -> fp16 W tile `bslot`
  auto dequantise = [&](int cslot, int bslot, int stage) {
#pragma unroll
    for (int i = 0; i < DC; ++i) {
      const uint4_t q = *reinterpret_cast<const uint4_t*>(gemm_lds + C_BASE + cslot * C_BYTES + d_src[i]);
      const uint32_t pair = *reinterpret_cast<const uint32_t*>(gemm_lds + S_BASE + cslot * S_BYTES + i * THREADS * 4 + tid * 4);
      const int kc = (tid + i * THREADS) % CPR;
      const int at = d_scale[i] + (k_base + stage * BKS + kc * 16) / block;  // the request fetched the dword at (at & ~1)
      const half_t sc = __builtin_bit_cast(half_t, (uint16_t)((at & 1) ? pair >> 16 : pair & 0xffffu));
      const half_t s2 = sc * (half_t)2.0f;
      const half2_t s2v = {s2, s2};
      half2_t d[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        d[2 * j] = dequant2(__builtin_amdgcn_perm(0u, q[j], 0x0c010c00u), s2v);
        d[2 * j + 1] = dequant2(__builtin_amdgcn_perm(0u, q[j], 0x0c030c02u), s2v);
      }
      const half8_t lo = {d[0].x, d[0].y, d[1].x, d[1].y, d[2].x, d[2].y, d[3].x, d[3].y};
      const half8_t hi = {d[4].x, d[4].y, d[5].x, d[5].y, d[6].x, d[6].y, d[7].x, d[7].y};
      unsigned char* tile = gemm_lds + B_BASE + bslot * B_STRIDE;
      *reinterpret_cast<half8_t*>(tile + d_dst0[i]) = hi_first ? hi : lo;
      *reinterpret_cast<half8_t*>(tile + d_dst1[i]) = hi_first ? lo : hi;
    }
  };

  // ---- the stage loop --------------------------------------------------------------------------
  // K slice s of a stage uses fragment buffer s & 1.  Per stage and wavefront:
  //   slices 0..2: read slice s+1 | request a third of the batch NS-1 ahead | multiply slice s
  //   slice 3:     wait for this wavefront's LDS accesses (it is then done with the stage) | wait
  //                for its own requests of the next stage | barrier | read slice 0 of the next
  //                stage | multiply slice 3
  // so fragments are always requested one slice before the matrix instructions that use them, also
  // across the stage boundary.  The fragment reads are ordinary loads: the compiler counts them
  // (lgkmcnt) and waits for exactly the fragments an instruction needs.
  constexpr int S4 = BK / 16;
  static_assert(S4 == 4, "the schedule below is written for four K slices per stage");
  half8_t fa[2][TM], fb[2][TN];
  auto read_frags = [&](int buf, int slot, int bslot, int s4) {
    const unsigned char* pa = gemm_lds + slot * A_STRIDE + a_row + pos[s4];
    const unsigned char* pb = gemm_lds + bslot * B_STRIDE + b_row + pos[s4];
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[buf][i] = *reinterpret_cast<const half8_t*>(pa + i * 32 * ROWB);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[buf][j] = *reinterpret_cast<const half8_t*>(pb + j * 32 * ROWB);
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[buf][i], fb[buf][j], acc[i][j], 0, 0, 0);
      }
    }
  };
  // one stage (lhs in ring slot `slot`, W tile `bslot`); FETCH: request batch `next` into slot
  // `fill`; MORE: another stage follows (slots `nslot`, `nbslot`), whose own requests are complete
  // once at most PEND younger ones are outstanding.  uint8 with MORE: between the first two slices
  // the codes of the next stage (ring slot nslot) become its fp16 tile nbslot.
  auto stage = [&](int slot, int bslot, auto fetch, int next, int fill, auto more, auto pend, int nslot, int nbslot,
                   int t) {
    constexpr bool FETCH = decltype(fetch)::value, MORE = decltype(more)::value;
    constexpr int PEND = decltype(pend)::value;
#pragma unroll
    for (int s4 = 0; s4 < 3; ++s4) {
      read_frags((s4 + 1) & 1, slot, bslot, s4 + 1);
      if constexpr (FETCH) {
#pragma unroll
        for (int idx = s4 * P / 3; idx < (s4 + 1) * P / 3; ++idx) issue_one(next, fill, idx);
      }
      __builtin_amdgcn_sched_barrier(0);
      multiply(s4 & 1);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (U8 && MORE) {
        if (s4 == 0) {
          dequantise(nslot, nbslot, t + 1);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if constexpr (MORE) {
      // this wavefront's reads of the stage (and its writes of the next fp16 tile) are complete
      // before it lets the others overwrite the slot / read the tile
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      wait_vmcnt<PEND>();
      asm volatile("s_barrier" ::: "memory");
      read_frags(0, nslot, nbslot, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    multiply(1);
    __builtin_amdgcn_sched_barrier(0);
  };

  if constexpr (U8) {
    // codes and scales of stage 0 (batch -1, into slot 0 of their rings), then the first batches
#pragma unroll
    for (int idx = PA; idx < P; ++idx) issue_one(-1, NS - 1, idx);
#pragma unroll
    for (int s0 = 0; s0 < NS - 1; ++s0) {
      if (s0 < nt) issue(s0, s0);
    }
    if (nt > 1) {
      wait_vmcnt<(NS - 1) * P>();  // everything older than the batches: codes and scales of stage 0
    } else {
      wait_vmcnt<0>();
    }
    asm volatile("s_barrier" ::: "memory");
    dequantise(0, 0, 0);
  } else {
#pragma unroll
    for (int s0 = 0; s0 < NS - 1; ++s0) {
      if (s0 < nt) issue(s0, s0);
    }
  }
  // stage 0 has to be there before anything is read
  if (nt > 1) {
    wait_vmcnt<(NS - 2) * P>();  // with nt < NS - 1 fewer requests exist: the wait is merely stricter
  } else {
    wait_vmcnt<0>();
  }
  __syncthreads();  // also orders the fp16 tile written just above (uint8) before its first reads
  read_frags(0, 0, 0, 0);
  int slot = 0, fill = NS - 1;  // ring slots of stage t and of batch t + NS - 1
  auto next_of = [](int v) { return v + 1 == NS ? 0 : v + 1; };
  const int n_main = max(nt - (NS - 1), 0);
  for (int t = 0; t < n_main; ++t) {
    // after this stage's requests (batch t+NS-1), batches t+2 .. t+NS-1 may stay in flight when
    // batch t+1 must have landed
    stage(slot, U8 ? (t & 1) : slot, std::true_type{}, t + NS - 1, fill, std::true_type{},
          std::integral_constant<int, (NS - 2) * P>{}, next_of(slot), U8 ? ((t + 1) & 1) : next_of(slot), t);
    slot = next_of(slot);
    fill = next_of(fill);
  }
  // the last NS-1 stages: nothing left to request, so simply wait for everything
  for (int t = n_main; t < nt; ++t) {
    if (t + 1 < nt) {
      stage(slot, U8 ? (t & 1) : slot, std::false_type{}, 0, 0, std::true_type{}, std::integral_constant<int, 0>{},
            next_of(slot), U8 ? ((t + 1) & 1) : next_of(slot), t);
    } else {
      stage(slot, U8 ? (t & 1) : slot, std::false_type{}, 0, 0, std::false_type{}, std::integral_constant<int, 0>{}, 0, 0,
            t);
    }
    slot = next_of(slot);
  }
  __syncthreads();  // the last stage has been read by everybody: LDS is free for the partial sums

  if constexpr (KS == 2) {
    float* part = reinterpret_cast<float*>(gemm_lds);
    if (group == 1) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            part[(((w4 * TM + i) * TN + j) * 16 + v) * 64 + lane] = acc[i][j][v];
          }
        }
      }
    }
    __syncthreads();
    if (group == 0) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            acc[i][j][v] += part[(((w4 * TM + i) * TN + j) * 16 + v) * 64 + lane];
          }
        }
      }
    }
  }

  half_t* old_lds = reinterpret_cast<half_t*>(gemm_lds);
  if constexpr (OLD_PIECES) {
    if (old_by_pieces) {
      if constexpr (KS == 2) __syncthreads();  // the partial sums above have been read
#pragma unroll
      for (int j = 0; j < OC; ++j) {
        const int c = tid + j * THREADS;
        *reinterpret_cast<uint4_t*>(old_lds + (c / (BN / 8)) * OLD_LD + (c % (BN / 8)) * 8) = old_piece[j];
      }
      __syncthreads();
    }
  }
  // epilogue as in gemm_kernel (llama_cu.cu:208-215)
  if (group == 0) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int gn = n0 + wn + j * 32 + (lane & 31);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int lm = wm + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
          const int gm = m0 + lm;
          if (gm < M && gn < N) {
            if constexpr (SPLIT) {
              part[((size_t)split * M + gm) * N + gn] = acc[i][j][v];
            } else {
              half_t* p = out + (size_t)gm * N + gn;
              float val = acc[i][j][v];
              if (beta != 0.0f) {
                const half_t before = old_by_pieces ? old_lds[lm * OLD_LD + wn + j * 32 + (lane & 31)] : *p;
                val = fmaf(beta, (float)before, val);
              }
              *p = round_f16(val);
            }
          }
        }
      }
    }
  }
}

// out_g[m][n] = fp16(sum over splits, in split order, of part[g][s][m][n] + beta * out_g[m][n]); blockIdx.y = g
__global__ __launch_bounds__(256) void splitk_reduce_kernel(half_t* out0, half_t* out1, half_t* out2,
                                                            const float* __restrict__ part, size_t mn, int splits,
                                                            float beta) {
  const int g = blockIdx.y;
  half_t* out = g == 0 ? out0 : (g == 1 ? out1 : out2);
  part += (size_t)g * splits * mn;
  const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= mn) {
    return;
  }
  if (i + 4 <= mn && mn % 4 == 0) {
    float4 sum = *reinterpret_cast<const float4*>(part + i);
    for (int s = 1; s < splits; ++s) {
      const float4 v = *reinterpret_cast<const float4*>(part + (size_t)s * mn + i);
      sum.x += v.x;
      sum.y += v.y;
      sum.z += v.z;
      sum.w += v.w;
    }
    const float v4[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float val = v4[e];
      if (beta != 0.0f) {
        val = fmaf(beta, (float)out[i + e], val);
      }
      out[i + e] = round_f16(val);
    }
    return;
  }
  for (size_t j = i; j < min(i + 4, mn); ++j) {
    float val = part[j];
    for (int s = 1; s < splits; ++s) {
      val += part[(size_t)s * mn + j];
    }
    if (beta != 0.0f) {
      val = fmaf(beta, (float)out[j], val);
    }
    out[j] = round_f16(val);
  }
}

// the arguments of one launch: matrix 0 and, for fused launches, up to two more of the same shape
struct operands_t {
  half_t* out;
  const void* W;
  const half_t* S;
  more_matrices_t more;
  int n_mats;
};

inline operands_t single_matrix(half_t* out, const void* W, const half_t* S) {
  return operands_t{out, W, S, more_matrices_t{{nullptr, nullptr}, {nullptr, nullptr}, {nullptr, nullptr}, 0}, 1};
}

template <int BM, int BN, int WM, int WN, int KS, int NS, bool U8>
int launch_dl(operands_t op, const half_t* A, int M, int K, int N, int block, float beta, hipStream_t st) {
  constexpr int ROWB = BK * KS * 2;
  constexpr int DCH = U8 ? BN * (BK * KS / 16) / (64 * WM * WN * KS) : 0;  // scale dwords per thread and stage
  constexpr size_t lds = (size_t)NS * BM * ROWB + (size_t)(U8 ? 2 : NS) * BN * ROWB +
                         (U8 ? (size_t)NS * (BN * BK * KS + 64 * WM * WN * KS * 4 * DCH) : 0);
  static_assert(lds <= 160 * 1024, "rings do not fit LDS");
  static_assert(KS == 1 || lds >= (size_t)BM * BN * 4 / 2, "LDS must hold one group's accumulators");
  const int tiles_m = (M + BM - 1) / BM, tiles_n_per = (N + BN - 1) / BN, tiles_n = tiles_n_per * op.n_mats;
  op.more.tiles_n_per = op.n_mats > 1 ? tiles_n_per : 0;
  auto kernel = gemm_dl_kernel<BM, BN, WM, WN, KS, NS, U8>;
  if constexpr (lds > 64 * 1024) {
    static bool raised[16] = {};  // per device, once
    int dev = 0;
    LCU_HIP(hipGetDevice(&dev));
    if (!raised[dev & 15]) {
      LCU_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      raised[dev & 15] = true;
    }
  }
  kernel<<<tiles_m * tiles_n, 64 * WM * WN * KS, lds, st>>>(op.out, A, op.W, op.S, M, K, N, block, beta, tiles_m,
                                                            tiles_n, nullptr, 1, op.more);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

// where a split-K launch left its partial sums: part[matrix][split][M][N] fp32
struct partial_sums_t {
  const float* part;
  int splits;
};

// BM x BN tiles of WM x WN wavefronts, the K stages of every tile dealt to `splits` workgroups
// (gemm_dl_kernel<.., SPLIT = true>), fp32 partial sums in the stream's workspace, then
// splitk_reduce_kernel -- or the caller's own kernel when `leave` is given.
template <int BM, int BN, int WM, int WN, bool U8>
int launch_split(operands_t op, const half_t* A, int M, int K, int N, int block, float beta, hipStream_t st, int splits,
                 float* part, partial_sums_t* leave = nullptr) {
  constexpr int KS = 1, NS = 3;
  constexpr int ROWB = BK * KS * 2;
  constexpr int DCH = U8 ? BN * (BK * KS / 16) / (64 * WM * WN * KS) : 0;
  constexpr size_t lds = (size_t)NS * BM * ROWB + (size_t)(U8 ? 2 : NS) * BN * ROWB +
                         (U8 ? (size_t)NS * (BN * BK * KS + 64 * WM * WN * KS * 4 * DCH) : 0);
  static_assert(lds <= 160 * 1024, "LDS");
  const int tiles_m = (M + BM - 1) / BM, tiles_n_per = (N + BN - 1) / BN, tiles_n = tiles_n_per * op.n_mats;
  op.more.tiles_n_per = op.n_mats > 1 ? tiles_n_per : 0;
  const size_t mn = (size_t)M * N;
  auto kernel = gemm_dl_kernel<BM, BN, WM, WN, KS, NS, U8, true>;
  if constexpr (lds > 64 * 1024) {
    static bool raised[16] = {};  // per device, once
    int dev = 0;
    LCU_HIP(hipGetDevice(&dev));
    if (!raised[dev & 15]) {
      LCU_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      raised[dev & 15] = true;
    }
  }
  kernel<<<tiles_m * tiles_n * splits, 64 * WM * WN * KS, lds, st>>>(op.out, A, op.W, op.S, M, K, N, block, beta, tiles_m,
                                                                     tiles_n, part, splits, op.more);
  LCU_LAUNCH_CHECK();
  if (leave) {  // the caller's own kernel adds the partial sums up (fused with what follows the product)
    leave->part = part;
    leave->splits = splits;
  } else {
    splitk_reduce_kernel<<<dim3((unsigned)((mn + 1023) / 1024), op.n_mats), 256, 0, st>>>(
        op.out, op.more.out[0], op.more.out[1], part, mn, splits, beta);
    LCU_LAUNCH_CHECK();
  }
  return LCU_OK;
}

// Few rows (2 .. 64: short prompts, where the reference takes its 16-row tile, llama_cu.cu:1481-1484):
// BM x 128 tiles with four wavefronts, the K stages split over enough workgroups to give every
// compute unit one.  Returns LCU_OK with *done = false when the shape does not suit it.
template <int BM, bool U8>
int launch_skinny(operands_t op, const half_t* A, int M, int K, int N, int block, float beta, hipStream_t st,
                  bool* done, partial_sums_t* leave = nullptr) {
  // a ring of six stages and 128-wide stages with eight wavefronts measured no faster
  constexpr int BN = 128;
  *done = false;
  device_state* ds = current_device_state();
  const workspace_t ws = workspace_for(st);
  if (ds == nullptr || ws.ptr == nullptr) {
    return LCU_OK;
  }
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN * op.n_mats;
  const int nt_all = K / BK;
  // one workgroup per compute unit and at least four stages each: more, shorter splits only add
  // partial sums (512 workgroups: 16 against 13 us at N = K = 4096)
  int splits = (ds->compute_units + tiles_m * tiles_n - 1) / (tiles_m * tiles_n);
  splits = max(1, min(splits, nt_all / 4));
  const size_t mn = (size_t)M * N;
  while (splits > 1 && (size_t)splits * mn * op.n_mats * sizeof(float) > ws.bytes) {
    --splits;
  }
  if ((size_t)splits * mn * op.n_mats * sizeof(float) > ws.bytes ||
      (long)tiles_m * tiles_n * splits < ds->compute_units / 2) {
    return LCU_OK;
  }
  const int rc = launch_split<BM, BN, 1, 4, U8>(op, A, M, K, N, block, beta, st, splits, (float*)ws.ptr, leave);
  *done = rc == LCU_OK;
  return rc;
}

// Many rows, few 256x128 tiles and a long K (W2 at 512 rows: 64 tiles, K = 11008): with one tile per
// workgroup most compute units idle, with smaller tiles every workgroup reads more operand bytes per
// multiply-add than its load path delivers.  So the large tiles stay and the K stages of each are
// dealt to cus / tiles workgroups, partial sums through the workspace -- when that leaves at least
// 40 stages per workgroup: the partial sums cost a second launch and M * N * 4 bytes per split each
// way (K = 11008, N = 4096: 73 -> 59 us with four splits; K = 4096, N = 4096: 25 -> 36 us with two).
// Returns the number of splits, 0 when the shape does not suit it.
inline int large_tile_splits(int M, int K, int N, int n_mats, long cus, size_t workspace_bytes) {
  const long tiles256 = (long)((M + 255) / 256) * ((N + 127) / 128) * n_mats;
  long splits = std::min<long>(cus / tiles256, 8);
  splits = std::min<long>(splits, K / BK / 40);
  if (M <= 64 || splits < 2 || (size_t)splits * M * N * n_mats * sizeof(float) > workspace_bytes) {
    return 0;
  }
  return (int)splits;
}

// The direct-to-LDS kernels fetch a thread's fp16 scale as the aligned 4-byte word that holds it:
// every scale array must then start on a 4-byte boundary and hold an even number of scales (the
// word of the last scale must not reach past the array).  Otherwise the register-staged kernel runs.
template <bool U8>
bool scale_words_ok(const operands_t& op, int K, int N, int block) {
  if constexpr (!U8) {
    return true;
  } else {
    if (((size_t)N * (size_t)(K / block)) % 2 != 0) {
      return false;
    }
    const half_t* all[3] = {op.S, op.n_mats > 1 ? op.more.S[0] : nullptr, op.n_mats > 2 ? op.more.S[1] : nullptr};
    for (const half_t* p : all) {
      if (p != nullptr && (reinterpret_cast<uintptr_t>(p) & 3) != 0) {
        return false;
      }
    }
    return true;
  }
}

// the split-K product of a few rows with its partial sums left in the workspace; *done = false when
// the shape does not take that path (nothing has been launched then)
template <bool U8>
int skinny_partial(operands_t op, const half_t* A, int M, int K, int N, int block, hipStream_t st, bool* done,
                   partial_sums_t* res) {
  *done = false;
  if (K % 128 != 0 || M > 64 || M < 1 || !scale_words_ok<U8>(op, K, N, block)) {
    return LCU_OK;
  }
  if constexpr (U8) {
    return launch_skinny<32, true>(op, A, M, K, N, block, 0.0f, st, done, res);
  } else {
    return M <= 32 ? launch_skinny<32, false>(op, A, M, K, N, block, 0.0f, st, done, res)
                   : launch_skinny<64, false>(op, A, M, K, N, block, 0.0f, st, done, res);
  }
}

// ---- kernels that add the partial sums up and go on with what follows the product in a batched
// decode step (llama_cu.cu:1144-1156, 1174-1176, 1180-1185), one row per sequence ----

__device__ __forceinline__ float2 sum_pair(const float* __restrict__ part, size_t at, size_t mn, int splits) {
  float2 v = *reinterpret_cast<const float2*>(part + at);
  for (int s = 1; s < splits; ++s) {
    const float2 w = *reinterpret_cast<const float2*>(part + (size_t)s * mn + at);
    v.x += w.x;
    v.y += w.y;
  }
  return v;
}

// Wq, Wk, Wv products -> fp16 -> rotary of q (to q_out) and k at pos[b]; rotated k and v into row
// pos[b] of sequence b's caches (what splitk_reduce_kernel + rope_store_batch_kernel do)
__global__ __launch_bounds__(256) void reduce_rope_store_kernel(half_t* __restrict__ q_out, const float* __restrict__ part,
                                                                int splits, int n_seq, int dim,
                                                                half_t* const* __restrict__ k_ptrs,
                                                                half_t* const* __restrict__ v_ptrs,
                                                                const int* __restrict__ pos_dev, int head_dim,
                                                                const float2* __restrict__ table, int max_pos) {
  const int pair = blockIdx.x * 256 + threadIdx.x;
  const int b = blockIdx.y;
  if (pair * 2 >= dim) return;
  const int c = pair * 2;
  const size_t mn = (size_t)n_seq * dim, at = (size_t)b * dim + c;
  const int pos = min(max(pos_dev[b], 0), max_pos);
  const float2 cs = table[(size_t)pos * (head_dim / 2) + (c % head_dim) / 2];
  const float2 qf = sum_pair(part, at, mn, splits);
  const float2 kf = sum_pair(part + (size_t)splits * mn, at, mn, splits);
  const float2 vf = sum_pair(part + (size_t)2 * splits * mn, at, mn, splits);
  // the products are rounded to fp16 before the rotary reads them (1144-1153)
  const float qr = (float)round_f16(qf.x), qi = (float)round_f16(qf.y);
  const float kr = (float)round_f16(kf.x), ki = (float)round_f16(kf.y);
  half2_t w;
  w.x = round_f16(fmaf(qr, cs.x, -(qi * cs.y)));
  w.y = round_f16(fmaf(qr, cs.y, qi * cs.x));
  *reinterpret_cast<half2_t*>(q_out + at) = w;
  const size_t dst = (size_t)pos * dim + c;
  w.x = round_f16(fmaf(kr, cs.x, -(ki * cs.y)));
  w.y = round_f16(fmaf(kr, cs.y, ki * cs.x));
  *reinterpret_cast<half2_t*>(k_ptrs[b] + dst) = w;
  w.x = round_f16(vf.x);
  w.y = round_f16(vf.y);
  *reinterpret_cast<half2_t*>(v_ptrs[b] + dst) = w;
}

// W1, W3 products -> fp16 each -> fp16(silu(w1) * w3)  (1180-1183, 533-539)
__global__ __launch_bounds__(256) void reduce_silu_kernel(half_t* __restrict__ out, const float* __restrict__ part,
                                                          int splits, size_t mn) {
  const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
  if (i >= mn) return;
  const float2 a = sum_pair(part, i, mn, splits);
  const float2 g = sum_pair(part + (size_t)splits * mn, i, mn, splits);
  const float v0 = (float)round_f16(a.x), v1 = (float)round_f16(a.y);
  half2_t w;
  w.x = round_f16(v0 / (1.0f + exp_ieee(-v0)) * (float)round_f16(g.x));
  w.y = round_f16(v1 / (1.0f + exp_ieee(-v1)) * (float)round_f16(g.y));
  *reinterpret_cast<half2_t*>(out + i) = w;
}

// x += product (one rounding of the fp32 sum, 1174 / 1185), then rms_norm of the new row with the
// next norm's weights (1176 / 1129 of the next layer / 1191).  One 1024-thread workgroup per row
// (up to 8192 columns: four pairs per thread, every partial sum requested before the first is
// used -- the launch is a handful of workgroups and nothing but latency); the norm as in
// rmsnorm_kernel, its sum of squares taken by the first 256 threads in the reference's association.
constexpr int RN_THREADS = 1024, RN_PAIRS = 4;
__global__ __launch_bounds__(RN_THREADS) void reduce_residual_norm_kernel(half_t* __restrict__ x,
                                                                          half_t* __restrict__ norm_out,
                                                                          const float* __restrict__ part, int splits,
                                                                          int n_seq, int cols,
                                                                          const half_t* __restrict__ norm_w, float eps) {
  extern __shared__ half_t row_lds[];
  __shared__ float red[8];
  const int b = blockIdx.x, tid = threadIdx.x;
  const size_t mn = (size_t)n_seq * cols;
  half_t* xr = x + (size_t)b * cols;
  float2 acc[RN_PAIRS];
  half2_t old[RN_PAIRS], wv[RN_PAIRS];
#pragma unroll
  for (int j = 0; j < RN_PAIRS; ++j) {
    const int c = min((tid + j * RN_THREADS) * 2, cols - 2);
    acc[j] = *reinterpret_cast<const float2*>(part + (size_t)b * cols + c);
    old[j] = *reinterpret_cast<const half2_t*>(xr + c);
    wv[j] = *reinterpret_cast<const half2_t*>(norm_w + c);
  }
  for (int s = 1; s < splits; ++s) {
#pragma unroll
    for (int j = 0; j < RN_PAIRS; ++j) {
      const int c = min((tid + j * RN_THREADS) * 2, cols - 2);
      const float2 w = *reinterpret_cast<const float2*>(part + (size_t)s * mn + (size_t)b * cols + c);
      acc[j].x += w.x;
      acc[j].y += w.y;
    }
  }
  half2_t val[RN_PAIRS];
#pragma unroll
  for (int j = 0; j < RN_PAIRS; ++j) {
    const int c = (tid + j * RN_THREADS) * 2;
    val[j].x = round_f16(fmaf(1.0f, (float)old[j].x, acc[j].x));
    val[j].y = round_f16(fmaf(1.0f, (float)old[j].y, acc[j].y));
    if (c < cols) {
      *reinterpret_cast<half2_t*>(xr + c) = val[j];
      *reinterpret_cast<half2_t*>(row_lds + c) = val[j];
    }
  }
  __syncthreads();
  float s = 0.0f;
  if (tid < 256) {
    for (int i = tid; i < cols; i += 256) {
      const float v = (float)row_lds[i];
      s = fmaf(v, v, s);
    }
  }
  // block256_sum_ref_order for the first 256 threads of a larger workgroup
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) {
    s += __shfl_xor(s, off, WAVE);
  }
  if (tid < 256 && (tid & 31) == 0) {
    red[tid >> 5] = s;
  }
  __syncthreads();
  float total = red[tid & 7];
#pragma unroll
  for (int off = 4; off > 0; off >>= 1) {
    total += __shfl_xor(total, off, WAVE);
  }
  const float rms_inv = 1.0f / sqrtf(total / (float)cols + eps);
  half_t* y = norm_out + (size_t)b * cols;
#pragma unroll
  for (int j = 0; j < RN_PAIRS; ++j) {
    const int c = (tid + j * RN_THREADS) * 2;
    if (c < cols) {
      half2_t r;
      r.x = round_f16((float)wv[j].x * (float)round_f16((float)val[j].x * rms_inv));
      r.y = round_f16((float)wv[j].y * (float)round_f16((float)val[j].y * rms_inv));
      *reinterpret_cast<half2_t*>(y + c) = r;
    }
  }
}

template <int BM, int BN, int KS>
constexpr size_t gemm_lds_bytes() {
  return (size_t)2 * (BM + BN) * (BK * KS + 8) * sizeof(half_t);
}

template <int BM, int BN, bool U8, bool KTAIL, int KS>
int launch_one(half_t* out, const half_t* A, const void* W, const half_t* S, int M, int K, int N, int block,
               float beta, int tiles_m, int tiles_n, hipStream_t st) {
  constexpr size_t lds = gemm_lds_bytes<BM, BN, KS>();
  static_assert(lds >= (size_t)BM * BN * 4 / 2 || KS == 1, "LDS must hold one group's accumulators");
  auto kernel = gemm_kernel<BM, BN, U8, KTAIL, KS>;
  if constexpr (lds > 64 * 1024) {
    static bool raised[16] = {};  // per device, once
    int dev = 0;
    LCU_HIP(hipGetDevice(&dev));
    if (!raised[dev & 15]) {
      LCU_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      raised[dev & 15] = true;
    }
  }
  kernel<<<tiles_m * tiles_n, 256 * KS, lds, st>>>(out, A, W, S, M, K, N, block, beta, tiles_m, tiles_n);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

template <int BM, int BN, bool U8, int KS>
int launch_gemm(half_t* out, const half_t* A, const void* W, const half_t* S, int M, int K, int N, int block,
                float beta, hipStream_t st) {
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  if (K % (BK * KS) == 0) {
    return launch_one<BM, BN, U8, false, KS>(out, A, W, S, M, K, N, block, beta, tiles_m, tiles_n, st);
  }
  return launch_one<BM, BN, U8, true, KS>(out, A, W, S, M, K, N, block, beta, tiles_m, tiles_n, st);
}

template <bool U8>
int dispatch_gemm(operands_t op, const half_t* A, int M, int K, int N, int block, float beta, hipStream_t st) {
  // Tile choice.  Large tiles read fewer operand bytes per multiply-add, and the per-CU load path
  // is what these kernels run against; but a compute unit needs two wavefronts per SIMD to overlap
  // LDS waits with matrix work.  So: 256x128 tiles with eight wavefronts when that still gives 160
  // workgroups (fp16 path); 128x128 with four when every compute unit gets one (two fit and
  // desynchronise: 344 such tiles at N = 11008 beat 344 workgroups of eight wavefronts); 128x64
  // with four wavefronts when there are more of them than compute units (two fit); else 128x64
  // with two groups of four wavefronts splitting the K stage, because then the grid cannot give a
  // compute unit a second workgroup (M = 512, N = 4096: 35 us against 41 us, K = 11008: 100 us
  // against 135 us with the register-staged kernel).
  // Several matrices of one shape (op.n_mats > 1) count as one product with n_mats * N columns --
  // unless each of them already fills the chip with 256x128 tiles and fusing saves no round of
  // workgroups (W1 + W3 at M = 512, N = 11008: 344 tiles take two rounds either way, and the fused
  // launch measured 132 us against 2 x 63 us).
  const bool whole_stages = K % 128 == 0 && scale_words_ok<U8>(op, K, N, block);
  if (op.n_mats > 1 && M > 64 && whole_stages) {
    device_state* ds = current_device_state();
    const long cus = ds && ds->compute_units > 0 ? ds->compute_units : 256;
    const long per = (long)((M + 255) / 256) * ((N + 127) / 128);
    if (per >= 160 && (per * op.n_mats + cus - 1) / cus >= op.n_mats * ((per + cus - 1) / cus)) {
      for (int g = 0; g < op.n_mats; ++g) {
        const operands_t one = single_matrix(g == 0 ? op.out : op.more.out[g - 1], g == 0 ? op.W : op.more.W[g - 1],
                                             g == 0 ? op.S : op.more.S[g - 1]);
        const int rc = dispatch_gemm<U8>(one, A, M, K, N, block, beta, st);
        if (rc != LCU_OK) {
          return rc;
        }
      }
      return LCU_OK;
    }
  }
  const long nm = op.n_mats;
  const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128) * nm;
  const long tiles64 = (long)((M + 127) / 128) * ((N + 63) / 64) * nm;
  if (whole_stages && M <= 64) {  // short prompts: the weight stream is what counts
    bool done = false;
    int rc;
    if constexpr (U8) {  // 64-row tiles with the code ring would leave LDS for one workgroup only
      rc = launch_skinny<32, true>(op, A, M, K, N, block, beta, st, &done);
    } else {
      rc = M <= 32 ? launch_skinny<32, false>(op, A, M, K, N, block, beta, st, &done)
                   : launch_skinny<64, false>(op, A, M, K, N, block, beta, st, &done);
    }
    if (rc != LCU_OK || done) {
      return rc;
    }
  }
  if (whole_stages) {  // whole stages: the direct-to-LDS kernels
    const long tiles256 = (long)((M + 255) / 256) * ((N + 127) / 128) * nm;
    if (tiles256 >= 160) return launch_dl<256, 128, 4, 2, 1, 3, U8>(op, A, M, K, N, block, beta, st);
    {
      device_state* ds = current_device_state();
      const workspace_t ws = workspace_for(st);
      if (ds != nullptr && ws.ptr != nullptr) {
        const int splits = large_tile_splits(M, K, N, op.n_mats, ds->compute_units > 0 ? ds->compute_units : 256, ws.bytes);
        if (splits > 0) {
          return launch_split<256, 128, 4, 2, U8>(op, A, M, K, N, block, beta, st, splits, (float*)ws.ptr);
        }
      }
    }
    if constexpr (!U8) {  // uint8 needs a code ring and two W tiles besides: too much LDS for two workgroups
      if (tiles128 >= 256) return launch_dl<128, 128, 2, 2, 1, 2, false>(op, A, M, K, N, block, beta, st);
    }
    if (tiles128 < 256) {
      if (tiles128 >= 160) return launch_dl<128, 128, 4, 2, 1, 3, U8>(op, A, M, K, N, block, beta, st);
      if (tiles64 > 256) return launch_dl<128, 64, 2, 2, 1, 3, U8>(op, A, M, K, N, block, beta, st);
      return launch_dl<128, 64, 2, 2, 2, 3, U8>(op, A, M, K, N, block, beta, st);
    }
  }
  // ragged K: the register-staged kernel, one matrix per launch
  for (int g = 0; g < op.n_mats; ++g) {
    half_t* out = g == 0 ? op.out : op.more.out[g - 1];
    const void* W = g == 0 ? op.W : op.more.W[g - 1];
    const half_t* S = g == 0 ? op.S : op.more.S[g - 1];
    const long t128 = tiles128 / nm, t64 = tiles64 / nm;
    int rc;
    if (t128 >= 256) {
      rc = launch_gemm<128, 128, U8, 1>(out, A, W, S, M, K, N, block, beta, st);
    } else if (t64 > 256) {
      rc = launch_gemm<128, 64, U8, 1>(out, A, W, S, M, K, N, block, beta, st);
    } else {
      rc = launch_gemm<128, 64, U8, 2>(out, A, W, S, M, K, N, block, beta, st);
    }
    if (rc != LCU_OK) {
      return rc;
    }
  }
  return LCU_OK;
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
  return dispatch_gemm<false>(single_matrix((half_t*)out_dev, rhs_dev, nullptr), (const half_t*)lhs_dev, M, K, N, 0, beta,
                              as_stream(stream));
}

int lcu_gemm_f16_nt_multi(void* const* out_dev, const void* lhs_dev, const void* const* rhs_dev, int n_mats, int M,
                          int K, int N, float beta, void* stream) {
  LCU_REQUIRE(out_dev && lhs_dev && rhs_dev && n_mats >= 1 && n_mats <= 3, "lcu_gemm_f16_nt_multi: bad arguments");
  for (int g = 0; g < n_mats; ++g) {
    LCU_REQUIRE(out_dev[g] && rhs_dev[g], "lcu_gemm_f16_nt_multi: null pointer");
  }
  if (M == 1 || n_mats == 1) {  // matrix-vector products and single matrices: the ordinary entry point
    for (int g = 0; g < n_mats; ++g) {
      const int rc = lcu_gemm_f16_nt(out_dev[g], lhs_dev, rhs_dev[g], M, K, N, beta, stream);
      if (rc != LCU_OK) return rc;
    }
    return LCU_OK;
  }
  LCU_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 8 == 0, "lcu_gemm_f16_nt_multi: bad shape M %d K %d N %d (K %% 8 == 0)", M,
              K, N);
  if (M == 0) return LCU_OK;
  LCU_REQUIRE((size_t)M * K * 2 < ((size_t)1 << 32) && (size_t)N * K * 2 < ((size_t)1 << 32),
              "lcu_gemm_f16_nt_multi: operands of 4 GiB or more are not supported");
  operands_t op = single_matrix((half_t*)out_dev[0], rhs_dev[0], nullptr);
  op.n_mats = n_mats;
  for (int g = 1; g < n_mats; ++g) {
    op.more.out[g - 1] = (half_t*)out_dev[g];
    op.more.W[g - 1] = rhs_dev[g];
  }
  return dispatch_gemm<false>(op, (const half_t*)lhs_dev, M, K, N, 0, beta, as_stream(stream));
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
  return dispatch_gemm<true>(single_matrix((half_t*)out_dev, codes_dev, (const half_t*)scales_dev), (const half_t*)lhs_dev,
                             M, K, N, block, beta, as_stream(stream));
}

int lcu_gemm_f16u8_nt_multi(void* const* out_dev, const void* lhs_dev, const void* const* codes_dev,
                            const void* const* scales_dev, int n_mats, int M, int K, int N, int block, float beta,
                            void* stream) {
  LCU_REQUIRE(out_dev && lhs_dev && codes_dev && scales_dev && n_mats >= 1 && n_mats <= 3,
              "lcu_gemm_f16u8_nt_multi: bad arguments");
  for (int g = 0; g < n_mats; ++g) {
    LCU_REQUIRE(out_dev[g] && codes_dev[g] && scales_dev[g], "lcu_gemm_f16u8_nt_multi: null pointer");
  }
  if (M == 1 || n_mats == 1) {
    for (int g = 0; g < n_mats; ++g) {
      const int rc = lcu_gemm_f16u8_nt(out_dev[g], lhs_dev, codes_dev[g], scales_dev[g], M, K, N, block, beta, stream);
      if (rc != LCU_OK) return rc;
    }
    return LCU_OK;
  }
  LCU_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 16 == 0 && block >= 16 && block % 16 == 0 && K % block == 0,
              "lcu_gemm_f16u8_nt_multi: bad shape M %d K %d N %d block %d", M, K, N, block);
  if (M == 0) return LCU_OK;
  LCU_REQUIRE((size_t)M * K * 2 < ((size_t)1 << 32) && (size_t)N * K < ((size_t)1 << 32),
              "lcu_gemm_f16u8_nt_multi: operands of 4 GiB or more are not supported");
  operands_t op = single_matrix((half_t*)out_dev[0], codes_dev[0], (const half_t*)scales_dev[0]);
  op.n_mats = n_mats;
  for (int g = 1; g < n_mats; ++g) {
    op.more.out[g - 1] = (half_t*)out_dev[g];
    op.more.W[g - 1] = codes_dev[g];
    op.more.S[g - 1] = (const half_t*)scales_dev[g];
  }
  return dispatch_gemm<true>(op, (const half_t*)lhs_dev, M, K, N, block, beta, as_stream(stream));
}

// ---- fused steps of a batched decode (one row per sequence) ----

static operands_t make_operands(void* const* outs, const void* const* values, const void* const* scales, int count) {
  operands_t op = single_matrix((half_t*)(outs ? outs[0] : nullptr), values[0], (const half_t*)(scales ? scales[0] : nullptr));
  op.n_mats = count;
  for (int g = 1; g < count; ++g) {
    op.more.out[g - 1] = (half_t*)(outs ? outs[g] : nullptr);
    op.more.W[g - 1] = values[g];
    op.more.S[g - 1] = (const half_t*)(scales ? scales[g] : nullptr);
  }
  return op;
}

int lcu_batch_qkv(void* q_out_dev, void* k_tmp_dev, void* v_tmp_dev, const void* lhs_dev, const void* const* w_dev,
                  const void* const* scales_dev, int block, int n_seq, int dim, int n_heads,
                  const void* k_cache_ptrs_dev, const void* v_cache_ptrs_dev, const void* pos_dev,
                  const void* table_dev, int table_positions, void* stream) {
  LCU_REQUIRE(q_out_dev && k_tmp_dev && v_tmp_dev && lhs_dev && w_dev && w_dev[0] && w_dev[1] && w_dev[2] &&
                  k_cache_ptrs_dev && v_cache_ptrs_dev && pos_dev && table_dev,
              "lcu_batch_qkv: null pointer");
  LCU_REQUIRE(n_seq >= 0 && dim > 0 && n_heads > 0 && dim % n_heads == 0 && (dim / n_heads) % 2 == 0 && dim % 16 == 0 &&
                  table_positions > 0,
              "lcu_batch_qkv: bad shape n_seq %d dim %d heads %d", n_seq, dim, n_heads);
  LCU_REQUIRE(block == 0 || (scales_dev && scales_dev[0] && scales_dev[1] && scales_dev[2] && block % 16 == 0 &&
                             dim % block == 0),
              "lcu_batch_qkv: quantised weights need scales and a block dividing dim");
  if (n_seq == 0) return LCU_OK;
  hipStream_t st = as_stream(stream);
  void* const outs[3] = {q_out_dev, k_tmp_dev, v_tmp_dev};
  bool done = false;
  partial_sums_t ps{};
  if (n_seq > 1) {
    const operands_t op = make_operands(outs, w_dev, block ? scales_dev : nullptr, 3);
    const int rc = block ? skinny_partial<true>(op, (const half_t*)lhs_dev, n_seq, dim, dim, block, st, &done, &ps)
                         : skinny_partial<false>(op, (const half_t*)lhs_dev, n_seq, dim, dim, 0, st, &done, &ps);
    if (rc != LCU_OK) return rc;
  }
  if (done) {
    reduce_rope_store_kernel<<<dim3((dim / 2 + 255) / 256, n_seq), 256, 0, st>>>(
        (half_t*)q_out_dev, ps.part, ps.splits, n_seq, dim, (half_t* const*)k_cache_ptrs_dev,
        (half_t* const*)v_cache_ptrs_dev, (const int*)pos_dev, dim / n_heads, (const float2*)table_dev,
        table_positions - 1);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
  }
  // any other shape: the three products, then rotary and cache append
  const int rc = block ? lcu_gemm_f16u8_nt_multi(outs, lhs_dev, w_dev, scales_dev, 3, n_seq, dim, dim, block, 0.0f, stream)
                       : lcu_gemm_f16_nt_multi(outs, lhs_dev, w_dev, 3, n_seq, dim, dim, 0.0f, stream);
  if (rc != LCU_OK) return rc;
  return lcu_rope_store_batch(q_out_dev, k_tmp_dev, v_tmp_dev, k_cache_ptrs_dev, v_cache_ptrs_dev, pos_dev, n_seq, dim,
                              n_heads, table_dev, table_positions, stream);
}

int lcu_batch_ffn_up(void* out_dev, void* w1_tmp_dev, void* w3_tmp_dev, const void* lhs_dev, const void* const* w_dev,
                     const void* const* scales_dev, int block, int n_seq, int dim, int ffn, void* stream) {
  LCU_REQUIRE(out_dev && w1_tmp_dev && w3_tmp_dev && lhs_dev && w_dev && w_dev[0] && w_dev[1], "lcu_batch_ffn_up: null pointer");
  LCU_REQUIRE(n_seq >= 0 && dim > 0 && ffn > 0 && dim % 16 == 0 && ffn % 2 == 0, "lcu_batch_ffn_up: bad shape n_seq %d dim %d ffn %d",
              n_seq, dim, ffn);
  LCU_REQUIRE(block == 0 || (scales_dev && scales_dev[0] && scales_dev[1] && block % 16 == 0 && dim % block == 0),
              "lcu_batch_ffn_up: quantised weights need scales and a block dividing dim");
  if (n_seq == 0) return LCU_OK;
  hipStream_t st = as_stream(stream);
  void* const outs[2] = {w1_tmp_dev, w3_tmp_dev};
  bool done = false;
  partial_sums_t ps{};
  if (n_seq > 1) {
    const operands_t op = make_operands(outs, w_dev, block ? scales_dev : nullptr, 2);
    const int rc = block ? skinny_partial<true>(op, (const half_t*)lhs_dev, n_seq, dim, ffn, block, st, &done, &ps)
                         : skinny_partial<false>(op, (const half_t*)lhs_dev, n_seq, dim, ffn, 0, st, &done, &ps);
    if (rc != LCU_OK) return rc;
  }
  if (done) {
    const size_t mn = (size_t)n_seq * ffn;
    reduce_silu_kernel<<<(unsigned)((mn / 2 + 255) / 256), 256, 0, st>>>((half_t*)out_dev, ps.part, ps.splits, mn);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
  }
  const int rc = block ? lcu_gemm_f16u8_nt_multi(outs, lhs_dev, w_dev, scales_dev, 2, n_seq, dim, ffn, block, 0.0f, stream)
                       : lcu_gemm_f16_nt_multi(outs, lhs_dev, w_dev, 2, n_seq, dim, ffn, 0.0f, stream);
  if (rc != LCU_OK) return rc;
  return lcu_silu_mul(out_dev, w1_tmp_dev, w3_tmp_dev, (size_t)n_seq * ffn, stream);
}

int lcu_batch_proj_norm(void* x_dev, void* norm_out_dev, const void* lhs_dev, const void* w_dev, const void* scales_dev,
                        int block, int n_seq, int K, int dim, const void* norm_w_dev, float eps, void* stream) {
  LCU_REQUIRE(x_dev && norm_out_dev && lhs_dev && w_dev && norm_w_dev, "lcu_batch_proj_norm: null pointer");
  LCU_REQUIRE(n_seq >= 0 && dim > 0 && K > 0 && K % 16 == 0 && dim % 2 == 0 && dim <= 24576,
              "lcu_batch_proj_norm: bad shape n_seq %d K %d dim %d", n_seq, K, dim);
  LCU_REQUIRE(block == 0 || (scales_dev && block % 16 == 0 && K % block == 0),
              "lcu_batch_proj_norm: quantised weights need scales and a block dividing K");
  if (n_seq == 0) return LCU_OK;
  hipStream_t st = as_stream(stream);
  bool done = false;
  partial_sums_t ps{};
  if (n_seq > 1 && dim <= RN_THREADS * RN_PAIRS * 2) {
    const operands_t op = single_matrix((half_t*)x_dev, w_dev, (const half_t*)(block ? scales_dev : nullptr));
    const int rc = block ? skinny_partial<true>(op, (const half_t*)lhs_dev, n_seq, K, dim, block, st, &done, &ps)
                         : skinny_partial<false>(op, (const half_t*)lhs_dev, n_seq, K, dim, 0, st, &done, &ps);
    if (rc != LCU_OK) return rc;
  }
  if (done) {
    reduce_residual_norm_kernel<<<n_seq, RN_THREADS, (size_t)dim * 2, st>>>(
        (half_t*)x_dev, (half_t*)norm_out_dev, ps.part, ps.splits, n_seq, dim, (const half_t*)norm_w_dev, eps);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
  }
  const int rc = block ? lcu_gemm_f16u8_nt(x_dev, lhs_dev, w_dev, scales_dev, n_seq, K, dim, block, 1.0f, stream)
                       : lcu_gemm_f16_nt(x_dev, lhs_dev, w_dev, n_seq, K, dim, 1.0f, stream);
  if (rc != LCU_OK) return rc;
  return lcu_rmsnorm(norm_out_dev, x_dev, norm_w_dev, n_seq, dim, eps, stream);
}

}  // extern "C"
