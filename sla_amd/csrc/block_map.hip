// Block-mask builder for Sparse-Linear Attention on gfx950.
//
// Stands in for sparse_linear_attention/utils.py:21-67 of the reference:
//   arg_k = k - mean_L(k); pooled_q = mean_pool(q, BLKQ); pooled_k = mean_pool(arg_k, BLKK);
//   score = pooled_q @ pooled_k^T; lut = topk(score); map = scatter(lut).
//
// All of this is HBM-bound streaming or tiny, so it runs on the vector ALUs with a
// FIXED fp32 summation order that a CPU checker can follow bit for bit:
//   block mean : rows added one at a time in ascending order, one IEEE division;
//   column mean: 64-row chunk sums (same order); groups of 32 consecutive chunk sums added in
//                ascending order; group sums added in ascending order; one IEEE division by L;
//   score      : acc = acc + (a_d * b_d), d ascending, no fused multiply-add.
// Selection is by (score descending, index ascending); -0.0 == +0.0.
#include "common.h"

#include <mutex>

#pragma clang fp contract(off)

namespace sla {

constexpr int KMEAN_CHUNK = 64;   // rows per level-1 sum
constexpr int KMEAN_GROUP = 32;   // level-1 sums per level-2 sum

// KEY_LOW_BIT: lowest bit of the fp32 image of a value of this type that can be non-zero.
struct IoF32 {
  typedef float raw;
  static constexpr int VEC = 4;
  static constexpr int KEY_LOW_BIT = 0;
  static __device__ __forceinline__ float ld(raw x) { return x; }
  static __device__ __forceinline__ raw st(float x) { return x; }
};
struct IoBf16 {
  typedef uint16_t raw;
  static constexpr int VEC = 8;
  static constexpr int KEY_LOW_BIT = 16;
  static __device__ __forceinline__ float ld(raw x) { return Elem<bf16_tag>::to_float(x); }
  static __device__ __forceinline__ raw st(float x) { return Elem<bf16_tag>::from_float(x); }
};
struct IoF16 {
  typedef uint16_t raw;
  static constexpr int VEC = 8;
  static constexpr int KEY_LOW_BIT = 13;
  static __device__ __forceinline__ float ld(raw x) { return Elem<f16_tag>::to_float(x); }
  static __device__ __forceinline__ raw st(float x) { return Elem<f16_tag>::from_float(x); }
};

template <typename IO>
struct alignas(16) Vec16 {
  typename IO::raw e[IO::VEC];
};

// MODE 0: fp32 block sums (no division)        -> out_f32 (BH, nblk, D)
// MODE 1: block mean in the input dtype        -> out     (BH, nblk, D)
// MODE 2: block mean of round(x - colmean)     -> out     (BH, nblk, D)
// One thread owns VEC adjacent columns of one block and walks its rows in order.
template <typename IO, int MODE>
static __device__ __forceinline__ void pool_body(const typename IO::raw* __restrict__ x, const RowLayout lay,
                                                 const typename IO::raw* __restrict__ colmean, void* __restrict__ out, int L,
                                                 int D, int BLK, int nblk, int bx, int bh) {
  constexpr int VEC = IO::VEC;
  const int tpr = D / VEC;
  const int bpw = 256 / tpr;
  const int sub = threadIdx.x / tpr;
  const int blk = bx * bpw + sub;
  const int c = (threadIdx.x - sub * tpr) * VEC;
  if (sub >= bpw || blk >= nblk) return;
  const int row0 = blk * BLK;
  const int nrows = min(BLK, L - row0);
  float acc[VEC];
  float cm[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
  if (MODE == 2) {
    Vec16<IO> m = *reinterpret_cast<const Vec16<IO>*>(colmean + (size_t)bh * D + c);
#pragma unroll
    for (int e = 0; e < VEC; ++e) cm[e] = IO::ld(m.e[e]);
  }
  const size_t pitch = (size_t)lay.sl;
  const typename IO::raw* p = x + lay.head(bh) + (size_t)row0 * pitch + c;
  // rows are fetched sixteen at a time (all loads of a batch in flight together), then added in row order
  constexpr int BATCH = 16;
  int r = 0;
  for (; r + BATCH <= nrows; r += BATCH) {
    Vec16<IO> v[BATCH];
#pragma unroll
    for (int i = 0; i < BATCH; ++i) v[i] = *reinterpret_cast<const Vec16<IO>*>(p + (size_t)(r + i) * pitch);
#pragma unroll
    for (int i = 0; i < BATCH; ++i)
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float f = IO::ld(v[i].e[e]);
        if (MODE == 2) f = IO::ld(IO::st(f - cm[e]));
        acc[e] = acc[e] + f;
      }
  }
  for (; r < nrows; ++r) {
    Vec16<IO> v = *reinterpret_cast<const Vec16<IO>*>(p + (size_t)r * pitch);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float f = IO::ld(v.e[e]);
      if (MODE == 2) f = IO::ld(IO::st(f - cm[e]));
      acc[e] = acc[e] + f;
    }
  }
  const size_t o = ((size_t)bh * nblk + blk) * D + c;
  if (MODE == 0) {
    float* of = reinterpret_cast<float*>(out) + o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) of[e] = acc[e];
  } else {
    const float cnt = (float)nrows;
    Vec16<IO> r;
#pragma unroll
    for (int e = 0; e < VEC; ++e) r.e[e] = IO::st(acc[e] / cnt);
    *reinterpret_cast<Vec16<IO>*>(reinterpret_cast<typename IO::raw*>(out) + o) = r;
  }
}

template <typename IO, int MODE>
__global__ __launch_bounds__(256) void pool_kernel(const typename IO::raw* __restrict__ x, const RowLayout lay,
                                                   const typename IO::raw* __restrict__ colmean,
                                                   void* __restrict__ out, int L, int D, int BLK, int nblk) {
  pool_body<IO, MODE>(x, lay, colmean, out, L, D, BLK, nblk, blockIdx.x, blockIdx.y);
}

// The two independent first passes of the mask builder in one launch (neither fills the memory system alone):
// blockIdx.z == 0: block means of q (MODE 1); z == 1: fp32 chunk sums of k (MODE 0, chunks of KMEAN_CHUNK rows).  K comes
// second because the next pass reads it again: what of it is still in the memory-side cache then is the part read last
// (module forward at B1 H12 L32760: 0.493 against 0.498 ms with k first).
template <typename IO>
__global__ __launch_bounds__(256) void pool_pair_kernel(const typename IO::raw* __restrict__ k, float* __restrict__ chunk_sums,
                                                        int nchunk, const typename IO::raw* __restrict__ q,
                                                        const RowLayout lay, typename IO::raw* __restrict__ pq, int BLKQ,
                                                        int nblkq, int L, int D) {
  if (blockIdx.z == 1)
    pool_body<IO, 0>(k, lay, nullptr, chunk_sums, L, D, KMEAN_CHUNK, nchunk, blockIdx.x, blockIdx.y);
  else
    pool_body<IO, 1>(q, lay, nullptr, pq, L, D, BLKQ, nblkq, blockIdx.x, blockIdx.y);
}

// Column mean of K, levels 2 and 3 of the fixed summation order:
//   group_sums[bh][g][d] = chunk sums of group g (KMEAN_GROUP consecutive chunks) added in ascending order;
//   colmean[bh][d]       = (group sums added in ascending order) / L, rounded to the input dtype.
__global__ __launch_bounds__(128) void colmean_group_kernel(const float* __restrict__ chunk_sums,
                                                            float* __restrict__ group_sums, int nchunk, int ngroup, int D) {
  const int g = blockIdx.x, bh = blockIdx.y;
  const int c0 = g * KMEAN_GROUP;
  const int n = min(KMEAN_GROUP, nchunk - c0);
  for (int d = threadIdx.x; d < D; d += 128) {
    const float* p = chunk_sums + ((size_t)bh * nchunk + c0) * D + d;
    float acc = 0.f;
#pragma unroll 8
    for (int i = 0; i < n; ++i) acc = acc + p[(size_t)i * D];
    group_sums[((size_t)bh * ngroup + g) * D + d] = acc;
  }
}

template <typename IO>
__global__ __launch_bounds__(128) void colmean_kernel(const float* __restrict__ group_sums,
                                                      typename IO::raw* __restrict__ colmean, int ngroup, int D, int L) {
  const int bh = blockIdx.y;
  const int d = blockIdx.x * blockDim.x + threadIdx.x;
  if (d >= D) return;
  const float* p = group_sums + (size_t)bh * ngroup * D + d;
  float acc = 0.f;
#pragma unroll 8
  for (int i = 0; i < ngroup; ++i) acc = acc + p[(size_t)i * D];
  colmean[(size_t)bh * D + d] = IO::st(acc / (float)L);
}

// Levels 2 and 3 in one launch when the group sums of a column slab fit in LDS: one workgroup per (head, slab of
// COLMEAN_SLAB columns), thread (gi, c) = (tid / COLMEAN_SLAB, tid % COLMEAN_SLAB) forms group sums gi, gi + 16, ...
// of its column; the first COLMEAN_SLAB threads then add the groups in ascending order.  (Small workgroups: the
// launch has to find room beside the memory-bound kernels that run on other streams at the same time.)
constexpr int COLMEAN_SLAB = 16;
constexpr int COLMEAN_MAX_GROUPS = 256;
template <typename IO>
__global__ __launch_bounds__(256) void colmean_fused_kernel(const float* __restrict__ chunk_sums,
                                                            typename IO::raw* __restrict__ colmean, int nchunk, int ngroup,
                                                            int D, int L) {
  __shared__ float gs[COLMEAN_MAX_GROUPS * COLMEAN_SLAB];
  const int bh = blockIdx.y, tid = threadIdx.x;
  const int c = tid % COLMEAN_SLAB, d = blockIdx.x * COLMEAN_SLAB + c;
  for (int g = tid / COLMEAN_SLAB; g < ngroup; g += 256 / COLMEAN_SLAB) {
    const int c0 = g * KMEAN_GROUP;
    const int n = min(KMEAN_GROUP, nchunk - c0);
    const float* p = chunk_sums + ((size_t)bh * nchunk + c0) * D + d;
    float acc = 0.f;
#pragma unroll 8
    for (int i = 0; i < n; ++i) acc = acc + p[(size_t)i * D];
    gs[g * COLMEAN_SLAB + c] = acc;
  }
  __syncthreads();
  if (tid < COLMEAN_SLAB) {
    float acc = 0.f;
    for (int g = 0; g < ngroup; ++g) acc = acc + gs[g * COLMEAN_SLAB + tid];
    colmean[(size_t)bh * D + d] = IO::st(acc / (float)L);
  }
}

// score[bh][m][n] = round_dtype( sum_d pq[m][d]*pk[n][d] ), d ascending, every product and every sum rounded to fp32.
// 64x64 outputs per workgroup, 4x4 per thread, operands staged through LDS 32 columns at a time.
// VECD (D a multiple of 32): every thread fetches eight adjacent d of one row of each operand with 16-byte loads,
// one chunk ahead of the chunk being accumulated.
template <typename IO, bool VECD>
__global__ __launch_bounds__(256) void score_kernel(const typename IO::raw* __restrict__ pq,
                                                    const typename IO::raw* __restrict__ pk,
                                                    typename IO::raw* __restrict__ score, int M, int N, int D) {
  constexpr int TS = 64, DC = 32, LD = TS + 4;
  constexpr int NV = 8 / IO::VEC;          // 16-byte loads per eight elements
  __shared__ __attribute__((aligned(16))) float sa[DC][LD];
  __shared__ __attribute__((aligned(16))) float sb[DC][LD];
  const int bh = blockIdx.z;
  const int m0 = blockIdx.y * TS, n0 = blockIdx.x * TS;
  const int tid = threadIdx.x;
  const int ty = tid >> 4, tx = tid & 15;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  const typename IO::raw* aq = pq + (size_t)bh * M * D;
  const typename IO::raw* bk = pk + (size_t)bh * N * D;
  const int lrow = tid >> 2, lseg = (tid & 3) * 8;
  Vec16<IO> va[NV], vb[NV];
  auto fetch = [&](int d0) {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
#pragma unroll
      for (int e = 0; e < IO::VEC; ++e) {
        va[v].e[e] = 0;
        vb[v].e[e] = 0;
      }
      if (m0 + lrow < M) va[v] = reinterpret_cast<const Vec16<IO>*>(aq + (size_t)(m0 + lrow) * D + d0 + lseg)[v];
      if (n0 + lrow < N) vb[v] = reinterpret_cast<const Vec16<IO>*>(bk + (size_t)(n0 + lrow) * D + d0 + lseg)[v];
    }
  };
  if (VECD) fetch(0);
  for (int d0 = 0; d0 < D; d0 += DC) {
    __syncthreads();
    if (VECD) {
#pragma unroll
      for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int e = 0; e < IO::VEC; ++e) {
          sa[lseg + v * IO::VEC + e][lrow] = IO::ld(va[v].e[e]);
          sb[lseg + v * IO::VEC + e][lrow] = IO::ld(vb[v].e[e]);
        }
    } else {
      for (int idx = tid; idx < TS * DC; idx += 256) {
        const int row = idx / DC, dd = idx % DC;
        const bool dok = d0 + dd < D;
        sa[dd][row] = (m0 + row < M && dok) ? IO::ld(aq[(size_t)(m0 + row) * D + d0 + dd]) : 0.f;
        sb[dd][row] = (n0 + row < N && dok) ? IO::ld(bk[(size_t)(n0 + row) * D + d0 + dd]) : 0.f;
      }
    }
    __syncthreads();
    if (VECD && d0 + DC < D) fetch(d0 + DC);
    const int dn = min(DC, D - d0);
    for (int dd = 0; dd < dn; ++dd) {
      const f32x4_t a = *reinterpret_cast<const f32x4_t*>(&sa[dd][ty * 4]);
      const f32x4_t b = *reinterpret_cast<const f32x4_t*>(&sb[dd][tx * 4]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (sizeof(typename IO::raw) == 2) {
            // the product of two 16-bit values is exact in fp32 (above the subnormal range), so the fused
            // form rounds the same sum once, exactly as the separate addition does, in half the instructions
            acc[i][j] = __builtin_fmaf(a[i], b[j], acc[i][j]);
          } else {
            const float prod = a[i] * b[j];
            acc[i][j] = acc[i][j] + prod;
          }
        }
    }
  }
  typename IO::raw* out = score + (size_t)bh * M * N;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) out[(size_t)m * N + n] = IO::st(acc[i][j]);
    }
  }
}

// The same scores from the matrix cores, for 16-bit dtypes.  v_mfma_f32_32x32x2_f32 adds its two products to the
// accumulator one after the other, each with a single rounding: k = 0 first, then k = 1.  A chain of them over
// d = 0, 2, 4, ... therefore is the d-ascending chain of fp32 fused multiply-adds of score_kernel, bit for bit (the
// product of two 16-bit values is exact in fp32, so fused or not makes no difference; values whose products fall
// into the fp32 subnormal range aside), at twice the rate of the vector ALU.
// 64 x 64NW scores per workgroup, one wave per 32 x 32NW part (NW independent accumulation chains).  The 64 pooled rows of either operand go through LDS
// (coalesced 16-byte loads; rows padded by 16 bytes, so that the row-per-lane reads are free of bank conflicts);
// lanes l and l + 32 read the same rows and feed the even and the odd d.  The rounded scores go back through LDS
// and leave in 256-byte runs.
template <typename IO, int D, int NW>
__global__ __launch_bounds__(256) void score_mfma_kernel(const typename IO::raw* __restrict__ pq,
                                                         const typename IO::raw* __restrict__ pk,
                                                         typename IO::raw* __restrict__ score, int M, int N) {
  static_assert(sizeof(typename IO::raw) == 2 && D % 32 == 0, "16-bit dtypes, 256 threads fetch whole rows");
  constexpr int NC = D / 8;              // 16-byte pieces per row
  constexpr int RS = D * 2 + 16;         // bytes between rows in LDS
  constexpr int OS = 64 * NW * 2 + 4;         // bytes between rows of the staged scores
  constexpr int TN = 64 * NW;            // scores per row of the workgroup's tile
  __shared__ __attribute__((aligned(16))) uint8_t sm[(64 + TN) * RS];
  static_assert(64 * OS <= (64 + TN) * RS, "the staged scores reuse the operand tiles");
  const int bh = blockIdx.z, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * (64 * NW);
  const __amdgpu_buffer_rsrc_t qh = make_rsrc(pq + (size_t)bh * M * D, (uint32_t)M * D * 2);    // rows past the end read as zero
  const __amdgpu_buffer_rsrc_t kh = make_rsrc(pk + (size_t)bh * N * D, (uint32_t)N * D * 2);
#pragma unroll
  for (int i = 0; i < 64 * NC / 256; ++i) {
    const int p = tid + 256 * i, row = p / NC, pc = p % NC;
    const i16x8_t a = buf_load_b128(qh, ((uint32_t)(m0 + row) * D + 8 * pc) * 2);
    i16x8_t b[NW];
#pragma unroll
    for (int t = 0; t < NW; ++t) b[t] = buf_load_b128(kh, ((uint32_t)(n0 + 64 * t + row) * D + 8 * pc) * 2);
    *reinterpret_cast<i16x8_t*>(sm + row * RS + pc * 16) = a;
#pragma unroll
    for (int t = 0; t < NW; ++t) *reinterpret_cast<i16x8_t*>(sm + (64 + 64 * t + row) * RS + pc * 16) = b[t];
  }
  __syncthreads();
  const int wm = wave >> 1, wn = wave & 1;
  const uint8_t* arow = sm + (wm * 32 + r) * RS;
  const uint8_t* brow = sm + (64 + wn * 32 * NW + r) * RS;      // this wave's NW tiles of 32 columns lie side by side
  f32x16_t acc[NW];
#pragma unroll
  for (int t = 0; t < NW; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
  const int sh = 16 * h;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const i32x4_t aw = *reinterpret_cast<const i32x4_t*>(arow + c * 16);
    i32x4_t bw[NW];
#pragma unroll
    for (int t = 0; t < NW; ++t) bw[t] = *reinterpret_cast<const i32x4_t*>(brow + 32 * t * RS + c * 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float av = IO::ld((typename IO::raw)((uint32_t)aw[j] >> sh));
#pragma unroll
      for (int t = 0; t < NW; ++t) {
        const float bv = IO::ld((typename IO::raw)((uint32_t)bw[t][j] >> sh));
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[t], 0, 0, 0);
      }
    }
  }
  __syncthreads();                       // every wave has read its operands: the tiles make room for the scores
#pragma unroll
  for (int t = 0; t < NW; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = wm * 32 + 8 * (i >> 2) + (i & 3) + 4 * h;
      *reinterpret_cast<typename IO::raw*>(sm + m * OS + (wn * 32 * NW + 32 * t + r) * 2) = IO::st(acc[t][i]);
    }
  __syncthreads();
  typename IO::raw* out = score + (size_t)bh * M * N;
  constexpr int TPR = 32 * NW;           // threads per row of staged scores, two scores each
  const int orow = tid / TPR, ocol = (tid % TPR) * 2;
#pragma unroll
  for (int pass = 0; pass < 64 * TPR / 256; ++pass) {
    const int ml = pass * (256 / TPR) + orow, m = m0 + ml, n = n0 + ocol;
    if (m >= M || n >= N) continue;
    const uint32_t two = *reinterpret_cast<const uint32_t*>(sm + ml * OS + ocol * 2);
    typename IO::raw* dst = out + (size_t)m * N + n;
    if (!(N & 1) && n + 1 < N) {
      *reinterpret_cast<uint32_t*>(dst) = two;          // (N even: every pair starts 4-byte aligned)
    } else {
      dst[0] = (typename IO::raw)(two & 0xffffu);
      if (n + 1 < N) dst[1] = (typename IO::raw)(two >> 16);
    }
  }
}

template <typename IO>
static void launch_score(const typename IO::raw* pq, const typename IO::raw* pk, typename IO::raw* score, int BH, int M, int N,
                         int D, hipStream_t st) {
  const dim3 grid(cdiv(N, 64), cdiv(M, 64), BH);
  if constexpr (sizeof(typename IO::raw) == 2) {
    const bool fits = (int64_t)M * D * 2 < (1ll << 32) && (int64_t)N * D * 2 < (1ll << 32);
    // (NW = 2, two column tiles per wave, is no faster: 159 against 153 us for 40 heads of 1182 x 1182 scores)
    if (D == 128 && fits) {
      hipLaunchKernelGGL((score_mfma_kernel<IO, 128, 1>), grid, dim3(256), 0, st, pq, pk, score, M, N);
      return;
    }
    if (D == 64 && fits) {
      hipLaunchKernelGGL((score_mfma_kernel<IO, 64, 1>), grid, dim3(256), 0, st, pq, pk, score, M, N);
      return;
    }
  }
  if (D % 32 == 0)
    hipLaunchKernelGGL((score_kernel<IO, true>), grid, dim3(256), 0, st, pq, pk, score, M, N, D);
  else
    hipLaunchKernelGGL((score_kernel<IO, false>), grid, dim3(256), 0, st, pq, pk, score, M, N, D);
}

// Monotone map float -> uint32 (larger float = larger key); -0.0 is folded onto +0.0.  The LOW_BIT
// low bits (zero in the fp32 image of every value of the score dtype) are cleared, also for negative
// values where the complement would set them, so the radix select can stop at LOW_BIT.
template <int LOW_BIT>
static __device__ __forceinline__ uint32_t order_key(float f) {
  uint32_t u = __float_as_uint(f);
  if (u == 0x80000000u) u = 0u;
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return u & ~((1u << LOW_BIT) - 1u);
}

// Inclusive prefix sum over the 64 lanes of a wave (data-parallel-primitive moves inside rows of 16 lanes, then the
// row totals are handed on).
static __device__ __forceinline__ int wave_inclusive_sum(int x, int lane) {
  const int rl = lane & 15;
  int t;
  t = __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false);      // row_shr:1
  if (rl >= 1) x += t;
  t = __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false);      // row_shr:2
  if (rl >= 2) x += t;
  t = __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false);      // row_shr:4
  if (rl >= 4) x += t;
  t = __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false);      // row_shr:8
  if (rl >= 8) x += t;
  t = __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false);      // row_bcast:15 (last lane of a row -> the next row)
  if ((lane & 31) >= 16) x += t;
  t = __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false);      // row_bcast:31 (lane 31 -> the upper half)
  if (lane >= 32) x += t;
  return x;
}

// One wavefront per (bh, m) row (four rows per workgroup): find the T-th largest key, then emit
// winners in ascending index order (ties at the threshold value go to the lowest indices).  Writes the int8 map row and the look-up-table row.
// EPL > 0: the row's keys live in EPL registers per lane (N <= 64*EPL); EPL == 0: keys in LDS.
// LOW_BIT: lowest key bit that can differ (16 for 16-bit score dtypes, whose low bits are zero).
template <typename IO, int EPL, int LOW_BIT>
__global__ __launch_bounds__(256) void topk_kernel(const typename IO::raw* __restrict__ score,
                                                   int8_t* __restrict__ sparse_map, void* __restrict__ lut, int lut64, int N,
                                                   int T, size_t nrows) {
  extern __shared__ uint32_t lds_keys[];
  // (the histograms are only used when the keys live in LDS: the register instances carry a token array)
  __shared__ __attribute__((aligned(16))) uint32_t hist_all[EPL == 0 ? 4 : 1][EPL == 0 ? 256 : 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t row = (size_t)blockIdx.x * 4 + wave;
  if (row >= nrows) return;
  const typename IO::raw* s = score + row * N;
  constexpr int NR = EPL > 0 ? EPL : 1;
  uint32_t kreg[NR];
  uint32_t* keys = lds_keys + (size_t)wave * (EPL > 0 ? 0 : N);
  const int nit = EPL > 0 ? EPL : (N + 63) / 64;
  // out-of-range slots hold key 0, below every real key (a real key has bit 31 set or is > 0 ... except
  // the most negative NaN pattern); they are excluded explicitly by the index test below.
  if (EPL > 0) {
#pragma unroll
    for (int e = 0; e < NR; ++e) {
      const int i = e * 64 + lane;
      kreg[e] = i < N ? order_key<LOW_BIT>(IO::ld(s[i])) : 0u;
    }
  } else {
    for (int i = lane; i < N; i += 64) keys[i] = order_key<LOW_BIT>(IO::ld(s[i]));
  }
  auto key_at = [&](int e) -> uint32_t {
    if (EPL > 0) return kreg[e < NR ? e : 0];
    const int i = e * 64 + lane;
    return i < N ? keys[i] : 0u;
  };
  // Keys in LDS: radix select, eight key bits per pass (two passes for bf16 scores): the keys that agree with the digits found
  // so far are counted per value of the next digit in a 256-bin histogram (LDS atomics of this wave on its own
  // bins); lane l then owns the four highest undecided digits 255 - 4l .. 252 - 4l, a prefix sum over the lanes
  // gives the number of keys above them, and the one lane whose digits straddle the wanted rank names the digit.
  if (T <= 0) {              // nothing to select (a ratio that rounds to no block at all): an all-zero map row, no table row
    int8_t* zrow = sparse_map + row * N;
    for (int i = lane; i < N; i += 64) zrow[i] = 0;
    return;
  }
  uint32_t thr = 0;          // digits decided so far
  int need = T;              // rank of the threshold among the keys that agree with them
  uint32_t* hist = hist_all[EPL == 0 ? wave : 0];
  if (EPL > 0) {
    // Keys in registers: the threshold is built bit by bit from the top, keeping a bit when at least T keys are at or
    // above the value it gives (one compare per key and bit, counted through the wave's ballot: no memory traffic and no
    // serialised atomics on the few histogram bins that the exponents of a row of scores fall into).  Slots past the
    // end of the row hold key 0 and are never at or above a candidate, which has at least one bit set.
    for (int b = 31; b >= LOW_BIT; --b) {
      const uint32_t cand = thr | (1u << b);
      int cnt = 0;
#pragma unroll
      for (int e = 0; e < NR; ++e) cnt += __popcll(__ballot(kreg[e] >= cand));
      if (cnt >= T) thr = cand;
    }
    int above = 0;
#pragma unroll
    for (int e = 0; e < NR; ++e) above += __popcll(__ballot(kreg[e] > thr));
    need = T - above;        // how many of the keys equal to the threshold are taken
  }
#pragma unroll
  for (int hi = EPL > 0 ? LOW_BIT : 32; hi > LOW_BIT;) {
    const int w = (hi - LOW_BIT) < 8 ? (hi - LOW_BIT) : 8;
    const int shift = hi - w;
    *reinterpret_cast<i32x4_t*>(&hist[4 * lane]) = i32x4_t{0, 0, 0, 0};
    wave_lds_fence();
    auto count_key = [&](int e, uint32_t kv) {
      const bool in = e * 64 + lane < N;
      const bool agrees = hi == 32 || ((kv ^ thr) >> (hi & 31)) == 0;
      if (in && agrees) atomicAdd(&hist[(kv >> shift) & ((1u << w) - 1u)], 1u);
    };
    if (EPL > 0) {
#pragma unroll
      for (int e = 0; e < NR; ++e) count_key(e, kreg[e]);
    } else {
      for (int e = 0; e < nit; ++e) count_key(e, key_at(e));
    }
    wave_lds_fence();
    const i32x4_t c4 = *reinterpret_cast<const i32x4_t*>(&hist[252 - 4 * lane]);    // digits 252 - 4l .. 255 - 4l
    const int c[4] = {c4[3], c4[2], c4[1], c4[0]};                                   // in descending order of the digit
    const int mine = c[0] + c[1] + c[2] + c[3];
    const int incl = wave_inclusive_sum(mine, lane);
    const int above = incl - mine;               // keys (among those that agree) whose digit is above all of this lane's
    const bool here = above < need && need <= incl;
    int digit = 0, rest = 0;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {             // (at most one of the four digits straddles the rank)
      int before = above;
#pragma unroll
      for (int t = 0; t < jj; ++t) before += c[t];
      if (before < need && need <= before + c[jj]) {
        digit = 255 - 4 * lane - jj;
        rest = need - before;
      }
    }
    const unsigned long long who = __ballot(here);
    const int src = who ? (int)__builtin_ctzll(who) : 0;
    digit = __builtin_amdgcn_readlane(digit, src);
    need = __builtin_amdgcn_readlane(rest, src);
    thr |= (uint32_t)digit << shift;
    hi = shift;
  }
  const int need_eq = need;
  int run_eq = 0, run_sel = 0;
  const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  int8_t* mrow = sparse_map + row * N;
  auto emit = [&](int e, uint32_t kv) {
    const int i = e * 64 + lane;
    const bool in = i < N;
    const bool gt = in && kv > thr;
    const bool eq = in && kv == thr;
    const unsigned long long beq = __ballot(eq);
    const int eq_rank = run_eq + __popcll(beq & lt_mask);
    const bool sel = gt || (eq && eq_rank < need_eq);
    const unsigned long long bsel = __ballot(sel);
    const int pos = run_sel + __popcll(bsel & lt_mask);
    if (in) mrow[i] = sel ? 1 : 0;
    if (sel && pos < T) {              // (pos < T always holds; the test keeps a wrong count from ever leaving the row)
      if (lut64)
        reinterpret_cast<long long*>(lut)[row * T + pos] = i;
      else
        reinterpret_cast<int*>(lut)[row * T + pos] = i;
    }
    run_eq += __popcll(beq);
    run_sel += __popcll(bsel);
  };
  if (EPL > 0) {
#pragma unroll
    for (int e = 0; e < NR; ++e)
      if (e * 64 < N) emit(e, kreg[e]);
  } else {
    for (int e = 0; e < nit; ++e) emit(e, key_at(e));
  }
}

template <typename IO>
static void launch_topk(const typename IO::raw* score, int8_t* sparse_map, void* lut, int lut64, int N, int T, size_t nrows,
                        hipStream_t st) {
  constexpr int LOW = IO::KEY_LOW_BIT;
  const dim3 grid((unsigned)((nrows + 3) / 4)), block(256);
  if (N <= 512)
    hipLaunchKernelGGL((topk_kernel<IO, 8, LOW>), grid, block, 0, st, score, sparse_map, lut, lut64, N, T, nrows);
  else if (N <= 1280)
    hipLaunchKernelGGL((topk_kernel<IO, 20, LOW>), grid, block, 0, st, score, sparse_map, lut, lut64, N, T, nrows);
  else if (N <= 2048)
    hipLaunchKernelGGL((topk_kernel<IO, 32, LOW>), grid, block, 0, st, score, sparse_map, lut, lut64, N, T, nrows);
  else
    hipLaunchKernelGGL((topk_kernel<IO, 0, LOW>), grid, block, (size_t)N * 16, st, score, sparse_map, lut, lut64, N, T, nrows);
}

struct MapWs {
  size_t chunk_sums, group_sums, colmean, pq, pk, score, total;
};

static MapWs map_ws(int dtype, int BH, int L, int D, int BLKQ, int BLKK) {
  const int64_t M = cdiv(L, BLKQ), N = cdiv(L, BLKK), nchunk = cdiv(L, KMEAN_CHUNK);
  const int64_t eb = elem_bytes(dtype);
  MapWs w;
  size_t off = 0;
  w.chunk_sums = off; off += align_up((int64_t)BH * nchunk * D * 4, 256);
  w.group_sums = off; off += align_up((int64_t)BH * cdiv((int)nchunk, KMEAN_GROUP) * D * 4, 256);
  w.colmean = off;    off += align_up((int64_t)BH * D * eb, 256);
  w.pq = off;         off += align_up((int64_t)BH * M * D * eb, 256);
  w.pk = off;         off += align_up((int64_t)BH * N * D * eb, 256);
  w.score = off;      off += align_up((int64_t)BH * M * N * eb, 256);
  w.total = off;
  return w;
}

int64_t block_map_workspace_bytes(int dtype, int BH, int L, int D, int BLKQ, int BLKK) {
  return (int64_t)map_ws(dtype, BH, L, D, BLKQ, BLKK).total;
}

static int validate_pool(int dtype, int BH, int L, int D, int BLK) {
  SLA_REQUIRE(dtype == SLA_F32 || dtype == SLA_BF16 || dtype == SLA_F16, SLA_ERR_BAD_ARG, "unknown dtype %d", dtype);
  SLA_REQUIRE(BH > 0 && L > 0 && D > 0 && BLK > 0, SLA_ERR_BAD_ARG, "non-positive size (BH=%d L=%d D=%d BLK=%d)", BH, L,
              D, BLK);
  const int vec = dtype == SLA_F32 ? 4 : 8;
  SLA_REQUIRE(D % vec == 0 && D / vec <= 256, SLA_ERR_UNSUPPORTED, "D=%d must be a multiple of %d and at most %d", D, vec,
              256 * vec);
  SLA_REQUIRE(BH <= 65535, SLA_ERR_UNSUPPORTED, "B*H=%d exceeds 65535", BH);
  return SLA_OK;
}

template <typename IO, int MODE>
static void launch_pool(const void* x, const RowLayout& lay, const void* colmean, void* out, int BH, int L, int D, int BLK,
                        hipStream_t st) {
  const int nblk = cdiv(L, BLK);
  const int bpw = 256 / (D / IO::VEC);
  dim3 grid(cdiv(nblk, bpw), BH);
  hipLaunchKernelGGL((pool_kernel<IO, MODE>), grid, dim3(256), 0, st, (const typename IO::raw*)x, lay,
                     (const typename IO::raw*)colmean, out, L, D, BLK, nblk);
}

// levels 2 and 3 of the K column mean from the chunk sums
template <typename IO>
static void launch_colmean_reduce(float* chunk_sums, float* group_sums, typename IO::raw* colmean, int BH, int L, int D,
                                  hipStream_t st) {
  const int nchunk = cdiv(L, KMEAN_CHUNK), ngroup = cdiv(nchunk, KMEAN_GROUP);
  if (D % COLMEAN_SLAB == 0 && ngroup <= COLMEAN_MAX_GROUPS) {
    hipLaunchKernelGGL((colmean_fused_kernel<IO>), dim3(D / COLMEAN_SLAB, BH), dim3(256), 0, st, chunk_sums, colmean, nchunk,
                       ngroup, D, L);
    return;
  }
  hipLaunchKernelGGL(colmean_group_kernel, dim3(ngroup, BH), dim3(128), 0, st, chunk_sums, group_sums, nchunk, ngroup, D);
  hipLaunchKernelGGL((colmean_kernel<IO>), dim3(cdiv(D, 128), BH), dim3(128), 0, st, group_sums, colmean, ngroup, D, L);
}

template <typename IO>
static void launch_k_colmean_t(const void* k, const RowLayout& lay, int BH, int L, int D, float* chunk_sums,
                               float* group_sums, typename IO::raw* colmean, hipStream_t st) {
  launch_pool<IO, 0>(k, lay, nullptr, chunk_sums, BH, L, D, KMEAN_CHUNK, st);
  launch_colmean_reduce<IO>(chunk_sums, group_sums, colmean, BH, L, D, st);
}

template <typename IO>
static int block_map_impl(const void* q, const void* k, const RowLayout& lay, int dtype, int BH, int L, int D, int BLKQ,
                          int BLKK, int topk, char* ws, int8_t* sparse_map, void* lut, int lut64, hipStream_t st) {
  const MapWs w = map_ws(dtype, BH, L, D, BLKQ, BLKK);
  const int M = cdiv(L, BLKQ), N = cdiv(L, BLKK);
  float* chunk_sums = (float*)(ws + w.chunk_sums);
  typename IO::raw* colmean = (typename IO::raw*)(ws + w.colmean);
  typename IO::raw* pq = (typename IO::raw*)(ws + w.pq);
  typename IO::raw* pk = (typename IO::raw*)(ws + w.pk);
  typename IO::raw* score = (typename IO::raw*)(ws + w.score);
  {
    // k chunk sums and q block means share one launch
    const int nchunk = cdiv(L, KMEAN_CHUNK);
    const int bpw = 256 / (D / IO::VEC);
    dim3 grid(cdiv(max(nchunk, M), bpw), BH, 2);
    hipLaunchKernelGGL((pool_pair_kernel<IO>), grid, dim3(256), 0, st, (const typename IO::raw*)k, chunk_sums, nchunk,
                       (const typename IO::raw*)q, lay, pq, BLKQ, M, L, D);
  }
  launch_colmean_reduce<IO>(chunk_sums, (float*)(ws + w.group_sums), colmean, BH, L, D, st);
  launch_pool<IO, 2>(k, lay, colmean, pk, BH, L, D, BLKK, st);
  launch_score<IO>(pq, pk, score, BH, M, N, D, st);
  // topk == 0 selects nothing: the kernel then only clears the map row.
  launch_topk<IO>(score, sparse_map, lut, lut64, N, topk, (size_t)BH * M, st);
  return check_launch("block map");
}

// Column mean of k over L in the fixed order, rounded to `dtype`.  scratch: fp32, at least
// k_colmean_scratch_floats(BH, L, D) elements; colmean: (BH, D) in `dtype`.
int64_t k_colmean_scratch_floats(int BH, int L, int D) {
  const int64_t nchunk = cdiv(L, KMEAN_CHUNK), ngroup = cdiv((int)nchunk, KMEAN_GROUP);
  return (int64_t)BH * (nchunk + ngroup) * D;
}
void launch_k_colmean(const void* k, const RowLayout& lay, int dtype, int BH, int L, int D, float* scratch, void* colmean,
                      hipStream_t st) {
  const int64_t nchunk = cdiv(L, KMEAN_CHUNK);
  float* chunk_sums = scratch;
  float* group_sums = scratch + (int64_t)BH * nchunk * D;
  if (dtype == SLA_F32)
    launch_k_colmean_t<IoF32>(k, lay, BH, L, D, chunk_sums, group_sums, (float*)colmean, st);
  else if (dtype == SLA_BF16)
    launch_k_colmean_t<IoBf16>(k, lay, BH, L, D, chunk_sums, group_sums, (uint16_t*)colmean, st);
  else
    launch_k_colmean_t<IoF16>(k, lay, BH, L, D, chunk_sums, group_sums, (uint16_t*)colmean, st);
}

// Scores and top-k selection from block means computed elsewhere (the quantisers of the SageSLA path
// produce them on the way): pq (BH, M, D), pk (BH, N, D) in `dtype`; score: (BH, M, N) elements of `dtype`.
void launch_map_from_pooled(int dtype, const void* pq, const void* pk, void* score, int BH, int M, int N, int D, int topk,
                            int8_t* sparse_map, void* lut, int lut64, hipStream_t st) {
  if (dtype == SLA_BF16) {
    launch_score<IoBf16>((const uint16_t*)pq, (const uint16_t*)pk, (uint16_t*)score, BH, M, N, D, st);
    launch_topk<IoBf16>((const uint16_t*)score, sparse_map, lut, lut64, N, topk, (size_t)BH * M, st);
  } else {
    launch_score<IoF16>((const uint16_t*)pq, (const uint16_t*)pk, (uint16_t*)score, BH, M, N, D, st);
    launch_topk<IoF16>((const uint16_t*)score, sparse_map, lut, lut64, N, topk, (size_t)BH * M, st);
  }
}

}  // namespace sla

using namespace sla;

extern "C" int sla_mean_pool(const void* x, void* out, int dtype, int BH, int L, int D, int BLK, void* stream) {
  int rc = validate_pool(dtype, BH, L, D, BLK);
  if (rc) return rc;
  SLA_REQUIRE(x && out, SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)x | (uintptr_t)out) % 16 == 0, SLA_ERR_BAD_ARG, "pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const RowLayout lay = contiguous_layout(BH, L, D);
  if (dtype == SLA_F32) launch_pool<IoF32, 1>(x, lay, nullptr, out, BH, L, D, BLK, st);
  else if (dtype == SLA_BF16) launch_pool<IoBf16, 1>(x, lay, nullptr, out, BH, L, D, BLK, st);
  else launch_pool<IoF16, 1>(x, lay, nullptr, out, BH, L, D, BLK, st);
  return check_launch("mean_pool");
}

static int block_map_entry(const void* q, const void* k, const int64_t* strides, int dtype, int B, int H, int L, int D,
                           int BLKQ, int BLKK, int topk, void* workspace, int64_t workspace_bytes, int8_t* sparse_map,
                           void* lut, int lut_elem_bytes, void* stream) {
  SLA_REQUIRE(B > 0 && H > 0, SLA_ERR_BAD_ARG, "non-positive batch/head count (B=%d H=%d)", B, H);
  const int64_t BH64 = (int64_t)B * H;
  SLA_REQUIRE(BH64 <= 65535, SLA_ERR_UNSUPPORTED, "B*H=%lld exceeds 65535", (long long)BH64);
  const int BH = (int)BH64;
  int rc = validate_pool(dtype, BH, L, D, BLKQ);
  if (rc) return rc;
  rc = validate_pool(dtype, BH, L, D, BLKK);
  if (rc) return rc;
  const int M = cdiv(L, BLKQ), N = cdiv(L, BLKK);
  SLA_REQUIRE(topk >= 0 && topk <= N, SLA_ERR_BAD_ARG, "topk=%d outside [0, %d]", topk, N);
  // (rows longer than the register instances hold keep their keys in LDS: four waves' rows of 4096 keys are 64 KB, plus
  //  4 KB of histograms, of the 160 KB a workgroup of this machine may use; L <= 262144 at 64-row key blocks)
  SLA_REQUIRE(N <= 4096, SLA_ERR_UNSUPPORTED, "more than 4096 key blocks (%d)", N);
  SLA_REQUIRE((int64_t)BH * M < (1ll << 31), SLA_ERR_UNSUPPORTED, "too many query-block rows");
  SLA_REQUIRE(lut_elem_bytes == 4 || lut_elem_bytes == 8, SLA_ERR_BAD_ARG, "lut_elem_bytes must be 4 or 8, got %d",
              lut_elem_bytes);
  SLA_REQUIRE(q && k && workspace && sparse_map && (lut || topk == 0), SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)workspace | (uintptr_t)lut) % 16 == 0, SLA_ERR_BAD_ARG,
              "pointers must be 16-byte aligned");
  const int64_t need = block_map_workspace_bytes(dtype, BH, L, D, BLKQ, BLKK);
  SLA_REQUIRE(workspace_bytes >= need, SLA_ERR_WORKSPACE, "workspace of %lld bytes, need %lld", (long long)workspace_bytes,
              (long long)need);
  RowLayout lay;
  rc = make_layout(strides, B, H, L, D, dtype == SLA_F32 ? 4 : 2, &lay);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  const int lut64 = lut_elem_bytes == 8;
  if (dtype == SLA_F32)
    return block_map_impl<IoF32>(q, k, lay, dtype, BH, L, D, BLKQ, BLKK, topk, ws, sparse_map, lut, lut64, st);
  if (dtype == SLA_BF16)
    return block_map_impl<IoBf16>(q, k, lay, dtype, BH, L, D, BLKQ, BLKK, topk, ws, sparse_map, lut, lut64, st);
  return block_map_impl<IoF16>(q, k, lay, dtype, BH, L, D, BLKQ, BLKK, topk, ws, sparse_map, lut, lut64, st);
}

extern "C" int sla_block_map_fwd(const void* q, const void* k, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK,
                                 int topk, void* workspace, int64_t workspace_bytes, int8_t* sparse_map, void* lut,
                                 int lut_elem_bytes, void* stream) {
  return block_map_entry(q, k, nullptr, dtype, B, H, L, D, BLKQ, BLKK, topk, workspace, workspace_bytes, sparse_map, lut,
                         lut_elem_bytes, stream);
}

// ---- the block-mask builder for callers that cannot allocate ---------------------------------------------------
// Same kernels as sla_block_map_fwd; the workspace is a fixed array in device memory that every GPU the library runs
// on holds from the moment the code object is loaded until the process ends.
static __device__ __align__(256) unsigned char scratch[SLA_STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[MAX_DEVICES];   // device address of `scratch` on each GPU, resolved on the first call there

// The array's name is only a handle on the host: its address in the current GPU's memory is looked up once per GPU.
int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  SLA_REQUIRE(e == hipSuccess && dev >= 0 && dev < MAX_DEVICES, SLA_ERR_LAUNCH, "hipGetDevice: %s (device %d)",
              hipGetErrorString(e), dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    SLA_REQUIRE(e == hipSuccess && p, SLA_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev,
                hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return SLA_OK;
}
}  // namespace

extern "C" int sla_block_map_fwd_static(const void* q, const void* k, int dtype, int B, int H, int L, int D, int BLKQ,
                                        int BLKK, int topk, int8_t* sparse_map, void* lut, int lut_elem_bytes,
                                        void* stream) {
  // sizes first (testable without a GPU): the problem must fit the fixed array
  SLA_REQUIRE(B > 0 && H > 0 && L > 0 && D > 0 && BLKQ > 0 && BLKK > 0 && (int64_t)B * H <= 65535, SLA_ERR_BAD_ARG,
              "bad size (B=%d H=%d L=%d D=%d BLKQ=%d BLKK=%d)", B, H, L, D, BLKQ, BLKK);
  SLA_REQUIRE(dtype == SLA_F32 || dtype == SLA_BF16 || dtype == SLA_F16, SLA_ERR_BAD_ARG, "unknown dtype %d", dtype);
  const int64_t need = block_map_workspace_bytes(dtype, B * H, L, D, BLKQ, BLKK);
  SLA_REQUIRE(need <= (int64_t)SLA_STATIC_SCRATCH_BYTES, SLA_ERR_WORKSPACE,
              "this problem needs %lld bytes of scratch, the static buffer holds %lld: use sla_block_map_fwd with a "
              "workspace of the caller's",
              (long long)need, (long long)SLA_STATIC_SCRATCH_BYTES);
  SLA_REQUIRE(q && k && sparse_map && (lut || topk == 0), SLA_ERR_BAD_ARG, "null pointer");
  void* ws = nullptr;
  int rc = static_scratch(&ws);
  if (rc) return rc;
  // every part of the scratch is written by one kernel of the sequence before a later one reads it: nothing
  // has to be cleared between calls
  return block_map_entry(q, k, nullptr, dtype, B, H, L, D, BLKQ, BLKK, topk, ws, (int64_t)SLA_STATIC_SCRATCH_BYTES,
                         sparse_map, lut, lut_elem_bytes, stream);
}

extern "C" int sla_block_map_fwd_strided(const void* q, const void* k, const int64_t* qk_strides, int dtype, int B, int H,
                                         int L, int D, int BLKQ, int BLKK, int topk, void* workspace,
                                         int64_t workspace_bytes, int8_t* sparse_map, void* lut, int lut_elem_bytes,
                                         void* stream) {
  SLA_REQUIRE(qk_strides, SLA_ERR_BAD_ARG, "null strides");
  return block_map_entry(q, k, qk_strides, dtype, B, H, L, D, BLKQ, BLKK, topk, workspace, workspace_bytes, sparse_map, lut,
                         lut_elem_bytes, stream);
}
