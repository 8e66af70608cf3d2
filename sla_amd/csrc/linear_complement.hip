// Linear branch over the NON-selected key blocks ("complement" mode), projection and final sum, for gfx950.
//
// The mounted reference computes the linear branch over all keys (sparse_linear_attention/core.py:92-96);
// the variant in which query block i only sees the key blocks it did not select for the sparse branch has no
// code there.  Definition used here (per head, S_i = look-up row of query block i, block size BLKK = 64):
//   h_j = phi(K_j)^T V_j (D x D),  z_j = sum_rows phi(K_j)            per key block j
//   H_i = sum_j h_j - sum_{j in S_i} h_j,   z_i likewise              per query block i
//   o_l = phi(Q_i) H_i / (1e-5 + phi(Q_i) . z_i);  out = residual + o_l W^T + b
// Rounding: phi, h_j, H_i, z_i, o_l are rounded to the 16-bit dtype where the global path rounds its
// counterparts; all sums of states are fp32 in a fixed order (ascending j, then the look-up row in order).
//
// Kernels:
//   block states : linear_state_partial_kernel with one 64-row slice per workgroup, 16-bit h_j^T, fp32 z_j
//   totals       : sum_j h_j, sum_j z_j in fp32 (groups of 16 blocks, then the groups)
//   out          : one workgroup per query block: gathers and subtracts the T selected states from the total
//                  (the same 32 KB-per-tile gather traffic as the sparse kernel's K/V tiles), rounds H_i^T
//                  into LDS and runs N^T = H_i^T phi(Q)^T, OUT^T = W Y^T for its rows in the transposed
//                  formulation of the global output kernel.
#include "linear_state.h"

namespace sla {

int validate_attn_shape(int dtype, int B, int H, int L, int D, int BLKQ, int BLKK, int topk, int lut_elem_bytes);
void launch_col_lists(const int8_t* sparse_map, int* list, int* count, int BH, int Mblk, int Nblk, hipStream_t st);
int64_t weight_grads_workspace_bytes(int BH, int L, int D);
void launch_weight_grads(int dtype, int D, const void* q, const void* dn, const void* gout, const void* y, const float* dden,
                         int BH, int L, int fmap, char* ws, float* d_weight, float* d_bias, hipStream_t st);

// Totals in two fixed-order levels: groups of TOTAL_GROUP consecutive key blocks, then the groups in order.
// level 1: grid (cdiv(D*D/8, 256), ngroup, BH), thread owns 8 adjacent elements of one group's D x D sum;
// level 2: grid (cdiv(D*D, 256), BH), thread owns one element.
constexpr int TOTAL_GROUP = 16;

template <typename Tag>
__global__ __launch_bounds__(256) void complement_group_kernel(const uint16_t* __restrict__ hblk,
                                                               const float* __restrict__ zblk, float* __restrict__ hgrp,
                                                               float* __restrict__ zgrp, int N, int D) {
  using E = Elem<Tag>;
  const int DD = D * D;
  const int grp = blockIdx.y, ngroup = gridDim.y, bh = blockIdx.z;
  const int j0 = grp * TOTAL_GROUP, j1 = min(N, j0 + TOTAL_GROUP);
  const int i = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (i < DD) {
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    const uint16_t* p = hblk + (size_t)bh * N * DD + i;
#pragma unroll 8
    for (int j = j0; j < j1; ++j) {
      const i16x8_t x = *reinterpret_cast<const i16x8_t*>(p + (size_t)j * DD);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += E::to_float((uint16_t)x[e]);
    }
    float* o = hgrp + ((size_t)bh * ngroup + grp) * DD + i;
    *reinterpret_cast<f32x4_t*>(o) = f32x4_t{acc[0], acc[1], acc[2], acc[3]};
    *reinterpret_cast<f32x4_t*>(o + 4) = f32x4_t{acc[4], acc[5], acc[6], acc[7]};
  }
  const int d = blockIdx.x * 256 + threadIdx.x;
  if (d < D) {
    float s = 0.f;
    for (int j = j0; j < j1; ++j) s += zblk[((size_t)bh * N + j) * D + d];
    zgrp[((size_t)bh * ngroup + grp) * D + d] = s;
  }
}

__global__ __launch_bounds__(256) void complement_total_kernel(const float* __restrict__ hgrp, const float* __restrict__ zgrp,
                                                               float* __restrict__ hall, float* __restrict__ zall, int ngroup,
                                                               int D) {
  const int DD = D * D;
  const int bh = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < DD) {
    float s = 0.f;
#pragma unroll 4
    for (int gi = 0; gi < ngroup; ++gi) s += hgrp[((size_t)bh * ngroup + gi) * DD + i];
    hall[(size_t)bh * DD + i] = s;
  }
  if (i < D) {
    float s = 0.f;
    for (int gi = 0; gi < ngroup; ++gi) s += zgrp[((size_t)bh * ngroup + gi) * D + i];
    zall[(size_t)bh * D + i] = s;
  }
}

// A D x D state held in fp32 registers: thread t of 256 owns the 16-byte chunks t + 256 c of the (row-major, 16-bit)
// block states, and element t of the z vectors when t < D.
template <int D>
static __device__ __forceinline__ void state_from_total(float (&acc)[D * D / 8 / 256][8], float& zacc,
                                                        const float* __restrict__ total, const float* __restrict__ ztotal,
                                                        int tid) {
#pragma unroll
  for (int c = 0; c < D * D / 8 / 256; ++c) {
    const int idx = (tid + 256 * c) * 8;
    const f32x4_t a = *reinterpret_cast<const f32x4_t*>(total + idx);
    const f32x4_t b = *reinterpret_cast<const f32x4_t*>(total + idx + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc[c][e] = a[e];
      acc[c][4 + e] = b[e];
    }
  }
  zacc = tid < D ? ztotal[tid] : 0.f;
}

// Adds or subtracts `count` listed block states, in list order.  `at(i)` is list entry i: a block index j >= 0 means
// "subtract block j", ~j (negative) means "add block j".  Two listed states are in flight while a third is being
// applied (the gather is latency-bound: bytes in flight per compute unit set its rate).
template <typename Tag, int D, typename At>
static __device__ __forceinline__ void apply_states(float (&acc)[D * D / 8 / 256][8], float& zacc,
                                                    const uint16_t* __restrict__ blocks, const float* __restrict__ zblocks,
                                                    int count, At at, int tid) {
  using E = Elem<Tag>;
  constexpr int DD = D * D;
  constexpr int NCH = DD / 8 / 256;
  i16x8_t ring[2][NCH];
  float zring[2] = {0.f, 0.f};
  float sgn[2] = {0.f, 0.f};
  auto fetch = [&](int slot, int i) {
    const int e = at(i);
    const int nb = e < 0 ? ~e : e;
    sgn[slot] = e < 0 ? 1.0f : -1.0f;
    const uint16_t* p = blocks + (size_t)nb * DD;
#pragma unroll
    for (int c = 0; c < NCH; ++c) ring[slot][c] = *reinterpret_cast<const i16x8_t*>(p + (tid + 256 * c) * 8);
    zring[slot] = tid < D ? zblocks[(size_t)nb * D + tid] : 0.f;
  };
  if (count > 0) fetch(0, 0);
  if (count > 1) fetch(1, 1);
  int it = 0;
  for (; it + 1 < count; it += 2) {       // slot parity is static inside the unrolled pair
    i16x8_t x[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) x[c] = ring[0][c];
    const float zx = zring[0], sx = sgn[0];
    if (it + 2 < count) fetch(0, it + 2);
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[c][e] += sx * E::to_float((uint16_t)x[c][e]);
    zacc += sx * zx;
#pragma unroll
    for (int c = 0; c < NCH; ++c) x[c] = ring[1][c];
    const float zy = zring[1], sy = sgn[1];
    if (it + 3 < count) fetch(1, it + 3);
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[c][e] += sy * E::to_float((uint16_t)x[c][e]);
    zacc += sy * zy;
  }
  if (it < count) {
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[c][e] += sgn[0] * E::to_float((uint16_t)ring[0][c][e]);
    zacc += sgn[0] * zring[0];
  }
}

// `total - sum of the listed blocks` (list entries are block indices, subtracted in list order).
// When the list names every block (`count == nblocks`) the difference is exactly zero by definition; it is
// returned as such instead of as the rounding residue of two fp32 sums formed in different orders, which the
// 1e-5 of the divisor would otherwise turn into an arbitrary result.
template <typename Tag, int D, typename At>
static __device__ __forceinline__ void gather_complement(float (&acc)[D * D / 8 / 256][8], float& zacc,
                                                         const float* __restrict__ total, const float* __restrict__ ztotal,
                                                         const uint16_t* __restrict__ blocks, const float* __restrict__ zblocks,
                                                         int count, int nblocks, At at, int tid) {
  if (count >= nblocks) {                    // (uniform over the workgroup)
#pragma unroll
    for (int c = 0; c < D * D / 8 / 256; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[c][e] = 0.f;
    zacc = 0.f;
    return;
  }
  state_from_total<D>(acc, zacc, total, ztotal, tid);
  apply_states<Tag, D>(acc, zacc, blocks, zblocks, count, at, tid);
}

// The gathered state, rounded to 16 bit, into an LDS matrix of D rows with row stride STR (same row-major
// order as the block states in memory).
template <typename Tag, int D, int STR>
static __device__ __forceinline__ void park_state(uint16_t* sH, const float (&acc)[D * D / 8 / 256][8], int tid) {
  using E = Elem<Tag>;
#pragma unroll
  for (int c = 0; c < D * D / 8 / 256; ++c) {
    const int idx = (tid + 256 * c) * 8;
    const int row = idx / D, col = idx % D;
    i32x4_t w;
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = (int)E::pack2(acc[c][2 * e], acc[c][2 * e + 1]);
    *reinterpret_cast<i32x4_t*>(&sH[row * STR + col]) = w;
  }
}

// Look-up rows of neighbouring query blocks share most of their entries, so a workgroup walks a run of COMPL_RUN
// consecutive query blocks of one head and keeps H_i in fp32 registers: the first block of the run gathers
// `total - its T selected states`, every later block only applies the difference of its look-up row against the
// previous one (adds back the states that dropped out, subtracts the new ones).  The difference lists are formed in
// a fixed order (dropped entries in the previous row's order, then new entries in this row's order), so results do
// not depend on scheduling.  Rows longer than COMPL_TMAX fall back to the full gather for every block.
constexpr int COMPL_RUN = 4;
constexpr int COMPL_TMAX = 256;

// The signed difference list between the previous look-up row (sPrev) and this one (sCur), both `T` entries in LDS:
// sList[0 .. ndrop) = ~j for the blocks j only the previous row names, sList[ndrop .. ndrop + nnew) = j for the blocks
// only this row names.  Returns ndrop + nnew.  All 256 threads call it; contains workgroup barriers.
static __device__ __forceinline__ int lut_difference(const int* sPrev, const int* sCur, int* sList, int (*sCnt)[4], int T,
                                                     int tid) {
  const int lane = tid & 63, wave = tid >> 6;
  bool isdrop = false, isnew = false;
  int p = 0, c = 0;
  if (tid < T) {
    p = sPrev[tid];
    c = sCur[tid];
    bool found_p = false, found_c = false;
    for (int u = 0; u < T; ++u) {
      found_p |= sCur[u] == p;
      found_c |= sPrev[u] == c;
    }
    isdrop = !found_p;
    isnew = !found_c;
  }
  const unsigned long long bd = __ballot(isdrop), bn = __ballot(isnew);
  if (lane == 0) {
    sCnt[0][wave] = __popcll(bd);
    sCnt[1][wave] = __popcll(bn);
  }
  __syncthreads();
  int ndrop = 0, nnew = 0, before_d = 0, before_n = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    before_d += w < wave ? sCnt[0][w] : 0;
    before_n += w < wave ? sCnt[1][w] : 0;
    ndrop += sCnt[0][w];
    nnew += sCnt[1][w];
  }
  const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  if (isdrop) sList[before_d + __popcll(bd & lt_mask)] = ~p;
  if (isnew) sList[ndrop + before_n + __popcll(bn & lt_mask)] = c;
  __syncthreads();
  return ndrop + nnew;
}

// 1-D grid over (head, run of COMPL_RUN query blocks) with the XCD-aware remap of the attention kernels: neighbouring
// runs select mostly the same key blocks, so their state reads hit the same XCD's L2.  256 threads.
template <typename Tag, int D, int BLKQ>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void complement_out_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ hblk,
                                                             const float* __restrict__ zblk, const float* __restrict__ hall,
                                                             const float* __restrict__ zall, const void* __restrict__ lut,
                                                             int lut64, const float* __restrict__ weight,
                                                             const float* __restrict__ bias, const uint16_t* __restrict__ residual,
                                                             uint16_t* __restrict__ out, int L, int Mblk, int N, int topk,
                                                             int fmap, int total) {
  using E = Elem<Tag>;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int STR = D + 8;
  constexpr int DD = D * D;
  constexpr int NCH = DD / 8 / 256;     // 16-byte chunks of the state per thread
  static_assert(DD / 8 % 256 == 0, "state does not divide among the threads");
  __shared__ __attribute__((aligned(16))) uint16_t sH[D * STR];    // H_i^T [d2][d1]
  __shared__ __attribute__((aligned(16))) uint16_t sW[D * STR];    // W [e][d2 in accumulator slot order]
  __shared__ float sBias[D];
  __shared__ float sZ[D];
  __shared__ int sPrev[COMPL_TMAX], sCur[COMPL_TMAX], sList[2 * COMPL_TMAX];
  __shared__ int sCnt[2][4];

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int runs = (Mblk + COMPL_RUN - 1) / COMPL_RUN;
  const int bh = logical / runs, mb0 = (logical - bh * runs) * COMPL_RUN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;

  // projection weight, 16 bit, columns in accumulator slot order; bias
  for (int idx = tid; idx < DD; idx += 256) {
    const int e = idx / D, d = idx % D;
    sW[e * STR + slot_order_pos(d)] = E::from_float(weight[idx]);
  }
  if (tid < D) sBias[tid] = round16<Tag>(bias[tid]);

  const uint16_t* hb = hblk + (size_t)bh * N * DD;
  const float* zb = zblk + (size_t)bh * N * D;
  const bool diffable = topk <= COMPL_TMAX && topk < N;
  float acc[NCH][8];
  float zacc;
#pragma nounroll
  for (int step = 0; step < COMPL_RUN; ++step) {
    const int mb = mb0 + step;
    if (mb >= Mblk) break;
    const size_t lut_row = ((size_t)bh * Mblk + mb) * topk;
    auto lut_at = [&](int i) -> int {
      return lut64 ? (int)reinterpret_cast<const long long*>(lut)[lut_row + i]
                   : reinterpret_cast<const int*>(lut)[lut_row + i];
    };
    // ---- H_i in fp32: total - selected for the first block of the run, the previous block's H plus the difference of
    // the two look-up rows afterwards ----
    const bool full = step == 0 || !diffable;          // (uniform over the workgroup)
    int count = topk;
    if (full) {
      if (diffable && tid < topk) sPrev[tid] = lut_at(tid);       // (read after the barriers below)
      if (topk >= N) {
        count = 0;                                                // everything selected: exactly zero, see gather_complement
#pragma unroll
        for (int c = 0; c < NCH; ++c)
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[c][e] = 0.f;
        zacc = 0.f;
      } else {
        state_from_total<D>(acc, zacc, hall + (size_t)bh * DD, zall + (size_t)bh * D, tid);
      }
    } else {
      if (tid < topk) sCur[tid] = lut_at(tid);
      __syncthreads();
      count = lut_difference(sPrev, sCur, sList, sCnt, topk, tid);
      if (tid < topk) sPrev[tid] = sCur[tid];                     // (every thread has passed the barriers of lut_difference)
    }
    auto entry_at = [&](int i) -> int { return full ? lut_at(i) : sList[i]; };
    apply_states<Tag, D>(acc, zacc, hb, zb, count, entry_at, tid);
    park_state<Tag, D, STR>(sH, acc, tid);
    if (tid < D) sZ[tid] = round16<Tag>(zacc);
    __syncthreads();
    if (wave < BLKQ / 32) {
      // ---- this wave's 32 queries ----
      const int qrow = mb * BLKQ + wave * 32 + r;
      const bool ok = qrow < L;
      const size_t off = ((size_t)bh * L + qrow) * D;
      i16x8_t xq[DC];
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        xq[c] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if (ok) xq[c] = *reinterpret_cast<const i16x8_t*>(q + off + 16 * c + 8 * g);
      }
      i16x8_t qf[DC];
      float den = phi_pack_den<Tag, DC>(fmap, xq, qf, [&](int c, int j) { return sZ[16 * c + 8 * g + j]; });
      den += __shfl_xor(den, 32);
      den = round16<Tag>(1e-5f + round16<Tag>(den));
      const float inv_den = 1.0f / den;

      // N^T = H_i^T phi(Q)^T ; Y^T = round(round(N^T) / den) packed straight into B-operand fragments
      i16x8_t yf[DT][2];
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        f32x16_t nacc;
#pragma unroll
        for (int i = 0; i < 16; ++i) nacc[i] = 0.f;
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          const i16x8_t a = *reinterpret_cast<const i16x8_t*>(&sH[(32 * t + r) * STR + 16 * c + 8 * g]);
          nacc = E::mfma32(a, qf[c], nacc);
        }
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {
          i32x4_t pw;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            pw[j] = (int)E::pack2(round16<Tag>(nacc[8 * c2 + 2 * j]) * inv_den, round16<Tag>(nacc[8 * c2 + 2 * j + 1]) * inv_den);
          yf[t][c2] = __builtin_bit_cast(i16x8_t, pw);
        }
      }
      // OUT^T = W Y^T : contraction chunk (t, c2) covers d2 = 32t + 16c2 .. +15 in slot order
#pragma unroll
      for (int et = 0; et < DT; ++et) {
        f32x16_t oacc;
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[i] = 0.f;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int c2 = 0; c2 < 2; ++c2) {
            const i16x8_t a = *reinterpret_cast<const i16x8_t*>(&sW[(32 * et + r) * STR + 16 * (2 * t + c2) + 8 * g]);
            oacc = E::mfma32(a, yf[t][c2], oacc);
          }
        if (ok) {
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const int e0 = 32 * et + 8 * i4 + 4 * g;
            float y[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) y[j] = round16<Tag>(oacc[4 * i4 + j] + sBias[e0 + j]);
            if (residual) {
              const i32x2_t rv = *reinterpret_cast<const i32x2_t*>(residual + off + e0);
              const uint16_t* rp = reinterpret_cast<const uint16_t*>(&rv);
#pragma unroll
              for (int j = 0; j < 4; ++j) y[j] += E::to_float(rp[j]);
            }
            i32x2_t w;
            w[0] = (int)E::pack2(y[0], y[1]);
            w[1] = (int)E::pack2(y[2], y[3]);
            *reinterpret_cast<i32x2_t*>(out + off + e0) = w;
          }
        }
      }
    }
    __syncthreads();                       // H_i^T and z_i are rewritten by the next block of the run
  }
}

// ---- backward ----------------------------------------------------------------------------
// With a = phi(q), c = phi(k), the states h_j, z_j, H_i, z_i as above, n = a H_i, den = 1e-5 + a . z_i, y = n / den,
// out = y W^T + b and G = d(out):
//   db = sum G ; dW = G^T y ; dy = G W ; dn = dy / den ; dden = -sum_d(dy * y) / den
//   da = dn H_i^T + dden z_i ; dq = phi'(q) da
//   dH_i = a_i^T dn_i (rows of query block i), dz_i = sum_rows dden a
//   G_j = sum_{i : j not in S_i} dH_i = sum_i dH_i - sum_{i in C_j} dH_i  (C_j = query blocks that selected j), gz_j likewise
//   dc = v G_j^T + gz_j ; dv = c G_j ; dk = phi'(k) dc                     (rows of key block j)
// Kernels (the totals, the per-block products and dW / db reuse kernels of the forward and of the global backward):
//   rows : one workgroup per query block: gathers H_i like the forward, then y, dy, dn, dden, da, dq for its rows on the
//          MFMA in transposed form; writes dq and the row-wise temporaries dn, y (16 bit), dden
//   kv   : one workgroup per key block: gathers G_j = total - listed dH_i, then dv, dc, dk for its 64 rows

// 1-D grid over (head, query block), XCD-aware order, 256 threads; waves 0 .. BLKQ/32-1 own 32 query rows each.
template <typename Tag, int D, int BLKQ>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void complement_bwd_rows_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ gout, const uint16_t* __restrict__ hblk,
    const float* __restrict__ zblk, const float* __restrict__ hall, const float* __restrict__ zall, const void* __restrict__ lut,
    int lut64, const uint16_t* __restrict__ wt, uint16_t* __restrict__ dq, uint16_t* __restrict__ dn_out,
    uint16_t* __restrict__ y_out, float* __restrict__ dden_out, int L, int Mblk, int N, int topk, int fmap, int total,
    int accumulate) {
  using E = Elem<Tag>;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int HSTR = D + 16;           // H_i^T is read row-wise (n^T = H^T a^T) and transposed (da^T = H dn^T)
  constexpr int XSTR = D + 8;
  constexpr int DD = D * D;
  constexpr int NCH = DD / 8 / 256;
  constexpr int XROWS = D > BLKQ ? D : BLKQ;
  __shared__ __attribute__((aligned(16))) uint16_t sHT[D * HSTR];      // H_i^T [d2][d1]
  // first the waves' staging tiles (q, G in), then W^T [d][e] (A of dy^T = W^T G^T), then staging tiles again (out)
  __shared__ __attribute__((aligned(16))) uint16_t sX[XROWS * XSTR];
  __shared__ float sZ[D];
  static_assert(TileRows<D>::SSTR == XSTR, "staging tiles and W^T share one row stride");

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int bh = logical / Mblk, mb = logical - bh * Mblk;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;
  const size_t lut_row = ((size_t)bh * Mblk + mb) * topk;
  auto lut_at = [&](int i) -> int {
    return lut64 ? (int)reinterpret_cast<const long long*>(lut)[lut_row + i]
                 : reinterpret_cast<const int*>(lut)[lut_row + i];
  };

  const int row0 = mb * BLKQ + wave * 32;
  const bool active = wave < BLKQ / 32 && row0 < L;     // (uniform per wave)
  const int rows_valid = min(32, L - row0);
  const int qrow = row0 + r;
  const bool ok = active && qrow < L;
  const size_t toff = ((size_t)bh * L + row0) * D;
  uint16_t* const stage = sX + wave * 32 * XSTR;

  // This wave's q and G rows are parked in LDS before the gather (held in registers they would not fit beside its
  // accumulators): q in the wave's staging tile, G in the still unused H_i^T buffer.
  constexpr bool G_IN_H = (BLKQ / 32) * 32 * XSTR <= D * HSTR;
  uint16_t* const gstage = G_IN_H ? sHT + wave * 32 * XSTR : stage;
  TileRows<D> gt;
  if (active) {
    TileRows<D> qt;
    qt.fetch(q + toff, rows_valid, lane);
    gt.fetch(gout + toff, rows_valid, lane);
    qt.park(stage, lane);
    if (G_IN_H) gt.park(gstage, lane);
  }
  float acc[NCH][8];
  float zacc;
  gather_complement<Tag, D>(acc, zacc, hall + (size_t)bh * DD, zall + (size_t)bh * D, hblk + (size_t)bh * N * DD,
                            zblk + (size_t)bh * N * D, topk, N, lut_at, tid);
  // G in B-operand order (d = 16c + 8g + j)
  i16x8_t gf[DC];
  if (active && G_IN_H) {
#pragma unroll
    for (int c = 0; c < DC; ++c) gf[c] = *reinterpret_cast<const i16x8_t*>(&gstage[r * XSTR + 16 * c + 8 * g]);
  }
  if (G_IN_H) __syncthreads();           // the G tiles have been read: the buffer takes H_i^T
  park_state<Tag, D, HSTR>(sHT, acc, tid);
  if (tid < D) sZ[tid] = round16<Tag>(zacc);
  __syncthreads();                       // H_i^T, z_i visible
  // q in B-operand order (d = 16c + 8g + j) -> a = phi(q) as B operand and the divisor; raw q in accumulator order
  // (d = 32t + 8i4 + 4g + j) for the gradient through phi
  i32x2_t xraw[DT][4];
  i16x8_t af[DC];
  float row_mx = 0.f, row_inv = 1.f, inv_den = 0.f;
  if (active) {
    float f[DC][8];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      const i16x8_t x = *reinterpret_cast<const i16x8_t*>(&stage[r * XSTR + 16 * c + 8 * g]);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)x[j]);
    }
#pragma unroll
    for (int t1 = 0; t1 < DT; ++t1)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        xraw[t1][i4] = *reinterpret_cast<const i32x2_t*>(&stage[r * XSTR + 32 * t1 + 8 * i4 + 4 * g]);
    if (!G_IN_H) {
      wave_lds_fence();
      gt.park(stage, lane);
#pragma unroll
      for (int c = 0; c < DC; ++c) gf[c] = *reinterpret_cast<const i16x8_t*>(&stage[r * XSTR + 16 * c + 8 * g]);
    }
    phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
    float den = 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i32x4_t pw;
#pragma unroll
      for (int j = 0; j < 8; ++j) den += f[c][j] * sZ[16 * c + 8 * g + j];
#pragma unroll
      for (int j = 0; j < 4; ++j) pw[j] = (int)E::pack2(f[c][2 * j], f[c][2 * j + 1]);
      af[c] = __builtin_bit_cast(i16x8_t, pw);
    }
    den += __shfl_xor(den, 32);
    den += 1e-5f;
    inv_den = 1.0f / den;
  }
  __syncthreads();                       // every wave has read its staging tile: the buffer takes W^T
  for (int idx = tid; idx < DD / 8; idx += 256) {
    const int row = idx / (D / 8), col = (idx % (D / 8)) * 8;
    *reinterpret_cast<i16x8_t*>(&sX[row * XSTR + col]) = *reinterpret_cast<const i16x8_t*>(wt + (size_t)row * D + col);
  }
  __syncthreads();                       // W^T visible

  float yv[DT][16], dnv[DT][16];
  if (active) {
    // y^T = (H_i^T a^T) / den ; dy^T = W^T G^T
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      f32x16_t yacc, dyacc;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        yacc[i] = 0.f;
        dyacc[i] = 0.f;
      }
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const i16x8_t a1 = *reinterpret_cast<const i16x8_t*>(&sHT[(32 * t + r) * HSTR + 16 * c + 8 * g]);
        yacc = E::mfma32(a1, af[c], yacc);
        const i16x8_t a2 = *reinterpret_cast<const i16x8_t*>(&sX[(32 * t + r) * XSTR + 16 * c + 8 * g]);
        dyacc = E::mfma32(a2, gf[c], dyacc);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        yv[t][i] = yacc[i];
        dnv[t][i] = dyacc[i];
      }
    }
  }
  __syncthreads();                       // W^T consumed: its rows are staging tiles again
  if (!active) return;

  float dden = 0.f;
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      yv[t][i] *= inv_den;
      dden += dnv[t][i] * yv[t][i];
      dnv[t][i] *= inv_den;          // dn^T
    }
  dden += __shfl_xor(dden, 32);
  dden = -dden * inv_den;
  if (ok && g == 0) dden_out[(size_t)bh * L + qrow] = dden;

  // dn^T as B operand: register 8c2+j of tile t is d2 = 32t + 16c2 + 8(j/4) + 4g + j%4
  i16x8_t dnf[DT][2];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2) {
      i32x4_t pw;
#pragma unroll
      for (int j = 0; j < 4; ++j) pw[j] = (int)E::pack2(dnv[t][8 * c2 + 2 * j], dnv[t][8 * c2 + 2 * j + 1]);
      dnf[t][c2] = __builtin_bit_cast(i16x8_t, pw);
    }
  TileRows<D> dq_old;
  if (accumulate) dq_old.fetch(dq + toff, rows_valid, lane);
  store_acc_tile<E, D>(stage, dnv, dn_out + toff, nullptr, rows_valid, lane);
  store_acc_tile<E, D>(stage, yv, y_out + toff, nullptr, rows_valid, lane);

  // da^T = H_i dn^T + z_i dden: rows d1 of H_i come out of H_i^T through the transposing read, the contraction
  // index d2 in the slot order of dn^T above
  const int tr_row = (lane & 15) >> 2;
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  float da[DT][16], xq[DT][16];
#pragma unroll
  for (int t1 = 0; t1 < DT; ++t1) {
    f32x16_t acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        const uint16_t* p0 = &sHT[(16 * (2 * t + c2) + 4 * g + tr_row) * HSTR + 32 * t1 + tr_col];
        acc = E::mfma32(concat4(lds_read_tr16(p0), lds_read_tr16(p0 + 8 * HSTR)), dnf[t][c2], acc);
      }
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int d0 = 32 * t1 + 8 * i4 + 4 * g;
      const uint16_t* xp = reinterpret_cast<const uint16_t*>(&xraw[t1][i4]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        da[t1][4 * i4 + j] = acc[4 * i4 + j] + sZ[d0 + j] * dden;
        xq[t1][4 * i4 + j] = E::to_float(xp[j]);
      }
    }
  }
  phi_backward<DT>(fmap, xq, da, row_mx, row_inv);
  store_acc_tile<E, D>(stage, da, dq + toff, accumulate ? &dq_old : nullptr, rows_valid, lane);
}

// 1-D grid over (head, key block), XCD-aware order, 256 threads; waves 0 and 1 own 32 key rows each.
// dhblk: per query block dH_i^T [d2][d1] (16 bit), dzblk: dz_i (fp32); gall / gzall: their sums over the query blocks.
template <typename Tag, int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void complement_bwd_kv_kernel(
    const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, const uint16_t* __restrict__ dhblk,
    const float* __restrict__ dzblk, const float* __restrict__ gall, const float* __restrict__ gzall,
    const int* __restrict__ list, const int* __restrict__ count, uint16_t* __restrict__ dk, uint16_t* __restrict__ dv, int L,
    int Mblk, int N, int fmap, int total, int accumulate) {
  using E = Elem<Tag>;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int GSTR = D + 16;           // G_j^T is read row-wise (dv^T = G^T c^T) and transposed (dc^T = G v^T)
  constexpr int SSTR = TileRows<D>::SSTR;
  constexpr int DD = D * D;
  constexpr int NCH = DD / 8 / 256;
  __shared__ __attribute__((aligned(16))) uint16_t sGT[D * GSTR];      // G_j^T [d2][d1]
  __shared__ __attribute__((aligned(16))) uint16_t sStage[2][32 * SSTR];
  __shared__ float sGZ[D];

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int bh = logical / N, nb = logical - bh * N;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;
  const int* mylist = list + ((size_t)bh * N + nb) * Mblk;
  auto list_at = [&](int i) -> int { return mylist[i]; };

  const int row0 = nb * 64 + wave * 32;
  const bool active = wave < 2 && row0 < L;
  const int rows_valid = min(32, L - row0);
  const size_t toff = ((size_t)bh * L + row0) * D;
  // this wave's k and v rows are parked in LDS before the gather: k in the wave's staging tile, v in the still
  // unused G_j^T buffer
  static_assert(2 * 32 * SSTR <= D * GSTR, "v tiles exceed the state buffer");
  uint16_t* const stage = sStage[wave & 1];
  uint16_t* const vstage = sGT + (wave & 1) * 32 * SSTR;
  if (active) {
    TileRows<D> kt, vt;
    kt.fetch(k + toff, rows_valid, lane);
    vt.fetch(v + toff, rows_valid, lane);
    kt.park(stage, lane);
    vt.park(vstage, lane);
  }
  float acc[NCH][8];
  float zacc;
  gather_complement<Tag, D>(acc, zacc, gall + (size_t)bh * DD, gzall + (size_t)bh * D, dhblk + (size_t)bh * Mblk * DD,
                            dzblk + (size_t)bh * Mblk * D, count[(size_t)bh * N + nb], Mblk, list_at, tid);
  i16x8_t vf[DC];
  if (active) {
#pragma unroll
    for (int c = 0; c < DC; ++c) vf[c] = *reinterpret_cast<const i16x8_t*>(&vstage[r * SSTR + 16 * c + 8 * g]);
  }
  __syncthreads();                       // the v tiles have been read: the buffer takes G_j^T
  park_state<Tag, D, GSTR>(sGT, acc, tid);
  if (tid < D) sGZ[tid] = zacc;
  __syncthreads();
  if (!active) return;

  float f[DC][8];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    const i16x8_t x = *reinterpret_cast<const i16x8_t*>(&stage[r * SSTR + 16 * c + 8 * g]);
#pragma unroll
    for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)x[j]);
  }
  i32x2_t xraw[DT][4];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) xraw[t][i4] = *reinterpret_cast<const i32x2_t*>(&stage[r * SSTR + 32 * t + 8 * i4 + 4 * g]);
  wave_lds_fence();
  float row_mx, row_inv;
  phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
  {
    // dv^T = G^T c^T
    i16x8_t cf[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i32x4_t pw;
#pragma unroll
      for (int j = 0; j < 4; ++j) pw[j] = (int)E::pack2(f[c][2 * j], f[c][2 * j + 1]);
      cf[c] = __builtin_bit_cast(i16x8_t, pw);
    }
    float dvv[DT][16];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      f32x16_t vacc;
#pragma unroll
      for (int i = 0; i < 16; ++i) vacc[i] = 0.f;
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const i16x8_t a2 = *reinterpret_cast<const i16x8_t*>(&sGT[(32 * t + r) * GSTR + 16 * c + 8 * g]);
        vacc = E::mfma32(a2, cf[c], vacc);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) dvv[t][i] = vacc[i];
    }
    if (accumulate)
      store_acc_tile<E, D, true>(stage, dvv, dv + toff, nullptr, rows_valid, lane);
    else
      store_acc_tile<E, D, false>(stage, dvv, dv + toff, nullptr, rows_valid, lane);
  }
  // dc^T = G v^T + gz ; dk = phi'(k) dc  (rows d1 of G through the transposing read, d2 in the order of v's fragments)
  const int tr_row = (lane & 15) >> 2;
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  float dc[DT][16], xk[DT][16];
#pragma unroll
  for (int t = 0; t < DT; ++t) {
    f32x16_t acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      const uint16_t* pa = &sGT[(16 * c + 8 * g + tr_row) * GSTR + 32 * t + tr_col];
      acc = E::mfma32(concat4(lds_read_tr16(pa), lds_read_tr16(pa + 4 * GSTR)), vf[c], acc);
    }
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int d0 = 32 * t + 8 * i4 + 4 * g;
      const uint16_t* xp = reinterpret_cast<const uint16_t*>(&xraw[t][i4]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dc[t][4 * i4 + j] = acc[4 * i4 + j] + sGZ[d0 + j];
        xk[t][4 * i4 + j] = E::to_float(xp[j]);
      }
    }
  }
  phi_backward<DT>(fmap, xk, dc, row_mx, row_inv);
  if (accumulate)
    store_acc_tile<E, D, true>(stage, dc, dk + toff, nullptr, rows_valid, lane);
  else
    store_acc_tile<E, D, false>(stage, dc, dk + toff, nullptr, rows_valid, lane);
}

// ---- host ---------------------------------------------------------------------------------
struct ComplWs {
  int ngroup;
  size_t hblk, zblk, hgrp, zgrp, hall, zall, total;
};
static ComplWs compl_ws(int BH, int L, int D) {
  const int64_t N = cdiv(L, 64);
  ComplWs w;
  size_t off = 0;
  w.hblk = off; off += align_up((int64_t)BH * N * D * D * 2, 256);
  w.zblk = off; off += align_up((int64_t)BH * N * D * 4, 256);
  w.ngroup = cdiv((int)N, TOTAL_GROUP);
  w.hgrp = off; off += align_up((int64_t)BH * w.ngroup * D * D * 4, 256);
  w.zgrp = off; off += align_up((int64_t)BH * w.ngroup * D * 4, 256);
  w.hall = off; off += align_up((int64_t)BH * D * D * 4, 256);
  w.zall = off; off += align_up((int64_t)BH * D * 4, 256);
  w.total = off;
  return w;
}
int64_t linear_complement_workspace_bytes(int BH, int L, int D) { return (int64_t)compl_ws(BH, L, D).total; }

template <typename Tag, int D, int BLKQ>
static int complement_impl(const void* q, const void* k, const void* v, const void* lut, int lut64, const float* weight,
                           const float* bias, const void* residual, void* out, int fmap, int BH, int L, int topk, char* ws,
                           hipStream_t st) {
  const ComplWs w = compl_ws(BH, L, D);
  const int N = cdiv(L, 64), Mblk = cdiv(L, BLKQ);
  uint16_t* hblk = (uint16_t*)(ws + w.hblk);
  float* zblk = (float*)(ws + w.zblk);
  float* hall = (float*)(ws + w.hall);
  float* zall = (float*)(ws + w.zall);
  hipLaunchKernelGGL((linear_state_partial_kernel<Tag, D, true>), dim3(N, BH), dim3(256), 0, st, (const uint16_t*)k,
                     (const uint16_t*)v, contiguous_layout(BH, L, D), (void*)hblk, zblk, L, 64, fmap);
  float* hgrp = (float*)(ws + w.hgrp);
  float* zgrp = (float*)(ws + w.zgrp);
  hipLaunchKernelGGL((complement_group_kernel<Tag>), dim3(cdiv(D * D / 8, 256), w.ngroup, BH), dim3(256), 0, st, hblk, zblk,
                     hgrp, zgrp, N, D);
  hipLaunchKernelGGL(complement_total_kernel, dim3(cdiv(D * D, 256), BH), dim3(256), 0, st, hgrp, zgrp, hall, zall, w.ngroup,
                     D);
  const int total = BH * cdiv(Mblk, COMPL_RUN);
  hipLaunchKernelGGL((complement_out_kernel<Tag, D, BLKQ>), dim3(xcd_grid(total)), dim3(256), 0, st, (const uint16_t*)q, hblk,
                     zblk, hall, zall, lut, lut64, weight, bias, (const uint16_t*)residual, (uint16_t*)out, L, Mblk, N, topk,
                     fmap, total);
  return check_launch("linear_complement_fwd");
}

// ---- backward, host -------------------------------------------------------------------------
struct ComplBwdWs {
  ComplWs fwd;
  int ngroup_q;
  size_t wt, dn, y, dden, dhblk, dzblk, dgrp, dzgrp, gall, gzall, wg, count, list, total;
};
static ComplBwdWs compl_bwd_ws(int BH, int L, int D, int BLKQ) {
  const int64_t N = cdiv(L, 64), M = cdiv(L, BLKQ);
  ComplBwdWs w;
  w.fwd = compl_ws(BH, L, D);
  w.ngroup_q = cdiv((int)M, TOTAL_GROUP);
  size_t off = w.fwd.total;
  w.wt = off;    off += align_up((int64_t)D * D * 2, 256);
  w.dn = off;    off += align_up((int64_t)BH * L * D * 2, 256);
  w.y = off;     off += align_up((int64_t)BH * L * D * 2, 256);
  w.dden = off;  off += align_up((int64_t)BH * L * 4, 256);
  w.dhblk = off; off += align_up((int64_t)BH * M * D * D * 2, 256);
  w.dzblk = off; off += align_up((int64_t)BH * M * D * 4, 256);
  w.dgrp = off;  off += align_up((int64_t)BH * w.ngroup_q * D * D * 4, 256);
  w.dzgrp = off; off += align_up((int64_t)BH * w.ngroup_q * D * 4, 256);
  w.gall = off;  off += align_up((int64_t)BH * D * D * 4, 256);
  w.gzall = off; off += align_up((int64_t)BH * D * 4, 256);
  w.wg = off;    off += align_up(weight_grads_workspace_bytes(BH, L, D), 256);
  w.count = off; off += align_up((int64_t)BH * N * 4, 256);
  w.list = off;  off += align_up((int64_t)BH * N * M * 4, 256);
  w.total = off;
  return w;
}
int64_t linear_complement_bwd_workspace_bytes(int BH, int L, int D, int BLKQ) {
  return (int64_t)compl_bwd_ws(BH, L, D, BLKQ).total;
}

template <typename Tag, int D, int BLKQ>
static int complement_bwd_impl(const void* q, const void* k, const void* v, const int8_t* sparse_map, const void* lut, int lut64,
                               const float* weight, const void* d_out, void* dq, void* dk, void* dv, float* d_weight,
                               float* d_bias, int dtype, int fmap, int BH, int L, int topk, int accumulate, char* ws,
                               hipStream_t st) {
  const ComplBwdWs w = compl_bwd_ws(BH, L, D, BLKQ);
  const int N = cdiv(L, 64), Mblk = cdiv(L, BLKQ);
  const RowLayout lay = contiguous_layout(BH, L, D);
  uint16_t* hblk = (uint16_t*)(ws + w.fwd.hblk);
  float* zblk = (float*)(ws + w.fwd.zblk);
  float* hall = (float*)(ws + w.fwd.hall);
  float* zall = (float*)(ws + w.fwd.zall);
  uint16_t* wt = (uint16_t*)(ws + w.wt);
  uint16_t* dn = (uint16_t*)(ws + w.dn);
  uint16_t* y = (uint16_t*)(ws + w.y);
  float* dden = (float*)(ws + w.dden);
  uint16_t* dhblk = (uint16_t*)(ws + w.dhblk);
  float* dzblk = (float*)(ws + w.dzblk);
  float* gall = (float*)(ws + w.gall);
  float* gzall = (float*)(ws + w.gzall);
  int* count = (int*)(ws + w.count);
  int* list = (int*)(ws + w.list);
  // the forward's states again: per key block, then their totals
  hipLaunchKernelGGL((linear_state_partial_kernel<Tag, D, true>), dim3(N, BH), dim3(256), 0, st, (const uint16_t*)k,
                     (const uint16_t*)v, lay, (void*)hblk, zblk, L, 64, fmap, (const float*)nullptr);
  hipLaunchKernelGGL((complement_group_kernel<Tag>), dim3(cdiv(D * D / 8, 256), w.fwd.ngroup, BH), dim3(256), 0, st, hblk, zblk,
                     (float*)(ws + w.fwd.hgrp), (float*)(ws + w.fwd.zgrp), N, D);
  hipLaunchKernelGGL(complement_total_kernel, dim3(cdiv(D * D, 256), BH), dim3(256), 0, st, (const float*)(ws + w.fwd.hgrp),
                     (const float*)(ws + w.fwd.zgrp), hall, zall, w.fwd.ngroup, D);
  hipLaunchKernelGGL((linear_prep_weight_kernel<Tag>), dim3(cdiv(D * D, 256)), dim3(256), 0, st, weight, wt, D);
  launch_col_lists(sparse_map, list, count, BH, Mblk, N, st);
  // rows: dq and the row temporaries
  const int total_q = BH * Mblk;
  hipLaunchKernelGGL((complement_bwd_rows_kernel<Tag, D, BLKQ>), dim3(xcd_grid(total_q)), dim3(256), 0, st, (const uint16_t*)q,
                     (const uint16_t*)d_out, hblk, zblk, hall, zall, lut, lut64, wt, (uint16_t*)dq, dn, y, dden, L, Mblk, N, topk,
                     fmap, total_q, accumulate);
  // per query block dH_i^T = (a_i^T dn_i)^T and dz_i = sum dden a (the state kernel with q, dn in the place of k, v),
  // then their totals
  hipLaunchKernelGGL((linear_state_partial_kernel<Tag, D, true, true>), dim3(Mblk, BH), dim3(256), 0, st, (const uint16_t*)q,
                     (const uint16_t*)dn, lay, (void*)dhblk, dzblk, L, BLKQ, fmap, (const float*)dden);
  hipLaunchKernelGGL((complement_group_kernel<Tag>), dim3(cdiv(D * D / 8, 256), w.ngroup_q, BH), dim3(256), 0, st, dhblk, dzblk,
                     (float*)(ws + w.dgrp), (float*)(ws + w.dzgrp), Mblk, D);
  hipLaunchKernelGGL(complement_total_kernel, dim3(cdiv(D * D, 256), BH), dim3(256), 0, st, (const float*)(ws + w.dgrp),
                     (const float*)(ws + w.dzgrp), gall, gzall, w.ngroup_q, D);
  // dW, db
  launch_weight_grads(dtype, D, q, dn, d_out, y, dden, BH, L, fmap, ws + w.wg, d_weight, d_bias, st);
  // dk, dv
  const int total_k = BH * N;
  hipLaunchKernelGGL((complement_bwd_kv_kernel<Tag, D>), dim3(xcd_grid(total_k)), dim3(256), 0, st, (const uint16_t*)k,
                     (const uint16_t*)v, dhblk, dzblk, gall, gzall, list, count, (uint16_t*)dk, (uint16_t*)dv, L, Mblk, N, fmap,
                     total_k, accumulate);
  return check_launch("linear_complement_bwd");
}

}  // namespace sla

using namespace sla;

extern "C" int sla_linear_complement_bwd(const void* q, const void* k, const void* v, const int8_t* sparse_map, const void* lut,
                                         int lut_elem_bytes, const float* weight, const float* bias, const void* d_out, void* dq,
                                         void* dk, void* dv, float* d_weight, float* d_bias, int dtype, int fmap, int B, int H,
                                         int L, int D, int BLKQ, int BLKK, int topk, int flags, void* workspace,
                                         int64_t workspace_bytes, void* stream) {
  int rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  rc = validate_attn_shape(dtype, B, H, L, D, BLKQ, BLKK, topk, lut_elem_bytes);
  if (rc) return rc;
  (void)bias;  // the bias does not enter any gradient
  SLA_REQUIRE((flags & ~SLA_BWD_ACCUMULATE) == 0, SLA_ERR_BAD_ARG, "unknown flag bits in %d", flags);
  SLA_REQUIRE(q && k && v && sparse_map && weight && d_out && dq && dk && dv && d_weight && d_bias && workspace &&
                  (lut || topk == 0),
              SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)d_out | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv |
               (uintptr_t)weight | (uintptr_t)workspace) % 16 == 0,
              SLA_ERR_BAD_ARG, "pointers must be 16-byte aligned");
  SLA_REQUIRE((int64_t)H * B <= 65535, SLA_ERR_UNSUPPORTED, "B*H exceeds 65535");
  const int BH = B * H;
  const int64_t need = linear_complement_bwd_workspace_bytes(BH, L, D, BLKQ);
  SLA_REQUIRE(workspace_bytes >= need, SLA_ERR_WORKSPACE, "workspace of %lld bytes, need %lld", (long long)workspace_bytes,
              (long long)need);
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  const int lut64 = lut_elem_bytes == 8;
  const int accumulate = flags & SLA_BWD_ACCUMULATE;
#define SLA_CPLB_CASE(TAG, DD, BQ)                                                                                      \
  if (D == DD && BLKQ == BQ)                                                                                            \
  return complement_bwd_impl<TAG, DD, BQ>(q, k, v, sparse_map, lut, lut64, weight, d_out, dq, dk, dv, d_weight, d_bias, \
                                          dtype, fmap, BH, L, topk, accumulate, ws, st)
  if (dtype == SLA_BF16) {
    SLA_CPLB_CASE(bf16_tag, 128, 64);
    SLA_CPLB_CASE(bf16_tag, 128, 128);
    SLA_CPLB_CASE(bf16_tag, 64, 64);
    SLA_CPLB_CASE(bf16_tag, 64, 128);
  } else {
    SLA_CPLB_CASE(f16_tag, 128, 64);
    SLA_CPLB_CASE(f16_tag, 128, 128);
    SLA_CPLB_CASE(f16_tag, 64, 64);
    SLA_CPLB_CASE(f16_tag, 64, 128);
  }
#undef SLA_CPLB_CASE
  set_error("unsupported D=%d BLKQ=%d", D, BLKQ);
  return SLA_ERR_UNSUPPORTED;
}

extern "C" int sla_linear_complement_fwd(const void* q, const void* k, const void* v, const void* lut, int lut_elem_bytes,
                                         const float* weight, const float* bias, const void* residual, void* out, int dtype,
                                         int fmap, int B, int H, int L, int D, int BLKQ, int BLKK, int topk, void* workspace,
                                         int64_t workspace_bytes, void* stream) {
  int rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  rc = validate_attn_shape(dtype, B, H, L, D, BLKQ, BLKK, topk, lut_elem_bytes);
  if (rc) return rc;
  SLA_REQUIRE(q && k && v && weight && bias && out && workspace && (lut || topk == 0), SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)residual | (uintptr_t)weight |
               (uintptr_t)workspace) % 16 == 0,
              SLA_ERR_BAD_ARG, "pointers must be 16-byte aligned");
  SLA_REQUIRE((int64_t)H * B <= 65535 && cdiv(L, BLKQ) <= 65535 * 32, SLA_ERR_UNSUPPORTED, "grid too large");
  const int BH = B * H;
  const int64_t need = linear_complement_workspace_bytes(BH, L, D);
  SLA_REQUIRE(workspace_bytes >= need, SLA_ERR_WORKSPACE, "workspace of %lld bytes, need %lld", (long long)workspace_bytes,
              (long long)need);
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  const int lut64 = lut_elem_bytes == 8;
#define SLA_CPL_CASE(TAG, DD, BQ) \
  if (D == DD && BLKQ == BQ)      \
  return complement_impl<TAG, DD, BQ>(q, k, v, lut, lut64, weight, bias, residual, out, fmap, BH, L, topk, ws, st)
  if (dtype == SLA_BF16) {
    SLA_CPL_CASE(bf16_tag, 128, 64);
    SLA_CPL_CASE(bf16_tag, 128, 128);
    SLA_CPL_CASE(bf16_tag, 64, 64);
    SLA_CPL_CASE(bf16_tag, 64, 128);
  } else {
    SLA_CPL_CASE(f16_tag, 128, 64);
    SLA_CPL_CASE(f16_tag, 128, 128);
    SLA_CPL_CASE(f16_tag, 64, 64);
    SLA_CPL_CASE(f16_tag, 64, 128);
  }
#undef SLA_CPL_CASE
  set_error("unsupported D=%d BLKQ=%d", D, BLKQ);
  return SLA_ERR_UNSUPPORTED;
}
