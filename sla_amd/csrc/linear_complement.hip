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

// 1-D grid over (head, query block) with the XCD-aware remap of the attention kernels: neighbouring query
// blocks select mostly the same key blocks, so their state reads hit the same XCD's L2.  256 threads.
template <typename Tag, int D, int BLKQ>
__global__ __launch_bounds__(256) void complement_out_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ hblk,
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

  // ---- H_i = total - selected, fp32, then 16 bit into LDS ----
  {
    float acc[NCH][8];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int idx = (tid + 256 * c) * 8;
      const f32x4_t a = *reinterpret_cast<const f32x4_t*>(hall + (size_t)bh * DD + idx);
      const f32x4_t b = *reinterpret_cast<const f32x4_t*>(hall + (size_t)bh * DD + idx + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[c][e] = a[e];
        acc[c][4 + e] = b[e];
      }
    }
    float zacc = tid < D ? zall[(size_t)bh * D + tid] : 0.f;
    const uint16_t* hb = hblk + (size_t)bh * N * DD;
    // two selected states are in flight while a third is being subtracted (the gather is latency-bound:
    // bytes in flight per compute unit set its rate)
    i16x8_t ring[2][NCH];
    float zring[2] = {0.f, 0.f};
    auto fetch = [&](int slot, int i) {
      const int nb = lut_at(i);
      const uint16_t* p = hb + (size_t)nb * DD;
#pragma unroll
      for (int c = 0; c < NCH; ++c) ring[slot][c] = *reinterpret_cast<const i16x8_t*>(p + (tid + 256 * c) * 8);
      zring[slot] = tid < D ? zblk[((size_t)bh * N + nb) * D + tid] : 0.f;
    };
    auto consume = [&](int slot) {
#pragma unroll
      for (int c = 0; c < NCH; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[c][e] -= E::to_float((uint16_t)ring[slot][c][e]);
      zacc -= zring[slot];
    };
    if (topk > 0) fetch(0, 0);
    if (topk > 1) fetch(1, 1);
    int it = 0;
    for (; it + 1 < topk; it += 2) {       // slot parity is static inside the unrolled pair
      i16x8_t x[NCH];
#pragma unroll
      for (int c = 0; c < NCH; ++c) x[c] = ring[0][c];
      const float zx = zring[0];
      if (it + 2 < topk) fetch(0, it + 2);
#pragma unroll
      for (int c = 0; c < NCH; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[c][e] -= E::to_float((uint16_t)x[c][e]);
      zacc -= zx;
#pragma unroll
      for (int c = 0; c < NCH; ++c) x[c] = ring[1][c];
      const float zy = zring[1];
      if (it + 3 < topk) fetch(1, it + 3);
#pragma unroll
      for (int c = 0; c < NCH; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[c][e] -= E::to_float((uint16_t)x[c][e]);
      zacc -= zy;
    }
    if (it < topk) consume(0);
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int idx = (tid + 256 * c) * 8;
      const int row = idx / D, col = idx % D;
      i32x4_t w;
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = (int)E::pack2(acc[c][2 * e], acc[c][2 * e + 1]);
      *reinterpret_cast<i32x4_t*>(&sH[row * STR + col]) = w;
    }
    // projection weight, 16 bit, columns in accumulator slot order
    for (int idx = tid; idx < DD; idx += 256) {
      const int e = idx / D, d = idx % D;
      sW[e * STR + slot_order_pos(d)] = E::from_float(weight[idx]);
    }
    if (tid < D) {
      sZ[tid] = round16<Tag>(zacc);
      sBias[tid] = round16<Tag>(bias[tid]);
    }
  }
  __syncthreads();
  if (wave >= BLKQ / 32) return;

  // ---- this wave's 32 queries ----
  const int qrow = mb * BLKQ + wave * 32 + r;
  const bool ok = qrow < L;
  const size_t off = ((size_t)bh * L + qrow) * D;
  float f[DC][8];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    i16x8_t x = {0, 0, 0, 0, 0, 0, 0, 0};
    if (ok) x = *reinterpret_cast<const i16x8_t*>(q + off + 16 * c + 8 * g);
#pragma unroll
    for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)x[j]);
  }
  float row_mx, row_inv;
  phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
  float den = 0.f;
  i16x8_t qf[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    i32x4_t pw;
#pragma unroll
    for (int j = 0; j < 8; ++j) den += round16<Tag>(f[c][j] * sZ[16 * c + 8 * g + j]);
#pragma unroll
    for (int j = 0; j < 4; ++j) pw[j] = (int)E::pack2(f[c][2 * j], f[c][2 * j + 1]);
    qf[c] = __builtin_bit_cast(i16x8_t, pw);
  }
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
  const int total = BH * Mblk;
  hipLaunchKernelGGL((complement_out_kernel<Tag, D, BLKQ>), dim3(xcd_grid(total)), dim3(256), 0, st, (const uint16_t*)q, hblk,
                     zblk, hall, zall, lut, lut64, weight, bias, (const uint16_t*)residual, (uint16_t*)out, L, Mblk, N, topk,
                     fmap, total);
  return check_launch("linear_complement_fwd");
}

}  // namespace sla

using namespace sla;

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
