// Block-sparse FlashAttention forward for gfx950 (bf16 / f16 MFMA, fp32 softmax).
//
// Stands in for _attn_fwd and _attention.forward of the reference
// (sparse_linear_attention/kernel.py:21-82, 242-274).
//
// One workgroup owns one query block (BLKQ rows); every wavefront owns 32 of its rows.
// The product is formed transposed: S^T = K Q^T with the 32x32x16 MFMA, so that in the
// accumulator layout a lane holds ONE query column and 16 key rows.  Row maxima and sums
// are then per-lane loops plus one exchange with lane^32, and the probabilities, once
// packed to 16 bit, already sit in the B-operand layout of the second product
// O^T = V^T P^T.  V^T fragments come out of LDS with the transposing 64-bit read.
// K/V tiles go global -> registers -> LDS; the next tile's global loads are in flight
// while the current tile is multiplied.
#include "common.h"

namespace sla {

template <typename Tag, int D, int BLKQ>
__global__ __launch_bounds__(BLKQ * 2) void sparse_fwd_kernel(const uint16_t* __restrict__ q,
                                                              const uint16_t* __restrict__ k,
                                                              const uint16_t* __restrict__ v,
                                                              const void* __restrict__ lut, int lut64,
                                                              uint16_t* __restrict__ o, float* __restrict__ lse, int L,
                                                              int Mblk, int topk, float scale_log2e, int total) {
  using E = Elem<Tag>;
  constexpr int BLKK = 64;
  constexpr int NT = BLKQ * 2;              // threads
  constexpr int DC = D / 16;                // 16-wide chunks of the head dim (QK^T contraction)
  constexpr int DT = D / 32;                // 32-row tiles of O^T
  constexpr int KSTR = D + 8;               // LDS row stride of K (elements): 16 B pad, conflict-free b128 reads
  constexpr int VSTR = D + 16;              // LDS row stride of V: 32 B pad, conflict-free transposed reads
  constexpr int CPR = D / 8;                // 16-byte chunks per row
  constexpr int NLD = BLKK * CPR / NT;      // 16-byte chunks each thread moves per tile
  static_assert(BLKK * CPR % NT == 0, "tile does not divide among the threads");

  __shared__ __attribute__((aligned(16))) uint16_t sK[BLKK * KSTR];
  __shared__ __attribute__((aligned(16))) uint16_t sV[BLKK * VSTR];

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int bh = logical / Mblk;
  const int mb = logical - bh * Mblk;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5;                  // which half of the MFMA contraction slots this lane feeds
  const int r = lane & 31;                  // query column (S^T, O^T) / key row (A operand)

  const size_t head_off = (size_t)bh * L * D;
  const uint16_t* qh = q + head_off;
  const uint16_t* kh = k + head_off;
  const uint16_t* vh = v + head_off;

  // Q^T fragments (B operand), resident for the whole loop.
  const int qrow = mb * BLKQ + wave * 32 + r;
  i16x8_t qf[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    if (qrow < L)
      qf[c] = *reinterpret_cast<const i16x8_t*>(qh + (size_t)qrow * D + 16 * c + 8 * g);
    else
      qf[c] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
  }

  const size_t lut_row = ((size_t)bh * Mblk + mb) * topk;
  auto lut_at = [&](int i) -> int {
    return lut64 ? (int)reinterpret_cast<const long long*>(lut)[lut_row + i]
                 : reinterpret_cast<const int*>(lut)[lut_row + i];
  };

  i16x8_t kreg[NLD], vreg[NLD];
  auto load_tile = [&](int nb) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int idx = tid + i * NT;
      const int row = idx / CPR, col = (idx % CPR) * 8;
      const int grow = nb * BLKK + row;
      if (grow < L) {
        kreg[i] = *reinterpret_cast<const i16x8_t*>(kh + (size_t)grow * D + col);
        vreg[i] = *reinterpret_cast<const i16x8_t*>(vh + (size_t)grow * D + col);
      } else {
        kreg[i] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
        vreg[i] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int idx = tid + i * NT;
      const int row = idx / CPR, col = (idx % CPR) * 8;
      *reinterpret_cast<i16x8_t*>(&sK[row * KSTR + col]) = kreg[i];
      *reinterpret_cast<i16x8_t*>(&sV[row * VSTR + col]) = vreg[i];
    }
  };

  f32x16_t oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;
  float m_run = -INFINITY;   // running maximum of the scaled scores of this lane's query
  float l_run = 0.f;         // this lane's share of the running sum (its 32 of the 64 key rows)

  // transposed-read addressing of V: lane i of a 16-lane group points at row i/4, cols 4*(i%4)
  const int tr_row = (lane & 15) >> 2;
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  int nb = topk > 0 ? lut_at(0) : 0;
  if (topk > 0) load_tile(nb);

  for (int it = 0; it < topk; ++it) {
    __syncthreads();                       // previous tile fully consumed
    store_tile();
    __syncthreads();
    const int kv_valid = L - nb * BLKK;    // rows of this tile that exist
    if (it + 1 < topk) {
      nb = lut_at(it + 1);
      load_tile(nb);                       // in flight during the math below
    }

    // ---- S^T = K Q^T : two 32-key sub-tiles ----
    f32x16_t s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[t][i] = 0.f;
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const i16x8_t a = *reinterpret_cast<const i16x8_t*>(&sK[(32 * t + r) * KSTR + 16 * c + 8 * g]);
        s[t] = E::mfma32(a, qf[c], s[t]);
      }
    }
    if (kv_valid < BLKK) {                 // partial last key block: rows past L never take part
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = 32 * t + 8 * (i >> 2) + 4 * g + (i & 3);
          if (key >= kv_valid) s[t][i] = -INFINITY;
        }
    }

    // ---- online softmax (base 2) ----
    float mx = s[0][0];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[t][i]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx * scale_log2e);
    const float alpha = fast_exp2(m_run - m_new);
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float p = fast_exp2(__builtin_fmaf(s[t][i], scale_log2e, -m_new));
        s[t][i] = p;
        psum += p;
      }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
    }

    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        i32x4_t pw;
#pragma unroll
        for (int j = 0; j < 4; ++j) pw[j] = (int)E::pack2(s[t][8 * c2 + 2 * j], s[t][8 * c2 + 2 * j + 1]);
        const i16x8_t pb = __builtin_bit_cast(i16x8_t, pw);
        const int key0 = 32 * t + 16 * c2 + 4 * g + tr_row;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const uint16_t* p0 = &sV[key0 * VSTR + 32 * dt + tr_col];
          const i16x4_t lo = lds_read_tr16(p0);
          const i16x4_t hi = lds_read_tr16(p0 + 8 * VSTR);
          oacc[dt] = E::mfma32(concat4(lo, hi), pb, oacc[dt]);
        }
      }
  }

  // ---- epilogue ----
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
  if (qrow < L) {
    uint16_t* orow = o + head_off + (size_t)qrow * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        i32x2_t w;
        w[0] = (int)E::pack2(oacc[dt][4 * i4 + 0] * inv, oacc[dt][4 * i4 + 1] * inv);
        w[1] = (int)E::pack2(oacc[dt][4 * i4 + 2] * inv, oacc[dt][4 * i4 + 3] * inv);
        *reinterpret_cast<i32x2_t*>(orow + 32 * dt + 8 * i4 + 4 * g) = w;
      }
    if (g == 0) lse[(size_t)bh * L + qrow] = m_run + fast_log2(l_tot);
  }
}

template <typename Tag>
static int launch_fwd(const void* q, const void* k, const void* v, const void* lut, int lut64, void* o, float* lse, int BH,
                      int L, int D, int BLKQ, int topk, float qk_scale, hipStream_t st) {
  const int Mblk = cdiv(L, BLKQ);
  const int64_t total64 = (int64_t)BH * Mblk;
  const int total = (int)total64;
  const int grid = xcd_grid(total);
  const float c = qk_scale * 1.4426950408889634f;
#define SLA_FWD_CASE(DD, BQ)                                                                                         \
  if (D == DD && BLKQ == BQ) {                                                                                       \
    hipLaunchKernelGGL((sparse_fwd_kernel<Tag, DD, BQ>), dim3(grid), dim3(BQ * 2), 0, st, (const uint16_t*)q,       \
                       (const uint16_t*)k, (const uint16_t*)v, lut, lut64, (uint16_t*)o, lse, L, Mblk, topk, c, total); \
    return check_launch("sparse_attn_fwd");                                                                          \
  }
  SLA_FWD_CASE(128, 64)
  SLA_FWD_CASE(128, 128)
  SLA_FWD_CASE(64, 64)
  SLA_FWD_CASE(64, 128)
#undef SLA_FWD_CASE
  set_error("unsupported D=%d BLKQ=%d", D, BLKQ);
  return SLA_ERR_UNSUPPORTED;
}

int validate_attn_shape(int dtype, int B, int H, int L, int D, int BLKQ, int BLKK, int topk, int lut_elem_bytes) {
  SLA_REQUIRE(B > 0 && H > 0 && L > 0, SLA_ERR_BAD_ARG, "non-positive size (B=%d H=%d L=%d)", B, H, L);
  SLA_REQUIRE(dtype == SLA_BF16 || dtype == SLA_F16, SLA_ERR_UNSUPPORTED, "attention kernels take bf16 or f16, got dtype %d",
              dtype);
  SLA_REQUIRE(BLKQ == 64 || BLKQ == 128, SLA_ERR_UNSUPPORTED, "BLOCK_M must be 64 or 128, got %d", BLKQ);
  SLA_REQUIRE(BLKK == 64, SLA_ERR_UNSUPPORTED, "BLOCK_N must be 64, got %d", BLKK);
  SLA_REQUIRE(D == 64 || D == 128, SLA_ERR_UNSUPPORTED, "head dim must be 64 or 128, got %d", D);
  const int N = cdiv(L, BLKK);
  SLA_REQUIRE(topk >= 0 && topk <= N, SLA_ERR_BAD_ARG, "topk=%d outside [0, %d]", topk, N);
  SLA_REQUIRE(lut_elem_bytes == 4 || lut_elem_bytes == 8, SLA_ERR_BAD_ARG, "lut_elem_bytes must be 4 or 8, got %d",
              lut_elem_bytes);
  SLA_REQUIRE((int64_t)B * H * cdiv(L, 64) < (1ll << 31) - 8, SLA_ERR_UNSUPPORTED, "too many blocks");
  return SLA_OK;
}

}  // namespace sla

using namespace sla;

extern "C" int sla_sparse_attn_fwd(const void* q, const void* k, const void* v, const void* lut, int lut_elem_bytes,
                                   void* o, float* lse, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK,
                                   int topk, float qk_scale, void* stream) {
  int rc = validate_attn_shape(dtype, B, H, L, D, BLKQ, BLKK, topk, lut_elem_bytes);
  if (rc) return rc;
  SLA_REQUIRE(q && k && v && o && lse && (lut || topk == 0), SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) % 16 == 0, SLA_ERR_BAD_ARG,
              "q, k, v, o must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const int BH = B * H;
  if (dtype == SLA_BF16)
    return launch_fwd<bf16_tag>(q, k, v, lut, lut_elem_bytes == 8, o, lse, BH, L, D, BLKQ, topk, qk_scale, st);
  return launch_fwd<f16_tag>(q, k, v, lut, lut_elem_bytes == 8, o, lse, BH, L, D, BLKQ, topk, qk_scale, st);
}
