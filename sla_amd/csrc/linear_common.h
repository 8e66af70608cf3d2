// Feature-map helpers shared by the linear-branch kernels (reference core.py:43-57).
#pragma once
#include "common.h"

namespace sla {

template <typename Tag>
static __device__ __forceinline__ float round16(float x) {
  return Elem<Tag>::to_float(Elem<Tag>::from_float(x));
}

// Two values rounded to 16 bit with one packing conversion; returns the packed pair (a in the low half).
template <typename Tag>
static __device__ __forceinline__ uint32_t round16_pair(float a, float b, float& ra, float& rb) {
  const uint32_t p = Elem<Tag>::pack2(a, b);
  ra = Elem<Tag>::to_float((uint16_t)(p & 0xffffu));
  rb = Elem<Tag>::to_float((uint16_t)(p >> 16));
  return p;
}

// relu(x) or elu(x)+1, rounded to 16 bit where the reference materialises a 16-bit tensor
// (elu: once after elu and again after the +1).
template <typename Tag>
static __device__ __forceinline__ float fmap_pointwise(int fmap, float x) {
  if (fmap == SLA_FMAP_RELU) return fmaxf(x, 0.f);
  const float e = x > 0.f ? x : (__expf(x) - 1.0f);
  return round16<Tag>(round16<Tag>(e) + 1.0f);
}

// phi over one row whose D values are split between lane (f: DC chunks of 8) and lane^32.
// For softmax, `mx` and `inv` return the row maximum and 1/sum so the row can be rebuilt later.
template <typename Tag, int DC>
static __device__ __forceinline__ void phi_row_pair(int fmap, float (&f)[DC][8], float& mx, float& inv) {
  mx = 0.f;
  inv = 1.f;
  if (fmap == SLA_FMAP_SOFTMAX) {
    mx = f[0][0];
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) mx = fmaxf(mx, f[c][j]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        f[c][j] = __expf(f[c][j] - mx);
        sum += f[c][j];
      }
    sum += __shfl_xor(sum, 32);
    inv = 1.0f / sum;
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = round16<Tag>(f[c][j] * inv);
  } else if (fmap == SLA_FMAP_RELU) {
    // (the choice of the map stays outside the loops over the elements: inside, every element's map would sit
    //  behind a branch of its own)
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = fmap_pointwise<Tag>(SLA_FMAP_RELU, f[c][j]);
  } else {
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = fmap_pointwise<Tag>(SLA_FMAP_ELU, f[c][j]);
  }
}

// phi of a row whose raw 16-bit values are split between lane (xq: DC chunks of 8) and lane^32, packed to 16 bit in `qf`
// (a packed pair is a register of an MFMA B operand), and this lane's part of the divisor's sum,
// sum_d round16(phi_d * z_d), z_d = zat(c, j) for element j of chunk c.  Values the reference rounds to 16 bit are rounded
// two at a time (one packing conversion for two) and taken apart again where the arithmetic goes on in fp32; the sum runs
// over the elements in ascending order.  The pointwise maps never hold the row as 64 floats.
template <typename Tag, int DC, typename ZAt>
static __device__ __forceinline__ float phi_pack_den(int fmap, const i16x8_t (&xq)[DC], i16x8_t (&qf)[DC], ZAt zat) {
  using E = Elem<Tag>;
  float den = 0.f;
  auto pair_done = [&](int c, int j2, float v0, float v1, i32x4_t& pw) __attribute__((always_inline)) {
    float g0, g1, p0, p1;
    pw[j2] = (int)round16_pair<Tag>(v0, v1, g0, g1);
    round16_pair<Tag>(g0 * zat(c, 2 * j2), g1 * zat(c, 2 * j2 + 1), p0, p1);
    den += p0;
    den += p1;
  };
  if (fmap == SLA_FMAP_SOFTMAX) {
    float f[DC][8];
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)xq[c][j]);
    float row_mx, row_inv;
    phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i32x4_t pw;
#pragma unroll
      for (int j2 = 0; j2 < 4; ++j2) pair_done(c, j2, f[c][2 * j2], f[c][2 * j2 + 1], pw);
      qf[c] = __builtin_bit_cast(i16x8_t, pw);
    }
  } else if (fmap == SLA_FMAP_RELU) {
    // (the choice of the map stays outside the loops over the elements)
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i32x4_t pw;
#pragma unroll
      for (int j2 = 0; j2 < 4; ++j2) {
        const uint32_t xx = (uint32_t)__builtin_bit_cast(i32x4_t, xq[c])[j2];
        pair_done(c, j2, fmaxf(E::to_float((uint16_t)(xx & 0xffffu)), 0.f), fmaxf(E::to_float((uint16_t)(xx >> 16)), 0.f), pw);
      }
      qf[c] = __builtin_bit_cast(i16x8_t, pw);
    }
  } else {
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i32x4_t pw;
#pragma unroll
      for (int j2 = 0; j2 < 4; ++j2) {
        const uint32_t xx = (uint32_t)__builtin_bit_cast(i32x4_t, xq[c])[j2];
        const float x0 = E::to_float((uint16_t)(xx & 0xffffu)), x1 = E::to_float((uint16_t)(xx >> 16));
        float e0, e1;                                    // elu, rounded; then + 1, rounded by pair_done
        round16_pair<Tag>(x0 > 0.f ? x0 : (__expf(x0) - 1.0f), x1 > 0.f ? x1 : (__expf(x1) - 1.0f), e0, e1);
        pair_done(c, j2, e0 + 1.0f, e1 + 1.0f, pw);
      }
      qf[c] = __builtin_bit_cast(i16x8_t, pw);
    }
  }
  return den;
}

// Gradient through phi for one row held in accumulator layout: `x` raw inputs, `gr` the gradient
// w.r.t. phi(x), both DT tiles of 16 values (this lane's half of the row; lane^32 has the rest).
template <int DT>
static __device__ __forceinline__ void phi_backward(int fmap, const float (&x)[DT][16], float (&gr)[DT][16], float mx,
                                                    float inv) {
  if (fmap == SLA_FMAP_RELU) {
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) gr[t][i] = x[t][i] > 0.f ? gr[t][i] : 0.f;
  } else if (fmap == SLA_FMAP_ELU) {
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) gr[t][i] = x[t][i] > 0.f ? gr[t][i] : gr[t][i] * __expf(x[t][i]);
  } else {
    float a[DT][16];
    float dot = 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        a[t][i] = __expf(x[t][i] - mx) * inv;
        dot += a[t][i] * gr[t][i];
      }
    dot += __shfl_xor(dot, 32);
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) gr[t][i] = a[t][i] * (gr[t][i] - dot);
  }
}

// Split of L among workgroups for the streaming state kernels.
struct LinSplit {
  int nsplit, rows_per_split;
};
// Slices of the sequence for the kernels that reduce over L: as many (head, slice) workgroups as fit the chip at
// once (`slots` = 256 compute units x workgroups per unit), never more, so there is no second, part-filled round.
// Slices are multiples of `gran` rows (the rows a kernel takes per step).
static inline LinSplit lin_split(int BH, int L, int slots = 768, int gran = 64) {
  int nsplit = slots / BH;
  const int max_split = cdiv(L, gran);
  if (nsplit > max_split) nsplit = max_split;
  if (nsplit < 1) nsplit = 1;
  LinSplit s;
  s.rows_per_split = cdiv(cdiv(L, nsplit), gran) * gran;
  s.nsplit = cdiv(L, s.rows_per_split);
  return s;
}

// Row-tile kernels: a workgroup stages per-head matrices once and then walks `tiles` steps of its head.
// With T steps per head, BH heads and room for wg_per_cu workgroups on each of the 256 compute units,
// pick `tiles` so that all workgroups are resident at once and carry near-equal work.
static inline int balanced_tiles(int T, int BH, int wg_per_cu) {
  const int slots = 256 * wg_per_cu;
  if (BH >= slots) return T < 8 ? T : 8;
  const int per_head = slots / BH;
  return cdiv(T, per_head);
}

int validate_linear(int dtype, int fmap, int B, int H, int L, int D);

}  // namespace sla
