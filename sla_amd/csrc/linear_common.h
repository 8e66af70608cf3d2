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
