// Backward of the linear-attention branch + projection for gfx950.
//
// Stands in for torch autograd through sparse_linear_attention/core.py:90-99 of the reference.
// With a = phi(q), c = phi(k), S = c^T v, z = sum c, n = a S, den = 1e-5 + a.z, y = n/den,
// out = y W^T + b and G = d(out):
//   db = sum G ; dW = G^T y ; dy = G W ; dn = dy/den ; dden = -sum_d(dy*y)/den
//   da = dn S^T + dden z ; dS = a^T dn ; dz = sum_l dden a
//   dc = v dS^T + dz ; dv = c dS ; dq = phi'(q) da ; dk = phi'(k) dc
//
// Kernels:
//   state build (shared with the forward) : S and z again from k, v
//   rows   : per 32 queries on one wave: y^T, dy^T, dn^T, da^T on the MFMA in transposed form (per-query
//            scalars stay per-lane), writes dq and the row-wise temporaries dn, y (16 bit) and dden
//   states : streams q, dn, G, y once; dS and dW on the MFMA (operands read transposed from LDS),
//            dz and db on the vector ALU; fp32 partials
//   reduce : fixed-order sums of the partials -> dS (16 bit, both orientations), dz, per-head dW, db;
//            a second small kernel adds the heads
//   kv     : per 32 keys on one wave: dc^T = dS v^T + dz, dv^T = dS^T c^T, dk = phi'(k) dc
#include "linear_state.h"

namespace sla {

// ---- rows ---------------------------------------------------------------------------------
template <typename Tag, int D>
__global__ __launch_bounds__(256) void linear_bwd_rows_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ gout, const uint16_t* __restrict__ kvt,
    const uint16_t* __restrict__ z, const float* __restrict__ weight, uint16_t* __restrict__ dq, uint16_t* __restrict__ dn_out,
    uint16_t* __restrict__ y_out, float* __restrict__ dden_out, int L, int fmap, int tiles_per_wg, int accumulate) {
  using E = Elem<Tag>;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int STR = D + 8;
  __shared__ __attribute__((aligned(16))) uint16_t sKVT[D * STR];  // [d2][d1]          A of n^T = KVT a^T
  __shared__ __attribute__((aligned(16))) uint16_t sKVP[D * STR];  // [d1][perm d2]     A of da^T = S dn^T
  __shared__ __attribute__((aligned(16))) uint16_t sWT[D * STR];   // [d][e]            A of dy^T = W^T G^T
  __shared__ __attribute__((aligned(16))) float sZ[D];

  const int bh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;

  {
    const uint16_t* src = kvt + (size_t)bh * D * D;
    for (int idx = tid; idx < D * D / 8; idx += 256) {
      const int row = idx / (D / 8), col = (idx % (D / 8)) * 8;
      *reinterpret_cast<i16x8_t*>(&sKVT[row * STR + col]) = *reinterpret_cast<const i16x8_t*>(src + (size_t)row * D + col);
    }
    // S[d1][d2] = KVT[d2][d1], columns re-ordered to the accumulator slot order:
    // slot j of chunk c, lane group gg  <->  d2 = 16c + 8*(j/4) + 4gg + j%4
    for (int idx = tid; idx < D * D; idx += 256) {
      const int d2 = idx / D, d1 = idx % D;
      const int c = d2 >> 4, w16 = d2 & 15;
      const int gg = (w16 >> 2) & 1, j = ((w16 >> 3) << 2) | (w16 & 3);
      sKVP[d1 * STR + 16 * c + 8 * gg + j] = src[idx];
    }
    for (int idx = tid; idx < D * D; idx += 256) {
      const int e = idx / D, d = idx % D;
      sWT[d * STR + e] = E::from_float(weight[idx]);
    }
    if (tid < D) sZ[tid] = E::to_float(z[(size_t)bh * D + tid]);
  }
  __syncthreads();

  const size_t head_off = (size_t)bh * L * D;
  for (int tt = 0; tt < tiles_per_wg; ++tt) {
    const int row0 = (blockIdx.x * tiles_per_wg + tt) * 128 + wave * 32;
    if (row0 >= L) break;
    const int qrow = row0 + r;
    const bool ok = qrow < L;
    const size_t roff = head_off + (size_t)qrow * D;

    float f[DC][8];
    i16x8_t gf[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i16x8_t x = {0, 0, 0, 0, 0, 0, 0, 0};
      gf[c] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
      if (ok) {
        x = *reinterpret_cast<const i16x8_t*>(q + roff + 16 * c + 8 * g);
        gf[c] = *reinterpret_cast<const i16x8_t*>(gout + roff + 16 * c + 8 * g);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)x[j]);
    }
    float row_mx, row_inv;
    phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
    float den = 0.f;
    i16x8_t af[DC];
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
    const float inv_den = 1.0f / den;

    // y^T = (KVT a^T) / den ; dy^T = W^T G^T
    f32x16_t yacc[DT], dyacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        yacc[t][i] = 0.f;
        dyacc[t][i] = 0.f;
      }
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const i16x8_t a1 = *reinterpret_cast<const i16x8_t*>(&sKVT[(32 * t + r) * STR + 16 * c + 8 * g]);
        yacc[t] = E::mfma32(a1, af[c], yacc[t]);
        const i16x8_t a2 = *reinterpret_cast<const i16x8_t*>(&sWT[(32 * t + r) * STR + 16 * c + 8 * g]);
        dyacc[t] = E::mfma32(a2, gf[c], dyacc[t]);
      }
    }
    float dden = 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        yacc[t][i] *= inv_den;
        dden += dyacc[t][i] * yacc[t][i];
        dyacc[t][i] *= inv_den;          // dn^T
      }
    dden += __shfl_xor(dden, 32);
    dden = -dden * inv_den;

    // dn^T as B operand; dn and y to memory for the state kernel
    i16x8_t dnf[DT][2];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        i32x4_t pw, yw;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          pw[j] = (int)E::pack2(dyacc[t][8 * c2 + 2 * j], dyacc[t][8 * c2 + 2 * j + 1]);
          yw[j] = (int)E::pack2(yacc[t][8 * c2 + 2 * j], yacc[t][8 * c2 + 2 * j + 1]);
        }
        dnf[t][c2] = __builtin_bit_cast(i16x8_t, pw);
        if (ok) {
          // registers 8c2..8c2+3 are d = 32t+16c2+4g.., registers 8c2+4..+7 are d = 32t+16c2+8+4g..
          const int d0 = 32 * t + 16 * c2 + 4 * g;
          *reinterpret_cast<i32x2_t*>(dn_out + roff + d0) = i32x2_t{pw[0], pw[1]};
          *reinterpret_cast<i32x2_t*>(dn_out + roff + d0 + 8) = i32x2_t{pw[2], pw[3]};
          *reinterpret_cast<i32x2_t*>(y_out + roff + d0) = i32x2_t{yw[0], yw[1]};
          *reinterpret_cast<i32x2_t*>(y_out + roff + d0 + 8) = i32x2_t{yw[2], yw[3]};
        }
      }
    if (ok && g == 0) dden_out[(size_t)bh * L + qrow] = dden;

    // da^T = S dn^T + z dden
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
          const i16x8_t a = *reinterpret_cast<const i16x8_t*>(&sKVP[(32 * t1 + r) * STR + 16 * (2 * t + c2) + 8 * g]);
          acc = E::mfma32(a, dnf[t][c2], acc);
        }
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = 32 * t1 + 8 * i4 + 4 * g;
        i32x2_t xv = {0, 0};
        if (ok) xv = *reinterpret_cast<const i32x2_t*>(q + roff + d0);
        const uint16_t* xp = reinterpret_cast<const uint16_t*>(&xv);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          da[t1][4 * i4 + j] = acc[4 * i4 + j] + sZ[d0 + j] * dden;
          xq[t1][4 * i4 + j] = E::to_float(xp[j]);
        }
      }
    }
    phi_backward<DT>(fmap, xq, da, row_mx, row_inv);
    if (ok) {
#pragma unroll
      for (int t1 = 0; t1 < DT; ++t1)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          uint16_t* dst = dq + roff + 32 * t1 + 8 * i4 + 4 * g;
          if (accumulate) {
            const i32x2_t old = *reinterpret_cast<const i32x2_t*>(dst);
            const uint16_t* op = reinterpret_cast<const uint16_t*>(&old);
#pragma unroll
            for (int j = 0; j < 4; ++j) da[t1][4 * i4 + j] += E::to_float(op[j]);
          }
          i32x2_t w;
          w[0] = (int)E::pack2(da[t1][4 * i4 + 0], da[t1][4 * i4 + 1]);
          w[1] = (int)E::pack2(da[t1][4 * i4 + 2], da[t1][4 * i4 + 3]);
          *reinterpret_cast<i32x2_t*>(dst) = w;
        }
    }
  }
}

// ---- states -------------------------------------------------------------------------------
// grid (nsplit, BH).  dS^T partial [d2][d1] per (bh, split); dW^T partial [d][e] per (bh, split).
template <typename Tag, int D>
__global__ __launch_bounds__(256) void linear_bwd_states_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ dn, const uint16_t* __restrict__ gout,
    const uint16_t* __restrict__ y, const float* __restrict__ dden, float* __restrict__ ds_part, float* __restrict__ dw_part,
    float* __restrict__ dz_part, float* __restrict__ db_part, int L, int rows_per_split, int fmap) {
  using E = Elem<Tag>;
  constexpr int TR = 64;
  constexpr int STR = D + 16;
  constexpr int CPR = D / 8;
  constexpr int RPP = 256 / CPR;
  constexpr int NP = TR / RPP;
  constexpr int DT = D / 32;
  constexpr int WPT = (DT * DT) / 4;

  __shared__ __attribute__((aligned(16))) uint16_t sA[TR * STR];
  __shared__ __attribute__((aligned(16))) uint16_t sDN[TR * STR];
  __shared__ __attribute__((aligned(16))) uint16_t sG[TR * STR];
  __shared__ __attribute__((aligned(16))) uint16_t sY[TR * STR];
  __shared__ float sRed[2][RPP][D];

  const int split = blockIdx.x, bh = blockIdx.y, nsplit = gridDim.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5;
  const int row_begin = split * rows_per_split;
  const int row_end = min(L, row_begin + rows_per_split);
  const size_t head_off = (size_t)bh * L * D;
  const int lrow = tid / CPR, lcol = (tid % CPR) * 8;

  f32x16_t sacc[WPT], wacc[WPT];
#pragma unroll
  for (int t = 0; t < WPT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      sacc[t][i] = 0.f;
      wacc[t][i] = 0.f;
    }
  float zacc[8], bacc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    zacc[e] = 0.f;
    bacc[e] = 0.f;
  }
  const int tr_row = (lane & 15) >> 2;
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  for (int r0 = row_begin; r0 < row_end; r0 += TR) {
    __syncthreads();
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int row = lrow + p * RPP;
      const int grow = r0 + row;
      const bool ok = grow < row_end;
      i16x8_t xq = {0, 0, 0, 0, 0, 0, 0, 0}, xdn = xq, xg = xq, xy = xq;
      float dd = 0.f;
      if (ok) {
        const size_t off = head_off + (size_t)grow * D + lcol;
        xq = *reinterpret_cast<const i16x8_t*>(q + off);
        xdn = *reinterpret_cast<const i16x8_t*>(dn + off);
        xg = *reinterpret_cast<const i16x8_t*>(gout + off);
        xy = *reinterpret_cast<const i16x8_t*>(y + off);
        dd = dden[(size_t)bh * L + grow];
      }
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = E::to_float((uint16_t)xq[e]);
      if (fmap == SLA_FMAP_SOFTMAX) {
        float mx = f[0];
#pragma unroll
        for (int e = 1; e < 8; ++e) mx = fmaxf(mx, f[e]);
#pragma unroll
        for (int s = 1; s < CPR; s <<= 1) mx = fmaxf(mx, __shfl_xor(mx, s));
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          f[e] = __expf(f[e] - mx);
          sum += f[e];
        }
#pragma unroll
        for (int s = 1; s < CPR; s <<= 1) sum += __shfl_xor(sum, s);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = round16<Tag>(f[e] * inv);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = fmap_pointwise<Tag>(fmap, f[e]);
      }
      i16x8_t fa;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (!ok) f[e] = 0.f;
        zacc[e] += dd * f[e];
        bacc[e] += E::to_float((uint16_t)xg[e]);
        fa[e] = (short)E::from_float(f[e]);
      }
      *reinterpret_cast<i16x8_t*>(&sA[row * STR + lcol]) = fa;
      *reinterpret_cast<i16x8_t*>(&sDN[row * STR + lcol]) = xdn;
      *reinterpret_cast<i16x8_t*>(&sG[row * STR + lcol]) = xg;
      *reinterpret_cast<i16x8_t*>(&sY[row * STR + lcol]) = xy;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < TR / 16; ++c) {
      const int l0 = 16 * c + 8 * g + tr_row;
#pragma unroll
      for (int t = 0; t < WPT; ++t) {
        const int tile = wave * WPT + t;
        const int mt = tile / DT, nt = tile % DT;
        const uint16_t* pa = &sA[l0 * STR + 32 * mt + tr_col];
        const uint16_t* pb = &sDN[l0 * STR + 32 * nt + tr_col];
        sacc[t] = E::mfma32(concat4(lds_read_tr16(pa), lds_read_tr16(pa + 4 * STR)),
                            concat4(lds_read_tr16(pb), lds_read_tr16(pb + 4 * STR)), sacc[t]);
        const uint16_t* pg = &sG[l0 * STR + 32 * mt + tr_col];
        const uint16_t* py = &sY[l0 * STR + 32 * nt + tr_col];
        wacc[t] = E::mfma32(concat4(lds_read_tr16(pg), lds_read_tr16(pg + 4 * STR)),
                            concat4(lds_read_tr16(py), lds_read_tr16(py + 4 * STR)), wacc[t]);
      }
    }
  }
  // accumulator: rows = first operand's index (d1 / e), column = second operand's index (d2 / d);
  // stored with the column as the slow axis: part[col][row]
  const size_t pidx = (size_t)bh * nsplit + split;
  float* so = ds_part + pidx * D * D;
  float* wo = dw_part + pidx * D * D;
#pragma unroll
  for (int t = 0; t < WPT; ++t) {
    const int tile = wave * WPT + t;
    const int mt = tile / DT, nt = tile % DT;
    const int col = 32 * nt + (lane & 31);
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const f32x4_t a = {sacc[t][4 * i4], sacc[t][4 * i4 + 1], sacc[t][4 * i4 + 2], sacc[t][4 * i4 + 3]};
      const f32x4_t b = {wacc[t][4 * i4], wacc[t][4 * i4 + 1], wacc[t][4 * i4 + 2], wacc[t][4 * i4 + 3]};
      *reinterpret_cast<f32x4_t*>(so + (size_t)col * D + 32 * mt + 8 * i4 + 4 * g) = a;
      *reinterpret_cast<f32x4_t*>(wo + (size_t)col * D + 32 * mt + 8 * i4 + 4 * g) = b;
    }
  }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    sRed[0][lrow][lcol + e] = zacc[e];
    sRed[1][lrow][lcol + e] = bacc[e];
  }
  __syncthreads();
  if (tid < D) {
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int rr = 0; rr < RPP; ++rr) {
      s0 += sRed[0][rr][tid];
      s1 += sRed[1][rr][tid];
    }
    dz_part[pidx * D + tid] = s0;
    db_part[pidx * D + tid] = s1;
  }
}

// ---- reduce -------------------------------------------------------------------------------
// Stage 1, grid (cdiv(D*D,256), BH): per head, add the split partials in ascending order:
//   dS (16 bit, both orientations), dz, and this head's dW^T / db (fp32).
// Stage 2, grid (cdiv(D*D,256)): add the per-head dW^T / db in ascending head order.
template <typename Tag>
__global__ __launch_bounds__(256) void linear_bwd_reduce_kernel(const float* __restrict__ ds_part,
                                                                const float* __restrict__ dw_part,
                                                                const float* __restrict__ dz_part,
                                                                const float* __restrict__ db_part, uint16_t* __restrict__ ds,
                                                                uint16_t* __restrict__ dst, float* __restrict__ dz,
                                                                float* __restrict__ dw_head, float* __restrict__ db_head,
                                                                int nsplit, int D) {
  using E = Elem<Tag>;
  const int DD = D * D;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int bh = blockIdx.y;
  if (i < DD) {
    const float* p = ds_part + (size_t)bh * nsplit * DD + i;
    const float* pw = dw_part + (size_t)bh * nsplit * DD + i;
    float s = 0.f, sw = 0.f;
#pragma unroll 4
    for (int sp = 0; sp < nsplit; ++sp) {
      s += p[(size_t)sp * DD];
      sw += pw[(size_t)sp * DD];
    }
    const int d2 = i / D, d1 = i % D;   // partial layout [d2][d1]
    const uint16_t h = E::from_float(s);
    dst[(size_t)bh * DD + i] = h;                 // dS^T [d2][d1]
    ds[(size_t)bh * DD + d1 * D + d2] = h;        // dS   [d1][d2]
    dw_head[(size_t)bh * DD + i] = sw;            // dW^T [d][e] of this head
  }
  if (i < D) {
    const float* p = dz_part + (size_t)bh * nsplit * D + i;
    const float* pb = db_part + (size_t)bh * nsplit * D + i;
    float s = 0.f, sb = 0.f;
    for (int sp = 0; sp < nsplit; ++sp) {
      s += p[(size_t)sp * D];
      sb += pb[(size_t)sp * D];
    }
    dz[(size_t)bh * D + i] = s;
    db_head[(size_t)bh * D + i] = sb;
  }
}

__global__ __launch_bounds__(256) void linear_bwd_reduce_heads_kernel(const float* __restrict__ dw_head,
                                                                      const float* __restrict__ db_head,
                                                                      float* __restrict__ d_weight, float* __restrict__ d_bias,
                                                                      int BH, int D) {
  const int DD = D * D;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < DD) {
    float s = 0.f;
#pragma unroll 4
    for (int h = 0; h < BH; ++h) s += dw_head[(size_t)h * DD + i];
    const int d = i / D, e = i % D;      // layout [d][e]
    d_weight[e * D + d] = s;
  }
  if (i < D) {
    float s = 0.f;
    for (int h = 0; h < BH; ++h) s += db_head[(size_t)h * D + i];
    d_bias[i] = s;
  }
}

// ---- kv -----------------------------------------------------------------------------------
template <typename Tag, int D>
__global__ __launch_bounds__(256) void linear_bwd_kv_kernel(const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
                                                            const uint16_t* __restrict__ ds, const uint16_t* __restrict__ dst,
                                                            const float* __restrict__ dz, uint16_t* __restrict__ dk,
                                                            uint16_t* __restrict__ dv, int L, int fmap, int tiles_per_wg,
                                                            int accumulate) {
  using E = Elem<Tag>;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int STR = D + 8;
  __shared__ __attribute__((aligned(16))) uint16_t sDS[D * STR];   // [d1][d2]  A of dc^T = dS v^T
  __shared__ __attribute__((aligned(16))) uint16_t sDST[D * STR];  // [d2][d1]  A of dv^T = dS^T c^T
  __shared__ __attribute__((aligned(16))) float sDZ[D];

  const int bh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;
  for (int idx = tid; idx < D * D / 8; idx += 256) {
    const int row = idx / (D / 8), col = (idx % (D / 8)) * 8;
    *reinterpret_cast<i16x8_t*>(&sDS[row * STR + col]) =
        *reinterpret_cast<const i16x8_t*>(ds + (size_t)bh * D * D + (size_t)row * D + col);
    *reinterpret_cast<i16x8_t*>(&sDST[row * STR + col]) =
        *reinterpret_cast<const i16x8_t*>(dst + (size_t)bh * D * D + (size_t)row * D + col);
  }
  if (tid < D) sDZ[tid] = dz[(size_t)bh * D + tid];
  __syncthreads();

  const size_t head_off = (size_t)bh * L * D;
  for (int tt = 0; tt < tiles_per_wg; ++tt) {
    const int row0 = (blockIdx.x * tiles_per_wg + tt) * 128 + wave * 32;
    if (row0 >= L) break;
    const int krow = row0 + r;
    const bool ok = krow < L;
    const size_t roff = head_off + (size_t)krow * D;

    float f[DC][8];
    i16x8_t vf[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i16x8_t x = {0, 0, 0, 0, 0, 0, 0, 0};
      vf[c] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
      if (ok) {
        x = *reinterpret_cast<const i16x8_t*>(k + roff + 16 * c + 8 * g);
        vf[c] = *reinterpret_cast<const i16x8_t*>(v + roff + 16 * c + 8 * g);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)x[j]);
    }
    float row_mx, row_inv;
    phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
    i16x8_t cf[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i32x4_t pw;
#pragma unroll
      for (int j = 0; j < 4; ++j) pw[j] = (int)E::pack2(f[c][2 * j], f[c][2 * j + 1]);
      cf[c] = __builtin_bit_cast(i16x8_t, pw);
    }
    float dc[DT][16], xk[DT][16];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      f32x16_t acc, vacc;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        acc[i] = 0.f;
        vacc[i] = 0.f;
      }
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const i16x8_t a1 = *reinterpret_cast<const i16x8_t*>(&sDS[(32 * t + r) * STR + 16 * c + 8 * g]);
        acc = E::mfma32(a1, vf[c], acc);
        const i16x8_t a2 = *reinterpret_cast<const i16x8_t*>(&sDST[(32 * t + r) * STR + 16 * c + 8 * g]);
        vacc = E::mfma32(a2, cf[c], vacc);
      }
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = 32 * t + 8 * i4 + 4 * g;
        i32x2_t xv = {0, 0};
        if (ok) xv = *reinterpret_cast<const i32x2_t*>(k + roff + d0);
        const uint16_t* xp = reinterpret_cast<const uint16_t*>(&xv);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          dc[t][4 * i4 + j] = acc[4 * i4 + j] + sDZ[d0 + j];
          xk[t][4 * i4 + j] = E::to_float(xp[j]);
        }
        if (ok) {
          float dvv[4] = {vacc[4 * i4 + 0], vacc[4 * i4 + 1], vacc[4 * i4 + 2], vacc[4 * i4 + 3]};
          if (accumulate) {
            const i32x2_t old = *reinterpret_cast<const i32x2_t*>(dv + roff + d0);
            const uint16_t* op = reinterpret_cast<const uint16_t*>(&old);
#pragma unroll
            for (int j = 0; j < 4; ++j) dvv[j] += E::to_float(op[j]);
          }
          i32x2_t w;
          w[0] = (int)E::pack2(dvv[0], dvv[1]);
          w[1] = (int)E::pack2(dvv[2], dvv[3]);
          *reinterpret_cast<i32x2_t*>(dv + roff + d0) = w;
        }
      }
    }
    phi_backward<DT>(fmap, xk, dc, row_mx, row_inv);
    if (ok) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          uint16_t* dst = dk + roff + 32 * t + 8 * i4 + 4 * g;
          if (accumulate) {
            const i32x2_t old = *reinterpret_cast<const i32x2_t*>(dst);
            const uint16_t* op = reinterpret_cast<const uint16_t*>(&old);
#pragma unroll
            for (int j = 0; j < 4; ++j) dc[t][4 * i4 + j] += E::to_float(op[j]);
          }
          i32x2_t w;
          w[0] = (int)E::pack2(dc[t][4 * i4 + 0], dc[t][4 * i4 + 1]);
          w[1] = (int)E::pack2(dc[t][4 * i4 + 2], dc[t][4 * i4 + 3]);
          *reinterpret_cast<i32x2_t*>(dst) = w;
        }
    }
  }
}

// ---- host ---------------------------------------------------------------------------------
struct LinBwdWs {
  LinWs fwd;
  size_t dn, y, dden, ds_part, dw_part, dz_part, db_part, ds, dst, dz, dw_head, db_head, total;
};
static LinBwdWs lin_bwd_ws(int BH, int L, int D) {
  LinBwdWs w;
  w.fwd = lin_ws(BH, L, D);
  const int64_t np = (int64_t)BH * w.fwd.nsplit;
  size_t off = w.fwd.total;
  w.dn = off;      off += align_up((int64_t)BH * L * D * 2, 256);
  w.y = off;       off += align_up((int64_t)BH * L * D * 2, 256);
  w.dden = off;    off += align_up((int64_t)BH * L * 4, 256);
  w.ds_part = off; off += align_up(np * D * D * 4, 256);
  w.dw_part = off; off += align_up(np * D * D * 4, 256);
  w.dz_part = off; off += align_up(np * D * 4, 256);
  w.db_part = off; off += align_up(np * D * 4, 256);
  w.ds = off;      off += align_up((int64_t)BH * D * D * 2, 256);
  w.dst = off;     off += align_up((int64_t)BH * D * D * 2, 256);
  w.dz = off;      off += align_up((int64_t)BH * D * 4, 256);
  w.dw_head = off; off += align_up((int64_t)BH * D * D * 4, 256);
  w.db_head = off; off += align_up((int64_t)BH * D * 4, 256);
  w.total = off;
  return w;
}
int64_t linear_bwd_workspace_bytes(int BH, int L, int D) { return (int64_t)lin_bwd_ws(BH, L, D).total; }

template <typename Tag, int D>
static int linear_bwd_impl(const void* q, const void* k, const void* v, const float* weight, const void* d_out, void* dq,
                           void* dk, void* dv, float* d_weight, float* d_bias, int fmap, int BH, int L, int accumulate,
                           char* ws, hipStream_t st) {
  const LinBwdWs w = lin_bwd_ws(BH, L, D);
  launch_state_build<Tag, D>(k, v, fmap, BH, L, ws, w.fwd, st);
  uint16_t* kvt = (uint16_t*)(ws + w.fwd.kvt);
  uint16_t* z = (uint16_t*)(ws + w.fwd.z);
  uint16_t* dn = (uint16_t*)(ws + w.dn);
  uint16_t* y = (uint16_t*)(ws + w.y);
  float* dden = (float*)(ws + w.dden);
  const int tiles = 4;
  const dim3 row_grid(cdiv(L, 128 * tiles), BH);
  hipLaunchKernelGGL((linear_bwd_rows_kernel<Tag, D>), row_grid, dim3(256), 0, st, (const uint16_t*)q,
                     (const uint16_t*)d_out, kvt, z, weight, (uint16_t*)dq, dn, y, dden, L, fmap, tiles, accumulate);
  hipLaunchKernelGGL((linear_bwd_states_kernel<Tag, D>), dim3(w.fwd.nsplit, BH), dim3(256), 0, st, (const uint16_t*)q, dn,
                     (const uint16_t*)d_out, y, dden, (float*)(ws + w.ds_part), (float*)(ws + w.dw_part),
                     (float*)(ws + w.dz_part), (float*)(ws + w.db_part), L, w.fwd.rows_per_split, fmap);
  hipLaunchKernelGGL((linear_bwd_reduce_kernel<Tag>), dim3(cdiv(D * D, 256), BH), dim3(256), 0, st,
                     (const float*)(ws + w.ds_part), (const float*)(ws + w.dw_part), (const float*)(ws + w.dz_part),
                     (const float*)(ws + w.db_part), (uint16_t*)(ws + w.ds), (uint16_t*)(ws + w.dst), (float*)(ws + w.dz),
                     (float*)(ws + w.dw_head), (float*)(ws + w.db_head), w.fwd.nsplit, D);
  hipLaunchKernelGGL(linear_bwd_reduce_heads_kernel, dim3(cdiv(D * D, 256)), dim3(256), 0, st,
                     (const float*)(ws + w.dw_head), (const float*)(ws + w.db_head), d_weight, d_bias, BH, D);
  hipLaunchKernelGGL((linear_bwd_kv_kernel<Tag, D>), row_grid, dim3(256), 0, st, (const uint16_t*)k, (const uint16_t*)v,
                     (const uint16_t*)(ws + w.ds), (const uint16_t*)(ws + w.dst), (const float*)(ws + w.dz), (uint16_t*)dk,
                     (uint16_t*)dv, L, fmap, tiles, accumulate);
  return check_launch("linear_bwd");
}

}  // namespace sla

using namespace sla;

extern "C" int sla_linear_bwd(const void* q, const void* k, const void* v, const float* weight, const float* bias,
                              const void* d_out, void* dq, void* dk, void* dv, float* d_weight, float* d_bias, int dtype,
                              int fmap, int B, int H, int L, int D, int accumulate, void* workspace,
                              int64_t workspace_bytes, void* stream) {
  int rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  (void)bias;  // the bias does not enter any gradient
  SLA_REQUIRE(q && k && v && weight && d_out && dq && dk && dv && d_weight && d_bias && workspace, SLA_ERR_BAD_ARG,
              "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)d_out | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv |
               (uintptr_t)weight | (uintptr_t)workspace) % 16 == 0,
              SLA_ERR_BAD_ARG, "pointers must be 16-byte aligned");
  const int BH = B * H;
  const int64_t need = linear_bwd_workspace_bytes(BH, L, D);
  SLA_REQUIRE(workspace_bytes >= need, SLA_ERR_WORKSPACE, "workspace of %lld bytes, need %lld", (long long)workspace_bytes,
              (long long)need);
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
#define SLA_LINB_CASE(TAG, DD) \
  return linear_bwd_impl<TAG, DD>(q, k, v, weight, d_out, dq, dk, dv, d_weight, d_bias, fmap, BH, L, accumulate, ws, st)
  if (dtype == SLA_BF16) {
    if (D == 128) SLA_LINB_CASE(bf16_tag, 128);
    SLA_LINB_CASE(bf16_tag, 64);
  }
  if (D == 128) SLA_LINB_CASE(f16_tag, 128);
  SLA_LINB_CASE(f16_tag, 64);
#undef SLA_LINB_CASE
}
