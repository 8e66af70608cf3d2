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
#include "bwd_steps.h"
#include "linear_bwd_stream.h"

namespace sla {

// ---- rows ---------------------------------------------------------------------------------
// grid (ceil(L / (32*NW*tiles)), BH), NW waves of 32 queries each.  Inputs and outputs move through a
// wave-private LDS staging tile so that global traffic is whole 256-byte rows; the next tile's q and G
// rows are fetched into registers while the current tile is computed.
template <typename Tag, int D, int NW>
__global__ __launch_bounds__(64 * NW) void linear_bwd_rows_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ gout, const uint16_t* __restrict__ kvt,
    const uint16_t* __restrict__ kvp, const uint16_t* __restrict__ z, const uint16_t* __restrict__ wt,
    uint16_t* __restrict__ dq, const RowLayout lin, const RowLayout ldo, uint16_t* __restrict__ dn_out,
    uint16_t* __restrict__ y_out, float* __restrict__ dden_out, int L, int fmap, int tiles_per_wg, int accumulate) {
  using E = Elem<Tag>;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int STR = D + 8;
  __shared__ __attribute__((aligned(16))) uint16_t sKVT[D * STR];  // [d2][d1]          A of n^T = KVT a^T
  __shared__ __attribute__((aligned(16))) uint16_t sKVP[D * STR];  // [d1][perm d2]     A of da^T = S dn^T
  __shared__ __attribute__((aligned(16))) uint16_t sWT[D * STR];   // [d][e]            A of dy^T = W^T G^T
  __shared__ __attribute__((aligned(16))) uint16_t sStage[NW][32 * STR];
  __shared__ __attribute__((aligned(16))) float sZ[D];

  const int bh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;

  {
    // all three operand matrices arrive in 16 bit and in the layout their MFMA reads want
    const uint16_t* src = kvt + (size_t)bh * D * D;
    const uint16_t* srcp = kvp + (size_t)bh * D * D;
    for (int idx = tid; idx < D * D / 8; idx += 64 * NW) {
      const int row = idx / (D / 8), col = (idx % (D / 8)) * 8;
      *reinterpret_cast<i16x8_t*>(&sKVT[row * STR + col]) = *reinterpret_cast<const i16x8_t*>(src + (size_t)row * D + col);
      *reinterpret_cast<i16x8_t*>(&sKVP[row * STR + col]) = *reinterpret_cast<const i16x8_t*>(srcp + (size_t)row * D + col);
      *reinterpret_cast<i16x8_t*>(&sWT[row * STR + col]) = *reinterpret_cast<const i16x8_t*>(wt + (size_t)row * D + col);
    }
    if (tid < D) sZ[tid] = E::to_float(z[(size_t)bh * D + tid]);
  }
  __syncthreads();

  // q and dq rows lie lin.sl elements apart, the rows of G ldo.sl; the temporaries dn, y are contiguous
  const size_t head_off = (size_t)bh * L * D;
  const size_t head_in = lin.head(bh), head_g = ldo.head(bh);
  const size_t pitch = (size_t)lin.sl, pitch_g = (size_t)ldo.sl;
  uint16_t* stage = sStage[wave];
  constexpr int STEP = 32 * NW;
  const int first_row = blockIdx.x * tiles_per_wg * STEP + wave * 32;
  TileRows<D> qt, gt;                  // q and G rows of the tile about to be processed
  if (first_row < L) {
    qt.fetch(q + head_in + (size_t)first_row * pitch, min(32, L - first_row), lane, pitch);
    gt.fetch(gout + head_g + (size_t)first_row * pitch_g, min(32, L - first_row), lane, pitch_g);
  }
  for (int tt = 0; tt < tiles_per_wg; ++tt) {
    const int row0 = first_row + tt * STEP;
    if (row0 >= L) break;
    const int rows_valid = min(32, L - row0);
    const int qrow = row0 + r;
    const bool ok = qrow < L;
    const size_t toff = head_off + (size_t)row0 * D;
    const size_t toff_in = head_in + (size_t)row0 * pitch;

    // q in B-operand order (d = 16c + 8g + j) and in accumulator order (d = 32t + 8i4 + 4g + j)
    qt.park(stage, lane);
    float f[DC][8];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      const i16x8_t x = *reinterpret_cast<const i16x8_t*>(&stage[r * STR + 16 * c + 8 * g]);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)x[j]);
    }
    i32x2_t xraw[DT][4];
#pragma unroll
    for (int t1 = 0; t1 < DT; ++t1)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        xraw[t1][i4] = *reinterpret_cast<const i32x2_t*>(&stage[r * STR + 32 * t1 + 8 * i4 + 4 * g]);
    wave_lds_fence();
    gt.park(stage, lane);
    i16x8_t gf[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) gf[c] = *reinterpret_cast<const i16x8_t*>(&stage[r * STR + 16 * c + 8 * g]);
    wave_lds_fence();
    TileRows<D> dq_old;
    if (accumulate) dq_old.fetch(dq + toff_in, rows_valid, lane, pitch);
    if (tt + 1 < tiles_per_wg && row0 + STEP < L) {
      qt.fetch(q + toff_in + (size_t)STEP * pitch, min(32, L - row0 - STEP), lane, pitch);
      gt.fetch(gout + head_g + (size_t)(row0 + STEP) * pitch_g, min(32, L - row0 - STEP), lane, pitch_g);
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
    float yv[DT][16], dnv[DT][16];
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
        const i16x8_t a1 = *reinterpret_cast<const i16x8_t*>(&sKVT[(32 * t + r) * STR + 16 * c + 8 * g]);
        yacc = E::mfma32(a1, af[c], yacc);
        const i16x8_t a2 = *reinterpret_cast<const i16x8_t*>(&sWT[(32 * t + r) * STR + 16 * c + 8 * g]);
        dyacc = E::mfma32(a2, gf[c], dyacc);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        yv[t][i] = yacc[i];
        dnv[t][i] = dyacc[i];
      }
    }
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

    // dn^T as B operand (register 8c2+j of tile t is d2 = 32t + 8*((8c2+j)/4) + 4g + j%4, the order sKVP's
    // columns are stored in); dn and y go to memory for the state kernel
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
    store_acc_tile<E, D>(stage, dnv, dn_out + toff, nullptr, rows_valid, lane);
    store_acc_tile<E, D>(stage, yv, y_out + toff, nullptr, rows_valid, lane);

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
        const uint16_t* xp = reinterpret_cast<const uint16_t*>(&xraw[t1][i4]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          da[t1][4 * i4 + j] = acc[4 * i4 + j] + sZ[d0 + j] * dden;
          xq[t1][4 * i4 + j] = E::to_float(xp[j]);
        }
      }
    }
    phi_backward<DT>(fmap, xq, da, row_mx, row_inv);
    store_acc_tile<E, D>(stage, da, dq + toff_in, accumulate ? &dq_old : nullptr, rows_valid, lane, pitch);
  }
}

// ---- states -------------------------------------------------------------------------------
// grid (nsplit, BH).  dS^T partial [d2][d1] per (bh, split); dW^T partial [d][e] per (bh, split).
template <typename Tag, int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void linear_bwd_states_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ dn, const uint16_t* __restrict__ gout,
    const uint16_t* __restrict__ y, const float* __restrict__ dden, const RowLayout lin, const RowLayout ldo,
    float* __restrict__ ds_part, float* __restrict__ dw_part, float* __restrict__ dz_part, float* __restrict__ db_part, int L,
    int rows_per_split, int fmap) {
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
  // the cross-thread sums of dz / db at the very end reuse the first two tiles (two workgroups per
  // compute unit need the LDS footprint below 80 KB)
  static_assert(2 * TR * STR * 2 >= 2 * RPP * D * 4, "reduction scratch does not fit the tiles it reuses");
  float (*sRed)[RPP][D] = reinterpret_cast<float (*)[RPP][D]>(sA);

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

  // (no register prefetch of the next tile: the second workgroup on the compute unit covers the latency,
  //  and the registers it would take are what lets that second workgroup fit)
  i16x8_t rq[NP], rdn[NP], rg[NP], ry[NP];
  float rdd[NP];
  auto fetch = [&](int r0) {
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int grow = r0 + lrow + p * RPP;
      rq[p] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
      rdn[p] = rq[p];
      rg[p] = rq[p];
      ry[p] = rq[p];
      rdd[p] = 0.f;
      if (grow < row_end) {
        const size_t off = head_off + (size_t)grow * D + lcol;          // dn, y: contiguous temporaries
        rq[p] = *reinterpret_cast<const i16x8_t*>(q + lin.head(bh) + (size_t)grow * (size_t)lin.sl + lcol);
        rdn[p] = *reinterpret_cast<const i16x8_t*>(dn + off);
        rg[p] = *reinterpret_cast<const i16x8_t*>(gout + ldo.head(bh) + (size_t)grow * (size_t)ldo.sl + lcol);
        ry[p] = *reinterpret_cast<const i16x8_t*>(y + off);
        rdd[p] = dden[(size_t)bh * L + grow];
      }
    }
  };
  for (int r0 = row_begin; r0 < row_end; r0 += TR) {
    fetch(r0);
    __syncthreads();
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int row = lrow + p * RPP;
      const int grow = r0 + row;
      const bool ok = grow < row_end;
      const i16x8_t xq = rq[p], xdn = rdn[p], xg = rg[p], xy = ry[p];
      const float dd = rdd[p];
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
      } else if (fmap == SLA_FMAP_RELU) {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = fmap_pointwise<Tag>(SLA_FMAP_RELU, f[e]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = fmap_pointwise<Tag>(SLA_FMAP_ELU, f[e]);
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
#pragma unroll 8
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
// Same tile traffic as the rows kernel: NW waves of 32 keys, whole-row global accesses through a
// wave-private staging tile.
// CONTIG: k, v, dk, dv are contiguous (B, H, L, D): the row pitch is the compile-time D.
template <typename Tag, int D, int NW, bool CONTIG>
__global__ __launch_bounds__(64 * NW) void linear_bwd_kv_kernel(const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
                                                                const uint16_t* __restrict__ ds,
                                                                const uint16_t* __restrict__ dst, const float* __restrict__ dz,
                                                                uint16_t* __restrict__ dk, uint16_t* __restrict__ dv,
                                                                const RowLayout lin, int L, int fmap, int tiles_per_wg,
                                                                int accumulate) {
  using E = Elem<Tag>;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int STR = D + 8;
  __shared__ __attribute__((aligned(16))) uint16_t sDS[D * STR];   // [d1][d2]  A of dc^T = dS v^T
  __shared__ __attribute__((aligned(16))) uint16_t sDST[D * STR];  // [d2][d1]  A of dv^T = dS^T c^T
  __shared__ __attribute__((aligned(16))) uint16_t sStage[NW][32 * STR];
  __shared__ __attribute__((aligned(16))) float sDZ[D];

  const int bh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;
  for (int idx = tid; idx < D * D / 8; idx += 64 * NW) {
    const int row = idx / (D / 8), col = (idx % (D / 8)) * 8;
    *reinterpret_cast<i16x8_t*>(&sDS[row * STR + col]) =
        *reinterpret_cast<const i16x8_t*>(ds + (size_t)bh * D * D + (size_t)row * D + col);
    *reinterpret_cast<i16x8_t*>(&sDST[row * STR + col]) =
        *reinterpret_cast<const i16x8_t*>(dst + (size_t)bh * D * D + (size_t)row * D + col);
  }
  if (tid < D) sDZ[tid] = dz[(size_t)bh * D + tid];
  __syncthreads();

  const size_t head_off = lin.head(bh);   // k, v, dk, dv rows: lin.sl elements apart
  const size_t pitch = CONTIG ? (size_t)D : (size_t)lin.sl;
  uint16_t* stage = sStage[wave];
  constexpr int STEP = 32 * NW;
  const int first_row = blockIdx.x * tiles_per_wg * STEP + wave * 32;
  for (int tt = 0; tt < tiles_per_wg; ++tt) {
    const int row0 = first_row + tt * STEP;
    if (row0 >= L) break;
    const int rows_valid = min(32, L - row0);
    const size_t toff = head_off + (size_t)row0 * pitch;

    // two waves share a SIMD and cover each other's load latency; registers are too scarce to fetch ahead
    TileRows<D> kt, vt;
    kt.fetch(k + toff, rows_valid, lane, pitch);
    vt.fetch(v + toff, rows_valid, lane, pitch);
    kt.park(stage, lane);
    float f[DC][8];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      const i16x8_t x = *reinterpret_cast<const i16x8_t*>(&stage[r * STR + 16 * c + 8 * g]);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)x[j]);
    }
    i32x2_t xraw[DT][4];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        xraw[t][i4] = *reinterpret_cast<const i32x2_t*>(&stage[r * STR + 32 * t + 8 * i4 + 4 * g]);
    wave_lds_fence();
    vt.park(stage, lane);
    i16x8_t vf[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) vf[c] = *reinterpret_cast<const i16x8_t*>(&stage[r * STR + 16 * c + 8 * g]);
    wave_lds_fence();
    float row_mx, row_inv;
    phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
    {
      // dv^T = dS^T c^T
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
          const i16x8_t a2 = *reinterpret_cast<const i16x8_t*>(&sDST[(32 * t + r) * STR + 16 * c + 8 * g]);
          vacc = E::mfma32(a2, cf[c], vacc);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) dvv[t][i] = vacc[i];
      }
      if (accumulate)
        store_acc_tile<E, D, true>(stage, dvv, dv + toff, nullptr, rows_valid, lane, pitch);
      else
        store_acc_tile<E, D, false>(stage, dvv, dv + toff, nullptr, rows_valid, lane, pitch);
    }
    // dc^T = dS v^T + dz ; dk = phi'(k) dc
    float dc[DT][16], xk[DT][16];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      f32x16_t acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const i16x8_t a1 = *reinterpret_cast<const i16x8_t*>(&sDS[(32 * t + r) * STR + 16 * c + 8 * g]);
        acc = E::mfma32(a1, vf[c], acc);
      }
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = 32 * t + 8 * i4 + 4 * g;
        const uint16_t* xp = reinterpret_cast<const uint16_t*>(&xraw[t][i4]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          dc[t][4 * i4 + j] = acc[4 * i4 + j] + sDZ[d0 + j];
          xk[t][4 * i4 + j] = E::to_float(xp[j]);
        }
      }
    }
    phi_backward<DT>(fmap, xk, dc, row_mx, row_inv);
    if (accumulate)
      store_acc_tile<E, D, true>(stage, dc, dk + toff, nullptr, rows_valid, lane, pitch);
    else
      store_acc_tile<E, D, false>(stage, dc, dk + toff, nullptr, rows_valid, lane, pitch);
  }
}

// ---- host ---------------------------------------------------------------------------------
struct LinBwdWs {
  LinWs fwd;
  LinSplit st;   // slices of the states kernel (two workgroups per compute unit)
  LinSplit ss;   // slices of the stream kernel (one workgroup per compute unit, 128 rows per step): never more than st's
  size_t dn, y, dden, ds_part, dw_part, dz_part, db_part, ds, dst, dz, dw_head, db_head, total;
};
static LinBwdWs lin_bwd_ws(int BH, int L, int D) {
  LinBwdWs w;
  w.fwd = lin_ws(BH, L, D);
  w.st = lin_split(BH, L, 512);
  w.ss = lin_split(BH, L, 256, LBS_TR);
  const int64_t np = (int64_t)BH * w.st.nsplit;
  size_t off = w.fwd.total;
  w.dn = off;      off += align_up((int64_t)BH * L * D * 2, 256);
  w.y = off;       off += align_up((int64_t)BH * L * D * 2, 256);
  w.dden = off;    off += align_up((int64_t)BH * L * 4, 256);
  w.ds_part = off; off += align_up(np * D * D * 4, 256);
  // (the stream path keeps M of every head there in both orientations: two matrices per head at least)
  w.dw_part = off; off += align_up((np > 2 * BH ? np : 2 * (int64_t)BH) * D * D * 4, 256);
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
                           void* dk, void* dv, const RowLayout& lin, const RowLayout& ldo, float* d_weight, float* d_bias,
                           int fmap, int BH, int L, int flags, char* ws, hipStream_t st, int steps) {
  if (steps == 0) return SLA_OK;        // (arguments checked, nothing asked for)
  const LinBwdWs w = lin_bwd_ws(BH, L, D);
  const int accumulate = flags & SLA_BWD_ACCUMULATE;
  if ((steps & LB_STATES) && !(flags & SLA_BWD_STATES_READY)) {
    // everything the forward's state build leaves: transposed state, z, and (fold) the folded state + 16-bit weight
    launch_state_build<Tag, D>(k, v, lin, weight, fmap, BH, L, ws, w.fwd, st, false);
    hipLaunchKernelGGL((linear_fold_kernel<Tag>), dim3(D / (1024 / D), BH), dim3(256), 0, st,
                       (const uint16_t*)(ws + w.fwd.kvt), weight, (uint16_t*)(ws + w.fwd.kvwt), (uint16_t*)(ws + w.fwd.wt), D);
  }
  uint16_t* kvt = (uint16_t*)(ws + w.fwd.kvt);
  uint16_t* z = (uint16_t*)(ws + w.fwd.z);
  constexpr int NW_ROWS = 4, NW_KV = 8;   // one workgroup per compute unit either way (LDS)
  const int tiles_kv = balanced_tiles(cdiv(L, 32 * NW_KV), BH, 1);
  // (the stream kernel addresses a head's rows through 32-bit buffer offsets)
  const auto fits32 = [&](const RowLayout& lay) { return ((int64_t)(L - 1) * lay.sl + D) * 2 < ((int64_t)1 << 32); };
  bool streamed = false;
  if constexpr (D == 128) streamed = fits32(lin) && fits32(ldo);
  if constexpr (D == 128) if (streamed) {
    // q and G once: dq, and the partial sums M^T, dz, db of every slice (the slices' partials and the per-head M^T
    // take the places of the two-matrix partials of the general path: ds_part, dw_part)
    float* m_part = (float*)(ws + w.ds_part);
    float* mt_head = (float*)(ws + w.dw_part);
    float* m_head = mt_head + (size_t)BH * D * D;
    if (steps & LB_QUERY) {
#define SLA_LBS_LAUNCH(FM)                                                                                                  \
  hipLaunchKernelGGL((linear_bwd_stream_kernel<Tag, FM>), dim3(w.ss.nsplit, BH), dim3(512), 0, st, (const uint16_t*)q,        \
                     (const uint16_t*)d_out, (const uint16_t*)(ws + w.fwd.kvwt), z, (uint16_t*)dq, lin, ldo, m_part,          \
                     (float*)(ws + w.dz_part), (float*)(ws + w.db_part), L, w.ss.rows_per_split, accumulate)
    if (fmap == SLA_FMAP_ELU) SLA_LBS_LAUNCH(SLA_FMAP_ELU);
    else if (fmap == SLA_FMAP_RELU) SLA_LBS_LAUNCH(SLA_FMAP_RELU);
    else SLA_LBS_LAUNCH(SLA_FMAP_SOFTMAX);
#undef SLA_LBS_LAUNCH
    }
    if (steps & LB_REDUCE) {
    hipLaunchKernelGGL(linear_bwd_sum_kernel, dim3(cdiv(D * D, 256), BH), dim3(256), 0, st, (const float*)m_part,
                       (const float*)(ws + w.dz_part), (const float*)(ws + w.db_part), mt_head, m_head, (float*)(ws + w.dz),
                       (float*)(ws + w.db_head), w.ss.nsplit, D);
    hipLaunchKernelGGL((linear_bwd_products_kernel<Tag>), dim3(D * D / 256, BH, 2), dim3(256), 0, st, (const float*)mt_head,
                       (const float*)m_head, weight, kvt, (uint16_t*)(ws + w.ds), (uint16_t*)(ws + w.dst), (float*)(ws + w.dw_head), D);
    }
  }
  if (!streamed) {
  uint16_t* dn = (uint16_t*)(ws + w.dn);
  uint16_t* y = (uint16_t*)(ws + w.y);
  float* dden = (float*)(ws + w.dden);
  const int tiles_rows = balanced_tiles(cdiv(L, 32 * NW_ROWS), BH, 1);
  if (steps & LB_QUERY) {
  hipLaunchKernelGGL((linear_bwd_rows_kernel<Tag, D, NW_ROWS>), dim3(cdiv(L, 32 * NW_ROWS * tiles_rows), BH), dim3(64 * NW_ROWS), 0, st, (const uint16_t*)q,
                     (const uint16_t*)d_out, kvt, (const uint16_t*)(ws + w.fwd.kvp), z, (const uint16_t*)(ws + w.fwd.wt), (uint16_t*)dq, lin, ldo, dn, y,
                     dden, L, fmap, tiles_rows, accumulate);
  hipLaunchKernelGGL((linear_bwd_states_kernel<Tag, D>), dim3(w.st.nsplit, BH), dim3(256), 0, st, (const uint16_t*)q, dn,
                     (const uint16_t*)d_out, y, dden, lin, ldo, (float*)(ws + w.ds_part), (float*)(ws + w.dw_part),
                     (float*)(ws + w.dz_part), (float*)(ws + w.db_part), L, w.st.rows_per_split, fmap);
  }
  if (steps & LB_REDUCE)
  hipLaunchKernelGGL((linear_bwd_reduce_kernel<Tag>), dim3(cdiv(D * D, 256), BH), dim3(256), 0, st,
                     (const float*)(ws + w.ds_part), (const float*)(ws + w.dw_part), (const float*)(ws + w.dz_part),
                     (const float*)(ws + w.db_part), (uint16_t*)(ws + w.ds), (uint16_t*)(ws + w.dst), (float*)(ws + w.dz),
                     (float*)(ws + w.dw_head), (float*)(ws + w.db_head), w.st.nsplit, D);
  }
  if (steps & LB_REDUCE)
    hipLaunchKernelGGL(linear_bwd_reduce_heads_kernel, dim3(cdiv(D * D, 256)), dim3(256), 0, st,
                       (const float*)(ws + w.dw_head), (const float*)(ws + w.db_head), d_weight, d_bias, BH, D);
  if (!(steps & LB_KEYS)) return check_launch("linear_bwd");
  if constexpr (D == 128) if (streamed) {
#define SLA_LBK_LAUNCH(FM)                                                                                                \
  hipLaunchKernelGGL((linear_bwd_keys_kernel<Tag, FM>), dim3(w.ss.nsplit, BH), dim3(512), 0, st, (const uint16_t*)k,        \
                     (const uint16_t*)v, (const uint16_t*)(ws + w.ds), (const uint16_t*)(ws + w.dst),                       \
                     (const float*)(ws + w.dz), (uint16_t*)dk, (uint16_t*)dv, lin, L, w.ss.rows_per_split, accumulate)
    if (fmap == SLA_FMAP_ELU) SLA_LBK_LAUNCH(SLA_FMAP_ELU);
    else if (fmap == SLA_FMAP_RELU) SLA_LBK_LAUNCH(SLA_FMAP_RELU);
    else SLA_LBK_LAUNCH(SLA_FMAP_SOFTMAX);
#undef SLA_LBK_LAUNCH
    return check_launch("linear_bwd");
  }
  if (lin.sl == D)
    hipLaunchKernelGGL((linear_bwd_kv_kernel<Tag, D, NW_KV, true>), dim3(cdiv(L, 32 * NW_KV * tiles_kv), BH), dim3(64 * NW_KV),
                       0, st, (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)(ws + w.ds),
                       (const uint16_t*)(ws + w.dst), (const float*)(ws + w.dz), (uint16_t*)dk, (uint16_t*)dv, lin, L, fmap,
                       tiles_kv, accumulate);
  else
    hipLaunchKernelGGL((linear_bwd_kv_kernel<Tag, D, NW_KV, false>), dim3(cdiv(L, 32 * NW_KV * tiles_kv), BH), dim3(64 * NW_KV),
                       0, st, (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)(ws + w.ds),
                       (const uint16_t*)(ws + w.dst), (const float*)(ws + w.dz), (uint16_t*)dk, (uint16_t*)dv, lin, L, fmap,
                       tiles_kv, accumulate);
  return check_launch("linear_bwd");
}

// dW and db alone, from the row-wise temporaries a rows kernel has left (used by the backward of the complement-mode
// linear branch, whose state gradients are per query block and formed elsewhere): the states kernel, its reduction and
// the sum over the heads.  `ws` is a region of weight_grads_workspace_bytes() bytes.
struct WeightGradWs {
  LinSplit st;
  size_t ds_part, dw_part, dz_part, db_part, ds, dst, dz, dw_head, db_head, total;
};
static WeightGradWs weight_grad_ws(int BH, int L, int D) {
  WeightGradWs w;
  w.st = lin_split(BH, L, 512);
  const int64_t np = (int64_t)BH * w.st.nsplit;
  size_t off = 0;
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
int64_t weight_grads_workspace_bytes(int BH, int L, int D) { return (int64_t)weight_grad_ws(BH, L, D).total; }

template <typename Tag, int D>
static void weight_grads_impl(const void* q, const void* dn, const void* gout, const void* y, const float* dden, int BH, int L,
                              int fmap, char* ws, float* d_weight, float* d_bias, hipStream_t st) {
  const WeightGradWs w = weight_grad_ws(BH, L, D);
  const RowLayout lay = contiguous_layout(BH, L, D);
  hipLaunchKernelGGL((linear_bwd_states_kernel<Tag, D>), dim3(w.st.nsplit, BH), dim3(256), 0, st, (const uint16_t*)q,
                     (const uint16_t*)dn, (const uint16_t*)gout, (const uint16_t*)y, dden, lay, lay, (float*)(ws + w.ds_part),
                     (float*)(ws + w.dw_part), (float*)(ws + w.dz_part), (float*)(ws + w.db_part), L, w.st.rows_per_split, fmap);
  hipLaunchKernelGGL((linear_bwd_reduce_kernel<Tag>), dim3(cdiv(D * D, 256), BH), dim3(256), 0, st,
                     (const float*)(ws + w.ds_part), (const float*)(ws + w.dw_part), (const float*)(ws + w.dz_part),
                     (const float*)(ws + w.db_part), (uint16_t*)(ws + w.ds), (uint16_t*)(ws + w.dst), (float*)(ws + w.dz),
                     (float*)(ws + w.dw_head), (float*)(ws + w.db_head), w.st.nsplit, D);
  hipLaunchKernelGGL(linear_bwd_reduce_heads_kernel, dim3(cdiv(D * D, 256)), dim3(256), 0, st,
                     (const float*)(ws + w.dw_head), (const float*)(ws + w.db_head), d_weight, d_bias, BH, D);
}
void launch_weight_grads(int dtype, int D, const void* q, const void* dn, const void* gout, const void* y, const float* dden,
                         int BH, int L, int fmap, char* ws, float* d_weight, float* d_bias, hipStream_t st) {
  if (dtype == SLA_BF16) {
    if (D == 128) weight_grads_impl<bf16_tag, 128>(q, dn, gout, y, dden, BH, L, fmap, ws, d_weight, d_bias, st);
    else weight_grads_impl<bf16_tag, 64>(q, dn, gout, y, dden, BH, L, fmap, ws, d_weight, d_bias, st);
  } else {
    if (D == 128) weight_grads_impl<f16_tag, 128>(q, dn, gout, y, dden, BH, L, fmap, ws, d_weight, d_bias, st);
    else weight_grads_impl<f16_tag, 64>(q, dn, gout, y, dden, BH, L, fmap, ws, d_weight, d_bias, st);
  }
}

int linear_bwd_steps(const void* q, const void* k, const void* v, const int64_t* qkv_strides, const float* weight,
                     const float* bias, const void* d_out, const int64_t* do_strides, void* dq, void* dk, void* dv,
                     float* d_weight, float* d_bias, int dtype, int fmap, int B, int H, int L, int D, int flags,
                     void* workspace, int64_t workspace_bytes, void* stream, int steps) {
  int rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  SLA_REQUIRE((flags & ~(SLA_BWD_ACCUMULATE | SLA_BWD_STATES_READY)) == 0, SLA_ERR_BAD_ARG, "unknown flag bits in %d", flags);
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
  RowLayout lin, ldo;
  rc = make_layout(qkv_strides, B, H, L, D, 2, &lin);
  if (rc) return rc;
  rc = make_layout(do_strides, B, H, L, D, 2, &ldo);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
#define SLA_LINB_CASE(TAG, DD) \
  return linear_bwd_impl<TAG, DD>(q, k, v, weight, d_out, dq, dk, dv, lin, ldo, d_weight, d_bias, fmap, BH, L, flags, ws, st, \
                                  steps)
  if (dtype == SLA_BF16) {
    if (D == 128) SLA_LINB_CASE(bf16_tag, 128);
    SLA_LINB_CASE(bf16_tag, 64);
  }
  if (D == 128) SLA_LINB_CASE(f16_tag, 128);
  SLA_LINB_CASE(f16_tag, 64);
#undef SLA_LINB_CASE
}

}  // namespace sla

using namespace sla;

extern "C" int sla_linear_bwd(const void* q, const void* k, const void* v, const float* weight, const float* bias,
                              const void* d_out, void* dq, void* dk, void* dv, float* d_weight, float* d_bias, int dtype,
                              int fmap, int B, int H, int L, int D, int flags, void* workspace,
                              int64_t workspace_bytes, void* stream) {
  return linear_bwd_steps(q, k, v, nullptr, weight, bias, d_out, nullptr, dq, dk, dv, d_weight, d_bias, dtype, fmap, B, H, L,
                          D, flags, workspace, workspace_bytes, stream, LB_ALL);
}

extern "C" int sla_linear_bwd_strided(const void* q, const void* k, const void* v, const int64_t* qkv_strides,
                                      const float* weight, const float* bias, const void* d_out, const int64_t* do_strides,
                                      void* dq, void* dk, void* dv, float* d_weight, float* d_bias, int dtype, int fmap,
                                      int B, int H, int L, int D, int flags, void* workspace, int64_t workspace_bytes,
                                      void* stream) {
  SLA_REQUIRE(qkv_strides && do_strides, SLA_ERR_BAD_ARG, "null strides");
  return linear_bwd_steps(q, k, v, qkv_strides, weight, bias, d_out, do_strides, dq, dk, dv, d_weight, d_bias, dtype, fmap, B,
                          H, L, D, flags, workspace, workspace_bytes, stream, LB_ALL);
}
