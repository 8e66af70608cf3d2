// Backward of the linear-attention branch + projection, query side, for head dim 128: one pass over q and G = d(out).
//
// With a = phi(q), S = phi(k)^T v, z = sum phi(k), den = 1e-5 + a.z, P = S W^T (the folded state of the forward,
// core.py:90-99 of the reference) the branch is out = a P / den + b, so per query row
//   t    = G P^T                         (the only product that needs the row's G)
//   dden = -(a.t) / den^2
//   da   = t / den + dden z ;  dq = phi'(q) da
// and the sums over the rows reduce to ONE D x D matrix and two vectors:
//   M  = sum_l (a_l / den_l)^T G_l       ->  dS = M W,  dW = M^T S     (small products per head, formed afterwards)
//   dz = sum_l dden_l a_l ;  db = sum_l G_l
// No row-wise temporary goes to memory: q and G are read once, dq is read (when accumulating) and written once.
//
//   stream   : grid (slices of L, heads), 8 waves.  Per 128 rows: every wave takes 16 rows through t, dden, da, dq
//              (16x16x32 products, the row spread over 4 lanes), leaves a/den and dq in LDS; then the workgroup adds the
//              tile's (a/den)^T G to M (32x32x16 products, both operands read transposed from LDS), dz and db on the
//              vector ALU, and writes the dq rows whole.
//   reduce   : fixed-order sums of the slices' partials -> M^T (fp32), dz, db per head
//   products : dS = M W (16 bit, both orientations) and this head's dW = M^T S (fp32)
#pragma once
#include "linear_state.h"

namespace sla {

// LDS tiles of 256-byte rows without padding: 16-byte piece p of row r sits at piece slot p ^ swz(r).  Row-wise
// 16-byte / 8-byte reads by 16 consecutive rows and transposing reads of 4 rows x 4 pieces both touch every bank once.
static __device__ __forceinline__ int lbs_swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
static __device__ __forceinline__ uint32_t lbs_off(int row, int col) {
  return (uint32_t)row * 256u + (uint32_t)(((col >> 3) ^ lbs_swz(row & 15)) << 4) + (uint32_t)(col & 7) * 2u;
}

constexpr int LBS_TR = 128;   // rows per step of the stream kernel

template <typename Tag, int FMAP>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void linear_bwd_stream_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ gout, const uint16_t* __restrict__ kvwt,
    const uint16_t* __restrict__ z, uint16_t* __restrict__ dq, const RowLayout lin, const RowLayout ldo,
    float* __restrict__ m_part, float* __restrict__ dz_part, float* __restrict__ db_part, int L, int rows_per_split,
    int accumulate) {
  // (the feature map is a template argument: as a run-time value every element's phi sits behind its own branch)
  using E = Elem<Tag>;
  constexpr int fmap = FMAP;
  constexpr int D = 128, TR = LBS_TR;
  constexpr int TILE = TR * D * 2;               // bytes of one swizzled tile of rows
  constexpr int PSTR = D * 2 + 16;               // row pitch of sP: 16 rows x 16 bytes of a row-wise read cover every bank
  __shared__ __attribute__((aligned(16))) char smem[3 * TILE + D * PSTR + 2 * D * 4];
  char* const sQ = smem;                         // raw q rows, then a/den of the same rows
  char* const sG = smem + TILE;                  // G rows
  char* const sO = smem + 2 * TILE;              // dq rows of this step (16 bit)
  char* const sP = smem + 3 * TILE;              // folded state, P[d1][e]
  float* const sZ = reinterpret_cast<float*>(smem + 3 * TILE + D * PSTR);   // z[d1]
  float* const sDD = sZ + D;                                                // dden * den per row of the step
  float (*sRed)[32][D] = reinterpret_cast<float (*)[32][D]>(smem);          // final cross-thread sums (over sQ)

  const int split = blockIdx.x, bh = blockIdx.y, nsplit = gridDim.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int row_begin = split * rows_per_split;
  const int row_end = min(L, row_begin + rows_per_split);
  // loader layout: thread = (row lrow + 32 p, 16-byte piece lp); + 8 KiB per p in a tile
  const int lrow = tid >> 4, lp = tid & 15;
  const uint32_t ld_off = lbs_off(lrow, 8 * lp);
  // row phase: lane = (row l of the wave's 16, quarter h): d1 = 16 T + 4 h + j
  const int l = lane & 15, h = lane >> 4;

  {
    // The folded state arrives as kvwt[e][d1]; the row phase wants rows of P[d1][e].  Through sQ: wave T turns the
    // 16 columns d1 = 16 T .. of the staged copy into rows by transposing reads.
    const uint16_t* src = kvwt + (size_t)bh * D * D;
#pragma unroll
    for (int p = 0; p < D / 32; ++p)
      *reinterpret_cast<i16x8_t*>(sQ + ld_off + p * 8192) =
          *reinterpret_cast<const i16x8_t*>(src + (size_t)(lrow + 32 * p) * D + 8 * lp);
    if (tid < D) sZ[tid] = E::to_float(z[(size_t)bh * D + tid]);
    __syncthreads();
    const int pe = 8 * h + (l >> 2);      // rows e = 32 c + pe .. + 3 and + 4 .. + 7, columns 16 wave + 4 (l % 4) ..
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint16_t* p0 = reinterpret_cast<const uint16_t*>(sQ + lbs_off(32 * c + pe, 16 * wave + 4 * (l & 3)));
      const uint16_t* p1 = reinterpret_cast<const uint16_t*>(sQ + lbs_off(32 * c + pe + 4, 16 * wave + 4 * (l & 3)));
      // lane (l, h) now holds P[16 wave + l][32 c + 8 h .. + 7]
      *reinterpret_cast<i16x8_t*>(sP + (16 * wave + l) * PSTR + (32 * c + 8 * h) * 2) =
          concat4(lds_read_tr16(p0), lds_read_tr16(p1));
    }
    __syncthreads();
  }

  const __amdgpu_buffer_rsrc_t q_rs = make_rsrc(q + lin.head(bh), lin.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t g_rs = make_rsrc(gout + ldo.head(bh), ldo.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t dq_rs = make_rsrc(dq + lin.head(bh), accumulate ? lin.head_range_bytes(L, D) : 0u);
  uint16_t* const dqh = dq + lin.head(bh);
  const size_t pitch = (size_t)lin.sl;
  const uint32_t pitch_b = (uint32_t)lin.sl * 2u, pitch_gb = (uint32_t)ldo.sl * 2u;

  // (rows past L lie outside the descriptors and read as zero: phi(0) meets G = 0 there and adds nothing)
  i16x8_t rq[4], rg[4];
  auto fetch_qg = [&](int r0) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const uint32_t grow = (uint32_t)(r0 + lrow + 32 * p);
      rq[p] = buf_load_b128(q_rs, grow * pitch_b + 16 * lp);
      rg[p] = buf_load_b128(g_rs, grow * pitch_gb + 16 * lp);
    }
  };

  // M tiles of this wave: rows d1 = 32 mt .., columns e = 32 nt0 .. and 32 (nt0 + 1) ..
  const int mt = wave >> 1, nt0 = 2 * (wave & 1);
  f32x16_t macc[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) macc[t][i] = 0.f;
  float zacc[8], bacc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    zacc[e] = 0.f;
    bacc[e] = 0.f;
  }

  const int prow = 16 * wave + l;
  uint32_t acc_off[8];        // (prow, 16 T + 4 h) in a row tile
#pragma unroll
  for (int T = 0; T < 8; ++T) acc_off[T] = lbs_off(prow, 16 * T + 4 * h);
  uint32_t g_off[4];          // (prow, 32 c + 8 h): G in B-operand order
#pragma unroll
  for (int c = 0; c < 4; ++c) g_off[c] = lbs_off(prow, 32 * c + 8 * h);
  // A operand of t^T = P G^T: row d1 = 16 T + l of sP, e = 32 c + 8 h ..: + 16 PSTR per T, + 64 bytes per c
  const char* const p_base = sP + l * PSTR + h * 16;
  // transposing reads of the M phase: rows 16 c + 8 g + (lane % 16) / 4 (+ 4), columns 32 tile + tr_col; + 4 KiB per c
  const int g2 = lane >> 5;
  const int tr_row = 8 * g2 + ((lane & 15) >> 2);
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  uint32_t ma_off[2], mb_off[2][2];
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    ma_off[hf] = lbs_off(tr_row + 4 * hf, 32 * mt + tr_col);
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) mb_off[hf][t2] = lbs_off(tr_row + 4 * hf, 32 * (nt0 + t2) + tr_col);
  }

  // dq rows leave a step late, every wave writing the 16 rows it computed (4 rows x 256 bytes per instruction), so
  // that only the wave's own order of LDS accesses matters.
  const int frow = 16 * wave + (lane >> 4);           // + 4 p
  uint32_t f_off[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) f_off[p] = lbs_off(frow + 4 * p, 8 * lp);
  i16x8_t rdq[4];
  auto flush_dq = [&](int r0) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int grow = r0 + frow + 4 * p;
      const i16x8_t o16 = *reinterpret_cast<const i16x8_t*>(sO + f_off[p]);
      // (not accumulating: the descriptor is empty and rdq reads as zero; x + 0 keeps the 16-bit value)
      i32x4_t w;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        w[j] = (int)E::pack2(E::to_float((uint16_t)o16[2 * j]) + E::to_float((uint16_t)rdq[p][2 * j]),
                             E::to_float((uint16_t)o16[2 * j + 1]) + E::to_float((uint16_t)rdq[p][2 * j + 1]));
      if (grow < row_end) *reinterpret_cast<i32x4_t*>(dqh + (size_t)grow * pitch + 8 * lp) = w;
    }
    wave_lds_fence();     // the row phase rewrites these rows of sO
  };

  fetch_qg(row_begin);
  for (int r0 = row_begin; r0 < row_end; r0 += TR) {
    // ---- tiles into LDS; db ----
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const uint32_t o = ld_off + p * 8192;
      *reinterpret_cast<i16x8_t*>(sQ + o) = rq[p];
      *reinterpret_cast<i16x8_t*>(sG + o) = rg[p];
#pragma unroll
      for (int e = 0; e < 8; ++e) bacc[e] += E::to_float((uint16_t)rg[p][e]);
    }
    __syncthreads();
    if (r0 + TR < row_end) fetch_qg(r0 + TR);
    // the previous step's dq rows leave now: what dq held was asked for a phase ago and has had time to arrive
    if (r0 > row_begin) flush_dq(r0 - TR);

    // ---- row phase ----
    {
      // (the raw rows stay packed until phi' needs them again)
      i16x4_t xraw[8];
#pragma unroll
      for (int T = 0; T < 8; ++T) xraw[T] = *reinterpret_cast<const i16x4_t*>(sQ + acc_off[T]);
      auto xv = [&](int T, int j) __attribute__((always_inline)) { return E::to_float((uint16_t)xraw[T][j]); };
      float mx = 0.f, inv = 1.f, inv_den;
      i32x2_t apk[8];         // a = phi(q), 16 bit (it is a 16-bit tensor in the reference)
      {
        float a[8][4];
        if (fmap == SLA_FMAP_SOFTMAX) {
          mx = xv(0, 0);
#pragma unroll
          for (int T = 0; T < 8; ++T)
#pragma unroll
            for (int j = 0; j < 4; ++j) mx = fmaxf(mx, xv(T, j));
          mx = fmaxf(mx, __shfl_xor(mx, 16));
          mx = fmaxf(mx, __shfl_xor(mx, 32));
          float sum = 0.f;
#pragma unroll
          for (int T = 0; T < 8; ++T)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              a[T][j] = __expf(xv(T, j) - mx);
              sum += a[T][j];
            }
          sum += __shfl_xor(sum, 16);
          sum += __shfl_xor(sum, 32);
          inv = 1.0f / sum;
#pragma unroll
          for (int T = 0; T < 8; ++T)
#pragma unroll
            for (int j = 0; j < 4; ++j) a[T][j] = round16<Tag>(a[T][j] * inv);
        } else {
#pragma unroll
          for (int T = 0; T < 8; ++T)
#pragma unroll
            for (int j = 0; j < 4; ++j) a[T][j] = fmap_pointwise<Tag>(fmap, xv(T, j));
        }
        float den = 0.f;
#pragma unroll
        for (int T = 0; T < 8; ++T) {
          const f32x4_t zz = *reinterpret_cast<const f32x4_t*>(sZ + 16 * T + 4 * h);
#pragma unroll
          for (int j = 0; j < 4; ++j) den += a[T][j] * zz[j];
        }
        den += __shfl_xor(den, 16);
        den += __shfl_xor(den, 32);
        den += 1e-5f;
        inv_den = 1.0f / den;
        // a/den takes the place of the raw row (this lane's own places)
#pragma unroll
        for (int T = 0; T < 8; ++T) {
          i32x2_t w;
          w[0] = (int)E::pack2(a[T][0] * inv_den, a[T][1] * inv_den);
          w[1] = (int)E::pack2(a[T][2] * inv_den, a[T][3] * inv_den);
          *reinterpret_cast<i32x2_t*>(sQ + acc_off[T]) = w;
          apk[T][0] = (int)E::pack2(a[T][0], a[T][1]);
          apk[T][1] = (int)E::pack2(a[T][2], a[T][3]);
        }
      }

      // t^T = P G^T: 8 tiles of 16 d1 x 16 rows
      f32x4_t t[8];
#pragma unroll
      for (int T = 0; T < 8; ++T) t[T] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const i16x8_t b = *reinterpret_cast<const i16x8_t*>(sG + g_off[c]);
#pragma unroll
        for (int T = 0; T < 8; ++T)
          t[T] = E::mfma16(*reinterpret_cast<const i16x8_t*>(p_base + T * 16 * PSTR + c * 64), b, t[T]);
      }
      float s = 0.f;
#pragma unroll
      for (int T = 0; T < 8; ++T)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t w = (uint32_t)apk[T][j >> 1];
          s += E::to_float((uint16_t)((j & 1) ? (w >> 16) : (w & 0xffff))) * t[T][j];
        }
      s += __shfl_xor(s, 16);
      s += __shfl_xor(s, 32);
      const float dden = -s * inv_den * inv_den;
      if (h == 0) sDD[prow] = -s * inv_den;     // dden * den: the weight of a/den in dz

      // da = t / den + dden z (in place), then dq = phi'(q) da
#pragma unroll
      for (int T = 0; T < 8; ++T) {
        const f32x4_t zz = *reinterpret_cast<const f32x4_t*>(sZ + 16 * T + 4 * h);
#pragma unroll
        for (int j = 0; j < 4; ++j) t[T][j] = __builtin_fmaf(t[T][j], inv_den, dden * zz[j]);
      }
      if (fmap == SLA_FMAP_RELU) {
#pragma unroll
        for (int T = 0; T < 8; ++T)
#pragma unroll
          for (int j = 0; j < 4; ++j) t[T][j] = xv(T, j) > 0.f ? t[T][j] : 0.f;
      } else if (fmap == SLA_FMAP_ELU) {
#pragma unroll
        for (int T = 0; T < 8; ++T)
#pragma unroll
          for (int j = 0; j < 4; ++j) t[T][j] = xv(T, j) > 0.f ? t[T][j] : t[T][j] * __expf(xv(T, j));
      } else {
        float dot = 0.f;
#pragma unroll
        for (int T = 0; T < 8; ++T)
#pragma unroll
          for (int j = 0; j < 4; ++j) dot += __expf(xv(T, j) - mx) * inv * t[T][j];       // the unrounded softmax
        dot += __shfl_xor(dot, 16);
        dot += __shfl_xor(dot, 32);
#pragma unroll
        for (int T = 0; T < 8; ++T)
#pragma unroll
          for (int j = 0; j < 4; ++j) t[T][j] = __expf(xv(T, j) - mx) * inv * (t[T][j] - dot);
      }
#pragma unroll
      for (int T = 0; T < 8; ++T) {
        i32x2_t w;
        w[0] = (int)E::pack2(t[T][0], t[T][1]);
        w[1] = (int)E::pack2(t[T][2], t[T][3]);
        *reinterpret_cast<i32x2_t*>(sO + acc_off[T]) = w;
      }
    }
    __syncthreads();

    // ---- M += (a/den)^T G ; dz ----
    // (what dq holds so far is asked for here, where the row phase's registers are free, and used in the next step)
#pragma unroll
    for (int p = 0; p < 4; ++p) rdq[p] = buf_load_b128(dq_rs, (uint32_t)(r0 + frow + 4 * p) * pitch_b + 16 * lp);
    __builtin_amdgcn_sched_barrier(0);      // (asked for first: the loop's next wait on memory covers these too)
#pragma unroll
    for (int c = 0; c < TR / 16; ++c) {
      const uint16_t* pa0 = reinterpret_cast<const uint16_t*>(sQ + ma_off[0] + c * 4096);
      const uint16_t* pa1 = reinterpret_cast<const uint16_t*>(sQ + ma_off[1] + c * 4096);
      const i16x8_t af = concat4(lds_read_tr16(pa0), lds_read_tr16(pa1));
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        const uint16_t* pb0 = reinterpret_cast<const uint16_t*>(sG + mb_off[0][t2] + c * 4096);
        const uint16_t* pb1 = reinterpret_cast<const uint16_t*>(sG + mb_off[1][t2] + c * 4096);
        macc[t2] = E::mfma32(af, concat4(lds_read_tr16(pb0), lds_read_tr16(pb1)), macc[t2]);
      }
    }
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int row = lrow + 32 * p;
      const uint32_t o = ld_off + p * 8192;
      const i16x8_t an = *reinterpret_cast<const i16x8_t*>(sQ + o);
      const float dd = sDD[row];
#pragma unroll
      for (int e = 0; e < 8; ++e) zacc[e] = __builtin_fmaf(dd, E::to_float((uint16_t)an[e]), zacc[e]);
    }
    __syncthreads();
  }
  flush_dq(row_begin + (row_end - 1 - row_begin) / TR * TR);

  // M^T partial [e][d1] (accumulator rows = d1, columns = e), fp32
  const size_t pidx = (size_t)bh * nsplit + split;
  float* mo = m_part + pidx * D * D;
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2) {
    const int col = 32 * (nt0 + t2) + (lane & 31);
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const f32x4_t v4 = {macc[t2][4 * i4], macc[t2][4 * i4 + 1], macc[t2][4 * i4 + 2], macc[t2][4 * i4 + 3]};
      *reinterpret_cast<f32x4_t*>(mo + (size_t)col * D + 32 * mt + 8 * i4 + 4 * g2) = v4;
    }
  }
  // (the loop's last barrier has passed: sQ is free)
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    sRed[0][lrow][8 * lp + e] = zacc[e];
    sRed[1][lrow][8 * lp + e] = bacc[e];
  }
  __syncthreads();
  if (tid < D) {
    float s0 = 0.f, s1 = 0.f;
#pragma unroll 8
    for (int rr = 0; rr < 32; ++rr) {
      s0 += sRed[0][rr][tid];
      s1 += sRed[1][rr][tid];
    }
    dz_part[pidx * D + tid] = s0;
    db_part[pidx * D + tid] = s1;
  }
}

// Key side of the same backward, head dim 128: dv = c dS, dc = v dS^T + dz, dk = phi'(k) dc with c = phi(k).
// grid (slices of L, heads), 8 waves; dS [d1][d2] and dS^T [d2][d1] (16 bit, rows padded by 16 bytes) and dz stay in LDS,
// every wave walks its own 16-key tiles of the slice and never meets another wave after the staging barrier:
//   rows of k, v (fetched a tile ahead) -> two wave-private swizzled 4 KB tiles; phi(k) takes the place of k;
//   dv^T = dS^T c^T and dc^T = dS v^T as 16x16x32 products (a key's row spread over 4 lanes, B operands read row-wise
//   from the wave's tiles); dk, dv go back over the tiles and leave as whole rows, added to what dk, dv held (asked
//   for at the start of the tile) when accumulating.
template <typename Tag, int FMAP>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void linear_bwd_keys_kernel(
    const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, const uint16_t* __restrict__ ds,
    const uint16_t* __restrict__ dst, const float* __restrict__ dz, uint16_t* __restrict__ dk, uint16_t* __restrict__ dv,
    const RowLayout lin, int L, int rows_per_split, int accumulate) {
  using E = Elem<Tag>;
  constexpr int fmap = FMAP;
  constexpr int D = 128;
  constexpr int PSTR = D * 2 + 16;               // row pitch of the staged matrices
  constexpr int WT = 16 * D * 2;                 // bytes of a wave's tile
  __shared__ __attribute__((aligned(16))) char smem[2 * D * PSTR + D * 4 + 8 * 2 * WT];
  char* const sDS = smem;                        // dS   [d1][d2]: A operand of dc^T = dS v^T
  char* const sDST = smem + D * PSTR;            // dS^T [d2][d1]: A operand of dv^T = dS^T c^T
  float* const sDZ = reinterpret_cast<float*>(smem + 2 * D * PSTR);

  const int split = blockIdx.x, bh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  char* const tK = smem + 2 * D * PSTR + D * 4 + wave * 2 * WT;    // k rows, then phi(k), then dk
  char* const tV = tK + WT;                                          // v rows, then dv
  const int row_begin = split * rows_per_split;
  const int row_end = min(L, row_begin + rows_per_split);
  {
    const uint16_t* s0 = ds + (size_t)bh * D * D;
    const uint16_t* s1 = dst + (size_t)bh * D * D;
    for (int idx = tid; idx < D * D / 8; idx += 512) {
      const int row = idx / (D / 8), col = (idx % (D / 8)) * 8;
      *reinterpret_cast<i16x8_t*>(sDS + row * PSTR + col * 2) = *reinterpret_cast<const i16x8_t*>(s0 + (size_t)row * D + col);
      *reinterpret_cast<i16x8_t*>(sDST + row * PSTR + col * 2) = *reinterpret_cast<const i16x8_t*>(s1 + (size_t)row * D + col);
    }
    if (tid < D) sDZ[tid] = dz[(size_t)bh * D + tid];
  }
  __syncthreads();

  const uint32_t range = lin.head_range_bytes(L, D);
  const __amdgpu_buffer_rsrc_t k_rs = make_rsrc(k + lin.head(bh), range);
  const __amdgpu_buffer_rsrc_t v_rs = make_rsrc(v + lin.head(bh), range);
  const __amdgpu_buffer_rsrc_t dk_rs = make_rsrc(dk + lin.head(bh), accumulate ? range : 0u);
  const __amdgpu_buffer_rsrc_t dv_rs = make_rsrc(dv + lin.head(bh), accumulate ? range : 0u);
  uint16_t* const dkh = dk + lin.head(bh);
  uint16_t* const dvh = dv + lin.head(bh);
  const size_t pitch = (size_t)lin.sl;
  const uint32_t pitch_b = (uint32_t)lin.sl * 2u;

  // loader / writer layout of a wave's tile: lane -> row lane / 16 + 4 p, 16-byte piece lane % 16
  const int frow = lane >> 4, lp = lane & 15;
  uint32_t f_off[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) f_off[p] = lbs_off(frow + 4 * p, 8 * lp);
  // product layout: lane = (key l of the tile's 16, quarter h): d = 16 T + 4 h + j
  const int l = lane & 15, h = lane >> 4;
  uint32_t acc_off[8];        // (l, 16 T + 4 h)
#pragma unroll
  for (int T = 0; T < 8; ++T) acc_off[T] = lbs_off(l, 16 * T + 4 * h);
  uint32_t b_off[4];          // (l, 32 c + 8 h): B-operand order
#pragma unroll
  for (int c = 0; c < 4; ++c) b_off[c] = lbs_off(l, 32 * c + 8 * h);
  const uint32_t a_base = (uint32_t)l * PSTR + (uint32_t)h * 16u;     // row 16 T + l of a staged matrix: + 16 PSTR per T, + 64 per c

  i16x8_t rk[4], rv[4];
  auto fetch_kv = [&](int r0) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const uint32_t o = (uint32_t)(r0 + frow + 4 * p) * pitch_b + 16 * lp;      // rows past L read as zero
      rk[p] = buf_load_b128(k_rs, o);
      rv[p] = buf_load_b128(v_rs, o);
    }
  };
  const int first = row_begin + 16 * wave;
  if (first < row_end) fetch_kv(first);
  for (int r0 = first; r0 < row_end; r0 += 128) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      *reinterpret_cast<i16x8_t*>(tK + f_off[p]) = rk[p];
      *reinterpret_cast<i16x8_t*>(tV + f_off[p]) = rv[p];
    }
    wave_lds_fence();
    // what dk, dv hold (for this tile) and the next tile's rows: both have the whole tile to arrive
    i16x8_t rdk[4], rdv[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const uint32_t o = (uint32_t)(r0 + frow + 4 * p) * pitch_b + 16 * lp;
      rdk[p] = buf_load_b128(dk_rs, o);
      rdv[p] = buf_load_b128(dv_rs, o);
    }
    if (r0 + 128 < row_end) fetch_kv(r0 + 128);

    i16x4_t xraw[8];
#pragma unroll
    for (int T = 0; T < 8; ++T) xraw[T] = *reinterpret_cast<const i16x4_t*>(tK + acc_off[T]);
    auto xv = [&](int T, int j) __attribute__((always_inline)) { return E::to_float((uint16_t)xraw[T][j]); };
    float mx = 0.f, inv = 1.f;
    {
      float a[8][4];
      if (fmap == SLA_FMAP_SOFTMAX) {
        mx = xv(0, 0);
#pragma unroll
        for (int T = 0; T < 8; ++T)
#pragma unroll
          for (int j = 0; j < 4; ++j) mx = fmaxf(mx, xv(T, j));
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        float sum = 0.f;
#pragma unroll
        for (int T = 0; T < 8; ++T)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            a[T][j] = __expf(xv(T, j) - mx);
            sum += a[T][j];
          }
        sum += __shfl_xor(sum, 16);
        sum += __shfl_xor(sum, 32);
        inv = 1.0f / sum;
#pragma unroll
        for (int T = 0; T < 8; ++T)
#pragma unroll
          for (int j = 0; j < 4; ++j) a[T][j] = round16<Tag>(a[T][j] * inv);
      } else {
#pragma unroll
        for (int T = 0; T < 8; ++T)
#pragma unroll
          for (int j = 0; j < 4; ++j) a[T][j] = fmap_pointwise<Tag>(fmap, xv(T, j));
      }
      // c = phi(k) over the raw rows (this lane's own places; a key's gradients depend on its own row only, so rows
      // past the end, which are never written, need no care)
#pragma unroll
      for (int T = 0; T < 8; ++T) {
        i32x2_t w;
        w[0] = (int)E::pack2(a[T][0], a[T][1]);
        w[1] = (int)E::pack2(a[T][2], a[T][3]);
        *reinterpret_cast<i32x2_t*>(tK + acc_off[T]) = w;
      }
    }
    wave_lds_fence();
    // dv^T = dS^T c^T ; dc^T = dS v^T
    f32x4_t dva[8], dca[8];
#pragma unroll
    for (int T = 0; T < 8; ++T) {
      dva[T] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      dca[T] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const i16x8_t cf = *reinterpret_cast<const i16x8_t*>(tK + b_off[c]);
      const i16x8_t vf = *reinterpret_cast<const i16x8_t*>(tV + b_off[c]);
#pragma unroll
      for (int T = 0; T < 8; ++T) {
        dva[T] = E::mfma16(*reinterpret_cast<const i16x8_t*>(sDST + a_base + T * 16 * PSTR + c * 64), cf, dva[T]);
        dca[T] = E::mfma16(*reinterpret_cast<const i16x8_t*>(sDS + a_base + T * 16 * PSTR + c * 64), vf, dca[T]);
      }
    }
    wave_lds_fence();      // (the tiles are rewritten below: every read of them above comes first)
    // dc += dz ; dk = phi'(k) dc
#pragma unroll
    for (int T = 0; T < 8; ++T) {
      const f32x4_t zz = *reinterpret_cast<const f32x4_t*>(sDZ + 16 * T + 4 * h);
#pragma unroll
      for (int j = 0; j < 4; ++j) dca[T][j] += zz[j];
    }
    if (fmap == SLA_FMAP_RELU) {
#pragma unroll
      for (int T = 0; T < 8; ++T)
#pragma unroll
        for (int j = 0; j < 4; ++j) dca[T][j] = xv(T, j) > 0.f ? dca[T][j] : 0.f;
    } else if (fmap == SLA_FMAP_ELU) {
#pragma unroll
      for (int T = 0; T < 8; ++T)
#pragma unroll
        for (int j = 0; j < 4; ++j) dca[T][j] = xv(T, j) > 0.f ? dca[T][j] : dca[T][j] * __expf(xv(T, j));
    } else {
      float dot = 0.f;
#pragma unroll
      for (int T = 0; T < 8; ++T)
#pragma unroll
        for (int j = 0; j < 4; ++j) dot += __expf(xv(T, j) - mx) * inv * dca[T][j];       // the unrounded softmax
      dot += __shfl_xor(dot, 16);
      dot += __shfl_xor(dot, 32);
#pragma unroll
      for (int T = 0; T < 8; ++T)
#pragma unroll
        for (int j = 0; j < 4; ++j) dca[T][j] = __expf(xv(T, j) - mx) * inv * (dca[T][j] - dot);
    }
#pragma unroll
    for (int T = 0; T < 8; ++T) {
      i32x2_t wk, wv;
      wk[0] = (int)E::pack2(dca[T][0], dca[T][1]);
      wk[1] = (int)E::pack2(dca[T][2], dca[T][3]);
      wv[0] = (int)E::pack2(dva[T][0], dva[T][1]);
      wv[1] = (int)E::pack2(dva[T][2], dva[T][3]);
      *reinterpret_cast<i32x2_t*>(tK + acc_off[T]) = wk;
      *reinterpret_cast<i32x2_t*>(tV + acc_off[T]) = wv;
    }
    wave_lds_fence();
    // whole rows out: 16-bit value + what the tensor held, one rounded add (nothing held when not accumulating)
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int grow = r0 + frow + 4 * p;
      const i16x8_t k16 = *reinterpret_cast<const i16x8_t*>(tK + f_off[p]);
      const i16x8_t v16 = *reinterpret_cast<const i16x8_t*>(tV + f_off[p]);
      i32x4_t wk, wv;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wk[j] = (int)E::pack2(E::to_float((uint16_t)k16[2 * j]) + E::to_float((uint16_t)rdk[p][2 * j]),
                              E::to_float((uint16_t)k16[2 * j + 1]) + E::to_float((uint16_t)rdk[p][2 * j + 1]));
        wv[j] = (int)E::pack2(E::to_float((uint16_t)v16[2 * j]) + E::to_float((uint16_t)rdv[p][2 * j]),
                              E::to_float((uint16_t)v16[2 * j + 1]) + E::to_float((uint16_t)rdv[p][2 * j + 1]));
      }
      if (grow < row_end) {
        *reinterpret_cast<i32x4_t*>(dkh + (size_t)grow * pitch + 8 * lp) = wk;
        *reinterpret_cast<i32x4_t*>(dvh + (size_t)grow * pitch + 8 * lp) = wv;
      }
    }
    wave_lds_fence();      // the next tile's rows go over these
  }
}

// Sums of the slices' partials in ascending slice order: M per head (fp32, both orientations), dz, db per head.
// grid (cdiv(D*D, 256), BH).
__global__ __launch_bounds__(256) void linear_bwd_sum_kernel(const float* __restrict__ m_part, const float* __restrict__ dz_part,
                                                             const float* __restrict__ db_part, float* __restrict__ mt_head,
                                                             float* __restrict__ m_head, float* __restrict__ dz,
                                                             float* __restrict__ db_head, int nsplit, int D) {
  const int DD = D * D;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int bh = blockIdx.y;
  if (i < DD) {
    const float* p = m_part + (size_t)bh * nsplit * DD + i;
    float s = 0.f;
#pragma unroll 8
    for (int sp = 0; sp < nsplit; ++sp) s += p[(size_t)sp * DD];
    mt_head[(size_t)bh * DD + i] = s;                               // M^T [e][d1]
    m_head[(size_t)bh * DD + (size_t)(i % D) * D + i / D] = s;      // M   [d1][e]
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

// Per head, from M (fp32, both orientations):
//   dS[d1][d2]    = sum_e  M^T[e][d1] * round16(W[e][d2])    -> ds [d1][d2] and dst [d2][d1], 16 bit
//   dW^T[d2][e]   = sum_d1 M[d1][e] * S[d1][d2]              -> dw_head [d2][e], fp32  (S^T = kvt[d2][d1], 16 bit)
// grid (D*D/256, BH, 2): z = 0 forms dS, z = 1 forms dW.  Ascending order of the summed index; a workgroup's threads
// share the first factor and read the second side by side.
template <typename Tag>
__global__ __launch_bounds__(256) void linear_bwd_products_kernel(const float* __restrict__ mt_head,
                                                                  const float* __restrict__ m_head,
                                                                  const float* __restrict__ weight,
                                                                  const uint16_t* __restrict__ kvt, uint16_t* __restrict__ ds,
                                                                  uint16_t* __restrict__ dst, float* __restrict__ dw_head,
                                                                  int D) {
  using E = Elem<Tag>;
  const int DD = D * D;
  const int bh = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= DD) return;
  if (blockIdx.z == 0) {
    const int d1 = i / D, d2 = i % D;
    const float* m = mt_head + (size_t)bh * DD + d1;
    const float* w = weight + d2;
    float acc = 0.f;
    for (int e0 = 0; e0 < D; e0 += 16) {       // (16 pairs of loads in flight, then their products in order)
      float a[16], b[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        a[j] = m[(size_t)(e0 + j) * D];
        b[j] = w[(size_t)(e0 + j) * D];
      }
#pragma unroll
      for (int j = 0; j < 16; ++j) acc = __builtin_fmaf(a[j], round16<Tag>(b[j]), acc);
    }
    const uint16_t hv = E::from_float(acc);
    ds[(size_t)bh * DD + i] = hv;
    dst[(size_t)bh * DD + (size_t)d2 * D + d1] = hv;
  } else {
    const int d2 = i / D, e = i % D;
    const uint16_t* s = kvt + (size_t)bh * DD + (size_t)d2 * D;
    const float* m = m_head + (size_t)bh * DD + e;
    float acc = 0.f;
    for (int d0 = 0; d0 < D; d0 += 16) {
      float a[16];
      const i16x8_t s0 = *reinterpret_cast<const i16x8_t*>(s + d0), s1 = *reinterpret_cast<const i16x8_t*>(s + d0 + 8);
#pragma unroll
      for (int j = 0; j < 16; ++j) a[j] = m[(size_t)(d0 + j) * D];
#pragma unroll
      for (int j = 0; j < 16; ++j) acc = __builtin_fmaf(a[j], E::to_float((uint16_t)(j < 8 ? s0[j] : s1[j - 8])), acc);
    }
    dw_head[(size_t)bh * DD + i] = acc;      // [d][e] with d = d2: the layout linear_bwd_reduce_heads_kernel adds up
  }
}

}  // namespace sla
