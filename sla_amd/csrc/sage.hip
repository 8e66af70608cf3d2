// SageSLA quantised forward for gfx950: INT8 QK^T and FP8 (e4m3) PV on the matrix cores.
//
// Stands in for the third-party calls of SageSLA/core.py:102-144 of the reference
// (spas_sage_attn get_vanilla_qk_quant, block_map_lut_triton, transpose_pad_permute_cuda,
// scale_fuse_quant_cuda, qk_int8_sv_f8_*): that extension is not part of the reference tree,
// so the scheme below follows its published description, not its code:
//   q_int8 = rint(q / sq), sq = max|q| / 127 over each block of BLKQ rows;
//   k_int8 = rint((k - mean_L k) / sk), sk per block of BLKK rows;
//   v_fp8  = e4m3(v / sv), sv[d] = max_L |v[:, d]| / v_range (448 by default; the reference's call passes 2.25);
//   S = (q_int8 . k_int8) * sq * sk * scale ; P = softmax numerators over the selected blocks ;
//   O = (e4m3(c P) . v_fp8) * sv / sum(e4m3(c P)), c = 112 with P <= 4 (reference maximum lagging by <= 2).
// The look-up table of the bf16 path is used as is (no delta encoding is needed here).
#include "common.h"
#include "sage_steps.h"

namespace sla {

int64_t k_colmean_scratch_floats(int BH, int L, int D);
void launch_k_colmean(const void* k, const RowLayout& lay, int dtype, int BH, int L, int D, float* scratch, void* colmean,
                      hipStream_t st);
void launch_map_from_pooled(int dtype, const void* pq, const void* pk, void* score, int BH, int M, int N, int D, int topk,
                            int8_t* sparse_map, void* lut, int lut64, hipStream_t st);

// ---- INT8 block quantisation ----------------------------------------------------------------
// One workgroup per (block, bh).  SUB_MEAN: subtract the per-head column mean first.
// POOL: also write the block mean the mask builder needs (of x, or of x - colmean rounded to 16 bit, as
// get_block_map pools it: utils.py:55-58 of the reference), summed row by row in fp32 and divided once,
// exactly as the pooling kernel of the mask builder does, so the block is read from memory once for both.
template <typename Tag, int D, int BLK, bool SUB_MEAN, bool POOL>
__global__ __launch_bounds__(256) void quant_int8_kernel(const uint16_t* __restrict__ x, const RowLayout lay,
                                                         const uint16_t* __restrict__ colmean, int8_t* __restrict__ xq,
                                                         float* __restrict__ scale, uint16_t* __restrict__ pooled, int L,
                                                         int nblk) {
  using E = Elem<Tag>;
  constexpr int CPR = D / 8;
  constexpr int RPP = 256 / CPR;
  constexpr int NP = BLK / RPP;
  constexpr int TSTR = D + 8;
  __shared__ float sred[4];
  __shared__ __attribute__((aligned(16))) uint16_t tile[POOL ? BLK * TSTR : 8];
  const int blk = blockIdx.x, bh = blockIdx.y;
  const int tid = threadIdx.x;
  const int lrow = tid / CPR, lcol = (tid % CPR) * 8;
  float cm[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) cm[e] = 0.f;
  if (SUB_MEAN) {
    const i16x8_t m = *reinterpret_cast<const i16x8_t*>(colmean + (size_t)bh * D + lcol);
#pragma unroll
    for (int e = 0; e < 8; ++e) cm[e] = E::to_float((uint16_t)m[e]);
  }
  // every row of the block is asked for before the first is used (rows past L lie outside the descriptor and read as
  // zero): one memory latency per block instead of one per row group
  const __amdgpu_buffer_rsrc_t xb = make_rsrc(x + lay.head(bh), lay.head_range_bytes(L, D));
  i16x8_t raw[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p)
    raw[p] = buf_load_b128(xb, (uint32_t)(blk * BLK + lrow + p * RPP) * (uint32_t)(lay.sl * 2) + (uint32_t)lcol * 2u);
  float val[NP][8];
  float amax = 0.f;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int grow = blk * BLK + lrow + p * RPP;
    i16x8_t v = raw[p];
    const bool ok = grow < L;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      val[p][e] = ok ? E::to_float((uint16_t)v[e]) - cm[e] : 0.f;
      amax = fmaxf(amax, fabsf(val[p][e]));
    }
    if (POOL) {
      if (SUB_MEAN) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (short)E::from_float(val[p][e]);
      }
      *reinterpret_cast<i16x8_t*>(&tile[(lrow + p * RPP) * TSTR + lcol]) = v;
    }
  }
#pragma unroll
  for (int s = 1; s < 64; s <<= 1) amax = fmaxf(amax, __shfl_xor(amax, s));
  if ((tid & 63) == 0) sred[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(sred[0], sred[1]), fmaxf(sred[2], sred[3]));
  const float sc = fmaxf(amax, 1e-30f) / 127.0f;
  if (tid == 0) scale[(size_t)bh * nblk + blk] = sc;
  const float inv_sc = 1.0f / sc;
  if (POOL && tid < D) {   // one column per thread (the barrier above also covers the tile)
    const int nrows = min(BLK, L - blk * BLK);
    float acc = 0.f;
    // rows are read sixteen at a time (all reads of a batch in flight together), then added in row order
    constexpr int BATCH = 16;
    int r = 0;
    for (; r + BATCH <= nrows; r += BATCH) {
      uint16_t t[BATCH];
#pragma unroll
      for (int i = 0; i < BATCH; ++i) t[i] = tile[(r + i) * TSTR + tid];
#pragma unroll
      for (int i = 0; i < BATCH; ++i) acc = acc + E::to_float(t[i]);
    }
    for (; r < nrows; ++r) acc = acc + E::to_float(tile[r * TSTR + tid]);
    pooled[((size_t)bh * nblk + blk) * D + tid] = E::from_float(acc / (float)nrows);
  }
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int grow = blk * BLK + lrow + p * RPP;
    if (grow >= L) continue;
    i32x2_t w;
    int8_t* b = reinterpret_cast<int8_t*>(&w);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      // round(val / sc) through the reciprocal: the product is within two units in the last place of the quotient
      // (< 3e-5 for |quotient| <= 127), so both round to the same integer unless the product lies that close to a
      // half-integer; those few elements take the division itself.
      const float t = val[p][e] * inv_sc;
      float r = rintf(t);
      if (fabsf(t - r) > 0.4999f) r = rintf(val[p][e] / sc);
      r = fminf(fmaxf(r, -127.f), 127.f);
      b[e] = (int8_t)(int)r;
    }
    *reinterpret_cast<i32x2_t*>(xq + ((size_t)bh * L + grow) * D + lcol) = w;
  }
}

// ---- FP8 per-channel quantisation of V ------------------------------------------------------
// pass 1: per (chunk of 256 rows, bh) column abs-max -> partial; pass 2: reduce partials;
// pass 3: v_fp8 = e4m3(v / scale).
template <typename Tag, int D>
__global__ __launch_bounds__(256) void v_amax_partial_kernel(const uint16_t* __restrict__ v, const RowLayout lay,
                                                             float* __restrict__ part, int L, int rows_per_chunk) {
  using E = Elem<Tag>;
  constexpr int CPR = D / 8;
  constexpr int RPP = 256 / CPR;
  __shared__ float sm[RPP][D];
  const int chunk = blockIdx.x, bh = blockIdx.y, nchunk = gridDim.x;
  const int tid = threadIdx.x;
  const int lrow = tid / CPR, lcol = (tid % CPR) * 8;
  const int r_end = min(L, (chunk + 1) * rows_per_chunk);
  float am[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) am[e] = 0.f;
  for (int row = chunk * rows_per_chunk + lrow; row < r_end; row += RPP) {
    const i16x8_t x = *reinterpret_cast<const i16x8_t*>(v + lay.head(bh) + (size_t)row * (size_t)lay.sl + lcol);
#pragma unroll
    for (int e = 0; e < 8; ++e) am[e] = fmaxf(am[e], fabsf(E::to_float((uint16_t)x[e])));
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) sm[lrow][lcol + e] = am[e];
  __syncthreads();
  if (tid < D) {
    float a = 0.f;
#pragma unroll
    for (int r = 0; r < RPP; ++r) a = fmaxf(a, sm[r][tid]);
    part[((size_t)bh * nchunk + chunk) * D + tid] = a;
  }
}

// grid (D / 16, BH), 256 threads: thread (cg, c) = (tid / 16, tid % 16) takes the maximum of column 16 blockIdx.x + c
// over chunks cg, cg + 16, ...; the 16 partial maxima per column meet in LDS.  (Small workgroups: the launch has to
// find room beside the memory-bound kernels of the other stream.)
__global__ __launch_bounds__(256) void v_scale_kernel(const float* __restrict__ part, float* __restrict__ v_scale, int nchunk,
                                                     int D, float v_range) {
  __shared__ float sm[256];
  const int bh = blockIdx.y, tid = threadIdx.x;
  const int d = blockIdx.x * 16 + (tid & 15), cg = tid >> 4;
  float a = 0.f;
  for (int c = cg; c < nchunk; c += 16) a = fmaxf(a, part[((size_t)bh * nchunk + c) * D + d]);
  sm[tid] = a;
  __syncthreads();
  if (tid < 16) {
    for (int j = 1; j < 16; ++j) a = fmaxf(a, sm[j * 16 + tid]);
    v_scale[(size_t)bh * D + d] = fmaxf(a, 1e-30f) / v_range;
  }
}

static __device__ __forceinline__ uint32_t cvt4_fp8(float a, float b, float c, float d) {
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return (uint32_t)w;
}

template <typename Tag, int D>
__global__ __launch_bounds__(256) void v_quant_fp8_kernel(const uint16_t* __restrict__ v, const RowLayout lay,
                                                          const float* __restrict__ v_scale, uint8_t* __restrict__ v8, int L) {
  using E = Elem<Tag>;
  constexpr int CPR = D / 8;
  constexpr int RPP = 256 / CPR;
  const int bh = blockIdx.y;
  const int row = blockIdx.x * RPP + threadIdx.x / CPR;
  const int lcol = (threadIdx.x % CPR) * 8;
  if (row >= L) return;
  const i16x8_t x = *reinterpret_cast<const i16x8_t*>(v + lay.head(bh) + (size_t)row * (size_t)lay.sl + lcol);
  float f[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = E::to_float((uint16_t)x[e]) / v_scale[(size_t)bh * D + lcol + e];
  i32x2_t w;
  w[0] = (int)cvt4_fp8(f[0], f[1], f[2], f[3]);
  w[1] = (int)cvt4_fp8(f[4], f[5], f[6], f[7]);
  *reinterpret_cast<i32x2_t*>(v8 + ((size_t)bh * L + row) * D + lcol) = w;
}

// ---- quantised block-sparse attention ----------------------------------------------------------
typedef __attribute__((address_space(3))) i32x2_t lds_i32x2_t;

// One workgroup per query block of BLKQ rows, one wave per 32 queries, two waves per SIMD.
// S^T = K8 Q8^T with v_mfma_i32_32x32x32_i8 (exact), dequantised by sq*sk*scale*log2(e) inside the exponent's
// FMA.  Both 32-key halves of a tile are exponentiated against one reference maximum and packed to e4m3: the
// 32 probabilities a lane then holds are, as they stand, its B operand of ONE v_mfma_f32_32x32x64_f8f6f4 per
// 32 output channels (O^T += V8^T P^T, contraction over all 64 keys of the tile); V^T fragments come from the
// row-major V tile with the transposing 8-bit LDS read, whose row addresses follow the accumulator's key order.
// The reference maximum only moves when a tile's maximum exceeds it by more than TAU = 2 (log2 units), so
// probabilities are at most 4; they are scaled by 112 = 448/4 to use the e4m3 range.
// K/V tiles: global -> registers -> LDS, double-buffered in LDS: the next tile is in flight during the whole
// current one and there is one barrier per tile.
template <typename OutTag, int D, int BLKQ>
__global__ __launch_bounds__(BLKQ * 2) __attribute__((amdgpu_waves_per_eu(2, 2))) void sage_fwd_kernel(
    const int8_t* __restrict__ q8, const float* __restrict__ q_scale, const int8_t* __restrict__ k8,
    const float* __restrict__ k_scale, const uint8_t* __restrict__ v8, const float* __restrict__ v_scale,
    const void* __restrict__ lut, int lut64, uint16_t* __restrict__ o, int L, int Mblk, int Nblk, int topk,
    float scale_log2e, int total) {
  using EO = Elem<OutTag>;
  constexpr int BLKK = 64;
  constexpr int NT = BLKQ * 2;
  constexpr int QC = D / 32;                // 32-wide int8 contraction chunks
  constexpr int DT = D / 32;                // 32-row tiles of O^T
  constexpr int STR = D + 16;               // bytes per LDS row
  constexpr int CPR = D / 16;               // 16-byte chunks per row
  constexpr int NLD = (BLKK * CPR + NT - 1) / NT;
  constexpr float TAU = 2.0f;
  // probabilities are scaled by 112 = 448 / 2^TAU, applied as an offset of the exponent
  constexpr float LOG2_P_SCALE = 6.807354922057604f;

  __shared__ __attribute__((aligned(16))) uint8_t sK[2][BLKK * STR];   // K of tile i lives in slot i % 2
  __shared__ __attribute__((aligned(16))) uint8_t sV[3][BLKK * STR];   // V of tile i lives in slot i % 3

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int bh = logical / Mblk;
  const int mb = logical - bh * Mblk;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;

  const size_t head_off = (size_t)bh * L * D;
  const uint32_t head_bytes = (uint32_t)L * D;
  const __amdgpu_buffer_rsrc_t qh = make_rsrc(q8 + head_off, head_bytes);
  const __amdgpu_buffer_rsrc_t kh = make_rsrc(k8 + head_off, head_bytes);
  const __amdgpu_buffer_rsrc_t vh = make_rsrc(v8 + head_off, head_bytes);
  const int qrow = mb * BLKQ + wave * 32 + r;
  i32x4_t qf[QC];
#pragma unroll
  for (int c = 0; c < QC; ++c)
    qf[c] = __builtin_bit_cast(i32x4_t, buf_load_b128(qh, (uint32_t)qrow * D + 32 * c + 16 * g));   // rows past L: 0
  const float qs = q_scale[(size_t)bh * Mblk + mb] * scale_log2e;
  const float* ksc = k_scale + (size_t)bh * Nblk;

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
      const int row = idx / CPR, col = (idx % CPR) * 16;
      // chunks past the tile (when the tile does not divide among the threads) and rows past L read as zero
      const uint32_t off = idx < BLKK * CPR ? (uint32_t)(nb * BLKK + row) * D + col : 0xfffffff0u;
      kreg[i] = buf_load_b128(kh, off);
      vreg[i] = buf_load_b128(vh, off);
    }
  };
  auto store_tile = [&](int kslot, int vslot) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int idx = tid + i * NT;
      if (idx < BLKK * CPR) {
        const int row = idx / CPR, col = (idx % CPR) * 16;
        *reinterpret_cast<i16x8_t*>(&sK[kslot][row * STR + col]) = kreg[i];
        *reinterpret_cast<i16x8_t*>(&sV[vslot][row * STR + col]) = vreg[i];
      }
    }
  };

  f32x16_t oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;
  float m_used = -INFINITY;   // reference maximum (log2 units)
  // Row sums of the e4m3 probabilities come from the matrix core as well: an A operand of ones makes every
  // row of this accumulator the sum over all 64 keys of a tile, so each lane holds l of its query column
  // (numerator and denominator then see the same rounded probabilities, and no vector-ALU adds are spent).
  f32x16_t lacc;
#pragma unroll
  for (int i = 0; i < 16; ++i) lacc[i] = 0.f;
  i32x8_t ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = 0x38383838;   // e4m3 1.0 in every byte

  // transposed 8-bit read: lane i of a 16-lane group passes the address of (row i/2, 8 bytes at
  // column 8*(i%2)) and receives column i of the 8x16 tile.  Row i/2 is mapped to the key that
  // accumulator slot i/2 of the probabilities holds: keys 4g+{0..3} and 8+4g+{0..3} of a 16-key chunk.
  const int li = lane & 15;
  const int slot = li >> 1;
  const int tr_key = 8 * (slot >> 2) + 4 * g + (slot & 3);
  const int tr_col = 16 * ((lane >> 4) & 1) + 8 * (li & 1);

  // The integer products start from the bit pattern of the float 1.5 * 2^23 instead of from zero: the integer
  // MAGIC + s, read as a float, IS the float 12582912 + s (|s| <= 128 * 127^2 < 2^22 stays inside the binade whose
  // unit in the last place is 1), so the scores reach the exponent's multiply-add without an int -> float
  // conversion per element; 12582912 * sc joins the constant that multiply-add subtracts.
  constexpr int MAGIC = 0x4B400000;
  constexpr float MAGIC_F = 12582912.0f;
  i32x16_t magic;
#pragma unroll
  for (int i = 0; i < 16; ++i) magic[i] = MAGIC;
  // S^T of one tile: MAGIC + raw int32 products of both 32-key halves
  auto scores = [&](int kslot, i32x16_t (&acc)[2]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int c = 0; c < QC; ++c) {
        const i32x4_t a = *reinterpret_cast<const i32x4_t*>(&sK[kslot][(32 * t + r) * STR + 32 * c + 16 * g]);
        acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, qf[c], c == 0 ? magic : acc[t], 0, 0, 0);
      }
    }
  };
  // softmax numerators of one tile (scores acc, dequantisation factor sc, kv_valid existing key rows),
  // packed to e4m3 in the B-operand order of the 64-key product
  auto probabilities = [&](const i32x16_t (&acc)[2], float sc, int kv_valid) -> i32x8_t {
    float s[2][16];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[t][i] = __int_as_float(acc[t][i]);         // = 12582912 + score
    if (kv_valid < BLKK) {                 // ragged last key block: missing rows take no part
      const int lim = kv_valid - 4 * g;    // key index of register i is 32t + 8(i/4) + i%4 + 4g
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (32 * t + 8 * (i >> 2) + (i & 3) >= lim) s[t][i] = -INFINITY;
    }
    // raw maximum of this lane's 32 scores (sc > 0, so the maximum commutes with the scaling)
    float mx = s[0][0];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[t][i]);
    mx -= MAGIC_F;                         // (exact: both are integers below 2^24)
    if (__any(mx * sc > m_used + TAU)) {   // rare: move the reference and rescale what is accumulated
      float m_new = fmaxf(mx, __shfl_xor(mx, 32)) * sc;
      m_new = fmaxf(m_used, m_new);
      const float f = fast_exp2(m_used - m_new);     // 0 on the first tile
      m_used = m_new;
#pragma unroll
      for (int i = 0; i < 16; ++i) lacc[i] *= f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dt][i] *= f;
    }
    // 112 p = exp2(s*sc - (m_used - log2 112)); -inf scores give exactly 0
    const float m_off = __builtin_fmaf(MAGIC_F, sc, m_used - LOG2_P_SCALE);
    i32x8_t pb;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        float pv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) pv[j] = fast_exp2(__builtin_fmaf(s[t][4 * i4 + j], sc, -m_off));
        pb[4 * t + i4] = (int)cvt4_fp8(pv[0], pv[1], pv[2], pv[3]);
      }
    return pb;
  };
  // l += sum_keys P ; O^T += V8^T P^T: one 64-key product per 32 output channels
  auto accumulate = [&](int vslot, const i32x8_t& pb) {
    // formats 0/0 = e4m3 for both operands, block scales 2^0
    lacc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ones, pb, lacc, 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      i32x8_t a;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {
          const int key = 32 * t + 16 * c2 + tr_key;
          const i32x2_t x = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2_t*)&sV[vslot][key * STR + 32 * dt + tr_col]);
          a[4 * t + 2 * c2] = x[0];
          a[4 * t + 2 * c2 + 1] = x[1];
        }
      oacc[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, pb, oacc[dt], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
    }
  };

  // Software pipeline over the selected tiles: step i issues the int8 products of tile i, then does the
  // exponentials of tile i-1 on the vector ALU while the matrix core works, then issues the fp8 products
  // of tile i-1.  Tile i+1 is in flight from global memory during the whole step.
  int nb = topk > 0 ? lut_at(0) : 0;
  int nb_next = topk > 1 ? lut_at(1) : 0;
  if (topk > 0) {
    load_tile(nb);
    store_tile(0, 0);
  }
  __syncthreads();
  i32x16_t acc_a[2], acc_b[2];              // scores of even / odd steps (ping-pong, no copies)
  float sc_prev = 0.f;
  int valid_prev = BLKK;
  int vslot_prev = 0, vslot = 0;
  auto step = [&](int it, i32x16_t (&acc)[2], const i32x16_t (&acc_prev)[2]) {
    const int kv_valid = L - nb * BLKK;
    // an all-zero block has scale 1e-30/127; the floor keeps -inf * sc = -inf (never NaN) for masked rows
    const float sc = fmaxf(qs * ksc[nb], 1e-37f);
    const bool more = it + 1 < topk;
    if (more) {
      nb = nb_next;
      nb_next = it + 2 < topk ? lut_at(it + 2) : 0;
      load_tile(nb);
    }
    scores(it & 1, acc);
    if (it > 0) {
      const i32x8_t pb = probabilities(acc_prev, sc_prev, valid_prev);
      accumulate(vslot_prev, pb);
    }
    sc_prev = sc;
    valid_prev = kv_valid;
    vslot_prev = vslot;
    vslot = vslot == 2 ? 0 : vslot + 1;
    if (more) store_tile((it + 1) & 1, vslot);
    __syncthreads();                       // next tile visible; K of this step and V of the previous one consumed
  };
  int it = 0;
  for (; it + 1 < topk; it += 2) {
    step(it, acc_a, acc_b);
    step(it + 1, acc_b, acc_a);
  }
  if (it < topk) {                         // odd count: one more step, its scores land in acc_a
    step(it, acc_a, acc_b);
    const i32x8_t pb = probabilities(acc_a, sc_prev, valid_prev);
    accumulate(vslot_prev, pb);
  } else if (topk > 0) {
    const i32x8_t pb = probabilities(acc_b, sc_prev, valid_prev);
    accumulate(vslot_prev, pb);
  }
  const float inv = 1.0f / lacc[0];        // P_SCALE cancels: numerator and l carry the same factor
  // The rounded rows go through LDS (every wave is done with the tiles) and leave as whole rows in streaming stores:
  // they are not read again here, and what does not stay behind as modified lines in L2 need not be written back when
  // the kernel ends.
  __syncthreads();
  {
    constexpr int SSTR = TileRows<D>::SSTR;
    static_assert(3 * 32 * SSTR * 2 <= (int)sizeof(sV) && 32 * SSTR * 2 <= (int)sizeof(sK), "staging tiles of four waves");
    uint16_t* const stage = wave < 3 ? reinterpret_cast<uint16_t*>(&sV[0][0]) + wave * (32 * SSTR)
                                     : reinterpret_cast<uint16_t*>(&sK[0][0]);
    const float* vs = v_scale + (size_t)bh * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = 32 * dt + 8 * i4 + 4 * g;
        const f32x4_t sv = *reinterpret_cast<const f32x4_t*>(vs + d0);
        i32x2_t w;
        w[0] = (int)EO::pack2(oacc[dt][4 * i4 + 0] * inv * sv[0], oacc[dt][4 * i4 + 1] * inv * sv[1]);
        w[1] = (int)EO::pack2(oacc[dt][4 * i4 + 2] * inv * sv[2], oacc[dt][4 * i4 + 3] * inv * sv[3]);
        *reinterpret_cast<i32x2_t*>(&stage[r * SSTR + d0]) = w;
      }
    wave_lds_fence();
    const int row0 = mb * BLKQ + wave * 32;
    TileRows<D> t;
    t.unpark(stage, lane);
    t.store_streaming(o + head_off + (size_t)row0 * D, L - row0, lane, D);
  }
}

// ---- host -------------------------------------------------------------------------------------
struct SageWs {
  int nchunk_v, rows_per_chunk_v;
  size_t chunk_sums, colmean, v_part, total;
};
static SageWs sage_ws(int BH, int L, int D) {
  SageWs w;
  w.rows_per_chunk_v = 256;
  w.nchunk_v = cdiv(L, w.rows_per_chunk_v);
  size_t off = 0;
  w.chunk_sums = off; off += align_up(k_colmean_scratch_floats(BH, L, D) * 4, 256);
  w.colmean = off;    off += align_up((int64_t)BH * D * 2, 256);
  w.v_part = off;     off += align_up((int64_t)BH * w.nchunk_v * D * 4, 256);
  w.total = off;
  return w;
}
int64_t sage_quant_workspace_bytes(int BH, int L, int D) { return (int64_t)sage_ws(BH, L, D).total; }

// workspace of the one-call preparation: the quantisers' workspace, then block means and scores
struct SagePrepWs {
  size_t pq, pk, score, total;
};
static SagePrepWs sage_prep_ws(int BH, int L, int D) {
  const int64_t M = cdiv(L, 128), N = cdiv(L, 64);
  SagePrepWs w;
  size_t off = sage_ws(BH, L, D).total;
  w.pq = off;    off += align_up((int64_t)BH * M * D * 2, 256);
  w.pk = off;    off += align_up((int64_t)BH * N * D * 2, 256);
  w.score = off; off += align_up((int64_t)BH * M * N * 2, 256);
  w.total = off;
  return w;
}
int64_t sage_prepare_workspace_bytes(int BH, int L, int D) { return (int64_t)sage_prep_ws(BH, L, D).total; }

static int validate_sage(int dtype, int B, int H, int L, int D, int BLKQ, int BLKK) {
  SLA_REQUIRE(B > 0 && H > 0 && L > 0, SLA_ERR_BAD_ARG, "non-positive size (B=%d H=%d L=%d)", B, H, L);
  SLA_REQUIRE((int64_t)B * H <= 65535, SLA_ERR_UNSUPPORTED, "B*H exceeds 65535");
  SLA_REQUIRE(dtype == SLA_BF16 || dtype == SLA_F16, SLA_ERR_UNSUPPORTED, "SageSLA takes bf16 or f16, got dtype %d", dtype);
  SLA_REQUIRE(D == 64 || D == 128, SLA_ERR_UNSUPPORTED, "headdim should be in [64, 128], got %d", D);
  SLA_REQUIRE(BLKQ == 128 && BLKK == 64, SLA_ERR_UNSUPPORTED, "SageSLA only supports BLKQ=128 and BLKK=64, got %d/%d", BLKQ,
              BLKK);
  return SLA_OK;
}

// range of the e4m3 values v is quantised to: the format's largest finite value (448) or less
int validate_v_range(float v_range) {
  SLA_REQUIRE(v_range > 0.f && v_range <= 448.f, SLA_ERR_BAD_ARG, "v_range=%g outside (0, 448]", (double)v_range);
  return SLA_OK;
}

template <typename Tag, int D>
static int quant_qk_impl(const void* q, const void* k, int dtype, int BH, int L, int8_t* q8, float* qs, int8_t* k8,
                         float* ks, char* ws, hipStream_t st) {
  const SageWs w = sage_ws(BH, L, D);
  const int M = cdiv(L, 128), N = cdiv(L, 64);
  const RowLayout lay = contiguous_layout(BH, L, D);
  launch_k_colmean(k, lay, dtype, BH, L, D, (float*)(ws + w.chunk_sums), ws + w.colmean, st);
  hipLaunchKernelGGL((quant_int8_kernel<Tag, D, 128, false, false>), dim3(M, BH), dim3(256), 0, st, (const uint16_t*)q, lay,
                     nullptr, q8, qs, nullptr, L, M);
  hipLaunchKernelGGL((quant_int8_kernel<Tag, D, 64, true, false>), dim3(N, BH), dim3(256), 0, st, (const uint16_t*)k, lay,
                     (const uint16_t*)(ws + w.colmean), k8, ks, nullptr, L, N);
  return check_launch("sage_quant_qk");
}

// Mask, INT8 q/k and FP8 v in one pass structure: the column mean of k is formed once (the mask builder
// and the quantiser both subtract it) and the quantisers emit the block means the scores are made of, so
// q is read once and k twice instead of q twice and k four times.
template <typename Tag, int D>
static int quant_v_impl(const void* v, const RowLayout& lay, int BH, int L, uint8_t* v8, float* vs, float v_range, char* ws,
                        hipStream_t st);

// (lay: where the rows of q, k, v lie; the quantised outputs are always contiguous (B, H, L, D))
template <typename Tag, int D>
static int prepare_impl(const void* q, const void* k, const void* v, const RowLayout& lay, int dtype, int BH, int L, int topk,
                        int8_t* sparse_map,
                        void* lut, int lut64, int8_t* q8, float* qs, int8_t* k8, float* ks, uint8_t* v8, float* vs, float v_range,
                        char* ws, hipStream_t st) {
  const SageWs w = sage_ws(BH, L, D);
  const SagePrepWs p = sage_prep_ws(BH, L, D);
  const int M = cdiv(L, 128), N = cdiv(L, 64);
  uint16_t* pq = (uint16_t*)(ws + p.pq);
  uint16_t* pk = (uint16_t*)(ws + p.pk);
  launch_k_colmean(k, lay, dtype, BH, L, D, (float*)(ws + w.chunk_sums), ws + w.colmean, st);
  hipLaunchKernelGGL((quant_int8_kernel<Tag, D, 128, false, true>), dim3(M, BH), dim3(256), 0, st, (const uint16_t*)q, lay,
                     nullptr, q8, qs, pq, L, M);
  hipLaunchKernelGGL((quant_int8_kernel<Tag, D, 64, true, true>), dim3(N, BH), dim3(256), 0, st, (const uint16_t*)k, lay,
                     (const uint16_t*)(ws + w.colmean), k8, ks, pk, L, N);
  launch_map_from_pooled(dtype, pq, pk, ws + p.score, BH, M, N, D, topk, sparse_map, lut, lut64, st);
  int rc = check_launch("sage_prepare");
  if (rc || !v) return rc;
  return quant_v_impl<Tag, D>(v, lay, BH, L, v8, vs, v_range, ws, st);
}

template <typename Tag, int D>
static int quant_v_impl(const void* v, const RowLayout& lay, int BH, int L, uint8_t* v8, float* vs, float v_range, char* ws,
                        hipStream_t st) {
  const SageWs w = sage_ws(BH, L, D);
  float* part = (float*)(ws + w.v_part);
  hipLaunchKernelGGL((v_amax_partial_kernel<Tag, D>), dim3(w.nchunk_v, BH), dim3(256), 0, st, (const uint16_t*)v, lay, part, L,
                     w.rows_per_chunk_v);
  hipLaunchKernelGGL(v_scale_kernel, dim3(D / 16, BH), dim3(256), 0, st, part, vs, w.nchunk_v, D, v_range);
  constexpr int RPP = 256 / (D / 8);
  hipLaunchKernelGGL((v_quant_fp8_kernel<Tag, D>), dim3(cdiv(L, RPP), BH), dim3(256), 0, st, (const uint16_t*)v, lay, vs, v8,
                     L);
  return check_launch("sage_quant_v");
}

int quant_v_from_partial_amax(const void* v, const RowLayout& lay, int dtype, int BH, int L, int D, const float* part,
                              int nparts, uint8_t* v8, float* vs, float v_range, hipStream_t st) {
  hipLaunchKernelGGL(v_scale_kernel, dim3(D / 16, BH), dim3(256), 0, st, part, vs, nparts, D, v_range);
#define SAGE_VQ_CASE(TAG, DD)                                                                                         \
  hipLaunchKernelGGL((v_quant_fp8_kernel<TAG, DD>), dim3(cdiv(L, 256 / (DD / 8)), BH), dim3(256), 0, st, (const uint16_t*)v, \
                     lay, vs, v8, L)
  if (dtype == SLA_BF16) {
    if (D == 128) SAGE_VQ_CASE(bf16_tag, 128);
    else SAGE_VQ_CASE(bf16_tag, 64);
  } else {
    if (D == 128) SAGE_VQ_CASE(f16_tag, 128);
    else SAGE_VQ_CASE(f16_tag, 64);
  }
#undef SAGE_VQ_CASE
  return check_launch("linear_state_quant_v");
}

}  // namespace sla

using namespace sla;

extern "C" int sage_quant_qk(const void* q, const void* k, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK,
                             int8_t* q_int8, float* q_scale, int8_t* k_int8, float* k_scale, void* workspace,
                             int64_t workspace_bytes, void* stream) {
  int rc = validate_sage(dtype, B, H, L, D, BLKQ, BLKK);
  if (rc) return rc;
  SLA_REQUIRE(q && k && q_int8 && q_scale && k_int8 && k_scale && workspace, SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)q_int8 | (uintptr_t)k_int8 | (uintptr_t)workspace) % 16 == 0,
              SLA_ERR_BAD_ARG, "pointers must be 16-byte aligned");
  const int BH = B * H;
  SLA_REQUIRE(workspace_bytes >= sage_quant_workspace_bytes(BH, L, D), SLA_ERR_WORKSPACE, "workspace too small");
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  if (dtype == SLA_BF16) {
    if (D == 128) return quant_qk_impl<bf16_tag, 128>(q, k, dtype, BH, L, q_int8, q_scale, k_int8, k_scale, ws, st);
    return quant_qk_impl<bf16_tag, 64>(q, k, dtype, BH, L, q_int8, q_scale, k_int8, k_scale, ws, st);
  }
  if (D == 128) return quant_qk_impl<f16_tag, 128>(q, k, dtype, BH, L, q_int8, q_scale, k_int8, k_scale, ws, st);
  return quant_qk_impl<f16_tag, 64>(q, k, dtype, BH, L, q_int8, q_scale, k_int8, k_scale, ws, st);
}

static int prepare_entry(const void* q, const void* k, const void* v, const int64_t* qkv_strides, int dtype, int B, int H, int L,
                         int D, int BLKQ, int BLKK, int topk, int8_t* sparse_map, void* lut, int lut_elem_bytes, int8_t* q_int8,
                         float* q_scale, int8_t* k_int8, float* k_scale, uint8_t* v_fp8, float* v_scale, float v_range,
                         void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = validate_sage(dtype, B, H, L, D, BLKQ, BLKK);
  if (rc) return rc;
  rc = validate_v_range(v_range);
  if (rc) return rc;
  RowLayout lay;
  rc = make_layout(qkv_strides, B, H, L, D, 2, &lay);
  if (rc) return rc;
  const int N = cdiv(L, 64);
  SLA_REQUIRE(topk >= 0 && topk <= N, SLA_ERR_BAD_ARG, "topk=%d outside [0, %d]", topk, N);
  SLA_REQUIRE(N <= 4096, SLA_ERR_UNSUPPORTED, "more than 4096 key blocks (%d)", N);
  SLA_REQUIRE(lut_elem_bytes == 4 || lut_elem_bytes == 8, SLA_ERR_BAD_ARG, "lut_elem_bytes must be 4 or 8, got %d",
              lut_elem_bytes);
  // (v, v_fp8 and v_scale may all three be NULL: the caller then quantises v itself with sage_quant_v, e.g. on another
  //  stream)
  SLA_REQUIRE(q && k && sparse_map && (lut || topk == 0) && q_int8 && q_scale && k_int8 && k_scale && workspace &&
                  ((v && v_fp8 && v_scale) || (!v && !v_fp8 && !v_scale)),
              SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)lut | (uintptr_t)q_int8 | (uintptr_t)k_int8 |
               (uintptr_t)v_fp8 | (uintptr_t)workspace) % 16 == 0,
              SLA_ERR_BAD_ARG, "pointers must be 16-byte aligned");
  const int BH = B * H;
  SLA_REQUIRE(workspace_bytes >= sage_prepare_workspace_bytes(BH, L, D), SLA_ERR_WORKSPACE, "workspace of %lld bytes, need %lld",
              (long long)workspace_bytes, (long long)sage_prepare_workspace_bytes(BH, L, D));
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  const int lut64 = lut_elem_bytes == 8;
#define SLA_PREP_CASE(TAG, DD) \
  return prepare_impl<TAG, DD>(q, k, v, lay, dtype, BH, L, topk, sparse_map, lut, lut64, q_int8, q_scale, k_int8, k_scale, \
                               v_fp8, v_scale, v_range, ws, st)
  if (dtype == SLA_BF16) {
    if (D == 128) SLA_PREP_CASE(bf16_tag, 128);
    SLA_PREP_CASE(bf16_tag, 64);
  }
  if (D == 128) SLA_PREP_CASE(f16_tag, 128);
  SLA_PREP_CASE(f16_tag, 64);
#undef SLA_PREP_CASE
}

extern "C" int sage_prepare(const void* q, const void* k, const void* v, int dtype, int B, int H, int L, int D, int BLKQ,
                            int BLKK, int topk, int8_t* sparse_map, void* lut, int lut_elem_bytes, int8_t* q_int8,
                            float* q_scale, int8_t* k_int8, float* k_scale, uint8_t* v_fp8, float* v_scale, float v_range,
                            void* workspace, int64_t workspace_bytes, void* stream) {
  return prepare_entry(q, k, v, nullptr, dtype, B, H, L, D, BLKQ, BLKK, topk, sparse_map, lut, lut_elem_bytes, q_int8, q_scale,
                       k_int8, k_scale, v_fp8, v_scale, v_range, workspace, workspace_bytes, stream);
}

extern "C" int sage_prepare_strided(const void* q, const void* k, const void* v, const int64_t* qkv_strides, int dtype, int B,
                                    int H, int L, int D, int BLKQ, int BLKK, int topk, int8_t* sparse_map, void* lut,
                                    int lut_elem_bytes, int8_t* q_int8, float* q_scale, int8_t* k_int8, float* k_scale,
                                    uint8_t* v_fp8, float* v_scale, float v_range, void* workspace,
                                    int64_t workspace_bytes, void* stream) {
  SLA_REQUIRE(qkv_strides, SLA_ERR_BAD_ARG, "null strides");
  return prepare_entry(q, k, v, qkv_strides, dtype, B, H, L, D, BLKQ, BLKK, topk, sparse_map, lut, lut_elem_bytes, q_int8,
                       q_scale, k_int8, k_scale, v_fp8, v_scale, v_range, workspace, workspace_bytes, stream);
}

static int quant_v_entry(const void* v, const int64_t* v_strides, int dtype, int B, int H, int L, int D, uint8_t* v_fp8,
                         float* v_scale, float v_range, void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = validate_sage(dtype, B, H, L, D, 128, 64);
  if (rc) return rc;
  rc = validate_v_range(v_range);
  if (rc) return rc;
  RowLayout lay;
  rc = make_layout(v_strides, B, H, L, D, 2, &lay);
  if (rc) return rc;
  SLA_REQUIRE(v && v_fp8 && v_scale && workspace, SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)v | (uintptr_t)v_fp8 | (uintptr_t)workspace) % 16 == 0, SLA_ERR_BAD_ARG,
              "pointers must be 16-byte aligned");
  const int BH = B * H;
  SLA_REQUIRE(workspace_bytes >= sage_quant_workspace_bytes(BH, L, D), SLA_ERR_WORKSPACE, "workspace too small");
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  if (dtype == SLA_BF16) {
    if (D == 128) return quant_v_impl<bf16_tag, 128>(v, lay, BH, L, v_fp8, v_scale, v_range, ws, st);
    return quant_v_impl<bf16_tag, 64>(v, lay, BH, L, v_fp8, v_scale, v_range, ws, st);
  }
  if (D == 128) return quant_v_impl<f16_tag, 128>(v, lay, BH, L, v_fp8, v_scale, v_range, ws, st);
  return quant_v_impl<f16_tag, 64>(v, lay, BH, L, v_fp8, v_scale, v_range, ws, st);
}

extern "C" int sage_quant_v(const void* v, int dtype, int B, int H, int L, int D, uint8_t* v_fp8, float* v_scale,
                            float v_range, void* workspace, int64_t workspace_bytes, void* stream) {
  return quant_v_entry(v, nullptr, dtype, B, H, L, D, v_fp8, v_scale, v_range, workspace, workspace_bytes, stream);
}

extern "C" int sage_quant_v_strided(const void* v, const int64_t* v_strides, int dtype, int B, int H, int L, int D,
                                    uint8_t* v_fp8, float* v_scale, float v_range, void* workspace,
                                    int64_t workspace_bytes, void* stream) {
  SLA_REQUIRE(v_strides, SLA_ERR_BAD_ARG, "null strides");
  return quant_v_entry(v, v_strides, dtype, B, H, L, D, v_fp8, v_scale, v_range, workspace, workspace_bytes, stream);
}

extern "C" int sage_sparse_attn_fwd(const int8_t* q_int8, const float* q_scale, const int8_t* k_int8,
                                    const float* k_scale, const uint8_t* v_fp8, const float* v_scale, const void* lut,
                                    int lut_elem_bytes, void* o, int out_dtype, int B, int H, int L, int D, int BLKQ,
                                    int BLKK, int topk, float qk_scale, void* stream) {
  int rc = validate_sage(out_dtype, B, H, L, D, BLKQ, BLKK);
  if (rc) return rc;
  const int Mblk = cdiv(L, BLKQ), Nblk = cdiv(L, BLKK);
  SLA_REQUIRE(topk >= 0 && topk <= Nblk, SLA_ERR_BAD_ARG, "topk=%d outside [0, %d]", topk, Nblk);
  SLA_REQUIRE(lut_elem_bytes == 4 || lut_elem_bytes == 8, SLA_ERR_BAD_ARG, "lut_elem_bytes must be 4 or 8");
  SLA_REQUIRE(q_int8 && q_scale && k_int8 && k_scale && v_fp8 && v_scale && o && (lut || topk == 0), SLA_ERR_BAD_ARG,
              "null pointer");
  SLA_REQUIRE(((uintptr_t)q_int8 | (uintptr_t)k_int8 | (uintptr_t)v_fp8 | (uintptr_t)o | (uintptr_t)v_scale) % 16 == 0,
              SLA_ERR_BAD_ARG, "pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const int BH = B * H;
  const int total = BH * Mblk;
  const float c = qk_scale * 1.4426950408889634f;
  const int lut64 = lut_elem_bytes == 8;
#define SAGE_CASE(TAG, DD)                                                                                              \
  hipLaunchKernelGGL((sage_fwd_kernel<TAG, DD, 128>), dim3(xcd_grid(total)), dim3(256), 0, st, q_int8, q_scale, k_int8, \
                     k_scale, v_fp8, v_scale, lut, lut64, (uint16_t*)o, L, Mblk, Nblk, topk, c, total);                 \
  return check_launch("sage_sparse_attn_fwd")
  if (out_dtype == SLA_BF16) {
    if (D == 128) { SAGE_CASE(bf16_tag, 128); }
    SAGE_CASE(bf16_tag, 64);
  }
  if (D == 128) { SAGE_CASE(f16_tag, 128); }
  SAGE_CASE(f16_tag, 64);
#undef SAGE_CASE
}
