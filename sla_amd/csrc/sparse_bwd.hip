// Block-sparse FlashAttention backward for gfx950.
//
// Stands in for _attn_bwd_preprocess, _attn_bwd_dq, _attn_bwd_dkdv and _attention.backward of
// the reference (sparse_linear_attention/kernel.py:85-237, 277-320):
//   delta = rowsum(o * do)
//   P = exp2(S*c - lse) on the selected blocks, dP = dO V^T, dS = P * (dP - delta)
//   dQ = scale * dS K ; dK = scale * dS^T Q ; dV = P^T dO
//
// Four kernels.
//   delta      : one pass over o and do.
//   col_lists  : the reference scans the dense int8 map column in the dK/dV kernel (about
//                1/density wasted iterations); here the map is turned once into per-key-block
//                lists of the query blocks that selected it.
//   dq         : per query block over its look-up table, products formed transposed as in the
//                forward (S^T = K Q^T, dP^T = V dO^T) so lse and delta are per-lane scalars and
//                dS^T leaves the accumulator in B-operand layout for dQ^T += K^T dS^T (K^T is
//                read from LDS with the transposing read).
//   dkdv       : per key block over its list; S = Q K^T and dP = dO V^T with K^T/V^T resident
//                in registers as B operands; P and dS leave the accumulators in B-operand layout
//                for dV^T += dO^T P and dK^T += Q^T dS (Q^T, dO^T via transposing LDS reads).
//                Four waves: two key halves x two halves of the head dimension.
#include "bwd_steps.h"

namespace sla {

int validate_attn_shape(int dtype, int B, int H, int L, int D, int BLKQ, int BLKK, int topk, int lut_elem_bytes);

// ---- delta ------------------------------------------------------------------------------
template <typename Tag, int D>
__global__ __launch_bounds__(256) void bwd_delta_kernel(const uint16_t* __restrict__ o, const uint16_t* __restrict__ d_o,
                                                        const RowLayout ldo, float* __restrict__ delta, size_t rows, int L) {
  using E = Elem<Tag>;
  constexpr int CPR = D / 8;
  const size_t row = (size_t)blockIdx.x * (256 / CPR) + threadIdx.x / CPR;   // = bh * L + l
  const int col = (threadIdx.x % CPR) * 8;
  float s = 0.f;
  if (row < rows) {
    const int bh = (int)(row / (size_t)L);
    const size_t l = row - (size_t)bh * L;
    const i16x8_t a = *reinterpret_cast<const i16x8_t*>(o + row * D + col);
    const i16x8_t b = *reinterpret_cast<const i16x8_t*>(d_o + ldo.head(bh) + l * (size_t)ldo.sl + col);
#pragma unroll
    for (int e = 0; e < 8; ++e) s += E::to_float((uint16_t)a[e]) * E::to_float((uint16_t)b[e]);
  }
#pragma unroll
  for (int sh = 1; sh < CPR; sh <<= 1) s += __shfl_xor(s, sh);
  if (row < rows && col == 0) delta[row] = s;
}

// ---- per-key-block lists ------------------------------------------------------------------
// One workgroup of COL_NW wavefronts per strip of 64 key blocks.  Every wavefront takes its own chunk of
// 64 map rows (query blocks): it reads them with coalesced 16-byte loads and transposes them through its
// private LDS tile; lane c counts the ones of column c in that chunk.  After a barrier every wave knows
// how many entries the chunks before its own contribute to each column and writes its matches at that
// offset, walking the chunk in row order, so list[bh][n][0..count) holds the selecting query blocks in
// ascending order.  Capacity Mblk per list (only `count` entries are ever touched).
constexpr int COL_NW = 8;
__global__ __launch_bounds__(64 * COL_NW) void bwd_col_lists_kernel(const int8_t* __restrict__ sparse_map,
                                                                    int* __restrict__ list, int* __restrict__ count,
                                                                    int Mblk, int Nblk, int vec_ok) {
  __shared__ __attribute__((aligned(16))) int8_t tile[COL_NW][64][80];
  __shared__ int cnt[COL_NW][64];
  const int bh = blockIdx.y;
  const int n0 = blockIdx.x * 64;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = n0 + lane;
  const int8_t* base = sparse_map + (size_t)bh * Mblk * Nblk;
  int* out = list + ((size_t)bh * Nblk + (n < Nblk ? n : 0)) * Mblk;
  // lane -> (row lr + 16j, 16-byte chunk lc) of the tile
  const int lr = lane >> 2, lc = (lane & 3) * 16;
  int done = 0;              // entries of column `lane` written by earlier rounds
  for (int r0 = 0; r0 < Mblk; r0 += 64 * COL_NW) {
    const int m0 = r0 + 64 * wave;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + lr + 16 * j;
      i32x4_t x = {0, 0, 0, 0};
      if (m < Mblk) {
        if (vec_ok && n0 + lc + 16 <= Nblk) {
          x = *reinterpret_cast<const i32x4_t*>(base + (size_t)m * Nblk + n0 + lc);
        } else {
          int8_t* b = reinterpret_cast<int8_t*>(&x);
          for (int e = 0; e < 16; ++e)
            if (n0 + lc + e < Nblk) b[e] = base[(size_t)m * Nblk + n0 + lc + e];
        }
      }
      *reinterpret_cast<i32x4_t*>(&tile[wave][lr + 16 * j][lc]) = x;
    }
    wave_lds_fence();
    int mine = 0;
#pragma unroll 16
    for (int r = 0; r < 64; ++r) mine += tile[wave][r][lane] == 1;
    cnt[wave][lane] = mine;
    __syncthreads();
    int before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < COL_NW; ++w) {
      const int cw = cnt[w][lane];
      before += w < wave ? cw : 0;
      all += cw;
    }
    if (n < Nblk) {
      int c = done + before;
#pragma unroll 16
      for (int r = 0; r < 64; ++r)
        if (tile[wave][r][lane] == 1) out[c++] = m0 + r;
    }
    done += all;
    __syncthreads();         // cnt and the tiles are rewritten by the next round
  }
  if (wave == 0 && n < Nblk) count[(size_t)bh * Nblk + n] = done;
}

// ---- work items of the dK/dV kernel --------------------------------------------------------
// A key block that very many query blocks selected (an attention "sink") would make one workgroup walk a list
// many times the average length.  Lists longer than `seg` entries are therefore cut into segments of `seg`; every
// segment is one work item.  item = {bh, key block, segment, slot}: slot < 0 for a key block with a single segment
// (the workgroup writes dK / dV itself), otherwise the index of the fp32 partial this segment writes; the partials
// of a key block occupy consecutive slots and are added in segment order by bwd_dkdv_reduce_kernel.
// One workgroup of 1024 threads walks all (head, key block) pairs in order, eight per thread and round, with a running
// prefix sum.
__global__ __launch_bounds__(1024) void bwd_segments_kernel(const int* __restrict__ count, int* __restrict__ nseg,
                                                            int* __restrict__ slot0, i32x4_t* __restrict__ items,
                                                            int* __restrict__ totals, int nblocks, int Nblk, int seg,
                                                            int max_items, int max_slots) {
  constexpr int EPT = 8;                      // consecutive (head, key block) pairs per thread and round
  __shared__ int wsum[2][16];
  __shared__ int base[2];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) base[0] = base[1] = 0;
  __syncthreads();
  for (int i0 = 0; i0 < nblocks; i0 += 1024 * EPT) {
    const int first = i0 + tid * EPT;
    int ns[EPT];
    int own_a = 0, own_b = 0;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      ns[e] = first + e < nblocks ? max(1, (count[first + e] + seg - 1) / seg) : 0;
      own_a += ns[e];
      own_b += ns[e] > 1 ? ns[e] : 0;
    }
    int a = own_a, b = own_b;                 // inclusive scans inside the wave
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int ta = __shfl_up(a, o), tb = __shfl_up(b, o);
      if (lane >= o) {
        a += ta;
        b += tb;
      }
    }
    if (lane == 63) {
      wsum[0][wave] = a;
      wsum[1][wave] = b;
    }
    __syncthreads();
    int pa = 0, pb = 0, ta = 0, tb = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      pa += w < wave ? wsum[0][w] : 0;
      pb += w < wave ? wsum[1][w] : 0;
      ta += wsum[0][w];
      tb += wsum[1][w];
    }
    int first_item = base[0] + pa + a - own_a, first_slot = base[1] + pb + b - own_b;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = first + e;
      if (i < nblocks) {
        const int ms = ns[e] > 1 ? ns[e] : 0;
        nseg[i] = ns[e];
        slot0[i] = first_slot;
        const int bh = i / Nblk, nb = i - bh * Nblk;
        // (a map whose rows hold more ones than the topk the workspace was sized for cannot overrun the tables: its
        //  surplus items are dropped)
        for (int sg = 0; sg < ns[e]; ++sg)
          if (first_item + sg < max_items && first_slot + ms <= max_slots)
            items[first_item + sg] = i32x4_t{bh, nb, sg, ns[e] > 1 ? first_slot + sg : -1};
          else if (first_item + sg < max_items)
            items[first_item + sg] = i32x4_t{bh, nb, sg, -2};
        first_item += ns[e];
        first_slot += ms;
      }
    }
    __syncthreads();
    if (tid == 0) {
      base[0] += ta;
      base[1] += tb;
    }
    __syncthreads();
  }
  if (tid == 0) {
    totals[0] = min(base[0], max_items);
    totals[1] = min(base[1], max_slots);
  }
}

// grid (Nblk, BH), 256 threads: key blocks whose list was cut add their partials (fp32, [slot][dk | dv][64][D]) in
// segment order and write dK, dV; all others leave at once.
template <typename Tag, int D>
__global__ __launch_bounds__(256) void bwd_dkdv_reduce_kernel(const int* __restrict__ nseg, const int* __restrict__ slot0,
                                                              const float* __restrict__ part, uint16_t* __restrict__ dk,
                                                              uint16_t* __restrict__ dv, const RowLayout lin, int L, int Nblk,
                                                              int max_slots) {
  using E = Elem<Tag>;
  const int nb = blockIdx.x, bh = blockIdx.y;
  const int ns = nseg[(size_t)bh * Nblk + nb];
  if (ns <= 1 || slot0[(size_t)bh * Nblk + nb] + ns > max_slots) return;
  const float* p0 = part + (size_t)slot0[(size_t)bh * Nblk + nb] * (2 * 64 * D);
  for (int idx = threadIdx.x * 4; idx < 2 * 64 * D; idx += 256 * 4) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int sg = 0; sg < ns; ++sg) acc += *reinterpret_cast<const f32x4_t*>(p0 + (size_t)sg * (2 * 64 * D) + idx);
    const int which = idx / (64 * D), rem = idx - which * (64 * D);
    const int row = nb * 64 + rem / D, col = rem % D;
    if (row < L) {
      i32x2_t w;
      w[0] = (int)E::pack2(acc[0], acc[1]);
      w[1] = (int)E::pack2(acc[2], acc[3]);
      uint16_t* dst = (which ? dv : dk) + lin.head(bh) + (size_t)row * (size_t)lin.sl + col;
      *reinterpret_cast<i32x2_t*>(dst) = w;
    }
  }
}

// ---- dQ ---------------------------------------------------------------------------------
// One workgroup per query block, one wave per 32 queries.  Register use is held to 256 so that two waves
// share a SIMD.  K and V tiles go global -> registers -> LDS; both tiles of the next step are in flight
// during the whole current step.
// CONTIG: all tensors are contiguous (B, H, L, D); the row pitch is then the compile-time D and every in-tile
// offset folds into an instruction immediate (the strided variant pays a few registers for the run-time pitch).
template <typename Tag, int D, int BLKQ, bool CONTIG>
__global__ __launch_bounds__(BLKQ * 2) __attribute__((amdgpu_waves_per_eu(D == 64 ? 3 : 2, D == 64 ? 3 : 2))) void bwd_dq_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
    const uint16_t* __restrict__ d_o, const float* __restrict__ lse, const float* __restrict__ delta,
    const void* __restrict__ lut, int lut64, uint16_t* __restrict__ dq, const RowLayout lin, const RowLayout ldo, int L,
    int Mblk, int topk, float qk_scale, int total) {
  using E = Elem<Tag>;
  constexpr int BLKK = 64;
  constexpr int NT = BLKQ * 2;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int KSTR = D + 16;   // K is read both row-wise and transposed
  constexpr int VSTR = D + 8;
  constexpr int CPR = D / 8;
  constexpr int NLD = BLKK * CPR / NT;

  __shared__ __attribute__((aligned(16))) uint16_t sK[BLKK * KSTR];
  __shared__ __attribute__((aligned(16))) uint16_t sV[BLKK * VSTR];

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int bh = logical / Mblk;
  const int mb = logical - bh * Mblk;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;
  const float c_log2e = qk_scale * 1.4426950408889634f;

  // q, k, v (and dq) rows of this head lie lin.sl elements apart, dO rows ldo.sl (D for contiguous tensors)
  const size_t head_off = CONTIG ? (size_t)bh * L * D : lin.head(bh);
  const uint32_t pitch = CONTIG ? D : (uint32_t)lin.sl, pitch_do = CONTIG ? D : (uint32_t)ldo.sl;
  const uint32_t head_bytes = CONTIG ? (uint32_t)L * D * 2 : lin.head_range_bytes(L, D);
  const __amdgpu_buffer_rsrc_t qh = make_rsrc(q + head_off, head_bytes);
  const __amdgpu_buffer_rsrc_t doh =
      make_rsrc(d_o + (CONTIG ? head_off : ldo.head(bh)), CONTIG ? head_bytes : ldo.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t kh = make_rsrc(k + head_off, head_bytes);
  const __amdgpu_buffer_rsrc_t vh = make_rsrc(v + head_off, head_bytes);
  const int qrow = mb * BLKQ + wave * 32 + r;
  const bool qok = qrow < L;

  i16x8_t qf[DC], dof[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    qf[c] = buf_load_b128(qh, ((uint32_t)qrow * pitch + 16 * c + 8 * g) * 2);      // rows past L read as zero
    dof[c] = buf_load_b128(doh, ((uint32_t)qrow * pitch_do + 16 * c + 8 * g) * 2);
  }
  // rows past L: lse = +inf makes every probability exactly 0 (the reference loads `other=inf`)
  const float lse_q = qok ? lse[(size_t)bh * L + qrow] : INFINITY;
  const float delta_q = qok ? delta[(size_t)bh * L + qrow] : 0.f;

  const size_t lut_row = ((size_t)bh * Mblk + mb) * topk;
  auto lut_at = [&](int i) -> int {
    return lut64 ? (int)reinterpret_cast<const long long*>(lut)[lut_row + i]
                 : reinterpret_cast<const int*>(lut)[lut_row + i];
  };
  i16x8_t kreg[NLD], vreg[NLD];
  // chunk i of a thread is row tid / CPR + i * (NT / CPR) of the tile.  With a run-time pitch the per-chunk
  // offsets are not instruction immediates; they are formed from one per-lane offset at every use (the opaque
  // copy keeps the compiler from hoisting eight of them out of the loop into registers it does not have).
  static_assert(NT % CPR == 0, "threads must cover whole rows");
  const uint32_t lane_off = ((uint32_t)(tid / CPR) * pitch + (tid % CPR) * 8) * 2;
  auto load_tile = [&](int nb) {
    uint32_t lo = lane_off + (uint32_t)(nb * BLKK) * pitch * 2;
    if (!CONTIG) asm volatile("" : "+v"(lo));
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const uint32_t off = lo + (uint32_t)(i * (NT / CPR)) * pitch * 2;      // rows past L read as zero
      kreg[i] = buf_load_b128(kh, off);
      vreg[i] = buf_load_b128(vh, off);
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

  f32x16_t dqacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) dqacc[dt][i] = 0.f;

  const int tr_row = (lane & 15) >> 2;
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  int nb = topk > 0 ? lut_at(0) : 0;
  int nb_next = topk > 1 ? lut_at(1) : 0;
  if (topk > 0) {
    load_tile(nb);
    store_tile();
  }
  __syncthreads();
  for (int it = 0; it < topk; ++it) {
    const bool more = it + 1 < topk;
    if (more) {
      nb = nb_next;
      nb_next = it + 2 < topk ? lut_at(it + 2) : 0;
      load_tile(nb);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      f32x16_t s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s[i] = 0.f;
        dp[i] = 0.f;
      }
      // (the group barriers fix the issue order: LDS reads run two fragments ahead of the MFMAs that use them)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const i16x8_t a = *reinterpret_cast<const i16x8_t*>(&sK[(32 * t + r) * KSTR + 16 * c + 8 * g]);
        s = E::mfma32(a, qf[c], s);
        const i16x8_t b = *reinterpret_cast<const i16x8_t*>(&sV[(32 * t + r) * VSTR + 16 * c + 8 * g]);
        dp = E::mfma32(b, dof[c], dp);
      }
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
      for (int i = 0; i < 2 * DC - 2; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_barrier(0);
      // dS^T = P^T * (dP^T - delta).  Key rows past L need no masking: their K rows are zero in LDS, so
      // whatever (finite) dS they get is multiplied by zero in dQ^T += K^T dS^T.
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float p = fast_exp2(__builtin_fmaf(s[i], c_log2e, -lse_q));
        s[i] = p * (dp[i] - delta_q);
      }
      i16x8_t dsb[2];
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        i32x4_t pw;
#pragma unroll
        for (int j = 0; j < 4; ++j) pw[j] = (int)E::pack2(s[8 * c2 + 2 * j], s[8 * c2 + 2 * j + 1]);
        dsb[c2] = __builtin_bit_cast(i16x8_t, pw);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        const int key0 = 32 * t + 16 * c2 + 4 * g + tr_row;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const uint16_t* p0 = &sK[key0 * KSTR + 32 * dt + tr_col];
          dqacc[dt] = E::mfma32(concat4(lds_read_tr16(p0), lds_read_tr16(p0 + 8 * KSTR)), dsb[c2], dqacc[dt]);
        }
      }
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
      for (int i = 0; i < 2 * DT - 2; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();                       // both tiles fully consumed
    if (more) store_tile();
    __syncthreads();                       // next tiles visible
  }
  if (qok) {
    uint16_t* orow = dq + head_off + (size_t)qrow * pitch;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        i32x2_t w;
        w[0] = (int)E::pack2(dqacc[dt][4 * i4 + 0] * qk_scale, dqacc[dt][4 * i4 + 1] * qk_scale);
        w[1] = (int)E::pack2(dqacc[dt][4 * i4 + 2] * qk_scale, dqacc[dt][4 * i4 + 3] * qk_scale);
        *reinterpret_cast<i32x2_t*>(orow + 32 * dt + 8 * i4 + 4 * g) = w;
      }
  }
}

// ---- dK, dV -----------------------------------------------------------------------------
// One workgroup of four waves per key block.  Wave (kh, dh): kh = wave % 2 selects keys 32kh..32kh+31 of
// the block, dh = wave / 2 selects the half of the head dimension whose dK^T / dV^T rows this wave
// accumulates.  Per tile of 64 query rows the two waves that share kh split the rows: each forms S and dP
// for its 32 rows, turns them into P and dS (accumulator layout = B-operand layout of the second
// products) and hands a copy to its partner through LDS; then each adds all 64 rows into its own half of
// dV^T += dO^T P and dK^T += Q^T dS.  Splitting the accumulators this way keeps a wave at 256 registers,
// so two waves share a SIMD.
template <typename Tag, int D, int BLKQ, bool CONTIG>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D == 64 ? 3 : 2, D == 64 ? 3 : 2))) void bwd_dkdv_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
    const uint16_t* __restrict__ d_o, const float* __restrict__ lse, const float* __restrict__ delta,
    const int* __restrict__ list, const int* __restrict__ count, const i32x4_t* __restrict__ items,
    const int* __restrict__ totals, float* __restrict__ part, int seg, uint16_t* __restrict__ dk, uint16_t* __restrict__ dv,
    const RowLayout lin, const RowLayout ldo, int L, int Mblk, int Nblk, float qk_scale) {
  using E = Elem<Tag>;
  constexpr int TQ = 64;                  // query rows per LDS tile
  constexpr int SUB = BLKQ / TQ;          // tiles per listed query block
  constexpr int NT = 256;
  constexpr int DC = D / 16;
  constexpr int DH = D / 64;              // 32-row tiles of dK^T / dV^T owned by one wave
  constexpr int STR = D + 16;             // Q and dO are read row-wise and transposed
  constexpr int CPR = D / 8;
  constexpr int NLD = TQ * CPR / NT;

  __shared__ __attribute__((aligned(16))) uint16_t sQ[TQ * STR];
  __shared__ __attribute__((aligned(16))) uint16_t sDO[TQ * STR];
  __shared__ __attribute__((aligned(16))) float sLse[TQ];
  __shared__ __attribute__((aligned(16))) float sDelta[TQ];
  __shared__ __attribute__((aligned(16))) i16x8_t sXP[4][2][64];    // [wave][16-row group][lane] packed P
  __shared__ __attribute__((aligned(16))) i16x8_t sXS[4][2][64];    // same for dS

  // The grid covers the largest possible number of work items; the actual number is known on the device only.
  // Every XCD takes one contiguous range of the actual items (consecutive workgroup ids go round-robin to the XCDs).
  const int total = totals[0];
  const int per_xcd = (total + 7) >> 3;
  if ((int)(blockIdx.x >> 3) >= per_xcd) return;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (logical >= total) return;
  const i32x4_t item = items[logical];
  const int bh = item[0], nb = item[1], sg = item[2], slot = item[3];
  if (slot < -1) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kh = wave & 1, dh = wave >> 1;
  const int g = lane >> 5, r = lane & 31;
  const float c_log2e = qk_scale * 1.4426950408889634f;

  const size_t head_off = CONTIG ? (size_t)bh * L * D : lin.head(bh);
  const uint32_t pitch = CONTIG ? D : (uint32_t)lin.sl, pitch_do = CONTIG ? D : (uint32_t)ldo.sl;
  const uint32_t head_bytes = CONTIG ? (uint32_t)L * D * 2 : lin.head_range_bytes(L, D);
  const __amdgpu_buffer_rsrc_t qh = make_rsrc(q + head_off, head_bytes);
  const __amdgpu_buffer_rsrc_t doh =
      make_rsrc(d_o + (CONTIG ? head_off : ldo.head(bh)), CONTIG ? head_bytes : ldo.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t kb = make_rsrc(k + head_off, head_bytes);
  const __amdgpu_buffer_rsrc_t vb = make_rsrc(v + head_off, head_bytes);
  const float* lseh = lse + (size_t)bh * L;
  const float* deltah = delta + (size_t)bh * L;

  // K^T and V^T fragments (B operands): this lane's key column, 8 adjacent d per chunk
  const int krow = nb * 64 + kh * 32 + r;
  const bool kok = krow < L;
  i16x8_t kf[DC], vf[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    kf[c] = buf_load_b128(kb, ((uint32_t)krow * pitch + 16 * c + 8 * g) * 2);     // rows past L read as zero
    vf[c] = buf_load_b128(vb, ((uint32_t)krow * pitch + 16 * c + 8 * g) * 2);
  }

  f32x16_t dkacc[DH], dvacc[DH];
#pragma unroll
  for (int dt = 0; dt < DH; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dkacc[dt][i] = 0.f;
      dvacc[dt][i] = 0.f;
    }

  const int* mylist = list + ((size_t)bh * Nblk + nb) * Mblk;
  // this work item's part of the list, in tiles of TQ query rows
  const int tile0 = sg * seg * SUB;
  const int ntile = min(count[(size_t)bh * Nblk + nb], (sg + 1) * seg) * SUB;

  i16x8_t qreg[NLD], doreg[NLD];
  float lreg = 0.f, dreg = 0.f;
  auto tile_row0 = [&](int ti) -> int { return mylist[ti / SUB] * BLKQ + (ti % SUB) * TQ; };
  // (per-chunk offsets formed at every use from one per-lane offset, as in the dQ kernel)
  static_assert(NT % CPR == 0, "threads must cover whole rows");
  const uint32_t lane_off = ((uint32_t)(tid / CPR) * pitch + (tid % CPR) * 8) * 2;
  const uint32_t lane_off_do = ((uint32_t)(tid / CPR) * pitch_do + (tid % CPR) * 8) * 2;
  auto load_tile = [&](int row0) {
    uint32_t lo = lane_off + (uint32_t)row0 * pitch * 2, lo_do = lane_off_do + (uint32_t)row0 * pitch_do * 2;
    asm volatile("" : "+v"(lo), "+v"(lo_do));
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      // rows past L read as zero
      qreg[i] = buf_load_b128(qh, lo + (uint32_t)(i * (NT / CPR)) * pitch * 2);
      doreg[i] = buf_load_b128(doh, lo_do + (uint32_t)(i * (NT / CPR)) * pitch_do * 2);
    }
    if (tid < TQ) {
      const int grow = row0 + tid;
      lreg = grow < L ? lseh[grow] : INFINITY;     // +inf -> probability 0 for rows past L
      dreg = grow < L ? deltah[grow] : 0.f;
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int idx = tid + i * NT;
      const int row = idx / CPR, col = (idx % CPR) * 8;
      *reinterpret_cast<i16x8_t*>(&sQ[row * STR + col]) = qreg[i];
      *reinterpret_cast<i16x8_t*>(&sDO[row * STR + col]) = doreg[i];
    }
    if (tid < TQ) {
      sLse[tid] = lreg;
      sDelta[tid] = dreg;
    }
  };

  const int tr_row = (lane & 15) >> 2;
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  int row_next = tile0 + 1 < ntile ? tile_row0(tile0 + 1) : 0;
  if (tile0 < ntile) {
    load_tile(tile_row0(tile0));
    store_tile();
  }
  __syncthreads();
  for (int ti = tile0; ti < ntile; ++ti) {
    if (ti + 1 < ntile) {
      load_tile(row_next);
      row_next = ti + 2 < ntile ? tile_row0(ti + 2) : 0;
    }
    // ---- phase 1: P and dS of query rows 32dh..32dh+31 of the tile against this wave's 32 keys ----
    f32x16_t s, dp;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = 0.f;
      dp[i] = 0.f;
    }
    // (the group barriers fix the issue order: LDS reads run a few fragments ahead of the MFMAs that use them)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      const i16x8_t a = *reinterpret_cast<const i16x8_t*>(&sQ[(32 * dh + r) * STR + 16 * c + 8 * g]);
      s = E::mfma32(a, kf[c], s);
      const i16x8_t b = *reinterpret_cast<const i16x8_t*>(&sDO[(32 * dh + r) * STR + 16 * c + 8 * g]);
      dp = E::mfma32(b, vf[c], dp);
    }
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
    for (int i = 0; i < 2 * DC - 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
    __builtin_amdgcn_sched_barrier(0);
    // accumulator rows are queries 32dh + 8*(i/4) + 4g + i%4; this lane's column is its key
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const f32x4_t l4 = *reinterpret_cast<const f32x4_t*>(&sLse[32 * dh + 8 * i4 + 4 * g]);
      const f32x4_t d4 = *reinterpret_cast<const f32x4_t*>(&sDelta[32 * dh + 8 * i4 + 4 * g]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = 4 * i4 + j;
        // (a key row past L only ever feeds its own, never stored, column of dK^T / dV^T: no masking needed)
        const float p = fast_exp2(__builtin_fmaf(s[i], c_log2e, -l4[j]));
        s[i] = p;
        dp[i] = p * (dp[i] - d4[j]);
      }
    }
    i16x8_t pmine[2], smine[2];
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2) {
      i32x4_t pw, dw;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pw[j] = (int)E::pack2(s[8 * c2 + 2 * j], s[8 * c2 + 2 * j + 1]);
        dw[j] = (int)E::pack2(dp[8 * c2 + 2 * j], dp[8 * c2 + 2 * j + 1]);
      }
      pmine[c2] = __builtin_bit_cast(i16x8_t, pw);
      smine[c2] = __builtin_bit_cast(i16x8_t, dw);
      sXP[wave][c2][lane] = pmine[c2];
      sXS[wave][c2][lane] = smine[c2];
    }
    __syncthreads();                       // partner's P and dS visible
    // ---- phase 2: all 64 query rows into this wave's half of dV^T and dK^T ----
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        // rows 32h + 16c2..: own registers when h == dh, else the partner's copy (wave ^ 2: same keys, other rows)
        i16x8_t pb = pmine[c2], dsb = smine[c2];
        if (h != dh) {
          pb = sXP[wave ^ 2][c2][lane];
          dsb = sXS[wave ^ 2][c2][lane];
        }
        const int q0 = 32 * h + 16 * c2 + 4 * g + tr_row;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int dt = 0; dt < DH; ++dt) {
          const int dcol = 32 * (DH * dh + dt) + tr_col;
          const uint16_t* pdo = &sDO[q0 * STR + dcol];
          dvacc[dt] = E::mfma32(concat4(lds_read_tr16(pdo), lds_read_tr16(pdo + 8 * STR)), pb, dvacc[dt]);
          const uint16_t* pq = &sQ[q0 * STR + dcol];
          dkacc[dt] = E::mfma32(concat4(lds_read_tr16(pq), lds_read_tr16(pq + 8 * STR)), dsb, dkacc[dt]);
        }
        // all eight transposing reads of this 16-row group first, then its four MFMAs
        __builtin_amdgcn_sched_group_barrier(0x100, 4 * DH, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * DH, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    __syncthreads();                       // tile and exchange buffers fully consumed
    if (ti + 1 < ntile) store_tile();
    __syncthreads();                       // next tile visible
  }
  if (slot >= 0) {
    // one segment of a long list: fp32 partial [dk | dv][64][D], added up by bwd_dkdv_reduce_kernel
    float* pk = part + (size_t)slot * (2 * 64 * D) + (size_t)(kh * 32 + r) * D;
    float* pv = pk + 64 * D;
#pragma unroll
    for (int dt = 0; dt < DH; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = 32 * (DH * dh + dt) + 8 * i4 + 4 * g;
        *reinterpret_cast<f32x4_t*>(pk + d0) = f32x4_t{dkacc[dt][4 * i4 + 0] * qk_scale, dkacc[dt][4 * i4 + 1] * qk_scale,
                                                       dkacc[dt][4 * i4 + 2] * qk_scale, dkacc[dt][4 * i4 + 3] * qk_scale};
        *reinterpret_cast<f32x4_t*>(pv + d0) =
            f32x4_t{dvacc[dt][4 * i4 + 0], dvacc[dt][4 * i4 + 1], dvacc[dt][4 * i4 + 2], dvacc[dt][4 * i4 + 3]};
      }
    return;
  }
  if (kok) {
    uint16_t* dkrow = dk + head_off + (size_t)krow * pitch;
    uint16_t* dvrow = dv + head_off + (size_t)krow * pitch;
#pragma unroll
    for (int dt = 0; dt < DH; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = 32 * (DH * dh + dt) + 8 * i4 + 4 * g;
        i32x2_t w;
        w[0] = (int)E::pack2(dkacc[dt][4 * i4 + 0] * qk_scale, dkacc[dt][4 * i4 + 1] * qk_scale);
        w[1] = (int)E::pack2(dkacc[dt][4 * i4 + 2] * qk_scale, dkacc[dt][4 * i4 + 3] * qk_scale);
        *reinterpret_cast<i32x2_t*>(dkrow + d0) = w;
        w[0] = (int)E::pack2(dvacc[dt][4 * i4 + 0], dvacc[dt][4 * i4 + 1]);
        w[1] = (int)E::pack2(dvacc[dt][4 * i4 + 2], dvacc[dt][4 * i4 + 3]);
        *reinterpret_cast<i32x2_t*>(dvrow + d0) = w;
      }
  }
}

// ---- host ---------------------------------------------------------------------------------
// list[bh][n][0..count[bh][n]) = the query blocks that selected key block n, ascending; capacity Mblk per list
// (also used by the backward of the complement-mode linear branch)
void launch_col_lists(const int8_t* sparse_map, int* list, int* count, int BH, int Mblk, int Nblk, hipStream_t st) {
  // 16-byte loads of map rows need 16-byte aligned rows
  const int vec_ok = (Nblk % 16 == 0) && ((uintptr_t)sparse_map % 16 == 0);
  hipLaunchKernelGGL(bwd_col_lists_kernel, dim3(cdiv(Nblk, 64), BH), dim3(64 * COL_NW), 0, st, sparse_map, list, count, Mblk, Nblk,
                     vec_ok);
}

}  // namespace sla
#include "sparse_bwd_stream.h"
namespace sla {

struct BwdWs {
  int seg;                  // longest stretch of a key block's list one workgroup walks
  int64_t max_items, max_slots;
  size_t delta, count, list, nseg, slot0, items, totals, part, total;
};
static BwdWs bwd_ws(int BH, int L, int D, int BLKQ, int BLKK, int topk) {
  const int64_t M = cdiv(L, BLKQ), N = cdiv(L, BLKK);
  BwdWs w;
  // A segment is at most a quarter of the list entries an average resident workgroup (2 per compute unit) walks, and
  // at least 64: balanced maps are never cut, and the fp32 partials of the worst case stay bounded (the lists of one
  // head hold M*topk entries in all, so at most 2*M*topk/seg segments belong to lists longer than seg).
  const int64_t entries = (int64_t)BH * M * topk;
  int64_t seg = (entries + 2047) / 2048;     // 512 resident workgroups, a quarter of the average each
  if (seg < 64) seg = 64;
  // (a work item's entries have to fit its LDS copy, which holds a 128-row query block as its two halves)
  const int64_t seg_cap = BLKQ == 128 ? DKDV_STREAM_MAX_SEG / 2 : DKDV_STREAM_MAX_SEG;
  if (seg > seg_cap) seg = seg_cap;
  w.seg = (int)seg;
  w.max_items = (int64_t)BH * N + entries / seg;
  w.max_slots = 2 * entries / seg;
  size_t off = 0;
  w.delta = off;  off += align_up((int64_t)BH * L * 4, 256);
  w.count = off;  off += align_up((int64_t)BH * N * 4, 256);
  w.list = off;   off += align_up((int64_t)BH * N * M * 4, 256);
  w.nseg = off;   off += align_up((int64_t)BH * N * 4, 256);
  w.slot0 = off;  off += align_up((int64_t)BH * N * 4, 256);
  w.items = off;  off += align_up(w.max_items * 16, 256);
  w.totals = off; off += 256;
  w.part = off;   off += align_up(w.max_slots * 2 * 64 * D * 4, 256);
  w.total = off;
  return w;
}
int64_t sparse_bwd_workspace_bytes(int BH, int L, int D, int BLKQ, int BLKK, int topk) {
  return (int64_t)bwd_ws(BH, L, D, BLKQ, BLKK, topk).total;
}

template <typename Tag, int D, int BLKQ>
static int bwd_impl(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                    const int8_t* sparse_map, const void* lut, int lut64, void* dq, void* dk, void* dv,
                    const RowLayout& lin, const RowLayout& ldo, int BH, int L, int topk, float qk_scale, char* ws,
                    hipStream_t st, int steps) {
  if (steps == 0) return SLA_OK;        // (arguments checked, nothing asked for)
  const BwdWs w = bwd_ws(BH, L, D, BLKQ, 64, topk);
  const int Mblk = cdiv(L, BLKQ), Nblk = cdiv(L, 64);
  float* delta = (float*)(ws + w.delta);
  int* count = (int*)(ws + w.count);
  int* list = (int*)(ws + w.list);
  const size_t rows = (size_t)BH * L;
  constexpr int RPB = 256 / (D / 8);
  if (steps & SB_LISTS) launch_col_lists(sparse_map, list, count, BH, Mblk, Nblk, st);
  int* nseg = (int*)(ws + w.nseg);
  int* slot0 = (int*)(ws + w.slot0);
  i32x4_t* items = (i32x4_t*)(ws + w.items);
  int* totals = (int*)(ws + w.totals);
  float* part = (float*)(ws + w.part);
  if (steps & SB_LISTS)
    hipLaunchKernelGGL(bwd_segments_kernel, dim3(1), dim3(1024), 0, st, count, nseg, slot0, items, totals, BH * Nblk, Nblk,
                       w.seg, (int)w.max_items, (int)w.max_slots);
  const int total_q = BH * Mblk;
  const bool contig = lin.sl == D && ldo.sl == D;
  // head dim 128 with 64-row query blocks has kernels of its own (32-bit byte offsets inside a head); a 128-row query
  // block goes through them as its two halves (`wide`), which follow the block's row of the table and its list entries
  const int wide = BLKQ == 128;
  const int Mblk64 = cdiv(L, 64);
  const int total_q64 = BH * Mblk64;
  const bool stream_dkdv = D == 128 && (BLKQ == 64 || BLKQ == 128) && (uint64_t)lin.sl * 2u * (uint64_t)L < (1ull << 31) &&
                           (uint64_t)ldo.sl * 2u * (uint64_t)L < (1ull << 31);
  // (enough query blocks for a wave on every SIMD; the stream kernel keeps a look-up row as 16-bit key block indices)
  const bool stream_dq = stream_dkdv && topk <= DQ_STREAM_MAX_T && total_q64 >= 1024 && Mblk64 <= 65535;
  // delta = rowsum(dO * O): the dQ kernel of the common shape forms it for its own rows, the general one reads it
  if ((steps & SB_DQ) && !stream_dq)
    hipLaunchKernelGGL((bwd_delta_kernel<Tag, D>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, st,
                       (const uint16_t*)o, (const uint16_t*)d_o, ldo, delta, rows, L);
#define SLA_BWD_LAUNCH(CONTIG)                                                                                              \
  if (!(steps & SB_DQ)) {                                                                                                   \
  } else if (stream_dq)                                                                                                     \
    hipLaunchKernelGGL((bwd_dq_stream_kernel<Tag>), dim3(xcd_grid(total_q64)), dim3(64), 0, st, (const uint16_t*)q,         \
                       (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)d_o, (const uint16_t*)o, lse, delta, lut,   \
                       lut64, (uint16_t*)dq, lin, ldo, L, Mblk64, topk, qk_scale, total_q64, wide);                        \
  else                                                                                                                      \
    hipLaunchKernelGGL((bwd_dq_kernel<Tag, D, BLKQ, CONTIG>), dim3(xcd_grid(total_q)), dim3(BLKQ * 2), 0, st,               \
                       (const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)d_o, lse, delta, lut,   \
                       lut64, (uint16_t*)dq, lin, ldo, L, Mblk, topk, qk_scale, total_q);                                  \
  if (!(steps & SB_DKDV)) {                                                                                                 \
  } else if (stream_dkdv)                                                                                                   \
    hipLaunchKernelGGL((bwd_dkdv_stream_kernel<Tag>), dim3(xcd_grid(w.max_items)), dim3(128), 0, st, (const uint16_t*)q,    \
                       (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)d_o, lse, delta, list, count, items,       \
                       totals, part, w.seg, (uint16_t*)dk, (uint16_t*)dv, lin, ldo, L, Mblk, Nblk, qk_scale, wide);       \
  else                                                                                                                      \
    hipLaunchKernelGGL((bwd_dkdv_kernel<Tag, D, BLKQ, CONTIG>), dim3(xcd_grid(w.max_items)), dim3(256), 0, st,             \
                       (const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)d_o, lse, delta, list,  \
                       count, items, totals, part, w.seg, (uint16_t*)dk, (uint16_t*)dv, lin, ldo, L, Mblk, Nblk, qk_scale);
  if (contig) {
    SLA_BWD_LAUNCH(true)
  } else {
    SLA_BWD_LAUNCH(false)
  }
#undef SLA_BWD_LAUNCH
  if (steps & SB_DKDV)
    hipLaunchKernelGGL((bwd_dkdv_reduce_kernel<Tag, D>), dim3(Nblk, BH), dim3(256), 0, st, nseg, slot0, part, (uint16_t*)dk,
                       (uint16_t*)dv, lin, L, Nblk, (int)w.max_slots);
  return check_launch("sparse_attn_bwd");
}

int attn_bwd_steps(const void* q, const void* k, const void* v, const int64_t* qkv_strides, const void* o, const void* d_o,
                   const int64_t* do_strides, const float* lse, const int8_t* sparse_map, const void* lut, int lut_elem_bytes,
                   void* dq, void* dk, void* dv, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK, int topk,
                   float qk_scale, void* workspace, int64_t workspace_bytes, void* stream, int steps) {
  int rc = validate_attn_shape(dtype, B, H, L, D, BLKQ, BLKK, topk, lut_elem_bytes);
  if (rc) return rc;
  SLA_REQUIRE(q && k && v && o && d_o && lse && sparse_map && dq && dk && dv && workspace && (lut || topk == 0),
              SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)d_o | (uintptr_t)dq | (uintptr_t)dk |
               (uintptr_t)dv | (uintptr_t)workspace) % 16 == 0,
              SLA_ERR_BAD_ARG, "tensors must be 16-byte aligned");
  SLA_REQUIRE((int64_t)B * H <= 65535, SLA_ERR_UNSUPPORTED, "B*H exceeds 65535");
  const int BH = B * H;
  const int64_t need = sparse_bwd_workspace_bytes(BH, L, D, BLKQ, BLKK, topk);
  SLA_REQUIRE(workspace_bytes >= need, SLA_ERR_WORKSPACE, "workspace of %lld bytes, need %lld", (long long)workspace_bytes,
              (long long)need);
  SLA_REQUIRE((int64_t)BH * cdiv(L, 64) * cdiv(L, BLKQ) < (1ll << 40), SLA_ERR_UNSUPPORTED, "block map too large");
  RowLayout lin, ldo;
  rc = make_layout(qkv_strides, B, H, L, D, 2, &lin);
  if (rc) return rc;
  rc = make_layout(do_strides, B, H, L, D, 2, &ldo);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  const int lut64 = lut_elem_bytes == 8;
#define SLA_BWD_CASE(TAG, DD, BQ)                                                                                          \
  if (D == DD && BLKQ == BQ)                                                                                               \
  return bwd_impl<TAG, DD, BQ>(q, k, v, o, d_o, lse, sparse_map, lut, lut64, dq, dk, dv, lin, ldo, BH, L, topk, qk_scale, \
                               ws, st, steps)
  if (dtype == SLA_BF16) {
    SLA_BWD_CASE(bf16_tag, 128, 64);
    SLA_BWD_CASE(bf16_tag, 128, 128);
    SLA_BWD_CASE(bf16_tag, 64, 64);
    SLA_BWD_CASE(bf16_tag, 64, 128);
  } else {
    SLA_BWD_CASE(f16_tag, 128, 64);
    SLA_BWD_CASE(f16_tag, 128, 128);
    SLA_BWD_CASE(f16_tag, 64, 64);
    SLA_BWD_CASE(f16_tag, 64, 128);
  }
#undef SLA_BWD_CASE
  set_error("unsupported D=%d BLKQ=%d", D, BLKQ);
  return SLA_ERR_UNSUPPORTED;
}

}  // namespace sla

using namespace sla;

extern "C" int sla_sparse_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                                   const float* lse, const int8_t* sparse_map, const void* lut, int lut_elem_bytes,
                                   void* dq, void* dk, void* dv, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK,
                                   int topk, float qk_scale, void* workspace, int64_t workspace_bytes, void* stream) {
  return attn_bwd_steps(q, k, v, nullptr, o, d_o, nullptr, lse, sparse_map, lut, lut_elem_bytes, dq, dk, dv, dtype, B, H, L,
                        D, BLKQ, BLKK, topk, qk_scale, workspace, workspace_bytes, stream, SB_ALL);
}

extern "C" int sla_sparse_attn_bwd_strided(const void* q, const void* k, const void* v, const int64_t* qkv_strides,
                                           const void* o, const void* d_o, const int64_t* do_strides, const float* lse,
                                           const int8_t* sparse_map, const void* lut, int lut_elem_bytes, void* dq, void* dk,
                                           void* dv, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK, int topk,
                                           float qk_scale, void* workspace, int64_t workspace_bytes, void* stream) {
  SLA_REQUIRE(qkv_strides && do_strides, SLA_ERR_BAD_ARG, "null strides");
  return attn_bwd_steps(q, k, v, qkv_strides, o, d_o, do_strides, lse, sparse_map, lut, lut_elem_bytes, dq, dk, dv, dtype, B,
                        H, L, D, BLKQ, BLKK, topk, qk_scale, workspace, workspace_bytes, stream, SB_ALL);
}
