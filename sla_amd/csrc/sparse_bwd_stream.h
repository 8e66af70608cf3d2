// dK / dV of the block-sparse attention backward for 64-row query blocks at head dim 128: one workgroup of two
// waves per key block (or per segment of a key block's list), one wave per SIMD.
//
// Stands in for _attn_bwd_dkdv of the reference (sparse_linear_attention/kernel.py:160-237) like bwd_dkdv_kernel,
// whose work items, lists and arithmetic it shares.  What differs:
//   * a wave owns 32 keys and the whole head dimension: K^T and V^T fragments (B operands of S = Q K^T and
//     dP = dO V^T) and the dK^T / dV^T accumulators (128 d x 32 keys each) stay in its registers, P and dS leave
//     the accumulators in the B-operand layout of dV^T += dO^T P and dK^T += Q^T dS.  Nothing is handed from wave
//     to wave, and there is one barrier per 32 query rows;
//   * Q and dO rows go from memory straight into LDS (buffer loads with the LDS bit), 32 rows at a time, into a
//     ring of four generations; the rows of unit u + 3 are requested while unit u is worked on.  Rows are unpadded;
//     the 16-byte pieces of a row are XOR-swizzled with the row index so that both the row-wise reads (A operands
//     of S and dP) and the transposing reads (A operands of the second products) are free of bank conflicts;
//   * the loop is rotated: the exponentials and the rest of the vector arithmetic of unit u run beside the first
//     products of unit u + 1, then come the second products of unit u.
#pragma once
#include "common.h"

namespace sla {

// 16 bytes per lane, memory -> LDS: lane l's piece lands at lds_base + lds_off + 16 l.  (Between a scalar write of M0
// and a memory -> LDS load that reads it the hardware wants one wait state; the compiler adds it to its own code and
// does not look into these instructions.)
static __device__ __forceinline__ void lds_dma_b128(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_off, uint32_t lds_base,
                                                    uint32_t lds_off) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_base), "v"(byte_off), "s"(rsrc),
               "s"(lds_off)
               : "memory", "scc");
}
// 4 bytes per lane: lane l's word lands at lds_base + lds_off + 4 l
static __device__ __forceinline__ void lds_dma_b32(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_off, uint32_t lds_base,
                                                   uint32_t lds_off) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" ::"s"(lds_base), "v"(byte_off), "s"(rsrc),
               "s"(lds_off)
               : "memory", "scc");
}

constexpr int DKDV_STREAM_MAX_SEG = 1024;      // list entries one work item may have (they are copied into LDS)

template <typename Tag>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(1, 1))) void bwd_dkdv_stream_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
    const uint16_t* __restrict__ d_o, const float* __restrict__ lse, const float* __restrict__ delta,
    const int* __restrict__ list, const int* __restrict__ count, const i32x4_t* __restrict__ items,
    const int* __restrict__ totals, float* __restrict__ part, int seg, uint16_t* __restrict__ dk, uint16_t* __restrict__ dv,
    const RowLayout lin, const RowLayout ldo, int L, int Mblk, int Nblk, float qk_scale, int wide) {
  // (wide = 1: the lists name 128-row query blocks; an entry is then walked as its two 64-row halves)
  using E = Elem<Tag>;
  constexpr int D = 128, DC = D / 16, DT = D / 32;
  constexpr int ROWB = D * 2;               // bytes per row in LDS (unpadded)
  constexpr int TILE = 32 * ROWB;           // 32 rows of Q or of dO
  constexpr int GEN = 2 * TILE + 256;       // one generation: Q rows, dO rows, 32 log-sum-exps, 32 deltas
  constexpr int NG = 4;
  constexpr int NREQ = 9;                   // requests per wave and unit: 4 x Q, 4 x dO (its 16 rows), 1 x lse or delta
  __shared__ __attribute__((aligned(16))) uint8_t smem[NG * GEN];
  // This work item's list entries.  (Read from memory inside the loop they would be vector loads - the inline assembly
  // keeps the compiler from using the scalar path - and waiting for a vector load means waiting for every memory ->
  // LDS request issued before it.)
  __shared__ int entries[DKDV_STREAM_MAX_SEG];

  // work item (see bwd_dkdv_kernel)
  const int total = totals[0];
  const int per_xcd = (total + 7) >> 3;
  if ((int)(blockIdx.x >> 3) >= per_xcd) return;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (logical >= total) return;
  const i32x4_t item = items[logical];
  const int bh = __builtin_amdgcn_readfirstlane(item[0]), nb = __builtin_amdgcn_readfirstlane(item[1]);
  const int sg = __builtin_amdgcn_readfirstlane(item[2]), slot = __builtin_amdgcn_readfirstlane(item[3]);
  if (slot < -1) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);         // keys 32w .. 32w+31 of the block
  const int g = lane >> 5, r = lane & 31;
  const float c_log2e = qk_scale * 1.4426950408889634f;

  const size_t head_off = lin.head(bh);
  const uint32_t pitch = (uint32_t)lin.sl, pitch_do = (uint32_t)ldo.sl;
  const __amdgpu_buffer_rsrc_t qh = make_rsrc(q + head_off, lin.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t doh = make_rsrc(d_o + ldo.head(bh), ldo.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t kb = make_rsrc(k + head_off, lin.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t vb = make_rsrc(v + head_off, lin.head_range_bytes(L, D));
  // wave 0 fetches the log-sum-exps of a unit, wave 1 its deltas
  const __amdgpu_buffer_rsrc_t ldh = make_rsrc((w ? delta : lse) + (size_t)bh * L, (uint32_t)L * 4);

  // The length of this key block's list and the first 128 entries of this work item's part of it are asked for before
  // the fragments below (loads come back in the order they were issued, and the first requests for Q and dO hang on
  // the entries); entries past the end of the list are read from inside its row of Mblk words and never used.
  const int* mylist = list + ((size_t)bh * Nblk + nb) * Mblk;
  const int e0 = sg * seg;
  const int count_lane = count[(size_t)bh * Nblk + nb];
  const int first_entry = mylist[min(e0 + (tid >> wide), Mblk - 1)];
  // K^T and V^T fragments (B operands): this lane's key column, 8 adjacent d per chunk; parked in accumulation registers
  const int krow = nb * 64 + w * 32 + r;
  const bool kok = krow < L;
  i16x8_t kf[DC], vf[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    kf[c] = buf_load_b128(kb, ((uint32_t)krow * pitch + 16 * c + 8 * g) * 2);     // rows past L read as zero
    vf[c] = buf_load_b128(vb, ((uint32_t)krow * pitch + 16 * c + 8 * g) * 2);
  }
  // Rows past L are never written into LDS (they lie outside the buffers), and what LDS holds in their place must
  // be finite: their probabilities are exactly 0 (log-sum-exp +inf), and 0 times a finite number adds nothing.
#pragma unroll
  for (int i = 0; i < (NG * GEN / 16 + 127) / 128; ++i)
    if (i * 128 + tid < NG * GEN / 16) reinterpret_cast<i32x4_t*>(smem)[i * 128 + tid] = i32x4_t{0, 0, 0, 0};

  f32x16_t dkacc[DT], dvacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dkacc[dt][i] = 0.f;
      dvacc[dt][i] = 0.f;
    }

  // this work item's part of the list, in units of 32 query rows (two per listed query block)
  const int e1 = min(__builtin_amdgcn_readfirstlane(count_lane), (sg + 1) * seg);
  const int nent = (e1 - e0) << wide;               // 64-row blocks this work item walks
  const int nunits = 2 * nent;
  auto entry_row0 = [&](int e) __attribute__((always_inline)) -> int {          // past the end: the last entry again (fetched, never used)
    return __builtin_amdgcn_readfirstlane(entries[min(e, nent - 1)]) * 64;
  };
  if (tid < (seg << wide)) entries[tid] = (first_entry << wide) + (tid & wide);
  for (int i = 128 + tid; i < nent; i += 128) entries[i] = (mylist[e0 + (i >> wide)] << wide) + (i & wide);

  // ---- addressing ----
  // A request moves 4 rows (64 lanes x 16 bytes): lane -> row 4j + lane / 16 of this wave's 16 rows, 16-byte slot
  // lane % 16, which receives piece (slot ^ swz(row)) of that row.  swz(row) = 4 (row % 4) + (row / 4) % 4: for one
  // piece the 16 rows of a row-wise read hit 16 different slots, and the 4 rows x 4 pieces of a transposing read too.
  auto swz = [](int row) __attribute__((always_inline)) { return ((row & 3) << 2) | ((row >> 2) & 3); };
  const uint32_t smem_addr = (uint32_t)(size_t)smem;
  const int lrow = lane >> 4, lslot = lane & 15;
  uint32_t qoff[4], dooff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 16 * w + 4 * j + lrow;                     // row of the unit (16 w: a multiple of 16, no part in swz)
    const uint32_t piece = (uint32_t)(lslot ^ swz(row & 15)) * 16;
    qoff[j] = (uint32_t)row * pitch * 2 + piece;
    dooff[j] = (uint32_t)row * pitch_do * 2 + piece;
  }
  // LDS addresses of this wave's 16 rows inside a tile and of its 32 words (log-sum-exps or deltas) behind the tiles
  const uint32_t rows_base = __builtin_amdgcn_readfirstlane(smem_addr + (uint32_t)(16 * w) * ROWB);
  const uint32_t ld_base = __builtin_amdgcn_readfirstlane(smem_addr + (uint32_t)w * 128);
  auto request = [&](int row0, int gen) __attribute__((always_inline)) {
    const uint32_t base = (uint32_t)gen * GEN;
    const uint32_t rq = (uint32_t)row0 * pitch * 2, rdo = (uint32_t)row0 * pitch_do * 2;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lds_dma_b128(qh, qoff[j] + rq, rows_base, base + j * 1024);
      lds_dma_b128(doh, dooff[j] + rdo, rows_base, base + TILE + j * 1024);
    }
    if (lane < 32) lds_dma_b32(ldh, (uint32_t)(row0 + lane) * 4, ld_base, base + 2 * TILE);
  };
  // row-wise fragment c of this lane: row r, piece 2c + g
  int rfo[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) rfo[c] = r * ROWB + (((2 * c + g) ^ swz(r & 15)) * 16);
  // transposed fragment (16 query rows x 32 d): rows 16 c2 + 4 g + (lane % 16) / 4 and 8 further on, 8 bytes at element
  // 4 (lane % 4) of the 16-column strip 2 dt + (lane / 16) % 2
  const int tr_row = 4 * g + ((lane & 15) >> 2);
  int tfo[2][DT];                    // [which of the two rows][dt], without the 16 c2 rows
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int row = tr_row + 8 * h;
      const int piece = 4 * dt + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
      tfo[h][dt] = row * ROWB + ((piece ^ swz(row & 15)) * 16) + (lane & 1) * 8;
    }

  // ---- prologue: units 0, 1, 2 requested; S and dP of unit 0 ----
  f32x16_t s_a, dp_a, s_b, dp_b;
  __syncthreads();                                             // the zeros and the entries are in place before anything is requested
  // first query rows of the listed blocks: E0 = of the entry of units u and u + 1, E1 = of the next one, E2 = of the one after
  int E0 = 0, E1 = 0, E2 = 0;
  if (nunits > 0) {
    E0 = entry_row0(0);
    E1 = entry_row0(1);
    E2 = entry_row0(2);
    request(E0, 0);
    request(E0 + 32, 1);
    request(E1, 2);
  }
  // (the wait for the K^T and V^T fragments comes here, behind the first requests, which only needed the list)
#pragma unroll
  for (int c = 0; c < DC; ++c) asm volatile("" : "+a"(kf[c]), "+a"(vf[c]));
  if (nunits > 0) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NREQ) : "memory");
    __syncthreads();
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      const i16x8_t a = *reinterpret_cast<const i16x8_t*>(smem + rfo[c]);
      const i16x8_t b = *reinterpret_cast<const i16x8_t*>(smem + TILE + rfo[c]);
      if (c == 0) {
        mfma_scores_first<Tag>(s_a, a, kf[c]);
        mfma_scores_first<Tag>(dp_a, b, vf[c]);
      } else {
        mfma_scores<Tag>(s_a, a, kf[c]);
        mfma_scores<Tag>(dp_a, b, vf[c]);
      }
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");         // (the vector ALU reads these results next)
  }

  // What one iteration fetches from LDS for the next one (the data landed long before): the log-sum-exps and deltas of
  // its 32 query rows (accumulator register 4 i4 + j of S / dP is query row 8 i4 + 4 g + j of the unit; this lane's
  // column is its key) and the transposed fragments of its first two groups of second products.
  f32x4_t l4[4], d4[4];
  i16x8_t trd[4], trq[4];            // transposed dO / Q fragments of group grp in slot grp % 4, fetched two groups ahead
  auto row_scalars = [&](const uint8_t* gen, int i4) __attribute__((always_inline)) {
    l4[i4] = *reinterpret_cast<const f32x4_t*>(gen + 2 * TILE + (8 * i4 + 4 * g) * 4);
    d4[i4] = *reinterpret_cast<const f32x4_t*>(gen + 2 * TILE + 128 + (8 * i4 + 4 * g) * 4);
  };
  auto tr_frags = [&](const uint8_t* gen, int grp) __attribute__((always_inline)) {
    const int c2 = grp >> 2, dt = grp & 3;
    const uint8_t* t0 = gen + 16 * c2 * ROWB;
    trd[grp & 3] = concat4(lds_read_tr16(reinterpret_cast<const uint16_t*>(t0 + TILE + tfo[0][dt])),
                           lds_read_tr16(reinterpret_cast<const uint16_t*>(t0 + TILE + tfo[1][dt])));
    trq[grp & 3] = concat4(lds_read_tr16(reinterpret_cast<const uint16_t*>(t0 + tfo[0][dt])),
                           lds_read_tr16(reinterpret_cast<const uint16_t*>(t0 + tfo[1][dt])));
  };
  if (nunits > 0) {
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) row_scalars(smem, i4);
    tr_frags(smem, 0);
    tr_frags(smem, 1);
  }

  // One iteration = unit u, 32 MFMAs:
  //   slots  0..15  S and dP of unit u + 1 (two chains)      beside: P and dS of unit u
  //   slots 16..31  dV^T += dO^T P, dK^T += Q^T dS of unit u  beside: the requests for unit u + 3, and what the next
  //                                                            iteration wants from LDS first (see above)
  // On entry: s_cur, dp_cur = Q K^T and dO V^T of unit u.  Before anything else: this wave's part of unit u + 1 has
  // landed (all but the latest nine requests), one barrier (the partner's part too; everyone is done with unit u - 1,
  // whose generation the requests for u + 3 overwrite).  A single wave per SIMD has nobody to hide its LDS latency:
  // every fragment is fetched three products (row-wise) or two groups (transposed) before it is used, and the first
  // four elements of the vector arithmetic run while the first row-wise fragments are on their way.
  // GU = u % 4: the generation of unit u.  (Unrolling four iterations to make it a constant costs more registers
  // than the kernel has: the compiler then spills the resident fragments.)
  auto iteration = [&](int GU, f32x16_t& s_cur, f32x16_t& dp_cur, f32x16_t& s_nxt, f32x16_t& dp_nxt, int row0_u,
                       int row0_req) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NREQ) : "memory");
    __syncthreads();
    const uint8_t* gu = smem + GU * GEN;                       // unit u: transposed reads
    const uint8_t* gn = smem + ((GU + 1) & 3) * GEN;           // unit u + 1: row-wise reads, scalars, first transposed reads
    i16x8_t af[4], bf[4];
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      af[c] = *reinterpret_cast<const i16x8_t*>(gn + rfo[c]);
      bf[c] = *reinterpret_cast<const i16x8_t*>(gn + TILE + rfo[c]);
    }
    if (__builtin_expect(row0_u + 32 > L, 0)) {                // rows past L: +inf makes every probability exactly 0
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (row0_u + 8 * i4 + 4 * g + j >= L) {
            l4[i4][j] = INFINITY;
            d4[i4][j] = 0.f;
          }
    }
    i32x4_t pw[2], dw[2];
    // element i of unit u: P = exp2(S c - lse), dS = P (dP - delta); packed in pairs
    auto element = [&](int i) __attribute__((always_inline)) {
      float p = fast_exp2(__builtin_fmaf(s_cur[i], c_log2e, -l4[i >> 2][i & 3]));
      float ds = p * (dp_cur[i] - d4[i >> 2][i & 3]);
      asm volatile("" : "+v"(p), "+v"(ds));
      s_cur[i] = p;
      dp_cur[i] = ds;
      if (i & 1) {
        uint32_t a = E::pack2(s_cur[i - 1], s_cur[i]), b = E::pack2(dp_cur[i - 1], dp_cur[i]);
        asm volatile("" : "+v"(a), "+v"(b));
        pw[i >> 3][(i >> 1) & 3] = (int)a;
        dw[i >> 3][(i >> 1) & 3] = (int)b;
      }
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) element(i);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      if (c + 3 < DC) {
        af[(c + 3) & 3] = *reinterpret_cast<const i16x8_t*>(gn + rfo[c + 3]);
        bf[(c + 3) & 3] = *reinterpret_cast<const i16x8_t*>(gn + TILE + rfo[c + 3]);
      }
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        if (half == 0) {
          if (c == 0) mfma_scores_first<Tag>(s_nxt, af[c & 3], kf[c]);
          else mfma_scores<Tag>(s_nxt, af[c & 3], kf[c]);
        } else {
          if (c == 0) mfma_scores_first<Tag>(dp_nxt, bf[c & 3], vf[c]);
          else mfma_scores<Tag>(dp_nxt, bf[c & 3], vf[c]);
        }
        const int sl = 2 * c + half;                           // twelve elements left for sixteen slots
        if (sl < 12) element(4 + sl);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // (a key row past L only ever feeds its own, never stored, column of dK^T / dV^T: no masking needed)
    const uint32_t req_base = (uint32_t)((GU + 3) & 3) * GEN;
    const uint32_t rq = (uint32_t)row0_req * pitch * 2, rdo = (uint32_t)row0_req * pitch_do * 2;
    // eight groups (c2, dt) of two products
#pragma unroll
    for (int grp = 0; grp < 8; ++grp) {
      const int c2 = grp >> 2, dt = grp & 3;
      if (grp + 2 < 8) tr_frags(gu, grp + 2);
      else tr_frags(gn, grp + 2 - 8);                          // the next unit's first two groups
      if (grp >= 4) row_scalars(gn, grp - 4);                  // and its scalars
      dvacc[dt] = E::mfma32(trd[grp & 3], __builtin_bit_cast(i16x8_t, pw[c2]), dvacc[dt]);
      dkacc[dt] = E::mfma32(trq[grp & 3], __builtin_bit_cast(i16x8_t, dw[c2]), dkacc[dt]);
      if (grp < 4) {
        lds_dma_b128(qh, qoff[grp] + rq, rows_base, req_base + grp * 1024);
        lds_dma_b128(doh, dooff[grp] + rdo, rows_base, req_base + TILE + grp * 1024);
      } else if (grp == 4) {
        if (lane < 32) lds_dma_b32(ldh, (uint32_t)(row0_req + lane) * 4, ld_base, req_base + 2 * TILE);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  for (int u = 0; u < nunits; u += 2) {
    const int E3 = entry_row0((u >> 1) + 3);                        // (looked up now, used two units from now)
    iteration(u & 3, s_a, dp_a, s_b, dp_b, E0, E1 + 32);            // unit u; requests unit u + 3
    iteration((u + 1) & 3, s_b, dp_b, s_a, dp_a, E0 + 32, E2);      // unit u + 1; requests u + 4
    E0 = E1;
    E1 = E2;
    E2 = E3;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // (nothing of this workgroup is in flight when it ends)

  if (slot >= 0) {
    // one segment of a long list: fp32 partial [dk | dv][64][D], added up by bwd_dkdv_reduce_kernel
    float* pk = part + (size_t)slot * (2 * 64 * D) + (size_t)(w * 32 + r) * D;
    float* pv = pk + 64 * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = 32 * dt + 8 * i4 + 4 * g;
        *reinterpret_cast<f32x4_t*>(pk + d0) = f32x4_t{dkacc[dt][4 * i4 + 0] * qk_scale, dkacc[dt][4 * i4 + 1] * qk_scale,
                                                       dkacc[dt][4 * i4 + 2] * qk_scale, dkacc[dt][4 * i4 + 3] * qk_scale};
        *reinterpret_cast<f32x4_t*>(pv + d0) =
            f32x4_t{dvacc[dt][4 * i4 + 0], dvacc[dt][4 * i4 + 1], dvacc[dt][4 * i4 + 2], dvacc[dt][4 * i4 + 3]};
      }
    return;
  }
  // The rounded rows go through LDS (both waves are done with the generations) and leave as whole rows in streaming
  // stores: they are not read again here, and what does not stay behind as modified lines in L2 need not be written
  // back when the kernel ends.
  __syncthreads();
  uint16_t* const stage = reinterpret_cast<uint16_t*>(smem) + w * (32 * TileRows<D>::SSTR);
  const int krow0 = nb * 64 + w * 32;
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    constexpr int SSTR = TileRows<D>::SSTR;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        i32x2_t wv;
        if (which == 0) {
          wv[0] = (int)E::pack2(dkacc[dt][4 * i4 + 0] * qk_scale, dkacc[dt][4 * i4 + 1] * qk_scale);
          wv[1] = (int)E::pack2(dkacc[dt][4 * i4 + 2] * qk_scale, dkacc[dt][4 * i4 + 3] * qk_scale);
        } else {
          wv[0] = (int)E::pack2(dvacc[dt][4 * i4 + 0], dvacc[dt][4 * i4 + 1]);
          wv[1] = (int)E::pack2(dvacc[dt][4 * i4 + 2], dvacc[dt][4 * i4 + 3]);
        }
        *reinterpret_cast<i32x2_t*>(&stage[r * SSTR + 32 * dt + 8 * i4 + 4 * g]) = wv;
      }
    wave_lds_fence();
    TileRows<D> t;
    t.unpark(stage, lane);
    t.store_streaming((which == 0 ? dk : dv) + head_off + (size_t)krow0 * pitch, L - krow0, lane, pitch);
    wave_lds_fence();
  }
}


// ---- dQ ------------------------------------------------------------------------------------------------------------
// dQ of the block-sparse attention backward for 64-row query blocks at head dim 128: one wave per query block, one wave
// per SIMD, no barriers.
//
// Stands in for _attn_bwd_dq of the reference (sparse_linear_attention/kernel.py:95-157) like bwd_dq_kernel, whose
// arithmetic it shares (S^T = K Q^T and dP^T = V dO^T, so that the log-sum-exp and delta of a query are per-lane
// scalars and dS^T leaves the accumulator as the B operand of dQ^T += K^T dS^T).  What differs:
//   * the wave owns all 64 query rows (two tiles of 32): Q^T and dO^T fragments and the dQ^T accumulators fill the
//     accumulation registers, and every transposed K fragment read from LDS feeds two products;
//   * K and V go from memory straight into LDS, 32 keys at a time, two generations each, swizzled like the Q / dO
//     rows of bwd_dkdv_stream_kernel; the 32 keys after next are requested as soon as the current ones are used up
//     (the transposed K fragments wait in registers), a unit and a half before they are wanted;
//   * inside a unit of 32 keys the two query tiles are staggered: S, dP of tile 0 | S, dP of tile 1 beside the
//     vector arithmetic of tile 0 | dQ of tile 0 beside the vector arithmetic of tile 1 | dQ of tile 1.
constexpr int DQ_STREAM_MAX_T = 2048;          // look-up rows longer than this take bwd_dq_kernel

template <typename Tag>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(1, 1))) void bwd_dq_stream_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
    const uint16_t* __restrict__ d_o, const uint16_t* __restrict__ o, const float* __restrict__ lse, float* __restrict__ delta,
    const void* __restrict__ lut, int lut64, uint16_t* __restrict__ dq, const RowLayout lin, const RowLayout ldo, int L,
    int Mblk, int topk, float qk_scale, int total, int wide) {
  // (Mblk: 64-row blocks per head.  wide = 1: the look-up table has one row per 128-row block, which both halves follow)
  using E = Elem<Tag>;
  constexpr int D = 128, DC = D / 16, DT = D / 32;
  constexpr int ROWB = D * 2;
  constexpr int TILE = 32 * ROWB;                 // 32 rows of K or V
  __shared__ __attribute__((aligned(16))) uint8_t smem[4 * TILE];      // K generation 0, 1; V generation 0, 1
  __shared__ uint16_t entries[DQ_STREAM_MAX_T];                        // this block's look-up row

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int bh = logical / Mblk;
  const int mb = logical - bh * Mblk;
  const int lane = threadIdx.x;
  const int g = lane >> 5, r = lane & 31;
  const float c_log2e = qk_scale * 1.4426950408889634f;

  const size_t head_off = lin.head(bh);
  const uint32_t pitch = (uint32_t)lin.sl, pitch_do = (uint32_t)ldo.sl;
  const uint32_t row_bytes = pitch * 2;
  const __amdgpu_buffer_rsrc_t qh = make_rsrc(q + head_off, lin.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t doh = make_rsrc(d_o + ldo.head(bh), ldo.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t kh = make_rsrc(k + head_off, lin.head_range_bytes(L, D));
  const __amdgpu_buffer_rsrc_t vh = make_rsrc(v + head_off, lin.head_range_bytes(L, D));
  const int qrow0 = mb * 64;

  // The first 64 entries of the look-up row are asked for before anything else: the first requests for K and V hang on
  // them, and loads come back in the order they were issued (the low word of a 64-bit entry is the entry).
  const size_t lut_row = wide ? ((size_t)bh * ((Mblk + 1) >> 1) + (mb >> 1)) * topk : ((size_t)bh * Mblk + mb) * topk;
  auto lut_at = [&](size_t i) __attribute__((always_inline)) -> int { return reinterpret_cast<const int*>(lut)[lut64 ? 2 * i : i]; };
  int first_entries = 0;
  if (topk > 0) first_entries = lut_at(lut_row + min(lane, topk - 1));      // (an empty table may be a null pointer)
  // Q^T and dO^T fragments (B operands; rows past L read as zero), per-lane scalars of the two query tiles
  // The rows of the forward's output come the same way: delta = rowsum(dO * O) (reference kernel.py:282-286, the
  // preprocess step) is formed here, for this block's rows, and written out for the dK/dV kernel.
  i16x8_t qf[2][DC], dof[2][DC], of[2][DC];
  float lse_q[2], delta_q[2];
  const __amdgpu_buffer_rsrc_t oh = make_rsrc(o + (size_t)bh * L * D, (uint32_t)L * D * 2);      // (contiguous (B, H, L, D))
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    const int qrow = qrow0 + 32 * qt + r;
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      qf[qt][c] = buf_load_b128(qh, ((uint32_t)qrow * pitch + 16 * c + 8 * g) * 2);
      dof[qt][c] = buf_load_b128(doh, ((uint32_t)qrow * pitch_do + 16 * c + 8 * g) * 2);
      of[qt][c] = buf_load_b128(oh, ((uint32_t)qrow * D + 16 * c + 8 * g) * 2);                  // rows past L: 0, delta 0
    }
    // rows past L: lse = +inf makes every probability exactly 0 (the reference loads `other=inf`)
    lse_q[qt] = qrow < L ? lse[(size_t)bh * L + qrow] : INFINITY;
  }
  if (lane < topk) entries[lane] = (uint16_t)first_entries;
  for (int i = 64 + lane; i < topk; i += 64) entries[i] = (uint16_t)lut_at(lut_row + i);
  // key rows past L are never written into LDS: what LDS holds in their place has to be finite (their probabilities
  // are masked to exactly 0 below)
#pragma unroll
  for (int i = 0; i < 4 * TILE / 16 / 64; ++i) reinterpret_cast<i32x4_t*>(smem)[i * 64 + lane] = i32x4_t{0, 0, 0, 0};
  wave_lds_fence();

  f32x16_t dqacc[DT][2];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int i = 0; i < 16; ++i) dqacc[dt][qt][i] = 0.f;

  // ---- addressing (see bwd_dkdv_stream_kernel) ----
  auto swz = [](int row) __attribute__((always_inline)) { return ((row & 3) << 2) | ((row >> 2) & 3); };
  const uint32_t smem_addr = __builtin_amdgcn_readfirstlane((uint32_t)(size_t)smem);
  const int lrow = lane >> 4, lslot = lane & 15;
  uint32_t koff[4];                  // request j covers rows 4 j + lane / 16 of the 32: j % 4 here, 16 rows more for j >= 4
#pragma unroll
  for (int j = 0; j < 4; ++j) koff[j] = (uint32_t)(4 * j + lrow) * row_bytes + (uint32_t)(lslot ^ swz(4 * j + lrow)) * 16;
  const int nunits = 2 * topk;
  auto unit_rows = [&](int u) __attribute__((always_inline)) -> int {           // first key row of unit u; past the end: the last unit again
    const int uc = min(u, nunits - 1);
    return __builtin_amdgcn_readfirstlane((int)entries[uc >> 1]) * 64 + 32 * (uc & 1);
  };
  auto request = [&](int key0, int GEN) __attribute__((always_inline)) {
    const uint32_t rb = (uint32_t)key0 * row_bytes;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t off = koff[j & 3] + rb + (uint32_t)(j >> 2) * 16 * row_bytes;
      lds_dma_b128(kh, off, smem_addr, GEN * TILE + j * 1024);
      lds_dma_b128(vh, off, smem_addr, (2 + GEN) * TILE + j * 1024);
    }
  };
  int rfo[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) rfo[c] = r * ROWB + (((2 * c + g) ^ swz(r & 15)) * 16);
  const int tr_row = 4 * g + ((lane & 15) >> 2);
  int tfo[2][DT];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int row = tr_row + 8 * h;
      const int piece = 4 * dt + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
      tfo[h][dt] = row * ROWB + ((piece ^ swz(row & 15)) * 16) + (lane & 1) * 8;
    }
  // One unit = 32 keys, 48 MFMAs.  GEN = u % 2.
  f32x16_t s0, dp0, s1, dp1;
  auto unit = [&](int GEN, int key0, int key0_next2) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");          // this unit's rows have landed (the next unit's 16 requests may be out)
    const uint8_t* kg = smem + GEN * TILE;
    const uint8_t* vg = smem + (2 + GEN) * TILE;
    const int valid = L - key0;                                // key rows of this unit that exist
    i16x8_t af[4], bf[4];                                      // row-wise fragments, three products ahead
    auto first_products = [&](f32x16_t& s, f32x16_t& dp, const i16x8_t (&qq)[DC], const i16x8_t (&dd)[DC], auto&& beside)
        __attribute__((always_inline)) {
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        af[c] = *reinterpret_cast<const i16x8_t*>(kg + rfo[c]);
        bf[c] = *reinterpret_cast<const i16x8_t*>(vg + rfo[c]);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        if (c + 3 < DC) {
          af[(c + 3) & 3] = *reinterpret_cast<const i16x8_t*>(kg + rfo[c + 3]);
          bf[(c + 3) & 3] = *reinterpret_cast<const i16x8_t*>(vg + rfo[c + 3]);
        }
        if (c == 0) mfma_scores_first<Tag>(s, af[0], qq[0]);
        else mfma_scores<Tag>(s, af[c & 3], qq[c]);
        beside(2 * c);
        __builtin_amdgcn_sched_barrier(0);
        if (c == 0) mfma_scores_first<Tag>(dp, bf[0], dd[0]);
        else mfma_scores<Tag>(dp, bf[c & 3], dd[c]);
        beside(2 * c + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // element i of a tile: dS^T = P^T (dP^T - delta), P = exp2(S c - lse); packed in pairs into the B operand
    auto element = [&](f32x16_t& s, f32x16_t& dp, int qt, i32x4_t (&dsw)[2], int i) __attribute__((always_inline)) {
      float p = fast_exp2(__builtin_fmaf(s[i], c_log2e, -lse_q[qt]));
      float ds = p * (dp[i] - delta_q[qt]);
      asm volatile("" : "+v"(ds));
      s[i] = ds;
      if (i & 1) {
        uint32_t a = E::pack2(s[i - 1], s[i]);
        asm volatile("" : "+v"(a));
        dsw[i >> 3][(i >> 1) & 3] = (int)a;
      }
    };
    auto mask_tail = [&](f32x16_t& s) __attribute__((always_inline)) {       // key index of register i is 8 (i / 4) + i % 4 + 4 g
      const int lim = valid - 4 * g;
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (8 * (i >> 2) + (i & 3) >= lim) s[i] = -INFINITY;
    };
    i32x4_t dsw0[2], dsw1[2];
    first_products(s0, dp0, qf[0], dof[0], [](int) __attribute__((always_inline)) {});
    // (the vector ALU keeps off a product's result for two products' time: the elements start in slot 2)
    first_products(s1, dp1, qf[1], dof[1], [&](int sl) __attribute__((always_inline)) {
      if (sl == 2 && __builtin_expect(valid < 32, 0)) mask_tail(s0);
      if (sl >= 2) element(s0, dp0, 0, dsw0, sl - 2);
      if (sl >= 14) element(s0, dp0, 0, dsw0, sl);             // sixteen elements in fourteen slots
    });
    // second products: transposed K fragments, fetched once and used by both query tiles
    i16x8_t trk[2][DT];
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const uint8_t* t0 = kg + 16 * c2 * ROWB;
        trk[c2][dt] = concat4(lds_read_tr16(reinterpret_cast<const uint16_t*>(t0 + tfo[0][dt])),
                              lds_read_tr16(reinterpret_cast<const uint16_t*>(t0 + tfo[1][dt])));
      }
    __builtin_amdgcn_sched_barrier(0);
    if (__builtin_expect(valid < 32, 0)) {
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
      mask_tail(s1);
    }
#pragma unroll
    for (int sl = 0; sl < 8; ++sl) {
      const int c2 = sl >> 2, dt = sl & 3;
      dqacc[dt][0] = E::mfma32(trk[c2][dt], __builtin_bit_cast(i16x8_t, dsw0[c2]), dqacc[dt][0]);
      // This unit's V has been used up, its K is in registers (or on its way there): their generation takes the unit
      // after next, a unit and a half before it is wanted.  One request per product: requests that follow each other
      // closely wait for the compute unit's one vector-memory path, and a single wave waits with them.  V first.
      {
        const uint32_t off = koff[sl & 3] + (uint32_t)key0_next2 * row_bytes + (uint32_t)(sl >> 2) * 16 * row_bytes;
        lds_dma_b128(vh, off, smem_addr, (2 + GEN) * TILE + sl * 1024);
      }
      if (sl >= 2) {
        element(s1, dp1, 1, dsw1, 2 * (sl - 2));
        element(s1, dp1, 1, dsw1, 2 * (sl - 2) + 1);
      }
      if (sl >= 6) {
        element(s1, dp1, 1, dsw1, 12 + 2 * (sl - 6));
        element(s1, dp1, 1, dsw1, 13 + 2 * (sl - 6));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int sl = 0; sl < 8; ++sl) {
      const int c2 = sl >> 2, dt = sl & 3;
      dqacc[dt][1] = E::mfma32(trk[c2][dt], __builtin_bit_cast(i16x8_t, dsw1[c2]), dqacc[dt][1]);
      if (sl == 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");        // (every read of K has long returned)
      const uint32_t off = koff[sl & 3] + (uint32_t)key0_next2 * row_bytes + (uint32_t)(sl >> 2) * 16 * row_bytes;
      lds_dma_b128(kh, off, smem_addr, GEN * TILE + sl * 1024);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  int key_cur = 0, key_n1 = 0;
  if (nunits > 0) {
    key_cur = unit_rows(0);
    key_n1 = unit_rows(1);
    request(key_cur, 0);
    request(key_n1, 1);
  }
  // delta of this lane's two rows.  The sum runs in the order of bwd_delta_kernel, whose thread t adds the eight products
  // of columns 8t .. 8t+7 one after the other and then meets threads t^1, t^2, t^4, t^8: here t = 2c + g, so the first
  // meeting is the one with lane^32 and the other three are between this lane's own chunks.
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    float part[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      float acc = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += E::to_float((uint16_t)of[qt][c][e]) * E::to_float((uint16_t)dof[qt][c][e]);
      part[c] = acc + __shfl_xor(acc, 32);
    }
#pragma unroll
    for (int sh = 1; sh < DC; sh <<= 1)
#pragma unroll
      for (int c = 0; c < DC; c += 2 * sh) part[c] = part[c] + part[c + sh];
    delta_q[qt] = part[0];
    const int qrow = qrow0 + 32 * qt + r;
    if (g == 0 && qrow < L) delta[(size_t)bh * L + qrow] = part[0];
  }
  // Q^T and dO^T are only ever MFMA operands and are parked in the accumulation registers (the wait for them comes
  // here, behind the first requests for K and V, which only needed the look-up row)
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
#pragma unroll
    for (int c = 0; c < DC; ++c) asm volatile("" : "+a"(qf[qt][c]), "+a"(dof[qt][c]));
  for (int u = 0; u < nunits; u += 2) {
    const int key_n2 = unit_rows(u + 2), key_n3 = unit_rows(u + 3);
    unit(0, key_cur, key_n2);
    unit(1, key_n1, key_n3);
    key_cur = key_n2;
    key_n1 = key_n3;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // (nothing of this workgroup is in flight when it ends)

  // The rounded rows go through LDS (the rings are free now) and leave as whole rows in streaming stores: they are not
  // read again here, and what does not stay behind as modified lines in L2 need not be written back when the kernel ends.
  uint16_t* const stage = reinterpret_cast<uint16_t*>(smem);
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    constexpr int SSTR = TileRows<D>::SSTR;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        i32x2_t wv;
        wv[0] = (int)E::pack2(dqacc[dt][qt][4 * i4 + 0] * qk_scale, dqacc[dt][qt][4 * i4 + 1] * qk_scale);
        wv[1] = (int)E::pack2(dqacc[dt][qt][4 * i4 + 2] * qk_scale, dqacc[dt][qt][4 * i4 + 3] * qk_scale);
        *reinterpret_cast<i32x2_t*>(&stage[r * SSTR + 32 * dt + 8 * i4 + 4 * g]) = wv;
      }
    wave_lds_fence();
    TileRows<D> t;
    t.unpark(stage, lane);
    t.store_streaming(dq + head_off + (size_t)(qrow0 + 32 * qt) * pitch, L - qrow0 - 32 * qt, lane, pitch);
    wave_lds_fence();
  }
}

}  // namespace sla
