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
// K/V tiles go global -> registers -> LDS; the next tile's K is in flight during QK^T and
// softmax, its V during PV.  Register use is held to 256 so two waves share a SIMD and one
// wave's softmax (vector ALU) overlaps the other's MFMAs (three waves at head dim 64, where the registers allow it:
// 6 % faster there).
#include "linear_state.h"

namespace sla {

// What the fused variant (FUSED = true) adds after the loop: the linear branch of the same query rows,
// out = o_s + (phi(q) KVW / divisor + bias), from the per-head state the linear state kernels left in
// their workspace (kvwt: KVW^T in 16 bit, zst: sum phi(k) in 16 bit).  The state is read from L2 in
// operand order, the raw q fragments are still in registers, and the product costs as many MFMAs as one
// more key tile.  o then receives the sum; o_s (optional) the attention output alone.
template <typename Tag, int D, int BLKQ, bool FUSED>
__global__ __launch_bounds__(BLKQ * 2) __attribute__((amdgpu_waves_per_eu(D == 64 ? 3 : 2, D == 64 ? 3 : 2))) void sparse_fwd_kernel(const uint16_t* __restrict__ q,
                                                              const uint16_t* __restrict__ k,
                                                              const uint16_t* __restrict__ v,
                                                              const void* __restrict__ lut, int lut64,
                                                              uint16_t* __restrict__ o, float* __restrict__ lse,
                                                              const RowLayout lin, const RowLayout lout, int L,
                                                              int Mblk, int topk, float scale_log2e, int total,
                                                              const uint16_t* __restrict__ kvwt,
                                                              const uint16_t* __restrict__ zst,
                                                              const float* __restrict__ bias, int fmap,
                                                              uint16_t* __restrict__ o_s) {
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

  __shared__ __attribute__((aligned(16))) uint16_t smem[BLKK * KSTR + BLKK * VSTR];
  uint16_t* const sK = smem;
  uint16_t* const sV = smem + BLKK * KSTR;

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int bh = logical / Mblk;
  const int mb = logical - bh * Mblk;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5;                  // which half of the MFMA contraction slots this lane feeds
  const int r = lane & 31;                  // query column (S^T, O^T) / key row (A operand)

  // q, k, v rows of this head: lin.sl elements apart (D for the contiguous layout); out rows: lout.sl apart
  const size_t head_off = lin.head(bh);
  const uint32_t pitch = (uint32_t)lin.sl;
  const uint32_t head_bytes = lin.head_range_bytes(L, D);
  const __amdgpu_buffer_rsrc_t kh = make_rsrc(k + head_off, head_bytes);
  const __amdgpu_buffer_rsrc_t vh = make_rsrc(v + head_off, head_bytes);

  // This wave's 32 query rows.  Q comes in and O goes out as whole 256-byte rows (16 adjacent lanes per
  // row) through a wave-private staging tile in LDS: a lane-per-row access pattern would touch 32 memory
  // lines with every instruction.
  const int qrow0 = mb * BLKQ + wave * 32;
  const int qrow = qrow0 + r;
  const int qrows_valid = min(32, L - qrow0);
  uint16_t* const stage = smem + wave * 32 * TileRows<D>::SSTR;
  static_assert(BLKQ / 32 * 32 * TileRows<D>::SSTR <= BLKK * KSTR + BLKK * VSTR, "staging tiles exceed the K/V buffers");
  TileRows<D> qt;
  qt.fetch(q + head_off + (size_t)qrow0 * pitch, qrows_valid, lane, pitch);   // rows past L: 0

  const size_t lut_row = ((size_t)bh * Mblk + mb) * topk;
  auto lut_at = [&](int i) -> int {
    return lut64 ? (int)reinterpret_cast<const long long*>(lut)[lut_row + i]
                 : reinterpret_cast<const int*>(lut)[lut_row + i];
  };

  // One set of staging registers carries K of the next tile during the QK^T phase and V of the
  // next tile during the PV phase (each LDS buffer is free while the other one is being read).
  i16x8_t stg[NLD];
  // chunk i of a thread is row tid / CPR + i * (NT / CPR) of the tile; the per-chunk offsets are formed from one
  // per-lane offset at every use (the opaque copy keeps the compiler from hoisting one register per chunk out
  // of the loop)
  static_assert(NT % CPR == 0, "threads must cover whole rows");
  const uint32_t lane_off = ((uint32_t)(tid / CPR) * pitch + (tid % CPR) * 8) * 2;
  auto load_rows_to = [&](i16x8_t (&dst)[NLD], const __amdgpu_buffer_rsrc_t& base, int nb) {
    uint32_t lo = lane_off + (uint32_t)(nb * BLKK) * pitch * 2;
    asm volatile("" : "+v"(lo));
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      // rows past L lie beyond the buffer range and read as zero (0 * garbage could be NaN)
      dst[i] = buf_load_b128(base, lo + (uint32_t)(i * (NT / CPR)) * pitch * 2);
    }
  };
  auto store_rows_from = [&](const i16x8_t (&src)[NLD], uint16_t* dst, int stride) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int idx = tid + i * NT;
      const int row = idx / CPR, col = (idx % CPR) * 8;
      *reinterpret_cast<i16x8_t*>(&dst[row * stride + col]) = src[i];
    }
  };
  auto load_rows = [&](const __amdgpu_buffer_rsrc_t& base, int nb) { load_rows_to(stg, base, nb); };
  auto store_rows = [&](uint16_t* dst, int stride) { store_rows_from(stg, dst, stride); };

  f32x16_t oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;

  // transposed-read addressing of V: lane i of a 16-lane group points at row i/4, cols 4*(i%4)
  const int tr_row = (lane & 15) >> 2;
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  // look-up-table entries are fetched two tiles ahead so their latency never sits in front of
  // the address computation of the K/V loads
  int nb = topk > 0 ? lut_at(0) : 0;
  int nb_next = topk > 1 ? lut_at(1) : 0;
  // Q and K of the first tile are in flight together; V follows as soon as Q has been parked
  i16x8_t stg_first[NLD];
  if (topk > 0) load_rows_to(stg_first, kh, nb);
  // Q^T fragments (B operand), resident for the whole loop
  qt.park(stage, lane);
  i16x8_t qf[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) qf[c] = *reinterpret_cast<const i16x8_t*>(&stage[r * TileRows<D>::SSTR + 16 * c + 8 * g]);
  if (topk > 0) load_rows(vh, nb);
  __syncthreads();                         // the staging tiles overlap the K buffer
  if (topk > 0) store_rows_from(stg_first, sK, KSTR);
  __syncthreads();

  // Reference maximum of the online softmax.  It is only moved when a sub-tile's maximum exceeds it
  // by more than TAU (in log2 units): probabilities are then at most 2^TAU, exact in fp32 and bf16,
  // and the final 1/l normalisation is unchanged.  Without a per-tile maximum on the critical path
  // the exponentials of one 32-key sub-tile can be issued in the shadow of the other sub-tile's MFMAs.
  constexpr float TAU = 8.0f;
  float m_used = -INFINITY;
  float l_run = 0.f;         // this lane's share of the running sum (its 32 of the 64 key rows)
  i16x8_t pb[2][2];          // packed probabilities of the two sub-tiles, B operands of the PV product

  // moves the reference maximum to at least `mx` (this lane's raw maximum of the sub-tile) and rescales
  // everything accumulated so far; `done` = number of sub-tiles of this tile already exponentiated
  auto raise_reference = [&](float mx, int done) {
    mx = fmaxf(mx, __shfl_xor(mx, 32)) * scale_log2e;
    const float m_new = fmaxf(m_used, mx);
    const float f = fast_exp2(m_used - m_new);     // 0 on the first tile (m_used = -inf)
    m_used = m_new;
    l_run *= f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[dt][i] *= f;
    if (done > 0) {
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        i32x4_t w = __builtin_bit_cast(i32x4_t, pb[0][c2]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t u = (uint32_t)w[j];
          w[j] = (int)E::pack2(E::to_float((uint16_t)(u & 0xffff)) * f, E::to_float((uint16_t)(u >> 16)) * f);
        }
        pb[0][c2] = __builtin_bit_cast(i16x8_t, w);
      }
    }
  };
  // exp2 of one sub-tile against the current reference; adds to l_run; packs into pb[t]
  auto softmax_subtile = [&](f32x16_t& sv, int t) {
    float psum = 0.f;
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2) {
      i32x4_t pw;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p0 = fast_exp2(__builtin_fmaf(sv[8 * c2 + 2 * j], scale_log2e, -m_used));
        const float p1 = fast_exp2(__builtin_fmaf(sv[8 * c2 + 2 * j + 1], scale_log2e, -m_used));
        psum += p0 + p1;
        pw[j] = (int)E::pack2(p0, p1);
      }
      pb[t][c2] = __builtin_bit_cast(i16x8_t, pw);
    }
    l_run += psum;
  };
  auto row_max = [&](const f32x16_t& sv) {
    float mx = sv[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, sv[i]);
    return mx;
  };
  auto mask_tail = [&](f32x16_t& sv, int t, int kv_valid) {
    const int lim = kv_valid - 4 * g;      // key index of register i is 32t + 8(i/4) + i%4 + 4g
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (32 * t + 8 * (i >> 2) + (i & 3) >= lim) sv[i] = -INFINITY;
  };
  auto read_vgroup = [&](int gi, i16x8_t (&vf)[DT]) {   // V^T fragments of 16-key group gi = 2t + c2
    const int key0 = 16 * gi + 4 * g + tr_row;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const uint16_t* p0 = &sV[key0 * VSTR + 32 * dt + tr_col];
      vf[dt] = concat4(lds_read_tr16(p0), lds_read_tr16(p0 + 8 * VSTR));
    }
  };

  for (int it = 0; it < topk; ++it) {
    // here: sK holds K of this tile, the staging registers hold V of this tile, sV is free
    const uint16_t* k0 = &sK[r * KSTR + 8 * g];
    i16x8_t ka[DC], kb[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) ka[c] = *reinterpret_cast<const i16x8_t*>(k0 + 16 * c);
    store_rows(sV, VSTR);
    const int kv_valid = L - nb * BLKK;    // rows of this tile that exist
    const bool tail = kv_valid < BLKK;
    const bool more = it + 1 < topk;
    if (more) {
      nb = nb_next;
      nb_next = it + 2 < topk ? lut_at(it + 2) : 0;
      load_rows(kh, nb);                   // K of the next tile, in flight until the middle of this one
    }

    // ---- A: S0^T = K[0:32] Q^T, with the fragments of K[32:64] fetched in its shadow ----
    f32x16_t s0, s1;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s0[i] = 0.f;
      s1[i] = 0.f;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      kb[c] = *reinterpret_cast<const i16x8_t*>(k0 + 32 * KSTR + 16 * c);
      s0 = E::mfma32(ka[c], qf[c], s0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // rare path (one branch, so the common path stays a straight line): the reference maximum has
    // to move, or this is the partial last key block whose missing rows are masked out first
    if (tail || __any(row_max(s0) * scale_log2e > m_used + TAU)) {
      if (tail) mask_tail(s0, 0, kv_valid);
      raise_reference(row_max(s0), 0);
    }
    __syncthreads();                       // every wave has its K fragments: sK is free; sV stores visible
    if (more) {
      store_rows(sK, KSTR);
      load_rows(vh, nb);                   // V of the next tile, in flight until the top of the next one
    }

    // ---- B: S1^T = K[32:64] Q^T  ||  exponentials of S0 ; V^T fragments of keys 0..31 fetched ----
    // (the group barriers fix the issue order: after every MFMA two LDS reads and seven vector-ALU
    //  instructions, two of them exponentials, are issued while the matrix core works)
    i16x8_t vf0[DT], vf1[DT];
    __builtin_amdgcn_sched_barrier(0);
    read_vgroup(0, vf0);
    read_vgroup(1, vf1);
#pragma unroll
    for (int c = 0; c < DC; ++c) s1 = E::mfma32(kb[c], qf[c], s1);
    softmax_subtile(s0, 0);
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
      __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (tail || __any(row_max(s1) * scale_log2e > m_used + TAU)) {
      if (tail) mask_tail(s1, 1, kv_valid);
      raise_reference(row_max(s1), 1);
    }

    // ---- C: O^T += V[0:32]^T P0^T  ||  exponentials of S1 ; V^T fragments of keys 32..63 fetched ----
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = E::mfma32(vf0[dt], pb[0][0], oacc[dt]);
    read_vgroup(2, vf0);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = E::mfma32(vf1[dt], pb[0][1], oacc[dt]);
    read_vgroup(3, vf1);
    softmax_subtile(s1, 1);
#pragma unroll
    for (int c = 0; c < 2 * DT; ++c) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
      __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- D: O^T += V[32:64]^T P1^T ----
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = E::mfma32(vf0[dt], pb[1][0], oacc[dt]);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = E::mfma32(vf1[dt], pb[1][1], oacc[dt]);
    __syncthreads();                       // sV fully consumed; sK stores visible
  }
  const float m_run = m_used;

  // ---- epilogue ----
  // (lane-derived indices are formed again from an opaque copy of the thread id, so that none of them is
  //  kept in a register, or spilled, across the loop)
  int tid_e = tid;
  asm volatile("" : "+v"(tid_e));
  const int lane_e = tid_e & 63, wave_e = tid_e >> 6;
  const int g_e = lane_e >> 5, r_e = lane_e & 31;
  uint16_t* const stage_e = smem + wave_e * 32 * TileRows<D>::SSTR;
  const int qrow0_e = mb * BLKQ + wave_e * 32;
  const int qrow_e = qrow0_e + r_e;
  const int qrows_valid_e = min(32, L - qrow0_e);
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
  // (the loop ended with a barrier: every wave is done with the K/V buffers, the staging tiles are free)
  constexpr int SSTR = TileRows<D>::SSTR;
  const size_t out_off = lout.head(bh) + (size_t)qrow0_e * (size_t)lout.sl;
  if (qrow_e < L && g_e == 0) lse[(size_t)bh * L + qrow_e] = m_run + fast_log2(l_tot);
  // normalised attention output of this lane, packed, into its row of the staging tile
  auto park_attention = [&]() {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        i32x2_t w;
        w[0] = (int)E::pack2(oacc[dt][4 * i4 + 0] * inv, oacc[dt][4 * i4 + 1] * inv);
        w[1] = (int)E::pack2(oacc[dt][4 * i4 + 2] * inv, oacc[dt][4 * i4 + 3] * inv);
        *reinterpret_cast<i32x2_t*>(&stage_e[r_e * SSTR + 32 * dt + 8 * i4 + 4 * g_e]) = w;
      }
    wave_lds_fence();
  };
  auto flush_rows = [&](uint16_t* dst_tile, size_t dst_pitch) {   // staging tile -> global rows
    TileRows<D> t;
    t.unpark(stage_e, lane_e);
    t.store_streaming(dst_tile, qrows_valid_e, lane_e, dst_pitch);
    wave_lds_fence();
  };
  if (!FUSED) {
    park_attention();
    flush_rows(o + out_off, (size_t)lout.sl);
  } else {
    // ---- linear branch of the same rows ----
    // The per-head state (32 KB) is read straight from L2 in MFMA A-operand order (row 32et + r, 16-byte
    // chunk 2c + g): no staging, no barrier, so the other workgroups of the compute unit keep running
    // their loops while this wave waits for its loads.
    const uint16_t* st_h = kvwt + (size_t)bh * D * D;
    const uint16_t* z_h = zst + (size_t)bh * D;
    // phi(q) from the resident raw q fragments: this lane holds d = 16c + 8g + j of its row
    float f[DC][8];
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)qf[c][j]);
    float row_mx, row_inv;
    phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
    float den = 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      const i16x8_t zc = *reinterpret_cast<const i16x8_t*>(z_h + 16 * c + 8 * g_e);
      i32x4_t pw;
#pragma unroll
      for (int j = 0; j < 8; ++j) den += round16<Tag>(f[c][j] * E::to_float((uint16_t)zc[j]));
#pragma unroll
      for (int j = 0; j < 4; ++j) pw[j] = (int)E::pack2(f[c][2 * j], f[c][2 * j + 1]);
      qf[c] = __builtin_bit_cast(i16x8_t, pw);
    }
    den += __shfl_xor(den, 32);
    den = round16<Tag>(1e-5f + round16<Tag>(den));
    const float inv_den = 1.0f / den;
#pragma unroll
    for (int et = 0; et < DT; ++et) {
      i16x8_t a[DC];
#pragma unroll
      for (int c = 0; c < DC; ++c) a[c] = *reinterpret_cast<const i16x8_t*>(st_h + (size_t)(32 * et + r_e) * D + 16 * c + 8 * g_e);
      f32x16_t acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
      for (int c = 0; c < DC; ++c) acc = E::mfma32(a[c], qf[c], acc);
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int e0 = 32 * et + 8 * i4 + 4 * g_e;
        const f32x4_t b4 = *reinterpret_cast<const f32x4_t*>(bias + e0);
        i32x2_t ws, wo;
        ws[0] = (int)E::pack2(oacc[et][4 * i4 + 0] * inv, oacc[et][4 * i4 + 1] * inv);
        ws[1] = (int)E::pack2(oacc[et][4 * i4 + 2] * inv, oacc[et][4 * i4 + 3] * inv);
        // the sum as the reference's tensor addition forms it: both summands in 16 bit, one rounded add
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint32_t x = (uint32_t)ws[h];
          const float l0 = round16<Tag>(pin_f32(__builtin_fmaf(acc[4 * i4 + 2 * h], inv_den, round16<Tag>(b4[2 * h]))));
          const float l1 = round16<Tag>(pin_f32(__builtin_fmaf(acc[4 * i4 + 2 * h + 1], inv_den, round16<Tag>(b4[2 * h + 1]))));
          wo[h] = (int)E::pack2(E::to_float((uint16_t)(x & 0xffff)) + l0, E::to_float((uint16_t)(x >> 16)) + l1);
        }
        *reinterpret_cast<i32x2_t*>(&stage_e[r_e * SSTR + e0]) = wo;
      }
    }
    wave_lds_fence();
    flush_rows(o + out_off, (size_t)lout.sl);
    if (o_s) {                 // (kept for a backward: always the contiguous (B, H, L, D) tensor)
      park_attention();
      flush_rows(o_s + ((size_t)bh * L + qrow0_e) * D, D);
    }
  }
}

}  // namespace sla
#include "sparse_fwd_pair.h"
namespace sla {

struct FusedLinear {        // state of the linear branch for the fused epilogue (all null / 0 when not fused)
  const uint16_t* kvwt;
  const uint16_t* zst;
  const float* bias;
  int fmap;
  uint16_t* o_s;
};

template <typename Tag>
static int launch_fwd(const void* q, const void* k, const void* v, const void* lut, int lut64, void* o, float* lse,
                      const RowLayout& lin, const RowLayout& lout, int BH, int L, int D, int BLKQ, int topk, float qk_scale,
                      const FusedLinear* fl, hipStream_t st) {
  const int Mblk = cdiv(L, BLKQ);
  const int64_t total64 = (int64_t)BH * Mblk;
  const int total = (int)total64;
  const int grid = xcd_grid(total);
  const float c = qk_scale * 1.4426950408889634f;
  // The common shape (head dim 128, 64-row query blocks) has a kernel of its own, which shares key blocks between
  // neighbouring query blocks; it addresses a head with 32-bit byte offsets and indexes key blocks with 12 bits.
  // (Two query blocks per workgroup halve the number of workgroups: a launch too small to give every compute unit
  // its two workgroups keeps one query block per workgroup.)
  // 128-row query blocks go the same way: the two halves of a block are a pair whose rows of the table are one row.
  const int Mblk64 = cdiv(L, 64);
  const int total_p = BH * ((Mblk64 + 1) / 2);
  if (D == 128 && (BLKQ == 64 || BLKQ == 128) && topk <= PAIR_MAX_T && Mblk64 <= 4096 &&
      (uint64_t)lin.sl * 2u * (uint64_t)L < (1ull << 31) && total_p >= 512) {
    const int grid_p = xcd_grid(total_p);
    const int one_row = BLKQ == 128;
    if (fl)
      hipLaunchKernelGGL((sparse_fwd_pair_kernel<Tag, true>), dim3(grid_p), dim3(256), 0, st, (const uint16_t*)q,
                         (const uint16_t*)k, (const uint16_t*)v, lut, lut64, (uint16_t*)o, lse, lin, lout, L, Mblk64, topk, c,
                         total_p, fl->kvwt, fl->zst, fl->bias, fl->fmap, fl->o_s, one_row);
    else
      hipLaunchKernelGGL((sparse_fwd_pair_kernel<Tag, false>), dim3(grid_p), dim3(256), 0, st, (const uint16_t*)q,
                         (const uint16_t*)k, (const uint16_t*)v, lut, lut64, (uint16_t*)o, lse, lin, lout, L, Mblk64, topk, c,
                         total_p, (const uint16_t*)nullptr, (const uint16_t*)nullptr, (const float*)nullptr, 0,
                         (uint16_t*)nullptr, one_row);
    return check_launch("sparse_attn_fwd");
  }
#define SLA_FWD_CASE(DD, BQ)                                                                                          \
  if (D == DD && BLKQ == BQ) {                                                                                        \
    if (fl)                                                                                                           \
      hipLaunchKernelGGL((sparse_fwd_kernel<Tag, DD, BQ, true>), dim3(grid), dim3(BQ * 2), 0, st, (const uint16_t*)q, \
                         (const uint16_t*)k, (const uint16_t*)v, lut, lut64, (uint16_t*)o, lse, lin, lout, L, Mblk,   \
                         topk, c, total, fl->kvwt, fl->zst, fl->bias, fl->fmap, fl->o_s);                             \
    else                                                                                                              \
      hipLaunchKernelGGL((sparse_fwd_kernel<Tag, DD, BQ, false>), dim3(grid), dim3(BQ * 2), 0, st,                   \
                         (const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, lut, lut64, (uint16_t*)o, lse,  \
                         lin, lout, L, Mblk, topk, c, total, (const uint16_t*)nullptr, (const uint16_t*)nullptr,      \
                         (const float*)nullptr, 0, (uint16_t*)nullptr);                                               \
    return check_launch("sparse_attn_fwd");                                                                           \
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
  SLA_REQUIRE((int64_t)(L + 128) * D * 2 < (1ll << 32), SLA_ERR_UNSUPPORTED, "one head exceeds 4 GiB");
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
  const RowLayout lay = contiguous_layout(H, L, D);
  if (dtype == SLA_BF16)
    return launch_fwd<bf16_tag>(q, k, v, lut, lut_elem_bytes == 8, o, lse, lay, lay, BH, L, D, BLKQ, topk, qk_scale, nullptr,
                                st);
  return launch_fwd<f16_tag>(q, k, v, lut, lut_elem_bytes == 8, o, lse, lay, lay, BH, L, D, BLKQ, topk, qk_scale, nullptr, st);
}

static int attn_linear_entry(const void* q, const void* k, const void* v, const int64_t* qkv_strides, const void* lut,
                             int lut_elem_bytes, const void* linear_workspace, int64_t linear_workspace_bytes,
                             const float* bias, void* o_s, void* out, const int64_t* out_strides, float* lse, int dtype,
                             int fmap, int B, int H, int L, int D, int BLKQ, int BLKK, int topk, float qk_scale,
                             void* stream) {
  int rc = validate_attn_shape(dtype, B, H, L, D, BLKQ, BLKK, topk, lut_elem_bytes);
  if (rc) return rc;
  rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  SLA_REQUIRE(q && k && v && out && lse && bias && linear_workspace && (lut || topk == 0), SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)o_s | (uintptr_t)linear_workspace) %
                      16 == 0,
              SLA_ERR_BAD_ARG, "q, k, v, out, o_s, workspace must be 16-byte aligned");
  const int BH = B * H;
  const LinWs w = lin_ws(BH, L, D);
  SLA_REQUIRE(linear_workspace_bytes >= (int64_t)w.total, SLA_ERR_WORKSPACE, "workspace of %lld bytes, need %lld",
              (long long)linear_workspace_bytes, (long long)w.total);
  const char* ws = (const char*)linear_workspace;
  FusedLinear fl{(const uint16_t*)(ws + w.kvwt), (const uint16_t*)(ws + w.z), bias, fmap, (uint16_t*)o_s};
  RowLayout lin, lout;
  rc = make_layout(qkv_strides, B, H, L, D, 2, &lin);
  if (rc) return rc;
  rc = make_layout(out_strides, B, H, L, D, 2, &lout);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == SLA_BF16)
    return launch_fwd<bf16_tag>(q, k, v, lut, lut_elem_bytes == 8, out, lse, lin, lout, BH, L, D, BLKQ, topk, qk_scale, &fl,
                                st);
  return launch_fwd<f16_tag>(q, k, v, lut, lut_elem_bytes == 8, out, lse, lin, lout, BH, L, D, BLKQ, topk, qk_scale, &fl, st);
}

extern "C" int sla_sparse_attn_linear_fwd(const void* q, const void* k, const void* v, const void* lut, int lut_elem_bytes,
                                          const void* linear_workspace, int64_t linear_workspace_bytes, const float* bias,
                                          void* o_s, void* out, float* lse, int dtype, int fmap, int B, int H, int L, int D,
                                          int BLKQ, int BLKK, int topk, float qk_scale, void* stream) {
  return attn_linear_entry(q, k, v, nullptr, lut, lut_elem_bytes, linear_workspace, linear_workspace_bytes, bias, o_s, out,
                           nullptr, lse, dtype, fmap, B, H, L, D, BLKQ, BLKK, topk, qk_scale, stream);
}

extern "C" int sla_sparse_attn_linear_fwd_strided(const void* q, const void* k, const void* v, const int64_t* qkv_strides,
                                                  const void* lut, int lut_elem_bytes, const void* linear_workspace,
                                                  int64_t linear_workspace_bytes, const float* bias, void* o_s, void* out,
                                                  const int64_t* out_strides, float* lse, int dtype, int fmap, int B, int H,
                                                  int L, int D, int BLKQ, int BLKK, int topk, float qk_scale,
                                                  void* stream) {
  SLA_REQUIRE(qkv_strides && out_strides, SLA_ERR_BAD_ARG, "null strides");
  return attn_linear_entry(q, k, v, qkv_strides, lut, lut_elem_bytes, linear_workspace, linear_workspace_bytes, bias, o_s,
                           out, out_strides, lse, dtype, fmap, B, H, L, D, BLKQ, BLKK, topk, qk_scale, stream);
}
