// Block-sparse FlashAttention forward for 64-row query blocks at head dim 128: two adjacent query blocks per
// workgroup, one wavefront per query block.
//
// Stands in for _attn_fwd of the reference (sparse_linear_attention/kernel.py:21-82) like sparse_fwd_kernel,
// whose arithmetic it shares (S^T = K Q^T, thresholded reference maximum, P^T as B operand of O^T = V^T P^T).
// What differs is who shares what:
//   * a wave owns all 64 rows of its query block (two 32-row tiles), so every K fragment and every V^T fragment
//     read from LDS feeds two MFMAs: half the LDS reads per MFMA of the 32-rows-per-wave kernel;
//   * neighbouring query blocks select mostly the same key blocks.  The two look-up rows of a pair are split
//     into the key blocks both selected ("shared": one copy of the tile in LDS for both waves) and the rest
//     ("own": as many on either side, each wave walks its own, two tiles in LDS), interleaved in the order of
//     the first row.  A pair that shares 19 of 25 key blocks moves 31 tiles instead of 50 from L2 into LDS;
//   * a wave has the whole register file of its SIMD (one wave per SIMD): the next half-tiles of K and V wait
//     in registers for a whole half-tile of arithmetic before they are needed, and the loop is rotated so that
//     the exponentials of half-tile u run beside the score products of u+1 and the output products of u.
// The unit of the loop is a half-tile of 32 keys.  K half-tiles live in a two-generation ring in LDS (u even /
// odd), V half-tiles likewise; each generation has two slots (slot 0: shared tile or wave 0's own, slot 1: wave
// 1's own).  Tiles go from global memory straight into LDS (buffer loads with the LDS bit: no staging registers, no
// LDS store instructions - a single wave per SIMD is bound by the instructions it has to issue, and a 16-byte LDS
// store costs as many issue cycles as five vector-ALU instructions).  Rows are unpadded in LDS; the 16-byte slots
// of a row are XOR-swizzled with the row index (by choosing which global piece a lane fetches), so that both the
// 128-bit row reads of K and the transposing reads of V are free of bank conflicts.  One workgroup barrier per unit.
// Minus the reference maximum (in the units of q . k) is the C operand of the first score product of a chain: what
// is left per score is one fp32 multiply by qk_scale * log2(e) before the exponential.  (Scaling Q instead, once, and
// rounding it to 16 bit again would spare that multiply and shift the log-sum-exp by up to 0.02: too much for the
// backward pass, which forms its probabilities from it.)
#pragma once
#include "linear_state.h"

namespace sla {

constexpr int PAIR_MAX_T = 1024;      // look-up rows longer than this, or more than 4096 key blocks, take sparse_fwd_kernel

template <typename Tag, bool FUSED>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(1, 1))) void sparse_fwd_pair_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, const void* __restrict__ lut,
    int lut64, uint16_t* __restrict__ o, float* __restrict__ lse, const RowLayout lin, const RowLayout lout, int L, int Mblk,
    int topk, float scale_log2e, int total, const uint16_t* __restrict__ kvwt, const uint16_t* __restrict__ zst,
    const float* __restrict__ bias, int fmap, uint16_t* __restrict__ o_s, int one_row) {
  using E = Elem<Tag>;
  constexpr int D = 128, DC = D / 16, DT = D / 32;
  constexpr int ROWB = D * 2;                         // bytes per row in LDS (unpadded)
  constexpr int SLOT = 32 * ROWB;                     // one half-tile: 8 KB
  constexpr int SSTR = TileRows<D>::SSTR;
  constexpr float PLIM = 1024.0f;   // a lane's 16 probabilities of a sub-tile may sum to this before the reference moves
  typedef __attribute__((address_space(3))) void lds_void;

  // K ring: [generation][slot] at (2 gen + slot) * SLOT; V ring: the same, 4 * SLOT further on
  __shared__ __attribute__((aligned(16))) uint8_t smem[8 * SLOT];
  __shared__ uint32_t bitmap[2][128];
  __shared__ uint16_t steps[2][PAIR_MAX_T];
  __shared__ uint16_t own_b[PAIR_MAX_T];        // the key blocks only the second row names (wave 1's scratch)
  __shared__ int repeated;
  static_assert(2 * 32 * SSTR * 2 <= 4 * SLOT, "the staging tiles of the epilogue exceed the K ring");

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int Mpair = (Mblk + 1) >> 1;
  const int bh = logical / Mpair;
  const int pj = logical - bh * Mpair;
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, r = lane & 31;
  const bool pair_full = 2 * pj + 1 < Mblk;            // the last block of a head with an odd block count has no partner:
  const int mb = (w == 1 && pair_full) ? 2 * pj + 1 : 2 * pj;   // wave 1 then repeats wave 0's block and stores nothing
  const bool writes = w == 0 || pair_full;

  const size_t head_off = lin.head(bh);
  const uint32_t pitch = (uint32_t)lin.sl;
  const uint32_t head_bytes = lin.head_range_bytes(L, D);
  const __amdgpu_buffer_rsrc_t kh = make_rsrc(k + head_off, head_bytes);
  const __amdgpu_buffer_rsrc_t vh = make_rsrc(v + head_off, head_bytes);

  // ---- the two look-up rows -> per-wave step lists
  // (one_row: the pair is one 128-row query block of the caller's, whose look-up table has one row per pair: both
  //  halves follow it, and every step is a shared one)
  const size_t rowA = one_row ? ((size_t)bh * Mpair + pj) * topk : ((size_t)bh * Mblk + 2 * pj) * topk;
  const size_t rowB = (pair_full && !one_row) ? rowA + topk : rowA;
  auto lut_at = [&](size_t i) __attribute__((always_inline)) -> int {       // (the low word of a 64-bit entry)
    return reinterpret_cast<const int*>(lut)[lut64 ? 2 * i : i];
  };
  // The first 64 entries of both rows are asked for before anything else: the schedule of the pair hangs on them, and
  // loads come back in the order they were issued.  They stay in registers for the passes below (lanes past the end
  // of a row hold its last entry and are not looked at).
  int a_raw = 0, b_raw = 0;
  if (topk > 0) {                              // (an empty look-up table may be a null pointer)
    a_raw = lut_at(rowA + min(lane, topk - 1));
    b_raw = lut_at(rowB + min(lane, topk - 1));
  }
  // This wave's 64 query rows are requested next, straight in B-operand order (lane = row, 16 bytes per 16-wide
  // chunk of the head dim): they arrive while the look-up rows are merged.  (A lane-per-row access touches 32 memory
  // lines per instruction; it happens once per workgroup and spares a trip through LDS and a barrier.)
  const int qrow0 = mb * 64;
  uint16_t* const stage = reinterpret_cast<uint16_t*>(smem) + w * 32 * SSTR;   // wave-private staging tile of the epilogue, 32 rows (overlaps the K ring)
  i16x8_t qf[2][DC];
  {
    const __amdgpu_buffer_rsrc_t qh = make_rsrc(q + head_off, head_bytes);
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int c = 0; c < DC; ++c)
        qf[qt][c] = buf_load_b128(qh, ((uint32_t)(qrow0 + 32 * qt + r) * pitch + 16 * c + 8 * g) * 2);   // rows past L: 0
  }
  // rows past L are never written into LDS; where V is concerned what LDS holds there meets a probability of exactly
  // 0 and must not be a NaN pattern left behind by an earlier kernel: a ragged sequence starts from a zeroed V ring
  if (L % 64 != 0) {
#pragma unroll
    for (int i = 0; i < 4 * SLOT / (128 * 16); ++i) reinterpret_cast<i32x4_t*>(smem + 4 * SLOT)[i * 128 + tid] = i32x4_t{0, 0, 0, 0};
  }

  // ---- per-wave step lists
  // (The split assumes what the mask builder guarantees: no key block twice in a row, every index below 4096.  A row
  //  that names a block twice makes the pair walk both rows unshared, in the order given, each block as often as it
  //  is named; an index is only ever used modulo 4096 here, and as it is where the rows of K and V are addressed,
  //  where the buffer bounds apply.)
  bitmap[0][tid] = 0;
  bitmap[1][tid] = 0;
  if (tid == 0) repeated = 0;
  __syncthreads();
  // Every wave reads both rows and marks its own row's blocks.
  for (int c0 = 0; c0 < topk; c0 += 64) {
    const int i = c0 + lane;
    if (i < topk) {
      const int a = (c0 == 0 ? a_raw : lut_at(rowA + i)) & 4095, b = (c0 == 0 ? b_raw : lut_at(rowB + i)) & 4095;
      const int x = w ? b : a;
      const uint32_t seen = atomicOr(&bitmap[w][x >> 5], 1u << (x & 31));
      if ((seen >> (x & 31)) & 1u) repeated = 1;
    }
  }
  __syncthreads();
  auto row_a = [&](int c0, int i) __attribute__((always_inline)) -> int {
    return c0 == 0 ? (a_raw & 4095) : (i < topk ? lut_at(rowA + i) & 4095 : 0);
  };
  auto row_b = [&](int c0, int i) __attribute__((always_inline)) -> int {
    return c0 == 0 ? (b_raw & 4095) : (i < topk ? lut_at(rowB + i) & 4095 : 0);
  };
  // Step p of the pair follows entry p of the first row: a key block the second row names as well is a shared step;
  // otherwise it is an own step, on which wave 0 takes that block and wave 1 the next block (in the order of its row)
  // that only the second row names: both rows have as many of those.  Key blocks so come in the order of the look-up
  // rows, ascending as the mask builder writes them, and the pairs that are resident on an XCD sweep K and V together.
  // Bit 15 of a step marks an own step.
  if (repeated) {
    const size_t rowW = w ? rowB : rowA;
    for (int i = lane; i < topk; i += 64) steps[w][i] = (uint16_t)((lut_at(rowW + i) & 4095) | 0x8000);
  } else {
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    if (w == 1) {                                // the second row's own blocks, in its order
      int n = 0;
      for (int c0 = 0; c0 < topk; c0 += 64) {
        const int i = c0 + lane;
        const int x = row_b(c0, i);
        const bool sel = i < topk && !((bitmap[0][x >> 5] >> (x & 31)) & 1u);
        const unsigned long long bal = __ballot(sel);
        if (sel) own_b[n + __popcll(bal & lt_mask)] = (uint16_t)x;
        n += __popcll(bal);
      }
      wave_lds_fence();
    }
    int n = 0;                                   // own steps before this chunk
    for (int c0 = 0; c0 < topk; c0 += 64) {
      const int i = c0 + lane;
      const int a = row_a(c0, i);
      const bool own = i < topk && !((bitmap[1][a >> 5] >> (a & 31)) & 1u);
      const unsigned long long bal = __ballot(own);
      if (i < topk) {
        int tile = a;
        if (own && w == 1) tile = own_b[n + __popcll(bal & lt_mask)];
        steps[w][i] = (uint16_t)(tile | (own ? 0x8000 : 0));
      }
      n += __popcll(bal);
    }
  }

  f32x16_t oacc[DT][2];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[dt][qt][i] = 0.f;
  // Reference maximum of the online softmax, in the exponent's units; minus the reference in all sixteen registers of
  // a tuple that is the C operand of the first score product of every chain.  The reference starts at 0 and the first
  // unit always takes the path that moves it.
  float m_used[2] = {0.f, 0.f};
  float l_run[2] = {0.f, 0.f};
  f32x16_t negm[2];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
#pragma unroll
    for (int i = 0; i < 16; ++i) negm[qt][i] = 0.f;

  // ---- addressing ----
  // unit u = 2 * step + half.  Shared steps: one tile, slot 0, wave w fetches rows 16w..16w+15 of the half-tile
  // (4 instructions of 1 KB for K, 4 for V).  Own steps: slot w, the wave fetches all 32 rows (8 + 8 instructions).
  // Instruction i of a half-tile fills LDS rows 4i..4i+3: lane -> row 4i + lane / 16, 16-byte slot lane % 16, which
  // receives piece (slot ^ swizzle(row)) of that row.  K: swizzle = row % 16 (the 16 rows of a row-wise read hit 16 different
  // slots); V: 4 (row % 4) + (row / 4) % 2 (so do the 4 rows x 4 pieces of a transposing read).
  // A single wave per SIMD pays issue time for every instruction, scalar ones included, so everything that does not
  // change inside the loop is formed here: per instruction there is one vector add (lane part + scalar row base), one
  // scalar add into M0 (LDS destination) and the load.
  const int nunits = 2 * topk;
  const int lrow = lane >> 4, lslot = lane & 15;
  const uint32_t smem_addr = (uint32_t)(size_t)smem;      // LDS address of the rings
  const uint32_t row_bytes = pitch * 2;                   // bytes between rows in memory
  uint32_t koff[4], voff[4];          // lane part of the byte offset of instruction j (mod 4): row 4j + lane / 16, swizzled piece
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    koff[j] = (uint32_t)(4 * j + lrow) * row_bytes + ((lslot ^ ((4 * j + lrow) & 15)) * 16);
    voff[j] = (uint32_t)(4 * j + lrow) * row_bytes + ((lslot ^ ((((4 * j + lrow) & 3) << 2) | (((4 * j + lrow) >> 2) & 1))) * 16);
  }
  // What the requests of a step need, by kind of step: the byte offset of the first row this wave fetches and the LDS
  // address (inside a slot pair) of its first instruction.
  struct Step {
    int tile;          // key block
    int own;           // 0: shared step, 1: own step
    uint32_t rb;       // byte offset in the head of the first row this wave fetches of half 0
    uint32_t dst;      // LDS byte address, relative to a generation's slot pair, of this wave's first instruction
  };
  auto step_of = [&](int entry) __attribute__((always_inline)) -> Step {
    const int own = entry >> 15, tile = entry & 4095;
    return Step{tile, own, (uint32_t)(tile * 64 + (own ? 0 : 16 * w)) * row_bytes,
                smem_addr + (uint32_t)(own ? w * SLOT : 4 * w * 1024)};
  };
  auto step_lookup = [&](int s_raw) __attribute__((always_inline)) -> int {       // (per lane; made scalar where it is used)
    return (int)steps[w][min(s_raw, topk - 1)];         // past the end: the last step again (fetched, never used)
  };
  const uint32_t half_bytes = 32 * row_bytes, quarter_bytes = 16 * row_bytes;
  // one request: 4 rows, global -> LDS.  `ring` = byte offset of the slot pair (generation, K or V) plus the instruction's 1 KB
  // (written as instructions: the compiler would make every later LDS read wait for a load it knows to target LDS;
  //  the wait for these loads is the one before the barrier at the end of an iteration.  Rows past L lie outside the
  //  buffer range: nothing is written for them and LDS keeps what it held, which is either the zeros it was filled
  //  with at the start or rows of an earlier tile: finite values, whose scores are masked and whose probabilities are 0)
#define SLA_PAIR_FETCH(RSRC, LANEOFF, ROWBASE, DST, RING)                                                              \
  do {                                                                                                                 \
    const uint32_t off_ = (LANEOFF) + (ROWBASE);                                                                       \
    asm volatile("s_add_u32 m0, %0, %3\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(DST), "v"(off_), "s"(RSRC),  \
                 "s"((uint32_t)(RING))                                                                                 \
                 : "memory", "scc");                                                                                   \
  } while (0)
  // fragment addressing (bytes from the start of the rings; the slot of the current kind of step is added when the
  // kind changes, once per kernel)
  int kfo[DC];                      // K fragment c of this lane: row r, piece 2c + g
#pragma unroll
  for (int c = 0; c < DC; ++c) kfo[c] = r * ROWB + (((2 * c + g) ^ (r & 15)) * 16);
  const int tr_row = (lane & 15) >> 2;
  const int v_row = 4 * g + tr_row;                  // + 16 * group (+ 8 for the second read)
  const int v_swz = ((v_row & 3) << 2) | ((v_row >> 2) & 1);      // (the same for row + 8)
  int vfo[DT];                      // V^T fragment dt: 8 bytes at element 4 * (lane % 4) of the 16-column strip 2 dt + (lane / 16) % 2
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int piece = 4 * dt + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    vfo[dt] = 4 * SLOT + v_row * ROWB + ((piece ^ v_swz) * 16) + (lane & 1) * 8;
  }
  // The fragment offsets point at the shared slot or at this wave's own slot; they move whenever the kind of the step
  // they read from changes (k_own / v_own: where they point now).
  int k_own = 0, v_own = 0;
  const int ragged_tile = (L & 63) ? (L >> 6) : -1;       // the only key block that can have missing rows

  // ---- pieces of the arithmetic ----
  auto row_max = [&](const f32x16_t& sv) __attribute__((always_inline)) {
    float mx = sv[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, sv[i]);
    return mx;
  };
  auto mask_tail = [&](f32x16_t& sv, int valid) __attribute__((always_inline)) {          // rows of this half-tile at or past `valid` do not exist
    const int lim = valid - 4 * g;                         // key index of register i is 8(i/4) + i%4 + 4g
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (8 * (i >> 2) + (i & 3) >= lim) sv[i] = -INFINITY;
  };
  // Moves the reference of query tile qt up to the maximum of sub-tile sv (whose registers hold score - old reference);
  // rescales what has been accumulated, re-bases sv and the already formed scores of the next unit (sn).
  auto raise_reference = [&](f32x16_t& sv, f32x16_t& sn, int qt, bool first) __attribute__((always_inline)) {
    float mx = row_max(sv);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float up = first ? mx : fmaxf(mx, 0.f);          // new reference - old reference
    const float f = first ? 0.f : fast_exp2(-up * scale_log2e);
    m_used[qt] += up;
    l_run[qt] *= f;
    // The output accumulators live in the accumulation registers and, on the common path, are only ever touched by
    // MFMAs.  They are scaled in place through one temporary, so that the register allocator has no reason to
    // move the whole accumulator through the vector registers around the loop.  (Not on the first unit, which every
    // wave sends through here to set its reference: nothing has been accumulated yet, and 64 registers times zero
    // would be 200 instructions for nothing.)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");     // (the last products into these registers and into sn have landed)
    if (!first) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float x = oacc[dt][qt][i], t;
          asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1"
                       : "+a"(x), "=&v"(t)
                       : "v"(f));
          oacc[dt][qt][i] = x;
        }
    }
    const float nm = -m_used[qt];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      sv[i] -= up;
      // (in place: written as a plain subtraction the compiler keeps the re-based scores in other registers than the
      //  scores, and pays for it with sixteen copies on the path that does not come here)
      float x = sn[i];
      asm volatile("v_sub_f32 %0, %0, %1" : "+v"(x) : "v"(up));
      sn[i] = x;
      float y = negm[qt][i];
      asm volatile("v_mov_b32 %0, %1" : "+v"(y) : "v"(nm));
      negm[qt][i] = y;
    }
  };
  auto zero16 = [&](f32x16_t& x) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] = 0.f;
  };
  auto read_k = [&](int gen, i16x8_t (&kf)[DC]) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < DC; ++c) kf[c] = *reinterpret_cast<const i16x8_t*>(smem + gen * 2 * SLOT + kfo[c]);
  };

  // ---- prologue: K_0, V_0, K_1 into LDS; S_0 ----
  f32x16_t s_a[2], s_b[2];        // scores of the current and of the next unit, swapping roles every iteration
  i16x8_t kf[DC];
  i16x8_t vf_a[2][DT], vf_b[2][DT];   // V^T fragments of the even / odd unit: [16-key group][32 output channels]
  i32x4_t pbw[2][2];                  // packed probabilities: [query tile][16-key group]
#pragma unroll
  for (int c2 = 0; c2 < 2; ++c2) {
    pbw[1][c2] = i32x4_t{0, 0, 0, 0};             // the first iteration's left-over products add nothing
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vf_b[c2][dt] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
  }
  Step cur{0, 0, 0, 0}, nxt{0, 0, 0, 0};
  if (nunits > 0) {
    cur = step_of(__builtin_amdgcn_readfirstlane(step_lookup(0)));
    nxt = step_of(__builtin_amdgcn_readfirstlane(step_lookup(1)));
    // K_0, V_0 (generation 0) and K_1 (generation 1) of the first step
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      SLA_PAIR_FETCH(kh, koff[j], cur.rb, cur.dst, 0 * SLOT + j * 1024);
      SLA_PAIR_FETCH(vh, voff[j], cur.rb, cur.dst, 4 * SLOT + j * 1024);
      SLA_PAIR_FETCH(kh, koff[j], cur.rb + half_bytes, cur.dst, 2 * SLOT + j * 1024);
    }
    if (cur.own) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        SLA_PAIR_FETCH(kh, koff[j], cur.rb + quarter_bytes, cur.dst, 0 * SLOT + 4096 + j * 1024);
        SLA_PAIR_FETCH(vh, voff[j], cur.rb + quarter_bytes, cur.dst, 4 * SLOT + 4096 + j * 1024);
        SLA_PAIR_FETCH(kh, koff[j], cur.rb + half_bytes + quarter_bytes, cur.dst, 2 * SLOT + 4096 + j * 1024);
      }
#pragma unroll
      for (int c = 0; c < DC; ++c) kfo[c] += w * SLOT;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) vfo[dt] += w * SLOT;
      k_own = v_own = 1;
    }
  }
  // Q is only ever an MFMA operand (unscaled: the scores stay in the units of q . k, the reference maximum too, and
  // qk_scale * log2(e) multiplies the exponent's argument in fp32) and is parked in the accumulation registers: the
  // vector registers are left for the score tiles, the fragments and the softmax arithmetic
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
#pragma unroll
    for (int c = 0; c < DC; ++c) asm volatile("" : "+a"(qf[qt][c]));
  if (nunits > 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    read_k(0, kf);
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {
        if (c == 0) mfma_scores_first<Tag>(s_a[qt], kf[c], qf[qt][c]);
        else mfma_scores<Tag>(s_a[qt], kf[c], qf[qt][c]);
      }
  }

  // One iteration = unit u, 32 MFMAs, every one of them followed by its share of the other work (the order is pinned
  // slot by slot: a single wave per SIMD has nobody else to fill its gaps):
  //   slots  0.. 7  O^T(query tile 1) += V_{u-1}^T P_{u-1}^T   (left over from the previous unit; operands in registers)
  //                 beside: exponentials of (u, query tile 0).  Before slot 4: wait for the requests of the previous
  //                 iteration, one barrier (the four products already queued keep the matrix pipe busy meanwhile).
  //                 From slot 4: K_{u+2} and V_{u+1} requested (memory -> LDS), fragments of K_{u+1}, then of V_u,
  //                 fetched from LDS
  //   slots  8..23  S_{u+1} = K_{u+1} Q^T (two chains)          beside: exponentials of (u, tile 0), then of (u, tile 1)
  //   slots 24..31  O^T(query tile 0) += V_u^T P_u^T            beside: rest of the exponentials of (u, tile 1)
  // After the barrier LDS holds K_{u+1} (generation (u+1)&1) and V_u (generation u&1); on entry s_cur = scores of u
  // minus the reference.  Unit u is half HALF of step `cur`; the half after it belongs to `cur` (HALF 0) or to `nxt`
  // (HALF 1).
  int step_index = 0;
  float e0 = 0.f, e1 = 0.f;           // one pair of exponentials on its way from the exponent to the packing
  auto pair_exp = [&](const f32x16_t& sv, int j) __attribute__((always_inline)) {
    e0 = fast_exp2(sv[2 * j] * scale_log2e);
    e1 = fast_exp2(sv[2 * j + 1] * scale_log2e);
    asm volatile("" : "+v"(e0), "+v"(e1));         // (stays in its slot: nothing moves this work towards its first use)
  };
  auto pair_pack = [&](int qt, int j, float& psum) __attribute__((always_inline)) {
    uint32_t pw = E::pack2(e0, e1);
    psum += e0 + e1;                               // (plain adds: a dot-product instruction beside the MFMAs stalls the matrix pipe)
    asm volatile("" : "+v"(pw), "+v"(psum));
    pbw[qt][j >> 2][j & 3] = (int)pw;
  };
  auto softmax_again = [&](const f32x16_t& sv, int qt) __attribute__((always_inline)) -> float {     // (rare path) all eight pairs of a sub-tile
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      pair_exp(sv, j);
      pair_pack(qt, j, psum);
    }
    return psum;
  };
  float ps_seed = INFINITY;
  auto iteration = [&](int HALF, f32x16_t (&s_cur)[2], f32x16_t (&s_nxt)[2], i16x8_t (&vf_prev)[2][DT],
                       i16x8_t (&vf_cur)[2][DT]) __attribute__((always_inline)) {
    const int gen = HALF;                          // generation of K_u / V_u; K_{u+1} lives in the other one
    if (__builtin_expect(cur.tile == ragged_tile, 0)) {
      const int valid = L - (cur.tile * 64 + 32 * HALF);   // rows of this half-tile that exist
      mask_tail(s_cur[0], valid);
      mask_tail(s_cur[1], valid);
    }
    // requests: K_{u+2} is half HALF of step nxt; V_{u+1} is half 1 of cur (HALF 0) or half 0 of nxt (HALF 1)
    const Step& vs = HALF == 0 ? cur : nxt;
    const uint32_t k_rb = nxt.rb + (HALF ? half_bytes : 0u);
    const uint32_t v_rb = vs.rb + (HALF ? 0u : half_bytes);
    // fragment reads: K_{u+1} is half 1 of cur (HALF 0) or half 0 of nxt (HALF 1); V_u is of cur.  Their slot changes
    // when the kind of step does.
    const int k_need = HALF ? nxt.own : cur.own;
    if (__builtin_expect(k_need != k_own, 0)) {
      const int d = k_need ? w * SLOT : -w * SLOT;
#pragma unroll
      for (int c = 0; c < DC; ++c) kfo[c] += d;
      k_own = k_need;
    }
    if (__builtin_expect(cur.own != v_own, 0)) {
      const int d = cur.own ? w * SLOT : -w * SLOT;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) vfo[dt] += d;
      v_own = cur.own;
    }
    // the key block of the step after next is looked up now and used at the end of the odd iteration
    int tile2_lane = 0;
    if (HALF) tile2_lane = step_lookup(step_index + 2);
    // (the first unit's sums start from infinity: that sends it down the path that sets the reference)
    float ps0 = HALF == 0 ? ps_seed : 0.f, ps1 = ps0;
    __builtin_amdgcn_sched_barrier(0);
    // ---- block A: slots 0..23 ----
#pragma unroll
    for (int sl = 0; sl < 24; ++sl) {
      if (sl == 4) {
        // The requests of the previous iteration have had twenty slots to land; four products are queued in the
        // matrix pipe while the two waves meet.  After the barrier: K_{u+1} and V_u are visible, and everyone has
        // fetched its fragments of K_u and V_{u-1}, whose places this iteration's requests overwrite.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
      }
      if (sl < 8) {
        const int c2 = sl >> 2, dt = sl & 3;
        oacc[dt][1] = E::mfma32(vf_prev[c2][dt], __builtin_bit_cast(i16x8_t, pbw[1][c2]), oacc[dt][1]);
      } else {
        const int c = (sl - 8) >> 1, qt = (sl - 8) & 1;
        if (c == 0) mfma_scores_first<Tag>(s_nxt[qt], kf[c], qf[qt][c], negm[qt]);
        else mfma_scores<Tag>(s_nxt[qt], kf[c], qf[qt][c]);
      }
      // exponentials: query tile 0 in slots 0..15, query tile 1 (first half) in slots 16..23
      if (sl < 16) {
        if ((sl & 1) == 0) pair_exp(s_cur[0], sl >> 1);
        else pair_pack(0, sl >> 1, ps0);
      } else {
        if ((sl & 1) == 0) pair_exp(s_cur[1], (sl - 16) >> 1);
        else pair_pack(1, (sl - 16) >> 1, ps1);
      }
      // memory -> LDS: K_{u+2} (generation of u: K_u was used up an iteration ago) and V_{u+1} (the other generation:
      // V_{u-1} was used up in the last iteration); 4 + 4 requests, 4 + 4 more on own steps
      if (sl >= 4 && sl < 8) {
        if (gen == 0) SLA_PAIR_FETCH(kh, koff[sl - 4], k_rb, nxt.dst, 0 * SLOT + (sl - 4) * 1024);
        else SLA_PAIR_FETCH(kh, koff[sl - 4], k_rb, nxt.dst, 2 * SLOT + (sl - 4) * 1024);
      } else if (sl >= 8 && sl < 12) {
        if (gen == 0) SLA_PAIR_FETCH(vh, voff[sl - 8], v_rb, vs.dst, 6 * SLOT + (sl - 8) * 1024);
        else SLA_PAIR_FETCH(vh, voff[sl - 8], v_rb, vs.dst, 4 * SLOT + (sl - 8) * 1024);
      }
      if (sl == 12 && nxt.own) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (gen == 0) SLA_PAIR_FETCH(kh, koff[j], k_rb + quarter_bytes, nxt.dst, 0 * SLOT + 4096 + j * 1024);
          else SLA_PAIR_FETCH(kh, koff[j], k_rb + quarter_bytes, nxt.dst, 2 * SLOT + 4096 + j * 1024);
        }
      }
      if (sl == 14 && vs.own) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (gen == 0) SLA_PAIR_FETCH(vh, voff[j], v_rb + quarter_bytes, vs.dst, 6 * SLOT + 4096 + j * 1024);
          else SLA_PAIR_FETCH(vh, voff[j], v_rb + quarter_bytes, vs.dst, 4 * SLOT + 4096 + j * 1024);
        }
      }
      // LDS reads: K_{u+1} fragments in slots 4..7 (used from slot 8 on), V_u fragments in slots 8..15
      if (sl >= 4 && sl < 8) {
        kf[2 * (sl - 4)] = *reinterpret_cast<const i16x8_t*>(smem + (gen ^ 1) * 2 * SLOT + kfo[2 * (sl - 4)]);
        kf[2 * (sl - 4) + 1] = *reinterpret_cast<const i16x8_t*>(smem + (gen ^ 1) * 2 * SLOT + kfo[2 * (sl - 4) + 1]);
      } else if (sl >= 8 && sl < 16) {
        const int gi = (sl - 8) >> 2, dt = (sl - 8) & 3;
        const uint8_t* p0 = smem + gen * 2 * SLOT + 16 * gi * ROWB + vfo[dt];
        vf_cur[gi][dt] = concat4(lds_read_tr16(reinterpret_cast<const uint16_t*>(p0)),
                                 lds_read_tr16(reinterpret_cast<const uint16_t*>(p0 + 8 * ROWB)));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // rare path (one branch): the probabilities came out too large (or this is the first unit, whose reference is a
    // placeholder): move the reference to this sub-tile's maximum and form them again
    const bool first = HALF == 0 && step_index == 0;       // (looked at on the rare path only)
    if (__builtin_expect(__any(!(ps0 <= PLIM)), 0)) {
      raise_reference(s_cur[0], s_nxt[0], 0, first);
      ps0 = softmax_again(s_cur[0], 0);
    }
    l_run[0] += ps0;
    __builtin_amdgcn_sched_barrier(0);
    // ---- block B: slots 24..31 ----
#pragma unroll
    for (int sl = 0; sl < 8; ++sl) {
      const int c2 = sl >> 2, dt = sl & 3;
      oacc[dt][0] = E::mfma32(vf_cur[c2][dt], __builtin_bit_cast(i16x8_t, pbw[0][c2]), oacc[dt][0]);
      if ((sl & 1) == 0) pair_exp(s_cur[1], 4 + (sl >> 1));
      else pair_pack(1, 4 + (sl >> 1), ps1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (__builtin_expect(__any(!(ps1 <= PLIM)), 0)) {
      raise_reference(s_cur[1], s_nxt[1], 1, first);
      ps1 = softmax_again(s_cur[1], 1);
    }
    l_run[1] += ps1;
    if (HALF == 0) ps_seed = 0.f;
    if (HALF) {
      cur = nxt;
      nxt = step_of(__builtin_amdgcn_readfirstlane(tile2_lane));
    }
  };

  for (; step_index < topk; ++step_index) {
    iteration(0, s_a, s_b, vf_b, vf_a);
    iteration(1, s_b, s_a, vf_a, vf_b);
  }
  // the last unit's products for query tile 1 (nunits is even: its fragments are in vf_b)
  if (nunits > 0) {
#pragma unroll
    for (int sl = 0; sl < 8; ++sl) {
      const int c2 = sl >> 2, dt = sl & 3;
      oacc[dt][1] = E::mfma32(vf_b[c2][dt], __builtin_bit_cast(i16x8_t, pbw[1][c2]), oacc[dt][1]);
    }
  }

  // ---- epilogue ----
  // every wave is done with the rings and no request is in flight: the staging tiles are free
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const size_t out_off = lout.head(bh) + (size_t)qrow0 * (size_t)lout.sl;
  // Fused linear branch: the per-head state KVW^T (D x D, 16 bit) goes into the V ring the way K half-tiles do (four
  // slots of 32 rows, swizzled pieces, each wave requests half); the q rows are the resident B operands of the score
  // products.  z and the bias come up front as well: at one wave per SIMD nothing hides a load issued where it is used.
  i16x8_t zreg[DC];
  f32x4_t breg[DT][4];
  if (FUSED) {
    const __amdgpu_buffer_rsrc_t sth = make_rsrc(kvwt + (size_t)bh * D * D, D * D * 2);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      // instruction i of this wave: rows 64w + 4i .. +3 of the state -> slot 4 + 2w + i / 8, rows 4 (i % 8) ..
      const int j = i & 3;
      const uint32_t soff = (uint32_t)(4 * j + lrow) * ROWB + ((lslot ^ ((4 * j + lrow) & 15)) * 16);
      SLA_PAIR_FETCH(sth, soff, (uint32_t)((64 * w + 4 * (i - j)) * ROWB), smem_addr, (4 + 2 * w + (i >> 3)) * SLOT + (i & 7) * 1024);
    }
    const uint16_t* z_h = zst + (size_t)bh * D;
#pragma unroll
    for (int c = 0; c < DC; ++c) zreg[c] = *reinterpret_cast<const i16x8_t*>(z_h + 16 * c + 8 * g);
#pragma unroll
    for (int et = 0; et < DT; ++et)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const f32x4_t b4 = *reinterpret_cast<const f32x4_t*>(bias + 32 * et + 8 * i4 + 4 * g);
        float b0, b1, b2, b3;
        round16_pair<Tag>(b4[0], b4[1], b0, b1);
        round16_pair<Tag>(b4[2], b4[3], b2, b3);
        breg[et][i4] = f32x4_t{b0, b1, b2, b3};
      }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    uint16_t* const stage_q = stage;
    const int rows_valid = writes ? min(32, L - qrow0 - 32 * qt) : 0;
    const float l_tot = l_run[qt] + __shfl_xor(l_run[qt], 32);
    const float inv = 1.0f / l_tot;
    const int qrow = qrow0 + 32 * qt + r;
    if (qrow < L && g == 0 && writes) lse[(size_t)bh * L + qrow] = m_used[qt] * scale_log2e + fast_log2(l_tot);
    auto park_attention = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          i32x2_t wv;
          wv[0] = (int)E::pack2(oacc[dt][qt][4 * i4 + 0] * inv, oacc[dt][qt][4 * i4 + 1] * inv);
          wv[1] = (int)E::pack2(oacc[dt][qt][4 * i4 + 2] * inv, oacc[dt][qt][4 * i4 + 3] * inv);
          *reinterpret_cast<i32x2_t*>(&stage_q[r * SSTR + 32 * dt + 8 * i4 + 4 * g]) = wv;
        }
      wave_lds_fence();
    };
    auto flush_rows = [&](uint16_t* dst_tile, size_t dst_pitch) __attribute__((always_inline)) {
      TileRows<D> t;
      t.unpark(stage_q, lane);
      t.store_streaming(dst_tile, rows_valid, lane, dst_pitch);
      wave_lds_fence();
    };
    if (!FUSED) {
      park_attention();
      flush_rows(o + out_off + (size_t)(32 * qt) * (size_t)lout.sl, (size_t)lout.sl);
    } else {
      // ---- linear branch of the same rows (see sparse_fwd_kernel) ----
      // (the resident B operands of the score products are the rows of q as they came from memory)
      // Values that the reference rounds to 16 bit are rounded two at a time (one conversion instruction packs two) and
      // taken apart again where the arithmetic goes on in fp32; a packed pair of phi(q) is a register of the B operand.
      float den = 0.f;
      i16x8_t fq[DC];
      auto pair_done = [&](int c, int j2, float v0, float v1, i32x4_t& pw) __attribute__((always_inline)) {
        float g0, g1, p0, p1;
        pw[j2] = (int)round16_pair<Tag>(v0, v1, g0, g1);
        const uint32_t zz = (uint32_t)__builtin_bit_cast(i32x4_t, zreg[c])[j2];
        round16_pair<Tag>(g0 * E::to_float((uint16_t)(zz & 0xffffu)), g1 * E::to_float((uint16_t)(zz >> 16)), p0, p1);
        den += p0;
        den += p1;
      };
      if (fmap == SLA_FMAP_SOFTMAX) {
        float f[DC][8];
#pragma unroll
        for (int c = 0; c < DC; ++c)
#pragma unroll
          for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)qf[qt][c][j]);
        float row_mx, row_inv;
        phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          i32x4_t pw;
#pragma unroll
          for (int j2 = 0; j2 < 4; ++j2) pair_done(c, j2, f[c][2 * j2], f[c][2 * j2 + 1], pw);
          fq[c] = __builtin_bit_cast(i16x8_t, pw);
        }
      } else if (fmap == SLA_FMAP_RELU) {
        // (the choice of the map stays outside the loops over the elements)
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          i32x4_t pw;
#pragma unroll
          for (int j2 = 0; j2 < 4; ++j2) {
            const uint32_t xx = (uint32_t)__builtin_bit_cast(i32x4_t, qf[qt][c])[j2];
            pair_done(c, j2, fmaxf(E::to_float((uint16_t)(xx & 0xffffu)), 0.f), fmaxf(E::to_float((uint16_t)(xx >> 16)), 0.f), pw);
          }
          fq[c] = __builtin_bit_cast(i16x8_t, pw);
        }
      } else {
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          i32x4_t pw;
#pragma unroll
          for (int j2 = 0; j2 < 4; ++j2) {
            const uint32_t xx = (uint32_t)__builtin_bit_cast(i32x4_t, qf[qt][c])[j2];
            const float x0 = E::to_float((uint16_t)(xx & 0xffffu)), x1 = E::to_float((uint16_t)(xx >> 16));
            float e0, e1;                                    // elu, rounded; then + 1, rounded by pair_done
            round16_pair<Tag>(x0 > 0.f ? x0 : (__expf(x0) - 1.0f), x1 > 0.f ? x1 : (__expf(x1) - 1.0f), e0, e1);
            pair_done(c, j2, e0 + 1.0f, e1 + 1.0f, pw);
          }
          fq[c] = __builtin_bit_cast(i16x8_t, pw);
        }
      }
      den += __shfl_xor(den, 32);
      den = round16<Tag>(1e-5f + round16<Tag>(den));
      const float inv_den = 1.0f / den;
#pragma unroll
      for (int et = 0; et < DT; ++et) {
        i16x8_t a[DC];
#pragma unroll
        for (int c = 0; c < DC; ++c)
          a[c] = *reinterpret_cast<const i16x8_t*>(smem + (4 + et) * SLOT + r * ROWB + (((2 * c + g) ^ (r & 15)) * 16));
        f32x16_t acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int c = 0; c < DC; ++c) acc = E::mfma32(a[c], fq[c], acc);
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          const int e0 = 32 * et + 8 * i4 + 4 * g;
          const f32x4_t b4 = breg[et][i4];
          i32x2_t ws, wo;
          ws[0] = (int)E::pack2(oacc[et][qt][4 * i4 + 0] * inv, oacc[et][qt][4 * i4 + 1] * inv);
          ws[1] = (int)E::pack2(oacc[et][qt][4 * i4 + 2] * inv, oacc[et][qt][4 * i4 + 3] * inv);
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const uint32_t x = (uint32_t)ws[h];
            float l0, l1;
            round16_pair<Tag>(pin_f32(__builtin_fmaf(acc[4 * i4 + 2 * h], inv_den, b4[2 * h])),
                              pin_f32(__builtin_fmaf(acc[4 * i4 + 2 * h + 1], inv_den, b4[2 * h + 1])), l0, l1);
            wo[h] = (int)E::pack2(E::to_float((uint16_t)(x & 0xffff)) + l0, E::to_float((uint16_t)(x >> 16)) + l1);
          }
          *reinterpret_cast<i32x2_t*>(&stage_q[r * SSTR + e0]) = wo;
        }
      }
      wave_lds_fence();
      flush_rows(o + out_off + (size_t)(32 * qt) * (size_t)lout.sl, (size_t)lout.sl);
      if (o_s) {
        park_attention();
        flush_rows(o_s + ((size_t)bh * L + qrow0 + 32 * qt) * D, D);
      }
    }
  }
}

#undef SLA_PAIR_FETCH

}  // namespace sla
