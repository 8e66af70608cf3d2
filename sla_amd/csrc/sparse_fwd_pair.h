// Block-sparse FlashAttention forward for 64-row query blocks at head dim 128: two adjacent query blocks per
// workgroup, two wavefronts per query block (32 query rows each), two workgroups per compute unit, so that every SIMD
// holds two waves of different workgroups.
//
// Stands in for _attn_fwd of the reference (sparse_linear_attention/kernel.py:21-82) like sparse_fwd_kernel,
// whose arithmetic it shares (S^T = K Q^T, thresholded reference maximum, P^T as B operand of O^T = V^T P^T).
// What the shape is chosen for:
//   * a lone wave on a SIMD issues in order, and on this machine an LDS read costs it about 13 cycles of issue, a
//     matrix product 12 and a vector-ALU instruction 4: the 24 fragment reads, 112 softmax instructions, requests and
//     bookkeeping of a 32-product unit add up to more than the 1024 cycles of its products, and every wait (barrier,
//     memory, the rare path of the softmax) stops the matrix pipe.  With two waves on a SIMD the LDS, memory and
//     scalar instructions of one wave issue beside the vector-ALU and matrix instructions of the other, and one wave's
//     waits are the other's issue slots;
//   * neighbouring query blocks select mostly the same key blocks.  The two look-up rows of a pair are split
//     into the key blocks both selected ("shared": one copy of the tile in LDS for all four waves) and the rest
//     ("own": as many on either side, each block's two waves walk their own, two tiles in LDS), interleaved in the
//     order of the first row.  A pair that shares 19 of 25 key blocks moves 31 tiles instead of 50 from L2 into LDS.
// The unit of the loop is a half-tile of 32 keys.  K half-tiles live in a two-generation ring in LDS (u even /
// odd), V half-tiles likewise; each generation has two slots (slot 0: shared tile or the first block's own, slot 1:
// the second block's own).  Tiles go from global memory straight into LDS (buffer loads with the LDS bit: no staging
// registers, no LDS store instructions).  Rows are unpadded in LDS; the 16-byte slots of a row are XOR-swizzled with
// the row index (by choosing which global piece a lane fetches), so that both the 128-bit row reads of K and the
// transposing reads of V are free of bank conflicts.  One workgroup barrier per unit.
// The scores stay in the units of q . k; the exponent's argument is one fused multiply-add, s * (qk_scale * log2 e) -
// m * (qk_scale * log2 e), with the reference maximum's part in one register per lane.  (Scaling Q instead, once, and
// rounding it to 16 bit again would spare that instruction and shift the log-sum-exp by up to 0.02: too much for the
// backward pass, which forms its probabilities from it.)
#pragma once
#include "linear_state.h"

namespace sla {

constexpr int PAIR_MAX_T = 1024;      // look-up rows longer than this, or more than 4096 key blocks, take sparse_fwd_kernel

template <typename Tag, bool FUSED>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void sparse_fwd_pair_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, const void* __restrict__ lut,
    int lut64, uint16_t* __restrict__ o, float* __restrict__ lse, const RowLayout lin, const RowLayout lout, int L, int Mblk,
    int topk, float scale_log2e, int total, const uint16_t* __restrict__ kvwt, const uint16_t* __restrict__ zst,
    const float* __restrict__ bias, int fmap, uint16_t* __restrict__ o_s, int one_row) {
  using E = Elem<Tag>;
  constexpr int D = 128, DC = D / 16, DT = D / 32;
  constexpr int ROWB = D * 2;                         // bytes per row in LDS (unpadded)
  constexpr int SLOT = 32 * ROWB;                     // one half-tile: 8 KB
  constexpr int SSTR = TileRows<D>::SSTR;
  constexpr float PLIM = 1024.0f;   // a lane's 16 probabilities of a unit may sum to this before the reference moves

  // K ring: [generation][slot] at (2 gen + slot) * SLOT; V ring: the same, 4 * SLOT further on
  // (the epilogue's four staging tiles start where the V ring does and end 2 KB past it)
  __shared__ __attribute__((aligned(16))) uint8_t smem[8 * SLOT + 2048];
  __shared__ uint32_t bitmap[2][128];
  __shared__ uint16_t steps[2][PAIR_MAX_T];
  __shared__ uint16_t own_b[PAIR_MAX_T];        // the key blocks only the second row names
  __shared__ int repeated;
  static_assert(4 * 32 * SSTR * 2 <= 4 * SLOT + 2048, "the staging tiles of the epilogue exceed their place");

  const int logical = xcd_remap(blockIdx.x, gridDim.x, total);
  if (logical < 0) return;
  const int Mpair = (Mblk + 1) >> 1;
  const int bh = logical / Mpair;
  const int pj = logical - bh * Mpair;
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int blk = w >> 1, qt = w & 1;                  // query block of the pair, 32-row tile of the block
  const int g = lane >> 5, r = lane & 31;
  const bool pair_full = 2 * pj + 1 < Mblk;            // the last block of a head with an odd block count has no partner:
  const int mb = (blk == 1 && pair_full) ? 2 * pj + 1 : 2 * pj;   // the second block's waves then repeat the first and store nothing
  const bool writes = blk == 0 || pair_full;

  const size_t head_off = lin.head(bh);
  const uint32_t pitch = (uint32_t)lin.sl;
  const uint32_t head_bytes = lin.head_range_bytes(L, D);

  // ---- the two look-up rows -> per-block step lists
  // (one_row: the pair is one 128-row query block of the caller's, whose look-up table has one row per pair: both
  //  halves follow it, and every step is a shared one)
  const size_t rowA = one_row ? ((size_t)bh * Mpair + pj) * topk : ((size_t)bh * Mblk + 2 * pj) * topk;
  const size_t rowB = (pair_full && !one_row) ? rowA + topk : rowA;
  auto lut_at = [&](size_t i) __attribute__((always_inline)) -> int {       // (the low word of a 64-bit entry)
    return reinterpret_cast<const int*>(lut)[lut64 ? 2 * i : i];
  };
  // The first 64 entries of both rows are asked for before anything else: the schedule of the pair hangs on them, and
  // loads come back in the order they were issued.  (Lanes past the end of a row hold its last entry and are not
  // looked at.)
  int a_raw = 0, b_raw = 0;
  if (topk > 0) {                              // (an empty look-up table may be a null pointer)
    a_raw = lut_at(rowA + min(lane, topk - 1));
    b_raw = lut_at(rowB + min(lane, topk - 1));
  }
  // This wave's 32 query rows are requested next, straight in B-operand order (lane = row, 16 bytes per 16-wide
  // chunk of the head dim): they arrive while the look-up rows are merged.
  const int qrow0 = mb * 64 + 32 * qt;
  i16x8_t qf[DC];
  {
    const __amdgpu_buffer_rsrc_t qh = make_rsrc(q + head_off, head_bytes);
#pragma unroll
    for (int c = 0; c < DC; ++c) qf[c] = buf_load_b128(qh, ((uint32_t)(qrow0 + r) * pitch + 16 * c + 8 * g) * 2);   // rows past L: 0
  }
  // The V ring starts from zeros.  The first iteration's left-over products read fragments of a half-tile that does not
  // exist, against probabilities of exactly 0; and rows past L are never written into LDS, so what LDS holds there meets
  // a probability of exactly 0 as well: neither may be a NaN pattern left behind by an earlier kernel.
#pragma unroll
  for (int i = 0; i < 4 * SLOT / (256 * 16); ++i) reinterpret_cast<i32x4_t*>(smem + 4 * SLOT)[i * 256 + tid] = i32x4_t{0, 0, 0, 0};

  // ---- per-block step lists (built by the first wave of each block)
  // (The split assumes what the mask builder guarantees: no key block twice in a row, every index below 4096.  A row
  //  that names a block twice makes the pair walk both rows unshared, in the order given, each block as often as it
  //  is named; an index is only ever used modulo 4096 here, and as it is where the rows of K and V are addressed,
  //  where the buffer bounds apply.)
  if (tid < 128) {
    bitmap[0][tid] = 0;
    bitmap[1][tid] = 0;
  }
  if (tid == 0) repeated = 0;
  __syncthreads();
  if (qt == 0) {
    for (int c0 = 0; c0 < topk; c0 += 64) {
      const int i = c0 + lane;
      if (i < topk) {
        const int a = (c0 == 0 ? a_raw : lut_at(rowA + i)) & 4095, b = (c0 == 0 ? b_raw : lut_at(rowB + i)) & 4095;
        const int x = blk ? b : a;
        const uint32_t seen = atomicOr(&bitmap[blk][x >> 5], 1u << (x & 31));
        if ((seen >> (x & 31)) & 1u) repeated = 1;
      }
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
  // otherwise it is an own step, on which the first block takes that key block and the second block the next one (in
  // the order of its row) that only the second row names: both rows have as many of those.  Key blocks so come in the
  // order of the look-up rows, ascending as the mask builder writes them, and the pairs that are resident on an XCD
  // sweep K and V together.  Bit 15 of a step marks an own step, bit 14 the key block with missing rows, bit 13 a step
  // of the second block whose kind differs from that of the step before it (its waves then read their fragments from
  // another slot): the loop looks at bits 13 and 14 with one branch per unit.
  const int ragged_tile = (L & 63) ? (L >> 6) : -1;       // the only key block that can have missing rows
  if (qt == 0) {
    if (repeated) {
      const size_t rowW = blk ? rowB : rowA;
      for (int i = lane; i < topk; i += 64) {
        const int tile = lut_at(rowW + i) & 4095;
        steps[blk][i] = (uint16_t)(tile | 0x8000 | (tile == ragged_tile ? 0x4000 : 0));
      }
    } else {
      const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
      if (blk == 1) {                              // the second row's own blocks, in its order
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
      int last_own = 0;                            // kind of the last step of the chunk before (the first step has no
                                                   // predecessor: the prologue points the fragment reads at its kind)
      for (int c0 = 0; c0 < topk; c0 += 64) {
        const int i = c0 + lane;
        const int a = row_a(c0, i);
        const bool own = i < topk && !((bitmap[1][a >> 5] >> (a & 31)) & 1u);
        const unsigned long long bal = __ballot(own);
        if (i < topk) {
          int tile = a;
          if (own && blk == 1) tile = own_b[n + __popcll(bal & lt_mask)];
          const int before = lane == 0 ? (c0 == 0 ? (int)own : last_own) : (int)((bal >> (lane - 1)) & 1ull);
          const int changes = blk == 1 && before != (int)own;
          steps[blk][i] = (uint16_t)(tile | (own ? 0x8000 : 0) | (tile == ragged_tile ? 0x4000 : 0) | (changes ? 0x2000 : 0));
        }
        last_own = (int)((bal >> 63) & 1ull);
        n += __popcll(bal);
      }
    }
  }
  __syncthreads();                                 // the lists are read by both waves of a block

  f32x16_t oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;
  // Reference maximum of the online softmax in the units of q . k, and minus the reference in the exponent's units (the
  // addend of the exponent's multiply-add).  The prologue sets it to the maximum of the first unit.
  float m_used = 0.f, nmc = 0.f, l_run = 0.f;

  // ---- addressing ----
  // unit u = 2 * step + half.  Shared steps: one tile, slot 0, wave w fetches rows 8w..8w+7 of the half-tile
  // (2 instructions of 1 KB for K, 2 for V).  Own steps: slot blk, the block's wave qt fetches rows 8qt..8qt+7 and
  // 16+8qt..16+8qt+7 (4 + 4 instructions).  Either way the rows of instruction j are 8qt + 4j + lane / 16 (mod 16):
  // lane -> row 4j + lane / 16 of the wave's rows, 16-byte slot lane % 16, which receives piece (slot ^ swizzle(row)) of
  // that row.  K: swizzle = row % 16 (the 16 rows of a row-wise read hit 16 different slots); V: 4 (row % 4) + (row / 4) % 2
  // (so do the 4 rows x 4 pieces of a transposing read).
  // An LDS read costs the wave that issues it about 13 cycles, a request 16 and more, a scalar instruction 4, and a wave
  // issues in order: whatever a request needs beyond the load itself is kept out of the loop.  The two instructions of
  // a pair share one LDS base (M0): the second one's instruction offset of 1 KB moves its LDS destination and, by
  // as much, its memory address, and its lane part makes up the difference to four rows.  The row the wave's first
  // request starts at is part of the buffer descriptor, formed with scalar instructions (its range ends with the
  // head's last row, so rows past L still lie outside it), not of the vector offset.
  const int nunits = 2 * topk;
  const int lrow = lane >> 4, lslot = lane & 15;
  const uint32_t smem_addr = (uint32_t)(size_t)smem;      // LDS address of the rings
  const uint32_t row_bytes = pitch * 2;                   // bytes between rows in memory (at least 256)
  uint32_t koff[2], voff[2];          // lane part of the byte offset of instruction j
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    koff[j] = (uint32_t)(4 * j + lrow) * row_bytes + ((lslot ^ ((8 * qt + 4 * j + lrow) & 15)) * 16) - 1024u * j;
    voff[j] = (uint32_t)(4 * j + lrow) * row_bytes + ((lslot ^ ((lrow << 2) | j)) * 16) - 1024u * j;
  }
  // What the requests of a step need, by kind of step: the byte offset of the first row this wave fetches and the LDS
  // address (inside a generation's slot pair) of its first instruction.
  struct Step {
    int tile;          // key block
    int own;           // 0: shared step, 1: own step
    int care;          // bit 1: the key block with missing rows; bit 0: fragment reads of this step move to another slot
    uint32_t rb;       // byte offset in the head of the first row this wave fetches of half 0
    uint32_t dst;      // LDS byte address, relative to a generation's slot pair, of this wave's first instruction
  };
  auto step_of = [&](int entry) __attribute__((always_inline)) -> Step {
    const int own = entry >> 15, tile = entry & 4095;
    return Step{tile, own, (entry >> 13) & 3, (uint32_t)(tile * 64 + (own ? 8 * qt : 8 * w)) * row_bytes,
                smem_addr + (uint32_t)(own ? blk * SLOT + 8 * qt * ROWB : 8 * w * ROWB)};
  };
  auto step_lookup = [&](int s_raw) __attribute__((always_inline)) -> int {       // (per lane; made scalar where it is used)
    return (int)steps[blk][min(s_raw, topk - 1)];       // past the end: the last step again (fetched, never used)
  };
  const uint32_t half_bytes = 32 * row_bytes, sixteen_rows = 16 * row_bytes;
  const uint8_t* const k_head = reinterpret_cast<const uint8_t*>(k + head_off);
  const uint8_t* const v_head = reinterpret_cast<const uint8_t*>(v + head_off);
  // buffer descriptor of the head's rows from byte `off` on, assembled in scalar registers (raw buffer, no stride, 32-bit
  // data format: the constants of make_rsrc; device addresses have 48 bits, so the upper word needs no masking)
  auto rows_from = [&](const uint8_t* head, uint32_t off) __attribute__((always_inline)) -> u32x4_t {
    const uint64_t a = (uint64_t)(uintptr_t)head + off;
    return u32x4_t{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
                   (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32)),
                   (uint32_t)max((int)head_bytes - (int)off, 0), 0x00020000u};      // (a head spans less than 2 GiB here)
  };
  // one pair of requests: 8 rows, global -> LDS.  `ring` = byte offset of the slot pair (generation, K or V) plus that of the
  // rows inside the wave's part (written as instructions: the compiler would make every later LDS read wait for a load
  //  it knows to target LDS; the wait for these loads is the one before the barrier of the next iteration.  Rows past
  //  L lie outside the buffer range: nothing is written for them and LDS keeps what it held, which is either the zeros
  //  it was filled with at the start or rows of an earlier tile: finite values, whose scores are masked and whose
  //  probabilities are 0.  The s_nop is the wait state the hardware wants between a scalar write of M0 and a memory ->
  //  LDS load that reads it.)
#define SLA_PAIR_FETCH2(RSRC, LANEOFF, DST, RING)                                                                      \
  asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %3, 0 offen lds\n\t"                                  \
               "buffer_load_dwordx4 %2, %3, 0 offen offset:1024 lds" ::"s"(DST), "v"((LANEOFF)[0]), "v"((LANEOFF)[1]),   \
               "s"(RSRC), "n"(RING)                                                                                    \
               : "memory", "scc")
  // all requests of this wave for one half-tile (HALFOFF: byte offset of the half inside the tile)
#define SLA_PAIR_FETCH_HALF(HEAD, LANEOFF, STEP, HALFOFF, RING)                                                        \
  do {                                                                                                                 \
    const u32x4_t rs_ = rows_from(HEAD, (STEP).rb + (HALFOFF));                                         \
    SLA_PAIR_FETCH2(rs_, LANEOFF, (STEP).dst, RING);                                                                   \
    if ((STEP).own) {                                                                                                  \
      const u32x4_t rs2_ = rows_from(HEAD, (STEP).rb + (HALFOFF) + sixteen_rows);                       \
      SLA_PAIR_FETCH2(rs2_, LANEOFF, (STEP).dst, (RING) + 4096);                                                       \
    }                                                                                                                  \
  } while (0)
  // fragment addressing (bytes from the start of the rings; the slot of the current kind of step is added when the
  // kind changes)
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
  // The fragment offsets point at the shared slot or at this block's own slot; they move whenever the kind of the step
  // they read from changes (k_own / v_own: where they point now).
  int k_own = 0, v_own = 0;
  auto point_k = [&](int need) __attribute__((always_inline)) {
    if (__builtin_expect(need != k_own, 0)) {
      const int d = need ? blk * SLOT : -blk * SLOT;
#pragma unroll
      for (int c = 0; c < DC; ++c) kfo[c] += d;
      k_own = need;
    }
  };
  auto point_v = [&](int need) __attribute__((always_inline)) {
    if (__builtin_expect(need != v_own, 0)) {
      const int d = need ? blk * SLOT : -blk * SLOT;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) vfo[dt] += d;
      v_own = need;
    }
  };

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
  // Moves the reference up to the maximum of unit sv (raw scores) and rescales what has been accumulated.
  auto raise_reference = [&](const f32x16_t& sv) __attribute__((always_inline)) {
    float mx = row_max(sv);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(mx, m_used);
    const float f = fast_exp2((m_used - m_new) * scale_log2e);
    m_used = m_new;
    nmc = -m_new * scale_log2e;
    l_run *= f;
    // The output accumulators live in the accumulation registers and, on the common path, are only ever touched by
    // MFMAs.  They are scaled in place through one temporary, so that the register allocator has no reason to
    // move the whole accumulator through the vector registers around the loop.
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");     // (the last products into these registers have landed)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float x = oacc[dt][i], t;
        asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1"
                     : "+a"(x), "=&v"(t)
                     : "v"(f));
        oacc[dt][i] = x;
      }
  };
  auto read_k = [&](int gen, i16x8_t (&kf)[DC]) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < DC; ++c) kf[c] = *reinterpret_cast<const i16x8_t*>(smem + gen * 2 * SLOT + kfo[c]);
  };

  // ---- prologue: K_0, K_1 into LDS; S_0; fragments of K_1; K_2 requested ----
  f32x16_t s_a, s_b;              // scores of the current and of the next unit, swapping roles every iteration
  i16x8_t kf[DC];                 // fragments of the K half-tile whose scores the next iteration forms
  i16x8_t vf[2][DT];              // V^T fragments of the previous unit: [16-key group][32 output channels]
  i32x4_t pb_a[2], pb_b[2];       // packed probabilities of the current and of the previous unit: [16-key group]
#pragma unroll
  for (int c2 = 0; c2 < 2; ++c2) pb_b[c2] = i32x4_t{0, 0, 0, 0};      // the first iteration's products add nothing
  Step cur{0, 0, 0, 0, 0}, nxt{0, 0, 0, 0, 0}, nn{0, 0, 0, 0, 0};
  // Q is only ever an MFMA operand and is parked in the accumulation registers: the vector registers are left for the
  // score tiles, the fragments and the softmax arithmetic
#pragma unroll
  for (int c = 0; c < DC; ++c) asm volatile("" : "+a"(qf[c]));
  if (nunits > 0) {
    cur = step_of(__builtin_amdgcn_readfirstlane(step_lookup(0)));
    nxt = step_of(__builtin_amdgcn_readfirstlane(step_lookup(1)));
    nn = step_of(__builtin_amdgcn_readfirstlane(step_lookup(2)));
    SLA_PAIR_FETCH_HALF(k_head, koff, cur, 0u, 0 * SLOT);           // K_0 -> K generation 0
    SLA_PAIR_FETCH_HALF(k_head, koff, cur, half_bytes, 2 * SLOT);   // K_1 -> K generation 1
    point_k(cur.own);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    read_k(0, kf);
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      if (c == 0) mfma_scores_first<Tag>(s_a, kf[c], qf[c]);
      else mfma_scores<Tag>(s_a, kf[c], qf[c]);
    }
    read_k(1, kf);
    point_v(cur.own);
    // (the score products are written as instructions: the compiler inserts no wait states between them and the vector
    //  ALU's first look at their result, which inside the loop is eight products away and here is not)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    __syncthreads();                                         // everyone has its fragments of K_0: its place is free
    SLA_PAIR_FETCH_HALF(k_head, koff, nxt, 0u, 0 * SLOT);           // K_2 -> K generation 0
    // the reference starts at the first unit's maximum (a first key block always has rows in its first half)
    if (cur.care & 2) mask_tail(s_a, L - cur.tile * 64);
    float mx = row_max(s_a);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    m_used = mx;
    nmc = -mx * scale_log2e;
  }

  // One iteration = unit u, 16 MFMAs of this wave, every one of them followed by its share of the other work (the order
  // is pinned slot by slot):
  //   slots 0.. 7  S_{u+1} = K_{u+1} Q^T (one chain; fragments read in the previous iteration)
  //   slots 8..15  O^T += V_{u-1}^T P_{u-1}^T   (left over from the previous unit)
  //   beside them, one per slot: the 16 exponentials of unit u; every second slot packs a pair.
  //   After slot 0: wait for the requests of the previous iteration, one barrier.  Then V_u and K_{u+3} are requested
  //   (memory -> LDS), the fragments of V_{u-1} are fetched from LDS in slots 1..8 and those of K_{u+2} in slots 8..15.
  // After the barrier LDS holds V_{u-1} (generation (u-1)&1) and K_{u+2} (generation u&1); on entry s_cur = scores of u.
  // Unit u is half HALF of step `cur`; u+1 belongs to `cur` (HALF 0) or `nxt` (HALF 1), u+2 to `nxt`, u+3 to `nxt`
  // (HALF 0) or `nn` (HALF 1); u-1 to the step before `cur` (HALF 0) or to `cur` (HALF 1).
  // (A score product's result is first looked at by the vector ALU eight products after the end of its chain.)
  int step_index = 0;
  auto softmax_unit = [&](const f32x16_t& sv, i32x4_t (&pb)[2]) __attribute__((always_inline)) -> float {     // (rare path) all eight pairs of a unit
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float e0 = fast_exp2(__builtin_fmaf(sv[2 * j], scale_log2e, nmc));
      const float e1 = fast_exp2(__builtin_fmaf(sv[2 * j + 1], scale_log2e, nmc));
      pb[j >> 2][j & 3] = (int)E::pack2(e0, e1);
      psum += e0 + e1;
    }
    return psum;
  };
  auto read_vf = [&](int gen, int f) __attribute__((always_inline)) {         // fragment f = 4 * group + dt of the V half-tile in `gen`
    const int gi = f >> 2, dt = f & 3;
    const uint8_t* p0 = smem + gen * 2 * SLOT + 16 * gi * ROWB + vfo[dt];
    vf[gi][dt] = concat4(lds_read_tr16(reinterpret_cast<const uint16_t*>(p0)),
                         lds_read_tr16(reinterpret_cast<const uint16_t*>(p0 + 8 * ROWB)));
  };
  auto iteration = [&](int HALF, f32x16_t& s_cur, f32x16_t& s_nxt, i32x4_t (&pb_cur)[2], i32x4_t (&pb_prev)[2])
                       __attribute__((always_inline)) {
    const int gen = HALF;
    // requests: V_u is half HALF of cur, into V generation u&1; K_{u+3} is half 1 of nxt (HALF 0) or half 0 of nn (HALF 1),
    // into the other K generation
    const Step& ks = HALF == 0 ? nxt : nn;
    // One branch for what few units need: the key block with missing rows, and the fragment reads moving to another
    // slot.  V_{u-1} and V_{u-2} lie in different steps when HALF is 1 (V_{u-1} is of cur), K_{u+2} and K_{u+1} when HALF
    // is 0 (K_{u+2} is of nxt).
    if (__builtin_expect(HALF == 0 ? ((cur.care & 2) | (nxt.care & 1)) : cur.care, 0)) {
      if (cur.care & 2) mask_tail(s_cur, L - (cur.tile * 64 + 32 * HALF));
      if (HALF == 0) point_k(nxt.own);
      else point_v(cur.own);
    }
    // the step after the next two is looked up now and used at the end of the odd iteration
    int entry3_lane = 0;
    if (HALF) entry3_lane = step_lookup(step_index + 3);
    float ps = 0.f;
    float e_prev = 0.f;
    float t_arg = __builtin_fmaf(s_cur[0], scale_log2e, nmc);      // the exponent's argument is formed a slot ahead of its
    __builtin_amdgcn_sched_barrier(0);                             // exponential, the sum a slot behind it
#pragma unroll
    for (int sl = 0; sl < 16; ++sl) {
      if (sl < 8) {
        if (sl == 0) mfma_scores_first<Tag>(s_nxt, kf[sl], qf[sl]);
        else mfma_scores<Tag>(s_nxt, kf[sl], qf[sl]);
      } else {
        const int c2 = (sl - 8) >> 2, dt = (sl - 8) & 3;
        oacc[dt] = E::mfma32(vf[c2][dt], __builtin_bit_cast(i16x8_t, pb_prev[c2]), oacc[dt]);
      }
      {                                    // one score of unit u: exponential, sum; every second slot packs a pair
        float e = fast_exp2(t_arg);
        asm volatile("" : "+v"(e));        // (stays in its slot: nothing moves this work towards its first use)
        if (sl < 15) t_arg = __builtin_fmaf(s_cur[sl + 1], scale_log2e, nmc);
        if (sl > 0) ps += e_prev;
        if (sl & 1) {
          uint32_t pw = E::pack2(e_prev, e);
          asm volatile("" : "+v"(pw), "+v"(ps));
          pb_cur[sl >> 3][(sl >> 1) & 3] = (int)pw;
        }
        if (sl == 15) ps += e;
        e_prev = e;
      }
      if (sl == 0) {
        // The requests of the previous iteration have had fourteen slots to land.  After the barrier: V_{u-1} and
        // K_{u+2} are visible, and everyone has fetched its fragments of V_{u-2} and K_{u+1}, whose places this
        // iteration's requests overwrite.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
      }
      // memory -> LDS: V_u in slot 1, K_{u+3} in slot 5, the further rows of own steps in slot 3 (one branch for both)
      if (sl == 1) {
        const u32x4_t rs = rows_from(v_head, cur.rb + (HALF ? half_bytes : 0u));
        if (gen) SLA_PAIR_FETCH2(rs, voff, cur.dst, 6 * SLOT);
        else SLA_PAIR_FETCH2(rs, voff, cur.dst, 4 * SLOT);
      } else if (sl == 5) {
        const u32x4_t rs = rows_from(k_head, ks.rb + (HALF ? 0u : half_bytes));
        if (gen) SLA_PAIR_FETCH2(rs, koff, ks.dst, 0 * SLOT);
        else SLA_PAIR_FETCH2(rs, koff, ks.dst, 2 * SLOT);
      } else if (sl == 3 && __builtin_expect(cur.own | ks.own, 0)) {
        if (cur.own) {
          const u32x4_t rs = rows_from(v_head, cur.rb + (HALF ? half_bytes : 0u) + sixteen_rows);
          if (gen) SLA_PAIR_FETCH2(rs, voff, cur.dst, 6 * SLOT + 4096);
          else SLA_PAIR_FETCH2(rs, voff, cur.dst, 4 * SLOT + 4096);
        }
        if (ks.own) {
          const u32x4_t rs = rows_from(k_head, ks.rb + (HALF ? 0u : half_bytes) + sixteen_rows);
          if (gen) SLA_PAIR_FETCH2(rs, koff, ks.dst, 0 * SLOT + 4096);
          else SLA_PAIR_FETCH2(rs, koff, ks.dst, 2 * SLOT + 4096);
        }
      }
      // LDS reads: V_{u-1} fragments in slots 1..8 (used from slot 8 on), K_{u+2} fragments in slots 8..15 (used from
      // slot 0 of the next iteration on)
      if (sl >= 1 && sl <= 8) read_vf(gen ^ 1, sl - 1);
      if (sl >= 8) kf[sl - 8] = *reinterpret_cast<const i16x8_t*>(smem + gen * 2 * SLOT + kfo[sl - 8]);
      __builtin_amdgcn_sched_barrier(0);
    }
    // rare path (one branch): the probabilities came out too large: move the reference to this unit's maximum and form
    // them again.  (The comparison is issued before the steps move on and looked at after: a branch on a fresh
    // vector comparison waits for it.)
    const unsigned long long too_large = __ballot(!(ps <= PLIM));
    if (HALF) {
      cur = nxt;
      nxt = nn;
      nn = step_of(__builtin_amdgcn_readfirstlane(entry3_lane));
    }
    if (__builtin_expect(too_large != 0ull, 0)) {
      raise_reference(s_cur);
      ps = softmax_unit(s_cur, pb_cur);
    }
    l_run += ps;
  };

  for (; step_index < topk; ++step_index) {
    iteration(0, s_a, s_b, pb_a, pb_b);
    iteration(1, s_b, s_a, pb_b, pb_a);
  }
  // the last unit's products (nunits is even: its probabilities are in pb_b, V_{nunits-1} is on its way into generation 1)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  // (what the rest needs of the lane's number is formed again here, from an opaque copy, so that none of it is kept in
  //  a register, or spilled, across the loop)
  int lane_e = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  asm volatile("" : "+v"(lane_e));
  const int g_e = lane_e >> 5, r_e = lane_e & 31, lrow_e = lane_e >> 4, lslot_e = lane_e & 15;
  if (FUSED) {
    // Fused linear branch: the per-head state KVW^T (D x D, 16 bit) goes into the K ring, which nobody reads any more,
    // the way K half-tiles do (rows of 256 bytes, swizzled pieces, each wave requests a quarter), while the last
    // products run.
    const uint8_t* st_b = reinterpret_cast<const uint8_t*>(kvwt + (size_t)bh * D * D);
    const uint64_t a = (uint64_t)(uintptr_t)st_b;
    const u32x4_t sth{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
                      (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32)), (uint32_t)(D * D * 2),
                      0x00020000u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = 32 * w + 4 * i + lrow_e;                 // (lane part: row 4 (i % 4) + lrow of sixteen, swizzled piece)
      const uint32_t soff = (uint32_t)(row * ROWB + ((lslot_e ^ ((4 * i + lrow_e) & 15)) * 16));
      const uint32_t ldst = smem_addr + (uint32_t)((32 * w + 4 * i) * ROWB);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(ldst), "v"(soff), "s"(sth) : "memory");
    }
  }
  if (nunits > 0) {
#pragma unroll
    for (int f = 0; f < 8; ++f) read_vf(1, f);
#pragma unroll
    for (int sl = 0; sl < 8; ++sl) {
      const int c2 = sl >> 2, dt = sl & 3;
      oacc[dt] = E::mfma32(vf[c2][dt], __builtin_bit_cast(i16x8_t, pb_b[c2]), oacc[dt]);
    }
  }

  // ---- epilogue ----
  // every wave is done with the V ring, and the state has landed: the staging tiles are free
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  uint16_t* const stage = reinterpret_cast<uint16_t*>(smem + 4 * SLOT) + w * 32 * SSTR;   // wave-private staging tile, 32 rows
  const size_t out_off = lout.head(bh) + (size_t)qrow0 * (size_t)lout.sl;
  const int rows_valid = writes ? min(32, L - qrow0) : 0;
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
  const int qrow = qrow0 + r_e;
  if (qrow < L && g_e == 0 && writes) lse[(size_t)bh * L + qrow] = m_used * scale_log2e + fast_log2(l_tot);
  auto park_attention = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        i32x2_t wv;
        wv[0] = (int)E::pack2(oacc[dt][4 * i4 + 0] * inv, oacc[dt][4 * i4 + 1] * inv);
        wv[1] = (int)E::pack2(oacc[dt][4 * i4 + 2] * inv, oacc[dt][4 * i4 + 3] * inv);
        *reinterpret_cast<i32x2_t*>(&stage[r_e * SSTR + 32 * dt + 8 * i4 + 4 * g_e]) = wv;
      }
    wave_lds_fence();
  };
  auto flush_rows = [&](uint16_t* dst_tile, size_t dst_pitch) __attribute__((always_inline)) {
    TileRows<D> t;
    t.unpark(stage, lane_e);
    t.store_streaming(dst_tile, rows_valid, lane_e, dst_pitch);
    wave_lds_fence();
  };
  if (!FUSED) {
    park_attention();
    flush_rows(o + out_off, (size_t)lout.sl);
  } else {
    // ---- linear branch of the same rows (see sparse_fwd_kernel) ----
    // The q rows are the resident B operands of the score products, as they came from memory.  (Taken over here from
    // the accumulation registers the loop read them from: left to itself the compiler keeps a second copy of them
    // across the loop for this use.)
#pragma unroll
    for (int c = 0; c < DC; ++c) asm volatile("" : "+a"(qf[c]));
    const uint16_t* z_h = zst + (size_t)bh * D;
    i16x8_t fq[DC], zreg[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) zreg[c] = *reinterpret_cast<const i16x8_t*>(z_h + 16 * c + 8 * g_e);
    float den = phi_pack_den<Tag, DC>(fmap, qf, fq, [&](int c, int j) __attribute__((always_inline)) {
      return E::to_float((uint16_t)zreg[c][j]);
    });
    den += __shfl_xor(den, 32);
    den = round16<Tag>(1e-5f + round16<Tag>(den));
    const float inv_den = 1.0f / den;
#pragma unroll
    for (int et = 0; et < DT; ++et) {
      i16x8_t a[DC];
#pragma unroll
      for (int c = 0; c < DC; ++c)
        a[c] = *reinterpret_cast<const i16x8_t*>(smem + (32 * et + r_e) * ROWB + (((2 * c + g_e) ^ (r_e & 15)) * 16));
      f32x16_t acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
      for (int c = 0; c < DC; ++c) acc = E::mfma32(a[c], fq[c], acc);
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int e0 = 32 * et + 8 * i4 + 4 * g_e;
        const f32x4_t b4 = *reinterpret_cast<const f32x4_t*>(bias + e0);
        float bb[4];
        round16_pair<Tag>(b4[0], b4[1], bb[0], bb[1]);
        round16_pair<Tag>(b4[2], b4[3], bb[2], bb[3]);
        i32x2_t ws, wo;
        ws[0] = (int)E::pack2(oacc[et][4 * i4 + 0] * inv, oacc[et][4 * i4 + 1] * inv);
        ws[1] = (int)E::pack2(oacc[et][4 * i4 + 2] * inv, oacc[et][4 * i4 + 3] * inv);
        // the sum as the reference's tensor addition forms it: both summands in 16 bit, one rounded add
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint32_t x = (uint32_t)ws[h];
          float l0, l1;
          round16_pair<Tag>(pin_f32(__builtin_fmaf(acc[4 * i4 + 2 * h], inv_den, bb[2 * h])),
                            pin_f32(__builtin_fmaf(acc[4 * i4 + 2 * h + 1], inv_den, bb[2 * h + 1])), l0, l1);
          wo[h] = (int)E::pack2(E::to_float((uint16_t)(x & 0xffff)) + l0, E::to_float((uint16_t)(x >> 16)) + l1);
        }
        *reinterpret_cast<i32x2_t*>(&stage[r_e * SSTR + e0]) = wo;
      }
    }
    wave_lds_fence();
    flush_rows(o + out_off, (size_t)lout.sl);
    if (o_s) {
      park_attention();
      flush_rows(o_s + ((size_t)bh * L + qrow0) * D, D);
    }
  }
}

#undef SLA_PAIR_FETCH2
#undef SLA_PAIR_FETCH_HALF

}  // namespace sla
