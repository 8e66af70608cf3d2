// Shared device/host helpers for the gfx950 SLA kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/sla_hip.h"

namespace sla {

// ---- error reporting -------------------------------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);

#define SLA_REQUIRE(cond, code, ...)      \
  do {                                    \
    if (!(cond)) {                        \
      ::sla::set_error(__VA_ARGS__);      \
      return (code);                      \
    }                                     \
  } while (0)

static inline int cdiv(int a, int b) { return (a + b - 1) / b; }
static inline int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }
static inline int elem_bytes(int dtype) { return dtype == SLA_F32 ? 4 : 2; }

// ---- vector types ------------------------------------------------------------
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short i16x4_t;
typedef __attribute__((__vector_size__(8 * sizeof(short)))) short i16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(2 * sizeof(int)))) int i32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4_t;
typedef __attribute__((__vector_size__(8 * sizeof(int)))) int i32x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(int)))) int i32x16_t;

struct bf16_tag {};
struct f16_tag {};

// 16-bit element traits: raw storage is uint16_t; conversions and MFMA by tag.
template <typename Tag>
struct Elem;

template <>
struct Elem<bf16_tag> {
  static __device__ __forceinline__ float to_float(uint16_t u) { return __uint_as_float(((uint32_t)u) << 16); }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    __bf16 b = (__bf16)f;  // round to nearest even
    return __builtin_bit_cast(uint16_t, b);
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    f32x2_t v = {a, b};
    bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
    return __builtin_bit_cast(uint32_t, r);
  }
  static __device__ __forceinline__ f32x16_t mfma32(i16x8_t a, i16x8_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
  }
  static __device__ __forceinline__ f32x4_t mfma16(i16x8_t a, i16x8_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
  }
};

template <>
struct Elem<f16_tag> {
  static __device__ __forceinline__ float to_float(uint16_t u) { return (float)__builtin_bit_cast(_Float16, u); }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    _Float16 h = (_Float16)f;
    return __builtin_bit_cast(uint16_t, h);
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    f32x2_t v = {a, b};
    f16x2_t r = __builtin_convertvector(v, f16x2_t);
    return __builtin_bit_cast(uint32_t, r);
  }
  static __device__ __forceinline__ f32x16_t mfma32(i16x8_t a, i16x8_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                  0, 0);
  }
  static __device__ __forceinline__ f32x4_t mfma16(i16x8_t a, i16x8_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                  0, 0);
  }
};

// LDS transposed read of four 16-bit elements.  Inside a 16-lane group, lane i
// passes the address of row (i/4), columns 4*(i%4)..+3 of a 4x16 tile and
// receives column i of that tile (rows 0..3).
typedef __attribute__((address_space(3))) i16x4_t lds_i16x4_t;
static __device__ __forceinline__ i16x4_t lds_read_tr16(const uint16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)p);
}

static __device__ __forceinline__ i16x8_t concat4(i16x4_t lo, i16x4_t hi) {
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Buffer-addressed loads: offsets past `bytes` return zero, so ragged tails need no branches.
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4_t;
static __device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
static __device__ __forceinline__ i16x8_t buf_load_b128(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
  return __builtin_bit_cast(i16x8_t, __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0));
}
// (The whole offset goes into the vector operand on purpose: the scalar offset operand of a buffer load takes no
//  part in the range check, and the kernels rely on out-of-range rows reading as zero.)

// Orders this wave's LDS writes before its later LDS reads when lanes exchange data through a
// wave-private region: the hardware keeps one wave's LDS operations in order, this keeps the compiler
// from moving them across the hand-over.  Emits no instruction.
static __device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---- row-contiguous output of a tile held in MFMA accumulator layout ---------------------------
// In the transposed formulations a lane owns one row (query / key) of a 32-row tile and, per 32-column
// tile dt and register group i4, the 4 adjacent columns 32dt + 8i4 + 4g.. of that row.  Storing those
// 8-byte pieces directly makes every lane of a wave touch a different 256-byte row.  Instead the wave
// parks the tile in a private LDS staging area and moves it with 16-byte accesses in which D/8 adjacent
// lanes cover one whole row; inputs take the same route in reverse.
// `stage` holds 32 rows of (D + 8) elements and is private to the calling wave (the LDS queue of a wave
// is in order, so no workgroup barrier is needed).
// Row-contiguous tile traffic: 32 rows of D 16-bit elements move as 16-byte pieces, D/8 adjacent lanes
// per row, D/16 pieces per lane.  Piece i of a lane is (row, col) = ((lane + 64 i) / (D/8), 8 ((lane + 64 i) % (D/8))).
template <int D>
struct TileRows {
  static constexpr int CPR = D / 8, N = 32 * CPR / 64, SSTR = D + 8;
  i16x8_t x[N];

  // global -> registers; rows at or past rows_valid read as zero; `pitch` = elements between rows in memory
  __device__ __forceinline__ void fetch(const uint16_t* gtile, int rows_valid, int lane, size_t pitch = D) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = lane + 64 * i, row = idx / CPR, col = (idx % CPR) * 8;
      x[i] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
      if (row < rows_valid) x[i] = *reinterpret_cast<const i16x8_t*>(gtile + (size_t)row * pitch + col);
    }
  }
  // registers -> the wave's staging tile
  __device__ __forceinline__ void park(uint16_t* stage, int lane) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = lane + 64 * i, row = idx / CPR, col = (idx % CPR) * 8;
      *reinterpret_cast<i16x8_t*>(&stage[row * SSTR + col]) = x[i];
    }
    wave_lds_fence();
  }
  // staging tile -> registers
  __device__ __forceinline__ void unpark(const uint16_t* stage, int lane) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = lane + 64 * i, row = idx / CPR, col = (idx % CPR) * 8;
      x[i] = *reinterpret_cast<const i16x8_t*>(&stage[row * SSTR + col]);
    }
  }
  // registers -> global
  __device__ __forceinline__ void store(uint16_t* gtile, int rows_valid, int lane, size_t pitch = D) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = lane + 64 * i, row = idx / CPR, col = (idx % CPR) * 8;
      if (row < rows_valid) *reinterpret_cast<i16x8_t*>(gtile + (size_t)row * pitch + col) = x[i];
    }
  }
  // registers -> global, as streaming stores: the rows are not read again by this kernel, and what does not stay behind as
  // modified lines in L2 does not have to be written back when the kernel ends, before the next one may start
  __device__ __forceinline__ void store_streaming(uint16_t* gtile, int rows_valid, int lane, size_t pitch = D) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = lane + 64 * i, row = idx / CPR, col = (idx % CPR) * 8;
      if (row < rows_valid) __builtin_nontemporal_store(x[i], reinterpret_cast<i16x8_t*>(gtile + (size_t)row * pitch + col));
    }
  }
  // this += other, element-wise in fp32 with one rounding
  template <typename E>
  __device__ __forceinline__ void add(const TileRows& o) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      i32x4_t w;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        w[j] = (int)E::pack2(E::to_float((uint16_t)x[i][2 * j]) + E::to_float((uint16_t)o.x[i][2 * j]),
                             E::to_float((uint16_t)x[i][2 * j + 1]) + E::to_float((uint16_t)o.x[i][2 * j + 1]));
      x[i] = __builtin_bit_cast(i16x8_t, w);
    }
  }
};

// Writes a tile held in accumulator register order (val[dt][16], lane = row) into the staging tile.
template <typename E, int D>
static __device__ __forceinline__ void park_acc_tile(uint16_t* stage, const float (&val)[D / 32][16], int lane) {
  constexpr int SSTR = D + 8;
  const int g = lane >> 5, r = lane & 31;
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      i32x2_t w;
      w[0] = (int)E::pack2(val[dt][4 * i4 + 0], val[dt][4 * i4 + 1]);
      w[1] = (int)E::pack2(val[dt][4 * i4 + 2], val[dt][4 * i4 + 3]);
      *reinterpret_cast<i32x2_t*>(&stage[r * SSTR + 32 * dt + 8 * i4 + 4 * g]) = w;
    }
  wave_lds_fence();
}

// Accumulator-order tile -> global rows.  An addend is added after the value has been rounded to
// 16 bit, as a separate 16-bit tensor addition would: `addend` is a tile fetched earlier; with
// ADD_DEST the addend is what the destination rows hold (read here, while the tile sits in LDS).
template <typename E, int D, bool ADD_DEST = false>
static __device__ __forceinline__ void store_acc_tile(uint16_t* stage, const float (&val)[D / 32][16], uint16_t* gtile,
                                                       const TileRows<D>* addend, int rows_valid, int lane,
                                                       size_t pitch = D) {
  TileRows<D> old;
  if (ADD_DEST) old.fetch(gtile, rows_valid, lane, pitch);
  park_acc_tile<E, D>(stage, val, lane);
  TileRows<D> t;
  t.unpark(stage, lane);
  if (ADD_DEST) t.template add<E>(old);
  else if (addend) t.template add<E>(*addend);
  t.store(gtile, rows_valid, lane, pitch);
  wave_lds_fence();   // the staging area may be rewritten right after
}

// Keeps an fp32 value as it is: stops the compiler from merging the operation that produced it with a
// following conversion to 16 bit (a mixed-precision fma rounds once, fp32-then-16-bit rounds twice), so
// that two kernels evaluating the same expression agree bit for bit.
static __device__ __forceinline__ float pin_f32(float x) {
  asm volatile("" : "+v"(x));
  return x;
}

// Matrix products with their result in vector registers (the vector ALU reads it next) and the resident B operand in
// accumulation registers.  Written as instructions because the compiler gives every MFMA of a function that uses
// accumulation registers an accumulation-register result and would copy the scores back one register at a time.
// INVARIANT the callers keep: the compiler sees no MFMA here, so its hazard recogniser inserts no wait states behind
// these instructions.  Between the last product of a chain and the first vector-ALU (or LDS / memory) instruction
// that reads or overwrites the chain's result registers there are either at least two further MFMAs (each holds
// the matrix pipe for 8 passes = 32 cycles, which covers the wait states an 8-pass product needs) or an explicit
// `s_nop 15; s_nop 15`.  The steady-state loops satisfy the first form by construction (the scores of a unit are
// consumed beside the next unit's products); prologues, ragged-tile masks and the rare re-basing of the reference
// maximum use the second.  Consecutive dependent products of one chain (result registers = C operand) need no
// software wait states.
template <typename Tag>
static __device__ __forceinline__ void mfma_scores_first(f32x16_t& d, const i16x8_t& a, const i16x8_t& b) {
  if constexpr (__is_same(Tag, bf16_tag))
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
  else
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
}
template <typename Tag>
static __device__ __forceinline__ void mfma_scores_first(f32x16_t& d, const i16x8_t& a, const i16x8_t& b, const f32x16_t& c) {
  if constexpr (__is_same(Tag, bf16_tag))
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "a"(b), "v"(c));
  else
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "a"(b), "v"(c));
}
template <typename Tag>
static __device__ __forceinline__ void mfma_scores(f32x16_t& d, const i16x8_t& a, const i16x8_t& b) {
  if constexpr (__is_same(Tag, bf16_tag))
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
  else
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
}

static __device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
static __device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Workgroup index remap: consecutive hardware workgroup ids go round-robin to
// the 8 XCDs; give every XCD one contiguous range of logical tiles so that
// neighbouring tiles (same head, adjacent query blocks) share that XCD's L2.
// The grid is rounded up to a multiple of 8; returns -1 for padding workgroups.
static __device__ __forceinline__ int xcd_remap(int wg, int grid, int total) {
  int per = grid >> 3;
  int logical = (wg & 7) * per + (wg >> 3);
  return logical < total ? logical : -1;
}

static inline int xcd_grid(int64_t total) { return (int)((total + 7) / 8 * 8); }

// Where the rows of a (B, H, L, D) tensor lie in memory: row l of head (b, h) starts `b*sb + h*sh + l*sl`
// elements after the base pointer, its D elements are adjacent.  The contiguous (B, H, L, D) tensor of the
// reference has (H*L*D, L*D, D); a (B, L, H, D) activation viewed as (B, H, L, D) has (L*H*D, D, H*D), and
// the q / k / v slices of a packed (B, L, 3, H, D) projection have (L*3*H*D, D, 3*H*D).
struct RowLayout {
  int64_t sb, sh, sl;
  int H;
  __host__ __device__ size_t head(int bh) const { return (size_t)(bh / H) * (size_t)sb + (size_t)(bh % H) * (size_t)sh; }
  // bytes from the first element of a head to the end of its last row (the range of a buffer descriptor:
  // rows past L then lie outside it and read as zero)
  __host__ __device__ uint32_t head_range_bytes(int L, int D) const { return (uint32_t)(((int64_t)(L - 1) * sl + D) * 2); }
};
static inline RowLayout contiguous_layout(int H, int L, int D) {
  return RowLayout{(int64_t)H * L * D, (int64_t)L * D, (int64_t)D, H};
}
// strides = {batch, head, row} in elements, or null for the contiguous (B, H, L, D) tensor.  Checks what the
// kernels rely on: rows do not overlap, every row starts 16-byte aligned, one head spans less than 4 GiB.
int make_layout(const int64_t* strides, int B, int H, int L, int D, int elem_bytes, RowLayout* out);

}  // namespace sla
