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

}  // namespace sla
