// phi(K)^T V and sum phi(K) state kernels of the linear branch (used by forward and backward).
#pragma once
#include "linear_common.h"

namespace sla {

// ---- kernel 1: partial states -----------------------------------------------------------
// grid (nsplit, BH), 256 threads.  Thread t moves 16-byte chunk (t%CPR) of rows t/CPR + i*RPP.
// OUT16: the D x D partial is written rounded to 16 bit (per-key-block states of the complement mode).
// ZW: zweight holds one fp32 per row of the head, (BH, L), and the z partial becomes sum_rows zweight * phi(k)
// instead of sum_rows phi(k) (used by the complement backward, where "k" is q and "v" a row gradient).
// VMAX: the largest |v| of every column over the slice goes to vmax_part[bh][split][D] (what the FP8 quantiser of v
// needs of v before it can start: v is streamed here anyway).
template <typename Tag, int D, bool OUT16 = false, bool ZW = false, bool VMAX = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void linear_state_partial_kernel(const uint16_t* __restrict__ k,
                                                                   const uint16_t* __restrict__ v, const RowLayout lay,
                                                                   void* __restrict__ kv_part_, float* __restrict__ z_part,
                                                                   int L, int rows_per_split, int fmap,
                                                                   const float* __restrict__ zweight = nullptr,
                                                                   float* __restrict__ vmax_part = nullptr) {
  using E = Elem<Tag>;
  constexpr int TR = 64;                 // rows per LDS tile
  constexpr int STR = D + 16;            // LDS row stride: transposed reads of 4 rows hit disjoint banks
  constexpr int CPR = D / 8;             // 16-byte chunks per row
  constexpr int RPP = 256 / CPR;         // rows covered by one pass of the 256 threads
  constexpr int NP = TR / RPP;           // passes per tile
  constexpr int DT = D / 32;             // 32-wide tiles along either state dimension
  constexpr int WPT = (DT * DT) / 4;     // output tiles per wave (4 waves)
  static_assert(DT * DT % 4 == 0, "state tiles must divide among 4 waves");

  __shared__ __attribute__((aligned(16))) uint16_t sK[TR * STR];
  __shared__ __attribute__((aligned(16))) uint16_t sV[TR * STR];
  __shared__ float sZ[RPP][D];

  const int split = blockIdx.x, bh = blockIdx.y, nsplit = gridDim.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5;
  const int row_begin = split * rows_per_split;
  const int row_end = min(L, row_begin + rows_per_split);
  const uint16_t* kh = k + lay.head(bh);
  const uint16_t* vh = v + lay.head(bh);
  const size_t pitch = (size_t)lay.sl;

  const int lrow = tid / CPR, lcol = (tid % CPR) * 8;

  // wave w owns output tiles w*WPT .. w*WPT+WPT-1; tile id = d1tile*DT + d2tile
  f32x16_t acc[WPT];
#pragma unroll
  for (int t = 0; t < WPT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
  float zacc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) zacc[e] = 0.f;
  // |v| of this thread's eight columns as 16-bit patterns without their sign bits: for bf16 and f16 alike the larger
  // magnitude has the larger pattern, so a packed unsigned maximum keeps two columns per register
  typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
  u16x2_t vmx[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) vmx[j] = u16x2_t{0, 0};

  const int tr_row = (lane & 15) >> 2;
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  // rows of the next tile are fetched into registers while the current tile is multiplied
  i16x8_t kreg[NP], vreg[NP];
  float wreg[NP];
  auto fetch = [&](int r0) {
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int grow = r0 + lrow + p * RPP;
      kreg[p] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
      vreg[p] = i16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
      wreg[p] = 1.0f;
      if (grow < row_end) {
        kreg[p] = *reinterpret_cast<const i16x8_t*>(kh + (size_t)grow * pitch + lcol);
        vreg[p] = *reinterpret_cast<const i16x8_t*>(vh + (size_t)grow * pitch + lcol);
        if (ZW) wreg[p] = zweight[(size_t)bh * L + grow];
      }
    }
  };
  if (row_begin < row_end) fetch(row_begin);
  for (int r0 = row_begin; r0 < row_end; r0 += TR) {
    __syncthreads();
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int row = lrow + p * RPP;
      const int grow = r0 + row;
      const i16x8_t kk = kreg[p], vv = vreg[p];
      const bool ok = grow < row_end;
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = E::to_float((uint16_t)kk[e]);
      if (fmap == SLA_FMAP_SOFTMAX) {
        // the CPR lanes that share this row are adjacent: reduce max and sum across them
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
      i16x8_t fk;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (!ok) f[e] = 0.f;              // rows past the end take no part (phi(0) is not 0 for elu/softmax)
        zacc[e] += ZW ? wreg[p] * f[e] : f[e];
        fk[e] = (short)E::from_float(f[e]);
      }
      *reinterpret_cast<i16x8_t*>(&sK[row * STR + lcol]) = fk;
      *reinterpret_cast<i16x8_t*>(&sV[row * STR + lcol]) = vv;
      if (VMAX) {                          // (rows past the end were fetched as zeros)
        const i32x4_t vw = __builtin_bit_cast(i32x4_t, vv);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          vmx[j] = __builtin_elementwise_max(vmx[j], __builtin_bit_cast(u16x2_t, vw[j] & 0x7fff7fff));
      }
    }
    __syncthreads();
    if (r0 + TR < row_end) fetch(r0 + TR);     // after the barrier: its fence would wait for these loads
#pragma unroll
    for (int c = 0; c < TR / 16; ++c) {
      const int l0 = 16 * c + 8 * g + tr_row;
#pragma unroll
      for (int t = 0; t < WPT; ++t) {
        const int tile = wave * WPT + t;
        const int d1t = tile / DT, d2t = tile % DT;
        const uint16_t* pa = &sK[l0 * STR + 32 * d1t + tr_col];
        const uint16_t* pb = &sV[l0 * STR + 32 * d2t + tr_col];
        const i16x8_t a = concat4(lds_read_tr16(pa), lds_read_tr16(pa + 4 * STR));
        const i16x8_t b = concat4(lds_read_tr16(pb), lds_read_tr16(pb + 4 * STR));
        acc[t] = E::mfma32(a, b, acc[t]);
      }
    }
  }

  // partial KV, stored transposed: kv_part[bh][split][d2][d1]
  const size_t part_off = ((size_t)bh * nsplit + split) * D * D;
#pragma unroll
  for (int t = 0; t < WPT; ++t) {
    const int tile = wave * WPT + t;
    const int d1t = tile / DT, d2t = tile % DT;
    const int d2 = 32 * d2t + (lane & 31);
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const size_t o = part_off + (size_t)d2 * D + 32 * d1t + 8 * i4 + 4 * g;
      if (OUT16) {
        i32x2_t w;
        w[0] = (int)E::pack2(acc[t][4 * i4], acc[t][4 * i4 + 1]);
        w[1] = (int)E::pack2(acc[t][4 * i4 + 2], acc[t][4 * i4 + 3]);
        *reinterpret_cast<i32x2_t*>(reinterpret_cast<uint16_t*>(kv_part_) + o) = w;
      } else {
        f32x4_t w = {acc[t][4 * i4], acc[t][4 * i4 + 1], acc[t][4 * i4 + 2], acc[t][4 * i4 + 3]};
        *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(kv_part_) + o) = w;
      }
    }
  }
  // partial z: reduce the RPP row groups through LDS
  __syncthreads();
#pragma unroll
  for (int e = 0; e < 8; ++e) sZ[lrow][lcol + e] = zacc[e];
  __syncthreads();
  if (tid < D) {
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < RPP; ++r) s += sZ[r][tid];
    z_part[((size_t)bh * nsplit + split) * D + tid] = s;
  }
  if (VMAX) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      sZ[lrow][lcol + 2 * j] = E::to_float(vmx[j][0]);
      sZ[lrow][lcol + 2 * j + 1] = E::to_float(vmx[j][1]);
    }
    __syncthreads();
    if (tid < D) {
      float a = 0.f;
#pragma unroll
      for (int r = 0; r < RPP; ++r) a = fmaxf(a, sZ[r][tid]);
      vmax_part[((size_t)bh * nsplit + split) * D + tid] = a;
    }
  }
}

// ---- kernel 2: reduce partials, round to 16 bit -------------------------------------------
// Position of column d2 inside a row whose columns are re-ordered to the accumulator slot order of the
// 32x32 MFMA: slot j of 16-column chunk c, lane group gg  <->  d2 = 16c + 8*(j/4) + 4gg + j%4.
static __device__ __host__ __forceinline__ int slot_order_pos(int d2) {
  const int c = d2 >> 4, w16 = d2 & 15;
  const int gg = (w16 >> 2) & 1, j = ((w16 >> 3) << 2) | (w16 & 3);
  return 16 * c + 8 * gg + j;
}

// kvt[bh][d2][d1] (transposed state) and kvp[bh][d1][slot order of d2] (for the backward's S dn^T product)
template <typename Tag>
__global__ void linear_state_reduce_kernel(const float* __restrict__ kv_part, const float* __restrict__ z_part,
                                           uint16_t* __restrict__ kvt, uint16_t* __restrict__ kvp, uint16_t* __restrict__ z,
                                           int nsplit, int DD, int D) {
  using E = Elem<Tag>;
  const int bh = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < DD) {
    const float* p = kv_part + (size_t)bh * nsplit * DD + i;
    float s = 0.f;
#pragma unroll 8
    for (int sp = 0; sp < nsplit; ++sp) s += p[(size_t)sp * DD];
    const uint16_t h = E::from_float(s);
    kvt[(size_t)bh * DD + i] = h;
    const int d2 = i / D, d1 = i % D;
    kvp[(size_t)bh * DD + d1 * D + slot_order_pos(d2)] = h;
  }
  if (i < D) {
    const float* p = z_part + (size_t)bh * nsplit * D + i;
    float s = 0.f;
#pragma unroll 8
    for (int sp = 0; sp < nsplit; ++sp) s += p[(size_t)sp * D];
    z[(size_t)bh * D + i] = E::from_float(s);
  }
}

// 16-bit transposed copy of the projection weight: wt[d][e] (A operand of dY^T = W^T G^T).
// One thread per element.
template <typename Tag>
__global__ void linear_prep_weight_kernel(const float* __restrict__ weight, uint16_t* __restrict__ wt, int D) {
  using E = Elem<Tag>;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= D * D) return;
  const int e = i / D, d = i % D;
  const uint16_t h = E::from_float(weight[i]);
  wt[d * D + e] = h;
}

// ---- kernel 3 (forward, and a backward that has to rebuild the states): fold the projection into the state -------------------------------------------------
// kvwt[bh][e][d1] = round16( sum_d2 round16(W[e][d2]) * KVT[d2][d1] ), fp32 accumulation in ascending d2.
// (phi(Q) KV / den) W^T = (phi(Q) (KV W^T)) / den, so the output kernel needs one product per query tile.
// grid (D / (1024 / D), BH), 256 threads: a workgroup forms 1024 / D rows e for all d1, thread = (row e, four adjacent d1).
// It sits between the state kernels and the attention kernel with nothing to overlap it, and its arithmetic is nothing:
// the head's state and the workgroup's rows of W come into LDS with every load in flight at once, the sums then run
// out of LDS.
// The workgroups of head 0 also leave the 16-bit transposed weight wt[d][e] that a backward reads (what
// linear_prep_weight_kernel writes), which saves the forward one launch in its chain of small kernels.
template <typename Tag>
__global__ __launch_bounds__(256) void linear_fold_kernel(const uint16_t* __restrict__ kvt, const float* __restrict__ weight,
                                                          uint16_t* __restrict__ kvwt, uint16_t* __restrict__ wt, int D) {
  using E = Elem<Tag>;
  __shared__ __attribute__((aligned(16))) uint16_t s_kv[128 * 128];      // [d2][d1]
  __shared__ float s_w[16 * 128];                                          // [row][d2], rounded to 16 bit
  const int bh = blockIdx.y, tid = threadIdx.x;
  const int groups = D >> 2;                       // threads per row e
  const int rows = 256 / groups;                   // rows e per workgroup (8 at D 128, 16 at D 64)
  const int e0 = blockIdx.x * rows;
  const uint16_t* src = kvt + (size_t)bh * D * D;
  for (int i = tid; i < D * D / 8; i += 256)
    reinterpret_cast<i16x8_t*>(s_kv)[i] = reinterpret_cast<const i16x8_t*>(src)[i];
  for (int i = tid; i < rows * D; i += 256) {
    const float wv = weight[(size_t)e0 * D + i];
    s_w[i] = round16<Tag>(wv);
    if (bh == 0) {
      const int e = e0 + i / D, d = i % D;
      wt[d * D + e] = E::from_float(wv);
    }
  }
  __syncthreads();
  const int el = tid / groups, d1 = (tid % groups) * 4;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const float* w = s_w + el * D;
#pragma unroll 8
  for (int d2 = 0; d2 < D; ++d2) {
    const i16x4_t kv4 = *reinterpret_cast<const i16x4_t*>(&s_kv[d2 * D + d1]);
    const float wv = w[d2];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] += wv * E::to_float((uint16_t)kv4[j]);
  }
  i32x2_t out;
  out[0] = (int)E::pack2(acc[0], acc[1]);
  out[1] = (int)E::pack2(acc[2], acc[3]);
  *reinterpret_cast<i32x2_t*>(kvwt + (size_t)bh * D * D + (size_t)(e0 + el) * D + d1) = out;
}

// ---- workspace layout of the state build -----------------------------------------------------
// The finished states (kvt .. wt) come first: `states_end` bytes that a caller may copy aside after the
// forward and put back at the start of the backward's workspace instead of having them rebuilt.
struct LinWs {
  int nsplit, rows_per_split;
  size_t kvt, kvp, kvwt, z, wt, states_end, kv_part, z_part, vmax_part, total;
};

static inline LinWs lin_ws(int BH, int L, int D) {
  LinWs w;
  // Two workgroups per compute unit: the state kernel shares the memory system with the mask builder's passes on the
  // other stream, and more, shorter slices (three per unit fit) only add partial states to write and to add up again
  // (module forward at B1 H12 L32760: 0.510 against 0.519 ms).
  const LinSplit sp = lin_split(BH, L, 512);
  w.nsplit = sp.nsplit;
  w.rows_per_split = sp.rows_per_split;
  size_t off = 0;
  w.kvt = off;     off += align_up((int64_t)BH * D * D * 2, 256);
  w.kvp = off;     off += align_up((int64_t)BH * D * D * 2, 256);
  w.kvwt = off;    off += align_up((int64_t)BH * D * D * 2, 256);
  w.z = off;       off += align_up((int64_t)BH * D * 2, 256);
  w.wt = off;      off += align_up((int64_t)D * D * 2, 256);
  w.states_end = off;
  w.kv_part = off; off += align_up((int64_t)BH * w.nsplit * D * D * 4, 256);
  w.z_part = off;  off += align_up((int64_t)BH * w.nsplit * D * 4, 256);
  w.vmax_part = off; off += align_up((int64_t)BH * w.nsplit * D * 4, 256);      // (filled on request: column maxima of |v| per slice)
  w.total = off;
  return w;
}


// Streams K and V once and leaves KVT, KVP, z (16 bit) and the 16-bit transposed weight in the workspace.
template <typename Tag, int D>
static inline void launch_state_build(const void* k, const void* v, const RowLayout& lay, const float* weight, int fmap,
                                      int BH, int L, char* ws, const LinWs& w, hipStream_t st, bool copy_weight = true) {
  float* kv_part = (float*)(ws + w.kv_part);
  float* z_part = (float*)(ws + w.z_part);
  uint16_t* kvt = (uint16_t*)(ws + w.kvt);
  uint16_t* z = (uint16_t*)(ws + w.z);
  hipLaunchKernelGGL((linear_state_partial_kernel<Tag, D>), dim3(w.nsplit, BH), dim3(256), 0, st, (const uint16_t*)k,
                     (const uint16_t*)v, lay, kv_part, z_part, L, w.rows_per_split, fmap);
  hipLaunchKernelGGL((linear_state_reduce_kernel<Tag>), dim3(cdiv(D * D, 256), BH), dim3(256), 0, st, kv_part, z_part, kvt,
                     (uint16_t*)(ws + w.kvp), z, w.nsplit, D * D, D);
  // (copy_weight = false: the caller's next kernel writes the 16-bit transposed weight on the side)
  if (copy_weight)
    hipLaunchKernelGGL((linear_prep_weight_kernel<Tag>), dim3(cdiv(D * D, 256)), dim3(256), 0, st, weight,
                       (uint16_t*)(ws + w.wt), D);
}

}  // namespace sla
