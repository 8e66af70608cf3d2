// Linear-attention branch, projection and final sum for gfx950.
//
// Stands in for sparse_linear_attention/core.py:90-100 of the reference:
//   fq = phi(q), fk = phi(k)                       (feature maps, 16-bit results)
//   kvsum = fk^T v (DxD), ksum = sum_L fk (1xD)      (16-bit results)
//   o_l = (fq kvsum) / (1e-5 + sum_d fq*ksum)        (16-bit results)
//   out = o_s + (o_l W^T + b)                        (W, b cast to 16 bit as autocast does)
//
// Kernels:
//   state_partial : streams K and V once; each workgroup owns a slice of L and forms its
//                   share of phi(K)^T V on the MFMA (both operands read transposed from LDS)
//                   and of sum phi(K) on the vector ALU; fp32 partials to the workspace.
//   state_reduce  : adds the partials in ascending slice order, rounds to 16 bit, stores the
//                   state TRANSPOSED (KVT[d2][d1]) so the next kernel reads MFMA rows directly.
//   fold          : KVW = KV W^T per head (16 bit), so numerator and projection are one product.
//   out           : one wavefront per 32 queries.  OUT^T = KVW^T phi(Q)^T is formed transposed so the
//                   per-query divisor is a per-lane scalar; the tile is scaled, biased, parked in LDS
//                   and written (plus the residual) with whole-row 16-byte accesses.
#include "linear_state.h"
#include "sage_steps.h"

namespace sla {

// ---- kernel 4: output --------------------------------------------------------------------
// grid (ceil(L / (128*TILES)), BH), 256 threads = 4 waves x 32 queries, TILES steps per workgroup.
// CONTIG: q and out are contiguous (B, H, L, D): the row pitch is the compile-time D.
template <typename Tag, int D, bool CONTIG>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void linear_out_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ kvwt,
                                                         const uint16_t* __restrict__ z, const float* __restrict__ bias,
                                                         const uint16_t* __restrict__ residual, uint16_t* __restrict__ out,
                                                         const RowLayout lq, const RowLayout lout, int L, int fmap,
                                                         int tiles_per_wg) {
  // (lq, lout: where the rows of q and of out lie; the residual is a contiguous (B, H, L, D) tensor)
  using E = Elem<Tag>;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int STR = D + 8;
  __shared__ __attribute__((aligned(16))) uint16_t sKVW[D * STR];       // [e][d1]
  __shared__ __attribute__((aligned(16))) uint16_t sStage[4][32 * STR];  // per-wave output staging
  __shared__ float sBias[D];
  __shared__ float sZ[D];

  const int bh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;

  // stage the folded state once per workgroup
  {
    const uint16_t* src = kvwt + (size_t)bh * D * D;
    for (int idx = tid; idx < D * D / 8; idx += 256) {
      const int row = idx / (D / 8), col = (idx % (D / 8)) * 8;
      *reinterpret_cast<i16x8_t*>(&sKVW[row * STR + col]) = *reinterpret_cast<const i16x8_t*>(src + (size_t)row * D + col);
    }
    if (tid < D) {
      sBias[tid] = round16<Tag>(bias[tid]);
      sZ[tid] = E::to_float(z[(size_t)bh * D + tid]);
    }
  }
  __syncthreads();

  const uint16_t* qh = q + (CONTIG ? (size_t)bh * L * D : lq.head(bh));
  uint16_t* const oh = out + (CONTIG ? (size_t)bh * L * D : lout.head(bh));
  const size_t pitch_q = CONTIG ? (size_t)D : (size_t)lq.sl, pitch_o = CONTIG ? (size_t)D : (size_t)lout.sl;
  uint16_t* stage = sStage[wave];
  const int first_row = blockIdx.x * tiles_per_wg * 128 + wave * 32;
  TileRows<D> qt;                      // q rows of the tile about to be processed, fetched one tile ahead
  if (first_row < L) qt.fetch(qh + (size_t)first_row * pitch_q, min(32, L - first_row), lane, pitch_q);
  for (int tt = 0; tt < tiles_per_wg; ++tt) {
    const int row0 = first_row + tt * 128;
    if (row0 >= L) break;
    const int rows_valid = min(32, L - row0);
    const size_t off = ((size_t)bh * L + row0) * D;

    // phi(q): this lane holds d = 16c + 8g + j of its row; lane^32 holds the other half
    qt.park(stage, lane);
    i16x8_t xq[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) xq[c] = *reinterpret_cast<const i16x8_t*>(&stage[r * STR + 16 * c + 8 * g]);
    wave_lds_fence();
    TileRows<D> res;
    if (residual) res.fetch(residual + off, rows_valid, lane);
    if (tt + 1 < tiles_per_wg && row0 + 128 < L)
      qt.fetch(qh + (size_t)(row0 + 128) * pitch_q, min(32, L - row0 - 128), lane, pitch_q);
    // divisor: 1e-5 + sum_d round16(fq*z), each step rounded to 16 bit as the reference's tensors are
    i16x8_t qf[DC];
    float den = phi_pack_den<Tag, DC>(fmap, xq, qf, [&](int c, int j) { return sZ[16 * c + 8 * g + j]; });
    den += __shfl_xor(den, 32);
    den = round16<Tag>(1e-5f + round16<Tag>(den));
    const float inv_den = 1.0f / den;

    // OUT^T = KVW^T-rows x phi(Q)^T : DT tiles of 32 output channels x 32 queries
    float val[DT][16];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      f32x16_t acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const i16x8_t a = *reinterpret_cast<const i16x8_t*>(&sKVW[(32 * t + r) * STR + 16 * c + 8 * g]);
        acc = E::mfma32(a, qf[c], acc);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) val[t][i] = pin_f32(__builtin_fmaf(acc[i], inv_den, sBias[32 * t + 8 * (i >> 2) + 4 * g + (i & 3)]));   // as in the fused epilogue
    }
    store_acc_tile<E, D>(stage, val, oh + (size_t)row0 * pitch_o, residual ? &res : nullptr, rows_valid, lane, pitch_o);
  }
}

// ---- host side ----------------------------------------------------------------------------
int64_t linear_fwd_workspace_bytes(int BH, int L, int D) { return (int64_t)lin_ws(BH, L, D).total; }
int64_t linear_states_bytes(int BH, int L, int D) { return (int64_t)lin_ws(BH, L, D).states_end; }

template <typename Tag, int D>
static int linear_state_impl(const void* k, const void* v, const RowLayout& lay, const float* weight, int fmap, int BH, int L,
                             char* ws, hipStream_t st) {
  const LinWs w = lin_ws(BH, L, D);
  launch_state_build<Tag, D>(k, v, lay, weight, fmap, BH, L, ws, w, st, false);
  hipLaunchKernelGGL((linear_fold_kernel<Tag>), dim3(D / (1024 / D), BH), dim3(256), 0, st,
                     (const uint16_t*)(ws + w.kvt), weight, (uint16_t*)(ws + w.kvwt), (uint16_t*)(ws + w.wt), D);
  return check_launch("linear_state_fwd");
}

// The same with v quantised to FP8 on the way: the state kernel, which streams v anyway, leaves the column maxima of
// |v| per slice, so that the quantiser's own pass over v for them is not needed; the scale and the FP8 copy of v come
// right behind the state kernel, the small kernels that finish the states after them.
template <typename Tag, int D>
static int linear_state_quant_v_impl(const void* k, const void* v, const RowLayout& lay, const float* weight, int dtype, int fmap,
                                     int BH, int L, char* ws, uint8_t* v_fp8, float* v_scale, float v_range, hipStream_t st) {
  const LinWs w = lin_ws(BH, L, D);
  hipLaunchKernelGGL((linear_state_partial_kernel<Tag, D, false, false, true>), dim3(w.nsplit, BH), dim3(256), 0, st,
                     (const uint16_t*)k, (const uint16_t*)v, lay, (float*)(ws + w.kv_part), (float*)(ws + w.z_part), L,
                     w.rows_per_split, fmap, (const float*)nullptr, (float*)(ws + w.vmax_part));
  int rc = quant_v_from_partial_amax(v, lay, dtype, BH, L, D, (const float*)(ws + w.vmax_part), w.nsplit, v_fp8, v_scale,
                                     v_range, st);
  if (rc) return rc;
  hipLaunchKernelGGL((linear_state_reduce_kernel<Tag>), dim3(cdiv(D * D, 256), BH), dim3(256), 0, st,
                     (const float*)(ws + w.kv_part), (const float*)(ws + w.z_part), (uint16_t*)(ws + w.kvt),
                     (uint16_t*)(ws + w.kvp), (uint16_t*)(ws + w.z), w.nsplit, D * D, D);
  hipLaunchKernelGGL((linear_fold_kernel<Tag>), dim3(D / (1024 / D), BH), dim3(256), 0, st,
                     (const uint16_t*)(ws + w.kvt), weight, (uint16_t*)(ws + w.kvwt), (uint16_t*)(ws + w.wt), D);
  return check_launch("linear_state_quant_v_fwd");
}

template <typename Tag, int D>
static int linear_out_impl(const void* q, const RowLayout& lq, const float* bias, const void* residual, void* out,
                           const RowLayout& lout, int fmap, int BH, int L, char* ws, hipStream_t st) {
  const LinWs w = lin_ws(BH, L, D);
  const int tiles = balanced_tiles(cdiv(L, 128), BH, 2);
  if (lq.sl == D && lout.sl == D && lq.sh == (int64_t)L * D && lout.sh == (int64_t)L * D && lq.sb == lq.sh * lq.H &&
      lout.sb == lout.sh * lout.H)
    hipLaunchKernelGGL((linear_out_kernel<Tag, D, true>), dim3(cdiv(L, 128 * tiles), BH), dim3(256), 0, st, (const uint16_t*)q,
                       (const uint16_t*)(ws + w.kvwt), (const uint16_t*)(ws + w.z), bias, (const uint16_t*)residual,
                       (uint16_t*)out, lq, lout, L, fmap, tiles);
  else
    hipLaunchKernelGGL((linear_out_kernel<Tag, D, false>), dim3(cdiv(L, 128 * tiles), BH), dim3(256), 0, st, (const uint16_t*)q,
                       (const uint16_t*)(ws + w.kvwt), (const uint16_t*)(ws + w.z), bias, (const uint16_t*)residual,
                       (uint16_t*)out, lq, lout, L, fmap, tiles);
  return check_launch("linear_out_fwd");
}

int validate_linear(int dtype, int fmap, int B, int H, int L, int D) {
  SLA_REQUIRE(B > 0 && H > 0 && L > 0, SLA_ERR_BAD_ARG, "non-positive size (B=%d H=%d L=%d)", B, H, L);
  SLA_REQUIRE((int64_t)B * H <= 65535, SLA_ERR_UNSUPPORTED, "B*H exceeds 65535");
  SLA_REQUIRE(dtype == SLA_BF16 || dtype == SLA_F16, SLA_ERR_UNSUPPORTED, "linear branch takes bf16 or f16, got dtype %d",
              dtype);
  SLA_REQUIRE(D == 64 || D == 128, SLA_ERR_UNSUPPORTED, "head dim must be 64 or 128, got %d", D);
  SLA_REQUIRE(fmap == SLA_FMAP_ELU || fmap == SLA_FMAP_RELU || fmap == SLA_FMAP_SOFTMAX, SLA_ERR_BAD_ARG,
              "unknown feature map %d", fmap);
  return SLA_OK;
}

}  // namespace sla

using namespace sla;

static int check_linear_ws(int BH, int L, int D, const void* workspace, int64_t workspace_bytes) {
  SLA_REQUIRE(workspace && (uintptr_t)workspace % 16 == 0, SLA_ERR_BAD_ARG, "workspace null or not 16-byte aligned");
  const int64_t need = linear_fwd_workspace_bytes(BH, L, D);
  SLA_REQUIRE(workspace_bytes >= need, SLA_ERR_WORKSPACE, "workspace of %lld bytes, need %lld", (long long)workspace_bytes,
              (long long)need);
  return SLA_OK;
}

static int linear_state_entry(const void* k, const void* v, const int64_t* strides, const float* weight, int dtype, int fmap,
                              int B, int H, int L, int D, void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  SLA_REQUIRE(k && v && weight, SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)k | (uintptr_t)v | (uintptr_t)weight) % 16 == 0, SLA_ERR_BAD_ARG,
              "pointers must be 16-byte aligned");
  const int BH = B * H;
  rc = check_linear_ws(BH, L, D, workspace, workspace_bytes);
  if (rc) return rc;
  RowLayout lay;
  rc = make_layout(strides, B, H, L, D, 2, &lay);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
#define SLA_LIN_CASE(TAG, DD) return linear_state_impl<TAG, DD>(k, v, lay, weight, fmap, BH, L, ws, st)
  if (dtype == SLA_BF16) {
    if (D == 128) SLA_LIN_CASE(bf16_tag, 128);
    SLA_LIN_CASE(bf16_tag, 64);
  }
  if (D == 128) SLA_LIN_CASE(f16_tag, 128);
  SLA_LIN_CASE(f16_tag, 64);
#undef SLA_LIN_CASE
}

extern "C" int sla_linear_state_fwd(const void* k, const void* v, const float* weight, int dtype, int fmap, int B, int H,
                                    int L, int D, void* workspace, int64_t workspace_bytes, void* stream) {
  return linear_state_entry(k, v, nullptr, weight, dtype, fmap, B, H, L, D, workspace, workspace_bytes, stream);
}

extern "C" int sla_linear_state_fwd_strided(const void* k, const void* v, const int64_t* kv_strides, const float* weight,
                                            int dtype, int fmap, int B, int H, int L, int D, void* workspace,
                                            int64_t workspace_bytes, void* stream) {
  SLA_REQUIRE(kv_strides, SLA_ERR_BAD_ARG, "null strides");
  return linear_state_entry(k, v, kv_strides, weight, dtype, fmap, B, H, L, D, workspace, workspace_bytes, stream);
}

static int linear_state_quant_v_entry(const void* k, const void* v, const int64_t* strides, const float* weight, int dtype,
                                      int fmap, int B, int H, int L, int D, void* workspace, int64_t workspace_bytes,
                                      uint8_t* v_fp8, float* v_scale, float v_range, void* stream) {
  int rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  rc = validate_v_range(v_range);
  if (rc) return rc;
  SLA_REQUIRE(k && v && weight && v_fp8 && v_scale, SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)k | (uintptr_t)v | (uintptr_t)weight | (uintptr_t)v_fp8) % 16 == 0, SLA_ERR_BAD_ARG,
              "pointers must be 16-byte aligned");
  const int BH = B * H;
  rc = check_linear_ws(BH, L, D, workspace, workspace_bytes);
  if (rc) return rc;
  RowLayout lay;
  rc = make_layout(strides, B, H, L, D, 2, &lay);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
#define SLA_LIN_CASE(TAG, DD) \
  return linear_state_quant_v_impl<TAG, DD>(k, v, lay, weight, dtype, fmap, BH, L, ws, v_fp8, v_scale, v_range, st)
  if (dtype == SLA_BF16) {
    if (D == 128) SLA_LIN_CASE(bf16_tag, 128);
    SLA_LIN_CASE(bf16_tag, 64);
  }
  if (D == 128) SLA_LIN_CASE(f16_tag, 128);
  SLA_LIN_CASE(f16_tag, 64);
#undef SLA_LIN_CASE
}

extern "C" int sla_linear_state_quant_v_fwd(const void* k, const void* v, const float* weight, int dtype, int fmap, int B,
                                            int H, int L, int D, void* workspace, int64_t workspace_bytes, uint8_t* v_fp8,
                                            float* v_scale, float v_range, void* stream) {
  return linear_state_quant_v_entry(k, v, nullptr, weight, dtype, fmap, B, H, L, D, workspace, workspace_bytes, v_fp8, v_scale,
                                    v_range, stream);
}

extern "C" int sla_linear_state_quant_v_fwd_strided(const void* k, const void* v, const int64_t* kv_strides,
                                                    const float* weight, int dtype, int fmap, int B, int H, int L, int D,
                                                    void* workspace, int64_t workspace_bytes, uint8_t* v_fp8,
                                                    float* v_scale, float v_range, void* stream) {
  SLA_REQUIRE(kv_strides, SLA_ERR_BAD_ARG, "null strides");
  return linear_state_quant_v_entry(k, v, kv_strides, weight, dtype, fmap, B, H, L, D, workspace, workspace_bytes, v_fp8,
                                    v_scale, v_range, stream);
}

static int linear_out_entry(const void* q, const int64_t* q_strides, const float* bias, const void* residual, void* out,
                            const int64_t* out_strides, int dtype, int fmap, int B, int H, int L, int D, void* workspace,
                            int64_t workspace_bytes, void* stream) {
  int rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  RowLayout lq, lout;
  rc = make_layout(q_strides, B, H, L, D, 2, &lq);
  if (rc) return rc;
  rc = make_layout(out_strides, B, H, L, D, 2, &lout);
  if (rc) return rc;
  SLA_REQUIRE(q && bias && out, SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)out | (uintptr_t)residual) % 16 == 0, SLA_ERR_BAD_ARG,
              "pointers must be 16-byte aligned");
  const int BH = B * H;
  rc = check_linear_ws(BH, L, D, workspace, workspace_bytes);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
#define SLA_LIN_CASE(TAG, DD) return linear_out_impl<TAG, DD>(q, lq, bias, residual, out, lout, fmap, BH, L, ws, st)
  if (dtype == SLA_BF16) {
    if (D == 128) SLA_LIN_CASE(bf16_tag, 128);
    SLA_LIN_CASE(bf16_tag, 64);
  }
  if (D == 128) SLA_LIN_CASE(f16_tag, 128);
  SLA_LIN_CASE(f16_tag, 64);
#undef SLA_LIN_CASE
}

extern "C" int sla_linear_out_fwd(const void* q, const float* bias, const void* residual, void* out, int dtype, int fmap,
                                  int B, int H, int L, int D, void* workspace, int64_t workspace_bytes, void* stream) {
  return linear_out_entry(q, nullptr, bias, residual, out, nullptr, dtype, fmap, B, H, L, D, workspace, workspace_bytes, stream);
}

extern "C" int sla_linear_out_fwd_strided(const void* q, const int64_t* q_strides, const float* bias, const void* residual,
                                          void* out, const int64_t* out_strides, int dtype, int fmap, int B, int H, int L,
                                          int D, void* workspace, int64_t workspace_bytes, void* stream) {
  SLA_REQUIRE(q_strides && out_strides, SLA_ERR_BAD_ARG, "null strides");
  return linear_out_entry(q, q_strides, bias, residual, out, out_strides, dtype, fmap, B, H, L, D, workspace, workspace_bytes,
                          stream);
}

extern "C" int sla_linear_fwd(const void* q, const void* k, const void* v, const float* weight, const float* bias,
                              const void* residual, void* out, int dtype, int fmap, int B, int H, int L, int D,
                              void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  SLA_REQUIRE(q && k && v && weight && bias && out && workspace, SLA_ERR_BAD_ARG, "null pointer");
  rc = sla_linear_state_fwd(k, v, weight, dtype, fmap, B, H, L, D, workspace, workspace_bytes, stream);
  if (rc) return rc;
  return sla_linear_out_fwd(q, bias, residual, out, dtype, fmap, B, H, L, D, workspace, workspace_bytes, stream);
}
