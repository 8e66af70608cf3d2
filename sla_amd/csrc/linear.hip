// Linear-attention branch, projection and final sum for gfx950.
//
// Stands in for sparse_linear_attention/core.py:90-100 of the reference:
//   fq = phi(q), fk = phi(k)                       (feature maps, 16-bit results)
//   kvsum = fk^T v (DxD), ksum = sum_L fk (1xD)      (16-bit results)
//   o_l = (fq kvsum) / (1e-5 + sum_d fq*ksum)        (16-bit results)
//   out = o_s + (o_l W^T + b)                        (W, b cast to 16 bit as autocast does)
//
// Three kernels:
//   state_partial : streams K and V once; each workgroup owns a slice of L and forms its
//                   share of phi(K)^T V on the MFMA (both operands read transposed from LDS)
//                   and of sum phi(K) on the vector ALU; fp32 partials to the workspace.
//   state_reduce  : adds the partials in ascending slice order, rounds to 16 bit, stores the
//                   state TRANSPOSED (KVT[d2][d1]) so the next kernel reads MFMA rows directly.
//   out           : one wavefront per 32 queries.  Both products are formed transposed
//                   (N^T = KVT phi(Q)^T, then OUT^T = W Y^T) so the per-query divisor is a
//                   per-lane scalar and Y^T leaves the first accumulator already in the
//                   B-operand layout of the second product.
#include "linear_state.h"

namespace sla {

// ---- kernel 3: output --------------------------------------------------------------------
// grid (ceil(L / (128*TILES)), BH), 256 threads = 4 waves x 32 queries, TILES steps per workgroup.
template <typename Tag, int D>
__global__ __launch_bounds__(256) void linear_out_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ kvt,
                                                         const uint16_t* __restrict__ z, const float* __restrict__ weight,
                                                         const float* __restrict__ bias, const uint16_t* __restrict__ residual,
                                                         uint16_t* __restrict__ out, int L, int fmap, int tiles_per_wg) {
  using E = Elem<Tag>;
  constexpr int DC = D / 16;
  constexpr int DT = D / 32;
  constexpr int STR = D + 8;
  __shared__ __attribute__((aligned(16))) uint16_t sKVT[D * STR];   // [d2][d1]
  __shared__ __attribute__((aligned(16))) uint16_t sW[D * STR];     // [e][slot-permuted d2]
  __shared__ float sBias[D];
  __shared__ float sZ[D];

  const int bh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;

  // stage the state and the projection once per workgroup
  {
    const uint16_t* src = kvt + (size_t)bh * D * D;
    for (int idx = tid; idx < D * D / 8; idx += 256) {
      const int row = idx / (D / 8), col = (idx % (D / 8)) * 8;
      *reinterpret_cast<i16x8_t*>(&sKVT[row * STR + col]) = *reinterpret_cast<const i16x8_t*>(src + (size_t)row * D + col);
    }
    // W[e][.] re-ordered so that the 8 contraction slots of lane group gg in chunk c are adjacent:
    // slot j <-> d2 = 16c + 8*(j/4) + 4gg + j%4  (the accumulator layout of the first product)
    for (int idx = tid; idx < D * DC * 2; idx += 256) {
      const int e = idx / (DC * 2), c = (idx / 2) % DC, gg = idx & 1;
      const float* w0 = weight + (size_t)e * D + 16 * c + 4 * gg;
      const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(w0);
      const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(w0 + 8);
      i32x4_t pw;
      pw[0] = (int)E::pack2(lo[0], lo[1]);
      pw[1] = (int)E::pack2(lo[2], lo[3]);
      pw[2] = (int)E::pack2(hi[0], hi[1]);
      pw[3] = (int)E::pack2(hi[2], hi[3]);
      *reinterpret_cast<i32x4_t*>(&sW[e * STR + 16 * c + 8 * gg]) = pw;
    }
    if (tid < D) {
      sBias[tid] = round16<Tag>(bias[tid]);
      sZ[tid] = E::to_float(z[(size_t)bh * D + tid]);
    }
  }
  __syncthreads();

  const uint16_t* qh = q + (size_t)bh * L * D;
  for (int tt = 0; tt < tiles_per_wg; ++tt) {
    const int row0 = (blockIdx.x * tiles_per_wg + tt) * 128 + wave * 32;
    if (row0 >= L) break;
    const int qrow = row0 + r;
    const bool ok = qrow < L;

    // phi(q): this lane holds d = 16c + 8g + j of its row; lane^32 holds the other half
    float f[DC][8];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i16x8_t x = {0, 0, 0, 0, 0, 0, 0, 0};
      if (ok) x = *reinterpret_cast<const i16x8_t*>(qh + (size_t)qrow * D + 16 * c + 8 * g);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[c][j] = E::to_float((uint16_t)x[j]);
    }
    float row_mx, row_inv;
    phi_row_pair<Tag, DC>(fmap, f, row_mx, row_inv);
    // divisor: 1e-5 + sum_d round16(fq*z), each step rounded to 16 bit as the reference's tensors are
    float den = 0.f;
    i16x8_t qf[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      i32x4_t pw;
#pragma unroll
      for (int j = 0; j < 8; ++j) den += round16<Tag>(f[c][j] * sZ[16 * c + 8 * g + j]);
#pragma unroll
      for (int j = 0; j < 4; ++j) pw[j] = (int)E::pack2(f[c][2 * j], f[c][2 * j + 1]);
      qf[c] = __builtin_bit_cast(i16x8_t, pw);
    }
    den += __shfl_xor(den, 32);
    den = round16<Tag>(1e-5f + round16<Tag>(den));
    const float inv_den = 1.0f / den;

    // N^T = KVT phi(Q)^T : DT tiles of 32 d2-rows x 32 queries
    f32x16_t nacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
      for (int i = 0; i < 16; ++i) nacc[t][i] = 0.f;
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const i16x8_t a = *reinterpret_cast<const i16x8_t*>(&sKVT[(32 * t + r) * STR + 16 * c + 8 * g]);
        nacc[t] = E::mfma32(a, qf[c], nacc[t]);
      }
    }
    // Y^T = round16(round16(N^T) / den), packed straight into B-operand fragments
    i16x8_t yf[DT][2];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        i32x4_t pw;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float a = round16<Tag>(nacc[t][8 * c2 + 2 * j]) * inv_den;
          const float b = round16<Tag>(nacc[t][8 * c2 + 2 * j + 1]) * inv_den;
          pw[j] = (int)E::pack2(a, b);
        }
        yf[t][c2] = __builtin_bit_cast(i16x8_t, pw);
      }
    // OUT^T = W Y^T : contraction chunk (t, c2) covers d2 = 32t + 16c2 .. +15
    f32x16_t oacc[DT];
#pragma unroll
    for (int et = 0; et < DT; ++et) {
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[et][i] = 0.f;
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {
          const i16x8_t a = *reinterpret_cast<const i16x8_t*>(&sW[(32 * et + r) * STR + 16 * (2 * t + c2) + 8 * g]);
          oacc[et] = E::mfma32(a, yf[t][c2], oacc[et]);
        }
    }
    if (ok) {
      const size_t off = ((size_t)bh * L + qrow) * D;
#pragma unroll
      for (int et = 0; et < DT; ++et)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          const int e0 = 32 * et + 8 * i4 + 4 * g;
          float y[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) y[j] = round16<Tag>(oacc[et][4 * i4 + j] + sBias[e0 + j]);
          if (residual) {
            const i32x2_t rv = *reinterpret_cast<const i32x2_t*>(residual + off + e0);
            const uint16_t* rp = reinterpret_cast<const uint16_t*>(&rv);
#pragma unroll
            for (int j = 0; j < 4; ++j) y[j] += E::to_float(rp[j]);
          }
          i32x2_t w;
          w[0] = (int)E::pack2(y[0], y[1]);
          w[1] = (int)E::pack2(y[2], y[3]);
          *reinterpret_cast<i32x2_t*>(out + off + e0) = w;
        }
    }
  }
}

// ---- host side ----------------------------------------------------------------------------
int64_t linear_fwd_workspace_bytes(int BH, int L, int D) { return (int64_t)lin_ws(BH, L, D).total; }

template <typename Tag, int D>
static int linear_fwd_impl(const void* q, const void* k, const void* v, const float* weight, const float* bias,
                           const void* residual, void* out, int fmap, int BH, int L, char* ws, hipStream_t st) {
  const LinWs w = lin_ws(BH, L, D);
  uint16_t* kvt = (uint16_t*)(ws + w.kvt);
  uint16_t* z = (uint16_t*)(ws + w.z);
  launch_state_build<Tag, D>(k, v, fmap, BH, L, ws, w, st);
  const int tiles = 4;
  hipLaunchKernelGGL((linear_out_kernel<Tag, D>), dim3(cdiv(L, 128 * tiles), BH), dim3(256), 0, st, (const uint16_t*)q, kvt,
                     z, weight, bias, (const uint16_t*)residual, (uint16_t*)out, L, fmap, tiles);
  return check_launch("linear_fwd");
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

extern "C" int sla_linear_fwd(const void* q, const void* k, const void* v, const float* weight, const float* bias,
                              const void* residual, void* out, int dtype, int fmap, int B, int H, int L, int D,
                              void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = validate_linear(dtype, fmap, B, H, L, D);
  if (rc) return rc;
  SLA_REQUIRE(q && k && v && weight && bias && out && workspace, SLA_ERR_BAD_ARG, "null pointer");
  SLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)residual | (uintptr_t)weight |
               (uintptr_t)workspace) % 16 == 0,
              SLA_ERR_BAD_ARG, "pointers must be 16-byte aligned");
  const int BH = B * H;
  const int64_t need = linear_fwd_workspace_bytes(BH, L, D);
  SLA_REQUIRE(workspace_bytes >= need, SLA_ERR_WORKSPACE, "workspace of %lld bytes, need %lld", (long long)workspace_bytes,
              (long long)need);
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
#define SLA_LIN_CASE(TAG, DD) return linear_fwd_impl<TAG, DD>(q, k, v, weight, bias, residual, out, fmap, BH, L, ws, st)
  if (dtype == SLA_BF16) {
    if (D == 128) SLA_LIN_CASE(bf16_tag, 128);
    SLA_LIN_CASE(bf16_tag, 64);
  }
  if (D == 128) SLA_LIN_CASE(f16_tag, 128);
  SLA_LIN_CASE(f16_tag, 64);
#undef SLA_LIN_CASE
}
