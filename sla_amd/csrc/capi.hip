// Library-wide pieces of the C ABI: version, error text, workspace sizes.
#include "common.h"

namespace sla {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return SLA_ERR_LAUNCH;
  }
  return SLA_OK;
}

int make_layout(const int64_t* strides, int B, int H, int L, int D, int elem_bytes, RowLayout* out) {
  if (!strides) {
    SLA_REQUIRE(((int64_t)(L + 255) * D + D) * elem_bytes < (1ll << 32), SLA_ERR_UNSUPPORTED,
                "one head spans 4 GiB or more (L=%d D=%d)", L, D);
    *out = contiguous_layout(H, L, D);
    return SLA_OK;
  }
  const int64_t sb = strides[0], sh = strides[1], sl = strides[2];
  const int64_t vec = 16 / elem_bytes;     // elements per 16-byte access
  SLA_REQUIRE(sl >= D && sh > 0 && sb > 0, SLA_ERR_BAD_ARG, "strides (%lld, %lld, %lld): the row stride must be at least D=%d and all must be positive",
              (long long)sb, (long long)sh, (long long)sl, D);
  SLA_REQUIRE(sb % vec == 0 && sh % vec == 0 && sl % vec == 0, SLA_ERR_BAD_ARG,
              "strides (%lld, %lld, %lld) must be multiples of %lld elements (16-byte aligned rows)", (long long)sb,
              (long long)sh, (long long)sl, (long long)vec);
  // rows of different heads must not overlap (the backward writes gradients through the same layout): either a
  // head's rows end before the next head starts, or the heads are interleaved inside one token's row
  SLA_REQUIRE(H == 1 || sh >= (int64_t)(L - 1) * sl + D || (sh >= D && sl >= (int64_t)(H - 1) * sh + D), SLA_ERR_BAD_ARG,
              "strides (%lld, %lld, %lld): rows of different heads overlap (H=%d L=%d D=%d)", (long long)sb, (long long)sh,
              (long long)sl, H, L, D);
  // (32-bit byte offsets inside a head; kernels that take whole tiles of rows form offsets of up to 255 rows past L,
  //  which must still lie beyond the head's range instead of wrapping around)
  SLA_REQUIRE(((int64_t)(L + 255) * sl + D) * elem_bytes < (1ll << 32), SLA_ERR_UNSUPPORTED,
              "one head spans 4 GiB or more with row stride %lld", (long long)sl);
  *out = RowLayout{sb, sh, sl, H};
  return SLA_OK;
}

int64_t block_map_workspace_bytes(int dtype, int BH, int L, int D, int BLKQ, int BLKK);
int64_t sparse_bwd_workspace_bytes(int BH, int L, int D, int BLKQ, int BLKK, int topk);
int64_t linear_fwd_workspace_bytes(int BH, int L, int D);
int64_t linear_bwd_workspace_bytes(int BH, int L, int D);
int64_t sage_quant_workspace_bytes(int BH, int L, int D);
int64_t sage_prepare_workspace_bytes(int BH, int L, int D);
int64_t linear_states_bytes(int BH, int L, int D);
int64_t linear_complement_workspace_bytes(int BH, int L, int D);
int64_t linear_complement_bwd_workspace_bytes(int BH, int L, int D, int BLKQ);

}  // namespace sla

using namespace sla;

extern "C" int sla_version(void) { return 1; }

extern "C" const char* sla_last_error(void) { return g_err; }

extern "C" int64_t sla_workspace_bytes(int op, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK, int topk) {
  SLA_REQUIRE(B > 0 && H > 0 && L > 0 && D > 0, SLA_ERR_BAD_ARG, "non-positive size (B=%d H=%d L=%d D=%d)", B, H, L, D);
  SLA_REQUIRE((int64_t)B * H <= 65535, SLA_ERR_UNSUPPORTED, "B*H exceeds 65535");
  const int BH = B * H;
  switch (op) {
    case SLA_WS_BLOCK_MAP:
      SLA_REQUIRE(BLKQ > 0 && BLKK > 0, SLA_ERR_BAD_ARG, "non-positive block size");
      SLA_REQUIRE(dtype == SLA_F32 || dtype == SLA_BF16 || dtype == SLA_F16, SLA_ERR_BAD_ARG, "unknown dtype %d", dtype);
      return block_map_workspace_bytes(dtype, BH, L, D, BLKQ, BLKK);
    case SLA_WS_SPARSE_BWD:
      SLA_REQUIRE(BLKQ > 0 && BLKK > 0 && topk >= 0, SLA_ERR_BAD_ARG, "bad block size / topk");
      return sparse_bwd_workspace_bytes(BH, L, D, BLKQ, BLKK, topk);
    case SLA_WS_LINEAR_FWD:
      return linear_fwd_workspace_bytes(BH, L, D);
    case SLA_WS_LINEAR_BWD:
      return linear_bwd_workspace_bytes(BH, L, D);
    case SLA_WS_SAGE_QUANT:
      return sage_quant_workspace_bytes(BH, L, D);
    case SLA_WS_LINEAR_STATES:
      return linear_states_bytes(BH, L, D);
    case SLA_WS_SAGE_PREPARE:
      return sage_prepare_workspace_bytes(BH, L, D);
    case SLA_WS_LINEAR_COMPLEMENT:
      return linear_complement_workspace_bytes(BH, L, D);
    case SLA_WS_LINEAR_COMPLEMENT_BWD:
      SLA_REQUIRE(BLKQ == 64 || BLKQ == 128, SLA_ERR_UNSUPPORTED, "BLKQ=%d (64 or 128)", BLKQ);
      return linear_complement_bwd_workspace_bytes(BH, L, D, BLKQ);
    default:
      set_error("unknown workspace op %d", op);
      return SLA_ERR_BAD_ARG;
  }
}
