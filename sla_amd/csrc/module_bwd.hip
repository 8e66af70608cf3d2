// Backward of the whole module (block-sparse attention + linear branch + projection) as one call.
//
// Stands in for autograd through SparseLinearAttention.forward of the reference (sparse_linear_attention/core.py:88-100:
// _attention.backward, kernel.py:277-320, and the autograd graph of calc_linear / proj_l).  It launches the kernels of
// sla_sparse_attn_bwd and sla_linear_bwd (with SLA_BWD_ACCUMULATE: the linear branch adds into dq, dk, dv), in this order
// on `stream`:
//     delta, dQ | linear branch: dq and the sums over the rows | dK/dV | linear branch: dk, dv
// and, when the caller passes a second stream, the short kernels on it beside the long ones:
//     the per-key-block lists of the map (needed by dK/dV only)            beside delta and dQ
//     dS, dz, d_weight, d_bias from the sums (needed by dk, dv of the linear branch)   beside dK/dV
// `stream` waits for everything put on `side_stream` before the call returns, so the caller orders later work by
// `stream` alone.  The results equal the two separate calls bit for bit.
#include "bwd_steps.h"

#include <mutex>

namespace sla {
namespace {

// Events that order the two streams, one set per device, made on first use and kept.  A call records and waits on them
// while it holds the lock: calls from several host threads take turns enqueueing.
struct SideEvents {
  hipEvent_t fork = nullptr, lists = nullptr, query = nullptr, reduced = nullptr;
};
std::mutex g_mu;
SideEvents g_ev[64];

int events_for_current_device(SideEvents** out) {
  int dev = 0;
  SLA_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64, SLA_ERR_LAUNCH, "no current device");
  SideEvents& e = g_ev[dev];
  if (!e.fork) {
    // all four or none: the set is published only when every event exists
    hipEvent_t made[4] = {nullptr, nullptr, nullptr, nullptr};
    for (int i = 0; i < 4; ++i) {
      if (hipEventCreateWithFlags(&made[i], hipEventDisableTiming) != hipSuccess) {
        for (int j = 0; j < i; ++j) (void)hipEventDestroy(made[j]);
        set_error("hipEventCreate failed");
        return SLA_ERR_LAUNCH;
      }
    }
    e.lists = made[1];
    e.query = made[2];
    e.reduced = made[3];
    e.fork = made[0];
  }
  *out = &e;
  return SLA_OK;
}

}  // namespace
}  // namespace sla

using namespace sla;

#define SLA_HIP_OK(call) SLA_REQUIRE((call) == hipSuccess, SLA_ERR_LAUNCH, #call " failed")

extern "C" int sla_module_bwd(const void* q, const void* k, const void* v, const int64_t* qkv_strides, const void* o_s,
                              const void* d_out, const int64_t* do_strides, const float* lse, const int8_t* sparse_map,
                              const void* lut, int lut_elem_bytes, const float* weight, const float* bias, void* dq, void* dk,
                              void* dv, float* d_weight, float* d_bias, int dtype, int fmap, int B, int H, int L, int D,
                              int BLKQ, int BLKK, int topk, float qk_scale, int flags, void* sparse_workspace,
                              int64_t sparse_workspace_bytes, void* linear_workspace, int64_t linear_workspace_bytes,
                              void* stream, void* side_stream) {
  SLA_REQUIRE((flags & ~SLA_BWD_STATES_READY) == 0, SLA_ERR_BAD_ARG, "unknown flag bits in %d", flags);
  SLA_REQUIRE((qkv_strides == nullptr) == (do_strides == nullptr), SLA_ERR_BAD_ARG, "pass both stride arrays or neither");
  const int lflags = flags | SLA_BWD_ACCUMULATE;
  hipStream_t st = (hipStream_t)stream, side = (hipStream_t)side_stream;
  const auto sparse = [&](hipStream_t s, int steps) {
    return attn_bwd_steps(q, k, v, qkv_strides, o_s, d_out, do_strides, lse, sparse_map, lut, lut_elem_bytes, dq, dk, dv, dtype,
                          B, H, L, D, BLKQ, BLKK, topk, qk_scale, sparse_workspace, sparse_workspace_bytes, s, steps);
  };
  const auto linear = [&](hipStream_t s, int steps) {
    return linear_bwd_steps(q, k, v, qkv_strides, weight, bias, d_out, do_strides, dq, dk, dv, d_weight, d_bias, dtype, fmap, B,
                            H, L, D, lflags, linear_workspace, linear_workspace_bytes, s, steps);
  };
  int rc;
  // every argument of both calls is checked before the first kernel of either is launched
  if ((rc = sparse(st, 0))) return rc;
  if ((rc = linear(st, 0))) return rc;
  if (!side || side == st) {
    // one stream: the same order, the short kernels in between
    if ((rc = sparse(st, SB_ALL))) return rc;
    return linear(st, LB_ALL);
  }
  std::lock_guard<std::mutex> lock(g_mu);
  SideEvents* ev;
  if ((rc = events_for_current_device(&ev))) return rc;
  // Once the second stream has been made to wait on `stream`, no path leaves this call without `stream` waiting for
  // the second one in turn: the caller orders later work (and the reuse of the workspaces) by `stream` alone, and a
  // capture in progress must not be left forked.
  const auto forked = [&]() -> int {
    int r;
    // side: lists of the map.  main: delta, dQ, then the query side of the linear branch
    if ((r = sparse(side, SB_LISTS))) return r;
    SLA_HIP_OK(hipEventRecord(ev->lists, side));
    if ((r = sparse(st, SB_DQ))) return r;
    if ((r = linear(st, LB_STATES | LB_QUERY))) return r;
    SLA_HIP_OK(hipEventRecord(ev->query, st));
    // side: the small products of the linear branch.  main: dK/dV, then the key side of the linear branch
    SLA_HIP_OK(hipStreamWaitEvent(side, ev->query, 0));
    if ((r = linear(side, LB_REDUCE))) return r;
    SLA_HIP_OK(hipEventRecord(ev->reduced, side));
    SLA_HIP_OK(hipStreamWaitEvent(st, ev->lists, 0));
    if ((r = sparse(st, SB_DKDV))) return r;
    SLA_HIP_OK(hipStreamWaitEvent(st, ev->reduced, 0));
    return linear(st, LB_KEYS);
  };
  SLA_HIP_OK(hipEventRecord(ev->fork, st));
  SLA_HIP_OK(hipStreamWaitEvent(side, ev->fork, 0));
  rc = forked();
  if (rc) {
    // join whatever the second stream was given before the failure (its last event may never have been recorded)
    if (hipEventRecord(ev->reduced, side) == hipSuccess) (void)hipStreamWaitEvent(st, ev->reduced, 0);
  }
  return rc;
}
