// The two backward calls of the module cut into steps, so that one caller can put the short kernels of both on a
// second stream beside the long ones (module_bwd.hip); each call on its own runs every step on one stream.
#pragma once
#include "common.h"

namespace sla {

// block-sparse attention backward
constexpr int SB_LISTS = 1;   // per-key-block lists of the map and their segments (needs the map only)
constexpr int SB_DQ = 2;      // delta and dQ (needs nothing of SB_LISTS)
constexpr int SB_DKDV = 4;    // dK / dV over the lists (needs SB_LISTS, and the delta of SB_DQ)
constexpr int SB_ALL = 7;
int attn_bwd_steps(const void* q, const void* k, const void* v, const int64_t* qkv_strides, const void* o, const void* d_o,
                   const int64_t* do_strides, const float* lse, const int8_t* sparse_map, const void* lut, int lut_elem_bytes,
                   void* dq, void* dk, void* dv, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK, int topk,
                   float qk_scale, void* workspace, int64_t workspace_bytes, void* stream, int steps);

// linear branch backward
constexpr int LB_STATES = 1;  // the forward's per-head states again (skipped with SLA_BWD_STATES_READY)
constexpr int LB_QUERY = 2;   // dq and the sums over the rows (needs LB_STATES)
constexpr int LB_REDUCE = 4;  // dS, dz, d_weight, d_bias from those sums (short kernels)
constexpr int LB_KEYS = 8;    // dk, dv (needs LB_REDUCE)
constexpr int LB_ALL = 15;
int linear_bwd_steps(const void* q, const void* k, const void* v, const int64_t* qkv_strides, const float* weight,
                     const float* bias, const void* d_out, const int64_t* do_strides, void* dq, void* dk, void* dv,
                     float* d_weight, float* d_bias, int dtype, int fmap, int B, int H, int L, int D, int flags,
                     void* workspace, int64_t workspace_bytes, void* stream, int steps);

}  // namespace sla
