/*
 * C ABI of the MI355X (gfx950) Sparse-Linear Attention kernels.
 *
 * The reference operator is Python; it has no FFI of its own.  Each entry point
 * below replaces one device-side step of the reference and names the reference
 * lines it stands in for (paths inside the reference checkout).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise; tensors are
 *     dense, row-major, (B,H,L,D) with D fastest;
 *   - the caller owns every buffer including workspaces (sizes from
 *     sla_workspace_bytes); the library allocates nothing and keeps no state;
 *   - `stream` is a hipStream_t passed as void*; all work is enqueued on it and
 *     no call synchronises with the host;
 *   - return value 0 = success, negative = error (see SLA_ERR_*); the message of
 *     the last error on the calling thread is returned by sla_last_error();
 *   - argument validation happens before any device work, so error paths can be
 *     exercised on a host without a GPU.
 */
#ifndef SLA_HIP_H
#define SLA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SLA_OK 0
#define SLA_ERR_BAD_ARG (-1)      /* null pointer, non-positive size, bad enum   */
#define SLA_ERR_UNSUPPORTED (-2)  /* shape / block size / dtype not implemented   */
#define SLA_ERR_LAUNCH (-3)       /* the HIP runtime refused a launch             */
#define SLA_ERR_WORKSPACE (-4)    /* workspace smaller than sla_workspace_bytes   */

/* element types */
#define SLA_F32 0
#define SLA_BF16 1
#define SLA_F16 2

/* feature maps of the linear branch (reference core.py:43-57) */
#define SLA_FMAP_ELU 0
#define SLA_FMAP_RELU 1
#define SLA_FMAP_SOFTMAX 2

/* operations that need a workspace */
#define SLA_WS_BLOCK_MAP 0
#define SLA_WS_SPARSE_BWD 1
#define SLA_WS_LINEAR_FWD 2
#define SLA_WS_LINEAR_BWD 3
#define SLA_WS_SAGE_QUANT 4
#define SLA_WS_LINEAR_COMPLEMENT 5
#define SLA_WS_SAGE_PREPARE 6
#define SLA_WS_LINEAR_STATES 7 /* not an operation: the leading bytes of the SLA_WS_LINEAR_FWD workspace that hold the
                                  finished per-head states (see sla_linear_bwd, SLA_BWD_STATES_READY) */
#define SLA_WS_LINEAR_COMPLEMENT_BWD 8

/* flags of sla_linear_bwd */
#define SLA_BWD_ACCUMULATE 1   /* dq, dk, dv already hold the sparse branch's gradients: add to them */
#define SLA_BWD_STATES_READY 2 /* the workspace already starts with the states of the forward: do not rebuild them */

int sla_version(void);
const char* sla_last_error(void);

/* Bytes of caller-provided workspace an operation needs for the given problem.
 * Returns a negative error code for unsupported arguments. */
int64_t sla_workspace_bytes(int op, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK, int topk);

/* Per-block mean over rows: x (B*H, L, D) -> out (B*H, ceil(L/BLK), D), same dtype.
 * Replaces mean_pool + compress_kernel, sparse_linear_attention/utils.py:21-52. */
int sla_mean_pool(const void* x, void* out, int dtype, int BH, int L, int D, int BLK, void* stream);

/* Block-mask builder: K mean smoothing, block pooling, pooled scores, per-row
 * top-k (ties to the lowest index).  Writes the int8 0/1 map (B*H, M, N) and the
 * ascending look-up table (B*H, M, topk) with elements of lut_elem_bytes (4 or 8).
 * topk = min(N, int(ratio*N)) is computed by the caller.
 * Limits: N = ceil(L/BLKK) <= 4096 key blocks (L <= 262144), B*H <= 65535; more returns SLA_ERR_UNSUPPORTED
 * (sage_prepare has the same limits).
 * Replaces get_block_map, sparse_linear_attention/utils.py:55-67. */
int sla_block_map_fwd(const void* q, const void* k, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK,
                      int topk, void* workspace, int64_t workspace_bytes, int8_t* sparse_map, void* lut,
                      int lut_elem_bytes, void* stream);

/* sla_block_map_fwd for callers that cannot allocate device memory and have no workspace to lend (code under HIP
 * graph capture, serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same kernels
 * and results as sla_block_map_fwd; the workspace is a fixed array of SLA_STATIC_SCRATCH_BYTES in device memory that
 * every GPU the library runs on holds until the process ends.  Problems whose sla_workspace_bytes(SLA_WS_BLOCK_MAP,
 * ...) exceeds that size are refused with SLA_ERR_WORKSPACE (B1 H12 L32760 D128 64/64 in bf16 needs 12.7 MB and fits).
 * Calls no hipMalloc / hipFree.  The first call on a GPU looks up the array's device address (make it once outside a
 * graph capture); the GPU that `stream` belongs to must be the current device.  All calls on one GPU share the array:
 * calls that overlap in time on one GPU (different streams) race; nothing in it needs clearing between calls. */
#define SLA_STATIC_SCRATCH_BYTES (16u << 20)
int sla_block_map_fwd_static(const void* q, const void* k, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK,
                             int topk, int8_t* sparse_map, void* lut, int lut_elem_bytes, void* stream);

/* Block-sparse FlashAttention forward over the look-up table.
 * o (B,H,L,D) in `dtype`, lse (B,H,L) fp32 = m + log2(l) in qk_scale*log2(e) units.
 * BLKQ in {64,128}, BLKK == 64, D in {64,128}, dtype bf16 or f16.
 * Replaces _attention.forward + _attn_fwd, sparse_linear_attention/kernel.py:21-82, 242-274. */
int sla_sparse_attn_fwd(const void* q, const void* k, const void* v, const void* lut, int lut_elem_bytes,
                        void* o, float* lse, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK,
                        int topk, float qk_scale, void* stream);

/* The attention forward with the module's linear branch and final sum fused into its epilogue:
 *   out = o_s + proj(o_l),  o_l = phi(q) KV / (1e-5 + phi(q) z)
 * for callers that own both branches.  `linear_workspace` is the workspace sla_linear_state_fwd filled for
 * the same k, v, weight, fmap (size SLA_WS_LINEAR_FWD); bias (D) fp32.  o_s (optional, may be NULL) receives
 * the attention output alone, which the backward needs; out and o_s in `dtype`.  Equal bit for bit to
 * sla_sparse_attn_fwd followed by sla_linear_out_fwd with residual = o_s.
 * Replaces kernel.py:21-82, 242-274 and core.py:90-100 (q feature map, rest of calc_linear, proj_l, sum). */
int sla_sparse_attn_linear_fwd(const void* q, const void* k, const void* v, const void* lut, int lut_elem_bytes,
                               const void* linear_workspace, int64_t linear_workspace_bytes, const float* bias,
                               void* o_s, void* out, float* lse, int dtype, int fmap, int B, int H, int L, int D,
                               int BLKQ, int BLKK, int topk, float qk_scale, void* stream);

/* Block-sparse FlashAttention backward: delta, dQ over the look-up table, dK/dV
 * over per-key-block lists built from the int8 map.  sparse_map and lut are the pair sla_block_map_fwd
 * produced: every map row holds `topk` ones, the same blocks the look-up row names (the workspace,
 * SLA_WS_SPARSE_BWD, is sized from topk; lists of key blocks that very many query blocks selected are cut
 * into segments whose fp32 partials are added in a fixed order, so the result does not depend on scheduling).
 * Replaces _attention.backward + _attn_bwd_preprocess/_dq/_dkdv,
 * sparse_linear_attention/kernel.py:85-237, 277-320. */
int sla_sparse_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                        const float* lse, const int8_t* sparse_map, const void* lut, int lut_elem_bytes,
                        void* dq, void* dk, void* dv, int dtype, int B, int H, int L, int D, int BLKQ,
                        int BLKK, int topk, float qk_scale, void* workspace, int64_t workspace_bytes,
                        void* stream);

/* Linear branch forward: feature maps, phi(K)^T V and sum phi(K) states, phi(Q) H / (1e-5 + phi(Q) z),
 * projection by W (D,D) fp32 and bias (D) fp32, plus `residual` (the sparse output, may be null).
 * out = residual + proj(o_l), in `dtype`.
 * Replaces sparse_linear_attention/core.py:90-100 (feature maps, calc_linear, proj_l, sum). */
int sla_linear_fwd(const void* q, const void* k, const void* v, const float* weight, const float* bias,
                   const void* residual, void* out, int dtype, int fmap, int B, int H, int L, int D,
                   void* workspace, int64_t workspace_bytes, void* stream);

/* The two halves of sla_linear_fwd, for callers that overlap them with other work: the state half
 * depends on k and v only (it can run beside the mask builder on another stream), the output half
 * consumes the workspace the state half filled (same workspace size, SLA_WS_LINEAR_FWD).
 * sla_linear_fwd == sla_linear_state_fwd followed by sla_linear_out_fwd on one stream.
 * Replace sparse_linear_attention/core.py:90-95 (feature map of k, calc_linear's k^T v and k sum) and
 * core.py:90-100 (feature map of q, the rest of calc_linear, proj_l, sum) respectively. */
int sla_linear_state_fwd(const void* k, const void* v, const float* weight, int dtype, int fmap, int B, int H, int L,
                         int D, void* workspace, int64_t workspace_bytes, void* stream);
int sla_linear_out_fwd(const void* q, const float* bias, const void* residual, void* out, int dtype, int fmap, int B,
                       int H, int L, int D, void* workspace, int64_t workspace_bytes, void* stream);

/* sla_linear_state_fwd and sage_quant_v (further down) in one call, for the quantised module, which needs both of the
 * same v: the state kernel streams v anyway and leaves the largest |v| of every column, so the quantiser's own pass over
 * v for them is not made.  workspace (SLA_WS_LINEAR_FWD), v_fp8, v_scale, v_range as in the two calls; the results equal
 * theirs bit for bit.  Kernels on `stream` in the order: states per slice of the sequence, scale, FP8 copy of v, sum of
 * the slices, projection folded in.
 * Replaces core.py:90-95 of sparse_linear_attention (feature map of k, calc_linear's k^T v and k sum) and
 * SageSLA/core.py:127-129 (per-channel FP8 quantisation of v). */
int sla_linear_state_quant_v_fwd(const void* k, const void* v, const float* weight, int dtype, int fmap, int B, int H,
                                 int L, int D, void* workspace, int64_t workspace_bytes, uint8_t* v_fp8, float* v_scale,
                                 float v_range, void* stream);

/* For callers whose activations are not laid out as contiguous (B, H, L, D): strided variants of the calls that
 * touch q, k, v, out and their gradients.  `*_strides` = {batch, head, row} strides in
 * elements of a tensor indexed (b, h, l, d) whose last dimension is contiguous: {H*L*D, L*D, D} for the
 * contiguous layout, {L*H*D, D, H*D} for a (B, L, H, D) activation, {L*3*H*D, D, 3*H*D} for the q / k / v
 * slices of a packed (B, L, 3, H, D) projection.  All strides must be multiples of 8 elements (4 for fp32
 * inputs of the mask builder) and one head must span less than 4 GiB.  Everything else as in the calls without
 * the suffix (workspaces, lut, lse and o_s keep their contiguous shapes).
 * They replace the layout copies either side of the operator in a transformer block
 * (evaluate/bench_kernel.py:68-71 of the reference: transpose(1, 2).contiguous() of q, k, v and of the output). */
int sla_block_map_fwd_strided(const void* q, const void* k, const int64_t* qk_strides, int dtype, int B, int H, int L,
                              int D, int BLKQ, int BLKK, int topk, void* workspace, int64_t workspace_bytes,
                              int8_t* sparse_map, void* lut, int lut_elem_bytes, void* stream);
int sla_linear_state_fwd_strided(const void* k, const void* v, const int64_t* kv_strides, const float* weight, int dtype,
                                 int fmap, int B, int H, int L, int D, void* workspace, int64_t workspace_bytes,
                                 void* stream);
int sla_linear_state_quant_v_fwd_strided(const void* k, const void* v, const int64_t* kv_strides, const float* weight,
                                         int dtype, int fmap, int B, int H, int L, int D, void* workspace,
                                         int64_t workspace_bytes, uint8_t* v_fp8, float* v_scale, float v_range,
                                         void* stream);
/* The two backward calls with strides: q, k, v, dq, dk, dv share `qkv_strides` (e.g. slices of one packed
 * (B, L, 3, H, D) buffer and of its gradient), d_o / d_out has `do_strides`; o (the saved o_s), lse and the
 * workspaces are contiguous as in the calls without the suffix. */
int sla_sparse_attn_bwd_strided(const void* q, const void* k, const void* v, const int64_t* qkv_strides, const void* o,
                                const void* d_o, const int64_t* do_strides, const float* lse, const int8_t* sparse_map,
                                const void* lut, int lut_elem_bytes, void* dq, void* dk, void* dv, int dtype, int B, int H,
                                int L, int D, int BLKQ, int BLKK, int topk, float qk_scale, void* workspace,
                                int64_t workspace_bytes, void* stream);
int sla_linear_bwd_strided(const void* q, const void* k, const void* v, const int64_t* qkv_strides, const float* weight,
                           const float* bias, const void* d_out, const int64_t* do_strides, void* dq, void* dk, void* dv,
                           float* d_weight, float* d_bias, int dtype, int fmap, int B, int H, int L, int D, int flags,
                           void* workspace, int64_t workspace_bytes, void* stream);
int sla_sparse_attn_linear_fwd_strided(const void* q, const void* k, const void* v, const int64_t* qkv_strides,
                                       const void* lut, int lut_elem_bytes, const void* linear_workspace,
                                       int64_t linear_workspace_bytes, const float* bias, void* o_s, void* out,
                                       const int64_t* out_strides, float* lse, int dtype, int fmap, int B, int H, int L,
                                       int D, int BLKQ, int BLKK, int topk, float qk_scale, void* stream);

/* Backward of the whole module in one call: the kernels of sla_sparse_attn_bwd(_strided) followed by those of
 * sla_linear_bwd(_strided) with SLA_BWD_ACCUMULATE (the linear branch adds into dq, dk, dv), results equal to those two
 * calls bit for bit.  The only flag is SLA_BWD_STATES_READY.  qkv_strides / do_strides: both NULL for contiguous
 * (B, H, L, D) tensors, else as in the strided calls.  o_s is the attention output the forward saved.  The two workspaces
 * are those of the two calls (SLA_WS_SPARSE_BWD, SLA_WS_LINEAR_BWD).
 * side_stream (may be NULL or equal to stream: then everything runs on `stream`) takes the short kernels - the
 * per-key-block lists of the map, and the per-head reductions and small products of the linear branch - so that they run
 * beside the long dQ and dK/dV kernels instead of between them; `stream` waits for all of it before the call's last
 * kernel, so later work needs ordering against `stream` only.  The streams must belong to the current device and have the
 * same (default) priority.  The first call with a second stream on a device creates four events (no device memory), kept
 * for later calls; calls from several host threads take turns enqueueing.
 * Replaces autograd through SparseLinearAttention.forward, sparse_linear_attention/core.py:88-100 with
 * kernel.py:277-320. */
int sla_module_bwd(const void* q, const void* k, const void* v, const int64_t* qkv_strides, const void* o_s,
                   const void* d_out, const int64_t* do_strides, const float* lse, const int8_t* sparse_map, const void* lut,
                   int lut_elem_bytes, const float* weight, const float* bias, void* dq, void* dk, void* dv, float* d_weight,
                   float* d_bias, int dtype, int fmap, int B, int H, int L, int D, int BLKQ, int BLKK, int topk,
                   float qk_scale, int flags, void* sparse_workspace, int64_t sparse_workspace_bytes, void* linear_workspace,
                   int64_t linear_workspace_bytes, void* stream, void* side_stream);

/* Linear branch in "complement" mode (opt-in): query block i attends linearly only to the key
 * blocks (of 64 rows) that its look-up row did NOT select; projection, bias and residual as in
 * sla_linear_fwd.  out = residual + proj(o_l).  lut as produced by sla_block_map_fwd; BLKK must be 64.
 * The mounted reference has no code for this variant (its README.md:8 names it; core.py:92-96 computes
 * the global one): the definition is the brute-force one stated in the oracle. */
int sla_linear_complement_fwd(const void* q, const void* k, const void* v, const void* lut, int lut_elem_bytes,
                              const float* weight, const float* bias, const void* residual, void* out, int dtype,
                              int fmap, int B, int H, int L, int D, int BLKQ, int BLKK, int topk, void* workspace,
                              int64_t workspace_bytes, void* stream);

/* Backward of sla_linear_complement_fwd: gradients of the complement-mode linear branch only (the residual's
 * gradient is d_out itself).  sparse_map and lut as produced by sla_block_map_fwd for the same q, k (the map
 * gives the per-key-block lists of selecting query blocks).  dq, dk, dv in `dtype`, d_weight (D,D) and d_bias (D)
 * fp32; flags: SLA_BWD_ACCUMULATE as in sla_linear_bwd.  Workspace: SLA_WS_LINEAR_COMPLEMENT_BWD.
 * No counterpart in the mounted reference (see sla_linear_complement_fwd); checked against autograd through
 * the oracle's definition. */
int sla_linear_complement_bwd(const void* q, const void* k, const void* v, const int8_t* sparse_map, const void* lut,
                              int lut_elem_bytes, const float* weight, const float* bias, const void* d_out, void* dq,
                              void* dk, void* dv, float* d_weight, float* d_bias, int dtype, int fmap, int B, int H,
                              int L, int D, int BLKQ, int BLKK, int topk, int flags, void* workspace,
                              int64_t workspace_bytes, void* stream);

/* Linear branch backward.  d_out is the gradient of `out` above.  Writes dq, dk, dv in `dtype`
 * (gradients of the linear branch only; the residual's gradient is d_out itself) and the
 * fp32 gradients of weight (D,D) and bias (D).  flags: with SLA_BWD_ACCUMULATE, dq/dk/dv already hold
 * the gradients of the sparse branch and the linear ones, rounded to `dtype`, are added to them
 * as a tensor addition in `dtype` would (the sum is formed in fp32 and rounded once more).
 * The backward needs the per-head states of the forward again; it rebuilds them from k and v unless
 * SLA_BWD_STATES_READY says that the caller has copied the first sla_workspace_bytes(SLA_WS_LINEAR_STATES, ..)
 * bytes of the forward's workspace (after sla_linear_state_fwd / sla_linear_fwd with the same k, v, weight)
 * to the start of this workspace.
 * Replaces torch autograd through sparse_linear_attention/core.py:90-99. */
int sla_linear_bwd(const void* q, const void* k, const void* v, const float* weight, const float* bias,
                   const void* d_out, void* dq, void* dk, void* dv, float* d_weight, float* d_bias,
                   int dtype, int fmap, int B, int H, int L, int D, int flags, void* workspace,
                   int64_t workspace_bytes, void* stream);

/* SageSLA: per-block INT8 quantisation of q (BLKQ rows) and of k - mean_L(k) (BLKK rows).
 * q_int8, k_int8 (B,H,L,D) int8; q_scale (B,H,M) fp32; k_scale (B,H,N) fp32.
 * Replaces k.mean + spas_sage_attn.utils.get_vanilla_qk_quant, SageSLA/core.py:102-108. */
int sage_quant_qk(const void* q, const void* k, int dtype, int B, int H, int L, int D, int BLKQ, int BLKK,
                  int8_t* q_int8, float* q_scale, int8_t* k_int8, float* k_scale, void* workspace,
                  int64_t workspace_bytes, void* stream);

/* SageSLA: per-channel FP8 e4m3 quantisation of v.  v_fp8 (B,H,L,D) e4m3fn bytes,
 * v_scale (B,H,D) fp32 = max_L|v| / v_range, v_fp8 = e4m3fn(v / v_scale), so |v_fp8| <= v_range.
 * v_range in (0, 448]: the reference's call passes 2.25 (SageSLA/core.py:129, sized for fp16 accumulators of the
 * PV product); this library's modules pass 448, the whole e4m3 range, because sage_sparse_attn_fwd accumulates
 * in fp32.  sage_sparse_attn_fwd takes either: it only multiplies by v_scale at the end.
 * Replaces spas_sage_attn._fused.transpose_pad_permute_cuda + scale_fuse_quant_cuda,
 * SageSLA/core.py:123-129. */
int sage_quant_v(const void* v, int dtype, int B, int H, int L, int D, uint8_t* v_fp8, float* v_scale, float v_range,
                 void* workspace, int64_t workspace_bytes, void* stream);

/* SageSLA: everything the quantised attention kernel needs, in one call: the block map of
 * sla_block_map_fwd (BLKQ 128, BLKK 64), the INT8 q / k of sage_quant_qk and the FP8 v of sage_quant_v,
 * with outputs identical to those three calls on the same q, k, v (which must already be in the compute
 * dtype).  The column mean of k is formed once and the quantisers emit the block means the scores are
 * made of, so q is read once and k twice.
 * Replaces get_block_map + k.mean + get_vanilla_qk_quant + the v quantisation, SageSLA/core.py:96-129. */
int sage_prepare(const void* q, const void* k, const void* v, int dtype, int B, int H, int L, int D, int BLKQ,
                 int BLKK, int topk, int8_t* sparse_map, void* lut, int lut_elem_bytes, int8_t* q_int8, float* q_scale,
                 int8_t* k_int8, float* k_scale, uint8_t* v_fp8, float* v_scale, float v_range, void* workspace,
                 int64_t workspace_bytes, void* stream);

/* SageSLA: quantised block-sparse attention, INT8 QK^T and FP8 PV on the matrix cores.
 * Replaces spas_sage_attn.utils.block_map_lut_triton + _qattn.qk_int8_sv_f8_*,
 * SageSLA/core.py:109, 136-144. */
int sage_sparse_attn_fwd(const int8_t* q_int8, const float* q_scale, const int8_t* k_int8,
                         const float* k_scale, const uint8_t* v_fp8, const float* v_scale, const void* lut,
                         int lut_elem_bytes, void* o, int out_dtype, int B, int H, int L, int D, int BLKQ,
                         int BLKK, int topk, float qk_scale, void* stream);

/* The SageSLA path on row-contiguous views (same stride convention as the other *_strided entry points):
 * q, k, v may be (B, L, H, D) activations or slices of a packed projection; the quantised tensors are always written
 * as contiguous (B, H, L, D), which is what sage_sparse_attn_fwd reads; sla_linear_out_fwd_strided reads q and
 * writes out where the caller's tensors lie (the residual, i.e. the attention output, is contiguous (B, H, L, D)).
 * They spare the caller the layout copies of bench_kernel.py:68-71 around the quantised operator. */
int sage_prepare_strided(const void* q, const void* k, const void* v, const int64_t* qkv_strides, int dtype, int B, int H,
                         int L, int D, int BLKQ, int BLKK, int topk, int8_t* sparse_map, void* lut, int lut_elem_bytes,
                         int8_t* q_int8, float* q_scale, int8_t* k_int8, float* k_scale, uint8_t* v_fp8, float* v_scale,
                         float v_range, void* workspace, int64_t workspace_bytes, void* stream);
int sage_quant_v_strided(const void* v, const int64_t* v_strides, int dtype, int B, int H, int L, int D, uint8_t* v_fp8,
                         float* v_scale, float v_range, void* workspace, int64_t workspace_bytes, void* stream);
int sla_linear_out_fwd_strided(const void* q, const int64_t* q_strides, const float* bias, const void* residual, void* out,
                               const int64_t* out_strides, int dtype, int fmap, int B, int H, int L, int D,
                               void* workspace, int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SLA_HIP_H */
