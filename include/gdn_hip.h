/*
 * gdn_hip.h - C ABI of libgdn_hip.so: the gated delta rule (Gated DeltaNet)
 * inference path as hand-written HIP kernels for gfx950 (MI355X).
 *
 * The reference (fla-org/flash-linear-attention) is Python + Triton and has no
 * FFI of its own; its boundary for this path is two Python functions.  Each
 * entry point below is what a binding for one of them calls, and cites the
 * reference interface it replaces.  All pointers are DEVICE pointers unless
 * stated otherwise; all tensors are contiguous, token-major, exactly as the
 * reference's `input_guard` hands them to its kernels
 * (fla/utils/_decorators.py:99-165).  Calls only enqueue work on `stream`
 * (a hipStream_t passed as void*, NULL = the null stream); they never
 * synchronise.  Return value: 0 on success, negative GDN_ERR_* otherwise;
 * gdn_last_error() then returns a message for the calling thread.
 */
#ifndef GDN_HIP_H
#define GDN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GDN_OK                 0
#define GDN_ERR_INVALID       -1   /* bad argument (Python shim raises ValueError)            */
#define GDN_ERR_UNSUPPORTED   -2   /* shape/dtype outside the kernels (NotImplementedError)   */
#define GDN_ERR_LAUNCH        -3   /* HIP runtime error at launch (RuntimeError)              */
#define GDN_ERR_WORKSPACE     -4   /* workspace too small                                     */

/* element types of q/k/v/o and of g/beta */
#define GDN_DTYPE_BF16 0
#define GDN_DTYPE_F16  1
#define GDN_DTYPE_F32  2

/* flag bits (the reference's keyword switches) */
#define GDN_FLAG_QK_L2NORM      (1u << 0)  /* use_qk_l2norm_in_kernel                           */
#define GDN_FLAG_BETA_SIGMOID   (1u << 1)  /* use_beta_sigmoid_in_kernel                        */
#define GDN_FLAG_NEG_EIGVAL     (1u << 2)  /* allow_neg_eigval (beta = 2*sigmoid)               */
#define GDN_FLAG_STATE_V_FIRST  (1u << 3)  /* state_v_first: states are [N,HV,V,K]              */
#define GDN_FLAG_BETA_VECTOR    (1u << 4)  /* beta is [B,T,HV,V] instead of [B,T,HV]            */
#define GDN_FLAG_CU_INT32       (1u << 5)  /* cu_seqlens / chunk tables are int32, else int64   */
#define GDN_FLAG_SLOT_INT32     (1u << 6)  /* state_slots / num_accepted are int32, else int64  */
#define GDN_FLAG_SLOT_PER_TOKEN (1u << 7)  /* state_slots is [N, slots_stride]: a slot per token */
#define GDN_FLAG_STATE_PER_TOKEN (1u << 8) /* ht is [tokens,HV,K,V]: the state after every token */
#define GDN_FLAG_STATE_BF16     (1u << 9)  /* h0 and ht hold bf16 states (decode at half the state traffic)  */
/* gdn_chunk_fwd only: force one form of the sequential stage instead of the automatic choice
 * (all forms give the same result up to rounding; used by tests and for tuning)                */
#define GDN_FLAG_SCAN_WIDE      (1u << 17) /* one workgroup per (sequence, head)                */
#define GDN_FLAG_SCAN_SEGMENTS  (1u << 18) /* time cut into segments (dense input, >= 8 chunks) */
#define GDN_FLAG_SEQ_ORDER      (1u << 19) /* chunk_offsets carries N more entries (see there)   */
#define GDN_FLAG_SCAN_NO_PAIR   (1u << 20) /* always one run per workgroup                      */
#define GDN_FLAG_SCAN_PAIR      (1u << 21) /* two runs per workgroup wherever two can share k rows */
#define GDN_FLAG_SCAN_NO_WARM   (1u << 22) /* time segments always start from exact states (first pass + merge) */
#define GDN_FLAG_RECORD_P       (1u << 23) /* the chunk-parallel stage also leaves P in its records (the scan forms P itself and never reads it) */

/* activation codes of the convolution and normalisation entry points */
#define GDN_ACT_NONE    0
#define GDN_ACT_SILU    1   /* swish / silu: x * sigmoid(x)                                  */
#define GDN_ACT_SIGMOID 2   /* gate of the normalisation only                                */

/* Library ABI version (bumped on any signature change). */
int gdn_hip_abi_version(void);

/* Message describing the last error raised on the calling thread ("" if none). */
const char* gdn_last_error(void);

/*
 * Token recurrence, used for decode and short prompts.
 * Replaces fused_recurrent_gated_delta_rule_fwd
 * (fla/ops/gated_delta_rule/fused_recurrent.py:184-250, kernel :30-181).
 *
 *   q, k   [B,T,H,K]   qkv_dtype          v, o  [B,T,HV,V]  qkv_dtype
 *   g      [B,T,HV]    gb_dtype or NULL   beta  [B,T,HV] (or [B,T,HV,V] with GDN_FLAG_BETA_VECTOR), gb_dtype, or NULL (=1)
 *   gk     [B,T,HV,K]  fp32 or NULL       gv    [B,T,HV,V]  fp32 or NULL
 *   A_log, dt_bias [HV] fp32 or NULL: when A_log != NULL, g is raw and the gate
 *          g = -exp(A_log)*softplus(g + dt_bias) is applied per step (use_gate_in_kernel)
 *   h0     [N,HV,K,V] fp32 or NULL (zero state)
 *   ht     [N,HV,K,V] fp32 or NULL (final state not stored); ht MAY alias h0 (in-place update)
 *   cu_seqlens [N+1] or NULL; when given B must be 1 and T is the packed length
 *   state_slots [N] or NULL: sequence n then keeps its state in slot state_slots[n] of a pool, i.e. h0 and ht
 *          are [num_slots,HV,K,V] and are addressed through the slot instead of n (continuous batching; the
 *          sibling KDA operator's ssm_state_indices, fla/ops/kda/fused_recurrent.py:27,75-91,145-159).  Slots
 *          must be distinct; other slots are not touched.
 *          With GDN_FLAG_SLOT_PER_TOKEN (speculative decoding, fla/ops/kda/fused_recurrent.py:131-145,203-219)
 *          state_slots is [N][slots_stride] (slots_stride >= tokens of the longest sequence): sequence n starts
 *          from slot state_slots[n][num_accepted[n]-1] (num_accepted [N], same integer type as state_slots; NULL:
 *          entry 0) and the state after its token t is written to slot state_slots[n][t] of ht.
 *   GDN_FLAG_STATE_PER_TOKEN: ht is [B*T,HV,K,V] and receives the state after every token (the reference's
 *          continuous-batching form without inplace_final_state, fused_recurrent.py:212-213); h0 as usual.
 *   GDN_FLAG_STATE_BF16 (no counterpart in the GDN reference, whose states are fp32): h0 and ht point at bf16 states
 *          [N or slots,HV,128,128], K-first; the recurrence runs in fp32 registers and the state is rounded once, when
 *          it is written back.  Needs h0, K = V = 128, no gk / gv / beta per column, states per sequence or per slot.
 *   N = B when cu_seqlens == NULL.  Requires K <= 256, K % 4 == 0, V % 4 == 0, HV % H == 0.
 *   T == 0: ht = h0 (zeros without h0).
 */
int gdn_fused_recurrent_fwd(
    const void* q, const void* k, const void* v,
    const void* g, const void* beta, const float* gk, const float* gv,
    const float* A_log, const float* dt_bias,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* state_slots, const void* num_accepted, int64_t slots_stride,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V, int64_t N,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * Replaces fla/ops/delta_rule/fused_recurrent.py:313-385 (fused_recurrent_delta_rule_bwd and its kernel :111-266): the
 * backward of the token recurrence of the delta rule without gates,
 *   u_t = v_t - S^T k_t;  S <- S + k_t (beta_t u_t)^T;  o_t = scale S^T q_t.
 *   q, k [B,T,H,K], v, dout [B,T,H,V] in qkv_dtype (bf16, f16 or f32); beta [B,T,H] (NULL = ones) or, with
 *   GDN_FLAG_BETA_VECTOR, [B,T,H,V], in gb_dtype; h0, dht [N,H,K,V] fp32 or NULL; cu_seqlens as in the forward.
 *   Outputs, all fp32: dq_part, dk_part [NVB,B,T,H,K] (partial over the NVB = V / gdn_fused_recurrent_delta_bwd_value_block(K)
 *   blocks of value columns: the caller adds them, as the reference does, :375-378), dv [B,T,H,V], db [NVB,B,T,H] (with
 *   GDN_FLAG_BETA_VECTOR [B,T,H,V]), dh0 [N,H,K,V] or NULL.  u_workspace [B,T,H,V] fp32 receives the residuals u_t (the
 *   reference keeps them from its forward kernel, :292-295; here the backward forms them again).
 *   K a multiple of 16 up to 256, V a multiple of the value block (32 for K <= 128, else 16); every tensor 16-byte aligned.
 *   Tokens outside every sequence (packed input) are not written.
 */
int64_t gdn_fused_recurrent_delta_bwd_value_block(int64_t K);
int gdn_fused_recurrent_delta_bwd(
    const void* q, const void* k, const void* v, const void* beta, const void* dout, const float* h0, const float* dht,
    float* dq_part, float* dk_part, float* dv, float* db, float* dh0, float* u_workspace, const void* cu_seqlens,
    int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N, float scale, int qkv_dtype, int gb_dtype, uint32_t flags,
    void* stream);

/*
 * Replaces fla/ops/kda/fused_recurrent.py:236-338 (fused_recurrent_kda_fwd and its kernel :37-233): the token recurrence of
 * the KDA operator, i.e. the gated delta rule with a decay per key feature,
 *   S <- diag(e^{g_t}) S;  d = beta_t (v_t - S^T k_t);  S <- S + k_t d^T;  o_t = scale S^T q_t.
 *   g [B,T,HV,K] fp32.  gate_mode 0: g is the log decay.  gate_mode 1 (use_gate_in_kernel, :168-181): the log decay is
 *   -exp(A_log[hv]) softplus(g + dt_bias[hv][k]); gate_mode 2 (with a lower bound): lower_bound sigmoid(exp(A_log[hv]) (g + dt_bias[hv][k])).
 *   A_log [HV] fp32 or NULL (mode 1: exp(1) then, as the reference's kernel; mode 2: factor 1), dt_bias [HV,K] fp32 or NULL.
 *   Everything else (beta per head or per value column, the flags for the l2 norm of q and k, the beta sigmoid, the V-first
 *   state layout, packed sequences, state pools with a slot per sequence or per token, states per token) as in
 *   gdn_fused_recurrent_fwd, on the same kernel; GDN_FLAG_STATE_BF16 is refused.
 */
int gdn_fused_recurrent_kda_fwd(
    const void* q, const void* k, const void* v,
    const float* g, const void* beta,
    const float* A_log, const float* dt_bias, float lower_bound, int gate_mode,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* state_slots, const void* num_accepted, int64_t slots_stride,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V, int64_t N,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * Replaces fla/ops/comba/fused_recurrent.py:123-170 (fused_recurrent_comba_fwd and its kernel :37-120): the token recurrence
 * of the comba operator in fp32,
 *   d = beta_t (v_t - S^T p_t);  S <- e^{g_t} S + k_t d^T;  o_t = scale S^T q_t
 * (the prediction uses the second key p and the state before the token's decay).
 *   q, k, p [B,T,H,K], v, o [B,T,HV,V] (qkv_dtype: bf16, f16 or f32), g [B,T,HV] (log decay), beta [B,T,HV] or, with
 *   GDN_FLAG_BETA_VECTOR, [B,T,HV,V] (gb_dtype; NULL: ones), h0, ht [N,HV,K,V] fp32 or NULL, cu_seqlens [N+1] or NULL.
 *   flags: GDN_FLAG_QK_L2NORM (q, k and p are normalised, :90-93), GDN_FLAG_BETA_VECTOR, GDN_FLAG_CU_INT32.
 *   K <= 256, K and V multiples of 4.  On the kernel of gdn_fused_recurrent_fwd.
 */
int gdn_fused_recurrent_comba_fwd(
    const void* q, const void* k, const void* p, const void* v,
    const void* g, const void* beta,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V, int64_t N,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * Bytes of device workspace gdn_chunk_fwd needs for the same N, T, num_chunks (64-token chunks; dense:
 * B*ceil(T/64); packed: sum over sequences of ceil(len/64)), head counts, packed (cu_seqlens given) and flags
 * (the scan flags change the plan and with it the size).  Returns 0 for unsupported (K,V).
 */
size_t gdn_chunk_workspace_bytes(int64_t N, int64_t T, int64_t num_chunks, int64_t H, int64_t HV, int64_t K, int64_t V,
                                 int packed, uint32_t flags);

/*
 * Chunked prefill, chunk size 64.  Replaces chunk_gated_delta_rule_fwd
 * (fla/ops/gated_delta_rule/chunk.py:33-123), i.e. the five launches
 * chunk_local_cumsum (fla/ops/utils/cumsum.py:243-277),
 * chunk_gated_delta_rule_fwd_intra (fla/ops/gated_delta_rule/chunk_fwd.py:332-428),
 * recompute_w_u_fwd (fla/ops/gated_delta_rule/wy_fast.py:255-294),
 * chunk_gated_delta_rule_fwd_h (fla/ops/common/chunk_delta_h.py:687-743) and
 * chunk_fwd_o (fla/ops/common/chunk_o.py:544-586).
 *
 *   q, k [B,T,H,K], v, o [B,T,HV,V] qkv_dtype (bf16 or f16); g, beta [B,T,HV] gb_dtype
 *   g == NULL: no decay, i.e. the delta rule without gates (chunk_delta_rule_fwd, fla/ops/delta_rule/chunk.py:25-70)
 *   A_log [HV] fp32 or NULL: with it, g holds raw gate inputs and the kernel forms
 *         g = -exp(A_log) * softplus(g + dt_bias) (dt_bias [HV] fp32 or NULL) - use_gate_in_kernel,
 *         gdn_gate_chunk_cumsum of fla/ops/gated_delta_rule/gate.py:63-106
 *   flags: GDN_FLAG_QK_L2NORM (q, k rows divided by sqrt(sum x^2 + 1e-6): l2norm_fwd of
 *         fla/modules/l2norm.py:84-109, applied as per-row factors, q and k are read as given),
 *         GDN_FLAG_BETA_SIGMOID / GDN_FLAG_NEG_EIGVAL (beta = [2*]sigmoid(beta):
 *         fla/ops/common/gate.py:19-31), GDN_FLAG_STATE_V_FIRST, GDN_FLAG_CU_INT32, the scan flags
 *   h0 [N,HV,K,V] fp32 or NULL; ht [N,HV,K,V] fp32 or NULL
 *   cu_seqlens [N+1] (device) or NULL
 *   chunk_table [num_chunks][2] (device; sequence id, chunk id inside the sequence) -
 *         prepare_chunk_indices of fla/ops/utils/index.py:156-164; NULL for dense input
 *   chunk_offsets [N+1] (device; exclusive prefix sum of chunks per sequence) -
 *         prepare_chunk_offsets of fla/ops/utils/index.py:167-172; NULL for dense input.
 *         With GDN_FLAG_SEQ_ORDER the array has N more entries: the sequence ids in the order in
 *         which the sequential kernel should start them (longest first keeps the CUs evenly loaded)
 *   workspace: at least gdn_chunk_workspace_bytes(...) bytes, 256-byte aligned
 *   T == 0 (or no chunk at all): ht = h0 (zeros without h0), nothing else is written.
 *   Requires HV % H == 0 and K, V multiples of 8: both up to 128, or 128 < K <= 256 (the reference's limit,
 *   fla/ops/common/chunk_delta_h.py:712) with V up to 8192.  State shapes of the kernels: 128 x 128 (key features
 *   past K count as zero, value columns past V are not stored), 64 x 64 for K, V <= 64, and 256 x 64-column blocks
 *   for wide keys; the Python host zero-pads head dims that are not multiples of 8 and splits V > 128 with K <= 128
 *   into value heads of 128 columns.
 */
int gdn_chunk_fwd(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* A_log, const float* dt_bias,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * The two stages of gdn_chunk_fwd as separate calls with the same argument list, so that a
 * caller can time or overlap them.  gdn_chunk_fwd(...) == gdn_chunk_fwd_prepare(...) followed
 * by gdn_chunk_fwd_scan(...) on the same stream and workspace.
 *   prepare: the chunk-parallel part - chunk_local_cumsum, chunk_gated_delta_rule_fwd_intra
 *            (gated beta*K*K^T, its unit-lower inverse, w, u) and the intra-chunk q*k^T of
 *            chunk_fwd_o (fla/ops/common/chunk_o.py:107-139); fills the workspace.
 *   scan:    chunk_gated_delta_rule_fwd_h fused with the rest of chunk_fwd_o; reads the
 *            workspace, writes o and ht.
 */
int gdn_chunk_fwd_prepare(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* A_log, const float* dt_bias,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);
int gdn_chunk_fwd_scan(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* A_log, const float* dt_bias,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * Backward pass of the chunked operator.  Replaces chunk_gated_delta_rule_bwd (fla/ops/gated_delta_rule/chunk.py:125-257):
 * recompute_w_u_fwd (fla/ops/gated_delta_rule/wy_fast.py:236-296), chunk_gated_delta_rule_fwd_h and
 * chunk_gated_delta_rule_bwd_dhu (fla/ops/common/chunk_delta_h.py:563-744, 747-828), chunk_bwd_dv_local and
 * chunk_bwd_dqkwg (fla/ops/common/chunk_o.py:647-697, 700-779), prepare_wy_repr_bwd (wy_fast.py:298-351) and the
 * reverse chunk_local_cumsum of dg (fla/ops/utils/cumsum.py).  Nothing is kept from the forward call: A, w, u, the
 * per-chunk states and v_new are computed again, into the workspace.
 *   q, k [B,T,H,K]; v, dout [B,T,HV,V] (qkv_dtype: bf16 or f16); g (log decay, may be NULL), beta [B,T,HV] (gb_dtype),
 *   both as the recurrence uses them: the activations of the forward call (l2 norm, gate, sigmoid) and their
 *   derivatives are the caller's, as in the reference (chunk.py:278-288, 385-393)
 *   h0, dht [N,HV,K,V] fp32 or NULL
 *   dq, dk [B,T,HV,K], dv [B,T,HV,V] in qkv_dtype: per VALUE head; with grouped heads the caller adds the HV/H
 *   gradients that belong to one q/k head; dg, dbeta [B,T,HV] fp32; dh0 [N,HV,K,V] fp32 or NULL
 *   cu_seqlens, chunk_table, chunk_offsets ([N+1] here), N, num_chunks: as for gdn_chunk_fwd
 *   workspace: at least gdn_chunk_bwd_workspace_bytes(num_chunks, HV, K) bytes (0: unsupported K), 256-byte aligned
 *   flags: GDN_FLAG_CU_INT32 only.  K = 128 or 256 (the reference's limit, fla/ops/common/chunk_delta_h.py:712) and V = 128 only: the Python host
 *   zero-pads other head dims and splits V > 128 into value heads of 128 columns.
 *   T == 0: dh0 = dht (zeros without dht), nothing else is written.
 */
size_t gdn_chunk_bwd_workspace_bytes(int64_t num_chunks, int64_t HV, int64_t K);
int gdn_chunk_bwd(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * gdn_chunk_bwd with the l2 normalisation of q and k taken inside (use_qk_l2norm_in_kernel): q and k are the rows as the
 * caller has them, dq and dk the gradients of THOSE rows.  Replaces l2norm_fwd (twice), chunk_gated_delta_rule_bwd and
 * l2norm_bwd (twice) of ChunkGatedDeltaRuleFunction.backward (fla/ops/gated_delta_rule/chunk.py:278-282, 385-393;
 * fla/modules/l2norm.py:222-298): the first kernel divides the rows by sqrt(sum x^2 + 1e-6) on their way in and leaves
 * them, with the factors, in the workspace for the kernels that follow; the kernels that produce dq and dk apply
 * dx = (dy - y (y . dy)) rstd per row to their fp32 results before they write them.
 * Arguments as for gdn_chunk_bwd, except:
 *   workspace: at least gdn_chunk_bwd_qk_l2norm_workspace_bytes(num_chunks, HV, K, B * T) bytes (0: unsupported K)
 *   H == HV and K = 128 only (GDN_ERR_UNSUPPORTED otherwise: call gdn_l2norm_fwd, gdn_chunk_bwd, then gdn_l2norm_bwd,
 *   which also adds up the value heads of a q/k head).
 */
size_t gdn_chunk_bwd_qk_l2norm_workspace_bytes(int64_t num_chunks, int64_t HV, int64_t K, int64_t tokens);
int gdn_chunk_bwd_qk_l2norm(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * Backward pass of the chunked comba operator.  Replaces chunk_comba_bwd (fla/ops/comba/chunk.py:92-178): the
 * gated delta rule's backward with the comba forms of recompute_w_u_fwd and prepare_wy_repr_bwd
 * (fla/ops/comba/wy_fast.py), which form A and w from the second key p and the decay in front of each token
 * (g0 = cumsum(g) - g, fla/ops/comba/utils.py), and the two reverse cumulative sums of dg (chunk.py:163-177).
 * Arguments as for gdn_chunk_bwd, and:
 *   p [B,T,H,K] in qkv_dtype: the key the prediction is made with, as the recurrence uses it (after its l2 norm, if any)
 *   dp [B,T,HV,K] in qkv_dtype, per value head like dq and dk
 *   g must not be NULL; K = 128 only (smaller head dims zero-padded by the caller), V = 128
 *   workspace: gdn_chunk_bwd_workspace_bytes(num_chunks, HV, 128)
 */
int gdn_chunk_comba_bwd(
    const void* q, const void* k, const void* p, const void* v, const void* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dp, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * gdn_chunk_comba_bwd with the l2 normalisation of q, k and p taken inside, as gdn_chunk_bwd_qk_l2norm does it for q and k:
 * q, k, p are the rows as the caller has them, dq, dk, dp the gradients of those rows.  Replaces the three l2norm_fwd and
 * three l2norm_bwd launches around chunk_comba_bwd in ChunkCombaFunction.backward (fla/ops/comba/chunk.py:277-280).
 * Arguments as for gdn_chunk_comba_bwd, except:
 *   workspace: at least gdn_chunk_comba_bwd_qk_l2norm_workspace_bytes(num_chunks, HV, B * T) bytes
 *   H == HV only (GDN_ERR_UNSUPPORTED otherwise).
 */
size_t gdn_chunk_comba_bwd_qk_l2norm_workspace_bytes(int64_t num_chunks, int64_t HV, int64_t tokens);
int gdn_chunk_comba_bwd_qk_l2norm(
    const void* q, const void* k, const void* p, const void* v, const void* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dp, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * Backward pass of the chunked KDA operator.  Replaces chunk_kda_bwd (fla/ops/kda/chunk_bwd.py, called from
 * ChunkKDAFunction.backward, fla/ops/kda/chunk.py:124-175): the forward's intermediates are computed again (the
 * chunk-parallel kernel of gdn_chunk_kda_fwd, then the state scan), then the reverse scan, dq / dk / dw and the way back
 * through w, u and the two matrices with a decay per pair of rows and key feature (the reference's
 * chunk_kda_bwd_intra / chunk_kda_bwd_wy_dqkg_fused), and the reverse chunk-local cumulative sum of dg.
 * Arguments as for gdn_chunk_bwd, except:
 *   g [B,T,HV,K] fp32: the log decay per key feature as the recurrence uses it (after the gate activation, whose
 *   derivative is the caller's, like those of the l2 norm and of the beta sigmoid); must not be NULL
 *   dg [B,T,HV,K] fp32
 *   K = V = 128 only (smaller head dims zero-padded by the caller; V > 128 as value heads of 128 columns)
 *   workspace: gdn_chunk_kda_bwd_workspace_bytes(num_chunks, HV)
 */
size_t gdn_chunk_kda_bwd_workspace_bytes(int64_t num_chunks, int64_t HV);
int gdn_chunk_kda_bwd(
    const void* q, const void* k, const void* v, const float* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * Row-wise l2 normalisation around gdn_chunk_bwd.  gdn_l2norm_fwd replaces l2norm_fwd (fla/modules/l2norm.py:222-262):
 * y[row] = x[row] / sqrt(sum x^2 + 1e-6) in x's dtype (bf16 or f16), rstd[row] = that factor; rows of D elements in,
 * rows of Dout >= D elements out (zeros from D on: the backward kernels want 128).  gdn_l2norm_bwd replaces l2norm_bwd
 * (fla/modules/l2norm.py:265-300) and the sum over grouped heads in front of it (chunk_gated_delta_rule_bwd returns dq, dk
 * per value head): dx[row] = (dy - y <dy, y>) rstd[row] with dy = sum over g < G of dyh[row][g]; rows of Din elements in
 * (dyh, y), the first Dout <= Din of them out; y == rstd == NULL: the sum alone.  Row lengths: multiples of 8 up to 256.
 */
int gdn_l2norm_fwd(const void* x, void* y, float* rstd, int64_t rows, int64_t D, int64_t Dout, int dtype, void* stream);
int gdn_l2norm_bwd(const void* dyh, const void* y, const float* rstd, void* dx, int64_t rows, int64_t G, int64_t Din,
                   int64_t Dout, int dtype, void* stream);

/*
 * Chunked forward of the KDA operator (a decay per key feature).  Replaces chunk_kda_fwd (fla/ops/kda/chunk_fwd.py:20-134):
 * the gate activation and chunk-local cumsum (fla/ops/kda/gate.py:27-94), chunk_kda_fwd_intra (fla/ops/kda/chunk_intra.py),
 * recompute_w_u_fwd (fla/ops/kda/wy_fast.py), chunk_gated_delta_rule_fwd_h with gk (fla/ops/common/chunk_delta_h.py:687-744) and
 * chunk_gla_fwd_o_gk (fla/ops/gla/chunk.py).
 *   q, k [B,T,H,K]; v [B,T,HV,V] (bf16 or f16); g [B,T,HV,K] fp32: log decay per key feature, or the raw gate input with
 *   gate_mode 1 (g <- -exp(A_log[hv]) softplus(g + dt_bias[hv][k])) or 2 (g <- lower_bound sigmoid(exp(A_log[hv]) (g + dt_bias[hv][k])));
 *   A_log [HV] or NULL (then exp(A_log) reads as e in mode 1 and as 1 in mode 2, as in the token recurrence), dt_bias [HV,K] or NULL
 *   beta [B,T,HV] (gb_dtype); h0, ht [N,HV,K,V] fp32 or NULL; o [B,T,HV,V] in qkv_dtype
 *   cu_seqlens, chunk_table, chunk_offsets ([N+1]), N, num_chunks: as for gdn_chunk_fwd
 *   workspace: at least gdn_chunk_kda_workspace_bytes(num_chunks, HV) bytes, 256-byte aligned
 *   flags: GDN_FLAG_CU_INT32, GDN_FLAG_QK_L2NORM, GDN_FLAG_BETA_SIGMOID, GDN_FLAG_NEG_EIGVAL.  K = V = 128 only: the Python host
 *   zero-pads smaller head dims and splits V > 128 into value heads of 128 columns.  T == 0: ht = h0 (zeros without h0).
 */
size_t gdn_chunk_kda_workspace_bytes(int64_t num_chunks, int64_t HV);
int gdn_chunk_kda_fwd(
    const void* q, const void* k, const void* v, const float* g, const void* beta,
    const float* A_log, const float* dt_bias, float lower_bound, int gate_mode,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * gdn_chunk_kda_fwd that also leaves the state in front of every chunk: what chunk_kda returns as `h` with
 * return_intermediate_states (fla/ops/kda/chunk.py:98-100, fla/ops/kda/chunk_fwd.py:130-131; the array
 * chunk_gated_delta_rule_fwd_h fills, fla/ops/common/chunk_delta_h.py:714-718).
 *   states [num_chunks, HV, K, V] in qkv_dtype (chunks in packed order: [B, NT, ...] for equal lengths), written by the scan
 */
int gdn_chunk_kda_fwd_states(
    const void* q, const void* k, const void* v, const float* g, const void* beta,
    const float* A_log, const float* dt_bias, float lower_bound, int gate_mode,
    const float* h0, float* ht, void* o, void* states,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * Chunked forward of the comba operator (one decay per token and head; the prediction uses a second key p and the state
 * before the token's decay).  Replaces chunk_comba_fwd (fla/ops/comba/chunk.py:22-90): chunk_comba_cumsum_scalar_fwd
 * (fla/ops/comba/utils.py), chunk_scaled_dot_comba_pkt_fwd and the triangular solve (fla/ops/comba/wy_fast.py), recompute_w_u_fwd,
 * chunk_gated_delta_rule_fwd_h and chunk_fwd_o; the sequential part is gdn_chunk_kda_fwd's.
 *   q, k, p [B,T,H,K]; v [B,T,HV,V] (bf16 or f16); g (natural-log decay), beta [B,T,HV] (gb_dtype);
 *   h0, ht [N,HV,K,V] fp32 or NULL; o [B,T,HV,V] in qkv_dtype; the rest as for gdn_chunk_kda_fwd, whose workspace size it shares.
 *   flags: GDN_FLAG_CU_INT32, GDN_FLAG_QK_L2NORM (normalises q, k and p, fla/ops/comba/chunk.py:202-205).  K = V = 128 only.
 */
int gdn_chunk_comba_fwd(
    const void* q, const void* k, const void* v, const void* p, const void* g, const void* beta,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * gdn_chunk_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * gdn_chunk_fwd minus the workspace: the kernels use a fixed array of GDN_CHUNK_STATIC_WORKSPACE_BYTES that the
 * library keeps in device memory (one per GPU it runs on, until the process ends).  The call allocates and frees
 * nothing.  Inputs whose workspace (gdn_chunk_workspace_bytes) exceeds the array are refused with
 * GDN_ERR_WORKSPACE; when only the plan with time segments is too large, whole sequences are scanned instead
 * (same result up to rounding).  All calls on one GPU share the array: calls that overlap on one GPU (two streams,
 * two threads) race, so serialise them.  The first call on a device looks up the array's address; make it
 * outside a graph capture.
 */
#define GDN_CHUNK_STATIC_WORKSPACE_BYTES (64u << 20)
int gdn_chunk_fwd_static(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* A_log, const float* dt_bias,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream);

/*
 * The two memory-bound steps either side of the operator in the layer
 * (fla/layers/gated_deltanet.py:246-300 and :355-359).
 *
 * Causal depthwise convolution over [token][channel] rows, prefill form.  Replaces causal_conv1d_fwd
 * (fla/modules/conv/triton/ops.py:37-96: kernel fla/modules/conv/triton/kernels.py:37-139 and, for
 * final_state, causal_conv1d_update_states, kernels.py:520-631).
 *
 *   y[t,d] = act(sum_{j<W} weight[d,j] * x[t-(W-1)+j, d] + bias[d]) + residual[t,d]
 *
 *   x        [B,T,D] x_dtype, rows stride_x_t elements apart, batches stride_x_n apart, channels adjacent
 *            (a slice of a wider projection is read in place)
 *   weight   [D,W] w_dtype; bias [D] w_dtype or NULL; residual [B,T,D] x_dtype contiguous or NULL
 *   initial_state [N,D,W] state_dtype or NULL: inputs before the start of each sequence (entry W-1 is the newest;
 *            entry 0 is never read, as in the reference)
 *   y        [B,T,D] x_dtype contiguous, or NULL (only the state is wanted: weight may then be NULL too);
 *            final_state [N,D,W] x_dtype or NULL (not stored): the last W inputs of
 *            each sequence, reaching back into initial_state (or zero) when the sequence is shorter
 *   cu_seqlens [N+1] or NULL (int64, or int32 with GDN_FLAG_CU_INT32); with it B must be 1; tokens outside
 *            [cu_seqlens[0], cu_seqlens[N]) are not written
 *   activation GDN_ACT_NONE or GDN_ACT_SILU.  Requires 1 <= W <= 8.
 */
int gdn_causal_conv1d_fwd(
    const void* x, const void* weight, const void* bias, const void* residual, const void* initial_state,
    void* y, void* final_state, const void* cu_seqlens,
    int64_t B, int64_t T, int64_t D, int64_t W, int64_t N, int64_t stride_x_n, int64_t stride_x_t,
    int x_dtype, int w_dtype, int state_dtype, int activation, uint32_t flags, void* stream);

/*
 * The same convolution for one new token per sequence (decode).  Replaces causal_conv1d_update
 * (fla/modules/conv/triton/ops.py:301-363, kernel fla/modules/conv/triton/kernels.py:356-421).
 *   x, y   N rows of D channels, rows stride_x_n / stride_y_n elements apart, x_dtype
 *   cache  [N,D,W] cache_dtype, updated IN PLACE: entries move one place towards 0 and x becomes entry W-1.
 *          NULL: the window counts as zero (x included), as in the reference kernel without a cache
 *   weight [D,W] w_dtype or NULL (taps of 1); bias [D] w_dtype or NULL; residual [N,D] x_dtype or NULL
 */
int gdn_causal_conv1d_update(
    const void* x, void* cache, const void* residual, const void* weight, const void* bias, void* y,
    int64_t N, int64_t D, int64_t W, int64_t stride_x_n, int64_t stride_y_n,
    int x_dtype, int w_dtype, int cache_dtype, int activation, void* stream);

/*
 * Layer / RMS normalisation of rows of D features with an output gate.  Replaces layer_norm_gated_fwd
 * (fla/modules/fused_norm_gate.py:456-538, kernels :36-108 and :125-189).
 *   r = x + residual ; y = (r - mean) * rstd * weight + bias ; y *= g * sigmoid(g) (GDN_ACT_SILU) or sigmoid(g)
 *   with rstd = 1/sqrt(var + eps); is_rms_norm != 0: mean = 0 and var = mean(r^2)
 *   x, g, y [T,D] x_dtype contiguous; weight, bias [D] w_dtype or NULL; residual [T,D] res_dtype or NULL;
 *   residual_out [T,D] res_out_dtype or NULL (r is not stored); mean, rstd [T] fp32 or NULL (not stored)
 *   Requires D * sizeof(element) < 64 KB.
 */
int gdn_norm_gated_fwd(
    const void* x, const void* g, const void* weight, const void* bias, const void* residual,
    void* y, void* residual_out, float* mean, float* rstd,
    int64_t T, int64_t D, float eps,
    int x_dtype, int w_dtype, int res_dtype, int res_out_dtype, int activation, int is_rms_norm, void* stream);

/*
 * Backward of gdn_causal_conv1d_fwd.  Replaces causal_conv1d_bwd (fla/modules/conv/triton/ops.py:147-249: kernel
 * fla/modules/conv/triton/kernels.py:142-353, and compute_dh0_triton, ops.py:100-144).
 *   x, weight, bias, initial_state, cu_seqlens, strides, dtypes, activation, flags: the forward's arguments (the output before
 *   the activation is recomputed from them); dy [B,T,D] x_dtype contiguous: gradient of y (the residual's gradient is dy itself);
 *   dht [N,D,W] x_dtype or NULL: gradient of final_state
 *   dx [B,T,D] x_dtype contiguous (packed input: tokens outside [cu_seqlens[0], cu_seqlens[N]) are not written)
 *   dw_part [parts,D,W], db_part [parts,D] (NULL without bias) fp32 with parts = ceil(num_tiles / GDN_CONV_BWD_TILES_PER_PART):
 *   one row of partial sums per run of that many 64-token tiles, to be added up by the caller (parts == 0: nothing is written);
 *   dh0 [N,D,W] fp32 or NULL (needs initial_state)
 *   tile_table [num_tiles,2]: (sequence, tile inside it) per 64-token tile of a packed input, in cu_seqlens' integer type
 *   (the chunk table of gdn_chunk_fwd); dense input: NULL and num_tiles = B * ceil(T / 64)
 *   Requires D and the strides of x to be multiples of 4 and rows that start on a boundary of four elements.
 */
#define GDN_CONV_BWD_TILES_PER_PART 8
int gdn_causal_conv1d_bwd(
    const void* x, const void* weight, const void* bias, const void* initial_state, const void* dy, const void* dht,
    void* dx, float* dw_part, float* db_part, float* dh0,
    const void* cu_seqlens, const void* tile_table,
    int64_t B, int64_t T, int64_t D, int64_t W, int64_t N, int64_t num_tiles, int64_t stride_x_n, int64_t stride_x_t,
    int x_dtype, int w_dtype, int state_dtype, int activation, uint32_t flags, void* stream);

/*
 * Backward of gdn_norm_gated_fwd.  Replaces layer_norm_gated_bwd (fla/modules/fused_norm_gate.py:541-650, kernels :192-453).
 *   dy, x, g, dx, dg: T rows of D features x_dtype, ld elements apart (ld >= D a multiple of 16 / sizeof(element), up to 2048;
 *   dy must read as zero from D on); x is what was normalised (the forward's residual_out when there was a residual);
 *   mean (NULL for rms norm), rstd [T] fp32 from the forward; dresidual (rows like dy) or NULL: gradient of residual_out, added to dx
 *   dw_part, db_part [parts,ld] fp32 (NULL without weight / bias): one row of partial sums per workgroup, to be added up by the caller
 */
int gdn_norm_gated_bwd(
    const void* dy, const void* x, const void* g, const void* weight, const void* bias,
    const float* mean, const float* rstd, const void* dresidual,
    void* dx, void* dg, float* dw_part, float* db_part,
    int64_t T, int64_t D, int64_t ld, int64_t parts,
    int x_dtype, int w_dtype, int activation, int is_rms_norm, void* stream);

/*
 * Measurement aid with no counterpart in the reference (bench.py --workload calib_rmw): the memory traffic and the
 * dependency of a decode step without its arithmetic.  Every 64 KB block of `data` (n_floats a multiple of 16384)
 * is read, reduced across its workgroup and written back in place.  xcd_run > 0: every XCD works on runs of that
 * many consecutive blocks (0: block b on XCD b % 8); workgroups_per_cu 1..8 caps the workgroups that share a CU
 * (0: no cap).  The decode kernel of gdn_fused_recurrent_fwd uses the shape (HV, 2).
 */
int gdn_calib_rmw(float* data, int64_t n_floats, int xcd_run, int workgroups_per_cu, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GDN_HIP_H */
