/*
 * C ABI of libfla_hip.so: hand-written gfx950 (MI355X) kernels for the chunked
 * linear-attention hot path of flash-linear-attention (chunk_gla,
 * chunk_gated_delta_rule, fused_recurrent_* and the sub-kernels they use).
 *
 * Every entry point takes plain device pointers and sizes plus the HIP stream
 * to launch on, launches asynchronously on that stream, never synchronises
 * and never allocates.  Return value: 0 on success, a positive hipError_t, or
 * a negative FLA_E_* code (argument / shape not supported).
 *
 * Layout: seq-first.  q,k [B,T,H,K]; v,o [B,T,H,V]; per-head scalars [B,T,H];
 * recurrent state fp32 [N,H,K,V].  Packed variable-length batches: B == 1,
 * offsets int64 [N+1] on the device (the reference's `offsets` / newer
 * `cu_seqlens`).  16-bit tensors are bf16 (FLA_BF16) or fp16 (FLA_F16).
 *
 * Each declaration cites the reference interface (path:line in
 * flash-linear-attention) whose kernel launch it replaces.
 */
#ifndef FLA_HIP_H_
#define FLA_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLA_ABI_VERSION 14

enum fla_dtype { FLA_F32 = 0, FLA_BF16 = 1, FLA_F16 = 2 };

enum fla_error {
  FLA_OK = 0,
  FLA_E_INVALID = -1,     /* null pointer / negative size / inconsistent arguments */
  FLA_E_UNSUPPORTED = -2, /* shape, dtype or chunk size outside what the kernels cover */
  FLA_E_ALIGNMENT = -3,   /* pointer or row pitch not aligned for vector access */
  FLA_E_SCRATCH = -4      /* input larger than the library's static scratch buffer (allocation-free entry point) */
};

typedef void* fla_stream_t; /* hipStream_t */

int fla_abi_version(void);
/* Static string for a code returned by any entry point (FLA_E_* or hipError_t). */
const char* fla_error_string(int code);

/* ------------------------------------------------------------------------
 * Integer bookkeeping for packed batches (host arithmetic, host pointers).
 * Replaces prepare_varlen_inputs (fla/ops/gla/chunk.py:1323-1330, inline copy
 * at fla/ops/gated_delta_rule/chunk.py:204-207) and the chunk-offset prefix
 * sums (fla/ops/common/chunk_h.py:274-279, chunk_delta_h.py:240-245).
 * ---------------------------------------------------------------------- */
/* Total number of chunks sum_n ceil(T_n / chunk_size); negative on bad input. */
int64_t fla_count_chunks(const int64_t* offsets_host, int64_t n_seqs, int64_t chunk_size);
/* indices_out [NT,2] = (sequence, chunk in sequence); chunk_offsets_out [N+1]
 * = exclusive prefix sum of per-sequence chunk counts.  Either may be NULL. */
int fla_prepare_chunk_indices(const int64_t* offsets_host, int64_t n_seqs, int64_t chunk_size,
                              int64_t* indices_out, int64_t* chunk_offsets_out);

/* ------------------------------------------------------------------------
 * chunk_local_cumsum (fla/ops/utils/cumsum.py:389-407; scalar kernel :24-57,
 * vector kernel :72-110).  g is [B,T,H] (S == 1) or [B,T,H,S] of g_dtype, out
 * is fp32 of the same shape.  chunk_size is a power of two.  For packed
 * batches pass offsets [N+1] and indices [NT,2] (device), else NULL.
 * ---------------------------------------------------------------------- */
int fla_chunk_local_cumsum(const void* g, float* out, int g_dtype,
                           int64_t B, int64_t T, int64_t H, int64_t S,
                           int64_t chunk_size, int reverse,
                           const int64_t* offsets, const int64_t* indices, int64_t NT,
                           fla_stream_t stream);

/* The inverse of fla_chunk_local_cumsum on fp32 data: out[t] = g_cumsum[t] - g_cumsum[t-1] inside every chunk
 * (the chunk's first row keeps its value; reverse: last row, differences taken towards the end).  For callers
 * of the reference's internal entry points that hold only the cumulative gates (chunk_gla_bwd called with
 * g=None, g_cumsum=..., fla/ops/gsa/chunk.py:741-757) while the kernels here start from the raw ones. */
int fla_chunk_local_cumsum_inverse(const float* g_cumsum, float* out, int64_t B, int64_t T, int64_t H, int64_t S,
                                   int64_t chunk_size, int reverse, const int64_t* offsets,
                                   const int64_t* indices, int64_t NT, fla_stream_t stream);

/* Cumulative sum over the whole sequence (not restarted at chunk boundaries), replaces
 * chunk_global_cumsum (fla/ops/utils/cumsum.py:308-386).  Two launches: chunk-local sums into
 * ws_local (fp32, same shape as s), then each chunk adds the totals of the chunks before
 * (reverse: after) it.  chunk_size is the caller's choice of parallel grain (a power of two;
 * sequence length / 64 keeps the second pass short); offsets/indices as for the local sum,
 * built for the same chunk_size.  out in out_dtype. */
int fla_chunk_global_cumsum(const void* s, float* ws_local, void* out, int s_dtype, int out_dtype, int64_t B,
                            int64_t T, int64_t H, int64_t S, int64_t chunk_size, int reverse,
                            const int64_t* offsets, const int64_t* indices, int64_t NT, fla_stream_t stream);

/* fla_chunk_global_cumsum without the workspace argument, for callers that cannot allocate: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose wrapper allocates its intermediates with torch).  The chunk-local sums go through a
 * static device array of FLA_STATIC_SCRATCH_FLOATS fp32 elements (16 MiB, held by every GPU the library
 * runs on until the process ends); B*T*H*S beyond that returns FLA_E_SCRATCH and launches nothing.  The
 * call allocates nothing; its first call on a device looks the array's address up (do that call outside
 * graph capture, with the stream's device current).  All calls on one GPU share the array: calls that
 * overlap on one GPU (two streams) race.  Same kernels and results as fla_chunk_global_cumsum. */
#define FLA_STATIC_SCRATCH_FLOATS (4 * 1024 * 1024)
int fla_chunk_global_cumsum_static(const void* s, void* out, int s_dtype, int out_dtype, int64_t B, int64_t T,
                                   int64_t H, int64_t S, int64_t chunk_size, int reverse, const int64_t* offsets,
                                   const int64_t* indices, int64_t NT, fla_stream_t stream);

/* ------------------------------------------------------------------------
 * Token-by-token recurrence, forward (fla/ops/common/fused_recurrent.py:322-378,
 * kernel :27-128).  Any of g [B,T,H], gk [B,T,H,K], gv [B,T,H,V] may be NULL;
 * the gates have dtype gate_dtype, q,k,v have dtype qkv_dtype and o has dtype
 * o_dtype.  h0 / ht are fp32 [N,H,K,V] or NULL; ht may alias h0 (state updated
 * in place - every (n,h) tile is read before it is written by the same
 * workgroup).  N = B, or the number of packed sequences when offsets != NULL.
 * ---------------------------------------------------------------------- */
int fla_fused_recurrent_fwd(const void* q, const void* k, const void* v,
                            const void* g, const void* gk, const void* gv,
                            void* o, const float* h0, float* ht,
                            const int64_t* offsets,
                            int qkv_dtype, int gate_dtype, int o_dtype,
                            int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                            float scale, int reverse, fla_stream_t stream);

/* Token-by-token backward of the same recurrence, replaces fused_recurrent_bwd
 * (fla/ops/common/fused_recurrent.py:381-468, kernel :131-319): two passes over the tokens (rebuild h_t and
 * emit dq; then the reverse scan of dh emitting dk, dv), fp32 arithmetic.  dout [B,T,H,V] in the q/k/v dtype;
 * h0, dht, dh0 fp32 [N,H,K,V] or NULL.  dq_partial and dk_partial are fp32 [ceil(V/64), B, T, H, K]: one slice
 * per 64 value columns, their sum over the first dimension is the gradient (the reference sums such partial
 * tensors as well, :445-447); dv is fp32 [B,T,H,V].  The gate gradients follow from these on the caller's side
 * (whole-sequence reverse cumulative sums of q*dq - k*dk and do*o - dv*v, :448-467).  K <= 256, V % 4 == 0. */
int fla_fused_recurrent_bwd(const void* q, const void* k, const void* v, const void* g, const void* gk,
                            const void* gv, const float* h0, const void* dout, const float* dht,
                            float* dq_partial, float* dk_partial, float* dv, float* dh0, const int64_t* offsets,
                            int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                            int64_t N, float scale, int reverse, fla_stream_t stream);

/* Gated delta rule recurrence, forward
 * (fla/ops/gated_delta_rule/fused_recurrent.py:113-167, kernel :19-110).
 * g [B,T,H] or NULL; beta [B,T,H] (beta_per_value == 0) or [B,T,H,V]
 * (beta_per_value == 1), NULL meaning 1.  g and beta have dtype gate_dtype. */
int fla_fused_recurrent_gated_delta_rule_fwd(const void* q, const void* k, const void* v,
                                             const void* g, const void* beta,
                                             void* o, const float* h0, float* ht,
                                             const int64_t* offsets,
                                             int qkv_dtype, int gate_dtype, int o_dtype,
                                             int beta_per_value,
                                             int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                                             int64_t N, float scale, fla_stream_t stream);

/* The same step on un-normalised q and k: every row enters as x / sqrt(sum x^2 + l2norm_eps), the l2 norm the
 * layer applies in front of the operator (fla/layers/gated_deltanet.py:234-237, fla/modules/l2norm.py), formed from
 * the rows the step loads anyway: two launches fewer per decode step. */
int fla_fused_recurrent_gated_delta_rule_fwd_l2norm(const void* q, const void* k, const void* v,
                                                    const void* g, const void* beta,
                                                    void* o, const float* h0, float* ht,
                                                    const int64_t* offsets,
                                                    int qkv_dtype, int gate_dtype, int o_dtype,
                                                    int beta_per_value,
                                                    int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                                                    int64_t N, float scale, float l2norm_eps,
                                                    fla_stream_t stream);

/* ------------------------------------------------------------------------
 * Chunked GLA forward (chunk size 64).
 *
 * fla_chunk_gla_fwd_h: inter-chunk state scan, replaces chunk_fwd_h with gk
 * (fla/ops/common/chunk_h.py:282-335, kernel :29-137).  gates are the raw
 * log-gates gk [B,T,H,K] (gates_are_cumsum == 0, the chunk-local prefix sum
 * is formed in the kernel) or their chunk-local cumsum (== 1, fp32 only).
 * h receives the state ENTERING every chunk, [B,NT,H,K,V] (packed:
 * [1,NT_total,H,K,V], addressed through chunk_offsets [N+1]); h_layout selects
 *   FLA_H_ROW_MAJOR  plain [K,V] tiles of dtype h_dtype (the reference layout),
 *   FLA_H_FRAGMENT   bf16/fp16 tiles in MFMA-fragment order, consumed only by
 *                    fla_chunk_gla_fwd_o / fla_chunk_fwd_o (same byte size),
 *   FLA_H_FRAGMENT_T the same with every tile transposed ([V,K] orientation), the
 *                    operand order of products that contract over V; consumed
 *                    only by the backward entry points.
 * h may be NULL when only ht is wanted.  h0, ht fp32 [N,H,K,V] or NULL.
 *
 * fla_chunk_gla_fwd_o: fused cumsum + intra-chunk gated scores + output,
 * replaces chunk_gla_fwd_intra_gk + chunk_gla_fwd_o_gk
 * (fla/ops/gla/chunk.py:840-938 kernels :29-170; :941-979 kernel :320-393).
 * h must be FLA_H_FRAGMENT.  A_out (optional, fp32 [B,T,H,64]) receives the
 * lower-triangular score matrix the reference saves for backward.
 * ---------------------------------------------------------------------- */
enum fla_h_layout { FLA_H_ROW_MAJOR = 0, FLA_H_FRAGMENT = 1, FLA_H_FRAGMENT_T = 2 };

int fla_chunk_gla_fwd_h(const void* k, const void* v, const void* gates, int gates_are_cumsum,
                        const float* h0, void* h, float* ht,
                        const int64_t* offsets, const int64_t* chunk_offsets,
                        int qkv_dtype, int gate_dtype, int h_dtype, int h_layout,
                        int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                        fla_stream_t stream);

int fla_chunk_gla_fwd_o(const void* q, const void* k, const void* v, const void* gates,
                        int gates_are_cumsum, const void* h, void* o, float* A_out,
                        const int64_t* offsets, const int64_t* indices, int64_t NT,
                        int qkv_dtype, int gate_dtype,
                        int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                        float scale, fla_stream_t stream);

/* Fused chunked GLA forward: o and the final state in one pass, the per-chunk
 * states stay on the chip.  Same result as fla_chunk_gla_fwd_h followed by
 * fla_chunk_gla_fwd_o (the launches of chunk_gla_fwd, fla/ops/gla/chunk.py:1156-1214)
 * with raw log-gates.  K in {64, 128}, V a multiple of 64.  h0, ht, offsets may be NULL.
 * The fused kernel scores a chunk with one reference point (exact while the
 * chunk-cumulative log-gate stays within +-80 per channel; +-8 for fp16 q/k/v, whose
 * range ends at 65504).  With the workspaces
 * ws_wide (int32 [chunks, H]) and ws_hwide (q/k/v dtype, [chunks, H, K*V]) given
 * (V <= 128), chunks outside that range are flagged on the device and their
 * output rows recomputed with exact pairwise exponents (the reference's diagonal
 * sub-block arithmetic, fla/ops/gla/chunk.py:113-170) by the workgroup that owns
 * them, after its last chunk (one launch in all; the 128-column kernel used for
 * more than 128 (sequence, head) pairs at K = V = 128 leaves them to a short
 * second launch);
 * packed batches then also need indices [NT,2] and chunk_offsets [N+1].
 * seq_order (int64 [N], a permutation of the sequence ids, or NULL) is the order
 * in which sequences are handed to the hardware; longest first balances a
 * packed batch. */
int fla_chunk_gla_fwd_fused(const void* q, const void* k, const void* v, const void* gates,
                            const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                            const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets,
                            const int64_t* seq_order, int64_t NT, int qkv_dtype, int gate_dtype,
                            int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                            float scale, fla_stream_t stream);

/* fla_chunk_gla_fwd_fused on the gate projection's output instead of the log-gates: the kernel itself forms
 * g = logsigmoid(gate_logits) / normalizer (then max(g, clamp_min) when has_clamp), the elementwise pass a GLA
 * layer runs in front of chunk_gla (fla/layers/gla.py:214-217), on its way to the prefix sums; the fp32
 * [B,T,H,K] log-gate tensor is never written or read.  gate_logits [B,T,H,K] in gate_dtype (fp32, or the
 * q/k/v dtype).  Forward without kept states; a pass that will be differentiated applies
 * fla_gate_logsigmoid_fwd and calls the entry points above. */
int fla_chunk_gla_fwd_fused_logits(const void* q, const void* k, const void* v, const void* gate_logits,
                                   const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                   const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets,
                                   const int64_t* seq_order, int64_t NT, int qkv_dtype, int gate_dtype, int64_t B,
                                   int64_t T, int64_t H, int64_t K, int64_t V, int64_t N, float scale,
                                   float normalizer, int has_clamp, float clamp_min, fla_stream_t stream);

/* Diagnostics: the scan of fla_chunk_gla_fwd_fused without the recomputation of flagged chunks (with the flag and
 * state hand-over stores of the range guard when the workspaces are given), so that a benchmark can put
 * events round the dominant kernel alone.  o is incomplete for flagged chunks. */
int fla_chunk_gla_fwd_fused_first_launch(const void* q, const void* k, const void* v, const void* gates,
                                         const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                         const int64_t* offsets, const int64_t* indices,
                                         const int64_t* chunk_offsets, const int64_t* seq_order, int64_t NT,
                                         int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H, int64_t K,
                                         int64_t V, int64_t N, float scale, fla_stream_t stream);

/* The same launch for a forward pass whose states are kept for the backward pass: additionally
 * writes the state entering every chunk to h_frag_t ([chunks, H, K*V] in the q/k/v dtype,
 * FLA_H_FRAGMENT_T order), i.e. what fla_chunk_gla_fwd_h would recompute for fla_chunk_gla_bwd
 * (the reference recomputes: fla/ops/gla/chunk.py:1239-1253).  With offsets, chunk_offsets is
 * required. */
int fla_chunk_gla_fwd_fused_states(const void* q, const void* k, const void* v, const void* gates,
                                   const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                   void* h_frag_t, const int64_t* offsets, const int64_t* indices,
                                   const int64_t* chunk_offsets, const int64_t* seq_order, int64_t NT,
                                   int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H, int64_t K,
                                   int64_t V, int64_t N, float scale, fla_stream_t stream);

/* fla_chunk_gla_fwd_fused_states that also leaves what the backward's reverse state scan would otherwise form
 * from q and the gates again (the reference's chunk_bwd_dh does, fla/ops/common/chunk_h.py:156-271): the gated
 * queries q_gated = q e^{G} ([B,T,H,K] in the q/k/v dtype, G the chunk-local prefix sum of the log-gates; rows
 * past the end of a short chunk are not written) and chunk_decay = e^{G_last} (fp32 [chunks, H, K]).  Hand both
 * to fla_chunk_gla_bwd_kept.  khat_t and scores (both or neither, q/k/v dtype): k^ = k e^{G_last - G} per chunk,
 * key-major [chunks, H, K, 64], and the chunk's causal score tile tril(q~ k~^T) (unscaled), [chunks, H, 64, 64]; with
 * them fla_chunk_gla_bwd_kept forms dv inside its reverse state scan. */
int fla_chunk_gla_fwd_fused_kept(const void* q, const void* k, const void* v, const void* gates,
                                 const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                 void* h_frag_t, void* q_gated, float* chunk_decay, void* khat_t, void* scores,
                                 const int64_t* offsets,
                                 const int64_t* indices, const int64_t* chunk_offsets, const int64_t* seq_order,
                                 int64_t NT, int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H,
                                 int64_t K, int64_t V, int64_t N, float scale, fla_stream_t stream);

/* The fused forward for one log-gate per (token, head), g fp32 [B,T,H]: chunk_simple_gla
 * (fla/ops/simple_gla/chunk.py:16-131: h_t = e^{g_t} h_{t-1} + k_t v_t^T, o_t = scale q_t^T h_t) without
 * the [B,T,H,K] gate tensor a call through fla_chunk_gla_fwd_fused would need.  Same kernel, the staging
 * waves load one gate word per row; everything else (workspaces of the range guard, h_frag_t as in
 * fla_chunk_gla_fwd_fused_states or NULL, q_gated and chunk_decay, khat_t and scores as in
 * fla_chunk_gla_fwd_fused_kept or NULL in pairs, packed batches) as for the entry points above. */
int fla_chunk_simple_gla_fwd_fused(const void* q, const void* k, const void* v, const float* g,
                                   const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                   void* h_frag_t, void* q_gated, float* chunk_decay, void* khat_t, void* scores,
                                   const int64_t* offsets, const int64_t* indices,
                                   const int64_t* chunk_offsets, const int64_t* seq_order, int64_t NT,
                                   int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                                   int64_t N, float scale, fla_stream_t stream);

/* chunk_simple_gla forward without kept activations (fla/ops/simple_gla/chunk.py:16-131: chunk_fwd_h + chunk_fwd_o
 * with one gate per (token, head)) on the delta-rule scan kernel with the delta rule taken out (v_new = v, no
 * correction term, no WY tile): q and k reach LDS as they are, the gates ride on the 64x64 score blocks, on the rows
 * of (q h) and on the rows of v, the chunk-local prefix sum of g is formed inside the launch, and the decay factors
 * e^{G_i - G_j} (j <= i) never exceed one, so no range guard is needed.  g: raw log-gates fp32 [B,T,H] or NULL.
 * K in {64, 128}, V a multiple of 64; packed batches as for fla_chunk_gated_delta_rule_fwd_scan. */
int fla_chunk_simple_gla_fwd_scan(const void* q, const void* k, const void* v, const float* g, const float* h0,
                                  void* o, float* ht, const int64_t* offsets, const int64_t* chunk_offsets,
                                  const int64_t* seq_order, int qkv_dtype, int64_t B, int64_t T, int64_t H,
                                  int64_t K, int64_t V, int64_t N, float scale, fla_stream_t stream);

/* ------------------------------------------------------------------------
 * Chunked gated delta rule forward (chunk size 64).  g_cumsum is the fp32
 * chunk-local prefix sum of the per-head log-gate [B,T,H] (from
 * fla_chunk_local_cumsum), or NULL for the un-gated delta rule; beta is fp32
 * [B,T,H].  K in {64,128,256}, V in {64,128} for the three entry points below.
 *
 * fla_gdr_fwd_wy: WY representation, replaces fwd_prepare_wy_repr +
 * fwd_recompute_w_u (fla/ops/gated_delta_rule/wy_fast.py:320-376 kernel
 * :111-236; :379-426 kernel :250-317): Aw = (I + strict_lower(diag(beta) K K^T))^-1,
 * Au = Aw * exp(g_i - g_j), w = Aw (beta K) [B,T,H,K], u = Au (beta V) [B,T,H,V].
 * Aw, Au (optional outputs, [B,T,H,64] in the q/k/v dtype) are what the
 * reference saves for backward; u may be NULL as well (a forward that forms v_new from
 * the triangular tiles of fla_gdr_fwd_prep keeps w and Aw alone).
 *
 * fla_chunk_gated_delta_rule_fwd_h: state scan, replaces
 * chunk_gated_delta_rule_fwd_h (fla/ops/common/chunk_delta_h.py:248-320,
 * kernel :27-119).  Writes the state entering every chunk to h (layout as for
 * fla_chunk_gla_fwd_h; may be NULL), v_new [B,T,H,V] (may be NULL) and ht.
 *
 * fla_chunk_fwd_o: output for scalar-gated models, replaces chunk_fwd_o
 * (fla/ops/common/chunk_o.py:444-495, kernel :23-101); h must be
 * FLA_H_FRAGMENT; v is v_new for the delta rule.
 * ---------------------------------------------------------------------- */
int fla_gdr_fwd_wy(const void* k, const void* v, const float* beta, const float* g_cumsum,
                   void* w, void* u, void* Aw, void* Au,
                   const int64_t* offsets, const int64_t* indices, int64_t NT, int qkv_dtype,
                   int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, fla_stream_t stream);

int fla_chunk_gated_delta_rule_fwd_h(const void* k, const void* w, const void* u, const float* g_cumsum,
                                     const float* h0, void* h, void* v_new, float* ht,
                                     const int64_t* offsets, const int64_t* chunk_offsets,
                                     int qkv_dtype, int h_dtype, int h_layout,
                                     int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                                     fla_stream_t stream);

/* The same scan with the per-chunk states written in both fragment orders: h_frag (FLA_H_FRAGMENT, for
 * fla_chunk_fwd_o) and h_frag_t (FLA_H_FRAGMENT_T, for fla_chunk_gated_delta_rule_bwd), both
 * [chunks, H, K*V] in the q/k/v dtype.  For callers that keep the states of the forward pass for the
 * backward pass instead of recomputing them as chunk_gated_delta_rule_bwd does
 * (fla/ops/gated_delta_rule/chunk.py:105-116). */
int fla_chunk_gated_delta_rule_fwd_h_both(const void* k, const void* w, const void* u, const float* g_cumsum,
                                          const float* h0, void* h_frag, void* h_frag_t, void* v_new, float* ht,
                                          const int64_t* offsets, const int64_t* chunk_offsets, int qkv_dtype,
                                          int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                                          fla_stream_t stream);

int fla_chunk_fwd_o(const void* q, const void* k, const void* v, const float* g_cumsum, const void* h, void* o,
                    const int64_t* offsets, const int64_t* indices, int64_t NT, int qkv_dtype,
                    int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, float scale, fla_stream_t stream);

/* The two-launch forward that forms neither w, u, v_new nor the per-chunk states (what
 * chunk_gated_delta_rule runs when nothing is kept for a backward pass).  fla_gdr_fwd_prep is the chunk-parallel part: it replaces
 * chunk_local_cumsum of the gate and fwd_prepare_wy_repr (fla/ops/gated_delta_rule/wy_fast.py:320-376), reads k,
 * beta and the gate, and leaves, per (chunk, head), one lower-triangular 64x64 matrix in the q/k/v dtype:
 *   Tu  = (Aw * Gamma) diag(beta),  Gamma_ij = exp(gamma_i - gamma_j)   (so that u = Tu v, e^{gamma} w = Tu e^{gamma} k)
 * stored as its ten 16x16 blocks on and below the diagonal (block (i, j) at index i (i + 1) / 2 + j, row-major
 * inside a block): AT is [chunks, H, 10, 16, 16] (chunk index as in `indices`, or b * ceil(T/64) + c).
 * g is the raw per-head log-gate [B,T,H] (g_is_cumsum == 0; its chunk-local prefix sum is formed in the kernel and
 * written to g_cumsum_out, fp32 [B,T,H], if that is given), or already the prefix sum (== 1), or NULL (no gate).
 * w [B,T,H,K] and Aw [B,T,H,64] in the q/k/v dtype, both given or both NULL: w = Aw (beta k) and Aw = (I + M)^-1 as
 * fwd_prepare_wy_repr leaves them (fla/ops/gated_delta_rule/wy_fast.py:320-376), for a forward that will be
 * differentiated (fla_chunk_gated_delta_rule_bwd reads them).
 * K in {64, 128}.
 * fla_chunk_gated_delta_rule_fwd_scan is the serial part (state scan + output, replaces
 * chunk_gated_delta_rule_fwd_h + chunk_fwd_o, fla/ops/gated_delta_rule/chunk.py:47-72): with h the state entering
 * a chunk and Aqk = scale tril(q k^T * Gamma) (the score product of chunk_fwd_o, fla/ops/common/chunk_o.py:86-97,
 * formed inside the scan one chunk ahead),  v_new = Tu (v - e^{gamma} (k h)),  o = scale e^{gamma} (q h) + Aqk v_new,
 * h <- e^{gamma_last} h + k^T (e^{gamma_last - gamma} v_new).  g_cumsum fp32 [B,T,H] or NULL; h0, ht fp32
 * [N,H,K,V] or NULL; packed batches need chunk_offsets [N+1]; seq_order as for fla_chunk_gla_fwd_fused.
 * v_new [B,T,H,V] and h_frag_t (the state entering every chunk, FLA_H_FRAGMENT_T, [chunks,H,K*V]), both in
 * the q/k/v dtype and both given or both NULL: what a forward that will be differentiated keeps for
 * fla_chunk_gated_delta_rule_bwd.  Aqk_out (only with those two, or NULL): the score tiles, packed like AT,
 * [chunks,H,10,16,16], for the same backward.
 * K in {64, 128}, V a multiple of 64. */
int fla_gdr_fwd_prep(const void* k, const float* beta, const float* g, int g_is_cumsum,
                     float* g_cumsum_out, void* AT, void* w, void* Aw, const int64_t* offsets,
                     const int64_t* indices,
                     int64_t NT, int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, fla_stream_t stream);

int fla_chunk_gated_delta_rule_fwd_scan(const void* q, const void* k, const void* v, const void* AT,
                                        const float* g_cumsum, const float* h0, void* o, float* ht,
                                        void* v_new, void* h_frag_t, void* Aqk_out, const int64_t* offsets,
                                        const int64_t* chunk_offsets,
                                        const int64_t* seq_order, int qkv_dtype, int64_t B, int64_t T, int64_t H,
                                        int64_t K, int64_t V, int64_t N, float scale, fla_stream_t stream);

/* The same two launches on un-normalised q and k: the operator works with x / sqrt(sum x^2 + eps) in place of every
 * q and k row, what the two l2_norm launches a gated DeltaNet layer runs in front of it leave
 * (fla/layers/gated_deltanet.py:234-235, fla/modules/l2norm.py:18-40), without writing or reading normalised tensors:
 * every place a normalised row enters is linear in it, so the per-row factors ride on quantities the kernels scale
 * anyway.  The first launch leaves the factors of k in k_rstd_out (fp32 [B,T,H]) for the second, which forms those
 * of q itself.  Forward without kept intermediates; a pass that will be differentiated runs fla_l2norm_fwd / _bwd
 * either side of the entry points above. */
int fla_gdr_fwd_prep_l2norm(const void* k, const float* beta, const float* g, int g_is_cumsum, float* g_cumsum_out,
                            void* AT, float* k_rstd_out, const int64_t* offsets, const int64_t* indices, int64_t NT,
                            int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, float eps,
                            fla_stream_t stream);
int fla_chunk_gated_delta_rule_fwd_scan_l2norm(const void* q, const void* k, const void* v, const void* AT,
                                               const float* g_cumsum, const float* k_rstd, const float* h0, void* o,
                                               float* ht, const int64_t* offsets, const int64_t* chunk_offsets,
                                               const int64_t* seq_order, int qkv_dtype, int64_t B, int64_t T,
                                               int64_t H, int64_t K, int64_t V, int64_t N, float scale, float eps,
                                               fla_stream_t stream);

/* The whole forward of chunk_gated_delta_rule in ONE launch (fla/ops/gated_delta_rule/chunk.py:20-73: cumsum,
 * fwd_prepare_wy_repr, chunk_gated_delta_rule_fwd_h, chunk_fwd_o): q, k, v, the raw per-head log-gate g (fp32
 * [B,T,H] or NULL) and beta (fp32 [B,T,H]) in, o and the final state out; no per-chunk tile crosses memory.  The
 * serial scan of fla_chunk_gated_delta_rule_fwd_scan with the WY operator of the next chunk formed on its matrix
 * waves: M = strict_lower(diag(beta) K K^T * Gamma) in 16x16 blocks, the four diagonal blocks inverted in fp32, and
 * v_new = (I + M)^-1 diag(beta) (v - e^{gamma} (k h)) by block forward substitution.  qk_l2norm: q and k are
 * un-normalised and every row is replaced by x / sqrt(sum x^2 + l2norm_eps) as it is staged
 * (fla/layers/gated_deltanet.py:234-235).  Forward without kept intermediates.  K in {64, 128}, V a multiple of 64;
 * packed batches pass offsets [N+1] (and optionally seq_order, as for fla_chunk_gla_fwd_fused); chunk_offsets is
 * accepted for symmetry with the two-launch form and not read. */
int fla_chunk_gated_delta_rule_fwd_onepass(const void* q, const void* k, const void* v, const float* g,
                                           const float* beta, const float* h0, void* o, float* ht,
                                           const int64_t* offsets, const int64_t* chunk_offsets,
                                           const int64_t* seq_order, int qkv_dtype, int64_t B, int64_t T, int64_t H,
                                           int64_t K, int64_t V, int64_t N, float scale, int qk_l2norm,
                                           float l2norm_eps, fla_stream_t stream);

/* ------------------------------------------------------------------------
 * Chunked GLA backward (chunk size 64), replaces chunk_gla_bwd
 * (fla/ops/gla/chunk.py:1217-1320: chunk_bwd_dh common/chunk_h.py:338-402,
 * chunk_gla_bwd_dv :1018, _dA :982, _dqk_intra :1057, _dqkg :1102).
 * Three launches on `stream`: reverse state scan, dv, dq/dk/dg.
 *   gates   raw log-gates [B,T,H,K] (fp32 or the q/k/v dtype)
 *   dout    gradient of o, [B,T,H,V] in the q/k/v dtype; dht fp32 [N,H,K,V] or NULL
 *   hT      forward states in FLA_H_FRAGMENT_T order (kept by fla_chunk_gla_fwd_fused_states
 *           or recomputed by fla_chunk_gla_fwd_h)
 *   dh_frag_t   workspace the size of hT: the gradient of the per-chunk states,
 *           FLA_H_FRAGMENT_T order
 *   dq, dk [B,T,H,K] and dv [B,T,H,V] in the q/k/v dtype; dg fp32 [B,T,H,K]
 *   (gradient w.r.t. the raw gates); dh0 fp32 [N,H,K,V] or NULL.
 *   wide    int32 [chunks, H] flags written by fla_chunk_gla_fwd_fused (ws_wide), or
 *           NULL.  The kernels score a chunk with one reference point (exact while
 *           the chunk-cumulative log-gate stays within +-80); for flagged chunks the
 *           intra-chunk terms are instead added by a fourth launch with pairwise
 *           exponents <= 0 (the reference's sub-block arithmetic,
 *           fla/ops/gla/chunk.py:409-567).
 * ---------------------------------------------------------------------- */
int fla_chunk_gla_bwd(const void* q, const void* k, const void* v, const void* gates, const void* dout,
                      const float* dht, const void* hT, void* dh_frag_t,
                      void* dq, void* dk, void* dv, float* dg, float* dh0, const int* wide,
                      const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets, int64_t NT,
                      int qkv_dtype, int gate_dtype,
                      int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                      float scale, fla_stream_t stream);

/* The same with q_gated and chunk_decay from fla_chunk_gla_fwd_fused_kept: the reverse state scan
 * (chunk_bwd_dh, fla/ops/common/chunk_h.py:338-402) streams them and do instead of re-forming prefix sums and
 * exponentials from q and the gates; results equal fla_chunk_gla_bwd's to rounding.  scale must not be 0.
 * khat_t and scores (both or NULL) as the forward left them: the scan then also forms dv = s P^T do + k^ dH
 * (chunk_gla_bwd_dv, fla/ops/gla/chunk.py:1037-1061) and the launch of its own for dv is skipped: two launches. */
int fla_chunk_gla_bwd_kept(const void* q, const void* k, const void* v, const void* gates, const void* dout,
                           const float* dht, const void* hT, const void* q_gated, const float* chunk_decay,
                           const void* khat_t, const void* scores, void* dh_frag_t, void* dq, void* dk, void* dv, float* dg, float* dh0, const int* wide,
                           const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets, int64_t NT,
                           int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                           int64_t N, float scale, fla_stream_t stream);

/* The backward of chunk_simple_gla (fla/ops/simple_gla/chunk.py:134-210: chunk_bwd_dh, chunk_bwd_dqkwg,
 * chunk_bwd_dv with one gate per (token, head)) on the same three launches: g fp32 [B,T,H] is read as it is (a lane
 * broadcasts its row's gate over its key channels) and dg, fp32 [B,T,H], which the caller zeroes, receives the
 * gate gradient summed over the key channels (each 64-channel slice of a head adds its share; the additions of
 * one entry happen in a fixed order).  hT, q_gated and chunk_decay as fla_chunk_simple_gla_fwd_fused left them;
 * everything else as for fla_chunk_gla_bwd_kept. */
int fla_chunk_simple_gla_bwd(const void* q, const void* k, const void* v, const float* g, const void* dout,
                             const float* dht, const void* hT, const void* q_gated, const float* chunk_decay,
                             const void* khat_t, const void* scores, void* dh_frag_t, void* dq, void* dk, void* dv, float* dg, float* dh0, const int* wide,
                             const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets, int64_t NT,
                             int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                             float scale, fla_stream_t stream);

/* ------------------------------------------------------------------------
 * The chunk-parallel stages of GLA under the operand layouts of the reference's internal
 * functions, for sibling operators that bring their own scores and states (RWKV6:
 * fla/ops/rwkv6/chunk.py:1163, 1227, 1236).  g_cumsum is the fp32 chunk-local prefix sum of the
 * log-gates [B,T,H,K]; A is [B,T,H,64] (fp32 or the q/k/v dtype, a_dtype); the states h / dh are
 * row-major [chunks, H, K, V] (fp32 or the q/k/v dtype), chunk index as in `indices` (packed)
 * or b * ceil(T/64) + c.  K in {64,128,256}, V a multiple of 64 (dA: V in {64,128,256}).
 *
 * fla_chunk_gla_fwd_o_gk replaces chunk_gla_fwd_o_gk (fla/ops/gla/chunk.py:941-979, kernel :320-393):
 *   o = (scale q e^{g}) h + tril(A) v.
 * fla_chunk_gla_bwd_dA replaces chunk_gla_bwd_dA (fla/ops/gla/chunk.py:982-1015, kernel :582-624):
 *   dA = scale tril(do v^T), fp32 [B,T,H,64].
 * fla_chunk_gla_bwd_dv replaces chunk_gla_bwd_dv (fla/ops/gla/chunk.py:1018-1054, kernel :642-710):
 *   dv = triu(A^T) do + (k e^{g_last - g}) dh, g_last the gate row of the chunk's last token.
 * ---------------------------------------------------------------------- */
int fla_chunk_gla_fwd_o_gk(const void* q, const void* v, const float* g_cumsum, const void* A, const void* h,
                           void* o, const int64_t* offsets, const int64_t* indices, int64_t NT,
                           int qkv_dtype, int a_dtype, int h_dtype, int64_t B, int64_t T, int64_t H,
                           int64_t K, int64_t V, float scale, fla_stream_t stream);

int fla_chunk_gla_bwd_dA(const void* v, const void* dout, float* dA, const int64_t* offsets,
                         const int64_t* indices, int64_t NT, int qkv_dtype, int64_t B, int64_t T,
                         int64_t H, int64_t V, float scale, fla_stream_t stream);

int fla_chunk_gla_bwd_dv(const void* k, const float* g_cumsum, const void* A, const void* dout,
                         const void* dh, void* dv, const int64_t* offsets, const int64_t* indices,
                         int64_t NT, int qkv_dtype, int a_dtype, int dh_dtype, int64_t B, int64_t T,
                         int64_t H, int64_t K, int64_t V, fla_stream_t stream);

/* Reverse state scan with row-major output, replaces chunk_bwd_dh for per-head (g, fp32 [B,T,H]) and / or
 * per-key (gk, fp32 [B,T,H,K]) chunk-cumulative log-gates, either may be NULL
 * (fla/ops/common/chunk_h.py:338-410, kernel :146-262):
 *   for c = last .. 0:  dh[c] <- dH;  dH <- e^{g_last} diag(e^{gk_last}) dH + (scale q e^{g} e^{gk})^T do,
 * starting from dht (fp32 [N,H,K,V] or NULL = 0); dh [chunks,H,K,V] (fp32 or the q/k/v dtype, dh_dtype) is the
 * gradient w.r.t. the state LEAVING each chunk, dh0 (fp32 [N,H,K,V] or NULL) what is left after chunk 0.
 * K and V multiples of 64; packed batches need chunk_offsets [N+1].  q and do have as many heads as the gates. */
int fla_chunk_bwd_dh(const void* q, const float* g, const float* gk, const void* dout, const float* dht,
                     void* dh, float* dh0, const int64_t* offsets, const int64_t* chunk_offsets,
                     int qkv_dtype, int dh_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                     int64_t N, float scale, fla_stream_t stream);

/* Row-major states [n_states, K, V] (fp32 or 16-bit, what chunk_fwd_h and chunk_gated_delta_rule_fwd_h return
 * in the reference: fla/ops/common/chunk_h.py:303, chunk_delta_h.py:289) re-ordered into FLA_H_FRAGMENT
 * (transposed == 0) or FLA_H_FRAGMENT_T (== 1) tiles of the 16-bit dst_dtype, for callers that hold the
 * reference's layout and hand the states to fla_chunk_fwd_o / fla_chunk_gla_fwd_o or a backward entry point.
 * K and V multiples of 32; not in place. */
int fla_states_to_fragments(const void* h_row_major, void* h_frag, int src_dtype, int dst_dtype,
                            int transposed, int64_t n_states, int64_t K, int64_t V, fla_stream_t stream);

/* Intra-chunk part of dv for the operators with a per-head gate, replaces chunk_bwd_dv_local
 * (fla/ops/common/chunk_o.py:551-599, kernel :379-441):
 *   dv_j = sum_{i>=j} scale (k_j . q_i) exp(g_i - g_j) do_i  within each chunk,
 * g_cumsum fp32 [B,T,H] (chunk-local prefix sum) or NULL.  K in {64,128,256}, V in {64,128}.
 * The first launch of fla_chunk_gated_delta_rule_bwd on its own. */
int fla_chunk_bwd_dv_local(const void* q, const void* k, const float* g_cumsum, const void* dout, void* dv,
                           const int64_t* offsets, const int64_t* indices, int64_t NT, int qkv_dtype,
                           int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, float scale,
                           fla_stream_t stream);

/* ------------------------------------------------------------------------
 * Chunked gated delta rule backward (chunk size 64), replaces
 * chunk_gated_delta_rule_bwd (fla/ops/gated_delta_rule/chunk.py:76-177):
 * chunk_bwd_dv_local (common/chunk_o.py:551), chunk_gated_delta_rule_bwd_dhu
 * (common/chunk_delta_h.py:323), chunk_bwd_dqkwg (common/chunk_o.py:602) and
 * bwd_prepare_wy_repr (gated_delta_rule/wy_fast.py:565).  Four launches, or three with Aqk.
 * Inputs recomputed by the caller with the forward entry points: w, v_new, Aw
 * (fla_gdr_fwd_wy, fla_chunk_gated_delta_rule_fwd_h) and hT (the per-chunk
 * states in FLA_H_FRAGMENT_T order).  g_cumsum fp32 [B,T,H] or NULL.
 * Aqk: the packed score tiles [chunks,H,10,16,16] that fla_chunk_gated_delta_rule_fwd_scan leaves on request, or
 * NULL.  With them (K <= 128) the reverse state scan forms dv_local = Aqk^T do itself: the chunk_bwd_dv_local
 * launch is skipped and ws_dv_local may be NULL.
 * Workspaces: ws_dv_local, ws_dv2 like v; ws_dh_frag_t like hT; ws_dw,
 * ws_dk_partial like k; ws_dgam_partial fp32 [K/64, B*T, H].
 * Outputs: dq, dk [B,T,H,K], dv [B,T,H,V] (q/k/v dtype); dbeta and dg fp32
 * [B,T,H]; dh0 fp32 [N,H,K,V] or NULL.  dg is the gradient w.r.t. the raw gate: the last launch
 * adds the slices of ws_dgam_partial to its own gate terms and takes the reverse chunk-local
 * cumulative sum (the reference's chunk_local_cumsum(dg, reverse=True), chunk.py:170-171);
 * without a gate (g_cumsum NULL) it holds nothing meaningful.
 * K in {64,128,256}, V in {64,128}.
 * ---------------------------------------------------------------------- */
int fla_chunk_gated_delta_rule_bwd(
    const void* q, const void* k, const void* v, const void* w, const void* v_new, const float* beta,
    const float* g_cumsum, const void* Aw, const void* dout, const float* dht, const void* hT, const void* Aqk,
    void* ws_dv_local, void* ws_dv2, void* ws_dh_frag_t, void* ws_dw, void* ws_dk_partial, float* ws_dgam_partial,
    void* dq, void* dk, void* dv, float* dbeta, float* dg, float* dh0,
    const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets, int64_t NT, int qkv_dtype,
    int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N, float scale, fla_stream_t stream);

/* The launches of fla_chunk_gated_delta_rule_bwd one by one, for callers that hold the reference's own
 * intermediates (the sibling operators that call these stages directly).  States cross this boundary in
 * FLA_H_FRAGMENT_T order; fla_states_to_fragments / fla_fragments_to_states convert from and to the
 * reference's row-major [.., K, V].  16-bit q/k/v dtype throughout, g_cumsum fp32 [B,T,H] or NULL.
 *
 * fla_chunk_gated_delta_rule_bwd_dhu replaces chunk_gated_delta_rule_bwd_dhu
 * (fla/ops/common/chunk_delta_h.py:323-391, kernel :136-237): reverse scan over the chunks of a sequence,
 *   dh[c] = dH;  dv2 = dv + (k e^{g_last-g}) dH;  dH <- e^{g_last} dH + (scale q e^g)^T do - (w e^g)^T dv2,
 * from dH = dht.  dv is the intra-chunk part (fla_chunk_bwd_dv_local), dv2 [B,T,H,V] the sum, dh_frag_t the
 * gradient w.r.t. the state leaving every chunk, dh0 fp32 [N,H,K,V] or NULL.  K in {64,128,256}, V % 32 == 0.
 *
 * fla_chunk_bwd_dqkwg replaces chunk_bwd_dqkwg (fla/ops/common/chunk_o.py:602-661, kernel :118-265) in the
 * form the delta rule calls it (w and dv given): dq, dk (without the WY path), dw in the q/k dtype and
 * dg_partial fp32 [K/64, B*T, H], whose sum over the first dim is the reference's dg (before the reverse
 * cumulative sum).  v_new is the delta rule's corrected value, dv the dv2 of the scan above.  K % 64 == 0,
 * V in {64,128}.
 *
 * fla_bwd_prepare_wy_repr replaces bwd_prepare_wy_repr (fla/ops/gated_delta_rule/wy_fast.py:565-625, kernel
 * :440-562): the gradient through w = Aw (beta k), u = Au (beta v) with Au = Aw * e^{g_i-g_j}.  Aw
 * [B,T,H,64]; dw like k, du like v.  Outputs dk (+ dk_in, a partial dk in the k dtype that is added before the
 * single rounding; may be NULL), dv, dbeta and dg fp32 [B,T,H].  K in {64,128,256}, V in {64,128}.
 *
 * fla_fwd_recompute_w_u replaces fwd_recompute_w_u (fla/ops/gated_delta_rule/wy_fast.py:320-371, kernel
 * :250-317): w = Aw (beta k), u = Au (beta v) on matrices the caller kept ([B,T,H,64], lower triangular).
 *
 * fla_fragments_to_states: the inverse of fla_states_to_fragments (16-bit fragments to 16-bit or fp32
 * row-major states). */
int fla_chunk_gated_delta_rule_bwd_dhu(const void* q, const void* k, const void* w, const float* g_cumsum,
                                       const float* dht, const void* dout, const void* dv, void* dh_frag_t,
                                       void* dv2, float* dh0, const int64_t* offsets,
                                       const int64_t* chunk_offsets, int qkv_dtype, int64_t B, int64_t T,
                                       int64_t H, int64_t K, int64_t V, int64_t N, float scale,
                                       fla_stream_t stream);
int fla_chunk_bwd_dqkwg(const void* q, const void* k, const void* v_new, const void* w, const float* g_cumsum,
                        const void* h_frag_t, const void* dh_frag_t, const void* dout, const void* dv, void* dq,
                        void* dk, void* dw, float* dg_partial, const int64_t* offsets, const int64_t* indices,
                        int64_t NT, int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                        float scale, fla_stream_t stream);
int fla_bwd_prepare_wy_repr(const void* k, const void* v, const float* beta, const float* g_cumsum, const void* Aw,
                            const void* dw, const void* du, const void* dk_in, void* dk, void* dv, float* dbeta,
                            float* dg, const int64_t* offsets, const int64_t* indices, int64_t NT, int qkv_dtype,
                            int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, fla_stream_t stream);
int fla_fwd_recompute_w_u(const void* k, const void* v, const float* beta, const void* Aw, const void* Au, void* w,
                          void* u, const int64_t* offsets, const int64_t* indices, int64_t NT, int qkv_dtype,
                          int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, fla_stream_t stream);
int fla_fragments_to_states(const void* h_frag, void* h_row_major, int src_dtype, int dst_dtype, int transposed,
                            int64_t n_states, int64_t K, int64_t V, fla_stream_t stream);

/* ------------------------------------------------------------------------
 * Row-wise steps either side of the chunk operators inside the layers
 * (fla/layers/gated_deltanet.py:234-235, fla/layers/gla.py:203-218).
 * Rows are the leading dimensions flattened: x is [M, N], N % 8 == 0, N <= 2048.
 *
 * fla_l2norm_fwd / _bwd replace l2norm_fwd / l2norm_bwd
 * (fla/modules/l2norm.py:91-132, :135-166): y = x / sqrt(sum x^2 + eps),
 * dx = dy*rstd - (sum dy*x) * rstd^3 * x.  x/dx in x_dtype, y in y_dtype, dy in dy_dtype.
 * ---------------------------------------------------------------------- */
int fla_l2norm_fwd(const void* x, void* y, int64_t M, int64_t N, float eps, int x_dtype, int y_dtype,
                   fla_stream_t stream);
int fla_l2norm_bwd(const void* x, const void* dy, void* dx, int64_t M, int64_t N, float eps, int x_dtype,
                   int dy_dtype, fla_stream_t stream);

/* fla_norm_swish_gate_fwd / _bwd replace layer_norm_fwd / layer_norm_bwd of the gated
 * norms (fla/modules/fused_norm_gate.py:186-256, :333-397) without residual:
 *   y = norm(x) * weight (+ bias) * gate * sigmoid(gate),
 * norm = RMS norm (is_rms_norm != 0) or layer norm.  x, gate, y, dy, dx, dgate [M,N] in
 * `dtype`; weight, bias fp32 [N] or NULL; mean (layer norm only) and rstd fp32 [M] are
 * written by the forward and read by the backward.  The backward leaves per-workgroup
 * column sums of the weight / bias gradients in dw_partial / db_partial, fp32
 * [fla_norm_swish_gate_workgroups(M, N), N] (either may be NULL); their sum over the first
 * dimension is the gradient. */
int fla_norm_swish_gate_workgroups(int64_t M, int64_t N);
int fla_norm_swish_gate_fwd(const void* x, const void* gate, const float* weight, const float* bias, void* y,
                            float* mean, float* rstd, int64_t M, int64_t N, float eps, int is_rms_norm,
                            int dtype, fla_stream_t stream);
int fla_norm_swish_gate_bwd(const void* dy, const void* x, const void* gate, const float* weight,
                            const float* bias, const float* mean, const float* rstd, void* dx, void* dgate,
                            float* dw_partial, float* db_partial, int64_t M, int64_t N, float eps,
                            int is_rms_norm, int dtype, fla_stream_t stream);

/* The same pair with the residual / prenorm arguments of layer_norm_fwd / layer_norm_bwd
 * (fla/modules/fused_norm_gate.py:68-74, :103-180; :265-271, :301-400).
 * Forward: the row that is normalised is x + residual (fp32 sum; residual [M,N] in `dtype` or fp32, or NULL);
 * residual_out, if given, receives that sum in `dtype` or fp32 (what the reference returns under prenorm and
 * keeps for its backward).  Backward: x is the tensor the forward normalised (x itself, or residual_out) in
 * x_dtype (`dtype` or fp32); dresidual (same type, or NULL) is the gradient that arrived for residual_out and is
 * added to dx; dresidual_in (same type, or NULL) receives a copy of dx, for a residual whose type differs from x's. */
int fla_norm_swish_gate_residual_fwd(const void* x, const void* gate, const float* weight, const float* bias,
                                     const void* residual, int residual_dtype, void* y, void* residual_out,
                                     int residual_out_dtype, float* mean, float* rstd, int64_t M, int64_t N,
                                     float eps, int is_rms_norm, int dtype, fla_stream_t stream);
int fla_norm_swish_gate_residual_bwd(const void* dy, const void* x, int x_dtype, const void* gate,
                                     const float* weight, const float* bias, const float* mean, const float* rstd,
                                     const void* dresidual, void* dx, void* dgate, void* dresidual_in,
                                     float* dw_partial, float* db_partial, int64_t M, int64_t N, float eps,
                                     int is_rms_norm, int dtype, fla_stream_t stream);

/* ------------------------------------------------------------------------
 * Depthwise causal convolution over time, channels last, replaces the external
 * causal_conv1d_fn / causal_conv1d_update calls of ShortConvolution
 * (fla/modules/convolution.py:171-186 and :188-211):
 *   y[b,t,d] = act(bias[d] + sum_{i<W} weight[d,i] * x[b, t-(W-1)+i, d]),  act = SiLU or identity.
 * x, y, dy, dx [B,T,D] in `dtype`, D % 8 == 0; weight fp32 [D,W], 2 <= W <= 4; bias fp32 [D]
 * or NULL.  The backward leaves per-workgroup partial sums of the weight / bias gradients in
 * dw_partial (fp32 [P,D,W]) and db_partial (fp32 [P,D] or NULL), P =
 * fla_causal_conv1d_bwd_partials(B, T); their sum over P is the gradient (deterministic, no
 * atomics).  The update is the single-token step: cache [B,D,W] (in `dtype`) is
 * shifted left by one and x [B,D] appended in place, y [B,D] = act(bias + sum cache*weight).
 * ---------------------------------------------------------------------- */
int fla_causal_conv1d_fwd(const void* x, const float* weight, const float* bias, void* y, int64_t B, int64_t T,
                          int64_t D, int64_t W, int silu, int dtype, fla_stream_t stream);
int fla_causal_conv1d_bwd_partials(int64_t B, int64_t T);
int fla_causal_conv1d_bwd(const void* x, const float* weight, const float* bias, const void* dy, void* dx,
                          float* dw_partial, float* db_partial, int64_t B, int64_t T, int64_t D, int64_t W, int silu,
                          int dtype, fla_stream_t stream);
int fla_causal_conv1d_update(const void* x, void* cache, const float* weight, const float* bias, void* y,
                             int64_t B, int64_t D, int64_t W, int silu, int dtype, fla_stream_t stream);

/* ------------------------------------------------------------------------
 * Gate pre-activations of the layers that call the chunk operators.
 *
 * fla_gate_logsigmoid_fwd / _bwd replace the elementwise torch ops in front of chunk_gla
 * (fla/layers/gla.py:214-217): y = logsigmoid(x) / normalizer, then max(y, clamp_min) when has_clamp;
 * dx = dy * sigmoid(-x) / normalizer where the clamp did not bind, 0 elsewhere.  n elements
 * (n % 8 == 0); x/dx in x_dtype, y in y_dtype (fp32, or x_dtype), dy in dy_dtype (fp32, or x_dtype).
 *
 * fla_gdn_gate_fwd / _bwd replace the two lines in front of chunk_gated_delta_rule
 * (fla/layers/gated_deltanet.py:236-237): g[m,h] = -exp(A_log[h]) * softplus(a[m,h] + dt_bias[h]) in
 * fp32 (softplus as torch.nn.functional.softplus, threshold 20) and beta = sigmoid(b) in b_dtype;
 * a, b [M,H] in a_dtype / b_dtype (both fp32 or the same 16-bit type), A_log, dt_bias fp32 [H] (dt_bias
 * may be NULL), H <= 256; b / beta (and dbeta / db) may be NULL together.  The backward writes da, db and
 * per-workgroup partial sums partials fp32 [P,2,H], P = fla_gdn_gate_workgroups(M, H): their sums over P
 * are the gradients of A_log (index 0) and dt_bias (index 1); fixed order, no atomics.
 * ---------------------------------------------------------------------- */
int fla_gate_logsigmoid_fwd(const void* x, void* y, int64_t n, float normalizer, int has_clamp, float clamp_min,
                            int x_dtype, int y_dtype, fla_stream_t stream);
int fla_gate_logsigmoid_bwd(const void* x, const void* dy, void* dx, int64_t n, float normalizer, int has_clamp,
                            float clamp_min, int x_dtype, int dy_dtype, fla_stream_t stream);
int fla_gdn_gate_workgroups(int64_t M, int64_t H);
int fla_gdn_gate_fwd(const void* a, const void* b, const float* A_log, const float* dt_bias, float* g, void* beta,
                     int64_t M, int64_t H, int a_dtype, int b_dtype, fla_stream_t stream);
int fla_gdn_gate_bwd(const void* a, const void* b, const float* A_log, const float* dt_bias, const float* dg,
                     const void* dbeta, void* da, void* db, float* partials, int64_t M, int64_t H, int a_dtype,
                     int b_dtype, fla_stream_t stream);

/* Diagnostics: C[M,N] (fp32) = A[M,Kd] * B[N,Kd]^T with bf16 operands, computed
 * with the same MFMA fragment helpers the kernels use (mode 0: 32x32x16 tiles,
 * mode 1: 16x16x32 tiles, mode 2: 32x32x16 with the permuted contraction order
 * used for fragment-layout states).  M, N multiples of 32, Kd of 32. */
int fla_selftest_mfma(const void* A, const void* B, float* C, int64_t M, int64_t N, int64_t Kd,
                      int mode, fla_stream_t stream);

/* Diagnostics: the rate at which a CU is fed when it streams rows the way the chunk scans do (no counterpart in the
 * reference; bench.py reports it beside the scans it bounds).  x holds n_tensors (1-4) tensors [B, T, H, 128] of 16-bit
 * elements, tensor_bytes apart; one 256-thread workgroup per CU reads every row of one (sequence, head) of all of
 * them, 64 rows at a time, and `share` workgroups read the same (sequence, head).  sink[B*H*share] receives the XOR of
 * all 32-bit words each workgroup read.  T a multiple of 64. */
int fla_selftest_stream_tiles(const void* x, int64_t tensor_bytes, int n_tensors, uint32_t* sink, int64_t B,
                              int64_t T, int64_t H, int share, fla_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FLA_HIP_H_ */
