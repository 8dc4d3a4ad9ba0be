/*
 * natsl.h -- C ABI of the MI355X (gfx950) implementation of the NAtS-L token-level hybrid
 * attention forward path.
 *
 * Plain pointers and sizes only: every pointer is DEVICE memory owned by the caller unless a
 * comment says "host"; tensors are dense, token-major [B,T,H,D] as in the reference
 * (src/nats/ops/mixed_ops/mixed_attn_gdn.py:49-50 makes its inputs contiguous).  Nothing here
 * allocates or synchronises with the host; work is enqueued on `stream`.  Two pieces of device
 * memory belong to the library and are shared by all calls on one GPU: the ticket counters of
 * natsl_softmax_sparse_fwd's persistent kernel (64 slots used in rotation, each zeroed on the
 * caller's stream ahead of the launch that uses it) and the scratch of
 * natsl_attn_masked_fwd_static; their comments say what that means for overlapping calls.
 * Each function returns NATSL_OK or a negative natsl_status; natsl_last_error() gives the
 * message for the calling thread.
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * reference repository root).
 */
#ifndef NATSL_H
#define NATSL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* natsl_stream_t; /* a hipStream_t */

enum natsl_dtype { NATSL_F32 = 0, NATSL_BF16 = 1 };

enum natsl_status {
  NATSL_OK = 0,
  NATSL_ERR_INVALID = -1,     /* inconsistent shapes / null pointers */
  NATSL_ERR_UNSUPPORTED = -2, /* a shape or dtype this build has no kernel for */
  NATSL_ERR_WORKSPACE = -3,   /* workspace too small */
  NATSL_ERR_LAUNCH = -4       /* the HIP runtime refused the launch */
};

/* flags for the linear-recurrent branches */
enum natsl_flags {
  NATSL_DECAY_NON_LINEAR = 1, /* decay_for_non_gdn_blocks / decay_for_non_mamba_blocks */
  NATSL_QK_L2NORM = 2,        /* lattn_use_qk_l2norm_in_kernel */
  NATSL_INTRA_CHUNK = 4,      /* the linear op also scores its own incomplete block ('all', 'gated_delta_net', 'mamba') */
  NATSL_QUERY_ONLY = 8        /* recurrent entries: outputs from the decayed block-start state, nothing updated ('attn') */
};

/* One row per packed sequence (cu_seqlens / cu_seqlens_nats of the reference, plus prefix
 * counts the kernels would otherwise have to scan for).  Pass seqs = NULL, n_seqs = 0 for a
 * regular [B,T,...] batch.  With a table, B must be 1, T is the packed length, TN the packed
 * number of selector blocks, and `total_units` is the sum over sequences of the entry point's
 * work unit (ceil(len/64) chunks for the linear branches and the router, ceil(len/256) query
 * tiles for the softmax branch); it is ignored for regular batches. */
typedef struct natsl_seq_row {
  int32_t bos;       /* first token of the sequence (flat token index) */
  int32_t eos;       /* one past its last token */
  int32_t bos_nats;  /* first selector block of the sequence (flat block index) */
  int32_t chunk_off; /* number of 64-token chunks in earlier sequences */
  int32_t qtile_off; /* number of 256-row softmax query tiles in earlier sequences */
  int32_t pad[3];
} natsl_seq_row;

int natsl_version(void);
const char* natsl_last_error(void);

/* Block mean of hidden [B,T,D] -> pooled [B,ceil(T/block),D] (same dtype), divisor
 * min(block, T - c*block).
 * Replaces mean_pooling (src/nats/ops/utils/pooling.py:26-57,190-207) as called by the layer at
 * src/nats/layers/natsl_attn_gdn.py:412-417. */
int natsl_mean_pool(const void* hidden, void* pooled, int B, int T, int D, int block, int dtype,
                    const natsl_seq_row* seqs, int n_seqs, int total_units, natsl_stream_t stream);

/* Selector: logits [B,TN,HN,2] -> types [B,TN,HN,2] in the same dtype with values exactly {0,1}
 * (softmax evaluated in fp32, rounded to the logits dtype, first maximum wins), optionally
 * forcing the last block of every sequence to 1 for both ops, and n_nats_blocks [B,HN,2] int32.
 * Replaces hard_softmax (src/nats/layers/natsl_attn_gdn.py:47-61) and the two statements at
 * src/nats/layers/natsl_attn_gdn.py:553-554. n_nats_blocks may be NULL. */
int natsl_hard_select(const void* logits, void* types, int32_t* n_nats_blocks, int B, int TN, int HN,
                      int dtype, int force_last, const natsl_seq_row* seqs, int n_seqs,
                      int total_units, natsl_stream_t stream);

/* Routing tables derived from types [B,TN,HN,2] (values rounded as the reference does at
 * src/nats/ops/mixed_ops/mixed_attn_gdn.py:88).  Any output may be NULL.
 *   nats_block_indices   int32 [B,TN,HN,2]   ascending ids of selected blocks, padded with TN
 *                                            (mixed_attn_gdn.py:93-97)
 *   n_nats_blocks        int32 [B,HN,2]      (mixed_attn_gdn.py:99-100)
 *   linear_chunk_offsets int64 [B*HN+1]      prepare_nats_chunk_offsets (src/nats/ops/nats_util.py:35-64)
 *   chunk_indices_linear int32 [cap,2]       prepare_nats_block_indices (nats_util.py:6-32); cap must be
 *                                            >= B*HN*TN*(block/64); rows beyond the total are untouched
 *   starting_h_idx       int64 [B,ceil(T/64),HN]   compute_starting_idx_for_chunks (nats_util.py:124-162)
 *   attn_n_iters         int64 [B,ceil(T/128),HN]  compute_attn_n_iters_per_block (nats_util.py:67-121)
 * The last two are defined for regular batches only (seqs == NULL). */
int natsl_route(const void* types, int types_dtype, int B, int TN, int HN, int T, int block,
                int32_t* nats_block_indices, int32_t* n_nats_blocks, int64_t* linear_chunk_offsets,
                int32_t* chunk_indices_linear, int64_t* starting_h_idx, int64_t* attn_n_iters,
                const natsl_seq_row* seqs, int n_seqs, int total_units, natsl_stream_t stream);

/* Softmax branch: causal attention in which a query sees its own block and every earlier block
 * typed "attention" (same_block_visible = 1), or only earlier attention blocks (= 0).
 * q [B,T,HQ,K], k [B,T,HKV,K], v [B,T,HKV,V] -> o [B,T,HQ,V] (same dtype), lse [B,T,HQ] fp32 in
 * log2 units; rows that see no key give o = 0, lse = 0.
 * Replaces parallel_attn_nats_fwd (src/nats/ops/attns/attns.py:1421-1531, kernel :62-353) as
 * called at src/nats/ops/mixed_ops/mixed_attn_gdn.py:111-117.
 * K, V in {64, 128}.  Unpacked input of whole 256-query tiles, at least two per compute unit (T % 256 == 0,
 * T <= 65536, block <= 2048), runs as a persistent kernel whose work queues are ticket counters in device
 * memory owned by the library: 64 slots used in rotation, the launch's slot zeroed by a small fill kernel
 * enqueued on `stream` right before it (both kernels can be captured into a HIP graph).  Launches may overlap
 * across streams as long as fewer than 64 of them are in flight on one GPU; a captured launch keeps the slot it
 * drew at capture, so replay it on the stream that also carries the eager launches. */
int natsl_softmax_sparse_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                             const void* types, int types_dtype, const int32_t* nats_block_indices,
                             const int32_t* n_nats_blocks, int B, int T, int HQ, int HKV, int HN, int K,
                             int V, int TN, int block, float scale, int same_block_visible, int dtype,
                             const natsl_seq_row* seqs, int n_seqs, int total_units, natsl_stream_t stream);

/* The same operation with the same results bit for bit, always as one workgroup per query tile (what
 * natsl_softmax_sparse_fwd itself runs for packed input, ragged lengths and small problems): for callers that
 * want no library-owned device state in the launch, and the regression check of the persistent kernel.
 * Same reference interface as natsl_softmax_sparse_fwd. */
int natsl_softmax_sparse_fwd_per_tile(const void* q, const void* k, const void* v, void* o, float* lse,
                             const void* types, int types_dtype, const int32_t* nats_block_indices,
                             const int32_t* n_nats_blocks, int B, int T, int HQ, int HKV, int HN, int K,
                             int V, int TN, int block, float scale, int same_block_visible, int dtype,
                             const natsl_seq_row* seqs, int n_seqs, int total_units, natsl_stream_t stream);

/* Which kernel natsl_softmax_sparse_fwd runs for a problem on the current device (host-side query, no launch;
 * the choice that src/nats/ops/attns/attns.py:1497-1512 leaves to Triton's autotuner). */
enum natsl_softmax_variant { NATSL_SOFTMAX_TILE_128 = 0, NATSL_SOFTMAX_TILE_256 = 1, NATSL_SOFTMAX_PERSISTENT = 2 };
int natsl_softmax_fwd_variant(int B, int T, int HQ, int HKV, int block, int packed);


/* Backward of the softmax branch: dq [B,T,HQ,K], dk [B,T,HKV,K], dv [B,T,HKV,V] (bf16, summed over the query heads of
 * a kv head) and dnats fp32 [B,TN,HQ], which must be ZERO on entry: per block typed "attention" and query head, the sum
 * of the score gradients dS = P (dP - delta) over (keys of the block) x (queries of later blocks), i.e. the gradient
 * with respect to a bias on that block's scores as later blocks see them; blocks not typed attention keep 0 unless
 * flags bit 1 is set (the reference's compute_dnats_for_invalid_blocks_attn, attns.py:1318-1325): then they get
 * sum min(exp2(s - lse), 1) (dP - delta) over the same (keys) x (later queries), what their keys would contribute if
 * they were visible.  flags bit 0: same_block_visible, as in the forward.  The caller sums dnats over the query heads
 * of a selector head.  o, lse are the forward's outputs, d_o the gradient of o.  workspace: natsl_softmax_bwd_workspace_bytes()
 * bytes (delta = rowsum(d_o * o), then the work-queue counters of the dk/dv kernel; nothing to initialise: every call resets
 * them, so calls that share a workspace must not overlap).  T * HQ * max(K, V) * 2 must stay below 2^32 (32-bit row offsets
 * within the input).  Packed sequences: B = 1 and `seqs` as in the forward, with total_qtiles the table's count of
 * 256-query tiles and total_chunks its count of 64-token chunks (n_nats_blocks is [n_seqs,HN,2]); else null, 0, 0, 0.
 * Replaces parallel_attn_nats_bwd (src/nats/ops/attns/attns.py:1562-1759; kernels :357-372, :383-708, :719-983) as
 * called at src/nats/ops/mixed_ops/mixed_attn_gdn.py:226-243. */
size_t natsl_softmax_bwd_workspace_bytes(int B, int T, int HQ);
int natsl_softmax_sparse_bwd(const void* q, const void* k, const void* v, const void* o, const float* lse, const void* d_o,
                             void* dq, void* dk, void* dv, float* dnats, const void* types, int types_dtype,
                             const int32_t* nats_block_indices, const int32_t* n_nats_blocks, int B, int T, int HQ, int HKV,
                             int HN, int K, int V, int TN, int block, float scale, int flags, int dtype,
                             void* workspace, size_t workspace_bytes, const natsl_seq_row* seqs, int n_seqs,
                             int total_qtiles, int total_chunks, natsl_stream_t stream);

/* Bytes of scratch the two linear-branch entry points need for `total_chunks` 64-token chunks
 * (sum over sequences of ceil(len/64)) and H heads. */
size_t natsl_linear_workspace_bytes(int64_t total_chunks, int H);

/* Gated DeltaNet branch, chunked forward.
 * q,k [B,T,H,K], v [B,T,H,V], beta [B,T,H] in `dtype`; g [B,T,H] fp32 log-decay; h0 / ht
 * [N,H,K,V] fp32 (either may be NULL) -> o [B,T,H,V] in `dtype`.
 * Optional prefill hand-off outputs: h_block_start [N,H,K,V] fp32 = the state that entered each
 * sequence's last selector block, g_block_sum [N,H] fp32 = the sum of g over that block (the two
 * quantities chunk_gated_delta_rule_nats_inference_fwd derives at
 * src/nats/ops/gated_delta_rule/chunk_fwd.py:178-206); pass NULL for both in training.
 * chunk_states (optional, for a backward): the state ENTERING every 64-token chunk, transposed and rounded as the kernel
 * uses it, bf16 [total_chunks][H][V][K] (total_chunks as for natsl_linear_workspace_bytes; the reference keeps the same
 * per-chunk states as `h`, src/nats/ops/common/chunk_delta_h.py:681-683); NULL = not stored.
 * chunk_v_new (optional, for a backward): the delta rule's corrected values v_new of every token, bf16 [B*T][H][V] (the
 * reference's `v_new`, chunk_delta_h.py:684); NULL = not stored.
 * The workspace is scratch between the entry's two kernels and its contents are the entry's own business, except after a call
 * with chunk_states: then it holds what natsl_linear_chunk_bwd reads (per chunk and head TmB, P and four scale vectors).  A
 * call without chunk_states may leave P out (a launch that fills the GPU forms it inside its second kernel).
 * Replaces l2norm_fwd + chunk_gated_delta_rule_nats_fwd
 * (src/nats/ops/mixed_ops/mixed_attn_gdn.py:119-164, src/nats/ops/gated_delta_rule/chunk.py:22-167). */
int natsl_gdn_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const void* beta,
                        const float* h0, void* o, float* ht, float* h_block_start, float* g_block_sum,
                        void* chunk_states, void* chunk_v_new, const void* types, int types_dtype, int B,
                        int T, int H, int HN, int K, int V, int TN, int block, float scale, int flags,
                        void* workspace, size_t workspace_bytes, int dtype, const natsl_seq_row* seqs,
                        int n_seqs, int total_units, natsl_stream_t stream);

/* Mamba2-style SSD branch, chunked forward (q = C, k = B, v = X*dt, g = A*dt).
 * h_block_start / g_block_sum / chunk_states as for the Gated DeltaNet entry (src/nats/ops/mamba/chunk_fwd.py:22-157).
 * Replaces chunk_mamba2_fwd (src/nats/ops/mamba/chunk.py:21-109) as called at
 * src/nats/ops/mixed_ops/mixed_attn_mamba.py:140-161. */
int natsl_mamba_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* h0,
                          void* o, float* ht, float* h_block_start, float* g_block_sum, void* chunk_states, const void* types,
                          int types_dtype, int B, int T, int H,
                          int HN, int K, int V, int TN, int block, float scale, int flags, void* workspace,
                          size_t workspace_bytes, int dtype, const natsl_seq_row* seqs, int n_seqs,
                          int total_units, natsl_stream_t stream);

/* Backward of the two chunked linear branches (delta_rule != 0: Gated DeltaNet, else Mamba2-style SSD); packed input as for the
 * forward (B = 1, the sequence table, TN = all blocks; dht, dh0 then hold one state per sequence).  Call the forward entry first with chunk_states and (delta rule) chunk_v_new and
 * keep its workspace (both forms: the reverse scan reads the scale vectors from it and, for the delta rule, the triangular solves
 * and the intra-chunk matrices).  Inputs as for the forward, plus
 *   v_new [B*T][H][V] (Mamba: v itself), d_o [B*T][H][V] bf16, dht [B][H][K][V] f32 or NULL,
 *   g_block_sums [B][TN][H] f32 = sum of g over every selector block (packed: flat over the sequences' blocks).
 * Outputs: dq, dk [B*T][H][K], dv [B*T][H][V] bf16; dg, dbeta (delta rule) [B*T][H] f32; dh0 [B][H][K][V] f32 or NULL;
 *   d_gate [chunks][H] f32 = derivative with respect to a gate on every chunk's state update (the selector's
 *   straight-through gradient for the linear operator, src/nats/ops/common/chunk_o.py:438-443, :487-492, before the sum over
 *   a block's chunks and a selector head's heads);
 *   d_rollback [chunks][H] f32 = what the decay of a rolled-back block adds to dg of each of its tokens (non-zero behind
 *   the last chunk of blocks that are not typed linear, NATSL_DECAY_NON_LINEAR only);
 *   d_chunk_states: scratch, bf16 [chunks][H][V][K] (the gradient of the state behind every chunk);
 *   dbeta_parts: scratch, f32 [B*T][H][V/16] (delta rule only).
 * K in {64, 128, 192}, V a multiple of 64.
 * Replaces chunk_gated_delta_rule_nats_bwd (src/nats/ops/gated_delta_rule/chunk.py:170-332) and the Mamba counterpart
 * (src/nats/ops/mamba/chunk.py:112-260). */
int natsl_linear_chunk_bwd(int delta_rule, const void* q, const void* k, const void* v_new, const float* g, const void* beta,
                           const void* d_o, const float* dht, const void* chunk_states, const void* types, int types_dtype,
                           const float* g_block_sums, const void* workspace, void* d_chunk_states, float* dbeta_parts,
                           void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0, float* d_gate, float* d_rollback, int B, int T,
                           int H, int HN, int K, int V, int TN, int block, float scale, int flags, int dtype,
                           const natsl_seq_row* seqs, int n_seqs, int total_chunks, natsl_stream_t stream);

/* Layer tail: y = (rms(x1)*w1*xw[...,0] + rms(x2)*w2*xw[...,1]) * gate*sigmoid(gate) with
 * rms(x) = x*rsqrt(mean(x^2)+eps); x1, x2, gate, y [rows, D] and x_weights [rows, 2] in `dtype`,
 * w1, w2 [D] in `w_dtype`.  D in {32, 64, 96, 128, 192, 256, 384, 512}.
 * Replaces the forward of FusedMultiInputRMSNormGated (src/nats/modules/fused_norm_gate.py:38-182)
 * as called at src/nats/layers/natsl_attn_gdn.py:652-661. */
int natsl_norm_gate_fwd(const void* x1, const void* x2, const void* gate, const void* x_weights, const void* w1,
                        const void* w2, void* y, int64_t rows, int D, int dtype, float eps, int w_dtype,
                        natsl_stream_t stream);

/* Backward of natsl_norm_gate_fwd: dx1, dx2, dgate [rows, D] in `dtype`; dx_weights [rows, 2] f32; dw1, dw2 [D] f32, the two
 * rows of ONE [2][D] tensor (dw2 == dw1 + D).  The weight gradients are summed over the rows in a fixed order (partial sums
 * per 128 rows in the workspace, then one reduction): the same bits on every run.
 * Replaces the backward of FusedMultiInputRMSNormGated (src/nats/modules/fused_norm_gate.py:185-420). */
size_t natsl_norm_gate_bwd_workspace_bytes(int64_t rows, int D);
int natsl_norm_gate_bwd(const void* x1, const void* x2, const void* gate, const void* x_weights, const void* w1,
                        const void* w2, const void* dy, void* dx1, void* dx2, void* dgate, float* dx_weights, float* dw1,
                        float* dw2, void* workspace, size_t workspace_bytes, int64_t rows, int D, int dtype, float eps,
                        int w_dtype, natsl_stream_t stream);

/* Layer glue, depthwise causal short convolution with its activation, on the layer's token-major tensors:
 * y[b,t,d] = act(bias[d] + sum_j w[d,j] e[b, t-(W-1)+j, d]) where e is x preceded by the W-1 inputs before it: the last
 * W-1 entries of `state` [B,D,W] (the cache of a previous call, in `state_dtype`), or zeros when state is NULL.
 * x, y [B,T,D] in `dtype` (f32 or bf16; sums in f32, one rounding); weight [D,W] (the [D,1,W] of a Conv1d), bias [D] or NULL
 * in `w_dtype`; activation 0 = none, 1 = silu; W in {2, 3, 4}; D % 8 == 0.  state_out [B,D,W] in `dtype`, or NULL: the
 * last W inputs of (state ++ x), what the next call takes as `state`; it must not alias `state`.
 * Replaces the forward of flash-linear-attention's ShortConvolution as called at
 * src/nats/layers/natsl_attn_gdn.py:425-491 and src/nats/layers/natsl_attn_mamba2.py:368-425. */
int natsl_short_conv_fwd(const void* x, const void* weight, const void* bias, const void* state, void* y, void* state_out,
                         int B, int T, int D, int W, int activation, int dtype, int w_dtype, int state_dtype,
                         natsl_stream_t stream);

/* Backward of natsl_short_conv_fwd: dx [B,T,D] in `dtype` (gradient of x; the cached state gets none), dweight fp32 [D,W],
 * dbias fp32 [D] or NULL, from x, weight, bias, state as given to the forward and dy [B,T,D] in `dtype`.  The pre-activation
 * is recomputed; the weight sums are reduced in a fixed order through the workspace
 * (natsl_short_conv_bwd_workspace_bytes(), fp32 partial sums per run of tokens): no atomics, repeatable bits.
 * Replaces the backward of flash-linear-attention's ShortConvolution under the same call sites. */
size_t natsl_short_conv_bwd_workspace_bytes(int B, int T, int D, int W);
int natsl_short_conv_bwd(const void* x, const void* weight, const void* bias, const void* state, const void* dy, void* dx,
                         float* dweight, float* dbias, void* workspace, size_t workspace_bytes, int B, int T, int D, int W,
                         int activation, int dtype, int w_dtype, int state_dtype, natsl_stream_t stream);

/* Layer glue, row normalisation: y = x * rsqrt(mean(x^2) + eps) * weight (l2 = 0, RMSNorm; weight [D] in `w_dtype` or NULL
 * for none) or y = x * rsqrt(sum(x^2) + eps) (l2 = 1).  x, y [rows, D] in `dtype` (f32 or bf16), arithmetic in f32.
 * D in {32, 64, 96, 128, 192, 256, 384, 512}.
 * Replaces the RMSNorm of the attention view's q and k (flash-linear-attention's, called at
 * src/nats/layers/natsl_attn_gdn.py:504-505) and the L2 normalisation of the Mamba layer's B and C
 * (src/nats/layers/natsl_attn_mamba2.py:469-470). */
int natsl_row_norm_fwd(const void* x, const void* weight, void* y, int64_t rows, int D, float eps, int l2, int dtype,
                       int w_dtype, natsl_stream_t stream);

/* Backward of natsl_row_norm_fwd: dx [rows, D] in `dtype`; dweight [D] f32 when a weight is given (summed over the rows in a
 * fixed order: partial sums per 128 rows in the workspace, then one reduction; no weight: workspace may be NULL).
 * Replaces the backward of the reference's RMSNorm / l2norm modules (fla.modules, as used at
 * src/nats/layers/natsl_attn_gdn.py:275-330). */
size_t natsl_row_norm_bwd_workspace_bytes(int64_t rows, int D);
int natsl_row_norm_bwd(const void* x, const void* weight, const void* dy, void* dx, float* dweight, void* workspace,
                       size_t workspace_bytes, int64_t rows, int D, float eps, int l2, int dtype, int w_dtype,
                       natsl_stream_t stream);

/* Decode: T tokens that continue the current (incomplete) selector block of N cached sequences, token by
 * token.  Per token: S *= e^g; d = beta (v - S^T k); S += k d^T; o = scale S^T q (k, q L2-normalised with
 * NATSL_QK_L2NORM).  Only the first min(T, block - n_tokens_in_block) tokens are processed.  If they
 * complete the block (n_tokens_in_block + T >= block) and the block is not typed linear, S is restored to
 * h_block_start (times e^(g_cumsum + sum of g) with NATSL_DECAY_NON_LINEAR), and in either case
 * h_block_start <- S.  q,k [N,T,H,K], v,o [N,T,H,V], beta [N,T,H] in `dtype`; g fp32 [N,T,H];
 * g_cumsum fp32 [N,H] or NULL (0): sum of g over the tokens already in the block; h0 fp32 [N,H,K,V] or NULL
 * (zeros); h_block_start fp32 [N,H,K,V] in/out; ht fp32 [N,H,K,V] or NULL; types [N,1,HN,2] (op 1 = linear);
 * n_tokens_in_block int32 [N] or NULL (then the scalar is used for every sequence).  K in {64, 128, 192}, V % 16 == 0.
 * With NATSL_QUERY_ONLY (the mode in which the linear operator skips the incomplete block, ops_for_incomplete_chunks = 'attn'):
 * o_t = scale q_t^T (e^(g_cumsum + g_1 + .. + g_t) h_block_start), no state is read from h0 or written; k, v, beta may be NULL
 * (the reference's branch without UPDATE_HS_FOR_EACH_ITER, fused_recurrent.py:156-201, as called for one-token steps at
 * src/nats/ops/mixed_ops/mixed_attn_gdn.py:510-527).
 * Replaces fused_recurrent_gated_delta_rule_nats_fwd, src/nats/ops/gated_delta_rule/fused_recurrent.py:360-470
 * (kernel :28-358) as called with update_hs_for_each_iter=True at
 * src/nats/ops/mixed_ops/mixed_attn_gdn.py:485-503. */
int natsl_gdn_recurrent_fwd(const void* q, const void* k, const void* v, const float* g, const float* g_cumsum,
                            const void* beta, const float* h0, float* h_block_start, void* o, float* ht,
                            const void* types, int types_dtype, const int32_t* n_tokens_in_block,
                            int n_tokens_in_block_scalar, int N, int T, int H, int HN, int K, int V, int block,
                            float scale, int flags, int dtype, natsl_stream_t stream);

/* The same for the Mamba2 (SSD) branch: S *= e^g; S += k v^T; o = scale S^T q (q = C, k = B, v = x*dt); no beta,
 * no normalisation (NATSL_QK_L2NORM is ignored).
 * Replaces fused_recurrent_mamba_nats_fwd (src/nats/ops/mamba/fused_recurrent.py, kernel :150-300) as called
 * at src/nats/ops/mixed_ops/mixed_attn_mamba.py:498-514. */
int natsl_mamba_recurrent_fwd(const void* q, const void* k, const void* v, const float* g, const float* g_cumsum,
                              const float* h0, float* h_block_start, void* o, float* ht, const void* types,
                              int types_dtype, const int32_t* n_tokens_in_block, int n_tokens_in_block_scalar, int N,
                              int T, int H, int HN, int K, int V, int block, float scale, int flags, int dtype,
                              natsl_stream_t stream);

/* Decode: softmax attention of TQ queries over TK cached keys under an explicit visibility mask.
 * q [B,TQ,HQ,K], k [B,TK,HKV,K], v [B,TK,HKV,V], o [B,TQ,HQ,V] in `dtype`; mask uint8 [B,HM,TQ,TK], non-zero =
 * visible, HM divides HQ; query head hq uses kv head hq/(HQ/HKV) and mask head hq/(HQ/HM).  A query that sees
 * no key gives 0.  With a workspace of natsl_attn_masked_workspace_bytes() the keys of one query are split over
 * several workgroups (needed to fill the GPU when B*TQ*HQ is small); with workspace = NULL one workgroup
 * handles a query.  k_batch_stride / v_batch_stride: elements from one sequence's keys / values to the next, for keys that
 * are the front part of a larger cache buffer [B,capacity,HKV,D] (a multiple of 8, at least TK*HKV*D); 0 = dense.
 * Replaces repeat_masks + torch.nn.functional.scaled_dot_product_attention at
 * src/nats/ops/mixed_ops/mixed_attn_gdn.py:475-481. */
size_t natsl_attn_masked_workspace_bytes(int B, int TQ, int TK, int HQ, int V);
int natsl_attn_masked_fwd(const void* q, const void* k, const void* v, const uint8_t* mask, void* o, int B, int TQ,
                          int TK, int HQ, int HKV, int HM, int K, int V, float scale, int dtype, void* workspace,
                          size_t workspace_bytes, int64_t k_batch_stride, int64_t v_batch_stride, natsl_stream_t stream);

/* natsl_attn_masked_fwd for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc): the same kernels with the split scratch in a device array of the library itself, so the caller
 * passes inputs and outputs only and the call allocates nothing.  It has no counterpart in the reference.  The array
 * holds natsl_attn_masked_static_scratch_bytes() = 256 KiB per GPU for the life of the process; a shape whose splits need
 * more (natsl_attn_masked_workspace_bytes() above that limit) is refused with NATSL_ERR_WORKSPACE.  Results are
 * identical to natsl_attn_masked_fwd with a workspace.  All calls on one GPU share the array: calls that overlap on
 * one GPU (different streams or threads) race. */
size_t natsl_attn_masked_static_scratch_bytes(void);
int natsl_attn_masked_fwd_static(const void* q, const void* k, const void* v, const uint8_t* mask, void* o, int B, int TQ,
                                 int TK, int HQ, int HKV, int HM, int K, int V, float scale, int dtype,
                                 natsl_stream_t stream);

/* KV cache of the softmax branch: keep the attention-typed blocks of a region of new tokens, per (sequence, kv
 * head), back to back behind the blocks already kept, and put the tokens of the incomplete last block at block
 * index tail_dst (the same for every head; pass -1 when the region ends on a block boundary).
 * src_k/src_v [B, src_tokens, HKV, K|V] hold the region from block src_block0 on: NB blocks of `block` tokens,
 * the first n_complete complete (n_complete = NB, or NB-1 with an incomplete block of tail_tokens tokens).
 * dst_k/dst_v [B, dst_tokens, HKV, K|V] is the cache; it may be the source itself (in place: same pointers and
 * sizes), since a kept block never moves towards the back.  types [B, NB, HN, 2] (f32 or bf16): column 0 equal to
 * 1 marks an attention-typed block; kv head h follows selector head h/(HKV/HN).  n_before int64 [B, HN] = blocks
 * already kept per (sequence, selector head), NULL = none.  The caller sizes the destination for the largest new
 * count (stores past dst_tokens are dropped, never issued).  The rest of the block at tail_dst is zero filled when
 * the block is moved or copied.
 * Replaces the gather/scatter at src/nats/models/utils.py:509-588 (NAtSLayerCache.update). */
int natsl_kv_compact(const void* src_k, const void* src_v, long long src_tokens, int src_block0, void* dst_k, void* dst_v,
                     long long dst_tokens, const void* types, int types_dtype, const int64_t* n_before, int B, int HKV,
                     int HN, int K, int V, int dtype, int block, int NB, int n_complete, int tail_dst, int tail_tokens,
                     natsl_stream_t stream);


#ifdef __cplusplus
}
#endif
#endif /* NATSL_H */
