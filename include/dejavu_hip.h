/*
 * C ABI of libdejavu_hip.so: hand-written gfx950 kernels for DejaVu's
 * contextual-sparsity decode path.
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless stated; fp16 tensors are
 *    row-major with a contiguous last dimension; row strides (ld*) are in
 *    elements and must be multiples of 8 (rows are read with 128-bit loads),
 *    and base pointers must be 16-byte aligned;
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *  - calls only enqueue work: no allocation, no synchronisation, no host
 *    copies.  Scratch memory is supplied by the caller (`workspace`);
 *  - index vectors hold int32 (idx_bytes = 4) or int64 (idx_bytes = 8) values;
 *    an index outside the valid range contributes zero instead of faulting;
 *  - return value: DV_OK (0) or a negative DV_ERR_* code; nothing throws.
 *
 * Each entry point names the reference interface it replaces
 * (paths relative to the FMInference/DejaVu checkout).
 */
#ifndef DEJAVU_HIP_H
#define DEJAVU_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DV_API __attribute__((visibility("default")))

#define DV_OK 0
#define DV_ERR_INVALID_ARG (-1)  /* null pointer, negative size, bad idx_bytes, k > n ... */
#define DV_ERR_UNSUPPORTED (-2)  /* shape outside what the kernels are built for        */
#define DV_ERR_ALIGNMENT (-3)    /* stride / size / pointer not a multiple of 8 elements  */
#define DV_ERR_WORKSPACE (-4)    /* workspace missing or too small                      */
#define DV_ERR_LAUNCH (-5)       /* the HIP runtime rejected the launch                 */

#define DV_ACT_ID 0
#define DV_ACT_RELU 1
#define DV_ACT_GELU 2         /* x * 0.5 * (1 + erf(x / sqrt(2)))               k_activations.py:136-139 */
#define DV_ACT_GELU_APPROX 3  /* tanh form                                      k_activations.py:148-155 */
#define DV_ACT_SQUARED_RELU 4 /* relu(x)^2                                      k_activations.py:92-100  */

/* Library version (major*10000 + minor*100 + patch). */
DV_API int dv_version(void);
/* Static string for a DV_* code. */
DV_API const char* dv_error_string(int code);

/* Lanes that share one row of length n in the predictor's fixed summation
 * order (16 for n <= 1024, else 64); tests restate the order from this. */
DV_API int dv_canonical_lanes(int n);

/*
 * Low-rank sparsity predictor, logits = Wb . fp16(Wa . x), both bias-free,
 * fp32 accumulation in a fixed order, fp16 results.
 * Replaces ParallelSP.forward, Dejavu/src/ops/fused_dense_sparse_dejavu.py:73-76
 * (duplicate at Dejavu/src/models/modules/mha_dejavu.py:1118-1121).
 *   x (B, d); Wa (r, d) row stride ldwa; Wb (n_out, r) row stride ldwb;
 *   hidden (B, r) scratch/output; logits (B, n_out).  1 <= B <= 64.
 * Up to 8 rows the summation order is the fixed one (bit-reproducible on the
 * host); 9..64 rows run as two MFMA products whose fp32 accumulation order is
 * the matrix core's own (same values within fp16 rounding).
 */
DV_API int dv_predictor_logits_f16(const void* x, const void* Wa, int64_t ldwa, const void* Wb,
                            int64_t ldwb, int B, int d, int r, int n_out, void* hidden,
                            void* logits, void* stream);

/*
 * The same with a workspace: for 9..64 rows the first product (r rows of d
 * elements: few row tiles) shares each block of x through LDS and is split over
 * the columns, each split writing fp32 partial sums that a second launch adds in
 * ascending order (deterministic); so is the second product when it has few rows.
 * workspace: dv_predictor_workspace_bytes(B, d, r) bytes, 16-byte aligned; with
 * NULL / 0 the call behaves like dv_predictor_logits_f16.  Up to 8 rows the
 * workspace is not used.
 */
DV_API size_t dv_predictor_workspace_bytes(int B, int d, int r);
DV_API int dv_predictor_logits_ws_f16(const void* x, const void* Wa, int64_t ldwa, const void* Wb,
                                      int64_t ldwb, int B, int d, int r, int n_out, void* hidden,
                                      void* logits, void* workspace, size_t workspace_bytes,
                                      void* stream);

/*
 * Index set of the k largest logits, ties to the lower index, written in
 * ascending index order.  For B > 1 a column's score is its maximum over the
 * B rows.  Replaces Tensor.topk(k, sorted=False) at
 * Dejavu/src/models/modules/mha_dejavu.py:1069, 1369, 1506-1507.
 *   logits (B, n) fp16; idx_out (k,) int32/int64.  n <= 65536, 0 <= k <= n.
 * dv_topk_f16: n <= 1024 is ranked in one workgroup; larger n (n % 8 == 0)
 *   takes three launches spread over many workgroups: per-workgroup key
 *   histograms, the threshold read off their sum plus per-workgroup counts,
 *   then the ordered emission (no atomics on global memory: deterministic,
 *   and no slower when many logits share a value).  workspace:
 *   dv_topk_workspace_bytes(n) bytes, no initialisation needed; calls sharing
 *   it must not overlap.
 * dv_topk_search_f16: same result in a single launch without scratch memory
 *   (16-step bitwise threshold search in one workgroup).
 */
DV_API size_t dv_topk_workspace_bytes(int n);
DV_API int dv_topk_f16(const void* logits, int B, int n, int k, void* idx_out, int idx_bytes,
                       void* workspace, size_t workspace_bytes, void* stream);
DV_API int dv_topk_search_f16(const void* logits, int B, int n, int k, void* idx_out,
                              int idx_bytes, void* stream);

/*
 * y = act(x . W[idx]^T + bias[idx]).  Replaces gather_gemv,
 * Dejavu/src/ops/triton/gather_gemv.py:198-254.
 *   x (B, N); W (Z, N) row stride ldw; bias (Z,) or NULL; idx (M,);
 *   y (B, M) fp16.  1 <= B <= 64 (the reference stops at 4): B <= 2 runs as a
 *   bandwidth-bound GEMV on the vector ALUs; 3 <= B <= 64 stages the gathered
 *   rows through LDS into 16x16x32 fp16 MFMA tiles.
 * idx == NULL: no gather, row m of W (a dense product y = act(x W[:M]^T + bias), M <= Z),
 * as the one-token decode step of a dense block or of the lm_head needs it.
 */
DV_API int dv_gather_gemv_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                       const void* idx, int idx_bytes, int B, int N, int Z, int M, int act,
                       void* y, void* stream);

/*
 * dv_gather_gemv_f16 with a workspace: from 17 batch rows on, the whole workgroup shares each block
 * of X through LDS (X leaves L2 once per 128 gathered rows instead of once per 16) and the columns
 * are also split over workgroups, each split writing fp32 partial sums that a second launch adds in
 * ascending order (deterministic) before bias and activation.
 *   workspace: dv_gather_gemv_workspace_bytes(B, N, M) bytes, 16-byte aligned, no initialisation
 *   needed; with NULL / too small a workspace, or fewer than 17 rows, the call is dv_gather_gemv_f16.
 */
DV_API size_t dv_gather_gemv_workspace_bytes(int B, int N, int M);
DV_API int dv_gather_gemv_ws_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                                 const void* idx, int idx_bytes, int B, int N, int Z, int M, int act,
                                 void* y, void* workspace, size_t workspace_bytes, void* stream);

/*
 * y = act(x . W^T + bias) for any number of rows, on the matrix cores: the dense products of the
 * prompt phase (Wqkv, out_proj, fc1 + activation, fc2), which the reference runs through
 * nn.Linear / fused_dense_lib (Dejavu/src/ops/fused_dense_sparse_dejavu.py:924-936 fused_mlp_func,
 * Dejavu/src/models/modules/mha_dejavu.py:1494-1496 Wqkv / out_proj of the dense branch).
 * Blocks of up to 128 rows of x are shared through LDS by a workgroup that streams 256 weight rows;
 * short matrices are also split over the columns (fp32 partial sums, added in ascending order).
 *   x (rows, N) row stride ldx; W (M, N) row stride ldw; bias (M,) or NULL; y (rows, M) row stride
 *   ldy; workspace: dv_dense_linear_workspace_bytes(rows, N, M) bytes (may be 0), 16-byte aligned.
 */
DV_API size_t dv_dense_linear_workspace_bytes(int rows, int N, int M);
DV_API int dv_dense_linear_f16(const void* x, int64_t ldx, const void* W, int64_t ldw, const void* bias,
                               int rows, int N, int M, int act, void* y, int64_t ldy, void* workspace,
                               size_t workspace_bytes, void* stream);

/*
 * y = x . W[idx] + bias.  Replaces gather_transposed_gemv,
 * Dejavu/src/ops/triton/gather_gemv.py:572-644 (deterministic: fixed-order
 * split over row groups instead of floating-point atomics).
 *   x (B, M); W (Z, N) row stride ldw; bias (N,) or NULL; idx (M,);
 *   y (B, N) fp16.  1 <= B <= 64 (vector ALUs up to 4; above, the weight tile is transposed in
 *   registers into 16x16x32 MFMA operands up to 32 rows, 32x32x16 operands up to 64).
 *   workspace: dv_gather_transposed_gemv_workspace_bytes(B, N, M) bytes, no
 *   initialisation needed; calls sharing it must not overlap.  y and workspace must be
 *   16-byte aligned (vector stores), else DV_ERR_ALIGNMENT.
 */
DV_API size_t dv_gather_transposed_gemv_workspace_bytes(int B, int N, int M);
DV_API int dv_gather_transposed_gemv_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                                  const void* idx, int idx_bytes, int B, int N, int Z, int M,
                                  void* y, void* workspace, size_t workspace_bytes,
                                  void* stream);

/*
 * dv_gather_transposed_gemv_f16 without a workspace argument and without any allocation: the
 * fp32 partial sums of the split go to a fixed DV_STATIC_SCRATCH_BYTES array in device memory
 * that belongs to the library (one per GPU, held until the process ends).  It has no
 * counterpart in the reference; it is for callers that cannot allocate or size scratch memory:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same kernels and same bits as dv_gather_transposed_gemv_f16.  Shapes whose partial sums
 * exceed the array (dv_gather_transposed_gemv_workspace_bytes(B, N, M) >
 * DV_STATIC_SCRATCH_BYTES: at the OPT shapes, batches above 32) return DV_ERR_WORKSPACE.
 * The array has DV_STATIC_SCRATCH_STREAMS slots of DV_STATIC_SCRATCH_BYTES; a stream keeps the slot
 * it is given at its first call for the life of the process, so calls on different streams do not
 * share partial sums (calls on one stream are ordered by the stream).  A call on one more stream
 * than there are slots returns DV_ERR_UNSUPPORTED; two host threads that launch on the SAME stream
 * without ordering their calls still race.  Nothing needs clearing between calls (every word is
 * written before it is read).  y must be 16-byte aligned.
 */
#define DV_STATIC_SCRATCH_BYTES (8u << 20)
#define DV_STATIC_SCRATCH_STREAMS 2
DV_API int dv_gather_transposed_gemv_static_f16(const void* x, const void* W, int64_t ldw,
                                                const void* bias, const void* idx, int idx_bytes,
                                                int B, int N, int Z, int M, void* y, void* stream);

/*
 * QKV projection restricted to the active heads and the live window tokens:
 *   y[b, t, h, :] = x[b, :] . W[t, h, :, :]^T + bias[t, h, :]
 * for h = head_idx[i] and every b = batch_idx[i, s] >= 0.  Nothing is written
 * for other heads / tokens (the reference leaves them uninitialised too).
 * Replaces qkv_proj_sparse, Dejavu/src/ops/triton/attention_proj_sparse.py:110-194.
 *   x (nb, d), nb <= 16; W (3, H, hd, d) contiguous; bias (3, H, hd) or NULL;
 *   head_idx (nnz,) int32; batch_idx (nnz, nb) int32; y (nb, 3, H, hd);
 *   hd in {32, 64, 128}.
 */
DV_API int dv_qkv_proj_sparse_f16(const void* x, const void* W, const void* bias,
                                  const void* head_idx, const void* batch_idx, int nb, int d,
                                  int H, int hd, int nnz, void* y, void* stream);

/*
 * dv_qkv_proj_sparse_f16 with the cache scatter of dv_kv_cache_copy_sparse_f16
 * fused into its epilogue: K and V rows are also written to
 * k_cache[0, h, :, token + padding[0], :] / v_cache[0, h, token + padding[0], :].
 * (qkv_proj_sparse followed by k_cache_copy_sparse + v_cache_copy_sparse with
 * seqlen_idx = batch_idx, Dejavu/src/models/modules/mha_dejavu.py:1333-1352, 1425-1438.)
 *   k_cache (1, H, hd/8, S, 8), v_cache (1, H, S, hd): both or neither NULL.
 */
DV_API int dv_qkv_proj_sparse_cache_f16(const void* x, const void* W, const void* bias,
                                        const void* head_idx, const void* batch_idx, int nb, int d,
                                        int H, int hd, int nnz, void* y, void* k_cache,
                                        void* v_cache, const void* padding, int S, void* stream);

/*
 * QKV projection of the active heads for one token of each of B sequences that share the head
 * set, with the K / V rows appended to per-sequence caches:
 *   y[b, t, h, :] = x[b, :] . W[t, h, :, :]^T + bias[t, h, :]   for h = head_idx[i], every b < B
 *   k_cache[b, h, :, p_b, :], v_cache[b, h, p_b, :] <- the K / V rows, p_b = positions[per_sample ? b : 0] + pos_add
 * Batch extension of qkv_proj_sparse + k/v_cache_copy_sparse
 * (Dejavu/src/models/modules/mha_dejavu.py:1333-1352, 1425-1438; the reference's sparse
 * attention is single-sequence, mha_dejavu.py:1469): all B rows are multiplied against each
 * weight tile on the matrix cores, the weights stream once.
 *   x (B, d) row stride ldx, B <= 32; W (3, H, hd, d); bias (3, H, hd) or NULL; head_idx (nnz,)
 *   int32; live: int32 or NULL, head i is skipped when live[i * live_stride] < 0 (a back-fill
 *   pass over one window token computes only the heads that miss it); y (B, 3, H, hd);
 *   k_cache (B, H, hd/8, S, 8), v_cache (B, H, S, hd): both or neither NULL; positions: device
 *   int32, (B,) when per_sample != 0, else (1,), or NULL (= 0); rows whose position is outside
 *   [0, S) are projected but not cached.  hd in {32, 64, 128}.  y, k_cache and v_cache must
 *   be 8-byte aligned (also for dv_qkv_window_batch_f16), else DV_ERR_ALIGNMENT.
 *   workspace: dv_qkv_proj_batch_workspace_bytes(B, d, nnz, hd) bytes (0 up to 8 rows), 16-byte
 *   aligned, no initialisation needed: from 9 rows on the block of X is shared through LDS by a
 *   workgroup that owns 128 weight rows, and the columns are split over workgroups (fp32 partial
 *   sums added in ascending order by a second launch); without it every 16-row tile fetches X itself.
 */
DV_API size_t dv_qkv_proj_batch_workspace_bytes(int B, int d, int nnz, int hd);
DV_API int dv_qkv_proj_batch_f16(const void* x, int64_t ldx, const void* W, const void* bias,
                                 const void* head_idx, const void* live, int live_stride, int nnz, int B,
                                 int d, int H, int hd, void* y, void* k_cache, void* v_cache,
                                 const void* positions, int per_sample, int pos_add, int S,
                                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same projection for ALL tokens of a shared back-fill window in one pass over the weights:
 *   x row s * nseq + b is window token s (< tokens <= 16) of sequence b (< nseq <= 32), row stride ldx;
 *   batch_idx (nnz, tokens) int32: (head i, token s) is computed when batch_idx[i, s] >= 0 (the
 *   tracker's output, Dejavu/src/models/modules/mha_dejavu.py:1124-1149, 1318-1329), a head with no
 *   such token is skipped altogether;
 *   y (nseq, 3, H, hd) receives the rows of the newest token (s = tokens - 1) only;
 *   the K / V rows of every computed (head, token) go to the caches at position
 *   positions[per_sample ? b : 0] + pos_add + s.
 * It replaces one dv_qkv_proj_batch_f16 pass per window token (the reference recomputes skipped
 * K / V rows of a single sequence through qkv_proj_sparse with up to 16 rows,
 * mha_dejavu.py:1333-1352): tokens * nseq rows are multiplied against each weight tile in blocks of
 * up to 128 rows.  workspace: dv_qkv_window_batch_workspace_bytes(...) bytes, 16-byte aligned.
 */
DV_API size_t dv_qkv_window_batch_workspace_bytes(int tokens, int nseq, int d, int nnz, int hd);
DV_API int dv_qkv_window_batch_f16(const void* x, int64_t ldx, const void* W, const void* bias,
                                   const void* head_idx, const void* batch_idx, int nnz, int tokens, int nseq,
                                   int d, int H, int hd, void* y, void* k_cache, void* v_cache,
                                   const void* positions, int per_sample, int pos_add, int S,
                                   void* workspace, size_t workspace_bytes, void* stream);

/*
 * Causal attention over the prompt, and the prompt's K / V rows written into the decode caches:
 *   ctx[b, t, h, :] = softmax_{s <= t}(q[b, t, h] . k[b, s, h] * scale) . v[b, s, h]
 *   k_cache[b, h, j / 8, pos0 + t, j % 8] = k[b, t, h, j];  v_cache[b, h, pos0 + t, j] = v[b, t, h, j]
 * fp32 scores and online softmax, fp16 probabilities into the second product.  Replaces the prompt
 * branch of the attention modules: _update_kv_cache (Dejavu/src/models/modules/mha_dejavu.py:385-447,
 * the permuted cache fill) followed by causal flash attention (mha_dejavu.py:1393-1410).
 *   qkv (B, T, 3, H, hd) contiguous, the output of the Wqkv product; ctx (B, T, H * hd);
 *   k_cache (B, H, hd/8, S, 8), v_cache (B, H, S, hd): both or neither NULL, pos0 + T <= S;
 *   hd in {64, 128}.
 */
DV_API int dv_prefill_attention_f16(const void* qkv, int B, int T, int H, int hd, float scale, void* ctx,
                                    void* k_cache, void* v_cache, int pos0, int S, void* stream);

/*
 * Scatter of (re)computed keys / values into the caches:
 *   k_cache[0, h, dp, s + pad, p] = k[s, h, dp*8 + p];  v_cache[0, h, s + pad, :] = v[s, h, :]
 * for h = head_idx[i], s = seq_idx[i, slot] >= 0.  Either cache may be NULL.
 * Replaces k_cache_copy_sparse / v_cache_copy_sparse,
 * Dejavu/src/ops/triton/attention_proj_sparse.py:525-590 and 396-456.
 *   k, v (nsrc, H, hd) with row stride ld_src; k_cache (1, H, hd/8, S, 8);
 *   v_cache (1, H, S, hd); head_idx (nnz,) int32; seq_idx (nnz, nslots) int32;
 *   padding: device int32[1] or NULL (= 0).
 */
DV_API int dv_kv_cache_copy_sparse_f16(const void* k, const void* v, int64_t ld_src, int nsrc,
                                       void* k_cache, void* v_cache, const void* head_idx,
                                       const void* seq_idx, int nnz, int nslots,
                                       const void* padding, int H, int hd, int S, void* stream);

/*
 * One decode step of the skipped-head back-fill window: stores the step's
 * LayerNorm output in the 16-row window buffer, returns for every active head
 * which window tokens still lack K/V (-1 = already there) and marks them done;
 * with flush != 0 (every 16th step) every head recomputes every window token
 * and the tracker is re-armed.  Replaces ParallelTracker.get_batch_idx / update /
 * reset and the x_cache write, Dejavu/src/models/modules/mha_dejavu.py:1124-1149,
 * 1318-1329, 1355-1359.
 *   x (d,) fp16; x_cache (16, d) fp16; tracker (H, 16) int32; head_idx (nnz,)
 *   int32 (ignored when flushing); batch_idx out: (nnz, counter+1) int32, or
 *   (H, 16) when flushing; 0 <= counter <= 15.
 */
DV_API int dv_window_step_f16(const void* x, void* x_cache, int d, void* tracker,
                              const void* head_idx, int nnz, int H, int counter, int flush,
                              void* batch_idx, void* stream);

/*
 * Writes the newest token's k, v at position pos (or lengths[b]) of the caches,
 * for all heads (head_idx NULL) or the listed ones.  This is the cache update
 * that ft_attention.single_query_attention performs internally (call sites
 * Dejavu/src/models/modules/mha_dejavu.py:1045-1053, 1439-1456).
 *   k, v (B, H, hd) with batch stride ld_src; k_cache (B, H, hd/8, S, 8);
 *   v_cache (B, H, S, hd); lengths: device int32[B] or NULL.
 */
DV_API int dv_kv_append_f16(const void* k, const void* v, int64_t ld_src, void* k_cache,
                            void* v_cache, const void* head_idx, int nheads, const void* lengths,
                            int pos, int B, int H, int hd, int S, void* stream);

/*
 * One-query attention over the fp16 KV cache for the listed heads (all if
 * head_idx is NULL): out[b, h, :] = softmax(q[b, h] . K^T * scale) . V over
 * positions [0, n_len) (or [0, lengths[b]] when lengths is given; then n_len
 * is the upper bound S).  fp32 scores, softmax and accumulation.  Rows of
 * `out` for unlisted heads are not written.  Replaces the attention part of
 * ft_attention.single_query_attention (same call sites as dv_kv_append_f16).
 *   q (B, H, hd) with batch stride ldq; out (B, H, hd) with batch stride ldo;
 *   hd in {32, 64, 128}; workspace: dv_decode_attention_workspace_bytes(...) bytes.
 */
DV_API size_t dv_decode_attention_workspace_bytes(int B, int nheads, int n_len, int hd);
DV_API int dv_decode_attention_f16(const void* q, int64_t ldq, const void* k_cache,
                                   const void* v_cache, const void* head_idx, int nheads,
                                   const void* lengths, int n_len, int B, int H, int hd, int S,
                                   float scale, void* out, int64_t ldo, void* workspace,
                                   size_t workspace_bytes, void* stream);

/*
 * dv_decode_attention_f16 followed by dv_out_proj_sparse_t_f16 without
 * materialising the context: the out_proj kernel merges the attention split
 * partials while it loads its activations.  Same arithmetic (the merged
 * context is rounded to fp16 as a stored one would be; the same bits for one and two rows, where
 * dv_out_proj_sparse_t_f16 adds its partial sums in fixed point too).
 *   head_idx (nheads,) int32, required; Wt (H*hd, N) row stride ldw; y (B, N);
 *   B <= 4; workspace: dv_attention_out_proj_workspace_bytes(...) bytes, no
 *   initialisation needed.
 * dv_attention_out_proj_rows_f16 (batch 1): the same with the weight in
 *   out_proj.weight's own (N, H, hd) layout, as dv_decode_attention_f16
 *   followed by dv_out_proj_sparse_f16 (same bits).  Every output row is
 *   complete inside one wavefront, so the attention partials + one launch
 *   give y, and with residual_in / residual_out (optional, (N,)) also
 *   residual_out = fp16(y + residual_in), the residual stream advanced as
 *   Dejavu/src/models/modules/block_dejavu.py:625-631 does before norm2.
 *   workspace: dv_decode_attention_workspace_bytes(1, nheads, n_len, hd).
 */
DV_API size_t dv_attention_out_proj_workspace_bytes(int B, int nheads, int n_len, int hd, int N);
DV_API int dv_attention_out_proj_f16(const void* q, int64_t ldq, const void* k_cache,
                                     const void* v_cache, const void* head_idx, int nheads,
                                     const void* lengths, int n_len, int B, int H, int hd, int S,
                                     float scale, const void* Wt, int64_t ldw, const void* bias,
                                     int N, void* y, void* workspace, size_t workspace_bytes,
                                     void* stream);
DV_API int dv_attention_out_proj_rows_f16(const void* q, int64_t ldq, const void* k_cache,
                                          const void* v_cache, const void* head_idx, int nheads,
                                          const void* lengths, int n_len, int H, int hd, int S,
                                          float scale, const void* W, const void* bias, int N,
                                          void* y, const void* residual_in, void* residual_out,
                                          void* workspace, size_t workspace_bytes, void* stream);

/*
 * y[b, n] = sum_{h in head_idx} x[b, h, :] . W[n, h, :] + bias[n], weight in
 * out_proj.weight's own (d, H, hd) layout.  Replaces out_proj_sparse,
 * Dejavu/src/ops/triton/attention_proj_sparse.py:274-338.
 *   x (B, H, hd) contiguous, B <= 16 (passes of four rows over the weights); W (N, H, hd)
 *   contiguous; head_idx int32; hd in {32, 64, 128}.
 */
DV_API int dv_out_proj_sparse_f16(const void* x, const void* W, const void* bias,
                                  const void* head_idx, int nnz, int B, int H, int hd, int N,
                                  void* y, void* stream);

/*
 * Same result from the transposed weight Wt = W^T, (H*hd, N) with row stride
 * ldw: the active heads become contiguous row blocks that stream like the fc2
 * gather (the reference does the same for fc2 with fc2_weight_t,
 * Dejavu/src/ops/fused_dense_sparse_dejavu.py:912-913).  Deterministic.
 *   workspace: dv_out_proj_sparse_t_workspace_bytes(...) bytes, no
 *   initialisation needed (may be shared with dv_gather_transposed_gemv_f16).  y and workspace
 *   must be 16-byte aligned.
 */
DV_API size_t dv_out_proj_sparse_t_workspace_bytes(int B, int N, int nnz, int hd);
DV_API int dv_out_proj_sparse_t_f16(const void* x, const void* Wt, int64_t ldw, const void* bias,
                                    const void* head_idx, int nnz, int B, int H, int hd, int N,
                                    void* y, void* workspace, size_t workspace_bytes,
                                    void* stream);

/*
 * dv_out_proj_sparse_t_f16 for 3..64 rows followed by the block's residual add + LayerNorm 2
 * (dv_add_layer_norm_f16 with h = the projection's output) with the split reduction and the LayerNorm
 * in ONE launch: normed = LayerNorm(fp16(y + residual)) * gamma + beta, residual_out = fp16(y + residual);
 * y itself is not returned.  Same bits as the two calls (attention_proj_sparse.py:194-305 +
 * block_dejavu.py:626-634).
 *   residual (B, N) or NULL; normed, residual_out (B, N), residual_out may be NULL; N <= 32768;
 *   workspace: dv_out_proj_sparse_t_ln_workspace_bytes(...) bytes, 16-byte aligned.
 */
DV_API size_t dv_out_proj_sparse_t_ln_workspace_bytes(int B, int nnz, int hd, int N);
DV_API int dv_out_proj_sparse_t_ln_f16(const void* x, const void* Wt, int64_t ldw, const void* bias,
                                       const void* head_idx, int nnz, int B, int H, int hd, int N,
                                       const void* residual, const void* gamma, const void* beta,
                                       float eps, void* normed, void* residual_out, void* workspace,
                                       size_t workspace_bytes, void* stream);

/*
 * The two halves of that add + LayerNorm when the LayerNorm is applied by the consumer of the
 * row (the same reference lines, block_dejavu.py:575-584):
 *   dv_add_ln_parts_f16: r_out = fp16(h + residual) (h alone when residual is NULL) and, for
 *     every 64 consecutive elements of r_out, the pair (sum, sum of squared deviations from the
 *     part's own mean) as two floats: parts (ceil(d / 64), 2).  From these pairs any consumer
 *     derives mean and variance of the row in a fixed order.
 *   dv_ln_qkv_proj_sparse_cache_f16: dv_qkv_proj_sparse_cache_f16 (below the reference's
 *     qkv_proj_sparse, attention_proj_sparse.py:110-194) for window position `token` = nb - 1,
 *     whose LayerNorm row is not in the window buffer yet: every workgroup normalises r1 itself
 *     (gamma, beta, eps) from `parts`, the normalised row is also stored to x_cache[token], the
 *     other nb - 1 rows are read from x_cache.  Bit-identical to dv_add_layer_norm_f16 followed
 *     by dv_qkv_proj_sparse_cache_f16.  With nb == 1 every head of head_idx is computed (at the
 *     first window position no head has the token yet; batch_idx is not read).
 *   h, residual, r_out, r1, gamma, beta: (d,); x_cache: (16, d); d % 8 == 0, d <= 32768;
 *   hd 64 or 128; the other arguments as dv_qkv_proj_sparse_cache_f16.
 */
DV_API int dv_add_ln_parts_f16(const void* h, const void* residual, int d, void* r_out, void* parts,
                               void* stream);
DV_API int dv_ln_qkv_proj_sparse_cache_f16(const void* r1, const void* parts, const void* gamma,
                                           const void* beta, float eps, void* x_cache, int token,
                                           const void* W, const void* bias, const void* head_idx,
                                           const void* batch_idx, int nb, int d, int H, int hd, int nnz,
                                           void* y, void* k_cache, void* v_cache, const void* padding,
                                           int S, void* stream);

/*
 * Fused residual add + LayerNorm of the pre-norm block:
 *   residual_out = fp16(h + residual)   (h alone when residual is NULL)
 *   y = LayerNorm(residual_out) * gamma + beta, fp32 statistics, fp16 out.
 * Replaces the unfused dropout(p=0) + add + nn.LayerNorm of
 * Dejavu/src/models/modules/block_dejavu.py:575-584 and 626-634 (and the
 * dropout_add_layer_norm extension call at :596-606, :648-658).
 *   h, residual, y, residual_out: (rows, d) contiguous; gamma, beta (d,);
 *   residual_out may be NULL; d % 8 == 0, d <= 32768.
 */
DV_API int dv_add_layer_norm_f16(const void* h, const void* residual, const void* gamma,
                                 const void* beta, float eps, int rows, int d, void* y,
                                 void* residual_out, void* stream);

/*
 * dv_add_layer_norm_f16 and dv_window_step_f16 in one launch, for `rows` sequences that share a
 * back-fill window: the normalised rows also go to x_cache_row (rows, d) -- the row of the window
 * buffer that belongs to this step (x_cache + counter * rows * d) -- and one more workgroup runs the
 * tracker step (block_dejavu.py:575-584 + mha_dejavu.py:1124-1149, 1318-1329).  Same outputs as the
 * two separate calls.  Arguments as there; x_cache_row 16-byte aligned.
 */
DV_API int dv_add_layer_norm_window_f16(const void* h, const void* residual, const void* gamma,
                                        const void* beta, float eps, int rows, int d, void* y,
                                        void* residual_out, void* x_cache_row, void* tracker,
                                        const void* head_idx, int nnz, int H, int counter, int flush,
                                        void* batch_idx, void* stream);

/*
 * The fc2 of one block and LayerNorm 1 of the next without a reduction launch of their own, for
 * 3..64 rows (the matrix-core path of dv_gather_transposed_gemv_f16):
 *  - dv_gather_transposed_gemv_partial_f16 is dv_gather_transposed_gemv_f16 (gather_gemv.py:572-644)
 *    without its last step: the fp32 sums of the row groups stay in `partial` (layout private to the
 *    library), their number goes to *groups (host memory).  *groups == 1: there was nothing to split,
 *    y (B, N) is complete and `partial` unused; otherwise y is not written.
 *      partial: dv_gather_transposed_gemv_partial_workspace_bytes(B, N, M) bytes, 16-byte aligned,
 *      left alone until one of the two consumers below has run.
 *  - dv_reduce_rows_f16 is the last step alone: y = fp16(sum of the groups + bias); a no-op for groups == 1.
 *  - dv_reduce_add_layer_norm_window_f16 is that step, the residual add and the LayerNorm that follow the
 *    MLP in the next block (block_dejavu.py:575-584) and, with tracker != NULL, the window step of the
 *    same position (dv_add_layer_norm_window_f16; mha_dejavu.py:1124-1149, 1318-1329) in ONE launch.
 *    h: the complete rows, read instead of `partial` when groups == 1.  tracker == NULL: no window step,
 *    x_cache_row .. batch_idx unused.  Other arguments as dv_add_layer_norm_window_f16.
 * Same bits as dv_gather_transposed_gemv_f16 followed by dv_add_layer_norm(_window)_f16.
 */
DV_API size_t dv_gather_transposed_gemv_partial_workspace_bytes(int B, int N, int M);
DV_API int dv_gather_transposed_gemv_partial_f16(const void* x, const void* W, int64_t ldw,
                                                 const void* bias, const void* idx, int idx_bytes, int B,
                                                 int N, int Z, int M, void* y, void* partial,
                                                 size_t partial_bytes, int* groups, void* stream);
DV_API int dv_reduce_rows_f16(const void* partial, int groups, const void* bias, int rows, int N,
                              void* y, void* stream);
DV_API int dv_reduce_add_layer_norm_window_f16(const void* partial, int groups, const void* bias,
                                               const void* h, const void* residual, const void* gamma,
                                               const void* beta, float eps, int rows, int d, void* y,
                                               void* residual_out, void* x_cache_row, void* tracker,
                                               const void* head_idx, int nnz, int H, int counter,
                                               int flush, void* batch_idx, void* stream);

/*
 * Greedy step of the generation loop (batch 1): next = argmax(logits[0 .. vocab)), first index
 * among equal values; then, all on the device so that a captured step can be replayed:
 * token[0] = next, sequences[out_index[0]++] = next, position[0]++, seq_pos[0]++ and, with
 * scores != NULL, scores[score_index[0]++, :vocab] = logits (rows of score_ld elements).
 * The two stores are skipped (the counters still advance) once out_index[0] reaches seq_capacity
 * or score_index[0] reaches score_rows: a replayed step cannot write past the buffers.
 * Replaces the sampling step of the greedy loop the reference takes from flash-attention v0.2.8
 * utils/generation.py (decode(): `sample(logits, top_k=1)` + sequence / length bookkeeping;
 * call site Dejavu/benchmarks/benchmark_generation_opt_dejavu.py:187-196).
 *   logits fp16; token, position, out_index, score_index int64[1]; seq_pos int32[1];
 *   sequences int64 (row of the output); scores fp16 or NULL.
 */
DV_API int dv_greedy_advance_f16(const void* logits, int vocab, void* token, void* position,
                                 void* seq_pos, void* sequences, int64_t seq_capacity, void* out_index,
                                 void* scores, int64_t score_ld, int64_t score_rows, void* score_index,
                                 void* stream);

/*
 * One decode step (batch 1, one new token) of a whole sparse block in eight
 * launches: add+LayerNorm 1, back-fill window step, QKV of the active heads with
 * cache scatter, attention, out_proj, add+LayerNorm 2, the sparse MLP, and beside
 * them the MLP top-k for this layer and both predictors (+ head top-k) for the
 * next layer.  Same arithmetic, kernel bodies and results as the separate entry
 * points called in the order of BlockMlpAttSparse.forward,
 * Dejavu/src/models/modules/block_dejavu.py:555-663 (mixer:
 * Dejavu/src/models/modules/mha_dejavu.py:1283-1511, mlp:
 * Dejavu/src/ops/fused_dense_sparse_dejavu.py:889-951).
 * The step that flushes the window (counter 15: every 16th token, all heads and
 * all 16 tokens, mha_dejavu.py:1320-1326) is taken with head_idx = 0..H-1 and
 * Hk = H.
 */
typedef struct dvSparseLayerArgs {
  /* shapes */
  int d, ffn, H, hd;      /* hidden, MLP width, heads, head_dim (64 or 128)            */
  int r_att, r_mlp;       /* predictor ranks                                           */
  int K, Hk, att_k;       /* active neurons; heads computed now; heads predicted next  */
  int S;                  /* KV cache capacity                                         */
  int counter;            /* window position of this token, 0..15 (15: flush, Hk == H) */
  int n_len;              /* cached positions to attend, newest token included         */
  int advance_window;     /* flush step only: != 0 adds 16 to cache_offset[0] once the  */
                          /* window's K/V rows are in the caches (the next window)      */
  float eps1, eps2, softmax_scale;
  /* inputs (device, fp16 unless stated) */
  const void* hidden;     /* (d,) output of the previous block's MLP                   */
  const void* residual;   /* (d,) residual stream, or NULL for the first block         */
  const void *ln1_w, *ln1_b, *ln2_w, *ln2_b;
  const void* Wqkv;       /* (3, H, hd, d)                                             */
  const void* bqkv;       /* (3, H, hd) or NULL                                        */
  const void* Wout_t;     /* (H*hd, d): out_proj.weight transposed                     */
  const void* bout;       /* (d,) or NULL                                              */
  const void *att_Wa, *att_Wb; /* (r_att, d), (H, r_att)                               */
  const void *W1, *b1;    /* (ffn, d), (ffn,) or NULL                                  */
  const void *W2t, *b2;   /* (ffn, d): fc2.weight transposed; (d,) or NULL             */
  const void *mlp_Wa, *mlp_Wb; /* (r_mlp, d), (ffn, r_mlp)                             */
  const void* head_idx;   /* (Hk,) int32 heads to compute                              */
  const void* mlp_logit_in; /* (ffn,) predictor logits for THIS layer's MLP            */
  void* cache_offset;     /* int32[1]: cache position of window token 0 (see advance_window) */
  const void* seq_pos;    /* int32[1] cache position of the newest token, or NULL: when   */
                          /* given it replaces n_len - 1, so that a captured launch     */
                          /* sequence can be replayed as the sequence grows (the role of */
                          /* lengths_per_sample, mha_dejavu.py:1439-1446)                */
  /* state, updated in place */
  void *k_cache, *v_cache; /* (1, H, hd/8, S, 8), (1, H, S, hd)                        */
  void* x_cache;          /* (16, d) LayerNorm-1 outputs of the window                 */
  void* tracker;          /* (H, 16) int32                                             */
  /* outputs */
  void* hidden_out;       /* (d,) MLP output                                           */
  void* residual_out;     /* (d,) residual stream after attention                      */
  void* mlp_logit_out;    /* (ffn,) logits for the NEXT layer's MLP                    */
  void* att_idx_out;      /* (att_k,) int32 heads for the NEXT layer                   */
  void* mlp_idx_out;      /* (K,) int64 neurons used by this layer                     */
  /* scratch: dv_sparse_layer_workspace_bytes() bytes, no initialisation needed */
  void* workspace;
  size_t workspace_bytes;
} dvSparseLayerArgs;

DV_API size_t dv_sparse_layer_workspace_bytes(const dvSparseLayerArgs* args);
DV_API int dv_sparse_layer_decode_f16(const dvSparseLayerArgs* args, void* stream);

/*
 * The same step for n_layers consecutive blocks of a model, the loop over the layers of
 * GPTModel.forward (Dejavu/src/models/gpt_dejavu.py:595-612) for one decode token:
 * block l + 1 takes (hidden_out, residual_out) of block l, whatever its own `hidden` /
 * `residual` say (they may be NULL for l > 0).  Equivalent to n_layers calls of
 * dv_sparse_layer_decode_f16, bit for bit, but the launch that finishes block l's MLP
 * output also does the residual add, the LayerNorm statistics, the key histogram and the
 * window step of block l + 1 (six launches per block instead of seven).
 * All blocks share d, ffn and H; the scratch is layers[0].workspace, at least the largest
 * dv_sparse_layer_workspace_bytes() of the blocks (the other blocks' workspace fields are
 * not read).  Every block's outputs are stored as documented above.  The predictions a
 * block consumes must be complete when its turn comes: buffers written by the block
 * before it (mlp_logit_out / att_idx_out of block l as mlp_logit_in / head_idx of block
 * l + 1) or by earlier work on the stream.
 */
DV_API int dv_sparse_layers_decode_f16(const dvSparseLayerArgs* layers, int n_layers, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DEJAVU_HIP_H */
