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
 *   hidden (B, r) scratch/output; logits (B, n_out).  1 <= B <= 8.
 */
DV_API int dv_predictor_logits_f16(const void* x, const void* Wa, int64_t ldwa, const void* Wb,
                            int64_t ldwb, int B, int d, int r, int n_out, void* hidden,
                            void* logits, void* stream);

/*
 * Index set of the k largest logits, ties to the lower index, written in
 * ascending index order.  For B > 1 a column's score is its maximum over the
 * B rows.  Replaces Tensor.topk(k, sorted=False) at
 * Dejavu/src/models/modules/mha_dejavu.py:1069, 1369, 1506-1507.
 *   logits (B, n) fp16; idx_out (k,) int32/int64.  n <= 65536, 0 <= k <= n.
 */
DV_API int dv_topk_f16(const void* logits, int B, int n, int k, void* idx_out, int idx_bytes,
                void* stream);

/*
 * y = act(x . W[idx]^T + bias[idx]).  Replaces gather_gemv,
 * Dejavu/src/ops/triton/gather_gemv.py:198-254.
 *   x (B, N); W (Z, N) row stride ldw; bias (Z,) or NULL; idx (M,);
 *   y (B, M) fp16.  1 <= B <= 4 (the reference's own limit).
 */
DV_API int dv_gather_gemv_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                       const void* idx, int idx_bytes, int B, int N, int Z, int M, int act,
                       void* y, void* stream);

/*
 * y = x . W[idx] + bias.  Replaces gather_transposed_gemv,
 * Dejavu/src/ops/triton/gather_gemv.py:572-644 (deterministic: fixed-order
 * split over row groups instead of floating-point atomics).
 *   x (B, M); W (Z, N) row stride ldw; bias (N,) or NULL; idx (M,);
 *   y (B, N) fp16.  1 <= B <= 4.
 *   workspace: dv_gather_transposed_gemv_workspace_bytes(B, N, M) bytes,
 *   zero-filled before its first use; calls sharing it must not overlap.
 */
DV_API size_t dv_gather_transposed_gemv_workspace_bytes(int B, int N, int M);
DV_API int dv_gather_transposed_gemv_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                                  const void* idx, int idx_bytes, int B, int N, int Z, int M,
                                  void* y, void* workspace, size_t workspace_bytes,
                                  void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DEJAVU_HIP_H */
