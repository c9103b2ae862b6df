// C ABI of libdejavu_hip.so (see include/dejavu_hip.h): argument checks on the
// host, then kernel launches on the caller's stream.  No allocation, no
// synchronisation.
#include "../../include/dejavu_hip.h"

#include <hip/hip_runtime.h>

#include "common.hpp"
#include "gemv_cols.hpp"
#include "gemv_rows.hpp"
#include "topk.hpp"

using namespace dv;

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool idx_ok(int idx_bytes) { return idx_bytes == 4 || idx_bytes == 8; }

inline int launch_status() { return hipGetLastError() == hipSuccess ? DV_OK : DV_ERR_LAUNCH; }

int compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      cus = v;
    else
      cus = 256;
  }
  return cus;
}

// ---- canonical (predictor) GEMV -------------------------------------------
template <int LANES, int U>
int launch_canonical(const half_t* X, const half_t* W, int64_t ldw, int B, int rows, int n,
                     half_t* Y, hipStream_t s) {
  constexpr int RW = kWave / LANES;
  const int ntasks = (rows + RW - 1) / RW;
  int blocks = (ntasks + 3) / 4;
  const int cap = compute_units() * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
#define DV_CASE(BB)                                                                            \
  case BB:                                                                                     \
    hipLaunchKernelGGL((canonical_gemv_kernel<LANES, BB, U>), dim3(blocks), dim3(256), 0, s, X, \
                       W, ldw, rows, n, Y);                                                    \
    break;
  switch (B) {
    DV_CASE(1) DV_CASE(2) DV_CASE(3) DV_CASE(4) DV_CASE(5) DV_CASE(6) DV_CASE(7) DV_CASE(8)
    default:
      return DV_ERR_UNSUPPORTED;
  }
#undef DV_CASE
  return launch_status();
}

int canonical_gemv(const half_t* X, const half_t* W, int64_t ldw, int B, int rows, int n,
                   half_t* Y, hipStream_t s) {
  if (dv_canonical_lanes(n) == 16) return launch_canonical<16, 8>(X, W, ldw, B, rows, n, Y, s);
  return launch_canonical<64, 8>(X, W, ldw, B, rows, n, Y, s);
}

// ---- gathered row GEMV (fc1) ----------------------------------------------
template <int B, int R, int U, bool RELU>
int launch_gather_rows(const half_t* x, const half_t* W, int64_t ldw, const half_t* bias,
                       const void* idx, int idx_bytes, int N, int Z, int M, half_t* y,
                       hipStream_t s) {
  auto kern = gather_rows_kernel<B, R, U, RELU>;
  const size_t lds = (size_t)B * N * sizeof(half_t);
  if (lds > 160 * 1024) return DV_ERR_UNSUPPORTED;
  static size_t lds_granted = 48 * 1024;
  if (lds > lds_granted) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return DV_ERR_UNSUPPORTED;
    lds_granted = lds;
  }
  const int ntasks = (M + R - 1) / R;
  int blocks = (ntasks + 3) / 4;
  const int cap = compute_units() * 8;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds, s, x, W, bias, idx, idx_bytes, N, ldw, Z,
                     M, y);
  return launch_status();
}

template <int B>
int gather_rows_b(const half_t* x, const half_t* W, int64_t ldw, const half_t* bias,
                  const void* idx, int idx_bytes, int N, int Z, int M, int act, half_t* y,
                  hipStream_t s) {
  constexpr int R = B <= 2 ? 2 : 1;
  if (act == DV_ACT_RELU)
    return launch_gather_rows<B, R, 4, true>(x, W, ldw, bias, idx, idx_bytes, N, Z, M, y, s);
  return launch_gather_rows<B, R, 4, false>(x, W, ldw, bias, idx, idx_bytes, N, Z, M, y, s);
}

// ---- gathered column GEMV (fc2 / out_proj over transposed weights) ----------
struct ColsPlan {
  int col_tiles, groups, rows_per_block;
};

ColsPlan plan_cols(int N, int M) {
  ColsPlan p;
  p.col_tiles = (N + kColTile - 1) / kColTile;
  const int target_blocks = compute_units() * 6;
  int groups = (target_blocks + p.col_tiles - 1) / p.col_tiles;
  int max_groups = (M + 15) / 16;  // at least 16 rows per workgroup
  if (max_groups < 1) max_groups = 1;
  if (groups > max_groups) groups = max_groups;
  if (groups < 1) groups = 1;
  int rpb = (M + groups - 1) / groups;
  rpb = (rpb + 3) & ~3;
  if (rpb < 4) rpb = 4;
  p.rows_per_block = rpb;
  p.groups = (M + rpb - 1) / rpb;
  if (p.groups < 1) p.groups = 1;
  return p;
}

size_t cols_workspace_bytes(int B, int N, int M) {
  const ColsPlan p = plan_cols(N, M);
  size_t partial = (size_t)p.groups * B * N * sizeof(float);
  partial = (partial + 255) & ~(size_t)255;
  return partial + (size_t)p.col_tiles * sizeof(unsigned);
}

int gather_cols(const half_t* x, int64_t ldx, int x_expanded, const half_t* W, int64_t ldw,
                const half_t* bias, const void* idx, int idx_bytes, int blk, int B, int N, int Z,
                int M, half_t* y, void* workspace, size_t workspace_bytes, hipStream_t s) {
  const ColsPlan p = plan_cols(N, M);
  if (workspace == nullptr || workspace_bytes < cols_workspace_bytes(B, N, M))
    return DV_ERR_WORKSPACE;
  size_t partial_bytes = (size_t)p.groups * B * N * sizeof(float);
  partial_bytes = (partial_bytes + 255) & ~(size_t)255;
  float* partial = reinterpret_cast<float*>(workspace);
  unsigned* counters =
      reinterpret_cast<unsigned*>(reinterpret_cast<unsigned char*>(workspace) + partial_bytes);
  dim3 grid(p.col_tiles, p.groups);
#define DV_CASE(BB)                                                                               \
  case BB:                                                                                        \
    hipLaunchKernelGGL((gather_cols_kernel<BB, 8>), grid, dim3(256), 0, s, x, ldx, x_expanded, W, \
                       ldw, bias, idx, idx_bytes, blk, N, Z, M, p.rows_per_block, partial,        \
                       counters, y);                                                              \
    break;
  switch (B) {
    DV_CASE(1) DV_CASE(2) DV_CASE(3) DV_CASE(4)
    default:
      return DV_ERR_UNSUPPORTED;
  }
#undef DV_CASE
  return launch_status();
}

}  // namespace

extern "C" {

int dv_version(void) { return 100; }

const char* dv_error_string(int code) {
  switch (code) {
    case DV_OK: return "ok";
    case DV_ERR_INVALID_ARG: return "invalid argument";
    case DV_ERR_UNSUPPORTED: return "unsupported shape";
    case DV_ERR_ALIGNMENT: return "pointer, size or stride not a multiple of 8 elements";
    case DV_ERR_WORKSPACE: return "workspace missing or too small";
    case DV_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown error";
  }
}

int dv_canonical_lanes(int n) { return n <= 1024 ? 16 : 64; }

int dv_predictor_logits_f16(const void* x, const void* Wa, int64_t ldwa, const void* Wb,
                            int64_t ldwb, int B, int d, int r, int n_out, void* hidden,
                            void* logits, void* stream) {
  if (!x || !Wa || !Wb || !hidden || !logits || d <= 0 || r <= 0 || n_out <= 0)
    return DV_ERR_INVALID_ARG;
  if (B < 1 || B > 8) return DV_ERR_UNSUPPORTED;
  if (d % 8 || r % 8 || ldwa % 8 || ldwb % 8 || ldwa < d || ldwb < r || !aligned16(x) ||
      !aligned16(Wa) || !aligned16(Wb) || !aligned16(hidden))
    return DV_ERR_ALIGNMENT;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  int rc = canonical_gemv(reinterpret_cast<const half_t*>(x), reinterpret_cast<const half_t*>(Wa),
                          ldwa, B, r, d, reinterpret_cast<half_t*>(hidden), s);
  if (rc != DV_OK) return rc;
  return canonical_gemv(reinterpret_cast<const half_t*>(hidden),
                        reinterpret_cast<const half_t*>(Wb), ldwb, B, n_out, r,
                        reinterpret_cast<half_t*>(logits), s);
}

int dv_topk_f16(const void* logits, int B, int n, int k, void* idx_out, int idx_bytes,
                void* stream) {
  if (!logits || B < 1 || n < 1 || k < 0 || k > n || !idx_ok(idx_bytes) || (k > 0 && !idx_out))
    return DV_ERR_INVALID_ARG;
  if (n > 65536) return DV_ERR_UNSUPPORTED;
  if (k == 0) return DV_OK;
  if (n % 8 == 0 && !aligned16(logits)) return DV_ERR_ALIGNMENT;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const half_t* lg = reinterpret_cast<const half_t*>(logits);
#define DV_TOPK(T, I, V)                                                                      \
  hipLaunchKernelGGL((topk_kernel<T, I, V>), dim3(1), dim3(T), 0, s, lg, B, n, k, idx_out, \
                     idx_bytes)
  if (n % 8 != 0) {
    // scalar-load variant, small inputs only (e.g. 12 or 20 attention heads)
    if (n > 1024 * 8) return DV_ERR_UNSUPPORTED;
    if (n <= 64 * 8)
      DV_TOPK(64, 8, false);
    else
      DV_TOPK(1024, 8, false);
  } else if (n <= 64 * 8)
    DV_TOPK(64, 8, true);
  else if (n <= 256 * 8)
    DV_TOPK(256, 8, true);
  else if (n <= 1024 * 8)
    DV_TOPK(1024, 8, true);
  else if (n <= 1024 * 16)
    DV_TOPK(1024, 16, true);
  else if (n <= 1024 * 24)
    DV_TOPK(1024, 24, true);
  else if (n <= 1024 * 32)
    DV_TOPK(1024, 32, true);
  else if (n <= 1024 * 40)
    DV_TOPK(1024, 40, true);
  else if (n <= 1024 * 48)
    DV_TOPK(1024, 48, true);
  else
    DV_TOPK(1024, 64, true);
#undef DV_TOPK
  return launch_status();
}

int dv_gather_gemv_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                       const void* idx, int idx_bytes, int B, int N, int Z, int M, int act,
                       void* y, void* stream) {
  if (!x || !W || !idx || !y || N <= 0 || Z <= 0 || M < 0 || !idx_ok(idx_bytes) ||
      (act != DV_ACT_ID && act != DV_ACT_RELU))
    return DV_ERR_INVALID_ARG;
  if (B < 1 || B > 4) return DV_ERR_UNSUPPORTED;
  if (N % 8 || ldw % 8 || ldw < N || !aligned16(x) || !aligned16(W)) return DV_ERR_ALIGNMENT;
  if (M == 0) return DV_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const half_t* xx = reinterpret_cast<const half_t*>(x);
  const half_t* ww = reinterpret_cast<const half_t*>(W);
  const half_t* bb = reinterpret_cast<const half_t*>(bias);
  half_t* yy = reinterpret_cast<half_t*>(y);
  switch (B) {
    case 1: return gather_rows_b<1>(xx, ww, ldw, bb, idx, idx_bytes, N, Z, M, act, yy, s);
    case 2: return gather_rows_b<2>(xx, ww, ldw, bb, idx, idx_bytes, N, Z, M, act, yy, s);
    case 3: return gather_rows_b<3>(xx, ww, ldw, bb, idx, idx_bytes, N, Z, M, act, yy, s);
    default: return gather_rows_b<4>(xx, ww, ldw, bb, idx, idx_bytes, N, Z, M, act, yy, s);
  }
}

size_t dv_gather_transposed_gemv_workspace_bytes(int B, int N, int M) {
  if (B < 1 || N < 1 || M < 0) return 0;
  return cols_workspace_bytes(B, N, M);
}

int dv_gather_transposed_gemv_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                                  const void* idx, int idx_bytes, int B, int N, int Z, int M,
                                  void* y, void* workspace, size_t workspace_bytes,
                                  void* stream) {
  if (!x || !W || !y || N <= 0 || Z <= 0 || M < 0 || !idx_ok(idx_bytes) || (M > 0 && !idx))
    return DV_ERR_INVALID_ARG;
  if (B < 1 || B > 4) return DV_ERR_UNSUPPORTED;
  if (N % 8 || ldw % 8 || ldw < N || !aligned16(W)) return DV_ERR_ALIGNMENT;
  return gather_cols(reinterpret_cast<const half_t*>(x), M, 0, reinterpret_cast<const half_t*>(W),
                     ldw, reinterpret_cast<const half_t*>(bias), idx, idx_bytes, 1, B, N, Z, M,
                     reinterpret_cast<half_t*>(y), workspace, workspace_bytes,
                     reinterpret_cast<hipStream_t>(stream));
}

}  // extern "C"
