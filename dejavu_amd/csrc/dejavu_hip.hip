// C ABI of libdejavu_hip.so (see include/dejavu_hip.h): argument checks on the
// host, then kernel launches on the caller's stream.  No allocation, no
// synchronisation.
#include "../../include/dejavu_hip.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <stdlib.h>

#include "attention.hpp"
#include "common.hpp"
#include "gemm_cols16.hpp"
#include "gemm_mfma.hpp"
#include "gemm_tiled.hpp"
#include "gemm_big.hpp"
#include "gemv_cols.hpp"
#include "gemv_rows.hpp"
#include "layer_fused.hpp"
#include "norm.hpp"
#include "prefill.hpp"
#include "qkv_mfma.hpp"
#include "topk.hpp"

using namespace dv;

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }  // null passes
inline bool idx_ok(int idx_bytes) { return idx_bytes == 4 || idx_bytes == 8; }

inline int launch_status() { return hipGetLastError() == hipSuccess ? DV_OK : DV_ERR_LAUNCH; }

constexpr int kMaxDevices = 64;

int current_device() {
  int dev = 0;
  return (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices) ? dev : -1;
}

// Compute units of the current device (remembered per device).
int compute_units() {
  static std::atomic<int> cus[kMaxDevices];
  const int dev = current_device();
  if (dev < 0) return 256;
  int v = cus[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cus[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

// Dynamic LDS above 48 KiB has to be granted per kernel and per device.  One object per kernel
// (static storage: starts at zero) remembers the largest size granted on each device, so a steady
// stream of calls asks the runtime for nothing but the current device.
struct LdsGrant {
  std::atomic<size_t> granted[kMaxDevices];
  int ensure(const void* fn, size_t bytes) {
    if (bytes <= 48 * 1024) return DV_OK;
    if (bytes > 160 * 1024) return DV_ERR_UNSUPPORTED;
    const int dev = current_device();
    if (dev < 0) return DV_ERR_UNSUPPORTED;
    if (bytes <= granted[dev].load(std::memory_order_relaxed)) return DV_OK;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
      return DV_ERR_UNSUPPORTED;
    granted[dev].store(bytes, std::memory_order_relaxed);
    return DV_OK;
  }
};

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
  // short rows (n <= 1024: X fits LDS as fp32): X in LDS, R weight rows per lane group.  Measured at
  // the OPT-175B predictor (49152 rows of 1000): batch 1, R = 2: 18 us against 22 us with one row per
  // group; batch 4: 98 us per MLP block with R = 1 against 102 us with R = 4; batch 8: 122 against 121.
  const size_t xlds = (size_t)B * n * sizeof(float);
  const bool use_xlds = LANES == 16 && xlds <= 48 * 1024;
  // Few rows (the head predictor's second product: 96 rows): one row per lane group, so that the rows
  // spread over as many wavefronts as possible (16 us -> a few us at batch 8: four rows per group left
  // six wavefronts with long dependent chains).
  const bool few_rows = B >= 5 && rows < RW * 4 * 4 * compute_units();
  const int xr = B >= 5 ? (few_rows ? 1 : 4) : (B == 1 ? 2 : 1);
  if (use_xlds) {
    blocks = ((rows + RW * xr - 1) / (RW * xr) + 3) / 4;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
  }
#define DV_CASE(BB)                                                                                \
  case BB:                                                                                         \
    if (use_xlds && few_rows)                                                                      \
      hipLaunchKernelGGL((canonical_gemv_xlds_kernel<LANES, BB, (BB >= 5 ? 4 : 8), 1>), dim3(blocks), \
                         dim3(256), xlds, s, X, W, ldw, rows, n, Y);                               \
    else if (use_xlds)                                                                             \
      hipLaunchKernelGGL((canonical_gemv_xlds_kernel<LANES, BB, (BB >= 5 ? 4 : 8), (BB >= 5 ? 4 : (BB == 1 ? 2 : 1))>), dim3(blocks), \
                         dim3(256), xlds, s, X, W, ldw, rows, n, Y);                               \
    else                                                                                           \
      hipLaunchKernelGGL((canonical_gemv_kernel<LANES, BB, U>), dim3(blocks), dim3(256), 0, s, X, W, ldw, rows, n, \
                         Y);                                                                       \
    break;
  switch (B) {
    DV_CASE(1) DV_CASE(2) DV_CASE(3) DV_CASE(4) DV_CASE(5) DV_CASE(6) DV_CASE(7) DV_CASE(8)
    default:
      return DV_ERR_UNSUPPORTED;
  }
#undef DV_CASE
  return launch_status();
}

// Long rows, three or more batch rows: the slices kernel (X shared through LDS); same bits.
template <int B>
int launch_canonical_slices(const half_t* X, const half_t* W, int64_t ldw, int rows, int n, half_t* Y,
                            hipStream_t s) {
  const size_t lds = (size_t)2 * B * kCanonSlice * sizeof(half_t);
  static LdsGrant grant;
  if (int rc = grant.ensure(reinterpret_cast<const void*>(canonical_gemv_slices_kernel<B>), lds); rc != DV_OK)
    return rc;
  int blocks = (rows + 3) / 4;
  const int cap = compute_units() * 4;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL((canonical_gemv_slices_kernel<B>), dim3(blocks), dim3(256), lds, s, X, W, ldw, rows, n, Y);
  return launch_status();
}

int canonical_gemv(const half_t* X, const half_t* W, int64_t ldw, int B, int rows, int n,
                   half_t* Y, hipStream_t s) {
  if (dv_canonical_lanes(n) == 16) return launch_canonical<16, 8>(X, W, ldw, B, rows, n, Y, s);
  switch (B) {  // measured at the OPT-175B predictor (1000 rows of 12288): see the kernel's header
    case 3: return launch_canonical_slices<3>(X, W, ldw, rows, n, Y, s);
    case 4: return launch_canonical_slices<4>(X, W, ldw, rows, n, Y, s);
    case 5: return launch_canonical_slices<5>(X, W, ldw, rows, n, Y, s);
    case 6: return launch_canonical_slices<6>(X, W, ldw, rows, n, Y, s);
    case 7: return launch_canonical_slices<7>(X, W, ldw, rows, n, Y, s);
    case 8: return launch_canonical_slices<8>(X, W, ldw, rows, n, Y, s);
    default: break;
  }
  return launch_canonical<64, 8>(X, W, ldw, B, rows, n, Y, s);
}

// ---- gathered row GEMV (fc1) ----------------------------------------------
template <int B, int R, int U, bool RELU>
int launch_gather_rows(const half_t* x, const half_t* W, int64_t ldw, const half_t* bias,
                       const void* idx, int idx_bytes, int N, int Z, int M, half_t* y, int act,
                       hipStream_t s) {
  auto kern = gather_rows_kernel<B, R, U, RELU>;
  const size_t lds = (size_t)B * N * sizeof(half_t);
  static LdsGrant grant;
  if (int rc = grant.ensure(reinterpret_cast<const void*>(kern), lds); rc != DV_OK) return rc;
  const int ntasks = (M + R - 1) / R;
  int blocks = (ntasks + 3) / 4;
  const int cap = compute_units() * 8;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds, s, x, W, bias, idx, idx_bytes, N, ldw, Z,
                     M, y, act);
  return launch_status();
}

template <int B>
int gather_rows_b(const half_t* x, const half_t* W, int64_t ldw, const half_t* bias,
                  const void* idx, int idx_bytes, int N, int Z, int M, int act, half_t* y,
                  hipStream_t s) {
  constexpr int R = B <= 2 ? 2 : 1;
  if (act != DV_ACT_ID)
    return launch_gather_rows<B, R, 4, true>(x, W, ldw, bias, idx, idx_bytes, N, Z, M, y, act, s);
  return launch_gather_rows<B, R, 4, false>(x, W, ldw, bias, idx, idx_bytes, N, Z, M, y, act, s);
}

// ---- gathered column GEMV (fc2 / out_proj over transposed weights) ----------
struct ColsPlan {
  int col_tiles, groups, rows_per_block;
};

// Three workgroups per compute unit measured best for the split over gathered
// rows; the partial sums are combined by a second, deterministic pass.
constexpr int kColsBlocksPerCu = 3;

ColsPlan plan_cols(int N, int M) {
  ColsPlan p;
  p.col_tiles = (N + kColTile - 1) / kColTile;
  const int target_blocks = compute_units() * kColsBlocksPerCu;
  int groups = (target_blocks + p.col_tiles - 1) / p.col_tiles;
  // At least 64 rows per workgroup (two full batches of 8 per wavefront): at the smaller shapes
  // three workgroups per compute unit would leave each with a handful of rows.  Measured, whole
  // layer, window start: OPT-13B 61.1 us and OPT-6.7B 61.5 us instead of 66.2 / 68.8 us with 16
  // rows as the floor; with 128 rows OPT-66B gains 3 us more but OPT-13B (10 column tiles: only
  // 160 workgroups) loses 2.5 us.  The OPT-175B layer has 128 rows per workgroup either way.
  int max_groups = (M + 63) / 64;
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

// Workspace: the fp32 partial sums of the row groups, (groups, B, N).  Every word a call reads
// it has written first, so the memory needs no initialisation.
size_t cols_workspace_bytes(int B, int N, int M) {
  const ColsPlan p = plan_cols(N, M);
  return (size_t)p.groups * B * N * sizeof(float);
}

// fixed: the row groups' partial sums are added in fixed point (also with a single group), the form
// the fused layer step uses for out_proj; else in fp32 in a fixed order (fc2)
template <int B, bool IDX64, bool BLOCKED>
void launch_cols(const ColsPlan& p, const half_t* x, int64_t ldx, int x_expanded, const half_t* W,
                 int64_t ldw, const half_t* bias, const void* idx, int blk, int N, int Z, int M,
                 float* partial, half_t* y, bool fixed, hipStream_t s) {
  dim3 grid(p.col_tiles, p.groups);
  hipLaunchKernelGGL((gather_cols_kernel<B, 8, IDX64, BLOCKED>), grid, dim3(256), 0, s, x, ldx, x_expanded, W, ldw,
                     bias, idx, blk, N, Z, M, p.rows_per_block, partial, y, (const float*)nullptr, 0, fixed ? 1 : 0);
  const int64_t total = (int64_t)B * N;
  if (fixed)
    hipLaunchKernelGGL(cols_reduce_kernel<true>, dim3((unsigned)((total + 63) / 64)), dim3(256), 0, s, partial, bias,
                       p.groups, B, N, y, (const half_t*)nullptr, (half_t*)nullptr);
  else if (p.groups > 1)
    hipLaunchKernelGGL(cols_reduce_kernel<false>, dim3((unsigned)((total + 63) / 64)), dim3(256), 0, s,
                       partial, bias, p.groups, B, N, y, (const half_t*)nullptr, (half_t*)nullptr);
}

int gather_cols(const half_t* x, int64_t ldx, int x_expanded, const half_t* W, int64_t ldw,
                const half_t* bias, const void* idx, int idx_bytes, int blk, int B, int N, int Z,
                int M, half_t* y, void* workspace, size_t workspace_bytes, hipStream_t s, bool fixed = false) {
  const ColsPlan p = plan_cols(N, M);
  if (workspace == nullptr || workspace_bytes < cols_workspace_bytes(B, N, M))
    return DV_ERR_WORKSPACE;
  float* partial = reinterpret_cast<float*>(workspace);
#define DV_ARGS p, x, ldx, x_expanded, W, ldw, bias, idx, blk, N, Z, M, partial, y, fixed, s
#define DV_CASE(BB)                                                   \
  case BB:                                                            \
    if (blk == 1) {                                                   \
      if (idx_bytes == 8) launch_cols<BB, true, false>(DV_ARGS);      \
      else launch_cols<BB, false, false>(DV_ARGS);                    \
    } else {                                                          \
      if (idx_bytes == 8) launch_cols<BB, true, true>(DV_ARGS);       \
      else launch_cols<BB, false, true>(DV_ARGS);                     \
    }                                                                 \
    break;
  switch (B) {
    DV_CASE(1) DV_CASE(2) DV_CASE(3) DV_CASE(4)
    default:
      return DV_ERR_UNSUPPORTED;
  }
#undef DV_CASE
#undef DV_ARGS
  return launch_status();
}

// Largest batch the vector-ALU kernels take; above it the MFMA kernels are faster (measured at
// the OPT-175B shape: fc1 19 us on MFMA against 24 / 39 us at batch 3 / 4; fc2 alone 22-24 us on the
// vector ALUs against 25 us on MFMA up to batch 4, but the matrix-core path writes two row groups of
// partial sums instead of sixteen and its reductions ride in the LayerNorm launches that follow: a whole
// batched layer step takes 170.3 against 177.5 us at batch 3 and 177.7 against 187.5 us at batch 4).
constexpr int kRowsVecMaxBatch = 2;
constexpr int kColsVecMaxBatch = 2;

// ---- batched gathered GEMMs on the matrix cores (5 <= B <= 64) -------------------
#ifndef DV_ROWS_XLDS
#define DV_ROWS_XLDS 1
#endif
template <int BT, bool IDX64, bool RELU>
int launch_rows_mfma(const half_t* x, const half_t* W, int64_t ldw, const half_t* bias, const void* idx,
                     int B, int N, int Z, int M, half_t* y, int act, hipStream_t s) {
  constexpr bool XLDS = DV_ROWS_XLDS && BT <= 2;
  auto kern = gather_rows_mfma_kernel<BT, IDX64, RELU, false, XLDS>;
  // one 16 x 256 staging tile per wavefront (two with X staged as well); the same memory later
  // holds the partial result tiles
  const size_t tile_bytes = (size_t)kMfmaWaves * (XLDS ? 2 : 1) * kMfmaRows * kMfmaLdsRow * sizeof(half_t);
  const size_t red_bytes = (size_t)kMfmaWaves * BT * 4 * 64 * sizeof(float);
  const size_t lds = tile_bytes > red_bytes ? tile_bytes : red_bytes;
  static LdsGrant grant;
  if (int rc = grant.ensure(reinterpret_cast<const void*>(kern), lds); rc != DV_OK) return rc;
  int blocks = (M + kMfmaRows - 1) / kMfmaRows;
  const int cap = compute_units() * 4;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(kMfmaWaves * 64), lds, s, x, W, bias, idx, B, N, ldw, Z, M, y, 0,
                     static_cast<float*>(nullptr), act);
  return launch_status();
}

int gather_rows_mfma(const half_t* x, const half_t* W, int64_t ldw, const half_t* bias, const void* idx,
                     int idx_bytes, int B, int N, int Z, int M, int act, half_t* y, hipStream_t s) {
  const bool relu = act != DV_ACT_ID, i64 = idx_bytes == 8;  // relu: an activation is applied (act says which)
#define DV_RM(BT)                                                                              \
  (relu ? (i64 ? launch_rows_mfma<BT, true, true>(x, W, ldw, bias, idx, B, N, Z, M, y, act, s)        \
               : launch_rows_mfma<BT, false, true>(x, W, ldw, bias, idx, B, N, Z, M, y, act, s))      \
        : (i64 ? launch_rows_mfma<BT, true, false>(x, W, ldw, bias, idx, B, N, Z, M, y, act, s)       \
               : launch_rows_mfma<BT, false, false>(x, W, ldw, bias, idx, B, N, Z, M, y, act, s)))
  if (B <= 16) return DV_RM(1);
  if (B <= 32) return DV_RM(2);
  return DV_RM(4);
#undef DV_RM
}

// Few row tiles, long rows: split the chunks of a row over gridDim.y as well (see the kernel).
// One chunk per wavefront at least; as many splits as it takes to have about two workgroups
// per compute unit.
struct RowsSplitPlan {
  int nsplit, chunks_per_split;
};

RowsSplitPlan plan_rows_split(int N, int M) {
  const int nchunks = (N + kMfmaKC - 1) / kMfmaKC;
  const int ntiles = (M + kMfmaRows - 1) / kMfmaRows;
  int want = ntiles > 0 ? 2 * compute_units() / ntiles : 1;
  if (want < 1) want = 1;
  int cps = (nchunks + want - 1) / want;
  cps = (cps + kMfmaWaves - 1) / kMfmaWaves * kMfmaWaves;
  RowsSplitPlan p;
  p.chunks_per_split = cps;
  p.nsplit = (nchunks + cps - 1) / cps;
  return p;
}

size_t rows_split_workspace_bytes(int B, int N, int M) {
  const RowsSplitPlan p = plan_rows_split(N, M);
  return p.nsplit > 1 ? (size_t)p.nsplit * B * M * sizeof(float) : 0;
}

// dense (no gather, bias or activation) product through the split kernel; falls back to the
// unsplit kernel when one split is enough or no workspace was given
int rows_mfma_dense(const half_t* x, const half_t* W, int64_t ldw, int B, int N, int M, half_t* y,
                    void* workspace, size_t workspace_bytes, hipStream_t s) {
  const RowsSplitPlan p = plan_rows_split(N, M);
  if (p.nsplit <= 1 || workspace == nullptr || workspace_bytes < rows_split_workspace_bytes(B, N, M) ||
      !aligned16(workspace))
    return gather_rows_mfma(x, W, ldw, nullptr, nullptr, 4, B, N, M, M, DV_ACT_ID, y, s);
  float* partial = reinterpret_cast<float*>(workspace);
  const int ntiles = (M + kMfmaRows - 1) / kMfmaRows;
  const dim3 grid(ntiles, p.nsplit);
  const size_t tile_bytes = (size_t)kMfmaWaves * kMfmaRows * kMfmaLdsRow * sizeof(half_t);
#define DV_RS(BT)                                                                                         \
  do {                                                                                                    \
    const size_t red_bytes = (size_t)kMfmaWaves * BT * 4 * 64 * sizeof(float);                            \
    const size_t lds = tile_bytes > red_bytes ? tile_bytes : red_bytes;                                   \
    static LdsGrant grant;                                                                                \
    if (int rc = grant.ensure(reinterpret_cast<const void*>(gather_rows_mfma_kernel<BT, false, false, true>), lds); \
        rc != DV_OK)                                                                                      \
      return rc;                                                                                          \
    hipLaunchKernelGGL((gather_rows_mfma_kernel<BT, false, false, true>), grid, dim3(kMfmaWaves * 64), lds, s, x, \
                       W, nullptr, nullptr, B, N, ldw, M, M, y, p.chunks_per_split, partial);             \
  } while (0)
  if (B <= 16) DV_RS(1);
  else if (B <= 32) DV_RS(2);
  else DV_RS(4);
#undef DV_RS
  const int64_t total = (int64_t)B * M;
  hipLaunchKernelGGL(rows_split_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, partial,
                     p.nsplit, total, y);
  return launch_status();
}

// Dense short rows (N <= 1024, no gather, no bias): every wavefront owns whole 16-row tiles and
// X sits in LDS.  The wavefront count per workgroup (one workgroup per compute unit) is the one
// that spreads the tiles most evenly.  Returns DV_ERR_UNSUPPORTED when the shape does not fit
// (the caller then takes the general kernel).
template <int BT>
int launch_rows_short(const half_t* x, const half_t* W, int64_t ldw, int B, int N, int M, half_t* y,
                      hipStream_t s) {
  const int ntiles = (M + kMfmaRows - 1) / kMfmaRows;
  const int cus = compute_units();
  int best_w = 0, best_cost = 0;
  for (int w = 8; w >= 4; --w) {
    const int cost = (ntiles + cus * w - 1) / (cus * w) * w;  // tiles the busiest compute unit walks
    if (best_w == 0 || cost < best_cost) {
      best_w = w;
      best_cost = cost;
    }
  }
  const int nchunks = (N + kMfmaKC - 1) / kMfmaKC;
  const size_t lds = ((size_t)16 * BT * (nchunks * kMfmaKC + kMfmaRowPad) +
                      (size_t)best_w * kMfmaRows * kMfmaLdsRow) * sizeof(half_t);
  static LdsGrant grant;
  if (int rc = grant.ensure(reinterpret_cast<const void*>(rows_short_mfma_kernel<BT>), lds); rc != DV_OK) return rc;
  int grid = (ntiles + best_w - 1) / best_w;
  if (grid > cus) grid = cus;
  hipLaunchKernelGGL((rows_short_mfma_kernel<BT>), dim3(grid), dim3(best_w * 64), lds, s, x, W, ldw, B, N, M, y);
  return launch_status();
}

// Shapes the short-row kernel is for: at most 32 batch rows (X in LDS), rows of at most 1024
// elements, and enough 16-row tiles to give every compute unit several wavefronts.
bool rows_short_fits(int B, int N, int M) {
  return B <= 32 && N <= 1024 && (M + kMfmaRows - 1) / kMfmaRows >= 4 * compute_units();
}

int rows_short_mfma(const half_t* x, const half_t* W, int64_t ldw, int B, int N, int M, half_t* y,
                    hipStream_t s) {
  return B <= 16 ? launch_rows_short<1>(x, W, ldw, B, N, M, y, s) : launch_rows_short<2>(x, W, ldw, B, N, M, y, s);
}

// ---- X-shared split-K products (gemm_tiled.hpp) ---------------------------------
struct TiledPlan {
  int bt, wt, kc, waves, xblocks, row_groups, nsplit, chunks_per_split;
};

TiledPlan plan_tiled(int B, int N, int M) {
  TiledPlan p;
  p.bt = B <= 16 ? 1 : (B <= 32 ? 2 : (B <= 64 ? 4 : 8));
  // Two and four batch tiles: 32 weight rows per wavefront and chunks of 128 columns (fewer LDS reads per
  // MFMA) once the matrix has rows enough to fill the device that way (QKV of 32 heads at 32 rows: 65.6 ->
  // 59.0 us; 64 rows: 96 -> 69 us); short matrices (fc1: 4096 rows, a predictor's 1000) keep 16 rows per
  // wavefront, chunks of 256 and more workgroups.
  const bool wide = p.bt >= 4 || (p.bt == 2 && M >= 32 * compute_units());
  p.kc = wide ? 128 : 256;
  p.xblocks = (B + 16 * p.bt - 1) / (16 * p.bt);
  const int cus = compute_units();
  const int nchunks = (N + p.kc - 1) / p.kc;
  // one batch tile: 32 rows per wavefront halve the LDS reads of X per weight byte; worth it when the
  // matrix still fills the device
  p.wt = (wide || (p.bt == 1 && (int64_t)M * p.xblocks >= (int64_t)256 * cus)) ? 2 : 1;
  // Workgroup size (8 wavefronts = 128 * wt rows, or 4) and column splits.  Measured at the OPT-175B
  // shapes (QKV of 32 heads: 12288 rows; fc1: 4096 rows; batch 16 / 32): what counts is one round of
  // workgroups over the device with loops as long as possible -- 192 workgroups of 24 chunks beat 768
  // of 6 (61 against 70 us), and workgroups of 4 wavefronts are only worth it when several are
  // resident per compute unit or when they double the chunks per workgroup (fc1: 24.2 against 25.9 us).
  double best_score = -1.0;
  p.waves = 8;
  p.nsplit = 1;
  const int max_split = nchunks / 4 > 1 ? (nchunks / 4 < 16 ? nchunks / 4 : 16) : 1;
  for (int waves = 8; waves >= (wide ? 8 : 4); waves -= 4) {
    const size_t lds = (size_t)(2 * 16 * p.bt + waves * 16 * p.wt) * (p.kc + kTgPad) * sizeof(half_t);
    const int resident = (int)((size_t)160 * 1024 / lds) > 0 ? (int)((size_t)160 * 1024 / lds) : 1;
    const int64_t groups = (M + waves * 16 * p.wt - 1) / (waves * 16 * p.wt);
    for (int ns = 1; ns <= max_split; ++ns) {
      const int cps = (nchunks + ns - 1) / ns;
      if ((nchunks + cps - 1) / cps != ns) continue;  // not realisable with whole chunks
      const int64_t wgs = groups * p.xblocks * ns;
      double fill;
      if (wgs <= cus) {
        fill = (double)wgs / cus;
      } else {
        const int64_t slots = (int64_t)cus * resident;
        fill = (double)wgs / (double)((wgs + slots - 1) / slots * slots);
      }
      const double loop = (double)cps / (cps + 4.0);  // start-up and drain of a workgroup, in chunks
      const double few_waves = (waves == 4 && wgs <= cus) ? 0.85 : 1.0;  // half the bytes in flight per unit
      const double extra = ns > 1 ? 4.0 * ns * (16.0 * p.bt * p.xblocks) / N : 0.0;  // partial bytes / weight bytes
      const double score = fill * loop * few_waves / (1.0 + extra);
      if (score > best_score + 1e-9) {
        best_score = score;
        p.waves = waves;
        p.nsplit = ns;
      }
    }
  }
  p.row_groups = (M + p.waves * 16 * p.wt - 1) / (p.waves * 16 * p.wt);
  p.chunks_per_split = (nchunks + p.nsplit - 1) / p.nsplit;
  return p;
}

bool big_applies(int B, int N);
size_t tiled_workspace_bytes(int B, int N, int M) {
  if (big_applies(B, N)) return 0;
  const TiledPlan p = plan_tiled(B, N, M);
  return p.nsplit > 1 ? (size_t)p.nsplit * B * M * sizeof(float) : 0;
}

template <int BT, int WT, int KC, int WAVES>
int launch_tiled(const TiledPlan& p, const half_t* X, int64_t ldx, const half_t* W, int64_t ldw, const half_t* bias,
                 const void* idx, int idx_bytes, int B, int N, int Z, int M, half_t* Y, int64_t ldy, int relu,
                 float* partial, hipStream_t s) {
  auto kern = gemm_tiled_mfma_kernel<BT, WT, KC, false, WAVES>;
  constexpr size_t lds = tiled_lds_bytes<BT, WT, KC, WAVES>();
  static LdsGrant grant;
  if (int rc = grant.ensure(reinterpret_cast<const void*>(kern), lds); rc != DV_OK) return rc;
  const dim3 grid(p.xblocks, p.row_groups, p.nsplit);
  hipLaunchKernelGGL(kern, grid, dim3(WAVES * 64), lds, s, X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y,
                     ldy, relu, p.nsplit > 1 ? p.chunks_per_split : 0, partial, QkvScatter{});
  return DV_OK;
}

// Many rows of X (two or more 128-row blocks): the product is bound by the matrix cores and by what
// the L2 delivers, and gemm_big_mfma_kernel (weights straight into MFMA operands, 64 * WT weight rows
// per workgroup) is the faster kernel -- measured at 12288 x 12288 against gemm_tiled_mfma_kernel:
// 256 rows 172 against 259 us, 512 rows 225 against 278 us, 2048 rows 793 against 797 us.  Same bits.
// WT: the tile height that fills the device best; on a tie the larger (fewer L2 reads per flop).
bool big_applies(int B, int N) { return B >= 200 && N % (kBgKC * kBgRing) == 0; }
int big_pick_wt(int B, int M, int max_wt) {
  const int cus = compute_units();
  const int xblocks = (B + kBgXRows - 1) / kBgXRows;
  int best_wt = 2;
  double best_fill = -1.0;
  for (int wt = 2; wt <= max_wt; ++wt) {
    const int64_t wgs = (int64_t)xblocks * ((M + 64 * wt - 1) / (64 * wt));
    const double fill = (double)wgs / (double)((wgs + cus - 1) / cus * cus);
    if (fill >= best_fill - 1e-9) {
      best_fill = fill;
      best_wt = wt;
    }
  }
  return best_wt;
}
template <int WT, bool QKV>
int launch_big(const half_t* X, int64_t ldx, const half_t* W, int64_t ldw, const half_t* bias, const void* idx,
               int idx_bytes, int B, int N, int Z, int M, half_t* Y, int64_t ldy, int act, const QkvScatter& qs,
               hipStream_t s) {
  auto kern = gemm_big_mfma_kernel<WT, QKV>;
  static LdsGrant grant;
  if (int rc = grant.ensure(reinterpret_cast<const void*>(kern), big_lds_bytes()); rc != DV_OK) return rc;
  const dim3 grid((B + kBgXRows - 1) / kBgXRows, (M + 64 * WT - 1) / (64 * WT));
  hipLaunchKernelGGL(kern, grid, dim3(256), big_lds_bytes(), s, X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y,
                     ldy, act, qs);
  return launch_status();
}
template <bool QKV>
int gemm_big(const half_t* X, int64_t ldx, const half_t* W, int64_t ldw, const half_t* bias, const void* idx,
             int idx_bytes, int B, int N, int Z, int M, half_t* Y, int64_t ldy, int act, const QkvScatter& qs,
             hipStream_t s) {
  // (the scatter epilogue of the QKV form leaves no registers for the tallest tile)
  constexpr int kMaxWt = QKV ? 3 : 4;
  switch (big_pick_wt(B, M, kMaxWt)) {
    case 2: return launch_big<2, QKV>(X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y, ldy, act, qs, s);
    case 3: return launch_big<3, QKV>(X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y, ldy, act, qs, s);
    default: return launch_big<(QKV ? 3 : 4), QKV>(X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y, ldy, act, qs, s);
  }
}

// QKV of the selected heads for B rows (see QkvScatter): M = 3 * Hk * hd output rows
int gemm_tiled_qkv(const half_t* X, int64_t ldx, const half_t* W, const half_t* bias, int B, int d, half_t* Y,
                   const QkvScatter& qs, void* workspace, size_t workspace_bytes, hipStream_t s) {
  const int M = 3 * qs.Hk * qs.hd, Z = 3 * qs.H * qs.hd;
  if (big_applies(B, d))
    return gemm_big<true>(X, ldx, W, (int64_t)d, bias, nullptr, 4, B, d, Z, M, Y, (int64_t)Z, 0, qs, s);
  const TiledPlan p = plan_tiled(B, d, M);
  float* partial = nullptr;
  if (p.nsplit > 1) {
    if (workspace == nullptr || !aligned16(workspace) || workspace_bytes < tiled_workspace_bytes(B, d, M))
      return DV_ERR_WORKSPACE;
    partial = reinterpret_cast<float*>(workspace);
  }
  const dim3 grid(p.xblocks, p.row_groups, p.nsplit);
  const int cps = p.nsplit > 1 ? p.chunks_per_split : 0;
#define DV_TQW(BT, WT, KC, WAVES)                                                                              \
  do {                                                                                                         \
    auto kern = gemm_tiled_mfma_kernel<BT, WT, KC, true, WAVES>;                                               \
    constexpr size_t lds = tiled_lds_bytes<BT, WT, KC, WAVES>();                                               \
    static LdsGrant grant;                                                                                     \
    if (int rc = grant.ensure(reinterpret_cast<const void*>(kern), lds); rc != DV_OK) return rc;               \
    hipLaunchKernelGGL(kern, grid, dim3(WAVES * 64), lds, s, X, ldx, W, (int64_t)d, bias,                      \
                       (const void*)nullptr, 4, B, d, Z, M, Y, (int64_t)Z, 0, cps, partial, qs);              \
  } while (0)
#define DV_TQ(BT, WT)                       \
  do {                                      \
    if (p.waves == 4) DV_TQW(BT, WT, 256, 4); \
    else DV_TQW(BT, WT, 256, 8);            \
  } while (0)
  if (p.bt == 1) { if (p.wt == 2) DV_TQ(1, 2); else DV_TQ(1, 1); }
  else if (p.bt == 2) { if (p.wt == 2) DV_TQW(2, 2, 128, 8); else DV_TQ(2, 1); }
  else if (p.bt == 4) DV_TQW(4, 2, 128, 8);
  else DV_TQW(8, 2, 128, 8);
#undef DV_TQW
#undef DV_TQ
  if (p.nsplit > 1) {
    const int64_t quads = (int64_t)B * M / 4;  // M = 3 * Hk * hd is a multiple of 4
    hipLaunchKernelGGL(qkv_split_reduce_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, partial,
                       p.nsplit, B, M, bias, Y, qs);
  }
  return launch_status();
}

// Y (B, M) row stride ldy = act(X (B, N) . W[idx]^T + bias[idx]); idx == nullptr: rows 0..M-1 of W.
int gemm_tiled(const half_t* X, int64_t ldx, const half_t* W, int64_t ldw, const half_t* bias, const void* idx,
               int idx_bytes, int B, int N, int Z, int M, int act, half_t* Y, int64_t ldy, void* workspace,
               size_t workspace_bytes, hipStream_t s) {
  if (big_applies(B, N))
    return gemm_big<false>(X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y, ldy, act, QkvScatter{}, s);
  const TiledPlan p = plan_tiled(B, N, M);
  float* partial = nullptr;
  if (p.nsplit > 1) {
    if (workspace == nullptr || !aligned16(workspace) || workspace_bytes < tiled_workspace_bytes(B, N, M))
      return DV_ERR_WORKSPACE;
    partial = reinterpret_cast<float*>(workspace);
  }
  const int relu = act;  // activation code of the epilogue (0: none)
  int rc;
#define DV_TG(BT, WT, KC)                                                                                          \
  do {                                                                                                             \
    if (p.waves == 4)                                                                                              \
      rc = launch_tiled<BT, WT, KC, 4>(p, X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y, ldy, relu, partial, s); \
    else                                                                                                           \
      rc = launch_tiled<BT, WT, KC, 8>(p, X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y, ldy, relu, partial, s); \
  } while (0)
  if (p.bt == 1) { if (p.wt == 2) DV_TG(1, 2, 256); else DV_TG(1, 1, 256); }
  else if (p.bt == 2) {
    if (p.wt == 2) rc = launch_tiled<2, 2, 128, 8>(p, X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y, ldy, relu, partial, s);
    else DV_TG(2, 1, 256);
  }
  else if (p.bt == 4) rc = launch_tiled<4, 2, 128, 8>(p, X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y, ldy, relu, partial, s);
  else rc = launch_tiled<8, 2, 128, 8>(p, X, ldx, W, ldw, bias, idx, idx_bytes, B, N, Z, M, Y, ldy, relu, partial, s);
#undef DV_TG
  if (rc != DV_OK) return rc;
  if (p.nsplit > 1) {
    const int64_t total = (int64_t)B * M;
    hipLaunchKernelGGL(gemm_split_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, partial,
                       p.nsplit, B, M, bias, idx, idx_bytes, Z, relu, Y, ldy);
  }
  return launch_status();
}

struct ColsMfmaPlan {
  int col_tiles, groups, rows_per_block;
};

ColsMfmaPlan plan_cols_mfma(int B, int N, int M) {
  ColsMfmaPlan p;
  // Every row group writes a (B, N) fp32 partial that a second pass reads back, so few, long
  // groups win.  Each wavefront keeps 16 KiB of weights in flight and three of them per compute
  // unit measured best for batch 8..64.  Up to batch 32 a workgroup's four wavefronts split the
  // group's rows and add their sums through LDS (a quarter of the partials: fc2 at the OPT-175B
  // shape 3 us faster at batch 16 and 32); above, they split the columns.
  const int waves_per_cu = 3;  // 4..16 measured 30-50 % slower for batch 5..32 (fc2, OPT-175B shape)
  const bool split_rows = B <= 32;
  const int col_tile = mfma_col_tile(split_rows ? 1 : 2);
  p.col_tiles = (N + col_tile - 1) / col_tile;
  const int blocks = (compute_units() * waves_per_cu + 3) / 4;
  int groups = (blocks + p.col_tiles - 1) / p.col_tiles;
  const int min_rows = split_rows ? kMfmaColSub * kMfmaColRows : kMfmaColRows;  // one pipeline step per wavefront
  const int max_groups = M > min_rows ? (M + min_rows - 1) / min_rows : 1;
  if (groups > max_groups) groups = max_groups;
  if (groups < 1) groups = 1;
  int rpb = (M + groups - 1) / groups;
  rpb = (rpb + min_rows - 1) / min_rows * min_rows;
  if (rpb < min_rows) rpb = min_rows;
  p.rows_per_block = rpb;
  p.groups = M > 0 ? (M + rpb - 1) / rpb : 1;
  return p;
}

// plan of gather_cols_mfma16_kernel (batch <= 32): 128 columns per workgroup of 4 wavefronts whose shares
// are whole double steps (64 rows); as many row groups as give every compute unit at most one workgroup
// (OPT-175B shape: 96 column tiles x 2 groups).  Alone the kernel is a little faster with more groups
// (fc2, batch 8: 22.7 us with 8 row groups, 24.4 with 4, 24.2 with 2; the 32x32x16 kernel: 26.7), but
// every group costs (B, N) fp32 partial sums written and read back, one workgroup per row reads all of
// them when the reduction rides in a LayerNorm launch, and the concurrent stream's kernels find no free
// compute unit: a whole layer step at batch 8 takes 213.3 / 217.4 / 211.7 / 234.2 us with 8 / 4 / 2 / 1 groups
// (209.4 with 2 groups and both reductions inside LayerNorm launches), at batch 16 260.9 / 260.3 / 260.9 /
// 288.1 us, at batch 32 350.6 us with 2 groups, 356.1 with 3 (288 workgroups: a second round), 387.6 with 1.
struct Cols16Plan {
  int col_tiles, groups, rows_per_block, rows_per_wave;
};
constexpr int kC16Waves = 4;

Cols16Plan plan_cols16(int B, int N, int M) {
  Cols16Plan p;
  p.col_tiles = (N + kC16Cols - 1) / kC16Cols;
  int groups = compute_units() / p.col_tiles;
  if (groups < 1) groups = 1;
  const int unit = kC16Waves * 2 * kC16Step;
  int rpb = ((M + groups - 1) / groups + unit - 1) / unit * unit;
  if (rpb > kC16Waves * kC16MaxRows) rpb = kC16Waves * kC16MaxRows;
  if (rpb < unit) rpb = unit;
  p.rows_per_block = rpb;
  p.rows_per_wave = rpb / kC16Waves;
  p.groups = M > 0 ? (M + rpb - 1) / rpb : 1;
  return p;
}

size_t cols_mfma_workspace_bytes(int B, int N, int M) {
  const ColsMfmaPlan p = plan_cols_mfma(B, N, M);
  const Cols16Plan q = plan_cols16(B, N, M);
  const int groups = p.groups > q.groups ? p.groups : q.groups;
  return (size_t)groups * B * N * sizeof(float);
}

// What follows a transposed product in the block: residual add + LayerNorm of its rows.  With a tail the
// split reduction and the LayerNorm are ONE launch (norm.hpp: LnRowFromPartials); y itself is not stored.
struct LnTail {
  const half_t* residual;
  const half_t* gamma;
  const half_t* beta;
  float eps;
  half_t* normed;
  half_t* residual_out;
  // non-null: no reduction launch at all; the number of row groups goes here and the caller's
  // consumer reduces (dv_reduce_add_layer_norm_window_f16, dv_reduce_rows_f16)
  int* deferred_groups = nullptr;
};

// the reduction (groups > 1: from the partial sums; else y is complete) with or without the tail
void launch_cols_reduce(const float* partial, const half_t* bias, int groups, int B, int N, half_t* y,
                        const LnTail* tail, hipStream_t s) {
  if (tail != nullptr && tail->deferred_groups != nullptr) {
    *tail->deferred_groups = groups;
    return;
  }
  if (tail == nullptr) {
    if (groups > 1) {
      const int64_t total = (int64_t)B * N;
      hipLaunchKernelGGL(cols_reduce_kernel<false>, dim3((unsigned)((total + 63) / 64)), dim3(256), 0, s, partial,
                         bias, groups, B, N, y, (const half_t*)nullptr, (half_t*)nullptr);
    }
    return;
  }
#define DV_RLN(T, V)                                                                                              \
  do {                                                                                                            \
    if (groups > 1)                                                                                               \
      hipLaunchKernelGGL((reduce_add_layer_norm_kernel<T, V>), dim3(B), dim3(T), 0, s, partial, bias, groups, B,  \
                         tail->residual, tail->gamma, tail->beta, tail->eps, N, tail->normed, tail->residual_out); \
    else                                                                                                          \
      hipLaunchKernelGGL((add_layer_norm_kernel<T, V>), dim3(B), dim3(T), 0, s, (const half_t*)y, tail->residual,   \
                         tail->gamma, tail->beta, tail->eps, N, tail->normed, tail->residual_out,                 \
                         (half_t*)nullptr);                                                                       \
  } while (0)
  if (N <= 256 * 8 * 1)
    DV_RLN(256, 1);
  else if (N <= 512 * 8 * 1)
    DV_RLN(512, 1);
  else if (N <= 1024 * 8 * 1)
    DV_RLN(1024, 1);
  else if (N <= 1024 * 8 * 2)
    DV_RLN(1024, 2);
  else
    DV_RLN(1024, 4);
#undef DV_RLN
}

template <int BT, bool IDX64, bool BLOCKED>
void launch_cols16(const Cols16Plan& p, const half_t* h, int64_t ldh, int x_expanded, const half_t* W, int64_t ldw,
                   const half_t* bias, const void* idx, int blk, int B, int N, int Z, int M, float* partial,
                   half_t* y, hipStream_t s, const LnTail* tail = nullptr) {
  hipLaunchKernelGGL((gather_cols_mfma16_kernel<BT, kC16Waves, IDX64, BLOCKED>), dim3(p.col_tiles, p.groups),
                     dim3(kC16Waves * 64), 0, s, h, ldh, x_expanded, W, ldw, bias, idx, blk, B, N, Z, M,
                     p.rows_per_block, p.rows_per_wave, partial, y);
  launch_cols_reduce(partial, bias, p.groups, B, N, y, tail, s);
}

template <int BT, bool IDX64, bool BLOCKED, bool HVEC>
void launch_cols_mfma(const ColsMfmaPlan& p, const half_t* h, int64_t ldh, int x_expanded, const half_t* W,
                      int64_t ldw, const half_t* bias, const void* idx, int blk, int B, int N, int Z, int M,
                      float* partial, half_t* y, hipStream_t s, const LnTail* tail = nullptr) {
  hipLaunchKernelGGL((gather_cols_mfma_kernel<BT, IDX64, BLOCKED, HVEC>), dim3(p.col_tiles, p.groups), dim3(256), 0,
                     s, h, ldh, x_expanded, W, ldw, bias, idx, blk, B, N, Z, M, p.rows_per_block, partial, y);
  launch_cols_reduce(partial, bias, p.groups, B, N, y, tail, s);
}

int gather_cols_mfma(const half_t* h, int64_t ldh, int x_expanded, const half_t* W, int64_t ldw,
                     const half_t* bias, const void* idx, int idx_bytes, int blk, int B, int N, int Z, int M,
                     half_t* y, void* workspace, size_t workspace_bytes, hipStream_t s,
                     const LnTail* tail = nullptr) {
  const ColsMfmaPlan p = plan_cols_mfma(B, N, M);
  if (workspace == nullptr || workspace_bytes < cols_mfma_workspace_bytes(B, N, M)) return DV_ERR_WORKSPACE;
  float* partial = reinterpret_cast<float*>(workspace);
  const bool i64 = idx_bytes == 8, blocked = blk != 1;
  const bool hvec = M % 8 == 0 && ldh % 8 == 0 && aligned16(h) && (!x_expanded || blk % 8 == 0);
  // up to 32 rows: the 16x16x32 kernel (it needs vector loads of H and, for a blocked row map, blocks
  // that are multiples of 8 rows)
  if (B <= 32 && hvec && M >= 8 && (blocked ? blk % 8 == 0 : !x_expanded)) {
    const Cols16Plan q = plan_cols16(B, N, M);
#define DV_C16(BT)                                                                                                   \
  do {                                                                                                               \
    if (blocked) {                                                                                                   \
      if (i64) launch_cols16<BT, true, true>(q, h, ldh, x_expanded, W, ldw, bias, idx, blk, B, N, Z, M, partial, y, s, tail);  \
      else launch_cols16<BT, false, true>(q, h, ldh, x_expanded, W, ldw, bias, idx, blk, B, N, Z, M, partial, y, s, tail);     \
    } else {                                                                                                         \
      if (i64) launch_cols16<BT, true, false>(q, h, ldh, x_expanded, W, ldw, bias, idx, blk, B, N, Z, M, partial, y, s, tail); \
      else launch_cols16<BT, false, false>(q, h, ldh, x_expanded, W, ldw, bias, idx, blk, B, N, Z, M, partial, y, s, tail);    \
    }                                                                                                                \
  } while (0)
    if (B <= 16) DV_C16(1);
    else DV_C16(2);
#undef DV_C16
    return launch_status();
  }
#define DV_ARGS p, h, ldh, x_expanded, W, ldw, bias, idx, blk, B, N, Z, M, partial, y, s, tail
#define DV_CM3(BT, I64, BLK)                                   \
  do {                                                         \
    if (hvec) launch_cols_mfma<BT, I64, BLK, true>(DV_ARGS);   \
    else launch_cols_mfma<BT, I64, BLK, false>(DV_ARGS);       \
  } while (0)
#define DV_CM(BT)                                  \
  do {                                             \
    if (blocked) {                                 \
      if (i64) DV_CM3(BT, true, true);             \
      else DV_CM3(BT, false, true);                \
    } else {                                       \
      if (i64) DV_CM3(BT, true, false);            \
      else DV_CM3(BT, false, false);               \
    }                                              \
  } while (0)
  if (B <= 32)
    DV_CM(1);
  else
    DV_CM(2);
#undef DV_CM3
#undef DV_ARGS
#undef DV_CM
  return launch_status();
}

// ---- head-sparse attention ---------------------------------------------------
template <int NBMAX>
int launch_qkv(const half_t* x, const half_t* W, const half_t* bias, const int* head_idx,
               const int* batch_idx, int nb, int d, int H, int hd, int nnz, half_t* y,
               half_t* k_cache, half_t* v_cache, const int* padding, int S, hipStream_t s) {
  constexpr int R = 2, U = 4;
  const int ntasks = nnz * 3 * (hd / R);
  int blocks = (ntasks + 3) / 4;
  const int cap = compute_units() * 8;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL((qkv_sparse_kernel<NBMAX, R, U>), dim3(blocks), dim3(256), 0, s, x, W, bias,
                     head_idx, batch_idx, nb, d, H, hd, nnz, y, k_cache, v_cache, padding, S);
  return launch_status();
}

// Window tokens from which one pass on the matrix cores (all 16 slots at a cost that hardly grows
// with the number of live ones) beats the per-token dot products.
// Measured at the OPT-175B shape: 47 us for one token on the vector path (49 us on MFMA), and
// 47..49 us for 2..16 tokens on MFMA against 52..95 us on the vector path.
inline bool qkv_use_mfma(int nb) { return nb >= 2; }
// Workgroups of 32 weight rows (half the x traffic, same bits) once there are enough of them
// to fill the device: the flush step of a window (all heads).
inline bool qkv_mfma_two_tiles(int nnz, int hd) {
  return hd % 32 == 0 && nnz * 3 * (hd / 32) >= 3 * compute_units();
}

int launch_qkv_mfma(const half_t* x, const half_t* W, const half_t* bias, const int* head_idx,
                    const int* batch_idx, int nb, int d, int H, int hd, int nnz, half_t* y,
                    half_t* k_cache, half_t* v_cache, const int* padding, int S, hipStream_t s) {
  if (qkv_mfma_two_tiles(nnz, hd))
    hipLaunchKernelGGL((qkv_window_mfma_kernel<kQkvMfmaWaves, 2>), dim3(nnz * 3 * (hd / 32)),
                       dim3(kQkvMfmaWaves * 64), 0, s, x, W, bias, head_idx, batch_idx, nb, d, H, hd, nnz, y,
                       k_cache, v_cache, padding, S);
  else
    hipLaunchKernelGGL((qkv_window_mfma_kernel<kQkvMfmaWaves, 1>), dim3(nnz * 3 * (hd / 16)),
                       dim3(kQkvMfmaWaves * 64), 0, s, x, W, bias, head_idx, batch_idx, nb, d, H, hd, nnz, y,
                       k_cache, v_cache, padding, S);
  return launch_status();
}

constexpr int kAttnWaves = 4;  // wavefronts (x64 positions) per attention workgroup
inline int attn_splits(int n_len) {
  return n_len > 0 ? (n_len + kAttnWaves * kWave - 1) / (kAttnWaves * kWave) : 1;
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

size_t dv_predictor_workspace_bytes(int B, int d, int r) {
  if (B <= 8 || B > 64 || d <= 0 || r <= 0) return 0;
  // the first product's column splits; the second product (rows of r elements) splits only when r is long,
  // allow for as many partial sums again
  const size_t first = tiled_workspace_bytes(B, d, r);
  const size_t floor_bytes = (size_t)1 << 20;
  return 2 * (first > floor_bytes ? first : floor_bytes);
}

int dv_predictor_logits_ws_f16(const void* x, const void* Wa, int64_t ldwa, const void* Wb, int64_t ldwb,
                               int B, int d, int r, int n_out, void* hidden, void* logits, void* workspace,
                               size_t workspace_bytes, void* stream) {
  if (!x || !Wa || !Wb || !hidden || !logits || d <= 0 || r <= 0 || n_out <= 0)
    return DV_ERR_INVALID_ARG;
  if (B < 1 || B > 64) return DV_ERR_UNSUPPORTED;
  if (d % 8 || r % 8 || ldwa % 8 || ldwb % 8 || ldwa < d || ldwb < r || !aligned16(x) ||
      !aligned16(Wa) || !aligned16(Wb) || !aligned16(hidden))
    return DV_ERR_ALIGNMENT;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (B > 8 && workspace != nullptr && aligned16(workspace) &&
      workspace_bytes >= dv_predictor_workspace_bytes(B, d, r) && ldwa >= d) {
    // more rows than the fixed-order kernel keeps accumulators for: both products on the matrix cores
    // (fp32 accumulation in the MFMA's own order).  First product (r rows of d elements: few row tiles):
    // the X-shared split-K kernel (measured at the OPT-175B predictor, batch 16 / 32: 33.6 / 38.8 us for
    // the whole MLP predictor against 37.2 / 44.1 us with one 16-row tile per workgroup).  Second
    // product: many short rows -> whole tiles per wavefront with X in LDS (rows_short); few rows (the
    // head predictor: 96) -> the X-shared kernel again (head predictor 17.7 / 21.6 against 18.7 / 25.3 us).
    int rc = gemm_tiled(reinterpret_cast<const half_t*>(x), d, reinterpret_cast<const half_t*>(Wa), ldwa, nullptr,
                        nullptr, 4, B, d, r, r, DV_ACT_ID, reinterpret_cast<half_t*>(hidden), r, workspace,
                        workspace_bytes, s);
    if (rc != DV_OK) return rc;
    const int pass_rows = B <= 32 ? B : 32;
    if (rows_short_fits(pass_rows, r, n_out) && aligned16(logits) && ((int64_t)32 * n_out) % 8 == 0) {
      for (int b0 = 0; b0 < B && rc == DV_OK; b0 += 32) {
        const int nb = B - b0 < 32 ? B - b0 : 32;
        rc = rows_short_mfma(reinterpret_cast<const half_t*>(hidden) + (int64_t)b0 * r,
                             reinterpret_cast<const half_t*>(Wb), ldwb, nb, r, n_out,
                             reinterpret_cast<half_t*>(logits) + (int64_t)b0 * n_out, s);
      }
      if (rc != DV_ERR_UNSUPPORTED) return rc;
    }
    if (tiled_workspace_bytes(B, r, n_out) <= workspace_bytes)
      return gemm_tiled(reinterpret_cast<const half_t*>(hidden), r, reinterpret_cast<const half_t*>(Wb), ldwb,
                        nullptr, nullptr, 4, B, r, n_out, n_out, DV_ACT_ID, reinterpret_cast<half_t*>(logits),
                        n_out, workspace, workspace_bytes, s);
    return gather_rows_mfma(reinterpret_cast<const half_t*>(hidden), reinterpret_cast<const half_t*>(Wb), ldwb,
                            nullptr, nullptr, 4, B, r, n_out, n_out, DV_ACT_ID,
                            reinterpret_cast<half_t*>(logits), s);
  }
  if (B > 8) {
    // more rows than the fixed-order kernel keeps accumulators for: both products on the
    // matrix cores (no gather, no bias), fp32 accumulation in the MFMA's own order.  The
    // first has few, long rows (split over the columns when a workspace is given), the
    // second many short ones (whole tiles per wavefront, X in LDS, up to 32 batch rows).
    int rc = rows_mfma_dense(reinterpret_cast<const half_t*>(x), reinterpret_cast<const half_t*>(Wa), ldwa, B, d, r,
                             reinterpret_cast<half_t*>(hidden), workspace, workspace_bytes, s);
    if (rc != DV_OK) return rc;
    // beyond 32 batch rows X no longer fits LDS next to the weight tiles: two passes of up to 32 rows
    // (the weights stream twice, still faster than re-reading X from L2 for every 16-row tile)
    const int pass_rows = B <= 32 ? B : 32;
    if (rows_short_fits(pass_rows, r, n_out) && aligned16(logits) && ((int64_t)32 * n_out) % 8 == 0) {
      rc = DV_OK;
      for (int b0 = 0; b0 < B && rc == DV_OK; b0 += 32) {
        const int nb = B - b0 < 32 ? B - b0 : 32;
        rc = rows_short_mfma(reinterpret_cast<const half_t*>(hidden) + (int64_t)b0 * r,
                             reinterpret_cast<const half_t*>(Wb), ldwb, nb, r, n_out,
                             reinterpret_cast<half_t*>(logits) + (int64_t)b0 * n_out, s);
      }
      if (rc != DV_ERR_UNSUPPORTED) return rc;
    }
    return gather_rows_mfma(reinterpret_cast<const half_t*>(hidden), reinterpret_cast<const half_t*>(Wb), ldwb,
                            nullptr, nullptr, 4, B, r, n_out, n_out, DV_ACT_ID,
                            reinterpret_cast<half_t*>(logits), s);
  }
  int rc = canonical_gemv(reinterpret_cast<const half_t*>(x), reinterpret_cast<const half_t*>(Wa),
                          ldwa, B, r, d, reinterpret_cast<half_t*>(hidden), s);
  if (rc != DV_OK) return rc;
  return canonical_gemv(reinterpret_cast<const half_t*>(hidden),
                        reinterpret_cast<const half_t*>(Wb), ldwb, B, n_out, r,
                        reinterpret_cast<half_t*>(logits), s);
}

int dv_predictor_logits_f16(const void* x, const void* Wa, int64_t ldwa, const void* Wb,
                            int64_t ldwb, int B, int d, int r, int n_out, void* hidden,
                            void* logits, void* stream) {
  return dv_predictor_logits_ws_f16(x, Wa, ldwa, Wb, ldwb, B, d, r, n_out, hidden, logits, nullptr, 0, stream);
}

}  // extern "C"
namespace {
// bytes of the per-workgroup histograms and counts; the batch-maximum row follows
size_t topk_max_row_offset(int) {
  return ((size_t)kTopkWords * sizeof(unsigned) + 15) & ~(size_t)15;
}
}  // namespace
extern "C" {

size_t dv_topk_workspace_bytes(int n) {
  if (n <= 1024) return 0;
  return topk_max_row_offset(n) + (size_t)n * sizeof(half_t);
}

int dv_topk_f16(const void* logits, int B, int n, int k, void* idx_out, int idx_bytes,
                void* workspace, size_t workspace_bytes, void* stream) {
  if (!logits || B < 1 || n < 1 || k < 0 || k > n || !idx_ok(idx_bytes) || (k > 0 && !idx_out))
    return DV_ERR_INVALID_ARG;
  if (n > 65536) return DV_ERR_UNSUPPORTED;
  if (k == 0) return DV_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const half_t* lg = reinterpret_cast<const half_t*>(logits);
  if (n <= 1024) {
    hipLaunchKernelGGL(topk_small_kernel, dim3(1), dim3(256), 0, s, lg, B, n, k, idx_out, idx_bytes);
    return launch_status();
  }
  if (n % 8 != 0) return DV_ERR_UNSUPPORTED;
  if (!aligned16(logits)) return DV_ERR_ALIGNMENT;
  if (!workspace || workspace_bytes < dv_topk_workspace_bytes(n) || !aligned16(workspace))
    return DV_ERR_WORKSPACE;
  unsigned* ws = reinterpret_cast<unsigned*>(workspace);
  const int blocks = (n + kTopkItemsPerBlock - 1) / kTopkItemsPerBlock;
  if (B > 1 && B <= 64) {
    // one pass reduces the batch to a row of column-wise maxima and takes that row's coarse histogram;
    // the selection then reads the row
    half_t* m = reinterpret_cast<half_t*>(reinterpret_cast<unsigned char*>(workspace) + topk_max_row_offset(n));
    hipLaunchKernelGGL(topk_batch_hist_kernel, dim3(blocks), dim3(256 * topk_batch_groups(B)), 0, s, lg, B, n, m, ws);
    lg = m;
    B = 1;
  } else {
    hipLaunchKernelGGL(topk_hist_kernel, dim3(blocks), dim3(256), 0, s, lg, B, n, ws);
  }
  hipLaunchKernelGGL(topk_count_kernel, dim3(blocks), dim3(256), 0, s, lg, B, n, k, ws);
  hipLaunchKernelGGL(topk_emit_kernel, dim3(blocks), dim3(256), 0, s, lg, B, n, k, ws, idx_out, idx_bytes);
  return launch_status();
}

int dv_greedy_advance_f16(const void* logits, int vocab, void* token, void* position, void* seq_pos,
                          void* sequences, int64_t seq_capacity, void* out_index, void* scores,
                          int64_t score_ld, int64_t score_rows, void* score_index, void* stream) {
  if (!logits || vocab < 1 || !token || !position || !seq_pos || !sequences || !out_index || seq_capacity < 0 ||
      (scores && (!score_index || score_ld < vocab || score_rows < 0)))
    return DV_ERR_INVALID_ARG;
  hipLaunchKernelGGL(greedy_advance_kernel, dim3(1), dim3(1024), 0, reinterpret_cast<hipStream_t>(stream),
                     reinterpret_cast<const half_t*>(logits), vocab, reinterpret_cast<int64_t*>(token),
                     reinterpret_cast<int64_t*>(position), reinterpret_cast<int*>(seq_pos),
                     reinterpret_cast<int64_t*>(sequences), reinterpret_cast<int64_t*>(out_index),
                     reinterpret_cast<half_t*>(scores), score_ld, reinterpret_cast<int64_t*>(score_index),
                     seq_capacity, score_rows);
  return launch_status();
}

// Single-launch variant without scratch memory (16-step bitwise search in one
// workgroup); same result, slower for large n.
int dv_topk_search_f16(const void* logits, int B, int n, int k, void* idx_out, int idx_bytes,
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
  if (!x || !W || N <= 0 || Z <= 0 || M < 0 || (idx && !idx_ok(idx_bytes)) || (M > 0 && !y) ||
      (!idx && M > Z) || act < DV_ACT_ID || act > DV_ACT_SQUARED_RELU)
    return DV_ERR_INVALID_ARG;
  if (B < 1 || B > 64) return DV_ERR_UNSUPPORTED;
  if (N % 8 || ldw % 8 || ldw < N || !aligned16(x) || !aligned16(W)) return DV_ERR_ALIGNMENT;
  if (M == 0) return DV_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const half_t* xx = reinterpret_cast<const half_t*>(x);
  const half_t* ww = reinterpret_cast<const half_t*>(W);
  const half_t* bb = reinterpret_cast<const half_t*>(bias);
  half_t* yy = reinterpret_cast<half_t*>(y);
  if (B > kRowsVecMaxBatch) return gather_rows_mfma(xx, ww, ldw, bb, idx, idx_bytes, B, N, Z, M, act, yy, s);
  switch (B) {
    case 1: return gather_rows_b<1>(xx, ww, ldw, bb, idx, idx_bytes, N, Z, M, act, yy, s);
    case 2: return gather_rows_b<2>(xx, ww, ldw, bb, idx, idx_bytes, N, Z, M, act, yy, s);
    case 3: return gather_rows_b<3>(xx, ww, ldw, bb, idx, idx_bytes, N, Z, M, act, yy, s);
    default: return gather_rows_b<4>(xx, ww, ldw, bb, idx, idx_bytes, N, Z, M, act, yy, s);
  }
}

// Batches from which the X-shared split-K kernel takes over from the 16-row-tile kernel (measured at
// the OPT-175B fc1: see the kernel table of the batched benchmark).
constexpr int kTiledMinBatch = 17;

size_t dv_gather_gemv_workspace_bytes(int B, int N, int M) {
  if (B < kTiledMinBatch || B > 64 || N <= 0 || M <= 0) return 0;
  return tiled_workspace_bytes(B, N, M);
}

int dv_gather_gemv_ws_f16(const void* x, const void* W, int64_t ldw, const void* bias, const void* idx,
                          int idx_bytes, int B, int N, int Z, int M, int act, void* y, void* workspace,
                          size_t workspace_bytes, void* stream) {
  if (B < kTiledMinBatch || B > 64 || M <= 0 || workspace == nullptr ||
      workspace_bytes < dv_gather_gemv_workspace_bytes(B, N, M) || !aligned16(workspace))
    return dv_gather_gemv_f16(x, W, ldw, bias, idx, idx_bytes, B, N, Z, M, act, y, stream);
  if (!x || !W || N <= 0 || Z <= 0 || (idx && !idx_ok(idx_bytes)) || !y || (!idx && M > Z) ||
      act < DV_ACT_ID || act > DV_ACT_SQUARED_RELU)
    return DV_ERR_INVALID_ARG;
  if (N % 8 || ldw % 8 || ldw < N || !aligned16(x) || !aligned16(W)) return DV_ERR_ALIGNMENT;
  return gemm_tiled(reinterpret_cast<const half_t*>(x), N, reinterpret_cast<const half_t*>(W), ldw,
                    reinterpret_cast<const half_t*>(bias), idx, idx_bytes, B, N, Z, M, act,
                    reinterpret_cast<half_t*>(y), M, workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}

size_t dv_dense_linear_workspace_bytes(int rows, int N, int M) {
  if (rows < 1 || N <= 0 || M <= 0) return 0;
  return tiled_workspace_bytes(rows, N, M);
}

int dv_dense_linear_f16(const void* x, int64_t ldx, const void* W, int64_t ldw, const void* bias, int rows, int N,
                        int M, int act, void* y, int64_t ldy, void* workspace, size_t workspace_bytes,
                        void* stream) {
  if (!x || !W || !y || rows < 0 || N <= 0 || M <= 0 || act < DV_ACT_ID || act > DV_ACT_SQUARED_RELU)
    return DV_ERR_INVALID_ARG;
  if (N % 8 || ldx % 8 || ldw % 8 || ldx < N || ldw < N || ldy < M || !aligned16(x) || !aligned16(W))
    return DV_ERR_ALIGNMENT;
  if (rows == 0) return DV_OK;
  return gemm_tiled(reinterpret_cast<const half_t*>(x), ldx, reinterpret_cast<const half_t*>(W), ldw,
                    reinterpret_cast<const half_t*>(bias), nullptr, 4, rows, N, M, M, act,
                    reinterpret_cast<half_t*>(y), ldy, workspace, workspace_bytes,
                    reinterpret_cast<hipStream_t>(stream));
}

size_t dv_gather_transposed_gemv_workspace_bytes(int B, int N, int M) {
  if (B < 1 || N < 1 || M < 0) return 0;
  return B > kColsVecMaxBatch ? cols_mfma_workspace_bytes(B, N, M) : cols_workspace_bytes(B, N, M);
}

int dv_gather_transposed_gemv_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                                  const void* idx, int idx_bytes, int B, int N, int Z, int M,
                                  void* y, void* workspace, size_t workspace_bytes,
                                  void* stream) {
  if (!W || !y || N <= 0 || Z <= 0 || M < 0 || !idx_ok(idx_bytes) || (M > 0 && (!idx || !x)))
    return DV_ERR_INVALID_ARG;
  if (B < 1 || B > 64) return DV_ERR_UNSUPPORTED;
  // y and the partial sums are written with 16-byte vector stores
  if (N % 8 || ldw % 8 || ldw < N || !aligned16(W) || !aligned16(y) || (workspace && !aligned16(workspace)))
    return DV_ERR_ALIGNMENT;
  if (B > kColsVecMaxBatch)
    return gather_cols_mfma(reinterpret_cast<const half_t*>(x), M, 0, reinterpret_cast<const half_t*>(W),
                            ldw, reinterpret_cast<const half_t*>(bias), idx, idx_bytes, 1, B, N, Z, M,
                            reinterpret_cast<half_t*>(y), workspace, workspace_bytes,
                            reinterpret_cast<hipStream_t>(stream));
  return gather_cols(reinterpret_cast<const half_t*>(x), M, 0, reinterpret_cast<const half_t*>(W),
                     ldw, reinterpret_cast<const half_t*>(bias), idx, idx_bytes, 1, B, N, Z, M,
                     reinterpret_cast<half_t*>(y), workspace, workspace_bytes,
                     reinterpret_cast<hipStream_t>(stream));
}

size_t dv_gather_transposed_gemv_partial_workspace_bytes(int B, int N, int M) {
  if (B <= kColsVecMaxBatch || B > 64 || N < 1 || M < 1) return 0;
  return cols_mfma_workspace_bytes(B, N, M);
}

int dv_gather_transposed_gemv_partial_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                                          const void* idx, int idx_bytes, int B, int N, int Z, int M, void* y,
                                          void* partial, size_t partial_bytes, int* groups, void* stream) {
  if (!W || !y || !x || !idx || !groups || N <= 0 || Z <= 0 || M < 1 || !idx_ok(idx_bytes)) return DV_ERR_INVALID_ARG;
  if (B <= kColsVecMaxBatch || B > 64) return DV_ERR_UNSUPPORTED;  // the matrix-core path of dv_gather_transposed_gemv_f16
  if (N % 8 || ldw % 8 || ldw < N || !aligned16(W) || !aligned16(y) || (partial && !aligned16(partial)))
    return DV_ERR_ALIGNMENT;
  LnTail tail{};
  tail.deferred_groups = groups;
  return gather_cols_mfma(reinterpret_cast<const half_t*>(x), M, 0, reinterpret_cast<const half_t*>(W), ldw,
                          reinterpret_cast<const half_t*>(bias), idx, idx_bytes, 1, B, N, Z, M,
                          reinterpret_cast<half_t*>(y), partial, partial_bytes, reinterpret_cast<hipStream_t>(stream),
                          &tail);
}

int dv_reduce_rows_f16(const void* partial, int groups, const void* bias, int rows, int N, void* y, void* stream) {
  if (!y || groups < 1 || rows < 1 || N <= 0 || (groups > 1 && !partial)) return DV_ERR_INVALID_ARG;
  if (N % 8 || !aligned16(y) || (partial && !aligned16(partial))) return DV_ERR_ALIGNMENT;
  launch_cols_reduce(reinterpret_cast<const float*>(partial), reinterpret_cast<const half_t*>(bias), groups, rows, N,
                     reinterpret_cast<half_t*>(y), nullptr, reinterpret_cast<hipStream_t>(stream));
  return launch_status();
}

}  // extern "C"
namespace {
// Scratch of dv_gather_transposed_gemv_static_f16: one array per device, resident until the
// process ends.  In host code the array's name is only a handle: the device address comes from
// hipGetSymbolAddress, once per device, and is what the kernels are given.
// The array is DV_STATIC_SCRATCH_STREAMS slots of DV_STATIC_SCRATCH_BYTES: a stream keeps the slot it
// was given at its first call (calls on one stream are ordered by the stream), so calls on
// different streams never share partial sums.
__device__ __align__(256) unsigned char scratch[(size_t)DV_STATIC_SCRATCH_STREAMS * DV_STATIC_SCRATCH_BYTES];
std::atomic<void*> scratch_ptr[kMaxDevices];
std::atomic<uintptr_t> scratch_owner[kMaxDevices][DV_STATIC_SCRATCH_STREAMS];  // stream handle + 1, 0: free

// Slot of `stream` on device `dev` (taken on first use), or -1 when every slot belongs to another stream.
int static_scratch_slot(int dev, void* stream) {
  const uintptr_t key = reinterpret_cast<uintptr_t>(stream) + 1;
  for (int i = 0; i < DV_STATIC_SCRATCH_STREAMS; ++i) {
    uintptr_t cur = scratch_owner[dev][i].load(std::memory_order_acquire);
    if (cur == key) return i;
    if (cur == 0 && scratch_owner[dev][i].compare_exchange_strong(cur, key, std::memory_order_acq_rel)) return i;
    if (cur == key) return i;  // another thread registered the same stream meanwhile
  }
  return -1;
}

int static_scratch(void** out, void* stream) {
  const int dev = current_device();
  if (dev < 0) return DV_ERR_UNSUPPORTED;
  const int slot = static_scratch_slot(dev, stream);
  if (slot < 0) return DV_ERR_UNSUPPORTED;
  void* p = scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return DV_ERR_LAUNCH;
    }
    scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = static_cast<unsigned char*>(p) + (size_t)slot * DV_STATIC_SCRATCH_BYTES;
  return DV_OK;
}
}  // namespace
extern "C" {

int dv_gather_transposed_gemv_static_f16(const void* x, const void* W, int64_t ldw, const void* bias,
                                         const void* idx, int idx_bytes, int B, int N, int Z, int M,
                                         void* y, void* stream) {
  if (B < 1 || N < 1 || M < 0) return DV_ERR_INVALID_ARG;
  if (B > 64) return DV_ERR_UNSUPPORTED;
  // the partial sums of this shape must fit the fixed array; nothing is allocated here
  const size_t need = dv_gather_transposed_gemv_workspace_bytes(B, N, M);
  if (need > (size_t)DV_STATIC_SCRATCH_BYTES) return DV_ERR_WORKSPACE;
  void* ws = nullptr;
  if (int rc = static_scratch(&ws, stream); rc != DV_OK) return rc;
  // every word of the partial sums is written before it is read: nothing to clear between calls
  return dv_gather_transposed_gemv_f16(x, W, ldw, bias, idx, idx_bytes, B, N, Z, M, y, ws,
                                       (size_t)DV_STATIC_SCRATCH_BYTES, stream);
}

int dv_qkv_proj_sparse_cache_f16(const void* x, const void* W, const void* bias,
                                 const void* head_idx, const void* batch_idx, int nb, int d, int H,
                                 int hd, int nnz, void* y, void* k_cache, void* v_cache,
                                 const void* padding, int S, void* stream) {
  if (!x || !W || !y || nb < 1 || d <= 0 || H <= 0 || nnz < 0 || (nnz > 0 && (!head_idx || !batch_idx)) ||
      ((k_cache == nullptr) != (v_cache == nullptr)) || (k_cache && S <= 0))
    return DV_ERR_INVALID_ARG;
  if (nb > 16 || (hd != 32 && hd != 64 && hd != 128)) return DV_ERR_UNSUPPORTED;
  if (d % 8 || !aligned16(x) || !aligned16(W)) return DV_ERR_ALIGNMENT;
  if (nnz == 0) return DV_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const half_t* xx = reinterpret_cast<const half_t*>(x);
  const half_t* ww = reinterpret_cast<const half_t*>(W);
  const half_t* bb = reinterpret_cast<const half_t*>(bias);
  const int* hi = reinterpret_cast<const int*>(head_idx);
  const int* bi = reinterpret_cast<const int*>(batch_idx);
  half_t* yy = reinterpret_cast<half_t*>(y);
  half_t* kc = reinterpret_cast<half_t*>(k_cache);
  half_t* vc = reinterpret_cast<half_t*>(v_cache);
  const int* pad = reinterpret_cast<const int*>(padding);
  if (qkv_use_mfma(nb))
    return launch_qkv_mfma(xx, ww, bb, hi, bi, nb, d, H, hd, nnz, yy, kc, vc, pad, S, s);
  return launch_qkv<1>(xx, ww, bb, hi, bi, nb, d, H, hd, nnz, yy, kc, vc, pad, S, s);
}

int dv_qkv_proj_sparse_f16(const void* x, const void* W, const void* bias, const void* head_idx,
                           const void* batch_idx, int nb, int d, int H, int hd, int nnz, void* y,
                           void* stream) {
  return dv_qkv_proj_sparse_cache_f16(x, W, bias, head_idx, batch_idx, nb, d, H, hd, nnz, y, nullptr,
                                      nullptr, nullptr, 0, stream);
}

// Batches from which the X-shared split-K kernel takes over from the one that fetches X per 16-row tile
constexpr int kQkvTiledMinBatch = 9;

size_t dv_qkv_proj_batch_workspace_bytes(int B, int d, int nnz, int hd) {
  if (B < kQkvTiledMinBatch || B > 32 || d <= 0 || nnz <= 0 || hd <= 0) return 0;
  return tiled_workspace_bytes(B, d, 3 * nnz * hd);
}

int dv_qkv_proj_batch_f16(const void* x, int64_t ldx, const void* W, const void* bias, const void* head_idx,
                          const void* live, int live_stride, int nnz, int B, int d, int H, int hd, void* y,
                          void* k_cache, void* v_cache, const void* positions, int per_sample, int pos_add,
                          int S, void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !W || !y || B < 1 || d <= 0 || H <= 0 || nnz < 0 || (nnz > 0 && !head_idx) ||
      ((k_cache == nullptr) != (v_cache == nullptr)) || (k_cache && S <= 0) || (live && live_stride < 1))
    return DV_ERR_INVALID_ARG;
  if (B > 32 || (hd != 32 && hd != 64 && hd != 128)) return DV_ERR_UNSUPPORTED;
  // y and the caches take 8-byte vector stores
  if (d % 8 || ldx % 8 || ldx < d || !aligned16(x) || !aligned16(W) || !aligned8(y) || !aligned8(k_cache) ||
      !aligned8(v_cache))
    return DV_ERR_ALIGNMENT;
  if (nnz == 0) return DV_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (B >= kQkvTiledMinBatch && (dv_qkv_proj_batch_workspace_bytes(B, d, nnz, hd) == 0 ||
                                 (workspace != nullptr && aligned16(workspace) &&
                                  workspace_bytes >= dv_qkv_proj_batch_workspace_bytes(B, d, nnz, hd)))) {
    const QkvScatter qs{reinterpret_cast<const int*>(head_idx), reinterpret_cast<const int*>(live), live_stride, nnz, H,
                        hd, reinterpret_cast<half_t*>(k_cache), reinterpret_cast<half_t*>(v_cache),
                        reinterpret_cast<const int*>(positions), per_sample, pos_add, S, B, 1, 0, 0};
    return gemm_tiled_qkv(reinterpret_cast<const half_t*>(x), ldx, reinterpret_cast<const half_t*>(W),
                          reinterpret_cast<const half_t*>(bias), B, d, reinterpret_cast<half_t*>(y), qs, workspace,
                          workspace_bytes, s);
  }
  const dim3 grid(nnz * 3 * (hd / 16));
#define DV_QB(XT)                                                                                          \
  hipLaunchKernelGGL((qkv_batch_mfma_kernel<kQkvMfmaWaves, XT>), grid, dim3(kQkvMfmaWaves * 64), 0, s,      \
                     reinterpret_cast<const half_t*>(x), ldx, reinterpret_cast<const half_t*>(W),          \
                     reinterpret_cast<const half_t*>(bias), reinterpret_cast<const int*>(head_idx),        \
                     reinterpret_cast<const int*>(live), live_stride, B, d, H, hd, nnz,                    \
                     reinterpret_cast<half_t*>(y), reinterpret_cast<half_t*>(k_cache),                     \
                     reinterpret_cast<half_t*>(v_cache), reinterpret_cast<const int*>(positions), per_sample, \
                     pos_add, S)
  if (B <= 16) DV_QB(1);
  else DV_QB(2);
#undef DV_QB
  return launch_status();
}

int dv_prefill_attention_f16(const void* qkv, int B, int T, int H, int hd, float scale, void* ctx, void* k_cache,
                             void* v_cache, int pos0, int S, void* stream) {
  if (!qkv || !ctx || B < 1 || T < 0 || H <= 0 || ((k_cache == nullptr) != (v_cache == nullptr)) ||
      (k_cache && (S <= 0 || pos0 < 0 || pos0 + T > S)))
    return DV_ERR_INVALID_ARG;
  if (hd != 64 && hd != 128) return DV_ERR_UNSUPPORTED;
  if (!aligned16(qkv) || (k_cache && (!aligned16(k_cache) || !aligned16(v_cache)))) return DV_ERR_ALIGNMENT;
  if (T == 0) return DV_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid((T + kPfWaves * 16 - 1) / (kPfWaves * 16), H, B);
  if (hd == 128)
    hipLaunchKernelGGL(prefill_attn_kernel<128>, grid, dim3(kPfWaves * 64), 0, s, reinterpret_cast<const half_t*>(qkv),
                       T, H, scale, reinterpret_cast<half_t*>(ctx), reinterpret_cast<half_t*>(k_cache),
                       reinterpret_cast<half_t*>(v_cache), pos0, S);
  else
    hipLaunchKernelGGL(prefill_attn_kernel<64>, grid, dim3(kPfWaves * 64), 0, s, reinterpret_cast<const half_t*>(qkv),
                       T, H, scale, reinterpret_cast<half_t*>(ctx), reinterpret_cast<half_t*>(k_cache),
                       reinterpret_cast<half_t*>(v_cache), pos0, S);
  return launch_status();
}

int dv_kv_cache_copy_sparse_f16(const void* k, const void* v, int64_t ld_src, int nsrc,
                                void* k_cache, void* v_cache, const void* head_idx,
                                const void* seq_idx, int nnz, int nslots, const void* padding,
                                int H, int hd, int S, void* stream) {
  if ((!k_cache && !v_cache) || (k_cache && !k) || (v_cache && !v) || nsrc < 0 || nnz < 0 ||
      nslots < 0 || H <= 0 || S <= 0 || (nnz > 0 && nslots > 0 && (!head_idx || !seq_idx)))
    return DV_ERR_INVALID_ARG;
  if (hd % 8 || hd > 1024 || hd <= 0) return DV_ERR_UNSUPPORTED;
  if (nnz == 0 || nslots == 0 || nsrc == 0) return DV_OK;
  hipLaunchKernelGGL(kv_cache_copy_kernel, dim3(nnz, nslots), dim3(hd), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const half_t*>(k),
                     reinterpret_cast<const half_t*>(v), ld_src, nsrc,
                     reinterpret_cast<half_t*>(k_cache), reinterpret_cast<half_t*>(v_cache),
                     reinterpret_cast<const int*>(head_idx), reinterpret_cast<const int*>(seq_idx),
                     nslots, reinterpret_cast<const int*>(padding), H, hd, S);
  return launch_status();
}

int dv_window_step_f16(const void* x, void* x_cache, int d, void* tracker, const void* head_idx,
                       int nnz, int H, int counter, int flush, void* batch_idx, void* stream) {
  if (!x || !x_cache || !tracker || !batch_idx || d <= 0 || H <= 0 || nnz < 0 || counter < 0 ||
      counter > 15 || (!flush && nnz > 0 && !head_idx))
    return DV_ERR_INVALID_ARG;
  const int work = d > H * 16 ? d : H * 16;
  int blocks = (work + 255) / 256;
  if (blocks > 64) blocks = 64;
  hipLaunchKernelGGL(window_step_kernel, dim3(blocks), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const half_t*>(x),
                     reinterpret_cast<half_t*>(x_cache), d, reinterpret_cast<int*>(tracker),
                     reinterpret_cast<const int*>(head_idx), nnz, H, counter, flush,
                     reinterpret_cast<int*>(batch_idx));
  return launch_status();
}

int dv_kv_append_f16(const void* k, const void* v, int64_t ld_src, void* k_cache, void* v_cache,
                     const void* head_idx, int nheads, const void* lengths, int pos, int B, int H,
                     int hd, int S, void* stream) {
  if (!k || !v || !k_cache || !v_cache || nheads < 0 || B < 1 || H <= 0 || S <= 0)
    return DV_ERR_INVALID_ARG;
  if (hd % 8 || hd > 1024 || hd <= 0) return DV_ERR_UNSUPPORTED;
  if (!lengths && (pos < 0 || pos >= S)) return DV_ERR_INVALID_ARG;
  const int heads = head_idx ? nheads : H;
  if (heads == 0) return DV_OK;
  hipLaunchKernelGGL(kv_append_kernel, dim3(heads, B), dim3(hd), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const half_t*>(k),
                     reinterpret_cast<const half_t*>(v), ld_src, reinterpret_cast<half_t*>(k_cache),
                     reinterpret_cast<half_t*>(v_cache), reinterpret_cast<const int*>(head_idx),
                     reinterpret_cast<const int*>(lengths), pos, H, hd, S);
  return launch_status();
}

size_t dv_decode_attention_workspace_bytes(int B, int nheads, int n_len, int hd) {
  if (B < 1 || nheads < 0 || n_len < 0 || hd <= 0) return 0;
  return (size_t)B * nheads * attn_splits(n_len) * (hd + 2) * sizeof(float);
}

namespace {
int launch_attn_partials(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                         const void* head_idx, int heads, const void* lengths, int n_len, int B, int H,
                         int hd, int S, float scale, float* part, hipStream_t s) {
  const int nsplit = attn_splits(n_len);
  const half_t* qq = reinterpret_cast<const half_t*>(q);
  const half_t* kc = reinterpret_cast<const half_t*>(k_cache);
  const half_t* vc = reinterpret_cast<const half_t*>(v_cache);
  const int* hi = reinterpret_cast<const int*>(head_idx);
  const int* ln = reinterpret_cast<const int*>(lengths);
  dim3 grid(nsplit, heads, B);
  if (hd == 128)
    hipLaunchKernelGGL((decode_attn_kernel<128, kAttnWaves>), grid, dim3(kAttnWaves * 64), 0, s, qq,
                       ldq, kc, vc, hi, ln, n_len, H, S, scale, nsplit, part);
  else if (hd == 64)
    hipLaunchKernelGGL((decode_attn_kernel<64, kAttnWaves>), grid, dim3(kAttnWaves * 64), 0, s, qq,
                       ldq, kc, vc, hi, ln, n_len, H, S, scale, nsplit, part);
  else
    hipLaunchKernelGGL((decode_attn_kernel<32, kAttnWaves>), grid, dim3(kAttnWaves * 64), 0, s, qq,
                       ldq, kc, vc, hi, ln, n_len, H, S, scale, nsplit, part);
  return launch_status();
}

// hd32: the caller also has the 32-wide head kernels (the attention alone has; the entry points that
// go on into out_proj do not)
int check_attn_args(const void* q, int64_t ldq, const void* k_cache, const void* v_cache, int nheads,
                    int n_len, int B, int H, int hd, int S, bool hd32 = false) {
  if (!q || !k_cache || !v_cache || nheads < 0 || B < 1 || H <= 0 || S <= 0 || n_len < 1 || n_len > S)
    return DV_ERR_INVALID_ARG;
  if (hd != 64 && hd != 128 && !(hd32 && hd == 32)) return DV_ERR_UNSUPPORTED;
  if (ldq % 8 || !aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache)) return DV_ERR_ALIGNMENT;
  return DV_OK;
}
}  // namespace

int dv_decode_attention_f16(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                            const void* head_idx, int nheads, const void* lengths, int n_len,
                            int B, int H, int hd, int S, float scale, void* out, int64_t ldo,
                            void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_attn_args(q, ldq, k_cache, v_cache, nheads, n_len, B, H, hd, S, true);
  if (rc != DV_OK) return rc;
  if (!out) return DV_ERR_INVALID_ARG;
  const int heads = head_idx ? nheads : H;
  if (heads == 0) return DV_OK;
  if (!workspace || workspace_bytes < dv_decode_attention_workspace_bytes(B, heads, n_len, hd))
    return DV_ERR_WORKSPACE;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // Two and more (sequence, head) pairs per compute unit: one workgroup per pair fills the device, the
  // whole attention is one launch without partial results.  (At one pair per compute unit the kernel
  // itself is as fast as partials + combine, 44 us against 43 + 5 at 8 x 32 heads x 2048 positions,
  // but its 1024-lane workgroups hold back the small kernels of a concurrent stream more.)
  if ((int64_t)B * heads >= (int64_t)compute_units() * 2) {
    const half_t* qq = reinterpret_cast<const half_t*>(q);
    const half_t* kc = reinterpret_cast<const half_t*>(k_cache);
    const half_t* vc = reinterpret_cast<const half_t*>(v_cache);
    const int* hi = reinterpret_cast<const int*>(head_idx);
    const int* ln = reinterpret_cast<const int*>(lengths);
    half_t* oo = reinterpret_cast<half_t*>(out);
    const dim3 grid(heads, B);
    if (hd == 128)
      hipLaunchKernelGGL((decode_attn_rows_kernel<128>), grid, dim3(kAttnRowWaves * 64), 0, s, qq, ldq, kc, vc, hi, ln,
                         n_len, H, S, scale, oo, ldo);
    else if (hd == 64)
      hipLaunchKernelGGL((decode_attn_rows_kernel<64>), grid, dim3(kAttnRowWaves * 64), 0, s, qq, ldq, kc, vc, hi, ln,
                         n_len, H, S, scale, oo, ldo);
    else
      hipLaunchKernelGGL((decode_attn_rows_kernel<32>), grid, dim3(kAttnRowWaves * 64), 0, s, qq, ldq, kc, vc, hi, ln,
                         n_len, H, S, scale, oo, ldo);
    return launch_status();
  }
  float* part = reinterpret_cast<float*>(workspace);
  rc = launch_attn_partials(q, ldq, k_cache, v_cache, head_idx, heads, lengths, n_len, B, H, hd, S,
                            scale, part, s);
  if (rc != DV_OK) return rc;
  const int nsplit = attn_splits(n_len);
  const int* hi = reinterpret_cast<const int*>(head_idx);
  half_t* oo = reinterpret_cast<half_t*>(out);
  if (hd == 128)
    hipLaunchKernelGGL((decode_attn_combine_kernel<128>), dim3(heads, B), dim3(128), 0, s, part,
                       hi, H, nsplit, oo, ldo);
  else if (hd == 64)
    hipLaunchKernelGGL((decode_attn_combine_kernel<64>), dim3(heads, B), dim3(64), 0, s, part, hi,
                       H, nsplit, oo, ldo);
  else
    hipLaunchKernelGGL((decode_attn_combine_kernel<32>), dim3(heads, B), dim3(32), 0, s, part, hi,
                       H, nsplit, oo, ldo);
  return launch_status();
}

namespace {
// out_proj over the (N, H, hd) weight from attention partials (batch 1); rin / rout optional
constexpr int kOutRowsR = 4, kOutRowsWaves = 8;
inline size_t out_rows_lds_bytes(int nnz, int hd) { return (size_t)nnz * hd * sizeof(half_t) + (size_t)nnz * 4; }
inline int out_rows_blocks(int N) {
  const int ntasks = (N + kOutRowsR - 1) / kOutRowsR;
  int blocks = (ntasks + kOutRowsWaves - 1) / kOutRowsWaves;
  const int cap = compute_units() * 2;
  return blocks > cap ? cap : blocks;
}
int grant_out_rows_lds(int hd, size_t lds) {
  static LdsGrant grant[2];
  const int v = hd == 128 ? 1 : 0;
  const void* fn = v ? reinterpret_cast<const void*>(out_proj_rows_attn_kernel<kOutRowsR, 128>)
                     : reinterpret_cast<const void*>(out_proj_rows_attn_kernel<kOutRowsR, 64>);
  return grant[v].ensure(fn, lds);
}
int launch_out_rows_attn(const float* part, int nsplit, const half_t* W, const half_t* bias, const int* head_idx,
                         int nnz, int H, int hd, int N, half_t* y, const half_t* rin, half_t* rout,
                         hipStream_t s) {
  const size_t lds = out_rows_lds_bytes(nnz, hd);
  const int rc = grant_out_rows_lds(hd, lds);
  if (rc != DV_OK) return rc;
  const dim3 grid(out_rows_blocks(N));
  if (hd == 128)
    hipLaunchKernelGGL((out_proj_rows_attn_kernel<kOutRowsR, 128>), grid, dim3(64 * kOutRowsWaves), lds, s, part,
                       nsplit, W, bias, head_idx, nnz, H, N, y, rin, rout);
  else
    hipLaunchKernelGGL((out_proj_rows_attn_kernel<kOutRowsR, 64>), grid, dim3(64 * kOutRowsWaves), lds, s, part,
                       nsplit, W, bias, head_idx, nnz, H, N, y, rin, rout);
  return DV_OK;
}
}  // namespace

int dv_attention_out_proj_rows_f16(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                                   const void* head_idx, int nheads, const void* lengths, int n_len, int H,
                                   int hd, int S, float scale, const void* W, const void* bias, int N,
                                   void* y, const void* residual_in, void* residual_out, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  int rc = check_attn_args(q, ldq, k_cache, v_cache, nheads, n_len, 1, H, hd, S);
  if (rc != DV_OK) return rc;
  if (!head_idx || !W || !y || N <= 0 || nheads < 1 || (residual_out && !residual_in)) return DV_ERR_INVALID_ARG;
  if (!aligned16(W)) return DV_ERR_ALIGNMENT;
  if (!workspace || !aligned16(workspace) ||
      workspace_bytes < dv_decode_attention_workspace_bytes(1, nheads, n_len, hd))
    return DV_ERR_WORKSPACE;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  float* part = reinterpret_cast<float*>(workspace);
  rc = launch_attn_partials(q, ldq, k_cache, v_cache, head_idx, nheads, lengths, n_len, 1, H, hd, S, scale,
                            part, s);
  if (rc != DV_OK) return rc;
  rc = launch_out_rows_attn(part, attn_splits(n_len), reinterpret_cast<const half_t*>(W),
                            reinterpret_cast<const half_t*>(bias), reinterpret_cast<const int*>(head_idx), nheads,
                            H, hd, N, reinterpret_cast<half_t*>(y), reinterpret_cast<const half_t*>(residual_in),
                            reinterpret_cast<half_t*>(residual_out), s);
  if (rc != DV_OK) return rc;
  return launch_status();
}

size_t dv_attention_out_proj_workspace_bytes(int B, int nheads, int n_len, int hd, int N) {
  if (B < 1 || nheads < 0 || n_len < 0 || hd <= 0 || N < 1) return 0;
  size_t a = dv_decode_attention_workspace_bytes(B, nheads, n_len, hd);
  a = (a + 255) & ~(size_t)255;
  return a + cols_workspace_bytes(B, N, nheads * hd);
}

int dv_attention_out_proj_f16(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                              const void* head_idx, int nheads, const void* lengths, int n_len,
                              int B, int H, int hd, int S, float scale, const void* Wt, int64_t ldw,
                              const void* bias, int N, void* y, void* workspace,
                              size_t workspace_bytes, void* stream) {
  int rc = check_attn_args(q, ldq, k_cache, v_cache, nheads, n_len, B, H, hd, S);
  if (rc != DV_OK) return rc;
  if (!head_idx || !Wt || !y || N <= 0) return DV_ERR_INVALID_ARG;
  if (B > 4) return DV_ERR_UNSUPPORTED;
  if (N % 8 || ldw % 8 || ldw < N || !aligned16(Wt)) return DV_ERR_ALIGNMENT;
  if (!workspace || !aligned16(workspace) ||
      workspace_bytes < dv_attention_out_proj_workspace_bytes(B, nheads, n_len, hd, N))
    return DV_ERR_WORKSPACE;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // layout: [out_proj partial sums][attention partials]
  const size_t cols_bytes = (cols_workspace_bytes(B, N, nheads * hd) + 255) & ~(size_t)255;
  unsigned char* base = reinterpret_cast<unsigned char*>(workspace);
  float* part = reinterpret_cast<float*>(base + cols_bytes);
  if (nheads > 0) {
    rc = launch_attn_partials(q, ldq, k_cache, v_cache, head_idx, nheads, lengths, n_len, B, H, hd, S,
                              scale, part, s);
    if (rc != DV_OK) return rc;
  }
  const int M = nheads * hd;
  const ColsPlan p = plan_cols(N, M);
  float* partial = reinterpret_cast<float*>(base);
  const half_t* ww = reinterpret_cast<const half_t*>(Wt);
  const half_t* bb = reinterpret_cast<const half_t*>(bias);
  half_t* yy = reinterpret_cast<half_t*>(y);
  dim3 grid(p.col_tiles, p.groups);
  const int nsplit = attn_splits(n_len);
#define DV_AO(BB)                                                                                 \
  hipLaunchKernelGGL((gather_cols_kernel<BB, 8, false, true, true>), grid, dim3(256), 0, s, \
                     (const half_t*)nullptr, (int64_t)0, 1, ww, ldw, bb, head_idx, hd, N, H * hd, M, \
                     p.rows_per_block, partial, yy, part, nsplit, 1)
  switch (B) {
    case 1: DV_AO(1); break;
    case 2: DV_AO(2); break;
    case 3: DV_AO(3); break;
    default: DV_AO(4); break;
  }
#undef DV_AO
  // the row groups' partial sums are added in fixed point: the same bits as the fused layer step,
  // which adds them with integer atomics
  const int64_t total = (int64_t)B * N;
  hipLaunchKernelGGL(cols_reduce_kernel<true>, dim3((unsigned)((total + 63) / 64)), dim3(256), 0, s, partial, bb,
                     p.groups, B, N, yy, (const half_t*)nullptr, (half_t*)nullptr);
  return launch_status();
}

int dv_out_proj_sparse_f16(const void* x, const void* W, const void* bias, const void* head_idx,
                           int nnz, int B, int H, int hd, int N, void* y, void* stream) {
  if (!x || !W || !y || nnz < 0 || B < 1 || H <= 0 || N <= 0 || (nnz > 0 && !head_idx))
    return DV_ERR_INVALID_ARG;
  if (B > 16 || (hd != 32 && hd != 64 && hd != 128)) return DV_ERR_UNSUPPORTED;
  if (!aligned16(x) || !aligned16(W)) return DV_ERR_ALIGNMENT;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  constexpr int R = 4;
  const int ntasks = (N + R - 1) / R;
  int blocks = (ntasks + 3) / 4;
  const int cap = compute_units() * 8;
  if (blocks > cap) blocks = cap;
  // up to four batch rows share one pass over the weights; larger batches (the reference takes up
  // to 16) run as passes of four: this layout is kept for compatibility, the transposed weight
  // (dv_out_proj_sparse_t_f16) is the one that streams a batch in a single pass
  for (int b0 = 0; b0 < B; b0 += 4) {
    const int nb = B - b0 < 4 ? B - b0 : 4;
    const half_t* xx = reinterpret_cast<const half_t*>(x) + (int64_t)b0 * H * hd;
    half_t* yy = reinterpret_cast<half_t*>(y) + (int64_t)b0 * N;
#define DV_OP(BB, HH)                                                                          \
  hipLaunchKernelGGL((out_proj_rows_kernel<BB, R, HH>), dim3(blocks), dim3(256), 0, s, xx,      \
                     reinterpret_cast<const half_t*>(W), reinterpret_cast<const half_t*>(bias), \
                     reinterpret_cast<const int*>(head_idx), nnz, H, N, yy)
#define DV_OPB(HH)                                                                   \
  switch (nb) {                                                                      \
    case 1: DV_OP(1, HH); break;                                                     \
    case 2: DV_OP(2, HH); break;                                                     \
    case 3: DV_OP(3, HH); break;                                                     \
    default: DV_OP(4, HH);                                                           \
  }
    if (hd == 128) { DV_OPB(128) } else if (hd == 64) { DV_OPB(64) } else { DV_OPB(32) }
#undef DV_OPB
#undef DV_OP
  }
  return launch_status();
}

size_t dv_out_proj_sparse_t_workspace_bytes(int B, int N, int nnz, int hd) {
  if (B < 1 || N < 1 || nnz < 0 || hd < 1) return 0;
  return B > kColsVecMaxBatch ? cols_mfma_workspace_bytes(B, N, nnz * hd) : cols_workspace_bytes(B, N, nnz * hd);
}

int dv_out_proj_sparse_t_f16(const void* x, const void* Wt, int64_t ldw, const void* bias,
                             const void* head_idx, int nnz, int B, int H, int hd, int N, void* y,
                             void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !Wt || !y || nnz < 0 || B < 1 || H <= 0 || hd <= 0 || N <= 0 || (nnz > 0 && !head_idx))
    return DV_ERR_INVALID_ARG;
  if (B > 64) return DV_ERR_UNSUPPORTED;
  if (N % 8 || ldw % 8 || ldw < N || !aligned16(Wt) || !aligned16(y) || (workspace && !aligned16(workspace)))
    return DV_ERR_ALIGNMENT;
  if (B > kColsVecMaxBatch)
    return gather_cols_mfma(reinterpret_cast<const half_t*>(x), (int64_t)H * hd, 1,
                            reinterpret_cast<const half_t*>(Wt), ldw, reinterpret_cast<const half_t*>(bias),
                            head_idx, 4, hd, B, N, H * hd, nnz * hd, reinterpret_cast<half_t*>(y), workspace,
                            workspace_bytes, reinterpret_cast<hipStream_t>(stream));
  // one and two rows: partial sums added in fixed point, the bits of dv_attention_out_proj_f16 and of
  // the fused layer step
  return gather_cols(reinterpret_cast<const half_t*>(x), (int64_t)H * hd, 1,
                     reinterpret_cast<const half_t*>(Wt), ldw, reinterpret_cast<const half_t*>(bias),
                     head_idx, 4, hd, B, N, H * hd, nnz * hd, reinterpret_cast<half_t*>(y),
                     workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream), true);
}

int dv_out_proj_sparse_t_ln_f16(const void* x, const void* Wt, int64_t ldw, const void* bias, const void* head_idx,
                                int nnz, int B, int H, int hd, int N, const void* residual, const void* gamma,
                                const void* beta, float eps, void* normed, void* residual_out, void* workspace,
                                size_t workspace_bytes, void* stream) {
  if (!x || !Wt || !normed || !gamma || !beta || nnz < 1 || B < 1 || H <= 0 || hd <= 0 || N <= 0 || !head_idx)
    return DV_ERR_INVALID_ARG;
  if (B <= kColsVecMaxBatch || B > 64 || N > 256 * 8 * 16) return DV_ERR_UNSUPPORTED;  // the matrix-core path of dv_out_proj_sparse_t_f16
  if (N % 8 || ldw % 8 || ldw < N || !aligned16(Wt) || !aligned16(normed) || !aligned16(gamma) || !aligned16(beta) ||
      (residual && !aligned16(residual)) || (residual_out && !aligned16(residual_out)) ||
      (workspace && !aligned16(workspace)))
    return DV_ERR_ALIGNMENT;
  // the product's own output row block (needed when a single row group stores it directly) sits behind the partials
  const size_t part_bytes = cols_mfma_workspace_bytes(B, N, nnz * hd);
  const size_t y_off = (part_bytes + 255) & ~(size_t)255;
  if (!workspace || workspace_bytes < y_off + (size_t)B * N * sizeof(half_t)) return DV_ERR_WORKSPACE;
  const LnTail tail{reinterpret_cast<const half_t*>(residual), reinterpret_cast<const half_t*>(gamma),
                    reinterpret_cast<const half_t*>(beta), eps, reinterpret_cast<half_t*>(normed),
                    reinterpret_cast<half_t*>(residual_out)};
  half_t* y = reinterpret_cast<half_t*>(reinterpret_cast<unsigned char*>(workspace) + y_off);
  return gather_cols_mfma(reinterpret_cast<const half_t*>(x), (int64_t)H * hd, 1, reinterpret_cast<const half_t*>(Wt),
                          ldw, reinterpret_cast<const half_t*>(bias), head_idx, 4, hd, B, N, H * hd, nnz * hd, y,
                          workspace, part_bytes, reinterpret_cast<hipStream_t>(stream), &tail);
}

size_t dv_out_proj_sparse_t_ln_workspace_bytes(int B, int nnz, int hd, int N) {
  if (B <= kColsVecMaxBatch || B > 64 || nnz <= 0 || hd <= 0 || N <= 0) return 0;
  return ((cols_mfma_workspace_bytes(B, N, nnz * hd) + 255) & ~(size_t)255) + (size_t)B * N * sizeof(half_t);
}

size_t dv_qkv_window_batch_workspace_bytes(int tokens, int nseq, int d, int nnz, int hd) {
  if (tokens < 1 || tokens > 16 || nseq < 1 || nseq > 32 || d <= 0 || nnz <= 0 || hd <= 0) return 0;
  return tiled_workspace_bytes(tokens * nseq, d, 3 * nnz * hd);
}

int dv_qkv_window_batch_f16(const void* x, int64_t ldx, const void* W, const void* bias, const void* head_idx,
                            const void* batch_idx, int nnz, int tokens, int nseq, int d, int H, int hd, void* y,
                            void* k_cache, void* v_cache, const void* positions, int per_sample, int pos_add,
                            int S, void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !W || !y || !batch_idx || tokens < 1 || nseq < 1 || d <= 0 || H <= 0 || nnz < 0 ||
      (nnz > 0 && !head_idx) || ((k_cache == nullptr) != (v_cache == nullptr)) || (k_cache && S <= 0))
    return DV_ERR_INVALID_ARG;
  if (tokens > 16 || nseq > 32 || (hd != 32 && hd != 64 && hd != 128)) return DV_ERR_UNSUPPORTED;
  if (d % 8 || ldx % 8 || ldx < d || !aligned16(x) || !aligned16(W) || !aligned8(y) || !aligned8(k_cache) ||
      !aligned8(v_cache))
    return DV_ERR_ALIGNMENT;
  if (nnz == 0) return DV_OK;
  const QkvScatter qs{reinterpret_cast<const int*>(head_idx), reinterpret_cast<const int*>(batch_idx), tokens, nnz, H,
                      hd, reinterpret_cast<half_t*>(k_cache), reinterpret_cast<half_t*>(v_cache),
                      reinterpret_cast<const int*>(positions), per_sample, pos_add, S, nseq, tokens, 1, tokens - 1};
  return gemm_tiled_qkv(reinterpret_cast<const half_t*>(x), ldx, reinterpret_cast<const half_t*>(W),
                        reinterpret_cast<const half_t*>(bias), tokens * nseq, d, reinterpret_cast<half_t*>(y), qs,
                        workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}

int dv_add_layer_norm_f16(const void* h, const void* residual, const void* gamma, const void* beta,
                          float eps, int rows, int d, void* y, void* residual_out, void* stream) {
  if (!h || !gamma || !beta || !y || rows < 0 || d <= 0) return DV_ERR_INVALID_ARG;
  if (d % 8 || !aligned16(h) || !aligned16(y) || !aligned16(gamma) || !aligned16(beta) ||
      (residual && !aligned16(residual)) || (residual_out && !aligned16(residual_out)))
    return DV_ERR_ALIGNMENT;
  if (d > 256 * 8 * 16) return DV_ERR_UNSUPPORTED;
  if (rows == 0) return DV_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define DV_LN(T, V)                                                                              \
  hipLaunchKernelGGL((add_layer_norm_kernel<T, V>), dim3(rows), dim3(T), 0, s,                    \
                     reinterpret_cast<const half_t*>(h), reinterpret_cast<const half_t*>(residual), \
                     reinterpret_cast<const half_t*>(gamma), reinterpret_cast<const half_t*>(beta), \
                     eps, d, reinterpret_cast<half_t*>(y), reinterpret_cast<half_t*>(residual_out))
  if (d <= 256 * 8 * 1)
    DV_LN(256, 1);
  else if (d <= 512 * 8 * 1)
    DV_LN(512, 1);
  else if (d <= 1024 * 8 * 1)
    DV_LN(1024, 1);
  else if (d <= 1024 * 8 * 2)
    DV_LN(1024, 2);
  else
    DV_LN(1024, 4);
#undef DV_LN
  return launch_status();
}

int dv_add_layer_norm_window_f16(const void* h, const void* residual, const void* gamma, const void* beta,
                                 float eps, int rows, int d, void* y, void* residual_out, void* x_cache_row,
                                 void* tracker, const void* head_idx, int nnz, int H, int counter, int flush,
                                 void* batch_idx, void* stream) {
  if (!h || !gamma || !beta || !y || !x_cache_row || !tracker || !batch_idx || rows < 1 || d <= 0 || H <= 0 ||
      nnz < 0 || counter < 0 || counter > 15 || (!flush && nnz > 0 && !head_idx))
    return DV_ERR_INVALID_ARG;
  if (d % 8 || !aligned16(h) || !aligned16(y) || !aligned16(gamma) || !aligned16(beta) || !aligned16(x_cache_row) ||
      (residual && !aligned16(residual)) || (residual_out && !aligned16(residual_out)))
    return DV_ERR_ALIGNMENT;
  if (d > 256 * 8 * 16) return DV_ERR_UNSUPPORTED;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define DV_LNW(T, V)                                                                                          \
  hipLaunchKernelGGL((add_layer_norm_window_kernel<T, V>), dim3(rows + 1), dim3(T), 0, s,                      \
                     reinterpret_cast<const half_t*>(h), reinterpret_cast<const half_t*>(residual),           \
                     reinterpret_cast<const half_t*>(gamma), reinterpret_cast<const half_t*>(beta), eps, d,    \
                     reinterpret_cast<half_t*>(y), reinterpret_cast<half_t*>(residual_out),                   \
                     reinterpret_cast<half_t*>(x_cache_row), rows, reinterpret_cast<int*>(tracker),            \
                     reinterpret_cast<const int*>(head_idx), nnz, H, counter, flush,                          \
                     reinterpret_cast<int*>(batch_idx))
  if (d <= 256 * 8 * 1)
    DV_LNW(256, 1);
  else if (d <= 512 * 8 * 1)
    DV_LNW(512, 1);
  else if (d <= 1024 * 8 * 1)
    DV_LNW(1024, 1);
  else if (d <= 1024 * 8 * 2)
    DV_LNW(1024, 2);
  else
    DV_LNW(1024, 4);
#undef DV_LNW
  return launch_status();
}

int dv_reduce_add_layer_norm_window_f16(const void* partial, int groups, const void* bias, const void* h,
                                        const void* residual, const void* gamma, const void* beta, float eps,
                                        int rows, int d, void* y, void* residual_out, void* x_cache_row,
                                        void* tracker, const void* head_idx, int nnz, int H, int counter, int flush,
                                        void* batch_idx, void* stream) {
  if (!gamma || !beta || !y || groups < 1 || rows < 1 || d <= 0 || (groups > 1 ? !partial : !h))
    return DV_ERR_INVALID_ARG;
  if (tracker && (!x_cache_row || !batch_idx || H <= 0 || nnz < 0 || counter < 0 || counter > 15 ||
                  (!flush && nnz > 0 && !head_idx)))
    return DV_ERR_INVALID_ARG;
  if (d % 8 || !aligned16(y) || !aligned16(gamma) || !aligned16(beta) || (partial && !aligned16(partial)) ||
      (h && !aligned16(h)) || (x_cache_row && !aligned16(x_cache_row)) || (residual && !aligned16(residual)) ||
      (residual_out && !aligned16(residual_out)) || (bias && !aligned16(bias)))
    return DV_ERR_ALIGNMENT;
  if (d > 256 * 8 * 16) return DV_ERR_UNSUPPORTED;
  if (!tracker) x_cache_row = nullptr;  // the window row belongs to the window step
  if (groups == 1) {  // the product stored its rows itself
    if (tracker)
      return dv_add_layer_norm_window_f16(h, residual, gamma, beta, eps, rows, d, y, residual_out, x_cache_row,
                                          tracker, head_idx, nnz, H, counter, flush, batch_idx, stream);
    return dv_add_layer_norm_f16(h, residual, gamma, beta, eps, rows, d, y, residual_out, stream);
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define DV_RLNW(T, V)                                                                                            \
  hipLaunchKernelGGL((reduce_add_layer_norm_window_kernel<T, V>), dim3(rows + (tracker ? 1 : 0)), dim3(T), 0, s, \
                     reinterpret_cast<const float*>(partial), reinterpret_cast<const half_t*>(bias), groups,     \
                     reinterpret_cast<const half_t*>(residual), reinterpret_cast<const half_t*>(gamma),          \
                     reinterpret_cast<const half_t*>(beta), eps, d, reinterpret_cast<half_t*>(y),                \
                     reinterpret_cast<half_t*>(residual_out), reinterpret_cast<half_t*>(x_cache_row), rows,      \
                     reinterpret_cast<int*>(tracker), reinterpret_cast<const int*>(head_idx), nnz, H, counter,   \
                     flush, reinterpret_cast<int*>(batch_idx))
  if (d <= 256 * 8 * 1)
    DV_RLNW(256, 1);
  else if (d <= 512 * 8 * 1)
    DV_RLNW(512, 1);
  else if (d <= 1024 * 8 * 1)
    DV_RLNW(1024, 1);
  else if (d <= 1024 * 8 * 2)
    DV_RLNW(1024, 2);
  else
    DV_RLNW(1024, 4);
#undef DV_RLNW
  return launch_status();
}

namespace {
struct LayerPlan {
  size_t off_topk, off_res1, off_parts, off_acc, off_qkv, off_batch_idx, off_hp_hidden, off_mp_hidden, off_h,
      off_head_logits, off_attn_part, off_cols_part, total;
  int nsplit;
  ColsPlan out_cols, fc2_cols;
};

inline size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

LayerPlan plan_layer(const dvSparseLayerArgs& a) {
  LayerPlan p;
  size_t o = 0;
  p.off_topk = o;
  o = align_up(o + dv_topk_workspace_bytes(a.ffn > 1024 ? a.ffn : 2048));
  p.off_res1 = o;         o = align_up(o + (size_t)a.d * 2);
  p.off_parts = o;        o = align_up(o + (size_t)((a.d + kLnPart - 1) / kLnPart) * sizeof(float2));
  p.off_acc = o;          o = align_up(o + (size_t)a.d * sizeof(long long));
  p.off_qkv = o;          o = align_up(o + (size_t)16 * 3 * a.H * a.hd * 2);
  p.off_batch_idx = o;    o = align_up(o + (size_t)a.H * 16 * 4);
  p.off_hp_hidden = o;    o = align_up(o + (size_t)a.r_att * 2);
  p.off_mp_hidden = o;    o = align_up(o + (size_t)a.r_mlp * 2);
  p.off_h = o;            o = align_up(o + (size_t)a.K * 2);
  p.off_head_logits = o;  o = align_up(o + (size_t)a.H * 2);
  p.nsplit = attn_splits(a.n_len > 0 ? a.S : 1);  // sized for the full cache
  p.off_attn_part = o;    o = align_up(o + (size_t)a.Hk * p.nsplit * (a.hd + 2) * 4);
  p.out_cols = plan_cols(a.d, a.Hk * a.hd);
  p.fc2_cols = plan_cols(a.d, a.K);
  p.off_cols_part = o;    o = align_up(o + (size_t)p.fc2_cols.groups * a.d * 4);
  p.total = o;
  return p;
}

int check_layer_args(const dvSparseLayerArgs& a, bool first) {
  if (!a.ln1_w || !a.ln1_b || !a.ln2_w || !a.ln2_b || !a.Wqkv || !a.Wout_t || !a.att_Wa ||
      !a.att_Wb || !a.W1 || !a.W2t || !a.mlp_Wa || !a.mlp_Wb || !a.head_idx || !a.mlp_logit_in ||
      !a.cache_offset || !a.k_cache || !a.v_cache || !a.x_cache || !a.tracker || !a.hidden_out ||
      !a.residual_out || !a.mlp_logit_out || !a.att_idx_out || !a.mlp_idx_out)
    return DV_ERR_INVALID_ARG;
  if (first && (!a.hidden || !a.workspace)) return DV_ERR_INVALID_ARG;
  if (a.d <= 0 || a.ffn <= 0 || a.H <= 0 || a.Hk < 1 || a.Hk > a.H || a.att_k < 1 || a.att_k > a.H ||
      a.K < 1 || a.K > a.ffn || a.r_att <= 0 || a.r_mlp <= 0 || a.S <= 0 || a.n_len < 1 || a.n_len > a.S ||
      a.counter < 0 || a.counter > 15 || (a.counter == 15 && a.Hk != a.H))
    return DV_ERR_INVALID_ARG;
  if ((a.hd != 64 && a.hd != 128) || a.H * a.hd != a.d || a.H > 1024 || a.ffn > 65536 || a.ffn <= 1024 ||
      a.d > 1024 * 8 * 4 || (size_t)a.d * 2 > 144 * 1024)
    return DV_ERR_UNSUPPORTED;
  if (a.d % 8 || a.ffn % 8 || a.r_att % 8 || a.r_mlp % 8) return DV_ERR_ALIGNMENT;
  return DV_OK;
}

// LayerNorm 1 + QKV (+ cache scatter) of a window position: one token on the vector ALUs, several on
// the matrix cores
int launch_ln_qkv(const QkvArgs& q, hipStream_t s) {
  const int cus = compute_units();
  const bool mfma = qkv_use_mfma(q.nb);
  const bool two = mfma && qkv_mfma_two_tiles(q.nnz, q.hd);
  if (mfma) {
    const dim3 grid(q.nnz * 3 * (q.hd / (two ? 32 : 16)));
    if (two) hipLaunchKernelGGL((layer_l2_kernel<-1>), grid, dim3(256), 0, s, q);
    else hipLaunchKernelGGL((layer_l2_kernel<0>), grid, dim3(256), 0, s, q);
  } else {
    // one task (two weight rows) per wavefront; workgroups of eight wavefronts when that still
    // leaves two per compute unit (fewer copies of the row to normalise), else of four
    const int ntasks = q.nnz * 3 * (q.hd / 2);
    const int waves = ntasks >= cus * 16 ? 8 : 4;
    int nq = (ntasks + waves - 1) / waves;
    if (nq > cus * (24 / waves)) nq = cus * (24 / waves);
    const size_t lds = (size_t)q.d * sizeof(half_t);
    static LdsGrant grant[2];
    if (q.d <= 16384) {
      if (int rc = grant[0].ensure(reinterpret_cast<const void*>(layer_l2_kernel<1>), lds); rc != DV_OK) return rc;
      hipLaunchKernelGGL((layer_l2_kernel<1>), dim3(nq), dim3(waves * 64), lds, s, q);
    } else {
      if (int rc = grant[1].ensure(reinterpret_cast<const void*>(layer_l2_kernel<2>), lds); rc != DV_OK) return rc;
      hipLaunchKernelGGL((layer_l2_kernel<2>), dim3(nq), dim3(waves * 64), lds, s, q);
    }
  }
  return launch_status();
}

// the scratch of a call is the first block's; every block of the call needs no more than it holds
size_t layers_workspace_bytes(const dvSparseLayerArgs* layers, int n) {
  size_t need = 0;
  for (int l = 0; l < n; ++l) {
    const size_t t = plan_layer(layers[l]).total;
    if (t > need) need = t;
  }
  return need;
}
}  // namespace

size_t dv_sparse_layer_workspace_bytes(const dvSparseLayerArgs* args) {
  if (!args || args->d <= 0 || args->ffn <= 0 || args->H <= 0 || args->Hk < 1 || args->K < 1) return 0;
  return plan_layer(*args).total;
}

int dv_sparse_layers_decode_f16(const dvSparseLayerArgs* layers, int n_layers, void* stream) {
  if (!layers || n_layers < 1) return DV_ERR_INVALID_ARG;
  for (int l = 0; l < n_layers; ++l) {
    const int rc = check_layer_args(layers[l], l == 0);
    if (rc != DV_OK) return rc;
    // one residual stream, and the scratch regions that travel from a block to the next at fixed offsets
    if (layers[l].d != layers[0].d || layers[l].ffn != layers[0].ffn || layers[l].H != layers[0].H)
      return DV_ERR_INVALID_ARG;
  }
  if (layers[0].workspace_bytes < layers_workspace_bytes(layers, n_layers) || !aligned16(layers[0].workspace))
    return DV_ERR_WORKSPACE;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  unsigned char* ws = reinterpret_cast<unsigned char*>(layers[0].workspace);
  auto CH = [](const void* q) { return reinterpret_cast<const half_t*>(q); };
  const int cus = compute_units();
  const int d = layers[0].d;
  const int nred = (d + 63) / 64;

  // P of block l: residual add (or the split reduction of block l - 1's fc2) + part statistics |
  // key histogram of block l's MLP logits | block l's window step.  prev == nullptr: the call's input.
  auto launch_pre = [&](const dvSparseLayerArgs* prev, const dvSparseLayerArgs& a) {
    const LayerPlan p = plan_layer(a);
    PreArgs pa;
    if (prev == nullptr) {
      pa.partial = nullptr;
      pa.bias = nullptr;
      pa.G = 1;
      pa.Y = const_cast<half_t*>(CH(a.hidden));
      pa.R = CH(a.residual);
    } else {
      const LayerPlan pp = plan_layer(*prev);
      // a single row group has stored the finished row itself
      pa.partial = pp.fc2_cols.groups > 1 ? reinterpret_cast<const float*>(ws + pp.off_cols_part) : nullptr;
      pa.bias = CH(prev->b2);
      pa.G = pp.fc2_cols.groups;
      pa.Y = reinterpret_cast<half_t*>(prev->hidden_out);
      pa.R = CH(prev->residual_out);
    }
    pa.d = d;
    pa.Rout = reinterpret_cast<half_t*>(ws + p.off_res1);
    pa.parts = reinterpret_cast<float2*>(ws + p.off_parts);
    pa.mlp_logits = CH(a.mlp_logit_in);
    pa.ffn = a.ffn;
    pa.topk_ws = reinterpret_cast<unsigned*>(ws + p.off_topk);
    pa.tracker = reinterpret_cast<int*>(a.tracker);
    pa.head_idx = reinterpret_cast<const int*>(a.head_idx);
    pa.nnz = a.Hk;
    pa.H = a.H;
    pa.counter = a.counter;
    pa.flush = a.counter == 15 ? 1 : 0;
    pa.batch_idx = reinterpret_cast<int*>(ws + p.off_batch_idx);
    const int nhist = (a.ffn + kTopkItemsPerBlock - 1) / kTopkItemsPerBlock;
    hipLaunchKernelGGL(layer_pre_kernel, dim3(nred + nhist + 1), dim3(256), 0, s, pa, nred, nhist);
  };

  for (int l = 0; l < n_layers; ++l) {
    const dvSparseLayerArgs& a = layers[l];
    const LayerPlan p = plan_layer(a);
    auto H16 = [&](size_t off) { return reinterpret_cast<half_t*>(ws + off); };
    unsigned* topk_ws = reinterpret_cast<unsigned*>(ws + p.off_topk);
    int* batch_idx = reinterpret_cast<int*>(ws + p.off_batch_idx);
    float* attn_part = reinterpret_cast<float*>(ws + p.off_attn_part);
    float* cols_part = reinterpret_cast<float*>(ws + p.off_cols_part);
    long long* acc = reinterpret_cast<long long*>(ws + p.off_acc);
    half_t* res1 = H16(p.off_res1);
    half_t* qkv = H16(p.off_qkv);
    half_t* hp_hidden = H16(p.off_hp_hidden);
    half_t* mp_hidden = H16(p.off_mp_hidden);
    half_t* hbuf = H16(p.off_h);
    half_t* head_logits = H16(p.off_head_logits);
    half_t* x_cache = reinterpret_cast<half_t*>(a.x_cache);
    const int* head_idx = reinterpret_cast<const int*>(a.head_idx);
    const int nb = a.counter + 1;
    const int topk_blocks = (a.ffn + kTopkItemsPerBlock - 1) / kTopkItemsPerBlock;

    if (l == 0) launch_pre(nullptr, a);
    // L2: LayerNorm 1 + QKV + cache scatter
    {
      QkvArgs q{x_cache, CH(a.Wqkv), CH(a.bqkv), head_idx, batch_idx, nb, a.d, a.H, a.hd, a.Hk, qkv,
                reinterpret_cast<half_t*>(a.k_cache), reinterpret_cast<half_t*>(a.v_cache),
                reinterpret_cast<const int*>(a.cache_offset), a.S,
                QkvLnArgs{res1, reinterpret_cast<const float2*>(ws + p.off_parts), CH(a.ln1_w), CH(a.ln1_b), a.eps1,
                          x_cache + (size_t)a.counter * a.d, a.counter}};
      if (int rc = launch_ln_qkv(q, s); rc != DV_OK) return rc;
    }
    // L3: attention partials | head predictor fc0 | top-k threshold and counts | accumulator reset.
    // The head predictor (input: the residual stream, output: only needed at the end of the step)
    // runs one launch later than it could: the QKV launch is the fullest one, this one has
    // bandwidth to spare.
    const int nsplit = a.seq_pos ? p.nsplit : attn_splits(a.n_len);
    {
      AttnArgs at{qkv + (size_t)a.counter * 3 * a.H * a.hd, (int64_t)3 * a.H * a.hd,
                  reinterpret_cast<const half_t*>(a.k_cache), reinterpret_cast<const half_t*>(a.v_cache),
                  head_idx, reinterpret_cast<const int*>(a.seq_pos), a.n_len, a.H, a.S, nsplit, a.Hk,
                  a.softmax_scale, attn_part};
      CanonArgs hp0{res1, CH(a.att_Wa), (int64_t)a.d, a.r_att, a.d, hp_hidden};
      const int na = nsplit * a.Hk;
      const int rw0 = a.d <= 1024 ? 4 * kCanonShortRows : 1;
      const int nh = ((a.r_att + rw0 - 1) / rw0 + 3) / 4;
      const dim3 grid(na + nh + topk_blocks + 1);
      int* advance_ptr = (a.counter == 15 && a.advance_window) ? reinterpret_cast<int*>(a.cache_offset) : nullptr;
      if (a.hd == 128)
        hipLaunchKernelGGL((layer_l3_kernel<128>), grid, dim3(256), 0, s, at, na, hp0, nh, CH(a.mlp_logit_in),
                           a.ffn, a.K, topk_ws, advance_ptr, 16, acc, a.d);
      else
        hipLaunchKernelGGL((layer_l3_kernel<64>), grid, dim3(256), 0, s, at, na, hp0, nh, CH(a.mlp_logit_in),
                           a.ffn, a.K, topk_ws, advance_ptr, 16, acc, a.d);
    }
    // L4: out_proj from the attention partials, sums added in fixed point | head predictor fc1 | top-k emission
    {
      const ColsPlan& c = p.out_cols;
      OutProjArgs o{CH(a.Wout_t), (int64_t)a.d, CH(a.bout), head_idx, a.hd, a.d, a.H * a.hd, a.Hk * a.hd,
                    c.rows_per_block, c.col_tiles, c.groups, acc, attn_part, nsplit};
      CanonArgs hp1{hp_hidden, CH(a.att_Wb), (int64_t)a.r_att, a.H, a.r_att, head_logits};
      const int rw1 = a.r_att <= 1024 ? 4 * kCanonShortRows : 1;
      const int nh1 = ((a.H + rw1 - 1) / rw1 + 3) / 4;
      const int no = c.col_tiles * c.groups;
      hipLaunchKernelGGL(layer_l4_kernel, dim3(no + nh1 + topk_blocks), dim3(256), 0, s, o, no, hp1, nh1,
                         CH(a.mlp_logit_in), a.ffn, a.K, topk_ws, reinterpret_cast<int64_t*>(a.mlp_idx_out),
                         topk_blocks);
    }
    const half_t* res2 = reinterpret_cast<const half_t*>(a.residual_out);
    const int64_t* mlp_idx = reinterpret_cast<const int64_t*>(a.mlp_idx_out);
    // L7: residual add + LayerNorm 2 + fc1 gather | MLP predictor fc0 | head top-k
    {
      RowsArgs f{acc, CH(a.bout), res1, reinterpret_cast<half_t*>(a.residual_out), CH(a.ln2_w), CH(a.ln2_b), a.eps2,
                 CH(a.W1), CH(a.b1), mlp_idx, a.d, (int64_t)a.d, a.ffn, a.K, hbuf};
      const int tasks = (a.K + 1) / 2;  // two gathered rows per wavefront
      const int waves = tasks >= cus * 8 ? 8 : 4;
      int nf = (tasks + waves - 1) / waves;
      if (nf > cus * (32 / waves)) nf = cus * (32 / waves);
      CanonArgs mp0{res2, CH(a.mlp_Wa), (int64_t)a.d, a.r_mlp, a.d, mp_hidden};
      const int rw0 = a.d <= 1024 ? 4 * kCanonShortRows : 1;
      const int nm = ((a.r_mlp + rw0 - 1) / rw0 + waves - 1) / waves;
      const size_t lds = (size_t)a.d * sizeof(half_t);
      static LdsGrant grant;
      if (int rc = grant.ensure(reinterpret_cast<const void*>(layer_l7_kernel), lds); rc != DV_OK) return rc;
      hipLaunchKernelGGL(layer_l7_kernel, dim3(nf + nm + 1), dim3(waves * 64), lds, s, f, nf, mp0, nm, head_logits,
                         a.H, a.att_k, reinterpret_cast<int*>(a.att_idx_out));
    }
    // L8: fc2 gather | MLP predictor fc1
    const ColsPlan& c = p.fc2_cols;
    {
      ColsArgs cc{hbuf, CH(a.W2t), (int64_t)a.d, mlp_idx, a.d, a.ffn, a.K, c.rows_per_block, c.col_tiles, c.groups,
                  cols_part, reinterpret_cast<half_t*>(a.hidden_out), CH(a.b2)};
      CanonArgs mp1{mp_hidden, CH(a.mlp_Wb), (int64_t)a.r_mlp, a.ffn, a.r_mlp,
                    reinterpret_cast<half_t*>(a.mlp_logit_out)};
      const int rw1 = a.r_mlp <= 1024 ? 4 * kCanonShortRows : 1;
      int nm = ((a.ffn + rw1 - 1) / rw1 + 3) / 4;
      if (nm > cus * 16) nm = cus * 16;
      const int nf = c.col_tiles * c.groups;
      hipLaunchKernelGGL(layer_l8_kernel, dim3(nf + nm), dim3(256), 0, s, cc, nf, mp1, nm);
    }
    // L9: the split reduction; with another block behind it, that block's P
    if (l + 1 < n_layers)
      launch_pre(&a, layers[l + 1]);
    else if (c.groups > 1)
      hipLaunchKernelGGL(cols_reduce_kernel<false>, dim3((unsigned)nred), dim3(256), 0, s, cols_part, CH(a.b2),
                         c.groups, 1, a.d, reinterpret_cast<half_t*>(a.hidden_out), (const half_t*)nullptr,
                         (half_t*)nullptr);
  }
  return launch_status();
}

int dv_sparse_layer_decode_f16(const dvSparseLayerArgs* args, void* stream) {
  return dv_sparse_layers_decode_f16(args, 1, stream);
}

int dv_add_ln_parts_f16(const void* h, const void* residual, int d, void* r_out, void* parts, void* stream) {
  if (!h || !r_out || !parts || d <= 0) return DV_ERR_INVALID_ARG;
  if (d % 8 || !aligned16(h) || !aligned16(r_out) || (residual && !aligned16(residual)) ||
      (reinterpret_cast<uintptr_t>(parts) & 7u))
    return DV_ERR_ALIGNMENT;
  if (d > kLnMaxParts * kLnPart) return DV_ERR_UNSUPPORTED;
  PreArgs pa{};
  pa.partial = nullptr;
  pa.bias = nullptr;
  pa.G = 1;
  pa.d = d;
  pa.Y = const_cast<half_t*>(reinterpret_cast<const half_t*>(h));  // read only: no partial sums to finish
  pa.R = reinterpret_cast<const half_t*>(residual);
  pa.Rout = reinterpret_cast<half_t*>(r_out);
  pa.parts = reinterpret_cast<float2*>(parts);
  const int nred = (d + 63) / 64;
  hipLaunchKernelGGL(layer_pre_kernel, dim3(nred), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), pa, nred, 0);
  return launch_status();
}

int dv_ln_qkv_proj_sparse_cache_f16(const void* r1, const void* parts, const void* gamma, const void* beta,
                                    float eps, void* x_cache, int token, const void* W, const void* bias,
                                    const void* head_idx, const void* batch_idx, int nb, int d, int H, int hd,
                                    int nnz, void* y, void* k_cache, void* v_cache, const void* padding, int S,
                                    void* stream) {
  if (!r1 || !parts || !gamma || !beta || !x_cache || !W || !y || nb < 1 || nb > 16 || token != nb - 1 || d <= 0 ||
      H <= 0 || nnz < 0 || nnz > H || (nnz > 0 && (!head_idx || !batch_idx)) || ((k_cache == nullptr) != (v_cache == nullptr)) ||
      (k_cache && S <= 0))
    return DV_ERR_INVALID_ARG;
  if ((hd != 64 && hd != 128) || d > kLnMaxParts * kLnPart || (size_t)d * 2 > 144 * 1024) return DV_ERR_UNSUPPORTED;
  if (d % 8 || !aligned16(r1) || !aligned16(gamma) || !aligned16(beta) || !aligned16(x_cache) || !aligned16(W) ||
      (reinterpret_cast<uintptr_t>(parts) & 7u))
    return DV_ERR_ALIGNMENT;
  if (nnz == 0) return DV_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  half_t* xc = reinterpret_cast<half_t*>(x_cache);
  QkvArgs q{xc, reinterpret_cast<const half_t*>(W), reinterpret_cast<const half_t*>(bias),
            reinterpret_cast<const int*>(head_idx), reinterpret_cast<const int*>(batch_idx), nb, d, H, hd, nnz,
            reinterpret_cast<half_t*>(y), reinterpret_cast<half_t*>(k_cache), reinterpret_cast<half_t*>(v_cache),
            reinterpret_cast<const int*>(padding), S,
            QkvLnArgs{reinterpret_cast<const half_t*>(r1), reinterpret_cast<const float2*>(parts),
                      reinterpret_cast<const half_t*>(gamma), reinterpret_cast<const half_t*>(beta), eps,
                      xc + (size_t)token * d, token}};
  return launch_ln_qkv(q, s);
}

}  // extern "C"
