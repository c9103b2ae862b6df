// Column-wise ("transposed") gathered GEMV: Y[b, :] = sum_m x[b, m] * W[row(m), :] + bias.
// Lanes own 8 adjacent output columns each and stream the gathered rows with
// 128-bit loads; no cross-lane reduction is needed.  The M rows are split over
// gridDim.y row groups; each group writes an fp32 partial and the last group
// to finish a column tile sums the partials in a fixed order (deterministic,
// no floating-point atomics) and adds the bias.
#pragma once
#include "common.hpp"

namespace dv {

constexpr int kColTile = 8 * kWave;  // 512 columns per workgroup

// Row mapping: with blk == 1, row(m) = idx[m] (sparse-MLP fc2 over W2^T).
// With blk > 1, row(m) = idx[m / blk] * blk + m % blk (out_proj over
// W_out^T, blk = head_dim, idx = active heads).
// x_expanded == 0: X is (B, M), x[b, m];  == 1: X is (B, Z), x[b, row(m)].
template <int B, int U>
__global__ __launch_bounds__(256) void gather_cols_kernel(
    const half_t* __restrict__ X, int64_t ldx, int x_expanded, const half_t* __restrict__ W,
    int64_t ldw, const half_t* __restrict__ bias, const void* __restrict__ idx, int idx_bytes,
    int blk, int N, int Z, int M, int rows_per_block, float* __restrict__ partial,
    unsigned* __restrict__ counters, half_t* __restrict__ Y) {
  __shared__ float red[4][B][kColTile];
  __shared__ int s_last;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ct = blockIdx.x;
  const int g = blockIdx.y;
  const int G = gridDim.y;
  const int col = ct * kColTile + lane * 8;
  const bool col_ok = col < N;  // N % 8 == 0, so a lane is all-in or all-out

  const int rpw = (rows_per_block + 3) >> 2;
  const int m_begin = g * rows_per_block + wave * rpw;
  int m_end = m_begin + rpw;
  if (m_end > (g + 1) * rows_per_block) m_end = (g + 1) * rows_per_block;
  if (m_end > M) m_end = M;

  float acc[B][8];
#pragma unroll
  for (int b = 0; b < B; ++b)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[b][e] = 0.f;

  for (int m0 = m_begin; m0 < m_end; m0 += U) {
    half8_t w[U];
    float xv[U][B];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int m = m0 + u;
      int64_t id = -1;
      if (m < m_end) {
        id = blk == 1 ? load_index(idx, idx_bytes, m)
                      : load_index(idx, idx_bytes, m / blk) * blk + m % blk;
      }
      const bool ok = id >= 0 && id < Z;
      w[u] = (ok && col_ok) ? load8_stream(W + id * ldw + col) : zero8();
#pragma unroll
      for (int b = 0; b < B; ++b)
        xv[u][b] = ok ? (float)X[(int64_t)b * ldx + (x_expanded ? id : (int64_t)m)] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int b = 0; b < B; ++b)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[b][e] = __builtin_fmaf((float)w[u][e], xv[u][b], acc[b][e]);
  }

  // combine the four wavefronts of the workgroup
#pragma unroll
  for (int b = 0; b < B; ++b)
#pragma unroll
    for (int e = 0; e < 8; ++e) red[wave][b][lane * 8 + e] = acc[b][e];
  __syncthreads();

  constexpr int PER_THREAD = B * kColTile / 256;
  float sum[PER_THREAD];
#pragma unroll
  for (int j = 0; j < PER_THREAD; ++j) {
    const int o = j * 256 + tid;  // o = b * kColTile + c
    const int b = o / kColTile, c = o % kColTile;
    sum[j] = (red[0][b][c] + red[1][b][c]) + (red[2][b][c] + red[3][b][c]);
  }

  if (G == 1) {
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) {
      const int o = j * 256 + tid;
      const int b = o / kColTile, c = ct * kColTile + o % kColTile;
      if (c < N) Y[(int64_t)b * N + c] = (half_t)(sum[j] + (bias ? (float)bias[c] : 0.f));
    }
    return;
  }

#pragma unroll
  for (int j = 0; j < PER_THREAD; ++j) {
    const int o = j * 256 + tid;
    const int b = o / kColTile, c = ct * kColTile + o % kColTile;
    if (c < N) partial[((int64_t)g * B + b) * N + c] = sum[j];
  }
  __threadfence();  // release the partials device-wide before signalling
  __syncthreads();
  if (tid == 0) {
    const unsigned old = atomicAdd(&counters[ct], 1u);
    s_last = (old == (unsigned)(G - 1));
  }
  __syncthreads();
  if (!s_last) return;
  __threadfence();  // acquire the other groups' partials
#pragma unroll
  for (int j = 0; j < PER_THREAD; ++j) {
    const int o = j * 256 + tid;
    const int b = o / kColTile, c = ct * kColTile + o % kColTile;
    if (c < N) {
      float s = 0.f;
      for (int gg = 0; gg < G; ++gg) s += partial[((int64_t)gg * B + b) * N + c];
      Y[(int64_t)b * N + c] = (half_t)(s + (bias ? (float)bias[c] : 0.f));
    }
  }
  if (tid == 0) counters[ct] = 0;  // leave the counter ready for the next launch
}

}  // namespace dv
