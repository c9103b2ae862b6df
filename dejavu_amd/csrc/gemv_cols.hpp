// Column-wise ("transposed") gathered GEMV: Y[b, :] = sum_m x[b, m] * W[row(m), :] + bias.
// Lanes own 8 adjacent output columns each and stream the gathered rows with
// 128-bit loads; no cross-lane reduction is needed.  The M rows are split over
// gridDim.y row groups; each group writes an fp32 partial, and the partials are
// summed in a fixed order (deterministic, no floating-point atomics) by
// cols_reduce_kernel.  (Reducing inside this kernel -- the last group to finish a
// column tile adds the partials -- measured slower than the second launch: 23.0 us
// against 20.2 us for fc2 at the OPT-175B shape.)
#pragma once
#include "common.hpp"
#include "norm.hpp"

namespace dv {

constexpr int kColTile = 8 * kWave;  // 512 columns per workgroup

// Row mapping: BLOCKED == false: row(m) = idx[m] (sparse-MLP fc2 over W2^T).
// BLOCKED == true: row(m) = idx[m / blk] * blk + m % blk (out_proj over
// W_out^T with blk = head_dim and idx = active heads).
// x_expanded == 0: X is (B, M), x[b, m];  != 0: X is (B, Z), x[b, row(m)].
// ATTN (with BLOCKED): the activations are not read from X but merged on the
// fly from the un-normalised attention partials { max, sum, o[blk] } of
// decode_attn_kernel (attn_nsplit splits per head), rounded to fp16 as a
// stored context vector would be.
// FIXED: the workgroup adds its partial sums, in fixed point, to acc_fixed (B, N) with 64-bit
// integer atomics instead of storing an fp32 partial per row group; acc_fixed must hold zeros
// when the launch starts.
template <int B, int U, bool IDX64, bool BLOCKED, bool ATTN, bool FIXED = false>
__device__ __forceinline__ void gather_cols_body(
    const half_t* __restrict__ X, int64_t ldx, int x_expanded, const half_t* __restrict__ W,
    int64_t ldw, const half_t* __restrict__ bias, const void* __restrict__ idx, int blk, int N,
    int Z, int M, int rows_per_block, float* __restrict__ partial,
    half_t* __restrict__ Y, const float* __restrict__ attn_part, int attn_nsplit, int ct, int g,
    int G, long long* __restrict__ acc_fixed = nullptr) {
  __shared__ float red[4][B][kColTile];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = ct * kColTile + lane * 8;
  const bool col_ok = col < N;  // N % 8 == 0, so a lane is all-in or all-out
  const half_t* wcol = W + (col_ok ? col : 0);

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

  // 64 rows at a time: lane l fetches the row id and the activations of row
  // mb + l once; the row loop then broadcasts them with readlane, so the
  // weight loads are issued back to back without scalar-load stalls.
  for (int mb = m_begin; mb < m_end; mb += kWave) {
    const int m = mb + lane;
    int rid = 0;
    bool ok = false;
    if (m < m_end) {
      int64_t id;
      if (BLOCKED) {
        const int q = m / blk;
        const int64_t h = IDX64 ? reinterpret_cast<const int64_t*>(idx)[q]
                                : (int64_t) reinterpret_cast<const int32_t*>(idx)[q];
        id = (h >= 0 && h < Z / blk) ? h * blk + (m - q * blk) : -1;
      } else {
        id = IDX64 ? reinterpret_cast<const int64_t*>(idx)[m]
                   : (int64_t) reinterpret_cast<const int32_t*>(idx)[m];
      }
      ok = id >= 0 && id < Z;
      rid = ok ? (int)id : 0;
    }
    // the loop over full batches of U rows is software-pipelined two batches deep (registers
    // wa / wb): two batches' weight loads are in flight during a batch's multiply-adds, and the
    // first two are issued before the activations (for ATTN: the merged attention partials)
    // are known
    const int cnt = (m_end - mb) < kWave ? (m_end - mb) : kWave;
    const int nfull = cnt / U;
    half8_t wa[U], wb[U];
    auto load_batch = [&](half8_t (&w)[U], int jb) {
#pragma unroll
      for (int u = 0; u < U; ++u)
        w[u] = load8_stream(wcol + (int64_t)__builtin_amdgcn_readlane(rid, jb * U + u) * ldw);
    };
    if (nfull > 0) load_batch(wa, 0);
    if (nfull > 1) load_batch(wb, 1);
    float xl[B];
    if (ATTN) {
      const int nheads = M / blk;
      const int q = ok ? m / blk : 0, jj = ok ? m - q * blk : 0;
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const float* p = attn_part + ((int64_t)b * nheads + q) * attn_nsplit * (blk + 2);
        float mx = -INFINITY, num = 0.f, den = 0.f;
        for (int s0 = 0; s0 < attn_nsplit; s0 += 8) {  // online merge, 8 splits' loads in flight
          float ms[8], ls[8], os[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const bool in = s0 + u < attn_nsplit;
            const float* ps = p + (int64_t)(in ? s0 + u : s0) * (blk + 2);
            ms[u] = in ? ps[0] : -INFINITY;
            ls[u] = ps[1];
            os[u] = ps[2 + jj];
          }
          float mc = mx;
#pragma unroll
          for (int u = 0; u < 8; ++u) mc = fmaxf(mc, ms[u]);
          if (mc == -INFINITY) continue;
          const float rescale = mx == -INFINITY ? 0.f : __expf(mx - mc);
          num *= rescale;
          den *= rescale;
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const float w = ms[u] == -INFINITY ? 0.f : __expf(ms[u] - mc);
            den += w * ls[u];
            num += w * os[u];
          }
          mx = mc;
        }
        xl[b] = ok ? (float)(half_t)(num / den) : 0.f;
      }
    } else {
#pragma unroll
      for (int b = 0; b < B; ++b)
        xl[b] = ok ? (float)X[(int64_t)b * ldx + (x_expanded ? (int64_t)rid : (int64_t)m)] : 0.f;
    }

    auto consume = [&](const half8_t (&w)[U], int j) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int b = 0; b < B; ++b) {
          const float xs = __builtin_bit_cast(
              float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xl[b]), j + u));
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[b][e] = __builtin_fmaf((float)w[u][e], xs, acc[b][e]);
        }
      }
    };
    int jb = 0;
    for (; jb + 3 < nfull; jb += 2) {  // batches jb, jb + 1 are in wa, wb; jb + 2, jb + 3 exist
      half8_t w[U];
#pragma unroll
      for (int u = 0; u < U; ++u) w[u] = wa[u];
      load_batch(wa, jb + 2);
      consume(w, jb * U);
#pragma unroll
      for (int u = 0; u < U; ++u) w[u] = wb[u];
      load_batch(wb, jb + 3);
      consume(w, (jb + 1) * U);
    }
    if (jb < nfull) {  // up to three batches left: jb in wa, jb + 1 in wb, jb + 2 not requested yet
      half8_t w[U];
#pragma unroll
      for (int u = 0; u < U; ++u) w[u] = wa[u];
      if (jb + 2 < nfull) load_batch(wa, jb + 2);
      consume(w, jb * U);
      if (jb + 1 < nfull) consume(wb, (jb + 1) * U);
      if (jb + 2 < nfull) consume(wa, (jb + 2) * U);
    }
    int j = nfull * U;
    if (j < cnt) {
      // fewer than U rows left: their loads are issued together like those of a full batch
      // (slots past the last row repeat it and take no part in the sums)
      half8_t w[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int jj = j + u < cnt ? j + u : cnt - 1;
        w[u] = load8_stream(wcol + (int64_t)__builtin_amdgcn_readlane(rid, jj) * ldw);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (j + u < cnt) {
#pragma unroll
          for (int b = 0; b < B; ++b) {
            const float xs = __builtin_bit_cast(
                float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xl[b]), j + u));
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[b][e] = __builtin_fmaf((float)w[u][e], xs, acc[b][e]);
          }
        }
      }
    }
  }

  // combine the four wavefronts of the workgroup
#pragma unroll
  for (int b = 0; b < B; ++b)
#pragma unroll
    for (int e = 0; e < 8; ++e) red[wave][b][lane * 8 + e] = col_ok ? acc[b][e] : 0.f;
  __syncthreads();

  constexpr int PER_THREAD = B * kColTile / 256;
  float sum[PER_THREAD];
#pragma unroll
  for (int j = 0; j < PER_THREAD; ++j) {
    const int o = j * 256 + tid;  // o = b * kColTile + c
    const int b = o / kColTile, c = o % kColTile;
    sum[j] = (red[0][b][c] + red[1][b][c]) + (red[2][b][c] + red[3][b][c]);
  }

  if constexpr (FIXED) {
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) {
      const int o = j * 256 + tid;
      const int b = o / kColTile, c = ct * kColTile + o % kColTile;
      if (c < N)
        __hip_atomic_fetch_add(reinterpret_cast<unsigned long long*>(acc_fixed) + (int64_t)b * N + c,
                               (unsigned long long)to_fixed(sum[j]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return;
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
}

template <int B, int U, bool IDX64, bool BLOCKED, bool ATTN = false>
__global__ __launch_bounds__(256) void gather_cols_kernel(
    const half_t* __restrict__ X, int64_t ldx, int x_expanded, const half_t* __restrict__ W,
    int64_t ldw, const half_t* __restrict__ bias, const void* __restrict__ idx, int blk, int N,
    int Z, int M, int rows_per_block, float* __restrict__ partial,
    half_t* __restrict__ Y, const float* __restrict__ attn_part = nullptr, int attn_nsplit = 0,
    int always_partial = 0) {
  // always_partial: a single row group also stores its partial (the caller runs the reduction)
  gather_cols_body<B, U, IDX64, BLOCKED, ATTN>(X, ldx, x_expanded, W, ldw, bias, idx, blk, N, Z, M,
                                                     rows_per_block, partial, Y, attn_part,
                                                     attn_nsplit, blockIdx.x, blockIdx.y,
                                                     always_partial ? 0 : (int)gridDim.y);
}

// Second pass of the non-fused path: Y[b, c] = fp16(sum_g partial[g, b, c] + bias[c]).
// A workgroup owns 64 outputs; its four wavefronts each add every fourth group
// (ascending), and the four slice sums are combined in a fixed order.
// FIXED: every partial is first brought to fixed point (to_fixed) and the sum is an integer sum:
// the same bits as the partials added with integer atomics in any order (gather_cols_body<FIXED>).
// With R / Rout (optional) the residual stream is advanced in the same pass:
// Rout[b, c] = fp16(Y[b, c] + R[b, c]), the rounded sum of the two fp16 values (R == nullptr: Rout = Y).
// partial == nullptr: Y already holds the result, only the residual add is done.
// parts (optional, B == 1): the LayerNorm statistics pair of the 64 values this workgroup stored
// to Rout (norm.hpp), parts[block_id].
template <bool FIXED>
__device__ __forceinline__ void cols_reduce_body(const float* __restrict__ partial,
                                                 const half_t* __restrict__ bias, int G, int B, int N,
                                                 half_t* __restrict__ Y, const half_t* __restrict__ R,
                                                 half_t* __restrict__ Rout, float2* __restrict__ parts,
                                                 int block_id) {
  __shared__ float red[4][kWave];
  __shared__ long long redq[FIXED ? 4 : 1][FIXED ? kWave : 1];
  __shared__ __attribute__((aligned(16))) half_t s_row[kWave];
  const int lane = threadIdx.x & 63;
  const int slice = threadIdx.x >> 6;
  const int64_t total = (int64_t)B * N;
  const int64_t o = (int64_t)block_id * kWave + lane;
  half_t out = (half_t)0.f;  // the value stored to Rout (slice 0)
  if (partial == nullptr) {  // Y is complete already (single row group): only the residual add
    if (slice != 0) return;
    if (o < total && Rout != nullptr) {
      out = R != nullptr ? (half_t)((float)Y[o] + (float)R[o]) : Y[o];
      Rout[o] = out;
    }
  } else {
    // bias and residual are requested together with the partial sums, not after the barrier
    float bv = 0.f, rv = 0.f;
    if (slice == 0 && o < total) {
      if (bias != nullptr) bv = (float)bias[o % N];
      if (Rout != nullptr && R != nullptr) rv = (float)R[o];
    }
    float s = 0.f;
    long long sq = 0;
    if (o < total) {
      const float* p = partial + o;
      int gg = slice;
      for (; gg + 28 < G; gg += 32) {
        float v[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) v[q] = p[(int64_t)(gg + 4 * q) * total];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          if (FIXED) sq += to_fixed(v[q]);
          else s += v[q];
        }
      }
      for (; gg < G; gg += 4) {
        if (FIXED) sq += to_fixed(p[(int64_t)gg * total]);
        else s += p[(int64_t)gg * total];
      }
    }
    if (FIXED) redq[slice][lane] = sq;
    else red[slice][lane] = s;
    __syncthreads();
    if (slice != 0) return;
    if (o < total) {
      const float r = FIXED ? from_fixed((redq[0][lane] + redq[1][lane]) + (redq[2][lane] + redq[3][lane]))
                            : (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
      const half_t y = (half_t)(r + bv);
      if (Y != nullptr) Y[o] = y;
      if (Rout != nullptr) {
        out = R != nullptr ? (half_t)((float)y + rv) : y;
        Rout[o] = out;
      }
    }
  }
  if (parts != nullptr) {  // wavefront 0 only (B == 1)
    s_row[lane] = out;  // lanes past the row end hold 0 and are not counted
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    int n_p = N - block_id * kWave;
    if (n_p > kWave) n_p = kWave;
    const bool present = lane < 8 && lane * 8 < n_p;
    const half8_t v = present ? load8(s_row + lane * 8) : zero8();
    const float2 st = ln_part_stats_lanes8(v, present, n_p);
    if (lane == 0) parts[block_id] = st;
  }
}

template <bool FIXED = false>
__global__ __launch_bounds__(256) void cols_reduce_kernel(const float* __restrict__ partial,
                                                          const half_t* __restrict__ bias, int G,
                                                          int B, int N, half_t* __restrict__ Y,
                                                          const half_t* __restrict__ R = nullptr,
                                                          half_t* __restrict__ Rout = nullptr) {
  cols_reduce_body<FIXED>(partial, bias, G, B, N, Y, R, Rout, nullptr, blockIdx.x);
}

}  // namespace dv
