// Row-wise GEMV kernels: every output element is the dot product of one weight
// row (contiguous in memory) with an activation vector.  Lanes of a wavefront
// stride along the row with 128-bit loads and reduce with a butterfly.
//
//  * canonical_gemv_kernel : dense rows, fully specified summation order
//                            (predictor fc0 / fc1, bit-exact contract)
//  * gather_rows_kernel    : rows picked by an index vector, bias + activation
//                            fused (sparse-MLP fc1)
#pragma once
#include "common.hpp"

namespace dv {

// ---------------------------------------------------------------------------
// Y[b, row] = fp16( sum_i W[row, i] * X[b, i] ) with the canonical order:
// lane `sub` of the LANES lanes that share a row folds elements
// c*8*LANES + 8*sub + e (c ascending, e = 0..7) into one fp32 accumulator, then
// the LANES partials are combined with an xor butterfly (LANES/2 .. 1).
// Requires n % 8 == 0 and ldw % 8 == 0.
// ---------------------------------------------------------------------------
// X_LDS: X points into LDS (a copy of the row the workgroup holds).
template <int LANES, int B, int U, bool X_LDS = false>
__device__ __forceinline__ void canonical_gemv_body(
    const half_t* __restrict__ X, const half_t* __restrict__ W, int64_t ldw, int rows, int n,
    half_t* __restrict__ Y, int block_id, int nblocks) {
  constexpr int RW = kWave / LANES;  // rows per wavefront pass
  constexpr int CH = 8 * LANES;      // elements per chunk
  const int lane = threadIdx.x & 63;
  const int sub = lane % LANES;
  const int grp = lane / LANES;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves_per_block = blockDim.x >> 6;
  const int ntasks = (rows + RW - 1) / RW;
  for (int t = block_id * waves_per_block + wave; t < ntasks; t += nblocks * waves_per_block) {
    const int row = t * RW + grp;
    const bool valid = row < rows;
    const half_t* wr = W + (int64_t)(valid ? row : 0) * ldw + sub * 8;
    const half_t* xr = X + sub * 8;
    float acc[B];
#pragma unroll
    for (int b = 0; b < B; ++b) acc[b] = 0.f;
    int base = 0;
    for (; base + U * CH <= n; base += U * CH) {
      half8_t w[U];
#pragma unroll
      for (int u = 0; u < U; ++u) w[u] = load8_stream(wr + base + u * CH);
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int b = 0; b < B; ++b)
          acc[b] = fma8_ordered(w[u], load8_from<X_LDS>(xr + (int64_t)b * n + base + u * CH), acc[b]);
      }
    }
    if (base < n) {
      // the remaining (fewer than U) chunks, the last one possibly partial: their loads are
      // issued together like those of a full group; lanes past the row end take no part
      half8_t w[U];
      bool in[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        in[u] = base + u * CH + sub * 8 < n;
        w[u] = in[u] ? load8_stream(wr + base + u * CH) : zero8();
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (in[u]) {
#pragma unroll
          for (int b = 0; b < B; ++b)
            acc[b] = fma8_ordered(w[u], load8_from<X_LDS>(xr + (int64_t)b * n + base + u * CH), acc[b]);
        }
      }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) acc[b] = butterfly_sum<LANES>(acc[b]);
    if (valid && sub == 0) {
#pragma unroll
      for (int b = 0; b < B; ++b) Y[(int64_t)b * rows + row] = (half_t)acc[b];
    }
  }
}

template <int LANES, int B, int U>
__global__ __launch_bounds__(256) void canonical_gemv_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, int64_t ldw, int rows, int n,
    half_t* __restrict__ Y) {
  canonical_gemv_body<LANES, B, U>(X, W, ldw, rows, n, Y, blockIdx.x, gridDim.x);
}

// Short rows (B * n floats fit LDS).  With one weight row per lane group a wavefront has only
// one row's loads in flight per group, and for B >= 2 every 16 bytes of weights need B * 16
// bytes of x from L1, which bounds the kernel before memory does.  Here X is converted once per
// workgroup to fp32 in LDS and a lane group owns R weight rows at a time (R times the loads in
// flight) that share each x read: row r of task t is
// (t * R + r) * (64 / LANES) + group.  Same products in the same order per output as
// canonical_gemv_body, so the same bits.  Dynamic LDS: B * n * 4 bytes.
// count fp16 values (a multiple of 8) -> fp32 in LDS, by the whole workgroup (which then synchronises)
template <bool X_LDS = false>
__device__ __forceinline__ void stage_x_f32(const half_t* __restrict__ X, int count, float* xf) {
  for (int i = threadIdx.x * 8; i < count; i += blockDim.x * 8) {
    const half8_t v = load8_from<X_LDS>(X + i);
#pragma unroll
    for (int e = 0; e < 8; ++e) xf[i + e] = (float)v[e];
  }
  __syncthreads();
}

template <int LANES, int B, int U, int R>
__device__ __forceinline__ void canonical_gemv_lds_body(const float* xf, const half_t* __restrict__ W,
                                                        int64_t ldw, int rows, int n,
                                                        half_t* __restrict__ Y, int block_id, int nblocks) {
  constexpr int RW = kWave / LANES;
  constexpr int CH = 8 * LANES;
  const int lane = threadIdx.x & 63;
  const int sub = lane % LANES;
  const int grp = lane / LANES;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ntasks = (rows + RW * R - 1) / (RW * R);
  const int waves_per_block = blockDim.x >> 6;
  for (int t = block_id * waves_per_block + wave; t < ntasks; t += nblocks * waves_per_block) {
    const half_t* wr[R];
    bool valid[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int row = (t * R + r) * RW + grp;
      valid[r] = row < rows;
      wr[r] = W + (int64_t)(valid[r] ? row : 0) * ldw + sub * 8;
    }
    float acc[R][B];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int b = 0; b < B; ++b) acc[r][b] = 0.f;
    // groups of U chunks; the last group may be short and its last chunk partial: all loads are
    // issued together, lanes past the row end take no part
    for (int base = 0; base < n; base += U * CH) {
      half8_t w[U][R];
      bool in[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        in[u] = base + u * CH + sub * 8 < n;
#pragma unroll
        for (int r = 0; r < R; ++r) w[u][r] = in[u] ? load8_stream(wr[r] + base + u * CH) : zero8();
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (in[u]) {
#pragma unroll
          for (int b = 0; b < B; ++b) {
            const float* xp = xf + b * n + base + u * CH + sub * 8;
            const float4_t lo = *reinterpret_cast<const float4_t*>(xp);
            const float4_t hi = *reinterpret_cast<const float4_t*>(xp + 4);
#pragma unroll
            for (int r = 0; r < R; ++r) {
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[r][b] = __builtin_fmaf((float)w[u][r][e], lo[e], acc[r][b]);
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[r][b] = __builtin_fmaf((float)w[u][r][4 + e], hi[e], acc[r][b]);
            }
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const float v = butterfly_sum<LANES>(acc[r][b]);
        const int row = (t * R + r) * RW + grp;
        if (valid[r] && sub == 0) Y[(int64_t)b * rows + row] = (half_t)v;
      }
  }
}

template <int LANES, int B, int U, int R>
__global__ __launch_bounds__(256) void canonical_gemv_xlds_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, int64_t ldw, int rows, int n,
    half_t* __restrict__ Y) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  float* xf = reinterpret_cast<float*>(smem_raw);
  stage_x_f32(X, B * n, xf);
  canonical_gemv_lds_body<LANES, B, U, R>(xf, W, ldw, rows, n, Y, blockIdx.x, gridDim.x);
}

// Long rows (64 lanes per row), several batch rows: canonical_gemv_body re-reads B x 16 bytes of X
// from L2 for every 16 bytes of weights (B rows of X do not fit LDS at n = 12288).  Here the
// workgroup walks the columns in slices of kCanonSlice elements; all its wavefronts (one weight row
// each) share the slice of X, staged as fp16 in LDS (double-buffered, one barrier per slice), and
// the next slice's weights and X are requested before the current slice is multiplied.  Per output
// the products are folded in the same (chunk, element) order and the same butterfly as
// canonical_gemv_body (chunks past the row end contribute w = x = 0): the same bits.
// Dynamic LDS: 2 * B * kCanonSlice halfs.  n % 8 == 0, ldw % 8 == 0.
constexpr int kCanonSlice = 2048;  // four chunks of 8 * 64 elements

template <int B>
__global__ __launch_bounds__(256) void canonical_gemv_slices_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, int64_t ldw, int rows, int n,
    half_t* __restrict__ Y) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  half_t* xs = reinterpret_cast<half_t*>(smem_raw);  // [2][B][kCanonSlice]
  constexpr int CH = 8 * kWave;
  constexpr int U = kCanonSlice / CH;               // chunks per slice
  constexpr int XV = B * kCanonSlice / 8 / 256;     // X vectors per thread and slice
  static_assert(B * kCanonSlice / 8 % 256 == 0, "slice staging does not tile");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nslices = (n + kCanonSlice - 1) / kCanonSlice;
  // X vector p of a thread: batch row (p * 256 + tid) / (kCanonSlice / 8), columns ((p * 256 + tid) % (kCanonSlice / 8)) * 8
  auto load_x = [&](half8_t (&xv)[XV], int sl) {
#pragma unroll
    for (int p = 0; p < XV; ++p) {
      const int o = p * 256 + tid;
      const int b = o / (kCanonSlice / 8), col = sl * kCanonSlice + (o % (kCanonSlice / 8)) * 8;
      xv[p] = col < n ? load8(X + (int64_t)b * n + col) : zero8();
    }
  };
  auto store_x = [&](const half8_t (&xv)[XV], int buf) {
#pragma unroll
    for (int p = 0; p < XV; ++p) store8(xs + (size_t)buf * B * kCanonSlice + (size_t)(p * 256 + tid) * 8, xv[p]);
  };
  for (int row0 = blockIdx.x * 4; row0 < rows; row0 += gridDim.x * 4) {  // uniform over the workgroup
    const int row = row0 + wave;
    const bool valid = row < rows;
    const half_t* wr = W + (int64_t)(valid ? row : 0) * ldw + lane * 8;
    auto load_w = [&](half8_t (&w)[U], int sl) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int col = sl * kCanonSlice + u * CH + lane * 8;
        w[u] = col < n ? load8_stream(wr + sl * kCanonSlice + u * CH) : zero8();
      }
    };
    float acc[B];
#pragma unroll
    for (int b = 0; b < B; ++b) acc[b] = 0.f;
    half8_t w[U], wn[U], xv[XV];
    __syncthreads();  // the previous row group's reads of the X buffers are done
    load_x(xv, 0);
    load_w(w, 0);
    store_x(xv, 0);
    for (int sl = 0; sl < nslices; ++sl) {
      const int buf = sl & 1;
      __syncthreads();  // slice sl is in LDS; every wavefront is done with slice sl - 1 (the other buffer)
      if (sl + 1 < nslices) {
        load_x(xv, sl + 1);
        load_w(wn, sl + 1);
      }
      const half_t* xb = xs + (size_t)buf * B * kCanonSlice + lane * 8;
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int b = 0; b < B; ++b) acc[b] = fma8_ordered(w[u], load8(xb + b * kCanonSlice + u * CH), acc[b]);
      }
      if (sl + 1 < nslices) {
        store_x(xv, buf ^ 1);
#pragma unroll
        for (int u = 0; u < U; ++u) w[u] = wn[u];
      }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const float v = butterfly_sum<kWave>(acc[b]);
      if (valid && lane == 0) Y[(int64_t)b * rows + row] = (half_t)v;
    }
  }
}

// ---------------------------------------------------------------------------
// Y[b, m] = act( sum_i W[idx[m], i] * X[b, i] + bias[idx[m]] ), fp16 out.
// One wavefront owns R gathered rows at a time (R independent load streams);
// X is staged once per workgroup in LDS.  An index outside [0, Z) yields 0
// instead of a wild read; idx == nullptr means no gather (row m of W: a dense product).  Requires n % 8 == 0 and ldw % 8 == 0.
// ---------------------------------------------------------------------------
// STAGED: the caller has already put X into xs (and synchronised the workgroup).
// RELU: an activation is applied, `act` says which (act_f; ReLU unless told otherwise).
template <int B, int R, int U, bool RELU, bool STAGED = false>
__device__ __forceinline__ void gather_rows_body(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const void* __restrict__ idx, int idx_bytes, int n, int64_t ldw, int Z, int M,
    half_t* __restrict__ Y, half_t* xs, int block_id, int nblocks, int act = 1) {
  if (!STAGED) {
    for (int i = threadIdx.x * 8; i < B * n; i += blockDim.x * 8) store8(xs + i, load8(X + i));
    __syncthreads();
  }

  constexpr int CH = 8 * kWave;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves_per_block = blockDim.x >> 6;
  const int ntasks = (M + R - 1) / R;
  for (int t = block_id * waves_per_block + wave; t < ntasks; t += nblocks * waves_per_block) {
    const half_t* wr[R];
    bool valid[R];
    int64_t rid[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int m = t * R + r;
      int64_t id = m < M ? (idx != nullptr ? load_index(idx, idx_bytes, m) : (int64_t)m) : -1;
      valid[r] = id >= 0 && id < Z;
      rid[r] = valid[r] ? id : 0;
      wr[r] = W + rid[r] * ldw + lane * 8;
    }
    float acc[R][B];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int b = 0; b < B; ++b) acc[r][b] = 0.f;

    int base = 0;
    for (; base + U * CH <= n; base += U * CH) {
      half8_t w[U][R];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < R; ++r) w[u][r] = load8_stream(wr[r] + base + u * CH);
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int b = 0; b < B; ++b) {
          const half8_t xv = load8(xs + b * n + base + u * CH + lane * 8);
#pragma unroll
          for (int r = 0; r < R; ++r) acc[r][b] = dot8_fast(w[u][r], xv, acc[r][b]);
        }
      }
    }
    for (; base < n; base += CH) {
      if (base + lane * 8 < n) {
        half8_t w[R];
#pragma unroll
        for (int r = 0; r < R; ++r) w[r] = load8_stream(wr[r] + base);
#pragma unroll
        for (int b = 0; b < B; ++b) {
          const half8_t xv = load8(xs + b * n + base + lane * 8);
#pragma unroll
          for (int r = 0; r < R; ++r) acc[r][b] = dot8_fast(w[r], xv, acc[r][b]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int m = t * R + r;
      float bv = 0.f;
      if (bias != nullptr && valid[r]) bv = (float)bias[rid[r]];
#pragma unroll
      for (int b = 0; b < B; ++b) {
        float v = butterfly_sum<kWave>(acc[r][b]) + bv;
        if (RELU) v = act_f(v, act);
        if (!valid[r]) v = 0.f;
        if (lane == 0 && m < M) Y[(int64_t)b * M + m] = (half_t)v;
      }
    }
  }
}

template <int B, int R, int U, bool RELU>
__global__ __launch_bounds__(256) void gather_rows_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const void* __restrict__ idx, int idx_bytes, int n, int64_t ldw, int Z, int M,
    half_t* __restrict__ Y, int act = 1) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  gather_rows_body<B, R, U, RELU>(X, W, bias, idx, idx_bytes, n, ldw, Z, M, Y,
                                  reinterpret_cast<half_t*>(smem_raw), blockIdx.x, gridDim.x, act);
}

}  // namespace dv
