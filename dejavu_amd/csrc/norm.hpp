// Fused residual add + LayerNorm for the pre-norm block:
//   r = fp16(h + residual)          (residual stream, stored in fp16)
//   y = fp16(LayerNorm(r) * gamma + beta)   (fp32 statistics, two-pass variance)
// One workgroup per row; the row is kept in registers between the passes.
#pragma once
#include "common.hpp"

namespace dv {

template <int THREADS>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = butterfly_sum<kWave>(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();  // scratch may still be read from the previous call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < THREADS / kWave; ++w) t += scratch[w];
  return t;
}

// MAXV: 8-element vectors held per thread; requires d % 8 == 0 and d <= THREADS * 8 * MAXV.
// Y2 (optional) receives a second copy of the normalised row (the back-fill window buffer).
template <int THREADS, int MAXV>
__device__ __forceinline__ void add_layer_norm_body(
    const half_t* __restrict__ H, const half_t* __restrict__ R, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, float eps, int d, half_t* __restrict__ Y,
    half_t* __restrict__ Rout, half_t* __restrict__ Y2, int64_t row) {
  __shared__ float scratch[THREADS / kWave];
  const int nvec = d / 8;
  half8_t v[MAXV], gm[MAXV], bt[MAXV];
#pragma unroll
  for (int j = 0; j < MAXV; ++j) {  // issued early: not needed until the last pass
    const int i = threadIdx.x + j * THREADS;
    gm[j] = i < nvec ? load8(gamma + i * 8) : zero8();
    bt[j] = i < nvec ? load8(beta + i * 8) : zero8();
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < MAXV; ++j) {
    const int i = threadIdx.x + j * THREADS;
    v[j] = zero8();
    if (i < nvec) {
      half8_t h = load8(H + row * d + i * 8);
      if (R != nullptr) {
        const half8_t r = load8(R + row * d + i * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = (half_t)((float)h[e] + (float)r[e]);
      }
      v[j] = h;
      if (Rout != nullptr) store8(Rout + row * d + i * 8, h);
#pragma unroll
      for (int e = 0; e < 8; ++e) s += (float)h[e];
    }
  }
  const float mean = block_sum<THREADS>(s, scratch) / (float)d;
  float q = 0.f;
#pragma unroll
  for (int j = 0; j < MAXV; ++j) {
    const int i = threadIdx.x + j * THREADS;
    if (i < nvec) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float c = (float)v[j][e] - mean;
        q += c * c;
      }
    }
  }
  const float rstd = rsqrtf(block_sum<THREADS>(q, scratch) / (float)d + eps);
#pragma unroll
  for (int j = 0; j < MAXV; ++j) {
    const int i = threadIdx.x + j * THREADS;
    if (i < nvec) {
      const half8_t g = gm[j];
      const half8_t b = bt[j];
      half8_t o;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        o[e] = (half_t)(((float)v[j][e] - mean) * rstd * (float)g[e] + (float)b[e]);
      store8(Y + row * d + i * 8, o);
      if (Y2 != nullptr) store8(Y2 + row * d + i * 8, o);
    }
  }
}

template <int THREADS, int MAXV>
__global__ __launch_bounds__(THREADS) void add_layer_norm_kernel(
    const half_t* __restrict__ H, const half_t* __restrict__ R, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, float eps, int d, half_t* __restrict__ Y,
    half_t* __restrict__ Rout) {
  add_layer_norm_body<THREADS, MAXV>(H, R, gamma, beta, eps, d, Y, Rout, nullptr, blockIdx.x);
}

}  // namespace dv
