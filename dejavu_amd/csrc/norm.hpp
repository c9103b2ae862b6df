// Fused residual add + LayerNorm for the pre-norm block:
//   r = fp16(h + residual)          (residual stream, stored in fp16)
//   y = fp16(LayerNorm(r) * gamma + beta)   (fp32 statistics, two-pass variance)
// One workgroup per row; the row is kept in registers between the passes.
//
// The summation order of the statistics is fixed by a layout of 1024 "virtual" threads:
// virtual thread t folds the elements of vectors t, t + 1024, ... in order, the 64 virtual
// threads of a wavefront are combined with an xor butterfly and the 16 wavefront sums are
// added in ascending order.  A workgroup of REAL = 1024 / Q threads runs Q virtual threads
// per thread (virtual thread t + q * REAL on thread t, i.e. the same lane of wavefront
// wave + q * REAL / 64), so that a 256-thread consumer that normalises the row on the fly
// produces the very same bits as the stand-alone 1024-thread kernel.
#pragma once
#include "common.hpp"

namespace dv {

constexpr int kLnVirtual = 1024;

template <int REAL>
__device__ __forceinline__ float block_sum_virtual(const float (&v)[kLnVirtual / REAL], float* scratch) {
  constexpr int Q = kLnVirtual / REAL;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();  // scratch may still be read from the previous call
#pragma unroll
  for (int q = 0; q < Q; ++q) {
    const float b = butterfly_sum<kWave>(v[q]);
    if (lane == 0) scratch[wave + q * (REAL / kWave)] = b;
  }
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < kLnVirtual / kWave; ++w) t += scratch[w];
  return t;
}

// MAXV: 8-element vectors per virtual thread; requires d % 8 == 0 and d <= 8192 * MAXV.
// Y may point to LDS (the row handed to a consumer in the same workgroup) or to memory;
// Y2 (optional) receives a second copy of the normalised row (the back-fill window buffer).
struct LnNoHook {
  __device__ __forceinline__ void operator()() const {}
};
// after_loads: called once the row's loads have been requested (a place to request memory the caller
// needs later: requests queued before the row's loads would delay them, the load counter retires in order)
template <int REAL, int MAXV, class AfterLoads = LnNoHook>
__device__ __forceinline__ void add_layer_norm_body(
    const half_t* __restrict__ H, const half_t* __restrict__ R, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, float eps, int d, half_t* __restrict__ Y,
    half_t* __restrict__ Rout, half_t* __restrict__ Y2, int64_t row, AfterLoads after_loads = AfterLoads()) {
  constexpr int Q = kLnVirtual / REAL;
  constexpr bool EARLY = Q * MAXV <= 4;  // gamma / beta fetched up front while registers allow
  __shared__ float scratch[kLnVirtual / kWave];
  const int nvec = d / 8;
  half8_t v[Q][MAXV], gm[EARLY ? Q : 1][EARLY ? MAXV : 1], bt[EARLY ? Q : 1][EARLY ? MAXV : 1];
  if (EARLY) {
#pragma unroll
    for (int q = 0; q < Q; ++q)
#pragma unroll
      for (int j = 0; j < MAXV; ++j) {  // issued early: not needed until the last pass
        const int i = threadIdx.x + q * REAL + j * kLnVirtual;
        gm[q][j] = i < nvec ? load8(gamma + i * 8) : zero8();
        bt[q][j] = i < nvec ? load8(beta + i * 8) : zero8();
      }
  }
  half8_t rr[Q][MAXV];
#pragma unroll
  for (int q = 0; q < Q; ++q)
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
      const int i = threadIdx.x + q * REAL + j * kLnVirtual;
      v[q][j] = i < nvec ? load8(H + row * d + i * 8) : zero8();
      rr[q][j] = (R != nullptr && i < nvec) ? load8(R + row * d + i * 8) : zero8();
    }
  after_loads();
  float s[Q];
#pragma unroll
  for (int q = 0; q < Q; ++q) {
    s[q] = 0.f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
      const int i = threadIdx.x + q * REAL + j * kLnVirtual;
      if (i < nvec) {
        half8_t h = v[q][j];
        if (R != nullptr) {
          const half8_t r = rr[q][j];
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = (half_t)((float)h[e] + (float)r[e]);
        }
        v[q][j] = h;
        if (Rout != nullptr) store8(Rout + row * d + i * 8, h);
#pragma unroll
        for (int e = 0; e < 8; ++e) s[q] += (float)h[e];
      }
    }
  }
  const float mean = block_sum_virtual<REAL>(s, scratch) / (float)d;
  float sq[Q];
#pragma unroll
  for (int q = 0; q < Q; ++q) {
    sq[q] = 0.f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
      const int i = threadIdx.x + q * REAL + j * kLnVirtual;
      if (i < nvec) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float c = (float)v[q][j][e] - mean;
          sq[q] = __builtin_fmaf(c, c, sq[q]);
        }
      }
    }
  }
  const float rstd = rsqrtf(block_sum_virtual<REAL>(sq, scratch) / (float)d + eps);
#pragma unroll
  for (int q = 0; q < Q; ++q)
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
      const int i = threadIdx.x + q * REAL + j * kLnVirtual;
      if (i < nvec) {
        const half8_t g = EARLY ? gm[q][j] : load8(gamma + i * 8);
        const half8_t b = EARLY ? bt[q][j] : load8(beta + i * 8);
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          o[e] = (half_t)__builtin_fmaf(((float)v[q][j][e] - mean) * rstd, (float)g[e], (float)b[e]);
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
