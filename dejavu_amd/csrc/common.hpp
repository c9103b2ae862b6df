// Shared device helpers for the gfx950 (CDNA4, wave64) kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dv {

constexpr int kWave = 64;

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// 128-bit global load of 8 fp16 values (address must be 16-byte aligned).
__device__ __forceinline__ half8_t load8(const half_t* p) {
  return *reinterpret_cast<const half8_t*>(p);
}
// Streaming variant: weights are read exactly once per launch, so do not let
// them displace x / idx / partials from the caches.
__device__ __forceinline__ half8_t load8_stream(const half_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(p));
}
// The same from a pointer that is known to point into LDS (a generic pointer would make the
// access a flat load, which the hardware cannot order against global loads without waiting for all).
__device__ __forceinline__ half8_t load8_lds(const half_t* p) {
  return *(const __attribute__((address_space(3))) half8_t*)(p);
}
template <bool LDS>
__device__ __forceinline__ half8_t load8_from(const half_t* p) {
  if constexpr (LDS) return load8_lds(p);
  else return load8(p);
}
__device__ __forceinline__ void store8(half_t* p, half8_t v) {
  *reinterpret_cast<half8_t*>(p) = v;
}

__device__ __forceinline__ half8_t zero8() {
  half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
  return z;
}

// acc += dot(w, x) over 8 fp16 pairs with fp32 fused multiply-adds, strictly in
// element order 0..7 (the predictor's canonical order depends on this).
__device__ __forceinline__ float fma8_ordered(half8_t w, half8_t x, float acc) {
#pragma unroll
  for (int e = 0; e < 8; ++e) acc = __builtin_fmaf((float)w[e], (float)x[e], acc);
  return acc;
}

// Same sum via v_dot2_f32_f16 (two MACs per instruction, fp32 accumulate); the
// pairing is not part of any bit-exact contract.
__device__ __forceinline__ float dot8_fast(half8_t w, half8_t x, float acc) {
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    half2_t a = {w[e], w[e + 1]};
    half2_t b = {x[e], x[e + 1]};
    acc = __builtin_amdgcn_fdot2(a, b, acc, false);
  }
  return acc;
}

// Xor-butterfly sum over groups of LANES consecutive lanes (LANES power of two,
// <= 64), offsets LANES/2 .. 1.  Every lane of the group ends with the total.
template <int LANES>
__device__ __forceinline__ float butterfly_sum(float v) {
#pragma unroll
  for (int off = LANES / 2; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

template <int LANES>
__device__ __forceinline__ float butterfly_max(float v) {
#pragma unroll
  for (int off = LANES / 2; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

__device__ __forceinline__ int64_t load_index(const void* idx, int idx_bytes, int i) {
  return idx_bytes == 8 ? reinterpret_cast<const int64_t*>(idx)[i]
                        : (int64_t) reinterpret_cast<const int32_t*>(idx)[i];
}

// Fixed-point form of an fp32 partial sum: v * 2^32 rounded to the nearest integer.  Integer
// additions commute, so partial sums added in this form give the same bits in any order.
__device__ __forceinline__ long long to_fixed(float v) { return __float2ll_rn(v * 4294967296.f); }
// Back to fp32 with three single-precision operations (no 64-bit arithmetic): the integer part is
// exact in fp32 for every sum of interest, the fraction is rounded to 24 bits, the sum once more.
// Every consumer of a fixed-point sum uses this function, so all of them see the same bits.
__device__ __forceinline__ float from_fixed(long long a) {
  const int hi = (int)(a >> 32);
  const unsigned lo = (unsigned)a;
  return __builtin_fmaf((float)lo, 2.3283064365386963e-10f, (float)hi);
}

__device__ __forceinline__ float relu_f(float x) { return x >= 0.f ? x : 0.f; }

// The activations of the reference's gathered fc1 (Dejavu/src/ops/triton/k_activations.py:73-162),
// applied to the fp32 sum (+ bias) before it is rounded to fp16.  Codes as DV_ACT_* of the C ABI.
__device__ __forceinline__ float act_f(float x, int act) {
  switch (act) {
    case 1: return relu_f(x);
    case 2: return x * 0.5f * (1.f + erff(x * 0.70710678118654752440f));                    // gelu
    case 3: return 0.5f * x * (1.f + tanhf(0.79788456080286535588f * x * (1.f + 0.044715f * x * x)));  // gelu_approx
    case 4: { const float r = relu_f(x); return r * r; }                                    // squared_relu
    default: return x;
  }
}

}  // namespace dv
