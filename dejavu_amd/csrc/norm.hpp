// Fused residual add + LayerNorm for the pre-norm block:
//   r = fp16(h + residual)          (residual stream, stored in fp16)
//   y = fp16(LayerNorm(r) * gamma + beta)   (fp32 statistics)
//
// The statistics are defined over PARTS of 64 consecutive elements so that they can be produced
// where the row is produced (64 columns per workgroup of a split reduction) and combined by
// whoever consumes the row, with the same bits everywhere:
//   vector v = 8 consecutive elements, part p = 8 consecutive vectors (the last part may be short)
//   t_v  = ((((((x0 + x1) + x2) + x3) + x4) + x5) + x6) + x7              (fp32, in this order)
//   s_p  = xor butterfly (4, 2, 1) over the part's eight t_v (absent vectors count 0)
//   m_p  = s_p / n_p                                    (n_p = number of elements of the part)
//   u_v  = fma chain over e = 0..7 of (x_e - m_p)^2, starting from 0
//   q_p  = xor butterfly (4, 2, 1) over the part's eight u_v
// and for the row (P parts), with "lane sum" = lane l of 64 adds parts l, l + 64, ... in ascending
// order and the 64 lane values are combined with an xor butterfly (32 .. 1):
//   mean = lane_sum(s_p) / d
//   var  = lane_sum(fma(n_p * (m_p - mean), m_p - mean, q_p)) / d      (parallel-variance form)
//   rstd = rsqrt(var + eps)
// A part's pair (s_p, q_p) is what travels between kernels (float2 per part).
#pragma once
#include "common.hpp"

namespace dv {

constexpr int kLnPart = 64;  // elements per part
constexpr int kLnMaxPartsConst = 512;  // d <= 32768

struct LnStats {
  float mean, rstd;
};

__device__ __forceinline__ float ln_vec_sum(half8_t h) {
  float t = (float)h[0];
#pragma unroll
  for (int e = 1; e < 8; ++e) t += (float)h[e];
  return t;
}

__device__ __forceinline__ float ln_vec_sq(half8_t h, float m) {
  float u = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float c = (float)h[e] - m;
    u = __builtin_fmaf(c, c, u);
  }
  return u;
}

__device__ __forceinline__ int ln_part_count(int p, int d) {
  const int left = d - p * kLnPart;
  return left < kLnPart ? left : kLnPart;
}

// (s_p, q_p) of the part that the 8 lanes of an aligned lane group hold one vector each of
// (`present`: this lane's vector exists).  Every lane of the group returns the pair.
__device__ __forceinline__ float2 ln_part_stats(half8_t v, bool present, int n_p) {
  const float s = butterfly_sum<8>(present ? ln_vec_sum(v) : 0.f);
  const float m = s / (float)n_p;
  const float q = butterfly_sum<8>(present ? ln_vec_sq(v, m) : 0.f);
  return make_float2(s, q);
}

// The same for a wavefront whose lanes 0..7 hold the part's vectors (the other lanes take part in
// the shuffles only); lanes 0..7 return the pair.
__device__ __forceinline__ float2 ln_part_stats_lanes8(half8_t v, bool present, int n_p) {
  return ln_part_stats(v, present, n_p);
}

// Row statistics from the P part pairs (global memory or LDS), computed by one full wavefront;
// every lane returns the same values.  The loads can be requested ahead of the arithmetic
// (ln_load_parts, then ln_combine_loaded).
// NP: pairs per lane, P <= 64 * NP
constexpr int kLnPartsPerLane = kLnMaxPartsConst / 64;

template <int NP>
struct LnParts {
  float2 v[NP];
};

template <int NP = kLnPartsPerLane>
__device__ __forceinline__ LnParts<NP> ln_load_parts(const float2* parts, int P) {
  const int lane = threadIdx.x & 63;
  LnParts<NP> r;
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int p = lane + k * kWave;
    r.v[k] = p < P ? parts[p] : make_float2(0.f, 0.f);
  }
  return r;
}

template <int NP>
__device__ __forceinline__ LnStats ln_combine_loaded(const LnParts<NP>& r, int P, int d, float eps) {
  const int lane = threadIdx.x & 63;
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NP; ++k)
    if (lane + k * kWave < P) s += r.v[k].x;
  const float mean = butterfly_sum<kWave>(s) / (float)d;
  float q = 0.f;
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    const int p = lane + k * kWave;
    if (p < P) {
      const float n = (float)ln_part_count(p, d);
      const float dm = r.v[k].x / n - mean;
      q += __builtin_fmaf(n * dm, dm, r.v[k].y);
    }
  }
  const float var = butterfly_sum<kWave>(q) / (float)d;
  LnStats st;
  st.mean = mean;
  st.rstd = rsqrtf(var + eps);
  return st;
}

__device__ __forceinline__ LnStats ln_combine(const float2* parts, int P, int d, float eps) {
  return ln_combine_loaded(ln_load_parts(parts, P), P, d, eps);
}

__device__ __forceinline__ half8_t ln_apply(half8_t r, half8_t g, half8_t b, LnStats st) {
  half8_t o;
#pragma unroll
  for (int e = 0; e < 8; ++e)
    o[e] = (half_t)__builtin_fmaf(((float)r[e] - st.mean) * st.rstd, (float)g[e], (float)b[e]);
  return o;
}

__device__ __forceinline__ half8_t add8_rounded(half8_t h, half8_t r) {
  half8_t o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (half_t)((float)h[e] + (float)r[e]);
  return o;
}

constexpr int kLnMaxParts = kLnMaxPartsConst;

// One row by one workgroup of THREADS threads; thread t holds vectors t, t + THREADS, ...
// (NV per thread; requires d % 8 == 0 and d <= 8 * THREADS * NV).
// Y may point to LDS (the row handed to a consumer in the same workgroup) or to memory;
// Y2 (optional) receives a second copy of the normalised row (the back-fill window buffer).
struct LnNoHook {
  __device__ __forceinline__ void operator()() const {}
};
// after_loads: called once the row's loads have been requested (a place to request memory the caller
// needs later: requests queued before the row's loads would delay them, the load counter retires in order)
// Where the row to be added and normalised comes from: vector i (8 columns) of row `row`.
struct LnRowFromMemory {
  const half_t* __restrict__ H;
  int d;
  __device__ __forceinline__ half8_t operator()(int i, int64_t row) const { return load8(H + row * d + i * 8); }
};
// ... or from the fp32 partial sums of a split product, partial[(g * rows + row) * d + column], added
// exactly as cols_reduce_kernel adds them (group g goes to accumulator g % 4 in ascending order, then
// (a0 + a1) + (a2 + a3), + bias, rounded to fp16): the reduction launch folded into the LayerNorm launch.
struct LnRowFromPartials {
  const float* __restrict__ partial;
  const half_t* __restrict__ bias;
  int G, d;
  int64_t total;  // rows * d
  __device__ __forceinline__ half8_t operator()(int i, int64_t row) const {
    const float* p = partial + row * d + i * 8;
    const half8_t bv = bias != nullptr ? load8(bias + i * 8) : zero8();  // requested with the first groups
    float a[4][8];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) a[k][e] = 0.f;
    for (int g0 = 0; g0 < G; g0 += 4) {
      float4_t lo[4], hi[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {  // groups past G re-read the last one and are not added
        const int g = g0 + k < G ? g0 + k : G - 1;
        lo[k] = *reinterpret_cast<const float4_t*>(p + (int64_t)g * total);
        hi[k] = *reinterpret_cast<const float4_t*>(p + (int64_t)g * total + 4);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (g0 + k < G) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            a[k][e] += lo[k][e];
            a[k][4 + e] += hi[k][e];
          }
        }
      }
    }
    half8_t y;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float r = (a[0][e] + a[1][e]) + (a[2][e] + a[3][e]);
      y[e] = (half_t)(r + (bias != nullptr ? (float)bv[e] : 0.f));
    }
    return y;
  }
};

template <int THREADS, int NV, class AfterLoads = LnNoHook, class Src = LnRowFromMemory>
__device__ __forceinline__ void add_layer_norm_src_body(
    Src src, const half_t* __restrict__ R, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, float eps, int d, half_t* __restrict__ Y,
    half_t* __restrict__ Rout, half_t* __restrict__ Y2, int64_t row, AfterLoads after_loads = AfterLoads()) {
  __shared__ float2 s_parts[kLnMaxParts];
  const int nvec = d / 8;
  const int P = (d + kLnPart - 1) / kLnPart;
  constexpr bool EARLY = NV <= 4;  // gamma / beta fetched with the row while registers allow
  half8_t v[NV], rr[NV], gm[EARLY ? NV : 1], bt[EARLY ? NV : 1];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * THREADS;
    rr[j] = (R != nullptr && i < nvec) ? load8(R + row * d + i * 8) : zero8();
    v[j] = i < nvec ? src(i, row) : zero8();
  }
  after_loads();
  if (EARLY) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {  // not needed until the last pass
      const int i = threadIdx.x + j * THREADS;
      gm[j] = i < nvec ? load8(gamma + i * 8) : zero8();
      bt[j] = i < nvec ? load8(beta + i * 8) : zero8();
    }
  }
  __syncthreads();  // s_parts may still be read from a previous call
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * THREADS;
    const bool present = i < nvec;
    if (present) {
      if (R != nullptr) v[j] = add8_rounded(v[j], rr[j]);
      if (Rout != nullptr) store8(Rout + row * d + i * 8, v[j]);
    }
    const int p = i >> 3;
    // whole lane groups of 8 are inside or outside [0, P) together
    const float2 sq = ln_part_stats(v[j], present, p < P ? ln_part_count(p, d) : kLnPart);
    if ((threadIdx.x & 7) == 0 && p < P) s_parts[p] = sq;
  }
  __syncthreads();
  const LnStats st = ln_combine(s_parts, P, d, eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * THREADS;
    if (i < nvec) {
      const half8_t o = ln_apply(v[j], EARLY ? gm[j] : load8(gamma + i * 8), EARLY ? bt[j] : load8(beta + i * 8), st);
      store8(Y + row * d + i * 8, o);
      if (Y2 != nullptr) store8(Y2 + row * d + i * 8, o);
    }
  }
}

template <int THREADS, int NV, class AfterLoads = LnNoHook>
__device__ __forceinline__ void add_layer_norm_body(
    const half_t* __restrict__ H, const half_t* __restrict__ R, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, float eps, int d, half_t* __restrict__ Y,
    half_t* __restrict__ Rout, half_t* __restrict__ Y2, int64_t row, AfterLoads after_loads = AfterLoads()) {
  add_layer_norm_src_body<THREADS, NV, AfterLoads, LnRowFromMemory>(LnRowFromMemory{H, d}, R, gamma, beta, eps, d, Y,
                                                                     Rout, Y2, row, after_loads);
}

// The same for a row that arrives as fixed-point sums (common.hpp: to_fixed): by a whole workgroup
// (a multiple of 64 threads, any d with d % 8 == 0),
//   y = fp16(acc * 2^-32 + bias),  r = fp16(y + R),  xs = fp16(LayerNorm(r) * gamma + beta)
// with xs (d halves) in LDS; r is also stored to Rout when given.  NORM == false: xs = r.  The
// caller synchronises the workgroup before it reads xs.  Same bits as the split reduction's
// fixed-point form followed by add_layer_norm_body.
template <bool NORM, class AfterLoads = LnNoHook>
__device__ __forceinline__ void fixed_add_layer_norm_body(
    const long long* __restrict__ acc, const half_t* __restrict__ bias, const half_t* __restrict__ R,
    const half_t* __restrict__ gamma, const half_t* __restrict__ beta, float eps, int d, half_t* xs,
    half_t* __restrict__ Rout, AfterLoads after_loads = AfterLoads()) {
  __shared__ float2 s_parts[kLnMaxParts];
  typedef long long ll2_t __attribute__((ext_vector_type(2)));
  const int nvec = d / 8;
  const int P = (d + kLnPart - 1) / kLnPart;
  const int T = blockDim.x;
  // The loads of a round of VB vectors per thread are requested together (one round trip per
  // round); a row of up to 8 * KEEP * T elements stays in registers until the statistics are
  // known, and its LayerNorm parameters are requested before the statistics are combined.
  constexpr int VB = 3, KEEP = 3;
  const bool single = nvec <= KEEP * T;
  half8_t r[KEEP], g[KEEP], b[KEEP];
#pragma unroll
  for (int k = 0; k < KEEP; ++k) r[k] = zero8();
  for (int i0 = 0, round = 0; i0 < nvec; i0 += VB * T, ++round) {  // the same trip count for every thread
    ll2_t a[VB][4];
    half8_t bv[VB], rv[VB];
#pragma unroll
    for (int j = 0; j < VB; ++j) {
      const int i = i0 + j * T + (int)threadIdx.x;
      if (i < nvec) {
        const ll2_t* ap = reinterpret_cast<const ll2_t*>(acc + (int64_t)i * 8);
#pragma unroll
        for (int q = 0; q < 4; ++q) a[j][q] = ap[q];
        bv[j] = bias != nullptr ? load8(bias + i * 8) : zero8();
        rv[j] = load8(R + i * 8);
      }
    }
    if (i0 == 0) after_loads();
#pragma unroll
    for (int j = 0; j < VB; ++j) {
      const int i = i0 + j * T + (int)threadIdx.x;
      const bool present = i < nvec;
      half8_t rr = zero8();
      if (present) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const half_t y = (half_t)(from_fixed(a[j][e >> 1][e & 1]) + (float)bv[j][e]);
          rr[e] = (half_t)((float)y + (float)rv[j][e]);
        }
        if (!NORM || !single) store8(xs + i * 8, rr);
        if (Rout != nullptr) store8(Rout + i * 8, rr);
      }
      if (NORM) {
        const int p = i >> 3;
        const float2 sq = ln_part_stats(rr, present, p < P ? ln_part_count(p, d) : kLnPart);
        if ((threadIdx.x & 7) == 0 && p < P) s_parts[p] = sq;
        if (single) {
#pragma unroll
          for (int k = 0; k < KEEP; ++k)
            if (k == round * VB + j) r[k] = rr;
        }
      }
    }
  }
  if (!NORM) return;
  if (single) {
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      const int i = k * T + (int)threadIdx.x;
      if (i < nvec) {
        g[k] = load8(gamma + i * 8);
        b[k] = load8(beta + i * 8);
      }
    }
  }
  __syncthreads();
  const LnStats st = ln_combine(s_parts, P, d, eps);
  if (single) {
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      const int i = k * T + (int)threadIdx.x;
      if (i < nvec) store8(xs + i * 8, ln_apply(r[k], g[k], b[k], st));
    }
    return;
  }
  for (int i = threadIdx.x; i < nvec; i += T)  // a thread's own vectors
    store8(xs + i * 8, ln_apply(load8(xs + i * 8), load8(gamma + i * 8), load8(beta + i * 8), st));
}

template <int THREADS, int NV>
__global__ __launch_bounds__(THREADS) void add_layer_norm_kernel(
    const half_t* __restrict__ H, const half_t* __restrict__ R, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, float eps, int d, half_t* __restrict__ Y,
    half_t* __restrict__ Rout, half_t* __restrict__ Y2 = nullptr) {
  add_layer_norm_body<THREADS, NV>(H, R, gamma, beta, eps, d, Y, Rout, Y2, blockIdx.x);
}

// add + LayerNorm of rows that arrive as the fp32 partial sums of a split product (LnRowFromPartials)
template <int THREADS, int NV>
__global__ __launch_bounds__(THREADS) void reduce_add_layer_norm_kernel(
    const float* __restrict__ partial, const half_t* __restrict__ bias, int G, int rows,
    const half_t* __restrict__ R, const half_t* __restrict__ gamma, const half_t* __restrict__ beta, float eps,
    int d, half_t* __restrict__ Y, half_t* __restrict__ Rout) {
  add_layer_norm_src_body<THREADS, NV, LnNoHook, LnRowFromPartials>(
      LnRowFromPartials{partial, bias, G, d, (int64_t)rows * d}, R, gamma, beta, eps, d, Y, Rout, nullptr, blockIdx.x);
}

}  // namespace dv
