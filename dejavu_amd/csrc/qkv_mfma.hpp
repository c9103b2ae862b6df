// QKV projection of the active heads for MANY window tokens at once, on the
// matrix cores.  When a head was skipped for several tokens of the back-fill
// window, its K / V rows of all those tokens are recomputed in one pass over the
// head's weights; with more than a few live tokens the per-token dot products of
// qkv_sparse_kernel become load-issue bound, whereas one
// v_mfma_f32_16x16x32_f16 multiplies 16 weight rows by all 16 window slots.
//
// A workgroup of WAVES wavefronts owns 16 consecutive weight rows of one
// (q|k|v, head) and splits the d columns among its wavefronts (contiguous
// ranges of 64-column steps).  Operands go from global memory straight to
// registers: lane l holds row (l % 16) of the A operand and window slot (l % 16)
// of the B operand.  Per 64-column step a lane loads columns 8 * (l / 16) .. + 7
// for one MFMA and the same columns + 32 for a second one (any assignment of
// columns to MFMA k positions is valid as long as A and B use the same one), so
// that each load instruction reads 64 contiguous bytes of every weight row.
// Result: value v of lane l is weight row 4 * (l / 16) + v, slot l % 16.  The
// WAVES partial tiles are added through LDS in wavefront order.
// Requires d % 64 == 0 and hd % 16 == 0.  Same outputs as qkv_sparse_body (the
// fp32 summation order differs).
#pragma once
#include "common.hpp"
#include "gemm_mfma.hpp"

namespace dv {

constexpr int kQkvMfmaWaves = 4;
constexpr int kQkvMfmaUnroll = 8;

template <int WAVES, int U>
__device__ __forceinline__ void qkv_window_mfma_body(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, const int* __restrict__ batch_idx, int nb, int d, int H,
    int hd, int nnz, half_t* __restrict__ Y, half_t* __restrict__ k_cache,
    half_t* __restrict__ v_cache, const int* __restrict__ padding, int S, int block_id,
    int nblocks) {
  __shared__ float s_red[WAVES][256];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, kg = lane >> 4;
  const int groups_per_head = hd / 16;
  const int ntasks = nnz * 3 * groups_per_head;
  const int steps = d / 64;
  const int s_begin = (int)((int64_t)steps * wave / WAVES);
  const int s_end = (int)((int64_t)steps * (wave + 1) / WAVES);
  for (int task = block_id; task < ntasks; task += nblocks) {
    const int i = task / (3 * groups_per_head);
    const int rem = task - i * 3 * groups_per_head;
    const int t = rem / groups_per_head;
    const int j0 = (rem - t * groups_per_head) * 16;
    const int h = head_idx[i];
    if (h < 0 || h >= H) continue;  // uniform over the workgroup
    int xb = l16 < nb ? batch_idx[i * nb + l16] : -1;
    if (xb >= nb) xb = -1;
    if (__ballot(xb >= 0) == 0) continue;  // every wavefront sees the same 16 slots
    const int64_t row0 = ((int64_t)t * H + h) * hd + j0;
    const half_t* wr = W + (row0 + l16) * d + kg * 8;
    const half_t* xr = X + (int64_t)(xb >= 0 ? xb : 0) * d + kg * 8;
    const bool live = xb >= 0;

    float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
    // U steps (2 U weight loads of 16 bytes per lane) are in flight at a time; steps past
    // the end of this wavefront's range contribute zeros
    for (int s = s_begin; s < s_end; s += U) {
      half8_t a[U][2], b[U][2];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool in = s + u < s_end;  // uniform over the wavefront
        a[u][0] = in ? load8_stream(wr + (int64_t)(s + u) * 64) : zero8();
        a[u][1] = in ? load8_stream(wr + (int64_t)(s + u) * 64 + 32) : zero8();
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool in = live && s + u < s_end;
        b[u][0] = in ? load8(xr + (int64_t)(s + u) * 64) : zero8();
        b[u][1] = in ? load8(xr + (int64_t)(s + u) * 64 + 32) : zero8();
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        acc = mfma_16x16x32(a[u][0], b[u][0], acc);
        acc = mfma_16x16x32(a[u][1], b[u][1], acc);
      }
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) s_red[wave][(4 * kg + v) * 16 + l16] = acc[v];
    __syncthreads();
    for (int o = threadIdx.x; o < 256; o += WAVES * kWave) {
      const int m = o >> 4, n = o & 15;
      int slot = n < nb ? batch_idx[i * nb + n] : -1;
      if (slot >= nb) slot = -1;
      if (slot >= 0) {
        float val = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) val += s_red[w][o];
        if (bias != nullptr) val += (float)bias[row0 + m];
        const half_t hv = (half_t)val;
        Y[(int64_t)slot * 3 * H * hd + row0 + m] = hv;
        if (t != 0 && k_cache != nullptr) {
          const int dst = slot + (padding ? padding[0] : 0);
          const int j = j0 + m;
          if (dst >= 0 && dst < S) {
            if (t == 1)
              k_cache[(((int64_t)h * (hd / 8) + j / 8) * S + dst) * 8 + (j & 7)] = hv;
            else
              v_cache[((int64_t)h * S + dst) * hd + j] = hv;
          }
        }
      }
    }
    __syncthreads();  // s_red is reused by the next task
  }
}

template <int WAVES, int U>
__global__ __launch_bounds__(WAVES * 64) void qkv_window_mfma_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, const int* __restrict__ batch_idx, int nb, int d, int H,
    int hd, int nnz, half_t* __restrict__ Y, half_t* __restrict__ k_cache,
    half_t* __restrict__ v_cache, const int* __restrict__ padding, int S) {
  qkv_window_mfma_body<WAVES, U>(X, W, bias, head_idx, batch_idx, nb, d, H, hd, nnz, Y, k_cache, v_cache,
                                 padding, S, blockIdx.x, gridDim.x);
}

}  // namespace dv
