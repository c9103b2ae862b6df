// Y[b, m] = act( sum_n X[b, n] * W[row(m), n] + bias[row(m)] ) for MANY rows of X (256 and more:
// long prompts, the late positions of a batched back-fill window), where the product is bound by
// the matrix cores and by LDS bandwidth rather than by the weight stream.
//
// gemm_tiled_mfma_kernel reads BOTH operands of every MFMA from LDS (the weights are staged through a
// wavefront-private tile): 10 KiB of LDS reads per 16 MFMAs of a wavefront, more than the LDS delivers
// at full matrix-core rate.  Here a workgroup of four wavefronts (one per SIMD, so each may keep up
// to 512 registers) owns 128 rows of X and 64 * WT weight rows; a wavefront keeps a 128 x (16 * WT)
// block of fp32 sums (8 * WT accumulator tiles) and
//  * takes its weight operands STRAIGHT from memory in MFMA layout (lane l: row l % 16, the 16 bytes
//    at k-group l / 16 of a 32-column step), four chunks of 64 columns ahead of their use (a ring of
//    register stages; every load is unconditional and statically indexed, so the compiler counts them);
//  * reads only the X operands from LDS: the 128 x 64 block of X of a chunk is staged once per
//    workgroup (double-buffered in LDS, loaded three chunks ahead, one workgroup barrier per chunk).
// LDS reads per MFMA fall to a quarter (8 KiB per 8 * WT MFMAs).  The workgroups that share a weight
// tile (the blocks of X) sit on one XCD, as in gemm_tiled_mfma_kernel, so the tile leaves HBM once.
// Same operand layout, same order of the k-steps and the same epilogue as gemm_tiled_mfma_kernel
// without column splits: the same bits.
// Requires N % 256 == 0 (four chunks per turn of the ring), ldx % 8 == 0, ldw % 8 == 0.
#pragma once
#include "common.hpp"
#include "gemm_mfma.hpp"
#include "gemm_tiled.hpp"

namespace dv {

constexpr int kBgXRows = 128;  // rows of X per workgroup
constexpr int kBgKC = 64;      // columns per chunk
constexpr int kBgRing = 4;     // chunks per turn of the weight ring (three in flight)
constexpr int kBgLd = kBgKC + 8;  // halfs per LDS row (bank spread)

constexpr size_t big_lds_bytes() { return (size_t)2 * kBgXRows * kBgLd * sizeof(half_t); }

template <int WT, bool QKV>
__global__ __launch_bounds__(256, 1) void gemm_big_mfma_kernel(
    const half_t* __restrict__ X, int64_t ldx, const half_t* __restrict__ W, int64_t ldw,
    const half_t* __restrict__ bias, const void* __restrict__ idx, int idx_bytes, int B, int N, int Z, int M,
    half_t* __restrict__ Y, int64_t ldy, int act, QkvScatter qs) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  half_t* xs = reinterpret_cast<half_t*>(smem_raw);  // [2][kBgXRows][kBgLd]
  constexpr int BT = kBgXRows / 16;
  constexpr int WROWS = 16 * WT;
  constexpr int XV = kBgXRows * (kBgKC / 8) / 256;  // X vectors per thread and chunk
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kg = lane >> 4;

  int bx = blockIdx.x, by = blockIdx.y;
  if (gridDim.x > 1 && gridDim.y % 8 == 0) {  // blocks of X that share a weight tile: one XCD
    const int lin = bx + (int)gridDim.x * by;
    const int xcd = lin & 7, q = lin >> 3;
    by = (q / (int)gridDim.x) * 8 + xcd;
    bx = q % (int)gridDim.x;
  }
  const int b0 = bx * kBgXRows;
  const int m0 = (by * 4 + wave) * WROWS;
  const int nchunks = N / kBgKC;

  int rid_mine = -1;  // weight row of output row m0 + lane (lanes < WROWS)
  if (lane < WROWS && m0 + lane < M) {
    const int m = m0 + lane;
    if (QKV) {
      rid_mine = qkv_row_of(qs, m);
    } else {
      const int64_t id = idx == nullptr ? (int64_t)m : load_index(idx, idx_bytes, m);
      rid_mine = (id >= 0 && id < Z) ? (int)id : -1;
    }
  }
  // operand pointers: tile wt, row l16, k-group kg.  Rows out of range read row 0 (never stored).
  const half_t* wptr[WT];
#pragma unroll
  for (int wt = 0; wt < WT; ++wt) {
    const int rid = __shfl(rid_mine, wt * 16 + l16, kWave);
    wptr[wt] = W + (int64_t)(rid >= 0 ? rid : 0) * ldw + kg * 8;
  }
  // X vector p of a thread: row (p * 256 + tid) / 8 of the block, columns (tid % 8) * 8 of the chunk.
  // Rows past B re-read the block's first row: their sums are never stored, and a row of X only
  // reaches its own outputs, so nothing has to be zeroed (and no load hides behind a branch).
  const half_t* xptr[XV];
#pragma unroll
  for (int p = 0; p < XV; ++p) {
    const int b = b0 + (p * 256 + tid) / (kBgKC / 8);
    xptr[p] = X + (int64_t)(b < B ? b : b0) * ldx + (tid % (kBgKC / 8)) * 8;
  }
  half_t* xdst = xs + ((tid / (kBgKC / 8)) * kBgLd + (tid % (kBgKC / 8)) * 8);  // + p * 32 rows, + buffer

  float4_t acc[WT][BT];
#pragma unroll
  for (int wt = 0; wt < WT; ++wt)
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) acc[wt][bt] = float4_t{0.f, 0.f, 0.f, 0.f};

  half8_t wr[kBgRing][2][WT];
  half8_t xr[kBgRing][XV];
  // chunks past the end (requested by the last turns of the ring) re-read chunk 0 and are never multiplied
  auto load_w = [&](half8_t (&w)[2][WT], int c) {
    const int col = (c < nchunks ? c : 0) * kBgKC;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int wt = 0; wt < WT; ++wt) w[ks][wt] = load8(wptr[wt] + col + ks * 32);
  };
  auto load_x = [&](half8_t (&x)[XV], int c) {
    const int col = (c < nchunks ? c : 0) * kBgKC;
#pragma unroll
    for (int p = 0; p < XV; ++p) x[p] = load8(xptr[p] + col);
  };
  auto store_x = [&](const half8_t (&x)[XV], int buf) {
#pragma unroll
    for (int p = 0; p < XV; ++p)
      store8(xdst + (size_t)buf * kBgXRows * kBgLd + (size_t)p * (256 / (kBgKC / 8)) * kBgLd, x[p]);
  };
  auto multiply = [&](const half8_t (&w)[2][WT], int buf) {
    const half_t* xb = xs + (size_t)buf * kBgXRows * kBgLd + l16 * kBgLd + kg * 8;
    half8_t b[2][BT];
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) b[0][bt] = load8(xb + bt * 16 * kBgLd);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      __builtin_amdgcn_sched_barrier(0);
      if (ks == 0) {
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) b[1][bt] = load8(xb + bt * 16 * kBgLd + 32);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int bt = 0; bt < BT; ++bt)
#pragma unroll
        for (int wt = 0; wt < WT; ++wt) acc[wt][bt] = mfma_16x16x32(w[ks][wt], b[ks][bt], acc[wt][bt]);
    }
  };
  // One chunk c (ring slots and buffers are compile-time per call site).  The load counter retires in
  // order, so what a step waits for decides how much stays in flight: X is requested BEFORE the
  // weights of the same step and three chunks ahead; handing chunk c + 1 of X to the other LDS buffer
  // (all wavefronts left it at the last barrier) then waits for loads two steps old and leaves the
  // weights of chunks c + 1 .. c + 3 on their way.
  auto step = [&](int c, half8_t (&w)[2][WT], half8_t (&wfree)[2][WT], half8_t (&xnext)[XV], half8_t (&xfree)[XV],
                  int buf) {
    __builtin_amdgcn_sched_barrier(0);
    load_x(xfree, c + kBgRing - 1);
    load_w(wfree, c + kBgRing - 1);
    __builtin_amdgcn_sched_barrier(0);
    store_x(xnext, buf ^ 1);
    multiply(w, buf);
    __syncthreads();
  };

  load_x(xr[0], 0);
  load_w(wr[0], 0);
  load_x(xr[1], 1);
  load_w(wr[1], 1);
  load_x(xr[2], 2);
  load_w(wr[2], 2);
  store_x(xr[0], 0);
  __syncthreads();
  for (int c = 0; c < nchunks; c += kBgRing) {
    step(c, wr[0], wr[3], xr[1], xr[3], 0);
    step(c + 1, wr[1], wr[0], xr[2], xr[0], 1);
    step(c + 2, wr[2], wr[1], xr[3], xr[1], 0);
    step(c + 3, wr[3], wr[2], xr[0], xr[2], 1);
  }

  // value v of a lane: output row m0 + wt * 16 + 4 * kg + v, X row b0 + bt * 16 + l16
  QkvXRow xrow[QKV ? BT : 1];
  if (QKV) {
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) xrow[bt] = qkv_x_row(qs, b0 + bt * 16 + l16);
  }
#pragma unroll
  for (int wt = 0; wt < WT; ++wt) {
    const int mrow = m0 + wt * 16 + 4 * kg;
    int rid[4];
    float bv[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      rid[v] = __shfl(rid_mine, wt * 16 + 4 * kg + v, kWave);
      bv[v] = (bias != nullptr && rid[v] >= 0) ? (float)bias[rid[v]] : 0.f;
    }
    QkvOutRows orow{};
    if (QKV) orow = qkv_out_rows(qs, mrow, rid[0]);
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) {
      const int b = b0 + bt * 16 + l16;
      if (b >= B || mrow >= M) continue;
      float val[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        val[v] = rid[v] >= 0 ? acc[wt][bt][v] + bv[v] : 0.f;
        if (act) val[v] = act_f(val[v], act);
      }
      if (QKV) {
        // the four values of a lane are four consecutive rows of one (q|k|v, head): hd % 4 == 0
        qkv_store4(qs, Y, xrow[bt], orow, val);
        continue;
      }
      half_t* dst = Y + (int64_t)b * ldy + mrow;
      if (mrow + 3 < M && (ldy & 3) == 0 && (reinterpret_cast<uintptr_t>(Y) & 7) == 0) {
        half4_t o = {(half_t)val[0], (half_t)val[1], (half_t)val[2], (half_t)val[3]};
        *reinterpret_cast<half4_t*>(dst) = o;
      } else {
#pragma unroll
        for (int v = 0; v < 4; ++v)
          if (mrow + v < M) dst[v] = (half_t)val[v];
      }
    }
  }
}

}  // namespace dv
