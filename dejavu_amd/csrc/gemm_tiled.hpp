// Y[b, m] = act( sum_n X[b, n] * W[row(m), n] + bias[row(m)] ) for a block of X rows that is
// SHARED through LDS by the whole workgroup, on the matrix cores: batched fc1 (17..64 rows),
// batched predictor products and the dense products of the prompt phase (128 rows per block).
//
// gather_rows_mfma_kernel gives every workgroup 16 weight rows and lets each wavefront fetch its
// own X operands, so X travels from L2 once per 16-row tile: B/16 times the weight bytes.  Here a
// workgroup of eight wavefronts owns 128 * WT weight rows (16 * WT per wavefront) and walks the
// columns in chunks of KC; per chunk the 16 * BT x KC block of X is staged ONCE into LDS by all
// 512 threads (double-buffered: one workgroup barrier per chunk) and every wavefront multiplies
// its private weight tile, staged through LDS as in the other MFMA kernels, against it.  X then
// travels once per 128 * WT rows.  One workgroup fills a compute unit's LDS, so every wavefront
// keeps TWO chunks of weights in flight (register stages A / B).
// Because that leaves few workgroups for short matrices, the columns are also split over gridDim.z (split-K): split s handles chunks [s * cps, (s + 1) * cps)
// and writes raw fp32 sums to partial[(s * B + b) * M + m]; gemm_split_reduce_kernel adds the splits
// in ascending order, then bias and activation.  With one split the result is written directly.
//
// Operands per v_mfma_f32_16x16x32_f16: A = 16 weight rows x 32 columns, B = 16 X rows x the same
// 32 columns; value v of lane l is weight row 4 * (l / 16) + v, X row l % 16: a lane ends with four
// consecutive m of one batch row (one 8-byte store).
// Grid: x = blocks of 16 * BT X rows (fastest: workgroups that share a weight tile are dispatched
// together), y = groups of 128 * WT weight rows, z = column splits.
// idx == nullptr: no gather (row m of W).  N % 8 == 0, ldx % 8 == 0, ldw % 8 == 0.
#pragma once
#include "common.hpp"
#include "gemm_mfma.hpp"

namespace dv {

constexpr int kTgWaves = 8;  // default; 4-wavefront workgroups (64 * WT rows) when more of them must be resident
constexpr int kTgPad = 8;  // halfs of padding per LDS row (bank spread)

template <int BT, int WT, int KC, int WAVES = kTgWaves>
constexpr size_t tiled_lds_bytes() {
  return (size_t)(2 * 16 * BT + WAVES * 16 * WT) * (KC + kTgPad) * sizeof(half_t);
}

// QKV mode: the M = 3 * Hk * hd output rows are the q, k, v rows of the selected heads
// (m = (t * Hk + i) * hd + j -> weight row (t * H + head_idx[i]) * hd + j).  The X rows are `tokens`
// window tokens of `nseq` sequences each, row r = s * nseq + b (tokens == 1: one token per sequence).
// live[i * live_stride + s * live_tstride] < 0 skips (head i, token s); a head with no live token, or out
// of range, is skipped altogether.  The result of token y_token goes to column `weight row` of
// Y (nseq, 3, H, hd); the K / V rows of every live (head, token) are appended to the per-sequence caches
// k_cache (nseq, H, hd/8, S, 8), v_cache (nseq, H, S, hd) at position
// positions[per_sample ? b : 0] + pos_add + s.
struct QkvScatter {
  const int* head_idx;
  const int* live;
  int live_stride, Hk, H, hd;
  half_t* k_cache;
  half_t* v_cache;
  const int* positions;
  int per_sample, pos_add, S;
  int nseq, tokens, live_tstride, y_token;
};

__device__ __forceinline__ int qkv_row_of(const QkvScatter& q, int m) {
  const int t = m / (q.Hk * q.hd);
  const int rem = m - t * q.Hk * q.hd;
  const int i = rem / q.hd, j = rem - i * q.hd;
  const int h = q.head_idx[i];
  if (h < 0 || h >= q.H || t > 2) return -1;
  if (q.live != nullptr) {
    bool any = false;
    for (int s = 0; s < q.tokens; ++s)
      any |= q.live[(int64_t)i * q.live_stride + (int64_t)s * q.live_tstride] >= 0;
    if (!any) return -1;
  }
  return (t * q.H + h) * q.hd + j;
}

// stores four finished values: consecutive output rows m .. m + 3 of X row r (m % 4 == 0, so they belong to
// one head and one 8-pack of the key cache; weight rows rid .. rid + 3): one 8-byte store to Y for the token
// that is wanted there and, for K / V rows, one to the cache
__device__ __forceinline__ void qkv_store4(const QkvScatter& q, half_t* __restrict__ Y, int r, int m, int rid,
                                           const float (&val)[4]) {
  const int s = q.tokens > 1 ? r / q.nseq : 0;
  const int b = r - s * q.nseq;
  if (q.live != nullptr && q.tokens > 1) {
    const int i = (m % (q.Hk * q.hd)) / q.hd;
    if (q.live[(int64_t)i * q.live_stride + (int64_t)s * q.live_tstride] < 0) return;
  }
  const half4_t o = {(half_t)val[0], (half_t)val[1], (half_t)val[2], (half_t)val[3]};
  if (s == q.y_token) *reinterpret_cast<half4_t*>(Y + (int64_t)b * 3 * q.H * q.hd + rid) = o;
  if (q.k_cache == nullptr) return;
  const int t = rid / (q.H * q.hd);
  if (t == 0) return;
  const int rem = rid - t * q.H * q.hd;
  const int h = rem / q.hd, j = rem - h * q.hd;
  const int dst = (q.positions ? q.positions[q.per_sample ? b : 0] : 0) + q.pos_add + s;
  if (dst < 0 || dst >= q.S) return;
  half_t* p = t == 1 ? q.k_cache + ((((int64_t)b * q.H + h) * (q.hd / 8) + j / 8) * q.S + dst) * 8 + (j & 7)
                     : q.v_cache + (((int64_t)b * q.H + h) * q.S + dst) * q.hd + j;
  *reinterpret_cast<half4_t*>(p) = o;
}

// qkv_store4 in two halves, for kernels whose lanes keep many (X row, output row) pairs: what depends
// on the X row alone and what depends on the output rows alone is worked out once each.
struct QkvXRow {  // X row r
  int s, b, dst;  // window token, sequence, cache position (-1: not cached)
};
struct QkvOutRows {  // output rows m .. m + 3, weight rows rid .. rid + 3 (one head)
  int i, t, rid;
  int64_t head_off;  // ((h) * (hd / 8) + j / 8) * S * 8 + (j & 7) for K, h * S * hd + j for V, without the sequence
};
__device__ __forceinline__ QkvXRow qkv_x_row(const QkvScatter& q, int r) {
  QkvXRow x;
  x.s = q.tokens > 1 ? r / q.nseq : 0;
  x.b = r - x.s * q.nseq;
  const int dst = (q.positions ? q.positions[q.per_sample ? x.b : 0] : 0) + q.pos_add + x.s;
  x.dst = (dst >= 0 && dst < q.S) ? dst : -1;
  return x;
}
__device__ __forceinline__ QkvOutRows qkv_out_rows(const QkvScatter& q, int m, int rid) {
  QkvOutRows o;
  o.i = (m % (q.Hk * q.hd)) / q.hd;
  o.rid = rid;
  o.t = rid >= 0 ? rid / (q.H * q.hd) : 0;
  const int rem = rid - o.t * q.H * q.hd;
  const int h = rem / q.hd, j = rem - h * q.hd;
  o.head_off = o.t == 1 ? ((int64_t)h * (q.hd / 8) + j / 8) * q.S * 8 + (j & 7) : (int64_t)h * q.S * q.hd + j;
  return o;
}
__device__ __forceinline__ void qkv_store4(const QkvScatter& q, half_t* __restrict__ Y, const QkvXRow& x,
                                           const QkvOutRows& o, const float (&val)[4]) {
  if (o.rid < 0) return;
  if (q.live != nullptr && q.tokens > 1 &&
      q.live[(int64_t)o.i * q.live_stride + (int64_t)x.s * q.live_tstride] < 0)
    return;
  const half4_t v = {(half_t)val[0], (half_t)val[1], (half_t)val[2], (half_t)val[3]};
  if (x.s == q.y_token) *reinterpret_cast<half4_t*>(Y + (int64_t)x.b * 3 * q.H * q.hd + o.rid) = v;
  if (q.k_cache == nullptr || o.t == 0 || x.dst < 0) return;
  half_t* p = o.t == 1 ? q.k_cache + (int64_t)x.b * q.H * q.hd * q.S + o.head_off + (int64_t)x.dst * 8
                       : q.v_cache + (int64_t)x.b * q.H * q.S * q.hd + o.head_off + (int64_t)x.dst * q.hd;
  *reinterpret_cast<half4_t*>(p) = v;
}

template <int BT, int WT, int KC, bool QKV = false, int WAVES = kTgWaves>
__global__ __launch_bounds__(WAVES * 64) void gemm_tiled_mfma_kernel(
    const half_t* __restrict__ X, int64_t ldx, const half_t* __restrict__ W, int64_t ldw,
    const half_t* __restrict__ bias, const void* __restrict__ idx, int idx_bytes, int B, int N, int Z, int M,
    half_t* __restrict__ Y, int64_t ldy, int relu, int chunks_per_split, float* __restrict__ partial,
    QkvScatter qs) {
  const bool SPLIT = chunks_per_split > 0;  // uniform
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  constexpr int LD = KC + kTgPad;
  constexpr int XROWS = 16 * BT, WROWS = 16 * WT;
  constexpr int VPR = KC / 8;                      // 16-byte vectors per staged row
  constexpr int XV = XROWS * VPR / (WAVES * 64);  // X vectors per thread and chunk
  constexpr int WV = WROWS * VPR / 64;               // weight vectors per lane and chunk
  static_assert(XROWS * VPR % (WAVES * 64) == 0 && WROWS * VPR % 64 == 0, "staging does not tile");
  half_t* xs = reinterpret_cast<half_t*>(smem_raw);                       // [2][XROWS][LD]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  half_t* ws = xs + (size_t)2 * XROWS * LD + (size_t)wave * WROWS * LD;  // [WROWS][LD], wavefront-private
  const int l16 = lane & 15, kg = lane >> 4;

  // Several blocks of X against the same weight rows: the workgroups that share a weight tile are
  // given consecutive slots of ONE XCD (workgroup ids go round the 8 XCDs, each with its own L2), so
  // that the tile leaves HBM once and the other blocks find it in that L2.
  int bx = blockIdx.x, by = blockIdx.y;
  if (gridDim.x > 1 && gridDim.y % 8 == 0) {
    const int lin = bx + (int)gridDim.x * by;
    const int xcd = lin & 7, q = lin >> 3;
    by = (q / (int)gridDim.x) * 8 + xcd;
    bx = q % (int)gridDim.x;
  }
  const int b0 = bx * XROWS;
  const int m0 = (by * WAVES + wave) * WROWS;  // first output row of this wavefront
  const int nchunks = (N + KC - 1) / KC;
  const int c_begin = SPLIT ? (int)blockIdx.z * chunks_per_split : 0;
  const int c_end = SPLIT ? (c_begin + chunks_per_split < nchunks ? c_begin + chunks_per_split : nchunks) : nchunks;

  // weight row of output row m0 + lane (lanes < WROWS), -1 when out of range
  int rid_mine = -1;
  if (lane < WROWS && m0 + lane < M) {
    const int m = m0 + lane;
    if (QKV) {
      rid_mine = qkv_row_of(qs, m);
    } else {
      const int64_t id = idx == nullptr ? (int64_t)m : load_index(idx, idx_bytes, m);
      rid_mine = (id >= 0 && id < Z) ? (int)id : -1;
    }
  }
  // staging coordinates: weight vector q of a lane is row q * (64 / VPR) + lane / VPR, columns (lane % VPR) * 8
  const int wv_row = lane / VPR, wv_col = (lane % VPR) * 8;
  const half_t* wrow[WV];
  unsigned wrow_ok = 0;
#pragma unroll
  for (int q = 0; q < WV; ++q) {
    const int rid = __shfl(rid_mine, q * (64 / VPR) + wv_row, kWave);
    wrow[q] = W + (int64_t)(rid >= 0 ? rid : 0) * ldw;
    wrow_ok |= (unsigned)(rid >= 0) << q;
  }
  // X vector p of a thread is row (p * 512 + tid) / VPR of the block, columns (tid % VPR) * 8
  const half_t* xrow[XV];
#pragma unroll
  for (int p = 0; p < XV; ++p) {
    const int b = b0 + (p * WAVES * 64 + tid) / VPR;
    xrow[p] = X + (int64_t)(b < B ? b : b0) * ldx;  // rows past B re-read the block's first row; never stored
  }
  const int xv_col = (tid % VPR) * 8;

  float4_t acc[WT][BT];
#pragma unroll
  for (int wt = 0; wt < WT; ++wt)
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) acc[wt][bt] = float4_t{0.f, 0.f, 0.f, 0.f};

  // All loads are unconditional so that the compiler can count them (two chunks stay in flight): a
  // chunk past the end of this split reads one fixed line instead (never stored).
  auto load_stage = [&](half8_t (&wstage)[WV], half8_t (&xstage)[XV], int c) {
    const bool live = c < c_end;
    int wc = c * KC + wv_col, xc = c * KC + xv_col;
    if (wc >= N) wc = 0;  // zeroed when stored
    if (xc >= N) xc = 0;
#pragma unroll
    for (int p = 0; p < XV; ++p) xstage[p] = load8(live ? xrow[p] + xc : X);
#pragma unroll
    for (int q = 0; q < WV; ++q) wstage[q] = load8_stream(live ? wrow[q] + wc : W);
  };
  auto store_stage = [&](const half8_t (&wstage)[WV], const half8_t (&xstage)[XV], int c, int buf) {
    const bool w_ok = c * KC + wv_col < N, x_ok = c * KC + xv_col < N;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");  // this wavefront's reads of its weight tile are done
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = 0; q < WV; ++q)
      store8(ws + (q * (64 / VPR) + wv_row) * LD + wv_col, (w_ok && ((wrow_ok >> q) & 1u)) ? wstage[q] : zero8());
    half_t* xb = xs + (size_t)buf * XROWS * LD;
#pragma unroll
    for (int p = 0; p < XV; ++p)
      store8(xb + ((p * WAVES * 64 + tid) / VPR) * LD + xv_col, x_ok ? xstage[p] : zero8());
  };
  // Per k-step all WT + BT operand reads are issued before the first MFMA (the compiler otherwise
  // alternates one LDS read, a full wait and two MFMAs: with many batch tiles the kernel is then
  // bound by LDS latency, not by the weight stream).  With few operands per step the next step's are
  // requested while the MFMAs of this one run (two register sets); with many (eight batch tiles) there
  // is one set and the other wavefront of the SIMD covers the wait.
  auto multiply = [&](int buf) {
    const half_t* xb = xs + (size_t)buf * XROWS * LD;
    constexpr int KS = KC / 32;
    constexpr int SETS = (WT + BT) <= 6 ? 2 : 1;
    half8_t a[SETS][WT], b[SETS][BT];
    auto fetch = [&](int ks, int slot) {
#pragma unroll
      for (int wt = 0; wt < WT; ++wt) a[slot][wt] = load8(ws + (wt * 16 + l16) * LD + ks * 32 + kg * 8);
#pragma unroll
      for (int bt = 0; bt < BT; ++bt) b[slot][bt] = load8(xb + (bt * 16 + l16) * LD + ks * 32 + kg * 8);
    };
    if (SETS == 2) fetch(0, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = SETS == 2 ? (ks & 1) : 0;
      __builtin_amdgcn_sched_barrier(0);
      if (SETS == 1)
        fetch(ks, 0);
      else if (ks + 1 < KS)
        fetch(ks + 1, cur ^ 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int bt = 0; bt < BT; ++bt)
#pragma unroll
        for (int wt = 0; wt < WT; ++wt) acc[wt][bt] = mfma_16x16x32(a[cur][wt], b[cur][bt], acc[wt][bt]);
    }
  };
  // One chunk: store its stage (weights: wavefront-private tile; X: buffer `buf`), one workgroup barrier
  // (the X block is complete, and every wavefront has finished the multiplies of the chunk before, so the
  // other X buffer may be overwritten next time), request the chunk two ahead, multiply.
  auto step = [&](half8_t (&wstage)[WV], half8_t (&xstage)[XV], int c, int buf) {
    store_stage(wstage, xstage, c, buf);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    load_stage(wstage, xstage, c + 2);
    __builtin_amdgcn_sched_barrier(0);
    multiply(buf);
  };

  half8_t wa[WV], xa[XV], wb[WV], xb2[XV];
  if (c_begin < c_end) {
    load_stage(wa, xa, c_begin);
    load_stage(wb, xb2, c_begin + 1);
    int c = c_begin;
    for (; c + 1 < c_end; c += 2) {
      step(wa, xa, c, 0);
      step(wb, xb2, c + 1, 1);
    }
    if (c < c_end) step(wa, xa, c, 0);
  }

  // value v of a lane: output row m0 + wt * 16 + 4 * kg + v, batch row b0 + bt * 16 + l16
#pragma unroll
  for (int wt = 0; wt < WT; ++wt) {
    const int mrow = m0 + wt * 16 + 4 * kg;
    int rid[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) rid[v] = __shfl(rid_mine, wt * 16 + 4 * kg + v, kWave);
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) {
      const int b = b0 + bt * 16 + l16;
      if (b >= B || mrow >= M) continue;
      float val[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) val[v] = rid[v] >= 0 ? acc[wt][bt][v] : 0.f;
      if (SPLIT) {
        float* dst = partial + ((int64_t)blockIdx.z * B + b) * M + mrow;
        if (mrow + 3 < M && (M & 3) == 0) {
          *reinterpret_cast<float4_t*>(dst) = float4_t{val[0], val[1], val[2], val[3]};
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (mrow + v < M) dst[v] = val[v];
        }
        continue;
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        if (bias != nullptr && rid[v] >= 0) val[v] += (float)bias[rid[v]];
        if (relu) val[v] = act_f(val[v], relu);
      }
      if (QKV) {
        // the four values of a lane are four consecutive rows of one (q|k|v, head): hd % 4 == 0
        if (rid[0] >= 0) qkv_store4(qs, Y, b, mrow, rid[0], val);
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

// Y[b, m] = act(sum_s partial[(s * B + b) * M + m] + bias[row(m)]), splits added in ascending order.
__global__ __launch_bounds__(256) void gemm_split_reduce_kernel(
    const float* __restrict__ partial, int nsplit, int B, int M, const half_t* __restrict__ bias,
    const void* __restrict__ idx, int idx_bytes, int Z, int relu, half_t* __restrict__ Y, int64_t ldy) {
  const int64_t total = (int64_t)B * M;
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= total) return;
  const int b = (int)(o / M), m = (int)(o - (int64_t)b * M);
  float s = 0.f;
  for (int y = 0; y < nsplit; ++y) s += partial[(int64_t)y * total + o];
  if (bias != nullptr) {
    const int64_t id = idx == nullptr ? (int64_t)m : load_index(idx, idx_bytes, m);
    if (id >= 0 && id < Z) s += (float)bias[id];
  }
  if (relu) s = act_f(s, relu);
  Y[(int64_t)b * ldy + m] = (half_t)s;
}

// QKV mode: sums the splits, adds the bias and scatters (Y and the caches).  A thread takes four
// consecutive output rows (one head, M % 4 == 0): 16-byte loads of the partial sums, 8-byte stores.
__global__ __launch_bounds__(256) void qkv_split_reduce_kernel(const float* __restrict__ partial, int nsplit, int B,
                                                               int M, const half_t* __restrict__ bias,
                                                               half_t* __restrict__ Y, QkvScatter qs) {
  const int64_t total = (int64_t)B * M;
  const int64_t o = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (o >= total) return;
  const int b = (int)(o / M), m = (int)(o - (int64_t)b * M);
  const int rid = qkv_row_of(qs, m);
  if (rid < 0) return;
  float4_t s = {0.f, 0.f, 0.f, 0.f};
  for (int y = 0; y < nsplit; ++y) s += *reinterpret_cast<const float4_t*>(partial + (int64_t)y * total + o);
  float val[4] = {s[0], s[1], s[2], s[3]};
  if (bias != nullptr) {
#pragma unroll
    for (int v = 0; v < 4; ++v) val[v] += (float)bias[rid + v];
  }
  qkv_store4(qs, Y, b, m, rid, val);
}

}  // namespace dv
