// QKV projection of the active heads for SEVERAL window tokens at once, on the
// matrix cores.  When a head was skipped for some tokens of the back-fill window,
// its K / V rows of all those tokens are recomputed in one pass over the head's
// weights: one v_mfma_f32_16x16x32_f16 multiplies 16 weight rows by all 16
// window slots, so the cost hardly grows with the number of back-filled tokens
// (the per-token dot products of qkv_sparse_kernel grow by about 40 % from 1 to
// 8 tokens).
//
// A workgroup of WAVES wavefronts owns 16 consecutive weight rows of one
// (q|k|v, head) and splits the d columns into chunks of 256 (wavefront w takes
// chunks w, w + WAVES, ...).  Same pipeline as gather_rows_mfma_kernel: a chunk's
// 16 x 256 weight tile is loaded with coalesced 512-byte row segments, stored to
// a wavefront-private LDS tile one step later and read back in MFMA operand
// layout; the x rows of the live slots come straight from memory (lanes of dead
// slots all read one and the same address, so they cost no traffic).  All loads
// are unconditional so that the compiler can count them: the next chunk's weight
// loads stay in flight during the MFMAs.  The WAVES partial tiles are added
// through LDS in wavefront order.  Requires d % 8 == 0 and hd % 16 == 0.  Same
// outputs as qkv_sparse_body (the fp32 summation order differs).
//
// TILES = 2: a workgroup owns 32 consecutive weight rows (two MFMA row tiles,
// hd % 32 == 0) and every x operand feeds two MFMAs, which halves the x traffic
// from L2; that matters when all 16 slots are live (the flush step of a window,
// where the x reads are as large as the weight reads).  Each accumulator sees
// the same operands in the same order as with TILES = 1: identical bits.
#pragma once
#include "attention.hpp"
#include "common.hpp"
#include "gemm_mfma.hpp"

namespace dv {

constexpr int kQkvMfmaWaves = 4;

//
// LN: the newest window token (slot ln.token) is not in X yet: its row is the residual stream row
// ln.R1, normalised on the fly from the precomputed statistics (QkvLnArgs).  Per chunk, the lower
// half of each wavefront normalises the chunk's 256 columns into a wavefront-private LDS row, from
// which the lanes of that slot take their operands; workgroup 0 also stores the normalised row
// to ln.x_row_out.  Same values as a stored LayerNorm row, so the same bits as without LN.
template <int WAVES, int TILES = 1, bool LN = false>
__device__ __forceinline__ void qkv_window_mfma_body(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, const int* __restrict__ batch_idx, int nb, int d, int H,
    int hd, int nnz, half_t* __restrict__ Y, half_t* __restrict__ k_cache,
    half_t* __restrict__ v_cache, const int* __restrict__ padding, int S, int block_id,
    int nblocks, const QkvLnArgs& ln = QkvLnArgs{}) {
  constexpr int kTile = kMfmaRows * kMfmaLdsRow;  // halves per 16-row tile
  __shared__ __attribute__((aligned(16))) half_t s_tiles[WAVES][TILES * kTile];
  __shared__ __attribute__((aligned(16))) half_t s_xnew[LN ? WAVES : 1][LN ? kMfmaKC : 8];
  static_assert(sizeof(half_t) * TILES * kTile >= TILES * 256 * sizeof(float), "tile too small for the reduction");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  half_t* tile = s_tiles[wave];
  const int l16 = lane & 15, kg = lane >> 4;       // MFMA operand coordinates
  const int l32 = lane & 31, half_id = lane >> 5;  // staging coordinates
  constexpr int ROWS = 16 * TILES;
  const int groups_per_head = hd / ROWS;
  const int ntasks = nnz * 3 * groups_per_head;
  const int nchunks = (d + kMfmaKC - 1) / kMfmaKC;
  constexpr int KS = kMfmaKC / 32;
  LnStats st{0.f, 0.f};
  if (LN) st = ln_combine(ln.parts, (d + kLnPart - 1) / kLnPart, d, ln.eps);

  for (int task = block_id; task < ntasks; task += nblocks) {
    const int i = task / (3 * groups_per_head);
    const int rem = task - i * 3 * groups_per_head;
    const int t = rem / groups_per_head;
    const int j0 = (rem - t * groups_per_head) * ROWS;
    const int h = head_idx[i];
    if (h < 0 || h >= H) continue;  // uniform over the workgroup
    int slot = l16 < nb ? batch_idx[i * nb + l16] : -1;
    if (slot >= nb) slot = -1;
    if (__ballot(slot >= 0) == 0) continue;  // every wavefront sees the same 16 slots
    const int64_t row0 = ((int64_t)t * H + h) * hd + j0;
    const bool is_new = LN && slot == ln.token;  // operands come from the LDS row
    // dead slots: every such lane reads the start of row 0 (one line per instruction)
    const bool live = slot >= 0 && !is_new;
    const half_t* xrow = X + (live ? (int64_t)slot * d : 0);
    const bool store_row = LN && block_id == 0 && task == 0;

    float4_t acc[TILES];
#pragma unroll
    for (int r = 0; r < TILES; ++r) acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};
    half8_t stage[8 * TILES];
    auto load_stage = [&](int c) {
      int col = c * kMfmaKC + l32 * 8;
      if (col >= d) col = 0;  // masked when stored
#pragma unroll
      for (int q = 0; q < 8 * TILES; ++q) stage[q] = load8_stream(W + (row0 + 2 * q + half_id) * d + col);
    };
    auto store_stage = [&](int c) {
      const bool col_ok = c * kMfmaKC + l32 * 8 < d;
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");  // previous tile fully read
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int q = 0; q < 8 * TILES; ++q)  // row 2q + half_id of the 16 * TILES rows: tiles are contiguous
        store8(tile + (2 * q + half_id) * kMfmaLdsRow + l32 * 8, col_ok ? stage[q] : zero8());
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
      __builtin_amdgcn_wave_barrier();
    };
    half8_t xb[KS];
    auto load_x = [&](int c) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        int kk = c * kMfmaKC + ks * 32 + kg * 8;
        if (kk >= d || !live) kk = 0;
        xb[ks] = load8(xrow + kk);
      }
    };
    auto multiply = [&]() {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int r = 0; r < TILES; ++r) {
          const half8_t a = load8(tile + (r * 16 + l16) * kMfmaLdsRow + ks * 32 + kg * 8);
          acc[r] = mfma_16x16x32(a, xb[ks], acc[r]);
        }
      }
    };
    // newest token: the chunk's 256 columns of the residual row and of the LayerNorm parameters,
    // four per lane
    half4_t nr, ng, nbt;
    auto load_new = [&](int c) {
      if (LN) {
        int col = c * kMfmaKC + lane * 4;
        if (col >= d) col = 0;  // masked when stored
        nr = *reinterpret_cast<const half4_t*>(ln.R1 + col);
        ng = *reinterpret_cast<const half4_t*>(ln.gamma + col);
        nbt = *reinterpret_cast<const half4_t*>(ln.beta + col);
      }
    };
    auto stage_new = [&](int c) {
      if (LN) {
        half_t* xn = s_xnew[wave];
        const int col = c * kMfmaKC + lane * 4;
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");  // the previous chunk's row fully read
        __builtin_amdgcn_wave_barrier();
        half4_t o = {0, 0, 0, 0};
        if (col < d) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o[e] = (half_t)__builtin_fmaf(((float)nr[e] - st.mean) * st.rstd, (float)ng[e], (float)nbt[e]);
        }
        *reinterpret_cast<half4_t*>(xn + lane * 4) = o;
        if (store_row && col < d) *reinterpret_cast<half4_t*>(ln.x_row_out + col) = o;
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (is_new) {  // LDS reads: they do not take part in the count of outstanding memory loads
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) xb[ks] = load8(xn + ks * 32 + kg * 8);
        }
      }
    };

    int c = wave;
    if (c < nchunks) {
      load_stage(c);
      for (; c + WAVES < nchunks; c += WAVES) {
        store_stage(c);
        // the x operands are requested BEFORE the next chunk's weights and the compiler must not
        // swap them: the load counter retires in order, so the multiplies can then wait for x
        // alone while the weight loads stay in flight
        load_x(c);
        load_new(c);
        __builtin_amdgcn_sched_barrier(0);
        load_stage(c + WAVES);
        __builtin_amdgcn_sched_barrier(0);
        stage_new(c);
        multiply();
      }
      store_stage(c);
      load_x(c);
      load_new(c);
      stage_new(c);
      multiply();
    }
    __syncthreads();  // every wavefront is done with its tile: reuse it for the reduction
    float* red = reinterpret_cast<float*>(tile);
#pragma unroll
    for (int r = 0; r < TILES; ++r)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[(r * 16 + 4 * kg + v) * 16 + l16] = acc[r][v];
    __syncthreads();
    for (int o = threadIdx.x; o < 256 * TILES; o += WAVES * kWave) {
      const int m = o >> 4, n = o & 15;
      int sl = n < nb ? batch_idx[i * nb + n] : -1;
      if (sl >= nb) sl = -1;
      if (sl >= 0) {
        float val = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) val += reinterpret_cast<const float*>(s_tiles[w])[o];
        if (bias != nullptr) val += (float)bias[row0 + m];
        const half_t hv = (half_t)val;
        Y[(int64_t)sl * 3 * H * hd + row0 + m] = hv;
        if (t != 0 && k_cache != nullptr) {
          const int dst = sl + (padding ? padding[0] : 0);
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
    __syncthreads();  // the tiles are staging memory again
  }
}

template <int WAVES, int TILES>
__global__ __launch_bounds__(WAVES * 64) void qkv_window_mfma_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, const int* __restrict__ batch_idx, int nb, int d, int H,
    int hd, int nnz, half_t* __restrict__ Y, half_t* __restrict__ k_cache,
    half_t* __restrict__ v_cache, const int* __restrict__ padding, int S) {
  qkv_window_mfma_body<WAVES, TILES>(X, W, bias, head_idx, batch_idx, nb, d, H, hd, nnz, Y, k_cache, v_cache,
                                     padding, S, blockIdx.x, gridDim.x);
}

// ---------------------------------------------------------------------------
// QKV projection of the active heads for ONE token of each of B sequences
// (B <= 16 * XT rows of X, all live), K / V rows appended to per-sequence caches.
// Same tile scheme as qkv_window_mfma_body with one 16-row weight tile per
// workgroup; XT batch tiles share every weight operand.  `live` (nnz, or null)
// lets a pass skip heads: head i is computed when live[i * live_stride] >= 0
// (a back-fill pass over one window token touches only the heads that miss it).
// Cache position of row b: positions[per_sample ? b : 0] + pos_add (positions
// null = 0); rows whose position falls outside [0, S) are projected but not
// cached.  Caches: k_cache (B, H, hd/8, S, 8), v_cache (B, H, S, hd).
// ---------------------------------------------------------------------------
template <int WAVES, int XT>
__device__ __forceinline__ void qkv_batch_mfma_body(
    const half_t* __restrict__ X, int64_t ldx, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, const int* __restrict__ live, int live_stride, int B, int d, int H,
    int hd, int nnz, half_t* __restrict__ Y, half_t* __restrict__ k_cache, half_t* __restrict__ v_cache,
    const int* __restrict__ positions, int per_sample, int pos_add, int S, int block_id, int nblocks) {
  constexpr int kTile = kMfmaRows * kMfmaLdsRow;
  __shared__ __attribute__((aligned(16))) half_t s_tiles[WAVES][kTile];
  static_assert(sizeof(half_t) * kTile >= XT * 256 * sizeof(float), "tile too small for the reduction");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  half_t* tile = s_tiles[wave];
  const int l16 = lane & 15, kg = lane >> 4;
  const int l32 = lane & 31, half_id = lane >> 5;
  const int groups_per_head = hd / 16;
  const int ntasks = nnz * 3 * groups_per_head;
  const int nchunks = (d + kMfmaKC - 1) / kMfmaKC;
  constexpr int KS = kMfmaKC / 32;

  const half_t* xrow[XT];
  bool row_live[XT];
#pragma unroll
  for (int xt = 0; xt < XT; ++xt) {
    const int n = xt * 16 + l16;
    row_live[xt] = n < B;
    xrow[xt] = X + (row_live[xt] ? (int64_t)n * ldx : 0);  // dead rows: one shared address
  }

  for (int task = block_id; task < ntasks; task += nblocks) {
    const int i = task / (3 * groups_per_head);
    const int rem = task - i * 3 * groups_per_head;
    const int t = rem / groups_per_head;
    const int j0 = (rem - t * groups_per_head) * 16;
    const int h = head_idx[i];
    if (h < 0 || h >= H) continue;  // uniform over the workgroup
    if (live != nullptr && live[(int64_t)i * live_stride] < 0) continue;
    const int64_t row0 = ((int64_t)t * H + h) * hd + j0;

    float4_t acc[XT];
#pragma unroll
    for (int xt = 0; xt < XT; ++xt) acc[xt] = float4_t{0.f, 0.f, 0.f, 0.f};
    half8_t stage[8];
    auto load_stage = [&](int c) {
      int col = c * kMfmaKC + l32 * 8;
      if (col >= d) col = 0;  // masked when stored
#pragma unroll
      for (int q = 0; q < 8; ++q) stage[q] = load8_stream(W + (row0 + 2 * q + half_id) * d + col);
    };
    auto store_stage = [&](int c) {
      const bool col_ok = c * kMfmaKC + l32 * 8 < d;
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");  // previous tile fully read
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int q = 0; q < 8; ++q)
        store8(tile + (2 * q + half_id) * kMfmaLdsRow + l32 * 8, col_ok ? stage[q] : zero8());
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
      __builtin_amdgcn_wave_barrier();
    };
    half8_t xb[XT][KS];
    auto load_x = [&](int c) {
#pragma unroll
      for (int xt = 0; xt < XT; ++xt)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          int kk = c * kMfmaKC + ks * 32 + kg * 8;
          if (kk >= d || !row_live[xt]) kk = 0;
          xb[xt][ks] = load8(xrow[xt] + kk);
        }
    };
    // columns beyond d meet zeros in the weight tile; the accumulator columns of dead rows are never stored
    auto multiply = [&]() {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const half8_t a = load8(tile + l16 * kMfmaLdsRow + ks * 32 + kg * 8);
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) acc[xt] = mfma_16x16x32(a, xb[xt][ks], acc[xt]);
      }
    };

    int c = wave;
    if (c < nchunks) {
      load_stage(c);
      for (; c + WAVES < nchunks; c += WAVES) {
        store_stage(c);
        load_x(c);  // x first, then the next weights: the load counter retires in order
        __builtin_amdgcn_sched_barrier(0);
        load_stage(c + WAVES);
        __builtin_amdgcn_sched_barrier(0);
        multiply();
      }
      store_stage(c);
      load_x(c);
      multiply();
    }
    __syncthreads();  // every wavefront is done with its tile: reuse it for the reduction
    float* red = reinterpret_cast<float*>(tile);
#pragma unroll
    for (int xt = 0; xt < XT; ++xt)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[(xt * 16 + l16) * 16 + 4 * kg + v] = acc[xt][v];  // [x row][weight row]
    __syncthreads();
    for (int o = threadIdx.x; o < 256 * XT; o += WAVES * kWave) {
      const int m = o & 15, n = o >> 4;  // weight row fastest: 32-byte runs in Y and the value cache
      if (n < B) {
        float val = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) val += reinterpret_cast<const float*>(s_tiles[w])[o];
        if (bias != nullptr) val += (float)bias[row0 + m];
        const half_t hv = (half_t)val;
        Y[(int64_t)n * 3 * H * hd + row0 + m] = hv;
        if (t != 0 && k_cache != nullptr) {
          const int dst = (positions ? positions[per_sample ? n : 0] : 0) + pos_add;
          const int j = j0 + m;
          if (dst >= 0 && dst < S) {
            if (t == 1)
              k_cache[((((int64_t)n * H + h) * (hd / 8) + j / 8) * S + dst) * 8 + (j & 7)] = hv;
            else
              v_cache[(((int64_t)n * H + h) * S + dst) * hd + j] = hv;
          }
        }
      }
    }
    __syncthreads();  // the tiles are staging memory again
  }
}

template <int WAVES, int XT>
__global__ __launch_bounds__(WAVES * 64) void qkv_batch_mfma_kernel(
    const half_t* __restrict__ X, int64_t ldx, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, const int* __restrict__ live, int live_stride, int B, int d, int H,
    int hd, int nnz, half_t* __restrict__ Y, half_t* __restrict__ k_cache, half_t* __restrict__ v_cache,
    const int* __restrict__ positions, int per_sample, int pos_add, int S) {
  qkv_batch_mfma_body<WAVES, XT>(X, ldx, W, bias, head_idx, live, live_stride, B, d, H, hd, nnz, Y, k_cache,
                                 v_cache, positions, per_sample, pos_add, S, blockIdx.x, gridDim.x);
}

}  // namespace dv
