// Batched (5 <= B <= 64) gathered GEMMs on the matrix cores.  The gathered weight
// rows are streamed with coalesced 128-bit loads into LDS and read back in MFMA
// operand layout.  fc1 (rows kernel) uses v_mfma_f32_16x16x32_f16 with the batch
// padded to tiles of 16; fc2 (columns kernel, here for 33..64 rows; up to 32 rows
// gemm_cols16.hpp) uses v_mfma_f32_32x32x16_f16 with the batch padded to tiles of 32.
//
// Operand layout of the 32x32x16 fp16 MFMA (64 lanes): lane l holds, for the A
// operand, 8 consecutive-k values of row (l % 32), k-group (l / 32); for the B
// operand 8 k values of column (l % 32), same k-group; the 32x32 fp32 result has
// 16 values per lane: value v is row 8*(v/4) + 4*(l/32) + (v%4), column l % 32.
#pragma once
#include "common.hpp"

namespace dv {

__device__ __forceinline__ float16_t mfma_32x32x16(half8_t a, half8_t b, float16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float4_t mfma_16x16x32(half8_t a, half8_t b, float4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// ---------------------------------------------------------------------------
// fc1: Y[b, m] = act( sum_n X[b, n] * W[idx[m], n] + bias[idx[m]] ), fp16 out.
// A workgroup of 8 wavefronts owns 16 gathered rows and splits the N columns
// into chunks of KC = 256: wavefront w takes chunks w, w + 8, ...  Per chunk it
// copies its 16 x 256 weight tile to a private LDS region with coalesced loads
// (2 rows per instruction, 512 contiguous bytes each), then issues KC/32
// v_mfma_f32_16x16x32_f16 per batch tile of 16, rows as the A operand
// (lane: row l % 16, k-group l / 16, 8 consecutive k) and X^T as the B operand
// (lane: batch column l % 16, same k-group).  Result layout: value v of lane l
// is row 4 * (l / 16) + v, column l % 16.  Per step a wavefront first stores the
// tile it loaded during the previous step, then issues the X loads of this step
// and the weight loads of the next one (all unconditional: addresses clamped,
// results masked, so that the compiler can count them) and only then multiplies:
// the weight stream stays in flight during the MFMAs.  The 8 partial tiles are
// summed through LDS in wavefront order.  idx == nullptr means no gather (row m
// of W).  N % 8 == 0, ldw % 8 == 0, B <= 16 * BT.
// ---------------------------------------------------------------------------
constexpr int kMfmaKC = 256;            // columns per staged chunk
constexpr int kMfmaRowPad = 8;          // halfs of padding per LDS row (bank spread)
constexpr int kMfmaLdsRow = kMfmaKC + kMfmaRowPad;
constexpr int kMfmaWaves = 8;
constexpr int kMfmaRows = 16;

// SPLIT: few row tiles with long rows (the first product of a predictor: ~1000 rows of d
// elements) would leave most compute units idle, so the chunks are also split over
// gridDim.y: workgroup (t, y) takes chunks [y * chunks_per_split, (y + 1) * chunks_per_split)
// and writes the raw fp32 sums to partial[(y * B + b) * M + m]; rows_split_reduce_kernel adds
// the splits in ascending order.  No bias / activation in this mode.
// XLDS (one batch tile only): the X operands take the same road as the weights -- coalesced loads
// (2 batch rows x 512 contiguous bytes per instruction) one step ahead, a wavefront-private LDS tile,
// read back in MFMA layout -- instead of 64-byte segments of 16 rows per load straight from memory.
template <int BT, bool IDX64, bool RELU, bool SPLIT = false, bool XLDS = false>
__global__ __launch_bounds__(kMfmaWaves * 64) void gather_rows_mfma_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const void* __restrict__ idx, int B, int N, int64_t ldw, int Z, int M, half_t* __restrict__ Y,
    int chunks_per_split = 0, float* __restrict__ partial = nullptr, int act = 1) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  static_assert(!XLDS || BT <= 2, "X through LDS: at most two batch tiles (passes through one LDS tile)");
  half_t* tile = reinterpret_cast<half_t*>(smem_raw) + (size_t)wave * (XLDS ? 2 : 1) * kMfmaRows * kMfmaLdsRow;
  half_t* xtile = tile + kMfmaRows * kMfmaLdsRow;
  float* red = reinterpret_cast<float*>(smem_raw);  // reused after the main loop
  const int l16 = lane & 15, kg = lane >> 4;  // MFMA operand coordinates
  const int l32 = lane & 31, half_id = lane >> 5;  // staging coordinates
  const int nchunks = (N + kMfmaKC - 1) / kMfmaKC;
  const int c_begin = SPLIT ? (int)blockIdx.y * chunks_per_split : 0;
  const int c_end = SPLIT ? (c_begin + chunks_per_split < nchunks ? c_begin + chunks_per_split : nchunks) : nchunks;
  constexpr int KS = kMfmaKC / 32;  // MFMA k-steps per chunk
  // batch tiles are multiplied in passes of at most two, to bound the X registers
  constexpr int BP = (BT < 2 || XLDS) ? 1 : 2;

  for (int t = blockIdx.x; t * kMfmaRows < M; t += gridDim.x) {
    // row id of output row (t*16 + l16), replicated over the four 16-lane groups
    const int m_mine = t * kMfmaRows + l16;
    int64_t id = -1;
    if (m_mine < M)
      id = idx == nullptr ? (int64_t)m_mine  // no gather: row m of W itself
           : IDX64        ? reinterpret_cast<const int64_t*>(idx)[m_mine]
                          : (int64_t) reinterpret_cast<const int32_t*>(idx)[m_mine];
    const bool ok_mine = id >= 0 && id < Z;
    const int rid_mine = ok_mine ? (int)id : 0;
    // the eight staging loads of a chunk: load q covers rows 2q and 2q+1
    const half_t* wrow[8];
    unsigned row_ok = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int row = 2 * q + half_id;
      wrow[q] = W + (int64_t)__shfl(rid_mine, row, kWave) * ldw;
      row_ok |= (unsigned)(__shfl((int)ok_mine, row, kWave) != 0) << q;
    }

    float4_t acc[BT];
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) acc[bt] = float4_t{0.f, 0.f, 0.f, 0.f};

    half8_t stage[8];
    half8_t xstage[XLDS ? BT : 1][XLDS ? 8 : 1];
    half8_t xhold[XLDS && BT > 1 ? 8 : 1];
    auto load_stage = [&](int c) {
      int col = c * kMfmaKC + l32 * 8;
      if (col >= N) col = 0;  // masked when stored
      if (XLDS) {  // batch rows past B re-read row 0; their results are dropped
#pragma unroll
        for (int bt = 0; bt < BT; ++bt)
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const int b = bt * 16 + 2 * q + half_id;
            xstage[bt][q] = load8(X + (int64_t)(b < B ? b : 0) * N + col);
          }
      }
#pragma unroll
      for (int q = 0; q < 8; ++q) stage[q] = load8_stream(wrow[q] + col);
    };
    auto store_stage = [&](int c) {
      const bool col_ok = c * kMfmaKC + l32 * 8 < N;
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");  // previous tile fully read
      __builtin_amdgcn_wave_barrier();
      if (XLDS) {
#pragma unroll
        for (int q = 0; q < 8; ++q) store8(xtile + (2 * q + half_id) * kMfmaLdsRow + l32 * 8, xstage[0][q]);
        if (BT > 1) {  // kept aside: the next chunk's loads are requested before the second pass
#pragma unroll
          for (int q = 0; q < 8; ++q) xhold[q] = xstage[BT - 1][q];
        }
      }
#pragma unroll
      for (int q = 0; q < 8; ++q)
        store8(tile + (2 * q + half_id) * kMfmaLdsRow + l32 * 8,
               (col_ok && ((row_ok >> q) & 1u)) ? stage[q] : zero8());
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
      __builtin_amdgcn_wave_barrier();
    };
    // X operands of chunk c for batch tiles [bt0, bt0 + BP): columns past N and batch rows
    // past B read a valid address; the weights there are zero / the results are dropped
    half8_t xb[KS][BP];
    auto load_x = [&](int c, int bt0) {
      if (XLDS) {
        if (bt0 > 0) {  // the second batch tile takes the first one's place in LDS
          __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int q = 0; q < 8; ++q)
            store8(xtile + (2 * q + half_id) * kMfmaLdsRow + l32 * 8, xhold[q]);
          __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
          __builtin_amdgcn_wave_barrier();
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) xb[ks][0] = load8(xtile + l16 * kMfmaLdsRow + ks * 32 + kg * 8);
        return;
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        int kk = c * kMfmaKC + ks * 32 + kg * 8;
        if (kk >= N) kk = 0;
#pragma unroll
        for (int p = 0; p < BP; ++p) {
          const int b = (bt0 + p) * 16 + l16;
          xb[ks][p] = load8(X + (int64_t)(b < B ? b : 0) * N + kk);
        }
      }
    };
    auto multiply = [&](int bt0) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const half8_t a = load8(tile + l16 * kMfmaLdsRow + ks * 32 + kg * 8);
#pragma unroll
        for (int p = 0; p < BP; ++p) acc[bt0 + p] = mfma_16x16x32(a, xb[ks][p], acc[bt0 + p]);
      }
    };

    int c = c_begin + wave;
    if (c < c_end) {
      load_stage(c);
      for (; c + kMfmaWaves < c_end; c += kMfmaWaves) {
        store_stage(c);
        // x before the next chunk's weights, and the compiler must not swap them: the load counter
        // retires in order, so the first multiplies wait for x alone while the weights stay in flight
        load_x(c, 0);
        __builtin_amdgcn_sched_barrier(0);
        load_stage(c + kMfmaWaves);
        __builtin_amdgcn_sched_barrier(0);
        multiply(0);
#pragma unroll
        for (int bt0 = BP; bt0 < BT; bt0 += BP) {
          load_x(c, bt0);
          multiply(bt0);
        }
      }
      store_stage(c);
#pragma unroll
      for (int bt0 = 0; bt0 < BT; bt0 += BP) {
        load_x(c, bt0);
        multiply(bt0);
      }
    }
    // sum the 8 wavefronts' partial tiles (fixed order) and finish
    __syncthreads();  // every wavefront is done with its staging region
#pragma unroll
    for (int bt = 0; bt < BT; ++bt)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[((wave * BT + bt) * 4 + v) * 64 + lane] = acc[bt][v];
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int bt = 0; bt < BT; ++bt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float val = 0.f;
#pragma unroll
          for (int w = 0; w < kMfmaWaves; ++w) val += red[((w * BT + bt) * 4 + v) * 64 + lane];
          const int row = 4 * kg + v;
          const int m = t * kMfmaRows + row;
          const int rid = __shfl(rid_mine, row, kWave);
          const bool ok = __shfl((int)ok_mine, row, kWave) != 0;
          if (SPLIT) {
            const int b = bt * 16 + l16;
            if (m < M && b < B) partial[((int64_t)blockIdx.y * B + b) * M + m] = ok ? val : 0.f;
            continue;
          }
          val += (bias != nullptr && ok) ? (float)bias[rid] : 0.f;
          if (RELU) val = act_f(val, act);  // RELU: an activation is applied, act says which
          if (!ok) val = 0.f;
          const int b = bt * 16 + l16;
          if (m < M && b < B) Y[(int64_t)b * M + m] = (half_t)val;
        }
    }
    __syncthreads();  // red is staging memory again
  }
}

// Y[o] = fp16(sum_y partial[y * total + o]), splits added in ascending order.
__global__ __launch_bounds__(256) void rows_split_reduce_kernel(const float* __restrict__ partial, int nsplit,
                                                                int64_t total, half_t* __restrict__ Y) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= total) return;
  float s = 0.f;
  for (int y = 0; y < nsplit; ++y) s += partial[(int64_t)y * total + o];
  Y[o] = (half_t)s;
}

// ---------------------------------------------------------------------------
// Dense product with SHORT rows: Y[b, m] = sum_n X[b, n] * W[m, n], N <= 1024 (the second
// product of a low-rank predictor: many rows of ~1000 elements).  Splitting such a row over
// eight wavefronts leaves most of them idle and makes every 16-row tile re-read all of X, so
// here every wavefront owns whole 16-row tiles (all N columns) and the workgroup stages X once
// in LDS, zero-padded to 16 * BT rows of ceil(N / 256) * 256 columns, for all its wavefronts
// and all the tiles they walk.  Weight tiles go through a wavefront-private LDS tile as in
// gather_rows_mfma_kernel; two chunks of 256 columns are in flight per wavefront (registers
// A / B), their loads unconditional and clamped so that the compiler can count them.  A lane
// ends up with 4 consecutive m of one batch row per batch tile: one 8-byte store when M % 4 == 0.
// blockDim.x = 64 * waves (the host picks the wavefront count that balances the tiles over the
// compute units); dynamic LDS = 16 * BT * (NC * 256 + 8) halfs + waves * 16 * 264 halfs.
// N % 8 == 0, ldw % 8 == 0, B <= 16 * BT.
// ---------------------------------------------------------------------------
template <int BT>
__global__ __launch_bounds__(512) void rows_short_mfma_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, int64_t ldw, int B, int N, int M,
    half_t* __restrict__ Y) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nwaves = blockDim.x >> 6;
  const int nchunks = (N + kMfmaKC - 1) / kMfmaKC;
  const int xs_row = nchunks * kMfmaKC + kMfmaRowPad;  // halfs per staged X row
  half_t* xs = reinterpret_cast<half_t*>(smem_raw);
  half_t* tile = xs + (size_t)16 * BT * xs_row + (size_t)wave * kMfmaRows * kMfmaLdsRow;
  const int l16 = lane & 15, kg = lane >> 4;
  const int l32 = lane & 31, half_id = lane >> 5;
  constexpr int KS = kMfmaKC / 32;

  // X, zero-padded, once per workgroup
  const int vec_per_row = nchunks * kMfmaKC / 8;
  for (int o = threadIdx.x; o < 16 * BT * vec_per_row; o += blockDim.x) {
    const int b = o / vec_per_row, col = (o - b * vec_per_row) * 8;
    store8(xs + (size_t)b * xs_row + col, (b < B && col < N) ? load8(X + (int64_t)b * N + col) : zero8());
  }
  __syncthreads();

  const int ntiles = (M + kMfmaRows - 1) / kMfmaRows;
  const int tstride = gridDim.x * nwaves;
  const int t_first = blockIdx.x * nwaves + wave;
  if (t_first >= ntiles) return;
  const int my_tiles = (ntiles - t_first + tstride - 1) / tstride;
  const int nsteps = my_tiles * nchunks;  // step s: tile t_first + (s / nchunks) * tstride, chunk s % nchunks

  // weight tile of step s into 8 registers: rows 2q + half_id, 8 columns at l32 * 8 (rows past M
  // and columns past N read a valid address and are zeroed when stored)
  auto load_stage = [&](half8_t (&stage)[8], int sidx) {
    const int t = t_first + (sidx / nchunks) * tstride, c = sidx % nchunks;
    int col = c * kMfmaKC + l32 * 8;
    if (col >= N) col = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      int m = t * kMfmaRows + 2 * q + half_id;
      if (m >= M) m = M - 1;
      stage[q] = load8_stream(W + (int64_t)m * ldw + col);
    }
  };
  auto store_stage = [&](const half8_t (&stage)[8], int sidx) {
    const int t = t_first + (sidx / nchunks) * tstride, c = sidx % nchunks;
    const bool col_ok = c * kMfmaKC + l32 * 8 < N;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");  // previous tile fully read
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const bool ok = col_ok && t * kMfmaRows + 2 * q + half_id < M;
      store8(tile + (2 * q + half_id) * kMfmaLdsRow + l32 * 8, ok ? stage[q] : zero8());
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };
  float4_t acc[BT];
  auto multiply = [&](int sidx) {
    const int c = sidx % nchunks;
    if (c == 0) {
#pragma unroll
      for (int bt = 0; bt < BT; ++bt) acc[bt] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const half8_t a = load8(tile + l16 * kMfmaLdsRow + ks * 32 + kg * 8);
#pragma unroll
      for (int bt = 0; bt < BT; ++bt) {
        const half8_t xv = load8(xs + (size_t)(bt * 16 + l16) * xs_row + c * kMfmaKC + ks * 32 + kg * 8);
        acc[bt] = mfma_16x16x32(a, xv, acc[bt]);
      }
    }
    if (c == nchunks - 1) {  // tile complete: value v of a lane is row 4 * kg + v, batch column l16
      const int t = t_first + (sidx / nchunks) * tstride;
      const int m0 = t * kMfmaRows + 4 * kg;
#pragma unroll
      for (int bt = 0; bt < BT; ++bt) {
        const int b = bt * 16 + l16;
        if (b < B) {
          half_t* y = Y + (int64_t)b * M + m0;
          if ((M & 3) == 0 && m0 < M) {
            half4_t o;
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = (half_t)acc[bt][v];
            *reinterpret_cast<half4_t*>(y) = o;
          } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
              if (m0 + v < M) y[v] = (half_t)acc[bt][v];
          }
        }
      }
    }
  };

  half8_t sa[8], sb[8];
  load_stage(sa, 0);
  if (nsteps > 1) load_stage(sb, 1);
  int sidx = 0;
  for (; sidx + 3 < nsteps; sidx += 2) {  // steps sidx, sidx + 1 with sidx + 2, sidx + 3 prefetched
    store_stage(sa, sidx);
    load_stage(sa, sidx + 2);
    multiply(sidx);
    store_stage(sb, sidx + 1);
    load_stage(sb, sidx + 3);
    multiply(sidx + 1);
  }
  // the last one to three steps: nothing, or one more tile, left to prefetch
  store_stage(sa, sidx);
  if (sidx + 2 < nsteps) load_stage(sa, sidx + 2);
  multiply(sidx);
  if (sidx + 1 < nsteps) {
    store_stage(sb, sidx + 1);
    multiply(sidx + 1);
  }
  if (sidx + 2 < nsteps) {
    store_stage(sa, sidx + 2);
    multiply(sidx + 2);
  }
}

// ---------------------------------------------------------------------------
// fc2 / out_proj over a transposed weight: Y[b, n] = sum_m H[b, m] * W[row(m), n].
// The contraction index m runs over gathered ROWS, while the MFMA wants 8
// consecutive k per lane: the transposition happens inside each lane's registers,
// no LDS involved.  A wavefront streams 256 columns; with one batch tile the four wavefronts of
// a workgroup share their 256 columns and take a quarter of the group's rows each.  Lanes 0..31 load 16 bytes
// (8 columns) of row m, lanes 32..63 the same columns of row m + 8, eight rows
// each per k-step of 16 (one load instruction reads 2 rows x 512 contiguous
// bytes).  A lane then holds an 8 x 8 block (8 rows x its 8 columns); read
// column-wise, column e of that block is exactly an operand of
// v_mfma_f32_32x32x16_f16 for output column 8 * (lane % 32) + e and k-group
// lane / 32, so eight MFMAs (e = 0..7) consume the 16 x 256 tile.  H^T (m x b) is
// the other operand, straight from memory.  Two k-steps (32 rows) are in flight per
// pipeline step; the next step's loads are issued before the MFMAs (all loads
// unconditional so that the compiler can count them).  Partial sums over the
// row groups (gridDim.y) go to `partial` [(g * B + b) * N + n] and are reduced by
// cols_reduce_kernel; with one group the result (+ bias) is written directly.
// Row mapping as gather_cols_kernel: BLOCKED ? idx[m / blk] * blk + m % blk : idx[m];
// x_expanded: H is (B, Z) indexed by row(m) instead of (B, M) indexed by m.
// HVEC: H is read with 128-bit loads; the host guarantees M % 8 == 0, ldh % 8 == 0, a
// 16-byte aligned H and, for the expanded layout, blk % 8 == 0 (groups of 8 rows never
// straddle a block).  Otherwise H is gathered element by element.
// ---------------------------------------------------------------------------
constexpr int kMfmaColWave = 256;                 // columns per wavefront
// Columns per workgroup.  One batch tile (B <= 32): the four wavefronts share 256 columns and split the
// rows.  Two batch tiles: 256 accumulator registers per lane leave no room for the exchange (it
// spilled: 110.6 us against 107.0 us for fc2 at batch 64), so there the wavefronts split the columns
// and every wavefront writes its own partial.
constexpr int mfma_col_tile(int bt) { return bt == 1 ? kMfmaColWave : 4 * kMfmaColWave; }
constexpr int kMfmaColRows = 32;                  // rows per pipeline step (two k-steps of 16)
constexpr int kMfmaColSub = 4;                    // row sub-ranges (wavefronts) per workgroup

template <int BT, bool IDX64, bool BLOCKED, bool HVEC>
__global__ __launch_bounds__(256) void gather_cols_mfma_kernel(
    const half_t* __restrict__ H, int64_t ldh, int x_expanded, const half_t* __restrict__ W,
    int64_t ldw, const half_t* __restrict__ bias, const void* __restrict__ idx, int blk, int B, int N,
    int Z, int M, int rows_per_block, float* __restrict__ partial, half_t* __restrict__ Y) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half_id = lane >> 5, l32 = lane & 31;
  const int ct = blockIdx.x, g = blockIdx.y, G = gridDim.y;
  constexpr bool SPLIT_ROWS = BT == 1;
  const int col0 = ct * mfma_col_tile(BT) + (SPLIT_ROWS ? 0 : wave * kMfmaColWave);
  // columns past N accumulate garbage that is never stored; their loads re-read column 0
  const int wcol = col0 + l32 * 8 < N ? col0 + l32 * 8 : 0;
  // the four wavefronts take consecutive quarters of the group's rows (whole pipeline steps)
  const int rpw = ((rows_per_block + kMfmaColSub - 1) / kMfmaColSub + kMfmaColRows - 1) / kMfmaColRows * kMfmaColRows;
  const int m_begin = g * rows_per_block + (SPLIT_ROWS ? wave * rpw : 0);
  int m_end = m_begin + (SPLIT_ROWS ? rpw : rows_per_block);
  if (m_end > (g + 1) * rows_per_block) m_end = (g + 1) * rows_per_block;
  if (m_end > M) m_end = M;
  const bool any_rows = m_begin < m_end;
  // raw index word of row (mb + l32); rows past the group re-read its first row
  auto fetch_index = [&](int mb) -> int64_t {
    if (!any_rows) return -1;
    int m = mb + l32;
    if (m >= m_end) m = m_begin;
    if (BLOCKED) m /= blk;
    return IDX64 ? reinterpret_cast<const int64_t*>(idx)[m]
                 : (int64_t) reinterpret_cast<const int32_t*>(idx)[m];
  };
  // weight row of row (mb + l32), or -1
  auto to_row = [&](int mb, int64_t raw) -> int {
    const int m = mb + l32;
    int64_t id = raw;
    if (BLOCKED) id = (raw >= 0 && raw < Z / blk) ? raw * blk + (m % blk) : -1;
    return (m < m_end && id >= 0 && id < Z) ? (int)id : -1;
  };

  float16_t acc[8][BT];
#pragma unroll
  for (int e = 0; e < 8; ++e)
#pragma unroll
    for (int bt = 0; bt < BT; ++bt)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[e][bt][v] = 0.f;

  constexpr int KS = kMfmaColRows / 16;  // MFMA k-steps per pipeline step
  constexpr int NQ = KS * 8;             // weight load instructions per step
  half8_t next[NQ];                      // rows of the step being loaded
  unsigned next_ok = 0;                  // bit q: next[q] holds a real row
  // load q of a step fetches row (q / 8) * 16 + half_id * 8 + q % 8 of the step
  auto load_stage = [&](int rid_all) {
    next_ok = 0;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int rid = __shfl(rid_all, (q / 8) * 16 + half_id * 8 + (q % 8), kWave);
      next[q] = load8_stream(W + (int64_t)(rid >= 0 ? rid : 0) * ldw + wcol);
      next_ok |= (unsigned)(rid >= 0) << q;
    }
  };
  half8_t hb[KS][BT];
  auto load_h = [&](int mb, int rid_cur) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int mk = ks * 16 + half_id * 8;  // first of this lane's 8 rows
      if (HVEC) {
        // the lane's 8 rows are 8 consecutive entries of H[b, :] (compact gather, or one head
        // block of the expanded layout): one 128-bit load.  Rows without a valid id carry
        // zero weights, so whatever (finite) value H holds there contributes nothing.
        const int rid0 = __shfl(rid_cur, mk, kWave);
        int64_t h0 = x_expanded ? (int64_t)(rid0 >= 0 ? rid0 : 0) : (int64_t)(mb + mk);
        if (!x_expanded && h0 + 8 > M) h0 = M - 8;  // M % 8 == 0 and M >= 8 here
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) {
          const int b = bt * 32 + l32;
          hb[ks][bt] = load8(H + (int64_t)(b < B ? b : 0) * ldh + h0);
        }
      } else {
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) {
          const int b = bt * 32 + l32;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int rid = __shfl(rid_cur, mk + j, kWave);
            const int m = mb + mk + j;
            hb[ks][bt][j] = (b < B && rid >= 0)
                                ? H[(int64_t)b * ldh + (x_expanded ? (int64_t)rid : (int64_t)m)]
                                : (half_t)0.f;
          }
        }
      }
    }
  };
  half8_t cur[NQ];  // rows of the step being multiplied
  auto consume = [&](unsigned cur_ok) {
    if (__ballot(cur_ok != (1u << NQ) - 1u) != 0) {  // rare: rows without a valid id
#pragma unroll
      for (int q = 0; q < NQ; ++q)
        if (!((cur_ok >> q) & 1u)) cur[q] = zero8();
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        half8_t a;  // column e of the lane's 8 x 8 block
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] = cur[ks * 8 + j][e];
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) acc[e][bt] = mfma_32x32x16(hb[ks][bt], a, acc[e][bt]);
      }
    }
  };

  if (any_rows) {
    int rid_cur = to_row(m_begin, fetch_index(m_begin));
    int rid_n1 = to_row(m_begin + kMfmaColRows, fetch_index(m_begin + kMfmaColRows));
    load_stage(rid_cur);
    int mb = m_begin;
    for (; mb + kMfmaColRows < m_end; mb += kMfmaColRows) {
      const unsigned cur_ok = next_ok;
#pragma unroll
      for (int q = 0; q < NQ; ++q) cur[q] = next[q];
      // H operands of this step and the index words of the step after next first, then the
      // weight loads of the next step: the wait for the former leaves the latter in flight
      load_h(mb, rid_cur);
      const int64_t raw_n2 = fetch_index(mb + 2 * kMfmaColRows);
      load_stage(rid_n1);
      consume(cur_ok);
      rid_cur = rid_n1;
      rid_n1 = to_row(mb + 2 * kMfmaColRows, raw_n2);
    }
    const unsigned cur_ok = next_ok;
#pragma unroll
    for (int q = 0; q < NQ; ++q) cur[q] = next[q];
    load_h(mb, rid_cur);
    consume(cur_ok);
  }
  // The four wavefronts' sums are added through LDS in the fixed order (w0 + w2) + (w1 + w3), one
  // batch tile at a time (2 x 32 KiB): a group then costs one (B, N) fp32 partial instead of four,
  // and the partials are what the second pass has to write and read back.
  __shared__ float red[SPLIT_ROWS ? 2 : 1][SPLIT_ROWS ? 8 * 16 : 1][kWave];
#pragma unroll
  for (int bt = 0; SPLIT_ROWS && bt < BT; ++bt) {
    if (wave >= 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int v = 0; v < 16; ++v) red[wave - 2][e * 16 + v][lane] = acc[e][bt][v];
    }
    __syncthreads();
    if (wave < 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[e][bt][v] += red[wave][e * 16 + v][lane];
    }
    __syncthreads();
    if (wave == 1) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int v = 0; v < 16; ++v) red[0][e * 16 + v][lane] = acc[e][bt][v];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[e][bt][v] += red[0][e * 16 + v][lane];
    }
    if (bt + 1 < BT) __syncthreads();
  }
  // H^T is the first operand, so result rows are batch entries and result columns the lane's
  // weight columns: value v of MFMA e is batch row 8 * (v / 4) + 4 * half_id + v % 4, column
  // 8 * l32 + e.  For a fixed v the eight MFMAs hold eight consecutive columns: one vector store.
  const int n0 = col0 + l32 * 8;
  if ((wave == 0 || !SPLIT_ROWS) && n0 < N) {  // N % 8 == 0: a lane's eight columns are all inside or all outside
#pragma unroll
    for (int bt = 0; bt < BT; ++bt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int b = bt * 32 + 8 * (v / 4) + 4 * half_id + (v % 4);
        if (b < B) {
          if (G == 1) {
            half8_t o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (half_t)(acc[e][bt][v] + (bias ? (float)bias[n0 + e] : 0.f));
            store8(Y + (int64_t)b * N + n0, o);
          } else {
            float4_t lo{acc[0][bt][v], acc[1][bt][v], acc[2][bt][v], acc[3][bt][v]};
            float4_t hi{acc[4][bt][v], acc[5][bt][v], acc[6][bt][v], acc[7][bt][v]};
            float* dst = partial + ((int64_t)g * B + b) * N + n0;
            *reinterpret_cast<float4_t*>(dst) = lo;
            *reinterpret_cast<float4_t*>(dst + 4) = hi;
          }
        }
      }
  }
}

}  // namespace dv
