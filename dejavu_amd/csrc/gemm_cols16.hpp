// fc2 / out_proj over a transposed weight for batches of 5..32 rows on v_mfma_f32_16x16x32_f16:
//   Y[b, n] = sum_m H[b, m] * W[row(m), n]      (row(m) as in gather_cols_kernel)
//
// The contraction runs over gathered ROWS while an MFMA operand wants 8 consecutive k per lane, so the
// weight tile is transposed inside each lane's registers (no LDS): lane (j = l % 16, kg = l / 16)
// loads 8 consecutive columns 8 j .. 8 j + 7 of the rows 8 kg .. 8 kg + 7 of a 32-row step (one load
// instruction = 4 rows x 256 contiguous bytes); column e of its 8 x 8 block is the B operand of MFMA e
// (k = its 8 rows, output column 8 j + e).  H (batch row i = l % 16, the same 8 rows) is the A operand,
// one 128-bit load per step and batch tile.  Eight MFMAs per batch tile consume a 32 x 128 tile and
// need 4 accumulator registers each (32 per batch tile; the 32x32x16 form of gather_cols_mfma_kernel
// needs 128), so that two workgroups fit a compute unit and twice the weight bytes are in flight.
//
// A workgroup of WAVES wavefronts owns 128 columns and one row group (gridDim.y groups); its wavefronts
// take consecutive shares of the group's rows and add their sums through LDS in a fixed tree order;
// the group's fp32 partial goes to partial[(g * B + b) * N + n] (cols_reduce_kernel adds the groups in
// ascending order), or with one group straight to Y (+ bias).  A wavefront first writes the weight-row
// ids of its share to a private LDS table (-1: no row), so the main loop has no dependent global loads:
// two steps (16 weight loads of 1 KiB) are in flight per wavefront, all unconditional.
//
// Requirements (checked on the host): M % 8 == 0, ldh % 8 == 0, H 16-byte aligned, N % 8 == 0,
// ldw % 8 == 0; BLOCKED: blk % 8 == 0; rows_per_wave a multiple of 64 and <= kC16MaxRows.
// Rows without a valid id contribute nothing (weights and H entries are zeroed for them).
#pragma once
#include "common.hpp"
#include "gemm_mfma.hpp"

namespace dv {

constexpr int kC16Cols = 128;      // columns per workgroup
constexpr int kC16Step = 32;       // rows per MFMA k-step
constexpr int kC16MaxRows = 1024;  // rows per wavefront (LDS id table)

template <int BT, int WAVES, bool IDX64, bool BLOCKED>
__global__ __launch_bounds__(WAVES * 64, 2) void gather_cols_mfma16_kernel(
    const half_t* __restrict__ H, int64_t ldh, int x_expanded, const half_t* __restrict__ W, int64_t ldw,
    const half_t* __restrict__ bias, const void* __restrict__ idx, int blk, int B, int N, int Z, int M,
    int rows_per_block, int rows_per_wave, float* __restrict__ partial, half_t* __restrict__ Y) {
  constexpr int NACC = 8 * BT * 4;  // accumulator values per lane
  // the id tables and, after the main loop, the exchange buffer of the reduction share one LDS block
  constexpr int kTabBytes = WAVES * kC16MaxRows * 4, kRedBytes = (WAVES / 2) * NACC * kWave * 4;
  __shared__ __attribute__((aligned(16))) unsigned char s_raw[kTabBytes > kRedBytes ? kTabBytes : kRedBytes];
  int(*s_rid)[kC16MaxRows] = reinterpret_cast<int(*)[kC16MaxRows]>(s_raw);
  float(*s_red)[NACC][kWave] = reinterpret_cast<float(*)[NACC][kWave]>(s_raw);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, kg = lane >> 4;
  const int ct = blockIdx.x, g = blockIdx.y, G = gridDim.y;
  const int col0 = ct * kC16Cols;
  // columns past N accumulate values that are never stored; their loads re-read column 0
  const int wcol = col0 + l16 * 8 < N ? col0 + l16 * 8 : 0;
  const int m_begin = g * rows_per_block + wave * rows_per_wave;
  int m_end = m_begin + rows_per_wave;
  if (m_end > (g + 1) * rows_per_block) m_end = (g + 1) * rows_per_block;
  if (m_end > M) m_end = M;
  const int nrows = m_end > m_begin ? m_end - m_begin : 0;
  const int nsteps = (nrows + 2 * kC16Step - 1) / (2 * kC16Step) * 2;  // even; 0 for an empty share

  // weight-row ids of the share, -1 where there is no row
  int* tab = s_rid[wave];
  for (int r = lane; r < nsteps * kC16Step; r += kWave) {
    const int m = m_begin + r;
    int64_t id = -1;
    if (m < m_end) {
      if (BLOCKED) {
        const int q = m / blk;
        const int64_t h = IDX64 ? reinterpret_cast<const int64_t*>(idx)[q]
                                : (int64_t) reinterpret_cast<const int32_t*>(idx)[q];
        id = (h >= 0 && h < Z / blk) ? h * blk + (m - q * blk) : -1;
      } else {
        id = IDX64 ? reinterpret_cast<const int64_t*>(idx)[m]
                   : (int64_t) reinterpret_cast<const int32_t*>(idx)[m];
      }
      if (id < 0 || id >= Z) id = -1;
    }
    tab[r] = (int)id;
  }
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();

  float4_t acc[8][BT];
#pragma unroll
  for (int e = 0; e < 8; ++e)
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) acc[e][bt] = float4_t{0.f, 0.f, 0.f, 0.f};

  struct Stage {
    half8_t w[8];
    half8_t h[BT];
    unsigned bad;  // bit q: row q of the lane's eight has no valid id
  };
  // requests step s: the lane's eight weight rows and its H operands
  auto load_step = [&](Stage& st, int s) {
    const int r0 = s * kC16Step + kg * 8;
    const int4 ia = *reinterpret_cast<const int4*>(tab + r0);
    const int4 ib = *reinterpret_cast<const int4*>(tab + r0 + 4);
    const int ids[8] = {ia.x, ia.y, ia.z, ia.w, ib.x, ib.y, ib.z, ib.w};
    unsigned bad = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      bad |= (unsigned)(ids[q] < 0) << q;
      st.w[q] = load8_stream(W + (int64_t)(ids[q] >= 0 ? ids[q] : 0) * ldw + wcol);
    }
    st.bad = bad;
    // H: eight consecutive entries (the compact layout, or one head block of the expanded one)
    int64_t h0 = x_expanded ? (int64_t)(ids[0] >= 0 ? ids[0] : 0) : (int64_t)(m_begin + r0);
    if (!x_expanded && h0 + 8 > M) h0 = 0;  // a group of eight past M: all eight rows are invalid
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) {
      const int b = bt * 16 + l16;
      st.h[bt] = load8(H + (int64_t)(b < B ? b : 0) * ldh + h0);
    }
  };
  auto multiply = [&](const half8_t (&bop)[8], const half8_t (&h)[BT]) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int bt = 0; bt < BT; ++bt) acc[e][bt] = mfma_16x16x32(h[bt], bop[e], acc[e][bt]);
  };
  // transposes the stage's 8 x 8 block into the eight B operands; rows without an id become zero
  // (and so do their H entries: H may hold anything there)
  auto transpose = [&](Stage& st, half8_t (&bop)[8], half8_t (&h)[BT]) {
    if (__ballot(st.bad != 0) != 0) {  // rare
#pragma unroll
      for (int q = 0; q < 8; ++q)
        if ((st.bad >> q) & 1u) {
          st.w[q] = zero8();
#pragma unroll
          for (int bt = 0; bt < BT; ++bt) st.h[bt][q] = (half_t)0.f;
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int q = 0; q < 8; ++q) bop[e][q] = st.w[q][e];
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) h[bt] = st.h[bt];
  };

  if (nsteps > 0) {
    Stage sa, sb;
    load_step(sa, 0);
    load_step(sb, 1);
    half8_t bop[8], hh[BT];
    int s = 0;
    for (; s + 2 < nsteps; s += 2) {  // nsteps is even: steps s + 2 and s + 3 exist
      transpose(sa, bop, hh);
      __builtin_amdgcn_sched_barrier(0);
      load_step(sa, s + 2);
      __builtin_amdgcn_sched_barrier(0);
      multiply(bop, hh);
      transpose(sb, bop, hh);
      __builtin_amdgcn_sched_barrier(0);
      load_step(sb, s + 3);
      __builtin_amdgcn_sched_barrier(0);
      multiply(bop, hh);
    }
    transpose(sa, bop, hh);
    multiply(bop, hh);
    transpose(sb, bop, hh);
    multiply(bop, hh);
  }

  // add the wavefronts' sums through LDS, halving the number of holders per round:
  // (w0 + w4) .. (w3 + w7), then (w0 + w2), (w1 + w3), then w0 + w1: a fixed order
  __syncthreads();  // every wavefront is done with its id table
#pragma unroll
  for (int stride = WAVES / 2; stride >= 1; stride >>= 1) {
    if (wave >= stride && wave < 2 * stride) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int bt = 0; bt < BT; ++bt)
#pragma unroll
          for (int v = 0; v < 4; ++v) s_red[wave - stride][(e * BT + bt) * 4 + v][lane] = acc[e][bt][v];
    }
    __syncthreads();
    if (wave < stride) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int bt = 0; bt < BT; ++bt)
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[e][bt][v] += s_red[wave][(e * BT + bt) * 4 + v][lane];
    }
    if (stride > 1) __syncthreads();
  }

  // value v of MFMA e: batch row 4 kg + v (+ 16 per batch tile), column col0 + 8 l16 + e; for a fixed
  // (bt, v) a lane holds eight consecutive columns
  const int n0 = col0 + l16 * 8;
  if (wave == 0 && n0 < N) {  // N % 8 == 0: a lane's eight columns are all inside or all outside
#pragma unroll
    for (int bt = 0; bt < BT; ++bt)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int b = bt * 16 + 4 * kg + v;
        if (b < B) {
          if (G == 1) {
            half8_t o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (half_t)(acc[e][bt][v] + (bias ? (float)bias[n0 + e] : 0.f));
            store8(Y + (int64_t)b * N + n0, o);
          } else {
            const float4_t lo{acc[0][bt][v], acc[1][bt][v], acc[2][bt][v], acc[3][bt][v]};
            const float4_t hi{acc[4][bt][v], acc[5][bt][v], acc[6][bt][v], acc[7][bt][v]};
            float* dst = partial + ((int64_t)g * B + b) * N + n0;
            *reinterpret_cast<float4_t*>(dst) = lo;
            *reinterpret_cast<float4_t*>(dst + 4) = hi;
          }
        }
      }
  }
}

}  // namespace dv
