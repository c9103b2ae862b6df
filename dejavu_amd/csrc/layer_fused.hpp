// One decode step of a whole sparse block in eight launches.  Kernels that are
// independent of each other share a launch ("roles" picked by workgroup index),
// so the small latency-bound pieces (LayerNorm, window step, predictors, top-k)
// run beside the bandwidth-bound ones instead of each paying a launch of its own.
// The role bodies are the very same device functions as the stand-alone kernels.
//
//  L1  add+LayerNorm 1 + back-fill window step          | key histogram of the MLP logits
//  L2  QKV (+ cache scatter) of the active heads
//  L3  attention partials over the active heads        | head predictor fc0 | top-k threshold + counts
//  L4  out_proj over W_out^T, merging the attention    | head predictor fc1 | top-k emission
//      partials on the fly
//  L5  split reduction (+ bias) + residual add
//  L6  LayerNorm 2 of the residual stream, computed inside the fc1 workgroups while they
//      stage their input row (same bits as the stand-alone kernel), then
//      fc1 gather (+bias, ReLU)                         | MLP predictor fc0  | head top-k
//  L8  fc2 gather                                       | MLP predictor fc1
//  L9  split reduction (+ bias)
#pragma once
#include "attention.hpp"
#include "common.hpp"
#include "gemv_cols.hpp"
#include "gemv_rows.hpp"
#include "norm.hpp"
#include "qkv_mfma.hpp"
#include "topk.hpp"

namespace dv {

constexpr int kLnThreads = 1024;

// ---- L1 -------------------------------------------------------------------
// Workgroup 0: LayerNorm + window step; the others: key histogram of this layer's MLP logits (an
// input of the step).  The histogram sits here because the QKV workgroups of the next launch fill
// every slot of the device for its whole duration: a role behind them would only start at its end.
template <int MAXV>
__global__ __launch_bounds__(kLnThreads) void layer_l1_kernel(
    const half_t* __restrict__ hidden, const half_t* __restrict__ residual,
    const half_t* __restrict__ gamma, const half_t* __restrict__ beta, float eps, int d,
    half_t* __restrict__ x, half_t* __restrict__ residual1, half_t* __restrict__ x_cache_row,
    int* __restrict__ tracker, const int* __restrict__ head_idx, int nnz, int H, int counter,
    int flush, int* __restrict__ batch_idx, const half_t* __restrict__ mlp_logits, int ffn,
    unsigned* __restrict__ topk_ws) {
  if (blockIdx.x != 0) {
    topk_hist_body(mlp_logits, 1, ffn, topk_ws, (int)blockIdx.x - 1);
    return;
  }
  add_layer_norm_body<kLnThreads, MAXV>(hidden, residual, gamma, beta, eps, d, x, residual1, x_cache_row, 0);
  window_tracker_step(tracker, head_idx, nnz, H, counter, flush, batch_idx);
}

// ---- L2 -------------------------------------------------------------------
struct QkvArgs {
  const half_t* X;  // window buffer rows [0, nb)
  const half_t* W;
  const half_t* bias;
  const int* head_idx;
  const int* batch_idx;
  int nb, d, H, hd, nnz;
  half_t* Y;
  half_t* k_cache;
  half_t* v_cache;
  const int* padding;
  int S;
};

struct CanonArgs {
  const half_t* X;
  const half_t* W;
  int64_t ldw;
  int rows, n;
  half_t* Y;
};

// canonical GEMV role with the lane count the fixed summation order prescribes for n; short rows
// take the variant with x in LDS and two weight rows per lane group (more loads in flight)
constexpr int kCanonShortRows = 2;

__device__ __forceinline__ void canonical_role(const CanonArgs& c, int block_id, int nblocks) {
  if (c.n <= 1024) {
    __shared__ __attribute__((aligned(16))) float s_xf[1024];
    stage_x_f32(c.X, c.n, s_xf);
    canonical_gemv_lds_body<16, 1, 8, kCanonShortRows>(s_xf, c.W, c.ldw, c.rows, c.n, c.Y, block_id, nblocks);
  } else
    canonical_gemv_body<64, 1, 8>(c.X, c.W, c.ldw, c.rows, c.n, c.Y, block_id, nblocks);
}

template <int NBMAX>
__global__ __launch_bounds__(256) void layer_l2_kernel(QkvArgs q) {
  if constexpr (NBMAX <= 0)  // several live window tokens: matrix-core variant (-1: 32-row workgroups)
    qkv_window_mfma_body<kQkvMfmaWaves, NBMAX == 0 ? 1 : 2>(q.X, q.W, q.bias, q.head_idx, q.batch_idx, q.nb, q.d,
                                                            q.H, q.hd, q.nnz, q.Y, q.k_cache, q.v_cache,
                                                            q.padding, q.S, blockIdx.x, gridDim.x);
  else
    qkv_sparse_body<NBMAX, 2, 4>(q.X, q.W, q.bias, q.head_idx, q.batch_idx, q.nb, q.d, q.H, q.hd, q.nnz, q.Y,
                                 q.k_cache, q.v_cache, q.padding, q.S, blockIdx.x, gridDim.x);
}

// ---- L3 -------------------------------------------------------------------
struct AttnArgs {
  const half_t* Q;
  int64_t ldq;
  const half_t* k_cache;
  const half_t* v_cache;
  const int* head_idx;
  const int* seq_pos;  // device position of the newest token, or nullptr (then n_len counts)
  int n_len, H, S, nsplit, nheads;
  float scale;
  float* part;
};

template <int HD>
__global__ __launch_bounds__(256) void layer_l3_kernel(AttnArgs a, int nblk_attn, CanonArgs hp0, int nblk_hp0,
                                                       const half_t* __restrict__ mlp_logits, int ffn,
                                                       int K, unsigned* __restrict__ topk_ws,
                                                       int* __restrict__ advance_ptr, int advance_by) {
  // flush step: the window's K / V rows went into the caches in the launch before this one; the
  // window now starts advance_by positions later (nothing in this launch or after it reads the value)
  if (advance_ptr != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *advance_ptr += advance_by;
  // the small roles with the longer dependency chains take the first block ids: they are dispatched first
  const int nblk_count = (int)gridDim.x - nblk_attn - nblk_hp0;
  int bid = blockIdx.x;
  if (bid < nblk_count) {
    topk_count_body(mlp_logits, 1, ffn, K, topk_ws, bid, nblk_count);
    return;
  }
  bid -= nblk_count;
  if (bid < nblk_hp0) {
    canonical_role(hp0, bid, nblk_hp0);
    return;
  }
  bid -= nblk_hp0;
  const int split = bid % a.nsplit, i = bid / a.nsplit;
  decode_attn_body<HD, 4>(a.Q, a.ldq, a.k_cache, a.v_cache, a.head_idx, a.seq_pos, a.n_len, a.H, a.S, a.scale,
                          a.nsplit, a.part, split, i, 0, a.nheads);
}

// ---- L4 -------------------------------------------------------------------
struct OutProjArgs {
  const half_t* W;
  int64_t ldw;
  const half_t* bias;
  const int* head_idx;
  int hd, N, Z, M, rows_per_block, col_tiles, groups;
  float* partial;
  half_t* Y;
  const float* attn_part;
  int nsplit;
};

__global__ __launch_bounds__(256) void layer_l4_kernel(OutProjArgs o, int nblk_out, CanonArgs hp1, int nblk_hp1,
                                                       const half_t* __restrict__ mlp_logits, int ffn,
                                                       int K, const unsigned* __restrict__ topk_ws,
                                                       int64_t* __restrict__ mlp_idx_out, int nblk_emit) {
  int bid = blockIdx.x;
  if (bid < nblk_emit) {
    topk_emit_body(mlp_logits, 1, ffn, K, topk_ws, mlp_idx_out, 8, bid, nblk_emit);
    return;
  }
  bid -= nblk_emit;
  if (bid < nblk_hp1) {
    canonical_role(hp1, bid, nblk_hp1);
    return;
  }
  bid -= nblk_hp1;
  const int ct = bid % o.col_tiles, g = bid / o.col_tiles;
  gather_cols_body<1, 8, false, true, true>(nullptr, 0, 1, o.W, o.ldw, o.bias, o.head_idx, o.hd, o.N,
                                            o.Z, o.M, o.rows_per_block, o.partial, o.Y,
                                            o.attn_part, o.nsplit, ct, g, o.groups);
}

// ---- L7 / L8 --------------------------------------------------------------
struct RowsArgs {
  const half_t* X;  // residual stream after attention: normalised on the fly
  const half_t* gamma;
  const half_t* beta;
  float eps;
  const half_t* W;
  const half_t* bias;
  const int64_t* idx;
  int n;
  int64_t ldw;
  int Z, M;
  half_t* Y;
};

template <int MAXV>
__global__ __launch_bounds__(256) void layer_l7_kernel(RowsArgs f, int nblk_fc1, CanonArgs mp0, int nblk_mp0,
                                                       const half_t* __restrict__ head_logits, int H, int att_k,
                                                       int* __restrict__ att_idx_out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int bid = blockIdx.x;
  if (bid < nblk_fc1) {
    // While the row is normalised the memory system would idle: one 4-byte load per lane touches the
    // 64 cache lines (2 rows x 4 KiB) this wavefront streams first, so they are on their way to L2.
    // Requested behind the row's own loads (the load counter retires in order).
    float touch = 0.f;
    const float* touch_ptr = nullptr;
    {
      const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
      const int m = (bid * 4 + wave) * 2 + (lane >> 5);
      // (only for long rows: measured -0.5 us per layer at d = 12288, +0.2 at 9216, +1.0 at 5120, where
      // the extra requests cost more than the head start gains)
      if (f.n >= 10240 && m < f.M && (lane & 31) * 64 < f.n) {
        const int64_t id = f.idx[m];
        if (id >= 0 && id < f.Z) touch_ptr = reinterpret_cast<const float*>(f.W + id * f.ldw + (lane & 31) * 64);
      }
    }
    half_t* xs = reinterpret_cast<half_t*>(smem_raw);
    add_layer_norm_body<256, MAXV>(f.X, nullptr, f.gamma, f.beta, f.eps, f.n, xs, nullptr, nullptr, 0, [&]() {
      __builtin_amdgcn_sched_barrier(0);
      if (touch_ptr != nullptr) touch = *touch_ptr;
      __builtin_amdgcn_sched_barrier(0);
    });
    __syncthreads();
    gather_rows_body<1, 2, 4, true, true>(nullptr, f.W, f.bias, f.idx, 8, f.n, f.ldw, f.Z, f.M, f.Y, xs, bid,
                                          nblk_fc1);
    asm volatile("" ::"v"(touch));  // keeps the load above alive; nothing reads its value
  } else if (bid < nblk_fc1 + nblk_mp0) {
    canonical_role(mp0, bid - nblk_fc1, nblk_mp0);
  } else {
    // head top-k for the next layer (rank selection, one workgroup)
    __shared__ unsigned s_key[1024];
    __shared__ unsigned s_sel[1024];
    for (int j = threadIdx.x; j < H; j += blockDim.x) s_key[j] = topk_key(head_logits[j]);
    __syncthreads();
    rank_select_emit(s_key, s_sel, H, att_k, att_idx_out, 4);
  }
}

struct ColsArgs {
  const half_t* X;
  const half_t* W;
  int64_t ldw;
  const int64_t* idx;
  int N, Z, M, rows_per_block, col_tiles, groups;
  float* partial;
  half_t* Y;
  const half_t* bias;
};

__global__ __launch_bounds__(256) void layer_l8_kernel(ColsArgs c, int nblk_fc2, CanonArgs mp1, int nblk_mp1) {
  const int bid = blockIdx.x;
  if (bid < nblk_fc2) {
    const int ct = bid % c.col_tiles, g = bid / c.col_tiles;
    gather_cols_body<1, 8, true, false, false>(c.X, c.M, 0, c.W, c.ldw, c.bias, c.idx, 1, c.N, c.Z, c.M,
                                               c.rows_per_block, c.partial, c.Y, nullptr, 0, ct, g,
                                               c.groups);
  } else {
    canonical_role(mp1, bid - nblk_fc2, nblk_mp1);
  }
}

}  // namespace dv
