// Decode steps of consecutive sparse blocks, six launches per block (seven for the first block of
// a call).  Kernels that are independent of each other share a launch ("roles" picked by
// workgroup index), so the small latency-bound pieces (window step, predictors, top-k) run beside
// the bandwidth-bound ones instead of each paying a launch of its own, and the two LayerNorms have
// no launch at all: the launch that completes a residual-stream row also leaves the statistics of
// its 64-column parts (norm.hpp), and the consumers normalise the row themselves.
//
//  P   (first block of a call only) residual add + part statistics | key histogram of the MLP
//      logits | back-fill window step
//  L2  QKV (+ cache scatter) of the active heads; every workgroup applies LayerNorm 1 to the
//      newest row from the part statistics
//  L3  attention partials over the active heads        | head predictor fc0 | top-k threshold + counts
//      | zeroing of the out_proj accumulators
//  L4  out_proj over W_out^T, merging the attention    | head predictor fc1 | top-k emission
//      partials on the fly; the row groups add their sums in fixed point with integer atomics
//      (order-independent, so deterministic)
//  L7  every fc1 workgroup rebuilds the residual row from the accumulators (+ bias + residual) and
//      applies LayerNorm 2 while staging it, then
//      fc1 gather (+bias, ReLU)                         | MLP predictor fc0  | head top-k
//  L8  fc2 gather                                       | MLP predictor fc1
//  L9  split reduction (+ bias); when another block follows in the call it is that block's P:
//      + residual add + part statistics | key histogram of the next MLP logits | next window step
#pragma once
#include "attention.hpp"
#include "common.hpp"
#include "gemv_cols.hpp"
#include "gemv_rows.hpp"
#include "norm.hpp"
#include "qkv_mfma.hpp"
#include "topk.hpp"

namespace dv {

// ---- P / L9 ---------------------------------------------------------------
// Role 1 (workgroups [0, nred)): 64 columns each of
//   y = fp16(sum of the fc2 partials + bias)      (partial != nullptr; stored to Y when given)
//   y = Y                                          (partial == nullptr: the block's input)
//   r1 = fp16(y + R) (R == nullptr: y) -> Rout, and the statistics pair of those 64 values -> parts
// Role 2 (nhist workgroups): key histogram of the MLP logits the block will select from.
// Role 3 (one workgroup): back-fill window step of the block.
struct PreArgs {
  const float* partial;
  const half_t* bias;
  int G, d;
  half_t* Y;
  const half_t* R;
  half_t* Rout;
  float2* parts;
  const half_t* mlp_logits;
  int ffn;
  unsigned* topk_ws;
  int* tracker;
  const int* head_idx;
  int nnz, H, counter, flush;
  int* batch_idx;
};

__global__ __launch_bounds__(256) void layer_pre_kernel(PreArgs p, int nred, int nhist) {
  const int bid = blockIdx.x;
  if (bid < nred) {
    cols_reduce_body<false>(p.partial, p.bias, p.G, 1, p.d, p.Y, p.R, p.Rout, p.parts, bid);
  } else if (bid < nred + nhist) {
    topk_hist_body(p.mlp_logits, 1, p.ffn, p.topk_ws, bid - nred);
  } else {
    window_tracker_step(p.tracker, p.head_idx, p.nnz, p.H, p.counter, p.flush, p.batch_idx);
  }
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
  QkvLnArgs ln;
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

// X_LDS: the input row is `x`, a copy the workgroup holds in LDS (else c.X)
template <bool X_LDS = false>
__device__ __forceinline__ void canonical_role(const CanonArgs& c, int block_id, int nblocks,
                                               const half_t* x = nullptr) {
  const half_t* xin = X_LDS ? x : c.X;
  if (c.n <= 1024) {
    __shared__ __attribute__((aligned(16))) float s_xf[1024];
    stage_x_f32<X_LDS>(xin, c.n, s_xf);
    canonical_gemv_lds_body<16, 1, 8, kCanonShortRows>(s_xf, c.W, c.ldw, c.rows, c.n, c.Y, block_id, nblocks);
  } else
    canonical_gemv_body<64, 1, 8, X_LDS>(xin, c.W, c.ldw, c.rows, c.n, c.Y, block_id, nblocks);
}

// NBMAX 1 (d <= 16384) / 2: one window token on the vector ALUs (workgroups of up to 512 threads,
// dynamic LDS: d halves); 0 / -1: several live window tokens on the matrix cores (-1: 32-row workgroups), 256 threads
// (the vector variant keeps six wavefronts per SIMD resident: three workgroups of 512 threads per
// compute unit hold every workgroup of the OPT-175B launch at once)
template <int NBMAX>
__global__ __launch_bounds__(NBMAX >= 1 ? 512 : 256, NBMAX >= 1 ? 6 : 1) void layer_l2_kernel(QkvArgs q) {
  if constexpr (NBMAX <= 0) {
    qkv_window_mfma_body<kQkvMfmaWaves, NBMAX == 0 ? 1 : 2, true>(q.X, q.W, q.bias, q.head_idx, q.batch_idx, q.nb,
                                                                  q.d, q.H, q.hd, q.nnz, q.Y, q.k_cache, q.v_cache,
                                                                  q.padding, q.S, blockIdx.x, gridDim.x, q.ln);
  } else {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    qkv_ln_token_body<2, 4, NBMAX == 1 ? 4 : 8>(q.ln, q.W, q.bias, q.head_idx, q.d, q.H, q.hd, q.nnz, q.Y, q.k_cache, q.v_cache,
                            q.padding, q.S, reinterpret_cast<half_t*>(smem_raw), blockIdx.x, gridDim.x);
  }
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
                                                       int* __restrict__ advance_ptr, int advance_by,
                                                       long long* __restrict__ acc_fixed, int acc_n) {
  // flush step: the window's K / V rows went into the caches in the launch before this one; the
  // window now starts advance_by positions later (nothing in this launch or after it reads the value)
  if (advance_ptr != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *advance_ptr += advance_by;
  // the last workgroup clears the accumulators the out_proj of the next launch adds to
  if (blockIdx.x == gridDim.x - 1) {
    typedef long long ll2_t __attribute__((ext_vector_type(2)));
    const ll2_t z = {0, 0};
    for (int i = threadIdx.x * 2; i < acc_n; i += 2 * 256) *reinterpret_cast<ll2_t*>(acc_fixed + i) = z;
    return;
  }
  // the small roles with the longer dependency chains take the first block ids: they are dispatched first
  const int nblk_count = (int)gridDim.x - 1 - nblk_attn - nblk_hp0;
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
  long long* acc_fixed;
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
  gather_cols_body<1, 8, false, true, true, true>(nullptr, 0, 1, o.W, o.ldw, nullptr, o.head_idx, o.hd, o.N,
                                                  o.Z, o.M, o.rows_per_block, nullptr, nullptr,
                                                  o.attn_part, o.nsplit, ct, g, o.groups, o.acc_fixed);
}

// ---- L7 / L8 --------------------------------------------------------------
struct RowsArgs {
  const long long* acc_fixed;  // out_proj sums of the step, fixed point
  const half_t* out_bias;
  const half_t* res1;          // residual stream before attention
  half_t* res2_out;            // residual stream after attention (stored by workgroup 0)
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

// Workgroups of 256 or 512 threads: every fc1 / predictor workgroup rebuilds the whole row, so the
// larger workgroups are taken when there are enough rows for them (half the copies).
__global__ __launch_bounds__(512, 4) void layer_l7_kernel(RowsArgs f, int nblk_fc1, CanonArgs mp0, int nblk_mp0,
                                                       const half_t* __restrict__ head_logits, int H, int att_k,
                                                       int* __restrict__ att_idx_out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int bid = blockIdx.x;
  if (bid < nblk_fc1) {
    // While the row is rebuilt and normalised the memory system would idle: one 4-byte load per lane
    // touches the 64 cache lines (2 rows x 4 KiB) this wavefront streams first, so they are on their
    // way to L2.  Requested behind the row's own loads (the load counter retires in order).
    float touch = 0.f;
    const float* touch_ptr = nullptr;
    {
      const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
      const int m = (bid * (int)(blockDim.x >> 6) + wave) * 2 + (lane >> 5);
      // (only for long rows: measured -0.5 us per layer at d = 12288, +0.2 at 9216, +1.0 at 5120, where
      // the extra requests cost more than the head start gains)
      if (f.n >= 10240 && m < f.M && (lane & 31) * 64 < f.n) {
        const int64_t id = f.idx[m];
        if (id >= 0 && id < f.Z) touch_ptr = reinterpret_cast<const float*>(f.W + id * f.ldw + (lane & 31) * 64);
      }
    }
    half_t* xs = reinterpret_cast<half_t*>(smem_raw);
    fixed_add_layer_norm_body<true>(f.acc_fixed, f.out_bias, f.res1, f.gamma, f.beta, f.eps, f.n, xs,
                                    bid == 0 ? f.res2_out : nullptr, [&]() {
                                      __builtin_amdgcn_sched_barrier(0);
                                      if (touch_ptr != nullptr) touch = *touch_ptr;
                                      __builtin_amdgcn_sched_barrier(0);
                                    });
    __syncthreads();
    gather_rows_body<1, 2, 4, true, true>(nullptr, f.W, f.bias, f.idx, 8, f.n, f.ldw, f.Z, f.M, f.Y, xs, bid,
                                          nblk_fc1);
    asm volatile("" ::"v"(touch));  // keeps the load above alive; nothing reads its value
  } else if (bid < nblk_fc1 + nblk_mp0) {
    // the MLP predictor reads the residual stream after attention, which no launch has stored:
    // these workgroups rebuild the row as well (without the LayerNorm)
    half_t* xs = reinterpret_cast<half_t*>(smem_raw);
    fixed_add_layer_norm_body<false>(f.acc_fixed, f.out_bias, f.res1, nullptr, nullptr, 0.f, f.n, xs, nullptr);
    __syncthreads();
    canonical_role<true>(mp0, bid - nblk_fc1, nblk_mp0, xs);
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
