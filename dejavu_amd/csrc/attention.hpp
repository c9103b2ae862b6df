// Head-sparse attention kernels for the decode step:
//   qkv_sparse_kernel     QKV projection of the active heads for the live window tokens
//   kv_cache_copy_kernel  scatter of (re)computed K / V rows into the caches
//   decode_attn_kernel    one-query attention over the fp16 KV cache, split along the sequence
//   decode_attn_combine_kernel  log-sum-exp merge of the sequence splits
//   out_proj_rows_kernel  out_proj over the active heads with the weight in (d, H, hd) layout
//
// Cache layouts (kept from the reference so the caches are interchangeable):
//   k_cache (B, H, hd/8, S, 8): for a fixed head and 8-wide slice of head_dim the S
//   positions are contiguous 16-byte packets, so a wavefront that maps lanes to
//   positions reads 1 KiB contiguous per load;  v_cache (B, H, S, hd).
#pragma once
#include "common.hpp"
#include "norm.hpp"

namespace dv {

// ---------------------------------------------------------------------------
// Y[b, t, h, j] = X[b, :] . W[t, h, j, :] + bias[t, h, j]
//   for i < nnz, h = head_idx[i], every slot s < nb with b = batch_idx[i, s] >= 0.
// X (nb, d); W (3, H, hd, d) contiguous; Y (nb, 3, H, hd).  Rows of one (t, h)
// are hd consecutive weight rows; a wavefront owns R of them at a time and
// keeps one accumulator per live slot.  Nothing is written for dead slots or
// unselected heads.  With k_cache / v_cache given, the K and V rows are also
// scattered into the caches at position (token + padding[0]).
// ---------------------------------------------------------------------------
template <int NBMAX, int R, int U>
__device__ __forceinline__ void qkv_sparse_body(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, const int* __restrict__ batch_idx, int nb, int d, int H,
    int hd, int nnz, half_t* __restrict__ Y, half_t* __restrict__ k_cache,
    half_t* __restrict__ v_cache, const int* __restrict__ padding, int S, int block_id,
    int nblocks) {
  constexpr int CH = 8 * kWave;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves_per_block = blockDim.x >> 6;
  const int groups_per_head = hd / R;  // hd % R == 0 (checked on the host)
  const int ntasks = nnz * 3 * groups_per_head;
  for (int task = block_id * waves_per_block + wave; task < ntasks;
       task += nblocks * waves_per_block) {
    const int i = task / (3 * groups_per_head);
    const int rem = task - i * 3 * groups_per_head;
    const int t = rem / groups_per_head;
    const int j0 = (rem - t * groups_per_head) * R;
    const int h = head_idx[i];
    if (h < 0 || h >= H) continue;
    int slot[NBMAX];
    bool any = false;
#pragma unroll
    for (int s = 0; s < NBMAX; ++s) {
      int b = s < nb ? batch_idx[i * nb + s] : -1;
      if (b >= nb) b = -1;
      slot[s] = b;
      any |= b >= 0;
    }
    if (!any) continue;
    const int64_t row0 = ((int64_t)t * H + h) * hd + j0;
    const half_t* wr = W + row0 * d + lane * 8;

    float acc[R][NBMAX];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int s = 0; s < NBMAX; ++s) acc[r][s] = 0.f;

    int base = 0;
    for (; base + U * CH <= d; base += U * CH) {
      half8_t w[U][R];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < R; ++r) w[u][r] = load8_stream(wr + (int64_t)r * d + base + u * CH);
#pragma unroll
      for (int s = 0; s < NBMAX; ++s) {
        if (slot[s] >= 0) {
          const half_t* xr = X + (int64_t)slot[s] * d + base + lane * 8;
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const half8_t xv = load8(xr + u * CH);
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r][s] = dot8_fast(w[u][r], xv, acc[r][s]);
          }
        }
      }
    }
    for (; base < d; base += CH) {
      if (base + lane * 8 < d) {
        half8_t w[R];
#pragma unroll
        for (int r = 0; r < R; ++r) w[r] = load8_stream(wr + (int64_t)r * d + base);
#pragma unroll
        for (int s = 0; s < NBMAX; ++s) {
          if (slot[s] >= 0) {
            const half8_t xv = load8(X + (int64_t)slot[s] * d + base + lane * 8);
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r][s] = dot8_fast(w[r], xv, acc[r][s]);
          }
        }
      }
    }
#pragma unroll
    for (int s = 0; s < NBMAX; ++s) {
      if (slot[s] >= 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          float v = butterfly_sum<kWave>(acc[r][s]);
          if (bias != nullptr) v += (float)bias[row0 + r];
          if (lane == 0) {
            const half_t hv = (half_t)v;
            Y[(int64_t)slot[s] * 3 * H * hd + row0 + r] = hv;
            // optional fused cache scatter (same arithmetic as kv_cache_copy_kernel)
            if (t != 0 && k_cache != nullptr) {
              const int dst = slot[s] + (padding ? padding[0] : 0);
              const int j = j0 + r;
              if (dst >= 0 && dst < S) {
                if (t == 1)
                  k_cache[(((int64_t)h * (hd / 8) + j / 8) * S + dst) * 8 + (j & 7)] = hv;
                else
                  v_cache[((int64_t)h * S + dst) * hd + j] = hv;
              }
            }
          }
        }
      }
    }
  }
}

template <int NBMAX, int R, int U>
__global__ __launch_bounds__(256) void qkv_sparse_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, const int* __restrict__ batch_idx, int nb, int d, int H,
    int hd, int nnz, half_t* __restrict__ Y, half_t* __restrict__ k_cache,
    half_t* __restrict__ v_cache, const int* __restrict__ padding, int S) {
  qkv_sparse_body<NBMAX, R, U>(X, W, bias, head_idx, batch_idx, nb, d, H, hd, nnz, Y, k_cache, v_cache,
                               padding, S, blockIdx.x, gridDim.x);
}

// The newest token of a back-fill window whose LayerNorm has not been applied yet: the residual
// stream row, the statistics pairs of its 64-element parts (norm.hpp) and the LayerNorm
// parameters.  A QKV workgroup normalises the row itself; workgroup 0 also stores the
// normalised row to `x_row_out` (the token's row of the window buffer).
struct QkvLnArgs {
  const half_t* R1;
  const float2* parts;
  const half_t* gamma;
  const half_t* beta;
  float eps;
  half_t* x_row_out;
  int token;  // index of the token in the window (its Y row and cache position offset)
};

// QKV of the active heads for that one token (every active head computes it: the first position
// of a window, where nothing is back-filled).  The whole workgroup normalises the row into LDS
// (xs: d halves) from the precomputed statistics, then every wavefront runs the dot products of
// qkv_sparse_body<1, R, U> (same products in the same order: the same bits) with x from LDS.
// NP: statistics pairs per lane (d <= 4096 * NP).
template <int R, int U, int NP>
__device__ __forceinline__ void qkv_ln_token_body(
    const QkvLnArgs& ln, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, int d, int H, int hd, int nnz, half_t* __restrict__ Y,
    half_t* __restrict__ k_cache, half_t* __restrict__ v_cache, const int* __restrict__ padding, int S,
    half_t* xs, int block_id, int nblocks) {
  constexpr int CH = 8 * kWave;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves_per_block = blockDim.x >> 6;
  const int groups_per_head = hd / R;
  const int ntasks = nnz * 3 * groups_per_head;
  const int task0 = block_id * waves_per_block + wave;

  // Requests in this order: the statistics pairs and the row (cache hits), then the first batch
  // of this wavefront's weights.  The load counter retires in order, so the row can be normalised
  // while the weights are still on their way.
  const int nvec = d / 8;
  const int P = (d + kLnPart - 1) / kLnPart;
  const LnParts<NP> lp = ln_load_parts<NP>(ln.parts, P);
  constexpr int VB = 3;  // vectors per thread and round; one round when d <= 8 * VB * blockDim.x
  half8_t xr[VB], xg[VB], xb[VB];
#pragma unroll
  for (int j = 0; j < VB; ++j) {
    const int i = j * blockDim.x + threadIdx.x;
    if (i < nvec) {
      xr[j] = load8(ln.R1 + i * 8);
      xg[j] = load8(ln.gamma + i * 8);
      xb[j] = load8(ln.beta + i * 8);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // first task's first batch (a full batch exists when d >= U * CH; shorter rows start in the loop)
  constexpr int PRE = U / 2;  // chunks of the first batch requested this early (registers are short here)
  half8_t w0[PRE][R];
  bool have_w0 = false;
  {
    const int i = task0 < ntasks ? task0 / (3 * groups_per_head) : 0;
    const int h = task0 < ntasks ? head_idx[i] : -1;
    if (h >= 0 && h < H && U * CH <= d) {
      const int rem = task0 - i * 3 * groups_per_head;
      const int t = rem / groups_per_head;
      const half_t* wr = W + (((int64_t)t * H + h) * hd + (rem - t * groups_per_head) * R) * d + lane * 8;
#pragma unroll
      for (int u = 0; u < PRE; ++u)
#pragma unroll
        for (int r = 0; r < R; ++r) w0[u][r] = load8_stream(wr + (int64_t)r * d + u * CH);
      have_w0 = true;
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  const LnStats st = ln_combine_loaded(lp, P, d, ln.eps);
#pragma unroll
  for (int j = 0; j < VB; ++j) {
    const int i = j * blockDim.x + threadIdx.x;
    if (i < nvec) {
      const half8_t o = ln_apply(xr[j], xg[j], xb[j], st);
      store8(xs + i * 8, o);
      if (block_id == 0) store8(ln.x_row_out + i * 8, o);
    }
  }
  for (int i = VB * blockDim.x + threadIdx.x; i < nvec; i += blockDim.x) {  // longer rows
    const half8_t o = ln_apply(load8(ln.R1 + i * 8), load8(ln.gamma + i * 8), load8(ln.beta + i * 8), st);
    store8(xs + i * 8, o);
    if (block_id == 0) store8(ln.x_row_out + i * 8, o);
  }
  __syncthreads();

  for (int task = task0; task < ntasks; task += nblocks * waves_per_block) {
    const int i = task / (3 * groups_per_head);
    const int rem = task - i * 3 * groups_per_head;
    const int t = rem / groups_per_head;
    const int j0 = (rem - t * groups_per_head) * R;
    const int h = head_idx[i];
    if (h < 0 || h >= H) continue;
    const int64_t row0 = ((int64_t)t * H + h) * hd + j0;
    const half_t* wr = W + row0 * d + lane * 8;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    int base = 0;
    for (; base + U * CH <= d; base += U * CH) {
      half8_t w[U][R];
      if (have_w0) {  // part of the batch was requested before the row was normalised
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int r = 0; r < R; ++r)
            w[u][r] = u < PRE ? w0[u < PRE ? u : 0][r] : load8_stream(wr + (int64_t)r * d + base + u * CH);
        have_w0 = false;
      } else {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int r = 0; r < R; ++r) w[u][r] = load8_stream(wr + (int64_t)r * d + base + u * CH);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const half8_t xv = load8(xs + base + u * CH + lane * 8);
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = dot8_fast(w[u][r], xv, acc[r]);
      }
    }
    for (; base < d; base += CH) {
      if (base + lane * 8 < d) {
        half8_t w[R];
#pragma unroll
        for (int r = 0; r < R; ++r) w[r] = load8_stream(wr + (int64_t)r * d + base);
        const half8_t xv = load8(xs + base + lane * 8);
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = dot8_fast(w[r], xv, acc[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float v = butterfly_sum<kWave>(acc[r]);
      if (bias != nullptr) v += (float)bias[row0 + r];
      if (lane == 0) {
        const half_t hv = (half_t)v;
        Y[(int64_t)ln.token * 3 * H * hd + row0 + r] = hv;
        if (t != 0 && k_cache != nullptr) {
          const int dst = ln.token + (padding ? padding[0] : 0);
          const int j = j0 + r;
          if (dst >= 0 && dst < S) {
            if (t == 1)
              k_cache[(((int64_t)h * (hd / 8) + j / 8) * S + dst) * 8 + (j & 7)] = hv;
            else
              v_cache[((int64_t)h * S + dst) * hd + j] = hv;
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// For i < nnz, h = head_idx[i], every slot with s = seq_idx[i, slot] >= 0:
//   k_cache[0, h, dp, s + pad, p] = K[s, h, dp*8 + p]      (if k_cache != null)
//   v_cache[0, h, s + pad, :]     = V[s, h, :]             (if v_cache != null)
// K / V are (nsrc, H, hd) views with row stride `ld_src` elements (rows of the
// (nb, 3, H, hd) projection output).  `padding` is a device int32 (or null = 0).
// One workgroup of hd threads per (slot, head).
// ---------------------------------------------------------------------------
__global__ void kv_cache_copy_kernel(const half_t* __restrict__ K, const half_t* __restrict__ V,
                                     int64_t ld_src, int nsrc, half_t* __restrict__ k_cache,
                                     half_t* __restrict__ v_cache, const int* __restrict__ head_idx,
                                     const int* __restrict__ seq_idx, int nslots,
                                     const int* __restrict__ padding, int H, int hd, int S) {
  const int i = blockIdx.x;
  const int slot = blockIdx.y;
  const int j = threadIdx.x;
  const int h = head_idx[i];
  const int s = seq_idx[i * nslots + slot];
  if (h < 0 || h >= H || s < 0 || s >= nsrc || j >= hd) return;
  const int dst = s + (padding ? padding[0] : 0);
  if (dst < 0 || dst >= S) return;
  const int64_t src = (int64_t)s * ld_src + (int64_t)h * hd + j;
  if (k_cache) k_cache[(((int64_t)h * (hd / 8) + j / 8) * S + dst) * 8 + (j & 7)] = K[src];
  if (v_cache) v_cache[((int64_t)h * S + dst) * hd + j] = V[src];
}

// One decode step of the skipped-head back-fill window.
//   x_cache[counter, :] = x
//   flush != 0: for every head h and s < 16: batch_idx[h, s] = s, tracker[h, s] = s
//   flush == 0: (counter == 0: the tracker is first re-initialised, tracker[h, s] = s;
//                a window always starts from that state)
//               for i < nnz, h = head_idx[i], s <= counter:
//                 batch_idx[i, s] = tracker[h, s];  tracker[h, s] = -1
// tracker is (H, 16) int32: tracker[h, s] == s while token s of the window has no
// K/V for head h, -1 once it has.  Heads in head_idx are distinct.  Workgroup 0
// owns the tracker (two phases separated by a barrier); all workgroups copy x.
// Tracker part, executed by ONE workgroup (any size).
__device__ __forceinline__ void window_tracker_step(int* __restrict__ tracker,
                                                    const int* __restrict__ head_idx, int nnz, int H,
                                                    int counter, int flush,
                                                    int* __restrict__ batch_idx) {
  if (flush) {
    for (int o = threadIdx.x; o < H * 16; o += blockDim.x) {
      tracker[o] = o & 15;
      batch_idx[o] = o & 15;
    }
    return;
  }
  if (counter == 0) {
    for (int o = threadIdx.x; o < H * 16; o += blockDim.x) tracker[o] = o & 15;
    __syncthreads();
  }
  const int nb = counter + 1;
  for (int o = threadIdx.x; o < nnz * nb; o += blockDim.x) {
    const int i = o / nb, s = o - i * nb;
    const int h = head_idx[i];
    if (h < 0 || h >= H) {
      batch_idx[o] = -1;
    } else {
      batch_idx[o] = tracker[h * 16 + s];
      tracker[h * 16 + s] = -1;
    }
  }
}

__global__ __launch_bounds__(256) void window_step_kernel(
    const half_t* __restrict__ x, half_t* __restrict__ x_cache, int d, int* __restrict__ tracker,
    const int* __restrict__ head_idx, int nnz, int H, int counter, int flush,
    int* __restrict__ batch_idx) {
  const int tid = blockIdx.x * blockDim.x + threadIdx.x;
  const int nthreads = gridDim.x * blockDim.x;
  for (int j = tid; j < d; j += nthreads) x_cache[(int64_t)counter * d + j] = x[j];
  if (blockIdx.x != 0) return;
  window_tracker_step(tracker, head_idx, nnz, H, counter, flush, batch_idx);
}

// add + LayerNorm of `rows` rows (one workgroup each; a second copy of the normalised rows goes to
// the window buffer's row of this step) and, in one more workgroup, the tracker step of the same
// window position: add_layer_norm_kernel and window_step_kernel in one launch.
template <int THREADS, int NV>
__global__ __launch_bounds__(THREADS) void add_layer_norm_window_kernel(
    const half_t* __restrict__ Hin, const half_t* __restrict__ R, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, float eps, int d, half_t* __restrict__ Y, half_t* __restrict__ Rout,
    half_t* __restrict__ x_cache_row, int rows, int* __restrict__ tracker, const int* __restrict__ head_idx,
    int nnz, int H, int counter, int flush, int* __restrict__ batch_idx) {
  if ((int)blockIdx.x == rows) {
    window_tracker_step(tracker, head_idx, nnz, H, counter, flush, batch_idx);
    return;
  }
  add_layer_norm_body<THREADS, NV>(Hin, R, gamma, beta, eps, d, Y, Rout, x_cache_row, blockIdx.x);
}

// The same for rows that arrive as the fp32 partial sums of a split product (the fc2 of the block
// before: its reduction, the residual add, LayerNorm 1 and the window step are one launch).
// tracker == nullptr: no window step (launch `rows` workgroups), x_cache_row may be nullptr.
template <int THREADS, int NV>
__global__ __launch_bounds__(THREADS) void reduce_add_layer_norm_window_kernel(
    const float* __restrict__ partial, const half_t* __restrict__ bias, int G, const half_t* __restrict__ R,
    const half_t* __restrict__ gamma, const half_t* __restrict__ beta, float eps, int d, half_t* __restrict__ Y,
    half_t* __restrict__ Rout, half_t* __restrict__ x_cache_row, int rows, int* __restrict__ tracker,
    const int* __restrict__ head_idx, int nnz, int H, int counter, int flush, int* __restrict__ batch_idx) {
  if ((int)blockIdx.x == rows) {
    window_tracker_step(tracker, head_idx, nnz, H, counter, flush, batch_idx);
    return;
  }
  add_layer_norm_src_body<THREADS, NV, LnNoHook, LnRowFromPartials>(
      LnRowFromPartials{partial, bias, G, d, (int64_t)rows * d}, R, gamma, beta, eps, d, Y, Rout, x_cache_row,
      blockIdx.x);
}

// Appends the newest token: for every batch row b and head (all, or head_idx):
//   k_cache[b, h, :, pos_b, :] = K[b, h, :],  v_cache[b, h, pos_b, :] = V[b, h, :]
// with pos_b = lengths[b] if lengths else pos.  K / V: (B, H, hd) with batch
// stride ld_src.  Grid (heads, B), hd threads.
__global__ void kv_append_kernel(const half_t* __restrict__ K, const half_t* __restrict__ V,
                                 int64_t ld_src, half_t* __restrict__ k_cache,
                                 half_t* __restrict__ v_cache, const int* __restrict__ head_idx,
                                 const int* __restrict__ lengths, int pos, int H, int hd, int S) {
  const int h = head_idx ? head_idx[blockIdx.x] : (int)blockIdx.x;
  const int b = blockIdx.y;
  const int j = threadIdx.x;
  const int p = lengths ? lengths[b] : pos;
  if (h < 0 || h >= H || p < 0 || p >= S || j >= hd) return;
  const int64_t src = (int64_t)b * ld_src + (int64_t)h * hd + j;
  const int64_t bh = (int64_t)b * H + h;
  k_cache[((bh * (hd / 8) + j / 8) * S + p) * 8 + (j & 7)] = K[src];
  v_cache[(bh * S + p) * hd + j] = V[src];
}

// ---------------------------------------------------------------------------
// One-query attention.  A workgroup of WAVES wavefronts handles WAVES*64 cached
// positions of one (head, batch row); inside a wavefront lanes map to positions
// for q.K (each lane reads its position's hd/8 packets) and to (row, 8-wide
// slice) for p.V.  All K and V loads of a wavefront are issued before any
// arithmetic.  The wavefronts are merged in LDS and the workgroup writes one
// un-normalised partial  part[(b, i, split)] = { max, sum, o[hd] }  (fp32).
// n_len = number of cached positions to attend (lengths[b] + 1 if lengths).
// ---------------------------------------------------------------------------
template <int HD, int WAVES>
__device__ __forceinline__ void decode_attn_body(
    const half_t* __restrict__ Q, int64_t ldq, const half_t* __restrict__ k_cache,
    const half_t* __restrict__ v_cache, const int* __restrict__ head_idx,
    const int* __restrict__ lengths, int n_len, int H, int S, float scale, int nsplit,
    float* __restrict__ part, int split, int i, int b, int nheads) {
  constexpr int PK = HD / 8;        // 16-byte packets per position / lanes per V row
  constexpr int RPI = kWave / PK;   // V rows per load instruction
  constexpr int VIT = kWave / RPI;  // V load instructions per wavefront (= PK)
  __shared__ float s_m[WAVES], s_l[WAVES];
  __shared__ float s_o[WAVES][HD];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int h = head_idx ? head_idx[i] : i;
  int len = lengths ? lengths[b] + 1 : n_len;
  if (len > S) len = S;  // a device-side length can never address past the cache
  float* out = part + (((int64_t)b * nheads + i) * nsplit + split) * (HD + 2);
  const bool head_ok = h >= 0 && h < H;
  const int p0 = (split * WAVES + wave) * kWave;
  float m = -INFINITY, l = 0.f;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  const int grp = lane / PK, sub = lane % PK;
  if (head_ok && p0 < len) {
    const int64_t bh = (int64_t)b * H + h;
    const int pos = p0 + lane;
    const bool pos_ok = pos < len;
    const int pos_c = pos_ok ? pos : len - 1;  // clamp: always a valid address
    half8_t kp[PK];
    const half_t* kbase = k_cache + (bh * PK * S + pos_c) * 8;
#pragma unroll
    for (int dp = 0; dp < PK; ++dp) kp[dp] = load8_stream(kbase + (int64_t)dp * S * 8);
    half8_t vv[VIT];
#pragma unroll
    for (int it = 0; it < VIT; ++it) {
      int row = p0 + it * RPI + grp;
      if (row >= len) row = len - 1;
      vv[it] = load8_stream(v_cache + (bh * S + row) * HD + sub * 8);
    }
    const half_t* q = Q + (int64_t)b * ldq + (int64_t)h * HD;
    float sc = 0.f;
#pragma unroll
    for (int dp = 0; dp < PK; ++dp) sc = dot8_fast(kp[dp], load8(q + dp * 8), sc);
    sc = pos_ok ? sc * scale : -INFINITY;
    m = butterfly_max<kWave>(sc);
    const float p = pos_ok ? __expf(sc - m) : 0.f;
    l = butterfly_sum<kWave>(p);
#pragma unroll
    for (int it = 0; it < VIT; ++it) {
      const float pr = __shfl(p, it * RPI + grp, kWave);  // 0 for positions >= len
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(pr, (float)vv[it][e], acc[e]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
#pragma unroll
      for (int off = PK; off < kWave; off <<= 1) acc[e] += __shfl_xor(acc[e], off, kWave);
    }
  }
  if (lane == 0) {
    s_m[wave] = m;
    s_l[wave] = l;
  }
  if (grp == 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) s_o[wave][sub * 8 + e] = acc[e];
  }
  __syncthreads();
  // merge the wavefronts (empty ones carry max = -inf, sum = 0)
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) M = fmaxf(M, s_m[w]);
  for (int j = threadIdx.x; j < HD + 2; j += WAVES * kWave) {
    float v = 0.f;
    if (j == 0) {
      v = M;
    } else {
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        const float sw = s_m[w] == -INFINITY ? 0.f : __expf(s_m[w] - M);
        v += sw * (j == 1 ? s_l[w] : s_o[w][j - 2]);
      }
    }
    out[j] = v;
  }
}

template <int HD, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void decode_attn_kernel(
    const half_t* __restrict__ Q, int64_t ldq, const half_t* __restrict__ k_cache,
    const half_t* __restrict__ v_cache, const int* __restrict__ head_idx,
    const int* __restrict__ lengths, int n_len, int H, int S, float scale, int nsplit,
    float* __restrict__ part) {
  decode_attn_body<HD, WAVES>(Q, ldq, k_cache, v_cache, head_idx, lengths, n_len, H, S, scale, nsplit, part,
                              blockIdx.x, blockIdx.y, blockIdx.z, gridDim.y);
}

// ---------------------------------------------------------------------------
// One-query attention for MANY (sequence, head) pairs (a batch of sequences: B * heads pairs fill
// the device by themselves): ONE workgroup of sixteen wavefronts per pair walks all cached
// positions, 1024 per turn (a wavefront its 64, as in decode_attn_body: lanes map to positions for
// q.K and to (row, 8-wide slice) for p.V, all K and V loads of a turn issued before its
// arithmetic), keeps a running maximum / sum / un-normalised output per wavefront (online softmax:
// the output is rescaled by exp(old max - new max), a wavefront-uniform factor, so the sums over the
// V rows stay spread over the lanes until the end), merges the sixteen wavefronts in LDS and writes
// the normalised fp16 result.  No partial results in memory and no combine launch.
// Grid (heads, B).  lengths as in decode_attn_body.
// ---------------------------------------------------------------------------
constexpr int kAttnRowWaves = 16;

template <int HD>
__global__ __launch_bounds__(kAttnRowWaves * 64) void decode_attn_rows_kernel(
    const half_t* __restrict__ Q, int64_t ldq, const half_t* __restrict__ k_cache,
    const half_t* __restrict__ v_cache, const int* __restrict__ head_idx, const int* __restrict__ lengths,
    int n_len, int H, int S, float scale, half_t* __restrict__ out, int64_t ldo) {
  constexpr int WAVES = kAttnRowWaves;
  constexpr int PK = HD / 8;        // 16-byte packets per position / lanes per V row
  constexpr int RPI = kWave / PK;   // V rows per load instruction
  constexpr int VIT = kWave / RPI;  // V load instructions per wavefront and turn (= PK)
  __shared__ float s_m[WAVES], s_l[WAVES];
  __shared__ float s_o[WAVES][HD];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int i = blockIdx.x, b = blockIdx.y;
  const int h = head_idx ? head_idx[i] : i;
  if (h < 0 || h >= H) return;  // uniform over the workgroup
  int len = lengths ? lengths[b] + 1 : n_len;
  if (len > S) len = S;  // a device-side length can never address past the cache
  const int grp = lane / PK, sub = lane % PK;
  const int64_t bh = (int64_t)b * H + h;
  const half_t* q = Q + (int64_t)b * ldq + (int64_t)h * HD;
  half8_t qv[PK];
#pragma unroll
  for (int dp = 0; dp < PK; ++dp) qv[dp] = load8(q + dp * 8);
  float m = -INFINITY, l = 0.f;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  for (int p0 = wave * kWave; p0 < len; p0 += WAVES * kWave) {  // uniform over the wavefront
    const int pos = p0 + lane;
    const bool pos_ok = pos < len;
    const int pos_c = pos_ok ? pos : len - 1;  // clamp: always a valid address
    half8_t kp[PK];
    const half_t* kbase = k_cache + (bh * PK * S + pos_c) * 8;
#pragma unroll
    for (int dp = 0; dp < PK; ++dp) kp[dp] = load8_stream(kbase + (int64_t)dp * S * 8);
    half8_t vv[VIT];
#pragma unroll
    for (int it = 0; it < VIT; ++it) {
      int row = p0 + it * RPI + grp;
      if (row >= len) row = len - 1;
      vv[it] = load8_stream(v_cache + (bh * S + row) * HD + sub * 8);
    }
    float sc = 0.f;
#pragma unroll
    for (int dp = 0; dp < PK; ++dp) sc = dot8_fast(kp[dp], qv[dp], sc);
    sc = pos_ok ? sc * scale : -INFINITY;
    const float m_new = fmaxf(m, butterfly_max<kWave>(sc));  // finite: position p0 is inside the length
    const float rescale = m == -INFINITY ? 0.f : __expf(m - m_new);
    const float p = pos_ok ? __expf(sc - m_new) : 0.f;
    l = l * rescale + butterfly_sum<kWave>(p);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= rescale;
#pragma unroll
    for (int it = 0; it < VIT; ++it) {
      const float pr = __shfl(p, it * RPI + grp, kWave);  // 0 for positions >= len
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(pr, (float)vv[it][e], acc[e]);
    }
    m = m_new;
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
#pragma unroll
    for (int off = PK; off < kWave; off <<= 1) acc[e] += __shfl_xor(acc[e], off, kWave);
  }
  if (lane == 0) {
    s_m[wave] = m;
    s_l[wave] = l;
  }
  if (grp == 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) s_o[wave][sub * 8 + e] = acc[e];
  }
  __syncthreads();
  // merge the wavefronts (those without a position carry max = -inf, sum = 0) and normalise
  if (threadIdx.x < HD) {
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) M = fmaxf(M, s_m[w]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float sw = s_m[w] == -INFINITY ? 0.f : __expf(s_m[w] - M);
      den += sw * s_l[w];
      num += sw * s_o[w][threadIdx.x];
    }
    out[(int64_t)b * ldo + (int64_t)h * HD + threadIdx.x] = (half_t)(num / den);
  }
}

// out[b, h, :] = sum_s o_s * exp(m_s - m) / sum_s l_s * exp(m_s - m).  Grid (heads, B), HD threads.
template <int HD>
__global__ __launch_bounds__(HD) void decode_attn_combine_kernel(
    const float* __restrict__ part, const int* __restrict__ head_idx, int H, int nsplit,
    half_t* __restrict__ out, int64_t ldo) {
  const int i = blockIdx.x;
  const int b = blockIdx.y;
  const int j = threadIdx.x;
  const int h = head_idx ? head_idx[i] : i;
  if (h < 0 || h >= H) return;
  const float* p = part + ((int64_t)b * gridDim.x + i) * nsplit * (HD + 2);
  float m = -INFINITY, num = 0.f, den = 0.f;
  for (int s0 = 0; s0 < nsplit; s0 += 8) {  // online merge, 8 splits' loads in flight
    float ms[8], ls[8], os[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const bool ok = s0 + q < nsplit;
      const float* ps = p + (int64_t)(ok ? s0 + q : s0) * (HD + 2);
      ms[q] = ok ? ps[0] : -INFINITY;
      ls[q] = ps[1];
      os[q] = ps[2 + j];
    }
    float mc = m;
#pragma unroll
    for (int q = 0; q < 8; ++q) mc = fmaxf(mc, ms[q]);
    if (mc == -INFINITY) continue;
    const float rescale = m == -INFINITY ? 0.f : __expf(m - mc);
    num *= rescale;
    den *= rescale;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const float w = ms[q] == -INFINITY ? 0.f : __expf(ms[q] - mc);
      den += w * ls[q];
      num += w * os[q];
    }
    m = mc;
  }
  out[(int64_t)b * ldo + (int64_t)h * HD + j] = (half_t)(num / den);
}

// ---------------------------------------------------------------------------
// Y[b, n] = sum_{i < nnz} X[b, h_i, :] . W[n, h_i, :] + bias[n] with W in the
// (d, H, hd) layout of out_proj.weight: every output row gathers nnz segments
// of hd contiguous values.  hd/8 lanes cover a segment, so a wavefront load
// touches 64/(hd/8) heads; R output rows share the activation loads.
// ---------------------------------------------------------------------------
template <int B, int R, int HD>
__global__ __launch_bounds__(256) void out_proj_rows_kernel(
    const half_t* __restrict__ X, const half_t* __restrict__ W, const half_t* __restrict__ bias,
    const int* __restrict__ head_idx, int nnz, int H, int N, half_t* __restrict__ Y) {
  constexpr int PK = HD / 8;
  constexpr int HPI = kWave / PK;  // heads per load instruction
  const int lane = threadIdx.x & 63;
  const int grp = lane / PK, sub = lane % PK;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves_per_block = blockDim.x >> 6;
  const int ntasks = (N + R - 1) / R;
  for (int task = blockIdx.x * waves_per_block + wave; task < ntasks;
       task += gridDim.x * waves_per_block) {
    const int n0 = task * R;
    float acc[R][B];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int b = 0; b < B; ++b) acc[r][b] = 0.f;
    for (int i0 = 0; i0 < nnz; i0 += HPI) {
      const int i = i0 + grp;
      int h = i < nnz ? head_idx[i] : -1;
      const bool ok = h >= 0 && h < H;
      if (!ok) h = 0;
      const int64_t seg = (int64_t)h * HD + sub * 8;
      half8_t w[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = n0 + r < N ? n0 + r : N - 1;
        w[r] = ok ? load8_stream(W + (int64_t)n * H * HD + seg) : zero8();
      }
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const half8_t xv = load8(X + (int64_t)b * H * HD + seg);
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r][b] = dot8_fast(w[r], xv, acc[r][b]);
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const float v = butterfly_sum<kWave>(acc[r][b]);
        const int n = n0 + r;
        if (lane == 0 && n < N) Y[(int64_t)b * N + n] = (half_t)(v + (bias ? (float)bias[n] : 0.f));
      }
  }
}

// ---------------------------------------------------------------------------
// out_proj in the (d, H, hd) layout straight from the un-normalised attention
// partials { max, sum, o[HD] } of decode_attn_kernel (batch 1):
//   ctx[i, :]  = fp16(merge over the splits of head_idx[i])     (arithmetic of decode_attn_combine_kernel)
//   Y[n]       = fp16(sum_i ctx[i, :] . W[n, head_idx[i], :] + bias[n])  (lane order of out_proj_rows_kernel)
//   Rout[n]    = fp16(Y[n] + Rin[n])                            (optional: the residual stream advanced)
// Every output row is complete inside one wavefront, so there is no cross-workgroup reduction
// and no second launch.  A workgroup first merges all partials into LDS (ctx: nnz * HD fp16,
// then nnz segment offsets); the weight loads of its first head group are already in flight
// by then.  A wavefront owns R rows: per head group (64 / (HD/8) heads) it issues R 16-byte
// loads per lane, one group ahead of the multiply-adds.
// Dynamic LDS: nnz * HD * 2 + nnz * 4 bytes.
// ---------------------------------------------------------------------------
template <int HD>
__device__ __forceinline__ half8_t attn_merge8(const float* __restrict__ p, int nsplit, int j0) {
  float m = -INFINITY, den = 0.f;
  float num[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) num[e] = 0.f;
  for (int s0 = 0; s0 < nsplit; s0 += 8) {  // online merge, 8 splits' loads in flight
    float ms[8], ls[8];
    float2 os[8][4];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const bool ok = s0 + q < nsplit;
      const float* ps = p + (int64_t)(ok ? s0 + q : s0) * (HD + 2);
      ms[q] = ok ? ps[0] : -INFINITY;
      ls[q] = ps[1];
#pragma unroll
      for (int v = 0; v < 4; ++v) os[q][v] = *reinterpret_cast<const float2*>(ps + 2 + j0 + 2 * v);
    }
    float mc = m;
#pragma unroll
    for (int q = 0; q < 8; ++q) mc = fmaxf(mc, ms[q]);
    if (mc == -INFINITY) continue;
    const float rescale = m == -INFINITY ? 0.f : __expf(m - mc);
    den *= rescale;
#pragma unroll
    for (int e = 0; e < 8; ++e) num[e] *= rescale;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const float w = ms[q] == -INFINITY ? 0.f : __expf(ms[q] - mc);
      den += w * ls[q];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        num[2 * v] += w * os[q][v].x;
        num[2 * v + 1] += w * os[q][v].y;
      }
    }
    m = mc;
  }
  half8_t out;
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (half_t)(num[e] / den);
  return out;
}

template <int R, int HD>
__device__ __forceinline__ void out_proj_rows_attn_body(
    const float* __restrict__ attn_part, int nsplit, const half_t* __restrict__ W,
    const half_t* __restrict__ bias, const int* __restrict__ head_idx, int nnz, int H, int N,
    half_t* __restrict__ Y, const half_t* __restrict__ Rin, half_t* __restrict__ Rout,
    unsigned char* __restrict__ smem, int block_id, int nblocks) {
  constexpr int PK = HD / 8;
  constexpr int HPI = kWave / PK;  // heads per load instruction
  half_t* ctx = reinterpret_cast<half_t*>(smem);
  int* s_seg = reinterpret_cast<int*>(smem + (size_t)nnz * HD * sizeof(half_t));
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int grp = lane / PK, sub = lane % PK;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int waves = blockDim.x >> 6;
  const int ntasks = (N + R - 1) / R;
  const int niter = (nnz + HPI - 1) / HPI;
  const int units = nnz * PK;
  const int64_t ldw = (int64_t)H * HD;

  // head ids this thread needs before LDS is filled: its merge unit and its first head group
  const int hu = tid < units ? head_idx[tid / PK] : -1;
  const int hg = grp < nnz ? head_idx[grp] : -1;
  // seg < 0 (dead lane): the lane reads one cache-resident address and its activations are zero
  auto load_group = [&](half8_t (&dst)[R], int n0, int seg) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = n0 + r < N ? n0 + r : N - 1;
      dst[r] = load8_stream(W + (seg < 0 ? (int64_t)0 : (int64_t)n * ldw + seg) + sub * 8);
    }
  };
  int task = block_id * waves + wave;
  half8_t w[R];
  if (task < ntasks) load_group(w, task * R, (hg >= 0 && hg < H) ? hg * HD : -1);  // in flight during the merge

  // merge the attention partials into LDS
  for (int u = tid; u < units; u += blockDim.x) {
    const int i = u / PK, j0 = (u - i * PK) * 8;
    const int h = u == tid ? hu : head_idx[i];
    half8_t c = zero8();
    if (h >= 0 && h < H) c = attn_merge8<HD>(attn_part + (int64_t)i * nsplit * (HD + 2), nsplit, j0);
    *reinterpret_cast<half8_t*>(ctx + (size_t)i * HD + j0) = c;
  }
  for (int i = tid; i < nnz; i += blockDim.x) {
    const int h = head_idx[i];
    s_seg[i] = (h >= 0 && h < H) ? h * HD : -1;
  }
  __syncthreads();

  for (; task < ntasks; task += nblocks * waves) {
    const int n0 = task * R;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    for (int it = 0; it < niter; ++it) {
      // next head group (after the last one: the first group of this wavefront's next task)
      half8_t wn[R];
      int itn = it + 1, nn = n0;
      if (itn == niter) {
        itn = 0;
        nn = (task + nblocks * waves) * R;
      }
      if (nn < N) {
        const int in = itn * HPI + grp;
        load_group(wn, nn, in < nnz ? s_seg[in] : -1);
      }
      const int i = it * HPI + grp;
      const bool live = i < nnz && s_seg[i < nnz ? i : 0] >= 0;
      half8_t x = zero8();
      if (live) x = *reinterpret_cast<const half8_t*>(ctx + (size_t)i * HD + sub * 8);
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] = dot8_fast(w[r], x, acc[r]);
#pragma unroll
      for (int r = 0; r < R; ++r) w[r] = wn[r];
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float v = butterfly_sum<kWave>(acc[r]);
      const int n = n0 + r;
      if (lane == r && n < N) {
        const half_t y = (half_t)(v + (bias ? (float)bias[n] : 0.f));
        Y[n] = y;
        if (Rout != nullptr) Rout[n] = (half_t)((float)y + (float)Rin[n]);
      }
    }
  }
}

template <int R, int HD>
__global__ __launch_bounds__(512) void out_proj_rows_attn_kernel(
    const float* __restrict__ attn_part, int nsplit, const half_t* __restrict__ W,
    const half_t* __restrict__ bias, const int* __restrict__ head_idx, int nnz, int H, int N,
    half_t* __restrict__ Y, const half_t* __restrict__ Rin, half_t* __restrict__ Rout) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  out_proj_rows_attn_body<R, HD>(attn_part, nsplit, W, bias, head_idx, nnz, H, N, Y, Rin, Rout, smem_raw,
                                 blockIdx.x, gridDim.x);
}

}  // namespace dv
