// Exact top-k index selection over fp16 logits with ties going to the lower
// index.  One workgroup keeps every key in registers, finds the k-th largest
// 16-bit key by a 16-step bitwise search (wavefront ballot counts + an LDS
// combine), then emits the selected indices in ascending order with one
// workgroup prefix sum.  No atomics, so the result is deterministic.
#pragma once
#include "common.hpp"

namespace dv {

// Monotone fp16 -> u16 key: larger value <=> larger key, -0 == +0, NaN on top.
__device__ __forceinline__ unsigned topk_key(half_t h) {
  unsigned bits = (unsigned)__builtin_bit_cast(unsigned short, h);
  if (bits == 0x8000u) bits = 0u;
  unsigned key = (bits & 0x8000u) ? ((~bits) & 0xFFFFu) : (bits | 0x8000u);
  if ((bits & 0x7FFFu) > 0x7C00u) key = 0xFFFFu;
  return key;
}

// logits: (B, n) fp16; the score of column j is the maximum key over the B rows.
// Thread t owns columns [t*ITEMS, (t+1)*ITEMS); requires n <= THREADS*ITEMS
// and 0 <= k <= n.  VEC reads 8 logits per 128-bit load and needs n % 8 == 0.  idx_out receives k indices (int32 or int64) ascending.
template <int THREADS, int ITEMS, bool VEC>
__global__ __launch_bounds__(THREADS) void topk_kernel(const half_t* __restrict__ logits, int B,
                                                       int n, int k, void* __restrict__ idx_out,
                                                       int idx_bytes) {
  constexpr int WAVES = THREADS / kWave;
  __shared__ unsigned s_cnt[2][WAVES];
  __shared__ unsigned s_gt[WAVES];
  __shared__ unsigned s_eq[WAVES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int base = tid * ITEMS;

  // two 16-bit keys per register: item 2j in the low half, 2j+1 in the high half
  unsigned key2[ITEMS / 2];
#pragma unroll
  for (int i = 0; i < ITEMS / 2; ++i) key2[i] = 0u;  // padding never reaches a real key
  for (int b = 0; b < B; ++b) {
    const half_t* row = logits + (int64_t)b * n;
    if (VEC) {
      // all loads of a row are issued back to back; out-of-range groups read
      // the (valid) start of the row and are masked afterwards
      half8_t v[ITEMS / 8];
#pragma unroll
      for (int i = 0; i < ITEMS / 8; ++i) {
        const int off = base + i * 8;
        v[i] = load8(row + (off < n ? off : 0));
      }
#pragma unroll
      for (int i = 0; i < ITEMS / 8; ++i) {
        const bool in = base + i * 8 < n;
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const unsigned lo = in ? topk_key(v[i][e]) : 0u;
          const unsigned hi = in ? topk_key(v[i][e + 1]) : 0u;
          const unsigned old = key2[(i * 8 + e) / 2];
          const unsigned olo = old & 0xFFFFu, ohi = old >> 16;
          key2[(i * 8 + e) / 2] = (lo > olo ? lo : olo) | ((hi > ohi ? hi : ohi) << 16);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < ITEMS; i += 2) {
        const unsigned lo = base + i < n ? topk_key(row[base + i]) : 0u;
        const unsigned hi = base + i + 1 < n ? topk_key(row[base + i + 1]) : 0u;
        const unsigned old = key2[i / 2];
        const unsigned olo = old & 0xFFFFu, ohi = old >> 16;
        key2[i / 2] = (lo > olo ? lo : olo) | ((hi > ohi ? hi : ohi) << 16);
      }
    }
  }

  // largest T with count(key >= T) >= k.  Per thread the count is kept as two
  // packed 16-bit counters: [key >= cand] = min(sat_sub(key, cand - 1), 1).
  unsigned T = 0u;
  for (int bit = 15; bit >= 0; --bit) {
    const unsigned cand = T | (1u << bit);
    const unsigned cm1 = (cand - 1u) * 0x00010001u;  // cand - 1 in both halves
    const unsigned one = 0x00010001u;
    unsigned acc2 = 0u;
#pragma unroll
    for (int i = 0; i < ITEMS / 2; ++i) {
      // written as instructions: the compiler otherwise expands the packed
      // saturating form into per-half compares and selects
      unsigned t;
      asm volatile("v_pk_sub_u16 %0, %1, %2 clamp" : "=v"(t) : "v"(key2[i]), "v"(cm1));
      asm volatile("v_pk_min_u16 %0, %1, %2" : "=v"(t) : "v"(t), "v"(one));
      asm volatile("v_pk_add_u16 %0, %1, %2" : "=v"(acc2) : "v"(acc2), "v"(t));
    }
    unsigned c = (acc2 & 0xFFFFu) + (acc2 >> 16);
#pragma unroll
    for (int off = kWave / 2; off >= 1; off >>= 1) c += __shfl_xor(c, off, kWave);
    const int buf = bit & 1;
    if (lane == 0) s_cnt[buf][wave] = c;
    __syncthreads();
    unsigned total = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) total += s_cnt[buf][w];
    if (total >= (unsigned)k) T = cand;
  }

  // per-thread counts above / at the threshold, then exclusive prefix sums
  unsigned gt = 0, eq = 0;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const unsigned kk = (i & 1) ? (key2[i / 2] >> 16) : (key2[i / 2] & 0xFFFFu);
    gt += kk > T;
    eq += kk == T;
  }
  unsigned gt_inc = gt, eq_inc = eq;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned g2 = __shfl_up(gt_inc, off, kWave);
    const unsigned e2 = __shfl_up(eq_inc, off, kWave);
    if (lane >= off) {
      gt_inc += g2;
      eq_inc += e2;
    }
  }
  if (lane == kWave - 1) {
    s_gt[wave] = gt_inc;
    s_eq[wave] = eq_inc;
  }
  __syncthreads();
  unsigned gt_before = gt_inc - gt, eq_before = eq_inc - eq, gt_total = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    if (w < wave) {
      gt_before += s_gt[w];
      eq_before += s_eq[w];
    }
    gt_total += s_gt[w];
  }
  const unsigned need = (unsigned)k - gt_total;  // ties to take, lowest index first
  unsigned pos = gt_before + (eq_before < need ? eq_before : need);
  unsigned eq_rank = eq_before;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const unsigned kk = (i & 1) ? (key2[i / 2] >> 16) : (key2[i / 2] & 0xFFFFu);
    bool take = kk > T;
    if (kk == T) {
      take = eq_rank < need;
      ++eq_rank;
    }
    if (take) {
      if (idx_bytes == 8)
        reinterpret_cast<int64_t*>(idx_out)[pos] = base + i;
      else
        reinterpret_cast<int32_t*>(idx_out)[pos] = base + i;
      ++pos;
    }
  }
}

// ---------------------------------------------------------------------------
// Small inputs (n <= 1024, e.g. attention heads): rank selection in one
// workgroup.  Element i is selected iff fewer than k elements beat it, where j
// beats i when key_j > key_i or (key_j == key_i and j < i); selected indices
// are written in ascending order.  Same result as topk_kernel.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void rank_select_emit(const unsigned* s_key, unsigned* s_sel, int n, int k,
                                                 void* idx_out, int idx_bytes) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const unsigned ki = s_key[i];
    int rank = 0;
    for (int j = 0; j < n; ++j) {
      const unsigned kj = s_key[j];
      rank += (kj > ki) || (kj == ki && j < i);
    }
    s_sel[i] = rank < k ? 1u : 0u;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    if (s_sel[i]) {
      int pos = 0;
      for (int j = 0; j < i; ++j) pos += (int)s_sel[j];
      if (idx_bytes == 8)
        reinterpret_cast<int64_t*>(idx_out)[pos] = i;
      else
        reinterpret_cast<int32_t*>(idx_out)[pos] = i;
    }
  }
}

__global__ __launch_bounds__(256) void topk_small_kernel(const half_t* __restrict__ logits, int B, int n,
                                                         int k, void* __restrict__ idx_out,
                                                         int idx_bytes) {
  __shared__ unsigned s_key[1024];
  __shared__ unsigned s_sel[1024];
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    unsigned key = 0u;
    for (int b0 = 0; b0 < B; b0 += 8) {  // eight rows requested at once (a batch is a chain of latencies otherwise)
      half_t v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = logits[(int64_t)(b0 + u < B ? b0 + u : B - 1) * n + i];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const unsigned kk = topk_key(v[u]);
        key = kk > key ? kk : key;
      }
    }
    s_key[i] = key;
  }
  __syncthreads();
  rank_select_emit(s_key, s_sel, n, k, idx_out, idx_bytes);
}

// ---------------------------------------------------------------------------
// Large inputs: three launches, every one spread over many workgroups (2048 columns each,
// at most kTopkMaxBlocks of them).  No global atomics and no state between calls: every
// workgroup publishes small per-workgroup histograms that the next launch adds up.
//  1) topk_hist_kernel: coarse histogram (key >> 8, 256 bins) of the workgroup's columns,
//     built in LDS, stored to wc[workgroup][256].
//  2) topk_count_kernel: every workgroup adds the coarse histograms, finds the coarse bin c*
//     in which the k-th largest key lies, and stores the fine histogram (key & 255) of ITS
//     columns inside c* to wf[workgroup][256] plus the number of its columns in higher bins.
//  3) topk_emit_kernel: every workgroup adds the fine histograms, which gives the threshold
//     key T and the number of ties to take; from the per-workgroup histograms of the
//     workgroups before it, it knows how many selected columns precede its own and emits its
//     indices with key > T and those of the first `need` columns with key == T at their exact
//     (ascending) positions.
// Workspace layout (u32): wc[32][256], wf[32][256], above[32], meta[4] = {c*, columns above c*},
// then (16-byte aligned) n fp16 values: the column-wise maximum of a batch
// (topk_batch_hist_kernel).
// ---------------------------------------------------------------------------
constexpr int kTopkItemsPerBlock = 256 * 8;
constexpr int kTopkBins = 256;
constexpr int kTopkMaxBlocks = 32;  // n <= 65536
constexpr int kTopkFineOff = kTopkMaxBlocks * kTopkBins;
constexpr int kTopkAboveOff = 2 * kTopkMaxBlocks * kTopkBins;
constexpr int kTopkMetaOff = kTopkAboveOff + kTopkMaxBlocks;
constexpr int kTopkWords = kTopkMetaOff + 4;

__device__ __forceinline__ void topk_load_keys(const half_t* __restrict__ logits, int B, int n, int i0,
                                               unsigned key[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) key[e] = 0u;
  if (i0 >= n) return;
  for (int b = 0; b < B; ++b) {
    const half8_t v = load8(logits + (int64_t)b * n + i0);  // n % 8 == 0
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const unsigned kk = topk_key(v[e]);
      key[e] = kk > key[e] ? kk : key[e];
    }
  }
}

// A workgroup covers 256 * 8 columns with its first 256 threads (further threads, if the launch
// has them, only take part in the barriers).
__device__ __forceinline__ void topk_hist_body(const half_t* __restrict__ logits, int B, int n,
                                               unsigned* __restrict__ ws, int block_id) {
  __shared__ unsigned s_coarse[kTopkBins];
  if (threadIdx.x < kTopkBins) s_coarse[threadIdx.x] = 0u;
  __syncthreads();
  const int i0 = (block_id * 256 + threadIdx.x) * 8;
  if (threadIdx.x < 256 && i0 < n) {
    unsigned key[8];
    topk_load_keys(logits, B, n, i0, key);
#pragma unroll
    for (int e = 0; e < 8; ++e) atomicAdd(&s_coarse[key[e] >> 8], 1u);
  }
  __syncthreads();
  if (threadIdx.x < kTopkBins) ws[block_id * kTopkBins + threadIdx.x] = s_coarse[threadIdx.x];
}

__global__ __launch_bounds__(256) void topk_hist_kernel(const half_t* __restrict__ logits, int B, int n,
                                                        unsigned* __restrict__ ws) {
  topk_hist_body(logits, B, n, ws, blockIdx.x);
}

// A (B, n) batch: the column-wise "maximum" as a row of fp16 values -- m[j] = the logit of column j with
// the largest key (among equal keys the larger bit pattern) -- and the coarse histogram of m's keys, in one
// launch.  Top-k over m equals top-k over the batch with the maximum-over-rows score, so the count and
// emit kernels then read one row instead of B.  Workgroup b owns columns [2048 b, 2048 (b + 1)); its
// threads form blockDim.x / 256 groups (1..4) of 256, group q takes rows 8 q .. 8 q + 7 (then 8 more every
// 8 * groups rows) of one 8-column vector per thread, all eight loads of a turn in flight together, and the
// groups' maxima meet in LDS: up to 32 rows are one round trip to memory.  Requires n % 8 == 0.
constexpr int kTopkBatchGroups = 4;
inline int topk_batch_groups(int B) { return B > 24 ? 4 : B > 16 ? 3 : B > 8 ? 2 : 1; }

__global__ __launch_bounds__(256 * kTopkBatchGroups) void topk_batch_hist_kernel(
    const half_t* __restrict__ logits, int B, int n, half_t* __restrict__ m, unsigned* __restrict__ ws) {
  __shared__ unsigned s_coarse[kTopkBins];
  __shared__ unsigned s_best[kTopkBatchGroups - 1][8][256];
  const int t = threadIdx.x & 255, q = threadIdx.x >> 8, groups = blockDim.x >> 8;
  if (q == 0) s_coarse[t] = 0u;
  const int i0 = (blockIdx.x * 256 + t) * 8;
  unsigned best[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) best[e] = 0u;  // below every packed value of a real row
  if (i0 < n) {
    for (int b0 = 8 * q; b0 < B; b0 += 8 * groups) {
      half8_t v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {  // past the batch the last row repeats (a maximum does not mind)
        const int b = b0 + u < B ? b0 + u : B - 1;
        v[u] = load8(logits + (int64_t)b * n + i0);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const half_t hv = v[u][e];
          const unsigned packed = (topk_key(hv) << 16) | (unsigned)__builtin_bit_cast(unsigned short, hv);
          best[e] = packed > best[e] ? packed : best[e];
        }
    }
  }
  if (q > 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) s_best[q - 1][e][t] = best[e];
  }
  __syncthreads();
  if (q == 0 && i0 < n) {
    for (int g = 1; g < groups; ++g) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const unsigned other = s_best[g - 1][e][t];
        best[e] = other > best[e] ? other : best[e];
      }
    }
    half8_t o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const unsigned short bits = (unsigned short)(best[e] & 0xFFFFu);
      o[e] = __builtin_bit_cast(half_t, bits);
      atomicAdd(&s_coarse[best[e] >> 24], 1u);  // key >> 8
    }
    store8(m + i0, o);
  }
  __syncthreads();
  if (q == 0) ws[blockIdx.x * kTopkBins + t] = s_coarse[t];
}

// Inclusive prefix sum over the 256 threads of a workgroup (s_w: 4 words of LDS).
__device__ __forceinline__ unsigned block256_inclusive_scan(unsigned v, unsigned* s_w) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned t = __shfl_up(v, off, kWave);
    if (lane >= off) v += t;
  }
  __syncthreads();  // s_w may still be read from a previous scan
  if (lane == kWave - 1) s_w[wave] = v;
  __syncthreads();
  for (int w = 0; w < wave; ++w) v += s_w[w];
  return v;
}

// In a 256-bin histogram given in DESCENDING bin order over the threads (thread t owns bin
// 255 - t, count c): the bin in which the k-th largest element lies and the number of elements
// in higher bins.  All threads return the same pair.
__device__ __forceinline__ void topk_crossing_bin(unsigned c, unsigned k, unsigned* s_w, unsigned* s_pair,
                                                  unsigned& bin, unsigned& above) {
  const unsigned inc = block256_inclusive_scan(c, s_w);
  if (inc - c < k && inc >= k) {
    s_pair[0] = 255u - threadIdx.x;
    s_pair[1] = inc - c;
  }
  __syncthreads();
  bin = s_pair[0];
  above = s_pair[1];
}

// 256 threads; nblocks = workgroups of the histogram launch = of this one.
__device__ __forceinline__ void topk_count_body(const half_t* __restrict__ logits, int B, int n, int k,
                                                unsigned* __restrict__ ws, int block_id, int nblocks) {
  __shared__ unsigned s_w[4], s_pair[2], s_fine[kTopkBins], s_gt[4];
  unsigned key[8];
  const int t = threadIdx.x;
  const int i0 = (block_id * 256 + t) * 8;
  topk_load_keys(logits, B, n, i0, key);  // issued before the histogram reads
  // all (at most 32) per-workgroup values of this thread's bin are requested at once: one round
  // trip instead of one per group of workgroups (clamped addresses, masked sums)
  unsigned c = 0;
  {
    unsigned v[kTopkMaxBlocks];
#pragma unroll
    for (int w = 0; w < kTopkMaxBlocks; ++w) v[w] = ws[(w < nblocks ? w : nblocks - 1) * kTopkBins + 255 - t];
#pragma unroll
    for (int w = 0; w < kTopkMaxBlocks; ++w) c += w < nblocks ? v[w] : 0u;
  }
  s_fine[t] = 0u;
  unsigned cstar, above_c;
  topk_crossing_bin(c, (unsigned)k, s_w, s_pair, cstar, above_c);  // (its barriers also cover s_fine)
  unsigned gt = 0;
  if (i0 < n) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const unsigned cb = key[e] >> 8;
      gt += cb > cstar;
      if (cb == cstar) atomicAdd(&s_fine[key[e] & 255u], 1u);
    }
  }
#pragma unroll
  for (int off = kWave / 2; off >= 1; off >>= 1) gt += __shfl_xor(gt, off, kWave);
  if ((t & 63) == 0) s_gt[t >> 6] = gt;
  __syncthreads();
  ws[kTopkFineOff + block_id * kTopkBins + t] = s_fine[t];
  if (t == 0) {
    ws[kTopkAboveOff + block_id] = s_gt[0] + s_gt[1] + s_gt[2] + s_gt[3];
    if (block_id == 0) {
      ws[kTopkMetaOff] = cstar;
      ws[kTopkMetaOff + 1] = above_c;
    }
  }
}

__global__ __launch_bounds__(256) void topk_count_kernel(const half_t* __restrict__ logits, int B, int n,
                                                         int k, unsigned* __restrict__ ws) {
  topk_count_body(logits, B, n, k, ws, blockIdx.x, gridDim.x);
}

__device__ __forceinline__ void topk_emit_body(const half_t* __restrict__ logits, int B, int n, int k,
                                               const unsigned* __restrict__ ws, void* __restrict__ idx_out,
                                               int idx_bytes, int block_id, int nblocks) {
  __shared__ unsigned s_w[4], s_pair[2], s_base[2];
  unsigned key[8];
  const int t = threadIdx.x;
  const int i0 = (block_id * 256 + t) * 8;
  topk_load_keys(logits, B, n, i0, key);
  const unsigned cstar = ws[kTopkMetaOff], above_c = ws[kTopkMetaOff + 1];
  // fine bins of c* in descending order: thread t owns fine bin 255 - t; `mine` counts that bin in
  // the workgroups before this one
  unsigned f = 0, mine = 0;
  {
    unsigned v[kTopkMaxBlocks];  // one round trip, as in topk_count_body
#pragma unroll
    for (int w = 0; w < kTopkMaxBlocks; ++w)
      v[w] = ws[kTopkFineOff + (w < nblocks ? w : nblocks - 1) * kTopkBins + 255 - t];
#pragma unroll
    for (int w = 0; w < kTopkMaxBlocks; ++w) {
      f += w < nblocks ? v[w] : 0u;
      mine += w < block_id ? v[w] : 0u;
    }
  }
  unsigned tlow, above_f;
  topk_crossing_bin(f, (unsigned)k - above_c, s_w, s_pair, tlow, above_f);
  const unsigned T = cstar * 256u + tlow;
  const unsigned need = (unsigned)k - above_c - above_f;  // ties to take, lowest index first
  // selected columns in the workgroups before this one: those in higher coarse bins, those in
  // higher fine bins of c*, and the ties
  unsigned gt_part = (255u - (unsigned)t > tlow) ? mine : 0u;
  if (t < block_id) gt_part += ws[kTopkAboveOff + t];  // block_id <= 32 <= 256 threads
  const unsigned gt_all = block256_inclusive_scan(gt_part, s_w);
  if (t == 255) s_base[0] = gt_all;
  if (255u - (unsigned)t == tlow) s_base[1] = mine;
  unsigned gt = 0, eq = 0;
  if (i0 < n) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      gt += key[e] > T;
      eq += key[e] == T;
    }
  }
  const unsigned gt_inc = block256_inclusive_scan(gt, s_w);
  const unsigned eq_inc = block256_inclusive_scan(eq, s_w);
  __syncthreads();
  const unsigned gt_before = s_base[0] + gt_inc - gt;
  const unsigned eq_before = s_base[1] + eq_inc - eq;
  unsigned pos = gt_before + (eq_before < need ? eq_before : need);
  unsigned eq_rank = eq_before;
  if (i0 < n) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      bool take = key[e] > T;
      if (key[e] == T) {
        take = eq_rank < need;
        ++eq_rank;
      }
      if (take) {
        if (idx_bytes == 8)
          reinterpret_cast<int64_t*>(idx_out)[pos] = i0 + e;
        else
          reinterpret_cast<int32_t*>(idx_out)[pos] = i0 + e;
        ++pos;
      }
    }
  }
}

__global__ __launch_bounds__(256) void topk_emit_kernel(const half_t* __restrict__ logits, int B, int n, int k,
                                                        const unsigned* __restrict__ ws,
                                                        void* __restrict__ idx_out, int idx_bytes) {
  topk_emit_body(logits, B, n, k, ws, idx_out, idx_bytes, blockIdx.x, gridDim.x);
}

// ---------------------------------------------------------------------------
// Greedy step of a generation loop (batch 1), one workgroup: next token = argmax of the logits
// (first index among equal values, NaN ranks highest -- as torch.argmax), then the device-side
// bookkeeping that lets a captured step be replayed: token <- next, sequences[out_index++] <-
// next, position++, seq_pos++; optionally the logits row is kept in scores[score_index++].
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void greedy_advance_kernel(
    const half_t* __restrict__ logits, int vocab, int64_t* __restrict__ token, int64_t* __restrict__ position,
    int* __restrict__ seq_pos, int64_t* __restrict__ sequences, int64_t* __restrict__ out_index,
    half_t* __restrict__ scores, int64_t score_ld, int64_t* __restrict__ score_index, int64_t seq_capacity,
    int64_t score_rows) {
  __shared__ unsigned s_key[16];
  __shared__ int s_idx[16];
  unsigned best = 0u;
  int best_i = 0x7fffffff;
  auto take = [&](half_t v, int i) {
    const unsigned k = topk_key(v) + 1u;  // +1: any element beats the empty start value
    if (k > best) {  // i ascends per thread: equal keys keep the lower index
      best = k;
      best_i = i;
    }
  };
  // 16-byte loads, eight of them in flight per thread (a thread's packets ascend in index)
  const int npk = (reinterpret_cast<uintptr_t>(logits) & 15) == 0 ? vocab / 8 : 0;
  for (int p0 = threadIdx.x; p0 < npk; p0 += 8 * blockDim.x) {
    half8_t v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int p = p0 + u * blockDim.x;
      v[u] = load8(logits + (int64_t)(p < npk ? p : p0) * 8);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int p = p0 + u * blockDim.x;
      if (p < npk) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const half_t hv = v[u][e];
          take(hv, p * 8 + e);
        }
      }
    }
  }
  for (int i = npk * 8 + threadIdx.x; i < vocab; i += blockDim.x) take(logits[i], i);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const unsigned ok = (unsigned)__shfl_xor((int)best, off, kWave);
    const int oi = __shfl_xor(best_i, off, kWave);
    if (ok > best || (ok == best && oi < best_i)) {
      best = ok;
      best_i = oi;
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    s_key[wave] = best;
    s_idx[wave] = best_i;
  }
  // a replay past the end of the output buffers (the host loop normally stops first) stores nothing
  if (scores != nullptr && score_index[0] >= 0 && score_index[0] < score_rows) {
    half_t* row = scores + score_index[0] * score_ld;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) row[i] = logits[i];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w)
      if (s_key[w] > best || (s_key[w] == best && s_idx[w] < best_i)) {
        best = s_key[w];
        best_i = s_idx[w];
      }
    token[0] = best_i;
    if (out_index[0] >= 0 && out_index[0] < seq_capacity) sequences[out_index[0]] = best_i;
    out_index[0] += 1;
    position[0] += 1;
    seq_pos[0] += 1;
    if (scores != nullptr) score_index[0] += 1;
  }
}

}  // namespace dv
