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
    for (int b = 0; b < B; ++b) {
      const unsigned kk = topk_key(logits[(int64_t)b * n + i]);
      key = kk > key ? kk : key;
    }
    s_key[i] = key;
  }
  __syncthreads();
  rank_select_emit(s_key, s_sel, n, k, idx_out, idx_bytes);
}

// ---------------------------------------------------------------------------
// Large inputs, two launches.
//  1) topk_hist_kernel (many workgroups): hist[key] += 1 for every column's key
//     (65536 bins, integer atomics => order-independent, deterministic).
//  2) topk_select_kernel (one workgroup of 1024): scans the histogram from the
//     top for the threshold key T (largest T with count(key >= T) >= k), clears
//     the histogram for the next call, then emits the indices with key > T and
//     the first k - count(key > T) indices with key == T, ascending, with one
//     workgroup prefix sum.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void topk_hist_kernel(const half_t* __restrict__ logits, int B, int n,
                                                        unsigned* __restrict__ hist) {
  const int i0 = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i0 >= n) return;
  unsigned key[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) key[e] = 0u;
  for (int b = 0; b < B; ++b) {
    const half8_t v = load8(logits + (int64_t)b * n + i0);  // n % 8 == 0
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const unsigned kk = topk_key(v[e]);
      key[e] = kk > key[e] ? kk : key[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) atomicAdd(&hist[key[e]], 1u);
}

template <int ITEMS>
__global__ __launch_bounds__(1024) void topk_select_kernel(const half_t* __restrict__ logits, int B,
                                                           int n, int k, unsigned* __restrict__ hist,
                                                           void* __restrict__ idx_out, int idx_bytes) {
  constexpr int THREADS = 1024, WAVES = THREADS / kWave, BINS = 65536 / THREADS;
  __shared__ unsigned s_a[WAVES], s_b[WAVES];
  __shared__ unsigned s_T, s_above;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  // keys of this thread's columns (issued first, consumed last)
  const int base = tid * ITEMS;
  half8_t v[ITEMS / 8];
#pragma unroll
  for (int i = 0; i < ITEMS / 8; ++i) {
    const int off = base + i * 8;
    v[i] = load8(logits + (off < n ? off : 0));
  }

  // thread t owns the 64 bins [65536 - 64 (t + 1), 65536 - 64 t): descending key order
  const int bin_lo = 65536 - BINS * (tid + 1);
  const uint4* hv = reinterpret_cast<const uint4*>(hist + bin_lo);
  unsigned mine = 0;
#pragma unroll
  for (int j = 0; j < BINS / 4; ++j) {
    const uint4 c = hv[j];
    mine += c.x + c.y + c.z + c.w;
  }
  // exclusive prefix (over descending keys) of the per-thread totals
  unsigned inc = mine;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned t2 = __shfl_up(inc, off, kWave);
    if (lane >= off) inc += t2;
  }
  if (lane == kWave - 1) s_a[wave] = inc;
  __syncthreads();
  unsigned before = inc - mine;
#pragma unroll
  for (int w = 0; w < WAVES; ++w)
    if (w < wave) before += s_a[w];
  // the thread whose bins make the running count reach k owns the threshold:
  // it walks its bins again, from the highest key down
  if (k > 0 && before < (unsigned)k && before + mine >= (unsigned)k) {
    unsigned run = before;
    for (int j = BINS - 1; j >= 0; --j) {
      const unsigned c = hist[bin_lo + j];
      if (run < (unsigned)k && run + c >= (unsigned)k) {
        s_T = (unsigned)(bin_lo + j);
        s_above = run;  // count(key > T)
      }
      run += c;
    }
  }
  __syncthreads();
  {  // leave the histogram cleared for the next call
    uint4* hz = reinterpret_cast<uint4*>(hist + bin_lo);
    const uint4 z = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < BINS / 4; ++j) hz[j] = z;
  }
  const unsigned T = s_T;
  const unsigned need = (unsigned)k - s_above;

  // B > 1: a column's key is the maximum over the rows
  unsigned key[ITEMS];
#pragma unroll
  for (int i = 0; i < ITEMS / 8; ++i) {
    const bool in = base + i * 8 < n;
#pragma unroll
    for (int e = 0; e < 8; ++e) key[i * 8 + e] = in ? topk_key(v[i][e]) : 0u;
  }
  for (int b = 1; b < B; ++b) {
#pragma unroll
    for (int i = 0; i < ITEMS / 8; ++i) {
      const int off = base + i * 8;
      if (off < n) {
        const half8_t w = load8(logits + (int64_t)b * n + off);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const unsigned kk = topk_key(w[e]);
          key[i * 8 + e] = kk > key[i * 8 + e] ? kk : key[i * 8 + e];
        }
      }
    }
  }
  unsigned gt = 0, eq = 0;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    gt += key[i] > T;
    eq += key[i] == T;
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
    s_a[wave] = gt_inc;
    s_b[wave] = eq_inc;
  }
  __syncthreads();
  unsigned gt_before = gt_inc - gt, eq_before = eq_inc - eq;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    if (w < wave) {
      gt_before += s_a[w];
      eq_before += s_b[w];
    }
  }
  unsigned pos = gt_before + (eq_before < need ? eq_before : need);
  unsigned eq_rank = eq_before;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    bool take = key[i] > T;
    if (key[i] == T) {
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

}  // namespace dv
