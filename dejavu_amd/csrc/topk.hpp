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
#pragma unroll
    for (int i = 0; i < ITEMS; i += 8) {
      half8_t v = zero8();
      bool have[8];
      if (VEC) {
        const bool in = base + i < n;
        if (in) v = load8(row + base + i);
#pragma unroll
        for (int e = 0; e < 8; ++e) have[e] = in;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          have[e] = base + i + e < n;
          if (have[e]) v[e] = row[base + i + e];
        }
      }
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const unsigned lo = have[e] ? topk_key(v[e]) : 0u;
        const unsigned hi = have[e + 1] ? topk_key(v[e + 1]) : 0u;
        const unsigned old = key2[(i + e) / 2];
        const unsigned olo = old & 0xFFFFu, ohi = old >> 16;
        key2[(i + e) / 2] = (lo > olo ? lo : olo) | ((hi > ohi ? hi : ohi) << 16);
      }
    }
  }

  // largest T with count(key >= T) >= k
  unsigned T = 0u;
  for (int bit = 15; bit >= 0; --bit) {
    const unsigned cand = T | (1u << bit);
    unsigned c = 0;
#pragma unroll
    for (int i = 0; i < ITEMS / 2; ++i) {
      // keep the keys packed across iterations (stops the unpacked halves from
      // being hoisted out of the search loop into twice the registers)
      asm volatile("" : "+v"(key2[i]));
      c += (unsigned)__popcll(__ballot((key2[i] & 0xFFFFu) >= cand));
      c += (unsigned)__popcll(__ballot((key2[i] >> 16) >= cand));
    }
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

}  // namespace dv
