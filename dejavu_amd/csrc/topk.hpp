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

}  // namespace dv
