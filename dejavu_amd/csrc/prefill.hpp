// Prompt-phase (prefill) causal attention on the matrix cores, writing the prompt's K / V rows
// straight into the decode caches.
//
//   ctx[b, t, h, :] = softmax_{s <= t}( q[b, t, h] . k[b, s, h] * scale ) . v[b, s, h]
//   k_cache[b, h, j / 8, pos0 + t, j % 8] = k[b, t, h, j];  v_cache[b, h, pos0 + t, j] = v[b, t, h, j]
//
// qkv is the output of the Wqkv product, (B, T, 3, H, hd) fp16.  A workgroup of four wavefronts
// handles 64 consecutive queries of one (b, h): wavefront w owns queries q0 .. q0 + 15 and walks the
// keys 0 .. q0 + 15 in blocks of 32 with an online softmax (fp32 scores, running maximum and sum):
//   S (16 x 32) = Q . K^T      v_mfma_f32_16x16x32_f16 over head_dim, K operands straight from memory
//   P = exp(S - max) as fp16, through a wavefront-private LDS tile into A-operand layout
//   O (16 x hd) += P . V       V block transposed through LDS so that a lane reads 8 consecutive keys
// Lane l of an MFMA result holds rows 4 * (l / 16) + v, column l % 16: the same lanes hold a query's
// scores and its output columns, so the running maximum / sum / rescale never leave the registers
// (row reductions are butterflies over the 16 lanes of a group).  The workgroup also copies its 64
// tokens' K and V rows into the caches (the packed key layout of the decode kernels).
// HD in {64, 128}.  Grid (ceil(T / 64), H, B), 256 threads.
#pragma once
#include "common.hpp"
#include "gemm_mfma.hpp"

namespace dv {

constexpr int kPfWaves = 4;
constexpr int kPfKeys = 32;            // keys per step
constexpr int kPfVtRow = kPfKeys + 8;  // halfs per row of the transposed V tile

template <int HD>
__global__ __launch_bounds__(kPfWaves * 64) void prefill_attn_kernel(
    const half_t* __restrict__ qkv, int T, int H, float scale, half_t* __restrict__ ctx,
    half_t* __restrict__ k_cache, half_t* __restrict__ v_cache, int pos0, int S) {
  __shared__ __attribute__((aligned(16))) half_t s_p[kPfWaves][16 * kPfVtRow];   // P tile, [query][key]
  __shared__ __attribute__((aligned(16))) half_t s_vt[kPfWaves][HD * kPfVtRow];  // V block, [column][key]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kg = lane >> 4;
  const int h = blockIdx.y, b = blockIdx.z;
  const int64_t tstride = (int64_t)3 * H * HD;  // elements between consecutive tokens
  const half_t* base = qkv + (int64_t)b * T * tstride + (int64_t)h * HD;
  const half_t* Qb = base;
  const half_t* Kb = base + (int64_t)H * HD;
  const half_t* Vb = base + (int64_t)2 * H * HD;
  const int t0 = blockIdx.x * (kPfWaves * 16);

  // ---- the workgroup's 64 tokens: K and V rows into the caches ----
  if (k_cache != nullptr) {
    const int64_t bh = (int64_t)b * H + h;
    for (int o = tid; o < kPfWaves * 16 * (HD / 8); o += kPfWaves * 64) {
      const int tt = o / (HD / 8), j8 = o % (HD / 8);
      const int t = t0 + tt, pos = pos0 + t;
      if (t < T && pos >= 0 && pos < S) {
        const half8_t kv = load8(Kb + (int64_t)t * tstride + j8 * 8);
        const half8_t vv = load8(Vb + (int64_t)t * tstride + j8 * 8);
        store8(k_cache + ((bh * (HD / 8) + j8) * S + pos) * 8, kv);
        store8(v_cache + (bh * S + pos) * HD + j8 * 8, vv);
      }
    }
  }

  const int q0 = t0 + wave * 16;
  if (q0 >= T) return;  // whole wavefront past the prompt (no workgroup barrier below)
  half_t* ps = s_p[wave];
  half_t* vt = s_vt[wave];
  constexpr int KS = HD / 32;   // MFMA k-steps over head_dim
  constexpr int JT = HD / 16;   // output column tiles

  // Q operands: lane (query l16, k-group kg) holds Q[q0 + l16][ks * 32 + kg * 8 ..]
  half8_t qa[KS];
  {
    const int q = q0 + l16 < T ? q0 + l16 : T - 1;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qa[ks] = load8(Qb + (int64_t)q * tstride + ks * 32 + kg * 8);
  }
  float4_t o_acc[JT];
#pragma unroll
  for (int jt = 0; jt < JT; ++jt) o_acc[jt] = float4_t{0.f, 0.f, 0.f, 0.f};
  float m_run[4], l_run[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    m_run[v] = -INFINITY;
    l_run[v] = 0.f;
  }

  const int k_end = q0 + 16 < T ? q0 + 16 : T;  // keys 0 .. k_end - 1 are visible to some query of the tile
  for (int k0 = 0; k0 < k_end; k0 += kPfKeys) {
    // scores of two 16-key tiles
    float4_t s_acc[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int key = k0 + st * 16 + l16 < T ? k0 + st * 16 + l16 : T - 1;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const half8_t kb = load8(Kb + (int64_t)key * tstride + ks * 32 + kg * 8);
        // A = keys, B = queries would transpose the result; here A = Q (rows = queries), B = K (columns = keys)
        s_acc[st] = mfma_16x16x32(qa[ks], kb, s_acc[st]);
      }
    }
    // V block, transposed into LDS: vt[column][key]; lane loads 8 columns of one key per instruction
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");  // the previous step's tile reads are done
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int p = 0; p < kPfKeys * (HD / 8) / 64; ++p) {
      const int o = p * 64 + lane;
      const int kk = o / (HD / 8), j8 = o % (HD / 8);
      const int key = k0 + kk < T ? k0 + kk : T - 1;
      const half8_t vv = load8(Vb + (int64_t)key * tstride + j8 * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) vt[(j8 * 8 + e) * kPfVtRow + kk] = vv[e];
    }
    // online softmax: value v of a lane is query q0 + 4 * kg + v, key k0 + st * 16 + l16
    float p_val[2][4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int q = q0 + 4 * kg + v;
      float sv[2];
      float mx = -INFINITY;
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const int key = k0 + st * 16 + l16;
        sv[st] = (key <= q && key < T) ? s_acc[st][v] * scale : -INFINITY;
        mx = fmaxf(mx, sv[st]);
      }
      mx = butterfly_max<16>(mx);
      const float m_new = fmaxf(m_run[v], mx);
      // a query row past T (or a block wholly above the diagonal for this row) keeps m = -inf: no contribution
      const float alpha = m_new == -INFINITY ? 1.f : __expf(m_run[v] - m_new);
      float sum = 0.f;
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const float pv = sv[st] == -INFINITY ? 0.f : __expf(sv[st] - m_new);
        p_val[st][v] = pv;
        sum += pv;
      }
      sum = butterfly_sum<16>(sum);
      l_run[v] = l_run[v] * alpha + sum;
      m_run[v] = m_new;
#pragma unroll
      for (int jt = 0; jt < JT; ++jt) o_acc[jt][v] *= alpha;
    }
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int v = 0; v < 4; ++v) ps[(4 * kg + v) * kPfVtRow + st * 16 + l16] = (half_t)p_val[st][v];
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // O += P . V: A = P (query l16, keys kg * 8 ..), B = V^T (column jt * 16 + l16, keys kg * 8 ..)
    const half8_t pa = load8(ps + l16 * kPfVtRow + kg * 8);
#pragma unroll
    for (int jt = 0; jt < JT; ++jt) {
      const half8_t vb = load8(vt + (jt * 16 + l16) * kPfVtRow + kg * 8);
      o_acc[jt] = mfma_16x16x32(pa, vb, o_acc[jt]);
    }
  }
  // normalise and store: value v of a lane is query q0 + 4 * kg + v, column jt * 16 + l16
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int q = q0 + 4 * kg + v;
    if (q >= T) continue;
    const float inv = l_run[v] > 0.f ? 1.f / l_run[v] : 0.f;
    half_t* dst = ctx + ((int64_t)b * T + q) * H * HD + (int64_t)h * HD;
#pragma unroll
    for (int jt = 0; jt < JT; ++jt) dst[jt * 16 + l16] = (half_t)(o_acc[jt][v] * inv);
  }
}

}  // namespace dv
