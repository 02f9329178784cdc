// Attention for many queries (prefill / prompt chunk) on the MFMA matrix cores:
// flash-style, causal / windowed, grouped-query, the queries being the last rows
// of the keys.
//
// grid = (ceil(seq/128), heads); a block of 4 waves takes 128 query rows of one
// head, a wave 32 of them.  Keys and values stream through LDS in tiles of 64
// rows.  The wave computes the TRANSPOSED score tile S^T = K Q^T (M = keys,
// N = queries): a lane then owns one query column, so the row max / row sum of
// the online softmax are in-lane reductions plus one exchange with lane^32, and
// the probabilities are already laid out as the B operand of O^T = V^T P^T.  V is
// transposed on its way into LDS so its fragments are k-contiguous.  All softmax
// state is f32 in the exp2 domain.
#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {

constexpr int BQ = 128;   // query rows per block
constexpr int BKV = 64;   // key rows per tile

// At least two waves a SIMD caps the register budget at 256, which makes the compiler keep MFMA
// accumulators in ordinary VGPRs: the softmax reads S and rescales O in place instead of copying
// every value out of (and back into) accumulation registers.
template <int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void mha_prefill_kernel(
    const bf16_t* __restrict__ Q, const bf16_t* __restrict__ K, const bf16_t* __restrict__ V,
    bf16_t* __restrict__ O, int group, int seq, int seq_len, int kv_len, float scale_log2,
    int causal, int window, long q_row_stride, long q_head_stride, long kv_row_stride,
    long kv_head_stride, const int* __restrict__ valid, const int* __restrict__ kv_valid) {
  constexpr int LDK = D + 8;     // K tile row (elements)
  constexpr int LDV = BKV + 8;   // V^T tile row
  constexpr int KS = D / 16;     // k16 steps of S^T
  constexpr int DT = D / 32;     // 32-row tiles of O^T
  constexpr int CPR = D / 8;     // 16-byte chunks a key row has
  constexpr int NL = BKV * CPR / 256;   // 16-byte loads a thread makes of K (and of V) per tile
  constexpr int K_TILE = BKV * LDK, V_TILE = D * LDV;
  __shared__ __align__(16) bf16_t Ks[2 * K_TILE];
  __shared__ __align__(16) bf16_t Vt[2 * V_TILE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, g = lane >> 5;
  const int head = blockIdx.y, kvh = head / group;
  // Heaviest (last) query blocks first under a causal mask.
  const int qb = gridDim.x - 1 - blockIdx.x;
  const int q0 = qb * BQ;

  const int q_tokens = valid ? bound_or(valid, seq) : seq_len;
  const int kv_tokens = kv_valid ? bound_or(kv_valid, kv_len) : (kv_len - seq + q_tokens);
  const bool masked_any = causal || window >= 0;
  const int offset = masked_any ? (kv_tokens - q_tokens) : 0;

  const int my_q = q0 + wave * 32 + col;            // this lane's query row
  const bool q_live = my_q < q_tokens;
  const int qpos = offset + my_q;
  const int wq_lo = offset + q0 + wave * 32;        // positions of the wave's first and last live query
  const int wq_hi = offset + min(q0 + wave * 32 + 31, q_tokens - 1);

  bf16_t* Oh = O + (size_t)head * q_head_stride;
  // Rows of this block past the bound: zeros.  A block wholly past it does only that.
  if (q0 >= q_tokens || offset < 0) {
    for (int i = tid; i < BQ * CPR; i += 256) {
      const int r = q0 + i / CPR, c = (i % CPR) * 8;
      if (r < seq) *reinterpret_cast<uint4*>(Oh + (size_t)r * q_row_stride + c) = make_uint4(0, 0, 0, 0);
    }
    return;
  }

  // Q^T fragments (B operand): lane holds query `col`, d = 16*s + 8*g .. +7.
  bf16x8 qf[KS];
  {
    const bf16_t* qp = Q + (size_t)head * q_head_stride + (size_t)my_q * q_row_stride + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (q_live) v = *reinterpret_cast<const uint4*>(qp + 16 * s);
      qf[s] = __builtin_bit_cast(bf16x8, v);
    }
  }

  f32x16 oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[t][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;   // the running max is of the raw (unscaled) scores

  // Keys this block's live queries can see.
  const int q_last = min(q0 + BQ, q_tokens) - 1;
  int kv_hi = kv_tokens;
  if (causal) kv_hi = min(kv_hi, offset + q_last + 1);
  else if (window >= 0) kv_hi = min(kv_hi, offset + q_last + window + 1);
  int kv_lo = 0;
  if (window >= 0) kv_lo = max(0, offset + q0 - window) / BKV * BKV;

  const bf16_t* Kh = K + (size_t)kvh * kv_head_stride;
  const bf16_t* Vh = V + (size_t)kvh * kv_head_stride;

  // Tile staging: K as stored; V two keys a load pair, transposed on the way into LDS.
  uint4 kreg[NL], vreg[NL];
  auto fetch = [&](int kv0) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int p = tid + i * 256;
      const int r = p / CPR, c = (p % CPR) * 8;
      kreg[i] = (kv0 + r < kv_tokens) ? *reinterpret_cast<const uint4*>(Kh + (size_t)(kv0 + r) * kv_row_stride + c)
                                      : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      // load i is key 2*pair + (i & 1) of strip `tid % CPR`, pair = tid / CPR + (i / 2) * (256 / CPR)
      const int strip = tid % CPR, key = 2 * (tid / CPR + (i >> 1) * (256 / CPR)) + (i & 1);
      vreg[i] = (kv0 + key < kv_tokens) ? *reinterpret_cast<const uint4*>(Vh + (size_t)(kv0 + key) * kv_row_stride + strip * 8)
                                        : make_uint4(0, 0, 0, 0);
    }
  };
  auto stage = [&](int buf) {
    bf16_t* kd = Ks + buf * K_TILE;
    bf16_t* vd = Vt + buf * V_TILE;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int p = tid + i * 256;
      *reinterpret_cast<uint4*>(kd + (p / CPR) * LDK + (p % CPR) * 8) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < NL; i += 2) {
      const int strip = tid % CPR, key = 2 * (tid / CPR + (i >> 1) * (256 / CPR));
      const uint32_t a[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
      const uint32_t b[4] = {vreg[i + 1].x, vreg[i + 1].y, vreg[i + 1].z, vreg[i + 1].w};
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
        *reinterpret_cast<uint32_t*>(vd + (strip * 8 + c) * LDV + key) = __builtin_amdgcn_perm(b[c >> 1], a[c >> 1], sel);
      }
    }
  };

  if (kv_lo < kv_hi) {
    fetch(kv_lo);
    stage(0);
  }
  __syncthreads();

  int buf = 0;
  for (int kv0 = kv_lo; kv0 < kv_hi; kv0 += BKV, buf ^= 1) {
    const bool more = kv0 + BKV < kv_hi;
    if (more) fetch(kv0 + BKV);   // in flight during this tile's MFMAs

    // Tiles wholly above the wave's last query (causal) hold nothing for it.
    const bool skip = causal && kv0 > wq_hi;
    if (!skip) {
      const bf16_t* kt = Ks + buf * K_TILE;
      const bf16_t* vt = Vt + buf * V_TILE;
      // S^T = K Q^T for the two 32-key halves of the tile.
      f32x16 sacc[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int e = 0; e < 16; ++e) sacc[t][e] = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(kt + (t * 32 + col) * LDK + 16 * s + 8 * g);
          sacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], sacc[t], 0, 0, 0);
        }
      }
      // Only tiles that touch a bound or the mask's edge pay for masking.  Element e of half t
      // is key kv0 + 32 t + 8 (e/4) + 4 g + e%4, query `col`.
      bool edge = kv0 + BKV > kv_tokens;
      if (causal) edge |= kv0 + BKV - 1 > wq_lo;
      else if (window >= 0) edge |= kv0 + BKV - 1 > wq_lo + window;
      if (window >= 0) edge |= kv0 < wq_hi - window;
      if (edge) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int kpos = kv0 + 32 * t + 8 * (e >> 2) + 4 * g + (e & 3);
            bool dead = kpos >= kv_tokens;
            if (causal) dead |= kpos > qpos;
            else if (window >= 0) dead |= kpos > qpos + window;
            if (window >= 0) dead |= kpos < qpos - window;
            if (dead) sacc[t][e] = -INFINITY;
          }
      }
      float rmax = sacc[0][0];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) rmax = fmaxf(rmax, sacc[t][e]);
      rmax = fmaxf(rmax, __shfl_xor(rmax, 32, 64));
      const float m_new = fmaxf(m_run, rmax);
      const float mc = (m_new == -INFINITY) ? 0.f : m_new * scale_log2;
      const float alpha = __builtin_amdgcn_exp2f(fmaf(m_run, scale_log2, -mc));  // exp2(-inf) = 0 at the start
      m_run = m_new;
      float rsum = 0.f;
      bf16x8 pf[2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          float p[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            p[j] = __builtin_amdgcn_exp2f(fmaf(sacc[t][8 * h + j], scale_log2, -mc));
            rsum += p[j];
          }
          pf[t][h] = __builtin_bit_cast(bf16x8, pack8(p));
        }
      l_run = l_run * alpha + rsum;
      // After the first tiles a new maximum is rare: rescale O only when some query's moved.
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int e = 0; e < 16; ++e) oacc[t][e] *= alpha;
      }

      // O^T += V^T P^T.  k slots of lane group g at (t, h): keys 32 t + 16 h + 4 g + 0..3 and the same + 8.
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const bf16_t* vp = vt + (dt * 32 + col) * LDV + 32 * t + 16 * h + 4 * g;
            const uint2 lo = *reinterpret_cast<const uint2*>(vp);
            const uint2 hi = *reinterpret_cast<const uint2*>(vp + 8);
            const bf16x8 vf = __builtin_bit_cast(bf16x8, make_uint4(lo.x, lo.y, hi.x, hi.y));
            oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[t][h], oacc[dt], 0, 0, 0);
          }
    }
    if (more) stage(buf ^ 1);   // the other buffer: everyone finished reading it a tile ago
    __syncthreads();
  }

  // Normalize and store: lane holds query `col`, columns 32 dt + 8 q + 4 g + 0..3.
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = (q_live && l_tot > 0.f) ? 1.0f / l_tot : 0.f;
  if (my_q < seq) {
    bf16_t* op = Oh + (size_t)my_q * q_row_stride;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float v0 = oacc[dt][4 * q + 0] * inv, v1 = oacc[dt][4 * q + 1] * inv,
                    v2 = oacc[dt][4 * q + 2] * inv, v3 = oacc[dt][4 * q + 3] * inv;
        *reinterpret_cast<uint2*>(op + 32 * dt + 8 * q + 4 * g) =
            make_uint2(pack_bf16(v0, v1), pack_bf16(v2, v3));
      }
  }
}

}  // namespace iron

using namespace iron;

extern "C" int iron_mha_prefill_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                     uint16_t* O, int heads, int kv_heads, int d, int seq,
                                     int seq_len, int kv_len, float scale, int causal, int window,
                                     int q_interleaved, int kv_interleaved, const int* valid,
                                     const int* kv_valid, void* stream) {
  IRON_REQUIRE(Q && K && V && O, "mha_prefill: null operand");
  IRON_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
               "mha_prefill: heads (%d) must be a positive multiple of kv_heads (%d)", heads, kv_heads);
  IRON_REQUIRE(d == 64 || d == 128, "mha_prefill: d (%d) must be 64 or 128", d);
  IRON_REQUIRE(seq > 0 && seq_len > 0 && seq_len <= seq,
               "mha_prefill: seq_len (%d) must be in [1, seq (%d)]", seq_len, seq);
  IRON_REQUIRE(kv_len >= seq, "mha_prefill: kv_len (%d) must be at least seq (%d): the queries are its last rows",
               kv_len, seq);
  IRON_REQUIRE(scale >= 0.f && scale < INFINITY, "mha_prefill: scale must be finite and not negative");
  IRON_REQUIRE((((uintptr_t)Q | (uintptr_t)K | (uintptr_t)V | (uintptr_t)O) & 15) == 0,
               "mha_prefill: operands must be 16-byte aligned");
  const long q_row = q_interleaved ? (long)heads * d : d;
  const long q_head = q_interleaved ? d : (long)seq * d;
  const long kv_row = kv_interleaved ? (long)kv_heads * d : d;
  const long kv_head = kv_interleaved ? d : (long)kv_len * d;
  const float scale_log2 = scale * 1.4426950408889634f;
  dim3 grid((seq + BQ - 1) / BQ, heads), block(256);
  hipStream_t s = (hipStream_t)stream;
  if (d == 64)
    hipLaunchKernelGGL((mha_prefill_kernel<64>), grid, block, 0, s, Q, K, V, O, heads / kv_heads, seq,
                       seq_len, kv_len, scale_log2, causal, window, q_row, q_head, kv_row, kv_head,
                       valid, kv_valid);
  else
    hipLaunchKernelGGL((mha_prefill_kernel<128>), grid, block, 0, s, Q, K, V, O, heads / kv_heads,
                       seq, seq_len, kv_len, scale_log2, causal, window, q_row, q_head, kv_row,
                       kv_head, valid, kv_valid);
  IRON_LAUNCH_CHECK();
}
