// Attention for one query token over a KV cache (decode): pure KV streaming,
// HBM-bandwidth bound.
//
// grid = (splits, kv_heads).  A block of 4 waves takes one contiguous slice of the
// keys of one KV head and serves all G query heads of its group from that single
// stream.  D/8 lanes cover one key row with 16-byte loads (a wave covers 512/D rows
// per step); scores are reduced across those lanes, the softmax is kept online in
// f32 in the exp2 domain per lane group, and lane groups, waves and finally splits
// are merged by the usual (max, sum, acc) rule.  A second small kernel merges the
// splits and writes bf16.
#include "../../include/iron_hip.h"
#include "common.h"

#include <mutex>

namespace iron {

constexpr int kMaxSplits = 128;
constexpr int kSingleMaxKeys = 2048;  // caches up to this many rows take the one-launch kernel

// 2^x for x <= 0 by the hardware's own instruction: a softmax weight small enough to be a denormal
// counts as 0, which saves the library routine's rescaling around every call.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

typedef __bf16 bf16x2_v __attribute__((ext_vector_type(2)));
// The dot product of two 16-byte runs of bf16.
__device__ __forceinline__ float dot8(const uint4& a, const uint4& b) {
  float d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_v, a.x), __builtin_bit_cast(bf16x2_v, b.x), 0.f, false);
  d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_v, a.y), __builtin_bit_cast(bf16x2_v, b.y), d, false);
  d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_v, a.z), __builtin_bit_cast(bf16x2_v, b.z), d, false);
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_v, a.w), __builtin_bit_cast(bf16x2_v, b.w), d, false);
}

// One wave's pass over key rows base + u*RW + rg for base = lo, lo + stride, ... while < hi, for
// the G query heads q0.. of one KV head, then the merge of the wave's lane groups: on return every
// lane holds the wave's (m, l) per head and acc = its 8 columns sub*8.. of the weighted V sum.
// STREAM: rows are read with streaming (non-temporal) loads -- right for a long cache read once per
// step; a short cache is better left to the caches, where the next step finds much of it again.
template <int D, int G, int U, bool STREAM>
__device__ __forceinline__ void decode_scan(const bf16_t* __restrict__ Q, const bf16_t* __restrict__ Kh,
                                            const bf16_t* __restrict__ Vh, int q0, int lo, int hi,
                                            int stride, long row_stride, float scale_log2,
                                            float (&m)[G], float (&l)[G], float (&acc)[G][8]) {
  constexpr int LPR = D / 8;     // lanes per key row
  constexpr int RW = 64 / LPR;   // rows a wave covers per step
  const int lane = threadIdx.x & 63;   // U = steps in flight
  const int sub = lane % LPR, rg = lane / LPR;

  // The queries stay packed bf16: a score is four two-element dot products (v_dot2c_f32_bf16: exact
  // products, float32 sums) of a key's 16 bytes as they were loaded, scaled once at the end.
  uint4 qp[G];
#pragma unroll
  for (int g = 0; g < G; ++g) qp[g] = *reinterpret_cast<const uint4*>(Q + (size_t)(q0 + g) * D + sub * 8);
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
  }
  Kh += sub * 8;
  Vh += sub * 8;

  for (int base = lo; base < hi; base += stride) {
    uint4 kv[U], vv[U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = base + u * RW + rg;
      live[u] = r < hi;
      const size_t off = (size_t)(live[u] ? r : (hi - 1)) * row_stride;
      kv[u] = STREAM ? load_stream(reinterpret_cast<const uint4*>(Kh + off)) : *reinterpret_cast<const uint4*>(Kh + off);
      vv[u] = STREAM ? load_stream(reinterpret_cast<const uint4*>(Vh + off)) : *reinterpret_cast<const uint4*>(Vh + off);
    }
    float s[U][G];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float d = dot8(qp[g], kv[u]);
        if (LPR == 8) d = group8_sum(d);
        else if (LPR == 16) d = group16_sum(d);
        else {
          d = group16_sum(d);
          d += __shfl_xor(d, 16, 64);
          if (LPR == 64) d += __shfl_xor(d, 32, 64);
        }
        s[u][g] = live[u] ? d * scale_log2 : -INFINITY;
      }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mx = m[g];
#pragma unroll
      for (int u = 0; u < U; ++u) mx = fmaxf(mx, s[u][g]);
      // A lane group whose rows are all past the end keeps -inf; exp2(-inf - 0) = 0.
      const float ref = (mx == -INFINITY) ? 0.f : mx;
      float p[U];
      float ps = 0.f;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        p[u] = fast_exp2(s[u][g] - ref);
        ps += p[u];
      }
      // The running sums are rescaled only on the steps where some lane's maximum moved: after a
      // cache's first rows that is rare, and the rescaling is a third of a step's arithmetic.
      if (__builtin_amdgcn_ballot_w64(mx != m[g]) != 0) {
        const float alpha = fast_exp2(m[g] - ref);
        l[g] *= alpha;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] *= alpha;
      }
      l[g] += ps;
      m[g] = mx;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float vf[8];
        unpack8(vv[u], vf);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = fmaf(p[u], vf[i], acc[g][i]);
      }
    }
  }

  // Merge the RW lane groups of the wave (lanes that share `sub`).
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int o = LPR; o < 64; o <<= 1) {
      const float mo = __shfl_xor(m[g], o, 64);
      const float lo2 = __shfl_xor(l[g], o, 64);
      const float mx = fmaxf(m[g], mo);
      const float ref = (mx == -INFINITY) ? 0.f : mx;
      const float a = exp2f(m[g] - ref), b = exp2f(mo - ref);
      l[g] = l[g] * a + lo2 * b;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float ao = __shfl_xor(acc[g][i], o, 64);
        acc[g][i] = acc[g][i] * a + ao * b;
      }
      m[g] = mx;
    }
  }
}

template <int D, int G, int U>
__global__ __launch_bounds__(256) void mha_decode_kernel(
    const bf16_t* __restrict__ Q, const bf16_t* __restrict__ K, const bf16_t* __restrict__ V,
    float* __restrict__ part, int kv_len, float scale_log2, int window, long row_stride,
    long head_stride, const int* __restrict__ kv_valid, const int* __restrict__ kv_first, int kv_rows) {
  constexpr int LPR = D / 8, RW = 64 / LPR;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPR, rg = lane / LPR;
  // KV heads vary fastest over the grid: blocks that run together then read whole cache rows between
  // them (all 1 KB of a row of 8 heads), not one head's 128 bytes of every row, which would keep a
  // fraction of the memory channels busy and leave the rest idle.
  const int split = blockIdx.y, nsplit = gridDim.y, kvh = blockIdx.x;
  if (kv_first) {   // the keys are a window of a longer buffer, rows *kv_first on (held inside it)
    const long first_row = max(0, min(*kv_first, kv_rows - kv_len));
    K += first_row * row_stride;
    V += first_row * row_stride;
  }

  const int kv_tokens = bound_or(kv_valid, kv_len);
  const int first = (window >= 0) ? max(0, kv_tokens - 1 - window) : 0;
  const int n = kv_tokens - first;
  // Slice of this block, in whole wave-steps so that waves split it evenly.
  int chunk = (n + nsplit - 1) / nsplit;
  chunk = (chunk + 4 * RW - 1) / (4 * RW) * (4 * RW);
  const int blo = first + split * chunk;
  const int wlo = blo + wave * (chunk / 4);
  const int whi = min(min(wlo + chunk / 4, blo + chunk), kv_tokens);

  float m[G], l[G], acc[G][8];
  decode_scan<D, G, U, true>(Q, K + (size_t)kvh * head_stride, V + (size_t)kvh * head_stride, kvh * G, wlo, whi,
                    U * RW, row_stride, scale_log2, m, l, acc);

  // Merge the 4 waves through LDS; wave 0 writes the block's partial.
  __shared__ float sm[4][G];
  __shared__ float sl[4][G];
  __shared__ float sacc[4][G][D];
  if (rg == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (sub == 0) {
        sm[wave][g] = m[g];
        sl[wave][g] = l[g];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) sacc[wave][g][sub * 8 + i] = acc[g][i];
    }
  }
  __syncthreads();
  // part layout: [head][split][D + 2] = {m, l, acc[D]}.
  for (int idx = threadIdx.x; idx < G * D; idx += 256) {
    const int g = idx / D, dd = idx % D;
    float mx = fmaxf(fmaxf(sm[0][g], sm[1][g]), fmaxf(sm[2][g], sm[3][g]));
    const float ref = (mx == -INFINITY) ? 0.f : mx;
    float lt = 0.f, at = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float e = exp2f(sm[w][g] - ref);
      lt += sl[w][g] * e;
      at += sacc[w][g][dd] * e;
    }
    float* out = part + ((size_t)(kvh * G + g) * nsplit + split) * (D + 2);
    out[2 + dd] = at;
    if (dd == 0) {
      out[0] = mx;
      out[1] = lt;
    }
  }
}

// One block per head merges the splits: thread s < nsplit turns split s's (m, l) into a weight
// in LDS, then thread dd sums column dd over the splits with independent (unrolled) loads.
template <int D>
__global__ void mha_decode_merge_kernel(const float* __restrict__ part, bf16_t* __restrict__ O,
                                        int nsplit) {
  __shared__ float wgt[kMaxSplits];
  __shared__ float red[2][4];
  const int head = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const float* p = part + (size_t)head * nsplit * (D + 2);
  float m = -INFINITY, l = 0.f;
  if (t < nsplit) {
    m = p[t * (D + 2)];
    l = p[t * (D + 2) + 1];
  }
  float mx = wave_max(m);
  if (lane == 0) red[0][wave] = mx;
  __syncthreads();
  mx = -INFINITY;
  for (int w = 0; w < (int)(blockDim.x >> 6); ++w) mx = fmaxf(mx, red[0][w]);
  const float ref = (mx == -INFINITY) ? 0.f : mx;
  const float e = exp2f(m - ref);  // 0 for the lanes past nsplit (m = -inf)
  if (t < nsplit) wgt[t] = e;
  float ls = wave_sum(l * e);
  if (lane == 0) red[1][wave] = ls;
  __syncthreads();
  float lt = 0.f;
  for (int w = 0; w < (int)(blockDim.x >> 6); ++w) lt += red[1][w];
  if (t < D) {
    float at = 0.f;
#pragma unroll 8
    for (int s = 0; s < nsplit; ++s) at = fmaf(p[s * (D + 2) + 2 + t], wgt[s], at);
    O[(size_t)head * D + t] = f32_to_bf16(lt > 0.f ? at / lt : 0.f);
  }
}

// Short caches: one block of 16 waves per query head scans the whole cache (wave w takes every
// 16th run of 8 steps), merges its waves through LDS and writes the output row itself -- one
// launch, no partials.  Blocks b and b + kv_heads serve the same KV head; with kv_heads a multiple
// of 8 they sit on one XCD and share its L2.
template <int D>
__global__ __launch_bounds__(1024) void mha_decode_single_kernel(
    const bf16_t* __restrict__ Q, const bf16_t* __restrict__ K, const bf16_t* __restrict__ V,
    bf16_t* __restrict__ O, int kv_len, int kv_heads, int group, float scale_log2, int window,
    long row_stride, long head_stride, const int* __restrict__ kv_valid, const int* __restrict__ kv_first,
    int kv_rows) {
  constexpr int LPR = D / 8, RW = 64 / LPR, WAVES = 16, U = 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPR, rg = lane / LPR;
  const int kvh = blockIdx.x % kv_heads, head = kvh * group + blockIdx.x / kv_heads;
  if (kv_first) {   // the keys are a window of a longer buffer, rows *kv_first on (held inside it)
    const long first_row = max(0, min(*kv_first, kv_rows - kv_len));
    K += first_row * row_stride;
    V += first_row * row_stride;
  }

  const int kv_tokens = bound_or(kv_valid, kv_len);
  const int first = (window >= 0) ? max(0, kv_tokens - 1 - window) : 0;

  float m[1], l[1], acc[1][8];
  decode_scan<D, 1, U, false>(Q, K + (size_t)kvh * head_stride, V + (size_t)kvh * head_stride, head,
                    first + wave * U * RW, kv_tokens, WAVES * U * RW, row_stride, scale_log2, m, l, acc);

  __shared__ float sm[WAVES];
  __shared__ float sl[WAVES];
  __shared__ float sacc[WAVES][D];
  if (rg == 0) {
    if (sub == 0) {
      sm[wave] = m[0];
      sl[wave] = l[0];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) sacc[wave][sub * 8 + i] = acc[0][i];
  }
  __syncthreads();
  if (threadIdx.x < D) {
    const int dd = threadIdx.x;
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, sm[w]);
    const float ref = (mx == -INFINITY) ? 0.f : mx;
    float lt = 0.f, at = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float e = exp2f(sm[w] - ref);
      lt += sl[w] * e;
      at += sacc[w][dd] * e;
    }
    O[(size_t)head * D + dd] = f32_to_bf16(lt > 0.f ? at / lt : 0.f);
  }
}

// Many queries, a block a (query row, head): the same scan as above per query, over the keys its
// mask leaves.  The shapes the MFMA prompt kernel does not take (512-wide heads: a 512-wide pair of
// K and V tiles does not fit its stage buffers and registers); what a row costs is its keys' bytes.
template <int D>
__global__ __launch_bounds__(1024) void mha_prefill_rows_kernel(
    const bf16_t* __restrict__ Q, const bf16_t* __restrict__ K, const bf16_t* __restrict__ V,
    bf16_t* __restrict__ O, int group, int seq, int seq_len, int kv_len, float scale_log2, int causal,
    int window, long q_row_stride, long q_head_stride, long kv_row_stride, long kv_head_stride,
    const int* __restrict__ valid, const int* __restrict__ kv_valid, const int* __restrict__ kv_first, int kv_rows) {
  constexpr int LPR = D / 8, RW = 64 / LPR, WAVES = 16, U = 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPR, rg = lane / LPR;
  const int head = blockIdx.x, row = blockIdx.y, kvh = head / group;
  if (kv_first) {   // the keys are a window of a longer buffer, rows *kv_first on (held inside it)
    const long first_row = max(0, min(*kv_first, kv_rows - kv_len));
    K += first_row * kv_row_stride;
    V += first_row * kv_row_stride;
  }

  const int q_tokens = valid ? bound_or(valid, seq) : seq_len;
  const int kv_tokens = kv_valid ? bound_or(kv_valid, kv_len) : (kv_len - seq + q_tokens);
  const bool masked = causal || window >= 0;
  const int offset = masked ? (kv_tokens - q_tokens) : 0;
  bf16_t* out = O + (size_t)head * q_head_stride + (size_t)row * q_row_stride;
  if (row >= q_tokens || offset < 0) {   // a row past the bound: zeros
    if (threadIdx.x < D) out[threadIdx.x] = 0;
    return;
  }
  const int qpos = offset + row;
  int hi = kv_tokens, lo = 0;
  if (causal) hi = min(hi, qpos + 1);
  else if (window >= 0) hi = min(hi, qpos + window + 1);
  if (window >= 0) lo = max(0, qpos - window);

  float m[1], l[1], acc[1][8];
  decode_scan<D, 1, U, false>(Q + (size_t)head * q_head_stride + (size_t)row * q_row_stride,
                              K + (size_t)kvh * kv_head_stride, V + (size_t)kvh * kv_head_stride, 0,
                              lo + wave * U * RW, hi, WAVES * U * RW, kv_row_stride, scale_log2, m, l, acc);

  __shared__ float sm[WAVES];
  __shared__ float sl[WAVES];
  __shared__ float sacc[WAVES][D];
  if (rg == 0) {
    if (sub == 0) {
      sm[wave] = m[0];
      sl[wave] = l[0];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) sacc[wave][sub * 8 + i] = acc[0][i];
  }
  __syncthreads();
  if (threadIdx.x < D) {
    const int dd = threadIdx.x;
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, sm[w]);
    const float ref = (mx == -INFINITY) ? 0.f : mx;
    float lt = 0.f, at = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float e = exp2f(sm[w] - ref);
      lt += sl[w] * e;
      at += sacc[w][dd] * e;
    }
    out[dd] = f32_to_bf16(lt > 0.f ? at / lt : 0.f);
  }
}

int launch_prefill_rows512(const bf16_t* Q, const bf16_t* K, const bf16_t* V, bf16_t* O, int heads, int group,
                           int seq, int seq_len, int kv_len, float scale_log2, int causal, int window,
                           long q_row_stride, long q_head_stride, long kv_row_stride, long kv_head_stride,
                           const int* valid, const int* kv_valid, const int* kv_first, int kv_rows, void* stream) {
  hipLaunchKernelGGL(mha_prefill_rows_kernel<512>, dim3(heads, seq), dim3(1024), 0, (hipStream_t)stream, Q, K, V, O,
                     group, seq, seq_len, kv_len, scale_log2, causal, window, q_row_stride, q_head_stride,
                     kv_row_stride, kv_head_stride, valid, kv_valid, kv_first, kv_rows);
  return 0;
}

template <int D, int G>
static void launch_decode(const bf16_t* Q, const bf16_t* K, const bf16_t* V, bf16_t* O, float* part,
                          int kv_heads, int kv_len, float scale_log2, int window, long row_stride,
                          long head_stride, const int* kv_valid, const int* kv_first, int kv_rows, int nsplit,
                          hipStream_t s) {
  // A wave's share of its block's slice in one pass where it fits eight steps (every byte of the
  // cache is then requested before any is needed), else four steps a pass.
  constexpr int RW = 64 / (D / 8);
  if (D <= 128 && G <= 4 && (kv_len + nsplit - 1) / nsplit > 4 * 4 * RW)
    hipLaunchKernelGGL((mha_decode_kernel<D, G, 8>), dim3(kv_heads, nsplit), dim3(256), 0, s, Q, K, V,
                       part, kv_len, scale_log2, window, row_stride, head_stride, kv_valid, kv_first, kv_rows);
  else
    hipLaunchKernelGGL((mha_decode_kernel<D, G, 4>), dim3(kv_heads, nsplit), dim3(256), 0, s, Q, K, V,
                       part, kv_len, scale_log2, window, row_stride, head_stride, kv_valid, kv_first, kv_rows);
  hipLaunchKernelGGL((mha_decode_merge_kernel<D>), dim3(kv_heads * G), dim3(D > kMaxSplits ? D : kMaxSplits), 0, s,
                     part, O, nsplit);
}

}  // namespace iron

using namespace iron;

extern "C" int64_t iron_mha_decode_workspace_bytes(int heads, int d) {
  return (int64_t)heads * kMaxSplits * (d + 2) * sizeof(float);
}

static int mha_decode(const uint16_t* Q, const uint16_t* K, const uint16_t* V, uint16_t* O, int heads, int kv_heads,
                      int d, int kv_len, float scale, int window, int kv_interleaved, const int* kv_valid,
                      const int* kv_first, int kv_rows, void* workspace, void* stream) {
  IRON_REQUIRE(Q && K && V && O && workspace, "mha_decode: null operand");
  IRON_REQUIRE(kv_first == nullptr || (kv_interleaved && kv_rows >= kv_len),
               "mha_decode: a window of the keys takes them row by row (kv_interleaved) out of kv_rows (%d) >= kv_len (%d)",
               kv_rows, kv_len);
  IRON_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
               "mha_decode: heads (%d) must be a positive multiple of kv_heads (%d)", heads, kv_heads);
  IRON_REQUIRE(kv_len > 0, "mha_decode: kv_len (%d) must be positive", kv_len);
  IRON_REQUIRE(scale >= 0.f && scale < INFINITY, "mha_decode: scale must be finite and not negative");
  IRON_REQUIRE((((uintptr_t)Q | (uintptr_t)K | (uintptr_t)V | (uintptr_t)workspace) & 15) == 0,
               "mha_decode: operands must be 16-byte aligned");
  const int G = heads / kv_heads;
  const long row_stride = kv_interleaved ? (long)kv_heads * d : d;
  const long head_stride = kv_interleaved ? d : (long)kv_len * d;
  // Measured: a split per 128 keys, at least 8 (short caches are launch-bound) and at most 64
  // (beyond that the merge of the splits costs more than the extra parallelism gains).
  int nsplit = (kv_len + 127) / 128;
  nsplit = nsplit < 8 ? 8 : (nsplit > 64 ? 64 : nsplit);
  if (kv_len > 64 * 256) nsplit = (kv_len + 255) / 256 > kMaxSplits ? kMaxSplits : (kv_len + 255) / 256;
  if (nsplit * 8 > kv_len) nsplit = kv_len >= 8 ? kv_len / 8 : 1;
  const float scale_log2 = scale * 1.4426950408889634f;
  hipStream_t s = (hipStream_t)stream;
  float* part = (float*)workspace;
  // Caches this short are launch-bound: one launch that needs no merge of splits.
  // ... and 512-wide heads take it at any length (no split kernel is built for them).
  if ((kv_len <= kSingleMaxKeys && (d == 64 || d == 128 || d == 256)) || d == 512) {
    const dim3 grid(heads), block(1024);
    if (d == 512)
      hipLaunchKernelGGL(mha_decode_single_kernel<512>, grid, block, 0, s, Q, K, V, O, kv_len, kv_heads, G,
                         scale_log2, window, row_stride, head_stride, kv_valid, kv_first, kv_rows);
    else if (d == 64)
      hipLaunchKernelGGL(mha_decode_single_kernel<64>, grid, block, 0, s, Q, K, V, O, kv_len, kv_heads, G,
                         scale_log2, window, row_stride, head_stride, kv_valid, kv_first, kv_rows);
    else if (d == 128)
      hipLaunchKernelGGL(mha_decode_single_kernel<128>, grid, block, 0, s, Q, K, V, O, kv_len, kv_heads, G,
                         scale_log2, window, row_stride, head_stride, kv_valid, kv_first, kv_rows);
    else
      hipLaunchKernelGGL(mha_decode_single_kernel<256>, grid, block, 0, s, Q, K, V, O, kv_len, kv_heads, G,
                         scale_log2, window, row_stride, head_stride, kv_valid, kv_first, kv_rows);
    IRON_LAUNCH_CHECK();
  }
#define IRON_DEC(DD, GG)                                                                        \
  if (d == DD && G == GG) {                                                                     \
    launch_decode<DD, GG>(Q, K, V, O, part, kv_heads, kv_len, scale_log2, window, row_stride,   \
                          head_stride, kv_valid, kv_first, kv_rows, nsplit, s);                 \
    IRON_LAUNCH_CHECK();                                                                        \
  }
#define IRON_DEC_D(DD) \
  IRON_DEC(DD, 1) IRON_DEC(DD, 2) IRON_DEC(DD, 3) IRON_DEC(DD, 4) IRON_DEC(DD, 5) IRON_DEC(DD, 6) IRON_DEC(DD, 8)
  IRON_DEC_D(64) IRON_DEC_D(128) IRON_DEC_D(256)
#undef IRON_DEC_D
#undef IRON_DEC
  IRON_REQUIRE(false, "mha_decode: no kernel for d=%d with %d query heads per KV head "
               "(d in {64,128,256} with a group in {1,2,3,4,5,6,8}, or d = 512)", d, G);
}

extern "C" int iron_mha_decode_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                    uint16_t* O, int heads, int kv_heads, int d, int kv_len,
                                    float scale, int window, int kv_interleaved,
                                    const int* kv_valid, void* workspace, void* stream) {
  return mha_decode(Q, K, V, O, heads, kv_heads, d, kv_len, scale, window, kv_interleaved, kv_valid, nullptr, 0,
                    workspace, stream);
}

// ---- the entry point that allocates nothing
//
// The split kernel's partial results in device memory the library itself holds: a file-scope array,
// one copy per GPU, there from the moment the code object is loaded until the process ends.  In host
// code the array's name is only a handle for hipGetSymbolAddress, never an address: the device
// address is asked for once per device, with that device current, and kept.
namespace iron {
constexpr int64_t kScratchBytes = 8 << 20;
constexpr int kScratchDevices = 64;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
static void* scratch_ptr[kScratchDevices];     // per device: the array's address there
static std::mutex scratch_mutex;

// The current device's copy of the array, or null with the reason set.
static void* scratch_here() {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess || device < 0 || device >= kScratchDevices) {
    set_error("mha_decode_static: no current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "index out of range");
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(scratch_mutex);
  if (scratch_ptr[device] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      set_error("mha_decode_static: the scratch array has no address on device %d (%s)", device, hipGetErrorString(e));
      return nullptr;
    }
    scratch_ptr[device] = p;
  }
  return scratch_ptr[device];
}
}  // namespace iron

extern "C" int64_t iron_mha_decode_static_max_bytes(void) { return kScratchBytes; }

extern "C" int iron_mha_decode_static_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                           uint16_t* O, int heads, int kv_heads, int d, int kv_len,
                                           float scale, int window, int kv_interleaved,
                                           const int* kv_valid, void* stream) {
  IRON_REQUIRE(heads > 0 && d > 0, "mha_decode_static: heads (%d) and d (%d) must be positive", heads, d);
  const int64_t need = iron_mha_decode_workspace_bytes(heads, d);
  IRON_REQUIRE(need <= kScratchBytes,
               "mha_decode_static: %d heads of width %d need %lld bytes of partial results; the library's own "
               "scratch holds %lld (use iron_mha_decode_bf16 with a workspace of the caller's)",
               heads, d, (long long)need, (long long)kScratchBytes);
  void* ws = scratch_here();
  if (ws == nullptr) return IRON_EINVAL;
  return mha_decode(Q, K, V, O, heads, kv_heads, d, kv_len, scale, window, kv_interleaved, kv_valid, nullptr, 0, ws,
                    stream);
}

extern "C" int iron_mha_decode_at_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                       uint16_t* O, int heads, int kv_heads, int d, int kv_len,
                                       float scale, int window, const int* kv_valid, const int* kv_first,
                                       int kv_rows, void* workspace, void* stream) {
  IRON_REQUIRE(kv_first != nullptr, "mha_decode_at: null kv_first");
  return mha_decode(Q, K, V, O, heads, kv_heads, d, kv_len, scale, window, 1, kv_valid, kv_first, kv_rows, workspace,
                    stream);
}
