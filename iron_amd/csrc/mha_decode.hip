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
#include <type_traits>

namespace iron {

constexpr int kMaxSplits = 128;      // what the workspace holds per head
constexpr int kScanMaxSplits = 128;  // the lane-scan kernels' own limit
constexpr int kSingleMaxKeys = 2048;  // lane-scan kernels: caches up to this many rows take the one-launch kernel
// One-shape launch: up to this many live keys one block a query head writes O itself.  Where the two
// forms cost the same inside that launch shape (32 / 8 heads of 64, an 8192-row cache, us at 1024 /
// 1280 / 1536 / 2048 live keys: one block a head 8.0 / 8.8 / 9.7 / 12.1, split + merge 9.0 / 9.0 /
// 9.0 / 9.5).
constexpr int kShortKeys = 1408;
constexpr int kComputeUnits = 256;    // MI355X: what the split count is sized for

// 2^x for x <= 0 by the hardware's own instruction: a softmax weight small enough to be a denormal
// counts as 0, which saves the library routine's rescaling around every call.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// f(x of this lane, x of lane ^ SPAN) for SPAN = 16 or 32: the swap leaves one of the two in each
// operand (which is which depends on the lane's side; f is symmetric).
template <int SPAN, typename F>
__device__ __forceinline__ float across_rows(float x, F f) {
  float a = x, b = x;
  if (SPAN == 16) asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  else asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return f(a, b);
}

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
    // Every key row of the pass is asked for before any value row: a CU's address path takes a
    // block's loads one after another (16 cycles each), and the scores and their exponentials then
    // run while the value rows are still on their way.
    uint4 kv[U], vv[U];
    bool live[U];
    size_t off[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = base + u * RW + rg;
      live[u] = r < hi;
      off[u] = (size_t)(live[u] ? r : (hi - 1)) * row_stride;
      kv[u] = STREAM ? load_stream(reinterpret_cast<const uint4*>(Kh + off[u])) : *reinterpret_cast<const uint4*>(Kh + off[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      vv[u] = STREAM ? load_stream(reinterpret_cast<const uint4*>(Vh + off[u])) : *reinterpret_cast<const uint4*>(Vh + off[u]);
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

  // Merge the RW lane groups of the wave (lanes that share `sub`): the maximum over them first, one
  // rescaling of a group's sums to it, then plain sums -- lane ^ 8 by a DPP rotation inside the row,
  // lane ^ 16 and lane ^ 32 by the row and half swaps, no trip through LDS (as three rounds of
  // shuffled (max, sum, columns) with two exponentials each, this tail was a tenth of the launch at
  // a few hundred keys).
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float mw = m[g];
    if (LPR <= 8) mw = fmaxf(mw, IRON_DPP(0.f, mw, 0x128, 0xF));   // row_ror:8
    if (LPR <= 16) mw = across_rows<16>(mw, [](float a, float b) { return fmaxf(a, b); });
    if (LPR <= 32) mw = across_rows<32>(mw, [](float a, float b) { return fmaxf(a, b); });
    const float ref = (mw == -INFINITY) ? 0.f : mw;
    const float a = fast_exp2(m[g] - ref);   // 0 for a group that saw no key
    float v[9];
    v[8] = l[g] * a;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = acc[g][i] * a;
#pragma unroll
    for (int i = 0; i < 9; ++i) {
      if (LPR <= 8) v[i] += IRON_DPP(0.f, v[i], 0x128, 0xF);
      if (LPR <= 16) v[i] = across_rows<16>(v[i], [](float a, float b) { return a + b; });
      if (LPR <= 32) v[i] = across_rows<32>(v[i], [](float a, float b) { return a + b; });
    }
    l[g] = v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = v[i];
    m[g] = mw;
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
      const float e = fast_exp2(sm[w][g] - ref);
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
  __shared__ float wgt[kScanMaxSplits];
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
  const float e = fast_exp2(m - ref);  // 0 for the lanes past nsplit (m = -inf)
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
      const float e = fast_exp2(sm[w] - ref);
      lt += sl[w] * e;
      at += sacc[w][dd] * e;
    }
    O[(size_t)head * D + dd] = f32_to_bf16(lt > 0.f ? at / lt : 0.f);
  }
}

// The run of keys a block of the split scan takes: an equal share of the live keys, in whole
// 16-key tiles for each of the 2^share_log2 waves that work on one KV head.  The scan and the merge
// both derive it from the same words.
__device__ __forceinline__ int decode_chunk(int live, int nsplit, int share_log2) {
  const int unit = 16 << share_log2;
  return ((live + nsplit - 1) / nsplit + unit - 1) & ~(unit - 1);
}

// ---- one query, one launch shape whatever the cache's length
//
// grid = (sets, nsplit) blocks of WAVES waves, as many as the chip has CUs; the blocks choose what to
// do by the live keys n = *kv_valid (less what a window drops), so the work and its spread over the
// chip follow the context and the cache only sizes the buffers.
//
// n <= short_keys: the first `heads` blocks each scan all keys for one query head with the
// lane-per-column scan above (16 waves a head: the launch is latency-bound, and this is the shortest
// chain) and write the output row; the others leave at once, and so does the merge launch behind.
//
// Otherwise the keys are dealt over the nsplit blocks of a set of KV heads in equal runs sized by n,
// and a block leaves (max, sum, O) per head for the merge.  Here the G query heads that share a KV
// head are the columns of a 16-wide MFMA tile (G <= 16; the rest are zero columns), so a key row is
// multiplied with all of them by one instruction stream whatever G is.  A wave works through its own
// run of keys 32 at a time.  S^T = K Q^T (M = keys, N = heads): the K rows are the A operand exactly
// as they lie in memory (lane -> key row lane % 16, 16-byte piece lane / 16 of a 32-wide k-step), so
// they go from global memory straight into registers.  A lane then owns one head column: the softmax
// is in-lane but for the maximum over the four lanes of a column, which is only exchanged on the
// (rare) steps where some lane's own maximum passes the column's reference.  The probabilities,
// rounded to bf16, are already the B operand of O^T = V^T P^T; V^T comes from the transposing LDS read
// of the wave's own 32-row V tile, which buffer loads put there as stored (16-byte chunks
// XOR-swizzled by 2 (row & 3), as the prompt kernel's).  Rows past the last live key lie outside the
// buffers and read as zeros.
template <int D, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void mha_decode_either_kernel(
    const bf16_t* __restrict__ Q, const bf16_t* __restrict__ K, const bf16_t* __restrict__ V,
    bf16_t* __restrict__ O, float* __restrict__ part, int kv_heads, int group, int hpb_log2, int kv_len,
    float scale_log2, int window, long row_stride, long head_stride, const int* __restrict__ kv_valid,
    const int* __restrict__ kv_first, int kv_rows, int short_keys) {
  constexpr int ROWB = D * 2;            // bytes of a V row in LDS
  constexpr int KS = D / 32;             // 32-wide k-steps of S^T
  constexpr int DT = D / 16;             // 16-row tiles of O^T
  constexpr int CPR = D / 8;             // 16-byte chunks of a row
  constexpr int TK = 32;                 // keys a step
  constexpr int TILE = TK * ROWB;        // bytes of a V tile
  constexpr int VINST = TILE / 1024;     // 1 KB loads into LDS a tile
  constexpr int RPI = 1024 / ROWB;       // rows one of them covers
  constexpr int WAVES_LOG2 = WAVES == 16 ? 4 : 3;
  static_assert(WAVES == 16 || WAVES == 8, "waves a block");
  extern __shared__ __align__(1024) char smem_dec[];   // WAVES x 2 x TILE bytes

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nsplit = gridDim.y;

  const int kv_tokens = bound_or(kv_valid, kv_len);
  const int first = (window >= 0) ? max(0, kv_tokens - 1 - window) : 0;
  const int live = kv_tokens - first;
  const long first_row = kv_first ? max(0, min(*kv_first, kv_rows - kv_len)) : 0;

  if (live <= short_keys) {
    // ---- few keys: block b is one query head, as mha_decode_single_kernel
    constexpr int LPR = D / 8, RW = 64 / LPR, U = 8;
    const int b = blockIdx.y * gridDim.x + blockIdx.x;
    if (b >= kv_heads * group) return;
    const int kvh = b % kv_heads, head = kvh * group + b / kv_heads;
    const int sub = lane % LPR, rg = lane / LPR;
    const bf16_t* Kh = K + (size_t)kvh * head_stride + first_row * row_stride;
    const bf16_t* Vh = V + (size_t)kvh * head_stride + first_row * row_stride;
    float m[1], l[1], acc[1][8];
    decode_scan<D, 1, U, false>(Q, Kh, Vh, head, first + wave * U * RW, kv_tokens, WAVES * U * RW, row_stride,
                                scale_log2, m, l, acc);
    float* sm = reinterpret_cast<float*>(smem_dec);   // [WAVES] maxima, [WAVES] sums, [WAVES][D] columns
    float* sl = sm + WAVES;
    float* sacc = sl + WAVES;
    if (rg == 0) {
      if (sub == 0) {
        sm[wave] = m[0];
        sl[wave] = l[0];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) sacc[wave * D + sub * 8 + i] = acc[0][i];
    }
    __syncthreads();
    if (tid < D) {
      float mx = -INFINITY;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, sm[w]);
      const float ref = (mx == -INFINITY) ? 0.f : mx;
      float lt = 0.f, at = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        const float e = fast_exp2(sm[w] - ref);
        lt += sl[w] * e;
        at += sacc[w * D + tid] * e;
      }
      O[(size_t)head * D + tid] = f32_to_bf16(lt > 0.f ? at / lt : 0.f);
    }
    return;
  }

  // ---- many keys: the block takes one run of them for 2^hpb_log2 KV heads at once, wave w on head
  // w % hpb (with the heads interleaved in a cache row, the block's loads then cover longer pieces of it).
  const int n = lane & 15, q = lane >> 4;   // head column, quarter of the k slots
  const int hpb = 1 << hpb_log2, share_log2 = WAVES_LOG2 - hpb_log2;
  const int split = blockIdx.y;
  const int kvh = (blockIdx.x << hpb_log2) + (wave & (hpb - 1));
  const int sub = wave >> hpb_log2;          // this wave's place among the 2^share_log2 on its head
  const int chunk = decode_chunk(live, nsplit, share_log2);
  const int blo = first + split * chunk, bhi = min(blo + chunk, kv_tokens);
  if (blo >= kv_tokens) return;   // the merge reads the splits that hold keys, no more
  // The wave's run of keys, in whole 16-key MFMA tiles.
  const int per = ((((bhi - blo) + (1 << share_log2) - 1) >> share_log2) + 15) & ~15;
  const int wlo = blo + sub * per, whi = min(wlo + per, bhi);
  const int steps = wlo < whi ? (whi - wlo + TK - 1) / TK : 0;

  const bf16_t* Kh = K + (size_t)kvh * head_stride + first_row * row_stride;
  const bf16_t* Vh = V + (size_t)kvh * head_stride + first_row * row_stride;
  const int row_bytes = (int)row_stride * 2;
  // The head's keys (values) up to the last of this wave's run are one buffer: rows past it -- the
  // next wave's, or past the last live key -- read as zeros and cost no traffic.
  const int reach = wlo < whi ? (whi - 1) * row_bytes + ROWB : 0;
  const __amdgpu_buffer_rsrc_t k_rows = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(Kh), 0, reach, 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rows = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(Vh), 0, reach, 0x00020000);

  // K fragments: tile t of the step, k-step s -> key 16 t + n, bytes 64 s + 16 q of its row.
  const int k_lane = n * row_bytes + 16 * q;
  // V into LDS: load i covers tile rows i RPI + lane / CPR; a lane fetches the logical chunk that the
  // row's swizzle maps to its physical one.
  int v_lane[VINST];
#pragma unroll
  for (int i = 0; i < VINST; ++i) {
    const int r = i * RPI + lane / CPR;
    v_lane[i] = r * row_bytes + (((lane % CPR) ^ ((r & 3) << 1)) << 4);
  }
  char* stage = smem_dec + wave * (2 * TILE);

  bf16x8 kf[2][2][KS];   // [register set][tile][k-step]
  auto issue_v = [&](int step, int set) {
    const int at = (wlo + step * TK) * row_bytes;
#pragma unroll
    for (int i = 0; i < VINST; ++i)
      // (the cast keeps the offset's type from depending on the template: as a dependent expression
      // the host pass drops the kernel's stub without a word)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rows, IRON_LDS_PTR(stage + set * TILE + i * 1024), 16,
                                               (int)v_lane[i] + at, 0, 0, 0);
  };
  auto issue = [&](int step, auto set_c) {
    constexpr int set = decltype(set_c)::value;
    const int at = (wlo + step * TK) * row_bytes;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int s = 0; s < KS; ++s)
        kf[set][t][s] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(
            k_rows, at + k_lane + t * 16 * row_bytes + 64 * s, 0, 0));
  };
  // Steps go in pairs: both steps' loads are out before either is waited for, and the next pair's go
  // out as each of this pair's register set and stage buffer falls free.  The wait is for everything
  // in flight, so it needs no count of what the compiler may have moved.
  using set0 = std::integral_constant<int, 0>;
  using set1 = std::integral_constant<int, 1>;
  if (steps > 0) {
    issue_v(0, 0);
    issue(0, set0{});
  }
  if (steps > 1) {
    issue_v(1, 1);
    issue(1, set1{});
  }

  // Q^T fragments (B operand): lane holds head column n, d = 32 s + 8 q .. + 7; zero columns past G.
  bf16x8 qf[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (n < group) v = *reinterpret_cast<const uint4*>(Q + (size_t)(kvh * group + n) * D + 32 * s + 8 * q);
    qf[s] = __builtin_bit_cast(bf16x8, v);
  }
  // V^T fragments (A operand of O^T): the lanes of quarter q point at rows 4 q + 0..3 (k slots 8 q + 0..3;
  // the same 16 rows on for slots 8 q + 4..7, as S^T's second tile lies in P), 4 columns each of the 16.
  const int v_swz = ((lane >> 2) & 3) << 1;
  unsigned v_frag[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    v_frag[dt] = (unsigned)(size_t)IRON_LDS_PTR(stage) + (4 * q + ((lane & 15) >> 2)) * ROWB +
                 (((2 * dt + ((lane & 3) >> 1)) ^ v_swz) << 4) + ((lane & 1) << 3);

  f32x4 oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_ref = -INFINITY, l_run = 0.f;   // the column's reference maximum (raw scores), this lane's sum

  auto compute = [&](int step, auto set_c) {
    constexpr int set = decltype(set_c)::value;
    TrFrag vf[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      vf[dt].lo = lds_read_tr16_at<set * TILE>(v_frag[dt]);
      vf[dt].hi = lds_read_tr16_at<set * TILE + 16 * ROWB>(v_frag[dt]);
    }
    f32x4 sacc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      sacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; ++s) sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[set][t][s], qf[s], sacc[t], 0, 0, 0);
    }
    // Element i of tile t is key k0 + 16 t + 4 q + i; the wave's last step may reach past its run.
    const int k0 = wlo + step * TK;
    const int left = whi - k0 - 4 * q;   // keys of this lane's tile-0 quarter inside the run (may be <= 0)
    const bool edge = k0 + TK > whi;
    if (edge) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (16 * t + i >= left) sacc[t][i] = -INFINITY;
    }
    float lm = sacc[0][0];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) lm = fmaxf(lm, sacc[t][i]);
    if (__builtin_amdgcn_ballot_w64(lm > m_ref) != 0) {
      float mx = fmaxf(lm, __shfl_xor(lm, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_ref, mx);
      // A column that had seen no key has zero sums to rescale; one that still has none keeps -inf.
      const float alpha = (m_ref == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_ref - m_new) * scale_log2);
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) oacc[dt][i] *= alpha;
      m_ref = m_new;
    }
    const float mc = (m_ref == -INFINITY) ? 0.f : m_ref * scale_log2;
    float p[8];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float e = __builtin_amdgcn_exp2f(fmaf(sacc[t][i], scale_log2, -mc));
        if (edge && 16 * t + i >= left) e = 0.f;   // also where the scale is 0 and -inf * 0 is no number
        p[4 * t + i] = e;
        l_run += e;
      }
    const bf16x8 pf = __builtin_bit_cast(bf16x8, pack8(p));
#pragma unroll
    for (int dt = 0; dt < DT; dt += 2) {
      lds_tr_wait(vf[dt], vf[dt + 1]);
      oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tr_join(vf[dt]), pf, oacc[dt], 0, 0, 0);
      oacc[dt + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tr_join(vf[dt + 1]), pf, oacc[dt + 1], 0, 0, 0);
    }
  };

  for (int step = 0; step < steps; step += 2) {
    wait_vmcnt<0>();
    compute(step, set0{});
    if (step + 2 < steps) {
      issue_v(step + 2, 0);
      issue(step + 2, set0{});
    }
    if (step + 1 < steps) {
      compute(step + 1, set1{});
      if (step + 3 < steps) {
        issue_v(step + 3, 1);
        issue(step + 3, set1{});
      }
    }
  }
  wait_vmcnt<0>();

  // The lane's sum over its own keys -> the column's.
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);

  // Waves hand (max, sum, O^T column) per head over through LDS (the stage buffers, once every wave
  // is out of its loop); thread (head, pair of d) folds the waves of its KV head, every read issued
  // before the first is used.  Eight bytes a write and a read: at a step or two a wave the launch is
  // as long as its instructions, these among them.
  __syncthreads();
  float* hand = reinterpret_cast<float*>(smem_dec);   // [WAVES][group][D + 2]
  static_assert(16 * (D + 2) * 4 <= 2 * TILE, "a wave's hand-over fits its own stage buffers");
  if (n < group) {
    float* mine = hand + ((size_t)wave * group + n) * (D + 2);
    if (q == 0) *reinterpret_cast<float2*>(mine) = make_float2(m_ref, l_run);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      *reinterpret_cast<float2*>(mine + 2 + 16 * dt + 4 * q) = make_float2(oacc[dt][0], oacc[dt][1]);
      *reinterpret_cast<float2*>(mine + 4 + 16 * dt + 4 * q) = make_float2(oacc[dt][2], oacc[dt][3]);
    }
  }
  __syncthreads();
  // Column hg = (head of the block's, query head of its group) lies in waves hw, hw + hpb, ...: entry
  // hg + j hpb group of the hand-over for j < share.
  const int share = 1 << share_log2;
  const int wave_step = (group << hpb_log2) * (D + 2);
  for (int idx = tid; idx < (group << hpb_log2) * (D / 2); idx += 64 * WAVES) {
    const int hg = idx / (D / 2), pair = idx % (D / 2);
    const float* col = hand + (size_t)hg * (D + 2);
    float2 mlv[WAVES], av[WAVES];
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      mlv[w] = make_float2(-INFINITY, 0.f);
      av[w] = make_float2(0.f, 0.f);
      if (w < share) {   // uniform over the block
        mlv[w] = *reinterpret_cast<const float2*>(col + w * wave_step);
        av[w] = *reinterpret_cast<const float2*>(col + w * wave_step + 2 + 2 * pair);
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, mlv[w].x);
    float lt = 0.f, at0 = 0.f, at1 = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float e = (mlv[w].x == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((mlv[w].x - mx) * scale_log2);
      lt = fmaf(mlv[w].y, e, lt);
      at0 = fmaf(av[w].x, e, at0);
      at1 = fmaf(av[w].y, e, at1);
    }
    // part layout: [head][split][D + 2] = {max in the exp2 domain, sum, O[D]}.
    const int head = (blockIdx.x << hpb_log2) * group + hg;
    float* out = part + ((size_t)head * nsplit + split) * (D + 2);
    *reinterpret_cast<float2*>(out + 2 + 2 * pair) = make_float2(at0, at1);
    if (pair == 0) *reinterpret_cast<float2*>(out) = make_float2((mx == -INFINITY) ? -INFINITY : mx * scale_log2, lt);
  }
}

// The splits' merge, a block of 4 D threads a head: thread (part, pair) sums columns 2 pair and
// 2 pair + 1 over the splits part, part + 8, ... that hold keys, PER of them at a time, and the eight
// parts are folded through LDS.  A thread's first PER are requested together with the bound, before
// it is known how many of them hold anything (the workspace is the caller's own memory, whatever it
// holds): one trip to memory, not two, for up to 8 PER splits (PER = 8 where the launch has at most
// 64 splits, so that no thread asks twice for a split).  Every load is 8 bytes -- a split's maximum
// and sum, or two columns: the launch's time is its load instructions (one column and one word a
// load took 1.3 us longer at 64 splits).  Leaves at once where the scan's blocks wrote the output
// themselves.
template <int D, int PER>
__global__ __launch_bounds__(4 * D) void mha_decode_either_merge_kernel(
    const float* __restrict__ part, bf16_t* __restrict__ O, int nsplit, int share_log2, int kv_len, int window,
    const int* __restrict__ kv_valid, int short_keys) {
  constexpr int PAIRS = D / 2;
  const int head = blockIdx.x, t = threadIdx.x % PAIRS, eighth = threadIdx.x / PAIRS;
  const float* p = part + (size_t)head * nsplit * (D + 2);
  float2 ml[PER], a[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int s = min(eighth + 8 * i, nsplit - 1);
    ml[i] = *reinterpret_cast<const float2*>(p + s * (D + 2));
    a[i] = *reinterpret_cast<const float2*>(p + s * (D + 2) + 2 + 2 * t);
  }
  const int kv_tokens = bound_or(kv_valid, kv_len);
  const int first = (window >= 0) ? max(0, kv_tokens - 1 - window) : 0;
  const int live = kv_tokens - first;
  if (live <= short_keys) return;
  const int chunk = decode_chunk(live, nsplit, share_log2);
  const int used = (live + chunk - 1) / chunk;
  float mx = -INFINITY, lt = 0.f, at0 = 0.f, at1 = 0.f;
  for (int s0 = eighth; s0 < used; s0 += 8 * PER) {
    if (s0 >= 8 * PER) {
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int s = min(s0 + 8 * i, used - 1);
        ml[i] = *reinterpret_cast<const float2*>(p + s * (D + 2));
        a[i] = *reinterpret_cast<const float2*>(p + s * (D + 2) + 2 + 2 * t);
      }
    }
    float cm = mx;
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (s0 + 8 * i < used) cm = fmaxf(cm, ml[i].x);
    const float keep = (mx == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mx - cm);
    lt *= keep;
    at0 *= keep;
    at1 *= keep;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const bool in = s0 + 8 * i < used && ml[i].x != -INFINITY;
      const float e = in ? __builtin_amdgcn_exp2f(ml[i].x - cm) : 0.f;
      lt = fmaf(in ? ml[i].y : 0.f, e, lt);
      at0 = fmaf(in ? a[i].x : 0.f, e, at0);
      at1 = fmaf(in ? a[i].y : 0.f, e, at1);
    }
    mx = cm;
  }
  __shared__ float fm[8][PAIRS], fl[8][PAIRS];
  __shared__ float2 fa[8][PAIRS];
  fm[eighth][t] = mx;
  fl[eighth][t] = lt;
  fa[eighth][t] = make_float2(at0, at1);
  __syncthreads();
  if (eighth != 0) return;
  float top = fm[0][t];
#pragma unroll
  for (int k = 1; k < 8; ++k) top = fmaxf(top, fm[k][t]);
  float ls = 0.f, as0 = 0.f, as1 = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const float e = (fm[k][t] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(fm[k][t] - top);
    ls = fmaf(fl[k][t], e, ls);
    as0 = fmaf(fa[k][t].x, e, as0);
    as1 = fmaf(fa[k][t].y, e, as1);
  }
  const unsigned lo = f32_to_bf16(ls > 0.f ? as0 / ls : 0.f), hi = f32_to_bf16(ls > 0.f ? as1 / ls : 0.f);
  reinterpret_cast<unsigned*>(O + (size_t)head * D)[t] = lo | (hi << 16);
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
  hipLaunchKernelGGL((mha_decode_merge_kernel<D>), dim3(kv_heads * G), dim3(D > kScanMaxSplits ? D : kScanMaxSplits), 0, s,
                     part, O, nsplit);
}


// The one-shape launch and, where the cache can hold more than `short_keys` rows, the merge behind it.
template <int D, int WAVES>
static int launch_decode_either(const bf16_t* Q, const bf16_t* K, const bf16_t* V, bf16_t* O, float* part, int kv_heads,
                                int group, int kv_len, float scale_log2, int window, long row_stride, long head_stride,
                                const int* kv_valid, const int* kv_first, int kv_rows, int short_keys, hipStream_t s) {
  constexpr size_t lds = (size_t)WAVES * 2 * 32 * D * 2;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&mha_decode_either_kernel<D, WAVES>), lds); e != hipSuccess) {
    set_error("mha_decode: %s", hipGetErrorString(e));
    return (int)e;
  }
  // A block of the split scan serves two KV heads where their number is even (with the heads
  // interleaved in a cache row its loads then cover 256-byte pieces: measured a tenth faster than one
  // head a block; four or eight heads a block stream faster still but leave more, smaller partial
  // results), and there are as many blocks as the chip has CUs -- and no fewer than query heads,
  // which the few-keys form needs -- whatever the cache's length.
  const int hpb_log2 = kv_heads % 2 == 0 ? 1 : 0;
  const int sets = kv_heads >> hpb_log2;
  int nsplit = kComputeUnits / sets;
  while (sets * nsplit < kv_heads * group) ++nsplit;
  nsplit = nsplit < 1 ? 1 : (nsplit > kMaxSplits ? kMaxSplits : nsplit);
  hipLaunchKernelGGL((mha_decode_either_kernel<D, WAVES>), dim3(sets, nsplit), dim3(64 * WAVES), lds, s, Q, K, V, O,
                     part, kv_heads, group, hpb_log2, kv_len, scale_log2, window, row_stride, head_stride, kv_valid,
                     kv_first, kv_rows, short_keys);
  if (nsplit <= 64)
    hipLaunchKernelGGL((mha_decode_either_merge_kernel<D, 8>), dim3(kv_heads * group), dim3(4 * D), 0, s, part, O,
                       nsplit, (WAVES == 16 ? 4 : 3) - hpb_log2, kv_len, window, kv_valid, short_keys);
  else
    hipLaunchKernelGGL((mha_decode_either_merge_kernel<D, 16>), dim3(kv_heads * group), dim3(4 * D), 0, s, part, O,
                       nsplit, (WAVES == 16 ? 4 : 3) - hpb_log2, kv_len, window, kv_valid, short_keys);
  return 0;
}

}  // namespace iron

using namespace iron;

extern "C" int64_t iron_mha_decode_workspace_bytes(int heads, int d) {
  return (int64_t)heads * kMaxSplits * (d + 2) * sizeof(float);
}

// form: 0 the default choice, 1 the lane-per-column scans, 2 the matrix-core scan (d = 64 / 128);
// short_keys: up to how many live keys the matrix-core scan's one block a KV head writes O itself (0: the default).
static int mha_decode(const uint16_t* Q, const uint16_t* K, const uint16_t* V, uint16_t* O, int heads, int kv_heads,
                      int d, int kv_len, float scale, int window, int kv_interleaved, const int* kv_valid,
                      const int* kv_first, int kv_rows, void* workspace, void* stream, int form = 0, int short_keys = 0) {
  IRON_REQUIRE(Q && K && V && O && workspace, "mha_decode: null operand");
  IRON_REQUIRE(kv_first == nullptr || (kv_interleaved && kv_rows >= kv_len),
               "mha_decode: a window of the keys takes them row by row (kv_interleaved) out of kv_rows (%d) >= kv_len (%d)",
               kv_rows, kv_len);
  IRON_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
               "mha_decode: heads (%d) must be a positive multiple of kv_heads (%d)", heads, kv_heads);
  IRON_REQUIRE(kv_len > 0, "mha_decode: kv_len (%d) must be positive", kv_len);
  IRON_REQUIRE(scale >= 0.f && scale < INFINITY, "mha_decode: scale must be finite and not negative");
  IRON_REQUIRE((((uintptr_t)Q | (uintptr_t)K | (uintptr_t)V | (uintptr_t)O | (uintptr_t)workspace) & 15) == 0,
               "mha_decode: operands must be 16-byte aligned");
  const int G = heads / kv_heads;
  const long row_stride = kv_interleaved ? (long)kv_heads * d : d;
  const long head_stride = kv_interleaved ? d : (long)kv_len * d;
  // Measured: a split per 128 keys, at least 8 (short caches are launch-bound) and at most 64
  // (beyond that the merge of the splits costs more than the extra parallelism gains).
  int nsplit = (kv_len + 127) / 128;
  nsplit = nsplit < 8 ? 8 : (nsplit > 64 ? 64 : nsplit);
  if (kv_len > 64 * 256) nsplit = (kv_len + 255) / 256 > kScanMaxSplits ? kScanMaxSplits : (kv_len + 255) / 256;
  if (nsplit * 8 > kv_len) nsplit = kv_len >= 8 ? kv_len / 8 : 1;
  const float scale_log2 = scale * 1.4426950408889634f;
  hipStream_t s = (hipStream_t)stream;
  float* part = (float*)workspace;
  IRON_REQUIRE(form >= 0 && form <= 2 && short_keys >= 0, "mha_decode: form (%d) is 0, 1 or 2 and short_keys (%d) not negative",
               form, short_keys);
  // Caches that can hold more rows than a single block scans well: one launch shape, the blocks
  // choosing by the live keys (d = 64 / 128).  Shorter ones, and the other widths, below.
  const bool either_fits = (d == 64 || d == 128) && G <= 16 && row_stride <= (1L << 20) &&
                           (long)kv_len * row_stride * 2 < (1L << 31) && heads <= kMaxSplits * kv_heads;
  IRON_REQUIRE(form != 2 || either_fits,
               "mha_decode: the one-shape launch takes d = 64 or 128, up to 16 query heads a KV head and keys within 2^31 bytes");
  const int upto = short_keys > 0 ? short_keys : kShortKeys;
  if (form == 2 || (form == 0 && either_fits && kv_len > (short_keys > 0 ? short_keys : kSingleMaxKeys))) {
    const int rc = d == 64 ? launch_decode_either<64, 16>(Q, K, V, O, part, kv_heads, G, kv_len, scale_log2, window, row_stride,
                                                          head_stride, kv_valid, kv_first, kv_rows, upto, s)
                           : launch_decode_either<128, 8>(Q, K, V, O, part, kv_heads, G, kv_len, scale_log2, window, row_stride,
                                                          head_stride, kv_valid, kv_first, kv_rows, upto, s);
    if (rc != 0) return rc;
    IRON_LAUNCH_CHECK();
  }
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
               "(d in {64,128} with up to 16, d = 256 with 1, 2, 3, 4, 5, 6 or 8, or d = 512)", d, G);
}

extern "C" int iron_mha_decode_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                    uint16_t* O, int heads, int kv_heads, int d, int kv_len,
                                    float scale, int window, int kv_interleaved,
                                    const int* kv_valid, void* workspace, void* stream) {
  return mha_decode(Q, K, V, O, heads, kv_heads, d, kv_len, scale, window, kv_interleaved, kv_valid, nullptr, 0,
                    workspace, stream);
}

extern "C" int iron_mha_decode_tuned_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                          uint16_t* O, int heads, int kv_heads, int d, int kv_len,
                                          float scale, int window, int kv_interleaved,
                                          const int* kv_valid, void* workspace, int form, int short_keys,
                                          void* stream) {
  return mha_decode(Q, K, V, O, heads, kv_heads, d, kv_len, scale, window, kv_interleaved, kv_valid, nullptr, 0,
                    workspace, stream, form, short_keys);
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
