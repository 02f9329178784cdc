// Fused decode-step kernels: each replaces a run of single-row operator steps of a decoder
// layer with one HBM-bound launch, keeping every rounding point of the unfused steps (each
// step's bf16 output is still rounded where the separate kernels round it), so a fused graph
// computes what the step-by-step graph computes.
//
//   gemv_fused:  [RMSNorm(weighted) ->] GEMV [-> + residual]             (o_proj/down_proj, LM head)
//                [RMSNorm ->] GEMV(gate), GEMV(up) -> SiLU -> Mul          (the gated MLP's first half)
//   decode_qkv:  RMSNorm -> GEMV q,k,v -> RoPE(q), RoPE(k) -> cache writes (attention's first half)
#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {


// All fused kernels share one shape: a block of 4 waves owns a few rows and its 256 threads
// split K in 16-byte chunks (thread t takes chunks t, t+256, ...), so the weight loads of a row
// are one contiguous stream per block, every lane has all its loads in flight before it needs
// any of them, and the activation chunk a thread normalises is the one it multiplies by.

// Block-wide sum through LDS (one barrier); every thread gets the total.
__device__ __forceinline__ float block_sum(float v, float* scratch4) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) scratch4[threadIdx.x >> 6] = v;
  __syncthreads();
  return scratch4[0] + scratch4[1] + scratch4[2] + scratch4[3];
}

// This thread's CH chunks of the activation as the GEMV sees them: x itself, or
// RMSNorm(x) * w rounded as the RMSNorm step rounds (the normed row to bf16, then the
// product to bf16).  In two halves so the caller can put its weight loads between them:
// memory returns in order, so the small activation loads go out first and are not held up
// behind the long weight stream.
template <int CH, bool NORM>
struct Activation {
  uint4 xv[CH], gv[CH];
  __device__ __forceinline__ void issue(const bf16_t* __restrict__ x, const bf16_t* __restrict__ nw, int K) {
    issue_row(x, K);
    issue_gains(nw, K);
  }
  // ... or apart, where the row's address is itself on its way from memory: the gains (and the
  // caller's weights) go out first and the row's loads once the address is in.
  __device__ __forceinline__ void issue_gains(const bf16_t* __restrict__ nw, int K) {
    if (!NORM) return;
    const __amdgpu_buffer_rsrc_t run = bounded_bytes(nw, 2 * K);
#pragma unroll
    for (int i = 0; i < CH; ++i) gv[i] = load_bounded(run, 16 * ((int)threadIdx.x + 256 * i));
  }
  __device__ __forceinline__ void issue_row(const bf16_t* __restrict__ x, int K) {
    const __amdgpu_buffer_rsrc_t run = bounded_bytes(x, 2 * K);
#pragma unroll
    for (int i = 0; i < CH; ++i) xv[i] = load_bounded(run, 16 * ((int)threadIdx.x + 256 * i));
  }
  // With NORM the block sums the squares together (one barrier).  The activation comes out as it
  // went in, packed bf16 (what the norm rounds to): the dot products below take it in pairs.
  __device__ __forceinline__ void finish(float eps, int K, float* scratch4, uint4 (&xp)[CH]) {
    if (!NORM) {
#pragma unroll
      for (int i = 0; i < CH; ++i) xp[i] = xv[i];
      return;
    }
    float xf[CH][8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      unpack8(xv[i], xf[i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = fmaf(xf[i][j], xf[i][j], ss);
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch4) / (float)K + eps);
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      float g[8];
      unpack8(gv[i], g);
#pragma unroll
      for (int j = 0; j < 8; ++j) xf[i][j] = round_bf16(xf[i][j] * inv) * g[j];
      xp[i] = pack8(xf[i]);   // the product's own rounding
    }
  }
};

// A weight row's chunks of this thread (zeros past the row's end), streamed past the caches.
template <int CH>
__device__ __forceinline__ void load_row(const bf16_t* __restrict__ row, int K, uint4 (&w)[CH]) {
  const __amdgpu_buffer_rsrc_t run = bounded_bytes(row, 2 * K);
#pragma unroll
  for (int i = 0; i < CH; ++i) w[i] = load_bounded_stream(run, 16 * ((int)threadIdx.x + 256 * i));
}

// A row's chunks times the activation's: two-element dot products of the bf16 pairs as they were
// loaded (v_dot2c_f32_bf16: exact products, float32 sums) -- a quarter of the instructions of
// widening both sides and a multiply-add an element, and what a resident block does after its
// loads have landed is time its CU's share of the memory system idles.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
template <int CH>
__device__ __forceinline__ float dot_row(const uint4 (&w)[CH], const uint4 (&xp)[CH]) {
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[i].x), __builtin_bit_cast(bf16x2_t, xp[i].x), acc, false);
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[i].y), __builtin_bit_cast(bf16x2_t, xp[i].y), acc, false);
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[i].z), __builtin_bit_cast(bf16x2_t, xp[i].z), acc, false);
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[i].w), __builtin_bit_cast(bf16x2_t, xp[i].w), acc, false);
  }
  return acc;
}

enum { EPI_NONE = 0, EPI_ADD = 1, EPI_SILU_MUL = 2, EPI_GELU_MUL = 3,     // 2 and 3: gate, up -> activation -> Mul
       EPI_GELU_ROW = 4, EPI_SILU_ROW = 5 };                               // activation -> Mul by a given row

// y = E(W @ N(x)) for RPW rows a block; K <= CH * 2048.
template <int RPW, int CH, bool NORM, int EPI>
__global__ __launch_bounds__(256) void gemv_fused_kernel(const bf16_t* __restrict__ W,
                                                         const bf16_t* __restrict__ W2,
                                                         const bf16_t* __restrict__ x,
                                                         const bf16_t* __restrict__ nw, float eps,
                                                         const bf16_t* __restrict__ res,
                                                         float res_scale, bf16_t* __restrict__ y,
                                                         int M, int K) {
  constexpr int MATS = (EPI == EPI_SILU_MUL || EPI == EPI_GELU_MUL) ? 2 : 1;
  __shared__ float scratch4[4];
  __shared__ float part[4][MATS][RPW];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row0 = blockIdx.x * RPW;
  // The residual a thread will add at the end is requested first, so that its trip to memory
  // passes under the weights' instead of after the block's last barrier.
  // (Every thread asks, the ones that add nothing for the block's last row again: behind a branch
  // for the few that need it, the wave that took it would wait for the word then and there.)
  bf16_t res_word = 0;
  if (EPI == EPI_ADD || EPI == EPI_GELU_ROW || EPI == EPI_SILU_ROW)
    res_word = res[min(row0 + min((int)threadIdx.x, RPW - 1), M - 1)];
  Activation<CH, NORM> act;
  act.issue(x, nw, K);
  uint4 w[MATS][RPW][CH];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int row = min(row0 + r, M - 1);
    load_row<CH>(W + (size_t)row * K, K, w[0][r]);
    if (MATS == 2) load_row<CH>(W2 + (size_t)row * K, K, w[MATS - 1][r]);
  }
  uint4 xf[CH];
  act.finish(eps, K, scratch4, xf);
#pragma unroll
  for (int m = 0; m < MATS; ++m)
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      const float a = wave_sum(dot_row<CH>(w[m][r], xf));
      if (lane == 0) part[wave][m][r] = a;
    }
  __syncthreads();
  if (threadIdx.x < RPW) {
    const int r = threadIdx.x, row = row0 + r;
    if (row < M) {
      float v = round_bf16(part[0][0][r] + part[1][0][r] + part[2][0][r] + part[3][0][r]);  // the GEMV's own rounding
      const float res_ahead = bf16_to_f32(res_word);
      if (EPI == EPI_ADD) v = fmaf(res_scale, v, res_ahead);   // scale 1: the plain sum
      if (EPI == EPI_GELU_ROW || EPI == EPI_SILU_ROW)          // the activation's own rounding, then the product's
        v = round_bf16(EPI == EPI_SILU_ROW ? silu_f32(v) : gelu_tanh_f32(v)) * res_ahead;
      if (EPI == EPI_SILU_MUL || EPI == EPI_GELU_MUL) {
        const float u = round_bf16(part[0][MATS - 1][r] + part[1][MATS - 1][r] + part[2][MATS - 1][r] +
                                   part[3][MATS - 1][r]);
        v = round_bf16(EPI == EPI_SILU_MUL ? silu_f32(v) : gelu_tanh_f32(v)) * u;
      }
      y[row] = f32_to_bf16(v);
    }
  }
}

// Attention's first half for one token.  A block takes PAIRS pairs of projection rows: for q and k
// a pair is the rows (h, j) and (h, j + D/2) that RoPE rotates together, for v two adjacent rows
// (with PAIRS = 2 the block's activation and gain loads, and its norm, serve four rows -- what the
// gate/up launch's blocks have; the pairs of a block are of one kind, which even pair counts ensure).
// TABLE: x is to be read from row *x_row of x_table (and left in x by the first block).
template <int D, int CH, bool TABLE, int PAIRS>
__global__ __launch_bounds__(256) void decode_qkv_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ nw, float eps,
    const bf16_t* __restrict__ Wq, const bf16_t* __restrict__ Wk, const bf16_t* __restrict__ Wv,
    const bf16_t* __restrict__ angles, bf16_t* __restrict__ q_out, bf16_t* __restrict__ keys,
    bf16_t* __restrict__ values, int K, int heads, int kv_heads, int cache_rows,
    const int* __restrict__ position, const int* __restrict__ angle_row, int angle_rows,
    const bf16_t* __restrict__ x_table, const int* __restrict__ x_row, int x_rows) {
  constexpr int HALF = D / 2;
  __shared__ float scratch4[4];
  __shared__ float part[4][PAIRS][2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pair0 = blockIdx.x * PAIRS;
  const int q_pairs = heads * HALF, k_pairs = kv_heads * HALF;

  // The block's kind (0 q, 1 k, 2 v) and its first pair's rows; pair p's follow at + p (+ 2 p for v).
  const bf16_t* Wm;
  int r0, step, j = 0, kind;
  if (pair0 < q_pairs) { kind = 0; Wm = Wq; const int h = pair0 / HALF; j = pair0 % HALF; r0 = h * D + j; step = HALF; }
  else if (pair0 < q_pairs + k_pairs) { kind = 1; Wm = Wk; const int p = pair0 - q_pairs; const int h = p / HALF; j = p % HALF; r0 = h * D + j; step = HALF; }
  else { kind = 2; Wm = Wv; const int p = pair0 - q_pairs - k_pairs; r0 = 2 * p; step = 1; }
  const int next = kind == 2 ? 2 : 1;   // from a pair's first row to the next pair's

  Activation<CH, true> act;
  uint4 w0[PAIRS][CH], w1[PAIRS][CH];
  if (!TABLE) {
    act.issue(x, nw, K);
#pragma unroll
    for (int p = 0; p < PAIRS; ++p) {
      load_row<CH>(Wm + (size_t)(r0 + p * next) * K, K, w0[p]);
      load_row<CH>(Wm + (size_t)(r0 + p * next + step) * K, K, w1[p]);
    }
  } else {
    // The token's row of an embedding table, named by a device word (held inside the table): the row
    // is read where it lies and the first block leaves the copy the layer's residual sum will read,
    // so the step's gather needs no launch of its own.  Everything that does not wait for the word
    // goes out ahead of it.
    act.issue_gains(nw, K);
#pragma unroll
    for (int p = 0; p < PAIRS; ++p) {
      load_row<CH>(Wm + (size_t)(r0 + p * next) * K, K, w0[p]);
      load_row<CH>(Wm + (size_t)(r0 + p * next + step) * K, K, w1[p]);
    }
    act.issue_row(x_table + (size_t)max(0, min(*x_row, x_rows - 1)) * K, K);
    if (blockIdx.x == 0) {
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const int c = threadIdx.x + 256 * i;
        if (c < (K >> 3)) reinterpret_cast<uint4*>(const_cast<bf16_t*>(x))[c] = act.xv[i];
      }
    }
  }
  // `angles` is the step's row itself, or a whole table whose row a device word names (held inside).
  // What the block's last threads need after the last barrier -- their pair's angle and the position
  // word -- is asked for here, behind the rows' loads (the word that names the angles' row is a trip
  // to memory of its own, which nothing above waits for) and under their trip to memory.
  // (The two words pinned here, among the loads in flight: left free, the compiler moves the position's
  // load down to its use after the last barrier, a trip to memory at the kernel's very end.)
  int pos_ahead = *position, angle_at = angle_row != nullptr ? *angle_row : 0;
  asm volatile("" : "+s"(pos_ahead), "+s"(angle_at));
  angles += (size_t)max(0, min(angle_at, angle_rows - 1)) * D;
  const int mine = min((int)threadIdx.x, PAIRS - 1);   // the pair this thread finishes, if it finishes one
  const float c_ahead = bf16_to_f32(angles[2 * (j + mine)]), s_ahead = bf16_to_f32(angles[2 * (j + mine) + 1]);
  uint4 xf[CH];
  act.finish(eps, K, scratch4, xf);
#pragma unroll
  for (int p = 0; p < PAIRS; ++p) {
    const float a0 = wave_sum(dot_row<CH>(w0[p], xf)), a1 = wave_sum(dot_row<CH>(w1[p], xf));
    if (lane == 0) { part[wave][p][0] = a0; part[wave][p][1] = a1; }
  }
  __syncthreads();
  if (threadIdx.x >= PAIRS) return;
  const int p = threadIdx.x, ra = r0 + p * next, rb = ra + step;
  float y0 = round_bf16(part[0][p][0] + part[1][p][0] + part[2][p][0] + part[3][p][0]);  // the projections' own rounding
  float y1 = round_bf16(part[0][p][1] + part[1][p][1] + part[2][p][1] + part[3][p][1]);
  if (kind != 2) {
    const float c = c_ahead, s = s_ahead;
    const float t0 = y0 * c - y1 * s, t1 = y1 * c + y0 * s;
    y0 = t0; y1 = t1;
  }
  if (kind == 0) {
    q_out[ra] = f32_to_bf16(y0);
    q_out[rb] = f32_to_bf16(y1);
  } else {
    const int pos = pos_ahead;
    if (pos >= 0 && pos < cache_rows) {
      bf16_t* dst = (kind == 1 ? keys : values) + (size_t)pos * kv_heads * D;
      dst[ra] = f32_to_bf16(y0);
      dst[rb] = f32_to_bf16(y1);
    }
  }
}


// Between a token's q/k/v projections and its attention, where the heads are normed one by one (q and
// k with learned gains, v without: Gemma's): RMSNorm per head, RoPE on q and k, and k's and v's rows
// into their cache rows (twice where the cache is a ring: the slot and its mirror) -- up to nine
// recorded steps, one launch.  A block a head row (q heads, then k's, then v's), 256 threads, each
// step computed exactly as its own kernel computes it (the norm's sum in rmsnorm_kernel's order, its
// two roundings; RoPE on the rounded row), so the rows are those kernels' bit for bit.
struct HeadRows {
  const bf16_t *q, *k, *v;            // (heads, d), (kv_heads, d) twice; k and v NULL where another layer owns the cache
  const bf16_t *q_gain, *k_gain;      // (d); NULL: that norm has no gain
  int norms;                          // bit 0: q is normed, 1: k, 2: v
  float eps;
  const bf16_t *q_angles, *k_angles;  // the call's RoPE rows (rotary columns, cos/sin interleaved); NULL: not rotated
  int rotary, two_halves;             // columns RoPE turns (<= d; the rest pass through)
  bf16_t* q_out;                      // (heads, d)
  bf16_t* dst[2][2];                  // [k, v][copy]: caches (cache_rows, kv_heads, d); NULL: no such copy
  const int* row[2][2];               // the cache row each copy goes to
  int cache_rows, heads, kv_heads, d;
};

__global__ __launch_bounds__(256) void decode_heads_kernel(HeadRows a) {
  __shared__ float part[4];
  __shared__ __align__(16) bf16_t held[2048];
  const int t = threadIdx.x, d = a.d, nchunk = d >> 3;
  const int b = blockIdx.x;
  const int kind = b < a.heads ? 0 : (b < a.heads + a.kv_heads ? 1 : 2);   // q, k, v
  const int head = kind == 0 ? b : b - a.heads - (kind - 1) * a.kv_heads;
  const bf16_t* src = (kind == 0 ? a.q : kind == 1 ? a.k : a.v) + (size_t)head * d;
  const bf16_t* gain = kind == 0 ? a.q_gain : (kind == 1 ? a.k_gain : nullptr);
  const bf16_t* angles = kind == 0 ? a.q_angles : (kind == 1 ? a.k_angles : nullptr);
  const bool normed = (a.norms >> kind) & 1;
  // Where the row goes: q to its output, k and v to their cache rows.
  int rows[2] = {0, 0};
  if (kind != 0) {
#pragma unroll
    for (int c = 0; c < 2; ++c)
      if (a.dst[kind - 1][c] != nullptr) rows[c] = *a.row[kind - 1][c];
  }

  uint4 xv = make_uint4(0, 0, 0, 0), gv = make_uint4(0, 0, 0, 0);
  if (t < nchunk) {
    xv = reinterpret_cast<const uint4*>(src)[t];
    if (normed && gain != nullptr) gv = reinterpret_cast<const uint4*>(gain)[t];
  }
  float f[8];
  unpack8(xv, f);
  if (normed) {
    float ss = 0.f;
    if (t < nchunk) {
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = fmaf(f[j], f[j], ss);
    }
    ss = wave_sum(ss);
    if ((t & 63) == 0) part[t >> 6] = ss;
    __syncthreads();
    const float inv = 1.0f / sqrtf((part[0] + part[1] + part[2] + part[3]) / (float)d + a.eps);
    if (gain != nullptr) {
      float g[8];
      unpack8(gv, g);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = round_bf16(f[j] * inv) * g[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = f[j] * inv;
    }
    xv = pack8(f);
  }
  if (angles != nullptr) {
    if (t < nchunk) reinterpret_cast<uint4*>(held)[t] = xv;
    __syncthreads();
    uint4 oa = make_uint4(0, 0, 0, 0), ob = oa;
    const int j = t, turning = a.rotary >> 4;   // thread j turns 8 column pairs
    if (j < turning) {
      float cs0[8], cs1[8], x1[8], x2[8], y1[8], y2[8];
      unpack8(reinterpret_cast<const uint4*>(angles + 16 * j)[0], cs0);
      unpack8(reinterpret_cast<const uint4*>(angles + 16 * j)[1], cs1);
      const float c[8] = {cs0[0], cs0[2], cs0[4], cs0[6], cs1[0], cs1[2], cs1[4], cs1[6]};
      const float sn[8] = {cs0[1], cs0[3], cs0[5], cs0[7], cs1[1], cs1[3], cs1[5], cs1[7]};
      if (a.two_halves) {
        const int half = a.rotary >> 1;
        unpack8(*reinterpret_cast<const uint4*>(held + 8 * j), x1);
        unpack8(*reinterpret_cast<const uint4*>(held + half + 8 * j), x2);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          y1[i] = x1[i] * c[i] - x2[i] * sn[i];
          y2[i] = x2[i] * c[i] + x1[i] * sn[i];
        }
        oa = pack8(y1);
        ob = pack8(y2);
      } else {
        float lo[8], hi[8];
        unpack8(*reinterpret_cast<const uint4*>(held + 16 * j), lo);
        unpack8(*reinterpret_cast<const uint4*>(held + 16 * j + 8), hi);
        const float e[8] = {lo[0], lo[2], lo[4], lo[6], hi[0], hi[2], hi[4], hi[6]};
        const float o[8] = {lo[1], lo[3], lo[5], lo[7], hi[1], hi[3], hi[5], hi[7]};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          y1[i] = e[i] * c[i] - o[i] * sn[i];
          y2[i] = o[i] * c[i] + e[i] * sn[i];
        }
        const float r0[8] = {y1[0], y2[0], y1[1], y2[1], y1[2], y2[2], y1[3], y2[3]};
        const float r1[8] = {y1[4], y2[4], y1[5], y2[5], y1[6], y2[6], y1[7], y2[7]};
        oa = pack8(r0);
        ob = pack8(r1);
      }
    }
    __syncthreads();   // every pair has been read before any is replaced
    if (j < turning) {
      if (a.two_halves) {
        *reinterpret_cast<uint4*>(held + 8 * j) = oa;
        *reinterpret_cast<uint4*>(held + (a.rotary >> 1) + 8 * j) = ob;
      } else {
        *reinterpret_cast<uint4*>(held + 16 * j) = oa;
        *reinterpret_cast<uint4*>(held + 16 * j + 8) = ob;
      }
    }
    __syncthreads();
    if (t < nchunk) xv = reinterpret_cast<const uint4*>(held)[t];
  }
  if (t >= nchunk) return;
  if (kind == 0) {
    reinterpret_cast<uint4*>(a.q_out + (size_t)head * d)[t] = xv;
    return;
  }
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    bf16_t* cache = a.dst[kind - 1][c];
    if (cache == nullptr || rows[c] < 0 || rows[c] >= a.cache_rows) continue;
    reinterpret_cast<uint4*>(cache + ((size_t)rows[c] * a.kv_heads + head) * d)[t] = xv;
  }
}

}  // namespace iron

using namespace iron;

extern "C" int iron_gemv_fused_bf16(const uint16_t* W, const uint16_t* W2, const uint16_t* x,
                                    const uint16_t* norm_w, float eps, const uint16_t* residual,
                                    float residual_scale, uint16_t* y, int M, int K, int epilogue,
                                    void* stream) {
  IRON_REQUIRE(W && x && y, "gemv_fused: null operand");
  IRON_REQUIRE(M > 0 && K > 0 && K % 8 == 0, "gemv_fused: M (%d) positive, K (%d) a positive multiple of 8", M, K);
  IRON_REQUIRE(epilogue >= 0 && epilogue <= 5, "gemv_fused: epilogue (%d) is 0 to 5", epilogue);
  IRON_REQUIRE((epilogue != EPI_ADD && epilogue != EPI_GELU_ROW && epilogue != EPI_SILU_ROW) || residual,
               "gemv_fused: epilogues 1, 4 and 5 take a second row (the residual, the factor); none given");
  IRON_REQUIRE((epilogue != EPI_SILU_MUL && epilogue != EPI_GELU_MUL) || W2, "gemv_fused: epilogues 2 and 3 take a second matrix; none given");
  IRON_REQUIRE((((uintptr_t)W | (uintptr_t)W2 | (uintptr_t)x | (uintptr_t)norm_w) & 15) == 0,
               "gemv_fused: operands must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const bool norm = norm_w != nullptr;
  IRON_REQUIRE(K <= 8 * 2048, "gemv_fused: K (%d) exceeds %d", K, 8 * 2048);
  const int ch = K <= 2048 ? 1 : (K <= 4096 ? 2 : (K <= 8192 ? 4 : 8));
  // Rows a block takes (measured inside a decoder's step, on 256 CUs): two where the matrix is tall
  // and a row is short, and for 16 KB rows of a matrix of a few thousand; else one.
  const bool pair_of_matrices = epilogue == EPI_SILU_MUL || epilogue == EPI_GELU_MUL;
  const bool plain_or_sum = epilogue == EPI_NONE || epilogue == EPI_ADD;
  const int rpw = pair_of_matrices ? (ch == 1 ? 2 : 1)
                  : (ch == 1 && M > 2048) ? (M >= 65536 ? 4 : 2)
                  : (ch == 4 && M >= 2048 && plain_or_sum) ? 2 : 1;
  const int blocks = (M + rpw - 1) / rpw;
#define IRON_FUSED(R, C, NRM, E)                                                                   \
  if (rpw == R && ch == C && norm == NRM && epilogue == E) {                                       \
    hipLaunchKernelGGL((gemv_fused_kernel<R, C, NRM, E>), dim3(blocks), dim3(256), 0, s, W, W2, x, \
                       norm_w, eps, residual, residual_scale, y, M, K);                            \
    IRON_LAUNCH_CHECK();                                                                           \
  }
#define IRON_FUSED_NE(R, C)                                                                        \
  IRON_FUSED(R, C, false, 0) IRON_FUSED(R, C, true, 0) IRON_FUSED(R, C, false, 1) IRON_FUSED(R, C, true, 1)
  IRON_FUSED_NE(1, 1) IRON_FUSED_NE(2, 1) IRON_FUSED_NE(4, 1) IRON_FUSED_NE(1, 2) IRON_FUSED_NE(1, 4) IRON_FUSED_NE(2, 4) IRON_FUSED_NE(1, 8)
  IRON_FUSED(2, 1, false, 2) IRON_FUSED(2, 1, true, 2) IRON_FUSED(1, 2, false, 2) IRON_FUSED(1, 2, true, 2)
  IRON_FUSED(1, 4, false, 2) IRON_FUSED(1, 4, true, 2) IRON_FUSED(1, 8, false, 2) IRON_FUSED(1, 8, true, 2)
  IRON_FUSED(2, 1, false, 3) IRON_FUSED(2, 1, true, 3) IRON_FUSED(1, 2, false, 3) IRON_FUSED(1, 2, true, 3)
  IRON_FUSED(1, 4, false, 3) IRON_FUSED(1, 4, true, 3) IRON_FUSED(1, 8, false, 3) IRON_FUSED(1, 8, true, 3)
  IRON_FUSED(1, 1, false, 4) IRON_FUSED(1, 2, false, 4) IRON_FUSED(1, 4, false, 4) IRON_FUSED(1, 8, false, 4)
  IRON_FUSED(1, 1, false, 5) IRON_FUSED(1, 2, false, 5) IRON_FUSED(1, 4, false, 5) IRON_FUSED(1, 8, false, 5)
  IRON_FUSED(2, 1, false, 4) IRON_FUSED(2, 1, false, 5)
#undef IRON_FUSED_NE
#undef IRON_FUSED
  IRON_REQUIRE(false, "gemv_fused: no kernel for this combination");
}

static int decode_qkv(const uint16_t* x, const uint16_t* norm_w, float eps, const uint16_t* Wq, const uint16_t* Wk,
                      const uint16_t* Wv, const uint16_t* angles, uint16_t* q_out, uint16_t* keys, uint16_t* values,
                      int hidden, int heads, int kv_heads, int d, int cache_rows, const int* position,
                      const int* angle_row, int angle_rows, const uint16_t* x_table, const int* x_row, int x_rows,
                      void* stream) {
  IRON_REQUIRE(x && norm_w && Wq && Wk && Wv && angles && q_out && keys && values && position,
               "decode_qkv: null operand");
  IRON_REQUIRE(hidden > 0 && hidden % 8 == 0, "decode_qkv: hidden (%d) must be a positive multiple of 8", hidden);
  IRON_REQUIRE(d == 64 || d == 128, "decode_qkv: d (%d) must be 64 or 128", d);
  IRON_REQUIRE(heads > 0 && kv_heads > 0 && cache_rows > 0, "decode_qkv: heads, kv_heads, cache_rows must be positive");
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)norm_w | (uintptr_t)Wq | (uintptr_t)Wk | (uintptr_t)Wv | (uintptr_t)x_table) & 15) == 0,
               "decode_qkv: operands must be 16-byte aligned");
  IRON_REQUIRE(hidden <= 8192, "decode_qkv: hidden (%d) exceeds 8192", hidden);
  IRON_REQUIRE(angle_row == nullptr || angle_rows > 0, "decode_qkv: a table of %d angle rows", angle_rows);
  IRON_REQUIRE(x_row == nullptr || (x_table != nullptr && x_rows > 0), "decode_qkv: a row of a table of %d rows", x_rows);
  const int pairs = heads * (d / 2) + 2 * kv_heads * (d / 2);
  const int ch = hidden <= 2048 ? 1 : (hidden <= 4096 ? 2 : 4);
  // Two pairs a block where a row is at most 4 KB (its chunks one a thread) and no block would span
  // two kinds of rows or a pair's two halves (q's and k's pair counts a multiple of D/2: even).
  const int per = ch == 1 ? 2 : 1;
  hipStream_t s = (hipStream_t)stream;
#define IRON_QKV(DD, C, P)                                                                          \
  if (d == DD && ch == C && per == P) {                                                             \
    if (x_row == nullptr)                                                                           \
      hipLaunchKernelGGL((decode_qkv_kernel<DD, C, false, P>), dim3(pairs / P), dim3(256), 0, s, x, norm_w, eps, Wq, Wk, Wv, \
                         angles, q_out, keys, values, hidden, heads, kv_heads, cache_rows, position, angle_row,        \
                         angle_rows, x_table, x_row, x_rows);                                                          \
    else                                                                                            \
      hipLaunchKernelGGL((decode_qkv_kernel<DD, C, true, P>), dim3(pairs / P), dim3(256), 0, s, x, norm_w, eps, Wq, Wk, Wv,  \
                         angles, q_out, keys, values, hidden, heads, kv_heads, cache_rows, position, angle_row,        \
                         angle_rows, x_table, x_row, x_rows);                                                          \
  }
  IRON_QKV(64, 1, 1) IRON_QKV(64, 2, 1) IRON_QKV(64, 4, 1) IRON_QKV(128, 1, 1) IRON_QKV(128, 2, 1) IRON_QKV(128, 4, 1)
  IRON_QKV(64, 1, 2) IRON_QKV(128, 1, 2)
#undef IRON_QKV
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_decode_qkv_bf16(const uint16_t* x, const uint16_t* norm_w, float eps,
                                    const uint16_t* Wq, const uint16_t* Wk, const uint16_t* Wv,
                                    const uint16_t* angles, uint16_t* q_out, uint16_t* keys,
                                    uint16_t* values, int hidden, int heads, int kv_heads, int d,
                                    int cache_rows, const int* position, const int* angle_row, int angle_rows,
                                    void* stream) {
  return decode_qkv(x, norm_w, eps, Wq, Wk, Wv, angles, q_out, keys, values, hidden, heads, kv_heads, d, cache_rows,
                    position, angle_row, angle_rows, nullptr, nullptr, 0, stream);
}

extern "C" int iron_decode_qkv_embed_bf16(const uint16_t* table, const int* token, int table_rows, uint16_t* x,
                                          const uint16_t* norm_w, float eps, const uint16_t* Wq, const uint16_t* Wk,
                                          const uint16_t* Wv, const uint16_t* angles, uint16_t* q_out, uint16_t* keys,
                                          uint16_t* values, int hidden, int heads, int kv_heads, int d, int cache_rows,
                                          const int* position, const int* angle_row, int angle_rows, void* stream) {
  IRON_REQUIRE(table && token && table_rows > 0, "decode_qkv_embed: a table of %d rows and the word that names the row", table_rows);
  return decode_qkv(x, norm_w, eps, Wq, Wk, Wv, angles, q_out, keys, values, hidden, heads, kv_heads, d, cache_rows,
                    position, angle_row, angle_rows, table, token, table_rows, stream);
}

extern "C" int iron_decode_heads_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, const uint16_t* q_gain,
                                      const uint16_t* k_gain, int norms, float eps, const uint16_t* q_angles,
                                      const uint16_t* k_angles, int rotary, int two_halves, uint16_t* q_out,
                                      uint16_t* keys, uint16_t* values, const int* row0, const int* row1,
                                      int cache_rows, int heads, int kv_heads, int d, void* stream) {
  IRON_REQUIRE(q && q_out, "decode_heads: null operand");
  IRON_REQUIRE((k == nullptr) == (v == nullptr), "decode_heads: k and v come together or not at all");
  IRON_REQUIRE(k == nullptr || (keys && values && row0 && cache_rows > 0),
               "decode_heads: k and v go to caches of %d rows at the row a device word names", cache_rows);
  IRON_REQUIRE(heads > 0 && kv_heads > 0 && d > 0 && d % 16 == 0 && d <= 2048,
               "decode_heads: heads (%d), kv_heads (%d) positive, d (%d) a multiple of 16 up to 2048", heads, kv_heads, d);
  IRON_REQUIRE(norms >= 0 && norms < 8, "decode_heads: norms (%d) is a mask of q (1), k (2), v (4)", norms);
  IRON_REQUIRE((q_angles == nullptr && k_angles == nullptr) || (rotary > 0 && rotary <= d && rotary % 16 == 0),
               "decode_heads: RoPE turns %d columns of a head of %d (a positive multiple of 16)", rotary, d);
  IRON_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)q_gain | (uintptr_t)k_gain | (uintptr_t)q_angles |
                 (uintptr_t)k_angles | (uintptr_t)q_out | (uintptr_t)keys | (uintptr_t)values) & 15) == 0,
               "decode_heads: operands must be 16-byte aligned");
  HeadRows a{};
  a.q = q; a.k = k; a.v = v;
  a.q_gain = q_gain; a.k_gain = k_gain;
  a.norms = norms; a.eps = eps;
  a.q_angles = q_angles; a.k_angles = k_angles;
  a.rotary = rotary; a.two_halves = two_halves;
  a.q_out = q_out;
  if (k != nullptr) {
    a.dst[0][0] = keys; a.dst[1][0] = values;
    a.row[0][0] = a.row[1][0] = row0;
    if (row1 != nullptr) {
      a.dst[0][1] = keys; a.dst[1][1] = values;
      a.row[0][1] = a.row[1][1] = row1;
    }
  }
  a.cache_rows = cache_rows; a.heads = heads; a.kv_heads = kv_heads; a.d = d;
  const int blocks = heads + (k != nullptr ? 2 * kv_heads : 0);
  hipLaunchKernelGGL(decode_heads_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
  IRON_LAUNCH_CHECK();
}
