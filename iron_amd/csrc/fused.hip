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

__device__ __forceinline__ float silu_ref(float v) { return v / (1.0f + __expf(-v)); }

// 1 / sqrt(mean(x^2) + eps) of a K-vector, computed by every wave for itself (x is L2-resident).
__device__ __forceinline__ float wave_inv_rms(const bf16_t* __restrict__ x, int K, float eps, int lane) {
  const uint4* xv = reinterpret_cast<const uint4*>(x);
  float ss = 0.f;
  for (int c = lane; c < (K >> 3); c += 64) {
    float f[8];
    unpack8(xv[c], f);
#pragma unroll
    for (int j = 0; j < 8; ++j) ss = fmaf(f[j], f[j], ss);
  }
  ss = wave_sum(ss);
  return 1.0f / sqrtf(ss / (float)K + eps);
}

// The 8 activations of chunk c as the GEMV sees them: x itself, or RMSNorm(x) * w rounded as
// the RMSNorm step rounds (the normed row to bf16, then the product to bf16).
template <bool NORM>
__device__ __forceinline__ void load_x(const bf16_t* __restrict__ x, const bf16_t* __restrict__ nw,
                                       float inv, int c, float (&xf)[8]) {
  unpack8(reinterpret_cast<const uint4*>(x)[c], xf);
  if (NORM) {
    float g[8];
    unpack8(reinterpret_cast<const uint4*>(nw)[c], g);
#pragma unroll
    for (int j = 0; j < 8; ++j) xf[j] = round_bf16(round_bf16(xf[j] * inv) * g[j]);
  }
}

enum { EPI_NONE = 0, EPI_ADD = 1, EPI_SILU_MUL = 2 };

// One wave per RPW rows, full K (so the rows' sums need no cross-wave merge).
template <int RPW, bool NORM, int EPI>
__global__ __launch_bounds__(256) void gemv_fused_kernel(const bf16_t* __restrict__ W,
                                                         const bf16_t* __restrict__ W2,
                                                         const bf16_t* __restrict__ x,
                                                         const bf16_t* __restrict__ nw, float eps,
                                                         const bf16_t* __restrict__ res,
                                                         bf16_t* __restrict__ y, int M, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row0 = (blockIdx.x * 4 + wave) * RPW;
  if (row0 >= M) return;
  const float inv = NORM ? wave_inv_rms(x, K, eps, lane) : 1.f;
  constexpr int MATS = EPI == EPI_SILU_MUL ? 2 : 1;
  float acc[MATS][RPW];
  const uint4* wrow[MATS][RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int row = min(row0 + r, M - 1);
    acc[0][r] = 0.f;
    wrow[0][r] = reinterpret_cast<const uint4*>(W + (size_t)row * K);
    if (MATS == 2) {
      acc[MATS - 1][r] = 0.f;
      wrow[MATS - 1][r] = reinterpret_cast<const uint4*>(W2 + (size_t)row * K);
    }
  }
  const int chunks = K >> 3;
#pragma unroll 4
  for (int c = lane; c < chunks; c += 64) {
    uint4 wv[MATS][RPW];
#pragma unroll
    for (int m = 0; m < MATS; ++m)
#pragma unroll
      for (int r = 0; r < RPW; ++r) wv[m][r] = load_stream(wrow[m][r] + c);
    float xf[8];
    load_x<NORM>(x, nw, inv, c, xf);
#pragma unroll
    for (int m = 0; m < MATS; ++m)
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        float wf[8];
        unpack8(wv[m][r], wf);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[m][r] = fmaf(wf[i], xf[i], acc[m][r]);
      }
  }
#pragma unroll
  for (int m = 0; m < MATS; ++m)
#pragma unroll
    for (int r = 0; r < RPW; ++r) acc[m][r] = wave_sum(acc[m][r]);
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      const int row = row0 + r;
      if (row >= M) break;
      float v = round_bf16(acc[0][r]);  // the GEMV step's own rounding
      if (EPI == EPI_ADD) v = v + bf16_to_f32(res[row]);
      if (EPI == EPI_SILU_MUL) v = round_bf16(silu_ref(v)) * round_bf16(acc[MATS - 1][r]);
      y[row] = f32_to_bf16(v);
    }
  }
}

// Attention's first half for one token.  A wave takes a PAIR of projection rows: for q and k
// the rows (h, j) and (h, j + D/2) that RoPE rotates together, for v two adjacent rows.
template <int D>
__global__ __launch_bounds__(256) void decode_qkv_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ nw, float eps,
    const bf16_t* __restrict__ Wq, const bf16_t* __restrict__ Wk, const bf16_t* __restrict__ Wv,
    const bf16_t* __restrict__ angles, bf16_t* __restrict__ q_out, bf16_t* __restrict__ keys,
    bf16_t* __restrict__ values, int K, int heads, int kv_heads, int cache_rows,
    const int* __restrict__ position) {
  constexpr int HALF = D / 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pair = blockIdx.x * 4 + wave;
  const int q_pairs = heads * HALF, k_pairs = kv_heads * HALF;
  if (pair >= q_pairs + 2 * k_pairs) return;
  const int pos = *position;
  const float inv = wave_inv_rms(x, K, eps, lane);

  const bf16_t* Wm;
  int r0, r1, j = 0, kind;  // kind 0 q, 1 k, 2 v
  if (pair < q_pairs) { kind = 0; Wm = Wq; const int h = pair / HALF; j = pair % HALF; r0 = h * D + j; r1 = r0 + HALF; }
  else if (pair < q_pairs + k_pairs) { kind = 1; Wm = Wk; const int p = pair - q_pairs; const int h = p / HALF; j = p % HALF; r0 = h * D + j; r1 = r0 + HALF; }
  else { kind = 2; Wm = Wv; const int p = pair - q_pairs - k_pairs; r0 = 2 * p; r1 = r0 + 1; }

  const uint4* w0 = reinterpret_cast<const uint4*>(Wm + (size_t)r0 * K);
  const uint4* w1 = reinterpret_cast<const uint4*>(Wm + (size_t)r1 * K);
  float a0 = 0.f, a1 = 0.f;
#pragma unroll 4
  for (int c = lane; c < (K >> 3); c += 64) {
    const uint4 v0 = load_stream(w0 + c), v1 = load_stream(w1 + c);
    float xf[8], f0[8], f1[8];
    load_x<true>(x, nw, inv, c, xf);
    unpack8(v0, f0);
    unpack8(v1, f1);
#pragma unroll
    for (int i = 0; i < 8; ++i) { a0 = fmaf(f0[i], xf[i], a0); a1 = fmaf(f1[i], xf[i], a1); }
  }
  a0 = wave_sum(a0);
  a1 = wave_sum(a1);
  if (lane != 0) return;
  float y0 = round_bf16(a0), y1 = round_bf16(a1);  // the projections' own rounding
  if (kind != 2) {
    const float c = bf16_to_f32(angles[2 * j]), s = bf16_to_f32(angles[2 * j + 1]);
    const float t0 = y0 * c - y1 * s, t1 = y1 * c + y0 * s;
    y0 = t0; y1 = t1;
  }
  if (kind == 0) {
    q_out[r0] = f32_to_bf16(y0);
    q_out[r1] = f32_to_bf16(y1);
  } else if (pos >= 0 && pos < cache_rows) {
    bf16_t* dst = (kind == 1 ? keys : values) + (size_t)pos * kv_heads * D;
    dst[r0] = f32_to_bf16(y0);
    dst[r1] = f32_to_bf16(y1);
  }
}

}  // namespace iron

using namespace iron;

extern "C" int iron_gemv_fused_bf16(const uint16_t* W, const uint16_t* W2, const uint16_t* x,
                                    const uint16_t* norm_w, float eps, const uint16_t* residual,
                                    uint16_t* y, int M, int K, int epilogue, void* stream) {
  IRON_REQUIRE(W && x && y, "gemv_fused: null operand");
  IRON_REQUIRE(M > 0 && K > 0 && K % 8 == 0, "gemv_fused: M (%d) positive, K (%d) a positive multiple of 8", M, K);
  IRON_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemv_fused: epilogue (%d) is 0, 1 or 2", epilogue);
  IRON_REQUIRE(epilogue != EPI_ADD || residual, "gemv_fused: epilogue 1 adds a residual; none given");
  IRON_REQUIRE(epilogue != EPI_SILU_MUL || W2, "gemv_fused: epilogue 2 takes a second matrix; none given");
  IRON_REQUIRE((((uintptr_t)W | (uintptr_t)W2 | (uintptr_t)x | (uintptr_t)norm_w) & 15) == 0,
               "gemv_fused: operands must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const bool norm = norm_w != nullptr;
  // Rows a wave takes: enough waves to fill the chip, several loads in flight a lane.
  const int rpw = (epilogue == EPI_SILU_MUL) ? 1 : (M >= 65536 ? 4 : (M >= 8192 ? 2 : 1));
  const int blocks = (M + 4 * rpw - 1) / (4 * rpw);
#define IRON_FUSED(R, NRM, E)                                                                      \
  if (rpw == R && norm == NRM && epilogue == E) {                                                  \
    hipLaunchKernelGGL((gemv_fused_kernel<R, NRM, E>), dim3(blocks), dim3(256), 0, s, W, W2, x,    \
                       norm_w, eps, residual, y, M, K);                                            \
    IRON_LAUNCH_CHECK();                                                                           \
  }
  IRON_FUSED(1, false, 0) IRON_FUSED(2, false, 0) IRON_FUSED(4, false, 0)
  IRON_FUSED(1, true, 0) IRON_FUSED(2, true, 0) IRON_FUSED(4, true, 0)
  IRON_FUSED(1, false, 1) IRON_FUSED(2, false, 1) IRON_FUSED(4, false, 1)
  IRON_FUSED(1, true, 1) IRON_FUSED(2, true, 1) IRON_FUSED(4, true, 1)
  IRON_FUSED(1, false, 2) IRON_FUSED(1, true, 2)
#undef IRON_FUSED
  IRON_REQUIRE(false, "gemv_fused: no kernel for this combination");
}

extern "C" int iron_decode_qkv_bf16(const uint16_t* x, const uint16_t* norm_w, float eps,
                                    const uint16_t* Wq, const uint16_t* Wk, const uint16_t* Wv,
                                    const uint16_t* angles, uint16_t* q_out, uint16_t* keys,
                                    uint16_t* values, int hidden, int heads, int kv_heads, int d,
                                    int cache_rows, const int* position, void* stream) {
  IRON_REQUIRE(x && norm_w && Wq && Wk && Wv && angles && q_out && keys && values && position,
               "decode_qkv: null operand");
  IRON_REQUIRE(hidden > 0 && hidden % 8 == 0, "decode_qkv: hidden (%d) must be a positive multiple of 8", hidden);
  IRON_REQUIRE(d == 64 || d == 128, "decode_qkv: d (%d) must be 64 or 128", d);
  IRON_REQUIRE(heads > 0 && kv_heads > 0 && cache_rows > 0, "decode_qkv: heads, kv_heads, cache_rows must be positive");
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)norm_w | (uintptr_t)Wq | (uintptr_t)Wk | (uintptr_t)Wv) & 15) == 0,
               "decode_qkv: operands must be 16-byte aligned");
  const int pairs = heads * (d / 2) + 2 * kv_heads * (d / 2);
  const int blocks = (pairs + 3) / 4;
  hipStream_t s = (hipStream_t)stream;
  if (d == 64)
    hipLaunchKernelGGL((decode_qkv_kernel<64>), dim3(blocks), dim3(256), 0, s, x, norm_w, eps, Wq, Wk, Wv,
                       angles, q_out, keys, values, hidden, heads, kv_heads, cache_rows, position);
  else
    hipLaunchKernelGGL((decode_qkv_kernel<128>), dim3(blocks), dim3(256), 0, s, x, norm_w, eps, Wq, Wk, Wv,
                       angles, q_out, keys, values, hidden, heads, kv_heads, cache_rows, position);
  IRON_LAUNCH_CHECK();
}
