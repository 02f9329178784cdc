// GEMV: y = W x, W (M,K) bf16 row-major, HBM-bandwidth bound.
//
// A block is 4 waves.  The waves of a block form (4 / KSPLIT) row groups x
// KSPLIT slices of K; a wave streams RPW rows of W over its K slice with
// 16-byte loads (a lane takes 8 consecutive bf16, the wave 512 per step),
// keeps partial sums in f32, reduces across lanes with shuffles and across the
// K slices through LDS.  Nothing but W is read more than once from HBM: x is
// 2*K bytes and stays in L2.
#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

template <int RPW, int KSPLIT>
__global__ __launch_bounds__(256) void gemv_kernel(const bf16_t* __restrict__ W,
                                                   const bf16_t* __restrict__ x,
                                                   bf16_t* __restrict__ y, int M, int K,
                                                   int repeat, const int* __restrict__ valid) {
  constexpr int ROW_GROUPS = 4 / KSPLIT;
  constexpr int ROWS_PER_BLOCK = ROW_GROUPS * RPW;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int kpart = wave % KSPLIT;
  const int rgroup = wave / KSPLIT;
  const int batch = blockIdx.y;
  const int rows = bound_or(valid, M);
  const int row0 = blockIdx.x * ROWS_PER_BLOCK + rgroup * RPW;

  const bf16_t* Wb = W + (size_t)(batch / repeat) * M * K;
  const bf16_t* xb = x + (size_t)batch * K;

  // K slice of this wave, in 8-element chunks.
  const int chunks = K >> 3;
  const int per = (chunks + KSPLIT - 1) / KSPLIT;
  const int c0 = kpart * per;
  const int c1 = min(chunks, c0 + per);

  float acc[RPW];
  const uint4* wrow[RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    acc[r] = 0.f;
    // A row past the end reads row M-1 again (never stored).
    int row = min(row0 + r, M - 1);
    wrow[r] = reinterpret_cast<const uint4*>(Wb + (size_t)row * K);
  }
  const uint4* xv = reinterpret_cast<const uint4*>(xb);

  if (row0 < rows) {
#pragma unroll 4
    for (int c = c0 + lane; c < c1; c += 64) {
      uint4 wv[RPW];
#pragma unroll
      for (int r = 0; r < RPW; ++r) wv[r] = load_stream(wrow[r] + c);
      // Two-element dot products of the bf16 pairs as loaded (v_dot2c_f32_bf16: exact products,
      // float32 sums), as the fused one-row kernels take theirs.
      const uint4 xp = xv[c];
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        acc[r] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, wv[r].x), __builtin_bit_cast(bf16x2_t, xp.x), acc[r], false);
        acc[r] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, wv[r].y), __builtin_bit_cast(bf16x2_t, xp.y), acc[r], false);
        acc[r] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, wv[r].z), __builtin_bit_cast(bf16x2_t, xp.z), acc[r], false);
        acc[r] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, wv[r].w), __builtin_bit_cast(bf16x2_t, xp.w), acc[r], false);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < RPW; ++r) acc[r] = wave_sum(acc[r]);

  if constexpr (KSPLIT > 1) {
    __shared__ float part[4][RPW];
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < RPW; ++r) part[wave][r] = acc[r];
    }
    __syncthreads();
    if (kpart == 0 && lane == 0) {
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        float s = 0.f;
#pragma unroll
        for (int p = 0; p < KSPLIT; ++p) s += part[rgroup * KSPLIT + p][r];
        int row = row0 + r;
        if (row < rows) y[(size_t)batch * M + row] = f32_to_bf16(s);
      }
    }
  } else {
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        int row = row0 + r;
        if (row < rows) y[(size_t)batch * M + row] = f32_to_bf16(acc[r]);
      }
    }
  }
}

template <int RPW, int KSPLIT>
static void launch_gemv(const bf16_t* W, const bf16_t* x, bf16_t* y, int M, int K, int batches,
                        int repeat, const int* valid, hipStream_t s) {
  constexpr int ROWS_PER_BLOCK = (4 / KSPLIT) * RPW;
  dim3 grid((M + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK, batches);
  hipLaunchKernelGGL((gemv_kernel<RPW, KSPLIT>), grid, dim3(256), 0, s, W, x, y, M, K, repeat,
                     valid);
}

}  // namespace iron

using namespace iron;

extern "C" int iron_gemv_bf16_tuned(const uint16_t* W, const uint16_t* x, uint16_t* y, int M,
                                    int K, int batches, int repeat, const int* valid,
                                    int rows_per_wave, int k_split, void* stream) {
  IRON_REQUIRE(W && x && y, "gemv: null operand");
  IRON_REQUIRE(M > 0 && K > 0 && batches > 0, "gemv: M (%d), K (%d), batches (%d) must be positive",
               M, K, batches);
  IRON_REQUIRE(K % 8 == 0, "gemv: K (%d) must be a multiple of 8 (16-byte loads)", K);
  IRON_REQUIRE(repeat >= 1 && batches % repeat == 0,
               "gemv: repeat (%d) must divide batches (%d)", repeat, batches);
  IRON_REQUIRE(batches <= 65535, "gemv: batches (%d) exceed the grid's y extent", batches);
  // One vector, no row bound, rows of up to 8 KB, no launch shape asked for: the fused one-row
  // kernel's body with nothing fused (a block's 256 threads split K, every load a bounded buffer load
  // issued before any is used) measured 3-8 % faster at these sizes than the wave-per-rows kernel
  // below, and is the same sum bit for bit at K = 2048.
  if (rows_per_wave == 0 && k_split == 0 && batches == 1 && valid == nullptr && K <= 4096 &&
      (((uintptr_t)W | (uintptr_t)x) & 15) == 0)
    return iron_gemv_fused_bf16(W, nullptr, x, nullptr, 0.f, nullptr, 1.f, y, M, K, 0, stream);
  hipStream_t s = (hipStream_t)stream;
  int rpw = rows_per_wave, ks = k_split;
  if (rpw == 0 || ks == 0) {
    // Measured on MI355X under graph replay over weights larger than the last-level cache: the
    // four waves of a block splitting K (one contiguous row stream per block) win at every
    // size once a row is at least 2 KB; tall matrices of short rows take 2-4 rows a wave.
    const long rows = (long)M * batches;
    const int chunks = K / 8;
    ks = chunks >= 128 ? 4 : (chunks >= 64 ? 2 : 1);
    if (chunks >= 1024) rpw = 1;
    else rpw = rows >= 65536 ? 4 : (rows >= 8192 ? 2 : 1);
  }
  const bf16_t* Wp = W; const bf16_t* xp = x; bf16_t* yp = y;
#define IRON_GEMV_CASE(R, S)                                                   \
  if (rpw == R && ks == S) {                                                    \
    launch_gemv<R, S>(Wp, xp, yp, M, K, batches, repeat, valid, s);             \
    IRON_LAUNCH_CHECK();                                                        \
  }
  IRON_GEMV_CASE(1, 1) IRON_GEMV_CASE(1, 2) IRON_GEMV_CASE(1, 4)
  IRON_GEMV_CASE(2, 1) IRON_GEMV_CASE(2, 2) IRON_GEMV_CASE(2, 4)
  IRON_GEMV_CASE(4, 1) IRON_GEMV_CASE(4, 2) IRON_GEMV_CASE(4, 4)
  IRON_GEMV_CASE(8, 1)
#undef IRON_GEMV_CASE
  IRON_REQUIRE(false, "gemv: no kernel for rows_per_wave=%d, k_split=%d", rpw, ks);
}

extern "C" int iron_gemv_bf16(const uint16_t* W, const uint16_t* x, uint16_t* y, int M, int K,
                              int batches, int repeat, const int* valid, void* stream) {
  return iron_gemv_bf16_tuned(W, x, y, M, K, batches, repeat, valid, 0, 0, stream);
}
