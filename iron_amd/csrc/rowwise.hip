// One-pass streaming kernels: RMSNorm (optionally weighted), RoPE, and the
// elementwise SiLU / mul / add / SiLU*mul.  All HBM-bandwidth bound: 16-byte
// loads and stores, f32 math, one rounding to bf16 per reference step.
#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {

// ---------------------------------------------------------------- RMSNorm
// One block per row.  A thread keeps up to CHUNKS 16-byte pieces of the row in
// registers between the sum of squares and the scaling, so the row is read once.
template <int CHUNKS>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const bf16_t* __restrict__ x,
                                                      const bf16_t* __restrict__ w,
                                                      bf16_t* __restrict__ y, int rows, int cols,
                                                      float eps, const int* __restrict__ valid,
                                                      const bf16_t* residual) {
  const int row = blockIdx.x;
  const int nchunk = cols >> 3;
  const uint4* wr = reinterpret_cast<const uint4*>(w);
  // The gains do not depend on the row or on the bound: their trip to memory goes out with the
  // bound's own instead of after the row's sum (three dependent trips a launch were two too many).
  uint4 gains[CHUNKS];
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    const int c = threadIdx.x + i * 256;
    gains[i] = (w != nullptr && c < nchunk) ? wr[c] : make_uint4(0, 0, 0, 0);
  }
  if (row >= bound_or(valid, rows)) return;
  const uint4* xr = reinterpret_cast<const uint4*>(x + (size_t)row * cols);
  uint4* yr = reinterpret_cast<uint4*>(y + (size_t)row * cols);
  // A residual (which y may be) the normed row is added to, rounded as the separate sum rounds.
  const uint4* rr = reinterpret_cast<const uint4*>(residual + (residual ? (size_t)row * cols : 0));

  uint4 held[CHUNKS], added[CHUNKS];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    const int c = threadIdx.x + i * 256;
    held[i] = c < nchunk ? xr[c] : make_uint4(0, 0, 0, 0);
    added[i] = (residual != nullptr && c < nchunk) ? rr[c] : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    float f[8];
    unpack8(held[i], f);
#pragma unroll
    for (int j = 0; j < 8; ++j) ss = fmaf(f[j], f[j], ss);
  }
  // Rows longer than CHUNKS*2048 elements: the rest is summed here and re-read below.
  for (int c = threadIdx.x + CHUNKS * 256; c < nchunk; c += 256) {
    float f[8];
    unpack8(xr[c], f);
#pragma unroll
    for (int j = 0; j < 8; ++j) ss = fmaf(f[j], f[j], ss);
  }
  ss = wave_sum(ss);
  __shared__ float part[4];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float total = part[0] + part[1] + part[2] + part[3];
  const float inv = 1.0f / sqrtf(total / (float)cols + eps);

  auto emit = [&](int c, const uint4& v, const uint4& gain, const uint4& add) {
    float f[8];
    unpack8(v, f);
    if (w != nullptr) {
      float g[8];
      unpack8(gain, g);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = round_bf16(f[j] * inv) * g[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = f[j] * inv;
    }
    if (residual != nullptr) {
      float r[8];
      unpack8(add, r);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = r[j] + round_bf16(f[j]);
    }
    yr[c] = pack8(f);
  };
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    int c = threadIdx.x + i * 256;
    if (c < nchunk) emit(c, held[i], gains[i], added[i]);
  }
  for (int c = threadIdx.x + CHUNKS * 256; c < nchunk; c += 256)
    emit(c, xr[c], w != nullptr ? wr[c] : make_uint4(0, 0, 0, 0), residual != nullptr ? rr[c] : make_uint4(0, 0, 0, 0));
}

// ------------------------------------------------------------------- RoPE
// A thread rotates 8 column pairs of one row: with two halves, columns
// [8j, 8j+8) of each half; interleaved, columns [16j, 16j+16).
template <bool TWO_HALVES>
__global__ __launch_bounds__(256) void rope_kernel(const bf16_t* __restrict__ x,
                                                   const bf16_t* __restrict__ angles,
                                                   bf16_t* __restrict__ y, int rows, int cols,
                                                   int rows_per_angle,
                                                   const int* __restrict__ valid, int row_cols) {
  const int per_row = cols >> 4;  // threads a row takes
  const long t = (long)blockIdx.x * 256 + threadIdx.x;
  const long row = t / per_row;
  const int j = (int)(t - row * per_row);
  if (row >= bound_or(valid, rows)) return;
  const int arow = (int)(row / rows_per_angle);
  // 8 (cos, sin) pairs: 16 bf16 = two 16-byte loads.
  const uint4* av = reinterpret_cast<const uint4*>(angles + (size_t)arow * cols + 16 * j);
  float cs0[8], cs1[8];
  unpack8(av[0], cs0);
  unpack8(av[1], cs1);
  float c[8] = {cs0[0], cs0[2], cs0[4], cs0[6], cs1[0], cs1[2], cs1[4], cs1[6]};
  float s[8] = {cs0[1], cs0[3], cs0[5], cs0[7], cs1[1], cs1[3], cs1[5], cs1[7]};
  // A row is row_cols wide, of which the first cols turn; the rest passes through unchanged
  // (a decoder whose RoPE covers part of each head), 16 bytes at a time over the row's threads.
  const bf16_t* xr = x + (size_t)row * row_cols;
  bf16_t* yr = y + (size_t)row * row_cols;
  for (int c = cols + 8 * j; c < row_cols; c += 8 * per_row)
    *reinterpret_cast<uint4*>(yr + c) = *reinterpret_cast<const uint4*>(xr + c);
  float a[8], b[8], oa[8], ob[8];
  if (TWO_HALVES) {
    const int half = cols >> 1;
    unpack8(*reinterpret_cast<const uint4*>(xr + 8 * j), a);
    unpack8(*reinterpret_cast<const uint4*>(xr + half + 8 * j), b);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      oa[i] = a[i] * c[i] - b[i] * s[i];
      ob[i] = b[i] * c[i] + a[i] * s[i];
    }
    *reinterpret_cast<uint4*>(yr + 8 * j) = pack8(oa);
    *reinterpret_cast<uint4*>(yr + half + 8 * j) = pack8(ob);
  } else {
    float lo[8], hi[8];
    unpack8(*reinterpret_cast<const uint4*>(xr + 16 * j), lo);
    unpack8(*reinterpret_cast<const uint4*>(xr + 16 * j + 8), hi);
    float e[8] = {lo[0], lo[2], lo[4], lo[6], hi[0], hi[2], hi[4], hi[6]};
    float o[8] = {lo[1], lo[3], lo[5], lo[7], hi[1], hi[3], hi[5], hi[7]};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      oa[i] = e[i] * c[i] - o[i] * s[i];
      ob[i] = o[i] * c[i] + e[i] * s[i];
    }
    float r0[8] = {oa[0], ob[0], oa[1], ob[1], oa[2], ob[2], oa[3], ob[3]};
    float r1[8] = {oa[4], ob[4], oa[5], ob[5], oa[6], ob[6], oa[7], ob[7]};
    *reinterpret_cast<uint4*>(yr + 16 * j) = pack8(r0);
    *reinterpret_cast<uint4*>(yr + 16 * j + 8) = pack8(r1);
  }
}

// ------------------------------------------------------------ elementwise
enum class Ew { kSilu, kMul, kAdd, kSiluMul };


template <Ew OP>
__device__ __forceinline__ float ew_apply(float a, float b) {
  if (OP == Ew::kSilu) return silu_f32(a);
  if (OP == Ew::kMul) return a * b;
  if (OP == Ew::kAdd) return a + b;
  return round_bf16(silu_f32(a)) * b;
}

template <Ew OP>
__global__ __launch_bounds__(256) void ew_kernel(const bf16_t* __restrict__ a,
                                                 const bf16_t* __restrict__ b,
                                                 bf16_t* __restrict__ y, long n,
                                                 const int* __restrict__ valid) {
  if (valid != nullptr) {
    long v = *valid;
    n = v < 0 ? 0 : (v < n ? v : n);
  }
  const long nchunk = n >> 3;
  const long stride = (long)gridDim.x * 256;
  const uint4* av = reinterpret_cast<const uint4*>(a);
  const uint4* bv = reinterpret_cast<const uint4*>(b);
  uint4* yv = reinterpret_cast<uint4*>(y);
  for (long c = (long)blockIdx.x * 256 + threadIdx.x; c < nchunk; c += stride) {
    float fa[8], fb[8], fy[8];
    unpack8(av[c], fa);
    if (OP != Ew::kSilu) unpack8(bv[c], fb);
#pragma unroll
    for (int i = 0; i < 8; ++i) fy[i] = ew_apply<OP>(fa[i], OP != Ew::kSilu ? fb[i] : 0.f);
    yv[c] = pack8(fy);
  }
  // The tail short of a 16-byte piece.
  if (blockIdx.x == 0) {
    long i = (nchunk << 3) + threadIdx.x;
    if (i < n) {
      float fa = bf16_to_f32(a[i]);
      float fb = OP != Ew::kSilu ? bf16_to_f32(b[i]) : 0.f;
      y[i] = f32_to_bf16(ew_apply<OP>(fa, fb));
    }
  }
}

template <Ew OP>
static int launch_ew(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t n, const int* valid,
                     void* stream, const char* name) {
  IRON_REQUIRE(a && y && (OP == Ew::kSilu || b), "%s: null operand", name);
  IRON_REQUIRE(n > 0, "%s: n (%lld) must be positive", name, (long long)n);
  IRON_REQUIRE((((uintptr_t)a | (uintptr_t)b | (uintptr_t)y) & 15) == 0,
               "%s: operands must be 16-byte aligned", name);
  long chunks = (n + 7) >> 3;
  long blocks = (chunks + 255) / 256;
  if (blocks > 256L * 16) blocks = 256L * 16;  // grid-stride beyond 16 blocks a CU
  hipLaunchKernelGGL((ew_kernel<OP>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a,
                     b, y, (long)n, valid);
  IRON_LAUNCH_CHECK();
}


// Every row of x (rows, cols) met elementwise by the one row `row` (cols): a projection's bias
// (add) or a per-column scale (mul).  A thread takes 16-byte pieces; the piece of `row` it needs
// stays in L1/L2.  `valid` bounds the rows.
template <Ew OP>
__global__ __launch_bounds__(256) void row_broadcast_kernel(const bf16_t* __restrict__ x,
                                                            const bf16_t* __restrict__ row,
                                                            bf16_t* __restrict__ y, int rows, int cols,
                                                            const int* __restrict__ valid) {
  rows = bound_or(valid, rows);
  const int cpr = cols >> 3;                 // 16-byte pieces a row has
  const long nchunk = (long)rows * cpr;
  const long stride = (long)gridDim.x * 256;
  const uint4* xv = reinterpret_cast<const uint4*>(x);
  const uint4* rv = reinterpret_cast<const uint4*>(row);
  uint4* yv = reinterpret_cast<uint4*>(y);
  for (long c = (long)blockIdx.x * 256 + threadIdx.x; c < nchunk; c += stride) {
    float fa[8], fb[8], fy[8];
    unpack8(xv[c], fa);
    unpack8(rv[c % cpr], fb);
#pragma unroll
    for (int i = 0; i < 8; ++i) fy[i] = ew_apply<OP>(fa[i], fb[i]);
    yv[c] = pack8(fy);
  }
}

}  // namespace iron

using namespace iron;

static int rmsnorm(const uint16_t* x, const uint16_t* w, const uint16_t* residual, uint16_t* y, int rows, int cols,
                   float eps, const int* valid, void* stream) {
  IRON_REQUIRE(x && y, "rmsnorm: null operand");
  IRON_REQUIRE(((uintptr_t)residual & 15) == 0, "rmsnorm: operands must be 16-byte aligned");
  IRON_REQUIRE(rows > 0 && cols > 0, "rmsnorm: rows (%d) and cols (%d) must be positive", rows, cols);
  IRON_REQUIRE(cols % 8 == 0, "rmsnorm: cols (%d) must be a multiple of 8", cols);
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) == 0,
               "rmsnorm: operands must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  if (cols <= 2048)
    hipLaunchKernelGGL((rmsnorm_kernel<1>), dim3(rows), dim3(256), 0, s, x, w, y, rows, cols, eps, valid, residual);
  else if (cols <= 4096)
    hipLaunchKernelGGL((rmsnorm_kernel<2>), dim3(rows), dim3(256), 0, s, x, w, y, rows, cols, eps, valid, residual);
  else
    hipLaunchKernelGGL((rmsnorm_kernel<4>), dim3(rows), dim3(256), 0, s, x, w, y, rows, cols, eps, valid, residual);
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_rmsnorm_bf16(const uint16_t* x, const uint16_t* w, uint16_t* y, int rows,
                                 int cols, float eps, const int* valid, void* stream) {
  return rmsnorm(x, w, nullptr, y, rows, cols, eps, valid, stream);
}

extern "C" int iron_rmsnorm_add_bf16(const uint16_t* x, const uint16_t* w, const uint16_t* residual,
                                     uint16_t* y, int rows, int cols, float eps, const int* valid,
                                     void* stream) {
  IRON_REQUIRE(residual, "rmsnorm_add: null residual");
  return rmsnorm(x, w, residual, y, rows, cols, eps, valid, stream);
}

static int rope_launch(const uint16_t* x, const uint16_t* angles, uint16_t* y, int rows, int row_cols, int cols,
                       int angle_rows, int two_halves, const int* valid, void* stream) {
  IRON_REQUIRE(x && angles && y, "rope: null operand");
  IRON_REQUIRE(rows > 0 && cols > 0 && angle_rows > 0,
               "rope: rows (%d), cols (%d), angle_rows (%d) must be positive", rows, cols, angle_rows);
  IRON_REQUIRE(cols % 16 == 0, "rope: cols (%d) must be a multiple of 16", cols);
  IRON_REQUIRE(row_cols >= cols && (row_cols - cols) % 8 == 0,
               "rope: a row of %d columns of which %d turn: the rest must be a multiple of 8", row_cols, cols);
  IRON_REQUIRE(angle_rows <= rows && rows % angle_rows == 0,
               "rope: angle_rows (%d) must divide rows (%d)", angle_rows, rows);
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)angles | (uintptr_t)y) & 15) == 0,
               "rope: operands must be 16-byte aligned");
  const long threads = (long)rows * (cols >> 4);
  const unsigned blocks = (unsigned)((threads + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (two_halves)
    hipLaunchKernelGGL((rope_kernel<true>), dim3(blocks), dim3(256), 0, s, x, angles, y, rows, cols,
                       rows / angle_rows, valid, row_cols);
  else
    hipLaunchKernelGGL((rope_kernel<false>), dim3(blocks), dim3(256), 0, s, x, angles, y, rows, cols,
                       rows / angle_rows, valid, row_cols);
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_rope_bf16(const uint16_t* x, const uint16_t* angles, uint16_t* y, int rows,
                              int cols, int angle_rows, int two_halves, const int* valid,
                              void* stream) {
  return rope_launch(x, angles, y, rows, cols, cols, angle_rows, two_halves, valid, stream);
}

extern "C" int iron_rope_partial_bf16(const uint16_t* x, const uint16_t* angles, uint16_t* y, int rows,
                                      int row_cols, int rotary_cols, int angle_rows, int two_halves,
                                      const int* valid, void* stream) {
  return rope_launch(x, angles, y, rows, row_cols, rotary_cols, angle_rows, two_halves, valid, stream);
}

extern "C" int iron_silu_bf16(const uint16_t* x, uint16_t* y, int64_t n, const int* valid,
                              void* stream) {
  return launch_ew<Ew::kSilu>(x, nullptr, y, n, valid, stream, "silu");
}
extern "C" int iron_mul_bf16(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t n,
                             const int* valid, void* stream) {
  return launch_ew<Ew::kMul>(a, b, y, n, valid, stream, "mul");
}
extern "C" int iron_add_bf16(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t n,
                             const int* valid, void* stream) {
  return launch_ew<Ew::kAdd>(a, b, y, n, valid, stream, "add");
}
extern "C" int iron_silu_mul_bf16(const uint16_t* g, const uint16_t* u, uint16_t* y, int64_t n,
                                  const int* valid, void* stream) {
  return launch_ew<Ew::kSiluMul>(g, u, y, n, valid, stream, "silu_mul");
}

extern "C" int iron_row_broadcast_bf16(const uint16_t* x, const uint16_t* row, uint16_t* y, int rows,
                                       int cols, int multiply, const int* valid, void* stream) {
  IRON_REQUIRE(x && row && y, "row_broadcast: null operand");
  IRON_REQUIRE(rows > 0 && cols > 0 && cols % 8 == 0,
               "row_broadcast: rows (%d) positive, cols (%d) a positive multiple of 8", rows, cols);
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)row | (uintptr_t)y) & 15) == 0,
               "row_broadcast: operands must be 16-byte aligned");
  long chunks = (long)rows * (cols >> 3);
  long blocks = (chunks + 255) / 256;
  if (blocks > 256L * 16) blocks = 256L * 16;
  if (multiply)
    hipLaunchKernelGGL((row_broadcast_kernel<Ew::kMul>), dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, x, row, y, rows, cols, valid);
  else
    hipLaunchKernelGGL((row_broadcast_kernel<Ew::kAdd>), dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, x, row, y, rows, cols, valid);
  IRON_LAUNCH_CHECK();
}
