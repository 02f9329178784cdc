// The operators the sibling decoders and their towers add to the hot path's: the unary
// activations (GELU, ReLU, Sigmoid, Tanh, Clamp), AXPY, LayerNorm and Softmax.  All stream their
// operands once in 16-byte pieces, compute in float32 and round once to bf16 (LayerNorm twice when
// weighted, as RMSNorm): bound by HBM.
#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {

// ------------------------------------------------------------------ unary
template <int KIND>
__device__ __forceinline__ float unary_apply(float v, float p0, float p1) {
  if (KIND == IRON_UNARY_GELU_TANH) return gelu_tanh_f32(v);
  if (KIND == IRON_UNARY_GELU_ERF) return 0.5f * v * (1.0f + erff(v * 0.7071067811865476f));
  if (KIND == IRON_UNARY_RELU) return v > 0.f ? v : 0.f;
  if (KIND == IRON_UNARY_SIGMOID) return 1.0f / (1.0f + __expf(-v));
  if (KIND == IRON_UNARY_TANH) return tanhf(v);
  return fminf(fmaxf(v, p0), p1);   // clamp
}

template <int KIND>
__global__ __launch_bounds__(256) void unary_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ y,
                                                    long n, float p0, float p1,
                                                    const int* __restrict__ valid) {
  if (valid != nullptr) {
    const long v = *valid;
    n = v < 0 ? 0 : (v < n ? v : n);
  }
  const long nchunk = n >> 3, stride = (long)gridDim.x * 256;
  const uint4* xv = reinterpret_cast<const uint4*>(x);
  uint4* yv = reinterpret_cast<uint4*>(y);
  for (long c = (long)blockIdx.x * 256 + threadIdx.x; c < nchunk; c += stride) {
    float f[8];
    unpack8(xv[c], f);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = unary_apply<KIND>(f[i], p0, p1);
    yv[c] = pack8(f);
  }
  if (blockIdx.x == 0) {   // the tail short of a 16-byte piece
    const long i = (nchunk << 3) + threadIdx.x;
    if (i < n) y[i] = f32_to_bf16(unary_apply<KIND>(bf16_to_f32(x[i]), p0, p1));
  }
}

__global__ __launch_bounds__(256) void axpy_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ y,
                                                   bf16_t* __restrict__ out, long n, float a,
                                                   const int* __restrict__ valid) {
  if (valid != nullptr) {
    const long v = *valid;
    n = v < 0 ? 0 : (v < n ? v : n);
  }
  const long nchunk = n >> 3, stride = (long)gridDim.x * 256;
  const uint4* xv = reinterpret_cast<const uint4*>(x);
  const uint4* yv = reinterpret_cast<const uint4*>(y);
  uint4* ov = reinterpret_cast<uint4*>(out);
  for (long c = (long)blockIdx.x * 256 + threadIdx.x; c < nchunk; c += stride) {
    float fx[8], fy[8];
    unpack8(xv[c], fx);
    unpack8(yv[c], fy);
#pragma unroll
    for (int i = 0; i < 8; ++i) fx[i] = fmaf(a, fx[i], fy[i]);
    ov[c] = pack8(fx);
  }
  if (blockIdx.x == 0) {
    const long i = (nchunk << 3) + threadIdx.x;
    if (i < n) out[i] = f32_to_bf16(fmaf(a, bf16_to_f32(x[i]), bf16_to_f32(y[i])));
  }
}

__device__ __forceinline__ float block_sum(float v, float* part) {
  v = wave_sum(v);
  __syncthreads();   // the parts' last readers are done
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
  __syncthreads();
  return part[0] + part[1] + part[2] + part[3];
}

__device__ __forceinline__ float block_max_f32(float v, float* part) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
}

// -------------------------------------------------------------- LayerNorm
// One block per row; a thread keeps up to CHUNKS 16-byte pieces of the row in registers between the
// mean, the variance about it and the scaling, so the row is read once (longer rows: the rest is
// read again from cache).  y = bf16((x - mean) / sqrt(var + eps)), then times the weight row and
// rounded again when there is one.
template <int CHUNKS>
__global__ __launch_bounds__(256) void layernorm_kernel(const bf16_t* __restrict__ x,
                                                        const bf16_t* __restrict__ w,
                                                        bf16_t* __restrict__ y, int rows, int cols,
                                                        float eps, const int* __restrict__ valid) {
  __shared__ float part[4];
  const int row = blockIdx.x;
  if (row >= bound_or(valid, rows)) return;
  const int nchunk = cols >> 3;
  const uint4* xr = reinterpret_cast<const uint4*>(x + (size_t)row * cols);
  uint4* yr = reinterpret_cast<uint4*>(y + (size_t)row * cols);
  const uint4* wr = reinterpret_cast<const uint4*>(w);

  // Every piece a thread keeps is asked for before any is used (as bounded loads: a thread past the
  // row's end reads zeros and takes no branch, behind which the compiler would wait for each load
  // where it stands).
  uint4 held[CHUNKS];
  const __amdgpu_buffer_rsrc_t row_bytes = bounded_bytes(xr, 2 * cols);
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) held[i] = load_bounded(row_bytes, 16 * ((int)threadIdx.x + i * 256));
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    float f[8];
    unpack8(held[i], f);   // zeros past the end add nothing
#pragma unroll
    for (int j = 0; j < 8; ++j) s += f[j];
  }
  for (int c = threadIdx.x + CHUNKS * 256; c < nchunk; c += 256) {
    float f[8];
    unpack8(xr[c], f);
#pragma unroll
    for (int j = 0; j < 8; ++j) s += f[j];
  }
  const float mean = block_sum(s, part) / (float)cols;
  float q = 0.f;
  auto spread = [&](const uint4& v) {
    float f[8];
    unpack8(v, f);
#pragma unroll
    for (int j = 0; j < 8; ++j) q = fmaf(f[j] - mean, f[j] - mean, q);
  };
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i)
    if (threadIdx.x + i * 256 < nchunk) spread(held[i]);
  for (int c = threadIdx.x + CHUNKS * 256; c < nchunk; c += 256) spread(xr[c]);
  const float inv = 1.0f / sqrtf(block_sum(q, part) / (float)cols + eps);

  auto emit = [&](int c, const uint4& v) {
    float f[8];
    unpack8(v, f);
    if (w != nullptr) {
      float g[8];
      unpack8(wr[c], g);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = round_bf16((f[j] - mean) * inv) * g[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = (f[j] - mean) * inv;
    }
    yr[c] = pack8(f);
  };
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i)
    if (threadIdx.x + i * 256 < nchunk) emit(threadIdx.x + i * 256, held[i]);
  for (int c = threadIdx.x + CHUNKS * 256; c < nchunk; c += 256) emit(c, xr[c]);
}

// ---------------------------------------------------------------- Softmax
// One block per row over its first `length` columns (a device word; the rest of the row is
// written zero): the logits (bf16, or float32 with F32) plus a float32 addend, soft-capped as
// cap * tanh(z / cap), then exp(z - max) / sum in float32 and one rounding.  A thread takes
// 8-column pieces; the first CHUNKS of them stay in registers from the maximum to the store (the
// row is read once), the pieces of a longer row are read and capped again from cache.
template <bool F32, int CHUNKS>
__global__ __launch_bounds__(256) void softmax_kernel(const void* __restrict__ x,
                                                      const float* __restrict__ addend,
                                                      bf16_t* __restrict__ y, int rows, int cols,
                                                      float soft_cap, const int* __restrict__ length) {
  __shared__ float part[4];
  const int row = blockIdx.x;
  const int n = bound_or(length, cols);
  const size_t base = (size_t)row * cols;
  const int pieces = cols >> 3, live = (n + 7) >> 3;   // pieces of the row, and those with a column under n
  // Piece c as it lies in memory (zeros past the row's end: the loads are bounded, no branch), and the
  // capped logits made of it; columns from n on are -inf (they weigh nothing).
  struct Raw {
    uint4 a, b;      // the piece's 8 logits: 16 bytes of bf16 (a), or 32 of float32 (a, b)
    uint4 pa, pb;    // the addend's 8 float32
  };
  const __amdgpu_buffer_rsrc_t x_row = bounded_bytes(reinterpret_cast<const char*>(x) + base * (F32 ? 4 : 2), cols * (F32 ? 4 : 2));
  const __amdgpu_buffer_rsrc_t add_row = bounded_bytes(addend != nullptr ? addend + base : nullptr, addend != nullptr ? cols * 4 : 0);
  auto fetch = [&](int c, Raw& r) {
    if (F32) {
      r.a = load_bounded(x_row, 32 * c);
      r.b = load_bounded(x_row, 32 * c + 16);
    } else {
      r.a = load_bounded(x_row, 16 * c);
    }
    if (addend != nullptr) {
      r.pa = load_bounded(add_row, 32 * c);
      r.pb = load_bounded(add_row, 32 * c + 16);
    }
  };
  auto capped = [&](int c, const Raw& r, float (&z)[8]) {
    if (F32) {
      z[0] = __uint_as_float(r.a.x); z[1] = __uint_as_float(r.a.y); z[2] = __uint_as_float(r.a.z); z[3] = __uint_as_float(r.a.w);
      z[4] = __uint_as_float(r.b.x); z[5] = __uint_as_float(r.b.y); z[6] = __uint_as_float(r.b.z); z[7] = __uint_as_float(r.b.w);
    } else {
      unpack8(r.a, z);
    }
    if (addend != nullptr) {
      z[0] += __uint_as_float(r.pa.x); z[1] += __uint_as_float(r.pa.y); z[2] += __uint_as_float(r.pa.z); z[3] += __uint_as_float(r.pa.w);
      z[4] += __uint_as_float(r.pb.x); z[5] += __uint_as_float(r.pb.y); z[6] += __uint_as_float(r.pb.z); z[7] += __uint_as_float(r.pb.w);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (soft_cap > 0.f) z[j] = soft_cap * tanhf(z[j] / soft_cap);
      if (8 * c + j >= n) z[j] = -INFINITY;
    }
  };
  auto logits = [&](int c, float (&z)[8]) {
    Raw r;
    fetch(c, r);
    capped(c, r, z);
  };
  // The pieces a thread keeps are all asked for before any is used.
  float held[CHUNKS][8];
  float m = -INFINITY;
  {
    Raw raw[CHUNKS];
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) fetch(threadIdx.x + i * 256, raw[i]);
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int c = threadIdx.x + i * 256;
      capped(c, raw[i], held[i]);   // -inf from column n on, so also for a thread past the live pieces
#pragma unroll
      for (int j = 0; j < 8; ++j) m = fmaxf(m, held[i][j]);
    }
  }
  for (int c = threadIdx.x + CHUNKS * 256; c < live; c += 256) {
    float z[8];
    logits(c, z);
#pragma unroll
    for (int j = 0; j < 8; ++j) m = fmaxf(m, z[j]);
  }
  m = block_max_f32(m, part);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    if (threadIdx.x + i * 256 < live) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        held[i][j] = __expf(held[i][j] - m);   // exp(-inf) = 0 past n
        s += held[i][j];
      }
    }
  }
  for (int c = threadIdx.x + CHUNKS * 256; c < live; c += 256) {
    float z[8];
    logits(c, z);
#pragma unroll
    for (int j = 0; j < 8; ++j) s += __expf(z[j] - m);
  }
  const float inv = 1.0f / block_sum(s, part);
  uint4* yr = reinterpret_cast<uint4*>(y + base);
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < live) {
#pragma unroll
      for (int j = 0; j < 8; ++j) held[i][j] *= inv;
      yr[c] = pack8(held[i]);
    }
  }
  for (int c = threadIdx.x + CHUNKS * 256; c < live; c += 256) {
    float z[8];
    logits(c, z);
#pragma unroll
    for (int j = 0; j < 8; ++j) z[j] = __expf(z[j] - m) * inv;
    yr[c] = pack8(z);
  }
  for (int c = live + threadIdx.x; c < pieces; c += 256) yr[c] = uint4{0, 0, 0, 0};
}

template <int KIND>
static void launch_unary(const uint16_t* x, uint16_t* y, int64_t n, float p0, float p1, const int* valid,
                         hipStream_t s) {
  long blocks = (((n + 7) >> 3) + 255) / 256;
  if (blocks > 256L * 16) blocks = 256L * 16;
  hipLaunchKernelGGL((unary_kernel<KIND>), dim3((unsigned)blocks), dim3(256), 0, s, x, y, (long)n, p0, p1, valid);
}

}  // namespace iron

using namespace iron;

extern "C" int iron_unary_bf16(const uint16_t* x, uint16_t* y, int64_t n, int kind, float p0, float p1,
                               const int* valid, void* stream) {
  IRON_REQUIRE(x && y, "unary: null operand");
  IRON_REQUIRE(n > 0, "unary: n (%lld) must be positive", (long long)n);
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)y) & 15) == 0, "unary: operands must be 16-byte aligned");
  IRON_REQUIRE(kind >= IRON_UNARY_GELU_TANH && kind <= IRON_UNARY_CLAMP, "unary: kind (%d) is not an IRON_UNARY_*", kind);
  IRON_REQUIRE(kind != IRON_UNARY_CLAMP || p0 <= p1, "unary: clamp's low (%g) exceeds its high (%g)", p0, p1);
  hipStream_t s = (hipStream_t)stream;
  switch (kind) {
    case IRON_UNARY_GELU_TANH: launch_unary<IRON_UNARY_GELU_TANH>(x, y, n, p0, p1, valid, s); break;
    case IRON_UNARY_GELU_ERF: launch_unary<IRON_UNARY_GELU_ERF>(x, y, n, p0, p1, valid, s); break;
    case IRON_UNARY_RELU: launch_unary<IRON_UNARY_RELU>(x, y, n, p0, p1, valid, s); break;
    case IRON_UNARY_SIGMOID: launch_unary<IRON_UNARY_SIGMOID>(x, y, n, p0, p1, valid, s); break;
    case IRON_UNARY_TANH: launch_unary<IRON_UNARY_TANH>(x, y, n, p0, p1, valid, s); break;
    default: launch_unary<IRON_UNARY_CLAMP>(x, y, n, p0, p1, valid, s); break;
  }
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_axpy_bf16(const uint16_t* x, const uint16_t* y, uint16_t* out, int64_t n, float a,
                              const int* valid, void* stream) {
  IRON_REQUIRE(x && y && out, "axpy: null operand");
  IRON_REQUIRE(n > 0, "axpy: n (%lld) must be positive", (long long)n);
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)y | (uintptr_t)out) & 15) == 0, "axpy: operands must be 16-byte aligned");
  long blocks = (((n + 7) >> 3) + 255) / 256;
  if (blocks > 256L * 16) blocks = 256L * 16;
  hipLaunchKernelGGL(axpy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, x, y, out, (long)n, a,
                     valid);
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_layernorm_bf16(const uint16_t* x, const uint16_t* w, uint16_t* y, int rows, int cols,
                                   float eps, const int* valid, void* stream) {
  IRON_REQUIRE(x && y, "layernorm: null operand");
  IRON_REQUIRE(rows > 0 && cols > 0, "layernorm: rows (%d) and cols (%d) must be positive", rows, cols);
  IRON_REQUIRE(cols % 8 == 0, "layernorm: cols (%d) must be a multiple of 8", cols);
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) == 0, "layernorm: operands must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  if (cols <= 2048)
    hipLaunchKernelGGL((layernorm_kernel<1>), dim3(rows), dim3(256), 0, s, x, w, y, rows, cols, eps, valid);
  else if (cols <= 4096)
    hipLaunchKernelGGL((layernorm_kernel<2>), dim3(rows), dim3(256), 0, s, x, w, y, rows, cols, eps, valid);
  else
    hipLaunchKernelGGL((layernorm_kernel<4>), dim3(rows), dim3(256), 0, s, x, w, y, rows, cols, eps, valid);
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_softmax_bf16(const void* x, int x_is_f32, const float* addend, uint16_t* y, int rows,
                                 int cols, float soft_cap, const int* length, void* stream) {
  IRON_REQUIRE(x && y, "softmax: null operand");
  IRON_REQUIRE(rows > 0 && cols > 0 && cols % 8 == 0, "softmax: rows (%d) positive, cols (%d) a positive multiple of 8",
               rows, cols);
  IRON_REQUIRE(soft_cap >= 0.f, "softmax: soft_cap (%g) must be positive, or 0 for none", soft_cap);
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)addend | (uintptr_t)y) & 15) == 0, "softmax: operands must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const bool wide = cols > 2048;
  if (x_is_f32) {
    if (wide)
      hipLaunchKernelGGL((softmax_kernel<true, 4>), dim3(rows), dim3(256), 0, s, x, addend, y, rows, cols, soft_cap, length);
    else
      hipLaunchKernelGGL((softmax_kernel<true, 1>), dim3(rows), dim3(256), 0, s, x, addend, y, rows, cols, soft_cap, length);
  } else {
    if (wide)
      hipLaunchKernelGGL((softmax_kernel<false, 4>), dim3(rows), dim3(256), 0, s, x, addend, y, rows, cols, soft_cap, length);
    else
      hipLaunchKernelGGL((softmax_kernel<false, 1>), dim3(rows), dim3(256), 0, s, x, addend, y, rows, cols, soft_cap, length);
  }
  IRON_LAUNCH_CHECK();
}
