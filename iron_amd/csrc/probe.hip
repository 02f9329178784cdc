// Measurement aid, no counterpart in the reference: the bf16 MFMA rate this GPU sustains from
// registers alone, with operands the caller provides.  The published dense peak assumes the top
// clock; under a power cap the clock an MFMA-bound kernel runs at depends on how many operand
// bits toggle, so the ceiling for real (random) data sits well below the ceiling for constants.
// A GEMM's MFMA utilisation is read against both.
#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {

__global__ __launch_bounds__(256) void probe_mfma_kernel(const uint32_t* __restrict__ operands,
                                                         int operand_words, float* __restrict__ sink,
                                                         int iters) {
  const int tid = threadIdx.x + blockIdx.x * 256;
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint4 va = make_uint4(0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u), vb = va;  // constants
    if (operands) {
      const uint32_t* p = operands + ((size_t)tid * 32 + i * 8) % (size_t)(operand_words - 8);
      va = make_uint4(p[0], p[1], p[2], p[3]);
      vb = make_uint4(p[4], p[5], p[6], p[7]);
    }
    a[i] = __builtin_bit_cast(bf16x8, va);
    b[i] = __builtin_bit_cast(bf16x8, vb);
  }
  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  sink[tid] = s;
}

}  // namespace iron

using namespace iron;

extern "C" int64_t iron_probe_mfma_flops(int iters) {
  return (int64_t)IRON_PROBE_BLOCKS * 4 * 16 * 32768 * (int64_t)iters;
}

extern "C" int iron_probe_mfma_bf16(const uint16_t* operands, int64_t operand_count, float* sink,
                                    int iters, void* stream) {
  IRON_REQUIRE(sink, "probe_mfma: null sink");
  IRON_REQUIRE(iters > 0, "probe_mfma: iters (%d) must be positive", iters);
  IRON_REQUIRE(operands == nullptr || (operand_count >= 64 && operand_count / 2 < (1ll << 30)),
               "probe_mfma: operands need at least 64 values");
  IRON_REQUIRE((((uintptr_t)operands | (uintptr_t)sink) & 3) == 0, "probe_mfma: operands must be 4-byte aligned");
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(IRON_PROBE_BLOCKS), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<const uint32_t*>(operands), (int)(operand_count / 2), sink, iters);
  IRON_LAUNCH_CHECK();
}
