// Exact data movers and the per-call word machinery: row gather (embedding
// lookup), row copy between views with per-call offsets (KV-cache write, RoPE
// table row, last-row pick), greedy argmax draw, and the device-side evaluation
// of per-call words that lets a captured decode step advance itself.
#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {

// One block per row; rows are row_bytes long, moved as 16-byte pieces where both
// ends are aligned, else as 4-byte words.
__device__ __forceinline__ void move_row(const char* __restrict__ s, char* __restrict__ d,
                                         long row_bytes) {
  if ((((uintptr_t)s | (uintptr_t)d | (uintptr_t)row_bytes) & 15) == 0) {
    const uint4* sv = reinterpret_cast<const uint4*>(s);
    uint4* dv = reinterpret_cast<uint4*>(d);
    for (long i = threadIdx.x; i < (row_bytes >> 4); i += blockDim.x) dv[i] = sv[i];
  } else {
    const uint32_t* sv = reinterpret_cast<const uint32_t*>(s);
    uint32_t* dv = reinterpret_cast<uint32_t*>(d);
    for (long i = threadIdx.x; i < (row_bytes >> 2); i += blockDim.x) dv[i] = sv[i];
  }
}

__global__ __launch_bounds__(256) void gather_rows_kernel(const char* __restrict__ table,
                                                          const int* __restrict__ ids,
                                                          char* __restrict__ out, int n_ids,
                                                          int table_rows, long row_bytes,
                                                          const int* __restrict__ valid) {
  const int n = bound_or(valid, n_ids);
  for (int i = blockIdx.x; i < n; i += gridDim.x) {
    const int id = ids[i];
    if (id < 0 || id >= table_rows) continue;
    move_row(table + (size_t)id * row_bytes, out + (size_t)i * row_bytes, row_bytes);
  }
}

__global__ __launch_bounds__(256) void copy_rows_kernel(const char* __restrict__ src,
                                                        char* __restrict__ dst, int rows,
                                                        long row_bytes, long src_stride,
                                                        long dst_stride, int src_rows, int dst_rows,
                                                        const int* __restrict__ src_row,
                                                        const int* __restrict__ dst_row,
                                                        const int* __restrict__ valid) {
  const int n = bound_or(valid, rows);
  const long s0 = src_row ? *src_row : 0;
  const long d0 = dst_row ? *dst_row : 0;
  for (int i = blockIdx.x; i < n; i += gridDim.x) {
    const long s = s0 + i, d = d0 + i;
    if (s < 0 || s >= src_rows || d < 0 || d >= dst_rows) continue;
    move_row(src + s * src_stride, dst + d * dst_stride, row_bytes);
  }
}

// First index of the largest value: larger value wins, then the smaller index.
struct Best {
  float v;
  int i;
};
__device__ __forceinline__ Best better(Best a, Best b) {
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

__global__ __launch_bounds__(1024) void argmax_kernel(const bf16_t* __restrict__ logits, int n,
                                                      int* __restrict__ token,
                                                      int* __restrict__ record, int record_len,
                                                      const int* __restrict__ at,
                                                      int* __restrict__ token_copy) {
  Best best{-INFINITY, 0x7fffffff};
  const int nchunk = n >> 3;
  const uint4* lv = reinterpret_cast<const uint4*>(logits);
  for (int c = threadIdx.x; c < nchunk; c += 1024) {
    float f[8];
    unpack8(lv[c], f);
#pragma unroll
    for (int j = 0; j < 8; ++j) best = better(best, Best{f[j], c * 8 + j});
  }
  for (int i = (nchunk << 3) + threadIdx.x; i < n; i += 1024)
    best = better(best, Best{bf16_to_f32(logits[i]), i});
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    Best other{__shfl_xor(best.v, o, 64), __shfl_xor(best.i, o, 64)};
    best = better(best, other);
  }
  __shared__ float sv[16];
  __shared__ int si[16];
  if ((threadIdx.x & 63) == 0) {
    sv[threadIdx.x >> 6] = best.v;
    si[threadIdx.x >> 6] = best.i;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    Best b{sv[0], si[0]};
    for (int w = 1; w < 16; ++w) b = better(b, Best{sv[w], si[w]});
    // Every logit NaN or -inf: index 0, as a scan from the left would leave it.
    int tok = b.i == 0x7fffffff ? 0 : b.i;
    *token = tok;
    if (token_copy != nullptr) *token_copy = tok;
    if (record != nullptr) {
      int where = at ? *at : 0;
      if (where >= 0 && where < record_len) record[where] = tok;
    }
  }
}

__global__ void eval_words_kernel(int* __restrict__ words, int n_words,
                                  const int* __restrict__ exprs, int n) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  for (int e = 0; e < n; ++e) {
    const int* x = exprs + 9 * e;
    const int dst = x[0], src = x[1];
    if (dst < 0 || dst >= n_words || src < 0 || src >= n_words) continue;
    long v = ((long)words[src] * x[2] + x[3]) >> x[4];
    v = v < x[5] ? x[5] : (v > x[6] ? x[6] : v);
    words[dst] = ((int)v & x[7]) + x[8];
  }
}

}  // namespace iron

using namespace iron;

extern "C" int iron_gather_rows(const void* table, const int* ids, void* out, int n_ids,
                                int table_rows, int64_t row_bytes, const int* valid, void* stream) {
  IRON_REQUIRE(table && ids && out, "gather_rows: null operand");
  IRON_REQUIRE(n_ids > 0 && table_rows > 0, "gather_rows: n_ids (%d) and table_rows (%d) must be positive",
               n_ids, table_rows);
  IRON_REQUIRE(row_bytes > 0 && row_bytes % 4 == 0, "gather_rows: row_bytes (%lld) must be a positive multiple of 4",
               (long long)row_bytes);
  IRON_REQUIRE((((uintptr_t)table | (uintptr_t)out) & 3) == 0, "gather_rows: operands must be 4-byte aligned");
  unsigned blocks = n_ids < 65535 ? n_ids : 65535;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                     (const char*)table, ids, (char*)out, n_ids, table_rows, (long)row_bytes, valid);
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_copy_rows(const void* src, void* dst, int rows, int64_t row_bytes,
                              int64_t src_stride, int64_t dst_stride, int src_rows, int dst_rows,
                              const int* src_row, const int* dst_row, const int* valid,
                              void* stream) {
  IRON_REQUIRE(src && dst, "copy_rows: null operand");
  IRON_REQUIRE(rows > 0 && src_rows > 0 && dst_rows > 0, "copy_rows: rows (%d), src_rows (%d), dst_rows (%d) must be positive",
               rows, src_rows, dst_rows);
  IRON_REQUIRE(row_bytes > 0 && row_bytes % 4 == 0, "copy_rows: row_bytes (%lld) must be a positive multiple of 4",
               (long long)row_bytes);
  IRON_REQUIRE(src_stride >= row_bytes && dst_stride >= row_bytes && src_stride % 4 == 0 && dst_stride % 4 == 0,
               "copy_rows: strides (%lld, %lld) must be multiples of 4 no shorter than a row (%lld)",
               (long long)src_stride, (long long)dst_stride, (long long)row_bytes);
  IRON_REQUIRE((((uintptr_t)src | (uintptr_t)dst) & 3) == 0, "copy_rows: operands must be 4-byte aligned");
  unsigned blocks = rows < 65535 ? rows : 65535;
  hipLaunchKernelGGL(copy_rows_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                     (const char*)src, (char*)dst, rows, (long)row_bytes, (long)src_stride,
                     (long)dst_stride, src_rows, dst_rows, src_row, dst_row, valid);
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_argmax_bf16(const uint16_t* logits, int n, int* token, int* record,
                                int record_len, const int* at, int* token_copy, void* stream) {
  IRON_REQUIRE(logits && token, "argmax: null operand");
  IRON_REQUIRE(n > 0, "argmax: n (%d) must be positive", n);
  IRON_REQUIRE(((uintptr_t)logits & 15) == 0, "argmax: logits must be 16-byte aligned");
  hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, logits, n, token,
                     record, record_len, at, token_copy);
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_eval_words(int* words, int n_words, const int* exprs, int n, void* stream) {
  IRON_REQUIRE(words && exprs, "eval_words: null operand");
  IRON_REQUIRE(n_words > 0 && n > 0, "eval_words: n_words (%d) and n (%d) must be positive", n_words, n);
  hipLaunchKernelGGL(eval_words_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, words, n_words,
                     exprs, n);
  IRON_LAUNCH_CHECK();
}
