// Shared device helpers for the gfx950 (CDNA4, wave64) kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#define IRON_OK 0
#define IRON_EINVAL 1

namespace iron {

constexpr int kWave = 64;

// Set by an entry point that refuses its arguments; read back by iron_last_error().
void set_error(const char* fmt, ...);

#define IRON_REQUIRE(cond, ...)        \
  do {                                 \
    if (!(cond)) {                     \
      ::iron::set_error(__VA_ARGS__);  \
      return IRON_EINVAL;              \
    }                                  \
  } while (0)

#define IRON_LAUNCH_CHECK()                          \
  do {                                               \
    hipError_t e__ = hipPeekAtLastError();           \
    if (e__ != hipSuccess) {                         \
      ::iron::set_error("%s", hipGetErrorString(e__)); \
      return (int)e__;                               \
    }                                                \
    return IRON_OK;                                  \
  } while (0)

// A kernel's opt-in to more dynamic LDS than a launch gets by default.  The attribute belongs to a
// device's copy of the function, so it is set once per device (that device current), from whichever
// host thread gets there first; two that race both set it, which is harmless.
struct LdsOptIn {
  std::atomic<uint64_t> done{0};
  hipError_t ensure(const void* kernel, size_t bytes) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (device & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
  }
};

typedef uint16_t bf16_t;  // storage

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

__device__ __forceinline__ float bf16_to_f32(bf16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) {
  return __builtin_bit_cast(float, w & 0xffff0000u);
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// Two floats -> packed bf16, round to nearest even, in hardware (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return (bf16_t)(pack_bf16(f, 0.f) & 0xffffu); }
// Round a float to the nearest bf16 and return it as float.
__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

__device__ __forceinline__ void unpack8(const uint4& v, float (&f)[8]) {
  f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x);
  f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
  f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z);
  f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
  uint4 v;
  v.x = pack_bf16(f[0], f[1]); v.y = pack_bf16(f[2], f[3]);
  v.z = pack_bf16(f[4], f[5]); v.w = pack_bf16(f[6], f[7]);
  return v;
}

// SiLU, and GELU by its tanh form, as every kernel here computes them, so that fused and separate
// launches round alike.
// (the quotient by the hardware's reciprocal, an ulp off the division's: a gated GEMM's epilogue runs
// this 64 times a thread with nothing left to hide it under)
__device__ __forceinline__ float silu_f32(float v) { return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v)); }
__device__ __forceinline__ float gelu_tanh_f32(float v) {
  const float inner = 0.7978845608028654f * (v + 0.044715f * v * v * v);
  return 0.5f * v * (1.0f + tanhf(inner));
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
// 16-byte streaming load that does not displace reusable lines in the caches.
__device__ __forceinline__ uint4 load_stream(const uint4* p) {
  u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
// `bytes` bytes as a bounded buffer: a 16-byte load at an offset past their end returns zeros, so a
// thread with no chunk of a row takes no branch around its load.  (Behind such a branch the compiler
// waits for the load where it stands, to move what arrived into the register the join expects, and
// a kernel's loads that were to be in flight together become one trip to memory after another.)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t bounded_bytes(const void* base, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ __forceinline__ uint4 load_bounded(__amdgpu_buffer_rsrc_t run, int offset) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(run, offset, 0, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint4 load_bounded_stream(__amdgpu_buffer_rsrc_t run, int offset) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(run, offset, 0, 2);   // 2: non-temporal
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store_stream(uint4* p, const uint4& v) {
  u32x4 w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(p));
}

// Wave-wide reductions on the DPP data path (no LDS traffic): within quads, half rows and
// rows, then across rows with the row broadcasts; lane 63 ends with the total.
#define IRON_DPP(old, v, ctrl, rows) \
  __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v), ctrl, rows, 0xF, false))
__device__ __forceinline__ float wave_sum(float v) {
  v += IRON_DPP(0.f, v, 0xB1, 0xF);   // quad_perm [1,0,3,2]
  v += IRON_DPP(0.f, v, 0x4E, 0xF);   // quad_perm [2,3,0,1]
  v += IRON_DPP(0.f, v, 0x141, 0xF);  // row_half_mirror
  v += IRON_DPP(0.f, v, 0x140, 0xF);  // row_mirror: every lane of a row holds the row's sum
  v += IRON_DPP(0.f, v, 0x142, 0xA);  // row_bcast15 into rows 1 and 3
  v += IRON_DPP(0.f, v, 0x143, 0xC);  // row_bcast31 into rows 2 and 3
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, IRON_DPP(v, v, 0xB1, 0xF));
  v = fmaxf(v, IRON_DPP(v, v, 0x4E, 0xF));
  v = fmaxf(v, IRON_DPP(v, v, 0x141, 0xF));
  v = fmaxf(v, IRON_DPP(v, v, 0x140, 0xF));
  v = fmaxf(v, IRON_DPP(v, v, 0x142, 0xA));
  v = fmaxf(v, IRON_DPP(v, v, 0x143, 0xC));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// Sum over each aligned group of 8 lanes (every lane of the group gets it).
__device__ __forceinline__ float group8_sum(float v) {
  v += IRON_DPP(0.f, v, 0xB1, 0xF);
  v += IRON_DPP(0.f, v, 0x4E, 0xF);
  v += IRON_DPP(0.f, v, 0x141, 0xF);
  return v;
}
// ... and of 16 lanes (a DPP row).
__device__ __forceinline__ float group16_sum(float v) {
  v = group8_sum(v);
  v += IRON_DPP(0.f, v, 0x140, 0xF);
  return v;
}

// A per-call bound read from device memory; a null pointer reads as `whole`.
__device__ __forceinline__ int bound_or(const int* p, int whole) {
  if (p == nullptr) return whole;
  int v = *p;
  return v < 0 ? 0 : (v > whole ? whole : v);
}

// ---- direct-to-LDS pipelines
#define IRON_GLOBAL_PTR(p) ((const void __attribute__((address_space(1)))*)(p))
#define IRON_LDS_PTR(p) ((void __attribute__((address_space(3)))*)(p))

// Rows of a matrix from `base` on as a raw buffer (no stride, 2 GiB of reach, 32-bit data): what a
// buffer load into LDS addresses with a 32-bit offset a lane.  `base` must be uniform over the wave.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t stage_rows(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
}

// acc += a b on the 16x16x32 MFMA, the accumulator held in place in accumulation registers.  As a
// builtin, sixty-four 4-register accumulators live across a loop make the register allocator
// rotate them through copies (some 200 moves an iteration); a tied operand leaves it no choice.
typedef int i32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void mfma_16x16x32_in_place(f32x4& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
               : "+a"(acc)
               : "v"(__builtin_bit_cast(i32x4, a)), "v"(__builtin_bit_cast(i32x4, b)));
}

__device__ __forceinline__ void block_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // gfx9 encoding: vmcnt = bits [3:0] and [15:14]; expcnt and lgkmcnt left at "no wait".
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}


typedef short short4v __attribute__((ext_vector_type(4)));

// The transposing LDS read, as inline assembly: through the builtin the compiler cannot tell the
// read from the direct-to-LDS loads in flight and waits for all of them (vmcnt(0)) before each
// one, which drains the prefetch.  The compiler does not count these reads, so their consumer
// must pass the results through lds_tr_wait() first.
__device__ __forceinline__ short4v lds_read_tr16(unsigned lds_addr) {
  short4v v;
  asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(lds_addr));
  return v;
}
// The same with a compile-time byte offset in the instruction's offset field (no address arithmetic).
template <int OFFSET>
__device__ __forceinline__ short4v lds_read_tr16_at(unsigned lds_addr) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "the offset field holds 16 bits");
  short4v v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(lds_addr), "n"(OFFSET));
  return v;
}
// A 16-byte LDS read the compiler does not count (for loops that also issue the reads above: the
// waits it would insert count only the reads it knows, so they come out too strict and wait for
// reads issued long after the one that is needed).  The result must pass through lds_wait_for<N>().
template <int OFFSET>
__device__ __forceinline__ bf16x8 lds_read_b128_at(unsigned lds_addr) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "the offset field holds 16 bits");
  i32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(lds_addr), "n"(OFFSET));
  return __builtin_bit_cast(bf16x8, v);
}
// Waits until at most N LDS reads issued after `frag`'s are outstanding (they return in order).
template <int N>
__device__ __forceinline__ void lds_wait_for(bf16x8& frag) {
  static_assert(N >= 0 && N <= 15, "the counter's field holds four bits");
  i32x4 v = __builtin_bit_cast(i32x4, frag);
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(N));
  frag = __builtin_bit_cast(bf16x8, v);
}
struct TrFrag {   // the two halves of a fragment, as the reads deliver them
  short4v lo, hi;
};
// Waits for every LDS read issued so far; the halves pass through it so that nothing derived from
// them (not even a register copy) can be scheduled before the wait.
__device__ __forceinline__ void lds_tr_wait(TrFrag& a, TrFrag& b) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi));
}
__device__ __forceinline__ bf16x8 tr_join(const TrFrag& f) {
  typedef short short8v __attribute__((ext_vector_type(8)));
  const short8v both = __builtin_shufflevector(f.lo, f.hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, both);
}


}  // namespace iron
