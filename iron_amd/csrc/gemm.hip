// GEMM: C = A @ B in bf16 on the MFMA matrix cores, f32 accumulation, one rounding.
//
// A block of 4 waves computes a BM x BN tile of C.  Per 64-wide K step the block
// stages a BM x 64 tile of A and a BN x 64 tile of B in LDS (both K-contiguous,
// rows padded to 72 elements so the 16-byte fragment reads of 32 consecutive rows
// fall in distinct banks), double-buffered: the global loads of step k+1 are in
// flight while the MFMAs of step k run.  A wave owns a (BM/WM) x (BN/WN) sub-tile
// as 32x32 MFMA tiles (v_mfma_f32_32x32x16_bf16: a lane supplies 8 consecutive k of
// one row of each operand).
//
// B as stored by a checkpoint, (N,K), is already K-contiguous.  B as (K,N) is
// transposed on its way into LDS: a thread loads a 4(k) x 8(n) patch and writes
// eight 8-byte k-runs.
//
// For a row-major C the MFMA is issued with the operands swapped (B tile as the
// "A" operand), so a lane ends up holding 4 consecutive columns of one row of C
// and stores them as 8 bytes.
#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {

constexpr int BK = 64;
constexpr int LDK = BK + 8;  // padded LDS row, in elements

// Zero the elements of an 8-element piece from index keep on.
__device__ __forceinline__ uint4 keep_first(uint4 v, int keep) {
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (2 * i >= keep) w[i] = 0;
    else if (2 * i + 1 >= keep) w[i] &= 0xffffu;
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

template <int BM, int BN, int WM, int WN, bool B_NK, bool C_NM>
__global__ __launch_bounds__(256) void gemm_kernel(const bf16_t* __restrict__ A,
                                                   const bf16_t* __restrict__ B,
                                                   bf16_t* __restrict__ C, int M, int N, int K,
                                                   const int* __restrict__ valid,
                                                   const int* __restrict__ valid_k, int tiles_m,
                                                   int tiles_n) {
  static_assert(WM * WN == 4, "4 waves");
  constexpr int TM = BM / WM / 32;  // MFMA tiles per wave along M
  constexpr int TN = BN / WN / 32;
  constexpr int A_PIECES = BM * (BK / 8) / 256;  // 16-byte pieces a thread loads of A
  constexpr int B_PIECES = BN * (BK / 8) / 256;

  extern __shared__ __align__(16) bf16_t smem[];
  bf16_t* As = smem;                  // [2][BM][LDK]
  bf16_t* Bs = smem + 2 * BM * LDK;   // [2][BN][LDK]

  const int Mv = bound_or(valid, M);
  const int Kv = bound_or(valid_k, K);

  // Tile order: consecutive blocks share a band of 8 tile rows, so the blocks
  // resident together re-read few panels of A and B from L2.
  int tm, tn;
  {
    const int bid = blockIdx.x;
    constexpr int BAND = 8;
    const int per_band = BAND * tiles_n;
    const int band = bid / per_band;
    const int first = band * BAND;
    const int height = min(BAND, tiles_m - first);
    const int in_band = bid - band * per_band;
    tm = first + in_band % height;
    tn = in_band / height;
  }
  const int m0 = tm * BM, n0 = tn * BN;
  if (m0 >= Mv) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  // (K,N) B: a pass covers 256/(BN/8) groups of 4 k rows; BK/4 groups make a tile.
  constexpr int B_NC = BN / 8;
  constexpr int B_KG = 256 / B_NC;
  constexpr int B_PASSES = (BK / 4 + B_KG - 1) / B_KG;
  uint4 a_reg[A_PIECES];
  uint4 b_reg[B_NK ? B_PIECES : 4 * B_PASSES];

  auto load_a = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_PIECES; ++i) {
      const int p = tid + i * 256;
      const int row = p >> 3, kc = (p & 7) * 8;
      const int gm = m0 + row, gk = k0 + kc;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (gm < Mv && gk < Kv) {
        v = *reinterpret_cast<const uint4*>(A + (size_t)gm * K + gk);
        if (gk + 8 > Kv) v = keep_first(v, Kv - gk);
      }
      a_reg[i] = v;
    }
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_PIECES; ++i) {
      const int p = tid + i * 256;
      const int row = p >> 3, kc = (p & 7) * 8;
      *reinterpret_cast<uint4*>(As + (buf * BM + row) * LDK + kc) = a_reg[i];
    }
  };
  auto load_b = [&](int k0) {
    if constexpr (B_NK) {
#pragma unroll
      for (int i = 0; i < B_PIECES; ++i) {
        const int p = tid + i * 256;
        const int row = p >> 3, kc = (p & 7) * 8;
        const int gn = n0 + row, gk = k0 + kc;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (gn < N && gk < Kv) {
          v = *reinterpret_cast<const uint4*>(B + (size_t)gn * K + gk);
          if (gk + 8 > Kv) v = keep_first(v, Kv - gk);
        }
        b_reg[i] = v;
      }
    } else {
      // A thread takes 4 consecutive k rows of one 8-column strip per pass.
#pragma unroll
      for (int j = 0; j < B_PASSES; ++j) {
        const int strip = tid % B_NC;
        const int kg = tid / B_NC + j * B_KG;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int gk = k0 + kg * 4 + r, gn = n0 + strip * 8;
          uint4 v = make_uint4(0, 0, 0, 0);
          if (kg < BK / 4 && gk < Kv && gn < N) {
            if (gn + 8 <= N) {
              v = *reinterpret_cast<const uint4*>(B + (size_t)gk * N + gn);
            } else {
              // N is not a multiple of 8 here only if the caller passed such an N;
              // read the columns that exist one by one.
              uint32_t w[4] = {0, 0, 0, 0};
              for (int c = 0; c < N - gn; ++c)
                w[c >> 1] |= (uint32_t)B[(size_t)gk * N + gn + c] << (16 * (c & 1));
              v = make_uint4(w[0], w[1], w[2], w[3]);
            }
          }
          b_reg[j * 4 + r] = v;
        }
      }
    }
  };
  auto store_b = [&](int buf) {
    if constexpr (B_NK) {
#pragma unroll
      for (int i = 0; i < B_PIECES; ++i) {
        const int p = tid + i * 256;
        const int row = p >> 3, kc = (p & 7) * 8;
        *reinterpret_cast<uint4*>(Bs + (buf * BN + row) * LDK + kc) = b_reg[i];
      }
    } else {
#pragma unroll
      for (int j = 0; j < B_PASSES; ++j) {
        const int strip = tid % B_NC;
        const int kg = tid / B_NC + j * B_KG;
        if (kg >= BK / 4) continue;
        const uint4 r0 = b_reg[j * 4 + 0], r1 = b_reg[j * 4 + 1], r2 = b_reg[j * 4 + 2],
                    r3 = b_reg[j * 4 + 3];
        const uint32_t w0[4] = {r0.x, r0.y, r0.z, r0.w}, w1[4] = {r1.x, r1.y, r1.z, r1.w},
                       w2[4] = {r2.x, r2.y, r2.z, r2.w}, w3[4] = {r3.x, r3.y, r3.z, r3.w};
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          // Column c of the strip: its 4 k values, k ascending.
          const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
          uint2 out;
          out.x = __builtin_amdgcn_perm(w1[c >> 1], w0[c >> 1], sel);
          out.y = __builtin_amdgcn_perm(w3[c >> 1], w2[c >> 1], sel);
          *reinterpret_cast<uint2*>(Bs + (buf * BN + strip * 8 + c) * LDK + kg * 4) = out;
        }
      }
    }
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int nk = (Kv + BK - 1) / BK;
  if (nk > 0) {
    load_a(0);
    load_b(0);
    store_a(0);
    store_b(0);
  }
  __syncthreads();

  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      load_a((kt + 1) * BK);
      load_b((kt + 1) * BK);
    }
    const bf16_t* Ab = As + (cur * BM + wm * (BM / WM) + frag_row) * LDK + frag_k;
    const bf16_t* Bb = Bs + (cur * BN + wn * (BN / WN) + frag_row) * LDK + frag_k;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const bf16x8*>(Ab + i * 32 * LDK + ks * 16);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bfr[j] = *reinterpret_cast<const bf16x8*>(Bb + j * 32 * LDK + ks * 16);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          if constexpr (C_NM)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[i][j], 0, 0, 0);
        }
    }
    if (kt + 1 < nk) {
      store_a(cur ^ 1);
      store_b(cur ^ 1);
    }
    __syncthreads();
  }

  // Epilogue.  Swapped operands (row-major C): lane holds row m = lane%32 and the
  // 4-column runs n = 8*q + 4*(lane/32) + 0..3, q = 0..3.  Unswapped (C as (N,M)):
  // lane holds column n = lane%32 and the 4-row runs of m.
  const int hi = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int mb = m0 + wm * (BM / WM) + i * 32;
      const int nb = n0 + wn * (BN / WN) + j * 32;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float v0 = acc[i][j][4 * q + 0], v1 = acc[i][j][4 * q + 1],
                    v2 = acc[i][j][4 * q + 2], v3 = acc[i][j][4 * q + 3];
        if constexpr (!C_NM) {
          const int m = mb + frag_row, n = nb + 8 * q + hi;
          if (m >= Mv || n >= N) continue;
          bf16_t* p = C + (size_t)m * N + n;
          if (n + 4 <= N && (N & 3) == 0) {
            *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16(v0, v1), pack_bf16(v2, v3));
          } else {
            const float v[4] = {v0, v1, v2, v3};
            for (int e = 0; e < 4 && n + e < N; ++e) p[e] = f32_to_bf16(v[e]);
          }
        } else {
          const int n = nb + frag_row, m = mb + 8 * q + hi;
          if (n >= N || m >= Mv) continue;
          bf16_t* p = C + (size_t)n * M + m;
          if (m + 4 <= Mv && (M & 3) == 0) {
            *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16(v0, v1), pack_bf16(v2, v3));
          } else {
            const float v[4] = {v0, v1, v2, v3};
            for (int e = 0; e < 4 && m + e < Mv; ++e) p[e] = f32_to_bf16(v[e]);
          }
        }
      }
    }
}

template <int BM, int BN, int WM, int WN>
static int launch_gemm(const bf16_t* A, const bf16_t* B, bf16_t* C, int M, int N, int K, int b_nk,
                       int c_nm, const int* valid, const int* valid_k, hipStream_t s) {
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const size_t lds = (size_t)2 * (BM + BN) * LDK * sizeof(bf16_t);
  dim3 grid(tiles_m * tiles_n), block(256);
#define IRON_GEMM_LAUNCH(BNK, CNM)                                                          \
  do {                                                                                      \
    auto kern = gemm_kernel<BM, BN, WM, WN, BNK, CNM>;                                      \
    static bool once = false;                                                               \
    if (!once) {                                                                            \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),               \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e != hipSuccess) { set_error("gemm: %s", hipGetErrorString(e)); return (int)e; }  \
      once = true;                                                                          \
    }                                                                                       \
    hipLaunchKernelGGL(kern, grid, block, lds, s, A, B, C, M, N, K, valid, valid_k, tiles_m, \
                       tiles_n);                                                            \
  } while (0)
  if (b_nk && c_nm) IRON_GEMM_LAUNCH(true, true);
  else if (b_nk) IRON_GEMM_LAUNCH(true, false);
  else if (c_nm) IRON_GEMM_LAUNCH(false, true);
  else IRON_GEMM_LAUNCH(false, false);
#undef IRON_GEMM_LAUNCH
  IRON_LAUNCH_CHECK();
}

}  // namespace iron

using namespace iron;

extern "C" int iron_gemm_bf16(const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K,
                              int b_col_maj, int c_col_maj, const int* valid, const int* valid_k,
                              void* stream) {
  IRON_REQUIRE(A && B && C, "gemm: null operand");
  IRON_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: M (%d), N (%d), K (%d) must be positive", M, N, K);
  IRON_REQUIRE(K % 8 == 0, "gemm: K (%d) must be a multiple of 8 (16-byte loads)", K);
  IRON_REQUIRE((((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) == 0,
               "gemm: operands must be 16-byte aligned");
  IRON_REQUIRE(b_col_maj || N % 8 == 0,
               "gemm: N (%d) must be a multiple of 8 when B is (K,N) (16-byte loads along N)", N);
  hipStream_t s = (hipStream_t)stream;
  // 128x128 tiles fill the 256 CUs once at 2048x2048; narrower problems take 64-wide tiles.
  const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
  if (tiles128 >= 128 || (M >= 128 && N >= 128))
    return launch_gemm<128, 128, 2, 2>(A, B, C, M, N, K, b_col_maj, c_col_maj, valid, valid_k, s);
  return launch_gemm<64, 64, 2, 2>(A, B, C, M, N, K, b_col_maj, c_col_maj, valid, valid_k, s);
}
