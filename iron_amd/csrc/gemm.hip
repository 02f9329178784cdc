// GEMM: C = A @ B in bf16 on the MFMA matrix cores, f32 accumulation, one rounding.
//
// Two families of kernels.  The general one (gemm_kernel, first below) takes every shape and
// option: a block of 4 waves computes a BM x BN tile of C; per 64-wide K step it stages a BM x 64
// tile of A and a BN x 64 tile of B in LDS through registers (both K-contiguous, rows padded to
// 72 elements so the 16-byte fragment reads of 32 consecutive rows fall in distinct banks),
// double-buffered; a wave owns a (BM/WM) x (BN/WN) sub-tile as 32x32x16 MFMA tiles; B as (K,N) is
// transposed on its way into LDS (a thread loads a 4(k) x 8(n) patch and writes eight 8-byte
// k-runs).  The fast ones (K a multiple of 64, row-major C) feed LDS straight from global memory
// and come in four tile sizes: 64 x 64, 128 x 128, 128 x 192 / 128 x 64 for the fused projections,
// and 256 x 256; each is described where it stands.
//
// For a row-major C the MFMA is issued with the operands swapped (B tile as the "A" operand), so a
// lane ends up holding 4 consecutive columns of one row of C and stores them as 8 bytes.
#include "../../include/iron_hip.h"
#include "common.h"

#include <type_traits>


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
#pragma unroll
            for (int e = 0; e < 4; ++e)   // (constant indices: a runtime trip count puts the array in scratch memory)
              if (n + e < N) p[e] = f32_to_bf16(v[e]);
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


// ---------------------------------------------------------------------------
// Fast paths: A (M,K) K-contiguous, K a multiple of 64, row-major C.
//
// Tiles stream global -> LDS directly (buffer loads with the LDS bit: no VGPR staging, and the
// L2 -> CU path delivers more per clock to LDS than to registers), several stages deep.  A wave
// instruction moves 8 rows x 128 B; the 16-byte chunk a lane fetches is XOR-swizzled by its row
// ((row >> 1) & 7) so the fragment reads of 16 consecutive rows fall in distinct bank groups
// although LDS rows are unpadded.  The stage barrier is a bare s_barrier: the fence
// __syncthreads() carries would wait for every outstanding load (vmcnt(0)) and drain the
// prefetch; each wave instead waits until only the younger stages are in flight.
constexpr int NT_STAGES = 4;
constexpr int PAIR_STAGES = 3;   // of the two-product body: 48 KB each

// B_KN (128 x 128 and 256 x 256 tiles): B is (K,N) row-major.  Its tile lands in LDS as stored, a
// row a k (a wave instruction moves 4 k-rows x 256 B, or 2 x 512 B; chunks swizzled by the row so
// that the four rows of a 16-lane group, and the groups of a pass, lie in different banks), and
// the fragments are fetched with the transposing LDS read (ds_read_b64_tr_b16): within 16 lanes,
// lane i points at 4 consecutive n of row k0 + i/4 and receives k0..k0+3 of column n0 + i%16.
// QKV: one launch for a prompt chunk's three projections and the rotation of two of them.  B, C and
// N then stand for q's weight (N,K), output and width; `qkv` brings k's and v's (each kv_n wide,
// widths multiples of the 128-column tile) and the chunk's angle rows (M, 64; cos and sin
// interleaved).  A block's tile column picks its matrix.  With 64-wide heads a wave's 64 columns are
// one head whose two halves are its two accumulator tiles, so q and k are rotated in registers:
// rounded to bf16 as the projection would store them, turned (two halves), rounded again.
struct QkvTail {
  const bf16_t* Bk;
  const bf16_t* Bv;
  bf16_t* Ck;
  bf16_t* Cv;
  const bf16_t* angles;
  int kv_n;
  // Not of the fused projections: a plain product's epilogue, C = bf16(residual_scale * bf16(A B) + residual)
  // (one fused multiply-add; residual (M, N) like C), when residual is not NULL.
  const bf16_t* residual;
  float residual_scale;
  // ... or, with gated set, C = bf16(bf16(act(residual)) * bf16(A B)): `residual` then holds a gated
  // feed-forward's other product, and this one leaves as the activated gate times it (1: SiLU,
  // 2: GELU by its tanh form).
  int gated;
  // Of the fused projections again: Ck and Cv are KV caches of kv_rows rows (a row kv_n wide, as the
  // projections write one), and the chunk's rows go to rows *kv_row0 on, when kv_row0 is not NULL.
  const int* kv_row0;
  int kv_rows;
  // Of a plain product on the 128 x 128 tiles, one block of several that share a tile's K: columns
  // k_begin .. k_begin + k_len of A and B (k_len 0: all of them), the float32 sums left at `partial`
  // (an (M, N) array of this slice's) instead of C; tile_plus1: the tile's number + 1 where the
  // kernel deals tiles itself instead of by the block's id.
  int k_begin, k_len, tile_plus1;
  float* partial;
};

__device__ __forceinline__ float gate_of(int kind, float g) { return kind == 2 ? gelu_tanh_f32(g) : silu_f32(g); }

// The k and v outputs moved to the chunk's rows of their caches.  The first row is held where the
// rows under the bound still end inside the cache, whatever the word holds.
__device__ __forceinline__ void to_cache_rows(QkvTail& t, const int* __restrict__ valid, int M) {
  if (t.kv_row0 == nullptr) return;
  const int rows = bound_or(valid, M);
  const int first = max(0, min(*t.kv_row0, t.kv_rows - rows));
  t.Ck += (size_t)first * t.kv_n;
  t.Cv += (size_t)first * t.kv_n;
}

// Which tile a block computes.  Blocks are dispatched in id order and dealt round-robin over the 8
// XCDs, each with an L2 of its own, so the order is chosen for what an XCD's blocks share:
// `patched` (whole 8 x 4-tile patches, a multiple of 8 of them): an XCD owns patches, whose A and B
// panels it re-reads from its own L2.  Few tile rows (under 8, and a multiple of 8 tile columns,
// e.g. the 512 live rows of a prompt chunk): an XCD owns whole columns of tiles, so the weight tile
// its blocks share crosses HBM once instead of once an XCD.  Otherwise bands of 8 tile rows.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int patched, int& tm, int& tn) {
  if (patched) {
    const int xcd = bid & 7, loc = bid >> 3;
    const int patch = (loc >> 5) * 8 + xcd, within = loc & 31;
    const int patches_n = tiles_n >> 2;
    tm = (patch / patches_n) * 8 + (within & 7);
    tn = (patch % patches_n) * 4 + (within >> 3);
  } else if (tiles_m < 8 && (tiles_n & 7) == 0) {
    const int xcd = bid & 7, loc = bid >> 3;
    tm = loc % tiles_m;
    tn = (loc / tiles_m) * 8 + xcd;
  } else {
    constexpr int BAND = 8;
    const int per_band = BAND * tiles_n, band = bid / per_band, first = band * BAND;
    const int height = min(BAND, tiles_m - first), in_band = bid - band * per_band;
    tm = first + in_band % height;
    tn = in_band / height;
  }
}

// 64 x 64 tiles, B as (N,K), for problems -- or row bounds -- whose 128 x 128 tiles would leave CUs
// idle (k/v projections, short chunks): the direct-to-LDS pipeline of the 128 x 128 kernel below
// (buffer loads, XOR-swizzled chunks) with a wave owning one 32x32x16 MFMA tile.  A stage is four
// MFMAs of a wave, far less than an LDS read takes to return, so the fragments of a WHOLE stage
// are read one stage ahead into a second register set: at the top of stage kt the stage's one
// barrier (stage kt+1 has landed in every wave, and nobody reads stage kt-1 any more), then the
// eight fragment reads of stage kt+1, the loads of stage kt+STAGES-1 into stage kt-1's buffer, and
// stage kt's four MFMAs out of registers on two accumulators (even and odd k-steps, so that no MFMA
// waits for the one before it).  Reading a k-step ahead, as the larger tiles do, left every MFMA
// waiting for its operands: 600 cycles a stage.  STAGES = 4 (64 KB: a CU holds two blocks) where
// the tiles outnumber the CUs, 8 (128 KB, more loads in flight) where a CU has one block anyway.
// `qkv` carries only the optional residual epilogue here.
template <int STAGES>
__device__ __forceinline__ void gemm_nt64_body(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B,
                                               bf16_t* __restrict__ C, int M, int N, int K,
                                               const int* __restrict__ valid, int tiles_m, int tiles_n,
                                               int patched, const QkvTail& qkv) {
  constexpr int NT_BM = 64, NT_BN = 64;
  constexpr int NT_A_BYTES = NT_BM * BK * 2, NT_STAGE_BYTES = (NT_BM + NT_BN) * BK * 2;
  constexpr int INST = NT_BM / 8 / 4;  // 1 KB loads of A (and of B) a wave issues per stage
  constexpr int LOADS = 2 * INST;
  constexpr int KSTEPS = BK / 16;
  static_assert(LOADS == KSTEPS && STAGES >= 4, "one load rides each k-step's MFMA");
  extern __shared__ __align__(16) char smem_nt[];
  const int Mv = bound_or(valid, M);

  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, patched, tm, tn);
  const int m0 = tm * NT_BM, n0 = tn * NT_BN;
  if (m0 >= Mv) return;

  // The wave's number is uniform, so what depends on it (LDS destinations, the rows it loads) stays
  // in scalar registers.
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane >> 3, pch = lane & 7;
  int a_voff[INST], b_voff[INST];
#pragma unroll
  for (int i = 0; i < INST; ++i) {
    const int r = (wave * INST + i) * 8 + lrow;
    const int lch = pch ^ ((r >> 1) & 7);
    // Rows past the end re-read the last row; what they produce is never stored.
    a_voff[i] = (int)(((size_t)(min(m0 + r, M - 1) - m0) * K + lch * 8) * 2);
    b_voff[i] = (int)(((size_t)(min(n0 + r, N - 1) - n0) * K + lch * 8) * 2);
  }
  const bf16_t* a_tile = A + (size_t)m0 * K;
  const bf16_t* b_tile = B + (size_t)n0 * K;
  // One load of the 2*INST a wave issues per stage (A's first, then B's).
  auto issue_one = [&](char* st, int kt, int idx) {
    const int k0 = kt * BK;
    if (idx < INST) {
      const __amdgpu_buffer_rsrc_t rows = stage_rows(a_tile + k0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rows, IRON_LDS_PTR(st + (wave * INST + idx) * 1024), 16,
                                               (int)a_voff[idx], 0, 0, 0);
    } else {
      const __amdgpu_buffer_rsrc_t rows = stage_rows(b_tile + k0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rows, IRON_LDS_PTR(st + NT_A_BYTES + (wave * INST + idx - INST) * 1024),
                                               16, (int)b_voff[idx - INST], 0, 0, 0);
    }
  };

  f32x16 acc[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[h][e] = 0.f;

  // acc[e]: row fr of the wave's tile, column 8 (e/4) + 4 kh + e%4.
  const int fr = lane & 31, kh = lane >> 5;
  const int m = m0 + wm * 32 + fr, nb = n0 + wn * 32 + 4 * kh;
  // A residual's pieces this lane will add in the epilogue are requested now, so that their
  // latency passes under the whole product instead of at its end (N a multiple of 4: 8-byte pieces).
  uint2 res[4];
  const bool res_ahead = qkv.residual != nullptr && (N & 3) == 0;
  if (res_ahead) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      res[q] = *reinterpret_cast<const uint2*>(qkv.residual + (size_t)min(m, M - 1) * N + min(nb + 8 * q, N - 4));
  }

  const int nk = K / BK;
  // Always STAGES-1 stages in flight before the loop (short K repeats its last stage), so the
  // loop's wait counts hold from the first iteration.
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
#pragma unroll
    for (int idx = 0; idx < LOADS; ++idx) issue_one(smem_nt + s * NT_STAGE_BYTES, min(s, nk - 1), idx);

  const int ra = wm * 32 + fr, rb = wn * 32 + fr;
  const int a_off = ra * 128, a_swz = (ra >> 1) & 7, b_off = NT_A_BYTES + rb * 128, b_swz = (rb >> 1) & 7;
  auto a_frag = [&](const char* st, int ks) {
    return *reinterpret_cast<const bf16x8*>(st + a_off + (((ks * 2 + kh) ^ a_swz) << 4));
  };
  auto b_frag = [&](const char* st, int ks) {
    return *reinterpret_cast<const bf16x8*>(st + b_off + (((ks * 2 + kh) ^ b_swz) << 4));
  };

  wait_vmcnt<(STAGES - 2) * LOADS>();   // stage 0 has landed once only the younger ones are out
  block_barrier();
  bf16x8 af[2][KSTEPS], bfr[2][KSTEPS];   // [stage parity][k-step]
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) { af[0][ks] = a_frag(smem_nt, ks); bfr[0][ks] = b_frag(smem_nt, ks); }
  // Two stages an iteration, so that the register sets are named at compile time.
  auto stage = [&](int kt, auto parity) {
    constexpr int P = decltype(parity)::value;
    // Of this wave's loads in flight the oldest LOADS are stage kt+1's; the STAGES-3 stages after it may stay out.
    wait_vmcnt<(STAGES - 3) * LOADS>();
    block_barrier();
    const char* st1 = smem_nt + ((kt + 1) % STAGES) * NT_STAGE_BYTES;     // past the end: a stage nobody needs
    char* nst = smem_nt + ((kt + STAGES - 1) % STAGES) * NT_STAGE_BYTES;  // stage kt-1's buffer
    const int kn = min(kt + STAGES - 1, nk - 1);   // past the end the last stage again: the wait counts stay exact
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      acc[ks & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[P][ks], af[P][ks], acc[ks & 1], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      af[P ^ 1][ks] = a_frag(st1, ks);
      bfr[P ^ 1][ks] = b_frag(st1, ks);
      issue_one(nst, kn, ks);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // (Unrolled over all its stage buffers, so that a fragment's stage rides in its read's offset
  // field as in the 128 x 128 loop, this loop measured the same: it waits for L2, not for issue slots.)
  int kt = 0;
  for (; kt + 1 < nk; kt += 2) {
    stage(kt, std::integral_constant<int, 0>{});
    stage(kt + 1, std::integral_constant<int, 1>{});
  }
  if (kt < nk) stage(kt, std::integral_constant<int, 0>{});

  wait_vmcnt<0>();  // the idle fetches of the last iterations land before the block's LDS is released
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[0][e] += acc[1][e];
  const bool vec = (N & 3) == 0;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int n = nb + 8 * q;
    if (m >= Mv || n >= N) continue;
    bf16_t* p = C + (size_t)m * N + n;
    if (qkv.residual != nullptr) {   // the product rounded as it would be stored, then scale * it + residual
      const bf16_t* r = qkv.residual + (size_t)m * N + n;
      float rf[4] = {0.f, 0.f, 0.f, 0.f};
      if (vec && n + 4 <= N) {
        const uint2 rv = res_ahead ? res[q] : *reinterpret_cast<const uint2*>(r);
        rf[0] = __uint_as_float(rv.x << 16); rf[1] = __uint_as_float(rv.x & 0xffff0000u);
        rf[2] = __uint_as_float(rv.y << 16); rf[3] = __uint_as_float(rv.y & 0xffff0000u);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) rf[e] = bf16_to_f32(r[e]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float prod = round_bf16(acc[0][4 * q + e]);
        acc[0][4 * q + e] = qkv.gated ? round_bf16(gate_of(qkv.gated, rf[e])) * prod : fmaf(qkv.residual_scale, prod, rf[e]);
      }
    }
    if (vec && n + 4 <= N) {
      *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16(acc[0][4 * q], acc[0][4 * q + 1]),
                                                pack_bf16(acc[0][4 * q + 2], acc[0][4 * q + 3]));
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < N) p[e] = f32_to_bf16(acc[0][4 * q + e]);
    }
  }
}

// 128 x 128 x 64 tiles, four stages of 32 KB fed straight from global memory into LDS (buffer loads:
// the tile's rows from the stage's k on are the buffer, rebuilt per stage with scalar instructions,
// a lane's place in it a constant 32-bit offset, so a load costs one scalar add for its LDS
// destination and no vector ALU work between two MFMAs); 16-byte chunks XOR-swizzled by the row so
// unpadded rows read conflict-free; a bare s_barrier and counted s_waitcnt vmcnt(N).  Four waves, a
// wave's 64 x 64 as 4 x 4 tiles of 16x16x32 MFMAs (two 32-wide k-steps a stage; the part sustains
// more of these under its power limit than of the 32x32x16 form), accumulators tied in place.  A
// wave is alone on its SIMD, so its own instruction stream interleaves: after an MFMA one fragment
// read of the next k-step or one prefetch load goes out, and the stage's one barrier sits before
// its second k-step, whose fragments are in registers by then.  B as (N,K), or as (K,N): then the
// stage lands as stored and the B operands come from transposing reads.  The output is staged
// through LDS so that it leaves as whole 128-byte row segments (16 bytes a lane).  QKV: the fused
// projections' per-tile choice of weight and output, RoPE on the accumulators.  Otherwise `qkv`
// carries the optional residual epilogue.
template <bool QKV, bool B_KN = false>
__device__ __forceinline__ void gemm_nt16_body(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B_,
                                               bf16_t* __restrict__ C_, int M, int N_, int K,
                                               const int* __restrict__ valid, int tiles_m, int tiles_n,
                                               int patched, const QkvTail& qkv) {
  constexpr int NT_BM = 128, NT_BN = 128;
  constexpr int NT_A_BYTES = NT_BM * BK * 2, NT_STAGE_BYTES = (NT_BM + NT_BN) * BK * 2;
  constexpr int INST = NT_BM / 8 / 4;  // 1 KB loads of A (and of B) a wave issues per stage
  constexpr int LOADS = 2 * INST;
  static_assert(BK == 64 && INST == 4, "two 32-wide k-steps a stage, eight loads a wave");
  static_assert(!(B_KN && QKV), "the fused projections read weights as stored, (N,K)");
  extern __shared__ __align__(16) char smem_nt[];
  const int Mv = bound_or(valid, M);

  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, patched, tm, tn);
  if constexpr (!QKV) {
    if (qkv.tile_plus1 > 0) {
      tm = (qkv.tile_plus1 - 1) / tiles_n;
      tn = (qkv.tile_plus1 - 1) % tiles_n;
    }
  }
  const int m0 = tm * NT_BM;
  if (m0 >= Mv) return;
  const bf16_t* B = B_;
  bf16_t* C = C_;
  int N = N_, which = 0;
  if constexpr (QKV) {
    const int q_tiles = N_ / NT_BN, kv_tiles = qkv.kv_n / NT_BN;
    if (tn >= q_tiles) {
      which = tn < q_tiles + kv_tiles ? 1 : 2;
      tn -= q_tiles + (which - 1) * kv_tiles;
      B = which == 1 ? qkv.Bk : qkv.Bv;
      C = which == 1 ? qkv.Ck : qkv.Cv;
      N = qkv.kv_n;
    }
  }
  const int n0 = tn * NT_BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane >> 3, pch = lane & 7;
  auto kn_swizzle = [](int k) { return ((k & 3) << 1) | (((k >> 3) & 1) << 3); };
  int a_voff[INST], b_voff[INST];
#pragma unroll
  for (int i = 0; i < INST; ++i) {
    const int r = (wave * INST + i) * 8 + lrow;
    const int lch = pch ^ ((r >> 1) & 7);
    // Rows past the end re-read the last row; what they produce is never stored.
    a_voff[i] = (int)(((size_t)(min(m0 + r, M - 1) - m0) * K + lch * 8) * 2);
    if constexpr (!B_KN) {
      b_voff[i] = (int)(((size_t)(min(n0 + r, N - 1) - n0) * K + lch * 8) * 2);
    } else {
      // B (K,N) lands as stored: 64 k-rows of 128 columns (256 bytes a row, four rows an
      // instruction), a row's 16 chunks XORed with kn_swizzle(row) for the transposing reads below.
      const int kr = (wave * INST + i) * 4 + (lane >> 4);
      b_voff[i] = (int)(((size_t)kr * N + ((lane & 15) ^ kn_swizzle(kr)) * 8) * 2);
    }
  }
  const int k_first = QKV || B_KN ? 0 : qkv.k_begin;
  const bf16_t* a_tile = A + (size_t)m0 * K + k_first;
  const bf16_t* b_tile = B_KN ? B + n0 : B + (size_t)n0 * K + k_first;
  auto issue_one = [&](char* st, int kt, int idx) {
    const int k0 = kt * BK;
    if (idx < INST) {
      const __amdgpu_buffer_rsrc_t rows = stage_rows(a_tile + k0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rows, IRON_LDS_PTR(st + (wave * INST + idx) * 1024), 16,
                                               (int)a_voff[idx], 0, 0, 0);
    } else {
      const __amdgpu_buffer_rsrc_t rows = stage_rows(b_tile + (B_KN ? (size_t)k0 * N : (size_t)k0));
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rows, IRON_LDS_PTR(st + NT_A_BYTES + (wave * INST + idx - INST) * 1024),
                                               16, (int)b_voff[idx - INST], 0, 0, 0);
    }
  };

  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;

  // Where this lane stores: rows r0 + lane / 8 of the wave's 64 (r0 = 0, 8, ..), 8 columns from 8 (lane % 8).
  const int out_row = lane >> 3, out_col = (lane & 7) * 8;
  const int out_n = n0 + wn * 64 + out_col;
  // A residual's pieces this lane will add in the epilogue are requested now, so that their
  // latency passes under the whole product instead of at its end (N a multiple of 8: 16-byte pieces).
  uint4 res[8];
  const bool res_ahead = !QKV && qkv.residual != nullptr && (N & 7) == 0;
  if constexpr (!QKV) {
    if (res_ahead) {
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const int m = min(m0 + wm * 64 + r * 8 + out_row, M - 1);
        res[r] = *reinterpret_cast<const uint4*>(qkv.residual + (size_t)m * N + min(out_n, N - 8));
      }
    }
  }

  const int nk = (!QKV && !B_KN && qkv.k_len > 0 ? qkv.k_len : K) / BK;
#pragma unroll
  for (int s = 0; s < NT_STAGES - 1; ++s)
#pragma unroll
    for (int idx = 0; idx < LOADS; ++idx) issue_one(smem_nt + s * NT_STAGE_BYTES, min(s, nk - 1), idx);

  // Fragments: lane -> row fr of a 16-row tile, 16-byte chunk kq of the k-step's four.
  const int fr = lane & 15, kq = lane >> 4;
  const int swz = (fr >> 1) & 7;   // tile rows are multiples of 16 apart: one swizzle for all
  const int a_row = (wm * 64 + fr) * 128, b_row = NT_A_BYTES + (wn * 64 + fr) * 128;
  auto a_frag = [&](const char* st, int ks, int i) {
    return *reinterpret_cast<const bf16x8*>(st + a_row + i * 16 * 128 + (((ks * 4 + kq) ^ swz) << 4));
  };
  auto b_frag = [&](const char* st, int ks, int j) {
    return *reinterpret_cast<const bf16x8*>(st + b_row + j * 16 * 128 + (((ks * 4 + kq) ^ swz) << 4));
  };

  // (K,N): the B operand of tile j wants, for column n = 16 j + fr, the k-step's k = 8 kq .. + 7; a
  // transposing read hands a 16-lane group the 4 k-rows x 16 columns its lanes point at, turned
  // round (a lane gets 4 k of one column): rows 8 kq .. + 3, then 8 kq + 4 .. + 7.
  const int tr_k = 8 * kq + ((lane & 15) >> 2), tr_n = wn * 64 + 4 * (lane & 3);
  const unsigned lds_base_nt = (unsigned)(size_t)IRON_LDS_PTR(smem_nt);
  const unsigned kn_base = lds_base_nt + NT_A_BYTES;
  // The lane's place in a stage's B tile for tile j (k-step 0, low half) is fixed for the whole loop;
  // the k-step (32 rows on) and the high half (4 rows on) leave the swizzle as it is -- kn_swizzle(k +
  // 4) = kn_swizzle(k) for k % 8 < 4, and k + 32 keeps the bits it reads -- and the (K,N) loop is
  // unrolled over the four stage buffers, so k-step, half and stage all ride in the reads' offset
  // fields (16 bits: a second set of lane addresses two stages on) and a fragment read costs no
  // vector arithmetic at all: with one wave a SIMD every vector instruction between two MFMAs is
  // time off the matrix pipe (sixteen adds a k-step, then four, then none: 2048^3 25.0 -> 23.5 -> 22.7 us).
  unsigned kn_lane[2][4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = tr_n + j * 16;
    kn_lane[0][j] = kn_base + (((n >> 3) ^ kn_swizzle(tr_k)) << 4) + ((n & 4) << 1) + tr_k * 256;
    kn_lane[1][j] = kn_lane[0][j] + 2 * NT_STAGE_BYTES;
  }
  auto b_frag_kn = [&](auto stage_c, int ks, int j, TrFrag& t) {
    constexpr int STAGE = decltype(stage_c)::value, OFF = (STAGE & 1) * NT_STAGE_BYTES;
    const unsigned at = kn_lane[STAGE >> 1][j];
    if (ks == 0) {
      t.lo = lds_read_tr16_at<OFF>(at);
      t.hi = lds_read_tr16_at<OFF + 4 * 256>(at);
    } else {
      t.lo = lds_read_tr16_at<OFF + 32 * 256>(at);
      t.hi = lds_read_tr16_at<OFF + 36 * 256>(at);
    }
  };
  TrFrag tfb[2][4];
  // The compiler does not count the transposing reads: a k-step's B fragments pass through this
  // wait before they are joined into operands.  LDS reads return in order and the only reads
  // issued after a k-step's B fragments are its four A fragments, so "at most four outstanding"
  // is "B has arrived".
  auto join_b = [&](int ks, bf16x8 (&b)[4]) {
    asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(tfb[ks][0].lo), "+v"(tfb[ks][0].hi), "+v"(tfb[ks][1].lo), "+v"(tfb[ks][1].hi),
                                           "+v"(tfb[ks][2].lo), "+v"(tfb[ks][2].hi), "+v"(tfb[ks][3].lo), "+v"(tfb[ks][3].hi));
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j] = tr_join(tfb[ks][j]);
  };
  // (K,N): the A fragments are read by uncounted reads as well, so that every wait of the loop is
  // this code's own.  With counted A reads the compiler's waits for them took no account of the
  // transposing reads issued in between and came out as "all but two outstanding" where eleven
  // were in flight: each k-step waited an LDS trip for fragments of the NEXT one (a quarter of
  // the loop's time).  The lane's place in a stage for k-step ks; tile row i is the read's offset.
  unsigned a_lane[2][2];   // [stage / 2][k-step]
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    a_lane[0][ks] = lds_base_nt + a_row + (((ks * 4 + kq) ^ swz) << 4);
    a_lane[1][ks] = a_lane[0][ks] + 2 * NT_STAGE_BYTES;
  }
  auto a_frags_kn = [&](auto stage_c, int ks, int i, bf16x8& out) {
    constexpr int STAGE = decltype(stage_c)::value, OFF = (STAGE & 1) * NT_STAGE_BYTES;
    const unsigned at = a_lane[STAGE >> 1][ks];
    if (i == 0) out = lds_read_b128_at<OFF + 0 * 16 * 128>(at);
    else if (i == 1) out = lds_read_b128_at<OFF + 1 * 16 * 128>(at);
    else if (i == 2) out = lds_read_b128_at<OFF + 2 * 16 * 128>(at);
    else out = lds_read_b128_at<OFF + 3 * 16 * 128>(at);
  };

  wait_vmcnt<(NT_STAGES - 2) * LOADS>();   // stage 0 has landed once only the two younger ones are out
  block_barrier();
  bf16x8 af[2][4], bfr[2][4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (B_KN) b_frag_kn(std::integral_constant<int, 0>{}, 0, i, tfb[0][i]);
    else bfr[0][i] = b_frag(smem_nt, 0, i);
  }
  __builtin_amdgcn_sched_barrier(0);   // B's reads first, then A's: join_b counts on that order
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (B_KN) a_frags_kn(std::integral_constant<int, 0>{}, 0, i, af[0][i]);
    else af[0][i] = a_frag(smem_nt, 0, i);
  }
  // One stage of the loop, which is unrolled over the four stage buffers: stage_c = kt % NT_STAGES,
  // so a fragment's place in LDS is a lane address fixed before the loop plus an offset field, and
  // nothing is computed for it between two MFMAs ((N,K) at 2048^3: 20.7 -> 20.0 us; (K,N) above).
  auto stage_step = [&](int kt, auto stage_c) {
    constexpr int STAGE = decltype(stage_c)::value;
    static_assert(STAGE >= 0 && STAGE < NT_STAGES, "a stage buffer");
    // Prefetch goes into the buffer of stage kt-1.  Past the end the last stage is fetched again
    // (into buffers nobody reads any more) rather than branch: every iteration issues the same
    // loads, which keeps the wait counts exact and the scheduling region whole.
    const int kn = min(kt + NT_STAGES - 1, nk - 1);
    constexpr int STAGE_NEXT = (STAGE + 1) % NT_STAGES;
    char* nst = smem_nt + ((STAGE + NT_STAGES - 1) % NT_STAGES) * NT_STAGE_BYTES;
    const char* st = smem_nt + STAGE * NT_STAGE_BYTES;
    const char* st1 = smem_nt + STAGE_NEXT * NT_STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      if (ks == 1) {
        // The stage's one barrier, before its second k-step (whose fragments are in registers): of
        // the loads in flight the oldest LOADS are stage kt+1's (then stage kt+2's, and the 4 issued
        // so far for stage kt+3); after it nobody reads stage kt any more.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_vmcnt<LOADS + 4>();
        block_barrier();
      }
      const char* from = ks == 0 ? st : st1;
      const int nks = ks ^ 1;
      if constexpr (B_KN) join_b(ks, bfr[ks]);
      // Source order is issue order (nothing crosses a sched_barrier): after an MFMA one fragment
      // read of the next k-step (B's first: its first MFMAs need all of them) or one load goes out.
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (B_KN) {
          // Reads in flight when tile row i starts, in issue order: this k-step's A fragments from
          // i on, then what this k-step has issued for the next one (8 transposing reads during
          // row 0, 4 A reads during row 1): fragment i has arrived once all but those after it have.
          if (i == 0) lds_wait_for<3>(af[ks][0]);         // after join_b: a1 a2 a3 may be out
          else if (i == 1) lds_wait_for<10>(af[ks][1]);   // a2 a3 + 8
          else if (i == 2) lds_wait_for<13>(af[ks][2]);   // a3 + 8 + 4
          else lds_wait_for<12>(af[ks][3]);               // 8 + 4
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          mfma_16x16x32_in_place(acc[i][j], bfr[ks][j], af[ks][i]);
          __builtin_amdgcn_sched_barrier(0);
          const int slot = i * 4 + j;
          if (slot < 4) {
            if constexpr (B_KN) {
              if (ks == 0) b_frag_kn(stage_c, nks, slot, tfb[nks][slot]);
              else b_frag_kn(std::integral_constant<int, STAGE_NEXT>{}, nks, slot, tfb[nks][slot]);
            } else {
              bfr[nks][slot] = b_frag(from, nks, slot);
            }
          } else if (slot < 8) {
            if constexpr (B_KN) {
              if (ks == 0) a_frags_kn(stage_c, nks, slot - 4, af[nks][slot - 4]);
              else a_frags_kn(std::integral_constant<int, STAGE_NEXT>{}, nks, slot - 4, af[nks][slot - 4]);
            } else {
              af[nks][slot - 4] = a_frag(from, nks, slot - 4);
            }
          } else if (slot & 1) issue_one(nst, kn, ks * 4 + (slot - 9) / 2);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
  static_assert(NT_STAGES == 4, "the loop below names the four stage buffers");
  for (int kt0 = 0; kt0 < nk; kt0 += NT_STAGES) {
    stage_step(kt0, std::integral_constant<int, 0>{});
    if (kt0 + 1 < nk) stage_step(kt0 + 1, std::integral_constant<int, 1>{});
    if (kt0 + 2 < nk) stage_step(kt0 + 2, std::integral_constant<int, 2>{});
    if (kt0 + 3 < nk) stage_step(kt0 + 3, std::integral_constant<int, 3>{});
  }

  wait_vmcnt<0>();   // the idle fetches of the last iterations land ...
  block_barrier();   // ... in every wave, and every wave is done with the stages, before LDS is reused

  if constexpr (QKV) {
    if (which < 2) {
      // acc[i][j][e] and acc[i][j + 2][e] are columns c and c + 32 of the wave's head, c = 16 j + 4 kq + e,
      // of row m = 16 i + fr: the pair RoPE turns by the angle row's (cos, sin) number c.
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = min(m0 + wm * 64 + i * 16 + fr, M - 1);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float cs[8];
          unpack8(*reinterpret_cast<const uint4*>(qkv.angles + (size_t)m * 64 + 2 * (16 * j + 4 * kq)), cs);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float x1 = round_bf16(acc[i][j][e]), x2 = round_bf16(acc[i][j + 2][e]);
            const float c = cs[2 * e], sn = cs[2 * e + 1];
            acc[i][j][e] = x1 * c - x2 * sn;
            acc[i][j + 2][e] = x2 * c + x1 * sn;
          }
        }
      }
    }
  }

  if constexpr (!QKV && !B_KN) {
    if (qkv.partial != nullptr) {
      // A slice of K: the float32 sums as they are, four columns of a row a lane and tile.
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = m0 + wm * 64 + i * 16 + fr;
        if (m >= Mv) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = n0 + wn * 64 + j * 16 + 4 * kq;
          if (n + 4 <= N) *reinterpret_cast<f32x4*>(qkv.partial + (size_t)m * N + n) = acc[i][j];
        }
      }
      return;
    }
  }
  // Output through LDS: the wave lays its 64 x 64 out row-major (rows padded by 16 bytes, which
  // spreads the 8-byte writes and the 16-byte reads over the banks) and each lane then owns 8
  // consecutive columns of a row: a row of the tile leaves as one 128-byte segment.
  constexpr int OROWB = 64 * 2 + 16;
  char* ot = smem_nt + wave * (64 * OROWB);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *reinterpret_cast<uint2*>(ot + (i * 16 + fr) * OROWB + (j * 16 + 4 * kq) * 2) =
          make_uint2(pack_bf16(acc[i][j][0], acc[i][j][1]), pack_bf16(acc[i][j][2], acc[i][j][3]));
  // The tile is private to the wave, whose LDS operations execute in order: no block barrier,
  // only a fence to keep the compiler from moving the reads above other lanes' writes.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const bool whole = (N & 7) == 0 && out_n + 8 <= N;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int row = r * 8 + out_row, m = m0 + wm * 64 + row;
    uint4 v = *reinterpret_cast<const uint4*>(ot + row * OROWB + out_col * 2);
    if (m >= Mv || out_n >= N) continue;
    bf16_t* p = C + (size_t)m * N + out_n;
    if constexpr (!QKV) {
      if (qkv.residual != nullptr) {   // the product rounded as it would be stored, then scale * it + residual
        float x[8], rf[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        unpack8(v, x);
        if (whole) {
          unpack8(res_ahead ? res[r] : *reinterpret_cast<const uint4*>(qkv.residual + (size_t)m * N + out_n), rf);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)   // (constant indices: a runtime trip count puts the array in scratch memory)
            if (out_n + e < N) rf[e] = bf16_to_f32(qkv.residual[(size_t)m * N + out_n + e]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e)
          x[e] = qkv.gated ? round_bf16(gate_of(qkv.gated, rf[e])) * x[e] : fmaf(qkv.residual_scale, x[e], rf[e]);
        v = pack8(x);
      }
    }
    if (whole) {
      *reinterpret_cast<uint4*>(p) = v;
    } else {
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (out_n + e < N) p[e] = (bf16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu));
    }
  }
}


template <bool B_KN, bool QKV, int T, int STAGES64 = 4>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const bf16_t* __restrict__ A,
                                                      const bf16_t* __restrict__ B,
                                                      bf16_t* __restrict__ C, int M, int N, int K,
                                                      const int* __restrict__ valid, int tiles_m,
                                                      int tiles_n, int patched, QkvTail qkv) {
  if constexpr (QKV) to_cache_rows(qkv, valid, M);
  static_assert(T == 2 || (T == 1 && !B_KN && !QKV), "64x64 tiles: B (N,K), plain or residual output");
  if constexpr (T == 2)
    gemm_nt16_body<QKV, B_KN>(A, B, C, M, N, K, valid, tiles_m, tiles_n, patched, qkv);
  else
    gemm_nt64_body<STAGES64>(A, B, C, M, N, K, valid, tiles_m, tiles_n, patched, qkv);
}

template <bool B_KN, bool QKV = false, int T = 2, int STAGES64 = 4>
static int launch_gemm_nt(const bf16_t* A, const bf16_t* B, bf16_t* C, int M, int N, int K,
                          const int* valid, hipStream_t s, QkvTail qkv = QkvTail{}) {
  constexpr int BM = 64 * T, BN = 64 * T;
  const int tiles_m = (M + BM - 1) / BM;
  const int tiles_n = QKV ? (N + 2 * qkv.kv_n) / BN : (N + BN - 1) / BN;
  if constexpr (T == 1 && STAGES64 == 4) {
    // No more 64 x 64 tiles than CUs: a CU has one block whatever its LDS, so the deeper pipeline.
    if ((long)tiles_m * tiles_n <= 256)
      return launch_gemm_nt<B_KN, QKV, 1, 8>(A, B, C, M, N, K, valid, s, qkv);
  }
  const size_t lds = (size_t)(T == 1 ? STAGES64 : NT_STAGES) * (BM + BN) * BK * 2;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&gemm_nt_kernel<B_KN, QKV, T, STAGES64>), lds); e != hipSuccess) {
    set_error("gemm: %s", hipGetErrorString(e));
    return (int)e;
  }
  const int patched = (tiles_m % 8 == 0 && tiles_n % 4 == 0 && ((tiles_m / 8) * (tiles_n / 4)) % 8 == 0) ? 1 : 0;
  hipLaunchKernelGGL((gemm_nt_kernel<B_KN, QKV, T, STAGES64>), dim3(tiles_m * tiles_n), dim3(256), lds, s, A, B, C, M, N, K,
                     valid, tiles_m, tiles_n, patched, qkv);
  IRON_LAUNCH_CHECK();
}

// The fused projections at 128 x 192 tiles: three 64-wide heads of the concatenated q | k | v head
// list a tile, so a 2048-row chunk of a 32 + 8 + 8-head layer is 16 x 16 = 256 tiles -- one a CU in
// one round, where 128 x 128 tiles make 384 (a round and a half, run as two).  Four waves stacked
// along m: a wave owns 32 rows x 192 columns (6 accumulator tiles), so every head's two halves sit
// in one wave and RoPE stays in registers.  Three stages of 40 KB; the loop is the 128 x 128
// kernel's (direct-to-LDS loads, pinned interleave, the stage's barrier before its last k-step).
// HPT = heads a tile: 3 as above, or 1 -- 128 x 64 tiles, for a row bound so short that wider
// tiles leave most CUs idle (512 rows of that layer: 192 tiles of one head against 64 of three).
constexpr int Q3_BM = 128, Q3_BN = 192, Q3_STAGES = 3;
constexpr int Q3_A_BYTES = Q3_BM * BK * 2, Q3_STAGE_BYTES = (Q3_BM + Q3_BN) * BK * 2;
constexpr int Q1_STAGE_BYTES = (Q3_BM + 64) * BK * 2, Q1_STAGES = 5;   // one head a tile: five 24 KB stages

template <int HPT>
__device__ __forceinline__ void qkv_heads_body(const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bq,
                                               bf16_t* __restrict__ Cq, int M, int heads, int kv_heads, int K,
                                               const int* __restrict__ valid, int tiles_m, int tiles_n,
                                               int patched, const QkvTail& qkv) {
  constexpr int Q3_BN = 64 * HPT, Q3_STAGE_BYTES = (Q3_BM + Q3_BN) * BK * 2, NACC = 2 * HPT;
  constexpr int A_INST = Q3_BM / 8 / 4, B_INST = Q3_BN / 8 / 4, LOADS = A_INST + B_INST;   // 4 + 6 (or 2) a wave
  constexpr int PER = LOADS / 3, REST = LOADS - 3 * PER;   // loads issued under each of a stage's first three k-steps, and its last
  static_assert(PER <= NACC && REST <= NACC, "a load rides an MFMA");
  extern __shared__ __align__(16) char smem_q3[];
  const int Mv = bound_or(valid, M);

  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, patched, tm, tn);
  const int m0 = tm * Q3_BM;
  if (m0 >= Mv) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane >> 3, pch = lane & 7;
  // Head g of the concatenated list: its weight rows and where its 64 columns go.
  auto head_weight = [&](int g) {
    if (g < heads) return Bq + (size_t)g * 64 * K;
    if (g < heads + kv_heads) return qkv.Bk + (size_t)(g - heads) * 64 * K;
    return qkv.Bv + (size_t)(g - heads - kv_heads) * 64 * K;
  };
  // Buffer loads straight into LDS (see gemm_nt16_body): the activations' tile rows are one buffer;
  // the eight weight rows of an instruction lie in one head, so each of a wave's weight
  // instructions has its own buffer, which starts at its first row.  The stage's k is the scalar
  // offset, a lane's place the constant vector offset.
  const __amdgpu_buffer_rsrc_t a_rows = stage_rows(A + (size_t)m0 * K);
  __amdgpu_buffer_rsrc_t b_rows[B_INST];
  int a_voff[A_INST], b_voff[B_INST];
#pragma unroll
  for (int i = 0; i < A_INST; ++i) {
    const int r = (wave * A_INST + i) * 8 + lrow;
    a_voff[i] = (int)(((size_t)(min(m0 + r, M - 1) - m0) * K + (pch ^ ((r >> 1) & 7)) * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < B_INST; ++i) {
    const int r0 = (wave * B_INST + i) * 8;   // first of the instruction's rows among the tile's weight rows: head r0 / 64, its row r0 % 64
    const int r = r0 + lrow;
    b_rows[i] = stage_rows(head_weight(tn * HPT + r0 / 64) + (size_t)(r0 % 64) * K);
    b_voff[i] = (int)(((size_t)lrow * K + (pch ^ ((r >> 1) & 7)) * 8) * 2);
  }
  auto issue_one = [&](char* st, int kt, int idx) {
    const int k_off = kt * BK * 2;
    if (idx < A_INST)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rows, IRON_LDS_PTR(st + (wave * A_INST + idx) * 1024), 16,
                                               (int)a_voff[idx], k_off, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rows[idx - A_INST],
                                               IRON_LDS_PTR(st + Q3_A_BYTES + (wave * B_INST + idx - A_INST) * 1024), 16,
                                               (int)b_voff[idx - A_INST], k_off, 0, 0);
  };

  f32x16 acc[NACC];
#pragma unroll
  for (int j = 0; j < NACC; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;

  const int nk = K / BK;
  const int fr = lane & 31, kh = lane >> 5;
  const int swz = (fr >> 1) & 7;   // tile rows are multiples of 32 apart: one swizzle for all
  const int a_off = (wave * 32 + fr) * 128, b_off = Q3_A_BYTES + fr * 128;
  auto frag = [&](const char* st, int off, int ks) {
    return *reinterpret_cast<const bf16x8*>(st + off + (((ks * 2 + kh) ^ swz) << 4));
  };
  if constexpr (HPT == 1) {
    // One head a tile: a k-step is two MFMAs of a wave, far less than an LDS read takes to return,
    // so -- as in gemm_nt64_body -- the fragments of a whole stage are read one stage ahead into a
    // second register set.  At the top of stage kt the one barrier (stage kt+1 has landed in every
    // wave, nobody reads stage kt-1 any more), then stage kt's eight MFMAs out of registers with
    // the twelve fragment reads of stage kt+1 and the six loads of stage kt+STAGES-1 between them.
    constexpr int STAGES = Q1_STAGES, KSTEPS = BK / 16;
    static_assert(LOADS == 6 && KSTEPS == 4, "six loads and twelve reads ride eight MFMAs");
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
#pragma unroll
      for (int idx = 0; idx < LOADS; ++idx) issue_one(smem_q3 + s * Q3_STAGE_BYTES, min(s, nk - 1), idx);
    wait_vmcnt<(STAGES - 2) * LOADS>();   // stage 0 has landed once only the younger ones are out
    block_barrier();
    bf16x8 af[2][KSTEPS], bfr[2][KSTEPS][2];   // [stage parity][k-step]([column half])
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      af[0][ks] = frag(smem_q3, a_off, ks);
      bfr[0][ks][0] = frag(smem_q3, b_off, ks);
      bfr[0][ks][1] = frag(smem_q3, b_off + 32 * 128, ks);
    }
    auto stage = [&](int kt, auto parity) {
      constexpr int P = decltype(parity)::value;
      // Of this wave's loads in flight the oldest LOADS are stage kt+1's; the STAGES-3 stages after it may stay out.
      wait_vmcnt<(STAGES - 3) * LOADS>();
      block_barrier();
      const char* st1 = smem_q3 + ((kt + 1) % STAGES) * Q3_STAGE_BYTES;     // past the end: a stage nobody needs
      char* nst = smem_q3 + ((kt + STAGES - 1) % STAGES) * Q3_STAGE_BYTES;  // stage kt-1's buffer
      const int kn = min(kt + STAGES - 1, nk - 1);   // past the end the last stage again: the wait counts stay exact
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[P][ks][0], af[P][ks], acc[0], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        af[P ^ 1][ks] = frag(st1, a_off, ks);
        bfr[P ^ 1][ks][0] = frag(st1, b_off, ks);
        if (ks < 2) issue_one(nst, kn, ks);
        __builtin_amdgcn_sched_barrier(0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[P][ks][1], af[P][ks], acc[1], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        bfr[P ^ 1][ks][1] = frag(st1, b_off + 32 * 128, ks);
        issue_one(nst, kn, 2 + ks);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    int kt = 0;
    for (; kt + 1 < nk; kt += 2) {
      stage(kt, std::integral_constant<int, 0>{});
      stage(kt + 1, std::integral_constant<int, 1>{});
    }
    if (kt < nk) stage(kt, std::integral_constant<int, 0>{});
  } else {
#pragma unroll
  for (int s = 0; s < Q3_STAGES - 1; ++s)
#pragma unroll
    for (int idx = 0; idx < LOADS; ++idx) issue_one(smem_q3 + s * Q3_STAGE_BYTES, min(s, nk - 1), idx);

  wait_vmcnt<LOADS>();   // stage 0 has landed once only stage 1's loads are out
  block_barrier();
  bf16x8 af[2], bfr[2][NACC];
  af[0] = frag(smem_q3, a_off, 0);
#pragma unroll
  for (int j = 0; j < NACC; ++j) bfr[0][j] = frag(smem_q3, b_off + j * 32 * 128, 0);
  // One stage of the loop, which is unrolled over the three stage buffers (stage_c = kt % Q3_STAGES):
  // a fragment's stage then rides in its read's offset field instead of a vector add a read.
  auto stage_step = [&](int kt, auto stage_c) {
    constexpr int S = decltype(stage_c)::value;
    const int kn = min(kt + Q3_STAGES - 1, nk - 1);
    char* nst = smem_q3 + ((S + Q3_STAGES - 1) % Q3_STAGES) * Q3_STAGE_BYTES;
    const char* st = smem_q3 + S * Q3_STAGE_BYTES;
    const char* st1 = smem_q3 + ((S + 1) % Q3_STAGES) * Q3_STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      const bool last = ks == BK / 16 - 1;
      if (last) {
        // Of the loads in flight the oldest LOADS are stage kt+1's; the 3 PER issued so far for stage
        // kt+2 may stay out.  After the barrier nobody reads stage kt any more.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_vmcnt<3 * PER>();
        block_barrier();
      }
      const char* from = last ? st1 : st;
      const int nks = last ? 0 : ks + 1;
#pragma unroll
      for (int j = 0; j < NACC; ++j) {
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[cur][j], af[cur], acc[j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (j == 0) af[nxt] = frag(from, a_off, nks);
        bfr[nxt][j] = frag(from, b_off + j * 32 * 128, nks);
        // A stage's loads (ten, or six): PER under each of the first three k-steps, the rest under the last.
        if (!last && j < PER) issue_one(nst, kn, ks * PER + j);
        if (last && j < REST) issue_one(nst, kn, 3 * PER + j);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  static_assert(Q3_STAGES == 3, "the loop below names the three stage buffers");
  for (int kt0 = 0; kt0 < nk; kt0 += Q3_STAGES) {
    stage_step(kt0, std::integral_constant<int, 0>{});
    if (kt0 + 1 < nk) stage_step(kt0 + 1, std::integral_constant<int, 1>{});
    if (kt0 + 2 < nk) stage_step(kt0 + 2, std::integral_constant<int, 2>{});
  }
  }
  wait_vmcnt<0>();   // the idle fetches of the last iterations land before the block's LDS is released

  // acc[2h][e] and acc[2h+1][e] are columns c and c + 32 of head h of the tile, c = 8 (e/4) + 4 kh + e%4,
  // of row fr of the wave's 32: the pair RoPE turns by the angle row's (cos, sin) number c.
  const int m = m0 + wave * 32 + fr;
  const bf16_t* ang = qkv.angles + (size_t)min(m, M - 1) * 64 + 8 * kh;
#pragma unroll
  for (int h = 0; h < HPT; ++h) {
    const int g = tn * HPT + h;
    bf16_t* C;
    int N, col;
    if (g < heads) { C = Cq; N = heads * 64; col = g * 64; }
    else if (g < heads + kv_heads) { C = qkv.Ck; N = kv_heads * 64; col = (g - heads) * 64; }
    else { C = qkv.Cv; N = kv_heads * 64; col = (g - heads - kv_heads) * 64; }
    if (g < heads + kv_heads) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float cs[8];
        unpack8(*reinterpret_cast<const uint4*>(ang + 16 * q), cs);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x1 = round_bf16(acc[2 * h][4 * q + e]), x2 = round_bf16(acc[2 * h + 1][4 * q + e]);
          const float c = cs[2 * e], sn = cs[2 * e + 1];
          acc[2 * h][4 * q + e] = x1 * c - x2 * sn;
          acc[2 * h + 1][4 * q + e] = x2 * c + x1 * sn;
        }
      }
    }
    if (m < Mv) {
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          bf16_t* p = C + (size_t)m * N + col + 32 * half + 8 * q + 4 * kh;
          const f32x16& a = acc[2 * h + half];
          *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16(a[4 * q], a[4 * q + 1]), pack_bf16(a[4 * q + 2], a[4 * q + 3]));
        }
    }
  }
}

__global__ __launch_bounds__(256) void qkv192_kernel(const bf16_t* __restrict__ A,
                                                     const bf16_t* __restrict__ Bq, bf16_t* __restrict__ Cq,
                                                     int M, int heads, int kv_heads, int K,
                                                     const int* __restrict__ valid, int tiles_m, int tiles_n,
                                                     int patched, QkvTail qkv) {
  to_cache_rows(qkv, valid, M);
  qkv_heads_body<3>(A, Bq, Cq, M, heads, kv_heads, K, valid, tiles_m, tiles_n, patched, qkv);
}

__global__ __launch_bounds__(256) void qkv64_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bq,
                                                    bf16_t* __restrict__ Cq, int M, int heads, int kv_heads, int K,
                                                    const int* __restrict__ valid, int tiles_m, int tiles_n,
                                                    int patched, QkvTail qkv) {
  to_cache_rows(qkv, valid, M);
  qkv_heads_body<1>(A, Bq, Cq, M, heads, kv_heads, K, valid, tiles_m, tiles_n, patched, qkv);
}

// Both tilings in one launch: the row bound is read on the device, and which tiling makes fewer
// rounds over the chip depends on it, so the blocks choose -- the 192-wide tiles when the bound is
// past `above` (if wide_top, else when it is not), the 128-wide ones otherwise.  The grid is the
// larger of the two; a block past its tiling's tiles leaves at once.
struct Tiling {
  int tiles_m, tiles_n, patched;
};
__global__ __launch_bounds__(256) void qkv_either_kernel(const bf16_t* __restrict__ A,
                                                         const bf16_t* __restrict__ Bq, bf16_t* __restrict__ Cq,
                                                         int M, int heads, int kv_heads, int K,
                                                         const int* __restrict__ valid, Tiling narrow, Tiling wide,
                                                         Tiling thin, int above, int wide_top, int thin_upto,
                                                         QkvTail qkv) {
  const int Mv = bound_or(valid, M);
  const bool past = Mv > above;
  to_cache_rows(qkv, valid, M);
  if (Mv <= thin_upto) {   // so few rows that one-head tiles still fit one round over the chip
    if ((int)blockIdx.x < thin.tiles_m * thin.tiles_n)
      qkv_heads_body<1>(A, Bq, Cq, M, heads, kv_heads, K, valid, thin.tiles_m, thin.tiles_n, thin.patched, qkv);
  } else if (wide.tiles_n > 0 && past == (wide_top != 0)) {
    if ((int)blockIdx.x < wide.tiles_m * wide.tiles_n)
      qkv_heads_body<3>(A, Bq, Cq, M, heads, kv_heads, K, valid, wide.tiles_m, wide.tiles_n, wide.patched, qkv);
  } else {
    if ((int)blockIdx.x < narrow.tiles_m * narrow.tiles_n)
      gemm_nt16_body<true>(A, Bq, Cq, M, heads * 64, K, valid, narrow.tiles_m, narrow.tiles_n, narrow.patched, qkv);
  }
}

static int patched_order(int tiles_m, int tiles_n) {
  return (tiles_m % 8 == 0 && tiles_n % 4 == 0 && ((tiles_m / 8) * (tiles_n / 4)) % 8 == 0) ? 1 : 0;
}

// wide_ok: the head count comes in threes (else the 192-wide tiling is never chosen).  thin_upto: the
// row bound up to which the one-head tiles run (0: never).
static int launch_qkv_either(const bf16_t* A, const bf16_t* Bq, bf16_t* Cq, int M, int heads, int kv_heads, int K,
                             const int* valid, hipStream_t s, QkvTail qkv, int above, bool wide_top, bool wide_ok,
                             int thin_upto) {
  const int tiles_m = (M + 127) / 128, total = heads + 2 * kv_heads;
  const Tiling narrow{tiles_m, total / 2, patched_order(tiles_m, total / 2)};
  const Tiling wide{wide_ok ? tiles_m : 0, wide_ok ? total / 3 : 0, wide_ok ? patched_order(tiles_m, total / 3) : 0};
  const int thin_m = (thin_upto + 127) / 128;
  const Tiling thin{thin_m, total, patched_order(thin_m, total)};
  const size_t lds_narrow = (size_t)NT_STAGES * 256 * BK * 2, lds_wide = (size_t)Q3_STAGES * Q3_STAGE_BYTES;
  const size_t lds = lds_narrow > lds_wide ? lds_narrow : lds_wide;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&qkv_either_kernel), lds); e != hipSuccess) {
    set_error("prefill_qkv: %s", hipGetErrorString(e));
    return (int)e;
  }
  int blocks = tiles_m * (narrow.tiles_n > wide.tiles_n ? narrow.tiles_n : wide.tiles_n);
  if (thin.tiles_m * thin.tiles_n > blocks) blocks = thin.tiles_m * thin.tiles_n;
  hipLaunchKernelGGL(qkv_either_kernel, dim3(blocks), dim3(256), lds, s, A, Bq, Cq, M, heads, kv_heads, K, valid, narrow,
                     wide, thin, above, wide_top ? 1 : 0, thin_upto, qkv);
  IRON_LAUNCH_CHECK();
}

static int launch_qkv64(const bf16_t* A, const bf16_t* Bq, bf16_t* Cq, int M, int heads, int kv_heads, int K,
                        const int* valid, hipStream_t s, QkvTail qkv) {
  const int tiles_m = (M + Q3_BM - 1) / Q3_BM, tiles_n = heads + 2 * kv_heads;
  const size_t lds = (size_t)Q1_STAGES * Q1_STAGE_BYTES;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&qkv64_kernel), lds); e != hipSuccess) {
    set_error("prefill_qkv: %s", hipGetErrorString(e));
    return (int)e;
  }
  hipLaunchKernelGGL(qkv64_kernel, dim3(tiles_m * tiles_n), dim3(256), lds, s, A, Bq, Cq, M, heads, kv_heads, K, valid,
                     tiles_m, tiles_n, patched_order(tiles_m, tiles_n), qkv);
  IRON_LAUNCH_CHECK();
}

static int launch_qkv192(const bf16_t* A, const bf16_t* Bq, bf16_t* Cq, int M, int heads, int kv_heads, int K,
                         const int* valid, hipStream_t s, QkvTail qkv) {
  const int tiles_m = (M + Q3_BM - 1) / Q3_BM, tiles_n = (heads + 2 * kv_heads) / 3;
  const size_t lds = (size_t)Q3_STAGES * Q3_STAGE_BYTES;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&qkv192_kernel), lds); e != hipSuccess) {
    set_error("prefill_qkv: %s", hipGetErrorString(e));
    return (int)e;
  }
  hipLaunchKernelGGL(qkv192_kernel, dim3(tiles_m * tiles_n), dim3(256), lds, s, A, Bq, Cq, M, heads, kv_heads, K, valid,
                     tiles_m, tiles_n, patched_order(tiles_m, tiles_n), qkv);
  IRON_LAUNCH_CHECK();
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
    static LdsOptIn opt_in;                                                               \
    if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), lds); e != hipSuccess) { \
      set_error("gemm: %s", hipGetErrorString(e));                                        \
      return (int)e;                                                                      \
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


// Large problems, B (N,K): 256x256x64 tiles, two 64 KB stages fed straight into LDS.  Against the
// 128x128 kernel a CU pulls half as many global bytes per flop -- the 64 B/clk a CU can move from L2
// into LDS is what bounds the smaller tile.  Eight waves, two a SIMD, each owning 128 x 64 of the
// tile (32 accumulator tiles of 16 x 16, 128 accumulation registers): one's loads and fragment reads
// issue under the other's MFMAs (2048 x 8192 x 2048 60.5 -> 56.5 us, 4096^3 111 -> 107.5 against four
// waves of 128 x 128; 8192^3 the same).  Within a wave the instruction stream still interleaves the
// next k-step's fragment reads and the next stages' loads with the MFMAs.  Where the blocks of one
// launch choose their tile size by a row bound (gemm_either_kernel) the large tile is four waves of
// 128 x 128, as every other tiling of that launch is four waves.
constexpr int BIG_BM = 256, BIG_BN = 256;
#ifndef IRON_BIG_WAVES
#define IRON_BIG_WAVES 8   // the stand-alone launch: two waves a SIMD, each 128 x 64 of the tile (4: one, 128 x 128)
#endif
constexpr int BIG_WAVES = IRON_BIG_WAVES;
#ifndef IRON_BIG_KB
#define IRON_BIG_KB 64
#endif
constexpr int BIG_KB = IRON_BIG_KB;   // k per stage: 64 (2 stages); 32 (4 stages of half-line rows) measured 13 % slower
#define BIG_OUT_ROW_BYTES(TN) ((TN) * 64 + 16)
constexpr int BIG_STAGE_BYTES = (BIG_BM + BIG_BN) * BK * 2;

template <int WAVES, int KB, bool B_KN = false, bool STREAM_OUT = false>
__device__ __forceinline__ void gemm_nt256_body(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B,
                                                bf16_t* __restrict__ C, int M, int N, int K,
                                                const int* __restrict__ valid, int tiles_m, int tiles_n,
                                                int patched) {
  static_assert(KB == 64, "k per stage: 64 (32 with four stages of half-line rows measured 13 % slower)");
  constexpr int ROWB = KB * 2;               // bytes of a tile row in LDS
  constexpr int CPR = KB / 8;                // its 16-byte chunks
  constexpr int RPI = 1024 / ROWB;           // rows one 1 KB load covers
  constexpr int A_BYTES = BIG_BM * ROWB, STAGE_BYTES = (BIG_BM + BIG_BN) * ROWB;
  constexpr int STAGES = KB == 64 ? 2 : 4;   // 128 KB either way
  constexpr int INST = BIG_BM / RPI / WAVES; // 1 KB loads of A (and of B) a wave issues per stage
  constexpr int TN = 8 / WAVES * 2;          // 32-column MFMA tiles a wave owns along n (4 or 2)
  extern __shared__ __align__(16) char smem_big[];
  const int Mv = bound_or(valid, M);

  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, patched, tm, tn);
  const int m0 = tm * BIG_BM, n0 = tn * BIG_BN;
  if (m0 >= Mv) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: LDS and global bases stay in scalar registers
  const int wm = wave / (WAVES / 2), wn = wave % (WAVES / 2);
  // Loader: instruction i of a wave moves rows (wave*INST + i)*RPI .. ; lane -> (row, physical
  // chunk); the logical chunk it fetches is the physical one swizzled by the row.
  const int lrow = lane / CPR, pch = lane % CPR;
  unsigned ld_off[2];   // byte offset of this lane's 16 bytes within an even / odd instruction's rows
#pragma unroll
  for (int par = 0; par < 2; ++par) {
    const int r = par * RPI + lrow;
    ld_off[par] = (unsigned)(((size_t)lrow * K + (pch ^ ((r >> 1) & (CPR - 1))) * 8) * 2);
  }
  // Loads go out as buffer loads straight into LDS: the rows a wave fetches are one buffer, the
  // lane's place within an instruction's rows is the (constant) vector offset and the instruction's
  // rows and the stage's k are the scalar offset, so a load costs two scalar adds and no vector ALU
  // work between two MFMAs.
  const __amdgpu_buffer_rsrc_t a_rows = stage_rows(A + (size_t)(m0 + wave * INST * RPI) * K);
  // B as (K,N) lands as stored: the stage's 64 k-rows of 256 columns (512 bytes a row, two rows an
  // instruction), a row's 32 chunks XORed with kn_swizzle(row) so that the transposing reads below
  // find the four rows of a 16-lane group, and the groups of a pass, in different banks.
  const __amdgpu_buffer_rsrc_t b_rows =
      stage_rows(B_KN ? B + n0 + (size_t)(wave * INST * 2) * N : B + (size_t)(n0 + wave * INST * RPI) * K);
  auto kn_swizzle = [](int k) { return ((k & 3) << 1) | (((k >> 3) & 3) << 3); };
  int kn_off[INST];   // (K,N): this lane's 16 bytes within instruction idx's two rows
#pragma unroll
  for (int idx = 0; idx < INST; ++idx) {
    const int kr = (wave * INST + idx) * 2 + (lane >> 5);   // the lane's k-row of the stage
    kn_off[idx] = (int)(((size_t)(lane >> 5) * N + ((lane & 31) ^ kn_swizzle(kr)) * 8) * 2);
  }
  const int inst_stride = RPI * K * 2;
  auto issue_one = [&](char* st, int kt, int idx) {
    const int k_off = kt * KB * 2;
    if (idx < INST)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rows, IRON_LDS_PTR(st + (wave * INST + idx) * 1024), 16,
                                               (int)ld_off[idx & 1], idx * inst_stride + k_off, 0, 0);
    else if constexpr (!B_KN)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rows, IRON_LDS_PTR(st + A_BYTES + (wave * INST + idx - INST) * 1024),
                                               16, (int)ld_off[idx & 1], (idx - INST) * inst_stride + k_off, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rows, IRON_LDS_PTR(st + A_BYTES + (wave * INST + idx - INST) * 1024),
                                               16, (int)kn_off[idx - INST], ((idx - INST) * 2 + kt * KB) * N * 2, 0, 0);
  };

  // The product runs on 16x16x32 MFMAs (a k-step is 32 wide, two a stage): on random operands the
  // part sustains about a sixth more of them than of the 32x32x16 form, at the same registers and
  // the same LDS reads per flop.  A wave's 128 x 128 is 8 x NT tiles of 16 x 16.
  constexpr int NT = TN * 2;                 // 16-column tiles a wave owns along n
  f32x4 acc[8][NT];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;

  const int nk = K / KB;
  static_assert(KB == 64 && (WAVES == 4 || WAVES == 8), "the loop below is written for two 64-wide stages and four or eight waves");
  // A stage's 2 INST loads go out in two halves of INST: the first under the last quarter of the
  // stage two before it (right after that stage's barrier freed the buffer), the second under the
  // first quarter of the stage before it; two quarters later, at that stage's barrier, all have landed.
  auto issue_half = [&](char* st, int kt, int half, int slot) { issue_one(st, kt, half * INST + slot); };
#pragma unroll
  for (int idx = 0; idx < 2 * INST; ++idx) issue_one(smem_big, 0, idx);
#pragma unroll
  for (int slot = 0; slot < INST; ++slot) issue_half(smem_big + STAGE_BYTES, min(1, nk - 1), 0, slot);

  // Fragments: lane -> row fr of a 16-row tile, 16-byte chunk kq of the k-step's four.
  const int fr = lane & 15, kq = lane >> 4;
  const int swz = (fr >> 1) & (CPR - 1);   // tile rows are multiples of 16 apart: one swizzle for all
  const int a_row = (wm * 128 + fr) * ROWB, b_row = A_BYTES + (wn * NT * 16 + fr) * ROWB;
  auto a_frag = [&](const char* st, int ks, int i) {
    return *reinterpret_cast<const bf16x8*>(st + a_row + i * 16 * ROWB + (((ks * 4 + kq) ^ swz) << 4));
  };
  auto b_frag = [&](const char* st, int ks, int j) {
    return *reinterpret_cast<const bf16x8*>(st + b_row + j * 16 * ROWB + (((ks * 4 + kq) ^ swz) << 4));
  };
  // (K,N): the B operand of tile j wants, for column n = 16 j + fr, the k-step's k = 8 kq .. + 7.  A
  // transposing read hands a 16-lane group the 4 x 16 block its lanes point at (4 k-rows, each
  // lane 4 columns) turned round: the lane gets 4 k of one column.  Rows 8 kq .. + 3 and 8 kq + 4 .. + 7.
  const int tr_k = 8 * kq + ((lane & 15) >> 2), tr_n = wn * NT * 16 + 4 * (lane & 3);
  const unsigned lds_base_big = (unsigned)(size_t)IRON_LDS_PTR(smem_big);
  const unsigned kn_base = lds_base_big + A_BYTES;
  // The lane's place in a stage's B tile for tile j (k-step 0, low half) is fixed before the loop; the
  // k-step (32 rows on) and the high half (4 rows on) leave the swizzle as it is and ride in the
  // reads' offset fields, so a k-step's reads cost one vector add a tile (the stage) and no more.
  // (Unrolled over its two stage buffers so that the stage too is an offset field, as the 128 x 128
  // loop is, this kernel spilled a hundred registers: two waves a SIMD leave it 256.)
  unsigned kn_lane[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = tr_n + j * 16;
    kn_lane[j] = kn_base + (((n >> 3) ^ kn_swizzle(tr_k)) << 4) + ((n & 4) << 1) + tr_k * 512;
  }
  auto b_frag_kn = [&](int stage_bytes, int ks, int j, TrFrag& t) {
    const unsigned at = kn_lane[j] + stage_bytes;
    if (ks == 0) {
      t.lo = lds_read_tr16_at<0>(at);
      t.hi = lds_read_tr16_at<4 * 512>(at);
    } else {
      t.lo = lds_read_tr16_at<32 * 512>(at);
      t.hi = lds_read_tr16_at<36 * 512>(at);
    }
  };
  // (K,N): the A fragments are read by uncounted reads as well, so that every wait of the loop is
  // this code's own (the compiler's waits for counted A reads take no account of the transposing
  // reads issued in between and come out far too strict).  A k-step's fragments, A's and B's, are
  // all issued before join_b's wait at its start, which they pass through.
  const unsigned a_lane[2] = {lds_base_big + a_row + (((0 * 4 + kq) ^ swz) << 4), lds_base_big + a_row + (((1 * 4 + kq) ^ swz) << 4)};
  auto a_frag_kn = [&](int stage_bytes, int ks, int i, bf16x8& out) {
    const unsigned at = a_lane[ks] + stage_bytes;
    if (i == 0) out = lds_read_b128_at<0 * 16 * ROWB>(at);
    else if (i == 1) out = lds_read_b128_at<1 * 16 * ROWB>(at);
    else if (i == 2) out = lds_read_b128_at<2 * 16 * ROWB>(at);
    else if (i == 3) out = lds_read_b128_at<3 * 16 * ROWB>(at);
    else if (i == 4) out = lds_read_b128_at<4 * 16 * ROWB>(at);
    else if (i == 5) out = lds_read_b128_at<5 * 16 * ROWB>(at);
    else if (i == 6) out = lds_read_b128_at<6 * 16 * ROWB>(at);
    else out = lds_read_b128_at<7 * 16 * ROWB>(at);
  };
  TrFrag tfb[2][NT];
  // The compiler does not count these reads: a k-step's fragments pass through this wait (every LDS
  // read issued so far) before they are used.
  auto join_b = [&](int ks, bf16x8 (&b)[NT], bf16x8 (&a)[8]) {
    i32x4 a0 = __builtin_bit_cast(i32x4, a[0]), a1 = __builtin_bit_cast(i32x4, a[1]), a2 = __builtin_bit_cast(i32x4, a[2]),
          a3 = __builtin_bit_cast(i32x4, a[3]), a4 = __builtin_bit_cast(i32x4, a[4]), a5 = __builtin_bit_cast(i32x4, a[5]),
          a6 = __builtin_bit_cast(i32x4, a[6]), a7 = __builtin_bit_cast(i32x4, a[7]);
    if constexpr (NT == 4)
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(tfb[ks][0].lo), "+v"(tfb[ks][0].hi), "+v"(tfb[ks][1].lo), "+v"(tfb[ks][1].hi),
                                             "+v"(tfb[ks][2].lo), "+v"(tfb[ks][2].hi), "+v"(tfb[ks][3].lo), "+v"(tfb[ks][3].hi),
                                             "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7));
    else
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(tfb[ks][0].lo), "+v"(tfb[ks][0].hi), "+v"(tfb[ks][1].lo), "+v"(tfb[ks][1].hi),
                                             "+v"(tfb[ks][2].lo), "+v"(tfb[ks][2].hi), "+v"(tfb[ks][3].lo), "+v"(tfb[ks][3].hi),
                                             "+v"(tfb[ks][4].lo), "+v"(tfb[ks][4].hi), "+v"(tfb[ks][5].lo), "+v"(tfb[ks][5].hi),
                                             "+v"(tfb[ks][6].lo), "+v"(tfb[ks][6].hi), "+v"(tfb[ks][7].lo), "+v"(tfb[ks][7].hi),
                                             "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7));
    a[0] = __builtin_bit_cast(bf16x8, a0); a[1] = __builtin_bit_cast(bf16x8, a1); a[2] = __builtin_bit_cast(bf16x8, a2);
    a[3] = __builtin_bit_cast(bf16x8, a3); a[4] = __builtin_bit_cast(bf16x8, a4); a[5] = __builtin_bit_cast(bf16x8, a5);
    a[6] = __builtin_bit_cast(bf16x8, a6); a[7] = __builtin_bit_cast(bf16x8, a7);
#pragma unroll
    for (int j = 0; j < NT; ++j) b[j] = tr_join(tfb[ks][j]);
  };

  wait_vmcnt<INST>();   // stage 0 has landed once only stage 1's first half is out
  block_barrier();
  bf16x8 af[2][8], bfr[2][NT];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if constexpr (B_KN) a_frag_kn(0, 0, i, af[0][i]);
    else af[0][i] = a_frag(smem_big, 0, i);
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if constexpr (B_KN) b_frag_kn(0, 0, j, tfb[0][j]);
    else bfr[0][j] = b_frag(smem_big, 0, j);
  }
  for (int kt = 0; kt < nk; ++kt) {
    // Past the end the last stage is fetched again (into buffers nobody reads any more) rather than
    // branch: a branch would end the scheduling region and undo the interleaving below.
    const int k1 = min(kt + 1, nk - 1), k2 = min(kt + 2, nk - 1);
    char* st = smem_big + (kt % STAGES) * STAGE_BYTES;          // this stage; then stage kt+2's buffer
    char* nst = smem_big + ((kt + 1) % STAGES) * STAGE_BYTES;   // stage kt+1's
    // A stage is two k-steps of 8 NT MFMAs, scheduled as four quarters (tile rows 0..3 and 4..7 of
    // a k-step).  Source order is issue order (nothing crosses a sched_barrier): after an MFMA one
    // fragment read or one load goes out.  A k-step's first MFMAs need all of its B fragments and
    // its first A fragment, so B's are read first.
    //   quarter 0: the second k-step's B fragments, and the second half of stage kt+1's loads
    //   quarter 1: the second k-step's A fragments
    //   quarter 2: nothing -- then the stage's one barrier: every wave's loads of stage kt+1 have
    //              landed and nobody reads stage kt any more (the last quarter's fragments are in registers)
    //   quarter 3: stage kt+1's first fragments, and the first half of stage kt+2's loads
    constexpr int SLOTS = 4 * NT;                              // MFMAs of a quarter
    constexpr int Q0_EVERY = (SLOTS - NT) / INST;              // quarter 0: a load every so many slots once B is read
    constexpr int Q3_FIRST = NT + 8, Q3_EVERY = (SLOTS - Q3_FIRST) / INST;
    static_assert(Q0_EVERY >= 1 && Q3_EVERY >= 1, "a quarter has a slot for each of its reads and loads");
    const int st_bytes = (kt % STAGES) * STAGE_BYTES, nst_bytes = ((kt + 1) % STAGES) * STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      if constexpr (B_KN) join_b(ks, bfr[ks], af[ks]);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int quarter = ks * 2 + (i >> 2), q = i & 3;   // q: the quarter's tile row
        if (quarter == 3 && q == 0) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          wait_vmcnt<0>();
          block_barrier();
        }
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          mfma_16x16x32_in_place(acc[i][j], bfr[ks][j], af[ks][i]);
          __builtin_amdgcn_sched_barrier(0);
          const int slot = q * NT + j;
          if (quarter == 0) {
            if (slot < NT) {
              if constexpr (B_KN) b_frag_kn(st_bytes, 1, slot, tfb[1][slot]);
              else bfr[1][slot] = b_frag(st, 1, slot);
            } else if ((slot - NT) % Q0_EVERY == 0 && (slot - NT) / Q0_EVERY < INST) issue_half(nst, k1, 1, (slot - NT) / Q0_EVERY);
          } else if (quarter == 1) {
            if (slot < 8) {
              if constexpr (B_KN) a_frag_kn(st_bytes, 1, slot, af[1][slot]);
              else af[1][slot] = a_frag(st, 1, slot);
            }
          } else if (quarter == 3) {
            if (slot < NT) {
              if constexpr (B_KN) b_frag_kn(nst_bytes, 0, slot, tfb[0][slot]);
              else bfr[0][slot] = b_frag(nst, 0, slot);
            } else if (slot < Q3_FIRST) {
              if constexpr (B_KN) a_frag_kn(nst_bytes, 0, slot - NT, af[0][slot - NT]);
              else af[0][slot - NT] = a_frag(nst, 0, slot - NT);
            } else if ((slot - Q3_FIRST) % Q3_EVERY == 0 && (slot - Q3_FIRST) / Q3_EVERY < INST)
              issue_half(st, k2, 0, (slot - Q3_FIRST) / Q3_EVERY);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }

  wait_vmcnt<0>();   // the last iteration's idle fetch must land before LDS is reused
  block_barrier();   // every wave is done reading the stages

  // Output through LDS: a wave lays its 128 x (16 NT) tile out row-major (rows padded by 16 bytes,
  // which spreads both the 8-byte writes below and the 16-byte reads over all banks) and stores
  // whole 16-byte pieces, so a row of the tile leaves as one contiguous segment.
  // acc[i][j][e]: row fr of A tile i, column 4*kq + e of B tile j.
  constexpr int OROWB = BIG_OUT_ROW_BYTES(TN);
  char* ot = smem_big + wave * (128 * OROWB);
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
      *reinterpret_cast<uint2*>(ot + (i * 16 + fr) * OROWB + (j * 16 + 4 * kq) * 2) =
          make_uint2(pack_bf16(acc[i][j][0], acc[i][j][1]), pack_bf16(acc[i][j][2], acc[i][j][3]));
  // The tile is private to the wave, whose LDS operations execute in order: no block barrier,
  // only a fence to keep the compiler from moving the reads above other lanes' writes.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  constexpr int LPRW = TN * 4;        // lanes (16 bytes each) per tile row
  constexpr int ORPI = 64 / LPRW;     // rows per instruction
  const int lr = lane / LPRW, lc = lane % LPRW;
  bf16_t* cbase = C + (size_t)(m0 + wm * 128) * N + n0 + wn * TN * 32 + lc * 8;
  // STREAM_OUT (the launch sets it over a long K): the tile leaves by non-temporal stores, so C's
  // lines do not stay in the XCD's L2 among the A and B panels its blocks re-read (8192^3: 790 ->
  // 750 us; 1 to 5 % from K = 4096 on, and 1.5 % slower at K = 2048, where a tile's stores are a
  // larger part of its time).  A template argument: as a branch on K the compiler merged the two
  // stores into one plain one.
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
#pragma unroll 4
  for (int r0 = 0; r0 < 128; r0 += ORPI) {
    const int r = r0 + lr;
    const uint4 v = *reinterpret_cast<const uint4*>(ot + r * OROWB + lc * 16);
    if (m0 + wm * 128 + r < Mv) {
      if constexpr (STREAM_OUT)
        __builtin_nontemporal_store(__builtin_bit_cast(u32x4_t, v), reinterpret_cast<u32x4_t*>(cbase + (size_t)r * N));
      else
        *reinterpret_cast<uint4*>(cbase + (size_t)r * N) = v;
    }
  }
}

template <int WAVES, int KB, bool B_KN = false, bool STREAM_OUT = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_nt256_kernel(const bf16_t* __restrict__ A,
                                                         const bf16_t* __restrict__ B,
                                                         bf16_t* __restrict__ C, int M, int N, int K,
                                                         const int* __restrict__ valid, int tiles_m,
                                                         int tiles_n, int patched) {
  gemm_nt256_body<WAVES, KB, B_KN, STREAM_OUT>(A, B, C, M, N, K, valid, tiles_m, tiles_n, patched);
}

// A row bound read on the device decides which tile size fills the chip best (512 valid rows of
// 2048 leave 64 of 256 large tiles), so under one the blocks of ONE launch choose: 256 x 256 tiles
// past `few256` rows (BIG: the shape takes them), 128 x 128 past `few128`, 64 x 64 below.  Each
// tiling's grid covers only the rows it can be chosen for; the launch's grid is the largest of
// them and a block past its tiling's tiles leaves at once.  LDS is the largest tiling's, so a CU
// holds one block whatever the choice.
template <bool BIG>
__global__ __launch_bounds__(256) void gemm_either_kernel(const bf16_t* __restrict__ A,
                                                          const bf16_t* __restrict__ B, bf16_t* __restrict__ C,
                                                          int M, int N, int K, const int* __restrict__ valid,
                                                          Tiling t256, Tiling t128, Tiling t64, int few256,
                                                          int few128, QkvTail tail) {
  // The blocks of this launch are four waves whatever the stand-alone large-tile launch uses.
  const int Mv = bound_or(valid, M), bid = blockIdx.x;
  if (BIG && Mv > few256) {
    if (bid < t256.tiles_m * t256.tiles_n)
      gemm_nt256_body<4, BIG_KB>(A, B, C, M, N, K, valid, t256.tiles_m, t256.tiles_n, t256.patched);
  } else if (Mv > few128) {
    if (bid < t128.tiles_m * t128.tiles_n)
      gemm_nt16_body<false>(A, B, C, M, N, K, valid, t128.tiles_m, t128.tiles_n, t128.patched, tail);
  } else {
    if (bid < t64.tiles_m * t64.tiles_n)
      gemm_nt64_body<8>(A, B, C, M, N, K, valid, t64.tiles_m, t64.tiles_n, t64.patched, tail);
  }
}

template <bool BIG>
static int launch_gemm_either(const bf16_t* A, const bf16_t* B, bf16_t* C, int M, int N, int K, const int* valid,
                              hipStream_t s, int few256, int few128, QkvTail tail = QkvTail{}) {
  // Rows a tiling can be chosen for: the large one all of them, the others up to the next one's bound.
  const int rows128 = BIG ? (few256 < M ? few256 : M) : M, rows64 = few128 < M ? few128 : M;
  const int n128 = (N + 127) / 128, n64 = (N + 63) / 64;
  const Tiling t256{BIG ? M / BIG_BM : 0, BIG ? N / BIG_BN : 0, BIG ? patched_order(M / BIG_BM, N / BIG_BN) : 0};
  // Tile rows rounded up to whole patches where that lets the XCD-aware order apply: the added
  // tiles lie past the bound any block of that tiling runs for, and leave at once.
  auto tiling = [](int tile_rows, int tile_cols) {
    const int whole = (tile_rows + 7) & ~7;
    if (tile_rows >= 8 && !patched_order(tile_rows, tile_cols) && patched_order(whole, tile_cols)) tile_rows = whole;
    return Tiling{tile_rows, tile_cols, patched_order(tile_rows, tile_cols)};
  };
  const Tiling t128 = tiling((rows128 + 127) / 128, n128), t64 = tiling((rows64 + 63) / 64, n64);
  constexpr size_t out_bytes = (size_t)4 * 128 * BIG_OUT_ROW_BYTES(4);   // this launch's large tiles are four waves'
  constexpr size_t lds256 = out_bytes > (size_t)2 * BIG_STAGE_BYTES ? out_bytes : (size_t)2 * BIG_STAGE_BYTES;
  constexpr size_t lds128 = (size_t)NT_STAGES * 256 * BK * 2;
  constexpr size_t lds = BIG ? (lds256 > lds128 ? lds256 : lds128) : lds128;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&gemm_either_kernel<BIG>), lds); e != hipSuccess) {
    set_error("gemm: %s", hipGetErrorString(e));
    return (int)e;
  }
  int blocks = t128.tiles_m * t128.tiles_n;
  if (t256.tiles_m * t256.tiles_n > blocks) blocks = t256.tiles_m * t256.tiles_n;
  if (t64.tiles_m * t64.tiles_n > blocks) blocks = t64.tiles_m * t64.tiles_n;
  hipLaunchKernelGGL((gemm_either_kernel<BIG>), dim3(blocks), dim3(256), lds, s, A, B, C, M, N, K, valid, t256, t128, t64,
                     few256, few128, tail);
  IRON_LAUNCH_CHECK();
}

// A residual product of few rows over a long K, followed by the RMSNorm of its rows (a prompt chunk's
// down projection: 512 live rows x 2048 columns over K = 8192, then the next layer's input norm).
// 128 x 128 tiles would occupy a quarter of the CUs and the 64 x 64 ones that fill the chip fetch
// every operand row twice as often, so a tile's K is dealt over `splits` blocks -- chosen on the
// device by the row bound: 4 while the live tiles fill a quarter of the chip, 2 up to half, else
// whole K -- each leaving its float32 sums in a workspace slice.  A second launch, a block a row,
// adds a row's slices in slice order (the same sums whatever ran first), rounds once, adds the
// residual, stores the row and norms it as rmsnorm_kernel does: that launch stands where the
// norm's own stood, so the slices' sum costs no launch of its own.
constexpr int kSplitKMax = 4;
__device__ __host__ inline int splitk_for(int live_tiles) {
  return live_tiles * 4 <= 256 ? 4 : (live_tiles * 2 <= 256 ? 2 : 1);
}
// Rows a slice of the workspace holds when K is dealt `splits` ways: the most that split count runs for.
__device__ __host__ inline size_t splitk_slice_rows(int splits, int tiles_n) {
  return (size_t)((256 / splits) / tiles_n) * 128;
}

__global__ __launch_bounds__(256) void gemm_splitk_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B,
                                                          bf16_t* __restrict__ C, int M, int N, int K,
                                                          const int* __restrict__ valid, Tiling whole, QkvTail tail,
                                                          float* __restrict__ partial) {
  const int Mv = bound_or(valid, M);
  const int tiles_n = whole.tiles_n, live_tiles = ((Mv + 127) / 128) * tiles_n;
  const int splits = splitk_for(live_tiles), id = blockIdx.x;
  if (splits == 1) {   // whole K a block, the residual in its epilogue: iron_gemm_residual_bf16's 128 x 128 launch
    if (id < whole.tiles_m * whole.tiles_n)
      gemm_nt16_body<false>(A, B, C, M, N, K, valid, whole.tiles_m, whole.tiles_n, whole.patched, tail);
    return;
  }
  // The live (tile, slice) pairs are the first ids, so that they go out one a CU whatever the
  // launch's size; an XCD (id mod 8) serves one slice of K and a band of tile columns, whose
  // A and B pieces it then re-reads from its own L2.
  const int live = live_tiles * splits;
  if (id >= live) return;
  int tile, split;
  if (live % 8 == 0) {
    const int xcd = id & 7, per = 8 / splits;
    split = xcd % splits;
    tile = (id >> 3) * per + xcd / splits;
  } else {
    split = id % splits;
    tile = id / splits;
  }
  tail.residual = nullptr;   // the second launch adds it
  tail.k_len = K / splits;
  tail.k_begin = split * tail.k_len;
  tail.partial = partial + (size_t)split * splitk_slice_rows(splits, tiles_n) * N;
  tail.tile_plus1 = tile + 1;
  gemm_nt16_body<false>(A, B, C, M, N, K, valid, (Mv + 127) / 128, tiles_n, 0, tail);
}

// The second launch: row `blockIdx.x` of C finished (from the slices, or as the first launch left
// it where K was not dealt) and normed into Y.  A thread holds CHUNKS 16-byte pieces of the row;
// every load of a piece goes out before any is used, through bounded buffers (a thread past the
// row's end reads zeros and takes no branch).  The norm's arithmetic is rmsnorm_kernel's, sum by
// sum, so Y is what iron_rmsnorm_bf16 makes of C bit for bit.
template <int CHUNKS>
__global__ __launch_bounds__(256) void gemm_finish_rows_kernel(const float* __restrict__ partial,
                                                               const bf16_t* residual, float scale, bf16_t* C,
                                                               const bf16_t* __restrict__ gain,
                                                               bf16_t* __restrict__ Y, int M, int N, float eps,
                                                               const int* __restrict__ valid, int tiles_n) {
  const int row = blockIdx.x, nchunk = N >> 3;
  const __amdgpu_buffer_rsrc_t gain_bytes = bounded_bytes(gain, N * 2);
  uint4 gains[CHUNKS];
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) gains[i] = load_bounded(gain_bytes, 16 * (threadIdx.x + 256 * i));
  const int Mv = bound_or(valid, M);
  if (row >= Mv) return;
  const int splits = splitk_for(((Mv + 127) / 128) * tiles_n);
  uint4* c_row = reinterpret_cast<uint4*>(C + (size_t)row * N);
  uint4 held[CHUNKS];
  if (splits == 1) {
    const __amdgpu_buffer_rsrc_t row_bytes = bounded_bytes(c_row, N * 2);
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) held[i] = load_bounded(row_bytes, 16 * (threadIdx.x + 256 * i));
  } else {
    const size_t slice = splitk_slice_rows(splits, tiles_n) * N;
    const __amdgpu_buffer_rsrc_t res_bytes = bounded_bytes(residual + (size_t)row * N, N * 2);
    uint4 added[CHUNKS], part[CHUNKS][kSplitKMax][2];
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      added[i] = load_bounded(res_bytes, 16 * (threadIdx.x + 256 * i));
#pragma unroll
      for (int sl = 0; sl < kSplitKMax; ++sl) {
        // slices past the split count: an empty buffer, zeros
        const __amdgpu_buffer_rsrc_t sums = bounded_bytes(partial + (sl < splits ? sl : 0) * slice + (size_t)row * N,
                                                          sl < splits ? N * 4 : 0);
        part[i][sl][0] = load_bounded(sums, 32 * (threadIdx.x + 256 * i));
        part[i][sl][1] = load_bounded(sums, 32 * (threadIdx.x + 256 * i) + 16);
      }
    }
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      float x[8], rf[8];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        f32x4 sum = __builtin_bit_cast(f32x4, part[i][0][h]);
#pragma unroll
        for (int sl = 1; sl < kSplitKMax; ++sl)
          if (sl < splits) sum += __builtin_bit_cast(f32x4, part[i][sl][h]);
#pragma unroll
        for (int e = 0; e < 4; ++e) x[4 * h + e] = sum[e];
      }
      unpack8(added[i], rf);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = fmaf(scale, round_bf16(x[e]), rf[e]);
      held[i] = pack8(x);
      const int c = threadIdx.x + 256 * i;
      if (c < nchunk) c_row[c] = held[i];
    }
  }

  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    float f[8];
    unpack8(held[i], f);
#pragma unroll
    for (int j = 0; j < 8; ++j) ss = fmaf(f[j], f[j], ss);
  }
  ss = wave_sum(ss);
  __shared__ float part_sums[4];
  if ((threadIdx.x & 63) == 0) part_sums[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float total = part_sums[0] + part_sums[1] + part_sums[2] + part_sums[3];
  const float inv = 1.0f / sqrtf(total / (float)N + eps);
  uint4* y_row = reinterpret_cast<uint4*>(Y + (size_t)row * N);
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    const int c = threadIdx.x + 256 * i;
    float f[8], g[8];
    unpack8(held[i], f);
    unpack8(gains[i], g);
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = round_bf16(f[j] * inv) * g[j];
    if (c < nchunk) y_row[c] = pack8(f);
  }
}

// A gated feed-forward's two first projections on one 128 x 128 tile position AT ONCE: a stage is the
// A tile and both weights' tiles (48 KB, three stages), an A fragment read out of LDS serves both
// products, and the gated epilogue has both accumulators in registers in the same layout, so the
// gate's product is stored (rounded, as the separate product stores it) and never read back.
// Against the same body run twice this fetches A once instead of twice (a quarter of the bytes a
// CU draws from L2 and a quarter of its LDS fragment reads).  Each product's MFMAs run in the order
// of the single-product body, so G and C are the separate launches' bit for bit.
__device__ __forceinline__ void gemm_nt16_pair_body(const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bg,
                                                    const bf16_t* __restrict__ Bu, bf16_t* __restrict__ G,
                                                    bf16_t* __restrict__ C, int M, int N, int K,
                                                    const int* __restrict__ valid, int tiles_m, int tiles_n,
                                                    int patched, int activation) {
  constexpr int NT_BM = 128, NT_BN = 128;
  constexpr int PART = NT_BM * BK * 2;             // a 128 x 64 tile's 16 KB: A, then the gate's, then the up projection's
  constexpr int STAGE = 3 * PART, STAGES = PAIR_STAGES;
  constexpr int INST = NT_BM / 8 / 4;              // 1 KB loads of each part a wave issues per stage
  constexpr int LOADS = 3 * INST;
  static_assert(BK == 64 && INST == 4, "two 32-wide k-steps a stage, twelve loads a wave");
  extern __shared__ __align__(16) char smem_nt[];
  const int Mv = bound_or(valid, M);

  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, patched, tm, tn);
  const int m0 = tm * NT_BM;
  if (m0 >= Mv) return;
  const int n0 = tn * NT_BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane >> 3, pch = lane & 7;
  int a_voff[INST], b_voff[INST];
#pragma unroll
  for (int i = 0; i < INST; ++i) {
    const int r = (wave * INST + i) * 8 + lrow;
    const int lch = pch ^ ((r >> 1) & 7);
    // Rows past the end re-read the last row; what they produce is never stored.
    a_voff[i] = (int)(((size_t)(min(m0 + r, M - 1) - m0) * K + lch * 8) * 2);
    b_voff[i] = (int)(((size_t)(min(n0 + r, N - 1) - n0) * K + lch * 8) * 2);
  }
  const bf16_t* a_tile = A + (size_t)m0 * K;
  const bf16_t* g_tile = Bg + (size_t)n0 * K;
  const bf16_t* u_tile = Bu + (size_t)n0 * K;
  auto issue_one = [&](char* st, int kt, int idx) {   // idx: 0..3 A, 4..7 the gate's weights, 8..11 the up projection's
    const int k0 = kt * BK, part = idx / INST, piece = idx % INST;
    const bf16_t* from = part == 0 ? a_tile : (part == 1 ? g_tile : u_tile);
    const __amdgpu_buffer_rsrc_t rows = stage_rows(from + k0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rows, IRON_LDS_PTR(st + part * PART + (wave * INST + piece) * 1024), 16,
                                             (int)(part == 0 ? a_voff[piece] : b_voff[piece]), 0, 0, 0);
  };

  f32x4 accg[4][4], accu[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) accg[i][j][e] = accu[i][j][e] = 0.f;

  const int nk = K / BK;
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
#pragma unroll
    for (int idx = 0; idx < LOADS; ++idx) issue_one(smem_nt + s * STAGE, min(s, nk - 1), idx);

  // Fragments: lane -> row fr of a 16-row tile, 16-byte chunk kq of the k-step's four.
  const int fr = lane & 15, kq = lane >> 4;
  const int swz = (fr >> 1) & 7;   // tile rows are multiples of 16 apart: one swizzle for all
  const int a_row = (wm * 64 + fr) * 128, b_row = (wn * 64 + fr) * 128;
  auto a_frag = [&](const char* st, int ks, int i) {
    return *reinterpret_cast<const bf16x8*>(st + a_row + i * 16 * 128 + (((ks * 4 + kq) ^ swz) << 4));
  };
  auto b_frag = [&](const char* st, int part, int ks, int j) {
    return *reinterpret_cast<const bf16x8*>(st + part * PART + b_row + j * 16 * 128 + (((ks * 4 + kq) ^ swz) << 4));
  };

  wait_vmcnt<(STAGES - 2) * LOADS>();   // stage 0 has landed once only the younger one is out
  block_barrier();
  bf16x8 af[2][4], bg[2][4], bu[2][4];
#pragma unroll
  for (int i = 0; i < 4; ++i) bg[0][i] = b_frag(smem_nt, 1, 0, i);
#pragma unroll
  for (int i = 0; i < 4; ++i) bu[0][i] = b_frag(smem_nt, 2, 0, i);
#pragma unroll
  for (int i = 0; i < 4; ++i) af[0][i] = a_frag(smem_nt, 0, i);
  // One stage of the loop, which is unrolled over the three stage buffers (stage_c = kt % STAGES): a
  // fragment's stage then rides in its read's offset field instead of a vector add a read.
  auto stage_step = [&](int kt, auto stage_c) {
    constexpr int S = decltype(stage_c)::value;
    // Prefetch goes into the buffer of stage kt-1.  Past the end the last stage is fetched again
    // (into buffers nobody reads any more) rather than branch: every iteration issues the same
    // loads, which keeps the wait counts exact and the scheduling region whole.
    const int kn = min(kt + STAGES - 1, nk - 1);
    char* nst = smem_nt + ((S + STAGES - 1) % STAGES) * STAGE;
    const char* st = smem_nt + S * STAGE;
    const char* st1 = smem_nt + ((S + 1) % STAGES) * STAGE;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      if (ks == 1) {
        // The stage's one barrier, before its second k-step (whose fragments are in registers): of
        // the loads in flight the oldest LOADS are stage kt+1's, then the half of stage kt+2's
        // issued so far; after it nobody reads stage kt any more.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_vmcnt<LOADS / 2>();
        block_barrier();
      }
      const char* from = ks == 0 ? st : st1;
      const int nks = ks ^ 1;
      // Source order is issue order (nothing crosses a sched_barrier): after an MFMA one fragment
      // read of the next k-step (the weights' first: its first MFMAs need all of them) or one load.
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (j < 4) mfma_16x16x32_in_place(accg[i][j], bg[ks][j], af[ks][i]);
          else mfma_16x16x32_in_place(accu[i][j - 4], bu[ks][j - 4], af[ks][i]);
          __builtin_amdgcn_sched_barrier(0);
          const int slot = i * 8 + j;
          if (slot < 4) bg[nks][slot] = b_frag(from, 1, nks, slot);
          else if (slot < 8) bu[nks][slot - 4] = b_frag(from, 2, nks, slot - 4);
          else if (slot < 12) af[nks][slot - 8] = a_frag(from, nks, slot - 8);
          else if ((slot & 1) && slot < 12 + LOADS) issue_one(nst, kn, ks * (LOADS / 2) + (slot - 13) / 2);
          __builtin_amdgcn_sched_barrier(0);
        }
    }
  };
  static_assert(STAGES == 3, "the loop below names the three stage buffers");
  for (int kt0 = 0; kt0 < nk; kt0 += STAGES) {
    stage_step(kt0, std::integral_constant<int, 0>{});
    if (kt0 + 1 < nk) stage_step(kt0 + 1, std::integral_constant<int, 1>{});
    if (kt0 + 2 < nk) stage_step(kt0 + 2, std::integral_constant<int, 2>{});
  }

  wait_vmcnt<0>();   // the idle fetches of the last iterations land ...
  block_barrier();   // ... in every wave, and every wave is done with the stages, before LDS is reused

  // Output through LDS, a product at a time: the wave lays its 64 x 64 out row-major (rows padded by
  // 16 bytes) and each lane then owns 8 consecutive columns of a row, so a row of the tile leaves as
  // one 128-byte segment.  First the gate's product as it is stored; then, made in the accumulators'
  // own layout, bf16(bf16(act(bf16 g)) * bf16 u).
  constexpr int OROWB = 64 * 2 + 16;
  char* ot = smem_nt + wave * (64 * OROWB);
  const int out_row = lane >> 3, out_col = (lane & 7) * 8;
  const int out_n = n0 + wn * 64 + out_col;
  const bool whole = (N & 7) == 0 && out_n + 8 <= N;
  auto leave = [&](bf16_t* to) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int row = r * 8 + out_row, m = m0 + wm * 64 + row;
      const uint4 v = *reinterpret_cast<const uint4*>(ot + row * OROWB + out_col * 2);
      if (m >= Mv || out_n >= N) continue;
      bf16_t* p = to + (size_t)m * N + out_n;
      if (whole) {
        *reinterpret_cast<uint4*>(p) = v;
      } else {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (out_n + e < N) p[e] = (bf16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu));
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();   // the rows are read before the next product overwrites them
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *reinterpret_cast<uint2*>(ot + (i * 16 + fr) * OROWB + (j * 16 + 4 * kq) * 2) =
          make_uint2(pack_bf16(accg[i][j][0], accg[i][j][1]), pack_bf16(accg[i][j][2], accg[i][j][3]));
  leave(G);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float c[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        c[e] = round_bf16(gate_of(activation, round_bf16(accg[i][j][e]))) * round_bf16(accu[i][j][e]);
      *reinterpret_cast<uint2*>(ot + (i * 16 + fr) * OROWB + (j * 16 + 4 * kq) * 2) =
          make_uint2(pack_bf16(c[0], c[1]), pack_bf16(c[2], c[3]));
    }
  leave(C);
}

// A gated feed-forward's two first projections over many rows as ONE launch: a block computes its
// tile of the gate's product and stores it (rounded, as the separate product stores it), then
// computes the same tile of the second product, whose epilogue reads the gate tile back -- the one
// this very block wrote, so nothing crosses between blocks -- and leaves bf16(bf16(act(g)) * bf16(u)).
// What goes is a launch boundary: the second launch's start, its first stages' fill and the first
// one's drain.  The tile size is chosen on the device by the row bound as in gemm_either_kernel.
__global__ __launch_bounds__(256) void gemm_gated_pair_kernel(const bf16_t* __restrict__ A,
                                                              const bf16_t* __restrict__ Bg,
                                                              const bf16_t* __restrict__ Bu, bf16_t* __restrict__ G,
                                                              bf16_t* __restrict__ C, int M, int N, int K,
                                                              const int* __restrict__ valid, Tiling t128, Tiling t64,
                                                              int few128, int activation) {
  const int Mv = bound_or(valid, M), bid = blockIdx.x;
  QkvTail none{}, gate{};
  gate.residual = G;
  gate.gated = activation;
  if (Mv > few128) {
    if (bid >= t128.tiles_m * t128.tiles_n) return;
    gemm_nt16_pair_body(A, Bg, Bu, G, C, M, N, K, valid, t128.tiles_m, t128.tiles_n, t128.patched, activation);
  } else {
    if (bid >= t64.tiles_m * t64.tiles_n) return;
    gemm_nt64_body<8>(A, Bg, G, M, N, K, valid, t64.tiles_m, t64.tiles_n, t64.patched, none);
    __syncthreads();
    gemm_nt64_body<8>(A, Bu, C, M, N, K, valid, t64.tiles_m, t64.tiles_n, t64.patched, gate);
  }
}

static int launch_gemm_gated_pair(const bf16_t* A, const bf16_t* Bg, const bf16_t* Bu, bf16_t* G, bf16_t* C, int M,
                                  int N, int K, const int* valid, int activation, hipStream_t s) {
  const int n128 = (N + 127) / 128, n64 = (N + 63) / 64;
  // 64 x 64 tiles up to the rows below which 128 x 128 ones would leave half the CUs idle (as iron_gemm_bf16).
  int few128 = n128 >= 128 ? 0 : 128 * (127 / n128);
  if (few128 > M) few128 = M;
  auto tiling = [](int tile_rows, int tile_cols) {
    const int whole = (tile_rows + 7) & ~7;
    if (tile_rows >= 8 && !patched_order(tile_rows, tile_cols) && patched_order(whole, tile_cols)) tile_rows = whole;
    return Tiling{tile_rows, tile_cols, patched_order(tile_rows, tile_cols)};
  };
  const Tiling t128 = tiling((M + 127) / 128, n128), t64 = tiling((few128 + 63) / 64, n64);
  constexpr size_t lds = (size_t)PAIR_STAGES * 3 * 128 * BK * 2;   // the two-product body's stages, more than the others'
  static_assert(lds >= (size_t)NT_STAGES * 256 * BK * 2, "the 64 x 64 body's stages fit too");
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&gemm_gated_pair_kernel), lds); e != hipSuccess) {
    set_error("gemm_gated_pair: %s", hipGetErrorString(e));
    return (int)e;
  }
  int blocks = t128.tiles_m * t128.tiles_n;
  if (t64.tiles_m * t64.tiles_n > blocks) blocks = t64.tiles_m * t64.tiles_n;
  hipLaunchKernelGGL(gemm_gated_pair_kernel, dim3(blocks), dim3(256), lds, s, A, Bg, Bu, G, C, M, N, K, valid, t128, t64,
                     few128, activation);
  IRON_LAUNCH_CHECK();
}

template <bool B_KN, bool STREAM_OUT>
static int launch_gemm_nt256_as(const bf16_t* A, const bf16_t* B, bf16_t* C, int M, int N, int K,
                                const int* valid, hipStream_t s) {
  const int tiles_m = M / BIG_BM, tiles_n = N / BIG_BN;
  constexpr size_t out_bytes = (size_t)BIG_WAVES * 128 * BIG_OUT_ROW_BYTES(8 / BIG_WAVES * 2);
  const size_t lds = out_bytes > (size_t)2 * BIG_STAGE_BYTES ? out_bytes : (size_t)2 * BIG_STAGE_BYTES;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&gemm_nt256_kernel<BIG_WAVES, BIG_KB, B_KN, STREAM_OUT>), lds);
      e != hipSuccess) {
    set_error("gemm: %s", hipGetErrorString(e));
    return (int)e;
  }
  const int patched = (tiles_m % 8 == 0 && tiles_n % 4 == 0 && ((tiles_m / 8) * (tiles_n / 4)) % 8 == 0) ? 1 : 0;
  hipLaunchKernelGGL((gemm_nt256_kernel<BIG_WAVES, BIG_KB, B_KN, STREAM_OUT>), dim3(tiles_m * tiles_n), dim3(BIG_WAVES * 64), lds, s,
                     A, B, C, M, N, K, valid, tiles_m, tiles_n, patched);
  IRON_LAUNCH_CHECK();
}

// Over a long K the tiles leave by non-temporal stores (see the body's epilogue).
template <bool B_KN = false>
static int launch_gemm_nt256(const bf16_t* A, const bf16_t* B, bf16_t* C, int M, int N, int K,
                             const int* valid, hipStream_t s) {
  if (K >= 4096) return launch_gemm_nt256_as<B_KN, true>(A, B, C, M, N, K, valid, s);
  return launch_gemm_nt256_as<B_KN, false>(A, B, C, M, N, K, valid, s);
}

}  // namespace iron

using namespace iron;

extern "C" int iron_gemm_bf16(const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K,
                              int b_col_maj, int c_col_maj, const int* valid, const int* valid_k,
                              void* stream) {
  IRON_REQUIRE(A && B && C, "gemm: null operand");
  IRON_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: M (%d), N (%d), K (%d) must be positive", M, N, K);
  IRON_REQUIRE(K % 8 == 0, "gemm: K (%d) must be a multiple of 8 (16-byte loads)", K);
  IRON_REQUIRE(K <= (1 << 22) && N <= (1 << 22),
               "gemm: K (%d) and N (%d) may be at most 2^22 (a tile's rows are addressed with 32-bit offsets)", K, N);
  IRON_REQUIRE((((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) == 0,
               "gemm: operands must be 16-byte aligned");
  IRON_REQUIRE(b_col_maj || N % 8 == 0,
               "gemm: N (%d) must be a multiple of 8 when B is (K,N) (16-byte loads along N)", N);
  hipStream_t s = (hipStream_t)stream;
  if (!c_col_maj && valid_k == nullptr && K % BK == 0 && M >= 64 && N >= 64) {
    // Enough whole 256x256 tiles to fill the chip: the large-tile kernel (offsets are 32-bit).
    if (b_col_maj && M % BIG_BM == 0 && N % BIG_BN == 0 && (long)(M / BIG_BM) * (N / BIG_BN) >= 192 &&
        K <= (1 << 24)) {
      // Under a row bound read on the device the large tiles may cover too few rows to fill the
      // chip (512 valid rows of 2048 leave 64 of 256 tiles): the blocks of one launch then choose
      // the tile size where the bound is known, on the device.
      const int tiles_n256 = N / BIG_BN, tiles_n128 = N / 128;
      const int few256 = tiles_n256 >= 128 ? 0 : BIG_BM * (128 / tiles_n256);   // rows up to which 128x128 tiles win
      const int few128 = tiles_n128 >= 128 ? 0 : 128 * (127 / tiles_n128);      // ... and 64x64 ones
      if (valid == nullptr || few256 == 0 || few256 >= M) return launch_gemm_nt256(A, B, C, M, N, K, valid, s);
      return launch_gemm_either<true>(A, B, C, M, N, K, valid, s, few256, few128);
    }
    if (b_col_maj) {
      // 128x128 tiles that would occupy under half the CUs give way to 64x64 ones: always, where
      // the shape says so; under a row bound, the blocks of one launch choose where the bound is
      // known (the few-row 64x64 tiles run the eight-stage pipeline, a block a CU, so nothing is
      // lost to the launch's 128 KB of LDS and the second, empty launch is saved).
      const int tiles_n128 = (N + 127) / 128;
      const long tiles128 = (long)((M + 127) / 128) * tiles_n128;
      if (tiles128 < 128) return launch_gemm_nt<false, false, 1>(A, B, C, M, N, K, valid, s);
      const int few = tiles_n128 >= 128 ? 0 : 128 * (127 / tiles_n128);   // rows up to which 64x64 tiles win
      if (valid == nullptr || few == 0 || few >= M) return launch_gemm_nt<false>(A, B, C, M, N, K, valid, s);
      return launch_gemm_either<false>(A, B, C, M, N, K, valid, s, 0, few);
    }
    // (K,N) B is read in whole tiles straight into LDS: N must be whole tiles.  Enough whole
    // 256x256 tiles to fill the chip, and a matrix a 32-bit byte offset spans: the large-tile kernel.
    if (valid == nullptr && M % BIG_BM == 0 && N % BIG_BN == 0 && (long)(M / BIG_BM) * (N / BIG_BN) >= 192 &&
        (long)K * N * 2 < (1L << 31))
      return launch_gemm_nt256<true>(A, B, C, M, N, K, valid, s);
    if (N % 128 == 0) return launch_gemm_nt<true>(A, B, C, M, N, K, valid, s);
  }
  // 128x128 tiles fill the 256 CUs once at 2048x2048; narrower problems take 64-wide tiles.
  const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
  if (tiles128 >= 128 || (M >= 128 && N >= 128))
    return launch_gemm<128, 128, 2, 2>(A, B, C, M, N, K, b_col_maj, c_col_maj, valid, valid_k, s);
  return launch_gemm<64, 64, 2, 2>(A, B, C, M, N, K, b_col_maj, c_col_maj, valid, valid_k, s);
}

// A product over many rows whose epilogue reads a second (M, N) operand: the residual sum or the gate.
static int gemm_with_tail(const char* what, const uint16_t* A, const uint16_t* B, const uint16_t* R, uint16_t* C,
                          int M, int N, int K, const QkvTail& tail, const int* valid, void* stream) {
  IRON_REQUIRE(A && B && R && C, "%s: null operand", what);
  IRON_REQUIRE(K <= (1 << 22) && N <= (1 << 22),
               "%s: K (%d) and N (%d) may be at most 2^22 (a tile's rows are addressed with 32-bit offsets)", what, K, N);
  IRON_REQUIRE(M >= 64 && N >= 64 && K > 0 && K % BK == 0,
               "%s: M (%d) and N (%d) at least 64, K (%d) a positive multiple of %d", what, M, N, K, BK);
  IRON_REQUIRE((((uintptr_t)A | (uintptr_t)B | (uintptr_t)R | (uintptr_t)C) & 15) == 0,
               "%s: operands must be 16-byte aligned", what);
  hipStream_t s = (hipStream_t)stream;
  // The tile sizes of iron_gemm_bf16's (N,K) path below the 256-wide ones.
  const int tiles_n128 = (N + 127) / 128;
  const long tiles128 = (long)((M + 127) / 128) * tiles_n128;
  if (tiles128 < 128) return launch_gemm_nt<false, false, 1>(A, B, C, M, N, K, valid, s, tail);
  const int few = tiles_n128 >= 128 ? 0 : 128 * (127 / tiles_n128);
  if (valid == nullptr || few == 0 || few >= M) return launch_gemm_nt<false>(A, B, C, M, N, K, valid, s, tail);
  return launch_gemm_either<false>(A, B, C, M, N, K, valid, s, 0, few, tail);
}

extern "C" int iron_gemm_residual_bf16(const uint16_t* A, const uint16_t* B, const uint16_t* R, uint16_t* C, int M,
                                       int N, int K, float residual_scale, const int* valid, void* stream) {
  QkvTail tail{};
  tail.residual = R;
  tail.residual_scale = residual_scale;
  return gemm_with_tail("gemm_residual", A, B, R, C, M, N, K, tail, valid, stream);
}

// Whether (and with how much workspace) a residual product followed by its rows' norm is worth
// dealing its K over several blocks: whole 128-column tiles too few to fill the chip at some row
// count, a K long enough to cut, rows a block of the second launch can hold.
extern "C" int64_t iron_gemm_residual_norm_workspace_bytes(int M, int N, int K) {
  if (M < 128 || N < 128 || N % 128 != 0 || N > 8192 || K < 4096 || K % (BK * kSplitKMax) != 0) return 0;
  const int tiles_n = N / 128;
  // splits x the rows a split count runs for is the same for every split count: 256 tiles' worth of rows.
  return (int64_t)(256 / tiles_n) * 128 * N * (int64_t)sizeof(float);
}

extern "C" int iron_gemm_residual_norm_bf16(const uint16_t* A, const uint16_t* B, const uint16_t* R,
                                            const uint16_t* gain, uint16_t* C, uint16_t* Y, int M, int N, int K,
                                            float residual_scale, float eps, const int* valid, void* workspace,
                                            void* stream) {
  IRON_REQUIRE(A && B && R && gain && C && Y && workspace, "gemm_residual_norm: null operand");
  IRON_REQUIRE(iron_gemm_residual_norm_workspace_bytes(M, N, K) > 0,
               "gemm_residual_norm: M (%d) at least 128, N (%d) a multiple of 128 up to 8192, K (%d) a multiple of %d "
               "from 4096 on (other shapes: iron_gemm_residual_bf16, then iron_rmsnorm_bf16)", M, N, K, BK * kSplitKMax);
  IRON_REQUIRE(K <= (1 << 22), "gemm_residual_norm: K (%d) may be at most 2^22 (a tile's rows are addressed with 32-bit offsets)", K);
  IRON_REQUIRE((((uintptr_t)A | (uintptr_t)B | (uintptr_t)R | (uintptr_t)gain | (uintptr_t)C | (uintptr_t)Y |
                 (uintptr_t)workspace) & 15) == 0,
               "gemm_residual_norm: operands must be 16-byte aligned");
  IRON_REQUIRE(Y != C && Y != R, "gemm_residual_norm: the normed rows need a buffer of their own");
  hipStream_t s = (hipStream_t)stream;
  int tiles_m = (M + 127) / 128;
  const int tiles_n = N / 128;
  // Whole-K tiles in the XCD-aware order where whole patches allow it (the added tile rows lie past M).
  if (tiles_m >= 8 && !patched_order(tiles_m, tiles_n) && patched_order((tiles_m + 7) & ~7, tiles_n))
    tiles_m = (tiles_m + 7) & ~7;
  const Tiling whole{tiles_m, tiles_n, patched_order(tiles_m, tiles_n)};
  QkvTail tail{};
  tail.residual = R;
  tail.residual_scale = residual_scale;
  constexpr size_t lds = (size_t)NT_STAGES * 256 * BK * 2;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&gemm_splitk_kernel), lds); e != hipSuccess) {
    set_error("gemm_residual_norm: %s", hipGetErrorString(e));
    return (int)e;
  }
  const int blocks = whole.tiles_m * whole.tiles_n > 256 ? whole.tiles_m * whole.tiles_n : 256;
  hipLaunchKernelGGL(gemm_splitk_kernel, dim3(blocks), dim3(256), lds, s, A, B, C, M, N, K, valid, whole, tail,
                     (float*)workspace);
  const int chunks = (N / 8 + 255) / 256;
#define IRON_FINISH(CH)                                                                                          \
  hipLaunchKernelGGL((gemm_finish_rows_kernel<CH>), dim3(M), dim3(256), 0, s, (const float*)workspace, R,        \
                     residual_scale, C, gain, Y, M, N, eps, valid, tiles_n)
  if (chunks <= 1) IRON_FINISH(1);
  else if (chunks == 2) IRON_FINISH(2);
  else IRON_FINISH(4);
#undef IRON_FINISH
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_gemm_gated_bf16(const uint16_t* A, const uint16_t* B, const uint16_t* G, uint16_t* C, int M,
                                    int N, int K, int activation, const int* valid, void* stream) {
  IRON_REQUIRE(activation == 1 || activation == 2, "gemm_gated: activation (%d) is 1 (SiLU) or 2 (GELU, tanh form)",
               activation);
  QkvTail tail{};
  tail.residual = G;
  tail.gated = activation;
  return gemm_with_tail("gemm_gated", A, B, G, C, M, N, K, tail, valid, stream);
}

extern "C" int iron_gemm_gated_pair_bf16(const uint16_t* A, const uint16_t* Bg, const uint16_t* Bu, uint16_t* G,
                                         uint16_t* C, int M, int N, int K, int activation, const int* valid,
                                         void* stream) {
  IRON_REQUIRE(A && Bg && Bu && G && C, "gemm_gated_pair: null operand");
  IRON_REQUIRE(activation == 1 || activation == 2, "gemm_gated_pair: activation (%d) is 1 (SiLU) or 2 (GELU, tanh form)",
               activation);
  IRON_REQUIRE(G != C, "gemm_gated_pair: the gate's product and the output are different buffers");
  IRON_REQUIRE(K <= (1 << 22) && N <= (1 << 22),
               "gemm_gated_pair: K (%d) and N (%d) may be at most 2^22 (a tile's rows are addressed with 32-bit offsets)", K, N);
  IRON_REQUIRE(M >= 64 && N >= 64 && K > 0 && K % BK == 0,
               "gemm_gated_pair: M (%d) and N (%d) at least 64, K (%d) a positive multiple of %d", M, N, K, BK);
  IRON_REQUIRE((((uintptr_t)A | (uintptr_t)Bg | (uintptr_t)Bu | (uintptr_t)G | (uintptr_t)C) & 15) == 0,
               "gemm_gated_pair: operands must be 16-byte aligned");
  return launch_gemm_gated_pair(A, Bg, Bu, G, C, M, N, K, valid, activation, (hipStream_t)stream);
}

static int prefill_qkv(const uint16_t* x, const uint16_t* Wq, const uint16_t* Wk, const uint16_t* Wv,
                       const uint16_t* angles, uint16_t* q_out, uint16_t* k_out, uint16_t* v_out, int rows,
                       int hidden, int heads, int kv_heads, int d, const int* valid, const int* kv_row0,
                       int kv_rows, void* stream) {
  IRON_REQUIRE(x && Wq && Wk && Wv && angles && q_out && k_out && v_out, "prefill_qkv: null operand");
  IRON_REQUIRE(d == 64, "prefill_qkv: d (%d) must be 64 (a wave's 64 output columns are one head)", d);
  IRON_REQUIRE(rows >= 64 && heads > 0 && kv_heads > 0 && heads % 2 == 0 && kv_heads % 2 == 0,
               "prefill_qkv: rows (%d) at least 64; heads (%d) and kv_heads (%d) positive and even "
               "(whole 128-column tiles)", rows, heads, kv_heads);
  IRON_REQUIRE(hidden > 0 && hidden % BK == 0, "prefill_qkv: hidden (%d) must be a positive multiple of %d", hidden, BK);
  IRON_REQUIRE(hidden <= (1 << 22), "prefill_qkv: hidden (%d) may be at most 2^22 (a tile's rows are addressed with 32-bit offsets)", hidden);
  IRON_REQUIRE((((uintptr_t)x | (uintptr_t)Wq | (uintptr_t)Wk | (uintptr_t)Wv | (uintptr_t)angles |
                 (uintptr_t)q_out | (uintptr_t)k_out | (uintptr_t)v_out) & 15) == 0,
               "prefill_qkv: operands must be 16-byte aligned");
  QkvTail tail{Wk, Wv, k_out, v_out, angles, kv_heads * d};
  tail.kv_row0 = kv_row0;
  tail.kv_rows = kv_rows;
  hipStream_t s = (hipStream_t)stream;
  // 192-wide tiles (three heads) when they make fewer rounds over the chip than 128-wide ones: in
  // units of a 128 x 128 tile's work a launch costs rounds x tile width.  The row bound is read on
  // the device, so with one the blocks of one launch choose the tiling by it.
  const int total = heads + 2 * kv_heads, cus = 256;
  auto cost = [&](int live_rows, int tile_n, int n_tiles) {
    const int tiles = ((live_rows + 127) / 128) * n_tiles;
    return (double)((tiles + cus - 1) / cus) * tile_n;
  };
  const bool wide_ok = total % 3 == 0;
  auto wide_wins = [&](int live_rows) {
    return wide_ok && cost(live_rows, 192, total / 3) < cost(live_rows, 128, total / 2);
  };
  // One-head tiles while they fit one round over the chip and beat both of the others' cost.
  auto thin_wins = [&](int live_rows) {
    const double c = cost(live_rows, 64, total);
    return ((live_rows + 127) / 128) * total <= cus && c < cost(live_rows, 128, total / 2) &&
           (!wide_ok || c < cost(live_rows, 192, total / 3));
  };
  int thin_upto = 0;
  for (int live = 128; live <= ((rows + 127) / 128) * 128; live += 128)
    if (thin_wins(live)) thin_upto = live;
  if (thin_upto >= rows) return launch_qkv64(x, Wq, q_out, rows, heads, kv_heads, hidden, valid, s, tail);
  // The bound above which the winner at `rows` wins, if the two ever change places below `rows`.
  int above = -1;
  if (valid != nullptr)
    for (int live = 128; live <= rows; live += 128)
      if (wide_wins(live) != wide_wins(rows)) above = live;
  if (valid == nullptr) thin_upto = 0;
  if (above < 0 && thin_upto == 0) {
    if (wide_wins(rows)) return launch_qkv192(x, Wq, q_out, rows, heads, kv_heads, hidden, valid, s, tail);
    return launch_gemm_nt<false, true>(x, Wq, q_out, rows, heads * d, hidden, valid, s, tail);
  }
  return launch_qkv_either(x, Wq, q_out, rows, heads, kv_heads, hidden, valid, s, tail, above, wide_wins(rows), wide_ok,
                           thin_upto);
}

extern "C" int iron_prefill_qkv_bf16(const uint16_t* x, const uint16_t* Wq, const uint16_t* Wk,
                                     const uint16_t* Wv, const uint16_t* angles, uint16_t* q_out,
                                     uint16_t* k_out, uint16_t* v_out, int rows, int hidden, int heads,
                                     int kv_heads, int d, const int* valid, void* stream) {
  return prefill_qkv(x, Wq, Wk, Wv, angles, q_out, k_out, v_out, rows, hidden, heads, kv_heads, d, valid, nullptr, 0,
                     stream);
}

extern "C" int iron_prefill_qkv_cache_bf16(const uint16_t* x, const uint16_t* Wq, const uint16_t* Wk,
                                           const uint16_t* Wv, const uint16_t* angles, uint16_t* q_out,
                                           uint16_t* keys, uint16_t* values, int rows, int hidden, int heads,
                                           int kv_heads, int d, int cache_rows, const int* start,
                                           const int* valid, void* stream) {
  IRON_REQUIRE(start != nullptr, "prefill_qkv_cache: null start");
  IRON_REQUIRE(cache_rows > 0, "prefill_qkv_cache: cache_rows (%d) must be positive", cache_rows);
  // Whatever the bound word holds it is at most `rows`: the rows under it then fit the cache from some row on.
  IRON_REQUIRE(rows <= cache_rows, "prefill_qkv_cache: the chunk's %d rows must fit the cache's %d", rows, cache_rows);
  return prefill_qkv(x, Wq, Wk, Wv, angles, q_out, keys, values, rows, hidden, heads, kv_heads, d, valid, start,
                     cache_rows, stream);
}
