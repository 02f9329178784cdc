// Attention for many queries (prefill / prompt chunk) on the MFMA matrix cores:
// flash-style, causal / windowed, grouped-query, the queries being the last rows
// of the keys.
//
// grid = ceil(seq/128) * heads; a block of 4 waves takes 128 query rows of one
// head, a wave 32 of them.  Keys and values stream through LDS in tiles of 64
// rows.  The wave computes the TRANSPOSED score tile S^T = K Q^T (M = keys,
// N = queries): a lane then owns one query column, so the row max / row sum of
// the online softmax are in-lane reductions plus one exchange with lane^32, and
// the probabilities are already laid out as the B operand of O^T = V^T P^T.  V^T
// fragments come from the transposing LDS read.  All softmax state is f32 in the
// exp2 domain; the reference the exponents are taken against follows the maxima
// lazily, and a tile whose sums of exponentials stay in range never takes its
// maximum (tile_step below).
#include "../../include/iron_hip.h"
#include "common.h"

#include <type_traits>

namespace iron {

// max(x, x of the lane 32 away) without a trip through LDS: the two halves of the wave swapped
// between two copies (v_permlane32_swap), then one maximum.  The wait states between a vector
// write and the swap that reads it, and between the swap and what reads its results, are in the
// statement, since the compiler does not look inside it.
__device__ __forceinline__ float max_with_other_half(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
}

constexpr int BQ = 128;   // query rows per block (four waves of 32; 64 where a block is two)
constexpr int BKV = 64;   // key rows per tile
constexpr float kLazyBits = 8.f;        // how far a maximum may run ahead of the reference the exponents are taken against
constexpr float kSumLow = 0x1p-60f, kSumHigh = 0x1p24f;   // a tile's sum of exponentials outside this range: take its maximum and redo it
constexpr int kCUs = 256;                // compute units the block orders below assume
constexpr int kFewBlocks = 512;          // launches of fewer blocks than this halve their blocks' queries (S = 1024 at 32 heads: 18.5 -> 13.9 us)
constexpr int kWideBigBlocks = 512;     // wide heads: launches of at least this many 128-query blocks keep that size
constexpr int kSplitMaxBlocks = 1024;   // launches of up to this many blocks split each block's tiles over two halves

// K and V tiles go straight from global memory into LDS (buffer loads with the LDS bit, no register staging), as
// stored: [64 keys][D], STAGES tiles deep.  16-byte chunks of a row are XOR-swizzled so unpadded
// rows read without bank conflicts: K by (key >> 1) & 7 for its 16-byte fragment reads, V by
// 2 * (key & 3) for the transposing reads (ds_read_b64_tr_b16) that deliver V^T fragments.  A bare
// s_barrier and counted s_waitcnt vmcnt keep the younger tiles' loads in flight across the barrier.
//
// At least two waves a SIMD caps the register budget at 256, which makes the compiler keep MFMA
// accumulators in ordinary VGPRs: the softmax reads S and rescales O in place instead of copying
// every value out of (and back into) accumulation registers.  The eight-wave form at d = 64 is held
// to 128 registers and two stages (64 KB), so that a CU holds two blocks at different places of their
// loops (S = 4096: 118 -> 95 us; the 64-query blocks of short prompts likewise); three four-wave blocks a CU measured slower than two (S = 8192:
// 382 against 365 us).
//
// SPLIT = 2: eight waves; waves 4..7 serve the same four groups of 32 queries as waves 0..3 but take
// the odd key tiles (their own loads, their own stage buffers), and the two halves' (max, sum, O)
// are merged through LDS at the end.  A query block's chain of tiles is half as long, which is what
// bounds a short sequence: its blocks are few and the one that sees every key finishes last.
//
// W: the waves that share a tile's loads, each with 32 of the block's 32 W queries.  Four; two
// where four would leave CUs without a block (a short prompt), so that twice as many blocks go out.
template <int D, int SPLIT, int W = 4>
__global__ __launch_bounds__(64 * W * SPLIT) __attribute__((amdgpu_waves_per_eu(W == 4 ? (D == 64 && SPLIT == 2 ? 4 : 2) : (D == 64 && SPLIT == 2 ? 2 : 1)))) void mha_prefill_kernel(
    const bf16_t* __restrict__ Q, const bf16_t* __restrict__ K, const bf16_t* __restrict__ V,
    bf16_t* __restrict__ O, int heads, int group, int seq, int seq_len, int kv_len, float scale_log2,
    int causal, int window, long q_row_stride, long q_head_stride, long kv_row_stride,
    long kv_head_stride, const int* __restrict__ valid, const int* __restrict__ kv_valid,
    const int* __restrict__ kv_first, int kv_rows) {
  constexpr int ROWB = D * 2;            // bytes of a tile row
  constexpr int KS = D / 16;             // k16 steps of S^T
  constexpr int DT = D / 32;             // 32-row tiles of O^T
  constexpr int CPR = D / 8;             // 16-byte chunks a row has
  constexpr int STAGES = D == 64 && SPLIT == 1 ? 3 : 2;
  constexpr int TILE = BKV * ROWB;       // bytes of a K (or V) tile
  constexpr int STAGE = 2 * TILE;
  constexpr int BQW = 32 * W;            // query rows of this block
  constexpr int INST = TILE / 1024 / W;  // 1 KB loads of K (and of V) a wave issues per tile
  constexpr int RPI = 1024 / ROWB;       // rows one load covers
  extern __shared__ __align__(1024) char smem_all[];   // SPLIT * STAGES * STAGE bytes

  const int tid = threadIdx.x, lane = tid & 63;
  // Which tiles, and which 32 queries -- uniform over the wave, so what depends on them (LDS
  // destinations, the rows a wave loads) stays in scalar registers.
  const int wave_id = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = wave_id / W, wave = wave_id % W;
  char* smem = smem_all + half * (STAGES * STAGE);            // this half's stage buffers
  const int col = lane & 31, g = lane >> 5;
  // Blocks are dispatched in id order, so the id runs over the query blocks from the last (under a
  // causal mask the heaviest: it sees the most keys) to the first, all heads of one query block
  // together: the long blocks start first and the short ones fill the tail.  Within a query block
  // the heads are dealt so that an XCD (block id mod 8) serves the heads of one KV group, whose
  // K and V it then reads from its own L2.
  const int j = blockIdx.x % heads;
  const int head = (heads % 8 == 0) ? (j % 8) * (heads / 8) + j / 8 : j;
  const int kvh = head / group;
  // A launch whose blocks are all resident two a CU (more blocks than CUs, no more than twice as
  // many): the second half of the ids runs from the lightest query block up, so the two blocks a CU
  // holds -- ids i and i + 256 -- are a heavy one and a light one, and every CU has the same work.
  const int nqb = (int)(gridDim.x / heads), at = (int)(blockIdx.x / heads);
  const bool folded = causal && gridDim.x > kCUs && gridDim.x <= 2 * kCUs && SPLIT == 2 && W == 4 && D == 64;
  const int qb = folded && at >= (nqb + 1) / 2 ? at - (nqb + 1) / 2 : nqb - 1 - at;
  const int q0 = qb * BQW;

  const int q_tokens = valid ? bound_or(valid, seq) : seq_len;
  const int kv_tokens = kv_valid ? bound_or(kv_valid, kv_len) : (kv_len - seq + q_tokens);
  const bool masked_any = causal || window >= 0;
  const int offset = masked_any ? (kv_tokens - q_tokens) : 0;

  const int my_q = q0 + wave * 32 + col;            // this lane's query row
  const bool q_live = my_q < q_tokens;
  const int qpos = offset + my_q;
  const int wq_lo = offset + q0 + wave * 32;        // positions of the wave's first and last live query
  const int wq_hi = offset + min(q0 + wave * 32 + 31, q_tokens - 1);

  bf16_t* Oh = O + (size_t)head * q_head_stride;
  // Rows of this block past the bound: zeros.  A block wholly past it does only that.
  if (q0 >= q_tokens || offset < 0) {
    for (int i = tid; i < BQW * CPR; i += 64 * W * SPLIT) {
      const int r = q0 + i / CPR, c = (i % CPR) * 8;
      if (r < seq) *reinterpret_cast<uint4*>(Oh + (size_t)r * q_row_stride + c) = make_uint4(0, 0, 0, 0);
    }
    return;
  }

  // Q^T fragments (B operand): lane holds query `col`, d = 16*s + 8*g .. +7.
  bf16x8 qf[KS];
  {
    const bf16_t* qp = Q + (size_t)head * q_head_stride + (size_t)my_q * q_row_stride + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (q_live) v = *reinterpret_cast<const uint4*>(qp + 16 * s);
      qf[s] = __builtin_bit_cast(bf16x8, v);
    }
  }

  f32x16 oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[t][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;   // the reference maximum (of the raw, unscaled scores) and the sum against it
  float mc = 0.f;                         // the reference in the exp2 domain, 0 while it is -inf

  // Keys this block's live queries can see.
  const int q_last = min(q0 + BQW, q_tokens) - 1;
  int kv_hi = kv_tokens;
  if (causal) kv_hi = min(kv_hi, offset + q_last + 1);
  else if (window >= 0) kv_hi = min(kv_hi, offset + q_last + window + 1);
  int kv_lo = 0;
  if (window >= 0) kv_lo = max(0, offset + q0 - window) / BKV * BKV;
  const int ntiles = (kv_hi - kv_lo + BKV - 1) / BKV;
  // This half's tiles are half, half + SPLIT, ...; both halves make the same number of steps (a
  // block's waves share its barriers), the last of which may be past this half's last tile: it
  // then loads the last tile again and computes nothing.
  const int steps = (ntiles + SPLIT - 1) / SPLIT;

  if (ntiles > 0) {
    // The keys may be a window of a longer buffer, rows *kv_first on (held inside the buffer).
    const long first_row = kv_first ? max(0, min(*kv_first, kv_rows - kv_len)) : 0;
    const bf16_t* Kh = K + (size_t)kvh * kv_head_stride + first_row * kv_row_stride;
    const bf16_t* Vh = V + (size_t)kvh * kv_head_stride + first_row * kv_row_stride;

    // Loader: buffer loads straight into LDS.  Load i of a wave covers tile rows
    // (wave*INST + i)*RPI .. ; lane -> (row, physical chunk), and fetches the logical chunk that
    // the row's swizzle maps there.  The buffer is the tile's rows of this head up to the last key
    // (rebuilt per tile with scalar instructions): a lane's place in it is a constant 32-bit
    // offset, and rows past the last key -- only the last tile can hold any -- lie outside the
    // buffer and read as zeros, which the mask below turns into zero weights.
    const int l_row = lane / CPR, l_pch = lane % CPR;
    const int row_bytes = (int)kv_row_stride * 2;
    int k_voff[INST], v_voff[INST];
#pragma unroll
    for (int i = 0; i < INST; ++i) {
      const int r = (wave * INST + i) * RPI + l_row;
      k_voff[i] = r * row_bytes + (l_pch ^ ((r >> 1) & 7)) * 16;
      v_voff[i] = r * row_bytes + (l_pch ^ ((r & 3) << 1)) * 16;
    }
    // The keys (and values) of the head that this block can see, from row kv_lo's start to the
    // last key's row end, are one buffer for the whole loop; a tile's place in it goes into the
    // lanes' offsets, the part of the address the bounds check sees.
    const int reach = (kv_tokens - kv_lo - 1) * row_bytes + ROWB;
    const __amdgpu_buffer_rsrc_t k_rows = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(Kh + (long)kv_lo * kv_row_stride), 0, reach, 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rows = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(Vh + (long)kv_lo * kv_row_stride), 0, reach, 0x00020000);
    const int tile_bytes = BKV * row_bytes;
    auto issue = [&](int tile, int buf) {
      char* st = smem + buf * STAGE;
      const int at = tile * tile_bytes;
#pragma unroll
      for (int i = 0; i < INST; ++i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rows, IRON_LDS_PTR(st + (wave * INST + i) * 1024), 16,
                                                 (int)k_voff[i] + at, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rows, IRON_LDS_PTR(st + TILE + (wave * INST + i) * 1024), 16,
                                                 (int)v_voff[i] + at, 0, 0, 0);
      }
    };
    // Always STAGES-1 tiles in flight before the loop and one more each iteration (past the end
    // the last tile again, into a buffer nobody reads), so the wait counts below are exact.
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue(min(s * SPLIT + half, ntiles - 1), s);

    // Fragment addressing.  K (A operand of S^T): lane reads key t*32 + col, chunk 2s + g.
    const int k_frag = col * ROWB, k_swz = (col >> 1) & 7;
    // V^T (A operand of O^T): for (t, h) a lane group g needs keys 32t + 16h + 4g + 0..3 (low
    // half of its k slots) and the same + 8 (high half) of column d = 32 dt + col.  In the
    // transposing read a lane points at 4 consecutive d of the key row 4g + (lane & 15) / 4 ...
    const int v_key = 4 * g + ((lane & 15) >> 2);
    const int v_swz = ((lane >> 2) & 3) << 1;           // 2 * (key & 3), the same for every (t, h)
    int v_frag[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int chunk = dt * 4 + (((lane >> 4) & 1) << 1) + ((lane & 3) >> 1);
      v_frag[dt] = v_key * ROWB + ((chunk ^ v_swz) << 4) + ((lane & 1) << 3);
    }
    const unsigned lds_base = (unsigned)(size_t)IRON_LDS_PTR(smem);
    // The keys this lane's query may see are one range of positions for the whole loop: key kpos
    // is masked out iff (unsigned)(kpos - see_lo) > see_span (an empty range lets nothing pass).
    int see_hi = kv_tokens - 1, see_lo = 0;
    if (causal) see_hi = min(see_hi, qpos);
    else if (window >= 0) see_hi = min(see_hi, qpos + window);
    if (window >= 0) see_lo = max(0, qpos - window);
    const unsigned see_span = see_hi >= see_lo ? (unsigned)(see_hi - see_lo) : 0u;
    if (see_hi < see_lo) see_lo = 1 << 30;

    // A step of the loop on stage buffer `buf`.
    auto tile_step = [&](int step, const int buf) {
      const int ahead_buf = (buf + STAGES - 1) % STAGES;
      const int tile = step * SPLIT + half;
      const int kv0 = kv_lo + tile * BKV;
      wait_vmcnt<(STAGES - 2) * 2 * INST>();   // this wave's share of the tile has landed
      block_barrier();                          // everyone's has; everyone is done with the step before
      if constexpr (SPLIT > 1) {
        if (tile >= ntiles) {   // past this half's last tile: keep the loads (and the wait counts) going
          issue(ntiles - 1, ahead_buf);
          return;
        }
      }
      {
        const char* kt = smem + buf * STAGE;
        const unsigned vt = lds_base + buf * STAGE + TILE;
        // S^T = K Q^T for the two 32-key halves of the tile.
        f32x16 sacc[2];
        // A half's K fragments are all requested before its MFMAs (one wait, not one a fragment),
        // and the second half's while the first half's MFMAs run.
        bf16x8 kf[2][KS];
#pragma unroll
        for (int s = 0; s < KS; ++s)
          kf[0][s] = *reinterpret_cast<const bf16x8*>(kt + k_frag + (((2 * s + g) ^ k_swz) << 4));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS; ++s)
          kf[1][s] = *reinterpret_cast<const bf16x8*>(kt + 32 * ROWB + k_frag + (((2 * s + g) ^ k_swz) << 4));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
          for (int e = 0; e < 16; ++e) sacc[t][e] = 0.f;
#pragma unroll
          for (int s = 0; s < KS; ++s)
            sacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[t][s], qf[s], sacc[t], 0, 0, 0);
        }
        // The prefetch goes out while the score MFMAs run (its buffer, tile - 1's, is free since
        // the barrier above).
        issue(min(tile + (STAGES - 1) * SPLIT, ntiles - 1), ahead_buf);
        // Only tiles that touch a bound or the mask's edge pay for masking.  Element e of half t
        // is key kv0 + 32 t + 8 (e/4) + 4 g + e%4, query `col`.
        bool edge = kv0 + BKV > kv_tokens;
        if (causal) edge |= kv0 + BKV - 1 > wq_lo;
        else if (window >= 0) edge |= kv0 + BKV - 1 > wq_lo + window;
        if (window >= 0) edge |= kv0 < wq_hi - window;
        if (edge) {
          const int rel = kv0 + 4 * g - see_lo;
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e)
              sacc[t][e] = (unsigned)(rel + 32 * t + 8 * (e >> 2) + (e & 3)) > see_span ? -INFINITY : sacc[t][e];
        }
        // The reference the exponents are taken against follows the maxima lazily: it moves, and
        // the sums so far are rescaled, only when some query's maximum has left it more than
        // kLazyBits doublings behind (moving on every new maximum rescaled two tiles in three at
        // S = 8192: any of a wave's 32 queries decides).  And a tile is first tried WITHOUT its
        // maximum: the exponentials against the reference as it stands, and only if some query's
        // sum of them is out of a wide range (a score far above the reference, or all of them
        // so far below it that the sum vanishes) is the maximum taken and the tile redone -- the
        // arithmetic is floating point throughout, so any reference that neither overflows nor
        // underflows gives the same quotient.  Edge tiles and queries that have no reference yet
        // take the maximum at once.
        bool careful = edge || __builtin_amdgcn_ballot_w64(m_run == -INFINITY) != 0;
        bool moves = false;
        float alpha = 1.f, rsum;
        bf16x8 pf[2][2];
        for (;;) {
          if (careful) {
            float rmax = sacc[0][0];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
              for (int e = 0; e < 16; ++e) rmax = fmaxf(rmax, sacc[t][e]);
            rmax = max_with_other_half(rmax);
            moves = __builtin_amdgcn_ballot_w64((rmax - m_run) * scale_log2 > kLazyBits) != 0;   // -inf - -inf: no
            if (moves) {
              const float m_new = fmaxf(m_run, rmax);
              const float mc_new = (m_new == -INFINITY) ? 0.f : m_new * scale_log2;
              alpha = __builtin_amdgcn_exp2f(fmaf(m_run, scale_log2, -mc_new));  // exp2(-inf) = 0 at the start
              m_run = m_new;
              mc = mc_new;
            }
          }
          rsum = 0.f;
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              float p[8];
#pragma unroll
              for (int j = 0; j < 8; ++j) {
                p[j] = __builtin_amdgcn_exp2f(fmaf(sacc[t][8 * h + j], scale_log2, -mc));
                rsum += p[j];
              }
              pf[t][h] = __builtin_bit_cast(bf16x8, pack8(p));
            }
          if (careful) break;
          if (__builtin_amdgcn_ballot_w64(!(rsum >= kSumLow && rsum <= kSumHigh)) == 0) break;
          careful = true;
        }
        l_run = l_run * alpha + rsum;
        if (moves) {   // the output sums follow the reference (here, where the scores' registers are free again)
#pragma unroll
          for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[t][e] *= alpha;
        }

        // O^T += V^T P^T, a 32-key half at a time so one wait covers a batch of reads; the key
        // offsets ride in the reads' offset fields.
        auto pv_half = [&](auto half) {
          constexpr int t = decltype(half)::value;
          TrFrag vf[DT][2];
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const unsigned a = vt + v_frag[dt];
            vf[dt][0].lo = lds_read_tr16_at<(32 * t) * ROWB>(a);
            vf[dt][0].hi = lds_read_tr16_at<(32 * t + 8) * ROWB>(a);
            vf[dt][1].lo = lds_read_tr16_at<(32 * t + 16) * ROWB>(a);
            vf[dt][1].hi = lds_read_tr16_at<(32 * t + 24) * ROWB>(a);
          }
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            lds_tr_wait(vf[dt][0], vf[dt][1]);
#pragma unroll
            for (int h = 0; h < 2; ++h)
              oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_join(vf[dt][h]), pf[t][h], oacc[dt], 0, 0, 0);
          }
        };
        pv_half(std::integral_constant<int, 0>{});
        pv_half(std::integral_constant<int, 1>{});
      }
    };
    if constexpr (SPLIT > 1) {
      // Few, long blocks (a short sequence): the loop unrolled over the stage buffers, so that a
      // fragment's place in its stage is an immediate of the read and the buffer arithmetic goes
      // (S = 2048: 3.5 % faster).  Where a CU holds several blocks at different places of the loop
      // the three-fold code measured 2.4 % slower (S = 8192), so there the loop stays rolled.
      // An odd count of steps is rounded up: the added step is past every half's last tile and, like
      // the odd half's own last step may be, only keeps the loads and the wait counts going (a tail
      // of single steps would be two more copies of the body, whose registers spilled).
      static_assert(STAGES == 2, "the loop below names the buffers");
      for (int step = 0; step < steps; step += STAGES) {
        tile_step(step, 0);
        tile_step(step + 1, 1);
      }
    } else {
      for (int step = 0; step < steps; ++step) tile_step(step, step % STAGES);
    }
    wait_vmcnt<0>();   // the idle fetches of the last iterations land before the block's LDS is released
  }

  if constexpr (SPLIT == 2) {
    // The odd tiles' half hands its (max, sum, O) over through LDS, a value a lane a row (no bank
    // conflicts); the even tiles' half folds it in by the usual rule and stores.
    constexpr int FIELDS = 2 + 16 * DT;
    static_assert(W * FIELDS * 64 * 4 <= SPLIT * STAGES * STAGE, "the hand-over fits the stage buffers");
    float* hand = reinterpret_cast<float*>(smem_all) + wave * FIELDS * 64 + lane;
    block_barrier();   // every wave is out of the tile loop: the stage buffers are free
    if (half == 1) {
      hand[0] = m_run;
      hand[64] = l_run;
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) hand[(2 + 16 * t + e) * 64] = oacc[t][e];
    }
    __syncthreads();
    if (half == 1) return;
    const float m_other = hand[0], l_other = hand[64];
    const float m_new = fmaxf(m_run, m_other);
    const float mc = (m_new == -INFINITY) ? 0.f : m_new * scale_log2;
    const float a_mine = __builtin_amdgcn_exp2f(fmaf(m_run, scale_log2, -mc));      // exp2(-inf) = 0: a half
    const float a_other = __builtin_amdgcn_exp2f(fmaf(m_other, scale_log2, -mc));   // that saw no key
    l_run = l_run * a_mine + l_other * a_other;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) oacc[t][e] = oacc[t][e] * a_mine + hand[(2 + 16 * t + e) * 64] * a_other;
  }

  // Normalize and store: lane holds query `col`, columns 32 dt + 8 q + 4 g + 0..3.
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = (q_live && l_tot > 0.f) ? 1.0f / l_tot : 0.f;
  if (my_q < seq) {
    // (The row's address is made here: computed where its inputs first are, it is 64 bits a lane held
    // -- at eight waves a block, spilled -- through the whole loop.)
    int row = my_q;
    asm volatile("" : "+v"(row));
    bf16_t* op = Oh + (size_t)row * q_row_stride;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float v0 = oacc[dt][4 * q + 0] * inv, v1 = oacc[dt][4 * q + 1] * inv,
                    v2 = oacc[dt][4 * q + 2] * inv, v3 = oacc[dt][4 * q + 3] * inv;
        *reinterpret_cast<uint2*>(op + 32 * dt + 8 * q + 4 * g) =
            make_uint2(pack_bf16(v0, v1), pack_bf16(v2, v3));
      }
  }
}

// ---- 256- and 512-wide heads (Gemma's)
//
// A 64-key tile pair of 512-wide rows, or a wave's 32 queries of 512-wide output, fit neither the
// stages nor the registers of the kernel above (and at 256 it is down to one wave a SIMD).  Here a
// wave owns QN groups of 16 queries, each the columns of a 16-wide MFMA tile
// (v_mfma_f32_16x16x32_bf16), as the heads of a KV group are in decode attention: S^T = K Q^T over
// 32-key tiles (two 16-key MFMA tiles, the D columns in D / 32 k-steps, Q^T held in registers), a
// lane then owns one query column a group, its four lanes exchanging their maximum only when one
// passes the column's reference; the probabilities, rounded to bf16, are the B operand of
// O^T = V^T P^T as they stand, and O^T is D / 16 tiles of 16 output columns a group.  One group at
// 512 and two at 256 are the same 128 accumulator and 64 Q^T registers a lane; with two, every K and
// V^T fragment read out of LDS serves two MFMAs (the LDS reads are what bounds the kernel).  W waves
// (16 QN W queries of one head; two waves a SIMD, which holds a wave to 256 registers, all of them
// ordinary -- given 512 the compiler kept the accumulators in accumulation registers and copied all
// 128 around the conditional rescale on every tile) share the K and V tiles: 32 keys each, two
// stages, sent from global memory straight into LDS 1 KB an instruction; a row's 16-byte chunks are
// XORed by key & 15 in K (a fragment read is 16 keys at one chunk: all banks once) and by
// 2 (key & 3) in V (the transposing read).  Masks, bounds and the block order are the kernel's above.
template <int D, int QN, int W>
__global__ __launch_bounds__(64 * W, 2) void mha_prefill_wide_kernel(
    const bf16_t* __restrict__ Q, const bf16_t* __restrict__ K, const bf16_t* __restrict__ V,
    bf16_t* __restrict__ O, int heads, int group, int seq, int seq_len, int kv_len, float scale_log2,
    int causal, int window, long q_row_stride, long q_head_stride, long kv_row_stride,
    long kv_head_stride, const int* __restrict__ valid, const int* __restrict__ kv_valid,
    const int* __restrict__ kv_first, int kv_rows) {
  constexpr int ROWB = D * 2;            // bytes of a tile row
  constexpr int KS = D / 32;             // 32-wide k-steps of S^T
  constexpr int DT = D / 16;             // 16-row tiles of O^T
  constexpr int CPR = D / 8;             // 16-byte chunks a row has
  constexpr int TK = 32;                 // keys a tile
  constexpr int WQ = 16 * QN;            // queries of a wave
  constexpr int BQW = WQ * W;            // and of a block
  constexpr int TILE = TK * ROWB;
  constexpr int STAGE = 2 * TILE;
  constexpr int RPI = 1024 / ROWB;       // rows a 1 KB load covers
  constexpr int INST = TK / RPI / W;     // loads of K (and of V) a wave issues per tile
  static_assert(CPR * RPI == 64 && INST >= 1 && KS % 4 == 0 && DT % 4 == 0, "the tile splits into whole 1 KB loads a wave");
  extern __shared__ __align__(1024) char smem_wide[];   // 2 * STAGE bytes

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, q = lane >> 4;   // query column, quarter of the k slots
  const int j = blockIdx.x % heads;
  const int head = (heads % 8 == 0) ? (j % 8) * (heads / 8) + j / 8 : j;
  const int kvh = head / group;
  // (Two four-wave blocks a CU where the stages are 64 KB: a heavy and a light query block, as above.)
  const int nqb = (int)(gridDim.x / heads), at = (int)(blockIdx.x / heads);
  const bool folded = causal && D == 256 && W == 4 && gridDim.x > kCUs && gridDim.x <= 2 * kCUs;
  const int qb = folded && at >= (nqb + 1) / 2 ? at - (nqb + 1) / 2 : nqb - 1 - at;
  const int q0 = qb * BQW;

  const int q_tokens = valid ? bound_or(valid, seq) : seq_len;
  const int kv_tokens = kv_valid ? bound_or(kv_valid, kv_len) : (kv_len - seq + q_tokens);
  const bool masked_any = causal || window >= 0;
  const int offset = masked_any ? (kv_tokens - q_tokens) : 0;

  int my_q[QN], qpos[QN];
  bool q_live[QN];
#pragma unroll
  for (int u = 0; u < QN; ++u) {
    my_q[u] = q0 + wave * WQ + 16 * u + n;
    q_live[u] = my_q[u] < q_tokens;
    qpos[u] = offset + my_q[u];
  }
  const int wq_lo = offset + q0 + wave * WQ;
  const int wq_hi = offset + min(q0 + wave * WQ + WQ - 1, q_tokens - 1);

  bf16_t* Oh = O + (size_t)head * q_head_stride;
  if (q0 >= q_tokens || offset < 0) {   // rows of this block past the bound: zeros
    for (int i = tid; i < BQW * CPR; i += 64 * W) {
      const int r = q0 + i / CPR, c = (i % CPR) * 8;
      if (r < seq) *reinterpret_cast<uint4*>(Oh + (size_t)r * q_row_stride + c) = make_uint4(0, 0, 0, 0);
    }
    return;
  }

  // Q^T fragments (B operand): lane holds query n of its group, d = 32 s + 8 q .. + 7.
  bf16x8 qf[QN][KS];
#pragma unroll
  for (int u = 0; u < QN; ++u) {
    const bf16_t* qp = Q + (size_t)head * q_head_stride + (size_t)my_q[u] * q_row_stride + 8 * q;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (q_live[u]) v = *reinterpret_cast<const uint4*>(qp + 32 * s);
      qf[u][s] = __builtin_bit_cast(bf16x8, v);
    }
  }
  f32x4 oacc[QN][DT];
  float m_ref[QN], l_run[QN];   // a column's reference maximum (raw scores), this lane's sum
  const float lazy_raw = scale_log2 > 0.f ? kLazyBits / scale_log2 : INFINITY;   // kLazyBits doublings, in raw scores
#pragma unroll
  for (int u = 0; u < QN; ++u) {
    m_ref[u] = -INFINITY;
    l_run[u] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[u][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int q_last = min(q0 + BQW, q_tokens) - 1;
  int kv_hi = kv_tokens;
  if (causal) kv_hi = min(kv_hi, offset + q_last + 1);
  else if (window >= 0) kv_hi = min(kv_hi, offset + q_last + window + 1);
  int kv_lo = 0;
  if (window >= 0) kv_lo = max(0, offset + q0 - window) / TK * TK;
  const int ntiles = (kv_hi - kv_lo + TK - 1) / TK;

  if (ntiles > 0) {
    const long first_row = kv_first ? max(0, min(*kv_first, kv_rows - kv_len)) : 0;
    const bf16_t* Kh = K + (size_t)kvh * kv_head_stride + first_row * kv_row_stride;
    const bf16_t* Vh = V + (size_t)kvh * kv_head_stride + first_row * kv_row_stride;
    const int row_bytes = (int)kv_row_stride * 2;
    // Load i of a wave covers tile rows (wave INST + i) RPI + lane / CPR: a lane lands at physical
    // chunk lane % CPR of its row and fetches the logical chunk the row's swizzle maps there.  The
    // first row of a load is even where a load has two, so the row's low bit is the lane's own and
    // the rest of the swizzle is the load's (a scalar): two vector instructions a load, made where
    // they are used, against sixteen registers held through the loop.
    const int l_row = lane / CPR, l_ch = lane % CPR;
    const int k_lane = l_row * row_bytes + ((l_ch ^ l_row) << 4);
    const int v_lane = l_row * row_bytes + ((l_ch ^ (l_row << 1)) << 4);
    const int reach = (kv_tokens - kv_lo - 1) * row_bytes + ROWB;
    const __amdgpu_buffer_rsrc_t k_rows = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(Kh + (long)kv_lo * kv_row_stride), 0, reach, 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rows = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(Vh + (long)kv_lo * kv_row_stride), 0, reach, 0x00020000);
    const int tile_bytes = TK * row_bytes;
    auto issue = [&](int tile, int buf) {
      char* st = smem_wide + buf * STAGE;
      const int at = tile * tile_bytes;
#pragma unroll
      for (int i = 0; i < INST; ++i) {
        const int piece = wave * INST + i, r = piece * RPI, row_at = at + r * row_bytes;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rows, IRON_LDS_PTR(st + piece * 1024), 16,
                                                 (int)(k_lane ^ ((r & 15) << 4)) + row_at, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rows, IRON_LDS_PTR(st + TILE + piece * 1024), 16,
                                                 (int)(v_lane ^ ((r & 3) << 5)) + row_at, 0, 0, 0);
      }
    };
    issue(0, 0);

    // K fragment (tile t, k-step s): key 16 t + n, logical chunk 4 s + q, physical (4 s + q) ^ n: with
    // s = 4 a + b that is 16 a + (4 (b ^ (n >> 2)) | (q ^ (n & 3))) -- four bases a lane, the rest immediates.
    int k_frag[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) k_frag[b] = n * ROWB + (((4 * (b ^ (n >> 2))) | (q ^ (n & 3))) << 4);
    // V^T fragment (output tile dt): the lanes of quarter q point at key rows 4 q + 0..3 (k slots
    // 8 q + 0..3; the same 16 rows on for slots 8 q + 4..7, as S^T's second tile lies in P), 4 of the
    // tile's 16 columns each; chunk 2 dt + (lane & 3) / 2, swizzled.  dt = 4 k + r: four bases, 128 k on.
    const int v_swz = ((lane >> 2) & 3) << 1;
    const unsigned lds_base = (unsigned)(size_t)IRON_LDS_PTR(smem_wide);
    unsigned v_frag[4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
      v_frag[r] = lds_base + TILE + (4 * q + ((lane & 15) >> 2)) * ROWB +
                  (((2 * r + ((lane & 3) >> 1)) ^ v_swz) << 4) + ((lane & 1) << 3);

    // The keys a lane's query may see: one range of positions for the whole loop.
    int see_lo[QN];
    unsigned see_span[QN];
#pragma unroll
    for (int u = 0; u < QN; ++u) {
      int see_hi = kv_tokens - 1;
      see_lo[u] = 0;
      if (causal) see_hi = min(see_hi, qpos[u]);
      else if (window >= 0) see_hi = min(see_hi, qpos[u] + window);
      if (window >= 0) see_lo[u] = max(0, qpos[u] - window);
      see_span[u] = see_hi >= see_lo[u] ? (unsigned)(see_hi - see_lo[u]) : 0u;
      if (see_hi < see_lo[u]) see_lo[u] = 1 << 30;
    }

    auto tile_step = [&](int tile, auto buf_c) {
      constexpr int buf = decltype(buf_c)::value;
      const int kv0 = kv_lo + tile * TK;
      wait_vmcnt<0>();    // this wave's share of the tile has landed
      block_barrier();    // everyone's has; everyone is done with the tile before
      issue(min(tile + 1, ntiles - 1), buf ^ 1);
      if (causal && kv0 > wq_hi) return;   // the tile lies past every query of this wave
      const char* kt = smem_wide + buf * STAGE;
      // S^T = K Q^T for the tile's two 16-key halves, every K fragment for all the wave's groups.
      f32x4 sacc[QN][2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int u = 0; u < QN; ++u) sacc[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int a = 0; a < KS / 4; ++a) {
          bf16x8 kf[4];
#pragma unroll
          for (int b = 0; b < 4; ++b)
            kf[b] = *reinterpret_cast<const bf16x8*>(kt + k_frag[b] + t * 16 * ROWB + a * 256);
#pragma unroll
          for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int u = 0; u < QN; ++u)
              sacc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[b], qf[u][4 * a + b], sacc[u][t], 0, 0, 0);
        }
      }
      // Element i of half t is key kv0 + 16 t + 4 q + i, query n of the group.
      bool edge = kv0 + TK > kv_tokens;
      if (causal) edge |= kv0 + TK - 1 > wq_lo;
      else if (window >= 0) edge |= kv0 + TK - 1 > wq_lo + window;
      if (window >= 0) edge |= kv0 < wq_hi - window;
      bf16x8 pf[QN];
#pragma unroll
      for (int u = 0; u < QN; ++u) {
        bool out[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            out[t][i] = edge && (unsigned)(kv0 + 16 * t + 4 * q + i - see_lo[u]) > see_span[u];
            if (out[t][i]) sacc[u][t][i] = -INFINITY;
          }
        float lm = sacc[u][0][0];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) lm = fmaxf(lm, sacc[u][t][i]);
        // The reference follows the maxima lazily: it moves (and the 16 DT sums a lane holds are
        // rescaled) only when some lane of the wave has left it more than kLazyBits doublings behind
        // or has none yet, so a probability is at most 2^kLazyBits -- nothing to float32 sums or to
        // bf16's exponent.  Moving on every new maximum rescaled on a third of the tiles and more (a
        // wave's 16 queries share the decision): 32 heads at S = 4096, d = 256: 375 -> 324 us.
        if (__builtin_amdgcn_ballot_w64(lm > m_ref[u] + lazy_raw) != 0) {
          float mx = fmaxf(lm, __shfl_xor(lm, 16, 64));
          mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
          const float m_new = fmaxf(m_ref[u], mx);
          // A column that had seen no key has zero sums to rescale; one that still has none keeps -inf.
          const float alpha = (m_ref[u] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_ref[u] - m_new) * scale_log2);
          l_run[u] *= alpha;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) oacc[u][dt][i] *= alpha;
          m_ref[u] = m_new;
        }
        const float mc = (m_ref[u] == -INFINITY) ? 0.f : m_ref[u] * scale_log2;
        float p[8];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float e = __builtin_amdgcn_exp2f(fmaf(sacc[u][t][i], scale_log2, -mc));
            if (out[t][i]) e = 0.f;   // also where the scale is 0 and -inf * 0 is no number
            p[4 * t + i] = e;
            l_run[u] += e;
          }
        pf[u] = __builtin_bit_cast(bf16x8, pack8(p));
      }
      // O^T += V^T P^T, four output tiles' fragments requested at a time, each for all the groups.
#pragma unroll
      for (int k = 0; k < DT / 4; ++k) {
        TrFrag vf[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const unsigned at = v_frag[r] + (buf * STAGE + 128 * k);
          vf[r].lo = lds_read_tr16_at<0>(at);
          vf[r].hi = lds_read_tr16_at<16 * ROWB>(at);
        }
        lds_tr_wait(vf[0], vf[1]);
        lds_tr_wait(vf[2], vf[3]);
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
          for (int u = 0; u < QN; ++u)
            oacc[u][4 * k + r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tr_join(vf[r]), pf[u], oacc[u][4 * k + r], 0, 0, 0);
      }
    };
    using buf0 = std::integral_constant<int, 0>;
    using buf1 = std::integral_constant<int, 1>;
    for (int tile = 0; tile < ntiles; tile += 2) {
      tile_step(tile, buf0{});
      if (tile + 1 < ntiles) tile_step(tile + 1, buf1{});
    }
    wait_vmcnt<0>();   // the idle fetch of the last iteration lands before the block's LDS is released
  }

  // The lane's sum over its own keys -> the column's; normalize and store: lane holds query n of the
  // group, columns 16 dt + 4 q + 0..3.
#pragma unroll
  for (int u = 0; u < QN; ++u) {
    float l_tot = l_run[u] + __shfl_xor(l_run[u], 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    const float inv = (q_live[u] && l_tot > 0.f) ? 1.0f / l_tot : 0.f;
    if (my_q[u] < seq) {
      int row = my_q[u];   // (the address made here, as in the kernel above)
      asm volatile("" : "+v"(row));
      bf16_t* op = Oh + (size_t)row * q_row_stride + 4 * q;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        *reinterpret_cast<uint2*>(op + 16 * dt) = make_uint2(pack_bf16(oacc[u][dt][0] * inv, oacc[u][dt][1] * inv),
                                                             pack_bf16(oacc[u][dt][2] * inv, oacc[u][dt][3] * inv));
    }
  }
}

struct PrefillArgs {
  const uint16_t *Q, *K, *V;
  uint16_t* O;
  int heads, group, seq, seq_len, kv_len;
  float scale_log2;
  int causal, window;
  long q_row, q_head, kv_row, kv_head;
  const int *valid, *kv_valid;
  const int* kv_first;
  int kv_rows;
};

// The stage buffers are dynamic LDS (more than the 64 KB a kernel may declare statically).
template <int D, int SPLIT, int W = 4>
static int launch_prefill(const PrefillArgs& a, int blocks, void* stream) {
  constexpr int STAGES = D == 64 && SPLIT == 1 ? 3 : 2;
  constexpr size_t lds = (size_t)SPLIT * STAGES * 2 * BKV * D * 2;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&mha_prefill_kernel<D, SPLIT, W>), lds); e != hipSuccess) {
    set_error("mha_prefill: %s", hipGetErrorString(e));
    return (int)e;
  }
  hipLaunchKernelGGL((mha_prefill_kernel<D, SPLIT, W>), dim3(blocks), dim3(64 * W * SPLIT), lds, (hipStream_t)stream, a.Q,
                     a.K, a.V, a.O, a.heads, a.group, a.seq, a.seq_len, a.kv_len, a.scale_log2, a.causal, a.window,
                     a.q_row, a.q_head, a.kv_row, a.kv_head, a.valid, a.kv_valid, a.kv_first, a.kv_rows);
  return 0;
}

template <int D, int QN, int W>
static int launch_prefill_wide(const PrefillArgs& a, void* stream) {
  constexpr size_t lds = (size_t)2 * 2 * 32 * D * 2;   // two stages of a 32-key K tile and V tile
  constexpr int block_queries = 16 * QN * W;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(&mha_prefill_wide_kernel<D, QN, W>), lds); e != hipSuccess) {
    set_error("mha_prefill: %s", hipGetErrorString(e));
    return (int)e;
  }
  hipLaunchKernelGGL((mha_prefill_wide_kernel<D, QN, W>), dim3(((a.seq + block_queries - 1) / block_queries) * a.heads),
                     dim3(64 * W), lds, (hipStream_t)stream, a.Q, a.K, a.V, a.O, a.heads, a.group, a.seq, a.seq_len, a.kv_len,
                     a.scale_log2, a.causal, a.window, a.q_row, a.q_head, a.kv_row, a.kv_head, a.valid, a.kv_valid,
                     a.kv_first, a.kv_rows);
  return 0;
}

}  // namespace iron

using namespace iron;

static int mha_prefill(const uint16_t* Q, const uint16_t* K, const uint16_t* V, uint16_t* O, int heads, int kv_heads,
                       int d, int seq, int seq_len, int kv_len, float scale, int causal, int window, int q_interleaved,
                       int kv_interleaved, const int* valid, const int* kv_valid, const int* kv_first, int kv_rows,
                       void* stream) {
  IRON_REQUIRE(Q && K && V && O, "mha_prefill: null operand");
  IRON_REQUIRE(kv_first == nullptr || (kv_interleaved && kv_rows >= kv_len),
               "mha_prefill: a window of the keys takes them row by row (kv_interleaved) out of kv_rows (%d) >= kv_len (%d)",
               kv_rows, kv_len);
  IRON_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
               "mha_prefill: heads (%d) must be a positive multiple of kv_heads (%d)", heads, kv_heads);
  IRON_REQUIRE(d == 64 || d == 128 || d == 256 || d == 512, "mha_prefill: d (%d) must be 64, 128, 256 or 512", d);
  IRON_REQUIRE(seq > 0 && seq_len > 0 && seq_len <= seq,
               "mha_prefill: seq_len (%d) must be in [1, seq (%d)]", seq_len, seq);
  IRON_REQUIRE(kv_len >= seq, "mha_prefill: kv_len (%d) must be at least seq (%d): the queries are its last rows",
               kv_len, seq);
  IRON_REQUIRE(scale >= 0.f && scale < INFINITY, "mha_prefill: scale must be finite and not negative");
  IRON_REQUIRE((((uintptr_t)Q | (uintptr_t)K | (uintptr_t)V | (uintptr_t)O) & 15) == 0,
               "mha_prefill: operands must be 16-byte aligned");
  const long q_row = q_interleaved ? (long)heads * d : d;
  const long q_head = q_interleaved ? d : (long)seq * d;
  const long kv_row = kv_interleaved ? (long)kv_heads * d : d;
  const long kv_head = kv_interleaved ? d : (long)kv_len * d;
  IRON_REQUIRE(kv_row <= (1L << 20), "mha_prefill: a key row spans %ld values, more than the 2^20 a tile's 32-bit offsets reach", kv_row);
  IRON_REQUIRE((long)kv_len * kv_row * 2 < (1L << 31),
               "mha_prefill: the keys of a head span %ld bytes, more than the 2^31 its loads' 32-bit offsets reach",
               (long)kv_len * kv_row * 2);
  const float scale_log2 = scale * 1.4426950408889634f;
  const int blocks = ((seq + BQ - 1) / BQ) * heads;
  // Few blocks (a short sequence): the longest block's chain of tiles bounds the launch, so its
  // tiles are split over two halves of eight waves.  Many blocks fill the chip better four waves each
  // (at d = 64, where two eight-wave blocks share a CU, only from S = 16384 at 32 heads on: S = 8192 365 -> 353-360 us).
  const bool split = blocks <= (d == 64 ? 4 * kSplitMaxBlocks : kSplitMaxBlocks);
  PrefillArgs a{Q, K, V, O, heads, heads / kv_heads, seq, seq_len, kv_len, scale_log2, causal, window,
                q_row, q_head, kv_row, kv_head, valid, kv_valid, kv_first, kv_rows};
  int rc;
  // Wide heads: 16-query groups on 16x16x32 tiles.  Blocks of 128 queries (eight waves) once those
  // fill the chip twice over, of 64 (four waves) below that; at 256, where two groups a wave fit the
  // registers, launches of a thousand blocks and more take two (half the LDS reads a flop: 32 heads at
  // S = 4096 382 against 424 us; at 2048 it is the other way round, 154 against 119).
  if (d == 512) rc = blocks >= kWideBigBlocks ? launch_prefill_wide<512, 1, 8>(a, stream) : launch_prefill_wide<512, 1, 4>(a, stream);
  else if (d == 256)
    rc = blocks >= 2 * kWideBigBlocks ? launch_prefill_wide<256, 2, 4>(a, stream)
         : blocks >= kWideBigBlocks   ? launch_prefill_wide<256, 1, 8>(a, stream)
                                      : launch_prefill_wide<256, 1, 4>(a, stream);
  // Fewer blocks of 128 queries than two a CU (a short prompt): blocks of 64, two waves a part.
  else if (d == 64 && blocks < kFewBlocks) rc = launch_prefill<64, 2, 2>(a, ((seq + 63) / 64) * heads, stream);
  else if (d == 64) rc = split ? launch_prefill<64, 2>(a, blocks, stream) : launch_prefill<64, 1>(a, blocks, stream);
  else if (split) rc = launch_prefill<128, 2>(a, blocks, stream);
  else rc = launch_prefill<128, 1>(a, blocks, stream);
  if (rc != 0) return rc;
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_mha_prefill_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                     uint16_t* O, int heads, int kv_heads, int d, int seq,
                                     int seq_len, int kv_len, float scale, int causal, int window,
                                     int q_interleaved, int kv_interleaved, const int* valid,
                                     const int* kv_valid, void* stream) {
  return mha_prefill(Q, K, V, O, heads, kv_heads, d, seq, seq_len, kv_len, scale, causal, window, q_interleaved,
                     kv_interleaved, valid, kv_valid, nullptr, 0, stream);
}

extern "C" int iron_mha_prefill_at_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                        uint16_t* O, int heads, int kv_heads, int d, int seq,
                                        int seq_len, int kv_len, float scale, int causal, int window,
                                        int q_interleaved, const int* valid, const int* kv_valid,
                                        const int* kv_first, int kv_rows, void* stream) {
  IRON_REQUIRE(kv_first != nullptr, "mha_prefill_at: null kv_first");
  return mha_prefill(Q, K, V, O, heads, kv_heads, d, seq, seq_len, kv_len, scale, causal, window, q_interleaved, 1,
                     valid, kv_valid, kv_first, kv_rows, stream);
}
