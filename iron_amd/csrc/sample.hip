// The token draw with a temperature: the top-k logits of a row, weighed in float64 and drawn
// from by a 53-bit number the host wrote ahead of time (the draw row).  One launch: every block
// selects the k best of its 2048 logits into a list in the workspace; the block that finishes
// last (a ticket) selects the k best of all lists, its first wave weighs them and one lane walks
// the running sum.  A selection of k from entries dealt over 256 threads:
//   1. each thread's best entry; the k-th best of those 256 is a floor no top-k entry is under;
//   2. every entry at or over the floor goes to a list in LDS (about k of them), which is ranked.
// Order everywhere: the larger logit first, of equals the lower index, NaN below every number.
#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {

constexpr int SAMPLE_THREADS = 256;
constexpr int SAMPLE_K_MAX = 64;        // candidates one wave weighs; entries of a block's list
constexpr int SAMPLE_SHARE = 2048;      // logits a block selects from: a 16-byte piece a thread
constexpr int SAMPLE_BLOCKS_MAX = 256;
constexpr int SAMPLE_LIST = SAMPLE_SHARE;

// Blocks done with their lists are counted in the first word of the caller's workspace (the lists
// start SAMPLE_TICKET_BYTES in): zero before the workspace's first launch, and the last block to come
// sets it back to zero, so launches that share no workspace share no counter.
constexpr int SAMPLE_TICKET_BYTES = 16;

// 16 raw bf16 bits -> a key whose unsigned order is the logits' order.
__device__ __forceinline__ uint32_t order_key(uint32_t b) {
  if ((b & 0x7fffu) > 0x7f80u) return 0u;   // NaN
  if (b == 0x8000u) b = 0u;                 // -0 ranks with +0
  return (b & 0x8000u) ? (~b & 0xffffu) : (b | 0x8000u);
}
__device__ __forceinline__ float key_value(uint32_t key) {
  const uint32_t raw = (key & 0x8000u) ? (key & 0x7fffu) : (~key & 0xffffu);
  return __uint_as_float(raw << 16);
}
// A logit as one number, never 0: the larger the better.
__device__ __forceinline__ uint64_t entry(uint32_t key, int index) {
  return ((uint64_t)key << 32) | (uint32_t)~(uint32_t)index;
}
__device__ __forceinline__ int entry_index(uint64_t e) { return (int)~(uint32_t)e; }

__device__ __forceinline__ uint64_t shfl_xor64(uint64_t v, int o) {
  const uint32_t lo = __shfl_xor((uint32_t)v, o, 64), hi = __shfl_xor((uint32_t)(v >> 32), o, 64);
  return ((uint64_t)hi << 32) | lo;
}

// The blocks' lists cross from one XCD's block to another's through device-scope atomic stores and
// loads (written through and read past the XCD's own L2), which costs less than a fence's
// write-back and invalidation of the whole L2 on either side of the ticket.
__device__ __forceinline__ void publish(uint64_t* where, uint64_t e) {
  __hip_atomic_store(where, e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t collect(const uint64_t* where) {
  return __hip_atomic_load(where, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct SampleShared {
  __align__(16) uint64_t best[SAMPLE_THREADS];   // each thread's best entry
  __align__(16) uint64_t list[SAMPLE_LIST];
  uint64_t cand[SAMPLE_K_MAX];
  uint64_t slots[SAMPLE_THREADS / 64];
  int listed;
  int last_block;
};

// The block's largest of `mine`, in every thread.
__device__ __forceinline__ uint64_t block_max(uint64_t mine, SampleShared& sh) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint64_t other = shfl_xor64(mine, o);
    mine = other > mine ? other : mine;
  }
  __syncthreads();   // the slots' last readers are done
  if ((threadIdx.x & 63) == 0) sh.slots[threadIdx.x >> 6] = mine;
  __syncthreads();
  uint64_t best = sh.slots[0];
#pragma unroll
  for (int w = 1; w < SAMPLE_THREADS / 64; ++w) best = sh.slots[w] > best ? sh.slots[w] : best;
  return best;
}

__device__ __forceinline__ int wave_count(bool yes) {
  return __builtin_popcountll(__builtin_amdgcn_ballot_w64(yes));
}

constexpr int RANK_PADDED = 128;   // list entries zeroed ahead, so short lists are ranked in whole batches

// The k best of the entries `each(f)` visits over the block's threads (each entry once, none 0,
// all different), into sh.cand[0..k) from the best; slots past the number of entries are 0.
template <typename Each>
__device__ __forceinline__ void select_best(int k, SampleShared& sh, Each&& each) {
  uint64_t mine = 0;
  each([&](uint64_t e) { mine = e > mine ? e : mine; });
  __syncthreads();   // whoever read best/list/cand before is done
  sh.best[threadIdx.x] = mine;
  if (threadIdx.x < SAMPLE_K_MAX) sh.cand[threadIdx.x] = 0;
  if (threadIdx.x < RANK_PADDED) sh.list[threadIdx.x] = 0;
  if (threadIdx.x == 0) sh.listed = 0;
  __syncthreads();
  // 1. The floor: the k-th best of the threads' bests (0 if fewer threads hold an entry), found
  // by every wave for itself, a bit at a time from the top: the largest v that k bests reach.
  uint64_t floor = 0;
  {
    const int lane = threadIdx.x & 63;
    const uint64_t b0 = sh.best[lane], b1 = sh.best[lane + 64], b2 = sh.best[lane + 128],
                   b3 = sh.best[lane + 192];
    // The key's 16 bits on the high words alone; then, while more than k bests still reach the
    // floor (equal keys), the index's bits -- from bit 18: an index is under 2^19, so bits 19..31
    // of its complement are set in every entry and are taken in one step.
    const uint32_t h0 = (uint32_t)(b0 >> 32), h1 = (uint32_t)(b1 >> 32), h2 = (uint32_t)(b2 >> 32),
                   h3 = (uint32_t)(b3 >> 32);
    uint32_t high = 0;
    int reach = SAMPLE_THREADS;
    for (int bit = 15; bit >= 0 && reach != k; --bit) {
      const uint32_t v = high | (1u << bit);
      const int r = wave_count(h0 >= v) + wave_count(h1 >= v) + wave_count(h2 >= v) + wave_count(h3 >= v);
      if (r >= k) {
        high = v;
        reach = r;
      }
    }
    floor = (uint64_t)high << 32;
    if (high != 0 && reach != k) {
      floor |= 0xfff80000u;
      for (int bit = 18; bit >= 0 && reach != k; --bit) {
        const uint64_t v = floor | (1ull << bit);
        const int r = wave_count(b0 >= v) + wave_count(b1 >= v) + wave_count(b2 >= v) + wave_count(b3 >= v);
        if (r >= k) {
          floor = v;
          reach = r;
        }
      }
    }
  }
  // 2. The entries at or over it, listed in any order, then ranked by counting the better ones.
  each([&](uint64_t e) {
    if (e >= floor) {
      const int slot = atomicAdd(&sh.listed, 1);
      if (slot < SAMPLE_LIST) sh.list[slot] = e;
    }
  });
  __syncthreads();
  const int m = sh.listed;
  if (m <= SAMPLE_LIST) {
    const int whole = (m <= RANK_PADDED - 8 ? m + 7 : m) & ~7;   // zeros past a short list rank nothing
    const ulonglong2* pairs = reinterpret_cast<const ulonglong2*>(sh.list);
    for (int i = threadIdx.x; i < m; i += SAMPLE_THREADS) {
      const uint64_t me = sh.list[i];
      int rank = 0, j = 0;
      for (; j < whole; j += 8) {
        const ulonglong2 v0 = pairs[j / 2], v1 = pairs[j / 2 + 1], v2 = pairs[j / 2 + 2], v3 = pairs[j / 2 + 3];
        rank += (v0.x > me) + (v0.y > me) + (v1.x > me) + (v1.y > me) + (v2.x > me) + (v2.y > me) +
                (v3.x > me) + (v3.y > me);
      }
      for (; j < m; ++j) rank += sh.list[j] > me;
      if (rank < k) sh.cand[rank] = me;
    }
  } else {
    // More than the list holds: the next best, k times.
    uint64_t under = ~0ull;
    for (int r = 0; r < k; ++r) {
      uint64_t best = 0;
      each([&](uint64_t e) { best = (e < under && e > best) ? e : best; });
      under = block_max(best, sh);
      if (under == 0) break;
      if (threadIdx.x == 0) sh.cand[r] = under;
    }
  }
  __syncthreads();
}

// exp(z), z <= 0, from IEEE double +, -, * alone and in this order, so the host computes the
// same bits: n = rint(z log2 e), r = z - n ln 2 in two steps, a degree-13 Taylor polynomial
// by Horner (no fused multiply-add), an exact scaling by 2^n.  Below -690 (and for NaN): 0.
__device__ double exp_det(double z) {
#pragma clang fp contract(off)
  if (!(z >= -690.0)) return 0.0;
  const double n = rint(z * 1.4426950408889634);
  const double r = (z - n * 6.93147180369123816490e-01) - n * 1.90821492927058770002e-10;
  const double c[14] = {1.0,
                        1.0,
                        1.0 / 2.0,
                        1.0 / 6.0,
                        1.0 / 24.0,
                        1.0 / 120.0,
                        1.0 / 720.0,
                        1.0 / 5040.0,
                        1.0 / 40320.0,
                        1.0 / 362880.0,
                        1.0 / 3628800.0,
                        1.0 / 39916800.0,
                        1.0 / 479001600.0,
                        1.0 / 6227020800.0};
  double p = c[13];
#pragma unroll
  for (int i = 12; i >= 0; --i) {
    p = p * r;
    p = p + c[i];
  }
  const long long scale = (long long)((int)n + 1023) << 52;   // 2^n, n in [-996, 0]
  return p * __longlong_as_double(scale);
}

// lists: gridDim.x lists of SAMPLE_K_MAX entries, from each block's best, 0 past its last.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const bf16_t* __restrict__ logits, int n, const int* __restrict__ draws, int draws_words,
    const int* __restrict__ row, int k_max, uint64_t* workspace, int* __restrict__ token,
    int* __restrict__ record, int record_len, const int* __restrict__ at,
    int* __restrict__ token_copy, int* words, int n_words, const int* __restrict__ exprs, int n_exprs) {
  __shared__ SampleShared sh;
  unsigned int* ticket = reinterpret_cast<unsigned int*>(workspace);
  uint64_t* lists = workspace + SAMPLE_TICKET_BYTES / 8;

  // The draw row: {temperature (float32 bits), top-k, the 53-bit number's low and high word}.
  // A row outside the buffer, like a temperature that is not positive, is the greedy draw.
  const int at_word = row ? *row : 0;
  uint32_t w0 = 0, w1 = 0, w2 = 0, w3 = 0;
  if (draws != nullptr && at_word >= 0 && at_word + 4 <= draws_words) {
    w0 = (uint32_t)draws[at_word];
    w1 = (uint32_t)draws[at_word + 1];
    w2 = (uint32_t)draws[at_word + 2];
    w3 = (uint32_t)draws[at_word + 3];
  }
  const float temperature = __uint_as_float(w0);
  int k = (int)w1 < 1 ? 1 : (int)w1;
  k = k > k_max ? k_max : k;
  k = k > n ? n : k;
  if (!(temperature > 0.f)) k = 1;   // zero, negative or NaN

  // This thread's piece of the block's share: up to 8 logits from `first`.
  const int first = blockIdx.x * SAMPLE_SHARE + threadIdx.x * 8;
  const int count = n - first < 0 ? 0 : (n - first > 8 ? 8 : n - first);
  uint32_t key[8];
  if (count == 8) {
    const uint4 v = *reinterpret_cast<const uint4*>(logits + first);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      key[2 * j] = order_key(w[j] & 0xffffu);
      key[2 * j + 1] = order_key(w[j] >> 16);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) key[j] = j < count ? order_key(logits[first + j]) : 0u;
  }
  auto own = [&](auto&& f) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < count) f(entry(key[j], first + j));
  };

  const int blocks = gridDim.x;
  if (k == 1) {
    // Greedy, or a top-1 draw: the best entry of the block, then of the blocks.
    uint64_t best = 0;
    own([&](uint64_t e) { best = e > best ? e : best; });
    best = block_max(best, sh);
    if (threadIdx.x == 0) sh.cand[0] = best;
    if (blocks > 1 && threadIdx.x == 0) publish(&lists[(size_t)blockIdx.x * SAMPLE_K_MAX], best);
  } else {
    select_best(k, sh, own);
    if (blocks > 1 && threadIdx.x < SAMPLE_K_MAX)
      publish(&lists[(size_t)blockIdx.x * SAMPLE_K_MAX + threadIdx.x], sh.cand[threadIdx.x]);
  }
  if (blocks > 1) {
    // The lists are out: each thread's agent-scope stores have been acknowledged from past the
    // XCD's L2 (the wait below counts them down) before the block's barrier, and the barrier comes
    // before the ticket, so a block that sees the last ticket finds every list where its own
    // agent-scope loads read: in device memory.  The ticket is relaxed on purpose: a release/acquire
    // pair at agent scope would write back and invalidate the whole L2 on either side (the logits
    // the head just wrote are dirty lines in it), which costs more than this kernel's other work.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0)
      sh.last_block = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                      (unsigned)blocks - 1;
    __syncthreads();
    if (!sh.last_block) return;
    if (k == 1) {
      uint64_t best = 0;
      for (int b = threadIdx.x; b < blocks; b += SAMPLE_THREADS) {
        const uint64_t e = collect(&lists[(size_t)b * SAMPLE_K_MAX]);
        best = e > best ? e : best;
      }
      best = block_max(best, sh);
      if (threadIdx.x == 0) sh.cand[0] = best;
    } else {
      // The lists' first k entries, a list every `stride` slots (odd, so the lists' heads fall to
      // different threads); thread t owns slots t + 256 i.  The first HOLD of them are read once,
      // all requested together, and kept in registers; the rest (longer rows) are read every pass.
      constexpr int HOLD = 20;
      const int stride = k | 1, slots = blocks * stride;
      uint64_t held[HOLD];
#pragma unroll
      for (int i = 0; i < HOLD; ++i) {
        const int slot = threadIdx.x + SAMPLE_THREADS * i;
        const int b = slot / stride, r = slot - b * stride;
        held[i] = (slot < slots && r < k) ? collect(&lists[(size_t)b * SAMPLE_K_MAX + r]) : 0;
      }
      select_best(k, sh, [&](auto&& f) {
#pragma unroll
        for (int i = 0; i < HOLD; ++i)
          if (held[i] != 0) f(held[i]);
        for (int slot = threadIdx.x + SAMPLE_THREADS * HOLD; slot < slots; slot += SAMPLE_THREADS) {
          const int b = slot / stride, r = slot - b * stride;
          const uint64_t e = r < k ? collect(&lists[(size_t)b * SAMPLE_K_MAX + r]) : 0;
          if (e != 0) f(e);
        }
      });
    }
    if (threadIdx.x == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();

  // The first wave: a candidate's weight a lane; every lane sums and walks them in order.
  if (threadIdx.x >= 64) return;
  // The step's own tail, where the caller asks for it (the word expressions of iron_eval_words: the
  // carried position, then every word derived from it and from the token drawn here).  Its operands
  // are requested now, a word and an expression a lane, so that their trips to memory pass under the
  // draw: evaluated one after the other from memory they would cost a trip each.
  const bool tail = n_exprs > 0, tail_in_lds = tail && n_words <= 64 && n_exprs <= 64;
  int my_word = 0, rec[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
  if (tail_in_lds) {
    if ((int)threadIdx.x < n_words) my_word = words[threadIdx.x];
    if ((int)threadIdx.x < n_exprs) {
#pragma unroll
      for (int f = 0; f < 9; ++f) rec[f] = exprs[9 * threadIdx.x + f];
    }
  }
  int tok = entry_index(sh.cand[0]);
  const float top = key_value((uint32_t)(sh.cand[0] >> 32));
  if (k > 1 && top - top == 0.f) {   // a finite best logit; else it draws itself
    double w = 0.0;
    const uint64_t mine = sh.cand[threadIdx.x];
    const uint32_t key_i = (uint32_t)(mine >> 32);
    if ((int)threadIdx.x < k && key_i != 0u)
      w = exp_det(((double)key_value(key_i) - (double)top) / (double)temperature);
    const int w_lo = (int)(uint32_t)__double_as_longlong(w), w_hi = (int)(__double_as_longlong(w) >> 32);
    auto weight = [&](int i) {
      const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane(w_lo, i), hi = (uint32_t)__builtin_amdgcn_readlane(w_hi, i);
      return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
    };
    double total = 0.0;
    for (int i = 0; i < k; ++i) total += weight(i);
    const double u = (double)(((uint64_t)(w3 & 0x1fffffu) << 32) | w2) * 0x1p-53;
    const double threshold = u * total;
    double running = 0.0;
    int last = 0, drawn = -1;
    for (int i = 0; i < k && drawn < 0; ++i) {
      const double wi = weight(i);
      running += wi;
      if (running > threshold) drawn = i;
      else if (wi > 0.0) last = i;
    }
    const int pick = drawn < 0 ? last : drawn;
    tok = entry_index(((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)(mine >> 32), pick) << 32) |
                      (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)mine, pick));
  }
  if (threadIdx.x == 0) {
    *token = tok;
    if (token_copy != nullptr) *token_copy = tok;
    if (record != nullptr) {
      const int where = at ? *at : 0;
      if (where >= 0 && where < record_len) record[where] = tok;
    }
    if (tail && !tail_in_lds) {   // more words or expressions than a wave holds: one by one, from memory
      for (int e = 0; e < n_exprs; ++e) {
        const int* x = exprs + 9 * e;
        const int dst = x[0], src = x[1];
        if (dst < 0 || dst >= n_words || src < 0 || src >= n_words) continue;
        long v = ((long)words[src] * x[2] + x[3]) >> x[4];
        v = v < x[5] ? x[5] : (v > x[6] ? x[6] : v);
        words[dst] = ((int)v & x[7]) + x[8];
      }
    }
  }
  if (tail_in_lds) {
    // The words in LDS (the wave is alone by now), the token where the caller carries it, the
    // expressions in order -- each from the lane that holds it -- and the words back, a lane each.
    int* wl = reinterpret_cast<int*>(sh.best);
    wl[threadIdx.x] = my_word;
    const long slot = token_copy != nullptr ? (long)(token_copy - words) : -1;
    if (threadIdx.x == 0 && slot >= 0 && slot < n_words) wl[slot] = tok;
    for (int e = 0; e < n_exprs; ++e) {
      int x[9];
#pragma unroll
      for (int f = 0; f < 9; ++f) x[f] = __builtin_amdgcn_readlane(rec[f], e);
      if (threadIdx.x == 0 && x[0] >= 0 && x[0] < n_words && x[1] >= 0 && x[1] < n_words) {
        long v = ((long)wl[x[1]] * x[2] + x[3]) >> x[4];
        v = v < x[5] ? x[5] : (v > x[6] ? x[6] : v);
        wl[x[0]] = ((int)v & x[7]) + x[8];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if ((int)threadIdx.x < n_words) words[threadIdx.x] = wl[threadIdx.x];
  }
}

}  // namespace iron

using namespace iron;

static int sample_blocks(int n) { return (n + SAMPLE_SHARE - 1) / SAMPLE_SHARE; }

extern "C" int64_t iron_sample_workspace_bytes(int n) {
  return SAMPLE_TICKET_BYTES + (int64_t)sample_blocks(n) * SAMPLE_K_MAX * 8;
}

static int sample_launch(const uint16_t* logits, int n, const int* draws, int draws_words, const int* row, int k_max,
                         void* workspace, int* token, int* record, int record_len, const int* at, int* token_copy,
                         int* words, int n_words, const int* exprs, int n_exprs, void* stream) {
  IRON_REQUIRE(logits && token, "sample: null operand");
  IRON_REQUIRE(n > 0 && sample_blocks(n) <= SAMPLE_BLOCKS_MAX, "sample: n (%d) must be from 1 to %d", n,
               SAMPLE_BLOCKS_MAX * SAMPLE_SHARE);
  IRON_REQUIRE(k_max >= 1 && k_max <= SAMPLE_K_MAX, "sample: k_max (%d) must be from 1 to %d", k_max,
               SAMPLE_K_MAX);
  IRON_REQUIRE(draws == nullptr || draws_words >= 4, "sample: draws hold %d words, a row is 4", draws_words);
  IRON_REQUIRE(((uintptr_t)logits & 15) == 0, "sample: logits must be 16-byte aligned");
  IRON_REQUIRE(sample_blocks(n) == 1 || (workspace && ((uintptr_t)workspace & 7) == 0),
               "sample: %d logits take an 8-byte aligned workspace of iron_sample_workspace_bytes(n)", n);
  IRON_REQUIRE(n_exprs == 0 || (words && exprs && n_words > 0 && n_exprs > 0),
               "sample: %d word expressions take the words (%d of them) and the table", n_exprs, n_words);
  hipLaunchKernelGGL(sample_kernel, dim3(sample_blocks(n)), dim3(SAMPLE_THREADS), 0, (hipStream_t)stream,
                     logits, n, draws, draws_words, row, k_max, (uint64_t*)workspace, token, record,
                     record_len, at, token_copy, words, n_words, exprs, n_exprs);
  IRON_LAUNCH_CHECK();
}

extern "C" int iron_sample_bf16(const uint16_t* logits, int n, const int* draws, int draws_words,
                                const int* row, int k_max, void* workspace, int* token, int* record,
                                int record_len, const int* at, int* token_copy, void* stream) {
  return sample_launch(logits, n, draws, draws_words, row, k_max, workspace, token, record, record_len, at,
                       token_copy, nullptr, 0, nullptr, 0, stream);
}

extern "C" int iron_sample_advance_bf16(const uint16_t* logits, int n, const int* draws, int draws_words,
                                        const int* row, int k_max, void* workspace, int* token, int* record,
                                        int record_len, const int* at, int* token_copy, int* words, int n_words,
                                        const int* exprs, int n_exprs, void* stream) {
  return sample_launch(logits, n, draws, draws_words, row, k_max, workspace, token, record, record_len, at,
                       token_copy, words, n_words, exprs, n_exprs, stream);
}
