/* libiron_hip.so -- C ABI of the hand-written gfx950 (MI355X) kernels behind the
 * IRON operator hot path.
 *
 * Every entry point: plain pointers and sizes, all data pointers are DEVICE
 * pointers owned by the caller, bf16 is 16-bit storage (uint16_t), one HIP
 * stream is passed in (void* = hipStream_t, NULL = the default stream).  No
 * entry point allocates, frees or synchronizes, so each may be recorded into a
 * HIP graph.  Return value: 0 = launched, 1 = arguments refused (the text is
 * in iron_last_error()), any other value = the hipError_t the launch raised.
 *
 * "const int* valid"-style arguments are per-call bounds read on the device at
 * run time (the reference's per-call scratchpad words,
 * iron/common/image/packaging.py:20); NULL means the whole extent.
 *
 * Citations are into the reference tree (amd/IRON).
 */
#ifndef IRON_HIP_H
#define IRON_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Library version (major*10000 + minor*100 + patch). */
int iron_version(void);
/* Text of the last refusal on this thread ("" if none). */
const char* iron_last_error(void);

/* C = A @ B, f32 accumulation, one rounding to bf16.
 * A (M,K) row-major.  B (K,N) row-major, or (N,K) row-major if b_col_maj.
 * C (M,N) row-major, or (N,M) if c_col_maj.  K % 8 == 0.
 * valid: rows of A computed (others of C untouched); valid_k: K actually summed.
 * Replaces GEMM.build()/kernels.linalg.mm: iron/operators/gemm.py:143,397-410,696-702. */
int iron_gemm_bf16(const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K,
                   int b_col_maj, int c_col_maj, const int* valid, const int* valid_k,
                   void* stream);

/* y[b] = W[b / repeat] @ x[b] for b in [0, batches): W (batches/repeat, M, K), x (batches, K),
 * y (batches, M); f32 accumulation, one rounding.  K % 8 == 0.
 * valid: rows of W computed.
 * Replaces GEMV.build()/linalg.mv: iron/operators/gemv.py:79,267-275,408-417. */
int iron_gemv_bf16(const uint16_t* W, const uint16_t* x, uint16_t* y, int M, int K, int batches,
                   int repeat, const int* valid, void* stream);
/* The same with the launch shape forced (rows a wave takes, waves splitting K); 0 = heuristic. */
int iron_gemv_bf16_tuned(const uint16_t* W, const uint16_t* x, uint16_t* y, int M, int K,
                         int batches, int repeat, const int* valid, int rows_per_wave,
                         int k_split, void* stream);

/* C = bf16(residual_scale * bf16(A B^T) + R) for the rows under *valid (or M): a projection over many
 * rows with its residual (a scale of 1: the plain sum; another: AXPY's) in the product's epilogue.
 * A (M,K), B (N,K), R and C (M,N); K % 64 == 0, M, N >= 64.  C may be R.
 * Replaces GEMM followed by ElementwiseAdd / AXPY (iron/lm/blocks.py:386-391,723-733), rounding
 * where they round. */
int iron_gemm_residual_bf16(const uint16_t* A, const uint16_t* B, const uint16_t* R, uint16_t* C, int M,
                            int N, int K, float residual_scale, const int* valid, void* stream);

/* The same product and sum for few rows over a long K, and the RMSNorm of the rows it leaves:
 * C = bf16(residual_scale * bf16(A B^T) + R), Y = RMSNorm(C) * gain as iron_rmsnorm_bf16 computes it
 * (Y is bit for bit what that call makes of C), for the rows under *valid (or M), in two launches.
 * While the bound leaves 128 x 128 tiles for no more than half the chip (512 live rows of a 2048-row
 * prompt chunk at N = 2048), each tile's K is dealt over 4 or 2 blocks that leave float32 sums in
 * `workspace`, and the second launch adds a row's slices in slice order before it rounds: the sums
 * are the same whatever ran first, and differ from iron_gemm_residual_bf16's in the last bits of the
 * float32 sum only.  A (M,K), B (N,K), R and C (M,N), gain (N), Y (M,N); C may be R, Y neither.
 * iron_gemm_residual_norm_workspace_bytes(M, N, K): the workspace's size (any contents), 0 for a
 * shape this entry refuses (M < 128, N not a multiple of 128 up to 8192, K under 4096 or not a
 * multiple of 256).
 * Replaces GEMM (down_proj), ElementwiseAdd / AXPY and the next RMSNorm
 * (iron/lm/blocks.py:723-733, then :688 of the next layer or the final norm). */
int64_t iron_gemm_residual_norm_workspace_bytes(int M, int N, int K);
int iron_gemm_residual_norm_bf16(const uint16_t* A, const uint16_t* B, const uint16_t* R,
                                 const uint16_t* gain, uint16_t* C, uint16_t* Y, int M, int N, int K,
                                 float residual_scale, float eps, const int* valid, void* workspace,
                                 void* stream);

/* C = bf16(bf16(act(G)) * bf16(A B^T)) for the rows under *valid (or M): a gated feed-forward's second
 * projection with the activated gate in its epilogue; activation 1: SiLU, 2: GELU by its tanh form.
 * A (M,K), B (N,K), G and C (M,N); K % 64 == 0, M, N >= 64.  C may be G.
 * Replaces GEMM (up_proj), SiLU or GELU (of gate_proj's product G) and ElementwiseMul
 * (iron/lm/blocks.py:688,697-699), rounding where they round. */
int iron_gemm_gated_bf16(const uint16_t* A, const uint16_t* B, const uint16_t* G, uint16_t* C, int M,
                         int N, int K, int activation, const int* valid, void* stream);
/* Both first projections of a gated feed-forward and the gate in one launch:
 * G = bf16(A Bg^T), C = bf16(bf16(act(G)) * bf16(A Bu^T)) for the rows under *valid (or M) -- what
 * iron_gemm_bf16 (gate_proj) followed by iron_gemm_gated_bf16 (up_proj) compute, bit for bit; a block
 * reads back only the tile of G it wrote itself.  A (M,K); Bg, Bu (N,K); G, C (M,N), distinct.
 * Replaces GEMM, GEMM, SiLU or GELU, ElementwiseMul (iron/lm/blocks.py:688,697-699). */
int iron_gemm_gated_pair_bf16(const uint16_t* A, const uint16_t* Bg, const uint16_t* Bu, uint16_t* G,
                              uint16_t* C, int M, int N, int K, int activation, const int* valid,
                              void* stream);

/* One-row fusions of a decoder layer (no single counterpart in the reference: each replaces a run
 * of its steps, iron/lm/blocks.py:627-648,697-699,723-733, and rounds where those steps round).
 *   y = E(W @ N(x)):  N = RMSNorm(x, eps) * norm_w when norm_w is not NULL (else x itself);
 *   epilogue 0: y = bf16(W N(x));  1: y = bf16(residual_scale * bf16(W N(x)) + residual), one fused
 *   multiply-add (a scale of 1 is the plain sum; another is AXPY's, iron/lm/blocks.py:386-391);
 *   2: y = bf16(bf16(silu(bf16(W N(x)))) * bf16(W2 N(x)))   (gate, up -> SiLU -> Mul);
 *   3: the same with GELU by its tanh form for SiLU (Gemma's feed-forward);
 *   4: y = bf16(bf16(gelu_tanh(bf16(W N(x)))) * residual), 5: the same with SiLU: a projection, its
 *   activation and the product with a given row (`residual` holds it; Gemma 4's per-layer input gate,
 *   iron/lm/blocks.py:793-796; norm_w must be NULL).
 * W, W2 (M,K); x, norm_w (K); residual, y (M).  K % 8 == 0. */
int iron_gemv_fused_bf16(const uint16_t* W, const uint16_t* W2, const uint16_t* x,
                         const uint16_t* norm_w, float eps, const uint16_t* residual,
                         float residual_scale, uint16_t* y, int M, int K, int epilogue, void* stream);

/* Attention's first half for one token: n = RMSNorm(x) * norm_w; q = Wq n, k = Wk n, v = Wv n
 * (each rounded to bf16); q and k rotated by the RoPE row `angles` (d bf16, cos/sin interleaved,
 * two halves); q -> q_out (heads*d), k -> keys[*position], v -> values[*position], caches
 * (cache_rows, kv_heads, d).  With angle_row not NULL, `angles` is a whole RoPE table of angle_rows
 * rows and the row is angles[*angle_row] (held inside the table): the step's copy of its table row
 * (iron/lm/blocks.py:394-431) then needs no launch of its own.  Replaces RMSNorm, 3 GEMV, 2 RoPE and
 * 2 Copy steps (iron/lm/blocks.py:472-502,627-648). */
int iron_decode_qkv_bf16(const uint16_t* x, const uint16_t* norm_w, float eps, const uint16_t* Wq,
                         const uint16_t* Wk, const uint16_t* Wv, const uint16_t* angles,
                         uint16_t* q_out, uint16_t* keys, uint16_t* values, int hidden, int heads,
                         int kv_heads, int d, int cache_rows, const int* position, const int* angle_row,
                         int angle_rows, void* stream);
/* The same for a decoder's first layer, whose input is the token's row of the embedding table
 * (table_rows, hidden): the row is read at table[*token] (held inside the table), and also written to
 * x (hidden), which the layer's residual sum reads -- the step's embedding lookup
 * (iron/lm/blocks.py:349-383, iron/lm/causal.py:292-299) then needs no launch of its own. */
int iron_decode_qkv_embed_bf16(const uint16_t* table, const int* token, int table_rows, uint16_t* x,
                               const uint16_t* norm_w, float eps, const uint16_t* Wq, const uint16_t* Wk,
                               const uint16_t* Wv, const uint16_t* angles, uint16_t* q_out, uint16_t* keys,
                               uint16_t* values, int hidden, int heads, int kv_heads, int d, int cache_rows,
                               const int* position, const int* angle_row, int angle_rows, void* stream);

/* Between a token's q/k/v projections and its attention where the heads are normed one by one
 * (Gemma's): RMSNorm of each q head (bit 0 of norms; gain q_gain or none), k head (bit 1; k_gain) and v
 * head (bit 2; no gain), RoPE on q and k by the call's angle rows (q_angles, k_angles: `rotary`
 * columns, cos/sin interleaved; the columns of a head past them pass through; NULL: not rotated), q ->
 * q_out (heads, d), k -> keys[*row0] and v -> values[*row0], caches (cache_rows, kv_heads, d), and
 * again at [*row1] where row1 is not NULL (a ring cache's mirror row).  k, v NULL: the layer reads
 * another layer's cache and only q is done.  Each step computed as its own kernel computes it.
 * Replaces up to 3 RMSNorm, 2 RoPE and 4 Copy steps (iron/lm/blocks.py:563-660,434-529). */
int iron_decode_heads_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, const uint16_t* q_gain,
                           const uint16_t* k_gain, int norms, float eps, const uint16_t* q_angles,
                           const uint16_t* k_angles, int rotary, int two_halves, uint16_t* q_out,
                           uint16_t* keys, uint16_t* values, const int* row0, const int* row1,
                           int cache_rows, int heads, int kv_heads, int d, void* stream);

/* A prompt chunk's three projections and the rotation of q and k in one launch (no single
 * counterpart in the reference: replaces 3 GEMM and 2 RoPE steps, iron/lm/blocks.py:617-648, and
 * rounds where those steps round): q = x Wq^T, k = x Wk^T, v = x Wv^T, each rounded to bf16; q and k
 * then turned by RoPE (two halves) with row r's angles `angles[r]` (rows, 64; cos and sin interleaved)
 * and rounded again.  x (rows, hidden); Wq (heads*d, hidden), Wk, Wv (kv_heads*d, hidden);
 * q_out (rows, heads*d), k_out, v_out (rows, kv_heads*d).  d == 64; heads, kv_heads even;
 * hidden % 64 == 0; rows >= 64.  valid: rows computed. */
int iron_prefill_qkv_bf16(const uint16_t* x, const uint16_t* Wq, const uint16_t* Wk,
                          const uint16_t* Wv, const uint16_t* angles, uint16_t* q_out,
                          uint16_t* k_out, uint16_t* v_out, int rows, int hidden, int heads,
                          int kv_heads, int d, const int* valid, void* stream);
/* The same with k and v written straight into the chunk's rows of the layer's KV caches, rows
 * *start on of keys and values (cache_rows, kv_heads*d): replaces the two Copy steps that follow as
 * well (iron/lm/blocks.py:472-486).  The first row is held where the rows under the bound end inside
 * the cache; rows <= cache_rows. */
int iron_prefill_qkv_cache_bf16(const uint16_t* x, const uint16_t* Wq, const uint16_t* Wk,
                                const uint16_t* Wv, const uint16_t* angles, uint16_t* q_out,
                                uint16_t* keys, uint16_t* values, int rows, int hidden, int heads,
                                int kv_heads, int d, int cache_rows, const int* start,
                                const int* valid, void* stream);

/* y = bf16(bf16(x * rsqrt(mean(x^2) + eps)) * w) per row; w NULL = unweighted (one rounding).
 * x,y (rows, cols); w (cols).  cols % 8 == 0.  valid: rows computed.
 * Replaces norm.rms_norm_eps + eltwise.mul_sized: iron/operators/rms_norm.py:10,
 * iron/common/elementwise.py:619-682. */
int iron_rmsnorm_bf16(const uint16_t* x, const uint16_t* w, uint16_t* y, int rows, int cols,
                      float eps, const int* valid, void* stream);
/* y = bf16(residual + the row above): a block's output normed again before its residual, the
 * sandwich layer's RMSNorm and ElementwiseAdd in one pass (iron/lm/blocks.py:748-767), rounding
 * where the two steps round.  residual (rows, cols); y may be residual. */
int iron_rmsnorm_add_bf16(const uint16_t* x, const uint16_t* w, const uint16_t* residual, uint16_t* y,
                          int rows, int cols, float eps, const int* valid, void* stream);

/* Rotary embedding of x (rows, cols) by the packed table angles (angle_rows, cols), cos and
 * sin interleaved; row r uses angle row r / (rows / angle_rows).  two_halves: rotate the two
 * halves of a row (else interleaved pairs).  cols % 16 == 0.  valid: rows computed.
 * Replaces datamovement.rope: iron/operators/rope.py:58,161-184. */
int iron_rope_bf16(const uint16_t* x, const uint16_t* angles, uint16_t* y, int rows, int cols,
                   int angle_rows, int two_halves, const int* valid, void* stream);

/* The same over the first rotary_cols columns of rows row_cols wide (angles (angle_rows, rotary_cols));
 * the columns past them are copied as they are.  (row_cols - rotary_cols) % 8 == 0.  A decoder whose
 * RoPE covers part of each head: one launch for the reference's copy out, rotation and copy back
 * (Attention.rotate, iron/lm/blocks.py:612-620). */
int iron_rope_partial_bf16(const uint16_t* x, const uint16_t* angles, uint16_t* y, int rows, int row_cols,
                           int rotary_cols, int angle_rows, int two_halves, const int* valid, void* stream);

/* Elementwise over n elements (valid: elements computed), f32 math, one rounding each:
 *   silu: y = x*sigmoid(x)   mul: y = a*b   add: y = a+b
 *   silu_mul: y = bf16(bf16(silu(g)) * u)  -- SiLU then ElementwiseMul, rounded between,
 * as two reference steps are.
 * Replaces activation.silu / eltwise.mul_sized / eltwise.add_sized:
 * iron/operators/silu.py:12, elementwise_mul.py:11, elementwise_add.py:11,
 * iron/common/elementwise.py:255-285. */
int iron_silu_bf16(const uint16_t* x, uint16_t* y, int64_t n, const int* valid, void* stream);
int iron_mul_bf16(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t n, const int* valid,
                  void* stream);
int iron_add_bf16(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t n, const int* valid,
                  void* stream);
int iron_silu_mul_bf16(const uint16_t* g, const uint16_t* u, uint16_t* y, int64_t n,
                       const int* valid, void* stream);

/* y[r] = bf16(x[r] + row) (or x[r] * row if multiply) for r < *valid (or rows): one row met by
 * every row, f32 math, one rounding.  x,y (rows, cols); row (cols).  cols % 8 == 0.
 * Replaces RowwiseAdd (a projection's bias) / RowwiseMul: iron/operators/elementwise_add.py:18,
 * elementwise_mul.py:18, iron/common/elementwise.py:797-867. */
int iron_row_broadcast_bf16(const uint16_t* x, const uint16_t* row, uint16_t* y, int rows, int cols,
                            int multiply, const int* valid, void* stream);

/* y[i] = bf16(f(x[i])) for i < *valid (or n), f32 math, one rounding; kind names f:
 * GELU by its tanh approximation or exact (x Phi(x)), ReLU, sigmoid, tanh, or the clamp to
 * [p0, p1] (p0, p1 are read by the clamp alone; the caller rounds them to bf16).
 * Replaces GELU / ReLU / Sigmoid / Tanh / Clamp: iron/operators/gelu.py:13, relu.py:11,
 * sigmoid.py:9, tanh.py:9, clamp.py:14 (each a UnaryElementwise, iron/common/elementwise.py:494). */
#define IRON_UNARY_GELU_TANH 0
#define IRON_UNARY_GELU_ERF 1
#define IRON_UNARY_RELU 2
#define IRON_UNARY_SIGMOID 3
#define IRON_UNARY_TANH 4
#define IRON_UNARY_CLAMP 5
int iron_unary_bf16(const uint16_t* x, uint16_t* y, int64_t n, int kind, float p0, float p1,
                    const int* valid, void* stream);

/* out[i] = bf16(a * x[i] + y[i]) for i < *valid (or n): one fused multiply-add in f32.
 * Replaces AXPY: iron/operators/axpy.py:13. */
int iron_axpy_bf16(const uint16_t* x, const uint16_t* y, uint16_t* out, int64_t n, float a,
                   const int* valid, void* stream);

/* y[r] = bf16((x[r] - mean) / sqrt(var + eps)) per row r < *valid (or rows), mean and the
 * variance about it in f32 (beta 0); with w, that row times w rounded again, as RMSNorm.
 * x,y (rows, cols); w (cols) or NULL.  cols % 8 == 0.
 * Replaces LayerNorm: iron/operators/layer_norm.py:10 over iron/common/elementwise.py:676-682. */
int iron_layernorm_bf16(const uint16_t* x, const uint16_t* w, uint16_t* y, int rows, int cols,
                        float eps, const int* valid, void* stream);

/* y[r, c] = softmax over the first *length (or cols) columns of row r, 0 in the columns past them:
 * z = x + addend (addend float32 or NULL), capped as soft_cap * tanh(z / soft_cap) when
 * soft_cap > 0, exp(z - max) / sum in f32, one rounding.  x (rows, cols) bf16, or float32 when
 * x_is_f32; y (rows, cols) bf16.  cols % 8 == 0.
 * Replaces Softmax without its band (window, period): iron/operators/softmax.py:62,523-545. */
int iron_softmax_bf16(const void* x, int x_is_f32, const float* addend, uint16_t* y, int rows,
                      int cols, float soft_cap, const int* length, void* stream);

/* Attention, many queries (prefill / prompt chunk).  Q,O: (seq, heads, d) if q_interleaved
 * else (heads, seq, d); K,V: (kv_len, kv_heads, d) if kv_interleaved else (kv_heads, kv_len, d).
 * The queries are the last rows of the keys: query i sits at position kv_tokens - q_tokens + i,
 * q_tokens = *valid (or seq_len), kv_tokens = *kv_valid (or kv_len - seq + q_tokens).
 * causal masks key > position; window >= 0 also masks key < position - window (and, when not
 * causal, key > position + window); window < 0 = none.  Rows >= q_tokens of O are zeros.
 * d in {64, 128, 256, 512} (MFMA tiles throughout: 32 queries a wave on 32x32x16 tiles at 64 and
 * 128, groups of 16 on 16x16x32 tiles at 256 and 512); heads % kv_heads == 0.
 * Replaces kernels.linalg.mha + partial_softmax + matmul_PV:
 * iron/operators/mha.py:191,574-667,1073-1116. */
int iron_mha_prefill_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V, uint16_t* O,
                          int heads, int kv_heads, int d, int seq, int seq_len, int kv_len,
                          float scale, int causal, int window, int q_interleaved,
                          int kv_interleaved, const int* valid, const int* kv_valid, void* stream);
/* The same over a window of a longer buffer of keys: K, V (kv_rows, kv_heads, d), of which the kv_len
 * rows from *kv_first on are the keys (the first row is held where they end inside the buffer).  What
 * a sliding-window layer's ring cache needs (iron/lm/blocks.py:504-529: the reference copies the
 * window into a staging tensor first; here attention reads it where it lies). */
int iron_mha_prefill_at_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V, uint16_t* O,
                             int heads, int kv_heads, int d, int seq, int seq_len, int kv_len,
                             float scale, int causal, int window, int q_interleaved, const int* valid,
                             const int* kv_valid, const int* kv_first, int kv_rows, void* stream);

/* Attention, one query (decode; the reference's "packed" MHA, seq_len == 1).
 * Q,O: (heads, d).  K,V as above.  kv_tokens = *kv_valid (or kv_len); the query sits at
 * kv_tokens - 1.  workspace: iron_mha_decode_workspace_bytes(heads, d) bytes of device memory.
 * Q, K, V, O and workspace 16-byte aligned.
 * d in {64, 128} with up to 16 query heads a KV head, d = 256 with 1, 2, 3, 4, 5, 6 or 8, or d = 512
 * with any.  The launches depend on (heads, kv_heads, d) and on whether kv_len can pass 2048 rows;
 * what they read, and how the keys are dealt over the chip, follow *kv_valid (a cache's length only
 * sizes the buffers: the reference's "attention over a cache costs the context, not the cache",
 * iron/operators/mha.py:275-278).
 * Replaces the packed single-query MHA: iron/operators/mha.py:476-477,1073-1116. */
int iron_mha_decode_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V, uint16_t* O,
                         int heads, int kv_heads, int d, int kv_len, float scale, int window,
                         int kv_interleaved, const int* kv_valid, void* workspace, void* stream);
int64_t iron_mha_decode_workspace_bytes(int heads, int d);
/* The same with the kernel form forced, for tests and measurements (as iron_gemv_bf16_tuned):
 * form 0 the default choice, 1 the lane-per-column scans, 2 the matrix-core scan (d = 64 or 128);
 * short_keys > 0: the live-key count up to which the matrix-core scan's one block a KV head writes
 * the output itself (beyond it the keys are dealt over every CU and a second launch merges). */
int iron_mha_decode_tuned_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V, uint16_t* O,
                               int heads, int kv_heads, int d, int kv_len, float scale, int window,
                               int kv_interleaved, const int* kv_valid, void* workspace, int form,
                               int short_keys, void* stream);
/* iron_mha_decode_bf16 for callers that cannot allocate (code under HIP-graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the same kernels, their split-KV partial results
 * in a scratch array the library holds in device memory itself (iron_mha_decode_static_max_bytes()
 * bytes on each GPU it runs on, until the process ends), so no workspace is passed and nothing is
 * allocated or freed.  Refused (1) when iron_mha_decode_workspace_bytes(heads, d) exceeds that size.
 * Every call on a GPU shares that GPU's array: calls that overlap on one GPU race.  Nothing in it
 * has to start at zero.  The first call on a device asks the runtime for the array's address there
 * (hipGetSymbolAddress, which may load the code object): make one call per device outside any stream
 * capture before recording calls into a graph.  No counterpart in the reference. */
int iron_mha_decode_static_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V, uint16_t* O,
                                int heads, int kv_heads, int d, int kv_len, float scale, int window,
                                int kv_interleaved, const int* kv_valid, void* stream);
int64_t iron_mha_decode_static_max_bytes(void);
/* One query over a window of a longer buffer of keys, as iron_mha_prefill_at_bf16. */
int iron_mha_decode_at_bf16(const uint16_t* Q, const uint16_t* K, const uint16_t* V, uint16_t* O,
                            int heads, int kv_heads, int d, int kv_len, float scale, int window,
                            const int* kv_valid, const int* kv_first, int kv_rows, void* workspace,
                            void* stream);

/* out[i] = table[ids[i]] for i < *valid (or n_ids); rows of row_bytes bytes (multiple of 4).
 * ids outside [0, table_rows) are skipped (the row is left untouched).
 * Replaces Copy's gather (embedding lookup): iron/operators/copy.py:72,546,839-902. */
int iron_gather_rows(const void* table, const int* ids, void* out, int n_ids, int table_rows,
                     int64_t row_bytes, const int* valid, void* stream);

/* dst[(*dst_row + i)] = src[(*src_row + i)] for i < *valid (or rows); NULL row index = 0.
 * Rows are row_bytes bytes (multiple of 4) at src_stride/dst_stride bytes apart; rows that
 * would land outside [0, src_rows) / [0, dst_rows) are skipped.
 * Replaces Copy between views with per-call offsets (KV-cache write, RoPE-table row,
 * last-row pick): iron/operators/copy.py:546,839-902. */
int iron_copy_rows(const void* src, void* dst, int rows, int64_t row_bytes, int64_t src_stride,
                   int64_t dst_stride, int src_rows, int dst_rows, const int* src_row,
                   const int* dst_row, const int* valid, void* stream);

/* Greedy draw: *token = index of the first largest logit among logits[0..n); when record is
 * not NULL also record[*at] = token (at NULL = 0; skipped if outside [0, record_len)), and when
 * token_copy is not NULL *token_copy = token (the carried `token` word of a decode loop: the draw
 * feeds the next step without a copy kernel between).
 * Replaces Sample with an all-zero draw row: iron/operators/sample.py:72-79,106,324-333. */
int iron_argmax_bf16(const uint16_t* logits, int n, int* token, int* record, int record_len,
                     const int* at, int* token_copy, void* stream);

/* The draw of one draw row: draws[*row .. *row+4) = {temperature as float32 bits, top-k, the low
 * and the high word of a 53-bit number} (row NULL = 0; draws NULL, a row outside
 * [0, draws_words) or a temperature that is not positive = the greedy draw above).  With a
 * temperature the candidates are the min(top-k, k_max) largest of logits[0..n), equals to the
 * lower index; candidate i weighs exp((l_i - l_0) / temperature) in float64 and the token is the
 * first whose running weight exceeds number * 2^-53 * total.  token, record, at, token_copy as
 * iron_argmax_bf16.  1 <= k_max <= 64; n <= 524288.  workspace: iron_sample_workspace_bytes(n)
 * bytes, 8-byte aligned (NULL allowed for n <= 2048); its first 16 bytes count the launch's blocks:
 * zero before the workspace's first launch, left zero by every launch; the rest may hold anything.
 * One launch; launches that share a workspace must not overlap.
 * Replaces Sample: iron/operators/sample.py:72-79,106-336 (its sample_ref is out of the
 * reference's tree; the arithmetic above is this library's own, fixed so a host computes the
 * same token bit for bit). */
int64_t iron_sample_workspace_bytes(int n);
int iron_sample_bf16(const uint16_t* logits, int n, const int* draws, int draws_words,
                     const int* row, int k_max, void* workspace, int* token, int* record,
                     int record_len, const int* at, int* token_copy, void* stream);

/* iron_sample_bf16 that ends a decode step: after the token is written (to token, record and
 * token_copy), the same launch evaluates the n_exprs word expressions of iron_eval_words over
 * words[0..n_words) -- the carried position and every word derived from it -- so a replayed step needs
 * no launch of its own for them.  Replaces Sample followed by the carry's Emit
 * (iron/operators/sample.py:106, iron/common/graph/carried.py:189-276). */
int iron_sample_advance_bf16(const uint16_t* logits, int n, const int* draws, int draws_words,
                             const int* row, int k_max, void* workspace, int* token, int* record,
                             int record_len, const int* at, int* token_copy, int* words, int n_words,
                             const int* exprs, int n_exprs, void* stream);

/* Evaluate n per-call word expressions in order, on the device, in one thread:
 *   words[e.dst] = (clamp(((words[e.src] * e.mul + e.add) >> e.shift), e.lo, e.hi) & e.mask) + e.post
 * exprs is n records of 9 int32 {dst, src, mul, add, shift, lo, hi, mask, post} in device memory
 * (mask -1 keeps every bit; 2^k - 1 is the remainder a ring of 2^k rows indexes by, post the
 * rows its mirror lies further on).
 * The device-side carry/Emit of a decode loop (position += 1, kv_valid = position + 1):
 * iron/common/graph/carried.py:189-276, iron/operators/emit.py. */
int iron_eval_words(int* words, int n_words, const int* exprs, int n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* IRON_HIP_H */
