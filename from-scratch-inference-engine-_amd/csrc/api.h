// C interface of the kernel library (loaded from Python through ctypes).
//
// Conventions: every function returns 0 on success; otherwise fsie_last_error() describes the
// refusal (sizes a kernel does not take are refused here, never computed wrongly).  Pointers are
// device pointers unless said otherwise.  `dtype` is the type of activations and matrices:
// 0 = float32, 1 = bfloat16.  All work is queued on `stream`; nothing synchronises.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define FSIE_GEMM_SKINNY_MAX_M 8
#define FSIE_GEMM_MFMA_SKINNY_MAX_M 64
#define FSIE_GEMM_MFMA_WIDE_MAX_M 128  // the product that shares x through LDS, on a fragment-ordered weight: eight tiles of 16 rows
#define FSIE_GEMM_MFMA_SKINNY_BEST_M 16  // above this the library product is faster on MI355X
#define FSIE_GEMM_MAX_SPLITS 16          // most slices of K a product may leave as partial sums

// one attention work item = 8 int32
#define FSIE_ATTN_ITEM_INTS 8
#define FSIE_ATTN_ITEM_SEQ 0      // row of the block table
#define FSIE_ATTN_ITEM_QROW 1     // first query row (token index within the step)
#define FSIE_ATTN_ITEM_NQ 2       // query tokens in the tile (0 = padding item, skipped)
#define FSIE_ATTN_ITEM_POS 3      // absolute position of the first query token
#define FSIE_ATTN_ITEM_KBEGIN 4   // first key
#define FSIE_ATTN_ITEM_KEND 5     // one past the last key
#define FSIE_ATTN_ITEM_PARTIAL 6  // -1: write the output; >= 0: first partial slot of the tile
// The first tokens of a request that a window keeps: keys below KEEP are seen whatever the window says.  With
// FSIE_ATTN_KEEP_WALK set the item also reads the keys [0, min(KEEP, KBEGIN)), before those of its own range.
#define FSIE_ATTN_ITEM_KEEP 7
#define FSIE_ATTN_KEEP_WALK (1 << 30)
// with FSIE_ATTN_POOL_WALK set (kernels that take pooled blocks) the item also reads the mean keys and values of the
// blocks of positions that lie wholly before its queries' windows, from the pools of pooled blocks
#define FSIE_ATTN_POOL_WALK (1 << 29)
// one merge item = 4 int32: {output row, first partial slot, number of splits, slot stride}
#define FSIE_ATTN_MERGE_INTS 4

#ifdef __cplusplus
extern "C" {
#endif

const char* fsie_last_error(void);
int fsie_version(void);
// Name of the architecture the device code was built for and of the device present.
int fsie_device_info(char* arch_out, int arch_len, int* n_compute_units);
// Compute units of the current device; 0 if there is no device to ask.
int fsie_device_compute_units(void);

// out[t] = table[ids[t]] * scale, float32
int fsie_embedding(const void* table, int dtype, const int32_t* ids, float* out, int n_tokens, int hidden,
                   int vocab, float scale, hipStream_t stream);
int fsie_rmsnorm(float* residual, const void* delta, const float* weight, void* out, const int32_t* rows,
                 int n_rows, int hidden, float eps, int dtype, int write_back, int n_parts, int total_rows,
                 hipStream_t stream);
// RMSNorm of a plain tensor (no residual stream): every row holds `groups` runs of `width` values
// (strides in elements), each run normalised by itself; `out` may be `x`.
int fsie_rmsnorm_plain(const void* x, int64_t x_stride, const float* weight, void* out, int64_t out_stride, int n_rows,
                       int groups, int width, float eps, int dtype, hipStream_t stream);
// Rows slots[0..n) of a table of n_slots rows of row_bytes set to zero; a negative slot is skipped.
int fsie_zero_rows(void* table, const int32_t* slots, int n, int64_t row_bytes, int n_slots, hipStream_t stream);
// Pages pages[0..n) (negative: skipped) of two pools of [planes][n_pages][page_bytes] set to zero.
int fsie_zero_pages(void* pool_a, void* pool_b, const int32_t* pages, int n, int planes, int n_pages,
                    int64_t page_bytes, hipStream_t stream);
// Counter-based random values (the random-weights mode): see elementwise.hip.
int fsie_random_fill(void* out, int64_t n, uint64_t key, int kind, float std, hipStream_t stream);
int fsie_swiglu(const void* x, void* out, int n_tokens, int inter, int dtype, hipStream_t stream);
// the same with the gate's activation named: 0 = SiLU, 1 = GELU in its tanh form
int fsie_gated_act(const void* x, void* out, int n_tokens, int inter, int dtype, int act, hipStream_t stream);
// The norm of a sublayer's output, the residual sum and the next norm in one pass:
//   v = residual + rmsnorm(delta; post_weight, post_eps);  out = rmsnorm(v; weight, eps)
// delta as for fsie_rmsnorm (one array of the activations' type, or n_parts float32 partial sums).
int fsie_sandwich_norm(float* residual, const void* delta, const float* post_weight, float post_eps, const float* weight,
                       float eps, void* out, const int32_t* rows, int n_rows, int hidden, int dtype, int write_back,
                       int n_parts, int total_rows, hipStream_t stream);
// out[t][h][:] = rmsnorm(o[t][h][:]; weight, eps) * act(gate[t][h][:]), a head `width` values wide; o float32, the sum
// in order of n_planes arrays [n_tokens][heads * width] that lie one after the other
int fsie_gated_headnorm(const float* o, int n_planes, const void* gate, int64_t gate_stride, const float* weight, void* out,
                        int n_tokens, int heads, int width, float eps, int act, int dtype, int64_t out_stride, float out_scale,
                        hipStream_t stream);
// x <- cap * tanh(x / cap) in place
int fsie_softcap(float* x, int64_t n, float cap, hipStream_t stream);

// Gated linear attention over the tokens of a step, from and to the per-request state (linear_attention.hip).
int fsie_gla_scan_shape(int heads, int dim, int vdim, int* prep_floats_per_token, int* out_planes, int* chunk_tokens,
                        int* chunk_min, int64_t* chunk_floats);
int fsie_gla_scan(const void* proj, int64_t proj_stride, int q_off, int k_off, int v_off, const float* z, float* state,
                  const int32_t* q_starts, const int32_t* seq_slots, int n_seqs, int n_tokens, float* prep, float* out,
                  float* chunk_work, int max_chunks, int heads, int dim, int vdim, float q_scale, float inv_tau,
                  int n_slots, int dtype, const float* head_decay, const void* qk, int64_t qk_stride, const float* cos_sin,
                  int rot_pairs, hipStream_t stream);
// cos_sin [n_tokens][rot_pairs][2] (or null and 0): the first 2 * rot_pairs channels of every q and k head are turned,
// channel i with channel i + rot_pairs, by the token's cosines and sines as they are read (float32).
// qk (or null): q and k are read from rows of their own, qk_stride values apart, at the same column offsets.
// head_decay (or null): float32 [heads]; with it z may be null and every key channel of head h decays by head_decay[h],
// the same for every token (retention: a fixed decay a head).

// Attention through a latent (latent_attention.hip): the norms of the latents, the gates and the cache row of
// every token; the rotation of pairs of neighbours; a product with a matrix of its own for every head.
// rot_pairs > 0: the rotated pairs are neighbours (2i, 2i + 1); rot_pairs < 0: -rot_pairs pairs (i, i + pairs)
int fsie_latent_prep(const void* proj, int64_t stride, int dq_off, int q_rank, int dkv_off, int kv_rank, int rot_dim,
                     int rot_pairs, int g_off, int heads, const float* q_weight, const float* kv_weight, float eps,
                     const float* cos_sin, void* cq, float* gate, const int32_t* slots, void* k_pool, void* v_pool,
                     int width, int page_size, int64_t pool_slots, int n_tokens, int dtype, hipStream_t stream);
int fsie_rope_pairs(const void* in, int64_t in_stride, int in_off, int in_hs, void* out, int64_t out_stride, int out_off,
                    int out_hs, int heads, int width, int rot_pairs, int out_width, const float* cos_sin, int n_tokens,
                    int dtype, hipStream_t stream);
int fsie_head_gemm(const void* x, int64_t x_stride, int x_off, int x_hs, const void* w, void* y, int64_t y_stride, int y_off,
                   int y_hs, const float* gate, int n_tokens, int heads, int N, int K, int dtype, hipStream_t stream);
// y = x rounded to `dtype` (a copy for float32)
int fsie_round_to(const float* x, void* y, int64_t total, int dtype, hipStream_t stream);
// y = a * x1 + b * x2, elementwise, float32 arithmetic, all three of `dtype`
int fsie_scaled_sum(const void* x1, float a, const void* x2, float b, void* y, int64_t total, int dtype, hipStream_t stream);
int fsie_residual_add(float* residual, const void* delta, int64_t total, int dtype, hipStream_t stream);
int fsie_bias_add(void* y, const float* bias, int rows, int cols, int dtype, hipStream_t stream);
// y [rows][cols] bfloat16 = parts[0] + parts[1] + ... (float32 [planes][rows][cols], added in their order) + bias
// (float32 [cols] or null), rounded once; cols a multiple of 4
int fsie_sum_round(const float* parts, int planes, const float* bias, void* y, int rows, int cols, hipStream_t stream);

int fsie_rope_kv_write(void* qkv, const int32_t* positions, const int32_t* slots, const double* inv_freq,
                       const float* bias, void* k_pool, void* v_pool, int n_tokens, int n_heads, int n_kv, int head_dim,
                       int rotary_dim, int page_size, int64_t pool_slots, int dtype, hipStream_t stream);

// the same with the whole head rotated by the cosines and sines of fsie_rope_table (head_dim % 8 == 0);
// parts (or null): the projection as n_parts float32 partial sums [n_parts][n_tokens][width], added in
// order; qkv then only receives the q heads
int fsie_rope_kv_write_table(void* qkv, const float* cos_sin, const int32_t* slots, const float* bias, void* k_pool,
                             void* v_pool, int n_tokens, int n_heads, int n_kv, int head_dim, int page_size,
                             int64_t pool_slots, int dtype, const float* parts, int n_parts, hipStream_t stream);

// table [n_tokens, half, 2] float32: cos and sin of positions[t] * inv_freq[i]
int fsie_rope_table(const int32_t* positions, const double* inv_freq, int n_tokens, int half, float* table,
                    hipStream_t stream);

// the same with every cosine and sine multiplied by `magnitude` (rotations whose scaling of the frequencies
// comes with a factor on the rotated vectors)
int fsie_rope_table_scaled(const int32_t* positions, const double* inv_freq, int n_tokens, int half, float magnitude,
                           float* table, hipStream_t stream);

// Layer norm over the residual stream, fused with the residual sum of up to two pending deltas (parts: 0 = one
// array of the activations' type, n = n float32 partial sums), one or two outputs that differ in weight and bias.
int fsie_layer_norm(float* residual, const void* delta_a, int parts_a, const void* delta_b, int parts_b, const float* w1,
                    const float* b1, void* out1, const float* w2, const float* b2, void* out2, const int32_t* rows,
                    int n_rows, int hidden, float eps, int dtype, int write_back, int total_rows, hipStream_t stream);
// Token rows times `scale` plus the hashed row of (previous token, token); last[slot] keeps a request's latest
// token + 1 from step to step (0: none) and is brought up to date after the rows are written.
int fsie_pair_embedding(const void* table, const void* pairs, int dtype, const int32_t* ids, const int32_t* q_starts,
                        const int32_t* seq_slots, int n_seqs, int32_t* last, int n_slots, float* out, int n_tokens,
                        int hidden, int vocab, int buckets, int64_t mul_prev, int64_t mul_cur, float scale,
                        hipStream_t stream);
// Between the fused q|k|v|gate projection and attention: head norms, partial rotation from the step's table, the
// mixing of values with another layer's, the gates' sigmoid, queries and cache entries in heads of D values.
int fsie_attention_prep(const void* proj, int64_t stride, int q_off, int k_off, int v_off, int g_off, int heads,
                        int kv_heads, int dim, int vdim, int D, const float* q_weight, const float* k_weight, float eps,
                        int pairs, const float* cos_sin, const void* v_other, int64_t v_other_stride, const float* mix,
                        void* q_out, float* gate, const int32_t* slots, void* k_pool, void* v_pool, int page_size,
                        int64_t pool_slots, int n_tokens, int dtype, int q_weight_stride, int v_unit_norm, float v_eps,
                        hipStream_t stream);
int fsie_gate_heads(const void* x, int D, const float* gate, void* y, int n_tokens, int heads, int vdim, int dtype,
                    int64_t y_stride, float y_scale, hipStream_t stream);

int fsie_gemm(const void* x, const void* w, const float* bias, void* y, int M, int N, int K, int dtype,
              int out_f32, int kind, hipStream_t stream);

// True float32 on the matrix cores (v_mfma_f32_16x16x4_f32) for up to 64 rows: the 32-bit path's decoding.
int fsie_gemm_mfma_fp32(const float* x, const float* w, const float* bias, float* y, int M, int N, int K, int waves,
                        hipStream_t stream);

int fsie_gemm_mfma_skinny(const void* x, const void* w, const float* bias, void* y, int M, int N, int K,
                          int out_f32, int waves, int blocks, int epilogue, int splits, hipStream_t stream);

int fsie_gemm_mfma_skinny_rope(const void* x, const void* w, const float* bias, void* y, int M, int K,
                               const int32_t* positions, const int32_t* slots, const double* inv_freq,
                               const float* cos_sin, void* k_pool,
                               void* v_pool, int n_heads, int n_kv, int head_dim, int page_size, int64_t pool_slots,
                               hipStream_t stream);

// 17 to 64 rows (any number up to 64 is taken): X shared through LDS, float32 result or partial sums
int fsie_gemm_mfma_wide_slice(int K, int splits);
int fsie_gemm_mfma_wide_best_splits(int M, int N, int K);
// (frags: w is the copy of the matrix in the order of the A fragments, made by fsie_fragment_order)
int fsie_gemm_mfma_wide(const void* x, const void* w, float* y, int M, int N, int K, int splits, int waves,
                        int blocks, int frags, hipStream_t stream);
// the rows of w are gate and up in turn: y is bfloat16 [M, N / 2], silu(gate) * up
int fsie_gemm_mfma_wide_swiglu(const void* x, const void* w, void* y, int M, int N, int K, int waves, int blocks,
                               int frags, hipStream_t stream);
// the same with the gate's activation named (0 = SiLU, 1 = GELU in its tanh form)
int fsie_gemm_mfma_wide_gated(const void* x, const void* w, void* y, int M, int N, int K, int waves, int blocks,
                              int frags, int act, hipStream_t stream);
// A bfloat16 matrix [N, K] (K a multiple of 32) copied so that the 64 16-byte units of a block of 16
// rows and 32 values of K lie together in the order of the lanes that hold them: a wave's load of W
// is then one piece of 1 KB.  The copy has fsie_fragment_order_size values (N rounded up to 16 rows).
// whether they take M rows of this shape (65 to FSIE_GEMM_MFMA_WIDE_MAX_M rows: only some launch shapes on a
// fragment-ordered weight)
int fsie_gemm_mfma_wide_takes(int M, int N, int K, int splits, int gate_up, int frags);
int64_t fsie_fragment_order_size(int N, int K);
int fsie_fragment_order(const void* w, void* out, int N, int K, hipStream_t stream);

int fsie_attention_scalar(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                          const int32_t* block_tables, int max_pages, const int32_t* items, int n_items,
                          void* out, float* partials, int n_heads, int n_kv, int head_dim, int page_size,
                          int window, float scale, int dtype, const float* sinks, float softcap, const void* k_pooled,
                          const void* v_pooled, const int32_t* pooled_tables, int pooled_max_pages, int pooled_page_size,
                          int pooled_tokens, hipStream_t stream);
// k_pooled .. pooled_tokens (or null and zeros): pools [units][n_kv][pooled_page_size][head_dim] and
// [units][n_kv][head_dim][pooled_page_size] that hold one mean key and value for every block of pooled_tokens positions,
// with their block table [requests][pooled_max_pages]; an item flagged FSIE_ATTN_POOL_WALK reads, beside its own keys,
// the blocks that lie wholly before a query's window (fsie_pool_blocks fills them).
// softcap (in every attention entry point that takes it): a positive number caps the scaled scores,
// s <- softcap * tanh(s / softcap), before the mask and the softmax; 0: scores as they are.
// sinks (or null, in every attention entry point that takes it): float32 [n_heads]; exp(sinks[h]) is one more
// term of the softmax denominator of every query row of head h.  It has no key and no value and is not scaled.
// Items that leave partial records ignore it; the merge that combines them adds it once.
int fsie_attention_merge(const float* partials, const int32_t* merges, int n_merges, void* out, int n_heads,
                         int head_dim, int dtype, const float* sinks, hipStream_t stream);
int fsie_attention_scalar_tile_tokens(int n_heads, int n_kv);
// The mean key and value of blocks of `block_tokens` consecutive positions, from the pages of keys and values to the
// pools of pooled blocks: jobs [n_jobs][2] = (request of the step, block), a request of -1: nothing.  Block b's
// positions b * block_tokens .. are read through the request's row of block_tables and summed in float32 in a fixed order
// (runs of consecutive positions, each in its order, then the runs in theirs);
// the entry goes to the page that pooled_tables names for b.
int fsie_pool_blocks(const void* k_pool, const void* v_pool, const int32_t* block_tables, int max_pages, int page_size,
                     void* k_pooled, void* v_pooled, const int32_t* pooled_tables, int pooled_max_pages, int pooled_page_size,
                     const int32_t* jobs, int n_jobs, int block_tokens, int n_kv, int head_dim, int dtype, hipStream_t stream);

int fsie_attention_mfma(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                        const int32_t* block_tables, int max_pages, const int32_t* items, int n_items, void* out,
                        float* partials, int n_heads, int n_kv, int head_dim, int page_size, int window, float scale,
                        int large, int waves, const float* sinks, float softcap, hipStream_t stream);
// the same for a step of one token a request, from the q/k/v product's partial sums: bias, rotation and the
// write into the pools happen in the kernel
int fsie_attention_mfma_qkv_ok(int head_dim, int page_size);
int fsie_attention_mfma_qkv(const float* sums, int n_parts, int n_tokens, const float* bias, const float* cos_sin,
                            const int32_t* slots, void* k_pool, void* v_pool, int64_t pool_slots,
                            const int32_t* block_tables, int max_pages, const int32_t* items, int n_items, void* out,
                            float* partials, int n_heads, int n_kv, int head_dim, int page_size, int window,
                            float scale, int waves, hipStream_t stream);
int fsie_attention_mfma_lds_ok(int head_dim, int page_size);
int fsie_attention_mfma_lds(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                            const int32_t* block_tables, int max_pages, const int32_t* items, const int32_t* groups,
                            int n_groups, void* out, int n_heads, int n_kv, int head_dim, int page_size, int window,
                            float scale, const float* sinks, float softcap, hipStream_t stream);
int fsie_attention_mfma_tiles(int head_dim, int large);
int fsie_attention_mfma_max_waves(int head_dim);

// ---- an entry point that allocates nothing --------------------------------------------------
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// fsie_attention_scalar / fsie_attention_mfma (small items) followed by fsie_attention_merge, as one
// call, with the partial records of the key splits kept in a buffer of FSIE_STATIC_SCRATCH_BYTES
// that the library itself holds on every GPU it runs on (a file-scope device array; nothing is
// allocated or freed, here or in any routine called from here).  The caller passes the inputs, the
// tables and the output as for those entry points; `n_partial_slots` is one more than the largest
// partial slot that `items` and `merges` name (slot = one query token of one split); a step that
// needs more than the buffer holds is refused with an error, never computed.  The two tables lie in
// device memory, which this call does not wait for: it runs the kernels on copies of them (kept in
// the same buffer, behind the records, and counted against its size) in which an item or merge that
// names a slot at or beyond `n_partial_slots` does nothing, so a wrong table leaves rows of `out`
// unwritten and never reaches memory outside the buffer.  `mfma` != 0: the
// matrix-core kernel (bfloat16), else the float32-arithmetic kernel.  Every call on a GPU uses
// that GPU's one buffer, which keeps the last call's contents: calls that overlap on one GPU
// (different streams, or threads) race; calls on one stream are ordered and safe.  Nothing needs
// clearing between calls: an item writes every record that a merge reads.
#define FSIE_STATIC_SCRATCH_BYTES (16 * 1024 * 1024)
int64_t fsie_static_scratch_bytes(void);
int fsie_attention_split_static(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                                const int32_t* block_tables, int max_pages, const int32_t* items, int n_items,
                                const int32_t* merges, int n_merges, int n_partial_slots, void* out, int n_heads,
                                int n_kv, int head_dim, int page_size, int window, float scale, int dtype, int mfma,
                                int waves, hipStream_t stream);

int fsie_sample(const float* logits, int n_rows, int vocab, const float* temperature, const int32_t* top_k,
                const float* top_p, const double* uniform, int32_t* out, hipStream_t stream);

// ---- RMS norm in groups, over a stream with up to two pending deltas ----------------------------
// x = residual + delta_scale * (delta1 + delta2) (either delta may be null; each is [total_rows, hidden] in its own
// type, FSIE_F32 or FSIE_BF16), written back to `residual` if write_back; the row is cut into `groups` equal
// consecutive parts, each divided by its own sqrt(mean(part^2) + eps); out1 = that times weight1 and, if weight2 is
// given, out2 = that times weight2 (two norms of one stream in one pass).  `rows` (or null) selects rows; the outputs
// have n_rows rows of type out_dtype.  Sums and the stream are float32.
int fsie_group_rmsnorm(float* residual, const void* delta1, int delta1_dtype, const void* delta2, int delta2_dtype,
                       float delta_scale, const float* weight1, const float* weight2, void* out1, void* out2,
                       const int32_t* rows, int n_rows, int hidden, int groups, float eps, int out_dtype, int write_back,
                       hipStream_t stream);

// ---- a short causal convolution over time, added to its input -----------------------------------
// y[t] = x[t] + sum_j w[:, j] * x[t - taps + 1 + j] within a request, channel by channel (w [hidden][taps], float32);
// the inputs before a portion's first token come from state[slot] [taps - 1][hidden] (float32, oldest first; zeros
// when the request starts), which is then brought up to date with the portion's last inputs (by the same kernel for
// a request's single token, by a second kernel for longer portions).
// x [n_tokens][hidden] float32, y in `dtype`; q_starts [n_seqs + 1], seq_slots [n_seqs]; every request of the step
// brings at least one token.  `state` is the slots' first record: consecutive slots lie `slot_stride` floats apart
// (several convolutions may share a slot).  x2, w2, y2 (all or none): a second convolution of the same sizes in the
// same launches, its state `second` floats into a slot's record.
int fsie_causal_conv(const float* x, const float* w, void* y, const float* x2, const float* w2, void* y2, float* state,
                     int64_t slot_stride, int64_t second, int n_slots, const int32_t* q_starts, const int32_t* seq_slots,
                     int n_seqs, int n_tokens, int hidden, int taps, int dtype, hipStream_t stream);

// ---- mLSTM: a matrix memory with exponential gates ------------------------------------------------
// gates [n_tokens][2 * heads] float32 (input gate logits, then forget gate logits); per request and head the running
// maximum m (state record's last part) is carried: i = cap tanh(gi / cap), f = logsigmoid(cap tanh(gf / cap)),
// m_t = max(f + m_(t-1), i).  Writes coef [n_tokens][heads][4] = (f, i, m_(t-1), m_t).
// Then the memory: S_t = keep S_(t-1) + take k v^T, n_t likewise with k alone; num[t][h][:] = S_t^T q, den[t][h] = n_t . q
// (q scaled by q_scale).  proj [n_tokens][stride] holds q (heads * dim from q_off), k (from k_off), v (heads * vdim
// from v_off).  state [n_slots][heads][dim * vdim + dim + 4] float32: S, n, m (and three unused numbers).
int64_t fsie_mlstm_state_floats(int dim, int vdim);
int fsie_mlstm_scan(const void* proj, int64_t stride, int q_off, int k_off, int v_off, int dtype, const float* gates,
                    float gate_cap, float q_scale, float* state, int n_slots, const int32_t* q_starts,
                    const int32_t* seq_slots, int n_seqs, int n_tokens, int heads, int dim, int vdim, float* coef,
                    float* num, float* den, float* chunk_work, int max_chunks, hipStream_t stream);
// The chunk kernels' work array: with `chunk_work` (room for max_chunks >= n_tokens / chunk_tokens + n_seqs chunks of
// chunk_floats floats) the portions of at least chunk_min tokens go sixteen tokens at a time on the matrix cores.
int fsie_mlstm_scan_shape(int heads, int dim, int vdim, int* chunk_tokens, int* chunk_min, int64_t* chunk_floats);
// y[t][h][:] = unit_rms(num / (max(|den|, exp(-m)) + 1e-6)) * weight[h][:] * sigmoid(gate[t][h][:]), y in `dtype`;
// gate rows lie `gate_stride` values apart (columns of the fused projection)
int fsie_mlstm_out(const float* num, const float* den, const float* coef, const void* gate, int64_t gate_stride,
                   const float* weight, void* y, int n_tokens, int heads, int vdim, float eps, int dtype,
                   hipStream_t stream);

// ---- routed experts ----------------------------------------------------------------------------------
// Router: logits z = x . W^T in float32 (x [n_tokens][hidden] and W [experts][hidden] in `dtype`), s = sigmoid(z); the
// `top` experts with the largest s + correction (ties: the lower index) are chosen; their weights are their s divided
// by the sum of the chosen s (+ 1e-20) times `scale`.  ids [n_tokens][top] int32, weights [n_tokens][top] float32.
int fsie_moe_route(const void* x, const void* router, const float* correction, int dtype, int32_t* ids, float* weights,
                   int n_tokens, int hidden, int experts, int top, float scale, int kind, int groups, int keep, int renorm,
                   hipStream_t stream);
// kind 0: sigmoid scores, 1: softmax over all experts.  groups > 1: experts in that many equal groups of neighbours, only
// those of the `keep` groups with the largest best score (+ correction) can be chosen.  renorm 0: the weights are the
// chosen scores themselves (times scale).  correction may be null.
// Groups the n = n_tokens * top (token, choice) pairs by expert: order[slot] = pair (slots of one expert are
// consecutive), slot_of[pair] = slot, and a table of row tiles of `tile_rows` slots that never cross an expert:
// tiles [max_tiles][3] = (expert, first slot, slots), max_tiles = ceil(n / tile_rows) + experts; unused tiles have 0 slots.
int fsie_moe_group(const int32_t* ids, int n_pairs, int experts, int tile_rows, int32_t* order, int32_t* slot_of,
                   int32_t* tiles, int max_tiles, hipStream_t stream);
// One product per expert over its tiles: out[slot] = epilogue(A[row(slot)] . W[expert]^T), W [experts][N][K] in `dtype`.
// gather_div > 0: row(slot) = order[slot] / gather_div (rows of A are tokens); 0: row(slot) = slot.
// epilogue 0: exact GELU, out in `dtype`; 1: times slot_weight[order[slot]], out float32; 2 + a (a: FsieGateAct): the rows
// of W[expert] are gate and up in turn (N even) and out [slots][N / 2] = act(gate) * up in `dtype`.  tile_rows: 16, 32, 64 or 128,
// the rows of a tile of `tiles`; fsie_moe_tile_rows names the one that suits a step of n_pairs pairs.
int fsie_moe_tile_rows(int n_pairs, int experts);
int fsie_moe_gemm(const void* a, const void* w, void* out, const int32_t* tiles, int max_tiles, const int32_t* order,
                  int gather_div, const float* pair_weight, int N, int K, int epilogue, int dtype, int tile_rows,
                  hipStream_t stream);
// y[t] = sum over the token's choices, in their order, of rows[slot_of[t * top + c]]; y float32 [n_tokens][hidden]
int fsie_moe_combine(const float* rows, const int32_t* slot_of, float* y, int n_tokens, int top, int hidden,
                     hipStream_t stream);

#ifdef __cplusplus
}
#endif
