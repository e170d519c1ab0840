// C interface of the gfx950 kernel libraries.  This file is the one declaration of every
// entry point: the host core's table of function pointers and the ctypes signatures of the
// Python side are both derived from it (a line "// @library NAME" says which library the
// declarations after it belong to; mk_last_error and mk_abi_version are in both).
// Pointers are device pointers unless a comment says otherwise; `stream` is a hipStream_t.
// Functions validate their arguments on the host against what the kernel and its grid
// assume, return 0 on success and non-zero after recording a message for mk_last_error().
// Dtype codes: 0 = float32, 1 = bfloat16.
#pragma once

#include <hip/hip_runtime.h>

#define MK_ABI_VERSION 21

#ifdef __cplusplus
extern "C" {
#endif

const char* mk_last_error();
int mk_abi_version();

// @library core: float32 arithmetic, float32 or bfloat16 storage

// out[t, :] = table[ids[t], :] * scale as float32 (the residual stream starts here).
int mk_embed(const int* ids, const void* table, int dtype, float* out, int tokens, int hidden,
             int vocab, float scale, hipStream_t stream);

// The residual stream of a step of few tokens in fixed point: 64-bit integers in units of
// 2^-32, into which projections add their results with integer atomics (the sum is the same
// in whatever order they arrive, and nothing has to add partial results up afterwards).
// mk_embed_fixed starts it; mk_rmsnorm_fixed normalises rows of it as mk_rmsnorm does rows of
// h; mk_fixed_add adds `count` float32 partial sums p[k * stride + i], i < n, into it.
int mk_embed_fixed(const int* ids, const void* table, int dtype, long long* out, int tokens,
                   int hidden, int vocab, float scale, hipStream_t stream);
int mk_rmsnorm_fixed(const long long* h64, const void* weight, int weight_dtype, float eps,
                     const int* rows, void* out, int out_dtype, int out_rows, int hidden,
                     hipStream_t stream);
int mk_fixed_add(long long* h64, const float* partials, int count, long long stride, long long n,
                 hipStream_t stream);

// logits[i] = cap * tanh(logits[i] / cap) for i < count, in place.
int mk_logit_cap(float* logits, long long count, float cap, hipStream_t stream);

// Per-request state of fixed size: rows of `state` [slots, width] (float32), a sequence's row
// being slots[token_seq[t]].  mk_state_store: every token at absolute position `at_position`
// writes its row of x [tokens, width] into its sequence's slot.  mk_state_load: every token's
// row of out is its sequence's row of the state.
int mk_state_store(const void* x, int dtype, float* state, const int* slots, const int* token_seq,
                   const int* positions, int at_position, int tokens, int width,
                   hipStream_t stream);
int mk_state_load(const float* state, const int* slots, const int* token_seq, void* out, int dtype,
                  int tokens, int width, hipStream_t stream);

// RMSNorm of rows of the float32 residual stream h, optionally after adding `num_partials`
// partial sums [p, row, hidden] (stride between partials in elements) into h.  `rows`, when
// not null, lists the rows of h to normalise; out row i then comes from h row rows[i].
int mk_rmsnorm(float* h, const float* partials, int num_partials, long long partial_stride,
               const void* weight, int weight_dtype, float eps, const int* rows, void* out,
               int out_dtype, int out_rows, int hidden, hipStream_t stream);

// out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i].
int mk_silu_mul(const void* gate_up, void* out, int dtype, int tokens, int inter,
                hipStream_t stream);

// Rotary encoding of the q and k heads of qkv [T, row_stride] (q in place) and the write of
// rotated k into the paged key cache [pages, n_kv, page_size, d] and of raw v into the value
// cache, which is transposed within a page: [pages, n_kv, d, page_size].  The first `rot`
// dims of a head turn, pair j being dims (j, j + rot/2), or (2j, 2j + 1) when `interleaved`.
int mk_rope_kv_write(void* qkv, int dtype, int row_stride, const float* cos_table,
                     const float* sin_table, int table_positions, const int* positions,
                     const int* token_seq, const int* block_table, int table_stride,
                     void* k_cache, void* v_cache, int page_size, int n_q, int n_kv, int d,
                     int rot, int interleaved, int write_kv, int tokens, hipStream_t stream);

// y = x W^T (+ bias) with float32 FMA.  accumulate: y (float32) += instead of =.
int mk_linear_generic(const void* x, const void* w, int dtype, const void* bias, int bias_dtype,
                      void* out, int out_dtype, int accumulate, int M, int N, int K, int lda,
                      int ldo, hipStream_t stream);

// Causal grouped-query attention over the paged cache for any mix of prompt portions and
// decoded tokens; window = 0 means all earlier keys.  score_cap > 0: the scaled score becomes
// cap * tanh(score / cap); distance_slopes (float32 [n_q], or null): slope[head] * (query
// position - key position) is subtracted from it.
int mk_attention_generic(const void* q, int q_stride, void* out, int out_stride,
                         const void* k_cache, const void* v_cache, int dtype,
                         const int* positions, const int* token_seq, const int* block_table,
                         int table_stride, int page_size, int n_q, int n_kv, int d, float scale,
                         int window, float score_cap, const float* distance_slopes, int tokens,
                         hipStream_t stream);

// mk_rope_kv_write for a projection that arrives as float32 partial sums [p, T, width] of a
// K-split product: the slices are added in order (with the bias) before the rotation; q goes
// to q_out [T, n_q d].
int mk_qkv_finish(const float* partials, int num_partials, long long partial_stride,
                  const void* bias, int bias_dtype, void* q_out, int dtype,
                  const float* cos_table, const float* sin_table, int table_positions,
                  const int* positions, const int* token_seq, const int* block_table,
                  int table_stride, void* k_cache, void* v_cache, int page_size, int n_q,
                  int n_kv, int d, int rot, int write_kv, int tokens, hipStream_t stream);

// out[i] = mean + std * normal(key, i) for i < n, rounded to the dtype: the values the host
// core's fill computes for the same key (random_normal.h), so random weights are the same
// numbers wherever they are drawn.
int mk_fill_normal(void* out, int dtype, long long n, unsigned long long key, float mean,
                   float std, hipStream_t stream);

// @library mfma: bfloat16 kernels on the matrix cores

// y = x W^T for 1 <= M <= 16 rows of x, K split into `slices` (ask mk_linear_skinny_slices
// for a good count): out is float32 [slices, M, N], to be summed over the slices.
int mk_linear_skinny_slices(int M, int N, int K);
int mk_linear_skinny(const void* x, const void* w, float* out, int M, int N, int K, int slices,
                     hipStream_t stream);

// out[M, N] (float32) += x W^T (+ bias) for 1 <= M <= 16, all of K in each workgroup;
// mk_linear_skinny_unsplit says whether that is the faster form for the shape.
int mk_linear_skinny_unsplit(int M, int N, int K);
int mk_linear_skinny_acc(const void* x, const void* w, const void* bias, int bias_dtype,
                         float* out, int M, int N, int K, hipStream_t stream);

// h64[M, N] (the fixed-point residual stream, see mk_embed_fixed) += x W^T (+ bias) for
// 1 <= M <= 16, K in `slices` slices as mk_linear_skinny takes them.
int mk_linear_skinny_fixed(const void* x, const void* w, const void* bias, int bias_dtype,
                           long long* h64, int M, int N, int K, int slices, hipStream_t stream);

// act[M, inter] (bfloat16) = silu(x Wg^T) * (x Wu^T) for w = [Wg | Wu] stacked [2 inter, K],
// 1 <= M <= 16.
int mk_gated_skinny(const void* x, const void* w, void* act, int M, int inter, int K,
                    hipStream_t stream);

// The gated and the q/k/v projection of at most 16 rows on x = rmsnorm(h64) * norm_w, which
// every workgroup makes for itself from the fixed-point residual stream h64 [M, K] (the norm
// needs no kernel of its own); K at most mk_skinny_normed_max_k(M).
int mk_skinny_normed_max_k(int M);
int mk_gated_skinny_normed(const long long* h64, const void* norm_w, int norm_dtype, float eps,
                           const void* w, void* act, int M, int inter, int K, hipStream_t stream);
int mk_qkv_skinny_normed(const long long* h64, const void* norm_w, int norm_dtype, float eps,
                         const void* w, const void* bias, int bias_dtype, void* q_out,
                         const float* cos_table, const float* sin_table, int table_positions,
                         const int* positions, const int* token_seq, const int* block_table,
                         int table_stride, void* k_cache, void* v_cache, int page_size, int n_q,
                         int n_kv, int d, int rotate, int M, int K, hipStream_t stream);

// The q/k/v projection of 1 <= M <= 64 tokens, w = [(n_q + 2 n_kv) d, K], with bias, rotation
// of q and k over the whole head (rotate != 0), q [M, n_q d] out and k, v written to the
// paged cache; n_kv = 0 projects the queries only.  d must be a multiple of 32.
int mk_qkv_skinny(const void* x, const void* w, const void* bias, int bias_dtype, void* q_out,
                  const float* cos_table, const float* sin_table, int table_positions,
                  const int* positions, const int* token_seq, const int* block_table,
                  int table_stride, void* k_cache, void* v_cache, int page_size, int n_q,
                  int n_kv, int d, int rotate, int M, int K, hipStream_t stream);

// The q/k/v projection as mk_qkv_skinny, for any M, tiled through LDS; config: a tile
// configuration, -1 for the one estimated fastest.
int mk_qkv_tiled(const void* x, const void* w, const void* bias, int bias_dtype, void* q_out,
                 const float* cos_table, const float* sin_table, int table_positions,
                 const int* positions, const int* token_seq, const int* block_table,
                 int table_stride, void* k_cache, void* v_cache, int page_size, int n_q,
                 int n_kv, int d, int rotate, int M, int K, int config, hipStream_t stream);

// The gated projection for any M, tiled through LDS; config: a tile configuration, -1 for the
// one estimated fastest.
int mk_gated_tiled_config(int M, int inter, int K);
int mk_gated_tiled(const void* x, const void* w, void* act, int M, int inter, int K, int config,
                   hipStream_t stream);

// y = x W^T (+ bias) for any M, tiled through LDS; output bfloat16 or float32, or float32
// accumulated into `out`.  config: a tile configuration, 0 .. mk_linear_tiled_configs() - 1
// (mk_linear_tiled_config picks the one estimated fastest for the shape and the bytes the
// epilogue moves per element of y; -1 does the same).
// mk_linear_tiled_partials: the same product as float32 partial sums out[slices, M, N] over
// slices of K, for few rows of x over a long K (mk_linear_tiled_slices: how many slices pay;
// any count that the 64-wide stages of K divide into is taken).
int mk_linear_tiled_slices(int M, int N, int K);
int mk_linear_tiled_partials(const void* x, const void* w, float* out, int M, int N, int K,
                             int slices, hipStream_t stream);
int mk_linear_tiled_configs(void);
int mk_linear_tiled_config(int M, int N, int K, int out_bytes);
int mk_linear_tiled(const void* x, const void* w, const void* bias, int bias_dtype, void* out,
                    int out_dtype, int accumulate, int M, int N, int K, int ldo, int config,
                    hipStream_t stream);

// Whether mk_attention_mfma takes this head size and page size.
int mk_attention_mfma_supported(int head_dim, int page_size);

// The most rows per tile (16, 32 or 64) mk_attention_mfma takes for this head size.
int mk_attention_mfma_max_rows(int head_dim);

// The same attention on the matrix cores.  The caller cuts the step into tiles of
// rows_per_tile rows (row f of a sequence = token f / G, head kvh * G + f % G):
// tile_seq / tile_row0 name each tile's sequence and first row.  cu_q [S+1] are the prefix sums of the sequences' token
// counts, kv_len [S] their lengths once this step's tokens are written.  With num_splits > 1
// the keys are split, split_blocks blocks of 32 keys per split (0: each tile's own range in
// num_splits equal parts), and part_o [tiles, n_kv, splits, rows_per_tile, d] /
// part_ml [.., rows_per_tile, 2] hold the partial results.  staged != 0: the tiles are of
// 4 * rows_per_tile rows, one per workgroup, whose wavefronts share the keys and values
// through LDS, `staged` (1, 2 or 4, at most what mk_attention_mfma_staged returns) groups of
// four wavefronts taking the key blocks in turn; for many rows per sequence, keys unsplit.
// staged = 8: the prompt kernel built on 32 x 32 x 16 products (wavefronts of 32 rows, blocks
// of 64 keys; tiles of 128 rows, rows_per_tile = 32), where mk_attention_mfma_wide says so.
// tile_seq = tile_row0 = null: no tile list, tile t is the one new token of sequence t
// (decoding; tiles of 16 rows, at most 16 heads a group, no window, split_blocks 0): part s of
// num_splits is then the blocks s, s + num_splits, ... of the keys, and the kernel asks for
// nothing before the block table.
// mk_attention_mfma_check: what mk_attention_mfma checks of its arguments before it launches,
// without the launch (0: it would take them; else mk_last_error() says why not).
int mk_attention_mfma_staged(int head_dim, int rows_per_tile);
int mk_attention_mfma_wide(int head_dim);
// The same kernel on tiles of 64 rows (two wavefronts a key group; staged = 8 * chains + 4):
// which numbers of chains exist at this head size (bit n - 1).
int mk_attention_mfma_wide_half(int head_dim);
// Which of these instantiations, as its `staged` code, measured fastest for a step of `wg128`
// workgroups of 128 rows or `wg64` of 64 (key/value heads counted) whose longest sequence is
// `blocks32` blocks of 32 keys, most of them this step's own or not (`fresh`); 0: none, the
// 16-row kernels are faster.
int mk_attention_mfma_wide_choice(int head_dim, int wg128, int wg64, int blocks32, int fresh);
int mk_attention_mfma_check(int q_stride, int out_stride, int num_tiles, int page_size, int n_q,
                            int n_kv, int d, float scale, int window, int rows_per_tile,
                            int staged, int num_splits, int split_blocks, int has_workspace);
int mk_attention_mfma(const void* q, int q_stride, void* out, int out_stride,
                      const void* k_cache, const void* v_cache, const int* tile_seq,
                      const int* tile_row0, int num_tiles, const int* cu_q, const int* kv_len,
                      const int* block_table, int table_stride, int page_size, int n_q, int n_kv,
                      int d, float scale, int window, int rows_per_tile, int staged,
                      int num_splits, int split_blocks, float* part_o, float* part_ml,
                      hipStream_t stream);

// Decoding with split keys, in two kernels instead of three.  mk_attention_mfma_parts is
// mk_attention_mfma without the merge of the key splits: the partial results stay in part_o /
// part_ml, mk_attention_mfma_parts_written(...) of them per (tile, kv head) (a workgroup's four
// wavefronts may have added four parts up already).  mk_attention_out then merges them and
// multiplies by the output matrix w_o [N, n_q d] in one kernel, for steps of one token per
// sequence (tile = token, M of them): out[slice, M, N] are float32 partial sums over slices of
// heads_per_slice query heads each (mk_attention_out_heads_per_slice: how many, for slices
// stored or, with `atomic`, added into the fixed-point stream; 0 where the sizes are not taken; mk_attention_out_max_parts: the most partial results per (tile, kv head)
// it takes), to be added up by whoever consumes the projection; or, with `out` null, the
// result is added into the fixed-point residual stream fixed_out [M, N] (see mk_embed_fixed).
// wide: 128 rows of w_o per workgroup instead of 64.
int mk_attention_mfma_parts_written(int rows_per_tile, int num_splits, int d);
int mk_attention_mfma_parts(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                            const int* tile_seq, const int* tile_row0, int num_tiles,
                            const int* cu_q, const int* kv_len, const int* block_table,
                            int table_stride, int page_size, int n_q, int n_kv, int d, float scale,
                            int window, int rows_per_tile, int num_splits, int split_blocks,
                            float* part_o, float* part_ml, hipStream_t stream);
int mk_attention_out_heads_per_slice(int n_q, int n_kv, int d, int M, int N, int atomic);
int mk_attention_out_max_parts(int M, int heads_per_slice);
int mk_attention_out(const float* part_o, const float* part_ml, int parts, const void* w_o,
                     float* out, long long* fixed_out, int M, int N, int n_q, int n_kv, int d,
                     int heads_per_slice, int wide, hipStream_t stream);

// @library core

// parts: optional scratch of rows * 64 * 8 bytes; with it, few rows of a large vocabulary
// are searched by 64 workgroups per row.
int mk_argmax(const float* logits, int rows, int vocab, long long row_stride, int* out,
              void* parts, hipStream_t stream);

// mk_argmax without a buffer of the caller's, and without any allocation: the partial results
// live in a device array inside the library (one per GPU, kept until the process ends), of
// mk_argmax_static_max_rows() rows; more rows are refused.  This entry point has no
// counterpart in the reference: it is for callers that cannot allocate (code under HIP graph
// capture, serving loops and harnesses that forbid hipMalloc).  Calls that overlap on one GPU
// share the array and race; calls on one stream, one after the other, are safe.  The first
// call on a device asks the runtime where the array lies; mk_argmax_static_init() does only
// that, for the current device, so that a caller can have it done before a stream capture
// begins.  Both may be called from several threads.
int mk_argmax_static_max_rows(void);
int mk_argmax_static_init(void);
int mk_argmax_static(const float* logits, int rows, int vocab, long long row_stride, int* out,
                     hipStream_t stream);

// One token per row: the argmax where temperature <= 0, else an inverse-CDF draw with the
// row's uniform number from softmax(logits / temperature) restricted to the nucleus top_p
// (top_ps null: no row restricts it, and the threshold search is skipped).  scratch:
// mk_sample_scratch_bytes(rows, top_ps != null) bytes, 256-byte aligned.
long long mk_sample_scratch_bytes(int rows, int nucleus);
int mk_sample(const float* logits, int rows, int vocab, long long row_stride,
              const float* temperatures, const float* top_ps, const float* uniforms,
              void* scratch, int* out, hipStream_t stream);

#ifdef __cplusplus
}
#endif
