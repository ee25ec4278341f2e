// The C interface of the kernel library (one build per compute dtype, same symbols).
//
// Conventions: `elem` pointers hold the build's compute dtype (bfloat16 or float32); the
// residual stream, logits and rotary tables are always float32; `*_is_f32` says how a gain
// or bias vector is stored; `stream` is a hipStream_t.  Every function checks its shapes on
// the host, launches on `stream` and returns 0, or a negative code with a message in
// axk_last_error().  Nothing here allocates device memory.
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* axk_last_error(void);
// The kernel instances compiled into the library (only_hit 0) or launched since the last reset
// (only_hit 1), a name a line, into buf; returns the bytes the whole list needs.  A test asserts
// that every instance is launched, and checked, by some test.
long axk_instances(char* buf, long size, int only_hit);
void axk_instances_reset(void);
// 1 for the bfloat16 build, 0 for float32; bytes of one element.
int axk_is_bf16(void);
int axk_elem_size(void);

// x[t, :] = table[tokens[t], :] widened to float32.  A token outside [0, vocab) is an error
// raised by the caller; the kernel clamps nothing.  packed: the table is a packed matrix (see
// axk_pack_matrix; a tied head's), else row-major.
int axk_embed(const int32_t* tokens, const void* table, int packed, float* x, int n_tokens, int dim, int vocab,
              void* stream);

// out[r, :] = (x[row(r), :] * inv_rms) * gain, row(r) = rows ? rows[r] : r.
// The sum of squares runs in 32-bit in an order that depends on `dim` alone.
int axk_rmsnorm(const float* x, const int32_t* rows, const void* gain, int gain_is_f32, void* out,
                int n_rows, int dim, float eps, void* stream);

// table[t, i] = (sin, cos)(positions[t] * freqs[i]) computed in float64, stored float32.
int axk_rope_table(const int32_t* positions, const double* freqs, float* table, int n_tokens,
                   int n_pairs, void* stream);

// Rotate-half on the first `rotary_dim` dims of each q and k head of qkv [T, (nh + 2 nkv) hd]
// (q in place), and store k and v rows into the paged cache at each token's position.
// write_kv = 0 rotates q only.  Cache layout: keys [page][kv head][slot in page][hd], values
// [page][kv head][hd][slot in page] (the positions of one dim are contiguous).
int axk_rope_kv_write(void* qkv, const float* table, const int32_t* positions, const int32_t* seq_rows,
                      const int32_t* block_table, int table_stride, void* k_cache, void* v_cache,
                      int n_tokens, int n_heads, int n_kv_heads, int head_dim, int rotary_dim,
                      int page_size, int write_kv, void* stream);

// Causal attention of every token of the step over its request's cached positions
// lo..=pos, lo = window > 0 ? max(0, pos + 1 - window) : 0.  q rows are `q_stride` elements
// apart; out is [T, nh * hd].  Positions are folded in blocks of 64 in ascending order.
int axk_attention(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                  const int32_t* block_table, int table_stride, const int32_t* positions,
                  const int32_t* seq_rows, void* out, int n_tokens, int n_heads, int n_kv_heads,
                  int head_dim, int page_size, int window, float scale, void* stream);

// The matrix-core attention kernels (bfloat16 build; the float32 build refuses them).
// axk_attention_fast_ok: 1 if they take this head size, page size and group of heads.
// axk_attention_prefill: tiles [n_tiles][4] = (first token, count <= 128) twice: consecutive
// tokens of one request, and a second such run (count 0: none) that the same block takes after
// the first; every token of the step in some run gets its row of `out`.  A causal prompt's runs
// see 1, 2, 3 ... blocks of positions: pairing one that sees many with one that sees few gives
// every block about the same work.
// axk_attention_decode: token_index [n_tokens] names single tokens (null: the first n_tokens
// tokens of the step); a token's range (from the chunk that holds the window's first position,
// or 0) is cut into chunks of axk_attention_decode_chunk positions, four blocks of 64 each.
// work [n_work] lists the chunks to compute, item = slot in token_index *
// axk_attention_decode_item_factor + chunk, or -1 for none: every chunk of every token once.  The
// blocks' results go through `partial` (axk_attention_decode_workspace floats) and a second launch
// folds them in ascending order; max_chunks is the most chunks any of the tokens has.
// Both kernels compute the same arithmetic (blocks of 64 positions aligned to absolute position,
// each with its own maximum, folded ascending): a position's result is bit for bit the same from
// either, alone or in any batch.
int axk_attention_fast_ok(int head_dim, int page_size, int n_heads, int n_kv_heads);
int axk_attention_prefill_tile(void);      // the most tokens of a run (128)
int axk_attention_prefill(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                          const int32_t* block_table, int table_stride, const int32_t* positions,
                          const int32_t* seq_rows, void* out, const int32_t* tiles, int n_tiles,
                          int n_heads, int n_kv_heads, int head_dim, int page_size, int window,
                          float scale, void* stream);
int axk_attention_decode_chunk(void);
int axk_attention_decode_item_factor(void);
long axk_attention_decode_workspace(int n_tokens, int n_heads, int head_dim, int max_chunks);
int axk_attention_decode(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                         const int32_t* block_table, int table_stride, const int32_t* positions,
                         const int32_t* seq_rows, void* out, const int32_t* token_index, int n_tokens,
                         const int32_t* work, int n_work, float* partial, int max_chunks, int n_heads,
                         int n_kv_heads, int head_dim, int page_size, int window, float scale, void* stream);

// The matrix-core products (bfloat16 build) read W packed: blocks of 16 rows x 32 k of 1 KB in
// the order in which a wave holds them as an MFMA operand, [row tile][k block], rows padded with
// zeros to a multiple of 16 (axk_packed_elems elements).  axk_pack_ok: whether a [rows, k] matrix
// (gated: [gate; up] halves for the SwiGLU epilogue) can be packed; what cannot is multiplied
// row-major by the 32-bit FMA kernel.
int axk_pack_ok(int rows, int k, int gated);
long axk_packed_elems(int rows, int k);
int axk_pack_matrix(const void* src, void* dst, int rows, int k, void* stream);

// out = epilogue(X [M, K] . W [N, K]^T + bias).  w_packed: W is packed (see above), else row-major.  mode 0: store elem [M, N]; 1: add into
// float32 [M, N] (the residual stream); 2: store float32 [M, N] (logits); 3: W holds 2 N rows,
// gate rows then up rows, and out elem [M, N] = silu(X . gate^T) * (X . up^T) (no bias).
// x_stride / out_stride: elements between rows.  workspace: axk_gemm_workspace(m, n, k, mode) bytes
// (0 for most shapes: then it may be null), 16-byte aligned; products of more than 16 rows with a
// matrix of several segments give each segment of K blocks of their own and add the segments' sums
// through it (at most 2 GB: a product of more rows than that holds runs in passes).
//
// With a packed W every output element is the sum, in ascending order, of axk_gemm_segments(n, k,
// gated) chains of 32x32x16 MFMAs over contiguous segments of K: the bits of a row do not depend on
// M, that is, on what else is in the batch.
long axk_gemm_workspace(int m, int n, int k, int mode);
int axk_gemm_segments(int n, int k, int gated);
int axk_gemm(const void* x, int x_stride, const void* w, int w_packed, const void* bias, int bias_is_f32, void* out,
             int out_stride, int m, int n, int k, int mode, void* workspace, long workspace_bytes, void* stream);

typedef struct {
  const void* norm_gain;
  int norm_gain_is_f32;
  void* norm_values;
  float norm_eps;
} GemmNormFold;     // the norm behind a product (axk_gemm_then_norm)

// The product that adds into float32 rows (mode 1, W packed) followed by the RMS norm of the new
// rows, for shapes that run with a block per segment of K (axk_gemm_then_norm_ok says 1): the
// kernel that adds the segments' sums also writes norm_values elem [M, N] =
// out / sqrt(mean(out^2) + norm_eps) * norm_gain.  Bit-identical to axk_gemm followed by
// axk_rmsnorm.  workspace: axk_gemm_workspace bytes, as for axk_gemm.
int axk_gemm_then_norm_ok(int m, int n, int k);
int axk_gemm_then_norm(const void* x, int x_stride, const void* w, const void* bias, int bias_is_f32, float* out,
                       int out_stride, int m, int n, int k, const void* norm_gain, int norm_gain_is_f32,
                       float norm_eps, void* norm_values, void* workspace, long workspace_bytes, void* stream);

// The attention's [q; k; v] product (W packed, [(n_heads + 2 n_kv_heads) head_dim, K], or the q rows alone
// if write_kv is 0) with what follows it in the same launches: bias, the rotary encoding of q and k
// heads over their whole width (table [M, head_dim / 2, 2]: sin, cos), q into qkv [M, >= n_heads
// head_dim], k and v into the request's pages (as axk_rope_kv_write stores them).  Up to 16 rows it
// is the product's epilogue; with more rows, where the product runs with a block per segment of K
// (axk_gemm_qkv_rope_ok says so; n = the rows of W), the kernel that adds the segments' sums rotates
// and stores; workspace: axk_gemm_workspace(m, n, k, 0) bytes.  Bit-identical to axk_gemm followed
// by axk_rope_kv_write.
int axk_gemm_qkv_rope_ok(int m, int n, int k, int head_dim, int rotary_dim);
int axk_gemm_qkv_rope(const void* x, int x_stride, const void* w, const void* bias, int bias_is_f32, void* qkv,
                      int qkv_stride, int m, int k, const float* table, const int32_t* positions,
                      const int32_t* seq_rows, const int32_t* block_table, int table_stride, void* k_cache,
                      void* v_cache, int n_heads, int n_kv_heads, int head_dim, int page_size, int write_kv,
                      void* workspace, long workspace_bytes, void* stream);

// Few rows (a decoding step), bfloat16 build: the gated product (out = silu(X Wg^T) * (X Wu^T), W
// the packed [gate; up] matrix) and the [q; k; v] product (as axk_gemm_qkv_rope) with the RMS norm
// of their operand inside: X = axk_rmsnorm(rows, gain, eps) is worked out in the kernel's own LDS
// and never stored.  Bit-identical to axk_rmsnorm followed by axk_gemm / axk_gemm_qkv_rope.
// axk_gemm_normed_ok(m, n, k, gated): whether these sizes are taken (up to 16 rows of a multiple of 256
// up to 4,096 columns, up to 8 rows of up to 5,120); the gain must be bfloat16 (gain_is_f32 = 0).
int axk_gemm_normed_ok(int m, int n, int k, int gated);
int axk_gemm_normed_glu(const float* rows, int rows_stride, const void* gain, int gain_is_f32, float eps, const void* w,
                        void* out, int out_stride, int m, int n, int k, void* stream);
int axk_gemm_normed_qkv_rope(const float* rows, int rows_stride, const void* gain, int gain_is_f32, float eps,
                             const void* w, const void* bias, int bias_is_f32, void* qkv, int qkv_stride, int m, int k,
                             const float* table, const int32_t* positions, const int32_t* seq_rows,
                             const int32_t* block_table, int table_stride, void* k_cache, void* v_cache, int n_heads,
                             int n_kv_heads, int head_dim, int page_size, int write_kv, void* stream);

// out[t, f] = silu(gu[t, f]) * gu[t, F + f]: gate in the first F columns, up in the last.
int axk_swiglu(const void* gate_up, void* out, int n_tokens, int n_ffn, void* stream);

// picks[r] = index of the largest logit of row r; of equal maxima the last; NaN never
// (all NaN: n - 1).  workspace: axk_argmax_workspace(n_rows, n) bytes, 8-byte aligned.
long axk_argmax_workspace(int n_rows, int n);
int axk_argmax(const float* logits, int logits_stride, int32_t* picks, int n_rows, int n, void* workspace,
               void* stream);

// axk_argmax without a workspace.  This entry point has no counterpart in the reference: it is
// for callers that cannot allocate or pass device memory beyond inputs and outputs (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The chunks' keys go
// through an array of the library's own, 128 KB on every GPU it runs on, for up to
// axk_argmax_static_max_rows() rows of up to axk_argmax_static_max_n() logits; more is refused.
// It allocates nothing and frees nothing.  Calls on one GPU share the array: calls that overlap
// there (different streams or threads) race; calls on one stream are ordered and safe.
int axk_argmax_static_max_rows(void);
int axk_argmax_static_max_n(void);
int axk_argmax_static(const float* logits, int logits_stride, int32_t* picks, int n_rows, int n, void* stream);

// Repeat penalty on `recent` ids, then the k best as 64-bit keys (order key of the logit <<
// 32 | id), unsorted, into cands[r, 0..k); the penalty is applied to `logits` in place.  recent is
// [n_rows, recent_stride] with n_recent[r] valid ids each; penalty 1 or n_recent 0: off.
// k <= cands_stride.  workspace: axk_topk_workspace(n_rows, n, cands_stride) bytes, 8-byte aligned
// (the k best of every slice of a row, of which a second launch takes the k best).
long axk_topk_workspace(int n_rows, int n, int cands_stride);
int axk_topk(float* logits, int logits_stride, const int32_t* recent, int recent_stride,
             const int32_t* n_recent, const float* penalty, const int32_t* k_of_row, uint64_t* cands,
             int cands_stride, int n_rows, int n, void* workspace, void* stream);

// dst[i] = value for i < n (a fill that may be captured into a graph).
int axk_fill_i32(int32_t* dst, int32_t value, int n, void* stream);
int axk_fill_f32(float* dst, float value, int n, void* stream);

#ifdef __cplusplus
}
#endif
