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

// axk_embed with every value multiplied by `scale` (32-bit) on the way.
int axk_embed_scaled(const int32_t* tokens, const void* table, int packed, float* x, int n_tokens, int dim, int vocab,
                     float scale, void* stream);

// A norm on a sublayer's output: x[r, :] += mult * ((y[r, :] * inv_rms(y[r, :])) * gain); `rounded`
// (elem [n_rows, dim], or null) also gets the new x in the compute dtype.
int axk_norm_add(const float* y, const void* gain, int gain_is_f32, float eps, float mult, float* x, void* rounded,
                 int n_rows, int dim, void* stream);
// x[r, :] = norm(alpha x[r, :] + y[r, :]) * gain: the norm behind the sum; kind 0: an RMS norm, kind 1: a
// layer norm (mean taken off, the variance the mean of the squared deviations).  `rounded` as above.
int axk_sum_norm(const float* y, float alpha, const void* gain, int gain_is_f32, float eps, int kind, float* x, void* rounded,
                 int n_rows, int dim, void* stream);
// Layer norm with a gain and no bias of float32 rows (rows: which, or null for all) into the compute dtype.
int axk_layernorm(const float* x, const int32_t* rows, const void* gain, int gain_is_f32, void* out, int n_rows, int dim,
                  float eps, void* stream);
// v[r, i] = cap tanh(v[r, i] / cap), in place on float32 rows row_stride apart.
int axk_softcap(float* v, long row_stride, int n_rows, int n, float cap, void* stream);
// v[r, i] *= factor, in place on float32 rows row_stride apart.
int axk_scale_rows(float* v, long row_stride, int n_rows, int n, float factor, void* stream);
// x[i] += factor * y[i] on n float32 values.
int axk_add_scaled(float* x, const float* y, float factor, long n, void* stream);
// out[i] = x[i] in the compute dtype.
int axk_round_rows(const float* x, void* out, long n, void* stream);
// out[t, :] = [a[t, :] | b[t, :]] in the compute dtype (a [n_rows, wa], b [n_rows, wb] float32).
int axk_concat_round(const float* a, int wa, const float* b, int wb, void* out, int n_rows, void* stream);
// In place on elem values; kind 0: the tanh form of GELU; kind 1: the exact (erf) GELU.
int axk_activation(void* v, long n, int kind, void* stream);
// out[t, f] = g sigmoid(alpha g) (u + 1), g = min(gate_up[t, f], limit), u = clamp(gate_up[t, F + f], -limit, limit).
int axk_clamped_glu(const void* gate_up, void* out, int n_tokens, int n_ffn, float limit, float alpha, void* stream);

// Grouped products (csrc/grouped_gemm.hip):
//   out[orow(r), g ogs + n] = epilogue(sum_k X[xrow(r), g xgs + k] W[g][n][k] + bias[g][n]),
// W elem [groups][n (2 n with glu)][k].  tiles == null: every row r < m meets every group
// (block-diagonal; x_rows and out_rows must be null).  tiles [.][3] = (group, first listed row,
// count <= tile_rows) with *n_tiles of them on the device (max_tiles: the most there can be;
// tile_rows 16, or 64 for many rows a group: tiles through LDS, the same chains, the same bits): the rows
// listed, x_rows / out_rows naming the row of X each reads and the row of out it writes (null:
// the listed row itself).  glu: g = min(gate, limit), u = clamp(up, -limit, limit), out = g
// sigmoid(alpha g) (u + shift); an infinite limit, alpha 1 and shift 0 are silu(gate) up.  gate (float32,
// rows gate_row_stride apart): out is multiplied by sigmoid(gate[orow, g ogs + n]), or with
// gate_per_group by sigmoid(gate[orow, g]), one number a group.  Strides count elements.  An output's chain over k depends on
// k, the strides' alignment and the build alone (axk_grouped_gemm_uses_mfma says which chain).  row_scale (float32
// [out rows], or null): the sums of out row r are multiplied by row_scale[r] before bias and epilogue (a factor on
// the row of X).
int axk_grouped_gemm_uses_mfma(int k, int x_is_f32, long x_row_stride, long x_group_stride);
int axk_grouped_gemm(const void* x, int x_is_f32, long x_row_stride, long x_group_stride, const int32_t* x_rows,
                     const void* w, const void* bias, int bias_is_f32, void* out, int out_is_f32, long out_row_stride,
                     long out_group_stride, const int32_t* out_rows, const float* gate, long gate_row_stride,
                     int gate_per_group, const float* row_scale, int glu, float glu_limit, float glu_alpha, float glu_shift,
                     const int32_t* tiles,
                     const int32_t* n_tiles, int max_tiles,
                     int tile_rows, int m, int n, int k, int groups, void* stream);

// Routing (csrc/moe.hip).  axk_route_topk: for each token the `top` largest of its n_experts
// logits (the largest first; of equal ones the lower expert) and the softmax over these.
// axk_route_scored: scores s = sigmoid(logits) that do not compete; chosen by s + correction (float32
// [n_experts], or null) among the experts of the `keep` best of `groups` equal groups of neighbours (a
// group's score: the sum of its two largest choice scores), weights s / (sum of the chosen s + 1e-20)
// * scale (without `normalize`: s * scale); rows of logits are logits_stride apart.  Up to 1,024 experts in up to
// 64 groups, up to 64 a token.
// axk_route_sort: the pairs p = t top + k in expert order (sorted, and each one's token in
// sorted_tokens) and the tiles (of up to tile_rows rows) of the grouped product, at most
// axk_route_max_tiles of them.
// place_of [n_pairs] (or null): where each pair stands in `sorted`; first_of [n_experts + 1] (or
// null): where each expert's pairs start there.
// axk_route_combine: y[t, :] (+)= sum_k weights[t, k] rows[t top + k, :], k ascending (with
// place_of: rows[place_of[t top + k], :]); weights may be null (all 1); extra (float32 [n_tokens, width], or null) is
// a further row a token, times sigmoid(extra_gate[t extra_gate_stride]) if extra_gate is given.  axk_gather_rows: out[r, :] = x[rows[r], :] (elem).
int axk_route_topk(const float* logits, int n_tokens, int n_experts, int top, int32_t* experts, float* weights, void* stream);
int axk_route_scored(const float* logits, long logits_stride, const float* correction, int n_tokens, int n_experts, int top,
                     int groups, int keep, float scale, int normalize, int32_t* experts, float* weights, void* stream);
int axk_route_max_tiles(int n_pairs, int n_experts, int tile_rows);
int axk_route_sort(const int32_t* experts, int n_pairs, int n_experts, int top, int32_t* sorted, int32_t* sorted_tokens,
                   int32_t* tiles, int32_t* n_tiles, int32_t* place_of, int32_t* first_of, int tile_rows, void* stream);
int axk_route_combine(const float* rows, const float* weights, float* y, int n_tokens, int top, int width, int accumulate,
                      const int32_t* place_of, const float* extra, const float* extra_gate, long extra_gate_stride, void* stream);
int axk_gather_rows(const void* x, long x_stride, const int32_t* rows, void* out, int n_rows, int width, void* stream);

// A short causal convolution per channel and a gated linear recurrence (csrc/recurrent.hip).  A
// request's state row (float32, rows state_stride apart) holds two copies of ([channels] of
// recurrent state, then [taps - 1][channels] of the convolution's last inputs, oldest first); zeros
// for a new request.  The state behind position p is in copy p & 1, so a step of one token reads one
// copy and writes the other, and gives the same result if it is run again.
// axk_causal_conv: u[t, c] = bias[c] + sum_k w[c, k] in(t - (taps - 1 - k)), inputs before the
// step from the state.  Reads the state only.
// axk_gated_scan: per request of the step (spans [n][3] = (slot, first token, tokens); null: each
// token a request of its own in slot seq_rows[t]) and channel, over its tokens in order:
// r = sigmoid(gates r), i = sigmoid(gates i), a = exp(-decay r softplus(lam)),
// S = a S + sqrt(1 - a^2) (i u), out = S gelu(y); then the state row is brought up to date
// (S, and the convolution's inputs from x).  gates [T, channels / block_width, 2 block_width].
// terms (float32 [n_tokens, 3, channels], with spans): what does not depend on the state is worked
// out for all tokens at once first, and the walk over a request's tokens is left with one
// multiply-add a step (the same bits; for long stretches of tokens).
int axk_causal_conv(const void* x, long x_stride, const void* w, const void* bias, int bias_is_f32, const float* state,
                    long state_stride, const int32_t* positions, const int32_t* seq_rows, float* u, int n_tokens,
                    int channels, int taps, void* stream);
int axk_gated_scan(const float* gates, const float* u, const void* y, long y_stride, const void* x, long x_stride,
                   const void* lam, int lam_is_f32, float decay, float* state, long state_stride, const int32_t* spans,
                   int n_spans, const int32_t* positions, const int32_t* seq_rows, void* out, int channels, int block_width,
                   int taps, float* terms, int n_tokens, void* stream);

// A selective state-space mixer in its recurrent form (csrc/state_space.hip).  A request's state row (float32, rows
// state_stride apart) holds two copies of copy_elems floats: the heads' states [heads][N][P] first, and from tail_at
// [taps - 1][channels] of the convolution's last inputs, oldest first; the state behind position p is in copy p & 1.
// axk_state_conv: u[t, c] = act(bias[c] + sum_k w[c, k] in(t - (taps - 1 - k))) over float32 rows x (silu: act is
// silu, else none), inputs before the step from the state; with heads > 0 also terms[t, h] = (dt, a) with
// dt = softplus(raw[t, h] + dt_bias[h]), a = exp(-exp(a_log[h]) dt).  Reads the state only.
// axk_state_space_scan: per request of the step (spans [n][3] = (slot, first token, tokens); null: each token a
// request of its own in slot seq_rows[t]) and head, over its tokens in order, S = a S + dt B x^T, y = S^T C + D x
// with u [T, channels] = [x: heads P | B: groups N | C: groups N]; y float32 [T, heads P]; then the state row is
// brought up to date (S, and the convolution's inputs from conv_in, float32 rows conv_in_stride apart).  With segs
// ([n_segs][4] = (slot, first token, tokens, whether the request's first), the requests' stretches cut into
// segments in order, none longer than longest_seg; spans5 [n][5] = (slot, first token, tokens, first segment, segments); ends float32 [n_segs,
// heads, N, P]; cum float32 [T, heads]) the segments run side by side and two more launches fold their end states
// and add what each segment's carried-in state gives its outputs (sums in another order than one walk's, by rounding).
// axk_gated_group_norm: out[t] = rms in `parts` equal parts of (y[t] silu(z[t])), times gain; out elem [T, width].
int axk_state_conv(const float* x, long x_stride, const void* w, const void* bias, int bias_is_f32, int silu, const float* state,
                   long state_stride, long copy_elems, long tail_at, const int32_t* positions, const int32_t* seq_rows, float* u,
                   int n_tokens, int channels, int taps, const float* raw, long raw_stride, const void* dt_bias,
                   int dt_bias_is_f32, const void* a_log, int a_log_is_f32, float* terms, int heads, void* stream);
int axk_state_space_scan(const float* u, const float* terms, const void* d_skip, int d_is_f32, float* state, long state_stride,
                         long copy_elems, long tail_at, const int32_t* spans, int n_spans, const int32_t* positions,
                         const int32_t* seq_rows, const float* conv_in, long conv_in_stride, float* y, int heads, int groups,
                         int vdim, int n_state, int taps, const int32_t* segs, int n_segs, int longest_seg, const int32_t* spans5,
                         float* ends, float* cum, void* stream);
int axk_gated_group_norm(const float* y, const float* z, long z_stride, const void* gain, int gain_is_f32, float eps, void* out,
                         int n_tokens, int width, int parts, void* stream);

// Attention over a latent cache (csrc/latent_attention.hip); a page is [page_size][rank + rot] elem
// (the latent and the rotated key part of each position), then [rank][page_size] (the latents again,
// the positions of one dim side by side): 2 rank + rot elements a position.
// axk_latent_prepare: from the float32 rows of the down projections, the normed query latent
// (cq elem [T, q_rank]; q_rank 0: none) and, with write_kv, the normed key/value latent and the
// rotated shared key part into the request's page.  axk_latent_query_rope: the rotated part of
// every head's query (q float32, rows q_stride apart) into q_full [T, heads, rank + rot] (places rank ..).
// Rotation: pairs (i, i + rot_dims / 2), or (2i, 2i + 1) with `neighbours`; cos and sin times `magnitude`.
// axk_latent_attention: o_lat [T, heads, rank] = softmax over lo ..= pos of (q_full . page row) scale, times
// the rows' first `rank` places; lo = window > 0 ? max(0, pos + 1 - window) : 0.  sink (float32 [heads], or
// null): the softmax's denominator also holds exp(sink[head]), once, with no value.
int axk_latent_prepare(const float* fused, long stride, int q_at, int q_rank, int kv_at, int rank, int rot, int rot_dims,
                       int neighbours, float magnitude, const void* q_gain, int q_gain_is_f32, const void* kv_gain, int kv_gain_is_f32, float eps,
                       const float* table, const int32_t* positions, const int32_t* seq_rows, const int32_t* block_table,
                       int table_stride, void* cache, int page_size, void* cq, int n_tokens, int write_kv, void* stream);
int axk_latent_query_rope(const float* q, long q_stride, int dim, int rot, int rot_dims, int neighbours, float magnitude,
                          const float* table, float* q_full, int rank, int heads, int n_tokens, void* stream);
// partial: axk_latent_attention_workspace floats (0 for most calls; with few tokens the blocks of 64
// positions of a token then run side by side and a second launch folds them), or null.  span: the most
// positions a row of the step sees, for attention without a window (0: not known).
int axk_latent_attention_uses_mfma(int heads, int rank, int rot, int page_size);
long axk_latent_attention_workspace(int n_tokens, int heads, int rank, int rot, int page_size, int window, int span);
int axk_latent_attention(const float* q_full, const void* cache, const int32_t* block_table, int table_stride,
                         const int32_t* positions, const int32_t* seq_rows, float* o_lat, int n_tokens, int heads, int rank,
                         int rot, int page_size, int window, int span, float scale, const float* sink, float* partial,
                         long partial_floats, void* stream);

// Grouped-query attention with one or two score maps a head, an optional norm of queries and keys, a
// sliding-window or chunked mask, bent scores and a gate (csrc/masked_attention.hip).  A page is
// [page_size][kv_heads maps dim] elem (key rows), then [kv_heads vdim][page_size] (values, the positions
// of one dim side by side).
// axk_heads_prepare: from the float32 rows of the projections (n_q query units and n_k key units of `dim`
// each, v_width values; v_at may equal k_at), units RMS-normed with a gain shared by all units (null: no
// norm), the first `rot` dims rotated by table [T, rot / 2, 2] (sin, cos; both scaled by `magnitude`) in
// pairs (2i, 2i + 1) if `neighbours` else (i, i + rot / 2); queries into q_out elem [T, n_q dim], keys and
// values into the page (if write_kv).  q_temp_every > 0: a query at position p is multiplied by
// 1 + q_temp_coef ln(floor((p + 1) / q_temp_every) + 1).
int axk_heads_prepare(const float* proj, long stride, int q_at, int n_q, int k_at, int n_k, int v_at, int v_width, int dim,
                      const void* q_gain, int q_gain_is_f32, const void* k_gain, int k_gain_is_f32, float eps, int rot,
                      int neighbours, float magnitude, const float* table, const int32_t* positions, const int32_t* seq_rows,
                      const int32_t* block_table, int table_stride, void* cache, int page_size, void* q_out, int n_tokens,
                      int write_kv, float q_temp_coef, int q_temp_every, void* stream);
// axk_masked_attention: q elem [T, heads maps dim] -> out elem [T, heads vdim].  mask_kind 0: all earlier
// positions; 1: the last mask_size positions; 2: the earlier positions of the same chunk of mask_size.
// softcap > 0: s <- softcap tanh(s / softcap).  maps 2: o = rms(a_1 - lambda a_2, eps) out_scale.  gate
// (float32 rows of gate_stride, or null): o *= sigmoid(gate), heads vdim numbers a row, or with gate_per_head
// one a head.  sink > -inf: the softmax's sum also holds exp(sink), a key of that score without a value.  tiles (int32 [n_tiles, 2]: first token,
// count; up to 16 consecutive tokens of one request each) or null (every token a tile of its own) are
// what the matrix-core kernel works on where axk_masked_attention_uses_mfma says 1.
// partial: axk_masked_attention_workspace floats (steps of few tokens: the blocks of 64 positions of a single token
// then run side by side and a second launch folds them; with mask_kind 0 as many blocks as `span`, the positions
// the step's longest row sees, make: 0 there means no such split), or null.
int axk_masked_attention_uses_mfma(int heads, int kv_heads, int maps, int dim, int vdim, int page_size);
long axk_masked_attention_workspace(int n_tokens, int heads, int kv_heads, int maps, int dim, int vdim, int page_size,
                                    int mask_kind, int mask_size, int span);
int axk_masked_attention(const void* q, const void* cache, const int32_t* block_table, int table_stride,
                         const int32_t* positions, const int32_t* seq_rows, const float* gate, long gate_stride, void* out,
                         int n_tokens, int heads, int kv_heads, int maps, int dim, int vdim, int page_size, int mask_kind,
                         int mask_size, float scale, float softcap, float lambda, float out_scale, float eps,
                         const int32_t* tiles, int n_tiles, float* partial, long partial_floats, float sink, int gate_per_head,
                         int span, void* stream);

#ifdef __cplusplus
}
#endif
