// C interface of libsprout_hip.so.  Every function returns 0 on success; otherwise
// sp_last_error() gives the reason.  Pointers are device pointers unless named host_*.
// dtype codes: 0 = float32, 1 = bfloat16.  All launches go to `stream`.
// Variants of an operation that parts may ask for are numbered, one `int` each; a number that no kernel
// implements is refused with an error, so another variant is an addition here and in the kernels, never a guess:
//   pairing of a rotation     0 = halves of the rotated dimensions (d with d + rotary_dim / 2, "neox")
//   activation of a gated product   0 = SiLU(g) * u (x / (1 + exp(-x)));  1 = clamped: g' = min(g, limit),
//                                   u' = clamp(u, -limit, limit), g' * sigmoid(1.702 g') * (u' + 1);  2 = max(g, 0) * u
#pragma once
#include <stdint.h>

extern "C" {

const char* sp_last_error();
int sp_version();

// residual[t, :] = table[tokens[t], :]            residual is float32 [T, H]
int sp_embed(void* stream, int table_dtype, const void* table, const int32_t* tokens, float* residual,
             int T, int H, int V);

// out[r, :] = rmsnorm(x[rows ? rows[r] : r, :]) * w      x float32 [*, H]; out [R, H] of out_dtype
int sp_rmsnorm(void* stream, const float* x, const int32_t* rows, int w_dtype, const void* w, float eps,
               int out_dtype, void* out, int R, int H);

// out = a[T, K] . w[N, K]^T (+ bias[N])
// mode 0: store as out_dtype [T, N];  mode 1: out (float32 [T, N]) += result;  mode 2: store float32
int sp_gemm(void* stream, int a_dtype, const void* a, int w_dtype, const void* w, int bias_dtype,
            const void* bias, int mode, int out_dtype, void* out, int T, int N, int K);

// Decode-sized products (T <= 64, bfloat16) with neighbouring work folded in.  Activations are x
// [T, K] bfloat16, or, with residual != null, rmsnorm(residual [T, K] float32) * norm_w computed inside.
// sp_fused_supported(kind, ...): kind 0..2 = plain modes of sp_gemm, 3 = sp_qkv_rope_cache, 4 = sp_gate_up_silu.
// `variant`: the pairing (kind 3) or the activation (kind 4) asked for; 0 otherwise.
int sp_fused_supported(int kind, int T, int N, int K, int hd, int rotary_dim, int norm, int variant);
// Whether folding the norm into the product (norm = 1 above) is faster than a norm kernel before it.
int sp_fused_norm_pays(int T, int N, int K);
// What the tiled product for many tokens would do with T x N x K, without running anything: kind 0 store,
// 1 accumulate, 2 gated (N = 2 I), 3 rotating (head size hd); plan = {block rows, block columns, splits of K,
// waves of a block}.
// Returns 1 where that kernel (for kind 3 its rotating epilogue) does not take the product.
int sp_pipe_plan(int kind, int T, int N, int K, int hd, int* plan);
// How that kernel numbers its blocks: tile_of[2 b], tile_of[2 b + 1] = token tile and weight tile of block b (which
// runs on XCD b % 8), -1 for a block with nothing to do; returns the number of blocks.  Runs nothing.
int sp_pipe_tiles(int tiles_t, int tiles_n, int* tile_of, int room);
int sp_gemm_decode(void* stream, const void* x, const float* residual, int norm_w_dtype, const void* norm_w, float eps,
                   const void* w, int bias_dtype, const void* bias, int mode, void* out, int T, int N, int K);
// q, k, v projection (+ bias), rotation of q and k, q to q_out [T, nq * hd], k and v into the paged pools.
// With more than 64 tokens (head sizes that are multiples of 64) the tiled product does it in its epilogue;
// cos_sin (may be null): the table of sp_rope_table for these positions, which saves it the sines and cosines.
int sp_qkv_rope_cache(void* stream, const void* x, const float* residual, int norm_w_dtype, const void* norm_w,
                      float eps, const void* w, int bias_dtype, const void* bias, void* q_out,
                      const int32_t* positions, const float* inv_freq, int rotary_dim, const int32_t* slot_mapping,
                      void* k_pool, void* v_pool, int T, int K, int nq, int nkv, int hd, int page_size,
                      const float* cos_sin, int pairing);
// out [T][half][2] = (cosine, sine) of positions[t] * inv_freq[d]: the same for every layer of a step.
// Both times `magnitude`; with inv_freq_tail (what float32 lost of the exact table, may be null) angles in float64.
int sp_rope_table(void* stream, const int32_t* positions, const float* inv_freq, const float* inv_freq_tail, int half,
                  float magnitude, float* out, int T);
// x[i] *= factor, float32
int sp_scale(void* stream, float* x, float factor, long long n);
// residual [T, H] += mult_a * scale_a[c] * a[t, c] (+ mult_b * scale_b[c] * b[t, c] where b is given); a, b float32.
int sp_scaled_add(void* stream, float* residual, const float* a, int scale_dtype, const void* scale_a, float mult_a,
                  const float* b, const void* scale_b, float mult_b, int T, int H);
// x [T, heads, width] *= sigmoid(gate[t * gate_stride + head])
int sp_head_gate(void* stream, int dtype, void* x, const void* gate, long long gate_stride, int T, int heads, int width);
// out [T, I] = act(x . w[:I]^T, x . w[I:]^T) (times sigmoid(row_gate[t * row_gate_stride]) where row_gate, float32, is given)
int sp_gate_up_silu(void* stream, const void* x, const float* residual, int norm_w_dtype, const void* norm_w, float eps,
                    const void* w, void* out, int T, int I, int K, int activation, float limit, const float* row_gate,
                    long long row_gate_stride);

// Rotates q and k heads of qkv[T, (nq + 2 nkv) * hd] in place (neox pairing, angle = position *
// inv_freq[d]) and writes k and v of every token into the paged pools at slot_mapping[t]
// (= page * page_size + offset; negative: not written).  nkv == 0: only q is rotated.
// The key pool is [pages][nkv][page_size][hd], the value pool [pages][nkv][hd][page_size], of `dtype`.
int sp_rope_cache(void* stream, int dtype, void* qkv, const int32_t* positions, const float* inv_freq,
                  const float* inv_freq_tail, int rotary_dim, const int32_t* slot_mapping, void* k_pool, void* v_pool, int T, int nq,
                  int nkv, int hd, int page_size, int num_pages, int pairing);

// Causal attention of a mixed batch over the paged pools.
// q: [T, q_stride] (head h at column h * hd), out: [T, nq * hd].
// Sequence s owns tokens q_start[s] .. q_start[s] + q_len[s]; their positions end at ctx_len[s] - 1.
// sp_attention_plan tells how the caller must list the work: tiles [n_tiles][2] = (sequence, first
// query of the tile within the sequence's tokens) of plan[0] queries each, over every sequence
// (plan[1] == 1) or over the sequences with more than one query only, the others being listed in
// decode_seqs (plan[1] == 0; a null decode_seqs stands for sequences 0 .. n_decode - 1, each of one query, so that
// q_start[s] == s, which saves the kernels two dependent reads).  max_decode_ctx: largest ctx_len among decode_seqs; max_tile_ctx: largest
// ctx_len among the sequences of the tile list (it only guides how a long walk over the keys is shared out
// between blocks: a smaller value than the truth costs time, not correctness); mean_tile_walk: the mean over
// the tiles of the keys a tile walks (likewise a hint, 0 if unknown: where the longest walk is much longer than
// the mean, as in a prompt's first portion, a block takes a long and a short tile).
// window <= 0: all keys; else keys with position - key < window.
// workspace: sp_attention_workspace_floats(...) floats of scratch for partial results.
int sp_attention_plan(int dtype, int hd, int page_size, int nq, int nkv, int kernel_kind, int* plan);
int64_t sp_attention_workspace_floats(int dtype, int hd, int page_size, int nq, int nkv, int kernel_kind,
                                      int n_decode, int max_decode_ctx, int n_tiles, int max_tile_ctx);
// scores: what stands between q . k and the softmax, numbered like the variants above: 0 = the scaled product and
// nothing else; 1 = the scaled product s squashed to softcap * tanh(s / softcap).  sinks (null: none): one float per
// query head whose exponential joins the softmax's denominator: a term without key or value, neither scaled nor
// capped.  mask_chunk > 0: a query sees only the keys of its own block of mask_chunk positions, counted from
// position 0 of the sequence (beside the window, if both are given).
int sp_attention(void* stream, int dtype, const void* q, int q_stride, const void* k_pool,
                 const void* v_pool, const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                 const int32_t* q_len, const int32_t* ctx_len, const int32_t* tiles, int n_tiles, int tile_q,
                 int max_tile_ctx, int mean_tile_walk, const int32_t* decode_seqs, int n_decode, int max_decode_ctx,
                 float* workspace, int64_t workspace_floats, void* out, int nq, int nkv, int hd, int page_size,
                 int num_pages, int window, float scale, int kernel_kind, int scores, float softcap, const float* sinks,
                 int mask_chunk, int keep_first);
// keep_first > 0: a sequence's first keep_first keys stay visible to every later query beside its window (kernel_kind 2 only).

// A step of one-query sequences only (bfloat16): attention with the output projection folded into the merge
// of the key chunks: residual[q_start[seq], :] += attention(seq) . w_o^T with w_o [hidden, nq * hd] bfloat16
// and residual float32 [rows, hidden].  sp_attention_decode_project_takes says whether a step is taken
// (several chunks of keys, at most 64 sequences, a narrow model); the workspace is sp_attention's for the step.
int sp_attention_decode_project_takes(int hd, int page_size, int nq, int nkv, int n_decode, int max_decode_ctx,
                                      int hidden);
int sp_attention_decode_project(void* stream, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                                const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                                const int32_t* ctx_len, const int32_t* decode_seqs, int n_decode, int max_decode_ctx,
                                float* workspace, int64_t workspace_floats, const void* w_o, float* residual,
                                int hidden, int nq, int nkv, int hd, int page_size, int num_pages, int window,
                                float scale, int scores, float softcap, const float* sinks, int mask_chunk);

// out[t, i] = act(gu[t, i], gu[t, I + i]) (times sigmoid(row_gate[t * row_gate_stride]) where row_gate, float32, is given)
int sp_silu_mul(void* stream, int dtype, const void* gu, void* out, int T, int I, int activation, float limit,
                const float* row_gate, long long row_gate_stride);

// Between the q/k/v projection and attention where keys and values differ in width (both are kept `width` wide, zeros
// behind) or q and k are normed as whole rows.  proj [T, stride] holds q (nq * dim), k (nkv * dim), v (nkv * vdim).
// q_norm / k_norm (both or neither): RMS norm over the whole q row and the whole k row times these weights, eps inside
// the root.  The first rotary_dim numbers of every q and k head turn (d with d + rotary_dim / 2) by positions *
// inv_freq (+ inv_freq_tail: in float64).  blend (one number lambda of `dtype`): v <- (1 - lambda) v + lambda first[t];
// keep_first: first[t] <- v instead.  q to q_out [T, nq * width]; k and v into the pools at slot_mapping (null or
// negative: not cached), keys [pages][nkv][page][width], values [pages][nkv][width][page].  Cosines and sines are
// multiplied by `magnitude`; with head_norm every q and k head is divided, after it has turned, by its root mean
// square over dim (eps inside the root, no weight).
int sp_qkv_prepare(void* stream, int dtype, const void* proj, long long stride, int nq, int nkv, int dim, int vdim, int width,
                   const void* q_norm, const void* k_norm, float eps, const int32_t* positions, const float* inv_freq,
                   const float* inv_freq_tail, int rotary_dim, const void* blend, void* first, int keep_first,
                   const int32_t* slot_mapping, void* k_pool, void* v_pool, int page_size, int num_pages, void* q_out, int T, float magnitude, int head_norm);

// dst (dst_dtype) = src (src_dtype), n elements

// tokens[i] = previous[source[i]] for every i < n with source[i] >= 0 (others are left as they are):
// The float32 path's decode-sized products (up to 16 tokens, everything float32) with neighbouring work folded in.
// Activations are x [T, K], or rmsnorm(x) * norm_w computed inside the kernel where norm_w [K] is given.
//   sp_gate_up_silu_f32:   out[T, I] = act(a . w[:I]^T) * (a . w[I:]^T)
//   sp_qkv_rope_cache_f32: q, k, v = a . w^T + bias; q and k heads turned whole by positions * inv_freq (angles
//                          in float64 where inv_freq_tail, the float64 table minus inv_freq, is given); q to
//                          q_out [T, nq * hd], k and v into the paged pools at slot_mapping.  Head sizes in 16s.
int sp_gate_up_silu_f32_takes(int T, int I, int K);
int sp_gate_up_silu_f32(void* stream, const float* x, const float* norm_w, float eps, const float* w, float* out,
                        int T, int I, int K, int activation, float limit, const float* row_gate, long long row_gate_stride);
int sp_qkv_rope_cache_f32_takes(int T, int K, int nq, int nkv, int hd, int rotary_dim, int pairing);
int sp_qkv_rope_cache_f32(void* stream, const float* x, const float* norm_w, float eps, const float* w, int bias_dtype,
                          const void* bias, float* q_out, const int32_t* positions, const float* inv_freq,
                          const float* inv_freq_tail, int rotary_dim, const int32_t* slot_mapping, float* k_pool,
                          float* v_pool, int T, int K, int nq, int nkv, int hd, int page_size, int num_pages, int pairing);

// dst[i] = a seeded random value, a function of (key, first + i) alone: the sum of twelve 16-bit fields of three
// 64-bit hashes, centred, times scale (+ offset if add_offset): near normal with deviation 65536 * scale.
// weights/random_init.py computes the same numbers on the host.
int sp_random_fill(void* stream, int dtype, void* dst, int64_t n, uint64_t key, int64_t first, float scale,
                   float offset, int add_offset);

// feeds tokens sampled by a step that the host has not read yet into the next step.  previous holds at
// least max(source) + 1 entries; a value outside [0, vocab) is replaced by 0.
int sp_feed_tokens(void* stream, int32_t* tokens, const int32_t* previous, const int32_t* source, int n, int vocab);

// Greedy / temperature sampling of R rows of float32 logits [R, V].
// temperature[r] == 0: lowest index of the maximum.  Else argmax of logits / temperature + Gumbel noise
// from a counter generator keyed by (seed[r], counter[r], column).
// out[r] = token, or -1 if a logit of the row is not finite.  workspace: R * 2 * blocks_per_row floats.
int sp_sample(void* stream, const float* logits, const float* temperature, const int64_t* seed,
              const int32_t* counter, int32_t* out, float* workspace, int R, int V);
int sp_sample_workspace_floats(int R, int V);

// sp_sample for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The partial results of the first
// stage go to a device array of the library's own (sp_sample_static_max_floats() floats, 256 KiB, one copy on
// every GPU the library is used on, kept until the process ends) instead of a workspace; the call allocates and
// frees nothing.  Sizes whose partial results (sp_sample_workspace_floats(R, V)) do not fit are refused.  The
// device of `stream` must be the current device.  All calls on one GPU share that GPU's array: calls whose
// kernels may overlap (different streams, no ordering between them) race; calls on one stream do not.  What an
// earlier call left in the array is never read.
int sp_sample_static(void* stream, const float* logits, const float* temperature, const int64_t* seed,
                     const int32_t* counter, int32_t* out, int R, int V);
int sp_sample_static_max_floats();

// Layer norm: out[r, :] = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w (+ b where b is given, of w's dtype),
// x float32 [*, H], rows as in sp_rmsnorm.  With w2 and out2 (both or neither; b2 optional) the normalised row is also
// written times a second weight.
int sp_layernorm(void* stream, const float* x, const int32_t* rows, int w_dtype, const void* w, const void* w2,
                 const void* b, const void* b2, float eps, int out_dtype, void* out, void* out2, int R, int H);

// residual[t, :] = table[tokens[t], :] + pairs[row, :] with row = (previous * mul_prev + tokens[t] * mul_cur) mod buckets,
// and row `buckets` (the table's last) at position 0.  The token before a step's first token of a sequence is read
// from last_token[state_slots[seq]] (int32, one entry per state slot), where the step's last token of the sequence
// is left for the next step.
int sp_embed_bigram(void* stream, int table_dtype, const void* table, const void* pairs, const int32_t* tokens,
                    const int32_t* positions, const int32_t* q_start, const int32_t* q_len, const int32_t* seq_of_token,
                    const int32_t* state_slots, int32_t* last_token, float* residual, int T, int H, int V,
                    long long buckets, long long mul_prev, long long mul_cur);

// Attention over a latent, between the input projections and the attention kernel.  A row of proj holds per head
// [dim unrotated, rot rotated] query numbers from column q_off on, and at dkv_off the latent (rank numbers) and
// one rotated key part (rot numbers).  Writes, per token: the RMS-normed latent and the turned key part as the key
// [rank + rot] of the one key/value head at slot_mapping[t] (null: nothing is cached), the latent as the value
// (the value pool's last rot columns are left alone), and every head's turned query part into
// q_out[t, head, rank : rank + rot] (rows of heads * (rank + rot)).  The first rot_dims numbers of a rotated part
// turn, (2i, 2i + 1) together, by positions[t] * freq[i] with cosine and sine times `magnitude`; exact != 0: the
// angle and its cosine and sine in float64.
int sp_latent_prepare(void* stream, int dtype, const void* proj, int proj_stride, int q_off, int heads, int dim, int rot,
                      int dkv_off, int rank, int norm_w_dtype, const void* norm_w, float eps, const int32_t* positions,
                      const double* freq, int rot_dims, float magnitude, int exact, const int32_t* slot_mapping,
                      void* k_pool, void* v_pool, int page_size, int num_pages, void* q_out, int T);

// Per-head products: out[t, h * out_head_stride + n] = sum_k a[t, h * a_head_stride + k] * w[h][n][k]
// (w [heads, N, K]; rows of a and out are a_stride and out_stride apart; all three of `dtype`), times
// sigmoid(gate[t * gate_stride + h]) where gate is given.
int sp_head_gemm(void* stream, int dtype, const void* a, long long a_stride, long long a_head_stride, const void* w,
                 void* out, long long out_stride, long long out_head_stride, const void* gate, long long gate_stride,
                 int T, int heads, int N, int K);

// A feed-forward with experts.  sp_route_topk: ids, weights [T, top] = the `top` largest of each token's `experts`
// float32 logits (falling, the lowest index wins a tie) and the softmax over those alone.  sp_route_sort orders the
// T * top pairs by expert: row_of_pair and its inverse pair_of_row, and tiles [n][3] = (expert, first row, rows) of at
// most tile_rows rows with n in *n_tiles (at most sp_route_max_tiles(pairs, experts, tile_rows)).  sp_expert_gate_up:
// out[row, :] = act(x[token] . w[e][:inner]^T) * (x[token] . w[e][inner:]^T) for the rows of every tile (token =
// pair_of_row[row] / top; w [experts, 2 inner, K]).  sp_expert_down: out[row, :] = act[row] . w[e]^T in float32
// (w [experts, hidden, inner]).  sp_route_combine: residual[t] += sum_k weights[t, k] * y[row_of_pair[t * top + k]].
// sp_group_tile_rows: the tile_rows to cut the list for: 128 where the `groups` own `rows` rows of which a group has
// at least 128 on average and the matrix-core kernels take the operands (`dtype` bfloat16, K in eights), else 64.
// The float32-arithmetic kernel takes lists cut for 64 only.
int sp_group_tile_rows(int dtype, long long rows, int groups, int K);
int sp_route_topk(void* stream, const float* logits, int32_t* ids, float* weights, int T, int experts, int top);
int sp_route_max_tiles(int pairs, int experts, int tile_rows);
int sp_route_sort(void* stream, const int32_t* ids, int pairs, int experts, int tile_rows, int32_t* row_of_pair,
                  int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles);
int sp_expert_gate_up(void* stream, int dtype, const void* x, const void* w, const int32_t* tiles, const int32_t* n_tiles,
                      int max_tiles, int tile_rows, const int32_t* pair_of_row, int top, void* out, int T, int experts,
                      int inner, int K, int activation, float limit);
int sp_expert_down(void* stream, int dtype, const void* act, const void* w, const int32_t* tiles, const int32_t* n_tiles,
                   int max_tiles, int tile_rows, float* out, int rows, int experts, int hidden, int inner);
// sp_route: sp_route_topk and sp_route_sort in one call (one launch up to 256 tokens).
int sp_route(void* stream, const float* logits, int32_t* ids, float* weights, int T, int experts, int top, int tile_rows,
             int32_t* row_of_pair, int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles);
int sp_route_combine(void* stream, const float* y, const int32_t* row_of_pair, const float* weights, int top,
                     float* residual, int T, int H);
// sp_route whose weights are the sigmoid of each chosen logit, not renormalised.  (sp_route_combine with null weights adds
// the rows as they are.)
int sp_route_sigmoid(void* stream, const float* logits, int32_t* ids, float* weights, int T, int experts, int top, int tile_rows,
                     int32_t* row_of_pair, int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles);
// sp_route with another rule of choice: scores = the softmax over all `outputs` logits of a token (rows `stride`
// apart); the choice goes by score + correction[e] (null: none) and only among the outputs of the `keep` of `groups`
// equal groups of neighbours whose best such sum is largest (the lower index wins every tie); weights = the chosen
// outputs' scores times `scale`.  Outputs from `real` on have no weights of their own (they return the token's input):
// they get rows but no tiles.  Up to 256 outputs.  sp_route_combine_identity is the weighted sum that goes with it: a
// choice whose id is `real` or more adds weight * x[t] (x [T, H] of x_dtype) instead of an output row.
int sp_route_scored(void* stream, const float* logits, long long stride, const float* correction, int groups, int keep,
                    float scale, int32_t* ids, float* weights, int T, int outputs, int real, int top, int tile_rows,
                    int32_t* row_of_pair, int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles);
int sp_route_combine_identity(void* stream, const float* y, const int32_t* row_of_pair, const float* weights, int top,
                              const int32_t* ids, int x_dtype, const void* x, int real, float* residual, int T, int H);

// Probes for the benchmark's report, not used by the engine: a kernel that only reads `bytes` of `data` (16-byte
// loads from `blocks` blocks of 256 threads), and one that only multiplies on the matrix cores (`blocks` blocks of four waves,
// `iterations` x 4 independent 32x32x16 bfloat16 products a wave; *flops receives the operations of one launch).
int sp_probe_read(void* stream, const void* data, int64_t bytes, int blocks, float* sink);
int sp_probe_mfma(void* stream, int blocks, int iterations, float* sink, double* flops);
// A gated linear recurrence over `width` channels behind a causal convolution of `taps` taps per channel.
// proj [T, stride] holds two branches of `width` numbers (biases added): at y_off the gate branch before its activation,
// at x_off the convolution's input.  u = conv(x) (conv_w [width, taps], last column the current token's; inputs before a
// request's first token are zeros); the channels fall into `blocks` equal parts, part b's gates are
// r = sigmoid(wa[b] u_b + ba[b]), i = sigmoid(wi[b] u_b + bi[b]) with the matrices INPUT-major ([blocks, in, out]);
// a = exp(-8 r softplus(lam)), S <- a S + sqrt(1 - a^2) i u per token, out [T, width] = S * gelu_tanh(y).
// state [slots, width] and tail [slots, taps - 1, width] (the last inputs of the convolution, oldest first; null for one
// tap) are float32 rows indexed by state_slots[request]; decay and drive are float32 scratch [T, width].
int sp_rglru_takes(int width, int blocks, int taps);
int sp_rglru(void* stream, int dtype, const void* proj, long long stride, int y_off, int x_off, int width, int blocks, int taps,
             const void* conv_w, const void* conv_b, const void* wa, const void* ba, const void* wi, const void* bi,
             const void* lam, const int32_t* q_start, const int32_t* q_len, const int32_t* seq_of_token,
             const int32_t* state_slots, float* state, float* tail, float* decay, float* drive, void* out, int T, int n_seqs,
             int max_q_len, float* carry);
// max_q_len: the most tokens one request brings to the step; carry: float32 scratch of sp_rglru_carry_floats numbers (null
// or a short longest portion: every request's tokens are walked in one go, else in chunks side by side).
long long sp_rglru_carry_floats(int width, int n_seqs, int max_q_len, int T);

// Retention: per head S <- decay[h] S + k v^T, o = S^T q, with q and k turned by the angles of cos_sin ([T, rotary_dim / 2, 2]
// of sp_rope_table: the first rotary_dim numbers of a head, d with d + rotary_dim / 2) and k times dim^(-1/2); o is divided
// by its root mean square over vdim (eps inside the root) and multiplied by silu(gate).  proj [T, stride] holds q, k
// (heads * dim), v and the gate (heads * vdim) at their offsets; state float32 [slots, heads, dim, vdim]; out [T, heads * vdim].
int sp_retention_takes(int dim, int vdim);
int sp_retention(void* stream, int dtype, const void* proj, long long stride, int q_off, int k_off, int v_off, int g_off, int heads,
                 int dim, int vdim, int rotary_dim, const float* cos_sin, const float* decay, float eps, const int32_t* q_start,
                 const int32_t* q_len, const int32_t* state_slots, float* state, void* out, int T, int n_seqs, int max_q_len,
                 float* scratch);
// max_q_len, scratch: as for sp_rglru, with sp_retention_scratch_floats numbers.
long long sp_retention_scratch_floats(int heads, int dim, int vdim, int n_seqs, int max_q_len, int T);

// ---- short causal convolutions, state-space scans and what goes with them (ssm.hip) ----
// y[t, c] = act(bias[c] + sum_j w[c, j] x[t - taps + 1 + j, c]) (+ x[t, c] with add_input), a causal convolution over
// time per channel within each request; inputs before a request's share of the step come from its state rows
// [slots, taps - 1, channels] (float32, oldest first; zeros in a fresh slot), which are left holding the request's last
// taps - 1 inputs.  x [T, x_stride] from column x_off on, out [T, out_stride] from out_off on, both of `dtype`, not the
// same memory; w TAP-major [taps, channels] and bias (may be null) of w_dtype.  act 0: none, 1: SiLU.  taps 1: no state.
// max_q_len: the most tokens one request brings to the step (0: unknown); where it is 1, one launch does it all.
int sp_short_conv(void* stream, int dtype, const void* x, long long x_stride, int x_off, int channels, int taps, int w_dtype,
                  const void* w, const void* bias, int act, int add_input, void* out, long long out_stride, int out_off,
                  const int32_t* q_start, const int32_t* q_len, const int32_t* seq_of_token, const int32_t* state_slots,
                  float* state, int T, int n_seqs, int max_q_len);
// out [T, parts * size] = x / sqrt(mean over each part of x^2 + eps) * w, every row in `parts` equal parts, x float32.
int sp_group_rmsnorm(void* stream, const float* x, int w_dtype, const void* w, float eps, int out_dtype, void* out, int T,
                     int parts, int size);
// In place on n numbers of `dtype`: kind 0 = x * Phi(x), the exact (erf) GELU.
int sp_activation(void* stream, int dtype, void* x, long long n, int kind);
// out[p, :] = x[p / top, :] * weights[p]   (p < T * top; x, out of `dtype` [.., H]; weights float32)
int sp_scale_rows(void* stream, int dtype, const void* x, const float* weights, int top, void* out, int T, int H);
// State-space duality scan (Mamba-2).  Per head n (group n / (heads / groups)) and token t of a request:
//   d = softplus(dt[t, n] + dt_bias[n]),  S <- exp(-exp(a_log[n]) d) S + d B_t u_t^T,  y_t = S^T C_t + skip[n] u_t,
// and out[t] = y_t * silu(z_t), float32 [T, heads * vdim].  z and dt are columns of proj [T, proj_stride] (z_off, dt_off);
// u (heads * vdim), B and C (groups * state each) are the columns of xbc [T, xbc_stride] in that order, of `dtype`.
// state float32 [slots, heads, state, vdim].  dt_bias, a_log, skip float32 [heads].  state up to 256.
int sp_ssd_scan(void* stream, int dtype, const void* proj, long long proj_stride, int z_off, int dt_off, const void* xbc,
                long long xbc_stride, int heads, int vdim, int state_size, int groups, const float* dt_bias, const float* a_log,
                const float* skip, const int32_t* q_start, const int32_t* q_len, const int32_t* state_slots, float* state,
                float* out, int T, int n_seqs, int max_q_len, float* scratch);
// max_q_len: the most tokens one request brings to the step; scratch: float32 scratch of sp_ssd_scan_scratch_floats numbers
// (null, or a short longest portion: every request's tokens are walked in one go, else in chunks side by side).
long long sp_ssd_scan_scratch_floats(int heads, int vdim, int state_size, int n_seqs, int max_q_len);
// Selective scan (Mamba).  Per channel c and token t: d = softplus(dt[t, c]) (dt float32 [T, inner], bias included),
//   S[c, :] <- exp(d a[c, :]) S[c, :] + d u[t, c] B_t,  y = S[c, :] . C_t + skip[c] u[t, c],  out[t, c] = y * silu(z[t, c]).
// u [T, u_stride] from u_off, z likewise, B and C (state numbers each) the columns of bc [T, bc_stride] from bc_off on, all
// of `dtype`; a float32 [inner, state] (negative), skip float32 [inner]; state float32 [slots, inner, state]; out of
// `dtype` [T, inner].  state up to 256.
int sp_selective_scan(void* stream, int dtype, const void* u, long long u_stride, int u_off, const void* z, long long z_stride,
                      int z_off, const float* dt, const void* bc, long long bc_stride, int bc_off, int inner, int state_size,
                      const float* a, const float* skip, const int32_t* q_start, const int32_t* q_len,
                      const int32_t* state_slots, float* state, void* out, int T, int n_seqs, int max_q_len, float* scratch);
// max_q_len, scratch: as for sp_ssd_scan, with sp_selective_scan_scratch_floats numbers.
long long sp_selective_scan_scratch_floats(int inner, int state_size, int n_seqs, int max_q_len);
// Queries and keys of attention whose heads' weights are mixed after the softmax.  qk [T, (nq + nkv) * dim] of `dtype`
// holds q then k.  Every head is divided by its root mean square (eps inside the root) and multiplied by q_norm or k_norm
// (dim numbers of w_dtype), then the first rotary_dim numbers turn, 2i with 2i + 1, by positions[t] * freq[i] (float64
// table; the angle is float64 for float32 storage, float32 otherwise).  The values are the keys as they came in.  For the
// attention kernels, which tie a value head to a key head, every (query head g, value head c) pair becomes a head of its
// own: query row [(kv(g) * nkv + c) * (nq / nkv) + g % (nq / nkv)] = q_g, key head [a * nkv + c] = k_a, value head
// [a * nkv + c] = v_c, at `width` numbers a head, zeros behind dim.  Keys and values go into the pools (nkv * nkv heads) at
// slot_mapping[t] (negative: not written), queries to q_out [T, nq * nkv * width].
int sp_qk_cross_prepare(void* stream, int dtype, const void* qk, int nq, int nkv, int dim, int width, int w_dtype,
                        const void* q_norm, const void* k_norm, float eps, const int32_t* positions, const double* freq,
                        int rotary_dim, const int32_t* slot_mapping, void* q_out, void* k_pool, void* v_pool, int page_size,
                        int T);
// out[t, h, :dim] = sum_g talk[h, g] * o[t, (kv(g) * nkv + kv(h)) * (nq / nkv) + g % (nq / nkv), :dim], o [T, nq * nkv * width]:
// the outputs of the heads made by sp_qk_cross_prepare, mixed by talk (float32 [nq, nq]).  out [T, nq * dim], both `dtype`.
int sp_head_mix(void* stream, int dtype, const void* o, const float* talk, int nq, int nkv, int dim, int width, void* out,
                int T);
}
