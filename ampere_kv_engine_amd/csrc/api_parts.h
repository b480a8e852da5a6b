// C entry points of the second kernel library (`libakv_parts.so`): the token-wise kernels, mixers and routed
// feed-forward of designs that keep their residual sum and norms in float32 throughout.  Conventions as in api.h:
// every function enqueues on `stream` and returns 0, a hipError_t of the launch, -1 for an unknown dtype code or -2 for
// sizes the kernel does not take.  dtype codes: 0 float32, 1 bfloat16.  Shapes are checked by the caller on the host.
#pragma once

#include <hip/hip_runtime.h>

extern "C" {

// ---- token-wise (tokenwise_f32.hip) ---------------------------------------------------------------------------------
// out[n] = table[id] + pairs[row], row = (previous id * mul_prev + id * mul_cur) mod buckets, or `buckets` for a
// request's first token.  The previous id of a portion's first token is the word `fed` of the request's slot.
int akv_embed_pairs(const int* ids, const void* table, const void* pairs, int dtype, float* out, int tokens, int hidden,
                    int vocab, long buckets, long mul_prev, long mul_cur, const int* seq_of_token, const int* q_start,
                    const int* positions, const int* seq_slots, int* slot_words, hipStream_t stream);
// word `fed` of every request's slot = the id of the last token it brought in this step
int akv_note_fed_tokens(const int* ids, const int* q_start, const int* seq_slots, int* slot_words, int seqs,
                        hipStream_t stream);
// stream [tokens, hidden] float32.  With `delta` (dtype): stream += delta / rms(delta) * post_weight (or += delta where
// post_weight is null: stream += delta_scale * delta).  With `offset` [hidden]: stream += offset, every row, after the
// branch.  With `out` (dtype): out = stream / rms(stream) * pre_weight, rounded once.  With `delta2` (dtype; only beside a
// `delta` that is not normed): stream += delta_scale * (delta + delta2) - two branches that read the same input.
int akv_norm_add_norm(float* stream_buf, const void* delta, const float* post_weight, float post_eps,
                      const float* pre_weight, float pre_eps, void* out, int dtype, int tokens, int hidden,
                      float delta_scale, const float* offset, const void* delta2, hipStream_t stream);
// out[n] = table[id] (with `accumulate`: out[n] += table[id]), float32; an id of -1: the token chosen last for the row's
// request, where the slot words are given
int akv_embed_rows(const int* ids, const void* table, int dtype, float* out, int tokens, int hidden, int vocab, int accumulate,
                   const int* seq_of_token, const int* seq_slots, const int* slot_words, hipStream_t stream);
// x [tokens, width] (x_dtype: float32 or `dtype`) at x_stride per token -> out (dtype) at out_stride per token =
// x / rms(x over the whole row) * weight (where `normed`; `weight` may be null) * act(gates[t * gate_stride + i]) * out_scale;
// gate_act 0: no gate, 1: sigmoid, 2: silu
int akv_norm_gate_rows(const void* x, int x_dtype, long x_stride, int width, int normed, const float* weight, float eps,
                       const void* gates, long gate_stride, int gate_act, void* out, int dtype, long out_stride,
                       float out_scale, long tokens, hipStream_t stream);
// out[n] = table[id] / rms(table[id]) * weight: the start of a residual sum that is normed before the first layer (an id
// of -1: the token chosen last for the row's request, where the slot words are given)
int akv_embed_normed(const int* ids, const void* table, int dtype, const float* weight, float eps, float* out, int tokens,
                     int hidden, int vocab, const int* seq_of_token, const int* seq_slots, const int* slot_words,
                     hipStream_t stream);
// out [tokens, inter] = act(gate_up[:, :inter]) * gate_up[:, inter:]; activation 0: silu, 1: the tanh form of gelu
int akv_gated_activation(const void* gate_up, void* out, int dtype, long tokens, int inter, int activation,
                         hipStream_t stream);
// maps [tokens, heads, 2, vdim] -> out [tokens, heads, vdim] = (a1 - lambda[0] a2) / rms(.) * after *
// sigmoid(gates[t * gate_stride + gate_at + h * vdim + i])
int akv_difference_norm_gate(const void* maps, const float* lambda, float eps, float after, const void* gates,
                             long gate_stride, long gate_at, void* out, int dtype, long tokens, int heads, int vdim,
                             hipStream_t stream);

// out = a * scale_a + b * scale_b (float32 arithmetic, one rounding)
int akv_scaled_sum(const void* a, float scale_a, const void* b, float scale_b, void* out, int dtype, long count,
                   hipStream_t stream);

// ---- attention with unit-normed queries and keys, softcap, chunks, sink and a gate per head (gated_attention.hip) ------
// projected [tokens, stride]: rows [q (q_heads x dim) | k (kv_heads x dim) | v (kv_heads x vdim) | ...].  Queries divided
// by their root mean square per head (where `normed`) go to q_out [tokens, q_heads, dim]; with `slot_map` the keys, the
// same way, and the values go to the token's slot of the pages: keys [pages, kv_heads, page, dim], values [pages,
// kv_heads, vdim, page].
// `maps` > 1: a head's queries and keys are `maps` vectors of `dim` side by side (rows [q (q_heads x maps x dim) | k (kv_heads
// x maps x dim) | v]), each normed and rotated for itself; key pages [pages, kv_heads, page, maps x dim].  `table`
// [table_positions, rot_dims / 2, 2] (cos, sin; null: no rotation): a vector's first rot_dims dimensions are rotated by the
// token's position, dimension i with i + rot_dims / 2 (`interleaved`: dimension 2 i with 2 i + 1).  `whole`: the root mean
// square is taken over all query vectors of the token at once, and over all its key vectors.  `q_weight` [q_heads x maps x
// dim], `k_weight` [kv_heads x maps x dim] (float32, may be null): multiplied in after the norm, before the rotation.
int akv_unit_norm_write(const void* projected, long stride, int dtype, long tokens, int q_heads, int kv_heads, int dim,
                        int vdim, float eps, int normed, const int* slot_map, void* k_pages, void* v_pages, int page_size,
                        long num_pages, void* q_out, int maps, const float* table, int table_positions, int rot_dims,
                        const int* positions, const float* q_weight, const float* k_weight, int whole, int interleaved,
                        hipStream_t stream);
// out [tokens, q_heads, vdim].  score = (q . k) * scale, then softcap * tanh(score / softcap) where softcap > 0; a query at
// position p sees the keys j <= p with j > p - window (window > 0; the request's first `keep_first` keys stay visible
// behind the window) and floor(j / chunk) = floor(p / chunk) (chunk > 0);
// with `sink` the softmax's denominator has one more term exp(0); with `gates` head h's output is multiplied by
// sigmoid(gates[t * gate_stride + gate_at + h]).  A token's outputs lie at out + t * out_stride, times out_scale.
// `row_waves` (1 .. 16) waves share a token's head: each takes every row_waves-th tile of 64 keys.  `sink_logits` [q_heads]
// float32 (with `sink`): the extra term is exp(sink_logits[h]).  `maps` > 1: `q_heads` counts query vectors, `maps` a head
// (out [tokens, q_heads, vdim] accordingly); vector v reads vector v % maps of its key head's record and the head's values.
int akv_gated_attention_rows(const void* q, const void* k_pages, const void* v_pages, const void* gates, long gate_stride,
                             int gate_at, const int* seq_of_token, const int* positions, const int* block_table,
                             const int* table_rows, int table_width, void* out, int dtype, long tokens, int q_heads,
                             int kv_heads, int dim, int vdim, int page_size, long num_pages, float scale, float softcap,
                             int chunk, int window, int sink, long out_stride, float out_scale, int row_waves,
                             const float* sink_logits, int maps, int keep_first, hipStream_t stream);

// The same for rows first_row .. tokens - 1 of a bfloat16 step, on the matrix cores: keys and values 32, 64, 128 or 256
// wide, pages of a multiple of 16 tokens (-2 otherwise); a request's rows follow each other in the order of their positions.
int akv_gated_attention_tiles(const void* q, const void* k_pages, const void* v_pages, const void* gates, long gate_stride,
                              int gate_at, const int* seq_of_token, const int* q_start, const int* positions,
                              const int* block_table, const int* table_rows, int table_width, void* out, int first_row,
                              int tokens, int q_heads, int kv_heads, int dim, int vdim, int page_size, long num_pages,
                              float scale, float softcap, int chunk, int window, int sink, long out_stride, float out_scale,
                              const float* sink_logits, int maps, int keep_first, hipStream_t stream);

// ---- mixers with a state of fixed size (recurrent_mixers.hip) ----------------------------------------------------------
// projected [tokens, stride]: rows [q | k (heads x dim each) | v | g (heads x vdim each)].  q and k are rotated over their
// first rot_dims dimensions (pairs i, i + rot_dims / 2; `table` [positions, rot_dims / 2, 2] holds cos and sin), k times
// key_scale; per request and head S [dim, vdim] (at state[slot * state_stride + head * dim * vdim]) <- decay S + k v^T,
// o = S^T q; out [tokens, heads, vdim] (a token's at out + t * out_stride) = o / rms(o) * silu(g) * out_scale.
// `input_act` 1: q, k and v pass silu as they are read.  `raw` [tokens, heads, vdim] float32 (may be null): the outputs o
// are left there as they are and `out` is not written - for a caller that norms and gates all heads together.
int akv_retention(const void* projected, long stride, int dtype, int seqs, int heads, int dim, int vdim, int rot_dims,
                  const float* table, int table_positions, float key_scale, const float* decay, float eps, float* state,
                  long state_stride, const int* q_start, const int* seq_slots, const int* positions, void* out,
                  long out_stride, float out_scale, int input_act, float* raw, hipStream_t stream);
// The same with every request's tokens cut into chunks of `length` that are worked on side by side - sums of k v^T per
// chunk, the states before the chunks one after the other, then every chunk's outputs: `sums` holds 2 * seqs * heads *
// chunks * dim * vdim floats, chunks = the most chunks a request of the step has.
int akv_retention_chunked(const void* projected, long stride, int dtype, int seqs, int heads, int dim, int vdim, int rot_dims,
                          const float* table, int table_positions, float key_scale, const float* decay, float eps,
                          float* state, long state_stride, const int* q_start, const int* seq_slots, const int* positions,
                          void* out, long out_stride, float out_scale, float* sums, int length, int chunks, int input_act,
                          float* raw, hipStream_t stream);
// u [tokens, channels]; gates [tokens, blocks, 2 * channels / blocks] float32 (a block's recurrence-gate logits, then its
// input-gate logits) before their biases `gate_bias` [blocks, 2 * channels / blocks]; a = exp(rate[c] * sigmoid(.));
// S [channels] at the start of a slot's state <- a S + sqrt(1 - a^2) sigmoid(.) u; out = S * gelu_tanh(y), y at
// `y_stride` per token.  A request's tokens are cut into `runs` runs (1 .. 64) whose decays' products and sums
// are folded in the order of the runs.
int akv_gated_linear_scan(const void* u, int dtype, const float* gates, const float* gate_bias, const float* rate,
                          const void* y, long y_stride, int seqs, int channels, int blocks, int runs, float* state,
                          long state_stride, const int* q_start, const int* seq_slots, void* out, hipStream_t stream);

// ---- the gated delta rule with a decay per key channel (delta_rule.hip) ---------------------------------------------------
// conv [tokens, conv_stride]: rows [q (groups x dim) | k (groups x dim) | v (heads x vdim)] after their convolutions and
// activations; head h reads q / k number h / (heads / groups).  q, k -> unit vectors (x / sqrt(sum x^2 + unit_eps)), q times
// q_scale; beta = sigmoid(beta_logits[t * beta_stride + h]); g = exp(-rate[h] * softplus(decay_logits[t, h, d] +
// decay_bias[h, d])).  Per request and head, S [dim, vdim] (in the slot as [heads, vdim, dim] float32):
// S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  out [tokens, heads x vdim] = o / rms(o) * norm_weight[i] *
// sigmoid(gates[t, h, i]).  `workspace`: akv_delta_rule_workspace(...) floats.  `longest`: the most
// tokens a request brings (chooses the walk's tile; the sums are the same either way).
long akv_delta_rule_workspace(int tokens, int heads, int groups, int dim, int vdim);
int akv_delta_rule(const void* conv, long conv_stride, int dtype, const void* beta_logits, long beta_stride,
                   const float* decay_logits, const float* decay_bias, const float* rate, const float* gates,
                   const float* norm_weight, float unit_eps, float norm_eps, float q_scale, float* state, long state_stride,
                   const int* q_start, const int* seq_slots, float* workspace, void* out, int tokens, int seqs, int heads,
                   int groups, int dim, int vdim, int longest, hipStream_t stream);

// ---- attention over a compressed latent (latent_attention.hip) ------------------------------------------------------
// down [tokens, q_rank (+ kv_rank + rot)]: q latent normed into `cq`; with `records`: the kv latent normed and the
// shared key part rotated (first `rot_dims` of its `rot` dimensions) into the token's record [kv_rank + rot].  With
// `latents_t` [pages, kv_rank, page_size] the normed latent is written there too, keys contiguous.  Rotation pairs are
// dimensions (i, i + rot_dims / 2), or (2 i, 2 i + 1) with `interleaved`.  `down_stride`: elements from one token's row of
// `down` to the next (0: the rows hold nothing else).
int akv_latent_encode(const void* down, int dtype, int tokens, int q_rank, int kv_rank, int rot, int rot_dims,
                      const float* q_weight, const float* kv_weight, float eps, const float* table, int table_positions,
                      const int* positions, const int* slot_map, void* cq, void* records, long record_slots,
                      void* latents_t, int page_size, int interleaved, long down_stride, hipStream_t stream);
// q [tokens, heads, dim + rot] -> q_abs[..., at : at + rot] (float32 or bfloat16, row width `width`), rotated by position
int akv_rotate_queries(const void* q, int dtype, long tokens, int heads, int dim, int rot, int rot_dims,
                       const float* table, int table_positions, const int* positions, void* q_abs, int out_dtype,
                       int width, int at, int interleaved, hipStream_t stream);
// y[t, h, j] = sum_i x[t, h, i] * w[h, i, j]   (w [heads, ins, outs]; x and y addressed by token and head strides)
int akv_heads_linear(const void* x, int x_dtype, long x_token_stride, long x_head_stride, const void* w, int w_dtype,
                     void* y, int y_dtype, long y_token_stride, long y_head_stride, int tokens, int heads, int ins,
                     int outs, hipStream_t stream);
// out[t, h, :kv_rank] = softmax over the window of (q_abs[t, h] . record) * scale, times the records' first kv_rank
int akv_latent_attend(const float* q_abs, const void* records, int dtype, const int* seq_of_token, const int* positions,
                      const int* block_table, const int* table_rows, int table_width, float* out, int tokens, int heads,
                      int kv_rank, int width, int page_size, long num_pages, float scale, int window,
                      hipStream_t stream);
// The same on the matrix cores, for bfloat16, heads that are a multiple of 16, records a multiple of 32 wide, latents
// of 128, 256 or 512 and pages of a multiple of 8 tokens (-2 otherwise).  `latents_t` [pages, kv_rank, page]: the
// records' first kv_rank dimensions once more, keys contiguous.  q_abs [tokens, heads, width] and out [tokens, heads,
// kv_rank] are bfloat16.  With `segments` > 1 a token's keys are cut into runs of `segment` keys (a multiple of 32, at
// absolute positions, counted from the run that holds its window's first key; the caller gives as many as the longest
// span needs), a wave each, whose shares meet in `parts` [tokens * heads * segments * (kv_rank + 2)] and are merged.
// `one_request`: every token is of the same request, in the order of their positions - blocks of neighbouring tokens
// then share each step's records through LDS.
int akv_latent_attend_mfma(const void* q_abs, const void* records, const void* latents_t, const int* seq_of_token,
                           const int* positions, const int* block_table, const int* table_rows, int table_width,
                           void* out, int tokens, int heads, int kv_rank, int width, int page_size, long num_pages,
                           float scale, int window, int segment, int segments, float* parts, int one_request,
                           hipStream_t stream);

// ---- selective scan (selective_scan.hip) ----------------------------------------------------------------------------
// x [tokens, channels] at `x_stride` per token; state [slots, state_stride] float32 holds (taps - 1) x channels at
// `conv_at`.  out = silu(conv + bias); akv_conv_taps with `activation` 0: out = conv + bias, 1: silu of it.
int akv_conv_silu(const void* x, long x_stride, int dtype, const void* weight, const void* bias, int w_dtype,
                  const float* state, long state_stride, long conv_at, const int* seq_of_token, const int* q_start,
                  const int* seq_slots, void* out, int tokens, int channels, int taps, hipStream_t stream);
int akv_conv_taps(const void* x, long x_stride, int dtype, const void* weight, const void* bias, int w_dtype,
                  const float* state, long state_stride, long conv_at, const int* seq_of_token, const int* q_start,
                  const int* seq_slots, void* out, int tokens, int channels, int taps, int activation,
                  hipStream_t stream);
int akv_conv_state_update(const void* x, long x_stride, int dtype, float* state, long state_stride, long conv_at,
                          const int* q_start, const int* seq_slots, int seqs, int channels, int taps,
                          hipStream_t stream);
// S [channels, n_state] at the start of a slot's state; dt [tokens, channels] (before softplus, which is taken in
// place), bc = [B | C] float32
int akv_selective_scan(const void* x, int dtype, float* dt, const float* bc, const void* z, long z_stride,
                       const float* a, const float* d, float* state, long state_stride, const int* q_start,
                       const int* seq_slots, void* out, int tokens, int seqs, int channels, int n_state,
                       hipStream_t stream);

// ---- routed feed-forward (routed.hip) -------------------------------------------------------------------------------
// logits [tokens, experts] float32 -> gates [tokens, experts] float32: the softmax score of the chosen experts, 0 elsewhere
int akv_route(const float* logits, float* gates, int tokens, int experts, int top, int groups, int keep,
              hipStream_t stream);
// logits [tokens, scored] -> gates: the `top` largest of the first `experts` logits get the softmax over themselves, the
// other experts 0, every further column its sigmoid.  `law` 1: logits [tokens, experts]; a chosen expert's gate is the
// sigmoid of its own logit, and every further column of gates [tokens, scored] becomes 1
int akv_route_chosen(const float* logits, float* gates, int tokens, int experts, int scored, int top, int law,
                     hipStream_t stream);
// act[t, c] = f(gates[t, e(c)] * up[t, c]) (`inside`) or gates[t, e(c)] * f(up[t, c]); f 0: gelu (erf), 1: gelu (tanh), 2: silu,
// 3: relu squared; e(c) = c / ff below experts * ff, else `experts`
int akv_gate_activation(const void* up, const float* gates, void* act, int dtype, long tokens, int experts, int ff,
                        int columns, int scored, int kind, int inside, hipStream_t stream);
// act[t, c] = gates[t, e(c)] * silu(gate_up[t, c]) * gate_up[t, columns + c]; e(c) = c / ff below experts * ff, else `experts`
int akv_gate_silu_mul(const void* gate_up, const float* gates, void* act, int dtype, long tokens, int experts, int ff,
                      int columns, int scored, hipStream_t stream);
// act[t, e * ff + j] = gates[t, e] * relu(up[t, e * ff + j])^2
int akv_gate_relu_squared(const void* up, const float* gates, void* act, int dtype, long tokens, int experts, int ff,
                          hipStream_t stream);
}
