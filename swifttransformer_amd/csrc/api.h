// C entry points of the kernel library.  Every function returns 0 on success;
// otherwise st_last_error() describes the refusal (bad sizes, unsupported head
// size, ...).  Pointers are device pointers unless noted; `stream` is the HIP
// stream to launch on.  dtype: 0 = float32, 1 = bfloat16 storage.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

extern "C" {

const char* st_last_error();

int st_lookup(void* out_f32, void* out_t, const int* ids, const void* table,
              const int* add_ids, int add_offset, const void* add_table,
              int table_rows, int add_rows, int num_rows, int width, int accumulate, int dtype, hipStream_t stream);

// center != 0: LayerNorm; center == 0: no mean is taken off (root-mean-square norm).
int st_layernorm(void* out_t, void* out_f32, const float* x, const int* rows,
                 const float* gamma, const float* beta, int num_rows, int width,
                 float eps, int center, int dtype, hipStream_t stream);

int st_kv_write(void* k_cache, void* v_cache, int64_t page_stride,
                const void* k_src, const void* v_src, int64_t src_stride,
                const int* token_item, const int* positions,
                const int* block_table, int max_pages, int page_size,
                int num_tokens, int num_kv_heads, int head_dim, int dtype, hipStream_t stream);

int st_cast(void* out, const void* in, int64_t n, int in_dtype, int out_dtype, hipStream_t stream);

// out[r, c] = act(a[r, c]) * (b ? b[r, c] : 1) over rows x width elements; the three row strides
// (in elements) are free, so a and b may be the two halves of one product's output.  `kind` as
// st_gemm's activation.  The reference's counterpart multiplies two whole arrays
// (src/csrc/kernel/fused_activ_multiply.cu:19-36).
int st_activation_multiply(void* out, int64_t out_stride, const void* a, int64_t a_stride,
                           const void* b, int64_t b_stride, int rows, int width, int kind, int dtype,
                           hipStream_t stream);

struct StGemmExtras;
// activation: the function between bias and residual, by number (csrc/activation.h): 0 none,
// 1 ReLU, 2 SiLU, 3 GELU in its tanh form, 4 GELU in its exact (erf) form, 5 the square of ReLU; others are refused.
int st_gemm(void* out, const void* x, const void* w, const float* bias, const float* residual,
            int M, int N, int K, int activation, int dtype, int out_f32, int algo,
            const StGemmExtras* extras, hipStream_t stream);
int st_gemm_path_counts(uint64_t* out, int reset);
int st_gemm_library_rule(int min_rows, int64_t min_weights, int min_depth);
// Which workgroup shapes a product with the norm prologue may take (for measurements and tests):
// bit 1 the wide ones (24 features) at all, bit 2 sixteen waves for them, and 32 features, bit 4
// 32 features tried before 24; 3 is the default.
int st_gemm_wide_workgroups(int mode);
int st_gemm_can_fuse_norm(int M, int N, int K, int dtype);
int st_gemm_wide_offered(int M, int N, int K, int dtype);
int st_gemm_wide_groups();
int st_gemm_can_fuse_merge(int M, int N, int K, int splits, int heads, int head_dim, int dtype);

// window > 0: a row reads the last `window` positions; window < 0: the positions of its own chunk of -window
// positions, chunks counted from the sequence's first position; softcap > 0: scaled scores pass through
// softcap * tanh(score / softcap) before the softmax.  The same for st_attn_prefill.
int st_attn_rows(void* out, float* part_o, float* part_lse, const void* q, int64_t q_stride,
                 const void* k_cache, const void* v_cache, int64_t page_stride,
                 const int* row_ids, const int* token_item, const int* positions,
                 const int* block_table, const float* head_slopes,
                 int max_pages, int page_size, int num_tokens, int num_q_heads,
                 int num_kv_heads, int head_dim, float scale, int window, float softcap, int num_splits,
                 int num_waves, int dtype, hipStream_t stream);

// No counterpart in the reference.  For callers that cannot allocate (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc): st_attn_rows with the key
// split's partial results kept in a static device array of the library (4 MiB per GPU, held
// until the process ends) instead of a workspace argument.  Calls no hipMalloc/hipFree.  Refuses
// num_tokens * num_q_heads * num_splits * (head_dim + 1) floats beyond that size.  Calls that
// overlap on one GPU share the array and race.  st_attn_rows_static_init() resolves the array's
// address on the current device ahead of the first call (the first call does it otherwise).
int st_attn_rows_static_init();
size_t st_attn_rows_static_capacity();
int st_attn_rows_static(void* out, const void* q, int64_t q_stride,
                        const void* k_cache, const void* v_cache, int64_t page_stride,
                        const int* row_ids, const int* token_item, const int* positions,
                        const int* block_table, const float* head_slopes,
                        int max_pages, int page_size, int num_tokens, int num_q_heads,
                        int num_kv_heads, int head_dim, float scale, int window, int num_splits,
                        int num_waves, int dtype, hipStream_t stream);

int st_attn_prefill(void* out, const void* q, int64_t q_stride,
                    const void* k_cache, const void* v_cache, int64_t page_stride,
                    const int* tile_item, const int* tile_q0, int num_tiles,
                    const int* item_tok_off, const int* item_start, const int* item_len,
                    const int* block_table, const float* head_slopes, int max_pages, int page_size,
                    int num_q_heads, int num_kv_heads, int head_dim, float scale, int window, float softcap,
                    int key_split, int tile_rows, int algo, int dtype, hipStream_t stream);

int st_has_attn_prefill();
int st_attn_prefill_tile_rows(int head_dim, int page_size, int max_pages, int num_q_heads, int num_rows, int dtype);

int st_gemm_library_init();
int st_gemm_library_tuning(int on);
int st_gemm_library_allow_workspace(int on);

int st_sample(int* out, const float* logits, int num_rows, int vocab, const float* temperature,
              const uint32_t* seeds, const uint32_t* draws, hipStream_t stream);

float st_hash_uniform(uint32_t seed_lo, uint32_t seed_hi, uint32_t draw, uint32_t v);

// ---- short causal convolution over time, one filter a channel (csrc/token_conv.hip)
// out[t, c] = act((x[t, c] if add_input) + bias[c] + sum_j w[c, j] * x(row of position p_t - taps + 1 + j, c)):
// x rows float or bfloat16 with stride x_stride; rows before the item's first row of this step come from
// state + slot * slot_stride, [taps - 1, channels] floats (the inputs at the last taps - 1 positions
// before it; zeros before the sequence's start).  st_token_conv_state then moves
// the state on by the step's rows.  Rows whose item is -1 are written as zeros.
int st_token_conv(void* out, const void* x, int64_t x_stride, int in_dtype, const float* w, const float* bias,
                  const float* state, int64_t slot_stride, const int* token_item, const int* item_tok_off,
                  const int* item_slot, int num_tokens, int channels, int taps, int add_input, int activation,
                  int out_dtype, hipStream_t stream);
int st_token_conv_state(float* state, int64_t slot_stride, const void* x, int64_t x_stride, int in_dtype,
                        const int* item_len, const int* item_tok_off, const int* item_slot, int num_items,
                        int channels, int taps, hipStream_t stream);

// ---- rotary positions, one-pool page write, two float rows side by side in the storage type (csrc/rotary.hip)
// In place on the rows' queries and keys: the rot_dims coordinates of every head from `offset` on,
// coordinate i paired with i + rot_dims / 2 (interleaved != 0: 2i with 2i + 1), turned by
// positions[t] * freq[i]; cosine and sine times `mult`.
int st_rotary(void* q, int64_t q_stride, int q_heads, void* k, int64_t k_stride, int k_heads, int head_dim,
              int rot_dims, int offset, int interleaved, const float* freq, float mult, const int* positions,
              int num_tokens, int dtype, hipStream_t stream);
// src[t, head, :] -> the token's entry of a pool [pages, heads, page_size, head_dim]; norm != 0: divided
// by its root mean square over head_dim (eps inside the root) on the way.
int st_paged_write(void* cache, int64_t page_stride, const void* src, int64_t src_stride, const int* token_item,
                   const int* positions, const int* block_table, int max_pages, int page_size, int num_tokens,
                   int heads, int head_dim, int norm, float eps, int dtype, hipStream_t stream);
int st_concat_cast(void* out, const float* a, int wa, const float* b, int wb, int num_rows, int dtype,
                   hipStream_t stream);

// ---- attention with heads coupled before the softmax, a sink and a window (csrc/sink_attention.hip)
int64_t st_sink_attention_lds(int heads, int key_dim, int mixed);
int st_sink_attention(void* out, float* part_o, float* part_ml, const void* q, int64_t q_stride,
                      const void* k_cache, int64_t k_page_stride, const void* v_cache, int64_t v_page_stride,
                      const float* mix, const int* token_item, const int* positions, const int* block_table,
                      int max_pages, int page_size, int num_tokens, int heads, int kv_heads, int key_dim,
                      int value_dim, float scale, int window, int keep_first, int sink, int splits, int dtype,
                      hipStream_t stream);

// ---- recurrences with one decay a head and token (csrc/state_scan.hip)
// mode 0: out_a = softplus(raw + bias), out_b = exp(-exp(a_log) * out_a), raw [T, heads];
// mode 1: out_a = sigmoid(raw[:, :heads]), out_b = exp(-exp(a_log) * softplus(raw[:, heads:] + bias)).
int st_recurrence_gates(float* out_a, float* out_b, const float* raw, int64_t raw_stride, const float* a_log,
                        const float* bias, int num_tokens, int heads, int mode, hipStream_t stream);
// x[t, head, :] <- x / sqrt(sum x^2 + eps) * scale, in place on float rows.
int st_unit_norm(float* x, int64_t stride, int num_tokens, int heads, int dim, float eps, float scale,
                 hipStream_t stream);
// mode 0: S <- b S + (a k) v^T, o = S^T q + skip v;  mode 1: S <- b S, u = a (v - S^T k), S <- S + k u^T,
// o = S^T q.  a, b float [T, heads] with rows gate_stride floats apart (0: one row of constants serves
// every token); q, k float rows of qk_heads heads; state [slots](slot_stride) [heads, key_dim, value_dim] float.
int st_state_scan(float* out, const float* q, int64_t q_stride, const float* k, int64_t k_stride, const float* v,
                  int64_t v_stride, const float* gate_a, const float* gate_b, int64_t gate_stride, const float* skip,
                  float* state,
                  int64_t slot_stride, const int* item_len, const int* item_tok_off, const int* item_slot,
                  int num_items, int max_item_rows, int heads, int qk_heads, int key_dim, int value_dim, int mode,
                  hipStream_t stream);
// out = val * rsqrt(mean(val^2) + eps) * gain (* act(gate) unless gate_first) over each of `groups`
// parts of a row, val = o (* act(gate) if gate_first); gain [width], or [groups * width] if gain_per_group;
// act: silu (gate_kind 0) or sigmoid (gate_kind 1).
int st_gated_group_norm(void* out, const float* o, const void* gate, int64_t gate_stride, const float* gain,
                        int num_tokens, int groups, int width, int gain_per_group, int gate_first, int gate_kind,
                        float eps, int dtype, hipStream_t stream);

// ---- retention in chunks (csrc/retention.hip): S <- decay_h S + (key_factor k) v^T, o = S^T q over each item's rows,
// from and back to the item's state slot, as products within chunks of st_retention_chunk_rows(key_dim) rows and a
// carry between them.  q, k float rows [heads * key_dim], v [heads * value_dim]; decay float [heads]; scratch: float
// [scratch_chunks, heads, key_dim, value_dim] with scratch_chunks >= num_rows / chunk rows + num_items.
int st_retention_chunk_rows(int key_dim);
int st_retention_chunks(float* out, const float* q, int64_t q_stride, const float* k, int64_t k_stride, const float* v,
                        int64_t v_stride, const float* decay, float key_factor, float* state, int64_t slot_stride,
                        const int* item_len, const int* item_tok_off, const int* item_slot, int num_items, int num_rows,
                        int heads, int key_dim, int value_dim, float* scratch, int64_t scratch_chunks,
                        hipStream_t stream);

// ---- gated linear attention (csrc/recurrent.hip)
// out = sigmoid(z)^(inv_tau) over n floats (out may be z).
int st_decay_gate(float* out, const float* z, int64_t n, float inv_tau, hipStream_t stream);
// Per item and head, from the state S [key_dim, value_dim] of the item's slot and over its rows in
// order: S = diag(a_t) S + k_t v_t^T, o_t = scale * S^T q_t; the state is stored back.  The key
// channels are dealt to parts of part_dim (4, 8 or 16); part p writes its share of every o_t to
// plane p of o_part [parts, T, heads * value_dim] (planes part_stride floats apart), and the sum
// of the planes is o.  q, k, v: rows of `dtype` with their strides in elements (head h at
// h * key_dim / h * value_dim); a: float [T, heads * key_dim]; state: float [slots, heads, key_dim, value_dim].
int st_gla_scan(float* o_part, int64_t part_stride, int part_dim, const void* q, int64_t q_stride,
                const void* k, int64_t k_stride, const void* v, int64_t v_stride, const float* a,
                float* state, const int* item_len, const int* item_tok_off, const int* item_slot,
                int num_items, int heads, int key_dim, int value_dim, float scale, int dtype, hipStream_t stream);
int st_gla_scan_parts(int key_dim, int part_dim);
// With o the sum of `parts` planes (part_stride floats apart):
// out[t, h, j] = o[t, h, j] * rsqrt(mean_j o[t, h, :]^2 + eps) * gain[j] * silu(g[t, h, j]); g: rows
// of `dtype` with stride g_stride; out: rows of `dtype`, dense.  Up to 256 value channels a head.
int st_gated_head_norm(void* out, const float* o, int parts, int64_t part_stride, const void* g, int64_t g_stride,
                       const float* gain, int num_tokens, int heads, int value_dim, float eps, int dtype,
                       hipStream_t stream);

// ---- latent cache (csrc/latent.hip)
// Row t of x (float, stride x_stride, `rank` values) is normalised, c = x * rsqrt(mean x^2 + eps) *
// gain, and stored as the token's entry of a one-head page pool whose entries are `entry` >= rank
// wide (the rest is cleared): [pages, 1, page_size, entry] of `dtype`.  tail > 0: the row's next `tail`
// values follow the latent in the entry as they are, or, with `freq` [tail / 2], turned by the token's
// position (pairs 2i, 2i + 1; angle position * freq[i]; cosine and sine times tail_mult): a key part that every
// head shares.
int st_latent_write(void* cache, int64_t page_stride, const float* x, int64_t x_stride, const float* gain,
                    const int* token_item, const int* positions, const int* block_table, int max_pages,
                    int page_size, int num_tokens, int rank, int entry, float eps, int tail, const float* freq,
                    float tail_mult, int dtype, hipStream_t stream);

// ---- routed experts (csrc/moe.hip)
// ids[t, j], weights[t, j] (j < top): the experts with the largest logits of row t, largest first,
// the lower index on ties, and their weights: mode 0 the sigmoid of each logit, mode 1 the softmax over
// the chosen logits alone, mode 2 each chosen expert's share of the softmax over all experts, where only the
// experts of the `keep` best of `groups` equal groups of neighbours (a group's rank: its largest logit) can be
// chosen.  Rows whose item is -1 get ids of -1.
int st_moe_route(int* ids, float* weights, const float* logits, const int* token_item, int num_tokens,
                 int experts, int top, int mode, int groups, int keep, hipStream_t stream);
// Sorts the num_pairs = tokens * top (token, choice) pairs by expert into tiles of `tile` (16, 64 or 128)
// places that hold one expert's pairs each: sorted[capacity] (pair index, or -1),
// place_of_pair[num_pairs] (or -1), tile_expert[capacity / tile] (or -1).
// capacity >= round_up(num_pairs, tile) + tile * experts.  The three calls below take the same `tile`.
int st_moe_align(int* sorted, int* place_of_pair, int* tile_expert, const int* ids, int num_pairs,
                 int experts, int capacity, int tile, hipStream_t stream);
// y[place, f] = g * sigmoid(1.702 g) * (u + 1) with g = min(s * (x_t . Wg[e, f]), limit) and
// u = clamp(s * (x_t . Wu[e, f]), -limit, limit), for the pair (t, j) at `place`, e its expert and s
// its weight (style 0); style 1: y[place, f] = silu(x_t . Wg[e, f]) * (x_t . Wu[e, f]), no weight and no
// limit (the weight then multiplies the expert's result, in st_moe_combine).
// x: [T, width]; w_gate, w_up: [experts, inner, width]; y: [capacity, inner].
int st_moe_up(void* y, const void* x, const void* w_gate, const void* w_up, const int* sorted,
              const int* tile_expert, const float* weights, int capacity, int tile, int top, int width, int inner,
              float limit, int style, int dtype, hipStream_t stream);
// pair_out[place, n] = y[place] . Wd[e, n] (top > 1), or, with top == 1, directly
// out[t, n] = residual[t, n] + out_scale * y[place] . Wd[e, n].  w_down: [experts, width, inner].
int st_moe_down(float* out, const float* residual, float* pair_out, const void* y, const void* w_down,
                const int* sorted, const int* tile_expert, int capacity, int tile, int top, int width, int inner,
                float out_scale, int dtype, hipStream_t stream);
// out[t, n] = residual[t, n] + out_scale * sum_j weights[t * top + j] * pair_out[place_of_pair[t * top + j], n]
// (weights null: ones; residual null: zeros)
int st_moe_combine(float* out, const float* residual, const float* pair_out, const int* place_of_pair,
                   const float* weights, int num_tokens, int top, int width, float out_scale, hipStream_t stream);

// ---- float operations on the residual stream (csrc/stream_ops.hip)
// y = tanh(alpha[0] * x[row]) * w + b (b may be null) of every row, or of the rows picked by `rows`
// (negative: skipped); base != null: y += base[row of the result]; out32 (float) and / or out_t (`dtype`).
// w2 != null: out_t receives tanh(alpha2[0] * y) * w2 + b2 instead of y (out32 still y).
int st_dynamic_tanh(void* out_t, float* out32, const float* x, const int* rows, const float* w, const float* b,
                    const float* alpha, const float* base, const float* w2, const float* b2, const float* alpha2,
                    int num_rows, int width, int dtype, hipStream_t stream);
// x[t] += y[t] * rsqrt(mean(y[t]^2) + eps) * w
int st_unit_add(float* x, const float* y, const float* w, int num_rows, int width, float eps, hipStream_t stream);
// out[t] = x[t] (+ first[t]) + vec
int st_row_add(float* out, const float* x, const float* first, const float* vec, int num_rows, int width,
               hipStream_t stream);

// x[t] += unit(P (gelu_tanh(G x[t]) * table[token_ids[t], :dim])) * gain, unit(y) = y * rsqrt(mean(y^2) + eps).
// table rows of `table_stride` elements, w_gate [dim, width], w_proj [width, dim] of `dtype`; x, gain float.
// Rows with token_item[t] < 0 (if given) are left alone; a token outside the table gates with zeros.
int st_token_side(float* x, const int* token_ids, const int* token_item, const void* table, int64_t table_stride,
                  int vocab, const void* w_gate, const void* w_proj, const float* gain, int num_rows, int dim,
                  int width, float eps, int dtype, hipStream_t stream);

// x[i] = cap * tanh(x[i] * scale / cap) over n floats in place (cap <= 0: x[i] * scale).
int st_scale_softcap(float* x, int64_t n, float scale, float cap, hipStream_t stream);

// ---- a residual stream of several copies (csrc/hyper_streams.hip); x float [rows, streams, width]
int st_streams_expand(float* out, const float* x, int num_rows, int streams, int width, hipStream_t stream);
int st_streams_sum(float* out, const float* x, const int* rows, int num_rows, int streams, int width,
                   hipStream_t stream);
int st_streams_read(void* out_t, float* out32, const float* x, const float* a, const float* gain, int num_rows,
                    int streams, int width, float eps, int dtype, hipStream_t stream);
int st_streams_write(float* x, const float* y, const float* mix, const float* b, void* out_t, const float* a2,
                     const float* gain2, int num_rows, int streams, int width, float eps2, int dtype,
                     hipStream_t stream);

// ---- token embedding times a factor plus a row chosen by a hash of the token and the one before (csrc/hashed_embedding.hip)
int st_hashed_embed(float* out, const int* ids, const int* positions, const int* token_item, const int* item_len,
                    const int* item_tok_off, const int* item_slot, int* last_token, const void* table,
                    const void* pairs, int num_tokens, int num_items, int vocab, int buckets, int64_t mul_prev,
                    int64_t mul_cur, float scale, int width, int dtype, hipStream_t stream);

// ---- queries and keys normalised over their whole projection, the keys as projected as values (csrc/tied_attention.hip)
int st_qk_norm_write(void* out_q, void* k_cache, void* v_cache, int64_t page_stride, const float* qk, int64_t stride,
                     const float* gain_q, const float* gain_k, const int* token_item, const int* positions,
                     const int* block_table, int max_pages, int page_size, int num_tokens, int heads, int kv_heads,
                     int head_dim, int head_pad, float eps, int write, int dtype, hipStream_t stream);

// Measurement kernels (csrc/probe.hip): a plain streaming read, and a kernel without work.
int st_probe_read(const void* src, int64_t bytes, void* sink, int workgroups, int pattern, hipStream_t stream);
int st_probe_empty(void* sink, hipStream_t stream);
int st_probe_fill(const void* src, int64_t region, void* sink, int workgroups, int turns, int to_lds,
                  hipStream_t stream);
int st_probe_mfma(void* sink, int workgroups, int rounds, int wide, hipStream_t stream);

}  // extern "C"
