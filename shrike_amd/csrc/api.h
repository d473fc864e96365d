// C entry points of libshrike_hip: thin host launchers around the gfx950
// kernels.  Every pointer is device memory unless said otherwise; `dtype` is
// 0 for float32 and 1 for bfloat16; `stream` is a hipStream_t.  A call returns
// 0 on success; otherwise shk_last_error() describes what was refused and
// nothing was launched.  Shapes are checked on the host before any launch.
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* shk_last_error(void);
int shk_version(void);

// dst[i] = src[i] for i < n, except dst[patch_at + j] = patch[j] for j < patch_n (patch
// may be null with patch_n 0).  src and dst may be device memory or page-locked host
// memory: small index arrays and tokens travel by this kernel, not by the copy engine.
int shk_copy_words(const int32_t* src, int32_t* dst, int n, const int32_t* patch, int patch_at,
                   int patch_n, void* stream);

// dst[r, :] = src[index[r], :] for r < rows: rows of `width` 32-bit words, src rows
// `ld` words apart; the caller promises 0 <= index[r] < src_rows.  index may be
// page-locked host memory.
int shk_gather_rows(const int32_t* src, long long ld, int src_rows, const int32_t* index, int32_t* dst,
                    int rows, int width, void* stream);

// Zeroes `bytes` bytes from dst, which must be 4-byte aligned (a fill kernel:
// it may be recorded into a HIP graph).
int shk_zero_bytes(void* dst, long long bytes, void* stream);

// out[i, :] = float(table[ids[i], :]) * scale; ids must lie in [0, vocab).
int shk_embed(const void* table, int dtype, const int32_t* ids, float* out, int n, int hidden,
              int vocab, float scale, void* stream);

// resid[r, :] += other[r, :] + vec[:] for r < n (float32; other and vec may be null).
int shk_add_rows(float* resid, const float* other, const float* vec, int n, int hidden, void* stream);

// resid[r, :] += d1[r, :] + d2[r, :], and cast[r, :] = the new resid[r, :] in `dtype`
// (d2 and cast may be null).  d1 and d2 are outputs of products: tensors of `dtype`
// (splits 0) or float32 partial sums [splits][n][hidden], added in order.
int shk_add_deltas(float* resid, const void* d1, int splits1, const void* d2, int splits2, void* cast,
                   int dtype, int n, int hidden, void* stream);

// A product's output that is normed by itself before it joins the stream:
// x = resid[row] + delta[row] * rsqrt(mean(delta[row]^2) + deps) * dweight, stored back
// with write_resid; with out != null, out[r] = x * rsqrt(mean(x^2) + eps) * weight as
// well (the norm that follows).  delta / delta_splits / rows / resid_rows as in
// shk_add_rmsnorm, except that delta has `dtype` or is float32 partial sums.
int shk_add_normed_rmsnorm(float* resid, const void* delta, int delta_splits, const float* dweight,
                           float deps, const float* weight, float eps, void* out, int dtype,
                           const int32_t* rows, int n, int hidden, int write_resid, int resid_rows,
                           void* stream);

// out[r, j] = act(a[r, j]) * table[ids[r] * ld + offset + j] for j < width: a gate times
// a slice of the table row that the token chooses.  ids must lie in [0, table_rows).
// a_splits > 0: a is float32 partial sums [a_splits][n][width], added in order.
int shk_act_mul_rows(const void* a, int a_splits, const void* table, int dtype, const int32_t* ids,
                     long long ld, int offset, int table_rows, void* out, int n, int width, int act,
                     void* stream);

// Residual add fused with RMSNorm.  For each of n rows r (row index rows[r]
// when `rows` is given, else r):  x = resid[row] (+ delta[row]);  if
// write_resid the sum is stored back into resid;  out[r] = x * rsqrt(mean(x^2)
// + eps) * weight.  resid is float32, delta and out have `dtype`, weight is
// float32.  delta_splits > 0: delta is float32 [delta_splits][resid rows][hidden],
// partial sums of a product split along k, added in order.
int shk_add_rmsnorm(float* resid, const void* delta, const float* weight, float eps, void* out,
                    int dtype, const int32_t* rows, int n, int hidden, int write_resid,
                    int delta_splits, int resid_rows, void* stream);

// out[i, j] = act(gu[i, j]) * gu[i, inter + j] for j < inter; gu is [n, 2*inter].
// act 1: SiLU; act 2: GELU in its tanh form; act 3: ReLU; act 4: g * sigmoid(1.702 g).  With limit > 0
// the gate is bounded from above, g <- min(g, limit), and the other factor from both sides, before
// anything else; up_shift is added to that factor: out = act(g) * (u + up_shift).
int shk_act_mul(const void* gu, void* out, int dtype, int n, int inter, int act, float limit, float up_shift,
                void* stream);

// A stream that is normed after every sum (postnorm.hip): resid[r, :] <- (x / sqrt(mean(x^2) + eps)) *
// weight with x = alpha * resid[r, :] + lscale * delta[r, :] (lscale float32 [hidden] or null: ones);
// delta has `dtype`, or is float32 partial sums [delta_splits][n][hidden] added in order, or is null
// (nothing is added).  cast (of `dtype`, or null) receives the new rows too.
int shk_postnorm(float* resid, const void* delta, int delta_splits, float alpha, const float* lscale,
                 const float* weight, float eps, void* cast, int dtype, int n, int hidden, void* stream);
// dst[i] = src[i] in `dtype`.
int shk_cast_rows(const float* src, void* dst, int dtype, long long numel, void* stream);
// out = act(x) elementwise: 1 SiLU, 2 GELU (tanh form), 3 ReLU, 4 the square of ReLU.
int shk_activate(const void* x, void* out, int dtype, long long numel, int act, void* stream);
// out = x * sigmoid(gate) elementwise.
int shk_gate_mul(const void* x, const void* gate, void* out, int dtype, long long numel, void* stream);

// out[n, m] (+)= a[n, k] @ w[m, k]^T + bias[m].  a and w have in_dtype, out has
// out_dtype, bias is float32 or null.  lda/ldo are row strides in elements.
// With `accumulate` the product is added to what out holds (out_dtype float32
// only).  The reduction order over k is the same for every row and column, so
// a row's result does not depend on which other rows are in the call.
int shk_gemm(const void* a, const void* w, const float* bias, void* out, int n, int m, int k,
             int lda, int ldo, int in_dtype, int out_dtype, int accumulate, void* stream);

// wt = the tiled layout of the row-major bfloat16 matrix w[m, k] (see
// gemm_bf16.hip): ceil(m/16) * ceil(k/32) tiles of 1 KiB.
int shk_retile_weight(const void* w, int m, int k, void* wt, void* stream);

// wt = the tiled layouts of a gated feed-forward's gate and up matrices ([m, k]
// each, given tiled) interleaved by blocks of 16 rows.
int shk_interleave_gate_up(const void* gate_t, const void* up_t, int m, int k, void* wt,
                           void* stream);

// out[n, m] (+)= a[n, k] @ w^T + bias with w given in the tiled layout; a is
// bfloat16 row-major with row stride lda; out is bfloat16 or float32.
// gated != 0: wt is an interleaved gate/up pair and out[n, m] = act(a @ gate^T) *
// (a @ up^T), without bias or accumulation; gated is the activation, 1 for SiLU,
// 2 for GELU in its tanh form, 3 for ReLU, 4 for g * sigmoid(1.702 g).  A gated product's
// `bias` is null or two floats, the gate's constants: with bias[0] > 0 the gate is bounded
// from above and the other factor from both sides by it before anything else, and bias[1]
// is added to that factor (as in shk_act_mul).
// ksplit > 1 (at most 64 rows, float32 output, no bias): the k range is shared
// by ksplit workgroups per block of weight rows and out is [ksplit][n][m], the
// partial sums, which the kernel that reads the product adds up in order
// (shk_add_rmsnorm, shk_rope_kv_store).  shk_gemm_bf16_splits says how many
// shares fill the chip for a shape (1: do not split).
int shk_gemm_bf16_tiled_weight(const void* a, const void* wt, const float* bias, void* out, int n,
                               int m, int k, int lda, int ldo, int out_dtype, int accumulate,
                               int gated, int ksplit, void* stream);
int shk_gemm_bf16_splits(int n, int m, int k);
// 2 where a product of many tokens runs as two (the weight rows whose tiles make whole
// rounds of the compute units, then the rest with tiles of its own), else 1.
int shk_gemm_bf16_parts(int n, int m, int k, int gated);

// The matrix instruction alone, for measuring its rate on operands of a given kind:
// workgroups x 4 wavefronts each multiply, iters times, a 64 x 64 x 32 block
// (2 * 64 * 64 * 32 flop) from `operands` (64 KiB of bfloat16), kept in registers.
// out: workgroups * 256 floats.
int shk_mfma_alone(const void* operands, float* out, int workgroups, int iters, void* stream);

// Position encoding and cache write for the n tokens of a step.  qkv is
// [n, (heads + 2*kv_heads) * head_dim]: queries, keys, values.  Queries and
// keys are rotated by position (pairs (i, i + rot_dim/2), angle position *
// inv_freq[i]); queries are rewritten in place; keys and values go to their
// page slots: page = tables[token_seq[t] * table_stride + position / page_size].
// The key pool holds each page's keys in slabs of 32 elements, [num_pages,
// kv_heads, head_dim / 32, page_size, 32] (one slab of head_dim elements where
// head_dim is no multiple of 32); the value pool is stored transposed,
// [num_pages, kv_heads, head_dim, page_size].  rot_dim 0 rotates nothing;
// write_kv 0 leaves the pools alone.
// splits > 0: the projections come as float32 partial sums `parts`
// [splits][n][width] of a product split along k; they are added in order, `bias`
// (float32 [width] or null) is added, and the rotated queries are written to
// qkv's query columns (qkv is then output only).
// pairing 1 pairs the neighbours (2i, 2i + 1) instead, with the same angle for pair i.
// v_from_k != 0: there are no value columns, qkv is [n, (heads + kv_heads) * head_dim],
// and a token's values are its keys as they were projected, before the rotation.
int shk_rope_kv_store(void* qkv, int dtype, int n, int heads, int kv_heads, int head_dim,
                      int rot_dim, const float* inv_freq, const int32_t* positions,
                      const int32_t* token_seq, const int32_t* tables, int table_stride,
                      void* k_pool, void* v_pool, int page_size, int num_pages, int write_kv,
                      const float* parts, int splits, const float* bias, int pairing,
                      int v_from_k, void* stream);

// Causal attention of n query tokens over their sequences' paged caches.
// Token t (position p, sequence s) reads keys j in (p - window, p] (all j <= p
// when window <= 0) through tables[s]; with chunk > 0 only those of them that lie
// in p's own block of `chunk` positions, floor(j / chunk) == floor(p / chunk) (the
// same two bounds in every attention launcher below).  q has row stride q_stride elements,
// out is [n, heads * v_dim].  Softmax and accumulation are float32.  v_dim is the size of
// a value (the value pool is [num_pages, kv_heads, v_dim, page_size]); softcap > 0 caps
// the scaled scores, s <- softcap * tanh(s / softcap); sinks (float32 [heads] or null)
// adds exp(sinks[head]) to the softmax's denominator, a term without key or value; dist_bias (float32
// [heads, bias_rows] or null) adds dist_bias[head, min(p - j, bias_rows - 1)] to the score after the cap.
int shk_attention(const void* q, int q_stride, void* out, int dtype, int n, int heads,
                  int kv_heads, int head_dim, const int32_t* positions, const int32_t* token_seq,
                  const int32_t* tables, int table_stride, int num_seqs, const void* k_pool,
                  const void* v_pool, int page_size, int num_pages, int window, int chunk, float scale,
                  int v_dim, float softcap, const float* sinks, const float* dist_bias, int bias_rows,
                  void* stream);

// Cache write for attention without rotation.  qkv is [n, heads * head_dim + kv_heads *
// (head_dim + v_dim)]: queries, keys, values.  q_every > 0: the queries of the token at
// position p are multiplied by 1 + q_coef * ln(floor((p + 1) / q_every) + 1), in place.
// v_eps > 0: each head's value is divided by sqrt(mean(v^2) + v_eps) before it is stored.
// Keys and values go to their page slots in the layouts of shk_rope_kv_store (values
// [num_pages, kv_heads, v_dim, page_size]); write_kv 0 leaves the pools alone.
// qk_eps > 0: every head of the queries and of the keys is divided by sqrt(mean(x^2) + qk_eps) first
// and multiplied by q_weight / k_weight (float32 [head_dim], shared by the heads; null: none).
// has_kv 0: qkv is [n, heads * head_dim], queries alone (a layer that reads another's cache).
int shk_qkv_store(void* qkv, int dtype, int n, int heads, int kv_heads, int head_dim, int v_dim,
                  float q_coef, int q_every, float v_eps, float qk_eps, const float* q_weight,
                  const float* k_weight, int has_kv, const int32_t* positions,
                  const int32_t* token_seq, const int32_t* tables, int table_stride, void* k_pool,
                  void* v_pool, int page_size, int num_pages, int write_kv, void* stream);

// 1 if the MFMA attention kernels take these shapes (head_dim a multiple of 32
// up to 256, page_size a multiple of 16, at most 16 query heads per key/value
// head, q rows 16-byte aligned); otherwise shk_attention serves them.
int shk_attention_supports_mfma(int heads, int kv_heads, int head_dim, int page_size, int q_stride);

// bfloat16 decode attention: sequence s has one query token, row s of q, at
// positions[s].  Its keys are split over nsplit wavefronts per key/value head;
// `partial` is float32 scratch of num_seqs * heads * nsplit * (head_dim + 2).
// streaming != 0: keys and values are fetched with non-temporal loads (faster when a
// launch reads tens of megabytes of them, slightly slower below; the result is the same).
// softcap / sinks / dist_bias as in shk_attention (0 and null: none).
int shk_attention_decode_bf16(const void* q, int q_stride, void* out, int num_seqs, int heads,
                              int kv_heads, int head_dim, const int32_t* positions,
                              const int32_t* tables, int table_stride, const void* k_pool,
                              const void* v_pool, int page_size, int window, int chunk, float scale,
                              float* partial, int nsplit, int streaming, float softcap, const float* sinks,
                              const float* dist_bias, int bias_rows, void* stream);

// bfloat16 attention for prompt portions, in tiles of 16 queries: tile i covers
// queries tile_q0[i] .. +16 of sequence tile_seq[i]'s portion.  cu_q[s] is the
// first token row of sequence s in q/out, ctx_lens[s] its length after the step.
int shk_attention_prefill_bf16(const void* q, int q_stride, void* out, int num_tiles, int heads,
                               int kv_heads, int head_dim, const int32_t* cu_q,
                               const int32_t* ctx_lens, const int32_t* tile_seq,
                               const int32_t* tile_q0, const int32_t* tables, int table_stride,
                               const void* k_pool, const void* v_pool, int page_size, int window, int chunk,
                               float scale, void* stream);

// The same for all query heads of a key/value head at once: a workgroup serves
// `tiles` = shk_attention_prefill_shared_tiles(...) consecutive 16-query tiles of
// one sequence (wg_seq, wg_q0 in steps of 16 * tiles) and stages each chunk of
// keys once in LDS.  small != 0: workgroups of 8 wavefronts instead of 16, with
// half as many tiles each, for portions that would otherwise make too few
// workgroups for the chip.  tiles == 0: the shape is not served (more query
// heads per key/value head than a workgroup has wavefronts, head_dim > 128).
// Entries are launched in the order of the list.  nsplit > 1 shares every entry's
// keys among nsplit workgroups (for a few queries far into a sequence, which alone
// would leave most of the chip idle); their results go through `partial`
// (prompt_tokens * heads * nsplit * (head_dim + 2) floats) and are merged into out.
// first_token: the index of the step's first prompt token (prompt tokens follow
// the single tokens); prompt_tokens: how many there are.
int shk_attention_prefill_shared_tiles(int heads, int kv_heads, int head_dim, int small);
int shk_attention_prefill_shared_bf16(const void* q, int q_stride, void* out, int num_wgs,
                                      int heads, int kv_heads, int head_dim, const int32_t* cu_q,
                                      const int32_t* ctx_lens, const int32_t* wg_seq,
                                      const int32_t* wg_q0, const int32_t* tables,
                                      int table_stride, const void* k_pool, const void* v_pool,
                                      int page_size, int window, int chunk, float scale, int small,
                                      float* partial, int nsplit, int first_token,
                                      int prompt_tokens, float softcap, const float* sinks,
                                      const float* dist_bias, int bias_rows, void* stream);

// Attention through latents (latent.hip).  shk_latent_prepare: `down` is [n, q_rank +
// kv_rank + rot_dim], a token's joint down-projection; q_latent [n, q_rank] receives
// down[:, :q_rank] * rsqrt(mean^2 + eps) * q_weight; the token's row of `pool`
// ([num_pages, page_size, kv_rank + rot_dim], page through tables as elsewhere) receives
// the next kv_rank columns normed likewise with kv_weight, then the last rot_dim columns
// with neighbouring pairs (2i, 2i + 1) turned by position * inv_freq[i].
int shk_latent_prepare(const void* down, int dtype, int n, int q_rank, int kv_rank, int rot_dim,
                       const float* q_weight, const float* kv_weight, float eps, const float* inv_freq,
                       const int32_t* positions, const int32_t* token_seq, const int32_t* tables,
                       int table_stride, void* q_latent, void* pool, int page_size, int num_pages,
                       int write_kv, void* stream);
// dst[t, h * dst_head + dst_off + e] = the rotation of src[t, h * src_head + src_off + e],
// e < rot_dim, pairs (2i, 2i + 1) turned by positions[t] * inv_freq[i]; rows src_row /
// dst_row elements apart.
int shk_rotate_heads(const void* src, int src_row, int src_head, int src_off, void* dst, int dst_row,
                     int dst_head, int dst_off, int dtype, int n, int heads, int rot_dim,
                     const float* inv_freq, const int32_t* positions, void* stream);
// q [n, heads, key_dim], out [n, heads, v_dim]: every head attends over the rows of the
// token's sequence in `pool` ([num_pages, page_size, key_dim]); score = q . row * scale, the
// values are the rows' first v_dim elements.  window / chunk as in shk_attention.
int shk_latent_attention(const void* q, void* out, int dtype, int n, int heads, int key_dim, int v_dim,
                         const int32_t* positions, const int32_t* token_seq, const int32_t* tables,
                         int table_stride, const void* pool, int page_size, int num_pages, int window,
                         int chunk, float scale, void* stream);

// The same on the matrix units for bfloat16 (latent_mfma.hip), where
// shk_latent_attention_supports_mfma says so.  nsplit > 1 shares every token's rows among nsplit
// workgroups, whose results pass through `partial` (n * heads * nsplit * (v_dim + 2) floats).
// tokens_per_group > 1 lets a workgroup serve up to that many (2 or 4) neighbouring tokens where
// their heads leave wavefronts free (prompt portions; the result is the same).
int shk_latent_attention_supports_mfma(int heads, int key_dim, int v_dim);
int shk_latent_attention_bf16(const void* q, void* out, int n, int heads, int key_dim, int v_dim,
                              const int32_t* positions, const int32_t* token_seq, const int32_t* tables,
                              int table_stride, const void* pool, int page_size, int num_pages, int window,
                              int chunk, float scale, float* partial, int nsplit, int tokens_per_group,
                              void* stream);

// A batch of products of one shape: out_b[n, m] = a_b[n, k] @ w_b[m, k]^T for b < batch, with
// a_b = a + b * a_batch (rows lda apart), w_b = w + b * w_batch (contiguous), out_b = out + b *
// out_batch (rows ldo apart); all of `dtype`, float32 accumulation in ascending k.
int shk_gemm_batched(const void* a, const void* w, void* out, int n, int m, int k, int lda, int ldo,
                     int batch, long long a_batch, long long w_batch, long long out_batch, int dtype,
                     void* stream);

// The mLSTM recurrence (mlstm.hip) for the tokens of a step.  proj [n, ld] float32 holds each
// token's projections: queries at column q_off ([heads, dim]), keys at k_off, values at v_off
// ([heads, v_dim]), the input and forget gates' pre-activations at i_off and f_off ([heads]);
// i_bias / f_bias [heads] are added; cap bounds the gates; queries are multiplied by q_scale.
// Sequence s owns rows cu_q[s] .. cu_q[s + 1]; its state lies at state + slots[s] *
// slot_stride (shk_mlstm_state_floats floats) and is taken as zero when the sequence's first
// row is at position 0.  out [n, heads * v_dim] float32 receives the normalised readout.
long long shk_mlstm_state_floats(int heads, int dim, int v_dim);
int shk_mlstm_scan(const float* proj, int ld, int q_off, int k_off, int v_off, int i_off, int f_off,
                   const float* i_bias, const float* f_bias, float cap, float q_scale, int num_seqs,
                   int heads, int dim, int v_dim, const int32_t* positions, const int32_t* cu_q,
                   const int32_t* slots, float* state, long long slot_stride, float* out, void* stream);
// out[t, h, :] = o[t, h, :] * rsqrt(mean(o[t, h, :]^2) + eps) * weight[h, :] * g(gate[t, h, :]);
// o float32 [n, heads * v_dim], gate float32 rows gate_ld apart, out of `dtype`.  weight may be
// null (none); gate_act 0: g is the sigmoid, 1: SiLU.
int shk_headnorm_gate(const float* o, const float* gate, int gate_ld, const float* weight, float eps,
                      void* out, int dtype, int n, int heads, int v_dim, int gate_act, void* stream);

// Layer norm with weight and bias around the float32 stream (layernorm.hip).  For each of n
// rows r (row index rows[r] when `rows` is given, else r): x = resid[row]; with delta, x += d,
// where d = delta[row] (of `dtype`, or float32 partial sums [delta_splits][resid_rows][hidden]),
// and with dweight d is normed by itself first: d <- (d - mean(d)) / sqrt(var(d) + deps) * dweight
// + dbias; with write_resid the sum is stored back.  With out, out[r] = (x - mean) / sqrt(var +
// eps) * weight + bias, of `dtype`, or float32 with out_f32 (out may then be resid itself).  The
// variance is the mean of the squared deviations; dbias and bias may be null.
int shk_add_layernorm(float* resid, const void* delta, int delta_splits, const float* dweight,
                      const float* dbias, float deps, const float* weight, const float* bias, float eps,
                      void* out, int dtype, int out_f32, const int32_t* rows, int n, int hidden,
                      int write_resid, int resid_rows, void* stream);
// out[r, :] = sum over j < count of coef[j] * history[j * stride + r * hidden + :], added in
// ascending j (float32).  With delta (as in shk_add_layernorm, always normed: dweight, dbias,
// deps), the newest stream, j = count - 1, first gains the normed addend and is stored back.
int shk_mix_history(float* history, long long stride, const float* coef, int count, float* out, int n,
                    int hidden, const void* delta, int delta_splits, const float* dweight,
                    const float* dbias, float deps, int dtype, void* stream);
// x <- x * scale, then with cap > 0: x <- cap * tanh(x / cap); float32, elementwise.
int shk_scale_softcap(float* x, long long numel, float scale, float cap, void* stream);

// Attention with weights mixed across heads after the softmax (attention_talking.hip), over the
// cache layouts of shk_attention: s_g = q_g . k * scale - r1[g] * ln(1 + r2[g] * distance) (r1,
// r2 null: no bias); p_g = exp(s_g) / (exp(sink) [with has_sink] + sum exp(s_g)); head h applies
// sum_g talk[h, g] p_g (talk null: the identity) to the values of its own key/value head.
// scratch: shk_attention_talking_scratch_floats(n, heads, v_dim, nshare) floats; nshare > 1
// shares every token's keys among that many workgroups.
long long shk_attention_talking_scratch_floats(int n, int heads, int v_dim, int nshare);
int shk_attention_talking(const void* q, int q_stride, void* out, int dtype, int n, int heads, int kv_heads,
                          int head_dim, int v_dim, const int32_t* positions, const int32_t* token_seq,
                          const int32_t* tables, int table_stride, const void* k_pool, const void* v_pool,
                          int page_size, int num_pages, int window, int chunk, float scale,
                          const float* r1, const float* r2, const float* talk, int has_sink, float sink,
                          float* scratch, int nshare, void* stream);

// The same for bfloat16 on the matrix units, where shk_attention_talking_supports_mfma says so:
// every head's own weights meet the values of every key/value head (one pass over the keys with a
// running maximum and sum), and the sums are mixed: o_h = sum_g talk[h, g] U[g, c(h)].  The step's
// first num_single tokens are single tokens of sequences 0 .. num_single - 1; prompt portions come
// as num_tiles tiles of 16 queries (tile_seq, tile_q0 counted from the portion's first query; cu_q[s]
// = sequence s's first row).  nsplit > 1 shares every single token's keys among that many workgroups,
// whose sums are joined in order.  scratch: shk_attention_talking_mfma_scratch_floats(...) floats.
int shk_attention_talking_supports_mfma(int head_dim, int v_dim, int page_size, int q_stride);
long long shk_attention_talking_mfma_scratch_floats(int n, int num_single, int heads, int kv_heads, int v_dim, int nsplit);
int shk_attention_talking_bf16(const void* q, int q_stride, void* out, int n, int num_single, int num_tiles,
                               int heads, int kv_heads, int head_dim, int v_dim, const int32_t* positions,
                               const int32_t* token_seq, const int32_t* cu_q, const int32_t* tile_seq,
                               const int32_t* tile_q0, const int32_t* tables, int table_stride, const void* k_pool,
                               const void* v_pool, int page_size, int num_pages, int window, int chunk, float scale,
                               const float* r1, const float* r2, const float* talk, int has_sink, float sink,
                               float* scratch, int nsplit, void* stream);

// The selective scan of Mamba and its causal convolution (ssm.hip).  A request's slot holds S
// [inner, states] float32 and then the convolution's last taps - 1 inputs [(taps - 1), inner].
// shk_conv_silu: y[t, c] = silu(bias[c] + sum_k taps[c, num_taps - 1 - k] * x[t - k, c]) over the
// sequence's earlier inputs (rows of this step, else the slot's kept ones, zero before position 0).
// shk_dt_softplus: dt[t, c] = softplus(b[c] + sum_r w[r, c] * low[t, r]), float32; w [rank, inner].
// shk_selective_scan: S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n, y_c = sum_n S[c, n] C_n +
// dskip_c x_c, out = y * silu(z); A = -exp(a_log); B and C are columns b_off, c_off of bc (float32);
// `raw` are the convolution's inputs of the step, of which the slot keeps the last taps - 1.
long long shk_selective_scan_state_floats(int inner, int states, int taps);
int shk_conv_silu(const void* x, int ldx, const float* taps, const float* bias, int num_taps, int inner,
                  const int32_t* positions, const int32_t* token_seq, const int32_t* cu_q,
                  const int32_t* slots, const float* state, long long slot_stride, int states, void* y,
                  int dtype, int n, void* stream);
int shk_dt_softplus(const float* low, int ld, const float* w, const float* b, int rank, int inner,
                    float* dt, int n, void* stream);
int shk_selective_scan(const float* dt, const void* x, const float* bc, int ld_bc, int b_off, int c_off,
                       const void* z, int ldz, const float* a_log, const float* dskip, int inner,
                       int states, int num_taps, const void* raw, int ld_raw, const int32_t* positions,
                       const int32_t* cu_q, const int32_t* slots, float* state, long long slot_stride,
                       void* out, int dtype, int num_seqs, void* stream);

// Retention (ssm.hip): per head S_t = decay[h] S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, over float32
// projections at columns q_off, k_off ([heads, dim]) and v_off ([heads, v_dim]) of proj; a slot
// holds S as [heads, v_dim, dim].  shk_rotate_half_rows turns the pairs (i, i + rot_dim / 2) of
// every head of float32 rows in place by positions[t] * inv_freq[i] and multiplies the head by mult.
long long shk_retention_state_floats(int heads, int dim, int v_dim);
int shk_rotate_half_rows(float* x, int ld, int off, int heads, int dim, int rot_dim, const float* inv_freq,
                         const int32_t* positions, float mult, int n, void* stream);
int shk_retention_scan(const float* proj, int ld, int q_off, int k_off, int v_off, const float* decay,
                       int num_seqs, int heads, int dim, int v_dim, const int32_t* positions,
                       const int32_t* cu_q, const int32_t* slots, float* state, long long slot_stride,
                       float* out, void* stream);

// A routed mixture of gated experts (moe.hip).  shk_moe_route: softmax over the experts' logits
// (float32 [n, ld]); the `top` largest of score + correction (null: none) are chosen [n, top],
// their weights [n, top] are their scores over the chosen ones' sum (+ 1e-20).
// shk_moe_experts: out[t] = add[t] (null: nothing) + sum_k weights[t, k] * W_down_e (act(W_gate_e
// x_t) * (W_up_e x_t)), e = chosen[t, k]; matrices stacked row-major [experts, ff, width] and
// [experts, width, ff]; act_buf [n * top, ff]; all of `dtype`; act 1 SiLU, 2 GELU (tanh form), 3 ReLU
// (experts without a gate whose activation is the square of ReLU pass their one matrix as both).
// add_gate (float32, one number per token, gate_ld apart; null: none): add[t] is multiplied by
// sigmoid(add_gate[t * gate_ld]).
int shk_moe_route(const float* logits, int ld, const float* correction, int experts, int top,
                  int32_t* chosen, float* weights, int n, void* stream);
int shk_moe_experts(const void* x, const int32_t* chosen, const float* weights, const void* w_gate,
                    const void* w_up, const void* w_down, const void* add, const float* add_gate, int gate_ld,
                    void* act_buf, void* out, int dtype, int n, int width, int ff, int experts, int top, int act, void* stream);
// The same for bfloat16 on the matrix units, expert by expert over the lists of the (token,
// expert) pairs that chose it (built on the device).  width and ff in multiples of 8; scratch:
// shk_moe_grouped_scratch_bytes(...) bytes, 16-byte aligned.
long long shk_moe_grouped_scratch_bytes(int n, int width, int experts, int top);
int shk_moe_experts_grouped(const void* x, const int32_t* chosen, const float* weights, const void* w_gate,
                            const void* w_up, const void* w_down, const void* add, const float* add_gate,
                            int gate_ld, void* act_buf, void* out, void* scratch, int n, int width, int ff, int experts, int top, int act, void* stream);

// out = a_pos z^2 + z / 2 where z > 0, a_neg (exp(z) - 1 - z) + z / 2 elsewhere; elementwise.
int shk_xielu(const void* x, void* out, int dtype, long long numel, float a_pos, float a_neg, void* stream);

// out[i, :] = float(table[ids[i], :]) + float(pair_table[row, :]) with row = (prev * mul_prev +
// ids[i] * mul_cur) mod buckets, prev the token before token i in its sequence; at position 0,
// which has none, row = buckets (pair_table has buckets + 1 rows).  For the first token of a
// step's portion prev is last_token[slots[seq]], where the sequence's step before left its last
// token; this call leaves the portion's last token there.
int shk_embed_pairs(const void* table, const void* pair_table, int dtype, const int32_t* ids,
                    const int32_t* positions, const int32_t* token_seq, const int32_t* cu_q,
                    const int32_t* slots, int32_t* last_token, float* out, int n, int hidden, int vocab,
                    int buckets, int mul_prev, int mul_cur, void* stream);

// out[r] = lowest index of the largest value of logits[r, :vocab].  Rows wider
// than 4096 are searched in chunks; scratch then holds
// shk_argmax_scratch_floats(rows, vocab) floats (0: not needed).
int shk_argmax(const float* logits, int32_t* out, int rows, int vocab, int ld, float* scratch,
               void* stream);
int shk_argmax_scratch_floats(int rows, int vocab);

// shk_argmax for callers that cannot allocate device memory or bring a workspace
// (code recorded into a HIP graph, tight serving loops, harnesses that forbid
// hipMalloc).  It has no counterpart in the reference.  The chunk results live
// in an array of shk_argmax_static_max_floats() floats (256 KiB) that the library
// holds on every GPU it runs on until the process ends; a call whose
// shk_argmax_scratch_floats(rows, vocab) exceeds that is refused.  No call
// allocates or frees anything.  All calls on one GPU share that GPU's array:
// calls that overlap there (two streams, two threads) race; calls in stream order
// do not, and nothing an earlier call left in the array is read.
int shk_argmax_static(const float* logits, int32_t* out, int rows, int vocab, int ld, void* stream);
int shk_argmax_static_max_floats(void);

// Temperature / top-p sampling of one token per row (see sampling.hip).
// temperature[r] == 0 takes the argmax.  uniforms[r] in [0, 1) is the draw.
// `scratch` holds scratch_floats >= shk_sample_scratch_floats(rows, vocab) floats,
// 16-byte aligned.  nucleus == 0 promises that every row's top_p is 1 or more
// (the passes that find the nucleus are then left out; top_p is not read).
int shk_sample(const float* logits, int32_t* out, const float* temperature, const float* top_p,
               const float* uniforms, float* scratch, long long scratch_floats, int rows, int vocab,
               int ld, int nucleus, void* stream);
long long shk_sample_scratch_floats(int rows, int vocab);

// A list of launches run by one call.  A shk_call names a launcher of this header that
// takes a stream (shk_call_id gives its number by name, -1 for others) and holds its
// arguments in order, one per slot: pointers and integers as they are, a float's bits
// in the low 32 bits; the slot of the launcher's own stream argument is ignored and
// `stream` is passed instead.  The calls run in order on `stream`; the first that
// refuses its arguments ends the run with its status and message (those before it
// have been launched).
#define SHK_CALL_MAX_ARGS 32
typedef struct shk_call {
  int32_t launcher;
  int32_t reserved;
  int64_t args[SHK_CALL_MAX_ARGS];
} shk_call;
int shk_call_id(const char* name);
int shk_run_calls(const shk_call* calls, int n, void* stream);

#ifdef __cplusplus
}
#endif
