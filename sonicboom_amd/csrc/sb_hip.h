/* C ABI of the sonicboom_amd HIP kernel library (gfx950).
 *
 * Conventions, in the manner of the reference's capi.h
 * (/root/reference/capi/include/sonicboom/capi.h:136-161): every entry point
 * returns a status, 0 on success; on failure the message of the calling
 * thread's last error is read with sb_last_error().  No exception crosses
 * this boundary.  All pointers are device pointers unless said otherwise;
 * `stream` is a hipStream_t.  Shapes are checked on the host before any
 * launch; a size that a kernel cannot take is refused with SB_ERR_UNSUPPORTED,
 * never computed wrongly.
 *
 * Element types are named by sb_dtype.  Tensors are row-major and dense unless
 * a stride is given.  The KV cache is paged: a layer's keys are
 * [pages][kv_heads][SB_PAGE][head_dim], its values transposed,
 * [pages][kv_heads][head_dim][SB_PAGE]; `page_table` is int32 [batch][max_pages]
 * and maps the logical page (position / SB_PAGE) of a sequence to a physical
 * page, -1 for none.  Within a row of keys (one slot of a page) and within a row
 * of values (one dimension over the page's slots) the groups of eight elements
 * are kept in a permuted order: sb_key_index and sb_value_index below say where
 * an element lies.  It is the order in which the matrix-core attention reads a
 * page from LDS without bank conflicts, so a page goes from the cache into LDS
 * as it lies.
 */
#ifndef SONICBOOM_AMD_SB_HIP_H
#define SONICBOOM_AMD_SB_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SB_PAGE 64

#if defined(__HIPCC__)
#define SB_INLINE static inline __host__ __device__
#else
#define SB_INLINE static inline
#endif

/* Offset (in elements) of element d of the key at slot `slot` (0..SB_PAGE-1)
 * within a page's [SB_PAGE][head_dim] block of one head: group d / 8 of the row
 * lies at group (d / 8) ^ s, s made of bits 0, 1, 3 and 4 of the slot, cut to the
 * largest power of two (up to 16) that divides the row's number of groups.
 * Head sizes that are no multiple of 16 keep the plain order. */
SB_INLINE int sb_key_swizzle(int slot, int head_dim) {
  if (head_dim % 16) return 0;
  const int groups = head_dim / 8;
  const int mask = groups % 16 == 0 ? 15 : (groups % 8 == 0 ? 7 : (groups % 4 == 0 ? 3 : 1));
  return ((slot & 3) | (((slot >> 3) & 3) << 2)) & mask;
}
SB_INLINE size_t sb_key_index(int slot, int d, int head_dim) {
  return (size_t)slot * (size_t)head_dim + (size_t)((((d >> 3) ^ sb_key_swizzle(slot, head_dim)) << 3) | (d & 7));
}
/* Offset of the value of dimension d at slot `slot` within a page's
 * [head_dim][SB_PAGE] block of one head: group slot / 8 of the row lies at group
 * (slot / 8) ^ ((d / 2) % 8). */
SB_INLINE size_t sb_value_index(int d, int slot) {
  return (size_t)d * SB_PAGE + (size_t)((((slot >> 3) ^ ((d >> 1) & 7)) << 3) | (slot & 7));
}

typedef enum sb_status {
  SB_OK = 0,
  SB_ERR_ARGUMENT = 1,    /* null pointer, negative size, inconsistent shapes */
  SB_ERR_UNSUPPORTED = 2, /* a size or type this kernel does not take */
  SB_ERR_LAUNCH = 3       /* the HIP runtime refused the launch */
} sb_status;

typedef enum sb_dtype { SB_F32 = 0, SB_BF16 = 1 } sb_dtype;

/* The `gated` argument of the products and of sb_gate_mul: not gated, or the activation (SiLU, the tanh
 * form of GELU, max(g, 0)) of the
 * gate in Y = act(X Wg^T) * (X Wu^T). */
typedef enum sb_gate { SB_GATE_NONE = 0, SB_GATE_SILU = 1, SB_GATE_GELU_TANH = 2, SB_GATE_RELU = 3 } sb_gate;

/* The `kind` argument of sb_activate.  xIELU takes two numbers (p, q) from memory: for z > 0
 * softplus(p) z^2 + z/2, else (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2. */
typedef enum sb_act { SB_ACT_SILU = 1, SB_ACT_GELU_TANH = 2, SB_ACT_XIELU = 3, SB_ACT_GELU_ERF = 4, SB_ACT_RELU_SQ = 5 } sb_act;

/* Message of this thread's last failed call ("" if none). Never NULL. */
const char *sb_last_error(void);
/* A JSON object naming the target architecture, the page size and the build flags. */
const char *sb_build_info(void);

/* out[t,:] = table[ids[t],:]  as f32.  An id outside [0,vocab) yields a NaN row. */
int sb_embed(float *out, const void *table, int table_dtype, const int32_t *ids,
             int n_rows, int width, int vocab, void *stream);

/* y[r,:] = (x[src,:] * inv) * w,  inv = 1/sqrt(mean(x[src,:]^2) + eps), src = rows ? rows[r] : r.
 * x is f32; y is out_dtype; w is w_dtype (NULL = no weight). */
int sb_rmsnorm(void *y, int out_dtype, const float *x, const void *w, int w_dtype,
               const int32_t *rows, int n_rows, int width, float eps, void *stream);

/* The same norm taken over each of `groups` equal consecutive parts of the row (the weight spans
 * the row); a row's bits do not depend on what else the launch holds. */
int sb_rmsnorm_grouped(void *y, int out_dtype, const float *x, const void *w, int w_dtype,
                       const int32_t *rows, int n_rows, int width, int groups, float eps, void *stream);

/* x[t,:] += scale * (sum_s partial[s][t][:] (+ bias)), slices in ascending order; with do_norm also
 * y[t,:] = the RMS norm of x[t,:] in `groups` parts, times w.  Any width that `groups` divides. */
int sb_reduce_scaled_group_norm(void *y, int y_dtype, float *x, const float *partial, int n_slices,
                                const void *bias, int bias_dtype, float scale, const void *w, int w_dtype,
                                int n_rows, int width, int groups, float eps, int do_norm, void *stream);

/* x[t,:] += sum_s partial[s][t][:] (+ bias), slices in ascending order; with do_norm
 * also y[t,:] = rmsnorm(x[t,:]) * w.  partial is f32 [n_slices][n_rows][width]. */
int sb_reduce_resid_norm(void *y, int y_dtype, float *x, const float *partial, int n_slices,
                         const void *bias, int bias_dtype, const void *w, int w_dtype, int n_rows,
                         int width, float eps, int do_norm, void *stream);

/* Y[t,n] = sum_k X[t,k] W[n,k] (+ bias[n]) (+ resid[t,n]).   Plain tiled kernel,
 * float accumulation in ascending k for every element whatever the batch.
 * resid is f32 [t,n] and may be the same buffer as Y (when Y is f32). */
int sb_gemm(void *y, int y_dtype, const void *x, int x_dtype, const void *w, int w_dtype,
            const void *bias, int bias_dtype, const float *resid,
            int n_rows, int n_out, int n_in, void *stream);

/* out[t,i] = act(gu[t,i]) * gu[t,width+i];  gu is [t, 2*width]; gate: SB_GATE_SILU or
 * SB_GATE_GELU_TANH. */
int sb_gate_mul(void *out, int out_dtype, const void *gu, int gu_dtype, int n_rows, int width, int gate,
                void *stream);
/* The same with the SiLU gate. */
int sb_silu_mul(void *out, int out_dtype, const void *gu, int gu_dtype,
                int n_rows, int width, void *stream);

/* resid[i] += y[i]  (resid f32, y of y_dtype). */
int sb_add_into(float *resid, const void *y, int y_dtype, size_t n, void *stream);

/* resid[i] += scale * y[i]  (resid f32, y of y_dtype). */
int sb_add_scaled(float *resid, const void *y, int y_dtype, float scale, size_t n, void *stream);

/* out[i] = act(in[i]), act an sb_act; params: the activation's numbers in memory (xIELU: two), of
 * params_dtype, NULL for the others. */
int sb_activate(void *out, int out_dtype, const void *in, int in_dtype, size_t n, int kind,
                const void *params, int params_dtype, void *stream);

/* dst[i] = src[i] converted. */
int sb_cast(void *dst, int dst_dtype, const void *src, int src_dtype, size_t n, void *stream);

/* Rotate the query heads and key heads of a step's qkv rows, write the queries
 * to q_out and store keys and values into the paged cache.
 *   qkv        [n_slices][n_rows, row_stride] of qkv_dtype, read only; a row is
 *              [heads_q*hd queries | heads_kv*hd keys | heads_kv*hd values];
 *              the slices (partial sums of the projection over K) are added
 *              in ascending order, then `bias` (f32 [row], may be NULL)
 *   q_out      [n_rows, heads_q*hd] of q_dtype
 *   inv_freq   f32 [rot_dims/2]: angle of pair i at position p is
 *              float(p)*inv_freq[i], divided by freq_factors[i] when given.
 *              NULL = no rotation.  Pair i is (i, i + rot_dims/2) of a head.
 *   row_pos    int32 [n_rows] absolute position;  row_seq int32 [n_rows] index
 *              of the row's sequence in page_table.
 *   k_cache/v_cache of cache_dtype; NULL (with heads_kv = 0) for a layer that
 *              stores nothing.
 */
int sb_rope_kv_store(void *q_out, int q_dtype, const void *qkv, int qkv_dtype, int row_stride,
                     int n_slices, const float *bias, const float *inv_freq, const float *freq_factors, int rot_dims,
                     const int32_t *row_pos, const int32_t *row_seq, void *k_cache, void *v_cache,
                     int cache_dtype, const int32_t *page_table, int max_pages, int n_pages_total,
                     int n_rows, int heads_q, int heads_kv, int head_dim, void *stream);

/* Attention of every row over its sequence's cached keys, position by position:
 * row r at position p of sequence s sees keys j with j <= p and (window == 0 or
 * p - j < window).  One wave per (row, query head), 64 keys at a time, online
 * softmax in f32 whose reduction order depends on key positions only.
 *   q   [n_rows, q_stride] of act_dtype (heads back to back at the row's start)
 *   out [n_rows, heads_q*hd] of act_dtype
 */
int sb_attention(void *out, const void *q, int act_dtype, int q_stride, const void *k_cache,
                 const void *v_cache, int cache_dtype, const int32_t *page_table, int max_pages,
                 int n_pages_total, const int32_t *row_pos, const int32_t *row_seq, int n_rows,
                 int heads_q, int heads_kv, int head_dim, float scale, int window, void *stream);

/* ---- a gated recurrence (csrc/recurrent.hip) -------------------------------------------------
 * minGRU over the rows of a step, sequence by sequence: from p f32 [n_rows, 3 * width] = the
 * pre-activations (a | u | g) of every row, z = sigmoid(a), cand = u + 1/2 (u >= 0) or sigmoid(u),
 * S = (1 - z) S + z cand, out[r,:] = S * silu(g); S of sequence s lives in state[slots[s]] (f32
 * [*, width]) and is left moved on.  chunks NULL: a thread a channel walks the rows in order.  Else
 * the rows in chunks of at most sb_mingru_chunk_rows() rows of one sequence, int32 [n_chunks, 4]
 * (first row, rows, sequence, 0) in row order, are folded in parallel, carried serially and walked in
 * parallel; folded: scratch of 2 * n_chunks * width floats. */
int sb_mingru_chunk_rows(void);
int sb_mingru_scan(void *out, int out_dtype, const float *p, float *state, const int32_t *cu_rows,
                   const int32_t *slots, int n_seqs, int n_rows, int width, const int32_t *chunks,
                   int n_chunks, float *folded, void *stream);

/* ---- latent attention (csrc/attention_latent.hip) --------------------------------------------
 * A layer keeps a row [c | r] per token (c: rank numbers, r: rot_dim rotated numbers shared by the
 * heads) in cache [pages][SB_PAGE][rank + rot_dim]; attention runs in the latent's space.
 * sb_latent_prepare: from a step's input-product rows p f32 [n_rows, row_stride]: queries at
 * q_off (head = [dim plain | rot_dim rotated]) -> q_plain [n_rows, heads, dim] and the rotated
 * parts behind the first rank numbers of q_latent [n_rows, heads, rank + rot_dim]; at kv_off (-1:
 * nothing is stored) rank numbers RMS-normed with c_weight and eps, and rot_dim rotated, stored
 * at the row's position.  The first rot_dims of rot_dim numbers turn, pair j by float(pos) *
 * inv_freq[j]; pairs (2j, 2j+1) when interleaved, else (j, j + rot_dims/2). */
int sb_latent_prepare(void *q_plain, void *q_latent, int act_dtype, const float *p, int row_stride,
                      int q_off, int kv_off, const void *c_weight, int c_w_dtype, float eps,
                      const float *inv_freq, int rot_dims, int interleaved, const int32_t *row_pos,
                      const int32_t *row_seq, void *cache, int cache_dtype, const int32_t *page_table,
                      int max_pages, int n_pages_total, int n_rows, int heads, int dim, int rot_dim,
                      int rank, void *stream);
/* out[t, a, o] = sum_i W[a][o][i] in[t, a, i], W [heads, n_out, n_in]; (t, a, .) of out at
 * t * out_stride + a * out_hstride, of in at t * in_stride + a * in_hstride; gate f32 or NULL:
 * times sigmoid(gate[t * gate_stride + a * n_out + o]). */
int sb_head_product(void *out, int out_dtype, int out_stride, int out_hstride, const void *in,
                    int in_dtype, int in_stride, int in_hstride, const void *w, int w_dtype,
                    const float *gate, int gate_stride, int n_rows, int heads, int n_in, int n_out,
                    void *stream);
/* out [n_rows, heads, rank]: for every row and head the softmax-weighted sum of the first rank
 * numbers of the cached rows j it sees (j <= p, and p - j < window unless window is 0), scores
 * scale * (q . row); q [n_rows, heads, rank + rot_dim].  One wave per (row, head). */
int sb_latent_attention(void *out, const void *q, int act_dtype, const void *cache, int cache_dtype,
                        const int32_t *page_table, int max_pages, int n_pages_total,
                        const int32_t *row_pos, const int32_t *row_seq, int n_rows, int heads, int rank,
                        int rot_dim, float scale, int window, void *stream);

/* The same two on the matrix cores, everything bfloat16 (csrc/attention_latent_mfma.hip); the
 * *_ok functions say whether the sizes are taken.  tiles int32 [n_tiles, 4] = (first row, rows,
 * sequence, 0): runs of up to tile_rows consecutive rows of a sequence, tile_rows 16 (a wave takes 16
 * rows of a head) or 1 (16 heads of a row).  n_splits > 1: every tile's keys are shared out over that
 * many blocks and put together by a second kernel, through part_o f32 [n_splits, n_rows, heads, rank]
 * and part_ml f32 [n_splits, n_rows, heads, 2]. */
int sb_head_product_bf16_ok(int out_stride, int out_hstride, int in_stride, int in_hstride, int n_in);
int sb_head_product_bf16(void *out, int out_stride, int out_hstride, const void *in, int in_stride,
                         int in_hstride, const void *w, const float *gate, int gate_stride, int n_rows,
                         int heads, int n_in, int n_out, void *stream);
int sb_latent_attention_tile_rows(void);
int sb_latent_attention_bf16_ok(int rank, int rot_dim);
int sb_latent_attention_bf16(void *out, const void *q, const void *cache, const int32_t *page_table,
                             int max_pages, int n_pages_total, const int32_t *row_pos, const int32_t *tiles,
                             int n_tiles, int heads, int rank, int rot_dim, float scale, int window,
                             int tile_rows, int n_splits, float *part_o, float *part_ml, int n_rows, void *stream);

/* ---- norms on what a sublayer gives back, an embedding with positions (csrc/outnorm.hip) --------
 * un(v) = v / sqrt(mean(v^2) + eps) * (offset + w): offset 1 for weights kept as multiplier minus one.
 * sb_offset_norm: y[r,:] = un(x[rows ? rows[r] : r,:]).
 * sb_norm_add: x[t,:] += un(sum_s a_s(t) part[s * slice_stride + t * row_stride + :] (+ b(t) extra[t,:])),
 *   a_s(t) = part_w ? part_w[t * part_w_stride + s] : 1, b(t) = extra_w ? extra_w[t * extra_w_stride] : 1;
 *   do_norm 0: the sum is added as it is; copy (NULL or of copy_dtype): the new x.
 * sb_embed_pos_norm: x[r,:] = table[ids[r],:] * scale (+ pos_table[row_pos[r],:]), normed with do_norm; an id
 *   or a position outside its table gives a row of NaN. */
int sb_offset_norm(void *y, int out_dtype, const float *x, const void *w, int w_dtype, const int32_t *rows,
                   int n_rows, int width, float eps, float offset, void *stream);
int sb_norm_add(float *x, void *copy, int copy_dtype, const float *part, int n_slices, size_t slice_stride,
                size_t row_stride, const float *part_w, int part_w_stride, const float *extra,
                const float *extra_w, int extra_w_stride, const void *w, int w_dtype, int n_rows, int width,
                float eps, float offset, int do_norm, void *stream);
int sb_embed_pos_norm(float *x, void *copy, int copy_dtype, const void *table, int table_dtype,
                      const void *pos_table, int pos_dtype, const int32_t *ids, const int32_t *row_pos,
                      int n_rows, int vocab, int n_positions, float scale, const void *w, int w_dtype,
                      int width, float eps, float offset, int do_norm, void *stream);
/* x[i] *= scale. */
int sb_scale(float *x, float scale, size_t n, void *stream);

/* ---- head norms, value mixing and store (csrc/headnorm_kv.hip) ---------------------------------
 * qkv f32 [n_slices][n_rows][row_stride] = [q: heads_q x dk | k: heads_kv x dk | v: heads_kv x dv], slices
 * added in ascending order; every head of q and k divided by its root mean square (eps inside the root)
 * times q_w / k_w [dk] (NULL: as it is); v <- (1 - lam) v + lam v_first when v_first is given; the v of
 * before the mixing to v_out when that is given; q out in q_dtype, k and v (store != 0) into the pages. */
int sb_headnorm_kv_store(void *q_out, int q_dtype, const float *qkv, int row_stride, int n_slices,
                         const void *q_w, const void *k_w, int w_dtype, float eps, const float *v_first,
                         const void *lam, int lam_dtype, float *v_out, const int32_t *row_pos,
                         const int32_t *row_seq, void *k_cache, void *v_cache, int cache_dtype,
                         const int32_t *page_table, int max_pages, int n_pages, int n_rows, int heads_q,
                         int heads_kv, int dk, int dv, int store, void *stream);

/* sb_attention with values of v_dim numbers a head (cache values [page][kv head][v_dim][position], out
 * [rows, heads_q * v_dim]), scores capped as softcap * tanh(s / softcap) when softcap > 0, and with `sink`
 * one more key of score 0 without a value in every softmax. */
int sb_attention_capped(void *out, const void *q, int act_dtype, int q_stride, const void *k_cache,
                        const void *v_cache, int cache_dtype, const int32_t *page_table, int max_pages,
                        int n_pages_total, const int32_t *row_pos, const int32_t *row_seq, int n_rows,
                        int heads_q, int heads_kv, int head_dim, int v_dim, float scale, int window,
                        float softcap, int sink, void *stream);

/* ---- routed experts (csrc/moe.hip, csrc/moe_mfma.hip) -------------------------------------------
 * sb_moe_route: from scores z f32 [rows, stride] the `top` largest of the first n_experts (ties to the
 *   lower number) in falling order, ids int32 [rows, top], and weights f32 [rows, top + 1]: the softmax
 *   over the chosen scores, then sigmoid(z[n_experts]) with has_gate (else 0).
 * sb_moe_router: the same from z = h w^T, w f32 [n_experts (+ 1), n_in], h of h_dtype, in one launch.
 * sb_moe_product: Y[p,:] = X[p / x_div,:] W_e^T, e = ids[p] (NULL: expert 0), W [experts][out (x 2 gated)][in];
 *   gated: g' sigmoid(alpha g') (u' + 1), g' = min(g, limit), u' = u cut to +-limit.  Plain kernel, any sizes.
 * sb_moe_group / sb_moe_product_bf16: the pairs laid out expert by expert on the device (order, tiles of
 *   tile_rows = sb_moe_tile_rows(pairs, experts) pairs, their count) and the product on the matrix cores.
 * sb_swish_clamp_mul: the gated pair of gu f32 [rows, 2 * width]. */
int sb_moe_max_top(void);
int sb_moe_route(int32_t *ids, float *weights, const float *z, int n_rows, int stride, int n_experts,
                 int top, int has_gate, void *stream);
int sb_moe_router(int32_t *ids, float *weights, const void *h, int h_dtype, const float *w, int n_rows,
                  int n_in, int n_experts, int top, int has_gate, void *stream);
int sb_moe_product(void *y, int y_dtype, const void *x, int x_dtype, const void *w, int w_dtype,
                   const int32_t *ids, int n_pairs, int x_div, int n_out, int n_in, int n_experts,
                   int gated, float limit, float alpha, void *stream);
int sb_moe_tile_rows(int n_pairs, int n_experts);
int sb_moe_group(const int32_t *ids, int n_pairs, int n_experts, int tile_rows, int32_t *order, int32_t *tiles,
                 int32_t *n_tiles, void *stream);
int sb_moe_product_bf16_ok(int n_in);
int sb_moe_product_bf16(void *y, int y_dtype, const void *x, const void *w, const int32_t *order,
                        const int32_t *tiles, const int32_t *n_tiles, int max_tiles, int tile_rows, int n_pairs,
                        int x_div, int n_out, int n_in, int gated, float limit, float alpha, void *stream);
int sb_swish_clamp_mul(void *out, int out_dtype, const float *gu, int n_rows, int width, float limit, float alpha,
                       void *stream);

/* The router with another kind of score: score_kind 0 as sb_moe_route / sb_moe_router; 1: the scores are
 * sigmoid(z), the `top` largest are chosen and their weights are those scores times score_scale (not
 * renormalized).  The experts' products take gated = 2 for the pair silu(g) u. */
int sb_moe_route_scored(int32_t *ids, float *weights, const float *z, int n_rows, int stride, int n_experts,
                        int top, int has_gate, int score_kind, float score_scale, void *stream);
int sb_moe_router_scored(int32_t *ids, float *weights, const void *h, int h_dtype, const float *w, int n_rows,
                         int n_in, int n_experts, int top, int has_gate, int score_kind, float score_scale,
                         void *stream);

/* A short causal convolution over time, channel by channel, over the rows of a step:
 *   y[t,c] = act(sum_j w[c,j] in[t - taps + 1 + j, c] (+ bias[c])) (+ in[t,c] with residual)
 * act 0 none, 1 SiLU.  The inputs before a step's first row are the sequence's state, f32
 * [slots][taps - 1][channels], the last taps - 1 inputs of the steps before (zeros for a new sequence);
 * sb_time_conv_keep moves it on after the rows have been computed, or sb_time_conv itself with keep = 1
 * when every sequence brings one row.  in/out may be column ranges of wider rows (strides in elements). */
int sb_time_conv_max_taps(void);
int sb_time_conv(void *out, int out_dtype, int out_stride, const void *in, int in_dtype, int in_stride, const void *w,
                 int w_dtype, const void *bias, int bias_dtype, float *state, const int32_t *row_seq,
                 const int32_t *cu_rows, const int32_t *slots, int n_rows, int n_seqs, int channels, int taps, int act,
                 int residual, int keep, void *stream);
int sb_time_conv_keep(const void *in, int in_dtype, int in_stride, float *state, const int32_t *cu_rows,
                      const int32_t *slots, int n_rows, int n_seqs, int channels, int taps, void *stream);

/* Recurrences with a float32 matrix per head and sequence (state[slots[s]]), walked row by row.
 * sb_ssd_scan: dt = softplus(dt_raw + dt_bias[a]); S = exp(-exp(a_log[a]) dt) S + dt B x^T (S is N x P);
 *   out = (S^T C + d_skip[a] x) silu(z); head a reads B, C of group a / (heads / groups); C lies c_off
 *   floats after B in a row of bc.
 * sb_delta_scan: q, k (of head a / (heads / kv_heads)) to unit vectors (eps_unit inside the root), q times
 *   D^-1/2; beta = sigmoid(b); g = exp(-exp(a_log[a]) softplus(decay + dt_bias)) per key channel;
 *   S = g S; u = beta (v - S^T k); S += k u^T; o = S^T q; out = o / sqrt(mean(o^2) + eps) w sigmoid(gate).
 *   qkv rows hold q [kv_heads D] | k [kv_heads D] | v [heads E].
 * With chunks (int32 [n_chunks, 4]: first row, rows <= chunk_rows, sequence, 0; sequence after sequence in row
 * order, each sequence's runs full but its last) both take the chunked form in three launches: every chunk from an
 * empty matrix, the chunks' results carried along each sequence, every chunk again from the matrix that comes in.
 * Scratch, float32: part [n_chunks, heads, N, P] and part_decay [n_chunks, heads] for sb_ssd_scan,
 * part [n_chunks, heads, D * E + D * D] for sb_delta_scan. */
int sb_state_scan_max_rows(void);
int sb_state_scan_max_cols(void);
int sb_state_scan_chunk_rows(void);
int sb_ssd_scan(float *out, int out_stride, const float *z, int z_stride, const float *x, int x_stride, const float *bc,
                int bc_stride, int c_off, const float *dt, int dt_stride, const float *dt_bias, const float *a_log,
                const float *d_skip, float *state, const int32_t *cu_rows, const int32_t *slots, int n_seqs, int heads,
                int groups, int N, int P, const int32_t *chunks, int n_chunks, int chunk_rows, float *part, float *part_decay,
                void *stream);
int sb_delta_scan(void *out, int out_dtype, int out_stride, const float *qkv, int qkv_stride, const float *beta,
                  int beta_stride, const float *decay, int decay_stride, const float *gate, int gate_stride,
                  const float *dt_bias, const float *a_log, const void *w, int w_dtype, float *state,
                  const int32_t *cu_rows, const int32_t *slots, int n_seqs, int heads, int kv_heads, int D, int E,
                  float eps, float eps_unit, const int32_t *chunks, int n_chunks, int chunk_rows, float *part, void *stream);

/* Attention whose heads share their weights.
 * sb_qk_rownorm_store: from f32 rows [q: heads_q dk | k: heads_kv dk]: q / rms(q, the whole part) * q_w *
 *   (1 + temp_coef ln(floor((p + 1) / temp_every) + 1)) out in q_dtype; with store, k / rms(k) * k_w into the
 *   key cache at the row's position and, with values_from_keys, k as it came into the value cache.
 * sb_attention_shared: O[row][g][c][:] = sum_j P_g(row, j) V_c(j), P_g the causal softmax of
 *   scale q_g . k_kv(g)(j) - r1[g] ln(1 + r2[g] (p - j)) (r1, r2 NULL: no bias); out f32.
 * sb_head_mix: out[row][h][:] = sum_g mix[h][g] O[row][g][kv(h)][:] (mix NULL: the identity); O of o_dtype. */
int sb_qk_rownorm_store(void *q_out, int q_dtype, const float *qk, int row_stride, const void *q_w, const void *k_w,
                        int w_dtype, float eps, float temp_coef, int temp_every, const int32_t *row_pos,
                        const int32_t *row_seq, const int32_t *page_table, int max_pages, int n_pages, void *k_cache,
                        void *v_cache, int cache_dtype, int n_rows, int heads_q, int heads_kv, int dk, int store,
                        int values_from_keys, void *stream);
int sb_attention_shared(float *out, const void *q, int act_dtype, const void *k_cache, const void *v_cache,
                        int cache_dtype, const int32_t *page_table, int max_pages, int n_pages_total,
                        const int32_t *row_pos, const int32_t *row_seq, int n_rows, int heads_q, int heads_kv,
                        int head_dim, int v_dim, float scale, const float *r1, const float *r2, void *stream);
int sb_head_mix(void *out, int out_dtype, const void *o, int o_dtype, const void *mix, int mix_dtype, int n_rows,
                int heads_q, int heads_kv, int v_dim, void *stream);

/* ids[r] = index of the first maximum of logits[r,:].  Two stages over
 * sb_argmax_parts(vocab) parts of a row; part_val / part_idx hold n_rows * parts
 * partial results (NULL allowed when parts == 1). */
int sb_argmax_parts(int vocab);
int sb_argmax(int32_t *ids, const float *logits, int n_rows, int vocab, float *part_val,
              int32_t *part_idx, void *stream);

/* sb_argmax for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  The caller passes the logits and the output
 * only; the first stage's partial results go to a fixed device array of
 * 512 KB that every GPU the library runs on holds until the process ends, so
 * n_rows * sb_argmax_parts(vocab) may be at most sb_argmax_noalloc_max_entries()
 * (65,536; e.g. 1,724 rows of 152,064 logits); more is refused with
 * SB_ERR_UNSUPPORTED.  The call allocates and frees nothing.  Every call on a
 * GPU shares that GPU's array: the first stage overwrites every entry the second
 * stage reads, so nothing is cleared, and two calls that overlap on one GPU
 * (different streams, or threads) race.  Same results as sb_argmax. */
int sb_argmax_noalloc_max_entries(void);
int sb_argmax_noalloc(int32_t *ids, const float *logits, int n_rows, int vocab, void *stream);

/* Sampling penalties on the logits in place, for `n_items` (row, token, count)
 * triples: v = v>0 ? v/rp : v*rp (when rp != 1), then v -= freq*count + presence.
 * exact != 0 uses the single-rounding fma form of the sampled path. */
int sb_penalize(float *logits, int vocab, const int32_t *item_row, const int32_t *item_token,
                const int32_t *item_count, int n_items, float repeat_penalty,
                float presence_penalty, float frequency_penalty, int exact, void *stream);

/* The mask of constrained decoding on logits [n_rows, vocab] in place: -inf wherever
 * a row's bitmap (uint8 [n_rows, n_bytes]; bit i & 7 of byte i >> 3 for id i; ids past
 * the bitmap are not allowed) does not allow the id. */
int sb_mask_logits(float *logits, int n_rows, int vocab, const uint8_t *bitmaps, int n_bytes, void *stream);

/* The `k` (<= 256) candidates with the largest z = logit / temperature of every
 * row (ties toward the lower id), ordered by (z descending, id ascending).
 * cand_id int32 [n_rows,k], cand_z f32 [n_rows,k]; rows with vocab < k are
 * filled with id -1.  Long rows are cut into parts whose best go through
 * `scratch`: sb_top_candidates_scratch(...) 64-bit words (NULL when that is 0). */
size_t sb_top_candidates_scratch(int n_rows, int vocab);
int sb_top_candidates(int32_t *cand_id, float *cand_z, const float *logits, int n_rows, int vocab,
                      int k, float temperature, uint64_t *scratch, void *stream);

/* One token per row from its candidates as sb_top_candidates wrote them (k <= 256
 * per row): the window of 30 below the best z, top-k (0: off), min-p
 * (log_min_p = ln(min_p) as a float; use_min_p 0: off), top-p (use_top_p 0: off;
 * running sums in float64, in order) and the Gumbel-max draw with word 0 of
 * Philox4x32-10 of counter (position, id, 0) under `seed`; ties to the lower id.
 * position int64 [n_rows]: the absolute position of each row's new token.
 * token int32 [n_rows]: -1 for a row that keeps no candidate. */
int sb_draw(int32_t *token, const int32_t *cand_id, const float *cand_z, const int64_t *position,
            int n_rows, int k, int top_k, int use_min_p, float log_min_p, int use_top_p, double top_p,
            uint64_t seed, void *stream);
/* The same with the positions taken from a decode step's device bookkeeping:
 * row r's new token takes position length_before[r] + 1. */
int sb_draw_after(int32_t *token, const int32_t *cand_id, const float *cand_z, const int32_t *length_before,
                  int n_rows, int k, int top_k, int use_min_p, float log_min_p, int use_top_p, double top_p,
                  uint64_t seed, void *stream);

/* ---- bf16 products on the matrix cores ----------------------------------
 * X bf16 [n_rows, n_in] row-major, n_in a multiple of 8, operands 16-byte
 * aligned.  W bf16 [n_out, n_in] row-major, or (packed != 0, or always for the
 * stream kernel) re-laid in 16 x 32 tiles of 1 KB in MFMA fragment order, rows
 * padded to 16 and k to 32, tiles of a row block consecutive in k; gated: the two
 * halves [gate; up] packed one after the other, Y = act(X Wg^T) * (X Wu^T) with the activation
 * that `gated` names (an sb_gate).
 * Y f32 or bf16; bias [n_out] f32 or bf16 or NULL; resid f32 [n_rows, n_out] or
 * NULL (may be Y itself).  The *_partial_* forms write the raw product in K
 * slices, f32 [slices][n_rows][n_out], slices as the matching *_slices says. */
int sb_gemm_skinny_max_rows(void);                       /* up to 64 rows, waves split K */
size_t sb_gemm_skinny_scratch(int n_rows, int n_out, int n_in, int gated);
int sb_gemm_skinny_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,
                        int bias_dtype, const float *resid, int n_rows, int n_out, int n_in, int gated,
                        int packed, float *scratch, size_t scratch_floats, void *stream);
int sb_gemm_skinny_slices(int n_rows, int n_out, int n_in);
int sb_gemm_skinny_partial_bf16(float *partial, const void *x, const void *w, int n_rows, int n_out,
                                int n_in, int packed, void *stream);
int sb_gemm_stream_max_rows(void);                       /* up to 128 rows, waves split the features */
/* `hint` (0: the launcher chooses; for tests and measurements): bits 0..7 waves per block (4..8),
 * bits 8..15 the K slices the partial form aims at (1..8).  `tile_shape`: -1 the launcher
 * chooses; else bits 0..3 the tile, 0 / 1 / 2 / 3 for 128 x 128, 256 x 128, 256 x 256, 128 x 256
 * outputs, and bits 4..5 the kernel: 0 the launcher's choice, 1 the one that stages tiles
 * through registers, 2 the one that loads them straight into LDS (packed weights, n_in a multiple
 * of 64; the only one with the 128 x 256 tile), 3 the same with a block for every tile. */
int sb_gemm_stream_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,
                        int bias_dtype, const float *resid, int n_rows, int n_out, int n_in, int gated,
                        int hint, void *stream);
int sb_gemm_stream_slices(int n_rows, int n_out, int n_in, int hint);     /* up to 64 rows */
int sb_gemm_stream_partial_bf16(float *partial, const void *x, const void *w, int n_rows, int n_out,
                                int n_in, int hint, void *stream);
int sb_gemm_mfma_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,   /* tiled */
                      int bias_dtype, const float *resid, int n_rows, int n_out, int n_in, int gated,
                      int packed, int tile_shape, void *stream);
/* The same with a multiplier on the product before the residual joins:
 * Y = resid_scale * (X W^T + bias) + resid. */
int sb_gemm_mfma_scaled_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,
                             int bias_dtype, const float *resid, float resid_scale, int n_rows, int n_out,
                             int n_in, int gated, int packed, int tile_shape, void *stream);
int sb_gemm_mfma_slices(int n_rows, int n_out, int n_in, int packed);
int sb_gemm_mfma_partial_bf16(float *partial, const void *x, const void *w, int n_rows, int n_out,
                              int n_in, int packed, void *stream);

/* Seeded normal weights: elements first .. first + n - 1 (first a multiple of 4) of tensor number
 * `tensor_index` under `seed`, as float32(mean + std z) (out_kind 0), the same rounded to bfloat16
 * (1), or the float64 standard normals z themselves (2).  Element e comes from Philox4x32-10 with
 * the seed as key and the counter (e / 4 low, e / 4 high, tensor_index, 0), words 0 and 1 making the
 * normals of elements 4c and 4c + 1, words 2 and 3 those of 4c + 2 and 4c + 3 (Box and Muller).  The
 * host computes the same bits (sonicboom_amd/weights/random_stream.py). */
int sb_random_normal(void *out, int out_kind, uint64_t n, uint64_t first, uint64_t seed, int tensor_index,
                     double mean, double std, void *stream);

/* ---- later forms of the kernels above: the shorter entry points call them with the arguments that
 * make them what they were ------------------------------------------------------------------------
 * sb_rmsnorm_pair: two RMS norms of the same rows (one root mean square, two weights, y2 may be NULL),
 *   the rows x_stride apart (parts of wider rows).
 * sb_sigmoid_mul: x[t, i] *= sigmoid(gate[t * gate_stride + i]).  sb_softcap: x <- cap tanh(x / cap).
 * sb_rope_kv_store_sized: value heads of v_dim numbers; every cosine and sine times `magnitude`.
 * sb_attention_sink: the sink's score a number of the query head's own (sink_scores f32 [heads_q]); an output
 *   gate, the result times sigmoid(gate[row * gate_stride + i]).
 * sb_latent_prepare_split: the latent's part read from rows of its own; `magnitude` as above.
 * sb_head_product_gated(_bf16): gate_per_head, one gate number a head.
 * sb_moe_route_grouped / sb_moe_router_grouped: score_kind 0 softmax over the chosen, 1 sigmoid, 2 softmax
 *   over all experts (weights not renormalized); experts in n_groups equal groups of neighbours of which
 *   the keep_groups with the largest best score can be chosen from.
 * The experts' products' `gated`: 0 as it is, 1 and 2 pairs, 3 one matrix row an output and max(z, 0)^2. */
int sb_rmsnorm_pair(void *y1, void *y2, int out_dtype, const float *x, int x_stride, const void *w1, const void *w2,
                    int w_dtype, int n_rows, int width, float eps, void *stream);
int sb_sigmoid_mul(void *x, int x_dtype, const float *gate, int gate_stride, int n_rows, int width, void *stream);
int sb_softcap(float *x, float cap, size_t n, void *stream);
int sb_rope_kv_store_sized(void *q_out, int q_dtype, const void *qkv, int qkv_dtype, int row_stride, int n_slices,
                           const float *bias, const float *inv_freq, const float *freq_factors, int rot_dims,
                           const int32_t *row_pos, const int32_t *row_seq, void *k_cache, void *v_cache, int cache_dtype,
                           const int32_t *page_table, int max_pages, int n_pages_total, int n_rows, int heads_q,
                           int heads_kv, int head_dim, int v_dim, float magnitude, void *stream);
int sb_attention_sink(void *out, const void *q, int act_dtype, int q_stride, const void *k_cache, const void *v_cache,
                      int cache_dtype, const int32_t *page_table, int max_pages, int n_pages_total,
                      const int32_t *row_pos, const int32_t *row_seq, int n_rows, int heads_q, int heads_kv, int head_dim,
                      int v_dim, float scale, int window, float softcap, int sink, const float *sink_scores,
                      const float *gate, int gate_stride, void *stream);
int sb_latent_prepare_split(void *q_plain, void *q_latent, int act_dtype, const float *p, int row_stride, int q_off,
                            const float *kv_rows, int kv_stride, int kv_off, const void *c_weight, int c_w_dtype, float eps,
                            const float *inv_freq, int rot_dims, int interleaved, float magnitude, const int32_t *row_pos,
                            const int32_t *row_seq, void *cache, int cache_dtype, const int32_t *page_table, int max_pages,
                            int n_pages_total, int n_rows, int heads, int dim, int rot_dim, int rank, void *stream);
int sb_head_product_gated(void *out, int out_dtype, int out_stride, int out_hstride, const void *in, int in_dtype,
                          int in_stride, int in_hstride, const void *w, int w_dtype, const float *gate, int gate_stride,
                          int gate_per_head, int n_rows, int heads, int n_in, int n_out, void *stream);
int sb_head_product_gated_bf16(void *out, int out_stride, int out_hstride, const void *in, int in_stride, int in_hstride,
                               const void *w, const float *gate, int gate_stride, int gate_per_head, int n_rows, int heads,
                               int n_in, int n_out, void *stream);
int sb_moe_route_grouped(int32_t *ids, float *weights, const float *z, int n_rows, int stride, int n_experts, int top,
                         int has_gate, int score_kind, float score_scale, int n_groups, int keep_groups, void *stream);
int sb_moe_router_grouped(int32_t *ids, float *weights, const void *h, int h_dtype, const float *w, int n_rows, int n_in,
                          int n_experts, int top, int has_gate, int score_kind, float score_scale, int n_groups,
                          int keep_groups, void *stream);

#ifdef __cplusplus
}
#endif
#endif
