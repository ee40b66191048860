// Attention whose heads share their weights: queries and keys normed over the whole projection,
// the values taken from the keys as projected, a query temperature that grows with the position,
// a bias by the logarithm of the distance, and the heads' softmax weights mixed by a matrix.
//
//   sb_qk_rownorm_store   from float32 rows [q: heads_q x dk | k: heads_kv x dk] (biases added):
//       q <- q / rms(q over the whole row part) * wq * (1 + coef ln(floor((p + 1) / every) + 1)), out in the
//       activation type; k <- k / rms(k) * wk into the key cache at the row's position; and, with
//       `values_from_keys`, k as it came in into the value cache (the value size is then dk).
//   sb_attention_shared   for query head g and value head c:  O[row, g, c, :] = sum_j P_g(row, j) V_c(j, :),
//       P_g = softmax over j <= p of  scale q_g . k_kv(g)(j) - r1_g ln(1 + r2_g (p - j)).
//       One wave per (row, g, c); float32 sums in an order that depends on the key positions alone.
//   sb_head_mix           out[row, h, :] = sum_g T[h, g] O[row, g, kv(h), :]: head h applies its mixed
//       weights sum_g T[h, g] P_g to the values of its own key/value head.
#include "common.h"

namespace {

constexpr int kMaxHeadDim = 256;

struct PrepArgs {
  void *q_out; int q_dtype;
  const float *qk; int row_stride;
  const void *q_w, *k_w; int w_dtype; float eps;
  float temp_coef; int temp_every;
  const int32_t *row_pos, *row_seq, *page_table; int max_pages, n_pages;
  void *k_cache, *v_cache; int cache_dtype;
  int heads_q, heads_kv, dk, store, values_from_keys;
};

__device__ __forceinline__ void st_dyn(void *p, int dtype, size_t i, float v) {
  if (dtype == SB_F32) ((float *)p)[i] = v;
  else ((bf16_t *)p)[i] = f32_to_bf16(v);
}

// sum of a double over the block's four waves, the same on every thread
__device__ __forceinline__ double block_sum4(double v, double *scratch) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  return ((scratch[0] + scratch[1]) + scratch[2]) + scratch[3];
}

__global__ void __launch_bounds__(256) qk_rownorm_store_kernel(PrepArgs a) {
  __shared__ double red[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float *src = a.qk + size_t(row) * a.row_stride;
  const int qw = a.heads_q * a.dk, kw = a.heads_kv * a.dk;
  const int pos = a.row_pos[row];
  double sq = 0.0;
  for (int i = tid; i < qw; i += 256) sq += double(src[i] * src[i]);
  const float q_inv = 1.0f / sqrtf(float(block_sum4(sq, red) / double(qw)) + a.eps);
  float temp = 1.0f;
  if (a.temp_coef != 0.0f) temp = 1.0f + a.temp_coef * logf(float((pos + 1) / a.temp_every) + 1.0f);
  for (int i = tid; i < qw; i += 256) {
    float v = src[i] * q_inv;
    if (a.q_w) v *= ld_dyn(a.q_w, a.w_dtype, i);
    st_dyn(a.q_out, a.q_dtype, size_t(row) * qw + i, v * temp);
  }
  if (!a.store) return;
  sq = 0.0;
  for (int i = tid; i < kw; i += 256) sq += double(src[qw + i] * src[qw + i]);
  const float k_inv = 1.0f / sqrtf(float(block_sum4(sq, red) / double(kw)) + a.eps);
  const int c = pos / SB_PAGE, slot = pos % SB_PAGE;
  int page = c < a.max_pages ? a.page_table[size_t(a.row_seq[row]) * a.max_pages + c] : -1;
  if (page < 0 || page >= a.n_pages) return;
  for (int i = tid; i < kw; i += 256) {
    const int head = i / a.dk, d = i % a.dk;
    const float raw = src[qw + i];
    float v = raw * k_inv;
    if (a.k_w) v *= ld_dyn(a.k_w, a.w_dtype, i);
    const size_t base = (size_t(page) * a.heads_kv + head) * SB_PAGE * a.dk;
    st_dyn(a.k_cache, a.cache_dtype, base + sb_key_index(slot, d, a.dk), v);
    if (a.values_from_keys) st_dyn(a.v_cache, a.cache_dtype, base + sb_value_index(d, slot), raw);
  }
}

template <typename TA, typename TC>
__global__ void __launch_bounds__(64)
attention_shared_kernel(float *__restrict__ out, const TA *__restrict__ q, const TC *__restrict__ k_cache,
                        const TC *__restrict__ v_cache, const int32_t *__restrict__ page_table, int max_pages,
                        int n_pages_total, const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seq,
                        int heads_q, int heads_kv, int head_dim, int v_dim, float scale, const float *__restrict__ r1,
                        const float *__restrict__ r2) {
  __shared__ float qs[kMaxHeadDim];
  __shared__ float ps[64];
  const int row = blockIdx.x, g = blockIdx.y, vh = blockIdx.z, lane = threadIdx.x;
  const int pos = row_pos[row], seq = row_seq[row];
  const int kvh = g / (heads_q / heads_kv);
  for (int d = lane; d < head_dim; d += 64) qs[d] = ld_f(q, (size_t(row) * heads_q + g) * head_dim + d);
  __syncthreads();
  const float b1 = r1 ? r1[g] : 0.0f, b2 = r2 ? r2[g] : 0.0f;
  const float neg_inf = -__builtin_inff();
  float m = neg_inf, l = 0.0f;
  float o[kMaxHeadDim / 64] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int c = 0; c <= pos / SB_PAGE; ++c) {
    const int page = c < max_pages ? page_table[size_t(seq) * max_pages + c] : -1;
    if (page < 0 || page >= n_pages_total) continue;  // uniform over the wave
    const TC *kp = k_cache + (size_t(page) * heads_kv + kvh) * SB_PAGE * head_dim;
    const TC *vp = v_cache + (size_t(page) * heads_kv + vh) * SB_PAGE * v_dim;
    const int j = c * SB_PAGE + lane;
    const bool visible = j <= pos;
    float s = neg_inf;
    if (visible) {
      float dot = 0.0f;
      for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], ld_f(kp, sb_key_index(lane, d, head_dim)), dot);
      s = dot * scale;
      if (r1) s -= b1 * log1pf(b2 * float(pos - j));
    }
    const float cm = wave_max(s);
    const float m_new = fmaxf(m, cm);
    const float p = visible ? expf(s - m_new) : 0.0f;
    const float alpha = expf(m - m_new);  // 0 for the first chunk
    l = l * alpha + wave_sum(p);
    ps[lane] = p;
    __syncthreads();
    const int j1 = min(pos - c * SB_PAGE, SB_PAGE - 1);
#pragma unroll
    for (int i = 0; i < kMaxHeadDim / 64; ++i) {
      const int d = lane + 64 * i;
      if (d < v_dim) {
        float acc = o[i] * alpha;
        for (int jj = 0; jj <= j1; ++jj) acc = fmaf(ps[jj], ld_f(vp, sb_value_index(d, jj)), acc);
        o[i] = acc;
      }
    }
    __syncthreads();
    m = m_new;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
  for (int i = 0; i < kMaxHeadDim / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < v_dim) out[((size_t(row) * heads_q + g) * heads_kv + vh) * v_dim + d] = o[i] * inv;
  }
}

// out[row, h, e] = sum over g of mix[h, g] * o[row, g, kv(h), e], in ascending g
__global__ void __launch_bounds__(256)
head_mix_kernel(void *__restrict__ out, int out_dtype, const void *__restrict__ o, int o_dtype, const void *__restrict__ mix,
                int mix_dtype, int heads_q, int heads_kv, int v_dim, size_t n) {
  const size_t idx = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= n) return;
  const int e = int(idx % v_dim), h = int((idx / v_dim) % heads_q);
  const size_t row = idx / (size_t(v_dim) * heads_q);
  const int vh = h / (heads_q / heads_kv);
  float acc = 0.0f;
  for (int g = 0; g < heads_q; ++g)
    acc = fmaf(mix ? ld_dyn(mix, mix_dtype, size_t(h) * heads_q + g) : (g == h ? 1.0f : 0.0f),
               ld_dyn(o, o_dtype, ((row * heads_q + g) * heads_kv + vh) * v_dim + e), acc);
  st_dyn(out, out_dtype, idx, acc);
}

}  // namespace

extern "C" int sb_qk_rownorm_store(void *q_out, int q_dtype, const float *qk, int row_stride, const void *q_w, const void *k_w,
                                   int w_dtype, float eps, float temp_coef, int temp_every, const int32_t *row_pos,
                                   const int32_t *row_seq, const int32_t *page_table, int max_pages, int n_pages, void *k_cache,
                                   void *v_cache, int cache_dtype, int n_rows, int heads_q, int heads_kv, int dk, int store,
                                   int values_from_keys, void *stream) {
  SB_REQUIRE(q_out && qk && row_pos, "sb_qk_rownorm_store: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads_q > 0 && heads_kv >= 0 && dk > 0 && row_stride >= (heads_q + (store ? heads_kv : 0)) * dk,
             "sb_qk_rownorm_store: bad sizes rows=%d heads=%d+%d dim=%d stride=%d", n_rows, heads_q, heads_kv, dk, row_stride);
  SB_REQUIRE(sb::valid_dtype(q_dtype) && (!(q_w || k_w) || sb::valid_dtype(w_dtype)), "sb_qk_rownorm_store: unknown dtype");
  SB_REQUIRE(temp_coef == 0.0f || temp_every > 0, "sb_qk_rownorm_store: the temperature's period must be positive");
  if (store) {
    SB_REQUIRE(row_seq && page_table && k_cache && max_pages > 0 && n_pages > 0 && sb::valid_dtype(cache_dtype) && heads_kv > 0,
               "sb_qk_rownorm_store: storing needs the cache and its tables");
    SB_REQUIRE(!values_from_keys || v_cache, "sb_qk_rownorm_store: no value cache");
  }
  if (n_rows == 0) return SB_OK;
  PrepArgs a{q_out, q_dtype, qk, row_stride, q_w, k_w, w_dtype, eps, temp_coef, temp_every, row_pos, row_seq, page_table,
             max_pages, n_pages, k_cache, v_cache, cache_dtype, heads_q, heads_kv, dk, store, values_from_keys};
  qk_rownorm_store_kernel<<<n_rows, 256, 0, (hipStream_t)stream>>>(a);
  return sb::check_launch("sb_qk_rownorm_store");
}

extern "C" int sb_attention_shared(float *out, const void *q, int act_dtype, const void *k_cache, const void *v_cache,
                                   int cache_dtype, const int32_t *page_table, int max_pages, int n_pages_total,
                                   const int32_t *row_pos, const int32_t *row_seq, int n_rows, int heads_q, int heads_kv,
                                   int head_dim, int v_dim, float scale, const float *r1, const float *r2, void *stream) {
  SB_REQUIRE(out && q && k_cache && v_cache && page_table && row_pos && row_seq, "sb_attention_shared: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads_q > 0 && heads_kv > 0 && heads_q % heads_kv == 0 && head_dim > 0 && v_dim > 0 &&
                 max_pages > 0 && n_pages_total > 0,
             "sb_attention_shared: bad sizes rows=%d heads_q=%d heads_kv=%d head_dim=%d", n_rows, heads_q, heads_kv, head_dim);
  SB_REQUIRE(sb::valid_dtype(act_dtype) && sb::valid_dtype(cache_dtype), "sb_attention_shared: unknown dtype");
  SB_REQUIRE((r1 == nullptr) == (r2 == nullptr), "sb_attention_shared: the distance bias needs both of its numbers");
  SB_SUPPORT(head_dim <= kMaxHeadDim && v_dim <= kMaxHeadDim, "sb_attention_shared: head sizes %d and %d are more than %d",
             head_dim, v_dim, kMaxHeadDim);
  SB_SUPPORT(heads_q <= 65535 && heads_kv <= 65535, "sb_attention_shared: more than 65535 heads");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(n_rows, heads_q, heads_kv);
#define SB_GO(TA, TC)                                                                                                 \
  attention_shared_kernel<TA, TC><<<grid, 64, 0, s>>>(out, (const TA *)q, (const TC *)k_cache, (const TC *)v_cache, \
                                                       page_table, max_pages, n_pages_total, row_pos, row_seq, heads_q, \
                                                       heads_kv, head_dim, v_dim, scale, r1, r2)
  if (act_dtype == SB_F32 && cache_dtype == SB_F32) SB_GO(float, float);
  else if (act_dtype == SB_BF16 && cache_dtype == SB_BF16) SB_GO(bf16_t, bf16_t);
  else if (act_dtype == SB_F32 && cache_dtype == SB_BF16) SB_GO(float, bf16_t);
  else SB_GO(bf16_t, float);
#undef SB_GO
  return sb::check_launch("sb_attention_shared");
}

extern "C" int sb_head_mix(void *out, int out_dtype, const void *o, int o_dtype, const void *mix, int mix_dtype, int n_rows,
                           int heads_q, int heads_kv, int v_dim, void *stream) {
  SB_REQUIRE(out && o, "sb_head_mix: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads_q > 0 && heads_kv > 0 && heads_q % heads_kv == 0 && v_dim > 0 && sb::valid_dtype(out_dtype) &&
                 sb::valid_dtype(o_dtype) && (!mix || sb::valid_dtype(mix_dtype)),
             "sb_head_mix: bad sizes rows=%d heads=%d kv=%d vdim=%d", n_rows, heads_q, heads_kv, v_dim);
  const size_t n = size_t(n_rows) * heads_q * v_dim;
  if (n == 0) return SB_OK;
  head_mix_kernel<<<unsigned((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(out, out_dtype, o, o_dtype, mix, mix_dtype, heads_q,
                                                                             heads_kv, v_dim, n);
  return sb::check_launch("sb_head_mix");
}
