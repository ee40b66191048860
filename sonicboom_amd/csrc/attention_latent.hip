// Latent attention: a layer keeps one compressed row per token, [c | r] with c the normed latent
// (kv_rank numbers) and r a rotated key part (rot_dim numbers) that all heads share; head a's key
// is [W_uk,a c | r] and its value W_uv,a c.
//
// The kernels run it in the latent's own space, which is all the cache holds:
//   score(t, s, a) = scale * (q_plain,a(t) . W_uk,a c_s + q_rot,a(t) . r_s)
//                  = scale * ([W_uk,a^T q_plain,a(t) | q_rot,a(t)] . [c_s | r_s])
//   out(t, a)      = W_uv,a (sum_s p(t, s, a) c_s)
// so a query is first carried into the latent space (sb_head_product with W_uk), attention runs
// over the cached rows with one shared "head" of keys and values (sb_latent_attention), and the
// result goes through W_uv (sb_head_product again, which also applies the output gate).  No key
// or value of a head is ever built.
//
//   sb_latent_prepare    a step's rows of the input product: norm and store c, rotate and store r,
//                        rotate the queries' rotated parts, split off their plain parts
//   sb_head_product      out[t, a, :] = W[a] in[t, a, :], one small matrix per head
//   sb_latent_attention  one wave per (row, head), 64 keys at a time, softmax in float32 whose
//                        order of sums depends on key positions only: the 32-bit path, and the
//                        bfloat16 path for sizes the matrix-core kernel does not take
#include "common.h"

namespace {

constexpr int kPrepThreads = 256;
constexpr int kMaxLatent = 1024;   // kv_rank + rot_dim the plain attention kernel takes
constexpr int kMaxRankRegs = 16;   // kv_rank <= 64 * this

// Pair j of a vector of `dims` rotated numbers: its two indices, interleaved (2j, 2j + 1) or in
// halves (j, j + dims / 2).
__device__ __forceinline__ void pair_index(int j, int dims, int interleaved, int &i0, int &i1) {
  if (interleaved) { i0 = 2 * j; i1 = 2 * j + 1; }
  else { i0 = j; i1 = j + dims / 2; }
}

template <typename TA, typename TC>
__global__ void __launch_bounds__(kPrepThreads)
latent_prepare_kernel(TA *__restrict__ q_plain, TA *__restrict__ q_latent, const float *__restrict__ p, int row_stride,
                      int q_off, int kv_off, const void *__restrict__ c_weight, int c_w_dtype, float eps,
                      const float *__restrict__ inv_freq, int rot_dims, int interleaved,
                      const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seq, TC *__restrict__ cache,
                      const int32_t *__restrict__ page_table, int max_pages, int n_pages_total, int heads, int dim,
                      int rot_dim, int rank, const float *__restrict__ kv_rows, int kv_stride, float magnitude) {
  // kv_rows (or NULL: p): the rows that hold the latent's part at kv_off, when the queries come from a
  // product of their own; magnitude: multiplies every cosine and sine
  __shared__ double wave_part[kPrepThreads / 64];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int pos = row_pos[row];
  const float *pr = p + size_t(row) * row_stride;
  const int latent = rank + rot_dim;
  const float fpos = float(pos);

  if (kv_off >= 0) {                                  // this layer keeps its own latent: norm, rotate, store
    const float *kv = (kv_rows ? kv_rows + size_t(row) * kv_stride : pr) + kv_off;
    double part = 0.0;
    for (int i = tid; i < rank; i += kPrepThreads) part += double(kv[i] * kv[i]);
    part = wave_sum(part);
    if ((tid & 63) == 0) wave_part[tid >> 6] = part;
    __syncthreads();
    double total = 0.0;
#pragma unroll
    for (int k = 0; k < kPrepThreads / 64; ++k) total += wave_part[k];
    const float inv = 1.0f / sqrtf(float(total / double(rank)) + eps);
    const int seq = row_seq[row];
    const int lp = pos / SB_PAGE;
    const int page = lp < max_pages ? page_table[size_t(seq) * max_pages + lp] : -1;
    if (page >= 0 && page < n_pages_total) {          // a row without a page (padding) stores nothing
      TC *dst = cache + (size_t(page) * SB_PAGE + pos % SB_PAGE) * latent;
      for (int i = tid; i < rank; i += kPrepThreads) {
        float o = kv[i] * inv;
        if (c_weight) o = o * ld_dyn(c_weight, c_w_dtype, i);
        st_f(dst, i, o);
      }
      const float *r = kv + rank;
      for (int j = tid; j < rot_dims / 2; j += kPrepThreads) {
        int i0, i1;
        pair_index(j, rot_dims, interleaved, i0, i1);
        const float a = fpos * inv_freq[j];
        float y0, y1;
        if (magnitude == 1.0f) rotate_pair(r[i0], r[i1], cosf(a), sinf(a), y0, y1);
        else rotate_pair(r[i0], r[i1], cosf(a) * magnitude, sinf(a) * magnitude, y0, y1);
        st_f(dst, rank + i0, y0);
        st_f(dst, rank + i1, y1);
      }
      for (int i = rot_dims + tid; i < rot_dim; i += kPrepThreads) st_f(dst, rank + i, r[i]);
    }
  }

  // queries: head a is [dim plain | rot_dim rotated]
  const float *q = pr + q_off;
  const int hd = dim + rot_dim;
  for (int e = tid; e < heads * dim; e += kPrepThreads) {
    const int a = e / dim, d = e - a * dim;
    st_f(q_plain, (size_t(row) * heads + a) * dim + d, q[a * hd + d]);
  }
  const int half = rot_dims / 2;
  for (int e = tid; e < heads * half; e += kPrepThreads) {
    const int a = e / half, j = e - a * half;
    int i0, i1;
    pair_index(j, rot_dims, interleaved, i0, i1);
    const float *qr = q + a * hd + dim;
    const float ang = fpos * inv_freq[j];
    float y0, y1;
    if (magnitude == 1.0f) rotate_pair(qr[i0], qr[i1], cosf(ang), sinf(ang), y0, y1);
    else rotate_pair(qr[i0], qr[i1], cosf(ang) * magnitude, sinf(ang) * magnitude, y0, y1);
    TA *dst = q_latent + (size_t(row) * heads + a) * latent + rank;
    st_f(dst, i0, y0);
    st_f(dst, i1, y1);
  }
  const int rest = rot_dim - rot_dims;
  for (int e = tid; e < heads * rest; e += kPrepThreads) {
    const int a = e / rest, i = rot_dims + (e - a * rest);
    st_f(q_latent, (size_t(row) * heads + a) * latent + rank + i, q[a * hd + dim + i]);
  }
}

// out[t, a, o] = sum_i W[a][o][i] in[t, a, i]  (times sigmoid(gate[t, a * n_out + o]) when gated).
// A block takes kHeadRows rows of one head; the rows' inputs wait in LDS, a thread owns output
// columns and sums in ascending i from zero, so an element's bits do not depend on the batch.
constexpr int kHeadRows = 8;
constexpr int kHeadThreads = 256;

template <typename TO, typename TI, typename TW>
__global__ void __launch_bounds__(kHeadThreads)
head_product_kernel(TO *__restrict__ out, int out_stride, int out_hstride, const TI *__restrict__ in, int in_stride,
                    int in_hstride, const TW *__restrict__ w, const float *__restrict__ gate, int gate_stride,
                    int n_rows, int n_in, int n_out, int gate_per_head) {
  extern __shared__ float xin[];                    // [kHeadRows][n_in]
  const int a = blockIdx.y;
  const int t0 = blockIdx.x * kHeadRows;
  const int nt = min(kHeadRows, n_rows - t0);
  for (int e = threadIdx.x; e < kHeadRows * n_in; e += kHeadThreads) {
    const int r = e / n_in, i = e - r * n_in;
    xin[e] = r < nt ? ld_f(in, size_t(t0 + r) * in_stride + size_t(a) * in_hstride + i) : 0.0f;
  }
  __syncthreads();
  const TW *wa = w + size_t(a) * n_in * n_out;
  for (int o = threadIdx.x; o < n_out; o += kHeadThreads) {
    float acc[kHeadRows];
#pragma unroll
    for (int r = 0; r < kHeadRows; ++r) acc[r] = 0.0f;
    const TW *wr = wa + size_t(o) * n_in;
    for (int i = 0; i < n_in; ++i) {
      const float wv = ld_f(wr, i);
#pragma unroll
      for (int r = 0; r < kHeadRows; ++r) acc[r] = fmaf(xin[r * n_in + i], wv, acc[r]);
    }
#pragma unroll
    for (int r = 0; r < kHeadRows; ++r) {
      if (r >= nt) break;
      float v = acc[r];
      if (gate) {
        const float g = gate[size_t(t0 + r) * gate_stride + (gate_per_head ? size_t(a) : size_t(a) * n_out + o)];
        v = v * (1.0f / (1.0f + expf(-g)));
      }
      st_f(out, size_t(t0 + r) * out_stride + size_t(a) * out_hstride + o, v);
    }
  }
}

// Attention of every row over its sequence's cached latent rows: row r at position p sees the
// rows j with j <= p and (window == 0 or p - j < window).  Keys are taken 64 at a time in chunks
// at absolute positions [64 c, 64 c + 64), lane l owning key 64 c + l; maximum, sum and output
// accumulate chunk after chunk and inside a chunk key after key, so a row's arithmetic is a
// function of its position and window alone.
template <typename TA, typename TC>
__global__ void __launch_bounds__(64)
latent_attention_kernel(TA *__restrict__ out, const TA *__restrict__ q, const TC *__restrict__ cache,
                        const int32_t *__restrict__ page_table, int max_pages, int n_pages_total,
                        const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seq, int heads, int rank,
                        int rot_dim, float scale, int window) {
  __shared__ float qs[kMaxLatent];
  __shared__ float ps[64];
  const int row = blockIdx.x, a = blockIdx.y, lane = threadIdx.x;
  const int pos = row_pos[row], seq = row_seq[row];
  const int latent = rank + rot_dim;
  for (int d = lane; d < latent; d += 64) qs[d] = ld_f(q, (size_t(row) * heads + a) * latent + d);
  __syncthreads();

  const int lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  const float neg_inf = -__builtin_inff();
  float m = neg_inf, l = 0.0f;
  float o[kMaxRankRegs];
#pragma unroll
  for (int i = 0; i < kMaxRankRegs; ++i) o[i] = 0.0f;

  for (int c = lo / SB_PAGE; c <= pos / SB_PAGE; ++c) {
    const int page = c < max_pages ? page_table[size_t(seq) * max_pages + c] : -1;
    if (page < 0 || page >= n_pages_total) continue;  // uniform over the wave
    const TC *rows = cache + size_t(page) * SB_PAGE * latent;
    const int j = c * SB_PAGE + lane;
    const bool visible = j >= lo && j <= pos;
    float s = neg_inf;
    if (visible) {
      const TC *kr = rows + size_t(lane) * latent;
      float dot = 0.0f;
      for (int d = 0; d < latent; ++d) dot = fmaf(qs[d], ld_f(kr, d), dot);
      s = dot * scale;
    }
    const float cm = wave_max(s);
    const float m_new = fmaxf(m, cm);
    const float pj = visible ? expf(s - m_new) : 0.0f;
    const float alpha = expf(m - m_new);  // 0 for the first chunk
    l = l * alpha + wave_sum(pj);
    ps[lane] = pj;
    __syncthreads();
    const int j0 = max(lo - c * SB_PAGE, 0), j1 = min(pos - c * SB_PAGE, SB_PAGE - 1);
#pragma unroll
    for (int i = 0; i < kMaxRankRegs; ++i) {
      const int d = lane + 64 * i;
      if (d < rank) {
        float acc = o[i] * alpha;
        for (int jj = j0; jj <= j1; ++jj) acc = fmaf(ps[jj], ld_f(rows, size_t(jj) * latent + d), acc);
        o[i] = acc;
      }
    }
    __syncthreads();
    m = m_new;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
  for (int i = 0; i < kMaxRankRegs; ++i) {
    const int d = lane + 64 * i;
    if (d < rank) st_f(out, (size_t(row) * heads + a) * rank + d, o[i] * inv);
  }
}

}  // namespace

// A step's rows of a latent-attention layer's input product, p f32 [n_rows, row_stride]:
//   queries at q_off, head a = [dim plain | rot_dim rotated]: the plain parts go to
//     q_plain [n_rows, heads, dim], the rotated parts, rotated, to q_latent [n_rows, heads,
//     rank + rot_dim] behind the first rank numbers (which sb_head_product fills);
//   at kv_off (or -1: the layer reads another layer's rows and stores nothing) rank numbers that
//     are RMS-normed (weight c_weight, eps) and rot_dim that are rotated, stored as the row
//     [c | r] of the row's position in cache [pages, SB_PAGE, rank + rot_dim].
// The first rot_dims of the rot_dim numbers turn, pair j by the angle float(pos) * inv_freq[j];
// pairs are (2j, 2j + 1) when interleaved, else (j, j + rot_dims / 2).
extern "C" int sb_latent_prepare_split(void *q_plain, void *q_latent, int act_dtype, const float *p, int row_stride,
                                       int q_off, const float *kv_rows, int kv_stride, int kv_off, const void *c_weight,
                                       int c_w_dtype, float eps, const float *inv_freq, int rot_dims, int interleaved,
                                       float magnitude, const int32_t *row_pos, const int32_t *row_seq, void *cache,
                                       int cache_dtype, const int32_t *page_table, int max_pages, int n_pages_total,
                                       int n_rows, int heads, int dim, int rot_dim, int rank, void *stream);
extern "C" int sb_latent_prepare(void *q_plain, void *q_latent, int act_dtype, const float *p, int row_stride,
                                 int q_off, int kv_off, const void *c_weight, int c_w_dtype, float eps,
                                 const float *inv_freq, int rot_dims, int interleaved, const int32_t *row_pos,
                                 const int32_t *row_seq, void *cache, int cache_dtype, const int32_t *page_table,
                                 int max_pages, int n_pages_total, int n_rows, int heads, int dim, int rot_dim,
                                 int rank, void *stream) {
  return sb_latent_prepare_split(q_plain, q_latent, act_dtype, p, row_stride, q_off, nullptr, 0, kv_off, c_weight, c_w_dtype,
                                 eps, inv_freq, rot_dims, interleaved, 1.0f, row_pos, row_seq, cache, cache_dtype, page_table,
                                 max_pages, n_pages_total, n_rows, heads, dim, rot_dim, rank, stream);
}

// The same with the latent's part read at kv_off of rows of their own, kv_rows f32 [n_rows, kv_stride] (NULL: of p,
// as above), for mixers whose queries come out of a second product, and with every cosine and sine times `magnitude`.
extern "C" int sb_latent_prepare_split(void *q_plain, void *q_latent, int act_dtype, const float *p, int row_stride,
                                       int q_off, const float *kv_rows, int kv_stride, int kv_off, const void *c_weight,
                                       int c_w_dtype, float eps, const float *inv_freq, int rot_dims, int interleaved,
                                       float magnitude, const int32_t *row_pos, const int32_t *row_seq, void *cache,
                                       int cache_dtype, const int32_t *page_table, int max_pages, int n_pages_total,
                                       int n_rows, int heads, int dim, int rot_dim, int rank, void *stream) {
  SB_REQUIRE(q_plain && q_latent && p && row_pos && row_seq, "sb_latent_prepare: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads > 0 && dim > 0 && rot_dim >= 0 && rank > 0, "sb_latent_prepare: bad sizes");
  SB_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= rot_dim, "sb_latent_prepare: %d of %d numbers rotate",
             rot_dims, rot_dim);
  SB_REQUIRE(rot_dims == 0 || inv_freq, "sb_latent_prepare: a rotation needs its table");
  SB_REQUIRE(q_off >= 0 && q_off + heads * (dim + rot_dim) <= row_stride &&
                 (kv_off < 0 || kv_off + rank + rot_dim <= (kv_rows ? kv_stride : row_stride)),
             "sb_latent_prepare: the parts do not fit a row of %d", row_stride);
  SB_REQUIRE(kv_off < 0 || (cache && page_table && max_pages > 0 && n_pages_total > 0),
             "sb_latent_prepare: a layer that stores needs its cache and page table");
  SB_REQUIRE(sb::valid_dtype(act_dtype) && (kv_off < 0 || sb::valid_dtype(cache_dtype)) &&
                 (!c_weight || sb::valid_dtype(c_w_dtype)),
             "sb_latent_prepare: unknown dtype");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
#define SB_GO(TA, TC)                                                                                         \
  latent_prepare_kernel<TA, TC><<<n_rows, kPrepThreads, 0, s>>>(                                              \
      (TA *)q_plain, (TA *)q_latent, p, row_stride, q_off, kv_off, c_weight, c_w_dtype, eps, inv_freq, rot_dims, \
      interleaved, row_pos, row_seq, (TC *)cache, page_table, max_pages, n_pages_total, heads, dim, rot_dim, rank, \
      kv_rows, kv_stride, magnitude)
  const int cdt = kv_off < 0 ? act_dtype : cache_dtype;
  if (act_dtype == SB_F32 && cdt == SB_F32) SB_GO(float, float);
  else if (act_dtype == SB_BF16 && cdt == SB_BF16) SB_GO(bf16_t, bf16_t);
  else if (act_dtype == SB_F32 && cdt == SB_BF16) SB_GO(float, bf16_t);
  else SB_GO(bf16_t, float);
#undef SB_GO
  return sb::check_launch("sb_latent_prepare");
}

// out[t, a, o] = sum_i W[a][o][i] in[t, a, i] for heads a, W [heads, n_out, n_in];
// element (t, a, .) of out lies at t * out_stride + a * out_hstride, of in at t * in_stride +
// a * in_hstride.  gate (f32, or NULL): the result is multiplied by sigmoid(gate[t * gate_stride +
// a * n_out + o]).  in and W of one type (f32 or bf16), out f32 or bf16.
extern "C" int sb_head_product_gated(void *out, int out_dtype, int out_stride, int out_hstride, const void *in,
                                     int in_dtype, int in_stride, int in_hstride, const void *w, int w_dtype,
                                     const float *gate, int gate_stride, int gate_per_head, int n_rows, int heads,
                                     int n_in, int n_out, void *stream);
extern "C" int sb_head_product(void *out, int out_dtype, int out_stride, int out_hstride, const void *in,
                               int in_dtype, int in_stride, int in_hstride, const void *w, int w_dtype,
                               const float *gate, int gate_stride, int n_rows, int heads, int n_in, int n_out,
                               void *stream) {
  return sb_head_product_gated(out, out_dtype, out_stride, out_hstride, in, in_dtype, in_stride, in_hstride, w, w_dtype, gate,
                               gate_stride, 0, n_rows, heads, n_in, n_out, stream);
}

// The same with gate_per_head: the gate holds one number a head, gate[t * gate_stride + a], for all of the
// head's outputs.
extern "C" int sb_head_product_gated(void *out, int out_dtype, int out_stride, int out_hstride, const void *in,
                                     int in_dtype, int in_stride, int in_hstride, const void *w, int w_dtype,
                                     const float *gate, int gate_stride, int gate_per_head, int n_rows, int heads,
                                     int n_in, int n_out, void *stream) {
  SB_REQUIRE(out && in && w, "sb_head_product: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads > 0 && n_in > 0 && n_out > 0, "sb_head_product: bad sizes");
  SB_REQUIRE(sb::valid_dtype(out_dtype) && sb::valid_dtype(in_dtype) && sb::valid_dtype(w_dtype),
             "sb_head_product: unknown dtype");
  SB_SUPPORT(heads <= 65535, "sb_head_product: more than 65535 heads");
  const size_t lds = size_t(kHeadRows) * n_in * sizeof(float);
  SB_SUPPORT(lds <= 64 * 1024, "sb_head_product: inner size %d is above the limit of %d", n_in, 64 * 1024 / 4 / kHeadRows);
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((n_rows + kHeadRows - 1) / kHeadRows, heads);
#define SB_GO(TO, TI, TW)                                                                                      \
  head_product_kernel<TO, TI, TW><<<grid, kHeadThreads, lds, s>>>((TO *)out, out_stride, out_hstride, (const TI *)in, \
                                                                  in_stride, in_hstride, (const TW *)w, gate,         \
                                                                  gate_stride, n_rows, n_in, n_out, gate_per_head)
  const int key = out_dtype * 4 + in_dtype * 2 + w_dtype;
  switch (key) {
    case 0: SB_GO(float, float, float); break;
    case 1: SB_GO(float, float, bf16_t); break;
    case 2: SB_GO(float, bf16_t, float); break;
    case 3: SB_GO(float, bf16_t, bf16_t); break;
    case 4: SB_GO(bf16_t, float, float); break;
    case 5: SB_GO(bf16_t, float, bf16_t); break;
    case 6: SB_GO(bf16_t, bf16_t, float); break;
    default: SB_GO(bf16_t, bf16_t, bf16_t); break;
  }
#undef SB_GO
  return sb::check_launch("sb_head_product");
}

// out [n_rows, heads, rank] = for every row and head the softmax-weighted sum of the first `rank`
// numbers of the cached rows it sees; q [n_rows, heads, rank + rot_dim]; cache [pages, SB_PAGE,
// rank + rot_dim].
extern "C" int sb_latent_attention(void *out, const void *q, int act_dtype, const void *cache, int cache_dtype,
                                   const int32_t *page_table, int max_pages, int n_pages_total,
                                   const int32_t *row_pos, const int32_t *row_seq, int n_rows, int heads, int rank,
                                   int rot_dim, float scale, int window, void *stream) {
  SB_REQUIRE(out && q && cache && page_table && row_pos && row_seq, "sb_latent_attention: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads > 0 && rank > 0 && rot_dim >= 0 && max_pages > 0 && n_pages_total > 0 && window >= 0,
             "sb_latent_attention: bad sizes");
  SB_REQUIRE(sb::valid_dtype(act_dtype) && sb::valid_dtype(cache_dtype), "sb_latent_attention: unknown dtype");
  SB_SUPPORT(rank + rot_dim <= kMaxLatent && rank <= 64 * kMaxRankRegs,
             "sb_latent_attention: a latent row of %d + %d is above the limit of %d", rank, rot_dim, kMaxLatent);
  SB_SUPPORT(heads <= 65535, "sb_latent_attention: more than 65535 heads");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(n_rows, heads);
#define SB_GO(TA, TC)                                                                                        \
  latent_attention_kernel<TA, TC><<<grid, 64, 0, s>>>((TA *)out, (const TA *)q, (const TC *)cache, page_table, \
                                                      max_pages, n_pages_total, row_pos, row_seq, heads, rank, \
                                                      rot_dim, scale, window)
  if (act_dtype == SB_F32 && cache_dtype == SB_F32) SB_GO(float, float);
  else if (act_dtype == SB_BF16 && cache_dtype == SB_BF16) SB_GO(bf16_t, bf16_t);
  else if (act_dtype == SB_F32 && cache_dtype == SB_BF16) SB_GO(float, bf16_t);
  else SB_GO(bf16_t, float);
#undef SB_GO
  return sb::check_launch("sb_latent_attention");
}
