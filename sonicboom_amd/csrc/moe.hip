// Routed experts: the choice, and the experts' products over the rows that chose them.
//
//   sb_moe_route    from router scores z f32 [rows, stride]: the `top` largest of the first
//                   n_experts (ties to the lower number), in falling order, and their weights, the
//                   softmax over the chosen scores alone; with has_gate also sigmoid(z[n_experts]),
//                   the multiplier of an expert that every row takes.
//                   ids int32 [rows, top]; weights f32 [rows, top + 1] (the last: the gate, or 0).
//   sb_moe_router   the router's product (float32 sums of a float32 matrix against rows of either type)
//                   and sb_moe_route's choice in one launch, a block a row.
//   sb_moe_product  Y[p,:] = X[p / x_div,:] W_e^T for every pair p = (row, choice), e = ids[p]
//                   (ids NULL: expert 0 for all); gated: W_e = [W_gate; W_up] and
//                   Y = g' sigmoid(alpha g') (u' + 1), g' = min(g, limit), u' = u cut to +-limit.
//                   The plain form: a thread an output, sums in ascending k, so a pair's bits depend
//                   on its row and expert alone.  Any sizes; f32 or bf16 operands.
#include "common.h"

namespace {

constexpr int kMaxTop = 16;

// One row's choice from its scores zr: the `top` largest in falling order (ties to the lower
// number), the softmax over them, the gate.
// score_kind 0: the weights are the softmax over the chosen z.  score_kind 1: the scores are sigmoid(z), the
// largest scores are chosen and the weights are those scores times score_scale, not renormalized.
// score_kind 2: the scores are the softmax of z over all experts; the largest are chosen (the order of z) and the
// weights are those scores times score_scale, not renormalized.
// n_groups > 1: the experts lie in that many equal groups of neighbours, a group's score is its largest score, and
// only experts of the keep_groups best groups (ties to the lower number) can be chosen.
__device__ __forceinline__ void route_row(int32_t *__restrict__ ids, float *__restrict__ weights, const float *zr, int r,
                                          int n_experts, int top, int has_gate, int score_kind = 0, float score_scale = 1.0f,
                                          int n_groups = 1, int keep_groups = 1) {
  int chosen[kMaxTop];
  float score[kMaxTop];
  unsigned long long open_groups = ~0ull;       // bit g: experts of group g can be chosen
  const int per_group = n_groups > 1 ? n_experts / n_groups : n_experts;
  if (n_groups > 1 && keep_groups < n_groups) {
    // (every kind of score rises with z, so the groups are ranked by their largest z)
    open_groups = 0ull;
    for (int k = 0; k < keep_groups; ++k) {
      int best = -1;
      float bz = 0.0f;
      for (int g = 0; g < n_groups; ++g) {
        if ((open_groups >> g) & 1ull) continue;
        float gz = -__builtin_inff();
        for (int e = g * per_group; e < (g + 1) * per_group; ++e) gz = fmaxf(gz, zr[e]);
        if (best < 0 || gz > bz) { best = g; bz = gz; }
      }
      open_groups |= 1ull << best;
    }
  }
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bz = 0.0f;
    for (int e = 0; e < n_experts; ++e) {
      if (n_groups > 1 && !((open_groups >> (e / per_group)) & 1ull)) continue;
      const float v = score_kind == 1 ? 1.0f / (1.0f + expf(-zr[e])) : zr[e];
      // candidates: below the last choice, or equal to it with a higher number (the order is
      // falling scores, rising numbers among equals); NaN scores are never chosen
      if (k > 0 && !(v < score[k - 1] || (v == score[k - 1] && e > chosen[k - 1]))) continue;
      if (best < 0 || v > bz) { best = e; bz = v; }
    }
    if (best < 0) { best = 0; bz = -__builtin_inff(); }
    chosen[k] = best;
    score[k] = bz;
  }
  float sum = 0.0f, w[kMaxTop];
  if (score_kind == 2) {
    // the softmax over all experts: the largest z of all, then the sum in ascending order of the experts
    float top_z = -__builtin_inff();
    for (int e = 0; e < n_experts; ++e) top_z = fmaxf(top_z, zr[e]);
    for (int e = 0; e < n_experts; ++e) sum += expf(zr[e] - top_z);
    for (int k = 0; k < top; ++k) w[k] = expf(score[k] - top_z);
  } else {
    for (int k = 0; k < top; ++k) { w[k] = expf(score[k] - score[0]); sum += w[k]; }
  }
  for (int k = 0; k < top; ++k) {
    ids[size_t(r) * top + k] = chosen[k];
    weights[size_t(r) * (top + 1) + k] = score_kind == 1 ? score[k] * score_scale : score_kind == 2 ? (w[k] / sum) * score_scale : w[k] / sum;
  }
  weights[size_t(r) * (top + 1) + top] = has_gate ? 1.0f / (1.0f + expf(-zr[n_experts])) : 0.0f;
}

__global__ void __launch_bounds__(64)
moe_route_kernel(int32_t *__restrict__ ids, float *__restrict__ weights, const float *__restrict__ z, int n_rows,
                 int stride, int n_experts, int top, int has_gate, int score_kind, float score_scale, int n_groups,
                 int keep_groups) {
  const int r = blockIdx.x * 64 + threadIdx.x;
  if (r >= n_rows) return;
  route_row(ids, weights, z + size_t(r) * stride, r, n_experts, top, has_gate, score_kind, score_scale, n_groups, keep_groups);
}

// The router's product and the choice in one launch: a block a row.  z_e = sum_k h[k] w[e][k] in
// float32, eight experts at a time; a thread takes the k of its place in every stretch of 256 (in
// eights when the row allows, so that a pass's loads are all in flight together), in ascending
// order, then a fixed butterfly over the wave and the four waves in ascending order: a row's scores
// depend on the row alone.  w is float32 [n_experts (+ 1), n_in], the last row the gate of the expert
// that every row takes.
__device__ __forceinline__ void load8(const float *p, float (&v)[8]) {
  const float4 a = reinterpret_cast<const float4 *>(p)[0], b = reinterpret_cast<const float4 *>(p)[1];
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t *p, float (&v)[8]) {
  const uint4 a = *reinterpret_cast<const uint4 *>(p);
  const uint32_t u[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(u[i] << 16); v[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u); }
}

template <typename TX>
__global__ void __launch_bounds__(256)
moe_router_kernel(int32_t *__restrict__ ids, float *__restrict__ weights, const TX *__restrict__ h,
                  const float *__restrict__ w, int n_rows, int n_in, int n_experts, int top, int has_gate, int score_kind,
                  float score_scale, int n_groups, int keep_groups) {
  extern __shared__ float zs[];                 // [n_z] scores, then [4][8] the waves' sums of a pass
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = blockIdx.x;
  const int n_z = n_experts + (has_gate ? 1 : 0);
  float *z = zs, *part = zs + n_z;
  const TX *hr = h + size_t(r) * n_in;
  const bool vec = n_in % 8 == 0 && (reinterpret_cast<uintptr_t>(hr) % 16 == 0) && (reinterpret_cast<uintptr_t>(w) % 16 == 0);
  for (int e0 = 0; e0 < n_z; e0 += 8) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (vec) {
      for (int k = tid * 8; k < n_in; k += 256 * 8) {
        float x[8];
        load8(hr + k, x);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (e0 + j < n_z) {
            float wv[8];
            load8(w + size_t(e0 + j) * n_in + k, wv);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[j] = fmaf(x[i], wv[i], acc[j]);
          }
        }
      }
    } else {
      for (int k = tid; k < n_in; k += 256) {
        const float x = ld_f(hr, k);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (e0 + j < n_z) acc[j] = fmaf(x, w[size_t(e0 + j) * n_in + k], acc[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float t = wave_sum(acc[j]);
      if (lane == 0) part[wave * 8 + j] = t;
    }
    __syncthreads();
    if (tid < 8 && e0 + tid < n_z) z[e0 + tid] = ((part[tid] + part[8 + tid]) + part[16 + tid]) + part[24 + tid];
    __syncthreads();
  }
  if (tid == 0) route_row(ids, weights, z, r, n_experts, top, has_gate, score_kind, score_scale, n_groups, keep_groups);
}

template <typename TO>
__global__ void swish_clamp_kernel(TO *__restrict__ out, const float *__restrict__ gu, int width, size_t n, float limit,
                                   float alpha) {
  const size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const size_t t = idx / width, i = idx % width;
  st_f(out, idx, swish_clamp_mul(gu[t * 2 * width + i], gu[t * 2 * width + width + i], limit, alpha));
}

template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(256)
moe_product_plain_kernel(TY *__restrict__ y, const TX *__restrict__ x, const TW *__restrict__ w,
                         const int32_t *__restrict__ ids, int x_div, int n_out, int n_in, int n_experts, int gated,
                         float limit, float alpha) {
  extern __shared__ float xs[];
  const int p = blockIdx.x;
  const int e = ids ? ids[p] : 0;
  const TX *xr = x + size_t(p / x_div) * n_in;
  for (int k = threadIdx.x; k < n_in; k += 256) xs[k] = ld_f(xr, k);
  __syncthreads();
  if (e < 0 || e >= n_experts) return;
  const int o = blockIdx.y * 256 + threadIdx.x;
  if (o >= n_out) return;
  const bool pair = expert_is_pair(gated);
  const size_t w_rows = size_t(pair ? 2 : 1) * n_out;
  const TW *wg = w + (size_t(e) * w_rows + o) * n_in;
  float g = 0.0f;
  for (int k = 0; k < n_in; ++k) g = fmaf(xs[k], ld_f(wg, k), g);
  if (!pair) g = expert_single(g, gated);
  if (pair) {
    const TW *wu = wg + size_t(n_out) * n_in;
    float u = 0.0f;
    for (int k = 0; k < n_in; ++k) u = fmaf(xs[k], ld_f(wu, k), u);
    g = expert_pair(g, u, gated, limit, alpha);
  }
  st_f(y, size_t(p) * n_out + o, g);
}

}  // namespace

extern "C" int sb_moe_max_top(void) { return kMaxTop; }

extern "C" int sb_moe_route_scored(int32_t *ids, float *weights, const float *z, int n_rows, int stride, int n_experts,
                                   int top, int has_gate, int score_kind, float score_scale, void *stream);
extern "C" int sb_moe_route(int32_t *ids, float *weights, const float *z, int n_rows, int stride, int n_experts,
                            int top, int has_gate, void *stream) {
  return sb_moe_route_scored(ids, weights, z, n_rows, stride, n_experts, top, has_gate, 0, 1.0f, stream);
}

extern "C" int sb_moe_route_grouped(int32_t *ids, float *weights, const float *z, int n_rows, int stride, int n_experts,
                                    int top, int has_gate, int score_kind, float score_scale, int n_groups, int keep_groups,
                                    void *stream);
extern "C" int sb_moe_route_scored(int32_t *ids, float *weights, const float *z, int n_rows, int stride, int n_experts,
                                   int top, int has_gate, int score_kind, float score_scale, void *stream) {
  return sb_moe_route_grouped(ids, weights, z, n_rows, stride, n_experts, top, has_gate, score_kind, score_scale, 1, 1, stream);
}

namespace {
// 0 when the groups fit the experts and the choice: equal groups, enough experts in the groups that stay
int check_groups(int n_experts, int top, int n_groups, int keep_groups) {
  return n_groups >= 1 && n_groups <= 64 && n_experts % n_groups == 0 && keep_groups >= 1 && keep_groups <= n_groups &&
         (n_groups == 1 || keep_groups * (n_experts / n_groups) >= top) ? 0 : 1;
}
}  // namespace

// The same with score_kind 2 (softmax over all experts, weights not renormalized) and with the experts in n_groups
// equal groups of neighbours of which the keep_groups with the largest best score can be chosen from.
extern "C" int sb_moe_route_grouped(int32_t *ids, float *weights, const float *z, int n_rows, int stride, int n_experts,
                                    int top, int has_gate, int score_kind, float score_scale, int n_groups, int keep_groups,
                                    void *stream) {
  SB_REQUIRE(ids && weights && z, "sb_moe_route: null pointer");
  SB_REQUIRE(score_kind >= 0 && score_kind <= 2, "sb_moe_route: unknown kind of score %d", score_kind);
  SB_REQUIRE(check_groups(n_experts, top, n_groups, keep_groups) == 0, "sb_moe_route: %d of %d groups do not fit %d experts and %d choices",
             keep_groups, n_groups, n_experts, top);
  SB_REQUIRE(n_rows >= 0 && n_experts > 0 && top > 0 && top <= n_experts && stride >= n_experts + (has_gate ? 1 : 0),
             "sb_moe_route: bad sizes rows=%d experts=%d top=%d stride=%d", n_rows, n_experts, top, stride);
  SB_SUPPORT(top <= kMaxTop, "sb_moe_route: %d choices a row are more than %d", top, kMaxTop);
  if (n_rows == 0) return SB_OK;
  moe_route_kernel<<<(n_rows + 63) / 64, 64, 0, (hipStream_t)stream>>>(ids, weights, z, n_rows, stride, n_experts, top, has_gate, score_kind, score_scale, n_groups, keep_groups);
  return sb::check_launch("sb_moe_route");
}

extern "C" int sb_moe_router_scored(int32_t *ids, float *weights, const void *h, int h_dtype, const float *w, int n_rows,
                                    int n_in, int n_experts, int top, int has_gate, int score_kind, float score_scale,
                                    void *stream);
extern "C" int sb_moe_router(int32_t *ids, float *weights, const void *h, int h_dtype, const float *w, int n_rows,
                             int n_in, int n_experts, int top, int has_gate, void *stream) {
  return sb_moe_router_scored(ids, weights, h, h_dtype, w, n_rows, n_in, n_experts, top, has_gate, 0, 1.0f, stream);
}

extern "C" int sb_moe_router_grouped(int32_t *ids, float *weights, const void *h, int h_dtype, const float *w, int n_rows,
                                     int n_in, int n_experts, int top, int has_gate, int score_kind, float score_scale,
                                     int n_groups, int keep_groups, void *stream);
extern "C" int sb_moe_router_scored(int32_t *ids, float *weights, const void *h, int h_dtype, const float *w, int n_rows,
                                    int n_in, int n_experts, int top, int has_gate, int score_kind, float score_scale,
                                    void *stream) {
  return sb_moe_router_grouped(ids, weights, h, h_dtype, w, n_rows, n_in, n_experts, top, has_gate, score_kind, score_scale, 1, 1,
                               stream);
}

extern "C" int sb_moe_router_grouped(int32_t *ids, float *weights, const void *h, int h_dtype, const float *w, int n_rows,
                                     int n_in, int n_experts, int top, int has_gate, int score_kind, float score_scale,
                                     int n_groups, int keep_groups, void *stream) {
  SB_REQUIRE(ids && weights && h && w, "sb_moe_router: null pointer");
  SB_REQUIRE(score_kind >= 0 && score_kind <= 2, "sb_moe_router: unknown kind of score %d", score_kind);
  SB_REQUIRE(check_groups(n_experts, top, n_groups, keep_groups) == 0, "sb_moe_router: %d of %d groups do not fit %d experts and %d choices",
             keep_groups, n_groups, n_experts, top);
  SB_REQUIRE(n_rows >= 0 && n_in > 0 && n_experts > 0 && top > 0 && top <= n_experts && sb::valid_dtype(h_dtype),
             "sb_moe_router: bad sizes rows=%d in=%d experts=%d top=%d", n_rows, n_in, n_experts, top);
  SB_SUPPORT(top <= kMaxTop && n_experts < 2048, "sb_moe_router: %d choices of %d experts are more than %d of 2047", top,
             n_experts, kMaxTop);
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = size_t(n_experts + 1 + 32) * sizeof(float);
  const unsigned blocks = n_rows;
  if (h_dtype == SB_F32) moe_router_kernel<float><<<blocks, 256, lds, s>>>(ids, weights, (const float *)h, w, n_rows, n_in, n_experts, top, has_gate, score_kind, score_scale, n_groups, keep_groups);
  else moe_router_kernel<bf16_t><<<blocks, 256, lds, s>>>(ids, weights, (const bf16_t *)h, w, n_rows, n_in, n_experts, top, has_gate, score_kind, score_scale, n_groups, keep_groups);
  return sb::check_launch("sb_moe_router");
}

// out[t,i] = g' sigmoid(alpha g') (u' + 1), g' = min(gu[t,i], limit), u' = gu[t,width+i] cut to +-limit; gu f32 [t, 2*width]
extern "C" int sb_swish_clamp_mul(void *out, int out_dtype, const float *gu, int n_rows, int width, float limit, float alpha,
                                  void *stream) {
  SB_REQUIRE(out && gu, "sb_swish_clamp_mul: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0 && sb::valid_dtype(out_dtype), "sb_swish_clamp_mul: bad sizes rows=%d width=%d", n_rows, width);
  const size_t n = size_t(n_rows) * width;
  if (n == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == SB_F32) swish_clamp_kernel<float><<<unsigned((n + 255) / 256), 256, 0, s>>>((float *)out, gu, width, n, limit, alpha);
  else swish_clamp_kernel<bf16_t><<<unsigned((n + 255) / 256), 256, 0, s>>>((bf16_t *)out, gu, width, n, limit, alpha);
  return sb::check_launch("sb_swish_clamp_mul");
}

extern "C" int sb_moe_product(void *y, int y_dtype, const void *x, int x_dtype, const void *w, int w_dtype,
                              const int32_t *ids, int n_pairs, int x_div, int n_out, int n_in, int n_experts,
                              int gated, float limit, float alpha, void *stream) {
  SB_REQUIRE(y && x && w, "sb_moe_product: null pointer");
  SB_REQUIRE(n_pairs >= 0 && x_div > 0 && n_out > 0 && n_in > 0 && n_experts > 0,
             "sb_moe_product: bad sizes pairs=%d out=%d in=%d experts=%d", n_pairs, n_out, n_in, n_experts);
  SB_REQUIRE(sb::valid_dtype(y_dtype) && sb::valid_dtype(x_dtype) && sb::valid_dtype(w_dtype), "sb_moe_product: unknown dtype");
  SB_SUPPORT(n_in <= 16384, "sb_moe_product: rows of %d are longer than 16384", n_in);
  if (n_pairs == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(n_pairs, (n_out + 255) / 256);
  const size_t lds = size_t(n_in) * sizeof(float);
#define SB_GO(TX, TW, TY)                                                                                   \
  moe_product_plain_kernel<TX, TW, TY><<<grid, 256, lds, s>>>((TY *)y, (const TX *)x, (const TW *)w, ids, x_div, \
                                                                n_out, n_in, n_experts, gated, limit, alpha)
  const int which = (x_dtype == SB_BF16 ? 4 : 0) + (w_dtype == SB_BF16 ? 2 : 0) + (y_dtype == SB_BF16 ? 1 : 0);
  switch (which) {
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
  return sb::check_launch("sb_moe_product");
}
