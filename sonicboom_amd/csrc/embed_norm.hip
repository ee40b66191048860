// Token embedding lookup and RMS norm.
//
// Formulas: /root/reference/core/src/model/emit.cpp:237-248 (row lookup, no
// scale), /root/reference/core/src/nn/norm.cpp:25-42 (eps inside the root,
// product order (x*inv)*w).  The mean of squares is accumulated in double, as
// the reference's default reduction does (/root/reference/core/src/nn/cpu_reduce.h:55-57).
#include "common.h"

namespace {

template <typename TT>
__global__ void embed_kernel(float *__restrict__ out, const TT *__restrict__ table,
                             const int32_t *__restrict__ ids, int width, int vocab) {
  const int row = blockIdx.x;
  const int id = ids[row];
  float *o = out + size_t(row) * width;
  if (id < 0 || id >= vocab) {
    for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = __uint_as_float(0x7fc00000u);
    return;
  }
  const TT *src = table + size_t(id) * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = ld_f(src, i);
}

constexpr int kNormThreads = 1024;
constexpr int kNormWaves = kNormThreads / 64;
constexpr int kNormKeep = 2;   // float4 groups of a row that a thread keeps in registers
constexpr int kMaxSlices = 8;  // K slices of a product that the fused kernel adds

// Sum of the squares of a block's kept values: per thread in ascending order, a fixed butterfly
// over the wave, then wave by wave in ascending order; all in double
// (/root/reference/core/src/nn/cpu_reduce.h:55-57 sums float products in double).
template <int WAVES = kNormWaves>
__device__ __forceinline__ double block_sum(double part) {
  __shared__ double wave_part[WAVES];
  part = wave_sum(part);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = part;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int k = 0; k < WAVES; ++k) total += wave_part[k];
  return total;
}

__device__ __forceinline__ double squares(const float4 &v) {
  return double(v.x * v.x) + double(v.y * v.y) + double(v.z * v.z) + double(v.w * v.w);
}

// Group g (four elements) of a normed row: (x * inv) * w, rounded to the output's type.  Rows and
// weights that start on 16 bytes (every tensor of the engine) take the weight and leave the
// result as one load and one store of 8 or 16 bytes; the arithmetic is the same either way.
template <typename TO>
__device__ __forceinline__ void write_normed(TO *yr, const float4 &v, int g, float inv, const void *w, int w_dtype) {
  const float x[4] = {v.x, v.y, v.z, v.w};
  float wv[4] = {1.f, 1.f, 1.f, 1.f};
  const bool aligned = ((reinterpret_cast<uintptr_t>(yr) | reinterpret_cast<uintptr_t>(w)) & 15) == 0;
  if (w) {
    if (aligned && w_dtype == SB_F32) {
      const float4 t = reinterpret_cast<const float4 *>(w)[g];
      wv[0] = t.x; wv[1] = t.y; wv[2] = t.z; wv[3] = t.w;
    } else if (aligned) {
      const uint2 t = reinterpret_cast<const uint2 *>(w)[g];
      wv[0] = bf16_to_f32(bf16_t(t.x & 0xffffu)); wv[1] = bf16_to_f32(bf16_t(t.x >> 16));
      wv[2] = bf16_to_f32(bf16_t(t.y & 0xffffu)); wv[3] = bf16_to_f32(bf16_t(t.y >> 16));
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) wv[e] = ld_dyn(w, w_dtype, g * 4 + e);
    }
  }
  float o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    o[e] = x[e] * inv;
    if (w) o[e] = o[e] * wv[e];
  }
  if (!aligned) {
#pragma unroll
    for (int e = 0; e < 4; ++e) st_f(yr, g * 4 + e, o[e]);
  } else if constexpr (sizeof(TO) == 4) {
    reinterpret_cast<float4 *>(yr)[g] = make_float4(o[0], o[1], o[2], o[3]);
  } else {
    reinterpret_cast<uint2 *>(yr)[g] = make_uint2(uint32_t(f32_to_bf16(o[0])) | uint32_t(f32_to_bf16(o[1])) << 16,
                                                   uint32_t(f32_to_bf16(o[2])) | uint32_t(f32_to_bf16(o[3])) << 16);
  }
}

// One block per row.  A thread takes float4 groups tid, tid + THREADS, ...; its loads are issued
// unconditionally (from a clamped address) so that all are in flight together, and the groups
// stay in registers for the second pass.  Rows wider than 4 * KEEP * THREADS, or not readable in
// groups of four, go through the scalar tail loops.  Few rows: 1024 threads keeping two groups
// each, to have the row's loads in flight at once; many rows of bfloat16 output: 256 threads
// keeping four, so that eight rows share a CU.
template <typename TO, int kNormThreads, int kNormKeep>
__global__ void __launch_bounds__(kNormThreads)
rmsnorm_kernel(TO *__restrict__ y, const float *__restrict__ x, const void *__restrict__ w,
               int w_dtype, const int32_t *__restrict__ rows, int width, float eps, int x_stride = 0,
               TO *__restrict__ y2 = nullptr, const void *__restrict__ w2 = nullptr) {
  // x_stride: the distance between rows of x when they are parts of wider rows (0: the width).
  // y2, w2: a second result of the same rows with a weight of its own (one root mean square for both).
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const float *xr = x + size_t(src) * (x_stride ? x_stride : width);
  TO *yr = y + size_t(r) * width;
  TO *yr2 = y2 ? y2 + size_t(r) * width : nullptr;
  const int tid = threadIdx.x;
  const bool vec = (width % 4 == 0) && (reinterpret_cast<uintptr_t>(xr) % 16 == 0);
  const int n_groups = vec ? width / 4 : 0;

  float4 keep[kNormKeep];
  double part = 0.0;
  if (n_groups > 0) {
#pragma unroll
    for (int i = 0; i < kNormKeep; ++i)
      keep[i] = reinterpret_cast<const float4 *>(xr)[min(tid + i * kNormThreads, n_groups - 1)];
#pragma unroll
    for (int i = 0; i < kNormKeep; ++i)
      if (tid + i * kNormThreads < n_groups) part += squares(keep[i]);
  }
  const int tail0 = min(n_groups, kNormKeep * kNormThreads) * 4;
  for (int i = tail0 + tid; i < width; i += kNormThreads) {
    const float v = xr[i];
    part += double(v * v);
  }
  const double total = block_sum<kNormThreads / 64>(part);
  const float mean = float(total / double(width));
  const float inv = 1.0f / sqrtf(mean + eps);
#pragma unroll
  for (int i = 0; i < kNormKeep; ++i) {
    const int g = tid + i * kNormThreads;
    if (g < n_groups) {
      write_normed(yr, keep[i], g, inv, w, w_dtype);
      if (yr2) write_normed(yr2, keep[i], g, inv, w2, w_dtype);
    }
  }
  for (int i = tail0 + tid; i < width; i += kNormThreads) {
    const float n = xr[i] * inv;
    st_f(yr, i, w ? n * ld_dyn(w, w_dtype, i) : n);
    if (yr2) st_f(yr2, i, w2 ? n * ld_dyn(w2, w_dtype, i) : n);
  }
}

// x[t,:] += sum_s partial[s][t][:] (+ bias), then optionally y[t,:] = rmsnorm(x[t,:]) * w.
// The slices are added in ascending order, then the bias, then the residual: the order of the
// unfused kernels (product, bias, residual).  width % 4 == 0 and width <= 8192 (host-checked).
// KEEP: float4 groups of the row per thread (1 for rows up to 4096 wide: nothing is loaded twice).
// SLICES: how many slices the unrolled loop loads (the count itself, or 8 for "up to 8").
template <typename TO, int KEEP, int SLICES>
__global__ void __launch_bounds__(kNormThreads)
reduce_resid_norm_kernel(TO *__restrict__ y, float *__restrict__ x, const float *__restrict__ partial,
                         int n_slices, size_t slice_stride, const void *__restrict__ bias, int bias_dtype,
                         const void *__restrict__ w, int w_dtype, int width, float eps, int do_norm) {
  const int r = blockIdx.x;
  float *xr = x + size_t(r) * width;
  const float *pr = partial + size_t(r) * width;
  const int tid = threadIdx.x;
  const int n_groups = width / 4;

  float4 keep[KEEP];
  double part = 0.0;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int g = tid + i * kNormThreads;
    const int gc = min(g, n_groups - 1);
    float4 p[SLICES];
#pragma unroll
    for (int s = 0; s < SLICES; ++s)
      p[s] = reinterpret_cast<const float4 *>(pr + min(s, n_slices - 1) * slice_stride)[gc];
    const float4 old = reinterpret_cast<const float4 *>(xr)[gc];
    float4 acc = p[0];
#pragma unroll
    for (int s = 1; s < SLICES; ++s)
      if (s < n_slices) { acc.x += p[s].x; acc.y += p[s].y; acc.z += p[s].z; acc.w += p[s].w; }
    if (bias) {
      acc.x += ld_dyn(bias, bias_dtype, gc * 4 + 0); acc.y += ld_dyn(bias, bias_dtype, gc * 4 + 1);
      acc.z += ld_dyn(bias, bias_dtype, gc * 4 + 2); acc.w += ld_dyn(bias, bias_dtype, gc * 4 + 3);
    }
    acc.x += old.x; acc.y += old.y; acc.z += old.z; acc.w += old.w;
    if (g < n_groups) {
      reinterpret_cast<float4 *>(xr)[g] = acc;
      part += squares(acc);
    }
    keep[i] = acc;
  }
  if (!do_norm) return;
  const double total = block_sum(part);
  const float mean = float(total / double(width));
  const float inv = 1.0f / sqrtf(mean + eps);
  TO *yr = y + size_t(r) * width;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int g = tid + i * kNormThreads;
    if (g < n_groups) write_normed(yr, keep[i], g, inv, w, w_dtype);
  }
}


// RMS norm in groups: the row is cut into `groups` equal consecutive parts and each is divided by
// its own sqrt(mean(part^2) + eps); the weight spans the row.  With `partial` the row is first
// updated, x[t,:] += scale * (sum of the slices in ascending order + bias).  One block of four
// waves per row.  A group belongs to one wave, or, when the row has fewer groups than the block has
// waves, to 4 / groups waves that take every such share of its elements and meet in LDS; the sums
// of squares are double and their order depends on the row's width and groups alone, so a row's
// result has the same bits whatever else the launch holds.
constexpr int kGroupThreads = 256;
constexpr int kGroupWaves = kGroupThreads / 64;

template <typename TO>
__global__ void __launch_bounds__(kGroupThreads)
group_norm_kernel(TO *__restrict__ y, float *x, const int32_t *__restrict__ rows,
                  const float *__restrict__ partial, int n_slices, size_t slice_stride,
                  const void *__restrict__ bias, int bias_dtype, float scale, const void *__restrict__ w,
                  int w_dtype, int width, int groups, float eps, int do_norm) {
  __shared__ double wave_part[kGroupWaves];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float *xr = x + size_t(src) * width;
  const float *pr = partial ? partial + size_t(r) * width : nullptr;
  TO *yr = y + size_t(r) * width;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int gw = width / groups;
  const int wpg = groups >= kGroupWaves ? 1 : kGroupWaves / groups;   // waves that share a group: 1, 2 or 4
  const int per_pass = kGroupWaves / wpg;                              // groups the block takes at a time
  // four elements a lane at a time where the parts allow it (every part a multiple of four wide, the
  // row on 16 bytes): the same sums in the same order per lane, only wider loads and stores
  const bool vec = (gw % 4 == 0) && ((reinterpret_cast<uintptr_t>(xr) | reinterpret_cast<uintptr_t>(pr) |
                                      (size_t(slice_stride) * 4)) % 16 == 0);
  for (int g0 = 0; g0 < groups; g0 += per_pass) {
    const int g = g0 + wave / wpg, k = wave % wpg;
    const bool active = g < groups;
    double part = 0.0;
    if (active && vec) {
      for (int i = 4 * (lane + 64 * k); i < gw; i += 256 * wpg) {
        const size_t e = size_t(g) * gw + i;
        float4 v;
        if (pr) {
          // every slice's load goes out before the first sum (a slice past the last is the last again, unused)
          float4 p4[kMaxSlices];
#pragma unroll
          for (int s = 0; s < kMaxSlices; ++s)
            p4[s] = *reinterpret_cast<const float4 *>(pr + size_t(min(s, n_slices - 1)) * slice_stride + e);
          float4 acc = p4[0];
#pragma unroll
          for (int s = 1; s < kMaxSlices; ++s)
            if (s < n_slices) { acc.x += p4[s].x; acc.y += p4[s].y; acc.z += p4[s].z; acc.w += p4[s].w; }
          if (bias) {
            acc.x += ld_dyn(bias, bias_dtype, e); acc.y += ld_dyn(bias, bias_dtype, e + 1);
            acc.z += ld_dyn(bias, bias_dtype, e + 2); acc.w += ld_dyn(bias, bias_dtype, e + 3);
          }
          const float4 old = *reinterpret_cast<const float4 *>(xr + e);
          v = make_float4(acc.x * scale + old.x, acc.y * scale + old.y, acc.z * scale + old.z, acc.w * scale + old.w);
          *reinterpret_cast<float4 *>(xr + e) = v;
        } else {
          v = *reinterpret_cast<const float4 *>(xr + e);
        }
        part += squares(v);
      }
    } else if (active) {
      for (int i = lane + 64 * k; i < gw; i += 64 * wpg) {
        const size_t e = size_t(g) * gw + i;
        float v;
        if (pr) {
          float acc = pr[e];
          for (int s = 1; s < n_slices; ++s) acc += pr[size_t(s) * slice_stride + e];
          if (bias) acc += ld_dyn(bias, bias_dtype, e);
          v = acc * scale + xr[e];
          xr[e] = v;
        } else {
          v = xr[e];
        }
        part += double(v * v);
      }
    }
    if (active) {
      part = wave_sum(part);
      if (lane == 0) wave_part[wave] = part;
    }
    if (!do_norm) continue;
    __syncthreads();
    if (active) {
      double total = 0.0;
      for (int j = 0; j < wpg; ++j) total += wave_part[(wave / wpg) * wpg + j];
      const float inv = 1.0f / sqrtf(float(total / double(gw)) + eps);
      if (vec) {
        for (int i = 4 * (lane + 64 * k); i < gw; i += 256 * wpg) {
          const size_t e = size_t(g) * gw + i;
          const float4 v = *reinterpret_cast<const float4 *>(xr + e);
          float o4[4] = {v.x * inv, v.y * inv, v.z * inv, v.w * inv};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (w) o4[j] = o4[j] * ld_dyn(w, w_dtype, e + j);
            st_f(yr, e + j, o4[j]);
          }
        }
      } else {
        for (int i = lane + 64 * k; i < gw; i += 64 * wpg) {
          const size_t e = size_t(g) * gw + i;
          float o = xr[e] * inv;
          if (w) o = o * ld_dyn(w, w_dtype, e);
          st_f(yr, e, o);
        }
      }
    }
    __syncthreads();
  }
}

}  // namespace

// y[r,:] = RMS norm of x[src,:] in `groups` equal consecutive parts, times w (see group_norm_kernel).
extern "C" int sb_rmsnorm_grouped(void *y, int out_dtype, const float *x, const void *w, int w_dtype,
                                  const int32_t *rows, int n_rows, int width, int groups, float eps, void *stream) {
  SB_REQUIRE(y && x, "sb_rmsnorm_grouped: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0 && groups > 0, "sb_rmsnorm_grouped: bad sizes rows=%d width=%d groups=%d",
             n_rows, width, groups);
  SB_REQUIRE(width % groups == 0, "sb_rmsnorm_grouped: %d groups do not divide a row of %d", groups, width);
  SB_REQUIRE(sb::valid_dtype(out_dtype) && (!w || sb::valid_dtype(w_dtype)), "sb_rmsnorm_grouped: unknown dtype");
  SB_REQUIRE(eps >= 0.0f, "sb_rmsnorm_grouped: eps must not be negative");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == SB_F32)
    group_norm_kernel<float><<<n_rows, kGroupThreads, 0, s>>>((float *)y, const_cast<float *>(x), rows, nullptr, 0, 0,
                                                              nullptr, 0, 1.0f, w, w_dtype, width, groups, eps, 1);
  else
    group_norm_kernel<bf16_t><<<n_rows, kGroupThreads, 0, s>>>((bf16_t *)y, const_cast<float *>(x), rows, nullptr, 0, 0,
                                                               nullptr, 0, 1.0f, w, w_dtype, width, groups, eps, 1);
  return sb::check_launch("sb_rmsnorm_grouped");
}

// x[t,:] += scale * (sum over slices of partial[s][t][:] (+ bias)); with do_norm also
// y[t,:] = the RMS norm of x[t,:] in `groups` parts, times w, in y_dtype.  Any width.
extern "C" int sb_reduce_scaled_group_norm(void *y, int y_dtype, float *x, const float *partial, int n_slices,
                                           const void *bias, int bias_dtype, float scale, const void *w, int w_dtype,
                                           int n_rows, int width, int groups, float eps, int do_norm, void *stream) {
  SB_REQUIRE(x && partial && (!do_norm || y), "sb_reduce_scaled_group_norm: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0 && n_slices >= 1 && groups > 0, "sb_reduce_scaled_group_norm: bad sizes");
  SB_SUPPORT(n_slices <= kMaxSlices, "sb_reduce_scaled_group_norm: %d slices, at most %d", n_slices, kMaxSlices);
  SB_REQUIRE(width % groups == 0, "sb_reduce_scaled_group_norm: %d groups do not divide a row of %d", groups, width);
  SB_REQUIRE((!do_norm || sb::valid_dtype(y_dtype)) && (!bias || sb::valid_dtype(bias_dtype)) &&
                 (!w || sb::valid_dtype(w_dtype)),
             "sb_reduce_scaled_group_norm: unknown dtype");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const size_t stride = size_t(n_rows) * width;
  if (!do_norm || y_dtype == SB_F32)
    group_norm_kernel<float><<<n_rows, kGroupThreads, 0, s>>>((float *)y, x, nullptr, partial, n_slices, stride, bias,
                                                              bias_dtype, scale, w, w_dtype, width, groups, eps, do_norm);
  else
    group_norm_kernel<bf16_t><<<n_rows, kGroupThreads, 0, s>>>((bf16_t *)y, x, nullptr, partial, n_slices, stride, bias,
                                                               bias_dtype, scale, w, w_dtype, width, groups, eps, do_norm);
  return sb::check_launch("sb_reduce_scaled_group_norm");
}

// The widest row sb_reduce_resid_norm takes.
extern "C" int sb_reduce_resid_norm_max_width(void) { return 4 * kNormKeep * kNormThreads; }

// x[t,:] += sum over slices of partial[s][t][:] (+ bias); with do_norm also
// y[t,:] = (x[t,:] * inv) * w in y_dtype.  partial is float [n_slices][n_rows][width].
extern "C" int sb_reduce_resid_norm(void *y, int y_dtype, float *x, const float *partial, int n_slices,
                                    const void *bias, int bias_dtype, const void *w, int w_dtype,
                                    int n_rows, int width, float eps, int do_norm, void *stream) {
  SB_REQUIRE(x && partial && (!do_norm || y), "sb_reduce_resid_norm: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0 && n_slices >= 1, "sb_reduce_resid_norm: bad sizes");
  SB_SUPPORT(n_slices <= kMaxSlices, "sb_reduce_resid_norm: %d slices, at most %d", n_slices, kMaxSlices);
  SB_REQUIRE((!do_norm || sb::valid_dtype(y_dtype)) && (!bias || sb::valid_dtype(bias_dtype)) &&
                 (!w || sb::valid_dtype(w_dtype)),
             "sb_reduce_resid_norm: unknown dtype");
  SB_SUPPORT(width % 4 == 0 && width <= sb_reduce_resid_norm_max_width(),
             "sb_reduce_resid_norm: width %d must be a multiple of 4 and at most %d", width,
             sb_reduce_resid_norm_max_width());
  SB_SUPPORT((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(partial)) % 16 == 0,
             "sb_reduce_resid_norm: operands must be 16-byte aligned");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const size_t stride = size_t(n_rows) * width;
#define SB_GO2(TO, KEEP, SLICES)                                                       \
  reduce_resid_norm_kernel<TO, KEEP, SLICES><<<n_rows, kNormThreads, 0, s>>>(         \
      (TO *)y, x, partial, n_slices, stride, bias, bias_dtype, w, w_dtype, width, eps, do_norm)
  // the usual slice counts have loops of their own length, so that no slice is loaded twice
#define SB_GO(TO, KEEP)                          \
  do {                                           \
    if (n_slices == 1) SB_GO2(TO, KEEP, 1);      \
    else if (n_slices == 2) SB_GO2(TO, KEEP, 2); \
    else if (n_slices <= 4) SB_GO2(TO, KEEP, 4); \
    else if (n_slices == 5) SB_GO2(TO, KEEP, 5); \
    else SB_GO2(TO, KEEP, kMaxSlices);           \
  } while (0)
  const bool narrow = width <= 4 * kNormThreads;
  if (!do_norm || y_dtype == SB_F32) {
    if (narrow) SB_GO(float, 1);
    else SB_GO(float, kNormKeep);
  } else {
    if (narrow) SB_GO(bf16_t, 1);
    else SB_GO(bf16_t, kNormKeep);
  }
#undef SB_GO
#undef SB_GO2
  return sb::check_launch("sb_reduce_resid_norm");
}

extern "C" int sb_embed(float *out, const void *table, int table_dtype, const int32_t *ids,
                        int n_rows, int width, int vocab, void *stream) {
  SB_REQUIRE(out && table && ids, "sb_embed: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0 && vocab > 0, "sb_embed: bad sizes rows=%d width=%d vocab=%d",
             n_rows, width, vocab);
  SB_REQUIRE(sb::valid_dtype(table_dtype), "sb_embed: unknown table dtype %d", table_dtype);
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == SB_F32)
    embed_kernel<float><<<n_rows, 256, 0, s>>>(out, (const float *)table, ids, width, vocab);
  else
    embed_kernel<bf16_t><<<n_rows, 256, 0, s>>>(out, (const bf16_t *)table, ids, width, vocab);
  return sb::check_launch("sb_embed");
}

extern "C" int sb_rmsnorm(void *y, int out_dtype, const float *x, const void *w, int w_dtype,
                          const int32_t *rows, int n_rows, int width, float eps, void *stream) {
  SB_REQUIRE(y && x, "sb_rmsnorm: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0, "sb_rmsnorm: bad sizes rows=%d width=%d", n_rows, width);
  SB_REQUIRE(sb::valid_dtype(out_dtype) && (!w || sb::valid_dtype(w_dtype)),
             "sb_rmsnorm: unknown dtype");
  SB_REQUIRE(eps >= 0.0f, "sb_rmsnorm: eps must not be negative");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  // The two block shapes sum a row's squares in different orders.  Float output is the true
  // 32-bit path, whose rows must not change by a bit with the number of rows that share the
  // launch: it keeps one shape.  bfloat16 output takes the faster shape for many rows.
  const bool many = n_rows >= 256;
  if (out_dtype == SB_F32) {
    rmsnorm_kernel<float, 1024, 2><<<n_rows, 1024, 0, s>>>((float *)y, x, w, w_dtype, rows, width, eps);
  } else {
    // (rows of 4,097 to 8,192: eight groups a thread, so that none goes through the scalar loops:
    // 2,048 rows of 8,192 27.7 us before)
    if (many && width > 4096) rmsnorm_kernel<bf16_t, 256, 8><<<n_rows, 256, 0, s>>>((bf16_t *)y, x, w, w_dtype, rows, width, eps);
    else if (many) rmsnorm_kernel<bf16_t, 256, 4><<<n_rows, 256, 0, s>>>((bf16_t *)y, x, w, w_dtype, rows, width, eps);
    else rmsnorm_kernel<bf16_t, 1024, 2><<<n_rows, 1024, 0, s>>>((bf16_t *)y, x, w, w_dtype, rows, width, eps);
  }
  return sb::check_launch("sb_rmsnorm");
}

// Two RMS norms of the same rows in one pass: y1 = (x inv) w1 and, when y2 is given, y2 = (x inv) w2,
// with one root mean square for both (two branches that read the same stream through norms of
// their own).  x_stride: the distance between rows of x (at least width), so that a part of wider
// rows can be normed where it lies.  The arithmetic of every number is sb_rmsnorm's.
extern "C" int sb_rmsnorm_pair(void *y1, void *y2, int out_dtype, const float *x, int x_stride, const void *w1,
                               const void *w2, int w_dtype, int n_rows, int width, float eps, void *stream) {
  SB_REQUIRE(y1 && x, "sb_rmsnorm_pair: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0 && x_stride >= width, "sb_rmsnorm_pair: bad sizes rows=%d width=%d stride=%d", n_rows,
             width, x_stride);
  SB_REQUIRE(sb::valid_dtype(out_dtype) && ((!w1 && !w2) || sb::valid_dtype(w_dtype)), "sb_rmsnorm_pair: unknown dtype");
  SB_REQUIRE(eps >= 0.0f, "sb_rmsnorm_pair: eps must not be negative");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const bool many = n_rows >= 256;
  if (out_dtype == SB_F32) {
    rmsnorm_kernel<float, 1024, 2><<<n_rows, 1024, 0, s>>>((float *)y1, x, w1, w_dtype, nullptr, width, eps, x_stride, (float *)y2, w2);
  } else {
    if (many && width > 4096) rmsnorm_kernel<bf16_t, 256, 8><<<n_rows, 256, 0, s>>>((bf16_t *)y1, x, w1, w_dtype, nullptr, width, eps, x_stride, (bf16_t *)y2, w2);
    else if (many) rmsnorm_kernel<bf16_t, 256, 4><<<n_rows, 256, 0, s>>>((bf16_t *)y1, x, w1, w_dtype, nullptr, width, eps, x_stride, (bf16_t *)y2, w2);
    else rmsnorm_kernel<bf16_t, 1024, 2><<<n_rows, 1024, 0, s>>>((bf16_t *)y1, x, w1, w_dtype, nullptr, width, eps, x_stride, (bf16_t *)y2, w2);
  }
  return sb::check_launch("sb_rmsnorm_pair");
}
