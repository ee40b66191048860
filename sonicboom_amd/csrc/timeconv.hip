// A short causal convolution over time, channel by channel, for the rows of a step.
//
//   y[t, c] = act(sum_j w[c, j] * in[t - taps + 1 + j, c] (+ bias[c])) (+ in[t, c] with `residual`)
//
// with in[] the rows of the sequence: those of this step, and before them the last taps - 1 inputs
// of the steps before, which are the sequence's state (float32 [slots, taps - 1, channels], zero for
// a new sequence, so that the rows before a sequence's start count as zeros).  The sum runs in
// ascending j in float32 whatever the source of an input, so a row's result is the same bits whether
// its neighbours came in the same step or in earlier ones.
//
// sb_time_conv computes the rows; sb_time_conv_keep then moves the state on (the last taps - 1
// inputs after this step).  When every sequence brings one row, `keep` = 1 makes the one launch do
// both: the thread of a row is then the only reader of its sequence's state.
#include "common.h"

namespace {

constexpr int kMaxTaps = 16;

struct ConvArgs {
  void *out; int out_dtype, out_stride;
  const void *in; int in_dtype, in_stride;
  const void *w; int w_dtype;
  const void *bias; int bias_dtype;
  float *state;
  const int32_t *row_seq, *cu_rows, *slots;
  int n_rows, channels, taps, act, residual, keep;
};

__device__ __forceinline__ void st_dyn(void *p, int dtype, size_t i, float v) {
  if (dtype == SB_F32) ((float *)p)[i] = v;
  else ((bf16_t *)p)[i] = f32_to_bf16(v);
}

// T: the taps when the kernel is compiled for their number (2 to 8), or 0 for any number up to kMaxTaps, where
// every loop runs to kMaxTaps under a test.
template <int T>
__global__ void __launch_bounds__(256) time_conv_kernel(ConvArgs a) {
  constexpr int kTop = T ? T : kMaxTaps;
  const int taps = T ? T : a.taps;
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int row = blockIdx.y;
  if (c >= a.channels) return;
  const int seq = a.row_seq[row];
  const int first = a.cu_rows[seq];
  const int r = row - first;                       // the row's number within its sequence's rows of this step
  float *st = a.state + (size_t(a.slots[seq]) * (taps - 1)) * a.channels + c;
  float in[kTop];
  // in[j]: the input taps - 1 - j rows back
#pragma unroll
  for (int j = 0; j < kTop; ++j) {
    in[j] = 0.0f;
    if (j < taps) {
      const int back = taps - 1 - j;
      if (back <= r) in[j] = ld_dyn(a.in, a.in_dtype, size_t(row - back) * a.in_stride + c);
      else in[j] = st[size_t(taps - 1 - (back - r)) * a.channels];      // state row k holds the input taps - 1 - k rows before the step
    }
  }
  float acc = 0.0f;
#pragma unroll
  for (int j = 0; j < kTop; ++j)
    if (j < taps) acc = fmaf(ld_dyn(a.w, a.w_dtype, size_t(c) * taps + j), in[j], acc);
  if (a.bias) acc += ld_dyn(a.bias, a.bias_dtype, c);
  if (a.act == 1) acc = acc / (1.0f + expf(-acc));
  float cur = 0.0f;
#pragma unroll
  for (int j = 0; j < kTop; ++j)
    if (j == taps - 1) cur = in[j];
  if (a.residual) acc += cur;
  st_dyn(a.out, a.out_dtype, size_t(row) * a.out_stride + c, acc);
  if (a.keep) {
    // one row a sequence: the state moves on by one
#pragma unroll
    for (int j = 1; j < kTop; ++j)
      if (j < taps) st[size_t(j - 1) * a.channels] = in[j];
  }
}

template <int T>
__global__ void __launch_bounds__(256) time_conv_keep_kernel(ConvArgs a) {
  constexpr int kTop = T ? T : kMaxTaps;
  const int taps = T ? T : a.taps;
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int seq = blockIdx.y;
  if (c >= a.channels) return;
  const int first = a.cu_rows[seq], n = a.cu_rows[seq + 1] - first;
  if (n <= 0) return;
  float *st = a.state + (size_t(a.slots[seq]) * (taps - 1)) * a.channels + c;
  float keep[kTop];
  // the new state row k holds the input at step row n - (taps - 1) + k; negative: an old state row
#pragma unroll
  for (int k = 0; k < kTop - 1; ++k) {
    keep[k] = 0.0f;
    if (k < taps - 1) {
      const int r = n - (taps - 1) + k;
      keep[k] = r >= 0 ? ld_dyn(a.in, a.in_dtype, size_t(first + r) * a.in_stride + c) : st[size_t(k + n) * a.channels];
    }
  }
#pragma unroll
  for (int k = 0; k < kTop - 1; ++k)
    if (k < taps - 1) st[size_t(k) * a.channels] = keep[k];
}

int check_args(const ConvArgs &a, int n_seqs, const char *what) {
  SB_REQUIRE(a.in && a.state && a.cu_rows && a.slots, "%s: null pointer", what);
  SB_REQUIRE(a.n_rows >= 0 && n_seqs >= 0 && a.channels > 0 && a.in_stride >= a.channels, "%s: bad sizes rows=%d channels=%d", what,
             a.n_rows, a.channels);
  SB_SUPPORT(a.taps >= 2 && a.taps <= kMaxTaps, "%s: %d taps are not between 2 and %d", what, a.taps, kMaxTaps);
  SB_REQUIRE(sb::valid_dtype(a.in_dtype), "%s: unknown dtype", what);
  SB_SUPPORT(a.n_rows <= 65535 * 1024 && n_seqs <= 65535, "%s: too many rows or sequences", what);
  return SB_OK;
}

}  // namespace

extern "C" int sb_time_conv_max_taps(void) { return kMaxTaps; }

extern "C" int sb_time_conv(void *out, int out_dtype, int out_stride, const void *in, int in_dtype, int in_stride, const void *w,
                            int w_dtype, const void *bias, int bias_dtype, float *state, const int32_t *row_seq,
                            const int32_t *cu_rows, const int32_t *slots, int n_rows, int n_seqs, int channels, int taps, int act,
                            int residual, int keep, void *stream) {
  ConvArgs a{out, out_dtype, out_stride, in, in_dtype, in_stride, w, w_dtype, bias, bias_dtype, state, row_seq, cu_rows, slots,
             n_rows, channels, taps, act, residual, keep};
  if (int e = check_args(a, n_seqs, "sb_time_conv")) return e;
  SB_REQUIRE(out && w && row_seq, "sb_time_conv: null pointer");
  SB_REQUIRE(sb::valid_dtype(out_dtype) && sb::valid_dtype(w_dtype) && (!bias || sb::valid_dtype(bias_dtype)) && out_stride >= channels,
             "sb_time_conv: bad output or weights");
  SB_REQUIRE(act == 0 || act == 1, "sb_time_conv: unknown activation %d", act);
  SB_REQUIRE(!keep || n_rows == n_seqs, "sb_time_conv: the state moves on in the same launch only when every sequence brings one row");
  SB_SUPPORT(n_rows <= 65535, "sb_time_conv: more than 65535 rows in one launch");
  if (n_rows == 0) return SB_OK;
  const dim3 grid((channels + 255) / 256, n_rows);
  hipStream_t s = (hipStream_t)stream;
  switch (taps) {
    case 2: time_conv_kernel<2><<<grid, 256, 0, s>>>(a); break;
    case 3: time_conv_kernel<3><<<grid, 256, 0, s>>>(a); break;
    case 4: time_conv_kernel<4><<<grid, 256, 0, s>>>(a); break;
    case 5: time_conv_kernel<5><<<grid, 256, 0, s>>>(a); break;
    case 6: time_conv_kernel<6><<<grid, 256, 0, s>>>(a); break;
    case 7: time_conv_kernel<7><<<grid, 256, 0, s>>>(a); break;
    case 8: time_conv_kernel<8><<<grid, 256, 0, s>>>(a); break;
    default: time_conv_kernel<0><<<grid, 256, 0, s>>>(a);
  }
  return sb::check_launch("sb_time_conv");
}

extern "C" int sb_time_conv_keep(const void *in, int in_dtype, int in_stride, float *state, const int32_t *cu_rows,
                                 const int32_t *slots, int n_rows, int n_seqs, int channels, int taps, void *stream) {
  ConvArgs a{nullptr, 0, 0, in, in_dtype, in_stride, nullptr, 0, nullptr, 0, state, nullptr, cu_rows, slots, n_rows, channels, taps, 0, 0, 0};
  if (int e = check_args(a, n_seqs, "sb_time_conv_keep")) return e;
  if (n_rows == 0 || n_seqs == 0) return SB_OK;
  const dim3 grid((channels + 255) / 256, n_seqs);
  hipStream_t s = (hipStream_t)stream;
  switch (taps) {
    case 2: time_conv_keep_kernel<2><<<grid, 256, 0, s>>>(a); break;
    case 3: time_conv_keep_kernel<3><<<grid, 256, 0, s>>>(a); break;
    case 4: time_conv_keep_kernel<4><<<grid, 256, 0, s>>>(a); break;
    case 5: time_conv_keep_kernel<5><<<grid, 256, 0, s>>>(a); break;
    case 6: time_conv_keep_kernel<6><<<grid, 256, 0, s>>>(a); break;
    case 7: time_conv_keep_kernel<7><<<grid, 256, 0, s>>>(a); break;
    case 8: time_conv_keep_kernel<8><<<grid, 256, 0, s>>>(a); break;
    default: time_conv_keep_kernel<0><<<grid, 256, 0, s>>>(a);
  }
  return sb::check_launch("sb_time_conv_keep");
}
