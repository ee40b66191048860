// Recurrences whose memory of a sequence is a matrix per head, in float32: the state-space scan
// with a scalar decay per head, and the delta rule with a decay per key channel.
//
// sb_ssd_scan (state-space duality form of a selective state space; S is N x P per head):
//     dt_t = softplus(dt_raw_t + dt_bias_a),  S_t = exp(-exp(A_log_a) dt_t) S_(t-1) + dt_t B_t x_t^T,
//     y_t = S_t^T C_t + D_a x_t,  out_t = y_t * silu(z_t)
//   head a reads B and C of group a / (heads / groups).
//
// sb_delta_scan (S is D x E per head; rows of S belong to key channels):
//     q, k made unit vectors per head (eps_unit inside the root), q also times D^(-1/2);
//     beta_t = sigmoid(b_t);  g_t = exp(-exp(A_log_a) softplus(a_t + dt_bias)) per key channel;
//     S <- g_t * S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t;
//     out_t = o_t / sqrt(mean(o_t^2) + eps) * w * sigmoid(gate_t)
//   head a reads q and k of head a / (heads / kv_heads).
//
// Both walk a sequence's rows in order, a block a (sequence, head), a thread a column of S, which
// stays in the thread's registers from the first row of the step to the last; the state of sequence
// s lies in state[slots[s]] and goes from step to step.  Every number of a row is computed by the
// same operations in the same order whatever the step it came in, so a prompt cut into steps, a
// batch and token-by-token decoding give the same bits.
#include "common.h"

namespace {

__device__ __forceinline__ float softplus_f(float a) { return a > 20.0f ? a : log1pf(expf(a)); }
__device__ __forceinline__ float sigmoid_f(float a) { return 1.0f / (1.0f + expf(-a)); }

// sum over the block's threads (blockDim.x a multiple of 64, at most 256), the same on every thread
__device__ __forceinline__ float block_sum(float v, float *scratch) {
  v = wave_sum(v);
  const int waves = blockDim.x >> 6;
  if (waves == 1) return v;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = scratch[0];
  for (int i = 1; i < waves; ++i) t += scratch[i];
  return t;
}

struct SsdArgs {
  float *out; int out_stride;
  const float *z; int z_stride;          // z_t[a * P + p]
  const float *x; int x_stride;          // x_t[a * P + p]
  const float *bc; int bc_stride;        // B_t[g * N + n], then C_t at bc + c_off
  int c_off;
  const float *dt; int dt_stride;        // dt_raw_t[a]
  const float *dt_bias, *a_log, *d_skip; // [heads]
  float *state;                          // [slots, heads, N, P]
  const int32_t *cu_rows, *slots;
  int heads, groups, N, P;
};

template <int NMAX>
__global__ void __launch_bounds__(256) ssd_scan_kernel(SsdArgs a) {
  __shared__ float bs[NMAX], cs[NMAX];
  const int seq = blockIdx.y, head = blockIdx.x, p = threadIdx.x;
  const int r0 = a.cu_rows[seq], r1 = a.cu_rows[seq + 1];
  if (r1 <= r0) return;
  const int g = head / (a.heads / a.groups);
  const bool live = p < a.P;
  float *sp = a.state + ((size_t(a.slots[seq]) * a.heads + head) * a.N) * a.P + p;
  float S[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n) S[n] = (live && n < a.N) ? sp[size_t(n) * a.P] : 0.0f;
  const float rate = expf(a.a_log[head]), bias = a.dt_bias[head], skip = a.d_skip[head];
  for (int r = r0; r < r1; ++r) {
    __syncthreads();
    for (int n = threadIdx.x; n < NMAX; n += blockDim.x) {
      bs[n] = n < a.N ? a.bc[size_t(r) * a.bc_stride + g * a.N + n] : 0.0f;
      cs[n] = n < a.N ? a.bc[size_t(r) * a.bc_stride + a.c_off + g * a.N + n] : 0.0f;
    }
    __syncthreads();
    const float dt = softplus_f(a.dt[size_t(r) * a.dt_stride + head] + bias);
    const float decay = expf(-rate * dt);
    const float xv = live ? a.x[size_t(r) * a.x_stride + head * a.P + p] : 0.0f;
    const float dx = dt * xv;
    float y = 0.0f;
#pragma unroll
    for (int n = 0; n < NMAX; ++n) {
      S[n] = fmaf(decay, S[n], bs[n] * dx);
      y = fmaf(S[n], cs[n], y);
    }
    if (live) {
      y = fmaf(skip, xv, y);
      const float zv = a.z[size_t(r) * a.z_stride + head * a.P + p];
      a.out[size_t(r) * a.out_stride + head * a.P + p] = y * (zv * sigmoid_f(zv));
    }
  }
  if (live) {
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < a.N) sp[size_t(n) * a.P] = S[n];
  }
}

struct DeltaArgs {
  void *out; int out_dtype, out_stride;  // out_t[a * E + e]
  const float *qkv; int qkv_stride;      // after the short convolution: q [G * D] | k [G * D] | v [H * E]
  const float *beta; int beta_stride;    // b_t[a] before the sigmoid
  const float *decay; int decay_stride;  // a_t[a * D + d] before bias and softplus
  const float *gate; int gate_stride;    // gate_t[a * E + e] before the sigmoid
  const float *dt_bias, *a_log;          // [heads * D], [heads]
  const void *w; int w_dtype;            // [E]
  float *state;                          // [slots, heads, D, E]
  const int32_t *cu_rows, *slots;
  int heads, kv_heads, D, E;
  float eps, eps_unit;
};

template <int DMAX>
__global__ void __launch_bounds__(256) delta_scan_kernel(DeltaArgs a) {
  __shared__ float qs[DMAX], ks[DMAX], gs[DMAX], red[4];
  const int seq = blockIdx.y, head = blockIdx.x, e = threadIdx.x;
  const int r0 = a.cu_rows[seq], r1 = a.cu_rows[seq + 1];
  if (r1 <= r0) return;
  const int kvh = head / (a.heads / a.kv_heads);
  const bool live = e < a.E;
  const int GD = a.kv_heads * a.D;
  float *sp = a.state + ((size_t(a.slots[seq]) * a.heads + head) * a.D) * a.E + e;
  float S[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = (live && d < a.D) ? sp[size_t(d) * a.E] : 0.0f;
  const float rate = expf(a.a_log[head]);
  const float q_mult = 1.0f / sqrtf(float(a.D));
  const float wv = live ? ld_dyn(a.w, a.w_dtype, e) : 0.0f;
  for (int r = r0; r < r1; ++r) {
    const float *row = a.qkv + size_t(r) * a.qkv_stride;
    // the head's query and key as unit vectors, and the decays of its key channels
    float qv = 0.0f, kv = 0.0f;
    __syncthreads();
    for (int d = threadIdx.x; d < DMAX; d += blockDim.x) {
      float q = 0.0f, k = 0.0f, g = 1.0f;
      if (d < a.D) {
        q = row[kvh * a.D + d];
        k = row[GD + kvh * a.D + d];
        g = expf(-rate * softplus_f(a.decay[size_t(r) * a.decay_stride + head * a.D + d] + a.dt_bias[head * a.D + d]));
      }
      qs[d] = q; ks[d] = k; gs[d] = g;
    }
    __syncthreads();
    // sums of squares in ascending d by every thread alike (D is small)
    float q2 = 0.0f, k2 = 0.0f;
    for (int d = 0; d < a.D; ++d) { q2 = fmaf(qs[d], qs[d], q2); k2 = fmaf(ks[d], ks[d], k2); }
    const float q_inv = q_mult / sqrtf(q2 + a.eps_unit), k_inv = 1.0f / sqrtf(k2 + a.eps_unit);
    (void)qv; (void)kv;
    const float beta = sigmoid_f(a.beta[size_t(r) * a.beta_stride + head]);
    const float v = live ? row[2 * GD + head * a.E + e] : 0.0f;
    float dot = 0.0f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      S[d] *= gs[d];
      dot = fmaf(S[d], ks[d] * k_inv, dot);
    }
    const float u = beta * (v - dot);
    float o = 0.0f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      S[d] = fmaf(ks[d] * k_inv, u, S[d]);
      o = fmaf(S[d], qs[d] * q_inv, o);
    }
    const float sq = block_sum(live ? o * o : 0.0f, red);
    const float inv = 1.0f / sqrtf(sq / float(a.E) + a.eps);
    if (live) {
      const float gate = sigmoid_f(a.gate[size_t(r) * a.gate_stride + head * a.E + e]);
      const float y = ((o * inv) * wv) * gate;
      const size_t at = size_t(r) * a.out_stride + head * a.E + e;
      if (a.out_dtype == SB_F32) ((float *)a.out)[at] = y;
      else ((bf16_t *)a.out)[at] = f32_to_bf16(y);
    }
  }
  if (live) {
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
      if (d < a.D) sp[size_t(d) * a.E] = S[d];
  }
}

}  // namespace

extern "C" int sb_state_scan_max_rows(void) { return 256; }      // rows of a head's state matrix (N, or D)
extern "C" int sb_state_scan_max_cols(void) { return 256; }      // its columns (P, or E)

extern "C" int sb_ssd_scan(float *out, int out_stride, const float *z, int z_stride, const float *x, int x_stride, const float *bc,
                           int bc_stride, int c_off, const float *dt, int dt_stride, const float *dt_bias, const float *a_log,
                           const float *d_skip, float *state, const int32_t *cu_rows, const int32_t *slots, int n_seqs, int heads,
                           int groups, int N, int P, void *stream) {
  SB_REQUIRE(out && z && x && bc && dt && dt_bias && a_log && d_skip && state && cu_rows && slots, "sb_ssd_scan: null pointer");
  SB_REQUIRE(n_seqs >= 0 && heads > 0 && groups > 0 && heads % groups == 0 && N > 0 && P > 0,
             "sb_ssd_scan: bad sizes heads=%d groups=%d state=%d vdim=%d", heads, groups, N, P);
  SB_SUPPORT(N <= 256 && P <= 256, "sb_ssd_scan: a state of %d x %d a head is more than 256 x 256", N, P);
  SB_SUPPORT(n_seqs <= 65535, "sb_ssd_scan: more than 65535 sequences");
  if (n_seqs == 0) return SB_OK;
  SsdArgs a{out, out_stride, z, z_stride, x, x_stride, bc, bc_stride, c_off, dt, dt_stride, dt_bias, a_log, d_skip, state,
            cu_rows, slots, heads, groups, N, P};
  const dim3 grid(heads, n_seqs);
  const int threads = ((P + 63) / 64) * 64;
  hipStream_t s = (hipStream_t)stream;
  if (N <= 16) ssd_scan_kernel<16><<<grid, threads, 0, s>>>(a);
  else if (N <= 32) ssd_scan_kernel<32><<<grid, threads, 0, s>>>(a);
  else if (N <= 64) ssd_scan_kernel<64><<<grid, threads, 0, s>>>(a);
  else if (N <= 128) ssd_scan_kernel<128><<<grid, threads, 0, s>>>(a);
  else ssd_scan_kernel<256><<<grid, threads, 0, s>>>(a);
  return sb::check_launch("sb_ssd_scan");
}

extern "C" int sb_delta_scan(void *out, int out_dtype, int out_stride, const float *qkv, int qkv_stride, const float *beta,
                             int beta_stride, const float *decay, int decay_stride, const float *gate, int gate_stride,
                             const float *dt_bias, const float *a_log, const void *w, int w_dtype, float *state,
                             const int32_t *cu_rows, const int32_t *slots, int n_seqs, int heads, int kv_heads, int D, int E,
                             float eps, float eps_unit, void *stream) {
  SB_REQUIRE(out && qkv && beta && decay && gate && dt_bias && a_log && w && state && cu_rows && slots, "sb_delta_scan: null pointer");
  SB_REQUIRE(n_seqs >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && D > 0 && E > 0 && sb::valid_dtype(out_dtype) &&
                 sb::valid_dtype(w_dtype),
             "sb_delta_scan: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", heads, kv_heads, D, E);
  SB_SUPPORT(D <= 256 && E <= 256, "sb_delta_scan: a state of %d x %d a head is more than 256 x 256", D, E);
  SB_SUPPORT(n_seqs <= 65535, "sb_delta_scan: more than 65535 sequences");
  if (n_seqs == 0) return SB_OK;
  DeltaArgs a{out, out_dtype, out_stride, qkv, qkv_stride, beta, beta_stride, decay, decay_stride, gate, gate_stride, dt_bias,
              a_log, w, w_dtype, state, cu_rows, slots, heads, kv_heads, D, E, eps, eps_unit};
  const dim3 grid(heads, n_seqs);
  const int threads = ((E + 63) / 64) * 64;
  hipStream_t s = (hipStream_t)stream;
  if (D <= 16) delta_scan_kernel<16><<<grid, threads, 0, s>>>(a);
  else if (D <= 32) delta_scan_kernel<32><<<grid, threads, 0, s>>>(a);
  else if (D <= 64) delta_scan_kernel<64><<<grid, threads, 0, s>>>(a);
  else if (D <= 128) delta_scan_kernel<128><<<grid, threads, 0, s>>>(a);
  else delta_scan_kernel<256><<<grid, threads, 0, s>>>(a);
  return sb::check_launch("sb_delta_scan");
}
