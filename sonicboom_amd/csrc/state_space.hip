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
// Both walk rows in order.  A thread holds up to 32 rows of two adjacent columns of S in registers, the
// lanes that share the columns sit side by side and sum by shuffles; eight rows at a time are staged in
// LDS (keys, queries, decays, values; each lane's share four floats further on, so that the lanes of a
// column read different banks), so a row costs no trip to memory of its own, and what follows the
// recurrence (gate, output norm, store) is done an element a thread after the eight rows.  The state of
// sequence s lies in state[slots[s]] and goes from step to step.
//
// Two forms.  The walk (WHOLE): a block a (sequence, head) from the sequence's first row of the step
// to its last.  Every number of a row is computed by the same operations in the same order whatever
// the step it came in, so a prompt cut into steps, a batch and token-by-token decoding give the same
// bits.  The chunked form, for long prompts, in three launches over runs ("chunks") of consecutive
// rows of one sequence, all in float32:
//   LOCAL  a block a (chunk, head): the walk from an empty matrix, which leaves the chunk's own
//          addition A_c; with it what the chunk does to the matrix that comes in: for the state
//          space one number, the product of the decays; for the delta rule the matrix M_c that the
//          same walk makes of the identity with values of zero (its D columns ride along as further
//          columns of the state), since S_out = M_c S_in + A_c;
//   carry  a sequence's chunks in order: S_in(c) is put where A_c lay, S_in(c + 1) = M_c S_in(c) + A_c,
//          and the last one is the sequence's state;
//   FROM   a block a (chunk, head): the walk from S_in(c) with the outputs.
#include "common.h"

namespace {

constexpr int RB = 8;          // rows staged in LDS at a time
constexpr int CB = 2;          // columns of S a thread holds
constexpr int CARRY_COLS = 4;  // value columns a block of the delta rule's carry moves on
enum { WHOLE = 0, LOCAL = 1, FROM = 2 };

__device__ __forceinline__ float softplus_f(float a) { return a > 20.0f ? a : log1pf(expf(a)); }
__device__ __forceinline__ float sigmoid_f(float a) { return 1.0f / (1.0f + expf(-a)); }

// the sum over the SPLIT adjacent lanes that share a column
template <int SPLIT>
__device__ __forceinline__ float lanes_sum(float v) {
#pragma unroll
  for (int off = 1; off < SPLIT; off <<= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Where element n of a staged row lies: each lane's share of SHARE elements starts four floats further on, so
// that the lanes that share a column, which read their shares at the same time, read different banks.
template <int SHARE>
__device__ __forceinline__ int staged(int n) { return n + (n / SHARE) * 4; }

// chunks of a sequence of `len` rows, and the first chunk of sequence `seq` in the list of all chunks
__device__ __forceinline__ int chunks_of(int len, int chunk_rows) { return (len + chunk_rows - 1) / chunk_rows; }
__device__ __forceinline__ int first_chunk(const int32_t *cu_rows, int seq, int chunk_rows) {
  int base = 0;
  for (int s = 0; s < seq; ++s) base += chunks_of(cu_rows[s + 1] - cu_rows[s], chunk_rows);
  return base;
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
  const int32_t *chunks;                 // [n_chunks, 4]: first row, rows, sequence, 0
  float *part;                           // [n_chunks, heads, N, P]: A_c, then S_in(c)
  float *part_decay;                     // [n_chunks, heads]: the logarithm of the chunk's product of decays
  int vec4;                              // B and C of a row can be read four numbers at a time
};

// A thread holds NMAX / SPLIT rows of CB adjacent columns of S; SPLIT adjacent lanes share the columns.
template <int NMAX, int SPLIT, int MODE>
__global__ void __launch_bounds__(256) ssd_scan_kernel(SsdArgs a) {
  constexpr int NT = NMAX / SPLIT;
  // xs holds a row's x until the row is walked and its y (with the skip) from then on
  __shared__ __attribute__((aligned(16))) float bs[RB][NMAX + 4 * SPLIT], cs[RB][NMAX + 4 * SPLIT];
  __shared__ float xs[RB][256], zs[RB][256], dts[RB], decs[RB], logs[RB];
  const int head = blockIdx.x, p0 = (threadIdx.x / SPLIT) * CB, n0 = (threadIdx.x % SPLIT) * NT;
  const int l0 = staged<NT>(n0);
  int seq, r0, r1;
  if (MODE == WHOLE) {
    seq = blockIdx.y; r0 = a.cu_rows[seq]; r1 = a.cu_rows[seq + 1];
  } else {
    const int32_t *c = a.chunks + 4 * size_t(blockIdx.y);
    r0 = c[0]; r1 = r0 + c[1]; seq = c[2];
  }
  if (r1 <= r0) return;
  const int g = head / (a.heads / a.groups);
  float *sp = MODE == WHOLE ? a.state + ((size_t(a.slots[seq]) * a.heads + head) * a.N) * a.P
                            : a.part + ((size_t(blockIdx.y) * a.heads + head) * a.N) * a.P;
  float S[CB][NT];
#pragma unroll
  for (int c = 0; c < CB; ++c)
#pragma unroll
    for (int n = 0; n < NT; ++n)
      S[c][n] = (MODE != LOCAL && p0 + c < a.P && n0 + n < a.N) ? sp[size_t(n0 + n) * a.P + p0 + c] : 0.0f;
  const float rate = expf(a.a_log[head]), bias = a.dt_bias[head], skip = a.d_skip[head];
  float log_decay = 0.0f;
  for (int rb = r0; rb < r1; rb += RB) {
    const int nr = min(RB, r1 - rb);
    __syncthreads();
    if (a.vec4) {
      // B and C of the rows, two loads of four numbers each a thread in flight
      constexpr int QUADS = NMAX / 4;
      for (int base = threadIdx.x; base < nr * QUADS; base += 2 * blockDim.x) {
        float4 bv[2], cv[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int i = base + u * blockDim.x, row = i / QUADS, n = (i % QUADS) * 4;
          const bool ok = i < nr * QUADS && n < a.N;
          const float *src = a.bc + size_t(rb + row) * a.bc_stride + g * a.N + n;
          bv[u] = ok ? *(const float4 *)src : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
          cv[u] = (MODE != LOCAL && ok) ? *(const float4 *)(src + a.c_off) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int i = base + u * blockDim.x, row = i / QUADS, n = (i % QUADS) * 4;
          if (i < nr * QUADS) {
            *(float4 *)&bs[row][staged<NT>(n)] = bv[u];
            if (MODE != LOCAL) *(float4 *)&cs[row][staged<NT>(n)] = cv[u];
          }
        }
      }
    } else {
      // B and C of the rows, four elements a thread in flight
      for (int base = threadIdx.x; base < nr * NMAX; base += 4 * blockDim.x) {
        float bv[4], cv[4];
  #pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = base + u * blockDim.x, row = i / NMAX, n = i % NMAX;
          const bool ok = i < nr * NMAX && n < a.N;
          const float *src = a.bc + size_t(rb + row) * a.bc_stride + g * a.N + n;
          bv[u] = ok ? src[0] : 0.0f;
          cv[u] = (MODE != LOCAL && ok) ? src[a.c_off] : 0.0f;
        }
  #pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = base + u * blockDim.x, row = i / NMAX, n = i % NMAX;
          if (i < nr * NMAX) {
            bs[row][staged<NT>(n)] = bv[u];
            if (MODE != LOCAL) cs[row][staged<NT>(n)] = cv[u];
          }
        }
      }
    }
    if (threadIdx.x < nr) {
      const float dt = softplus_f(a.dt[size_t(rb + threadIdx.x) * a.dt_stride + head] + bias);
      dts[threadIdx.x] = dt;
      logs[threadIdx.x] = -rate * dt;
      decs[threadIdx.x] = expf(-rate * dt);
    }
    if (n0 == 0) {
#pragma unroll
      for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int c = 0; c < CB; ++c)
          if (i < nr) {
            const bool ok = p0 + c < a.P;
            xs[i][p0 + c] = ok ? a.x[size_t(rb + i) * a.x_stride + head * a.P + p0 + c] : 0.0f;
            if (MODE != LOCAL) zs[i][p0 + c] = ok ? a.z[size_t(rb + i) * a.z_stride + head * a.P + p0 + c] : 0.0f;
          }
    }
    __syncthreads();
#pragma unroll 1
    for (int i = 0; i < nr; ++i) {
      const float dt = dts[i], decay = decs[i];
      if (MODE == LOCAL) log_decay += logs[i];
      float xv[CB], dx[CB], y[CB];
#pragma unroll
      for (int c = 0; c < CB; ++c) { xv[c] = xs[i][p0 + c]; dx[c] = dt * xv[c]; y[c] = 0.0f; }
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const float b = bs[i][l0 + n], cc = MODE != LOCAL ? cs[i][l0 + n] : 0.0f;
#pragma unroll
        for (int c = 0; c < CB; ++c) {
          S[c][n] = fmaf(decay, S[c][n], b * dx[c]);
          if (MODE != LOCAL) y[c] = fmaf(S[c][n], cc, y[c]);
        }
      }
      if (MODE != LOCAL) {
#pragma unroll
        for (int c = 0; c < CB; ++c) {
          const float yy = fmaf(skip, xv[c], lanes_sum<SPLIT>(y[c]));
          if (n0 == 0) xs[i][p0 + c] = yy;         // the lanes that share the column have read x by now
        }
      }
    }
    if (MODE != LOCAL) {
      // the gate and the store, an element a thread
      __syncthreads();
      for (int i = 0; i < nr; ++i)
        for (int p = threadIdx.x; p < a.P; p += blockDim.x) {
          const float zv = zs[i][p];
          a.out[size_t(rb + i) * a.out_stride + head * a.P + p] = xs[i][p] * (zv * sigmoid_f(zv));
        }
    }
  }
  if (MODE != FROM) {
#pragma unroll
    for (int c = 0; c < CB; ++c)
#pragma unroll
      for (int n = 0; n < NT; ++n)
        if (p0 + c < a.P && n0 + n < a.N) sp[size_t(n0 + n) * a.P + p0 + c] = S[c][n];
  }
  if (MODE == LOCAL && threadIdx.x == 0) a.part_decay[size_t(blockIdx.y) * a.heads + head] = log_decay;
}

// A sequence's chunks in order, a thread an element of the head's matrix: part[c] <- S_in(c),
// S_in(c + 1) = exp(log decay of c) S_in(c) + A_c, and the last one into the state.
__global__ void __launch_bounds__(256) ssd_carry_kernel(SsdArgs a, int chunk_rows) {
  const int head = blockIdx.x, seq = blockIdx.y;
  const int len = a.cu_rows[seq + 1] - a.cu_rows[seq];
  if (len <= 0) return;
  const int NP = a.N * a.P;
  const int e = blockIdx.z * blockDim.x + threadIdx.x;
  if (e >= NP) return;
  const int c0 = first_chunk(a.cu_rows, seq, chunk_rows), n = chunks_of(len, chunk_rows);
  float *sp = a.state + (size_t(a.slots[seq]) * a.heads + head) * NP + e;
  float cur = *sp;
  float *pp = a.part + (size_t(c0) * a.heads + head) * NP + e;
  const size_t step = size_t(a.heads) * NP;
  float add = *pp;
  for (int c = 0; c < n; ++c) {
    const float next = c + 1 < n ? pp[step] : 0.0f;
    *pp = cur;
    cur = fmaf(expf(a.part_decay[size_t(c0 + c) * a.heads + head]), cur, add);
    add = next;
    pp += step;
  }
  *sp = cur;
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
  const int32_t *chunks;                 // [n_chunks, 4]: first row, rows, sequence, 0
  float *part;                           // [n_chunks, heads, D * E + D * D]: A_c (then S_in(c)) [D, E] | M_c transposed [D, D]
  int vec4;                              // q, k, the decays and their bias can be read four numbers at a time
};

// A thread holds DMAX / SPLIT rows of CB adjacent columns of S; SPLIT adjacent lanes share the columns.
// LOCAL: blockIdx.z picks the block's columns among [values | identity]; the identity's columns leave as
// M_c transposed (element [k][d] is what row k of the matrix that comes in adds to row d).
template <int DMAX, int SPLIT, int MODE>
__global__ void __launch_bounds__(256) delta_scan_kernel(DeltaArgs a) {
  constexpr int DT = DMAX / SPLIT;
  __shared__ __attribute__((aligned(16))) float qs[MODE == LOCAL ? 1 : RB][DMAX + 4 * SPLIT], ks[RB][DMAX + 4 * SPLIT],
      gs[RB][DMAX + 4 * SPLIT];
  __shared__ float vs[RB][512], os[MODE == LOCAL ? 1 : RB][512], q_inv[RB], k_inv[RB], betas[RB], o_inv[RB];
  const int head = blockIdx.x;
  const int cl = (threadIdx.x / SPLIT) * CB, d0 = (threadIdx.x % SPLIT) * DT, l0 = staged<DT>(d0);
  const int col0 = (MODE == LOCAL ? blockIdx.z * (blockDim.x / SPLIT) * CB : 0) + cl;
  const int n_cols = MODE == LOCAL ? a.E + a.D : a.E;
  int seq, r0, r1;
  if (MODE == WHOLE) {
    seq = blockIdx.y; r0 = a.cu_rows[seq]; r1 = a.cu_rows[seq + 1];
  } else {
    const int32_t *c = a.chunks + 4 * size_t(blockIdx.y);
    r0 = c[0]; r1 = r0 + c[1]; seq = c[2];
  }
  if (r1 <= r0) return;
  const int kvh = head / (a.heads / a.kv_heads);
  const int GD = a.kv_heads * a.D;
  float *sp = MODE == WHOLE ? a.state + ((size_t(a.slots[seq]) * a.heads + head) * a.D) * a.E
                            : a.part + (size_t(blockIdx.y) * a.heads + head) * a.D * (a.E + a.D);
  float S[CB][DT];
#pragma unroll
  for (int c = 0; c < CB; ++c)
#pragma unroll
    for (int d = 0; d < DT; ++d) {
      const int col = col0 + c;
      if (MODE == LOCAL) S[c][d] = (col >= a.E && d0 + d == col - a.E) ? 1.0f : 0.0f;
      else S[c][d] = (col < a.E && d0 + d < a.D) ? sp[size_t(d0 + d) * a.E + col] : 0.0f;
    }
  const float rate = expf(a.a_log[head]);
  const float q_mult = 1.0f / sqrtf(float(a.D));
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (int rb = r0; rb < r1; rb += RB) {
    const int nr = min(RB, r1 - rb);
    __syncthreads();
    if (a.vec4) {
      // the head's queries and keys as they came, and the decays of its key channels, four numbers a load
      constexpr int QUADS = DMAX / 4;
      for (int i = threadIdx.x; i < nr * QUADS; i += blockDim.x) {
        const int row = i / QUADS, d = (i % QUADS) * 4;
        const bool ok = d < a.D;
        const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        const float *src = a.qkv + size_t(rb + row) * a.qkv_stride + kvh * a.D + d;
        const float4 qv = (MODE != LOCAL && ok) ? *(const float4 *)src : zero;
        const float4 kv = ok ? *(const float4 *)(src + GD) : zero;
        const float4 av = ok ? *(const float4 *)(a.decay + size_t(rb + row) * a.decay_stride + head * a.D + d) : zero;
        const float4 bv = ok ? *(const float4 *)(a.dt_bias + head * a.D + d) : zero;
        float4 gv = make_float4(1.0f, 1.0f, 1.0f, 1.0f);
        if (ok) {
          gv.x = expf(-rate * softplus_f(av.x + bv.x)); gv.y = expf(-rate * softplus_f(av.y + bv.y));
          gv.z = expf(-rate * softplus_f(av.z + bv.z)); gv.w = expf(-rate * softplus_f(av.w + bv.w));
        }
        const int at = staged<DT>(d);
        if (MODE != LOCAL) *(float4 *)&qs[row][at] = qv;
        *(float4 *)&ks[row][at] = kv;
        *(float4 *)&gs[row][at] = gv;
      }
    } else {
      // the head's queries and keys as they came, and the decays of its key channels; four elements a thread in flight
      for (int base = threadIdx.x; base < nr * DMAX; base += 4 * blockDim.x) {
        float qv[4], kv[4], gv[4];
  #pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = base + u * blockDim.x, row = i / DMAX, d = i % DMAX;
          const bool ok = i < nr * DMAX && d < a.D;
          const float *src = a.qkv + size_t(rb + row) * a.qkv_stride + kvh * a.D + d;
          qv[u] = (MODE != LOCAL && ok) ? src[0] : 0.0f;
          kv[u] = ok ? src[GD] : 0.0f;
          gv[u] = ok ? a.decay[size_t(rb + row) * a.decay_stride + head * a.D + d] + a.dt_bias[head * a.D + d] : 0.0f;
        }
  #pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = base + u * blockDim.x, row = i / DMAX, d = i % DMAX;
          if (i < nr * DMAX) {
            if (MODE != LOCAL) qs[row][staged<DT>(d)] = qv[u];
            ks[row][staged<DT>(d)] = kv[u];
            gs[row][staged<DT>(d)] = d < a.D ? expf(-rate * softplus_f(gv[u])) : 1.0f;
          }
        }
      }
    }
    if (d0 == 0) {
#pragma unroll
      for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int c = 0; c < CB; ++c)
          if (i < nr) vs[i][cl + c] = col0 + c < a.E ? a.qkv[size_t(rb + i) * a.qkv_stride + 2 * GD + head * a.E + col0 + c] : 0.0f;
    }
    if (threadIdx.x < nr) betas[threadIdx.x] = sigmoid_f(a.beta[size_t(rb + threadIdx.x) * a.beta_stride + head]);
    __syncthreads();
    // unit vectors: a wave a row, the squares summed lane by lane and then over the wave
    for (int i = wave; i < nr; i += waves) {
      float q2 = 0.0f, k2 = 0.0f;
      for (int d = lane; d < a.D; d += 64) {
        const int at = staged<DT>(d);
        if (MODE != LOCAL) q2 = fmaf(qs[i][at], qs[i][at], q2);
        k2 = fmaf(ks[i][at], ks[i][at], k2);
      }
      k2 = wave_sum(k2);
      if (MODE != LOCAL) q2 = wave_sum(q2);
      if (lane == 0) {
        k_inv[i] = 1.0f / sqrtf(k2 + a.eps_unit);
        if (MODE != LOCAL) q_inv[i] = q_mult / sqrtf(q2 + a.eps_unit);
      }
    }
    __syncthreads();
#pragma unroll 1
    for (int i = 0; i < nr; ++i) {
      const float kn = k_inv[i], beta = betas[i];
      float dot[CB], uk[CB], o[CB];
#pragma unroll
      for (int c = 0; c < CB; ++c) dot[c] = o[c] = 0.0f;
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        const float g = gs[i][l0 + d], k = ks[i][l0 + d];
#pragma unroll
        for (int c = 0; c < CB; ++c) {
          S[c][d] *= g;
          dot[c] = fmaf(S[c][d], k, dot[c]);
        }
      }
#pragma unroll
      for (int c = 0; c < CB; ++c) uk[c] = (beta * (vs[i][cl + c] - lanes_sum<SPLIT>(dot[c]) * kn)) * kn;
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        const float k = ks[i][l0 + d], q = MODE != LOCAL ? qs[i][l0 + d] : 0.0f;
#pragma unroll
        for (int c = 0; c < CB; ++c) {
          S[c][d] = fmaf(k, uk[c], S[c][d]);
          if (MODE != LOCAL) o[c] = fmaf(S[c][d], q, o[c]);
        }
      }
      if (MODE != LOCAL) {
#pragma unroll
        for (int c = 0; c < CB; ++c) {
          const float oo = lanes_sum<SPLIT>(o[c]) * q_inv[i];
          if (d0 == 0) os[i][cl + c] = col0 + c < a.E ? oo : 0.0f;
        }
      }
    }
    if (MODE != LOCAL) {
      __syncthreads();
      for (int i = wave; i < nr; i += waves) {
        float sq = 0.0f;
        for (int e = lane; e < a.E; e += 64) sq = fmaf(os[i][e], os[i][e], sq);
        sq = wave_sum(sq);
        if (lane == 0) o_inv[i] = 1.0f / sqrtf(sq / float(a.E) + a.eps);
      }
      __syncthreads();
      // norm's weight, gate and store, an element a thread
      // (a block wider than the head takes several rows a pass)
      const int pass = max(1, int(blockDim.x) / a.E), i0 = threadIdx.x / a.E;
      for (int e = threadIdx.x - i0 * a.E; i0 < pass && e < a.E; e += blockDim.x) {
        const float wv = ld_dyn(a.w, a.w_dtype, e);
        for (int i = i0; i < nr; i += pass) {
          const float gate = sigmoid_f(a.gate[size_t(rb + i) * a.gate_stride + head * a.E + e]);
          const float y = ((os[i][e] * o_inv[i]) * wv) * gate;
          const size_t at = size_t(rb + i) * a.out_stride + head * a.E + e;
          if (a.out_dtype == SB_F32) ((float *)a.out)[at] = y;
          else ((bf16_t *)a.out)[at] = f32_to_bf16(y);
        }
      }
    }
  }
  if (MODE != FROM) {
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      const int col = col0 + c;
      if (col >= n_cols) continue;
      // a value column into [D, E]; a column of the identity into the transposed [D, D] behind it
      float *dst = col < a.E ? sp + col : sp + size_t(a.D) * a.E + size_t(col - a.E) * a.D;
      const size_t stride = col < a.E ? a.E : 1;
#pragma unroll
      for (int d = 0; d < DT; ++d)
        if (d0 + d < a.D) dst[size_t(d0 + d) * stride] = S[c][d];
    }
  }
}

// A sequence's chunks in order, a block CARRY_COLS value columns of a head, a thread a key channel d and
// CPT of the columns: part[c] <- S_in(c), S_in(c + 1) = M_c S_in(c) + A_c, the last one into the state.
// M_c lies transposed, so the lanes of a wave read neighbouring numbers.
template <int CPT>
__global__ void __launch_bounds__(256) delta_carry_kernel(DeltaArgs a, int chunk_rows, int d_threads) {
  __shared__ float s_in[256][CARRY_COLS];
  const int head = blockIdx.x, seq = blockIdx.y;
  const int len = a.cu_rows[seq + 1] - a.cu_rows[seq];
  if (len <= 0) return;
  const int d = threadIdx.x % d_threads, j0 = (threadIdx.x / d_threads) * CPT;
  const int e0 = blockIdx.z * CARRY_COLS + j0;
  const bool row_live = d < a.D;
  const int c0 = first_chunk(a.cu_rows, seq, chunk_rows), n = chunks_of(len, chunk_rows);
  float *sp = a.state + ((size_t(a.slots[seq]) * a.heads + head) * a.D + d) * a.E + e0;
  float cur[CPT];
#pragma unroll
  for (int j = 0; j < CPT; ++j) cur[j] = (row_live && e0 + j < a.E) ? sp[j] : 0.0f;
  const size_t part_size = size_t(a.D) * (a.E + a.D);
  for (int c = 0; c < n; ++c) {
    float *base = a.part + (size_t(c0 + c) * a.heads + head) * part_size;
    float *pp = base + size_t(d) * a.E + e0;
    float acc[CPT];
#pragma unroll
    for (int j = 0; j < CPT; ++j) acc[j] = (row_live && e0 + j < a.E) ? pp[j] : 0.0f;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < CPT; ++j) s_in[d][j0 + j] = cur[j];
    __syncthreads();
    if (row_live) {
#pragma unroll
      for (int j = 0; j < CPT; ++j)
        if (e0 + j < a.E) pp[j] = cur[j];
      const float *mrow = base + size_t(a.D) * a.E;     // row k of M_c transposed, the same for every thread
      for (int k0 = 0; k0 < a.D; k0 += 32) {            // 32 numbers of M_c a thread in flight
        float mv[32];
        if (k0 + 32 <= a.D) {
#pragma unroll
          for (int u = 0; u < 32; ++u) { mv[u] = mrow[d]; mrow += a.D; }
        } else {
#pragma unroll
          for (int u = 0; u < 32; ++u) { mv[u] = k0 + u < a.D ? mrow[d] : 0.0f; mrow += a.D; }
        }
#pragma unroll
        for (int u = 0; u < 32; ++u)
#pragma unroll
          for (int j = 0; j < CPT; ++j) acc[j] = fmaf(mv[u], s_in[(k0 + u) & 255][j0 + j], acc[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < CPT; ++j) cur[j] = acc[j];
  }
  if (row_live) {
#pragma unroll
    for (int j = 0; j < CPT; ++j)
      if (e0 + j < a.E) sp[j] = cur[j];
  }
}

// Lanes that share a column: as many as keep a thread's share of its columns at 32 rows, while the block's
// `cols` columns, CB a thread, still fit its 256 threads.
int lanes_a_column(int rows, int cols) {
  int split = rows > 128 ? 8 : rows > 64 ? 4 : rows > 32 ? 2 : 1;
  while (split > 1 && ((cols + CB - 1) / CB) * split > 256) split >>= 1;
  return split;
}
inline int scan_threads(int cols, int split) { return ((((cols + CB - 1) / CB) * split + 63) / 64) * 64; }

template <int MODE>
int launch_ssd(const SsdArgs &a, dim3 grid, int split, hipStream_t s) {
  const int threads = scan_threads(a.P, split);
  if (a.N <= 16 && split == 1) ssd_scan_kernel<16, 1, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.N <= 32 && split == 1) ssd_scan_kernel<32, 1, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.N <= 64 && split == 2) ssd_scan_kernel<64, 2, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.N <= 128 && split == 2) ssd_scan_kernel<128, 2, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.N <= 128 && split == 4) ssd_scan_kernel<128, 4, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.N <= 256 && split == 2) ssd_scan_kernel<256, 2, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.N <= 256 && split == 4) ssd_scan_kernel<256, 4, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.N <= 256 && split == 8) ssd_scan_kernel<256, 8, MODE><<<grid, threads, 0, s>>>(a);
  else return sb::fail(SB_ERR_UNSUPPORTED, "sb_ssd_scan: no kernel for a state of %d rows over %d lanes", a.N, split);
  return SB_OK;
}

template <int MODE>
int launch_delta(const DeltaArgs &a, dim3 grid, int threads, int split, hipStream_t s) {
  if (a.D <= 16 && split == 1) delta_scan_kernel<16, 1, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.D <= 32 && split == 1) delta_scan_kernel<32, 1, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.D <= 64 && split == 2) delta_scan_kernel<64, 2, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.D <= 128 && split == 2) delta_scan_kernel<128, 2, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.D <= 128 && split == 4) delta_scan_kernel<128, 4, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.D <= 256 && split == 2) delta_scan_kernel<256, 2, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.D <= 256 && split == 4) delta_scan_kernel<256, 4, MODE><<<grid, threads, 0, s>>>(a);
  else if (a.D <= 256 && split == 8) delta_scan_kernel<256, 8, MODE><<<grid, threads, 0, s>>>(a);
  else return sb::fail(SB_ERR_UNSUPPORTED, "sb_delta_scan: no kernel for a state of %d rows over %d lanes", a.D, split);
  return SB_OK;
}

}  // namespace

extern "C" int sb_state_scan_max_rows(void) { return 256; }      // rows of a head's state matrix (N, or D)
extern "C" int sb_state_scan_max_cols(void) { return 256; }      // its columns (P, or E)
extern "C" int sb_state_scan_chunk_rows(void) { return 64; }     // the rows of a chunk of the chunked forms

// chunks != null: the chunked form over n_chunks runs of at most chunk_rows rows, sequence after sequence in
// row order, each sequence's runs full but its last; part [n_chunks, heads, N, P] and part_decay
// [n_chunks, heads] are scratch.
extern "C" int sb_ssd_scan(float *out, int out_stride, const float *z, int z_stride, const float *x, int x_stride, const float *bc,
                           int bc_stride, int c_off, const float *dt, int dt_stride, const float *dt_bias, const float *a_log,
                           const float *d_skip, float *state, const int32_t *cu_rows, const int32_t *slots, int n_seqs, int heads,
                           int groups, int N, int P, const int32_t *chunks, int n_chunks, int chunk_rows, float *part,
                           float *part_decay, void *stream) {
  SB_REQUIRE(out && z && x && bc && dt && dt_bias && a_log && d_skip && state && cu_rows && slots, "sb_ssd_scan: null pointer");
  SB_REQUIRE(n_seqs >= 0 && heads > 0 && groups > 0 && heads % groups == 0 && N > 0 && P > 0,
             "sb_ssd_scan: bad sizes heads=%d groups=%d state=%d vdim=%d", heads, groups, N, P);
  SB_SUPPORT(N <= 256 && P <= 256, "sb_ssd_scan: a state of %d x %d a head is more than 256 x 256", N, P);
  SB_SUPPORT(n_seqs <= 65535, "sb_ssd_scan: more than 65535 sequences");
  SB_REQUIRE(!chunks || (n_chunks > 0 && chunk_rows > 0 && part && part_decay), "sb_ssd_scan: chunks without their scratch");
  SB_SUPPORT(!chunks || n_chunks <= 65535, "sb_ssd_scan: more than 65535 chunks");
  if (n_seqs == 0) return SB_OK;
  SsdArgs a{out, out_stride, z, z_stride, x, x_stride, bc, bc_stride, c_off, dt, dt_stride, dt_bias, a_log, d_skip, state,
            cu_rows, slots, heads, groups, N, P, chunks, part, part_decay,
            (N % 4 == 0 && bc_stride % 4 == 0 && c_off % 4 == 0 && (uintptr_t)bc % 16 == 0) ? 1 : 0};
  const int split = lanes_a_column(N, P);
  hipStream_t s = (hipStream_t)stream;
  if (!chunks) {
    if (int rc = launch_ssd<WHOLE>(a, dim3(heads, n_seqs), split, s)) return rc;
    return sb::check_launch("sb_ssd_scan");
  }
  if (int rc = launch_ssd<LOCAL>(a, dim3(heads, n_chunks), split, s)) return rc;
  ssd_carry_kernel<<<dim3(heads, n_seqs, (N * P + 255) / 256), 256, 0, s>>>(a, chunk_rows);
  if (int rc = launch_ssd<FROM>(a, dim3(heads, n_chunks), split, s)) return rc;
  return sb::check_launch("sb_ssd_scan (chunked)");
}

// chunks != null: the chunked form, as for sb_ssd_scan; part [n_chunks, heads, D * (E + D)] is scratch.
extern "C" int sb_delta_scan(void *out, int out_dtype, int out_stride, const float *qkv, int qkv_stride, const float *beta,
                             int beta_stride, const float *decay, int decay_stride, const float *gate, int gate_stride,
                             const float *dt_bias, const float *a_log, const void *w, int w_dtype, float *state,
                             const int32_t *cu_rows, const int32_t *slots, int n_seqs, int heads, int kv_heads, int D, int E,
                             float eps, float eps_unit, const int32_t *chunks, int n_chunks, int chunk_rows, float *part,
                             void *stream) {
  SB_REQUIRE(out && qkv && beta && decay && gate && dt_bias && a_log && w && state && cu_rows && slots, "sb_delta_scan: null pointer");
  SB_REQUIRE(n_seqs >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && D > 0 && E > 0 && sb::valid_dtype(out_dtype) &&
                 sb::valid_dtype(w_dtype),
             "sb_delta_scan: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", heads, kv_heads, D, E);
  SB_SUPPORT(D <= 256 && E <= 256, "sb_delta_scan: a state of %d x %d a head is more than 256 x 256", D, E);
  SB_SUPPORT(n_seqs <= 65535, "sb_delta_scan: more than 65535 sequences");
  SB_REQUIRE(!chunks || (n_chunks > 0 && chunk_rows > 0 && part), "sb_delta_scan: chunks without their scratch");
  SB_SUPPORT(!chunks || n_chunks <= 65535, "sb_delta_scan: more than 65535 chunks");
  if (n_seqs == 0) return SB_OK;
  DeltaArgs a{out, out_dtype, out_stride, qkv, qkv_stride, beta, beta_stride, decay, decay_stride, gate, gate_stride, dt_bias,
              a_log, w, w_dtype, state, cu_rows, slots, heads, kv_heads, D, E, eps, eps_unit, chunks, part,
              (D % 4 == 0 && qkv_stride % 4 == 0 && decay_stride % 4 == 0 && (uintptr_t)qkv % 16 == 0 && (uintptr_t)decay % 16 == 0 &&
               (uintptr_t)dt_bias % 16 == 0) ? 1 : 0};
  const int split = lanes_a_column(D, E);
  const int threads = scan_threads(E, split);
  hipStream_t s = (hipStream_t)stream;
  if (!chunks) {
    if (int rc = launch_delta<WHOLE>(a, dim3(heads, n_seqs), threads, split, s)) return rc;
    return sb::check_launch("sb_delta_scan");
  }
  // every chunk from an empty matrix: blocks of 256 threads over the columns [values | identity]
  const int local_cols = (256 / split) * CB;
  if (int rc = launch_delta<LOCAL>(a, dim3(heads, n_chunks, (E + D + local_cols - 1) / local_cols), 256, split, s)) return rc;
  const int d_threads = ((D + 63) / 64) * 64;          // 64, 128, 192 or 256
  const int per_row = d_threads == 64 ? 4 : d_threads == 128 ? 2 : 1;
  const dim3 grid(heads, n_seqs, (E + CARRY_COLS - 1) / CARRY_COLS);
  if (per_row == 4) delta_carry_kernel<CARRY_COLS / 4><<<grid, d_threads * 4, 0, s>>>(a, chunk_rows, d_threads);
  else if (per_row == 2) delta_carry_kernel<CARRY_COLS / 2><<<grid, d_threads * 2, 0, s>>>(a, chunk_rows, d_threads);
  else delta_carry_kernel<CARRY_COLS><<<grid, d_threads, 0, s>>>(a, chunk_rows, d_threads);
  if (int rc = launch_delta<FROM>(a, dim3(heads, n_chunks), threads, split, s)) return rc;
  return sb::check_launch("sb_delta_scan (chunked)");
}
