// Latent attention on the matrix cores (bfloat16): the per-head products that carry queries into
// the latent space and results out of it, and attention over the cached latent rows.
//
// sb_head_product_bf16: out[t, a, :] = W[a] in[t, a, :], W[a] [n_out, n_in] (output-major).  A wave
// takes 16 rows of one head and 64 outputs; both operands go from global memory straight into
// MFMA 16x16x32 fragments (a lane's eight k are 16 consecutive bytes on either side), the result
// lands as four consecutive outputs of one row per lane.
//
// sb_latent_attention_bf16: all query heads read the same cached rows [c | r], so a block stages
// a page of 64 rows once in LDS, twice over: as it lies (a key's numbers consecutive: the A
// operand of S^T = K Q^T) and with the latent part turned (a number's keys consecutive: the A
// operand of O^T = C^T P^T), half a page at a time in two buffers that take turns, and its eight
// waves run four tiles of 16 query columns against it, two waves a tile.
// In a prompt step a wave's 16 columns are 16 consecutive rows of one head; in a decode step they
// are 16 heads of the one row.  The next half's rows are asked of memory before the current
// half's products start, wait in registers and go into the other buffer afterwards.  Softmax runs
// in the result layout of S^T (a lane holds 8 keys of one column; column maximum and sum over the four lane groups), P goes
// back in as the B operand of the second product without leaving registers: the keys of a
// 32-key step are taken in the order the first product left them, by V's fragment reads.
#include "mfma.h"

namespace {

constexpr int kThreads = 256;      // of the per-head product
constexpr int kAttnThreads = 512;  // of attention: eight waves,
constexpr int kColGroups = 4;      // four tiles of 16 query columns,
constexpr int kParts = 2;          // two waves a tile
constexpr int kPadK = 8;     // bf16 a key row is padded by in LDS
constexpr int kHalf = 32;    // keys of a step
constexpr int kVtStride = kHalf + 8;
constexpr float kLazy = 8.0f;   // how far (in powers of two) a score may pass the running maximum before it moves

template <bool GATED>
__global__ void __launch_bounds__(kThreads)
head_product_mfma_kernel(bf16_t *__restrict__ out, int out_stride, int out_hstride, const bf16_t *__restrict__ in,
                         int in_stride, int in_hstride, const bf16_t *__restrict__ w, const float *__restrict__ gate,
                         int gate_stride, int n_rows, int n_in, int n_out, int gate_per_head) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int a = blockIdx.y;
  const int t = blockIdx.x * 64 + wave * 16 + (lane & 15);      // this lane's row (B operand's column)
  const int o0 = blockIdx.z * 64;
  const int g = lane >> 4;
  const bf16_t *xin = in + size_t(min(t, n_rows - 1)) * in_stride + size_t(a) * in_hstride;
  const bf16_t *wa = w + size_t(a) * n_out * n_in;
  floatx4_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
  // four steps of 32 k at a time: their twenty loads go out together, then the sixteen products
  for (int k0 = 0; k0 < n_in; k0 += 128) {
    uint4 b[4], av[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + 32 * u + 8 * g;
      const bool kin = k < n_in;                                 // n_in is a multiple of 8
      b[u] = ld16(xin + (kin ? k : 0), kin && t < n_rows);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int o = o0 + 16 * j + (lane & 15);
        av[u][j] = ld16(wa + size_t(min(o, n_out - 1)) * n_in + (kin ? k : 0), kin && o < n_out);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = mfma16(as_bf16x8(av[u][j]), as_bf16x8(b[u]), acc[j]);
  }
  if (t >= n_rows) return;
  // a lane holds four neighbouring outputs of its row: one 8-byte store where the row's layout allows
  const bool wide = (out_stride % 4 == 0) && (out_hstride % 4 == 0) && (reinterpret_cast<uintptr_t>(out) % 8 == 0);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int ob = o0 + 16 * j + 4 * g;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = acc[j][i];
      if (GATED && ob + i < n_out) {
        const float gv = gate[size_t(t) * gate_stride + (gate_per_head ? size_t(a) : size_t(a) * n_out + ob + i)];
        v[i] = v[i] * (1.0f / (1.0f + expf(-gv)));
      }
    }
    bf16_t *dst = out + size_t(t) * out_stride + size_t(a) * out_hstride + ob;
    if (wide && ob + 3 < n_out) {
      *reinterpret_cast<uint2 *>(dst) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (ob + i < n_out) dst[i] = f32_to_bf16(v[i]);
    }
  }
}

// KQ: steps of 32 over a latent row that the unrolled loops cover; NV: tiles of 16 over the latent part.
// A page is worked on in two halves of kHalf keys; LDS holds two halves at a time (the one the
// waves read and the one being written), each as key rows [kHalf][lk] and as turned latent rows
// [nv * 16][kVtStride].  Eight waves: a tile of 16 query columns belongs to two waves, which both
// work out its scores and weights and take half of the latent part's tiles each in the second
// product, so that a wave's accumulators and fragments leave room for two waves a SIMD.
template <int KQ, int NV>
__global__ void __launch_bounds__(kAttnThreads)
latent_attention_mfma_kernel(bf16_t *__restrict__ out, const bf16_t *__restrict__ q, const bf16_t *__restrict__ cache,
                             const int32_t *__restrict__ page_table, int max_pages, int n_pages_total,
                             const int32_t *__restrict__ row_pos, const int32_t *__restrict__ tiles, int heads, int rank,
                             int rot_dim, float scale, int window, int tile_rows, int n_splits,
                             float *__restrict__ part_o, float *__restrict__ part_ml, int n_rows) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int latent = rank + rot_dim;
  const int kq = (latent + 31) / 32, nv = (rank + 15) / 16;
  const int lk = kq * 32 + kPadK;                    // bf16 per staged key row
  const int ks_size = kHalf * lk, vt_size = nv * 16 * kVtStride;
  bf16_t *ks_base = reinterpret_cast<bf16_t *>(lds); // [2][kHalf][lk]
  bf16_t *vt_base = ks_base + 2 * ks_size;           // [2][nv * 16][kVtStride]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, g = lane >> 4;
  // the last tiles of a prompt see the most keys: they go first, so that the short ones fill the end
  const int tile = int(gridDim.x) - 1 - int(blockIdx.x);
  const int r0 = tiles[4 * tile], n_tile = tiles[4 * tile + 1], seq = tiles[4 * tile + 2];
  const int heads_per_wave = 16 / tile_rows;
  const int group = wave / kParts, part = wave % kParts;       // the wave's tile of columns, and its share of the latent part
  const int nv_part = (nv + kParts - 1) / kParts;
  const int head = (blockIdx.y * kColGroups + group) * heads_per_wave + col / tile_rows;
  const int r = col % tile_rows;
  const bool wave_works = (blockIdx.y * kColGroups + group) * heads_per_wave < heads;
  const bool valid = r < n_tile && head < heads;
  const int row = r0 + min(r, n_tile - 1);
  const int pos0 = row_pos[r0];
  const int pos = pos0 + min(r, n_tile - 1);         // a tile's rows are consecutive positions of one sequence
  const int lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  const int lo_blk = (window > 0 && pos0 >= window) ? pos0 - window + 1 : 0;
  const int hi_blk = pos0 + n_tile - 1;

  // the pads that staging never writes must not hold what multiplies to NaN
  for (int i = tid; i < 2 * kHalf * (lk - latent); i += kAttnThreads) {
    const int key = i / (lk - latent), e = i - key * (lk - latent);
    ks_base[key * lk + latent + e] = 0;
  }
  for (int b = 0; b < 2; ++b)
    for (int i = tid; i < (nv * 16 - rank) * kVtStride; i += kAttnThreads) vt_base[b * vt_size + rank * kVtStride + i] = 0;

  // this lane's query fragments: column (row, head), k = 32 kk + 8 g .. + 7
  uint4 qf[KQ];
  const bf16_t *qrow = q + (size_t(row) * heads + min(head, heads - 1)) * latent;
#pragma unroll
  for (int kk = 0; kk < KQ; ++kk) {
    const int k = 32 * kk + 8 * g;
    qf[kk] = ld16(qrow + (k < latent ? k : 0), valid && k < latent);      // latent is a multiple of 8
  }

  const float neg_inf = -__builtin_inff();
  const float scale2 = scale * 1.4426950408889634f;     // scores in units of ln 2: the weights are exp2
  float m_run = neg_inf, l_run = 0.0f;
  constexpr int NVP = (NV + kParts - 1) / kParts;
  floatx4_t o[NVP];
#pragma unroll
  for (int v = 0; v < NVP; ++v) o[v] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  // staging: a half is kHalf rows of latent / 8 chunks of 16 bytes; thread (key = idx % kHalf, chunk = idx / kHalf)
  const int chunks = latent / 8;
  constexpr int kMaxStage = (KQ * 32 / 8 * kHalf + kAttnThreads - 1) / kAttnThreads;
  uint4 set_a[kMaxStage], set_b[kMaxStage];      // two halves on their way from memory to LDS
  int h_first = lo_blk / kHalf, h_last = hi_blk / kHalf;                // halves count from the sequence's start
  if (n_splits > 1) {                                                   // this block's share of them
    const int per = (h_last - h_first + n_splits) / n_splits;
    h_first += int(blockIdx.z) * per;
    h_last = min(h_last, h_first + per - 1);
  }
  auto page_of = [&](int h) -> int {
    const int c = h / (SB_PAGE / kHalf);
    const int p = c < max_pages ? page_table[size_t(seq) * max_pages + c] : -1;
    return (p >= 0 && p < n_pages_total) ? p : -1;
  };
  auto load_half = [&](int h, uint4 (&staged)[kMaxStage]) {
    const int page = page_of(h);
    const bf16_t *src = cache + (size_t(max(page, 0)) * SB_PAGE + (h % (SB_PAGE / kHalf)) * kHalf) * latent;
#pragma unroll
    for (int it = 0; it < kMaxStage; ++it) {
      const int idx = tid + it * kAttnThreads;
      const int key = idx % kHalf, chunk = idx / kHalf;
      staged[it] = ld16(src + size_t(key) * latent + 8 * min(chunk, chunks - 1), page >= 0 && chunk < chunks);
    }
  };
  // A thread holds eight numbers of one key; the turned copy wants a number's keys side by side.
  // Neighbouring lanes hold neighbouring keys of the same chunk, so a pair of lanes swaps half of
  // what it holds (two DPP moves inside the quad) and each writes four whole 32-bit words, (even
  // key, odd key) of one number each: the even lane numbers 0 to 3 of the chunk, the odd lane 4 to 7.
  // (Written as single 16-bit stores, two lanes a word, this step took as long as all the products.)
  auto store_half = [&](int b, const uint4 (&staged)[kMaxStage]) {
    bf16_t *ks = ks_base + b * ks_size;
    uint32_t *vt32 = reinterpret_cast<uint32_t *>(vt_base + b * vt_size);
    const bool even = (lane & 1) == 0;
#pragma unroll
    for (int it = 0; it < kMaxStage; ++it) {
      const int idx = tid + it * kAttnThreads;
      const int key = idx % kHalf, chunk = idx / kHalf;
      const uint4 st = staged[it];
      const uint32_t send0 = even ? st.z : st.x, send1 = even ? st.w : st.y;
      const uint32_t recv0 = uint32_t(__builtin_amdgcn_update_dpp(0, int(send0), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
      const uint32_t recv1 = uint32_t(__builtin_amdgcn_update_dpp(0, int(send1), 0xB1, 0xF, 0xF, true));
      if (chunk >= chunks) continue;
      *reinterpret_cast<uint4 *>(ks + key * lk + 8 * chunk) = st;
      if (8 * chunk < rank) {                       // rank is a multiple of 8: a chunk lies inside or outside
        const uint32_t mine0 = even ? st.x : st.z, mine1 = even ? st.y : st.w;
        const uint32_t lo0 = even ? mine0 : recv0, hi0 = even ? recv0 : mine0;   // the even key's numbers, the odd key's
        const uint32_t lo1 = even ? mine1 : recv1, hi1 = even ? recv1 : mine1;
        const int d = 8 * chunk + (even ? 0 : 4);
        uint32_t *dst = vt32 + (d * kVtStride + (key & ~1)) / 2;
        dst[0 * (kVtStride / 2)] = (lo0 & 0xffffu) | (hi0 << 16);
        dst[1 * (kVtStride / 2)] = (lo0 >> 16) | (hi0 & 0xffff0000u);
        dst[2 * (kVtStride / 2)] = (lo1 & 0xffffu) | (hi1 << 16);
        dst[3 * (kVtStride / 2)] = (lo1 >> 16) | (hi1 & 0xffff0000u);
      }
    }
  };

  // Halves h (being worked on, in LDS buffer buf), h1 (on its way, in the set `held`) and h2 (asked for
  // now, into the set `free`): a half's loads go out two steps before its rows are stored, so that
  // they have a whole step of products and a step of stores to land.
  auto next_half = [&](int h) -> int {
    ++h;
    while (h <= h_last && page_of(h) < 0) ++h;        // pages that are not there hold no visible key
    return h;
  };
  int h = next_half(h_first - 1), h1 = h_last + 1;
  int buf = 0;
  if (h <= h_last) {
    load_half(h, set_a);
    store_half(0, set_a);
    h1 = next_half(h);
    if (h1 <= h_last) load_half(h1, set_a);
  }
  __syncthreads();                                    // the pads and the first half are written
  auto step = [&](uint4 (&held)[kMaxStage], uint4 (&free)[kMaxStage]) {
    const int h2 = h1 <= h_last ? next_half(h1) : h1;
    if (h2 <= h_last) load_half(h2, free);

    if (wave_works) {
      const bf16_t *ks = ks_base + buf * ks_size, *vt = vt_base + buf * vt_size;
      floatx4_t s[2] = {floatx4_t{0.f, 0.f, 0.f, 0.f}, floatx4_t{0.f, 0.f, 0.f, 0.f}};
      const bf16_t *kr = ks + col * lk + 8 * g;
#pragma unroll
      for (int kk = 0; kk < KQ; ++kk) {
        if (kk >= kq) continue;
#pragma unroll
        for (int t = 0; t < 2; ++t)
          s[t] = mfma16(as_bf16x8(*reinterpret_cast<const uint4 *>(kr + 16 * t * lk + 32 * kk)), as_bf16x8(qf[kk]), s[t]);
      }
      // s[t][i] = score of key kHalf h + 16 t + 4 g + i for this lane's column, in units of ln 2
      float mx = neg_inf;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = h * kHalf + 16 * t + 4 * g + i;
          const bool vis = valid && j >= lo && j <= pos;
          s[t][i] = vis ? s[t][i] * scale2 : neg_inf;
          mx = fmaxf(mx, s[t][i]);
        }
      mx = max_over_lane_groups(mx);
      // the maximum the sums are relative to moves only when a score passes it by kLazy (2^kLazy in
      // the weights, which float32 sums and bfloat16 weights carry easily): most steps then leave
      // the accumulators alone
      if (__any(mx > m_run + kLazy)) {
        const float m_new = fmaxf(m_run, mx);
        const float alpha = m_new == neg_inf ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);   // 0 while nothing has been seen
        l_run *= alpha;
#pragma unroll
        for (int v = 0; v < NVP; ++v)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[v][i] *= alpha;
        m_run = m_new;
      }
      const float m_safe = m_run == neg_inf ? 0.0f : m_run;
      float sum = 0.0f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s[t][i] = __builtin_amdgcn_exp2f(s[t][i] - m_safe);
          sum += s[t][i];
        }
      l_run += sum;
      const uint4 pf = make_uint4(pack_bf16(s[0][0], s[0][1]), pack_bf16(s[0][2], s[0][3]),
                                  pack_bf16(s[1][0], s[1][1]), pack_bf16(s[1][2], s[1][3]));
#pragma unroll
      for (int v = 0; v < NVP; ++v) {
        const int vg = part * nv_part + v;
        if (v >= nv_part || vg >= nv) continue;
        const bf16_t *vr = vt + (16 * vg + col) * kVtStride + 4 * g;
        const uint2 lo8 = *reinterpret_cast<const uint2 *>(vr);
        const uint2 hi8 = *reinterpret_cast<const uint2 *>(vr + 16);
        o[v] = mfma16(as_bf16x8(make_uint4(lo8.x, lo8.y, hi8.x, hi8.y)), as_bf16x8(pf), o[v]);
      }
    }
    // nobody reads the other buffer any more: its readers passed the barrier that ended the step before
    if (h1 <= h_last) store_half(buf ^ 1, held);
    __syncthreads();
    buf ^= 1;
    h = h1;
    h1 = h2;
  };
  while (h <= h_last) {
    step(set_a, set_b);
    if (h > h_last) break;
    step(set_b, set_a);
  }

  if (!wave_works) return;
  float l_tot = l_run + __shfl_xor(l_run, 16, 64);
  l_tot += __shfl_xor(l_tot, 32, 64);
  if (!valid) return;
  if (n_splits > 1) {               // unnormalized sums, with the maximum they are relative to, for the merge
    const size_t column = size_t(blockIdx.z) * n_rows * heads + size_t(row) * heads + head;
    float *po = part_o + column * rank;
#pragma unroll
    for (int v = 0; v < NVP; ++v) {
      const int vg = part * nv_part + v;
      if (v >= nv_part || vg >= nv) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (16 * vg + 4 * g + i < rank) po[16 * vg + 4 * g + i] = o[v][i];
    }
    if (g == 0 && part == 0) {
      part_ml[2 * column] = m_run;
      part_ml[2 * column + 1] = l_tot;
    }
    return;
  }
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  bf16_t *orow = out + (size_t(row) * heads + head) * rank;
#pragma unroll
  for (int v = 0; v < NVP; ++v) {
    const int vg = part * nv_part + v;
    if (v >= nv_part || vg >= nv) continue;
    const int d = 16 * vg + 4 * g;
    if (d + 3 < rank) {
      *reinterpret_cast<uint2 *>(orow + d) = make_uint2(pack_bf16(o[v][0] * inv, o[v][1] * inv),
                                                        pack_bf16(o[v][2] * inv, o[v][3] * inv));
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (d + i < rank) orow[d + i] = f32_to_bf16(o[v][i] * inv);
    }
  }
}

// out[column, :] = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M), M the largest m_s: the shares of
// a column's keys that n_splits blocks worked on, put together.  A block a column; the shares'
// weights 2^(m_s - M) wait in LDS, and a thread asks for eight shares of its numbers at a time.
constexpr int kMaxSplits = 512;

__global__ void __launch_bounds__(256)
latent_merge_kernel(bf16_t *__restrict__ out, const float *__restrict__ part_o, const float *__restrict__ part_ml,
                    int n_splits, size_t n_columns, int rank) {
  __shared__ float weight[kMaxSplits];
  __shared__ float wave_l[4];
  const size_t column = blockIdx.x;
  const int tid = threadIdx.x;
  float m = -__builtin_inff();
  for (int s = tid; s < n_splits; s += 256) m = fmaxf(m, part_ml[2 * (size_t(s) * n_columns + column)]);
  m = wave_max(m);
  if ((tid & 63) == 0) wave_l[tid >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(wave_l[0], wave_l[1]), fmaxf(wave_l[2], wave_l[3]));
  __syncthreads();
  float l = 0.0f;
  for (int s = tid; s < n_splits; s += 256) {
    const float ms = part_ml[2 * (size_t(s) * n_columns + column)];
    const float ws = ms > -__builtin_inff() ? exp2f(ms - m) : 0.0f;
    weight[s] = ws;
    l += part_ml[2 * (size_t(s) * n_columns + column) + 1] * ws;
  }
  l = wave_sum(l);
  if ((tid & 63) == 0) wave_l[tid >> 6] = l;
  __syncthreads();
  l = (wave_l[0] + wave_l[1]) + (wave_l[2] + wave_l[3]);
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  for (int d = tid; d < rank; d += 256) {
    float acc = 0.0f;
    for (int s0 = 0; s0 < n_splits; s0 += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        v[u] = part_o[(size_t(min(s0 + u, n_splits - 1)) * n_columns + column) * rank + d];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < n_splits) acc += v[u] * weight[s0 + u];
    }
    out[column * rank + d] = f32_to_bf16(acc * inv);
  }
}

template <int KQ, int NV>
int launch_attention(bf16_t *out, const bf16_t *q, const bf16_t *cache, const int32_t *page_table, int max_pages,
                     int n_pages_total, const int32_t *row_pos, const int32_t *tiles, int n_tiles, int heads, int rank,
                     int rot_dim, float scale, int window, int tile_rows, int n_splits, float *part_o, float *part_ml,
                     int n_rows, hipStream_t s) {
  const int latent = rank + rot_dim;
  const int kq = (latent + 31) / 32, nv = (rank + 15) / 16;
  const size_t lds = 2 * (size_t(kHalf) * (kq * 32 + kPadK) + size_t(nv) * 16 * kVtStride) * sizeof(bf16_t);
  static bool raised = false;              // once per kernel of this shape: more dynamic LDS than the default allows
  if (!raised) {
    if (hipFuncSetAttribute((const void *)latent_attention_mfma_kernel<KQ, NV>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
      (void)hipGetLastError();
    raised = true;
  }
  const int heads_per_block = kColGroups * (16 / tile_rows);
  dim3 grid(n_tiles, (heads + heads_per_block - 1) / heads_per_block, n_splits);
  latent_attention_mfma_kernel<KQ, NV><<<grid, kAttnThreads, lds, s>>>(out, q, cache, page_table, max_pages, n_pages_total,
                                                                   row_pos, tiles, heads, rank, rot_dim, scale, window,
                                                                   tile_rows, n_splits, part_o, part_ml, n_rows);
  if (n_splits > 1)
    latent_merge_kernel<<<unsigned(size_t(n_rows) * heads), 256, 0, s>>>(out, part_o, part_ml, n_splits,
                                                                         size_t(n_rows) * heads, rank);
  return sb::check_launch("sb_latent_attention_bf16");
}

}  // namespace

// 1 when sb_head_product_bf16 takes these sizes and strides (all in elements).
extern "C" int sb_head_product_bf16_ok(int out_stride, int out_hstride, int in_stride, int in_hstride, int n_in) {
  (void)out_stride; (void)out_hstride;
  return n_in % 8 == 0 && in_stride % 8 == 0 && in_hstride % 8 == 0;
}

// out[t, a, o] = sum_i W[a][o][i] in[t, a, i] on the matrix cores; everything bfloat16, gate f32 or NULL
// (times sigmoid(gate[t * gate_stride + a * n_out + o])); in and W 16-byte aligned.
extern "C" int sb_head_product_gated_bf16(void *out, int out_stride, int out_hstride, const void *in, int in_stride,
                                          int in_hstride, const void *w, const float *gate, int gate_stride,
                                          int gate_per_head, int n_rows, int heads, int n_in, int n_out, void *stream);
extern "C" int sb_head_product_bf16(void *out, int out_stride, int out_hstride, const void *in, int in_stride,
                                    int in_hstride, const void *w, const float *gate, int gate_stride, int n_rows,
                                    int heads, int n_in, int n_out, void *stream) {
  return sb_head_product_gated_bf16(out, out_stride, out_hstride, in, in_stride, in_hstride, w, gate, gate_stride, 0, n_rows,
                                    heads, n_in, n_out, stream);
}

// The same with gate_per_head: the gate holds one number a head, gate[t * gate_stride + a], for all of the
// head's outputs.
extern "C" int sb_head_product_gated_bf16(void *out, int out_stride, int out_hstride, const void *in, int in_stride,
                                          int in_hstride, const void *w, const float *gate, int gate_stride,
                                          int gate_per_head, int n_rows, int heads, int n_in, int n_out, void *stream) {
  SB_REQUIRE(out && in && w, "sb_head_product_bf16: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads > 0 && n_in > 0 && n_out > 0, "sb_head_product_bf16: bad sizes");
  SB_SUPPORT(sb_head_product_bf16_ok(out_stride, out_hstride, in_stride, in_hstride, n_in),
             "sb_head_product_bf16: inner size and strides must be multiples of 8");
  SB_SUPPORT((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sb_head_product_bf16: operands must be 16-byte aligned");
  SB_SUPPORT(heads <= 65535 && (n_out + 63) / 64 <= 65535, "sb_head_product_bf16: too many heads or outputs");
  if (n_rows == 0) return SB_OK;
  dim3 grid((n_rows + 63) / 64, heads, (n_out + 63) / 64);
  hipStream_t s = (hipStream_t)stream;
  if (gate)
    head_product_mfma_kernel<true><<<grid, kThreads, 0, s>>>((bf16_t *)out, out_stride, out_hstride, (const bf16_t *)in,
                                                             in_stride, in_hstride, (const bf16_t *)w, gate, gate_stride,
                                                             n_rows, n_in, n_out, gate_per_head);
  else
    head_product_mfma_kernel<false><<<grid, kThreads, 0, s>>>((bf16_t *)out, out_stride, out_hstride, (const bf16_t *)in,
                                                              in_stride, in_hstride, (const bf16_t *)w, gate, gate_stride,
                                                              n_rows, n_in, n_out, gate_per_head);
  return sb::check_launch("sb_head_product_bf16");
}

// The height of the runs of rows (`tiles`) that a prompt step's launch takes.
extern "C" int sb_latent_attention_tile_rows(void) { return 16; }

// 1 when sb_latent_attention_bf16 takes these sizes.
extern "C" int sb_latent_attention_bf16_ok(int rank, int rot_dim) {
  return rank > 0 && rot_dim >= 0 && rank % 8 == 0 && rot_dim % 8 == 0 && rank + rot_dim <= 576 && rank <= 512;
}

// Attention over cached latent rows on the matrix cores, everything bfloat16 (see the head of the
// file).  tiles int32 [n_tiles, 4] = (first row, rows, sequence, 0): runs of up to tile_rows
// consecutive rows of one sequence; tile_rows 16 for a prompt step, 1 for a step of single rows
// (a wave then takes 16 heads of a row).  out [n_rows, heads, rank], q [n_rows, heads, rank + rot_dim].
// n_splits > 1: the keys of every tile are shared out over that many blocks, whose unnormalized sums
// go through part_o (f32 [n_splits, n_rows, heads, rank]) and part_ml (f32 [n_splits, n_rows, heads, 2])
// and are put together by a second kernel: for steps of few rows over many keys.
extern "C" int sb_latent_attention_bf16(void *out, const void *q, const void *cache, const int32_t *page_table,
                                        int max_pages, int n_pages_total, const int32_t *row_pos, const int32_t *tiles,
                                        int n_tiles, int heads, int rank, int rot_dim, float scale, int window,
                                        int tile_rows, int n_splits, float *part_o, float *part_ml, int n_rows,
                                        void *stream) {
  SB_REQUIRE(out && q && cache && page_table && row_pos && tiles, "sb_latent_attention_bf16: null pointer");
  SB_REQUIRE(n_tiles >= 0 && heads > 0 && max_pages > 0 && n_pages_total > 0 && window >= 0,
             "sb_latent_attention_bf16: bad sizes");
  SB_REQUIRE(tile_rows == 16 || tile_rows == 1, "sb_latent_attention_bf16: tiles of 16 rows or of one");
  SB_REQUIRE(n_splits >= 1 && n_splits <= kMaxSplits && n_rows >= 0 && (n_splits == 1 || (part_o && part_ml)),
             "sb_latent_attention_bf16: shares of the keys need their scratch");
  SB_SUPPORT(sb_latent_attention_bf16_ok(rank, rot_dim), "sb_latent_attention_bf16: a latent row of %d + %d is not taken",
             rank, rot_dim);
  SB_SUPPORT((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(cache) | reinterpret_cast<uintptr_t>(out)) % 16 == 0,
             "sb_latent_attention_bf16: operands must be 16-byte aligned");
  if (n_tiles == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const int kq = (rank + rot_dim + 31) / 32, nv = (rank + 15) / 16;
#define SB_GO(KQ, NV)                                                                                              \
  return launch_attention<KQ, NV>((bf16_t *)out, (const bf16_t *)q, (const bf16_t *)cache, page_table, max_pages,    \
                                  n_pages_total, row_pos, tiles, n_tiles, heads, rank, rot_dim, scale, window, tile_rows,  \
                                  n_splits, part_o, part_ml, n_rows, s)
  if (kq <= 6 && nv <= 8) SB_GO(6, 8);
  if (kq <= 10 && nv <= 16) SB_GO(10, 16);
  SB_GO(18, 32);
#undef SB_GO
}
