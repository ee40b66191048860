// Attention on the matrix cores for mixers whose keys and values have sizes of their own, whose
// scores may be capped by a tanh and whose softmax may hold a sink (one more key of score 0
// without a value): compiled with -DSB_KEY_DIM=<dk> -DSB_VALUE_DIM=<dv>, both multiples of 16.
//
// One kernel for prompt steps and single rows.  A block is a run of up to 16 consecutive rows of
// one sequence (a row tile) times one kv head; its four waves are four query heads of that kv
// head's group (more heads: further blocks).  Every page of the cache is staged once per block in
// LDS as it lies (the cache keeps a page's rows in the order the fragments are read without bank
// conflicts: sb_key_index, sb_value_index) and shared by the waves; the next page's loads are in
// flight while this one is attended.
//
//   S^T = K Q^T   MFMA 16x16x32, A = 16 keys x 32 d from LDS, B = Q^T kept in registers
//   O^T = V^T P^T MFMA 16x16x32, A = 16 d x 32 keys from LDS, B = P^T straight from the S^T tiles:
//         row r of an S^T tile stands for key 8 (r / 4) + 4 t + r % 4 of a half page (t the tile), so
//         the eight probabilities a lane holds after two tiles are eight consecutive keys.
//
// Two further forms of the score and of the result, for mixers whose heads share their weights:
// a bias by the logarithm of the distance, score - r1[h] ln(1 + r2[h] (p - j)) (`dist_r1`, `dist_r2`), and
// `all_values`: every query head's weights applied to the values of every kv head, not its own alone
// (the grid then holds a block per value head too, and the result is [rows, heads_q, heads_kv, dv]).
//
// Softmax in float32, running maximum and sum per query column, scores kept times log2(e) so that the
// weights are powers of two; a sink starts the maximum at 0 and the sum at 1.  Steps of few rows
// share the pages of a sequence out over `chunks` blocks, which leave (unnormed result, maximum,
// sum) for the merge kernel.
#include "mfma.h"

#if !defined(SB_KEY_DIM) || !defined(SB_VALUE_DIM)
#error "compile with -DSB_KEY_DIM=<key size> -DSB_VALUE_DIM=<value size>"
#endif
static_assert(SB_KEY_DIM % 16 == 0 && SB_KEY_DIM >= 16 && SB_KEY_DIM <= 256, "key size: 16..256 in steps of 16");
static_assert(SB_VALUE_DIM % 16 == 0 && SB_VALUE_DIM >= 16 && SB_VALUE_DIM <= 256, "value size: 16..256 in steps of 16");

namespace sb {
char *error_slot() {
  static thread_local char slot[kErrorLen] = "";
  return slot;
}
}  // namespace sb

extern "C" const char *sb_cattn_last_error(void) { return sb::error_slot(); }
extern "C" int sb_cattn_key_dim(void) { return SB_KEY_DIM; }
extern "C" int sb_cattn_value_dim(void) { return SB_VALUE_DIM; }

namespace {

constexpr int DK = SB_KEY_DIM, DV = SB_VALUE_DIM;
constexpr int KSTEPS = (DK + 31) / 32;      // steps of 32 d of the score product
constexpr int DT = DV / 16;                 // tiles of 16 d of the result
constexpr int NW = 4;                       // waves (query heads) a block
constexpr int kThreads = 64 * NW;
constexpr int kKeyChunks = SB_PAGE * DK / 8;    // 16-byte chunks of a page's keys of one head
constexpr int kValChunks = SB_PAGE * DV / 8;
constexpr int kKeyLoads = (kKeyChunks + kThreads - 1) / kThreads;
constexpr int kValLoads = (kValChunks + kThreads - 1) / kThreads;
constexpr int kTile = 16;
constexpr int kPagesInLds = 2048;           // page numbers of a block's stretch that are looked up ahead (131,072 keys)

struct Args {
  bf16_t *out;                 // [rows, heads_q * DV], or NULL when partial results are written
  float *part_o, *part_ml;     // [chunks][rows][heads_q][DV], [chunks][rows][heads_q][2]
  const bf16_t *q;             // [rows, heads_q * DK]
  const bf16_t *k_cache, *v_cache;
  const int32_t *page_table; int max_pages, n_pages;
  const int32_t *row_pos, *tiles;
  int n_rows, heads_q, heads_kv;
  float scale, softcap; int window, sink, chunk_pages;
  const float *dist_r1, *dist_r2;      // [heads_q] or NULL: the bias by the distance's logarithm
  int all_values;                      // 1: blockIdx.y also counts the kv head whose values are read
  const float *sink_scores;            // [heads_q] or NULL: the sink's score a head (NULL: 0)
  const float *gate; int gate_stride;  // [rows, gate_stride] or NULL: the result times sigmoid(gate[row][h * DV + d])
  unsigned round_blocks;       // blocks the GPU takes one of per CU
};

constexpr float kLog2e = 1.4426950408889634f;

// softcap * tanh(s / softcap) by the hardware's exponential and reciprocal: tanh(x) = 1 - 2 / (2^(2 x log2 e) + 1).
// two_log2e_over_cap = 2 log2(e) / softcap.
__device__ __forceinline__ float capped(float s, float cap, float two_log2e_over_cap) {
  const float t = fminf(s * two_log2e_over_cap, 60.0f);          // 2^60 + 1 is 2^60 in float32: tanh is 1 by then
  return cap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(t) + 1.0f));
}

__global__ void __launch_bounds__(kThreads) capped_attention_kernel(Args a) {
  __shared__ uint4 k_lds[kKeyChunks];
  __shared__ uint4 v_lds[kValChunks];
  __shared__ int page_lds[kPagesInLds];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 15, g = lane >> 4;
  const int group = a.heads_q / a.heads_kv, zgroups = (group + NW - 1) / NW;
  const int kv_blocks = a.heads_kv * zgroups;
  const int vh_own = a.all_values ? int(blockIdx.y) / kv_blocks : -1;       // the kv head whose values this block reads
  const int by = int(blockIdx.y) % kv_blocks;
  const int kvh = by / zgroups, hz = by % zgroups;
  const int vh = a.all_values ? vh_own : kvh;
  const int out_heads = a.all_values ? a.heads_q * a.heads_kv : a.heads_q;   // heads of the result's rows
  const int hg = hz * NW + wave;                  // the wave's head within the group
  const bool has_head = hg < group;
  const int h = kvh * group + (has_head ? hg : 0);
  // Later rows of a sequence see more pages.  All blocks of a prompt step are usually resident at once, a CU
  // holding blocks a whole round of the GPU apart: every other round of 256 blocks walks the tiles from
  // the far end, so that a CU's blocks are a heavy and a light one.
  // (one direction for all blocks of a (head group, chunk): every tile is taken once)
  const unsigned first_of_row = gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  const int tile_no = ((first_of_row / a.round_blocks) & 1) ? int(gridDim.x) - 1 - int(blockIdx.x) : int(blockIdx.x);
  const int32_t *tile = a.tiles + size_t(tile_no) * 4;
  const int r0 = tile[0], nr = tile[1], seq = tile[2];
  const int chunk = blockIdx.z;
  const int p0 = a.row_pos[r0], p_last = p0 + nr - 1;
  const int lo = (a.window > 0 && p0 >= a.window) ? p0 - a.window + 1 : 0;      // oldest key any row of the tile reads
  int page_lo = lo / SB_PAGE, page_hi = p_last / SB_PAGE;
  if (a.chunk_pages > 0) {
    page_lo = max(page_lo, chunk * a.chunk_pages);
    page_hi = min(page_hi, (chunk + 1) * a.chunk_pages - 1);
  }
  const int32_t *table = a.page_table + size_t(seq) * a.max_pages;

  // the queries of the wave's head: B operand, column = row of the tile
  bf16x8_t qf[KSTEPS];
#pragma unroll
  for (int kc = 0; kc < KSTEPS; ++kc) {
    const int d = 32 * kc + 8 * g;
    qf[kc] = as_bf16x8(ld16(a.q + (size_t(r0 + col) * a.heads_q + h) * DK + d, has_head && col < nr && d < DK));
  }
  const int q_pos = p0 + col;
  const int q_lo = (a.window > 0 && q_pos >= a.window) ? q_pos - a.window + 1 : 0;

  const float neg_inf = -__builtin_inff();
  const bool with_sink = a.sink && chunk == 0;
  // (scores are kept times log2(e): so is the sink's)
  float m = with_sink ? ((a.sink_scores && has_head) ? a.sink_scores[h] * kLog2e : 0.0f) : neg_inf;
  float l = (with_sink && g == 0) ? 1.0f : 0.0f;      // a lane's share of the column's sum
  floatx4_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
  const float cap_arg = a.softcap > 0.0f ? a.scale * 2.0f * kLog2e / a.softcap : 0.0f;      // the scale rides along
  // scores are kept times log2(e), so that the weights are powers of two: the sink's score stays 0
  const float scale2 = a.scale * kLog2e, cap2 = a.softcap * kLog2e;
  // r1 ln(1 + r2 d) log2(e) = r1 log2(1 + r2 d): the hardware's logarithm is the one to base two
  const float r1 = (a.dist_r1 && has_head) ? a.dist_r1[h] : 0.0f, r2 = (a.dist_r2 && has_head) ? a.dist_r2[h] : 0.0f;

  // two pages' loads are in flight while a third is attended (a CU holds few of these blocks: a page's
  // round trip to memory would otherwise show once per page)
  uint4 kreg[2][kKeyLoads], vreg[2][kValLoads];
  // The block's page numbers go into LDS first: a look-up in memory inside the loop would have every
  // fetch wait for the loads of the page before it (the memory counter runs in order), and the two
  // pages in flight would be one.
  const int n_block_pages = page_hi - page_lo + 1;
  const bool pages_in_lds = n_block_pages <= kPagesInLds;
  if (pages_in_lds) {
    for (int i = tid; i < n_block_pages; i += kThreads) {
      const int c = page_lo + i;
      int page = (c >= 0 && c < a.max_pages) ? table[c] : -1;
      page_lds[i] = page >= a.n_pages ? -1 : page;
    }
    __syncthreads();
  }
  auto fetch = [&](uint4 *kr, uint4 *vr, int c) {
    int page;
    if (pages_in_lds) {
      page = page_lds[c - page_lo];
    } else {
      page = (c >= 0 && c < a.max_pages) ? table[c] : -1;
      if (page >= a.n_pages) page = -1;
    }
    const uint4 *kp = reinterpret_cast<const uint4 *>(a.k_cache + (size_t(max(page, 0)) * a.heads_kv + kvh) * SB_PAGE * DK);
    const uint4 *vp = reinterpret_cast<const uint4 *>(a.v_cache + (size_t(max(page, 0)) * a.heads_kv + vh) * SB_PAGE * DV);
#pragma unroll
    for (int i = 0; i < kKeyLoads; ++i) {
      const int idx = tid + i * kThreads;
      kr[i] = (page >= 0 && idx < kKeyChunks) ? kp[idx] : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int i = 0; i < kValLoads; ++i) {
      const int idx = tid + i * kThreads;
      vr[i] = (page >= 0 && idx < kValChunks) ? vp[idx] : make_uint4(0u, 0u, 0u, 0u);
    }
  };
  auto stage = [&](const uint4 *kr, const uint4 *vr) {
#pragma unroll
    for (int i = 0; i < kKeyLoads; ++i) {
      const int idx = tid + i * kThreads;
      if (idx < kKeyChunks) k_lds[idx] = kr[i];
    }
#pragma unroll
    for (int i = 0; i < kValLoads; ++i) {
      const int idx = tid + i * kThreads;
      if (idx < kValChunks) v_lds[idx] = vr[i];
    }
  };

  auto attend = [&](uint4 *kr, uint4 *vr, int c) {
    __syncthreads();            // the page before has been read by every wave
    stage(kr, vr);
    __syncthreads();
    if (c + 2 <= page_hi) fetch(kr, vr, c + 2);
    if (!has_head) return;
    const bf16_t *kl = reinterpret_cast<const bf16_t *>(k_lds);
    const bf16_t *vl = reinterpret_cast<const bf16_t *>(v_lds);
#pragma unroll
    for (int hp = 0; hp < 2; ++hp) {
      const int first = c * SB_PAGE + 32 * hp;          // position of the half page's first key
      if (first > p_last || first + 31 < lo) continue;  // uniform over the block
      // every row of the tile sees every key of this half page: no score needs a test (uniform)
      const bool whole = nr == kTile && first + 31 <= p0 && (a.window == 0 || first >= p_last - a.window + 1);
      // every fragment of the half page is asked of LDS before the first product: the keys' for the
      // scores, and the values' too, which arrive while the softmax is worked out (read one by one
      // before its product, each fragment's trip through LDS showed in full: a CU holds few waves here)
      uint4 kf[2][KSTEPS], vf[DT];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int slot = 32 * hp + 8 * (col >> 2) + 4 * t + (col & 3);
#pragma unroll
        for (int kc = 0; kc < KSTEPS; ++kc) {
          const int d = 32 * kc + 8 * g;
          kf[t][kc] = d < DK ? *reinterpret_cast<const uint4 *>(kl + sb_key_index(slot, d, DK)) : make_uint4(0u, 0u, 0u, 0u);
        }
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        vf[dt] = *reinterpret_cast<const uint4 *>(vl + sb_value_index(16 * dt + col, 32 * hp + 8 * g));
      floatx4_t s[2] = {floatx4_t{0.f, 0.f, 0.f, 0.f}, floatx4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int kc = 0; kc < KSTEPS; ++kc)
#pragma unroll
        for (int t = 0; t < 2; ++t) s[t] = mfma16(as_bf16x8(kf[t][kc]), qf[kc], s[t]);      // the two tiles in turn
      // the lane's eight scores: keys first + 8 g + 4 t + i of query column `col`, times log2(e)
      float sc[8];
      float mx = neg_inf;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v;
          if (a.softcap > 0.0f) v = capped(s[t][i], cap2, cap_arg);
          else v = s[t][i] * scale2;
          sc[4 * t + i] = v;
        }
      if (a.dist_r1) {        // uniform over the block
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float dist = float(max(q_pos - (first + 8 * g + e), 0));
          sc[e] -= r1 * __builtin_amdgcn_logf(fmaf(r2, dist, 1.0f));
        }
      }
      if (!whole) {           // uniform over the block: only pages on the diagonal or at a window's edge test their scores
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int j = first + 8 * g + e;
          const bool visible = col < nr && j <= q_pos && j >= q_lo;
          sc[e] = visible ? sc[e] : neg_inf;
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) mx = fmaxf(mx, sc[e]);
      mx = max_over_lane_groups(mx);
      const float m_new = fmaxf(m, mx);
      const float alpha = m == neg_inf ? 0.0f : __builtin_amdgcn_exp2f(m - m_new);
      float psum = 0.0f, p[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p[e] = __builtin_amdgcn_exp2f(sc[e] - m_new);      // 2^(-inf) is 0: a hidden key, or a row that has seen none yet
        psum += p[e];
      }
      if (m_new == neg_inf) {                               // (-inf) - (-inf) is no number
        psum = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) p[e] = 0.0f;
      }
      l = l * alpha + psum;
      m = m_new;
      uint4 pw;
      pw.x = pack_bf16(p[0], p[1]); pw.y = pack_bf16(p[2], p[3]);
      pw.z = pack_bf16(p[4], p[5]); pw.w = pack_bf16(p[6], p[7]);
      const bf16x8_t pf = as_bf16x8(pw);
      // the results so far shrink only when some row's maximum has moved (uniform over the wave)
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[dt][i] *= alpha;
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[dt] = mfma16(as_bf16x8(vf[dt]), pf, o[dt]);
    }
  };
  if (page_lo <= page_hi) fetch(kreg[0], vreg[0], page_lo);
  if (page_lo + 1 <= page_hi) fetch(kreg[1], vreg[1], page_lo + 1);
  for (int c = page_lo; c <= page_hi; c += 2) {
    attend(kreg[0], vreg[0], c);
    if (c + 1 <= page_hi) attend(kreg[1], vreg[1], c + 1);
  }

  // the column's sum over the four lane groups
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!has_head || col >= nr) return;
  const int row = r0 + col;
  if (a.out) {
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    bf16_t *dst = a.out + (size_t(row) * out_heads + (a.all_values ? h * a.heads_kv + vh : h)) * DV;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      float r[4] = {o[dt][0] * inv, o[dt][1] * inv, o[dt][2] * inv, o[dt][3] * inv};
      if (a.gate) {
        const float *gp = a.gate + size_t(row) * a.gate_stride + size_t(h) * DV + 16 * dt + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = r[i] * (1.0f / (1.0f + expf(-gp[i])));
      }
      uint2 w;
      w.x = pack_bf16(r[0], r[1]);
      w.y = pack_bf16(r[2], r[3]);
      *reinterpret_cast<uint2 *>(dst + 16 * dt + 4 * g) = w;
    }
  } else {
    const size_t at = (size_t(chunk) * a.n_rows + row) * out_heads + (a.all_values ? h * a.heads_kv + vh : h);
    float *dst = a.part_o + at * DV;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      *reinterpret_cast<float4 *>(dst + 16 * dt + 4 * g) = make_float4(o[dt][0], o[dt][1], o[dt][2], o[dt][3]);
    if (g == 0) {
      a.part_ml[at * 2] = m;
      a.part_ml[at * 2 + 1] = l;
    }
  }
}

// out[row][h][:] = sum_c o_c exp(m_c - M) / sum_c l_c exp(m_c - M), M the largest m_c: a thread a number.
// Up to kMergeAtOnce chunks have their maxima, sums and results asked for before anything is added
// (chunks past the last read the last again and count nothing); more chunks go in rounds of as many.
constexpr int kMergeAtOnce = 16;

__global__ void __launch_bounds__(256)
merge_kernel(bf16_t *__restrict__ out, const float *__restrict__ part_o, const float *__restrict__ part_ml, int chunks,
             size_t n_heads /* rows * heads_q */, const float *__restrict__ gate, int gate_stride, int heads_q) {
  const size_t idx = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= n_heads * DV) return;
  const size_t rh = idx / DV;
  const float neg_inf = -__builtin_inff();
  float big = neg_inf;
  for (int c0 = 0; c0 < chunks; c0 += kMergeAtOnce) {
    float mc[kMergeAtOnce];
#pragma unroll
    for (int i = 0; i < kMergeAtOnce; ++i) mc[i] = part_ml[(size_t(min(c0 + i, chunks - 1)) * n_heads + rh) * 2];
#pragma unroll
    for (int i = 0; i < kMergeAtOnce; ++i) big = fmaxf(big, mc[i]);
  }
  float num = 0.0f, den = 0.0f;
  for (int c0 = 0; c0 < chunks; c0 += kMergeAtOnce) {
    float mc[kMergeAtOnce], lc[kMergeAtOnce], oc[kMergeAtOnce];
#pragma unroll
    for (int i = 0; i < kMergeAtOnce; ++i) {
      const size_t c = size_t(min(c0 + i, chunks - 1));
      mc[i] = part_ml[(c * n_heads + rh) * 2];
      lc[i] = part_ml[(c * n_heads + rh) * 2 + 1];
      oc[i] = part_o[c * n_heads * DV + idx];
    }
#pragma unroll
    for (int i = 0; i < kMergeAtOnce; ++i) {
      if (c0 + i >= chunks || mc[i] == neg_inf) continue;
      const float w = __builtin_amdgcn_exp2f(mc[i] - big);          // the maxima are kept times log2(e)
      num = fmaf(w, oc[i], num);
      den = fmaf(w, lc[i], den);
    }
  }
  float r = den > 0.0f ? num / den : 0.0f;
  if (gate) {
    const size_t row = rh / heads_q;
    r = r * (1.0f / (1.0f + expf(-gate[row * gate_stride + (idx - row * heads_q * DV)])));
  }
  out[idx] = f32_to_bf16(r);
}

}  // namespace

extern "C" int sb_cattn_tile_rows(void) { return kTile; }

// out bf16 [rows, heads_q * dv]; q bf16 [rows, heads_q * dk]; tiles int32 [n_tiles, 4] = (first row,
// rows <= 16, sequence, 0), consecutive rows of one sequence.  chunks > 1: the pages of every tile
// are shared out over that many blocks of chunk_pages pages each (chunks * chunk_pages >= max_pages)
// and merged; part_o f32 [chunks * rows * heads_q * dv] and part_ml f32 [chunks * rows * heads_q * 2]
// are the scratch for that.
extern "C" int sb_cattn_shared_bf16(void *out, const void *q, const void *k_cache, const void *v_cache,
                                    const int32_t *page_table, int max_pages, int n_pages, const int32_t *row_pos,
                                    const int32_t *tiles, int n_tiles, int n_rows, int heads_q, int heads_kv, float scale,
                                    int window, float softcap, int sink, int chunks, int chunk_pages, float *part_o,
                                    float *part_ml, const float *dist_r1, const float *dist_r2, int all_values,
                                    void *stream);

extern "C" int sb_cattn_bf16(void *out, const void *q, const void *k_cache, const void *v_cache,
                             const int32_t *page_table, int max_pages, int n_pages, const int32_t *row_pos,
                             const int32_t *tiles, int n_tiles, int n_rows, int heads_q, int heads_kv, float scale,
                             int window, float softcap, int sink, int chunks, int chunk_pages, float *part_o,
                             float *part_ml, void *stream) {
  return sb_cattn_shared_bf16(out, q, k_cache, v_cache, page_table, max_pages, n_pages, row_pos, tiles, n_tiles, n_rows,
                              heads_q, heads_kv, scale, window, softcap, sink, chunks, chunk_pages, part_o, part_ml, nullptr,
                              nullptr, 0, stream);
}

extern "C" int sb_cattn_sink_bf16(void *out, const void *q, const void *k_cache, const void *v_cache,
                                  const int32_t *page_table, int max_pages, int n_pages, const int32_t *row_pos,
                                  const int32_t *tiles, int n_tiles, int n_rows, int heads_q, int heads_kv, float scale,
                                  int window, float softcap, int sink, int chunks, int chunk_pages, float *part_o,
                                  float *part_ml, const float *dist_r1, const float *dist_r2, int all_values,
                                  const float *sink_scores, const float *gate, int gate_stride, void *stream);

// The same with the bias r1[h] ln(1 + r2[h] distance) taken off every score (dist_r1, dist_r2 f32 [heads_q], or both
// NULL) and, with all_values, every query head's weights applied to the values of every kv head: out bf16
// [rows, heads_q, heads_kv, dv], the scratch heads_kv times as large.
extern "C" int sb_cattn_shared_bf16(void *out, const void *q, const void *k_cache, const void *v_cache,
                                    const int32_t *page_table, int max_pages, int n_pages, const int32_t *row_pos,
                                    const int32_t *tiles, int n_tiles, int n_rows, int heads_q, int heads_kv, float scale,
                                    int window, float softcap, int sink, int chunks, int chunk_pages, float *part_o,
                                    float *part_ml, const float *dist_r1, const float *dist_r2, int all_values,
                                    void *stream) {
  return sb_cattn_sink_bf16(out, q, k_cache, v_cache, page_table, max_pages, n_pages, row_pos, tiles, n_tiles, n_rows, heads_q,
                            heads_kv, scale, window, softcap, sink, chunks, chunk_pages, part_o, part_ml, dist_r1, dist_r2,
                            all_values, nullptr, nullptr, 0, stream);
}

// The same with a sink whose score is a number of the query head's own (sink_scores f32 [heads_q], as it is: not
// scaled, not capped; NULL: 0), and with an output gate (f32 [rows, gate_stride] or NULL; not with all_values): the
// result times sigmoid(gate[row * gate_stride + h * dv + d]).
extern "C" int sb_cattn_sink_bf16(void *out, const void *q, const void *k_cache, const void *v_cache,
                                  const int32_t *page_table, int max_pages, int n_pages, const int32_t *row_pos,
                                  const int32_t *tiles, int n_tiles, int n_rows, int heads_q, int heads_kv, float scale,
                                  int window, float softcap, int sink, int chunks, int chunk_pages, float *part_o,
                                  float *part_ml, const float *dist_r1, const float *dist_r2, int all_values,
                                  const float *sink_scores, const float *gate, int gate_stride, void *stream) {
  SB_REQUIRE(!sink_scores || sink, "sb_cattn_bf16: scores of a sink that is switched off");
  SB_REQUIRE(!gate || (!all_values && gate_stride >= heads_q * DV), "sb_cattn_bf16: the gate's rows of %d are too short", gate_stride);
  SB_REQUIRE((dist_r1 == nullptr) == (dist_r2 == nullptr), "sb_cattn_bf16: the distance bias needs both of its numbers");
  SB_REQUIRE(out && q && k_cache && v_cache && page_table && row_pos && tiles, "sb_cattn_bf16: null pointer");
  SB_REQUIRE(n_tiles >= 0 && n_rows >= 0 && heads_q > 0 && heads_kv > 0 && max_pages > 0 && n_pages > 0 && window >= 0,
             "sb_cattn_bf16: bad sizes tiles=%d rows=%d heads=%d/%d", n_tiles, n_rows, heads_q, heads_kv);
  SB_REQUIRE(heads_q % heads_kv == 0, "sb_cattn_bf16: %d query heads are not a multiple of %d kv heads", heads_q, heads_kv);
  SB_REQUIRE(softcap >= 0.0f, "sb_cattn_bf16: the cap of the scores must not be negative");
  SB_REQUIRE(chunks >= 1 && (chunks == 1 || (part_o && part_ml && chunk_pages > 0 &&
                                             (long long)chunks * chunk_pages >= max_pages)),
             "sb_cattn_bf16: %d chunks of %d pages do not cover %d pages, or have no scratch", chunks, chunk_pages, max_pages);
  if (n_tiles == 0 || n_rows == 0) return SB_OK;
  const int group = heads_q / heads_kv, zgroups = (group + NW - 1) / NW;
  const int value_heads = all_values ? heads_kv : 1;
  SB_SUPPORT((long long)heads_kv * zgroups * value_heads <= 65535 && chunks <= 65535,
             "sb_cattn_bf16: too many heads or chunks for one grid");
  hipStream_t s = (hipStream_t)stream;
  Args a;
  a.out = chunks == 1 ? (bf16_t *)out : nullptr;
  a.part_o = part_o; a.part_ml = part_ml;
  a.q = (const bf16_t *)q; a.k_cache = (const bf16_t *)k_cache; a.v_cache = (const bf16_t *)v_cache;
  a.page_table = page_table; a.max_pages = max_pages; a.n_pages = n_pages; a.row_pos = row_pos; a.tiles = tiles;
  a.n_rows = n_rows; a.heads_q = heads_q; a.heads_kv = heads_kv; a.scale = scale; a.softcap = softcap;
  a.window = window; a.sink = sink; a.chunk_pages = chunks == 1 ? 0 : chunk_pages;
  a.round_blocks = unsigned(sb::cu_count());
  a.dist_r1 = dist_r1; a.dist_r2 = dist_r2; a.all_values = all_values ? 1 : 0;
  a.sink_scores = sink_scores;
  a.gate = chunks == 1 ? gate : nullptr; a.gate_stride = gate_stride;      // (partial results are gated when they are merged)
  capped_attention_kernel<<<dim3(n_tiles, heads_kv * zgroups * value_heads, chunks), kThreads, 0, s>>>(a);
  int st = sb::check_launch("sb_cattn_bf16");
  if (st != SB_OK || chunks == 1) return st;
  const size_t n = size_t(n_rows) * heads_q * value_heads * DV;
  merge_kernel<<<unsigned((n + 255) / 256), 256, 0, s>>>((bf16_t *)out, part_o, part_ml, chunks,
                                                         size_t(n_rows) * heads_q * value_heads, gate, gate_stride, heads_q);
  return sb::check_launch("sb_cattn_merge");
}
