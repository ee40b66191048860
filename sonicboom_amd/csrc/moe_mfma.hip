// The experts' products on the matrix cores: pairs (row, choice) grouped by expert on the device,
// then one grid of tiles, each a run of pairs of one expert times 128 matrix rows.
//
//   sb_moe_group      one block: counts the pairs of every expert, lays the experts' pairs one after
//                     the other (`order`: pair numbers, expert by expert) and lists the tiles
//                     (expert, first place in `order`, pairs <= tile height); the number of tiles
//                     stays on the device, the product's grid is sized for the most there can be.
//                     Within an expert the order of the pairs is whatever the atomics give: every
//                     number of a product's result is one dot product summed in k order, so it
//                     does not depend on where in a tile its pair sits.
//   sb_moe_product_bf16   Y[pair,:] = X[pair / x_div,:] W_e^T, bf16 operands, float32 sums:
//                     blocks of four waves in 2 x 2, a wave 16 * MT rows x 64 matrix rows, operand
//                     tiles of 64 k staged in LDS (16-byte chunks XOR-swizzled by row) with the next
//                     tile's loads in flight, MFMA 16x16x32.  Gated: a block's 128 matrix rows are 64
//                     gate rows and the 64 up rows that belong to them, and the epilogue leaves
//                     g' sigmoid(alpha g') (u' + 1), g' = min(g, limit), u' = u cut to +-limit.
#include "mfma.h"

namespace {

constexpr int BK = 64, BN = 128, kThreads = 256;

__global__ void __launch_bounds__(1024)
moe_group_kernel(const int32_t *__restrict__ ids, int n_pairs, int n_experts, int tile_rows, int32_t *__restrict__ order,
                 int32_t *__restrict__ tiles, int32_t *__restrict__ n_tiles) {
  extern __shared__ int sm[];
  int *counts = sm, *cursor = sm + n_experts;
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < n_experts) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < n_experts; ++e) {
      const int c = counts[e];
      cursor[e] = at;
      for (int r = 0; r < c; r += tile_rows) {
        tiles[4 * nt] = e; tiles[4 * nt + 1] = at + r; tiles[4 * nt + 2] = min(tile_rows, c - r); tiles[4 * nt + 3] = 0;
        ++nt;
      }
      at += c;
    }
    *n_tiles = nt;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < n_experts) order[atomicAdd(&cursor[e], 1)] = p;
  }
}

struct Args {
  void *y; int y_f32;
  const bf16_t *x, *w;
  const int32_t *order, *tiles, *n_tiles;      // NULL: one expert, the pairs in their own order
  int n_pairs, x_div, n_out, n_in, gated;      // gated: the kind of pair, 0 when an output is one matrix row
  float limit, alpha;
  int single;                                  // the activation of an output that is no pair (expert_single)
};

// LDS place (in 16-byte chunks) of chunk c of row r of a tile whose rows are 8 chunks long
__device__ __forceinline__ int lds_at(int r, int c) { return r * 8 + (c ^ (r & 7)); }

template <int MT>      // row tiles of 16 a wave: the block takes 32 * MT pairs
__global__ void __launch_bounds__(kThreads) moe_product_kernel(Args a) {
  constexpr int BM = 32 * MT;
  constexpr int kALoads = BM * 8 / kThreads, kBLoads = BN * 8 / kThreads;
  __shared__ uint4 a_lds[BM * 8];
  __shared__ uint4 b_lds[BN * 8];
  __shared__ int pair_of[BM];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 15, g = lane >> 4;
  const int wr = wave >> 1, wc = wave & 1;
  int expert = 0, first = blockIdx.x * BM, rows = min(BM, a.n_pairs - first);
  if (a.tiles) {
    if (int(blockIdx.x) >= *a.n_tiles) return;
    expert = a.tiles[4 * blockIdx.x]; first = a.tiles[4 * blockIdx.x + 1]; rows = a.tiles[4 * blockIdx.x + 2];
  } else if (rows <= 0) {
    return;
  }
  const int n_cols = a.gated ? BN / 2 : BN;          // results a block leaves per pair
  const int n0 = blockIdx.y * n_cols;
  for (int i = tid; i < BM; i += kThreads) pair_of[i] = i < rows ? (a.order ? a.order[first + i] : first + i) : -1;
  __syncthreads();

  // which matrix row feeds LDS row j of the B tile: plain, n0 + j; gated, per half of 64 LDS rows
  // (a column of waves) 32 gate rows then the 32 up rows of the same results
  const size_t w_rows = size_t(a.gated ? 2 : 1) * a.n_out;
  const bf16_t *we = a.w + size_t(expert) * w_rows * a.n_in;
  const bf16_t *a_src[kALoads];
  const bf16_t *b_src[kBLoads];
  int a_chunk[kALoads], b_chunk[kBLoads];
#pragma unroll
  for (int i = 0; i < kALoads; ++i) {
    const int idx = tid + i * kThreads, r = idx >> 3;
    a_chunk[i] = idx & 7;
    const int p = pair_of[r];
    a_src[i] = p >= 0 ? a.x + size_t(p / a.x_div) * a.n_in : nullptr;
  }
#pragma unroll
  for (int i = 0; i < kBLoads; ++i) {
    const int idx = tid + i * kThreads, j = idx >> 3;
    b_chunk[i] = idx & 7;
    int n;
    if (a.gated) {
      const int half = j >> 6, within = j & 63;
      n = n0 + 32 * half + (within & 31);
      b_src[i] = n < a.n_out ? we + (size_t(within >> 5) * a.n_out + n) * a.n_in : nullptr;
    } else {
      n = n0 + j;
      b_src[i] = n < a.n_out ? we + size_t(n) * a.n_in : nullptr;
    }
  }
  // the low tile (few pairs an expert: decode steps, whose few blocks a CU would wait for memory once
  // per k tile) keeps two k tiles' loads in flight while a third is multiplied; the high tile, whose
  // accumulators take the registers, one
  constexpr int DEPTH = MT <= 2 ? 2 : 1;
  uint4 areg[DEPTH][kALoads], breg[DEPTH][kBLoads];
  auto fetch = [&](uint4 *ar, uint4 *br, int k0) {
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      const int k = k0 + 8 * a_chunk[i];
      ar[i] = (a_src[i] && k < a.n_in) ? *reinterpret_cast<const uint4 *>(a_src[i] + k) : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      const int k = k0 + 8 * b_chunk[i];
      br[i] = (b_src[i] && k < a.n_in) ? *reinterpret_cast<const uint4 *>(b_src[i] + k) : make_uint4(0u, 0u, 0u, 0u);
    }
  };

  floatx4_t acc[MT][4];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int f = 0; f < 4; ++f) acc[i][f] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  auto step = [&](uint4 *ar, uint4 *br, int k0) {
    __syncthreads();        // the tile before has been read
#pragma unroll
    for (int i = 0; i < kALoads; ++i) { const int idx = tid + i * kThreads; a_lds[lds_at(idx >> 3, idx & 7)] = ar[i]; }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) { const int idx = tid + i * kThreads; b_lds[lds_at(idx >> 3, idx & 7)] = br[i]; }
    __syncthreads();
    if (k0 + DEPTH * BK < a.n_in) fetch(ar, br, k0 + DEPTH * BK);
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      const int c = 4 * ks + g;
      bf16x8_t af[MT], bf[4];
#pragma unroll
      for (int i = 0; i < MT; ++i) af[i] = as_bf16x8(a_lds[lds_at(16 * MT * wr + 16 * i + col, c)]);
#pragma unroll
      for (int f = 0; f < 4; ++f) bf[f] = as_bf16x8(b_lds[lds_at(64 * wc + 16 * f + col, c)]);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[i][f] = mfma16(af[i], bf[f], acc[i][f]);
    }
  };
  fetch(areg[0], breg[0], 0);
  if (DEPTH == 2 && BK < a.n_in) fetch(areg[DEPTH - 1], breg[DEPTH - 1], BK);
  for (int k0 = 0; k0 < a.n_in; k0 += DEPTH * BK) {
    step(areg[0], breg[0], k0);
    if (DEPTH == 2 && k0 + BK < a.n_in) step(areg[DEPTH - 1], breg[DEPTH - 1], k0 + BK);
  }

  // acc[i][f][e]: pair row 16 MT wr + 16 i + 4 g + e, matrix row (of the wave's 64) 16 f + col
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int p = pair_of[16 * MT * wr + 16 * i + 4 * g + e];
      if (p < 0) continue;
#pragma unroll
      for (int f = 0; f < (a.gated ? 2 : 4); ++f) {
        const int n = a.gated ? n0 + 32 * wc + 16 * f + col : n0 + 64 * wc + 16 * f + col;
        if (n >= a.n_out) continue;
        const float v = a.gated ? expert_pair(acc[i][f][e], acc[i][f + 2][e], a.gated, a.limit, a.alpha)
                                : expert_single(acc[i][f][e], a.single);
        if (a.y_f32) ((float *)a.y)[size_t(p) * a.n_out + n] = v;
        else ((bf16_t *)a.y)[size_t(p) * a.n_out + n] = f32_to_bf16(v);
      }
    }
}

}  // namespace

extern "C" int sb_moe_tile_rows(int n_pairs, int n_experts) {
  return (long long)n_pairs >= 96LL * n_experts ? 128 : 64;
}

// order int32 [n_pairs]; tiles int32 [4 * (n_pairs / tile_rows + n_experts + 1)]; n_tiles int32 [1]
extern "C" int sb_moe_group(const int32_t *ids, int n_pairs, int n_experts, int tile_rows, int32_t *order, int32_t *tiles,
                            int32_t *n_tiles, void *stream) {
  SB_REQUIRE(ids && order && tiles && n_tiles, "sb_moe_group: null pointer");
  SB_REQUIRE(n_pairs >= 0 && n_experts > 0 && (tile_rows == 64 || tile_rows == 128), "sb_moe_group: bad sizes pairs=%d experts=%d tile=%d",
             n_pairs, n_experts, tile_rows);
  SB_SUPPORT(n_experts <= 4096, "sb_moe_group: more than 4096 experts");
  moe_group_kernel<<<1, 1024, 2 * size_t(n_experts) * sizeof(int), (hipStream_t)stream>>>(ids, n_pairs, n_experts, tile_rows, order,
                                                                                         tiles, n_tiles);
  return sb::check_launch("sb_moe_group");
}

extern "C" int sb_moe_product_bf16_ok(int n_in) { return n_in % 8 == 0 ? 1 : 0; }

extern "C" int sb_moe_product_bf16(void *y, int y_dtype, const void *x, const void *w, const int32_t *order,
                                   const int32_t *tiles, const int32_t *n_tiles, int max_tiles, int tile_rows, int n_pairs,
                                   int x_div, int n_out, int n_in, int gated, float limit, float alpha, void *stream) {
  SB_REQUIRE(y && x && w, "sb_moe_product_bf16: null pointer");
  SB_REQUIRE(n_pairs >= 0 && x_div > 0 && n_out > 0 && n_in > 0 && (tile_rows == 64 || tile_rows == 128),
             "sb_moe_product_bf16: bad sizes pairs=%d out=%d in=%d tile=%d", n_pairs, n_out, n_in, tile_rows);
  SB_REQUIRE((order && tiles && n_tiles && max_tiles > 0) || (!order && !tiles && !n_tiles),
             "sb_moe_product_bf16: the grouping comes whole or not at all");
  SB_REQUIRE(sb::valid_dtype(y_dtype), "sb_moe_product_bf16: unknown dtype");
  SB_SUPPORT(n_in % 8 == 0, "sb_moe_product_bf16: an inner size of %d is no multiple of 8", n_in);
  if (n_pairs == 0) return SB_OK;
  const bool pair = expert_is_pair(gated);
  const Args a{y, y_dtype == SB_F32 ? 1 : 0, (const bf16_t *)x, (const bf16_t *)w, order, tiles, n_tiles, n_pairs, x_div, n_out, n_in,
               pair ? gated : 0, limit, alpha, pair ? 0 : gated};
  const int n_cols = pair ? BN / 2 : BN;
  const unsigned gx = tiles ? unsigned(max_tiles) : unsigned((n_pairs + tile_rows - 1) / tile_rows);
  const dim3 grid(gx, (n_out + n_cols - 1) / n_cols);
  SB_SUPPORT(grid.y <= 65535, "sb_moe_product_bf16: too many columns for one grid");
  hipStream_t s = (hipStream_t)stream;
  if (tile_rows == 128) moe_product_kernel<4><<<grid, kThreads, 0, s>>>(a);
  else moe_product_kernel<2><<<grid, kThreads, 0, s>>>(a);
  return sb::check_launch("sb_moe_product_bf16");
}
