// Tile functions of stk_dsd, shared by its kernels (dsd.hip) and by the launches that compute a dsd together with
// another product on the same topology (grad.hip).
#pragma once
#include "common.h"
#include "gemm_core.h"

namespace stk {

struct DsdArgs {
  const elem_t* data;
  const int32_t* walk_offsets;
  const void* walk_columns;
  const int32_t* walk_blocks;  // indirect block ids (transposed operand) or null
  const elem_t* rhs;
  int64_t ldb;
  elem_t* out;
  int64_t ldc;
  int block_rows;
  int n;
  int idx32;
  int small;       // little work per compute unit: four-wave tiles
  // scattered output rows (the SCATTER kernels): row r of the product goes to row row_map[r] of `out`, multiplied by
  // row_scale[row_map[r]] when row_scale is given; rows whose entry is not in [0, out_rows) are dropped
  const int32_t* row_map;
  const float* row_scale;
  int out_rows;
};

// A checked dsd: the kernels' arguments, the plan's lists of the walked lines (null without a plan), layout flags.
struct DsdProblem {
  DsdArgs g;
  PlanLists lists;
  bool ta, bk, stream_rhs, empty;
};
int dsd_problem(const char* who, int64_t m, int64_t k, int64_t n,
                const void* data, const int32_t* offsets, const void* column_indices,
                const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                int transpose_a, const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                void* out, int64_t out_stride_m, int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan,
                DsdProblem* p);

// acc += the products of walk entries [e0, e1) of LINES block rows starting at `bi` (identical
// patterns when LINES > 1) with output columns [n0, n0 + Cfg::TN).  Only the first `lines` of the
// LINES rows exist; the others are computed on the last one's blocks and dropped by the caller.
template <class Cfg, int BLK, bool TRANS_A, bool FULL, int LINES>
__device__ __forceinline__ void dsd_accumulate(f32x16_t (&acc)[Cfg::IM][Cfg::JN], const DsdArgs& g, int bi, int n0, int e0, int e1, char* smem,
                                               int lines = LINES) {
  static_assert(Cfg::TM == LINES * BLK && Cfg::A_PARTS == LINES && Cfg::A_KMAJOR == !TRANS_A, "one operand part per block row");
  constexpr int KT = Cfg::KT;
  constexpr int kTilesPerBlock = BLK / KT;
  int start[LINES];
#pragma unroll
  for (int l = 0; l < LINES; l++) start[l] = g.walk_offsets[bi + (l < lines ? l : lines - 1)];
  const elem_t* b0 = g.rhs + (int64_t)n0 * (Cfg::B_KMAJOR ? g.ldb : 1);
  const int64_t b_kstride = Cfg::B_KMAJOR ? 1 : g.ldb;
  const int64_t b_part = (int64_t)Cfg::PN * (Cfg::B_KMAJOR ? g.ldb : 1);
  const int n_valid = (g.n - n0 < Cfg::TN) ? g.n - n0 : Cfg::TN;
  const int lane = threadIdx.x & 63;
  for (int s0 = e0; s0 < e1; s0 += kMaxSegments) {
    const int cnt = (e1 - s0 < kMaxSegments) ? e1 - s0 : kMaxSegments;
    // Lane i of every wavefront holds the (k block, block id) pair of walk entry s0 + i, so
    // that the K loop gets them with a lane read instead of a load.
    const int e = lane < cnt ? lane : cnt - 1;
    const int seg_k = load_index(g.walk_columns, start[0] + s0 + e, g.idx32);
    int seg_block[LINES];
#pragma unroll
    for (int l = 0; l < LINES; l++) seg_block[l] = TRANS_A ? g.walk_blocks[start[l] + s0 + e] : start[l] + s0 + e;
    auto tile_fn = [&](int t) {
      const int seg = t / kTilesPerBlock, sub = t % kTilesPerBlock;
      const int64_t kb = __builtin_amdgcn_readlane(seg_k, seg);
      TilePtrs p;
#pragma unroll
      for (int l = 0; l < LINES; l++)
        p.a[l] = g.data + (int64_t)__builtin_amdgcn_readlane(seg_block[l], seg) * (BLK * BLK) + sub * KT * (TRANS_A ? BLK : 1);
      p.b[0] = b0 + (kb * BLK + sub * KT) * b_kstride;
      p.b[1] = p.b[0] + b_part;
      p.k_valid = KT;
      return p;
    };
    if constexpr (FULL) mainloop_dma<Cfg>(acc, cnt * kTilesPerBlock, tile_fn, BLK, g.ldb, smem);
    else mainloop_reg<Cfg>(acc, cnt * kTilesPerBlock, tile_fn, BLK, g.ldb, BLK, n_valid, smem);
  }
}

// Writes the finished tile: the first `rows` rows from block row `bi` onwards, columns from n0.
template <class Cfg, int BLK, bool SCATTER = false>
__device__ __forceinline__ void dsd_store(f32x16_t (&acc)[Cfg::IM][Cfg::JN], const DsdArgs& g, int bi, int n0, char* smem, int rows = Cfg::TM) {
  const int n_valid = (g.n - n0 < Cfg::TN) ? g.n - n0 : Cfg::TN;
  const WaveCoords w = wave_coords<Cfg>();
  const int wm0 = wave_m0<Cfg>(w), wn0 = wave_n0<Cfg>(w);
  if constexpr (SCATTER)
    epilogue<Cfg, STK_STREAM_STORES, true>(acc, g.out + n0 + wn0, g.ldc, rows - wm0, n_valid - wn0, smem, 64, kNoActivation, nullptr, 0, 0,
                                           g.row_map + (int64_t)bi * BLK + wm0, g.row_scale, g.out_rows);
  else
    epilogue<Cfg, STK_STREAM_STORES>(acc, g.out + ((int64_t)bi * BLK + wm0) * g.ldc + n0 + wn0, g.ldc, rows - wm0, n_valid - wn0, smem);
}

// The whole tile of LINES block rows starting at `bi` (the first `lines` of them exist), output columns
// [n0, n0 + Cfg::TN).
template <class Cfg, int BLK, bool TRANS_A, bool FULL, int LINES, bool SCATTER = false>
__device__ __forceinline__ void dsd_tile(const DsdArgs& g, int bi, int n0, char* smem, int lines = LINES) {
  f32x16_t acc[Cfg::IM][Cfg::JN] = {};
  dsd_accumulate<Cfg, BLK, TRANS_A, FULL, LINES>(acc, g, bi, n0, 0, g.walk_offsets[bi + 1] - g.walk_offsets[bi], smem, lines);
  dsd_store<Cfg, BLK, SCATTER>(acc, g, bi, n0, smem, lines * BLK);
}

// The tile of a launch over the plan's lists of lines (128-blocks, eight wavefronts) that workgroup `bid` takes,
// the large ones first:
//   pairs of identical rows   256x256 tiles
//   three identical rows      384x128 tiles: the dense operand, the big stream when rows
//                             are long, is still read only once for the three
//   lone rows                 128x256 tiles
// False when the lists have fewer tiles than that; bid then counts on past them.
template <class Fused, class Triple, class Single, bool TRANS_A, bool SCATTER = false>
__device__ __forceinline__ bool dsd_plan_tile(const DsdArgs& g, const PlanLists& plan, int& bid, char* smem) {
  static_assert(Fused::TN == Single::TN && Fused::TN == 2 * Triple::TN, "same column tiling");
  const int ntn = g.n / Fused::TN;
  const int pair_tiles = const_ints(plan.counts)[kTallPairs] * ntn;
  const int triple_tiles = const_ints(plan.counts)[kTallTriples] * 2 * ntn;
  const int single_tiles = const_ints(plan.counts)[kTallSingles] * ntn;
  if (bid < pair_tiles) {
    const int item = xcd_item(bid, pair_tiles, ntn, plan.group(kTallPairs));
    dsd_tile<Fused, 128, TRANS_A, true, 2, SCATTER>(g, const_ints(plan.list(kTallPairs))[item / ntn], (item % ntn) * Fused::TN, smem);
    return true;
  }
  bid -= pair_tiles;
  if (bid < triple_tiles) {
    const int item = xcd_item(bid, triple_tiles, 2 * ntn, plan.group(kTallTriples));
    dsd_tile<Triple, 128, TRANS_A, true, 3, SCATTER>(g, const_ints(plan.list(kTallTriples))[item / (2 * ntn)], (item % (2 * ntn)) * Triple::TN, smem);
    return true;
  }
  bid -= triple_tiles;
  if (bid < single_tiles) {
    // (in order of length: no contiguous shares; by stripes of the dense operand when the plan says so, in its 256-wide tiles)
    const int item = xcd_lines(bid, single_tiles, ntn, (plan.stripe_from(true) + 1) >> 1);
    dsd_tile<Single, 128, TRANS_A, true, 1, SCATTER>(g, const_ints(plan.list(kTallSingles))[item / ntn], (item % ntn) * Single::TN, smem);
    return true;
  }
  bid -= single_tiles;
  return false;
}

}  // namespace stk
