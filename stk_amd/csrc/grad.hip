// stk_dsd_dds: the two operand gradients of a sampled product in one launch.
//
// The backward pass of S = lhs x rhs (sampled on a topology) computes dS x rhs^T, a dsd, and lhs^T x dS, a dds,
// from the same sparse values dS.  Here both run as one grid: first the tiles of the dsd (long walks along a block
// row), then the tiles of the dds (short walks down a block column), so that the many short tiles fill the compute
// units that the last long ones leave idle, and the blocks of dS that the dsd brought into the caches are still
// on their way through them when the dds asks for them.  The tiles are the ones of stk_dsd and stk_dds
// (dsd_tile.h, dds_tile.h), so the results are theirs bit for bit.
#include "dds_tile.h"
#include "dsd_tile.h"

namespace stk {

// 128-blocks, eight wavefronts, tiles from the plan's lists as in dsd_fused_kernel and dds_fused_kernel.
template <class DsdFused, class DsdTriple, class DsdSingle, class DdsFused, class DdsSingle>
__global__ __launch_bounds__(512, 2) void dsd_dds_kernel(DsdArgs d, PlanLists rows, DdsArgs s, PlanLists cols) {
  extern __shared__ __align__(16) char smem[];
  static_assert(DsdFused::TN == DsdSingle::TN && DsdFused::TN == 2 * DsdTriple::TN && DdsFused::TM == DdsSingle::TM, "same tiling");
  const int ntn = d.n / DsdFused::TN, ntm = s.m / DdsFused::TM;
  int bid = blockIdx.x;
  {
    const int pair_tiles = const_ints(rows.counts)[kTallPairs] * ntn;
    const int triple_tiles = const_ints(rows.counts)[kTallTriples] * 2 * ntn;
    const int single_tiles = const_ints(rows.counts)[kTallSingles] * ntn;
    if (bid < pair_tiles) {
      const int item = xcd_item(bid, pair_tiles, ntn, rows.group(kTallPairs));
      dsd_tile<DsdFused, 128, false, true, 2>(d, const_ints(rows.list(kTallPairs))[item / ntn], (item % ntn) * DsdFused::TN, smem);
      return;
    }
    bid -= pair_tiles;
    if (bid < triple_tiles) {
      const int item = xcd_item(bid, triple_tiles, 2 * ntn, rows.group(kTallTriples));
      dsd_tile<DsdTriple, 128, false, true, 3>(d, const_ints(rows.list(kTallTriples))[item / (2 * ntn)], (item % (2 * ntn)) * DsdTriple::TN, smem);
      return;
    }
    bid -= triple_tiles;
    if (bid < single_tiles) {
      const int item = xcd_grouped(bid, single_tiles);  // (in order of length: no contiguous shares)
      dsd_tile<DsdSingle, 128, false, true, 1>(d, const_ints(rows.list(kTallSingles))[item / ntn], (item % ntn) * DsdSingle::TN, smem);
      return;
    }
    bid -= single_tiles;
  }
  const int pair_tiles = const_ints(cols.counts)[kPairs] * ntm, single_tiles = const_ints(cols.counts)[kSingles] * ntm;
  if (bid < pair_tiles) {
    const int item = xcd_item(bid, pair_tiles, ntm, cols.group(kPairs));
    dds_tile<DdsFused, 128, false, true, 2>(s, const_ints(cols.list(kPairs))[item / ntm], (item % ntm) * DdsFused::TM, smem);
    return;
  }
  bid -= pair_tiles;
  if (bid < single_tiles) {
    const int item = xcd_grouped(bid, single_tiles);  // (in order of length: no contiguous shares)
    dds_tile<DdsSingle, 128, false, true, 1>(s, const_ints(cols.list(kSingles))[item / ntm], (item % ntm) * DdsSingle::TM, smem);
  }
}

constexpr int largest(int a, int b, int c, int d, int e) {
  int most = a;
  for (int v : {b, c, d, e}) most = v > most ? v : most;
  return most;
}

// rhs of the dsd K-major (a .t() view), lhs of the dds MN-major (a .t() view): the layouts the backward pass of a
// product of two row-major operands produces.  STREAM: the lhs panels of the dds are read about once.
template <bool BF16, bool STREAM>
static void launch_dsd_dds(const DsdArgs& d, const PlanLists& rows, const DdsArgs& s, const PlanLists& cols, hipStream_t stream) {
  // the configurations of launch_dsd (K-major rhs: 64-deep K-tiles on two stages) and launch_dds (MN-major lhs)
  using DsdFused = TileCfg<4, 2, 2, 4, 1, 2, 2, true, true, BF16, 64, 2>;
  using DsdSingle = TileCfg<2, 4, 2, 2, 1, 1, 2, true, true, BF16, 64, 2>;
  using DsdTriple = TileCfg<4, 2, 3, 2, 1, 3, 1, true, true, BF16, 64, 2>;
  using DdsFused = TileCfg<4, 2, 2, 4, 1, 2, 2, false, false, BF16, STK_DDS_KT, STK_DDS_STAGES, STREAM>;
  using DdsSingle = TileCfg<4, 2, 2, 2, 1, 2, 1, false, false, BF16, STK_DDS_KT, STK_DDS_STAGES, STREAM>;
  constexpr int lds = largest(DsdFused::kSmemBytes, DsdSingle::kSmemBytes, DsdTriple::kSmemBytes, DdsFused::kSmemBytes, DdsSingle::kSmemBytes);
  auto kernel = &dsd_dds_kernel<DsdFused, DsdTriple, DsdSingle, DdsFused, DdsSingle>;
  static const int once = (set_lds_limit(kernel, lds), 0);
  (void)once;
  // upper bound: every line a tile of its own in both products
  const int grid = d.block_rows * (d.n / DsdFused::TN) + s.block_cols * (s.m / DdsFused::TM);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(512), lds, stream, d, rows, s, cols);
}

}  // namespace stk

extern "C" int stk_dsd_dds(int64_t m, int64_t k,
                           const void* data, const int32_t* offsets, const void* column_indices,
                           const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                           int64_t n_dsd, const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n, void* out_dsd, int64_t out_dsd_stride,
                           int64_t m_dds, const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k, void* out_dds, int64_t out_dds_stride,
                           int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream) {
  using namespace stk;
  DsdProblem dsd;
  DdsProblem dds;
  int rc = dsd_problem("stk_dsd_dds", m, k, n_dsd, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 0, rhs, rhs_stride_k,
                       rhs_stride_n, out_dsd, out_dsd_stride, nnz, blocking, dtype, index_dtype, plan, &dsd);
  if (rc != STK_OK) return rc;
  rc = dds_problem("stk_dsd_dds", m_dds, m, k, lhs, lhs_stride_m, lhs_stride_k, data, offsets, column_indices, offsets_t, column_indices_t,
                   block_offsets_t, 0, out_dds, out_dds_stride, nnz, blocking, dtype, index_dtype, plan, &dds);
  if (rc != STK_OK) return rc;
  const bool together = plan && blocking == 128 && nnz > 0 && !dsd.empty && !dds.empty && dsd.bk && !dds.ak && n_dsd % 256 == 0 &&
                        m_dds % 256 == 0 && !dsd.g.small && !dds.g.small;
  if (!together) {
    // shapes or layouts the joint launch has no tiles for: the two products one after the other
    rc = stk_dsd(m, k, n_dsd, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 0, rhs, rhs_stride_k, rhs_stride_n,
                 out_dsd, out_dsd_stride, nnz, blocking, dtype, index_dtype, plan, nullptr, 0, stream);
    if (rc != STK_OK) return rc;
    return stk_dds(m_dds, m, k, lhs, lhs_stride_m, lhs_stride_k, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 0,
                   out_dds, out_dds_stride, nnz, blocking, dtype, index_dtype, plan, stream);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == STK_BF16) {
    if (dds.stream_lhs) launch_dsd_dds<true, true>(dsd.g, dsd.lists, dds.g, dds.lists, s);
    else launch_dsd_dds<true, false>(dsd.g, dsd.lists, dds.g, dds.lists, s);
  } else {
    if (dds.stream_lhs) launch_dsd_dds<false, true>(dsd.g, dsd.lists, dds.g, dds.lists, s);
    else launch_dsd_dds<false, false>(dsd.g, dsd.lists, dds.g, dds.lists, s);
  }
  return check_launch("stk_dsd_dds");
}
