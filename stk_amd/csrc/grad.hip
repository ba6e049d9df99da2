// stk_dsd_dds, stk_dsd_dsd and stk_sdd_dsd: the two gradients of a product in one launch.
//
// The backward pass of S = lhs x rhs (sampled on a topology) computes dS x rhs^T, a dsd, and lhs^T x dS, a dds,
// from the same sparse values dS.  Here both run as one grid: first the tiles of the dsd (long walks along a block
// row), then the tiles of the dds (short walks down a block column), so that the many short tiles fill the compute
// units that the last long ones leave idle, and the blocks of dS that the dsd brought into the caches are still
// on their way through them when the dds asks for them.  The tiles are the ones of stk_dsd and stk_dds
// (dsd_tile.h, dds_tile.h), so the results are theirs bit for bit.
//
// When rhs reached the sampled product as a .t() view of a row-major [n, k] tensor (weights stored one row per output
// feature), the second gradient is wanted in that tensor's layout: dS^T x lhs, a dsd on the transposed dS.
// stk_dsd_dsd runs that pair the same way, the long row walks first, the short column walks behind them.
//
// The backward pass of y = op(S) x rhs computes dy x rhs^T on the topology, an sdd, and op(S)^T x dy, a dsd, from
// the same dy.  stk_sdd_dsd runs them as one grid in the same way: the tiles of the sdd, which contract over all
// of rhs's columns, then the tiles of the dsd (sdd_tile.h, dsd_tile.h).
#include "dds_tile.h"
#include "dsd_tile.h"
#include "sdd_tile.h"
#include <initializer_list>

namespace stk {

// 128-blocks, eight wavefronts, tiles from the plan's lists as in dsd_fused_kernel and dds_fused_kernel.
template <class DsdFused, class DsdTriple, class DsdSingle, class DdsFused, class DdsSingle>
__global__ __launch_bounds__(512, 2) void dsd_dds_kernel(DsdArgs d, PlanLists rows, DdsArgs s, PlanLists cols) {
  extern __shared__ __align__(16) char smem[];
  static_assert(DdsFused::TM == DdsSingle::TM, "same row tiling");
  const int ntm = s.m / DdsFused::TM;
  int bid = blockIdx.x;
  if (dsd_plan_tile<DsdFused, DsdTriple, DsdSingle, false>(d, rows, bid, smem)) return;
  const int pair_tiles = const_ints(cols.counts)[kPairs] * ntm, single_tiles = const_ints(cols.counts)[kSingles] * ntm;
  if (bid < pair_tiles) {
    const int item = xcd_item(bid, pair_tiles, ntm, cols.group(kPairs));
    dds_tile<DdsFused, 128, false, true, 2>(s, const_ints(cols.list(kPairs))[item / ntm], (item % ntm) * DdsFused::TM, smem);
    return;
  }
  bid -= pair_tiles;
  if (bid < single_tiles) {
    // (in order of length: no contiguous shares; by stripes of the dense operand when the plan says so, in its 256-wide tiles)
    const int item = xcd_lines(bid, single_tiles, ntm, (cols.stripe_from(false) + 1) >> 1);
    dds_tile<DdsSingle, 128, false, true, 1>(s, const_ints(cols.list(kSingles))[item / ntm], (item % ntm) * DdsSingle::TM, smem);
  }
}

constexpr int largest(std::initializer_list<int> values) {
  int most = 0;
  for (int v : values) most = v > most ? v : most;
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
  constexpr int lds = largest({DsdFused::kSmemBytes, DsdSingle::kSmemBytes, DsdTriple::kSmemBytes, DdsFused::kSmemBytes, DdsSingle::kSmemBytes});
  auto kernel = &dsd_dds_kernel<DsdFused, DsdTriple, DsdSingle, DdsFused, DdsSingle>;
  static const int once = (set_lds_limit(kernel, lds), 0);
  (void)once;
  // upper bound: every line a tile of its own in both products
  const int grid = d.block_rows * (d.n / DsdFused::TN) + s.block_cols * (s.m / DdsFused::TM);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(512), lds, stream, d, rows, s, cols);
}

// 128-blocks, eight wavefronts: the tiles of S x rhs from the plan's lists of block rows, then the tiles of
// S^T x rhs_t from its lists of block columns, both as in dsd_fused_kernel.
template <class Fused, class Triple, class Single, class FusedT, class TripleT, class SingleT>
__global__ __launch_bounds__(512, 2) void dsd_dsd_kernel(DsdArgs d, PlanLists rows, DsdArgs t, PlanLists cols) {
  extern __shared__ __align__(16) char smem[];
  int bid = blockIdx.x;
  if (dsd_plan_tile<Fused, Triple, Single, false>(d, rows, bid, smem)) return;
  dsd_plan_tile<FusedT, TripleT, SingleT, true>(t, cols, bid, smem);
}

// Both dense operands row-major.  STREAM / STREAM_T: the rhs panels of the product are read about once.
template <bool BF16, bool STREAM, bool STREAM_T>
static void launch_dsd_dsd(const DsdArgs& d, const PlanLists& rows, const DsdArgs& t, const PlanLists& cols, hipStream_t stream) {
  // the configurations of launch_dsd for the plain and for the transposed sparse operand
  using Fused = TileCfg<4, 2, 2, 4, 1, 2, 2, true, false, BF16, STK_DSD_KT, STK_DSD_STAGES, false, STREAM>;
  using Single = TileCfg<2, 4, 2, 2, 1, 1, 2, true, false, BF16, STK_DSD_KT, STK_DSD_STAGES, false, STREAM>;
  using Triple = TileCfg<4, 2, 3, 2, 1, 3, 1, true, false, BF16, STK_DSD_KT, STK_DSD_STAGES, false, STREAM>;
  using FusedT = TileCfg<4, 2, 2, 4, 1, 2, 2, false, false, BF16, STK_DSD_T_KT, STK_DSD_T_STAGES, false, STREAM_T>;
  using SingleT = TileCfg<2, 4, 2, 2, 1, 1, 2, false, false, BF16, STK_DSD_T_KT, STK_DSD_T_STAGES, false, STREAM_T>;
  using TripleT = TileCfg<4, 2, 3, 2, 1, 3, 1, false, false, BF16, STK_DSD_T_KT, STK_DSD_T_STAGES, false, STREAM_T>;
  constexpr int lds = largest({Fused::kSmemBytes, Single::kSmemBytes, Triple::kSmemBytes, FusedT::kSmemBytes, SingleT::kSmemBytes,
                               TripleT::kSmemBytes});
  auto kernel = &dsd_dsd_kernel<Fused, Triple, Single, FusedT, TripleT, SingleT>;
  static const int once = (set_lds_limit(kernel, lds), 0);
  (void)once;
  // upper bound: every line a tile of its own in both products
  const int grid = d.block_rows * (d.n / Fused::TN) + t.block_rows * (t.n / FusedT::TN);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(512), lds, stream, d, rows, t, cols);
}

// 128-blocks, eight wavefronts: the first `walkers` workgroups (one per compute unit) walk the tile list of the sdd as
// in sdd_fused_kernel; the workgroups behind them take the tiles of the dsd from the plan's lists of lines as in
// dsd_fused_kernel, one each, as the walkers leave.  The grid is an upper bound for the dsd.
template <class SddQuad, class SddPair, class SddTriple, class DsdFused, class DsdTriple, class DsdSingle, bool TRANS_A>
__global__ __launch_bounds__(512, 2) void sdd_dsd_kernel(SddArgs a, DsdArgs d, PlanLists lines, int walkers) {
  extern __shared__ __align__(16) char smem[];
  int bid = blockIdx.x;
  if (bid < walkers) {
    sdd_walk_plan<SddQuad, SddPair, SddTriple, true>(a, bid, walkers, smem);
    return;
  }
  bid -= walkers;
  dsd_plan_tile<DsdFused, DsdTriple, DsdSingle, TRANS_A>(d, lines, bid, smem);
}

// Both operands of the sdd K-major (a row-major lhs and a .t() view as rhs), rhs of the dsd row-major: the layouts the
// backward pass of a product with a row-major rhs produces.  STREAM: the rhs panels of the dsd are read about once.
template <bool BF16, bool TRANS_A, bool STREAM>
static void launch_sdd_dsd(const SddArgs& a, const DsdArgs& d, const PlanLists& lines, hipStream_t stream) {
  // the configurations of launch_sdd (both operands K-major: 64-deep K-tiles on two stages) and launch_dsd
  using SddQuad = TileCfg<4, 2, 2, 4, 1, 2, 2, true, true, BF16, 64, 2>;
  using SddPair = TileCfg<2, 4, 2, 2, 1, 1, 2, true, true, BF16, 64, 2>;
  using SddTriple = TileCfg<4, 2, 3, 2, 1, 3, 1, true, true, BF16, 64, 2>;
  constexpr int KT = TRANS_A ? STK_DSD_T_KT : STK_DSD_KT, S = TRANS_A ? STK_DSD_T_STAGES : STK_DSD_STAGES;
  using DsdFused = TileCfg<4, 2, 2, 4, 1, 2, 2, !TRANS_A, false, BF16, KT, S, false, STREAM>;
  using DsdSingle = TileCfg<2, 4, 2, 2, 1, 1, 2, !TRANS_A, false, BF16, KT, S, false, STREAM>;
  using DsdTriple = TileCfg<4, 2, 3, 2, 1, 3, 1, !TRANS_A, false, BF16, KT, S, false, STREAM>;
  constexpr int lds = largest({SddQuad::kSmemBytes, SddPair::kSmemBytes, SddTriple::kSmemBytes, DsdFused::kSmemBytes, DsdSingle::kSmemBytes,
                               DsdTriple::kSmemBytes});
  auto kernel = &sdd_dsd_kernel<SddQuad, SddPair, SddTriple, DsdFused, DsdTriple, DsdSingle, TRANS_A>;
  static const int once = (set_lds_limit(kernel, lds), 0);
  (void)once;
  // the walkers of the sdd (as many as it would have workgroups on its own), then every line of the dsd a tile of its own
  const int most = (int)sdd_max_tiles(a.block_rows, a.nnz), units = STK_SDD_PERSISTENT ? compute_units() : 0;
  const int walkers = units > 0 && units < most ? units : most;
  const int grid = walkers + d.block_rows * (d.n / DsdFused::TN);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(512), lds, stream, a, d, lines, walkers);
}

}  // namespace stk

extern "C" int stk_dsd_dds(int64_t m, int64_t k,
                           const void* data, const int32_t* offsets, const void* column_indices,
                           const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                           int64_t n_dsd, const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n, void* out_dsd, int64_t out_dsd_stride,
                           int64_t m_dds, const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k, void* out_dds, int64_t out_dds_stride,
                           int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream) {
  using namespace stk;
  if (dtype == STK_F32) {
    // float32 values have no joint launch: the two products one after the other
    const int first = stk_dsd(m, k, n_dsd, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 0, rhs, rhs_stride_k, rhs_stride_n,
                              out_dsd, out_dsd_stride, nnz, blocking, dtype, index_dtype, plan, nullptr, 0, stream);
    if (first != STK_OK) return first;
    return stk_dds(m_dds, m, k, lhs, lhs_stride_m, lhs_stride_k, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 0,
                   out_dds, out_dds_stride, nnz, blocking, dtype, index_dtype, plan, stream);
  }
  DsdProblem dsd;
  DdsProblem dds;
  int rc = dsd_problem("stk_dsd_dds", m, k, n_dsd, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 0, rhs, rhs_stride_k,
                       rhs_stride_n, out_dsd, out_dsd_stride, nnz, blocking, dtype, index_dtype, plan, &dsd);
  if (rc != STK_OK) return rc;
  rc = dds_problem("stk_dsd_dds", m_dds, m, k, lhs, lhs_stride_m, lhs_stride_k, data, offsets, column_indices, offsets_t, column_indices_t,
                   block_offsets_t, 0, out_dds, out_dds_stride, nnz, blocking, dtype, index_dtype, plan, &dds);
  if (rc != STK_OK) return rc;
  // (the grid of the one launch - an upper bound on the tiles of both products - must be a 32-bit count)
  const bool together = plan && blocking == 128 && nnz > 0 && !dsd.empty && !dds.empty && dsd.bk && !dds.ak && n_dsd % 256 == 0 &&
                        m_dds % 256 == 0 && !dsd.g.small && !dds.g.small &&
                        (int64_t)dsd.g.block_rows * (n_dsd / 256) + (int64_t)dds.g.block_cols * (m_dds / 256) <= INT32_MAX;
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

extern "C" int stk_dsd_dsd(int64_t m, int64_t k,
                           const void* data, const int32_t* offsets, const void* column_indices,
                           const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                           int64_t n, const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n, void* out, int64_t out_stride,
                           int64_t n_t, const void* rhs_t, int64_t rhs_t_stride_k, int64_t rhs_t_stride_n, void* out_t, int64_t out_t_stride,
                           int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream) {
  using namespace stk;
  if (dtype == STK_F32) {
    const int first = stk_dsd(m, k, n, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 0, rhs, rhs_stride_k, rhs_stride_n, out,
                              out_stride, nnz, blocking, dtype, index_dtype, plan, nullptr, 0, stream);
    if (first != STK_OK) return first;
    return stk_dsd(k, m, n_t, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 1, rhs_t, rhs_t_stride_k, rhs_t_stride_n,
                   out_t, out_t_stride, nnz, blocking, dtype, index_dtype, plan, nullptr, 0, stream);
  }
  DsdProblem plain, transposed;
  int rc = dsd_problem("stk_dsd_dsd", m, k, n, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 0, rhs, rhs_stride_k,
                       rhs_stride_n, out, out_stride, nnz, blocking, dtype, index_dtype, plan, &plain);
  if (rc != STK_OK) return rc;
  rc = dsd_problem("stk_dsd_dsd", k, m, n_t, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 1, rhs_t, rhs_t_stride_k,
                   rhs_t_stride_n, out_t, out_t_stride, nnz, blocking, dtype, index_dtype, plan, &transposed);
  if (rc != STK_OK) return rc;
  // (the grid of the one launch - an upper bound on the tiles of both products - must be a 32-bit count)
  const bool together = plan && blocking == 128 && nnz > 0 && !plain.empty && !transposed.empty && !plain.bk && !transposed.bk && n % 256 == 0 &&
                        n_t % 256 == 0 && !plain.g.small && !transposed.g.small &&
                        (int64_t)plain.g.block_rows * (n / 256) + (int64_t)transposed.g.block_rows * (n_t / 256) <= INT32_MAX;
  if (!together) {
    // shapes or layouts the joint launch has no tiles for: the two products one after the other
    rc = stk_dsd(m, k, n, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 0, rhs, rhs_stride_k, rhs_stride_n, out,
                 out_stride, nnz, blocking, dtype, index_dtype, plan, nullptr, 0, stream);
    if (rc != STK_OK) return rc;
    return stk_dsd(k, m, n_t, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, 1, rhs_t, rhs_t_stride_k, rhs_t_stride_n,
                   out_t, out_t_stride, nnz, blocking, dtype, index_dtype, plan, nullptr, 0, stream);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
#define STK_DSD_DSD_CASE(BF, ST, STT)                                                                            \
  if ((dtype == STK_BF16) == BF && plain.stream_rhs == ST && transposed.stream_rhs == STT) {                      \
    launch_dsd_dsd<BF, ST, STT>(plain.g, plain.lists, transposed.g, transposed.lists, s);                         \
    return check_launch("stk_dsd_dsd");                                                                           \
  }
  STK_DSD_DSD_CASE(true, true, true) STK_DSD_DSD_CASE(true, true, false) STK_DSD_DSD_CASE(true, false, true) STK_DSD_DSD_CASE(true, false, false)
  STK_DSD_DSD_CASE(false, true, true) STK_DSD_DSD_CASE(false, true, false) STK_DSD_DSD_CASE(false, false, true) STK_DSD_DSD_CASE(false, false, false)
  return fail(STK_ERR_UNSUPPORTED, "stk_dsd_dsd: no kernel for this configuration");
}

extern "C" int stk_sdd_dsd(int64_t m, int64_t n,
                           const int32_t* offsets, const void* row_indices, const void* column_indices,
                           const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                           const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                           const void* rhs_sdd, int64_t rhs_sdd_stride_k, int64_t rhs_sdd_stride_n, int64_t k_sdd, void* out_sdd,
                           const void* data, int transpose_a, int64_t n_dsd, const void* rhs_dsd, int64_t rhs_dsd_stride_k, int64_t rhs_dsd_stride_n,
                           void* out_dsd, int64_t out_dsd_stride,
                           int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream) {
  using namespace stk;
  if (dtype == STK_F32) {
    const int first = stk_sdd(lhs, lhs_stride_m, lhs_stride_k, rhs_sdd, rhs_sdd_stride_k, rhs_sdd_stride_n, m, k_sdd, n, out_sdd, offsets, row_indices,
                              column_indices, block_offsets_t, nnz, blocking, dtype, index_dtype, plan, stream);
    if (first != STK_OK) return first;
    return stk_dsd(transpose_a ? n : m, transpose_a ? m : n, n_dsd, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t,
                   transpose_a, rhs_dsd, rhs_dsd_stride_k, rhs_dsd_stride_n, out_dsd, out_dsd_stride, nnz, blocking, dtype, index_dtype, plan, nullptr, 0,
                   stream);
  }
  SddProblem sdd;
  DsdProblem dsd;
  int rc = sdd_problem("stk_sdd_dsd", lhs, lhs_stride_m, lhs_stride_k, rhs_sdd, rhs_sdd_stride_k, rhs_sdd_stride_n, m, k_sdd, n, out_sdd, offsets,
                       row_indices, column_indices, block_offsets_t, nnz, blocking, dtype, index_dtype, plan, STK_ACT_NONE, nullptr, &sdd);
  if (rc != STK_OK) return rc;
  // the dsd multiplies op(S): [m, n] as stored, [n, m] transposed
  const int64_t m_dsd = transpose_a ? n : m, k_dsd = transpose_a ? m : n;
  rc = dsd_problem("stk_sdd_dsd", m_dsd, k_dsd, n_dsd, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, transpose_a,
                   rhs_dsd, rhs_dsd_stride_k, rhs_dsd_stride_n, out_dsd, out_dsd_stride, nnz, blocking, dtype, index_dtype, plan, &dsd);
  if (rc != STK_OK) return rc;
  const bool together = plan && blocking == 128 && !sdd.empty && !dsd.empty && sdd.g.tiles && nnz > compute_units() && sdd.ak && sdd.bk &&
                        k_sdd % 64 == 0 && !dsd.bk && n_dsd % 256 == 0 && !dsd.g.small &&
                        sdd_max_tiles(sdd.g.block_rows, nnz) + (int64_t)dsd.g.block_rows * (n_dsd / 256) <= INT32_MAX;
  if (!together) {
    // shapes or layouts the joint launch has no tiles for: the two products one after the other
    rc = stk_sdd(lhs, lhs_stride_m, lhs_stride_k, rhs_sdd, rhs_sdd_stride_k, rhs_sdd_stride_n, m, k_sdd, n, out_sdd, offsets, row_indices,
                 column_indices, block_offsets_t, nnz, blocking, dtype, index_dtype, plan, stream);
    if (rc != STK_OK) return rc;
    return stk_dsd(m_dsd, k_dsd, n_dsd, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, transpose_a, rhs_dsd,
                   rhs_dsd_stride_k, rhs_dsd_stride_n, out_dsd, out_dsd_stride, nnz, blocking, dtype, index_dtype, plan, nullptr, 0, stream);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
#define STK_SDD_DSD_CASE(BF, TA)                                                                   \
  if ((dtype == STK_BF16) == BF && dsd.ta == TA) {                                                 \
    if (dsd.stream_rhs) launch_sdd_dsd<BF, TA, true>(sdd.g, dsd.g, dsd.lists, s);                  \
    else launch_sdd_dsd<BF, TA, false>(sdd.g, dsd.g, dsd.lists, s);                                \
    return check_launch("stk_sdd_dsd");                                                            \
  }
  STK_SDD_DSD_CASE(true, true) STK_SDD_DSD_CASE(true, false) STK_SDD_DSD_CASE(false, true) STK_SDD_DSD_CASE(false, false)
  return fail(STK_ERR_UNSUPPORTED, "stk_sdd_dsd: no kernel for this configuration");
}
