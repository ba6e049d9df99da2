// stk_dds: dense = dense x op(sparse).
//
// A workgroup produces, for one tile of output rows, the output columns of one
// block column of op(sparse) - or of two neighbouring block columns with identical
// patterns, which then share every tile of the dense operand.  It walks the CSC
// column segment of the sparse operand (for a transposed sparse operand: the CSR
// row with direct block ids).
#include "dds_tile.h"

namespace stk {

// One block column per workgroup (four wavefronts).
template <class Cfg, int BLK, bool TRANS_B, bool FULL>
__global__ __launch_bounds__(Cfg::kThreads, 2) void dds_kernel(DdsArgs g) {
  extern __shared__ __align__(16) char smem[];
  const int ntm = (g.m + Cfg::TM - 1) / Cfg::TM;
  const int item = xcd_grouped(blockIdx.x, g.block_cols * ntm);  // no plan, no hint about the lines: small groups
  dds_tile<Cfg, BLK, TRANS_B, FULL, 1>(g, item / ntm, (item % ntm) * Cfg::TM, smem);
}

// Every block column on its own (four wavefronts), in the order of the plan's lists: the columns of the pairs,
// then the lone columns longest first - for launches with little work per compute unit, where the order in which
// the tiles start decides how evenly the units are loaded.
template <class Cfg, int BLK, bool TRANS_B>
__global__ __launch_bounds__(Cfg::kThreads, 2) void dds_lines_kernel(DdsArgs g, PlanLists plan) {
  extern __shared__ __align__(16) char smem[];
  const int ntm = (g.m + Cfg::TM - 1) / Cfg::TM;
  const int pairs = const_ints(plan.counts)[kPairs];
  const int tiles = (2 * pairs + const_ints(plan.counts)[kSingles]) * ntm;
  if ((int)blockIdx.x >= tiles) return;
  const int item = xcd_lines(blockIdx.x, tiles, ntm, plan.stripe_from(false));   // (by stripes of lhs rows when the columns share little)
  const int l = item / ntm;
  const int line = l < 2 * pairs ? const_ints(plan.list(kPairs))[l >> 1] + (l & 1) : const_ints(plan.list(kSingles))[l - 2 * pairs];
  dds_tile<Cfg, BLK, TRANS_B, true, 1>(g, line, (item % ntm) * Cfg::TM, smem);
}

// The lone block columns of a plan's list, one per workgroup (four wavefronts): what dds_fused64_kernel leaves.
template <class Cfg, int BLK, bool TRANS_B, bool FULL>
__global__ __launch_bounds__(Cfg::kThreads, 2) void dds_singles_kernel(DdsArgs g, PlanLists plan) {
  extern __shared__ __align__(16) char smem[];
  const int ntm = (g.m + Cfg::TM - 1) / Cfg::TM;
  const int tiles = const_ints(plan.counts)[kTallSingles] * ntm;
  if ((int)blockIdx.x >= tiles) return;
  const int item = xcd_grouped(blockIdx.x, tiles);
  dds_tile<Cfg, BLK, TRANS_B, FULL, 1>(g, const_ints(plan.list(kTallSingles))[item / ntm], (item % ntm) * Cfg::TM, smem);
}

// 64-blocks with a plan built for them, eight wavefronts: groups of four identical block columns as 256x256
// tiles (a group of three runs on the same shape with its fourth column dropped), pairs as 256x128 tiles; the
// dense operand is then read once per 256 or 128 columns instead of once per 64.  Lone columns are left to
// dds_singles_kernel.  The grid is an upper bound; the surplus leaves at once.
template <class Quad, class Pair, bool TRANS_B>
__global__ __launch_bounds__(512, 2) void dds_fused64_kernel(DdsArgs g, PlanLists plan) {
  extern __shared__ __align__(16) char smem[];
  static_assert(Quad::TM == Pair::TM, "same row tiling");
  const int ntm = g.m / Quad::TM;
  const int quad_tiles = const_ints(plan.counts)[kPairs] * ntm, triple_tiles = const_ints(plan.counts)[kTallTriples] * ntm;
  const int pair_tiles = const_ints(plan.counts)[kTallPairs] * ntm;
  int bid = blockIdx.x;
  // pairs first: they hold the lines that were too long for groups of four, the longest tiles of the launch
  if (bid < pair_tiles) {
    const int item = xcd_item(bid, pair_tiles, ntm, plan.group(kTallPairs));
    dds_tile<Pair, 64, TRANS_B, true, 2>(g, const_ints(plan.list(kTallPairs))[item / ntm], (item % ntm) * Pair::TM, smem, 2);
    return;
  }
  bid -= pair_tiles;
  if (bid < quad_tiles) {
    const int item = xcd_item(bid, quad_tiles, ntm, plan.group(kPairs));
    dds_tile<Quad, 64, TRANS_B, true, 4>(g, const_ints(plan.list(kPairs))[item / ntm], (item % ntm) * Quad::TM, smem, 4);
    return;
  }
  bid -= quad_tiles;
  if (bid < triple_tiles) {
    const int item = xcd_item(bid, triple_tiles, ntm, plan.group(kTallTriples));
    dds_tile<Quad, 64, TRANS_B, true, 4>(g, const_ints(plan.list(kTallTriples))[item / ntm], (item % ntm) * Quad::TM, smem, 3);
  }
}

// 128-blocks, eight wavefronts: 256x256 tiles over the pairs of identical block columns, then
// 256x128 tiles over the lone ones, taken from the lists of the plan (covered columns get no
// tile).  Without a plan every column is a lone column.
//
// One workgroup of this kernel fills a compute unit (its ring takes most of the LDS), so the grid is one workgroup
// per compute unit and every workgroup walks the tiles with the stride of the grid - the order in which the hardware
// would hand them out one launch at a time, without the launch (0.75 us per tile, measured with an empty kernel on
// the same grid) and without the three dependent loads of a tile's walk (list entry, offsets, entries: 1.1 us) in
// front of its first transfer: the walk of the next tile is looked up through the scalar unit while the first
// transfers of the current one are in flight.
// The id of the tile that a workgroup takes in its round `round` of a launch of one workgroup per compute unit: the
// tiles of a round are consecutive ids, and a workgroup keeps its compute die (id mod 8, the die its own id lies on),
// but odd rounds hand the tiles of a die out in reverse.  A list sorted by length then gives every workgroup a long
// tile of one round and a short one of the next, as the hardware's own hand-out to whoever is free first would.
__device__ __forceinline__ int round_tile(int round) {
  const int slots = gridDim.x >> 3, die = blockIdx.x & 7, slot = blockIdx.x >> 3;
  if ((gridDim.x & 7) || !(round & 1)) return round * gridDim.x + blockIdx.x;
  return round * gridDim.x + (slots - 1 - slot) * 8 + die;
}

// The tiles [first, first + count) of the launch, all of LINES block columns, that this workgroup takes (round_tile);
// locate(id) gives a tile's first block column and first output row.  `round` counts on from the call before.
template <class Cfg, bool TRANS_B, int LINES, class Locate>
__device__ __forceinline__ void dds_walk_tiles(const DdsArgs& g, int first, int count, Locate&& locate, char* smem, int& round, bool& used_lds) {
  int id = round_tile(round);
  while (id < first) id = round_tile(++round);
  if (id >= first + count) return;
  int line, m0;
  locate(id, line, m0);
  DdsWalk<LINES> walk;
  if (!dds_walk_scalar<LINES, TRANS_B>(g, line, LINES, walk)) walk = dds_walk<LINES, TRANS_B>(g, line, LINES);
  for (;;) {
    if (used_lds) __syncthreads();  // the staging area of the last tile's stores is the first ring stage of this one
    used_lds = true;
    const int next_id = round_tile(++round);
    const bool more = next_id < first + count;
    int next_line = line, next_m0 = m0;
    DdsWalk<LINES> next_walk = walk;
    bool have_next = false;
    auto look_ahead = [&] {
      if (more) {
        locate(next_id, next_line, next_m0);
        have_next = dds_walk_scalar<LINES, TRANS_B>(g, next_line, LINES, next_walk);
      }
    };
    if (walk.nseg <= 0) look_ahead();  // (a column without blocks has no main loop to hide it behind)
    dds_tile_of<Cfg, 128, TRANS_B, true, LINES>(g, walk, m0, smem, LINES, look_ahead);
    if (!more) return;
    id = next_id;
    line = next_line;
    m0 = next_m0;
    if (have_next) walk = next_walk;
    else walk = dds_walk<LINES, TRANS_B>(g, line, LINES);
  }
}

template <class Fused, class Single, bool TRANS_B>
__global__ __launch_bounds__(512, 2) void dds_fused_kernel(DdsArgs g, PlanLists plan) {
  extern __shared__ __align__(16) char smem[];
  static_assert(Fused::TM == Single::TM, "same row tiling");
  const int ntm = g.m / Fused::TM;
  bool used_lds = false;
  int round = 0;
  if (!plan.counts) {
    const int total = g.block_cols * ntm;
    dds_walk_tiles<Single, TRANS_B, 1>(g, 0, total, [&](int id, int& line, int& m0) {
      const int item = xcd_grouped(id, total);
      line = item / ntm, m0 = (item % ntm) * Single::TM;
    }, smem, round, used_lds);
    return;
  }
  const int pair_tiles = const_ints(plan.counts)[kPairs] * ntm, single_tiles = const_ints(plan.counts)[kSingles] * ntm;
  dds_walk_tiles<Fused, TRANS_B, 2>(g, 0, pair_tiles, [&](int id, int& line, int& m0) {
    const int item = xcd_item(id, pair_tiles, ntm, plan.group(kPairs));
    line = const_ints(plan.list(kPairs))[item / ntm], m0 = (item % ntm) * Fused::TM;
  }, smem, round, used_lds);
  // (in order of length: no contiguous shares; by stripes of the dense operand when the plan says so, in its 256-wide tiles)
  const int stripe_from = (plan.stripe_from(false) + 1) >> 1;
  dds_walk_tiles<Single, TRANS_B, 1>(g, pair_tiles, single_tiles, [&](int id, int& line, int& m0) {
    const int item = xcd_lines(id - pair_tiles, id, single_tiles, ntm, stripe_from);
    line = const_ints(plan.list(kSingles))[item / ntm], m0 = (item % ntm) * Single::TM;
  }, smem, round, used_lds);
}

template <class Cfg, int BLK, bool TRANS_B, bool FULL>
static void launch_one(const DdsArgs& g, hipStream_t stream) {
  static const int once = (set_lds_limit(&dds_kernel<Cfg, BLK, TRANS_B, FULL>, Cfg::kSmemBytes), 0);
  (void)once;
  const int ntm = (g.m + Cfg::TM - 1) / Cfg::TM;
  hipLaunchKernelGGL((dds_kernel<Cfg, BLK, TRANS_B, FULL>), dim3(g.block_cols * ntm), dim3(Cfg::kThreads), Cfg::kSmemBytes, stream, g);
}

// STREAM: every lhs column panel is read by few tiles and is loaded non-temporally.
template <bool BF16, int BLK, bool AK, bool TRANS_B, bool STREAM>
static void launch_dds(const DdsArgs& g, const PlanLists& plan, hipStream_t stream) {
  // K-major dense operand (row-major lhs): a 32-deep K-tile would use half of every 128-byte line it touches, so
  // 64-deep K-tiles (two stages fit) beat the deeper ring of 32-deep ones
  constexpr int KT = AK ? 64 : STK_DDS_KT, S = AK ? 2 : STK_DDS_STAGES;
  if constexpr (BLK == 128) {
    // eight wavefronts: 2x4... see dsd.hip; here 4x2 of 64x128 over two block columns, or 4x2 of 64x64 over one
    using Fused = TileCfg<4, 2, 2, 4, 1, 2, 2, AK, TRANS_B, BF16, KT, S, STREAM>;
    using Single = TileCfg<4, 2, 2, 2, 1, 2, 1, AK, TRANS_B, BF16, KT, S, STREAM>;
    // four wavefronts, 128x128, for row counts that are not a multiple of 256
    using Narrow = TileCfg<2, 2, 2, 2, 1, 1, 1, AK, TRANS_B, BF16, KT, S, STREAM>;
    using Reg = TileCfg<2, 2, 2, 2, 1, 1, 1, AK, TRANS_B, BF16, 64, 2>;
    if (g.m % Fused::TM == 0 && !g.small) {
      constexpr int lds = Fused::kSmemBytes > Single::kSmemBytes ? Fused::kSmemBytes : Single::kSmemBytes;
      static const int once = (set_lds_limit(&dds_fused_kernel<Fused, Single, TRANS_B>, lds), 0);
      (void)once;
      // one workgroup per compute unit; the tiles are at most one per block column and row tile
      const int units = compute_units(), tiles = g.block_cols * (g.m / Fused::TM);
      hipLaunchKernelGGL((dds_fused_kernel<Fused, Single, TRANS_B>), dim3(units > 0 && units < tiles ? units : tiles), dim3(512), lds, stream, g, plan);
    } else if (g.m % Narrow::TM == 0 && plan.counts) {
      static const int once = (set_lds_limit(&dds_lines_kernel<Narrow, BLK, TRANS_B>, Narrow::kSmemBytes), 0);
      (void)once;
      hipLaunchKernelGGL((dds_lines_kernel<Narrow, BLK, TRANS_B>), dim3(g.block_cols * (g.m / Narrow::TM)), dim3(Narrow::kThreads),
                         Narrow::kSmemBytes, stream, g, plan);
    } else if (g.m % Narrow::TM == 0) {
      launch_one<Narrow, BLK, TRANS_B, true>(g, stream);
    } else {
      launch_one<Reg, BLK, TRANS_B, false>(g, stream);  // ragged m: predicated register staging
    }
  } else {
    // 64-blocks: 4x1 wavefronts of 64x64 (tile 256x64)
    using Dma = TileCfg<4, 1, 2, 2, 1, 1, 1, AK, TRANS_B, BF16, 64, 2, STREAM>;
    if (plan.counts && g.m % 256 == 0 && !g.small) {
      // groups of identical block columns on eight wavefronts (4x2 of 64x128 over four block columns, 4x2 of 64x64
      // over two), then the lone columns one per four-wave workgroup; both grids are upper bounds
      using Quad = TileCfg<4, 2, 2, 4, 1, 2, 4, AK, TRANS_B, BF16, 64, 2, STREAM>;
      using Pair = TileCfg<4, 2, 2, 2, 1, 2, 2, AK, TRANS_B, BF16, 64, 2, STREAM>;
      constexpr int lds = Quad::kSmemBytes > Pair::kSmemBytes ? Quad::kSmemBytes : Pair::kSmemBytes;
      static const int once = (set_lds_limit(&dds_fused64_kernel<Quad, Pair, TRANS_B>, lds), set_lds_limit(&dds_singles_kernel<Dma, 64, TRANS_B, true>, Dma::kSmemBytes), 0);
      (void)once;
      const int ntm = g.m / 256;
      hipLaunchKernelGGL((dds_fused64_kernel<Quad, Pair, TRANS_B>), dim3((g.block_cols + 1) / 2 * ntm), dim3(512), lds, stream, g, plan);
      hipLaunchKernelGGL((dds_singles_kernel<Dma, 64, TRANS_B, true>), dim3(g.block_cols * ntm), dim3(Dma::kThreads), Dma::kSmemBytes, stream, g, plan);
      return;
    }
    if (g.m % Dma::TM == 0) launch_one<Dma, BLK, TRANS_B, true>(g, stream);
    else launch_one<Dma, BLK, TRANS_B, false>(g, stream);
  }
}

}  // namespace stk

// Checks the arguments of a dds and turns them into the kernels' view of the problem.  STK_OK with p->empty set when
// there is nothing to compute.
int stk::dds_problem(const char* who, int64_t m, int64_t k, int64_t n,
                     const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                     const void* data, const int32_t* offsets, const void* column_indices,
                     const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                     int transpose_b, void* out, int64_t out_stride_m,
                     int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, DdsProblem* p) {
  p->empty = false;
  if (blocking != 64 && blocking != 128) return fail(STK_ERR_UNSUPPORTED, "%s: blocking %d (64 or 128)", who, blocking);
  if (dtype != STK_F16 && dtype != STK_BF16) return fail(STK_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "%s: index dtype %d", who, index_dtype);
  if (m < 0 || n < 0 || k < 0 || nnz < 0) return fail(STK_ERR_DIMS, "%s: negative size", who);
  if (k % blocking || n % blocking || m % 8)
    return fail(STK_ERR_DIMS, "incompatible dimensions: dense [%lld, %lld] x sparse [%lld, %lld] with blocking %d",
                (long long)m, (long long)k, (long long)k, (long long)n, blocking);
  if (m == 0 || n == 0) {
    p->empty = true;
    return STK_OK;
  }
  const int64_t block_cols = n / blocking;
  if (block_cols * ((m + 63) / 64) > INT32_MAX || m > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "%s: size exceeds 32-bit range", who);
  const bool ak = lhs_stride_k == 1;   // row-major lhs: K-major tile
  if (!ak && lhs_stride_m != 1) return fail(STK_ERR_UNSUPPORTED, "%s: lhs needs a unit stride", who);
  const int64_t lda = ak ? lhs_stride_m : lhs_stride_k;
  if (lda % 8 || out_stride_m % 8 || !aligned16(lhs) || !aligned16(out) || !aligned16(data))
    return fail(STK_ERR_UNSUPPORTED, "%s: operands need 16-byte aligned bases and leading dimensions divisible by 8", who);
  if (lda >= (1 << 24)) return fail(STK_ERR_UNSUPPORTED, "%s: leading dimension exceeds 2^24 elements", who);
  const bool tb = transpose_b != 0;
  DdsArgs& g = p->g;
  g.lhs = static_cast<const elem_t*>(lhs);
  g.lda = lda;
  g.data = static_cast<const elem_t*>(data);
  g.walk_offsets = tb ? offsets : offsets_t;
  g.walk_columns = tb ? column_indices : column_indices_t;
  g.walk_blocks = tb ? nullptr : block_offsets_t;
  g.out = static_cast<elem_t*>(out);
  g.ldc = out_stride_m;
  g.m = (int)m;
  g.block_cols = (int)block_cols;
  g.idx32 = index_dtype == STK_I32;
  // a dense-operand column panel (one block of k) is read once per tile that walks a block in that block row of
  // op(S): with few blocks per row it is streamed
  // (lhs with unit stride along m only: a K-major tile uses half a cache line per K-tile and needs the line to stay)
  p->stream_lhs = !ak && nnz <= 4 * (k / blocking);
  p->ak = ak;
  p->tb = tb;
  g.small = nnz * (m / 128) < kSmallWorkPerUnit * compute_units();
  g.scalar_walk = ((reinterpret_cast<uintptr_t>(g.walk_columns) | reinterpret_cast<uintptr_t>(g.walk_blocks)) & 3u) == 0;
  if (!g.walk_offsets || (nnz > 0 && (!g.walk_columns || (!tb && !g.walk_blocks) || !data))) return fail(STK_ERR_DIMS, "%s: missing metadata pointer", who);
  // lists of the walked lines: block columns of the stored matrix [k, n], or block rows of the stored [n, k]
  p->lists = PlanLists{nullptr, nullptr, 0};
  if (plan) p->lists = tb ? plan_lists_of(plan_body(plan, n / blocking, nnz), n / blocking, k / blocking, false)
                          : plan_lists_of(plan_body(plan, k / blocking, nnz), k / blocking, n / blocking, true);
  return STK_OK;
}

extern "C" int stk_dds(int64_t m, int64_t k, int64_t n,
                       const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                       const void* data, const int32_t* offsets, const void* column_indices,
                       const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                       int transpose_b,
                       void* out, int64_t out_stride_m,
                       int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream) {
  using namespace stk;
  if (dtype == STK_F32) {
    if (m < 0 || n < 0 || k < 0 || nnz < 0) return fail(STK_ERR_DIMS, "stk_dds: negative size");
    if (blocking > 0 && (k % blocking || n % blocking))
      return fail(STK_ERR_DIMS, "incompatible dimensions: dense [%lld, %lld] x sparse [%lld, %lld] with blocking %d", (long long)m, (long long)k,
                  (long long)k, (long long)n, blocking);
    const bool tb = transpose_b != 0;
    if (!tb && nnz > 0 && !block_offsets_t) return fail(STK_ERR_DIMS, "stk_dds: missing metadata pointer");
    return walk_f32(false, "stk_dds", blocking > 0 ? n / blocking : 0, m, data, tb ? offsets : offsets_t, tb ? column_indices : column_indices_t,
                    tb ? nullptr : block_offsets_t, tb, lhs, lhs_stride_m, lhs_stride_k, out, out_stride_m, nnz, blocking, index_dtype,
                    static_cast<hipStream_t>(stream));
  }
  DdsProblem problem;
  const int rc = dds_problem("stk_dds", m, k, n, lhs, lhs_stride_m, lhs_stride_k, data, offsets, column_indices, offsets_t, column_indices_t,
                             block_offsets_t, transpose_b, out, out_stride_m, nnz, blocking, dtype, index_dtype, plan, &problem);
  if (rc != STK_OK || problem.empty) return rc;
  const DdsArgs& g = problem.g;
  const PlanLists& lists = problem.lists;
  const bool ak = problem.ak, tb = problem.tb, stream_lhs = problem.stream_lhs;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define STK_DDS_CASE(BF, BLK, AK, TB)                                         \
  if ((dtype == STK_BF16) == BF && blocking == BLK && ak == AK && tb == TB) { \
    if (!AK && stream_lhs) launch_dds<BF, BLK, AK, TB, !AK>(g, lists, s);         \
    else launch_dds<BF, BLK, AK, TB, false>(g, lists, s);                         \
    return check_launch("stk_dds");                                           \
  }
#define STK_DDS_LAYOUTS(BF, BLK) \
  STK_DDS_CASE(BF, BLK, true, true) STK_DDS_CASE(BF, BLK, true, false) STK_DDS_CASE(BF, BLK, false, true) STK_DDS_CASE(BF, BLK, false, false)
  STK_DDS_LAYOUTS(true, 128) STK_DDS_LAYOUTS(false, 128) STK_DDS_LAYOUTS(true, 64) STK_DDS_LAYOUTS(false, 64)
  return fail(STK_ERR_UNSUPPORTED, "stk_dds: no kernel for this configuration");
}
