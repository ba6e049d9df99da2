// stk_sdd: sampled dense x dense product into the nonzero blocks of a topology.
//
// 128-blocks are computed two neighbours of a block row at a time: the eight wavefronts
// compute a 128x256 tile that stages the lhs row panel once.  When the fusion plan says
// that the next block row repeats this one, the workgroup also takes the two blocks
// below and computes a 256x256 tile (2x2 blocks): both lhs panels and both rhs panels
// are staged once for four blocks.  The plan lists the tiles in the order in which the
// workgroups take them.
// 64-blocks run one per workgroup with the K-tile split across four wavefronts.
#include "sdd_tile.h"

namespace stk {

// 128-blocks, eight wavefronts.  With a plan the workgroups take their tiles from its list: two
// neighbouring blocks of a block row (1x2 blocks, 128x256), together with the two blocks below when
// the next row repeats this one (2x2 blocks, 256x256), or one block with the two below it for the last
// three rows of a run of odd length (3x1 blocks, 384x128); rows covered that way get no workgroup, the
// grid is an upper bound and the surplus leaves at once.  Without a plan the blocks are taken two
// at a time in CSR order and every row is on its own.
template <class Quad, class Pair, class Triple, bool FULL>
__global__ __launch_bounds__(512, 2) void sdd_fused_kernel(SddArgs g) {
  extern __shared__ __align__(16) char smem[];
  sdd_fused_tile<Quad, Pair, Triple, FULL>(g, smem);
}

// 64-blocks with a plan: a tile of up to 4 x 4 blocks.  rows identical block rows starting at r0 (their
// blocks are nseg apart), cols neighbouring blocks starting at p0.  Cfg is 256x256 (4 x 4) or 128x256
// (2 x 4); rows and columns the tile does not have are computed on the first one's operands and dropped.
template <class Cfg, bool FULL>
__device__ __forceinline__ void sdd_tile64(const SddArgs& g, int r0, int p0, int rows, int cols, int nseg, char* smem) {
  static_assert(Cfg::PM == 64 && Cfg::PN == 64 && Cfg::B_PARTS == 4, "one operand part per block row / column");
  constexpr int KT = Cfg::KT;
  const elem_t* a0[Cfg::A_PARTS];
  const elem_t* b0[4];
#pragma unroll
  for (int i = 0; i < Cfg::A_PARTS; i++) a0[i] = g.lhs + (int64_t)(r0 + (i < rows ? i : 0)) * 64 * (Cfg::A_KMAJOR ? g.lda : 1);
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int c = uniform(load_index(g.column_indices, p0 + (j < cols ? j : 0), g.idx32));
    b0[j] = g.rhs + (int64_t)c * 64 * (Cfg::B_KMAJOR ? g.ldb : 1);
  }
  const int64_t a_step = Cfg::A_KMAJOR ? KT : KT * g.lda;
  const int64_t b_step = Cfg::B_KMAJOR ? KT : KT * g.ldb;
  const int k = g.k;
  const int ntiles = (k + KT - 1) / KT;
  f32x16_t acc[Cfg::IM][Cfg::JN] = {};
  auto tile_fn = [&](int t) {
    TilePtrs p;
#pragma unroll
    for (int i = 0; i < Cfg::A_PARTS; i++) p.a[i] = a0[i] + t * a_step;
#pragma unroll
    for (int j = 0; j < 4; j++) p.b[j] = b0[j] + t * b_step;
    const int left = k - t * KT;
    p.k_valid = left < KT ? left : KT;
    return p;
  };
  static_assert(FULL, "full K-tiles only");
  mainloop_dma<Cfg>(acc, ntiles, tile_fn, g.lda, g.ldb, smem);
  // the wavefront's sub-tile: one block row, one or two blocks wide
  const WaveCoords w = wave_coords<Cfg>();
  const int i = wave_m0<Cfg>(w) / 64, j = wave_n0<Cfg>(w) / 64;
  constexpr int kWide = Cfg::JN / 2;  // blocks per wavefront
  const bool have = i < rows && j < cols;
  const int block = have ? p0 + i * nseg + j : 0;
  const int n_valid = !have ? 0 : (cols - j < kWide ? cols - j : kWide) * 64;
  epilogue<Cfg, false>(acc, g.out + (int64_t)block * 4096, 64, have ? 64 : 0, n_valid, smem, 4096, g.activation,
                       g.multiplier ? g.multiplier + (int64_t)block * 4096 : nullptr, 0, 0, nullptr, nullptr, 0,
                       g.sums ? g.sums + (int64_t)block * 4096 : nullptr);
}

template <class Quad, class Pair>
__global__ __launch_bounds__(512, 2) void sdd_fused64_kernel(SddArgs g) {
  extern __shared__ __align__(16) char smem[];
  const int count = const_ints(g.tiles)[0];
  if ((int)blockIdx.x >= count) return;
  const int item = xcd_tile(blockIdx.x, count);
  const int p0 = const_ints(g.tiles)[2 + 2 * item], shape = const_ints(g.tiles)[3 + 2 * item];
  const int rows = shape & 0xff, cols = shape >> 8;
  const int r0 = uniform(load_index(g.row_indices, p0, g.idx32));
  const int nseg = const_ints(g.offsets)[r0 + 1] - const_ints(g.offsets)[r0];
  if (rows > 2) sdd_tile64<Quad, true>(g, r0, p0, rows, cols, nseg, smem);
  else sdd_tile64<Pair, true>(g, r0, p0, rows, cols, nseg, smem);
}

// One block per workgroup (four wavefronts).
template <class Cfg, int BLK, bool FULL>
__global__ __launch_bounds__(Cfg::kThreads, 2) void sdd_single_kernel(SddArgs g) {
  extern __shared__ __align__(16) char smem[];
  const int item = xcd_chunked(blockIdx.x, g.nnz);
  const int p = uniform(g.block_order ? g.block_order[item] : item);
  const int r = uniform(load_index(g.row_indices, p, g.idx32));
  const int c = uniform(load_index(g.column_indices, p, g.idx32));
  const int rr[3] = {r, r, r}, cc[2] = {c, c}, pp[3][2] = {{p, -1}, {-1, -1}, {-1, -1}};
  sdd_tile<Cfg, BLK, FULL>(g, rr, cc, pp, smem);
}

// 128-blocks with k a multiple of the K-tile depth KT: the direct-to-LDS pipeline with STAGES ring stages.
template <bool BF16, bool AK, bool BK, bool STREAM, int KT, int STAGES>
static void launch_sdd128(const SddArgs& g, hipStream_t stream) {
  // eight wavefronts: 4x2 of 64x128 over 2x2 blocks, or 2x4 of 64x64 over 1x2 blocks
  using Quad = TileCfg<4, 2, 2, 4, 1, 2, 2, AK, BK, BF16, KT, STAGES, false, STREAM>;
  using Pair = TileCfg<2, 4, 2, 2, 1, 1, 2, AK, BK, BF16, KT, STAGES, false, STREAM>;
  // 4x2 wavefronts of 96x64 over three block rows and one block column
  using Triple = TileCfg<4, 2, 3, 2, 1, 3, 1, AK, BK, BF16, KT, STAGES, false, STREAM>;
  // four wavefronts, one block: for launches with fewer blocks than the fused tiles need to fill the GPU
  using One = TileCfg<2, 2, 2, 2, 1, 1, 1, AK, BK, BF16, KT, STAGES, false, STREAM>;
  if (g.nnz <= compute_units()) {
    static const int once = (set_lds_limit(&sdd_single_kernel<One, 128, true>, One::kSmemBytes), 0);
    (void)once;
    hipLaunchKernelGGL((sdd_single_kernel<One, 128, true>), dim3(g.nnz), dim3(One::kThreads), One::kSmemBytes, stream, g);
    return;
  }
  constexpr int lds0 = Quad::kSmemBytes > Pair::kSmemBytes ? Quad::kSmemBytes : Pair::kSmemBytes;
  constexpr int lds = lds0 > Triple::kSmemBytes ? lds0 : Triple::kSmemBytes;
  static const int once = (set_lds_limit(&sdd_fused_kernel<Quad, Pair, Triple, true>, lds), 0);
  (void)once;
  // with a plan: at most one tile per two blocks of a row, rounded up per row
  // with a plan: one workgroup per compute unit (the tiles' LDS leaves room for one), which walks the list of tiles;
  // at most one tile per two blocks of a row, rounded up per row
  const int most = (int)sdd_max_tiles(g.block_rows, g.nnz), units = STK_SDD_PERSISTENT ? compute_units() : 0;
  const int grid = g.tiles ? (units > 0 && units < most ? units : most) : (g.nnz + 1) / 2;
  hipLaunchKernelGGL((sdd_fused_kernel<Quad, Pair, Triple, true>), dim3(grid), dim3(512), lds, stream, g);
}

// STREAM: every rhs column panel is read by few tiles and is loaded non-temporally.
template <bool BF16, int BLK, bool AK, bool BK, bool STREAM>
static void launch_sdd(const SddArgs& g, hipStream_t stream) {
  if constexpr (BLK == 128) {
    using Reg = TileCfg<2, 2, 2, 2, 1, 1, 1, AK, BK, BF16, 64, 2>;
    if (AK && BK && g.k % 64 == 0) {
      // both operands K-major: a 32-deep K-tile would use half of every 128-byte line it touches, so 64-deep
      // K-tiles (two stages fit) beat the deeper ring of 32-deep ones
      launch_sdd128<BF16, AK, BK, STREAM, 64, 2>(g, stream);
    } else if (g.k % STK_SDD_KT == 0) {
      launch_sdd128<BF16, AK, BK, STREAM, STK_SDD_KT, STK_SDD_STAGES>(g, stream);
    } else {
      // ragged k: one block per workgroup, predicated register staging
      hipLaunchKernelGGL((sdd_single_kernel<Reg, 128, false>), dim3(g.nnz), dim3(Reg::kThreads), Reg::kSmemBytes, stream, g);
    }
  } else {
    if (g.tiles && g.k % 64 == 0) {
      // eight wavefronts: 4x2 of 64x128 over 4x4 blocks, or 2x4 of 64x64 over 2x4 blocks
      using Quad = TileCfg<4, 2, 2, 4, 1, 4, 4, AK, BK, BF16, 64, 2, false, STREAM>;
      using Pair = TileCfg<2, 4, 2, 2, 1, 2, 4, AK, BK, BF16, 64, 2, false, STREAM>;
      constexpr int lds = Quad::kSmemBytes > Pair::kSmemBytes ? Quad::kSmemBytes : Pair::kSmemBytes;
      static const int once = (set_lds_limit(&sdd_fused64_kernel<Quad, Pair>, lds), 0);
      (void)once;
      hipLaunchKernelGGL((sdd_fused64_kernel<Quad, Pair>), dim3((int)sdd_max_tiles(g.block_rows, g.nnz)), dim3(512), lds, stream, g);
      return;
    }
    // the four wavefronts split each K-tile of 64
    using Dma = TileCfg<1, 1, 2, 2, 4, 1, 1, AK, BK, BF16, 64, 4, false, STREAM>;
    using Reg = TileCfg<1, 1, 2, 2, 4, 1, 1, AK, BK, BF16, 64, 2>;
    if (g.k % 64 == 0) hipLaunchKernelGGL((sdd_single_kernel<Dma, 64, true>), dim3(g.nnz), dim3(Dma::kThreads), Dma::kSmemBytes, stream, g);
    else hipLaunchKernelGGL((sdd_single_kernel<Reg, 64, false>), dim3(g.nnz), dim3(Reg::kThreads), Reg::kSmemBytes, stream, g);
  }
}

}  // namespace stk

extern "C" int stk_sdd(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                       const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                       int64_t m, int64_t k, int64_t n,
                       void* out, const int32_t* offsets, const void* row_indices, const void* column_indices,
                       const int32_t* block_order, int64_t nnz,
                       int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream) {
  return stk_sdd_fused(lhs, lhs_stride_m, lhs_stride_k, rhs, rhs_stride_k, rhs_stride_n, m, k, n, out, offsets, row_indices, column_indices,
                       block_order, nnz, blocking, dtype, index_dtype, plan, STK_ACT_NONE, nullptr, stream);
}

// Checks the arguments of an sdd and turns them into the kernels' view of the problem.  STK_OK with p->empty set
// when there is nothing to compute.
int stk::sdd_problem(const char* who, const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                     const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n, int64_t m, int64_t k, int64_t n,
                     void* out, const int32_t* offsets, const void* row_indices, const void* column_indices,
                     const int32_t* block_order, int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan,
                     int activation, const void* multiplier, SddProblem* p) {
  static_assert(STK_ACT_NONE == kNoActivation && STK_ACT_RELU == kRelu && STK_ACT_GELU_TANH == kGeluTanh && STK_ACT_GELU == kGeluErf &&
                    STK_ACT_SILU == kSilu && STK_ACT_RELU_GRAD == kReluGrad && STK_ACT_GELU_TANH_GRAD == kGeluTanhGrad &&
                    STK_ACT_GELU_GRAD == kGeluErfGrad && STK_ACT_SILU_GRAD == kSiluGrad, "the header's activation codes are the kernels'");
  p->empty = false;
  if (activation < 0 || activation >= kActivations) return fail(STK_ERR_UNSUPPORTED, "%s: activation %d", who, activation);
  if (multiplier && !aligned16(multiplier)) return fail(STK_ERR_UNSUPPORTED, "%s: multiplier needs a 16-byte aligned base", who);
  if (blocking != 64 && blocking != 128) return fail(STK_ERR_UNSUPPORTED, "%s: blocking %d (64 or 128)", who, blocking);
  if (dtype != STK_F16 && dtype != STK_BF16) return fail(STK_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "%s: index dtype %d", who, index_dtype);
  if (m < 0 || n < 0 || k < 0 || nnz < 0) return fail(STK_ERR_DIMS, "%s: negative size", who);
  if (m % blocking || n % blocking || k % 32)
    return fail(STK_ERR_DIMS, "incompatible dimensions: [%lld, %lld] x [%lld, %lld] with blocking %d (m, n must be divisible by the blocking, k by 32)",
                (long long)m, (long long)k, (long long)k, (long long)n, blocking);
  if (k > INT32_MAX || nnz > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "%s: size exceeds 32-bit range", who);
  if (nnz == 0) {
    p->empty = true;
    return STK_OK;
  }
  const bool ak = lhs_stride_k == 1;   // row-major lhs: K-major tile
  const bool bk = rhs_stride_n != 1;   // .t() view of a row-major [n, k]: K-major tile
  if (!ak && lhs_stride_m != 1) return fail(STK_ERR_UNSUPPORTED, "%s: lhs needs a unit stride", who);
  if (bk && rhs_stride_k != 1) return fail(STK_ERR_UNSUPPORTED, "%s: rhs needs a unit stride", who);
  const int64_t lda = ak ? lhs_stride_m : lhs_stride_k;
  const int64_t ldb = bk ? rhs_stride_n : rhs_stride_k;
  if (lda % 8 || ldb % 8 || !aligned16(lhs) || !aligned16(rhs) || !aligned16(out))
    return fail(STK_ERR_UNSUPPORTED, "%s: operands need 16-byte aligned bases and leading dimensions divisible by 8", who);
  if (lda >= (1 << 24) || ldb >= (1 << 24)) return fail(STK_ERR_UNSUPPORTED, "%s: leading dimension exceeds 2^24 elements", who);
  p->g = SddArgs{static_cast<const elem_t*>(lhs), lda, static_cast<const elem_t*>(rhs), ldb, (int)k,
                 static_cast<elem_t*>(out), offsets, row_indices, column_indices, block_order,
                 plan && offsets ? reinterpret_cast<const int32_t*>(plan) : nullptr, (int)nnz, (int)(m / blocking), index_dtype == STK_I32,
                 activation, static_cast<const elem_t*>(multiplier)};
  p->g.scalar_indices = index_dtype == STK_I32 || !((reinterpret_cast<uintptr_t>(row_indices) | reinterpret_cast<uintptr_t>(column_indices)) & 3u);
  p->ak = ak;
  p->bk = bk;
  // an rhs column panel is read once per tile that holds a block of that block column: with few
  // blocks per column (a block-diagonal MoE layout has one or two tiles per expert) it is streamed
  // (row-major rhs only: a K-major tile uses half a cache line per K-tile and needs the line to stay)
  p->stream_rhs = !bk && nnz <= 4 * (n / blocking);
  return STK_OK;
}

extern "C" int stk_sdd_fused(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                             const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                             int64_t m, int64_t k, int64_t n,
                             void* out, const int32_t* offsets, const void* row_indices, const void* column_indices,
                             const int32_t* block_order, int64_t nnz,
                             int blocking, int dtype, int index_dtype, const uint8_t* plan,
                             int activation, const void* multiplier, stk_stream_t stream) {
  return stk_sdd_fused_sums(lhs, lhs_stride_m, lhs_stride_k, rhs, rhs_stride_k, rhs_stride_n, m, k, n, out, offsets, row_indices, column_indices,
                            block_order, nnz, blocking, dtype, index_dtype, plan, activation, multiplier, nullptr, stream);
}

extern "C" int stk_sdd_fused_sums(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                                  const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                                  int64_t m, int64_t k, int64_t n,
                                  void* out, const int32_t* offsets, const void* row_indices, const void* column_indices,
                                  const int32_t* block_order, int64_t nnz,
                                  int blocking, int dtype, int index_dtype, const uint8_t* plan,
                                  int activation, const void* multiplier, void* sums, stk_stream_t stream) {
  using namespace stk;
  if (sums && (dtype == STK_F32 || !aligned16(sums) || sums == out))
    return fail(STK_ERR_UNSUPPORTED, "stk_sdd_fused_sums: the sums go to a 16-byte aligned array of their own, 16-bit values only");
  if (dtype == STK_F32)
    return sdd_f32(lhs, lhs_stride_m, lhs_stride_k, rhs, rhs_stride_k, rhs_stride_n, m, k, n, out, row_indices, column_indices, nnz, blocking,
                   index_dtype, activation, multiplier, static_cast<hipStream_t>(stream));
  SddProblem problem;
  const int rc = sdd_problem("stk_sdd", lhs, lhs_stride_m, lhs_stride_k, rhs, rhs_stride_k, rhs_stride_n, m, k, n, out, offsets, row_indices,
                             column_indices, block_order, nnz, blocking, dtype, index_dtype, plan, activation, multiplier, &problem);
  if (rc != STK_OK || problem.empty) return rc;
  problem.g.sums = static_cast<elem_t*>(sums);
  const SddArgs& g = problem.g;
  const bool ak = problem.ak, bk = problem.bk, stream_rhs = problem.stream_rhs;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define STK_SDD_CASE(BF, BLK, AK, BK)                                         \
  if ((dtype == STK_BF16) == BF && blocking == BLK && ak == AK && bk == BK) { \
    if (!BK && stream_rhs) launch_sdd<BF, BLK, AK, BK, !BK>(g, s);            \
    else launch_sdd<BF, BLK, AK, BK, false>(g, s);                            \
    return check_launch("stk_sdd");                                           \
  }
#define STK_SDD_LAYOUTS(BF, BLK) \
  STK_SDD_CASE(BF, BLK, true, true) STK_SDD_CASE(BF, BLK, true, false) STK_SDD_CASE(BF, BLK, false, true) STK_SDD_CASE(BF, BLK, false, false)
  STK_SDD_LAYOUTS(true, 128) STK_SDD_LAYOUTS(false, 128) STK_SDD_LAYOUTS(true, 64) STK_SDD_LAYOUTS(false, 64)
  return fail(STK_ERR_UNSUPPORTED, "stk_sdd: no kernel for this configuration");
}
