// stk_sdd_gather: the sampled product of a routed layer, x[rows of the padded layout] x rhs, straight from the token
// rows: what stk_padded_gather followed by stk_sdd_fused computes, without the padded copy of the tokens in between.
// The transfers of the lhs tiles take every row of the padded layout from the token row it is a copy of (a row
// offset per lane, computed once per tile); the rows that are padding are computed on the first token row and set to
// zero before the store, which is what the zero rows of a padded copy give.
#include "sdd_tile.h"

namespace stk {

template <class Quad, class Pair, class Triple>
__global__ __launch_bounds__(512, 2) void sdd_gather_fused_kernel(SddArgs g) {
  extern __shared__ __align__(16) char smem[];
  sdd_fused_tile<Quad, Pair, Triple, true, true>(g, smem);
}

// One block per workgroup (four wavefronts): launches with fewer blocks than the fused tiles need to fill the GPU.
template <class Cfg>
__global__ __launch_bounds__(Cfg::kThreads, 2) void sdd_gather_single_kernel(SddArgs g) {
  extern __shared__ __align__(16) char smem[];
  const int p = xcd_chunked(blockIdx.x, g.nnz);
  const int r = uniform(load_index(g.row_indices, p, g.idx32));
  const int c = uniform(load_index(g.column_indices, p, g.idx32));
  const int rr[3] = {r, r, r}, cc[2] = {c, c}, pp[3][2] = {{p, -1}, {-1, -1}, {-1, -1}};
  sdd_tile<Cfg, 128, true, true>(g, rr, cc, pp, smem);
}

// The tilings of stk_sdd on 128-blocks (row-major lhs), with gathered lhs rows.
template <bool BF16, bool BK, bool STREAM, int KT, int STAGES>
static void launch_gather128(const SddArgs& g, hipStream_t stream) {
  using Quad = TileCfg<4, 2, 2, 4, 1, 2, 2, true, BK, BF16, KT, STAGES, false, STREAM>;
  using Pair = TileCfg<2, 4, 2, 2, 1, 1, 2, true, BK, BF16, KT, STAGES, false, STREAM>;
  using Triple = TileCfg<4, 2, 3, 2, 1, 3, 1, true, BK, BF16, KT, STAGES, false, STREAM>;
  using One = TileCfg<2, 2, 2, 2, 1, 1, 1, true, BK, BF16, KT, STAGES, false, STREAM>;
  if (g.nnz <= compute_units()) {
    static const int once = (set_lds_limit(&sdd_gather_single_kernel<One>, One::kSmemBytes), 0);
    (void)once;
    hipLaunchKernelGGL((sdd_gather_single_kernel<One>), dim3(g.nnz), dim3(One::kThreads), One::kSmemBytes, stream, g);
    return;
  }
  constexpr int lds0 = Quad::kSmemBytes > Pair::kSmemBytes ? Quad::kSmemBytes : Pair::kSmemBytes;
  constexpr int lds = lds0 > Triple::kSmemBytes ? lds0 : Triple::kSmemBytes;
  static const int once = (set_lds_limit(&sdd_gather_fused_kernel<Quad, Pair, Triple>, lds), 0);
  (void)once;
  // with a plan: one workgroup per compute unit (the tiles' LDS leaves room for one), which walks the list of tiles;
  // at most one tile per two blocks of a row, rounded up per row
  const int most = (int)sdd_max_tiles(g.block_rows, g.nnz), units = STK_SDD_PERSISTENT ? compute_units() : 0;
  const int grid = g.tiles ? (units > 0 && units < most ? units : most) : (g.nnz + 1) / 2;
  hipLaunchKernelGGL((sdd_gather_fused_kernel<Quad, Pair, Triple>), dim3(grid), dim3(512), lds, stream, g);
}

template <bool BF16>
static void launch_gather(const SddArgs& g, bool bk, bool stream_rhs, hipStream_t stream) {
  if (bk) {
    // both operands K-major: 64-deep K-tiles when k allows (whole 128-byte lines), as in stk_sdd
    if (g.k % 64 == 0) launch_gather128<BF16, true, false, 64, 2>(g, stream);
    else launch_gather128<BF16, true, false, STK_SDD_KT, STK_SDD_STAGES>(g, stream);
  } else if (stream_rhs) {
    launch_gather128<BF16, false, true, STK_SDD_KT, STK_SDD_STAGES>(g, stream);
  } else {
    launch_gather128<BF16, false, false, STK_SDD_KT, STK_SDD_STAGES>(g, stream);
  }
}

}  // namespace stk

extern "C" int stk_sdd_gather(const void* tokens, int64_t num_tokens, int64_t token_stride, const int32_t* row_slots, int top_k,
                              const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n, int64_t m, int64_t k, int64_t n,
                              void* out, const int32_t* offsets, const void* row_indices, const void* column_indices, int64_t nnz,
                              int blocking, int dtype, int index_dtype, const uint8_t* plan, int activation, stk_stream_t stream) {
  using namespace stk;
  const char* who = "stk_sdd_gather";
  if (blocking != 128) return fail(STK_ERR_UNSUPPORTED, "%s: blocking %d (128 only)", who, blocking);
  if (dtype != STK_F16 && dtype != STK_BF16) return fail(STK_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
  if (top_k < 1 || num_tokens < 0) return fail(STK_ERR_DIMS, "%s: %lld tokens, top_k %d", who, (long long)num_tokens, top_k);
  if (activation > STK_ACT_SILU) return fail(STK_ERR_UNSUPPORTED, "%s: activation %d (a derivative does not map a row of zeros to zeros)", who, activation);
  if (nnz > 0 && (!row_slots || num_tokens == 0)) return fail(STK_ERR_DIMS, "%s: no tokens or no row_slots", who);
  // the transfers address a token row by a 32-bit byte offset from the first one
  if (num_tokens * token_stride * 2 >= (int64_t(1) << 32) || num_tokens * top_k > INT32_MAX)
    return fail(STK_ERR_UNSUPPORTED, "%s: the token rows span 4 GiB or more", who);
  SddProblem problem;
  const int rc = sdd_problem(who, tokens, token_stride, 1, rhs, rhs_stride_k, rhs_stride_n, m, k, n, out, offsets, row_indices, column_indices,
                             nullptr, nnz, blocking, dtype, index_dtype, plan, activation, nullptr, &problem);
  if (rc != STK_OK || problem.empty) return rc;
  SddArgs g = problem.g;
  g.row_slots = row_slots;
  g.top_k = top_k;
  g.slots = (int)(num_tokens * top_k);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == STK_BF16) launch_gather<true>(g, problem.bk, problem.stream_rhs, s);
  else launch_gather<false>(g, problem.bk, problem.stream_rhs, s);
  return check_launch(who);
}
