// Tile functions of stk_sdd, shared by its kernels (sdd.hip) and by the launch that computes an sdd and a dsd on
// the same topology together (grad.hip).
#pragma once
#include "common.h"
#include "gemm_core.h"

namespace stk {

struct SddArgs {
  const elem_t* lhs;
  int64_t lda;
  const elem_t* rhs;
  int64_t ldb;
  int k;
  elem_t* out;
  const int32_t* offsets;  // CSR row pointers (needed for fused block rows) or null
  const void* row_indices;
  const void* column_indices;
  const int32_t* block_order;
  const int32_t* tiles;  // fusion plan: count, unused, then (first block id, rows | columns << 8) per tile; or null
  int nnz;
  int block_rows;
  int idx32;
  int activation;            // applied to the fp32 sums (an Activation value)
  const elem_t* multiplier;  // values of a matrix with the same topology, multiplied in after the rounding; or null
  // gathered lhs rows (the GATHER kernels): row r of the lhs is row row_slots[r] / top_k of `lhs`, a row of zeros
  // where row_slots[r] is not in [0, slots)
  const int32_t* row_slots;
  int top_k;
  int slots;
  elem_t* sums;  // laid out like `out`: receives the rounded sums themselves (before activation and multiplier); or null
  int scalar_indices;  // row_indices and column_indices may be read through the scalar unit (see scalar_index())
};

// The row of SddArgs::lhs that row `r` of a gathered lhs is taken from; negative: a row of zeros.
__device__ __forceinline__ int gathered_row(const SddArgs& g, int r) {
  const int s = g.row_slots[r];
  return (s < 0 || s >= g.slots) ? -1 : s / g.top_k;
}

// A tile of Cfg::A_PARTS block rows x Cfg::B_PARTS block columns.  r[i] / c[j] are the
// block rows / columns, p[i][j] the output block ids (negative: not stored).
// GATHER: the rows of the lhs are gathered (SddArgs::row_slots); the transfers of the lhs tiles then take every row
// from where it lies, and rows of zeros are computed on the array's first row and set to zero afterwards.
// after_prologue: see mainloop_dma (direct-to-LDS pipeline only).
template <class Cfg, int BLK, bool FULL, bool GATHER = false, class Hook>
__device__ __forceinline__ void sdd_tile(const SddArgs& g, const int (&r)[3], const int (&c)[2], const int (&p)[3][2], char* smem,
                                         Hook&& after_prologue) {
  static_assert(Cfg::PM == BLK && Cfg::PN == BLK && Cfg::A_PARTS <= 3 && Cfg::B_PARTS <= 2, "one operand part per block row / column");
  static_assert(!GATHER || (FULL && Cfg::A_KMAJOR), "gathered rows: row-major lhs, direct-to-LDS pipeline");
  constexpr int KT = Cfg::KT;
  // K-major: ld is the stride between rows of the tile; MN-major: between k rows.
  const elem_t* a0[3];
  const elem_t* b0[2];
#pragma unroll
  for (int i = 0; i < 3; i++) a0[i] = GATHER ? g.lhs : g.lhs + (int64_t)r[i] * BLK * (Cfg::A_KMAJOR ? g.lda : 1);
#pragma unroll
  for (int j = 0; j < 2; j++) b0[j] = g.rhs + (int64_t)c[j] * BLK * (Cfg::B_KMAJOR ? g.ldb : 1);
  const int64_t a_step = Cfg::A_KMAJOR ? KT : KT * g.lda;
  const int64_t b_step = Cfg::B_KMAJOR ? KT : KT * g.ldb;
  const int k = g.k;
  const int ntiles = (k + KT - 1) / KT;
  f32x16_t acc[Cfg::IM][Cfg::JN] = {};
  auto tile_fn = [&](int t) {
    const int left = k - t * KT;
    return TilePtrs{{a0[0] + t * a_step, a0[1] + t * a_step, a0[2] + t * a_step}, {b0[0] + t * b_step, b0[1] + t * b_step}, left < KT ? left : KT};
  };
  if constexpr (GATHER) {
    mainloop_dma<Cfg>(acc, ntiles, tile_fn, g.lda, g.ldb, smem, after_prologue, [&](int q, int row) {
      const int from = gathered_row(g, r[q] * BLK + row);
      return from < 0 ? 0 : from;
    });
  } else if constexpr (FULL) {
    mainloop_dma<Cfg>(acc, ntiles, tile_fn, g.lda, g.ldb, smem, after_prologue);
  } else {
    mainloop_reg<Cfg>(acc, ntiles, tile_fn, g.lda, g.ldb, BLK, BLK, smem);
  }
  const WaveCoords w = wave_coords<Cfg>();
  const int m0 = wave_m0<Cfg>(w), n0 = wave_n0<Cfg>(w);
  if constexpr (GATHER) {
    // lane l holds row 32 i + l % 32 of the wavefront's sub-tile in acc[i][..]
#pragma unroll
    for (int i = 0; i < Cfg::IM; i++) {
      const int m = m0 + 32 * i + (w.lane & 31);
      const int part = m / BLK;
      const int br = part == 0 ? r[0] : (part == 1 ? r[1] : r[2]);
      if (gathered_row(g, br * BLK + m % BLK) < 0) {
#pragma unroll
        for (int j = 0; j < Cfg::JN; j++) acc[i][j] = f32x16_t{};
      }
    }
  }
  if constexpr (Cfg::A_PARTS == 3) {
    // Three stored blocks below each other, one block wide; a wavefront's 96 rows may lie in two of them.
    // Addressed as rows of the first block that run on, with the distance between the blocks added per block.
    const int64_t at = (int64_t)p[0][0] * BLK * BLK + (int64_t)m0 * BLK + n0;
    epilogue<Cfg, false>(acc, g.out + at, BLK, Cfg::TM - m0, BLK - n0, smem, 64, g.activation, g.multiplier ? g.multiplier + at : nullptr,
                         m0, (int64_t)(p[1][0] - p[0][0] - 1) * BLK * BLK, nullptr, nullptr, 0, g.sums ? g.sums + at : nullptr);
  } else {
    const int block = p[m0 / BLK][n0 / BLK];  // the output block this wavefront writes into
    const int64_t at = (int64_t)(block < 0 ? 0 : block) * BLK * BLK + (int64_t)(m0 % BLK) * BLK + (n0 % BLK);
    epilogue<Cfg, false>(acc, g.out + at, BLK, block < 0 ? 0 : BLK - (m0 % BLK), BLK - (n0 % BLK), smem, 64, g.activation,
                         g.multiplier ? g.multiplier + at : nullptr, 0, 0, nullptr, nullptr, 0, g.sums ? g.sums + at : nullptr);
  }
}

template <class Cfg, int BLK, bool FULL, bool GATHER = false>
__device__ __forceinline__ void sdd_tile(const SddArgs& g, const int (&r)[3], const int (&c)[2], const int (&p)[3][2], char* smem) {
  sdd_tile<Cfg, BLK, FULL, GATHER>(g, r, c, p, smem, [] {});
}

// A tile of the plan's list (128-blocks): its first block, its shape (rows | columns << 8), the block row and the
// number of blocks in it, and the block columns of its one or two blocks.
struct SddPlanTile {
  int p0, shape, r0, nseg, c0, c1;
};
// SCALAR: through the scalar unit only (SddArgs::scalar_indices must hold): nothing that counts as a vector memory
// operation, so that it can run while the transfers of a tile are in flight.
template <bool SCALAR>
__device__ __forceinline__ SddPlanTile sdd_plan_tile_of(const SddArgs& g, int item) {
  SddPlanTile t;
  t.p0 = const_ints(g.tiles)[2 + 2 * item], t.shape = const_ints(g.tiles)[3 + 2 * item];
  const bool has1 = (t.shape >> 8) == 2;
  if constexpr (SCALAR) {
    t.r0 = scalar_index(g.row_indices, t.p0, g.idx32);
    t.c0 = scalar_index(g.column_indices, t.p0, g.idx32);
    t.c1 = has1 ? scalar_index(g.column_indices, t.p0 + 1, g.idx32) : t.c0;
  } else {
    t.r0 = uniform(load_index(g.row_indices, t.p0, g.idx32));
    t.c0 = uniform(load_index(g.column_indices, t.p0, g.idx32));
    t.c1 = has1 ? uniform(load_index(g.column_indices, t.p0 + 1, g.idx32)) : t.c0;
  }
  t.nseg = const_ints(g.offsets)[t.r0 + 1] - const_ints(g.offsets)[t.r0];
  return t;
}

// The tile `item` of the plan's list (128-blocks): two neighbouring blocks of a block row (1x2 blocks, 128x256),
// together with the two blocks below when the next row repeats this one (2x2 blocks, 256x256), or one block with
// the two below it for the last three rows of a run of odd length (3x1 blocks, 384x128).
template <class Quad, class Pair, class Triple, bool FULL, bool GATHER = false, class Hook>
__device__ __forceinline__ void sdd_plan_tile(const SddArgs& g, const SddPlanTile& t, char* smem, Hook&& after_prologue) {
  const int p0 = t.p0, r0 = t.r0, nseg = t.nseg, c0 = t.c0, c1 = t.c1;
  const bool has1 = (t.shape >> 8) == 2;  // an odd row ends with a tile of one block
  const int rows = t.shape & 0xff;
  const int below = rows >= 2 ? p0 + nseg : -1;
  if (rows == 3) {
    // the last three rows of a run of identical rows: one block wide, so that the rhs panel is read once for the three
    const int rr[3] = {r0, r0 + 1, r0 + 2}, cc[2] = {c0, c0}, pp[3][2] = {{p0, -1}, {below, -1}, {below + nseg, -1}};
    sdd_tile<Triple, 128, FULL, GATHER>(g, rr, cc, pp, smem, after_prologue);
  } else if (below >= 0) {
    const int rr[3] = {r0, r0 + 1, r0}, cc[2] = {c0, c1}, pp[3][2] = {{p0, has1 ? p0 + 1 : -1}, {below, has1 ? below + 1 : -1}, {-1, -1}};
    sdd_tile<Quad, 128, FULL, GATHER>(g, rr, cc, pp, smem, after_prologue);
  } else {
    const int rr[3] = {r0, r0, r0}, cc[2] = {c0, c1}, pp[3][2] = {{p0, has1 ? p0 + 1 : -1}, {-1, -1}, {-1, -1}};
    sdd_tile<Pair, 128, FULL, GATHER>(g, rr, cc, pp, smem, after_prologue);
  }
}
template <class Quad, class Pair, class Triple, bool FULL, bool GATHER = false>
__device__ __forceinline__ void sdd_plan_tile(const SddArgs& g, int item, char* smem) {
  sdd_plan_tile<Quad, Pair, Triple, FULL, GATHER>(g, sdd_plan_tile_of<false>(g, item), smem, [] {});
}

// The tiles first, first + stride, ... of the plan's list, one after the other (a workgroup of a launch with fewer
// workgroups than tiles: one per compute unit).  With a stride that is a multiple of the number of compute dies,
// which take workgroup ids in turn, every tile stays on the die it would have run on as a workgroup of its own.
// While the first transfers of a tile are in flight, the next tile's entry of the list and its indices are looked
// up through the scalar unit.
template <class Quad, class Pair, class Triple, bool FULL, bool GATHER = false>
__device__ __forceinline__ void sdd_walk_plan(const SddArgs& g, int first, int stride, char* smem) {
  const int count = const_ints(g.tiles)[0];
  if (first >= count) return;
  SddPlanTile tile = sdd_plan_tile_of<false>(g, xcd_tile(first, count));
  for (int id = first; id < count; id += stride) {
    const int next_id = id + stride;
    SddPlanTile next = tile;
    bool looked_up = false;
    if constexpr (FULL) {
      sdd_plan_tile<Quad, Pair, Triple, FULL, GATHER>(g, tile, smem, [&] {
        if (next_id < count && g.scalar_indices) next = sdd_plan_tile_of<true>(g, xcd_tile(next_id, count)), looked_up = true;
      });
    } else {
      sdd_plan_tile<Quad, Pair, Triple, FULL, GATHER>(g, tile, smem, [] {});
    }
    if (next_id < count && !looked_up) next = sdd_plan_tile_of<false>(g, xcd_tile(next_id, count));
    tile = next;
    __syncthreads();  // the epilogue staging buffer is part of the next tile's first stage
  }
}

// What workgroup blockIdx.x of a launch over 128-blocks with eight wavefronts computes: its tiles of the plan's list
// (the launch has one workgroup per compute unit, or fewer tiles than that), or without a plan the blockIdx.x-th pair
// of blocks in CSR order (every row on its own).
template <class Quad, class Pair, class Triple, bool FULL, bool GATHER = false>
__device__ __forceinline__ void sdd_fused_tile(const SddArgs& g, char* smem) {
  if (g.tiles) {
    sdd_walk_plan<Quad, Pair, Triple, FULL, GATHER>(g, blockIdx.x, gridDim.x, smem);
    return;
  }
  const int npairs = (g.nnz + 1) >> 1;
  const int q = xcd_chunked(blockIdx.x, npairs);
  const int p0 = 2 * q;
  const bool has1 = p0 + 1 < g.nnz;
  const int r0 = uniform(load_index(g.row_indices, p0, g.idx32));
  const int r1 = has1 ? uniform(load_index(g.row_indices, p0 + 1, g.idx32)) : -1;
  const int c0 = uniform(load_index(g.column_indices, p0, g.idx32));
  const int c1 = has1 ? uniform(load_index(g.column_indices, p0 + 1, g.idx32)) : c0;
  if (r1 != r0) {
    // the two blocks lie in different rows (or the second does not exist): one at a time
#pragma unroll 1
    for (int i = 0; i < (has1 ? 2 : 1); i++) {
      const int r = i ? r1 : r0, c = i ? c1 : c0;
      const int rr[3] = {r, r, r}, cc[2] = {c, c}, pp[3][2] = {{p0 + i, -1}, {-1, -1}, {-1, -1}};
      sdd_tile<Pair, 128, FULL, GATHER>(g, rr, cc, pp, smem);
      __syncthreads();  // the epilogue staging buffer is part of the next pass's first stage
    }
    return;
  }
  const int rr[3] = {r0, r0, r0}, cc[2] = {c0, c1}, pp[3][2] = {{p0, p0 + 1}, {-1, -1}, {-1, -1}};
  sdd_tile<Pair, 128, FULL, GATHER>(g, rr, cc, pp, smem);
}

// A checked sdd: the kernels' arguments and the operands' layouts.
struct SddProblem {
  SddArgs g;
  bool ak, bk, stream_rhs, empty;
};
int sdd_problem(const char* who, const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n, int64_t m, int64_t k, int64_t n,
                void* out, const int32_t* offsets, const void* row_indices, const void* column_indices,
                const int32_t* block_order, int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan,
                int activation, const void* multiplier, SddProblem* p);

}  // namespace stk
