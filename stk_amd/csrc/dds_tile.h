// Tile function of stk_dds, shared by its kernels (dds.hip) and by the launch that computes a dsd and a dds on
// the same sparse operand together (grad.hip).
#pragma once
#include "common.h"
#include "gemm_core.h"

namespace stk {

struct DdsArgs {
  const elem_t* lhs;
  int64_t lda;
  const elem_t* data;
  const int32_t* walk_offsets;
  const void* walk_columns;
  const int32_t* walk_blocks;  // indirect block ids (non-transposed operand) or null
  elem_t* out;
  int64_t ldc;
  int m;
  int block_cols;
  int idx32;
  int small;       // little work per compute unit: four-wave tiles
};

// A checked dds: the kernels' arguments, the plan's lists of the walked lines (null without a plan), layout flags.
struct DdsProblem {
  DdsArgs g;
  PlanLists lists;
  bool ak, tb, stream_lhs, empty;
};
int dds_problem(const char* who, int64_t m, int64_t k, int64_t n,
                const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                const void* data, const int32_t* offsets, const void* column_indices,
                const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                int transpose_b, void* out, int64_t out_stride_m,
                int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, DdsProblem* p);

// LINES block columns starting at `bj` (identical patterns when LINES > 1), output
// rows [m0, m0 + Cfg::TM).  Only the first `lines` of the LINES columns exist; the others are
// computed on the last one's blocks and dropped.
template <class Cfg, int BLK, bool TRANS_B, bool FULL, int LINES>
__device__ __forceinline__ void dds_tile(const DdsArgs& g, int bj, int m0, char* smem, int lines = LINES) {
  static_assert(Cfg::TN == LINES * BLK && Cfg::B_PARTS == LINES && Cfg::B_KMAJOR == TRANS_B, "one operand part per block column");
  constexpr int KT = Cfg::KT;
  constexpr int kTilesPerBlock = BLK / KT;
  int start[LINES];
#pragma unroll
  for (int l = 0; l < LINES; l++) start[l] = g.walk_offsets[bj + (l < lines ? l : lines - 1)];
  const int nseg = g.walk_offsets[bj + 1] - start[0];
  const elem_t* a0 = g.lhs + (int64_t)m0 * (Cfg::A_KMAJOR ? g.lda : 1);
  const int64_t a_kstride = Cfg::A_KMAJOR ? 1 : g.lda;
  const int64_t a_part = (int64_t)Cfg::PM * (Cfg::A_KMAJOR ? g.lda : 1);
  const int m_valid = (g.m - m0 < Cfg::TM) ? g.m - m0 : Cfg::TM;
  const int lane = threadIdx.x & 63;
  f32x16_t acc[Cfg::IM][Cfg::JN] = {};
  for (int s0 = 0; s0 < nseg; s0 += kMaxSegments) {
    const int cnt = (nseg - s0 < kMaxSegments) ? nseg - s0 : kMaxSegments;
    // Lane i of every wavefront holds the (k block, block id) pair of walk entry s0 + i, so
    // that the K loop gets them with a lane read instead of a load.
    const int e = lane < cnt ? lane : cnt - 1;
    const int seg_k = load_index(g.walk_columns, start[0] + s0 + e, g.idx32);
    int seg_block[LINES];
#pragma unroll
    for (int l = 0; l < LINES; l++) seg_block[l] = TRANS_B ? start[l] + s0 + e : g.walk_blocks[start[l] + s0 + e];
    auto tile_fn = [&](int t) {
      const int seg = t / kTilesPerBlock, sub = t % kTilesPerBlock;
      const int64_t kb = __builtin_amdgcn_readlane(seg_k, seg);
      TilePtrs p;
      p.a[0] = a0 + (kb * BLK + sub * KT) * a_kstride;
      p.a[1] = p.a[0] + a_part;
#pragma unroll
      for (int l = 0; l < LINES; l++)
        p.b[l] = g.data + (int64_t)__builtin_amdgcn_readlane(seg_block[l], seg) * (BLK * BLK) + sub * KT * (TRANS_B ? 1 : BLK);
      p.k_valid = KT;
      return p;
    };
    if constexpr (FULL) mainloop_dma<Cfg>(acc, cnt * kTilesPerBlock, tile_fn, g.lda, BLK, smem);
    else mainloop_reg<Cfg>(acc, cnt * kTilesPerBlock, tile_fn, g.lda, BLK, m_valid, BLK, smem);
  }
  const WaveCoords w = wave_coords<Cfg>();
  const int wm0 = wave_m0<Cfg>(w), wn0 = wave_n0<Cfg>(w);
  epilogue<Cfg, STK_STREAM_STORES>(acc, g.out + (int64_t)(m0 + wm0) * g.ldc + (int64_t)bj * BLK + wn0, g.ldc, m_valid - wm0, lines * BLK - wn0, smem);
}

}  // namespace stk
