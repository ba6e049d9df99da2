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
  int scalar_walk; // the index arrays of the walk start at multiples of four bytes: the scalar unit can read them
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

// The walk of LINES block columns starting at `bj` as the K loop wants it: lane i of every wavefront holds the
// (k block, block id) pair of walk entry i, so that the K loop gets them with a lane read instead of a load.  Only the
// first `lines` of the LINES columns exist (identical patterns when LINES > 1); the others repeat the last one.
template <int LINES>
struct DdsWalk {
  int bj, nseg;
  int start[LINES];
  int seg_k;             // entries [0, kMaxSegments) of the walk
  int seg_block[LINES];
};

// Entries [s0, s0 + cnt) of the walk, one per lane, fetched with vector loads.
template <int LINES, bool TRANS_B>
__device__ __forceinline__ void dds_walk_entries(const DdsArgs& g, DdsWalk<LINES>& w, int s0, int cnt) {
  const int lane = threadIdx.x & 63;
  const int e = lane < cnt ? lane : cnt - 1;
  w.seg_k = load_index(g.walk_columns, w.start[0] + s0 + e, g.idx32);
#pragma unroll
  for (int l = 0; l < LINES; l++) w.seg_block[l] = TRANS_B ? w.start[l] + s0 + e : g.walk_blocks[w.start[l] + s0 + e];
}

template <int LINES, bool TRANS_B>
__device__ __forceinline__ DdsWalk<LINES> dds_walk(const DdsArgs& g, int bj, int lines) {
  DdsWalk<LINES> w;
  w.bj = bj;
#pragma unroll
  for (int l = 0; l < LINES; l++) w.start[l] = g.walk_offsets[bj + (l < lines ? l : lines - 1)];
  w.nseg = g.walk_offsets[bj + 1] - w.start[0];
  if (w.nseg > 0) dds_walk_entries<LINES, TRANS_B>(g, w, 0, w.nseg < kMaxSegments ? w.nseg : kMaxSegments);
  return w;
}

// The same through the scalar unit, for walks of at most kScalarWalk entries (the block columns of a mixture-of-experts
// topology hold as many blocks as their expert has block rows): three dependent scalar loads - offsets, then the
// entries - and lane selects, no vector memory access, so that a workgroup can look its next tile up while the
// transfers of the current one are in flight without touching their in-order completion count.  False (and w
// incomplete) when the walk is longer or the index arrays cannot be read as 32-bit words.
constexpr int kScalarWalk = 4;
template <int LINES, bool TRANS_B>
__device__ __forceinline__ bool dds_walk_scalar(const DdsArgs& g, int bj, int lines, DdsWalk<LINES>& w) {
  w.bj = bj;
#pragma unroll
  for (int l = 0; l < LINES; l++) w.start[l] = const_ints(g.walk_offsets)[bj + (l < lines ? l : lines - 1)];
  w.nseg = const_ints(g.walk_offsets)[bj + 1] - w.start[0];
  if (w.nseg > kScalarWalk || !g.scalar_walk) return false;
  w.seg_k = 0;
#pragma unroll
  for (int l = 0; l < LINES; l++) w.seg_block[l] = 0;
  if (w.nseg <= 0) return true;
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < kScalarWalk; i++) {
    const int e = i < w.nseg ? i : w.nseg - 1;
    const int k = scalar_index(g.walk_columns, w.start[0] + e, g.idx32);
    w.seg_k = (i == 0 || lane == i) ? k : w.seg_k;
#pragma unroll
    for (int l = 0; l < LINES; l++) {
      const int b = TRANS_B ? w.start[l] + e : const_ints(g.walk_blocks)[w.start[l] + e];
      w.seg_block[l] = (i == 0 || lane == i) ? b : w.seg_block[l];
    }
  }
  return true;
}

// The tile of the LINES block columns of walk `w`, output rows [m0, m0 + Cfg::TM).  after_prologue: see mainloop_dma
// (called once, inside the first main loop; not at all for a walk without entries).
template <class Cfg, int BLK, bool TRANS_B, bool FULL, int LINES, class Hook>
__device__ __forceinline__ void dds_tile_of(const DdsArgs& g, DdsWalk<LINES> w, int m0, char* smem, int lines, Hook&& after_prologue) {
  static_assert(Cfg::TN == LINES * BLK && Cfg::B_PARTS == LINES && Cfg::B_KMAJOR == TRANS_B, "one operand part per block column");
  constexpr int KT = Cfg::KT;
  constexpr int kTilesPerBlock = BLK / KT;
  const int nseg = w.nseg, bj = w.bj;
  const elem_t* a0 = g.lhs + (int64_t)m0 * (Cfg::A_KMAJOR ? g.lda : 1);
  const int64_t a_kstride = Cfg::A_KMAJOR ? 1 : g.lda;
  const int64_t a_part = (int64_t)Cfg::PM * (Cfg::A_KMAJOR ? g.lda : 1);
  const int m_valid = (g.m - m0 < Cfg::TM) ? g.m - m0 : Cfg::TM;
  f32x16_t acc[Cfg::IM][Cfg::JN] = {};
  for (int s0 = 0; s0 < nseg; s0 += kMaxSegments) {
    const int cnt = (nseg - s0 < kMaxSegments) ? nseg - s0 : kMaxSegments;
    if (s0 > 0) dds_walk_entries<LINES, TRANS_B>(g, w, s0, cnt);
    const int seg_k = w.seg_k;
    int seg_block[LINES];
#pragma unroll
    for (int l = 0; l < LINES; l++) seg_block[l] = w.seg_block[l];
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
    if constexpr (FULL) {
      mainloop_dma<Cfg>(acc, cnt * kTilesPerBlock, tile_fn, g.lda, BLK, smem, [&] {
        if (s0 == 0) after_prologue();
      });
    } else {
      mainloop_reg<Cfg>(acc, cnt * kTilesPerBlock, tile_fn, g.lda, BLK, m_valid, BLK, smem);
    }
  }
  const WaveCoords wc = wave_coords<Cfg>();
  const int wm0 = wave_m0<Cfg>(wc), wn0 = wave_n0<Cfg>(wc);
  epilogue<Cfg, STK_STREAM_STORES>(acc, g.out + (int64_t)(m0 + wm0) * g.ldc + (int64_t)bj * BLK + wn0, g.ldc, m_valid - wm0, lines * BLK - wn0, smem);
}

// LINES block columns starting at `bj` (identical patterns when LINES > 1), output
// rows [m0, m0 + Cfg::TM).  Only the first `lines` of the LINES columns exist; the others are
// computed on the last one's blocks and dropped.
template <class Cfg, int BLK, bool TRANS_B, bool FULL, int LINES>
__device__ __forceinline__ void dds_tile(const DdsArgs& g, int bj, int m0, char* smem, int lines = LINES) {
  dds_tile_of<Cfg, BLK, TRANS_B, FULL, LINES>(g, dds_walk<LINES, TRANS_B>(g, bj, lines), m0, smem, lines, [] {});
}

}  // namespace stk
