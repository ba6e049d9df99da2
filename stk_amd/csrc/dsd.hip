// stk_dsd: dense = op(sparse) x dense.
//
// A workgroup produces the output rows of one block row of op(sparse) - or of two
// or three neighbouring block rows with identical patterns, which then share every
// tile of the dense operand - for one tile of output columns.  It walks the nonzero blocks
// of the row (for a transposed sparse operand: the CSC column segment with
// indirect block ids).
#include "dsd_tile.h"

namespace stk {

// One block row per workgroup (four wavefronts).
template <class Cfg, int BLK, bool TRANS_A, bool FULL>
__global__ __launch_bounds__(Cfg::kThreads, 2) void dsd_kernel(DsdArgs g) {
  extern __shared__ __align__(16) char smem[];
  const int ntn = (g.n + Cfg::TN - 1) / Cfg::TN;
  const int item = xcd_grouped(blockIdx.x, g.block_rows * ntn);  // no plan, no hint about the lines: small groups
  dsd_tile<Cfg, BLK, TRANS_A, FULL, 1>(g, item / ntn, (item % ntn) * Cfg::TN, smem);
}

// Every block row on its own (four wavefronts), in the order of the plan's lists: the rows of the pairs, of the
// threes, then the lone rows longest first - for launches with little work per compute unit, where the order in
// which the tiles start decides how evenly the units are loaded.  When the plan says that the rows share little
// (a random pattern), every compute die takes a stripe of the dense operand's columns for all rows instead of all
// columns for some rows, and fetches that stripe once (xcd_lines).
template <class Cfg, int BLK, bool TRANS_A>
__global__ __launch_bounds__(Cfg::kThreads, 2) void dsd_lines_kernel(DsdArgs g, PlanLists plan) {
  extern __shared__ __align__(16) char smem[];
  const int ntn = (g.n + Cfg::TN - 1) / Cfg::TN;
  const int pairs = const_ints(plan.counts)[kTallPairs], triples = const_ints(plan.counts)[kTallTriples];
  const int tiles = (2 * pairs + 3 * triples + const_ints(plan.counts)[kTallSingles]) * ntn;
  if ((int)blockIdx.x >= tiles) return;
  const int item = xcd_lines(blockIdx.x, tiles, ntn, plan.stripe_from(true));
  int l = item / ntn, line;
  if (l < 2 * pairs) line = const_ints(plan.list(kTallPairs))[l >> 1] + (l & 1);
  else if ((l -= 2 * pairs) < 3 * triples) line = const_ints(plan.list(kTallTriples))[l / 3] + l % 3;
  else line = const_ints(plan.list(kTallSingles))[l - 3 * triples];
  dsd_tile<Cfg, BLK, TRANS_A, true, 1>(g, line, (item % ntn) * Cfg::TN, smem);
}

// The lone block rows of a plan's list, one per workgroup (four wavefronts): what dsd_fused64_kernel leaves.
template <class Cfg, int BLK, bool TRANS_A, bool FULL>
__global__ __launch_bounds__(Cfg::kThreads, 2) void dsd_singles_kernel(DsdArgs g, PlanLists plan) {
  extern __shared__ __align__(16) char smem[];
  const int ntn = (g.n + Cfg::TN - 1) / Cfg::TN;
  const int tiles = const_ints(plan.counts)[kTallSingles] * ntn;
  if ((int)blockIdx.x >= tiles) return;
  const int item = xcd_grouped(blockIdx.x, tiles);
  dsd_tile<Cfg, BLK, TRANS_A, FULL, 1>(g, const_ints(plan.list(kTallSingles))[item / ntn], (item % ntn) * Cfg::TN, smem);
}

// 64-blocks with a plan built for them, eight wavefronts: groups of four identical block rows as 256x256
// tiles, groups of three as 192x256 tiles, pairs as 128x256 tiles; the dense
// operand is then read once per 256 or 128 rows instead of once per 64.  Lone rows are left to
// dsd_singles_kernel.  The grid is an upper bound; the surplus leaves at once.
template <class Quad, class Pair, class Three, bool TRANS_A>
__global__ __launch_bounds__(512, 2) void dsd_fused64_kernel(DsdArgs g, PlanLists plan) {
  extern __shared__ __align__(16) char smem[];
  static_assert(Quad::TN == Pair::TN && Quad::TN == Three::TN, "same column tiling");
  const int ntn = g.n / Quad::TN;
  const int quad_tiles = const_ints(plan.counts)[kPairs] * ntn, triple_tiles = const_ints(plan.counts)[kTallTriples] * ntn;
  const int pair_tiles = const_ints(plan.counts)[kTallPairs] * ntn;
  int bid = blockIdx.x;
  // pairs first: they hold the lines that were too long for groups of four, the longest tiles of the launch
  if (bid < pair_tiles) {
    const int item = xcd_item(bid, pair_tiles, ntn, plan.group(kTallPairs));
    dsd_tile<Pair, 64, TRANS_A, true, 2>(g, const_ints(plan.list(kTallPairs))[item / ntn], (item % ntn) * Pair::TN, smem, 2);
    return;
  }
  bid -= pair_tiles;
  if (bid < quad_tiles) {
    const int item = xcd_item(bid, quad_tiles, ntn, plan.group(kPairs));
    dsd_tile<Quad, 64, TRANS_A, true, 4>(g, const_ints(plan.list(kPairs))[item / ntn], (item % ntn) * Quad::TN, smem, 4);
    return;
  }
  bid -= quad_tiles;
  if (bid < triple_tiles) {
    const int item = xcd_item(bid, triple_tiles, ntn, plan.group(kTallTriples));
    dsd_tile<Three, 64, TRANS_A, true, 3>(g, const_ints(plan.list(kTallTriples))[item / ntn], (item % ntn) * Three::TN, smem);
  }
}

// 128-blocks, eight wavefronts.  The workgroups take their tiles from the lists of the plan (dsd_plan_tile).
// Covered rows get no workgroup; the grid is an upper bound and the surplus leaves at once.
// Without a plan every row is a lone row.
// SCATTER: the rows of the result are scattered (DsdArgs::row_map).
template <class Fused, class Triple, class Single, bool TRANS_A, bool SCATTER = false>
__global__ __launch_bounds__(512, 2) void dsd_fused_kernel(DsdArgs g, PlanLists plan) {
  extern __shared__ __align__(16) char smem[];
  int bid = blockIdx.x;
  if (!plan.counts) {
    const int ntn = g.n / Fused::TN;
    const int item = xcd_grouped(bid, g.block_rows * ntn);
    dsd_tile<Single, 128, TRANS_A, true, 1, SCATTER>(g, item / ntn, (item % ntn) * Single::TN, smem);
    return;
  }
  dsd_plan_tile<Fused, Triple, Single, TRANS_A, SCATTER>(g, plan, bid, smem);
}

// ---------------------------------------------------------------------------
// Variant for launches whose tiles fill the compute units a few times only.  The workgroups
// of the whole rounds take whole tiles as above; the tiles left for the last round are cut
// into `slices` slices along k (the plan says how many; 1: not at all), one workgroup each,
// so that the round fills the machine.  Whoever finishes a slice puts the fp32 partial tile
// in its slot of the workspace and counts itself on the tile's counter; the one that
// arrives last adds the partial tiles in the order of the slices and writes the result (it
// leaves the counter at zero for the next launch).  Nobody waits for anybody.  A workgroup
// that can see that it is the last skips the store of its own partial tile.
// ---------------------------------------------------------------------------
struct TailArgs {
  int32_t* counters;  // one per tile of the last round; zero between launches
  float* slots;       // `slices` per tile of the last round, kSlotFloats each
  int workgroups;     // workgroups per round: the compute units
  int capacity;       // slots the workspace holds; the last round is cut no further than fits
};
constexpr int kSlotFloats = 512 * 128;  // 512 threads x up to 8 accumulators of 16 values
constexpr int kTailBlock = 32;          // tiles whose slices are interleaved: 4 neighbours on each of the 8 compute dies

// acc = ((slice 0 + slice 1) + ...) over SLICES partial tiles, where slice ME is in acc and the others are in
// consecutive slots starting at `first` (already offset by the thread).  One accumulator at a time, the loads of
// all the other slices in flight together.
template <class Cfg, int SLICES, int ME>
__device__ __forceinline__ void add_slices_in_order(f32x16_t (&acc)[Cfg::IM][Cfg::JN], const float* first) {
  static_assert(kMaxTailSlices == 4 && SLICES <= kMaxTailSlices && ME < SLICES, "slices");
#pragma unroll
  for (int a = 0; a < Cfg::IM * Cfg::JN; a++) {
    float v[SLICES][16];
#pragma unroll
    for (int sl = 0; sl < SLICES; sl++) {
      if (sl == ME) continue;
#pragma unroll
      for (int r = 0; r < 16; r++)
        v[sl][r] = __hip_atomic_load(first + (int64_t)sl * kSlotFloats + (a * 16 + r) * 512, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    f32x16_t& mine = acc[a / Cfg::JN][a % Cfg::JN];
#pragma unroll
    for (int r = 0; r < 16; r++) {
      float sum = ME == 0 ? mine[r] : v[0][r];
#pragma unroll
      for (int sl = 1; sl < SLICES; sl++) sum += sl == ME ? mine[r] : v[sl][r];
      mine[r] = sum;
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// Slice `slice` of `slices` of the tile (LINES block rows from bi, columns from n0), the `ordinal`-th tile of the last
// round; the tile owns the slots [ordinal * slices, (ordinal + 1) * slices) of the workspace.
template <class Cfg, bool TRANS_A, int LINES, bool SCATTER = false>
__device__ __forceinline__ void dsd_slice(const DsdArgs& g, const TailArgs& t, int bi, int n0, int slice, int slices, int ordinal, char* smem, int* flag) {
  constexpr int kAcc = Cfg::IM * Cfg::JN;
  static_assert(kAcc * 16 * 512 <= kSlotFloats, "slot too small");
  const int nseg = g.walk_offsets[bi + 1] - g.walk_offsets[bi];
  const int64_t first_slot = (int64_t)ordinal * slices;
  if (slices > nseg) slices = nseg > 1 ? nseg : 1;
  if (slice >= slices) return;
  const int e0 = slice * nseg / slices, e1 = (slice + 1) * nseg / slices;
  const int tid = threadIdx.x;
  f32x16_t acc[Cfg::IM][Cfg::JN] = {};
  dsd_accumulate<Cfg, 128, TRANS_A, true, LINES>(acc, g, bi, n0, e0, e1, smem);
  if (slices == 1) {
    dsd_store<Cfg, 128, SCATTER>(acc, g, bi, n0, smem);
    return;
  }
  // Partial tiles and the counter are read and written with device-scope atomic accesses only: these
  // go to memory past the L2 of the compute die (which is not coherent with the other dies' L2),
  // without the whole-cache write-back and invalidate that device-scope fences would cost.  A slot
  // holds value r of accumulator a of thread t at (16 a + r) * 512 + t.
  const int others = slices - 1;
  int32_t* counter = t.counters + ordinal;
  auto slot_of = [&](int sl) { return t.slots + (first_slot + sl) * kSlotFloats + tid; };
  if (tid == 0) *flag = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  int arrived = uniform(*flag);
  if (arrived != others) {
    float* mine = slot_of(slice);
#pragma unroll
    for (int a = 0; a < kAcc; a++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        __hip_atomic_store(mine + (a * 16 + r) * 512, acc[a / Cfg::JN][a % Cfg::JN][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    wait_vmcnt<0>();  // the stores have reached memory ...
    __syncthreads();  // ... those of every wavefront, before the workgroup counts itself (and *flag has been read)
    if (tid == 0) *flag = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    arrived = uniform(*flag);
  }
  if (arrived != others) return;
  // Last to arrive: the counter said so after every other slice's stores had reached memory.
  if (others == 1) {
    // two slices: a + b in either order.  Four accumulators (64 loads per thread) at a time: all
    // loads in flight at once would not fit the register file next to the accumulators.
    const float* theirs = slot_of(1 - slice);
    constexpr int kBatch = kAcc % 4 == 0 ? 4 : 3;
    static_assert(kAcc % kBatch == 0, "whole batches");
#pragma unroll
    for (int a0 = 0; a0 < kAcc; a0 += kBatch) {
      float v[kBatch][16];
#pragma unroll
      for (int a = 0; a < kBatch; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) v[a][r] = __hip_atomic_load(theirs + ((a0 + a) * 16 + r) * 512, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int a = 0; a < kBatch; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[(a0 + a) / Cfg::JN][(a0 + a) % Cfg::JN][r] += v[a][r];
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
    // more: always in the order of the slices, whoever does the adding
    const float* first = slot_of(0);
    switch (slices * kMaxTailSlices + slice) {
      case 3 * kMaxTailSlices + 0: add_slices_in_order<Cfg, 3, 0>(acc, first); break;
      case 3 * kMaxTailSlices + 1: add_slices_in_order<Cfg, 3, 1>(acc, first); break;
      case 3 * kMaxTailSlices + 2: add_slices_in_order<Cfg, 3, 2>(acc, first); break;
      case 4 * kMaxTailSlices + 0: add_slices_in_order<Cfg, 4, 0>(acc, first); break;
      case 4 * kMaxTailSlices + 1: add_slices_in_order<Cfg, 4, 1>(acc, first); break;
      case 4 * kMaxTailSlices + 2: add_slices_in_order<Cfg, 4, 2>(acc, first); break;
      default: add_slices_in_order<Cfg, 4, 3>(acc, first); break;
    }
  }
  dsd_store<Cfg, 128, SCATTER>(acc, g, bi, n0, smem);
  if (tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <class Fused, class Triple, class Single, bool TRANS_A, bool SCATTER = false>
__global__ __launch_bounds__(512, 2) void dsd_sliced_kernel(DsdArgs g, PlanLists plan, TailArgs t) {
  extern __shared__ __align__(16) char smem[];
  __shared__ int flag;
  static_assert(Fused::TN == Single::TN && Fused::TN == 2 * Triple::TN, "same column tiling");
  const int ntn = g.n / Fused::TN;
  const int pair_tiles = const_ints(plan.counts)[kTallPairs] * ntn;
  const int triple_tiles = const_ints(plan.counts)[kTallTriples] * 2 * ntn;
  const int single_tiles = const_ints(plan.counts)[kTallSingles] * ntn;
  const int tiles = pair_tiles + triple_tiles + single_tiles;
  int slices = uniform(plan.hints[(ntn < kTailSliceColumns ? ntn : kTailSliceColumns) - 1]);
  const bool spread = (const_ints(plan.hints)[kSpreadHint / 4] & 0xff) != 0;
  if (slices < 1 || slices > kMaxTailSlices) slices = 1;
  // whole rounds first; the rest (all of it when there is less than one round) is the last round
  int whole = (slices > 1 && tiles > 0) ? (tiles - 1) / t.workgroups * t.workgroups : tiles;
  if (slices > 1 && (tiles - whole) * slices > t.capacity) {
    // a workspace smaller than the plan would like: fewer slices, or none
    slices = t.capacity / (tiles - whole);
    if (slices < 2) slices = 1, whole = tiles;
  }
  int item = blockIdx.x, slice = 0;
  if (item >= whole) {
    // last round: blocks of kTailBlock tiles, slice by slice, so that neighbouring tiles (which share
    // the sparse operand in the L2 of their compute die) work on the same stretch of k at the same time
    const int j = item - whole, r = j % (kTailBlock * slices);
    slice = r / kTailBlock;
    item = whole + j / (kTailBlock * slices) * kTailBlock + r % kTailBlock;
    if (item >= tiles) return;
  } else {
    slices = 1;
  }
  const int ordinal = item - whole;  // among the tiles of the last round: 0 .. workgroups - 1
  if (item < pair_tiles) {
    const int i = xcd_share(item, pair_tiles, spread);
    dsd_slice<Fused, TRANS_A, 2, SCATTER>(g, t, const_ints(plan.list(kTallPairs))[i / ntn], (i % ntn) * Fused::TN, slice, slices, ordinal, smem, &flag);
    return;
  }
  item -= pair_tiles;
  if (item < triple_tiles) {
    const int i = xcd_share(item, triple_tiles, spread);
    dsd_slice<Triple, TRANS_A, 3, SCATTER>(g, t, const_ints(plan.list(kTallTriples))[i / (2 * ntn)], (i % (2 * ntn)) * Triple::TN, slice, slices, ordinal, smem, &flag);
    return;
  }
  item -= triple_tiles;
  // (in order of length: no contiguous shares.)  When the plan says that the lone lines share little, the lines whose tiles all
  // lie in the whole rounds, where a workgroup's id is its item, are dealt by stripes of the dense operand (xcd_lines; the
  // list must start at a multiple of the eight dies, so that every line's tiles stay among themselves); what is left
  // of the list is taken in order.
  const int from = (plan.stripe_from(true) + 1) >> 1, lead = pair_tiles + triple_tiles;
  int i;
  if (from != 0 && ntn >= from && !(ntn & 7) && !(lead & 7)) {
    const int striped = whole > lead ? (whole - lead) / ntn * ntn : 0;
    i = item < striped ? xcd_lines(item, striped, ntn, from) : item;
  } else {
    i = xcd_grouped(item, single_tiles);
  }
  dsd_slice<Single, TRANS_A, 1, SCATTER>(g, t, const_ints(plan.list(kTallSingles))[i / ntn], (i % ntn) * Single::TN, slice, slices, ordinal, smem, &flag);
}

template <class Cfg, int BLK, bool TRANS_A, bool FULL>
static void launch_one(const DsdArgs& g, hipStream_t stream) {
  static const int once = (set_lds_limit(&dsd_kernel<Cfg, BLK, TRANS_A, FULL>, Cfg::kSmemBytes), 0);
  (void)once;
  const int ntn = (g.n + Cfg::TN - 1) / Cfg::TN;
  hipLaunchKernelGGL((dsd_kernel<Cfg, BLK, TRANS_A, FULL>), dim3(g.block_rows * ntn), dim3(Cfg::kThreads), Cfg::kSmemBytes, stream, g);
}

// Workspace of a launch with a sliced last round: counters, then the slots.
static size_t tail_counter_bytes(int workgroups) { return static_cast<size_t>((workgroups * 4 + 255) / 256 * 256); }
static size_t tail_workspace_bytes(int workgroups) {
  return tail_counter_bytes(workgroups) + sizeof(float) * kSlotFloats * kMaxTailSlices * static_cast<size_t>(workgroups);
}

// STREAM: every rhs row panel is read by few tiles and is loaded non-temporally.
template <bool BF16, int BLK, bool TRANS_A, bool BK, bool STREAM>
static void launch_dsd(const DsdArgs& g, const PlanLists& plan, const TailArgs* tail, hipStream_t stream) {
  // K-major dense operand (a .t() view): a 32-deep K-tile would use half of every 128-byte line it touches, so
  // 64-deep K-tiles (two stages fit) beat the deeper ring of 32-deep ones
  constexpr int KT = BK ? STK_DSD_BK_KT : (TRANS_A ? STK_DSD_T_KT : STK_DSD_KT), S = BK ? STK_DSD_BK_STAGES : (TRANS_A ? STK_DSD_T_STAGES : STK_DSD_STAGES);
  if constexpr (BLK == 128) {
    // eight wavefronts: 4x2 of 64x128 over two block rows, or 2x4 of 64x64 over one
    using Fused = TileCfg<4, 2, 2, 4, 1, 2, 2, !TRANS_A, BK, BF16, KT, S, false, STREAM>;
    using Single = TileCfg<2, 4, 2, 2, 1, 1, 2, !TRANS_A, BK, BF16, KT, S, false, STREAM>;
    // four wavefronts, 128x128, for column counts that are not a multiple of 256
    // (a K-major operand - sparse blocks that are not transposed, or a .t() view as rhs - in 64-deep K-tiles, whose rows are
    // whole 128-byte lines: on these small tiles that outweighs the deeper ring, config 2 dsd 42.5 -> 38.5 us)
    constexpr int NKT = (!TRANS_A || BK) ? 64 : KT, NS = (!TRANS_A || BK) ? 2 : S;
    using Narrow = TileCfg<2, 2, 2, 2, 1, 1, 1, !TRANS_A, BK, BF16, NKT, NS, false, STREAM>;
    using Reg = TileCfg<2, 2, 2, 2, 1, 1, 1, !TRANS_A, BK, BF16, 64, 2>;
    // 4x2 wavefronts of 96x64 over three block rows and 128 columns
    using Triple = TileCfg<4, 2, 3, 2, 1, 3, 1, !TRANS_A, BK, BF16, KT, S, false, STREAM>;
    if (g.n % Fused::TN == 0 && !g.small) {
      constexpr int lds0 = Fused::kSmemBytes > Single::kSmemBytes ? Fused::kSmemBytes : Single::kSmemBytes;
      constexpr int lds = lds0 > Triple::kSmemBytes ? lds0 : Triple::kSmemBytes;
      if (tail) {
        static const int once = (set_lds_limit(&dsd_sliced_kernel<Fused, Triple, Single, TRANS_A>, lds), 0);
        (void)once;
        // upper bound: every line a tile of its own, plus the slices of a full last round (rounded up to whole blocks)
        const int grid = g.block_rows * (g.n / Fused::TN) + kMaxTailSlices * (tail->workgroups + kTailBlock);
        hipLaunchKernelGGL((dsd_sliced_kernel<Fused, Triple, Single, TRANS_A>), dim3(grid), dim3(512), lds, stream, g, plan, *tail);
        return;
      }
      static const int once = (set_lds_limit(&dsd_fused_kernel<Fused, Triple, Single, TRANS_A>, lds), 0);
      (void)once;
      hipLaunchKernelGGL((dsd_fused_kernel<Fused, Triple, Single, TRANS_A>), dim3(g.block_rows * (g.n / Fused::TN)), dim3(512), lds, stream, g, plan);
    } else if (g.n % Narrow::TN == 0 && plan.counts) {
      static const int once = (set_lds_limit(&dsd_lines_kernel<Narrow, BLK, TRANS_A>, Narrow::kSmemBytes), 0);
      (void)once;
      hipLaunchKernelGGL((dsd_lines_kernel<Narrow, BLK, TRANS_A>), dim3(g.block_rows * (g.n / Narrow::TN)), dim3(Narrow::kThreads),
                         Narrow::kSmemBytes, stream, g, plan);
    } else if (g.n % Narrow::TN == 0) {
      launch_one<Narrow, BLK, TRANS_A, true>(g, stream);
    } else {
      launch_one<Reg, BLK, TRANS_A, false>(g, stream);  // ragged n: predicated register staging
    }
  } else {
    // 64-blocks: 1x4 wavefronts of 64x64 (tile 64x256)
    using Dma = TileCfg<1, 4, 2, 2, 1, 1, 1, !TRANS_A, BK, BF16, 64, 2, false, STREAM>;
    if (plan.counts && g.n % 256 == 0 && !g.small) {
      // groups of identical block rows on eight wavefronts (4x2 of 64x128 over four block rows, 2x4 of 64x64 over
      // two), then the lone rows one per four-wave workgroup; both grids are upper bounds
      using Quad = TileCfg<4, 2, 2, 4, 1, 4, 2, !TRANS_A, BK, BF16, 64, 2, false, STREAM>;
      using Pair = TileCfg<2, 4, 2, 2, 1, 2, 2, !TRANS_A, BK, BF16, 64, 2, false, STREAM>;
      // 2x4 wavefronts of 96x64 over three block rows: a group of three on a tile of its own size
      using Three = TileCfg<2, 4, 3, 2, 1, 3, 2, !TRANS_A, BK, BF16, 64, 2, false, STREAM>;
      constexpr int lds = Quad::kSmemBytes > Pair::kSmemBytes ? Quad::kSmemBytes : Pair::kSmemBytes;
      static_assert(Three::kSmemBytes <= lds, "the tile of three block rows fits where the tile of four does");
      static const int once = (set_lds_limit(&dsd_fused64_kernel<Quad, Pair, Three, TRANS_A>, lds), set_lds_limit(&dsd_singles_kernel<Dma, 64, TRANS_A, true>, Dma::kSmemBytes), 0);
      (void)once;
      const int ntn = g.n / 256;
      hipLaunchKernelGGL((dsd_fused64_kernel<Quad, Pair, Three, TRANS_A>), dim3((g.block_rows + 1) / 2 * ntn), dim3(512), lds, stream, g, plan);
      hipLaunchKernelGGL((dsd_singles_kernel<Dma, 64, TRANS_A, true>), dim3(g.block_rows * ntn), dim3(Dma::kThreads), Dma::kSmemBytes, stream, g, plan);
      return;
    }
    if (g.n % Dma::TN == 0) launch_one<Dma, BLK, TRANS_A, true>(g, stream);
    else launch_one<Dma, BLK, TRANS_A, false>(g, stream);
  }
}

// stk_dsd_scatter: the launches of a dsd on 128-blocks with eight wavefronts (sparse operand not transposed), with
// the rows of the result scattered.
template <bool BF16, bool BK, bool STREAM>
static void launch_dsd_scatter(const DsdArgs& g, const PlanLists& plan, const TailArgs* tail, hipStream_t stream) {
  constexpr int KT = BK ? STK_DSD_BK_KT : STK_DSD_KT, S = BK ? STK_DSD_BK_STAGES : STK_DSD_STAGES;
  using Fused = TileCfg<4, 2, 2, 4, 1, 2, 2, true, BK, BF16, KT, S, false, STREAM>;
  using Single = TileCfg<2, 4, 2, 2, 1, 1, 2, true, BK, BF16, KT, S, false, STREAM>;
  using Triple = TileCfg<4, 2, 3, 2, 1, 3, 1, true, BK, BF16, KT, S, false, STREAM>;
  constexpr int lds0 = Fused::kSmemBytes > Single::kSmemBytes ? Fused::kSmemBytes : Single::kSmemBytes;
  constexpr int lds = lds0 > Triple::kSmemBytes ? lds0 : Triple::kSmemBytes;
  if (tail) {
    static const int once = (set_lds_limit(&dsd_sliced_kernel<Fused, Triple, Single, false, true>, lds), 0);
    (void)once;
    const int grid = g.block_rows * (g.n / Fused::TN) + kMaxTailSlices * (tail->workgroups + kTailBlock);
    hipLaunchKernelGGL((dsd_sliced_kernel<Fused, Triple, Single, false, true>), dim3(grid), dim3(512), lds, stream, g, plan, *tail);
    return;
  }
  static const int once = (set_lds_limit(&dsd_fused_kernel<Fused, Triple, Single, false, true>, lds), 0);
  (void)once;
  hipLaunchKernelGGL((dsd_fused_kernel<Fused, Triple, Single, false, true>), dim3(g.block_rows * (g.n / Fused::TN)), dim3(512), lds, stream, g, plan);
}

// The sliced last round of a dsd launch, if this one gets one: for launches of a few rounds of tiles (with many
// rounds the last one matters little and the plain kernel is used as it is); the plan says whether and how the last
// round is cut.  STK_OK with *sliced set or cleared.
static int tail_of(const char* who, const DsdArgs& g, int64_t n, int64_t nnz, int blocking, const uint8_t* plan, void* workspace,
                   int64_t workspace_bytes, TailArgs* tail, bool* sliced) {
  *sliced = false;
  if (!(workspace && plan && blocking == 128 && n % 256 == 0 && nnz > 0 && !g.small)) return STK_OK;
  const int workgroups = compute_units();
  if (workgroups <= 0 || (int64_t)g.block_rows * (n / 128) / 3 >= 8 * (int64_t)workgroups) return STK_OK;
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(STK_ERR_WORKSPACE, "%s: the workspace must be 256-byte aligned", who);
  const int64_t capacity = (workspace_bytes - (int64_t)tail_counter_bytes(workgroups)) / (int64_t)(sizeof(float) * kSlotFloats);
  if (capacity < 2) return STK_OK;
  *sliced = true;
  tail->counters = static_cast<int32_t*>(workspace);
  tail->slots = reinterpret_cast<float*>(static_cast<char*>(workspace) + tail_counter_bytes(workgroups));
  tail->workgroups = workgroups;
  tail->capacity = (int)(capacity < kMaxTailSlices * (int64_t)workgroups ? capacity : kMaxTailSlices * (int64_t)workgroups);
  return STK_OK;
}

}  // namespace stk

// Checks the arguments of a dsd and turns them into the kernels' view of the problem.  STK_OK with p->empty set when
// there is nothing to compute.
int stk::dsd_problem(const char* who, int64_t m, int64_t k, int64_t n,
                     const void* data, const int32_t* offsets, const void* column_indices,
                     const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                     int transpose_a, const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                     void* out, int64_t out_stride_m, int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan,
                     DsdProblem* p) {
  p->empty = false;
  if (blocking != 64 && blocking != 128) return fail(STK_ERR_UNSUPPORTED, "%s: blocking %d (64 or 128)", who, blocking);
  if (dtype != STK_F16 && dtype != STK_BF16) return fail(STK_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "%s: index dtype %d", who, index_dtype);
  if (m < 0 || n < 0 || k < 0 || nnz < 0) return fail(STK_ERR_DIMS, "%s: negative size", who);
  if (m % blocking || k % blocking || n % 8)
    return fail(STK_ERR_DIMS, "incompatible dimensions: sparse [%lld, %lld] x dense [%lld, %lld] with blocking %d",
                (long long)m, (long long)k, (long long)k, (long long)n, blocking);
  if (m == 0 || n == 0) {
    p->empty = true;
    return STK_OK;
  }
  const int64_t block_rows = m / blocking;
  if (block_rows * ((n + 63) / 64) > INT32_MAX || n > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "%s: size exceeds 32-bit range", who);
  const bool bk = rhs_stride_n != 1;   // .t() view of a row-major [n, k]: K-major tile
  if (bk && rhs_stride_k != 1) return fail(STK_ERR_UNSUPPORTED, "%s: rhs needs a unit stride", who);
  const int64_t ldb = bk ? rhs_stride_n : rhs_stride_k;
  if (ldb % 8 || out_stride_m % 8 || !aligned16(rhs) || !aligned16(out) || !aligned16(data))
    return fail(STK_ERR_UNSUPPORTED, "%s: operands need 16-byte aligned bases and leading dimensions divisible by 8", who);
  if (ldb >= (1 << 24)) return fail(STK_ERR_UNSUPPORTED, "%s: leading dimension exceeds 2^24 elements", who);
  const bool ta = transpose_a != 0;
  DsdArgs& g = p->g;
  g.data = static_cast<const elem_t*>(data);
  g.walk_offsets = ta ? offsets_t : offsets;
  g.walk_columns = ta ? column_indices_t : column_indices;
  g.walk_blocks = ta ? block_offsets_t : nullptr;
  g.rhs = static_cast<const elem_t*>(rhs);
  g.ldb = ldb;
  g.out = static_cast<elem_t*>(out);
  g.ldc = out_stride_m;
  g.block_rows = (int)block_rows;
  g.n = (int)n;
  g.idx32 = index_dtype == STK_I32;
  g.row_map = nullptr;
  g.row_scale = nullptr;
  g.out_rows = 0;
  // a dense-operand row panel (one block of k) is read once per tile that walks a block in that block column of
  // op(S): with few blocks per column (a block-diagonal MoE layout has one fused tile per expert) it is streamed
  // (row-major rhs only: a K-major tile uses half a cache line per K-tile and needs the line to stay)
  p->stream_rhs = !bk && nnz <= 4 * (k / blocking);
  p->ta = ta;
  p->bk = bk;
  g.small = nnz * (n / 128) < kSmallWorkPerUnit * compute_units();
  if (!g.walk_offsets || (nnz > 0 && (!g.walk_columns || (ta && !g.walk_blocks) || !data))) return fail(STK_ERR_DIMS, "%s: missing metadata pointer", who);
  // lists of the walked lines: block rows of the stored matrix [m, k], or block columns of the stored [k, m]
  p->lists = PlanLists{nullptr, nullptr, 0};
  if (plan) p->lists = ta ? plan_lists_of(plan_body(plan, k / blocking, nnz), k / blocking, m / blocking, true)
                          : plan_lists_of(plan_body(plan, m / blocking, nnz), m / blocking, k / blocking, false);
  return STK_OK;
}

extern "C" int stk_dsd(int64_t m, int64_t k, int64_t n,
                       const void* data, const int32_t* offsets, const void* column_indices,
                       const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                       int transpose_a,
                       const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                       void* out, int64_t out_stride_m,
                       int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan,
                       void* workspace, int64_t workspace_bytes, stk_stream_t stream) {
  using namespace stk;
  if (dtype == STK_F32) {
    if (m < 0 || n < 0 || k < 0 || nnz < 0) return fail(STK_ERR_DIMS, "stk_dsd: negative size");
    if (blocking > 0 && (m % blocking || k % blocking))
      return fail(STK_ERR_DIMS, "incompatible dimensions: sparse [%lld, %lld] x dense [%lld, %lld] with blocking %d", (long long)m, (long long)k,
                  (long long)k, (long long)n, blocking);
    const bool ta = transpose_a != 0;
    if (ta && nnz > 0 && !block_offsets_t) return fail(STK_ERR_DIMS, "stk_dsd: missing metadata pointer");
    return walk_f32(true, "stk_dsd", blocking > 0 ? m / blocking : 0, n, data, ta ? offsets_t : offsets, ta ? column_indices_t : column_indices,
                    ta ? block_offsets_t : nullptr, !ta, rhs, rhs_stride_n, rhs_stride_k, out, out_stride_m, nnz, blocking, index_dtype,
                    static_cast<hipStream_t>(stream));
  }
  DsdProblem problem;
  const int rc = dsd_problem("stk_dsd", m, k, n, data, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t, transpose_a, rhs,
                             rhs_stride_k, rhs_stride_n, out, out_stride_m, nnz, blocking, dtype, index_dtype, plan, &problem);
  if (rc != STK_OK || problem.empty) return rc;
  const DsdArgs& g = problem.g;
  const PlanLists& lists = problem.lists;
  const bool ta = problem.ta, bk = problem.bk, stream_rhs = problem.stream_rhs;
  TailArgs tail{};
  bool sliced = false;
  const int tail_rc = tail_of("stk_dsd", g, n, nnz, blocking, plan, workspace, workspace_bytes, &tail, &sliced);
  if (tail_rc != STK_OK) return tail_rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define STK_DSD_CASE(BF, BLK, TA, BK)                                                          \
  if ((dtype == STK_BF16) == BF && blocking == BLK && ta == TA && bk == BK) {                  \
    if (!BK && stream_rhs) launch_dsd<BF, BLK, TA, BK, !BK>(g, lists, sliced ? &tail : nullptr, s); \
    else launch_dsd<BF, BLK, TA, BK, false>(g, lists, sliced ? &tail : nullptr, s);            \
    return check_launch("stk_dsd");                                                            \
  }
#define STK_DSD_LAYOUTS(BF, BLK) \
  STK_DSD_CASE(BF, BLK, true, true) STK_DSD_CASE(BF, BLK, true, false) STK_DSD_CASE(BF, BLK, false, true) STK_DSD_CASE(BF, BLK, false, false)
  STK_DSD_LAYOUTS(true, 128) STK_DSD_LAYOUTS(false, 128) STK_DSD_LAYOUTS(true, 64) STK_DSD_LAYOUTS(false, 64)
  return fail(STK_ERR_UNSUPPORTED, "stk_dsd: no kernel for this configuration");
}

extern "C" int stk_dsd_scatter(int64_t m, int64_t k, int64_t n, const void* data, const int32_t* offsets, const void* column_indices,
                               const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                               const int32_t* row_slots, const float* weights, int64_t num_tokens, void* out, int64_t out_stride_m,
                               int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan,
                               void* workspace, int64_t workspace_bytes, stk_stream_t stream) {
  using namespace stk;
  const char* who = "stk_dsd_scatter";
  if (blocking != 128) return fail(STK_ERR_UNSUPPORTED, "%s: blocking %d (128 only)", who, blocking);
  if (num_tokens < 0 || num_tokens > INT32_MAX) return fail(STK_ERR_DIMS, "%s: %lld tokens", who, (long long)num_tokens);
  DsdProblem problem;
  const int rc = dsd_problem(who, m, k, n, data, offsets, column_indices, nullptr, nullptr, nullptr, 0, rhs, rhs_stride_k, rhs_stride_n, out,
                             out_stride_m, nnz, blocking, dtype, index_dtype, plan, &problem);
  if (rc != STK_OK || problem.empty || num_tokens == 0) return rc;
  if (!row_slots) return fail(STK_ERR_DIMS, "%s: missing row_slots", who);
  if (n % 256 || problem.g.small)
    return fail(STK_ERR_UNSUPPORTED, "%s: needs a multiple of 256 columns and at least %lld blocks x 128 columns per compute unit", who,
                (long long)kSmallWorkPerUnit);
  DsdArgs g = problem.g;
  g.row_map = row_slots;
  g.row_scale = weights;
  g.out_rows = (int)num_tokens;
  TailArgs tail{};
  bool sliced = false;
  const int tail_rc = tail_of(who, g, n, nnz, blocking, plan, workspace, workspace_bytes, &tail, &sliced);
  if (tail_rc != STK_OK) return tail_rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const TailArgs* t = sliced ? &tail : nullptr;
  const bool bf = dtype == STK_BF16;
  if (problem.bk) {
    if (bf) launch_dsd_scatter<true, true, false>(g, problem.lists, t, s);
    else launch_dsd_scatter<false, true, false>(g, problem.lists, t, s);
  } else if (problem.stream_rhs) {
    if (bf) launch_dsd_scatter<true, false, true>(g, problem.lists, t, s);
    else launch_dsd_scatter<false, false, true>(g, problem.lists, t, s);
  } else {
    if (bf) launch_dsd_scatter<true, false, false>(g, problem.lists, t, s);
    else launch_dsd_scatter<false, false, false>(g, problem.lists, t, s);
  }
  return check_launch(who);
}

extern "C" int64_t stk_dsd_workspace_counter_bytes(void) {
  const int workgroups = stk::compute_units();
  return workgroups > 0 ? (int64_t)stk::tail_counter_bytes(workgroups) : 0;
}

extern "C" int64_t stk_dsd_workspace_slot_bytes(void) { return (int64_t)(sizeof(float) * stk::kSlotFloats); }

extern "C" int64_t stk_dsd_workspace_bytes(int64_t m, int64_t n, int blocking) {
  using namespace stk;
  if (blocking != 128 || m <= 0 || n <= 0 || m % 128 || n % 256) return 0;
  const int workgroups = compute_units();
  if (workgroups <= 0 || (m / 128) * (n / 128) / 3 >= 8 * (int64_t)workgroups) return 0;
  return (int64_t)tail_workspace_bytes(workgroups);
}
