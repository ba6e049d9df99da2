// Fusion plan: which neighbouring block rows (and block columns) of a topology
// have identical patterns and can be computed together as one 256-wide tile.
//
// role[i] = 0  line i is computed on its own
//           1  line i is computed together with line i + 1 (same length, same
//              indices entry by entry, not empty)
//           2  line i is covered by line i - 1
// A maximal run of identical lines is paired greedily from its start:
// (0,1), (2,3), ...  The plan holds the roles of the block rows (walking
// offsets / column_indices) followed by the roles of the block columns
// (walking offsets_t / column_indices_t), a scratch area of the same size, and a
// second set of roles (rows, then columns) for kernels that can also tile three
// lines high: the same pairing, except that the last three lines of a run of odd
// length >= 3 form one group,
//   tall[i] = 3  line i is computed together with lines i + 1 and i + 2
// (0, 1, 2 as above).  A dense operand that is streamed once per tile is then read
// once, not twice, for such a run of three.
// Behind the roles come, as int32, ten counts and ten lists of lines, five per
// direction (block rows first): role 1, role 0, tall 1, tall 3, tall 0 - ascending, except that the two lists of
// lone lines (role 0, tall 0) are in order of descending length (min(blocks, 255); equal lengths ascending) when
// they have at most 4096 entries.  The product
// kernels take their work from these lists, so that no workgroup is launched for a
// covered line.  Last come, per direction, sixteen bytes for stk_dsd: into how many slices
// along k the tiles of the last, partly filled round of workgroups are cut when the dense
// operand has 256 (t + 1) columns, t = 0 .. 15 (1: not at all).  The plan depends on the
// topology (and on the number of compute units of the device it is built on) only, so
// callers may build it once and reuse it for every product on that topology.
//
// A plan built for blocking 64 groups the lines by fours instead (stk_dsd and stk_dds then compute up to four
// identical lines as one 256-wide tile): a run of identical lines is cut from its start into fours while they
// last, and the three, two or one lines that are left form one more group (a four and one line left over become
// a three and a pair).  Lines so long that a tile over four
// of them would be more than a compute unit's share of the whole product (four times their blocks exceed
// 4 nnz / compute units: the expert that takes half of the tokens of a skewed routing) are cut into pairs
// instead, which the kernels start first.  Both role arrays then hold, for the
// first line of a group, the number of its lines (0 for the other lines), and the lists are
//   list 0 (role 1's place)  first lines of groups of four      list 3 (tall 3's place)  of groups of three
//   list 2 (tall 1's place)  of pairs                           list 4 (tall 0's place)  lone lines
// with list 1 empty.
#include "common.h"
#include "wave_scan.h"

namespace stk {

// When the tiles of a launch fill the compute units a few times only, the last round
// leaves most of them idle.  Cutting the tiles of that round into k slices along the
// contraction (workgroups add the partial tiles up) fills the round better, at the price of
// the partial tiles' round trip through memory.  Which k pays is found by playing the
// hardware's dispatch through: workgroups start in order, each on the compute unit that
// is free first.  Tiles of one kind take equally long here (the lines' average length), so
// the compute units are kept as a few groups (free time, how many) in ascending order.
constexpr int kSortCapacity = 4096;  // lone lines that are put in order of their lengths (more: left as they are)
constexpr int kSimGroups = 24;    // groups alive at a time
constexpr int kSimCapacity = 48;  // room for the queue to move along before it is shifted back
struct DispatchSim {
  float* time;  // kSimCapacity entries each, private to the thread
  int* count;
  int head, tail;  // the groups are entries [head, tail), ascending in time
  __host__ __device__ void reset(int units) { time[0] = 0.f, count[0] = units, head = 0, tail = 1; }
  // n work items of the same duration
  __host__ __device__ void run(int n, float duration) {
    while (n > 0) {
      const int m = n < count[head] ? n : count[head];
      const float t = time[head] + duration;
      n -= m;
      count[head] -= m;
      if (count[head] == 0) head++;
      if (tail == kSimCapacity) {
        for (int i = head; i < tail; i++) time[i - head] = time[i], count[i - head] = count[i];
        tail -= head, head = 0;
      }
      int at = tail;
      while (at > head && time[at - 1] > t) at--;
      if (at > head && time[at - 1] == t) {
        count[at - 1] += m;
      } else if (tail - head == kSimGroups) {
        // out of groups: join a neighbour (a small error in a rare case)
        count[at < tail ? at : tail - 1] += m;
      } else {
        for (int i = tail; i > at; i--) time[i] = time[i - 1], count[i] = count[i - 1];
        time[at] = t, count[at] = m, tail++;
      }
    }
  }
  __host__ __device__ float end() const { return time[tail - 1]; }
};

// Simulated end of a launch whose last round is cut into k slices.  tiles[]: pairs, threes, lone lines;
// length: average blocks per line.
__host__ __device__ inline float simulate_launch(DispatchSim& sim, const int (&tiles)[3], float length, int units, int k) {
  // Durations in units of one block of k of a 256x256 tile (about 5 us).  Measured on an MI355X: a workgroup
  // spends about 4 such units outside its K loop (start, first loads, store), and 2 more when its tile is a
  // slice (partial tile out to memory and back in, the counter); 384x128 and 128x256 tiles take 0.75 and 0.58
  // of a 256x256 tile's time per block.
  const float start = 4.f, seam = 2.f;
  const float duration[3] = {length, 0.75f * length, 0.58f * length};
  const int total = tiles[0] + tiles[1] + tiles[2];
  const int whole = (total - 1) / units * units;
  sim.reset(units);
  int left = whole, tail[3];
  for (int kind = 0; kind < 3; kind++) {
    const int n = tiles[kind] < left ? tiles[kind] : left;
    sim.run(n, duration[kind] + start);
    left -= n;
    tail[kind] = tiles[kind] - n;
  }
  for (int slice = 0; slice < k; slice++)
    for (int kind = 0; kind < 3; kind++) sim.run(tail[kind], k == 1 ? duration[kind] + start : duration[kind] / k + start + seam);
  return sim.end();
}

// With more than four rounds of tiles the last one matters too little to be worth the simulation.
__host__ __device__ inline bool tail_slices_considered(int64_t tiles, int units) { return tiles > 0 && units > 0 && tiles <= 4 * (int64_t)units; }

// Slices for the tiles of the last round, given the simulated ends for k = 1 .. kMaxTailSlices: the k with the
// shortest launch, 1 unless k > 1 saves 2 %.
__host__ __device__ inline int choose_tail_slices(const float (&end)[kMaxTailSlices]) {
  int best = 1;
  float best_end = end[0];
  for (int k = 2; k <= kMaxTailSlices; k++)
    if (end[k - 1] < best_end && end[k - 1] < 0.98f * end[0]) best = k, best_end = end[k - 1];
  return best;
}

// Step 1, one wavefront per line (both directions in one launch): same[i] = line i + 1
// repeats line i.  The flags go to the scratch half of the plan.
template <typename IDX>
__global__ __launch_bounds__(256) void plan_same_kernel(
    const int32_t* __restrict__ offsets, const IDX* __restrict__ column_indices, int block_rows,
    const int32_t* __restrict__ offsets_t, const IDX* __restrict__ column_indices_t, int block_cols,
    uint8_t* __restrict__ plan) {
  const int lane = threadIdx.x & 63;
  int i = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= block_rows + block_cols) return;
  const bool cols = i >= block_rows;
  const int32_t* offs = cols ? offsets_t : offsets;
  const IDX* idx = cols ? column_indices_t : column_indices;
  const int lines = cols ? block_cols : block_rows;
  uint8_t* same = plan + block_rows + block_cols + (cols ? block_rows : 0);
  if (cols) i -= block_rows;
  bool eq = false;
  if (i + 1 < lines) {
    const int a = offs[i], b = offs[i + 1], c = offs[i + 2];
    eq = (b - a == c - b) && (b > a);
    if (eq) {
      bool diff = false;
      for (int e = lane; e < b - a; e += 64) diff |= idx[a + e] != idx[b + e];
      eq = __ballot(diff) == 0;
    }
  }
  if (lane == 0) same[i] = eq ? 1 : 0;
}

// Block rows of the sdd tile that line i owns (0: an earlier line's tile covers it).  pos: its place in its run
// of identical lines.  same[j]: line j + 1 repeats line j (0 for the last line).
//   most == 4: the run is cut from its start into fours while they last; what is left - three, two or one
//              lines - forms one more group (a four and one line left over become a three and a pair);
//   most == 2: into pairs, and the last three lines of a run of odd length (three or more) form a group of
//              three, whose tiles are one block wide; a run of one line is a single line.
__device__ __forceinline__ int sdd_rows_owned(const uint8_t* same, int i, int pos, int most) {
  if (most == 2) {
    if (pos & 1) return 0;
    int left = 1;  // lines from this one to the end of the run, at most four
    while (left < 4 && same[i + left - 1]) left++;
    if (left == 3) return 3;
    if (left == 1) return pos == 0 ? 1 : 0;  // the third line of a group of three
    return 2;
  }
  // most == 4.  A run of n lines is cut from its start into fours; what is left forms one more group of three or
  // two, or a lone line if the run is one line - except that the last five lines of a run of 4 q + 1 lines (q >= 1)
  // form a three and a pair rather than a four and a lone line, which would run on a tile with most of its rows
  // dropped.  Seen from a line: groups start at positions 0, 4, 8, ... and, for that pair, at the position 3 mod 4
  // from which exactly two lines are left.
  const int q = pos & 3;
  int left = 1;  // lines from this one to the end of the run, at most six
  while (left < 6 && same[i + left - 1]) left++;
  if (q == 0) {
    if (left == 1 && pos >= 4) return 0;  // the last line of a run of 4 q + 1: covered by the pair before it
    return left >= 6 || left == 4 ? 4 : (left == 5 ? 3 : left);
  }
  if (q == 3 && left == 2) return 2;
  return 0;
}
// The same for the groups of stk_dsd / stk_dds with 64-blocks: fours (as above) unless the lines are `heavy`, then
// pairs from the start of the run with a lone line left over when its length is odd.
__device__ __forceinline__ int lines_owned64(const uint8_t* same, int i, int pos, bool heavy) {
  if (!heavy) return sdd_rows_owned(same, i, pos, 4);
  if (pos & 1) return 0;
  return same[i] ? 2 : 1;
}
// A tile over four lines of `blocks` blocks each would be more than a compute unit's share of a product whose
// other dimension has four tiles.
__device__ __forceinline__ bool heavy_line(int blocks, int64_t nnz, int compute_units) {
  const int64_t share = nnz * 4 / (compute_units > 0 ? compute_units : 1);
  return 4 * (int64_t)blocks > (share > 1 ? share : 1);
}
// Blocks side by side in the tiles of a group of `rows` lines.
// (most_cols == 2: a group of three rows has tiles of 3 x 1 blocks; most_cols == 4: every tile is up to four wide)
__device__ __forceinline__ int sdd_cols_of(int rows, int most_cols) { return (rows == 3 && most_cols == 2) ? 1 : most_cols; }

// Step 2, one workgroup of 1024 threads per direction (blockIdx.x = 0: rows, 1: columns):
// position of every line inside its run of identical lines, then the roles.
__global__ __launch_bounds__(1024) void plan_roles_kernel(const int32_t* __restrict__ offsets, int block_rows,
                                                          const int32_t* __restrict__ offsets_t, int block_cols,
                                                          int compute_units, uint8_t* __restrict__ plan, int32_t* __restrict__ sdd, int max_sdd_tiles,
                                                          int sdd_rows, int sdd_cols, int most) {
  __shared__ int wave_last[16];
  __shared__ int sort_count[256];
  __shared__ int sort_line[kSortCapacity];
  __shared__ uint8_t sort_key[kSortCapacity];
  __shared__ uint16_t sort_wave[16 * 256];  // per wavefront and key: a count, then the place of the first such entry
  __shared__ float sim_time[kTailSliceColumns * kMaxTailSlices][kSimCapacity];
  __shared__ int sim_count[kTailSliceColumns * kMaxTailSlices][kSimCapacity];
  const bool cols = blockIdx.x == 1;
  const int lines = cols ? block_cols : block_rows;
  uint8_t* tail_slices = plan + plan_slices_offset(block_rows, block_cols) + (cols ? kPlanHintBytes : 0);
  if (lines == 0) {
    if (threadIdx.x < kPlanLists) reinterpret_cast<int32_t*>(plan + plan_list_offset(block_rows, block_cols))[(cols ? kPlanLists : 0) + threadIdx.x] = 0;
    if (threadIdx.x < kPlanHintBytes) tail_slices[threadIdx.x] = threadIdx.x < kTailSliceColumns ? 1 : 0;
    if (!cols && threadIdx.x == 0) sdd[0] = 0;
    return;
  }
  uint8_t* role = plan + (cols ? block_rows : 0);
  const uint8_t* same = plan + block_rows + block_cols + (cols ? block_rows : 0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // start of the run that contains the line before this thread's chunk: exclusive
  // max-scan over the chunks' last run starts
  const int per = (lines + 1023) / 1024;
  const int lo = tid * per < lines ? tid * per : lines;
  const int hi = lo + per < lines ? lo + per : lines;
  int last = -1;
  for (int i = lo; i < hi; i++)
    if (i == 0 || same[i - 1] == 0) last = i;
  int v = last;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int o = __shfl_up(v, d, 64);
    if (lane >= d && o > v) v = o;
  }
  if (lane == 63) wave_last[wave] = v;
  __syncthreads();
  int start = __shfl_up(v, 1, 64);
  if (lane == 0) start = -1;
  for (int w = 0; w < wave; w++) start = wave_last[w] > start ? wave_last[w] : start;
  const int start_of_chunk = start;
  uint8_t* tall = plan + 2 * (block_rows + block_cols) + (cols ? block_rows : 0);
  int mine[kPlanLists] = {0, 0, 0, 0, 0};  // this thread's lines per list
  for (int i = lo; i < hi; i++) {
    if (i == 0 || same[i - 1] == 0) start = i;
    const int pos = i - start;
    if (most == 4) {
      // groups of up to four lines: the first line of a group holds the group's size
      const int32_t* offs = cols ? offsets_t : offsets;
      const int n = lines_owned64(same, i, pos, heavy_line(offs[i + 1] - offs[i], offs[lines], compute_units));
      role[i] = tall[i] = (uint8_t)n;
      mine[kPairs] += n == 4;
      mine[kTallTriples] += n == 3;
      mine[kTallPairs] += n == 2;
      mine[kTallSingles] += n == 1;
      continue;
    }
    const int r = (pos & 1) ? 2 : (same[i] ? 1 : 0);
    int t = 2;  // odd positions, and the last line of an odd run of three or more, are covered
    if ((pos & 1) == 0) {
      if (!same[i]) t = pos >= 2 ? 2 : 0;
      else t = (same[i + 1] && !same[i + 2]) ? 3 : 1;  // exactly three lines left: one group of three
    }
    role[i] = r;
    tall[i] = t;
    mine[0] += r == 1;
    mine[1] += r == 0;
    mine[2] += t == 1;
    mine[3] += t == 3;
    mine[4] += t == 0;
  }
  // compacted ascending lists of the lines that own a tile, one exclusive scan per list
  int32_t* lists = reinterpret_cast<int32_t*>(plan + plan_list_offset(block_rows, block_cols));
  int totals[kPlanLists];
#pragma unroll
  for (int kind = 0; kind < kPlanLists; kind++) {
    __syncthreads();
    int inc = mine[kind];
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      int o = __shfl_up(inc, d, 64);
      if (lane >= d) inc += o;
    }
    if (lane == 63) wave_last[wave] = inc;
    __syncthreads();
    int base = inc - mine[kind], total = 0;
    for (int w = 0; w < 16; w++) {
      if (w < wave) base += wave_last[w];
      total += wave_last[w];
    }
    int32_t* list = lists + 2 * kPlanLists + (cols ? kPlanLists * block_rows : 0) + kind * lines;
    if (tid == 0) lists[(cols ? kPlanLists : 0) + kind] = total;
    totals[kind] = total;
    const uint8_t* from = kind < 2 ? role : tall;
    int want = kind == 0 ? 1 : kind == 1 ? 0 : kind == 2 ? 1 : kind == 3 ? 3 : 0;
    if (most == 4) want = kind == kPairs ? 4 : kind == kTallTriples ? 3 : kind == kTallPairs ? 2 : kind == kTallSingles ? 1 : -1;
    for (int i = lo; i < hi; i++)
      if (from[i] == want) list[base++] = i;
  }
  // Every list longest first (lines of equal length keep their order, so the lines of an expert stay neighbours):
  // workgroups start in list order, so the long walks begin early and the short ones fill the end of the launch,
  // wherever the long lines lie in the matrix.  A counting sort on min(blocks, 255) in LDS; a list that is in this
  // order already (all lines equally long: the block rows of a dMoE topology) is left alone, lists longer than
  // kSortCapacity stay in ascending order.
  {
    const int32_t* offs = cols ? offsets_t : offsets;
    for (int kind = 0; kind < kPlanLists; kind++) {
      const int count = totals[kind];
      if (count < 2 || count > kSortCapacity) continue;  // (the same for every thread)
      int32_t* list = lists + 2 * kPlanLists + (cols ? kPlanLists * block_rows : 0) + kind * lines;
      __syncthreads();  // the list is complete, the last sort is over
      if (tid < 256) sort_count[tid] = 0;
      for (int e = tid; e < count; e += 1024) {
        const int line = list[e], blocks = offs[line + 1] - offs[line];
        sort_line[e] = line;
        sort_key[e] = (uint8_t)(255 - (blocks < 255 ? blocks : 255));  // ascending key = descending length
      }
      __syncthreads();
      int unordered = 0;
      for (int e = tid; e + 1 < count; e += 1024) unordered |= sort_key[e] > sort_key[e + 1];
      if (__syncthreads_or(unordered) == 0) continue;
      for (int e = tid; e < count; e += 1024) atomicAdd(&sort_count[sort_key[e]], 1);
      __syncthreads();
      // sort_count[k]: where the entries with key k begin (an exclusive scan over the keys)
      {
        int total;
        const int begin = block_exclusive_scan(tid < 256 ? sort_count[tid] : 0, wave_last, &total);
        if (tid < 256) sort_count[tid] = begin;
      }
      // 1024 entries at a time, in list order: an entry goes behind the entries with its key that came before it -
      // those of earlier rounds (sort_count runs on), of earlier wavefronts of this round (sort_wave) and of
      // earlier lanes of its wavefront (counted with ballots, one distinct key of the wavefront at a time)
      for (int e0 = 0; e0 < count; e0 += 1024) {
        for (int i = tid; i < 16 * 256; i += 1024) sort_wave[i] = 0;
        __syncthreads();
        const int e = e0 + tid;
        const bool valid = e < count;
        const int key = valid ? sort_key[e] : -1;
        int rank = 0;
        uint64_t todo = __ballot(valid);
        while (todo) {
          const int k = __builtin_amdgcn_readlane(key, __ffsll((unsigned long long)todo) - 1);
          const uint64_t same = __ballot(key == k);
          if (key == k) rank = __popcll(same & ((1ull << lane) - 1));
          if (lane == 0) sort_wave[wave * 256 + k] = (uint16_t)__popcll(same);
          todo &= ~same;
        }
        __syncthreads();
        if (tid < 256) {
          int at = sort_count[tid];
          for (int w = 0; w < 16; w++) {
            const int n = sort_wave[w * 256 + tid];
            sort_wave[w * 256 + tid] = (uint16_t)at;
            at += n;
          }
          sort_count[tid] = at;
        }
        __syncthreads();
        if (valid) list[sort_wave[wave * 256 + key] + rank] = sort_line[e];
        __syncthreads();
      }
    }
    __syncthreads();
    // How many consecutive entries of each list go to one compute die at a time (xcd_item): as many as hold a
    // quarter of a die's share of the list's blocks when they are as long as the first, the longest, entry - the
    // first group is the heaviest, and a die that gets too much of the launch in one piece holds it up - rounded
    // down to a power of two, between 1 and 32.
    int blocks_of_groups[2] = {0, 0};  // (thread 0) blocks of one line per entry: lists of pairs / lone lines, lists with threes
    for (int kind = 0; kind < kPlanLists; kind++) {
      const int count = totals[kind];
      const int32_t* list = lists + 2 * kPlanLists + (cols ? kPlanLists * block_rows : 0) + kind * lines;
      int mine_blocks = 0;
      for (int e = tid; e < count; e += 1024) {
        const int line = list[e];
        mine_blocks += offs[line + 1] - offs[line];
      }
      int total_blocks;
      block_exclusive_scan(mine_blocks, wave_last, &total_blocks);
      if (tid == 0) {
        int entries = 1;
        if (count > 0) {
          const int first = list[0], longest = offs[first + 1] - offs[first];
          const int fit = total_blocks / (32 * (longest > 0 ? longest : 1));
          while (entries < 32 && 2 * entries <= fit) entries *= 2;
        }
        tail_slices[kGroupHint + kind] = (uint8_t)entries;
        blocks_of_groups[kind >= kTallPairs ? 1 : 0] += total_blocks;
      }
    }
    if (tid == 0) {
      // from which width of the dense operand on stripes beat lines (kStripeHint); plans for 128-blocks only
      const int64_t nnz = offs[lines];
      const int others = cols ? block_rows : block_cols;
      for (int family = 0; family < 2; family++) {
        const int64_t saved = (int64_t)blocks_of_groups[family] - others;  // dense panels that stripes fetch fewer
        int from = 0;
        if (most == 2 && saved > 0) {
          const int64_t tiles = (7 * nnz + saved - 1) / saved;  // 896 nnz / saved columns, in tiles of 128 columns
          from = tiles > 255 ? 0 : (tiles < 1 ? 1 : (int)tiles);
        }
        tail_slices[kStripeHint + (family ? 0 : 1)] = (uint8_t)from;
      }
    }
    __syncthreads();
  }
  // Tiles of stk_sdd (block rows only), row by row: groups of identical rows (sdd_rows_owned) times up to
  // sdd_cols neighbouring blocks (one for a group of three rows).
  if (!cols) {
    int own = 0, first = start_of_chunk;
    for (int i = lo; i < hi; i++) {
      if (i == 0 || same[i - 1] == 0) first = i;
      const int rows = sdd_rows_owned(same, i, i - first, sdd_rows);
      if (rows) own += (offsets[i + 1] - offsets[i] + sdd_cols_of(rows, sdd_cols) - 1) / sdd_cols_of(rows, sdd_cols);
    }
    __syncthreads();
    int inc = own;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      int o = __shfl_up(inc, d, 64);
      if (lane >= d) inc += o;
    }
    if (lane == 63) wave_last[wave] = inc;
    __syncthreads();
    int base = inc - own, total = 0;
    for (int w = 0; w < 16; w++) {
      if (w < wave) base += wave_last[w];
      total += wave_last[w];
    }
    const bool fits = total <= max_sdd_tiles;  // (more only if nnz was not offsets[block_rows])
    if (tid == 0) sdd[0] = fits ? total : 0, sdd[1] = 0;
    int32_t* at = sdd + 2 + 2 * (int64_t)base;
    first = start_of_chunk;
    for (int i = lo; i < hi && fits; i++) {
      if (i == 0 || same[i - 1] == 0) first = i;
      const int rows = sdd_rows_owned(same, i, i - first, sdd_rows);
      if (rows == 0) continue;
      const int nseg = offsets[i + 1] - offsets[i], p = offsets[i];
      const int wide = sdd_cols_of(rows, sdd_cols);
      for (int j = 0; j < nseg; j += wide, at += 2) {
        at[0] = p + j;
        at[1] = rows | ((nseg - j < wide ? nseg - j : wide) << 8);
      }
    }
  }
  // slices for the last round of stk_dsd: one thread per (width of the dense operand, slice count) simulates
  // the launch; the first of each four picks
  static_assert(kTailSliceColumns * kMaxTailSlices == 64 && kMaxTailSlices == 4, "one wavefront");
  if (tid < 64) {
    const int32_t* offs = cols ? offsets_t : offsets;
    const int ntn = tid / kMaxTailSlices + 1;  // column tiles of 256
    const int tiles[3] = {totals[kTallPairs] * ntn, totals[kTallTriples] * 2 * ntn, totals[kTallSingles] * ntn};
    DispatchSim sim{sim_time[tid], sim_count[tid], 0, 0};
    float end = 0.f;
    if (tail_slices_considered(tiles[0] + tiles[1] + tiles[2], compute_units) && offs)
      end = simulate_launch(sim, tiles, (float)offs[lines] / (float)lines, compute_units, tid % kMaxTailSlices + 1);
    float ends[kMaxTailSlices];
#pragma unroll
    for (int k = 0; k < kMaxTailSlices; k++) ends[k] = __shfl(end, (tid & ~3) + k, 64);
    if (tid % kMaxTailSlices == 0) tail_slices[tid / kMaxTailSlices] = (uint8_t)choose_tail_slices(ends);
  }
  // Do equal eighths of the lines hold about equal numbers of blocks?  If not (one share 25 % above the mean),
  // the products spread the list over the XCDs in small groups instead of eight contiguous shares.
  if (tid == 64) {
    const int32_t* offs = cols ? offsets_t : offsets;
    int spread = 0;
    if (offs) {
      const int64_t total = offs[lines];
      for (int c = 0; c < 8; c++) {
        const int64_t share = offs[(int64_t)(c + 1) * lines / 8] - offs[(int64_t)c * lines / 8];
        if (share * 32 > total * 5) spread = 1;  // > 1.25 / 8 of the blocks
      }
    }
    tail_slices[kSpreadHint] = (uint8_t)spread;
  }
}

}  // namespace stk

extern "C" size_t stk_plan_bytes(int64_t block_rows, int64_t block_cols, int64_t nnz) {
  if (block_rows < 0 || block_cols < 0 || nnz < 0) return 0;
  return stk::plan_sdd_bytes(block_rows, nnz) + stk::plan_slices_offset(block_rows, block_cols) + 2 * stk::kPlanHintBytes;
}

extern "C" int stk_dsd_tail_slices(int64_t pair_tiles, int64_t triple_tiles, int64_t single_tiles, double blocks_per_line, int compute_units) {
  using namespace stk;
  if (pair_tiles < 0 || triple_tiles < 0 || single_tiles < 0 || pair_tiles + triple_tiles + single_tiles > INT32_MAX) return 1;
  if (!tail_slices_considered(pair_tiles + triple_tiles + single_tiles, compute_units)) return 1;
  float time[kSimCapacity];
  int count[kSimCapacity];
  DispatchSim sim{time, count, 0, 0};
  const int tiles[3] = {(int)pair_tiles, (int)triple_tiles, (int)single_tiles};
  float ends[kMaxTailSlices];
  for (int k = 1; k <= kMaxTailSlices; k++) ends[k - 1] = simulate_launch(sim, tiles, (float)blocks_per_line, compute_units, k);
  return choose_tail_slices(ends);
}

extern "C" int stk_build_plan(const int32_t* offsets, const void* column_indices, int64_t block_rows,
                              const int32_t* offsets_t, const void* column_indices_t, int64_t block_cols,
                              int64_t nnz, int blocking, int index_dtype, uint8_t* plan, size_t plan_bytes, stk_stream_t stream) {
  using namespace stk;
  if (blocking != 64 && blocking != 128) return fail(STK_ERR_UNSUPPORTED, "stk_build_plan: blocking %d (64 or 128)", blocking);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_build_plan: index dtype %d", index_dtype);
  if (block_rows < 0 || block_cols < 0 || block_rows >= INT32_MAX || block_cols >= INT32_MAX || nnz < 0 || nnz >= INT32_MAX)
    return fail(STK_ERR_DIMS, "stk_build_plan: bad size");
  if (block_rows + block_cols == 0) return STK_OK;
  if (!plan || plan_bytes < stk_plan_bytes(block_rows, block_cols, nnz))
    return fail(STK_ERR_WORKSPACE, "stk_build_plan: plan buffer of %zu bytes needed", stk_plan_bytes(block_rows, block_cols, nnz));
  if (reinterpret_cast<uintptr_t>(plan) & 3u) return fail(STK_ERR_UNSUPPORTED, "stk_build_plan: plan buffer needs 4-byte alignment");
  int32_t* sdd = reinterpret_cast<int32_t*>(plan);
  plan += plan_sdd_bytes(block_rows, nnz);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int grid = (int)((block_rows + block_cols + 3) / 4);
  if (index_dtype == STK_I32)
    hipLaunchKernelGGL((plan_same_kernel<int32_t>), dim3(grid), dim3(256), 0, s, offsets, static_cast<const int32_t*>(column_indices),
                       (int)block_rows, offsets_t, static_cast<const int32_t*>(column_indices_t), (int)block_cols, plan);
  else
    hipLaunchKernelGGL((plan_same_kernel<int16_t>), dim3(grid), dim3(256), 0, s, offsets, static_cast<const int16_t*>(column_indices),
                       (int)block_rows, offsets_t, static_cast<const int16_t*>(column_indices_t), (int)block_cols, plan);
  hipLaunchKernelGGL(plan_roles_kernel, dim3(2), dim3(1024), 0, s, offsets, (int)block_rows, offsets_t, (int)block_cols, compute_units(), plan, sdd,
                     (int)sdd_max_tiles(block_rows, nnz), blocking == 64 ? 4 : 2, blocking == 64 ? 4 : 2, blocking == 64 ? 4 : 2);
  return check_launch("stk_build_plan");
}
