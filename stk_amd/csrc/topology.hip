// Topology and format kernels: row_indices, transpose metadata (stable radix
// sort built on wavefront ballots and scans), to_dense, to_sparse.
// All integer work; results are bit-exact by construction.
#include "common.h"
#include "wave_scan.h"

namespace stk {

// ------------------------------------------------------------ row_indices
template <typename IDX>
__global__ void row_indices_kernel(const int32_t* __restrict__ offsets, int block_rows, int64_t nnz, IDX* __restrict__ out) {
  for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < nnz; p += (int64_t)gridDim.x * blockDim.x) {
    // last row r with offsets[r] <= p (empty rows repeat an offset and are skipped)
    int lo = 0, hi = block_rows;
    while (hi - lo > 1) {
      int mid = (lo + hi) >> 1;
      if (offsets[mid] <= p) lo = mid; else hi = mid;
    }
    out[p] = static_cast<IDX>(lo);
  }
}

// ------------------------------------------------------- transpose metadata
// Least-significant-digit radix sort of (block column, block id) pairs, 8 bits
// per pass.  A wavefront owns a tile of 1024 consecutive pairs.  Per pass:
//   histogram  per-tile digit counts, stored digit-major [256][tiles]
//   scan       one exclusive scan over that table = first output slot of every
//              (digit, tile) pair
//   scatter    the tile walks its pairs in order, 64 at a time; lanes holding
//              the same digit find each other with 8 ballots, take consecutive
//              slots in lane order and bump the digit's cursor.  In-order walk
//              plus lane order keeps the sort stable.
constexpr int kTile = 1024;

template <typename IDX, bool FIRST>
__device__ __forceinline__ int sort_key(const void* __restrict__ keys, int64_t i) {
  if constexpr (FIRST) return static_cast<int>(static_cast<const IDX*>(keys)[i]);
  else return static_cast<const int32_t*>(keys)[i];
}

template <typename IDX, bool FIRST>
__global__ __launch_bounds__(kWave) void radix_histogram_kernel(const void* __restrict__ keys, int64_t n, int shift,
                                                                int tiles, int32_t* __restrict__ hist) {
  __shared__ int counts[256];
  const int lane = threadIdx.x;
  const int tile = blockIdx.x;
  for (int d = lane; d < 256; d += kWave) counts[d] = 0;
  __syncthreads();
  for (int i = 0; i < kTile / kWave; i++) {
    int64_t idx = (int64_t)tile * kTile + i * kWave + lane;
    if (idx < n) atomicAdd(&counts[(sort_key<IDX, FIRST>(keys, idx) >> shift) & 255], 1);
  }
  __syncthreads();
  for (int d = lane; d < 256; d += kWave) hist[(int64_t)d * tiles + tile] = counts[d];
}

__global__ __launch_bounds__(1024) void exclusive_scan_kernel(int32_t* __restrict__ v, int64_t n) {
  __shared__ int part[16];
  const int64_t per = (n + 1023) / 1024;
  const int64_t lo = threadIdx.x * per;
  const int64_t hi = (lo + per < n) ? lo + per : n;
  int sum = 0;
  for (int64_t i = lo; i < hi; i++) sum += v[i];
  int total;
  int run = block_exclusive_scan(sum, part, &total);
  for (int64_t i = lo; i < hi; i++) {
    int x = v[i];
    v[i] = run;
    run += x;
  }
}

template <typename IDX, bool FIRST>
__global__ __launch_bounds__(kWave) void radix_scatter_kernel(const void* __restrict__ keys_in, const int32_t* __restrict__ vals_in,
                                                              int64_t n, int shift, int tiles, const int32_t* __restrict__ hist,
                                                              int32_t* __restrict__ keys_out, int32_t* __restrict__ vals_out) {
  __shared__ int cursor[256];
  const int lane = threadIdx.x;
  const int tile = blockIdx.x;
  for (int d = lane; d < 256; d += kWave) cursor[d] = hist[(int64_t)d * tiles + tile];
  __syncthreads();
  for (int i = 0; i < kTile / kWave; i++) {
    const int64_t idx = (int64_t)tile * kTile + i * kWave + lane;
    const bool valid = idx < n;
    int key = 0, val = 0, digit = 0;
    if (valid) {
      key = sort_key<IDX, FIRST>(keys_in, idx);
      val = FIRST ? (int)idx : vals_in[idx];
      digit = (key >> shift) & 255;
    }
    uint64_t same = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      uint64_t bal = __ballot(valid && ((digit >> b) & 1));
      same &= ((digit >> b) & 1) ? bal : ~bal;
    }
    int pos = 0;
    if (valid) pos = cursor[digit] + __popcll(same & lanes_below(lane));
    __syncthreads();
    if (valid) {
      keys_out[pos] = key;
      vals_out[pos] = val;
      if ((same >> lane) >> 1 == 0) cursor[digit] += __popcll(same);  // highest lane of the group
    }
    __syncthreads();
  }
}

template <typename IDX>
__global__ void transpose_finalize_kernel(const int32_t* __restrict__ keys, const int32_t* __restrict__ vals,
                                          const IDX* __restrict__ row_indices, int64_t nnz, int block_cols,
                                          IDX* __restrict__ column_indices_t, int32_t* __restrict__ offsets_t,
                                          int32_t* __restrict__ block_offsets_t) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t t0 = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  for (int64_t i = t0; i < nnz; i += stride) {
    int v = vals[i];
    block_offsets_t[i] = v;
    column_indices_t[i] = row_indices[v];
  }
  for (int64_t c = t0; c <= block_cols; c += stride) {
    // number of sorted keys below c
    int64_t lo = 0, hi = nnz;
    while (lo < hi) {
      int64_t mid = (lo + hi) >> 1;
      if (keys[mid] < c) lo = mid + 1; else hi = mid;
    }
    offsets_t[c] = (int32_t)lo;
  }
}

// The whole transpose for up to kSmallSort blocks in one launch of one workgroup: the same radix passes
// (sixteen wavefronts, each owning a contiguous sixteenth of the pairs; counts and cursors per (digit,
// wavefront) in LDS) and the final gather, separated by workgroup barriers instead of kernel boundaries.
// Seven dependent launches cost more than the work itself at these sizes.  16-bit indices carry the block row
// in the upper half of the key (the digits of the lower half are sorted only), which saves the gather at the end.
// offsets_t is filled from the places where the sorted column changes.
constexpr int kSmallSort = 16384;

// Key of pair idx in the first pass: the block column; 16-bit indices carry the block row above it.
template <typename IDX>
__device__ __forceinline__ int first_key(const IDX* __restrict__ row_indices, const IDX* __restrict__ column_indices, int idx) {
  if constexpr (sizeof(IDX) == 2) return (static_cast<int>(row_indices[idx]) << 16) | static_cast<int>(static_cast<uint16_t>(column_indices[idx]));
  else return static_cast<int>(column_indices[idx]);
}

template <typename IDX>
__global__ __launch_bounds__(1024) void transpose_small_kernel(const IDX* __restrict__ row_indices, const IDX* __restrict__ column_indices,
                                                               int nnz, int block_cols, int passes, int32_t* keys0, int32_t* keys1,
                                                               int32_t* vals0, int32_t* vals1, IDX* __restrict__ column_indices_t,
                                                               int32_t* __restrict__ offsets_t, int32_t* __restrict__ block_offsets_t) {
  __shared__ int table[256 * 16];  // [digit][wavefront]
  __shared__ int part[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per = ((nnz + 15) / 16 + 63) / 64 * 64;  // pairs per wavefront
  const int lo = wave * per < nnz ? wave * per : nnz;
  const int hi = lo + per < nnz ? lo + per : nnz;
  const int32_t* keys = nullptr;
  const int32_t* vals = nullptr;
  for (int p = 0; p < passes; p++) {
    const int shift = 8 * p;
    int32_t* keys_out = (p & 1) ? keys1 : keys0;
    int32_t* vals_out = (p & 1) ? vals1 : vals0;
    for (int i = tid; i < 256 * 16; i += 1024) table[i] = 0;
    __syncthreads();
    // counts, then first output slot, per (digit, wavefront)
    for (int i0 = lo; i0 < hi; i0 += 64) {
      const int idx = i0 + lane;
      const bool valid = idx < hi;
      const int key = !valid ? 0 : p == 0 ? first_key(row_indices, column_indices, idx) : keys[idx];
      const int digit = (key >> shift) & 255;
      uint64_t same = __ballot(valid);
#pragma unroll
      for (int b = 0; b < 8; b++) {
        const uint64_t bal = __ballot(valid && ((digit >> b) & 1));
        same &= ((digit >> b) & 1) ? bal : ~bal;
      }
      if (valid && (same >> lane) >> 1 == 0) table[digit * 16 + wave] += __popcll(same);  // highest lane of the group
    }
    __syncthreads();
    int mine[4], sum = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) mine[i] = table[4 * tid + i], sum += mine[i];
    int total;
    int run = block_exclusive_scan(sum, part, &total);
#pragma unroll
    for (int i = 0; i < 4; i++) table[4 * tid + i] = run, run += mine[i];
    __syncthreads();
    // scatter: every wavefront walks its pairs in order
    for (int i0 = lo; i0 < hi; i0 += 64) {
      const int idx = i0 + lane;
      const bool valid = idx < hi;
      const int key = !valid ? 0 : p == 0 ? first_key(row_indices, column_indices, idx) : keys[idx];
      const int val = !valid ? 0 : p == 0 ? idx : vals[idx];
      const int digit = (key >> shift) & 255;
      uint64_t same = __ballot(valid);
#pragma unroll
      for (int b = 0; b < 8; b++) {
        const uint64_t bal = __ballot(valid && ((digit >> b) & 1));
        same &= ((digit >> b) & 1) ? bal : ~bal;
      }
      if (valid) {
        const int first = table[digit * 16 + wave];
        const int pos = first + __popcll(same & lanes_below(lane));
        keys_out[pos] = key;
        vals_out[pos] = val;
        if ((same >> lane) >> 1 == 0) table[digit * 16 + wave] = first + __popcll(same);
      }
    }
    __syncthreads();  // the pairs written above are read below and in the next pass by other wavefronts
    keys = keys_out;
    vals = vals_out;
  }
  constexpr bool kPacked = sizeof(IDX) == 2;
  for (int i = tid; i < nnz; i += 1024) {
    const int v = vals[i], key = keys[i];
    block_offsets_t[i] = v;
    column_indices_t[i] = kPacked ? static_cast<IDX>(key >> 16) : row_indices[v];
    // offsets_t[c] = i for every column c behind the one before and up to this one
    const int col = kPacked ? key & 0xffff : key;
    const int before = i == 0 ? -1 : kPacked ? keys[i - 1] & 0xffff : keys[i - 1];
    for (int c = before + 1; c <= col; c++) offsets_t[c] = i;
  }
  const int last = nnz == 0 ? -1 : kPacked ? keys[nnz - 1] & 0xffff : keys[nnz - 1];
  for (int c = last + 1 + tid; c <= block_cols; c += 1024) offsets_t[c] = nnz;
}

template <typename IDX>
static int transpose_meta_impl(const void* row_indices, const void* column_indices, int64_t nnz, int64_t block_cols,
                               void* column_indices_t, int32_t* offsets_t, int32_t* block_offsets_t,
                               void* workspace, hipStream_t s) {
  const int tiles = (int)((nnz + kTile - 1) / kTile);
  int32_t* keys[2] = {static_cast<int32_t*>(workspace), static_cast<int32_t*>(workspace) + nnz};
  int32_t* vals[2] = {keys[1] + nnz, keys[1] + 2 * nnz};
  int32_t* hist = vals[1] + nnz;
  int bits = 0;
  while (bits < 31 && ((int64_t)1 << bits) < block_cols) bits++;
  const int passes = bits <= 8 ? 1 : (bits + 7) / 8;
  if (nnz > 0 && nnz <= kSmallSort && block_cols < INT32_MAX) {
    hipLaunchKernelGGL((transpose_small_kernel<IDX>), dim3(1), dim3(1024), 0, s, static_cast<const IDX*>(row_indices),
                       static_cast<const IDX*>(column_indices), (int)nnz, (int)block_cols, passes, keys[0], keys[1], vals[0], vals[1],
                       static_cast<IDX*>(column_indices_t), offsets_t, block_offsets_t);
    return check_launch("stk_transpose_meta");
  }
  const void* kin = column_indices;
  const int32_t* vin = nullptr;
  for (int p = 0; p < passes && nnz > 0; p++) {
    const int shift = 8 * p;
    int32_t* kout = keys[p & 1];
    int32_t* vout = vals[p & 1];
    if (p == 0) {
      hipLaunchKernelGGL((radix_histogram_kernel<IDX, true>), dim3(tiles), dim3(kWave), 0, s, kin, nnz, shift, tiles, hist);
    } else {
      hipLaunchKernelGGL((radix_histogram_kernel<IDX, false>), dim3(tiles), dim3(kWave), 0, s, kin, nnz, shift, tiles, hist);
    }
    hipLaunchKernelGGL(exclusive_scan_kernel, dim3(1), dim3(1024), 0, s, hist, (int64_t)256 * tiles);
    if (p == 0) {
      hipLaunchKernelGGL((radix_scatter_kernel<IDX, true>), dim3(tiles), dim3(kWave), 0, s, kin, vin, nnz, shift, tiles, hist, kout, vout);
    } else {
      hipLaunchKernelGGL((radix_scatter_kernel<IDX, false>), dim3(tiles), dim3(kWave), 0, s, kin, vin, nnz, shift, tiles, hist, kout, vout);
    }
    kin = kout;
    vin = vout;
  }
  const int64_t work = (nnz > block_cols + 1) ? nnz : block_cols + 1;
  const int grid = (int)((work + 255) / 256 < 4096 ? (work + 255) / 256 : 4096);
  hipLaunchKernelGGL((transpose_finalize_kernel<IDX>), dim3(grid), dim3(256), 0, s, static_cast<const int32_t*>(kin), vin,
                     static_cast<const IDX*>(row_indices), nnz, (int)block_cols, static_cast<IDX*>(column_indices_t),
                     offsets_t, block_offsets_t);
  return check_launch("stk_transpose_meta");
}

// ------------------------------------------------------------ to_dense
__global__ void zero_fill_kernel(unsigned char* __restrict__ out, int64_t bytes) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t t0 = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t n16 = bytes / 16;
  uint4 z = {0u, 0u, 0u, 0u};
  for (int64_t i = t0; i < n16; i += stride) reinterpret_cast<uint4*>(out)[i] = z;
  for (int64_t i = n16 * 16 + t0; i < bytes; i += stride) out[i] = 0;
}

// Moves VEC-element pieces between the blocked and the dense layout.
// TO_DENSE: dense[(r b + i) ld + c b + j] = data[p][i][j]; otherwise the reverse.
template <typename VEC_T, typename IDX, bool TO_DENSE>
__global__ void block_copy_kernel(VEC_T* __restrict__ data, VEC_T* __restrict__ dense, const IDX* __restrict__ row_indices,
                                  const IDX* __restrict__ column_indices, int64_t pieces, int b_vec, int b, int64_t ld_vec) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t per_block = (int64_t)b * b_vec;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < pieces; e += stride) {
    int64_t p = e / per_block;
    int rem = (int)(e - p * per_block);
    int i = rem / b_vec, j = rem - i * b_vec;
    int64_t d = ((int64_t)row_indices[p] * b + i) * ld_vec + (int64_t)column_indices[p] * b_vec + j;
    if constexpr (TO_DENSE) dense[d] = data[e]; else data[e] = dense[d];
  }
}

template <bool TO_DENSE>
static int block_copy(void* data, void* dense, const void* rows, const void* cols, int64_t nnz, int b, int64_t ld,
                      int elem_bytes, int idx32, hipStream_t s) {
  if (nnz == 0) return STK_OK;
  // widest piece (in bytes) that divides a block row and keeps every address aligned
  int vec_bytes = elem_bytes;
  while (vec_bytes < 16 && (b * elem_bytes) % (vec_bytes * 2) == 0 && (ld * elem_bytes) % (vec_bytes * 2) == 0 &&
         (reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(dense)) % (vec_bytes * 2) == 0)
    vec_bytes *= 2;
  const int b_vec = b * elem_bytes / vec_bytes;
  const int64_t ld_vec = ld * elem_bytes / vec_bytes;
  const int64_t pieces = nnz * b * b_vec;
  const int grid = (int)((pieces + 255) / 256 < 65536 ? (pieces + 255) / 256 : 65536);
#define STK_COPY_CASE(BYTES, TYPE)                                                                                  \
  if (vec_bytes == BYTES) {                                                                                         \
    if (idx32)                                                                                                      \
      hipLaunchKernelGGL((block_copy_kernel<TYPE, int32_t, TO_DENSE>), dim3(grid), dim3(256), 0, s, (TYPE*)data,    \
                         (TYPE*)dense, (const int32_t*)rows, (const int32_t*)cols, pieces, b_vec, b, ld_vec);       \
    else                                                                                                            \
      hipLaunchKernelGGL((block_copy_kernel<TYPE, int16_t, TO_DENSE>), dim3(grid), dim3(256), 0, s, (TYPE*)data,    \
                         (TYPE*)dense, (const int16_t*)rows, (const int16_t*)cols, pieces, b_vec, b, ld_vec);       \
  }
  STK_COPY_CASE(2, uint16_t) STK_COPY_CASE(4, uint32_t) STK_COPY_CASE(8, uint2) STK_COPY_CASE(16, uint4)
#undef STK_COPY_CASE
  return check_launch("block copy");
}

// ------------------------------------------------------------ to_sparse
// One wavefront per block: does the block hold any element that is not +-0?
template <typename E>
__global__ __launch_bounds__(256) void block_mask_kernel(const E* __restrict__ x, int64_t ld, int b, int block_cols,
                                                         int64_t blocks, uint8_t* __restrict__ mask) {
  const int lane = threadIdx.x & 63;
  const int64_t wave0 = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  constexpr E kAbs = static_cast<E>(~(E(1) << (sizeof(E) * 8 - 1)));
  for (int64_t blk = wave0; blk < blocks; blk += nwaves) {
    const int64_t r = blk / block_cols, c = blk - r * block_cols;
    const E* base = x + r * b * ld + c * b;
    bool any = false;
    for (int e = lane; e < b * b; e += kWave) {
      int i = e / b, j = e - i * b;
      any |= (base[(int64_t)i * ld + j] & kAbs) != 0;
    }
    uint64_t bal = __ballot(any);
    if (lane == 0) mask[blk] = bal != 0;
  }
}

// The same with 16 bytes per lane, for blocks whose rows are a power-of-two number (at most 64) of aligned
// 16-byte pieces: a wavefront covers 64 >> log2_pieces block rows per load, keeps four and then eight loads in flight,
// and reads no further when the first four loads hold a nonzero element.
template <int ELEM_BYTES>
__global__ __launch_bounds__(256) void block_mask_vec_kernel(const char* __restrict__ x, int64_t ld_bytes, int b, int log2_pieces,
                                                             int block_cols, int64_t blocks, uint8_t* __restrict__ mask) {
  const int lane = threadIdx.x & 63;
  const int64_t wave0 = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  constexpr uint32_t kAbs = ELEM_BYTES == 2 ? 0x7fff7fffu : 0x7fffffffu;   // everything but the sign bits
  const int rows_per_load = 64 >> log2_pieces;
  const int row0 = lane >> log2_pieces;
  const int64_t lane_offset = (int64_t)row0 * ld_bytes + (int64_t)(lane & ((1 << log2_pieces) - 1)) * 16;
  for (int64_t blk = wave0; blk < blocks; blk += nwaves) {
    const int64_t r = blk / block_cols, c = blk - r * block_cols;
    const char* base = x + r * b * ld_bytes + c * (int64_t)b * ELEM_BYTES + lane_offset;
    uint32_t any = 0;
    // The first four loads decide for almost every nonzero block; a block that is zero so far is read to its end,
    // eight loads in flight, with nothing to wait for between the steps.
    auto read = [&](int i0, int loads) {
      uint4 v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int i = i0 + u * rows_per_load + row0;
        v[u] = make_uint4(0u, 0u, 0u, 0u);
        if (u < loads && i < b) v[u] = *reinterpret_cast<const uint4*>(base + (int64_t)(i0 + u * rows_per_load) * ld_bytes);
      }
#pragma unroll
      for (int u = 0; u < 8; u++) any |= (v[u].x | v[u].y | v[u].z | v[u].w) & kAbs;
    };
    read(0, 4);
    if (__ballot(any != 0) == 0)
      for (int i0 = 4 * rows_per_load; i0 < b; i0 += 8 * rows_per_load) read(i0, 8);
    const uint64_t bal = __ballot(any != 0);
    if (lane == 0) mask[blk] = bal != 0;
  }
}

// offsets[0] = 0, offsets[r + 1] = number of nonzero blocks in rows 0..r.  One workgroup; a wavefront counts a
// block row at a time (coalesced reads of the mask), sixteen rows per round, then a scan over the rounds' counts.
__global__ __launch_bounds__(1024) void row_offsets_kernel(const uint8_t* __restrict__ mask, int block_rows, int block_cols,
                                                           int32_t* __restrict__ offsets, int32_t* __restrict__ total_out) {
  __shared__ int part[16];
  __shared__ int counts[1024];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int carry = 0;
  if (threadIdx.x == 0) offsets[0] = 0;
  for (int r0 = 0; r0 < block_rows; r0 += 1024) {
    // rows r0 + wave, r0 + wave + 16, ...: one per wavefront and step
    for (int q = wave; q < 1024 && r0 + q < block_rows; q += 16) {
      int cnt = 0;
      for (int c = lane; c < block_cols; c += kWave) cnt += mask[(int64_t)(r0 + q) * block_cols + c];
      cnt = wave_inclusive_scan(cnt, lane);
      if (lane == kWave - 1) counts[q] = cnt;
    }
    __syncthreads();
    const int r = r0 + threadIdx.x;
    const int cnt = r < block_rows ? counts[threadIdx.x] : 0;
    int total;
    const int ex = block_exclusive_scan(cnt, part, &total);
    if (r < block_rows) offsets[r + 1] = carry + ex + cnt;
    carry += total;
    __syncthreads();
  }
  if (total_out && threadIdx.x == 0) {
    // (may be pinned host memory that the host polls: a system-scope store, made visible at once)
    __hip_atomic_store(total_out, carry, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// One wavefront per block row: nonzero block columns compacted in ascending order.
template <typename IDX>
__global__ __launch_bounds__(256) void block_coordinates_kernel(const uint8_t* __restrict__ mask, const int32_t* __restrict__ offsets,
                                                                int block_rows, int block_cols, IDX* __restrict__ row_indices,
                                                                IDX* __restrict__ column_indices) {
  const int lane = threadIdx.x & 63;
  const int64_t wave0 = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t r = wave0; r < block_rows; r += nwaves) {
    int out = offsets[r];
    for (int c0 = 0; c0 < block_cols; c0 += kWave) {
      int c = c0 + lane;
      bool nz = c < block_cols && mask[r * block_cols + c];
      uint64_t bal = __ballot(nz);
      if (nz) {
        int pos = out + __popcll(bal & lanes_below(lane));
        row_indices[pos] = static_cast<IDX>(r);
        column_indices[pos] = static_cast<IDX>(c);
      }
      out += __popcll(bal);
    }
  }
}

// ------------------------------------------------------------ dMoE topology
// Block-diagonal pattern of a dropless mixture-of-experts layer: expert e owns the
// block rows [first_e, first_e + R_e) given by the padded bins and the `width` block
// columns starting at e * width.  Everything is a closed form of (block row, expert):
//   block p = i * width + j          row_indices[p] = i, column_indices[p] = e(i) * width + j
//   offsets[i] = i * width
//   column c = e * width + j         offsets_t[c] = first_e * width + j * R_e
//   entry r of that column           column_indices_t = first_e + r, block_offsets_t = (first_e + r) * width + j
// which is also what a stable sort by column of the (row, column) pairs gives.
// Expert of a block row: the first bin that ends beyond it (rows past the last bin go to the last expert).
__device__ __forceinline__ int expert_of_row(const int32_t* __restrict__ bins, int experts, int64_t row_end_exclusive_probe) {
  int lo = 0, hi = experts - 1;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (bins[mid] > row_end_exclusive_probe) hi = mid;
    else lo = mid + 1;
  }
  return lo;
}

template <typename IDX>
__global__ __launch_bounds__(256) void dmoe_topology_kernel(
    const int32_t* __restrict__ bins, int experts, int blocking, int block_rows, int width,
    int32_t* __restrict__ offsets, IDX* __restrict__ row_indices, IDX* __restrict__ column_indices,
    int32_t* __restrict__ offsets_t, IDX* __restrict__ column_indices_t, int32_t* __restrict__ block_offsets_t) {
  const int64_t nnz = (int64_t)block_rows * width;
  const int64_t columns = (int64_t)experts * width;
  const int64_t work = nnz > columns + 1 ? nnz : columns + 1;
  for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < work; p += (int64_t)gridDim.x * blockDim.x) {
    if (p < nnz) {
      const int i = (int)(p / width), j = (int)(p % width);
      const int e = expert_of_row(bins, experts, (int64_t)i * blocking);
      int first = e == 0 ? 0 : bins[e - 1] / blocking;
      int last = e == experts - 1 ? block_rows : bins[e] / blocking;  // rows past the last bin stay with the last expert
      if (first > block_rows) first = block_rows;  // bins that claim more rows than exist: stay inside the arrays
      if (last > block_rows) last = block_rows;
      row_indices[p] = (IDX)i;
      column_indices[p] = (IDX)(e * width + j);
      if (j == 0) offsets[i] = i * width;
      const int64_t q = (int64_t)first * width + (int64_t)j * (last - first) + (i - first);
      column_indices_t[q] = (IDX)i;
      block_offsets_t[q] = (int32_t)p;
    }
    if (p <= columns) {
      if (p == columns) {
        offsets_t[p] = (int32_t)nnz;
        offsets[block_rows] = (int32_t)nnz;
      } else {
        const int e = (int)(p / width), j = (int)(p % width);
        int first = e == 0 ? 0 : bins[e - 1] / blocking;
        int last = e == experts - 1 ? block_rows : bins[e] / blocking;
        if (first > block_rows) first = block_rows;
        if (last > block_rows) last = block_rows;
        offsets_t[p] = (int32_t)((int64_t)first * width + (int64_t)j * (last - first));
      }
    }
  }
}

static thread_local char g_error[kErrorBufferBytes] = "";
char* error_buffer() { return g_error; }

}  // namespace stk

using namespace stk;

extern "C" const char* stk_last_error(void) { return error_buffer(); }
extern "C" int stk_abi_version(void) { return STK_AMD_ABI_VERSION; }

extern "C" int stk_stream_capture_id(stk_stream_t stream, uint64_t* id) {
  if (!id) return fail(STK_ERR_DIMS, "stk_stream_capture_id: null output");
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long capture = 0;
  *id = 0;
  const hipError_t e = hipStreamGetCaptureInfo(static_cast<hipStream_t>(stream), &status, &capture);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // the query's own failure is not left behind for the next launch check
    return fail(STK_ERR_HIP, "stk_stream_capture_id: %s", hipGetErrorString(e));
  }
  if (status == hipStreamCaptureStatusActive) *id = capture ? (uint64_t)capture : UINT64_MAX;
  return STK_OK;
}

extern "C" int stk_row_indices(const int32_t* offsets, int64_t block_rows, int64_t nnz, void* out, int index_dtype,
                               stk_stream_t stream) {
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_row_indices: index dtype %d", index_dtype);
  if (block_rows < 0 || nnz < 0 || block_rows > INT32_MAX) return fail(STK_ERR_DIMS, "stk_row_indices: bad size");
  if (nnz == 0) return STK_OK;
  if (block_rows == 0) return fail(STK_ERR_DIMS, "stk_row_indices: %lld blocks but no block rows", (long long)nnz);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int grid = (int)((nnz + 255) / 256 < 65536 ? (nnz + 255) / 256 : 65536);
  if (index_dtype == STK_I32)
    hipLaunchKernelGGL((row_indices_kernel<int32_t>), dim3(grid), dim3(256), 0, s, offsets, (int)block_rows, nnz, static_cast<int32_t*>(out));
  else
    hipLaunchKernelGGL((row_indices_kernel<int16_t>), dim3(grid), dim3(256), 0, s, offsets, (int)block_rows, nnz, static_cast<int16_t*>(out));
  return check_launch("stk_row_indices");
}

extern "C" size_t stk_transpose_meta_workspace_bytes(int64_t nnz) {
  if (nnz < 0) nnz = 0;
  const int64_t tiles = (nnz + kTile - 1) / kTile;
  return static_cast<size_t>(4 * nnz + 256 * tiles + 4) * sizeof(int32_t);
}

extern "C" int stk_transpose_meta(const void* row_indices, const void* column_indices, int64_t nnz, int64_t block_cols,
                                  int index_dtype, void* column_indices_t, int32_t* offsets_t, int32_t* block_offsets_t,
                                  void* workspace, size_t workspace_bytes, stk_stream_t stream) {
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_transpose_meta: index dtype %d", index_dtype);
  if (nnz < 0 || block_cols < 0 || nnz > INT32_MAX || block_cols >= INT32_MAX) return fail(STK_ERR_DIMS, "stk_transpose_meta: bad size");
  if (nnz > 0 && (!workspace || workspace_bytes < stk_transpose_meta_workspace_bytes(nnz)))
    return fail(STK_ERR_WORKSPACE, "stk_transpose_meta: workspace of %zu bytes needed", stk_transpose_meta_workspace_bytes(nnz));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (index_dtype == STK_I32)
    return transpose_meta_impl<int32_t>(row_indices, column_indices, nnz, block_cols, column_indices_t, offsets_t, block_offsets_t, workspace, s);
  return transpose_meta_impl<int16_t>(row_indices, column_indices, nnz, block_cols, column_indices_t, offsets_t, block_offsets_t, workspace, s);
}

extern "C" int stk_to_dense(const void* data, const void* row_indices, const void* column_indices, int64_t nnz, int blocking,
                            int64_t rows, int64_t cols, int elem_bytes, int index_dtype, void* out, stk_stream_t stream) {
  if (elem_bytes != 2 && elem_bytes != 4) return fail(STK_ERR_UNSUPPORTED, "stk_to_dense: element size %d", elem_bytes);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_to_dense: index dtype %d", index_dtype);
  if (blocking <= 0 || rows < 0 || cols < 0 || nnz < 0 || rows % blocking || cols % blocking)
    return fail(STK_ERR_DIMS, "stk_to_dense: [%lld, %lld] is not divisible by blocking %d", (long long)rows, (long long)cols, blocking);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t bytes = rows * cols * elem_bytes;
  if (bytes == 0) return STK_OK;
  const int grid = (int)((bytes / 16 + 255) / 256 < 65536 ? (bytes / 16 + 255) / 256 + 1 : 65536);
  hipLaunchKernelGGL(zero_fill_kernel, dim3(grid), dim3(256), 0, s, static_cast<unsigned char*>(out), bytes);
  int rc = check_launch("stk_to_dense");
  if (rc) return rc;
  return block_copy<true>(const_cast<void*>(data), out, row_indices, column_indices, nnz, blocking, cols, elem_bytes,
                          index_dtype == STK_I32, s);
}

extern "C" int stk_to_sparse_count(const void* x, int64_t rows, int64_t cols, int64_t x_stride, int blocking, int elem_bytes,
                                   uint8_t* mask, int32_t* offsets, stk_stream_t stream) {
  return stk_to_sparse_count_nnz(x, rows, cols, x_stride, blocking, elem_bytes, mask, offsets, nullptr, stream);
}

extern "C" int stk_to_sparse_count_nnz(const void* x, int64_t rows, int64_t cols, int64_t x_stride, int blocking, int elem_bytes,
                                       uint8_t* mask, int32_t* offsets, int32_t* nnz_out, stk_stream_t stream) {
  if (elem_bytes != 2 && elem_bytes != 4) return fail(STK_ERR_UNSUPPORTED, "stk_to_sparse_count: element size %d", elem_bytes);
  if (blocking <= 0 || rows < 0 || cols < 0 || rows % blocking || cols % blocking)
    return fail(STK_ERR_DIMS, "stk_to_sparse_count: [%lld, %lld] is not divisible by blocking %d", (long long)rows, (long long)cols, blocking);
  const int64_t br = rows / blocking, bc = cols / blocking;
  if (br > INT32_MAX || bc > INT32_MAX || (int64_t)blocking * blocking > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "stk_to_sparse_count: size exceeds 32-bit range");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t blocks = br * bc;
  // 16-byte loads when a block row is a power-of-two number (up to 64) of aligned 16-byte pieces
  const int64_t row_bytes = (int64_t)blocking * elem_bytes;
  int log2_pieces = -1;
  if (row_bytes % 16 == 0 && (x_stride * elem_bytes) % 16 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0)
    for (int l = 0; l <= 6; l++)
      if (row_bytes == (16 << l)) log2_pieces = l;
  if (blocks > 0 && log2_pieces >= 0) {
    const int grid = (int)((blocks + 3) / 4 < 262144 ? (blocks + 3) / 4 : 262144);
    if (elem_bytes == 2)
      hipLaunchKernelGGL((block_mask_vec_kernel<2>), dim3(grid), dim3(256), 0, s, static_cast<const char*>(x), x_stride * elem_bytes, blocking,
                         log2_pieces, (int)bc, blocks, mask);
    else
      hipLaunchKernelGGL((block_mask_vec_kernel<4>), dim3(grid), dim3(256), 0, s, static_cast<const char*>(x), x_stride * elem_bytes, blocking,
                         log2_pieces, (int)bc, blocks, mask);
  } else if (blocks > 0) {
    const int grid = (int)((blocks + 3) / 4 < 65536 ? (blocks + 3) / 4 : 65536);
    if (elem_bytes == 2)
      hipLaunchKernelGGL((block_mask_kernel<uint16_t>), dim3(grid), dim3(256), 0, s, static_cast<const uint16_t*>(x), x_stride, blocking, (int)bc, blocks, mask);
    else
      hipLaunchKernelGGL((block_mask_kernel<uint32_t>), dim3(grid), dim3(256), 0, s, static_cast<const uint32_t*>(x), x_stride, blocking, (int)bc, blocks, mask);
  }
  hipLaunchKernelGGL(row_offsets_kernel, dim3(1), dim3(1024), 0, s, mask, (int)br, (int)bc, offsets, nnz_out);
  return check_launch("stk_to_sparse_count");
}

extern "C" int stk_to_sparse_coordinates(int64_t rows, int64_t cols, int blocking, const uint8_t* mask, const int32_t* offsets,
                                         void* row_indices, void* column_indices, int index_dtype, stk_stream_t stream) {
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_to_sparse_coordinates: index dtype %d", index_dtype);
  if (blocking <= 0 || rows < 0 || cols < 0 || rows % blocking || cols % blocking)
    return fail(STK_ERR_DIMS, "stk_to_sparse_coordinates: [%lld, %lld] is not divisible by blocking %d", (long long)rows, (long long)cols, blocking);
  const int64_t br = rows / blocking, bc = cols / blocking;
  if (br == 0 || bc == 0) return STK_OK;
  if (br > INT32_MAX || bc > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "stk_to_sparse_coordinates: size exceeds 32-bit range");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int grid = (int)((br + 3) / 4 < 65536 ? (br + 3) / 4 : 65536);
  if (index_dtype == STK_I32)
    hipLaunchKernelGGL((block_coordinates_kernel<int32_t>), dim3(grid), dim3(256), 0, s, mask, offsets, (int)br, (int)bc,
                       static_cast<int32_t*>(row_indices), static_cast<int32_t*>(column_indices));
  else
    hipLaunchKernelGGL((block_coordinates_kernel<int16_t>), dim3(grid), dim3(256), 0, s, mask, offsets, (int)br, (int)bc,
                       static_cast<int16_t*>(row_indices), static_cast<int16_t*>(column_indices));
  return check_launch("stk_to_sparse_coordinates");
}

extern "C" int stk_to_sparse_gather(const void* x, int64_t rows, int64_t cols, int64_t x_stride, int blocking, int elem_bytes,
                                    const void* row_indices, const void* column_indices, int64_t nnz, int index_dtype, void* data,
                                    stk_stream_t stream) {
  if (elem_bytes != 2 && elem_bytes != 4) return fail(STK_ERR_UNSUPPORTED, "stk_to_sparse_gather: element size %d", elem_bytes);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_to_sparse_gather: index dtype %d", index_dtype);
  if (blocking <= 0 || rows < 0 || cols < 0 || rows % blocking || cols % blocking)
    return fail(STK_ERR_DIMS, "stk_to_sparse_gather: [%lld, %lld] is not divisible by blocking %d", (long long)rows, (long long)cols, blocking);
  if (rows == 0 || cols == 0 || nnz <= 0) return STK_OK;
  return block_copy<false>(data, const_cast<void*>(x), row_indices, column_indices, nnz, blocking, x_stride, elem_bytes,
                           index_dtype == STK_I32, static_cast<hipStream_t>(stream));
}

extern "C" int stk_to_sparse_fill(const void* x, int64_t rows, int64_t cols, int64_t x_stride, int blocking, int elem_bytes,
                                  const uint8_t* mask, const int32_t* offsets, int64_t nnz, void* data, void* row_indices,
                                  void* column_indices, int index_dtype, stk_stream_t stream) {
  if (elem_bytes != 2 && elem_bytes != 4) return fail(STK_ERR_UNSUPPORTED, "stk_to_sparse_fill: element size %d", elem_bytes);
  if (nnz <= 0) return STK_OK;
  const int rc = stk_to_sparse_coordinates(rows, cols, blocking, mask, offsets, row_indices, column_indices, index_dtype, stream);
  if (rc != STK_OK) return rc;
  return stk_to_sparse_gather(x, rows, cols, x_stride, blocking, elem_bytes, row_indices, column_indices, nnz, index_dtype, data, stream);
}

extern "C" int stk_dmoe_topology(const int32_t* padded_bins, int64_t num_experts, int blocking, int64_t block_rows,
                                 int64_t blocks_per_row, int index_dtype, int32_t* offsets, void* row_indices,
                                 void* column_indices, int32_t* offsets_t, void* column_indices_t, int32_t* block_offsets_t,
                                 stk_stream_t stream) {
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_dmoe_topology: index dtype %d", index_dtype);
  if (num_experts <= 0 || blocking <= 0 || block_rows < 0 || blocks_per_row <= 0)
    return fail(STK_ERR_DIMS, "stk_dmoe_topology: %lld experts, blocking %d, %lld block rows of %lld blocks", (long long)num_experts,
                blocking, (long long)block_rows, (long long)blocks_per_row);
  const int64_t nnz = block_rows * blocks_per_row, columns = num_experts * blocks_per_row;
  if (nnz > INT32_MAX || columns >= INT32_MAX || block_rows * blocking > INT32_MAX)
    return fail(STK_ERR_UNSUPPORTED, "stk_dmoe_topology: size exceeds 32-bit range");
  if (index_dtype == STK_I16 && (block_rows > 32767 || columns > 32767))
    return fail(STK_ERR_DIMS, "stk_dmoe_topology: %lld block rows x %lld block columns do not fit 16-bit indices", (long long)block_rows, (long long)columns);
  if (!padded_bins || !offsets || !offsets_t || (nnz > 0 && (!row_indices || !column_indices || !column_indices_t || !block_offsets_t)))
    return fail(STK_ERR_DIMS, "stk_dmoe_topology: missing pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t work = nnz > columns + 1 ? nnz : columns + 1;
  const int grid = (int)((work + 255) / 256 < 65536 ? (work + 255) / 256 : 65536);
  if (index_dtype == STK_I32)
    hipLaunchKernelGGL((dmoe_topology_kernel<int32_t>), dim3(grid), dim3(256), 0, s, padded_bins, (int)num_experts, blocking, (int)block_rows,
                       (int)blocks_per_row, offsets, static_cast<int32_t*>(row_indices), static_cast<int32_t*>(column_indices), offsets_t,
                       static_cast<int32_t*>(column_indices_t), block_offsets_t);
  else
    hipLaunchKernelGGL((dmoe_topology_kernel<int16_t>), dim3(grid), dim3(256), 0, s, padded_bins, (int)num_experts, blocking, (int)block_rows,
                       (int)blocks_per_row, offsets, static_cast<int16_t*>(row_indices), static_cast<int16_t*>(column_indices), offsets_t,
                       static_cast<int16_t*>(column_indices_t), block_offsets_t);
  return check_launch("stk_dmoe_topology");
}
