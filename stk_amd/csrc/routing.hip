// Token routing of a dropless mixture-of-experts layer: the step on either side of the
// block-sparse products.  stk_route sorts the (token, choice) slots by expert with a stable
// counting sort and lays every expert's rows out in a bin padded to the block size;
// stk_padded_gather / stk_padded_scatter move the token rows into that layout and back.
// The index work is bit-exact by construction; the copies move 16 bytes per lane.
#include <atomic>

#include "common.h"
#include "wave_scan.h"

// The scatter's sums are defined with every product and every sum rounded on its own, so this file is
// compiled with -ffp-contract=off (see the Makefile): no fused multiply-add.

namespace stk {

constexpr int kRouteTile = 256;     // consecutive slots owned by one wavefront
constexpr int kMaxExperts = 1024;   // one thread per expert in route_bins_kernel

__device__ __forceinline__ int clamp_expert(int e, int experts) { return e < 0 ? 0 : (e >= experts ? experts - 1 : e); }

// Per-tile slot counts, expert-major: table[e * tiles + tile].  Also marks every row of the padded
// layout as padding; route_scatter_kernel then names the rows that hold a slot.
__global__ __launch_bounds__(kWave) void route_histogram_kernel(const int32_t* __restrict__ top_experts, int64_t slots, int experts,
                                                                int tiles, int32_t* __restrict__ table,
                                                                int32_t* __restrict__ row_slots, int64_t padded_rows) {
  __shared__ int counts[kMaxExperts];
  const int lane = threadIdx.x;
  const int tile = blockIdx.x;
  for (int e = lane; e < experts; e += kWave) counts[e] = 0;
  __syncthreads();
  for (int i = 0; i < kRouteTile / kWave; i++) {
    const int64_t idx = (int64_t)tile * kRouteTile + i * kWave + lane;
    if (idx < slots) atomicAdd(&counts[clamp_expert(top_experts[idx], experts)], 1);
  }
  __syncthreads();
  for (int e = lane; e < experts; e += kWave) table[(int64_t)e * tiles + tile] = counts[e];
  for (int64_t r = (int64_t)tile * kWave + lane; r < padded_rows; r += (int64_t)tiles * kWave) row_slots[r] = -1;
}

// One workgroup.  A wavefront per expert turns the expert's row of the table into an exclusive scan over the
// tiles (= position of the tile's first slot among the expert's slots); the totals give
// bins[e] = slots of experts 0..e and padded_bins[e] = the same with every expert rounded up to a
// multiple of `blocking`.
__global__ __launch_bounds__(1024) void route_bins_kernel(int32_t* __restrict__ table, int experts, int tiles, int blocking,
                                                          int32_t* __restrict__ bins, int32_t* __restrict__ padded_bins) {
  __shared__ int part[16];
  __shared__ int counts[kMaxExperts];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int e = wave; e < experts; e += 16) {
    int32_t* row = table + (int64_t)e * tiles;
    int carry = 0;
    for (int base = 0; base < tiles; base += 4 * kWave) {   // four consecutive tiles per lane
      const int i = base + 4 * lane;
      int v[4], sum = 0;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        v[j] = i + j < tiles ? row[i + j] : 0;
        sum += v[j];
      }
      const int inc = wave_inclusive_scan(sum, lane);
      int run = carry + inc - sum;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        if (i + j < tiles) row[i + j] = run;
        run += v[j];
      }
      carry += __shfl(inc, kWave - 1, kWave);
    }
    if (lane == 0) counts[e] = carry;
  }
  __syncthreads();
  const int e = threadIdx.x;
  const int count = e < experts ? counts[e] : 0;
  const int padded = (count + blocking - 1) / blocking * blocking;
  int total;
  const int before = block_exclusive_scan(count, part, &total);
  const int padded_before = block_exclusive_scan(padded, part, &total);
  if (e < experts) {
    bins[e] = before + count;
    padded_bins[e] = padded_before + padded;
  }
}

// The tile walks its slots in order, 64 at a time; lanes with the same expert find each other with
// `bits` ballots, take consecutive positions in lane order and bump the expert's cursor: a stable sort.
__global__ __launch_bounds__(kWave) void route_scatter_kernel(const int32_t* __restrict__ top_experts, int64_t slots, int experts, int bits,
                                                              int tiles, const int32_t* __restrict__ table,
                                                              const int32_t* __restrict__ bins, const int32_t* __restrict__ padded_bins,
                                                              int32_t* __restrict__ indices, int32_t* __restrict__ bin_ids,
                                                              int32_t* __restrict__ slot_rows, int32_t* __restrict__ row_slots,
                                                              int64_t padded_rows) {
  __shared__ int cursor[kMaxExperts];
  __shared__ int shift[kMaxExperts];   // row in the padded layout minus sorted position, per expert
  const int lane = threadIdx.x;
  const int tile = blockIdx.x;
  for (int e = lane; e < experts; e += kWave) {
    const int first = e ? bins[e - 1] : 0;
    cursor[e] = first + table[(int64_t)e * tiles + tile];
    shift[e] = (e ? padded_bins[e - 1] : 0) - first;
  }
  __syncthreads();
  for (int i = 0; i < kRouteTile / kWave; i++) {
    const int64_t idx = (int64_t)tile * kRouteTile + i * kWave + lane;
    const bool valid = idx < slots;
    const int e = valid ? clamp_expert(top_experts[idx], experts) : 0;
    uint64_t same = __ballot(valid);
    for (int b = 0; b < bits; b++) {
      const uint64_t bal = __ballot(valid && ((e >> b) & 1));
      same &= ((e >> b) & 1) ? bal : ~bal;
    }
    int pos = 0;
    if (valid) pos = cursor[e] + __popcll(same & lanes_below(lane));
    __syncthreads();
    if (valid) {
      const int row = pos + shift[e];
      indices[pos] = (int)idx;
      bin_ids[pos] = e;
      slot_rows[idx] = row;
      if (row < padded_rows) row_slots[row] = (int)idx;
      if ((same >> lane) >> 1 == 0) cursor[e] += __popcll(same);  // highest lane of the group
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- row copies
// Eight 16-bit elements.
struct alignas(16) Pack8 { uint32_t w[4]; };

template <int DTYPE> __device__ __forceinline__ float to_float(uint16_t h);
template <> __device__ __forceinline__ float to_float<STK_BF16>(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
template <> __device__ __forceinline__ float to_float<STK_F16>(uint16_t h) { return static_cast<float>(__builtin_bit_cast(_Float16, h)); }

// Round to nearest, ties to even.
template <int DTYPE> __device__ __forceinline__ uint16_t from_float(float f);
template <> __device__ __forceinline__ uint16_t from_float<STK_BF16>(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);  // quiet NaN
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
template <> __device__ __forceinline__ uint16_t from_float<STK_F16>(float f) {
  // The fp32 value is final here: without this the compiler merges the multiplication before it and this
  // conversion into one mixed-precision instruction, which does not round the product to fp32 first.
  asm volatile("" : "+v"(f));
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

// acc[j] += w * element j of p, as a separately rounded product and sum.
template <int DTYPE>
__device__ __forceinline__ void accumulate(float (&acc)[8], float w, const Pack8& p) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    acc[2 * j] = __fadd_rn(acc[2 * j], __fmul_rn(w, to_float<DTYPE>((uint16_t)(p.w[j] & 0xffffu))));
    acc[2 * j + 1] = __fadd_rn(acc[2 * j + 1], __fmul_rn(w, to_float<DTYPE>((uint16_t)(p.w[j] >> 16))));
  }
}
// acc[j] = w * element j of p.
template <int DTYPE>
__device__ __forceinline__ void product(float (&acc)[8], float w, const Pack8& p) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    acc[2 * j] = __fmul_rn(w, to_float<DTYPE>((uint16_t)(p.w[j] & 0xffffu)));
    acc[2 * j + 1] = __fmul_rn(w, to_float<DTYPE>((uint16_t)(p.w[j] >> 16)));
  }
}
template <int DTYPE>
__device__ __forceinline__ Pack8 pack(const float (&acc)[8]) {
  Pack8 p;
#pragma unroll
  for (int j = 0; j < 4; j++) p.w[j] = (uint32_t)from_float<DTYPE>(acc[2 * j]) | ((uint32_t)from_float<DTYPE>(acc[2 * j + 1]) << 16);
  return p;
}

// Copies a row of cols8 16-byte pieces with the whole wavefront, two loads in flight per lane.
__device__ __forceinline__ void copy_row(Pack8* __restrict__ dst, const Pack8* __restrict__ src, int cols8, int lane) {
  int c = lane;
  for (; c + kWave < cols8; c += 2 * kWave) {
    const Pack8 a = src[c], b = src[c + kWave];
    dst[c] = a;
    dst[c + kWave] = b;
  }
  for (; c < cols8; c += kWave) dst[c] = src[c];
}

// One wavefront per row of the padded layout: out[r] = (weights[s]) * x[s / top_k] for the slot s that
// lives in row r, zeros for a padding row.  cols8 = columns / 8.
template <int DTYPE, bool WEIGHTED>
__global__ __launch_bounds__(256) void padded_gather_kernel(const uint16_t* __restrict__ x, int64_t x_stride,
                                                            const int32_t* __restrict__ row_slots, const float* __restrict__ weights,
                                                            int top_k, int64_t slots, int64_t rows, int cols8,
                                                            uint16_t* __restrict__ out, int64_t out_stride) {
  const int lane = threadIdx.x & 63;
  const int64_t waves = (int64_t)gridDim.x * (blockDim.x >> 6);
  for (int64_t r = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); r < rows; r += waves) {
    const int s = row_slots[r];
    Pack8* dst = reinterpret_cast<Pack8*>(out + r * out_stride);
    if (s < 0 || s >= slots) {
      for (int c = lane; c < cols8; c += kWave) dst[c] = Pack8{{0u, 0u, 0u, 0u}};
      continue;
    }
    const Pack8* src = reinterpret_cast<const Pack8*>(x + (int64_t)(s / top_k) * x_stride);
    if constexpr (WEIGHTED) {
      const float w = weights[s];
      for (int c = lane; c < cols8; c += kWave) {
        float acc[8];
        product<DTYPE>(acc, w, src[c]);
        dst[c] = pack<DTYPE>(acc);
      }
    } else {
      copy_row(dst, src, cols8, lane);
    }
  }
}

// A token whose TOP_K rows all exist: rows and weights are read once, then the columns are walked with
// the TOP_K loads of a piece in flight together.  Same operations in the same order as the general loop.
template <int DTYPE, bool WEIGHTED, int TOP_K>
__device__ __forceinline__ void scatter_token(const uint16_t* __restrict__ x, int64_t x_stride, const int32_t* __restrict__ slot_rows,
                                              const float* __restrict__ weights, int64_t t, int cols8, int lane, Pack8* __restrict__ dst) {
  const Pack8* src[TOP_K];
  float w[TOP_K];
#pragma unroll
  for (int k = 0; k < TOP_K; k++) {
    src[k] = reinterpret_cast<const Pack8*>(x + (int64_t)slot_rows[t * TOP_K + k] * x_stride);
    w[k] = WEIGHTED ? weights[t * TOP_K + k] : 1.0f;
  }
  int c = lane;
  for (; c + kWave < cols8; c += 2 * kWave) {   // two pieces per lane: 2 TOP_K loads in flight
    Pack8 p[TOP_K], q[TOP_K];
#pragma unroll
    for (int k = 0; k < TOP_K; k++) {
      p[k] = src[k][c];
      q[k] = src[k][c + kWave];
    }
    float acc[8], acd[8];
    product<DTYPE>(acc, w[0], p[0]);
    product<DTYPE>(acd, w[0], q[0]);
#pragma unroll
    for (int k = 1; k < TOP_K; k++) {
      accumulate<DTYPE>(acc, w[k], p[k]);
      accumulate<DTYPE>(acd, w[k], q[k]);
    }
    dst[c] = pack<DTYPE>(acc);
    dst[c + kWave] = pack<DTYPE>(acd);
  }
  for (; c < cols8; c += kWave) {
    Pack8 p[TOP_K];
#pragma unroll
    for (int k = 0; k < TOP_K; k++) p[k] = src[k][c];
    float acc[8];
    product<DTYPE>(acc, w[0], p[0]);
#pragma unroll
    for (int k = 1; k < TOP_K; k++) accumulate<DTYPE>(acc, w[k], p[k]);
    dst[c] = pack<DTYPE>(acc);
  }
}

template <int TOP_K>
__device__ __forceinline__ bool all_rows_exist(const int32_t* __restrict__ slot_rows, int64_t t, int64_t rows) {
  bool ok = true;
#pragma unroll
  for (int k = 0; k < TOP_K; k++) {
    const int row = slot_rows[t * TOP_K + k];
    ok = ok && row >= 0 && row < rows;
  }
  return ok;
}

// One wavefront per token: out[t] = sum over its top_k choices, in that order, of
// (weights[s]) * x[slot_rows[s]], s = t * top_k + choice; fp32 products and sums, each rounded on its
// own (no fused multiply-add), starting from the first product; one rounding to 16 bits at the end.
template <int DTYPE, bool WEIGHTED>
__global__ __launch_bounds__(256) void padded_scatter_kernel(const uint16_t* __restrict__ x, int64_t x_stride,
                                                             const int32_t* __restrict__ slot_rows, const float* __restrict__ weights,
                                                             int top_k, int64_t tokens, int64_t rows, int cols8,
                                                             uint16_t* __restrict__ out, int64_t out_stride) {
  const int lane = threadIdx.x & 63;
  const int64_t waves = (int64_t)gridDim.x * (blockDim.x >> 6);
  for (int64_t t = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); t < tokens; t += waves) {
    Pack8* dst = reinterpret_cast<Pack8*>(out + t * out_stride);
    if (top_k == 1 && !WEIGHTED) {
      const int row = slot_rows[t];
      if (row >= 0 && row < rows) {
        copy_row(dst, reinterpret_cast<const Pack8*>(x + (int64_t)row * x_stride), cols8, lane);
      } else {
        for (int c = lane; c < cols8; c += kWave) dst[c] = Pack8{{0u, 0u, 0u, 0u}};
      }
      continue;
    }
    if (top_k == 2 && all_rows_exist<2>(slot_rows, t, rows)) {
      scatter_token<DTYPE, WEIGHTED, 2>(x, x_stride, slot_rows, weights, t, cols8, lane, dst);
      continue;
    }
    if (top_k == 4 && all_rows_exist<4>(slot_rows, t, rows)) {
      scatter_token<DTYPE, WEIGHTED, 4>(x, x_stride, slot_rows, weights, t, cols8, lane, dst);
      continue;
    }
    for (int c = lane; c < cols8; c += kWave) {
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      bool first = true;
      for (int k = 0; k < top_k; k++) {
        const int64_t s = t * top_k + k;
        const int row = slot_rows[s];
        if (row < 0 || row >= rows) continue;
        const float w = WEIGHTED ? weights[s] : 1.0f;
        const Pack8 p = reinterpret_cast<const Pack8*>(x + (int64_t)row * x_stride)[c];
        if (first) product<DTYPE>(acc, w, p); else accumulate<DTYPE>(acc, w, p);
        first = false;
      }
      dst[c] = pack<DTYPE>(acc);
    }
  }
}

// One wavefront per slot: out[s] = <x[slot_rows[s]], grad[s / top_k]>, fp32 (the gradient of
// stk_padded_scatter with respect to weights[s]).
template <int DTYPE>
__global__ __launch_bounds__(256) void scatter_weight_gradient_kernel(const uint16_t* __restrict__ x, int64_t x_stride,
                                                                      const uint16_t* __restrict__ grad, int64_t grad_stride,
                                                                      const int32_t* __restrict__ slot_rows, int top_k, int64_t slots,
                                                                      int64_t rows, int cols8, float* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int64_t waves = (int64_t)gridDim.x * (blockDim.x >> 6);
  for (int64_t s = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); s < slots; s += waves) {
    const int row = slot_rows[s];
    float sum = 0.f;
    if (row >= 0 && row < rows) {
      const Pack8* a = reinterpret_cast<const Pack8*>(x + (int64_t)row * x_stride);
      const Pack8* g = reinterpret_cast<const Pack8*>(grad + (s / top_k) * grad_stride);
      for (int c = lane; c < cols8; c += kWave) {
        const Pack8 pa = a[c], pg = g[c];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          sum += to_float<DTYPE>((uint16_t)(pa.w[j] & 0xffffu)) * to_float<DTYPE>((uint16_t)(pg.w[j] & 0xffffu));
          sum += to_float<DTYPE>((uint16_t)(pa.w[j] >> 16)) * to_float<DTYPE>((uint16_t)(pg.w[j] >> 16));
        }
      }
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) sum += __shfl_xor(sum, d, kWave);
    if (lane == 0) out[s] = sum;
  }
}

static int copy_grid(int64_t lines) {
  const int64_t groups = (lines + 3) / 4;
  return (int)(groups < 1 ? 1 : (groups < 262144 ? groups : 262144));
}

static int check_rows(const char* who, const void* p, int64_t stride, int64_t cols) {
  if (cols % 8) return fail(STK_ERR_UNSUPPORTED, "%s: %lld columns are not a multiple of 8", who, (long long)cols);
  if (!aligned16(p) || stride % 8 || stride < cols)
    return fail(STK_ERR_UNSUPPORTED, "%s: rows must start at multiples of 16 bytes (stride %lld)", who, (long long)stride);
  return STK_OK;
}

}  // namespace stk

using namespace stk;

extern "C" size_t stk_route_workspace_bytes(int64_t slots, int64_t num_experts) {
  if (slots < 0) slots = 0;
  if (num_experts < 1) num_experts = 1;
  const int64_t tiles = (slots + kRouteTile - 1) / kRouteTile;
  return static_cast<size_t>(num_experts * (tiles > 0 ? tiles : 1)) * sizeof(int32_t);
}

// Argument checks shared by the two routing entry points.
static int route_check(const char* who, const int32_t* top_experts, int64_t slots, int64_t num_experts, int blocking, int64_t padded_rows,
                       const int32_t* indices, const int32_t* bin_ids, const int32_t* bins, const int32_t* padded_bins,
                       const int32_t* slot_rows, const int32_t* row_slots) {
  if (slots < 0 || num_experts <= 0 || blocking <= 0 || padded_rows < 0)
    return fail(STK_ERR_DIMS, "%s: %lld slots, %lld experts, blocking %d, %lld rows", who, (long long)slots, (long long)num_experts,
                blocking, (long long)padded_rows);
  if (num_experts > kMaxExperts) return fail(STK_ERR_UNSUPPORTED, "%s: at most %d experts", who, kMaxExperts);
  if (slots + num_experts * (int64_t)blocking > INT32_MAX || padded_rows > INT32_MAX)
    return fail(STK_ERR_UNSUPPORTED, "%s: size exceeds 32-bit range", who);
  if (!bins || !padded_bins || (slots > 0 && (!top_experts || !indices || !bin_ids || !slot_rows)) || (padded_rows > 0 && !row_slots))
    return fail(STK_ERR_DIMS, "%s: missing pointer", who);
  return STK_OK;
}

// The three launches of a routing; `table` holds stk_route_workspace_bytes(slots, num_experts) bytes.  Every entry of
// the table that is read is written first (the histogram writes a count for every expert of every tile), so the
// table needs no initial value.
static void route_launch(const int32_t* top_experts, int64_t slots, int64_t num_experts, int blocking, int64_t padded_rows,
                         int32_t* indices, int32_t* bin_ids, int32_t* bins, int32_t* padded_bins, int32_t* slot_rows, int32_t* row_slots,
                         int32_t* table, hipStream_t s) {
  const int real_tiles = (int)((slots + kRouteTile - 1) / kRouteTile);
  const int tiles = real_tiles > 0 ? real_tiles : 1;   // one tile without slots still clears its counts and row_slots
  int bits = 0;
  while (((int64_t)1 << bits) < num_experts) bits++;
  hipLaunchKernelGGL(route_histogram_kernel, dim3(tiles), dim3(kWave), 0, s, top_experts, slots, (int)num_experts, tiles, table,
                     row_slots, padded_rows);
  hipLaunchKernelGGL(route_bins_kernel, dim3(1), dim3(1024), 0, s, table, (int)num_experts, tiles, blocking, bins, padded_bins);
  if (slots > 0)
    hipLaunchKernelGGL(route_scatter_kernel, dim3(tiles), dim3(kWave), 0, s, top_experts, slots, (int)num_experts, bits, tiles, table,
                       bins, padded_bins, indices, bin_ids, slot_rows, row_slots, padded_rows);
}

extern "C" int stk_route(const int32_t* top_experts, int64_t slots, int64_t num_experts, int blocking, int64_t padded_rows,
                         int32_t* indices, int32_t* bin_ids, int32_t* bins, int32_t* padded_bins,
                         int32_t* slot_rows, int32_t* row_slots, void* workspace, size_t workspace_bytes, stk_stream_t stream) {
  const int rc = route_check("stk_route", top_experts, slots, num_experts, blocking, padded_rows, indices, bin_ids, bins, padded_bins,
                             slot_rows, row_slots);
  if (rc != STK_OK) return rc;
  if (!workspace || workspace_bytes < stk_route_workspace_bytes(slots, num_experts))
    return fail(STK_ERR_WORKSPACE, "stk_route: workspace of %zu bytes needed", stk_route_workspace_bytes(slots, num_experts));
  route_launch(top_experts, slots, num_experts, blocking, padded_rows, indices, bin_ids, bins, padded_bins, slot_rows, row_slots,
               static_cast<int32_t*>(workspace), static_cast<hipStream_t>(stream));
  return check_launch("stk_route");
}

// ---------------------------------------------------------------- routing without a workspace argument
// The table of stk_route kept in device memory that belongs to the library: one array per GPU, there from the moment
// the code object is loaded until the process ends.  Host code never uses the array's name as an address: its
// address on a device is asked for once, with that device current, and kept.
namespace stk {
constexpr size_t kRouteScratchBytes = STK_ROUTE_STATIC_MAX_ENTRIES * sizeof(int32_t);
static __device__ __align__(256) unsigned char route_scratch[kRouteScratchBytes];
constexpr int kMaxDevices = 64;
static std::atomic<void*> route_scratch_of_device[kMaxDevices];

// Address of route_scratch on the current device (null with the error set when it cannot be had).
static void* route_scratch_address() {
  int dev = -1;
  const hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail(STK_ERR_HIP, "stk_route_static: no usable current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "device index out of range");
    return nullptr;
  }
  void* p = route_scratch_of_device[dev].load(std::memory_order_acquire);
  if (p) return p;
  const hipError_t r = hipGetSymbolAddress(&p, HIP_SYMBOL(route_scratch));
  if (r != hipSuccess || !p) {
    fail(STK_ERR_HIP, "stk_route_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(r));
    return nullptr;
  }
  route_scratch_of_device[dev].store(p, std::memory_order_release);   // every thread that asks gets the same answer
  return p;
}
}  // namespace stk

extern "C" int stk_route_static(const int32_t* top_experts, int64_t slots, int64_t num_experts, int blocking, int64_t padded_rows,
                                int32_t* indices, int32_t* bin_ids, int32_t* bins, int32_t* padded_bins,
                                int32_t* slot_rows, int32_t* row_slots, stk_stream_t stream) {
  const int rc = route_check("stk_route_static", top_experts, slots, num_experts, blocking, padded_rows, indices, bin_ids, bins,
                             padded_bins, slot_rows, row_slots);
  if (rc != STK_OK) return rc;
  const size_t need = stk_route_workspace_bytes(slots, num_experts);
  if (need > kRouteScratchBytes)
    return fail(STK_ERR_WORKSPACE,
                "stk_route_static: %lld slots over %lld experts need a table of %zu bytes, the built-in one holds %zu "
                "(experts x ceil(slots / %d) <= %d); use stk_route with a workspace",
                (long long)slots, (long long)num_experts, need, kRouteScratchBytes, kRouteTile, STK_ROUTE_STATIC_MAX_ENTRIES);
  void* table = route_scratch_address();
  if (!table) return STK_ERR_HIP;
  route_launch(top_experts, slots, num_experts, blocking, padded_rows, indices, bin_ids, bins, padded_bins, slot_rows, row_slots,
               static_cast<int32_t*>(table), static_cast<hipStream_t>(stream));
  return check_launch("stk_route_static");
}

extern "C" int stk_padded_gather(const void* x, int64_t tokens, int64_t cols, int64_t x_stride, const int32_t* row_slots,
                                 const float* weights, int top_k, int64_t padded_rows, void* out, int64_t out_stride, int dtype,
                                 stk_stream_t stream) {
  if (dtype != STK_F16 && dtype != STK_BF16) return fail(STK_ERR_UNSUPPORTED, "stk_padded_gather: dtype %d", dtype);
  if (tokens < 0 || cols < 0 || top_k <= 0 || padded_rows < 0)
    return fail(STK_ERR_DIMS, "stk_padded_gather: %lld tokens x %lld, top_k %d, %lld rows", (long long)tokens, (long long)cols, top_k,
                (long long)padded_rows);
  if (tokens * top_k > INT32_MAX || cols / 8 > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "stk_padded_gather: size exceeds 32-bit range");
  if (padded_rows == 0 || cols == 0) return STK_OK;
  if (!row_slots || !out || (tokens > 0 && !x)) return fail(STK_ERR_DIMS, "stk_padded_gather: missing pointer");
  int rc = check_rows("stk_padded_gather", out, out_stride, cols);
  if (!rc && tokens > 0) rc = check_rows("stk_padded_gather", x, x_stride, cols);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t* xs = static_cast<const uint16_t*>(x);
  uint16_t* os = static_cast<uint16_t*>(out);
  const int64_t slots = tokens * top_k;
  const int grid = copy_grid(padded_rows), c8 = (int)(cols / 8);
  if (!weights)
    hipLaunchKernelGGL((padded_gather_kernel<STK_BF16, false>), dim3(grid), dim3(256), 0, s, xs, x_stride, row_slots, weights, top_k, slots,
                       padded_rows, c8, os, out_stride);
  else if (dtype == STK_BF16)
    hipLaunchKernelGGL((padded_gather_kernel<STK_BF16, true>), dim3(grid), dim3(256), 0, s, xs, x_stride, row_slots, weights, top_k, slots,
                       padded_rows, c8, os, out_stride);
  else
    hipLaunchKernelGGL((padded_gather_kernel<STK_F16, true>), dim3(grid), dim3(256), 0, s, xs, x_stride, row_slots, weights, top_k, slots,
                       padded_rows, c8, os, out_stride);
  return check_launch("stk_padded_gather");
}

extern "C" int stk_padded_scatter(const void* x, int64_t padded_rows, int64_t cols, int64_t x_stride, const int32_t* slot_rows,
                                  const float* weights, int top_k, int64_t tokens, void* out, int64_t out_stride, int dtype,
                                  stk_stream_t stream) {
  if (dtype != STK_F16 && dtype != STK_BF16) return fail(STK_ERR_UNSUPPORTED, "stk_padded_scatter: dtype %d", dtype);
  if (tokens < 0 || cols < 0 || top_k <= 0 || padded_rows < 0)
    return fail(STK_ERR_DIMS, "stk_padded_scatter: %lld tokens x %lld, top_k %d, %lld rows", (long long)tokens, (long long)cols, top_k,
                (long long)padded_rows);
  if (tokens * top_k > INT32_MAX || cols / 8 > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "stk_padded_scatter: size exceeds 32-bit range");
  if (tokens == 0 || cols == 0) return STK_OK;
  if (!slot_rows || !out || (padded_rows > 0 && !x)) return fail(STK_ERR_DIMS, "stk_padded_scatter: missing pointer");
  int rc = check_rows("stk_padded_scatter", out, out_stride, cols);
  if (!rc && padded_rows > 0) rc = check_rows("stk_padded_scatter", x, x_stride, cols);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t* xs = static_cast<const uint16_t*>(x);
  uint16_t* os = static_cast<uint16_t*>(out);
  const int grid = copy_grid(tokens), c8 = (int)(cols / 8);
#define STK_SCATTER(D, W) \
  hipLaunchKernelGGL((padded_scatter_kernel<D, W>), dim3(grid), dim3(256), 0, s, xs, x_stride, slot_rows, weights, top_k, tokens, padded_rows, \
                     c8, os, out_stride)
  if (dtype == STK_BF16) { if (weights) STK_SCATTER(STK_BF16, true); else STK_SCATTER(STK_BF16, false); }
  else { if (weights) STK_SCATTER(STK_F16, true); else STK_SCATTER(STK_F16, false); }
#undef STK_SCATTER
  return check_launch("stk_padded_scatter");
}

extern "C" int stk_padded_scatter_weight_gradient(const void* x, int64_t padded_rows, int64_t cols, int64_t x_stride,
                                                  const void* grad, int64_t grad_stride, const int32_t* slot_rows, int top_k,
                                                  int64_t tokens, float* out, int dtype, stk_stream_t stream) {
  const char* who = "stk_padded_scatter_weight_gradient";
  if (dtype != STK_F16 && dtype != STK_BF16) return fail(STK_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
  if (tokens < 0 || cols < 0 || top_k <= 0 || padded_rows < 0)
    return fail(STK_ERR_DIMS, "%s: %lld tokens x %lld, top_k %d, %lld rows", who, (long long)tokens, (long long)cols, top_k, (long long)padded_rows);
  if (tokens * top_k > INT32_MAX || cols / 8 > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "%s: size exceeds 32-bit range", who);
  if (tokens == 0) return STK_OK;
  if (!slot_rows || !out || !grad || (padded_rows > 0 && !x)) return fail(STK_ERR_DIMS, "%s: missing pointer", who);
  int rc = check_rows(who, grad, grad_stride, cols);
  if (!rc && padded_rows > 0) rc = check_rows(who, x, x_stride, cols);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t slots = tokens * top_k;
  const int grid = copy_grid(slots), c8 = (int)(cols / 8);
  if (dtype == STK_BF16)
    hipLaunchKernelGGL((scatter_weight_gradient_kernel<STK_BF16>), dim3(grid), dim3(256), 0, s, static_cast<const uint16_t*>(x), x_stride,
                       static_cast<const uint16_t*>(grad), grad_stride, slot_rows, top_k, slots, padded_rows, c8, out);
  else
    hipLaunchKernelGGL((scatter_weight_gradient_kernel<STK_F16>), dim3(grid), dim3(256), 0, s, static_cast<const uint16_t*>(x), x_stride,
                       static_cast<const uint16_t*>(grad), grad_stride, slot_rows, top_k, slots, padded_rows, c8, out);
  return check_launch(who);
}
