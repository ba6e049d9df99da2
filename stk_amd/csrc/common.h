// Host-side helpers shared by the C ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/stk_amd.h"

// Pipeline shape of the 128-block kernels: K-tile length and number of LDS stages
// (STAGES - 1 K-tiles are in flight while one is being multiplied).
#ifndef STK_SDD_KT
#define STK_SDD_KT 32
#define STK_SDD_STAGES 4
#endif
#ifndef STK_SDD_PERSISTENT
#define STK_SDD_PERSISTENT 1   // stk_sdd with a plan: one workgroup per compute unit that walks the tile list
#endif
#ifndef STK_DSD_KT
#define STK_DSD_KT 32
#define STK_DSD_STAGES 4
#endif
#ifndef STK_DSD_BK_KT
#define STK_DSD_BK_KT 64   // K-major dense operand
#define STK_DSD_BK_STAGES 2
#endif
#ifndef STK_DSD_T_KT
#define STK_DSD_T_KT 32
#define STK_DSD_T_STAGES 4
#endif
#ifndef STK_DDS_KT
#define STK_DDS_KT 32
#define STK_DDS_STAGES 4
#endif

// Large dense results (dsd, dds) are written with non-temporal stores, so that they do not displace the
// operands from the caches.
#ifndef STK_STREAM_STORES
#define STK_STREAM_STORES true
#endif

namespace stk {

// Per-thread message behind stk_last_error().
char* error_buffer();
constexpr int kErrorBufferBytes = 512;

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), kErrorBufferBytes, fmt, ap);
  va_end(ap);
  return code;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(STK_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return STK_OK;
}

// float32 values (fp32.hip): the products hand STK_F32 problems to these.
int sdd_f32(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k, const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
            int64_t m, int64_t k, int64_t n, void* out, const void* row_indices, const void* column_indices, int64_t nnz,
            int blocking, int index_dtype, int activation, const void* multiplier, hipStream_t stream);
int walk_f32(bool sparse_lhs, const char* who, int64_t lines, int64_t free_extent, const void* data, const int32_t* walk_offsets,
             const void* walk_positions, const int32_t* walk_blocks, bool line_major, const void* dense, int64_t dense_stride_free,
             int64_t dense_stride_k, void* out, int64_t out_stride_m, int64_t nnz, int blocking, int index_dtype, hipStream_t stream);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Layout of a fusion plan (see plan.hip).  First the tiles of stk_sdd (their size depends on the block
// rows and the blocks only, so that stk_sdd finds the rest without knowing for how many block columns
// the plan was built): int32 count, int32 unused, then (block id, block id below or -1) pairs in the
// order in which workgroups take them.  Behind that
// (plan_body()): pair roles of the block rows and block columns, scratch of the same size, roles with
// groups of three, then int32 counts[2][kPlanLists] and the lists [2][kPlanLists][lines].
__host__ __device__ inline int64_t sdd_max_tiles(int64_t block_rows, int64_t nnz) { return (nnz + block_rows + 1) / 2; }
__host__ __device__ inline size_t plan_sdd_bytes(int64_t block_rows, int64_t nnz) {
  return static_cast<size_t>(8 + 8 * sdd_max_tiles(block_rows, nnz));
}
inline const uint8_t* plan_body(const uint8_t* plan, int64_t block_rows, int64_t nnz) { return plan + plan_sdd_bytes(block_rows, nnz); }
constexpr int kPlanLists = 5;
enum PlanList { kPairs = 0, kSingles = 1, kTallPairs = 2, kTallTriples = 3, kTallSingles = 4 };
__host__ __device__ inline size_t plan_list_offset(int64_t block_rows, int64_t block_cols) {
  return static_cast<size_t>((3 * (block_rows + block_cols) + 3) / 4 * 4);
}
// Behind the lists: per direction kPlanHintBytes bytes of hints for the launches.  Bytes 0 .. kTailSliceColumns - 1:
// entry t = slices (1 .. kMaxTailSlices) along k for the tiles of the last round of a stk_dsd launch whose dense
// operand has 256 (t + 1) columns (wider: as 256 * 16).  Byte kSpreadHint: 1 when equal eighths of the lines hold
// unequal numbers of blocks (read by the dsd with a sliced last round, see xcd_share()).
// Bytes kGroupHint .. kGroupHint + kPlanLists - 1: for each list, how many consecutive entries go to one compute die
// at a time (see xcd_item()).  Bytes kStripeHint, kStripeHint + 1 (plans for 128-blocks): from how many 128-wide tiles
// of the dense operand on the launches that give every line a tile of its own deal their tiles to the compute dies by
// stripes of the dense operand instead of by lines (0: never), for the lists of threes / pairs / lone lines and for the
// lists of pairs / lone lines.  By lines, a die fetches the dense panel of every block of its lines (G panels in all, G =
// the blocks of one line per group of identical lines) and every sparse block once; by stripes, a die fetches its
// stripe of every panel (K panels in all, K = the lines of the other direction) and every sparse block: stripes move
// less when 1024 nnz + K w < 128 nnz + G w for a dense operand of w 256-byte columns, w > 896 nnz / (G - K).
constexpr int kTailSliceColumns = 16;
constexpr int kSpreadHint = 16;
constexpr int kGroupHint = 17;
constexpr int kStripeHint = 22;
constexpr int kPlanHintBytes = 32;
constexpr int kMaxTailSlices = 4;
__host__ __device__ inline size_t plan_slices_offset(int64_t block_rows, int64_t block_cols) {
  return plan_list_offset(block_rows, block_cols) + sizeof(int32_t) * static_cast<size_t>(kPlanLists * (2 + block_rows + block_cols));
}
// Lists of one direction of a plan: count[k] lines in list[k], k a PlanList.
struct PlanLists {
  const int32_t* counts;
  const int32_t* lists;
  int lines;
  const uint8_t* hints;  // kPlanHintBytes of this direction
  __host__ __device__ const int32_t* list(int k) const { return lists + (int64_t)k * lines; }
  // entries of list k that go to one compute die at a time (a wave-uniform, scalar read)
  __device__ int group(int k) const {
    typedef const __attribute__((address_space(4))) int32_t* words_t;
    const int at = kGroupHint + k;
    const int e = (((words_t)(uintptr_t)hints)[at >> 2] >> (8 * (at & 3))) & 0xff;
    return e > 0 ? e : 1;
  }
  // 128-wide tiles of the dense operand from which on a launch over lone lines deals by stripes; 0: never
  __device__ int stripe_from(bool tall) const {
    typedef const __attribute__((address_space(4))) int32_t* words_t;
    const int at = kStripeHint + (tall ? 0 : 1);
    return (((words_t)(uintptr_t)hints)[at >> 2] >> (8 * (at & 3))) & 0xff;
  }
};
inline PlanLists plan_lists_of(const uint8_t* plan, int64_t block_rows, int64_t block_cols, bool columns) {
  const int32_t* base = reinterpret_cast<const int32_t*>(plan + plan_list_offset(block_rows, block_cols));
  return PlanLists{base + (columns ? kPlanLists : 0), base + 2 * kPlanLists + (columns ? kPlanLists * block_rows : 0),
                   (int)(columns ? block_cols : block_rows), plan + plan_slices_offset(block_rows, block_cols) + (columns ? kPlanHintBytes : 0)};
}

// Launches with less work than this per compute unit (in products of one 128-block with 128 columns or rows of
// the dense operand) run on four-wave 128x128 tiles, two workgroups per compute unit: with so few, short tiles
// the start and the stores of a workgroup are what counts, and a second workgroup on the unit hides them
// (config 2, 4096^2 with 256 blocks: dsd 58 -> 53 us, dds 62 -> 52 us).
#ifndef STK_SMALL_WORK_PER_UNIT
#define STK_SMALL_WORK_PER_UNIT 40
#endif
constexpr int64_t kSmallWorkPerUnit = STK_SMALL_WORK_PER_UNIT;

// Compute units of the current device (0 when it cannot be asked).
inline int compute_units() {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  return cus;
}

// Kernels whose tiles need more dynamic LDS than the default limit say so once.
template <class Kernel>
inline void set_lds_limit(Kernel kernel, int bytes) {
  if (bytes > 60000) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

// Read-only metadata read through the constant address space: wave-uniform loads become scalar loads.
typedef const __attribute__((address_space(4))) int32_t* cint_t;
__device__ __forceinline__ cint_t const_ints(const void* p) { return (cint_t)(uintptr_t)p; }

// Entry i of an index array through the scalar unit (a wave-uniform i; 16-bit entries are read as halves of 32-bit
// words, so the array must start at a multiple of four bytes).
__device__ __forceinline__ int scalar_index(const void* p, int i, int idx32) {
  if (idx32) return const_ints(p)[i];
  return (int)(int16_t)(const_ints(p)[i >> 1] >> (16 * (i & 1)));
}

__device__ __forceinline__ int load_index(const void* __restrict__ p, int64_t i, int idx32) {
  return idx32 ? static_cast<const int32_t*>(p)[i] : static_cast<int>(static_cast<const int16_t*>(p)[i]);
}

}  // namespace stk
