// float32 values in the three products.
//
// The reference's launchers pass whatever dtype the tensors have to kernels that accumulate in fp32
// (stk/backend/triton_kernels.py:250, 306, 358; ACC_TYPE :248): float32 operands are legal there.  The 16-bit
// tile engine (gemm_core.h) does not take them, so stk_sdd / stk_dsd / stk_dds hand STK_F32 problems to the
// kernels here: one workgroup of four wavefronts per BLK x BLK output tile, v_mfma_f32_32x32x2_f32 on operand
// tiles staged through LDS as [k][m] and [k][n], 16 k at a time, the next K-tile on its way in registers while
// the current one is multiplied.  Operands are read with their element strides as they are (row-major, .t()
// views or anything else), so nothing is copied or converted; ragged dense extents are predicated.  The walks
// are those of the 16-bit kernels.  A plan, a workspace or a block order are ignored: results never depend on them.
#include "common.h"
#include "gemm_core.h"

namespace stk {

namespace f32 {

constexpr int kKT = 16;        // k per staged tile
constexpr int kThreads = 256;  // 2 x 2 wavefronts
constexpr int kPad = 4;        // floats between LDS rows: the staging writes of a K-major tile spread over the banks

typedef float f32x4 __attribute__((ext_vector_type(4)));

// One operand of a K-tile: EXT (m or n extent) x kKT elements at p[mn * s_mn + k * s_k], mn < valid, held by a
// thread as EXT * kKT / kThreads values.  K-major (s_k == 1): consecutive threads run along k; otherwise along mn.
template <int EXT>
struct Staged {
  static constexpr int kPer = EXT * kKT / kThreads;  // 8 (EXT 128) or 4 (EXT 64)
  float v[kPer];
  __device__ __forceinline__ static void place(int i, int tid, bool kmajor, int& mn, int& k) {
    const int e = i * kThreads + tid;
    if (kmajor) mn = e / kKT, k = e % kKT;
    else mn = e % EXT, k = e / EXT;
  }
  __device__ __forceinline__ void load(const float* p, int64_t s_mn, int64_t s_k, int valid, int tid) {
    const bool kmajor = s_k == 1;
#pragma unroll
    for (int i = 0; i < kPer; i++) {
      int mn, k;
      place(i, tid, kmajor, mn, k);
      v[i] = mn < valid ? p[mn * s_mn + k * s_k] : 0.f;
    }
  }
  __device__ __forceinline__ void store(float* lds, int64_t s_k, int tid) const {
    const bool kmajor = s_k == 1;
#pragma unroll
    for (int i = 0; i < kPer; i++) {
      int mn, k;
      place(i, tid, kmajor, mn, k);
      lds[k * (EXT + kPad) + mn] = v[i];
    }
  }
};

template <int BLK>
struct Tile {
  static constexpr int kW = BLK / 64;  // 32x32 MFMA tiles per wavefront in each direction (wave tile BLK/2 x BLK/2)
  static constexpr int kLdsFloats = 2 * kKT * (BLK + kPad);
  f32x16_t acc[kW][kW];

  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int i = 0; i < kW; i++)
#pragma unroll
      for (int j = 0; j < kW; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  }

  // acc += A [BLK x klen] * B [klen x BLK]; A element (m, k) at a[m * a_sm + k * a_sk], B element (k, n) at
  // b[k * b_sk + n * b_sn]; rows >= m_valid of A and columns >= n_valid of B count as zero.  klen is a multiple of kKT.
  __device__ __forceinline__ void accumulate(const float* a, int64_t a_sm, int64_t a_sk, int m_valid,
                                             const float* b, int64_t b_sk, int64_t b_sn, int n_valid, int klen, float* lds) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = (wave & 1) * (BLK / 2), n0 = (wave >> 1) * (BLK / 2);
    float* as = lds;
    float* bs = lds + kKT * (BLK + kPad);
    Staged<BLK> ra, rb;
    ra.load(a, a_sm, a_sk, m_valid, tid);
    rb.load(b, b_sn, b_sk, n_valid, tid);
    for (int k0 = 0; k0 < klen; k0 += kKT) {
      __syncthreads();  // the previous K-tile has been read by every wavefront
      ra.store(as, a_sk, tid);
      rb.store(bs, b_sk, tid);
      __syncthreads();
      if (k0 + kKT < klen) {
        ra.load(a + (int64_t)(k0 + kKT) * a_sk, a_sm, a_sk, m_valid, tid);
        rb.load(b + (int64_t)(k0 + kKT) * b_sk, b_sn, b_sk, n_valid, tid);
      }
#pragma unroll
      for (int ks = 0; ks < kKT; ks += 2) {
        // lane l: element (m or n = l % 32, k = ks + l / 32) of each 32-wide strip
        const int k = ks + (lane >> 5);
        float fa[kW], fb[kW];
#pragma unroll
        for (int i = 0; i < kW; i++) fa[i] = as[k * (BLK + kPad) + m0 + 32 * i + (lane & 31)];
#pragma unroll
        for (int j = 0; j < kW; j++) fb[j] = bs[k * (BLK + kPad) + n0 + 32 * j + (lane & 31)];
        // operands swapped, as in the 16-bit engine: a lane then owns four consecutive columns of one output row
#pragma unroll
        for (int i = 0; i < kW; i++)
#pragma unroll
          for (int j = 0; j < kW; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j], fa[i], acc[i][j], 0, 0, 0);
      }
    }
  }

  // out[m * ldc + n] = act(acc) (* mul[m * ldc + n]) for m < m_valid, n < n_valid; out points at the tile's corner.
  // Lane l holds in acc[i][j][4 g + q] the element (m = 32 i + l % 32, n = 32 j + 8 g + 4 (l / 32) + q) of its wave tile.
  __device__ __forceinline__ void store(float* out, int64_t ldc, int m_valid, int n_valid, int activation, const float* mul) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = (wave & 1) * (BLK / 2), n0 = (wave >> 1) * (BLK / 2);
    const bool vector = (ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15u) == 0) &&
                        (!mul || (reinterpret_cast<uintptr_t>(mul) & 15u) == 0);
#pragma unroll
    for (int i = 0; i < kW; i++)
#pragma unroll
      for (int j = 0; j < kW; j++) {
        if (activation != kNoActivation) activate_all(acc[i][j], activation);
        const int m = m0 + 32 * i + (lane & 31);
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const int n = n0 + 32 * j + 8 * g + 4 * (lane >> 5);
          if (m >= m_valid || n >= n_valid) continue;
          const int64_t at = (int64_t)m * ldc + n;
          f32x4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
          if (vector && n + 4 <= n_valid) {
            if (mul) v *= *reinterpret_cast<const f32x4*>(mul + at);
            *reinterpret_cast<f32x4*>(out + at) = v;
          } else {
#pragma unroll
            for (int q = 0; q < 4; q++)
              if (n + q < n_valid) out[at + q] = mul ? v[q] * mul[at + q] : v[q];
          }
        }
      }
  }
};

struct SddArgs {
  const float* lhs;
  int64_t lsm, lsk;
  const float* rhs;
  int64_t rsk, rsn;
  int k;
  float* out;
  const void* row_indices;
  const void* column_indices;
  int idx32;
  int activation;
  const float* multiplier;
};

template <int BLK>
__global__ __launch_bounds__(kThreads) void sdd_kernel(SddArgs g) {
  __shared__ float lds[Tile<BLK>::kLdsFloats];
  const int64_t p = blockIdx.x;
  const int64_t r = load_index(g.row_indices, p, g.idx32), c = load_index(g.column_indices, p, g.idx32);
  Tile<BLK> t;
  t.clear();
  t.accumulate(g.lhs + r * BLK * g.lsm, g.lsm, g.lsk, BLK, g.rhs + c * BLK * g.rsn, g.rsk, g.rsn, BLK, g.k, lds);
  t.store(g.out + p * BLK * BLK, BLK, BLK, BLK, g.activation, g.multiplier ? g.multiplier + p * BLK * BLK : nullptr);
}

// One line of op(S) against a BLK-wide tile of the dense operand.  SPARSE_LHS: dsd (the line is a block row of op(S),
// the dense operand is the rhs); otherwise dds (the line is a block column, the dense operand is the lhs).
struct WalkArgs {
  const float* data;
  const int32_t* walk_offsets;
  const void* walk_positions;
  const int32_t* walk_blocks;  // indirect block ids, or null: the entry number is the block id
  const float* dense;
  int64_t ds_outer, ds_k;      // dense element strides: along its free dimension (n of the rhs, m of the lhs) and along k
  int64_t bs_mn, bs_k;         // element strides inside a stored block: along the line's own dimension and along k
  float* out;
  int64_t ldc;
  int free_extent;             // n (dsd) or m (dds)
  int idx32;
};

template <int BLK, bool SPARSE_LHS>
__global__ __launch_bounds__(kThreads) void walk_kernel(WalkArgs g) {
  __shared__ float lds[Tile<BLK>::kLdsFloats];
  const int tiles = (g.free_extent + BLK - 1) / BLK;
  const int line = blockIdx.x / tiles, f0 = (blockIdx.x % tiles) * BLK;
  const int valid = g.free_extent - f0 < BLK ? g.free_extent - f0 : BLK;
  Tile<BLK> t;
  t.clear();
  const int begin = g.walk_offsets[line], end = g.walk_offsets[line + 1];
  for (int e = begin; e < end; e++) {
    const int64_t kb = load_index(g.walk_positions, e, g.idx32);
    const float* blk = g.data + (int64_t)(g.walk_blocks ? g.walk_blocks[e] : e) * BLK * BLK;
    const float* dense = g.dense + kb * BLK * g.ds_k + (int64_t)f0 * g.ds_outer;
    if constexpr (SPARSE_LHS) t.accumulate(blk, g.bs_mn, g.bs_k, BLK, dense, g.ds_k, g.ds_outer, valid, BLK, lds);
    else t.accumulate(dense, g.ds_outer, g.ds_k, valid, blk, g.bs_k, g.bs_mn, BLK, BLK, lds);
  }
  if constexpr (SPARSE_LHS) t.store(g.out + (int64_t)line * BLK * g.ldc + f0, g.ldc, BLK, valid, kNoActivation, nullptr);
  else t.store(g.out + (int64_t)f0 * g.ldc + (int64_t)line * BLK, g.ldc, valid, BLK, kNoActivation, nullptr);
}

}  // namespace f32

int sdd_f32(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k, const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
            int64_t m, int64_t k, int64_t n, void* out, const void* row_indices, const void* column_indices, int64_t nnz,
            int blocking, int index_dtype, int activation, const void* multiplier, hipStream_t stream) {
  if (activation < 0 || activation >= kActivations) return fail(STK_ERR_UNSUPPORTED, "stk_sdd: activation %d", activation);
  if (blocking != 64 && blocking != 128) return fail(STK_ERR_UNSUPPORTED, "stk_sdd: blocking %d (64 or 128)", blocking);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_sdd: index dtype %d", index_dtype);
  if (m < 0 || n < 0 || k < 0 || nnz < 0) return fail(STK_ERR_DIMS, "stk_sdd: negative size");
  if (m % blocking || n % blocking || k % 32)
    return fail(STK_ERR_DIMS, "incompatible dimensions: [%lld, %lld] x [%lld, %lld] with blocking %d (m, n must be divisible by the blocking, k by 32)",
                (long long)m, (long long)k, (long long)k, (long long)n, blocking);
  if (k > INT32_MAX || nnz > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "stk_sdd: size exceeds 32-bit range");
  if (nnz == 0) return STK_OK;
  if (!lhs || !rhs || !out || !row_indices || !column_indices) return fail(STK_ERR_DIMS, "stk_sdd: missing pointer");
  const f32::SddArgs g{static_cast<const float*>(lhs), lhs_stride_m, lhs_stride_k, static_cast<const float*>(rhs), rhs_stride_k, rhs_stride_n,
                       (int)k, static_cast<float*>(out), row_indices, column_indices, index_dtype == STK_I32, activation,
                       static_cast<const float*>(multiplier)};
  if (blocking == 128) hipLaunchKernelGGL(f32::sdd_kernel<128>, dim3((unsigned)nnz), dim3(f32::kThreads), 0, stream, g);
  else hipLaunchKernelGGL(f32::sdd_kernel<64>, dim3((unsigned)nnz), dim3(f32::kThreads), 0, stream, g);
  return check_launch("stk_sdd");
}

// dsd (sparse_lhs) or dds on float32 values over the `lines` walked lines of op(S); `free_extent` is n of the rhs (dsd)
// or m of the lhs (dds), with element strides (dense_stride_free, dense_stride_k).  line_major: the rows of a stored
// block run along the walked line's own dimension (dsd of S, dds of S^T); otherwise along k (dsd of S^T, dds of S).
int walk_f32(bool sparse_lhs, const char* who, int64_t lines, int64_t free_extent, const void* data, const int32_t* walk_offsets,
             const void* walk_positions, const int32_t* walk_blocks, bool line_major, const void* dense, int64_t dense_stride_free,
             int64_t dense_stride_k, void* out, int64_t out_stride_m, int64_t nnz, int blocking, int index_dtype, hipStream_t stream) {
  if (blocking != 64 && blocking != 128) return fail(STK_ERR_UNSUPPORTED, "%s: blocking %d (64 or 128)", who, blocking);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "%s: index dtype %d", who, index_dtype);
  if (lines == 0 || free_extent == 0) return STK_OK;
  const int64_t tiles = (free_extent + blocking - 1) / blocking;
  if (lines * tiles > INT32_MAX || free_extent > INT32_MAX) return fail(STK_ERR_UNSUPPORTED, "%s: size exceeds 32-bit range", who);
  if (!walk_offsets || !out || (nnz > 0 && (!walk_positions || !data || !dense))) return fail(STK_ERR_DIMS, "%s: missing metadata pointer", who);
  const int64_t b = blocking;
  const f32::WalkArgs g{static_cast<const float*>(data), walk_offsets, walk_positions, walk_blocks, static_cast<const float*>(dense),
                        dense_stride_free, dense_stride_k, line_major ? b : 1, line_major ? 1 : b,
                        static_cast<float*>(out), out_stride_m, (int)free_extent, index_dtype == STK_I32};
  const dim3 grid((unsigned)(lines * tiles));
  if (sparse_lhs) {
    if (blocking == 128) hipLaunchKernelGGL((f32::walk_kernel<128, true>), grid, dim3(f32::kThreads), 0, stream, g);
    else hipLaunchKernelGGL((f32::walk_kernel<64, true>), grid, dim3(f32::kThreads), 0, stream, g);
  } else {
    if (blocking == 128) hipLaunchKernelGGL((f32::walk_kernel<128, false>), grid, dim3(f32::kThreads), 0, stream, g);
    else hipLaunchKernelGGL((f32::walk_kernel<64, false>), grid, dim3(f32::kThreads), 0, stream, g);
  }
  return check_launch(who);
}

}  // namespace stk
