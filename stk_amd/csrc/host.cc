// libstk_amd_host.so: host (CPU) twins of the entry points of libstk_amd.so, for tensors in host memory.
// Plain C++ without any GPU code.  The products pack their operand tiles into contiguous fp32 buffers
// (which is where element types and strides are dealt with), multiply them with one small fp32 routine that
// accumulates in ascending order of k, and round the sums once to the value type.  The index walks are those
// of the device kernels: CSR rows with direct block ids, or CSC columns with block_offsets_t.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "../../include/stk_amd_host.h"

namespace {

thread_local char g_error[512];

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

// ---- 16-bit floating point <-> fp32 ------------------------------------------------------------------------
inline float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
inline uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
inline float bf16_to_float(uint16_t h) { return bits_to_float((uint32_t)h << 16); }
inline uint16_t float_to_bf16(float f) {
  const uint32_t u = float_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // NaN stays NaN (quiet)
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);                    // round to nearest, ties to even
}
inline float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
  if (exp == 0x1fu) return bits_to_float(sign | 0x7f800000u | (man << 13));
  if (exp != 0) return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
  if (man == 0) return bits_to_float(sign);
  // subnormal: man * 2^-24, exact in fp32
  const float v = (float)man * 5.9604644775390625e-8f;
  return sign ? -v : v;
}
inline uint16_t float_to_half(float f) {
  const uint32_t u = float_to_bits(f), sign = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu));  // NaN
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds to infinity (>= 65520), or is infinity
  if (a < 0x33000001u) return (uint16_t)sign;               // <= 2^-25: rounds to zero (the tie 2^-25 goes to even = 0)
  if (a < 0x38800000u) {
    // result is subnormal: value = m * 2^-24 with m = round(|f| * 2^24)
    const int e = (int)(a >> 23);                           // biased exponent, 102 .. 112
    const uint32_t man = (a & 0x7fffffu) | 0x800000u;       // 24-bit significand, |f| = man * 2^(e - 150)
    const int shift = 126 - e;                              // m = man >> shift, shift in 14 .. 24
    const uint32_t q = man >> shift, rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    const uint32_t m = q + ((rem > half || (rem == half && (q & 1u))) ? 1u : 0u);
    return (uint16_t)(sign | m);                            // m may reach 0x400: the smallest normal number
  }
  const uint32_t r = a + 0xfffu + ((a >> 13) & 1u);         // round the 13 dropped bits, ties to even
  return (uint16_t)(sign | ((r - 0x38000000u) >> 13));
}

template <int DTYPE>
struct Value;
template <>
struct Value<STK_F16> {
  typedef uint16_t type;
  static float load(uint16_t v) { return half_to_float(v); }
  static uint16_t store(float f) { return float_to_half(f); }
};
template <>
struct Value<STK_BF16> {
  typedef uint16_t type;
  static float load(uint16_t v) { return bf16_to_float(v); }
  static uint16_t store(float f) { return float_to_bf16(f); }
};
template <>
struct Value<STK_F32> {
  typedef float type;
  static float load(float v) { return v; }
  static float store(float f) { return f; }
};

inline int64_t index_at(const void* p, int64_t i, int index_dtype) {
  return index_dtype == STK_I32 ? (int64_t) static_cast<const int32_t*>(p)[i] : (int64_t) static_cast<const int16_t*>(p)[i];
}
inline void index_put(void* p, int64_t i, int64_t v, int index_dtype) {
  if (index_dtype == STK_I32) static_cast<int32_t*>(p)[i] = (int32_t)v;
  else static_cast<int16_t*>(p)[i] = (int16_t)v;
}

// dst[r][c] (contiguous, `cols` wide) = src[r * stride_r + c * stride_c] as fp32, r < rows, c < cols.
template <int DTYPE>
void pack(float* dst, const void* src, int64_t stride_r, int64_t stride_c, int64_t rows, int64_t cols) {
  typedef typename Value<DTYPE>::type T;
  const T* s = static_cast<const T*>(src);
  for (int64_t r = 0; r < rows; r++)
    for (int64_t c = 0; c < cols; c++) dst[r * cols + c] = Value<DTYPE>::load(s[r * stride_r + c * stride_c]);
}

// acc[mm][nn] += a[mm][kk] * b[kk][nn], all contiguous; every element sums its products in ascending k.
void multiply_add(float* acc, const float* a, const float* b, int64_t mm, int64_t kk, int64_t nn) {
  for (int64_t i = 0; i < mm; i++) {
    float* c = acc + i * nn;
    for (int64_t k = 0; k < kk; k++) {
      const float av = a[i * kk + k];
      const float* br = b + k * nn;
      for (int64_t j = 0; j < nn; j++) c[j] += av * br[j];
    }
  }
}

template <int DTYPE>
void store_tile(void* out, int64_t ld, const float* acc, int64_t rows, int64_t cols) {
  typedef typename Value<DTYPE>::type T;
  T* o = static_cast<T*>(out);
  for (int64_t r = 0; r < rows; r++)
    for (int64_t c = 0; c < cols; c++) o[r * ld + c] = Value<DTYPE>::store(acc[r * cols + c]);
}

constexpr int64_t kChunk = 256;  // extent of the dense operand handled at a time

template <int DTYPE>
void sdd_blocks(const void* lhs, int64_t lsm, int64_t lsk, const void* rhs, int64_t rsk, int64_t rsn, int64_t k,
                void* out, const void* row_indices, const void* column_indices, int64_t nnz, int64_t b, int index_dtype) {
  typedef typename Value<DTYPE>::type T;
#pragma omp parallel
  {
    std::vector<float> a(b * kChunk), bt(kChunk * b), acc(b * b);
#pragma omp for schedule(dynamic)
    for (int64_t p = 0; p < nnz; p++) {
      const int64_t r = index_at(row_indices, p, index_dtype), c = index_at(column_indices, p, index_dtype);
      std::fill(acc.begin(), acc.end(), 0.f);
      for (int64_t k0 = 0; k0 < k; k0 += kChunk) {
        const int64_t kk = std::min(kChunk, k - k0);
        pack<DTYPE>(a.data(), static_cast<const T*>(lhs) + r * b * lsm + k0 * lsk, lsm, lsk, b, kk);
        pack<DTYPE>(bt.data(), static_cast<const T*>(rhs) + k0 * rsk + c * b * rsn, rsk, rsn, kk, b);
        multiply_add(acc.data(), a.data(), bt.data(), b, kk, b);
      }
      store_tile<DTYPE>(static_cast<T*>(out) + p * b * b, b, acc.data(), b, b);
    }
  }
}

// The walk of one line of op(S): entries [begin, end), entry e lies at block position pos(e) of the contraction and
// holds block block(e) of `data`.
struct Walk {
  const int32_t* offsets;
  const void* positions;
  const int32_t* blocks;  // null: the entry number is the block id
  int index_dtype;
  int64_t begin(int64_t line) const { return offsets[line]; }
  int64_t end(int64_t line) const { return offsets[line + 1]; }
  int64_t pos(int64_t e) const { return index_at(positions, e, index_dtype); }
  int64_t block(int64_t e) const { return blocks ? (int64_t)blocks[e] : e; }
};

template <int DTYPE>
void dsd_rows(int64_t block_rows, int64_t n, const void* data, const Walk& w, bool transposed,
              const void* rhs, int64_t rsk, int64_t rsn, void* out, int64_t ldc, int64_t b) {
  typedef typename Value<DTYPE>::type T;
  const int64_t chunks = (n + kChunk - 1) / kChunk;
#pragma omp parallel
  {
    std::vector<float> a(b * b), bt(b * kChunk), acc(b * kChunk);
#pragma omp for schedule(dynamic) collapse(2)
    for (int64_t i = 0; i < block_rows; i++)
      for (int64_t j = 0; j < chunks; j++) {
        const int64_t n0 = j * kChunk, nn = std::min(kChunk, n - n0);
        std::fill(acc.begin(), acc.begin() + b * nn, 0.f);
        for (int64_t e = w.begin(i); e < w.end(i); e++) {
          const T* blk = static_cast<const T*>(data) + w.block(e) * b * b;
          // op(S) block [row][k]: the stored block, or its transpose
          pack<DTYPE>(a.data(), blk, transposed ? 1 : b, transposed ? b : 1, b, b);
          pack<DTYPE>(bt.data(), static_cast<const T*>(rhs) + w.pos(e) * b * rsk + n0 * rsn, rsk, rsn, b, nn);
          multiply_add(acc.data(), a.data(), bt.data(), b, b, nn);
        }
        store_tile<DTYPE>(static_cast<T*>(out) + i * b * ldc + n0, ldc, acc.data(), b, nn);
      }
  }
}

template <int DTYPE>
void dds_columns(int64_t m, int64_t block_cols, const void* lhs, int64_t lsm, int64_t lsk, const void* data, const Walk& w,
                 bool transposed, void* out, int64_t ldc, int64_t b) {
  typedef typename Value<DTYPE>::type T;
  const int64_t chunks = (m + kChunk - 1) / kChunk;
#pragma omp parallel
  {
    std::vector<float> a(kChunk * b), bt(b * b), acc(kChunk * b);
#pragma omp for schedule(dynamic) collapse(2)
    for (int64_t i = 0; i < chunks; i++)
      for (int64_t j = 0; j < block_cols; j++) {
        const int64_t m0 = i * kChunk, mm = std::min(kChunk, m - m0);
        std::fill(acc.begin(), acc.begin() + mm * b, 0.f);
        for (int64_t e = w.begin(j); e < w.end(j); e++) {
          const T* blk = static_cast<const T*>(data) + w.block(e) * b * b;
          pack<DTYPE>(a.data(), static_cast<const T*>(lhs) + m0 * lsm + w.pos(e) * b * lsk, lsm, lsk, mm, b);
          // op(S) block [k][column]: the stored block, or its transpose
          pack<DTYPE>(bt.data(), blk, transposed ? 1 : b, transposed ? b : 1, b, b);
          multiply_add(acc.data(), a.data(), bt.data(), mm, b, b);
        }
        store_tile<DTYPE>(static_cast<T*>(out) + m0 * ldc + j * b, ldc, acc.data(), mm, b);
      }
  }
}

int check_types(const char* who, int blocking, int dtype, int index_dtype) {
  if (blocking <= 0) return fail(STK_ERR_UNSUPPORTED, "%s: blocking %d", who, blocking);
  if (dtype != STK_F16 && dtype != STK_BF16 && dtype != STK_F32) return fail(STK_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "%s: index dtype %d", who, index_dtype);
  return STK_OK;
}

// A block of elem_bytes-wide elements holds one whose bits, the sign bit aside, are not all zero.
template <class U>
bool block_nonzero(const U* x, int64_t stride, int64_t b) {
  const U magnitude = (U) ~((U)1 << (8 * sizeof(U) - 1));
  for (int64_t r = 0; r < b; r++)
    for (int64_t c = 0; c < b; c++)
      if (x[r * stride + c] & magnitude) return true;
  return false;
}

}  // namespace

extern "C" const char* stk_cpu_last_error(void) { return g_error; }

extern "C" int stk_cpu_sdd(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                           const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                           int64_t m, int64_t k, int64_t n,
                           void* out, const void* row_indices, const void* column_indices, int64_t nnz,
                           int blocking, int dtype, int index_dtype) {
  if (const int rc = check_types("stk_cpu_sdd", blocking, dtype, index_dtype)) return rc;
  if (m < 0 || n < 0 || k < 0 || nnz < 0) return fail(STK_ERR_DIMS, "stk_cpu_sdd: negative size");
  if (m % blocking || n % blocking)
    return fail(STK_ERR_DIMS, "incompatible dimensions: [%lld, %lld] x [%lld, %lld] with blocking %d", (long long)m, (long long)k,
                (long long)k, (long long)n, blocking);
  if (nnz == 0) return STK_OK;
  if (!lhs || !rhs || !out || !row_indices || !column_indices) return fail(STK_ERR_DIMS, "stk_cpu_sdd: missing pointer");
  for (int64_t p = 0; p < nnz; p++) {
    const int64_t r = index_at(row_indices, p, index_dtype), c = index_at(column_indices, p, index_dtype);
    if (r < 0 || r >= m / blocking || c < 0 || c >= n / blocking) return fail(STK_ERR_DIMS, "stk_cpu_sdd: block %lld lies outside the matrix", (long long)p);
  }
#define STK_CPU_SDD(D) \
  if (dtype == D) sdd_blocks<D>(lhs, lhs_stride_m, lhs_stride_k, rhs, rhs_stride_k, rhs_stride_n, k, out, row_indices, column_indices, nnz, blocking, index_dtype);
  STK_CPU_SDD(STK_F16) STK_CPU_SDD(STK_BF16) STK_CPU_SDD(STK_F32)
  return STK_OK;
}

// The walk of a product over the lines of op(S) with `lines` lines whose entries address `positions` block positions of
// the contraction; checked against the sizes before anything is read through it.
static int checked_walk(const char* who, const Walk& w, int64_t lines, int64_t positions, int64_t nnz) {
  if (!w.offsets) return fail(STK_ERR_DIMS, "%s: missing metadata pointer", who);
  if (w.offsets[0] != 0 || w.offsets[lines] != nnz) return fail(STK_ERR_DIMS, "%s: offsets do not span the %lld blocks", who, (long long)nnz);
  for (int64_t l = 0; l < lines; l++)
    if (w.offsets[l] > w.offsets[l + 1]) return fail(STK_ERR_DIMS, "%s: offsets decrease at line %lld", who, (long long)l);
  if (nnz > 0 && !w.positions) return fail(STK_ERR_DIMS, "%s: missing metadata pointer", who);
  for (int64_t e = 0; e < nnz; e++) {
    if (w.pos(e) < 0 || w.pos(e) >= positions) return fail(STK_ERR_DIMS, "%s: walk entry %lld lies outside the matrix", who, (long long)e);
    if (w.block(e) < 0 || w.block(e) >= nnz) return fail(STK_ERR_DIMS, "%s: walk entry %lld names block %lld of %lld", who, (long long)e, (long long)w.block(e), (long long)nnz);
  }
  return STK_OK;
}

extern "C" int stk_cpu_dsd(int64_t m, int64_t k, int64_t n,
                           const void* data, const int32_t* offsets, const void* column_indices,
                           const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                           int transpose_a,
                           const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                           void* out, int64_t out_stride_m,
                           int64_t nnz, int blocking, int dtype, int index_dtype) {
  if (const int rc = check_types("stk_cpu_dsd", blocking, dtype, index_dtype)) return rc;
  if (m < 0 || n < 0 || k < 0 || nnz < 0) return fail(STK_ERR_DIMS, "stk_cpu_dsd: negative size");
  if (m % blocking || k % blocking)
    return fail(STK_ERR_DIMS, "incompatible dimensions: sparse [%lld, %lld] x dense [%lld, %lld] with blocking %d", (long long)m,
                (long long)k, (long long)k, (long long)n, blocking);
  if (m == 0 || n == 0) return STK_OK;
  if (transpose_a && nnz > 0 && !block_offsets_t) return fail(STK_ERR_DIMS, "stk_cpu_dsd: missing metadata pointer");
  // non-transposed: CSR rows, entry = block id; transposed: CSC columns with indirect block ids (triton_kernels.py:128-133, 260-262)
  const Walk w = transpose_a ? Walk{offsets_t, column_indices_t, block_offsets_t, index_dtype} : Walk{offsets, column_indices, nullptr, index_dtype};
  if (const int rc = checked_walk("stk_cpu_dsd", w, m / blocking, k / blocking, nnz)) return rc;
  if (!out || (nnz > 0 && (!data || !rhs))) return fail(STK_ERR_DIMS, "stk_cpu_dsd: missing pointer");
#define STK_CPU_DSD(D) \
  if (dtype == D) dsd_rows<D>(m / blocking, n, data, w, transpose_a != 0, rhs, rhs_stride_k, rhs_stride_n, out, out_stride_m, blocking);
  STK_CPU_DSD(STK_F16) STK_CPU_DSD(STK_BF16) STK_CPU_DSD(STK_F32)
  return STK_OK;
}

extern "C" int stk_cpu_dds(int64_t m, int64_t k, int64_t n,
                           const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                           const void* data, const int32_t* offsets, const void* column_indices,
                           const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                           int transpose_b,
                           void* out, int64_t out_stride_m,
                           int64_t nnz, int blocking, int dtype, int index_dtype) {
  if (const int rc = check_types("stk_cpu_dds", blocking, dtype, index_dtype)) return rc;
  if (m < 0 || n < 0 || k < 0 || nnz < 0) return fail(STK_ERR_DIMS, "stk_cpu_dds: negative size");
  if (k % blocking || n % blocking)
    return fail(STK_ERR_DIMS, "incompatible dimensions: dense [%lld, %lld] x sparse [%lld, %lld] with blocking %d", (long long)m,
                (long long)k, (long long)k, (long long)n, blocking);
  if (m == 0 || n == 0) return STK_OK;
  if (!transpose_b && nnz > 0 && !block_offsets_t) return fail(STK_ERR_DIMS, "stk_cpu_dds: missing metadata pointer");
  // non-transposed: CSC columns with indirect block ids; transposed: CSR rows of the stored matrix (triton_kernels.py:206-211, 310-320)
  const Walk w = transpose_b ? Walk{offsets, column_indices, nullptr, index_dtype} : Walk{offsets_t, column_indices_t, block_offsets_t, index_dtype};
  if (const int rc = checked_walk("stk_cpu_dds", w, n / blocking, k / blocking, nnz)) return rc;
  if (!out || (nnz > 0 && (!data || !lhs))) return fail(STK_ERR_DIMS, "stk_cpu_dds: missing pointer");
#define STK_CPU_DDS(D) \
  if (dtype == D) dds_columns<D>(m, n / blocking, lhs, lhs_stride_m, lhs_stride_k, data, w, transpose_b != 0, out, out_stride_m, blocking);
  STK_CPU_DDS(STK_F16) STK_CPU_DDS(STK_BF16) STK_CPU_DDS(STK_F32)
  return STK_OK;
}

extern "C" int stk_cpu_row_indices(const int32_t* offsets, int64_t block_rows, int64_t nnz, void* out, int index_dtype) {
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_cpu_row_indices: index dtype %d", index_dtype);
  if (block_rows < 0 || nnz < 0) return fail(STK_ERR_DIMS, "stk_cpu_row_indices: negative size");
  if (nnz == 0) return STK_OK;
  if (!offsets || !out) return fail(STK_ERR_DIMS, "stk_cpu_row_indices: missing pointer");
  for (int64_t r = 0; r < block_rows; r++) {
    const int64_t lo = offsets[r], hi = offsets[r + 1];
    if (lo < 0 || hi < lo || hi > nnz) return fail(STK_ERR_DIMS, "stk_cpu_row_indices: offsets of row %lld lie outside [0, %lld]", (long long)r, (long long)nnz);
    for (int64_t p = lo; p < hi; p++) index_put(out, p, r, index_dtype);
  }
  return STK_OK;
}

extern "C" int stk_cpu_transpose_meta(const void* row_indices, const void* column_indices, int64_t nnz, int64_t block_cols,
                                      int index_dtype, void* column_indices_t, int32_t* offsets_t, int32_t* block_offsets_t) {
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_cpu_transpose_meta: index dtype %d", index_dtype);
  if (nnz < 0 || block_cols < 0) return fail(STK_ERR_DIMS, "stk_cpu_transpose_meta: negative size");
  if (!offsets_t || (nnz > 0 && (!row_indices || !column_indices || !column_indices_t || !block_offsets_t)))
    return fail(STK_ERR_DIMS, "stk_cpu_transpose_meta: missing pointer");
  // counting sort by block column: a histogram, its exclusive scan, and a scatter in ascending block id (stable)
  std::vector<int32_t> cursor(block_cols + 1, 0);
  for (int64_t p = 0; p < nnz; p++) {
    const int64_t c = index_at(column_indices, p, index_dtype);
    if (c < 0 || c >= block_cols) return fail(STK_ERR_DIMS, "stk_cpu_transpose_meta: block %lld lies in column %lld of %lld", (long long)p, (long long)c, (long long)block_cols);
    cursor[c + 1]++;
  }
  for (int64_t c = 0; c < block_cols; c++) cursor[c + 1] += cursor[c];
  for (int64_t c = 0; c <= block_cols; c++) offsets_t[c] = cursor[c];
  for (int64_t p = 0; p < nnz; p++) {
    const int64_t c = index_at(column_indices, p, index_dtype);
    const int32_t at = cursor[c]++;
    index_put(column_indices_t, at, index_at(row_indices, p, index_dtype), index_dtype);
    block_offsets_t[at] = (int32_t)p;
  }
  return STK_OK;
}

extern "C" int stk_cpu_to_dense(const void* data, const void* row_indices, const void* column_indices,
                                int64_t nnz, int blocking, int64_t rows, int64_t cols,
                                int elem_bytes, int index_dtype, void* out) {
  if (blocking <= 0 || (elem_bytes != 2 && elem_bytes != 4)) return fail(STK_ERR_UNSUPPORTED, "stk_cpu_to_dense: blocking %d, %d-byte elements", blocking, elem_bytes);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_cpu_to_dense: index dtype %d", index_dtype);
  if (rows < 0 || cols < 0 || nnz < 0 || rows % blocking || cols % blocking) return fail(STK_ERR_DIMS, "stk_cpu_to_dense: [%lld, %lld] with blocking %d", (long long)rows, (long long)cols, blocking);
  if (rows == 0 || cols == 0) return STK_OK;
  if (!out || (nnz > 0 && (!data || !row_indices || !column_indices))) return fail(STK_ERR_DIMS, "stk_cpu_to_dense: missing pointer");
  const int64_t b = blocking, row_bytes = b * elem_bytes;
  memset(out, 0, (size_t)(rows * cols * elem_bytes));
  for (int64_t p = 0; p < nnz; p++) {
    const int64_t r = index_at(row_indices, p, index_dtype), c = index_at(column_indices, p, index_dtype);
    if (r < 0 || r >= rows / b || c < 0 || c >= cols / b) return fail(STK_ERR_DIMS, "stk_cpu_to_dense: block %lld lies outside the matrix", (long long)p);
    const char* src = static_cast<const char*>(data) + p * b * row_bytes;
    char* dst = static_cast<char*>(out) + (r * b * cols + c * b) * elem_bytes;
    for (int64_t i = 0; i < b; i++) memcpy(dst + i * cols * elem_bytes, src + i * row_bytes, (size_t)row_bytes);
  }
  return STK_OK;
}

extern "C" int stk_cpu_to_sparse_count(const void* x, int64_t rows, int64_t cols, int64_t x_stride,
                                       int blocking, int elem_bytes, uint8_t* mask, int32_t* offsets) {
  if (blocking <= 0 || (elem_bytes != 2 && elem_bytes != 4)) return fail(STK_ERR_UNSUPPORTED, "stk_cpu_to_sparse_count: blocking %d, %d-byte elements", blocking, elem_bytes);
  if (rows < 0 || cols < 0 || rows % blocking || cols % blocking) return fail(STK_ERR_DIMS, "stk_cpu_to_sparse_count: [%lld, %lld] with blocking %d", (long long)rows, (long long)cols, blocking);
  if (!offsets) return fail(STK_ERR_DIMS, "stk_cpu_to_sparse_count: missing pointer");
  const int64_t b = blocking, br = rows / b, bc = cols / b;
  if (br * bc > 0 && (!x || !mask)) return fail(STK_ERR_DIMS, "stk_cpu_to_sparse_count: missing pointer");
  offsets[0] = 0;
  for (int64_t i = 0; i < br; i++) {
    int32_t count = 0;
    for (int64_t j = 0; j < bc; j++) {
      const int64_t at = i * b * x_stride + j * b;
      const bool nz = elem_bytes == 2 ? block_nonzero(static_cast<const uint16_t*>(x) + at, x_stride, b)
                                      : block_nonzero(static_cast<const uint32_t*>(x) + at, x_stride, b);
      mask[i * bc + j] = nz;
      count += nz;
    }
    offsets[i + 1] = offsets[i] + count;
  }
  return STK_OK;
}

extern "C" int stk_cpu_to_sparse_fill(const void* x, int64_t rows, int64_t cols, int64_t x_stride,
                                      int blocking, int elem_bytes,
                                      const uint8_t* mask, const int32_t* offsets, int64_t nnz,
                                      void* data, void* row_indices, void* column_indices, int index_dtype) {
  if (blocking <= 0 || (elem_bytes != 2 && elem_bytes != 4)) return fail(STK_ERR_UNSUPPORTED, "stk_cpu_to_sparse_fill: blocking %d, %d-byte elements", blocking, elem_bytes);
  if (index_dtype != STK_I16 && index_dtype != STK_I32) return fail(STK_ERR_UNSUPPORTED, "stk_cpu_to_sparse_fill: index dtype %d", index_dtype);
  if (rows < 0 || cols < 0 || nnz < 0 || rows % blocking || cols % blocking) return fail(STK_ERR_DIMS, "stk_cpu_to_sparse_fill: [%lld, %lld] with blocking %d", (long long)rows, (long long)cols, blocking);
  const int64_t b = blocking, br = rows / b, bc = cols / b, row_bytes = b * elem_bytes;
  if (!offsets || offsets[br] != nnz) return fail(STK_ERR_DIMS, "stk_cpu_to_sparse_fill: nnz does not match the offsets");
  if (nnz == 0) return STK_OK;
  if (!x || !mask || !data || !row_indices || !column_indices) return fail(STK_ERR_DIMS, "stk_cpu_to_sparse_fill: missing pointer");
  int64_t p = 0;
  for (int64_t i = 0; i < br; i++)
    for (int64_t j = 0; j < bc; j++) {
      if (!mask[i * bc + j]) continue;
      if (p >= nnz) return fail(STK_ERR_DIMS, "stk_cpu_to_sparse_fill: the mask holds more than nnz blocks");
      index_put(row_indices, p, i, index_dtype);
      index_put(column_indices, p, j, index_dtype);
      const char* src = static_cast<const char*>(x) + (i * b * x_stride + j * b) * elem_bytes;
      char* dst = static_cast<char*>(data) + p * b * row_bytes;
      for (int64_t r = 0; r < b; r++) memcpy(dst + r * row_bytes, src + r * x_stride * elem_bytes, (size_t)row_bytes);
      p++;
    }
  if (p != nnz) return fail(STK_ERR_DIMS, "stk_cpu_to_sparse_fill: the mask holds %lld blocks, not %lld", (long long)p, (long long)nnz);
  return STK_OK;
}
