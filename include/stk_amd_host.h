/*
 * stk_amd_host.h - C ABI of the host (CPU) twins of the block-sparse backend.
 *
 * libstk_amd_host.so holds plain C++ implementations, without any GPU code, of the entry points of
 * stk_amd.h that a caller with tensors in host memory needs: the three products and the format helpers.
 * The reference has no CPU kernels for the products (its Triton kernels need a GPU); its tests build
 * every matrix on the host (stk/ops/linear_ops_test.py:57-63) and its "CPU plumbing" configuration
 * checks products on host tensors against to_dense + torch.matmul (linear_ops_test.py:83-96, 110-111).
 * These functions are what such host tensors are dispatched to; device tensors never come here.
 *
 * Every pointer is a host pointer.  Calls are synchronous and re-entrant; they return the status codes
 * of stk_amd.h, with the message of the last failure on the calling thread behind stk_cpu_last_error().
 * Layouts, argument meaning and the order of arguments are those of the device functions of the same
 * name without the `cpu_`, minus the plan, the workspace and the stream.  Differences:
 *   - values may be STK_F16, STK_BF16 or STK_F32; sums are accumulated in fp32 in ascending order of k
 *     (the accumulator type of the reference's kernels, stk/backend/triton_kernels.py:248, 304, 356)
 *     and rounded once to the value type;
 *   - `blocking` may be any positive number;
 *   - dense operands may have any element strides.
 */
#ifndef STK_AMD_HOST_H_
#define STK_AMD_HOST_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef STK_OK
#define STK_OK 0
#define STK_ERR_DIMS 1
#define STK_ERR_UNSUPPORTED 2
#define STK_F16 0
#define STK_BF16 1
#define STK_F32 2
#define STK_I16 0
#define STK_I32 1
#endif

const char* stk_cpu_last_error(void);

/* sdd(), stk/backend/triton_kernels.py:332-379: out[p] = lhs[block row r_p, :] * rhs[:, block column c_p]. */
int stk_cpu_sdd(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                int64_t m, int64_t k, int64_t n,
                void* out, const void* row_indices, const void* column_indices, int64_t nnz,
                int blocking, int dtype, int index_dtype);

/* dsd(), stk/backend/triton_kernels.py:222-276: out[m, n] = op(S)[m, k] * rhs[k, n]; every element of out is written. */
int stk_cpu_dsd(int64_t m, int64_t k, int64_t n,
                const void* data, const int32_t* offsets, const void* column_indices,
                const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                int transpose_a,
                const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                void* out, int64_t out_stride_m,
                int64_t nnz, int blocking, int dtype, int index_dtype);

/* dds(), stk/backend/triton_kernels.py:278-330: out[m, n] = lhs[m, k] * op(S)[k, n]. */
int stk_cpu_dds(int64_t m, int64_t k, int64_t n,
                const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                const void* data, const int32_t* offsets, const void* column_indices,
                const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                int transpose_b,
                void* out, int64_t out_stride_m,
                int64_t nnz, int blocking, int dtype, int index_dtype);

/* row_indices(), stk/backend/triton_kernels.py:381-393. */
int stk_cpu_row_indices(const int32_t* offsets, int64_t block_rows, int64_t nnz, void* out, int index_dtype);

/* _transpose(), stk/matrix.py:105-123, with the stable tie order (ascending block id inside a block column). */
int stk_cpu_transpose_meta(const void* row_indices, const void* column_indices, int64_t nnz, int64_t block_cols,
                           int index_dtype, void* column_indices_t, int32_t* offsets_t, int32_t* block_offsets_t);

/* to_dense(), stk/ops/matrix_ops.py:36-47.  elem_bytes is 2 or 4. */
int stk_cpu_to_dense(const void* data, const void* row_indices, const void* column_indices,
                     int64_t nnz, int blocking, int64_t rows, int64_t cols,
                     int elem_bytes, int index_dtype, void* out);

/*
 * to_sparse(), stk/ops/matrix_ops.py:64-85, in the two phases of stk_to_sparse_count / stk_to_sparse_fill:
 * mask[Rb*Cb] = the block holds an element whose bits, sign bit aside, are not all zero (for floating-point
 * elements: not +-0, which is sum(|x|) != 0, matrix_ops.py:50-59), offsets = exclusive scan of the row counts;
 * then the coordinates in row-major order and the gathered values.  elem_bytes is 2 or 4.
 */
int stk_cpu_to_sparse_count(const void* x, int64_t rows, int64_t cols, int64_t x_stride,
                            int blocking, int elem_bytes, uint8_t* mask, int32_t* offsets);
int stk_cpu_to_sparse_fill(const void* x, int64_t rows, int64_t cols, int64_t x_stride,
                           int blocking, int elem_bytes,
                           const uint8_t* mask, const int32_t* offsets, int64_t nnz,
                           void* data, void* row_indices, void* column_indices, int index_dtype);

#ifdef __cplusplus
}
#endif
#endif /* STK_AMD_HOST_H_ */
