/*
 * stk_amd.h - C ABI of the MI355X (gfx950) block-sparse matmul backend.
 *
 * The library replaces the kernel layer of stanford-futuredata/stk
 * (stk/backend/triton_kernels.py) and the device work hidden in its format
 * helpers (stk/matrix.py, stk/ops/matrix_ops.py).  Every entry point takes raw
 * device pointers and sizes, launches asynchronously on the given HIP stream
 * (NULL = the default stream) on the current device, allocates nothing that
 * outlives the call, and returns a status code.  All pointers are device
 * pointers unless stated otherwise.  File:line citations name the reference
 * interface each function stands in for.
 *
 * Sparse operands use the reference's hybrid blocked-CSR-COO layout
 * (stk/matrix.py:126-157):
 *   data              [nnz, b, b]   block values, row-major inside a block
 *   row_indices       [nnz]         block row of block p         (int16 or int32)
 *   column_indices    [nnz]         block column of block p      (int16 or int32)
 *   offsets           [Rb + 1]      CSR row pointers             (int32)
 *   column_indices_t  [nnz]         block rows in CSC order      (int16 or int32)
 *   offsets_t         [Cb + 1]      CSC column pointers          (int32)
 *   block_offsets_t   [nnz]         block ids in CSC order       (int32)
 * b (the blocking) is 64 or 128 for the products and any positive value for
 * the format helpers.
 */
#ifndef STK_AMD_H_
#define STK_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define STK_AMD_ABI_VERSION 16

/* status codes */
#define STK_OK 0
#define STK_ERR_DIMS 1        /* shape contract violated: the reference raises AssertionError here */
#define STK_ERR_UNSUPPORTED 2 /* dtype / blocking / stride / alignment this build has no kernel for */
#define STK_ERR_HIP 3         /* a HIP runtime call failed; see stk_last_error() */
#define STK_ERR_WORKSPACE 4   /* workspace pointer missing or too small */

/*
 * Element types of values.  The reference's launchers take whatever dtype the tensors have and accumulate in fp32
 * (stk/backend/triton_kernels.py:250, 306, 358; ACC_TYPE :248).  Here float16 and bfloat16 run on the 16-bit MFMA tile
 * engine; float32 runs on fp32 MFMA kernels of its own (one output block per workgroup, any element strides, no
 * fusion plan or workspace - a compatibility path, not a tuned one).  All three accumulate in fp32 and round once.
 * Anything else is refused with STK_ERR_UNSUPPORTED - nothing is converted silently.  The format helpers (to_dense,
 * to_sparse) take 2- and 4-byte elements.
 */
#define STK_F16 0
#define STK_BF16 1
#define STK_F32 2

/* element types of row/column indices */
#define STK_I16 0
#define STK_I32 1

/* activations of stk_sdd_fused */
#define STK_ACT_NONE 0
#define STK_ACT_RELU 1
#define STK_ACT_GELU_TANH 2 /* 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) */
#define STK_ACT_GELU 3      /* 0.5 x (1 + erf(x / sqrt 2)) */
#define STK_ACT_SILU 4      /* x / (1 + exp(-x)) */
/* the derivatives of the four: with the incoming gradient as the multiplier, stk_sdd_fused then yields the gradient with
 * respect to the sums of a stk_sdd_fused that applied the function, in the one pass that recomputes the sums */
#define STK_ACT_RELU_GRAD 5
#define STK_ACT_GELU_TANH_GRAD 6
#define STK_ACT_GELU_GRAD 7
#define STK_ACT_SILU_GRAD 8

typedef void* stk_stream_t; /* hipStream_t */

/* Message for the last non-zero status returned on the calling thread. */
const char* stk_last_error(void);
int stk_abi_version(void);

/*
 * *id = identifier of the graph capture under way on `stream`, 0 when the stream is not capturing.  No counterpart
 * in the reference (its launches go through Triton, which knows nothing of captures): it is for bindings that cache
 * device buffers between calls, as the Python boundary does with fusion plans and the dsd workspace.  A buffer that
 * is allocated or filled while a capture is under way exists only in that graph's replays, so such a cache must not
 * hand it to launches outside that capture.
 */
int stk_stream_capture_id(stk_stream_t stream, uint64_t* id);

/*
 * Fusion plan of a topology: which neighbouring block rows (and block columns) repeat
 * each other's pattern, so that two of them (for stk_dsd also the last three of an odd
 * run) can be computed together as one tile and share every read of the other operand.
 * No counterpart in the reference; it is derived data like the transpose metadata and
 * depends on (offsets, column_indices, offsets_t, column_indices_t) only, so it can be
 * built once per topology.  plan holds stk_plan_bytes(Rb, Cb, nnz) bytes (4-byte aligned),
 * nnz = offsets[Rb].  It starts with the tiles of stk_sdd: an int32 count, an unused int32
 * and (first block id, rows | columns << 8) pairs - up to 2 (blocking 128) or 4 (blocking
 * 64) neighbouring blocks of a block row, with the blocks below them in up to 2 or 4
 * rows when the next rows repeat this one (with blocking 128 the last three rows of an odd
 * run of identical rows form tiles of 3 rows x 1 block) - row by row, in the order in which
 * workgroups take them.  Behind that: Rb block-row roles and Cb
 * block-column roles (0 alone, 1 computed with the next line, 2 covered by an earlier
 * line), scratch of the same size, the same roles with groups of three (3 = computed with
 * the next two lines), then as int32 ten counts and ten lists of the lines that
 * own a tile (per direction: role 1, role 0, and with groups of three 1, 3, 0), from which
 * stk_dsd and stk_dds take their work, and 2 x 32 bytes of hints for their launches.  The
 * lists are in order of descending length of their lines (lengths above 255 blocks count
 * as 255; ties, and lists of more than 4096 lines, ascend), so that a launch starts its
 * longest walks first wherever they lie in the matrix.
 * A plan built with blocking 64 groups the lines by fours instead of pairs (lists: first lines of groups of four,
 * none, of pairs, of groups of three, lone lines; lines too long for a compute unit's share are cut into pairs); a
 * plan must be passed only to products with the blocking it was built with.
 * Rb / Cb / nnz must be those of the stored matrix whenever the plan is passed to a
 * product (stk_sdd reads the tiles only and also accepts a plan built with Cb = 0).
 * The products accept plan == NULL (no fusion); results do not depend on it.
 */
size_t stk_plan_bytes(int64_t block_rows, int64_t block_cols, int64_t nnz);
int stk_build_plan(const int32_t* offsets, const void* column_indices, int64_t block_rows,
                   const int32_t* offsets_t, const void* column_indices_t, int64_t block_cols,
                   int64_t nnz, int blocking, int index_dtype, uint8_t* plan, size_t plan_bytes, stk_stream_t stream);

/*
 * Sampled dense-dense product: out[p] = lhs[r_p*b:(r_p+1)*b, :] * rhs[:, c_p*b:(c_p+1)*b]
 * for every nonzero block p, fp32 accumulation, result rounded to `dtype`.
 * Replaces sdd(), stk/backend/triton_kernels.py:332-379 (kernel :34-68), called
 * from stk/backend/sputnik.py:263-269.
 *
 * lhs is [m, k] with element strides (lhs_stride_m, lhs_stride_k), rhs is [k, n]
 * with (rhs_stride_k, rhs_stride_n); one stride of each operand must be 1
 * (row-major or a .t() view), the other a multiple of 8, and base pointers
 * 16-byte aligned.  m and n must be multiples of `blocking`, k of 32
 * (triton_kernels.py:15-19) - otherwise STK_ERR_DIMS.  out is [nnz, b, b]
 * contiguous.  Blocks must be stored in CSR order (row_indices ascending), as
 * the format requires.  offsets (CSR row pointers) and plan are optional and only
 * used together, to fuse repeated block rows (m / blocking and nnz must be the Rb and nnz
 * the plan was built with).  block_order, if not NULL, is a
 * permutation of [0, nnz) giving the order in which workgroups visit 64x64
 * blocks; results do not depend on it.
 */
int stk_sdd(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
            const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
            int64_t m, int64_t k, int64_t n,
            void* out, const int32_t* offsets, const void* row_indices, const void* column_indices,
            const int32_t* block_order, int64_t nnz,
            int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream);

/*
 * stk_sdd with the element-wise work on its sparse result done while the result is stored:
 *   out[p] = round(round(act(lhs[r_p rows, :] * rhs[:, c_p columns])) * multiplier[p])
 * act (an STK_ACT_* code) is applied to the fp32 sums, the result is rounded to `dtype`;
 * multiplier, if not NULL, holds the values [nnz, b, b] of a matrix with the same topology
 * (16-byte aligned, same dtype, may be `out` itself only if no other stream reads it), and the
 * product of the two 16-bit values is rounded once more (with one of the derivative codes, whose product with the
 * multiplier is a gradient, the fp32 derivative is multiplied and the product rounded once) - what an activation on the
 * values of the sparse result followed by mul(), stk/ops/eltwise_ops.py:3-28, gives (the reference and its callers
 * run these as separate passes over the values: MoE layers apply the activation to the result of
 * sdd(), stk/ops/linear_ops.py:37-59, and gated layers multiply two such results).  With
 * STK_ACT_NONE and no multiplier it is stk_sdd.  All other arguments as for stk_sdd.
 */
int stk_sdd_fused(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                  const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                  int64_t m, int64_t k, int64_t n,
                  void* out, const int32_t* offsets, const void* row_indices, const void* column_indices,
                  const int32_t* block_order, int64_t nnz,
                  int blocking, int dtype, int index_dtype, const uint8_t* plan,
                  int activation, const void* multiplier, stk_stream_t stream);

/*
 * stk_sdd_fused that also keeps the sums: `sums` (NULL: not kept, the call is stk_sdd_fused), an array laid out like
 * `out` and distinct from it, receives round(lhs * rhs) block by block - what stk_sdd would have stored - while `out`
 * receives the activated and multiplied values.  A training step that keeps them gets the gradient with respect to the
 * sums from stk_activation_product, one pass over the values, instead of from a second product that computes the sums
 * again; it then stores what the reference's callers store (they keep the result of sdd(),
 * stk/ops/linear_ops.py:37-59, for the backward pass of their activation).  16-bit values only.
 */
int stk_sdd_fused_sums(const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                       const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                       int64_t m, int64_t k, int64_t n,
                       void* out, const int32_t* offsets, const void* row_indices, const void* column_indices,
                       const int32_t* block_order, int64_t nnz,
                       int blocking, int dtype, int index_dtype, const uint8_t* plan,
                       int activation, const void* multiplier, void* sums, stk_stream_t stream);

/*
 * out[i] = round(round(act(sums[i])) * factor[i]) for i < count (factor NULL: the first rounding only; a derivative
 * code: round(act'(sums[i]) * factor[i]), one rounding): the element-wise arithmetic of stk_sdd_fused's store applied
 * to stored 16-bit sums.  act is any STK_ACT_* code; with a
 * derivative and the incoming gradient as `factor` this is the gradient with respect to the sums.  count a multiple
 * of 8, arrays 16-byte aligned, `out` may be `factor` or `sums`.  Stands in for the element-wise passes that the
 * reference's callers run in torch on the values of a Matrix (stk/ops/eltwise_ops.py:3-28 is their multiplication).
 */
int stk_activation_product(const void* sums, const void* factor, void* out, int64_t count, int activation, int dtype,
                           stk_stream_t stream);

/*
 * out[m, n] = op(S)[m, k] * rhs[k, n], op = transpose when transpose_a != 0.
 * (m, k) is the logical (already transposed) shape of the sparse operand.
 * Replaces dsd(), stk/backend/triton_kernels.py:222-276 (kernel :83-145), called
 * from stk/backend/sputnik.py:116-126.  Every element of out is written (zero
 * rows where op(S) has no block).  out is row-major with leading dimension
 * out_stride_m.  rhs strides as for stk_sdd.  STK_ERR_DIMS when m, k are not
 * multiples of `blocking` or n is not a multiple of 8.
 * Non-transposed walks offsets / column_indices; transposed walks offsets_t /
 * column_indices_t / block_offsets_t (triton_kernels.py:128-133, 260-262).
 * plan (optional) is the fusion plan of the stored matrix.
 * workspace (optional; no counterpart in the reference; used with a plan only) lets a
 * launch whose tiles would fill the GPU only a few times cut the tiles of its last,
 * partly filled round into slices along k, computed by different workgroups.  It is
 * 256-byte aligned device memory: stk_dsd_workspace_counter_bytes() bytes of counters, which
 * must be zero before the first launch that uses them (every launch that completes leaves
 * them zero), followed by room for partial tiles of stk_dsd_workspace_slot_bytes() bytes
 * each.  stk_dsd_workspace_bytes(m, n, blocking) is the size with which no launch of this
 * shape is limited (0: this shape never uses a workspace); a smaller one is accepted and the
 * last round is cut into fewer slices, or not at all, so that its partial tiles fit.
 * Launches that may overlap need separate workspaces.  With a workspace the sums over k
 * of the sliced tiles are associated differently (fp32), so results can differ in the
 * last bit from those without; they are the same from run to run.  STK_ERR_WORKSPACE
 * when it is misaligned.
 */
int64_t stk_dsd_workspace_bytes(int64_t m, int64_t n, int blocking);
int64_t stk_dsd_workspace_counter_bytes(void);
int64_t stk_dsd_workspace_slot_bytes(void);
/*
 * The rule behind the slice counts that stk_build_plan stores for stk_dsd, evaluated on the
 * host (for inspection and tests): into how many slices along k (1 .. 4) the tiles of the last
 * round are cut, given the tiles of the launch by kind (two block rows x 256 columns, three x
 * 128, one x 256), the average number of blocks per walked line and the compute units.
 */
int stk_dsd_tail_slices(int64_t pair_tiles, int64_t triple_tiles, int64_t single_tiles, double blocks_per_line, int compute_units);
int stk_dsd(int64_t m, int64_t k, int64_t n,
            const void* data, const int32_t* offsets, const void* column_indices,
            const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
            int transpose_a,
            const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
            void* out, int64_t out_stride_m,
            int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan,
            void* workspace, int64_t workspace_bytes, stk_stream_t stream);

/*
 * out[m, n] = lhs[m, k] * op(S)[k, n], op = transpose when transpose_b != 0.
 * (k, n) is the logical shape of the sparse operand.  Replaces dds(),
 * stk/backend/triton_kernels.py:278-330 (kernel :160-220), called from
 * stk/backend/sputnik.py:189-199.  Non-transposed walks offsets_t /
 * column_indices_t / block_offsets_t; transposed walks offsets / column_indices
 * (triton_kernels.py:206-211, 310-320).  plan (optional) is the fusion plan of
 * the stored matrix.
 */
int stk_dds(int64_t m, int64_t k, int64_t n,
            const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
            const void* data, const int32_t* offsets, const void* column_indices,
            const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
            int transpose_b,
            void* out, int64_t out_stride_m,
            int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream);

/*
 * Both operand gradients of a sampled product S = lhs * rhs in one call.  With the incoming gradient dS given as the
 * values `data` of a matrix [m, k] with S's topology,
 *   out_dsd [m, n_dsd]  = S [m, k] * rhs [k, n_dsd]        the gradient with respect to lhs (rhs here = rhs^T there)
 *   out_dds [m_dds, k]  = lhs [m_dds, m] * S [m, k]        the gradient with respect to rhs (lhs here = lhs^T there)
 * Replaces the pair of backend calls in SDD.backward, stk/backend/sputnik.py:274-299 (dsd at :280-288, dds at
 * :289-297), which read dS twice in two launches.  With blocking 128, a plan, rhs as a .t() view of a row-major
 * [n_dsd, k] and lhs as a .t() view of a row-major [m, m_dds] (what the backward pass of a product of two
 * row-major operands passes), n_dsd and m_dds multiples of 256, both products run as one grid: the long tiles of
 * the dsd first, the short tiles of the dds behind them.  Any other case runs stk_dsd (without a workspace) and
 * then stk_dds.  Either way the results are those of stk_dsd without a workspace and of stk_dds, bit for bit.
 * Arguments as for stk_dsd and stk_dds with transpose flags 0.
 */
int stk_dsd_dds(int64_t m, int64_t k,
                const void* data, const int32_t* offsets, const void* column_indices,
                const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                int64_t n_dsd, const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n, void* out_dsd, int64_t out_dsd_stride,
                int64_t m_dds, const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k, void* out_dds, int64_t out_dds_stride,
                int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream);

/*
 * The same pair for a sampled product whose rhs was a .t() view of a row-major [k, n_t'] tensor (weights stored one
 * row per output feature): the gradient with respect to that tensor is wanted in its own layout,
 *   out   [m, n]    = S [m, k] * rhs [k, n]            the gradient with respect to lhs (rhs here = the row-major tensor)
 *   out_t [k, n_t]  = S^T [k, m] * rhs_t [m, n_t]      the gradient with respect to the row-major tensor (rhs_t here = lhs there)
 * two dsd products on the same values, which SDD.backward (stk/backend/sputnik.py:274-299) issues as two backend
 * calls.  With blocking 128, a plan, row-major rhs and rhs_t and n, n_t multiples of 256 they run as one grid (the tiles
 * of the first, then of the second); any other case runs stk_dsd twice (without a workspace).  Either way the results
 * are those of the two stk_dsd calls without a workspace, bit for bit.
 */
int stk_dsd_dsd(int64_t m, int64_t k,
                const void* data, const int32_t* offsets, const void* column_indices,
                const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                int64_t n, const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n, void* out, int64_t out_stride,
                int64_t n_t, const void* rhs_t, int64_t rhs_t_stride_k, int64_t rhs_t_stride_n, void* out_t, int64_t out_t_stride,
                int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream);

/*
 * Both gradients of y = op(S) * rhs in one call.  With the incoming gradient dy and S's topology [m, n],
 *   out_sdd (nnz blocks) = lhs [m, k_sdd] * rhs_sdd [k_sdd, n] on the topology   the gradient with respect to S's values
 *   out_dsd [.., n_dsd]  = op(S) * rhs_dsd [.., n_dsd], S's values in `data`     the gradient with respect to rhs
 * where for op(S) = S the caller passes lhs = dy, rhs_sdd = rhs^T, transpose_a = 1 and rhs_dsd = dy, and for
 * op(S) = S^T lhs = rhs, rhs_sdd = dy^T, transpose_a = 0 and rhs_dsd = dy.  Replaces the pair of backend calls in
 * DSD.backward, stk/backend/sputnik.py:131-155 (sdd at :139-145, dsd at :146-154), which are two launches.  With
 * blocking 128, a plan, more nonzero blocks than compute units, a row-major lhs and rhs_sdd as a .t() view of a
 * row-major [n, k_sdd] with k_sdd a multiple of 64, and a row-major rhs_dsd with n_dsd a multiple of 256, both
 * products run as one grid: the tiles of the sdd first, the tiles of the dsd behind them.  Any other case runs stk_sdd
 * and then stk_dsd (without a workspace).  Either way the results are those of stk_sdd and of stk_dsd without a
 * workspace, bit for bit.  Arguments as for stk_sdd (block_order = block_offsets_t) and stk_dsd.
 */
int stk_sdd_dsd(int64_t m, int64_t n,
                const int32_t* offsets, const void* row_indices, const void* column_indices,
                const int32_t* offsets_t, const void* column_indices_t, const int32_t* block_offsets_t,
                const void* lhs, int64_t lhs_stride_m, int64_t lhs_stride_k,
                const void* rhs_sdd, int64_t rhs_sdd_stride_k, int64_t rhs_sdd_stride_n, int64_t k_sdd, void* out_sdd,
                const void* data, int transpose_a, int64_t n_dsd, const void* rhs_dsd, int64_t rhs_dsd_stride_k, int64_t rhs_dsd_stride_n,
                void* out_dsd, int64_t out_dsd_stride,
                int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan, stk_stream_t stream);

/*
 * COO block-row index from CSR offsets: out[offsets[r] .. offsets[r+1]) = r.
 * Replaces row_indices(), stk/backend/triton_kernels.py:381-393, called from
 * stk/backend/sputnik.py:312.  out has nnz elements of index_dtype.
 */
int stk_row_indices(const int32_t* offsets, int64_t block_rows, int64_t nnz,
                    void* out, int index_dtype, stk_stream_t stream);

/*
 * Transpose (CSC) metadata of a blocked-CSR pattern: a stable sort of the
 * blocks by block column.  Replaces _transpose(), stk/matrix.py:105-123
 * (argsort + gather + histc + cumsum).  Ties keep ascending block id, the
 * order a CSR->CSC conversion gives; the reference's own tie order is
 * unspecified (non-stable argsort, matrix.py:110).
 * workspace must hold stk_transpose_meta_workspace_bytes(nnz) bytes.
 */
size_t stk_transpose_meta_workspace_bytes(int64_t nnz);
int stk_transpose_meta(const void* row_indices, const void* column_indices,
                       int64_t nnz, int64_t block_cols, int index_dtype,
                       void* column_indices_t, int32_t* offsets_t, int32_t* block_offsets_t,
                       void* workspace, size_t workspace_bytes, stk_stream_t stream);

/*
 * Blocked -> dense [rows, cols] row-major with zeros outside the blocks.
 * Replaces to_dense(), stk/ops/matrix_ops.py:36-47 (zeros + scatter_).
 * elem_bytes is 2 or 4.
 */
int stk_to_dense(const void* data, const void* row_indices, const void* column_indices,
                 int64_t nnz, int blocking, int64_t rows, int64_t cols,
                 int elem_bytes, int index_dtype, void* out, stk_stream_t stream);

/*
 * Dense -> blocked, in two phases because nnz depends on the values
 * (stk/ops/matrix_ops.py:64-85; the reference synchronises in torch.nonzero too).
 *   count: mask[Rb*Cb] (uint8, row-major) = block holds an element that is not
 *          +-0 (equivalent to sum(|x|) != 0, matrix_ops.py:50-59), and
 *          offsets[Rb+1] = exclusive scan of the per-row counts.  The caller
 *          reads nnz = offsets[Rb] back and allocates the outputs.
 *   fill:  row_indices / column_indices in row-major order of the nonzero
 *          blocks and data[nnz, b, b] gathered from x; nnz is the value read
 *          back after count.
 * x is [rows, cols] row-major with leading dimension x_stride; elem_bytes 2 or 4.
 * stk_to_sparse_count_nnz also stores nnz at nnz_out (NULL: not stored) as the last thing
 * the launch does, with a system-scope release store; nnz_out may be device memory or pinned
 * host memory that the device can write.  A caller that set the word to a value nnz cannot
 * take (-1) before the call may poll it from the host instead of waiting for the stream;
 * offsets and mask are complete in device memory when the value appears.
 */
int stk_to_sparse_count(const void* x, int64_t rows, int64_t cols, int64_t x_stride,
                        int blocking, int elem_bytes,
                        uint8_t* mask, int32_t* offsets, stk_stream_t stream);
int stk_to_sparse_count_nnz(const void* x, int64_t rows, int64_t cols, int64_t x_stride,
                            int blocking, int elem_bytes,
                            uint8_t* mask, int32_t* offsets, int32_t* nnz_out, stk_stream_t stream);
int stk_to_sparse_fill(const void* x, int64_t rows, int64_t cols, int64_t x_stride,
                       int blocking, int elem_bytes,
                       const uint8_t* mask, const int32_t* offsets, int64_t nnz,
                       void* data, void* row_indices, void* column_indices,
                       int index_dtype, stk_stream_t stream);
/*
 * The two halves of stk_to_sparse_fill on their own.  The coordinates depend on mask and
 * offsets only, not on nnz read back by the host: a caller that has room for Rb*Cb indices
 * can launch them behind the count, before it waits for nnz, and has only the gather of the
 * values left to launch afterwards (row_indices / column_indices: the first nnz entries are
 * written).
 */
int stk_to_sparse_coordinates(int64_t rows, int64_t cols, int blocking,
                              const uint8_t* mask, const int32_t* offsets,
                              void* row_indices, void* column_indices, int index_dtype, stk_stream_t stream);
int stk_to_sparse_gather(const void* x, int64_t rows, int64_t cols, int64_t x_stride,
                         int blocking, int elem_bytes,
                         const void* row_indices, const void* column_indices, int64_t nnz,
                         int index_dtype, void* data, stk_stream_t stream);

/*
 * Topology of a dropless mixture-of-experts layer, built in one launch from the
 * per-expert row counts: the block-diagonal matrix [block_rows * b, num_experts *
 * blocks_per_row * b] in which expert e owns the rows of its bin and the
 * blocks_per_row block columns starting at e * blocks_per_row.  The reference has no
 * builder (its callers assemble these arrays with torch statements, stk.ops.row_indices
 * - stk/ops/matrix_ops.py:96-98 - and the sort in _transpose, stk/matrix.py:105-123);
 * the outputs are the arguments of its Matrix constructor, stk/matrix.py:134-157, with
 * the transpose metadata supplied so that no sort runs.
 * padded_bins[e] (device, int32) = rows of experts 0..e together, every expert padded to
 * a multiple of `blocking`; block_rows * blocking must equal padded_bins[num_experts - 1]
 * (rows beyond it are given to the last expert).  Experts without rows own empty columns.
 * offsets has block_rows + 1 elements, offsets_t num_experts * blocks_per_row + 1, the
 * others nnz = block_rows * blocks_per_row.  Bit-identical to stk_row_indices and
 * stk_transpose_meta applied to the same pattern.
 */
int stk_dmoe_topology(const int32_t* padded_bins, int64_t num_experts, int blocking, int64_t block_rows,
                      int64_t blocks_per_row, int index_dtype,
                      int32_t* offsets, void* row_indices, void* column_indices,
                      int32_t* offsets_t, void* column_indices_t, int32_t* block_offsets_t,
                      stk_stream_t stream);

/*
 * Token routing of a dropless mixture-of-experts layer: the producer of the rows that
 * stk_sdd multiplies and the consumer of the rows that stk_dsd returns.  The reference has
 * no counterpart (its callers sort, count and pad with torch statements and copy the rows
 * with kernels of their own before they build stk.Matrix, stk/matrix.py:134-157); the
 * outputs are defined here.
 *
 * A slot is one (token, choice) pair, s = token * top_k + choice; top_experts[s] (device,
 * int32, 0 <= value < num_experts; values outside are clamped into that range) is the
 * expert it goes to.  stk_route writes
 *   indices[slots]      slot numbers in a stable sort by expert (ties keep ascending s)
 *   bin_ids[slots]      top_experts[indices[i]]
 *   bins[E]             slots of experts 0..e together (inclusive prefix sum)
 *   padded_bins[E]      the same with every expert rounded up to a multiple of `blocking`:
 *                       expert e owns the rows [padded_bins[e-1], padded_bins[e]) of the
 *                       padded layout and fills the first bins[e] - bins[e-1] of them
 *                       (this is the padded_bins argument of stk_dmoe_topology)
 *   slot_rows[slots]    row of slot s in the padded layout:
 *                       slot_rows[indices[i]] = i - bins[e-1] + padded_bins[e-1], e = bin_ids[i]
 *   row_slots[padded_rows]  the inverse: slot held by a row, -1 for a padding row
 * padded_rows is the number of rows the caller gives the padded layout; it must not be
 * below padded_bins[E-1] (rows beyond it are padding, slots beyond it would be dropped from
 * row_slots).  Any multiple of `blocking` that is not below slots + E * (blocking - 1) is safe
 * without reading padded_bins back.  At most 1024 experts.
 * workspace must hold stk_route_workspace_bytes(slots, num_experts) bytes.
 */
size_t stk_route_workspace_bytes(int64_t slots, int64_t num_experts);
int stk_route(const int32_t* top_experts, int64_t slots, int64_t num_experts, int blocking, int64_t padded_rows,
              int32_t* indices, int32_t* bin_ids, int32_t* bins, int32_t* padded_bins,
              int32_t* slot_rows, int32_t* row_slots,
              void* workspace, size_t workspace_bytes, stk_stream_t stream);

/*
 * stk_route for callers that cannot allocate device memory or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the same three launches with the same
 * outputs, bit for bit, but the per-tile table lives in a device array that belongs to the library
 * (STK_ROUTE_STATIC_MAX_ENTRIES int32 entries = 4 MiB on every GPU the library runs on, held until the process
 * ends).  No counterpart in the reference.  The call allocates nothing and frees nothing; the first call on a
 * device resolves the array's address on that device (make it outside a capture).  Sizes with
 * num_experts * ceil(slots / 256) > STK_ROUTE_STATIC_MAX_ENTRIES are refused with STK_ERR_WORKSPACE.  All calls
 * on one GPU share the array: calls that may overlap on one GPU (different streams without an ordering between
 * them) race; calls on one stream, or ordered by events, do not.  The table needs no clearing between calls
 * (every entry that is read is written first).
 */
#define STK_ROUTE_STATIC_MAX_ENTRIES (1 << 20)
int stk_route_static(const int32_t* top_experts, int64_t slots, int64_t num_experts, int blocking, int64_t padded_rows,
                     int32_t* indices, int32_t* bin_ids, int32_t* bins, int32_t* padded_bins,
                     int32_t* slot_rows, int32_t* row_slots, stk_stream_t stream);

/*
 * Rows of x [tokens, cols] copied into the padded layout: out[r] = x[row_slots[r] / top_k],
 * zeros where row_slots[r] < 0.  With weights (fp32, one per slot, or NULL) the row is
 * multiplied by weights[row_slots[r]] in fp32 and rounded once (this is the gradient of
 * stk_padded_scatter with respect to its x).  No counterpart in the reference (see
 * stk_route).  dtype STK_F16 / STK_BF16; cols a multiple of 8, rows 16-byte aligned;
 * strides in elements.
 */
int stk_padded_gather(const void* x, int64_t tokens, int64_t cols, int64_t x_stride,
                      const int32_t* row_slots, const float* weights, int top_k, int64_t padded_rows,
                      void* out, int64_t out_stride, int dtype, stk_stream_t stream);

/*
 * The way back: out[t] = sum over choice = 0 .. top_k-1, in that order, of
 * weights[s] * x[slot_rows[s]], s = t * top_k + choice (weights NULL = all ones).  Products
 * and sums are fp32, each rounded on its own, starting from the first product; the result
 * is rounded once to dtype.  Every output row is written, no atomics: results do not
 * depend on the launch.  It is also the gradient of stk_padded_gather (weights NULL).
 * No counterpart in the reference (see stk_route).
 */
int stk_padded_scatter(const void* x, int64_t padded_rows, int64_t cols, int64_t x_stride,
                       const int32_t* slot_rows, const float* weights, int top_k, int64_t tokens,
                       void* out, int64_t out_stride, int dtype, stk_stream_t stream);

/*
 * Gradient of stk_padded_scatter with respect to its weights:
 * out[s] = <x[slot_rows[s]], grad[s / top_k]> in fp32, grad [tokens, cols].
 * No counterpart in the reference (see stk_route).
 */
int stk_padded_scatter_weight_gradient(const void* x, int64_t padded_rows, int64_t cols, int64_t x_stride,
                                       const void* grad, int64_t grad_stride,
                                       const int32_t* slot_rows, int top_k, int64_t tokens,
                                       float* out, int dtype, stk_stream_t stream);

/*
 * stk_padded_gather (weights NULL) and stk_sdd_fused in one launch: the sampled product of the padded layout's rows
 * with rhs, read straight from the token rows, so that the padded copy of the tokens is neither written nor read.
 *   out (nnz blocks) = act(lhs [m, k] * rhs [k, n]) on the topology,  lhs[r] = tokens[row_slots[r] / top_k],
 * a row of zeros where row_slots[r] is not in [0, num_tokens * top_k).  tokens is [num_tokens, k], row-major with
 * token_stride elements between rows; row_slots has m entries (stk_route writes it).  The other arguments are those of
 * stk_sdd_fused (no block_order, no multiplier; activation one of STK_ACT_NONE .. STK_ACT_SILU, which map the zero
 * rows to zeros).  Bit-identical to the two calls it replaces.  128-blocks only, and the token rows must span less
 * than 4 GiB; STK_ERR_UNSUPPORTED otherwise (callers then make the two calls).  No counterpart in the reference,
 * whose callers gather with their own kernels (see stk_route) in front of sdd, stk/backend/sputnik.py:206-237.
 */
int stk_sdd_gather(const void* tokens, int64_t num_tokens, int64_t token_stride, const int32_t* row_slots, int top_k,
                   const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n, int64_t m, int64_t k, int64_t n,
                   void* out, const int32_t* offsets, const void* row_indices, const void* column_indices, int64_t nnz,
                   int blocking, int dtype, int index_dtype, const uint8_t* plan, int activation, stk_stream_t stream);

/*
 * stk_dsd (sparse operand not transposed) and stk_padded_scatter for top_k = 1 in one launch: the rows of
 * S [m, k] * rhs [k, n] go straight to the token rows they belong to, so that the padded result is neither written
 * nor read.
 *   out[row_slots[r]] = (weights[row_slots[r]] *) (S * rhs)[r]   for every r with row_slots[r] in [0, num_tokens)
 * The sums are rounded to dtype, then multiplied by the fp32 weight and rounded again (weights NULL: not at all),
 * which is what the two calls do; the results are theirs bit for bit.  Rows of `out` that no r names are not
 * written (stk_route with top_k = 1 names every token).  out is [num_tokens, n] with out_stride_m elements between
 * rows.  The other arguments are those of stk_dsd, workspace included.  128-blocks, n a multiple of 256 and a launch
 * that stk_dsd would run on its eight-wavefront tiles only; STK_ERR_UNSUPPORTED otherwise (callers then make the two
 * calls).  No counterpart in the reference (see stk_route); replaces its dsd, stk/backend/sputnik.py:51-120, for
 * this use.
 */
int stk_dsd_scatter(int64_t m, int64_t k, int64_t n, const void* data, const int32_t* offsets, const void* column_indices,
                    const void* rhs, int64_t rhs_stride_k, int64_t rhs_stride_n,
                    const int32_t* row_slots, const float* weights, int64_t num_tokens, void* out, int64_t out_stride_m,
                    int64_t nnz, int blocking, int dtype, int index_dtype, const uint8_t* plan,
                    void* workspace, int64_t workspace_bytes, stk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* STK_AMD_H_ */
