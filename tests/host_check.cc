// Sanitizer harness for the host library (stk_amd/csrc/host.cc): built together with that source under
// -fsanitize=address,undefined by tests/test_host_products.py.  Every operand, output and metadata array lives in a heap
// allocation of exactly its size, so an access one element outside any of them is reported.  Results are checked
// against dense loops written here (fp32 operands, double sums).
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <random>
#include <vector>

#include "../include/stk_amd_host.h"

static int g_failures = 0;
#define CHECK(cond, ...)                 \
  do {                                   \
    if (!(cond)) {                       \
      printf("FAILED %s:%d: ", __FILE__, __LINE__); \
      printf(__VA_ARGS__);               \
      printf("\n");                      \
      g_failures++;                      \
    }                                    \
  } while (0)

struct Pattern {
  int64_t rows, cols, b, br, bc, nnz;
  std::vector<uint8_t> mask;            // [br * bc]
  std::vector<float> dense;             // [rows * cols], zeros outside the blocks
};

static Pattern make_pattern(std::mt19937& rng, int64_t br, int64_t bc, int64_t b, double density) {
  Pattern p{br * b, bc * b, b, br, bc, 0, std::vector<uint8_t>(br * bc), std::vector<float>(br * b * bc * b, 0.f)};
  std::uniform_real_distribution<double> u(0.0, 1.0);
  std::normal_distribution<float> g(0.f, 1.f);
  for (int64_t i = 0; i < br; i++)
    for (int64_t j = 0; j < bc; j++) {
      // (row 1 and column 2 stay empty when they exist: zero-length walks)
      const bool on = u(rng) < density && !(br > 2 && i == 1) && !(bc > 3 && j == 2);
      p.mask[i * bc + j] = on;
      p.nnz += on;
      if (on)
        for (int64_t r = 0; r < b; r++)
          for (int64_t c = 0; c < b; c++) {
            float v = g(rng);
            if (v == 0.f) v = 1.f;
            p.dense[(i * b + r) * p.cols + j * b + c] = v;
          }
    }
  return p;
}

template <class I>
struct Sparse {
  std::vector<float> data;
  std::vector<I> row, col, col_t;
  std::vector<int32_t> offsets, offsets_t, block_offsets_t;
};

template <class I>
static void run_case(std::mt19937& rng, int64_t br, int64_t bc, int64_t b, double density, int64_t n, int index_dtype) {
  const Pattern p = make_pattern(rng, br, bc, b, density);
  std::normal_distribution<float> g(0.f, 1.f);
  // ---- to_sparse in two phases
  std::vector<uint8_t> mask(br * bc ? br * bc : 1);
  Sparse<I> s;
  s.offsets.resize(br + 1);
  int rc = stk_cpu_to_sparse_count(p.dense.data(), p.rows, p.cols, p.cols, (int)b, 4, mask.data(), s.offsets.data());
  CHECK(rc == STK_OK, "to_sparse_count: %s", stk_cpu_last_error());
  CHECK(s.offsets[br] == p.nnz, "nnz %d vs %lld", s.offsets[br], (long long)p.nnz);
  for (int64_t i = 0; i < br * bc; i++) CHECK(mask[i] == p.mask[i], "mask[%lld]", (long long)i);
  const int64_t nnz = p.nnz;
  s.data.resize(nnz * b * b);
  s.row.resize(nnz);
  s.col.resize(nnz);
  rc = stk_cpu_to_sparse_fill(p.dense.data(), p.rows, p.cols, p.cols, (int)b, 4, mask.data(), s.offsets.data(), nnz, s.data.data(),
                              s.row.data(), s.col.data(), index_dtype);
  CHECK(rc == STK_OK, "to_sparse_fill: %s", stk_cpu_last_error());
  // ---- row_indices and transpose metadata
  std::vector<I> row2(nnz);
  rc = stk_cpu_row_indices(s.offsets.data(), br, nnz, row2.data(), index_dtype);
  CHECK(rc == STK_OK, "row_indices: %s", stk_cpu_last_error());
  for (int64_t q = 0; q < nnz; q++) CHECK(row2[q] == s.row[q], "row_indices[%lld]", (long long)q);
  s.col_t.resize(nnz);
  s.offsets_t.resize(bc + 1);
  s.block_offsets_t.resize(nnz);
  rc = stk_cpu_transpose_meta(s.row.data(), s.col.data(), nnz, bc, index_dtype, s.col_t.data(), s.offsets_t.data(), s.block_offsets_t.data());
  CHECK(rc == STK_OK, "transpose_meta: %s", stk_cpu_last_error());
  {
    // CSC order: columns ascending, rows ascending inside a column
    int64_t at = 0;
    for (int64_t j = 0; j < bc; j++) {
      CHECK(s.offsets_t[j] == at, "offsets_t[%lld]", (long long)j);
      for (int64_t i = 0; i < br; i++)
        if (p.mask[i * bc + j]) {
          CHECK(s.col_t[at] == (I)i, "column_indices_t[%lld]", (long long)at);
          const int32_t q = s.block_offsets_t[at];
          CHECK(q >= 0 && q < nnz && s.row[q] == (I)i && s.col[q] == (I)j, "block_offsets_t[%lld]", (long long)at);
          at++;
        }
    }
    CHECK(s.offsets_t[bc] == nnz, "offsets_t end");
  }
  // ---- to_dense round trip
  std::vector<float> back(p.rows * p.cols ? p.rows * p.cols : 1, 7.f);
  rc = stk_cpu_to_dense(s.data.data(), s.row.data(), s.col.data(), nnz, (int)b, p.rows, p.cols, 4, index_dtype, back.data());
  CHECK(rc == STK_OK, "to_dense: %s", stk_cpu_last_error());
  CHECK(memcmp(back.data(), p.dense.data(), sizeof(float) * p.rows * p.cols) == 0, "to_dense round trip");
  // ---- products, both transposes, row-major and transposed dense operands
  auto close = [](float got, double want) { return fabs(got - want) <= 1e-4 * fabs(want) + 1e-3; };
  for (int trans = 0; trans < 2; trans++)
    for (int view = 0; view < 2; view++) {
      const int64_t m = trans ? p.cols : p.rows, k = trans ? p.rows : p.cols;
      auto S = [&](int64_t i, int64_t j) { return trans ? p.dense[j * p.cols + i] : p.dense[i * p.cols + j]; };
      // dsd: out [m, n] = op(S) [m, k] * rhs [k, n]; rhs stored [k, n] or as the transpose [n, k]
      std::vector<float> rhs(k * n ? k * n : 1);
      for (auto& v : rhs) v = g(rng);
      const int64_t rsk = view ? 1 : n, rsn = view ? k : 1;
      std::vector<float> out(m * n ? m * n : 1, 9.f);
      rc = stk_cpu_dsd(m, k, n, s.data.data(), s.offsets.data(), s.col.data(), s.offsets_t.data(), s.col_t.data(), s.block_offsets_t.data(),
                       trans, rhs.data(), rsk, rsn, out.data(), n, nnz, (int)b, STK_F32, index_dtype);
      CHECK(rc == STK_OK, "dsd: %s", stk_cpu_last_error());
      for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++) {
          double want = 0;
          for (int64_t kk = 0; kk < k; kk++) want += (double)S(i, kk) * rhs[kk * rsk + j * rsn];
          CHECK(close(out[i * n + j], want), "dsd trans %d view %d (%lld, %lld): %g vs %g", trans, view, (long long)i, (long long)j, out[i * n + j], want);
        }
      // dds: out [n, k'] = lhs [n, m'] * op(S) [m', k'] with op(S) = [m, k] above
      std::vector<float> lhs(n * m ? n * m : 1);
      for (auto& v : lhs) v = g(rng);
      const int64_t lsm = view ? 1 : m, lsk = view ? n : 1;
      std::vector<float> out2(n * k ? n * k : 1, 9.f);
      rc = stk_cpu_dds(n, m, k, lhs.data(), lsm, lsk, s.data.data(), s.offsets.data(), s.col.data(), s.offsets_t.data(), s.col_t.data(),
                       s.block_offsets_t.data(), trans, out2.data(), k, nnz, (int)b, STK_F32, index_dtype);
      CHECK(rc == STK_OK, "dds: %s", stk_cpu_last_error());
      for (int64_t i = 0; i < n; i++)
        for (int64_t j = 0; j < k; j++) {
          double want = 0;
          for (int64_t kk = 0; kk < m; kk++) want += (double)lhs[i * lsm + kk * lsk] * S(kk, j);
          CHECK(close(out2[i * k + j], want), "dds trans %d view %d (%lld, %lld): %g vs %g", trans, view, (long long)i, (long long)j, out2[i * k + j], want);
        }
    }
  // ---- sdd on the pattern, contraction length 2 n + 1 (odd on purpose: the host twins take any k)
  for (int view = 0; view < 2; view++) {
    const int64_t k = 2 * n + 1;
    std::vector<float> lhs(p.rows * k ? p.rows * k : 1), rhs(k * p.cols ? k * p.cols : 1);
    for (auto& v : lhs) v = g(rng);
    for (auto& v : rhs) v = g(rng);
    const int64_t lsm = view ? 1 : k, lsk = view ? p.rows : 1, rsk = view ? 1 : p.cols, rsn = view ? k : 1;
    std::vector<float> out(nnz * b * b ? nnz * b * b : 1, 9.f);
    rc = stk_cpu_sdd(lhs.data(), lsm, lsk, rhs.data(), rsk, rsn, p.rows, k, p.cols, out.data(), s.row.data(), s.col.data(), nnz, (int)b, STK_F32, index_dtype);
    CHECK(rc == STK_OK, "sdd: %s", stk_cpu_last_error());
    for (int64_t q = 0; q < nnz; q++)
      for (int64_t r = 0; r < b; r++)
        for (int64_t c = 0; c < b; c++) {
          const int64_t i = s.row[q] * b + r, j = s.col[q] * b + c;
          double want = 0;
          for (int64_t kk = 0; kk < k; kk++) want += (double)lhs[i * lsm + kk * lsk] * rhs[kk * rsk + j * rsn];
          CHECK(close(out[(q * b + r) * b + c], want), "sdd view %d block %lld (%lld, %lld)", view, (long long)q, (long long)r, (long long)c);
        }
  }
  // ---- 16-bit values run the same walks (values themselves are checked from Python against torch's conversions)
  {
    std::vector<uint16_t> d16(nnz * b * b ? nnz * b * b : 1, 0x3c00), rhs16(p.cols * n ? p.cols * n : 1, 0x3c00), out16(p.rows * n ? p.rows * n : 1);
    rc = stk_cpu_dsd(p.rows, p.cols, n, d16.data(), s.offsets.data(), s.col.data(), s.offsets_t.data(), s.col_t.data(), s.block_offsets_t.data(), 0,
                     rhs16.data(), n, 1, out16.data(), n, nnz, (int)b, STK_F16, index_dtype);
    CHECK(rc == STK_OK, "dsd f16: %s", stk_cpu_last_error());
    for (int64_t i = 0; i < br && n > 0; i++) {
      // a row of ones times ones = number of stored elements in the row (exact in fp16 up to 2048)
      const int64_t count = (s.offsets[i + 1] - s.offsets[i]) * b;
      if (count <= 2048) {
        uint16_t want = 0;
        if (count > 0) {
          int e = 0;
          int64_t c = count;
          while (c >= 2) c >>= 1, e++;
          want = (uint16_t)(((e + 15) << 10) | (((count << 10) >> e) & 0x3ff));
        }
        CHECK(out16[i * b * n] == want, "dsd f16 row %lld: %04x vs %04x", (long long)i, out16[i * b * n], want);
      }
    }
  }
  // ---- refused metadata: a column index outside the matrix, offsets that do not span the blocks
  if (nnz > 0) {
    std::vector<I> bad(s.col);
    bad[nnz - 1] = (I)bc;
    std::vector<float> rhs(p.cols * n ? p.cols * n : 1, 1.f), out(p.rows * n ? p.rows * n : 1);
    if (n > 0) {
      rc = stk_cpu_dsd(p.rows, p.cols, n, s.data.data(), s.offsets.data(), bad.data(), s.offsets_t.data(), s.col_t.data(), s.block_offsets_t.data(), 0,
                       rhs.data(), n, 1, out.data(), n, nnz, (int)b, STK_F32, index_dtype);
      CHECK(rc == STK_ERR_DIMS, "dsd with a column index outside the matrix was not refused");
      rc = stk_cpu_dsd(p.rows, p.cols, n, s.data.data(), s.offsets.data(), s.col.data(), s.offsets_t.data(), s.col_t.data(), s.block_offsets_t.data(), 0,
                       rhs.data(), n, 1, out.data(), n, nnz + 1, (int)b, STK_F32, index_dtype);
      CHECK(rc == STK_ERR_DIMS, "dsd with a wrong block count was not refused");
    }
    std::vector<float> dense(p.rows * p.cols);
    rc = stk_cpu_to_dense(s.data.data(), s.row.data(), bad.data(), nnz, (int)b, p.rows, p.cols, 4, index_dtype, dense.data());
    CHECK(rc == STK_ERR_DIMS, "to_dense with a column index outside the matrix was not refused");
    rc = stk_cpu_transpose_meta(s.row.data(), bad.data(), nnz, bc, index_dtype, s.col_t.data(), s.offsets_t.data(), s.block_offsets_t.data());
    CHECK(rc == STK_ERR_DIMS, "transpose_meta with a column index outside the matrix was not refused");
  }
}

int main() {
  std::mt19937 rng(20240);
  const struct { int64_t br, bc, b; double density; int64_t n; } cases[] = {
      {5, 7, 4, 0.5, 9},  {1, 1, 8, 1.0, 8},  {6, 4, 16, 0.4, 33}, {3, 9, 1, 0.6, 5},    {4, 4, 32, 0.0, 16},
      {8, 3, 8, 0.9, 300}, {2, 12, 2, 0.3, 1}, {7, 7, 3, 0.5, 0},  {3, 2, 64, 0.7, 70}, {1, 5, 128, 0.6, 40},
  };
  for (const auto& c : cases) {
    run_case<int16_t>(rng, c.br, c.bc, c.b, c.density, c.n, STK_I16);
    run_case<int32_t>(rng, c.br, c.bc, c.b, c.density, c.n, STK_I32);
  }
  if (g_failures) {
    printf("host_check: %d failures\n", g_failures);
    return 1;
  }
  printf("host_check ok\n");
  return 0;
}
