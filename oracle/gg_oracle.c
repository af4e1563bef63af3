/*
 * CPU oracle for the grouped-GEMM path.  TEST INFRASTRUCTURE ONLY: nothing
 * shipped may call into this file; it exists so the HIP kernels can be checked
 * against an independent, slow, obviously-correct restatement.
 *
 * What it restates (reference file:line):
 *   - per-expert GEMM loops and their pointer bumps: csrc/grouped_gemm.cu:396-416
 *     (fixed K, ragged M: NN / NT) and csrc/grouped_gemm.cu:418-435 (ragged K: TN);
 *     numerics of one GEMM (bf16 in, fp32 accumulate, alpha=1, beta=0, one bf16
 *     rounding on store): csrc/grouped_gemm.cu:373-394.
 *   - host-side problem table (dims, leading dimensions, running element
 *     offsets, k==0 => zero-fill, stable sort by k descending for TN):
 *     csrc/grouped_gemm.cu:146-222.
 *   - device-side problem table closed forms (exclusive prefix sum of
 *     batch_sizes): csrc/fill_arguments.cuh:34-98.  The reference evaluates some
 *     of those products in 32-bit; this oracle evaluates them in int64 on purpose.
 *   - k==0 outputs are zeros: csrc/fill_arguments.cuh:100-119,
 *     csrc/grouped_gemm.cu:177-189.
 *
 * How it is pinned (tests/test_oracle.py): the GEMM loops against torch.matmul
 * on fp32-upcast slices (a library routine), the ZeroK known answer of
 * grouped_gemm/ops_test.py:143-158, the ZeroSize vector of ops_test.py:124,
 * non-square shapes so a transposed operand fails; the two problem-table
 * functions against each other and against a brute-force walk in Python ints.
 */
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even, NaN kept quiet */
static uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* One row-major GEMM C(m,n) = op(A) op(B), fp32 accumulate.
 * trans_a: A is stored (k,m) row-major; trans_b: B is stored (n,k) row-major.
 * Follows the argument meaning of CublasGemm, csrc/grouped_gemm.cu:373-394. */
static void gemm_one(const uint16_t *a, const uint16_t *b, uint16_t *c_bf16, float *c_f32,
                     int64_t m, int64_t n, int64_t k, int trans_a, int trans_b) {
  for (int64_t i = 0; i < m; ++i) {
    for (int64_t j = 0; j < n; ++j) {
      float acc = 0.0f;
      for (int64_t p = 0; p < k; ++p) {
        float x = bf16_to_f32(trans_a ? a[p * m + i] : a[i * k + p]);
        float y = bf16_to_f32(trans_b ? b[j * k + p] : b[p * n + j]);
        acc += x * y;
      }
      if (c_f32) c_f32[i * n + j] = acc;
      if (c_bf16) c_bf16[i * n + j] = f32_to_bf16(acc);
    }
  }
}

/* Grouped GEMM, all three layouts.  Either output pointer may be NULL.
 *   !trans_a: a (tokens, hidden_in), b (E, hidden_in, hidden_out) or, with trans_b,
 *             (E, hidden_out, hidden_in); c (tokens, hidden_out).
 *             Loop and pointer bumps: csrc/grouped_gemm.cu:407-415.
 *   trans_a:  a (tokens, hidden_in), b (tokens, hidden_out), c (E, hidden_in, hidden_out);
 *             per expert c[e] = a_e^T b_e with k = batch_sizes[e].
 *             Loop and pointer bumps: csrc/grouped_gemm.cu:426-434.
 * Returns 0, or -1 if trans_a && trans_b (rejected at csrc/grouped_gemm.cu:476). */
int gg_oracle_gmm(const uint16_t *a, const uint16_t *b, uint16_t *c_bf16, float *c_f32,
                  const int64_t *batch_sizes, int64_t num_experts, int64_t hidden_in,
                  int64_t hidden_out, int trans_a, int trans_b) {
  if (trans_a && trans_b) return -1;
  if (!trans_a) {
    int64_t b_rows = trans_b ? hidden_out : hidden_in;
    int64_t b_cols = trans_b ? hidden_in : hidden_out;
    for (int64_t e = 0; e < num_experts; ++e) {
      int64_t m = batch_sizes[e];
      gemm_one(a, b, c_bf16, c_f32, m, hidden_out, hidden_in, 0, trans_b);
      a += m * hidden_in;
      b += b_rows * b_cols;
      if (c_bf16) c_bf16 += m * hidden_out;
      if (c_f32) c_f32 += m * hidden_out;
    }
  } else {
    int64_t m = hidden_in, n = hidden_out;
    for (int64_t e = 0; e < num_experts; ++e) {
      int64_t k = batch_sizes[e];
      gemm_one(a, b, c_bf16, c_f32, m, n, k, 1, 0); /* k == 0 writes zeros */
      a += k * m;
      b += k * n;
      if (c_bf16) c_bf16 += m * n;
      if (c_f32) c_f32 += m * n;
    }
  }
  return 0;
}

/* Row layout of the problem table, one row of GG_ORACLE_COLS int64 per expert. */
enum { COL_M, COL_N, COL_K, COL_LDA, COL_LDB, COL_LDC, COL_AOFF, COL_BOFF, COL_COFF,
       GG_ORACLE_COLS };

static void fill_ld(int64_t *row, int trans_a, int trans_b) {
  /* packed layouts: row-major ld = #columns, column-major ld = #rows
   * (csrc/grouped_gemm.cu:38-39, 165-167; csrc/fill_arguments.cuh:69-71) */
  row[COL_LDA] = trans_a ? row[COL_M] : row[COL_K];
  row[COL_LDB] = trans_b ? row[COL_K] : row[COL_N];
  row[COL_LDC] = row[COL_N];
}

/* Problem table by walking the host loop (csrc/grouped_gemm.cu:159-190) with running
 * element counters.  Dims are reported before the k==0 masking; `zero_fill[e]` is 1
 * where the reference memsets c[e].  `order` receives the stable descending-k
 * permutation for trans_a (csrc/grouped_gemm.cu:193-207), identity otherwise. */
void gg_oracle_table_walk(const int64_t *batch_sizes, int64_t num_experts, int64_t hidden_in,
                          int64_t hidden_out, int trans_a, int trans_b, int64_t *table,
                          int64_t *zero_fill, int64_t *order) {
  int64_t ea = 0, eb = 0, ec = 0;
  for (int64_t e = 0; e < num_experts; ++e) {
    int64_t *row = table + e * GG_ORACLE_COLS;
    row[COL_M] = trans_a ? hidden_in : batch_sizes[e];
    row[COL_N] = hidden_out;
    row[COL_K] = trans_a ? batch_sizes[e] : hidden_in;
    fill_ld(row, trans_a, trans_b);
    row[COL_AOFF] = ea;
    row[COL_BOFF] = eb;
    row[COL_COFF] = ec;
    ea += row[COL_M] * row[COL_K];
    eb += row[COL_K] * row[COL_N];
    ec += row[COL_M] * row[COL_N];
    zero_fill[e] = (row[COL_K] == 0);
    order[e] = e;
  }
  if (trans_a) { /* stable insertion sort, k descending */
    for (int64_t i = 1; i < num_experts; ++i) {
      int64_t idx = order[i], key = table[idx * GG_ORACLE_COLS + COL_K], j = i - 1;
      while (j >= 0 && table[order[j] * GG_ORACLE_COLS + COL_K] < key) {
        order[j + 1] = order[j];
        --j;
      }
      order[j + 1] = idx;
    }
  }
}

/* Problem table from the closed forms of the device builder
 * (csrc/fill_arguments.cuh:63-78), evaluated in int64. */
void gg_oracle_table_closed(const int64_t *batch_sizes, int64_t num_experts, int64_t hidden_in,
                            int64_t hidden_out, int trans_a, int trans_b, int64_t *table) {
  int64_t cumsum = 0;
  for (int64_t e = 0; e < num_experts; ++e) {
    int64_t *row = table + e * GG_ORACLE_COLS;
    row[COL_M] = trans_a ? hidden_in : batch_sizes[e];
    row[COL_N] = hidden_out;
    row[COL_K] = trans_a ? batch_sizes[e] : hidden_in;
    fill_ld(row, trans_a, trans_b);
    row[COL_AOFF] = trans_a ? row[COL_M] * cumsum : cumsum * row[COL_K];
    row[COL_BOFF] = (trans_a ? cumsum : e * row[COL_K]) * row[COL_N];
    row[COL_COFF] = (trans_a ? e * row[COL_M] : cumsum) * row[COL_N];
    cumsum += batch_sizes[e];
  }
}

int gg_oracle_table_cols(void) { return GG_ORACLE_COLS; }
