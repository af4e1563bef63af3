/*
 * C ABI of the MI355X (gfx950) grouped-GEMM library, libgrouped_gemm_hip.so.
 *
 * Plain pointers and sizes only; no torch types.  This is the boundary a binding of
 * the reference's extension entry point would link against: the reference exposes
 * one function, grouped_gemm::GroupedGemm(a, b, c, batch_sizes, trans_a, trans_b)
 * (csrc/grouped_gemm.h:5-9, bound at csrc/ops.cu:8), and everything below that call
 * (csrc/grouped_gemm.cu:324-464, csrc/fill_arguments.cuh:34-131) is replaced by
 * gg_gmm_bf16.
 *
 * All functions return 0 on success and a negative GG_E* code on failure;
 * gg_last_error() then holds a message for the calling thread.  Nothing here
 * synchronises the device or allocates device memory.
 */
#ifndef GROUPED_GEMM_HIP_H_
#define GROUPED_GEMM_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GG_OK 0
#define GG_EINVAL (-1)   /* bad argument (null pointer, negative size, both transposes, ...) */
#define GG_ELIMIT (-2)   /* a documented limit is exceeded (alignment, group count, 32-bit ranges) */
#define GG_EHIP (-3)     /* a HIP runtime call failed */

/* Most groups one launch schedules on the device.  Same value as the reference's
 * kMaxExperts (csrc/fill_arguments.cuh:11, enforced at csrc/grouped_gemm.cu:120-124).
 * Host-resident batch_sizes with more groups are split into several launches. */
#define GG_MAX_GROUPS_PER_LAUNCH 512

/* Columns of one row of the table written by gg_debug_schedule. */
#define GG_SCHED_COLS 12
/* m, n, k, lda, ldb, ldc, a_off, b_off, c_off (elements), first_tile, num_tiles, rows_used */

/*
 * Grouped GEMM, bf16 in, fp32 accumulate, bf16 out, alpha = 1, beta = 0.
 *
 * Replaces grouped_gemm::GroupedGemm's compute (csrc/grouped_gemm.cu:470-564 calling
 * CutlassGroupedGemm :324-371 or CublasGroupedGemm / CublasGroupedGemmVariableK
 * :396-435).  With S_e the exclusive prefix sum of batch_sizes and m_e = batch_sizes[e]:
 *
 *   trans_a = 0, trans_b = 0:  c[S_e : S_e+m_e, :] = a[S_e : S_e+m_e, :] @ b[e]
 *       a (tokens, hidden_in), b (num_groups, hidden_in, hidden_out), c (tokens, hidden_out)
 *   trans_a = 0, trans_b = 1:  c[S_e : S_e+m_e, :] = a[S_e : S_e+m_e, :] @ b[e]^T
 *       b (num_groups, hidden_out, hidden_in)
 *   trans_a = 1, trans_b = 0:  c[e] = a[S_e : S_e+m_e, :]^T @ b[S_e : S_e+m_e, :]
 *       a (tokens, hidden_in), b (tokens, hidden_out), c (num_groups, hidden_in, hidden_out);
 *       an empty group writes zeros to c[e].
 *
 * a, b, c: device pointers to contiguous row-major bf16.  Every element of c covered by
 * a group is overwritten; rows of c past sum(batch_sizes) are not touched.
 * batch_sizes: int64[num_groups], in host memory (batch_sizes_on_device = 0) or device
 * memory (1).  Device-resident sizes are read by the kernel itself; the host never
 * waits for them.  Rows a group would take past `tokens` are ignored, so no size
 * vector can make the kernel read or write outside a, b or c.
 * stream: a hipStream_t (NULL = the default stream).
 *
 * Limits (GG_ELIMIT): a, b and c 16-byte aligned, hidden_in and hidden_out multiples of 8
 * (16-byte rows, the same alignment the reference's kernel configuration assumes,
 * csrc/grouped_gemm.cu:41-66) and below 2^22; tokens below 2^31; num_groups <= GG_MAX_GROUPS_PER_LAUNCH when
 * batch_sizes is on the device.
 */
int gg_gmm_bf16(const void* a, const void* b, void* c, const int64_t* batch_sizes,
                int batch_sizes_on_device, int64_t num_groups, int64_t tokens,
                int64_t hidden_in, int64_t hidden_out, int trans_a, int trans_b,
                void* stream);

/*
 * Weight gradient accumulated in fp32: c[e] += a[S_e : S_e+m_e, :]^T @ b[S_e : S_e+m_e, :] for
 * every group, the trans_a layout of gg_gmm_bf16 with an fp32 output that is added to instead of
 * a bf16 output that is overwritten (alpha = 1, beta = 1).  a (tokens, hidden_in) and
 * b (tokens, hidden_out) bf16, c (num_groups, hidden_in, hidden_out) fp32, all row-major and
 * contiguous; c[e] of an empty group is left as it is.
 *
 * No counterpart in the reference, whose kernels fix alpha = 1, beta = 0 and a bf16 output
 * (csrc/grouped_gemm.cu:255-257, 469); for trainers that keep fp32 main gradients and would
 * otherwise run a second pass over c to add the bf16 result to them.
 * Limits as for gg_gmm_bf16, with hidden_in and hidden_out below 2^20.
 */
int gg_gmm_bf16_acc_f32(const void* a, const void* b, float* c, const int64_t* batch_sizes,
                        int batch_sizes_on_device, int64_t num_groups, int64_t tokens,
                        int64_t hidden_in, int64_t hidden_out, void* stream);

/*
 * Runs only the on-device scheduler of gg_gmm_bf16 (same device code, same
 * arguments) and writes what it derived to `table_out`, a device buffer of
 * num_groups * GG_SCHED_COLS int64: per group the problem (m, n, k), leading
 * dimensions, element offsets of its A, B and C blocks, its first tile index, its tile
 * count and the rows of `a` it uses.  The first nine columns are the quantities of
 * the reference's problem table (csrc/fill_arguments.cuh:63-78,
 * csrc/grouped_gemm.cu:159-175) and must equal its int64 closed forms bit for bit.
 * num_groups <= GG_MAX_GROUPS_PER_LAUNCH.
 */
int gg_debug_schedule(const int64_t* batch_sizes, int batch_sizes_on_device,
                      int64_t num_groups, int64_t tokens, int64_t hidden_in,
                      int64_t hidden_out, int trans_a, int trans_b, int64_t* table_out,
                      void* stream);

/* Output tile (rows, columns) and depth slice the kernel uses for a call with these arguments
 * (calls whose groups average few rows get a shorter tile); for reports and for checking the
 * tile counts of gg_debug_schedule. */
int gg_tile_shape(int64_t num_groups, int64_t tokens, int trans_a, int trans_b, int* bm, int* bn,
                  int* bk);

/* Message of the last failure on the calling thread ("" if none). */
const char* gg_last_error(void);

/* Library version, major * 10000 + minor * 100 + patch. */
int gg_version(void);

#ifdef __cplusplus
}
#endif
#endif /* GROUPED_GEMM_HIP_H_ */
