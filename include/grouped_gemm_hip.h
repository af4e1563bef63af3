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
 * gg_last_error() then holds a message for the calling thread
 * (gg_workspace_bytes_for returns a size).  No entry point synchronises the device or
 * allocates device memory.
 */
#ifndef GROUPED_GEMM_HIP_H_
#define GROUPED_GEMM_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GG_OK 0
#define GG_EINVAL (-1)   /* bad argument (null pointer, negative size, both transposes, ...) */
#define GG_ELIMIT (-2)   /* a documented limit is exceeded (alignment, 32-bit ranges, workspace) */
#define GG_EHIP (-3)     /* a HIP runtime call failed */

/* Most groups one launch schedules on the device.  Same value as the reference's
 * kMaxExperts (csrc/fill_arguments.cuh:11, enforced at csrc/grouped_gemm.cu:120-124).
 * Calls with more groups are split into several launches, whether batch_sizes lives on the
 * host or on the device (the reference rejects the latter). */
#define GG_MAX_GROUPS_PER_LAUNCH 512

/* Columns of one row of the table written by gg_debug_schedule:
 * m, n, k, lda, ldb, ldc, a_off, b_off, c_off (elements), first_tile, num_tiles, rows_used,
 * first_runt_tile, num_runt_tiles. */
#define GG_SCHED_COLS 14

/* Element types of a and b (and of c, unless it is the fp32 accumulator). */
#define GG_DTYPE_BF16 0
#define GG_DTYPE_F16 1
#define GG_DTYPE_F8E4M3 2   /* OCP e4m3 (torch.float8_e4m3fn) in a and b, bf16 in c */
#define GG_DTYPE_F8E5M2 3   /* OCP e5m2 (torch.float8_e5m2) in a and b, bf16 in c */

/* bits a launch ORs into *gg_gmm_args.size_status */
#define GG_STATUS_NEGATIVE_SIZE 1   /* a device-resident batch size was negative (taken as 0) */
#define GG_STATUS_ROWS_PAST_END 2   /* device-resident sizes sum past `tokens` (rows past the end dropped) */

/* gg_gmm_args.epilogue */
#define GG_EPILOGUE_NONE 0
#define GG_EPILOGUE_SWIGLU 1   /* b holds gate | up columns; c = silu(a @ gate) * (a @ up) */

/* Bytes of workspace that let any call cut the tiles of its last, partly filled round along the
 * depth (see gg_gmm): 4096 bytes of arrival counters and 256 partial tiles of 256 x 256 floats. */
#define GG_WORKSPACE_BYTES (4096 + 256 * 256 * 256 * 4)

/* gg_gmm_args.flags: debugging switches, for comparing the ways a call can be scheduled.  None
 * changes what is computed; results agree to within fp32 summation order. */
#define GG_FLAG_WHOLE_TILES 1   /* never cut the tiles of the last round into pieces */
#define GG_FLAG_ONE_CLASS 2     /* hand out a tall group's short last tile row in place, not after all other tiles */
#define GG_FLAG_ROW_PIECES 4    /* ignore the workspace: cut the last round's tiles along the rows only */
#define GG_FLAG_GROUP_ORDER 8   /* hand out the groups' tiles in group order, also where the library would hand them out by their number of tile rows (many short groups, trans_a = 0) */

/*
 * One-time set-up for the current device: checks that it is a gfx950 and raises the LDS limit
 * of every kernel variant.  Every other entry point does the same on its first call on a
 * device; call this first where that first call must not happen inside a HIP graph capture.
 */
int gg_init(void);

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
 * waits for them.  Each size is clamped to [0, tokens] and rows a group would take past
 * `tokens` are ignored, so no size vector can make the kernel read or write outside a, b or c.
 * Host-resident sizes that are negative or sum past `tokens` are rejected (GG_EINVAL).
 * stream: a hipStream_t (NULL = the default stream).
 *
 * One persistent launch (one per 512 groups).  Uses no workspace: the tiles of a partly filled
 * last round are cut along their rows only; gg_gmm with a workspace cuts them along the depth.
 *
 * Limits (GG_ELIMIT): hidden_in and hidden_out below 2^22; tokens below 2^31.  Hidden sizes that
 * are multiples of 8 with a, b and c on 16-byte boundaries (the alignment the reference's kernel
 * configuration assumes, csrc/grouped_gemm.cu:41-66) run on the streaming kernels, and so do
 * operands on 4-byte boundaries with even hidden sizes; other sizes and alignments run on slower,
 * general kernels (see gg_gmm).
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
 * The general form: everything gg_gmm_bf16 and gg_gmm_bf16_acc_f32 do, selected by fields, plus
 * what the reference's entry point (csrc/grouped_gemm.cu:470-564) has no argument for.  Zero
 * the struct, set struct_bytes = sizeof(gg_gmm_args), fill in what is needed.
 *
 *   dtype         GG_DTYPE_*: element type of a and b, and of c for the two-byte types (fp8
 *                 operands give a bf16 c).  The reference rejects everything but bf16
 *                 (csrc/grouped_gemm.cu:492, 505-506).
 *   hidden_in, hidden_out
 *                 Any size below 2^22 (the reference's default build runs any size through
 *                 cuBLAS, csrc/grouped_gemm.cu:373-394, its grouped kernel assumes multiples of
 *                 8, :469).  Multiples of 8 with 16-byte aligned two-byte operands run on the
 *                 streaming kernels, and so do fp8 operands whose contiguous dimensions are
 *                 multiples of 16, and, with the plain epilogue (no SwiGLU, no fp32 accumulation),
 *                 two-byte operands on 4-byte boundaries with even hidden sizes; everything else
 *                 (odd sizes, 2-byte boundaries) on slower, general ones.
 *   a_row_index   int32[tokens] on the device, or NULL: row r of the product's left operand is
 *                 row a_row_index[r] of `a` (a gather fused into the load: `a` is the tensor
 *                 before the permutation that sorts rows by group, and may have any number of
 *                 rows).  The reference takes rows already sorted (grouped_gemm/ops.py:8).
 *   b_row_index   the same for the rows of b, trans_a layout only.
 *   c_row_index   int32[tokens] on the device, or NULL: row r of the output is stored to row
 *                 c_row_index[r] of c (a scatter fused into the store; not with trans_a).  Rows of
 *                 c that no index names are not touched.  c_row_index must not name a row twice.
 *                 An index that names no row of its tensor (negative, or past the row count
 *                 below) is a missing row on every kernel: zeros on the way in, nothing stored
 *                 on the way out; no such index can make a kernel touch memory outside a, b, c.
 *   a_num_rows, b_num_rows, c_num_rows
 *                 Rows of a, b and c in memory when a row index redirects them (0: `tokens`).
 *                 With two-byte elements, aligned operands and a and c below 4 GiB the NN and NT
 *                 layouts run indexed on the streaming kernels; otherwise, and with trans_a, on
 *                 the general ones.
 *   size_status   int32 word on the device, or NULL.  Host-resident batch_sizes that are negative
 *                 or sum past `tokens` are rejected; device-resident ones cannot be (the host
 *                 never reads them) and are clamped instead.  With a status word the kernel ORs
 *                 GG_STATUS_* bits into it when it had to clamp, for the caller to read whenever
 *                 it next synchronises.  Never cleared by the library.
 *   epilogue      GG_EPILOGUE_SWIGLU (not with trans_a or accumulate_f32): b holds two matrices
 *                 per group side by side, gate and up: (num_groups, hidden_in, 2 * hidden_out), or
 *                 (num_groups, 2 * hidden_out, hidden_in) with trans_b, gate first.  c (tokens,
 *                 hidden_out) = silu(a @ gate) * (a @ up) with silu(x) = x / (1 + exp(-x)), both
 *                 products accumulated and combined in fp32, rounded once.  The reference has no
 *                 epilogue hook (alpha = 1, beta = 0, csrc/grouped_gemm.cu:255).
 *   accumulate_f32  1: c is fp32 and is added to (trans_a = 1 only), as gg_gmm_bf16_acc_f32.
 *   workspace, workspace_bytes
 *                 Device memory the call may use for partial results, or NULL.  When the last
 *                 round of the persistent grid is at most half full, each of its tiles is cut
 *                 into 2 or 4 pieces along the depth; a piece adds up its depth slices into an
 *                 fp32 partial tile in the workspace, and the piece that finishes last sums the
 *                 partial tiles in piece order and stores the result, so the output does not
 *                 depend on timing.  With trans_a = 1, when a group is so much deeper than the
 *                 rest that its tiles alone would set the length of the launch, the tiles of
 *                 such groups are cut the same way and handed out first (instead of the last
 *                 round's).  The first 4096 bytes (arrival counters) must be zero
 *                 before the first call and are zero again after every call; the rest needs no
 *                 initialisation.  GG_WORKSPACE_BYTES serves every call; a smaller workspace
 *                 (at least 4096 + one 256 KiB tile) serves fewer pieces; 256-byte aligned.
 *                 Calls that share a workspace must not overlap in time (same stream is enough).
 *   flags         GG_FLAG_* bits.
 */
typedef struct gg_gmm_args {
  uint32_t struct_bytes;
  int32_t dtype;
  const void* a;
  const void* b;
  void* c;
  const int64_t* batch_sizes;
  int32_t batch_sizes_on_device;
  int32_t trans_a;
  int32_t trans_b;
  int32_t accumulate_f32;
  int64_t num_groups;
  int64_t tokens;
  int64_t hidden_in;
  int64_t hidden_out;
  void* workspace;
  uint64_t workspace_bytes;
  int32_t flags;
  int32_t reserved0;
  void* stream;
  const int32_t* a_row_index;
  const int32_t* b_row_index;
  const int32_t* c_row_index;
  int64_t a_num_rows;
  int64_t c_num_rows;
  int32_t epilogue;
  int32_t b_num_rows;
  int32_t* size_status;
} gg_gmm_args;

int gg_gmm(const gg_gmm_args* args);

/*
 * Bytes of workspace the call described by `args` can make use of: 0 when no launch of it ever
 * cuts tiles along the depth (general kernels, row indices, the SwiGLU epilogue, or a product too
 * shallow for depth pieces to pay: fewer than 96 depth slices of 64 two-byte or 128 one-byte
 * elements, the depth of the trans_a layout being what one group could hold, i.e. all rows),
 * GG_WORKSPACE_BYTES otherwise.  Looks at the sizes, flags
 * and pointers' alignment only; args->workspace is ignored.  A caller that keeps workspaces
 * (one per stream) need not allocate one for calls this returns 0 for.  No counterpart in the
 * reference, which asks CUTLASS for its workspace size per call (csrc/grouped_gemm.cu:347-349).
 */
uint64_t gg_workspace_bytes_for(const gg_gmm_args* args);

/*
 * gg_gmm for callers that cannot allocate and have no workspace to bring: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference.  Same arguments and same results as gg_gmm called with a workspace of
 * GG_WORKSPACE_BYTES, except that args->workspace must be NULL: the partial tiles and arrival
 * counters live in a static device array of GG_WORKSPACE_BYTES (64 MiB + 4 KiB) inside the
 * library, one per GPU, held until the process ends.  Calls no hipMalloc, hipFree or any
 * allocating routine; the counters are cleared by a small fill kernel on the stream ahead of the
 * GEMM launch.  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU
 * (different streams, different threads) race on it and must be serialised by the caller.
 * The array holds one partial tile per workgroup of a launch of up to 256 workgroups: a device
 * with more compute units is rejected (GG_ELIMIT), as is a non-NULL workspace (GG_EINVAL).
 * gg_init (or any earlier call of the library on that device) must come first where the call
 * itself must not allocate or is being captured: the first call on a device loads the kernels'
 * code object, raises their LDS limits and looks the array's address up.  Without depth pieces to
 * cut (gg_workspace_bytes_for returns 0) the result equals gg_gmm's with workspace = NULL.
 */
int gg_gmm_no_alloc(const gg_gmm_args* args);

/*
 * Runs only the on-device scheduler of gg_gmm_bf16 (same device code, same
 * arguments) and writes what it derived to `table_out`, a device buffer of
 * num_groups * GG_SCHED_COLS int64: per group the problem (m, n, k), leading
 * dimensions, element offsets of its A, B and C blocks, its first tile index, its tile
 * count, the rows of `a` it uses, and the first index and count of its tiles of the second
 * class (the much shorter last tile row of a tall group, handed out after all other tiles).
 * The first nine columns are the quantities of the reference's problem table
 * (csrc/fill_arguments.cuh:63-78, csrc/grouped_gemm.cu:159-175) and must equal its int64
 * closed forms bit for bit.  num_groups <= GG_MAX_GROUPS_PER_LAUNCH.
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
