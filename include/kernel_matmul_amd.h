/*
 * kernel_matmul_amd — C ABI of the MI355X (gfx950) KernelMatmul library.
 *
 * Every entry point takes plain pointers, sizes and strides; no torch types cross this
 * boundary.  Device entry points take device pointers plus a hipStream_t (as void*) and
 * only enqueue work on that stream; they never synchronise and never allocate.  Host entry
 * points (the range builders) take host pointers and run on the calling thread.
 *
 * Conventions shared by all device entry points
 *   - All floating point data is fp32, all index data is int32.
 *   - `batch_rank` (0..KM_MAX_BATCH_RANK) and `batch_sizes[batch_rank]` describe the common
 *     batch shape.  Every tensor argument comes with a `*_strides` array holding, in
 *     elements, first the `batch_rank` batch strides and then the strides of its own
 *     trailing dimensions.  Stride 0 (expanded views) and non-contiguous views are fine.
 *   - The sparsity pattern is block-row based with a fixed block of KM_BLOCK_SIZE rows:
 *     row block i of batch item b covers columns [start[b,i], end[b,i]).
 *   - `params` holds the *user facing* hyper-parameters; the transform to the form used
 *     on the device and the chain rule back for gradients are done inside the kernels:
 *         KM_KERNEL_RBF              [lengthscale, outputscale]
 *         KM_KERNEL_SPECTRAL         [lengthscale, frequency, outputscale]
 *         KM_KERNEL_LOCALLY_PERIODIC [lengthscale_rbf, lengthscale_periodic, period, outputscale]
 *   - Outputs are contiguous, allocated by the caller, and fully overwritten.
 *   - Return value: 0 (KM_OK) on success, otherwise a negative KM_ERR_* code; a message
 *     for the calling thread's last failure is available from km_last_error().
 */
#ifndef KERNEL_MATMUL_AMD_H
#define KERNEL_MATMUL_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KM_BLOCK_SIZE 128
#define KM_MAX_BATCH_RANK 6
#define KM_MAX_PARAMS 4

#define KM_KERNEL_RBF 0
#define KM_KERNEL_SPECTRAL 1
#define KM_KERNEL_LOCALLY_PERIODIC 2

#define KM_OK 0
#define KM_ERR_INVALID_ARGUMENT (-1)
#define KM_ERR_UNSUPPORTED (-2)
#define KM_ERR_LAUNCH (-3)
#define KM_ERR_WORKSPACE (-4)

/* Launch tuning, all optional (pass NULL for the built-in gfx950 table).
 * Replaces the per-define-set JIT autotuner of the reference
 * (kernel_matmul/configurations.py:84-118): nothing is compiled at run time, the values
 * only select among ahead-of-time instantiated kernels. */
typedef struct km_launch_options {
    int variant;          /* 0 = table, 1 = VALU FMA contraction, 2 = fp32 MFMA contraction (rbf and
                             spectral kernels with at most 32 rhs columns through the same column
                             tables as 3, the cosine of the phase difference per entry from
                             tabulated cosines and sines; others evaluated directly as with 6),
                             3 = split-fp16 (hi+lo) MFMA contraction with fp32 accumulation; rbf
                             and spectral kernels with at most 16 rhs columns go through
                             per-wavefront column tables (spectral in phase-split form), spectral
                             kernels with 17 to 32 columns too (cosine per entry from tabulated
                             phases),
                             4 = split-fp16 MFMA with the kernel evaluated directly per pair,
                             5 = split-fp16 MFMA with the rhs operand prepared once per workgroup
                             of four row blocks (rows_per_wave / col_splits must stay 0),
                             6 = fp32 MFMA contraction with every entry evaluated directly.
                             The table picks 5 for large locally periodic problems with at most
                             16 rhs columns and 3 otherwise. */
    int rows_per_wave;    /* 0 = table; else 16, 32, 64 or 128 rows of x1 per wavefront */
    int col_splits;       /* 0 = table; else 1, 2, 4 or 8 wavefronts sharing one row range */
    int reserved;         /* tail handling, for measurements: 0 = table; 1 = no tail balancing (no
                             16-row pieces, no grouped launch); 2 + v + (h << 16) = grouped launch of
                             the table kernel with the last v row-block items of every XCD split by
                             columns over a workgroup (v = 0: none split), the last h - 1 of them
                             also into two halves of 64 rows (h = 0: a quarter of v) */
} km_launch_options;

/* Message for the last error returned on the calling thread ("" if none). */
const char* km_last_error(void);

/* Library version as major*10000 + minor*100 + patch. */
int km_version(void);

/* Number of kernel hyper-parameters for a kernel type, or -1 if unknown.
 * (reference: KM_NUM_PARAMS, native/common/kernel_function.cuh:3-16) */
int km_num_params(int kernel_type);

/* ------------------------------------------------------------------------------------
 * Range builders (host).  Replace native/ranges/ranges.cpp:8-62, 64-101, 103-150 of the
 * reference (pybind module km___ranges, ranges.cpp:152-156).  Inputs are contiguous host
 * arrays x1[num_batch][n1], x2[num_batch][n2], sorted ascending per row; outputs are
 * start/end[num_batch][ceil(n1/block_size)].  All comparisons are done in fp32.
 * ---------------------------------------------------------------------------------- */
int km_make_ranges(const float* x1, const float* x2, int64_t num_batch, int64_t n1, int64_t n2,
                   float cutoff, int block_size, int align, int32_t* start, int32_t* end);

int km_make_ranges_symmetric(const float* x, int64_t num_batch, int64_t n, float cutoff,
                             int block_size, int32_t* start, int32_t* end);

/* start/end[num_batch][rows] -> start_t/end_t[num_batch][ceil(x2_size/block_size)].
 * The input must be block aligned (the caller checks, as kernel_matmul/ranges.py:110-113). */
int km_transpose_ranges(const int32_t* start, const int32_t* end, int64_t num_batch,
                        int64_t rows, int x1_size, int x2_size, int block_size, int32_t* start_t,
                        int32_t* end_t);

/* Same three functions on device-resident data, enqueued on `stream` with no host round
 * trip (the reference copies to the host and back, ranges.cpp:11-15, 61).  Results are
 * identical to the host functions for inputs that are sorted ascending and cutoff >= 0. */
int km_make_ranges_device(const float* x1, const float* x2, int64_t num_batch, int64_t n1,
                          int64_t n2, float cutoff, int block_size, int align, int32_t* start,
                          int32_t* end, void* stream);

int km_make_ranges_symmetric_device(const float* x, int64_t num_batch, int64_t n, float cutoff,
                                    int block_size, int32_t* start, int32_t* end, void* stream);

/* ------------------------------------------------------------------------------------
 * matmul.  out[b,i,c] = sum_{j in [start[b,i/128], end[b,i/128])} k(x1[b,i], x2[b,j]) rhs[b,j,c]
 * Replaces `call` of module km___matmul___* (native/matmul/matmul.cpp:6-17,
 * native/matmul/matmul.cu:160-203).
 *   x1[batch..., m], x2[batch..., n], rhs[batch..., n, k], params[batch..., P],
 *   start/end[batch..., ceil(m/128)], out[batch..., m, k] contiguous.
 * The strides of x1, x2 and rhs along their own dimensions must not be negative, and those of x2
 * and rhs at most 2^22 elements (KM_ERR_UNSUPPORTED otherwise); batch strides are free.
 * ---------------------------------------------------------------------------------- */
int km_matmul(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
              int64_t k, const float* x1, const int64_t* x1_strides, const float* x2,
              const int64_t* x2_strides, const float* rhs, const int64_t* rhs_strides,
              const float* params, const int64_t* params_strides, const int32_t* start,
              const int64_t* start_strides, const int32_t* end, const int64_t* end_strides,
              float* out, const km_launch_options* options, void* stream);

/* Which ahead-of-time kernel and decomposition km_matmul would pick for a problem of this
 * size (host only; nothing is launched).  Writes a short description such as
 * "km::fwd_table_f16<spectral, G=1, R=8>: 128 rows per wavefront, ..." into `text`.
 * Stands in for the reference's autotune report (kernel_matmul/native_function.py:56-69,
 * which prints the winning define set). */
int km_matmul_describe(int kernel_type, int64_t num_batches, int64_t m, int64_t n, int64_t k,
                       const km_launch_options* options, char* text, size_t text_bytes);

/* Which kernels and decomposition km_param_grad would pick for contiguous operands of this
 * size (host only; nothing is launched): the feature form or the pairwise form, and the number
 * of column shares per row block.  Like km_matmul_describe, it stands in for the reference's
 * autotune report (kernel_matmul/native_function.py:56-69). */
int km_param_grad_describe(int kernel_type, int64_t num_batches, int64_t m, int64_t c, char* text,
                           size_t text_bytes);

/* ------------------------------------------------------------------------------------
 * Hyper-parameter gradient of a bilinear form through the masked kernel matrix:
 *   grad[b,p] = d/d params[b,p]  sum_{(i,j) in mask} (sum_c left[b,i,c] right[b,j,c]) K[b,i,j]
 * One kernel serves both reference operators:
 *   - matmul_bwd  (native/matmul_bwd/matmul_bwd.cpp:6-19, matmul_bwd.cu:182-221):
 *         left = out_grad[batch..., m, k], right = rhs[batch..., n, k]
 *   - bilinear_derivative (native/bilinear_derivative/bilinear_derivative.cpp:6-21,
 *     bilinear_derivative.cu:138-183): left = left_vecs, right = right_vecs.
 * grad[batch..., P] contiguous.  `workspace` is device scratch of at least
 * km_param_grad_workspace_size(...) bytes; its contents on entry do not matter.
 * The reduction order is fixed, so results are run-to-run reproducible.
 * ---------------------------------------------------------------------------------- */
size_t km_param_grad_workspace_size(int kernel_type, int batch_rank, const int64_t* batch_sizes,
                                    int64_t m, int64_t n, int64_t c);

int km_param_grad(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m,
                  int64_t n, int64_t c, const float* x1, const int64_t* x1_strides,
                  const float* x2, const int64_t* x2_strides, const float* left,
                  const int64_t* left_strides, const float* right, const int64_t* right_strides,
                  const float* params, const int64_t* params_strides, const int32_t* start,
                  const int64_t* start_strides, const int32_t* end, const int64_t* end_strides,
                  float* grad, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------
 * km_param_grad without any allocation: the same computation with the scratch in a static
 * device array of KM_STATIC_SCRATCH_BYTES that the library keeps on every GPU it runs on
 * until the process ends.  No counterpart in the reference (its operators allocate their
 * scratch with torch::zeros on every call, native/matmul_bwd/matmul_bwd.cu:203-206); it is
 * for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Results are bit-identical to km_param_grad.
 *   - Problems whose km_param_grad_workspace_size() exceeds KM_STATIC_SCRATCH_BYTES are
 *     rejected with KM_ERR_WORKSPACE (4 MiB holds 262144 row-block x column-split partial
 *     rows, e.g. n = 10^6 with batch 32).
 *   - Every call on one GPU uses that GPU's single array: calls that overlap on one GPU
 *     (different streams or threads) race; serialise them or use km_param_grad.
 *   - The first call on a device looks the array's address up (hipGetSymbolAddress); make
 *     that call outside graph capture.
 * ---------------------------------------------------------------------------------- */
#define KM_STATIC_SCRATCH_BYTES (4u << 20)

int km_param_grad_static(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m,
                         int64_t n, int64_t c, const float* x1, const int64_t* x1_strides,
                         const float* x2, const int64_t* x2_strides, const float* left,
                         const int64_t* left_strides, const float* right,
                         const int64_t* right_strides, const float* params,
                         const int64_t* params_strides, const int32_t* start,
                         const int64_t* start_strides, const int32_t* end,
                         const int64_t* end_strides, float* grad, void* stream);

/* ------------------------------------------------------------------------------------
 * index.  out[q] = K[batch_index_0[q], ..., row_index[q], col_index[q]], 0 outside the mask.
 * Replaces `call` of module km___index___* (native/index/index.cpp:6-24,
 * native/index/index.cu:69-101).  The index tensors share the shape
 * index_sizes[index_rank] (last dimension = entries per index batch); `batch_index[d]`
 * selects along batch dimension d of x1/x2/params/start/end.  out is contiguous with the
 * index shape.
 * ---------------------------------------------------------------------------------- */
int km_index(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
             const float* x1, const int64_t* x1_strides, const float* x2,
             const int64_t* x2_strides, const float* params, const int64_t* params_strides,
             const int32_t* start, const int64_t* start_strides, const int32_t* end,
             const int64_t* end_strides, int index_rank, const int64_t* index_sizes,
             const int32_t* const* batch_index, const int64_t* const* batch_index_strides,
             const int32_t* row_index, const int64_t* row_index_strides,
             const int32_t* col_index, const int64_t* col_index_strides, float* out,
             void* stream);

/* ------------------------------------------------------------------------------------
 * index_bwd.  grad[b,p] = d/d params[b,p] sum_{q : batch(q) = b} out_grad[q] * K-entry(q)
 * with the entries addressed exactly as in km_index; out_grad has the index shape.
 * Replaces `call` of module km___index_bwd___* (native/index_bwd/index_bwd.cpp,
 * native/index_bwd/index_bwd.cu:12-112).  grad[batch..., P] contiguous; `workspace` of at
 * least km_index_bwd_workspace_size(number of index entries) bytes, contents irrelevant.
 * ---------------------------------------------------------------------------------- */
size_t km_index_bwd_workspace_size(int64_t num_entries);

int km_index_bwd(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
                 const float* x1, const int64_t* x1_strides, const float* x2,
                 const int64_t* x2_strides, const float* params, const int64_t* params_strides,
                 const int32_t* start, const int64_t* start_strides, const int32_t* end,
                 const int64_t* end_strides, int index_rank, const int64_t* index_sizes,
                 const int32_t* const* batch_index, const int64_t* const* batch_index_strides,
                 const int32_t* row_index, const int64_t* row_index_strides,
                 const int32_t* col_index, const int64_t* col_index_strides,
                 const float* out_grad, const int64_t* out_grad_strides, float* grad,
                 void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------
 * dense.  out[b,i,j] = K[b,i,j] for j in the row block's [start, end), 0 elsewhere;
 * out[batch..., m, n] contiguous and fully written.  Replaces `call` of module
 * km___dense___* (native/dense/dense.cpp, native/dense/dense.cu:12-98).
 * ---------------------------------------------------------------------------------- */
int km_dense(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
             const float* x1, const int64_t* x1_strides, const float* x2,
             const int64_t* x2_strides, const float* params, const int64_t* params_strides,
             const int32_t* start, const int64_t* start_strides, const int32_t* end,
             const int64_t* end_strides, float* out, void* stream);

/* ------------------------------------------------------------------------------------
 * dense_bwd.  grad[b,p] = d/d params[b,p] sum_{(i,j) in mask} out_grad[b,i,j] K[b,i,j].
 * Replaces `call` of module km___dense_bwd___* (native/dense_bwd/dense_bwd.cpp,
 * native/dense_bwd/dense_bwd.cu:12-116).  out_grad[batch..., m, n] with strides;
 * grad[batch..., P] contiguous; workspace as for km_param_grad (same size function).
 * ---------------------------------------------------------------------------------- */
int km_dense_bwd(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
                 const float* x1, const int64_t* x1_strides, const float* x2,
                 const int64_t* x2_strides, const float* params, const int64_t* params_strides,
                 const int32_t* start, const int64_t* start_strides, const int32_t* end,
                 const int64_t* end_strides, const float* out_grad,
                 const int64_t* out_grad_strides, float* grad, void* workspace,
                 size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* KERNEL_MATMUL_AMD_H */
