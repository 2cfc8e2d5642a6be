// Host-side problem descriptions shared by the C-ABI layer and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace km {

enum {
    KM_VARIANT_AUTO = 0,
    KM_VARIANT_VALU = 1,
    KM_VARIANT_MFMA_F32 = 2,         // fp32 MFMA; rbf and spectral kernels up to 32 rhs columns through the column tables
    KM_VARIANT_MFMA_F16 = 3,         // split-fp16 MFMA; spectral kernels in phase-split form
    KM_VARIANT_MFMA_F16_DIRECT = 4,  // split-fp16 MFMA with the cosine evaluated per pair
    KM_VARIANT_BLOCK = 5,            // split-fp16 MFMA, rhs operand prepared once per workgroup of 4 row blocks
    KM_VARIANT_MFMA_F32_DIRECT = 6   // fp32 MFMA with every entry evaluated directly, operands straight from memory
};

struct MatmulProblem {
    int kernel_type;
    int batch_rank;
    const int64_t* batch_sizes;
    long long num_batches;
    int64_t m, n, k;
    const float* x1;
    const int64_t* x1_strides;
    const float* x2;
    const int64_t* x2_strides;
    const float* rhs;
    const int64_t* rhs_strides;
    const float* params;
    const int64_t* params_strides;
    const int32_t* start;
    const int64_t* start_strides;
    const int32_t* end;
    const int64_t* end_strides;
    float* out;
};

// Which ahead-of-time instantiation runs and with what decomposition.
struct MatmulPlan {
    int variant;     // one of the KM_VARIANT_* values above except KM_VARIANT_AUTO
    int k_chunk;     // rhs columns handled per workgroup (MFMA: 16/32/64, VALU: 4/8/16)
    int row_groups;  // MFMA: groups of 16 rows per wavefront (1, 2, 4, 8)
    int col_splits;  // MFMA: wavefronts per workgroup sharing one column range (1, 2, 4, 8)
    int tail_balance;  // split-fp16 kernels: cut the uneven remainder into 16-row pieces
    int phase_split;   // KM_VARIANT_BLOCK: spectral kernel in phase-split form
    long long group_tail;  // table kernel: >= 0 selects the grouped launch (workgroups of 4 wavefronts) with
                           // this many items per XCD split by columns at the end; < 0: one wavefront per workgroup
    long long group_tail_halves;  // how many of those, the very last, also run as two halves of 64 rows
};

hipError_t launch_matmul(const MatmulProblem& p, const MatmulPlan& plan, hipStream_t stream);
hipError_t launch_matmul_block(const MatmulProblem& p, const MatmulPlan& plan, hipStream_t stream);

struct ParamGradProblem {
    int kernel_type;
    int batch_rank;
    const int64_t* batch_sizes;
    long long num_batches;
    int64_t m, n, c;
    const float* x1;
    const int64_t* x1_strides;
    const float* x2;
    const int64_t* x2_strides;
    const float* left;
    const int64_t* left_strides;
    const float* right;
    const int64_t* right_strides;
    const float* params;
    const int64_t* params_strides;
    const int32_t* start;
    const int64_t* start_strides;
    const int32_t* end;
    const int64_t* end_strides;
    float* grad;
    void* workspace;
};

// Partial sums written by the first pass: one row of KM_MAX_PARAMS floats per wavefront.
long long param_grad_partials_per_batch(int64_t m, long long num_batches);
// Same for the feature form of the first pass at vector width c (0 where the form does not apply).
long long param_grad_feature_partials_per_batch(int kernel_type, int64_t m, long long num_batches, int64_t c);
// Which kernels and decomposition launch_param_grad picks for contiguous operands of this size.
void describe_param_grad(int kernel_type, int64_t m, long long num_batches, int64_t c, char* text,
                         size_t text_bytes);
hipError_t launch_param_grad(const ParamGradProblem& p, hipStream_t stream);

struct IndexProblem {
    int kernel_type;
    int batch_rank;
    const int64_t* batch_sizes;
    int64_t m, n;
    const float* x1;
    const int64_t* x1_strides;
    const float* x2;
    const int64_t* x2_strides;
    const float* params;
    const int64_t* params_strides;
    const int32_t* start;
    const int64_t* start_strides;
    const int32_t* end;
    const int64_t* end_strides;
    int index_rank;
    const int64_t* index_sizes;
    const int32_t* const* batch_index;
    const int64_t* const* batch_index_strides;
    const int32_t* row_index;
    const int64_t* row_index_strides;
    const int32_t* col_index;
    const int64_t* col_index_strides;
    float* out;
};

hipError_t launch_index(const IndexProblem& p, hipStream_t stream);

// index_bwd: the index problem plus the incoming gradient (same shape as the index tensors),
// the output [batch..., P] and scratch of index_bwd_workspace_bytes().
struct IndexBwdProblem {
    IndexProblem index;
    long long num_batches;
    const float* out_grad;
    const int64_t* out_grad_strides;
    float* grad;
    void* workspace;
};
size_t index_bwd_workspace_bytes(long long total_entries);
hipError_t launch_index_bwd(const IndexBwdProblem& p, hipStream_t stream);

struct DenseProblem {
    int kernel_type;
    int batch_rank;
    const int64_t* batch_sizes;
    long long num_batches;
    int64_t m, n;
    const float* x1;
    const int64_t* x1_strides;
    const float* x2;
    const int64_t* x2_strides;
    const float* params;
    const int64_t* params_strides;
    const int32_t* start;
    const int64_t* start_strides;
    const int32_t* end;
    const int64_t* end_strides;
    float* out;                      // dense
    const float* weights;            // dense_bwd: out_grad [batch..., m, n]
    const int64_t* weights_strides;
    float* grad;                     // dense_bwd: [batch..., P]
    void* workspace;                 // dense_bwd
};

hipError_t launch_dense(const DenseProblem& p, hipStream_t stream);
hipError_t launch_dense_bwd(const DenseProblem& p, hipStream_t stream);

struct BatchShape;
struct BatchStrides;
hipError_t launch_param_grad_reduce(int kernel_type, const BatchShape& batch, long long num_batches,
                                    long long partial_rows, const float* partials,
                                    const float* params, const BatchStrides& params_bs,
                                    long long params_s, float* grad, hipStream_t stream);

hipError_t launch_make_ranges(const float* x1, const float* x2, int64_t num_batch, int64_t n1,
                              int64_t n2, float cutoff, int block_size, int align, int32_t* start,
                              int32_t* end, hipStream_t stream);
hipError_t launch_make_ranges_symmetric(const float* x, int64_t num_batch, int64_t n, float cutoff,
                                        int block_size, int32_t* start, int32_t* end,
                                        hipStream_t stream);

}  // namespace km
