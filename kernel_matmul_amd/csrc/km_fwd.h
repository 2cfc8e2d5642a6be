// Definitions shared by the forward (K @ rhs) kernels.
#pragma once

#include "km_common.h"

namespace km {

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half8v join_half2x4(const half2v (&p)[4]) {
    const half4v a = __builtin_shufflevector(p[0], p[1], 0, 1, 2, 3);
    const half4v b = __builtin_shufflevector(p[2], p[3], 0, 1, 2, 3);
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Launch arguments of the forward kernels (batch dimensions already collapsed).
struct FwdArgs {
    BatchShape batch;
    long long num_batches;
    long long total_items;   // row chunks * batches
    long long items_per_xcd;
    int m, n, k;
    int chunks_per_block;    // 128 / rows per workgroup
    int tail_items;          // per XCD: row-block items at the end that are split 8 ways by rows
    const float* x1;
    const float* x2;
    const float* rhs;
    const float* params;
    const int* start;
    const int* end;
    float* out;
    BatchStrides x1_bs, x2_bs, rhs_bs, params_bs, start_bs, end_bs;
    long long x1_s, x2_s, rhs_s0, rhs_s1, params_s, start_s, end_s;
};

struct MatmulProblem;
// Collapses the batch dimensions and copies pointers, sizes and strides (item counts are left
// to the caller).
void fill_fwd_args(const MatmulProblem& p, FwdArgs* args);

// The split-fp16 kernels evaluate K / sigma scaled by 2^14 (folded into the exponent of the
// base-2 exponential) so that its hi and lo halves stay inside the fp16 exponent range.
#define KM_F16_KSCALE_LOG2 14

// Phase f * (x - c) in revolutions, reduced to [-0.5, 0.5].  It is needed once per row or column
// (never per pair), so it is formed in double precision: neither the difference to the
// reference point nor the product is rounded before the reduction, and the result carries
// half an fp32 ulp of 0.5 (3e-8 revolutions) whatever the distance to c.
__device__ __forceinline__ float phase_rev(float f, float x, float c) {
    const double p = (double)f * ((double)x - (double)c);
    return (float)(p - __builtin_rint(p));
}

}  // namespace km
