// Hyper-parameter gradient of sum_{(i,j) in mask} C[i,j] K[i,j] with C = left @ right^T.
// Serves the reference operators matmul_bwd (left = out_grad, right = rhs;
// native/matmul_bwd/matmul_bwd.cu:12-221) and bilinear_derivative
// (native/bilinear_derivative/bilinear_derivative.cu:12-183), which compute the same sum.
//
// Pass 1 (param_grad_partial): a wavefront owns 128 rows and a share of the row block's
// column range.  Per 16-column chunk and 16-row group the coefficient tile C (16x16) is
// formed on the matrix pipe from left/right (v_mfma_f32_16x16x4_f32 over the vector
// columns); its D layout gives each lane 4 (row, col) pairs, for which the lane evaluates
// the kernel derivatives and accumulates per-lane sums.  The sums are combined across the
// wavefront with DPP/permute shuffles and written as one partial row per wavefront.
// Pass 2 (param_grad_reduce): one workgroup per batch item adds the partial rows in a
// fixed order in fp64 and applies the chain rule back to the user parameters
// (native/common/kernel_function.cuh:221-251).  No atomics: results are reproducible.
#include "km_batch.h"
#include "km_common.h"
#include "km_launch.h"

namespace km {

struct GradArgs {
    BatchShape batch;
    long long num_batches;
    long long total_items;  // row blocks * col splits * batches
    long long items_per_xcd;
    int m, n, c;
    int col_splits;
    const float* x1;
    const float* x2;
    const float* left;
    const float* right;
    const float* params;
    const int* start;
    const int* end;
    float* partials;  // [num_batches][row_blocks * col_splits][KM_MAX_PARAMS]
    BatchStrides x1_bs, x2_bs, left_bs, right_bs, params_bs, start_bs, end_bs;
    long long x1_s, x2_s, left_s0, left_s1, right_s0, right_s1, params_s, start_s, end_s;
};

// TL > 0: the vector width c is at most 4*TL and the left operand stays in registers.
// TL == 0: any c; the left operand is re-read (from L1/L2) for every column chunk.
template <int KT, int TL>
__global__ void __launch_bounds__(64) param_grad_partial(const GradArgs a) {
    constexpr int R = 8;
    const int lane = threadIdx.x;
    const int li = lane & 15;
    const int kk = lane >> 4;

    const long long item = xcd_item(blockIdx.x, a.items_per_xcd);
    if (item >= a.total_items) {
        return;
    }
    const long long b = item % a.num_batches;
    const long long rest = item / a.num_batches;
    const int split = (int)(rest % a.col_splits);
    const int row_block = (int)(rest / a.col_splits);
    const int row0 = row_block * KM_BLOCK_SIZE;

    int bidx[KM_MAX_BATCH_RANK];
    batch_multi_index(a.batch, b, bidx);
    const float* __restrict__ x1 = a.x1 + batch_offset(a.batch, a.x1_bs, bidx);
    const float* __restrict__ x2 = a.x2 + batch_offset(a.batch, a.x2_bs, bidx);
    const float* __restrict__ left = a.left + batch_offset(a.batch, a.left_bs, bidx);
    const float* __restrict__ right = a.right + batch_offset(a.batch, a.right_bs, bidx);
    const float* __restrict__ params = a.params + batch_offset(a.batch, a.params_bs, bidx);
    int range_start = a.start[batch_offset(a.batch, a.start_bs, bidx) + row_block * a.start_s];
    int range_end = a.end[batch_offset(a.batch, a.end_bs, bidx) + row_block * a.end_s];
    range_start = max(range_start, 0);
    range_end = min(range_end, a.n);

    const KernelConsts kc = make_consts<KT>(params, a.params_s, false);

    // Column share of this wavefront, in whole chunks of 16 columns.
    const int width = max(range_end - range_start, 0);
    const int per_split = ((width + a.col_splits - 1) / a.col_splits + 15) & ~15;
    const int col_begin = range_start + split * per_split;
    const int col_end = min(range_end, col_begin + per_split);

    // x1 for the 4 rows per row group this lane owns in the D layout.
    float x1q[R][4];
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int row = min(row0 + 16 * r + 4 * kk + v, a.m - 1);
            x1q[r][v] = x1[(long long)row * a.x1_s];
        }
    }

    // Left operand (A layout): row = row0 + 16 r + li, vector column = 4 t + kk.
    constexpr int TLR = TL > 0 ? TL : 1;
    float lreg[R][TLR];
    if (TL > 0) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = row0 + 16 * r + li;
#pragma unroll
            for (int t = 0; t < TLR; t++) {
                const int cc = 4 * t + kk;
                lreg[r][t] = (row < a.m && cc < a.c)
                                 ? left[(long long)row * a.left_s0 + (long long)cc * a.left_s1]
                                 : 0.0f;
            }
        }
    }

    float acc[KM_MAX_PARAMS] = {0.0f, 0.0f, 0.0f, 0.0f};

    for (int n0 = col_begin; n0 < col_end; n0 += 16) {
        const int col = n0 + li;
        const bool col_ok = col < col_end;
        const int col_c = min(col, col_end - 1);
        const float x2v = x2[(long long)col_c * a.x2_s];

        float4v coef[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            coef[r] = (float4v){0.0f, 0.0f, 0.0f, 0.0f};
        }

        if (TL > 0) {
#pragma unroll
            for (int t = 0; t < TLR; t++) {
                const int cc = 4 * t + kk;
                const float rv = (col_ok && cc < a.c)
                                     ? right[(long long)col_c * a.right_s0 + (long long)cc * a.right_s1]
                                     : 0.0f;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    coef[r] = __builtin_amdgcn_mfma_f32_16x16x4f32(lreg[r][t], rv, coef[r], 0, 0, 0);
                }
            }
        } else {
            for (int c0 = 0; c0 < a.c; c0 += 4) {
                const int cc = c0 + kk;
                const float rv = (col_ok && cc < a.c)
                                     ? right[(long long)col_c * a.right_s0 + (long long)cc * a.right_s1]
                                     : 0.0f;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const int row = row0 + 16 * r + li;
                    const float lv = (row < a.m && cc < a.c)
                                         ? left[(long long)row * a.left_s0 + (long long)cc * a.left_s1]
                                         : 0.0f;
                    coef[r] = __builtin_amdgcn_mfma_f32_16x16x4f32(lv, rv, coef[r], 0, 0, 0);
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; r++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                accumulate_pair<KT>(x1q[r][v], x2v, coef[r][v], kc, acc);
            }
        }
    }

    const long long partial_rows = a.total_items / a.num_batches;
    float* __restrict__ prow = a.partials + (b * partial_rows + rest) * KM_MAX_PARAMS;
#pragma unroll
    for (int p = 0; p < KM_MAX_PARAMS; p++) {
        const float total = wave_sum(acc[p]);
        if (lane == 0) {
            prow[p] = total;
        }
    }
}

struct ReduceArgs {
    BatchShape batch;
    long long partial_rows;
    const float* partials;
    const float* params;
    BatchStrides params_bs;
    long long params_s;
    float* grad;  // [num_batches][P]
};

template <int KT>
__global__ void __launch_bounds__(256) param_grad_reduce(const ReduceArgs a) {
    constexpr int P = KernelTraits<KT>::P;
    __shared__ double sh[KM_MAX_PARAMS][256];
    const long long b = blockIdx.x;
    const float* __restrict__ rows = a.partials + b * a.partial_rows * KM_MAX_PARAMS;

    double sum[KM_MAX_PARAMS] = {0.0, 0.0, 0.0, 0.0};
    for (long long i = threadIdx.x; i < a.partial_rows; i += 256) {
#pragma unroll
        for (int p = 0; p < KM_MAX_PARAMS; p++) {
            sum[p] += (double)rows[i * KM_MAX_PARAMS + p];
        }
    }
#pragma unroll
    for (int p = 0; p < KM_MAX_PARAMS; p++) {
        sh[p][threadIdx.x] = sum[p];
    }
    __syncthreads();
    for (int half = 128; half >= 1; half >>= 1) {
        if ((int)threadIdx.x < half) {
#pragma unroll
            for (int p = 0; p < KM_MAX_PARAMS; p++) {
                sh[p][threadIdx.x] += sh[p][threadIdx.x + half];
            }
        }
        __syncthreads();
    }
    if (threadIdx.x != 0) {
        return;
    }

    int bidx[KM_MAX_BATCH_RANK];
    batch_multi_index(a.batch, b, bidx);
    const float* __restrict__ params = a.params + batch_offset(a.batch, a.params_bs, bidx);
    float* __restrict__ g = a.grad + b * P;
    finish_param_grad<KT>(sh[0][0], sh[1][0], sh[2][0], sh[3][0], params, a.params_s, g);
}

// ---------------------------------------------------------------------------------------
// Host dispatch.
// ---------------------------------------------------------------------------------------
static int grad_col_splits(int64_t m, long long num_batches) {
    // Enough wavefronts to populate the 1024 SIMDs of the device several times over when the
    // row-block count alone does not.
    const long long row_blocks = (m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    const long long base = row_blocks * num_batches;
    if (base <= 0) {
        return 1;
    }
    long long s = (4096 + base - 1) / base;
    if (s < 1) s = 1;
    if (s > 16) s = 16;
    return (int)s;
}

long long param_grad_partials_per_batch(int64_t m, long long num_batches) {
    const long long row_blocks = (m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    return row_blocks * grad_col_splits(m, num_batches);
}

template <int KT>
static hipError_t launch_partial(const GradArgs& a, unsigned grid_x, hipStream_t stream) {
    if (a.c <= 4) {
        hipLaunchKernelGGL((param_grad_partial<KT, 1>), dim3(grid_x), dim3(64), 0, stream, a);
    } else if (a.c <= 8) {
        hipLaunchKernelGGL((param_grad_partial<KT, 2>), dim3(grid_x), dim3(64), 0, stream, a);
    } else if (a.c <= 16) {
        hipLaunchKernelGGL((param_grad_partial<KT, 4>), dim3(grid_x), dim3(64), 0, stream, a);
    } else {
        hipLaunchKernelGGL((param_grad_partial<KT, 0>), dim3(grid_x), dim3(64), 0, stream, a);
    }
    return hipGetLastError();
}

hipError_t launch_param_grad_reduce(int kernel_type, const BatchShape& batch, long long num_batches,
                                    long long partial_rows, const float* partials,
                                    const float* params, const BatchStrides& params_bs,
                                    long long params_s, float* grad, hipStream_t stream) {
    ReduceArgs ra;
    ra.batch = batch;
    ra.partial_rows = partial_rows;
    ra.partials = partials;
    ra.params = params;
    ra.params_bs = params_bs;
    ra.params_s = params_s;
    ra.grad = grad;
    const unsigned rgrid = (unsigned)num_batches;
    switch (kernel_type) {
        case KM_KERNEL_RBF:
            hipLaunchKernelGGL((param_grad_reduce<KM_KERNEL_RBF>), dim3(rgrid), dim3(256), 0, stream, ra);
            break;
        case KM_KERNEL_SPECTRAL:
            hipLaunchKernelGGL((param_grad_reduce<KM_KERNEL_SPECTRAL>), dim3(rgrid), dim3(256), 0, stream, ra);
            break;
        default:
            hipLaunchKernelGGL((param_grad_reduce<KM_KERNEL_LOCALLY_PERIODIC>), dim3(rgrid), dim3(256), 0, stream, ra);
            break;
    }
    return hipGetLastError();
}

hipError_t launch_param_grad(const ParamGradProblem& p, hipStream_t stream) {
    GradArgs a;
    const int r = p.batch_rank;
    const int64_t* const strides[7] = {p.x1_strides, p.x2_strides, p.left_strides, p.right_strides,
                                       p.params_strides, p.start_strides, p.end_strides};
    BatchStrides* outs[7] = {&a.x1_bs, &a.x2_bs, &a.left_bs, &a.right_bs,
                             &a.params_bs, &a.start_bs, &a.end_bs};
    collapse_batch<7>(r, p.batch_sizes, strides, &a.batch, outs);
    a.num_batches = p.num_batches;
    a.m = (int)p.m;
    a.n = (int)p.n;
    a.c = (int)p.c;
    a.col_splits = grad_col_splits(p.m, p.num_batches);
    const long long row_blocks = (p.m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    a.total_items = row_blocks * a.col_splits * p.num_batches;
    a.items_per_xcd = (a.total_items + KM_NUM_XCD - 1) / KM_NUM_XCD;
    a.x1 = p.x1;
    a.x2 = p.x2;
    a.left = p.left;
    a.right = p.right;
    a.params = p.params;
    a.start = p.start;
    a.end = p.end;
    a.partials = (float*)p.workspace;
    a.x1_s = p.x1_strides[r];
    a.x2_s = p.x2_strides[r];
    a.left_s0 = p.left_strides[r];
    a.left_s1 = p.left_strides[r + 1];
    a.right_s0 = p.right_strides[r];
    a.right_s1 = p.right_strides[r + 1];
    a.params_s = p.params_strides[r];
    a.start_s = p.start_strides[r];
    a.end_s = p.end_strides[r];

    const unsigned grid_x = (unsigned)(a.items_per_xcd * KM_NUM_XCD);
    if (grid_x > 0) {  // no rows: the reduce pass alone writes the zero gradient
        hipError_t err;
        switch (p.kernel_type) {
            case KM_KERNEL_RBF: err = launch_partial<KM_KERNEL_RBF>(a, grid_x, stream); break;
            case KM_KERNEL_SPECTRAL: err = launch_partial<KM_KERNEL_SPECTRAL>(a, grid_x, stream); break;
            default: err = launch_partial<KM_KERNEL_LOCALLY_PERIODIC>(a, grid_x, stream); break;
        }
        if (err != hipSuccess) {
            return err;
        }
    }

    return launch_param_grad_reduce(p.kernel_type, a.batch, p.num_batches, row_blocks * a.col_splits,
                                    a.partials, p.params, a.params_bs, a.params_s, p.grad, stream);
}

}  // namespace km
