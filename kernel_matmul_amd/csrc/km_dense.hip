// Dense materialisation of the masked kernel matrix and the hyper-parameter gradient of a
// weighted sum of its entries.
//   dense     : out[b,i,j] = K[b,i,j] inside the row block's [start, end), 0 outside
//               (native/dense/dense.cu:12-98 of the reference; here the zeros are written by
//               the same kernel, so the output needs no prior clearing).
//   dense_bwd : grad[b,p] = d/d params[b,p] sum_{(i,j) in mask} out_grad[b,i,j] K[b,i,j]
//               (native/dense_bwd/dense_bwd.cu:12-116).
// Both stream an m x n fp32 matrix through HBM (4 B per entry): they are bandwidth bound.
#include "km_batch.h"
#include "km_common.h"
#include "km_launch.h"

namespace km {

struct DenseArgs {
    BatchShape batch;
    long long num_batches;
    long long total_items;  // row blocks * col splits * batches
    long long items_per_xcd;
    int m, n;
    int col_splits;
    int cols_per_split;    // dense: columns per share, a multiple of 64
    const float* x1;
    const float* x2;
    const float* params;
    const int* start;
    const int* end;
    float* out;            // dense: [num_batches][m][n]
    const float* weights;  // dense_bwd: out_grad, batch/inner strides below
    float* partials;       // dense_bwd: [num_batches][row_blocks * col_splits][KM_MAX_PARAMS]
    BatchStrides x1_bs, x2_bs, params_bs, start_bs, end_bs, weights_bs;
    long long x1_s, x2_s, params_s, start_s, end_s, weights_s0, weights_s1;
};

struct DenseView {
    long long b;
    long long rest;
    const float* x1;
    const float* x2;
    const float* params;
    const float* weights;
    int range_start, range_end;
};

__device__ __forceinline__ DenseView dense_view(const DenseArgs& a, long long item, int divisor,
                                                int* row_block, int* split) {
    DenseView v;
    v.b = item % a.num_batches;
    v.rest = item / a.num_batches;
    *split = (int)(v.rest % divisor);
    *row_block = (int)(v.rest / divisor);
    int bidx[KM_MAX_BATCH_RANK];
    batch_multi_index(a.batch, v.b, bidx);
    v.x1 = a.x1 + batch_offset(a.batch, a.x1_bs, bidx);
    v.x2 = a.x2 + batch_offset(a.batch, a.x2_bs, bidx);
    v.params = a.params + batch_offset(a.batch, a.params_bs, bidx);
    v.weights = a.weights ? a.weights + batch_offset(a.batch, a.weights_bs, bidx) : nullptr;
    v.range_start = max(a.start[batch_offset(a.batch, a.start_bs, bidx) + *row_block * a.start_s], 0);
    v.range_end = min(a.end[batch_offset(a.batch, a.end_bs, bidx) + *row_block * a.end_s], a.n);
    return v;
}

// One workgroup of 256 threads per (row block, column share, batch item): each wavefront writes
// 32 of the block's rows over the share's columns, lanes run along the columns so that stores are
// 256 B contiguous.  The column shares only exist to fill the device when row blocks x batch
// items are few.  A wavefront keeps its 32 row coordinates one per lane and broadcasts them with
// v_readlane (no load inside the row loop).
template <int KT>
__global__ void __launch_bounds__(256) dense_kernel(const DenseArgs a) {
    const long long item = xcd_item(blockIdx.x, a.items_per_xcd);
    if (item >= a.total_items) {
        return;
    }
    int row_block, split;
    const DenseView v = dense_view(a, item, a.col_splits, &row_block, &split);
    const int col_lo = split * a.cols_per_split;
    const int col_hi = min(a.n, col_lo + a.cols_per_split);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row_begin = row_block * KM_BLOCK_SIZE + wave * 32;
    const int rows = min(32, a.m - row_begin);
    if (rows <= 0 || col_lo >= col_hi) {
        return;
    }
    const KernelConsts kc = make_consts<KT>(v.params, a.params_s, true);
    float* __restrict__ out = a.out + v.b * (long long)a.m * a.n + (long long)row_begin * a.n;
    const int x1_bits = __float_as_int(v.x1[(long long)(row_begin + min(lane, rows - 1)) * a.x1_s]);
    for (int col0 = col_lo; col0 < col_hi; col0 += 64) {
        const int col = col0 + lane;
        const bool in_matrix = col < col_hi;
        const bool in_range = in_matrix && col >= v.range_start && col < v.range_end;
        float* __restrict__ o = out + col;
        // Wave-uniform choice: column tiles fully outside the range are only cleared.
        if (col0 < v.range_end && col0 + 64 > v.range_start) {
            const float x2v = in_range ? v.x2[(long long)col * a.x2_s] : 0.0f;
            for (int r = 0; r < rows; r++) {
                const float x1v = __int_as_float(__builtin_amdgcn_readlane(x1_bits, r));
                const float kv = kernel_value<KT>(x1v, x2v, kc) * kc.sgn;
                if (in_matrix) {
                    o[(long long)r * a.n] = in_range ? kv : 0.0f;
                }
            }
        } else if (in_matrix) {
            for (int r = 0; r < rows; r++) {
                o[(long long)r * a.n] = 0.0f;
            }
        }
    }
}

// One wavefront per (row block, column split, batch item): lanes run along the columns,
// the 128 rows are walked one by one (x1 is wave-uniform), weights are read 256 B contiguous.
template <int KT>
__global__ void __launch_bounds__(64) dense_bwd_partial(const DenseArgs a) {
    const long long item = xcd_item(blockIdx.x, a.items_per_xcd);
    if (item >= a.total_items) {
        return;
    }
    int row_block, split;
    const DenseView v = dense_view(a, item, a.col_splits, &row_block, &split);
    const KernelConsts kc = make_consts<KT>(v.params, a.params_s, false);
    const int lane = threadIdx.x;

    const int width = max(v.range_end - v.range_start, 0);
    const int per_split = ((width + a.col_splits - 1) / a.col_splits + 63) & ~63;
    const int col_begin = v.range_start + split * per_split;
    const int col_end = min(v.range_end, col_begin + per_split);
    const int row_begin = row_block * KM_BLOCK_SIZE;
    const int row_end = min(row_begin + KM_BLOCK_SIZE, a.m);

    // The block's 128 row coordinates, two per lane (rows past the matrix repeat the last one;
    // their weights are zero).
    const int x1_lo = __float_as_int(v.x1[(long long)min(row_begin + lane, a.m - 1) * a.x1_s]);
    const int x1_hi = __float_as_int(v.x1[(long long)min(row_begin + 64 + lane, a.m - 1) * a.x1_s]);

    float acc[KM_MAX_PARAMS] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int col0 = col_begin; col0 < col_end; col0 += 64) {
        const int col = col0 + lane;
        const bool ok = col < col_end;
        const int colc = min(col, col_end - 1);
        const float x2v = v.x2[(long long)colc * a.x2_s];
        const float* __restrict__ wcol = v.weights + (long long)colc * a.weights_s1;
        // 8 rows at a time: their weights are requested together, their coordinates come from
        // the lanes that hold them (below) by v_readlane.
        for (int row0 = row_begin; row0 < row_end; row0 += 8) {
            float wv[8];
#pragma unroll
            for (int t = 0; t < 8; t++) {
                const int row = row0 + t;
                wv[t] = (ok && row < row_end) ? wcol[(long long)row * a.weights_s0] : 0.0f;
            }
            const int x1_bits = row0 - row_begin < 64 ? x1_lo : x1_hi;
            const int first = (row0 - row_begin) & 63;
#pragma unroll
            for (int t = 0; t < 8; t++) {
                const float x1v = __int_as_float(__builtin_amdgcn_readlane(x1_bits, first + t));
                accumulate_pair<KT>(x1v, x2v, wv[t], kc, acc);
            }
        }
    }
    const long long partial_rows = a.total_items / a.num_batches;
    float* __restrict__ prow = a.partials + (v.b * partial_rows + v.rest) * KM_MAX_PARAMS;
#pragma unroll
    for (int p = 0; p < KM_MAX_PARAMS; p++) {
        const float total = wave_sum(acc[p]);
        if (lane == 0) {
            prow[p] = total;
        }
    }
}

static void fill_common(DenseArgs& a, const DenseProblem& p) {
    a.num_batches = p.num_batches;
    a.m = (int)p.m;
    a.n = (int)p.n;
    a.x1 = p.x1;
    a.x2 = p.x2;
    a.params = p.params;
    a.start = p.start;
    a.end = p.end;
    a.out = p.out;
    a.weights = p.weights;
    a.partials = (float*)p.workspace;
    const int r = p.batch_rank;
    a.x1_s = p.x1_strides[r];
    a.x2_s = p.x2_strides[r];
    a.params_s = p.params_strides[r];
    a.start_s = p.start_strides[r];
    a.end_s = p.end_strides[r];
    a.weights_s0 = p.weights ? p.weights_strides[r] : 0;
    a.weights_s1 = p.weights ? p.weights_strides[r + 1] : 0;
}

hipError_t launch_dense(const DenseProblem& p, hipStream_t stream) {
    DenseArgs a;
    const int64_t* const strides[5] = {p.x1_strides, p.x2_strides, p.params_strides,
                                       p.start_strides, p.end_strides};
    BatchStrides* outs[5] = {&a.x1_bs, &a.x2_bs, &a.params_bs, &a.start_bs, &a.end_bs};
    collapse_batch<5>(p.batch_rank, p.batch_sizes, strides, &a.batch, outs);
    fill_common(a, p);
    a.weights = nullptr;
    const long long row_blocks = (p.m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    // Column shares of at least 256 columns until there are 2048 workgroups (8 per CU).
    const long long base = row_blocks * p.num_batches;
    long long splits = base > 0 ? (2048 + base - 1) / base : 1;
    const long long most = (p.n + 255) / 256;
    if (splits > most) splits = most;
    if (splits < 1) splits = 1;
    a.cols_per_split = (int)((((p.n + splits - 1) / splits) + 63) / 64 * 64);
    if (a.cols_per_split < 64) a.cols_per_split = 64;
    a.col_splits = (int)((p.n + a.cols_per_split - 1) / a.cols_per_split);
    if (a.col_splits < 1) a.col_splits = 1;
    a.total_items = row_blocks * a.col_splits * p.num_batches;
    a.items_per_xcd = (a.total_items + KM_NUM_XCD - 1) / KM_NUM_XCD;
    const unsigned grid = (unsigned)(a.items_per_xcd * KM_NUM_XCD);
    switch (p.kernel_type) {
        case KM_KERNEL_RBF:
            hipLaunchKernelGGL((dense_kernel<KM_KERNEL_RBF>), dim3(grid), dim3(256), 0, stream, a);
            break;
        case KM_KERNEL_SPECTRAL:
            hipLaunchKernelGGL((dense_kernel<KM_KERNEL_SPECTRAL>), dim3(grid), dim3(256), 0, stream, a);
            break;
        default:
            hipLaunchKernelGGL((dense_kernel<KM_KERNEL_LOCALLY_PERIODIC>), dim3(grid), dim3(256), 0, stream, a);
            break;
    }
    return hipGetLastError();
}

hipError_t launch_dense_bwd(const DenseProblem& p, hipStream_t stream) {
    DenseArgs a;
    const int64_t* const strides[6] = {p.x1_strides, p.x2_strides, p.params_strides,
                                       p.start_strides, p.end_strides, p.weights_strides};
    BatchStrides* outs[6] = {&a.x1_bs, &a.x2_bs, &a.params_bs, &a.start_bs, &a.end_bs, &a.weights_bs};
    collapse_batch<6>(p.batch_rank, p.batch_sizes, strides, &a.batch, outs);
    fill_common(a, p);
    const long long row_blocks = (p.m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    a.col_splits = (int)(param_grad_partials_per_batch(p.m, p.num_batches) / (row_blocks > 0 ? row_blocks : 1));
    if (a.col_splits < 1) a.col_splits = 1;
    a.total_items = row_blocks * a.col_splits * p.num_batches;
    a.items_per_xcd = (a.total_items + KM_NUM_XCD - 1) / KM_NUM_XCD;
    const unsigned grid = (unsigned)(a.items_per_xcd * KM_NUM_XCD);
    if (grid > 0) {
        switch (p.kernel_type) {
            case KM_KERNEL_RBF:
                hipLaunchKernelGGL((dense_bwd_partial<KM_KERNEL_RBF>), dim3(grid), dim3(64), 0, stream, a);
                break;
            case KM_KERNEL_SPECTRAL:
                hipLaunchKernelGGL((dense_bwd_partial<KM_KERNEL_SPECTRAL>), dim3(grid), dim3(64), 0, stream, a);
                break;
            default:
                hipLaunchKernelGGL((dense_bwd_partial<KM_KERNEL_LOCALLY_PERIODIC>), dim3(grid), dim3(64), 0, stream, a);
                break;
        }
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) {
            return err;
        }
    }
    return launch_param_grad_reduce(p.kernel_type, a.batch, p.num_batches, row_blocks * a.col_splits,
                                    a.partials, p.params, a.params_bs, a.params_s, p.grad, stream);
}

}  // namespace km
